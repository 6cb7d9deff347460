// placeholder until the fused kernels land
#pragma once
#include "ndc_common.h"
namespace ndc { namespace fused {
static inline bool supported(const KGeom &) { return false; }
static inline size_t backward_ws(const KGeom &, int, int, int) { return 0; }
template <class BE, typename T>
static int forward(const KGeom &, const T *, const T *, const float *, const float *, T *, T *, void *) { return -2; }
template <class BE, typename T>
static int backward(const KGeom &, const T *, const T *, const T *, const float *, const float *, const T *, T *, T *, float *, float *, void *, void *) { return -2; }
}}
