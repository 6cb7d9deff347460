"""A training step recorded into a HIP graph (``training.GraphedTrainStep``) against the same
steps run eagerly: every replay, with eager work and synchronisations between the replays."""

import copy

import pytest
import torch
from torch import nn

import deconver_amd as dc
from deconver_amd import training as T

pytestmark = pytest.mark.gpu


def _network(dims):
    torch.manual_seed(0)
    if dims == 3:
        return dc.Deconver(in_channels=2, out_channels=1, spatial_dims=3, encoder_depth=(1, 1, 1),
                           encoder_width=(64, 128, 256), strides=(1, 2, 2), decoder_depth=(1, 1),
                           kernel_size=(3, 3, 3), groups=-1, ratio=4, norm=nn.InstanceNorm3d)
    return dc.Deconver(in_channels=3, out_channels=1, spatial_dims=2, encoder_depth=(1, 1, 1),
                       encoder_width=(32, 64, 128), strides=(1, 2, 2), decoder_depth=(1, 1),
                       kernel_size=(5, 5), groups=-1, ratio=4, norm=nn.InstanceNorm2d)


@pytest.mark.parametrize("dims,size,autocast", [(3, 32, torch.bfloat16), (2, 64, None)])
def test_replayed_steps_equal_eager_steps(dims, size, autocast):
    eager = _network(dims).cuda()
    graphed = copy.deepcopy(eager)
    opt_e, opt_g = T.make_optimizer(eager, capturable=True), T.make_optimizer(graphed, capturable=True)
    make = T.ellipsoid_phantoms if dims == 3 else T.smoothed_noise_masks
    batches = [make(1, 2 if dims == 3 else 3, (size,) * dims, seed=s, device="cuda") for s in range(5)]
    step = T.GraphedTrainStep(graphed, opt_g, *batches[0], autocast_dtype=autocast)
    # construction left parameters and optimiser state as they were
    for p, q in zip(eager.parameters(), graphed.parameters()):
        assert torch.equal(p, q)
    # The library's kernels give the same bits recorded or not; the GEMM library may pick another
    # algorithm while a graph is being recorded, so a step's loss agrees to the storage precision,
    # and stays there over the steps (a replay that read stale or unset memory would not)
    tol = 2e-3 if autocast is not None else 2e-5
    for images, targets in batches:
        want = T.train_step(eager, opt_e, images, targets, autocast_dtype=autocast)
        torch.cuda.synchronize()
        got = step(images, targets)
        torch.cuda.synchronize()
        assert torch.isfinite(got)
        assert abs(float(got) - float(want)) <= tol * max(1.0, abs(float(want))), (float(got), float(want))
        scratch = torch.randn(1 << 20, device="cuda").sum()     # eager work between the replays
        assert torch.isfinite(scratch)


def test_needs_a_capturable_optimizer_and_a_fixed_shape():
    model = _network(2).cuda()
    images, targets = T.smoothed_noise_masks(1, 3, (32, 32), seed=0, device="cuda")
    with pytest.raises(ValueError):
        T.GraphedTrainStep(model, T.make_optimizer(model), images, targets)
    step = T.GraphedTrainStep(model, T.make_optimizer(model, capturable=True), images, targets)
    with pytest.raises(ValueError):
        step(images[:, :, :16], targets[:, :, :16])
