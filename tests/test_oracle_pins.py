"""Pins of the CPU oracle (oracle/ndc_oracle.py).

The reference's tests store no vectors for this path, so the oracle is pinned by what the
mathematics fixes; each check is chosen so that a plausible mistake (dropped term, flipped
tap, transposed channel pair, wrong pad) fails it.
"""

import numpy as np
import pytest
import torch

from oracle import ndc_oracle as O

torch.set_default_dtype(torch.float32)

GEOMS = [
    # (C, groups, sc, kernel, spatial)
    (6, 3, 2, (3, 3, 3), (5, 4, 3)),     # groups not in {1, C}, m = 2
    (4, 4, 4, (3, 3, 3), (4, 5, 6)),     # depthwise, ratio 4
    (4, 1, 3, (3, 3, 3), (3, 4, 3)),     # one group, m = 4
    (4, 4, 4, (5, 5), (7, 6)),           # 2-D 5x5 depthwise
    (6, 2, 2, (3, 5, 3), (4, 6, 3)),     # anisotropic kernel
    (8, 8, 2, (5,), (11,)),              # 1-D
]


def _rand(shape, seed, positive=True):
    g = torch.Generator().manual_seed(seed)
    t = torch.rand(*shape, generator=g, dtype=torch.float64)
    return t if positive else t - 0.5


def _case(C, G, sc, ks, sp, B=2, seed=0, positive_h=True):
    m = C // G
    x = _rand((B, C, *sp), seed)
    z = _rand((B, G * sc, *sp), seed + 1, positive=False)
    h = _rand((C, sc, *ks), seed + 2, positive=positive_h)
    if not positive_h:
        h = torch.relu(h)
    bias = _rand((G * sc,), seed + 3, positive=False)
    return x, z, h, bias, m


@pytest.mark.parametrize("geom", GEOMS)
def test_K_A_match_bruteforce(geom, bruteforce):
    C, G, sc, ks, sp = geom
    x, z, h, _, m = _case(*geom)
    k_t = O.op_K(z, h, G, m, sc).numpy()
    a_t = O.op_A(x, h, G, m, sc).numpy()
    np.testing.assert_allclose(k_t, bruteforce.K(z.numpy(), h.numpy(), G, m, sc).reshape(k_t.shape),
                               rtol=0, atol=1e-12)
    np.testing.assert_allclose(a_t, bruteforce.A(x.numpy(), h.numpy(), G, m, sc).reshape(a_t.shape),
                               rtol=0, atol=1e-12)


@pytest.mark.parametrize("geom", GEOMS)
def test_adjoint_identity(geom):
    C, G, sc, ks, sp = geom
    x, z, h, _, m = _case(*geom)
    lhs = (O.op_K(z, h, G, m, sc) * x).sum()
    rhs = (z * O.op_A(x, h, G, m, sc)).sum()
    assert abs(lhs - rhs) <= 1e-12 * abs(lhs)


@pytest.mark.parametrize("geom", GEOMS)
def test_literal_batched_form_equals_grouped_form(geom, bruteforce):
    """reference.py's batch-folded convs == one grouped conv when the filter is batch-invariant,
    and both equal the brute-force update."""
    C, G, sc, ks, sp = geom
    x, z, h0, bias, m = _case(*geom, positive_h=False)
    h0 = h0 - 0.1  # some negative entries so that relu(h0) matters
    w = _rand((G * sc, C), 7, positive=False)
    layer = O.OracleNDC(C, ks, source_channels=sc, groups=G)
    y_lit = layer.forward(x, w, bias, h0)
    y_grp = O.layer_forward_grouped(x, w, bias, h0, G, sc)
    assert O.rel_err(y_grp, y_lit) < 1e-12
    zz = torch.nn.functional.conv1d(x.flatten(2), w.unsqueeze(-1)).view(x.shape[0], -1, *sp)
    out_bf, _ = bruteforce.update(x.numpy(), zz.numpy(), torch.relu(h0).numpy(), bias.numpy(),
                                  G, m, sc, 1e-16, True)
    assert O.rel_err(torch.from_numpy(out_bf).view_as(y_lit), y_lit) < 1e-10


def test_delta_kernel_special_case():
    """h = centre tap only: K(s) = sum_i s_i, A(x)_i = x."""
    C, sc, ks, sp = 3, 4, (3, 3, 3), (4, 5, 3)
    x = _rand((2, C, *sp), 0)
    s = _rand((2, C * sc, *sp), 1)
    h = torch.zeros(C, sc, *ks, dtype=torch.float64)
    h[:, :, 1, 1, 1] = 1.0
    k = O.op_K(s, h, C, 1, sc)
    assert torch.allclose(k, s.view(2, C, sc, *sp).sum(2), atol=1e-14)
    a = O.op_A(x, h, C, 1, sc)
    assert torch.allclose(a, x.repeat_interleave(sc, dim=1), atol=1e-14)


def test_off_centre_delta_fixes_tap_direction():
    """A single off-centre tap shifts K one way and A the other (catches a flipped tap)."""
    x = torch.zeros(1, 1, 5, 5, dtype=torch.float64)
    x[0, 0, 2, 2] = 1.0
    h = torch.zeros(1, 1, 3, 3, dtype=torch.float64)
    h[0, 0, 0, 2] = 1.0  # tau = (0, 2): offset (-1, +1)
    k = O.op_K(x, h, 1, 1, 1)
    # K(u)[p] = u[p + tau - pad]  ->  the impulse at (2,2) shows up at p = (3,1)
    assert k[0, 0, 3, 1] == 1.0 and k.sum() == 1.0
    a = O.op_A(x, h, 1, 1, 1)
    # A(v)[p] = v[p + pad - tau]  ->  the impulse shows up at p = (1,3)
    assert a[0, 0, 1, 3] == 1.0 and a.sum() == 1.0


@pytest.mark.parametrize("geom", GEOMS[:4])
def test_fixed_point_zero_and_sign(geom):
    C, G, sc, ks, sp = geom
    _, z, h, _, m = _case(*geom)
    s = z.abs() + 0.1
    x = O.op_K(s, h, G, m, sc)
    out, _ = O.update_grouped(x, s, h, None, G, m, sc, 1e-16, False)
    assert O.rel_err(out, s) < 1e-10            # x = K(s) exactly  =>  s is a fixed point
    s0 = s.clone()
    s0[:, ::2] = 0
    out0, _ = O.update_grouped(x, s0, h, None, G, m, sc, 1e-16, False)
    assert (out0[:, ::2] == 0).all()            # s = 0 stays 0
    assert (out0 >= 0).all()                    # non-negativity is preserved


@pytest.mark.parametrize("geom", GEOMS[:3])
def test_scaling_laws(geom):
    C, G, sc, ks, sp = geom
    x, z, h, _, m = _case(*geom)
    s = z.abs() + 0.05
    base, _ = O.update_grouped(x, s, h, None, G, m, sc, 1e-16, False)
    ax, _ = O.update_grouped(3.0 * x, s, h, None, G, m, sc, 1e-16, False)
    bs, _ = O.update_grouped(x, 5.0 * s, h, None, G, m, sc, 1e-16, False)
    ch, _ = O.update_grouped(x, s, 2.0 * h, None, G, m, sc, 1e-16, False)
    assert O.rel_err(ax, 3.0 * base) < 1e-10
    assert O.rel_err(bs, base) < 1e-10
    assert O.rel_err(ch, base / 2.0) < 1e-10


def test_constant_field_closed_form_interior():
    """x = a, s = c constant, depthwise: out_i = a / sum_{j,tau} h[j,tau] away from the border."""
    C, sc, ks, sp = 2, 3, (3, 3, 3), (9, 9, 9)
    a, c = 0.7, 1.3
    h = _rand((C, sc, *ks), 5) + 0.1
    x = torch.full((1, C, *sp), a, dtype=torch.float64)
    s = torch.full((1, C * sc, *sp), c, dtype=torch.float64)
    out, _ = O.update_grouped(x, s, h, None, C, 1, sc, 1e-16, False)
    inner = out[..., 2:-2, 2:-2, 2:-2].reshape(C, sc, -1)
    expect = a / h.reshape(C, -1).sum(1)
    for ch in range(C):
        assert torch.allclose(inner[ch], expect[ch].expand_as(inner[ch]), rtol=1e-12)


def test_update_first_iteration_bias_relu_and_padding():
    """Bias is added before the ReLU and the zero padding applies to s, not z
    (a bias-padded border would change K(s) near the edge)."""
    C, G, sc, ks, sp = 2, 2, 2, (3, 3), (4, 4)
    x, z, h, bias, m = _case(C, G, sc, ks, sp)
    bias = bias.abs() + 0.5
    out, t1 = O.update_grouped(x, z, h, bias, G, m, sc, 1e-16, True)
    s = torch.relu(z + bias.view(1, -1, 1, 1))
    sp_ = torch.nn.functional.pad(s, (1, 1, 1, 1))
    t1_manual = torch.zeros_like(t1)
    for g in range(G):
        for i in range(sc):
            for a in range(3):
                for b in range(3):
                    t1_manual[:, g] += sp_[:, g * sc + i, a:a + 4, b:b + 4] * h[g, i, a, b]
    assert torch.allclose(t1, t1_manual, atol=1e-13)


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("relu", [True, False])
def test_analytic_backward_matches_autograd_and_bruteforce(geom, relu, bruteforce):
    C, G, sc, ks, sp = geom
    x, z, h, bias, m = _case(*geom)
    if not relu:
        z = z.abs() + 0.05
    gout = _rand(z.shape, 11, positive=False)
    xr, zr, hr, br = (t.clone().requires_grad_(True) for t in (x, z, h, bias))
    out, _ = O.update_grouped(xr, zr, hr, br, G, m, sc, 1e-16, relu)
    out.backward(gout)
    gx, gz, gh, gb = O.update_backward(x, z, h, bias, gout, G, m, sc, 1e-16, relu)
    for name, mine, auto in (("gx", gx, xr.grad), ("gz", gz, zr.grad), ("gh", gh, hr.grad),
                             ("gb", gb, br.grad)):
        assert O.rel_err(mine, auto) < 1e-10, name
    bx, bz, bh, bb = bruteforce.backward(x.numpy(), z.numpy(), h.numpy(), bias.numpy(),
                                         gout.numpy(), G, m, sc, 1e-16, relu)
    for name, mine, bf in (("gx", gx, bx), ("gz", gz, bz), ("gh", gh, bh), ("gb", gb, bb)):
        assert O.rel_err(torch.from_numpy(bf).view_as(mine), mine) < 1e-10, name


def test_bruteforce_backward_matches_finite_differences(bruteforce):
    """Independent of torch: central differences of the brute-force update."""
    C, G, sc, ks, sp = 4, 2, 2, (3, 3, 3), (3, 4, 3)
    x, z, h, bias, m = _case(C, G, sc, ks, sp, B=1)
    z = z + 0.7  # keep z + b away from the ReLU kink
    gout = _rand(z.shape, 11, positive=False).numpy()
    args = [x.numpy().copy(), z.numpy().copy(), h.numpy().copy(), bias.numpy().copy()]
    grads = bruteforce.backward(*args, gout, G, m, sc, 1e-16, True)
    rng = np.random.default_rng(0)
    for which in range(4):
        for _ in range(4):
            idx = tuple(rng.integers(0, s) for s in args[which].shape)
            step = 1e-6
            plus = [a.copy() for a in args]
            minus = [a.copy() for a in args]
            plus[which][idx] += step
            minus[which][idx] -= step
            fp = (bruteforce.update(*plus, G, m, sc, 1e-16, True)[0] * gout).sum()
            fm = (bruteforce.update(*minus, G, m, sc, 1e-16, True)[0] * gout).sum()
            fd = (fp - fm) / (2 * step)
            got = grads[which].reshape(args[which].shape)[idx]
            assert abs(fd - got) <= 1e-6 * max(1.0, abs(got)), (which, idx, fd, got)


def test_gradcheck_grouped_update():
    C, G, sc, ks, sp = 2, 2, 2, (3, 3), (4, 3)
    x, z, h, bias, m = _case(C, G, sc, ks, sp, B=1)
    z = z + 0.7
    fn = lambda x_, z_, h_, b_: O.update_grouped(x_, z_, h_, b_, G, m, sc, 1e-16, True)[0]
    inputs = tuple(t.clone().requires_grad_(True) for t in (x, z, h, bias))
    assert torch.autograd.gradcheck(fn, inputs, eps=1e-6, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("iters", [(3, 1), (2, 2), (3, 3), (3, 0)])
def test_truncated_backprop_contract(iters):
    """Iterations before num_iters - num_grad_iters + 1 run without grad; if all are cut the
    parameters get no gradient at all (test_deconv_equivalence.py:142-169)."""
    num_iters, num_grad = iters
    C, G, sc, ks, sp = 4, 4, 2, (3, 3, 3), (4, 4, 4)
    x, _, h0, bias, _ = _case(C, G, sc, ks, sp)
    bias = bias + 1.0
    w = _rand((G * sc, C), 3, positive=False)
    params = [t.clone().requires_grad_(True) for t in (w, bias, h0)]
    layer = O.OracleNDC(C, ks, source_channels=sc, groups=G, num_iters=num_iters,
                        num_grad_iters=num_grad)
    y = layer.forward(x, *params)
    y2 = O.layer_forward_grouped(x, *[p.detach() for p in params], G, sc, num_iters=num_iters,
                                 num_grad_iters=num_grad)
    assert O.rel_err(y2, y.detach()) < 1e-10
    if num_grad == 0:
        assert not y.requires_grad
        return
    y.sum().backward()
    # projection gradients only flow if the first (projection-fed) iteration is differentiable
    if num_grad < num_iters:
        assert params[0].grad is None and params[1].grad is None
    else:
        assert params[0].grad is not None and params[1].grad is not None
    assert params[2].grad is not None


def test_default_parameter_distributions():
    g = torch.Generator().manual_seed(0)
    w, b, h0 = O.default_parameters(32, (3, 3, 3), 4, 32, generator=g)
    bound_h = 1.0 / (4 * 27) ** 0.5
    assert h0.shape == (32, 4, 3, 3, 3) and h0.abs().max() <= bound_h
    assert abs(h0.std().item() - bound_h / 3 ** 0.5) < 0.1 * bound_h
    assert w.shape == (128, 32, 1) and w.abs().max() <= 1 / 32 ** 0.5
    assert b.shape == (128,) and b.abs().max() <= 1 / 32 ** 0.5
