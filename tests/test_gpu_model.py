"""The Deconver network with its NDC layers on the HIP kernels, against the functional
model oracle (CPU, float64) from the same state dict; one training step; data generators."""

import pytest
import torch
from torch import nn

import deconver_amd as dc
from deconver_amd import training as T
from oracle import ndc_oracle as O
from oracle.model_oracle import deconver_forward

pytestmark = pytest.mark.gpu

NET_2D = dict(in_channels=3, out_channels=2, spatial_dims=2, encoder_depth=(1, 1, 1),
              encoder_width=(16, 32, 48), strides=(1, 2, 2), decoder_depth=(1, 1),
              norm=nn.InstanceNorm2d, kernel_size=(5, 5), groups=-1, ratio=4)
NET_3D = dict(in_channels=2, out_channels=1, spatial_dims=3, encoder_depth=(1, 1, 1),
              encoder_width=(16, 32, 64), strides=(1, 2, 2), decoder_depth=(1, 1),
              norm=nn.InstanceNorm3d, kernel_size=(3, 3, 3), groups=-1, ratio=4)


def _ndc_layers(model):
    return [m for m in model.modules() if isinstance(m, dc.Deconv)]


@pytest.mark.parametrize("cfg,spatial", [(NET_2D, (32, 24)), (NET_3D, (16, 12, 20))])
def test_model_on_hip_matches_oracle(cfg, spatial):
    """Tolerances of the reference's network test (tests/test_deconv_equivalence.py:314-329):
    forward 1e-4, gradients 5e-3 of the largest reference entry."""
    torch.manual_seed(0)
    model = dc.Deconver(**cfg).cuda()
    x = torch.rand(2, cfg["in_channels"], *spatial, device="cuda")
    for layer in _ndc_layers(model):
        assert layer.fast_path_applicable(torch.empty(1, layer.channels, *spatial, device="cuda"))
    y = model(x)
    g = torch.randn_like(y)
    y.backward(g)
    state = {k: v.detach().cpu().double().requires_grad_(True)
             for k, v in model.state_dict().items()}
    yr = deconver_forward(state, x.cpu().double(), cfg)
    yr.backward(g.cpu().double())
    assert O.rel_err(y.cpu(), yr) < 1e-4
    worst = max((O.rel_err(p.grad.cpu(), state[n].grad), n) for n, p in model.named_parameters())
    assert worst[0] < 5e-3, worst


def test_training_step_reduces_loss_and_matches_pytorch_route():
    """A few AdamW steps under bf16 autocast on the HIP route lower the loss, and track the
    same model trained on the layer's PyTorch route."""
    images, targets = T.ellipsoid_phantoms(2, 2, (32, 32, 32), seed=0, device="cuda")
    losses = {}
    for route, extra in (("hip", {}), ("pytorch", {"stride": 1})):
        torch.manual_seed(0)
        model = dc.Deconver(**NET_3D, **extra).cuda()
        on_hip = all(m.fast_path_applicable(torch.empty(1, m.channels, 8, 8, 8, device="cuda"))
                     for m in _ndc_layers(model))
        assert on_hip == (route == "hip")
        opt = T.make_optimizer(model)
        losses[route] = [float(T.train_step(model, opt, images, targets,
                                            autocast_dtype=torch.bfloat16)) for _ in range(6)]
    assert losses["hip"][-1] < losses["hip"][0]
    for a, b in zip(losses["hip"], losses["pytorch"]):
        assert abs(a - b) < 3e-2 * abs(b), losses


def test_synthetic_data_statistics():
    images, masks = T.smoothed_noise_masks(4, 3, (128, 128), seed=0)
    assert images.min() >= 0 and images.max() < 1
    assert abs(float(masks.mean()) - 0.3) < 0.01
    vols, targets = T.ellipsoid_phantoms(2, 2, (64, 64, 64), seed=0)
    inside = vols[vols != 0]
    assert abs(float(inside.mean())) < 1e-3 and abs(float(inside.std()) - 1) < 1e-2
    assert 0.002 < float(targets.mean()) < 0.03
    assert float((targets * (vols[:, :1] == 0)).sum()) == 0     # lesions lie inside the mask
