"""Training-step pieces and the benchmark's command-line contract, on CPU."""

import json
import math
import os
import subprocess
import sys

import torch
from torch import nn

import deconver_amd as dc
from deconver_amd import training as T

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_dice_bce_closed_forms():
    target = torch.zeros(1, 1, 4, 4)
    target[..., :2, :] = 1.0
    # confident and right: both terms vanish (dice -> (2*8+1)/(8+8+1) = 1)
    big = (target * 2 - 1) * 40.0
    assert float(T.dice_bce_loss(big, target)) < 1e-6
    # zero logits: BCE = ln 2, p = 1/2 everywhere: dice = (2*4+1)/(8+8+1) = 9/17
    zero = torch.zeros_like(target)
    assert abs(float(T.dice_bce_loss(zero, target)) - (math.log(2) + 1 - 9 / 17)) < 1e-6
    # empty target, confident background: dice term (0+1)/(0+0+1) = 1 -> loss 0
    assert float(T.dice_bce_loss(-big.abs(), torch.zeros_like(target))) < 1e-6
    # gradient flows and is finite
    logits = torch.randn(2, 1, 4, 4, requires_grad=True)
    T.dice_bce_loss(logits, target.expand(2, -1, -1, -1)).backward()
    assert torch.isfinite(logits.grad).all() and logits.grad.abs().sum() > 0


def test_synthetic_data():
    images, masks = T.smoothed_noise_masks(4, 3, (96, 96), seed=0)
    assert images.shape == (4, 3, 96, 96) and masks.shape == (4, 1, 96, 96)
    assert images.min() >= 0 and images.max() < 1
    assert set(masks.unique().tolist()) <= {0.0, 1.0}
    assert abs(float(masks.mean()) - 0.3) < 0.01
    again, _ = T.smoothed_noise_masks(4, 3, (96, 96), seed=0)
    assert torch.equal(images, again)                       # seeded
    vols, targets = T.ellipsoid_phantoms(2, 2, (48, 48, 48), seed=0)
    inside = vols[vols != 0]
    assert abs(float(inside.mean())) < 1e-3 and abs(float(inside.std()) - 1) < 2e-2
    assert 0.002 < float(targets.mean()) < 0.03
    assert float((targets * (vols[:, :1] == 0)).sum()) == 0   # lesions lie inside the mask


def test_train_step_lowers_loss_on_cpu():
    torch.manual_seed(0)
    model = dc.Deconver(in_channels=2, out_channels=1, spatial_dims=3, encoder_depth=(1, 1),
                        encoder_width=(8, 16), strides=(1, 2), decoder_depth=(1,),
                        norm=nn.InstanceNorm3d, kernel_size=(3, 3, 3), groups=-1, ratio=2)
    opt = T.make_optimizer(model)
    assert isinstance(opt, torch.optim.AdamW)
    images, targets = T.ellipsoid_phantoms(1, 2, (16, 16, 16), seed=1)
    losses = [float(T.train_step(model, opt, images, targets)) for _ in range(5)]
    assert losses[-1] < losses[0]


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True)
    assert proc.returncode == 2
    assert "one-GPU" in proc.stderr and proc.stdout.strip() == ""


def test_bench_traffic_file_is_valid():
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
        t = json.load(f)
    assert set(t["bf16"]) == {"forward", "backward_pass1", "backward_pass2"}
    assert all(isinstance(v, int) and v > 0 for v in t["bf16"].values())
