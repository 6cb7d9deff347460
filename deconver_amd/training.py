"""Training-step pieces for the model-level workloads: loss, synthetic data, one step.

The reference ships no loss, optimiser or data pipeline (its README shows forward passes
only, ``README.md:44-88``); the model-level benchmark configurations name them in words
("Dice+BCE with AdamW", thresholded smoothed noise, ellipsoid phantoms).  These are this
package's definitions of those words, kept small and deterministic:

    loss   = BCEWithLogits(l, y) + 1 - (2 sum(p y) + 1) / (sum(p) + sum(y) + 1),  p = sigmoid(l)
             (sums over each sample's voxels, mean over samples and channels)
    optim  = AdamW(lr = 1e-3, weight_decay = 1e-2)
"""

from __future__ import annotations

import math
from typing import Callable, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn

__all__ = ["dice_bce_loss", "make_optimizer", "smoothed_noise_masks", "ellipsoid_phantoms",
           "train_step", "GraphedTrainStep"]


def _voxel_sum(t: Tensor) -> Tensor:
    """``t.sum(-1)`` of a ``(B, C, n)`` tensor in two stages when ``n`` is long: a reduction to
    B*C outputs runs on B*C workgroups (two, for a batch of two one-channel volumes: 0.27 ms
    per sum of 2 M voxels on an MI355X), 1 024 partial sums per row fill the device."""
    n = t.shape[-1]
    for chunks in (1024, 256, 64):
        if n % chunks == 0 and n // chunks >= 256:
            return t.view(*t.shape[:-1], chunks, n // chunks).sum(-1).sum(-1)
    return t.sum(-1)


def dice_bce_loss(logits: Tensor, target: Tensor) -> Tensor:
    """Binary cross-entropy on the logits plus soft Dice loss with +1 smoothing, float32."""
    logits = logits.float()
    target = target.float()
    bce = F.binary_cross_entropy_with_logits(logits, target)
    p = torch.sigmoid(logits).flatten(2)
    y = target.flatten(2)
    dice = (2 * _voxel_sum(p * y) + 1) / (_voxel_sum(p) + _voxel_sum(y) + 1)
    return bce + (1 - dice).mean()


def make_optimizer(model: nn.Module, capturable: bool = False) -> torch.optim.Optimizer:
    """AdamW as above; ``capturable`` keeps its step counters on the device, which
    ``GraphedTrainStep`` needs."""
    return torch.optim.AdamW(model.parameters(), lr=1e-3, weight_decay=1e-2, capturable=capturable)


def _gaussian_blur(t: Tensor, sigma: float) -> Tensor:
    """Separable Gaussian smoothing of a ``(B, 1, *S)`` tensor along every spatial axis."""
    radius = max(1, int(3 * sigma))
    taps = torch.arange(-radius, radius + 1, dtype=t.dtype, device=t.device)
    kernel = torch.exp(-0.5 * (taps / sigma) ** 2)
    kernel = kernel / kernel.sum()
    nd = t.dim() - 2
    conv = {2: F.conv2d, 3: F.conv3d}[nd]
    for axis in range(nd):
        shape = [1, 1] + [1] * nd
        shape[2 + axis] = kernel.numel()
        pad = [0] * nd
        pad[axis] = radius
        t = conv(t, kernel.view(shape), padding=tuple(pad))
    return t


def smoothed_noise_masks(batch: int, channels: int, size: Sequence[int], *, foreground: float = 0.3,
                         sigma: float = 4.0, seed: int = 0,
                         device: torch.device | str = "cpu") -> Tuple[Tensor, Tensor]:
    """Images uniform in [0, 1) and binary masks from Gaussian-smoothed noise thresholded
    at its ``1 - foreground`` quantile (about 30 % foreground by default)."""
    gen = torch.Generator().manual_seed(seed)
    images = torch.rand(batch, channels, *size, generator=gen)
    noise = _gaussian_blur(torch.randn(batch, 1, *size, generator=gen), sigma)
    cut = torch.quantile(noise.flatten(1), 1 - foreground, dim=1).view(-1, 1, *([1] * len(size)))
    masks = (noise > cut).float()
    return images.to(device), masks.to(device)


def _ellipsoid(grid: Sequence[Tensor], centre: Sequence[float], radii: Sequence[float]) -> Tensor:
    acc = torch.zeros_like(grid[0])
    for g, c, r in zip(grid, centre, radii):
        acc = acc + ((g - c) / r) ** 2
    return acc <= 1.0


def ellipsoid_phantoms(batch: int, channels: int, size: Sequence[int], *, seed: int = 0,
                       device: torch.device | str = "cpu") -> Tuple[Tensor, Tensor]:
    """Volumes with N(0,1) intensities (z-scored over the mask) inside a random ellipsoid
    "brain" and 0 outside; targets of 1-5 small ellipsoid "lesions" inside it (about 1 %
    foreground)."""
    gen = torch.Generator().manual_seed(seed)
    nd = len(size)
    grid = torch.meshgrid(*[torch.arange(s, dtype=torch.float32) for s in size], indexing="ij")
    rand = lambda lo, hi: lo + (hi - lo) * torch.rand((), generator=gen).item()
    images = torch.zeros(batch, channels, *size)
    targets = torch.zeros(batch, 1, *size)
    for b in range(batch):
        centre = [s * rand(0.45, 0.55) for s in size]
        radii = [s * rand(0.35, 0.45) for s in size]
        brain = _ellipsoid(grid, centre, radii)
        values = torch.randn(channels, *size, generator=gen)
        inside = values[:, brain]
        values = (values - inside.mean(1).view(-1, *([1] * nd))) / inside.std(1).view(-1, *([1] * nd))
        images[b] = values * brain
        # lesion radii such that the expected total is about 1 % of the volume
        n_lesions = int(torch.randint(1, 6, (), generator=gen).item())
        r_rel = (0.01 / n_lesions / (math.pi * (4 / 3 if nd == 3 else 1))) ** (1 / nd)
        lesion = torch.zeros_like(brain)
        for _ in range(n_lesions):
            c = [ci + ri * rand(-0.5, 0.5) for ci, ri in zip(centre, radii)]
            r = [s * r_rel * rand(0.8, 1.25) for s in size]
            lesion |= _ellipsoid(grid, c, r)
        targets[b, 0] = (lesion & brain).float()
    return images.to(device), targets.to(device)


def train_step(model: nn.Module, optimizer: torch.optim.Optimizer, images: Tensor, targets: Tensor,
               *, autocast_dtype: Optional[torch.dtype] = None,
               loss_fn: Callable[[Tensor, Tensor], Tensor] = dice_bce_loss) -> Tensor:
    """One optimisation step: forward (under autocast when a dtype is given), loss in
    float32, backward, AdamW update.  Returns the detached loss."""
    optimizer.zero_grad(set_to_none=True)
    if autocast_dtype is None:
        loss = loss_fn(model(images), targets)
    else:
        with torch.autocast(device_type=images.device.type, dtype=autocast_dtype):
            logits = model(images)
        loss = loss_fn(logits, targets)
    loss.backward()
    optimizer.step()
    return loss.detach()


class GraphedTrainStep:
    """``train_step`` recorded once into a HIP graph and replayed: for batches small enough that
    a step is bound by the rate at which the host can launch its ~600 kernels (a 3-D step on
    one 32^3 volume: 11 ms eager, 7 ms replayed; a 2-D step on one 128^2 image: 14 ms against
    6 ms on an MI355X), not for the large configurations, whose step keeps the GPU busy.

    The batch shape is fixed at construction.  Construction runs ``warmup`` steps on the given
    batch (the library sizes its launches and the allocator fills its pools on first use),
    records the step, and then puts parameters and optimiser state back to what they were, so
    that the first call is the first step.  The optimiser must keep its state on the device
    (``make_optimizer(model, capturable=True)``).  Every call copies the batch into the
    recorded input buffers, replays, and returns the loss of that step."""

    def __init__(self, model: nn.Module, optimizer: torch.optim.Optimizer, images: Tensor, targets: Tensor,
                 *, autocast_dtype: Optional[torch.dtype] = None,
                 loss_fn: Callable[[Tensor, Tensor], Tensor] = dice_bce_loss, warmup: int = 3):
        if not images.is_cuda:
            raise ValueError("GraphedTrainStep records GPU work: the batch must be on the GPU")
        if not all(group.get("capturable", False) for group in optimizer.param_groups):
            raise ValueError("the optimiser must be built with capturable=True")
        self.model, self.optimizer = model, optimizer
        self.images, self.targets = images.clone(), targets.clone()
        params = [p for group in optimizer.param_groups for p in group["params"]]
        saved_params = [p.detach().clone() for p in params]
        saved_state = {id(p): {k: v.clone() for k, v in optimizer.state[p].items() if torch.is_tensor(v)}
                       for p in params if p in optimizer.state}

        def step():
            return train_step(model, optimizer, self.images, self.targets, autocast_dtype=autocast_dtype,
                              loss_fn=loss_fn)

        side = torch.cuda.Stream(device=images.device)
        side.wait_stream(torch.cuda.current_stream(images.device))
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):
                step()
        torch.cuda.current_stream(images.device).wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self._loss = step()
        # back to the state before the warm-up steps (in place: the graph holds these tensors)
        with torch.no_grad():
            for p, old in zip(params, saved_params):
                p.copy_(old)
                for k, v in optimizer.state.get(p, {}).items():
                    if torch.is_tensor(v):
                        before = saved_state.get(id(p), {}).get(k)
                        v.zero_() if before is None else v.copy_(before)

    def __call__(self, images: Tensor, targets: Tensor) -> Tensor:
        if images.shape != self.images.shape or targets.shape != self.targets.shape:
            raise ValueError("GraphedTrainStep replays one batch shape")
        self.images.copy_(images)
        self.targets.copy_(targets)
        self.graph.replay()
        return self._loss.clone()
