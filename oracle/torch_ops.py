"""The reference step as its own sequence of torch calls -- TEST INFRASTRUCTURE ONLY.

``reference_step_ops`` issues, tensor for tensor, the ATen calls of
``ramtorch/stochastic_optimizers/adamw.py:160-222`` (upcasts, ``mul_/add_``,
``mul_/addcmul_``, ``sqrt / bcs + eps``, decay ``mul_``, ``addcdiv_``, three
stochastic-rounding write-backs).  The arithmetic of the reference *is* these
torch kernels, so running them on the GPU box is what pins the rounding
sequence ("flavour") that the C oracle and the HIP kernel must reproduce, and
running them on CPU tensors is the CPU baseline of the benchmark.

Differences from the reference, all deliberate: the rounding noise can be
passed in (so results are comparable bit for bit), no device synchronisation,
and the fp32 values before rounding are returned.
"""
from __future__ import annotations

import torch


def sr_write_(target: torch.Tensor, source_fp32: torch.Tensor, noise_i32: torch.Tensor) -> None:
    """copy_stochastic_ (adamw.py:14-30) with the randint result supplied."""
    result = noise_i32.clone()
    result.add_(source_fp32.view(dtype=torch.int32))
    result.bitwise_and_(-65536)
    target.copy_(result.view(dtype=torch.float32))


def draw_noise(shape, seed: int, device) -> torch.Tensor:
    """The reference's own draw (adamw.py:10-21)."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    return torch.randint(low=0, high=(1 << 16), size=shape, dtype=torch.int32, device=device, generator=gen)


def noise_to_i32(noise_i16: torch.Tensor) -> torch.Tensor:
    """int16 bit pattern -> the int32 in [0, 65536) that randint would have produced."""
    return noise_i16.to(torch.int32) & 0xFFFF


@torch.no_grad()
def reference_step_ops(p, grad, ema, ema_squared, *, lr, betas, eps, weight_decay, step, noise=None,
                       compute_device=None, centralization=0):
    """In-place step on ``p`` / ``ema`` / ``ema_squared``; ``step`` is the value
    after the increment (adamw.py:177).  ``noise`` = three int16 tensors, or
    None to draw as the reference does (seeds step+42 / +69 / +420).
    Returns the fp32 (p, ema, ema_squared) before rounding."""
    dev = compute_device if compute_device is not None else p.device
    ema_fp32 = ema.to(dev, non_blocking=True, dtype=torch.float32)                    # :160
    ema_squared_fp32 = ema_squared.to(dev, non_blocking=True, dtype=torch.float32)    # :163
    g = grad.to(torch.float32).to(dev, non_blocking=True)                             # :167
    p_fp32 = p.to(dev, dtype=torch.float32, non_blocking=True)                        # :168
    if g is grad:
        g = g.clone()
    if p_fp32 is p:
        p_fp32 = p_fp32.clone()
    if ema_fp32 is ema:
        ema_fp32 = ema_fp32.clone()
    if ema_squared_fp32 is ema_squared:
        ema_squared_fp32 = ema_squared_fp32.clone()

    if centralization != 0:
        g.sub_(g.mean(dim=tuple(range(1, g.dim())), keepdim=True).mul_(centralization))   # :179-184

    beta1, beta2 = betas
    bias_correction = 1 - beta1 ** step                                               # :186
    bias_correction_sqrt = (1 - beta2 ** step) ** (1 / 2)                             # :187
    step_size = lr / bias_correction                                                  # :188

    ema_fp32.mul_(beta1).add_(g, alpha=1 - beta1)                                     # :190
    ema_squared_fp32.mul_(beta2).addcmul_(g, g, value=1 - beta2)                      # :191
    denom = (ema_squared_fp32.sqrt() / bias_correction_sqrt).add_(eps)                # :193
    if weight_decay != 0:
        p_fp32.mul_(1 - step_size * weight_decay)                                     # :198
    p_fp32.addcdiv_(ema_fp32, denom, value=-step_size)                                # :200

    if noise is None:
        n_p = draw_noise(p_fp32.shape, step + 42, p_fp32.device)                      # :206
        n_m = draw_noise(p_fp32.shape, step + 69, p_fp32.device)                      # :216
        n_v = draw_noise(p_fp32.shape, step + 420, p_fp32.device)                     # :218
    else:
        n_p, n_m, n_v = (noise_to_i32(n.to(p_fp32.device)).view(p_fp32.shape) for n in noise)
    if p.dtype == torch.bfloat16:
        sr_write_(p, p_fp32, n_p)
    else:
        p.copy_(p_fp32)                                                               # :208,214
    if ema.dtype == torch.bfloat16:
        sr_write_(ema, ema_fp32, n_m)
        sr_write_(ema_squared, ema_squared_fp32, n_v)
    else:
        ema.copy_(ema_fp32)                                                           # :221
        ema_squared.copy_(ema_squared_fp32)                                           # :222
    return p_fp32, ema_fp32, ema_squared_fp32
