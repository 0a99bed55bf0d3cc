"""Writes tests/golden/torch_gpu_step.npz: outputs of torch's own GPU (ROCm)
elementwise kernels for the op sequence of the reference step.

The reference's arithmetic lives in torch's ATen kernels (third-party, not in
the reference tree) and the reference always computes on a GPU, so these
vectors are what "the reference's result" means for given inputs and noise.
Run on a machine with an AMD GPU:

    python tests/golden/make_torch_gpu_golden.py

Inputs are regenerated from seeds by oracle.synth_inputs / synth_noise, so
only the outputs are stored: fp32 values before rounding and bf16 results.
Cases cover several step counts, weight_decay == 0, and edge values (zeros,
denormals, large magnitudes).
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402
from oracle import torch_ops  # noqa: E402

CASES = [
    # name, n, seed, hparams, step
    ("cfg0_step10", 4096, 1234, dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01), 10),
    ("step1", 2048, 11, dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01), 1),
    ("step100_nodecay", 2048, 12, dict(lr=3e-4, betas=(0.95, 0.99), eps=1e-6, weight_decay=0.0), 100),
    ("step5000", 2048, 13, dict(lr=2.5e-3, betas=(0.8, 0.9999), eps=1e-10, weight_decay=0.1), 5000),
]


def edge_inputs():
    """bf16 bit patterns that stress sqrt / division / rounding: zeros, the
    smallest denormals and normals, huge values, exact powers of two."""
    vals = [0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080, 0x0100, 0x3F80, 0xBF80, 0x7F7F, 0xFF7F,
            0x4000, 0x3F00, 0x1234, 0x9234, 0x2B00, 0x6000, 0x0F00, 0x3DCC, 0x3A83]
    pos = [x & 0x7FFF for x in vals]
    import itertools
    combos = list(itertools.product(range(len(vals)), repeat=2))
    p = np.array([vals[a] for a, b in combos], np.uint16)
    g = np.array([vals[b] for a, b in combos], np.uint16)
    m = np.array([vals[(a + b) % len(vals)] for a, b in combos], np.uint16)
    v = np.array([pos[(a * 7 + b) % len(vals)] for a, b in combos], np.uint16)
    return p, g, m, v


def to_t(a, dt=torch.bfloat16):
    return torch.from_numpy(a.view(np.int16).copy()).view(dt).cuda()


def run(p, g, m, v, noise, hp, step):
    P, G, M, V = to_t(p), to_t(g), to_t(m), to_t(v)
    NZ = [torch.from_numpy(z.view(np.int16).copy()).cuda() for z in noise]
    p32, m32, v32 = torch_ops.reference_step_ops(P, G, M, V, step=step, noise=NZ, **hp)
    torch.cuda.synchronize()
    out = {}
    for k, t in (("p32", p32), ("m32", m32), ("v32", v32)):
        out[k] = t.cpu().numpy().view(np.uint32)
    for k, t in (("p16", P), ("m16", M), ("v16", V)):
        out[k] = t.cpu().view(torch.int16).numpy().view(np.uint16)
    return out


def main():
    assert torch.cuda.is_available(), "needs a GPU"
    blob = {"torch_version": np.array(torch.__version__), "device": np.array(torch.cuda.get_device_name(0))}
    for name, n, seed, hp, step in CASES:
        p, g, m, v = oracle.synth_inputs(n, seed)
        noise = oracle.synth_noise(n, seed)
        for k, a in run(p, g, m, v, noise, hp, step).items():
            blob[f"{name}/{k}"] = a
    p, g, m, v = edge_inputs()
    noise = oracle.synth_noise(p.size, 99)
    hp = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    for k, a in run(p, g, m, v, noise, hp, 10).items():
        blob[f"edge/{k}"] = a
    out_dir = os.environ.get("GOLDEN_OUT", os.path.dirname(os.path.abspath(__file__)))
    os.makedirs(out_dir, exist_ok=True)
    path = os.path.join(out_dir, "torch_gpu_step.npz")
    np.savez_compressed(path, **blob)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
