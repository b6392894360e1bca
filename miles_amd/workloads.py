"""Seeded synthetic inputs shared by the parity tests, smoke() and bench.py.

Everything is generated on the CPU in fp32 with an explicit torch.Generator and
then rounded to the storage dtype, so the CPU oracle and the GPU kernels see the
same bits.  The shape lists and the random / boundary / zeros / maxes patterns
restate the reference's own test inputs:
  tests/fast-gpu/test_mxfp8_quantizer.py:26-59   (MXFP8 shapes, 16*randn, +-512 boundary)
  tests/fast-gpu/test_nvfp4_quantizer.py:43-76   (NVFP4 shapes, randn, +-12 boundary)
  tests/fast-gpu/test_nvfp4_quantizer.py:507-530 (signed zeros, first row zero)
"""

from __future__ import annotations

import torch

REFERENCE_SHAPES = [
    (1, 64),
    (1, 1024),
    (3, 128),
    (16, 64),
    (64, 128),
    (128, 64),
    (256, 128),
    (512, 256),
    (128, 1024),
    (1024, 2048),
    (7168, 2048),
    (2048, 7168),
    (128, 16384),
]
SMALL_REFERENCE_SHAPES = REFERENCE_SHAPES[:9]
NVFP4_QDQ_SHAPES = [(1, 16), (1, 32), (3, 48), (1, 64), (3, 128), (16, 64), (31, 128), (32, 128), (128, 64),
                    (128, 1024), (256, 256), (1024, 2048)]
PATTERNS = ["random", "boundary", "zeros", "maxes"]


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def reference_pattern(kind: str, shape, dtype=torch.bfloat16, *, spread: float, amplitude: float = 1.0,
                      seed: int = 42) -> torch.Tensor:
    """`spread` is the boundary sweep half-width: 512 for the FP8 tests, 12 for NVFP4."""
    m, n = shape
    if kind == "random":
        return (amplitude * torch.randn((m, n), generator=_gen(seed), dtype=torch.float32)).to(dtype)
    if kind == "boundary":
        half = (n + 1) // 2
        base = torch.linspace(-spread, spread, steps=half, dtype=torch.float32)
        eps = torch.full_like(base, 1e-3)
        row = torch.empty(2 * half, dtype=torch.float32)
        row[0::2] = base - eps
        row[1::2] = base + eps
        row = row[:n]
        return row.unsqueeze(0).repeat(m, 1).to(dtype)
    if kind == "zeros":
        return torch.zeros((m, n), dtype=dtype)
    if kind == "signed_zeros":
        return torch.tensor([-0.0, 0.0], dtype=torch.float32).repeat(m, n // 2).to(dtype)
    if kind == "maxes":
        return torch.full((m, n), torch.finfo(dtype).max, dtype=dtype)
    raise ValueError(kind)


def gaussian_outliers(shape, *, std: float, p_outlier: float, gain: float, seed: int,
                      dtype=torch.bfloat16) -> torch.Tensor:
    """x = std*randn; a fraction p_outlier of entries multiplied by gain."""
    g = _gen(seed)
    x = std * torch.randn(shape, generator=g, dtype=torch.float32)
    if p_outlier > 0:
        mask = torch.rand(shape, generator=g, dtype=torch.float32) < p_outlier
        x = torch.where(mask, x * gain, x)
    return x.to(dtype)


def student_t_rows(shape, *, std: float, seed: int, dtype=torch.bfloat16) -> torch.Tensor:
    """x = std*randn * r_i with a per-row heavy-tailed factor r_i = |t_i|, t_i ~ Student-t(3)."""
    g = _gen(seed)
    m, n = shape
    x = std * torch.randn(shape, generator=g, dtype=torch.float32)
    z = torch.randn((m, 1), generator=g, dtype=torch.float32)
    chi2 = (torch.randn((m, 3), generator=g, dtype=torch.float32) ** 2).sum(dim=1, keepdim=True)
    r = (z / torch.sqrt(chi2 / 3.0)).abs()
    return (x * r).to(dtype)


# ---- the five benchmark configurations --------------------------------------
QWEN3_4B = dict(hidden=2560, q=4096, kv=1024, ffn=9728, layers=36)


def c1_mlp(seed: int = 1001):
    """One Qwen3-4B MLP: gate/up [9728,2560], down [2560,9728]; N(0,0.02), 0.1% outliers x20,
    tile (1,1) of gate all zero."""
    out = {}
    for i, (name, shape) in enumerate([("gate_proj", (9728, 2560)), ("up_proj", (9728, 2560)),
                                       ("down_proj", (2560, 9728))]):
        w = gaussian_outliers(shape, std=0.02, p_outlier=0.001, gain=20.0, seed=seed + i)
        if name == "gate_proj":
            w[128:256, 128:256] = 0
        out[name] = w
    return out


def c2_layer_shapes():
    h, q, kv, f = QWEN3_4B["hidden"], QWEN3_4B["q"], QWEN3_4B["kv"], QWEN3_4B["ffn"]
    return [("self_attn.q_proj", (q, h)), ("self_attn.k_proj", (kv, h)), ("self_attn.v_proj", (kv, h)),
            ("self_attn.o_proj", (h, q)), ("mlp.gate_proj", (f, h)), ("mlp.up_proj", (f, h)),
            ("mlp.down_proj", (h, f))]


def c2_tensor(layer: int, idx: int, shape, seed: int = 2001):
    return gaussian_outliers(shape, std=0.02, p_outlier=0.001, gain=20.0, seed=seed + layer * 7 + idx)


def c3_expert(layer: int, expert: int, which: int, seed: int = 3001):
    """Qwen3-30B-A3B expert: which 0/1 = gate/up [768,2048], 2 = down [2048,768]."""
    shape = (768, 2048) if which < 2 else (2048, 768)
    return student_t_rows(shape, std=0.02, seed=seed + (layer * 128 + expert) * 3 + which)


def c4_expert(expert: int, which: int, seed: int = 4001):
    """Kimi-K2-shaped expert: gate/up [2048,7168], down [7168,2048]; N(0,0.015)+0.05% x30."""
    shape = (2048, 7168) if which < 2 else (7168, 2048)
    return gaussian_outliers(shape, std=0.015, p_outlier=0.0005, gain=30.0, seed=seed + expert * 3 + which)


def c5_expert(expert: int, which: int, seed: int = 5001):
    """DeepSeek-V3-shaped expert: gate/up [2048,7168], down [7168,2048]; N(0,0.02)."""
    shape = (2048, 7168) if which < 2 else (7168, 2048)
    return gaussian_outliers(shape, std=0.02, p_outlier=0.0, gain=1.0, seed=seed + expert * 3 + which)
