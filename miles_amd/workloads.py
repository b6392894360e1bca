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


# ---- the same configurations generated on the GPU ---------------------------------------------------------
# Whole models are too large to generate on the CPU in reasonable time (3.6e9 to 2.9e10 elements): these build the
# Megatron-named parameter sets of the benchmark configurations on the device with a seeded device generator.  A
# checker that needs the same bits on the host copies the tensors back.
def device_gaussian_outliers(shape, gen, *, std=0.02, p_outlier=0.001, gain=20.0):
    """bf16 N(0, std) with a fraction p_outlier of entries multiplied by gain."""
    x = torch.randn(shape, generator=gen, device=gen.device, dtype=torch.float32) * std
    if p_outlier > 0:
        x = torch.where(torch.rand(shape, generator=gen, device=gen.device) < p_outlier, x * gain, x)
    return x.to(torch.bfloat16)


def device_student_t_rows(shape, gen, *, std=0.02):
    """bf16 std*randn scaled per row by |t|, t ~ Student-t(3) (= z / sqrt(chi2_3 / 3)): heavy-tailed row magnitudes."""
    m, _ = shape
    x = torch.randn(shape, generator=gen, device=gen.device, dtype=torch.float32) * std
    z = torch.randn((m, 1), generator=gen, device=gen.device, dtype=torch.float32)
    chi2 = (torch.randn((m, 3), generator=gen, device=gen.device, dtype=torch.float32) ** 2).sum(dim=1, keepdim=True)
    return (x * (z / torch.sqrt(chi2 / 3.0)).abs()).to(torch.bfloat16)


def qwen3_4b_megatron(gen, *, layers=QWEN3_4B["layers"], buffer_bytes=512 * 1024**2):
    """Megatron-named parameters of Qwen3-4B (hidden 2560, 32 q heads / 8 kv groups of 128, ffn 9728, `layers` decoder
    layers, embeddings and norms included) -> (args, weights, number of elements the FP8 sync quantizes)."""
    from argparse import Namespace

    h, heads, groups, hd, ffn, vocab = 2560, 32, 8, 128, 9728, 151936
    dev = gen.device
    w = {"module.module.embedding.word_embeddings.weight": device_gaussian_outliers((vocab, h), gen, p_outlier=0)}
    for i in range(layers):
        L = f"module.module.decoder.layers.{i}."
        w[L + "self_attention.linear_qkv.layer_norm_weight"] = torch.ones(h, device=dev, dtype=torch.bfloat16)
        w[L + "self_attention.linear_qkv.weight"] = device_gaussian_outliers(((heads + 2 * groups) * hd, h), gen)
        w[L + "self_attention.q_layernorm.weight"] = torch.ones(hd, device=dev, dtype=torch.bfloat16)
        w[L + "self_attention.k_layernorm.weight"] = torch.ones(hd, device=dev, dtype=torch.bfloat16)
        w[L + "self_attention.linear_proj.weight"] = device_gaussian_outliers((h, heads * hd), gen)
        w[L + "mlp.linear_fc1.layer_norm_weight"] = torch.ones(h, device=dev, dtype=torch.bfloat16)
        w[L + "mlp.linear_fc1.weight"] = device_gaussian_outliers((2 * ffn, h), gen)
        w[L + "mlp.linear_fc2.weight"] = device_gaussian_outliers((h, ffn), gen)
    w["module.module.decoder.final_layernorm.weight"] = torch.ones(h, device=dev, dtype=torch.bfloat16)
    args = Namespace(hidden_size=h, num_attention_heads=heads, num_query_groups=groups, kv_channels=hd,
                     vocab_size=vocab, num_layers=layers, update_weight_buffer_size=buffer_bytes, q_lora_rank=None)
    quantized_elems = layers * (heads * hd * h + 2 * groups * hd * h + h * heads * hd + 3 * ffn * h)
    return args, w, quantized_elems


# the three MoE configurations: model name of the name map, quantization config, (layers, experts, ffn, hidden) and the
# distribution of the expert weights
MOE_CONFIGS = {
    "C3": dict(model_name="qwen3moe", cfg={"quant_method": "mxfp8"}, shape=(48, 128, 768, 2048), dist="student_t"),
    "C4": dict(model_name="kimi_k2",
               cfg={"quant_method": "compressed-tensors", "format": "pack-quantized",
                    "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": True, "num_bits": 4,
                                                              "type": "int"}}}},
               shape=(1, 384, 2048, 7168), dist="outliers_0.015"),
    "C5a": dict(model_name="deepseekv3", cfg={"quant_method": "modelopt", "quant_algo": "NVFP4"},
                shape=(1, 256, 2048, 7168), dist="gaussian_0.02"),
}


def device_expert_tensor(shape, gen, dist: str):
    if dist == "student_t":
        return device_student_t_rows(shape, gen, std=0.02)
    if dist == "outliers_0.015":
        return device_gaussian_outliers(shape, gen, std=0.015, p_outlier=0.0005, gain=30.0)
    if dist == "gaussian_0.02":
        return device_gaussian_outliers(shape, gen, std=0.02, p_outlier=0.0)
    raise ValueError(dist)


def moe_megatron(gen, *, layers, experts, ffn, hidden, dist, buffer_bytes=512 * 1024**2):
    """Megatron-named routed-expert parameters (fused gate/up `linear_fc1` [2*ffn, hidden], `linear_fc2` [hidden, ffn])
    -> (args, weights, elements)."""
    from argparse import Namespace

    w = {}
    for layer in range(layers):
        L = f"module.module.decoder.layers.{layer}."
        for e in range(experts):
            w[L + f"mlp.experts.linear_fc1.weight{e}"] = device_expert_tensor((2 * ffn, hidden), gen, dist)
            w[L + f"mlp.experts.linear_fc2.weight{e}"] = device_expert_tensor((hidden, ffn), gen, dist)
    args = Namespace(hidden_size=hidden, num_attention_heads=32, num_query_groups=4, kv_channels=128, vocab_size=1000,
                     num_layers=layers, update_weight_buffer_size=buffer_bytes, q_lora_rank=None)
    return args, w, layers * experts * 3 * ffn * hidden


def int4_packed_basenames(layers: int, experts: int) -> set[str]:
    """The module names a compressed-tensors checkpoint stores packed: every routed expert projection."""
    return {f"model.layers.{l}.mlp.experts.{e}.{p}_proj" for l in range(layers) for e in range(experts)
            for p in ("gate", "up", "down")}
