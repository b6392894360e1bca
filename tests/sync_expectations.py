"""What a whole weight sync must hand out, computed on the CPU with the oracle, and the comparison of a sync's
output stream with it: names and order, shapes and dtypes, a 64-bit FNV-1a fingerprint of every tensor on both sides,
and the full bytes of a deterministic sample (first, last, every 17th tensor).

Test infrastructure: used by the whole-configuration GPU tests and by bench.py's parity check, never by the product.
The expectation follows the reference's loop (hf_weight_iterator_direct.py:77-146): every Megatron parameter goes
through its name map, and every HF tensor the quantization config selects through the quantizer.
"""

from __future__ import annotations

from concurrent.futures import ThreadPoolExecutor

import torch

from miles_amd.megatron_to_hf import name_maps

SAMPLE_EVERY = 17


def _bits(t: torch.Tensor) -> torch.Tensor:
    t = t.detach().contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])


def reference_stream_order(names):
    """Parameter names in the order the reference streams them (hf_weight_iterator_direct.py:39-43,85-108,339-341):
    sorted by name, every parameter outside the routed experts before the first routed-expert parameter."""
    routed = lambda n: ".experts." in n and ".shared_experts." not in n
    ordered = sorted(names)
    return [n for n in ordered if not routed(n)] + [n for n in ordered if routed(n)]


def expected_dense_fp8(oracle, args, cpu_params, quantizer: str = "fp8_blockwise_cast"):
    """HF stream of a dense Qwen-style model synced to FP8 128x128: every *_proj.weight becomes codes + scales."""
    quantize = {"fp8_blockwise_cast": oracle.fp8_blockwise_cast, "block_fp8": lambda t: oracle.block_fp8(t, (128, 128))}[quantizer]
    out = []
    for name in reference_stream_order(cpu_params):
        param = cpu_params[name]
        if "word_embeddings" in name or "output_layer" in name:
            param = param[: args.vocab_size]
        for hf, t in name_maps.convert_qwen2_to_hf(args, name, param):
            if hf.endswith("_proj.weight"):
                q, s = quantize(t.contiguous())
                out += [(hf, q), (hf.replace(".weight", ".weight_scale_inv"), s)]
            else:
                out.append((hf, t))
    return out


def expected_moe(oracle, fmt: str, args, cpu_params, basenames=None):
    """HF stream of routed experts synced to `fmt` ("mxfp8", "int4_g128", "nvfp4")."""
    out = []
    for name in reference_stream_order(cpu_params):
        param = cpu_params[name]
        if fmt == "mxfp8":
            for hf, t in name_maps.convert_qwen3moe_to_hf(args, name, param):
                q, s = oracle.mxfp8_quantize(t.contiguous())
                out += [(hf, q), (hf.replace(".weight", ".weight_scale_inv"), s)]
        elif fmt == "int4_g128":
            for hf, t in name_maps.convert_deepseekv3_to_hf(args, name, param):
                assert hf.removesuffix(".weight") in basenames, hf
                packed, scale, _ = oracle.pack_layer(t.contiguous(), 128)
                out += [(hf.replace(".weight", ".weight_packed"), packed), (hf.replace(".weight", ".weight_scale"), scale),
                        (hf.replace(".weight", ".weight_shape"), torch.tensor(t.shape, dtype=torch.int32))]
        elif fmt == "nvfp4":
            hf = name_maps.convert_deepseekv3_to_hf(args, name, param)
            if len(hf) == 2:      # fused gate / up: one amax over both
                results = oracle.nvfp4_quantize_1d_pair(hf[0][1].contiguous(), hf[1][1].contiguous())
            else:
                results = [oracle.nvfp4_quantize_1d(hf[0][1].contiguous())]
            for (n, _), (q, s, g) in zip(hf, results):
                out += [(n, q), (n.replace(".weight", ".weight_scale"), s), (n.replace(".weight", ".weight_scale_2"), g)]
        else:
            raise ValueError(fmt)
    return out


def fingerprints(oracle, tensors, threads: int = 16) -> list[int]:
    """FNV-1a 64 of every tensor's bytes (the C routine releases the interpreter lock, so threads run side by side)."""
    tensors = [t.detach().contiguous() for t in tensors]
    with ThreadPoolExecutor(max_workers=threads) as pool:
        return list(pool.map(oracle.fnv1a64, tensors))


def compare_streams(oracle, got, want, label: str) -> dict:
    """`got` / `want`: lists of (name, CPU tensor).  Raises AssertionError naming every tensor that differs."""
    got_names, want_names = [n for n, _ in got], [n for n, _ in want]
    assert got_names == want_names, (f"{label}: names / order differ (first at index "
                                     f"{next((i for i, (a, b) in enumerate(zip(got_names, want_names)) if a != b), min(len(got_names), len(want_names)))}; "
                                     f"{len(got_names)} vs {len(want_names)} tensors)")
    for (n, g), (_, w) in zip(got, want):
        assert g.shape == w.shape and g.dtype == w.dtype, f"{label}: {n} is {tuple(g.shape)} {g.dtype}, expected {tuple(w.shape)} {w.dtype}"
    hg, hw = fingerprints(oracle, [t for _, t in got]), fingerprints(oracle, [t for _, t in want])
    bad = [n for n, a, b in zip(got_names, hg, hw) if a != b]
    assert not bad, f"{label}: {len(bad)} of {len(got)} tensors differ from the oracle by fingerprint, first: {bad[:5]}"
    sample = sorted(set(range(0, len(got), SAMPLE_EVERY)) | ({0, len(got) - 1} if got else set()))
    for i in sample:
        assert torch.equal(_bits(got[i][1]), _bits(want[i][1])), f"{label}: {got_names[i]} differs from the oracle in its bytes"
    return {"tensors": len(got), "fingerprinted": len(got), "byte_compared": len(sample),
            "bytes": sum(t.numel() * t.element_size() for _, t in got)}
