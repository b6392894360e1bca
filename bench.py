#!/usr/bin/env python3
"""Benchmark of the weight-quantization hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu-baseline]

One step = one full Qwen3-4B weight sync to FP8 128x128 block scales (BASELINE.json configs[1]): the 36
layers' Megatron-named bf16 parameters, resident in HBM, stream through the sync driver
(name map -> fp8_blockwise_cast -> buckets) exactly as a trainer->engine update would, with the consumer
replaced by a no-op.  `value` is algorithmic GB/s of that sync (input read once + codes and scales written
once, 3.000244 B/element) and `ms_per_step` the wall-clock milliseconds per full-model sync.

The JSON line also carries
  roofline      the dominant kernel (fp8_block128_kernel, one grouped launch per bucket) timed live with
                events on the launch stream; peak = 8 TB/s HBM
  cpu_baseline  the CPU oracle (bit-exact port) timed on the host cores on a bounded sample of the workload
  per_quantizer GB/s of every quantizer on its BASELINE.json configuration shape (not part of `value`)
  parity        every tensor one sync hands out compared with the oracle (fingerprints of all, bytes of a sample)
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
BYTES_PER_ELEM = {"fp8_block": 2 + 1 + 4 / 16384, "fp8_dequant": 1 + 4 / 16384 + 2, "mxfp8": 2 + 1 + 1 / 32,
                  "int4_g128": 2 + 0.5 + 2 / 128, "nvfp4": 2 + 0.5 + 1 / 16,
                  # formats either side of the path: MXFP4 (group 32), INT4 unpack, asymmetric INT4 (one zero-point nibble per group)
                  "mxfp4": 2 + 0.5 + 1 / 32, "mxfp4_dequant": 0.5 + 1 / 32 + 2, "int4_unpack": 0.5 + 2 / 128 + 2,
                  "int4_g128_asym": 2 + 0.5 + 2 / 128 + 0.5 / 128, "fake_quant_bf16": 2 + 2, "act_quant": 2 + 1 + 4 / 128, "fake_int4_bf16": 2 + 2 + 2 / 128, "fp8_channel": 2 + 1,
                  "mxfp4_to_fp8": 0.5 + 1 / 32 + 1 + 4 / 16384, "fp8_to_mxfp8": 1 + 4 / 16384 + 1 + 1 / 32}
# HBM bytes per element of the FP8 tile kernel measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each
# scaled by the same counter on a plain 1 GiB copy (read 2.0003 + write 1.0005 B per element)
MEASURED_FP8_TRAFFIC_BYTES_PER_ELEM = 3.0008

METRIC = "HBM GB/s (% of peak) per quantizer; ms per full-model BF16->FP8 weight sync"
DEV = "cuda:0"


def _synth(shape, gen, *, std=0.02, p=0.001, gain=20.0):
    """bf16 N(0, std) with a fraction p of entries multiplied by gain, generated on the GPU."""
    from miles_amd import workloads as W

    return W.device_gaussian_outliers(shape, gen, std=std, p_outlier=p, gain=gain)


def qwen3_4b_megatron_weights(gen):
    """Megatron-named parameters of Qwen3-4B: hidden 2560, 32 q heads / 8 kv groups of 128, ffn 9728, 36 layers."""
    from miles_amd import workloads as W

    return W.qwen3_4b_megatron(gen)


TIMED_ITERS = 5        # repetitions per per-quantizer measurement (1 in the counter-collection run)


def _event_ms(fn, iters):
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def _event_ms_each(fn, before_each, iters):
    """As _event_ms, with `before_each()` run ahead of every repetition and kept out of the timed span (it stands for
    what the trainer does between two syncs): one event pair per repetition."""
    total = 0.0
    for _ in range(iters):
        before_each()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        total += e0.elapsed_time(e1)
    return total / iters


def _best_ms(fn):
    """Per-quantizer figure: the fastest of three timed runs of TIMED_ITERS repetitions (memory that the allocator mapped
    a moment ago streams slower on its first passes); a single run when counters are being collected."""
    return min(_event_ms(fn, TIMED_ITERS) for _ in range(1 if TIMED_ITERS == 1 else 3))


def _record(build):
    """Record the quantizer calls of `build()` into a replayable batch."""
    from miles_amd import launch

    with launch.recording() as batch:
        outs = build()
    batch.device = torch.device(DEV)
    batch.freeze()
    batch.run()
    torch.cuda.synchronize()
    return batch, outs


def per_quantizer(gen):
    """GB/s of each quantizer on its configuration shape (a bounded number of tensors, replayed batches)."""
    from miles_amd.kernels.quant.int4_fake import pack_layer
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant
    from miles_amd.utils.mxfp8 import mxfp8_quantize
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d, nvfp4_quantize_1d_pair
    from miles_amd import workloads as W

    res = {}

    def run(name, key, elems, build, note, prepare=None, before_each=None):
        batch, outs = _record(build)
        if prepare is not None:
            prepare(batch)
        if before_each is not None:
            ms = min(_event_ms_each(batch.run, before_each, TIMED_ITERS) for _ in range(1 if TIMED_ITERS == 1 else 3))
        else:
            ms = _best_ms(batch.run)
        gbps = elems * BYTES_PER_ELEM[key] / ms / 1e6
        res[name] = {"GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "ms": round(ms, 4),
                     "elements": elems, "workload": note}
        del batch, outs     # no empty_cache(): freshly mapped device memory streams measurably slower than reused blocks

    # C1: one Qwen3-4B MLP, block_fp8; 8 distinct copies so that the 256 MB memory-side cache cannot hold the input
    mlp = [[_synth((9728, 2560), gen), _synth((9728, 2560), gen), _synth((2560, 9728), gen)] for _ in range(8)]
    mlp[0][0][128:256, 128:256] = 0
    run("C1_block_fp8", "fp8_block", 8 * 3 * 9728 * 2560,
        lambda: [block_fp8(t, [128, 128]) for m in mlp for t in m], "8 x Qwen3-4B MLP (gate, up, down), block_fp8")
    del mlp
    # C3: Qwen3-30B-A3B experts, MXFP8; 2 layers of 128 experts
    experts = [(W.device_student_t_rows((1536, 2048), gen), W.device_student_t_rows((2048, 768), gen)) for _ in range(256)]
    run("C3_mxfp8", "mxfp8", 256 * 3 * 768 * 2048,
        lambda: [mxfp8_quantize(t) for fc1, fc2 in experts for t in (*fc1.chunk(2, dim=0), fc2)],
        "2 layers x 128 experts (gate, up [768,2048], down [2048,768]), 0.02 N(0,1) x Student-t(3) row scales")
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast
    run("next_fp8_cast_small_experts", "fp8_block", 256 * 3 * 768 * 2048,
        lambda: [fp8_blockwise_cast(t) for fc1, fc2 in experts for t in (*fc1.chunk(2, dim=0), fc2)],
        "the same 768 expert matrices through the sync path's FP8 128x128 quantizer (one launch over a device table)")
    del experts
    # C4: Kimi-K2-shaped experts, 32 of them, N(0, 0.015) + 0.05 % outliers x 30
    experts = [(_synth((4096, 7168), gen, std=0.015, p=0.0005, gain=30.0), _synth((7168, 2048), gen, std=0.015, p=0.0005, gain=30.0))
               for _ in range(32)]
    n = 32 * 3 * 2048 * 7168
    run("C4_int4_g128_pack", "int4_g128", n,
        lambda: [pack_layer(t, 128) for fc1, fc2 in experts for t in (*fc1.chunk(2, dim=0), fc2)],
        "32 experts (gate, up [2048,7168], down [7168,2048]), pack_layer group 128")
    del experts
    # C5: DeepSeek-V3-shaped experts, 32 of them, N(0, 0.02)
    experts = [(_synth((4096, 7168), gen, p=0), _synth((7168, 2048), gen, p=0)) for _ in range(32)]

    def nvfp4_all():
        out = []
        for fc1, fc2 in experts:
            out.append(nvfp4_quantize_1d_pair(*fc1.chunk(2, dim=0)))
            out.append(nvfp4_quantize_1d(fc2))
        return out

    # NVFP4 as the sync driver runs it: the first sync of a model takes two passes (amax, then quantize); every later sync
    # quantizes in one pass with the amax its records kept and repeats only the tensors whose amax moved
    run("C5a_nvfp4", "nvfp4", n, nvfp4_all,
        "32 experts, gate/up paired + down; steady-state sync: one pass with the amax carried over from the previous sync "
        "(checked on the way; here no amax moves)", prepare=lambda b: b.carry_amax())
    run("C5a_nvfp4_first_sync", "nvfp4", n, nvfp4_all, "as C5a, first sync of a model: amax pass + quantize pass")
    res.update(nvfp4_after_update(gen, experts, nvfp4_all, n))
    firsts = [t.view(-1)[:1] for fc1, fc2 in experts for t in (fc1, fc2)]
    for f in firsts:
        f.fill_(1.0)            # the largest element of every tensor (of every gate/up pair), toggled below
    toggle = [4.0]

    def move_every_amax():
        torch._foreach_mul_(firsts, toggle[0])
        toggle[0] = 1.0 / toggle[0]

    run("C5a_nvfp4_every_amax_moved", "nvfp4", n, nvfp4_all,
        "as C5a, worst case of the carried amax: every tensor's amax differs from the last sync's; the batch sees that "
        "in the moved-record count of the syncs before and submits the plain two-pass form (the first-sync cost)",
        prepare=lambda b: b.carry_amax(), before_each=move_every_amax)
    os.environ["NVTE_NVFP4_4OVER6"] = "weights"        # Four Over Six: two candidates per block, e4m3 max 256
    try:
        run("C5a_nvfp4_four_over_six", "nvfp4", n, nvfp4_all,
            "as C5a (steady state) with NVTE_NVFP4_4OVER6=weights (MAE, e4m3 max 256)", prepare=lambda b: b.carry_amax())
    finally:
        del os.environ["NVTE_NVFP4_4OVER6"]
    run("C5b_block_fp8", "fp8_block", n,
        lambda: [block_fp8(t, [128, 128]) for fc1, fc2 in experts for t in (*fc1.chunk(2, dim=0), fc2)],
        "32 experts, block_fp8")
    quantized = [block_fp8(t, [128, 128]) for fc1, fc2 in experts for t in (*fc1.chunk(2, dim=0), fc2)]
    torch.cuda.synchronize()
    del experts
    run("C5b_fp8_dequant", "fp8_dequant", n, lambda: [weight_dequant(q, s) for q, s in quantized],
        "32 experts, FP8 block -> bf16")
    del quantized
    # the same four quantizers on fp16 weights (a model trained in fp16): their kernels have fp16 instances
    half = [(_synth((4096, 7168), gen, p=0).to(torch.float16), _synth((7168, 2048), gen, p=0).to(torch.float16)) for _ in range(32)]
    parts = lambda: [t for fc1, fc2 in half for t in (*fc1.chunk(2, dim=0), fc2)]
    note = "32 DeepSeek-V3-shaped experts held in fp16"
    run("fp16_weights_fp8_blockwise_cast", "fp8_block", n, lambda: [fp8_blockwise_cast(t) for t in parts()], note)
    run("fp16_weights_mxfp8", "mxfp8", n, lambda: [mxfp8_quantize(t) for t in parts()], note)
    run("fp16_weights_int4_g128_pack", "int4_g128", n, lambda: [pack_layer(t, 128) for t in parts()], note)
    run("fp16_weights_nvfp4", "nvfp4", n, lambda: [nvfp4_quantize_1d(t) for t in parts()], note + ", amax carried over",
        prepare=lambda b: b.carry_amax())
    del half
    res.update(adjacent_formats(gen))
    return res


def nvfp4_after_update(gen, experts, build, elems):
    """NVFP4 syncs with a training step between them.  fp32 master weights take an Adam-sized step (every element moves
    by lr x a unit-variance direction) and are rounded to bf16 in place; the sync after each step is timed on its own
    (events around the job list) and the amax records say how many tensors had to be quantized in the second pass.
    A weight's bf16 value changes when its master crosses a rounding boundary, so with lr = 1e-6 (an RL fine-tuning
    rate) about one element in a hundred changes per step and a tensor's amax only now and then."""
    from miles_amd import _lib

    tensors = [t for fc1, fc2 in experts for t in (fc1, fc2)]
    out = {}
    for lr, label in ((1e-6, "lr1e-6"), (1e-4, "lr1e-4")):
        masters = [t.float() for t in tensors]
        batch, outs = _record(build)
        batch.carry_amax()
        batch.run()
        torch.cuda.synchronize()
        total_ms, redone, records, changed, steps = 0.0, 0, 0, 0.0, 8
        for _ in range(steps):
            before = tensors[0].clone()
            for m, t in zip(masters, tensors):
                m.add_(torch.randn(m.shape, generator=gen, device=DEV), alpha=lr)
                t.copy_(m)
            changed += (tensors[0] != before).float().mean().item()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            batch.run()
            e1.record()
            torch.cuda.synchronize()
            total_ms += e0.elapsed_time(e1)
            recs = torch.stack([r[_lib.RECORD_REDO_WORD] for r in batch.amax_records()])
            redone += int(recs.sum().item())
            records += recs.numel()
        ms = total_ms / steps
        gbps = elems * BYTES_PER_ELEM["nvfp4"] / ms / 1e6
        out[f"C5a_nvfp4_after_update_{label}"] = {
            "GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "ms": round(ms, 4), "elements": elems,
            "fraction_of_tensors_quantized_in_the_second_pass": round(redone / max(records, 1), 4),
            "fraction_of_bf16_values_changed_per_step": round(changed / steps, 4),
            "workload": f"as C5a, {steps} syncs each after an optimizer step of size lr = {lr:g} on fp32 master weights "
                        "(unit-variance direction), rounded to bf16 in place"}
        for m, t in zip(masters, tensors):
            del m
        del masters, batch, outs
    return out


def full_configs(gen):
    """The three MoE configurations at their full element counts and on their own data distributions, each as one whole
    weight sync through the driver (`WeightUpdater` with a replayed plan, 512 MiB buckets): every expert of every layer
    at its real shape.  Timed like the headline: K syncs between two events on the launch stream and a wall clock."""
    from miles_amd import workloads as W
    from miles_amd.weight_update.updater import WeightUpdater

    def sync(key, fmt, note):
        conf = W.MOE_CONFIGS[key]
        layers, experts, ffn, hidden = conf["shape"]
        args, weights, elems = W.moe_megatron(gen, layers=layers, experts=experts, ffn=ffn, hidden=hidden, dist=conf["dist"])
        extra = {"packed_weight_basenames": W.int4_packed_basenames(layers, experts)} if fmt == "int4_g128" else {}
        seen = {"buckets": 0, "tensors": 0}

        def consume(bucket):
            seen["buckets"] += 1
            seen["tensors"] += len(bucket)

        torch.cuda.synchronize()
        resident = torch.cuda.memory_allocated()
        upd = WeightUpdater(args, weights_getter=lambda: weights, model_name=conf["model_name"],
                            quantization_config=conf["cfg"], send_bucket=consume, **extra)
        t0 = time.perf_counter()
        upd.update_weights()
        torch.cuda.synchronize()
        first_s = time.perf_counter() - t0
        assert upd._plan is not None and upd._plan.replayable, key
        # untimed syncs until the GPU is out of its idle clocks (the first sync after a pause runs 10 % longer)
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.2:
            upd.update_weights()
            torch.cuda.synchronize()
        seen.update(buckets=0, tensors=0)
        steps = 10
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            upd.update_weights()
        e1.record()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / steps * 1e3
        gpu_ms = e0.elapsed_time(e1) / steps
        gbps = elems * BYTES_PER_ELEM[fmt] / ms / 1e6
        out = {"GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "ms_per_sync": round(ms, 3),
               "gpu_ms_per_sync": round(gpu_ms, 3), "elements": elems, "megatron_tensors": len(weights),
               "hf_tensors_per_sync": seen["tensors"] // steps, "buckets_per_sync": seen["buckets"] // steps,
               "jobs": len(upd._plan.batch), "first_sync_s": round(first_s, 2),
               "sync_output_bytes_resident": torch.cuda.memory_allocated() - resident, "workload": note}
        del upd, weights
        return out

    return {
        "C3_full": sync("C3", "mxfp8", "Qwen3-30B-A3B: 48 layers x 128 experts, gate/up [768,2048] down [2048,768], MXFP8 1x32 "
                                       "E8M0, rows 0.02 N(0,1) x |Student-t(3)|"),
        "C4_full": sync("C4", "int4_g128", "Kimi-K2-shaped: 384 experts, gate/up [2048,7168] down [7168,2048], INT4 group 128 "
                                           "packed, N(0,0.015) + 0.05% x30"),
        "C5a_full": sync("C5a", "nvfp4", "DeepSeek-V3-shaped: 256 experts, gate/up [2048,7168] paired + down [7168,2048], "
                                         "NVFP4 1x16, N(0,0.02); steady state (amax carried over, none moved)"),
    }


def full_model_block_fp8(weights, elems):
    """The whole model through the offline tool's quantizer (`block_fp8`: exact division, all-zero-tile rule) instead
    of the sync path's `fp8_blockwise_cast`: same tensors and traffic, the variant whose bytes the reference's CPU code
    can confirm."""
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8

    targets = [t for name, t in weights.items() if t.dim() == 2 and "embedding" not in name and "output_layer" not in name]
    assert sum(t.numel() for t in targets) == elems
    batch, outs = _record(lambda: [block_fp8(t, [128, 128]) for t in targets])
    ms = _best_ms(batch.run)
    gbps = elems * BYTES_PER_ELEM["fp8_block"] / ms / 1e6
    del batch, outs
    return {"GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "ms": round(ms, 4), "elements": elems,
            "workload": "all 36 Qwen3-4B layers (fused qkv, o, fc1, fc2 as stored), block_fp8, one job list"}


def adjacent_formats(gen):
    """GB/s of the kernels either side of the path (MXFP4 pack / unpack, INT4 unpack, asymmetric INT4 pack, the two
    re-coders) on eight [16384, 7168] tensors, each as one job list: the way the converters submit a shard."""
    from miles_amd.kernels.quant.int4_fake import pack_layer
    from miles_amd.tools.convert_kimi_int4_to_bf16 import _dequantize_tensor
    from miles_amd.utils.mxfp4 import dequantize_mxfp4, quantize_mxfp4

    res = {}
    shape, count = (16384, 7168), 8
    elems = count * shape[0] * shape[1]
    ws = [_synth(shape, gen, std=0.015, p=0.0005, gain=30.0) for _ in range(count)]

    def run(name, key, fn, note):
        fn()
        torch.cuda.synchronize()
        ms = _best_ms(fn)
        gbps = elems * BYTES_PER_ELEM[key] / ms / 1e6
        res[name] = {"GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "ms": round(ms, 4),
                     "elements": elems, "workload": note}

    batch, m4 = _record(lambda: [quantize_mxfp4(w, 32) for w in ws])
    ms = _best_ms(batch.run)
    gbps = elems * BYTES_PER_ELEM["mxfp4"] / ms / 1e6
    res["next_mxfp4_quant"] = {"GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "ms": round(ms, 4),
                               "elements": elems, "workload": "8 x [16384,7168] bf16, group 32, one grouped launch"}
    del batch
    # (the converters unpack a shard's tensors together, launch.deferred: the lines are job lists)
    batch, outs = _record(lambda: [dequantize_mxfp4(p, s, 32) for p, s in m4])
    run("next_mxfp4_dequant", "mxfp4_dequant", batch.run, "MXFP4 -> bf16, one job list (single calls: 0.80 of peak at this size)")
    del batch, outs
    from miles_amd.tools.convert_mxfp4_to_fp8 import cast_e2m1fn_to_e4m3fn
    # the converter submits a shard's casts together (launch.deferred), so the line is a job list too
    batch, outs = _record(lambda: [cast_e2m1fn_to_e4m3fn(p.view(torch.int8), s) for p, s in m4])
    run("next_mxfp4_to_fp8_recode", "mxfp4_to_fp8", batch.run,
        "MXFP4 -> e4m3 with 128x128 fp32 tile scales, one job list: tile scales, then a flat stream (single calls: 0.65 of peak at this size)")
    del batch, outs, m4
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8
    from miles_amd.utils.mxfp8 import requantize_fp8_block_to_mxfp8
    f8 = [block_fp8(w, [128, 128]) for w in ws]
    batch, outs = _record(lambda: [requantize_fp8_block_to_mxfp8(q, s) for q, s in f8])
    run("next_fp8_to_mxfp8", "fp8_to_mxfp8", batch.run,
        "FP8 128x128 block-scaled codes (general fp32 scales) -> MXFP8 in one pass, as the MXFP8 converter submits a shard: one job list")
    del batch, outs, f8
    i4 = [pack_layer(w, 128) for w in ws]
    batch, outs = _record(lambda: [_dequantize_tensor(p, s, shape, 128) for p, s, _ in i4])
    run("next_int4_unpack", "int4_unpack", batch.run, "INT4 g128 -> bf16, one job list (single calls: 0.78 of peak at this size)")
    del batch, outs
    del i4
    batch, outs = _record(lambda: [pack_layer(w, 128, sym=False) for w in ws])
    run("next_int4_g128_asym_pack", "int4_g128_asym", batch.run,
        "pack_layer(sym=False), group 128, as the sync path runs it: one job list, two grouped launches")
    del batch, outs
    from miles_amd.tools.convert_hf_to_fp8 import channel_fp8, tensor_fp8
    run("a2_channel_fp8", "fp8_channel", lambda: [channel_fp8(w) for w in ws], "one scale per row, rows read once")
    # per-tensor FP8 is a job of the batched driver: timed as a replayed job list, like the sync path runs it
    batch, outs = _record(lambda: [tensor_fp8(w) for w in ws])
    ms = _best_ms(batch.run)
    gbps = elems * BYTES_PER_ELEM["fp8_channel"] / ms / 1e6
    res["a2_tensor_fp8_first_sync"] = {"GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "ms": round(ms, 4),
                                       "elements": elems, "workload": "one scale per tensor, first sync of a model: amax pass + "
                                       "quantize pass (5 B/element moved, 3 counted)"}
    batch.carry_amax()
    ms = _best_ms(batch.run)
    gbps = elems * BYTES_PER_ELEM["fp8_channel"] / ms / 1e6
    res["a2_tensor_fp8"] = {"GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "ms": round(ms, 4),
                            "elements": elems, "workload": "one scale per tensor, steady-state sync: one pass with the amax "
                            "carried over from the previous sync (checked on the way; here no amax moves)"}
    del batch, outs
    from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda
    run("a8_fake_int4_quant_1x128", "fake_int4_bf16", lambda: [fake_int4_quant_cuda(w, [1, 128], True) for w in ws],
        "fake_int4_quant_cuda(x, (1,128), sym): bf16 in, bf16 integer codes + bf16 scales out")
    from miles_amd.kernels.quant.nvfp4_qdq import NVFP4QDQConfig, compute_nvfp4_amax, fused_nvfp4_qdq
    amaxes = [compute_nvfp4_amax(w) for w in ws]
    run("next_nvfp4_qdq", "fake_quant_bf16", lambda: [fused_nvfp4_qdq(w, a, NVFP4QDQConfig()) for w, a in zip(ws, amaxes)],
        "fused NVFP4 quantize-dequantize given the amax, bf16 in, bf16 out")
    from miles_amd.kernels.quant import fake_quant as fq
    for name, fn in (("fp8", fq.fake_quant_fp8_forward), ("fp4", fq.fake_quant_fp4_forward),
                     ("compressed_kv", fq.fake_quant_compressed_kv_forward)):
        run(f"next_fake_quant_{name}", "fake_quant_bf16", lambda fn=fn: [fn(w) for w in ws], "bf16 in, bf16 out")
    from miles_amd.kernels.quant.fp8_act_quant import act_quant, fp8_simulate
    run("next_act_quant_fp8_1x128", "act_quant", lambda: [act_quant(w, 128, "ue8m0") for w in ws],
        "1x128 groups, power-of-two fp32 scales, bf16 -> e4m3 codes")
    run("next_fp8_simulate_1x128", "fake_quant_bf16", lambda: [fp8_simulate(w, 128) for w in ws],
        "1x128 quantize + cast back in one pass, bf16 in, bf16 out")
    return res


def packed_payload(args, weights, fp8_cfg, steps):
    """The same sync producing the flattened transport payload of every bucket (the reference's broadcast_packed
    mode).  `in_place_ms`: quantizers write into the payload, only pass-through tensors are copied.
    `flatten_after_ms`: the reference's order of work -- quantize, then copy every tensor of the bucket into the
    payload -- with this library's own grouped copy kernel."""
    from miles_amd.weight_update.packed_bucket import pack_bucket
    from miles_amd.weight_update.updater import WeightUpdater

    def timed(updater):
        updater.update_weights()
        updater.update_weights()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            updater.update_weights()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    seen = {"bytes": 0}
    in_place = WeightUpdater(args, weights_getter=lambda: weights, model_name="qwen3", quantization_config=fp8_cfg,
                             send_bucket=lambda b: seen.__setitem__("bytes", seen["bytes"] + b.flat.numel()),
                             packed_buckets=True)
    ms_in_place = timed(in_place)
    assert in_place._plan is not None and in_place._plan.replayable
    payload_bytes = seen["bytes"] // (steps + 2)
    del in_place
    after = WeightUpdater(args, weights_getter=lambda: weights, model_name="qwen3", quantization_config=fp8_cfg,
                          send_bucket=pack_bucket)
    ms_after = timed(after)
    return {"in_place_ms": round(ms_in_place, 4), "flatten_after_ms": round(ms_after, 4), "payload_bytes": payload_bytes,
            "note": "one sync = quantize + build every bucket's flat payload (embeddings and norms included)"}


def launches_per_sync(plan):
    """Kernel launches of one replayed sync: every submission of the plan is cut into launches of up to MAX_GROUP
    consecutive jobs of one kind (the headline sync has only FP8 128x128 jobs)."""
    from miles_amd import _lib

    n, done = 0, 0
    for mark in plan.submission_marks():
        n += -(-(mark - done) // _lib.MAX_GROUP) if mark > done else 0
        done = max(done, mark)
    return n


def roofline(plan, elems, steps, gpu_ms):
    """The dominant kernel over the timed region itself: `gpu_ms` is the time between two events recorded on the launch
    stream around the `steps` timed syncs.  The launches run back to back on that one stream, so the elapsed time over
    their count is the average launch duration plus the gap to the next launch: it can only understate the kernel, and
    launches_per_sync x avg_launch_us <= ms_per_step holds by construction (the wall clock contains the event span)."""
    launches = launches_per_sync(plan)
    avg_us = gpu_ms * 1e3 / (steps * launches)
    bytes_per_launch = elems * BYTES_PER_ELEM["fp8_block"] / launches
    achieved = bytes_per_launch / avg_us / 1e3
    return {"bound": "hbm", "kernel": "mq::fp8_block128_kernel<1, mq::TileTable, 0>", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
            "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": round(MEASURED_FP8_TRAFFIC_BYTES_PER_ELEM * elems / launches),
            "launches_per_sync": launches, "avg_launch_us": round(avg_us, 2),
            "algorithmic_bytes_per_launch": round(bytes_per_launch),
            "timed_with": f"one event pair on the launch stream around the {steps} timed syncs ({steps * launches} launches)"}


def cpu_baseline(weights, args, budget_s=12.0):
    """The oracle's fp8_blockwise_cast on layer 0's HF tensors, repeated until `budget_s` of CPU time is spent."""
    from miles_amd.megatron_to_hf import name_maps
    from oracle import mq_oracle

    mq_oracle.build()
    tensors = []
    for rest in ("self_attention.linear_qkv.weight", "self_attention.linear_proj.weight", "mlp.linear_fc1.weight",
                 "mlp.linear_fc2.weight"):
        name = "module.module.decoder.layers.0." + rest
        for _hf, t in name_maps.convert_qwen2_to_hf(args, name, weights[name].cpu()):
            tensors.append(t.contiguous())
    elems = sum(t.numel() for t in tensors)
    t0 = time.perf_counter()
    reps = 0
    while True:
        for t in tensors:
            mq_oracle.fp8_blockwise_cast(t)
        reps += 1
        if time.perf_counter() - t0 > budget_s:
            break
    dt = time.perf_counter() - t0
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    out = {"value": round(reps * elems * BYTES_PER_ELEM["fp8_block"] / dt / 1e9, 3), "unit": "GB/s", "cores": threads,
           "kind": "port", "sample": f"{reps} x one Qwen3-4B layer (q,k,v,o,gate,up,down = {elems} elements) through "
                                      f"the OpenMP C oracle's fp8_blockwise_cast, {dt:.1f} s"}
    out["torch_cpu_op_chain"] = _torch_cpu_block_fp8(tensors[-3])
    return out


def _torch_cpu_block_fp8(w, budget_s=4.0):
    """The offline tool's block_fp8 as the reference writes it -- pad, reshape to tiles, abs/max, divide, clamp, cast
    (tools/convert_hf_to_fp8.py:39-70) -- run by PyTorch's CPU kernels on one gate_proj: the closest thing to the
    reference's own CPU path.  Reported next to the oracle figure, not used for anything else."""
    n, k = w.shape
    nt, kt = -(-n // 128), -(-k // 128)

    def chain():
        padded = torch.nn.functional.pad(w, (0, kt * 128 - k, 0, nt * 128 - n), mode="constant", value=0.0)
        tiles = padded.reshape(nt, 128, kt, 128)
        amax = tiles.abs().max(dim=1, keepdim=True)[0].max(dim=3, keepdim=True)[0]
        scale = amax.to(torch.float32) / 448.0
        q = (tiles / scale).clamp(min=-448.0, max=448.0).reshape(nt * 128, kt * 128).to(torch.float8_e4m3fn)
        return q[:n, :k], scale

    chain()
    t0, reps = time.perf_counter(), 0
    while time.perf_counter() - t0 < budget_s:
        chain()
        reps += 1
    dt = time.perf_counter() - t0
    return {"value": round(reps * w.numel() * BYTES_PER_ELEM["fp8_block"] / dt / 1e9, 3), "unit": "GB/s",
            "cores": torch.get_num_threads(), "sample": f"{reps} x block_fp8 op chain on gate_proj {tuple(w.shape)}, {dt:.1f} s"}


def parity_whole_sync(weights, args, updater):
    """Every tensor one sync hands out (252 quantized weights with their scales, embeddings and norms) against the
    oracle applied to the same weights: names and order, a 64-bit fingerprint of every tensor, full bytes of the first,
    the last and every 17th."""
    from oracle import mq_oracle
    from tests import sync_expectations as E

    mq_oracle.build()
    want = E.expected_dense_fp8(mq_oracle, args, {k: v.cpu() for k, v in weights.items()})
    got = []
    consumer, updater.send_bucket = updater.send_bucket, lambda bucket: got.extend((n, t.cpu()) for n, t in bucket)
    try:
        updater.update_weights()
        torch.cuda.synchronize()
    finally:
        updater.send_bucket = consumer
    try:
        stats = E.compare_streams(mq_oracle, got, want, "timed sync")
    except AssertionError as exc:
        raise SystemExit(f"PARITY FAILURE: {exc}") from None
    quantized = sum(n.endswith("_proj.weight") for n, _ in want)
    return (f"ok ({quantized} quantized tensors + their scales + {stats['tensors'] - 2 * quantized} pass-through tensors of the "
            f"whole sync: every 64-bit fingerprint equal to the oracle's, {stats['byte_compared']} tensors compared byte for byte)")


def stream_ceilings():
    """What plain streaming kernels reach on this GPU: torch's own elementwise kernels on 4 GiB operands, and the
    library's byte-copy job (one 16-byte unit per lane, no loop) on the same buffers: yardsticks for the per-quantizer
    fractions."""
    from miles_amd.weight_update.packed_bucket import submit_copy

    n = 1 << 31
    x = torch.empty(n, dtype=torch.bfloat16, device=DEV).normal_()
    y = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    q = torch.empty(n, dtype=torch.float8_e4m3fn, device=DEV)
    res = {}
    for name, fn, nbytes in (("fill_write_only", lambda: y.fill_(1.0), 2 * n),
                             ("copy_bf16_1r_1w", lambda: y.copy_(x), 4 * n),
                             ("library_copy_job_1r_1w", lambda: submit_copy(x, y), 4 * n),
                             ("cast_bf16_to_fp8_2r_1w", lambda: q.copy_(x), 3 * n),
                             ("cast_fp8_to_bf16_1r_2w", lambda: y.copy_(q), 3 * n)):
        fn()
        torch.cuda.synchronize()
        ms = min(_event_ms(fn, 5) for _ in range(3))
        res[name] = {"GBps": round(nbytes / ms / 1e6, 1), "ms": round(ms, 4)}
    del q
    # the library's probes: kernels that only move bytes, in the access shapes of the quantizers (2 GiB on the larger side)
    from miles_amd import _lib, _probes
    from miles_amd._probes import FLAT_1_2, FLAT_2_1, LOOP_2_1, TILE_2_1, TILE_READ, TILE_WRITE
    lib, stream, big = _probes.load(), _lib.stream_ptr(x.device), 1 << 31

    def probe(name, shape, param, moved):
        def fn():
            _probes.check(lib.mqp_stream_probe(shape, x.data_ptr(), y.data_ptr(), big, param, stream))
        fn()
        torch.cuda.synchronize()
        ms = min(_event_ms(fn, 10) for _ in range(3))
        res[name] = {"GBps": round(moved / ms / 1e6, 1), "ms": round(ms, 4)}

    for units in (1, 2, 4, 8):
        probe(f"flat_2r_1w_{units}_units_per_lane", FLAT_2_1, units, big * 3 // 2)
    for groups in (2048, 16384, 65536, 262144):
        probe(f"loop_2r_1w_{groups}_workgroups", LOOP_2_1, groups, big * 3 // 2)
    for units in (1, 2):
        probe(f"flat_1r_2w_{units}_units_per_lane", FLAT_1_2, units, big * 3 // 2)
    for k in (2048, 2560, 4096, 5120, 7168, 8192, 9728):
        elems = (big // 2 // k // 128 * 128) * k
        probe(f"tile128_2r_1w_K{k}", TILE_2_1, k, elems * 3)
        probe(f"tile128_read_only_K{k}", TILE_READ, k, elems * 2)
        probe(f"tile128_write_only_K{k}", TILE_WRITE, k, elems)
    del x, y
    res.update(tile_launch_lengths())
    return res


def tile_launch_lengths():
    """The FP8 tile kernel on every 2-D weight of Qwen3-4B as one job list, with the driver's cut of long runs of tile
    jobs set to different lengths (mq_tune_tile_launch_tiles; 0: no cut, up to 64 tensors per launch)."""
    import ctypes

    from miles_amd import _lib
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast

    gen = torch.Generator(device=DEV)
    gen.manual_seed(1234)
    _, weights, _ = qwen3_4b_megatron_weights(gen)
    targets = [t for name, t in weights.items() if t.dim() == 2 and "embedding" not in name and "output_layer" not in name]
    elems = sum(t.numel() for t in targets)
    batch, outs = _record(lambda: [fp8_blockwise_cast(t) for t in targets])
    res = {}
    lib, compiled_in = _lib.load(), ctypes.c_int64(0)
    _lib.check(lib.mq_tune_tile_launch_tiles(0, ctypes.byref(compiled_in)))
    try:
        for cap in (0, 98304, 49152, 36864, 24576, 16384, 8192, 4096):
            _lib.check(lib.mq_tune_tile_launch_tiles(cap, None))
            for _ in range(3):
                batch.run()
            ms = _best_ms(batch.run)
            res[f"qwen3_4b_fp8_cast_launches_of_{cap}_tiles"] = {"GBps": round(elems * BYTES_PER_ELEM["fp8_block"] / ms / 1e6, 1),
                                                                 "ms": round(ms, 4)}
    finally:
        _lib.check(lib.mq_tune_tile_launch_tiles(compiled_in.value, None))
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-extras", action="store_true", help="skip the per-quantizer section")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-workload", action="store_true",
                    help="counter-collection run: three 1 GiB plain copies (calibration), three syncs, no timing")
    ap.add_argument("--pmc-quantizers", action="store_true",
                    help="counter-collection run: three 1 GiB plain copies (calibration), then every workload of the "
                         "per-quantizer section exactly twice, no timing")
    ap.add_argument("--stream-ceilings", action="store_true",
                    help="only torch's fill / copy / cast kernels on 4 GiB operands: what plain streaming reaches here (one JSON line)")
    ap.add_argument("--full-configs", action="store_true",
                    help="only the three MoE configurations at full size, each as one whole sync (one JSON line; the "
                         "default run includes them under per_quantizer)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no cross-GPU part (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs the MI355X: no GPU visible")
    from miles_amd import _lib, _probes
    from miles_amd.weight_update.updater import WeightUpdater

    _lib.load()   # fails loudly if the HIP library is not built
    gen = torch.Generator(device=DEV)
    gen.manual_seed(2001)
    if a.stream_ceilings:
        print(json.dumps({"stream_ceilings": stream_ceilings()}))
        return
    if a.full_configs:
        print(json.dumps({"full_configs": full_configs(gen)}))
        return
    if a.pmc_quantizers:
        global TIMED_ITERS
        TIMED_ITERS = 1
        n = 1 << 30
        src, dst = torch.empty(n, dtype=torch.uint8, device=DEV), torch.empty(n, dtype=torch.uint8, device=DEV)
        src.fill_(1)
        for _ in range(3):
            _probes.check(_probes.load().mqp_copy_bytes(src.data_ptr(), dst.data_ptr(), n, _lib.stream_ptr(torch.device(DEV))))
        del src, dst
        res = per_quantizer(gen)
        print(json.dumps({"pmc_quantizers": "3 x mqp_copy_bytes(1 GiB), then each workload twice",
                          "elements": {k: v["elements"] for k, v in res.items()}}))
        return
    args, weights, elems = qwen3_4b_megatron_weights(gen)
    fp8_cfg = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}
    sent = {"buckets": 0, "bytes": 0}

    def consume(bucket):
        sent["buckets"] += 1
        sent["bytes"] += sum(t.nbytes for _n, t in bucket)

    updater = WeightUpdater(args, weights_getter=lambda: weights, model_name="qwen3", quantization_config=fp8_cfg,
                            send_bucket=consume)
    torch.cuda.synchronize()
    plan_bytes = torch.cuda.memory_allocated()
    updater.update_weights()          # builds the plan (first sync pays the per-parameter Python work)
    torch.cuda.synchronize()
    plan_bytes = torch.cuda.memory_allocated() - plan_bytes      # device memory the sync's outputs occupy from now on
    if a.pmc_workload:
        n = 1 << 30
        src, dst = torch.empty(n, dtype=torch.uint8, device=DEV), torch.empty(n, dtype=torch.uint8, device=DEV)
        src.fill_(1)
        for _ in range(3):
            _probes.check(_probes.load().mqp_copy_bytes(src.data_ptr(), dst.data_ptr(), n, _lib.stream_ptr(torch.device(DEV))))
        for _ in range(2):
            updater.update_weights()
        torch.cuda.synchronize()
        print(json.dumps({"pmc_workload": "3 x mqp_copy_bytes(1 GiB), 3 x Qwen3-4B FP8 sync", "quantized_elements": elems}))
        return
    # bring the GPU out of its idle power state first: the first ~20 syncs after start-up run about 5 % slower than
    # the steady state however many warm-up steps are requested (untimed, like the warm-up steps that follow)
    t_spin = time.perf_counter()
    while time.perf_counter() - t_spin < 0.2:
        updater.update_weights()
        torch.cuda.synchronize()
    for _ in range(a.warmup):
        updater.update_weights()
    torch.cuda.synchronize()
    sent.update(buckets=0, bytes=0)
    # the timed region: K syncs between two wall-clock reads, and inside them between two events on the launch stream
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(a.steps):
        updater.update_weights()
    e1.record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    gpu_ms = e0.elapsed_time(e1)
    ms_per_step = dt / a.steps * 1e3
    algorithmic_bytes = elems * BYTES_PER_ELEM["fp8_block"]
    value = algorithmic_bytes / (dt / a.steps) / 1e9

    plan = updater._plan
    assert plan is not None and plan.replayable, "the benchmark expects the replayable plan path"
    assert all(rec[0] == _lib.JOB_FP8_BLOCKWISE_CAST for rec in plan.batch.records), "the headline sync runs one kernel only"
    line = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "io_dtypes": "bf16 in -> float8_e4m3fn codes + fp32 tile scales out (arithmetic in fp32)",
        "data": "synthetic",
        "config": {"workload": "configs[1]: full Qwen3-4B weight sync to FP8 e4m3 128x128 block scales, 36 layers "
                               "(q[4096,2560] k/v[1024,2560] o[2560,4096] gate/up[9728,2560] down[2560,9728]), bf16 "
                               "N(0,0.02) + 0.1% x20 outliers, embeddings and norms passed through as bf16",
                   "quantizer": "fp8_blockwise_cast (sync path)", "quantized_elements": elems,
                   "algorithmic_bytes": round(algorithmic_bytes), "buckets_per_sync": sent["buckets"] // max(a.steps, 1),
                   "bucket_bytes": args.update_weight_buffer_size, "gpus": "one GPU; no second GPU is used or measured"},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "roofline": roofline(plan, elems, a.steps, gpu_ms),
        "sync_output_bytes_resident": plan_bytes,
        "parity": parity_whole_sync(weights, args, updater),
    }
    if not a.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(weights, args)
    if not a.no_extras:
        del updater, plan
        line["packed_payload"] = packed_payload(args, weights, fp8_cfg, min(a.steps, 20))
        c2_block_fp8 = full_model_block_fp8(weights, elems)
        weights.clear()
        line["per_quantizer"] = {"C2_block_fp8": c2_block_fp8, **per_quantizer(gen), **full_configs(gen)}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
