"""End-to-end sync driver on the GPU: Megatron-named parameters -> WeightUpdater -> buckets of quantized HF
tensors, compared tensor by tensor with the oracle applied to the HF tensors the name maps produce."""

import os
from argparse import Namespace

import pytest
import torch

from miles_amd import _lib
from miles_amd import workloads as W
from miles_amd.megatron_to_hf import name_maps
from miles_amd.weight_update.updater import WeightUpdater
from tests.sync_expectations import reference_stream_order

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn

_SCALE = max(1, int(os.environ.get("MQ_RANDOM_SCALE", "1")))     # multiplies the seeded random model cases
ARGS = Namespace(hidden_size=256, num_attention_heads=4, num_query_groups=2, kv_channels=128, vocab_size=1000,
                 num_layers=2, update_weight_buffer_size=1 << 20, q_lora_rank=None)
FP8_CFG = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}


def _bits(t):
    t = t.detach().cpu().contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()])


def _same(got, want, what):
    g, w = _bits(got), _bits(want)
    assert g.shape == w.shape, f"{what}: shape {tuple(g.shape)} vs {tuple(w.shape)}"
    assert torch.equal(g, w), f"{what}: {(g != w).sum().item()} of {g.numel()} differ"


def _ordered(params):
    """(name, parameter) pairs in the order the reference streams a model: by name, routed experts last."""
    return [(n, params[n]) for n in reference_stream_order(params)]


def _dense_model(seed):
    """Megatron-named bf16 parameters of a 2-layer Qwen3-style dense model (CPU)."""
    p, k = {}, 0

    def rnd(shape):
        nonlocal k
        k += 1
        return W.gaussian_outliers(shape, std=0.02, p_outlier=0.001, gain=20.0, seed=seed + k)

    p["module.module.embedding.word_embeddings.weight"] = rnd((1024, 256))     # padded vocab
    for layer in range(2):
        L = f"module.module.decoder.layers.{layer}."
        p[L + "self_attention.linear_qkv.layer_norm_weight"] = rnd((256,))
        p[L + "self_attention.linear_qkv.weight"] = rnd((2 * (2 + 1 + 1) * 128, 256))
        p[L + "self_attention.q_layernorm.weight"] = rnd((128,))
        p[L + "self_attention.k_layernorm.weight"] = rnd((128,))
        p[L + "self_attention.linear_proj.weight"] = rnd((256, 512))
        p[L + "mlp.linear_fc1.layer_norm_weight"] = rnd((256,))
        p[L + "mlp.linear_fc1.weight"] = rnd((2 * 384, 256))
        p[L + "mlp.linear_fc2.weight"] = rnd((256, 384))
    p["module.module.decoder.final_layernorm.weight"] = rnd((256,))
    p["module.module.output_layer.weight"] = rnd((1024, 256))
    return p


def _expected_fp8(oracle, cpu_params):
    """(name, tensor) list the sync must produce: HF order of the name map, weights cast per tile."""
    out = []
    for name, param in _ordered(cpu_params):
        if "word_embeddings" in name or "output_layer" in name:
            param = param[:1000]
        for hf, t in name_maps.convert_qwen2_to_hf(ARGS, name, param):
            quantized = hf.endswith("_proj.weight")
            if quantized:
                q, s = oracle.fp8_blockwise_cast(t.contiguous())
                out += [(hf, q), (hf.replace(".weight", ".weight_scale_inv"), s)]
            else:
                out.append((hf, t))
    return out


def _snapshot(bucket):
    """What a consumer must do to keep a bucket past its own send: copy it (the sync reuses the memory for a later
    bucket).  A packed bucket is copied as one payload."""
    from miles_amd.weight_update.packed_bucket import PackedBucket

    if isinstance(bucket, PackedBucket):
        return PackedBucket(bucket.flat.clone(), bucket.metadata)
    return [(n, t.clone()) for n, t in bucket]


def _run(updater):
    got = []
    updater.send_bucket = lambda bucket: got.append(_snapshot(bucket))
    updater.update_weights()
    torch.cuda.synchronize()
    return got


@pytest.mark.parametrize("use_plan", [True, False])
def test_dense_fp8_sync_matches_oracle_and_replays(oracle, use_plan):
    cpu = _dense_model(10)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="qwen3", quantization_config=FP8_CFG,
                        send_bucket=None, use_plan=use_plan)
    buckets = _run(upd)
    flat = [nt for b in buckets for nt in b]
    want = _expected_fp8(oracle, cpu)
    assert [n for n, _ in flat] == [n for n, _ in want]
    for (n, g), (_, w) in zip(flat, want):
        _same(g, w, n)
    assert len(buckets) > 1
    for b in buckets[:-1]:      # a closed bucket stays under the limit unless it is a single oversized unit
        assert sum(t.nbytes for _, t in b) < ARGS.update_weight_buffer_size or len(b) <= 3
    metrics = upd.pop_metrics()
    assert set(metrics) == {"update_weights_implementation"} and upd.pop_metrics() == {}     # no finalize hook, no such span
    finalized = []
    upd.finalize = lambda version: (torch.cuda.synchronize(), finalized.append(version))
    _run(upd)
    metrics = upd.pop_metrics()
    assert finalized == [upd.weight_version] and metrics["finalize_and_resume_engines"] > 0 and metrics["update_weights_implementation"] > 0
    upd.finalize = None
    q_proj = dict(flat)["model.layers.0.self_attn.q_proj.weight"]
    assert q_proj.dtype == F8 and q_proj.shape == (512, 256)
    # the weights change in place (an optimizer step); the next sync must see the new values
    cpu2 = _dense_model(500)
    for k in dev:
        dev[k].copy_(cpu2[k])
    plan = upd._plan
    buckets2 = _run(upd)
    if use_plan:
        assert upd._plan is plan and plan is not None and plan.replayable      # the same plan, replayed
    want2 = _expected_fp8(oracle, cpu2)
    for (n, g), (_, w) in zip([nt for b in buckets2 for nt in b], want2):
        _same(g, w, n + " (second sync)")
    # a different parameter set (new storage) invalidates the plan
    dev3 = {k: v.clone() for k, v in dev.items()}
    upd.weights_getter = lambda: dev3
    buckets3 = _run(upd)
    for (n, g), (_, w) in zip([nt for b in buckets3 for nt in b], want2):
        _same(g, w, n + " (new storage)")


def _family_model(family, seed):
    """The dense model above renamed for another family: Llama has no q/k norms and names the second norm
    `pre_mlp_layernorm`; GLM-4 adds a norm after attention and after the MLP and a bias on the fused q/k/v."""
    p = _dense_model(seed)
    for layer in range(2):
        L = f"module.module.decoder.layers.{layer}."
        if family == "llama":
            del p[L + "self_attention.q_layernorm.weight"], p[L + "self_attention.k_layernorm.weight"]
            p[L + "pre_mlp_layernorm.weight"] = p.pop(L + "mlp.linear_fc1.layer_norm_weight")
        else:
            p[L + "self_attention.linear_qkv.bias"] = W.gaussian_outliers((1024,), std=0.02, p_outlier=0.0, gain=1.0, seed=seed + 90 + layer)
            p[L + "post_self_attn_layernorm.weight"] = W.gaussian_outliers((256,), std=0.02, p_outlier=0.0, gain=1.0, seed=seed + 70 + layer)
            p[L + "post_mlp_layernorm.weight"] = W.gaussian_outliers((256,), std=0.02, p_outlier=0.0, gain=1.0, seed=seed + 80 + layer)
    return p


def _family_expected(oracle, family, cpu):
    """HF names written out by hand (megatron_to_hf/llama.py:6-44, glm4.py:6-60), weights of *_proj cast per tile."""
    out = []

    def emit(name, t):
        if name.endswith("_proj.weight"):
            q, s = oracle.fp8_blockwise_cast(t.contiguous())
            out.extend([(name, q), (name.replace(".weight", ".weight_scale_inv"), s)])
        else:
            out.append((name, t))

    def qkv(t):
        g = t.view(2, 4, 128, *t.shape[1:])
        return g[:, :2].reshape(512, *t.shape[1:]), g[:, 2].reshape(256, *t.shape[1:]), g[:, 3].reshape(256, *t.shape[1:])

    for name, t in _ordered(cpu):
        if "decoder.layers." not in name:
            hf = {"embedding.word_embeddings.weight": "model.embed_tokens.weight", "output_layer.weight": "lm_head.weight",
                  "decoder.final_layernorm.weight": "model.norm.weight"}[name[len("module.module."):]]
            emit(hf, t[:1000] if t.dim() == 2 else t)
            continue
        layer, rest = name[len("module.module.decoder.layers."):].split(".", 1)
        H = f"model.layers.{layer}."
        if rest in ("self_attention.linear_qkv.weight", "self_attention.linear_qkv.bias"):
            for proj, part in zip("qkv", qkv(t)):
                emit(f"{H}self_attn.{proj}_proj.{rest.rsplit('.', 1)[1]}", part)
        elif rest == "mlp.linear_fc1.weight" and family == "llama":
            emit(H + "mlp.gate_proj.weight", t[:384])
            emit(H + "mlp.up_proj.weight", t[384:])
        else:
            emit(H + {"mlp.linear_fc1.weight": "mlp.gate_up_proj.weight", "mlp.linear_fc2.weight": "mlp.down_proj.weight",
                      "self_attention.linear_proj.weight": "self_attn.o_proj.weight",
                      "self_attention.linear_qkv.layer_norm_weight": "input_layernorm.weight",
                      "mlp.linear_fc1.layer_norm_weight": "post_attention_layernorm.weight",
                      "pre_mlp_layernorm.weight": "post_attention_layernorm.weight",
                      "self_attention.q_layernorm.weight": "self_attn.q_norm.weight",
                      "self_attention.k_layernorm.weight": "self_attn.k_norm.weight",
                      "post_self_attn_layernorm.weight": "post_self_attn_layernorm.weight",
                      "post_mlp_layernorm.weight": "post_mlp_layernorm.weight"}[rest], t)
    return out


@pytest.mark.parametrize("family,model_name", [("llama", "Llama-3.1-8B"), ("glm4", "glm4")])
def test_llama_and_glm4_fp8_sync_and_replay(oracle, family, model_name):
    cpu = _family_model(family, 40)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name=model_name, quantization_config=FP8_CFG, send_bucket=None)
    for sync, seed in enumerate((40, 41, 42)):
        if sync:
            cpu = _family_model(family, seed)
            for k in dev:
                dev[k].copy_(cpu[k])
        flat = [nt for b in _run(upd) for nt in b]
        want = _family_expected(oracle, family, cpu)
        assert [n for n, _ in flat] == [n for n, _ in want]
        for (n, g), (_, w) in zip(flat, want):
            _same(g, w, f"{family} sync {sync}: {n}")
    assert upd._plan is not None and upd._plan.replayable


def test_modules_to_not_convert_keep_bf16_and_2d_shape(oracle):
    cpu = _dense_model(20)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    cfg = dict(FP8_CFG, modules_to_not_convert=["model.layers.1.self_attn.k_proj"])
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="qwen3", quantization_config=cfg, send_bucket=None)
    flat = dict(nt for b in _run(upd) for nt in b)
    k1 = flat["model.layers.1.self_attn.k_proj.weight"]
    assert k1.dtype == torch.bfloat16 and k1.shape == (256, 256)
    assert "model.layers.1.self_attn.k_proj.weight_scale_inv" not in flat
    want = dict(name_maps.convert_qwen2_to_hf(ARGS, "module.module.decoder.layers.1.self_attention.linear_qkv.weight",
                                              cpu["module.module.decoder.layers.1.self_attention.linear_qkv.weight"]))
    _same(k1, want["model.layers.1.self_attn.k_proj.weight"], "unquantized k_proj")
    assert flat["model.layers.1.self_attn.q_proj.weight"].dtype == F8
    # the regrouped bf16 k_proj is produced by copy jobs: the plan is replayed and hands out current values
    assert upd._plan is not None and upd._plan.replayable
    cpu2 = _dense_model(21)
    for k in dev:
        dev[k].copy_(cpu2[k])
    flat = dict(nt for b in _run(upd) for nt in b)
    want = dict(name_maps.convert_qwen2_to_hf(ARGS, "module.module.decoder.layers.1.self_attention.linear_qkv.weight",
                                              cpu2["module.module.decoder.layers.1.self_attention.linear_qkv.weight"]))
    _same(flat["model.layers.1.self_attn.k_proj.weight"], want["model.layers.1.self_attn.k_proj.weight"], "k_proj after a step")


def _moe_model(seed, experts=4, ffn=128, hidden=256):
    p, k = {}, 0
    for layer in range(2):
        L = f"module.module.decoder.layers.{layer}."
        p[L + "mlp.router.weight"] = W.gaussian_outliers((experts, hidden), std=0.02, p_outlier=0, gain=1, seed=seed + 900 + layer)
        for e in range(experts):
            k += 1
            p[L + f"mlp.experts.linear_fc1.weight{e}"] = W.student_t_rows((2 * ffn, hidden), std=0.02, seed=seed + 2 * k)
            p[L + f"mlp.experts.linear_fc2.weight{e}"] = W.student_t_rows((hidden, ffn), std=0.02, seed=seed + 2 * k + 1)
    return p


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_moe_mxfp8_sync(oracle, dtype):
    cpu = {k: v.to(dtype) for k, v in _moe_model(30).items()}
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="qwen3moe", quantization_config={"quant_method": "mxfp8"},
                        send_bucket=None)
    for round_ in range(2):
        flat = [nt for b in _run(upd) for nt in b]
        want = []
        for name, param in _ordered(cpu):
            for hf, t in name_maps.convert_qwen3moe_to_hf(ARGS, name, param):
                if "experts" in hf:
                    q, s = oracle.mxfp8_quantize(t.contiguous())
                    want += [(hf, q), (hf.replace(".weight", ".weight_scale_inv"), s)]
                else:
                    want.append((hf, t))
        assert [n for n, _ in flat] == [n for n, _ in want]
        for (n, g), (_, w) in zip(flat, want):
            _same(g, w, f"{n} sync {round_}")
        cpu = {k: v.to(dtype) for k, v in _moe_model(31).items()}
        for k in dev:
            dev[k].copy_(cpu[k])


def test_moe_nvfp4_sync_pairs_share_amax(oracle):
    cpu = _moe_model(40)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="deepseekv3",
                        quantization_config={"quant_method": "modelopt", "quant_algo": "NVFP4"}, send_bucket=None)
    # sync 0 records the plan (amax pass + quantize pass); later syncs replay it with the amax carried over: sync 1 on
    # new weights (every amax moved), sync 2 on the same weights (none moved), sync 3 with one expert's amax moved
    changed = _moe_model(41)
    one_moved = {k: v.clone() for k, v in changed.items()}
    moved_name = next(k for k in one_moved if "linear_fc1" in k)
    one_moved[moved_name].mul_(2.0)
    syncs = [cpu, changed, changed, one_moved]
    for sync_, cpu in enumerate(syncs):
        for k in dev:
            dev[k].copy_(cpu[k])
        flat = [nt for b in _run(upd) for nt in b]
        want = []
        for name, param in _ordered(cpu):
            hf = name_maps.convert_deepseekv3_to_hf(ARGS, name, param)
            if "linear_fc1" in name:
                (gn, g), (un, u) = hf
                for n, (q, s, gl) in zip((gn, un), oracle.nvfp4_quantize_1d_pair(g.contiguous(), u.contiguous())):
                    want += [(n, q), (n.replace(".weight", ".weight_scale"), s), (n.replace(".weight", ".weight_scale_2"), gl)]
            elif "linear_fc2" in name:
                n, t = hf[0]
                q, s, gl = oracle.nvfp4_quantize_1d(t)
                want += [(n, q), (n.replace(".weight", ".weight_scale"), s), (n.replace(".weight", ".weight_scale_2"), gl)]
            else:
                want += hf
        assert [n for n, _ in flat] == [n for n, _ in want]
        for (n, g), (_, w) in zip(flat, want):
            _same(g, w, f"{n} sync {sync_}")
    assert upd._plan.replayable
    assert any(r[upd._plan.batch.P1] & 8 for r in upd._plan.batch.records), "replays should carry the amax over"


def test_moe_int4_compressed_tensors_sync(oracle):
    cpu = _moe_model(50)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    cfg = {"quant_method": "compressed-tensors", "format": "pack-quantized",
           "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": True, "num_bits": 4, "type": "int"}}}}
    basenames = {f"model.layers.{l}.mlp.experts.{e}.{p}_proj" for l in range(2) for e in range(4) for p in ("gate", "up", "down")}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="kimi_k2", quantization_config=cfg, send_bucket=None,
                        packed_weight_basenames=basenames)
    flat = [nt for b in _run(upd) for nt in b]
    want = []
    for name, param in _ordered(cpu):
        for hf, t in name_maps.convert_deepseekv3_to_hf(ARGS, name, param):
            if hf.removesuffix(".weight") in basenames:
                packed, scale, _ = oracle.pack_layer(t.contiguous(), 128)
                want += [(hf.replace(".weight", ".weight_packed"), packed), (hf.replace(".weight", ".weight_scale"), scale),
                         (hf.replace(".weight", ".weight_shape"), torch.tensor(t.shape, dtype=torch.int32))]
            else:
                want.append((hf, t))
    assert [n for n, _ in flat] == [n for n, _ in want]
    for (n, g), (_, w) in zip(flat, want):
        _same(g, w, n)


@pytest.mark.parametrize("packed", [False, True])
def test_moe_int4_asymmetric_sync_is_planned_and_replayed(oracle, packed):
    # symmetric: False adds zero points (quantizer_compressed_tensors.py:286-301); the asymmetric packer is a job too
    cfg = {"quant_method": "compressed-tensors", "format": "pack-quantized",
           "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": False, "num_bits": 4, "type": "int"}}}}
    basenames = {f"model.layers.{l}.mlp.experts.{e}.{p}_proj" for l in range(2) for e in range(4) for p in ("gate", "up", "down")}
    cpu = _moe_model(55)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="kimi_k2", quantization_config=cfg, send_bucket=None,
                        packed_weight_basenames=basenames, packed_buckets=packed)
    for round_ in range(3):
        flat = [nt for b in _run(upd) for nt in b]
        want = []
        for name, param in _ordered(cpu):
            for hf, t in name_maps.convert_deepseekv3_to_hf(ARGS, name, param):
                if hf.removesuffix(".weight") in basenames:
                    p_, s_, z_ = oracle.pack_layer(t.contiguous(), 128, sym=False)
                    want += [(hf.replace(".weight", ".weight_zero_point"), z_),      # the reference's order (:296-301)
                             (hf.replace(".weight", ".weight_packed"), p_), (hf.replace(".weight", ".weight_scale"), s_),
                             (hf.replace(".weight", ".weight_shape"), torch.tensor(t.shape, dtype=torch.int32))]
                else:
                    want.append((hf, t))
        assert [n for n, _ in flat] == [n for n, _ in want]
        for (n, g), (_, w) in zip(flat, want):
            _same(g, w, f"{n} sync {round_}")
        cpu = _moe_model(56 + round_)
        for k in dev:
            dev[k].copy_(cpu[k])
    assert upd._plan is not None and upd._plan.replayable


# ---------------------------------------------------------------------------------------------------
# packed transport buckets: quantizers write straight into the flat payload
def _payload_bytes(named):
    return torch.cat([_bits(t).reshape(-1).view(torch.uint8) for _, t in named]) if named else torch.empty(0, dtype=torch.uint8)


def test_packed_buckets_fp8_plan_writes_payload_in_place(oracle):
    from miles_amd.weight_update.packed_bucket import PackedBucket

    cpu = _dense_model(10)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    # plan_arenas=None: every bucket keeps an arena of its own, so all of them can be looked at after the sync
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="qwen3", quantization_config=FP8_CFG,
                        send_bucket=None, packed_buckets=True, plan_arenas=None)
    got = []
    upd.send_bucket = got.append
    upd.update_weights()
    torch.cuda.synchronize()
    assert len(got) > 1 and all(isinstance(b, PackedBucket) for b in got)
    want = _expected_fp8(oracle, cpu)
    flat_names = [n for b in got for n, _ in b]
    assert flat_names == [n for n, _ in want]
    it = iter(want)
    for b in got:
        expect = [next(it) for _ in b]
        for (n, g), (_, w) in zip(b, expect):
            _same(g, w, n)
        # the payload is the byte-for-byte concatenation of the bucket's tensors, described by the metadata
        assert torch.equal(b.get_flattened_tensor().cpu(), _payload_bytes(expect))
        off = 0
        for m, (n, w) in zip(b.get_metadata(), expect):
            assert (m.name, tuple(m.shape), m.dtype, m.start_idx, m.numel) == (n, tuple(w.shape), w.dtype, off, w.numel())
            off = m.end_idx
        assert off == b.flat.numel()
        for _, t in b:      # every tensor is a view of the payload
            assert b.flat.data_ptr() <= t.data_ptr() < b.flat.data_ptr() + max(b.flat.numel(), 1)
    assert upd._plan is not None and upd._plan.replayable
    # quantizer outputs live in the payloads; the only ones outside are codes whose slot is not 16-byte aligned (it
    # follows a scale grid of odd size), and those reach the payload through a copy job
    payload = {(b.flat.data_ptr(), b.flat.data_ptr() + b.flat.numel()) for b in got}
    copied_from = {rec[2] for rec in upd._plan.batch.records if rec[0] == _lib.JOB_COPY}
    outputs = upd._plan.batch.output_pointers()
    outside = [ptr for ptr in outputs if not any(lo <= ptr < hi for lo, hi in payload)]
    assert all(ptr in copied_from for ptr in outside) and len(outside) < len(outputs) / 2
    # optimizer step, replay: same payload buffers, new contents
    cpu2 = _dense_model(500)
    for k in dev:
        dev[k].copy_(cpu2[k])
    first = [b.flat.data_ptr() for b in got]
    got.clear()
    upd.update_weights()
    torch.cuda.synchronize()
    assert [b.flat.data_ptr() for b in got] == first
    it = iter(_expected_fp8(oracle, cpu2))
    for b in got:
        expect = [next(it) for _ in b]
        assert torch.equal(b.flat.cpu(), _payload_bytes(expect))


def test_packed_buckets_without_plan_and_layout_errors(oracle):
    from miles_amd.weight_update.packed_bucket import PackedBucket, pack_bucket

    cpu = _dense_model(30)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="qwen3", quantization_config=FP8_CFG,
                        send_bucket=None, use_plan=False, packed_buckets=True)
    got = []
    upd.send_bucket = lambda b: got.append(_snapshot(b))
    upd.update_weights()
    torch.cuda.synchronize()
    it = iter(_expected_fp8(oracle, cpu))
    for b in got:
        assert isinstance(b, PackedBucket)
        assert torch.equal(b.flat.cpu(), _payload_bytes([next(it) for _ in b]))
    # ragged sizes and unaligned pointers go through the byte path of the grouped copy
    g = torch.Generator().manual_seed(3)
    odd = [("a", torch.randint(0, 255, (1003,), dtype=torch.uint8, generator=g).to(DEV)[3:]),
           ("b", torch.randint(0, 255, (40000,), dtype=torch.uint8, generator=g).to(DEV)),
           ("c", torch.randn(0, device=DEV)),
           ("d", torch.randint(0, 255, (17,), dtype=torch.uint8, generator=g).to(DEV))]
    packed = pack_bucket(odd)
    torch.cuda.synchronize()
    assert torch.equal(packed.flat.cpu(), _payload_bytes(odd))
    # the reference's layout rule (protocols/broadcast.py:201-205)
    with pytest.raises(ValueError, match="Unaligned flattened weight scale: byte offset 3"):
        pack_bucket([("w", torch.zeros(3, dtype=torch.uint8, device=DEV)), ("scale", torch.zeros(2, device=DEV))])


def _mixed_bucket():
    """The tensor mix of the reference's wire-format test (tests/fast/backends/training_utils/weight_update/
    test_broadcast_packed.py:41-50): transposed and strided views, an e4m3 vector, a 0-dim scalar, an empty tensor."""
    return [("expert.weight", torch.arange(16, dtype=torch.uint8).reshape(2, 8).T),
            ("expert.weight_scale", torch.tensor([0, 128, 126, 255], dtype=torch.uint8).view(torch.float8_e4m3fn)),
            ("expert.weight_scale_2", torch.tensor(-0.0, dtype=torch.float32)),
            ("dense.weight", torch.arange(8, dtype=torch.bfloat16).reshape(2, 4).T),
            ("strided_bf16.weight", torch.arange(8, dtype=torch.bfloat16)[::2]),
            ("strided_fp32.weight", torch.arange(8, dtype=torch.float32)[::2]),
            ("empty", torch.empty((0, 2), dtype=torch.float32))]


def test_pack_bucket_keeps_mixed_dtype_bytes_scalar_shapes_and_strided_views():
    from miles_amd.weight_update.packed_bucket import pack_bucket

    cpu = _mixed_bucket()
    packed = pack_bucket([(n, t.to(DEV)) for n, t in cpu])
    torch.cuda.synchronize()
    assert [n for n, _ in packed] == [n for n, _ in cpu]
    for (_, want), (_, got), meta in zip(cpu, packed, packed.get_metadata()):
        assert got.shape == want.shape and got.dtype == want.dtype and got.is_contiguous()
        assert meta.numel == want.numel() and meta.end_idx - meta.start_idx == want.numel() * want.element_size()
        assert torch.equal(got.cpu().flatten().view(torch.uint8), want.contiguous().flatten().view(torch.uint8))
    assert torch.equal(packed.get_flattened_tensor().cpu(), _payload_bytes(cpu))
    assert [t.shape for _, t in packed.reconstruct_tensors()] == [t.shape for _, t in cpu]


def test_packed_sync_of_a_model_with_strided_pass_through_tensors_falls_back_to_flattening(monkeypatch):
    # a strided view cannot be byte-copied into a payload slot by a job: the plan is refused once and every sync flattens
    # its buckets after the fact, still current after the weights change in place
    from miles_amd.weight_update.packed_bucket import PackedBucket

    base = torch.arange(64, dtype=torch.bfloat16, device=DEV).reshape(8, 8)
    weights = {"w": base}
    upd = WeightUpdater(ARGS, weights_getter=lambda: weights, model_name="qwen3", quantization_config=None, send_bucket=None,
                        packed_buckets=True)
    calls = []

    def fake_iter(ws):
        calls.append(1)
        yield [("a.weight", ws["w"].t()), ("b.weight", ws["w"][:, ::2]), ("c.weight", ws["w"])]

    monkeypatch.setattr(upd._iterator, "iter_hf_weights", fake_iter)
    for step in range(3):
        got = []
        upd.send_bucket = lambda b: got.append(_snapshot(b))
        upd.update_weights()
        torch.cuda.synchronize()
        assert len(got) == 1 and isinstance(got[0], PackedBucket)
        want = [("a.weight", base.t().cpu()), ("b.weight", base[:, ::2].cpu()), ("c.weight", base.cpu())]
        assert torch.equal(got[0].flat.cpu(), _payload_bytes(want)), f"sync {step}"
        base.add_(1)
    assert upd._plan is None and len(calls) == 4       # recorded once (refused), then one pass per sync


def test_copy_jobs_that_depend_on_each_other_run_in_order():
    # one submission: a -> b, b -> c, then c -> a shifted by 16 bytes (overlapping its own source's neighbour); copy jobs of
    # one launch run in no order, so the driver has to cut the launches at each dependency
    from miles_amd import launch
    from miles_amd.weight_update.packed_bucket import submit_copy

    g = torch.Generator().manual_seed(77)
    a = torch.randint(0, 255, (4096,), dtype=torch.uint8, generator=g).to(DEV)
    b, c = torch.zeros_like(a), torch.zeros_like(a)
    before = a.cpu().clone()
    with launch.deferred() as batch:
        submit_copy(a, b)
        submit_copy(b, c)
        submit_copy(c[:4080], a[16:])
        assert len(batch) == 3
    torch.cuda.synchronize()
    assert torch.equal(b.cpu(), before) and torch.equal(c.cpu(), before)
    assert torch.equal(a.cpu()[16:], before[:4080]) and torch.equal(a.cpu()[:16], before[:16])


def test_unquantized_sync_hands_out_current_regrouped_qkv():
    # without quantization q / k / v are regrouped copies of the fused attention weight: the copies are jobs of the plan,
    # so a replay refreshes them (a tensor a torch op had materialised would hand out last step's values)
    cpu = _dense_model(40)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    for packed in (False, True):
        upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="qwen3", quantization_config=None,
                            send_bucket=None, packed_buckets=packed)
        _run(upd)
        cpu2 = _dense_model(600 + packed)
        for k in dev:
            dev[k].copy_(cpu2[k])
        flat = dict(nt for b in _run(upd) for nt in b)
        want = dict(name_maps.convert_qwen2_to_hf(ARGS, "module.module.decoder.layers.1.self_attention.linear_qkv.weight",
                                                  cpu2["module.module.decoder.layers.1.self_attention.linear_qkv.weight"]))
        for n, w in want.items():
            _same(flat[n], w, n)
        assert upd._plan is not None and upd._plan.replayable
        if packed:      # q / k / v are assembled in their payload slots: 6 gathering 2-D copies, 19 pass-through copies, none twice
            assert len(upd._plan.batch) == 25


def test_packed_buckets_int4_moe_two_syncs(oracle):
    cfg = {"quant_method": "compressed-tensors", "format": "pack-quantized",
           "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": True, "num_bits": 4, "type": "int"}}}}
    basenames = {f"model.layers.{l}.mlp.experts.{e}.{p}_proj" for l in range(2) for e in range(4) for p in ("gate", "up", "down")}
    cpu = _moe_model(50)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="kimi_k2", quantization_config=cfg, send_bucket=None,
                        packed_weight_basenames=basenames, packed_buckets=True)
    for seed in (50, 700):
        src = _moe_model(seed)
        for k in dev:
            dev[k].copy_(src[k])
        got = []
        upd.send_bucket = lambda b: got.append(_snapshot(b))
        upd.update_weights()
        torch.cuda.synchronize()
        want = []
        for name, param in _ordered(src):
            for hf, t in name_maps.convert_deepseekv3_to_hf(ARGS, name, param):
                if hf.removesuffix(".weight") in basenames:
                    p, s, _ = oracle.pack_layer(t.contiguous(), 128)
                    want += [(hf.replace(".weight", ".weight_packed"), p), (hf.replace(".weight", ".weight_scale"), s),
                             (hf.replace(".weight", ".weight_shape"), torch.tensor(t.shape, dtype=torch.int32))]
                else:
                    want.append((hf, t))
        it = iter(want)
        for b in got:
            expect = [next(it) for _ in b]
            assert [n for n, _ in b] == [n for n, _ in expect]
            assert torch.equal(b.flat.cpu(), _payload_bytes(expect)), f"payload of a bucket differs (seed {seed})"


def test_dense_fp8_sync_with_power_of_two_scales(oracle, monkeypatch):
    # NVTE_FP8_BLOCK_SCALING_FP32_SCALES=0 routes the block cast through per_block_cast_to_fp8 (quantizer_fp8.py:139-147)
    monkeypatch.setenv("NVTE_FP8_BLOCK_SCALING_FP32_SCALES", "0")
    cpu = _dense_model(60)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="qwen3", quantization_config=FP8_CFG, send_bucket=None)
    for _ in range(2):      # recorded plan, then its replay
        flat = dict(nt for b in _run(upd) for nt in b)
        for name, param in _ordered(cpu):
            for hf, t in name_maps.convert_qwen2_to_hf(ARGS, name, param):
                if hf.endswith("_proj.weight"):
                    q, s = oracle.per_block_cast_to_fp8(t.contiguous())
                    _same(flat[hf], q, hf)
                    _same(flat[hf.replace(".weight", ".weight_scale_inv")], s, hf + " scale")
    assert upd._plan is not None and upd._plan.replayable


@pytest.mark.parametrize("packed", [False, True])
def test_dense_fp8_sync_with_one_scale_per_tensor(oracle, packed):
    # no weight_block_size in the config: the per-tensor branch (quantizer_fp8.py:153-158), scale name `.weight_scale`.
    # Every quantizer call is a job of the batched driver and q / k / v are regrouped by copy jobs, so the sync is planned
    # and replayed, from the second replay on with the amax carried over
    cfg = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic"}
    cpu = _dense_model(62)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="qwen3", quantization_config=cfg, send_bucket=None,
                        packed_buckets=packed)
    for round_ in range(4):
        flat = [nt for b in _run(upd) for nt in b]
        want = []
        for name, param in _ordered(cpu):
            if "word_embeddings" in name or "output_layer" in name:
                param = param[:1000]
            for hf, t in name_maps.convert_qwen2_to_hf(ARGS, name, param):
                if hf.endswith("_proj.weight"):
                    q, sc = oracle.tensor_fp8(t.contiguous())
                    want += [(hf, q), (hf.replace(".weight", ".weight_scale"), sc)]
                else:
                    want.append((hf, t))
        assert [n for n, _ in flat] == [n for n, _ in want]
        for (n, g), (_, w) in zip(flat, want):
            _same(g, w, f"{n} sync {round_}")
        if round_ != 1:             # rounds 1 and 2 see the same weights: no amax moves between them
            cpu = _dense_model(63 + round_)
            for k in dev:
                dev[k].copy_(cpu[k])
    assert upd._plan is not None and upd._plan.replayable
    assert any(r[upd._plan.batch.KIND] == 10 and r[upd._plan.batch.P1] & 8 for r in upd._plan.batch.records)


@pytest.mark.parametrize("packed", [False, True])
def test_dense_fp8_sync_with_packed_ue8m0_scales(oracle, packed):
    # DeepGEMM requantization (quantizer_fp8.py:140-142): power-of-two tile scales, then four exponent bytes per int32
    # in a row-contiguous layout; the packer consumes the scales of a job recorded just before it
    import copy
    args = copy.copy(ARGS)
    args.deepgemm_weight_requant_ue8m0 = True
    cpu = _dense_model(61)
    for name in list(cpu):      # an MLP width of 640 gives down_proj five tile columns: two words per row, a strided view
        if name.endswith("mlp.linear_fc1.weight"):
            cpu[name] = W.gaussian_outliers((2 * 640, 256), std=0.02, p_outlier=0.001, gain=20.0, seed=611)
        elif name.endswith("mlp.linear_fc2.weight"):
            cpu[name] = W.gaussian_outliers((256, 640), std=0.02, p_outlier=0.001, gain=20.0, seed=612)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(args, weights_getter=lambda: dev, model_name="qwen3", quantization_config=FP8_CFG, send_bucket=None,
                        packed_buckets=packed)
    for _ in range(3):      # recorded plan, then two replays
        flat = dict(nt for b in _run(upd) for nt in b)
        for name, param in _ordered(cpu):
            for hf, t in name_maps.convert_qwen2_to_hf(args, name, param):
                if hf.endswith("_proj.weight"):
                    q, s = oracle.per_block_cast_to_fp8(t.contiguous())
                    want = oracle.transform_scale_ue8m0(s, t.shape[0])
                    got = flat[hf.replace(".weight", ".weight_scale_inv")]
                    _same(flat[hf], q, hf)
                    assert got.dtype == torch.int32 and got.shape == want.shape, hf
                    assert torch.equal(got.cpu(), want), hf + " packed scale"
                    assert got.is_contiguous() if packed else got.stride() == want.stride(), hf
    assert upd._plan is not None and upd._plan.replayable


# ---------------------------------------------------------------------------------------------------------------------
# randomly shaped dense models through the whole driver (seeded; shapes the fixed models above do not reach: head
# sizes that rule the in-place q/k/v views out, hidden sizes off the 128 grid, buffer sizes that cut anywhere)
def _random_dense_case(seed):
    import random
    from argparse import Namespace

    rng = random.Random(f"miles-driver-{seed}")
    head = rng.choice([64, 128])
    groups = rng.choice([1, 2, 4])
    q_per_group = rng.choice([1, 2, 4])
    hidden = rng.choice([128, 192, 256, 320])
    ffn = 8 * rng.randint(8, 60)
    layers = rng.randint(1, 3)
    vocab = rng.choice([257, 512, 1000])
    args = Namespace(hidden_size=hidden, num_attention_heads=groups * q_per_group, num_query_groups=groups, kv_channels=head,
                     vocab_size=vocab, num_layers=layers, update_weight_buffer_size=rng.choice([1 << 16, 1 << 18, 1 << 20, 1 << 24]),
                     q_lora_rank=None)
    p, k = {}, 0

    def rnd(shape):
        nonlocal k
        k += 1
        return W.gaussian_outliers(shape, std=0.02, p_outlier=0.002, gain=20.0, seed=9000 + 100 * seed + k)

    p["module.module.embedding.word_embeddings.weight"] = rnd((vocab, hidden))
    for layer in range(layers):
        L = f"module.module.decoder.layers.{layer}."
        p[L + "self_attention.linear_qkv.layer_norm_weight"] = rnd((hidden,))
        p[L + "self_attention.linear_qkv.weight"] = rnd((groups * (q_per_group + 2) * head, hidden))
        p[L + "self_attention.linear_proj.weight"] = rnd((hidden, groups * q_per_group * head))
        p[L + "mlp.linear_fc1.layer_norm_weight"] = rnd((hidden,))
        p[L + "mlp.linear_fc1.weight"] = rnd((2 * ffn, hidden))
        p[L + "mlp.linear_fc2.weight"] = rnd((hidden, ffn))
    p["module.module.decoder.final_layernorm.weight"] = rnd((hidden,))
    return args, p


@pytest.mark.parametrize("seed", range(10 * _SCALE))
@pytest.mark.parametrize("packed", [False, True])
def test_random_dense_models_sync_and_replay(oracle, seed, packed):
    args, cpu = _random_dense_case(seed)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(args, weights_getter=lambda: dev, model_name="qwen3", quantization_config=FP8_CFG, send_bucket=None,
                        packed_buckets=packed)

    def expected(params):
        out = []
        for name, param in _ordered(params):
            for hf, t in name_maps.convert_qwen2_to_hf(args, name, param):
                if hf.endswith("_proj.weight"):
                    q, s = oracle.fp8_blockwise_cast(t.contiguous())
                    out += [(hf, q), (hf.replace(".weight", ".weight_scale_inv"), s)]
                else:
                    out.append((hf, t))
        return out

    for round_ in range(3):                       # recording sync, then two replays with changed weights in between
        buckets = []
        upd.send_bucket = lambda b: buckets.append(_snapshot(b))
        upd.update_weights()
        torch.cuda.synchronize()
        flat = [nt for b in buckets for nt in b]
        want = expected(cpu)
        assert [n for n, _ in flat] == [n for n, _ in want]
        for (n, g), (_, w) in zip(flat, want):
            _same(g, w, f"{n} (sync {round_})")
        if packed:
            for b in buckets:
                rebuilt = torch.cat([t.contiguous().view(torch.uint8).reshape(-1) for _, t in b]) if len(b) else b.flat
                assert torch.equal(b.flat, rebuilt)
        _, cpu = _random_dense_case(seed + 1000 * (round_ + 1))
        if set(cpu) != set(dev) or any(cpu[k].shape != dev[k].shape for k in cpu):
            break                                   # the follow-up case happens to have other shapes: nothing to copy into
        for k in dev:
            dev[k].copy_(cpu[k])


# ---------------------------------------------------------------------------------------------------------------------
# randomly shaped MoE layers through the driver, in the three expert formats
def _random_moe_case(seed):
    import random
    from argparse import Namespace

    rng = random.Random(f"miles-moe-{seed}")
    experts = rng.choice([1, 2, 3, 8])
    hidden = 128 * rng.randint(1, 3)
    ffn = 128 * rng.randint(1, 3)
    layers = rng.randint(1, 2)
    args = Namespace(hidden_size=hidden, num_attention_heads=4, num_query_groups=2, kv_channels=64, vocab_size=1000, num_layers=layers,
                     update_weight_buffer_size=rng.choice([1 << 16, 1 << 19, 1 << 22]), q_lora_rank=None)
    p, k = {}, 0
    for layer in range(layers):
        L = f"module.module.decoder.layers.{layer}."
        p[L + "mlp.router.weight"] = W.gaussian_outliers((experts, hidden), std=0.02, p_outlier=0, gain=1, seed=7000 + 10 * seed + layer)
        for e in range(experts):
            k += 1
            p[L + f"mlp.experts.linear_fc1.weight{e}"] = W.student_t_rows((2 * ffn, hidden), std=0.02, seed=7100 + 100 * seed + 2 * k)
            p[L + f"mlp.experts.linear_fc2.weight{e}"] = W.student_t_rows((hidden, ffn), std=0.02, seed=7101 + 100 * seed + 2 * k)
    return args, p, experts, layers


def _moe_expected(oracle, fmt, args, params, basenames):
    want = []
    for name, param in _ordered(params):
        if fmt == "mxfp8":
            for hf, t in name_maps.convert_qwen3moe_to_hf(args, name, param):
                if "experts" in hf:
                    q, s = oracle.mxfp8_quantize(t.contiguous())
                    want += [(hf, q), (hf.replace(".weight", ".weight_scale_inv"), s)]
                else:
                    want.append((hf, t))
            continue
        hf = name_maps.convert_deepseekv3_to_hf(args, name, param)
        if fmt == "nvfp4" and "linear_fc1" in name:
            (gn, g), (un, u) = hf
            for n, (q, s, gl) in zip((gn, un), oracle.nvfp4_quantize_1d_pair(g.contiguous(), u.contiguous())):
                want += [(n, q), (n.replace(".weight", ".weight_scale"), s), (n.replace(".weight", ".weight_scale_2"), gl)]
        elif fmt == "nvfp4" and "linear_fc2" in name:
            n, t = hf[0]
            q, s, gl = oracle.nvfp4_quantize_1d(t)
            want += [(n, q), (n.replace(".weight", ".weight_scale"), s), (n.replace(".weight", ".weight_scale_2"), gl)]
        elif fmt == "int4":
            for n, t in hf:
                if n.removesuffix(".weight") in basenames:
                    packed, scale, _ = oracle.pack_layer(t.contiguous(), 128)
                    want += [(n.replace(".weight", ".weight_packed"), packed), (n.replace(".weight", ".weight_scale"), scale),
                             (n.replace(".weight", ".weight_shape"), torch.tensor(t.shape, dtype=torch.int32))]
                else:
                    want.append((n, t))
        else:
            want += hf
    return want


@pytest.mark.parametrize("seed", range(6 * _SCALE))
@pytest.mark.parametrize("fmt", ["mxfp8", "nvfp4", "int4"])
@pytest.mark.parametrize("packed", [False, True])
def test_random_moe_models_sync_and_replay(oracle, seed, fmt, packed):
    args, cpu, experts, layers = _random_moe_case(seed)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    basenames = {f"model.layers.{l}.mlp.experts.{e}.{p}_proj" for l in range(layers) for e in range(experts) for p in ("gate", "up", "down")}
    model, cfg, extra = {
        "mxfp8": ("qwen3moe", {"quant_method": "mxfp8"}, {}),
        "nvfp4": ("deepseekv3", {"quant_method": "modelopt", "quant_algo": "NVFP4"}, {}),
        "int4": ("kimi_k2", {"quant_method": "compressed-tensors", "format": "pack-quantized",
                             "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": True, "num_bits": 4, "type": "int"}}}},
                 {"packed_weight_basenames": basenames}),
    }[fmt]
    upd = WeightUpdater(args, weights_getter=lambda: dev, model_name=model, quantization_config=cfg, send_bucket=None,
                        packed_buckets=packed, **extra)
    for round_ in range(3):
        buckets = []
        upd.send_bucket = lambda b: buckets.append(_snapshot(b))
        upd.update_weights()
        torch.cuda.synchronize()
        flat = [nt for b in buckets for nt in b]
        want = _moe_expected(oracle, fmt, args, cpu, basenames)
        assert [n for n, _ in flat] == [n for n, _ in want]
        for (n, g), (_, w) in zip(flat, want):
            _same(g, w, f"{n} (sync {round_})")
        if packed:
            for b in buckets:
                assert torch.equal(b.flat.cpu(), _payload_bytes(list(b)))
        cpu = {k: W.student_t_rows(tuple(v.shape), std=0.03, seed=8000 + 37 * seed + round_ * 1000 + i) if v.dim() == 2 and "router" not in k else v
               for i, (k, v) in enumerate(cpu.items())}
        for k in dev:
            dev[k].copy_(cpu[k])
    assert upd._plan is not None and upd._plan.replayable


def test_dsa_indexer_half_rotation_is_replayable():
    # DeepSeek's DSA indexer with rope interleave swaps the two 64-channel halves of each 128-wide head: copy jobs on the
    # GPU (the torch concatenation of the CPU path would hand out stale values on replay)
    from argparse import Namespace

    from miles_amd import launch

    args = Namespace(**vars(ARGS), indexer_rope_interleave=True)
    g = torch.Generator().manual_seed(91)
    cpu = {"self_attention.wq_b.weight": torch.randn(4 * 128, 96, generator=g).to(torch.bfloat16),
           "self_attention.wk.weight": torch.randn(128, 256, generator=g).to(torch.bfloat16),
           "self_attention.k_norm.weight": torch.randn(128, generator=g).to(torch.bfloat16),
           "self_attention.k_norm.bias": torch.randn(128, generator=g).to(torch.bfloat16)}
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    name = "module.module.decoder.layers.0."
    with launch.recording() as batch:
        got = {k: name_maps.convert_deepseekv3_to_hf(args, name + k, v) for k, v in dev.items()}
    assert batch.direct_calls == 0 and len(batch) == 4 * 2         # each rotation: one 2-D copy job per half
    batch.device = torch.device(DEV)
    for round_ in range(2):
        batch.run()
        torch.cuda.synchronize()
        for k, v in cpu.items():
            (want_name, want), = name_maps.convert_deepseekv3_to_hf(args, name + k, v)      # torch path on the CPU
            (got_name, got_t), = got[k]
            assert got_name == want_name
            _same(got_t, want, f"{k} round {round_}")
        for k in cpu:
            cpu[k] = (cpu[k].float() * 1.5 + 0.25).to(torch.bfloat16)
            dev[k].copy_(cpu[k])


def test_mimo_mtp_sync_swaps_projection_halves_and_replays(oracle):
    # MiMo = the dense map + MTP layers under model.mtp_layers.<i>; the MTP input projection swaps its column halves
    # (megatron_to_hf/mimo.py:41-43), as copy jobs on the GPU so that a replayed sync sees the current weights
    def model(seed):
        p = _dense_model(seed)
        M = "module.module.mtp.layers.0."
        g = torch.Generator().manual_seed(seed)
        p[M + "enorm.weight"] = torch.randn(256, generator=g).to(torch.bfloat16)
        p[M + "hnorm.weight"] = torch.randn(256, generator=g).to(torch.bfloat16)
        p[M + "eh_proj.weight"] = (torch.randn(256, 512, generator=g) * 0.02).to(torch.bfloat16)
        p[M + "transformer_layer.mlp.linear_fc2.weight"] = (torch.randn(256, 384, generator=g) * 0.02).to(torch.bfloat16)
        p[M + "final_layernorm.weight"] = torch.randn(256, generator=g).to(torch.bfloat16)
        return p

    cpu = model(60)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="mimo", quantization_config=FP8_CFG, send_bucket=None)
    for sync, seed in enumerate((60, 61, 62)):
        if sync:
            cpu = model(seed)
            for k in dev:
                dev[k].copy_(cpu[k])
        got = dict(nt for b in _run(upd) for nt in b)
        M = "module.module.mtp.layers.0."
        eh = cpu[M + "eh_proj.weight"]
        # eh_proj is not among the linears the FP8 processor quantizes (quantizer_fp8.py:84-103): bf16, halves swapped
        _same(got["model.mtp_layers.0.input_proj.weight"], torch.cat([eh[:, 256:], eh[:, :256]], dim=1), f"input_proj sync {sync}")
        assert "model.mtp_layers.0.input_proj.weight_scale_inv" not in got
        q, s = oracle.fp8_blockwise_cast(cpu[M + "transformer_layer.mlp.linear_fc2.weight"])
        _same(got["model.mtp_layers.0.mlp.down_proj.weight"], q, f"mtp down_proj sync {sync}")
        _same(got["model.mtp_layers.0.mlp.down_proj.weight_scale_inv"], s, f"mtp down_proj scales sync {sync}")
        for mg, hf in (("enorm", "token_layernorm"), ("hnorm", "hidden_layernorm"), ("final_layernorm", "final_layernorm")):
            _same(got[f"model.mtp_layers.0.{hf}.weight"], cpu[M + mg + ".weight"], f"{hf} sync {sync}")
        want_dense = _expected_fp8(oracle, {k: v for k, v in cpu.items() if ".mtp." not in k})
        for n, w in want_dense:
            _same(got[n], w, f"{n} sync {sync}")
    assert upd._plan is not None and upd._plan.replayable


def test_quantize_nvfp4_on_a_stack_inside_a_batch_and_replayed(oracle):
    """A 3-D weight (a stack of expert matrices) quantized inside a deferred batch: the stacked outputs are written by
    the jobs, so they hold the results once the batch has run, and a recorded batch re-run after an in-place weight
    change produces the new results at the same addresses."""
    from miles_amd import launch
    from miles_amd.megatron_to_hf.processors.quantizer_nvfp4 import quantize_nvfp4

    def expected(cpu):
        per = [oracle.nvfp4_quantize_1d(cpu[i].contiguous()) for i in range(cpu.shape[0])]
        return tuple(torch.stack(f) for f in zip(*per))

    cpu = torch.stack([W.gaussian_outliers((64, 128), std=0.02 * (i + 1), p_outlier=0.01, gain=20.0, seed=300 + i)
                       for i in range(3)])
    dev = cpu.to(DEV)
    with launch.deferred():
        got = quantize_nvfp4(dev)
    torch.cuda.synchronize()
    for g, w, what in zip(got, expected(cpu), ("codes", "block scales", "global scales")):
        _same(g, w, f"deferred stack {what}")
    with launch.recording() as batch:
        got = quantize_nvfp4(dev)
    batch.device = torch.device(DEV)
    batch.run()
    cpu2 = torch.stack([W.gaussian_outliers((64, 128), std=0.05, p_outlier=0.0, gain=1.0, seed=400 + i) for i in range(3)])
    dev.copy_(cpu2)
    batch.run()
    torch.cuda.synchronize()
    for g, w, what in zip(got, expected(cpu2), ("codes", "block scales", "global scales")):
        _same(g, w, f"replayed stack {what}")


def test_plan_outputs_rotate_through_two_arenas(oracle):
    """A recorded sync holds two buckets' worth of output memory, whatever the number of buckets: bucket k lives in arena
    k mod 2.  A consumer that queues its reads of bucket k on the launch stream (no host synchronisation) gets the right
    bytes although bucket k + 2 overwrites the same memory later in the same sync."""
    cpu = _dense_model(60)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    args = Namespace(**{**vars(ARGS), "update_weight_buffer_size": 1 << 18})        # small buckets: six or more of them
    upd = WeightUpdater(args, weights_getter=lambda: dev, model_name="qwen3", quantization_config=FP8_CFG, send_bucket=None)
    seen, copies = [], []

    def consume(bucket):
        # address range of the job-written tensors of this bucket, and stream-ordered copies of everything in it
        made = [t for n, t in bucket if t.dtype in (F8, torch.float32)]
        if made:      # a bucket of pass-through tensors only (the embedding) hands out views of the parameters
            seen.append((len(copies), min(t.data_ptr() for t in made), max(t.data_ptr() + t.nbytes for t in made),
                         sum(t.nbytes for t in made)))
        copies.append([(n, t.clone()) for n, t in bucket])

    for round_ in range(2):
        seen.clear(), copies.clear()
        upd.send_bucket = consume
        upd.update_weights()
        torch.cuda.synchronize()
        flat = [nt for b in copies for nt in b]
        want = _expected_fp8(oracle, cpu)
        assert [n for n, _ in flat] == [n for n, _ in want]
        for (n, g), (_, w) in zip(flat, want):
            _same(g, w, f"{n} (sync {round_})")
        cpu = _dense_model(61)
        for k in dev:
            dev[k].copy_(cpu[k])
    plan = upd._plan
    assert plan is not None and plan.replayable and plan.ring == 2 and len(seen) >= 4
    largest = max(nbytes for _, _, _, nbytes in seen)
    assert plan.arena_bytes <= 2 * (largest + 256 * 64), "two arenas of the largest bucket (plus alignment padding)"
    assert torch.cuda.memory_allocated() - before - sum(t.nbytes for b in copies for _, t in b) <= plan.arena_bytes + (1 << 20)
    starts = {}
    for k, lo, hi, _ in seen:                  # buckets of the same parity share an arena, neighbours never overlap
        assert starts.setdefault(k % 2, lo) == lo
    for (k, lo, hi, _), (k2, lo2, hi2, _) in zip(seen, seen[1:]):
        if k2 == k + 1:
            assert hi <= lo2 or hi2 <= lo
    assert len(starts) == 2
    # an arena per bucket on request: every bucket of the sync stays valid until the next sync
    keep = WeightUpdater(args, weights_getter=lambda: dev, model_name="qwen3", quantization_config=FP8_CFG, send_bucket=None,
                         plan_arenas=None)
    held = []
    keep.send_bucket = held.append
    keep.update_weights()
    torch.cuda.synchronize()
    for (n, g), (_, w) in zip([nt for b in held for nt in b], _expected_fp8(oracle, cpu)):
        _same(g, w, f"{n} (an arena per bucket)")
    assert keep._plan.ring == len(held)


@pytest.mark.parametrize("hand_back", ["host_wait", "stream_wait"])
def test_a_consumer_on_another_stream_reads_the_right_bytes(oracle, hand_back):
    """What a transfer protocol on its own stream (a broadcast, say) must do with a bucket of a two-arena plan: make its
    stream wait for the launch stream before it reads, and before `send_bucket` returns either wait on the host for its
    stream or make the launch stream wait for it -- bucket k + 2 is written into the memory of bucket k.  The consumer
    here is slow on purpose (it sleeps on its stream before every copy), over six or more buckets and two syncs."""
    cpu = _dense_model(70)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    args = Namespace(**{**vars(ARGS), "update_weight_buffer_size": 1 << 18})
    upd = WeightUpdater(args, weights_getter=lambda: dev, model_name="qwen3", quantization_config=FP8_CFG, send_bucket=None)
    side = torch.cuda.Stream(device=DEV)
    copies = []

    def consume(bucket):
        launch_stream = torch.cuda.current_stream()
        side.wait_stream(launch_stream)                  # the bucket's kernels are queued on the launch stream
        with torch.cuda.stream(side):
            torch.cuda._sleep(2_000_000)                 # about a millisecond: the reads run well after this call returns
            copies.append([(n, t.clone()) for n, t in bucket])
        if hand_back == "host_wait":
            side.synchronize()
        else:
            launch_stream.wait_stream(side)              # nothing queued later on the launch stream overtakes the reads

    for round_ in range(2):
        copies.clear()
        upd.send_bucket = consume
        upd.update_weights()
        torch.cuda.synchronize()
        assert len(copies) >= 6
        flat = [nt for b in copies for nt in b]
        want = _expected_fp8(oracle, cpu)
        assert [n for n, _ in flat] == [n for n, _ in want]
        for (n, g), (_, w) in zip(flat, want):
            _same(g, w, f"{n} (sync {round_}, {hand_back})")
        cpu = _dense_model(71)
        for k in dev:
            dev[k].copy_(cpu[k])
    assert upd._plan is not None and upd._plan.replayable and upd._plan.ring == 2


def test_recording_a_sync_holds_no_more_than_a_few_buckets():
    """While a sync is recorded nothing is executed and every bucket's first output buffers are released as soon as the
    bucket has its place in an arena: the peak stays near the arenas' size instead of the size of all outputs."""
    from miles_amd import workloads as Wl

    gen = torch.Generator(device=DEV)
    gen.manual_seed(9)
    args, weights, elems = Wl.moe_megatron(gen, layers=1, experts=48, ffn=2048, hidden=7168, dist="gaussian_0.02",
                                           buffer_bytes=64 << 20)
    conf = Wl.MOE_CONFIGS["C4"]
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    upd = WeightUpdater(args, weights_getter=lambda: weights, model_name=conf["model_name"], quantization_config=conf["cfg"],
                        send_bucket=lambda b: None, packed_weight_basenames=Wl.int4_packed_basenames(1, 48))
    upd.update_weights()
    torch.cuda.synchronize()
    outputs = elems * (0.5 + 2 / 128)              # packed words + bf16 scales of the whole model
    plan = upd._plan
    assert plan is not None and plan.replayable and len(plan.buckets) >= 8
    assert plan.arena_bytes <= 2 * (64 << 20) + (4 << 20)
    peak = torch.cuda.max_memory_allocated() - base
    assert peak <= plan.arena_bytes + 3 * (64 << 20), f"recording peaked at {peak} bytes for {outputs:.0f} bytes of outputs"
    assert outputs > 5 * plan.arena_bytes


@pytest.mark.parametrize("fmt", ["mxfp8", "mxfp4", "int4", "int4_asym", "fp8", "block_fp8", "mxfp8_f16", "fp8_f16"])
def test_launches_with_a_device_table_cover_hundreds_of_tensors(oracle, fmt):
    """More than MQ_MAX_GROUP jobs of a table kind: the batch copies their descriptors to device memory and one launch
    covers the lot.  Shapes vary inside the 25 % band that keeps a group together, with a few far outside it (which
    cut the group), an FP8 tile job in the middle, and the list is also submitted in two ranges that start mid-table."""
    from miles_amd import launch
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast
    from miles_amd.megatron_to_hf.processors.quantizer_compressed_tensors import pack_layer
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8
    from miles_amd.utils.mxfp4 import quantize_mxfp4
    from miles_amd.utils.mxfp8 import mxfp8_quantize

    # (the two kernels with fp16 instances also run the list with every third tensor in fp16: launches split by dtype)
    mixed_dtypes = fmt.endswith("_f16")
    fmt = fmt.removesuffix("_f16")
    g = torch.Generator().manual_seed(77)
    shapes = [(int(torch.randint(52, 64, (1,), generator=g)), 256) for _ in range(150)]
    shapes[40], shapes[41], shapes[120] = (8, 128), (300, 256), (1, 128)
    if fmt == "int4_asym":          # packed zero points take eight rows to a word
        shapes = [((r + 7) // 8 * 8, k) for r, k in shapes]
    if fmt in ("fp8", "block_fp8"):  # 128x128 tiles: two row tiles by three column tiles, the last of each partial
        shapes = [(130 + (r * 7 + i) % 120, 264 + 8 * (i % 3)) for i, (r, k) in enumerate(shapes)]
        shapes[40], shapes[41], shapes[120], shapes[130] = (8, 128), (1300, 256), (1, 8), (256, 384)
    ws = [W.student_t_rows(s, std=0.02, seed=7700 + i) for i, s in enumerate(shapes)]
    if mixed_dtypes:        # runs of fp16 tensors long enough for a table launch of their own, and single ones
        ws = [w.to(torch.float16) if (i % 3 == 0 or 80 <= i < 150) else w for i, w in enumerate(ws)]
    dev = [w.to(DEV) for w in ws]
    tile_w = W.gaussian_outliers((256, 384), std=0.02, p_outlier=0.001, gain=20.0, seed=7)

    def quantize(w):
        if fmt == "fp8":
            return fp8_blockwise_cast(w)
        if fmt == "block_fp8":
            return block_fp8(w, [128, 128])
        if fmt == "mxfp8":
            return mxfp8_quantize(w)
        if fmt == "mxfp4":
            return quantize_mxfp4(w, 32)
        return pack_layer(w, 128, sym=fmt == "int4")[:3 if fmt == "int4_asym" else 2]

    def expected(w):
        if fmt == "fp8":
            return oracle.fp8_blockwise_cast(w)
        if fmt == "block_fp8":
            return oracle.block_fp8(w, (128, 128))
        if fmt == "mxfp8":
            return oracle.mxfp8_quantize(w)
        if fmt == "mxfp4":
            return oracle.quantize_mxfp4(w, 32)
        return oracle.pack_layer(w, 128, sym=fmt == "int4")[:3 if fmt == "int4_asym" else 2]

    with launch.recording() as batch:
        outs = [quantize(w) for w in dev[:75]]
        tile_out = fp8_blockwise_cast(tile_w.to(DEV))
        outs += [quantize(w) for w in dev[75:]]
    batch.freeze()
    assert batch._table is not None and batch._table.numel() == len(batch) * _lib.TABLE_ENTRY_BYTES

    def check(what):
        torch.cuda.synchronize()
        for i, (w, out) in enumerate(zip(ws, outs)):
            for k, (got, want) in enumerate(zip(out, expected(w))):
                _same(got, want, f"{fmt} tensor {i} {tuple(w.shape)} output {k} ({what})")
        for got, want in zip(tile_out, oracle.fp8_blockwise_cast(tile_w)):
            _same(got, want, f"fp8 tile job between the {fmt} jobs ({what})")

    def poison():
        for out in (*outs, tile_out):
            for t in out:
                t.view(torch.uint8).fill_(0x5A)

    batch.run()
    check("one submission")
    poison()
    batch.run_range(0, 70)
    batch.run_range(70, len(batch))
    check("two ranges")
    # the same list through the kernel-argument form
    poison()
    batch._table = None
    batch.run()
    check("without the table")


@pytest.mark.parametrize("form", ["searched", "table"])
def test_long_runs_of_tile_jobs_are_cut_into_launches_of_equal_size(oracle, form):
    """A run of FP8 tile jobs of more than 36 864 tiles goes out as several launches (the tile kernel streams faster in
    launches of moderate length).  Both launch forms: 44 tensors of 896 tiles (descriptors in the kernel arguments,
    cut in two) and 420 tensors of 96 tiles (device table, cut in two); every output against the oracle, also on the
    replay and when the list is submitted in two ranges that start mid-run."""
    from miles_amd import launch
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8

    if form == "searched":
        shapes, quantize, expected = [(2048, 7168)] * 44, lambda w: block_fp8(w, [128, 128]), lambda w: oracle.block_fp8(w, (128, 128))
    else:
        shapes = [(768, 2048) if i % 3 else (2048, 768) for i in range(420)]
        quantize, expected = fp8_blockwise_cast, oracle.fp8_blockwise_cast
    assert sum(-(-r // 128) * -(-c // 128) for r, c in shapes) > 36864
    ws = [W.gaussian_outliers(s, std=0.02, p_outlier=0.001, gain=20.0, seed=9100 + i) for i, s in enumerate(shapes)]
    dev = [w.to(DEV) for w in ws]
    with launch.recording() as batch:
        outs = [quantize(w) for w in dev]
    batch.freeze()
    assert (batch._table is not None) == (form == "table")
    want = [expected(w) for w in ws]
    half = len(batch) // 2 + 3
    for what, run in (("one submission", batch.run), ("replay", batch.run),
                      ("two ranges", lambda: (batch.run_range(0, half), batch.run_range(half, len(batch))))):
        for out in outs:
            for t in out:
                t.view(torch.uint8).fill_(0x5A)
        run()
        torch.cuda.synchronize()
        for i, (out, exp) in enumerate(zip(outs, want)):
            for k, (got, w_) in enumerate(zip(out, exp)):
                _same(got, w_, f"tensor {i} output {k} ({what})")


@pytest.mark.parametrize("odd", ["offset", "fp32", "fp16"])
def test_fused_qkv_that_the_tuned_kernel_cannot_read_in_place_is_regrouped(oracle, odd):
    """Row-blocked q / k / v views are switched on per model, by shape.  A fused qkv parameter that starts two bytes into
    a flat buffer, or a model held in fp32, is outside what the tile kernel reads in place: the name map regroups it
    with copy jobs instead, and the sync stays correct and replayable.  A model held in fp16 is read in place like a
    bf16 one (the tile kernel has an fp16 instance): no copy job reads its fused qkv weights."""
    from miles_amd import _lib

    cpu = _dense_model(31)
    if odd != "offset":
        cpu = {k: v.to(torch.float16 if odd == "fp16" else torch.float32) for k, v in cpu.items()}
    dev = {}
    for k, v in cpu.items():
        if odd == "offset" and k.endswith("linear_qkv.weight"):
            flat = torch.empty(v.numel() + 1, dtype=v.dtype, device=DEV)
            dev[k] = flat[1:].view(v.shape).copy_(v)
            assert dev[k].data_ptr() % 16 == 2
        else:
            dev[k] = v.to(DEV)
    upd = WeightUpdater(ARGS, weights_getter=lambda: dev, model_name="qwen3", quantization_config=FP8_CFG,
                        send_bucket=None)
    assert upd.args.qkv_row_block_views
    for label in ("first sync", "replay"):
        flat = [nt for b in _run(upd) for nt in b]
        want = _expected_fp8(oracle, cpu)
        assert [n for n, _ in flat] == [n for n, _ in want]
        for (n, g), (_, w) in zip(flat, want):
            _same(g, w, f"{n} ({label})")
        assert upd._plan is not None and upd._plan.replayable
        cpu = {k: (v.float() * 0.5).to(v.dtype) for k, v in cpu.items()}
        for k in dev:
            dev[k].copy_(cpu[k])
    qkv = [(t.data_ptr(), t.data_ptr() + t.nbytes) for k, t in dev.items() if k.endswith("linear_qkv.weight")]
    copies_of_qkv = [rec for rec in upd._plan.batch.records
                     if rec[0] == _lib.JOB_COPY and any(lo <= rec[2] < hi for lo, hi in qkv)]
    assert (len(copies_of_qkv) == 0) == (odd == "fp16")


@pytest.mark.parametrize("rows,row_bytes,src_pitch,dst_pitch,offset", [
    (64, 8192, 16384, 8192, 0), (37, 100, 131, 257, 0), (1, 5000, 5000, 5000, 0), (9, 40000, 40016, 50000, 0),
    (16, 4096, 8192, 8192, 3), (300, 16, 48, 16, 0), (5, 16384, 16384, 32768, 0)])
def test_copy_jobs_with_row_pitches(rows, row_bytes, src_pitch, dst_pitch, offset):
    """The 2-D form of a copy job: rows of bytes at one pitch in the source and another in the destination; what lies
    between the destination rows stays untouched.  Run alone and as members of one grouped launch."""
    from miles_amd import launch
    from miles_amd.weight_update.packed_bucket import submit_copy_rows

    g = torch.Generator().manual_seed(rows * 7 + row_bytes)

    def case():
        src = torch.randint(0, 256, (rows * src_pitch + offset,), dtype=torch.uint8, generator=g).to(DEV)
        dst = torch.full((rows * dst_pitch + offset,), 0xA5, dtype=torch.uint8, device=DEV)
        sv = src[offset:].view(rows, src_pitch)[:, :row_bytes]
        dv = dst[offset:].view(rows, dst_pitch)[:, :row_bytes]
        return src, dst, sv, dv

    def check(src, dst, sv, dv, what):
        want = torch.full_like(dst, 0xA5)
        want[offset:].view(rows, dst_pitch)[:, :row_bytes] = sv
        assert torch.equal(dst, want), what

    one = case()
    submit_copy_rows(one[2], one[3])
    torch.cuda.synchronize()
    check(*one, "single job")
    many = [case() for _ in range(5)]
    with launch.deferred():
        for _, _, sv, dv in many:
            submit_copy_rows(sv, dv)
    torch.cuda.synchronize()
    for c in many:
        check(*c, "grouped jobs")


def test_a_2d_copy_that_reads_what_an_earlier_copy_wrote_runs_after_it():
    from miles_amd import launch
    from miles_amd.weight_update.packed_bucket import submit_copy, submit_copy_rows

    a = torch.arange(64 * 64, dtype=torch.int32, device=DEV).view(64, 64)
    b = torch.zeros_like(a)
    c = torch.zeros(64, 32, dtype=torch.int32, device=DEV)
    with launch.deferred():
        submit_copy(a.view(-1), b.view(-1))
        submit_copy_rows(b[:, 32:], c)                      # reads rows of b: must see what the first job wrote
    torch.cuda.synchronize()
    assert torch.equal(c, a[:, 32:])


def test_snapshot_publisher_writes_the_quantized_model(oracle, tmp_path):
    """The export entry of the weight iterator: shards on disk hold what the sync would have sent."""
    import json

    import safetensors.torch

    from miles_amd.weight_update.hf_weight_iterator import HfWeightIteratorDirect
    from miles_amd.weight_update.snapshot_publisher import SnapshotPublisher

    cpu = _dense_model(77)
    dev = {k: v.to(DEV) for k, v in cpu.items()}
    iterator = HfWeightIteratorDirect(ARGS, model_name="qwen3", quantization_config=FP8_CFG)
    SnapshotPublisher(iterator).write_model(tmp_path, weights=dev, hf_checkpoint=str(tmp_path / "absent"))
    index = json.loads((tmp_path / "model.safetensors.index.json").read_text())
    got = {}
    for shard in sorted(set(index["weight_map"].values())):
        got.update(safetensors.torch.load_file(tmp_path / shard))
    want = _expected_fp8(oracle, cpu)
    assert list(index["weight_map"]) == [n for n, _ in want]
    for n, w in want:
        _same(got[n], w, n)
    assert index["metadata"]["total_size"] == sum(t.numel() * t.element_size() for _, t in want)


def test_stream_probes_run_and_refuse_bad_arguments():
    """The measurement-only probes of libmq_probes.so: every shape runs on a small buffer, stays inside it, and refuses
    what it cannot take; the plain copy copies."""
    from miles_amd import _probes

    lib = _probes.load()
    nbytes = 3 * 128 * 1024 * 2 + 4096                   # a [384, 1024] matrix of 2-byte elements and a little more
    src = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=DEV)
    guard = 4096
    dst = torch.full((nbytes + guard,), 0xA5, dtype=torch.uint8, device=DEV)
    stream = _lib.stream_ptr(src.device)
    for shape, param in ((0, 1), (0, 2), (0, 4), (0, 8), (1, 1), (1, 2), (2, 512), (3, 1024), (4, 1024), (5, 1024), (3, 128)):
        assert lib.mqp_stream_probe(shape, src.data_ptr(), dst.data_ptr(), nbytes, param, stream) == 0, (shape, param)
    torch.cuda.synchronize()
    assert bool((dst[nbytes:] == 0xA5).all())
    for shape, param, size in ((0, 3, nbytes), (2, 100, nbytes), (3, 100, nbytes), (9, 1, nbytes), (0, 2, nbytes + 8), (3, 1 << 30, nbytes)):
        assert lib.mqp_stream_probe(shape, src.data_ptr(), dst.data_ptr(), size, param, stream) != 0, (shape, param, size)
    assert lib.mqp_stream_probe(0, None, dst.data_ptr(), nbytes, 2, stream) != 0
    assert b"aligned" in lib.mqp_last_error()
    dst.fill_(0xA5)
    assert lib.mqp_copy_bytes(src.data_ptr(), dst.data_ptr(), nbytes - nbytes % 4096, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(dst[: nbytes - nbytes % 4096], src[: nbytes - nbytes % 4096]) and bool((dst[nbytes:] == 0xA5).all())
    assert lib.mqp_copy_bytes(src.data_ptr(), dst.data_ptr(), 100, stream) != 0


def test_the_launch_cut_can_be_tuned_and_results_do_not_depend_on_it(oracle):
    """mq_tune_tile_launch_tiles sets the length at which runs of tile jobs are cut into launches and hands back the
    one it replaces; the outputs are the same bytes whatever the length."""
    import ctypes

    from miles_amd import launch
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast

    lib = _lib.load()
    ws = [W.gaussian_outliers((512, 640), std=0.02, p_outlier=0.001, gain=20.0, seed=9300 + i) for i in range(12)]
    dev = [w.to(DEV) for w in ws]
    want = [oracle.fp8_blockwise_cast(w) for w in ws]
    with launch.recording() as batch:
        outs = [fp8_blockwise_cast(w) for w in dev]
    batch.device = torch.device(DEV)
    first, previous = ctypes.c_int64(-1), ctypes.c_int64(-1)
    assert lib.mq_tune_tile_launch_tiles(50, ctypes.byref(first)) == 0 and first.value > 0       # 240 tiles in launches of 48
    try:
        for length in (50, 0, 7, 100000):
            assert lib.mq_tune_tile_launch_tiles(length, ctypes.byref(previous)) == 0
            for q, s in outs:
                q.view(torch.uint8).fill_(0x5A), s.fill_(-1.0)
            batch.run()
            torch.cuda.synchronize()
            for i, ((q, s), (wq, ws_)) in enumerate(zip(outs, want)):
                _same(q, wq, f"tensor {i} codes (launches of {length})"), _same(s, ws_, f"tensor {i} scales (launches of {length})")
        assert previous.value == 7
        assert lib.mq_tune_tile_launch_tiles(-1, None) != 0
    finally:
        assert lib.mq_tune_tile_launch_tiles(first.value, None) == 0


def test_amax_feedback_counters_through_the_c_abi():
    """mq_run_jobs_feedback with the caller's own counter words and no host mirror: tensors folded and tensors whose
    record held another amax before, summed over the calls."""
    from miles_amd import launch
    from miles_amd.tools.convert_hf_to_fp8 import tensor_fp8

    ws = [W.gaussian_outliers((64, 256), std=0.02, p_outlier=0.0, gain=1.0, seed=9700 + i).to(DEV) for i in range(5)]
    with launch.recording() as batch:
        outs = [tensor_fp8(w) for w in ws]
    arr = batch.freeze()
    lib = _lib.load()
    words = torch.zeros(2, dtype=torch.int32, device=DEV)
    stream = _lib.stream_ptr(torch.device(DEV))
    assert lib.mq_run_jobs_feedback(arr, len(batch), None, words.data_ptr(), None, stream) == 0
    assert lib.mq_run_jobs_feedback(arr, len(batch), None, words.data_ptr(), None, stream) == 0
    ws[2].mul_(2.0)
    assert lib.mq_run_jobs_feedback(arr, len(batch), None, words.data_ptr(), None, stream) == 0
    torch.cuda.synchronize()
    moved, folded = words.cpu().tolist()
    # the records start out uninitialised, so every first fold may or may not count as moved; afterwards only tensor 2
    assert folded == 15 and 1 <= moved <= 6
    assert lib.mq_run_jobs_feedback(arr, len(batch), None, words.data_ptr() + 2, None, stream) != 0      # misaligned words
    # a host mirror: pinned memory is taken (every fold launch refreshes it with the counters the launches before left),
    # anything else -- pageable host memory, device memory, a mirror without counters -- is refused before any launch
    mirror = torch.zeros(2, dtype=torch.int32).pin_memory()
    assert lib.mq_run_jobs_feedback(arr, len(batch), None, words.data_ptr(), mirror.data_ptr(), stream) == 0
    assert lib.mq_run_jobs_feedback(arr, len(batch), None, words.data_ptr(), mirror.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert mirror.tolist() == [moved, 20] and words.cpu().tolist() == [moved, 25]      # nothing moved; the mirror lags one fold launch
    pageable = torch.zeros(2, dtype=torch.int32)
    assert lib.mq_run_jobs_feedback(arr, len(batch), None, words.data_ptr(), pageable.data_ptr(), stream) != 0
    assert b"pinned" in lib.mq_last_error()
    assert lib.mq_run_jobs_feedback(arr, len(batch), None, words.data_ptr(), words.data_ptr(), stream) != 0
    assert lib.mq_run_jobs_feedback(arr, len(batch), None, None, mirror.data_ptr(), stream) != 0
    torch.cuda.synchronize()
    assert words.cpu().tolist() == [moved, 25]
    assert outs[0][0].dtype == torch.float8_e4m3fn


@pytest.mark.parametrize("fmt", ["nvfp4", "tensor_fp8"])
def test_amax_quantizers_over_a_device_table_first_run_carried_and_moved(oracle, fmt):
    """NVFP4 (pairs sharing a record and single tensors) and per-tensor FP8 with more jobs than one launch's kernel
    arguments hold: the amax pass, the fold and the quantizer read their descriptors from the device table; then the
    carried-over form on unchanged weights, and after some amaxes moved."""
    from miles_amd import launch
    from miles_amd.tools.convert_hf_to_fp8 import tensor_fp8
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d, nvfp4_quantize_1d_pair

    g = torch.Generator().manual_seed(91)
    shapes = [(int(torch.randint(52, 64, (1,), generator=g)), 256) for _ in range(120)]
    shapes[60] = (300, 256)                       # far outside the band of the others: cuts the group
    cpu = [W.gaussian_outliers(s, std=0.02, p_outlier=0.001, gain=20.0, seed=9100 + i) for i, s in enumerate(shapes)]
    pairs_cpu = [[W.gaussian_outliers((56, 256), std=0.02, p_outlier=0.001, gain=20.0, seed=9500 + 2 * i + h) for h in range(2)]
                 for i in range(30)]
    dev = [w.to(DEV) for w in cpu]
    pairs_dev = [[w.to(DEV) for w in p] for p in pairs_cpu]
    with launch.recording() as batch:
        if fmt == "nvfp4":
            outs, pair_outs = [], []
            for i, w in enumerate(dev):
                outs.append(nvfp4_quantize_1d(w))
                if i % 4 == 0:
                    pair_outs.append(nvfp4_quantize_1d_pair(*pairs_dev[i // 4]))
        else:
            outs, pair_outs = [tensor_fp8(w) for w in dev], []
    batch.freeze()
    assert batch._table is not None and len(batch) > _lib.MAX_GROUP

    def check(what):
        batch.run()
        torch.cuda.synchronize()
        for i, (w, got) in enumerate(zip(dev, outs)):
            want = oracle.nvfp4_quantize_1d(w.cpu()) if fmt == "nvfp4" else oracle.tensor_fp8(w.cpu())
            for k, (g_, w_) in enumerate(zip(got, want)):
                _same(g_, w_, f"{what}: tensor {i} output {k}")
        for i, got in enumerate(pair_outs):
            want = oracle.nvfp4_quantize_1d_pair(pairs_dev[i][0].cpu(), pairs_dev[i][1].cpu())
            for half in range(2):
                for k, (g_, w_) in enumerate(zip(got[half], want[half])):
                    _same(g_, w_, f"{what}: pair {i} half {half} output {k}")

    check("first run")
    assert batch.carry_amax() == len(batch)
    batch.freeze()
    assert batch._table is not None
    check("carried, unchanged weights")
    for i in (3, 50, 119):
        dev[i].mul_(3.0)
    if pair_outs:
        pairs_dev[7][1].mul_(0.25)
        pairs_dev[20][0].mul_(4.0)
    check("some amaxes moved")
    check("and stayed (the marked records take two passes once more)")
    check("settled")
    redo = torch.stack([r[_lib.RECORD_REDO_WORD] for r in batch.amax_records()]).cpu()
    assert int(redo.sum()) == 0
    assert batch.last_form == "carried"
    # Every amax moves on every sync: once the batch has seen that (the count of moved records comes back with the
    # sync after), it submits the plain two-pass form, and returns to the carried one when the amaxes hold still.
    factor = 2.0
    forms = []
    for step in range(5):
        for w in dev:
            w.mul_(factor)
        for pair in pairs_dev if pair_outs else []:
            pair[0].mul_(factor)
        factor = 1.0 / factor
        check(f"every amax moved, sync {step}")
        forms.append(batch.last_form)
    assert forms[0] == "carried" and forms[-1] == "plain", forms
    check("held still, reported by the plain form")
    assert batch.last_form == "plain"
    check("held still, second sync")            # the count a sync reads may lag by one sync
    check("carried again")
    assert batch.last_form == "carried"
    check("and still")
    assert batch.last_form == "carried"
