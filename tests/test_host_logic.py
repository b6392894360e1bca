"""Host-side logic of the sync path on the CPU: bucketing, gather batches, name maps and the quantizer
dispatch (with the kernels replaced by shape-only stand-ins).  The bucketing cases restate the reference's
tests/fast/backends/training_utils/weight_update/test_bucketing.py and
tests/fast/backends/megatron_utils/test_hf_weight_iterator_direct.py:109-120; the dispatch cases restate
tests/fast-gpu/test_mxfp8_quantizer.py:85-147 and tests/fast-gpu/test_nvfp4_quantizer.py:146-231."""

from argparse import Namespace

import pytest
import torch

from miles_amd.megatron_to_hf import convert_to_hf, name_maps
from miles_amd.megatron_to_hf import processors as P
from miles_amd.megatron_to_hf.processors import quantizer_fp8, quantizer_mxfp8, quantizer_nvfp4
from miles_amd.utils.mxfp8 import should_use_mxfp8
from miles_amd.weight_update.bucketing import (AtomicUpdateGroup, assemble_atomic_update_groups,
                                               get_hf_atomic_update_groups, pack_units_by_size)
from miles_amd.weight_update.hf_weight_iterator import ParamInfo, _pack_param_infos_by_size


def _unit(*names, numel=4):
    return [(name, torch.zeros(numel, dtype=torch.uint8)) for name in names]


def _names(units):
    return [[n for n, _ in u] for u in units]


PAIR = AtomicUpdateGroup("pair", (".b.weight", ".c.weight"))


class TestAtomicGroups:
    def test_ungrouped_units_stream_through(self):
        opt = AtomicUpdateGroup("pair", (".b.weight", ".c.weight"), optional=True)
        out = list(assemble_atomic_update_groups([_unit("layers.0.a.weight"), _unit("layers.1.a.weight")], [opt]))
        assert _names(out) == [["layers.0.a.weight"], ["layers.1.a.weight"]]

    def test_members_merge_in_suffix_order(self):
        units = [_unit("layers.0.a.weight"), _unit("layers.0.c.weight"), _unit("layers.0.b.weight")]
        out = list(assemble_atomic_update_groups(units, [PAIR]))
        assert _names(out) == [["layers.0.a.weight"], ["layers.0.b.weight", "layers.0.c.weight"]]

    def test_merge_is_per_prefix(self):
        units = [_unit("layers.0.b.weight"), _unit("layers.1.b.weight"), _unit("layers.1.c.weight"),
                 _unit("layers.0.c.weight")]
        out = list(assemble_atomic_update_groups(units, [PAIR]))
        assert _names(out) == [["layers.1.b.weight", "layers.1.c.weight"], ["layers.0.b.weight", "layers.0.c.weight"]]

    def test_scales_ride_with_their_weight(self):
        units = [_unit("layers.0.b.weight", "layers.0.b.weight_scale_inv"),
                 _unit("layers.0.c.weight", "layers.0.c.weight_scale_inv")]
        out = list(assemble_atomic_update_groups(units, [PAIR]))
        assert _names(out) == [["layers.0.b.weight", "layers.0.b.weight_scale_inv", "layers.0.c.weight",
                                "layers.0.c.weight_scale_inv"]]

    def test_empty_units_are_skipped(self):
        assert _names(assemble_atomic_update_groups([[], _unit("layers.0.a.weight")], [])) == [["layers.0.a.weight"]]

    @pytest.mark.parametrize("units,groups,message", [
        ([_unit("layers.0.b.weight")], [PAIR], "Incomplete atomic update groups"),
        ([_unit("layers.0.a.weight")], [PAIR], "matched no params"),
        ([_unit("layers.0.b.weight", "layers.0.c.weight")], [PAIR], "matches multiple"),
        ([], [AtomicUpdateGroup("empty", ())], "has no suffixes"),
        ([], [AtomicUpdateGroup("dup", (".a", ".a"))], "duplicate suffixes"),
        ([], [AtomicUpdateGroup("k", (".a",)), AtomicUpdateGroup("k", (".b",))], "Duplicate atomic update group keys"),
    ])
    def test_errors(self, units, groups, message):
        with pytest.raises(AssertionError, match=message):
            list(assemble_atomic_update_groups(units, groups))

    def test_optional_group_may_match_nothing(self):
        opt = AtomicUpdateGroup("pair", (".b.weight", ".c.weight"), optional=True)
        assert len(list(assemble_atomic_update_groups([_unit("layers.0.a.weight")], [opt]))) == 1

    def test_model_groups(self):
        assert get_hf_atomic_update_groups("qwen3") == []
        assert [g.key for g in get_hf_atomic_update_groups("DeepSeek-V3", q_lora_rank=1536)] == ["q_lora_a_proj"]
        assert [g.key for g in get_hf_atomic_update_groups("deepseek_v4")][0] == "wqkv_a"
        assert get_hf_atomic_update_groups("deepseekv41")[0].suffixes == (".attn.wq_a.weight", ".attn.wkv.weight")


class TestPacking:
    def test_bucket_closes_when_next_unit_would_reach_the_limit(self):
        units = [_unit("a"), _unit("b"), _unit("c")]
        assert _names(pack_units_by_size(units, max_bytes=9)) == [["a", "b"], ["c"]]
        assert _names(pack_units_by_size(units, max_bytes=8)) == [["a"], ["b"], ["c"]]   # 4 + 4 >= 8 closes

    def test_units_are_never_split(self):
        assert _names(pack_units_by_size([_unit("a"), _unit("b1", "b2")], max_bytes=6)) == [["a"], ["b1", "b2"]]

    def test_empty_stream(self):
        assert list(pack_units_by_size([], max_bytes=8)) == []

    def test_gather_batches_by_size_only(self):
        infos = [ParamInfo(n, torch.float32, torch.Size([s]), s) for n, s in [("layer.a", 4), ("layer.b", 2), ("layer.c", 4)]]
        args = Namespace(update_weight_buffer_size=6)
        assert [[i.name for i in b] for b in _pack_param_infos_by_size(args, infos)] == [["layer.a", "layer.b"], ["layer.c"]]
        assert [[i.name for i in b] for b in _pack_param_infos_by_size(args, infos, size_multiplier=2)] == \
            [["layer.a"], ["layer.b"], ["layer.c"]]

    def test_non_expert_parameters_stream_before_the_routed_experts_in_name_order(self):
        """The reference sorts the parameter infos by name and sends every non-expert gather batch before the first
        expert batch (hf_weight_iterator_direct.py:39-43, 85-108, 339-341); shared experts are not routed experts."""
        from miles_amd.weight_update.hf_weight_iterator import (HfWeightIteratorDirect, _expert_share_of_this_rank,
                                                                _split_param_infos, is_routed_expert_param)

        L = "module.module.decoder.layers."
        names = [L + "1.mlp.experts.linear_fc2.weight0", L + "0.mlp.experts.linear_fc1.weight10", L + "1.self_attention.linear_proj.weight",
                 L + "0.mlp.experts.linear_fc1.weight2", L + "0.mlp.shared_experts.experts.0.linear_fc1.weight", L + "0.mlp.router.weight",
                 "module.module.embedding.word_embeddings.weight", L + "10.mlp.router.weight", L + "2.mlp.router.weight"]
        infos = [ParamInfo(n, torch.bfloat16, torch.Size([2]), 4) for n in names]
        non_expert, expert = _split_param_infos(infos)
        assert [i.name for i in non_expert] == [
            L + "0.mlp.router.weight", L + "0.mlp.shared_experts.experts.0.linear_fc1.weight", L + "1.self_attention.linear_proj.weight",
            L + "10.mlp.router.weight", L + "2.mlp.router.weight", "module.module.embedding.word_embeddings.weight"]
        assert [i.name for i in expert] == [L + "0.mlp.experts.linear_fc1.weight10", L + "0.mlp.experts.linear_fc1.weight2",
                                            L + "1.mlp.experts.linear_fc2.weight0"]
        assert is_routed_expert_param(L + "3.mlp.experts.linear_fc1.weight7") and not is_routed_expert_param(names[4])
        assert _expert_share_of_this_rank(expert) == expert
        with pytest.raises(ValueError, match="Cannot identify the routed expert"):
            _expert_share_of_this_rank([ParamInfo(L + "0.mlp.experts.linear_fc1.bias", torch.bfloat16, torch.Size([2]), 4)])

        # the iterator walks them in that order whatever the order of the mapping, in batches of the buffer size
        seen = []

        class Spy(HfWeightIteratorDirect):
            def _convert_batch(self, named_params):
                seen.append([n for n, _ in named_params])
                return []

        it = Spy(Namespace(update_weight_buffer_size=8), model_name="qwen3moe", quantization_config=None)
        assert list(it._iter_hf_param_units({n: torch.zeros(2, dtype=torch.bfloat16) for n in names}, materialize=True)) == []
        want = [i.name for i in non_expert] + [i.name for i in expert]
        assert [n for batch in seen for n in batch] == want
        assert [len(b) for b in seen] == [2, 2, 2, 2, 1]        # six non-expert parameters, then three experts: no mixed batch


# ---------------------------------------------------------------------------------------------------------
QWEN_ARGS = Namespace(hidden_size=64, num_attention_heads=4, num_query_groups=2, kv_channels=16, vocab_size=100,
                      num_layers=4)


class TestNameMaps:
    def test_qwen2_layer(self):
        L = "module.module.decoder.layers.3."
        qkv = torch.arange((4 + 2 * 2) * 16 * 64, dtype=torch.float32).reshape(-1, 64)
        out = name_maps.convert_qwen2_to_hf(QWEN_ARGS, L + "self_attention.linear_qkv.weight", qkv)
        assert [n for n, _ in out] == [f"model.layers.3.self_attn.{p}_proj.weight" for p in "qkv"]
        q, k, v = (t for _, t in out)
        assert q.shape == (64, 64) and k.shape == (32, 64) and v.shape == (32, 64)
        grouped = qkv.view(2, 4, 16, 64)     # per group: 2 q heads, 1 k, 1 v
        assert torch.equal(q, grouped[:, :2].reshape(-1, 64)) and torch.equal(k, grouped[:, 2].reshape(-1, 64))
        assert torch.equal(v, grouped[:, 3].reshape(-1, 64))
        fc1 = torch.randn(40, 64)
        gate_up = name_maps.convert_qwen2_to_hf(QWEN_ARGS, L + "mlp.linear_fc1.weight", fc1)
        assert [n for n, _ in gate_up] == ["model.layers.3.mlp.gate_proj.weight", "model.layers.3.mlp.up_proj.weight"]
        gate, up = gate_up[0][1], gate_up[1][1]
        assert gate.data_ptr() == fc1.data_ptr() and up.data_ptr() == fc1[20:].data_ptr()   # views, not copies
        for rest, hf in [("self_attention.linear_proj.weight", "self_attn.o_proj.weight"),
                         ("mlp.linear_fc2.weight", "mlp.down_proj.weight"),
                         ("self_attention.linear_qkv.layer_norm_weight", "input_layernorm.weight"),
                         ("mlp.linear_fc1.layer_norm_weight", "post_attention_layernorm.weight"),
                         ("self_attention.q_layernorm.weight", "self_attn.q_norm.weight")]:
            assert name_maps.convert_qwen2_to_hf(QWEN_ARGS, L + rest, fc1)[0][0] == "model.layers.3." + hf
        assert name_maps.convert_qwen2_to_hf(QWEN_ARGS, "module.module.embedding.word_embeddings.weight", fc1)[0][0] \
            == "model.embed_tokens.weight"
        with pytest.raises(ValueError, match="Unknown parameter name"):
            name_maps.convert_qwen2_to_hf(QWEN_ARGS, L + "mlp.router.weight", fc1)

    def test_row_block_views_opt_in(self):
        args = Namespace(**vars(QWEN_ARGS), qkv_row_block_views=True)
        name = "module.module.decoder.layers.0.self_attention.linear_qkv.weight"
        qkv = torch.randn((4 + 2 * 2) * 16, 64).to(torch.bfloat16)
        out = name_maps.convert_qwen2_to_hf(args, name, qkv)
        ref = name_maps.convert_qwen2_to_hf(QWEN_ARGS, name, qkv)
        for (n, view), (n2, copy) in zip(out, ref):
            assert n == n2 and view.dim() == 3 and view.untyped_storage().data_ptr() == qkv.untyped_storage().data_ptr()
            assert torch.equal(view.reshape(-1, 64), copy)
        # what the tile kernel cannot read in place is regrouped as without the opt-in: another dtype, or storage that
        # starts off a 16-byte boundary
        flat = torch.empty(qkv.numel() + 1, dtype=torch.bfloat16)
        for odd in (qkv.float(), flat[1:].view(qkv.shape).copy_(qkv)):
            got = name_maps.convert_qwen2_to_hf(args, name, odd)
            for (n, t), (n2, copy) in zip(got, ref):
                assert n == n2 and t.dim() == 2 and torch.equal(t.to(torch.bfloat16), copy)

    def test_moe_experts(self):
        fc1 = torch.randn(32, 64)
        L = "module.module.decoder.layers.7."
        for fn, shared in [(name_maps.convert_qwen3moe_to_hf, "shared_expert"), (name_maps.convert_deepseekv3_to_hf, "shared_experts")]:
            out = fn(QWEN_ARGS, L + "mlp.experts.linear_fc1.weight12", fc1)
            assert [n for n, _ in out] == ["model.layers.7.mlp.experts.12.gate_proj.weight",
                                           "model.layers.7.mlp.experts.12.up_proj.weight"]
            assert fn(QWEN_ARGS, L + "mlp.experts.linear_fc2.weight3", fc1)[0][0] == "model.layers.7.mlp.experts.3.down_proj.weight"
            assert fn(QWEN_ARGS, L + "mlp.shared_experts.linear_fc2.weight", fc1)[0][0] == f"model.layers.7.mlp.{shared}.down_proj.weight"
            assert fn(QWEN_ARGS, L + "mlp.router.weight", fc1)[0][0] == "model.layers.7.mlp.gate.weight"
        out = name_maps.convert_deepseekv3_to_hf(QWEN_ARGS, L + "self_attention.linear_kv_down_proj.weight", fc1)
        assert out[0][0] == "model.layers.7.self_attn.kv_a_proj_with_mqa.weight"
        out = name_maps.convert_deepseekv3_to_hf(QWEN_ARGS, "module.module.mtp.layers.0.eh_proj.weight", fc1)
        assert out[0][0] == "model.layers.4.eh_proj.weight"
        out = name_maps.convert_deepseekv3_to_hf(QWEN_ARGS, "module.module.mtp.layers.1.transformer_layer.mlp.linear_fc2.weight", fc1)
        assert out[0][0] == "model.layers.5.mlp.down_proj.weight"

    def test_convert_to_hf_strips_vocab_padding_and_picks_family(self):
        emb = torch.randn(128, 64)
        out = convert_to_hf(QWEN_ARGS, "qwen3", "module.module.embedding.word_embeddings.weight", emb)
        assert out[0][1].shape == (100, 64)
        with pytest.raises(ValueError, match="Unsupported model"):
            convert_to_hf(QWEN_ARGS, "mystery", "module.module.embedding.word_embeddings.weight", emb)


# ---------------------------------------------------------------------------------------------------------
@pytest.fixture
def fake_kernels(monkeypatch):
    """Shape-only stand-ins for the GPU quantizers so that the dispatch logic runs on the CPU."""
    calls = []

    def fake_cast(w, block_size=None):
        calls.append(("fp8", tuple(w.shape)))
        return torch.zeros(w.shape, dtype=torch.uint8), torch.zeros(1)

    def fake_tensor(w):
        calls.append(("fp8_tensor", tuple(w.shape)))
        return torch.zeros(w.shape, dtype=torch.uint8), torch.zeros(1)

    def fake_mx(w):
        calls.append(("mxfp8", tuple(w.shape)))
        return torch.zeros(w.shape, dtype=torch.uint8), torch.zeros((*w.shape[:-1], w.shape[-1] // 32), dtype=torch.uint8)

    def nv_outputs(w):
        return torch.zeros(w.shape[0], w.shape[1] // 2, dtype=torch.uint8), torch.zeros(w.shape[0], w.shape[1] // 16), torch.ones(())

    def fake_nv(w, *, out=None):
        calls.append(("nvfp4", tuple(w.shape)))
        if out is not None:                       # a stack's matrices are written into slices of the stacked outputs
            assert [tuple(t.shape) for t in out] == [(w.shape[0], w.shape[1] // 2), (w.shape[0], w.shape[1] // 16), ()]
            out[2].fill_(1.0)
            return out
        return nv_outputs(w)

    def fake_pair(a, b):
        calls.append(("nvfp4_pair", tuple(a.shape), tuple(b.shape)))
        return nv_outputs(a), nv_outputs(b)

    monkeypatch.setattr(quantizer_fp8, "fp8_blockwise_cast", fake_cast)
    monkeypatch.setattr(quantizer_fp8, "tensor_fp8", fake_tensor)
    monkeypatch.setattr(quantizer_mxfp8, "mxfp8_quantize", fake_mx)
    monkeypatch.setattr(quantizer_nvfp4, "nvfp4_quantize_1d", fake_nv)
    monkeypatch.setattr(quantizer_nvfp4, "nvfp4_quantize_1d_pair", fake_pair)
    return calls


FP8_CFG = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}
W = torch.zeros(4, 32, dtype=torch.bfloat16)


class TestDispatch:
    def test_none_config_and_unmatched_names_return_the_same_list(self, fake_kernels):
        params = [("model.norm.weight", W)]
        assert P.quantize_params(None, "module.module.decoder.final_layernorm.weight", params, None) is params
        for cfg in (FP8_CFG, {"quant_method": "mxfp8"}, {"quant_method": "nvfp4"}):
            assert P.quantize_params(None, "module.module.decoder.final_layernorm.weight", params, cfg) is params
            assert P.quantize_params(None, "module.module.decoder.layers.0.self_attention.q_layernorm.weight", params, cfg) is params
        assert fake_kernels == []

    def test_fp8_names_and_scale_suffix(self, fake_kernels):
        params = [("model.layers.0.self_attn.o_proj.weight", W)]
        out = P.quantize_params(None, "module.module.decoder.layers.0.self_attention.linear_proj.weight", params, FP8_CFG)
        assert [n for n, _ in out] == ["model.layers.0.self_attn.o_proj.weight", "model.layers.0.self_attn.o_proj.weight_scale_inv"]
        cfg = {k: v for k, v in FP8_CFG.items() if k != "weight_block_size"}
        out = P.quantize_params(None, "module.module.decoder.layers.0.self_attention.linear_proj.weight", params, cfg)
        assert [n for n, _ in out][1] == "model.layers.0.self_attn.o_proj.weight_scale" and fake_kernels[-1][0] == "fp8_tensor"

    def test_fp8_experts_drop_bf16_scale_entries_and_mtp_layers_match(self, fake_kernels):
        params = [("model.layers.1.mlp.experts.5.down_proj.weight", W), ("model.layers.1.mlp.experts.5.down_proj.weight_scale", W)]
        out = P.quantize_params(None, "module.module.decoder.layers.1.mlp.experts.linear_fc2.weight5", params, FP8_CFG)
        assert [n for n, _ in out] == ["model.layers.1.mlp.experts.5.down_proj.weight", "model.layers.1.mlp.experts.5.down_proj.weight_scale_inv"]
        out = P.quantize_params(None, "module.module.mtp.layers.0.transformer_layer.mlp.linear_fc2.weight",
                                [("model.layers.4.mlp.down_proj.weight", W)], FP8_CFG)
        assert len(out) == 2
        shared = P.quantize_params(None, "module.module.decoder.layers.1.mlp.shared_experts.linear_fc1.weight",
                                   [("a.gate_proj.weight", W), ("a.up_proj.weight", W)], FP8_CFG)
        assert len(shared) == 4

    def test_fp8_honours_modules_to_not_convert_and_indexer_flag(self, fake_kernels):
        cfg = dict(FP8_CFG, modules_to_not_convert=["model.layers.0.self_attn.o_proj"])
        params = [("model.layers.0.self_attn.o_proj.weight", W)]
        out = P.quantize_params(None, "module.module.decoder.layers.0.self_attention.linear_proj.weight", params, cfg)
        assert out == params and fake_kernels == []
        wk = [("model.layers.0.self_attn.indexer.wk.weight", W)]
        name = "module.module.decoder.layers.0.self_attention.wk.weight"
        assert len(P.quantize_params(Namespace(indexer_rope_interleave=False), name, wk, FP8_CFG)) == 2
        assert P.quantize_params(Namespace(indexer_rope_interleave=True), name, wk, FP8_CFG) is wk

    def test_fused_module_must_be_skipped_whole(self):
        mapping = {"qkv_proj": ["q_proj", "k_proj", "v_proj"]}
        assert quantizer_fp8.is_layer_skipped("m.qkv_proj", ["m.q_proj", "m.k_proj", "m.v_proj"], mapping)
        assert not quantizer_fp8.is_layer_skipped("m.qkv_proj", [], mapping)
        with pytest.raises(ValueError, match="some but not all shards"):
            quantizer_fp8.is_layer_skipped("m.qkv_proj", ["m.q_proj"], mapping)

    def test_mxfp8_respects_extra_high_precision_and_bf16_head_tail(self, fake_kernels):
        params = [("model.layers.0.mlp.experts.0.down_proj.weight", W)]
        cfg = {"quant_method": "mxfp8"}
        args = Namespace(extra_high_precision_layers_megatron=("linear_fc2",))
        assert P.quantize_params(args, "decoder.layers.0.mlp.experts.linear_fc2.weight0", params, cfg) is params
        args = Namespace(first_last_layers_bf16=True, num_layers=4, num_layers_at_start_in_bf16=1, num_layers_at_end_in_bf16=1)
        for layer in (0, 3):
            assert P.quantize_params(args, f"decoder.layers.{layer}.mlp.experts.linear_fc2.weight0", params, cfg) is params
        out = P.quantize_params(args, "decoder.layers.1.mlp.experts.linear_fc2.weight0", params, cfg)
        assert [n for n, _ in out] == ["model.layers.0.mlp.experts.0.down_proj.weight", "model.layers.0.mlp.experts.0.down_proj.weight_scale_inv"]
        assert out[1][1].dtype == torch.uint8

    def test_should_use_mxfp8(self):
        name = "model.layers.0.mlp.experts.0.down_proj.weight"
        assert should_use_mxfp8(name, (4, 32), torch.bfloat16)
        assert not should_use_mxfp8(name, (4, 32), torch.bfloat16, skip_substrings=("mlp.experts.0",))
        assert should_use_mxfp8(name, (4, 32), torch.bfloat16, skip_substrings=("mlp.experts.1",))
        assert not should_use_mxfp8(name, (4, 48), torch.bfloat16) and not should_use_mxfp8(name, (32,), torch.bfloat16)
        assert not should_use_mxfp8("model.norm.weight", (4, 32), torch.bfloat16)
        assert not should_use_mxfp8(name, (4, 32), torch.float8_e4m3fn) and should_use_mxfp8(name, (4, 32), torch.float8_e4m3fn, allow_source_fp8=True)
        assert should_use_mxfp8(name, (4, 16), torch.uint8, packed_mxfp4_experts=True)

    def test_nvfp4_pairs_gate_and_up_and_names_outputs(self, fake_kernels):
        cfg = {"quant_method": "nvfp4"}
        fc1 = [("model.layers.0.mlp.experts.0.gate_proj.weight", W), ("model.layers.0.mlp.experts.0.up_proj.weight", W)]
        out = P.quantize_params(None, "decoder.layers.0.mlp.experts.linear_fc1.weight0", fc1, cfg)
        assert [n for n, _ in out] == [f"model.layers.0.mlp.experts.0.{p}_proj.{s}" for p in ("gate", "up")
                                       for s in ("weight", "weight_scale", "weight_scale_2")]
        assert fake_kernels == [("nvfp4_pair", (4, 32), (4, 32))]
        assert not any(n.endswith("input_scale") for n, _ in out)
        down = [("model.layers.0.mlp.experts.0.down_proj.weight", W)]
        assert len(P.quantize_params(None, "module.module.decoder.layers.0.mlp.experts.linear_fc2.weight0", down, cfg)) == 3
        # dense layers, MTP layers and non-decoder towers stay in high precision
        dense = [("model.layers.0.mlp.down_proj.weight", W)]
        assert P.quantize_params(None, "module.module.decoder.layers.0.mlp.linear_fc2.weight", dense, cfg) is dense
        assert P.quantize_params(None, "module.module.mtp.layers.0.mlp.experts.linear_fc2.weight0", down, cfg) is down

    def test_nvfp4_errors_and_ignore_rules(self, fake_kernels):
        cfg = {"quant_method": "nvfp4"}
        gate_only = [("model.layers.0.mlp.experts.0.gate_proj.weight", W)]
        with pytest.raises(ValueError, match="requires gate/up tensors to be quantized together"):
            P.quantize_params(None, "decoder.layers.0.mlp.experts.linear_fc1.weight0", gate_only, cfg)
        with pytest.raises(ValueError, match="must be divisible by 16"):
            P.quantize_params(None, "decoder.layers.0.mlp.experts.linear_fc2.weight0",
                              [("model.layers.0.mlp.experts.0.down_proj.weight", torch.zeros(4, 24, dtype=torch.bfloat16))], cfg)
        with pytest.raises(NotImplementedError, match="fp4-param-gather"):
            P.quantize_params(Namespace(fp4_param=True), "decoder.layers.0.mlp.experts.linear_fc2.weight0", gate_only, cfg)
        args = Namespace(extra_high_precision_layers_megatron=("linear_fc1",))
        assert P.quantize_params(args, "decoder.layers.0.mlp.experts.linear_fc1.weight0", gate_only, cfg) is gate_only
        down = [("model.layers.0.mlp.experts.0.down_proj.weight", W)]
        for rules in (["model.layers.0.mlp.experts"], ["re:model\\.layers\\.0\\..*"], "model.layers.0"):
            out = P.quantize_params(None, "decoder.layers.0.mlp.experts.linear_fc2.weight0", down, dict(cfg, ignore=rules))
            assert out == down
        out = P.quantize_params(None, "decoder.layers.0.mlp.experts.linear_fc2.weight0", down,
                                dict(cfg, exclude_modules=["model.layers.1"]))
        assert len(out) == 3

    def test_nvfp4_three_dimensional_weights_are_stacked(self, fake_kernels):
        q, s, g = quantizer_nvfp4.quantize_nvfp4(torch.zeros(3, 4, 32, dtype=torch.bfloat16))
        assert q.shape == (3, 4, 16) and s.shape == (3, 4, 2) and g.shape == (3,)
        with pytest.raises(ValueError, match="Unsupported weight rank"):
            quantizer_nvfp4.quantize_nvfp4(torch.zeros(32))

    def test_compressed_tensors_output_names(self, monkeypatch):
        from miles_amd.megatron_to_hf.processors import quantizer_compressed_tensors as C

        monkeypatch.setattr(C, "pack_layer", lambda w, g, sym: (torch.zeros(w.shape[0], w.shape[1] // 8, dtype=torch.int32),
                                                                 torch.zeros(w.shape[0], w.shape[1] // g, dtype=w.dtype), None))
        cfg = {"quant_method": "compressed-tensors", "format": "pack-quantized",
               "config_groups": {"group_0": {"weights": {"group_size": 32, "symmetric": True, "num_bits": 4}}}}
        params = [("model.layers.0.mlp.experts.0.down_proj.weight", W), ("model.layers.0.mlp.gate.weight", W)]
        out = P.quantize_params(None, "x", params, cfg, {"model.layers.0.mlp.experts.0.down_proj"})
        assert [n for n, _ in out] == ["model.layers.0.mlp.experts.0.down_proj.weight_packed",
                                       "model.layers.0.mlp.experts.0.down_proj.weight_scale",
                                       "model.layers.0.mlp.experts.0.down_proj.weight_shape",
                                       "model.layers.0.mlp.gate.weight"]
        assert out[2][1].tolist() == [4, 32] and out[2][1].dtype == torch.int32
        with pytest.raises(AssertionError, match="packed weight names"):
            P.quantize_params(None, "x", params, cfg)


def test_division_by_the_nvfp4_numerators_is_exact_with_one_fma_correction():
    # Four Over Six divides every dequantized candidate by 6 * e4m3_max.  The gfx950 kernel uses
    # q0 = x*y; r = fma(-q0, d, x); q = fma(r, y, q0) with y = RN(1/d): check it against the IEEE quotient on a
    # large sample of mantissas here (the exhaustive sweep over all 2^23 mantissas was run once in C).
    import numpy as np
    rng = np.random.default_rng(1)
    for d in (2688.0, 1536.0):
        d32 = np.float32(d)
        y = np.float32(1.0) / d32
        m = rng.integers(0, 1 << 23, size=1 << 20, dtype=np.uint32)
        x = ((np.uint32(127) << np.uint32(23)) | m).view(np.float32)
        q0 = x * y
        r = (-(q0.astype(np.float64) * np.float64(d32)) + x.astype(np.float64)).astype(np.float32)   # exact: the fma's value
        q = (r.astype(np.float64) * np.float64(y) + q0.astype(np.float64)).astype(np.float32)
        assert np.array_equal(q, x / d32)


def test_sync_plan_matches_quick_and_full_forms():
    # the quick form (same tensor objects, same addresses) and the full signature must agree on what a parameter set is
    from miles_amd.weight_update.sync_plan import SyncPlan, weights_signature

    weights = {f"p{i}": torch.zeros(4, 8) for i in range(5)}
    plan = SyncPlan(batch=None, buckets=[], jobs_done_at_bucket=[], signature=weights_signature(weights), replayable=True)
    plan.remember(weights)
    assert plan.matches(weights)
    assert plan.matches(dict(weights))                                    # another mapping, same objects
    assert plan.matches({k: v.view(4, 8) for k, v in weights.items()})    # other objects, same storage and shape: full form
    assert not plan.matches({k: v.view(8, 4) for k, v in weights.items()})
    assert not plan.matches({k: v.clone() for k, v in weights.items()})
    assert not plan.matches({k: weights[k] for k in list(weights)[:4]})
    assert not plan.matches({("q" + k): v for k, v in weights.items()})   # same objects under other names
    weights["p2"].data = torch.zeros(4, 8)                                # storage swapped under the same object
    assert not plan.matches(weights)
    plan.remember(weights)
    assert plan.matches(weights)
    weights["p3"].resize_(2, 8)                                           # same object, same address, fewer elements
    assert not plan.matches(weights)
    plan.remember(weights)
    plan.signature = weights_signature(weights)
    assert plan.matches(weights)
    weights["p4"].set_(weights["p4"].untyped_storage(), 0, (8, 4))        # same object, address and size, another shape
    assert not plan.matches(weights)
    plan.replayable = False
    plan.remember(weights)
    assert not plan.matches(weights)


def test_sync_plan_identity_test_leaves_the_collector_alone():
    """The quick form runs once per sync over every parameter.  It must not hold thousands of freshly made container
    objects (one `torch.Size` per tensor) at a time: that many allocations between two collections make Python's
    collector run, and its full collection over the objects of a large plan stalls the sync for tens of milliseconds."""
    import gc

    from miles_amd.weight_update.sync_plan import SyncPlan, weights_signature

    weights = {f"p{i}": torch.zeros(2, 3) for i in range(6000)}
    plan = SyncPlan(batch=None, buckets=[], jobs_done_at_bucket=[], signature=weights_signature(weights), replayable=True)
    plan.remember(weights)
    runs = []
    watch = lambda phase, info: runs.append(info["generation"]) if phase == "start" else None
    gc.collect()
    gc.callbacks.append(watch)
    try:
        for _ in range(3):
            assert plan.matches(weights)
    finally:
        gc.callbacks.remove(watch)
    assert len(runs) <= 1, f"three identity tests over 6000 tensors made the collector run {len(runs)} times"


def test_sync_plan_tops_up_small_trailing_launches_only():
    from miles_amd import _lib, launch
    from miles_amd.weight_update.sync_plan import SyncPlan

    def plan_with(jobs, marks):
        batch = launch.JobBatch()
        batch.replace_records(jobs)
        return SyncPlan(batch=batch, buckets=[[] for _ in marks], jobs_done_at_bucket=marks, signature=(), replayable=True)

    def job(kind, elements, aux=None):
        return (kind, 1, 1, 2, 3, aux, None, 1, elements, elements, 0, 0, 0, 0)

    small = [job(_lib.JOB_MXFP8, 1 << 20) for _ in range(200)]
    # 70 small jobs: one full group and a trailing launch of 6 -> topped up to 128; the next bucket is then covered up to 128
    assert plan_with(small, [70, 120, 200]).submission_marks() == [128, 128, 200]
    # a submission that ends on a group boundary stays where it is
    assert plan_with(small, [64, 200]).submission_marks() == [64, 200]
    big = [job(_lib.JOB_FP8_BLOCKWISE_CAST, 1 << 25) for _ in range(100)]
    assert plan_with(big, [35, 70, 100]).submission_marks() == [35, 70, 100]          # 35 x 32 Mi elements: not small
    # NVFP4 jobs that share an amax record (a gate/up pair) are never separated by a topped-up cut
    pairs = []
    for p in range(100):
        pairs += [job(_lib.JOB_NVFP4, 1 << 16, aux=1000 + p), job(_lib.JOB_NVFP4, 1 << 16, aux=1000 + p),
                  job(_lib.JOB_NVFP4, 1 << 16, aux=5000 + p)]
    marks = plan_with(pairs, [9, 300]).submission_marks()
    assert marks[0] >= 64 and pairs[marks[0]][5] != pairs[marks[0] - 1][5]
    assert marks == [65, 300]      # index 64 is the second job of a pair: the cut moves to 65


# ---------------------------------------------------------------------------------------------------
# NVFP4 fake-QAT switch (miles/utils/nvfp4_fake_qat.py; the reference's TestNVFP4FakeQATAdapter)
def test_nvfp4_fake_qat_switch_off_returns_the_same_list(monkeypatch):
    from miles_amd.utils import nvfp4_fake_qat as qat

    weights = [torch.nn.Parameter(torch.empty(4, 16))]
    for value in ("0", "true", ""):
        monkeypatch.setenv(qat.NVFP4_FAKE_QAT_FLAG, value)
        assert qat.maybe_fake_quantize_nvfp4_weight_tensors(weights) is weights
    monkeypatch.delenv(qat.NVFP4_FAKE_QAT_FLAG)
    assert qat.maybe_fake_quantize_nvfp4_weight_tensors(weights) is weights


def test_nvfp4_fake_qat_switch_on_reads_the_configuration_once(monkeypatch):
    from miles_amd.kernels.quant import nvfp4_qdq
    from miles_amd.utils import nvfp4_fake_qat as qat

    weights = [torch.nn.Parameter(torch.empty(4, 16)) for _ in range(3)]
    images = [torch.empty_like(w) for w in weights]
    config, seen, reads = object(), [], []
    monkeypatch.setattr(nvfp4_qdq, "current_nvfp4_qdq_config", lambda: reads.append(1) or config)
    monkeypatch.setattr(nvfp4_qdq, "fake_nvfp4_quantization_ste", lambda w, c: seen.append((w, c)) or images[len(seen) - 1])
    monkeypatch.setenv(qat.NVFP4_FAKE_QAT_FLAG, "1")
    out = qat.maybe_fake_quantize_nvfp4_weight_tensors(weights)
    assert len(reads) == 1 and len(out) == 3
    assert all(o is i for o, i in zip(out, images))
    assert all(w is got_w and c is config for w, (got_w, c) in zip(weights, seen))


# ---------------------------------------------------------------------------------------------------
# Llama and GLM-4 dense name maps (megatron_to_hf/llama.py, glm4.py)
def test_llama_and_glm4_name_maps():
    from argparse import Namespace

    from miles_amd.megatron_to_hf import convert_to_hf, name_maps

    args = Namespace(hidden_size=64, num_attention_heads=4, num_query_groups=2, kv_channels=16, vocab_size=100)
    L = "module.module.decoder.layers.3."
    qkv = torch.arange(2 * (2 + 1 + 1) * 16 * 64, dtype=torch.float32).reshape(-1, 64)
    fc1 = torch.arange(2 * 24 * 64, dtype=torch.float32).reshape(48, 64)

    names = lambda out: [n for n, _ in out]
    llama = name_maps.convert_llama_to_hf
    assert names(llama(args, L + "self_attention.linear_qkv.weight", qkv)) == [
        f"model.layers.3.self_attn.{p}_proj.weight" for p in "qkv"]
    q, k, v = (t for _, t in llama(args, L + "self_attention.linear_qkv.weight", qkv))
    grouped = qkv.view(2, 4, 16, 64)
    assert torch.equal(q, grouped[:, :2].reshape(-1, 64)) and torch.equal(k, grouped[:, 2].reshape(-1, 64))
    assert torch.equal(v, grouped[:, 3].reshape(-1, 64))
    gate_up = llama(args, L + "mlp.linear_fc1.weight", fc1)
    assert names(gate_up) == ["model.layers.3.mlp.gate_proj.weight", "model.layers.3.mlp.up_proj.weight"]
    assert torch.equal(gate_up[0][1], fc1[:24]) and torch.equal(gate_up[1][1], fc1[24:])
    assert names(llama(args, L + "pre_mlp_layernorm.weight", fc1[0])) == ["model.layers.3.post_attention_layernorm.weight"]
    assert names(llama(args, "module.module.output_layer.weight", fc1)) == ["lm_head.weight"]
    for unknown in ("self_attention.linear_qkv.bias", "self_attention.q_layernorm.weight", "input_layernorm.weight"):
        with pytest.raises(ValueError, match="Unknown parameter name"):
            llama(args, L + unknown, fc1[0])

    glm4 = name_maps.convert_glm4_to_hf
    fused = glm4(args, L + "mlp.linear_fc1.weight", fc1)
    assert names(fused) == ["model.layers.3.mlp.gate_up_proj.weight"] and fused[0][1] is fc1      # gate and up stay fused
    assert names(glm4(args, L + "post_self_attn_layernorm.weight", fc1[0])) == ["model.layers.3.post_self_attn_layernorm.weight"]
    assert names(glm4(args, L + "post_mlp_layernorm.weight", fc1[0])) == ["model.layers.3.post_mlp_layernorm.weight"]
    assert names(glm4(args, L + "self_attention.linear_qkv.bias", torch.arange(128.0))) == [
        f"model.layers.3.self_attn.{p}_proj.bias" for p in "qkv"]
    with pytest.raises(ValueError, match="Unknown parameter name"):
        glm4(args, L + "pre_mlp_layernorm.weight", fc1[0])

    # dispatch by model name: glm4 before qwen*, llama last; GLM-4 MoE is a different map and is refused, not mis-mapped
    assert names(convert_to_hf(args, "Llama-3.1-8B", L + "mlp.linear_fc2.weight", fc1)) == ["model.layers.3.mlp.down_proj.weight"]
    assert names(convert_to_hf(args, "glm4", L + "mlp.linear_fc1.weight", fc1)) == ["model.layers.3.mlp.gate_up_proj.weight"]
    for other_family in ("qwen3next", "Qwen3_5-MoE", "glm5_next", "deepseekv4", "kimi_k3", "kimi_k25", "kimivl"):      # maps not built here: refused, never mis-mapped
        with pytest.raises(ValueError, match="Unsupported model"):
            convert_to_hf(args, other_family, L + "mlp.linear_fc1.weight", fc1)


def test_glm4moe_name_map():
    from argparse import Namespace

    from miles_amd.megatron_to_hf import convert_to_hf

    args = Namespace(hidden_size=64, num_attention_heads=4, num_query_groups=2, kv_channels=16, vocab_size=100, num_layers=5)
    names = lambda name, t: [n for n, _ in convert_to_hf(args, "glm4moe", name, t)]
    L = "module.module.decoder.layers.2."
    w = torch.arange(48 * 64, dtype=torch.float32).reshape(48, 64)
    assert names(L + "mlp.experts.linear_fc1.weight7", w) == [
        "model.layers.2.mlp.experts.7.gate_proj.weight", "model.layers.2.mlp.experts.7.up_proj.weight"]
    assert names(L + "mlp.experts.linear_fc2.weight7", w) == ["model.layers.2.mlp.experts.7.down_proj.weight"]
    assert names(L + "mlp.shared_experts.linear_fc1.weight", w) == [
        "model.layers.2.mlp.shared_experts.gate_proj.weight", "model.layers.2.mlp.shared_experts.up_proj.weight"]
    assert names(L + "mlp.shared_experts.linear_fc2.weight", w) == ["model.layers.2.mlp.shared_experts.down_proj.weight"]
    assert names(L + "mlp.router.weight", w) == ["model.layers.2.mlp.gate.weight"]
    assert names(L + "mlp.router.expert_bias", w[0]) == ["model.layers.2.mlp.gate.e_score_correction_bias"]
    assert names(L + "post_self_attn_layernorm.weight", w[0]) == ["model.layers.2.post_self_attn_layernorm.weight"]
    assert names(L + "post_mlp_layernorm.weight", w[0]) == ["model.layers.2.post_mlp_layernorm.weight"]
    assert names(L + "mlp.linear_fc1.weight", w) == ["model.layers.2.mlp.gate_proj.weight", "model.layers.2.mlp.up_proj.weight"]
    assert names(L + "self_attention.linear_qkv.bias", torch.arange(128.0)) == [
        f"model.layers.2.self_attn.{p}_proj.bias" for p in "qkv"]
    # MTP layers come after the decoder's, and the transformer layer inside one goes through the same map
    M = "module.module.mtp.layers.1."
    assert names(M + "eh_proj.weight", w) == ["model.layers.6.eh_proj.weight"]
    assert names(M + "final_layernorm.weight", w[0]) == ["model.layers.6.shared_head.norm.weight"]
    assert names(M + "transformer_layer.mlp.experts.linear_fc2.weight3", w) == ["model.layers.6.mlp.experts.3.down_proj.weight"]
    assert names(M + "transformer_layer.self_attention.linear_proj.weight", w) == ["model.layers.6.self_attn.o_proj.weight"]
    for bad in (L + "mlp.shared_experts.gate_weight", L + "mlp.experts.linear_fc3.weight0", L + "input_layernorm.weight",
                "module.module.unknown.weight"):
        with pytest.raises(ValueError, match="Unknown"):
            names(bad, w)


def test_mimo_name_map():
    from argparse import Namespace

    from miles_amd.megatron_to_hf import convert_to_hf

    args = Namespace(hidden_size=64, num_attention_heads=4, num_query_groups=2, kv_channels=16, vocab_size=100, num_layers=5)
    conv = lambda name, t: convert_to_hf(args, "MiMo-7B", name, t)
    w = torch.arange(64 * 128, dtype=torch.float32).reshape(64, 128)
    M = "module.module.mtp.layers.0."
    (name, swapped), = conv(M + "eh_proj.weight", w)
    assert name == "model.mtp_layers.0.input_proj.weight"
    assert torch.equal(swapped[:, :64], w[:, 64:]) and torch.equal(swapped[:, 64:], w[:, :64])
    assert [n for n, _ in conv(M + "enorm.weight", w[0])] == ["model.mtp_layers.0.token_layernorm.weight"]
    assert [n for n, _ in conv(M + "hnorm.weight", w[0])] == ["model.mtp_layers.0.hidden_layernorm.weight"]
    assert [n for n, _ in conv(M + "final_layernorm.weight", w[0])] == ["model.mtp_layers.0.final_layernorm.weight"]
    assert [n for n, _ in conv(M + "transformer_layer.mlp.linear_fc1.weight", w)] == [
        "model.mtp_layers.0.mlp.gate_proj.weight", "model.mtp_layers.0.mlp.up_proj.weight"]
    assert [n for n, _ in conv(M + "mtp_model_layer.self_attention.linear_proj.weight", w)] == [
        "model.mtp_layers.0.self_attn.o_proj.weight"]
    assert [n for n, _ in conv("module.module.decoder.layers.4.self_attention.q_layernorm.weight", w[0])] == [
        "model.layers.4.self_attn.q_norm.weight"]
    with pytest.raises(ValueError, match="Unknown MTP component"):
        conv(M + "something_else.weight", w)
    with pytest.raises(ValueError, match="Invalid MTP parameter name"):
        conv("module.module.mtp.weight", w)


def test_shared_divisor_division_is_exact_and_keeps_the_sign_of_zero():
    # The FP8 / INT4 kernels divide many elements by one scale s with y = RN(1/s):
    #   q0 = x*y; e = fma(q0, s, -x); q = fma(-e, y, q0)
    # For bf16 / fp16 numerators this must be the IEEE quotient, signed zeros included (the exhaustive sweep over all
    # 2^23 divisor mantissas x all numerator mantissas was run once in C; this is a large sample plus the zero cases).
    # The two FMAs are evaluated in float64: the residual e is exactly representable, and q0 - e*y has fewer than 53
    # significant bits between its largest and smallest term, so float64 holds both results before the one rounding.
    import numpy as np
    rng = np.random.default_rng(7)
    n = 1 << 21
    s = ((rng.integers(90, 170, size=n, dtype=np.uint32) << np.uint32(23)) | rng.integers(0, 1 << 23, size=n, dtype=np.uint32)).view(np.float32)
    xm = rng.integers(0, 1 << 10, size=n, dtype=np.uint32) << np.uint32(13)          # up to 11 significant bits
    x = ((rng.integers(0, 2, size=n, dtype=np.uint32) << np.uint32(31)) | (rng.integers(100, 150, size=n, dtype=np.uint32) << np.uint32(23)) | xm).view(np.float32)
    x[:1024:2] = np.float32(-0.0)
    x[1:1024:2] = np.float32(0.0)
    y = np.float32(1.0) / s
    q0 = x * y
    e = (q0.astype(np.float64) * s.astype(np.float64) - x.astype(np.float64)).astype(np.float32)
    q = (q0.astype(np.float64) - e.astype(np.float64) * y.astype(np.float64)).astype(np.float32)
    want = x / s
    assert np.array_equal(q.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(np.signbit(q[:1024]), np.signbit(x[:1024])) and not q[:1024].any()


# ---------------------------------------------------------------------------------------------------
# quantized snapshot export (miles/backends/training_utils/weight_update/snapshot_publisher.py:62-99)
def test_snapshot_publisher_writes_shards_index_and_metadata(tmp_path):
    import json

    import safetensors.torch

    from miles_amd.weight_update.hf_weight_iterator import HfWeightIteratorDirect
    from miles_amd.weight_update.snapshot_publisher import SnapshotPublisher

    args = Namespace(**vars(QWEN_ARGS), update_weight_buffer_size=20000)
    L = "module.module.decoder.layers.0."
    weights = {"module.module.embedding.word_embeddings.weight": torch.randn(100, 64).to(torch.bfloat16),
               L + "self_attention.linear_proj.weight": torch.randn(64, 64).to(torch.bfloat16),
               L + "mlp.linear_fc1.weight": torch.randn(64, 64).to(torch.bfloat16),
               L + "mlp.linear_fc2.weight": torch.randn(64, 32).to(torch.bfloat16),
               "module.module.decoder.final_layernorm.weight": torch.randn(64).to(torch.bfloat16)}
    base = tmp_path / "base"
    base.mkdir()
    (base / "config.json").write_text('{"model_type": "qwen3"}')
    (base / "tokenizer.json").write_text("{}")
    (base / "model.safetensors.index.json").write_text('{"weight_map": {"stale": "x"}}')
    (base / "model-00001-of-00001.safetensors").write_bytes(b"not copied")
    out = tmp_path / "snapshot"
    out.mkdir()
    iterator = HfWeightIteratorDirect(args, model_name="qwen3", quantization_config=None)
    SnapshotPublisher(iterator).write_model(out, weights=weights, hf_checkpoint=str(base))

    index = json.loads((out / "model.safetensors.index.json").read_text())
    shards = sorted(p.name for p in out.glob("model-*.safetensors"))
    assert len(shards) > 1 and shards[0] == "model-00001.safetensors" and set(index["weight_map"].values()) == set(shards)
    assert sorted(p.name for p in out.iterdir() if not p.name.startswith("model")) == ["config.json", "tokenizer.json"]
    got = {}
    for shard in shards:
        got.update(safetensors.torch.load_file(out / shard))
    want = {}
    for name, param in weights.items():
        want.update(dict(name_maps.convert_qwen2_to_hf(args, name, param)))
    assert set(got) == set(want) == set(index["weight_map"])
    for name, t in want.items():
        assert torch.equal(got[name], t.contiguous())
    assert index["metadata"]["total_size"] == sum(t.numel() * t.element_size() for t in want.values())
    # a base checkpoint that is not a local directory: the shards and the index are still written
    out2 = tmp_path / "snapshot2"
    out2.mkdir()
    SnapshotPublisher(iterator).write_model(out2, weights=weights, hf_checkpoint="Qwen/Qwen3-4B")
    assert (out2 / "model.safetensors.index.json").exists() and not (out2 / "config.json").exists()
    with pytest.raises(AssertionError, match="produced no weights"):
        SnapshotPublisher(iterator).write_model(out2, weights={}, hf_checkpoint=str(base))
