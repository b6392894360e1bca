"""Megatron -> HuggingFace parameter naming for the model families on the benchmark path.

Table-driven restatement of the reference's per-model converters:
  convert_qwen2_to_hf       miles/backends/megatron_utils/megatron_to_hf/qwen2.py:5-75      (Qwen2 / Qwen3 dense)
  convert_qwen3moe_to_hf    .../megatron_to_hf/qwen3moe.py:6-117                            (Qwen3 MoE)
  convert_deepseekv3_to_hf  .../megatron_to_hf/deepseekv3.py:18-175                         (DeepSeek-V3 / Kimi-K2 / GLM MoE-DSA)
Each returns a list of (hf_name, tensor); fused QKV is split per query group and fused gate/up is chunked,
as views where PyTorch allows (chunk) and copies where it does not (the QKV regrouping).
"""

from __future__ import annotations

import re

import torch

_TOP_LEVEL = {
    "module.module.embedding.word_embeddings.weight": "model.embed_tokens.weight",
    "module.module.output_layer.weight": "lm_head.weight",
    "module.module.decoder.final_layernorm.weight": "model.norm.weight",
}
_DECODER = re.compile(r"module\.module\.decoder\.layers\.(\d+)\.(.+)")
_MTP = re.compile(r"module\.module\.mtp\.layers\.(\d+)\.(.+)")
_ROUTED = re.compile(r"mlp.experts\.(.+)\.weight(\d+)")
_SHARED = re.compile(r"mlp.shared_experts\.(.+)")

# one-to-one renames inside a decoder layer: Megatron `rest` -> HF suffix after "model.layers.<i>."
_COMMON_RENAMES = {
    "self_attention.linear_proj.weight": "self_attn.o_proj.weight",
    "mlp.linear_fc2.weight": "mlp.down_proj.weight",
    "self_attention.linear_qkv.layer_norm_weight": "input_layernorm.weight",
    "mlp.linear_fc1.layer_norm_weight": "post_attention_layernorm.weight",
    "pre_mlp_layernorm.weight": "post_attention_layernorm.weight",
}
_QWEN2_RENAMES = {
    **_COMMON_RENAMES,
    "input_layernorm.weight": "input_layernorm.weight",
    "self_attention.q_layernorm.weight": "self_attn.q_norm.weight",
    "self_attention.k_layernorm.weight": "self_attn.k_norm.weight",
}
_QWEN3MOE_RENAMES = {
    **_COMMON_RENAMES,
    "mlp.router.weight": "mlp.gate.weight",
    "mlp.router.expert_bias": "mlp.gate.e_score_correction_bias",
    "self_attention.q_layernorm.weight": "self_attn.q_norm.weight",
    "self_attention.k_layernorm.weight": "self_attn.k_norm.weight",
}
_DSV3_NATIVE_DSA = {
    "self_attention.core_attention.indexer.linear_wq_b.weight": "self_attn.indexer.wq_b.weight",
    "self_attention.core_attention.indexer.linear_wk.weight": "self_attn.indexer.wk.weight",
    "self_attention.core_attention.indexer.linear_weights_proj.weight": "self_attn.indexer.weights_proj.weight",
    "self_attention.core_attention.indexer.k_norm.weight": "self_attn.indexer.k_norm.weight",
    "self_attention.core_attention.indexer.k_norm.bias": "self_attn.indexer.k_norm.bias",
    "self_attention.q_layernorm.weight": "self_attn.q_a_layernorm.weight",
    "self_attention.kv_layernorm.weight": "self_attn.kv_a_layernorm.weight",
}
_DSV3_RENAMES = {
    **_COMMON_RENAMES,
    "input_layernorm.weight": "input_layernorm.weight",
    "self_attention.linear_q_proj.weight": "self_attn.q_proj.weight",
    "self_attention.linear_q_down_proj.weight": "self_attn.q_a_proj.weight",
    "self_attention.linear_q_up_proj.layer_norm_weight": "self_attn.q_a_layernorm.weight",
    "self_attention.linear_q_up_proj.weight": "self_attn.q_b_proj.weight",
    "self_attention.linear_kv_down_proj.weight": "self_attn.kv_a_proj_with_mqa.weight",
    "self_attention.linear_kv_up_proj.layer_norm_weight": "self_attn.kv_a_layernorm.weight",
    "self_attention.linear_kv_up_proj.weight": "self_attn.kv_b_proj.weight",
    "self_attention.weights_proj.weight": "self_attn.indexer.weights_proj.weight",
    "mlp.router.weight": "mlp.gate.weight",
    "mlp.router.expert_bias": "mlp.gate.e_score_correction_bias",
}


def _head_dim(args) -> int:
    kv = getattr(args, "kv_channels", None)
    return kv if kv is not None else args.hidden_size // args.num_attention_heads


def gather_groups(parts: torch.Tensor, shape) -> torch.Tensor:
    """`parts` [groups, ...] is a strided selection of each group's rows (or elements) whose per-group piece is
    contiguous; returns the pieces back to back as a tensor of `shape`.  On the GPU the regrouping is one 2-D byte-copy
    job (one job per group where the pieces cannot be seen as rows of one view) instead of a torch copy, so a recorded sync can repeat it on the current weights (a replayed plan hands
    out the same output tensor, refreshed by the job)."""
    if parts.device.type != "cuda":
        return parts.reshape(shape)
    from miles_amd.weight_update.packed_bucket import submit_copy, submit_copy_rows

    out = torch.empty(parts.numel(), dtype=parts.dtype, device=parts.device).view(shape)
    flat = out.view(parts.shape[0], -1)
    try:
        rows = parts.view(parts.shape[0], -1)      # the groups' pieces one group pitch apart: a single 2-D copy job
    except RuntimeError:
        rows = None
    if rows is not None and parts.numel():
        submit_copy_rows(rows, flat)
    else:
        for g in range(parts.shape[0]):
            submit_copy(parts[g].reshape(-1), flat[g])
    return out


def _split_qkv_weight(args, layer: str, param: torch.Tensor):
    groups = args.num_query_groups
    q_per_group = args.num_attention_heads // groups
    grouped = param.view(groups, -1, _head_dim(args), args.hidden_size)
    q, k, v = torch.split(grouped, [q_per_group, 1, 1], dim=1)
    # opt-in of the batched sync driver: hand q / k / v on as [groups, rows, hidden] VIEWS of the fused weight; the
    # FP8 kernel reads the row blocks in place and the regrouping copy disappears.  Only the tuned kernel reads such
    # views, and it takes contiguous bf16 or fp16 storage that starts on a 16-byte boundary: a parameter carved out of
    # a flat buffer at an odd offset, or held in fp32, is regrouped with copy jobs like everywhere else.
    in_place = (getattr(args, "qkv_row_block_views", False) and param.dtype in (torch.bfloat16, torch.float16)
                and param.is_contiguous() and param.data_ptr() % 16 == 0)
    if in_place:
        return [(f"model.layers.{layer}.self_attn.{n}_proj.weight", t.flatten(1, 2))
                for n, t in (("q", q), ("k", k), ("v", v))]
    return [(f"model.layers.{layer}.self_attn.{n}_proj.weight", gather_groups(t, (-1, args.hidden_size)))
            for n, t in (("q", q), ("k", k), ("v", v))]


def _split_qkv_bias(args, layer: str, param: torch.Tensor):
    groups = args.num_query_groups
    q_per_group = args.num_attention_heads // groups
    hd = _head_dim(args)
    q, k, v = torch.split(param.view(groups, -1), [q_per_group * hd, hd, hd], dim=1)
    return [(f"model.layers.{layer}.self_attn.{n}_proj.bias", gather_groups(t, (-1,)))
            for n, t in (("q", q), ("k", k), ("v", v))]


def _gate_up(prefix: str, param: torch.Tensor):
    gate, up = param.chunk(2, dim=0)
    return [(f"{prefix}.gate_proj.weight", gate), (f"{prefix}.up_proj.weight", up)]


def _routed_expert(name: str, layer: str, rest: str, param: torch.Tensor):
    m = _ROUTED.match(rest)
    if not m:
        return None
    linear, expert = m.groups()
    prefix = f"model.layers.{layer}.mlp.experts.{expert}"
    if linear == "linear_fc1":
        return _gate_up(prefix, param)
    if linear == "linear_fc2":
        return [(f"{prefix}.down_proj.weight", param)]
    raise ValueError(f"Unknown expert parameter name: {name}")


def _shared_expert(name: str, layer: str, rest: str, param: torch.Tensor, module: str, gate_key: bool):
    m = _SHARED.match(rest)
    if not m:
        return None
    sub = m.group(1)
    prefix = f"model.layers.{layer}.mlp.{module}"
    if sub == "linear_fc1.weight":
        return _gate_up(prefix, param)
    if sub == "linear_fc2.weight":
        return [(f"{prefix}.down_proj.weight", param)]
    if gate_key and sub == "gate_weight":
        return [(f"model.layers.{layer}.mlp.shared_expert_gate.weight", param)]
    raise ValueError(f"Unknown shared expert parameter name: {name}")


def _dense_layer(args, layer: str, rest: str, param: torch.Tensor, renames: dict[str, str]):
    if rest in renames:
        return [(f"model.layers.{layer}.{renames[rest]}", param)]
    if rest == "self_attention.linear_qkv.weight":
        return _split_qkv_weight(args, layer, param)
    if rest == "self_attention.linear_qkv.bias":
        return _split_qkv_bias(args, layer, param)
    if rest == "mlp.linear_fc1.weight":
        return _gate_up(f"model.layers.{layer}.mlp", param)
    return None


def convert_qwen2_to_hf(args, name, param):
    if name in _TOP_LEVEL:
        return [(_TOP_LEVEL[name], param)]
    m = _DECODER.match(name)
    if m:
        out = _dense_layer(args, m.group(1), m.group(2), param, _QWEN2_RENAMES)
        if out is not None:
            return out
    raise ValueError(f"Unknown parameter name: {name}")


# Llama (reference: megatron_to_hf/llama.py:5-53): the dense layer without q / k norms, biases or a separate
# input_layernorm entry.  GLM-4 (reference: megatron_to_hf/glm4.py): gate and up stay fused as gate_up_proj, q / k / v
# biases exist, and the two sandwich norms keep their Megatron names.
_LLAMA_RENAMES = dict(_COMMON_RENAMES)
_GLM4_RENAMES = {
    "self_attention.linear_proj.weight": "self_attn.o_proj.weight",
    "mlp.linear_fc2.weight": "mlp.down_proj.weight",
    "mlp.linear_fc1.weight": "mlp.gate_up_proj.weight",
    "self_attention.linear_qkv.layer_norm_weight": "input_layernorm.weight",
    "mlp.linear_fc1.layer_norm_weight": "post_attention_layernorm.weight",
    "self_attention.q_layernorm.weight": "self_attn.q_norm.weight",
    "self_attention.k_layernorm.weight": "self_attn.k_norm.weight",
    "post_self_attn_layernorm.weight": "post_self_attn_layernorm.weight",
    "post_mlp_layernorm.weight": "post_mlp_layernorm.weight",
}


def _convert_dense_family(args, name, param, renames, *, qkv_bias: bool):
    if name in _TOP_LEVEL:
        return [(_TOP_LEVEL[name], param)]
    m = _DECODER.match(name)
    if m and (qkv_bias or m.group(2) != "self_attention.linear_qkv.bias"):
        out = _dense_layer(args, m.group(1), m.group(2), param, renames)
        if out is not None:
            return out
    raise ValueError(f"Unknown parameter name: {name}")


def convert_llama_to_hf(args, name, param):
    return _convert_dense_family(args, name, param, _LLAMA_RENAMES, qkv_bias=False)


def convert_glm4_to_hf(args, name, param):
    return _convert_dense_family(args, name, param, _GLM4_RENAMES, qkv_bias=True)


def convert_qwen3moe_to_hf(args, name, param):
    if name in _TOP_LEVEL:
        return [(_TOP_LEVEL[name], param)]
    m = _DECODER.match(name)
    if m:
        layer, rest = m.groups()
        out = (_routed_expert(name, layer, rest, param)
               or _shared_expert(name, layer, rest, param, "shared_expert", gate_key=True)
               or _dense_layer(args, layer, rest, param, _QWEN3MOE_RENAMES))
        if out is not None:
            return out
    raise ValueError(f"Unknown parameter name: {name}")


def _mtp_layer(args, name: str, param: torch.Tensor, convert):
    """A multi-token-prediction layer is numbered after the decoder layers; its own four tensors are renamed here, the
    transformer layer inside it goes back through `convert` under that number."""
    m = _MTP.match(name)
    if not m:
        return None
    layer = int(m.group(1)) + args.num_layers
    rest = m.group(2)
    direct = {"eh_proj.weight": "eh_proj.weight", "enorm.weight": "enorm.weight", "hnorm.weight": "hnorm.weight",
              "final_layernorm.weight": "shared_head.norm.weight"}
    if rest in direct:
        return [(f"model.layers.{layer}.{direct[rest]}", param)]
    inner = f"module.module.decoder.layers.{layer}.{rest}".replace("transformer_layer.", "").replace("mtp_model_layer.", "")
    return convert(args, inner, param)


_GLM4MOE_RENAMES = {
    **_QWEN3MOE_RENAMES,
    "post_self_attn_layernorm.weight": "post_self_attn_layernorm.weight",
    "post_mlp_layernorm.weight": "post_mlp_layernorm.weight",
}


def convert_glm4moe_to_hf(args, name, param):
    """GLM-4 MoE (reference: megatron_to_hf/glm4moe.py:6-139): routed and shared experts split into gate / up / down,
    q / k / v regrouped, the norms after attention and after the MLP kept, MTP layers numbered after the decoder's."""
    if name in _TOP_LEVEL:
        return [(_TOP_LEVEL[name], param)]
    m = _DECODER.match(name)
    if m:
        layer, rest = m.groups()
        out = (_routed_expert(name, layer, rest, param)
               or _shared_expert(name, layer, rest, param, "shared_experts", gate_key=False)
               or _dense_layer(args, layer, rest, param, _GLM4MOE_RENAMES))
        if out is not None:
            return out
    out = _mtp_layer(args, name, param, convert_glm4moe_to_hf)
    if out is not None:
        return out
    raise ValueError(f"Unknown parameter name: {name}")


def _rotate_halves(t: torch.Tensor, dim: int) -> torch.Tensor:
    """Swap the two halves along `dim` (64 + 64 channels of a DSA indexer head, the two input halves of MiMo's MTP
    projection).  On the GPU each half is one 2-D byte-copy job, so a recorded sync repeats the swap on
    the current weights; elsewhere a torch concatenation."""
    a, b = t.chunk(2, dim=dim)
    if t.device.type != "cuda" or not t.is_contiguous():
        return torch.cat([b, a], dim=dim)
    from miles_amd.weight_update.packed_bucket import submit_copy_rows

    out = torch.empty_like(t)
    first, second = out.chunk(2, dim=dim)
    lead = 1
    for size in t.shape[:dim]:
        lead *= size
    for src, dst in ((b, first), (a, second)):
        # views: each leading index owns one contiguous run, and the runs are one row pitch apart -- one 2-D copy job
        submit_copy_rows(src.reshape(lead, -1), dst.reshape(lead, -1))
    return out


_MIMO_MTP_DIRECT = {"enorm.weight": "token_layernorm.weight", "hnorm.weight": "hidden_layernorm.weight",
                    "eh_proj.weight": "input_proj.weight", "final_layernorm.weight": "final_layernorm.weight"}


def convert_mimo_to_hf(args, name, param):
    """MiMo (reference: megatron_to_hf/mimo.py:6-75): the Qwen2 map, plus MTP layers that HF keeps under
    `model.mtp_layers.<i>` with their own numbering; the MTP input projection swaps its two column halves."""
    if "mtp" not in name:
        return convert_qwen2_to_hf(args, name, param)
    m = _MTP.match(name)
    if not m:
        raise ValueError(f"Invalid MTP parameter name: {name}")
    layer, rest = m.groups()
    if rest in _MIMO_MTP_DIRECT:
        if rest == "eh_proj.weight":
            param = _rotate_halves(param, 1)
        return [(f"model.mtp_layers.{layer}.{_MIMO_MTP_DIRECT[rest]}", param)]
    for prefix in ("transformer_layer.", "mtp_model_layer."):
        if rest.startswith(prefix):
            inner = convert_qwen2_to_hf(args, f"module.module.decoder.layers.{layer}.{rest[len(prefix):]}", param)
            return [(hf.replace(f"model.layers.{layer}", f"model.mtp_layers.{layer}"), t) for hf, t in inner]
    raise ValueError(f"Unknown MTP component: {rest} in {name}")


def _dsv3_indexer(args, layer: str, rest: str, param: torch.Tensor):
    """DSA indexer tensors; with rope interleave the two 64-channel halves of each 128-wide head swap."""
    interleave = getattr(args, "indexer_rope_interleave", False)
    base = f"model.layers.{layer}.self_attn.indexer"
    if rest == "self_attention.wq_b.weight":
        w = param
        if interleave:
            w = _rotate_halves(w.view(-1, 128, w.shape[-1]), 1).view(-1, w.shape[-1])
        return [(f"{base}.wq_b.weight", w)]
    if rest == "self_attention.wk.weight":
        w = param
        if interleave:
            w = _rotate_halves(w, 0).view(-1, w.shape[-1])
        return [(f"{base}.wk.weight", w)]
    if rest in ("self_attention.k_norm.weight", "self_attention.k_norm.bias"):
        w = _rotate_halves(param, 0) if interleave else param
        return [(f"{base}.k_norm.{rest.rsplit('.', 1)[1]}", w)]
    return None


def convert_deepseekv3_to_hf(args, name, param):
    if name in _TOP_LEVEL:
        return [(_TOP_LEVEL[name], param)]
    m = _DECODER.match(name)
    if m:
        layer, rest = m.groups()
        if rest in _DSV3_NATIVE_DSA:
            return [(f"model.layers.{layer}.{_DSV3_NATIVE_DSA[rest]}", param)]
        out = (_routed_expert(name, layer, rest, param)
               or _shared_expert(name, layer, rest, param, "shared_experts", gate_key=False)
               or _dsv3_indexer(args, layer, rest, param))
        if out is None and rest != "self_attention.linear_qkv.weight":
            out = _dense_layer(args, layer, rest, param, _DSV3_RENAMES)
        if out is not None:
            return out
    out = _mtp_layer(args, name, param, convert_deepseekv3_to_hf)
    if out is not None:
        return out
    raise ValueError(f"Unknown parameter name: {name}")
