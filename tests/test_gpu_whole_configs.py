"""Whole benchmark configurations through the sync driver, every output tensor checked against the oracle.

The per-tensor parity tests cover each quantizer at the configurations' real shapes; these cover the driver at scale:
all 36 layers of the Qwen3-4B FP8 sync (252 quantized tensors with their row-blocked q / k / v offsets, nine buckets,
grouped launches of up to 64 tensors, run-ahead submissions, the packed transport payload) and whole expert layers of
the three MoE configurations.  Weights are generated on the GPU and copied back for the oracle, so both sides see the
same bits; every tensor a sync hands out is copied to the host while its bucket is valid and compared by a 64-bit
fingerprint, a deterministic sample byte by byte (tests/sync_expectations.py).

Sizes: C2, one whole C3 layer (128 experts), all 384 experts of C4 and all 256 of C5a (about 40 s and 25 s of host
time for the oracle and the fingerprints).  MQ_WHOLE_CONFIG_EXPERTS=<n> caps the number of experts for a quicker run.
"""

import os

import pytest
import torch

from miles_amd import workloads as W
from miles_amd.weight_update.updater import WeightUpdater
from tests import sync_expectations as E

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]
DEV = "cuda:0"
FP8_CFG = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}


def _gen(seed):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    return g


def _sync_to_host(updater):
    """One sync; every bucket is copied to the host while it is valid (what a consumer does before the next bucket)."""
    got, buckets = [], []

    def consume(bucket):
        buckets.append(len(bucket))
        got.extend((n, t.cpu()) for n, t in bucket)

    updater.send_bucket = consume
    updater.update_weights()
    torch.cuda.synchronize()
    return got, buckets


def _refill(weights, seed, make):
    """New values in place: same tensor objects, same addresses."""
    gen = _gen(seed)
    for name, t in weights.items():
        if t.dim() == 2:
            t.copy_(make(tuple(t.shape), gen))


def _host(weights):
    return {k: v.cpu() for k, v in weights.items()}


def test_c2_qwen3_4b_fp8_sync_every_tensor(oracle):
    args, weights, elems = W.qwen3_4b_megatron(_gen(2001))
    assert elems == 3_633_315_840
    make = lambda shape, gen: W.device_gaussian_outliers(shape, gen)
    first = _host(weights)
    want = E.expected_dense_fp8(oracle, args, first)
    assert sum(n.endswith("_proj.weight") for n, _ in want) == 252
    upd = WeightUpdater(args, weights_getter=lambda: weights, model_name="qwen3", quantization_config=FP8_CFG, send_bucket=None)
    got, buckets = _sync_to_host(upd)                       # the recording sync
    assert upd._plan is not None and upd._plan.replayable and len(buckets) >= 8
    stats = E.compare_streams(oracle, got, want, "C2 recorded")
    assert stats["tensors"] == len(want) == 252 * 2 + 1 + 36 * 4 + 1
    del got
    _refill(weights, 2002, make)                            # an optimizer step's worth of change: every value, in place
    want2 = E.expected_dense_fp8(oracle, args, _host(weights))
    got, buckets2 = _sync_to_host(upd)                      # replayed plan
    assert buckets2 == buckets
    E.compare_streams(oracle, got, want2, "C2 replayed after an in-place change")
    del got, upd
    packed = WeightUpdater(args, weights_getter=lambda: weights, model_name="qwen3", quantization_config=FP8_CFG,
                           send_bucket=None, packed_buckets=True)
    got, _ = _sync_to_host(packed)                          # packed payloads, recording sync
    assert packed._plan is not None and packed._plan.replayable
    E.compare_streams(oracle, got, want2, "C2 packed payload")
    del got
    for name, t in weights.items():                         # back to the first values: the replay must follow
        t.copy_(first[name])
    got, _ = _sync_to_host(packed)
    E.compare_streams(oracle, got, want, "C2 packed payload replayed")


def _experts(key):
    experts = W.MOE_CONFIGS[key]["shape"][1]
    cap = os.environ.get("MQ_WHOLE_CONFIG_EXPERTS", "")
    return min(experts, int(cap)) if cap else experts


@pytest.mark.parametrize("key,fmt", [("C3", "mxfp8"), ("C4", "int4_g128"), ("C5a", "nvfp4")])
def test_moe_layer_sync_every_tensor(oracle, key, fmt):
    conf = W.MOE_CONFIGS[key]
    _, _, ffn, hidden = conf["shape"]
    experts = _experts(key)
    args, weights, elems = W.moe_megatron(_gen(3001), layers=1, experts=experts, ffn=ffn, hidden=hidden, dist=conf["dist"])
    basenames = W.int4_packed_basenames(1, experts) if fmt == "int4_g128" else None
    make = lambda shape, gen: W.device_expert_tensor(shape, gen, conf["dist"])
    upd = WeightUpdater(args, weights_getter=lambda: weights, model_name=conf["model_name"], quantization_config=conf["cfg"],
                        send_bucket=None, packed_weight_basenames=basenames)
    want = E.expected_moe(oracle, fmt, args, _host(weights), basenames)
    got, buckets = _sync_to_host(upd)
    assert upd._plan is not None and upd._plan.replayable
    stats = E.compare_streams(oracle, got, want, f"{key} recorded")
    per_tensor = {"mxfp8": 2, "int4_g128": 3, "nvfp4": 3}[fmt]
    assert stats["tensors"] == experts * 3 * per_tensor
    del got
    # two replays on changed weights: for NVFP4 the first one runs with the amax carried over and every amax moved,
    # the second (same weights again) with none moved
    _refill(weights, 3002, make)
    want = E.expected_moe(oracle, fmt, args, _host(weights), basenames)
    for round_ in range(2):
        got, buckets2 = _sync_to_host(upd)
        assert buckets2 == buckets
        E.compare_streams(oracle, got, want, f"{key} replay {round_} after an in-place change")
        del got
