"""The Four Over Six quantizer decides most blocks from a cheaper error estimate (`nv_block_error_estimate` in
miles_amd/csrc/mq_nvfp4.hip) and computes the reference's exact error sums only for a wavefront that holds a block too
close to call.  This file checks the claim behind that on the CPU, in numpy's fp32 arithmetic, over millions of random
blocks: whenever the two estimates differ by more than the kernel's guard, the exact sums -- the reference's
`nvfp4_qdq.py:893-953` terms, restated as the oracle states them -- compare the same way; and the guard is rarely needed.
Both error measures the estimate serves are covered: the sum of absolute differences (default) and of squares (MSE).
"""

import numpy as np
import pytest
import torch

F32 = np.float32
E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=F32)
FLT_MAX = np.finfo(F32).max


def _bf16(x):
    return torch.from_numpy(np.ascontiguousarray(x, dtype=F32)).to(torch.bfloat16).float().numpy()


def _blocks(n, seed, dtype_bits):
    """n blocks of 16 values (bf16 or fp16 valued) with magnitudes over many binades, and a tensor amax >= every block's."""
    g = np.random.default_rng(seed)
    x = g.standard_normal((n, 16)).astype(F32) * np.exp(g.standard_normal((n, 1)) * 3.0).astype(F32)
    x *= (g.random((n, 16)) > 0.05)                           # some zeros
    if dtype_bits == 16:
        x = torch.from_numpy(x).clamp(-6e4, 6e4).to(torch.float16).float().numpy()
    else:
        x = _bf16(x)
    bmax = np.abs(x).max(axis=1)
    grow = np.exp2(g.integers(0, 9, n)).astype(F32) * (1 + g.integers(0, 8, n).astype(F32) / 8)
    amax = bmax * grow
    amax = torch.from_numpy(amax).to(torch.float16 if dtype_bits == 16 else torch.bfloat16).float().numpy()
    amax = np.where(np.isfinite(amax), amax, bmax)
    amax = np.maximum(amax, bmax)                             # the tensor amax is at least the block's
    keep = bmax > 0
    return x[keep], bmax[keep], amax[keep]


def _seq_sum(terms):
    total = np.zeros(terms.shape[0], dtype=F32)
    for j in range(terms.shape[1]):
        total = (total + terms[:, j]).astype(F32)
    return total


def _term(diff, squared):
    with np.errstate(over="ignore", under="ignore"):
        return (diff * diff).astype(F32) if squared else np.abs(diff)


def _candidate(oracle, x, s_hp, s_dec):
    sc = oracle.f32_to_e4m3fn(torch.from_numpy(np.minimum(s_hp, F32(448.0))), sat=True)
    s_f = sc.view(torch.float8_e4m3fn).float().numpy()
    with np.errstate(divide="ignore", over="ignore"):
        inv = np.minimum(F32(1.0) / (s_f * s_dec).astype(F32), FLT_MAX).astype(F32)
    codes = oracle.f32_to_e2m1(torch.from_numpy((x * inv[:, None]).astype(F32))).numpy()
    q = E2M1[codes & 7] * np.where(codes & 8, F32(-1.0), F32(1.0)).astype(F32)
    return s_f, q.astype(F32)


@pytest.mark.parametrize("squared", [False, True], ids=["mae", "mse"])
@pytest.mark.parametrize("e4m3_max", [448, 256])
@pytest.mark.parametrize("dtype_bits", [8, 16])       # bf16 (8 significant bits) and fp16 (11) values
def test_the_estimate_decides_as_the_exact_error_sums_do(oracle, e4m3_max, dtype_bits, squared):
    x, bmax, amax = _blocks(1_500_000, seed=e4m3_max + dtype_bits + 1000 * squared, dtype_bits=dtype_bits)
    denom = F32(6 * e4m3_max)
    with np.errstate(over="ignore"):
        enc = np.minimum(denom / amax, FLT_MAX).astype(F32)
    s_dec = (F32(1.0) / enc).astype(F32)
    s6_hp = ((bmax / F32(6.0)).astype(F32) * enc).astype(F32)
    s4_hp = (s6_hp * F32(1.5)).astype(F32)
    exact, estimate, slope, scale = {}, {}, {}, {}
    for name, s_hp in (("4", s4_hp), ("6", s6_hp)):
        s_f, q = _candidate(oracle, x, s_hp, s_dec)
        # the reference's terms: RN(RN(RN(q * s) * amax) / denom) - x, summed in element order in fp32
        dq = (((q * s_f[:, None]).astype(F32) * amax[:, None]).astype(F32) / denom).astype(F32)
        exact[name] = _seq_sum(_term((dq - x).astype(F32), squared))
        # the kernel's estimate: a = RN(s * amax / denom), terms |fma(q, a, -x)| (one rounding: taken through float64,
        # where q * a - x is exact)
        a = ((s_f * amax).astype(F32) / denom).astype(F32)
        fma = (q.astype(np.float64) * a[:, None].astype(np.float64) - x.astype(np.float64)).astype(F32)
        estimate[name] = _seq_sum(_term(fma, squared))
        slope[name] = a
        scale[name] = s_f
    if squared:
        # the hardware square root may come out one unit in the last place low: taken two low here
        with np.errstate(over="ignore", invalid="ignore"):
            root = {k: (np.sqrt((estimate[k] + F32(2.0 ** -100)).astype(F32)) * F32(1 - 2.0 ** -22)).astype(F32)
                    for k in "46"}
            e = {k: (F32(2.0 ** -24) * (F32(25.0) * slope[k] + F32(2.0) * bmax)).astype(F32) for k in "46"}
            guard = (F32(17.0) * (e["4"] * root["4"] + e["6"] * root["6"]) + F32(33.0) * (e["4"] * e["4"] + e["6"] * e["6"])
                     + F32(2.0 ** -17) * (estimate["4"] + estimate["6"]) + F32(2.0 ** -100)).astype(F32)
    else:
        guard = (F32(2.0 ** -19) * (F32(32.0) * (slope["4"] + slope["6"]) + F32(4.0) * bmax
                                    + F32(4.0) * (estimate["4"] + estimate["6"]))).astype(F32)
    # (two candidates with one scale byte are the same candidate: the block that holds the tensor's maximum)
    decided = (np.abs((estimate["4"] - estimate["6"]).astype(F32)) > guard) | (scale["4"] == scale["6"])
    pick4_exact = exact["4"] < exact["6"]
    pick4_estimate = estimate["4"] < estimate["6"]
    wrong = decided & (pick4_exact != pick4_estimate)
    assert not wrong.any(), f"{int(wrong.sum())} decided blocks pick another candidate than the exact sums"
    # the guard is rarely needed, both candidates win, and without it the estimate alone would not be exact
    assert (~decided).mean() < 2e-3, float((~decided).mean())
    assert 0.05 < pick4_exact.mean() < 0.95
    # half a guard would already be unsound somewhere, or at least the estimates differ from the exact sums in places
    assert (estimate["4"] != exact["4"]).any() or (estimate["6"] != exact["6"]).any()
