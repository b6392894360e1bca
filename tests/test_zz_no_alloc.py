"""mq_fp8_scaled_quant_static -- the entry point that allocates nothing -- against mq_fp8_scaled_quant.

Both are called with raw pointers through the C ABI.  The static form keeps its amax workspace in a device array
of the library, shared by every call on the GPU, so each case makes two calls in a row, the second on a smaller
input: whatever the first call left in the workspace must not reach the second call's result.  Bytes of codes and
scales must be identical to the existing entry point's (which the parity tests hold to the CPU oracle).
"""

import pytest
import torch

from miles_amd import workloads as W

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _floor(dtype):
    return float(torch.tensor(1e-12, dtype=dtype).float())     # clamp(min=1e-12) acts in the weight dtype


def _both(lib, w, per_channel):
    """(codes, scale) of the existing entry point and of the static one for the same input."""
    from miles_amd import _lib

    M, K = w.shape
    code = _lib.DTYPE_CODE[w.dtype]
    outs = []
    for static in (False, True):
        q = torch.full((M, K), 0x55, dtype=torch.uint8, device=DEV)
        s = torch.full((M if per_channel else 1,), -1.0, dtype=torch.float32, device=DEV)
        if static:
            rc = lib.mq_fp8_scaled_quant_static(w.data_ptr(), code, w.stride(0), q.data_ptr(), s.data_ptr(), M, K,
                                                int(per_channel), _floor(w.dtype), None)
        else:
            ws = torch.empty(max(M, 1), dtype=torch.int32, device=DEV)
            rc = lib.mq_fp8_scaled_quant(w.data_ptr(), code, w.stride(0), q.data_ptr(), s.data_ptr(), ws.data_ptr(), M, K,
                                         int(per_channel), _floor(w.dtype), None)
        assert rc == 0, lib.mq_last_error()
        outs.append((q, s))
    torch.cuda.synchronize()
    return outs


# (dtype, per_channel, first shape, second smaller shape): bf16 per tensor takes the flat two-pass kernels (one
# workspace word, cleared by the call), fp32 / fp16 and K > 16384 take the row kernels (one word per row)
CASES = [
    (torch.bfloat16, False, (512, 1024), (96, 256)),
    (torch.bfloat16, True, (300, 512), (40, 128)),
    (torch.bfloat16, True, (64, 20480), (8, 16392)),
    (torch.float32, True, (257, 384), (31, 72)),
    (torch.float16, False, (200, 136), (3, 40)),
    (torch.float32, False, (128, 1000), (16, 24)),
]


@pytest.mark.parametrize("dtype,per_channel,first,second", CASES)
def test_static_workspace_matches_the_workspace_argument(dtype, per_channel, first, second):
    from miles_amd import _lib

    lib = _lib.load()
    # the first input is much larger in magnitude than the second: a stale amax would flatten the second call's codes
    big = (W.gaussian_outliers(first, std=3.0, p_outlier=0.01, gain=20.0, seed=11).float()).to(dtype).to(DEV)
    small = (W.gaussian_outliers(second, std=0.01, p_outlier=0.0, gain=1.0, seed=12).float()).to(dtype).to(DEV)
    for w, what in ((big, "first call"), (small, "second, smaller call")):
        (q_ref, s_ref), (q_st, s_st) = _both(lib, w, per_channel)
        assert torch.equal(s_st.cpu().view(torch.int32), s_ref.cpu().view(torch.int32)), f"{what}: scales differ"
        assert torch.equal(q_st.cpu(), q_ref.cpu()), f"{what}: codes differ"
        assert (q_st.cpu() != 0x55).any()


def test_static_entry_point_allocates_nothing_and_checks_its_limit():
    from miles_amd import _lib

    lib = _lib.load()
    w = torch.randn(64, 256, device=DEV).to(torch.bfloat16)
    q = torch.empty((64, 256), dtype=torch.uint8, device=DEV)
    s = torch.empty(64, dtype=torch.float32, device=DEV)
    args = (w.data_ptr(), 0, 256, q.data_ptr(), s.data_ptr(), 64, 256)
    assert lib.mq_fp8_scaled_quant_static(*args, 0, _floor(w.dtype), None) == 0      # address lookup done
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for per_channel in (0, 1, 0):
        assert lib.mq_fp8_scaled_quant_static(*args, per_channel, _floor(w.dtype), None) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, "device memory was allocated by the static entry point"
    # beyond the static array: refused with a message, nothing launched
    limit = 262144
    assert lib.mq_fp8_scaled_quant_static(w.data_ptr(), 0, 8, q.data_ptr(), s.data_ptr(), limit + 1, 8, 1,
                                          _floor(w.dtype), None) == -1
    assert b"262144" in lib.mq_last_error()
    # an empty tensor is fine (and is the call to make before a graph capture)
    assert lib.mq_fp8_scaled_quant_static(None, 0, 0, None, None, 0, 0, 1, _floor(w.dtype), None) == 0


def test_static_calls_in_flight_on_two_streams_take_different_words():
    """Consecutive calls take consecutive pieces of the static array, so per-tensor calls queued on two streams at once
    (every one of them used to clear, fill and read word 0) do not disturb each other's amax."""
    from miles_amd import _lib

    lib = _lib.load()
    big = (W.gaussian_outliers((4096, 4096), std=3.0, p_outlier=0.01, gain=20.0, seed=21).float()).to(torch.bfloat16).to(DEV)
    small = (W.gaussian_outliers((4096, 4096), std=0.01, p_outlier=0.0, gain=1.0, seed=22).float()).to(torch.bfloat16).to(DEV)
    want = {}
    for name, w in (("big", big), ("small", small)):
        (q_ref, s_ref), _ = _both(lib, w, False)
        want[name] = (q_ref.cpu(), s_ref.cpu())
    streams = [torch.cuda.Stream(device=DEV), torch.cuda.Stream(device=DEV)]
    outs = []
    torch.cuda.synchronize()
    for rep in range(8):                                   # sixteen calls queued without a wait in between
        for (name, w), stream in zip((("big", big), ("small", small)), streams):
            q = torch.full((4096, 4096), 0x55, dtype=torch.uint8, device=DEV)
            s = torch.full((1,), -1.0, dtype=torch.float32, device=DEV)
            outs.append((name, q, s))
    torch.cuda.synchronize()
    for i, (name, q, s) in enumerate(outs):
        w = big if name == "big" else small
        rc = lib.mq_fp8_scaled_quant_static(w.data_ptr(), 0, w.stride(0), q.data_ptr(), s.data_ptr(), 4096, 4096, 0,
                                            _floor(w.dtype), streams[i % 2].cuda_stream)
        assert rc == 0, lib.mq_last_error()
    torch.cuda.synchronize()
    for i, (name, q, s) in enumerate(outs):
        assert torch.equal(s.cpu().view(torch.int32), want[name][1].view(torch.int32)), f"call {i} ({name}): scale differs"
        assert torch.equal(q.cpu(), want[name][0]), f"call {i} ({name}): codes differ"
