"""The C-ABI libraries load and export every symbol their headers declare (no GPU needed): libmiles_quant.so for
include/miles_quant.h, and libmq_probes.so -- self-tests and streaming probes, not part of the product -- for
include/miles_quant_probes.h."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols(header="miles_quant.h", prefix="mq_"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = _declared_symbols()
    for required in ["mq_fp8_block_quant", "mq_fp8_blockwise_cast", "mq_fp8_block_dequant", "mq_mxfp8_quant",
                     "mq_int4_group_quant_pack", "mq_int4_fake_quant", "mq_nvfp4_amax", "mq_nvfp4_quant"]:
        assert required in syms


def test_library_exports_every_declared_symbol():
    from miles_amd import _lib

    if not os.path.exists(_lib.lib_path()):
        pytest.fail(f"{_lib.lib_path()} not built: run `python -m miles_amd.build`")
    lib = ctypes.CDLL(_lib.lib_path())
    missing = [s for s in _declared_symbols() if not hasattr(lib, s)]
    assert not missing, f"declared in miles_quant.h but not exported: {missing}"
    assert _lib.load().mq_version() == 1
    # the ctypes signature table covers every declared compute entry point
    declared = set(_declared_symbols()) - {"mq_version", "mq_last_error"}
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)


def test_probes_library_exports_its_header_and_the_product_library_holds_none_of_it():
    from miles_amd import _lib, _probes

    if not os.path.exists(_probes.lib_path()):
        pytest.fail(f"{_probes.lib_path()} not built: run `python -m miles_amd.build`")
    declared = _declared_symbols("miles_quant_probes.h", "mqp_")
    lib = ctypes.CDLL(_probes.lib_path())
    assert declared and not [s for s in declared if not hasattr(lib, s)]
    assert set(declared) - {"mqp_last_error"} == set(_probes.SIGNATURES)
    product = ctypes.CDLL(_lib.lib_path())
    leaked = [s for s in declared + ["mq_selftest_convert", "mq_selftest_reciprocal", "mq_stream_probe", "mq_copy_bytes"]
              if hasattr(product, s)]
    assert not leaked, f"measurement scaffolding exported by the product library: {leaked}"
    assert not [s for s in _declared_symbols() if s.startswith("mqp_")]


def test_wrappers_refuse_cpu_tensors():
    import torch

    from miles_amd import _lib
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8
    from miles_amd.utils.mxfp8 import mxfp8_quantize
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d

    w = torch.zeros(32, 64, dtype=torch.bfloat16)
    for fn, args in [(block_fp8, (w, [128, 128])), (fp8_blockwise_cast, (w,)), (mxfp8_quantize, (w,)),
                     (nvfp4_quantize_1d, (w,))]:
        with pytest.raises(_lib.MilesQuantError, match="GPU"):
            fn(*args)


def test_python_constants_match_the_header():
    """Job kinds, flags and record sizes are written down twice (C header, ctypes side): they must agree."""
    from miles_amd import _lib
    from miles_amd.tools.convert_hf_to_fp8 import _AMAX_RECORD_WORDS
    from miles_amd.utils.nvfp4 import AMAX_RECORD_WORDS

    text = open(os.path.join(ROOT, "include", "miles_quant.h")).read()
    enums = {name: int(value) for name, value in re.findall(r"\b(MQ_[A-Z0-9_]+)\s*=\s*(\d+)", text)}
    defines = {name: value for name, value in re.findall(r"#define\s+(MQ_[A-Z0-9_]+)\s+(\S.*)", text)}
    kinds = {k[len("MQ_JOB_"):]: v for k, v in enums.items() if k.startswith("MQ_JOB_")}
    assert kinds and all(getattr(_lib, "JOB_" + k) == v for k, v in kinds.items())
    assert len(kinds) == len({getattr(_lib, n) for n in dir(_lib) if n.startswith("JOB_")})
    for name in ("NVFP4_4OVER6", "NVFP4_ERR_MSE", "NVFP4_ERR_FP16", "NVFP4_CARRY_AMAX"):
        assert getattr(_lib, name) == enums["MQ_" + name]
    assert _lib.MAX_GROUP == int(defines["MQ_MAX_GROUP"])
    assert (_lib.TABLE_ENTRY_BYTES, _lib.TABLE_GROUP) == (int(defines["MQ_JOB_TABLE_ENTRY_BYTES"]), int(defines["MQ_TABLE_GROUP"]))
    words = int(defines["MQ_NVFP4_SECTION_WORDS"]) * (int(defines["MQ_NVFP4_SECTIONS"]) + 1)
    assert AMAX_RECORD_WORDS == _AMAX_RECORD_WORDS == words
    amax_word = int(defines["MQ_NVFP4_SECTION_WORDS"]) * int(defines["MQ_NVFP4_SECTIONS"])
    assert defines["MQ_NVFP4_RECORD_REDO_WORD"] == "(MQ_NVFP4_RECORD_AMAX_WORD + 4)"
    assert defines["MQ_NVFP4_RECORD_VOLATILE_WORD"] == "(MQ_NVFP4_RECORD_AMAX_WORD + 5)"
    assert (_lib.RECORD_AMAX_WORD, _lib.RECORD_REDO_WORD, _lib.RECORD_VOLATILE_WORD) == (amax_word, amax_word + 4, amax_word + 5)
    assert (_lib.MQ_BF16, _lib.MQ_F16, _lib.MQ_F32) == (enums["MQ_BF16"], enums["MQ_F16"], enums["MQ_F32"])
