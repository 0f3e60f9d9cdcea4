"""CPU-only checks of the C-ABI boundary: libq8_hip.so loads, exports every function include/q8_hip.h
declares, the ctypes signatures cover them all, and argument validation (which runs before any HIP call)
reports errors through status codes and q8_last_error()."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "q8_hip.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(q8_[a-z0-9_]+)\s*\(", text)))


def test_header_functions_are_exported_and_bound():
    from q8_kernels_amd import _lib
    names = _declared_functions()
    assert "q8_gemm" in names and "q8_attn_fwd" in names and "q8_quant_rows" in names and len(names) >= 10
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), "libq8_hip.so does not export %s" % n
        assert n in _lib.SIGNATURES, "no ctypes signature for %s" % n
    for n in _lib.SIGNATURES:
        assert n in names, "%s is bound but not declared in include/q8_hip.h" % n


def test_header_enums_match_python_constants():
    from q8_kernels_amd import _lib
    text = open(HEADER).read()
    for name in ("Q8_I8", "Q8_E4M3", "Q8_BF16", "Q8_F16", "Q8_F32", "Q8_QUANT_RNE", "Q8_QUANT_SCALE_DIV",
                 "Q8_V_DS", "Q8_V_SD", "Q8_ATTN_SUM_ROUNDED_P", "Q8_ATTN_P_UNIT_RANGE", "Q8_ATTN_O_TOKEN_MAJOR"):
        m = re.search(r"\b%s\s*=\s*(-?\d+)" % name, text)
        assert m, name
        assert int(m.group(1)) == getattr(_lib, name), name


def test_strerror_and_argument_validation_without_gpu():
    from q8_kernels_amd import _lib
    L = _lib.lib()
    assert L.q8_strerror(0) == b"ok"
    assert b"shape" in L.q8_strerror(-3)
    # null pointers, bad dims, bad dtypes, bad alignment: rejected before anything touches the device
    assert L.q8_quant_rows(None, _lib.Q8_BF16, None, _lib.Q8_I8, None, 4, 64, 64, 0, None) == -1
    assert L.q8_quant_rows(16, _lib.Q8_BF16, 16, _lib.Q8_I8, 16, 4, 12, 12, 0, None) == -3
    assert b"multiple of 8" in L.q8_last_error()
    assert L.q8_quant_rows(16, _lib.Q8_BF16, 16, _lib.Q8_BF16, 16, 4, 64, 64, 0, None) == -2
    assert L.q8_quant_rows(16, _lib.Q8_BF16, 16, _lib.Q8_I8, 16, 4, 64, 64, 64, None) == -6
    assert L.q8_quant_rows(8, _lib.Q8_BF16, 16, _lib.Q8_I8, 16, 4, 64, 64, 0, None) == -4
    assert L.q8_fht(16, _lib.Q8_F32, 16, _lib.Q8_BF16, 4, 64, 1.0, None) == -2
    assert L.q8_fht(16, _lib.Q8_BF16, 16, _lib.Q8_BF16, 4, 65536, 1.0, None) == -3
    assert L.q8_rope(16, _lib.Q8_BF16, None, None, 16, _lib.Q8_BF16, 4, 64, None) == -1
    assert L.q8_gemm(16, 16, None, 16, 16, 16, 1, 1, 8, 8, 24, _lib.Q8_I8, _lib.Q8_BF16, 0, None) == -3
    assert L.q8_gemm(16, 16, None, 16, 16, 16, 2, 3, 8, 8, 32, _lib.Q8_I8, _lib.Q8_BF16, 0, None) == -3
    assert L.q8_gemm(16, 16, None, 16, 16, 16, 1, 1, 8, 8, 32, _lib.Q8_BF16, _lib.Q8_BF16, 0, None) == -2
    assert L.q8_gemm(16, 16, None, None, 16, 16, 1, 1, 8, 8, 32, _lib.Q8_I8, _lib.Q8_BF16, 0, None) == -1
    assert L.q8_attn_fwd(16, 16, 16, 16, None, None, None, None, 1, 1, 16, 16, 128, 0, 16, 0.125, _lib.Q8_BF16, 0, None) == -3
    assert b"head dim" in L.q8_last_error()
    assert L.q8_attn_fwd(16, 16, 16, 16, None, 16, None, None, 1, 1, 16, 16, 64, 0, 16, 0.125, _lib.Q8_BF16, 0, None) == -1
    assert L.q8_attn_fwd(16, 16, 16, 16, None, None, None, None, 1, 1, 16, 16, 64, 0, 16, 0.125, _lib.Q8_F16, 0, None) == -2
    with pytest.raises(_lib.Q8Error):
        _lib.check(-3)


def test_python_wrappers_refuse_cpu_tensors():
    import torch
    from q8_kernels_amd import _C
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        _C.tokenwise_quant(x)
    with pytest.raises(RuntimeError):
        _C.fast_hadamard_transform(x, 1.0)
    with pytest.raises(RuntimeError):
        _C.rms_norm(x)
    a = torch.zeros(16, 32, dtype=torch.int8)
    with pytest.raises(RuntimeError):
        _C.q8_mm(a, a, torch.ones(16), torch.ones(16), False, torch.bfloat16)


def test_functional_asserts_match_reference_contract():
    """dtype / scale pairing rules of the reference wrappers (functional/linear.py:25-28,141-145) fire on CPU tensors
    before any kernel is reached."""
    import torch
    from q8_kernels_amd.functional.linear import fp8_linear, q8_linear
    a16 = torch.zeros(4, 32, dtype=torch.bfloat16)
    a8 = torch.zeros(4, 32, dtype=torch.int8)
    with pytest.raises(AssertionError):
        q8_linear(a8, a8)  # int8 operands need scales
    with pytest.raises(AssertionError):
        q8_linear(a16, a16, scale_a=torch.ones(4))  # 16-bit operands forbid them
    with pytest.raises(AssertionError):
        q8_linear(a16, torch.zeros(4, 16, dtype=torch.bfloat16))  # K mismatch
    with pytest.raises(AssertionError):
        q8_linear(a16, a16, bias=torch.zeros(4, dtype=torch.bfloat16))  # bias must be fp32
    with pytest.raises(AssertionError):
        fp8_linear(a16, a16)  # out_dtype must be 16-bit
    with pytest.raises(AssertionError):
        fp8_linear(a16, a16, out_dtype=torch.float8_e4m3fn)


def test_weight_converter_key_mapping():
    from q8_kernels_amd.utils import converted_key
    p = "transformer_blocks.3."
    assert converted_key("proj_in.weight") == ("proj_in.weight", "keep")
    assert converted_key(p + "scale_shift_table") == (p + "scale_shift_table", "keep")
    assert converted_key(p + "attn1.to_out.0.weight") == (p + "attn1.to_out.weight", "quantize")
    assert converted_key(p + "attn1.to_out.0.bias") == (p + "attn1.to_out.bias", "fp32")
    assert converted_key(p + "attn2.q_norm.weight") == (p + "attn2.q_norm.weight", "fp32")
    assert converted_key(p + "attn2.to_k.weight") == (p + "attn2.to_k.weight", "quantize")
    assert converted_key(p + "ff.net.0.proj.weight") == (p + "ff.act.proj.weight", "quantize")
    assert converted_key(p + "ff.net.2.bias") == (p + "ff.proj_down.bias", "fp32")
