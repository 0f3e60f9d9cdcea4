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
                 "Q8_V_DS", "Q8_V_SD", "Q8_ATTN_SUM_ROUNDED_P", "Q8_ATTN_P_UNIT_RANGE", "Q8_ATTN_O_TOKEN_MAJOR", "Q8_ATTN_LAZY_MAX",
                 "Q8_PREP_FHT", "Q8_PREP_PAIR_TABLES", "Q8_PREP_SHARED_TABLES",
                 "Q8_GEMM_KERNEL_PIPE256", "Q8_GEMM_KERNEL_TILE128", "Q8_GEMM_KERNEL_TILE64", "Q8_GEMM_KERNEL_PERSIST256",
                 "Q8_GEMM_KERNEL_PERSIST192", "Q8_GEMM_KERNEL_RESIDUAL"):
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
    # more rows than one launch can cover (2^31 - 1 workgroups): refused, not truncated
    assert L.q8_quant_rows(16, _lib.Q8_BF16, 16, _lib.Q8_I8, 16, 1 << 40, 32768, 32768, 0, None) == -3
    assert b"too many rows" in L.q8_last_error()
    assert L.q8_fht(16, _lib.Q8_BF16, 16, _lib.Q8_BF16, 1 << 40, 32768, 1.0, None) == -3
    assert b"too many rows" in L.q8_last_error()
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


def test_argument_validation_of_the_fused_and_elementwise_entry_points():
    from q8_kernels_amd import _lib
    L = _lib.lib()
    B16, E4, I8, F32 = _lib.Q8_BF16, _lib.Q8_E4M3, _lib.Q8_I8, _lib.Q8_F32
    # rows == 0 is a no-op before anything else is looked at
    assert L.q8_fma(None, E4, None, F32, None, F32, None, E4, 0, 64, 1, 1, 0.0, None) == 0
    assert L.q8_fht_quant_rows(None, B16, None, I8, None, 0, 64, 1.0, B16, 0, None) == 0
    assert L.q8_attn_prep_qk(None, 512, None, None, None, None, None, 0, 5, 8, 64, 1, 1.0, B16, None) == 0
    assert L.q8_fma(None, E4, 16, F32, 16, F32, 16, E4, 4, 64, 1, 1, 0.0, None) == -1
    assert L.q8_fma(16, E4, 16, F32, 16, F32, 16, E4, 4, 60, 1, 1, 0.0, None) == -3
    assert L.q8_fma(16, E4, 16, F32, 16, F32, 16, E4, 4, 64, 0, 1, 0.0, None) == -3
    assert L.q8_fma(16, F32, 16, F32, 16, F32, 16, E4, 4, 64, 1, 1, 0.0, None) == -2
    assert L.q8_fma(16, B16, 8, B16, 16, F32, 16, E4, 4, 64, 1, 1, 0.0, None) == -4
    assert L.q8_gelu(16, B16, 16, B16, 12, None) == -3
    # q8_adaln_rows(table, timestep, rows, params, tokens, dim, stream)
    assert L.q8_adaln_rows(None, None, None, 6, 0, 2048, None) == 0        # no tokens
    assert L.q8_adaln_rows(16, 16, None, 6, 2, 2048, None) == -1
    assert L.q8_adaln_rows(16, 16, 16, 6, 2, 2044, None) == -3             # dim % 8
    assert L.q8_adaln_rows(16, 16, 16, 0, 2, 2048, None) == -3
    assert L.q8_adaln_rows(16, 8, 16, 6, 2, 2048, None) == -4
    assert L.q8_gelu_backward(16, B16, None, B16, 16, B16, 64, None) == -1
    assert L.q8_rope_backward(16, B16, None, 16, 16, B16, 4, 64, None) == -1
    assert L.q8_rmsnorm_backward(16, B16, None, 16, B16, None, 16, B16, 4, 64, None) == -1
    assert L.q8_rmsnorm_backward(16, B16, 16, 16, F32, None, 16, B16, 4, 64, None) == -2
    assert L.q8_fht_quant_rows(16, B16, 16, B16, 16, 4, 64, 1.0, B16, 0, None) == -2
    assert L.q8_fht_quant_rows(16, B16, 16, I8, 16, 4, 64, 1.0, E4, 0, None) == -2   # e4m3 intermediate needs an e4m3 input
    assert L.q8_rmsnorm_quant_rows(16, B16, 8, 16, I8, 16, None, 4, 64, 0.0, B16, 0, None) == -4
    assert L.q8_attn_prep_qk(16, 512, None, None, None, 16, None, 1, 5, 8, 32, 1, 1.0, B16, None) == -3
    assert b"head dim" in L.q8_last_error()
    assert L.q8_attn_prep_qk(16, 512, None, None, None, 16, None, 1, 5, 12, 64, 1, 1.0, B16, None) == -3   # H * D = 768
    assert L.q8_attn_prep_qk(16, 500, None, None, None, 16, None, 1, 5, 8, 64, 1, 1.0, B16, None) == -3    # stride < H * D
    assert L.q8_attn_prep_qk(16, 512, None, 16, None, 16, None, 1, 5, 8, 64, 1, 1.0, B16, None) == -1      # cos without sin
    assert L.q8_attn_prep_qk(16, 512, None, 16, 16, 16, None, 1, 5, 8, 64, 8, 1.0, B16, None) == -6        # unknown flag bit
    assert L.q8_attn_prep_qk(16, 512, None, None, None, 16, None, 1, 5, 8, 64, 1 | _lib.Q8_PREP_PAIR_TABLES, 1.0, B16, None) == -6  # table flag, no tables
    assert L.q8_attn_prep_qk_pair(16, 512, 16, 512, None, None, None, None, 16, None, 16, None, 1, 5, 8, 64,
                                  _lib.Q8_PREP_SHARED_TABLES, 1.0, B16, None) == -6
    assert L.q8_attn_prep_qk_pair(16, 512, None, 512, None, None, None, None, 16, None, 16, None, 1, 5, 8, 64, 1, 1.0, B16, None) == -1
    assert L.q8_attn_prep_qk_pair(16, 512, 16, 512, None, None, None, None, 16, 16, 16, None, 1, 5, 8, 64, 1, 1.0, B16, None) == -1
    # q8_attn_prep_qkv(xq, sq, xk, sk, xv, sv, nwq, nwk, cos, sin, cq, scq, ck, sck, cv, scv, B, S, H, D, fht, scale, mid, stream)
    assert L.q8_attn_prep_qkv(None, 512, None, 512, None, 512, None, None, None, None, None, None, None, None, None, None,
                              0, 5, 8, 64, 1, 1.0, B16, None) == -1                                  # no V at all
    assert L.q8_attn_prep_qkv(16, 512, 16, 512, 16, 512, None, None, None, None, 16, None, 16, None, None, None,
                              1, 5, 8, 64, 1, 1.0, B16, None) == -1                                  # V given, its codes not
    assert L.q8_attn_prep_qkv(16, 512, 16, 512, 16, 500, None, None, None, None, 16, None, 16, None, 16, None,
                              1, 5, 8, 64, 1, 1.0, B16, None) == -3                                  # V stride < H * D
    assert L.q8_attn_prep_qkv(16, 512, 16, 512, 16, 512, None, None, None, None, 16, 16, 16, 16, 16, None,
                              1, 5, 8, 64, 1, 1.0, B16, None) == -1                                  # scales for q, k but not v
    assert L.q8_attn_prep_qkv(16, 512, 16, 512, 8, 512, None, None, None, None, 16, None, 16, None, 16, None,
                              1, 5, 8, 64, 1, 1.0, B16, None) == -4                                  # V not 16-byte aligned
    assert L.q8_attn_prep_qkv(16, 512, 16, 512, 16, 512, None, None, None, None, 16, None, 16, None, 16, None,
                              0, 5, 8, 64, 1, 1.0, B16, None) == 0                                   # no tokens: nothing to do
    # q8_attn_prep_kv(xk, sk, xv, sv, nwk, cos, sin, ck, sck, cv, scv, B, S, H, D, fht, scale, mid, stream)
    assert L.q8_attn_prep_kv(None, 512, None, 512, None, None, None, None, None, None, None, 0, 5, 8, 64, 1, 1.0, B16, None) == -1  # no V
    assert L.q8_attn_prep_kv(None, 512, 16, 512, None, None, None, None, None, None, None, 0, 5, 8, 64, 1, 1.0, B16, None) == 0    # no tokens
    assert L.q8_attn_prep_kv(16, 512, 16, 512, None, None, None, 16, None, None, None, 1, 5, 8, 64, 1, 1.0, B16, None) == -1       # no V codes
    assert L.q8_attn_prep_kv(16, 512, 16, 500, None, None, None, 16, None, 16, None, 1, 5, 8, 64, 1, 1.0, B16, None) == -3        # V stride
    assert L.q8_attn_prep_kv(16, 512, 16, 512, None, None, None, 16, 16, 16, None, 1, 5, 8, 64, 1, 1.0, B16, None) == -1          # scales of K only
    assert L.q8_attn_prep_v(16, 512, 16, None, 1, 5, 8, 64, 5, None) == -3                          # S_pad % 16
    assert L.q8_attn_prep_v(16, 512, 16, None, 1, 5, 8, 128, 16, None) == -3
    assert L.q8_gemm_residual(16, 16, None, 16, 16, None, 16, 1, 1, 8, 8, 384, I8, 0, None) == -1
    assert L.q8_gemm_residual(16, 16, None, 16, 16, 16, 16, 1, 1, 8, 8, 256, I8, 0, None) == -3     # K must exceed 256
    assert L.q8_gemm_residual(16, 16, None, 16, 16, 16, 16, 1, 1, 8, 12, 384, I8, 0, None) == -3    # N % 8
    # q8_gemm_gated_residual(A, B, bias, sa, sb, residual, gate, rows_per_gate, C, M, N, K, in_dtype, fuse_gelu, stream)
    assert L.q8_gemm_gated_residual(16, 16, None, 16, 16, 16, None, 768, 16, 1536, 8, 384, I8, 0, None) == -1    # no gate
    assert L.q8_gemm_gated_residual(16, 16, None, 16, 16, 16, 16, 100, 16, 1536, 8, 384, I8, 0, None) == -3      # rows per gate % 768
    assert b"768" in L.q8_last_error()
    assert L.q8_gemm_gated_residual(16, 16, None, 16, 16, 16, 8, 768, 16, 1536, 8, 384, I8, 0, None) == -4       # gate alignment
    assert L.q8_gemm_gated_residual(16, 16, None, 16, 16, 16, 16, 768, 16, 1536, 8, 256, I8, 0, None) == -3      # K must exceed 256
    assert L.q8_gemm_gated_residual(16, 16, None, 16, 16, 16, 16, 768, 16, 0, 8, 384, I8, 0, None) == 0          # no rows
    # q8_gemm_qkv(A, B, bias, sa, sb, C, v_codes, M, N, K, v_col0, tokens, v_fht_scale, in_dtype, stream)
    assert L.q8_gemm_qkv(16, 16, None, 16, 16, 16, None, 64, 768, 384, 512, 32, 0.0, I8, None) == -1     # no v_codes
    assert L.q8_gemm_qkv(16, 16, None, 16, 16, 16, 16, 64, 768, 384, 576, 32, 0.0, I8, None) == -3       # split off a tile boundary
    assert L.q8_gemm_qkv(16, 16, None, 16, 16, 16, 16, 64, 768, 384, 512, 48, 0.0, I8, None) == -3       # rows are not whole batch elements
    assert L.q8_gemm_qkv(16, 16, None, 16, 16, 16, 16, 64, 768, 256, 512, 32, 0.0, I8, None) == -3       # K must exceed 256
    assert L.q8_gemm_qkv(16, 16, None, 16, 16, 16, 8, 64, 768, 384, 512, 32, 0.0, I8, None) == -4        # v_codes alignment
    assert L.q8_gemm_qkv(16, 16, None, 16, 16, 16, 16, 64, 768, 384, 512, 32, -1.0, I8, None) == -3      # a negative Hadamard factor
    assert L.q8_gemm_qkv(16, 16, None, 16, 16, 16, 16, 0, 768, 384, 512, 32, 0.0, I8, None) == 0         # no rows
    assert L.q8_gemm_set_config(7) == -6
    assert L.q8_attn_set_config(5) == -6 and L.q8_attn_set_config(-1) == -6
    # q8_attn_fwd(q, k, v, o, kv_len, sq, sk, sv, B, H, M, N, D, v_layout, v_row_stride, scale, out_dtype, flags, stream)
    assert L.q8_attn_fwd(16, 16, 16, 16, None, None, None, None, 1, 1, 8, 8, 64, 2, 16, 0.125, B16, 0, None) == -3   # V layout 2
    assert L.q8_attn_fwd(16, 16, 16, 16, None, None, None, None, 1, 1, 8, 8, 64, _lib.Q8_V_DS, 8, 0.125, B16, 0, None) == -3  # V^T stride
    lazy_unit = _lib.Q8_ATTN_LAZY_MAX | _lib.Q8_ATTN_P_UNIT_RANGE   # the trailing maximum needs the head room above 2^5
    assert L.q8_attn_fwd(16, 16, 16, 16, None, None, None, None, 1, 1, 8, 8, 64, 0, 16, 0.125, B16, lazy_unit, None) == -6
    assert L.q8_attn_fwd(16, 16, 16, 16, None, None, None, None, 1, 1, 8, 8, 64, 0, 16, 0.125, B16, 16, None) == -6  # unknown flag
    # the row sum over rounded probabilities is defined for unit scales
    assert L.q8_attn_fwd(16, 16, 16, 16, None, 16, 16, 16, 1, 1, 8, 8, 64, 0, 16, 0.125, B16, _lib.Q8_ATTN_SUM_ROUNDED_P, None) == -6
    assert b"unit scales" in L.q8_last_error()
    assert L.q8_attn_set_config(1) == 0
    try:  # the 4 waves x 64 queries shape reads V^T only
        assert L.q8_attn_fwd(16, 16, 16, 16, None, None, None, None, 1, 1, 8, 8, 64, _lib.Q8_V_SD, 0, 0.125, B16, 0, None) == -6
    finally:
        assert L.q8_attn_set_config(0) == 0


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


def test_missing_library_is_an_error_not_a_fallback():
    """A fresh interpreter with the library path pointed at nothing: the loader (and with it every call that reaches
    it) raises the build hint, and no operator hands back a result for CPU tensors instead. What a machine without a
    GPU cannot show - an operator on a device tensor reaching the loader - is test_api_gpu.py's version of this."""
    import subprocess
    import sys
    code = (
        "import sys, torch\n"
        "sys.path.insert(0, %r)\n"
        "from q8_kernels_amd import _lib\n"
        "_lib.LIB_PATH = '/nonexistent/libq8_hip.so'\n"
        "from q8_kernels_amd import _C\n"
        "x = torch.zeros(4, 64, dtype=torch.bfloat16)\n"
        "for name, fn in (('loader', _lib.lib), ('device_info', _lib.device_info), ('quant_cpu', lambda: _C.tokenwise_quant(x, None))):\n"
        "    try:\n"
        "        fn()\n"
        "    except RuntimeError as e:\n"
        "        print(name, '|', e)\n"
        "    else:\n"
        "        print(name, '| RETURNED')\n" % ROOT)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    got = dict(line.split(" | ", 1) for line in r.stdout.strip().splitlines())
    assert "no fallback" in got["loader"] and "/nonexistent/libq8_hip.so" in got["loader"]
    assert "no fallback" in got["device_info"]
    assert "CUDA" in got["quant_cpu"] and "RETURNED" not in got["quant_cpu"]


def test_bench_refuses_more_than_one_gpu():
    """bench.py --gpus N with N > 1 exits with a message that says why (nothing here spans GPUs)."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and "--gpus 2" in r.stderr
    assert r.stdout.strip() == ""


def test_precompute_freqs_cis_matches_the_oracle_tables():
    """The package's own builder of the 3-D rotary tables against the oracle's restatement of
    q8_kernels/models/LTXVideo.py:85-148 (itself pinned by explicit loops over frequency and axis)."""
    import torch
    from oracle import q8_oracle as O
    from q8_kernels_amd.functional.rope import precompute_freqs_cis, video_index_grid
    grid = video_index_grid(3, 4, 5, batch=2)
    assert grid.shape == (2, 3, 60) and grid[0, :, 27].tolist() == [1.0, 1.0, 2.0]
    for dim in (2048, 256, 100):
        cos, sin = precompute_freqs_cis(grid, dim)
        want_cos, want_sin = O.ref_freqs_cis(grid, dim)
        assert cos.dtype == torch.float32 and cos.shape == (2, 60, dim)
        assert torch.allclose(cos, want_cos, atol=1e-6) and torch.allclose(sin, want_sin, atol=1e-6)
        assert torch.equal(cos[..., 0::2], cos[..., 1::2]) and torch.equal(sin[..., 0::2], sin[..., 1::2])
    # the benchmark's 16 x 16 x 24 grid: frame indices up to 15 over max_pos 20, where a product with the rounded reciprocal
    # of 20 differs from the reference's division by one ulp and the top frequency turns that into 2e-3 in the tables.
    # Bit equality with the oracle's division-based restatement.
    grid = video_index_grid(16, 16, 24, batch=1)
    cos, sin = precompute_freqs_cis(grid, 2048)
    want_cos, want_sin = O.ref_freqs_cis(grid, 2048)
    assert torch.equal(cos, want_cos) and torch.equal(sin, want_sin)
