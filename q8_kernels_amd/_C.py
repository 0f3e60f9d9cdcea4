"""Tensor-level entry points with the names, argument order and return shapes of the reference's four
pybind11 modules (q8_kernels_cuda.{gemm,quantizer,ops,flash_attention}._C), implemented on top of the
C ABI of libq8_hip.so. Outputs are allocated here with torch (as the reference's C++ glue does), inputs
are borrowed, launches go to the current torch stream of the input's device and do not synchronise.
"""
from typing import List, Optional

import torch

from . import _lib
from ._lib import Q8_BF16, Q8_E4M3, Q8_F16, Q8_F32, Q8_I8

_DT = {
    torch.int8: Q8_I8,
    torch.float8_e4m3fn: Q8_E4M3,
    torch.bfloat16: Q8_BF16,
    torch.float16: Q8_F16,
    torch.float32: Q8_F32,
}


def _dt(dtype, who):
    try:
        return _DT[dtype]
    except KeyError:
        raise RuntimeError("%s not implemented for type '%s'" % (who, dtype))


def _require_gpu(t, name):
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA (HIP) tensor" % name)


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _as_rows(x):
    """x.reshape(-1, dim) with unit last stride (csrc/quantizer/tokenwise_quant.cpp:79-82)."""
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) < x2.shape[1]):
        x2 = x2.contiguous()
    return x2


# ----------------------------------------------------------------------------- quantizer._C

def tokenwise_quant(x: torch.Tensor, out_type: Optional[torch.dtype] = None, *, round_half_even: bool = False,
                    scale_as_division: bool = False) -> List[torch.Tensor]:
    """csrc/quantizer/tokenwise_quant.cpp:74-111. Returns [codes(x.shape), scales(x.shape[:-1]) fp32].

    out_type None -> int8. The two keyword flags select the documented variants of the arithmetic
    (int8 round-half-even; stored scale absmax/QMAX); the defaults reproduce the reference.
    """
    _require_gpu(x, "x")
    shape = x.shape
    x2 = _as_rows(x)
    out_type = torch.int8 if out_type is None else out_type
    if out_type not in (torch.int8, torch.float8_e4m3fn):
        raise RuntimeError("tokenwise_quant not implemented for output type '%s'" % out_type)
    rows, dim = x2.shape
    out = torch.empty((rows, dim), dtype=out_type, device=x.device)
    scales = torch.empty((rows,), dtype=torch.float32, device=x.device)
    flags = (_lib.Q8_QUANT_RNE if round_half_even else 0) | (_lib.Q8_QUANT_SCALE_DIV if scale_as_division else 0)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_quant_rows(x2.data_ptr(), _dt(x2.dtype, "tokenwise_quant"), out.data_ptr(),
                                            _dt(out_type, "tokenwise_quant"), scales.data_ptr(), rows, dim,
                                            x2.stride(0) if rows > 1 else dim, flags, _stream(x)))
    return [out.reshape(shape), scales.reshape(shape[:-1])]


# ----------------------------------------------------------------------------- ops._C

def fast_hadamard_transform(x: torch.Tensor, scale: float, out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """csrc/fast_hadamard/fast_hadamard_transform.cpp:70-121. out_type None -> x.dtype."""
    if x.dtype not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError("fast_hadamard_transform: input must be bfloat16 or float8_e4m3fn")
    _require_gpu(x, "x")
    shape = x.shape
    dim_og = shape[-1]
    x2 = x.reshape(-1, dim_og)
    if dim_og % 8 != 0:
        if x2.dtype == torch.float8_e4m3fn:
            x2 = torch.nn.functional.pad(x2.view(torch.uint8), (0, 8 - dim_og % 8)).view(torch.float8_e4m3fn)
        else:
            x2 = torch.nn.functional.pad(x2, (0, 8 - dim_og % 8))
    x2 = x2.contiguous()
    rows, dim = x2.shape
    if dim > 32768:
        raise RuntimeError("fast_hadamard_transform only supports hidden dimension at most 32768 for now")
    out_type = x.dtype if out_type is None else out_type
    if out_type not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError("fast_hadamard_transform: output must be bfloat16 or float8_e4m3fn")
    out = torch.empty((rows, dim), dtype=out_type, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_fht(x2.data_ptr(), _DT[x2.dtype], out.data_ptr(), _DT[out_type], rows, dim,
                                     float(scale), _stream(x)))
    if dim_og % 8 != 0:
        out = out[:, :dim_og]
    return out.reshape(shape)


def rms_norm(x: torch.Tensor, weights: Optional[torch.Tensor] = None, out_type: Optional[torch.dtype] = None, *,
             eps: float = 0.0) -> List[torch.Tensor]:
    """csrc/ops/rms_norm.cpp:103-154. Returns [y(x.shape), rstd(x.shape[:-1]) fp32]; no epsilon by default."""
    _require_gpu(x, "x")
    if x.dtype not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError("rms_norm: input must be bfloat16 or float8_e4m3fn")
    shape = x.shape
    x2 = x.reshape(-1, shape[-1]).contiguous()
    rows, dim = x2.shape
    out_type = x.dtype if out_type is None else out_type
    if out_type not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError("rms_norm: output must be bfloat16 or float8_e4m3fn")
    if weights is not None:
        if weights.dtype != torch.float32 or not weights.is_cuda:
            raise RuntimeError("rms norm: weights error")
        if weights.numel() != dim:
            raise RuntimeError("rms norm: weights must have %d elements" % dim)
        weights = weights.contiguous()
    out = torch.empty((rows, dim), dtype=out_type, device=x.device)
    rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_rmsnorm(x2.data_ptr(), _DT[x2.dtype], _ptr(weights), out.data_ptr(), _DT[out_type],
                                         rstd.data_ptr(), rows, dim, float(eps), _stream(x)))
    return [out.reshape(shape), rstd.reshape(shape[:-1])]


def rope(x: torch.Tensor, cos_freqs: torch.Tensor, sin_freqs: torch.Tensor,
         out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """csrc/ops/rope.cpp:96-146: interleaved-pair rotation with fp32 tables of x's shape."""
    if cos_freqs.dtype != torch.float32 or sin_freqs.dtype != torch.float32:
        raise RuntimeError("rope: cos/sin tables must be float32")
    _require_gpu(x, "x")
    _require_gpu(cos_freqs, "cos_freqs")
    _require_gpu(sin_freqs, "sin_freqs")
    if cos_freqs.shape != x.shape or sin_freqs.shape != x.shape:
        raise RuntimeError("rope: cos/sin tables must have the shape of x")
    if x.dtype not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError("rope: input must be bfloat16 or float8_e4m3fn")
    shape = x.shape
    dim = shape[-1]
    x2 = x.reshape(-1, dim).contiguous()
    c2 = cos_freqs.reshape(-1, dim).contiguous()
    s2 = sin_freqs.reshape(-1, dim).contiguous()
    out_type = x.dtype if out_type is None else out_type
    if out_type not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError("rope: output must be bfloat16 or float8_e4m3fn")
    out = torch.empty(x2.shape, dtype=out_type, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_rope(x2.data_ptr(), _DT[x2.dtype], c2.data_ptr(), s2.data_ptr(), out.data_ptr(),
                                      _DT[out_type], x2.shape[0], dim, _stream(x)))
    return out.reshape(shape)


# ----------------------------------------------------------------------------- gemm._C

def _check_input(t, name):
    _require_gpu(t, name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)


def _mm(a, b, bias, a_scales, b_scales, fuse_gelu, out_type, in_dtype, who, residual=None, gate=None):
    """Shape rules of csrc/gemm/q8_gemm_api.cpp:45-91: a [.,M,K], b [.,N,K], result always [batch,M,N].
    residual (bfloat16, batch*M*N elements, bfloat16 output only): out = bf16(bf16(result) + residual), in the GEMM's
    epilogue where the kernel supports the shape, otherwise by a separate addition with the same two roundings.
    gate (with residual; bfloat16 [G, N] or [G, 1, N], G dividing the batch*M rows: row r uses gate row r // (rows / G)):
    out = bf16(fma(bf16(result), gate, residual)), in the epilogue where the kernel supports the shape, otherwise by the
    fused multiply-add kernel on the projection's output: the same bits."""
    _check_input(a, "a")
    _check_input(b, "b")
    if a.dtype != in_dtype or b.dtype != in_dtype:
        raise RuntimeError("%s: a and b must be %s" % (who, in_dtype))
    if a.dim() not in (2, 3) or b.dim() not in (2, 3):
        raise RuntimeError("%s: a and b must be 2-D or 3-D" % who)
    bs_a, m = (a.shape[0], a.shape[1]) if a.dim() == 3 else (1, a.shape[0])
    bs_b, n = (b.shape[0], b.shape[1]) if b.dim() == 3 else (1, b.shape[0])
    k = a.shape[-1]
    if b.shape[-1] != k:
        raise RuntimeError("%s: K mismatch (%d vs %d)" % (who, k, b.shape[-1]))
    if not (bs_a == bs_b or bs_a == 1 or bs_b == 1):
        raise RuntimeError("Batch missmatch")
    batch = max(bs_a, bs_b)
    out_type = torch.float8_e4m3fn if out_type is None else out_type
    if out_type not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError("%s: out_type must be bfloat16 or float8_e4m3fn, got %s" % (who, out_type))
    for t, name, cnt in ((a_scales, "a_scales", bs_a * m), (b_scales, "b_scales", bs_b * n)):
        _check_input(t, name)
        if t.dtype != torch.float32 or t.numel() != cnt:
            raise RuntimeError("%s: %s must be float32 with %d elements" % (who, name, cnt))
    if bias is not None:
        _check_input(bias, "bias")
        if bias.dtype != torch.float32 or bias.numel() != n:
            raise RuntimeError("%s: bias must be float32 with %d elements" % (who, n))
    out = torch.empty((batch, m, n), dtype=out_type, device=a.device)
    if gate is not None and residual is None:
        raise RuntimeError("%s: a gate comes with a residual" % who)
    if residual is not None:
        _require_gpu(residual, "residual")
        if out_type != torch.bfloat16 or residual.dtype != torch.bfloat16 or residual.numel() != out.numel():
            raise RuntimeError("%s: residual must be bfloat16 with the output's element count, output bfloat16" % who)
        residual = residual.contiguous()
        fusable = n % 8 == 0 and k % 128 == 0 and k > 256 and m * k < 2 ** 32 and n * k < 2 ** 32 and residual.data_ptr() % 16 == 0
        if gate is not None:
            _require_gpu(gate, "gate")
            rows = batch * m
            if gate.dtype != torch.bfloat16 or gate.shape[-1] != n or gate.numel() % n != 0 or rows % (gate.numel() // n) != 0:
                raise RuntimeError("%s: gate must be bfloat16 [G, N] with G dividing the %d output rows" % (who, rows))
            gate = gate.contiguous()
            groups = gate.numel() // n
            per = rows // groups
            if (fusable and bs_b == 1 and per % 768 == 0 and rows * k < 2 ** 32 and gate.data_ptr() % 16 == 0):
                with torch.cuda.device(a.device):  # one batch of batch * M rows: a and a_scales are contiguous over them
                    _lib.check(_lib.lib().q8_gemm_gated_residual(
                        a.data_ptr(), b.data_ptr(), _ptr(bias), a_scales.data_ptr(), b_scales.data_ptr(), residual.data_ptr(),
                        gate.data_ptr(), per, out.data_ptr(), rows, n, k, _DT[in_dtype], 1 if fuse_gelu else 0, _stream(a)))
                return out
            with torch.cuda.device(a.device):
                _lib.check(_lib.lib().q8_gemm(a.data_ptr(), b.data_ptr(), _ptr(bias), a_scales.data_ptr(), b_scales.data_ptr(),
                                              out.data_ptr(), bs_a, bs_b, m, n, k, _DT[in_dtype], _DT[out_type],
                                              1 if fuse_gelu else 0, _stream(a)))
            return fma_8bit(out.view(groups, per, n), gate.view(groups, 1, n), residual.view(groups, per, n)).view(batch, m, n)
        if fusable:
            with torch.cuda.device(a.device):
                _lib.check(_lib.lib().q8_gemm_residual(a.data_ptr(), b.data_ptr(), _ptr(bias), a_scales.data_ptr(),
                                                       b_scales.data_ptr(), residual.data_ptr(), out.data_ptr(), bs_a, bs_b,
                                                       m, n, k, _DT[in_dtype], 1 if fuse_gelu else 0, _stream(a)))
            return out
    with torch.cuda.device(a.device):
        _lib.check(_lib.lib().q8_gemm(a.data_ptr(), b.data_ptr(), _ptr(bias), a_scales.data_ptr(), b_scales.data_ptr(),
                                      out.data_ptr(), bs_a, bs_b, m, n, k, _DT[in_dtype], _DT[out_type],
                                      1 if fuse_gelu else 0, _stream(a)))
    if residual is not None:
        out += residual.view(out.shape)
    return out


def q8_mm(a, b, a_scales, b_scales, fuse_gelu: bool, out_type: Optional[torch.dtype] = None, *,
          residual: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """csrc/gemm/q8_gemm_api.cpp:40-97."""
    return _mm(a, b, None, a_scales, b_scales, fuse_gelu, out_type, torch.int8, "q8_mm", residual, gate)


def q8_mm_bias(a, b, bias, a_scales, b_scales, fuse_gelu: bool, out_type: Optional[torch.dtype] = None, *,
               residual: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """csrc/gemm/q8_gemm_api.cpp:100-164."""
    return _mm(a, b, bias, a_scales, b_scales, fuse_gelu, out_type, torch.int8, "q8_mm_bias", residual, gate)


def fp8_mm(a, b, a_scales, b_scales, fuse_gelu: bool, out_type: Optional[torch.dtype] = None, *,
           residual: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """csrc/gemm/q8_gemm_api.cpp:167-224."""
    return _mm(a, b, None, a_scales, b_scales, fuse_gelu, out_type, torch.float8_e4m3fn, "fp8_mm", residual, gate)


def fp8_mm_bias(a, b, bias, a_scales, b_scales, fuse_gelu: bool, out_type: Optional[torch.dtype] = None, *,
                residual: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """csrc/gemm/q8_gemm_api.cpp:227-291."""
    return _mm(a, b, bias, a_scales, b_scales, fuse_gelu, out_type, torch.float8_e4m3fn, "fp8_mm_bias", residual, gate)


def mm_bias_qkv(a, b, bias, a_scales, b_scales, tokens: int, v_col0: int, fht_scale: float = 0.0):
    """The GEMM of a fused QKV projection with the cast of V in its epilogue: a [B*S, K] codes (int8 or e4m3, rows of B
    batch elements of `tokens` tokens), b [N, K], fp32 bias [N] or None, fp32 row / column scales. Returns (qk, v_codes):
    qk bfloat16 [B, S, v_col0] (the Q and K columns as q8_mm_bias / fp8_mm_bias give them) and v_codes e4m3
    [B, (N - v_col0) / 64, S, 64], the bf16-rounded V columns cast to e4m3 token-major per head, what attn_prep_qkv
    produces from the bfloat16 projection and flash_attention takes with v_token_major=True.
    fht_scale != 0: every head of the v_codes columns goes through the 64-point Hadamard transform times fht_scale
    before the cast, what attn_prep_qk(x, heads, None, None, True, fht_scale) makes of the bfloat16 projection: with
    v_col0 == 0 the query (or key) operand of an attention with apply_qk_hadamard straight from its projection."""
    _check_input(a, "a")
    _check_input(b, "b")
    if a.dtype != b.dtype or a.dtype not in (torch.int8, torch.float8_e4m3fn) or a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise RuntimeError("mm_bias_qkv: a [M,K] and b [N,K] must both be int8 or e4m3 with equal K")
    m, k, n = a.shape[0], a.shape[1], b.shape[0]
    if tokens <= 0 or m % tokens != 0:
        raise RuntimeError("mm_bias_qkv: %d rows are not batch elements of %d tokens" % (m, tokens))
    for t, name, cnt in ((a_scales, "a_scales", m), (b_scales, "b_scales", n)):
        _check_input(t, name)
        if t.dtype != torch.float32 or t.numel() != cnt:
            raise RuntimeError("mm_bias_qkv: %s must be float32 with %d elements" % (name, cnt))
    if bias is not None:
        _check_input(bias, "bias")
        if bias.dtype != torch.float32 or bias.numel() != n:
            raise RuntimeError("mm_bias_qkv: bias must be float32 with %d elements" % n)
    if not (0 <= v_col0 < n) or (n - v_col0) % 64 != 0:
        raise RuntimeError("mm_bias_qkv: v_col0 = %d does not split N = %d into Q/K columns and heads of 64" % (v_col0, n))
    bsz = m // tokens
    # (v_col0 == 0: a V projection of its own; qk comes back without columns)
    qk = torch.empty((bsz, tokens, v_col0), dtype=torch.bfloat16, device=a.device)
    vc = torch.empty((bsz, (n - v_col0) // 64, tokens, 64), dtype=torch.float8_e4m3fn, device=a.device)
    if m == 0:
        return qk, vc
    with torch.cuda.device(a.device):
        _lib.check(_lib.lib().q8_gemm_qkv(a.data_ptr(), b.data_ptr(), _ptr(bias), a_scales.data_ptr(), b_scales.data_ptr(),
                                          qk.data_ptr() if v_col0 else None, vc.data_ptr(), m, n, k, v_col0, tokens,
                                          float(fht_scale), Q8_I8 if a.dtype == torch.int8 else Q8_E4M3, _stream(a)))
    return qk, vc


def q8_mm_i32(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Raw int32 accumulators a @ b.T of the int8 GEMM mainloop (2-D operands), for bit-exact checks."""
    _check_input(a, "a")
    _check_input(b, "b")
    if a.dtype != torch.int8 or b.dtype != torch.int8 or a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise RuntimeError("q8_mm_i32: a [M,K] and b [N,K] must be int8 with equal K")
    out = torch.empty((a.shape[0], b.shape[0]), dtype=torch.int32, device=a.device)
    with torch.cuda.device(a.device):
        _lib.check(_lib.lib().q8_gemm_i32(a.data_ptr(), b.data_ptr(), out.data_ptr(), a.shape[0], b.shape[0], a.shape[1],
                                          _stream(a)))
    return out


# ----------------------------------------------------------------------------- flash_attention._C

def flash_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float,
                    batch_mask: Optional[torch.Tensor] = None, *, out_dtype: Optional[torch.dtype] = None,
                    q_scales: Optional[torch.Tensor] = None, k_scales: Optional[torch.Tensor] = None,
                    v_scales: Optional[torch.Tensor] = None, sum_rounded_p: bool = False,
                    p_unit_range: bool = False, token_major_out: bool = False,
                    v_token_major: bool = False, lazy_max: bool = False) -> torch.Tensor:
    """csrc/flash_attention/flash_attention.cpp:18-48.

    q [B,H,M,64], k [B,H,N,64], v [B,H,64,Nv] (pre-transposed, Nv >= N, Nv % 16 == 0), all e4m3 and contiguous;
    batch_mask int32 [B] of valid KV lengths. Returns [B,H,M,64] in out_dtype (None -> e4m3 like the reference).
    The keyword arguments are extensions: bf16 output, per-token dequantisation scales
    (q_scales [B,H,M], k_scales / v_scales [B,H,N], fp32), and p_unit_range=True to round the probabilities
    on the reference's grid (p <= 1) instead of the default 2^8 p, which does not flush small weights;
    token_major_out=True returns [B,M,H*64], the transpose(1, 2).reshape the callers apply next;
    v_token_major=True takes v as [B,H,N,64] (k's layout): the kernel turns the tiles itself, no transposed copy;
    lazy_max=True lets the maximum the probabilities are formed against trail the running maximum by up to a factor 8
    (fewer rescalings of the accumulators: about 5 % faster on long sequences, the largest weight of a row no longer
    exact; not with p_unit_range); sum_rounded_p=True normalises by the sum of the rounded probabilities (the ones that
    multiply v), taken on the matrix pipe: outputs are convex combinations of v's rows, about 6 % faster on long
    sequences, unit scales only.
    """
    for t, name in ((q, "q"), (k, "k"), (v, "v")):
        _check_input(t, name)
        if t.dtype != torch.float8_e4m3fn or t.dim() != 4:
            raise RuntimeError("flash_attention: %s must be a 4-D float8_e4m3fn tensor" % name)
    bs, heads, m, d = q.shape
    n = k.shape[2]
    if k.shape[0] != bs or k.shape[1] != heads or k.shape[3] != d:
        raise RuntimeError("flash_attention: k shape mismatch")
    if v_token_major:
        if tuple(v.shape) != tuple(k.shape):
            raise RuntimeError("flash_attention: a token-major v must have k's shape [B,H,N,D]")
    elif v.shape[0] != bs or v.shape[1] != heads or v.shape[2] != d or v.shape[3] < n:
        raise RuntimeError("flash_attention: v must be [B,H,D,Nv] with Nv >= N")
    if batch_mask is not None:
        if batch_mask.dtype != torch.int32:
            raise RuntimeError("flash attn: mask type error")
        if batch_mask.dim() != 1 or batch_mask.shape[0] != bs:
            raise RuntimeError("flash attn: mask batch error")
        _check_input(batch_mask, "batch_mask")
    scales = (q_scales, k_scales, v_scales)
    if any(s is not None for s in scales):
        if any(s is None for s in scales):
            raise RuntimeError("flash_attention: q_scales, k_scales and v_scales must be given together")
        for s, cnt, name in ((q_scales, bs * heads * m, "q_scales"), (k_scales, bs * heads * n, "k_scales"),
                             (v_scales, bs * heads * n, "v_scales")):
            _check_input(s, name)
            if s.dtype != torch.float32 or s.numel() != cnt:
                raise RuntimeError("flash_attention: %s must be float32 with %d elements" % (name, cnt))
    out_dtype = torch.float8_e4m3fn if out_dtype is None else out_dtype
    if out_dtype not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError("flash_attention: out_dtype must be bfloat16 or float8_e4m3fn")
    out = torch.empty((bs, m, heads * d) if token_major_out else (bs, heads, m, d), dtype=out_dtype, device=q.device)
    with torch.cuda.device(q.device):
        _lib.check(_lib.lib().q8_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), _ptr(batch_mask),
                                          _ptr(q_scales), _ptr(k_scales), _ptr(v_scales), bs, heads, m, n, d,
                                          _lib.Q8_V_SD if v_token_major else _lib.Q8_V_DS, v.shape[3],
                                          float(softmax_scale), _DT[out_dtype],
                                          (_lib.Q8_ATTN_SUM_ROUNDED_P if sum_rounded_p else 0) |
                                          (_lib.Q8_ATTN_P_UNIT_RANGE if p_unit_range else 0) |
                                          (_lib.Q8_ATTN_O_TOKEN_MAJOR if token_major_out else 0) |
                                          (_lib.Q8_ATTN_LAZY_MAX if lazy_max else 0), _stream(q)))
    return out


# ----------------------------------------------------------------------------- fused row kernels
# No counterpart among the reference's bindings: each replaces a sequence of two or more of the calls above and
# returns the same bits (intermediate values are rounded to bfloat16 where the sequence stores a bfloat16 tensor).

def _quant_out(x2, out_type, who):
    out_type = torch.int8 if out_type is None else out_type
    if out_type not in (torch.int8, torch.float8_e4m3fn):
        raise RuntimeError("%s not implemented for output type '%s'" % (who, out_type))
    rows, dim = x2.shape
    return (out_type, torch.empty((rows, dim), dtype=out_type, device=x2.device),
            torch.empty((rows,), dtype=torch.float32, device=x2.device))


def fht_quant(x: torch.Tensor, scale: float, out_type: Optional[torch.dtype] = None, *,
              round_intermediate: bool = True, mid_type: Optional[torch.dtype] = None) -> List[torch.Tensor]:
    """tokenwise_quant(fast_hadamard_transform(x, scale, mid_type), out_type) in one pass over x.
    x bfloat16 or e4m3 with last dim a multiple of 8; mid_type None -> bfloat16 (float8_e4m3fn is allowed for an
    e4m3 x: what hadamard_transform returns for it by default). Returns [codes(x.shape), scales(x.shape[:-1])]."""
    _require_gpu(x, "x")
    if x.dtype not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError("fht_quant: input must be bfloat16 or float8_e4m3fn")
    shape = x.shape
    x2 = x.reshape(-1, shape[-1]).contiguous()
    out_type, out, scales = _quant_out(x2, out_type, "fht_quant")
    rows, dim = x2.shape
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_fht_quant_rows(x2.data_ptr(), _DT[x2.dtype], out.data_ptr(), _DT[out_type],
                                                scales.data_ptr(), rows, dim, float(scale),
                                                (_DT[mid_type] if mid_type is not None else Q8_BF16) if round_intermediate
                                                else Q8_F32, 0, _stream(x)))
    return [out.reshape(shape), scales.reshape(shape[:-1])]


def rms_norm_quant(x: torch.Tensor, weights: Optional[torch.Tensor] = None, out_type: Optional[torch.dtype] = None, *,
                   eps: float = 0.0, round_intermediate: bool = True) -> List[torch.Tensor]:
    """tokenwise_quant(rms_norm(x, weights, bfloat16)[0], out_type) in one pass over x.
    Returns [codes(x.shape), scales(x.shape[:-1]), rstd(x.shape[:-1])]."""
    _require_gpu(x, "x")
    if x.dtype not in (torch.bfloat16, torch.float8_e4m3fn):
        raise RuntimeError("rms_norm_quant: input must be bfloat16 or float8_e4m3fn")
    if weights is not None and (weights.dtype != torch.float32 or not weights.is_cuda):
        raise RuntimeError("rms_norm_quant: weights must be a float32 CUDA tensor")
    shape = x.shape
    x2 = x.reshape(-1, shape[-1]).contiguous()
    out_type, out, scales = _quant_out(x2, out_type, "rms_norm_quant")
    rows, dim = x2.shape
    if weights is not None and weights.numel() != dim:
        raise RuntimeError("rms_norm_quant: weights must have %d elements" % dim)
    rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_rmsnorm_quant_rows(x2.data_ptr(), _DT[x2.dtype], _ptr(weights), out.data_ptr(),
                                                    _DT[out_type], scales.data_ptr(), rstd.data_ptr(), rows, dim,
                                                    float(eps), Q8_BF16 if round_intermediate else Q8_F32, 0,
                                                    _stream(x)))
    return [out.reshape(shape), scales.reshape(shape[:-1]), rstd.reshape(shape[:-1])]


def norm_mod_fht_quant(x: torch.Tensor, norm: bool = True, norm_weight: Optional[torch.Tensor] = None,
                       mod_scale: Optional[torch.Tensor] = None, mod_shift: Optional[torch.Tensor] = None,
                       scale_add: float = 0.0, fht_scale: Optional[float] = None,
                       out_type: Optional[torch.dtype] = None) -> List[torch.Tensor]:
    """bfloat16 x [B, T, dim] -> [codes, scales] of quant(FHT(fma(rms_norm(x, norm_weight), mod_scale + scale_add,
    mod_shift)) * fht_scale) in one pass; every step is optional (norm False, mod_scale / mod_shift None, fht_scale
    None) and rounds to bfloat16 like the separate operators. mod_scale / mod_shift: [B, 1 or T, dim], bfloat16 or
    float32. out_type None -> int8."""
    _require_gpu(x, "x")
    if x.dtype != torch.bfloat16 or x.dim() != 3:
        raise RuntimeError("norm_mod_fht_quant: x must be a bfloat16 tensor [B, T, dim]")
    shape = x.shape
    x2 = x.reshape(-1, shape[-1]).contiguous()
    out_type, out, scales = _quant_out(x2, out_type, "norm_mod_fht_quant")
    rows, dim = x2.shape
    if norm_weight is not None and (norm_weight.dtype != torch.float32 or not norm_weight.is_cuda or norm_weight.numel() != dim):
        raise RuntimeError("norm_mod_fht_quant: norm weights must be a float32 CUDA tensor with dim elements")
    if (mod_scale is None) != (mod_shift is None):
        raise RuntimeError("norm_mod_fht_quant: mod_scale and mod_shift come together")
    rows_per_mod, mod_dt = 1, Q8_BF16
    if mod_scale is not None:
        for t in (mod_scale, mod_shift):
            _require_gpu(t, "modulation")
            if (t.dtype != mod_scale.dtype or t.dtype not in (torch.bfloat16, torch.float32) or t.dim() != 3 or t.shape[0] != shape[0]
                    or t.shape[-1] != dim or t.shape[1] != mod_scale.shape[1] or t.shape[1] not in (1, shape[1])):
                raise RuntimeError("norm_mod_fht_quant: mod_scale / mod_shift must be [B, 1 or T, dim], both bfloat16 or float32")
        mod_scale, mod_shift = mod_scale.contiguous(), mod_shift.contiguous()
        rows_per_mod, mod_dt = shape[1] // mod_scale.shape[1], _DT[mod_scale.dtype]
    norm_w = None if norm_weight is None else norm_weight.contiguous()  # bound to a name: alive across the launch
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_norm_mod_fht_quant_rows(
            x2.data_ptr(), _ptr(norm_w), int(norm), _ptr(mod_scale),
            _ptr(mod_shift), mod_dt, rows_per_mod, float(scale_add), int(fht_scale is not None),
            float(fht_scale if fht_scale is not None else 1.0), out.data_ptr(), _DT[out_type], scales.data_ptr(), rows, dim,
            0, _stream(x)))
    return [out.reshape(shape), scales.reshape(shape[:-1])]


def _token_major(x, num_heads, who):
    """x [B, S, H*D] bfloat16 with unit last stride and one row stride over (B, S)."""
    _require_gpu(x, "x")
    if x.dtype != torch.bfloat16 or x.dim() != 3:
        raise RuntimeError("%s: x must be a bfloat16 tensor [B, S, H*D]" % who)
    b, s, dim = x.shape
    if dim % num_heads != 0:
        raise RuntimeError("%s: last dim %d is not divisible by %d heads" % (who, dim, num_heads))
    if x.stride(2) != 1 or (b > 1 and x.stride(0) != s * x.stride(1)) or x.data_ptr() % 16 != 0 or x.stride(1) % 8 != 0:
        x = x.contiguous()
    return x, b, s, dim // num_heads


def _norm_w(w, x):
    if w is None:
        return None
    if w.dtype != torch.float32 or not w.is_cuda or w.numel() != x.shape[-1]:
        raise RuntimeError("attn_prep_qk: norm weights must be float32 CUDA tensors with H*D elements")
    return w.contiguous()


def _rope_tables(cos, sin, b, s, dim, who):
    """The rotation tables of an attention prologue and the flag bits that describe their layout: float32 CUDA tensors
    whose last dimension is H*D (one entry per element) or H*D/2 (one per rotated pair, Q8_PREP_PAIR_TABLES) and whose
    leading dimensions hold B*S rows (one per token) or S rows (the positions of one batch element, serving all B:
    Q8_PREP_SHARED_TABLES). Returns (cos, sin, flags)."""
    if (cos is None) != (sin is None):
        raise RuntimeError("%s: cos and sin come together" % who)
    if cos is None:
        return None, None, 0
    flags = 0
    for t in (cos, sin):
        if t.dtype != torch.float32 or not t.is_cuda or t.shape != cos.shape or t.dim() < 2:
            raise RuntimeError("%s: tables must be float32 CUDA tensors of one shape" % who)
    last, rows = cos.shape[-1], cos.numel() // max(1, cos.shape[-1])
    if last == dim // 2 and dim % 2 == 0 and last != dim:
        flags |= _lib.Q8_PREP_PAIR_TABLES
    elif last != dim:
        raise RuntimeError("%s: the tables' last dimension must be H*D = %d or H*D/2" % (who, dim))
    if rows == s and b > 1:
        flags |= _lib.Q8_PREP_SHARED_TABLES
    elif rows != b * s:
        raise RuntimeError("%s: tables must hold one row per token (%d) or per position (%d)" % (who, b * s, s))
    return cos.contiguous(), sin.contiguous(), flags


def attn_prep_qk(x: torch.Tensor, num_heads: int, cos: Optional[torch.Tensor] = None,
                 sin: Optional[torch.Tensor] = None, apply_fht: bool = True, scale: float = 1.0,
                 per_token_scales: bool = False, *, round_intermediate: bool = True,
                 norm_weight: Optional[torch.Tensor] = None):
    """x [B, S, H*D] bfloat16 (a strided slice of a fused projection is fine) -> e4m3 [B, H, S, D]:
    optional RMSNorm over the H*D row (norm_weight fp32 [H*D], no epsilon), optional RoPE (tables fp32 [B, S, H*D]; or the same values stored once, [S, H*D] for positions shared by the batch
    and / or last dimension H*D/2 for one entry per rotated pair: functional.rope.compact_freqs_cis makes them), head split, optional D-point Hadamard transform times `scale`,
    then the direct e4m3 cast, or per-(token, head) absmax quantization when per_token_scales
    (returns (codes, scales [B, H, S]) in that case)."""
    x, b, s, d = _token_major(x, num_heads, "attn_prep_qk")
    cos, sin, tflags = _rope_tables(cos, sin, b, s, num_heads * d, "attn_prep_qk")
    codes = torch.empty((b, num_heads, s, d), dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty((b, num_heads, s), dtype=torch.float32, device=x.device) if per_token_scales else None
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_attn_prep_qk(x.data_ptr(), x.stride(1), _ptr(_norm_w(norm_weight, x)), _ptr(cos), _ptr(sin),
                                              codes.data_ptr(),
                                              _ptr(scales), b, s, num_heads, d, int(apply_fht) | tflags, float(scale),
                                              Q8_BF16 if round_intermediate else Q8_F32, _stream(x)))
    return (codes, scales) if per_token_scales else codes


def attn_prep_qk_pair(q: torch.Tensor, k: torch.Tensor, num_heads: int, cos: Optional[torch.Tensor] = None,
                      sin: Optional[torch.Tensor] = None, apply_fht: bool = True, scale: float = 1.0,
                      per_token_scales: bool = False, *, round_intermediate: bool = True,
                      q_norm_weight: Optional[torch.Tensor] = None, k_norm_weight: Optional[torch.Tensor] = None):
    """attn_prep_qk for the Q and K projections of a self-attention in one pass (the tables are read once).
    Returns (q_out, k_out), each what attn_prep_qk returns."""
    q, b, s, d = _token_major(q, num_heads, "attn_prep_qk_pair")
    k, bk, sk, dk = _token_major(k, num_heads, "attn_prep_qk_pair")
    if (bk, sk, dk) != (b, s, d):
        raise RuntimeError("attn_prep_qk_pair: q and k must have the same shape")
    cos, sin, tflags = _rope_tables(cos, sin, b, s, num_heads * d, "attn_prep_qk_pair")
    mk = lambda: torch.empty((b, num_heads, s, d), dtype=torch.float8_e4m3fn, device=q.device)  # noqa: E731
    mks = lambda: torch.empty((b, num_heads, s), dtype=torch.float32, device=q.device) if per_token_scales else None  # noqa: E731
    cq, ck, sq, sk_ = mk(), mk(), mks(), mks()
    with torch.cuda.device(q.device):
        _lib.check(_lib.lib().q8_attn_prep_qk_pair(q.data_ptr(), q.stride(1), k.data_ptr(), k.stride(1),
                                                   _ptr(_norm_w(q_norm_weight, q)), _ptr(_norm_w(k_norm_weight, k)),
                                                   _ptr(cos), _ptr(sin),
                                                   cq.data_ptr(), _ptr(sq), ck.data_ptr(), _ptr(sk_), b, s, num_heads, d,
                                                   int(apply_fht) | tflags, float(scale),
                                                   Q8_BF16 if round_intermediate else Q8_F32, _stream(q)))
    return ((cq, sq), (ck, sk_)) if per_token_scales else (cq, ck)


def attn_prep_qkv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, num_heads: int, cos: Optional[torch.Tensor] = None,
                  sin: Optional[torch.Tensor] = None, apply_fht: bool = True, scale: float = 1.0,
                  per_token_scales: bool = False, *, round_intermediate: bool = True,
                  q_norm_weight: Optional[torch.Tensor] = None, k_norm_weight: Optional[torch.Tensor] = None):
    """attn_prep_qk_pair, and the V projection of the same tokens is cast to e4m3 in the same pass, token-major per head
    ([B, H, S, D], what flash_attention takes with v_token_major=True). Returns (q_out, k_out, v_out), each codes or
    (codes, scales [B, H, S]) with per_token_scales."""
    q, b, s, d = _token_major(q, num_heads, "attn_prep_qkv")
    k, bk, sk, dk = _token_major(k, num_heads, "attn_prep_qkv")
    v, bv, sv, dv = _token_major(v, num_heads, "attn_prep_qkv")
    if (bk, sk, dk) != (b, s, d) or (bv, sv, dv) != (b, s, d):
        raise RuntimeError("attn_prep_qkv: q, k and v must have the same shape")
    cos, sin, tflags = _rope_tables(cos, sin, b, s, num_heads * d, "attn_prep_qkv")
    mk = lambda: torch.empty((b, num_heads, s, d), dtype=torch.float8_e4m3fn, device=q.device)  # noqa: E731
    mks = lambda: torch.empty((b, num_heads, s), dtype=torch.float32, device=q.device) if per_token_scales else None  # noqa: E731
    cq, ck, cv, sq, sk_, sv_ = mk(), mk(), mk(), mks(), mks(), mks()
    with torch.cuda.device(q.device):
        _lib.check(_lib.lib().q8_attn_prep_qkv(q.data_ptr(), q.stride(1), k.data_ptr(), k.stride(1), v.data_ptr(), v.stride(1),
                                               _ptr(_norm_w(q_norm_weight, q)), _ptr(_norm_w(k_norm_weight, k)),
                                               _ptr(cos), _ptr(sin), cq.data_ptr(), _ptr(sq), ck.data_ptr(), _ptr(sk_),
                                               cv.data_ptr(), _ptr(sv_), b, s, num_heads, d, int(apply_fht) | tflags, float(scale),
                                               Q8_BF16 if round_intermediate else Q8_F32, _stream(q)))
    return ((cq, sq), (ck, sk_), (cv, sv_)) if per_token_scales else (cq, ck, cv)


def attn_prep_kv(k: torch.Tensor, v: torch.Tensor, num_heads: int, cos: Optional[torch.Tensor] = None,
                 sin: Optional[torch.Tensor] = None, apply_fht: bool = True, scale: float = 1.0,
                 per_token_scales: bool = False, *, round_intermediate: bool = True,
                 norm_weight: Optional[torch.Tensor] = None):
    """attn_prep_qk on k, and the V projection of the same tokens is cast to e4m3 in the same pass, token-major per head
    ([B, H, S, D], what flash_attention takes with v_token_major=True): keys and values of a cross-attention in one
    launch. Returns (k_out, v_out), each codes or (codes, scales [B, H, S]) with per_token_scales."""
    k, b, s, d = _token_major(k, num_heads, "attn_prep_kv")
    v, bv, sv, dv = _token_major(v, num_heads, "attn_prep_kv")
    if (bv, sv, dv) != (b, s, d):
        raise RuntimeError("attn_prep_kv: k and v must have the same shape")
    cos, sin, tflags = _rope_tables(cos, sin, b, s, num_heads * d, "attn_prep_kv")
    mk = lambda: torch.empty((b, num_heads, s, d), dtype=torch.float8_e4m3fn, device=k.device)  # noqa: E731
    mks = lambda: torch.empty((b, num_heads, s), dtype=torch.float32, device=k.device) if per_token_scales else None  # noqa: E731
    ck, cv, sk_, sv_ = mk(), mk(), mks(), mks()
    nw = _norm_w(norm_weight, k)  # bound to a name: alive across the launch
    with torch.cuda.device(k.device):
        _lib.check(_lib.lib().q8_attn_prep_kv(k.data_ptr(), k.stride(1), v.data_ptr(), v.stride(1), _ptr(nw), _ptr(cos), _ptr(sin),
                                              ck.data_ptr(), _ptr(sk_), cv.data_ptr(), _ptr(sv_), b, s, num_heads, d,
                                              int(apply_fht) | tflags, float(scale), Q8_BF16 if round_intermediate else Q8_F32, _stream(k)))
    return ((ck, sk_), (cv, sv_)) if per_token_scales else (ck, cv)


def attn_prep_v(x: torch.Tensor, num_heads: int, per_token_scales: bool = False):
    """x [B, S, H*64] bfloat16 -> e4m3 [B, H, 64, S_pad] (S_pad = S rounded up to 16, zero filled), the V operand
    of flash_attention; with per_token_scales also scales [B, H, S]."""
    x, b, s, d = _token_major(x, num_heads, "attn_prep_v")
    s_pad = (s + 15) // 16 * 16
    codes = torch.empty((b, num_heads, d, s_pad), dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty((b, num_heads, s), dtype=torch.float32, device=x.device) if per_token_scales else None
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_attn_prep_v(x.data_ptr(), x.stride(1), codes.data_ptr(), _ptr(scales), b, s,
                                             num_heads, d, s_pad, _stream(x)))
    return (codes, scales) if per_token_scales else codes


# ----------------------------------------------------------------------------- ops._C: fma and the backward operators

_EW = (torch.bfloat16, torch.float8_e4m3fn)


def _rows2d(t, name):
    _require_gpu(t, name)
    t2 = t.reshape(-1, t.shape[-1])
    return t2 if t2.is_contiguous() else t2.contiguous()


def adaln_rows(table: torch.Tensor, timestep: torch.Tensor) -> torch.Tensor:
    """The modulation rows of an AdaLN block (q8_kernels/blocks/ltx_transformer_block.py:30-36): table float32 [P, dim],
    timestep float32 [B, T, P * dim] -> bfloat16 [P, B, T, dim] = bf16(table[p] + timestep[b, t, p*dim:(p+1)*dim]); slice p
    is the contiguous [B, T, dim] tensor that `(table[None, None] + timestep.reshape(B, T, P, dim)).unbind(2)[p]` gives after
    its cast to bfloat16."""
    _require_gpu(table, "table")
    _require_gpu(timestep, "timestep")
    if table.dtype != torch.float32 or timestep.dtype != torch.float32 or table.dim() != 2 or timestep.dim() != 3:
        raise RuntimeError("adaln_rows: table float32 [P, dim] and timestep float32 [B, T, P*dim]")
    p, dim = table.shape
    b, t, pd = timestep.shape
    if pd != p * dim:
        raise RuntimeError("adaln_rows: timestep's last dimension %d is not %d parameters x %d" % (pd, p, dim))
    table, timestep = table.contiguous(), timestep.contiguous()
    rows = torch.empty((p, b, t, dim), dtype=torch.bfloat16, device=table.device)
    with torch.cuda.device(table.device):
        _lib.check(_lib.lib().q8_adaln_rows(table.data_ptr(), timestep.data_ptr(), rows.data_ptr(), p, b * t, dim, _stream(table)))
    return rows


def fma_8bit(x: torch.Tensor, y: torch.Tensor, z: torch.Tensor, scale_add: float = 0.0, *,
             out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """csrc/ops/fma.cpp:63-112: x * (y + scale_add) + z for x [B, T, dim] e4m3, y and z [B, T or 1, dim]
    (fp32/fp32, fp32/e4m3 or bf16/bf16 in the reference; any mix of the three here). Returns x's shape in x's
    dtype; bfloat16 x and `out_type` are extensions."""
    if x.dtype not in _EW:
        raise RuntimeError("fma_8bit: x must be float8_e4m3fn (or bfloat16)")
    if x.dim() != 3:
        raise RuntimeError("fma_8bit: x must be 3-D")
    for t, name in ((y, "y"), (z, "z")):
        if t.dtype not in (torch.float32, torch.bfloat16, torch.float8_e4m3fn):
            raise RuntimeError("fma not implemented for input type '%s'" % t.dtype)
        if t.shape[-1] != x.shape[-1]:
            raise RuntimeError("fma: channels missmatch")
        if t.dim() != 3 or t.shape[0] != x.shape[0] or t.shape[-2] not in (1, x.shape[-2]):
            raise RuntimeError("fma: token missmatch")
    out_type = x.dtype if out_type is None else out_type
    if out_type not in _EW:
        raise RuntimeError("fma_8bit: output must be bfloat16 or float8_e4m3fn")
    shape = x.shape
    x2, y2, z2 = _rows2d(x, "x"), _rows2d(y, "y"), _rows2d(z, "z")
    rows, dim = x2.shape
    out = torch.empty((rows, dim), dtype=out_type, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_fma(x2.data_ptr(), _DT[x2.dtype], y2.data_ptr(), _DT[y2.dtype], z2.data_ptr(),
                                     _DT[z2.dtype], out.data_ptr(), _DT[out_type], rows, dim,
                                     shape[-2] // y.shape[-2], shape[-2] // z.shape[-2], float(scale_add), _stream(x)))
    return out.reshape(shape)


def _ew_out(x, out_type, who):
    out_type = x.dtype if out_type is None else out_type
    if x.dtype not in _EW or out_type not in _EW:
        raise RuntimeError("%s: input and output must be bfloat16 or float8_e4m3fn" % who)
    if x.shape[-1] % 8 != 0:
        raise RuntimeError("%s: last dim must be a multiple of 8" % who)
    return out_type


def gelu_forward(x: torch.Tensor, out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """csrc/ops/gelu_act.cpp (gelu_forward): tanh-GELU, out_type None -> x.dtype."""
    out_type = _ew_out(x, out_type, "gelu_forward")
    x2 = _rows2d(x, "x")
    out = torch.empty(x2.shape, dtype=out_type, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_gelu(x2.data_ptr(), _DT[x2.dtype], out.data_ptr(), _DT[out_type], x2.numel(), _stream(x)))
    return out.reshape(x.shape)


def gelu_backward(x: torch.Tensor, grad_output: torch.Tensor, out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """csrc/ops/gelu_act.cpp (gelu_backward): grad_output * dGELU/dx at x, out_type None -> x.dtype."""
    out_type = _ew_out(x, out_type, "gelu_backward")
    if grad_output.shape != x.shape or grad_output.dtype not in _EW:
        raise RuntimeError("gelu_backward: grad_output must have x's shape and be bfloat16 or float8_e4m3fn")
    x2, g2 = _rows2d(x, "x"), _rows2d(grad_output, "grad_output")
    out = torch.empty(x2.shape, dtype=out_type, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().q8_gelu_backward(x2.data_ptr(), _DT[x2.dtype], g2.data_ptr(), _DT[g2.dtype], out.data_ptr(),
                                               _DT[out_type], x2.numel(), _stream(x)))
    return out.reshape(x.shape)


def rope_backward(grad_out: torch.Tensor, cos_freqs: torch.Tensor, sin_freqs: torch.Tensor,
                  out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """csrc/ops/rope.cpp:150-200: the transposed rotation applied to grad_out."""
    if cos_freqs.dtype != torch.float32 or sin_freqs.dtype != torch.float32:
        raise RuntimeError("rope_backward: cos/sin tables must be float32")
    if cos_freqs.shape != grad_out.shape or sin_freqs.shape != grad_out.shape:
        raise RuntimeError("rope_backward: cos/sin tables must have the shape of grad_out")
    out_type = _ew_out(grad_out, out_type, "rope_backward")
    g2, c2, s2 = _rows2d(grad_out, "grad_out"), _rows2d(cos_freqs, "cos_freqs"), _rows2d(sin_freqs, "sin_freqs")
    out = torch.empty(g2.shape, dtype=out_type, device=grad_out.device)
    with torch.cuda.device(grad_out.device):
        _lib.check(_lib.lib().q8_rope_backward(g2.data_ptr(), _DT[g2.dtype], c2.data_ptr(), s2.data_ptr(), out.data_ptr(),
                                               _DT[out_type], g2.shape[0], g2.shape[1], _stream(grad_out)))
    return out.reshape(grad_out.shape)


def rms_norm_backward(x_normed: torch.Tensor, x_norms: torch.Tensor, grad_out: torch.Tensor,
                      weights: Optional[torch.Tensor] = None, out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """csrc/ops/rms_norm.cpp (rms_norm_backward): dx from the forward's outputs (x_normed, x_norms = rstd per row)."""
    out_type = _ew_out(x_normed, out_type, "rms_norm_backward")
    if grad_out.shape != x_normed.shape or grad_out.dtype not in _EW:
        raise RuntimeError("rms_norm_backward: grad_out must have x_normed's shape and be bfloat16 or float8_e4m3fn")
    y2, g2 = _rows2d(x_normed, "x_normed"), _rows2d(grad_out, "grad_out")
    rows, dim = y2.shape
    _require_gpu(x_norms, "x_norms")
    if x_norms.dtype != torch.float32 or x_norms.numel() != rows:
        raise RuntimeError("rms_norm_backward: x_norms must be float32 with one value per row")
    if weights is not None and (weights.dtype != torch.float32 or not weights.is_cuda or weights.numel() != dim):
        raise RuntimeError("rms_norm_backward: weights error")
    out = torch.empty((rows, dim), dtype=out_type, device=x_normed.device)
    norms, w = x_norms.contiguous(), (None if weights is None else weights.contiguous())  # alive across the launch
    with torch.cuda.device(x_normed.device):
        _lib.check(_lib.lib().q8_rmsnorm_backward(y2.data_ptr(), _DT[y2.dtype], norms.data_ptr(), g2.data_ptr(),
                                                  _DT[g2.dtype], _ptr(w),
                                                  out.data_ptr(), _DT[out_type], rows, dim, _stream(x_normed)))
    return out.reshape(x_normed.shape)
