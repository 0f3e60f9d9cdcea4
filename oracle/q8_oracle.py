"""CPU oracle for the 8-bit hot path of q8_kernels: a plain torch/numpy restatement of what the
reference's CUDA kernels and Python wrappers compute.

THIS IS TEST INFRASTRUCTURE. It is the checker for the HIP kernels (tests/, the smoke run and the CPU
baseline leg of bench.py); the product (q8_kernels_amd/) never imports it.

Every function cites the reference file:line it follows (paths relative to the reference root).
The reference ships no tests or golden vectors, so each function is pinned in tests/test_oracle.py by
independent closed forms (scipy Hadamard matrix, brute-force e4m3 rounding tables, exact integer matmul,
float64 softmax, complex-number rotation ...).

Pinning status:
  pinned by closed forms ....... e4m3 casts, ref_fht, ref_quant, ref_gemm_i32, ref_gemm_fp8_acc,
                                 ref_epilogue, ref_rms_norm, ref_rope, ref_attention, ref_freqs_cis,
                                 ref_fma (exact rational arithmetic), ref_gelu_backward, ref_rms_norm_backward,
                                 ref_rope_backward (float64 autograd of the forward formulas, adjoint identity)
  pinned by a dense evaluation . ref_attention_module, ref_ltx_block, ref_dit_block: float64 x @ W.T / softmax /
                                 modulation on the unquantized weights, written from the reference's module text;
                                 mutants of it (swapped shift and scale, a missing gate, norm after the rotation,
                                 rotation in the cross-attention, no mask ...) are each rejected
  parity unpinned (bit level) .. the low-order bits the reference gets from nvcc --use_fast_math
                                 (approximate division in the quantizer, tanhf / exp2f / rsqrtf) and the
                                 accumulation order inside mma.sync; unobservable without an sm_89 GPU.
                                 Quantizer: the int8 code of a NaN element (an undefined C++ conversion in the
                                 reference), a row of nothing but NaN, the sign of NaN codes.
"""
import math
from typing import Optional, Tuple

import numpy as np
import torch

E4M3 = torch.float8_e4m3fn
LOG2E = 1.4426950408889634

# ------------------------------------------------------------------------------------------- casts


def e4m3_c10(x: torch.Tensor) -> torch.Tensor:
    """fp32 -> e4m3fn as c10::Float8_e4m3fn(float): RNE, |x| > 464 and NaN -> NaN code (0x7f | sign).
    This is the cast behind every `out_vals_store[i] = out_vals[i]` in the row kernels, e.g.
    csrc/quantizer/tokenwise_quant_cuda.cu:47-55, csrc/fast_hadamard/fast_hadamard_transform_common.h:146-161.
    torch's CPU cast is that same routine."""
    return x.to(torch.float32).to(E4M3)


def e4m3_sat(x: torch.Tensor) -> torch.Tensor:
    """fp32 -> e4m3fn, RNE, saturating to +-448, NaN stays NaN (__NV_SATFINITE):
    csrc/gemm/fp8_matmul_bias.cu:42-52, csrc/flash_attention/flash_attention_cuda.cu:151-167."""
    x = x.to(torch.float32)
    return torch.where(torch.isnan(x), x, x.clamp(-448.0, 448.0)).to(E4M3)


def e4m3_decode_table() -> np.ndarray:
    """The 256 values of OCP e4m3fn from the bit layout (sign, 4-bit exponent bias 7, 3-bit mantissa;
    no infinities, S.1111.111 = NaN). Independent of torch; used to pin the casts."""
    out = np.zeros(256, dtype=np.float64)
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 7
        if e == 0xF and m == 7:
            out[code] = np.nan
        elif e == 0:
            out[code] = s * (m / 8.0) * 2.0 ** (-6)
        else:
            out[code] = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return out


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Store conversion of the row kernels: bf16/fp16 RNE, e4m3 with c10 semantics."""
    if dtype == E4M3:
        return e4m3_c10(x)
    return x.to(dtype)


# ------------------------------------------------------------------------------------------- FHT


def ref_fht(x: torch.Tensor, scale: Optional[float] = None, out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """Fast Walsh-Hadamard transform on the last dim, fp32 butterflies in ascending stride order, then
    `* scale` and the store cast. Follows csrc/fast_hadamard/fast_hadamard_transform_cuda.cu:84-108
    (thread -> warp -> cross-warp -> chunk stages, all ascending in the element-index bit) and
    csrc/fast_hadamard/fast_hadamard_transform.cpp:57,86-92 (pad to a multiple of 8, N = next power of
    two, implicit zero padding). Default scale 1/sqrt(dim) and out_type=None -> input dtype are those of
    q8_kernels/functional/fast_hadamard.py:24-38 and fast_hadamard_transform.cpp:94-99."""
    dim = x.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(dim)
    out_type = x.dtype if out_type is None else out_type
    dim8 = (dim + 7) // 8 * 8
    n = 8
    while n < dim8:
        n *= 2
    v = torch.zeros(x.shape[:-1] + (n,), dtype=torch.float32)
    v[..., :dim] = x.to(torch.float32)
    rows = v.reshape(-1, n)
    stride = 1
    while stride < n:
        r = rows.reshape(-1, n // (2 * stride), 2, stride)
        a, b = r[:, :, 0, :], r[:, :, 1, :]
        rows = torch.stack((a + b, a - b), dim=2).reshape(-1, n)
        stride *= 2
    y = rows.reshape(v.shape)[..., :dim] * torch.tensor(scale, dtype=torch.float32)
    return cast(y, out_type)


# ------------------------------------------------------------------------------------------- quantizer


def ref_quant(x: torch.Tensor, out_type: Optional[torch.dtype] = None, round_half_even: bool = False,
              scale_as_division: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Token-wise absmax quantizer, csrc/quantizer/tokenwise_quant_cuda.cu:115-148 in IEEE fp32:
        a = max|x|;  r = QMAX / a;  q = x * r;  int8: round() (half away from zero) then cast,
        e4m3: c10 cast;  stored scale = 1 / r.     QMAX = 127 / 448 (:10-12); out_type None -> int8
        (csrc/quantizer/tokenwise_quant.cpp:88-93).
    Deviations selected by flags: round_half_even (BASELINE config 2), scale_as_division
    (scale = a / QMAX). A zero row gives codes 0 and scale 0 (the reference yields NaN codes there).
    Non-finite input: the reference's row maximum is a chain of CUDA max(float, float), i.e. fmaxf (:115-132), which
    skips NaN operands, so a NaN element leaves the scale and the other codes of its row alone and only becomes a NaN
    code itself (e4m3; its int8 code is a C++ conversion of NaN, undefined); an infinite element makes the scale
    infinite, the finite elements' codes zero and its own code NaN (inf * 0). A row of nothing but NaN is not modelled."""
    out_type = torch.int8 if out_type is None else out_type
    xf = x.to(torch.float32)
    ax = xf.abs()
    a = torch.where(ax.isnan(), torch.zeros_like(ax), ax).amax(dim=-1, keepdim=True)
    qmax = torch.tensor(127.0 if out_type == torch.int8 else 448.0, dtype=torch.float32)
    nz = a > 0
    r = torch.where(nz, qmax / torch.where(nz, a, torch.ones_like(a)), torch.zeros_like(a))
    q = xf * r
    if out_type == torch.int8:
        if round_half_even:
            q = torch.round(q)  # torch.round is half-to-even
        else:
            q = torch.sign(q) * torch.floor(q.abs() + 0.5)  # C round(): half away from zero
        codes = q.to(torch.int8)
    else:
        codes = e4m3_c10(q)
    if scale_as_division:
        s = torch.where(nz, a / qmax, torch.zeros_like(a))
    else:
        s = torch.where(nz, 1.0 / torch.where(nz, r, torch.ones_like(r)), torch.zeros_like(a))
    return codes, s.squeeze(-1)


# ------------------------------------------------------------------------------------------- GEMM


def ref_gemm_i32(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Exact int32 accumulators a @ b.T of the int8 GEMM (mma.sync S32S8S8S32, csrc/gemm/q8_matmul_bias.cu:446).
    float64 holds every partial sum exactly (|sum| <= 127^2 K < 2^53)."""
    acc = a.to(torch.float64) @ b.to(torch.float64).transpose(-1, -2)
    return acc.to(torch.int64).to(torch.int32)


def ref_gemm_fp8_acc(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """sum_k a[m,k] b[n,k] for e4m3 operands: products are exact, accumulated in float64 (the kernels
    accumulate in fp32 in hardware order, hence a tolerance in the tests). csrc/gemm/fp8_matmul_bias.cu:262-314."""
    return a.to(torch.float64) @ b.to(torch.float64).transpose(-1, -2)


def gelu_tanh(v: torch.Tensor) -> torch.Tensor:
    """0.5 v (1 + tanh(0.79788456 (v + 0.044715 v^3))), csrc/gemm/fp8_matmul_bias.cu:31-35."""
    return 0.5 * v * (1.0 + torch.tanh(0.7978845608028654 * (v + 0.044715 * v * v * v)))


def ref_epilogue(acc: torch.Tensor, sa: torch.Tensor, sb: torch.Tensor, bias: Optional[torch.Tensor], fuse_gelu: bool,
                 out_type: Optional[torch.dtype]) -> torch.Tensor:
    """v = acc * (sa[m] * sb[n]) (+ bias[n]); optional tanh-GELU; bf16 RNE or e4m3 saturating store.
    csrc/gemm/fp8_matmul_bias.cu:352-369 (order of the dequantisation), q8_matmul_bias.cu:315-320
    (int32 -> float), q8_gemm_api.cpp:82-87 (out_type None -> e4m3). acc: [..., M, N]; sa: [..., M]; sb: [..., N]."""
    out_type = E4M3 if out_type is None else out_type
    s = (sa.to(torch.float32).unsqueeze(-1) * sb.to(torch.float32).unsqueeze(-2)).to(torch.float64)
    v = acc.to(torch.float64) * s
    if bias is not None:
        v = v + bias.to(torch.float64)
    v = v.to(torch.float32)
    if fuse_gelu:
        v = gelu_tanh(v.to(torch.float64)).to(torch.float32)
    if out_type == E4M3:
        return e4m3_sat(v)
    return v.to(out_type)


def _bcast_mm(fn, a, b):
    """Batch rule of csrc/gemm/q8_gemm_api.cpp:45-78: 2-D operands count as batch 1, result is 3-D."""
    a3 = a if a.dim() == 3 else a.unsqueeze(0)
    b3 = b if b.dim() == 3 else b.unsqueeze(0)
    assert a3.shape[0] == b3.shape[0] or a3.shape[0] == 1 or b3.shape[0] == 1, "Batch missmatch"
    return fn(a3, b3)


def ref_q8_mm(a, b, bias, a_scales, b_scales, fuse_gelu=False, out_type=None):
    """q8_mm / q8_mm_bias (csrc/gemm/q8_gemm_api.cpp:40-164): int8 operands, result [batch, M, N]."""
    acc = _bcast_mm(ref_gemm_i32, a, b)
    bs_a = a.shape[0] if a.dim() == 3 else 1
    bs_b = b.shape[0] if b.dim() == 3 else 1
    sa = a_scales.reshape(bs_a, -1)
    sb = b_scales.reshape(bs_b, -1)
    return ref_epilogue(acc, sa, sb, bias, fuse_gelu, out_type)


def ref_fp8_mm(a, b, bias, a_scales, b_scales, fuse_gelu=False, out_type=None):
    """fp8_mm / fp8_mm_bias (csrc/gemm/q8_gemm_api.cpp:167-291)."""
    acc = _bcast_mm(ref_gemm_fp8_acc, a, b)
    bs_a = a.shape[0] if a.dim() == 3 else 1
    bs_b = b.shape[0] if b.dim() == 3 else 1
    return ref_epilogue(acc, a_scales.reshape(bs_a, -1), b_scales.reshape(bs_b, -1), bias, fuse_gelu, out_type)


def _is_16bit(t):
    return t.dtype in (torch.float16, torch.bfloat16)


def ref_q8_linear(a, b, bias=None, scale_a=None, scale_b=None, fuse_gelu=False, out_dtype=None):
    """Q8LinearFunc.forward, q8_kernels/functional/linear.py:24-42: 16-bit / fp8 operands are rotated by the
    FHT and quantized to int8 per row first."""
    if a.dtype == E4M3 or _is_16bit(a):
        a, scale_a = ref_quant(ref_fht(a))
    if b.dtype == E4M3 or _is_16bit(b):
        b, scale_b = ref_quant(ref_fht(b))
    return ref_q8_mm(a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype)


def ref_fp8_linear(a, b, bias=None, scale_a=None, scale_b=None, use_hadamard=False, out_dtype=None, fuse_gelu=False):
    """FP8LinearFunc.forward, q8_kernels/functional/linear.py:138-159 (fuse_gelu is hard-wired False there;
    the kernel beneath supports it, csrc/gemm/q8_gemm_api.cpp:227)."""
    qf = (lambda t: ref_quant(ref_fht(t), E4M3)) if use_hadamard else (lambda t: ref_quant(t, E4M3))
    if _is_16bit(a):
        a, scale_a = qf(a)
    if _is_16bit(b):
        b, scale_b = qf(b)
    return ref_fp8_mm(a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype)


# ------------------------------------------------------------------------------------------- attention


def ref_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float,
                  kv_len: Optional[torch.Tensor] = None, sq=None, sk=None, sv=None,
                  round_p: bool = True, out_dtype: Optional[torch.dtype] = None, return_weighted_abs: bool = False,
                  p_scale: float = 1.0, sum_rounded: bool = False):
    """Attention on e4m3 operands as the reference kernel defines it (csrc/flash_attention/
    flash_attention_cuda.cu:171-248,437,487-497; mask: flash_attention_cuda_mask.cu:244,319):
        s_ij = (q_i . k_j) * scale (* sq_i sk_j);  keys j >= kv_len[b] masked;
        p_ij = exp(s_ij - max_j s_ij);  l_i = sum_j p_ij (unrounded);
        o_i = sum_j e4m3_sat(p_ij) v_j / l_i;  rows with l_i == 0 are divided by 1.
    Per-token dequantisation scales (an extension, the reference kernel has unit scales): V's scale enters
    P before its cast as sv_j / max_j sv_j and the common factor is applied to o_i.
    q [B,H,M,D], k, v [B,H,N,D] (v NOT transposed here). With round_p=False this is plain fp32-style
    softmax attention on the dequantised inputs (evaluated in float64), the accuracy target of the
    BASELINE configs. out_dtype None returns float64; bf16 -> RNE; e4m3 -> saturating cast.
    p_scale: the probabilities are rounded as e4m3_sat(p_scale * p). The default 1 is the reference (weights below
    2^-10 flush to zero); the HIP kernel's own default is 2^8, which cancels in o / l, and the tests of that default
    pass p_scale=256 explicitly.
    sum_rounded (unit scales only): l_i sums the ROUNDED probabilities, the ones that multiply V, so that o_i is a true
    convex combination of the v_j (the HIP kernel's Q8_ATTN_SUM_ROUNDED_P; the reference sums the unrounded ones).
    The online kernel rounds p against the running maximum, so its P-hat differs from this one in the
    last e4m3 bit here and there: comparisons carry a tolerance. With return_weighted_abs the function also
    returns W = sum_j p_ij |v_j| / l_i and U = sum_j |v_j| / l_i: rounding every weight with relative error eps
    (2^-4 for normal e4m3 values) or absolute error delta (2^-10 / p_scale in the subnormal range) moves o_i
    by at most eps W + delta U, the rigorous bound the tests use."""
    qd, kd, vd = q.to(torch.float64), k.to(torch.float64), v.to(torch.float64)
    s = qd @ kd.transpose(-1, -2) * softmax_scale
    if sq is not None:
        s = s * sq.to(torch.float64).unsqueeze(-1) * sk.to(torch.float64).unsqueeze(-2)
    n = k.shape[2]
    if kv_len is not None:
        keep = torch.arange(n)[None, :] < kv_len.to(torch.int64)[:, None]
        s = s.masked_fill(~keep[:, None, None, :], float("-inf"))
    m = s.amax(dim=-1, keepdim=True)
    m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    p = torch.exp(s - m)
    l = p.sum(dim=-1, keepdim=True)
    pv, sv_ref = p, None
    if sv is not None:
        svd = sv.to(torch.float64)
        if kv_len is not None:
            svd = torch.where(keep[:, None, :], svd, torch.zeros_like(svd))
        sv_ref = svd.amax(dim=-1, keepdim=True)
        pv = p * (svd / torch.where(sv_ref > 0, sv_ref, torch.ones_like(sv_ref))).unsqueeze(-2)
    if round_p:
        pv = e4m3_sat((pv * p_scale).to(torch.float32)).to(torch.float64) / p_scale
    if sum_rounded:
        if sv is not None or not round_p:
            raise ValueError("sum_rounded is defined for rounded probabilities without per-token scales")
        l = pv.sum(dim=-1, keepdim=True)
    o = pv @ vd
    if sv_ref is not None:
        o = o * sv_ref.unsqueeze(-1)
    lsafe = torch.where(l == 0, torch.ones_like(l), l)
    o = o / lsafe
    if return_weighted_abs:
        vabs = vd.abs() if sv is None else vd.abs() * sv.to(torch.float64).unsqueeze(-1)
        if kv_len is not None:
            vabs = torch.where(keep[:, None, :, None], vabs, torch.zeros_like(vabs))
        return o, (p @ vabs) / lsafe, vabs.sum(dim=-2, keepdim=True) / lsafe
    if out_dtype is None:
        return o
    if out_dtype == E4M3:
        return e4m3_sat(o.to(torch.float32))
    return o.to(torch.float32).to(out_dtype)


def ref_flash_attn_func(q, k, v, softmax_scale=None, batch_mask=None, apply_qk_hadamard=False, out_dtype=None,
                        round_p=True, p_scale=1.0):
    """FlashAttnFunc.forward, q8_kernels/functional/flash_attention.py:18-61: head dim padded to a multiple of
    32, V cast straight to e4m3, Q and K either cast straight (kernel scale = softmax_scale) or rotated by the
    FHT with sqrt(softmax_scale)/sqrt(D) folded into both (kernel scale = 1). Output e4m3 like the
    reference unless out_dtype says otherwise; sliced back to the original head dim. p_scale as in ref_attention
    (1 = the reference's rounding of the probabilities)."""
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    d_og = q.shape[-1]
    if d_og % 32 != 0:
        pad = 32 - d_og % 32
        q, k, v = (torch.nn.functional.pad(t.float(), [0, pad]).to(t.dtype) for t in (q, k, v))
    if _is_16bit(v):
        v = e4m3_c10(v)
    if apply_qk_hadamard:
        hd = math.sqrt(1 / q.shape[-1])
        q = ref_fht(q, hd * math.sqrt(softmax_scale), E4M3)
        k = ref_fht(k, hd * math.sqrt(softmax_scale), E4M3)
        kernel_scale = 1.0
    else:
        if _is_16bit(q):
            q = e4m3_c10(q)
        if _is_16bit(k):
            k = e4m3_c10(k)
        kernel_scale = softmax_scale
    o = ref_attention(q, k, v, kernel_scale, batch_mask, round_p=round_p,
                      out_dtype=E4M3 if out_dtype is None else out_dtype, p_scale=p_scale)
    return o[..., :d_og]


# ------------------------------------------------------------------------------------------- RMSNorm / RoPE


def ref_rms_norm(x: torch.Tensor, weights: Optional[torch.Tensor] = None, out_type: Optional[torch.dtype] = None,
                 eps: float = 0.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """y = (x * rsqrt(mean(x^2))) * w, no epsilon; returns (y, rstd). csrc/ops/rms_norm_cuda.cu:127-169;
    out_type None -> input dtype (csrc/ops/rms_norm.cpp:120-125). The mean is taken in float64 here."""
    out_type = x.dtype if out_type is None else out_type
    xf = x.to(torch.float32)
    ms = (xf.to(torch.float64) ** 2).mean(dim=-1, keepdim=True) + eps
    rstd = (1.0 / torch.sqrt(ms)).to(torch.float32)
    y = xf * rstd
    if weights is not None:
        y = y * weights.to(torch.float32)
    return cast(y, out_type), rstd.squeeze(-1)


def ref_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """Interleaved-pair rotation with per-element fp32 tables, csrc/ops/rope_cuda.cu:99-103:
        y[2i] = x[2i] cos[2i] - x[2i+1] sin[2i];   y[2i+1] = x[2i+1] cos[2i+1] + x[2i] sin[2i+1]
    (the same formula as the torch fallback q8_kernels/functional/rope.py:27-41). Products and the sum
    round separately in fp32."""
    out_type = x.dtype if out_type is None else out_type
    xf = x.to(torch.float32)
    x0, x1 = xf[..., 0::2], xf[..., 1::2]
    c0, c1 = cos[..., 0::2], cos[..., 1::2]
    s0, s1 = sin[..., 0::2], sin[..., 1::2]
    y0 = x0 * c0 - x1 * s0
    y1 = x1 * c1 + x0 * s1
    y = torch.stack((y0, y1), dim=-1).reshape(xf.shape)
    return cast(y, out_type)


def ref_freqs_cis(indices_grid: torch.Tensor, dim: int = 2048, theta: float = 10000.0,
                  max_pos=(20, 2048, 2048)) -> Tuple[torch.Tensor, torch.Tensor]:
    """3-D fractional RoPE tables, q8_kernels/models/LTXVideo.py:85-148 (spacing 'exp'):
    indices_grid [B, 3, T] -> (cos, sin) fp32 [B, T, dim]."""
    frac = torch.stack([indices_grid[:, i] / max_pos[i] for i in range(3)], dim=-1)
    idx = theta ** torch.linspace(math.log(1, theta), math.log(theta, theta), dim // 6, dtype=torch.float32)
    idx = idx * math.pi / 2
    freqs = (idx * (frac.unsqueeze(-1) * 2 - 1)).transpose(-1, -2).flatten(2)
    cos = freqs.cos().repeat_interleave(2, dim=-1)
    sin = freqs.sin().repeat_interleave(2, dim=-1)
    if dim % 6 != 0:
        cos = torch.cat([torch.ones_like(cos[:, :, : dim % 6]), cos], dim=-1)
        sin = torch.cat([torch.zeros_like(cos[:, :, : dim % 6]), sin], dim=-1)
    return cos.to(torch.float32), sin.to(torch.float32)


# ------------------------------------------------------------------------------------------- fma, GELU, backward ops


def ref_fma(x: torch.Tensor, y: torch.Tensor, z: torch.Tensor, scale_add: float = 0.0,
            out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """out = x * (y + scale_add) + z with y, z [B, T or 1, dim] broadcast over tokens, csrc/ops/fma_cuda.cu:94 and
    csrc/ops/fma.cpp:85-86; output in x's dtype (fma.cpp:99). y + scale_add rounds to fp32; the product and the
    sum round once (the expression contracts to a fused multiply-add), evaluated here in float64 where the
    product of an 8- or 16-bit x with an fp32 factor is exact."""
    out_type = x.dtype if out_type is None else out_type
    ys = (y.to(torch.float32) + torch.tensor(scale_add, dtype=torch.float32)).to(torch.float64)
    v = x.to(torch.float32).to(torch.float64) * ys + z.to(torch.float32).to(torch.float64)
    return cast(v.to(torch.float32), out_type)


def ref_gelu_forward(x: torch.Tensor, out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """tanh-GELU, csrc/ops/gelu_forward_cuda.cu:12-16; out_type None -> input dtype. Evaluated in float64."""
    out_type = x.dtype if out_type is None else out_type
    return cast(gelu_tanh(x.to(torch.float32).to(torch.float64)).to(torch.float32), out_type)


def ref_gelu_backward(x: torch.Tensor, grad_output: torch.Tensor, out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """grad * (0.5 (1 + phi) + 0.5 x phi'), phi = tanh(tau), tau = k (x + c x^3),
    phi' = (1 - phi^2) k (1 + 3 c x^2): csrc/ops/gelu_backward_cuda.cu:94-100. Evaluated in float64."""
    out_type = x.dtype if out_type is None else out_type
    k, c = 0.7978845608028654, 0.044715
    xv = x.to(torch.float32).to(torch.float64)
    g = grad_output.to(torch.float32).to(torch.float64)
    phi = torch.tanh(k * (xv + c * xv ** 3))
    dphi = (1.0 - phi * phi) * (k * (1.0 + 3.0 * c * xv * xv))
    return cast((g * (0.5 * (1.0 + phi) + 0.5 * xv * dphi)).to(torch.float32), out_type)


def ref_rope_backward(grad_out: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                      out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """The transpose of ref_rope's rotation, csrc/ops/rope_backward_cuda.cu:106-107:
        o[2i] = g[2i] cos[2i] + g[2i+1] sin[2i+1];   o[2i+1] = -g[2i] sin[2i] + g[2i+1] cos[2i+1]."""
    out_type = grad_out.dtype if out_type is None else out_type
    g = grad_out.to(torch.float32)
    g0, g1 = g[..., 0::2], g[..., 1::2]
    c0, c1 = cos[..., 0::2], cos[..., 1::2]
    s0, s1 = sin[..., 0::2], sin[..., 1::2]
    o0 = g0 * c0 + g1 * s1
    o1 = -g0 * s0 + g1 * c1
    return cast(torch.stack((o0, o1), dim=-1).reshape(g.shape), out_type)


def ref_rms_norm_backward(x_normed: torch.Tensor, x_norms: torch.Tensor, grad_out: torch.Tensor,
                          weights: Optional[torch.Tensor] = None, out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """dx = rstd / dim * (dim * g * w - y / w * sum_j g_j y_j) from the forward's outputs y = x_normed and
    rstd = x_norms: csrc/ops/rms_norm_backward_cuda.cu:140-160. Evaluated in float64."""
    out_type = x_normed.dtype if out_type is None else out_type
    y = x_normed.to(torch.float32).to(torch.float64)
    g = grad_out.to(torch.float32).to(torch.float64)
    w = torch.ones(y.shape[-1], dtype=torch.float64) if weights is None else weights.to(torch.float64)
    dim = y.shape[-1]
    dot = (g * y).sum(dim=-1, keepdim=True)
    r = x_norms.to(torch.float64).reshape(y.shape[:-1] + (1,))
    return cast((r / dim * (dim * g * w - y / w * dot)).to(torch.float32), out_type)


# ------------------------------------------------------------------------------------------- block composition


def ref_dit_block(hidden, text, freqs_cis, text_lens, params, num_heads, head_dim=64, p_scale=1.0):
    """The simplified LTX-style fp8 block of the benchmark configuration, composed from the functions above
    (op order as q8_kernels/modules/attention.py:45-106 and q8_kernels/modules/ffn.py:10-17 chain them):
    RMSNorm -> fp8 QKV -> RoPE(q, k) -> fp8 Hadamard self-attention -> out projection (+res) -> RMSNorm ->
    fp8 cross-attention with valid lengths (+res) -> RMSNorm -> fp8 FFN with fused bias+GELU (+res).
    `params[name]` = (e4m3 weight [out, in], fp32 scales [out], fp32 bias [out]); `params['norm*']` = fp32 [dim]."""
    bf16 = torch.bfloat16
    b = hidden.shape[0]
    dim = num_heads * head_dim

    def lin(name, x, gelu=False):
        w, s, bias = params[name]
        return ref_fp8_linear(x, w, bias, None, s, False, bf16, fuse_gelu=gelu)

    def heads(t):
        return t.reshape(b, -1, num_heads, head_dim).transpose(1, 2)

    def merge(t):
        return t.transpose(1, 2).reshape(b, -1, dim)

    h, _ = ref_rms_norm(hidden, params["norm1"])
    q, k, v = lin("to_qkv", h).split(dim, dim=-1)
    q, k = ref_rope(q, *freqs_cis), ref_rope(k, *freqs_cis)
    a = ref_flash_attn_func(heads(q), heads(k), heads(v), None, None, True, out_dtype=bf16, p_scale=p_scale)
    hidden = hidden + lin("to_out", merge(a))
    h, _ = ref_rms_norm(hidden, params["norm2"])
    a = ref_flash_attn_func(heads(lin("to_q2", h)), heads(lin("to_k2", text)), heads(lin("to_v2", text)), None, text_lens, True,
                            out_dtype=bf16, p_scale=p_scale)
    hidden = hidden + lin("to_out2", merge(a))
    h, _ = ref_rms_norm(hidden, params["norm3"])
    return hidden + lin("ff_down", lin("ff_up", h, gelu=True))


def ref_attention_module(p, prefix, x, num_heads, head_dim, freqs_cis=None, context=None, lens=None,
                         non_mm=torch.bfloat16, mm_out=torch.bfloat16, p_scale=1.0):
    """q8_kernels/modules/attention.py:45-106 with attn_type 'q8_kernels': int8 projections, qk-RMSNorm over the
    full inner dim, RoPE on self-attention, fp8 flash attention with Hadamard (e4m3 output), output projection.
    p[prefix + name] = (int8 weight, fp32 scales, fp32 bias or None); p[prefix + 'q_norm' / 'k_norm'] = fp32 [inner]."""
    b = x.shape[0]

    def lin(name, t):
        w, s, bias = p[prefix + name]
        return ref_q8_linear(t, w, bias, None, s, False, mm_out)

    def heads(t):
        return t.reshape(b, -1, num_heads, head_dim).transpose(1, 2)

    src = x if context is None else context
    q, k, v = lin("to_q", x), lin("to_k", src), lin("to_v", src)
    q, _ = ref_rms_norm(q, p[prefix + "q_norm"], non_mm)
    k, _ = ref_rms_norm(k, p[prefix + "k_norm"], non_mm)
    if context is None and freqs_cis is not None:
        q, k = ref_rope(q, freqs_cis[0], freqs_cis[1], non_mm), ref_rope(k, freqs_cis[0], freqs_cis[1], non_mm)
    a = ref_flash_attn_func(heads(q), heads(k), heads(v), None, lens, True, p_scale=p_scale)
    a = a.transpose(1, 2).reshape(b, -1, num_heads * head_dim)
    return lin("to_out", a).to(non_mm)


def ref_ltx_block(p, hidden, freqs_cis, context, context_lens, timestep, num_heads, head_dim, p_scale=1.0):
    """q8_kernels/blocks/ltx_transformer_block.py:21-58 with bfloat16 activations; the modulations and gated
    residuals are evaluated as fused multiply-adds (ref_fma). p['scale_shift_table'] fp32 [6, dim],
    p['norm1'] / p['norm2'] = fp32 [dim] or None, attention parameters under 'attn1.' / 'attn2.',
    feed-forward under 'ff.up' / 'ff.down'."""
    bf16 = torch.bfloat16
    b = hidden.shape[0]
    ada = p["scale_shift_table"][None, None] + timestep.reshape(b, timestep.shape[1], 6, -1)
    shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = (t.to(bf16) for t in ada.unbind(dim=2))
    h, _ = ref_rms_norm(hidden, p["norm1"], bf16)
    h = ref_fma(h, scale_msa, shift_msa, 1.0)
    a = ref_attention_module(p, "attn1.", h, num_heads, head_dim, freqs_cis, p_scale=p_scale)
    hidden = ref_fma(a, gate_msa, hidden, 0.0)
    a = ref_attention_module(p, "attn2.", hidden, num_heads, head_dim, None, context, context_lens, p_scale=p_scale)
    hidden = a + hidden
    h, _ = ref_rms_norm(hidden, p["norm2"], bf16)
    h = ref_fma(h, scale_mlp, shift_mlp, 1.0)
    w, s, bias = p["ff.up"]
    up = ref_q8_linear(h, w, bias, None, s, True, bf16)
    w, s, bias = p["ff.down"]
    ff = ref_q8_linear(up, w, bias, None, s, False, bf16).to(bf16)
    return ref_fma(ff.reshape(hidden.shape), gate_mlp, hidden, 0.0)
