"""Pins the CPU oracle (oracle/q8_oracle.py) against independent closed forms. The reference ships no
tests or golden vectors, so every oracle function is checked against something that does not share its
formula: the e4m3 bit layout, scipy's Hadamard matrix, integer matmul, torch's own gelu/SDPA, complex
rotation, brute-force loops on tiny inputs."""
import math

import numpy as np
import pytest
import scipy.linalg
import torch

from oracle import q8_oracle as O

E4M3 = torch.float8_e4m3fn


# ------------------------------------------------------------------ e4m3 casts

def _nearest_e4m3_bruteforce(vals):
    """RNE to the e4m3fn grid by exhaustive search over the 254 finite codes (ties -> even mantissa)."""
    table = O.e4m3_decode_table()
    finite = [(table[c], c) for c in range(256) if not np.isnan(table[c])]
    out = []
    for v in vals:
        if np.isnan(v):
            out.append(None)
            continue
        best, best_codes = None, []
        for t, c in finite:
            d = abs(float(v) - t)
            if best is None or d < best:
                best, best_codes = d, [c]
            elif d == best:
                best_codes.append(c)
        if len(best_codes) > 1:
            # zero has two codes; otherwise pick the even mantissa
            nz = [c for c in best_codes if table[c] != 0 or True]
            even = [c for c in nz if (c & 1) == 0]
            sign = 0x80 if np.signbit(v) else 0
            even = [c for c in even if (c & 0x80) == sign] or even
            best_codes = even
        out.append(best_codes[0])
    return out


def test_e4m3_decode_table_matches_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    t = codes.view(E4M3).to(torch.float64).numpy()
    ref = O.e4m3_decode_table()
    assert np.array_equal(np.isnan(t), np.isnan(ref))
    assert np.array_equal(t[~np.isnan(t)], ref[~np.isnan(ref)])
    assert ref[0x7E] == 448.0 and ref[0x01] == 2.0 ** -9 and ref[0x08] == 2.0 ** -6


def test_e4m3_c10_is_rne_with_nan_above_464():
    g = torch.Generator().manual_seed(1)
    vals = torch.cat([
        torch.randn(400, generator=g) * 3,
        torch.randn(200, generator=g) * 200,
        torch.randn(200, generator=g) * 0.01,
        torch.tensor([0.0, -0.0, 448.0, -448.0, 464.0, -464.0, 2.0 ** -9, 2.0 ** -10, 3 * 2.0 ** -10, 1.0625, 1.1875, 0.0009765625]),
    ]).to(torch.float32)
    got = O.e4m3_c10(vals).view(torch.uint8).numpy()
    inside = vals.abs() <= 464.0
    want = _nearest_e4m3_bruteforce(vals[inside].numpy())
    table = O.e4m3_decode_table()
    for g_code, w_code, v in zip(got[inside.numpy()], want, vals[inside].numpy()):
        assert table[g_code] == table[w_code], (v, g_code, w_code)
    # above 464: NaN code with the sign kept
    big = torch.tensor([464.0001, 465.0, 480.0, 1e6, -465.0, float("inf"), float("nan")], dtype=torch.float32)
    codes = O.e4m3_c10(big).view(torch.uint8).tolist()
    assert codes == [0x7F, 0x7F, 0x7F, 0x7F, 0xFF, 0x7F, 0x7F]


def test_e4m3_sat_clamps_and_keeps_nan():
    x = torch.tensor([500.0, -1e9, 448.0, 463.0, 3.0, float("nan"), float("inf")], dtype=torch.float32)
    codes = O.e4m3_sat(x).view(torch.uint8).tolist()
    assert codes[:5] == [0x7E, 0xFE, 0x7E, 0x7E, 0x44]
    assert codes[5] & 0x7F == 0x7F and codes[6] == 0x7E


# ------------------------------------------------------------------ FHT

@pytest.mark.parametrize("dim", [8, 16, 64, 128, 512, 2048, 4096])
def test_fht_matches_scipy_hadamard(dim):
    g = torch.Generator().manual_seed(dim)
    x = torch.randn(5, dim, generator=g).to(torch.bfloat16)
    H = torch.tensor(scipy.linalg.hadamard(dim), dtype=torch.float64)
    want = x.to(torch.float64) @ H / math.sqrt(dim)
    got = O.ref_fht(x, out_type=torch.bfloat16)
    # the docstring equivalence of the reference (fast_hadamard.py:33), up to bf16 rounding of the output
    assert torch.equal(got, (want.to(torch.float32)).to(torch.bfloat16)) or \
        (got.to(torch.float64) - want).abs().max() <= 2 ** -7 * want.abs().max()
    # exact on small integers (every partial sum is exactly representable)
    xi = torch.randint(-3, 4, (4, dim), generator=g).to(torch.bfloat16)
    got_i = O.ref_fht(xi, scale=1.0, out_type=torch.bfloat16).to(torch.float64)
    want_i = (xi.to(torch.float64) @ H).to(torch.float32).to(torch.bfloat16).to(torch.float64)
    assert torch.equal(got_i, want_i)


def test_fht_involution_and_parseval():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(3, 256, generator=g)
    xb = x.to(torch.bfloat16)
    # run in fp32 without the bf16 store in between: emulate by feeding exactly representable values
    y = O.ref_fht(xb, out_type=torch.bfloat16)
    e_in = (xb.to(torch.float64) ** 2).sum(-1)
    e_out = (y.to(torch.float64) ** 2).sum(-1)
    assert torch.allclose(e_in, e_out, rtol=2e-2)
    z = O.ref_fht(y, out_type=torch.bfloat16)
    assert (z.to(torch.float64) - xb.to(torch.float64)).abs().max() < 0.05


@pytest.mark.parametrize("dim", [24, 40, 100, 1536])
def test_fht_zero_pads_to_next_power_of_two(dim):
    g = torch.Generator().manual_seed(dim)
    x = torch.randint(-2, 3, (3, dim), generator=g).to(torch.bfloat16)
    n = 1 << (dim - 1).bit_length()
    H = torch.tensor(scipy.linalg.hadamard(n), dtype=torch.float64)
    xp = torch.zeros(3, n, dtype=torch.float64)
    xp[:, :dim] = x.to(torch.float64)
    want = (xp @ H)[:, :dim]
    got = O.ref_fht(x, scale=1.0, out_type=torch.bfloat16).to(torch.float64)
    assert torch.equal(got, want.to(torch.float32).to(torch.bfloat16).to(torch.float64))


def test_fht_fp8_output_uses_c10_cast():
    x = torch.full((1, 64), 30.0).to(torch.bfloat16)
    y = O.ref_fht(x, scale=1.0, out_type=E4M3).view(torch.uint8)
    assert y[0, 0].item() == 0x7F  # 1920 > 464 -> NaN, not saturation
    assert (y[0, 1:] == 0).all()


# ------------------------------------------------------------------ quantizer

@pytest.mark.parametrize("out_type,qmax", [(torch.int8, 127.0), (E4M3, 448.0)])
def test_quant_closed_form_properties(out_type, qmax):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(16, 256, generator=g).to(torch.bfloat16)
    codes, scales = O.ref_quant(x, out_type)
    assert codes.shape == x.shape and scales.shape == x.shape[:-1] and scales.dtype == torch.float32
    a = x.float().abs().amax(-1)
    # scale * QMAX = absmax up to 1 ulp of the two fp32 divisions
    assert torch.allclose(scales * qmax, a, rtol=3e-7)
    deq = codes.to(torch.float32) * scales[:, None]
    step = scales[:, None] * (1.0 if out_type == torch.int8 else 32.0)  # e4m3 step at the top binade is 32
    assert ((deq - x.float()).abs() <= 0.5 * step + 1e-6).all()
    # the absmax element maps to +-QMAX exactly
    idx = x.float().abs().argmax(-1)
    top = codes.to(torch.float32)[torch.arange(16), idx]
    assert (top.abs() == qmax).all()


def test_quant_rounding_modes_and_zero_row():
    # x*r lands exactly on .5 -> half-away vs half-even differ
    x = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -2.5, 0.0, 3.0]], dtype=torch.float32)
    away, s = O.ref_quant(x, torch.int8)
    even, _ = O.ref_quant(x, torch.int8, round_half_even=True)
    assert away.tolist() == [[127, 1, 2, 3, -1, -3, 0, 3]]
    assert even.tolist() == [[127, 0, 2, 2, 0, -2, 0, 3]]
    assert s.item() == 1.0
    z = torch.zeros(2, 8, dtype=torch.bfloat16)
    for t in (torch.int8, E4M3):
        c, sc = O.ref_quant(z, t)
        assert (c.view(torch.uint8) == 0).all() and (sc == 0).all()


def test_quant_scale_forms_agree_to_one_ulp():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(64, 64, generator=g).to(torch.bfloat16)
    c1, s1 = O.ref_quant(x, E4M3)
    c2, s2 = O.ref_quant(x, E4M3, scale_as_division=True)
    assert torch.equal(c1.view(torch.uint8), c2.view(torch.uint8))
    ulp = torch.abs(s1) * 2 ** -23
    assert ((s1 - s2).abs() <= ulp).all()
    assert torch.equal(s2, x.float().abs().amax(-1) / 448.0)


# ------------------------------------------------------------------ GEMM

def test_gemm_i32_exact_against_integer_matmul():
    g = torch.Generator().manual_seed(11)
    a = torch.randint(-128, 128, (37, 96), generator=g, dtype=torch.int8)
    b = torch.randint(-128, 128, (29, 96), generator=g, dtype=torch.int8)
    want = a.numpy().astype(np.int64) @ b.numpy().astype(np.int64).T
    got = O.ref_gemm_i32(a, b)
    assert got.dtype == torch.int32 and np.array_equal(got.numpy().astype(np.int64), want)
    # worst case magnitude stays exact
    a2 = torch.full((2, 4096), -128, dtype=torch.int8)
    assert O.ref_gemm_i32(a2, a2)[0, 0].item() == 128 * 128 * 4096


def test_gemm_fp8_acc_matches_bruteforce():
    g = torch.Generator().manual_seed(12)
    a = O.e4m3_c10(torch.randn(5, 32, generator=g) * 4)
    b = O.e4m3_c10(torch.randn(6, 32, generator=g) * 4)
    tab = O.e4m3_decode_table()
    av, bv = tab[a.view(torch.uint8).numpy()], tab[b.view(torch.uint8).numpy()]
    want = np.array([[sum(av[i, k] * bv[j, k] for k in range(32)) for j in range(6)] for i in range(5)])
    assert np.allclose(O.ref_gemm_fp8_acc(a, b).numpy(), want, rtol=0, atol=1e-9)


def test_epilogue_matches_torch_gelu_and_casts():
    g = torch.Generator().manual_seed(13)
    acc = torch.randint(-20000, 20000, (2, 7, 9), generator=g, dtype=torch.int32)
    sa = torch.rand(2, 7, generator=g) * 1e-2
    sb = torch.rand(1, 9, generator=g) * 1e-2
    bias = torch.randn(9, generator=g)
    v = acc.double() * (sa.float()[..., :, None] * sb.float()[..., None, :]).double() + bias.double()
    want = torch.nn.functional.gelu(v, approximate="tanh")
    got = O.ref_epilogue(acc, sa, sb, bias, True, torch.bfloat16)
    assert got.dtype == torch.bfloat16
    assert (got.double() - want).abs().max() <= 2 ** -8 * want.abs().max() + 1e-6
    # no gelu, e4m3 default output saturates
    big = O.ref_epilogue(torch.tensor([[[10 ** 6, -10 ** 6, 3]]]), torch.ones(1, 1), torch.ones(1, 3), None, False, None)
    assert big.dtype == E4M3 and big.view(torch.uint8).tolist() == [[[0x7E, 0xFE, 0x44]]]


def test_mm_batch_broadcast_shapes():
    g = torch.Generator().manual_seed(14)
    a = torch.randint(-5, 6, (3, 4, 16), generator=g, dtype=torch.int8)
    b = torch.randint(-5, 6, (8, 16), generator=g, dtype=torch.int8)
    sa, sb = torch.ones(3, 4), torch.ones(8)
    out = O.ref_q8_mm(a, b, None, sa, sb, False, torch.bfloat16)
    assert out.shape == (3, 4, 8)
    want = torch.einsum("zmk,nk->zmn", a.double(), b.double())
    assert torch.equal(out.double(), want)
    out2 = O.ref_q8_mm(a[0], b, None, sa[0], sb, False, torch.bfloat16)
    assert out2.shape == (1, 4, 8)


def test_linear_compositions_reduce_to_plain_matmul():
    """(xH)(WH)^T = xW^T for the orthonormal rotation: both linears approximate the bf16 linear."""
    g = torch.Generator().manual_seed(15)
    x = torch.randn(2, 16, 128, generator=g).to(torch.bfloat16)
    w = (torch.randn(32, 128, generator=g) * 0.05).to(torch.bfloat16)
    bias = torch.randn(32, generator=g) * 0.1
    want = x.double() @ w.double().T + bias.double()
    for out in (O.ref_q8_linear(x, w, bias, out_dtype=torch.bfloat16),
                O.ref_fp8_linear(x, w, bias, out_dtype=torch.bfloat16),
                O.ref_fp8_linear(x, w, bias, use_hadamard=True, out_dtype=torch.bfloat16)):
        assert out.shape == (2, 16, 32)
        cos = torch.nn.functional.cosine_similarity(out.double().flatten(), want.flatten(), dim=0)
        assert cos > 0.995


# ------------------------------------------------------------------ attention

def test_attention_unrounded_equals_torch_sdpa():
    g = torch.Generator().manual_seed(21)
    q = O.e4m3_c10(torch.randn(2, 3, 40, 64, generator=g))
    k = O.e4m3_c10(torch.randn(2, 3, 50, 64, generator=g))
    v = O.e4m3_c10(torch.randn(2, 3, 50, 64, generator=g))
    lens = torch.tensor([50, 17], dtype=torch.int32)
    got = O.ref_attention(q, k, v, 0.125, lens, round_p=False)
    keep = torch.arange(50)[None, :] < lens[:, None]
    mask = torch.zeros(2, 1, 1, 50, dtype=torch.float64).masked_fill(~keep[:, None, None, :], float("-inf"))
    want = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double(), attn_mask=mask, scale=0.125)
    assert torch.allclose(got, want, atol=1e-12)


def test_attention_rounded_p_invariants():
    g = torch.Generator().manual_seed(22)
    q = O.e4m3_c10(torch.randn(1, 2, 33, 64, generator=g))
    k = O.e4m3_c10(torch.randn(1, 2, 70, 64, generator=g))
    v = O.e4m3_c10(torch.randn(1, 2, 70, 64, generator=g))
    lens = torch.tensor([41], dtype=torch.int32)
    o = O.ref_attention(q, k, v, 0.125, lens)  # the reference's grid: p <= 1
    exact, wabs, uabs = O.ref_attention(q, k, v, 0.125, lens, round_p=False, return_weighted_abs=True)
    # e4m3 rounding of p is a <= 2^-4 relative (normal range) / 2^-10 absolute (below it) perturbation of each weight
    assert ((o - exact).abs() <= 2.0 ** -4 * wabs + 2.0 ** -10 * uabs + 1e-12).all()
    assert torch.equal(o, O.ref_attention(q, k, v, 0.125, lens, p_scale=1.0)), "the default is the reference's p_scale = 1"
    # probabilities scaled by 2^8 before the cast (the HIP kernel's default): the subnormal floor drops to 2^-18
    o256 = O.ref_attention(q, k, v, 0.125, lens, p_scale=256.0)
    assert ((o256 - exact).abs() <= 2.0 ** -4 * wabs + 2.0 ** -18 * uabs + 1e-12).all()
    # masked keys carry no weight: changing them changes nothing
    v2 = v.clone().view(torch.uint8)
    v2[:, :, 41:, :] = 0x7E
    k2 = k.clone().view(torch.uint8)
    k2[:, :, 41:, :] = 0x30
    o2 = O.ref_attention(q, k2.view(E4M3), v2.view(E4M3), 0.125, lens)
    assert torch.equal(o, o2)
    # fully masked batch -> zeros (l = 0 divides by 1)
    oz = O.ref_attention(q, k, v, 0.125, torch.tensor([0], dtype=torch.int32))
    assert (oz == 0).all()
    # per-token scales are plain dequantisation
    sq, sk, sv = torch.rand(1, 2, 33, generator=g) + 0.5, torch.rand(1, 2, 70, generator=g) + 0.5, torch.rand(1, 2, 70, generator=g) + 0.5
    os_ = O.ref_attention(q, k, v, 0.125, lens, sq, sk, sv, round_p=False)
    want = O.ref_attention(q.double() * sq[..., None], k.double() * sk[..., None], v.double() * sv[..., None], 0.125, lens, round_p=False)
    assert torch.allclose(os_, want, atol=1e-10)


def test_attention_sum_of_rounded_probabilities_is_a_convex_combination():
    """sum_rounded=True normalises by the weights that multiply V: a V whose rows are all equal comes back exactly,
    whatever the rounding did to the weights (the default, which sums the unrounded ones, does not), every output lies
    inside the per-channel range of the valid v_j, and the distance to exact attention obeys the bound of a 2^-4
    perturbation of the weights in numerator and denominator."""
    g = torch.Generator().manual_seed(24)
    q = O.e4m3_c10(torch.randn(1, 2, 33, 64, generator=g) * 2)
    k = O.e4m3_c10(torch.randn(1, 2, 70, 64, generator=g) * 2)
    row = O.e4m3_c10(torch.randn(64, generator=g))
    v_const = row.expand(1, 2, 70, 64).contiguous()
    lens = torch.tensor([41], dtype=torch.int32)
    o = O.ref_attention(q, k, v_const, 0.125, lens, sum_rounded=True)
    assert torch.allclose(o, row.double().expand_as(o), rtol=1e-14, atol=0)
    plain = O.ref_attention(q, k, v_const, 0.125, lens)
    assert (plain - row.double()).abs().max() > 1e-4
    v = O.e4m3_c10(torch.randn(1, 2, 70, 64, generator=g))
    o = O.ref_attention(q, k, v, 0.125, lens, sum_rounded=True, p_scale=256.0)
    lo, hi = v[:, :, :41].double().amin(dim=2, keepdim=True), v[:, :, :41].double().amax(dim=2, keepdim=True)
    assert (o >= lo - 1e-12).all() and (o <= hi + 1e-12).all()
    exact, wabs, uabs = O.ref_attention(q, k, v, 0.125, lens, round_p=False, return_weighted_abs=True)
    eps = 2.0 ** -4
    assert ((o - exact).abs() <= (eps * wabs + 2.0 ** -18 * uabs + eps * exact.abs()) / (1 - eps) + 1e-12).all()
    with pytest.raises(ValueError):
        O.ref_attention(q, k, v, 0.125, lens, torch.ones(1, 2, 33), torch.ones(1, 2, 70), torch.ones(1, 2, 70), sum_rounded=True)


def test_flash_attn_func_hadamard_identity():
    """(Hq).(Hk)/D = q.k: with the rotation the result approximates plain attention on the bf16 inputs."""
    g = torch.Generator().manual_seed(23)
    q = torch.randn(1, 2, 48, 64, generator=g).to(torch.bfloat16)
    k = torch.randn(1, 2, 80, 64, generator=g).to(torch.bfloat16)
    v = torch.randn(1, 2, 80, 64, generator=g).to(torch.bfloat16)
    want = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double())
    for had in (False, True):
        o = O.ref_flash_attn_func(q, k, v, apply_qk_hadamard=had, out_dtype=torch.bfloat16)
        assert o.shape == q.shape and o.dtype == torch.bfloat16
        cos = torch.nn.functional.cosine_similarity(o.double().flatten(), want.flatten(), dim=0)
        assert cos > 0.99
    assert O.ref_flash_attn_func(q, k, v).dtype == E4M3


# ------------------------------------------------------------------ RMSNorm / RoPE / tables

def test_rms_norm_closed_form():
    g = torch.Generator().manual_seed(31)
    x = torch.randn(6, 128, generator=g).to(torch.bfloat16)
    w = torch.rand(128, generator=g) + 0.5
    y, rstd = O.ref_rms_norm(x, w, torch.bfloat16)
    xd = x.double()
    want_r = 1.0 / np.sqrt((xd.numpy() ** 2).mean(-1))
    assert np.allclose(rstd.numpy(), want_r, rtol=1e-6)
    want = xd * torch.tensor(want_r)[:, None] * w.double()
    assert (y.double() - want).abs().max() <= 2 ** -8 * want.abs().max() + 1e-6
    y1, _ = O.ref_rms_norm(x, None, None)
    assert y1.dtype == torch.bfloat16
    # unit RMS after normalisation
    assert torch.allclose((y1.double() ** 2).mean(-1), torch.ones(6, dtype=torch.float64), atol=2e-2)


def test_rope_is_complex_rotation():
    g = torch.Generator().manual_seed(32)
    x = torch.randn(2, 5, 32, generator=g).to(torch.bfloat16)
    ang = torch.rand(2, 5, 16, generator=g) * 6.28
    cos = ang.cos().repeat_interleave(2, -1)
    sin = ang.sin().repeat_interleave(2, -1)
    y = O.ref_rope(x, cos, sin, torch.bfloat16)
    z = torch.view_as_complex(x.float().reshape(2, 5, 16, 2).contiguous()) * torch.polar(torch.ones_like(ang), ang)
    want = torch.view_as_real(z).reshape(2, 5, 32)
    assert (y.float() - want).abs().max() <= 2 ** -8 * want.abs().max() + 1e-6
    # per-element tables: the odd/even entries may differ, follow the formula literally
    cos2, sin2 = torch.randn(1, 1, 4, generator=g), torch.randn(1, 1, 4, generator=g)
    xx = torch.tensor([[[1.0, 2.0, 3.0, 4.0]]]).to(torch.bfloat16)
    yy = O.ref_rope(xx, cos2, sin2, torch.bfloat16).float()[0, 0]
    c, s = cos2[0, 0], sin2[0, 0]
    want2 = torch.stack([1 * c[0] - 2 * s[0], 2 * c[1] + 1 * s[1], 3 * c[2] - 4 * s[2], 4 * c[3] + 3 * s[3]])
    assert torch.equal(yy, want2.to(torch.bfloat16).float())


def test_freqs_cis_against_loops():
    dim, theta, max_pos = 26, 100.0, (20, 2048, 2048)
    grid = torch.tensor([[[0.0, 3.0], [5.0, 100.0], [7.0, 2047.0]]])  # [1, 3, 2]
    cos, sin = O.ref_freqs_cis(grid, dim, theta, max_pos)
    assert cos.shape == (1, 2, dim) and cos.dtype == torch.float32
    nf = dim // 6
    for t in range(2):
        assert cos[0, t, 0] == 1 and cos[0, t, 1] == 1 and sin[0, t, 0] == 0 and sin[0, t, 1] == 0  # dim % 6 = 2 pad
        for f in range(nf):
            w = theta ** (f / (nf - 1)) * math.pi / 2
            for axis in range(3):
                frac = grid[0, axis, t].item() / max_pos[axis]
                a = w * (2 * frac - 1)
                col = 2 + 2 * (f * 3 + axis)
                assert abs(cos[0, t, col].item() - math.cos(a)) < 1e-5
                assert cos[0, t, col] == cos[0, t, col + 1]
                assert abs(sin[0, t, col].item() - math.sin(a)) < 1e-5


# ------------------------------------------------------------------ fma, GELU, backward operators

def test_fma_against_exact_rational_arithmetic():
    from fractions import Fraction
    g = torch.Generator().manual_seed(31)
    x = O.e4m3_c10(torch.randn(2, 3, 8, generator=g) * 3)
    y = torch.randn(2, 1, 8, generator=g)
    z = O.e4m3_c10(torch.randn(2, 3, 8, generator=g))
    got = O.ref_fma(x, y, z, 1.0).view(torch.uint8)
    table = O.e4m3_decode_table()
    finite = [(float(table[c]), c) for c in range(256) if np.isfinite(table[c])]
    for b in range(2):
        for t in range(3):
            for i in range(8):
                ys = float((y[b, 0, i] + torch.tensor(1.0)).item())  # the fp32 sum y + scale_add
                exact = Fraction(float(x[b, t, i])) * Fraction(ys) + Fraction(float(z[b, t, i]))
                # nearest e4m3 value of the exact result (no tie and far from the fp32 rounding step in these data)
                best = min(finite, key=lambda vc: abs(Fraction(vc[0]) - exact))
                assert table[int(got[b, t, i])] == best[0], (b, t, i)


def test_fma_broadcast_and_dtypes():
    g = torch.Generator().manual_seed(32)
    x = (torch.randn(2, 5, 16, generator=g)).to(torch.bfloat16)
    y = torch.randn(2, 1, 16, generator=g).to(torch.bfloat16)
    z = torch.randn(2, 5, 16, generator=g).to(torch.bfloat16)
    want = (x.double() * (y.float() + 1.0).double() + z.double()).float().to(torch.bfloat16)
    assert torch.equal(O.ref_fma(x, y, z, 1.0), want)


def test_gelu_backward_is_the_derivative_of_gelu_forward():
    g = torch.Generator().manual_seed(33)
    x = (torch.randn(4, 64, generator=g) * 2).to(torch.bfloat16)
    go = torch.randn(4, 64, generator=g).to(torch.bfloat16)
    xd = x.double().requires_grad_(True)
    torch.nn.functional.gelu(xd, approximate="tanh").backward(go.double())
    got = O.ref_gelu_backward(x, go, torch.bfloat16)
    assert torch.equal(got, xd.grad.float().to(torch.bfloat16))
    fwd = O.ref_gelu_forward(x, torch.bfloat16)
    assert torch.equal(fwd, torch.nn.functional.gelu(x.double(), approximate="tanh").float().to(torch.bfloat16))


def test_rope_backward_is_the_adjoint_of_rope():
    g = torch.Generator().manual_seed(34)
    x = torch.randn(3, 32, generator=g)
    go = torch.randn(3, 32, generator=g)
    cos, sin = torch.randn(3, 32, generator=g), torch.randn(3, 32, generator=g)  # unequal within pairs on purpose
    # <rope(x), g> == <x, rope_backward(g)> for every x, g
    lhs = (O.ref_rope(x.to(torch.bfloat16), cos, sin, torch.float32).double() * go.to(torch.bfloat16).double()).sum()
    rhs = (x.to(torch.bfloat16).double() * O.ref_rope_backward(go.to(torch.bfloat16), cos, sin, torch.float32).double()).sum()
    assert abs(float(lhs - rhs)) < 1e-4 * max(1.0, abs(float(lhs)))
    # and against float64 autograd of the forward formula
    gb = go.to(torch.bfloat16)
    xd = x.double().requires_grad_(True)
    y0 = xd[:, 0::2] * cos[:, 0::2].double() - xd[:, 1::2] * sin[:, 0::2].double()
    y1 = xd[:, 1::2] * cos[:, 1::2].double() + xd[:, 0::2] * sin[:, 1::2].double()
    torch.stack((y0, y1), -1).reshape(3, 32).backward(gb.double())
    got = O.ref_rope_backward(gb, cos, sin, torch.float32)
    assert torch.allclose(got.double(), xd.grad, rtol=1e-6, atol=1e-6)


def test_rms_norm_backward_against_autograd():
    g = torch.Generator().manual_seed(35)
    for with_w in (False, True):
        x = torch.randn(5, 48, generator=g, dtype=torch.float64)
        w = (1 + 0.2 * torch.randn(48, generator=g)).float() if with_w else None
        go = torch.randn(5, 48, generator=g, dtype=torch.float64)
        xd = x.clone().requires_grad_(True)
        rstd = 1.0 / torch.sqrt((xd ** 2).mean(-1, keepdim=True))
        y = xd * rstd * (w.double() if with_w else 1.0)
        y.backward(go)
        # feed the formula with exact (float64 -> fp32) forward outputs; fp32 operands are not a kernel type, so
        # the oracle is called with out_type float32 on bf16-free data through its float path
        got = O.ref_rms_norm_backward(y.detach().float(), rstd.detach().float().squeeze(-1), go.float(), w, torch.float32)
        assert torch.allclose(got.double(), xd.grad, rtol=2e-5, atol=2e-6)


def test_quant_nan_elements_do_not_touch_the_rest_of_the_row():
    """fmaxf semantics of the reference's row maximum (csrc/quantizer/tokenwise_quant_cuda.cu:115-132), pinned without
    the oracle's own formula: the row with its NaN elements replaced by zeros (which cannot be the maximum) must give the
    same scale and the same codes everywhere else; the NaN elements themselves come out as e4m3 NaN codes. An infinite
    element: infinite scale, zero codes for the finite elements, a NaN code for itself (inf * 0)."""
    g = torch.Generator().manual_seed(21)
    x = (torch.randn(6, 64, generator=g) * 3).to(torch.bfloat16)
    nan_at = [(1, 5), (3, 0), (3, 63), (4, 17)]
    for r, c in nan_at:
        x[r, c] = float("nan")
    clean = torch.where(x.isnan(), torch.zeros_like(x), x)
    keep = ~x.isnan()
    for out_type in (torch.int8, O.E4M3):
        codes, scales = O.ref_quant(x, out_type)
        want_codes, want_scales = O.ref_quant(clean, out_type)
        assert torch.equal(scales, want_scales)
        view = (lambda t: t.view(torch.uint8)) if out_type == O.E4M3 else (lambda t: t)
        assert torch.equal(view(codes)[keep], view(want_codes)[keep])
        if out_type == O.E4M3:
            assert all((int(view(codes)[r, c]) & 0x7F) == 0x7F for r, c in nan_at)
    y = (torch.randn(2, 32, generator=g)).to(torch.bfloat16)
    y[0, 3] = float("inf")
    y[1, 9] = float("-inf")
    codes, scales = O.ref_quant(y, O.E4M3)
    assert torch.isinf(scales).all()
    u = codes.view(torch.uint8)
    finite = ~y.isinf()
    assert ((u[finite] & 0x7F) == 0).all()            # +-0
    assert ((u[~finite] & 0x7F) == 0x7F).all()        # NaN


# ------------------------------------------------------------------ block compositions against dense float64
#
# ref_attention_module, ref_ltx_block and ref_dit_block chain the operators above; what they decide is ORDER:
# which modulation row is the shift and which the scale, which residual is gated, whether the qk-norm comes before
# the rotation, which attention is rotated at all. They are pinned here against a dense float64 evaluation written
# from the text of q8_kernels/blocks/ltx_transformer_block.py:21-58, q8_kernels/modules/attention.py:45-106 and
# q8_kernels/modules/ffn.py:10-17 with the ORIGINAL (unquantized) weights: plain x @ W.T, softmax, no rotation, no
# quantization. Every mutant of that evaluation (swapped shift / scale, a missing gate, ...) must be rejected.

def _cos(a, b):
    return torch.nn.functional.cosine_similarity(a.double().flatten(), b.double().flatten(), dim=0).item()


def _dense_rms(x, w=None):
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True))
    return y if w is None else y * w.double()


def _dense_rope(x, cos, sin):
    """Pairs (x[2i], x[2i+1]) as complex numbers times exp(i phi); the tables repeat every value twice."""
    z = torch.view_as_complex(x.reshape(x.shape[:-1] + (-1, 2)).contiguous())
    rot = torch.complex(cos[..., 0::2].double(), sin[..., 0::2].double())
    return torch.view_as_real(z * rot).reshape(x.shape)


def _dense_mha(q, k, v, heads, hd, lens=None):
    b = q.shape[0]
    split = lambda t: t.reshape(b, -1, heads, hd).transpose(1, 2)  # noqa: E731
    q, k, v = split(q), split(k), split(v)
    s = q @ k.transpose(-1, -2) / math.sqrt(hd)
    if lens is not None:
        keep = torch.arange(k.shape[2])[None, :] < lens.to(torch.int64)[:, None]
        s = s.masked_fill(~keep[:, None, None, :], float("-inf"))
    return (torch.softmax(s, dim=-1) @ v).transpose(1, 2).reshape(b, -1, heads * hd)


def _dense_attention_module(W, prefix, x, heads, hd, freqs=None, ctx=None, lens=None, mutate=""):
    """modules/attention.py:45-106: projections, qk-RMSNorm over the whole inner dim, rotation of q and k in
    self-attention only, softmax attention with the valid-length mask, output projection."""
    lin = lambda n, t: t @ W[prefix + n][0].double().T + W[prefix + n][1].double()  # noqa: E731
    src = x if ctx is None else ctx
    q, k, v = lin("to_q", x), lin("to_k", src), lin("to_v", src)
    if mutate == "norm_after_rope" and ctx is None:
        q, k = _dense_rope(q, *freqs), _dense_rope(k, *freqs)
    q, k = _dense_rms(q, W[prefix + "q_norm"]), _dense_rms(k, W[prefix + "k_norm"])
    if mutate == "no_qk_norm_weight":
        q, k = _dense_rms(lin("to_q", x)), _dense_rms(lin("to_k", src))
    rope_here = (ctx is None and mutate != "norm_after_rope" and mutate != "no_rope") or (ctx is not None and mutate == "rope_cross")
    if rope_here:
        q = _dense_rope(q, *freqs)
        if ctx is None:
            k = _dense_rope(k, *freqs)
    if mutate == "swap_kv":
        k, v = v, k
    return lin("to_out", _dense_mha(q, k, v, heads, hd, None if mutate == "no_mask" else lens))


def _dense_ltx_block(W, hidden, freqs, ctx, lens, timestep, heads, hd, mutate=""):
    """blocks/ltx_transformer_block.py:21-58 in float64."""
    b = hidden.shape[0]
    ada = W["scale_shift_table"].double()[None, None] + timestep.double().reshape(b, timestep.shape[1], 6, -1)
    shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = ada.unbind(dim=2)
    if mutate == "swap_shift_scale":
        shift_msa, scale_msa, shift_mlp, scale_mlp = scale_msa, shift_msa, scale_mlp, shift_mlp
    if mutate == "swap_msa_mlp":
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = shift_mlp, scale_mlp, gate_mlp, shift_msa, scale_msa, gate_msa
    one = 0.0 if mutate == "scale_without_one" else 1.0
    h = hidden.double()
    n = _dense_rms(h) * (one + scale_msa) + shift_msa
    a = _dense_attention_module(W, "attn1.", n, heads, hd, freqs, mutate=mutate)
    h = (a if mutate == "no_gate_msa" else gate_msa * a) + h
    a = _dense_attention_module(W, "attn2.", h, heads, hd, freqs, ctx.double(), lens, mutate=mutate)
    h = (gate_msa * a if mutate == "gate_on_cross" else a) + h
    n = _dense_rms(h) * (one + scale_mlp) + shift_mlp
    up = torch.nn.functional.gelu(n @ W["ff.up"][0].double().T + W["ff.up"][1].double(), approximate="none" if mutate == "no_gelu" else "tanh")
    if mutate == "no_gelu":
        up = n @ W["ff.up"][0].double().T + W["ff.up"][1].double()
    ff = up @ W["ff.down"][0].double().T + W["ff.down"][1].double()
    return (ff if mutate == "no_gate_mlp" else gate_mlp * ff) + h


def _ltx_case(seed=71, dim=256, heads=4, hd=64, kv_dim=128, s_tok=48, s_txt=24):
    """Dense weights W[name] = (weight, bias), and the quantized parameter dict the oracle block takes: int8 codes of
    the rotated weight with per-row scales, as Q8Linear.from_linear stores them (modules/linear.py:36-49)."""
    g = torch.Generator().manual_seed(seed)
    bf16 = torch.bfloat16
    W, P = {}, {}
    shapes = {"to_q": (dim, dim), "to_k": (dim, kv_dim), "to_v": (dim, kv_dim), "to_out": (dim, dim)}
    for a in ("attn1.", "attn2."):
        for n, (o, i) in shapes.items():
            i = dim if (a == "attn1." or n in ("to_q", "to_out")) else i
            W[a + n] = ((torch.randn(o, i, generator=g) / math.sqrt(i)).to(bf16), torch.randn(o, generator=g) * 0.1)
        for n in ("q_norm", "k_norm"):
            W[a + n] = P[a + n] = torch.rand(dim, generator=g) * 1.6 + 0.2  # uneven inside a rotated pair: the norm does not commute with the rotation
    W["ff.up"] = ((torch.randn(4 * dim, dim, generator=g) / math.sqrt(dim)).to(bf16), torch.randn(4 * dim, generator=g) * 0.1)
    W["ff.down"] = ((torch.randn(dim, 4 * dim, generator=g) / math.sqrt(4 * dim)).to(bf16), torch.randn(dim, generator=g) * 0.1)
    for n, val in list(W.items()):
        if isinstance(val, tuple):
            codes, scales = O.ref_quant(O.ref_fht(val[0]))
            P[n] = (codes, scales, val[1])
    W["scale_shift_table"] = P["scale_shift_table"] = torch.randn(6, dim, generator=g) / dim ** 0.5
    P["norm1"] = P["norm2"] = None
    hidden = torch.randn(2, s_tok, dim, generator=g).to(bf16)
    ctx = torch.randn(2, s_txt, kv_dim, generator=g).to(bf16)
    timestep = torch.randn(2, 1, 6 * dim, generator=g) * 0.5
    grid = torch.stack(torch.meshgrid(torch.arange(2), torch.arange(4), torch.arange(6), indexing="ij")).reshape(3, -1)
    freqs = O.ref_freqs_cis(grid[None].float().repeat(2, 1, 1), dim)
    lens = torch.tensor([24, 7], dtype=torch.int32)
    return W, P, hidden, freqs, ctx, lens, timestep, heads, hd


LTX_MUTANTS = ["swap_shift_scale", "swap_msa_mlp", "scale_without_one", "no_gate_msa", "gate_on_cross", "no_gate_mlp",
               "no_gelu", "norm_after_rope", "no_rope", "rope_cross", "no_mask", "swap_kv", "no_qk_norm_weight"]


def test_ltx_block_composition_against_dense_float64():
    W, P, hidden, freqs, ctx, lens, timestep, heads, hd = _ltx_case()
    got = O.ref_ltx_block(P, hidden, freqs, ctx, lens, timestep, heads, hd)
    assert got.shape == hidden.shape and got.dtype == torch.bfloat16
    want = _dense_ltx_block(W, hidden, freqs, ctx, lens, timestep, heads, hd)
    clean = _cos(got, want)
    assert clean >= 0.99, clean
    rel = ((got.double() - want).norm() / want.norm()).item()
    # every mutant of the dense evaluation is further from the oracle than the 8-bit noise of the clean one
    for mut in LTX_MUTANTS:
        bad = _dense_ltx_block(W, hidden, freqs, ctx, lens, timestep, heads, hd, mutate=mut)
        rel_bad = ((got.double() - bad).norm() / bad.norm()).item()
        assert rel_bad > 1.5 * rel and _cos(got, bad) < clean, (mut, rel_bad, rel, _cos(got, bad), clean)


def test_attention_module_composition_against_dense_float64():
    W, P, hidden, freqs, ctx, lens, timestep, heads, hd = _ltx_case(seed=72)
    for prefix, kw_o, kw_d in (("attn1.", dict(freqs_cis=freqs), dict(freqs=freqs)),
                               ("attn2.", dict(context=ctx, lens=lens), dict(freqs=freqs, ctx=ctx.double(), lens=lens))):
        got = O.ref_attention_module(P, prefix, hidden, heads, hd, **kw_o)
        want = _dense_attention_module(W, prefix, hidden.double(), heads, hd, **kw_d)
        assert got.shape == want.shape and got.dtype == torch.bfloat16
        clean = _cos(got, want)
        assert clean >= 0.99, (prefix, clean)
        rel = ((got.double() - want).norm() / want.norm()).item()
        muts = ["norm_after_rope", "no_rope", "swap_kv", "no_qk_norm_weight"] if prefix == "attn1." else ["rope_cross", "no_mask", "swap_kv", "no_qk_norm_weight"]
        for mut in muts:
            bad = _dense_attention_module(W, prefix, hidden.double(), heads, hd, mutate=mut, **kw_d)
            rel_bad = ((got.double() - bad).norm() / bad.norm()).item()
            assert rel_bad > 2.0 * rel, (prefix, mut, rel_bad, rel)


def _dense_dit_block(W, hidden, text, freqs, lens, heads, hd, mutate=""):
    """RMSNorm -> QKV -> rotation of q, k -> self-attention -> out projection (+ residual) -> RMSNorm -> cross-attention
    with valid lengths (+ residual) -> RMSNorm -> FFN with tanh-GELU (+ residual), all in float64 on dense weights."""
    lin = lambda n, t: t @ W[n][0].double().T + W[n][1].double()  # noqa: E731
    dim = heads * hd
    h = hidden.double()
    q, k, v = lin("to_qkv", _dense_rms(h, W["norm1"])).split(dim, dim=-1)
    if mutate == "qkv_order":
        k, q, v = q, k, v
    if mutate != "no_rope":
        q, k = _dense_rope(q, *freqs), _dense_rope(k, *freqs)
    a = lin("to_out", _dense_mha(q, k, v, heads, hd))
    h = a if mutate == "no_residual1" else h + a
    n = _dense_rms(h, W["norm2"])
    t = text.double()
    a = _dense_mha(lin("to_q2", n), lin("to_k2", t), lin("to_v2", t), heads, hd, None if mutate == "no_mask" else lens)
    h = h + lin("to_out2", a)
    n = _dense_rms(h, W["norm1" if mutate == "wrong_norm" else "norm3"])
    up = lin("ff_up", n)
    if mutate != "no_gelu":
        up = torch.nn.functional.gelu(up, approximate="tanh")
    ff = lin("ff_down", up)
    return ff if mutate == "no_residual3" else h + ff


def test_dit_block_composition_against_dense_float64():
    g = torch.Generator().manual_seed(73)
    bf16 = torch.bfloat16
    dim, heads, hd, ffn, s_tok, s_txt = 256, 4, 64, 512, 48, 24
    W, P = {}, {}
    for n, (o, i) in {"to_qkv": (3 * dim, dim), "to_out": (dim, dim), "to_q2": (dim, dim), "to_k2": (dim, dim), "to_v2": (dim, dim),
                      "to_out2": (dim, dim), "ff_up": (ffn, dim), "ff_down": (dim, ffn)}.items():
        W[n] = ((torch.randn(o, i, generator=g) / math.sqrt(i)).to(bf16), torch.randn(o, generator=g) * 0.1)
        codes, scales = O.ref_quant(W[n][0], E4M3)
        P[n] = (codes, scales, W[n][1])
    for n in ("norm1", "norm2", "norm3"):
        W[n] = P[n] = torch.rand(dim, generator=g) + 0.5
    hidden = torch.randn(2, s_tok, dim, generator=g).to(bf16)
    text = torch.randn(2, s_txt, dim, generator=g).to(bf16)
    grid = torch.stack(torch.meshgrid(torch.arange(2), torch.arange(4), torch.arange(6), indexing="ij")).reshape(3, -1)
    freqs = O.ref_freqs_cis(grid[None].float().repeat(2, 1, 1), dim)
    lens = torch.tensor([24, 5], dtype=torch.int32)
    got = O.ref_dit_block(hidden, text, freqs, lens, P, heads, hd)
    want = _dense_dit_block(W, hidden, text, freqs, lens, heads, hd)
    assert got.shape == hidden.shape and got.dtype == bf16
    clean = _cos(got, want)
    assert clean >= 0.99, clean
    rel = ((got.double() - want).norm() / want.norm()).item()
    for mut in ("qkv_order", "no_rope", "no_residual1", "no_mask", "wrong_norm", "no_gelu", "no_residual3"):
        bad = _dense_dit_block(W, hidden, text, freqs, lens, heads, hd, mutate=mut)
        rel_bad = ((got.double() - bad).norm() / bad.norm()).item()
        assert rel_bad > 2.0 * rel and _cos(got, bad) < clean, (mut, rel_bad, rel)
