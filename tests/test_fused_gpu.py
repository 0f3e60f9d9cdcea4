"""GPU parity of the fused row kernels (FHT+quantizer, RMSNorm+quantizer, attention prologues) through
q8_kernels_amd._C -> libq8_hip.so. Each fused kernel must return the same bits as the CPU oracle's composition
of the separate operators (and therefore as the separate HIP kernels, which are checked on their own)."""
import pytest
import torch

from oracle import q8_oracle as O
from tests.util import E4M3, assert_bit_equal

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _C():
    from q8_kernels_amd import _C as C
    return C


# ------------------------------------------------------------------ FHT -> quantizer

@pytest.mark.parametrize("dim", [64, 512, 1000, 2048, 4096, 8192])
@pytest.mark.parametrize("out_type", [torch.int8, E4M3])
def test_fht_quant_bit_exact(dev, dim, out_type):
    g = torch.Generator().manual_seed(dim + 1)
    for rows in (1, 33, 130):
        x = (torch.randn(rows, dim, generator=g) * 2).to(BF16)
        x[rows // 2] = 0
        scale = dim ** -0.5
        codes, scales = _C().fht_quant(x.to(dev), scale, out_type)
        wc, ws = O.ref_quant(O.ref_fht(x, scale, BF16), out_type)
        assert_bit_equal(codes, wc, "codes dim=%d rows=%d" % (dim, rows))
        assert_bit_equal(scales, ws, "scales dim=%d rows=%d" % (dim, rows))


@pytest.mark.parametrize("dim", [64, 2048, 8192, 1536])
def test_fht_quant_rows_of_signed_zeros(dev, dim):
    """Rows of zeros of both signs, bf16 and e4m3 inputs: codes (e4m3 keeps the sign of a zero), scales 0. The transform
    carries signs differently from the sequential network and must still hand the quantizer the reference's zeros."""
    g = torch.Generator().manual_seed(dim + 77)
    rows = 21
    xb = (torch.randn(rows, dim, generator=g) * 2).to(BF16)
    neg = torch.tensor(-0.0, dtype=BF16)
    xb[0] = neg
    xb[3] = torch.where(torch.rand(dim, generator=g) < 0.5, neg, torch.tensor(0.0, dtype=BF16))
    xb[7] = 0.0
    xb[rows - 1] = neg
    xb[rows - 1, dim // 3] = 0.0
    x8 = O.e4m3_c10(xb.float())  # e4m3 input with the same zeros (code 0x80 for -0)
    assert (x8.view(torch.uint8)[0] == 0x80).all()
    for x, mids in ((xb, (BF16,)), (x8, (BF16, E4M3))):
        for mid in mids:
            for out_type in (E4M3, None):
                kw = {} if mid == BF16 else {"mid_type": E4M3}
                codes, scales = _C().fht_quant(x.to(dev), dim ** -0.5, out_type, **kw)
                wc, ws = O.ref_quant(O.ref_fht(x, dim ** -0.5, mid), out_type)
                what = "dim=%d in=%s mid=%s out=%s" % (dim, x.dtype, mid, out_type)
                assert_bit_equal(codes, wc, "codes " + what)
                assert_bit_equal(scales, ws, "scales " + what)
    # the transform alone on the e4m3 input
    got = _C().fast_hadamard_transform(x8.to(dev), dim ** -0.5, BF16)
    assert_bit_equal(got, O.ref_fht(x8, dim ** -0.5, BF16), "fht of e4m3 zeros dim=%d" % dim)


def test_fht_quant_fp8_input_and_unrounded_intermediate(dev):
    g = torch.Generator().manual_seed(5)
    x = O.e4m3_c10(torch.randn(3, 7, 256, generator=g) * 4)
    codes, scales = _C().fht_quant(x.to(dev), 1.0 / 16, None)
    wc, ws = O.ref_quant(O.ref_fht(x, 1.0 / 16, BF16), None)
    assert codes.shape == x.shape and scales.shape == x.shape[:-1]
    assert_bit_equal(codes, wc, "codes")
    assert_bit_equal(scales, ws, "scales")
    # without the bf16 rounding of the transform: quantizer applied to the fp32 transform
    xb = (torch.randn(9, 512, generator=g)).to(BF16)
    codes, scales = _C().fht_quant(xb.to(dev), 512 ** -0.5, E4M3, round_intermediate=False)
    y32 = O.ref_fht(xb, 512 ** -0.5, torch.float32) if _accepts_f32() else None
    if y32 is not None:
        wc, ws = O.ref_quant(y32, E4M3)
        assert_bit_equal(codes, wc, "codes (fp32 intermediate)")
        assert_bit_equal(scales, ws, "scales (fp32 intermediate)")


def _accepts_f32():
    try:
        return O.ref_fht(torch.zeros(1, 8, dtype=BF16), 1.0, torch.float32).dtype == torch.float32
    except Exception:
        return False


def test_fht_quant_e4m3_intermediate(dev):
    """e4m3 in, e4m3 intermediate (what the int8 linear does to an fp8 activation): quantize(hadamard_transform(x))."""
    g = torch.Generator().manual_seed(8)
    x = O.e4m3_c10(torch.randn(37, 2048, generator=g) * 3)
    for out_type in (None, E4M3):
        codes, scales = _C().fht_quant(x.to(dev), 2048 ** -0.5, out_type, mid_type=E4M3)
        wc, ws = O.ref_quant(O.ref_fht(x, 2048 ** -0.5, E4M3), out_type)
        assert_bit_equal(codes, wc, "codes")
        assert_bit_equal(scales, ws, "scales")


@pytest.mark.parametrize("shape", [(2, 70, 8, 64), (1, 33, 32, 64), (2, 9, 24, 64), (2, 37, 4, 64)])
@pytest.mark.parametrize("pair", [False, True])
def test_attn_prep_qk_with_qk_rmsnorm(dev, shape, pair):
    """RMSNorm over the whole token row, then RoPE, head split, FHT and the cast: equal to the separate kernels."""
    b, s, h, d = shape
    dim = h * d
    g = torch.Generator().manual_seed(dim + s)
    q, k = ((torch.randn(b, s, dim, generator=g) * 1.5).to(BF16).to(dev) for _ in range(2))
    wq, wk = ((1 + 0.1 * torch.randn(dim, generator=g)).to(dev) for _ in range(2))
    ang = torch.rand(b, s, dim // 2, generator=g) * 6.28
    cos, sin = torch.cos(ang).repeat_interleave(2, -1).to(dev), torch.sin(ang).repeat_interleave(2, -1).to(dev)
    wantq = _C().attn_prep_qk(_C().rms_norm(q, wq, BF16)[0], h, cos, sin, True, 0.125)
    wantk = _C().attn_prep_qk(_C().rms_norm(k, wk, BF16)[0], h, cos, sin, True, 0.125)
    if pair:
        gotq, gotk = _C().attn_prep_qk_pair(q, k, h, cos, sin, True, 0.125, q_norm_weight=wq, k_norm_weight=wk)
    else:
        gotq = _C().attn_prep_qk(q, h, cos, sin, True, 0.125, norm_weight=wq)
        gotk = _C().attn_prep_qk(k, h, cos, sin, True, 0.125, norm_weight=wk)
    assert_bit_equal(gotq, wantq, "q")
    assert_bit_equal(gotk, wantk, "k")
    # and against the oracle's composition (the row sum of squares is accumulated in another order there)
    yo = O.ref_rope(O.ref_rms_norm(q.cpu(), wq.cpu(), BF16)[0], cos.cpu(), sin.cpu(), BF16)
    want = O.ref_fht(_heads(yo, h), 0.125, E4M3)
    assert float((gotq.cpu().view(torch.uint8) != want.view(torch.uint8)).float().mean()) < 0.01


def test_fht_quant_equals_separate_kernels_full_size(dev):
    g = torch.Generator().manual_seed(6)
    x = torch.randn(12288, 2048, generator=g).to(BF16).to(dev)
    codes, scales = _C().fht_quant(x, 2048 ** -0.5, None)
    wc, ws = _C().tokenwise_quant(_C().fast_hadamard_transform(x, 2048 ** -0.5, None), None)
    assert_bit_equal(codes, wc, "codes")
    assert_bit_equal(scales, ws, "scales")


# ------------------------------------------------------------------ RMSNorm -> quantizer

@pytest.mark.parametrize("dim", [64, 1000, 2048, 8192])
@pytest.mark.parametrize("out_type", [torch.int8, E4M3])
def test_rmsnorm_quant(dev, dim, out_type):
    g = torch.Generator().manual_seed(dim + 2)
    for rows, with_w in ((1, True), (37, True), (130, False)):
        x = (torch.randn(rows, dim, generator=g) * 1.7).to(BF16)
        w = (1 + 0.1 * torch.randn(dim, generator=g)) if with_w else None
        codes, scales, rstd = _C().rms_norm_quant(x.to(dev), None if w is None else w.to(dev), out_type)
        # the separate kernels use the same summation order: bit for bit
        y, rstd_sep = _C().rms_norm(x.to(dev), None if w is None else w.to(dev), BF16)
        wc, ws = _C().tokenwise_quant(y, out_type)
        assert_bit_equal(codes, wc, "codes vs separate kernels")
        assert_bit_equal(scales, ws, "scales vs separate kernels")
        assert_bit_equal(rstd, rstd_sep, "rstd vs separate kernels")
        # against the oracle: the row sum of squares is accumulated in another order, so rstd may differ in its
        # last bits and a code may move by one step where x * rstd * w falls on a rounding boundary
        yo, ro = O.ref_rms_norm(x, w, BF16)
        oc, os_ = O.ref_quant(yo, out_type)
        assert torch.allclose(rstd.cpu(), ro, rtol=2e-6, atol=0)
        deq = codes.cpu().float() * scales.cpu()[:, None]
        want = oc.float() * os_[:, None]
        step = os_[:, None] * (1.0 if out_type == torch.int8 else 32.0)
        assert bool(((deq - want).abs() <= step * 1.001).all())
        assert float((codes.cpu().view(torch.uint8) != oc.view(torch.uint8)).float().mean()) < 0.01


# ------------------------------------------------------------------ attention prologues

def _heads(t, h):
    b, s, dim = t.shape
    return t.view(b, s, h, dim // h).transpose(1, 2).contiguous()


@pytest.mark.parametrize("shape", [(2, 70, 8, 64), (1, 33, 32, 64), (2, 19, 8, 128), (1, 5, 64, 64), (2, 37, 4, 64),
                                   (3, 5, 1, 64), (1, 9, 24, 64), (2, 7, 2, 128)])
@pytest.mark.parametrize("rope", [False, True])
@pytest.mark.parametrize("fht", [False, True])
@pytest.mark.parametrize("scaled", [False, True])
def test_attn_prep_qk(dev, shape, rope, fht, scaled):
    b, s, h, d = shape
    dim = h * d
    g = torch.Generator().manual_seed(b * 1000 + s + dim)
    x = (torch.randn(b, s, dim, generator=g) * 1.5).to(BF16)
    x[0, s // 2] = 0
    cos = sin = None
    if rope:
        ang = torch.rand(b, s, dim // 2, generator=g) * 6.28
        cos, sin = torch.cos(ang).repeat_interleave(2, -1), torch.sin(ang).repeat_interleave(2, -1)
    scale = (d ** -0.5) * (0.125 ** 0.5)
    got = _C().attn_prep_qk(x.to(dev), h, None if cos is None else cos.to(dev), None if sin is None else sin.to(dev),
                            fht, scale, scaled)
    y = O.ref_rope(x, cos, sin, BF16) if rope else x
    y = _heads(y, h)
    if scaled:
        y = O.ref_fht(y, scale, BF16) if fht else y
        wc, ws = O.ref_quant(y, E4M3)
        assert_bit_equal(got[0], wc, "codes")
        assert_bit_equal(got[1], ws, "scales")
    else:
        want = O.ref_fht(y, scale, E4M3) if fht else O.e4m3_c10(y)
        assert_bit_equal(got, want, "codes")


def _pair_tables(b, s, dim, g, shared):
    """tables in the layout the LTX transformer builds (every angle twice); shared: one grid for the whole batch"""
    ang = torch.rand(1 if shared else b, s, dim // 2, generator=g) * 6.28
    cos, sin = torch.cos(ang).repeat_interleave(2, -1), torch.sin(ang).repeat_interleave(2, -1)
    return cos.expand(b, -1, -1).contiguous(), sin.expand(b, -1, -1).contiguous()


@pytest.mark.parametrize("shape", [(2, 70, 8, 64), (3, 33, 32, 64), (2, 19, 8, 128), (1, 9, 24, 64), (2, 5, 1, 64), (2, 130, 64, 64)])
@pytest.mark.parametrize("form", ["pairs", "shared", "pairs+shared"])
@pytest.mark.parametrize("scaled", [False, True])
def test_attn_prep_compact_tables_give_the_bits_of_full_tables(dev, shape, form, scaled):
    """The rotation tables with their repeated values stored once ([.., H*D/2]: one entry per rotated pair; [1, S, ..]: one
    position grid for all batch elements) through all four prologues, with the qk-norm in front: bit-equal to the full
    [B, S, H*D] tables, which test_attn_prep_qk checks against the oracle."""
    b, s, h, d = shape
    dim = h * d
    g = torch.Generator().manual_seed(b * 1000 + s + dim)
    q, k, v = ((torch.randn(b, s, dim, generator=g) * 1.5).to(BF16).to(dev) for _ in range(3))
    wq, wk = (1 + 0.1 * torch.randn(dim, generator=g)).to(dev), (1 + 0.1 * torch.randn(dim, generator=g)).to(dev)
    cos, sin = _pair_tables(b, s, dim, g, "shared" in form)
    cc, sc = cos, sin
    if "pairs" in form:
        cc, sc = cc[..., 0::2], sc[..., 0::2]
    if "shared" in form:
        cc, sc = cc[:1], sc[:1]
    full, comp = (cos.to(dev), sin.to(dev)), (cc.contiguous().to(dev), sc.contiguous().to(dev))
    scale = (d ** -0.5) * (0.125 ** 0.5)
    flat = lambda r: [t for part in (r if isinstance(r, (tuple, list)) else (r,)) for t in (part if isinstance(part, (tuple, list)) else (part,))]  # noqa: E731
    calls = [lambda t: _C().attn_prep_qk(q, h, t[0], t[1], True, scale, scaled, norm_weight=wq),
             lambda t: _C().attn_prep_qk_pair(q, k, h, t[0], t[1], True, scale, scaled, q_norm_weight=wq, k_norm_weight=wk),
             lambda t: _C().attn_prep_kv(k, v, h, t[0], t[1], False, 1.0, scaled)]
    if d == 64:
        calls.append(lambda t: _C().attn_prep_qkv(q, k, v, h, t[0], t[1], True, scale, scaled))
    for i, call in enumerate(calls):
        for a, c in zip(flat(call(full)), flat(call(comp))):
            assert_bit_equal(c, a, "%s call %d" % (form, i))


def test_compact_freqs_cis_detects_caches_and_follows_changes(dev):
    """compact_freqs_cis on the tables precompute_freqs_cis builds (both properties), on tables with one property or none,
    the cache (same objects back, dropped by clear_compact_freqs_cache), an in-place change of the tables, and the
    fused attention path with and without it: same bits."""
    from q8_kernels_amd.functional import fused as FU, rope as R
    R.clear_compact_freqs_cache()
    cos, sin = R.precompute_freqs_cis(R.video_index_grid(3, 4, 5, batch=2, device=dev), 512)
    c, s = R.compact_freqs_cis(cos, sin)
    assert c.shape == (1, 60, 256) and s.shape == (1, 60, 256)
    assert torch.equal(c[0].repeat_interleave(2, -1), cos[1]) and torch.equal(s[0].repeat_interleave(2, -1), sin[0])
    c2, s2 = R.compact_freqs_cis(cos, sin)
    assert c2 is c and s2 is s                     # from the cache
    g = torch.Generator().manual_seed(3)
    q, k, v = ((torch.randn(2, 60, 512, generator=g)).to(BF16).to(dev) for _ in range(3))
    on = FU.flash_attn_token_major(q, k, v, 8, None, None, True, (cos, sin), BF16)
    R.compact_tables = False
    try:
        assert R.compact_freqs_cis(cos, sin)[0] is cos
        off = FU.flash_attn_token_major(q, k, v, 8, None, None, True, (cos, sin), BF16)
    finally:
        R.compact_tables = True
    assert_bit_equal(on, off, "fused attention with compact tables")
    # one batch element moved: no longer shared, still one entry per pair; seen through the version counter
    cos[1, 7] = cos[1, 8]
    sin[1, 7] = sin[1, 8]
    c3, s3 = R.compact_freqs_cis(cos, sin)
    assert c3.shape == (2, 60, 256) and torch.equal(c3.repeat_interleave(2, -1), cos)
    assert_bit_equal(FU.flash_attn_token_major(q, k, v, 8, None, None, True, (cos, sin), BF16),
                     FU.flash_attn_token_major(q, k, v, 8, None, None, True, (c3.repeat_interleave(2, -1), s3.repeat_interleave(2, -1)), BF16),
                     "after the change")
    # pairs differ: only the batch property is left; neither: the tables themselves
    cb, sb = torch.randn(1, 60, 512, device=dev).expand(2, -1, -1).contiguous(), torch.randn(1, 60, 512, device=dev).expand(2, -1, -1).contiguous()
    assert R.compact_freqs_cis(cb, sb)[0].shape == (1, 60, 512)
    cn, sn = torch.randn(2, 60, 512, device=dev), torch.randn(2, 60, 512, device=dev)
    assert R.compact_freqs_cis(cn, sn)[0] is cn
    assert len(R._COMPACT_CACHE) == 2              # the last two table pairs
    R.clear_compact_freqs_cache()
    assert R._COMPACT_CACHE == []


@pytest.mark.parametrize("shape", [(2, 70, 8, 64), (1, 33, 32, 64), (2, 7, 2, 128)])
@pytest.mark.parametrize("rope", [False, True])
@pytest.mark.parametrize("scaled", [False, True])
def test_attn_prep_qk_pair_equals_two_single_calls(dev, shape, rope, scaled):
    b, s, h, d = shape
    g = torch.Generator().manual_seed(s * 7 + h)
    qkv = (torch.randn(b, s, 3 * h * d, generator=g) * 1.5).to(BF16).to(dev)
    q, k = qkv[..., :h * d], qkv[..., h * d:2 * h * d]
    cos = sin = None
    if rope:
        ang = torch.rand(b, s, h * d // 2, generator=g) * 6.28
        cos, sin = torch.cos(ang).repeat_interleave(2, -1).to(dev), torch.sin(ang).repeat_interleave(2, -1).to(dev)
    pq, pk = _C().attn_prep_qk_pair(q, k, h, cos, sin, True, 0.125, scaled)
    sq, sk = _C().attn_prep_qk(q, h, cos, sin, True, 0.125, scaled), _C().attn_prep_qk(k, h, cos, sin, True, 0.125, scaled)
    if scaled:
        for got, want in ((pq, sq), (pk, sk)):
            assert_bit_equal(got[0], want[0], "codes")
            assert_bit_equal(got[1], want[1], "scales")
    else:
        assert_bit_equal(pq, sq, "q codes")
        assert_bit_equal(pk, sk, "k codes")


@pytest.mark.parametrize("shape", [(2, 70, 8, 64), (1, 33, 32, 64), (3, 5, 1, 64), (1, 300, 24, 64), (2, 19, 8, 128)])
@pytest.mark.parametrize("scaled", [False, True])
def test_attn_prep_qkv_equals_pair_plus_cast_of_v(dev, shape, scaled):
    """One pass over the three slices of a fused QKV projection: Q and K as attn_prep_qk_pair gives them, V as the
    e4m3 cast (or per (token, head) quantisation) of its heads, token-major [B, H, S, D]."""
    b, s, h, d = shape
    g = torch.Generator().manual_seed(s * 11 + h)
    qkv = (torch.randn(b, s, 3 * h * d, generator=g) * 1.5).to(BF16)
    qkv[0, s // 3] = 0
    qkv_d = qkv.to(dev)
    q, k, v = (qkv_d[..., i * h * d:(i + 1) * h * d] for i in range(3))
    ang = torch.rand(b, s, h * d // 2, generator=g) * 6.28
    cos, sin = torch.cos(ang).repeat_interleave(2, -1).to(dev), torch.sin(ang).repeat_interleave(2, -1).to(dev)
    gq, gk, gv = _C().attn_prep_qkv(q, k, v, h, cos, sin, True, 0.125, scaled)
    wq, wk = _C().attn_prep_qk_pair(q, k, h, cos, sin, True, 0.125, scaled)
    vh = qkv[..., 2 * h * d:].reshape(b, s, h, d).transpose(1, 2).contiguous()
    if scaled:
        wv = O.ref_quant(vh, E4M3)
        for got, want, what in ((gq, wq, "q"), (gk, wk, "k"), (gv, wv, "v")):
            assert_bit_equal(got[0], want[0], what + " codes")
            assert_bit_equal(got[1], want[1], what + " scales")
    else:
        assert_bit_equal(gq, wq, "q codes")
        assert_bit_equal(gk, wk, "k codes")
        assert_bit_equal(gv, O.e4m3_c10(vh), "v codes")


@pytest.mark.parametrize("shape", [(2, 128, 32, 64), (1, 33, 8, 64), (3, 5, 1, 64), (2, 19, 8, 128)])
@pytest.mark.parametrize("scaled", [False, True])
def test_attn_prep_kv_equals_single_call_plus_cast_of_v(dev, shape, scaled):
    """Keys and values of a cross-attention in one launch (strided slices of a fused K/V projection): K as attn_prep_qk
    gives it, V as the e4m3 cast (or per (token, head) quantisation) of its heads, token-major [B, H, S, D]."""
    b, s, h, d = shape
    g = torch.Generator().manual_seed(s * 13 + h)
    kv = (torch.randn(b, s, 2 * h * d, generator=g) * 1.5).to(BF16)
    kv[0, s // 3] = 0
    kv_d = kv.to(dev)
    k, v = kv_d[..., :h * d], kv_d[..., h * d:]
    w = (torch.rand(h * d, generator=g) + 0.5).to(dev)
    gk, gv = _C().attn_prep_kv(k, v, h, None, None, True, 0.125, scaled, norm_weight=w)
    wk = _C().attn_prep_qk(k, h, None, None, True, 0.125, scaled, norm_weight=w)
    vh = kv[..., h * d:].reshape(b, s, h, d).transpose(1, 2).contiguous()
    if scaled:
        wv = O.ref_quant(vh, E4M3)
        for got, want, what in ((gk, wk, "k"), (gv, wv, "v")):
            assert_bit_equal(got[0], want[0], what + " codes")
            assert_bit_equal(got[1], want[1], what + " scales")
    else:
        assert_bit_equal(gk, wk, "k codes")
        assert_bit_equal(gv, O.e4m3_c10(vh), "v codes")


def test_attn_prep_qk_strided_slice_of_fused_projection(dev):
    g = torch.Generator().manual_seed(77)
    qkv = torch.randn(2, 50, 3 * 2048, generator=g).to(BF16)
    qkv_d = qkv.to(dev)
    for i in range(3):
        got = _C().attn_prep_qk(qkv_d[..., i * 2048:(i + 1) * 2048], 32, None, None, True, 0.125, False)
        want = O.ref_fht(_heads(qkv[..., i * 2048:(i + 1) * 2048].contiguous(), 32), 0.125, E4M3)
        assert_bit_equal(got, want, "slice %d" % i)


@pytest.mark.parametrize("shape", [(2, 70, 8), (1, 128, 32), (2, 16, 3), (1, 6144, 2)])
@pytest.mark.parametrize("scaled", [False, True])
def test_attn_prep_v(dev, shape, scaled):
    b, s, h = shape
    g = torch.Generator().manual_seed(s + h)
    x = (torch.randn(b, s, h * 64, generator=g) * 2).to(BF16)
    got = _C().attn_prep_v(x.to(dev), h, scaled)
    s_pad = (s + 15) // 16 * 16
    v = _heads(x, h)  # [b, h, s, 64]
    if scaled:
        wc, ws = O.ref_quant(v, E4M3)
        assert_bit_equal(got[1], ws, "scales")
        got = got[0]
    else:
        wc = O.e4m3_c10(v)
    want = torch.zeros(b, h, 64, s_pad, dtype=torch.uint8)
    want[..., :s] = wc.view(torch.uint8).transpose(2, 3)
    assert got.shape == (b, h, 64, s_pad)
    assert torch.equal(got.cpu().view(torch.uint8), want)


def test_prologues_feed_attention_like_the_functional_path(dev):
    """flash_attn_func on [B,H,S,D] tensors == prologue kernels on the token-major projections + the kernel."""
    import q8_kernels_amd.functional as Q8F
    g = torch.Generator().manual_seed(91)
    b, s, h, d = 2, 200, 8, 64
    q, k, v = ((torch.randn(b, s, h * d, generator=g)).to(BF16).to(dev) for _ in range(3))
    want = Q8F.flash_attention.flash_attn_func(_heads(q, h), _heads(k, h), _heads(v, h), apply_qk_hadamard=True,
                                               out_dtype=BF16)
    sc = (d ** -0.5) * ((d ** -0.5) ** 0.5)
    qc = _C().attn_prep_qk(q, h, None, None, True, sc)
    kc = _C().attn_prep_qk(k, h, None, None, True, sc)
    vc = _C().attn_prep_v(v, h)
    got = _C().flash_attention(qc, kc, vc, 1.0, None, out_dtype=BF16)
    assert_bit_equal(got, want, "attention output")


def test_attention_module_v_cast_in_gemm_equals_both_other_paths(dev):
    """Self-attention of the Attention module at a width the persistent GEMM takes (512): with cast_v_in_gemm the V
    projection's GEMM writes the attention kernel's e4m3 operand itself; the output has the bits of the path where V
    passes through memory as bfloat16 and of the operator-by-operator sequence. The calls into q8_gemm_qkv are counted."""
    import torch.nn as nn
    import q8_kernels_amd._C as C
    from q8_kernels_amd.modules import Attention, Q8Linear
    torch.manual_seed(5)
    attn = Attention(512, 8, 64, bias=True, out_bias=True, qk_rms_norm=True, use_rope=True).to(dev)
    for name in ("to_q", "to_k", "to_v", "to_out"):
        m = getattr(attn, name)
        src = nn.Linear(m.in_features, m.out_features).to(dev).to(BF16)
        q = Q8Linear.from_linear(src)
        m.weight.data, m.scales.data, m.bias.data = q.weight.data, q.scales.data, q.bias.data
    x = torch.randn(2, 300, 512, device=dev).to(BF16)
    ang = torch.rand(2, 300, 256, device=dev) * 6.28
    freqs = (torch.cos(ang).repeat_interleave(2, -1), torch.sin(ang).repeat_interleave(2, -1))
    kw = dict(freqs_cis=freqs, mm_out_dtype=BF16, attn_type="q8_kernels")
    saved, calls = C.mm_bias_qkv, {"qkv": 0}
    def counted(*a, **k):
        calls["qkv"] += 1
        return saved(*a, **k)
    try:
        C.mm_bias_qkv = counted
        with torch.no_grad():
            in_gemm = attn(x, **kw)
            assert calls["qkv"] == 1, "the V projection did not take q8_gemm_qkv"
            Attention.cast_v_in_gemm = False
            through_memory = attn(x, **kw)
            Attention.fuse_prologue = False
            seq = attn(x, **kw)
        assert calls["qkv"] == 1
    finally:
        C.mm_bias_qkv = saved
        Attention.cast_v_in_gemm, Attention.fuse_prologue = True, True
    assert_bit_equal(in_gemm, through_memory, "V cast in the GEMM vs V through memory")
    assert_bit_equal(in_gemm, seq, "V cast in the GEMM vs operator sequence")


def test_attention_module_fused_projections_equal_separate_layers(dev):
    """fuse_projections: q, k, v of a self-attention (one q8_gemm_qkv over the three weights) and k, v of a cross-attention
    (one GEMM over the two) give the bits of one GEMM per layer; the concatenated weights follow a replaced layer weight."""
    import torch.nn as nn
    import q8_kernels_amd.functional.linear as FL
    from q8_kernels_amd.modules import Attention, Q8Linear
    torch.manual_seed(11)

    def fill(attn):
        for name in ("to_q", "to_k", "to_v", "to_out"):
            m = getattr(attn, name)
            q = Q8Linear.from_linear(nn.Linear(m.in_features, m.out_features).to(dev).to(BF16))
            m.weight.data, m.scales.data, m.bias.data = q.weight.data, q.scales.data, q.bias.data
        return attn

    self_attn = fill(Attention(512, 8, 64, bias=True, out_bias=True, qk_rms_norm=True, use_rope=True).to(dev))
    cross = fill(Attention(512, 8, 64, bias=True, out_bias=True, kv_dim=384).to(dev))
    x = torch.randn(2, 300, 512, device=dev).to(BF16)
    text = torch.randn(2, 40, 384, device=dev).to(BF16)
    lens = torch.tensor([40, 13], dtype=torch.int32, device=dev)
    ang = torch.rand(2, 300, 256, device=dev) * 6.28
    freqs = (torch.cos(ang).repeat_interleave(2, -1), torch.sin(ang).repeat_interleave(2, -1))
    kw_self = dict(freqs_cis=freqs, mm_out_dtype=BF16, attn_type="q8_kernels")
    kw_cross = dict(encoder_hidden_states=text, attention_mask=lens, mm_out_dtype=BF16, attn_type="q8_kernels")
    saved, calls = FL.q8_linear, {"n": 0}
    def counted(*a, **k):
        calls["n"] += 1
        return saved(*a, **k)
    try:
        FL.q8_linear = counted
        with torch.no_grad():
            fused_self, n_self = self_attn(x, **kw_self), calls["n"]
            fused_cross, n_cross = cross(x, **kw_cross), calls["n"] - n_self
            # a replaced weight is seen
            q = Q8Linear.from_linear(nn.Linear(384, 512).to(dev).to(BF16))
            cross.to_k.weight.data, cross.to_k.scales.data = q.weight.data, q.scales.data
            fused_cross2 = cross(x, **kw_cross)
            Attention.fuse_projections = False
            calls["n"] = 0
            sep_self, m_self = self_attn(x, **kw_self), calls["n"]
            sep_cross2, m_cross = cross(x, **kw_cross), calls["n"] - m_self
    finally:
        FL.q8_linear = saved
        Attention.fuse_projections = True
    assert (n_self, m_self) == (1, 3), "self-attention: %d / %d calls of q8_linear (the output projection; q, k on top without fusion)" % (n_self, m_self)
    assert (n_cross, m_cross) == (3, 4), "cross-attention: %d / %d calls of q8_linear" % (n_cross, m_cross)
    assert_bit_equal(fused_self, sep_self, "self-attention, fused projections vs separate layers")
    assert_bit_equal(fused_cross2, sep_cross2, "cross-attention after a weight replacement, fused vs separate")
    assert not torch.equal(fused_cross, fused_cross2), "the concatenated weights did not follow the replaced layer"


def test_attention_module_fused_path_equals_operator_sequence(dev):
    import torch.nn as nn
    from q8_kernels_amd.modules import Attention, Q8Linear
    torch.manual_seed(2)
    attn = Attention(256, 8, 64, bias=True, out_bias=True, qk_rms_norm=True, use_rope=True).to(dev)
    for name in ("to_q", "to_k", "to_v", "to_out"):
        m = getattr(attn, name)
        src = nn.Linear(m.in_features, m.out_features).to(dev).to(BF16)
        q = Q8Linear.from_linear(src)
        m.weight.data, m.scales.data, m.bias.data = q.weight.data, q.scales.data, q.bias.data
    x = torch.randn(2, 77, 256, device=dev).to(BF16)
    ang = torch.rand(2, 77, 256, device=dev) * 6.28
    freqs = (torch.cos(ang).repeat_interleave(2, -1), torch.sin(ang).repeat_interleave(2, -1))
    kw = dict(freqs_cis=freqs, mm_out_dtype=BF16, attn_type="q8_kernels")
    # both gated sites are counted, so that the comparison cannot pass by both runs taking the same path
    import q8_kernels_amd.functional.fused as FU
    saved, calls = (FU.hadamard_quantize, FU.flash_attn_token_major), {"rotate": 0, "prologue": 0}
    def rotate(*a, **k):
        calls["rotate"] += 1
        return saved[0](*a, **k)
    def prologue(*a, **k):
        calls["prologue"] += 1
        return saved[1](*a, **k)
    try:
        FU.hadamard_quantize, FU.flash_attn_token_major = rotate, prologue
        fused = attn(x, **kw)
        assert calls == {"rotate": 1, "prologue": 1}, f"fused path not taken: {calls}"
        Attention.fuse_prologue = False
        seq = attn(x, **kw)
        assert calls == {"rotate": 1, "prologue": 1}, f"operator path used a fused kernel: {calls}"
    finally:
        FU.hadamard_quantize, FU.flash_attn_token_major = saved
        Attention.fuse_prologue = True
    assert_bit_equal(fused, seq, "attention module output")
