"""GPU parity of the fp8 flash-attention forward against the float64 oracle.

Tolerance, stated in _check: the element-wise bound that the e4m3 rounding of P implies (2^-4 of the
probability-weighted mean of |V|), cosine >= 0.999 against unrounded attention on the dequantised inputs, and
twice the bound against the oracle that rounds P."""
import pytest
import torch

from oracle import q8_oracle as O
from tests.util import E4M3, cosine

pytestmark = pytest.mark.gpu


def _C():
    from q8_kernels_amd import _C as C
    return C


def _vt(v8):
    """[B,H,N,D] e4m3 -> the kernel's [B,H,D,Nv] layout, Nv = N rounded up to 16, zero padded."""
    n = v8.shape[2]
    nv = (n + 15) // 16 * 16
    vt = torch.zeros(v8.shape[0], v8.shape[1], v8.shape[3], nv, dtype=torch.uint8)
    vt[..., :n] = v8.view(torch.uint8).transpose(2, 3)
    return vt.view(E4M3)


def _inputs(seed, b, h, m, n, std=1.0):
    g = torch.Generator().manual_seed(seed)
    q = O.e4m3_c10(torch.randn(b, h, m, 64, generator=g) * std)
    k = O.e4m3_c10(torch.randn(b, h, n, 64, generator=g) * std)
    v = O.e4m3_c10(torch.randn(b, h, n, 64, generator=g))
    return q, k, v


def _check(got, q, k, v, scale, lens=None, sc=(None, None, None), what="", p_scale=256.0, p_floor=None):
    """Kernel output against float64 attention on the dequantised inputs.
    Rigorous part: P is rounded to e4m3 before it multiplies V: relative error <= 2^-4 per weight in the normal
    range, absolute error <= 2^-10 / p_scale below it, so |o - o_exact| <= 2^-4 W + (2^-10 / p_scale) U with
    W = sum_j p_ij |v_j| / l_i and U = sum_j |v_j| / l_i, plus the bf16 rounding of the output (2^-8 |o|).
    Statistical part: the rounding errors average out, cosine >= 0.999 and the mean error stays below half of
    the mean bound. Against the oracle that rounds P (relative to the final row maximum, the kernel rounds
    relative to the running one) the distance is at most twice the bound. p_floor: the smallest factor the kernel may
    have scaled a probability by when that is not p_scale (lazy_max: 2^5 .. 2^8); it sets the subnormal term."""
    g = got.cpu().double()
    exact, wabs, uabs = O.ref_attention(q, k, v, scale, lens, *sc, round_p=False, return_weighted_abs=True)
    rounded = O.ref_attention(q, k, v, scale, lens, *sc, round_p=True, p_scale=p_scale)
    assert not torch.isnan(g).any(), what
    bound = 2.0 ** -4 * 1.02 * wabs + 2.0 ** -10 / (p_floor or p_scale) * uabs + 2.0 ** -8 * exact.abs() + 1e-6
    e_exact, e_round = (g - exact).abs(), (g - rounded).abs()
    assert (e_exact <= bound).all(), "%s: max-abs vs exact %g exceeds the e4m3 rounding bound (worst ratio %g)" % (
        what, e_exact.max().item(), (e_exact / bound).max().item())
    assert (e_round <= 2 * bound).all(), "%s: max-abs vs rounded-P oracle %g" % (what, e_round.max().item())
    if exact.abs().max() > 0:
        assert e_exact.mean() <= 0.5 * bound.mean(), "%s: mean error %g vs mean bound %g" % (what, e_exact.mean().item(), bound.mean().item())
        assert cosine(g, exact) >= 0.999, "%s: cosine %g" % (what, cosine(g, exact))


@pytest.fixture(params=[0, 1, 2, 4], ids=["default", "4waves_x64q", "4waves_x32q", "8waves_x32q"])
def attn_cfg(request):
    """every workgroup shape q8_attn_set_config offers (the library's default is the first)"""
    from q8_kernels_amd import _lib
    _lib.check(_lib.lib().q8_attn_set_config(request.param))
    yield request.param
    _lib.check(_lib.lib().q8_attn_set_config(0))


@pytest.fixture(params=[False, True], ids=["p_2^8", "p_reference_grid"])
def p_grid(request):
    """The two grids the probabilities are rounded on: the kernel's default e4m3(2^8 p) (the oracle is then told
    p_scale=256) and, with p_unit_range=True, the reference's own e4m3(p), p <= 1
    (csrc/flash_attention/flash_attention_cuda.cu:197-221), checked against the oracle's default p_scale=1.
    Yields (keyword arguments of the call, the oracle's p_scale)."""
    return ({"p_unit_range": True}, 1.0) if request.param else ({}, 256.0)


@pytest.mark.parametrize("m,n", [(256, 64), (64, 128), (1, 1), (33, 17), (255, 100), (257, 200), (300, 640), (512, 1000)])
def test_attention_shapes(dev, attn_cfg, p_grid, m, n):
    kw, p_scale = p_grid
    q, k, v = _inputs(m * 1000 + n, 2, 3, m, n)
    got = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, None, out_dtype=torch.bfloat16, **kw)
    assert got.shape == (2, 3, m, 64) and got.dtype == torch.bfloat16
    _check(got, q, k, v, 0.125, what="m=%d n=%d" % (m, n), p_scale=p_scale)


@pytest.mark.parametrize("m,n", [(130, 300), (200, 100)])
def test_attention_fp8_output_default(dev, p_grid, m, n):
    """e4m3 output (the reference's only output type) of the general and of the short-sequence kernel, on both grids"""
    kw, p_scale = p_grid
    q, k, v = _inputs(5, 1, 2, m, n)
    got = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, None, **kw)
    assert got.dtype == E4M3
    want = O.ref_attention(q, k, v, 0.125, None, out_dtype=E4M3, p_scale=p_scale)
    g, w = got.cpu().float(), want.float()
    assert not torch.isnan(g).any()
    assert ((g - w).abs() <= 0.13 * w.abs() + 0.03).all()


@pytest.mark.parametrize("lens", [[128, 16], [1, 64], [65, 127], [0, 100], [63, 200]])
def test_attention_kv_length_mask(dev, attn_cfg, p_grid, lens):
    kw, p_scale = p_grid
    n = 128
    q, k, v = _inputs(sum(lens), 2, 4, 200, n)
    kv_len = torch.tensor(lens, dtype=torch.int32)
    got = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, kv_len.to(dev), out_dtype=torch.bfloat16, **kw)
    _check(got, q, k, v, 0.125, kv_len.clamp(max=n), what="lens=%s" % lens, p_scale=p_scale)
    # masked keys and values have no influence at all
    k2, v2 = k.clone().view(torch.uint8), v.clone().view(torch.uint8)
    for b, ln in enumerate(lens):
        k2[b, :, min(ln, n):] = 0x55
        v2[b, :, min(ln, n):] = 0x7E
    got2 = _C().flash_attention(q.to(dev), k2.view(E4M3).to(dev), _vt(v2.view(E4M3)).to(dev), 0.125, kv_len.to(dev),
                                out_dtype=torch.bfloat16, **kw)
    assert torch.equal(got.cpu().view(torch.int16), got2.cpu().view(torch.int16))
    for b, ln in enumerate(lens):
        if ln == 0:
            assert (got[b].cpu().float() == 0).all()  # nothing to attend to: zeros


@pytest.mark.parametrize("n", [100, 300])
def test_attention_nan_codes(dev, attn_cfg, n):
    """The e4m3 NaN code (0x7f) behaves as in float attention on the dequantised operands: in a valid key it makes every
    query row of that (batch, head) NaN, in a query it makes that row NaN and no other, and in a key past the valid length
    it has no influence at all (a masked VALUE must be finite: its weight is zero, and 0 * NaN is NaN in any arithmetic).
    (100 keys: the short-sequence kernel, 300: the general one.)"""
    q, k, v = _inputs(5, 2, 2, 150, n)
    kv_len = torch.tensor([n, n - 40], dtype=torch.int32)
    run = lambda q_, k_, v_: _C().flash_attention(q_.to(dev), k_.to(dev), _vt(v_).to(dev), 0.125, kv_len.to(dev),
                                                  out_dtype=torch.bfloat16).cpu()
    base = run(q, k, v)
    assert not torch.isnan(base).any()
    k2 = k.clone().view(torch.uint8)
    k2[0, 1, 17, 3] = 0x7f               # a valid key of (batch 0, head 1)
    k2[1, :, n - 40:, :] = 0x7f          # masked keys of batch 1
    v2 = v.clone().view(torch.uint8)
    v2[1, :, n - 40:, :] = 0x7e          # masked values of batch 1: the largest finite code
    q2 = q.clone().view(torch.uint8)
    q2[1, 0, 77, 40] = 0x7f              # one query row of (batch 1, head 0)
    got = run(q2.view(E4M3), k2.view(E4M3), v2.view(E4M3))
    assert torch.isnan(got[0, 1]).all()
    assert torch.isnan(got[1, 0, 77]).all()
    keep = torch.ones(2, 2, 150, dtype=torch.bool)
    keep[0, 1] = False
    keep[1, 0, 77] = False
    assert torch.equal(got[keep].view(torch.int16), base[keep].view(torch.int16))


def test_attention_large_logits_and_scale(dev):
    q, k, v = _inputs(77, 1, 2, 128, 256, std=4.0)
    for scale in (0.125, 0.02, 1.0):
        got = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), scale, None, out_dtype=torch.bfloat16)
        _check(got, q, k, v, scale, what="scale=%g" % scale)


@pytest.mark.parametrize("m,n,std", [(300, 640, 1.0), (96, 2000, 2.0), (257, 200, 1.0), (64, 4096, 0.5)])
def test_attention_lazy_max(dev, attn_cfg, m, n, std):
    """lazy_max=True: the maximum a row's probabilities are formed against trails the running maximum by at most 3 in log2
    (p between 2^5 and 2^8 times the true softmax numerator): same rounding bound with the subnormal term of 2^5, masked
    and per-token-scaled calls included; every workgroup shape gives the same bits (each row decides for itself)."""
    from q8_kernels_amd import _lib
    q, k, v = _inputs(m + n, 2, 2, m, n, std=std)
    lens = torch.tensor([n, max(1, n // 3)], dtype=torch.int32)
    run = lambda **kw: _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, lens.to(dev), out_dtype=torch.bfloat16, **kw)
    got = run(lazy_max=True)
    _check(got, q, k, v, 0.125, lens, what="lazy maximum m=%d n=%d" % (m, n), p_floor=32.0)
    _lib.check(_lib.lib().q8_attn_set_config(0))
    assert torch.equal(got.cpu().view(torch.int16), run(lazy_max=True).cpu().view(torch.int16))
    with pytest.raises(RuntimeError, match="LAZY_MAX"):
        run(lazy_max=True, p_unit_range=True)
    g = torch.Generator().manual_seed(n)
    sq, sk, sv = (torch.rand(2, 2, r, generator=g) + 0.5 for r in (m, n, n))
    got_s = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, lens.to(dev), out_dtype=torch.bfloat16, lazy_max=True,
                                 q_scales=sq.to(dev), k_scales=sk.to(dev), v_scales=sv.to(dev))
    _check(got_s, q, k, v, 0.125, lens, (sq, sk, sv), what="lazy maximum, per-token scales", p_floor=32.0 * 0.5 / 1.5)


def test_attention_lazy_max_short_sequences_unchanged(dev):
    """N <= 128 runs the short-sequence kernel, which knows the final maximum: lazy_max changes nothing"""
    q, k, v = _inputs(3, 2, 2, 200, 100)
    a = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, None, out_dtype=torch.bfloat16)
    b = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, None, out_dtype=torch.bfloat16, lazy_max=True)
    assert torch.equal(a.cpu().view(torch.int16), b.cpu().view(torch.int16))


@pytest.mark.parametrize("cfg", [0, 2, 4])
@pytest.mark.parametrize("m,n,std", [(300, 640, 1.0), (96, 2000, 2.0), (257, 200, 1.0), (200, 100, 1.0), (33, 17, 1.0)])
def test_attention_sum_rounded_p(dev, cfg, m, n, std):
    """sum_rounded_p=True: the row sum runs over the e4m3-rounded probabilities (on the matrix pipe in the general kernel),
    so every output is a convex combination of the valid v_j: a V with equal rows comes back bit for bit, outputs stay
    inside the per-channel range of V, the distance to exact attention obeys the bound of a 2^-4 perturbation of the
    weights in numerator and denominator, the distance to the oracle with the same definition twice that; all workgroup
    shapes, both V layouts and the combination with lazy_max; refused with per-token scales and the 4 x 64 shape."""
    from q8_kernels_amd import _lib
    q, k, v = _inputs(7 * m + n, 2, 2, m, n, std=std)
    lens = torch.tensor([n, max(1, n // 3)], dtype=torch.int32)
    C = _C()
    _lib.check(_lib.lib().q8_attn_set_config(cfg))
    try:
        run = lambda vv, **kw: C.flash_attention(q.to(dev), k.to(dev), _vt(vv).to(dev), 0.125, lens.to(dev), out_dtype=torch.bfloat16,
                                                 sum_rounded_p=True, **kw)
        row = O.e4m3_c10(torch.randn(64, generator=torch.Generator().manual_seed(n)))
        v_const = row.expand(2, 2, n, 64).contiguous()
        for kw in ({}, {"lazy_max": True}):
            got = run(v_const, **kw)
            assert torch.equal(got.cpu(), row.to(torch.bfloat16).expand(2, 2, m, 64)), "equal rows of V must come back exactly %s" % kw
        got = run(v)
        got_tok = C.flash_attention(q.to(dev), k.to(dev), v.to(dev), 0.125, lens.to(dev), out_dtype=torch.bfloat16, sum_rounded_p=True,
                                    v_token_major=True)
        assert torch.equal(got.cpu().view(torch.int16), got_tok.cpu().view(torch.int16))  # both layouts take the same kernel
        lazy = run(v, lazy_max=True)
    finally:
        _lib.check(_lib.lib().q8_attn_set_config(0))
    # every shape of the general kernel gives the same bits; for N <= 128 the library's default is the short-sequence kernel
    # (another rounding of P), so the general kernel's default shape (config 3) is the baseline there
    _lib.check(_lib.lib().q8_attn_set_config(3 if (n <= 128 and cfg != 0) else 0))
    try:
        base = run(v)
    finally:
        _lib.check(_lib.lib().q8_attn_set_config(0))
    assert torch.equal(got.cpu().view(torch.int16), base.cpu().view(torch.int16)), "config %d against the default shape" % cfg
    g = got.cpu().double()
    exact, wabs, uabs = O.ref_attention(q, k, v, 0.125, lens, round_p=False, return_weighted_abs=True)
    same_def = O.ref_attention(q, k, v, 0.125, lens, p_scale=256.0, sum_rounded=True)
    eps = 2.0 ** -4 * 1.02
    for out, floor in ((g, 256.0), (got_tok.cpu().double(), 256.0), (lazy.cpu().double(), 32.0)):
        sub = 2.0 ** -10 / floor
        bound = (eps * wabs + sub * uabs + (eps + sub * n) * exact.abs()) / (1 - eps) + 2.0 ** -8 * exact.abs() + 1e-6
        assert ((out - exact).abs() <= bound).all(), (out - exact).abs().max().item()
        assert ((out - same_def).abs() <= 2 * bound).all()
        assert cosine(out, exact) >= 0.999
        for b in range(2):
            vb = v[b, :, :int(lens[b])].double()
            lo, hi = vb.amin(dim=1, keepdim=True), vb.amax(dim=1, keepdim=True)
            tol = 2.0 ** -8 * torch.maximum(lo.abs(), hi.abs())   # bf16 rounding of the output
            assert (out[b] >= lo - tol).all() and (out[b] <= hi + tol).all(), "outside the range of V"
    sc = torch.ones(2, 2, max(m, n), device=dev)
    with pytest.raises(RuntimeError, match="unit scales"):
        C.flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, None, out_dtype=torch.bfloat16, sum_rounded_p=True,
                          q_scales=sc[..., :m].contiguous(), k_scales=sc[..., :n].contiguous(), v_scales=sc[..., :n].contiguous())
    if n > 128:
        _lib.check(_lib.lib().q8_attn_set_config(1))
        try:
            with pytest.raises(RuntimeError, match="4 waves x 64"):
                run(v)
        finally:
            _lib.check(_lib.lib().q8_attn_set_config(0))


def test_attention_reference_probability_range(dev):
    """p_unit_range=True rounds the probabilities on the reference's grid (p <= 1): same checks with the larger
    subnormal term, and on a long flat row the default (2^8 p) is the more accurate of the two."""
    q, k, v = _inputs(31, 1, 2, 96, 2000, std=2.0)
    ref_mode = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, None, out_dtype=torch.bfloat16, p_unit_range=True)
    _check(ref_mode, q, k, v, 0.125, what="p <= 1", p_scale=1.0)
    dflt = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, None, out_dtype=torch.bfloat16)
    _check(dflt, q, k, v, 0.125, what="2^8 p")
    exact = O.ref_attention(q, k, v, 0.125, None, round_p=False)
    assert (dflt.cpu().double() - exact).abs().mean() < (ref_mode.cpu().double() - exact).abs().mean()


def test_attention_per_token_scales(dev, attn_cfg, p_grid):
    kw, p_scale = p_grid
    g = torch.Generator().manual_seed(9)
    b, h, m, n = 2, 2, 150, 333
    qf = torch.randn(b, h, m, 64, generator=g) * (torch.rand(b, h, m, 1, generator=g) * 4 + 0.2)
    kf = torch.randn(b, h, n, 64, generator=g) * (torch.rand(b, h, n, 1, generator=g) * 4 + 0.2)
    vf = torch.randn(b, h, n, 64, generator=g) * (torch.rand(b, h, n, 1, generator=g) * 2 + 0.5)
    (q, sq), (k, sk), (v, sv) = (O.ref_quant(t.to(torch.bfloat16), E4M3) for t in (qf, kf, vf))
    lens = torch.tensor([333, 77], dtype=torch.int32)
    got = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, lens.to(dev), out_dtype=torch.bfloat16,
                               q_scales=sq.to(dev), k_scales=sk.to(dev), v_scales=sv.to(dev), **kw)
    _check(got, q, k, v, 0.125, lens, (sq, sk, sv), what="per-token scales", p_scale=p_scale)
    full = torch.nn.functional.scaled_dot_product_attention(
        qf.double(), kf.double(), vf.double(),
        attn_mask=torch.zeros(b, 1, 1, n, dtype=torch.float64).masked_fill(
            ~(torch.arange(n)[None, :] < lens[:, None])[:, None, None, :], float("-inf")))
    assert cosine(got.cpu(), full) > 0.99


def test_attention_config3_self_attention_hadamard(dev, p_grid):
    """B=2, H=32, S=6144, D=64, non-causal; Q/K/V bf16 ~ N(0,1) with one head-dim channel scaled x20; Q and K
    rotated by the normalised 64-point Hadamard transform, everything quantised per token to e4m3, softmax
    scale 1/8, bf16 output. The whole problem runs on the GPU; the oracle checks four (batch, head) pairs."""
    kw, p_scale = p_grid
    C = _C()
    g = torch.Generator().manual_seed(3)
    B, H, S = 2, 32, 6144
    q, k, v = (torch.randn(B, H, S, 64, generator=g).to(torch.bfloat16) for _ in range(3))
    for t in (q, k, v):
        t[..., int(torch.randperm(64, generator=g)[0])] *= 20
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    qr, kr = C.fast_hadamard_transform(qd, 0.125, torch.bfloat16), C.fast_hadamard_transform(kd, 0.125, torch.bfloat16)
    (q8, sq), (k8, sk), (v8, sv) = C.tokenwise_quant(qr, E4M3), C.tokenwise_quant(kr, E4M3), C.tokenwise_quant(vd, E4M3)
    vt = v8.view(torch.uint8).transpose(2, 3).contiguous().view(E4M3)
    out = C.flash_attention(q8, k8, vt, 0.125, None, out_dtype=torch.bfloat16, q_scales=sq, k_scales=sk, v_scales=sv, **kw)
    assert out.shape == (B, H, S, 64)
    for (b, h) in [(0, 0), (0, 17), (1, 5), (1, 31)]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        oq, osq = O.ref_quant(O.ref_fht(q[sl], 0.125, torch.bfloat16), E4M3)
        ok, osk = O.ref_quant(O.ref_fht(k[sl], 0.125, torch.bfloat16), E4M3)
        ov, osv = O.ref_quant(v[sl], E4M3)
        assert torch.equal(q8[sl].cpu().view(torch.uint8), oq.view(torch.uint8))
        assert torch.equal(sk[sl].cpu(), osk)
        _check(out[sl], oq, ok, ov, 0.125, None, (osq, osk, osv), what="config 3 (b=%d,h=%d)" % (b, h), p_scale=p_scale)
        # against attention on the unquantised bf16 inputs: with a x20 outlier channel in q and k the logits have a
        # standard deviation near 50 and single keys dominate, so e4m3 rounding of q and k can change the winner;
        # this measures the quantisation scheme, not the kernel
        plain = torch.nn.functional.scaled_dot_product_attention(q[sl].double(), k[sl].double(), v[sl].double())
        assert cosine(out[sl].cpu(), plain) >= 0.9
    # size-independent property at full size: every output row is a convex combination of V rows
    vmax = (v8.float() * sv[..., None]).amax(dim=2, keepdim=True)
    vmin = (v8.float() * sv[..., None]).amin(dim=2, keepdim=True)
    o = out.float()
    slack = 0.02 * (vmax - vmin) + 0.02
    assert bool(((o <= vmax + slack) & (o >= vmin - slack)).all())


def test_attention_config4_cross_attention_mask(dev, p_grid):
    """B=2, H=32, 6144 queries, 128 text keys, valid lengths drawn from 16..128, reference-style direct casts with
    the Hadamard rotation (softmax scale folded into Q and K)."""
    kw, p_scale = p_grid
    g = torch.Generator().manual_seed(4)
    B, H, M, N = 2, 32, 6144, 128
    q = torch.randn(B, H, M, 64, generator=g).to(torch.bfloat16)
    k = torch.randn(B, H, N, 64, generator=g).to(torch.bfloat16)
    v = torch.randn(B, H, N, 64, generator=g).to(torch.bfloat16)
    lens = torch.randint(16, 129, (B,), generator=g, dtype=torch.int32)
    from q8_kernels_amd.functional.flash_attention import flash_attn_func
    out = flash_attn_func(q.to(dev), k.to(dev), v.to(dev), None, lens.to(dev), True, out_dtype=torch.bfloat16, **kw)
    assert out.shape == (B, H, M, 64)
    s = (1 / 64) ** 0.5 * (0.125 ** 0.5)
    q8, k8, v8 = O.ref_fht(q, s, E4M3), O.ref_fht(k, s, E4M3), O.e4m3_c10(v)
    hs = slice(0, 32, 11)
    _check(out[:, hs], q8[:, hs], k8[:, hs], v8[:, hs], 1.0, lens, what="config 4", p_scale=p_scale)
    mask = torch.zeros(B, 1, 1, N, dtype=torch.float64).masked_fill(~(torch.arange(N)[None, :] < lens[:, None])[:, None, None, :], float("-inf"))
    plain = torch.nn.functional.scaled_dot_product_attention(q[:, hs].double(), k[:, hs].double(), v[:, hs].double(), attn_mask=mask)
    assert cosine(out[:, hs].cpu(), plain) >= 0.998  # accuracy of the direct e4m3 casts, not of the kernel


def test_attention_config4_cross_attention_mask_per_token_scales(dev, p_grid):
    """Config 4 with per-token e4m3 quantisation of Q, K (after the Hadamard rotation) and V: 6144 queries, 128 text keys,
    valid lengths drawn from 16..128. The whole problem runs on the GPU; the oracle checks four (batch, head) pairs, and
    masked keys and values have no influence at all."""
    kw, p_scale = p_grid
    C = _C()
    g = torch.Generator().manual_seed(44)
    B, H, M, N = 2, 32, 6144, 128
    q = torch.randn(B, H, M, 64, generator=g).to(torch.bfloat16)
    k, v = (torch.randn(B, H, N, 64, generator=g).to(torch.bfloat16) for _ in range(2))
    lens = torch.randint(16, 129, (B,), generator=g, dtype=torch.int32)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    qr, kr = C.fast_hadamard_transform(qd, 0.125, torch.bfloat16), C.fast_hadamard_transform(kd, 0.125, torch.bfloat16)
    (q8, sq), (k8, sk), (v8, sv) = C.tokenwise_quant(qr, E4M3), C.tokenwise_quant(kr, E4M3), C.tokenwise_quant(vd, E4M3)
    vt = v8.view(torch.uint8).transpose(2, 3).contiguous().view(E4M3)
    out = C.flash_attention(q8, k8, vt, 0.125, lens.to(dev), out_dtype=torch.bfloat16, q_scales=sq, k_scales=sk, v_scales=sv, **kw)
    assert out.shape == (B, H, M, 64)
    for (b, h) in [(0, 0), (0, 21), (1, 7), (1, 31)]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        oq, osq = O.ref_quant(O.ref_fht(q[sl], 0.125, torch.bfloat16), E4M3)
        ok, osk = O.ref_quant(O.ref_fht(k[sl], 0.125, torch.bfloat16), E4M3)
        ov, osv = O.ref_quant(v[sl], E4M3)
        _check(out[sl], oq, ok, ov, 0.125, lens[b:b + 1], (osq, osk, osv), what="config 4 per token (b=%d,h=%d)" % (b, h), p_scale=p_scale)
    k2, v2, sk2, sv2 = k8.clone().view(torch.uint8), v8.clone().view(torch.uint8), sk.clone(), sv.clone()
    for b in range(B):
        ln = int(lens[b])
        k2[b, :, ln:], v2[b, :, ln:], sk2[b, :, ln:], sv2[b, :, ln:] = 0x55, 0x7E, 1e3, 1e3
    vt2 = v2.transpose(2, 3).contiguous().view(E4M3)
    out2 = C.flash_attention(q8, k2.view(E4M3), vt2, 0.125, lens.to(dev), out_dtype=torch.bfloat16, q_scales=sq, k_scales=sk2,
                             v_scales=sv2, **kw)
    # (the common factor max_j sv_j runs over the valid keys only, so the masked scales must not show either)
    assert torch.equal(out.cpu().view(torch.int16), out2.cpu().view(torch.int16))


def test_attention_rejects_bad_arguments(dev):
    from q8_kernels_amd import Q8Error
    q, k, v = _inputs(1, 1, 1, 16, 16)
    vt = _vt(v)
    with pytest.raises(RuntimeError):
        _C().flash_attention(q.to(dev), k.to(dev), vt.to(dev), 0.125, torch.tensor([16], device=dev))  # int64 mask
    with pytest.raises(RuntimeError):
        _C().flash_attention(q.to(dev).float(), k.to(dev), vt.to(dev), 0.125, None)
    q32 = O.e4m3_c10(torch.zeros(1, 1, 16, 32))
    with pytest.raises(Q8Error):
        _C().flash_attention(q32.to(dev), q32.to(dev), O.e4m3_c10(torch.zeros(1, 1, 32, 16)).to(dev), 0.125, None)


@pytest.mark.parametrize("sweep_seed", [31, 32])
def test_attention_random_shapes(dev, sweep_seed):
    """Seeded sweep between the fixed cases above: random query and key counts (ragged against the 32-query and
    64-key tiles), batch and head counts, key-length masks including 0 and the full length, direct casts or per-token
    scales, logit spreads, every workgroup shape; the same bounds as everywhere in this file."""
    import random
    from q8_kernels_amd import _lib
    rnd = random.Random(sweep_seed)
    for case in range(14):
        b, h = rnd.choice([(1, 1), (1, 3), (2, 2), (3, 1)])
        m, n = rnd.randint(1, 420), rnd.randint(1, 900)
        cfg = rnd.choice([0, 1, 2, 4])
        scaled, masked = rnd.random() < 0.4, rnd.random() < 0.6
        std = rnd.choice([0.5, 1.0, 2.0])
        seed = rnd.randint(0, 1 << 30)
        what = "sweep %d case %d: b=%d h=%d m=%d n=%d cfg=%d scaled=%s masked=%s std=%g seed=%d" % (
            sweep_seed, case, b, h, m, n, cfg, scaled, masked, std, seed)
        g = torch.Generator().manual_seed(seed)
        lens = None
        if masked:
            lens = torch.tensor([rnd.choice([0, 1, n, rnd.randint(1, n)]) for _ in range(b)], dtype=torch.int32)
        if scaled:
            qf = torch.randn(b, h, m, 64, generator=g) * (torch.rand(b, h, m, 1, generator=g) * 4 + 0.2) * std
            kf = torch.randn(b, h, n, 64, generator=g) * (torch.rand(b, h, n, 1, generator=g) * 4 + 0.2)
            vf = torch.randn(b, h, n, 64, generator=g) * (torch.rand(b, h, n, 1, generator=g) * 2 + 0.5)
            (q, sq), (k, sk), (v, sv) = (O.ref_quant(t.to(torch.bfloat16), E4M3) for t in (qf, kf, vf))
            sc = (sq, sk, sv)
        else:
            q, k, v = _inputs(seed, b, h, m, n, std)
            sc = (None, None, None)
        _lib.check(_lib.lib().q8_attn_set_config(cfg))
        try:
            got = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, None if lens is None else lens.to(dev),
                                       out_dtype=torch.bfloat16,
                                       **({"q_scales": sq.to(dev), "k_scales": sk.to(dev), "v_scales": sv.to(dev)} if scaled else {}))
        finally:
            _lib.check(_lib.lib().q8_attn_set_config(0))
        assert got.shape == (b, h, m, 64), what
        _check(got, q, k, v, 0.125, lens, sc, what=what)


def test_workgroup_shapes_give_identical_bits(dev):
    """A query row meets the same 64-key tiles in the same order whatever the workgroup shape, so the shapes
    of q8_attn_set_config have to agree bit for bit (direct casts with a mask, and per-token scales)."""
    from q8_kernels_amd import _lib
    g = torch.Generator().manual_seed(77)
    b, h, m, n = 2, 3, 333, 517
    q, k, v = _inputs(77, b, h, m, n)
    lens = torch.tensor([517, 130], dtype=torch.int32)
    qf = torch.randn(b, h, m, 64, generator=g) * (torch.rand(b, h, m, 1, generator=g) * 4 + 0.2)
    kf = torch.randn(b, h, n, 64, generator=g) * (torch.rand(b, h, n, 1, generator=g) * 4 + 0.2)
    vf = torch.randn(b, h, n, 64, generator=g) * (torch.rand(b, h, n, 1, generator=g) * 2 + 0.5)
    (q2, sq), (k2, sk), (v2, sv) = (O.ref_quant(t.to(torch.bfloat16), E4M3) for t in (qf, kf, vf))
    outs = {}
    try:
        for cfg in (0, 1, 2, 4):
            _lib.check(_lib.lib().q8_attn_set_config(cfg))
            plain = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, lens.to(dev), out_dtype=torch.bfloat16)
            scaled = _C().flash_attention(q2.to(dev), k2.to(dev), _vt(v2).to(dev), 0.125, lens.to(dev), out_dtype=torch.bfloat16,
                                          q_scales=sq.to(dev), k_scales=sk.to(dev), v_scales=sv.to(dev))
            outs[cfg] = (plain.cpu().view(torch.int16), scaled.cpu().view(torch.int16))
    finally:
        _lib.check(_lib.lib().q8_attn_set_config(0))
    for cfg in (1, 2, 4):
        assert torch.equal(outs[cfg][0], outs[0][0]), "direct casts, shape %d" % cfg
        assert torch.equal(outs[cfg][1], outs[0][1]), "per-token scales, shape %d" % cfg


def test_zero_query_row_with_scales_and_masked_keys(dev, attn_cfg):
    """An all-zero query row is quantized to scale 0. With a partial or masked tile its masked keys are -inf, and
    -inf times that zero scale must not turn the row into NaN: zero logits weigh the valid keys uniformly, as the
    oracle does."""
    g = torch.Generator().manual_seed(15)
    b, h, m, n = 2, 2, 70, 100
    qf = torch.randn(b, h, m, 64, generator=g)
    qf[0, 0, 3] = 0
    qf[1, 1, 64:] = 0
    kf, vf = torch.randn(b, h, n, 64, generator=g), torch.randn(b, h, n, 64, generator=g)
    (q, sq), (k, sk), (v, sv) = (O.ref_quant(t.to(torch.bfloat16), E4M3) for t in (qf, kf, vf))
    assert sq[0, 0, 3] == 0 and (sq[1, 1, 64:] == 0).all()
    lens = torch.tensor([100, 37], dtype=torch.int32)
    got = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, lens.to(dev), out_dtype=torch.bfloat16,
                               q_scales=sq.to(dev), k_scales=sk.to(dev), v_scales=sv.to(dev))
    assert not torch.isnan(got).any()
    _check(got, q, k, v, 0.125, lens, (sq, sk, sv), what="zero query rows")
    mean_v = (v[1, 1, :37].double() * sv[1, 1, :37, None].double()).mean(dim=0)
    assert (got[1, 1, 64:].cpu().double() - mean_v).abs().max() <= 0.07 * mean_v.abs().max() + 0.02


@pytest.mark.parametrize("n,lens", [(128, [128, 16]), (100, [37, 100]), (64, [64, 1]), (17, [0, 17]), (1, [1, 1])])
@pytest.mark.parametrize("scaled", [False, True])
def test_short_kv_path(dev, n, lens, scaled):
    """N <= 128 takes the kernel that keeps K and V of a (batch, head) in LDS and rounds P against the final maximum
    (single-pass softmax), with unit scales and with per-token scales. Same bars as the general kernel, which is forced
    for comparison (config 3): both against the oracle, and the two must differ somewhere when there are two key blocks
    (they round P against different maxima), which shows that the two calls took different kernels."""
    from q8_kernels_amd import _lib
    b, h, m = 2, 3, 1000
    if scaled:
        g = torch.Generator().manual_seed(9000 + n)
        qf = torch.randn(b, h, m, 64, generator=g) * (torch.rand(b, h, m, 1, generator=g) * 4 + 0.2)
        kf = torch.randn(b, h, n, 64, generator=g) * (torch.rand(b, h, n, 1, generator=g) * 4 + 0.2)
        vf = torch.randn(b, h, n, 64, generator=g) * (torch.rand(b, h, n, 1, generator=g) * 2 + 0.5)
        (q, sq), (k, sk), (v, sv) = (O.ref_quant(t.to(torch.bfloat16), E4M3) for t in (qf, kf, vf))
        kw = dict(q_scales=sq.to(dev), k_scales=sk.to(dev), v_scales=sv.to(dev))
        sc = (sq, sk, sv)
    else:
        q, k, v = _inputs(7000 + n, b, h, m, n)
        kw, sc = {}, (None, None, None)
    l = torch.tensor(lens, dtype=torch.int32)
    args = (q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, l.to(dev))
    short = _C().flash_attention(*args, out_dtype=torch.bfloat16, **kw)
    try:
        _lib.check(_lib.lib().q8_attn_set_config(3))
        general = _C().flash_attention(*args, out_dtype=torch.bfloat16, **kw)
    finally:
        _lib.check(_lib.lib().q8_attn_set_config(0))
    _check(short, q, k, v, 0.125, l, sc, what="short KV N=%d" % n)
    _check(general, q, k, v, 0.125, l, sc, what="general N=%d" % n)
    assert not torch.equal(short, general) or n <= 64, "both calls took the same kernel"
    # token-major output, token-major V, e4m3 output and the reference's P grid through the same path
    tok = _C().flash_attention(*args, out_dtype=torch.bfloat16, token_major_out=True, **kw)
    assert torch.equal(tok.view(b, m, h, 64).transpose(1, 2), short), "token-major output differs"
    vtok = _C().flash_attention(q.to(dev), k.to(dev), v.to(dev), 0.125, l.to(dev), out_dtype=torch.bfloat16, v_token_major=True, **kw)
    assert torch.equal(vtok, short), "token-major V differs"
    o8 = _C().flash_attention(*args, **kw)
    assert o8.dtype == E4M3 and ((o8.cpu().float() - short.cpu().float()).abs() <= 0.07 * short.cpu().float().abs() + 0.02).all()
    unit = _C().flash_attention(*args, out_dtype=torch.bfloat16, p_unit_range=True, **kw)
    _check(unit, q, k, v, 0.125, l, sc, what="short KV, p <= 1", p_scale=1.0)


@pytest.mark.parametrize("b,h,m,n,lens", [(5, 2, 200, 100, [100, 0, 64, 7, 65]), (3, 40, 2500, 128, [128, 1, 90]),
                                          (1, 1, 31, 128, [128]), (4, 1, 70, 65, None)])
def test_short_kv_batches_and_tile_walk(dev, b, h, m, n, lens):
    """The short-sequence kernel over more than two batches (the LDS halves alternate, a batch without valid keys lies
    between batches with one and two key blocks), several tiles per wave with a ragged last tile, and more workgroups
    than fit the device at once: against the oracle for every batch, and a batch's output must not depend on what the
    other batches hold (each batch alone gives the same bits)."""
    q, k, v = _inputs(8100 + b * 7 + m, b, h, m, n)
    l = None if lens is None else torch.tensor(lens, dtype=torch.int32)
    ld = None if l is None else l.to(dev)
    got = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, ld, out_dtype=torch.bfloat16)
    _check(got[:, :2], q[:, :2], k[:, :2], v[:, :2], 0.125, l, what="short KV b=%d h=%d m=%d n=%d" % (b, h, m, n))
    if lens is not None and 0 in lens:
        assert (got[lens.index(0)] == 0).all(), "a batch without valid keys gives zeros"
    for i in range(b):
        alone = _C().flash_attention(q[i:i + 1].to(dev), k[i:i + 1].to(dev), _vt(v[i:i + 1]).to(dev), 0.125,
                                     None if ld is None else ld[i:i + 1].contiguous(), out_dtype=torch.bfloat16)
        assert torch.equal(alone[0], got[i]), "batch %d depends on its neighbours" % i


@pytest.mark.parametrize("m,n,lens", [(256, 64, None), (33, 17, None), (300, 640, None), (512, 1000, [1000, 333]),
                                      (130, 128, [128, 5]), (70, 200, [0, 200]), (1, 1, None), (257, 6144, None)])
@pytest.mark.parametrize("scaled", [False, True])
def test_token_major_v_gives_the_bits_of_the_transposed_layout(dev, m, n, lens, scaled):
    """V passed as [B,H,N,64] (turned by the kernel while it reads its LDS tile) against the same V passed
    pre-transposed: the two paths feed identical operands to identical arithmetic, so every output bit agrees;
    the transposed layout is checked against the oracle once more here."""
    from q8_kernels_amd import _lib
    b, h = 2, 3
    g = torch.Generator().manual_seed(m * 31 + n)
    if scaled:
        qf = torch.randn(b, h, m, 64, generator=g) * (torch.rand(b, h, m, 1, generator=g) * 4 + 0.2)
        kf = torch.randn(b, h, n, 64, generator=g) * (torch.rand(b, h, n, 1, generator=g) * 4 + 0.2)
        vf = torch.randn(b, h, n, 64, generator=g) * (torch.rand(b, h, n, 1, generator=g) * 2 + 0.5)
        (q, sq), (k, sk), (v, sv) = (O.ref_quant(t.to(torch.bfloat16), E4M3) for t in (qf, kf, vf))
        kw = dict(q_scales=sq.to(dev), k_scales=sk.to(dev), v_scales=sv.to(dev))
        sc = (sq, sk, sv)
    else:
        q, k, v = _inputs(m * 1000 + n, b, h, m, n)
        kw, sc = {}, (None, None, None)
    lens_t = None if lens is None else torch.tensor(lens, dtype=torch.int32)
    lens_d = None if lens is None else lens_t.to(dev)
    for out_dtype in (torch.bfloat16, E4M3):
        # the default shape of the mode, both shapes that read token-major V and the general kernel where a short
        # sequence would take the LDS-resident one: each against the transposed layout under the same configuration
        for cfg in (0, 2, 3, 4):
            _lib.check(_lib.lib().q8_attn_set_config(cfg))
            try:
                want = _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev), 0.125, lens_d, out_dtype=out_dtype, **kw)
                got = _C().flash_attention(q.to(dev), k.to(dev), v.to(dev), 0.125, lens_d, out_dtype=out_dtype,
                                           v_token_major=True, **kw)
            finally:
                _lib.check(_lib.lib().q8_attn_set_config(0))
            assert torch.equal(got.view(torch.uint8 if out_dtype == E4M3 else torch.int16).cpu(),
                               want.view(torch.uint8 if out_dtype == E4M3 else torch.int16).cpu()), (m, n, lens, scaled, out_dtype, cfg)
    if n <= 1000:
        got = _C().flash_attention(q.to(dev), k.to(dev), v.to(dev), 0.125, lens_d, out_dtype=torch.bfloat16,
                                   v_token_major=True, **kw)
        _check(got, q, k, v, 0.125, lens_t, sc, what="token-major V m=%d n=%d" % (m, n))


def test_token_major_v_rejects_what_it_cannot_do(dev):
    from q8_kernels_amd import Q8Error, _lib
    q, k, v = _inputs(3, 1, 1, 64, 64)
    with pytest.raises(RuntimeError):  # a token-major V has K's shape
        _C().flash_attention(q.to(dev), k.to(dev), _vt(v).to(dev)[..., :48], 0.125, None, v_token_major=True)
    _lib.check(_lib.lib().q8_attn_set_config(1))
    try:
        with pytest.raises(Q8Error):
            _C().flash_attention(q.to(dev), k.to(dev), v.to(dev), 0.125, None, v_token_major=True)
    finally:
        _lib.check(_lib.lib().q8_attn_set_config(0))
