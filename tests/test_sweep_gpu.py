"""Seeded random sweep of the bit-exact row operators against the oracle: dimensions anywhere in the documented range
(multiples of 8 up to 32768, most of them not powers of two), odd row counts, all-zero rows, amplitudes from 1e-3 to
1e4, both code types and both rounding rules. The fixed lists of the other test files name their cases; this one
covers the combinations between them. A failure message carries everything needed to rebuild the case."""
import random

import pytest
import torch

from oracle import q8_oracle as O
from tests.util import E4M3, assert_bit_equal

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _C():
    from q8_kernels_amd import _C as C
    return C


def _dim(rnd):
    kind = rnd.random()
    if kind < 0.35:
        return rnd.choice([8, 16, 64, 128, 256, 512, 1024, 2048, 4096, 8192, 16384, 32768])
    if kind < 0.8:
        return 8 * rnd.randint(1, 1100)
    return 8 * rnd.randint(1100, 4096)


@pytest.mark.parametrize("sweep_seed", [11, 12, 13])
def test_row_operators_random_shapes(dev, sweep_seed):
    rnd = random.Random(sweep_seed)
    for case in range(40):
        op = rnd.choice(["quant", "quant", "fht", "fht", "fht_quant", "rope", "fma", "rms_quant"])
        dim = _dim(rnd)
        if op in ("rope", "fma") and dim > 8192:
            dim = 8 * rnd.randint(1, 1024)
        rows = rnd.choice([1, 2, 3, 5, 7, 17, 63, 64, 65, 130, 257]) if dim <= 8192 else rnd.choice([1, 2, 3, 5, 9])
        seed = rnd.randint(0, 1 << 30)
        g = torch.Generator().manual_seed(seed)
        amp = rnd.choice([1e-3, 1.0, 30.0, 1e4])
        x = (torch.randn(rows, dim, generator=g) * amp).to(BF16)
        if rnd.random() < 0.15:
            x[rnd.randrange(rows)] = 0
        out_type = rnd.choice([torch.int8, E4M3])
        what = "sweep %d case %d: %s rows=%d dim=%d seed=%d amp=%g out=%s" % (sweep_seed, case, op, rows, dim, seed, amp, out_type)
        if op == "quant":
            rhe = rnd.random() < 0.3
            codes, scales = _C().tokenwise_quant(x.to(dev), out_type, round_half_even=rhe)
            want_codes, want_scales = O.ref_quant(x, out_type, round_half_even=rhe)
            assert_bit_equal(codes, want_codes, what + " rne=%s codes" % rhe)
            assert_bit_equal(scales, want_scales, what + " scales")
        elif op == "fht":
            scale = rnd.choice([1.0, dim ** -0.5, 0.125])
            to = rnd.choice([BF16, E4M3])
            assert_bit_equal(_C().fast_hadamard_transform(x.to(dev), scale, to), O.ref_fht(x, scale, to), what + " scale=%g to=%s" % (scale, to))
        elif op == "fht_quant":
            codes, scales = _C().fht_quant(x.to(dev), dim ** -0.5, out_type, mid_type=BF16)
            want_codes, want_scales = O.ref_quant(O.ref_fht(x, dim ** -0.5, BF16), out_type)
            assert_bit_equal(codes, want_codes, what + " codes")
            assert_bit_equal(scales, want_scales, what + " scales")
        elif op == "rope":
            cos, sin = torch.randn(rows, dim, generator=g), torch.randn(rows, dim, generator=g)
            assert_bit_equal(_C().rope(x.to(dev), cos.to(dev), sin.to(dev), None), O.ref_rope(x, cos, sin, None), what)
        elif op == "fma":
            b = rnd.choice([1, 2]) if rows >= 2 else 1
            t = max(1, rows // b)
            x3 = x[:b * t].reshape(b, t, dim).contiguous()
            tm = rnd.choice([1, t])
            yt, zt = rnd.choice([BF16, torch.float32]), rnd.choice([BF16, torch.float32])
            y = (torch.randn(b, tm, dim, generator=g) * 0.3).to(yt)
            z = torch.randn(b, tm, dim, generator=g).to(zt)
            scale_add = rnd.choice([0.0, 1.0])
            got = _C().fma_8bit(x3.to(dev), y.to(dev), z.to(dev), scale_add)
            assert_bit_equal(got, O.ref_fma(x3, y, z, scale_add), what + " y=%s z=%s mod_rows=%d add=%g" % (yt, zt, tm, scale_add))
        else:  # rms_quant: against the two separate HIP kernels (same summation order), as in test_fused_gpu.py
            w = 1 + 0.1 * torch.randn(dim, generator=g)
            codes, scales, _ = _C().rms_norm_quant(x.to(dev), w.to(dev), out_type)
            want_codes, want_scales = _C().tokenwise_quant(_C().rms_norm(x.to(dev), w.to(dev), BF16)[0], out_type)
            assert_bit_equal(codes, want_codes, what + " codes")
            assert_bit_equal(scales, want_scales, what + " scales")


def _gemm_cfg(c):
    from q8_kernels_amd import _lib
    _lib.check(_lib.lib().q8_gemm_set_config(c))


@pytest.mark.parametrize("sweep_seed", [21, 22])
def test_gemm_random_shapes(dev, sweep_seed):
    """int32 accumulators of random (M, N, K) under every kernel pin: bit-exact. The persistent kernel's bf16 path on
    random shapes it takes (N % 8 == 0, K a multiple of 128 above 256), with batches, both tile heights, GELU and the
    residual epilogue: at most one bf16 ulp from the oracle (int8 operands make the accumulators exact), the residual
    form bit-equal to the separate addition, and the persistent kernel is the one that ran."""
    from q8_kernels_amd import _lib
    rnd = random.Random(sweep_seed)
    for case in range(30):
        seed = rnd.randint(0, 1 << 30)
        g = torch.Generator().manual_seed(seed)
        if rnd.random() < 0.6:
            m, n, k = rnd.randint(1, 700), rnd.randint(1, 700), 16 * rnd.randint(1, 80)
            cfg = rnd.choice([0, 1, 2, 3, 4])  # automatic choice and the four kernel pins
            a = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
            b = torch.randint(-128, 128, (n, k), generator=g, dtype=torch.int8)
            _gemm_cfg(cfg)
            try:
                got = _C().q8_mm_i32(a.to(dev), b.to(dev))
            finally:
                _gemm_cfg(0)
            assert_bit_equal(got, O.ref_gemm_i32(a, b), "sweep %d case %d: acc m=%d n=%d k=%d cfg=%d seed=%d" % (sweep_seed, case, m, n, k, cfg, seed))
            continue
        m, n, k = rnd.randint(1, 3000), 8 * rnd.randint(1, 400), 128 * rnd.randint(3, 10)
        ba, bb = rnd.choice([(1, 1), (1, 1), (2, 1), (1, 2)])
        rows, gelu, with_res = rnd.choice([40, 43, 44]), rnd.random() < 0.5, rnd.random() < 0.3
        a = torch.randint(-128, 128, ((ba, m, k) if ba > 1 else (m, k)), generator=g, dtype=torch.int8).to(dev)
        b = torch.randint(-128, 128, ((bb, n, k) if bb > 1 else (n, k)), generator=g, dtype=torch.int8).to(dev)
        sa = torch.rand(ba * m, generator=g) * 2e-3 + 1e-4
        sb = torch.rand(bb * n, generator=g) * 2e-2 + 1e-3
        bias = torch.randn(n, generator=g)
        what = "sweep %d case %d: persistent m=%d n=%d k=%d batches=%d,%d rows=%d gelu=%s seed=%d" % (sweep_seed, case, m, n, k, ba, bb, rows, gelu, seed)
        _gemm_cfg(4)
        _gemm_cfg(rows)
        try:
            got = _C().q8_mm_bias(a, b, bias.to(dev), sa.to(dev), sb.to(dev), gelu, BF16)
            assert _lib.lib().q8_gemm_last_kernel() in (_lib.Q8_GEMM_KERNEL_PERSIST256, _lib.Q8_GEMM_KERNEL_PERSIST192), what
            if with_res:
                res = torch.randn(got.shape, generator=g).to(BF16).to(dev)
                fused = _C().q8_mm_bias(a, b, bias.to(dev), sa.to(dev), sb.to(dev), gelu, BF16, residual=res)
                assert _lib.lib().q8_gemm_last_kernel() & _lib.Q8_GEMM_KERNEL_RESIDUAL, what
                assert_bit_equal(fused, got + res, what + " residual")
        finally:
            _gemm_cfg(40)
            _gemm_cfg(0)
        want = O.ref_q8_mm(a.cpu(), b.cpu(), bias, sa, sb, gelu, BF16)
        assert got.shape == want.shape, what
        diff = (got.cpu().view(torch.int16).int() - want.view(torch.int16).int()).abs()
        # far in GELU's negative tail the oracle's float64 1 + tanh cancels to zero while the kernel keeps the tiny value
        diff = torch.where((got.cpu().float() - want.float()).abs() <= 1e-7, torch.zeros_like(diff), diff)
        assert int(diff.max()) <= 1, what + ": %d ulp" % int(diff.max())


@pytest.mark.parametrize("sweep_seed", [41, 42])
def test_head_major_epilogue_and_compact_tables_random_shapes(dev, sweep_seed):
    """The GEMM epilogue that transforms and casts heads (q8_gemm_qkv with a Hadamard factor) on random head counts, splits,
    depths, token counts, batches, operand types and tile heights: the plain columns are the plain GEMM's, the codes the
    oracle's hadamard_transform(out_type=e4m3) of its bf16 result. The attention prologues on rotation tables that store
    repeated values once (per pair, per batch, both), random shapes and options: bit-equal to the full tables."""
    from q8_kernels_amd import _lib
    rnd = random.Random(sweep_seed)
    for case in range(20):
        seed = rnd.randint(0, 1 << 30)
        g = torch.Generator().manual_seed(seed)
        heads, v0 = rnd.choice([1, 2, 3, 4, 8, 12, 32]), rnd.choice([0, 0, 256, 512])
        n, k = v0 + 64 * heads, 128 * rnd.randint(3, 12)
        tokens, b = rnd.choice([1, 5, 33, 64, 200, 257, 700]), rnd.choice([1, 1, 2, 3])
        m, i8 = b * tokens, rnd.random() < 0.5
        if i8:
            a = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
            w = torch.randint(-128, 128, (n, k), generator=g, dtype=torch.int8)
            sa, sw = torch.rand(m, generator=g) * 2e-3 + 1e-4, torch.rand(n, generator=g) * 2e-2 + 1e-3
        else:
            a, w = O.e4m3_c10(torch.randn(m, k, generator=g) * 30), O.e4m3_c10(torch.randn(n, k, generator=g) * 30)
            sa, sw = torch.rand(m, generator=g) * 1e-2 + 1e-4, torch.rand(n, generator=g) * 1e-2 + 1e-4
        bias = torch.randn(n, generator=g)
        args = (a.to(dev), w.to(dev), bias.to(dev), sa.to(dev), sw.to(dev))
        scale, rows = rnd.choice([0.0442, 0.125, 1.0]), rnd.choice([40, 43, 44])
        what = "sweep %d case %d seed %d: heads=%d v0=%d k=%d tokens=%d b=%d int8=%s rows=%d scale=%g" % (
            sweep_seed, case, seed, heads, v0, k, tokens, b, i8, rows, scale)
        _gemm_cfg(rows)
        try:
            qk, vc = _C().mm_bias_qkv(*args, tokens, v0, scale)
        finally:
            _gemm_cfg(40)
        want = (_C().q8_mm_bias if i8 else _C().fp8_mm_bias)(*args, False, BF16).reshape(b, tokens, n)
        assert_bit_equal(qk, want[..., :v0].contiguous(), what + " plain columns")
        assert_bit_equal(vc, O.ref_fht(want[..., v0:].cpu().reshape(b, tokens, heads, 64).transpose(1, 2).contiguous(), scale, E4M3), what + " codes")
        # the prologues on compact tables
        d, h = rnd.choice([64, 64, 128]), rnd.choice([1, 2, 4, 8, 16, 32, 64])
        dim = h * d
        if dim not in (64, 128, 256) and (dim % 512 or dim > 4096):
            continue
        s, bb = rnd.choice([1, 3, 17, 64, 130, 301]), rnd.choice([1, 2, 3, 5])
        q, kk, v = ((torch.randn(bb, s, dim, generator=g) * 1.5).to(BF16).to(dev) for _ in range(3))
        shared = rnd.random() < 0.6
        ang = torch.rand(1 if shared else bb, s, dim // 2, generator=g) * 6.28
        cos = torch.cos(ang).repeat_interleave(2, -1).expand(bb, -1, -1).contiguous().to(dev)
        sin = torch.sin(ang).repeat_interleave(2, -1).expand(bb, -1, -1).contiguous().to(dev)
        form = rnd.choice(["pairs", "shared", "both"]) if shared else "pairs"
        tc, ts = (cos, sin) if form == "shared" else (cos[..., 0::2], sin[..., 0::2])
        if form != "pairs":
            tc, ts = tc[:1], ts[:1]
        tc, ts = tc.contiguous(), ts.contiguous()
        scaled, fht = rnd.random() < 0.5, rnd.random() < 0.7
        wq = (1 + 0.1 * torch.randn(dim, generator=g)).to(dev) if rnd.random() < 0.5 else None
        what = "sweep %d case %d seed %d: tables b=%d s=%d h=%d d=%d form=%s scaled=%s fht=%s norm=%s" % (
            sweep_seed, case, seed, bb, s, h, d, form, scaled, fht, wq is not None)
        calls = [lambda c_, s_: _C().attn_prep_qk(q, h, c_, s_, fht, 0.0442, scaled, norm_weight=wq),
                 lambda c_, s_: _C().attn_prep_qk_pair(q, kk, h, c_, s_, fht, 0.0442, scaled, q_norm_weight=wq, k_norm_weight=wq),
                 lambda c_, s_: _C().attn_prep_kv(kk, v, h, c_, s_, fht, 0.0442, scaled, norm_weight=wq)]
        if d == 64:
            calls.append(lambda c_, s_: _C().attn_prep_qkv(q, kk, v, h, c_, s_, fht, 0.0442, scaled, q_norm_weight=wq, k_norm_weight=wq))
        flat = lambda r: [t for part in (r if isinstance(r, (tuple, list)) else (r,)) for t in (part if isinstance(part, (tuple, list)) else (part,))]  # noqa: E731
        for i, call in enumerate(calls):
            for full_t, compact_t in zip(flat(call(cos, sin)), flat(call(tc, ts))):
                assert_bit_equal(compact_t, full_t, what + " call %d" % i)
