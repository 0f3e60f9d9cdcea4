"""GPU parity of the row kernels (quantizer, FHT, RMSNorm, RoPE) against the CPU oracle, through
q8_kernels_amd._C -> libq8_hip.so. Integer / code outputs are compared bit for bit."""
import pytest
import torch

from oracle import q8_oracle as O
from tests.util import E4M3, assert_bit_equal, bf16_ulp, bits

pytestmark = pytest.mark.gpu


def _C():
    from q8_kernels_amd import _C as C
    return C


# ------------------------------------------------------------------ casts (through RoPE with cos = 1, sin = 0)

def test_bf16_to_e4m3_cast_all_patterns(dev):
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    x = torch.stack((pats, torch.zeros_like(pats)), dim=-1).reshape(64, 2048)  # pairs (pattern, 0): y[2i] = pattern
    ones, zeros = torch.ones(64, 2048), torch.zeros(64, 2048)
    got = _C().rope(x.to(dev), ones.to(dev), zeros.to(dev), E4M3).cpu().view(torch.uint8)[:, 0::2]
    want = O.ref_rope(x, ones, zeros, E4M3).view(torch.uint8)[:, 0::2]
    nan = (want & 0x7F) == 0x7F  # the sign of a NaN produced by arithmetic is not defined: compare modulo sign
    assert torch.equal(got[~nan], want[~nan])
    assert bool(((got[nan] & 0x7F) == 0x7F).all())
    assert int(nan.sum()) > 100  # the overflow range |x| > 464 is covered


def test_e4m3_to_bf16_decode_all_codes(dev):
    x = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(E4M3).reshape(4, 64)
    ones, zeros = torch.ones(4, 64), torch.zeros(4, 64)
    got = _C().rope(x.to(dev), ones.to(dev), zeros.to(dev), torch.bfloat16)
    want = O.ref_rope(x, ones, zeros, torch.bfloat16)
    g, w = got.cpu().float(), want.float()
    nan = torch.isnan(w)
    assert torch.equal(torch.isnan(g), nan)
    assert torch.equal(g[~nan], w[~nan])


# ------------------------------------------------------------------ quantizer

@pytest.mark.parametrize("dim", [8, 64, 128, 1000 // 8 * 8, 1536, 2048, 4096, 8192, 10240])
@pytest.mark.parametrize("out_type", [torch.int8, E4M3])
def test_quant_bit_exact(dev, dim, out_type):
    g = torch.Generator().manual_seed(dim)
    for rows in (1, 33, 257):
        x = (torch.randn(rows, dim, generator=g) * 3).to(torch.bfloat16)
        x[rows // 2] = 0  # a zero row
        codes, scales = _C().tokenwise_quant(x.to(dev), out_type)
        wc, ws = O.ref_quant(x, out_type)
        assert_bit_equal(codes, wc, "codes dim=%d rows=%d" % (dim, rows))
        assert_bit_equal(scales, ws, "scales dim=%d rows=%d" % (dim, rows))


@pytest.mark.parametrize("in_dtype", [torch.float32, torch.float16, torch.bfloat16, E4M3])
def test_quant_input_dtypes_flags_and_shapes(dev, in_dtype):
    g = torch.Generator().manual_seed(17)
    x = (torch.randn(2, 5, 256, generator=g) * 2)
    x = O.e4m3_c10(x) if in_dtype == E4M3 else x.to(in_dtype)
    for kw in ({}, {"round_half_even": True}, {"scale_as_division": True}):
        for out_type in (None, E4M3):
            codes, scales = _C().tokenwise_quant(x.to(dev), out_type, **kw)
            wc, ws = O.ref_quant(x, out_type, **kw)
            assert codes.shape == x.shape and scales.shape == x.shape[:-1]
            assert_bit_equal(codes, wc, "codes %s %s" % (in_dtype, kw))
            assert_bit_equal(scales, ws, "scales %s %s" % (in_dtype, kw))


def test_quant_half_ties(dev):
    x = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -2.5, 0.0, 3.0]], dtype=torch.float32)
    away, _ = _C().tokenwise_quant(x.to(dev))
    even, _ = _C().tokenwise_quant(x.to(dev), round_half_even=True)
    assert away.cpu().tolist() == [[127, 1, 2, 3, -1, -3, 0, 3]]
    assert even.cpu().tolist() == [[127, 0, 2, 2, 0, -2, 0, 3]]


def test_quant_strided_rows_and_full_size(dev):
    g = torch.Generator().manual_seed(19)
    big = torch.randn(64, 4096, generator=g).to(torch.bfloat16)
    view = big[:, :2048]  # row stride 4096, unit column stride
    codes, scales = _C().tokenwise_quant(big.to(dev)[:, :2048], E4M3)
    wc, ws = O.ref_quant(view, E4M3)
    assert_bit_equal(codes, wc, "strided codes")
    assert_bit_equal(scales, ws, "strided scales")
    # the block-sized workload: [12288, 2048] tokens
    x = torch.randn(12288, 2048, generator=g).to(torch.bfloat16)
    for out_type in (torch.int8, E4M3):
        codes, scales = _C().tokenwise_quant(x.to(dev), out_type)
        wc, ws = O.ref_quant(x, out_type)
        assert_bit_equal(codes, wc, "full-size codes")
        assert_bit_equal(scales, ws, "full-size scales")


def test_quant_rejects_bad_arguments(dev):
    from q8_kernels_amd import Q8Error
    with pytest.raises(Q8Error):
        _C().tokenwise_quant(torch.zeros(4, 12, dtype=torch.bfloat16, device=dev))
    with pytest.raises(RuntimeError):
        _C().tokenwise_quant(torch.zeros(4, 16, dtype=torch.bfloat16))  # CPU tensor
    with pytest.raises(RuntimeError):
        _C().tokenwise_quant(torch.zeros(4, 16, dtype=torch.bfloat16, device=dev), torch.float16)
    c, s = _C().tokenwise_quant(torch.zeros(0, 16, dtype=torch.bfloat16, device=dev))
    assert c.shape == (0, 16) and s.shape == (0,)


# ------------------------------------------------------------------ FHT

@pytest.mark.parametrize("dim", [8, 16, 32, 64, 128, 256, 512, 1024, 2048, 4096, 8192, 16384, 32768])
def test_fht_bit_exact_pow2(dev, dim):
    g = torch.Generator().manual_seed(dim)
    rows = 5 if dim >= 8192 else 67
    x = torch.randn(rows, dim, generator=g).to(torch.bfloat16)
    for out_type in (torch.bfloat16, E4M3):
        got = _C().fast_hadamard_transform(x.to(dev), dim ** -0.5, out_type)
        assert_bit_equal(got, O.ref_fht(x, dim ** -0.5, out_type), "fht dim=%d -> %s" % (dim, out_type))


@pytest.mark.parametrize("dim", [24, 100, 1536, 10240, 5000])
def test_fht_zero_padding_and_odd_dims(dev, dim):
    g = torch.Generator().manual_seed(dim)
    x = torch.randn(9, dim, generator=g).to(torch.bfloat16)
    got = _C().fast_hadamard_transform(x.to(dev), 0.05, None)
    assert got.dtype == torch.bfloat16 and got.shape == x.shape
    assert_bit_equal(got, O.ref_fht(x, 0.05, None), "fht dim=%d" % dim)


def test_fht_fp8_input_and_head_dim_rows(dev):
    g = torch.Generator().manual_seed(5)
    x8 = O.e4m3_c10(torch.randn(3, 7, 2048, generator=g))
    got = _C().fast_hadamard_transform(x8.to(dev), 2048 ** -0.5, None)
    assert got.dtype == E4M3
    assert_bit_equal(got, O.ref_fht(x8, 2048 ** -0.5, None), "fht e4m3 -> e4m3")
    got = _C().fast_hadamard_transform(x8.to(dev), 2048 ** -0.5, torch.bfloat16)
    assert_bit_equal(got, O.ref_fht(x8, 2048 ** -0.5, torch.bfloat16), "fht e4m3 -> bf16")
    # attention-shaped: [B, H, S, 64] with an outlier channel; overflow must become the NaN code
    q = torch.randn(2, 4, 300, 64, generator=g).to(torch.bfloat16)
    q[..., 5] *= 20
    for scale in (0.125 * 0.125 ** 0.5, 40.0):
        got = _C().fast_hadamard_transform(q.to(dev), scale, E4M3)
        assert_bit_equal(got, O.ref_fht(q, scale, E4M3), "fht D=64 scale=%g" % scale)


@pytest.mark.parametrize("dim", [8, 16, 64, 128, 512, 2048, 4096, 8192, 16384, 32768, 1536])
def test_fht_signed_zeros_and_exact_cancellations(dev, dim):
    """Rows of zeros of both signs keep the signs the sequential network gives them (a sum of -0 and -0 is -0),
    rows with one or two non-zero entries produce exact cancellations (+0), and zero rows sit among non-zero rows
    of the same wave and block."""
    g = torch.Generator().manual_seed(1000 + dim)
    rows = 13 if dim >= 8192 else 70
    x = torch.randn(rows, dim, generator=g).to(torch.bfloat16)
    neg_zero = torch.tensor(-0.0, dtype=torch.bfloat16)
    x[1] = 0.0
    x[2] = neg_zero
    x[3] = torch.where(torch.rand(dim, generator=g) < 0.5, neg_zero, torch.tensor(0.0, dtype=torch.bfloat16))
    x[4] = neg_zero
    x[4, 0] = 0.0
    x[5] = 0.0
    x[5, dim // 2] = 1.5          # one non-zero: every output is +-1.5 * scale
    x[6] = neg_zero
    x[6, 1], x[6, dim - 1] = 2.0, 2.0   # half of the outputs cancel exactly
    x[rows - 1] = torch.where(torch.rand(dim, generator=g) < 0.3, neg_zero, torch.tensor(0.0, dtype=torch.bfloat16))
    for out_type in (torch.bfloat16, E4M3):
        got = _C().fast_hadamard_transform(x.to(dev), dim ** -0.5, out_type)
        want = O.ref_fht(x, dim ** -0.5, out_type)
        assert (bits(want[2]) != bits(want[1])).any(), "the case needs negative zeros among the wanted outputs"
        assert_bit_equal(got, want, "fht signed zeros dim=%d -> %s" % (dim, out_type))


def test_fht_full_size_and_involution(dev):
    g = torch.Generator().manual_seed(6)
    x = torch.randn(12288, 2048, generator=g).to(torch.bfloat16)
    y = _C().fast_hadamard_transform(x.to(dev), 2048 ** -0.5, None)
    assert_bit_equal(y, O.ref_fht(x), "fht [12288, 2048]")
    z = _C().fast_hadamard_transform(y, 2048 ** -0.5, None).cpu()
    assert (z.float() - x.float()).abs().max() < 0.1  # H H = N I, up to two bf16 roundings


# ------------------------------------------------------------------ RMSNorm

@pytest.mark.parametrize("dim", [64, 2048, 8192, 1536])
@pytest.mark.parametrize("affine", [False, True])
def test_rms_norm(dev, dim, affine):
    g = torch.Generator().manual_seed(dim + affine)
    x = (torch.randn(3, 41, dim, generator=g) * 2).to(torch.bfloat16)
    w = (torch.rand(dim, generator=g) + 0.5) if affine else None
    for out_type in (None, E4M3):
        y, rstd = _C().rms_norm(x.to(dev), None if w is None else w.to(dev), out_type)
        wy, wr = O.ref_rms_norm(x, w, out_type)
        assert y.shape == x.shape and rstd.shape == x.shape[:-1]
        # the row sum runs in fp32 in a tree order: rstd within 4 ulp of the float64 value
        assert torch.allclose(rstd.cpu(), wr, rtol=1e-6, atol=0)
        if out_type is None:
            err = (y.cpu().double() - wy.double()).abs()
            assert (err <= bf16_ulp(wy)).all() and (err > 0).float().mean() < 0.01
        else:
            gd, wd = y.cpu().float(), wy.float()
            assert ((gd - wd).abs() <= 0.126 * wd.abs() + 2 ** -9).all()
            assert (y.cpu().view(torch.uint8) != wy.view(torch.uint8)).float().mean() < 0.01


def test_rms_norm_no_epsilon_zero_row(dev):
    x = torch.zeros(2, 64, dtype=torch.bfloat16)
    x[1] = 1
    y, rstd = _C().rms_norm(x.to(dev))
    assert torch.isinf(rstd[0]).item() and torch.isnan(y[0].float()).all()  # 0 * inf, like the reference
    assert rstd[1].item() == 1.0 and (y[1].float() == 1).all()
    y2, r2 = _C().rms_norm(x.to(dev), eps=1e-6)
    assert (y2[0].float() == 0).all()


# ------------------------------------------------------------------ RoPE

@pytest.mark.parametrize("shape", [(2, 33, 2048), (1, 7, 64), (3, 1, 8192), (5, 24)])
def test_rope_bit_exact(dev, shape):
    g = torch.Generator().manual_seed(len(shape) + shape[-1])
    x = torch.randn(*shape, generator=g).to(torch.bfloat16)
    cos, sin = torch.randn(*shape, generator=g), torch.randn(*shape, generator=g)
    for xin in (x, O.e4m3_c10(x.float())):
        for out_type in (None, torch.bfloat16, E4M3):
            got = _C().rope(xin.to(dev), cos.to(dev), sin.to(dev), out_type)
            assert_bit_equal(got, O.ref_rope(xin, cos, sin, out_type), "rope %s -> %s" % (xin.dtype, out_type))


def test_rope_ltx_tables_full_size(dev):
    f, hh, ww = 16, 16, 24
    t = torch.stack(torch.meshgrid(torch.arange(f), torch.arange(hh), torch.arange(ww), indexing="ij")).reshape(3, -1)
    grid = t[None].float().repeat(2, 1, 1)
    cos, sin = O.ref_freqs_cis(grid, 2048)
    assert cos.shape == (2, 6144, 2048)
    g = torch.Generator().manual_seed(9)
    x = torch.randn(2, 6144, 2048, generator=g).to(torch.bfloat16)
    got = _C().rope(x.to(dev), cos.to(dev), sin.to(dev), None)
    assert_bit_equal(got, O.ref_rope(x, cos, sin, None), "rope [2, 6144, 2048]")
    # rotation preserves the norm of every pair (tables have cos[2i] == cos[2i+1])
    n_in = x.float().reshape(2, 6144, 1024, 2).norm(dim=-1)
    n_out = got.cpu().float().reshape(2, 6144, 1024, 2).norm(dim=-1)
    assert torch.allclose(n_in, n_out, rtol=2e-2, atol=1e-2)


def test_rope_rejects_bad_arguments(dev):
    x = torch.zeros(2, 16, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError):
        _C().rope(x, torch.zeros(2, 8, device=dev), torch.zeros(2, 8, device=dev))
    with pytest.raises(RuntimeError):
        _C().rope(x, torch.zeros(2, 16, device=dev, dtype=torch.float64), torch.zeros(2, 16, device=dev))


def test_rows_beyond_2_31_elements(dev):
    """[1 100 000, 2048] bf16: 2.25e9 elements, 4.5 GB; element 2^31 and byte 2^32 fall into row 1 048 576. Quantizer,
    FHT and the fused FHT + quantizer on rows at the start, around that row and at the end, against the oracle."""
    from q8_kernels_amd import _C
    rows, dim = 1_100_000, 2048
    torch.manual_seed(4)
    x = torch.randn(rows, dim, device=dev, dtype=torch.bfloat16)
    assert x.numel() > (1 << 31)
    codes, scales = _C.tokenwise_quant(x, torch.int8)
    y = _C.fast_hadamard_transform(x, dim ** -0.5, torch.bfloat16)
    fcodes, fscales = _C.fht_quant(x, dim ** -0.5, torch.int8, mid_type=torch.bfloat16)
    torch.cuda.synchronize()
    mark = (1 << 31) // dim
    for lo in (0, mark - 32, rows - 64):
        sl = slice(lo, lo + 64)
        xs = x[sl].cpu()
        want_codes, want_scales = O.ref_quant(xs, torch.int8)
        assert_bit_equal(codes[sl], want_codes, "quantizer codes, rows from %d" % lo)
        assert_bit_equal(scales[sl], want_scales, "quantizer scales, rows from %d" % lo)
        want_y = O.ref_fht(xs, dim ** -0.5, torch.bfloat16)
        assert_bit_equal(y[sl], want_y, "FHT, rows from %d" % lo)
        want_fc, want_fs = O.ref_quant(want_y, torch.int8)
        assert_bit_equal(fcodes[sl], want_fc, "FHT + quantizer codes, rows from %d" % lo)
        assert_bit_equal(fscales[sl], want_fs, "FHT + quantizer scales, rows from %d" % lo)
    del x, y, codes, fcodes
    torch.cuda.empty_cache()


def test_zero_rows_everywhere(dev):
    """Tensors without rows pass through every row operator (outputs of the matching empty shapes, no launch)."""
    from q8_kernels_amd import _C
    bf16 = torch.bfloat16
    x = torch.zeros(0, 64, dtype=bf16, device=dev)
    x3 = torch.zeros(2, 0, 64, dtype=bf16, device=dev)
    w = torch.ones(64, device=dev)
    tab = torch.zeros(0, 64, device=dev)
    assert _C.fast_hadamard_transform(x, 1.0, None).shape == (0, 64)
    y, rstd = _C.rms_norm(x, w, None)
    assert y.shape == (0, 64) and rstd.shape == (0,)
    assert _C.rope(x, tab, tab, None).shape == (0, 64)
    codes, scales = _C.fht_quant(x, 0.125, torch.int8)
    assert codes.shape == (0, 64) and scales.shape == (0,)
    codes, scales, rstd = _C.rms_norm_quant(x, w, E4M3)
    assert codes.shape == (0, 64) and scales.shape == (0,) and rstd.shape == (0,)
    mod = torch.zeros(2, 1, 64, dtype=bf16, device=dev)
    codes, scales = _C.norm_mod_fht_quant(x3, True, None, mod, mod, 1.0, 0.125, torch.int8)
    assert codes.shape == (2, 0, 64) and scales.shape == (2, 0)
    assert _C.fma_8bit(x3, mod, mod, 1.0).shape == (2, 0, 64)
    assert _C.gelu_forward(x).shape == (0, 64)
    torch.cuda.synchronize()


def test_quantizer_non_finite_elements(dev):
    """A NaN element is skipped by the row maximum (the reference's fmaxf chain): scale and the other codes as without
    it, itself an e4m3 NaN code (sign not compared; its int8 code is undefined in the reference and not compared).
    An infinite element: infinite scale, zeros, NaN for itself. Kernel against the oracle."""
    from q8_kernels_amd import _C
    g = torch.Generator().manual_seed(22)
    x = (torch.randn(8, 2048, generator=g) * 2).to(torch.bfloat16)
    x[1, 5] = float("nan")
    x[2, 3] = float("inf")
    x[3, 7] = float("-inf")
    x[4, 0] = float("nan")
    x[4, 2047] = float("nan")
    x[5, 100] = float("nan")
    x[5, 200] = float("inf")
    special = ~torch.isfinite(x)
    for out_type in (torch.int8, E4M3):
        codes, scales = _C.tokenwise_quant(x.to(dev), out_type)
        want_codes, want_scales = O.ref_quant(x, out_type)
        assert_bit_equal(scales, want_scales, "scales %s" % out_type)
        got, want = codes.cpu(), want_codes
        if out_type == E4M3:
            got, want = got.view(torch.uint8), want.view(torch.uint8)
            assert torch.equal(got[special] & 0x7F, want[special] & 0x7F), "codes of the non-finite elements"
        assert torch.equal(got[~special], want[~special]), "codes of the finite elements, %s" % out_type
