"""GPU parity of the 8-bit GEMM: int32 accumulators bit-exact, dequantised outputs within a stated
tolerance of the float64 oracle."""
import pytest
import torch

from oracle import q8_oracle as O
from tests.util import E4M3, assert_bit_equal, bf16_ulp, cosine

pytestmark = pytest.mark.gpu


def _C():
    from q8_kernels_amd import _C as C
    return C


def _set_cfg(c):
    from q8_kernels_amd import _lib
    _lib.check(_lib.lib().q8_gemm_set_config(c))


from q8_kernels_amd._lib import (Q8_GEMM_KERNEL_PERSIST192 as K_PERSIST192, Q8_GEMM_KERNEL_PERSIST256 as K_PERSIST256,  # noqa: E402
                                 Q8_GEMM_KERNEL_PIPE256 as K_PIPE256, Q8_GEMM_KERNEL_RESIDUAL as K_RESIDUAL,
                                 Q8_GEMM_KERNEL_TILE128 as K_TILE128, Q8_GEMM_KERNEL_TILE64 as K_TILE64)


PERSISTENT_KERNELS = {K_PERSIST256, K_PERSIST192}  # the workgroup-per-CU kernels that walk over several tiles


def _last_kernel():
    from q8_kernels_amd import _lib
    return _lib.lib().q8_gemm_last_kernel()


def _kernels_for(cfg, n, k, bf16_out=True):
    """The kernels a call may launch under q8_gemm_set_config(cfg): the pins 1, 2 and 3 always hold; 4 means the
    persistent kernel for the shapes it takes (bf16 or e4m3 output, N % 8 == 0, K a multiple of 128 above 256) and the
    per-tile pipelined kernel otherwise. Asserted after the calls below so that a test of a pinned kernel cannot
    pass on a silent fall-back to another one."""
    if cfg == 1:
        return {K_PIPE256}
    if cfg == 2:
        return {K_TILE128}
    if cfg == 3:
        return {K_TILE64}
    eligible = bf16_out and n % 8 == 0 and k > 256 and k % 128 == 0
    return {K_PERSIST256, K_PERSIST192} if eligible else {K_PIPE256}


@pytest.fixture(params=[1, 2, 3, 4], ids=["tile256", "tile128", "tile64", "persistent256"])
def tile_cfg(request):
    _set_cfg(request.param)
    yield request.param
    _set_cfg(0)


def _rand_i8(g, *shape):
    return torch.randint(-128, 128, shape, generator=g, dtype=torch.int8)


def _check_float_out(got, want64, what):
    """bf16 outputs: the kernel accumulates in fp32 (MFMA order) and uses the hardware exp2 / rcp for the
    GELU, the oracle float64: allow 2 bf16 ulp plus 2^-9 of the row scale, and demand cosine >= 0.99999."""
    g = got.cpu().double()
    tol = 2 * bf16_ulp(want64) + 2.0 ** -9 * want64.abs().mean()
    err = (g - want64).abs()
    assert (err <= tol).all(), "%s: max err %g (tol %g at worst)" % (what, err.max().item(), tol[err.argmax()].item() if tol.dim() else tol)
    assert cosine(g, want64) >= 0.99999, what


# ------------------------------------------------------------------ int8: exact accumulators

@pytest.mark.parametrize("mnk", [(256, 256, 128), (16, 8, 16), (1, 1, 32), (300, 200, 144), (257, 129, 2048), (513, 384, 400)])
def test_int8_accumulators_bit_exact(dev, tile_cfg, mnk):
    m, n, k = mnk
    g = torch.Generator().manual_seed(m * 7 + n * 3 + k)
    a, b = _rand_i8(g, m, k), _rand_i8(g, n, k)
    got = _C().q8_mm_i32(a.to(dev), b.to(dev))
    assert _last_kernel() in _kernels_for(tile_cfg, n, k, bf16_out=False)
    assert_bit_equal(got, O.ref_gemm_i32(a, b), "int32 acc %s" % (mnk,))


def test_int8_config2_bit_exact_and_dequant(dev):
    """A int8 [6144, 2048], B int8 [2048, 2048] from per-row absmax quantisation (round to nearest even) of
    N(0,1) and N(0,0.02) bf16 tensors; int32 accumulators must match exactly, then dequantise with bias."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(6144, 2048, generator=g).to(torch.bfloat16)
    w = (torch.randn(2048, 2048, generator=g) * 0.02).to(torch.bfloat16)
    bias = (torch.randn(2048, generator=g) * 0.02).to(torch.bfloat16).float()
    a, sa = O.ref_quant(x, torch.int8, round_half_even=True)
    b, sb = O.ref_quant(w, torch.int8, round_half_even=True)
    # the quantizer kernel yields the same codes
    ga, gsa = _C().tokenwise_quant(x.to(dev), torch.int8, round_half_even=True)
    assert_bit_equal(ga, a, "config-2 A codes")
    assert_bit_equal(gsa, sa, "config-2 A scales")
    acc = _C().q8_mm_i32(a.to(dev), b.to(dev))
    want_acc = O.ref_gemm_i32(a, b)
    assert_bit_equal(acc, want_acc, "config-2 int32 accumulators")
    out = _C().q8_mm_bias(a.to(dev), b.to(dev), bias.to(dev), sa.to(dev), sb.to(dev), False, torch.bfloat16)
    assert out.shape == (1, 6144, 2048) and out.dtype == torch.bfloat16
    want = O.ref_epilogue(want_acc[None], sa[None], sb[None], bias, False, torch.bfloat16)
    # same exact accumulators, one fma and one rounding: at most the last bf16 bit may differ
    diff = (out.cpu().view(torch.int16).int() - want.view(torch.int16).int()).abs()
    assert diff.max() <= 1 and (diff > 0).float().mean() < 1e-3
    # and it approximates the bf16 linear it stands for
    ref = x.double() @ w.double().T + bias.double()
    assert cosine(out.cpu(), ref) > 0.999



@pytest.mark.parametrize("pin,kernel", [(44, K_PERSIST256), (43, K_PERSIST192)], ids=["256rows", "192rows"])
@pytest.mark.parametrize("mnk", [(2304, 8192, 2048), (1600, 10248, 640)])
def test_int8_persistent_kernel_accumulators_bit_exact(dev, pin, kernel, mnk):
    """The persistent kernel (the one that serves config 2 and the block's int8 linears) has no int32 output; its
    accumulators are observed through the bf16 store instead: with sparse operands in {-1, 0, 1} every |acc| stays far
    below 256, where bf16 holds integers exactly, and with unit scales and no bias the stored value IS the accumulator
    (csrc/gemm/q8_matmul_bias.cu:315-320: float(acc) * (sa * sb)). More tiles than CUs, both tile heights, one shape
    with ragged edges in M and N; the oracle's integer matmul is evaluated in float32, exact for these magnitudes."""
    m, n, k = mnk
    g = torch.Generator().manual_seed(m + n + k)

    def sparse(rows):
        u = torch.rand(rows, k, generator=g)
        return ((u < 0.05).to(torch.int8) - (u > 0.95).to(torch.int8))

    a, b = sparse(m), sparse(n)
    # a few denser rows of either operand so that the accumulators are not all tiny (still far below 256)
    a[::97] = ((torch.rand(a[::97].shape, generator=g) < 0.2).to(torch.int8))
    b[::89] = ((torch.rand(b[::89].shape, generator=g) < 0.2).to(torch.int8))
    want = a.float() @ b.float().T + 0.0  # (+ 0.0: a sum of negative zeros becomes the +0 of an integer zero)
    assert want.abs().max() <= 256 and want.abs().max() >= 15
    assert torch.equal(want[:64, :64].long(), O.ref_gemm_i32(a[:64], b[:64]).long())  # the float32 evaluation is the oracle's integers
    ones_m, ones_n = torch.ones(m, device=dev), torch.ones(n, device=dev)
    _set_cfg(4)
    _set_cfg(pin)
    try:
        out = _C().q8_mm(a.to(dev), b.to(dev), ones_m, ones_n, False, torch.bfloat16)
        assert _last_kernel() == kernel
    finally:
        _set_cfg(40)
        _set_cfg(0)
    assert_bit_equal(out[0], want.to(torch.bfloat16), "persistent int8 accumulators %s" % (mnk,))

# ------------------------------------------------------------------ epilogue variants

@pytest.mark.parametrize("in_dtype", ["i8", "fp8"])
@pytest.mark.parametrize("fuse_gelu", [False, True])
@pytest.mark.parametrize("with_bias", [False, True])
def test_mm_epilogue_vs_oracle(dev, tile_cfg, in_dtype, fuse_gelu, with_bias):
    g = torch.Generator().manual_seed(100 + fuse_gelu * 2 + with_bias)
    m, n, k = 200, 264, 384
    if in_dtype == "i8":
        a, b = _rand_i8(g, m, k), _rand_i8(g, n, k)
        sa, sb = torch.rand(m, generator=g) * 2e-3 + 1e-4, torch.rand(n, generator=g) * 2e-2 + 1e-3
        mm, mmb, ref = _C().q8_mm, _C().q8_mm_bias, O.ref_q8_mm
    else:
        a, b = O.e4m3_c10(torch.randn(m, k, generator=g) * 50), O.e4m3_c10(torch.randn(n, k, generator=g) * 50)
        sa, sb = torch.rand(m, generator=g) * 1e-2 + 1e-4, torch.rand(n, generator=g) * 1e-2 + 1e-4
        mm, mmb, ref = _C().fp8_mm, _C().fp8_mm_bias, O.ref_fp8_mm
    bias = torch.randn(n, generator=g) if with_bias else None
    args = (a.to(dev), b.to(dev)) + ((bias.to(dev),) if with_bias else ()) + (sa.to(dev), sb.to(dev), fuse_gelu)
    fn = mmb if with_bias else mm
    got = fn(*args, torch.bfloat16)
    assert _last_kernel() in _kernels_for(tile_cfg, n, k), "kernel %d under config %d" % (_last_kernel(), tile_cfg)
    assert got.shape == (1, m, n)
    acc = O.ref_gemm_i32(a, b).double() if in_dtype == "i8" else O.ref_gemm_fp8_acc(a, b)
    v = acc * (sa[:, None] * sb[None, :]).double() + (bias.double() if with_bias else 0)
    want64 = torch.nn.functional.gelu(v, approximate="tanh") if fuse_gelu else v
    _check_float_out(got[0], want64, "%s gelu=%s bias=%s" % (in_dtype, fuse_gelu, with_bias))
    # e4m3 output (the reference's default out_type): saturating cast of the same value
    got8 = fn(*args, None)
    assert _last_kernel() in _kernels_for(tile_cfg, n, k), "e4m3 output: kernel %d under config %d" % (_last_kernel(), tile_cfg)
    assert got8.dtype == E4M3
    want8 = ref(a, b, bias, sa, sb, fuse_gelu, None)[0]
    g8, w8 = got8[0].cpu().float(), want8.float()
    assert not torch.isnan(g8).any()
    assert ((g8 - w8).abs() <= 0.126 * w8.abs() + 2 ** -9).all()
    assert (got8[0].cpu().view(torch.uint8) != want8.view(torch.uint8)).float().mean() < 0.02


def test_mm_e4m3_output_saturates(dev):
    a = torch.full((16, 32), 127, dtype=torch.int8)
    b = torch.full((16, 32), 127, dtype=torch.int8)
    b[8:] = -127
    ones = torch.ones(16)
    out = _C().q8_mm(a.to(dev), b.to(dev), ones.to(dev), ones.to(dev), False, None)
    codes = out.cpu().view(torch.uint8)[0]
    assert (codes[:, :8] == 0x7E).all() and (codes[:, 8:] == 0xFE).all()


def test_mm_batch_broadcast(dev, tile_cfg):
    g = torch.Generator().manual_seed(7)
    m, n, k = 70, 48, 64
    a3, b3 = _rand_i8(g, 3, m, k), _rand_i8(g, 3, n, k)
    sa3, sb3 = torch.rand(3, m, generator=g) * 1e-2, torch.rand(3, n, generator=g) * 1e-2
    bias = torch.randn(n, generator=g)
    cases = [(a3, b3[0], sa3, sb3[0]), (a3[0], b3, sa3[0], sb3), (a3, b3, sa3, sb3), (a3[1], b3[2], sa3[1], sb3[2])]
    for a, b, sa, sb in cases:
        got = _C().q8_mm_bias(a.to(dev), b.to(dev), bias.to(dev), sa.contiguous().to(dev), sb.contiguous().to(dev), False, torch.bfloat16)
        assert _last_kernel() in _kernels_for(tile_cfg, n, k)
        want = O.ref_q8_mm(a, b, bias, sa, sb, False, torch.bfloat16)
        assert got.shape == want.shape
        diff = (got.cpu().view(torch.int16).int() - want.view(torch.int16).int()).abs()
        assert diff.max() <= 1, "batch case a%s b%s" % (tuple(a.shape), tuple(b.shape))


@pytest.mark.parametrize("case", [(1, 1, 4352, 4096, 384), (3, 1, 1100, 4600, 512), (1, 2, 2300, 2816, 640)])
@pytest.mark.parametrize("fuse_gelu", [False, True])
@pytest.mark.parametrize("tile_rows", [43, 44], ids=["rows192", "rows256"])
def test_persistent_kernel_many_tiles_fp8(dev, case, fuse_gelu, tile_rows):
    """The same walk over many tiles, ragged edges and batches with e4m3 operands (fp32 accumulation in MFMA order
    against the oracle's float64: the tolerance of the other fp8 checks)."""
    ba, bb, m, n, k = case
    g = torch.Generator().manual_seed(m + n + 5)
    a = O.e4m3_c10(torch.randn(*((ba, m, k) if ba > 1 else (m, k)), generator=g) * 50)
    b = O.e4m3_c10(torch.randn(*((bb, n, k) if bb > 1 else (n, k)), generator=g) * 50)
    sa = torch.rand(ba * m, generator=g) * 1e-2 + 1e-4
    sb = torch.rand(bb * n, generator=g) * 1e-2 + 1e-4
    bias = torch.randn(n, generator=g)
    _set_cfg(4)
    _set_cfg(tile_rows)
    try:
        got = _C().fp8_mm_bias(a.to(dev), b.to(dev), bias.to(dev), sa.to(dev), sb.to(dev), fuse_gelu, torch.bfloat16)
        assert _last_kernel() == (K_PERSIST192 if tile_rows == 43 else K_PERSIST256)
    finally:
        _set_cfg(40)
        _set_cfg(0)
    want = O.ref_fp8_mm(a, b, bias, sa, sb, fuse_gelu, torch.float64)
    assert got.shape == want.shape
    _check_float_out(got, want, "fp8 persistent %s" % (case,))


@pytest.mark.parametrize("case", [(1, 1, 4352, 4096, 384), (3, 1, 1100, 4600, 512), (1, 2, 2300, 2816, 640)])
@pytest.mark.parametrize("fuse_gelu", [False, True])
@pytest.mark.parametrize("tile_rows", [43, 44], ids=["rows192", "rows256"])
def test_persistent_kernel_many_tiles_per_workgroup(dev, case, fuse_gelu, tile_rows):
    """More 256x256 tiles than CUs (272, 270 and 198+ with ragged edges and batch broadcast), so that workgroups of the
    persistent kernel cross tile and batch boundaries; int8 operands make the accumulators exact, the epilogue
    is fp32 on both sides: at most one bf16 ulp."""
    ba, bb, m, n, k = case
    g = torch.Generator().manual_seed(m + n)
    a = _rand_i8(g, ba, m, k) if ba > 1 else _rand_i8(g, m, k)
    b = _rand_i8(g, bb, n, k) if bb > 1 else _rand_i8(g, n, k)
    sa = torch.rand(ba * m, generator=g) * 2e-3 + 1e-4
    sb = torch.rand(bb * n, generator=g) * 2e-2 + 1e-3
    bias = torch.randn(n, generator=g)
    _set_cfg(4)
    _set_cfg(tile_rows)  # force the 192- or the 256-row tile of the persistent kernel
    try:
        got = _C().q8_mm_bias(a.to(dev), b.to(dev), bias.to(dev), sa.to(dev), sb.to(dev), fuse_gelu, torch.bfloat16)
        assert _last_kernel() == (K_PERSIST192 if tile_rows == 43 else K_PERSIST256)
    finally:
        _set_cfg(40)
        _set_cfg(0)
    want = O.ref_q8_mm(a, b, bias, sa, sb, fuse_gelu, torch.bfloat16)
    assert got.shape == want.shape
    diff = (got.cpu().view(torch.int16).int() - want.view(torch.int16).int()).abs()
    # far in GELU's negative tail the float64 formula 1 + tanh cancels to zero while the kernel keeps the tiny value
    diff = torch.where((got.cpu().float() - want.float()).abs() <= 1e-7, torch.zeros_like(diff), diff)
    assert int(diff.max()) <= 1, "max %d ulp at %s" % (int(diff.max()), (diff == diff.max()).nonzero()[0].tolist())
    assert float((diff > 0).float().mean()) < (0.02 if fuse_gelu else 0.002)


@pytest.mark.parametrize("case", [(1, 1, 2300, 2816, 640), (2, 1, 1100, 4608, 384), (1, 1, 200, 264, 208)])
@pytest.mark.parametrize("fuse_gelu", [False, True])
@pytest.mark.parametrize("tile_rows", [40, 43, 44], ids=["rows_auto", "rows192", "rows256"])
def test_residual_in_epilogue_equals_separate_addition(dev, case, fuse_gelu, tile_rows):
    """out = residual + linear(a): the fused epilogue (first two cases, persistent kernel) and the fallback (last case,
    K not a multiple of 128) both give the bits of the bf16 GEMM followed by a bf16 addition."""
    ba, bb, m, n, k = case
    g = torch.Generator().manual_seed(m + n + 1)
    a = (_rand_i8(g, ba, m, k) if ba > 1 else _rand_i8(g, m, k)).to(dev)
    b = _rand_i8(g, n, k).to(dev)
    sa = (torch.rand(ba * m, generator=g) * 2e-3 + 1e-4).to(dev)
    sb = (torch.rand(n, generator=g) * 2e-2 + 1e-3).to(dev)
    bias = torch.randn(n, generator=g).to(dev)
    res = torch.randn(ba, m, n, generator=g).to(torch.bfloat16).to(dev)
    _set_cfg(4)
    _set_cfg(tile_rows)
    try:
        plain = _C().q8_mm_bias(a, b, bias, sa, sb, fuse_gelu, torch.bfloat16)
        assert _last_kernel() in _kernels_for(4, n, k)
        fused = _C().q8_mm_bias(a, b, bias, sa, sb, fuse_gelu, torch.bfloat16, residual=res)
        if k % 128 == 0:  # added in the persistent kernel's epilogue
            want_kernels = {40: {K_PERSIST256, K_PERSIST192}, 43: {K_PERSIST192}, 44: {K_PERSIST256}}[tile_rows]
            assert _last_kernel() in {kk | K_RESIDUAL for kk in want_kernels}
        else:             # the GEMM without residual, then a separate addition
            assert _last_kernel() == K_PIPE256
    finally:
        _set_cfg(40)
        _set_cfg(0)
    assert_bit_equal(fused, plain + res, "residual epilogue")


@pytest.mark.parametrize("case", [(2, 1536, 768, 384), (3, 768, 2304, 640), (1, 2304, 520, 512), (2, 100, 264, 384)])
@pytest.mark.parametrize("in_dtype", ["int8", "fp8"])
@pytest.mark.parametrize("fuse_gelu", [False, True])
@pytest.mark.parametrize("tile_rows", [43, 44], ids=["rows192", "rows256"])
def test_gated_residual_in_epilogue_equals_the_fused_multiply_add(dev, case, in_dtype, fuse_gelu, tile_rows):
    """out = linear(a) * gate + residual with one gate row per batch element (the AdaLN block's gated residual): the
    epilogue form (tokens per batch element a multiple of 768: a tile never meets two gate rows) and the fallback (last
    case) both give the bits of the bf16 GEMM followed by the fused multiply-add kernel. 3-D activations [B, T, K]."""
    bsz, t, n, k = case
    g = torch.Generator().manual_seed(bsz * 7 + t + n)
    if in_dtype == "int8":
        a, b = _rand_i8(g, bsz, t, k).to(dev), _rand_i8(g, n, k).to(dev)
        sa = (torch.rand(bsz * t, generator=g) * 2e-3 + 1e-4).to(dev)
        mm = _C().q8_mm_bias
    else:
        a, b = O.e4m3_c10(torch.randn(bsz, t, k, generator=g)).to(dev), O.e4m3_c10(torch.randn(n, k, generator=g)).to(dev)
        sa = (torch.rand(bsz * t, generator=g) * 2e-1 + 1e-2).to(dev)
        mm = _C().fp8_mm_bias
    sb = (torch.rand(n, generator=g) * 2e-2 + 1e-3).to(dev)
    bias = torch.randn(n, generator=g).to(dev)
    res = torch.randn(bsz, t, n, generator=g).to(torch.bfloat16).to(dev)
    gate = (torch.randn(bsz, 1, n, generator=g) * 0.7).to(torch.bfloat16).to(dev)
    gate[0, 0, :8] = 0  # a closed gate passes the residual through
    _set_cfg(4)
    _set_cfg(tile_rows)
    try:
        plain = mm(a, b, bias, sa, sb, fuse_gelu, torch.bfloat16)
        fused = mm(a, b, bias, sa, sb, fuse_gelu, torch.bfloat16, residual=res, gate=gate)
        if t % 768 == 0:
            assert _last_kernel() == ({43: K_PERSIST192, 44: K_PERSIST256}[tile_rows] | K_RESIDUAL)
    finally:
        _set_cfg(40)
        _set_cfg(0)
    want = _C().fma_8bit(plain, gate, res)
    assert_bit_equal(fused, want, "gated residual epilogue")
    assert torch.equal(fused[0, :, :8], res[0, :, :8])


# ------------------------------------------------------------------ fp8 at the benchmark shapes

@pytest.mark.parametrize("m", [2048, 6144])
def test_fp8_linear_bias_gelu_config1(dev, m):
    """X bf16 [m, 2048] ~ N(0,1); W bf16 [8192, 2048] ~ N(0,0.02); bias ~ N(0,0.02); per-row e4m3 quantisation;
    out = GELU(acc * sx * sw + bias) in bf16. Tolerance: 2 bf16 ulp + 2^-9 mean|out| against float64, cosine
    >= 0.99999; and cosine >= 0.999 against the unquantised bf16 linear."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(m, 2048, generator=g).to(torch.bfloat16)
    w = (torch.randn(8192, 2048, generator=g) * 0.02).to(torch.bfloat16)
    bias = (torch.randn(8192, generator=g) * 0.02).to(torch.bfloat16).float()
    xq, sx = _C().tokenwise_quant(x.to(dev), E4M3)
    wq, sw = _C().tokenwise_quant(w.to(dev), E4M3)
    oxq, osx = O.ref_quant(x, E4M3)
    owq, osw = O.ref_quant(w, E4M3)
    assert_bit_equal(xq, oxq, "X codes")
    assert_bit_equal(sx, osx, "X scales")
    assert_bit_equal(wq, owq, "W codes")
    assert_bit_equal(sw, osw, "W scales")
    out = _C().fp8_mm_bias(xq, wq, bias.to(dev), sx, sw, True, torch.bfloat16)
    assert out.shape == (1, m, 8192)
    acc = O.ref_gemm_fp8_acc(oxq, owq)
    v = acc * (osx[:, None] * osw[None, :]).double() + bias.double()
    want64 = torch.nn.functional.gelu(v, approximate="tanh")
    _check_float_out(out[0], want64, "config-1 m=%d" % m)
    full = torch.nn.functional.gelu(x.double() @ w.double().T + bias.double(), approximate="tanh")
    assert cosine(out[0].cpu(), full) > 0.999


def test_mm_rejects_bad_arguments(dev):
    from q8_kernels_amd import Q8Error
    a = torch.zeros(16, 24, dtype=torch.int8, device=dev)
    s = torch.ones(16, device=dev)
    with pytest.raises(Q8Error):  # K % 16 != 0
        _C().q8_mm(a, a, s, s, False, torch.bfloat16)
    a = torch.zeros(16, 32, dtype=torch.int8, device=dev)
    with pytest.raises(RuntimeError):  # fp16 output is not supported (the reference returns garbage)
        _C().q8_mm(a, a, s, s, False, torch.float16)
    with pytest.raises(RuntimeError):
        _C().q8_mm(a, a.t(), s, s, False, torch.bfloat16)  # not contiguous
    with pytest.raises(RuntimeError):
        _C().fp8_mm(a, a, s, s, False, torch.bfloat16)  # wrong operand dtype
    with pytest.raises(RuntimeError):
        _C().q8_mm(torch.zeros(2, 16, 32, dtype=torch.int8, device=dev), torch.zeros(3, 16, 32, dtype=torch.int8, device=dev),
                   torch.ones(32, device=dev), torch.ones(48, device=dev), False, torch.bfloat16)


# ------------------------------------------------------------------ operand sizes around 4 GiB

@pytest.mark.parametrize("rows_over", [-64, 64], ids=["just_below_4GiB_persistent", "above_4GiB_per_tile"])
def test_operand_around_4_gib(dev, rows_over):
    """A [M, 2048] int8 with M * K = 4 GiB -/+ 128 KiB. Below the limit the persistent kernel takes it and its 32-bit
    byte offsets run up to just under 2^32 (far beyond 2^31: they have to be treated as unsigned); above it the
    dispatcher has to fall back to the per-tile kernel with its 64-bit addresses. Rows at the start, around the 2 GiB
    mark and at the end are checked against the oracle (int8 operands, exact accumulators: at most one bf16 ulp)."""
    k, n = 2048, 256
    m = (1 << 32) // k + rows_over
    torch.manual_seed(3)
    a = torch.randint(-128, 128, (m, k), dtype=torch.int8, device=dev)
    b = torch.randint(-128, 128, (n, k), dtype=torch.int8, device=dev)
    sa = torch.rand(m, device=dev) * 2e-3 + 1e-4
    sb = torch.rand(n, device=dev) * 2e-2 + 1e-3
    bias = torch.randn(n, device=dev)
    assert a.numel() == m * k and (a.numel() < (1 << 32)) == (rows_over < 0)
    out = _C().q8_mm_bias(a, b, bias, sa, sb, False, torch.bfloat16)
    kernel = _last_kernel()
    torch.cuda.synchronize()
    if rows_over < 0:
        assert kernel in (K_PERSIST256, K_PERSIST192), kernel
    else:
        assert kernel == K_PIPE256, kernel
    assert out.shape == (1, m, n)
    half = (1 << 31) // k
    for lo in (0, half - 150, m - 300):
        rows = slice(lo, lo + 300)
        want = O.ref_q8_mm(a[rows].cpu(), b.cpu(), bias.cpu(), sa[rows].cpu(), sb.cpu(), False, torch.bfloat16)
        diff = (out[0, rows].cpu().view(torch.int16).int() - want[0].view(torch.int16).int()).abs()
        assert int(diff.max()) <= 1, "rows %d..%d: %d ulp" % (lo, lo + 300, int(diff.max()))
    del a, out
    torch.cuda.empty_cache()


# ------------------------------------------------------------------ the block's M = 12288 GEMM shapes

@pytest.mark.parametrize("nk", [(2048, 2048), (2048, 8192)], ids=["projection_K2048", "ffn_down_K8192"])
def test_fp8_linear_block_shapes_m12288(dev, nk):
    """The fp8 linears of the DiT block at their real size, tokens [12288, K] x weight [2048, K] + bias -> bf16, against
    the float64 oracle on row blocks from the start, the middle (across a tile boundary) and the end of M. The kernel
    that ran must be one of the persistent family (the large-problem path these shapes are timed on)."""
    n, k = nk
    m = 12288
    g = torch.Generator().manual_seed(12 + k)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16)
    bias = (torch.randn(n, generator=g) * 0.02).to(torch.bfloat16).float()
    xq, sx = _C().tokenwise_quant(x.to(dev), E4M3)
    wq, sw = _C().tokenwise_quant(w.to(dev), E4M3)
    out = _C().fp8_mm_bias(xq, wq, bias.to(dev), sx, sw, False, torch.bfloat16)
    kernel = _last_kernel()
    assert kernel in PERSISTENT_KERNELS, kernel
    assert out.shape == (1, m, n)
    owq, osw = O.ref_quant(w, E4M3)
    assert_bit_equal(wq, owq, "W codes")
    for lo in (0, 6144 - 160, m - 320):
        rows = slice(lo, lo + 320)
        oxq, osx = O.ref_quant(x[rows], E4M3)
        assert_bit_equal(xq[rows], oxq, "X codes")
        v = O.ref_gemm_fp8_acc(oxq, owq) * (osx[:, None] * osw[None, :]).double() + bias.double()
        _check_float_out(out[0, rows], v, "M=12288 N=%d K=%d rows %d.." % (n, k, lo))
    assert torch.isfinite(out.float()).all()
    # the reference's default output type (out_type None -> e4m3, saturating cast) takes the same kernel family
    out8 = _C().fp8_mm_bias(xq, wq, bias.to(dev), sx, sw, False, None)
    assert _last_kernel() in PERSISTENT_KERNELS, _last_kernel()
    assert out8.dtype == E4M3 and out8.shape == (1, m, n)
    for lo in (0, m - 320):
        rows = slice(lo, lo + 320)
        oxq, osx = O.ref_quant(x[rows], E4M3)
        v = O.ref_gemm_fp8_acc(oxq, owq) * (osx[:, None] * osw[None, :]).double() + bias.double()
        want8 = O.e4m3_sat(v.float())
        g8 = out8[0, rows].cpu()
        assert not torch.isnan(g8.float()).any()
        # fp32 accumulation order moves a value across an e4m3 rounding boundary now and then: never by more than one code
        # (codes are sign-magnitude: taken as signed step counts, so that -0 = +0 and the smallest negative value is one
        # step from zero)
        steps = lambda c: (c & 0x7F) * (1 - 2 * (c >> 7))  # noqa: E731
        diff = (steps(g8.view(torch.uint8).int()) - steps(want8.view(torch.uint8).int())).abs()
        assert int(diff.max()) <= 1 and (diff > 0).float().mean() < 0.01, (int(diff.max()), (diff > 0).float().mean().item())


@pytest.mark.parametrize("in_dtype", ["fp8", "i8"])
@pytest.mark.parametrize("shape", [(2, 96, 768, 384, 512), (1, 200, 768, 640, 256), (3, 192, 1024, 512, 768)])
@pytest.mark.parametrize("rows", [43, 44], ids=["tile192", "tile256"])
def test_qkv_gemm_casts_v_in_its_epilogue(dev, in_dtype, shape, rows):
    """q8_gemm_qkv: the Q / K columns are those of the plain GEMM, the V columns the c10 e4m3 cast of the plain GEMM's
    bf16 result, token-major per head ([B, H, S, 64]): bit-equal to the GEMM followed by the cast that the attention
    prologue applies, under both tile heights of the persistent kernel."""
    from q8_kernels_amd import _lib
    b, s, n, k, v0 = shape
    g = torch.Generator().manual_seed(n + k + s)
    if in_dtype == "i8":
        a, w = _rand_i8(g, b * s, k), _rand_i8(g, n, k)
        sa, sw = torch.rand(b * s, generator=g) * 2e-3 + 1e-4, torch.rand(n, generator=g) * 2e-2 + 1e-3
        mmb = _C().q8_mm_bias
    else:
        a, w = O.e4m3_c10(torch.randn(b * s, k, generator=g) * 50), O.e4m3_c10(torch.randn(n, k, generator=g) * 50)
        sa, sw = torch.rand(b * s, generator=g) * 1e-2 + 1e-4, torch.rand(n, generator=g) * 1e-2 + 1e-4
        mmb = _C().fp8_mm_bias
    sw[v0 + 5] = 30.0   # a column of V beyond the e4m3 range: its codes are the NaN code of the c10 cast
    bias = torch.randn(n, generator=g)
    args = (a.to(dev), w.to(dev), bias.to(dev), sa.to(dev), sw.to(dev))
    _set_cfg(rows)
    try:
        qk, vc = _C().mm_bias_qkv(*args, s, v0)
        assert _last_kernel() in PERSISTENT_KERNELS
    finally:
        _set_cfg(40)
    want = mmb(*args, False, torch.bfloat16).reshape(b, s, n)
    assert torch.equal(qk.view(torch.int16), want[..., :v0].contiguous().view(torch.int16)), "Q / K columns"
    h = (n - v0) // 64
    want_v = O.e4m3_c10(want[..., v0:].cpu().reshape(b, s, h, 64).transpose(1, 2).contiguous())
    got_v, want_v8 = vc.cpu().view(torch.uint8), want_v.view(torch.uint8)
    nan = (want_v8 & 0x7f) == 0x7f
    assert nan.any() and torch.equal(got_v & 0x7f == 0x7f, nan), "NaN codes of the overflowing column"
    assert torch.equal(got_v[~nan], want_v8[~nan]), "V codes"
    with pytest.raises(RuntimeError):
        _C().mm_bias_qkv(*args, s, v0 + 64)       # the split is not on a tile boundary
    with pytest.raises(RuntimeError):
        _C().mm_bias_qkv(*args, s + 1, v0)        # rows are not whole batch elements


@pytest.mark.parametrize("in_dtype", ["fp8", "i8"])
@pytest.mark.parametrize("shape", [(2, 96, 512, 384, 0), (1, 200, 768, 640, 256), (3, 192, 1024, 512, 0), (1, 333, 256, 1024, 0)])
@pytest.mark.parametrize("rows", [43, 44], ids=["tile192", "tile256"])
def test_qkv_gemm_hadamard_of_the_heads_in_its_epilogue(dev, in_dtype, shape, rows):
    """q8_gemm_qkv with a Hadamard factor: the head-major e4m3 columns are the 64-point transform (times the factor) of the
    plain GEMM's bf16 result per head, bit-equal to the oracle's hadamard_transform(out_type=e4m3) of that result and to
    the attention prologue run on it; rows of zeros (a zero row scale) keep the signs of their zeros. The other columns
    are those of the plain GEMM."""
    b, s, n, k, v0 = shape
    g = torch.Generator().manual_seed(n + k + s)
    if in_dtype == "i8":
        a, w = _rand_i8(g, b * s, k), _rand_i8(g, n, k)
        sa, sw = torch.rand(b * s, generator=g) * 2e-3 + 1e-4, torch.rand(n, generator=g) * 2e-2 + 1e-3
        mmb = _C().q8_mm_bias
    else:
        a, w = O.e4m3_c10(torch.randn(b * s, k, generator=g) * 50), O.e4m3_c10(torch.randn(n, k, generator=g) * 50)
        sa, sw = torch.rand(b * s, generator=g) * 1e-2 + 1e-4, torch.rand(n, generator=g) * 1e-2 + 1e-4
        mmb = _C().fp8_mm_bias
    sa[3] = 0.0                                   # a token whose projection is the bias alone
    bias = torch.randn(n, generator=g)
    bias[v0:v0 + 64] = -0.0                        # ... and in its first head zeros of either sign (acc * 0 - 0)
    args = (a.to(dev), w.to(dev), bias.to(dev), sa.to(dev), sw.to(dev))
    scale = (64 ** -0.5) * (0.125 ** 0.5)
    _set_cfg(rows)
    try:
        qk, vc = _C().mm_bias_qkv(*args, s, v0, scale)
        assert _last_kernel() in PERSISTENT_KERNELS
    finally:
        _set_cfg(40)
    want = mmb(*args, False, torch.bfloat16).reshape(b, s, n)
    assert torch.equal(qk.view(torch.int16), want[..., :v0].contiguous().view(torch.int16)), "the other columns"
    h = (n - v0) // 64
    heads = want[..., v0:].cpu().reshape(b, s, h, 64).transpose(1, 2).contiguous()
    assert_bit_equal(vc, O.ref_fht(heads, scale, E4M3), "against the oracle's transform of the bf16 projection")
    assert_bit_equal(vc, _C().attn_prep_qk(want[..., v0:], h, None, None, True, scale), "against the attention prologue")
