"""GPU parity of fma_8bit, GELU forward / backward, RoPE backward, RMSNorm backward and of the Python layers built
on them (autograd functions, LoRA linear, LTX transformer block) against the CPU oracle."""
import pytest
import torch

from oracle import q8_oracle as O
from tests.util import E4M3, assert_bit_equal, cosine

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _C():
    from q8_kernels_amd import _C as C
    return C


def _ulp_close(got, want, what, max_frac=2e-3, atol=None):
    """Equal up to one unit in the last place of the output format on at most max_frac of the elements
    (the kernels evaluate exp / rcp with the hardware approximations, the oracle in float64); elements within
    the absolute tolerance `atol` (a tensor) are accepted as they are."""
    got, want = got.cpu(), want.cpu()
    assert got.dtype == want.dtype and got.shape == want.shape
    if got.dtype == E4M3:
        gi, wi = got.view(torch.uint8).int(), want.view(torch.uint8).int()
        mag = lambda t: torch.where((t & 0x80) != 0, -(t & 0x7F), t & 0x7F)  # noqa: E731  sign-magnitude -> integer order
        d = (mag(gi) - mag(wi)).abs()
    else:
        gi, wi = got.view(torch.int16).int(), want.view(torch.int16).int()
        mag = lambda t: torch.where(t < 0, -(t & 0x7FFF), t)  # noqa: E731
        d = (mag(gi) - mag(wi)).abs()
    if atol is not None:
        d = torch.where((got.double() - want.double()).abs() <= atol.double(), torch.zeros_like(d), d)
    assert int(d.max()) <= 1, "%s: max distance %d ulp" % (what, int(d.max()))
    assert float((d > 0).float().mean()) <= max_frac, "%s: %.4f of the elements differ" % (what, float((d > 0).float().mean()))


# ------------------------------------------------------------------ fma

@pytest.mark.parametrize("types", [(torch.float32, torch.float32), (torch.float32, E4M3), (BF16, BF16), (E4M3, BF16)])
@pytest.mark.parametrize("x_type", [E4M3, BF16])
def test_fma_bit_exact(dev, types, x_type):
    g = torch.Generator().manual_seed(41)
    b, t, dim = 3, 37, 2048
    to = lambda v, dt: O.e4m3_c10(v) if dt == E4M3 else v.to(dt)  # noqa: E731
    x = to(torch.randn(b, t, dim, generator=g) * 2, x_type)
    for ty, tz in ((1, 1), (1, t), (t, 1), (t, t)):
        y = to(torch.randn(b, ty, dim, generator=g), types[0])
        z = to(torch.randn(b, tz, dim, generator=g), types[1])
        got = _C().fma_8bit(x.to(dev), y.to(dev), z.to(dev), 1.0)
        assert_bit_equal(got, O.ref_fma(x, y, z, 1.0), "fma y rows %d z rows %d" % (ty, tz))
    got = _C().fma_8bit(x.to(dev), y.to(dev), z.to(dev), 0.0, out_type=BF16)
    assert_bit_equal(got, O.ref_fma(x, y, z, 0.0, BF16), "fma bf16 output")


def test_fma_rejects_bad_arguments(dev):
    x = torch.zeros(2, 4, 64, device=dev).to(E4M3)
    y = torch.zeros(2, 1, 64, device=dev)
    with pytest.raises(RuntimeError):
        _C().fma_8bit(x, torch.zeros(2, 1, 32, device=dev), y)          # channels
    with pytest.raises(RuntimeError):
        _C().fma_8bit(x, torch.zeros(2, 3, 64, device=dev), y)          # tokens
    with pytest.raises(RuntimeError):
        _C().fma_8bit(x, y.to(torch.float16), y)                        # dtype


# ------------------------------------------------------------------ GELU forward / backward

@pytest.mark.parametrize("in_type", [BF16, E4M3])
@pytest.mark.parametrize("out_type", [BF16, E4M3])
def test_gelu_forward_and_backward(dev, in_type, out_type):
    g = torch.Generator().manual_seed(42)
    x = torch.randn(33, 512, generator=g) * 3
    x[0, :16] = torch.tensor([0.0, -0.0, 1e-3, -1e-3, 20.0, -20.0, 100.0, -100.0, 5.0, -5.0, 0.5, -0.5, 2.0, -2.0, 8.0, -8.0])
    x = O.e4m3_c10(x) if in_type == E4M3 else x.to(BF16)
    go = torch.randn(33, 512, generator=g)
    go = O.e4m3_c10(go) if out_type == E4M3 else go.to(BF16)
    # far in the negative tail the literal formula 1 + tanh(tau) cancels (in float64 below 1e-16, in the reference's
    # fp32 below 6e-8); the kernels form 0.5 (1 + tanh) without cancellation, so there only an absolute bound applies
    tail = x.float().abs() * 2.0 ** -24
    _ulp_close(_C().gelu_forward(x.to(dev), out_type), O.ref_gelu_forward(x, out_type), "gelu forward", atol=tail)
    _ulp_close(_C().gelu_backward(x.to(dev), go.to(dev), out_type), O.ref_gelu_backward(x, go, out_type), "gelu backward",
               atol=tail * go.float().abs() * 8)


# ------------------------------------------------------------------ RoPE backward

@pytest.mark.parametrize("in_type", [BF16, E4M3])
@pytest.mark.parametrize("out_type", [BF16, E4M3])
def test_rope_backward_bit_exact(dev, in_type, out_type):
    g = torch.Generator().manual_seed(43)
    go = torch.randn(2, 19, 256, generator=g)
    go = O.e4m3_c10(go) if in_type == E4M3 else go.to(BF16)
    ang = torch.rand(2, 19, 128, generator=g) * 6.28
    cos, sin = torch.cos(ang).repeat_interleave(2, -1), torch.sin(ang).repeat_interleave(2, -1)
    got = _C().rope_backward(go.to(dev), cos.to(dev), sin.to(dev), out_type)
    assert_bit_equal(got, O.ref_rope_backward(go, cos, sin, out_type), "rope backward")


# ------------------------------------------------------------------ RMSNorm backward

@pytest.mark.parametrize("dim", [64, 1000, 2048, 8192])
def test_rms_norm_backward(dev, dim):
    g = torch.Generator().manual_seed(44 + dim)
    x = (torch.randn(37, dim, generator=g) * 1.3).to(BF16)
    go = torch.randn(37, dim, generator=g).to(BF16)
    for w in (None, 1 + 0.1 * torch.randn(dim, generator=g)):
        y, rstd = O.ref_rms_norm(x, w, BF16)
        got = _C().rms_norm_backward(y.to(dev), rstd.to(dev), go.to(dev), None if w is None else w.to(dev), BF16)
        want = O.ref_rms_norm_backward(y, rstd, go, w, BF16)
        # the row dot product is summed in fp32 in another order than the oracle's float64: compare to the
        # unrounded float64 result with a bound of one bf16 ulp plus the dot product's rounding share
        ref64 = O.ref_rms_norm_backward(y, rstd, go, w, torch.float32).double()
        err = (got.cpu().double() - ref64).abs()
        tol = ref64.abs() * 2.0 ** -8 + (y.double().abs() * rstd.double()[:, None]) * 1e-5 + 1e-7
        assert bool((err <= tol).all()), float((err - tol).max())
        assert float((got.cpu().view(torch.int16) != want.view(torch.int16)).float().mean()) < 0.02


def test_autograd_functions_call_the_backward_kernels(dev):
    import q8_kernels_amd.functional as Q8F
    g = torch.Generator().manual_seed(45)
    x = torch.randn(2, 9, 256, generator=g).to(BF16)
    w = (1 + 0.1 * torch.randn(256, generator=g))
    go = torch.randn(2, 9, 256, generator=g).to(BF16)
    xd = x.to(dev).requires_grad_(True)
    y = Q8F.rms_norm.rms_norm_8bit(xd, w.to(dev), BF16)
    y.backward(go.to(dev))
    yo, ro = O.ref_rms_norm(x, w, BF16)
    assert cosine(xd.grad.cpu(), O.ref_rms_norm_backward(yo, ro, go, w, BF16)) > 0.99999
    ang = torch.rand(2, 9, 128, generator=g) * 6.28
    cos, sin = torch.cos(ang).repeat_interleave(2, -1), torch.sin(ang).repeat_interleave(2, -1)
    xd = x.to(dev).requires_grad_(True)
    Q8F.rope.apply_rope(xd, cos.to(dev), sin.to(dev), BF16).backward(go.to(dev))
    assert_bit_equal(xd.grad, O.ref_rope_backward(go, cos, sin, BF16), "rope autograd")


# ------------------------------------------------------------------ linear backward and LoRA

def test_linear_backward_and_lora(dev):
    import torch.nn as nn
    import q8_kernels_amd.functional as Q8F
    from q8_kernels_amd.modules import Q8Linear, Q8LinearLora
    torch.manual_seed(46)
    lin = nn.Linear(256, 128).to(dev).to(BF16)
    x = torch.randn(2, 33, 256, device=dev).to(BF16)
    go = torch.randn(2, 33, 128, device=dev).to(BF16)
    want_dx = (go.double() @ lin.weight.data.double())
    # int8 path with Hadamard, and fp8 path with and without
    q8 = Q8Linear.from_linear(lin)
    xd = x.clone().requires_grad_(True)
    q8(xd, out_dtype=BF16).backward(go)
    assert xd.grad.shape == x.shape and cosine(xd.grad.cpu(), want_dx.cpu()) > 0.995
    for had in (False, True):
        xd = x.clone().requires_grad_(True)
        Q8F.linear.fp8_linear(xd, lin.weight.data, lin.bias.data.float(), use_hadamard=had, out_dtype=BF16).backward(go)
        assert cosine(xd.grad.cpu(), want_dx.cpu()) > 0.995
    # LoRA: forward = base + adapter, gradients of the adapter match autograd of the dense formula
    lora = Q8LinearLora.from_linear(q8, r=8)
    with torch.no_grad():
        lora.lora_b.copy_((torch.randn(128, 8, device=dev) * 0.05).to(BF16))
    for gelu in (False, True):
        lora.zero_grad()
        xd = x.clone().requires_grad_(True)
        y = lora(xd, fuse_gelu=gelu, out_dtype=BF16)
        y.backward(go)
        xr = x.double().clone().requires_grad_(True)
        la, lb = lora.lora_a.data.double().clone().requires_grad_(True), lora.lora_b.data.double().clone().requires_grad_(True)
        pre = xr @ lin.weight.data.double().T + lin.bias.data.double() + (xr @ la.T) @ lb.T
        yr = torch.nn.functional.gelu(pre, approximate="tanh") if gelu else pre
        yr.backward(go.double())
        assert y.shape == (2, 33, 128) and cosine(y.detach().cpu(), yr.detach().cpu()) > 0.998
        assert cosine(xd.grad.cpu(), xr.grad.cpu()) > 0.99
        assert cosine(lora.lora_a.grad.cpu(), la.grad.cpu()) > 0.99
        assert cosine(lora.lora_b.grad.cpu(), lb.grad.cpu()) > 0.99


def test_gradients_reach_every_input_that_asks_for_one(dev):
    """Three places where a gradient used to be dropped without an error: a bare hadamard_transform, fp8_linear with a
    fused GELU or residual, q8_linear with a fused GELU. Each against float64 autograd of the dense formula."""
    import scipy.linalg
    import q8_kernels_amd.functional as Q8F
    g = torch.Generator().manual_seed(50)
    x = torch.randn(3, 17, 256, generator=g).to(BF16)
    go = torch.randn(3, 17, 256, generator=g).to(BF16)
    # hadamard_transform: y = x H / 16, dy/dx = H / 16 (symmetric)
    xd = x.to(dev).requires_grad_(True)
    y = Q8F.fast_hadamard.hadamard_transform(xd)
    assert y.requires_grad and y.grad_fn is not None
    y.backward(go.to(dev))
    H = torch.tensor(scipy.linalg.hadamard(256), dtype=torch.float64) / 16.0
    assert xd.grad.dtype == BF16 and cosine(xd.grad.cpu(), go.double() @ H) > 0.99999
    # linears with fused epilogues
    w = (torch.randn(128, 256, generator=g) / 16).to(BF16)
    bias = torch.randn(128, generator=g) * 0.1
    res = torch.randn(3, 17, 128, generator=g).to(BF16)
    go2 = torch.randn(3, 17, 128, generator=g).to(BF16)
    for kind in ("fp8_gelu", "fp8_residual", "fp8_gelu_residual", "q8_gelu"):
        xd = x.to(dev).requires_grad_(True)
        rd = res.to(dev).requires_grad_(True)
        if kind.startswith("fp8"):
            out = Q8F.linear.fp8_linear(xd, w.to(dev), bias.to(dev), out_dtype=BF16, fuse_gelu="gelu" in kind,
                                        residual=rd if "residual" in kind else None)
        else:
            out = Q8F.linear.q8_linear(xd, w.to(dev), bias.to(dev), fuse_gelu=True, out_dtype=BF16)
        assert out.grad_fn is not None, kind
        out.reshape(3, 17, 128).backward(go2.to(dev))
        xr = x.double().requires_grad_(True)
        rr = res.double().requires_grad_(True)
        pre = xr @ w.double().T + bias.double()
        want = torch.nn.functional.gelu(pre, approximate="tanh") if "gelu" in kind else pre
        if "residual" in kind:
            want = want + rr
        want.backward(go2.double())
        assert cosine(out.detach().cpu(), want.detach()) > 0.998, kind
        assert cosine(xd.grad.cpu(), xr.grad) > 0.99, kind
        if "residual" in kind:
            assert cosine(rd.grad.cpu(), rr.grad) > 0.99999, kind


def test_ltx_block_modulation_table_gets_its_gradient(dev):
    """scale_shift_table is a parameter. With gradients enabled and an input that does not need one, the block must
    not take the fused prologue (which carries no gradient): the table's gradient through scale and shift, not only
    through the gates, is compared with float64 autograd of the dense block on the dequantized weights."""
    import scipy.linalg
    import torch.nn as nn
    from q8_kernels_amd.blocks import LTXTransformerBlock
    from q8_kernels_amd.modules import Q8Linear
    from tests.test_oracle import _dense_ltx_block
    torch.manual_seed(51)
    dim, heads, hd, kv_dim, s_tok, s_txt = 256, 4, 64, 128, 48, 24
    blk = LTXTransformerBlock(dim, heads, hd, kv_dim, bias=True, use_rope=True, norm_affine=False).to(dev)
    W = {}
    for name, m in blk.named_modules():
        if isinstance(m, Q8Linear):
            src = nn.Linear(m.in_features, m.out_features).to(dev).to(BF16)
            q = Q8Linear.from_linear(src)
            m.weight.data, m.scales.data, m.bias.data = q.weight.data, q.scales.data, q.bias.data
            key = {"ff.act.proj": "ff.up", "ff.proj_down": "ff.down"}.get(name, name)
            W[key] = (src.weight.data.cpu(), src.bias.data.float().cpu())
    for a in ("attn1", "attn2"):
        W[a + ".q_norm"] = getattr(blk, a).q_norm.weight.data.cpu()
        W[a + ".k_norm"] = getattr(blk, a).k_norm.weight.data.cpu()
    g = torch.Generator().manual_seed(52)
    hidden = torch.randn(2, s_tok, dim, generator=g).to(BF16)
    text = torch.randn(2, s_txt, kv_dim, generator=g).to(BF16)
    timestep = torch.randn(2, 1, 6 * dim, generator=g) * 0.3
    go = torch.randn(2, s_tok, dim, generator=g).to(BF16)
    grid = torch.stack(torch.meshgrid(torch.arange(2), torch.arange(4), torch.arange(6), indexing="ij")).reshape(3, -1)
    cos, sin = O.ref_freqs_cis(grid[None].float().repeat(2, 1, 1), dim)
    lens = torch.tensor([24, 9], dtype=torch.int32)
    impl, calls = _C().norm_mod_fht_quant, []
    def counted(*a, **k):
        calls.append(1)
        return impl(*a, **k)
    try:
        _C().norm_mod_fht_quant = counted
        out = blk(hidden.to(dev), (cos.to(dev), sin.to(dev)), None, text.to(dev), lens.to(dev), timestep.to(dev),
                  attn_type="torch")  # the differentiable attention (the fp8 kernel is forward-only, as in the reference)
    finally:
        _C().norm_mod_fht_quant = impl
    assert not calls, "the fused prologue ran although scale_shift_table needs a gradient"
    out.backward(go.to(dev))
    got = blk.scale_shift_table.grad
    assert got is not None and torch.isfinite(got).all()
    Wd = dict(W)
    table = blk.scale_shift_table.data.cpu().double().requires_grad_(True)
    Wd["scale_shift_table"] = table
    want_out = _dense_ltx_block(Wd, hidden, (cos, sin), text, lens, timestep, heads, hd)
    want_out.backward(go.double())
    assert cosine(out.detach().cpu(), want_out.detach()) > 0.995
    for row, name in enumerate(("shift_msa", "scale_msa", "gate_msa", "shift_mlp", "scale_mlp", "gate_mlp")):
        assert got[row].abs().max() > 0, name
        assert cosine(got[row].cpu(), table.grad[row]) > 0.97, (name, cosine(got[row].cpu(), table.grad[row]))


# ------------------------------------------------------------------ LTX transformer block

def test_ltx_transformer_block_matches_oracle(dev):
    import torch.nn as nn
    from q8_kernels_amd.blocks import LTXTransformerBlock
    from q8_kernels_amd.modules import Q8Linear
    torch.manual_seed(47)
    dim, heads, hd, kv_dim, s_tok, s_txt = 256, 4, 64, 192, 96, 24
    blk = LTXTransformerBlock(dim, heads, hd, kv_dim, bias=True, use_rope=True, norm_affine=False).to(dev)
    params = {"scale_shift_table": blk.scale_shift_table.data.cpu(), "norm1": None, "norm2": None}
    for name, m in blk.named_modules():
        if isinstance(m, Q8Linear):
            src = nn.Linear(m.in_features, m.out_features).to(dev).to(BF16)
            q = Q8Linear.from_linear(src)
            m.weight.data, m.scales.data, m.bias.data = q.weight.data, q.scales.data, q.bias.data
            key = {"ff.act.proj": "ff.up", "ff.proj_down": "ff.down"}.get(name, name)
            params[key] = (m.weight.data.cpu(), m.scales.data.cpu(), m.bias.data.cpu())
    for a in ("attn1", "attn2"):
        params[a + ".q_norm"] = getattr(blk, a).q_norm.weight.data.cpu()
        params[a + ".k_norm"] = getattr(blk, a).k_norm.weight.data.cpu()
    g = torch.Generator().manual_seed(48)
    hidden = torch.randn(2, s_tok, dim, generator=g).to(BF16)
    text = torch.randn(2, s_txt, kv_dim, generator=g).to(BF16)
    timestep = (torch.randn(2, 1, 6 * dim, generator=g) * 0.3)
    grid = torch.stack(torch.meshgrid(torch.arange(4), torch.arange(4), torch.arange(6), indexing="ij")).reshape(3, -1)
    cos, sin = O.ref_freqs_cis(grid[None].float().repeat(2, 1, 1), dim)
    lens = torch.tensor([24, 9], dtype=torch.int32)
    with torch.no_grad():
        got = blk(hidden.to(dev), (cos.to(dev), sin.to(dev)), None, text.to(dev), lens.to(dev), timestep.to(dev),
                  attn_type="q8_kernels")
    want = O.ref_ltx_block(params, hidden, (cos, sin), text, lens, timestep, heads, hd, p_scale=256.0)  # the kernel's default P grid
    assert got.shape == hidden.shape and got.dtype == BF16
    assert cosine(got.cpu(), want) > 0.999
    assert (got.cpu().double() - want.double()).abs().max() <= 0.06 * want.double().abs().max()
    # operator by operator (no fused prologues anywhere): the same bits. The fused kernel is counted, so that
    # the comparison cannot pass by both runs taking the same path.
    from q8_kernels_amd.modules import Attention
    impl, calls = _C().norm_mod_fht_quant, []
    mm_impl, with_residual, with_gate = _C().q8_mm_bias, [], []
    def counted(*a, **k):
        calls.append(1)
        return impl(*a, **k)
    def counted_mm(*a, **k):
        if k.get("residual") is not None:
            with_residual.append(1)
        if k.get("gate") is not None:
            with_gate.append(1)
        return mm_impl(*a, **k)
    run = lambda: blk(hidden.to(dev), (cos.to(dev), sin.to(dev)), None, text.to(dev), lens.to(dev),  # noqa: E731
                      timestep.to(dev), attn_type="q8_kernels")
    try:
        _C().norm_mod_fht_quant, _C().q8_mm_bias = counted, counted_mm
        with torch.no_grad():
            again = run()
        assert len(calls) == 2, f"fused prologue ran {len(calls)} times, expected 2 (attn1 and feed-forward)"
        assert len(with_residual) == 3, f"{len(with_residual)} GEMMs carried a residual, expected 3 (the output projections of attn1 and attn2, the feed-forward's down projection)"
        assert len(with_gate) == 2, f"{len(with_gate)} GEMMs carried a gate, expected 2 (attn1 and the feed-forward)"
        LTXTransformerBlock.fuse_prologue = Attention.fuse_prologue = False
        with torch.no_grad():
            seq = run()
        assert len(calls) == 2, "the operator-by-operator path called the fused prologue"
        assert len(with_residual) == 3 and len(with_gate) == 2, "the operator-by-operator path added a residual inside a GEMM"
    finally:
        _C().norm_mod_fht_quant, _C().q8_mm_bias = impl, mm_impl
        LTXTransformerBlock.fuse_prologue = Attention.fuse_prologue = True
    assert_bit_equal(got, again, "fused block, second run")
    assert_bit_equal(got, seq, "fused block vs operator sequence")


def test_ltx_block_gated_residuals_in_the_gemm_epilogue(dev):
    """768 tokens per batch element at dim 512: the two gated residuals of the block run inside the persistent GEMM's
    epilogue (asserted through the record of the kernel that ran). The block gives the bits of the operator-by-operator
    sequence, whose gated residuals are separate fused multiply-add kernels."""
    import torch.nn as nn
    from q8_kernels_amd import _lib
    from q8_kernels_amd.blocks import LTXTransformerBlock
    from q8_kernels_amd.modules import Attention, Q8Linear
    torch.manual_seed(53)
    dim, heads, hd, kv_dim, s_tok, s_txt = 512, 8, 64, 256, 768, 40
    blk = LTXTransformerBlock(dim, heads, hd, kv_dim, bias=True, use_rope=True, norm_affine=False).to(dev)
    for name, m in blk.named_modules():
        if isinstance(m, Q8Linear):
            q = Q8Linear.from_linear(nn.Linear(m.in_features, m.out_features).to(dev).to(BF16))
            m.weight.data, m.scales.data, m.bias.data = q.weight.data, q.scales.data, q.bias.data
    g = torch.Generator().manual_seed(54)
    hidden = torch.randn(2, s_tok, dim, generator=g).to(BF16).to(dev)
    text = torch.randn(2, s_txt, kv_dim, generator=g).to(BF16).to(dev)
    timestep = (torch.randn(2, 1, 6 * dim, generator=g) * 0.3).to(dev)
    grid = torch.stack(torch.meshgrid(torch.arange(8), torch.arange(8), torch.arange(12), indexing="ij")).reshape(3, -1)
    cos, sin = (t.to(dev) for t in O.ref_freqs_cis(grid[None].float().repeat(2, 1, 1), dim))
    lens = torch.tensor([40, 17], dtype=torch.int32).to(dev)
    mm_impl, kernels = _C().q8_mm_bias, []
    def recording_mm(*a, **k):
        out = mm_impl(*a, **k)
        if k.get("gate") is not None:
            kernels.append(_lib.lib().q8_gemm_last_kernel())
        return out
    run = lambda: blk(hidden, (cos, sin), None, text, lens, timestep, attn_type="q8_kernels")  # noqa: E731
    try:
        _C().q8_mm_bias = recording_mm
        with torch.no_grad():
            fused = run()
        assert len(kernels) == 2 and all(kk & _lib.Q8_GEMM_KERNEL_RESIDUAL for kk in kernels), kernels
        LTXTransformerBlock.fuse_prologue = Attention.fuse_prologue = False
        with torch.no_grad():
            seq = run()
        assert len(kernels) == 2, "the operator-by-operator path passed a gate into a GEMM"
    finally:
        _C().q8_mm_bias = mm_impl
        LTXTransformerBlock.fuse_prologue = Attention.fuse_prologue = True
    assert torch.isfinite(fused.float()).all()
    assert_bit_equal(fused, seq, "block with gated epilogues vs operator sequence")


@pytest.mark.parametrize("dim", [256, 1000, 2048, 8192])
@pytest.mark.parametrize("out_type", [torch.int8, E4M3])
def test_norm_mod_fht_quant_equals_the_operator_sequence(dev, dim, out_type):
    g = torch.Generator().manual_seed(dim + 3)
    b, t = 2, 19
    x = (torch.randn(b, t, dim, generator=g) * 1.3).to(BF16)
    w = 1 + 0.1 * torch.randn(dim, generator=g)
    for tm, mod_type in ((1, BF16), (t, BF16), (1, torch.float32)):
        sc = (torch.randn(b, tm, dim, generator=g) * 0.2).to(mod_type)
        sh = (torch.randn(b, tm, dim, generator=g) * 0.2).to(mod_type)
        codes, scales = _C().norm_mod_fht_quant(x.to(dev), True, w.to(dev), sc.to(dev), sh.to(dev), 1.0, dim ** -0.5, out_type)
        y = O.ref_fma(O.ref_rms_norm(x, w, BF16)[0], sc, sh, 1.0)
        # the separate HIP kernels (same summation order): bit for bit
        yd = _C().fma_8bit(_C().rms_norm(x.to(dev), w.to(dev), BF16)[0], sc.to(dev), sh.to(dev), 1.0)
        wc, ws = _C().tokenwise_quant(_C().fast_hadamard_transform(yd, dim ** -0.5, None), out_type)
        assert_bit_equal(codes, wc, "codes vs separate kernels")
        assert_bit_equal(scales, ws, "scales vs separate kernels")
        # the oracle (float64 sum of squares): codes may move where a value sits on a rounding boundary
        oc, _ = O.ref_quant(O.ref_fht(y, dim ** -0.5, BF16), out_type)
        assert float((codes.cpu().view(torch.uint8) != oc.view(torch.uint8)).float().mean()) < 0.02
    # steps switched off: plain FHT + quantizer, and plain quantizer
    codes, scales = _C().norm_mod_fht_quant(x.to(dev), False, None, None, None, 0.0, dim ** -0.5, out_type)
    wc, ws = O.ref_quant(O.ref_fht(x, dim ** -0.5, BF16), out_type)
    assert_bit_equal(codes, wc, "fht + quant")
    assert_bit_equal(scales, ws, "fht + quant scales")
    codes, scales = _C().norm_mod_fht_quant(x.to(dev), False, None, None, None, 0.0, None, out_type)
    wc, ws = O.ref_quant(x, out_type)
    assert_bit_equal(codes, wc, "quant only")


# ------------------------------------------------------------------ weight conversion

def test_convert_state_dict_loads_into_the_block(dev):
    from q8_kernels_amd.blocks import LTXTransformerBlock
    from q8_kernels_amd.utils import convert_state_dict
    dim, heads, hd, kv_dim = 256, 4, 64, 192
    g = torch.Generator().manual_seed(49)
    rnd = lambda *s: (torch.randn(*s, generator=g) * 0.05).to(BF16)  # noqa: E731
    p = "transformer_blocks.0."
    orig = {"proj_in.weight": rnd(dim, 32), p + "scale_shift_table": torch.randn(6, dim, generator=g)}
    for a, kd in (("attn1", dim), ("attn2", kv_dim)):
        for name, i in (("to_q", dim), ("to_k", kd), ("to_v", kd), ("to_out.0", dim)):
            orig[p + "%s.%s.weight" % (a, name)] = rnd(dim, i)
            orig[p + "%s.%s.bias" % (a, name)] = rnd(dim)
        orig[p + a + ".q_norm.weight"] = 1 + rnd(dim)
        orig[p + a + ".k_norm.weight"] = 1 + rnd(dim)
    orig[p + "ff.net.0.proj.weight"], orig[p + "ff.net.0.proj.bias"] = rnd(4 * dim, dim), rnd(4 * dim)
    orig[p + "ff.net.2.weight"], orig[p + "ff.net.2.bias"] = rnd(dim, 4 * dim), rnd(dim)
    new = convert_state_dict(orig, torch.device(dev))
    assert new["proj_in.weight"] is orig["proj_in.weight"]
    assert p + "attn1.to_out.weight" in new and p + "attn1.to_out.0.weight" not in new
    wq, ws = O.ref_quant(O.ref_fht(orig[p + "ff.net.2.weight"]))
    assert_bit_equal(new[p + "ff.proj_down.weight"], wq, "converted codes")
    assert_bit_equal(new[p + "ff.proj_down.scales"], ws, "converted scales")
    assert new[p + "attn2.k_norm.weight"].dtype == torch.float32 and new[p + "ff.act.proj.bias"].dtype == torch.float32
    blk = LTXTransformerBlock(dim, heads, hd, kv_dim, bias=True, use_rope=True, norm_affine=False).to(dev)
    missing, unexpected = blk.load_state_dict({k[len(p):]: v for k, v in new.items() if k.startswith(p)}, strict=True)
    assert not missing and not unexpected
    assert blk.ff.proj_down.weight.dtype == torch.int8 and blk.attn1.to_q.scales.dtype == torch.float32


@pytest.mark.parametrize("shape", [(2, 1, 6, 2048), (3, 5, 6, 512), (1, 1, 2, 8), (2, 700, 6, 64)])
def test_adaln_rows(dev, shape):
    """q8_adaln_rows: bf16(table + timestep) per modulation parameter, each parameter's rows contiguous - the bits of the
    torch expression of the block (q8_kernels/blocks/ltx_transformer_block.py:30-36) followed by the cast."""
    b, t, p, dim = shape
    g = torch.Generator().manual_seed(b * 100 + t + dim)
    table = (torch.randn(p, dim, generator=g) / dim ** 0.5)
    ts = torch.randn(b, t, p * dim, generator=g) * 0.3
    got = _C().adaln_rows(table.to(dev), ts.to(dev))
    want = (table[None, None] + ts.reshape(b, t, p, dim)).to(torch.bfloat16).permute(2, 0, 1, 3).contiguous()
    assert got.shape == (p, b, t, dim) and got.is_contiguous()
    assert_bit_equal(got, want, "modulation rows")
    with pytest.raises(RuntimeError):
        _C().adaln_rows(table.to(dev), ts[..., :-8].to(dev))
