"""Helpers shared by the GPU parity tests."""
import torch

E4M3 = torch.float8_e4m3fn


def bits(t: torch.Tensor) -> torch.Tensor:
    """Raw bit pattern of a tensor (for bit-exact comparisons that treat NaN codes as equal)."""
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16)
    if t.dtype == E4M3:
        return t.view(torch.uint8)
    if t.dtype == torch.float32:
        return t.view(torch.int32)
    return t


def assert_bit_equal(got: torch.Tensor, want: torch.Tensor, what: str = ""):
    got, want = got.cpu(), want.cpu()
    assert got.shape == want.shape, "%s: shape %s vs %s" % (what, tuple(got.shape), tuple(want.shape))
    assert got.dtype == want.dtype, "%s: dtype %s vs %s" % (what, got.dtype, want.dtype)
    gb, wb = bits(got), bits(want)
    if not torch.equal(gb, wb):
        diff = (gb != wb)
        idx = diff.nonzero()[0].tolist()
        raise AssertionError("%s: %d of %d elements differ, first at %s: got %s want %s" % (
            what, int(diff.sum()), diff.numel(), idx, got[tuple(idx)].float().item() if got.dtype != torch.int8 else got[tuple(idx)].item(),
            want[tuple(idx)].float().item() if want.dtype != torch.int8 else want[tuple(idx)].item()))


def bf16_ulp(x: torch.Tensor) -> torch.Tensor:
    """Size of one bf16 ulp at |x| (fp64), floor at the smallest normal binade used in the tests."""
    ax = x.abs().double().clamp_min(2.0 ** -60)
    return torch.exp2(torch.floor(torch.log2(ax)) - 7)


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.detach().double().flatten(), b.detach().double().flatten()
    return float((a @ b) / (a.norm() * b.norm()).clamp_min(1e-300))
