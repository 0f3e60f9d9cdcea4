"""Rotary embedding with full-shape fp32 tables (reference: q8_kernels/functional/rope.py:9-44).

The reference's apply_rope runs a pure-torch formula (its CUDA op is commented out); this one runs
the HIP kernels, which evaluate the same interleaved-pair formula and its transpose in fp32."""
from typing import Optional

import torch

from .._C import rope, rope_backward


class ROPE(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cos_freqs, sin_freqs, out_type):
        ctx.save_for_backward(cos_freqs, sin_freqs)
        ctx.out_type = out_type
        return rope(x, cos_freqs, sin_freqs, out_type)

    @staticmethod
    def backward(ctx, grad_output):
        cos_freqs, sin_freqs = ctx.saved_tensors
        return rope_backward(grad_output, cos_freqs, sin_freqs, ctx.out_type), None, None, None


def apply_rope(x: torch.Tensor, cos_freqs: torch.Tensor, sin_freqs: torch.Tensor,
               out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    assert x.dtype in (torch.float8_e4m3fn, torch.bfloat16), "apply_rope: x must be bf16 or e4m3"
    assert cos_freqs.dtype == torch.float and sin_freqs.dtype == torch.float, "apply_rope: tables must be fp32"
    assert cos_freqs.shape == x.shape and sin_freqs.shape == x.shape, "apply_rope: tables must match x"
    if torch.is_grad_enabled() and x.requires_grad:
        return ROPE.apply(x, cos_freqs, sin_freqs, out_type)
    return rope(x, cos_freqs, sin_freqs, out_type)


def video_index_grid(frames: int, height: int, width: int, batch: int = 1, device=None) -> torch.Tensor:
    """Integer (t, y, x) coordinates of a frames x height x width latent grid, token order t-major: float32
    [batch, 3, frames * height * width], the `indices_grid` that precompute_freqs_cis takes."""
    axes = [torch.arange(n, dtype=torch.float32, device=device) for n in (frames, height, width)]
    t, y, x = torch.meshgrid(*axes, indexing="ij")
    return torch.stack((t, y, x)).reshape(1, 3, -1).expand(batch, -1, -1)


def precompute_freqs_cis(indices_grid: torch.Tensor, dim: int, theta: float = 10000.0,
                         max_pos=(20, 2048, 2048), spacing: str = "exp"):
    """The 3-D fractional rotary tables of the LTX-Video transformer (q8_kernels/models/LTXVideo.py:85-148):
    indices_grid [B, 3, T] -> (cos, sin), float32 [B, T, dim], in the layout apply_rope takes.

    Each of the dim // 6 frequencies w_f is applied to the three coordinates c_a / max_pos[a] mapped to [-1, 1]
    ('exp', 'linear', 'sqrt') or left in [0, 1] ('exp_2'); column 6 f + 2 a (+ 1) of the tables holds the angle
    w_f * position_a, every angle twice (the two members of a rotated pair), and the dim % 6 left-over columns in front
    are the identity rotation."""
    import math
    n = dim // 6
    dev = indices_grid.device
    if spacing == "exp":
        w = theta ** torch.linspace(0.0, 1.0, n, device=dev, dtype=torch.float32)
    elif spacing == "exp_2":
        w = (1.0 / theta ** (torch.arange(0, dim, 6, device=dev) / dim)).to(torch.float32)
    elif spacing == "linear":
        w = torch.linspace(1.0, theta, n, device=dev, dtype=torch.float32)
    elif spacing == "sqrt":
        w = torch.linspace(1.0, theta ** 2, n, device=dev, dtype=torch.float32).sqrt()
    else:
        raise ValueError("precompute_freqs_cis: spacing %r" % (spacing,))
    w = w * (math.pi / 2)
    # a true division, like the reference's indices_grid[:, i] / max_pos[i]: a multiplication by the rounded reciprocal
    # differs by one ulp for max_pos = 20, and the highest frequency (theta * pi / 2) amplifies that to 2e-3 in the tables
    div = torch.tensor([float(m) for m in max_pos], dtype=torch.float32, device=dev)
    pos = indices_grid.to(torch.float32) / div[None, :, None]       # [B, 3, T] fractional positions
    if spacing != "exp_2":
        pos = pos * 2 - 1
    ang = pos.transpose(1, 2)[:, :, None, :] * w[None, None, :, None]  # [B, T, n, 3]: frequency-major, axis-minor
    ang = ang.reshape(ang.shape[0], ang.shape[1], 3 * n)
    b, t = ang.shape[:2]
    cos = torch.ones(b, t, dim, dtype=torch.float32, device=dev)
    sin = torch.zeros(b, t, dim, dtype=torch.float32, device=dev)
    lead = dim - 6 * n
    cos[:, :, lead:] = ang.cos().repeat_interleave(2, dim=-1)
    sin[:, :, lead:] = ang.sin().repeat_interleave(2, dim=-1)
    return cos, sin


# compact_freqs_cis: the most recent results, [(key, (cos, sin) as given, (cos, sin) compact)]
_COMPACT_CACHE = []
compact_tables = True  # False: the fused attention prologues read the tables as they are given


def clear_compact_freqs_cache():
    """Drops the compact tables kept by compact_freqs_cis, and its references to the tables they were made from."""
    del _COMPACT_CACHE[:]


def compact_freqs_cis(cos: torch.Tensor, sin: torch.Tensor, keep: int = 2):
    """(cos, sin) float32 [B, T, dim] -> the same values stored once, for the fused attention prologues
    (_C.attn_prep_qk and its siblings), which then read a quarter of the table bytes and give the same bits:

      * tables whose two entries of every rotated pair are equal (precompute_freqs_cis repeats every angle twice, like
        q8_kernels/models/LTXVideo.py:95-148) become [.., dim / 2], one entry per pair;
      * tables that are the same for every batch element (one position grid for the whole batch) become [1, T, ..].

    Whether a table has these properties is read off its values (two comparisons over the tables, with a device
    synchronisation), once: the result is kept for the last `keep` table pairs, keyed by their storage, shape and
    version counter, together with a reference to the tables themselves, so that the storage cannot be handed to
    another tensor while the entry lives (clear_compact_freqs_cache drops both). In-place changes through torch bump the
    version counter and are seen; writes that bypass it are not. Tables that have neither property, that require a
    gradient, or that are first met while a graph is being captured (no synchronisation allowed) come back unchanged."""
    if (not compact_tables or cos.dim() != 3 or cos.shape != sin.shape or not cos.is_cuda or not sin.is_cuda
            or cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.requires_grad or sin.requires_grad):
        return cos, sin
    key = (cos.device, cos.data_ptr(), cos._version, sin.data_ptr(), sin._version, tuple(cos.shape), cos.stride(), sin.stride())
    for k, _, res in _COMPACT_CACHE:
        if k == key:
            return res
    if torch.cuda.is_current_stream_capturing():
        return cos, sin
    c, s = cos, sin
    if c.shape[-1] % 2 == 0 and torch.equal(c[..., 0::2], c[..., 1::2]) and torch.equal(s[..., 0::2], s[..., 1::2]):
        c, s = c[..., 0::2], s[..., 0::2]
    if c.shape[0] > 1 and bool((c == c[:1]).all()) and bool((s == s[:1]).all()):
        c, s = c[:1], s[:1]
    res = (cos, sin) if c is cos else (c.contiguous(), s.contiguous())
    _COMPACT_CACHE.insert(0, (key, (cos, sin), res))
    del _COMPACT_CACHE[max(1, keep):]
    return res
