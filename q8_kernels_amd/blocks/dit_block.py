"""An LTX-Video-style DiT block assembled from the fp8 ops of this package:

    RMSNorm -> fp8 QKV linear -> 3-D RoPE on q, k -> fp8 Hadamard self-attention -> out projection (+ residual)
    -> RMSNorm -> fp8 cross-attention to the text states with a per-batch valid length (+ residual)
    -> RMSNorm -> fp8 FFN with bias + tanh-GELU fused into the first GEMM (+ residual)

It is the simplified block of the benchmark configuration (hidden 2048, 32 heads x 64, FFN 8192), built
on the same kernels that the reference's LTXTransformerBlock (q8_kernels/blocks/ltx_transformer_block.py:21-58)
reaches through its modules; AdaLN modulation and the qk-RMSNorm of that block are not part of it.
"""
import torch
import torch.nn as nn

from .. import _C
from .. import functional as Q8F
from ..modules.linear import FP8Linear
from ..modules.rms_norm import RMSNorm


class Fp8DiTBlock(nn.Module):
    # True (default): RMSNorm + quantizer, the attention prologues and the residual additions run fused into their
    # neighbours; False: one operator per step of the docstring's sequence. Both give the same bits.
    fuse = True
    # True (default): the cross-attention's queries leave their projection's GEMM as the attention kernel's e4m3 operand
    # (Hadamard transform per head and cast in the epilogue); False: the projection is written as bfloat16 and the
    # attention prologue reads it back. Same bits.
    fuse_query_epilogue = True

    def __init__(self, dim: int = 2048, num_heads: int = 32, head_dim: int = 64, ffn_dim: int = 8192,
                 text_dim: int = 2048, device=None):
        super().__init__()
        assert num_heads * head_dim == dim
        self.dim, self.num_heads, self.head_dim = dim, num_heads, head_dim
        self.norm1, self.norm2, self.norm3 = (RMSNorm(dim, True, device) for _ in range(3))
        mk = lambda i, o: FP8Linear(i, o, bias=True, device=device)  # noqa: E731
        self.to_qkv = mk(dim, 3 * dim)
        self.to_out = mk(dim, dim)
        # the K and V projections of the text states share their input: one layer of 2 * dim outputs (K first), like to_qkv
        self.to_q2, self.to_kv2, self.to_out2 = mk(dim, dim), mk(text_dim, 2 * dim), mk(dim, dim)
        self.ff_up, self.ff_down = mk(dim, ffn_dim), mk(ffn_dim, dim)

    @torch.no_grad()
    def init_random(self, std: float = 0.02, seed: int = 0):
        """Random weights ~ N(0, std) quantized per output channel to e4m3, biases ~ N(0, std) in fp32."""
        g = torch.Generator().manual_seed(seed)
        for m in self.modules():
            if isinstance(m, FP8Linear):
                dev = m.weight.device
                w = (torch.randn(m.weight.shape, generator=g) * std).to(torch.bfloat16).to(dev)
                m.weight.data, m.scales.data = Q8F.quantizer.quantize_fp8(w)
                m.bias.data = (torch.randn(m.bias.shape, generator=g) * std).to(torch.bfloat16).float().to(dev)
        return self

    def _lin(self, layer, x, fuse_gelu=False, residual=None):
        """layer(x) (+ residual, added in the GEMM's epilogue)."""
        return Q8F.linear.fp8_linear(x, layer.weight.data, layer.bias.data, None, layer.scales, False, x.dtype,
                                     fuse_gelu=fuse_gelu, residual=residual)

    def _norm_lin(self, norm, layer, x, fuse_gelu=False):
        """layer(norm(x)) with the norm and the e4m3 quantizer of the layer's input in one kernel."""
        codes, scales = Q8F.fused.rms_norm_quantize(x, norm.weight, torch.float8_e4m3fn)
        return Q8F.linear.fp8_linear(codes, layer.weight.data, layer.bias.data, scales, layer.scales, False, x.dtype,
                                     fuse_gelu=fuse_gelu)

    def _forward_by_operator(self, hidden, text, freqs_cis, text_lens):
        bf16 = torch.bfloat16
        d, h = self.dim, self.num_heads
        b = hidden.shape[0]
        heads = lambda t: t.reshape(b, -1, h, self.head_dim).transpose(1, 2)  # noqa: E731
        merge = lambda t: t.transpose(1, 2).reshape(b, -1, d)  # noqa: E731
        lin = lambda layer, x, gelu=False: Q8F.linear.fp8_linear(  # noqa: E731
            x, layer.weight.data, layer.bias.data, None, layer.scales, False, bf16, fuse_gelu=gelu).reshape(b, -1, layer.out_features)
        q, k, v = lin(self.to_qkv, self.norm1(hidden)).split(d, dim=-1)
        q, k = Q8F.rope.apply_rope(q.contiguous(), *freqs_cis), Q8F.rope.apply_rope(k.contiguous(), *freqs_cis)
        a = Q8F.flash_attention.flash_attn_func(heads(q), heads(k), heads(v), None, None, True, out_dtype=bf16)
        hidden = hidden + lin(self.to_out, merge(a))
        n = self.norm2(hidden)
        k2, v2 = lin(self.to_kv2, text).split(d, dim=-1)
        a = Q8F.flash_attention.flash_attn_func(heads(lin(self.to_q2, n)), heads(k2), heads(v2), None, text_lens, True, out_dtype=bf16)
        hidden = hidden + lin(self.to_out2, merge(a))
        return hidden + lin(self.ff_down, lin(self.ff_up, self.norm3(hidden), True))

    def forward(self, hidden, text, freqs_cis, text_lens):
        if not self.fuse:
            return self._forward_by_operator(hidden, text, freqs_cis, text_lens)
        bf16 = torch.bfloat16
        d, h = self.dim, self.num_heads
        # self-attention: q, k, v are read in place from the fused projection by the attention prologue kernels
        # (what the persistent GEMM kernel takes: K = d a multiple of 128 above 256, operands below 2^32 bytes)
        gemm_writes_codes = (self.head_dim == 64 and d > 256 and d % 128 == 0 and hidden.numel() < 2 ** 32
                             and self.to_qkv.weight.numel() < 2 ** 32)
        if gemm_writes_codes:
            # the V columns leave the projection's GEMM as the attention kernel's e4m3 operand, token-major per head
            # (shapes of the persistent GEMM kernel: K = d a multiple of 128 above 256, the split 2 d on a tile boundary)
            codes, scales = Q8F.fused.rms_norm_quantize(hidden, self.norm1.weight, torch.float8_e4m3fn)
            qk, v_codes = _C.mm_bias_qkv(codes.reshape(-1, d), self.to_qkv.weight.data, self.to_qkv.bias.data, scales.reshape(-1),
                                         self.to_qkv.scales, hidden.shape[1], 2 * d)
            a = Q8F.fused.flash_attn_token_major(qk[..., :d], qk[..., d:], None, h, apply_qk_hadamard=True,
                                                 freqs_cis=freqs_cis, out_dtype=bf16, v_codes=v_codes)
        else:
            qkv = self._norm_lin(self.norm1, self.to_qkv, hidden)
            a = Q8F.fused.flash_attn_token_major(qkv[..., :d], qkv[..., d:2 * d], qkv[..., 2 * d:], h,
                                                 apply_qk_hadamard=True, freqs_cis=freqs_cis, out_dtype=bf16)
        hidden = self._lin(self.to_out, a, residual=hidden)
        # cross-attention to the text states
        kv2 = self._lin(self.to_kv2, text)  # k and v are read in place, like q, k, v of the self-attention
        k2, v2 = kv2[..., :d], kv2[..., d:]
        if self.fuse_query_epilogue and gemm_writes_codes:
            # the queries leave their projection's GEMM as the attention kernel's operand: Hadamard transform per head and
            # e4m3 cast in the epilogue (no rotation and no norm lies between the projection and the attention here)
            codes, scales = Q8F.fused.rms_norm_quantize(hidden, self.norm2.weight, torch.float8_e4m3fn)
            _, q_codes = _C.mm_bias_qkv(codes.reshape(-1, d), self.to_q2.weight.data, self.to_q2.bias.data, scales.reshape(-1),
                                        self.to_q2.scales, hidden.shape[1], 0, Q8F.fused.qk_hadamard_scale(self.head_dim))
            a = Q8F.fused.flash_attn_token_major(None, k2, v2, h, batch_mask=text_lens, apply_qk_hadamard=True,
                                                 out_dtype=bf16, q_codes=q_codes)
        else:
            q2 = self._norm_lin(self.norm2, self.to_q2, hidden)
            a = Q8F.fused.flash_attn_token_major(q2, k2, v2, h, batch_mask=text_lens, apply_qk_hadamard=True,
                                                 out_dtype=bf16)
        hidden = self._lin(self.to_out2, a, residual=hidden)
        # feed-forward
        up = self._norm_lin(self.norm3, self.ff_up, hidden, fuse_gelu=True)
        return self._lin(self.ff_down, up, residual=hidden)
