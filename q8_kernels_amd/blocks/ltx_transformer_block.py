"""The AdaLN-modulated LTX-Video transformer block (reference: q8_kernels/blocks/ltx_transformer_block.py:9-58):
RMSNorm -> scale/shift -> self-attention (qk-RMSNorm, RoPE) -> gated residual -> cross-attention -> residual ->
RMSNorm -> scale/shift -> feed-forward -> gated residual, on int8 (Q8Linear) projections.

The modulations `norm(x) * (1 + scale) + shift` and the gated residuals `gate * y + x` run as one fused
multiply-add kernel each (multiply_add, fp32 arithmetic, one rounding to bfloat16); the reference evaluates
them with torch element-wise kernels that round to bfloat16 after every operation."""
import torch
import torch.nn as nn

from .. import _C
from .. import functional as Q8F
from ..modules.attention import Attention
from ..modules.ffn import FeedForward
from ..modules.rms_norm import RMSNorm


class LTXTransformerBlock(nn.Module):
    # True (default): norm, modulation, Hadamard rotation and int8 quantization in front of attn1 and of the
    # feed-forward run as one kernel; False: operator by operator. Both give the same bits.
    fuse_prologue = True

    def __init__(self, dim, num_heads, head_dim, kv_dim, bias=True, use_rope=True, norm_affine=False):
        super().__init__()
        self.norm1 = RMSNorm(dim, norm_affine)
        self.attn1 = Attention(dim, num_heads, head_dim, bias, bias, qk_rms_norm=True, kv_dim=None, use_rope=use_rope)
        self.attn2 = Attention(dim, num_heads, head_dim, bias, bias, qk_rms_norm=True, kv_dim=kv_dim, use_rope=False)
        self.norm2 = RMSNorm(dim, norm_affine)
        self.ff = FeedForward(dim, bias=bias)
        self.scale_shift_table = nn.Parameter(torch.randn(6, dim) / dim ** 0.5)

    @staticmethod
    def _fma(x, y, z, add):
        """x * (y + add) + z with y, z [B, 1 or T, dim]: one kernel for bfloat16 activations on the GPU."""
        if (x.dtype == torch.bfloat16 and x.is_cuda and x.dim() == 3 and x.shape[-1] % 8 == 0
                and not (torch.is_grad_enabled() and (x.requires_grad or y.requires_grad or z.requires_grad))):
            bf = lambda t: t.to(torch.bfloat16).contiguous()  # noqa: E731
            return Q8F.fma.multiply_add(x.contiguous(), bf(y), bf(z), add)
        return (x * (y + add) + z).to(x.dtype)  # differentiable; in x's dtype like the kernel's result

    def forward(self, hidden_states, freqs_cis, attention_mask, encoder_hidden_states, encoder_attention_mask,
                timestep, mm_out_dtype=torch.bfloat16, non_mm_precision=torch.bfloat16, attn_type="torch"):
        num_ada_params = self.scale_shift_table.shape[0]
        timestep_rows = timestep.reshape(hidden_states.shape[0], timestep.shape[1], num_ada_params, -1)
        # the fused prologue goes through the C ABI and carries no gradient: it is taken only when neither the input nor
        # the modulation (scale_shift_table is a parameter, timestep may be the output of a trained embedding) needs one
        fuse = (self.fuse_prologue and hidden_states.is_cuda and hidden_states.dtype == torch.bfloat16
                and non_mm_precision == torch.bfloat16 and hidden_states.dim() == 3 and hidden_states.shape[-1] % 8 == 0
                and not (torch.is_grad_enabled() and (hidden_states.requires_grad or self.scale_shift_table.requires_grad
                                                      or timestep.requires_grad)))
        # (cast and layout change in one copy kernel; nothing at all for a contiguous bfloat16 tensor)
        bf = lambda t: t.to(torch.bfloat16, memory_format=torch.contiguous_format)  # noqa: E731
        if fuse and timestep_rows.dtype == self.scale_shift_table.dtype == torch.float32:
            # the six modulation rows as contiguous bfloat16 tensors [B, T, dim] cut from ONE tensor laid out [6, B, T, dim],
            # written by the addition itself (fp32 sum, rounded once on the way out: bf16(table + timestep), the values the
            # separate cast gives) - one small kernel (q8_adaln_rows; torch's strided, casting addition takes 10 us for these
            # 24 K elements) instead of an addition, a layout change and six casts
            if timestep_rows.shape[-1] % 8 == 0 and num_ada_params <= 64 and timestep.dim() == 3:
                rows = _C.adaln_rows(self.scale_shift_table.data, timestep)
            else:
                rows = torch.empty((num_ada_params,) + tuple(timestep_rows.shape[:2]) + (timestep_rows.shape[-1],),
                                   dtype=torch.bfloat16, device=hidden_states.device)
                torch.add(self.scale_shift_table[None, None], timestep_rows, out=rows.permute(1, 2, 0, 3))
            shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = rows.unbind(dim=0)
        else:
            ada_values = self.scale_shift_table[None, None] + timestep_rows
            shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = ada_values.unbind(dim=2)
            if fuse:
                shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = bf(ada_values.permute(2, 0, 1, 3)).unbind(dim=0)

        if fuse:  # (int8 codes, row scales) of the rotated, modulated norm: what attn1's projections would compute
            norm_hidden_states = Q8F.fused.norm_modulate_quantize(hidden_states, self.norm1.weight, bf(scale_msa),
                                                                  bf(shift_msa), 1.0)
        else:
            norm_hidden_states = self._fma(self.norm1(hidden_states, non_mm_precision), scale_msa, shift_msa, 1.0)
        # with the fused path the gated residuals `y * gate + x` are formed in the epilogue of the projection that produces y
        # (attn1's output projection, the feed-forward's down projection): the bits of the fused multiply-add kernel
        gated = fuse and mm_out_dtype == torch.bfloat16
        if gated:
            hidden_states = self.attn1(norm_hidden_states, freqs_cis, None, attention_mask, non_mm_precision, mm_out_dtype,
                                       attn_type=attn_type, residual=hidden_states, gate=gate_msa)
        else:
            attn_output = self.attn1(norm_hidden_states, freqs_cis, None, attention_mask, non_mm_precision, mm_out_dtype,
                                     attn_type=attn_type)
            hidden_states = self._fma(attn_output, gate_msa, hidden_states, 0.0)

        # the residual around the cross-attention is added in the epilogue of its output projection where that applies
        hidden_states = self.attn2(hidden_states, freqs_cis=freqs_cis, encoder_hidden_states=encoder_hidden_states,
                                   attention_mask=encoder_attention_mask, non_mm_precision=non_mm_precision,
                                   mm_out_dtype=mm_out_dtype, attn_type=attn_type, residual=hidden_states)

        if fuse:
            codes, row_scales = Q8F.fused.norm_modulate_quantize(hidden_states, self.norm2.weight, bf(scale_mlp),
                                                                 bf(shift_mlp), 1.0)
            if gated:
                return self.ff(codes, out_dtype=mm_out_dtype, x_scales=row_scales, residual=hidden_states, gate=gate_mlp)
            ff_output = self.ff(codes, out_dtype=mm_out_dtype, x_scales=row_scales).to(non_mm_precision)
        else:
            norm_hidden_states = self._fma(self.norm2(hidden_states, non_mm_precision), scale_mlp, shift_mlp, 1.0)
            ff_output = self.ff(norm_hidden_states, out_dtype=mm_out_dtype).to(non_mm_precision)
        hidden_states = self._fma(ff_output, gate_mlp, hidden_states, 0.0)
        return hidden_states
