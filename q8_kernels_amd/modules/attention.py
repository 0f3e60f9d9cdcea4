"""Multi-head attention over Q8Linear projections (reference: q8_kernels/modules/attention.py:15-106).

attn_type 'q8_kernels' runs the fp8 flash-attention kernel, 'torch' (the reference's default) runs
torch SDPA in `non_mm_precision`."""
from typing import Optional

import torch
import torch.nn as nn

from .. import _C
from .. import functional as Q8F
from .linear import Q8Linear
from .rms_norm import RMSNorm


class Attention(nn.Module):
    # False runs the reference's operator sequence (rope, split heads, flash_attn_func, merge) kernel by kernel;
    # True (default) takes the fused prologue kernels where they apply. Both give the same bits.
    fuse_prologue = True
    # True (default): on the fused self-attention path the V projection's GEMM writes the attention kernel's e4m3 operand
    # itself; False: V passes through memory as bfloat16 and the prologue casts it. The same bits either way.
    cast_v_in_gemm = True
    # True (default): on the fused path the projections that share an input run as ONE GEMM over the concatenation of their
    # weights - q, k, v of a self-attention (V leaves it as the attention kernel's e4m3 operand), k and v of a
    # cross-attention - instead of one launch per layer. The concatenation is a copy made on first use and made again when a
    # layer's weight, scales or bias is replaced or modified through the parameter (in-place writes through `.data` are not
    # seen: call invalidate_fused_weights() after them). Every output column depends on its own weight row only and is
    # accumulated in the same order whatever the tile it falls into: the same bits as the separate layers.
    fuse_projections = True

    def __init__(self, query_dim: int, num_heads: int, head_dim: int, bias: bool = False, out_bias: bool = False,
                 out_dim: Optional[int] = None, qk_rms_norm: bool = False, kv_dim: Optional[int] = None,
                 use_rope: bool = False):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.query_dim = query_dim
        self.bias = bias
        self.out_bias = out_bias
        self.inner_dim = num_heads * head_dim
        self.qk_rms_norm = qk_rms_norm
        if qk_rms_norm:
            self.q_norm = RMSNorm(self.inner_dim)
            self.k_norm = RMSNorm(self.inner_dim)
        self.use_rope = use_rope
        kv_dim = query_dim if kv_dim is None else kv_dim
        out_dim = query_dim if out_dim is None else out_dim
        self.to_q = Q8Linear(query_dim, self.inner_dim, bias=bias)
        self.to_k = Q8Linear(kv_dim, self.inner_dim, bias=bias)
        self.to_v = Q8Linear(kv_dim, self.inner_dim, bias=bias)
        self.to_out = Q8Linear(self.inner_dim, out_dim, out_bias)

    def invalidate_fused_weights(self):
        """Drop the concatenated copies of the projection weights (they are rebuilt on the next call)."""
        self.__dict__.pop("_fused_weights", None)

    def _fused_weights_of(self, names):
        """(weight, bias or None, scales) of the layers `names` concatenated along the output dimension; None when the
        copy would have to be made while a graph is being captured (it would live in the graph's memory pool and die with
        the graph: the caller then takes the separate layers)."""
        layers = [getattr(self, n) for n in names]
        tensors = [t for layer in layers for t in (layer.weight, layer.scales, layer.bias) if t is not None]
        key = tuple((t.data_ptr(), t._version, tuple(t.shape)) for t in tensors)
        cache = self.__dict__.setdefault("_fused_weights", {})
        hit = cache.get(names)
        if hit is None or hit[0] != key:
            if layers[0].weight.is_cuda and torch.cuda.is_current_stream_capturing():
                return None
            weight = torch.cat([layer.weight.data for layer in layers])
            scales = torch.cat([layer.scales for layer in layers])
            bias = None
            if any(layer.bias is not None for layer in layers):
                bias = torch.cat([layer.bias.data if layer.bias is not None
                                  else torch.zeros(layer.out_features, dtype=torch.float32, device=weight.device) for layer in layers])
            hit = cache[names] = (key, weight, bias, scales)
        return hit[1], hit[2], hit[3]

    def _can_fuse_projections(self, names, mm_out_dtype, non_mm_precision, attn_type):
        layers = [getattr(self, n) for n in names]
        k_in = layers[0].in_features
        return (self.fuse_projections and self.fuse_prologue and attn_type == "q8_kernels" and self.head_dim == 64
                and mm_out_dtype == torch.bfloat16 and non_mm_precision == torch.bfloat16 and not torch.is_grad_enabled()
                and all(type(layer) is Q8Linear and layer.in_features == k_in and layer.out_features == self.inner_dim for layer in layers)
                and (self.inner_dim in (64, 128, 256) or (self.inner_dim % 512 == 0 and self.inner_dim <= 4096))
                and len(layers) * self.inner_dim * k_in < 2 ** 32)

    def _norm_weight(self, norm):
        if norm.weight is not None:
            return norm.weight
        return torch.ones(self.inner_dim, dtype=torch.float32, device=self.to_q.weight.device)

    def _split_heads(self, t, batch):
        return t.view(batch, -1, self.num_heads, self.head_dim).transpose(1, 2)

    def _project_out(self, hidden_states, mm_out_dtype, non_mm_precision, residual, gate=None):
        if residual is None:
            return self.to_out(hidden_states, out_dtype=mm_out_dtype).to(non_mm_precision)
        if (self.fuse_prologue and mm_out_dtype == torch.bfloat16 and non_mm_precision == torch.bfloat16
                and residual.dtype == torch.bfloat16 and hidden_states.is_cuda
                and (gate is None or gate.dtype == torch.bfloat16)):
            return self.to_out(hidden_states, out_dtype=mm_out_dtype, residual=residual.contiguous(), gate=gate)
        out = self.to_out(hidden_states, out_dtype=mm_out_dtype).to(non_mm_precision)
        if gate is None:
            return out + residual
        if (out.is_cuda and out.dtype == torch.bfloat16 and residual.dtype == torch.bfloat16 and gate.dtype == torch.bfloat16
                and not (torch.is_grad_enabled() and any(t.requires_grad for t in (out, gate, residual)))):
            # one rounding, like the epilogue form: fma(out, gate, residual) on the fused multiply-add kernel
            return Q8F.fma.multiply_add(out.reshape(residual.shape), gate, residual.contiguous(), 0.0)
        return out * gate + residual

    def forward(self, hidden_states, freqs_cis=None, encoder_hidden_states=None, attention_mask=None,
                non_mm_precision=torch.bfloat16, mm_out_dtype=None, apply_qk_hadamard=True, attn_type="torch",
                residual=None, gate=None):
        """hidden_states: the activations, or (for self-attention) a tuple (int8 codes, row scales) of their
        Hadamard-rotated quantization, which is what the q / k / v projections consume.
        residual (optional, the output's shape): the result is residual + attention(...), as the blocks compute it
        (q8_kernels/blocks/ltx_transformer_block.py:41-51); with bfloat16 everywhere the addition happens in the
        epilogue of the output projection. gate (optional, with residual, [B, 1, dim]): attention(...) * gate + residual, the
        gated residual of the AdaLN block (ltx_transformer_block.py:44), one fused multiply-add in that epilogue."""
        if attention_mask is not None and attention_mask.ndim > 1 and attn_type == "q8_kernels":
            # [B, Skv] 0/1 mask -> valid lengths, the reference's rule (first zero; an all-ones row gives 0)
            attention_mask = attention_mask.argmin(-1).squeeze().int()

        kv_src = hidden_states if encoder_hidden_states is None else encoder_hidden_states

        def project(layers, x):
            """[layer(x) for layer in layers]; x is rotated and int8-quantized once for all of them (every Q8Linear
            would do exactly that to the same x on its own)."""
            if isinstance(x, tuple):  # already (int8 codes, row scales)
                return [layer(x[0], x[1], out_dtype=mm_out_dtype) for layer in layers]
            if (self.fuse_prologue and len(layers) > 1 and x.is_cuda and Q8F.fused.can_fuse_hadamard_quantize(x)
                    and not (torch.is_grad_enabled() and x.requires_grad)):  # the shared codes carry no gradient
                xq, xs = Q8F.fused.hadamard_quantize(x)
                return [layer(xq, xs, out_dtype=mm_out_dtype) for layer in layers]
            return [layer(x, out_dtype=mm_out_dtype) for layer in layers]

        v_codes = None
        if encoder_hidden_states is None:
            value = None
            x = hidden_states
            k_in = self.to_v.in_features
            if (self.fuse_prologue and self.cast_v_in_gemm and attn_type == "q8_kernels" and self.head_dim == 64 and type(self.to_v) is Q8Linear
                    and mm_out_dtype == torch.bfloat16 and non_mm_precision == torch.bfloat16
                    and (self.inner_dim in (64, 128, 256) or (self.inner_dim % 512 == 0 and self.inner_dim <= 4096))
                    and k_in > 256 and k_in % 128 == 0 and not torch.is_grad_enabled()):
                # self-attention on the fused path: the V projection's GEMM writes the attention kernel's e4m3 operand itself
                # (the bf16-rounded result, cast, token-major per head), so V never exists as a bfloat16 tensor
                if not isinstance(x, tuple) and x.is_cuda and x.dim() == 3 and Q8F.fused.can_fuse_hadamard_quantize(x):
                    x = Q8F.fused.hadamard_quantize(x)
                # (and the operand sizes the persistent GEMM addresses with 32-bit offsets; larger ones take the plain projection)
                if (isinstance(x, tuple) and x[0].dim() == 3 and x[0].dtype == torch.int8
                        and x[0].numel() < 2 ** 32 and self.to_v.weight.numel() < 2 ** 32):
                    if (self._can_fuse_projections(("to_q", "to_k", "to_v"), mm_out_dtype, non_mm_precision, attn_type)
                            and (2 * self.inner_dim) % 256 == 0):
                        # one GEMM over [Wq; Wk; Wv]: Q and K come back as the two halves of one bfloat16 tensor (read in place
                        # by the prologue), the V columns as e4m3 codes
                        fused = self._fused_weights_of(("to_q", "to_k", "to_v"))
                    else:
                        fused = None
                    if fused is not None:
                        qk, v_codes = _C.mm_bias_qkv(x[0].reshape(-1, k_in), fused[0], fused[1], x[1].reshape(-1), fused[2], x[0].shape[1],
                                                     2 * self.inner_dim)
                        query, key = qk[..., :self.inner_dim], qk[..., self.inner_dim:]
                    else:
                        query, key = project([self.to_q, self.to_k], x)
                        v_codes = _C.mm_bias_qkv(x[0].reshape(-1, k_in), self.to_v.weight.data, self.to_v._bias(), x[1].reshape(-1),
                                                 self.to_v.scales, x[0].shape[1], 0)[1]
            if v_codes is None:
                query, key, value = project([self.to_q, self.to_k, self.to_v], x)
        else:
            (query,) = project([self.to_q], hidden_states)
            kv = None
            if self._can_fuse_projections(("to_k", "to_v"), mm_out_dtype, non_mm_precision, attn_type):
                xkv = kv_src
                if not isinstance(xkv, tuple) and xkv.is_cuda and xkv.dim() == 3 and Q8F.fused.can_fuse_hadamard_quantize(xkv):
                    xkv = Q8F.fused.hadamard_quantize(xkv)
                if isinstance(xkv, tuple) and xkv[0].dim() == 3 and xkv[0].dtype == torch.int8:
                    kv_src = xkv  # (should the separate layers run after all, they take these codes)
                    fused = self._fused_weights_of(("to_k", "to_v"))
                    if fused is not None:
                        # one GEMM over [Wk; Wv]: K and V are the two halves of one tensor, read in place by the prologue
                        kv = Q8F.linear.q8_linear(xkv[0], fused[0], fused[1], xkv[1], fused[2], False, mm_out_dtype)
                        kv = kv.reshape(xkv[0].shape[0], xkv[0].shape[1], 2 * self.inner_dim)
                        key, value = kv[..., :self.inner_dim], kv[..., self.inner_dim:]
            if kv is None:
                key, value = project([self.to_k, self.to_v], kv_src)
        rope = encoder_hidden_states is None and self.use_rope
        batch = query.shape[0]
        if (self.fuse_prologue and attn_type == "q8_kernels" and self.head_dim == 64
                and (self.inner_dim in (64, 128, 256) or (self.inner_dim % 512 == 0 and self.inner_dim <= 4096))
                and non_mm_precision == torch.bfloat16 and query.dim() == 3
                and all(t.dtype == torch.bfloat16 for t in (query, key, value) if t is not None)
                and not (torch.is_grad_enabled() and any(t.requires_grad for t in (query, key, value) if t is not None))):
            # qk-RMSNorm, RoPE, head split, Hadamard and the e4m3 cast in one prologue kernel, head-merged attention
            # output: the same bits as the sequence below
            hidden_states = Q8F.fused.flash_attn_token_major(
                query, key, value, self.num_heads, batch_mask=attention_mask, apply_qk_hadamard=apply_qk_hadamard,
                freqs_cis=freqs_cis if rope else None,
                q_norm_weight=self._norm_weight(self.q_norm) if self.qk_rms_norm else None,
                k_norm_weight=self._norm_weight(self.k_norm) if self.qk_rms_norm else None, v_codes=v_codes)
            return self._project_out(hidden_states, mm_out_dtype, non_mm_precision, residual, gate)
        assert v_codes is None, "the V codes are only produced for the fused path"
        if self.qk_rms_norm:
            query = self.q_norm(query, non_mm_precision)
            key = self.k_norm(key, non_mm_precision)
        if rope:
            query = Q8F.rope.apply_rope(query, freqs_cis[0], freqs_cis[1], out_type=non_mm_precision)
            key = Q8F.rope.apply_rope(key, freqs_cis[0], freqs_cis[1], out_type=non_mm_precision)

        query, key, value = (self._split_heads(t, batch) for t in (query, key, value))

        if attn_type == "q8_kernels":
            hidden_states = Q8F.flash_attention.flash_attn_func(query, key, value, batch_mask=attention_mask,
                                                                apply_qk_hadamard=apply_qk_hadamard)
        elif attn_type == "torch":
            query, key, value = (t.to(non_mm_precision) for t in (query, key, value))
            if attention_mask is not None:
                # [batch] valid lengths -> additive [batch, heads, 1, keys] mask
                pos = torch.arange(key.shape[2], device=query.device).expand(batch, -1)
                add = torch.where(pos < attention_mask.unsqueeze(-1), 0.0, float("-inf"))
                attention_mask = add[:, None, None, :].expand(-1, self.num_heads, -1, -1).to(query.dtype)
            hidden_states = torch.nn.functional.scaled_dot_product_attention(
                query, key, value, attn_mask=attention_mask, dropout_p=0.0, is_causal=False)
        else:
            raise ValueError(f"Invalid attention type: {attn_type}")

        hidden_states = hidden_states.transpose(1, 2).reshape(batch, -1, self.inner_dim).contiguous()
        return self._project_out(hidden_states, mm_out_dtype, non_mm_precision, residual, gate)
