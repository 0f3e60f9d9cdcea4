"""Writes tests/golden/q8_golden.npz: small seeded inputs with the outputs of the CPU oracle, plus tables that
come from closed forms (scipy's Hadamard matrix, the e4m3 bit layout, exact integer products). The reference ships
no test vectors of its own; these fixtures freeze the oracle so that a later edit of it cannot pass unnoticed, and
give the GPU tests inputs whose expected outputs do not depend on code that runs at test time.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import scipy.linalg
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import q8_oracle as O  # noqa: E402

E4M3 = torch.float8_e4m3fn


def u8(t):
    return t.view(torch.uint8).numpy()


def bf16_bits(t):
    return t.view(torch.int16).numpy()


def main():
    g = torch.Generator().manual_seed(20240607)
    out = {}
    out["e4m3_table"] = O.e4m3_decode_table()
    # quantizer
    x = (torch.randn(6, 64, generator=g) * 2.5).to(torch.bfloat16)
    x[3] = 0
    out["quant_x_bf16"] = bf16_bits(x)
    for name, kw in (("i8", dict(out_type=torch.int8)), ("i8_rne", dict(out_type=torch.int8, round_half_even=True)),
                     ("e4m3", dict(out_type=E4M3))):
        c, s = O.ref_quant(x, **kw)
        out["quant_%s_codes" % name] = u8(c) if c.dtype == E4M3 else c.numpy()
        out["quant_%s_scales" % name] = s.numpy()
    # FHT: closed form on small integers is exact
    xi = torch.randint(-4, 5, (4, 128), generator=g).to(torch.bfloat16)
    out["fht_x_bf16"] = bf16_bits(xi)
    out["fht_closed_form"] = xi.double().numpy() @ scipy.linalg.hadamard(128)
    out["fht_oracle_bf16"] = bf16_bits(O.ref_fht(xi, 1.0, torch.bfloat16))
    xr = torch.randn(3, 2048, generator=g).to(torch.bfloat16)
    out["fht2048_x_bf16"] = bf16_bits(xr)
    out["fht2048_oracle_bf16"] = bf16_bits(O.ref_fht(xr))
    out["fht2048_oracle_e4m3"] = u8(O.ref_fht(xr, None, E4M3))
    # int8 GEMM: exact
    a = torch.randint(-128, 128, (40, 96), generator=g, dtype=torch.int8)
    b = torch.randint(-128, 128, (24, 96), generator=g, dtype=torch.int8)
    out["gemm_a_i8"], out["gemm_b_i8"] = a.numpy(), b.numpy()
    out["gemm_acc_i32"] = (a.numpy().astype(np.int64) @ b.numpy().astype(np.int64).T).astype(np.int32)
    sa, sb, bias = torch.rand(40, generator=g) * 1e-2, torch.rand(24, generator=g) * 1e-2, torch.randn(24, generator=g)
    out["gemm_sa"], out["gemm_sb"], out["gemm_bias"] = sa.numpy(), sb.numpy(), bias.numpy()
    out["gemm_out_gelu_bf16"] = bf16_bits(O.ref_q8_mm(a, b, bias, sa, sb, True, torch.bfloat16)[0])
    out["gemm_out_e4m3"] = u8(O.ref_q8_mm(a, b, bias, sa, sb, False, None)[0])
    # attention
    q = O.e4m3_c10(torch.randn(1, 2, 40, 64, generator=g))
    k = O.e4m3_c10(torch.randn(1, 2, 72, 64, generator=g))
    v = O.e4m3_c10(torch.randn(1, 2, 72, 64, generator=g))
    lens = torch.tensor([50], dtype=torch.int32)
    out["attn_q"], out["attn_k"], out["attn_v"], out["attn_len"] = u8(q), u8(k), u8(v), lens.numpy()
    out["attn_exact_f64"] = O.ref_attention(q, k, v, 0.125, lens, round_p=False).numpy()
    out["attn_rounded_f64"] = O.ref_attention(q, k, v, 0.125, lens, round_p=True, p_scale=256.0).numpy()
    out["attn_rounded_unit_f64"] = O.ref_attention(q, k, v, 0.125, lens, round_p=True, p_scale=1.0).numpy()
    # RMSNorm / RoPE
    xn = torch.randn(5, 64, generator=g).to(torch.bfloat16)
    w = torch.rand(64, generator=g) + 0.5
    y, r = O.ref_rms_norm(xn, w)
    out["rms_x_bf16"], out["rms_w"], out["rms_y_bf16"], out["rms_rstd"] = bf16_bits(xn), w.numpy(), bf16_bits(y), r.numpy()
    cos, sin = torch.randn(5, 64, generator=g), torch.randn(5, 64, generator=g)
    out["rope_cos"], out["rope_sin"], out["rope_y_bf16"] = cos.numpy(), sin.numpy(), bf16_bits(O.ref_rope(xn, cos, sin))
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "q8_golden.npz"), **out)
    print("wrote q8_golden.npz with %d arrays" % len(out))


if __name__ == "__main__":
    main()
