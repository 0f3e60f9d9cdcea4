"""The committed fixtures (tests/golden/q8_golden.npz, written by tests/golden/make_golden.py) against the oracle
on the CPU and against the HIP kernels on the GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import q8_oracle as O

E4M3 = torch.float8_e4m3fn
G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "q8_golden.npz"))


def bf16(name):
    return torch.from_numpy(G[name].copy()).view(torch.bfloat16)


def e4m3(name):
    return torch.from_numpy(G[name].copy()).view(E4M3)


def test_fixture_closed_forms_agree_with_oracle():
    assert np.array_equal(np.nan_to_num(G["e4m3_table"], nan=-1), np.nan_to_num(O.e4m3_decode_table(), nan=-1))
    x = bf16("fht_x_bf16")
    want = torch.from_numpy(G["fht_closed_form"]).to(torch.float32).to(torch.bfloat16)
    assert torch.equal(O.ref_fht(x, 1.0, torch.bfloat16).view(torch.int16), want.view(torch.int16))
    a, b = torch.from_numpy(G["gemm_a_i8"].copy()), torch.from_numpy(G["gemm_b_i8"].copy())
    assert np.array_equal(O.ref_gemm_i32(a, b).numpy(), G["gemm_acc_i32"])


def test_oracle_reproduces_fixture():
    x = bf16("quant_x_bf16")
    for name, kw in (("i8", dict(out_type=torch.int8)), ("i8_rne", dict(out_type=torch.int8, round_half_even=True)),
                     ("e4m3", dict(out_type=E4M3))):
        c, s = O.ref_quant(x, **kw)
        got = c.view(torch.uint8).numpy() if c.dtype == E4M3 else c.numpy()
        assert np.array_equal(got, G["quant_%s_codes" % name]) and np.array_equal(s.numpy(), G["quant_%s_scales" % name])
    xr = bf16("fht2048_x_bf16")
    assert np.array_equal(O.ref_fht(xr).view(torch.int16).numpy(), G["fht2048_oracle_bf16"])
    assert np.array_equal(O.ref_fht(xr, None, E4M3).view(torch.uint8).numpy(), G["fht2048_oracle_e4m3"])
    q, k, v = e4m3("attn_q"), e4m3("attn_k"), e4m3("attn_v")
    lens = torch.from_numpy(G["attn_len"].copy())
    assert np.allclose(O.ref_attention(q, k, v, 0.125, lens, round_p=False).numpy(), G["attn_exact_f64"], atol=1e-12)
    assert np.allclose(O.ref_attention(q, k, v, 0.125, lens, round_p=True, p_scale=256.0).numpy(), G["attn_rounded_f64"], atol=1e-12)
    assert np.allclose(O.ref_attention(q, k, v, 0.125, lens, round_p=True).numpy(), G["attn_rounded_unit_f64"], atol=1e-12)
    xn = bf16("rms_x_bf16")
    y, r = O.ref_rms_norm(xn, torch.from_numpy(G["rms_w"].copy()))
    assert np.array_equal(y.view(torch.int16).numpy(), G["rms_y_bf16"]) and np.array_equal(r.numpy(), G["rms_rstd"])
    yr = O.ref_rope(xn, torch.from_numpy(G["rope_cos"].copy()), torch.from_numpy(G["rope_sin"].copy()))
    assert np.array_equal(yr.view(torch.int16).numpy(), G["rope_y_bf16"])


@pytest.mark.gpu
def test_hip_kernels_reproduce_fixture(dev):
    from q8_kernels_amd import _C
    x = bf16("quant_x_bf16").to(dev)
    c, s = _C.tokenwise_quant(x)
    assert np.array_equal(c.cpu().numpy(), G["quant_i8_codes"]) and np.array_equal(s.cpu().numpy(), G["quant_i8_scales"])
    c, s = _C.tokenwise_quant(x, None, round_half_even=True)
    assert np.array_equal(c.cpu().numpy(), G["quant_i8_rne_codes"])
    c, s = _C.tokenwise_quant(x, E4M3)
    assert np.array_equal(c.cpu().view(torch.uint8).numpy(), G["quant_e4m3_codes"]) and np.array_equal(s.cpu().numpy(), G["quant_e4m3_scales"])
    y = _C.fast_hadamard_transform(bf16("fht_x_bf16").to(dev), 1.0, None)
    assert np.array_equal(y.cpu().float().numpy().astype(np.float64), G["fht_closed_form"])  # small integers: exact
    xr = bf16("fht2048_x_bf16").to(dev)
    assert np.array_equal(_C.fast_hadamard_transform(xr, 2048 ** -0.5, None).cpu().view(torch.int16).numpy(), G["fht2048_oracle_bf16"])
    assert np.array_equal(_C.fast_hadamard_transform(xr, 2048 ** -0.5, E4M3).cpu().view(torch.uint8).numpy(), G["fht2048_oracle_e4m3"])
    a, b = torch.from_numpy(G["gemm_a_i8"].copy()).to(dev), torch.from_numpy(G["gemm_b_i8"].copy()).to(dev)
    assert np.array_equal(_C.q8_mm_i32(a, b).cpu().numpy(), G["gemm_acc_i32"])
    sa, sb, bias = (torch.from_numpy(G[n].copy()).to(dev) for n in ("gemm_sa", "gemm_sb", "gemm_bias"))
    out = _C.q8_mm_bias(a, b, bias, sa, sb, True, torch.bfloat16)[0].cpu()
    d = np.abs(out.view(torch.int16).numpy().astype(np.int32) - G["gemm_out_gelu_bf16"].astype(np.int32))
    # far in GELU's negative tail the fixture's float64 formula 1 + tanh cancels to -0 while the kernel keeps the tiny
    # value (about -1e-20): those elements are compared absolutely
    want = torch.from_numpy(G["gemm_out_gelu_bf16"].astype(np.int16)).view(torch.bfloat16).float().numpy()
    d[np.abs(out.float().numpy() - want) <= 1e-7] = 0
    assert d.max() <= 2
    out8 = _C.q8_mm_bias(a, b, bias, sa, sb, False, None)[0].cpu().view(torch.uint8).numpy()
    assert (out8 != G["gemm_out_e4m3"]).mean() < 0.02
    q, k, v = e4m3("attn_q"), e4m3("attn_k"), e4m3("attn_v")
    vt = torch.zeros(1, 2, 64, 80, dtype=torch.uint8)
    vt[..., :72] = v.view(torch.uint8).transpose(2, 3)
    o = _C.flash_attention(q.to(dev), k.to(dev), vt.view(E4M3).to(dev), 0.125, torch.from_numpy(G["attn_len"].copy()).to(dev),
                           out_dtype=torch.bfloat16).cpu().double().numpy()
    assert np.abs(o - G["attn_exact_f64"]).max() < 0.05 and np.abs(o - G["attn_rounded_f64"]).max() < 0.05
    xn = bf16("rms_x_bf16").to(dev)
    y, r = _C.rms_norm(xn, torch.from_numpy(G["rms_w"].copy()).to(dev))
    assert np.allclose(r.cpu().numpy(), G["rms_rstd"], rtol=1e-6)
    assert np.abs(y.cpu().view(torch.int16).numpy().astype(np.int32) - G["rms_y_bf16"].astype(np.int32)).max() <= 1
    yr = _C.rope(xn, torch.from_numpy(G["rope_cos"].copy()).to(dev), torch.from_numpy(G["rope_sin"].copy()).to(dev))
    assert np.array_equal(yr.cpu().view(torch.int16).numpy(), G["rope_y_bf16"])
