"""Pins oracle/mlp.py (the arithmetic) without any reference output:
row independence (split == unsplit), a float64 closed form, the independent
plain-C restatement, and torch's own float8 conversion for the e4m3 codec."""
import numpy as np
import pytest
import torch

from oracle import cref, mlp


def u16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def from_u16(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def test_split_equals_unsplit_fp32():
    x, wg, wu, wd = mlp.make_inputs(256, 1024, 2816)
    whole = mlp.mlp_unsplit(x, wg, wu, wd)
    for split in ([0, 128, 256], [0, 13, 256], [0, 64, 128, 192, 256]):
        parts = mlp.mlp_schedule(x, wg, wu, wd, split)
        rel = (parts - whole).abs().max() / whole.abs().max()
        assert rel < 1e-6, rel  # row-wise independent up to GEMM blocking effects


def test_fp32_layer_against_float64_closed_form():
    x, wg, wu, wd = mlp.make_inputs(64, 256, 704)
    xd, wgd, wud, wdd = (t.double() for t in (x, wg, wu, wd))
    g = xd @ wgd.t()
    want = ((g / (1 + torch.exp(-g))) * (xd @ wud.t())) @ wdd.t()
    got = mlp.mlp_unsplit(x, wg, wu, wd)
    assert ((got.double() - want).abs().max() / want.abs().max()) < 1e-5


def test_gemm_against_c_restatement():
    x, wg, _, _ = mlp.make_inputs(48, 128, 96)
    c = cref.gemm_nt_f32(x.numpy(), wg.numpy())
    t = torch.nn.functional.linear(x, wg).numpy()
    assert np.abs(c - t).max() / np.abs(c).max() < 1e-6
    # transposed-operand mistake would change the shape; a dropped term or wrong index the values
    xb, wb = x.bfloat16(), wg.bfloat16()
    cb = from_u16(cref.gemm_nt_bf16(u16(xb), u16(wb)))
    tb = torch.nn.functional.linear(xb.float(), wb.float()).bfloat16()
    assert (cb.float() - tb.float()).abs().max() <= 2 ** -7 * tb.float().abs().max()


def test_silu_mul_exact_is_bit_equal_to_c_up_to_exp_rounding():
    g = torch.randn(64, 256).mul(4).bfloat16()
    u = torch.randn(64, 256).bfloat16()
    want = from_u16(cref.silu_mul_bf16(u16(g), u16(u), round_silu=False))
    got = mlp.silu_mul_exact(g, u)
    diff = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs()
    assert diff.max() <= 1 and (diff > 0).float().mean() < 0.01
    # special values
    g0 = torch.tensor([[0.0, -0.0, 30.0, -30.0, 1.0, -1.0, 88.0, -88.0]]).bfloat16()
    u0 = torch.ones_like(g0)
    got0 = mlp.silu_mul_exact(g0, u0).float()
    assert got0[0, 0] == 0 and got0[0, 2] == 30.0 and abs(got0[0, 3]) < 1e-11
    assert abs(got0[0, 4] - 0.7310585786) < 4e-3 and abs(got0[0, 5] + 0.2689414214) < 2e-3


def test_silu_mul_eager_rounds_silu_first():
    g = torch.randn(32, 128).mul(3).bfloat16()
    u = torch.randn(32, 128).bfloat16()
    want = from_u16(cref.silu_mul_bf16(u16(g), u16(u), round_silu=True))
    got = mlp.silu_mul_eager(g, u)
    diff = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs()
    assert diff.max() <= 1 and (diff > 0).float().mean() < 0.01


def test_rms_norm_against_c_and_textbook():
    x = torch.randn(16, 512).bfloat16()
    w = (1 + 0.1 * torch.randn(512)).bfloat16()
    got = mlp.rms_norm(x, w, 1e-5)
    want = from_u16(cref.rmsnorm_bf16(u16(x), u16(w), 1e-5))
    diff = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs()
    assert diff.max() <= 1
    text = x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-5) * w.float()
    assert (got.float() - text).abs().max() <= 2 ** -6 * text.abs().max()
    # unit rows: mean of squares 1 -> output == weight (up to eps)
    ones = torch.ones(2, 512).bfloat16()
    assert torch.equal(mlp.rms_norm(ones, w, 0.0), w.expand(2, -1))


def test_e4m3_codec_against_torch_and_format():
    vals = mlp.E4M3_VALUES
    assert vals[0x7E] == 448.0 and vals[0x01] == 2.0 ** -9 and vals[0x08] == 2.0 ** -6 and np.isnan(vals[0x7F])
    # decode == torch's own view of the same bytes
    codes = torch.arange(256, dtype=torch.uint8)
    t = codes.view(torch.float8_e4m3fn).float()
    ok = ~torch.isnan(t)
    assert torch.equal(torch.from_numpy(mlp.e4m3_decode(codes.numpy()))[ok], t[ok])
    # encode == torch's round-to-nearest-even conversion inside the finite range
    x = torch.cat([torch.randn(20000) * 100, torch.linspace(-448, 448, 4097), torch.randn(2000) * 0.01])
    x = x.clamp(-448, 448)
    want = x.to(torch.float8_e4m3fn).view(torch.uint8)
    got = torch.from_numpy(mlp.e4m3_encode(x.numpy()))
    same = (got == want) | ((got & 0x7F == 0) & (want & 0x7F == 0))  # +-0 are the same value
    assert bool(same.all())
    # saturation
    assert list(mlp.e4m3_encode(np.array([1e6, -1e6], dtype=np.float32))) == [0x7E, 0xFE]
    # exact representables round-trip
    finite = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    assert np.array_equal(mlp.e4m3_encode(mlp.e4m3_decode(finite)) & 0x7F, finite & 0x7F)


def test_quant_roundtrip_error_bound():
    x = torch.randn(64, 256).bfloat16()
    q, s = mlp.quant_e4m3(x)
    back = mlp.dequant(q, s)
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 for normal values
    big = x.float().abs() > s.item() * 2 ** -6
    rel = ((back - x.float()).abs() / x.float().abs().clamp_min(1e-30))[big]
    assert rel.max() <= 2 ** -4 + 1e-6
    assert back.abs().max() <= x.float().abs().max() * (1 + 1e-6)
