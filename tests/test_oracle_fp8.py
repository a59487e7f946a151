"""Pins oracle/fp8.py: e4m3fn table, the software encoder and the per-row quantiser (CPU only)."""

import numpy as np
import torch

from oracle import fp8


def test_table_matches_torch_decode_of_all_256_codes():
    codes = torch.arange(256, dtype=torch.uint8)
    via_torch = codes.view(torch.float8_e4m3fn).float().numpy()
    table = fp8.e4m3fn_table()
    assert np.array_equal(np.isnan(table), np.isnan(via_torch))
    ok = ~np.isnan(table)
    assert np.array_equal(table[ok], via_torch[ok])
    # spot values straight from the format definition
    assert table[0x7E] == 448.0 and table[0xFE] == -448.0  # max finite
    assert table[0x01] == 2.0**-9 and table[0x08] == 2.0**-6  # min subnormal / min normal
    assert table[0x38] == 1.0 and np.isnan(table[0x7F]) and np.isnan(table[0xFF])
    assert np.signbit(table[0x80]) and table[0x80] == 0.0  # negative zero


def test_every_code_is_a_bf16_value():
    t = torch.from_numpy(fp8.e4m3fn_table())
    ok = ~torch.isnan(t)
    assert torch.equal(t[ok].to(torch.bfloat16).float(), t[ok])


def test_software_encoder_matches_torch_cast():
    g = torch.Generator().manual_seed(1)
    x = torch.cat(
        [
            torch.randn(20000, generator=g) * 100.0,
            torch.randn(20000, generator=g) * 0.01,
            torch.linspace(-448.0, 448.0, 7001),
            torch.tensor([0.0, -0.0, 2.0**-10, 2.0**-9, 1.5 * 2.0**-9, 447.9, 448.0, -448.0]),
        ]
    ).float()
    x = x[x.abs() <= 448.0]
    ours = fp8.encode_e4m3fn_rne(x)
    theirs = x.to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(ours, theirs)


def test_software_encoder_ties_to_even():
    # exact midpoints between neighbouring codes must land on the even mantissa
    table = torch.from_numpy(fp8.e4m3fn_table())
    pos = table[:0x7F]  # 0 .. 448 ascending
    mids = (pos[:-1].double() + pos[1:].double()) / 2
    enc = fp8.encode_e4m3fn_rne(mids.float())
    lo = torch.arange(0, 0x7E)
    expect = torch.where(lo % 2 == 0, lo, lo + 1).to(torch.uint8)
    assert torch.equal(enc, expect)
    assert torch.equal(mids.float().to(torch.float8_e4m3fn).view(torch.uint8), expect)


def test_quantiser_invariants():
    g = torch.Generator().manual_seed(0)
    w = torch.randn(96, 720, generator=g) * 0.02
    w[7] = 0.0  # an all-zero row exercises the 1e-12 clamp
    w8, s = fp8.quantize_weight_rows(w)
    assert w8.dtype == torch.float8_e4m3fn and s.dtype == torch.float32 and s.shape == (96,)
    assert float(s[7]) == np.float32(1e-12) and torch.all(w8[7].float() == 0)
    amax = w.abs().amax(dim=1)
    live = amax > 0
    assert torch.equal(s[live], (amax / 448.0)[live])
    # the row maximum maps onto +-448 exactly and nothing saturates
    assert torch.all(w8.float().abs().amax(dim=1)[live] == 448.0)
    assert not torch.isnan(w8.float()).any()
    # codes equal the independent encoder applied to W/scale
    assert torch.equal(w8.view(torch.uint8), fp8.encode_e4m3fn_rne(w / s[:, None]))
    # re-quantising the dequantised weight with the stored scale is byte-exact
    deq = fp8.dequantize_rows(w8, s)
    again = (deq / s[:, None]).to(torch.float8_e4m3fn)
    assert torch.equal(again.view(torch.uint8), w8.view(torch.uint8))
    # error bound of docs/fastWAM_weight_quantization.md:26-30: half a ULP of the top binade
    rel = ((deq - w).abs().amax(dim=1) / amax.clamp_min(1e-30))[live]
    assert float(rel.max()) <= 16.0 / 448.0 + 1e-6


def test_decode_helper_uses_table():
    codes = torch.tensor([0x38, 0xB8, 0x7E, 0x00], dtype=torch.uint8)
    assert fp8.decode_e4m3fn(codes).tolist() == [1.0, -1.0, 448.0, 0.0]
