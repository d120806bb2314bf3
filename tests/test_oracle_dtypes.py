"""Pins the oracle's storage roundings (bf16 / fp16, round to nearest even)
against libtorch's casts, exhaustively where the domain is small."""
import ctypes

import numpy as np
import torch


def _all_u16():
    return torch.arange(65536, dtype=torch.int32).to(torch.int16)


def test_bf16_widen_exhaustive(oracle):
    lib = oracle.lib()
    bits = _all_u16()
    ref = bits.view(torch.bfloat16).float()
    got = torch.tensor([lib.eko_bf16_to_f32(int(b) & 0xffff) for b in bits.tolist()])
    assert torch.equal(torch.isnan(ref), torch.isnan(got))
    ok = ~torch.isnan(ref)
    assert torch.equal(ref[ok].view(torch.int32), got[ok].view(torch.int32))


def test_f16_widen_exhaustive(oracle):
    lib = oracle.lib()
    bits = _all_u16()
    ref = bits.view(torch.float16).float()
    got = torch.tensor([lib.eko_f16_to_f32(int(b) & 0xffff) for b in bits.tolist()])
    ok = ~torch.isnan(ref)
    assert torch.equal(torch.isnan(ref), torch.isnan(got))
    assert torch.equal(ref[ok].view(torch.int32), got[ok].view(torch.int32))


def _probe_floats():
    g = torch.Generator().manual_seed(7)
    rnd = torch.randn(20000, generator=g) * torch.exp(torch.randn(20000, generator=g) * 6)
    # every 16-bit value, its neighbours and the exact midpoints between neighbours (ties)
    b16 = _all_u16().view(torch.bfloat16).float()
    f16 = _all_u16().view(torch.float16).float()
    parts = [rnd, b16, f16]
    for base in (b16, f16):
        fin = base[torch.isfinite(base)]
        srt = torch.sort(fin).values
        mid = ((srt[1:].double() + srt[:-1].double()) / 2).float()
        parts += [mid, torch.nextafter(mid, torch.tensor(float("inf"))), torch.nextafter(mid, torch.tensor(-float("inf")))]
    parts.append(torch.tensor([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 3e38, -3e38]))
    v = torch.cat(parts)
    return v[torch.isfinite(v)]


def test_narrowing_matches_libtorch(oracle):
    lib = oracle.lib()
    v = _probe_floats()
    ref_b = v.to(torch.bfloat16).view(torch.int16).to(torch.int32) & 0xffff
    ref_h = v.to(torch.float16).view(torch.int16).to(torch.int32) & 0xffff
    vals = v.tolist()
    got_b = torch.tensor([lib.eko_f32_to_bf16(x) for x in vals], dtype=torch.int32)
    got_h = torch.tensor([lib.eko_f32_to_f16(x) for x in vals], dtype=torch.int32)
    assert torch.equal(ref_b, got_b)
    assert torch.equal(ref_h, got_h)


def test_narrowing_nan(oracle):
    lib = oracle.lib()
    assert np.isnan(lib.eko_bf16_to_f32(lib.eko_f32_to_bf16(float("nan"))))
    assert np.isnan(lib.eko_f16_to_f32(lib.eko_f32_to_f16(float("nan"))))


def test_fp8_e4m3fn_exhaustive(oracle):
    """All 256 encodings: against libtorch's float8_e4m3fn widening (bit for bit, NaNs as NaNs)
    and against facts of the format that a wrong bias, a missing subnormal branch or an
    infinity would break: max finite 448, smallest subnormal 2^-9, 0x38 = 1, sign symmetry,
    monotone over the positive finite codes."""
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    got = oracle.fp8_e4m3fn_to_f32(codes)
    ref = codes.view(torch.float8_e4m3fn).float()
    nan = torch.isnan(ref)
    assert nan.tolist() == [(c & 0x7f) == 0x7f for c in range(256)] and torch.equal(torch.isnan(got), nan)
    assert torch.equal(got[~nan].view(torch.int32), ref[~nan].view(torch.int32))          # signed zeros included
    assert float(got[0x7e]) == 448.0 and float(got[0x01]) == 2.0 ** -9 and float(got[0x38]) == 1.0
    assert float(got[0x08]) == 2.0 ** -6 and float(got[0x07]) == 7 * 2.0 ** -9              # first normal, last subnormal
    pos = got[:0x7f]
    assert bool((pos[1:] > pos[:-1]).all()) and not bool(torch.isinf(got).any())
    assert torch.equal(got[0x80:0xff], -got[:0x7f])
