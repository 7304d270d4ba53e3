"""Pins the C oracle's fp8 e4m3fn arithmetic without the GPU.

The encoder is checked against PyTorch's own float8_e4m3fn cast (an independent software
implementation of the same OCP format), the decoder against the format's closed form, and
the quantiser against the special cases the reference's convention fixes."""
import math

import numpy as np
import torch

import oracle


def test_decode_table_is_the_format_closed_form():
    table = oracle.fp8_decode_table()
    for c in range(256):
        s, e, m = c >> 7, (c >> 3) & 15, c & 7
        if e == 15 and m == 7:
            assert math.isnan(table[c])
            continue
        val = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        assert table[c].item() == (-val if s else val)
    assert table[0x7e].item() == 448.0 and table[0x08].item() == 2.0 ** -6 and table[0x01].item() == 2.0 ** -9
    torch_table = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    finite = ~torch.isnan(torch_table)
    assert torch.equal(table[finite], torch_table[finite])


def test_encode_matches_torch_cast_on_all_bf16_patterns_and_random_fp32():
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16).float()
    x = x[torch.isfinite(x)]
    g = torch.Generator().manual_seed(0)
    r = torch.randn(50000, generator=g) * torch.exp(torch.randn(50000, generator=g) * 4)
    # dense sweep across the subnormal / normal boundary and the saturation edge
    edge = torch.cat([torch.linspace(0, 2.0 ** -5, 20001), torch.linspace(400, 480, 8001)])
    allx = torch.cat([x, r, edge, -edge])
    ours = oracle.fp8_encode(allx)
    theirs = allx.to(torch.float8_e4m3fn).view(torch.uint8)
    # torch maps every |x| > 464 (and NaN) to the NaN code with the sign kept, as we do
    assert torch.equal(ours, theirs)


def test_encode_special_cases():
    enc = lambda v: oracle.c_lib().oracle_f32_to_e4m3fn(v)
    assert enc(0.0) == 0x00 and enc(-0.0) == 0x80
    assert enc(448.0) == 0x7e and enc(-448.0) == 0xfe
    assert enc(2.0 ** -9) == 0x01 and enc(2.0 ** -10) == 0x00          # tie to even (0)
    assert enc(3 * 2.0 ** -10) == 0x02                                  # tie to even (2)
    assert enc(np.nextafter(np.float32(2.0 ** -10), np.float32(1))) == 0x01
    assert enc(2.0 ** -6) == 0x08 and enc(0.9999 * 2.0 ** -6) == 0x08  # rounds up into the normals
    assert enc(464.0) == 0x7e and enc(465.0) == 0x7f                   # tie to even, then no finite code
    assert enc(1.0) == 0x38 and enc(1.0625) == 0x38 and enc(1.1875) == 0x3a  # ties to even mantissa


def test_quantiser_follows_reference_convention():
    # x * (1.0f / scale), clamp to +-448, cast (kernels/cuda/fp8_quant.cu:92-103, fp8_quant_utils.cuh:111-130)
    lib = oracle.c_lib()
    q = lambda v, s: lib.oracle_fp8_quantize(v, np.float32(1.0) / np.float32(s))
    assert q(1e9, 1.0) == 0x7e and q(-1e9, 1.0) == 0xfe                # saturate finite
    assert q(float("inf"), 1.0) == 0x7e
    assert q(float("nan"), 1.0) == 0x7e                                # fminf/fmaxf drop the NaN
    assert q(0.0, 0.5) == 0x00
    assert q(3.0, 3.0 / 448.0) in (0x7e,)                              # absmax maps to the top code
    # reciprocal-then-multiply, not divide: 7 * (1/7f) rounds below 1 in fp32 while 7/7 == 1
    x, s = np.float32(7.0), np.float32(7.0)
    assert np.float32(x * (np.float32(1.0) / s)) == np.float32(1.0)  # sanity of the example itself
    # the ATen form of the same convention agrees on finite inputs
    g = torch.Generator().manual_seed(1)
    xs = (torch.randn(64, 4, 128, generator=g) * 3).to(torch.bfloat16)
    scale = oracle.kv_head_scales(xs)
    ref = oracle.aten_fp8_quantize(xs, scale)
    kc = torch.zeros(4, 16, 4, 128, dtype=torch.uint8)
    oracle.reshape_and_cache(xs, None, kc, None, torch.arange(64, dtype=torch.int32), scale, None)
    assert torch.equal(kc.view(64, 4, 128), ref)


def test_head_scales_closed_form():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(33, 3, 64, generator=g).to(torch.bfloat16)
    x[:, 1] = 0
    s = oracle.kv_head_scales(x)
    expect = (x.float().abs().amax(dim=(0, 2)) / 448.0).clamp_min(1e-12)
    assert torch.equal(s, expect) and s[1].item() == np.float32(1e-12)
