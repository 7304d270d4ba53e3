"""The CPU oracles reproduce the committed fixtures of tests/golden/ (written by tests/golden/make_fixtures.py from
the same oracles): a guard on the CHECKERS against drift of libtorch or libm between boxes.  Bit-exact for bytes and
integer work; the attention outputs within one bf16 step (ATen-order oracle) and 1e-6 (fp64 oracle)."""
import hashlib
import json
import math
import os

import numpy as np
import torch

import oracle
from helpers import fill_caches_cpu
from xllm_amd import workloads

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def sha(t):
    return hashlib.sha256(t.contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()


def test_fp8_table_and_encoder_digest():
    fx = json.load(open(os.path.join(GOLDEN, "fp8_e4m3fn_table.json")))
    table = oracle.fp8_decode_table()
    assert table.view(torch.int32).tolist() == fx["decode_table_f32_bits"]
    # spot values of the format itself, so that the fixture cannot drift together with the oracle
    want = {0x00: 0.0, 0x38: 1.0, 0x7e: 448.0, 0xb8: -1.0, 0x01: 2.0 ** -9, 0x08: 2.0 ** -6}
    got = torch.tensor(fx["decode_table_f32_bits"], dtype=torch.int32).view(torch.float32)
    for code, value in want.items():
        assert got[code].item() == value
    assert math.isnan(got[0x7f].item()) and math.isnan(got[0xff].item())
    every_bf16 = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    assert sha(oracle.fp8_encode(every_bf16)) == fx["encode_all_bf16_sha256"]


def test_merge_known_answers_from_the_fixture():
    fx = json.load(open(os.path.join(GOLDEN, "dcp_attention_merge.json")))
    log = lambda x: torch.tensor(x, dtype=torch.float64).log().float()   # exp(lse) = 0 stands for lse = -inf
    for case in fx["cases"]:
        o = torch.tensor(case["partial_out"], dtype=torch.float32)
        l = log(case["partial_lse_exp"])
        for merge in (oracle.lse_merge, lambda a, b: tuple(t.float() for t in oracle.aten_lse_merge(a, b))):
            out, lse = merge(o, l)
            assert torch.allclose(out, torch.tensor(case["out"]), atol=1e-6)
            want = log(case["lse_exp"])
            assert torch.equal(torch.isneginf(lse), torch.isneginf(want))
            fin = ~torch.isneginf(want)
            assert torch.allclose(lse[fin], want[fin], atol=1e-6)


def bf16_steps_apart(a_bits, b_bits):
    """Distance in representable bf16 values between two arrays of bit patterns (same sign assumed where it counts)."""
    key = lambda x: np.where(x < 0, -(x.astype(np.int32) & 0x7fff), x.astype(np.int32))
    return np.abs(key(a_bits) - key(b_bits))


def test_tiny_configuration_against_the_fixture():
    fx = np.load(os.path.join(GOLDEN, "tiny_decode.npz"), allow_pickle=False)
    cfg = workloads.CONFIGS["tiny"]
    inp = workloads.make_inputs(cfg, int(fx["seed"]))
    lay = inp.layout
    digest = hashlib.sha256()
    for t in (lay.seq_lens, lay.block_table, lay.new_slots, inp.q, inp.k_ctx, inp.v_ctx, inp.k_new, inp.v_new):
        digest.update(t.contiguous().view(torch.uint8).numpy().tobytes())
    assert digest.hexdigest() == str(fx["inputs_sha256"]), \
        "the seeded input generator (torch's CPU generator) gives other bytes on this box: the fixture does not apply"
    assert np.array_equal(lay.seq_lens.numpy(), fx["seq_lens"])
    kc, vc = fill_caches_cpu(inp)
    assert sha(kc) == str(fx["k_cache_sha256"]) and sha(vc) == str(fx["v_cache_sha256"])
    aten = oracle.aten_paged_decode(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale)
    steps = bf16_steps_apart(aten.contiguous().view(torch.int16).numpy(), fx["aten_out_bf16_bits"])
    assert steps.max() <= 1, f"the ATen-order oracle moved by {steps.max()} bf16 steps on this box"
    f64 = oracle.paged_decode_f64(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale)
    f64 = f64[0] if isinstance(f64, tuple) else f64
    assert np.abs(f64.float().numpy() - fx["f64_out_f32"]).max() <= 1e-6
    # fp8 pages
    ks = oracle.kv_head_scales(torch.cat([inp.k_ctx, inp.k_new]))
    vs = oracle.kv_head_scales(torch.cat([inp.v_ctx, inp.v_new]))
    assert np.array_equal(ks.numpy(), fx["fp8_k_scale"]) and np.array_equal(vs.numpy(), fx["fp8_v_scale"])
    kq, vq = fill_caches_cpu(inp, cache_dtype=torch.float8_e4m3fn, k_scale=ks, v_scale=vs)
    assert sha(kq) == str(fx["fp8_k_cache_sha256"]) and sha(vq) == str(fx["fp8_v_cache_sha256"])
    aten8 = oracle.aten_paged_decode(inp.q, kq.view(torch.float8_e4m3fn), vq.view(torch.float8_e4m3fn), lay.block_table,
                                     lay.seq_lens, cfg.scale, ks, vs)
    steps = bf16_steps_apart(aten8.contiguous().view(torch.int16).numpy(), fx["fp8_aten_out_bf16_bits"])
    assert steps.max() <= 1
