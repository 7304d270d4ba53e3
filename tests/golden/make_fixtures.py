#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden/ from this build's CPU oracles, in this container.

    python tests/golden/make_fixtures.py

The fixtures guard the CHECKERS, not the GPU path: the oracles are pinned by closed forms and by the reference's
own known answers (tests/test_oracle_*.py), but they are built on libtorch and libm, which differ from image to
image (the scaled-dot-product CPU kernel may change the last bf16 bit between torch versions).  A test on another
box that finds the oracle off these files knows that the checker moved, not the kernels.  What is stored:

  fp8_e4m3fn_table.json      the 256 decoded values of the fp8 e4m3fn codes as float32 bit patterns, and the sha256 of
                             the encoder's 65536-byte answer to every bf16 bit pattern at scale 1
  dcp_attention_merge.json   the three known answers of the reference's DcpAttentionMergeTest
                             (tests/core/layers/mlu/dcp_attention_merge_test.cpp:34-75): inputs and expected outputs
  tiny_decode.npz            configuration 1 (batch 4, 8/8 heads, head dim 128, block 16, contexts 64..512, 256 pages,
                             seed 1234): sha256 of the generated inputs and of the K and V cache bytes after
                             reshape_and_cache, the ATen-order oracle's output (bf16 bit patterns) and the fp64 oracle's
                             output (float32), with bf16 pages and with fp8 pages + per-head scales (cache digests,
                             scales, ATen-order output)
"""
import hashlib
import json
import math
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oracle  # noqa: E402
from xllm_amd import workloads  # noqa: E402

TINY_SEED = 1234


def sha(t):
    return hashlib.sha256(t.contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()


def fp8_fixture():
    table = oracle.fp8_decode_table()                      # [256] float32
    bits = table.view(torch.int32).tolist()
    every_bf16 = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    codes = oracle.fp8_encode(every_bf16)
    return {"decode_table_f32_bits": bits, "encode_all_bf16_sha256": sha(codes),
            "note": "code -> float32 bit pattern (NaN codes 0x7f / 0xff keep their payload); encoder digest over "
                    "bf16 patterns 0x0000..0xffff in order"}


def merge_fixture():
    inf = "-inf"
    return {"source": "tests/core/layers/mlu/dcp_attention_merge_test.cpp:34-75",
            "cases": [
                {"partial_out": [[[[2.0, 4.0]]], [[[6.0, 8.0]]]], "partial_lse_exp": [[[2.0]], [[6.0]]],
                 "out": [[[5.0, 7.0]]], "lse_exp": [[8.0]]},
                {"partial_out": [[[[0.0, 0.0]]], [[[3.0, 9.0]]]], "partial_lse_exp": [[[0.0]], [[4.0]]],
                 "out": [[[3.0, 9.0]]], "lse_exp": [[4.0]]},
                {"partial_out": [[[[1.0, 1.0, 1.0], [1.0, 1.0, 1.0]]], [[[1.0, 1.0, 1.0], [1.0, 1.0, 1.0]]]],
                 "partial_lse_exp": [[[0.0, 0.0]], [[0.0, 0.0]]],
                 "out": [[[0.0, 0.0, 0.0], [0.0, 0.0, 0.0]]], "lse_exp": [[0.0, 0.0]]}],
            "note": "LSEs are stored as exp(lse): 0.0 stands for lse = " + inf}


def tiny_fixture():
    from helpers import fill_caches_cpu
    cfg = workloads.CONFIGS["tiny"]
    inp = workloads.make_inputs(cfg, TINY_SEED)
    lay = inp.layout
    out = {"seed": np.int64(TINY_SEED)}
    digest = hashlib.sha256()
    for t in (lay.seq_lens, lay.block_table, lay.new_slots, inp.q, inp.k_ctx, inp.v_ctx, inp.k_new, inp.v_new):
        digest.update(t.contiguous().view(torch.uint8).numpy().tobytes())
    out["inputs_sha256"] = np.array(digest.hexdigest())
    out["seq_lens"] = lay.seq_lens.numpy()
    kc, vc = fill_caches_cpu(inp)
    out["k_cache_sha256"], out["v_cache_sha256"] = np.array(sha(kc)), np.array(sha(vc))
    aten = oracle.aten_paged_decode(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale)
    out["aten_out_bf16_bits"] = aten.contiguous().view(torch.int16).numpy()
    f64 = oracle.paged_decode_f64(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale)
    f64 = f64[0] if isinstance(f64, tuple) else f64
    out["f64_out_f32"] = f64.float().numpy()
    # fp8 pages with per-head scales of the same rows
    ks = oracle.kv_head_scales(torch.cat([inp.k_ctx, inp.k_new]))
    vs = oracle.kv_head_scales(torch.cat([inp.v_ctx, inp.v_new]))
    kq, vq = fill_caches_cpu(inp, cache_dtype=torch.float8_e4m3fn, k_scale=ks, v_scale=vs)
    out["fp8_k_scale"], out["fp8_v_scale"] = ks.numpy(), vs.numpy()
    out["fp8_k_cache_sha256"], out["fp8_v_cache_sha256"] = np.array(sha(kq)), np.array(sha(vq))
    aten8 = oracle.aten_paged_decode(inp.q, kq.view(torch.float8_e4m3fn), vq.view(torch.float8_e4m3fn), lay.block_table,
                                     lay.seq_lens, cfg.scale, ks, vs)
    out["fp8_aten_out_bf16_bits"] = aten8.contiguous().view(torch.int16).numpy()
    return out


def main():
    with open(os.path.join(HERE, "fp8_e4m3fn_table.json"), "w") as f:
        json.dump(fp8_fixture(), f)
        f.write("\n")
    with open(os.path.join(HERE, "dcp_attention_merge.json"), "w") as f:
        json.dump(merge_fixture(), f, indent=1)
        f.write("\n")
    np.savez_compressed(os.path.join(HERE, "tiny_decode.npz"), **tiny_fixture())
    for name in sorted(os.listdir(HERE)):
        print(name, os.path.getsize(os.path.join(HERE, name)))


if __name__ == "__main__":
    main()
