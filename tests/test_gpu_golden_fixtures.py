"""The GPU path against the committed golden vectors of configuration 1 (tests/golden/tiny_decode.npz): cache bytes
bit for bit (bf16 pages, and fp8 pages with per-head scales), attention output within the tolerance of the path
(max-abs 2e-2, mean-abs 2e-3) of the stored output of the reference's libtorch decode order.  No CPU checker runs
here: the expected values are data."""
import hashlib
import os

import numpy as np
import pytest
import torch

from helpers import MAX_ABS_TOL, MEAN_ABS_TOL, fill_caches_gpu
from xllm_amd import ops, workloads

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def sha(t):
    return hashlib.sha256(t.contiguous().cpu().view(torch.uint8).numpy().tobytes()).hexdigest()


def close(out, bits):
    want = torch.from_numpy(bits.copy()).view(torch.bfloat16).float()
    diff = (out.float().cpu() - want).abs()
    assert diff.max() <= MAX_ABS_TOL and diff.mean() <= MEAN_ABS_TOL, (diff.max().item(), diff.mean().item())


def test_tiny_configuration_against_the_golden_vectors(device):
    fx = np.load(os.path.join(GOLDEN, "tiny_decode.npz"), allow_pickle=False)
    cfg = workloads.CONFIGS["tiny"]
    inp = workloads.make_inputs(cfg, int(fx["seed"]))
    lay = inp.layout
    digest = hashlib.sha256()
    for t in (lay.seq_lens, lay.block_table, lay.new_slots, inp.q, inp.k_ctx, inp.v_ctx, inp.k_new, inp.v_new):
        digest.update(t.contiguous().view(torch.uint8).numpy().tobytes())
    if digest.hexdigest() != str(fx["inputs_sha256"]):
        pytest.skip("torch's CPU generator gives other bytes on this box: the fixture does not apply")
    q, table, lens = inp.q.to(device), lay.block_table.to(device), lay.seq_lens.to(device)
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    assert sha(kg) == str(fx["k_cache_sha256"]) and sha(vg) == str(fx["v_cache_sha256"])
    out, _ = ops.batch_decode(q, kg, torch.empty_like(q), table, lens, v_cache=vg, scale=cfg.scale)
    close(out, fx["aten_out_bf16_bits"])
    k8, v8, ks, vs = fill_caches_gpu(inp, device, cache_dtype=torch.float8_e4m3fn)
    assert np.array_equal(ks.cpu().numpy(), fx["fp8_k_scale"]) and np.array_equal(vs.cpu().numpy(), fx["fp8_v_scale"])
    assert sha(k8) == str(fx["fp8_k_cache_sha256"]) and sha(v8) == str(fx["fp8_v_cache_sha256"])
    out8, _ = ops.batch_decode(q, k8, torch.empty_like(q), table, lens, v_cache=v8, k_cache_quant_scale=ks,
                               v_cache_quant_scale=vs, scale=cfg.scale)
    close(out8, fx["fp8_aten_out_bf16_bits"])
