"""The entry point that allocates nothing, xllm_mi355_paged_decode_gqa_static, against the entry point with a caller
workspace, through the C ABI: two calls in a row on the scratch the library holds, the second with a smaller
input; bit-identical outputs and LSEs (the kernels and the schedule are the same)."""
import pytest
import torch

import oracle
from helpers import assert_close_to_reference, fill_caches_gpu
from xllm_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu


def _call(lib, static, inp, kg, vg, ks, vs, device):
    cfg, lay = inp.cfg, inp.layout
    q = inp.q.to(device)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((cfg.batch, cfg.n_q_heads), float("nan"), dtype=torch.float32, device=device)
    table = lay.block_table.to(device)
    lens = lay.seq_lens.to(device)
    stream = torch.cuda.current_stream(device).cuda_stream
    ptr = lambda t: None if t is None else t.data_ptr()
    head = (q.data_ptr(), kg.data_ptr(), vg.data_ptr(), out.data_ptr(), lse.data_ptr(), table.data_ptr(),
            table.stride(0), lens.data_ptr(), ptr(ks), ptr(vs), cfg.batch, cfg.n_q_heads, cfg.n_kv_heads,
            cfg.head_dim, cfg.block_size, lay.num_blocks, q.stride(0), out.stride(0), int(lay.seq_lens.max()), -1,
            cfg.scale)
    code = capi.FP8_E4M3 if kg.dtype == torch.float8_e4m3fn else capi.BF16
    if static:
        # once outside the measurement (the first call on a device looks the scratch address up), then with the
        # device's memory watched: neither the driver's free memory nor torch's allocator may move across the call
        capi.check(lib.xllm_mi355_paged_decode_gqa_static(*head, capi.BF16, code, stream), "decode")
        torch.cuda.synchronize()
        free_before, _ = torch.cuda.mem_get_info(device)
        torch_before = torch.cuda.memory_allocated(device), torch.cuda.memory_reserved(device)
        rc = lib.xllm_mi355_paged_decode_gqa_static(*head, capi.BF16, code, stream)
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info(device)
        assert free_after == free_before, "the static entry point changed the device's free memory"
        assert (torch.cuda.memory_allocated(device), torch.cuda.memory_reserved(device)) == torch_before
    else:
        ws = ops.decode_workspace(device, lib.xllm_mi355_paged_decode_gqa_workspace_bytes(
            cfg.batch, cfg.n_q_heads, cfg.head_dim))
        rc = lib.xllm_mi355_paged_decode_gqa(*head, ws.data_ptr(), ws.numel(), capi.BF16, code, stream)
    capi.check(rc, "decode")
    torch.cuda.synchronize()
    return out, lse


def test_static_scratch_entry_point_matches_the_workspace_entry_point(device):
    lib = capi.lib()
    # contexts that span several workers (partials + merge through the scratch), then a smaller batch on the
    # same scratch, which still holds the first call's partials; then fp8 pages, head dim 256 (matrix-core kernel
    # with 8-token stages) and a block size of 8, which the dot-product kernel serves on the same scratch
    cases = [workloads.DecodeConfig("static_a", 48, 32, 8, 128, 16, 500, 3000),
             workloads.DecodeConfig("static_b", 5, 32, 8, 128, 16, 100, 900),
             workloads.DecodeConfig("static_fp8", 6, 32, 8, 128, 16, 300, 2500, cache_dtype="fp8"),
             workloads.DecodeConfig("static_d256", 4, 8, 2, 256, 32, 200, 1500),
             workloads.DecodeConfig("static_rows_bs8", 7, 32, 8, 128, 8, 100, 1200)]
    for i, cfg in enumerate(cases):
        inp = workloads.make_inputs(cfg, 70 + i)
        fp8 = cfg.cache_dtype == "fp8"
        kg, vg, ks, vs = fill_caches_gpu(inp, device, cache_dtype=torch.float8_e4m3fn if fp8 else None)
        out_s, lse_s = _call(lib, True, inp, kg, vg, ks, vs, device)
        out_w, lse_w = _call(lib, False, inp, kg, vg, ks, vs, device)
        assert torch.equal(out_s.view(torch.int16), out_w.view(torch.int16)), cfg.name
        assert torch.equal(lse_s, lse_w), cfg.name
        lay = inp.layout
        ref = oracle.aten_paged_decode(inp.q, kg.cpu(), vg.cpu(), lay.block_table, lay.seq_lens, cfg.scale,
                                       None if ks is None else ks.cpu(), None if vs is None else vs.cpu())
        assert_close_to_reference(out_s, ref, cfg.name)
    assert lib.xllm_mi355_decode_status(None, torch.cuda.current_stream(device).cuda_stream) == 0


def test_static_scratch_entry_point_rejects_what_does_not_fit(device):
    lib = capi.lib()
    fake = 1 << 20
    # more sequences than one launch holds: the slices of a longer batch would share the scratch
    rc = lib.xllm_mi355_paged_decode_gqa_static(fake, fake, fake, fake, None, fake, 8, fake, None, None, 2049, 32, 8,
                                                128, 16, 100, 4096, 4096, 100, -1, 0.1, capi.BF16, capi.BF16, None)
    assert rc == -7 and b"scratch" in lib.xllm_mi355_error_string(rc)
