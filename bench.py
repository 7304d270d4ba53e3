#!/usr/bin/env python3
"""Benchmark of the paged-KV decode path on one MI355X.

A step = one pass of the hot path over one synthetic decode batch that is already resident in
HBM: reshape_and_cache of the step's new K/V rows, then the paged decode attention over the
whole context.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

Without --workload every benchmark configuration runs: `tiny` as the correctness gate, then
llama3_8b, long_b256, fp8_kv and mla_dsv3, each timed over K steps after W warm-up steps.  The
headline fields of the line are those of long_b256 (the largest configuration that fits one GPU);
`per_config` carries the same fields for each of the four.  Every configuration's GPU output is
compared with the CPU checker on the sequences the CPU baseline samples (`parity`).
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published
METRIC = "paged-decode tokens/s + achieved HBM GB/s (% of 8 TB/s) on 1 MI355X"
ALL = ("llama3_8b", "long_b256", "fp8_kv", "mla_dsv3")
HEADLINE = "long_b256"
# The timed steps go round this many copies of the KV cache at different addresses, so that no step finds a page of
# the step before in a cache: two copies of the smallest timed cache (577 MB) put 1.15 GB between two reads of a page,
# against 256 MB of last-level cache.  (`same_cache` in the line is the loop over one copy.)
ROTATE = 2
MAX_ABS_TOL, MEAN_ABS_TOL = 2e-2, 2e-3   # attention output against the reference's libtorch CPU path, bf16


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed run of the step before the warm-up steps, until the clocks have settled")
    ap.add_argument("--workload", default="all",
                    help="all (default) | tiny | llama3_8b | long_b256 | fp8_kv | mla_dsv3 (the five configurations); "
                         "gqa_d64 | gqa_d64_fp8 | gqa_d256 | gqa_d256_fp8 | mla_tp8 (side workloads)")
    ap.add_argument("--seed", type=int, default=2)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU baseline (and with it the parity check)")
    ap.add_argument("--no-planned", action="store_true",
                    help="skip the second timed loop (the GQA step with the plan made once per step)")
    ap.add_argument("--two-calls", action="store_true",
                    help="GQA: time the pair reshape_and_cache + paged_decode_gqa as the step instead of the one call "
                         "write_and_decode_gqa, and do not time the other form beside the step (two_calls / one_call "
                         "in the default line)")
    ap.add_argument("--graph", action="store_true",
                    help="add a third timed loop: the step captured in a HIP graph and replayed (graph_replay in the line)")
    ap.add_argument("--cpu-sample", type=int, default=0, help="sequences timed on the CPU (0 = auto)")
    ap.add_argument("--calibrate", action="store_true",
                    help="run only the plain stream_read / stream_copy kernels over 1 GiB (counter calibration)")
    ap.add_argument("--neighbours", action="store_true",
                    help="time the ops on either side of the decode (reshape_and_cache, fused norm + rope + cache write, "
                         "the absorbed-weight batched matmuls of MLA, the gather of paged rows) and print their line")
    ap.add_argument("--traffic-json", default=os.path.join(ROOT, "profiles", "traffic.json"),
                    help="measured HBM bytes per launch by workload (written from rocprofv3 --pmc runs)")
    return ap.parse_args()


def cpu_baseline(inp, k_cache, v_cache, k_scale, v_scale, gpu_out, n_sample, budget_s):
    """Time the checker (the ATen-op-order restatement of the reference's libtorch CPU path) on the first
    n_sample sequences of the same workload (0 = as many as fit ~budget_s per pass), and compare what it
    computes with what the GPU computed for the same sequences: the rows the step's reshape_and_cache wrote
    (bit for bit) and the attention output (max / mean absolute difference).  A reported baseline and a
    checker, never the product path."""
    import torch
    import oracle
    cfg, lay = inp.cfg, inp.layout
    kc = k_cache.cpu()
    vc = None if v_cache is None else v_cache.cpu()
    ks = None if k_scale is None else k_scale.cpu()
    vs = None if v_scale is None else v_scale.cpu()
    if n_sample <= 0:
        # size the sample from one sequence's cost
        probe_q = inp.q[:1].cpu().contiguous()
        t0 = time.perf_counter()
        for _ in range(2):
            oracle.aten_paged_decode(probe_q, kc, vc, lay.block_table[:1].contiguous(),
                                     lay.seq_lens[:1].contiguous(), cfg.scale, ks, vs, dv=cfg.dv)
        per_token = (time.perf_counter() - t0) / 2 / max(1, int(lay.seq_lens[0]))
        mean_len = float(lay.seq_lens.float().mean())
        n_sample = max(1, min(cfg.batch, int(budget_s / (per_token * mean_len))))
    idx = list(range(min(n_sample, cfg.batch)))
    q = inp.q[idx].cpu().contiguous()
    table = lay.block_table[idx].contiguous()
    lens = lay.seq_lens[idx].contiguous()
    k_new = inp.k_new[idx].cpu().contiguous()
    v_new = None if inp.v_new is None else inp.v_new[idx].cpu().contiguous()
    slots = lay.new_slots[idx].contiguous()
    fp8 = kc.dtype == torch.float8_e4m3fn
    kc_store = kc.view(torch.uint8) if fp8 else kc
    vc_store = None if vc is None else (vc.view(torch.uint8) if fp8 else vc)
    # the GPU wrote these rows in every step; blank them in the copy so that the checker's write is what is compared
    gpu_k_rows = kc_store.view(-1, kc_store.shape[-2] * kc_store.shape[-1])[slots.long()].clone()
    gpu_v_rows = None if vc_store is None else vc_store.view(-1, vc_store.shape[-2] * vc_store.shape[-1])[slots.long()].clone()
    kc_store.view(-1, kc_store.shape[-2] * kc_store.shape[-1])[slots.long()] = 0
    if vc_store is not None:
        vc_store.view(-1, vc_store.shape[-2] * vc_store.shape[-1])[slots.long()] = 0

    def one():
        oracle.reshape_and_cache(k_new, v_new, kc_store, vc_store, slots, ks, vs)
        return oracle.aten_paged_decode(q, kc, vc, table, lens, cfg.scale, ks, vs, dv=cfg.dv)

    ref = one()  # warm-up; also the reference output
    cache_equal = torch.equal(kc_store.view(-1, gpu_k_rows.shape[1])[slots.long()], gpu_k_rows)
    if vc_store is not None:
        cache_equal = cache_equal and torch.equal(vc_store.view(-1, gpu_v_rows.shape[1])[slots.long()], gpu_v_rows)
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
        if sum(times) > 3 * budget_s:
            break
    t = statistics.median(times)
    diff = (gpu_out[idx].float().cpu().reshape(ref.shape) - ref.float()).abs()
    finite = bool(torch.isfinite(gpu_out.float()).all())
    parity = {
        "max_abs": float(diff.max()), "mean_abs": float(diff.mean()), "cache_bytes_equal": bool(cache_equal),
        "tolerance": {"max_abs": MAX_ABS_TOL, "mean_abs": MEAN_ABS_TOL},
        "sequences": len(idx),
        "ok": bool(finite and cache_equal and diff.max() <= MAX_ABS_TOL and diff.mean() <= MEAN_ABS_TOL),
        "against": "ATen-op-order restatement of the reference's libtorch CPU decode, same bytes",
    }
    baseline = {
        "value": len(idx) / t,
        "unit": "tokens/s",
        "cores": oracle.aten_lib().aten_oracle_num_threads(),
        "kind": "port",
        "sample": f"first {len(idx)} of {cfg.batch} sequences of the same workload "
                  f"({int(lens.sum())} context tokens), median of {len(times)} runs, "
                  f"{t * 1e3:.1f} ms per pass",
    }
    return baseline, parity


def collect_ms(lib, n):
    ms = (ctypes.c_float * n)()
    got = lib.xllm_mi355_profile_collect(ms, n)
    if got < 0:
        raise RuntimeError(f"xllm_mi355_profile_collect failed: {got}")
    return [ms[i] for i in range(got)]


def stream_rate(lib, capi, torch, dev, nbytes, copy=False, reps=10):
    """GB/s of the library's plain read (or copy) kernel over nbytes: what this GPU sustains for a
    working set of that size, measured with the same event hook as the decode kernel."""
    nbytes = max(16, nbytes // 16 * 16)
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty(nbytes, dtype=torch.uint8, device=dev) if copy else None
    stream = torch.cuda.current_stream(dev).cuda_stream

    def run():
        if copy:
            return lib.xllm_mi355_stream_copy(dst.data_ptr(), src.data_ptr(), nbytes, stream)
        return lib.xllm_mi355_stream_read(src.data_ptr(), nbytes, None, stream)

    for _ in range(3):
        capi.check(run(), "stream kernel")
    torch.cuda.synchronize()
    capi.check(lib.xllm_mi355_profile_enable(reps), "profile_enable")
    for _ in range(reps):
        run()
    ms = collect_ms(lib, reps)
    avg = sum(ms) / max(len(ms), 1)
    return (2 if copy else 1) * nbytes / (avg * 1e-3) / 1e9, avg


def calibrate(lib, capi, torch, dev):
    nbytes = 1 << 30
    read_gbs, read_ms = stream_rate(lib, capi, torch, dev, nbytes)
    copy_gbs, copy_ms = stream_rate(lib, capi, torch, dev, nbytes, copy=True)
    return {"bytes": nbytes, "stream_read_gbs": read_gbs, "stream_read_ms": read_ms,
            "stream_copy_gbs_read_plus_write": copy_gbs, "stream_copy_ms": copy_ms}


def neighbours(ops, workloads, torch, dev, steps, lib=None, capi=None):
    """The ops that feed the decode and take its result, at the shapes of the benchmark configurations: every one is
    HBM-bound integer / byte movement or a skinny batched matmul, so each is priced by its algorithmic bytes."""
    import math
    g = torch.Generator().manual_seed(0)

    def timed(fn):
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps * 1e3

    rows = []

    def row(op, kernel, shape, us, nbytes):
        # the yardstick: the library's plain copy kernel moving the same number of bytes (half read, half written),
        # timed by its own event pair
        copy_gbs = None
        if lib is not None:
            copy_gbs, _ = stream_rate(lib, capi, torch, dev, nbytes // 2, copy=True, reps=20)
        # ... and the runtime's own device-to-device copy of the same bytes (Tensor.copy_), timed like the op
        src = torch.empty(nbytes // 2, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        torch_us = timed(lambda: dst.copy_(src))
        del src, dst
        rows.append({"op": op, "kernel": kernel, "shape": shape, "us": us, "algorithmic_bytes": nbytes,
                     "gbs": nbytes / us / 1e3, "frac_of_hbm_peak": nbytes / us / 1e3 / HBM_PEAK_GBS,
                     "plain_copy_gbs_same_bytes": copy_gbs,
                     "torch_copy_gbs_same_bytes": nbytes // 2 * 2 / torch_us / 1e3})

    # reshape_and_cache: a prefill chunk of 8192 tokens into bf16 pages (configuration 2's heads), read + write
    T, nk, D = 8192, 8, 128
    k = torch.randn(T, nk, D, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(T, nk, D, generator=g).to(torch.bfloat16).to(dev)
    P = T // 16 + 8
    kc = torch.zeros(P, 16, nk, D, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    slots = torch.randperm(P * 16, generator=g)[:T].to(torch.int32).to(dev)
    prm = ops.ReshapePagedCacheParams(key=k, value=v, k_cache=kc, v_cache=vc, slot_mapping=slots)
    row("reshape_and_cache", "reshape_vec_kernel", f"{T} tokens x {nk} KV heads x {D}, bf16 pages of 16",
        timed(lambda: ops.reshape_paged_cache(prm)), workloads.reshape_bytes(T, nk * D, 2, 2, 2))
    # fused q/k norm + rope + cache write of the same chunk: reads q, k, v once, writes q, k and the two cache rows
    nq = 32
    qkv = (torch.randn(T, (nq + 2 * nk) * D, generator=g) * 0.3).to(torch.bfloat16).to(dev)
    qw = torch.ones(D, dtype=torch.bfloat16, device=dev)
    ang = torch.rand(4096, D // 2, generator=g) * 6.28
    cs = torch.cat([ang.cos(), ang.sin()], 1).to(dev)
    pos = torch.randint(0, 4096, (T,), generator=g).to(dev)
    row("fused_qk_norm_rope + cache write", "rope_and_cache_kernel", f"{T} tokens, {nq}/{nk} heads x {D}",
        timed(lambda: ops.fused_qk_norm_rope(qkv, nq, nk, nk, D, 1e-6, qw, qw, cs, False, pos, k_cache=kc, v_cache=vc,
                                             slot_mapping=slots)),
        T * (nq + nk) * D * 2 * 2 + T * 2 * nk * D * 2 * 2)
    # the two absorbed-weight matmuls around the MLA decode of configuration 5 (64 tokens, 128 heads)
    for K, N in ((128, 512), (512, 128)):
        H, Tq = 128, 64
        x = torch.randn(Tq, H, K, generator=g).to(torch.bfloat16).to(dev)
        w = (torch.randn(H, K, N, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(dev)
        out = torch.empty(Tq, H, N, dtype=torch.bfloat16, device=dev)
        row("absorbed_bmm", "absorbed_bmm_kernel", f"{Tq} tokens x {H} heads, [{K}] x [{K}, {N}]",
            timed(lambda: ops.absorbed_bmm(x, w, out=out)), H * K * N * 2 + Tq * H * (K + N) * 2)
    # gather of the paged latent rows of configuration 5 into a packed tensor (chunked prefill reads it)
    cfg = workloads.CONFIGS["mla_dsv3"]
    lay = workloads.make_layout(cfg, 1)
    lat = torch.randn(lay.num_blocks, cfg.block_size, 1, 576, generator=g).to(torch.bfloat16).to(dev)
    cu = torch.zeros(cfg.batch + 1, dtype=torch.int32)
    cu[1:] = lay.seq_lens.cumsum(0)
    total = int(cu[-1])
    tab, cu = lay.block_table.to(dev), cu.to(dev)
    row("gather_mla_latent_cache", "gather_paged_rows_kernel", f"{total} rows of 1152 bytes from pages of {cfg.block_size}",
        timed(lambda: ops.gather_mla_latent_cache(lat, tab, cu, total)), 2 * total * 1152)
    return {"neighbour_ops": rows, "steps": steps, "peak_gbs": HBM_PEAK_GBS,
            "note": "torch events around the loop of calls (launch gaps included)"}


# The KV caches of every workload are views of ONE pool, allocated before anything else on the device, as a server
# allocates its KV pool at start-up, and nothing is handed back to the driver between workloads.  Device memory that
# a process frees (torch.cuda.empty_cache) and allocates again is slower to work from: a workload that ran after such
# a cycle took 386.7 us per decode launch against 373.2-373.7 us without it (fp8_kv; alone in a process 373.6 us).
_KV_POOL = None


def kv_pool_reserve(torch, dev, nbytes):
    global _KV_POOL
    if _KV_POOL is None or _KV_POOL.numel() < nbytes:
        _KV_POOL = None
        _KV_POOL = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    return _KV_POOL


def kv_pool_caches(torch, dev, shape, dtype, n):
    """n zeroed caches of `shape` as views of the pool."""
    one = 1
    for x in shape:
        one *= x
    one *= torch.empty(0, dtype=dtype).element_size()
    stride = (one + 4095) // 4096 * 4096
    pool = kv_pool_reserve(torch, dev, stride * n)
    views = []
    for i in range(n):
        v = pool[i * stride : i * stride + one].view(dtype).view(shape)
        v.zero_()
        views.append(v)
    return views


def kv_pool_bytes(workloads, names, seed):
    need = 0
    for name in names:
        cfg = workloads.CONFIGS[name]
        lay = workloads.make_layout(cfg, seed)
        one = lay.num_blocks * cfg.block_size * cfg.n_kv_heads * cfg.head_dim * (1 if cfg.cache_dtype == "fp8" else 2)
        need = max(need, ((one + 4095) // 4096 * 4096) * (1 if cfg.mla else 2) * ROTATE)
    return need


def decode_kernel_name(cfg):
    if cfg.mla:
        knob = os.environ.get("XLLM_MI355_MLA_KERNEL", "")[:1]
        if knob == "h" or cfg.n_q_heads <= 64:
            return "mla_decode16_kernel"
        return "mla_decode_ds_kernel" if knob == "n" else "mla_decode_w4_kernel"
    mfma = cfg.head_dim in (64, 128, 256) and cfg.block_size >= 16 \
        and cfg.block_size & (cfg.block_size - 1) == 0 and os.environ.get("XLLM_MI355_GQA_KERNEL", "")[:1] != "r"
    return "gqa_mfma_kernel" if mfma else "gqa_decode_kernel"


def run_workload(name, args, lib, capi, ops, workloads, torch, dev, cpu_budget_s):
    cfg = workloads.CONFIGS[name]
    fp8 = cfg.cache_dtype == "fp8"

    # ---- build the resident workload: context rows go into the cache through the op itself
    inp = workloads.make_inputs(cfg, args.seed, device=dev)
    lay = inp.layout
    cache_dt = torch.float8_e4m3fn if fp8 else torch.bfloat16
    shape = (lay.num_blocks, cfg.block_size, cfg.n_kv_heads, cfg.head_dim)
    views = kv_pool_caches(torch, dev, shape, cache_dt, (1 if cfg.mla else 2) * ROTATE)
    k_caches = views[:ROTATE]
    v_caches = [None] * ROTATE if cfg.mla else views[ROTATE:]
    k_cache, v_cache = k_caches[0], v_caches[0]
    k_scale = v_scale = None
    if fp8:
        k_scale = ops.kv_head_scales(torch.cat([inp.k_ctx, inp.k_new]))
        v_scale = ops.kv_head_scales(torch.cat([inp.v_ctx, inp.v_new]))
    store = ops.quant_to_paged_cache if fp8 else ops.reshape_paged_cache
    ctx_slots = lay.ctx_slots.to(dev)
    new_slots = lay.new_slots.to(dev)
    store(ops.ReshapePagedCacheParams(key=inp.k_ctx, value=inp.v_ctx, k_cache=k_cache, v_cache=v_cache,
                                      slot_mapping=ctx_slots, k_cache_scale=k_scale, v_cache_scale=v_scale))
    inp.k_ctx = inp.v_ctx = None   # (the context now lives in the cache)
    for i in range(1, ROTATE):     # the other copies: the same bytes at other addresses
        k_caches[i].view(torch.uint8).copy_(k_cache.view(torch.uint8))
        if v_cache is not None:
            v_caches[i].view(torch.uint8).copy_(v_cache.view(torch.uint8))
    table = lay.block_table.to(dev)
    seq_lens = lay.seq_lens.to(dev)
    max_len = int(lay.seq_lens.max())
    new_params = ops.ReshapePagedCacheParams(key=inp.k_new, value=inp.v_new, k_cache=k_cache,
                                             v_cache=v_cache, slot_mapping=new_slots,
                                             k_cache_scale=k_scale, v_cache_scale=v_scale)
    if cfg.mla:
        mla = ops.DenseDecodeParams(
            q_nope=inp.q[:, :, : cfg.v_dim].contiguous().view(cfg.batch, 1, cfg.n_q_heads, cfg.v_dim),
            q_pe=inp.q[:, :, cfg.v_dim :].contiguous().view(cfg.batch, 1, cfg.n_q_heads, cfg.head_dim - cfg.v_dim),
            k_cache=k_cache, seqlens_k=seq_lens, block_table=table, head_size_v=cfg.v_dim,
            softmax_scale=cfg.scale)
    out = torch.empty(cfg.batch, cfg.n_q_heads, cfg.dv, dtype=torch.bfloat16, device=dev)

    # The timed loop calls the C ABI directly with pre-bound arguments (what a C++ caller does);
    # one untimed pass through the Python op mirror first checks the same arguments.
    store(new_params)
    if cfg.mla:
        ops.dense_decode(mla, max_seq_len=max_len)
    else:
        ops.batch_decode(inp.q, k_cache, out, table, seq_lens, v_cache=v_cache,
                         k_cache_quant_scale=k_scale, v_cache_quant_scale=v_scale, scale=cfg.scale,
                         max_seq_len=max_len)
    stream = torch.cuda.current_stream(dev).cuda_stream
    ptr = lambda t: None if t is None else t.data_ptr()
    code = {torch.bfloat16: capi.BF16, torch.float8_e4m3fn: capi.FP8_E4M3}
    row = cfg.n_kv_heads * cfg.head_dim
    reshape_fn = lib.xllm_mi355_reshape_and_cache
    if cfg.mla:
        ws_bytes = lib.xllm_mi355_paged_decode_mla_workspace_bytes(cfg.batch, cfg.n_q_heads, max_len)
    else:
        ws_bytes = lib.xllm_mi355_paged_decode_gqa_workspace_bytes(cfg.batch, cfg.n_q_heads, cfg.head_dim)
    ws = ops.decode_workspace(dev, ws_bytes)
    if cfg.mla:
        out = torch.empty(cfg.batch, 1, cfg.n_q_heads, cfg.v_dim, dtype=torch.bfloat16, device=dev)
        decode_fn = lib.xllm_mi355_paged_decode_mla
    else:
        decode_fn = lib.xllm_mi355_paged_decode_gqa

    def bound_args(kc, vc):
        reshape_args = (ptr(inp.k_new), ptr(inp.v_new), ptr(kc), ptr(vc), ptr(new_slots),
                        ptr(k_scale), ptr(v_scale), cfg.batch, cfg.n_kv_heads, cfg.head_dim, cfg.block_size,
                        lay.num_blocks, row, row, capi.BF16, code[cache_dt], stream)
        if cfg.mla:
            decode_args = (ptr(mla.q_nope), ptr(mla.q_pe), ptr(kc), ptr(out), None, ptr(table),
                           table.stride(0), ptr(seq_lens), cfg.batch, cfg.n_q_heads, cfg.v_dim,
                           cfg.head_dim - cfg.v_dim, cfg.block_size, lay.num_blocks, max_len, cfg.scale,
                           ptr(ws), ws.numel(), capi.BF16, stream)
        else:
            decode_args = (ptr(inp.q), ptr(kc), ptr(vc), ptr(out), None, ptr(table),
                           table.stride(0), ptr(seq_lens), ptr(k_scale), ptr(v_scale), cfg.batch,
                           cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, lay.num_blocks,
                           inp.q.stride(0), out.stride(0), max_len, -1, cfg.scale, ptr(ws), ws.numel(),
                           capi.BF16, code[cache_dt], stream)
        return reshape_args, decode_args

    bound = [bound_args(k_caches[i], v_caches[i]) for i in range(ROTATE)]
    reshape_args, decode_args = bound[0]
    # GQA: the step as the attention layer issues it, one call that stores the new rows and attends
    # (xllm_mi355_write_and_decode_gqa); the pair of calls it replaces is timed beside it.  MLA: the pair is the step
    # (xllm_mi355_write_and_decode_mla takes as long, with a decode kernel that is longer by the store it holds), and
    # the one call is timed beside it.
    one_call = not args.two_calls and not cfg.mla
    one_fn = lib.xllm_mi355_write_and_decode_mla if cfg.mla else lib.xllm_mi355_write_and_decode_gqa

    def one_call_args(d_args, plan=None):
        plan_args = (ptr(plan), 0 if plan is None else plan.numel())
        if cfg.mla:
            return (ptr(inp.k_new), ptr(new_slots), row) + plan_args + d_args
        return (ptr(inp.k_new), ptr(inp.v_new), ptr(new_slots), row, row) + plan_args \
            + d_args[:8] + (None, None, None) + d_args[8:]

    def step_calls(i, one, plan=None):
        """The calls of one step on cache copy i: [(fn, args), ...]."""
        r_args, d_args = bound[i]
        if one:
            return [(one_fn, one_call_args(d_args, plan))]
        if plan is None:
            return [(reshape_fn, r_args), (decode_fn, d_args)]
        if cfg.mla:
            return [(reshape_fn, r_args), (lib.xllm_mi355_paged_decode_mla_planned, (ptr(plan), plan.numel()) + d_args)]
        return [(reshape_fn, r_args), (lib.xllm_mi355_paged_decode_gqa_planned,
                                       (ptr(plan), plan.numel()) + d_args[:8] + (None, None, None) + d_args[8:])]

    def make_step(copies, one=one_call, plan=None):
        state = [0]
        calls = [step_calls(i, one, plan) for i in range(copies)]

        def step():
            todo = calls[state[0] % copies]
            state[0] += 1
            for fn, fn_args in todo:
                rc = fn(*fn_args)
                if rc:
                    capi.check(rc, "bench step")
        return step

    def timed_loop(step, events):
        """W warm-up steps, then K steps between two synchronisations.  With `events` every decode and merge launch of
        the K steps carries an event pair (their kernel times come back; the wall clock of such a loop is not used:
        the instrumented launch path is not the one a caller takes)."""
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        if events:
            capi.check(lib.xllm_mi355_profile_enable(2 * args.steps), "profile_enable")
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        if not events:
            return elapsed / args.steps * 1e3, None, None
        ms = collect_ms(lib, 2 * args.steps)   # per step: the decode kernel, then the merge kernel
        return elapsed / args.steps * 1e3, sum(ms[0::2]) / max(len(ms[0::2]), 1), sum(ms[1::2]) / max(len(ms[1::2]), 1)

    # The first tens of milliseconds of work after an idle period run at other clocks than the steady state a
    # serving loop sees (kernel times swing by 20-30 % over the first ~100 launches): run the step untimed until
    # --settle-ms have passed, then the W warm-up steps, then the K timed ones.
    step = make_step(ROTATE)
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
    # the headline: plain launches (no event pairs), the caches taken in turn
    ms_per_step, _, _ = timed_loop(step, events=False)
    # the kernels' own times: the same loop with an event pair on every decode and merge launch
    instrumented_ms_per_step, kernel_ms, merge_ms = timed_loop(step, events=True)
    ops.decode_status(dev)                 # raises if a wait inside a decode kernel gave up
    # the same two loops over ONE copy of the cache (every step reads the pages the step before read)
    same_step = make_step(1)
    same_ms_per_step, _, _ = timed_loop(same_step, events=False)
    _, same_kernel_ms, same_merge_ms = timed_loop(same_step, events=True)
    same_cache = {"ms_per_step": same_ms_per_step, "kernel_ms": same_kernel_ms, "merge_kernel_ms": same_merge_ms,
                  "tokens_per_s": cfg.batch / (same_ms_per_step * 1e-3)}
    # the other form of the step: the pair of calls (store, then decode) beside the one call, or the one call beside
    # the pair
    two_calls = other_form = None
    if not args.two_calls:
        other_step = make_step(ROTATE, one=not one_call)
        other_ms_per_step, _, _ = timed_loop(other_step, events=False)
        _, other_kernel_ms, other_merge_ms = timed_loop(other_step, events=True)
        other_out = out.clone()
        step()
        torch.cuda.synchronize()
        other_form = {"ms_per_step": other_ms_per_step, "kernel_ms": other_kernel_ms, "merge_kernel_ms": other_merge_ms,
                      "tokens_per_s": cfg.batch / (other_ms_per_step * 1e-3),
                      "bit_identical": bool(torch.equal(other_out, out))}
        if one_call:
            two_calls = other_form
    elapsed = ms_per_step * 1e-3 * args.steps

    # ---- the same step as the layers after the first see it when the step was planned once (not the headline:
    # `value` above is the self-contained call, which derives its schedule in every launch)
    planned = None
    if not args.no_planned and (not cfg.mla or cfg.n_q_heads > 64):
        plan = torch.empty(lib.xllm_mi355_paged_decode_plan_bytes(), dtype=torch.uint8, device=dev)
        if cfg.mla:
            plan_fn = lib.xllm_mi355_paged_decode_mla_plan
            plan_args = (ptr(plan), plan.numel(), ptr(table), table.stride(0), ptr(seq_lens), cfg.batch, cfg.n_q_heads,
                         cfg.block_size, stream)
        else:
            plan_fn = lib.xllm_mi355_paged_decode_gqa_plan
            plan_args = (ptr(plan), plan.numel(), ptr(table), table.stride(0), ptr(seq_lens), None, None, None, cfg.batch,
                         cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, -1, code[cache_dt], stream)
        plain_out = out.clone()
        planned_step = make_step(ROTATE, plan=plan)

        capi.check(lib.xllm_mi355_profile_enable(1), "profile_enable")
        capi.check(plan_fn(*plan_args), "the plan of the step")
        torch.cuda.synchronize()
        plan_ms = collect_ms(lib, 1)
        p_ms_per_step, _, _ = timed_loop(planned_step, events=False)
        _, p_kernel_ms, p_merge_ms = timed_loop(planned_step, events=True)
        ops.decode_status(dev)
        planned = {"kernel_ms": p_kernel_ms, "merge_kernel_ms": p_merge_ms,
                   "ms_per_step": p_ms_per_step, "plan_kernel_ms": plan_ms[0] if plan_ms else None,
                   "bit_identical": bool(torch.equal(plain_out, out))}

    # ---- the same step captured once in a HIP graph and replayed, as the reference's graph executor runs a decode
    # step (not the headline either: `value` is the eager loop above)
    graph_replay = None
    if args.graph:
        ref_out = out.clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            cs = torch.cuda.current_stream(dev).cuda_stream
            for fn, fn_args in step_calls(0, one_call):
                capi.check(fn(*(fn_args[:-1] + (cs,))), "bench captured step")
        t_settle = time.perf_counter()   # (the capture left the GPU idle: let the clocks settle again)
        while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
            for _ in range(20):
                graph.replay()
            torch.cuda.synchronize()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        g_elapsed = time.perf_counter() - t0
        graph_replay = {"ms_per_step": g_elapsed / args.steps * 1e3,
                        "tokens_per_s": cfg.batch / (g_elapsed / args.steps),
                        "bit_identical": bool(torch.equal(ref_out, out))}
        del graph

    tokens_per_s = cfg.batch / (ms_per_step * 1e-3)

    # ---- roofline of the dominant kernel (the decode kernel), from algorithmic work
    traffic = None
    try:
        with open(args.traffic_json) as f:
            traffic = json.load(f).get(name, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        pass
    op_ms = kernel_ms + merge_ms
    if cfg.mla:
        nbytes, flops = workloads.mla_bytes_flops(cfg, lay.seq_lens)
    else:
        nbytes, flops = workloads.gqa_bytes(cfg, lay.seq_lens, 1 if fp8 else 2), None
    if cfg.mla and cfg.n_q_heads > 64:
        achieved = flops / (kernel_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic,
                    "op_frac": flops / (op_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                    "hbm_gbs": nbytes / (kernel_ms * 1e-3) / 1e9}
    else:
        # GQA, and MLA with the few heads of a tensor-parallel shard (30-120 flop per cache byte, far below the ridge)
        achieved = nbytes / (kernel_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                    "op_frac": nbytes / (op_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    roofline.update({"kernel": decode_kernel_name(cfg), "kernel_ms": kernel_ms, "merge_kernel_ms": merge_ms,
                     "algorithmic_bytes": nbytes,
                     "traffic_source": "profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this "
                                       "workload, scaled by a plain copy of known size; a constant of the build, not "
                                       "measured in this run",
                     "kernel_ms_source": "HIP event pairs on the decode and merge dispatches of a second loop of "
                                         "the same steps; ms_per_step and value come from the loop without them"})
    if flops is not None:
        roofline["algorithmic_flops"] = flops
    if planned is not None:
        p_op = (planned["kernel_ms"] + planned["merge_kernel_ms"]) * 1e-3
        planned["op_frac"] = (flops / p_op / 1e12 / MFMA_BF16_PEAK_TFLOPS) if roofline["bound"] == "mfma" \
            else (nbytes / p_op / 1e9 / HBM_PEAK_GBS)
        roofline["planned"] = planned
    # the same number of bytes through the plain read kernel: the rate this GPU sustains at this size
    roofline["stream_read_gbs_same_bytes"], _ = stream_rate(lib, capi, torch, dev, nbytes)

    result = {
        "metric": METRIC,
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": args.settle_ms,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3 KV, bf16 Q/O, fp32 accumulate" if fp8 else "bf16 (fp32 accumulate)",
        "data": "synthetic",
        "config": {
            "workload": name,
            "batch": cfg.batch, "n_q_heads": cfg.n_q_heads, "n_kv_heads": cfg.n_kv_heads,
            "head_dim": cfg.head_dim, "block_size": cfg.block_size,
            "context_tokens": int(lay.seq_lens.sum()), "max_context": max_len,
            "step": (("write_and_decode_mla: the new latent rows" if cfg.mla else "write_and_decode_gqa: the new K/V rows")
                     + " stored and attended to in one call, inputs resident in HBM"
                     if one_call else
                     "reshape_and_cache(new K/V rows) + paged decode attention, inputs resident in HBM"),
        },
        "instrumented_ms_per_step": instrumented_ms_per_step,
        "kv_cache_copies_in_rotation": ROTATE,
        "same_cache": same_cache,
        "two_calls": two_calls,
        "one_call": None if one_call else other_form,
        "hbm_gbs_whole_step": (nbytes + workloads.reshape_bytes(
            cfg.batch, cfg.n_kv_heads * cfg.head_dim, 2, 1 if fp8 else 2, 1 if cfg.mla else 2))
            / (ms_per_step * 1e-3) / 1e9,
        "roofline": roofline,
    }
    if graph_replay is not None:
        result["graph_replay"] = graph_replay
    if not args.no_cpu_baseline:
        result["cpu_baseline"], result["parity"] = cpu_baseline(
            inp, k_cache, v_cache, k_scale, v_scale, out.view(cfg.batch, cfg.n_q_heads, cfg.dv), args.cpu_sample,
            cpu_budget_s)
    # (no torch.cuda.empty_cache() here: memory handed back to the driver and allocated again makes the kernels of the
    # next workload 1-3.5 % slower, see kv_pool_caches; a serving process keeps its allocations anyway)
    del k_cache, v_cache, k_caches, v_caches, views, inp, out
    return result


def main():
    args = parse_args()
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        print("bench.py: this build runs on ONE GPU (every box has one); --gpus N with N > 1 is not "
              "supported. The path shards by sequence or KV head with no exchange inside the op.",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from xllm_amd import capi, ops, workloads

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    lib = capi.lib()  # raises if the HIP library has not been built
    dev = torch.device("cuda:0")
    if args.calibrate:
        print(json.dumps(calibrate(lib, capi, torch, dev)))
        return
    if args.neighbours:
        print(json.dumps(neighbours(ops, workloads, torch, dev, max(args.steps, 1), lib, capi)))
        return
    run = lambda name, budget: run_workload(name, args, lib, capi, ops, workloads, torch, dev, budget)
    if args.workload != "all":
        result = run(args.workload, 6.0)
    else:
        kv_pool_reserve(torch, dev, kv_pool_bytes(workloads, ["tiny"] + list(ALL), args.seed))
        # the correctness gate first: a wrong path is not timed
        gate = run("tiny", 1.0)
        if not args.no_cpu_baseline and not gate["parity"]["ok"]:
            print(f"bench.py: the tiny configuration fails parity: {gate['parity']}", file=sys.stderr)
            sys.exit(3)
        per = {}
        for name in ALL:
            per[name] = run(name, 5.0 if name == HEADLINE else 2.0)
            print(f"bench.py: {name}: {per[name]['ms_per_step']:.4f} ms/step, roofline {per[name]['roofline']['frac']:.3f}",
                  file=sys.stderr, flush=True)
        result = dict(per[HEADLINE])
        result["gate"] = {"workload": "tiny", "parity": gate.get("parity")}
        keep = ("value", "unit", "ms_per_step", "dtype", "config", "hbm_gbs_whole_step", "roofline", "cpu_baseline",
                "parity", "same_cache", "two_calls", "one_call", "instrumented_ms_per_step",
                "kv_cache_copies_in_rotation")
        result["per_config"] = [{k: per[name][k] for k in keep if k in per[name]} for name in ALL]
        if not args.no_cpu_baseline:
            result["parity_all_ok"] = all(per[name]["parity"]["ok"] for name in ALL) and gate["parity"]["ok"]
    print(json.dumps(result))
    if not args.no_cpu_baseline:
        bad = [name for name, ok in ((result["config"]["workload"], result["parity"]["ok"]),) if not ok]
        bad += [p["config"]["workload"] for p in result.get("per_config", []) if not p["parity"]["ok"]]
        if bad:
            print(f"bench.py: parity FAILED for {sorted(set(bad))}", file=sys.stderr)
            sys.exit(3)


if __name__ == "__main__":
    main()
