#!/usr/bin/env python3
"""Benchmark of the paged-KV decode path on one MI355X.

A step = one pass of the hot path over one synthetic decode batch that is already resident in
HBM: reshape_and_cache of the step's new K/V rows, then the paged decode attention over the
whole context.  Prints ONE JSON line (see README of the contract in the repository docs).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="llama3_8b",
                    help="tiny | llama3_8b | long_b256 | fp8_kv | mla_dsv3 (the five configurations); gqa_d64 | mla_tp8 (side workloads)")
    ap.add_argument("--seed", type=int, default=2)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample", type=int, default=0, help="sequences timed on the CPU (0 = auto)")
    ap.add_argument("--calibrate", action="store_true",
                    help="run only the plain stream_read / stream_copy kernels over 1 GiB (counter calibration)")
    ap.add_argument("--traffic-json", default=os.path.join(ROOT, "profiles", "traffic.json"),
                    help="measured HBM bytes per launch by workload (written from rocprofv3 --pmc runs)")
    return ap.parse_args()


def cpu_baseline(inp, k_cache, v_cache, k_scale, v_scale, n_sample, budget_s=6.0):
    """Time the checker (the ATen-op-order restatement of the reference's libtorch CPU path) on the
    first n_sample sequences of the same workload (0 = as many as fit ~budget_s per pass).  A reported
    baseline, never the product path."""
    import torch
    import oracle
    cfg, lay = inp.cfg, inp.layout
    if n_sample <= 0:
        # size the sample from one sequence's cost
        probe_q = inp.q[:1].cpu().contiguous()
        kc0 = k_cache.cpu()
        vc0 = None if v_cache is None else v_cache.cpu()
        ks0 = None if k_scale is None else k_scale.cpu()
        vs0 = None if v_scale is None else v_scale.cpu()
        t0 = time.perf_counter()
        for _ in range(2):
            oracle.aten_paged_decode(probe_q, kc0, vc0, lay.block_table[:1].contiguous(),
                                     lay.seq_lens[:1].contiguous(), cfg.scale, ks0, vs0, dv=cfg.dv)
        per_token = (time.perf_counter() - t0) / 2 / max(1, int(lay.seq_lens[0]))
        mean_len = float(lay.seq_lens.float().mean())
        n_sample = max(1, min(cfg.batch, int(budget_s / (per_token * mean_len))))
    idx = list(range(min(n_sample, cfg.batch)))
    q = inp.q[idx].cpu().contiguous()
    kc = k_cache.cpu()
    vc = None if v_cache is None else v_cache.cpu()
    table = lay.block_table[idx].contiguous()
    lens = lay.seq_lens[idx].contiguous()
    ks = None if k_scale is None else k_scale.cpu()
    vs = None if v_scale is None else v_scale.cpu()
    k_new = inp.k_new[idx].cpu().contiguous()
    v_new = None if inp.v_new is None else inp.v_new[idx].cpu().contiguous()
    slots = lay.new_slots[idx].contiguous()
    kc_store = kc.view(torch.uint8) if kc.dtype == torch.float8_e4m3fn else kc
    vc_store = None if vc is None else (vc.view(torch.uint8) if vc.dtype == torch.float8_e4m3fn else vc)

    def one():
        oracle.reshape_and_cache(k_new, v_new, kc_store, vc_store, slots, ks, vs)
        return oracle.aten_paged_decode(q, kc, vc, table, lens, cfg.scale, ks, vs, dv=cfg.dv)

    one()  # warm-up
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
        if sum(times) > 30:
            break
    t = statistics.median(times)
    return {
        "value": len(idx) / t,
        "unit": "tokens/s",
        "cores": oracle.aten_lib().aten_oracle_num_threads(),
        "kind": "port",
        "sample": f"first {len(idx)} of {cfg.batch} sequences of the same workload "
                  f"({int(lens.sum())} context tokens), median of {len(times)} runs, "
                  f"{t * 1e3:.1f} ms per pass",
    }


def stream_rate(lib, capi, torch, dev, nbytes, copy=False, reps=10):
    """GB/s of the library's plain read (or copy) kernel over nbytes: what this GPU sustains for a
    working set of that size, measured with the same event hook as the decode kernel."""
    import ctypes
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
    ms = (ctypes.c_float * reps)()
    n = lib.xllm_mi355_profile_collect(ms, reps)
    avg = sum(ms[i] for i in range(n)) / max(n, 1)
    return (2 if copy else 1) * nbytes / (avg * 1e-3) / 1e9, avg


def calibrate(lib, capi, torch, dev):
    nbytes = 1 << 30
    read_gbs, read_ms = stream_rate(lib, capi, torch, dev, nbytes)
    copy_gbs, copy_ms = stream_rate(lib, capi, torch, dev, nbytes, copy=True)
    return {"bytes": nbytes, "stream_read_gbs": read_gbs, "stream_read_ms": read_ms,
            "stream_copy_gbs_read_plus_write": copy_gbs, "stream_copy_ms": copy_ms}


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
    cfg = workloads.CONFIGS[args.workload]
    fp8 = cfg.cache_dtype == "fp8"

    # ---- build the resident workload: context rows go into the cache through the op itself
    inp = workloads.make_inputs(cfg, args.seed, device=dev)
    lay = inp.layout
    cache_dt = torch.float8_e4m3fn if fp8 else torch.bfloat16
    shape = (lay.num_blocks, cfg.block_size, cfg.n_kv_heads, cfg.head_dim)
    k_cache = torch.zeros(shape, dtype=cache_dt, device=dev)
    v_cache = None if cfg.mla else torch.zeros(shape, dtype=cache_dt, device=dev)
    k_scale = v_scale = None
    if fp8:
        k_scale = ops.kv_head_scales(torch.cat([inp.k_ctx, inp.k_new]))
        v_scale = ops.kv_head_scales(torch.cat([inp.v_ctx, inp.v_new]))
    store = ops.quant_to_paged_cache if fp8 else ops.reshape_paged_cache
    ctx_slots = lay.ctx_slots.to(dev)
    new_slots = lay.new_slots.to(dev)
    store(ops.ReshapePagedCacheParams(key=inp.k_ctx, value=inp.v_ctx, k_cache=k_cache, v_cache=v_cache,
                                      slot_mapping=ctx_slots, k_cache_scale=k_scale, v_cache_scale=v_scale))
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
    reshape_args = (ptr(inp.k_new), ptr(inp.v_new), ptr(k_cache), ptr(v_cache), ptr(new_slots),
                    ptr(k_scale), ptr(v_scale), cfg.batch, cfg.n_kv_heads, cfg.head_dim, cfg.block_size,
                    lay.num_blocks, row, row, capi.BF16, code[cache_dt], stream)
    ws_bytes = lib.xllm_mi355_paged_decode_workspace_bytes(cfg.batch, cfg.n_q_heads, cfg.dv, max_len)
    ws = ops.decode_workspace(dev, ws_bytes)
    if cfg.mla:
        out = torch.empty(cfg.batch, 1, cfg.n_q_heads, cfg.v_dim, dtype=torch.bfloat16, device=dev)
        decode_fn = lib.xllm_mi355_paged_decode_mla
        decode_args = (ptr(mla.q_nope), ptr(mla.q_pe), ptr(k_cache), ptr(out), None, ptr(table),
                       table.stride(0), ptr(seq_lens), cfg.batch, cfg.n_q_heads, cfg.v_dim,
                       cfg.head_dim - cfg.v_dim, cfg.block_size, lay.num_blocks, max_len, cfg.scale,
                       ptr(ws), ws.numel(), capi.BF16, stream)
    else:
        decode_fn = lib.xllm_mi355_paged_decode_gqa
        decode_args = (ptr(inp.q), ptr(k_cache), ptr(v_cache), ptr(out), None, ptr(table),
                       table.stride(0), ptr(seq_lens), ptr(k_scale), ptr(v_scale), cfg.batch,
                       cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, lay.num_blocks,
                       inp.q.stride(0), out.stride(0), max_len, cfg.scale, ptr(ws), ws.numel(),
                       capi.BF16, code[cache_dt], stream)
    reshape_fn = lib.xllm_mi355_reshape_and_cache

    def step():
        rc = reshape_fn(*reshape_args)
        rc2 = decode_fn(*decode_args)
        if rc or rc2:
            capi.check(rc or rc2, "bench step")

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    capi.check(lib.xllm_mi355_profile_enable(args.steps), "profile_enable")
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    import ctypes
    ms = (ctypes.c_float * args.steps)()
    n = lib.xllm_mi355_profile_collect(ms, args.steps)
    kernel_ms = sum(ms[i] for i in range(n)) / max(n, 1)

    ms_per_step = elapsed / args.steps * 1e3
    tokens_per_s = cfg.batch / (ms_per_step * 1e-3)

    # ---- roofline of the dominant kernel (the decode kernel), from algorithmic work
    traffic = None
    try:
        with open(args.traffic_json) as f:
            traffic = json.load(f).get(args.workload, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        pass
    if cfg.mla and cfg.n_q_heads <= 64:
        # the few heads of a tensor-parallel shard: 30-120 flop per cache byte, far below the ridge: HBM bound
        nbytes, flops = workloads.mla_bytes_flops(cfg, lay.seq_lens)
        achieved = nbytes / (kernel_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "kernel": "mla_decode16_kernel",
                    "kernel_ms": kernel_ms, "algorithmic_bytes": nbytes, "algorithmic_flops": flops}
    elif cfg.mla:
        nbytes, flops = workloads.mla_bytes_flops(cfg, lay.seq_lens)
        achieved = flops / (kernel_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS,
                    "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic,
                    "kernel": "mla_decode16_kernel", "kernel_ms": kernel_ms, "algorithmic_flops": flops,
                    "algorithmic_bytes": nbytes,
                    "hbm_gbs": nbytes / (kernel_ms * 1e-3) / 1e9}
    else:
        nbytes = workloads.gqa_bytes(cfg, lay.seq_lens, 1 if fp8 else 2)
        achieved = nbytes / (kernel_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                    "kernel": ("gqa_mfma_kernel" if cfg.head_dim == 128 or (cfg.head_dim == 64 and cfg.cache_dtype != "fp8")
                               else "gqa_decode_kernel"),
                    "kernel_ms": kernel_ms, "algorithmic_bytes": nbytes}

    # the same number of bytes through the plain read kernel: the rate this GPU sustains at this size
    roofline["stream_read_gbs_same_bytes"], _ = stream_rate(lib, capi, torch, dev, nbytes)

    result = {
        "metric": "paged-decode tokens/s + achieved HBM GB/s (% of 8 TB/s) on 1 MI355X",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3 KV, bf16 Q/O, fp32 accumulate" if fp8 else "bf16 (fp32 accumulate)",
        "data": "synthetic",
        "config": {
            "workload": args.workload,
            "batch": cfg.batch, "n_q_heads": cfg.n_q_heads, "n_kv_heads": cfg.n_kv_heads,
            "head_dim": cfg.head_dim, "block_size": cfg.block_size,
            "context_tokens": int(lay.seq_lens.sum()), "max_context": max_len,
            "step": "reshape_and_cache(new K/V rows) + paged decode attention, inputs resident in HBM",
        },
        "hbm_gbs_whole_step": (nbytes + workloads.reshape_bytes(
            cfg.batch, cfg.n_kv_heads * cfg.head_dim, 2, 1 if fp8 else 2, 1 if cfg.mla else 2))
            / (ms_per_step * 1e-3) / 1e9,
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(inp, k_cache, v_cache, k_scale, v_scale, args.cpu_sample)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
