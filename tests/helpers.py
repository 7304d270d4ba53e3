"""Shared pieces of the parity tests: run the GPU path and the CPU checker on the same bytes."""
import torch

import oracle
from xllm_amd import ops, workloads

# Tolerance of the attention output against the reference's libtorch CPU path, in bf16.
MAX_ABS_TOL = 2e-2
MEAN_ABS_TOL = 2e-3


def fill_caches_gpu(inp, device, cache_dtype=None, pad_pages=0):
    """Write the context rows, then this step's rows, through the op under test."""
    cfg, lay = inp.cfg, inp.layout
    dt = cache_dtype or inp.k_ctx.dtype
    shape = (lay.num_blocks, cfg.block_size, cfg.n_kv_heads, cfg.head_dim)
    k_cache = torch.zeros(shape, dtype=dt, device=device)
    v_cache = None if cfg.mla else torch.zeros(shape, dtype=dt, device=device)
    k_scale = v_scale = None
    quant = dt in (torch.float8_e4m3fn, torch.uint8)
    if quant:
        k_scale = ops.kv_head_scales(torch.cat([inp.k_ctx, inp.k_new]).to(device))
        v_scale = ops.kv_head_scales(torch.cat([inp.v_ctx, inp.v_new]).to(device))
    fn = ops.quant_to_paged_cache if quant else ops.reshape_paged_cache
    for k, v, slots in ((inp.k_ctx, inp.v_ctx, lay.ctx_slots), (inp.k_new, inp.v_new, lay.new_slots)):
        if k.shape[0] == 0:
            continue
        fn(ops.ReshapePagedCacheParams(
            key=k.to(device), value=None if v is None else v.to(device), k_cache=k_cache,
            v_cache=v_cache, slot_mapping=slots.to(device), k_cache_scale=k_scale, v_cache_scale=v_scale))
    return k_cache, v_cache, k_scale, v_scale


def fill_caches_cpu(inp, cache_dtype=None, k_scale=None, v_scale=None):
    cfg, lay = inp.cfg, inp.layout
    dt = cache_dtype or inp.k_ctx.dtype
    shape = (lay.num_blocks, cfg.block_size, cfg.n_kv_heads, cfg.head_dim)
    store_dt = torch.uint8 if dt in (torch.float8_e4m3fn, torch.uint8) else dt
    k_cache = torch.zeros(shape, dtype=store_dt)
    v_cache = None if cfg.mla else torch.zeros(shape, dtype=store_dt)
    for k, v, slots in ((inp.k_ctx, inp.v_ctx, lay.ctx_slots), (inp.k_new, inp.v_new, lay.new_slots)):
        if k.shape[0] == 0:
            continue
        oracle.reshape_and_cache(k.cpu(), None if v is None else v.cpu(), k_cache, v_cache, slots.cpu(),
                                 k_scale, v_scale)
    return k_cache, v_cache


def assert_close_to_reference(actual, expected, what=""):
    a = actual.detach().float().cpu()
    e = expected.detach().float().cpu()
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    assert torch.isfinite(a).all(), f"{what}: non-finite output"
    diff = (a - e).abs()
    mx, mean = diff.max().item(), diff.mean().item()
    assert mx <= MAX_ABS_TOL and mean <= MEAN_ABS_TOL, f"{what}: max-abs {mx:.3e}, mean-abs {mean:.3e}"
    return mx, mean


def trimmed_context(k_cache, v_cache, block_table, seq_lens, first_tokens):
    """The paged caches of the contexts cut to their tokens [first_tokens[b], seq_lens[b]): new caches whose pages
    hold those rows from row 0 on, with their table and lengths.  The block-table oracle on this layout is the
    reference of a sliding-window decode."""
    P, bs = k_cache.shape[0], k_cache.shape[1]
    B = seq_lens.numel()
    kf = k_cache.reshape(P * bs, *k_cache.shape[2:])
    vf = None if v_cache is None else v_cache.reshape(P * bs, *v_cache.shape[2:])
    new_lens = (seq_lens - first_tokens).to(torch.int32)
    n_pages = (new_lens.long() + bs - 1) // bs
    total = int(n_pages.sum())
    nk = torch.zeros(total * bs, *k_cache.shape[2:], dtype=k_cache.dtype)
    nv = None if v_cache is None else torch.zeros_like(nk)
    table = torch.zeros(B, max(1, int(n_pages.max())), dtype=torch.int32)
    page = 0
    for b in range(B):
        t = torch.arange(int(first_tokens[b]), int(seq_lens[b]))
        slots = block_table[b, t // bs].long() * bs + t % bs
        n = t.numel()
        nk[page * bs : page * bs + n] = kf[slots]
        if nv is not None:
            nv[page * bs : page * bs + n] = vf[slots]
        table[b, : int(n_pages[b])] = torch.arange(page, page + int(n_pages[b]), dtype=torch.int32)
        page += int(n_pages[b])
    shape = (total, bs, *k_cache.shape[2:])
    return nk.view(shape), None if nv is None else nv.view(shape), table, new_lens
