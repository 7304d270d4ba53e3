"""xllm_mi355_write_and_decode_gqa, the decode step of an attention layer in one call (the reference issues
reshape_paged_cache and then batch_decode per layer and step, layers/dcu/torch_attention.cpp:138-144 and :285-347),
against the two calls it replaces: same bytes in both caches, same output bits, same LSE.  The caches start with the
contexts' old tokens and a NaN pattern in every other slot, so a worker that attended to what the slot held before the
step (instead of the step's row) would show."""
import pytest
import torch

import oracle
from helpers import assert_close_to_reference
from xllm_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu

C = workloads.DecodeConfig
CASES = [
    # the matrix-core kernel writes the rows itself
    (C("w_llama", 24, 32, 8, 128, 16, 1, 3000), torch.bfloat16),
    (C("w_fp16", 9, 32, 8, 128, 16, 1, 900), torch.float16),
    (C("w_fp8", 12, 32, 8, 128, 16, 1, 2500, cache_dtype="fp8"), torch.bfloat16),
    (C("w_d64", 7, 16, 4, 64, 32, 1, 1500), torch.bfloat16),
    (C("w_d64_fp8", 7, 16, 4, 64, 32, 1, 1500, cache_dtype="fp8"), torch.bfloat16),
    (C("w_d256", 6, 8, 2, 256, 32, 1, 1200), torch.bfloat16),
    (C("w_d256_fp8", 4, 8, 2, 256, 32, 1, 900, cache_dtype="fp8"), torch.bfloat16),
    (C("w_group32", 5, 64, 2, 128, 16, 1, 2000), torch.bfloat16),     # two head blocks per KV head store the same row
    (C("w_bs128", 10, 64, 8, 128, 128, 1, 4000), torch.bfloat16),
    (C("w_long", 3, 32, 8, 128, 16, 20000, 40000), torch.bfloat16),   # contexts cut over many workers
    # served by the other kernels: the library issues the two launches itself
    (C("w_bs8", 6, 32, 8, 128, 8, 1, 700), torch.bfloat16),
    (C("w_bs24_fp8", 4, 8, 2, 128, 24, 1, 900, cache_dtype="fp8"), torch.bfloat16),
]


def _caches_before_the_step(inp, device, fp8, dtype):
    """Caches that hold the contexts' earlier tokens; all other slots (the step's among them) hold NaNs."""
    cfg, lay = inp.cfg, inp.layout
    shape = (lay.num_blocks, cfg.block_size, cfg.n_kv_heads, cfg.head_dim)
    if fp8:
        kc = torch.full(shape, 0x7F, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
        vc = torch.full(shape, 0x7F, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
        ks = ops.kv_head_scales(torch.cat([inp.k_ctx, inp.k_new]).to(device))
        vs = ops.kv_head_scales(torch.cat([inp.v_ctx, inp.v_new]).to(device))
        fn = ops.quant_to_paged_cache
    else:
        kc = torch.full(shape, float("nan"), dtype=dtype, device=device)
        vc = torch.full(shape, float("nan"), dtype=dtype, device=device)
        ks = vs = None
        fn = ops.reshape_paged_cache
    if inp.k_ctx.shape[0] > 0:
        fn(ops.ReshapePagedCacheParams(key=inp.k_ctx.to(device), value=inp.v_ctx.to(device), k_cache=kc, v_cache=vc,
                                       slot_mapping=lay.ctx_slots.to(device), k_cache_scale=ks, v_cache_scale=vs))
    return kc, vc, ks, vs, fn


def _bits(t):
    return t.view(torch.uint8) if t.element_size() == 1 else t.view(torch.int16)


@pytest.mark.parametrize("cfg,dtype", CASES, ids=[c.name for c, _ in CASES])
@pytest.mark.parametrize("planned", [False, True], ids=["unplanned", "planned"])
def test_one_call_equals_store_then_decode(device, cfg, dtype, planned):
    inp = workloads.make_inputs(cfg, 900 + len(cfg.name), dtype=dtype)
    lay = inp.layout
    fp8 = cfg.cache_dtype == "fp8"
    kc0, vc0, ks, vs, store = _caches_before_the_step(inp, device, fp8, dtype)
    q = inp.q.to(device)
    k_new, v_new = inp.k_new.to(device), inp.v_new.to(device)
    slots = lay.new_slots.to(device).clone()
    skipped = -1
    if cfg.batch >= 5:   # one sequence's row is not stored (a padded entry of the slot mapping)
        skipped = 2
        slots[skipped] = -1
    table, lens = lay.block_table.to(device), lay.seq_lens.to(device)
    plan = None
    if planned:
        plan = ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, kc0.dtype,
                                           block_table=table, seq_lens=lens)

    # the pair
    kc_a, vc_a = kc0.clone(), vc0.clone()
    store(ops.ReshapePagedCacheParams(key=k_new, value=v_new, k_cache=kc_a, v_cache=vc_a, slot_mapping=slots,
                                      k_cache_scale=ks, v_cache_scale=vs))
    out_a, lse_a = ops.batch_decode(q, kc_a, torch.full_like(q, float("nan")), table, lens, v_cache=vc_a,
                                    k_cache_quant_scale=ks, v_cache_quant_scale=vs, scale=cfg.scale, return_lse=True,
                                    plan=plan)
    # the one call
    kc_b, vc_b = kc0.clone(), vc0.clone()
    out_b, lse_b = ops.batch_decode(q, kc_b, torch.full_like(q, float("nan")), table, lens, v_cache=vc_b,
                                    k_cache_quant_scale=ks, v_cache_quant_scale=vs, scale=cfg.scale, return_lse=True,
                                    plan=plan, new_key=k_new, new_value=v_new, slot_mapping=slots)
    torch.cuda.synchronize()
    ops.decode_status(device)
    assert torch.equal(_bits(kc_a), _bits(kc_b)), "K cache bytes differ"
    assert torch.equal(_bits(vc_a), _bits(vc_b)), "V cache bytes differ"
    live = torch.ones(cfg.batch, dtype=torch.bool, device=device)
    if skipped >= 0:
        live[skipped] = False   # attends to a NaN row in both forms
    assert torch.equal(_bits(out_a[live]), _bits(out_b[live]))
    assert torch.equal(lse_a[live], lse_b[live])
    assert torch.isfinite(out_b[live].float()).all()
    # and the pair is the reference's result
    ref = oracle.aten_paged_decode(inp.q[live.cpu()], kc_a.cpu(), vc_a.cpu(), lay.block_table[live.cpu()],
                                   lay.seq_lens[live.cpu()], cfg.scale, None if ks is None else ks.cpu(),
                                   None if vs is None else vs.cpu())
    assert_close_to_reference(out_b[live], ref, cfg.name)


def test_one_call_with_csr_addressing_and_strided_rows(device):
    """Through the C ABI: CSR page lists, and key / value rows that are slices of a fused QKV projection (token stride
    above Hkv * D)."""
    lib = capi.lib()
    cfg = C("w_csr", 11, 32, 8, 128, 16, 1, 1800)
    inp = workloads.make_inputs(cfg, 77)
    lay = inp.layout
    kc0, vc0, _, _, _ = _caches_before_the_step(inp, device, False, torch.bfloat16)
    q = inp.q.to(device)
    Hq, Hkv, D = cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim
    qkv = torch.randn(cfg.batch, (Hq + 2 * Hkv) * D, device=device).to(torch.bfloat16)
    qkv[:, Hq * D:(Hq + Hkv) * D] = inp.k_new.to(device).view(cfg.batch, -1)
    qkv[:, (Hq + Hkv) * D:] = inp.v_new.to(device).view(cfg.batch, -1)
    k_new = qkv[:, Hq * D:(Hq + Hkv) * D].view(cfg.batch, Hkv, D)
    v_new = qkv[:, (Hq + Hkv) * D:].view(cfg.batch, Hkv, D)
    slots = lay.new_slots.to(device)
    n_pages = (lay.seq_lens + cfg.block_size - 1) // cfg.block_size
    indptr = torch.zeros(cfg.batch + 1, dtype=torch.int32)
    indptr[1:] = torch.cumsum(n_pages, 0)
    indices = torch.cat([lay.block_table[b, :int(n_pages[b])] for b in range(cfg.batch)]).to(torch.int32)
    last = (lay.seq_lens - (n_pages - 1) * cfg.block_size).to(torch.int32)
    indptr, indices, last = indptr.to(device), indices.to(device), last.to(device)
    ws = ops.decode_workspace(device, lib.xllm_mi355_paged_decode_gqa_workspace_bytes(cfg.batch, Hq, D))
    stream = torch.cuda.current_stream(device).cuda_stream

    kc_a, vc_a = kc0.clone(), vc0.clone()
    ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=k_new, value=v_new, k_cache=kc_a, v_cache=vc_a,
                                                        slot_mapping=slots))
    out_a = torch.full_like(q, float("nan"))
    ops.batch_decode_csr(q, kc_a, vc_a, indptr, indices, last, -1, cfg.scale, out_a)
    kc_b, vc_b = kc0.clone(), vc0.clone()
    out_b = torch.full_like(q, float("nan"))
    rc = lib.xllm_mi355_write_and_decode_gqa(
        k_new.data_ptr(), v_new.data_ptr(), slots.data_ptr(), k_new.stride(0), v_new.stride(0), None, 0, q.data_ptr(),
        kc_b.data_ptr(), vc_b.data_ptr(), out_b.data_ptr(), None, None, 0, None, indptr.data_ptr(), indices.data_ptr(),
        last.data_ptr(), None, None, cfg.batch, Hq, Hkv, D, cfg.block_size, lay.num_blocks, q.stride(0),
        out_b.stride(0), int(lay.seq_lens.max()), -1, cfg.scale, ws.data_ptr(), ws.numel(), capi.BF16, capi.BF16, stream)
    capi.check(rc, "write_and_decode")
    torch.cuda.synchronize()
    assert torch.equal(_bits(kc_a), _bits(kc_b)) and torch.equal(_bits(vc_a), _bits(vc_b))
    assert torch.equal(_bits(out_a), _bits(out_b))
    assert torch.isfinite(out_b.float()).all()


def _pair_and_one_call(inp, device, dtype, fp8, slots, **kw):
    cfg, lay = inp.cfg, inp.layout
    kc0, vc0, ks, vs, store = _caches_before_the_step(inp, device, fp8, dtype)
    q = inp.q.to(device)
    k_new, v_new = inp.k_new.to(device), inp.v_new.to(device)
    table, lens = lay.block_table.to(device), lay.seq_lens.to(device)
    kc_a, vc_a = kc0.clone(), vc0.clone()
    store(ops.ReshapePagedCacheParams(key=k_new, value=v_new, k_cache=kc_a, v_cache=vc_a, slot_mapping=slots,
                                      k_cache_scale=ks, v_cache_scale=vs))
    out_a, lse_a = ops.batch_decode(q, kc_a, torch.full_like(q, float("nan")), table, lens, v_cache=vc_a,
                                    k_cache_quant_scale=ks, v_cache_quant_scale=vs, scale=cfg.scale, return_lse=True, **kw)
    kc_b, vc_b = kc0.clone(), vc0.clone()
    out_b, lse_b = ops.batch_decode(q, kc_b, torch.full_like(q, float("nan")), table, lens, v_cache=vc_b,
                                    k_cache_quant_scale=ks, v_cache_quant_scale=vs, scale=cfg.scale, return_lse=True,
                                    new_key=k_new, new_value=v_new, slot_mapping=slots, **kw)
    torch.cuda.synchronize()
    ops.decode_status(device)
    assert torch.equal(_bits(kc_a), _bits(kc_b)) and torch.equal(_bits(vc_a), _bits(vc_b)), cfg.name
    return out_a, lse_a, out_b, lse_b


def test_one_call_with_a_sliding_window_fp16_over_fp8_and_slots_beyond_the_cache(device):
    # a window (the first scheduled stage of a context is not its first)
    cfg = C("w_window", 9, 32, 8, 128, 16, 1, 2500)
    inp = workloads.make_inputs(cfg, 31)
    slots = inp.layout.new_slots.to(device)
    out_a, lse_a, out_b, lse_b = _pair_and_one_call(inp, device, torch.bfloat16, False, slots, window_left=300)
    assert torch.equal(_bits(out_a), _bits(out_b)) and torch.equal(lse_a, lse_b)
    assert torch.isfinite(out_b.float()).all()
    # an fp16 query over fp8 pages: the rows are quantised from fp16 inside the decode launch
    cfg = C("w_fp16_fp8", 7, 16, 4, 128, 32, 1, 1800, cache_dtype="fp8")
    inp = workloads.make_inputs(cfg, 32, dtype=torch.float16)
    slots = inp.layout.new_slots.to(device)
    out_a, lse_a, out_b, lse_b = _pair_and_one_call(inp, device, torch.float16, True, slots)
    assert torch.equal(_bits(out_a), _bits(out_b)) and torch.equal(lse_a, lse_b)
    assert torch.isfinite(out_b.float()).all()
    # a slot beyond the cache is skipped like a negative one (the caches stay equal; that sequence attends to the NaN row)
    cfg = C("w_beyond", 6, 32, 8, 128, 16, 20, 900)
    inp = workloads.make_inputs(cfg, 33)
    slots = inp.layout.new_slots.to(device).clone()
    slots[4] = inp.layout.num_blocks * cfg.block_size + 5
    out_a, lse_a, out_b, lse_b = _pair_and_one_call(inp, device, torch.bfloat16, False, slots)
    live = torch.ones(cfg.batch, dtype=torch.bool, device=device)
    live[4] = False
    assert torch.equal(_bits(out_a[live]), _bits(out_b[live])) and torch.equal(lse_a[live], lse_b[live])
    assert torch.isfinite(out_b[live].float()).all()


def test_one_call_on_a_batch_decoded_in_slices(device):
    # more sequences than one launch takes: every slice stores the rows of its own sequences
    cfg = C("w_slices", 2100, 4, 1, 128, 16, 1, 40)
    inp = workloads.make_inputs(cfg, 34)
    slots = inp.layout.new_slots.to(device)
    out_a, lse_a, out_b, lse_b = _pair_and_one_call(inp, device, torch.bfloat16, False, slots)
    assert torch.equal(_bits(out_a), _bits(out_b)) and torch.equal(lse_a, lse_b)
    assert torch.isfinite(out_b.float()).all()


def test_one_call_rejects_missing_rows(device):
    lib = capi.lib()
    fake = 1 << 20
    rc = lib.xllm_mi355_write_and_decode_gqa(
        None, fake, fake, 1024, 1024, None, 0, fake, fake, fake, fake, None, fake, 8, fake, None, None, None, None, None,
        4, 32, 8, 128, 16, 100, 4096, 4096, 100, -1, 0.1, fake, 1 << 30, capi.BF16, capi.BF16, None)
    assert rc == -1
    # rows narrower than Hkv * D
    rc = lib.xllm_mi355_write_and_decode_gqa(
        fake, fake, fake, 512, 1024, None, 0, fake, fake, fake, fake, None, fake, 8, fake, None, None, None, None, None,
        4, 32, 8, 128, 16, 100, 4096, 4096, 100, -1, 0.1, fake, 1 << 30, capi.BF16, capi.BF16, None)
    assert rc == -1
    # an undersized plan
    rc = lib.xllm_mi355_write_and_decode_gqa(
        fake, fake, fake, 1024, 1024, fake, 4096, fake, fake, fake, fake, None, fake, 8, fake, None, None, None, None,
        None, 4, 32, 8, 128, 16, 100, 4096, 4096, 100, -1, 0.1, fake, 1 << 30, capi.BF16, capi.BF16, None)
    assert rc == -4


# ---- the MLA layer's step: store_latent_cache + decode_flash_mla (layers/dcu/deepseek_v2_attention.cpp:221-229,
# :242-263) in one call, against the two calls

def _mla_cfg(name, batch, heads, lo, hi, bs=64):
    import math
    return C(name, batch, heads, 1, 576, bs, lo, hi, mla=True, v_dim=512, sigma=0.5, sm_scale=1.0 / math.sqrt(192.0))


MLA_CASES = [
    # mla_decode_w4_kernel stores the rows itself
    (_mla_cfg("m_128", 6, 128, 1, 3000), torch.bfloat16),
    (_mla_cfg("m_128_fp16", 4, 128, 1, 2000), torch.float16),
    (_mla_cfg("m_80_bs16", 5, 80, 1, 1500, bs=16), torch.bfloat16),
    (_mla_cfg("m_256", 3, 256, 1, 2500), torch.bfloat16),          # two workgroups per team store the same row
    (_mla_cfg("m_long", 2, 128, 30000, 50000), torch.bfloat16),    # contexts cut over many workgroups
    (_mla_cfg("m_many", 300, 128, 1, 90), torch.bfloat16),         # several whole contexts per workgroup
    # the other kernels: the library issues the two launches itself
    (_mla_cfg("m_16", 6, 16, 1, 1200), torch.bfloat16),
    (_mla_cfg("m_bs24", 4, 128, 1, 900, bs=24), torch.bfloat16),
]


@pytest.mark.parametrize("cfg,dtype", MLA_CASES, ids=[c.name for c, _ in MLA_CASES])
@pytest.mark.parametrize("planned", [False, True], ids=["unplanned", "planned"])
def test_mla_one_call_equals_store_then_decode(device, cfg, dtype, planned):
    inp = workloads.make_inputs(cfg, 700 + len(cfg.name), dtype=dtype)
    lay = inp.layout
    B, H = cfg.batch, cfg.n_q_heads
    shape = (lay.num_blocks, cfg.block_size, 1, cfg.head_dim)
    kc0 = torch.full(shape, float("nan"), dtype=dtype, device=device)
    if inp.k_ctx.shape[0] > 0:
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=inp.k_ctx.to(device), value=None, k_cache=kc0, v_cache=None,
                                                            slot_mapping=lay.ctx_slots.to(device)))
    # the step's rows as a slice of a wider buffer (the layer's kv_a projection output), 16-byte aligned rows
    wide = torch.zeros(B, cfg.head_dim + 64, dtype=dtype, device=device)
    wide[:, : cfg.head_dim] = inp.k_new.to(device).view(B, cfg.head_dim)
    latent = wide[:, : cfg.head_dim]
    slots = lay.new_slots.to(device).clone()
    skipped = -1
    if B >= 5:
        skipped = 1
        slots[skipped] = -1
    q = inp.q.to(device)
    table, lens = lay.block_table.to(device), lay.seq_lens.to(device)

    def params(kc):
        return ops.DenseDecodeParams(q_nope=q[:, :, : cfg.v_dim].contiguous().view(B, 1, H, cfg.v_dim),
                                     q_pe=q[:, :, cfg.v_dim:].contiguous().view(B, 1, H, cfg.head_dim - cfg.v_dim),
                                     k_cache=kc, seqlens_k=lens, block_table=table, head_size_v=cfg.v_dim,
                                     softmax_scale=cfg.scale)
    plan = ops.get_mla_decoding_metadata(lens, table, H, cfg.block_size) if planned else None
    kc_a = kc0.clone()
    ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=latent.unsqueeze(1), value=None, k_cache=kc_a, v_cache=None,
                                                        slot_mapping=slots))
    out_a, lse_a = ops.dense_decode(params(kc_a), return_lse=True, metadata=plan)
    kc_b = kc0.clone()
    out_b, lse_b = ops.dense_decode(params(kc_b), return_lse=True, metadata=plan, new_latent=latent, slot_mapping=slots)
    torch.cuda.synchronize()
    ops.decode_status(device)
    assert torch.equal(_bits(kc_a), _bits(kc_b)), "latent cache bytes differ"
    live = torch.ones(B, dtype=torch.bool, device=device)
    if skipped >= 0:
        live[skipped] = False
    assert torch.equal(_bits(out_a[live]), _bits(out_b[live]))
    assert torch.equal(lse_a[live], lse_b[live])
    assert torch.isfinite(out_b[live].float()).all()
    if cfg.name != "m_long":   # (the CPU checker on 80 000 tokens of 128 heads takes minutes; the pair is checked elsewhere)
        lc = live.cpu()
        ref = oracle.aten_paged_decode(inp.q[lc], kc_a.cpu(), None, lay.block_table[lc], lay.seq_lens[lc], cfg.scale,
                                       dv=cfg.v_dim)
        assert_close_to_reference(out_b[live].view(-1, H, cfg.v_dim), ref, cfg.name)


def test_mla_one_call_rejects_missing_rows(device):
    lib = capi.lib()
    fake = 1 << 20
    tail = (fake, fake, fake, fake, None, fake, 8, fake, 4, 128, 512, 64, 64, 100, 4096, 0.1, fake, 1 << 30, capi.BF16, None)
    assert lib.xllm_mi355_write_and_decode_mla(None, fake, 576, None, 0, *tail) == -1
    assert lib.xllm_mi355_write_and_decode_mla(fake, fake, 512, None, 0, *tail) == -1      # rows narrower than 576
    assert lib.xllm_mi355_write_and_decode_mla(fake, fake, 576, fake, 4096, *tail) == -4   # an undersized plan


def test_one_call_on_random_shapes(device):
    """Random head counts, head dims, block sizes, page types, batch sizes and lengths (lengths around the stage
    boundaries included): the one call and the pair leave the same bytes everywhere."""
    g = torch.Generator().manual_seed(2024)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))

    for case in range(14):
        D = [64, 128, 128, 256][ri(0, 3)]
        fp8 = ri(0, 2) == 0
        Hkv = [1, 2, 3, 4, 8][ri(0, 4)]
        Hq = Hkv * [1, 2, 4, 5, 8, 16, 20][ri(0, 6)]
        bs = [8, 16, 32, 64, 128][ri(0, 4)]
        batch = [1, 2, 7, 33, 64, 130][ri(0, 5)]
        hi = [17, 70, 600, 3000][ri(0, 3)]
        if batch * hi * Hkv * D > 4e8:
            batch = max(1, batch // 8)
        dtype = torch.float16 if ri(0, 3) == 0 else torch.bfloat16
        cfg = C(f"w_rand{case}", batch, Hq, Hkv, D, bs, 1, hi, cache_dtype="fp8" if fp8 else "bf16")
        inp = workloads.make_inputs(cfg, 5000 + case, dtype=dtype)
        slots = inp.layout.new_slots.to(device).clone()
        dead = None
        if batch > 2 and ri(0, 1) == 0:
            dead = ri(0, batch - 1)
            slots[dead] = -1
        out_a, lse_a, out_b, lse_b = _pair_and_one_call(inp, device, dtype, fp8, slots)
        live = torch.ones(batch, dtype=torch.bool, device=device)
        if dead is not None:
            live[dead] = False
        what = f"{cfg.name}: Hq {Hq} Hkv {Hkv} D {D} bs {bs} fp8 {fp8} batch {batch} hi {hi} {dtype}"
        assert torch.equal(_bits(out_a[live]), _bits(out_b[live])), what
        assert torch.equal(lse_a[live], lse_b[live]), what
        assert torch.isfinite(out_b[live].float()).all(), what
