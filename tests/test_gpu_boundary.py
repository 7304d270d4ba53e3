"""The parts of the reference's interface either side of the two ops, through the C ABI and the C++ host side: sliding
window, the base-2 two-way combine, multi-token and fp16 MLA decode, and the layer-level write-then-attend call."""
import math

import pytest
import torch

import oracle
from helpers import assert_close_to_reference, fill_caches_cpu, fill_caches_gpu, trimmed_context
from xllm_amd import ops, torch_ops, workloads

pytestmark = pytest.mark.gpu


def _window_reference(inp, kc, vc, window, ks=None, vs=None):
    lay, cfg = inp.layout, inp.cfg
    first = (lay.seq_lens - 1 - window).clamp_min(0)
    nk, nv, table, lens = trimmed_context(kc, vc, lay.block_table, lay.seq_lens, first)
    return oracle.aten_paged_decode(inp.q, nk, nv, table, lens, cfg.scale, ks, vs)


@pytest.mark.parametrize("bs", [16, 128])
def test_sliding_window_skips_pages_before_the_window_and_masks_its_first_stage(device, bs):
    # windows shorter than a stage, not aligned to stages or pages, longer than some contexts, and none
    cfg = workloads.DecodeConfig(f"win_bs{bs}", 9, 32, 8, 128, bs, 40, 3000)
    inp = workloads.make_inputs(cfg, 50 + bs)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    kc, vc = kg.cpu(), vg.cpu()
    q = inp.q.to(device)
    table, lens = lay.block_table.to(device), lay.seq_lens.to(device)
    for window in (0, 5, 15, 16, 100, 1000, 1023, 1024, 5000):
        out = torch.empty_like(q)
        out, lse = ops.batch_decode(q, kg, out, table, lens, v_cache=vg, scale=cfg.scale, return_lse=True,
                                    window_left=window)
        torch.cuda.synchronize()
        assert_close_to_reference(out, _window_reference(inp, kc, vc, window), f"window {window}")
        # CSR addressing, same window
        out_c = torch.empty_like(q)
        ops.batch_decode_csr(q, kg, vg, lay.indptr.to(device), lay.indices.to(device), lay.last_page_len.to(device),
                             window, cfg.scale, out_c)
        assert torch.equal(out_c, out)
    out = torch.empty_like(q)
    ops.batch_decode(q, kg, out, table, lens, v_cache=vg, scale=cfg.scale, window_left=-1)
    ref = oracle.aten_paged_decode(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale)
    assert_close_to_reference(out, ref, "no window")


def test_sliding_window_fp8_pages_other_kernels_and_query_chunks(device):
    # fp8 pages (32-token stages) on the matrix-core kernel
    cfg = workloads.DecodeConfig("win_fp8", 5, 32, 8, 128, 16, 100, 2500, cache_dtype="fp8")
    inp = workloads.make_inputs(cfg, 61)
    lay = inp.layout
    kg, vg, ks, vs = fill_caches_gpu(inp, device, cache_dtype=torch.float8_e4m3fn)
    q = inp.q.to(device)
    for window in (7, 31, 32, 700):
        out = torch.empty_like(q)
        ops.batch_decode(q, kg, out, lay.block_table.to(device), lay.seq_lens.to(device), v_cache=vg,
                         k_cache_quant_scale=ks, v_cache_quant_scale=vs, scale=cfg.scale, window_left=window)
        ref = _window_reference(inp, kg.cpu(), vg.cpu(), window, ks.cpu(), vs.cpu())
        assert_close_to_reference(out, ref, f"fp8 window {window}")
    # the dot-product kernel (block size 8) and head dims 64 and 256
    for D, Hq, Hkv, blk in ((128, 8, 2, 8), (64, 16, 4, 16), (256, 8, 2, 32)):
        cfg = workloads.DecodeConfig(f"win_d{D}", 4, Hq, Hkv, D, blk, 30, 1500)
        inp = workloads.make_inputs(cfg, 62 + D)
        lay = inp.layout
        kg, vg, _, _ = fill_caches_gpu(inp, device)
        q = inp.q.to(device)
        for window in (3, 64, 65, 400):
            out = torch.empty_like(q)
            ops.batch_decode(q, kg, out, lay.block_table.to(device), lay.seq_lens.to(device), v_cache=vg,
                             scale=cfg.scale, window_left=window)
            assert_close_to_reference(out, _window_reference(inp, kg.cpu(), vg.cpu(), window), f"D{D} window {window}")
    # query chunks: every token's window counts from its own position
    cfg = workloads.DecodeConfig("win_chunks", 4, 16, 4, 128, 16, 200, 900)
    inp = workloads.make_inputs(cfg, 63)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    q_lens = torch.tensor([3, 1, 5, 2])
    cu = torch.zeros(5, dtype=torch.int32)
    cu[1:] = torch.cumsum(q_lens, 0)
    T = int(cu[-1])
    qq = workloads.randn_16bit((T, cfg.n_q_heads, cfg.head_dim), 1.0, torch.Generator().manual_seed(9), "cpu")
    window = 150
    out = torch.empty(T, cfg.n_q_heads, cfg.head_dim, dtype=torch.bfloat16, device=device)
    ops.paged_forward(qq.to(device), out, kg, vg, lay.block_table.to(device), lay.seq_lens.to(device), cu.to(device),
                      scale=cfg.scale, is_causal=True, max_query_len=5, window_left=window)
    kc, vc = kg.cpu(), vg.cpu()
    for b in range(cfg.batch):
        for j in range(int(q_lens[b])):
            L = int(lay.seq_lens[b]) - int(q_lens[b]) + j + 1
            first = max(0, L - 1 - window)
            nk, nv, table, lens = trimmed_context(kc, vc, lay.block_table[b : b + 1], torch.tensor([L], dtype=torch.int32),
                                                  torch.tensor([first]))
            t = int(cu[b]) + j
            ref = oracle.aten_paged_decode(qq[t : t + 1].contiguous(), nk, nv, table, lens, cfg.scale)
            assert_close_to_reference(out[t : t + 1], ref, f"chunk token {b}/{j}")


def test_base2_two_way_combine(device):
    ln2 = math.log(2.0)
    # the reference's known answers of the natural-log merge (dcp_attention_merge_test.cpp:34-63), LSEs in base 2
    a = torch.tensor([[[2.0, 4.0]]], device=device)
    b = torch.tensor([[[6.0, 8.0]]], device=device)
    la = torch.tensor([[[math.log(2.0) / ln2]]], device=device)
    lb = torch.tensor([[[math.log(6.0) / ln2]]], device=device)
    out = ops.lse_combine(None, a, la, b, lb)
    assert torch.allclose(out.cpu(), torch.tensor([[[5.0, 7.0]]]), atol=1e-6)
    out = ops.lse_combine(None, torch.zeros_like(a), torch.full_like(la, -math.inf), torch.tensor([[[3.0, 9.0]]], device=device),
                          torch.full_like(lb, 2.0))
    assert torch.equal(out.cpu(), torch.tensor([[[3.0, 9.0]]]))
    # random inputs of every type against the C oracle, through the Python mirror and the C++ host side
    xops = torch_ops.load()
    g = torch.Generator().manual_seed(12)
    for dt, tol in ((torch.float32, 2e-6), (torch.bfloat16, 8e-3), (torch.float16, 1e-3)):
        so, uo = torch.randn(7, 12, 128, generator=g).to(dt), torch.randn(7, 12, 128, generator=g).to(dt)
        sl, ul = torch.randn(7, 12, 1, generator=g) * 5, torch.randn(7, 12, 1, generator=g) * 5
        ref, _ = oracle.lse_combine(so, sl, uo, ul)
        got = ops.lse_combine(None, so.to(device), sl.to(device), uo.to(device), ul.to(device))
        assert got.dtype == dt and torch.allclose(got.float().cpu(), ref, rtol=tol, atol=tol)
        via_shim = torch.empty_like(got)
        xops.lse_combine(via_shim, so.to(device), sl.to(device), uo.to(device), ul.to(device))
        assert torch.equal(via_shim, got)
    # decode halves merged in base 2 equal the full decode
    cfg = workloads.DecodeConfig("combine", 3, 8, 2, 128, 16, 200, 900)
    inp = workloads.make_inputs(cfg, 13)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    q = inp.q.to(device)
    full = torch.empty_like(q)
    ops.batch_decode(q, kg, full, lay.block_table.to(device), lay.seq_lens.to(device), v_cache=vg, scale=cfg.scale)
    half = (lay.seq_lens // 32) * 16
    o1, o2 = torch.empty_like(q), torch.empty_like(q)
    _, l1 = ops.batch_decode(q, kg, o1, lay.block_table.to(device), half.to(device), v_cache=vg, scale=cfg.scale, return_lse=True)
    table2 = torch.zeros_like(lay.block_table)
    for b in range(cfg.batch):
        n = int(half[b]) // 16
        rest = lay.block_table.shape[1] - n
        table2[b, :rest] = lay.block_table[b, n:]
    _, l2 = ops.batch_decode(q, kg, o2, table2.to(device), (lay.seq_lens - half).to(device), v_cache=vg, scale=cfg.scale,
                             return_lse=True)
    merged = ops.lse_combine(None, o1, l1 / ln2, o2, l2 / ln2)
    assert (merged.float() - full.float()).abs().max() <= 1e-2


def _mla_inputs(batch, heads, lo, hi, seed, dtype=torch.bfloat16, bs=64):
    cfg = workloads.DecodeConfig("mla", batch, heads, 1, 576, bs, lo, hi, mla=True, v_dim=512, sigma=0.5,
                                 sm_scale=1.0 / math.sqrt(192.0))
    inp = workloads.make_inputs(cfg, seed, dtype=dtype)
    return cfg, inp


def test_mla_multi_token_steps_fold_into_heads_and_the_causal_form(device):
    # S_q = 3 query tokens per sequence against the same pages (a multi-token speculative step)
    B, Sq, H = 3, 3, 16
    cfg, inp = _mla_inputs(B, Sq * H, 150, 1200, 21)
    lay = inp.layout
    kg, _, _, _ = fill_caches_gpu(inp, device)
    kc = kg.cpu()
    q = inp.q.to(device).view(B, Sq, H, 576)
    for causal in (False, True):
        p = ops.DenseDecodeParams(q_nope=q[..., :512], q_pe=q[..., 512:], k_cache=kg, seqlens_k=lay.seq_lens.to(device),
                                  block_table=lay.block_table.to(device), head_size_v=512, softmax_scale=cfg.scale,
                                  is_causal=causal, kind=ops.DenseDecodeKind.kQNopePe)
        out, lse = ops.dense_decode(p, return_lse=True)
        assert out.shape == (B, Sq, H, 512) and lse.shape == (B, H, Sq)
        for j in range(Sq):
            lens = lay.seq_lens - (Sq - 1 - j) if causal else lay.seq_lens
            qj = inp.q.view(B, Sq, H, 576)[:, j].contiguous()
            ref = oracle.aten_paged_decode(qj, kc, None, lay.block_table, lens.contiguous(), cfg.scale, dv=512)
            assert_close_to_reference(out[:, j], ref, f"S_q token {j} causal {causal}")
            ref_lse = oracle.aten_paged_decode_lse(qj, kc, lay.block_table, lens.contiguous(), cfg.scale)
            assert torch.allclose(lse[:, :, j].cpu(), ref_lse, rtol=1e-3, atol=1e-3)
        # the C++ host side returns the same
        xops = torch_ops.load()
        out2, lse2 = xops.mla_dense_decode(p.q_nope, p.q_pe, kg, p.seqlens_k, p.block_table, 512, cfg.scale, causal)
        assert torch.equal(out2, out) and torch.equal(lse2, lse)
    with pytest.raises(ValueError):
        p.kind = 7
        ops.dense_decode(p)


def test_mla_fp16(device):
    for heads, bs in ((128, 64), (16, 64), (8, 24)):   # the default kernel, its small-head form, the per-tile kernel
        cfg, inp = _mla_inputs(3, heads, 100, 1500, 30 + heads, dtype=torch.float16, bs=bs)
        lay = inp.layout
        kg, _, _, _ = fill_caches_gpu(inp, device)
        kc, _ = fill_caches_cpu(inp)
        assert torch.equal(kg.cpu(), kc)
        q = inp.q.to(device).view(3, 1, heads, 576)
        p = ops.DenseDecodeParams(q_nope=q[..., :512], q_pe=q[..., 512:], k_cache=kg, seqlens_k=lay.seq_lens.to(device),
                                  block_table=lay.block_table.to(device), head_size_v=512, softmax_scale=cfg.scale)
        out, lse = ops.dense_decode(p, return_lse=True)
        assert out.dtype == torch.float16
        ref = oracle.aten_paged_decode(inp.q, kc, None, lay.block_table, lay.seq_lens, cfg.scale, dv=512)
        assert_close_to_reference(out.view(3, heads, 512), ref, f"fp16 mla {heads}")
        ref_lse = oracle.aten_paged_decode_lse(inp.q, kc, lay.block_table, lay.seq_lens, cfg.scale)
        assert torch.allclose(lse.view(3, heads).cpu(), ref_lse, rtol=1e-3, atol=1e-3)
    with pytest.raises(TypeError):   # a cache of another type than q
        p.k_cache = kg.to(torch.bfloat16)
        ops.dense_decode(p)


@pytest.mark.parametrize("fp8", [False, True])
def test_layer_forward_writes_then_attends(device, fp8):
    """AttentionImpl::forward(AttentionMetadata, query, key, value, KVCache) -> (output [T, Hq * D], lse?) of
    layers/dcu/attention.cpp:55-112: the step's rows go into the cache (the quantising store when the cache carries
    scales, layers/mlu/attention.cpp:109-117), then every sequence attends to its whole context."""
    xops = torch_ops.load()
    cfg = workloads.DecodeConfig("layer", 6, 32, 8, 128, 16, 60, 1500, cache_dtype="fp8" if fp8 else "bf16")
    inp = workloads.make_inputs(cfg, 77)
    lay = inp.layout
    cache_dt = torch.float8_e4m3fn if fp8 else torch.bfloat16
    shape = (lay.num_blocks, cfg.block_size, cfg.n_kv_heads, cfg.head_dim)
    kg = torch.zeros(shape, dtype=cache_dt, device=device)
    vg = torch.zeros_like(kg)
    ks = vs = None
    if fp8:
        ks = ops.kv_head_scales(torch.cat([inp.k_ctx, inp.k_new]).to(device))
        vs = ops.kv_head_scales(torch.cat([inp.v_ctx, inp.v_new]).to(device))
    store = ops.quant_to_paged_cache if fp8 else ops.reshape_paged_cache
    store(ops.ReshapePagedCacheParams(key=inp.k_ctx.to(device), value=inp.v_ctx.to(device), k_cache=kg, v_cache=vg,
                                      slot_mapping=lay.ctx_slots.to(device), k_cache_scale=ks, v_cache_scale=vs))
    B, Hq, Hkv, D = cfg.batch, cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim
    query = inp.q.to(device).view(B, Hq * D)
    key = inp.k_new.to(device).view(B, Hkv * D)
    value = inp.v_new.to(device).view(B, Hkv * D)
    out, lse = xops.attention_layer_forward(query, key, value, kg, vg, ks, vs, lay.new_slots.to(device),
                                            lay.block_table.to(device), lay.seq_lens.to(device), None,
                                            int(lay.seq_lens.max()), 1, Hq, D, Hkv, cfg.scale, -1, True, True)
    torch.cuda.synchronize()
    assert out.shape == (B, Hq * D) and lse.shape == (B, Hq, 1) and lse.dtype == torch.float32
    kc, vc = fill_caches_cpu(inp, cache_dt, None if ks is None else ks.cpu(), None if vs is None else vs.cpu())
    view = torch.uint8 if fp8 else torch.bfloat16
    assert torch.equal(kg.view(view).cpu(), kc) and torch.equal(vg.view(view).cpu(), vc), "the step's rows were not stored"
    ref = oracle.aten_paged_decode(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale,
                                   None if ks is None else ks.cpu(), None if vs is None else vs.cpu())
    assert_close_to_reference(out.view(B, Hq, D), ref, "layer forward")
    ref_lse = oracle.aten_paged_decode_lse(inp.q, kc, lay.block_table, lay.seq_lens, cfg.scale,
                                           None if ks is None else ks.cpu())
    assert torch.allclose(lse.view(B, Hq).cpu(), ref_lse, rtol=1e-3, atol=1e-3)
    # a sliding window of the layer (sliding_window_ of layers/dcu/flash_attention.cpp:484) and no LSE
    out_w, none = xops.attention_layer_forward(query, key, value, kg, vg, ks, vs, lay.new_slots.to(device),
                                               lay.block_table.to(device), lay.seq_lens.to(device), None,
                                               int(lay.seq_lens.max()), 1, Hq, D, Hkv, cfg.scale, 200, True, False)
    assert none is None
    first = (lay.seq_lens - 1 - 200).clamp_min(0)
    nk, nv, table, lens = trimmed_context(kc, vc, lay.block_table, lay.seq_lens, first)
    ref_w = oracle.aten_paged_decode(inp.q, nk, nv, table, lens, cfg.scale, None if ks is None else ks.cpu(),
                                     None if vs is None else vs.cpu())
    assert_close_to_reference(out_w.view(B, Hq, D), ref_w, "layer forward, window 200")
    # max_seq_len == 0: nothing to do, the output comes back untouched in shape [T, Hq * D]
    out0, _ = xops.attention_layer_forward(query, key, value, kg, vg, ks, vs, lay.new_slots.to(device),
                                           lay.block_table.to(device), lay.seq_lens.to(device), None, 0, 1, Hq, D, Hkv,
                                           cfg.scale, -1, True, False)
    assert out0.shape == (B, Hq * D)


def test_layer_forward_with_query_chunks(device):
    # chunked prefill with short chunks through the same layer call (layers/dcu/flash_attention.cpp:447-545)
    xops = torch_ops.load()
    cfg = workloads.DecodeConfig("layer_chunks", 3, 16, 4, 128, 16, 100, 700)
    inp = workloads.make_inputs(cfg, 78)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)     # the whole context, chunk included, is in the cache
    q_lens = torch.tensor([4, 1, 2])
    cu = torch.zeros(4, dtype=torch.int32)
    cu[1:] = torch.cumsum(q_lens, 0)
    T = int(cu[-1])
    gen = torch.Generator().manual_seed(5)
    qq = workloads.randn_16bit((T, 16, 128), 1.0, gen, "cpu")
    kk = workloads.randn_16bit((T, 4, 128), 1.0, gen, "cpu")
    vv = workloads.randn_16bit((T, 4, 128), 1.0, gen, "cpu")
    # slots of the chunk tokens: the last q_len positions of each context
    slots = []
    for b in range(3):
        L = int(lay.seq_lens[b])
        for j in range(int(q_lens[b])):
            t = L - int(q_lens[b]) + j
            slots.append(int(lay.block_table[b, t // 16]) * 16 + t % 16)
    slots = torch.tensor(slots, dtype=torch.int32)
    out, _ = xops.attention_layer_forward(qq.to(device).view(T, -1), kk.to(device).view(T, -1), vv.to(device).view(T, -1),
                                          kg, vg, None, None, slots.to(device), lay.block_table.to(device),
                                          lay.seq_lens.to(device), cu.to(device), int(lay.seq_lens.max()), 4, 16, 128, 4,
                                          cfg.scale, -1, True, False)
    kc, vc = kg.cpu(), vg.cpu()
    assert torch.equal(kc.view(-1, 4, 128)[slots.long()], kk) and torch.equal(vc.view(-1, 4, 128)[slots.long()], vv)
    ref = oracle.aten_paged_forward(qq, kc, vc, lay.block_table, lay.seq_lens, cu, cfg.scale, causal=True)
    assert_close_to_reference(out.view(T, 16, 128), ref, "layer forward, chunks")


def test_host_side_refuses_what_the_kernels_cannot_take(device):
    xops = torch_ops.load()
    cfg = workloads.DecodeConfig("neg", 2, 8, 2, 128, 16, 20, 60)
    inp = workloads.make_inputs(cfg, 3)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    q = inp.q.to(device)
    out = torch.empty_like(q)
    table, lens = lay.block_table.to(device), lay.seq_lens.to(device)
    narrow = torch.zeros(kg.shape[0], 16, 2, 64, dtype=torch.bfloat16, device=device)
    bad_calls = [
        lambda: xops.batch_decode(q, kg, vg, out.float(), table, lens, None, None, 0, cfg.scale),            # output dtype
        lambda: xops.batch_decode(q, kg, narrow, out, table, lens, None, None, 0, cfg.scale),                # v_cache shape
        lambda: xops.batch_decode(q, kg.view(torch.uint8)[..., :128].contiguous(), vg.view(torch.uint8)[..., :128].contiguous(),
                                  out, table, lens, None, None, 0, cfg.scale),                               # fp8 without scales
        lambda: xops.reshape_paged_cache(lay.new_slots.to(device), inp.k_new.to(device), inp.v_new.to(device), narrow, narrow),
        lambda: xops.quant_to_paged_cache(lay.new_slots.to(device), inp.k_new.to(device), inp.v_new.to(device),
                                          kg.view(torch.uint8)[..., :128].contiguous(), vg.view(torch.uint8)[..., :128].contiguous(),
                                          torch.ones(3, device=device), torch.ones(2, device=device)),       # scale count
        lambda: ops.batch_decode(q, kg, out.float(), table, lens, v_cache=vg),
        lambda: ops.batch_decode(q, kg, out, table, lens, v_cache=narrow),
    ]
    for call in bad_calls:
        with pytest.raises(Exception):
            call()
    # the fused norm + rope + cache write: a uint8 (fp8) cache without scales, a cache of another shape, int64 slots
    qkv = torch.zeros(2, (8 + 2 + 2) * 128, dtype=torch.bfloat16, device=device)
    w = torch.ones(128, dtype=torch.bfloat16, device=device)
    cs = torch.zeros(64, 128, device=device)
    pos = torch.zeros(2, dtype=torch.int64, device=device)
    k8 = torch.zeros(kg.shape, dtype=torch.uint8, device=device)
    slots = lay.new_slots.to(device)
    for kwargs in (dict(k_cache=k8, v_cache=k8.clone(), slot_mapping=slots),
                   dict(k_cache=narrow, v_cache=narrow.clone(), slot_mapping=slots),
                   dict(k_cache=kg, v_cache=vg, slot_mapping=slots.long()),
                   dict(k_cache=kg.to(torch.float16), v_cache=vg.to(torch.float16), slot_mapping=slots),
                   dict(k_cache=kg, v_cache=vg, slot_mapping=slots.cpu())):
        with pytest.raises(Exception):
            ops.fused_qk_norm_rope(qkv, 8, 2, 2, 128, 1e-6, w, w, cs, False, pos, **kwargs)
    with pytest.raises(Exception):
        ops.fused_qk_norm_rope(qkv, 8, 2, 2, 128, 1e-6, w.cpu(), w, cs, False, pos)
