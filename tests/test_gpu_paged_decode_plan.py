"""GPU tests of the step plan: a decode call that starts from a plan runs the same kernels over the same ranges as one
that derives its schedule itself, so its outputs must be bit-identical; the plain call is checked against the
reference's libtorch CPU path elsewhere and once more here."""
import pytest
import torch

import oracle
from helpers import assert_close_to_reference, fill_caches_gpu
from xllm_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu


def _both(inp, kg, vg, device, ks=None, vs=None, window_left=-1, lens=None):
    cfg, lay = inp.cfg, inp.layout
    q = inp.q.to(device)
    table = lay.block_table.to(device)
    lens = (lay.seq_lens if lens is None else lens).to(device)
    hi = max(1, int(lens.max()))
    plain, plain_lse = ops.batch_decode(q, kg, torch.empty_like(q), table, lens, v_cache=vg, k_cache_quant_scale=ks,
                                        v_cache_quant_scale=vs, scale=cfg.scale, return_lse=True, max_seq_len=hi,
                                        window_left=window_left)
    plan = ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, kg.dtype,
                                       block_table=table, seq_lens=lens, window_left=window_left)
    outs = []
    for _ in range(2):  # the layers of a step share the plan
        o, l = ops.batch_decode(q, kg, torch.full_like(q, 7.0), table, lens, v_cache=vg, k_cache_quant_scale=ks,
                                v_cache_quant_scale=vs, scale=cfg.scale, return_lse=True, max_seq_len=hi,
                                window_left=window_left, plan=plan)
        outs.append((o, l))
    torch.cuda.synchronize()
    for o, l in outs:
        assert torch.equal(o, plain), cfg.name
        assert torch.equal(l, plain_lse), cfg.name
    assert ops.decode_status(device) == 0
    return plain


def test_planned_decode_is_bit_identical_on_the_benchmark_shapes(device):
    for name, batch, seed in (("llama3_8b", 64, 3), ("long_b256", 24, 4)):
        cfg = workloads.scaled(workloads.CONFIGS[name], batch=batch)
        inp = workloads.make_inputs(cfg, seed, device=device)
        kg, vg, _, _ = fill_caches_gpu(inp, device)
        out = _both(inp, kg, vg, device)
        lay = inp.layout
        sample = [0, 1, batch // 2, batch - 1]
        ref = oracle.aten_paged_decode(inp.q.cpu()[sample].contiguous(), kg.cpu(), vg.cpu(),
                                       lay.block_table[sample].contiguous(), lay.seq_lens[sample].contiguous(), cfg.scale)
        assert_close_to_reference(out[sample], ref, cfg.name)


def test_planned_decode_over_shapes_windows_and_empty_sequences(device):
    g = torch.Generator().manual_seed(11)
    # (Hq, Hkv, D, block size, fp8): the stage sizes and head-block groupings of the matrix-core kernel, and a
    # shape that the kernel does not serve (block size 8), which takes no plan
    shapes = ((32, 8, 128, 16, False), (32, 8, 128, 16, True), (8, 2, 64, 32, False), (16, 4, 64, 16, True),
              (6, 1, 256, 128, False), (40, 2, 128, 16, False), (12, 3, 128, 64, False), (8, 2, 128, 8, False),
              (4, 1, 256, 16, True))
    for i, (Hq, Hkv, D, bs, fp8) in enumerate(shapes):
        batch = int(torch.randint(1, 40, (1,), generator=g))
        cfg = workloads.DecodeConfig(f"plan_{Hq}_{Hkv}_{D}_{bs}_{fp8}", batch, Hq, Hkv, D, bs, 1, 1500,
                                     cache_dtype="fp8" if fp8 else "bf16")
        inp = workloads.make_inputs(cfg, 300 + i, device=device)
        kg, vg, ks, vs = fill_caches_gpu(inp, device, cache_dtype=torch.float8_e4m3fn if fp8 else None)
        _both(inp, kg, vg, device, ks, vs)
        _both(inp, kg, vg, device, ks, vs, window_left=200)
        lens = inp.layout.seq_lens.clone()
        lens[torch.rand(batch, generator=g) < 0.4] = 0
        _both(inp, kg, vg, device, ks, vs, lens=lens)
        _both(inp, kg, vg, device, ks, vs, lens=torch.zeros_like(lens))


def test_batches_decoded_in_slices_and_tiny_batches_with_a_plan(device):
    # more sequences than one launch takes (the plan is not used then), and fewer work items than workers
    for batch, hi in ((2100, 40), (1, 5), (3, 70)):
        cfg = workloads.DecodeConfig(f"plan_b{batch}", batch, 32, 8, 128, 16, 1, hi)
        inp = workloads.make_inputs(cfg, 500 + batch, device=device)
        kg, vg, _, _ = fill_caches_gpu(inp, device)
        _both(inp, kg, vg, device)


def test_planned_decode_in_csr_form(device):
    cfg = workloads.scaled(workloads.CONFIGS["llama3_8b"], batch=37, len_lo=1, len_hi=3000)
    inp = workloads.make_inputs(cfg, 21, device=device)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    q = inp.q.to(device)
    indptr, indices, last = lay.indptr.to(device), lay.indices.to(device), lay.last_page_len.to(device)
    hi = int(lay.seq_lens.max())
    plain = ops.batch_decode_csr(q, kg, vg, indptr, indices, last, -1, cfg.scale, torch.empty_like(q), max_seq_len=hi)
    plan = ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, kg.dtype,
                                       paged_kv_indptr=indptr, paged_kv_indices=indices, paged_kv_last_page_len=last)
    planned = ops.batch_decode_csr(q, kg, vg, indptr, indices, last, -1, cfg.scale, torch.full_like(q, 7.0),
                                   max_seq_len=hi, plan=plan)
    torch.cuda.synchronize()
    assert torch.equal(plain, planned)
    assert ops.decode_status(device) == 0


def test_a_plan_for_another_shape_is_reported(device):
    cfg = workloads.scaled(workloads.CONFIGS["llama3_8b"], batch=9)
    inp = workloads.make_inputs(cfg, 5, device=device)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    q, table, lens = inp.q.to(device), lay.block_table.to(device), lay.seq_lens.to(device)
    assert ops.decode_status(device) == 0
    # made for 8 of the 9 sequences
    plan = ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, kg.dtype,
                                       block_table=table[:8], seq_lens=lens[:8].contiguous())
    ops.batch_decode(q, kg, torch.empty_like(q), table, lens, v_cache=vg, scale=cfg.scale, plan=plan)
    with pytest.raises(capi.XllmMi355Error, match="plan"):
        ops.decode_status(device)
    assert ops.decode_status(device) == 0   # reported once
    good = ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, kg.dtype,
                                       block_table=table, seq_lens=lens, plan=plan)
    assert good.data_ptr() == plan.data_ptr()
    a, _ = ops.batch_decode(q, kg, torch.empty_like(q), table, lens, v_cache=vg, scale=cfg.scale, plan=good)
    b, _ = ops.batch_decode(q, kg, torch.empty_like(q), table, lens, v_cache=vg, scale=cfg.scale)
    assert torch.equal(a, b)
    assert ops.decode_status(device) == 0
    with pytest.raises(ValueError):   # a plan buffer that is too small
        ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, kg.dtype,
                                    block_table=table, seq_lens=lens, plan=plan[:4096])


def test_a_plan_that_was_not_made_again_for_new_lengths_is_reported(device):
    """The serving-loop mistake: the lengths move on, the shape stays, the plan of the step before is passed again.
    The kernels follow the old ranges (their reads stay inside the tables and the caches, also when contexts shrank
    or emptied), and the status call says so."""
    cfg = workloads.scaled(workloads.CONFIGS["llama3_8b"], batch=19, len_lo=40, len_hi=900)
    inp = workloads.make_inputs(cfg, 6, device=device)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    q, table = inp.q.to(device), lay.block_table.to(device)
    lens = lay.seq_lens.to(device)
    plan_of = lambda l: ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size,
                                                    kg.dtype, block_table=table, seq_lens=l)
    assert ops.decode_status(device) == 0
    plan = plan_of(lens)
    shorter = (lens - 1).contiguous()                       # one token fewer each: the same work items, other lengths
    much_shorter = torch.clamp(lens - 300, min=0).contiguous()   # contexts that shrank by pages, some to nothing
    one_moved = lens.clone()
    one_moved[7] -= 1
    for stale in (shorter, much_shorter, one_moved):
        ops.batch_decode(q, kg, torch.empty_like(q), table, stale, v_cache=vg, scale=cfg.scale, plan=plan)
        with pytest.raises(capi.XllmMi355Error, match="plan"):
            ops.decode_status(device)
        assert ops.decode_status(device) == 0
        # planned again for those lengths: bit-identical to the plain call, nothing to report
        a, _ = ops.batch_decode(q, kg, torch.empty_like(q), table, stale, v_cache=vg, scale=cfg.scale,
                                plan=plan_of(stale))
        b, _ = ops.batch_decode(q, kg, torch.empty_like(q), table, stale, v_cache=vg, scale=cfg.scale)
        assert torch.equal(a, b)
        assert ops.decode_status(device) == 0
    # CSR form, the last sequence emptied under the old plan
    indptr, indices, last = lay.indptr.to(device), lay.indices.to(device), lay.last_page_len.to(device)
    plan = ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, kg.dtype,
                                       paged_kv_indptr=indptr, paged_kv_indices=indices, paged_kv_last_page_len=last)
    emptied = indptr.clone()
    emptied[-1] = emptied[-2]
    ops.batch_decode_csr(q, kg, vg, emptied, indices, last, -1, cfg.scale, torch.empty_like(q), plan=plan)
    with pytest.raises(capi.XllmMi355Error, match="plan"):
        ops.decode_status(device)
    assert ops.decode_status(device) == 0


def test_a_captured_step_plans_again_on_every_replay(device):
    # plan + two planned layers in one graph; the lengths change between replays (the persistent buffers of a
    # captured decode step), eager calls run in between
    cfg = workloads.DecodeConfig("plan_graph", 48, 32, 8, 128, 16, 200, 2500)
    inp = workloads.make_inputs(cfg, 31, device=device)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    q, table = inp.q.to(device), lay.block_table.to(device)
    lens = lay.seq_lens.to(device).clone()
    plan = ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, kg.dtype,
                                       block_table=table, seq_lens=lens)
    o1, o2 = torch.zeros_like(q), torch.zeros_like(q)
    ops.batch_decode(q, kg, o1, table, lens, v_cache=vg, scale=cfg.scale, max_seq_len=2500, plan=plan)  # warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, kg.dtype,
                                    block_table=table, seq_lens=lens, plan=plan)
        ops.batch_decode(q, kg, o1, table, lens, v_cache=vg, scale=cfg.scale, max_seq_len=2500, plan=plan)
        ops.batch_decode(q, kg, o2, table, lens, v_cache=vg, scale=cfg.scale, max_seq_len=2500, plan=plan)
    g = torch.Generator().manual_seed(3)
    for rep in range(4):
        cut = torch.randint(0, 200, (cfg.batch,), generator=g, dtype=torch.int32)
        cut[torch.rand(cfg.batch, generator=g) < 0.2] = 100000   # some sequences leave the batch
        lens.copy_(torch.clamp(lay.seq_lens - cut, min=0).to(device))
        o1.zero_()
        o2.zero_()
        graph.replay()
        torch.cuda.synchronize()
        eager, _ = ops.batch_decode(q, kg, torch.empty_like(q), table, lens, v_cache=vg, scale=cfg.scale, max_seq_len=2500)
        torch.cuda.synchronize()
        assert torch.equal(o1, eager) and torch.equal(o2, eager), f"replay {rep}"
    assert ops.decode_status(device) == 0


def test_layer_zero_plans_and_the_other_layers_decode_from_its_plan(device):
    """AttentionMetadata::plan_info of the reference (layers/common/attention_metadata.h:163): every layer's forward
    calls update_decode_plan_info, which returns at once unless layer_id == 0
    (layers/cuda/flashinfer_planinfo.cpp:263-264), and hands the plan to batch_decode."""
    from xllm_amd import torch_ops
    xops = torch_ops.load()
    cfg = workloads.DecodeConfig("layer_plan", 21, 32, 8, 128, 16, 60, 2500)
    inp = workloads.make_inputs(cfg, 78)
    lay = inp.layout
    B, Hq, Hkv, D = cfg.batch, cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim
    caches = []
    for layer in range(3):   # every layer has its own cache; the tables and lengths are the step's
        kg = torch.zeros(lay.num_blocks, cfg.block_size, Hkv, D, dtype=torch.bfloat16, device=device)
        vg = torch.zeros_like(kg)
        scale = 1.0 + 0.25 * layer
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(
            key=(inp.k_ctx * scale).to(device), value=(inp.v_ctx * scale).to(device), k_cache=kg, v_cache=vg,
            slot_mapping=lay.ctx_slots.to(device)))
        caches.append((kg, vg))
    query = inp.q.to(device).view(B, Hq * D)
    key = inp.k_new.to(device).view(B, Hkv * D)
    value = inp.v_new.to(device).view(B, Hkv * D)
    table, lens, slots = lay.block_table.to(device), lay.seq_lens.to(device), lay.new_slots.to(device)
    hi = int(lay.seq_lens.max())

    def layer_forward(layer, plan, layer_id):
        kg, vg = caches[layer]
        out, lse = xops.attention_layer_forward(query, key, value, kg, vg, None, None, slots, table, lens, None, hi, 1,
                                                Hq, D, Hkv, cfg.scale, -1, True, True, plan, layer_id)
        return out.clone(), lse.clone()

    plain = [layer_forward(layer, None, -1) for layer in range(3)]
    plan = torch.zeros(capi.lib().xllm_mi355_paged_decode_plan_bytes(), dtype=torch.uint8, device=device)
    planned = [layer_forward(layer, plan, layer) for layer in range(3)]
    torch.cuda.synchronize()
    assert int(plan.view(torch.int32)[0]) != 0, "layer 0 did not plan"
    for (a, al), (b, bl) in zip(plain, planned):
        assert torch.equal(a, b) and torch.equal(al, bl)
    assert not torch.equal(plain[0][0], plain[1][0])
    assert ops.decode_status(device) == 0
    # the dispatcher ops on their own
    p2 = xops.update_decode_plan(table, lens, Hq, Hkv, D, cfg.block_size, -1, False)
    kg, vg = caches[0]
    q3 = inp.q.to(device)
    a, _ = xops.batch_decode(q3, kg, vg, torch.empty_like(q3), table, lens, None, None, hi, cfg.scale, p2)
    b, _ = xops.batch_decode(q3, kg, vg, torch.empty_like(q3), table, lens, None, None, hi, cfg.scale)
    assert torch.equal(a, b)
    w2, w = p2.view(torch.int32), plan.view(torch.int32)   # the same plan: its first word and the item prefix
    assert int(w2[0]) == int(w[0]) and torch.equal(w2[64 : 64 + B + 2], w[64 : 64 + B + 2])


def test_random_shapes_plain_planned_and_both_kinds_of_stores_agree(device):
    # head dims, head groupings, block sizes, batch sizes, windows, fp8 pages and empty sequences drawn at random: the
    # planned call and either kind of stores must reproduce the plain call bit for bit; small cases also go to the oracle
    lib = capi.lib()
    g = torch.Generator().manual_seed(5)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))

    for case in range(16):
        D = [64, 128, 128, 256][ri(0, 3)]
        fp8 = ri(0, 3) == 0
        Hkv = [1, 2, 3, 4, 8][ri(0, 4)]
        Hq = Hkv * [1, 2, 4, 5, 8, 16, 20][ri(0, 6)]
        bs = [16, 32, 64, 128][ri(0, 3)]
        batch = [1, 2, 7, 33, 64, 130, 300][ri(0, 6)]
        hi = [40, 600, 3000][ri(0, 2)]
        if batch * hi * Hkv * D > 1e9:
            hi = 600
        window = [-1, -1, 100, 1000][ri(0, 3)]
        cfg = workloads.DecodeConfig(f"rnd{case}_{batch}_{Hq}_{Hkv}_{D}_{bs}", batch, Hq, Hkv, D, bs, 1, hi,
                                     cache_dtype="fp8" if fp8 else "bf16")
        inp = workloads.make_inputs(cfg, 1000 + case, device=device)
        lay = inp.layout
        kg, vg, ks, vs = fill_caches_gpu(inp, device, cache_dtype=torch.float8_e4m3fn if fp8 else None)
        lens = lay.seq_lens.clone()
        if ri(0, 2) == 0:
            lens[torch.rand(batch, generator=g) < 0.3] = 0
        q, table, lens_d = inp.q.to(device), lay.block_table.to(device), lens.to(device)
        longest = max(1, int(lens.max()))

        def run(plan=None):
            o, l = ops.batch_decode(q, kg, torch.full_like(q, 3.0), table, lens_d, v_cache=vg, k_cache_quant_scale=ks,
                                    v_cache_quant_scale=vs, scale=cfg.scale, return_lse=True, max_seq_len=longest,
                                    window_left=window, plan=plan)
            torch.cuda.synchronize()
            return o, l

        base = run()
        plan = ops.update_decode_plan_info(Hq, Hkv, D, bs, kg.dtype, block_table=table, seq_lens=lens_d,
                                           window_left=window)
        outs = [run(plan)]
        try:
            for kind in (0, 1):
                assert lib.xllm_mi355_debug_set(3, kind) == 0
                outs += [run(), run(plan)]
        finally:
            assert lib.xllm_mi355_debug_set(3, -1) == 0
        for o, l in outs:
            assert torch.equal(o, base[0]) and torch.equal(l, base[1]), cfg.name
        assert ops.decode_status(device) == 0
        keep = (lens > 0).nonzero().flatten()
        if batch * hi <= 40000 and window < 0 and len(keep) > 0:
            ref = oracle.aten_paged_decode(inp.q.cpu()[keep].contiguous(), kg.cpu(), vg.cpu(),
                                           lay.block_table[keep].contiguous(), lens[keep].contiguous(), cfg.scale,
                                           None if ks is None else ks.cpu(), None if vs is None else vs.cpu())
            assert_close_to_reference(base[0][keep.to(device)], ref, cfg.name)


# ---- the MLA decode from a plan -------------------------------------------------------------------------------------

def _mla_cfg(name, batch, heads, lo, hi, bs=64):
    import math
    return workloads.DecodeConfig(name, batch, heads, 1, 576, bs, lo, hi, mla=True, v_dim=512, sigma=0.5,
                                  sm_scale=1.0 / math.sqrt(192.0))


def _mla_params(inp, kg, device, lens=None):
    cfg, lay = inp.cfg, inp.layout
    q = inp.q.to(device)
    B, H = cfg.batch, cfg.n_q_heads
    return ops.DenseDecodeParams(
        q_nope=q[:, :, :512].contiguous().view(B, 1, H, 512), q_pe=q[:, :, 512:].contiguous().view(B, 1, H, 64),
        k_cache=kg, seqlens_k=(lay.seq_lens if lens is None else lens).to(device), block_table=lay.block_table.to(device),
        head_size_v=512, softmax_scale=cfg.scale)


def test_mla_planned_decode_is_bit_identical(device):
    g = torch.Generator().manual_seed(3)
    # 128 heads (one workgroup per team), a ragged last head block, two workgroups per team, a block size of 16, many
    # short sequences, fewer tiles than workgroups; and head counts / block sizes that take no plan (other kernels)
    cases = [_mla_cfg("p128", 7, 128, 200, 5000), _mla_cfg("p80", 4, 80, 100, 3000), _mla_cfg("p200", 3, 200, 500, 4000),
             _mla_cfg("p_bs16", 5, 128, 100, 2500, bs=16), _mla_cfg("p_short", 300, 128, 1, 150),
             _mla_cfg("p_tiny", 2, 128, 1, 70), _mla_cfg("p16", 6, 16, 100, 2000), _mla_cfg("p_bs8", 3, 128, 50, 600, bs=8)]
    for n, cfg in enumerate(cases):
        inp = workloads.make_inputs(cfg, 900 + n)
        kg, _, _, _ = fill_caches_gpu(inp, device)
        lens = inp.layout.seq_lens.clone()
        if cfg.batch > 4:
            lens[torch.rand(cfg.batch, generator=g) < 0.25] = 0
        p = _mla_params(inp, kg, device, lens)
        plain, plain_lse = ops.dense_decode(p, return_lse=True)
        plan = ops.get_mla_decoding_metadata(p.seqlens_k, p.block_table, cfg.n_q_heads, cfg.block_size)
        for _ in range(2):   # the layers of a step share the plan
            out, lse = ops.dense_decode(p, return_lse=True, metadata=plan)
            assert torch.equal(out.view(torch.int16), plain.view(torch.int16)), cfg.name
            assert torch.equal(lse, plain_lse), cfg.name
        assert ops.decode_status(device) == 0
    lib = capi.lib()
    cfg = cases[0]
    inp = workloads.make_inputs(cfg, 900)
    kg, _, _, _ = fill_caches_gpu(inp, device)
    p = _mla_params(inp, kg, device)
    plain = ops.dense_decode(p)
    plan = ops.get_mla_decoding_metadata(p.seqlens_k, p.block_table, cfg.n_q_heads, cfg.block_size)
    try:   # the merge inside the decode kernel, from a plan
        assert lib.xllm_mi355_debug_set(4, 1) == 0
        assert torch.equal(ops.dense_decode(p, metadata=plan), plain)
    finally:
        assert lib.xllm_mi355_debug_set(4, -1) == 0
    assert ops.decode_status(device) == 0


def test_a_stale_mla_plan_is_reported(device):
    cfg = _mla_cfg("stale", 9, 128, 300, 4000)
    inp = workloads.make_inputs(cfg, 31)
    kg, _, _, _ = fill_caches_gpu(inp, device)
    p = _mla_params(inp, kg, device)
    assert ops.decode_status(device) == 0
    plan = ops.get_mla_decoding_metadata(p.seqlens_k, p.block_table, cfg.n_q_heads, cfg.block_size)
    good = ops.dense_decode(p, metadata=plan)
    assert ops.decode_status(device) == 0
    # the lengths moved on, the plan did not
    for lens in ((inp.layout.seq_lens - 1), torch.clamp(inp.layout.seq_lens - 900, min=0)):
        q = _mla_params(inp, kg, device, lens.to(torch.int32).contiguous())
        ops.dense_decode(q, metadata=plan)
        with pytest.raises(capi.XllmMi355Error, match="plan"):
            ops.decode_status(device)
        assert ops.decode_status(device) == 0
        fresh = ops.get_mla_decoding_metadata(q.seqlens_k, q.block_table, cfg.n_q_heads, cfg.block_size, plan=plan)
        assert fresh.data_ptr() == plan.data_ptr()
        assert torch.equal(ops.dense_decode(q, metadata=fresh), ops.dense_decode(q))
        assert ops.decode_status(device) == 0
    # a plan made for another batch: nothing is written
    other = ops.get_mla_decoding_metadata(p.seqlens_k[:8].contiguous(), p.block_table[:8], cfg.n_q_heads, cfg.block_size)
    ops.dense_decode(p, metadata=other)
    with pytest.raises(capi.XllmMi355Error, match="plan"):
        ops.decode_status(device)
    assert ops.decode_status(device) == 0
    again = ops.get_mla_decoding_metadata(p.seqlens_k, p.block_table, cfg.n_q_heads, cfg.block_size)
    assert torch.equal(ops.dense_decode(p, metadata=again), good) and ops.decode_status(device) == 0


def test_a_captured_mla_step_plans_again_on_every_replay(device):
    # plan + decode captured once; the replays see new lengths and tables in the same buffers and plan from them
    cfg = _mla_cfg("pgraph", 6, 128, 100, 2500)
    inputs = [workloads.make_inputs(cfg, 440 + i) for i in range(3)]
    width = max(inp.layout.block_table.shape[1] for inp in inputs)
    blocks = max(inp.layout.num_blocks for inp in inputs)
    k_cache = torch.zeros(blocks, cfg.block_size, 1, 576, dtype=torch.bfloat16, device=device)
    table = torch.zeros(cfg.batch, width, dtype=torch.int32, device=device)
    lens = torch.zeros(cfg.batch, dtype=torch.int32, device=device)
    q_nope = torch.zeros(cfg.batch, 1, cfg.n_q_heads, 512, dtype=torch.bfloat16, device=device)
    q_pe = torch.zeros(cfg.batch, 1, cfg.n_q_heads, 64, dtype=torch.bfloat16, device=device)
    plan = torch.zeros(capi.lib().xllm_mi355_paged_decode_plan_bytes(), dtype=torch.uint8, device=device)
    result = {}

    def load(inp):
        lay = inp.layout
        k_cache.zero_()
        for k, slots in ((inp.k_ctx, lay.ctx_slots), (inp.k_new, lay.new_slots)):
            ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=k.to(device), value=None, k_cache=k_cache,
                                                                v_cache=None, slot_mapping=slots.to(device)))
        table.zero_()
        table[:, : lay.block_table.shape[1]] = lay.block_table.to(device)
        lens.copy_(lay.seq_lens.to(device))
        q = inp.q.to(device)
        q_nope.copy_(q[:, :, :512].reshape(cfg.batch, 1, cfg.n_q_heads, 512))
        q_pe.copy_(q[:, :, 512:].reshape(cfg.batch, 1, cfg.n_q_heads, 64))

    def params():
        return ops.DenseDecodeParams(q_nope=q_nope, q_pe=q_pe, k_cache=k_cache, seqlens_k=lens, block_table=table,
                                     head_size_v=512, softmax_scale=cfg.scale)

    def step():
        ops.get_mla_decoding_metadata(lens, table, cfg.n_q_heads, cfg.block_size, plan=plan)
        result["a"] = ops.dense_decode(params(), max_seq_len=width * cfg.block_size, metadata=plan)
        result["b"] = ops.dense_decode(params(), max_seq_len=width * cfg.block_size, metadata=plan)   # a second layer

    load(inputs[0])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up outside the capture: workspace allocation, kernel attributes
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for inp in inputs[1:] + inputs[:1]:
        load(inp)
        eager = ops.dense_decode(params(), max_seq_len=width * cfg.block_size)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(result["a"], eager) and torch.equal(result["b"], eager)
        assert ops.decode_status(device) == 0
