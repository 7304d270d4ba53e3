"""GPU parity of the MLA latent-KV paged decode against the reference's libtorch CPU path."""
import math

import pytest
import torch

import oracle
from helpers import assert_close_to_reference, fill_caches_cpu, fill_caches_gpu
from xllm_amd import ops, workloads

pytestmark = pytest.mark.gpu


def _decode_gpu(inp, k_cache, device, return_lse=True, table=None, seq_lens=None):
    cfg, lay = inp.cfg, inp.layout
    q = inp.q.to(device)
    B, H = cfg.batch, cfg.n_q_heads
    lens = lay.seq_lens if seq_lens is None else seq_lens
    p = ops.DenseDecodeParams(
        q_nope=q[:, :, : cfg.v_dim].contiguous().view(B, 1, H, cfg.v_dim),
        q_pe=q[:, :, cfg.v_dim :].contiguous().view(B, 1, H, cfg.head_dim - cfg.v_dim),
        k_cache=k_cache, seqlens_k=lens.to(device),
        block_table=(lay.block_table if table is None else table).to(device),
        head_size_v=cfg.v_dim, softmax_scale=cfg.scale)
    res = ops.dense_decode(p, return_lse=return_lse, max_seq_len=int(lens.max()))
    torch.cuda.synchronize()
    if return_lse:
        return res[0].view(B, H, cfg.v_dim), res[1].view(B, H)
    return res.view(B, H, cfg.v_dim), None


def _mla_cfg(name, batch, heads, lo, hi, bs=64):
    return workloads.DecodeConfig(name, batch, heads, 1, 576, bs, lo, hi, mla=True, v_dim=512, sigma=0.5,
                                  sm_scale=1.0 / math.sqrt(192.0))


def _check(cfg, seed, device):
    inp = workloads.make_inputs(cfg, seed)
    lay = inp.layout
    kg, _, _, _ = fill_caches_gpu(inp, device)
    kc, _ = fill_caches_cpu(inp)
    assert torch.equal(kg.cpu(), kc), "latent cache bytes must be bit-exact"
    out, lse = _decode_gpu(inp, kg, device)
    ref = oracle.aten_paged_decode(inp.q, kc, None, lay.block_table, lay.seq_lens, cfg.scale, dv=cfg.v_dim)
    assert_close_to_reference(out, ref, cfg.name)
    ref_lse = oracle.aten_paged_decode_lse(inp.q, kc, lay.block_table, lay.seq_lens, cfg.scale)
    assert torch.allclose(lse.cpu(), ref_lse, rtol=1e-3, atol=1e-3)
    return inp, kg, out, lse


def test_config5_shape_reduced_batch_and_context(device):
    _check(_mla_cfg("mla128", 3, 128, 100, 1500), 5, device)


def test_head_counts_of_tp_shards_and_reference_test_shape(device):
    # 128 heads / tp; H = 2 is the shape of MluMlaDecodeLseTest (dcp_attention_merge_test.cpp:77-144)
    for heads in (2, 16, 32, 64, 80):
        _check(_mla_cfg(f"mla{heads}", 2, heads, 1, 400), 40 + heads, device)


def _select_kernel(name):
    """The MLA kernel choice (the library reads the environment variable once per process)."""
    from xllm_amd import capi
    assert capi.lib().xllm_mi355_debug_set(1, ord(name[0]) if name else 0) == 0


def test_batches_larger_than_a_workgroup_and_than_a_launch(device):
    # more sequences than threads in a workgroup (several per thread in the tile prefix) and more than one launch
    # holds (1024), in the default kernel and in the one for other block sizes
    for knob in ("", "pairs"):
        _select_kernel(knob)
        try:
            _check(_mla_cfg(f"mla_b600_{knob}", 600, 16, 1, 150), 90, device)
        finally:
            _select_kernel("")
    _check(_mla_cfg("mla_b1100", 1100, 8, 1, 80), 91, device)


def test_reference_lse_closed_form_two_tokens(device):
    # ReturnsFloat32NaturalLogNormalizer: H=2, D=576, Dv=512, L=2, page of 16 rows, scale 1/sqrt(576)
    g = torch.Generator().manual_seed(0)
    q = torch.rand(1, 2, 576, generator=g).to(torch.bfloat16)
    cache = torch.rand(1, 16, 1, 576, generator=g).to(torch.bfloat16)
    scale = 1.0 / math.sqrt(576.0)
    p = ops.DenseDecodeParams(
        q_nope=q[:, :, :512].contiguous().view(1, 1, 2, 512).to(device),
        q_pe=q[:, :, 512:].contiguous().view(1, 1, 2, 64).to(device), k_cache=cache.to(device),
        seqlens_k=torch.tensor([2], dtype=torch.int32, device=device),
        block_table=torch.zeros(1, 1, dtype=torch.int32, device=device), head_size_v=512, softmax_scale=scale)
    out, lse = ops.dense_decode(p, return_lse=True)
    assert lse.dtype == torch.float32 and tuple(lse.shape) == (1, 2, 1)
    scores = (q[0].float() @ cache[0, :2, 0].float().T) * scale
    assert torch.allclose(lse.cpu().view(2), torch.logsumexp(scores, -1), rtol=1e-3, atol=1e-3)
    expect = torch.softmax(scores, -1) @ cache[0, :2, 0, :512].float()
    assert torch.allclose(out.cpu().float().view(2, 512), expect, atol=1e-2)


def test_block_sizes_other_than_64_and_long_context_splits(device):
    _check(_mla_cfg("bs16", 2, 16, 50, 700, bs=16), 3, device)
    _check(_mla_cfg("bs128", 2, 32, 50, 900, bs=128), 4, device)
    _check(_mla_cfg("long", 1, 128, 6000, 9000), 6, device)


def test_small_and_odd_block_sizes_and_page_table_chunks(device):
    # block sizes below 16 or not a power of two take the kernel with the per-tile exchange
    _check(_mla_cfg("bs8", 2, 32, 40, 500, bs=8), 11, device)
    _check(_mla_cfg("bs24", 2, 16, 40, 500, bs=24), 12, device)
    # block 16: the page table is walked in chunks of 64 pages = 1024 tokens; contexts that end
    # just before, at and after chunk and sub-tile boundaries
    for i, L in enumerate((1023, 1024, 1025, 1056, 2047, 2049, 3100)):
        _check(_mla_cfg(f"chunks{L}", 1, 16, L, L, bs=16), 20 + i, device)
    # many short sequences: workgroups own several whole contexts
    _check(_mla_cfg("short", 96, 16, 1, 200, bs=16), 13, device)


def test_token_blocks_on_different_wavefronts_for_few_heads(device):
    # at most 64 heads: the two 16-token blocks of a sub-tile go to different wavefronts whose states are merged
    # at the end of a run.  Contexts long enough to span several workgroups (partials of merged states), head
    # counts that leave the last head block partly or wholly empty, and lengths whose last sub-tile has nothing
    # for the second token block.
    for heads, seed in ((48, 3), (64, 4), (24, 5), (16, 6)):
        _check(_mla_cfg(f"few{heads}", 5, heads, 1200, 4000), seed, device)
    for L in (1, 16, 17, 33, 48, 65):  # the generator draws lengths from [lo, hi]: pin them one by one
        _check(_mla_cfg(f"few32_L{L}", 2, 32, L, L), 50 + L, device)


def _rising_scores_case(heads, lo, hi, bs, device):
    cfg = _mla_cfg(f"ramp{heads}", 3, heads, lo, hi, bs=bs)
    inp = workloads.make_inputs(cfg, 31)
    lay = inp.layout
    inp.q[:, :, 512:] = 2.0
    for b in range(cfg.batch):
        o0, o1 = int(lay.ctx_offsets[b]), int(lay.ctx_offsets[b + 1])
        n = o1 - o0
        ramp = (torch.arange(n, dtype=torch.float32) * (9.0 / max(n, 1))).to(torch.bfloat16)
        inp.k_ctx[o0:o1, 0, 512:] = ramp[:, None]
    inp.k_new[:, 0, 512:] = 9.0
    kg, _, _, _ = fill_caches_gpu(inp, device)
    kc, _ = fill_caches_cpu(inp)
    out, lse = _decode_gpu(inp, kg, device)
    ref = oracle.aten_paged_decode(inp.q, kc, None, lay.block_table, lay.seq_lens, cfg.scale, dv=cfg.v_dim)
    assert_close_to_reference(out, ref, cfg.name)
    ref_lse = oracle.aten_paged_decode_lse(inp.q, kc, lay.block_table, lay.seq_lens, cfg.scale)
    assert torch.allclose(lse.cpu(), ref_lse, rtol=1e-3, atol=1e-3)


def test_scores_that_rise_along_the_context(device):
    # the rope dims of K carry a ramp and those of Q a constant, so the scores rise by about 120 log2 units from
    # the first token to the last: every running maximum is overtaken many times and whatever was accumulated
    # before has to be rescaled (or restarted) again and again; V = K[..., :512] is unaffected
    for heads, lo, hi, bs in ((128, 1500, 2500, 64), (16, 700, 900, 16), (32, 1500, 2500, 64)):
        _rising_scores_case(heads, lo, hi, bs, device)


def test_other_kernels_for_more_than_64_heads(device):
    # the default for more than 64 heads has four wavefronts of 512 registers with 32 heads each; "narrow" (eight
    # wavefronts, 16 heads each, P.V by dim block) and "heads" (16 heads per wavefront, both products by head
    # block) stay selectable
    for knob in ("narrow", "heads"):
        _select_kernel(knob)
        try:
            _check(_mla_cfg(f"mla128_{knob}", 3, 128, 100, 1500), 5, device)
            _check(_mla_cfg(f"mla80_{knob}", 2, 80, 1, 400), 120, device)
            _check(_mla_cfg(f"long_{knob}", 1, 128, 3000, 5000), 6, device)
            _rising_scores_case(128, 1500, 2500, 64, device)
        finally:
            _select_kernel("")


def test_head_counts_that_do_not_fill_their_blocks(device):
    # more than 64 heads, not a multiple of 16 nor of 128: the last 16-head block of the partial tiles is part
    # empty, the second workgroup of a team holds 72 heads; contexts long enough to be cut into partial runs
    _check(_mla_cfg("mla100", 2, 100, 2000, 5000), 31, device)
    _check(_mla_cfg("mla200", 2, 200, 1, 3000), 32, device)
    _check(_mla_cfg("mla72_many", 70, 72, 1, 300), 33, device)


def test_random_batches_with_empty_sequences_on_the_default_kernel(device):
    # Random batch sizes, head counts and length ranges; some sequences emptied (length 0: the output row is zero and
    # the LSE -inf, and the schedule gives them no share).  The oracle takes non-empty sequences, so the emptied rows
    # are checked by themselves and the others against a decode of the same batch without them.
    g = torch.Generator().manual_seed(2025)
    for case in range(6):
        batch = int(torch.randint(1, 90, (1,), generator=g))
        heads = (128, 96, 160, 256, 72, 112)[case]
        lo = int(torch.randint(1, 300, (1,), generator=g))
        hi = lo + int(torch.randint(1, 2000, (1,), generator=g))
        cfg = _mla_cfg(f"rand{case}_b{batch}_h{heads}", batch, heads, lo, hi)
        inp, kg, out, lse = _check(cfg, 1000 + case, device)
        lens = inp.layout.seq_lens.clone()
        empty = torch.rand(batch, generator=g) < 0.3
        if not bool(empty.any()):
            empty[0] = True
        lens[empty] = 0
        if int(lens.max()) == 0:
            continue
        out2, lse2 = _decode_gpu(inp, kg, device, seq_lens=lens)
        keep = ~empty
        assert torch.equal(out2[empty].cpu(), torch.zeros_like(out2[empty].cpu()))
        assert bool(torch.isinf(lse2[empty]).all()) and bool((lse2[empty] < 0).all())
        # the other rows: the same contexts, cut at other places by the schedule (fewer tiles to deal out)
        assert torch.allclose(out2[keep].float().cpu(), out[keep].float().cpu(), atol=2e-2)
        assert torch.allclose(lse2[keep].cpu(), lse[keep].cpu(), rtol=1e-3, atol=1e-3)


def test_many_short_sequences_with_128_heads(device):
    # more sequences than workgroups: a workgroup meets several contexts in one launch (whole ones written
    # directly, the pieces at both ends of its range as partials), and a batch beyond what one launch holds;
    # the default kernel and the eight-wavefront one
    for knob in ("", "narrow"):
        _select_kernel(knob)
        try:
            _check(_mla_cfg(f"mla128_b300_{knob}", 300, 128, 1, 150), 17, device)
            _check(_mla_cfg(f"mla128_b600_{knob}", 600, 128, 40, 100), 18, device)
        finally:
            _select_kernel("")
    _check(_mla_cfg("mla128_b1100", 1100, 128, 1, 40), 19, device)


def test_head_counts_page_table_chunk_boundaries_and_long_contexts(device):
    _check(_mla_cfg("d128", 3, 128, 100, 1500), 5, device)
    for heads in (2, 16, 80):
        _check(_mla_cfg(f"d{heads}", 2, heads, 1, 400), 60 + heads, device)
    for i, L in enumerate((1023, 1025, 2049, 3100)):  # page-table chunk boundaries (block 16: 1024 tokens per chunk)
        _check(_mla_cfg(f"chunks{L}", 1, 16, L, L, bs=16), 70 + i, device)
        _check(_mla_cfg(f"chunks128_{L}", 1, 128, L, L, bs=16), 80 + i, device)
    _check(_mla_cfg("short", 96, 16, 1, 200, bs=16), 13, device)
    _check(_mla_cfg("long", 1, 128, 6000, 9000), 6, device)


def _set_fold(on):
    """Whether the default kernel for more than 64 heads merges split contexts itself (1) or leaves them to a second
    launch (0); -1 gives the choice back to the environment."""
    from xllm_amd import capi
    assert capi.lib().xllm_mi355_debug_set(4, on) == 0


def test_merge_inside_the_decode_kernel_is_the_same_bits_as_the_merge_launch(device):
    # contexts cut across many workgroups, across two, whole ones, empty ones; head counts that fill one workgroup per
    # team, leave its last head block ragged, or need two workgroups per team; fewer tiles than workgroups
    g = torch.Generator().manual_seed(5)
    cases = [_mla_cfg("fold_b3", 3, 128, 100, 1500), _mla_cfg("fold_b9_long", 9, 128, 3000, 9000),
             _mla_cfg("fold_b40", 40, 128, 1, 700), _mla_cfg("fold_h80", 5, 80, 200, 4000),
             _mla_cfg("fold_h200", 4, 200, 500, 5000), _mla_cfg("fold_one", 1, 128, 12000, 12000),
             _mla_cfg("fold_tiny", 2, 128, 1, 90), _mla_cfg("fold_bs16", 6, 128, 300, 2500, bs=16)]
    for n, cfg in enumerate(cases):
        inp = workloads.make_inputs(cfg, 700 + n)
        kg, _, _, _ = fill_caches_gpu(inp, device)
        lens = inp.layout.seq_lens.clone()
        if cfg.batch > 4:
            lens[torch.rand(cfg.batch, generator=g) < 0.3] = 0
        results = []
        try:
            for on in (0, 1, 1):   # (twice with the merge inside: the counters it leaves behind must be back at zero)
                _set_fold(on)
                results.append(_decode_gpu(inp, kg, device, seq_lens=lens))
        finally:
            _set_fold(-1)
        assert ops.decode_status(device) == 0
        for out, lse in results[1:]:
            assert torch.equal(out.view(torch.int16), results[0][0].view(torch.int16)), cfg.name
            assert torch.equal(lse, results[0][1]), cfg.name
        if n in (0, 3, 6):
            live = torch.nonzero(lens > 0).flatten().tolist()
            ref = oracle.aten_paged_decode(inp.q[live].contiguous(), kg.cpu(), None, inp.layout.block_table[live].contiguous(),
                                           lens[live].contiguous(), cfg.scale, dv=cfg.v_dim)
            assert_close_to_reference(results[1][0][live], ref, cfg.name)
            dead = torch.nonzero(lens == 0).flatten().tolist()
            assert not results[1][0][dead].float().abs().any() and torch.isneginf(results[1][1][dead]).all()


def test_a_merging_workgroup_that_gives_up_is_reported(device):
    """The workgroups that merge a context wait for its pieces with a bounded poll.  With the bound at zero they give
    up at once (every wavefront still ends normally): the status call reports it, clears the counters the launch left
    behind, and the next launch is right again."""
    from xllm_amd import capi
    lib = capi.lib()
    cfg = _mla_cfg("fold_stall", 3, 128, 2500, 6000)
    inp = workloads.make_inputs(cfg, 77)
    kg, _, _, _ = fill_caches_gpu(inp, device)
    good, good_lse = _decode_gpu(inp, kg, device)
    assert ops.decode_status(device) == 0
    try:
        _set_fold(1)
        assert lib.xllm_mi355_debug_set(0, 0) == 0
        _decode_gpu(inp, kg, device)
        assert lib.xllm_mi355_debug_set(0, -1) == 0
        with pytest.raises(capi.XllmMi355Error, match="gave up"):
            ops.decode_status(device)
        assert ops.decode_status(device) == 0   # reported once, then cleared
        again, again_lse = _decode_gpu(inp, kg, device)
        assert torch.equal(again, good) and torch.equal(again_lse, good_lse) and ops.decode_status(device) == 0
    finally:
        assert lib.xllm_mi355_debug_set(0, -1) == 0
        _set_fold(-1)


def test_shard_merge_equals_full_decode(device):
    # ArtificialShardMergeMatchesFullCacheDecode (dcp_attention_merge_test.cpp:146-224): rtol/atol 1e-2, 1e-3
    cfg = _mla_cfg("merge", 4, 128, 256, 2000)
    inp, kg, full, full_lse = _check(cfg, 9, device)
    lay = inp.layout
    bs = cfg.block_size
    n_pages = (lay.seq_lens + bs - 1) // bs
    h = (n_pages + 1) // 2
    len_a = torch.minimum(lay.seq_lens, h * bs)
    len_b = lay.seq_lens - len_a
    table_b = torch.zeros_like(lay.block_table)
    for b in range(cfg.batch):
        nb = int(n_pages[b] - h[b])
        table_b[b, :nb] = lay.block_table[b, int(h[b]) : int(h[b]) + nb]
    oa, la = _decode_gpu(inp, kg, device, seq_lens=len_a)
    ob, lb = _decode_gpu(inp, kg, device, table=table_b, seq_lens=len_b)
    B, H = cfg.batch, cfg.n_q_heads
    merged, mlse = ops.merge_dcp_attention_shards(
        torch.stack([oa.view(B, 1, H, 512), ob.view(B, 1, H, 512)]),
        torch.stack([la.view(B, H, 1), lb.view(B, H, 1)]))
    assert torch.allclose(merged.view_as(full).float(), full.float(), rtol=1e-2, atol=1e-2)
    assert torch.allclose(mlse.view_as(full_lse), full_lse, rtol=1e-3, atol=1e-3)


def test_full_size_config5_sampled_parity(device):
    cfg = workloads.CONFIGS["mla_dsv3"]
    inp = workloads.make_inputs(cfg, 2, device=device)
    lay = inp.layout
    kg, _, _, _ = fill_caches_gpu(inp, device)
    out, lse = _decode_gpu(inp, kg, device)
    sample = [int(lay.seq_lens.argmin()), int(lay.seq_lens.argmax())]
    kc = kg.cpu()
    ref = oracle.aten_paged_decode(inp.q.cpu()[sample].contiguous(), kc, None,
                                   lay.block_table[sample].contiguous(), lay.seq_lens[sample].contiguous(),
                                   cfg.scale, dv=512)
    assert_close_to_reference(out[sample], ref, "cfg5 sample")
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()


def test_step_captured_in_a_graph_follows_new_metadata(device):
    # latent store + dense_decode captured once and replayed over rewritten persistent buffers
    # (runtime/dcu_graph_executor_impl.h:114-170); eager work and synchronisations between the replays
    cfg = _mla_cfg("graph", 6, 128, 100, 2500)
    inputs = [workloads.make_inputs(cfg, 400 + i) for i in range(2)]
    width = max(inp.layout.block_table.shape[1] for inp in inputs)
    blocks = max(inp.layout.num_blocks for inp in inputs)
    k_cache = torch.zeros(blocks, cfg.block_size, 1, 576, dtype=torch.bfloat16, device=device)
    table = torch.zeros(cfg.batch, width, dtype=torch.int32, device=device)
    lens = torch.zeros(cfg.batch, dtype=torch.int32, device=device)
    slots = torch.zeros(cfg.batch, dtype=torch.int32, device=device)
    q_nope = torch.zeros(cfg.batch, 1, cfg.n_q_heads, 512, dtype=torch.bfloat16, device=device)
    q_pe = torch.zeros(cfg.batch, 1, cfg.n_q_heads, 64, dtype=torch.bfloat16, device=device)
    k_new = torch.zeros(cfg.batch, 1, 576, dtype=torch.bfloat16, device=device)
    result = {}

    def load(inp):
        lay = inp.layout
        k_cache.zero_()
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=inp.k_ctx.to(device), value=None, k_cache=k_cache,
                                                            v_cache=None, slot_mapping=lay.ctx_slots.to(device)))
        table.zero_()
        table[:, : lay.block_table.shape[1]] = lay.block_table.to(device)
        lens.copy_(lay.seq_lens.to(device))
        slots.copy_(lay.new_slots.to(device))
        q = inp.q.to(device)
        q_nope.copy_(q[:, :, :512].reshape(cfg.batch, 1, cfg.n_q_heads, 512))
        q_pe.copy_(q[:, :, 512:].reshape(cfg.batch, 1, cfg.n_q_heads, 64))
        k_new.copy_(inp.k_new.to(device))

    def step():
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=k_new, value=None, k_cache=k_cache, v_cache=None,
                                                            slot_mapping=slots))
        p = ops.DenseDecodeParams(q_nope=q_nope, q_pe=q_pe, k_cache=k_cache, seqlens_k=lens, block_table=table,
                                  head_size_v=512, softmax_scale=cfg.scale)
        result["out"] = ops.dense_decode(p, max_seq_len=width * cfg.block_size)

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
    captured_out = result["out"]
    for rep in range(4):
        inp = inputs[rep % 2]
        load(inp)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = captured_out.clone()
        load(inp)
        step()
        torch.cuda.synchronize()
        assert torch.equal(replayed, result["out"]), f"replay {rep}"
        kc, _ = fill_caches_cpu(inp)
        lay = inp.layout
        ref = oracle.aten_paged_decode(inp.q, kc, None, lay.block_table, lay.seq_lens, cfg.scale, dv=512)
        assert_close_to_reference(replayed.view(cfg.batch, cfg.n_q_heads, 512), ref, f"mla graph replay {rep}")


def test_step_captured_in_a_graph_with_the_merge_inside_the_decode_kernel(device):
    # the same capture with the decode kernel merging split contexts itself: the counters it keeps in the workspace
    # must be back at zero after every replay
    try:
        _set_fold(1)
        test_step_captured_in_a_graph_follows_new_metadata(device)
    finally:
        _set_fold(-1)


def test_absorbed_attention_layer_captured_in_a_graph(device):
    # The decode branch of the reference's absorbed MLA attention (layers/dcu/deepseek_v2_attention.cpp:221-263,
    # 428-432) as one captured step: q_nope . w_kc, latent store, dense decode, output . w_vc -- replayed over
    # rewritten persistent buffers with eager work between the replays, every replay equal to the eager step bit
    # for bit and within the path's tolerance of the same chain on the oracle.  16 heads: a tensor-parallel shard.
    H = 16
    cfg = _mla_cfg("layer", 5, H, 100, 1500)
    g = torch.Generator().manual_seed(77)
    w_kc = (torch.randn(H, 128, 512, generator=g) / math.sqrt(128)).bfloat16()
    w_vc = (torch.randn(H, 512, 128, generator=g) / math.sqrt(512)).bfloat16()
    inputs = [workloads.make_inputs(cfg, 500 + i) for i in range(2)]
    qs = [(0.5 * torch.randn(cfg.batch, H, 192, generator=g)).bfloat16() for _ in inputs]
    width = max(inp.layout.block_table.shape[1] for inp in inputs)
    blocks = max(inp.layout.num_blocks for inp in inputs)
    k_cache = torch.zeros(blocks, cfg.block_size, 1, 576, dtype=torch.bfloat16, device=device)
    table = torch.zeros(cfg.batch, width, dtype=torch.int32, device=device)
    lens = torch.zeros(cfg.batch, dtype=torch.int32, device=device)
    slots = torch.zeros(cfg.batch, dtype=torch.int32, device=device)
    q = torch.zeros(cfg.batch, H, 192, dtype=torch.bfloat16, device=device)
    q_pe = torch.zeros(cfg.batch, 1, H, 64, dtype=torch.bfloat16, device=device)
    q_abs = torch.zeros(cfg.batch, H, 512, dtype=torch.bfloat16, device=device)
    proj = torch.zeros(cfg.batch, H, 128, dtype=torch.bfloat16, device=device)
    k_new = torch.zeros(cfg.batch, 1, 576, dtype=torch.bfloat16, device=device)
    wk, wv = w_kc.to(device), w_vc.to(device)

    def load(inp, qi):
        lay = inp.layout
        k_cache.zero_()
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=inp.k_ctx.to(device), value=None, k_cache=k_cache,
                                                            v_cache=None, slot_mapping=lay.ctx_slots.to(device)))
        table.zero_()
        table[:, : lay.block_table.shape[1]] = lay.block_table.to(device)
        lens.copy_(lay.seq_lens.to(device))
        slots.copy_(lay.new_slots.to(device))
        q.copy_(qi.to(device))
        q_pe.copy_(qi[:, :, 128:].reshape(cfg.batch, 1, H, 64).to(device))
        k_new.copy_(inp.k_new.to(device))

    def step():
        ops.absorbed_bmm(q[:, :, :128], wk, out=q_abs)
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=k_new, value=None, k_cache=k_cache, v_cache=None,
                                                            slot_mapping=slots))
        p = ops.DenseDecodeParams(q_nope=q_abs.view(cfg.batch, 1, H, 512), q_pe=q_pe, k_cache=k_cache, seqlens_k=lens,
                                  block_table=table, head_size_v=512, softmax_scale=cfg.scale)
        att = ops.dense_decode(p, max_seq_len=width * cfg.block_size)
        ops.absorbed_bmm(att.view(cfg.batch, H, 512), wv, out=proj)

    load(inputs[0], qs[0])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up outside the capture: workspace allocation, kernel attributes
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(4):
        inp, qi = inputs[rep % 2], qs[rep % 2]
        load(inp, qi)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = proj.clone()
        load(inp, qi)
        step()
        torch.cuda.synchronize()
        assert torch.equal(replayed, proj), f"replay {rep}"
        kc, _ = fill_caches_cpu(inp)
        lay = inp.layout
        qa, _ = oracle.absorbed_bmm(qi[:, :, :128], w_kc)
        att = oracle.aten_paged_decode(torch.cat([qa, qi[:, :, 128:]], dim=-1), kc, None, lay.block_table, lay.seq_lens,
                                       cfg.scale, dv=512)
        _, want = oracle.absorbed_bmm(att, w_vc)
        assert_close_to_reference(replayed, want, f"absorbed layer replay {rep}")


def _bmm_case(T, H, K, N, seed, wide=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, K + wide, generator=g).bfloat16()
    w = (torch.randn(H, K, N, generator=g) / math.sqrt(K)).bfloat16()
    return x[..., :K], w


@pytest.mark.parametrize("T,H,K,N,wide", [
    (64, 128, 128, 512, 64),   # q_nope [B, H, 128] (a slice of q [B, H, 192]) with w_kc_ of DeepSeek-V3
    (64, 128, 512, 128, 0),    # the decode output with w_vc_
    (1, 16, 128, 512, 64),     # one token, a tensor-parallel shard of the heads
    (67, 5, 256, 192, 0),      # token count that fills neither a wavefront nor a workgroup
    (100, 4, 128, 128, 0),     # two token blocks per wavefront, the second one ragged
    (200, 3, 128, 64, 8),      # four token blocks per wavefront
    (700, 2, 256, 64, 0),      # several workgroups along the tokens
    (300, 4, 128, 512, 64),    # many tokens: 128 output columns per workgroup
    (261, 3, 512, 128, 0),
])
def test_absorbed_products_either_side_of_the_decode(device, T, H, K, N, wide):
    # bmm(x.transpose(0, 1), w).transpose(0, 1) of layers/dcu/deepseek_v2_attention.cpp:428-430 and 231-238.
    # Tolerance: fp32 accumulation and one rounding to bf16: half a bf16 unit in the last place of the exact
    # value (2^-8 relative at most) plus 1e-4 for the order of the fp32 sums.
    x, w = _bmm_case(T, H, K, N, seed=T + K)
    ref, exact = oracle.absorbed_bmm(x, w)
    xd = x.to(device) if wide == 0 else torch.cat([x, torch.zeros(T, H, wide, dtype=x.dtype)], dim=-1).to(device)[..., :K]
    got = ops.absorbed_bmm(xd, w.to(device)).cpu()
    assert got.shape == (T, H, N) and got.dtype == torch.bfloat16
    err = (got.float() - exact).abs()
    bound = exact.abs() * 2.0 ** -8 + 1e-4
    assert (err <= bound).all(), f"max excess {(err - bound).max().item():.3e}"
    assert (got != ref).float().mean().item() < 0.01  # the two roundings agree except at ties of the sum order
    # into a slice of a wider output, as a caller that concatenates would
    out = torch.full((T, H, N + 8), 7.0, dtype=torch.bfloat16, device=device)
    ops.absorbed_bmm(xd, w.to(device), out=out[..., :N])
    assert torch.equal(out[..., :N].cpu(), got) and (out[..., N:] == 7.0).all()


def test_absorbed_product_selects_columns_bit_exactly_and_rejects_what_it_cannot_do(device):
    g = torch.Generator().manual_seed(3)
    T, H, K, N = 33, 6, 128, 64
    x = torch.randn(T, H, K, generator=g).bfloat16()
    perm = torch.stack([torch.randperm(K, generator=g)[:N] for _ in range(H)])
    sel = torch.zeros(H, K, N)
    for h in range(H):
        sel[h, perm[h], torch.arange(N)] = 1.0
    got = ops.absorbed_bmm(x.to(device), sel.bfloat16().to(device)).cpu()
    assert torch.equal(got, torch.stack([x[:, h, perm[h]] for h in range(H)], dim=1))
    assert ops.absorbed_bmm(x[:0].to(device), sel.bfloat16().to(device)).shape == (0, H, N)
    with pytest.raises(ValueError):
        ops.absorbed_bmm(x.to(device), sel[:, :64].bfloat16().to(device))        # K of x and w differ
    with pytest.raises(RuntimeError):
        ops.absorbed_bmm(x[..., :96].to(device), sel[:, :96].bfloat16().contiguous().to(device))  # K not a multiple of 128
    with pytest.raises(RuntimeError):
        ops.absorbed_bmm(x.half().to(device), sel.half().to(device))             # bf16 only
