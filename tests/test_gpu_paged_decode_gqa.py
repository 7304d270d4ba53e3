"""GPU parity of the GQA paged decode against the reference's libtorch CPU path (ATen oracle)."""
import math

import pytest
import torch

import oracle
from helpers import assert_close_to_reference, fill_caches_cpu, fill_caches_gpu
from xllm_amd import ops, workloads

pytestmark = pytest.mark.gpu


def _decode_gpu(inp, k_cache, v_cache, device, k_scale=None, v_scale=None, return_lse=True, table=None):
    cfg, lay = inp.cfg, inp.layout
    q = inp.q.to(device)
    out = torch.empty_like(q)
    table = (lay.block_table if table is None else table).to(device)
    out, lse = ops.batch_decode(q, k_cache, out, table, lay.seq_lens.to(device), v_cache=v_cache,
                                k_cache_quant_scale=k_scale, v_cache_quant_scale=v_scale,
                                scale=cfg.scale, return_lse=return_lse,
                                max_seq_len=int(lay.seq_lens.max()))
    torch.cuda.synchronize()
    return out, lse


def _check_config(cfg, seed, device, dtype=torch.bfloat16):
    inp = workloads.make_inputs(cfg, seed, dtype=dtype)
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    kc, vc = fill_caches_cpu(inp)
    assert torch.equal(kg.cpu(), kc) and torch.equal(vg.cpu(), vc), "cache bytes must be bit-exact"
    out, lse = _decode_gpu(inp, kg, vg, device)
    lay = inp.layout
    ref = oracle.aten_paged_decode(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale)
    mx, mean = assert_close_to_reference(out, ref, cfg.name)
    ref_lse = oracle.aten_paged_decode_lse(inp.q, kc, lay.block_table, lay.seq_lens, cfg.scale)
    assert torch.allclose(lse.cpu().view_as(ref_lse), ref_lse, rtol=1e-3, atol=1e-3)
    return mx, mean


def test_config1_tiny_write_then_attend(device):
    _check_config(workloads.CONFIGS["tiny"], 1234, device)


def test_config2_llama3_shape_reduced_batch(device):
    cfg = workloads.scaled(workloads.CONFIGS["llama3_8b"], batch=8)
    _check_config(cfg, 2024, device)


def test_config3_block128_group8_split_k(device):
    cfg = workloads.scaled(workloads.CONFIGS["long_b256"], batch=6)
    _check_config(cfg, 77, device)


def test_fp16_and_other_head_dims(device):
    for D, Hq, Hkv, dt in ((64, 8, 2, torch.float16), (256, 6, 1, torch.bfloat16), (128, 28, 4, torch.float16),
                           (128, 4, 4, torch.bfloat16), (128, 16, 8, torch.bfloat16), (64, 40, 2, torch.bfloat16)):
        cfg = workloads.DecodeConfig(f"d{D}_h{Hq}_{Hkv}", 5, Hq, Hkv, D, 32, 1, 700)
        _check_config(cfg, 100 + D + Hq, device, dtype=dt)


def test_fp32_query_over_fp32_pages(device):
    """What reshape_and_cache stores for an fp32 model can be attended: fp32 query, fp32 pages, fp32 output and LSE,
    against the libtorch decode in fp32 (no 16-bit rounding on either side: a tight tolerance).  The shapes of the
    reference's own fp32 cache cases (tests/core/kernels/dcu/reshape_paged_cache_test.cpp:135-158) and the three
    head dims; contexts shorter than a workgroup's four wavefronts, empty ones, a sliding window, the CSR form."""
    cases = [workloads.DecodeConfig("f32_ref_a", 4, 1, 1, 64, 16, 1, 40), workloads.DecodeConfig("f32_ref_b", 3, 4, 4, 128, 16, 1, 60),
             workloads.DecodeConfig("f32_gqa", 5, 8, 2, 128, 32, 100, 900), workloads.DecodeConfig("f32_d256", 2, 6, 3, 256, 16, 50, 300)]
    for n, cfg in enumerate(cases):
        inp = workloads.make_inputs(cfg, 50 + n, dtype=torch.float32)
        lay = inp.layout
        kg, vg, _, _ = fill_caches_gpu(inp, device)
        kc, vc = fill_caches_cpu(inp)
        assert kg.dtype == torch.float32 and torch.equal(kg.cpu(), kc) and torch.equal(vg.cpu(), vc)
        q = inp.q.to(device)
        table = lay.block_table.to(device)
        lens = lay.seq_lens.clone()
        if cfg.batch > 3:
            lens[1] = 0
        out, lse = ops.batch_decode(q, kg, torch.empty_like(q), table, lens.to(device), v_cache=vg, scale=cfg.scale,
                                    return_lse=True)
        live = torch.nonzero(lens > 0).flatten().tolist()
        ref = oracle.aten_paged_decode(inp.q[live].contiguous(), kc, vc, lay.block_table[live].contiguous(),
                                       lens[live].contiguous(), cfg.scale)
        assert out.dtype == torch.float32
        assert torch.allclose(out.cpu()[live], ref, rtol=2e-4, atol=2e-5), cfg.name
        ref_lse = oracle.aten_paged_decode_lse(inp.q[live].contiguous(), kc, lay.block_table[live].contiguous(),
                                               lens[live].contiguous(), cfg.scale)
        assert torch.allclose(lse.cpu().view(cfg.batch, -1)[live], ref_lse.view(len(live), -1), rtol=1e-4, atol=1e-4)
        dead = torch.nonzero(lens == 0).flatten().tolist()
        assert not out.cpu()[dead].abs().any() and torch.isneginf(lse.cpu().view(cfg.batch, -1)[dead]).all()
        if n == 2:
            # the window through the oracle on the trimmed context; the CSR form through the table form
            from helpers import trimmed_context
            win = 64
            first = torch.clamp(lay.seq_lens - 1 - win, min=0)
            wout, _ = ops.batch_decode(q, kg, torch.empty_like(q), table, lay.seq_lens.to(device), v_cache=vg,
                                       scale=cfg.scale, window_left=win)
            tk, tv, ttable, tlens = trimmed_context(kc, vc, lay.block_table, lay.seq_lens, first)
            wref = oracle.aten_paged_decode(inp.q, tk, tv, ttable, tlens, cfg.scale)
            assert torch.allclose(wout.cpu(), wref, rtol=2e-4, atol=2e-5)
            full, _ = ops.batch_decode(q, kg, torch.empty_like(q), table, lay.seq_lens.to(device), v_cache=vg, scale=cfg.scale)
            csr = ops.batch_decode_csr(q, kg, vg, lay.indptr.to(device), lay.indices.to(device),
                                       lay.last_page_len.to(device), -1, cfg.scale, torch.empty_like(q))
            assert torch.equal(csr, full)


def test_head_dim_64_with_fp8_pages_on_the_matrix_core_kernel(device):
    # fp8 pages with head dim 64: rows of 64 bytes, 64 tokens per stage multiplied as two halves of 32.  Group sizes
    # 1, 4, 16 and one that needs two head blocks; block sizes 16 / 64 / 128; lengths around the 16-, 32- and
    # 64-token boundaries; contexts long enough to span workers.
    for name, batch, Hq, Hkv, bs, lo, hi in (("g1", 4, 4, 4, 32, 1, 700), ("g4", 5, 32, 8, 16, 1, 3000),
                                             ("g16", 3, 16, 1, 128, 100, 2500), ("g20", 3, 40, 2, 64, 50, 1200),
                                             ("long", 3, 8, 2, 16, 20000, 40000)):
        _check_fp8(workloads.DecodeConfig(f"d64_fp8_{name}", batch, Hq, Hkv, 64, bs, lo, hi, cache_dtype="fp8"), 700 + Hq, device)
    for L in (1, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 96, 129):
        _check_fp8(workloads.DecodeConfig(f"d64_fp8_L{L}", 2, 8, 2, 64, 16, L, L, cache_dtype="fp8"), 800 + L, device)


def test_head_dim_256_on_the_matrix_core_kernel(device):
    # head dim 256 with a power-of-two block size >= 16: rows of 512 bytes, 8 tokens per stage in a 16-row score
    # block whose upper half is masked.  Group sizes 1, 4, 16 and one that needs two head blocks; block sizes
    # 16 / 64 / 128; contexts from one token to several workers' worth; lengths around the 8- and 16-token
    # boundaries; fp16; a sliding window through the same entry.
    for name, batch, Hq, Hkv, bs, lo, hi, dt in (("g1", 4, 4, 4, 32, 1, 700, torch.bfloat16),
                                                 ("g4", 5, 16, 4, 16, 1, 3000, torch.bfloat16),
                                                 ("g16", 3, 16, 1, 128, 100, 2500, torch.float16),
                                                 ("g20", 3, 40, 2, 64, 50, 1200, torch.bfloat16),
                                                 ("long", 3, 8, 2, 16, 10000, 20000, torch.bfloat16)):
        _check_config(workloads.DecodeConfig(f"d256_{name}", batch, Hq, Hkv, 256, bs, lo, hi), 500 + Hq, device, dtype=dt)
    for L in (1, 7, 8, 9, 15, 16, 17, 24, 33, 64, 65):
        _check_config(workloads.DecodeConfig(f"d256_L{L}", 2, 8, 2, 256, 16, L, L), 600 + L, device)


def test_merge_inside_the_decode_kernel(device):
    # the opt-in path where the worker that brings a context's last piece merges the partials (no merge launch):
    # contexts that span many workers, short ones that no worker splits, empty sequences, LSE, fp8, head dim 256,
    # and twice in a row on the same workspace (the arrival counters return to zero by themselves)
    from xllm_amd import capi
    lib = capi.lib()
    assert lib.xllm_mi355_debug_set(2, 1) == 0
    try:
        for rep in range(2):
            _check_config(workloads.scaled(workloads.CONFIGS["llama3_8b"], batch=8), 2024 + rep, device)
            _check_config(workloads.DecodeConfig("fold_long", 2, 8, 2, 128, 16, 20000, 30000), 11 + rep, device)
            _check_config(workloads.DecodeConfig("fold_short", 300, 8, 2, 128, 16, 1, 40), 12 + rep, device)
            _check_config(workloads.DecodeConfig("fold_d256", 3, 8, 2, 256, 16, 500, 6000), 13 + rep, device)
            _check_fp8(workloads.DecodeConfig("fold_fp8", 4, 32, 8, 128, 16, 300, 5000, cache_dtype="fp8"), 14 + rep, device)
        cfg = workloads.DecodeConfig("fold_empty", 5, 8, 2, 128, 16, 100, 3000)
        inp = workloads.make_inputs(cfg, 15)
        inp.layout.seq_lens[1] = 0
        inp.layout.seq_lens[4] = 0
        kg, vg, _, _ = fill_caches_gpu(inp, device)
        out, lse = _decode_gpu(inp, kg, vg, device)
        lay = inp.layout
        keep = torch.tensor([0, 2, 3])
        ref = oracle.aten_paged_decode(inp.q[keep], kg.cpu(), vg.cpu(), lay.block_table[keep], lay.seq_lens[keep], cfg.scale)
        assert_close_to_reference(out[keep.to(out.device)], ref, cfg.name)
        assert torch.all(out[1] == 0) and torch.all(out[4] == 0) and torch.all(torch.isneginf(lse[1])) and torch.all(torch.isneginf(lse[4]))
        assert ops.decode_status(device) == 0
    finally:
        assert lib.xllm_mi355_debug_set(2, 0) == 0


def test_head_dim_64_on_the_matrix_core_kernel(device):
    # head dim 64 with a power-of-two block size >= 16: rows of 128 bytes, 32 tokens per stage, two score blocks.
    # Group sizes that fill 1, 4 and all 16 columns and one that needs two head blocks; block sizes 16 / 64 / 128;
    # contexts from one token to several workers' worth; lengths around the 16- and 32-token boundaries; fp16.
    for name, batch, Hq, Hkv, bs, lo, hi, dt in (("g1", 4, 4, 4, 32, 1, 700, torch.bfloat16),
                                                 ("g4", 5, 32, 8, 16, 1, 3000, torch.bfloat16),
                                                 ("g16", 3, 16, 1, 128, 100, 2500, torch.float16),
                                                 ("g20", 3, 40, 2, 64, 50, 1200, torch.bfloat16),
                                                 ("long", 3, 8, 2, 16, 20000, 40000, torch.bfloat16)):
        _check_config(workloads.DecodeConfig(f"d64_{name}", batch, Hq, Hkv, 64, bs, lo, hi), 300 + Hq, device, dtype=dt)
    for L in (1, 15, 16, 17, 31, 32, 33, 48, 64, 65):
        _check_config(workloads.DecodeConfig(f"d64_L{L}", 2, 8, 2, 64, 16, L, L), 400 + L, device)


def test_reference_npu_case_130_tokens_block128(device):
    # Qwen35_27B_TP4_KvCacheCrosses128TokenBoundary (tests/core/kernels/npu/npu_xllm_ops_test.cpp:305-394):
    # seq 130, block 128, 3 blocks, Hq 6 / Hkv 1 / D 256, scale 1/16, table [[2, 0]], tolerance 5e-2
    g = torch.Generator().manual_seed(20260730)
    key = torch.randn(130, 1, 256, generator=g).to(torch.bfloat16)
    value = torch.randn(130, 1, 256, generator=g).to(torch.bfloat16)
    query = (0.25 * torch.randn(1, 6, 256, generator=g)).to(torch.bfloat16)
    slots = torch.cat([torch.arange(256, 384), torch.arange(0, 2)]).to(torch.int32)
    kg = torch.zeros(3, 128, 1, 256, dtype=torch.bfloat16, device=device)
    vg = torch.zeros_like(kg)
    ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=key.to(device), value=value.to(device),
                                                        k_cache=kg, v_cache=vg, slot_mapping=slots.to(device)))
    table = torch.tensor([[2, 0]], dtype=torch.int32, device=device)
    lens = torch.tensor([130], dtype=torch.int32, device=device)
    out = torch.empty(1, 6, 256, dtype=torch.bfloat16, device=device)
    ops.batch_decode(query.to(device), kg, out, table, lens, v_cache=vg, scale=1.0 / 16.0)
    # decode_attention_reference of the same test file (:109-125): fp32 matmul / softmax
    qf, kf, vf = query.float()[0], key.float()[:, 0], value.float()[:, 0]
    expected = torch.softmax(qf @ kf.T / 16.0, -1) @ vf
    assert torch.allclose(out.cpu().float()[0], expected, rtol=5e-2, atol=5e-2)
    assert (out.cpu().float()[0] - expected).abs().max() < 2e-2


def test_invariants_single_token_equal_rows_and_page_permutation(device):
    cfg = workloads.DecodeConfig("inv", 3, 8, 2, 128, 16, 200, 300)
    inp = workloads.make_inputs(cfg, 5)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    # (1) L = 1: the output is V[0] of the mapped KV head, bit for bit
    one = torch.ones_like(lay.seq_lens)
    q = inp.q.to(device)
    out = torch.empty_like(q)
    ops.batch_decode(q, kg, out, lay.block_table.to(device), one.to(device), v_cache=vg, scale=cfg.scale)
    for b in range(cfg.batch):
        v0 = vg[lay.block_table[b, 0].item(), 0]                         # [Hkv, D]
        assert torch.equal(out[b], v0.repeat_interleave(cfg.n_q_heads // cfg.n_kv_heads, 0))
    # (2) moving every page to another physical page, table permuted accordingly: identical bits
    out_a, _ = _decode_gpu(inp, kg, vg, device)
    perm = torch.randperm(lay.num_blocks, generator=torch.Generator().manual_seed(9))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(lay.num_blocks)
    kg2, vg2 = kg[perm.to(device)], vg[perm.to(device)]                  # new page j holds old page perm[j]
    table2 = inv[lay.block_table.long().clamp(0, lay.num_blocks - 1)].to(torch.int32)
    out_b, _ = _decode_gpu(inp, kg2.contiguous(), vg2.contiguous(), device, table=table2)
    assert torch.equal(out_a, out_b)
    # (3) all V rows equal -> out == that row; all K rows equal -> out == mean(V) (uniform softmax)
    vconst = torch.randn(cfg.n_kv_heads, cfg.head_dim, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    vg3 = vconst.to(device).expand_as(vg).contiguous()
    out_c, _ = _decode_gpu(inp, kg, vg3, device)
    expect = vconst.repeat_interleave(cfg.n_q_heads // cfg.n_kv_heads, 0).float()
    assert (out_c.cpu().float() - expect).abs().max() <= 2 ** -7 * expect.abs().max()


def test_table_padding_is_never_read_and_strided_views(device):
    cfg = workloads.DecodeConfig("pad", 4, 8, 4, 128, 16, 30, 400)
    inp = workloads.make_inputs(cfg, 31)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    out_a, _ = _decode_gpu(inp, kg, vg, device)
    # poison every unused column with huge / negative page ids
    t = lay.block_table.clone()
    for b in range(cfg.batch):
        n = (int(lay.seq_lens[b]) + cfg.block_size - 1) // cfg.block_size
        t[b, n:] = torch.tensor([-1, 2 ** 30, -2 ** 31][: t.shape[1] - n] + [7] * max(0, t.shape[1] - n - 3))
    out_b, _ = _decode_gpu(inp, kg, vg, device, table=t)
    assert torch.equal(out_a, out_b)
    # a wide persistent table buffer (row stride > width) and a strided query, as under graph capture
    wide = torch.full((cfg.batch, 1024), -1, dtype=torch.int32, device=device)
    wide[:, : t.shape[1]] = lay.block_table.to(device)
    qkv = torch.zeros(cfg.batch, 3 * cfg.n_q_heads * cfg.head_dim, dtype=torch.bfloat16, device=device)
    qview = qkv[:, : cfg.n_q_heads * cfg.head_dim].view(cfg.batch, cfg.n_q_heads, cfg.head_dim)
    qview.copy_(inp.q.to(device))
    out_c = torch.empty(cfg.batch, cfg.n_q_heads, cfg.head_dim, dtype=torch.bfloat16, device=device)
    ops.batch_decode(qview, kg, out_c, wide[:, : t.shape[1]], lay.seq_lens.to(device), v_cache=vg,
                     scale=cfg.scale, max_seq_len=int(lay.seq_lens.max()))
    assert torch.equal(out_a, out_c)


def test_csr_form_matches_block_table_form_and_csr_oracle(device):
    cfg = workloads.scaled(workloads.CONFIGS["llama3_8b"], batch=5, len_lo=17, len_hi=900)
    inp = workloads.make_inputs(cfg, 8)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    out_a, _ = _decode_gpu(inp, kg, vg, device)
    q = inp.q.to(device)
    out_b = torch.empty_like(q)
    ops.batch_decode_csr(q, kg, vg, lay.indptr.to(device), lay.indices.to(device),
                         lay.last_page_len.to(device), -1, cfg.scale, out_b, max_seq_len=int(lay.seq_lens.max()))
    assert torch.equal(out_a, out_b)
    ref = oracle.aten_paged_decode_csr(inp.q, kg.cpu(), vg.cpu(), lay.indptr, lay.indices, lay.last_page_len)
    assert_close_to_reference(out_b, ref, "csr")
    # CSR -> table builder against the C oracle
    tg, lg = ops.build_block_table_from_paged_kv(lay.indptr.to(device), lay.indices.to(device),
                                                 lay.last_page_len.to(device), lay.block_table.shape[1],
                                                 cfg.block_size)
    tc, lc = oracle.build_block_table(lay.indptr, lay.indices, lay.last_page_len, lay.block_table.shape[1],
                                      cfg.block_size)
    assert torch.equal(tg.cpu(), tc) and torch.equal(lg.cpu(), lc) and torch.equal(lc, lay.seq_lens)


def _check_fp8(cfg, seed, device):
    inp = workloads.make_inputs(cfg, seed)
    lay = inp.layout
    kg, vg, ks, vs = fill_caches_gpu(inp, device, cache_dtype=torch.float8_e4m3fn)
    kc, vc = fill_caches_cpu(inp, torch.float8_e4m3fn, ks.cpu(), vs.cpu())
    assert torch.equal(kg.view(torch.uint8).cpu(), kc) and torch.equal(vg.view(torch.uint8).cpu(), vc)
    out, lse = _decode_gpu(inp, kg, vg, device, ks, vs)
    ref = oracle.aten_paged_decode(inp.q, kc.view(torch.float8_e4m3fn), vc.view(torch.float8_e4m3fn),
                                   lay.block_table, lay.seq_lens, cfg.scale, ks.cpu(), vs.cpu())
    assert_close_to_reference(out, ref, "fp8 " + cfg.name)


def test_fp8_kv_cache_decode(device):
    cfg = workloads.scaled(workloads.CONFIGS["fp8_kv"], batch=4, len_lo=300, len_hi=3000)
    _check_fp8(cfg, 4242, device)


def test_head_dim_256_with_fp8_pages_on_the_matrix_core_kernel(device):
    # rows of 256 bytes: 16 tokens per stage, one score block, the second half of the 32-token P.V masked.  Group
    # sizes 1, 4, 16 and one with two head blocks; block sizes 16 / 64; contexts from one token to many workers'
    # worth; lengths around the 16-token boundaries; the dot-product kernel on the same inputs agrees closely.
    for name, batch, Hq, Hkv, bs, lo, hi in (("g1", 4, 4, 4, 32, 1, 700), ("g4", 5, 16, 4, 16, 1, 3000),
                                             ("g16", 3, 16, 1, 64, 100, 2500), ("g20", 3, 40, 2, 64, 50, 1200),
                                             ("long", 3, 8, 2, 16, 10000, 20000)):
        _check_fp8(workloads.DecodeConfig(f"d256_fp8_{name}", batch, Hq, Hkv, 256, bs, lo, hi, cache_dtype="fp8"),
                   800 + Hq, device)
    for L in (1, 15, 16, 17, 31, 32, 33, 48, 65):
        _check_fp8(workloads.DecodeConfig(f"d256_fp8_L{L}", 2, 8, 2, 256, 16, L, L, cache_dtype="fp8"), 900 + L, device)


def test_kv_head_counts_and_the_heads_read_side_by_side(device):
    # The four workers of a workgroup read four adjacent KV heads side by side when the KV heads come in fours
    # (12 = three groups), two when they come in pairs (6, 2), one otherwise (3, 1); contexts long enough to be cut
    # into partial runs, and many short ones, so that the merge finds every head block's partials with the right
    # member of every workgroup.
    for Hq, Hkv in ((24, 12), (12, 6), (6, 3), (48, 12), (4, 2), (7, 1)):
        cfg = workloads.DecodeConfig(f"lock_h{Hq}_{Hkv}", 6, Hq, Hkv, 128, 16, 900, 5000)
        _check_config(cfg, 700 + Hq + Hkv, device)
        cfg = workloads.DecodeConfig(f"lock_short_h{Hq}_{Hkv}", 200, Hq, Hkv, 128, 16, 1, 120)
        _check_config(cfg, 800 + Hq + Hkv, device)
    cfg = workloads.DecodeConfig("lock_fp8_h24_12", 6, 24, 12, 128, 16, 900, 5000, cache_dtype="fp8")
    _check_fp8(cfg, 901, device)


def test_whole_contexts_in_one_workgroup_every_group_size(device):
    # Few short sequences: every context is a single item, so one workgroup sees it whole and
    # writes the caller's output itself (no partials, no merge), with most wavefronts idle.
    # Then contexts of a few items each, enough of them that workgroups own several whole ones.
    for Hq, Hkv in ((4, 4), (8, 4), (12, 4), (16, 4), (20, 4), (28, 4), (32, 4)):
        for batch, hi in ((5, 64), (160, 400)):
            cfg = workloads.DecodeConfig(f"whole_h{Hq}_{Hkv}_b{batch}", batch, Hq, Hkv, 128, 32, 1, hi)
            _check_config(cfg, 300 + Hq + batch, device)
    for Hq, Hkv in ((8, 4), (28, 4), (32, 4)):
        cfg = workloads.DecodeConfig(f"whole_fp8_h{Hq}_{Hkv}", 5, Hq, Hkv, 128, 32, 1, 64, cache_dtype="fp8")
        _check_fp8(cfg, 400 + Hq, device)
        cfg = workloads.DecodeConfig(f"whole_fp8_h{Hq}_{Hkv}_b96", 96, Hq, Hkv, 128, 32, 1, 500, cache_dtype="fp8")
        _check_fp8(cfg, 500 + Hq, device)
    for D, Hq, Hkv in ((64, 16, 2), (256, 8, 1)):
        cfg = workloads.DecodeConfig(f"whole_d{D}", 5, Hq, Hkv, D, 16, 1, 64)
        _check_config(cfg, 600 + D, device)


def test_block_sizes_and_page_table_chunks_of_both_kernels(device):
    # head_dim 128: block sizes >= 16 that are powers of two take the matrix-core kernel (which walks
    # the page table in chunks of 64 pages), the others the dot-product kernel
    for bs in (1, 8, 16, 24, 32, 64, 256):
        cfg = workloads.DecodeConfig(f"bs{bs}", 3, 8, 2, 128, bs, 30, 900)
        _check_config(cfg, 700 + bs, device)
    # contexts that end just before, at and after chunk (1024 tokens at block 16) and stage boundaries
    for i, L in enumerate((1023, 1024, 1025, 1040, 2047, 2048, 2049, 5000)):
        cfg = workloads.DecodeConfig(f"chunks{L}", 1, 4, 1, 128, 16, L, L)
        _check_config(cfg, 800 + i, device)
    for i, L in enumerate((2047, 2048, 2049, 2080)):
        cfg = workloads.DecodeConfig(f"chunks_fp8_{L}", 1, 4, 1, 128, 16, L, L, cache_dtype="fp8")
        _check_fp8(cfg, 850 + i, device)
    # more than 16 query heads per KV head: two head blocks per KV head
    cfg = workloads.DecodeConfig("group24", 2, 48, 2, 128, 16, 100, 600)
    _check_config(cfg, 900, device)


def test_random_shapes_with_empty_sequences(device):
    # Random head counts, block sizes, batch sizes and length ranges on the matrix-core kernel, each decoded a second
    # time with some sequences emptied: their rows are zero with an LSE of -inf, the others agree with the first
    # decode (the same contexts, cut at other places because fewer stages are dealt out).
    g = torch.Generator().manual_seed(77)
    shapes = ((32, 8, 128), (16, 4, 128), (24, 12, 128), (12, 6, 64), (40, 2, 128), (8, 8, 128), (9, 3, 128), (16, 4, 256))
    for case, (Hq, Hkv, D) in enumerate(shapes):
        batch = int(torch.randint(1, 150, (1,), generator=g))
        bs = (16, 32, 64, 128)[int(torch.randint(0, 4, (1,), generator=g))]
        lo = int(torch.randint(1, 200, (1,), generator=g))
        hi = lo + int(torch.randint(1, 1500, (1,), generator=g))
        cfg = workloads.DecodeConfig(f"rand{case}_h{Hq}_{Hkv}_d{D}_b{batch}_bs{bs}", batch, Hq, Hkv, D, bs, lo, hi)
        _check_config(cfg, 1100 + case, device)
        inp = workloads.make_inputs(cfg, 1100 + case)
        lay = inp.layout
        kg, vg, _, _ = fill_caches_gpu(inp, device)
        out, lse = _decode_gpu(inp, kg, vg, device)
        lens = lay.seq_lens.clone()
        empty = torch.rand(batch, generator=g) < 0.3
        empty[int(torch.randint(0, batch, (1,), generator=g))] = True
        lens[empty] = 0
        q = inp.q.to(device)
        out2 = torch.full_like(q, 7.0)
        out2, lse2 = ops.batch_decode(q, kg, out2, lay.block_table.to(device), lens.to(device), v_cache=vg,
                                      scale=cfg.scale, return_lse=True)
        torch.cuda.synchronize()
        assert (out2[empty] == 0).all() and torch.isneginf(lse2[empty]).all()
        keep = ~empty
        if bool(keep.any()):
            assert torch.allclose(out2[keep].float().cpu(), out[keep].float().cpu(), atol=2e-2)
            assert torch.allclose(lse2[keep].cpu().view(-1), lse[keep].cpu().view(-1), rtol=1e-3, atol=1e-3)


def test_empty_sequence_and_argument_errors(device):
    cfg = workloads.DecodeConfig("e", 3, 8, 2, 128, 16, 10, 50)
    inp = workloads.make_inputs(cfg, 2)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    lens = lay.seq_lens.clone()
    lens[1] = 0
    q = inp.q.to(device)
    out = torch.full_like(q, 7.0)
    out, lse = ops.batch_decode(q, kg, out, lay.block_table.to(device), lens.to(device), v_cache=vg,
                                scale=cfg.scale, return_lse=True)
    assert (out[1] == 0).all() and torch.isneginf(lse[1]).all()
    with pytest.raises(Exception):
        ops.batch_decode(q[:, :, :100], kg, out, lay.block_table.to(device), lens.to(device), v_cache=vg)
    with pytest.raises(Exception):
        ops.batch_decode(q.cpu(), kg, out, lay.block_table.to(device), lens.to(device), v_cache=vg)


def test_full_size_config2_split_invariance_and_sampled_parity(device):
    """The llama3_8b workload (batch 64, 32 / 8 heads, block 16, contexts of 512 to 4096 tokens) at full size: (a) sequences sampled from the batch agree with the oracle,
    (b) LSE-merging the decode of two context halves equals the unsplit decode."""
    cfg = workloads.CONFIGS["llama3_8b"]
    inp = workloads.make_inputs(cfg, 2, device=device)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    out, lse = _decode_gpu(inp, kg, vg, device)
    sample = [0, 17, 41, 63]
    kc, vc = kg.cpu(), vg.cpu()
    ref = oracle.aten_paged_decode(inp.q.cpu()[sample].contiguous(), kc, vc,
                                   lay.block_table[sample].contiguous(), lay.seq_lens[sample].contiguous(),
                                   cfg.scale)
    assert_close_to_reference(out[sample], ref, "cfg2 sample")
    # halves: first ceil(n/2) pages, and the rest as its own table
    bs = cfg.block_size
    n_pages = (lay.seq_lens + bs - 1) // bs
    h = (n_pages + 1) // 2
    len_a = torch.minimum(lay.seq_lens, h * bs)
    len_b = lay.seq_lens - len_a
    table_b = torch.zeros_like(lay.block_table)
    for b in range(cfg.batch):
        nb = int(n_pages[b] - h[b])
        table_b[b, :nb] = lay.block_table[b, int(h[b]) : int(h[b]) + nb]
    q = inp.q
    parts_o, parts_l = [], []
    for table, lens in ((lay.block_table, len_a), (table_b, len_b)):
        o = torch.empty_like(q)
        o, l = ops.batch_decode(q, kg, o, table.to(device), lens.to(device), v_cache=vg, scale=cfg.scale,
                                return_lse=True, max_seq_len=int(lens.max()))
        parts_o.append(o.view(cfg.batch, 1, cfg.n_q_heads, cfg.head_dim))
        parts_l.append(l.view(cfg.batch, cfg.n_q_heads, 1))
    merged, mlse = ops.merge_dcp_attention_shards(torch.stack(parts_o), torch.stack(parts_l))
    diff = (merged.view_as(out).float() - out.float()).abs()
    assert diff.max() <= 1e-2 and diff.mean() <= 1e-3
    assert torch.allclose(mlse.view_as(lse), lse, rtol=1e-3, atol=1e-3)


def test_long_item_lists_of_the_matrix_core_kernel(device):
    # Batches that give every pair of wavefronts of the matrix-core kernel 140 to 330 stages (the loading
    # wavefront laps the ring of its pair dozens of times): sampled sequences against the oracle, launches in a
    # row on one workspace bit-identical, a captured launch replayed with eager launches in between.
    def twice(run):
        first = run()
        again = run()
        torch.cuda.synchronize()
        assert torch.equal(first, again)
        return first

    for batch, lo, hi in ((64, 3000, 6000), (150, 3000, 6000)):
        cfg = workloads.DecodeConfig(f"long_b{batch}", batch, 32, 8, 128, 16, lo, hi)
        inp = workloads.make_inputs(cfg, 900 + batch, device=device)
        lay = inp.layout
        kg, vg, _, _ = fill_caches_gpu(inp, device)
        out = twice(lambda: _decode_gpu(inp, kg, vg, device)[0])
        sample = list(range(0, batch, 5)) + list(range(batch - 12, batch))
        ref = oracle.aten_paged_decode(inp.q.cpu()[sample].contiguous(), kg.cpu(), vg.cpu(),
                                       lay.block_table[sample].contiguous(), lay.seq_lens[sample].contiguous(), cfg.scale)
        assert_close_to_reference(out[sample], ref, cfg.name)
        if batch == 64:
            q, table, lens = inp.q.to(device), lay.block_table.to(device), lay.seq_lens.to(device)
            captured = torch.zeros_like(q)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                ops.batch_decode(q, kg, captured, table, lens, v_cache=vg, scale=cfg.scale, max_seq_len=hi)
            for rep in range(3):
                captured.zero_()
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(captured, out), f"replay {rep}"
                assert torch.equal(_decode_gpu(inp, kg, vg, device)[0], out)
    # fp8 pages (stages of 32 tokens) and query chunks in the MFMA columns
    cfg = workloads.DecodeConfig("long_fp8", 192, 32, 8, 128, 16, 2000, 4000, cache_dtype="fp8")
    inp = workloads.make_inputs(cfg, 77, device=device)
    lay = inp.layout
    kg, vg, ks, vs = fill_caches_gpu(inp, device, cache_dtype=torch.float8_e4m3fn)
    out = twice(lambda: _decode_gpu(inp, kg, vg, device, ks, vs)[0])
    sample = list(range(0, 192, 17)) + list(range(184, 192))
    ref = oracle.aten_paged_decode(inp.q.cpu()[sample].contiguous(), kg.cpu(), vg.cpu(), lay.block_table[sample].contiguous(),
                                   lay.seq_lens[sample].contiguous(), cfg.scale, ks.cpu(), vs.cpu())
    assert_close_to_reference(out[sample], ref, cfg.name)

    cfg = workloads.DecodeConfig("long_chunks", 64, 32, 8, 128, 16, 3000, 6000)
    inp = workloads.make_inputs(cfg, 78, device=device)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    g = torch.Generator().manual_seed(5)
    q_lens = torch.randint(1, 5, (cfg.batch,), generator=g)
    cu = torch.tensor([0] + list(q_lens.cumsum(0)), dtype=torch.int32)
    q = (torch.randn(int(cu[-1]), 32, 128, generator=g) * cfg.sigma).to(torch.bfloat16).to(device)
    out = twice(lambda: ops.paged_forward(q, torch.empty_like(q), kg, vg, lay.block_table.to(device), lay.seq_lens.to(device),
                                          cu.to(device), scale=cfg.scale, is_causal=True, max_query_len=4))
    ref = oracle.aten_paged_forward(q.cpu(), kg.cpu(), vg.cpu(), lay.block_table, lay.seq_lens, cu, cfg.scale, causal=True)
    assert_close_to_reference(out, ref, cfg.name)


def test_batches_larger_than_a_workgroup_and_than_a_launch(device):
    # more sequences than threads in a workgroup (the item prefix then sums several sequences per thread and
    # the workers read the lengths from memory), and more than one launch holds (2048): both kernels
    for name, batch, Hq, Hkv, D, bs, hi in (("b700_mfma", 700, 8, 2, 128, 16, 200), ("b700_rows", 700, 8, 2, 64, 16, 120),
                                            ("b2300_mfma", 2300, 4, 1, 128, 16, 70), ("b2300_rows", 2300, 4, 2, 256, 8, 40)):
        cfg = workloads.DecodeConfig(name, batch, Hq, Hkv, D, bs, 1, hi)
        _check_config(cfg, 40 + batch + D, device)


def test_short_query_chunks_through_the_decode_kernels(device):
    # chunked prefill / speculative-decoding verification (layers/dcu/flash_attention.cpp:447-545): up to 16 query
    # tokens per sequence, the chunk being the tail of its context; both decode kernels, causal and not
    for name, Hq, Hkv, D, bs, lo, hi, batch in (("mfma", 32, 8, 128, 16, 1, 900, 7), ("rows", 8, 2, 64, 32, 1, 500, 5),
                                                ("long", 16, 2, 128, 128, 2000, 5000, 2)):
        cfg = workloads.DecodeConfig(f"chunks_{name}", batch, Hq, Hkv, D, bs, lo, hi)
        inp = workloads.make_inputs(cfg, 50 + batch)
        lay = inp.layout
        g = torch.Generator().manual_seed(99)
        q_lens = [int(torch.randint(1, min(16, int(L)) + 1, (1,), generator=g)) for L in lay.seq_lens]
        cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
        q = (torch.randn(int(cu[-1]), Hq, D, generator=g) * cfg.sigma).to(torch.bfloat16)
        kg, vg, _, _ = fill_caches_gpu(inp, device)
        kc, vc = fill_caches_cpu(inp)
        for causal in (True, False):
            out = ops.paged_forward(q.to(device), torch.empty_like(q, device=device), kg, vg,
                                    lay.block_table.to(device), lay.seq_lens.to(device), cu.to(device),
                                    scale=cfg.scale, is_causal=causal)
            torch.cuda.synchronize()
            ref = oracle.aten_paged_forward(q, kc, vc, lay.block_table, lay.seq_lens, cu, cfg.scale, causal=causal)
            assert_close_to_reference(out, ref, f"{cfg.name} causal={causal}")
    # chunks whose (token, head) pairs fit the 16 columns of the matrix-core kernel share one pass over the pages:
    # group 4 with up to 4 tokens, group 8 with up to 2, one KV head per query head with up to 16; fp16; a
    # sequence without query tokens; bounds larger than the chunks
    for name, Hq, Hkv, bs, lo, hi, batch, bound, dt in (("g4", 32, 8, 16, 1, 900, 9, 4, torch.bfloat16),
                                                        ("g8", 64, 8, 128, 300, 3000, 4, 2, torch.bfloat16),
                                                        ("g1", 4, 4, 32, 20, 400, 5, 16, torch.float16),
                                                        ("g2", 8, 4, 16, 1, 2000, 6, 8, torch.bfloat16),
                                                        # longer chunks take several column blocks per KV head
                                                        ("g4_16", 32, 8, 16, 40, 1200, 5, 16, torch.bfloat16),
                                                        ("g8_7", 64, 8, 64, 30, 800, 4, 7, torch.bfloat16)):
        cfg = workloads.DecodeConfig(f"packed_{name}", batch, Hq, Hkv, 128, bs, lo, hi)
        inp = workloads.make_inputs(cfg, 70 + batch, dtype=dt)
        lay = inp.layout
        g = torch.Generator().manual_seed(7 + batch)
        q_lens = [int(torch.randint(1, min(bound, int(L)) + 1, (1,), generator=g)) for L in lay.seq_lens]
        q_lens[1] = 0                                   # a sequence that takes no part in this step
        cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
        q = (torch.randn(int(cu[-1]), Hq, 128, generator=g) * cfg.sigma).to(dt)
        kg, vg, _, _ = fill_caches_gpu(inp, device)
        kc, vc = fill_caches_cpu(inp)
        for causal in (True, False):
            out = ops.paged_forward(q.to(device), torch.empty_like(q, device=device), kg, vg,
                                    lay.block_table.to(device), lay.seq_lens.to(device), cu.to(device),
                                    scale=cfg.scale, is_causal=causal, max_query_len=bound)
            torch.cuda.synchronize()
            ref = oracle.aten_paged_forward(q, kc, vc, lay.block_table, lay.seq_lens, cu, cfg.scale, causal=causal)
            assert_close_to_reference(out, ref, f"{cfg.name} causal={causal}")
            spread = ops.paged_forward(q.to(device), torch.empty_like(q, device=device), kg, vg,
                                       lay.block_table.to(device), lay.seq_lens.to(device), cu.to(device),
                                       scale=cfg.scale, is_causal=causal)      # one entry per token
            torch.cuda.synchronize()
            assert (out.float() - spread.float()).abs().max() < 2e-2
    # one token per sequence is plain decode, bit for bit
    cfg = workloads.DecodeConfig("chunks_one", 6, 32, 8, 128, 16, 1, 700)
    inp = workloads.make_inputs(cfg, 8)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    ones = torch.arange(cfg.batch + 1, dtype=torch.int32, device=device)
    q = inp.q.to(device)
    a = ops.paged_forward(q, torch.empty_like(q), kg, vg, lay.block_table.to(device), lay.seq_lens.to(device), ones,
                          scale=cfg.scale)
    b, _ = ops.batch_decode(q, kg, torch.empty_like(q), lay.block_table.to(device), lay.seq_lens.to(device),
                            v_cache=vg, scale=cfg.scale)
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_step_captured_in_a_graph_follows_new_metadata(device):
    # The reference's graph executor replays one captured decode step while it rewrites the metadata in
    # persistent buffers (runtime/dcu_graph_executor_impl.h:114-170).  Capture cache write + decode once, then
    # replay with other lengths, slots and query rows; eager work and synchronisations sit between the replays
    # and every replay is checked against the eager result of the same inputs.
    cfg = workloads.DecodeConfig("graph", 12, 32, 8, 128, 16, 50, 1500)
    inputs = [workloads.make_inputs(cfg, 300 + i) for i in range(3)]
    width = max(inp.layout.block_table.shape[1] for inp in inputs)
    blocks = max(inp.layout.num_blocks for inp in inputs)
    shape = (blocks, cfg.block_size, cfg.n_kv_heads, cfg.head_dim)
    k_cache = torch.zeros(shape, dtype=torch.bfloat16, device=device)
    v_cache = torch.zeros_like(k_cache)
    # persistent buffers of the captured step
    table = torch.zeros(cfg.batch, width, dtype=torch.int32, device=device)
    lens = torch.zeros(cfg.batch, dtype=torch.int32, device=device)
    slots = torch.zeros(cfg.batch, dtype=torch.int32, device=device)
    q = torch.zeros(cfg.batch, cfg.n_q_heads, cfg.head_dim, dtype=torch.bfloat16, device=device)
    k_new = torch.zeros(cfg.batch, cfg.n_kv_heads, cfg.head_dim, dtype=torch.bfloat16, device=device)
    v_new = torch.zeros_like(k_new)
    out = torch.zeros_like(q)

    def load(inp):  # what the executor does before a replay: fill the caches' context, rewrite the metadata
        lay = inp.layout
        k_cache.zero_()
        v_cache.zero_()
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(
            key=inp.k_ctx.to(device), value=inp.v_ctx.to(device), k_cache=k_cache, v_cache=v_cache,
            slot_mapping=lay.ctx_slots.to(device)))
        table.zero_()
        table[:, : lay.block_table.shape[1]] = lay.block_table.to(device)
        lens.copy_(lay.seq_lens.to(device))
        slots.copy_(lay.new_slots.to(device))
        q.copy_(inp.q.to(device))
        k_new.copy_(inp.k_new.to(device))
        v_new.copy_(inp.v_new.to(device))

    def step():
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=k_new, value=v_new, k_cache=k_cache, v_cache=v_cache,
                                                            slot_mapping=slots))
        ops.batch_decode(q, k_cache, out, table, lens, v_cache=v_cache, scale=cfg.scale,
                         max_seq_len=width * cfg.block_size)

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
    for rep in range(6):
        inp = inputs[rep % 3]
        load(inp)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.clone()
        out.zero_()
        load(inp)
        step()
        torch.cuda.synchronize()
        assert torch.equal(replayed, out), f"replay {rep}"
        kc, vc = fill_caches_cpu(inp)
        lay = inp.layout
        ref = oracle.aten_paged_decode(inp.q, kc[: blocks], vc[: blocks], lay.block_table, lay.seq_lens, cfg.scale)
        assert_close_to_reference(replayed, ref, f"graph replay {rep}")


def test_norm_rope_cache_write_and_decode_captured_in_a_graph(device):
    # The attention layer's decode step as the reference runs it (layers/common/qwen2_attention.cpp:144-186 then the
    # attention op): fused q/k norm + RoPE on the qkv buffer with the cache write folded in, then the paged decode
    # reading q as a strided view of that buffer.  Captured once, replayed over rewritten buffers, every replay
    # equal to the eager step bit for bit and within the path's tolerance of the same chain on the oracle.
    cfg = workloads.DecodeConfig("layer", 9, 32, 8, 128, 16, 50, 1200)
    Hq, Hkv, D, B = cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.batch
    g = torch.Generator().manual_seed(9)
    qw, kw = (1 + 0.1 * torch.randn(D, generator=g)).bfloat16(), (1 + 0.1 * torch.randn(D, generator=g)).bfloat16()
    ang = torch.rand(2048, D // 2, generator=g) * 6.28
    cos_sin = torch.cat([ang.cos(), ang.sin()], 1)
    inputs = [workloads.make_inputs(cfg, 600 + i) for i in range(2)]
    raws = [torch.cat([inp.q.reshape(B, -1), inp.k_new.reshape(B, -1), inp.v_new.reshape(B, -1)], 1).contiguous() for inp in inputs]
    width = max(inp.layout.block_table.shape[1] for inp in inputs)
    blocks = max(inp.layout.num_blocks for inp in inputs)
    k_cache = torch.zeros(blocks, cfg.block_size, Hkv, D, dtype=torch.bfloat16, device=device)
    v_cache = torch.zeros_like(k_cache)
    table = torch.zeros(B, width, dtype=torch.int32, device=device)
    lens = torch.zeros(B, dtype=torch.int32, device=device)
    slots = torch.zeros(B, dtype=torch.int32, device=device)
    pos = torch.zeros(B, dtype=torch.int64, device=device)
    qkv = torch.zeros(B, (Hq + 2 * Hkv) * D, dtype=torch.bfloat16, device=device)
    out = torch.zeros(B, Hq, D, dtype=torch.bfloat16, device=device)
    qwd, kwd, csd = qw.to(device), kw.to(device), cos_sin.to(device)

    def load(inp, raw):
        lay = inp.layout
        k_cache.zero_()
        v_cache.zero_()
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(
            key=inp.k_ctx.to(device), value=inp.v_ctx.to(device), k_cache=k_cache, v_cache=v_cache,
            slot_mapping=lay.ctx_slots.to(device)))
        table.zero_()
        table[:, : lay.block_table.shape[1]] = lay.block_table.to(device)
        lens.copy_(lay.seq_lens.to(device))
        slots.copy_(lay.new_slots.to(device))
        pos.copy_((lay.seq_lens - 1).long().to(device))
        qkv.copy_(raw.to(device))

    def step():
        ops.fused_qk_norm_rope(qkv, Hq, Hkv, Hkv, D, 1e-6, qwd, kwd, csd, False, pos, k_cache=k_cache, v_cache=v_cache,
                               slot_mapping=slots)
        ops.batch_decode(qkv[:, : Hq * D].view(B, Hq, D), k_cache, out, table, lens, v_cache=v_cache, scale=cfg.scale,
                         max_seq_len=width * cfg.block_size)

    load(inputs[0], raws[0])
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
        inp, raw = inputs[rep % 2], raws[rep % 2]
        load(inp, raw)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.clone()
        out.zero_()
        load(inp, raw)
        step()
        torch.cuda.synchronize()
        assert torch.equal(replayed, out), f"replay {rep}"
        lay = inp.layout
        want = oracle.fused_qk_norm_rope(raw, Hq, Hkv, Hkv, D, 1e-6, qw, kw, cos_sin, False, (lay.seq_lens - 1).long())
        kc, vc = fill_caches_cpu(inp)
        new = lay.new_slots.long()
        kc.view(-1, Hkv, D)[new] = want[:, Hq * D : (Hq + Hkv) * D].view(B, Hkv, D)
        vc.view(-1, Hkv, D)[new] = want[:, (Hq + Hkv) * D :].view(B, Hkv, D)
        ref = oracle.aten_paged_decode(want[:, : Hq * D].view(B, Hq, D).contiguous(), kc, vc, lay.block_table, lay.seq_lens,
                                       cfg.scale)
        assert_close_to_reference(replayed, ref, f"layer step replay {rep}")


def test_graph_captured_at_a_small_batch_survives_a_larger_eager_call(device):
    """The workspace is allocated once and its layout does not depend on the batch: a graph captured at batch 32
    replays correctly after an eager call at batch 128 (and after MLA and varlen calls) has used the same
    workspace."""
    small = workloads.DecodeConfig("ws_small", 32, 32, 8, 128, 16, 600, 2500)
    large = workloads.DecodeConfig("ws_large", 128, 32, 8, 128, 16, 600, 2500)
    inp_s, inp_l = workloads.make_inputs(small, 31), workloads.make_inputs(large, 32)
    ks_, vs_, _, _ = fill_caches_gpu(inp_s, device)
    kl_, vl_, _, _ = fill_caches_gpu(inp_l, device)
    q = inp_s.q.to(device)
    table, lens = inp_s.layout.block_table.to(device), inp_s.layout.seq_lens.to(device)
    out = torch.empty_like(q)
    eager, _ = _decode_gpu(inp_s, ks_, vs_, device)
    ws_before = ops.decode_workspace(device, 0).data_ptr()
    side = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        ops.batch_decode(q, ks_, out, table, lens, v_cache=vs_, scale=small.scale, max_seq_len=2500)  # warm-up
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            ops.batch_decode(q, ks_, out, table, lens, v_cache=vs_, scale=small.scale, max_seq_len=2500)
    torch.cuda.current_stream(device).wait_stream(side)
    torch.cuda.synchronize()
    for _ in range(2):
        big, _ = _decode_gpu(inp_l, kl_, vl_, device)
        ref = oracle.aten_paged_decode(inp_l.q[:4].contiguous(), kl_.cpu(), vl_.cpu(), inp_l.layout.block_table[:4].contiguous(),
                                       inp_l.layout.seq_lens[:4].contiguous(), large.scale)
        assert_close_to_reference(big[:4], ref, "large eager")
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
    assert ops.decode_workspace(device, 0).data_ptr() == ws_before
    with pytest.raises(RuntimeError):
        ops.decode_workspace(device, 1 << 40)


def test_a_wait_that_gives_up_is_reported(device):
    """With the poll bound at zero the first wait of a wavefront on its partner gives up: every wavefront still
    exits normally, the launch returns, and xllm_mi355_decode_status reports it once."""
    from xllm_amd import capi
    lib = capi.lib()
    cfg = workloads.DecodeConfig("stall", 8, 32, 8, 128, 16, 400, 1200)
    inp = workloads.make_inputs(cfg, 5)
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    good, _ = _decode_gpu(inp, kg, vg, device)
    assert ops.decode_status(device) == 0
    try:
        assert lib.xllm_mi355_debug_set(0, 0) == 0
        _decode_gpu(inp, kg, vg, device)
    finally:
        assert lib.xllm_mi355_debug_set(0, -1) == 0
    with pytest.raises(capi.XllmMi355Error, match="gave up"):
        ops.decode_status(device)
    assert ops.decode_status(device) == 0   # reported once, then cleared
    again, _ = _decode_gpu(inp, kg, vg, device)
    assert torch.equal(again, good) and ops.decode_status(device) == 0


def test_both_kinds_of_stores_write_the_same_bytes(device):
    # the matrix-core kernel writes output and partial rows with ordinary or with non-temporal stores (the library
    # chooses by the size of the launch): the same bytes either way, for whole contexts, contexts cut across workers,
    # fp8 pages, other head dims and packed query chunks; the first case is also checked against the oracle
    from xllm_amd import capi
    lib = capi.lib()

    def both(run):
        outs = []
        try:
            for kind in (0, 1):
                assert lib.xllm_mi355_debug_set(3, kind) == 0
                outs.append(run())
                torch.cuda.synchronize()
        finally:
            assert lib.xllm_mi355_debug_set(3, -1) == 0
        for a, b in zip(outs[0], outs[1]):
            assert torch.equal(a, b)
        return outs[1]

    shapes = (("st_g4", 40, 32, 8, 128, 16, 1, 3000, False), ("st_g8", 12, 64, 8, 128, 128, 500, 9000, False),
              ("st_fp8", 9, 32, 8, 128, 16, 100, 5000, True), ("st_d64", 17, 16, 4, 64, 32, 1, 2000, False),
              ("st_d256", 5, 6, 1, 256, 16, 50, 4000, False), ("st_short", 300, 8, 2, 128, 16, 1, 40, False))
    for i, (name, batch, Hq, Hkv, D, bs, lo, hi, fp8) in enumerate(shapes):
        cfg = workloads.DecodeConfig(name, batch, Hq, Hkv, D, bs, lo, hi, cache_dtype="fp8" if fp8 else "bf16")
        inp = workloads.make_inputs(cfg, 800 + i, device=device)
        kg, vg, ks, vs = fill_caches_gpu(inp, device, cache_dtype=torch.float8_e4m3fn if fp8 else None)
        out, lse = both(lambda: _decode_gpu(inp, kg, vg, device, ks, vs))
        if i == 0:
            lay = inp.layout
            ref = oracle.aten_paged_decode(inp.q.cpu(), kg.cpu(), vg.cpu(), lay.block_table, lay.seq_lens, cfg.scale)
            assert_close_to_reference(out, ref, name)
    cfg = workloads.DecodeConfig("st_chunks", 11, 32, 8, 128, 16, 30, 2500)
    inp = workloads.make_inputs(cfg, 820, device=device)
    lay = inp.layout
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    g = torch.Generator().manual_seed(4)
    q_lens = torch.randint(1, 9, (cfg.batch,), generator=g)
    cu = torch.tensor([0] + list(q_lens.cumsum(0)), dtype=torch.int32).to(device)
    q = (torch.randn(int(cu[-1]), 32, 128, generator=g) * cfg.sigma).to(torch.bfloat16).to(device)
    both(lambda: (ops.paged_forward(q, torch.empty_like(q), kg, vg, lay.block_table.to(device), lay.seq_lens.to(device),
                                    cu, scale=cfg.scale, is_causal=True, max_query_len=8),))
    assert ops.decode_status(device) == 0
