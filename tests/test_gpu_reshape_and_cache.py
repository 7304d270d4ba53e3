"""GPU parity of reshape_and_cache against the C oracle: cache bytes must be identical."""
import pytest
import torch

import oracle
from xllm_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu

# The five shape cases of ReshapePagedCacheTest.MatchesReference
# (tests/core/kernels/dcu/reshape_paged_cache_test.cpp:135-158): tokens, blocks, bs, heads, dim, dtype
REFERENCE_CASES = [
    (4, 1, 16, 1, 64, torch.float32),
    (32, 8, 16, 4, 128, torch.float16),
    (64, 4, 64, 8, 128, torch.bfloat16),
    (256, 16, 64, 8, 128, torch.float16),
    (1, 4, 16, 4, 128, torch.float32),
]


def _run_both(key, value, slots, shape, cache_dtype, device, k_scale=None, v_scale=None):
    store = torch.uint8 if cache_dtype == torch.float8_e4m3fn else cache_dtype
    kc = torch.zeros(shape, dtype=store)
    vc = None if value is None else torch.zeros(shape, dtype=store)
    oracle.reshape_and_cache(key, value, kc, vc, slots, k_scale, v_scale)
    kg = torch.zeros(shape, dtype=store, device=device)
    vg = None if value is None else torch.zeros(shape, dtype=store, device=device)
    p = ops.ReshapePagedCacheParams(
        key=key.to(device), value=None if value is None else value.to(device), k_cache=kg, v_cache=vg,
        slot_mapping=slots.to(device),
        k_cache_scale=None if k_scale is None else k_scale.to(device),
        v_cache_scale=None if v_scale is None else v_scale.to(device))
    (ops.quant_to_paged_cache if k_scale is not None else ops.reshape_paged_cache)(p)
    torch.cuda.synchronize()
    return (kc, vc), (kg.cpu(), None if vg is None else vg.cpu())


def _equal_bytes(a, b):
    return torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8))


@pytest.mark.parametrize("case", REFERENCE_CASES)
def test_reference_shape_cases_bit_exact(device, case):
    T, P, bs, H, D, dt = case
    g = torch.Generator().manual_seed(2026)
    key = torch.randn(T, H, D, generator=g).to(dt)
    value = torch.randn(T, H, D, generator=g).to(dt)
    slots = torch.randperm(P * bs, generator=g)[:T].to(torch.int32)
    (kc, vc), (kg, vg) = _run_both(key, value, slots, (P, bs, H, D), dt, device)
    assert _equal_bytes(kc, kg) and _equal_bytes(vc, vg)
    assert kc.float().abs().sum() > 0


def test_crosses_block_boundary_like_reference(device):
    # Qwen35_27B_TP4_KvCacheCrosses128TokenBoundary (tests/core/kernels/npu/npu_xllm_ops_test.cpp:305-364):
    # 130 tokens, block 128, 3 physical blocks, slots [256..383] ++ [0, 1]
    g = torch.Generator().manual_seed(20260730)
    key = torch.randn(130, 1, 256, generator=g).to(torch.bfloat16)
    value = torch.randn(130, 1, 256, generator=g).to(torch.bfloat16)
    slots = torch.cat([torch.arange(256, 384), torch.arange(0, 2)]).to(torch.int32)
    (kc, vc), (kg, vg) = _run_both(key, value, slots, (3, 128, 1, 256), torch.bfloat16, device)
    expected = torch.zeros(3, 128, 1, 256, dtype=torch.bfloat16)
    expected[2] = key[:128]
    expected[0, :2] = key[128:]
    assert torch.equal(kg, expected)
    assert torch.equal(kg, kc) and torch.equal(vg, vc)


def test_negative_and_out_of_range_slots_skipped_and_rest_untouched(device):
    g = torch.Generator().manual_seed(7)
    T, P, bs, H, D = 16, 4, 16, 2, 128
    key = torch.randn(T, H, D, generator=g).to(torch.bfloat16)
    value = torch.randn(T, H, D, generator=g).to(torch.bfloat16)
    slots = torch.randperm(P * bs, generator=g)[:T].to(torch.int32)
    slots[3] = -1
    slots[5] = -7
    slots[9] = P * bs + 5
    kg = torch.full((P, bs, H, D), 3.0, dtype=torch.bfloat16, device=device)
    vg = torch.full((P, bs, H, D), -2.0, dtype=torch.bfloat16, device=device)
    ops.reshape_paged_cache(ops.ReshapePagedCacheParams(
        key=key.to(device), value=value.to(device), k_cache=kg, v_cache=vg, slot_mapping=slots.to(device)))
    kc = torch.full((P, bs, H, D), 3.0, dtype=torch.bfloat16)
    vc = torch.full((P, bs, H, D), -2.0, dtype=torch.bfloat16)
    oracle.reshape_and_cache(key, value, kc, vc, slots)
    assert torch.equal(kg.cpu(), kc) and torch.equal(vg.cpu(), vc)
    written = set(int(s) for s in slots if 0 <= s < P * bs)
    flat = kg.cpu().view(P * bs, -1)
    for s in range(P * bs):
        if s not in written:
            assert (flat[s] == 3.0).all()


def test_independent_token_strides_and_unaligned_rows(device):
    g = torch.Generator().manual_seed(11)
    T, P, bs, H, D = 9, 3, 8, 2, 128
    # K and V are slices of one fused qkv buffer: different offsets, a common long stride
    qkv = torch.randn(T, 6 * H * D, generator=g).to(torch.bfloat16)
    key = qkv[:, 2 * H * D : 3 * H * D].view(T, H, D)
    value = qkv[:, 5 * H * D :].view(T, H, D)
    slots = torch.randperm(P * bs, generator=g)[:T].to(torch.int32)
    dev_qkv = qkv.to(device)
    kg = torch.zeros(P, bs, H, D, dtype=torch.bfloat16, device=device)
    vg = torch.zeros_like(kg)
    ops.reshape_paged_cache(ops.ReshapePagedCacheParams(
        key=dev_qkv[:, 2 * H * D : 3 * H * D].view(T, H, D), value=dev_qkv[:, 5 * H * D :].view(T, H, D),
        k_cache=kg, v_cache=vg, slot_mapping=slots.to(device)))
    kc = torch.zeros(P, bs, H, D, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    oracle.reshape_and_cache(key, value, kc, vc, slots)
    assert torch.equal(kg.cpu(), kc) and torch.equal(vg.cpu(), vc)
    # head_dim 20 (40-byte rows): the element-wise kernel
    key2 = torch.randn(5, 3, 20, generator=g).to(torch.float16)
    val2 = torch.randn(5, 3, 20, generator=g).to(torch.float16)
    s2 = torch.tensor([4, 0, 7, 2, 5], dtype=torch.int32)
    (kc2, vc2), (kg2, vg2) = _run_both(key2, val2, s2, (2, 4, 3, 20), torch.float16, device)
    assert torch.equal(kc2, kg2) and torch.equal(vc2, vg2)


def test_mla_latent_store_without_value(device):
    # k_cache.view({-1, 576}).index_copy_(0, slots, latent) of layers/dcu/deepseek_v2_attention.cpp:221-229
    g = torch.Generator().manual_seed(5)
    T, P, bs = 64, 8, 64
    latent = (0.5 * torch.randn(T, 1, 576, generator=g)).to(torch.bfloat16)
    slots = torch.randperm(P * bs, generator=g)[:T].to(torch.int32)
    (kc, _), (kg, _) = _run_both(latent, None, slots, (P, bs, 1, 576), torch.bfloat16, device)
    expected = torch.zeros(P * bs, 576, dtype=torch.bfloat16)
    expected.index_copy_(0, slots.to(torch.int64), latent.view(T, 576))
    assert torch.equal(kg.view(P * bs, 576), expected) and torch.equal(kg, kc)


def test_fp8_exhaustive_bf16_patterns_bit_exact(device):
    # every bf16 bit pattern through the quantising store, several scales, vs the C oracle
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16).view(512, 1, 128)
    slots = torch.arange(512, dtype=torch.int32)
    for scale in (1.0, 0.00390625, 0.013671875, 3.0e-3, 1.7, 1e-12, 37.5):
        ks = torch.tensor([scale], dtype=torch.float32)
        vs = torch.tensor([scale * 0.75], dtype=torch.float32)
        (kc, vc), (kg, vg) = _run_both(x, x, slots, (32, 16, 1, 128), torch.float8_e4m3fn, device, ks, vs)
        assert torch.equal(kc, kg), f"K codes differ at scale {scale}"
        assert torch.equal(vc, vg), f"V codes differ at scale {scale}"


def test_fp8_per_head_scales_fp16_fp32_inputs(device):
    g = torch.Generator().manual_seed(99)
    for dt in (torch.float16, torch.float32, torch.bfloat16):
        T, P, bs, H, D = 40, 4, 16, 8, 128
        key = (torch.randn(T, H, D, generator=g) * torch.linspace(0.1, 30, H).view(1, H, 1)).to(dt)
        value = torch.randn(T, H, D, generator=g).to(dt)
        slots = torch.randperm(P * bs, generator=g)[:T].to(torch.int32)
        ks = oracle.kv_head_scales(key)
        vs = oracle.kv_head_scales(value)
        gk = ops.kv_head_scales(key.to(device)).cpu()
        gv = ops.kv_head_scales(value.to(device)).cpu()
        assert torch.equal(gk, ks) and torch.equal(gv, vs), "per-head scales must match bit for bit"
        (kc, vc), (kg, vg) = _run_both(key, value, slots, (P, bs, H, D), torch.float8_e4m3fn, device, ks, vs)
        assert torch.equal(kc, kg) and torch.equal(vc, vg)
        # properties the reference's fp8 tests check (tests/core/kernels/cuda/fp8_quant_test.cpp:70-82,321-348)
        deq = kg.view(torch.float8_e4m3fn).float()
        assert torch.isfinite(deq).all() and deq.abs().max() <= 448


def test_prefill_sized_scatter_is_a_permutation(device):
    # full-size property: scattering to a permutation of all slots and gathering back is the identity
    g = torch.Generator(device=device).manual_seed(3)
    P, bs, H, D = 2048, 16, 8, 128
    T = P * bs
    key = torch.randn(T, H, D, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    value = torch.randn(T, H, D, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    slots = torch.randperm(T, generator=g, device=device).to(torch.int32)
    kg = torch.zeros(P, bs, H, D, dtype=torch.bfloat16, device=device)
    vg = torch.zeros_like(kg)
    ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=key, value=value, k_cache=kg, v_cache=vg,
                                                        slot_mapping=slots))
    assert torch.equal(kg.view(T, H, D)[slots.long()], key)
    assert torch.equal(vg.view(T, H, D)[slots.long()], value)


def test_gather_of_paged_latent_rows(device):
    # dcu::gather_mla_latent_cache (kernels/dcu/gather_mla_latent_cache.hip): bit-exact against the oracle, with
    # ragged lengths, padding ids in the table, and row lengths that take the 16-, 4- and 1-byte paths
    from helpers import fill_caches_cpu
    for dim, dtype, bs in ((576, torch.bfloat16, 64), (576, torch.bfloat16, 16), (130, torch.float16, 16),
                           (33, torch.uint8, 32)):
        cfg = workloads.DecodeConfig(f"gather{dim}", 7, 4, 1, 576, bs, 1, 900, mla=True, v_dim=512)
        lay = workloads.make_layout(cfg, 17 + dim)
        g = torch.Generator().manual_seed(dim)
        kc = torch.randint(0, 250, (lay.num_blocks, bs, 1, dim), generator=g, dtype=torch.uint8)
        kc = kc if dtype == torch.uint8 else kc.to(torch.float32).to(dtype)
        cu = torch.zeros(cfg.batch + 1, dtype=torch.int32)
        cu[1:] = lay.seq_lens.cumsum(0)
        total = int(cu[-1])
        table = lay.block_table.clone()
        table[2, 0] = -1                      # a lost page: its rows stay as they were
        table[3, 1:] = -1
        ref = oracle.gather_paged_rows(kc, table, cu, total)
        out = ops.gather_mla_latent_cache(kc.to(device), table.to(device), cu.to(device), total)
        torch.cuda.synchronize()
        touched = torch.ones(total, dtype=torch.bool)
        for b in (2, 3):
            for t in range(int(lay.seq_lens[b])):
                if int(table[b, t // bs]) < 0:
                    touched[int(cu[b]) + t] = False
        assert torch.equal(out.cpu()[touched].view(torch.uint8), ref[touched].view(torch.uint8)), (dim, dtype)


def test_decode_metadata_update_is_bit_exact(device):
    # update_llm_decode_metadata (kernels/cuda/llm_decode_metadata_update.cu:27-104): integer copies and fills;
    # every array equals the oracle's, the sentinel outside the padded range included
    from test_oracle_reshape import _metadata_case
    for seed, batch, padded, tokens in ((1, 7, 7, None), (2, 5, 16, None), (3, 1, 8, None), (4, 6, 32, 12),
                                        (5, 40, 64, None), (6, 0, 4, 0), (7, 1500, 2048, None)):
        src, want = _metadata_case(seed, batch, padded, tokens)
        _, got = _metadata_case(seed, batch, padded, tokens)
        n_tok, n_idx = src["tokens"].numel(), src["paged_kv_indices"].numel()
        oracle.llm_decode_metadata_update(src, want, n_tok, padded, batch, n_idx)
        s = {k: v.to(device) for k, v in src.items()}
        d = {k: v.to(device) for k, v in got.items()}
        ops.update_llm_decode_metadata(ops.LlmDecodeMetadataUpdateParams(
            src_tokens=s["tokens"], src_positions=s["positions"], src_new_cache_slots=s["new_cache_slots"],
            src_kv_seq_lens=s["kv_seq_lens"], src_paged_kv_indptr=s["paged_kv_indptr"],
            src_paged_kv_indices=s["paged_kv_indices"], src_paged_kv_last_page_len=s["paged_kv_last_page_len"],
            dst_tokens=d["tokens"], dst_positions=d["positions"], dst_new_cache_slots=d["new_cache_slots"],
            dst_kv_seq_lens=d["kv_seq_lens"], dst_kv_seq_lens_delta=d["kv_seq_lens_delta"],
            dst_paged_kv_indptr=d["paged_kv_indptr"], dst_paged_kv_indices=d["paged_kv_indices"],
            dst_paged_kv_last_page_len=d["paged_kv_last_page_len"], actual_num_tokens=n_tok,
            padded_num_tokens=padded, actual_batch_size=batch, actual_indices_size=n_idx))
        torch.cuda.synchronize()
        for k in want:
            assert torch.equal(d[k].cpu(), want[k]), (seed, k)


def test_fused_qk_norm_rope_and_its_cache_write(device):
    # fused_qk_norm_rope (kernels/cuda/fused_qknorm_rope.cu): q and k heads within the reference test's tolerance
    # of the oracle (fp32 arithmetic, one rounding), v untouched; with a cache, the pages hold bit for bit what
    # reshape_and_cache writes from the rotated buffer (16-bit and fp8 pages, skipped slots included).
    g = torch.Generator().manual_seed(11)
    cases = ((17, 8, 4, 4, 128, 128, torch.float16, torch.float32, False), (11, 6, 2, 2, 64, 64, torch.bfloat16, torch.float32, True),
             (64, 32, 8, 8, 128, 128, torch.bfloat16, torch.bfloat16, False), (5, 4, 2, 2, 256, 128, torch.bfloat16, torch.float16, False),
             (9, 4, 4, 4, 128, 64, torch.float16, torch.float32, True), (1, 16, 2, 2, 64, 32, torch.bfloat16, torch.float32, False),
             # prefill sizes, where a lane group takes four (token, head) units: unit counts that are not multiples of
             # four, head counts that let a group straddle two tokens
             (4999, 11, 3, 3, 128, 128, torch.bfloat16, torch.float32, False),
             (4501, 13, 2, 2, 64, 64, torch.float16, torch.float32, True),
             # ... with 128-dim heads a unit is 16 lanes of 16 bytes there: groups of one token (48 heads), a partial
             # rotary dim in both pair layouts, and one whose halves are not whole 16-byte pieces (32 lanes again)
             (1400, 32, 8, 8, 128, 64, torch.bfloat16, torch.float32, True),
             (1400, 32, 8, 8, 128, 32, torch.float16, torch.float16, False),
             (1400, 32, 8, 8, 128, 8, torch.bfloat16, torch.float32, False))
    for T, n_q, n_k, n_v, D, rd, dt, cdt, inter in cases:
        qkv = (torch.randn(T, (n_q + n_k + n_v) * D, generator=g) * 0.3).to(dt)
        qw, kw = (1 + 0.2 * torch.randn(D, generator=g)).to(dt), (1 + 0.2 * torch.randn(D, generator=g)).to(dt)
        ang = torch.rand(300, rd // 2, generator=g) * 6.28
        cs = torch.cat([ang.cos(), ang.sin()], 1).to(cdt)
        pos = torch.randint(0, 300, (T,), generator=g)
        want = oracle.fused_qk_norm_rope(qkv, n_q, n_k, n_v, D, 1e-6, qw, kw, cs, inter, pos)
        got = ops.fused_qk_norm_rope(qkv.to(device), n_q, n_k, n_v, D, 1e-6, qw.to(device), kw.to(device),
                                     cs.to(device), inter, pos.to(device))
        torch.cuda.synchronize()
        tol = 2e-3 if dt == torch.float16 else 1.6e-2    # one unit in the last place of the 16-bit type
        assert torch.allclose(got.cpu().float(), want.float(), rtol=tol, atol=tol), (T, D, inter)
        assert (got.cpu().float() - want.float()).abs().mean() < 2e-4
        assert torch.equal(got.cpu()[:, (n_q + n_k) * D :], qkv[:, (n_q + n_k) * D :])
        # the same launch with the cache write
        bs = 16
        P = max(12, T // bs + 2)
        slots = torch.randperm(P * bs, generator=g)[:T].to(torch.int32)
        slots[0] = -1
        for cache_dt in (dt, torch.float8_e4m3fn):
            kc = torch.zeros(P, bs, n_k, D, dtype=cache_dt, device=device)
            vc = torch.zeros_like(kc)
            ks = (0.5 + torch.rand(n_k, generator=g)).to(device) if cache_dt == torch.float8_e4m3fn else None
            vs = (0.5 + torch.rand(n_k, generator=g)).to(device) if cache_dt == torch.float8_e4m3fn else None
            buf = ops.fused_qk_norm_rope(qkv.to(device), n_q, n_k, n_v, D, 1e-6, qw.to(device), kw.to(device),
                                         cs.to(device), inter, pos.to(device), k_cache=kc, v_cache=vc,
                                         slot_mapping=slots.to(device), k_cache_scale=ks, v_cache_scale=vs)
            torch.cuda.synchronize()
            assert torch.equal(buf, got)
            kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
            k_rows = buf[:, n_q * D : (n_q + n_k) * D].view(T, n_k, D)
            v_rows = buf[:, (n_q + n_k) * D :].view(T, n_v, D)
            params = ops.ReshapePagedCacheParams(key=k_rows, value=v_rows, k_cache=kc2, v_cache=vc2,
                                                 slot_mapping=slots.to(device), k_cache_scale=ks, v_cache_scale=vs)
            (ops.quant_to_paged_cache if ks is not None else ops.reshape_paged_cache)(params)
            torch.cuda.synchronize()
            assert torch.equal(kc.view(torch.uint8), kc2.view(torch.uint8))
            assert torch.equal(vc.view(torch.uint8), vc2.view(torch.uint8))


def test_block_table_padding_mask_is_bit_exact(device):
    # mask_block_table_padding (layers/dcu/flash_attention.cpp:194-218): bit-exact against the oracle on ragged
    # lengths (empty, one token, page boundaries, the full width), a wide table, a strided table view, and in place
    g = torch.Generator().manual_seed(12)
    for bs, W, B in ((16, 9, 8), (64, 300, 40), (128, 1, 3)):
        lens = torch.randint(0, W * bs + 1, (B,), generator=g, dtype=torch.int32)
        lens[:3] = torch.tensor([0, 1, W * bs][:3], dtype=torch.int32)
        wide = torch.randint(0, 1000, (B, W + 5), generator=g, dtype=torch.int32)
        table = wide[:, :W]
        ref = oracle.mask_block_table_padding(table, lens, bs)
        got = ops.mask_block_table_padding(wide.to(device)[:, :W], lens.to(device), bs)
        assert torch.equal(got.cpu(), ref)
        own = table.contiguous().to(device)
        rc = capi.lib().xllm_mi355_mask_block_table_padding(own.data_ptr(), W, lens.to(device).data_ptr(), own.data_ptr(),
                                                            W, B, W, bs, torch.cuda.current_stream(device).cuda_stream)
        assert rc == 0
        assert torch.equal(own.cpu(), ref)
    with pytest.raises(ValueError):
        ops.mask_block_table_padding(table.to(device), lens[:-1].to(device), bs)
