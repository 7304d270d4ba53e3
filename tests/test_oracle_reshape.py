"""Pins the C oracle's reshape_and_cache: it is a permutation copy, so it is checked against
torch indexing on the reference tests' own shape cases."""
import pytest
import torch

import oracle

CASES = [  # tests/core/kernels/dcu/reshape_paged_cache_test.cpp:135-158
    (4, 1, 16, 1, 64, torch.float32),
    (32, 8, 16, 4, 128, torch.float16),
    (64, 4, 64, 8, 128, torch.bfloat16),
    (256, 16, 64, 8, 128, torch.float16),
    (1, 4, 16, 4, 128, torch.float32),
]


@pytest.mark.parametrize("case", CASES)
def test_matches_index_assignment(case):
    T, P, bs, H, D, dt = case
    g = torch.Generator().manual_seed(2026)
    key = torch.randn(T, H, D, generator=g).to(dt)
    value = torch.randn(T, H, D, generator=g).to(dt)
    slots = torch.randperm(P * bs, generator=g)[:T].to(torch.int32)
    kc = torch.zeros(P, bs, H, D, dtype=dt)
    vc = torch.zeros_like(kc)
    oracle.reshape_and_cache(key, value, kc, vc, slots)
    ek = torch.zeros(P * bs, H, D, dtype=dt)
    ev = torch.zeros_like(ek)
    ek[slots.long()] = key
    ev[slots.long()] = value
    assert torch.equal(kc.view(P * bs, H, D), ek) and torch.equal(vc.view(P * bs, H, D), ev)


def test_npu_case_and_negative_slots_and_strides():
    g = torch.Generator().manual_seed(20260730)
    key = torch.randn(130, 1, 256, generator=g).to(torch.bfloat16)
    value = torch.randn(130, 1, 256, generator=g).to(torch.bfloat16)
    slots = torch.cat([torch.arange(256, 384), torch.arange(0, 2)]).to(torch.int32)
    kc = torch.zeros(3, 128, 1, 256, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    oracle.reshape_and_cache(key, value, kc, vc, slots)
    expected = torch.zeros_like(kc)
    expected[2] = key[:128]
    expected[0, :2] = key[128:]
    assert torch.equal(kc, expected)
    # negative slot skipped, independent strides
    big = torch.randn(6, 4 * 2 * 32, generator=g).to(torch.float16)
    k = big[:, 64:128].view(6, 2, 32)
    v = big[:, 192:].view(6, 2, 32)
    s = torch.tensor([3, -1, 0, 7, -5, 2], dtype=torch.int32)
    kc = torch.full((2, 4, 2, 32), 9.0, dtype=torch.float16)
    vc = torch.full((2, 4, 2, 32), 9.0, dtype=torch.float16)
    oracle.reshape_and_cache(k, v, kc, vc, s)
    flat_k, flat_v = kc.view(8, 2, 32), vc.view(8, 2, 32)
    for t, slot in enumerate(s.tolist()):
        if slot >= 0:
            assert torch.equal(flat_k[slot], k[t]) and torch.equal(flat_v[slot], v[t])
    for slot in (1, 4, 5, 6):
        assert (flat_k[slot] == 9).all() and (flat_v[slot] == 9).all()


def test_gather_of_paged_rows_is_the_inverse_of_the_scatter():
    # gather_mla_latent_cache (kernels/dcu/gather_mla_latent_cache.hip:32-75): the rows a sequence scattered
    # into its pages come back in token order, sequence after sequence; padding ids (-1) leave rows untouched
    import oracle
    from helpers import fill_caches_cpu
    from xllm_amd import workloads
    cfg = workloads.DecodeConfig("gather", 5, 16, 1, 576, 16, 1, 300, mla=True, v_dim=512)
    inp = workloads.make_inputs(cfg, 4)
    lay = inp.layout
    kc, _ = fill_caches_cpu(inp)
    cu = torch.zeros(cfg.batch + 1, dtype=torch.int32)
    cu[1:] = lay.seq_lens.cumsum(0)
    total = int(cu[-1])
    out = oracle.gather_paged_rows(kc, lay.block_table, cu, total)
    for b in range(cfg.batch):
        lo, hi = int(lay.ctx_offsets[b]), int(lay.ctx_offsets[b + 1])
        rows = torch.cat([inp.k_ctx[lo:hi, 0], inp.k_new[b]])
        assert torch.equal(out[int(cu[b]) : int(cu[b + 1])], rows)
    # brute force with torch indexing, and a table whose second sequence lost a page
    table = lay.block_table.clone()
    table[1, 0] = -1
    got = oracle.gather_paged_rows(kc, table, cu, total, fill=7)
    flat = kc.view(-1, 576)
    for b in range(cfg.batch):
        for t in range(int(lay.seq_lens[b])):
            page = int(table[b, t // 16])
            expect = flat[page * 16 + t % 16] if page >= 0 else torch.full((576,), 7, dtype=kc.dtype)
            assert torch.equal(got[int(cu[b]) + t], expect)


def _metadata_case(seed, batch, padded, tokens=None):
    """A decode step's metadata as the executor holds it (cumulative lengths, CSR pages) and persistent buffers
    filled with a sentinel."""
    g = torch.Generator().manual_seed(seed)
    tokens = batch if tokens is None else tokens
    lens = torch.randint(1, 300, (batch,), generator=g, dtype=torch.int32)
    pages = (lens + 15) // 16
    src = {
        "tokens": torch.randint(0, 32000, (tokens,), generator=g, dtype=torch.int32),
        "positions": torch.randint(0, 4096, (tokens,), generator=g, dtype=torch.int32),
        "new_cache_slots": torch.randint(0, 1 << 20, (tokens,), generator=g, dtype=torch.int32),
        "kv_seq_lens": torch.cat([torch.zeros(1, dtype=torch.int32), lens.cumsum(0).to(torch.int32)]),
        "paged_kv_indptr": torch.cat([torch.zeros(1, dtype=torch.int32), pages.cumsum(0).to(torch.int32)]),
        "paged_kv_indices": torch.randint(0, 5000, (int(pages.sum()),), generator=g, dtype=torch.int32),
        "paged_kv_last_page_len": ((lens - 1) % 16 + 1).to(torch.int32),
    }
    width = max(padded, tokens, batch) + 3
    dst = {k: torch.full((width + (1 if k in ("kv_seq_lens", "paged_kv_indptr") else 0),), -77, dtype=torch.int32)
           for k in ("tokens", "positions", "new_cache_slots", "kv_seq_lens", "kv_seq_lens_delta", "paged_kv_indptr",
                     "paged_kv_last_page_len")}
    dst["paged_kv_indices"] = torch.full((int(pages.sum()) + 5,), -77, dtype=torch.int32)
    return src, dst


def _metadata_by_slices(src, dst, n_tok, n_pad, batch, n_idx):
    """The executor's slow path that the kernel replaces: slice copies and fills
    (xllm/core/runtime/cuda_graph_executor_impl.cpp:397-453 and the FlashInfer buffers after it)."""
    for k in ("tokens", "positions", "new_cache_slots"):
        dst[k][:n_tok] = src[k][:n_tok]
    if n_pad > n_tok:
        dst["tokens"][n_tok:n_pad] = 0
        dst["positions"][n_tok:n_pad] = 0
        dst["new_cache_slots"][n_tok:n_pad] = -1
    for k in ("kv_seq_lens", "paged_kv_indptr"):
        dst[k][: batch + 1] = src[k][: batch + 1]
        if n_pad > batch:
            dst[k][batch + 1 : n_pad + 1] = src[k][batch]
    dst["kv_seq_lens_delta"][:batch] = src["kv_seq_lens"][1 : batch + 1] - src["kv_seq_lens"][:batch]
    dst["paged_kv_last_page_len"][:batch] = src["paged_kv_last_page_len"][:batch]
    if n_pad > batch:
        dst["kv_seq_lens_delta"][batch:n_pad] = 0
        dst["paged_kv_last_page_len"][batch:n_pad] = 1
    dst["paged_kv_indices"][:n_idx] = src["paged_kv_indices"][:n_idx]
    return dst


def test_decode_metadata_update_rules_equal_the_slice_copies_they_replace():
    # llm_decode_metadata_update.cu:27-71 states the update index by index; the executor path it replaces states it
    # as slice copies and fills.  Equal on: no padding, padding, fewer sequences than tokens (speculative steps),
    # an empty step, and nothing outside the padded range is touched (sentinel -77 survives).
    import oracle
    for seed, batch, padded, tokens in ((1, 7, 7, None), (2, 5, 16, None), (3, 1, 8, None), (4, 6, 32, 12),
                                        (5, 40, 64, None), (6, 0, 4, 0)):
        src, a = _metadata_case(seed, batch, padded, tokens)
        _, b = _metadata_case(seed, batch, padded, tokens)
        n_tok = src["tokens"].numel()
        n_idx = src["paged_kv_indices"].numel()
        oracle.llm_decode_metadata_update(src, a, n_tok, padded, batch, n_idx)
        _metadata_by_slices(src, b, n_tok, padded, batch, n_idx)
        for k in a:
            assert torch.equal(a[k], b[k]), (seed, k)
        assert int(a["tokens"][max(padded, n_tok)]) == -77 and int(a["kv_seq_lens"][max(padded, batch) + 1]) == -77
        if padded > batch:
            assert int(a["kv_seq_lens"][padded]) == int(src["kv_seq_lens"][batch])
            assert int(a["paged_kv_last_page_len"][padded - 1]) == 1 and int(a["new_cache_slots"][padded - 1]) == -1


def test_block_table_padding_mask_against_the_reference_expression():
    # mask_block_table_padding (layers/dcu/flash_attention.cpp:194-218) written with the reference's own tensor
    # expression: columns at or beyond ceil(len / bs) become -1 whatever they hold (page id 0 is a valid page and
    # survives inside a sequence), the others are kept; empty sequences lose every column.
    g = torch.Generator().manual_seed(4)
    for bs, W in ((16, 9), (64, 5), (128, 1)):
        lens = torch.tensor([0, 1, bs - 1, bs, bs + 1, W * bs, W * bs - 1, 3 * bs // 2], dtype=torch.int32).clamp(max=W * bs)
        table = torch.randint(0, 50, (lens.numel(), W + 3), generator=g, dtype=torch.int32)[:, :W]  # row stride > width
        table[:, 0] = 0                                            # a valid page 0 in the first column
        got = oracle.mask_block_table_padding(table, lens, bs)
        pages = ((lens.long() + bs - 1) // bs).view(-1, 1)
        want = table.clone().masked_fill_(torch.arange(W).view(1, -1) >= pages, -1)
        assert torch.equal(got, want)
        assert (got[1:, 0] == 0).all() and (got[0] == -1).all()
