"""Pins the two attention oracles and the LSE merge without the GPU.

aten_oracle.cpp restates the reference's libtorch decode op for op; paged_kv_oracle.c is exact
fp64 softmax attention.  They are checked against each other, against closed forms and against
the known answers the reference's own tests hold."""
import math

import pytest
import torch

import oracle
from helpers import fill_caches_cpu
from xllm_amd import workloads


def _setup(cfg, seed, dtype=torch.bfloat16):
    inp = workloads.make_inputs(cfg, seed, dtype=dtype)
    kc, vc = fill_caches_cpu(inp)
    return inp, kc, vc


def _dense_reference(inp, b):
    """Textbook attention from the token streams, no paging at all (fp64)."""
    cfg, lay = inp.cfg, inp.layout
    lo, hi = int(lay.ctx_offsets[b]), int(lay.ctx_offsets[b + 1])
    k = torch.cat([inp.k_ctx[lo:hi], inp.k_new[b : b + 1]]).double()
    v = k[..., : cfg.dv] if cfg.mla else torch.cat([inp.v_ctx[lo:hi], inp.v_new[b : b + 1]]).double()
    g = cfg.n_q_heads // cfg.n_kv_heads
    q = inp.q[b].double()
    outs, lses = [], []
    for h in range(cfg.n_q_heads):
        s = (k[:, h // g] @ q[h]) * cfg.scale
        p = torch.softmax(s, 0)
        outs.append(p @ v[:, h // g])
        lses.append(torch.logsumexp(s, 0))
    return torch.stack(outs), torch.stack(lses)


@pytest.mark.parametrize("name,batch", [("tiny", 4), ("llama3_8b", 2), ("long_b256", 2), ("mla_dsv3", 1)])
def test_f64_oracle_equals_dense_attention_and_aten_oracle_is_within_bf16_rounding(name, batch):
    cfg = workloads.scaled(workloads.CONFIGS[name], batch=batch, len_hi=min(workloads.CONFIGS[name].len_hi, 3000))
    inp, kc, vc = _setup(cfg, 11)
    lay = inp.layout
    out64, lse64 = oracle.paged_decode_f64(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale, dv=cfg.dv)
    for b in range(cfg.batch):
        o, l = _dense_reference(inp, b)
        assert torch.allclose(out64[b].double(), o, rtol=1e-5, atol=1e-6)
        assert torch.allclose(lse64[b].double(), l, rtol=1e-6, atol=1e-5)
    aten = oracle.aten_paged_decode(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale, dv=cfg.dv)
    diff = (aten.float() - out64).abs()
    assert diff.max() < 2e-3 and diff.mean() < 2e-4, (diff.max(), diff.mean())
    lse = oracle.aten_paged_decode_lse(inp.q, kc, lay.block_table, lay.seq_lens, cfg.scale)
    assert torch.allclose(lse, lse64, rtol=1e-4, atol=1e-4)


def test_invariants_of_both_oracles():
    cfg = workloads.DecodeConfig("inv", 3, 8, 2, 64, 16, 40, 90)
    inp, kc, vc = _setup(cfg, 3)
    lay = inp.layout
    g = cfg.n_q_heads // cfg.n_kv_heads
    # L = 1 -> V[0] of the mapped head (checks the head mapping h -> h / group too)
    one = torch.ones_like(lay.seq_lens)
    for fn in (lambda: oracle.aten_paged_decode(inp.q, kc, vc, lay.block_table, one, cfg.scale).float(),
               lambda: oracle.paged_decode_f64(inp.q, kc, vc, lay.block_table, one, cfg.scale)[0]):
        out = fn()
        for b in range(cfg.batch):
            v0 = vc[lay.block_table[b, 0].item(), 0].float()
            assert torch.equal(out[b], v0.repeat_interleave(g, 0))
    # equal K rows -> mean of V; equal V rows -> V
    kc_eq = kc.clone()
    kc_eq[:] = kc[0, 0]
    out, _ = oracle.paged_decode_f64(inp.q, kc_eq, vc, lay.block_table, lay.seq_lens, cfg.scale)
    for b in range(cfg.batch):
        L = int(lay.seq_lens[b])
        lo, hi = int(lay.ctx_offsets[b]), int(lay.ctx_offsets[b + 1])
        vmean = torch.cat([inp.v_ctx[lo:hi], inp.v_new[b : b + 1]]).double().mean(0)
        assert torch.allclose(out[b].double(), vmean.repeat_interleave(g, 0), atol=1e-6)
    # page permutation
    perm = torch.randperm(lay.num_blocks, generator=torch.Generator().manual_seed(4))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(lay.num_blocks)
    t2 = inv[lay.block_table.long()].to(torch.int32)
    a = oracle.aten_paged_decode(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale)
    b_ = oracle.aten_paged_decode(inp.q, kc[perm].contiguous(), vc[perm].contiguous(), t2, lay.seq_lens, cfg.scale)
    assert torch.equal(a, b_)


def test_csr_oracle_equals_block_table_oracle_at_default_scale():
    cfg = workloads.DecodeConfig("csr", 4, 8, 4, 128, 16, 5, 300)
    inp, kc, vc = _setup(cfg, 9)
    lay = inp.layout
    a = oracle.aten_paged_decode(inp.q, kc, vc, lay.block_table, lay.seq_lens, 1.0 / math.sqrt(128))
    b = oracle.aten_paged_decode_csr(inp.q, kc, vc, lay.indptr, lay.indices, lay.last_page_len)
    assert (a.float() - b.float()).abs().max() <= 2 ** -8 * a.float().abs().max()
    table, lens = oracle.build_block_table(lay.indptr, lay.indices, lay.last_page_len, 40, 16)
    assert torch.equal(lens, lay.seq_lens)
    w = lay.block_table.shape[1]
    for bb in range(cfg.batch):
        n = int(lay.indptr[bb + 1] - lay.indptr[bb])
        assert torch.equal(table[bb, :n], lay.block_table[bb, :n]) and (table[bb, n:] == -1).all()


def test_mla_lse_closed_form_like_reference_test():
    # MluMlaDecodeLseTest.ReturnsFloat32NaturalLogNormalizer
    # (tests/core/layers/mlu/dcp_attention_merge_test.cpp:77-144): H=2, D=576, Dv=512, L=2
    g = torch.Generator().manual_seed(0)
    q = torch.rand(1, 2, 576, generator=g).to(torch.bfloat16)
    cache = torch.rand(1, 16, 1, 576, generator=g).to(torch.bfloat16)
    table = torch.zeros(1, 1, dtype=torch.int32)
    lens = torch.tensor([2], dtype=torch.int32)
    scale = 1.0 / math.sqrt(576.0)
    expected = torch.logsumexp((q[0].float() @ cache[0, :2, 0].float().T) * scale, -1)
    _, lse64 = oracle.paged_decode_f64(q, cache, None, table, lens, scale, dv=512)
    lse = oracle.aten_paged_decode_lse(q, cache, table, lens, scale)
    assert lse.dtype == torch.float32 and tuple(lse.shape) == (1, 2)
    assert torch.allclose(lse[0], expected, rtol=1e-3, atol=1e-3)
    assert torch.allclose(lse64[0], expected, rtol=1e-3, atol=1e-3)
    out = oracle.aten_paged_decode(q, cache, None, table, lens, scale, dv=512)
    p = torch.softmax((q[0].float() @ cache[0, :2, 0].float().T) * scale, -1)
    assert torch.allclose(out[0].float(), p @ cache[0, :2, 0, :512].float(), atol=1e-2)


MERGE_FNS = [
    lambda o, l: oracle.lse_merge(o, l),
    lambda o, l: tuple(t.float() for t in oracle.aten_lse_merge(o, l)),
]


@pytest.mark.parametrize("merge", MERGE_FNS)
def test_merge_known_answers_of_the_reference(merge):
    # DcpAttentionMergeTest (tests/core/layers/mlu/dcp_attention_merge_test.cpp:34-75)
    o = torch.tensor([2.0, 4.0, 6.0, 8.0]).reshape(2, 1, 1, 2)
    l = torch.tensor([math.log(2.0), math.log(6.0)]).reshape(2, 1, 1)
    out, lse = merge(o, l)
    assert torch.allclose(out, torch.tensor([5.0, 7.0]).reshape(1, 1, 2))
    assert torch.allclose(lse, torch.tensor([math.log(8.0)]).reshape(1, 1))
    o = torch.tensor([0.0, 0.0, 3.0, 9.0]).reshape(2, 1, 1, 2)
    l = torch.tensor([-math.inf, math.log(4.0)]).reshape(2, 1, 1)
    out, lse = merge(o, l)
    assert torch.equal(out, torch.tensor([3.0, 9.0]).reshape(1, 1, 2))
    assert torch.allclose(lse, torch.tensor([math.log(4.0)]).reshape(1, 1))
    o = torch.ones(2, 1, 2, 3)
    l = torch.full((2, 1, 2), -math.inf)
    out, lse = merge(o, l)
    assert torch.equal(out, torch.zeros(1, 2, 3)) and torch.isneginf(lse).all()


def test_merge_of_context_shards_equals_unsplit_decode():
    # ArtificialShardMergeMatchesFullCacheDecode (same file :146-224), tolerances 1e-2 / 1e-3
    cfg = workloads.DecodeConfig("m", 2, 4, 1, 576, 16, 40, 64, mla=True, v_dim=512, sigma=0.5,
                                 sm_scale=1 / math.sqrt(576.0))
    inp, kc, _ = _setup(cfg, 21)
    lay = inp.layout
    full, full_lse = oracle.paged_decode_f64(inp.q, kc, None, lay.block_table, lay.seq_lens, cfg.scale, dv=512)
    # shard A: first 2 pages (32 tokens); shard B: the rest through a shifted table
    la = torch.full_like(lay.seq_lens, 32)
    lb = lay.seq_lens - 32
    tb = torch.zeros_like(lay.block_table)
    tb[:, :-2] = lay.block_table[:, 2:]
    oa, lsa = oracle.paged_decode_f64(inp.q, kc, None, lay.block_table, la, cfg.scale, dv=512)
    ob, lsb = oracle.paged_decode_f64(inp.q, kc, None, tb, lb, cfg.scale, dv=512)
    for merge in MERGE_FNS:
        out, lse = merge(torch.stack([oa, ob]), torch.stack([lsa, lsb]))
        assert torch.allclose(out, full, rtol=1e-2, atol=1e-2) and torch.allclose(lse, full_lse, rtol=1e-3, atol=1e-3)
        assert (out - full).abs().max() < 1e-5


def _chunk_inputs(cfg, seed, max_q=16):
    """A decode workload whose last q_len tokens of every context form the query chunk."""
    inp = workloads.make_inputs(cfg, seed)
    lay = inp.layout
    g = torch.Generator().manual_seed(seed + 7)
    q_lens = [int(torch.randint(1, min(max_q, int(L)) + 1, (1,), generator=g)) for L in lay.seq_lens]
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    q = (torch.randn(int(cu[-1]), cfg.n_q_heads, cfg.head_dim, generator=g) * cfg.sigma).to(torch.bfloat16)
    return inp, q, cu, q_lens


def test_query_chunks_equal_dense_attention_with_the_causal_mask_at_the_bottom_right():
    cfg = workloads.DecodeConfig("chunks", 4, 8, 2, 64, 16, 5, 120)
    inp, q, cu, q_lens = _chunk_inputs(cfg, 21)
    kc, vc = fill_caches_cpu(inp)
    lay = inp.layout
    g = cfg.n_q_heads // cfg.n_kv_heads
    for causal in (True, False):
        out = oracle.aten_paged_forward(q, kc, vc, lay.block_table, lay.seq_lens, cu, cfg.scale, causal=causal)
        for b in range(cfg.batch):
            lo, hi = int(lay.ctx_offsets[b]), int(lay.ctx_offsets[b + 1])
            k = torch.cat([inp.k_ctx[lo:hi], inp.k_new[b : b + 1]]).double()   # [L, Hkv, D]
            v = torch.cat([inp.v_ctx[lo:hi], inp.v_new[b : b + 1]]).double()
            L, n = k.shape[0], q_lens[b]
            qb = q[int(cu[b]) : int(cu[b + 1])].double()                      # [n, Hq, D]
            s = torch.einsum("nhd,lhd->hnl", qb, k.repeat_interleave(g, 1)) * cfg.scale
            if causal:  # query j sees keys 0 .. L - n + j
                mask = torch.arange(L)[None, :] > (L - n + torch.arange(n))[:, None]
                s = s.masked_fill(mask[None], float("-inf"))
            ref = torch.einsum("hnl,lhd->nhd", torch.softmax(s, -1), v.repeat_interleave(g, 1))
            got = out[int(cu[b]) : int(cu[b + 1])].double()
            assert (got - ref).abs().max() < 3e-3, (causal, b)
    # a chunk of one token is plain decode
    ones = torch.arange(cfg.batch + 1, dtype=torch.int32)
    q1 = inp.q.contiguous()
    assert torch.equal(oracle.aten_paged_forward(q1, kc, vc, lay.block_table, lay.seq_lens, ones, cfg.scale),
                       oracle.aten_paged_decode(q1, kc, vc, lay.block_table, lay.seq_lens, cfg.scale))


def _reference_test_formula(qkv, n_q, n_k, D, eps, qw, kw, cos_sin, interleave, pos):
    """The torch reference of the reference's own test (tests/core/kernels/dcu/fused_qknorm_rope_test.cpp:27-118):
    it rounds to the qkv dtype between the norm and the rotation, which the kernel does not."""
    T = qkv.shape[0]
    rd = cos_sin.shape[1]
    h = rd // 2
    out = qkv.clone()
    for lo, n, w in ((0, n_q, qw), (n_q * D, n_k, kw)):
        x = qkv[:, lo : lo + n * D].view(T, n, D).float()
        x = (x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w.float().view(1, 1, D)).to(qkv.dtype).float()
        sel = cos_sin.index_select(0, pos)
        cos, sin = sel[:, :h].view(T, 1, h), sel[:, h:].view(T, 1, h)
        rot, rest = x[..., :rd], x[..., rd:]
        if interleave:
            r = rot.reshape(T, n, h, 2)
            ev, od = r[..., 0], r[..., 1]
            rot = torch.stack([ev * cos - od * sin, ev * sin + od * cos], -1).view(T, n, rd)
        else:
            a, b = rot[..., :h], rot[..., h:]
            rot = torch.cat([a * cos - b * sin, b * cos + a * sin], -1)
        out[:, lo : lo + n * D] = torch.cat([rot, rest], -1).to(qkv.dtype).view(T, n * D)
    return out


def test_fused_qk_norm_rope_oracle_known_rotations_and_the_reference_tests_formula():
    import oracle
    g = torch.Generator().manual_seed(2026)
    # (a) the two cases of the reference's test, against its torch formula, with its tolerance
    for T, n_q, n_k, n_v, D, max_pos, dt, sig, inter in ((17, 8, 4, 4, 128, 512, torch.float16, 0.2, False),
                                                         (11, 6, 2, 2, 64, 256, torch.bfloat16, 0.15, True)):
        qkv = (torch.randn(T, (n_q + n_k + n_v) * D, generator=g) * sig).to(dt)
        qw, kw = torch.randn(D, generator=g).to(dt), torch.randn(D, generator=g).to(dt)
        cs = torch.randn(max_pos, D, generator=g)
        pos = torch.randint(0, max_pos, (T,), generator=g)
        got = oracle.fused_qk_norm_rope(qkv, n_q, n_k, n_v, D, 1e-6, qw, kw, cs, inter, pos)
        want = _reference_test_formula(qkv, n_q, n_k, D, 1e-6, qw, kw, cs, inter, pos)
        # (bf16 carries 8 bits: one rounding step between the two formulas is 2^-8 relative)
        tol = 2e-3 if dt == torch.float16 else 1.6e-2
        assert torch.allclose(got.float(), want.float(), rtol=tol, atol=tol)
        assert torch.equal(got[:, (n_q + n_k) * D :], qkv[:, (n_q + n_k) * D :])   # v untouched
    # (b) known answers.  No norm, a quarter turn (cos 0, sin 1): split form (a, b) -> (-b, a), interleaved
    # (e, o) -> (-o, e), exactly; a zero turn returns the input; partial rotary_dim leaves the tail alone
    T, n_q, n_k, D = 3, 2, 1, 64
    x = torch.randn(T, (n_q + n_k) * D, generator=g).to(torch.bfloat16)
    pos = torch.tensor([0, 1, 1])
    for rd in (64, 32):
        h = rd // 2
        cs = torch.zeros(2, rd)
        cs[0, :h] = 1.0          # position 0: zero turn
        cs[1, h:] = 1.0          # position 1: quarter turn
        v = x.view(T, n_q + n_k, D)
        for inter in (False, True):
            got = oracle.fused_qk_norm_rope(x, n_q, n_k, 0, D, 0.0, None, None, cs, inter, pos).view(T, n_q + n_k, D)
            assert torch.equal(got[0], v[0])
            assert torch.equal(got[1:, :, rd:], v[1:, :, rd:])
            if inter:
                assert torch.equal(got[1:, :, 0:rd:2], -v[1:, :, 1:rd:2]) and torch.equal(got[1:, :, 1:rd:2], v[1:, :, 0:rd:2])
            else:
                assert torch.equal(got[1:, :, :h], -v[1:, :, h:rd]) and torch.equal(got[1:, :, h:rd], v[1:, :, :h])
    # (c) the norm: unit weights give unit mean square; a rotation by any angle keeps it
    D = 128
    x = (torch.randn(5, 3 * D, generator=g) * 3).to(torch.bfloat16)
    ang = torch.rand(7, D // 2, generator=g) * 6.28
    cs = torch.cat([ang.cos(), ang.sin()], 1)
    ones = torch.ones(D, dtype=torch.bfloat16)
    got = oracle.fused_qk_norm_rope(x, 2, 1, 0, D, 1e-6, ones, ones, cs, False, torch.tensor([0, 3, 6, 2, 2]))
    ms = (got.float().view(5, 3, D) ** 2).mean(-1)
    assert torch.allclose(ms, torch.ones_like(ms), atol=1e-2)


def test_absorbed_bmm_oracle_against_loops_and_selections():
    # The per-head products of the absorbed MLA attention (layers/dcu/deepseek_v2_attention.cpp:428-430, 231-238).
    # Pins: explicit loops on a small case (a transposed operand or a swapped head/token index fails them),
    # one-hot weights that select and permute columns (exact in bf16), and the reference's own expression on
    # head-major views.
    g = torch.Generator().manual_seed(5)
    T, H, K, N = 3, 4, 6, 5
    x = torch.randn(T, H, K, generator=g).bfloat16()
    w = torch.randn(H, K, N, generator=g).bfloat16()
    y, exact = oracle.absorbed_bmm(x, w)
    loops = torch.zeros(T, H, N, dtype=torch.float64)
    for t in range(T):
        for h in range(H):
            for n in range(N):
                loops[t, h, n] = sum(float(x[t, h, k]) * float(w[h, k, n]) for k in range(K))
    assert torch.allclose(exact.double(), loops, rtol=1e-6, atol=1e-6)
    assert torch.equal(y, exact.bfloat16())
    assert y.shape == (T, H, N) and y.dtype == torch.bfloat16
    # head h picks column perm[h][n] of x: the result is a gather, bit for bit
    perm = torch.stack([torch.randperm(K, generator=g)[:N] for _ in range(H)])
    sel = torch.zeros(H, K, N)
    for h in range(H):
        sel[h, perm[h], torch.arange(N)] = 1.0
    y_sel, _ = oracle.absorbed_bmm(x, sel.bfloat16())
    want = torch.stack([x[:, h, perm[h]] for h in range(H)], dim=1)
    assert torch.equal(y_sel, want)
    # the reference's expression, on a slice of a wider tensor as q_nope is
    q = torch.randn(T, H, K + 2, generator=g).bfloat16()
    y_slice, _ = oracle.absorbed_bmm(q[..., :K], w)
    ref = torch.bmm(q[..., :K].float().transpose(0, 1), w.float()).transpose(0, 1)
    assert torch.equal(y_slice, ref.bfloat16())


def test_fp8_dequant_branch_of_both_oracles():
    """Decode on an fp8 cache with per-head scales must equal, bit for bit, decode on a 16-bit cache that
    holds (decode_table[code] * scale[h]).to(q dtype): the dequantisation rule stated for the fp8 pages
    (the int8 precedent of xllm/core/layers/mlu/attention.cpp:171-222).  A scale applied to the wrong head,
    taken from the other tensor, squared or dropped changes the 16-bit cache and fails the comparison."""
    cfg = workloads.DecodeConfig("fp8pin", 3, 8, 4, 128, 16, 33, 150)
    inp = workloads.make_inputs(cfg, 21)
    lay = inp.layout
    k_scale = oracle.kv_head_scales(torch.cat([inp.k_ctx, inp.k_new]))
    v_scale = oracle.kv_head_scales(torch.cat([inp.v_ctx, inp.v_new])) * 1.5   # K and V scales differ per head
    assert len(set(k_scale.tolist())) == cfg.n_kv_heads and not torch.equal(k_scale, v_scale)
    kc8, vc8 = fill_caches_cpu(inp, torch.uint8, k_scale, v_scale)
    table = oracle.fp8_decode_table()
    for dt in (torch.bfloat16, torch.float16):
        q = inp.q.to(dt)
        kc16 = (table[kc8.long()] * k_scale.view(1, 1, -1, 1)).to(dt)
        vc16 = (table[vc8.long()] * v_scale.view(1, 1, -1, 1)).to(dt)
        a8 = oracle.aten_paged_decode(q, kc8, vc8, lay.block_table, lay.seq_lens, cfg.scale, k_scale, v_scale)
        a16 = oracle.aten_paged_decode(q, kc16, vc16, lay.block_table, lay.seq_lens, cfg.scale)
        assert torch.equal(a8.view(torch.int16), a16.view(torch.int16))
        f8, l8 = oracle.paged_decode_f64(q, kc8, vc8, lay.block_table, lay.seq_lens, cfg.scale, k_scale, v_scale)
        f16, l16 = oracle.paged_decode_f64(q, kc16, vc16, lay.block_table, lay.seq_lens, cfg.scale)
        assert torch.equal(f8, f16) and torch.equal(l8, l16)
        lse8 = oracle.aten_paged_decode_lse(q, kc8, lay.block_table, lay.seq_lens, cfg.scale, k_scale)
        lse16 = oracle.aten_paged_decode_lse(q, kc16, lay.block_table, lay.seq_lens, cfg.scale)
        assert torch.equal(lse8, lse16)
    # the torch view of the same bytes is the same cache
    a8v = oracle.aten_paged_decode(inp.q, kc8.view(torch.float8_e4m3fn), vc8.view(torch.float8_e4m3fn),
                                   lay.block_table, lay.seq_lens, cfg.scale, k_scale, v_scale)
    a8u = oracle.aten_paged_decode(inp.q, kc8, vc8, lay.block_table, lay.seq_lens, cfg.scale, k_scale, v_scale)
    assert torch.equal(a8v, a8u)


def test_fp8_decode_known_answer():
    """All codes 0x38 (= 1.0) in K and V, V scale 0.5: every score is equal, so the output is 0.5 exactly and
    the LSE is log(L) + scale * k_scale * sum(q)."""
    B, Hq, Hkv, D, bs, L = 2, 4, 2, 64, 16, 37
    kc = torch.full((8, bs, Hkv, D), 0x38, dtype=torch.uint8)
    vc = kc.clone()
    q = torch.ones(B, Hq, D, dtype=torch.bfloat16)
    table = torch.arange(8, dtype=torch.int32).view(2, 4)
    lens = torch.tensor([L, 5], dtype=torch.int32)
    ks = torch.tensor([2.0, 0.25])
    vs = torch.tensor([0.5, 0.125])
    out = oracle.aten_paged_decode(q, kc, vc, table, lens, 0.125, ks, vs)
    out64, lse64 = oracle.paged_decode_f64(q, kc, vc, table, lens, 0.125, ks, vs)
    for o in (out.float(), out64):
        assert torch.all(o[:, :2] == 0.5) and torch.all(o[:, 2:] == 0.125)
    expect = torch.log(lens.double()).view(2, 1) + 0.125 * D * ks.double().repeat_interleave(2).view(1, 4)
    assert torch.allclose(lse64.double(), expect, atol=1e-5)
    lse = oracle.aten_paged_decode_lse(q, kc, table, lens, 0.125, ks)
    assert torch.allclose(lse.double(), expect, atol=1e-4)


def test_base2_two_way_combine_oracle():
    """The known answers of the reference's merge tests (dcp_attention_merge_test.cpp:34-63) with the LSEs
    rescaled to base 2 (natural-log LSE / ln 2), the natural-log merge oracle on random inputs, and the
    equal-weights and one-sided special cases.  A swapped weight, a natural-log exponential or a missing
    normalisation fails one of them."""
    ln2 = math.log(2.0)
    o_a = torch.tensor([[[2.0, 4.0]]]); o_b = torch.tensor([[[6.0, 8.0]]])
    out, merged = oracle.lse_combine(o_a, torch.tensor([[[math.log(2.0) / ln2]]]), o_b, torch.tensor([[[math.log(6.0) / ln2]]]))
    assert torch.allclose(out, torch.tensor([[[5.0, 7.0]]]), atol=1e-6)
    assert torch.allclose(merged, torch.tensor([[[math.log(8.0) / ln2]]]), atol=1e-6)
    out, merged = oracle.lse_combine(torch.zeros(1, 1, 2), torch.tensor([[[-math.inf]]]), torch.tensor([[[3.0, 9.0]]]),
                                     torch.tensor([[[2.0]]]))
    assert torch.equal(out, torch.tensor([[[3.0, 9.0]]])) and torch.equal(merged, torch.tensor([[[2.0]]]))
    # equal LSEs: the mean; the merged LSE is one more (base 2)
    out, merged = oracle.lse_combine(o_a, torch.tensor([[[3.0]]]), o_b, torch.tensor([[[3.0]]]))
    assert torch.equal(out, torch.tensor([[[4.0, 6.0]]])) and torch.equal(merged, torch.tensor([[[4.0]]]))
    # random inputs against the natural-log merge oracle (two shards)
    g = torch.Generator().manual_seed(3)
    a, b = torch.randn(3, 5, 16, generator=g), torch.randn(3, 5, 16, generator=g)
    la, lb = torch.randn(3, 5, 1, generator=g) * 4, torch.randn(3, 5, 1, generator=g) * 4
    out, merged = oracle.lse_combine(a, la, b, lb)
    ref, ref_lse = oracle.lse_merge(torch.stack([a, b]), torch.stack([la, lb]).squeeze(-1) * ln2)
    assert torch.allclose(out, ref, rtol=1e-5, atol=1e-6)
    assert torch.allclose(merged.squeeze(-1) * ln2, ref_lse, rtol=1e-5, atol=1e-5)
    # both inputs empty: NaN, as the reference's arithmetic gives
    out, _ = oracle.lse_combine(o_a, torch.tensor([[[-math.inf]]]), o_b, torch.tensor([[[-math.inf]]]))
    assert torch.isnan(out).all()
