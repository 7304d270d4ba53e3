"""The C++ host side (torch::Tensor interface registered as torch.ops.xllm_ops.*) gives the same
bytes as the direct C-ABI calls and follows the reference's schema."""
import math

import pytest
import torch

import oracle
from helpers import assert_close_to_reference, fill_caches_cpu
from xllm_amd import ops, workloads

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def xops(device):
    from xllm_amd import torch_ops
    return torch_ops.load()


def test_reshape_and_decode_through_the_dispatcher(device, xops):
    cfg = workloads.scaled(workloads.CONFIGS["llama3_8b"], batch=6, len_lo=40, len_hi=1500)
    inp = workloads.make_inputs(cfg, 17)
    lay = inp.layout
    shape = (lay.num_blocks, cfg.block_size, cfg.n_kv_heads, cfg.head_dim)
    kg = torch.zeros(shape, dtype=torch.bfloat16, device=device)
    vg = torch.zeros_like(kg)
    for k, v, slots in ((inp.k_ctx, inp.v_ctx, lay.ctx_slots), (inp.k_new, inp.v_new, lay.new_slots)):
        ret = xops.reshape_paged_cache(slots.to(device), k.to(device), v.to(device), kg, vg)
        assert ret.data_ptr() == kg.data_ptr()          # the reference's op returns key_cache
    kc, vc = fill_caches_cpu(inp)
    assert torch.equal(kg.cpu(), kc) and torch.equal(vg.cpu(), vc)
    q = inp.q.to(device)
    out = torch.empty_like(q)
    out, lse = xops.batch_decode(q, kg, vg, out, lay.block_table.to(device), lay.seq_lens.to(device), None, None,
                                 int(lay.seq_lens.max()), cfg.scale)
    ref = oracle.aten_paged_decode(inp.q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale)
    assert_close_to_reference(out, ref, "dispatcher batch_decode")
    direct = torch.empty_like(q)
    ops.batch_decode(q, kg, direct, lay.block_table.to(device), lay.seq_lens.to(device), v_cache=vg,
                     scale=cfg.scale, max_seq_len=int(lay.seq_lens.max()))
    assert torch.equal(out, direct)
    assert tuple(lse.shape) == (cfg.batch, cfg.n_q_heads, 1) and lse.dtype == torch.float32


def test_fp8_mla_and_merge_through_the_dispatcher(device, xops):
    g = torch.Generator().manual_seed(3)
    T, P, bs, H, D = 48, 4, 16, 2, 128
    key = torch.randn(T, H, D, generator=g).to(torch.bfloat16)
    val = torch.randn(T, H, D, generator=g).to(torch.bfloat16)
    slots = torch.randperm(P * bs, generator=g)[:T].to(torch.int32)
    ks, vs = oracle.kv_head_scales(key), oracle.kv_head_scales(val)
    kg = torch.zeros(P, bs, H, D, dtype=torch.float8_e4m3fn, device=device)
    vg = torch.zeros_like(kg)
    xops.quant_to_paged_cache(slots.to(device), key.to(device), val.to(device), kg, vg, ks.to(device), vs.to(device))
    kc = torch.zeros(P, bs, H, D, dtype=torch.uint8)
    vc = torch.zeros_like(kc)
    oracle.reshape_and_cache(key, val, kc, vc, slots, ks, vs)
    assert torch.equal(kg.view(torch.uint8).cpu(), kc) and torch.equal(vg.view(torch.uint8).cpu(), vc)

    cfg = workloads.DecodeConfig("mla", 2, 16, 1, 576, 64, 30, 300, mla=True, v_dim=512, sigma=0.5,
                                 sm_scale=1 / math.sqrt(192.0))
    inp = workloads.make_inputs(cfg, 5)
    lay = inp.layout
    cache = torch.zeros(lay.num_blocks, 64, 1, 576, dtype=torch.bfloat16, device=device)
    for k, slots in ((inp.k_ctx, lay.ctx_slots), (inp.k_new, lay.new_slots)):
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=k.to(device), k_cache=cache,
                                                            slot_mapping=slots.to(device)))
    q = inp.q.to(device)
    out, lse = xops.mla_dense_decode(q[:, :, :512].contiguous().view(2, 1, 16, 512),
                                     q[:, :, 512:].contiguous().view(2, 1, 16, 64), cache,
                                     lay.seq_lens.to(device), lay.block_table.to(device), 512, cfg.scale)
    ref = oracle.aten_paged_decode(inp.q, cache.cpu(), None, lay.block_table, lay.seq_lens, cfg.scale, dv=512)
    assert_close_to_reference(out.view(2, 16, 512), ref, "dispatcher mla")
    # DcpAttentionMergeTest.WeightsPartialOutputsByNaturalLogLse on the device
    po = torch.tensor([2.0, 4.0, 6.0, 8.0], device=device).reshape(2, 1, 1, 1, 2)
    pl = torch.tensor([math.log(2.0), math.log(6.0)], device=device).reshape(2, 1, 1, 1)
    mo, ml = xops.merge_dcp_attention_shards(po, pl)
    assert torch.allclose(mo.cpu(), torch.tensor([5.0, 7.0]).reshape(1, 1, 1, 2))
    assert torch.allclose(ml.cpu(), torch.tensor([math.log(8.0)]).reshape(1, 1, 1))
    po = torch.tensor([0.0, 0.0, 3.0, 9.0], device=device).reshape(2, 1, 1, 1, 2)
    pl = torch.tensor([-math.inf, math.log(4.0)], device=device).reshape(2, 1, 1, 1)
    mo, ml = xops.merge_dcp_attention_shards(po, pl)
    assert torch.equal(mo.cpu(), torch.tensor([3.0, 9.0]).reshape(1, 1, 1, 2))
    mo, ml = xops.merge_dcp_attention_shards(torch.ones(2, 1, 1, 2, 3, device=device),
                                             torch.full((2, 1, 2, 1), -math.inf, device=device))
    assert torch.equal(mo.cpu(), torch.zeros(1, 1, 2, 3)) and torch.isneginf(ml).all()


def test_mla_store_and_decode_in_one_call_through_the_dispatcher(device, xops):
    """mla_dense_decode with latent_cache and slot_mapping (flash_mla::store_and_dense_decode) against the store
    followed by the decode, both through the dispatcher: 128 heads (the rows are stored inside the decode launch) and
    16 heads (the host side's library call issues two launches), with and without the step's plan."""
    for heads in (128, 16):
        cfg = workloads.DecodeConfig(f"mla{heads}", 4, heads, 1, 576, 64, 1, 900, mla=True, v_dim=512, sigma=0.5,
                                     sm_scale=1 / math.sqrt(192.0))
        inp = workloads.make_inputs(cfg, 50 + heads)
        lay = inp.layout
        cache0 = torch.full((lay.num_blocks, 64, 1, 576), float("nan"), dtype=torch.bfloat16, device=device)
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=inp.k_ctx.to(device), k_cache=cache0,
                                                            slot_mapping=lay.ctx_slots.to(device)))
        q = inp.q.to(device)
        qn = q[:, :, :512].contiguous().view(4, 1, heads, 512)
        qp = q[:, :, 512:].contiguous().view(4, 1, heads, 64)
        lens, table = lay.seq_lens.to(device), lay.block_table.to(device)
        latent, slots = inp.k_new.to(device), lay.new_slots.to(device)
        for planned in (False, True):
            plan = xops.mla_decoding_metadata(lens, table, heads, 64) if planned else None
            ca = cache0.clone()
            ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=latent, k_cache=ca, slot_mapping=slots))
            out_a, lse_a = xops.mla_dense_decode(qn, qp, ca, lens, table, 512, cfg.scale, False, plan)
            cb = cache0.clone()
            out_b, lse_b = xops.mla_dense_decode(qn, qp, cb, lens, table, 512, cfg.scale, False, plan, latent, slots)
            torch.cuda.synchronize()
            assert torch.equal(ca.view(torch.int16), cb.view(torch.int16))
            assert torch.equal(out_a.view(torch.int16), out_b.view(torch.int16)) and torch.equal(lse_a, lse_b)
            assert torch.isfinite(out_b.float()).all()
        ref = oracle.aten_paged_decode(inp.q, cb.cpu(), None, lay.block_table, lay.seq_lens, cfg.scale, dv=512)
        assert_close_to_reference(out_b.view(4, heads, 512), ref, cfg.name)


def test_query_chunks_and_latent_gather_through_the_dispatcher(device, xops):
    cfg = workloads.DecodeConfig("shim_chunks", 5, 32, 8, 128, 16, 10, 600)
    inp = workloads.make_inputs(cfg, 23)
    lay = inp.layout
    from helpers import fill_caches_gpu
    kg, vg, _, _ = fill_caches_gpu(inp, device)
    g = torch.Generator().manual_seed(5)
    q_lens = [int(torch.randint(1, min(16, int(L)) + 1, (1,), generator=g)) for L in lay.seq_lens]
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    q = (torch.randn(int(cu[-1]), cfg.n_q_heads, cfg.head_dim, generator=g) * cfg.sigma).to(torch.bfloat16).to(device)
    out = xops.paged_forward(q, torch.empty_like(q), kg, vg, lay.block_table.to(device), lay.seq_lens.to(device),
                             cu.to(device), cfg.scale, True, 0, 0)
    direct = ops.paged_forward(q, torch.empty_like(q), kg, vg, lay.block_table.to(device), lay.seq_lens.to(device),
                               cu.to(device), scale=cfg.scale)
    torch.cuda.synchronize()
    assert torch.equal(out, direct)
    # latent gather with the reference's argument list
    mla = workloads.DecodeConfig("shim_gather", 4, 16, 1, 576, 64, 1, 500, mla=True, v_dim=512)
    inp = workloads.make_inputs(mla, 9)
    lay = inp.layout
    kc, _ = fill_caches_cpu(inp)
    kv_cu = torch.zeros(mla.batch + 1, dtype=torch.int32)
    kv_cu[1:] = lay.seq_lens.cumsum(0)
    got = xops.gather_mla_latent_cache(kc.to(device), lay.block_table.to(device), kv_cu.to(device), int(kv_cu[-1]),
                                       int(lay.seq_lens.max()))
    assert torch.equal(got.cpu(), oracle.gather_paged_rows(kc, lay.block_table, kv_cu, int(kv_cu[-1])))


def test_norm_rope_and_metadata_update_through_the_host_side(device, xops):
    # fused_qk_norm_rope with the reference's arguments (kernels/cuda/cuda_ops_api.h:235-249) and its variant that
    # also writes the cache: same bytes as the direct C-ABI calls
    g = torch.Generator().manual_seed(3)
    T, n_q, n_k, D = 9, 8, 2, 128
    qkv = (torch.randn(T, (n_q + 2 * n_k) * D, generator=g) * 0.3).to(torch.bfloat16).to(device)
    qw = (1 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).to(device)
    kw = (1 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).to(device)
    ang = torch.rand(64, D // 2, generator=g) * 6.28
    cs = torch.cat([ang.cos(), ang.sin()], 1).to(device)
    pos = torch.randint(0, 64, (T,), generator=g).to(device)
    slots = torch.randperm(64, generator=g)[:T].to(torch.int32).to(device)
    direct = ops.fused_qk_norm_rope(qkv.clone(), n_q, n_k, n_k, D, 1e-6, qw, kw, cs, False, pos)
    via = qkv.clone()
    ret = xops.fused_qk_norm_rope(via, n_q, n_k, n_k, D, 1e-6, qw, kw, cs, False, pos)
    torch.cuda.synchronize()
    assert torch.equal(via, direct) and ret.data_ptr() == via.data_ptr()   # the reference's op returns qkv
    kc = torch.zeros(4, 16, n_k, D, dtype=torch.bfloat16, device=device)
    vc = torch.zeros_like(kc)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(kc)
    via2 = qkv.clone()
    xops.fused_qk_norm_rope_and_cache(via2, n_q, n_k, n_k, D, 1e-6, qw, kw, cs, False, pos, slots, kc, vc, None, None)
    ops.fused_qk_norm_rope(qkv.clone(), n_q, n_k, n_k, D, 1e-6, qw, kw, cs, False, pos, k_cache=kc2, v_cache=vc2,
                           slot_mapping=slots)
    torch.cuda.synchronize()
    assert torch.equal(via2, direct) and torch.equal(kc, kc2) and torch.equal(vc, vc2) and bool(kc.abs().sum() > 0)
    # the graph executor's metadata update under the reference's op name and schema
    # (kernels/cuda/cuda_ops_library.cpp:161-252, 288-295), against the oracle
    from test_oracle_reshape import _metadata_case
    src, want = _metadata_case(21, 9, 16)
    _, got = _metadata_case(21, 9, 16)
    n_tok, n_idx = src["tokens"].numel(), src["paged_kv_indices"].numel()
    oracle.llm_decode_metadata_update(src, want, n_tok, 16, 9, n_idx)
    sd = {k: v.to(device) for k, v in src.items()}
    dd = {k: v.to(device) for k, v in got.items()}
    ret = xops.update_decode_graph_metadata(sd["tokens"], sd["positions"], sd["new_cache_slots"], sd["kv_seq_lens"],
                                            sd["paged_kv_indptr"], sd["paged_kv_indices"], sd["paged_kv_last_page_len"],
                                            dd["tokens"], dd["positions"], dd["new_cache_slots"], dd["kv_seq_lens"],
                                            dd["kv_seq_lens_delta"], dd["paged_kv_indptr"], dd["paged_kv_indices"],
                                            dd["paged_kv_last_page_len"], 16)
    torch.cuda.synchronize()
    assert ret.data_ptr() == dd["tokens"].data_ptr()
    for k in want:
        assert torch.equal(dd[k].cpu(), want[k]), k


def test_absorbed_products_through_the_host_side(device, xops):
    # the two bmm calls of the absorbed MLA attention (layers/dcu/deepseek_v2_attention.cpp:428-430, 231-238)
    # written the reference's way against the op that stands for them: same values as the direct C-ABI call, and
    # the decode kernel between them takes the result as it comes
    g = torch.Generator().manual_seed(21)
    T, H = 5, 16
    q = torch.randn(T, H, 192, generator=g).bfloat16().to(device)
    w_kc = (torch.randn(H, 128, 512, generator=g) / math.sqrt(128)).bfloat16().to(device)
    w_vc = (torch.randn(H, 512, 128, generator=g) / math.sqrt(512)).bfloat16().to(device)
    q_nope = q[..., :128]
    got = xops.mla_absorbed_bmm(q_nope, w_kc)
    assert got.is_contiguous() and got.shape == (T, H, 512)
    assert torch.equal(got, ops.absorbed_bmm(q_nope, w_kc))
    _, exact = oracle.absorbed_bmm(q_nope.cpu(), w_kc.cpu())
    assert ((got.cpu().float() - exact).abs() <= exact.abs() * 2.0 ** -8 + 1e-4).all()
    back = xops.mla_absorbed_bmm(got, w_vc)
    _, exact = oracle.absorbed_bmm(got.cpu(), w_vc.cpu())
    assert ((back.cpu().float() - exact).abs() <= exact.abs() * 2.0 ** -8 + 1e-4).all()
    with pytest.raises(RuntimeError):
        xops.mla_absorbed_bmm(q_nope, w_vc)


def test_block_table_padding_mask_through_the_host_side(device, xops):
    # mask_block_table_padding with the reference's arguments (layers/dcu/flash_attention.cpp:194-218); int64
    # lengths as torch::diff leaves them are accepted
    g = torch.Generator().manual_seed(2)
    table = torch.randint(0, 99, (6, 12), generator=g, dtype=torch.int32)
    lens = torch.tensor([0, 5, 16, 17, 12 * 16, 100], dtype=torch.int64)
    got = xops.mask_block_table_padding(table.to(device), lens.to(device), 16)
    assert got.dtype == torch.int32
    assert torch.equal(got.cpu(), oracle.mask_block_table_padding(table, lens.int(), 16))
