"""The five benchmark configurations at FULL size and on their WHOLE batch: cache bytes bit-exact and every
sequence's attention output against the reference's libtorch CPU path (the ATen oracle).

Cost on a 16-core host: tiny and llama3_8b a fraction of a second, long_b256 and fp8_kv a few seconds, mla_dsv3
about half a minute of oracle time, plus the transfer of the caches (up to 4 GB) to the host."""
import pytest
import torch

import oracle
from helpers import assert_close_to_reference
from xllm_amd import ops, workloads

pytestmark = pytest.mark.gpu


def _expected_cache(inp, k_scale, v_scale):
    """The caches the reference's scatter produces from the token streams, on the CPU.  16-bit pages: the
    permutation copy of the C oracle.  fp8 pages: the ATen form of the quantisation (byte-equal to the C oracle on
    finite inputs, which the CPU tests pin) in slabs, scattered by slot."""
    cfg, lay = inp.cfg, inp.layout
    shape = (lay.num_blocks, cfg.block_size, cfg.n_kv_heads, cfg.head_dim)
    fp8 = cfg.cache_dtype == "fp8"
    kc = torch.zeros(shape, dtype=torch.uint8 if fp8 else torch.bfloat16)
    vc = None if cfg.mla else torch.zeros_like(kc)
    for k, v, slots in ((inp.k_ctx, inp.v_ctx, lay.ctx_slots), (inp.k_new, inp.v_new, lay.new_slots)):
        k = k.cpu()
        v = None if v is None else v.cpu()
        if not fp8:
            oracle.reshape_and_cache(k, v, kc, vc, slots)
            continue
        rows = slots.long()
        for x, cache, scale in ((k, kc, k_scale), (v, vc, v_scale)):
            flat = cache.view(-1, cfg.n_kv_heads * cfg.head_dim)
            for i in range(0, x.shape[0], 1 << 17):
                part = x[i : i + (1 << 17)].contiguous()
                flat[rows[i : i + (1 << 17)]] = oracle.aten_fp8_quantize(part, scale).view(part.shape[0], -1)
    return kc, vc


@pytest.mark.parametrize("name", ["tiny", "llama3_8b", "long_b256", "fp8_kv", "mla_dsv3"])
def test_whole_batch_full_size_parity(device, name):
    cfg = workloads.CONFIGS[name]
    inp = workloads.make_inputs(cfg, 2, device=device)
    lay = inp.layout
    fp8 = cfg.cache_dtype == "fp8"
    shape = (lay.num_blocks, cfg.block_size, cfg.n_kv_heads, cfg.head_dim)
    kg = torch.zeros(shape, dtype=torch.float8_e4m3fn if fp8 else torch.bfloat16, device=device)
    vg = None if cfg.mla else torch.zeros_like(kg)
    ks = vs = None
    if fp8:
        ks = ops.kv_head_scales(torch.cat([inp.k_ctx, inp.k_new]))
        vs = ops.kv_head_scales(torch.cat([inp.v_ctx, inp.v_new]))
        assert torch.equal(ks.cpu(), oracle.kv_head_scales(torch.cat([inp.k_ctx, inp.k_new]).cpu()))
        assert torch.equal(vs.cpu(), oracle.kv_head_scales(torch.cat([inp.v_ctx, inp.v_new]).cpu()))
    store = ops.quant_to_paged_cache if fp8 else ops.reshape_paged_cache
    for k, v, slots in ((inp.k_ctx, inp.v_ctx, lay.ctx_slots), (inp.k_new, inp.v_new, lay.new_slots)):
        store(ops.ReshapePagedCacheParams(key=k, value=v, k_cache=kg, v_cache=vg, slot_mapping=slots.to(device),
                                          k_cache_scale=ks, v_cache_scale=vs))
    max_len = int(lay.seq_lens.max())
    if cfg.mla:
        B, H = cfg.batch, cfg.n_q_heads
        p = ops.DenseDecodeParams(
            q_nope=inp.q[:, :, : cfg.v_dim].contiguous().view(B, 1, H, cfg.v_dim),
            q_pe=inp.q[:, :, cfg.v_dim :].contiguous().view(B, 1, H, cfg.head_dim - cfg.v_dim),
            k_cache=kg, seqlens_k=lay.seq_lens.to(device), block_table=lay.block_table.to(device),
            head_size_v=cfg.v_dim, softmax_scale=cfg.scale)
        out, lse = ops.dense_decode(p, return_lse=True, max_seq_len=max_len)
        out = out.view(B, H, cfg.v_dim)
    else:
        out = torch.empty_like(inp.q)
        out, lse = ops.batch_decode(inp.q, kg, out, lay.block_table.to(device), lay.seq_lens.to(device), v_cache=vg,
                                    k_cache_quant_scale=ks, v_cache_quant_scale=vs, scale=cfg.scale,
                                    return_lse=True, max_seq_len=max_len)
        # the same step from a plan made once (as the layers after the first see it): bit-identical
        plan = ops.update_decode_plan_info(cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size, kg.dtype,
                                           block_table=lay.block_table.to(device), seq_lens=lay.seq_lens.to(device))
        out_p, lse_p = ops.batch_decode(inp.q, kg, torch.empty_like(inp.q), lay.block_table.to(device),
                                        lay.seq_lens.to(device), v_cache=vg, k_cache_quant_scale=ks,
                                        v_cache_quant_scale=vs, scale=cfg.scale, return_lse=True, max_seq_len=max_len,
                                        plan=plan)
        assert torch.equal(out_p, out) and torch.equal(lse_p, lse), "planned decode differs from the plain one"
        assert ops.decode_status(device) == 0
    torch.cuda.synchronize()
    out, lse = out.cpu(), lse.cpu().view(cfg.batch, cfg.n_q_heads)

    # (1) cache bytes, all of them
    ks_c = None if ks is None else ks.cpu()
    vs_c = None if vs is None else vs.cpu()
    kc, vc = _expected_cache(inp, ks_c, vs_c)
    kg_c = kg.cpu()
    vg_c = None if vg is None else vg.cpu()
    del kg, vg
    assert torch.equal(kg_c.view(kc.dtype), kc), "K cache bytes differ from the reference scatter"
    if vc is not None:
        assert torch.equal(vg_c.view(vc.dtype), vc), "V cache bytes differ from the reference scatter"
    del kg_c, vg_c

    # (2) every sequence of the batch against the reference's libtorch decode
    q = inp.q.cpu()
    ref = oracle.aten_paged_decode(q, kc, vc, lay.block_table, lay.seq_lens, cfg.scale, ks_c, vs_c, dv=cfg.dv)
    mx, mean = assert_close_to_reference(out, ref, name)
    print(f"{name}: {cfg.batch} sequences, {int(lay.seq_lens.sum())} context tokens, longest {max_len}: "
          f"max-abs {mx:.3e} mean-abs {mean:.3e}")
    # the LSE of a sample (the oracle computes it with a second pass over the pages)
    sample = sorted({0, cfg.batch // 2, cfg.batch - 1, int(lay.seq_lens.argmax()), int(lay.seq_lens.argmin())})
    ref_lse = oracle.aten_paged_decode_lse(q[sample].contiguous(), kc, lay.block_table[sample].contiguous(),
                                           lay.seq_lens[sample].contiguous(), cfg.scale, ks_c)
    assert torch.allclose(lse[sample], ref_lse, rtol=1e-3, atol=1e-3)
