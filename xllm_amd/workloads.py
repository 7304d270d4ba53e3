"""Synthetic paged-decode workloads: the five benchmark configurations and a seeded
generator of their inputs (context lengths, permuted block tables, slot mappings, K/V/Q).

Everything here is plain tensor construction shared by the tests and the benchmark; the
same bytes are handed to the GPU path and, as CPU copies, to the checker.
"""
import math
from dataclasses import dataclass, replace

import torch


@dataclass(frozen=True)
class DecodeConfig:
    name: str
    batch: int
    n_q_heads: int
    n_kv_heads: int
    head_dim: int          # QK dim (MLA: latent + rope)
    block_size: int
    len_lo: int
    len_hi: int
    len_dist: str = "uniform"   # "uniform" | "loguniform"
    cache_dtype: str = "bf16"   # "bf16" | "fp8"
    mla: bool = False
    v_dim: int = 0              # MLA: latent dim
    sigma: float = 1.0
    sm_scale: float = 0.0       # 0 -> 1/sqrt(head_dim)
    pool_pages: int = 0         # 0 -> ceil(total pages * 1.10)

    @property
    def scale(self):
        return self.sm_scale if self.sm_scale > 0 else 1.0 / math.sqrt(self.head_dim)

    @property
    def dv(self):
        return self.v_dim if self.mla else self.head_dim


CONFIGS = {
    "tiny": DecodeConfig("tiny", 4, 8, 8, 128, 16, 64, 512, pool_pages=256),
    "llama3_8b": DecodeConfig("llama3_8b", 64, 32, 8, 128, 16, 512, 4096),
    "long_b256": DecodeConfig("long_b256", 256, 64, 8, 128, 128, 1024, 8192, len_dist="loguniform"),
    "fp8_kv": DecodeConfig("fp8_kv", 128, 32, 8, 128, 16, 2048, 16384, cache_dtype="fp8"),
    "mla_dsv3": DecodeConfig("mla_dsv3", 64, 128, 1, 576, 64, 2048, 16384, mla=True, v_dim=512,
                             sigma=0.5, sm_scale=1.0 / math.sqrt(192.0)),
    # side workloads (not among the five configurations above): 64-dim and 256-dim heads, and the MLA head count of an
    # 8-way tensor-parallel shard
    "gqa_d64": DecodeConfig("gqa_d64", 64, 32, 8, 64, 16, 1024, 8192),
    "gqa_d256": DecodeConfig("gqa_d256", 64, 16, 4, 256, 16, 512, 4096),
    "gqa_d64_fp8": DecodeConfig("gqa_d64_fp8", 64, 32, 8, 64, 16, 2048, 16384, cache_dtype="fp8"),
    "gqa_d256_fp8": DecodeConfig("gqa_d256_fp8", 64, 16, 4, 256, 16, 1024, 8192, cache_dtype="fp8"),
    "mla_tp8": DecodeConfig("mla_tp8", 64, 16, 1, 576, 64, 2048, 16384, mla=True, v_dim=512,
                            sigma=0.5, sm_scale=1.0 / math.sqrt(192.0)),
}


def scaled(cfg, batch=None, len_lo=None, len_hi=None):
    """A smaller instance of a configuration (same head layout) for oracle-sized tests."""
    return replace(cfg, batch=batch or cfg.batch, len_lo=len_lo or cfg.len_lo,
                   len_hi=len_hi or cfg.len_hi, pool_pages=0)


def draw_seq_lens(cfg, gen):
    if cfg.len_dist == "loguniform":
        u = torch.rand(cfg.batch, generator=gen, dtype=torch.float64)
        lens = torch.exp(math.log(cfg.len_lo) + u * (math.log(cfg.len_hi) - math.log(cfg.len_lo)))
        lens = lens.round().clamp(cfg.len_lo, cfg.len_hi).to(torch.int32)
    else:
        lens = torch.randint(cfg.len_lo, cfg.len_hi + 1, (cfg.batch,), generator=gen, dtype=torch.int32)
    return lens


@dataclass
class PageLayout:
    seq_lens: torch.Tensor        # [B] int32 (context incl. the new token)
    block_table: torch.Tensor     # [B, W] int32, padding value `pad`
    num_blocks: int
    indptr: torch.Tensor          # CSR forms of the same layout
    indices: torch.Tensor
    last_page_len: torch.Tensor
    ctx_slots: torch.Tensor       # [sum(L-1)] int32: slots of the tokens already cached
    new_slots: torch.Tensor       # [B] int32: slot of each sequence's new token
    ctx_offsets: torch.Tensor     # [B+1] int64 offsets into the context token stream


def make_layout(cfg, seed, pad=0, extra_cols=3):
    """Context lengths, a seeded random permutation of the page pool dealt to the sequences,
    and the slot ids of every token.  `pad` fills unused table columns (the reference pads
    with 0; its DCU layer rewrites that to -1)."""
    gen = torch.Generator().manual_seed(seed)
    lens = draw_seq_lens(cfg, gen)
    bs = cfg.block_size
    n_pages = (lens.to(torch.int64) + bs - 1) // bs
    total = int(n_pages.sum())
    pool = cfg.pool_pages if cfg.pool_pages else int(math.ceil(total * 1.10))
    assert pool >= total, "page pool too small for the drawn context lengths"
    perm = torch.randperm(pool, generator=gen, dtype=torch.int64)[:total].to(torch.int32)
    indptr = torch.zeros(cfg.batch + 1, dtype=torch.int32)
    indptr[1:] = torch.cumsum(n_pages, 0).to(torch.int32)
    width = int(n_pages.max()) + extra_cols
    table = torch.full((cfg.batch, width), pad, dtype=torch.int32)
    for b in range(cfg.batch):
        table[b, : int(n_pages[b])] = perm[int(indptr[b]) : int(indptr[b + 1])]
    last_page_len = (lens - (n_pages.to(torch.int32) - 1) * bs).to(torch.int32)

    # slot of token t of sequence b: table[b, t // bs] * bs + t % bs
    ctx_slots, new_slots = [], []
    offsets = torch.zeros(cfg.batch + 1, dtype=torch.int64)
    for b in range(cfg.batch):
        L = int(lens[b])
        t = torch.arange(L, dtype=torch.int64)
        slots = table[b, (t // bs)].to(torch.int64) * bs + t % bs
        ctx_slots.append(slots[: L - 1].to(torch.int32))
        new_slots.append(slots[L - 1 :].to(torch.int32))
        offsets[b + 1] = offsets[b] + (L - 1)
    return PageLayout(lens, table, pool, indptr, perm.contiguous(), last_page_len,
                      torch.cat(ctx_slots), torch.cat(new_slots), offsets)


def randn_16bit(shape, sigma, gen, device, dtype=torch.bfloat16, chunk=1 << 26):
    """N(0, sigma) drawn in fp32 and rounded once; generated in slabs to bound memory."""
    out = torch.empty(shape, dtype=dtype, device=device)
    flat = out.view(-1)
    for i in range(0, flat.numel(), chunk):
        n = min(chunk, flat.numel() - i)
        flat[i : i + n] = (torch.randn(n, generator=gen, device=device, dtype=torch.float32) * sigma).to(dtype)
    return out


@dataclass
class DecodeInputs:
    cfg: DecodeConfig
    layout: PageLayout
    q: torch.Tensor          # [B, Hq, Dqk]
    k_ctx: torch.Tensor      # [sum(L-1), Hkv, Dqk]  rows already in the cache
    v_ctx: torch.Tensor      # same for V (None for MLA)
    k_new: torch.Tensor      # [B, Hkv, Dqk]  this step's rows
    v_new: torch.Tensor


def make_inputs(cfg, seed, device="cpu", dtype=torch.bfloat16, layout=None):
    layout = layout or make_layout(cfg, seed)
    gen = torch.Generator(device=device).manual_seed(seed + 1)
    n_ctx = int(layout.ctx_offsets[-1])
    B, Hq, Hkv, D = cfg.batch, cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim
    q = randn_16bit((B, Hq, D), cfg.sigma, gen, device, dtype)
    k_ctx = randn_16bit((n_ctx, Hkv, D), cfg.sigma, gen, device, dtype)
    k_new = randn_16bit((B, Hkv, D), cfg.sigma, gen, device, dtype)
    v_ctx = v_new = None
    if not cfg.mla:
        v_ctx = randn_16bit((n_ctx, Hkv, D), cfg.sigma, gen, device, dtype)
        v_new = randn_16bit((B, Hkv, D), cfg.sigma, gen, device, dtype)
    return DecodeInputs(cfg, layout, q, k_ctx, v_ctx, k_new, v_new)


def gqa_bytes(cfg, seq_lens, elem_bytes_kv, elem_bytes_q=2):
    """Algorithmic HBM bytes of one GQA decode: every K and V element of every context token
    once, Q in and O out once, the used block-table entries and seq_lens once."""
    lens = seq_lens.to(torch.int64)
    kv = int(lens.sum()) * cfg.n_kv_heads * cfg.head_dim * 2 * elem_bytes_kv
    qo = cfg.batch * cfg.n_q_heads * cfg.head_dim * 2 * elem_bytes_q
    table = int(((lens + cfg.block_size - 1) // cfg.block_size).sum()) * 4 + cfg.batch * 4
    return kv + qo + table


def mla_bytes_flops(cfg, seq_lens):
    lens = int(seq_lens.to(torch.int64).sum())
    nbytes = lens * cfg.head_dim * 2 + cfg.batch * cfg.n_q_heads * (cfg.head_dim + cfg.v_dim) * 2
    flops = lens * cfg.n_q_heads * 2 * (cfg.head_dim + cfg.v_dim)
    return nbytes, flops


def reshape_bytes(n_tokens, row_elems, in_bytes, cache_bytes, tensors=2):
    return n_tokens * row_elems * tensors * (in_bytes + cache_bytes) + n_tokens * 4
