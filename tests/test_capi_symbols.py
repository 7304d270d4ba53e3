"""The C-ABI library loads without a GPU and exports exactly what include/xllm_mi355.h declares."""
import ctypes
import os
import re

import pytest

from xllm_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "xllm_mi355.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xllm_mi355_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_table_agree():
    declared = _declared_functions()
    assert declared, "no declarations found in the header"
    assert sorted(capi.SIGNATURES) == declared


def test_library_loads_and_exports_every_declared_symbol():
    if not os.path.exists(capi.LIB_PATH):
        pytest.fail(f"{capi.LIB_PATH} is missing: run `python -m xllm_amd.build`")
    lib = ctypes.CDLL(capi.LIB_PATH)
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"


def test_host_only_entry_points_without_a_gpu():
    lib = capi.lib()
    assert re.fullmatch(rb"\d+\.\d+\.\d+", lib.xllm_mi355_version())
    assert lib.xllm_mi355_error_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6, -7):
        assert len(lib.xllm_mi355_error_string(code)) > 4
    # argument validation happens before any HIP call
    assert lib.xllm_mi355_reshape_and_cache(None, None, None, None, None, None, None, 4, 8, 128, 16, 10,
                                            1024, 1024, capi.BF16, capi.BF16, None) == -1
    assert lib.xllm_mi355_paged_decode_gqa(None, None, None, None, None, None, 0, None, None, None, 4, 32,
                                           8, 128, 16, 10, 4096, 4096, 100, -1, 0.1, None, 0, capi.BF16,
                                           capi.BF16, None) == -1
    assert lib.xllm_mi355_paged_decode_mla(None, None, None, None, None, None, 0, None, 4, 128, 512, 64, 64,
                                           10, 100, 0.1, None, 0, capi.BF16, None) == -1
    assert lib.xllm_mi355_lse_merge(None, None, None, None, 2, 1, 1, 8, capi.FP32, None) == -1
    assert lib.xllm_mi355_reshape_and_cache(None, None, None, None, None, None, None, 0, 8, 128, 16, 10,
                                            1024, 1024, capi.BF16, capi.BF16, None) == 0  # no tokens: no-op
    # the entry points either side of the path: null pointers, shapes and alignments they do not take
    fake = 1 << 20  # an aligned non-null address: the calls below return before anything is launched
    bmm = lib.xllm_mi355_mla_absorbed_bmm
    assert bmm(None, None, None, 4, 16, 128, 512, 2048, 128, 8192, 512, capi.BF16, None) == -1
    assert bmm(fake, fake, fake, 0, 16, 128, 512, 2048, 128, 8192, 512, capi.BF16, None) == 0      # no tokens: no-op
    assert bmm(fake, fake, fake, 4, 16, 96, 512, 1536, 96, 8192, 512, capi.BF16, None) == -3       # K not a multiple of 128
    assert bmm(fake, fake, fake, 4, 16, 128, 48, 2048, 128, 768, 48, capi.BF16, None) == -3        # N not a multiple of 64
    assert bmm(fake, fake, fake, 4, 16, 128, 512, 2048, 128, 8192, 512, capi.FP16, None) == -2     # bf16 only
    assert bmm(fake + 2, fake, fake, 4, 16, 128, 512, 2048, 128, 8192, 512, capi.BF16, None) == -5
    assert bmm(fake, fake, fake, 4, 16, 128, 512, 2048, 64, 8192, 512, capi.BF16, None) == -1      # heads overlap in x
    mask = lib.xllm_mi355_mask_block_table_padding
    assert mask(None, 8, None, None, 8, 4, 8, 16, None) == -1
    assert mask(fake, 4, fake, fake, 8, 4, 8, 16, None) == -1                                      # row stride below the width
    assert mask(fake, 8, fake, fake, 8, 4, 8, 0, None) == -1                                       # block size
    assert mask(fake, 8, fake, fake, 8, 0, 8, 16, None) == 0                                       # empty batch: no-op
    assert lib.xllm_mi355_rope_and_cache(fake, None, None, fake + 4, fake, None, None, None, None, None, 4, 6144, 32, 8,
                                         8, 128, 128, 1e-6, 0, 16, 10, capi.BF16, capi.FP32, capi.BF16, None) == -5
    # workspace sizes are positive and grow with the head dim
    a = lib.xllm_mi355_paged_decode_gqa_workspace_bytes(64, 32, 128)
    b = lib.xllm_mi355_paged_decode_gqa_workspace_bytes(64, 32, 256)
    c = lib.xllm_mi355_paged_decode_mla_workspace_bytes(64, 128, 16384)
    assert 0 < a < b and c > 0
    # the variant is named, not guessed from a width: a GQA head dim of 512 is not taken for the MLA latent
    assert lib.xllm_mi355_paged_decode_gqa_workspace_bytes(64, 32, 512) > b
    # (the first form of the call still answers, for callers written against it)
    assert lib.xllm_mi355_paged_decode_workspace_bytes(64, 32, 128, 4096) == a
    assert lib.xllm_mi355_paged_decode_workspace_bytes(64, 128, 512, 16384) == c


def test_planned_decode_refuses_a_short_plan_buffer_before_any_launch():
    """A planned decode reads its plan up to the last word before it looks at the signature: a buffer that is too
    small must be refused on the host (XLLM_MI355_EWORKSPACE), whatever else the call holds."""
    lib = capi.lib()
    fake = 1 << 20
    need = lib.xllm_mi355_paged_decode_plan_bytes()
    assert need > 1 << 20

    def planned(plan, plan_bytes):
        return lib.xllm_mi355_paged_decode_gqa_planned(
            plan, plan_bytes, fake, fake, fake, fake, None, fake, 8, fake, None, None, None, None, None,
            4, 32, 8, 128, 16, 10, 4096, 4096, 100, -1, 0.1, fake, 1 << 30, capi.BF16, capi.BF16, None)

    assert planned(None, need) == -1
    assert planned(fake, 0) == -4
    assert planned(fake, 4096) == -4
    assert planned(fake, need - 1) == -4

    def mla_planned(plan, plan_bytes):
        return lib.xllm_mi355_paged_decode_mla_planned(
            plan, plan_bytes, fake, fake, fake, fake, None, fake, 8, fake, 4, 128, 512, 64, 64, 10, 100, 0.1, fake,
            1 << 30, capi.BF16, None)

    assert mla_planned(None, need) == -1
    assert mla_planned(fake, 4096) == -4
    assert mla_planned(fake, need - 1) == -4
    assert lib.xllm_mi355_paged_decode_mla_plan(fake, need - 1, fake, 8, fake, 4, 128, 64, None) == -4
    assert lib.xllm_mi355_paged_decode_mla_plan(fake, need, None, 8, fake, 4, 128, 64, None) == -1


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(capi.XllmMi355Error):
        capi.lib()


def test_python_ops_refuse_cpu_tensors():
    import torch
    from xllm_amd import ops
    k = torch.zeros(2, 1, 64, dtype=torch.bfloat16)
    cache = torch.zeros(1, 16, 1, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=k, value=k, k_cache=cache, v_cache=cache,
                                                            slot_mapping=torch.zeros(2, dtype=torch.int32)))
    # every op of the mirror refuses host tensors: there is no CPU path behind it
    x = torch.zeros(2, 4, 128, dtype=torch.bfloat16)
    w = torch.zeros(4, 128, 64, dtype=torch.bfloat16)
    table = torch.zeros(2, 3, dtype=torch.int32)
    lens = torch.ones(2, dtype=torch.int32)
    qkv = torch.zeros(2, 6 * 64, dtype=torch.bfloat16)
    for call in (lambda: ops.absorbed_bmm(x, w),
                 lambda: ops.mask_block_table_padding(table, lens, 16),
                 lambda: ops.fused_qk_norm_rope(qkv, 4, 1, 1, 64, 1e-6, torch.ones(64, dtype=torch.bfloat16),
                                                torch.ones(64, dtype=torch.bfloat16), torch.zeros(8, 64), False,
                                                torch.zeros(2, dtype=torch.int64)),
                 lambda: ops.gather_mla_latent_cache(torch.zeros(1, 16, 1, 576, dtype=torch.bfloat16), table,
                                                     torch.zeros(3, dtype=torch.int32), 4)):
        with pytest.raises(ValueError):
            call()
