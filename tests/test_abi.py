"""The C-ABI library loads and exports every symbol include/hipattn.h declares (no compute calls)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "hipattn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hipattn_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = _declared_functions()
    for must in ("hipattn_mask_stage", "hipattn_select_stage", "hipattn_finalize_indices", "hipattn_bsa_prefill",
                 "hipattn_bsa_decode_partial", "hipattn_bsa_decode_merge", "hipattn_bsa_decode", "hipattn_version"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from hip_attn import _native

    lib = ctypes.CDLL(_native.lib_path())
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/hipattn.h but not exported"
    assert b"gfx950" in _native.lib().hipattn_version()


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "hip-attention_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.lower(), f"{f} mentions the oracle"


def test_cpu_tensor_is_rejected_loudly():
    import pytest
    import torch
    from hip_attn import HiPAttentionArgs12, hip_attention_12
    from hip_attn._native import HipAttnError

    q = torch.zeros(1, 4, 2, 64)
    with pytest.raises(HipAttnError):
        hip_attention_12(q, q, q, HiPAttentionArgs12())


def test_far_key_rows_predicate():
    """hipattn_kv_rows_beyond_32gib: the rule the scan launcher applies before it uses 31-bit piece numbers."""
    from hip_attn import _native

    lib = _native.lib()
    BF16 = 1  # HIPATTN_BF16

    def kv(tsrc, hkv, hid, batch_stride=None, paged=0, fp8=0):
        s = _native.KVStruct()
        s.paged, s.HKV, s.tsrc, s.fp8 = paged, hkv, tsrc, fp8
        s.k_stride_h, s.k_stride_t = hid, hkv * hid
        s.k_stride_b = batch_stride if batch_stride is not None else tsrc * hkv * hid
        return s

    def far(s, B, hid, dtype=BF16):
        return lib.hipattn_kv_rows_beyond_32gib(ctypes.byref(s), ctypes.c_int32(B), ctypes.c_int32(hid), ctypes.c_int32(dtype))

    # 1M keys x 8 heads x 128 bf16 = 2 GiB per item: 15 items stay under 32 GiB, 16 reach it, 17 exceed it
    assert far(kv(1 << 20, 8, 128), 15, 128) == 0
    assert far(kv(1 << 20, 8, 128), 16, 128) == 1
    assert far(kv(1 << 20, 8, 128), 17, 128) == 1
    # one byte short of 32 GiB / exactly 32 GiB in a single item
    assert far(kv((1 << 24) - 1, 8, 128), 1, 128) == 0
    assert far(kv(1 << 24, 8, 128), 1, 128) == 1
    # a batch stride wider than the item (a view into a larger buffer) counts
    assert far(kv(1 << 20, 8, 128, batch_stride=1 << 34), 2, 128) == 1
    assert far(kv(1 << 20, 8, 128, batch_stride=-(1 << 34)), 2, 128) == 1
    # fp8 rows are half as long; a paged pool cannot be judged from its description
    assert far(kv(1 << 24, 8, 128, fp8=1), 1, 128) == 0
    assert far(kv(1 << 10, 8, 128, paged=1), 1, 128) == 1
    assert lib.hipattn_kv_rows_beyond_32gib(None, ctypes.c_int32(1), ctypes.c_int32(128), ctypes.c_int32(BF16)) < 0
