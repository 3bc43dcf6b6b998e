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
