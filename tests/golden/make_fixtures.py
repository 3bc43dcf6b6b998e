#!/usr/bin/env python3
"""Writes the fixtures in this directory: small seeded inputs and what the CPU oracle returns for them.

The reference repository holds no golden vectors or known-answer files for ``hip_attention_12`` (its tests compare
against its own kernels at run time), so these vectors come from ``oracle/`` -- the restatement that the tests under
``tests/test_oracle_*.py`` pin against closed forms and brute force.  They freeze that behaviour: a later change to
the oracle or to the kernels that alters a selected block shows up against files that do not move.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

from oracle import hip12 as O  # noqa: E402
from helpers import make_inputs, to_paged  # noqa: E402

CASES = {
    # name: (input kwargs, page size or None, sequence lengths or None, args)
    "f32_dense_prefill": (
        dict(seed=101, B=1, TQ=96, TK=640, H=2, HKV=1, D=32, dtype="f32"), None, None,
        dict(sink_token_size=16, sliding_window_size=128, second_stage_k=128, block_sparse_block_size_q=32,
             stages=[(32, 2, 32, None, 1), (32, 2, 8, 256, 1), (32, 1, 2, 128, 1)])),
    "bf16_paged_decode_gqa": (
        dict(seed=102, B=2, TQ=1, TK=512, H=4, HKV=2, D=64, dtype="bf16"), 4, [512, 300],
        dict(sink_token_size=16, sliding_window_size=64, second_stage_k=128,
             stages=[(64, 4, 32, None, 1), (64, 4, 16, 256, 1), (64, 1, 8, 128, 1)])),
    "bf16_dense_prefill_gqa": (
        dict(seed=103, B=1, TQ=128, TK=768, H=4, HKV=2, D=64, dtype="bf16"), None, None,
        dict(sink_token_size=32, sliding_window_size=128, second_stage_k=256,
             stages=[(64, 4, 64, None, 1), (64, 4, 16, 512, 1), (64, 1, 8, 256, 1)])),
}


def build(name):
    kw, page, lens, a = CASES[name]
    kw = dict(kw)
    if lens is not None:
        kw["pos"] = (np.array(lens) - 1)[:, None] if kw["TQ"] == 1 else None
    X = make_inputs(**kw)
    if page is not None:
        X = to_paged(X, page, seed=kw["seed"], seq_lens=lens)
    A = O.OArgs(**{**a, "stages": [O.OStage(*s) for s in a["stages"]],
                   "extend_context_length": kw["TK"]})
    return X, A


def main():
    for name in CASES:
        X, A = build(name)
        ctx, meta = O.hip_attention_12(X, A)
        arrays = dict(q=X.q, pos=X.pos, context=ctx, indices=meta.indices, ks=meta.ks, ks_start_end=meta.ks_start_end,
                      mask_access=meta.mask_access, sa_access=meta.sa_access)
        for key in ("k", "v", "k_cache", "v_cache", "block_table", "cache_seq_lens"):
            val = getattr(X, key)
            if val is not None:
                arrays[key] = val
        arrays["spec"] = np.frombuffer(json.dumps({"dtype": X.dtype, "args": CASES[name][3],
                                                   "extend_context_length": CASES[name][0]["TK"]}).encode(), dtype=np.uint8)
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **arrays)
        print(name, os.path.getsize(path), "bytes; indices", meta.indices.shape)


if __name__ == "__main__":
    main()
