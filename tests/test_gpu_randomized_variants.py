"""Randomly drawn shapes through both families of scan kernels.

The coalesced row fetch (forced on launches of any width, 16-row and 32-row matrix instructions alternating) and the
plain scans must select the same blocks, set the same access flags and give the same context, bit for bit: a score
depends on nothing but its token and comes from the same chain of matrix instructions in every variant.  The draw
covers head dims 64 / 128, GQA groups of 1 to 8, batches of 1 to 3, prefill and single-token queries, dense tensors
and paged caches of page size 1 and 16 with ragged sequence lengths.  Every eighth case is also run through the oracle.
"""
import os
import random

import numpy as np
import pytest
import torch

from oracle import hip12 as O
from helpers import make_inputs, to_paged
from gpu_utils import assert_context_close, assert_metadata_equal, run_product

pytestmark = pytest.mark.gpu

_SWITCHES = ("HIPATTN_MASK_DMA", "HIPATTN_MASK_DMA_INLINE", "HIPATTN_MASK_M16", "HIP_ATTN_PRESCALE_K")


def _draw(rng, it):
    D = rng.choice([64, 128, 128])
    HKV = rng.choice([1, 2, 4])
    G = rng.choice([1, 2, 4, 4, 8])
    decode = rng.random() < 0.4
    TK = rng.choice([3000, 4096, 8192, 12000])
    TQ = 1 if decode else rng.choice([64, 200, 300, 512])
    B = rng.choice([1, 2, 3])
    paged = rng.choice([1, 16]) if decode else rng.choice([0, 0, 1, 16])
    sw = rng.choice([256, 512, 1024])
    return dict(D=D, HKV=HKV, H=HKV * G, decode=decode, TK=TK, TQ=TQ, B=B, paged=paged, sw=sw, seed=100 + it)


def test_coalesced_and_plain_scans_agree_on_random_shapes():
    rng = random.Random(7)
    saved = {k: os.environ.get(k) for k in _SWITCHES}
    try:
        for it in range(32):
            c = _draw(rng, it)
            print(f"[case {it}] {c}", flush=True)
            if c["decode"]:
                lens = np.array([rng.randint(c["TK"] // 2, c["TK"]) for _ in range(c["B"])])
                X = make_inputs(c["seed"], B=c["B"], TQ=1, TK=c["TK"], H=c["H"], HKV=c["HKV"], D=c["D"], dtype="bf16",
                                pos=(lens - 1)[:, None])
            else:
                lens = None
                X = make_inputs(c["seed"], B=c["B"], TQ=c["TQ"], TK=c["TK"], H=c["H"], HKV=c["HKV"], D=c["D"], dtype="bf16")
            A = O.OArgs(sliding_window_size=c["sw"])
            if c["paged"]:
                X = to_paged(X, c["paged"], seed=it, seq_lens=lens) if c["decode"] else to_paged(X, c["paged"], seed=it)
                A.extend_context_length = c["TK"]
            os.environ["HIP_ATTN_PRESCALE_K"] = "0" if c["decode"] else "1"
            res = {}
            for tag, env in (("coalesced", {"HIPATTN_MASK_DMA": "2", "HIPATTN_MASK_DMA_INLINE": "1",
                                            "HIPATTN_MASK_M16": str(it % 2)}),
                             ("plain", {"HIPATTN_MASK_DMA": "0", "HIPATTN_MASK_DMA_INLINE": "0"})):
                os.environ.update(env)
                ctx, meta = run_product(X, A, require_cache_statistics=True)
                res[tag] = (ctx, meta)
            (ca, ma), (cb, mb) = res["coalesced"], res["plain"]
            assert torch.equal(ma.indices, mb.indices) and torch.equal(ma.ks, mb.ks), f"case {it}: masks differ"
            assert torch.equal(ma.mask_cache_statistics.access_counter, mb.mask_cache_statistics.access_counter), \
                f"case {it}: access flags differ"
            assert torch.equal(ca.view(torch.int16), cb.view(torch.int16)), f"case {it}: contexts differ"
            if it % 8 == 0:
                octx, ometa = O.hip_attention_12(X, A)
                assert_metadata_equal(ma, ometa)
                assert_context_close(ca, octx, "bf16")
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
