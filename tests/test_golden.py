"""Committed fixtures (tests/golden/*.npz): the oracle still reproduces them; the GPU path matches them.

These vectors were written by ``tests/golden/make_fixtures.py`` from the CPU oracle (the reference repository ships
no golden vectors for this path); ``tests/golden/reference_*.npz``, written by an execution of the reference itself,
are covered by ``tests/test_golden_reference.py``.
"""
import glob
import json
import os

import numpy as np
import pytest

from oracle import hip12 as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FILES = sorted(f for f in glob.glob(os.path.join(GOLDEN, "*.npz")) if not os.path.basename(f).startswith("reference_"))


def load(path):
    z = np.load(path, allow_pickle=False)
    spec = json.loads(bytes(z["spec"]).decode())
    get = lambda k: z[k] if k in z.files else None  # noqa: E731
    X = O.OInputs(spec["dtype"], z["q"], z["pos"], k=get("k"), v=get("v"), k_cache=get("k_cache"),
                  v_cache=get("v_cache"), block_table=get("block_table"), cache_seq_lens=get("cache_seq_lens"))
    a = spec["args"]
    A = O.OArgs(**{**a, "stages": [O.OStage(*s) for s in a["stages"]],
                   "extend_context_length": spec["extend_context_length"]})
    return z, X, A


def test_fixtures_present():
    assert len(FILES) >= 3


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[:-4] for f in FILES])
def test_oracle_reproduces_fixture(path):
    z, X, A = load(path)
    ctx, meta = O.hip_attention_12(X, A)
    assert np.array_equal(meta.indices, z["indices"])
    assert np.array_equal(meta.ks, z["ks"])
    assert np.array_equal(meta.ks_start_end, z["ks_start_end"])
    assert np.array_equal(meta.mask_access, z["mask_access"])
    assert np.array_equal(meta.sa_access, z["sa_access"])
    assert np.array_equal(ctx, z["context"])
    # the vectors are not degenerate: blocks are selected and they differ between query blocks or batch items
    assert int(z["ks"].min()) > 0 and int((z["indices"] < O.INT64_MAX).sum()) > 0


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[:-4] for f in FILES])
def test_gpu_matches_fixture(path):
    import torch

    from gpu_utils import assert_context_close, run_product

    print(f"[case] golden {os.path.basename(path)}", flush=True)
    z, X, A = load(path)
    ctx, meta = run_product(X, A)
    assert np.array_equal(meta.indices.cpu().numpy(), z["indices"])
    assert np.array_equal(meta.ks.cpu().numpy(), z["ks"])
    assert np.array_equal(meta.ks_start_end.cpu().numpy(), z["ks_start_end"])
    assert np.array_equal(meta.mask_cache_statistics.access_counter.cpu().numpy(), z["mask_access"])
    assert np.array_equal(meta.sa_cache_statistics.access_counter.cpu().numpy(), z["sa_access"])
    assert_context_close(ctx, z["context"], X.dtype)
    assert isinstance(ctx, torch.Tensor)
