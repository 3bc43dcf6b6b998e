"""Shared synthetic-input builders for the oracle and GPU parity tests."""
import numpy as np

from oracle import hip12 as O


def make_inputs(seed, B, TQ, TK, H, HKV, D, dtype="f32", pos=None, scale=1.0):
    rng = np.random.default_rng(seed)
    q = (rng.standard_normal((B, TQ, H, D)) * scale).astype(np.float32)
    k = rng.standard_normal((B, TK, HKV, D)).astype(np.float32)
    v = rng.standard_normal((B, TK, HKV, D)).astype(np.float32)
    if pos is None:
        pos = np.broadcast_to((np.arange(TQ) + TK - TQ)[None], (B, TQ))
    pos = np.ascontiguousarray(pos, dtype=np.int64)
    if dtype == "bf16":
        q, k, v = (O.f32_to_bf16_bits(a) for a in (q, k, v))
    return O.OInputs(dtype, q, pos, k=k, v=v)


def to_paged(X, page_size, seed=0, seq_lens=None, extra_pages=3):
    """Scatter dense K/V into a paged cache through a shuffled block table (page 0 is a dummy)."""
    B, TK, HKV, D = X.k.shape
    rng = np.random.default_rng(seed)
    per = -(-TK // page_size)
    npages = B * per + 1 + extra_pages
    perm = rng.permutation(np.arange(1, npages))[: B * per].reshape(B, per)
    kc = np.zeros((npages, page_size, HKV, D), dtype=X.k.dtype)
    vc = np.zeros_like(kc)
    for b in range(B):
        for p in range(per):
            t0 = p * page_size
            t1 = min(TK, t0 + page_size)
            kc[perm[b, p], : t1 - t0] = X.k[b, t0:t1]
            vc[perm[b, p], : t1 - t0] = X.v[b, t0:t1]
    if seq_lens is None:
        seq_lens = X.pos.max(axis=1) + 1
    return O.OInputs(X.dtype, X.q, X.pos, k_cache=kc, v_cache=vc,
                     block_table=perm.astype(np.int64), cache_seq_lens=np.asarray(seq_lens, dtype=np.int64))


def widen(a, dtype):
    return O.bf16_bits_to_f32(a) if dtype == "bf16" else np.asarray(a, dtype=np.float32)


def tiny_args(**kw):
    base = dict(sink_token_size=16, sliding_window_size=256, second_stage_k=512, block_sparse_block_size_q=32,
                stages=[O.OStage(32, 2, 64, None, 1), O.OStage(32, 2, 16, 2048, 1), O.OStage(32, 1, 2, 1024, 1)])
    base.update(kw)
    return O.OArgs(**base)


def rope_tables(length, D, dtype="f32", theta=10000.0):
    """cos/sin tables [length, D] in the layout serving stacks keep (both halves repeat the D/2 frequencies),
    as float32 values representable in ``dtype``; also returns the float64 angles [length, D/2]."""
    inv = theta ** (-np.arange(0, D, 2, dtype=np.float64) / D)
    ang = np.arange(length, dtype=np.float64)[:, None] * inv[None, :]
    cos = np.concatenate([np.cos(ang), np.cos(ang)], axis=1).astype(np.float32)
    sin = np.concatenate([np.sin(ang), np.sin(ang)], axis=1).astype(np.float32)
    if dtype == "bf16":
        cos = O.bf16_bits_to_f32(O.f32_to_bf16_bits(cos))
        sin = O.bf16_bits_to_f32(O.f32_to_bf16_bits(sin))
    return cos, sin, ang


def with_rope(X, length, dtype=None, scan_backend=None, sa_backend=None):
    """Attach RoPE tables (and optionally the rotation rules) to an OInputs."""
    D = X.q.shape[-1]
    cos, sin, _ = rope_tables(length, D, dtype or X.dtype)
    X.rope_cos, X.rope_sin = cos, sin
    X.scan_backend, X.sa_backend = scan_backend, sa_backend
    return X
