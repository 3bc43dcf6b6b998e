"""Random small configurations: an execution of the reference (Triton's CPU interpreter) against the oracle.

Run in a container that holds the reference checkout (never on the GPU box):

    python tests/golden/sweep_against_reference.py SEED COUNT [/root/reference]

Every configuration draws batch size, lengths, head counts, head dim, three scan stages (block sizes, strides, chunk
sizes, stage_k, stage stride), sink, window, second_stage_k, stage_early_terminate, the attention block size, dense or paged keys and,
sometimes, RoPE on load; it runs the operator once fresh, once with the returned metadata handed back and once
restarting from the cached inputs of stage 1, and prints whether block indices, ks and access flags are equal and how
far the contexts are apart.  Prefixes are kept long enough for every stage to have more scored chunks than it keeps:
with fewer, the reference's ``torch.topk`` has to choose among never-scored chunks of equal score, and its choice on
the CPU is arbitrary (the oracle and the HIP path take the lowest positions).  Decode with ``sink_token_size == 0``
ends in a ZeroDivisionError inside the reference (its launcher divides by the number of sink programs), and a restart
at a stage whose block size or stride differs from stage 0's is refused by the oracle: both print as ERROR.
"""
import os, sys, time, traceback
HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)
import numpy as np, torch
import make_reference_fixtures as G
from oracle import hip12 as O
ext, meta = G.load_reference(sys.argv[3] if len(sys.argv) > 3 else '/root/reference')
rng = np.random.default_rng(int(sys.argv[1]) if len(sys.argv) > 1 else 0)
N = int(sys.argv[2]) if len(sys.argv) > 2 else 10

def one(case):
    B, TQ, TK, H, HKV, D, stages, sink, sw, second_k, bsbq, lens, page, extend, bk_arg, early, mctx = case
    g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
    short = lambda t: t.to(torch.bfloat16).float()
    q = short(torch.randn((B, TQ, H, D), generator=g) * 0.5); k = short(torch.randn((B, TK, HKV, D), generator=g)); v = short(torch.randn((B, TK, HKV, D), generator=g))
    if lens is None: pos = (torch.arange(TQ) + TK - TQ)[None].expand(B, TQ).contiguous()
    else: pos = (torch.tensor(lens, dtype=torch.int64)[:, None] - TQ + torch.arange(TQ)[None]).contiguous()
    kw = dict(sink_token_size=sink, sliding_window_size=sw, second_stage_k=second_k, block_sparse_block_size_q=bsbq,
              stages=[meta.ScanStage(stage_block_size_q=a, stage_block_stride_q=b, stage_chunk_size=c, stage_k=d, stage_stride=e) for (a, b, c, d, e) in stages],
              require_cache_statistics=True, position_ids=pos, block_size_k=bk_arg, stage_early_terminate=early,
              model_context_length=mctx)
    okw = dict(sink_token_size=sink, sliding_window_size=sw, second_stage_k=second_k, block_sparse_block_size_q=bsbq,
               stages=[O.OStage(*s) for s in stages], block_size_k=bk_arg, stage_early_terminate=early,
               model_context_length=mctx)
    X = None
    if extend is not None:
        cos, sin = G.rope_tables(2 * TK, D); cos, sin = short(cos), short(sin)
        kw.update(using_extend=True, need_apply_rope=True, rope_cos=cos, rope_sin=sin, scan_extend_backend=extend[0], sa_extend_backend=extend[1])
        okw.update(using_extend=True, need_apply_rope=True, scan_extend_backend=extend[0], sa_extend_backend=extend[1])
    if page > 0:
        per = -(-TK // page); npages = B * per + 4
        perm = (torch.randperm(npages - 1, generator=g)[: B * per] + 1).reshape(B, per)
        kc = torch.zeros((npages, page, HKV, D)); vc = torch.zeros_like(kc)
        for b in range(B):
            for pg in range(per):
                t0, t1 = pg * page, min(TK, (pg + 1) * page)
                kc[perm[b, pg], : t1 - t0] = k[b, t0:t1]; vc[perm[b, pg], : t1 - t0] = v[b, t0:t1]
        seq = pos.max(dim=1).values + 1
        kw.update(k_cache=kc, v_cache=vc, block_table=perm.to(torch.int64), cache_seq_lens=seq.to(torch.int64), extend_context_length=TK)
        ctx, md = ext.dual_stage_quadratic_hip_attention(q, None, None, args=meta.HiPAttentionArgs(**kw))
        X = O.OInputs("f32", q.numpy(), pos.numpy(), k_cache=kc.numpy(), v_cache=vc.numpy(), block_table=perm.numpy().astype(np.int64), cache_seq_lens=seq.numpy().astype(np.int64))
        okw["extend_context_length"] = TK
    else:
        ctx, md = ext.dual_stage_quadratic_hip_attention(q, k, v, args=meta.HiPAttentionArgs(**kw))
        X = O.OInputs("f32", q.numpy(), pos.numpy(), k=k.numpy(), v=v.numpy())
    if extend is not None: X.rope_cos, X.rope_sin = cos.numpy(), sin.numpy()
    octx, ometa = O.hip_attention_12(X, O.OArgs(**okw))
    # second call with the metadata handed back (mask reused), and one restarting from stage 1's cached inputs
    kd = (None, None) if page > 0 else (k, v)
    ctx2, md2 = ext.dual_stage_quadratic_hip_attention(q, *kd, args=meta.HiPAttentionArgs(**kw), cached_metadata=md)
    octx2, _ = O.hip_attention_12(X, O.OArgs(**okw), cached=ometa)
    err2 = float(np.abs(octx2 - ctx2.float().numpy()).max())
    part = meta.HiPAttentionOutputMetadata(indices=None, ks=None, ks_count=None, ks_start_end=None, mask_cache_statistics=None, sa_cache_statistics=None, stage_caches=list(md.stage_caches[:2]))
    ctx3, md3 = ext.dual_stage_quadratic_hip_attention(q, *kd, args=meta.HiPAttentionArgs(**kw), cached_metadata=part)
    opart = O.OMetadata(None, None, None, None, stage_caches=list(ometa.stage_caches[:2]))
    octx3, ometa3 = O.hip_attention_12(X, O.OArgs(**okw), cached=opart)
    err3 = float(np.abs(octx3 - ctx3.float().numpy()).max()) if np.array_equal(ometa3.indices, md3.indices.numpy()) else 99.0
    ok_idx = np.array_equal(ometa.indices, md.indices.numpy()) and np.array_equal(ometa.ks, md.ks.numpy())
    err = max(float(np.abs(octx - ctx.float().numpy()).max()), err2, err3)
    fl = lambda st: (st.access_counter > 0).numpy()
    ok_fl = np.array_equal(ometa.mask_access > 0, fl(md.mask_cache_statistics)) and np.array_equal(ometa.sa_access > 0, fl(md.sa_cache_statistics))
    return ok_idx, err, ok_fl

def rand_case():
    D = int(rng.choice([32, 64])); HKV = int(rng.choice([1, 2])); G_ = int(rng.choice([1, 2, 4])); H = HKV * G_
    B = int(rng.choice([1, 2]))
    decode = rng.random() < 0.4
    TK = int(rng.choice([1536, 2048, 3072]))
    TQ = 1 if decode else int(rng.choice([32, 48, 64, 100, 128]))
    c0 = int(rng.choice([32, 64])); c1 = int(rng.choice([8, 16])); c2 = int(rng.choice([1, 2, 4, 8]))
    if c2 > c1: c2 = c1
    bq0 = int(rng.choice([32, 64])); bq2 = int(rng.choice([16, 32])) if bq0 == 32 else int(rng.choice([32, 64]))
    bq1 = bq0 if rng.random() < 0.5 else bq2
    sq0 = int(rng.choice([1, 2, 4])); sq1 = int(rng.choice([1, 2])); sq2 = int(rng.choice([1, 2]))
    sq0 = min(sq0, bq0 // 16); sq1 = min(sq1, bq1 // 16); sq2 = min(sq2, bq2 // 16)
    k1 = int(rng.choice([4, 8])) * c0; k2 = int(rng.choice([8, 16, 32])) * c1
    ss0 = int(rng.choice([1, 1, 2]))
    stages = [(bq0, sq0, c0, None, ss0), (bq1, sq1, c1, k1, 1), (bq2, sq2, c2, k2, 1)]
    sink = int(rng.choice([0, 4, 16, 32, 100])); sw = int(rng.choice([64, 128, 256])) ; sw = max(sw, 2 * c0)
    second_k = int(rng.choice([16, 32, 64])) * c2
    second_k = min(second_k, k2)
    bsbq = int(rng.choice([16, 32, 64])); bsbq = min(bsbq, bq2) if rng.random() < 0.7 else bsbq
    lens = None
    if decode or rng.random() < 0.4:
        lens = [int(rng.integers(int(0.75 * TK), TK + 1)) for _ in range(B)]
    page = int(rng.choice([0, 0, 1, 4, 16]))
    extend = None
    if rng.random() < 0.4:
        extend = (str(rng.choice(["relative", "streaming", "infllm", "dynamic_extend"])), str(rng.choice(["streaming", "infllm"])))
    bk_arg = int(rng.choice([32, 64]))
    early = int(rng.choice([1, 1, 2, 4]))
    mctx = int(rng.choice([131072, 1024, 512]))  # small values put the queries beyond the model's context
    return (B, TQ, TK, H, HKV, D, stages, sink, sw, second_k, bsbq, lens, page, extend, bk_arg, early, mctx)

for i in range(N):
    case = rand_case()
    t0 = time.time()
    try:
        ok_idx, err, ok_fl = one(case)
        tag = "OK " if (ok_idx and err < 5e-5 and ok_fl) else "MISMATCH"
        print(f"[{i}] {tag} idx={ok_idx} ctx_err={err:.2e} flags={ok_fl} {time.time()-t0:.0f}s case={case}", flush=True)
    except AssertionError as e:
        tb = traceback.extract_tb(e.__traceback__)[-1]
        print(f"[{i}] ASSERT at {os.path.basename(tb.filename)}:{tb.lineno} {tb.line} case={case}", flush=True)
    except Exception as e:
        tb = traceback.extract_tb(e.__traceback__)[-1]
        print(f"[{i}] ERROR {type(e).__name__}: {str(e)[:200]} at {os.path.basename(tb.filename)}:{tb.lineno} case={case}", flush=True)
