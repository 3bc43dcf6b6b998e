"""Golden vectors from an execution of the reference's own v1.2 code (mask estimation + sparse attention).

Run in a container that holds the reference checkout (never on the GPU box):

    python tests/golden/make_reference_fixtures.py /root/reference

The reference cannot be imported as a package here: ``hip_attn/__init__.py`` pulls model code and the v1.0 / v1.1
generations, and the v1.2 modules import ``cv2``, ``numba``, ``cuda`` (cuda-python) and a JIT-compiled cupy helper,
none of which are installed.  This script therefore
  * registers empty parent packages (``hip_attn``, ``hip_attn.v1_2``, ``hip_attn.utils``, ``hip_attn.v1_1...``) whose
    ``__path__`` points into the checkout, so that the five v1.2 modules and ``utils/rope.py`` load by their own
    names without any ``__init__`` running,
  * registers placeholder modules for the absent third-party imports (they are only used by debug plotting and by
    the UVM cache, which these fixtures do not touch),
  * runs the Triton kernels under ``TRITON_INTERPRET=1`` (Triton's CPU interpreter) on CPU tensors, with the three
    ``torch.cuda`` calls of the driver answered for a machine without a GPU.
Only data leaves this script: inputs and the reference's outputs, saved as ``reference_*.npz`` next to it.
"""
import os
import sys
import types

os.environ["TRITON_INTERPRET"] = "1"
os.environ.setdefault("HIP_DISABLE_AUTOTUNE", "1")

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def _package(name, path):
    m = types.ModuleType(name)
    m.__path__ = [path]
    sys.modules[name] = m
    return m


def _placeholder(name, **attrs):
    m = types.ModuleType(name)
    for k, v in attrs.items():
        setattr(m, k, v)
    sys.modules[name] = m
    return m


def load_reference(root):
    src = os.path.join(root, "src", "hip_attn")
    _package("hip_attn", src)
    _package("hip_attn.v1_2", os.path.join(src, "v1_2"))
    _package("hip_attn.utils", os.path.join(src, "utils"))
    _package("hip_attn.v1_1", os.path.join(src, "v1_1"))
    _package("hip_attn.v1_1.offload_runner", os.path.join(src, "v1_1", "offload_runner"))

    def _decorator(*a, **k):  # numba.njit / numba.jit used with and without arguments
        if len(a) == 1 and callable(a[0]) and not k:
            return a[0]
        return lambda f: f

    _placeholder("cv2")
    nb = _placeholder("numba", njit=_decorator, jit=_decorator, prange=range)
    nb.cuda = _placeholder("numba.cuda", jit=_decorator)
    cu = _placeholder("cuda")
    cu.cudart = _placeholder("cuda.cudart")
    _placeholder("hip_attn.v1_1.offload_runner.tensor_from_pointer", alloc_managed_tensor=None, sizeof=None)

    # the driver asks the CUDA runtime about devices and graph capture (attention_extend.py:1980, 2196-2197, 2636)
    torch.cuda.current_device = lambda: 0
    torch.cuda.set_device = lambda *_a, **_k: None
    torch.cuda.is_current_stream_capturing = lambda: False
    torch.cuda.get_device_name = lambda *_a, **_k: "none"  # only picks autotune candidates (attention_extend_bsa.py:571)

    import hip_attn.v1_2.attention_extend as ext
    import hip_attn.v1_2.attention_metadata as meta
    return ext, meta


def rope_tables(length, D, theta=10000.0):
    inv = theta ** (-np.arange(0, D, 2, dtype=np.float64) / D)
    ang = np.arange(length, dtype=np.float64)[:, None] * inv[None, :]
    cos = np.concatenate([np.cos(ang), np.cos(ang)], axis=1).astype(np.float32)
    sin = np.concatenate([np.sin(ang), np.sin(ang)], axis=1).astype(np.float32)
    return torch.from_numpy(cos), torch.from_numpy(sin)


def bits16(t):
    """Upper halves of the float32 patterns (exact: the values were rounded to 8 significant bits)."""
    w = t.float().contiguous().view(torch.int32)
    assert bool(((w & 0xFFFF) == 0).all())
    return ((w >> 16) & 0xFFFF).to(torch.int32).numpy().astype(np.uint16)


def access_flags(md, suffix):
    """Which key rows the mask estimation and the attention touched (counters > 0), bit-packed."""
    out = {}
    for name, st in (("mask_access", md.mask_cache_statistics), ("sa_access", md.sa_cache_statistics)):
        if st is not None and st.access_counter is not None:
            flags = (st.access_counter > 0).numpy()
            out[f"{name}_shape{suffix}"] = np.array(flags.shape)
            out[f"{name}{suffix}"] = np.packbits(flags.reshape(-1))
    return out


def make_case(ext, meta, name, seed, B, TQ, TK, H, HKV, D, stages, sink, sw, second_k, bsbq, dtype=torch.float32,
              lens=None, page_size=0, extend=None, softcap=None, block_size_k=64, replay=False, exact=False,
              model_ctx=None, early=None, causal=True, rope_len=None):
    """One call of the reference operator; ``lens`` (decode: TQ == 1) places each sequence's query at lens[b] - 1;
    ``page_size`` > 0 moves K/V into a paged cache behind a shuffled block table; ``extend`` = (scan rule, sa rule)
    turns on RoPE applied on load; ``model_ctx`` sets model_context_length (the dynamic_extend rule reads it);
    ``early`` sets stage_early_terminate; ``causal=False`` passes ``is_causal=False`` (attention kernels only)."""
    g = torch.Generator().manual_seed(seed)
    # values with 8 significant bits, so that the files can hold q, k, v as 16-bit patterns
    short = lambda t: t.to(torch.bfloat16).to(dtype)  # noqa: E731
    if exact:  # full float32 draws, v = k: stored as float32, v not stored
        q = torch.randn((B, TQ, H, D), generator=g, dtype=torch.float32)
        k = torch.randn((B, TK, HKV, D), generator=g, dtype=torch.float32)
        v = k.clone()
    else:
        q = short(torch.randn((B, TQ, H, D), generator=g, dtype=torch.float32) * 0.5)
        k = short(torch.randn((B, TK, HKV, D), generator=g, dtype=torch.float32))
        v = short(torch.randn((B, TK, HKV, D), generator=g, dtype=torch.float32))
    if lens is None:
        pos = (torch.arange(TQ) + TK - TQ)[None].expand(B, TQ).contiguous()
    else:
        pos = (torch.tensor(lens, dtype=torch.int64)[:, None] - TQ + torch.arange(TQ)[None]).contiguous()
    kw = dict(sink_token_size=sink, sliding_window_size=sw, second_stage_k=second_k, block_sparse_block_size_q=bsbq,
              stages=[meta.ScanStage(stage_block_size_q=a, stage_block_stride_q=b, stage_chunk_size=c, stage_k=d,
                                     stage_stride=e) for (a, b, c, d, e) in stages],
              require_cache_statistics=True, position_ids=pos, block_size_k=block_size_k)
    extra = {}
    if extend is not None:
        cos, sin = rope_tables(rope_len or 2 * TK, D)
        kw.update(using_extend=True, need_apply_rope=True, rope_cos=cos.to(dtype), rope_sin=sin.to(dtype),
                  scan_extend_backend=extend[0], sa_extend_backend=extend[1])
        extra.update(rope_cos=cos.to(dtype).float().numpy(), rope_sin=sin.to(dtype).float().numpy(),
                     scan_backend=extend[0], sa_backend=extend[1])
    if model_ctx is not None:
        kw.update(model_context_length=model_ctx)
        extra.update(model_context_length=model_ctx)
    if softcap is not None:
        kw.update(logit_softcap=softcap)
        extra.update(softcap=softcap)
    if early is not None:
        kw.update(stage_early_terminate=early)
        extra.update(stage_early_terminate=early)
    if not causal:
        kw.update(is_causal=False)
        extra.update(is_causal=0)
    if page_size > 0:
        per = -(-TK // page_size)
        npages = B * per + 4
        perm = (torch.randperm(npages - 1, generator=g)[: B * per] + 1).reshape(B, per)
        kc = torch.zeros((npages, page_size, HKV, D), dtype=dtype)
        vc = torch.zeros_like(kc)
        for b in range(B):
            for pg in range(per):
                t0, t1 = pg * page_size, min(TK, (pg + 1) * page_size)
                kc[perm[b, pg], : t1 - t0] = k[b, t0:t1]
                vc[perm[b, pg], : t1 - t0] = v[b, t0:t1]
        seq = pos.max(dim=1).values + 1
        kw.update(k_cache=kc, v_cache=vc, block_table=perm.to(torch.int64), cache_seq_lens=seq.to(torch.int64),
                  extend_context_length=TK)
        extra.update(k_cache=bits16(kc), v_cache=bits16(vc), block_table=perm.numpy(),
                     cache_seq_lens=seq.numpy(), page_size=page_size)
        args = meta.HiPAttentionArgs(**kw)
        ctx, md = ext.dual_stage_quadratic_hip_attention(q, None, None, args=args)
    else:
        args = meta.HiPAttentionArgs(**kw)
        ctx, md = ext.dual_stage_quadratic_hip_attention(q, k, v, args=args)
    extra.update(access_flags(md, ""))
    if replay:
        # restart from the inputs of stage 1 (the chunk list stage 0 produced), as a serving step with a cached
        # first stage does
        part = meta.HiPAttentionOutputMetadata(indices=None, ks=None, ks_count=None, ks_start_end=None,
                                               mask_cache_statistics=None, sa_cache_statistics=None,
                                               stage_caches=list(md.stage_caches[:2]))
        kd = (None, None) if page_size > 0 else (k, v)
        ctx_r, md_r = ext.dual_stage_quadratic_hip_attention(q, *kd, args=meta.HiPAttentionArgs(**kw), cached_metadata=part)
        extra.update(context_replay=ctx_r.float().numpy(), indices_replay=md_r.indices.numpy())
    path = os.path.join(HERE, f"reference_{name}.npz")
    if page_size > 0:  # the cache and the block table hold the same rows
        extra.update(max_tsrc=TK)
    elif exact:
        extra.update(k=k.numpy(), v_is_k=1)
    else:
        extra.update(k=bits16(k), v=bits16(v))
    np.savez_compressed(
        path, q=q.numpy() if exact else bits16(q), pos=pos.numpy(),
        context=ctx.float().numpy(), indices=md.indices.numpy(), ks=md.ks.numpy(), ks_start_end=md.ks_start_end.numpy(),
        stages=np.array([[-1 if x is None else x for x in s] for s in stages], dtype=np.int64),
        sink=sink, sw=sw, second_k=second_k, bsbq=bsbq, bf16=int(dtype == torch.bfloat16), block_size_k=block_size_k,
        **extra)
    print("wrote", path, "context", tuple(ctx.shape), "indices", tuple(md.indices.shape), flush=True)


def sweep_case(seed):
    """A random small configuration, drawn from ``seed``: batch, lengths, head counts, head dim, three scan stages
    (block sizes, strides, chunk sizes, stage_k, stage stride), sink, window, second_stage_k, stage_early_terminate,
    the attention block size, dense or paged keys and, sometimes, RoPE on load.  Prefixes stay long enough for every
    stage to score more chunks than it keeps (with fewer, the reference's ``torch.topk`` chooses among never-scored
    chunks of equal score, arbitrarily on the CPU), stage_early_terminate stays at or below the last chunk size (a
    stage whose chunks are narrower is not scored at all, which leaves the same arbitrary choice), and a decode case
    keeps a sink (the reference's decode launcher divides by its number of sink programs)."""
    rng = np.random.default_rng(seed)
    D = int(rng.choice([32, 64])); HKV = int(rng.choice([1, 2])); H = HKV * int(rng.choice([1, 2, 4]))
    B = int(rng.choice([1, 2]))
    decode = rng.random() < 0.4
    TK = int(rng.choice([1536, 2048]))
    TQ = 1 if decode else int(rng.choice([32, 48, 64, 100, 128]))
    c0 = int(rng.choice([32, 64])); c1 = int(rng.choice([8, 16])); c2 = min(c1, int(rng.choice([1, 2, 4, 8])))
    bq0 = int(rng.choice([32, 64])); bq2 = int(rng.choice([16, 32])) if bq0 == 32 else int(rng.choice([32, 64]))
    bq1 = bq0 if rng.random() < 0.5 else bq2
    sq0 = min(int(rng.choice([1, 2, 4])), bq0 // 16); sq1 = min(int(rng.choice([1, 2])), bq1 // 16)
    sq2 = min(int(rng.choice([1, 2])), bq2 // 16)
    k1 = int(rng.choice([4, 8])) * c0; k2 = int(rng.choice([8, 16, 32])) * c1
    stages = [(bq0, sq0, c0, None, int(rng.choice([1, 1, 2]))), (bq1, sq1, c1, k1, 1), (bq2, sq2, c2, k2, 1)]
    sink = int(rng.choice([4, 16, 32, 100] if decode else [0, 4, 16, 32, 100]))
    sw = max(int(rng.choice([64, 128, 256])), 2 * c0)
    second_k = min(int(rng.choice([16, 32, 64])) * c2, k2)
    bsbq = int(rng.choice([16, 32, 64]))
    if rng.random() < 0.7:
        bsbq = min(bsbq, bq2)
    lens = None
    if decode or rng.random() < 0.4:
        lens = [int(rng.integers(int(0.75 * TK), TK + 1)) for _ in range(B)]
    extra = dict(lens=lens, page_size=int(rng.choice([0, 0, 1, 4, 16])), block_size_k=int(rng.choice([32, 64])),
                 early=min(c2, int(rng.choice([1, 1, 2, 4]))), model_ctx=int(rng.choice([131072, 1024, 512])))
    if rng.random() < 0.4:
        extra["extend"] = (str(rng.choice(["relative", "streaming", "infllm", "dynamic_extend"])),
                           str(rng.choice(["streaming", "infllm"])))
    return (int(rng.integers(1 << 30)), B, TQ, TK, H, HKV, D, stages, sink, sw, second_k, bsbq, extra)


SWEEP_SEEDS = (101, 102, 103, 104, 105, 106, 107, 108)  # committed witnesses of the random sweep


def make_paged_api_case(name, seed, B, TQ, TK, H, HKV, D, lens, spec, layer_ids, orig_context_len, rope):
    """``forward_paged_hip`` (the serving entry point, paged_hip.py:35-320) on a token-granular pool: one call per
    layer id, and for decode a second call that hands the first call's metadata back."""
    import hip_attn.v1_2.paged_hip as paged
    from hip_attn.v1_2.hip_config import HiPAttentionConfig

    g = torch.Generator().manual_seed(seed)
    short = lambda t: t.to(torch.bfloat16).float()  # noqa: E731
    q = short(torch.randn((B, TQ, H, D), generator=g) * 0.5)
    k = short(torch.randn((B, TK, HKV, D), generator=g))
    v = short(torch.randn((B, TK, HKV, D), generator=g))
    lens_t = torch.tensor(lens, dtype=torch.int64)
    pos = (lens_t[:, None] - TQ + torch.arange(TQ)[None, :]).contiguous()
    slots = (torch.randperm(B * TK + 7, generator=g)[: B * TK] + 1).reshape(B, TK)
    kc = torch.zeros((B * TK + 8, HKV, D))
    vc = torch.zeros_like(kc)
    for b in range(B):
        kc[slots[b]] = k[b]
        vc[slots[b]] = v[b]
    req_to_tokens = torch.zeros((B + 3, TK), dtype=torch.int32)
    pool_idx = torch.tensor([2, 0, 4][:B])
    req_to_tokens[pool_idx] = slots.to(torch.int32)
    cfg = HiPAttentionConfig(json_or_path=spec)
    cos = sin = None
    out = {}
    if rope:
        cos, sin = rope_tables(2 * TK, D)
        cos, sin = short(cos), short(sin)
        out.update(rope_cos=bits16(cos), rope_sin=bits16(sin))
    decode = TQ == 1
    for layer_id in layer_ids:
        kw = dict(sm_scale=D ** -0.5, batch_size=B, k_cache=kc, v_cache=vc, offload_cache=None,
                  positions=pos.reshape(-1), seq_lens=lens_t, req_to_tokens=req_to_tokens, req_pool_indices=pool_idx,
                  rope_cos=cos, rope_sin=sin, layer_id=layer_id, logit_cap=0.0, orig_context_len=orig_context_len,
                  max_context_len=TK, is_prefill=not decode, hip_config=cfg, is_decode=decode)
        o, md = paged.forward_paged_hip(q.reshape(B * TQ, H, D), **kw)
        out[f"o_{layer_id}"] = o.float().numpy()
        out[f"indices_{layer_id}"] = md.indices.numpy()
        out[f"ks_{layer_id}"] = md.ks.numpy()
        out.update(access_flags(md, f"_{layer_id}"))
        if decode:
            o2, _ = paged.forward_paged_hip(q.reshape(B * TQ, H, D), cached_metadata=md, **kw)
            out[f"o_cached_{layer_id}"] = o2.float().numpy()
    path = os.path.join(HERE, f"reference_{name}.npz")
    np.savez_compressed(path, q=bits16(q), k_cache=bits16(kc), v_cache=bits16(vc), positions=pos.numpy(),
                        seq_lens=lens_t.numpy(), req_to_tokens=req_to_tokens.numpy(), req_pool_indices=pool_idx.numpy(),
                        spec=np.frombuffer(spec.encode(), dtype=np.uint8), layer_ids=np.array(layer_ids),
                        orig_context_len=orig_context_len, max_context_len=TK, TQ=TQ, **out)
    print("wrote", path, flush=True)


def make_pool_layout_case(name, spec, heads, layers, context_length):
    """Buffer names, shapes, formats and dtypes of ``HiPMetadataCachePool`` (hip_memory_pool.py:55-222)."""
    import json

    from hip_attn.v1_2.hip_config import HiPAttentionConfig
    from hip_attn.v1_2.hip_memory_pool import HiPMetadataCachePool

    cfg = HiPAttentionConfig(json_or_path=spec)
    pool = HiPMetadataCachePool(max_total_num_tokens=1 << 20, query_head_num=heads, layer_num=layers,
                                context_length=context_length, device="cpu", hip_config=cfg)
    layout = [{n: dict(shape=list(b.buffer.shape), store=str(b.buffer.dtype), dtype=str(b.dtype), format=b.batch_format)
               for n, b in layer.items()} for layer in pool.cache]
    path = os.path.join(HERE, f"reference_{name}.json")
    with open(path, "w") as f:
        json.dump(dict(spec=spec, heads=heads, layers=layers, context_length=context_length, layout=layout,
                       allocated_bytes=int(pool.allocated_gpu_bytes)), f, indent=1)
    print("wrote", path, flush=True)


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    only = sys.argv[2:] or None
    ext, meta = load_reference(root)
    tiny = [(32, 2, 64, None, 1), (32, 2, 16, 2048, 1), (32, 1, 2, 1024, 1)]
    strided = [(64, 4, 64, None, 2), (32, 2, 16, 1024, 1), (32, 1, 4, 512, 1)]
    default = [(64, 4, 256, None, 1), (64, 4, 32, 32768, 1), (64, 1, 8, 8192, 1)]
    cases = {
        # name: (seed, B, TQ, TK, H, HKV, D, stages, sink, sw, second_k, bsbq, extras)
        "f32_prefill_tiny": (0, 1, 64, 1024, 2, 1, 32, tiny, 16, 256, 512, 32, dict(replay=True)),
        "f32_prefill_gqa_ragged": (1, 2, 80, 1536, 4, 2, 32, tiny, 16, 256, 512, 32, {}),
        "f32_decode_paged": (2, 2, 1, 2048, 4, 2, 32, tiny, 16, 256, 512, 32, dict(lens=[2048, 1500], page_size=8, replay=True)),
        "f32_prefill_rope_relative": (3, 1, 64, 1024, 2, 1, 32, tiny, 16, 256, 512, 32, dict(extend=("relative", "streaming"))),
        "f32_prefill_rope_streaming": (4, 1, 64, 1024, 2, 1, 32, tiny, 16, 256, 512, 32, dict(extend=("streaming", "streaming"))),
        "f32_decode_rope_infllm": (5, 2, 1, 1536, 4, 2, 32, tiny, 16, 256, 512, 32,
                                   dict(lens=[1536, 1100], extend=("infllm", "infllm"))),
        # the smallest benchmark configuration: 512 queries against 4096 keys, 4 heads over 1, head dim 64, float32
        "f32_smallest_benchmark_prefill": (0, 1, 512, 4096, 4, 1, 64, tiny, 16, 256, 512, 32, dict(exact=True)),
        "f32_prefill_stride_d64": (8, 1, 128, 2048, 4, 2, 64, strided, 32, 128, 256, 32, {}),
        "f32_decode_default_stages": (9, 1, 1, 8192, 2, 1, 32, default, 256, 512, 2048, 64, {}),
        # dynamic_extend in the scan: the context reaches beyond the model's, so old keys are squeezed into it
        "f32_prefill_rope_dynamic": (10, 1, 64, 2048, 2, 1, 32, tiny, 16, 256, 512, 32,
                                     dict(extend=("dynamic_extend", "streaming"), model_ctx=1024)),
        "f32_decode_rope_dynamic": (11, 2, 1, 2048, 4, 2, 32, tiny, 16, 256, 512, 32,
                                    dict(lens=[2048, 1500], page_size=8, extend=("dynamic_extend", "infllm"), model_ctx=512)),
        # dynamic_extend inside block sparse attention: cos / sin of the squeezed position blended with the streaming ones
        "f32_prefill_sa_rope_dynamic": (12, 1, 96, 2048, 4, 2, 32, tiny, 16, 256, 512, 32,
                                        dict(extend=("relative", "dynamic_extend"), model_ctx=1024)),
        "f32_decode_sa_rope_dynamic": (13, 2, 1, 2048, 4, 2, 32, tiny, 16, 256, 512, 32,
                                       dict(lens=[2048, 1400], page_size=4, extend=("streaming", "dynamic_extend"), model_ctx=512)),
        # self_extend in the scan: keys older than 8192 positions are grouped by sixteen once the block reaches beyond
        # the model's context (the quotient of the negative distance is truncated toward zero, by the interpreter too)
        # (one case, and tables just long enough: 9216 keys make this the largest vector)
        "f32_prefill_rope_self_extend": (16, 1, 64, 9216, 2, 1, 32, tiny, 16, 256, 512, 32,
                                         dict(extend=("self_extend", "streaming"), model_ctx=4096, rope_len=9216 + 64)),
        # is_causal=False: the attention kernels drop the key <= query test (the scan is not told)
        "f32_prefill_non_causal": (14, 2, 96, 1536, 4, 2, 32, tiny, 16, 256, 512, 32, dict(causal=False)),
        "f32_decode_non_causal": (15, 2, 1, 2048, 4, 2, 32, tiny, 16, 256, 512, 32,
                                  dict(lens=[2048, 1300], page_size=8, causal=False)),
        # Not generated: Triton's interpreter has no bfloat16 constants (``get_bf16``) and cannot call
        # ``libdevice.tanh`` (logit_softcap) outside a compiled kernel, so bfloat16 inputs and soft-capped logits
        # have no vectors from the reference.
    }
    for sd in SWEEP_SEEDS:
        cases[f"f32_sweep_{sd}"] = sweep_case(sd)
    for name, (seed, B, TQ, TK, H, HKV, D, stages, sink, sw, second_k, bsbq, extra) in cases.items():
        if only and name not in only:
            continue
        make_case(ext, meta, name, seed, B, TQ, TK, H, HKV, D, stages, sink, sw, second_k, bsbq, **extra)
    layers = ('"dense_layers": [0], "layers": [{"second_stage_k": 256, "sliding_window_size": 256}, '
              '{"second_stage_k": 128, "sliding_window_size": 256}], "prefill_layers": [{"second_stage_k": 256, '
              '"sliding_window_size": 256}, {"second_stage_k": 128, "sliding_window_size": 256}]')
    api_cases = {
        # name: (seed, B, TQ, TK, H, HKV, D, lens, config, layer ids, orig_context_len, rope tables)
        "f32_paged_api_prefill": (20, 1, 192, 2048, 4, 2, 32, [2048], '{"using_extend": false, %s}' % layers, [7], 4096, False),
        "f32_paged_api_decode_rope": (21, 2, 1, 3072, 4, 2, 32, [3072, 2000], "{%s}" % layers, [0, 5], 131072, True),
    }
    layers2 = ('"dense_layers": [0, 3], "layers": [{"second_stage_k": 256, "sliding_window_size": 256, '
               '"sink_token_size": 64}, {"second_stage_k": 128, "sliding_window_size": 128}], "prefill_layers": '
               '[{"second_stage_k": 256, "sliding_window_size": 256}, {"second_stage_k": 128, '
               '"sliding_window_size": 512, "sink_token_size": 32}]')
    api_cases.update({
        # two sequences of different lengths, 100 new tokens each (one call per layer), per-layer sink sizes
        "f32_paged_api_prefill_ragged": (30, 2, 100, 2048, 4, 2, 32, [2048, 1500],
                                         '{"using_extend": false, %s}' % layers2, [3, 2], 8192, False),
        # 130 new tokens with RoPE on load: the last 64 go through the second call
        "f32_paged_api_prefill_rope_split": (33, 1, 130, 2048, 4, 1, 64, [1700], "{%s}" % layers2, [5], 2048, True),
    })
    for name, spec in api_cases.items():
        if only and name not in only:
            continue
        make_paged_api_case(name, *spec)
    if not only or "metadata_pool_layout" in only:
        make_pool_layout_case("metadata_pool_layout", '{"metadata_cache_max_batch_size": 6, %s}' % layers, 8, 3, 32768)


if __name__ == "__main__":
    main()
