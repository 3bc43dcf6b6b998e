"""Offload cache on the GPU: results equal the resident run bit for bit, replacement equals a textbook LRU.

The reference validates its offload path by comparing against a resident run (``src/hip_attn/v1_2/paged_hip.py:
161-194``, squared error below 1e-7); here the same kernels read the same bytes, so equality is exact.
"""
import numpy as np
import pytest
import torch

from oracle import hip12 as O
from helpers import make_inputs, to_paged
from gpu_utils import assert_context_close, assert_metadata_equal, to_torch

pytestmark = pytest.mark.gpu


# ---------------------------------------------------------------------------------------------------------
# replacement policy against a model, driven directly on the cache's device arrays
# ---------------------------------------------------------------------------------------------------------
class LruModel:
    """Exact LRU by step: victims are the slots with the smallest (last-use step, slot id)."""

    def __init__(self, slots, max_fetch):
        self.slots, self.max_fetch = slots, max_fetch
        self.last_use = [-1] * slots
        self.backref = [-1] * slots
        self.where = {}
        self.step = 0

    def run_step(self, accessed):
        hits = [e for e in accessed if e in self.where]
        for e in hits:
            self.last_use[self.where[e]] = self.step
        misses = sorted(e for e in accessed if e not in self.where)
        used_now = len(set(self.where[e] for e in hits))
        m = min(len(misses), self.max_fetch, self.slots - used_now)
        victims = sorted(sorted(range(self.slots), key=lambda s: (self.last_use[s], s))[:m])
        evicted = 0
        for e, s in zip(misses[:m], victims):
            if self.backref[s] >= 0:
                del self.where[self.backref[s]]
                evicted += 1
            self.backref[s] = e
            self.where[e] = s
            self.last_use[s] = self.step
        self.step += 1
        return used_now, len(misses), m, evicted


@pytest.mark.parametrize("slots,max_fetch,blocks,heads,seed", [(8, 5, 20, 2, 0), (50, 64, 300, 3, 1), (5000, 300, 9000, 2, 2)])
def test_cache_replacement_matches_lru_model(slots, max_fetch, blocks, heads, seed):
    from hip_attn.offload import GPUCache, UVMCache

    print(f"[case] lru model slots={slots} max_fetch={max_fetch} blocks={blocks} heads={heads}", flush=True)
    dev = torch.device("cuda")
    bt, D = 4, 32
    rows = blocks * bt - 1  # last block is partial
    pool = UVMCache(0, rows, heads, D, torch.bfloat16, dev)
    g = torch.Generator().manual_seed(seed)
    pool.bank_cpu.copy_(torch.randn(pool.bank_cpu.shape, generator=g).to(torch.bfloat16))
    cache = GPUCache(pool, None, slots * bt, block_tokens=bt, max_fetch=max_fetch)
    assert cache.slots == slots and cache.n_blocks == blocks
    model = LruModel(slots, max_fetch)
    rng = np.random.default_rng(seed)
    entries = heads * blocks
    hot = rng.permutation(entries)[: max(2, slots // 2)]
    for step in range(24):
        # a hot set that mostly stays plus a drifting cold tail, as attention over a growing context does
        n_hot = rng.integers(1, len(hot) + 1)
        n_cold = rng.integers(0, max(2, slots // 3))
        accessed = sorted(set(rng.choice(hot, n_hot, replace=False).tolist()) |
                          set(rng.integers(0, entries, n_cold).tolist()))
        # what the reading kernels do: stamp resident blocks with the step, flag the others
        acc = torch.tensor(accessed, dtype=torch.int64, device=dev)
        slot_of = cache.table.view(-1)[acc]
        res = slot_of >= 0
        cache.last_use[slot_of[res].long()] = step
        cache.miss.view(-1)[acc[~res]] = 1
        cache.handle_cache_miss()
        exp = model.run_step(accessed)
        st = cache.statistics()
        assert (st["last_hit"], st["last_missed"], st["last_fetched"]) == exp[:3], (step, st, exp)
        table = cache.table.view(-1).cpu().numpy()
        want = np.full(entries, -1, dtype=np.int32)
        for e, s in model.where.items():
            want[e] = s
        assert np.array_equal(table, want), f"step {step}: table differs from the LRU model"
        assert np.array_equal(cache.backref.cpu().numpy(), np.array(model.backref, dtype=np.int32))
        assert np.array_equal(cache.last_use.cpu().numpy(), np.array(model.last_use, dtype=np.int32))
        assert int(cache.miss.sum()) == 0
    # bank content: every resident block holds the pool rows it stands for (zero beyond the pool)
    bank = cache.bank.view(slots, bt, D).cpu()
    host = torch.zeros((blocks * bt, heads, D), dtype=torch.bfloat16)
    host[:rows] = pool.bank_cpu
    for e, s in list(model.where.items())[:200]:
        h, blk = divmod(e, blocks)
        assert torch.equal(bank[s].view(torch.int16), host[blk * bt:(blk + 1) * bt, h].view(torch.int16)), (e, s)
    assert st["steps"] == 24


# ---------------------------------------------------------------------------------------------------------
# the operator over an offloaded pool
# ---------------------------------------------------------------------------------------------------------
def _offloaded_case(seed, B, TK, H, HKV, D, lens, TQ):
    pos = np.stack([np.arange(TQ) + l - TQ for l in lens])
    X = make_inputs(seed, B=B, TQ=TQ, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", pos=pos)
    XP = to_paged(X, 1, seed=seed + 1, seq_lens=lens)
    return X, XP


def _args(XP, A, **kw):
    from hip_attn import HiPAttentionArgs12, ScanStage12

    return HiPAttentionArgs12(
        sink_token_size=A.sink_token_size, sliding_window_size=A.sliding_window_size, block_size_k=A.block_size_k,
        second_stage_k=A.second_stage_k,
        stages=[ScanStage12(stage_block_size_q=s.stage_block_size_q, stage_block_stride_q=s.stage_block_stride_q,
                            stage_chunk_size=s.stage_chunk_size, stage_k=s.stage_k, stage_stride=s.stage_stride)
                for s in A.stages],
        extend_context_length=A.extend_context_length, block_sparse_block_size_q=A.block_sparse_block_size_q,
        position_ids=torch.from_numpy(np.ascontiguousarray(XP.pos)).cuda(),
        block_table=torch.from_numpy(XP.block_table).cuda(), cache_seq_lens=torch.from_numpy(XP.cache_seq_lens).cuda(),
        **kw)


def _fill(cache, XP):
    rows = XP.k_cache.shape[0]
    table = torch.arange(rows, dtype=torch.int64)
    k = to_torch(XP.k_cache[:, 0], "bf16", "cpu")
    v = to_torch(XP.v_cache[:, 0], "bf16", "cpu")
    cache.set_kv_buffer(table, table.cuda(), k, v)


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16)


@pytest.mark.parametrize("TQ,sa_tokens", [(1, 1 << 20), (64, 1 << 20), (1, 1024)])
def test_offloaded_equals_resident_and_oracle(TQ, sa_tokens):
    from hip_attn import HiPOffloadCache, hip_attention_12

    print(f"[case] offload TQ={TQ} sa_tokens={sa_tokens}", flush=True)
    B, TK, H, HKV, D = 2, 2048, 8, 2, 128
    lens = np.array([2048, 1500])
    X, XP = _offloaded_case(40 + TQ, B, TK, H, HKV, D, lens, TQ)
    A = O.OArgs(sliding_window_size=256, second_stage_k=512, extend_context_length=TK,
                stages=[O.OStage(64, 4, 64, None, 1), O.OStage(64, 4, 16, 1024, 1), O.OStage(64, 1, 8, 512, 1)])
    octx, ometa = O.hip_attention_12(XP, A)

    rows = XP.k_cache.shape[0]
    cache = HiPOffloadCache(0, rows, 1 << 20, sa_tokens, HKV, D, torch.bfloat16, torch.device("cuda"))
    _fill(cache, XP)
    q = to_torch(X.q, "bf16")
    res_args = _args(XP, A, k_cache=to_torch(XP.k_cache, "bf16"), v_cache=to_torch(XP.v_cache, "bf16"))
    ctx_res, meta_res = hip_attention_12(q, None, None, res_args)
    assert_metadata_equal(meta_res, ometa)

    seen_hit = False
    for step in range(3):
        off_args = _args(XP, A, offload_cache=cache)
        ctx, meta = hip_attention_12(q, None, None, off_args)
        torch.cuda.synchronize()
        assert_metadata_equal(meta, ometa)
        assert torch.equal(_bits(ctx), _bits(ctx_res)), f"step {step}: offloaded context differs from the resident one"
        assert_context_close(ctx, octx, "bf16")
        # statistics: flags are 0/1, misses are accesses, a cold cache misses everything it touches
        for st in (meta.mask_cache_statistics, meta.sa_cache_statistics):
            a, m = st.access_counter, st.cache_miss_counter
            assert a.shape == (B, HKV, rows) and int(a.max()) == 1 and int(a.min()) == 0
            assert bool(((m == 1) <= (a == 1)).all())
            if step == 0:
                assert torch.equal(a, m)
        cache.handle_cache_miss(meta)
        sm, ss = cache.mask_k_cache.statistics(), cache.sa_kv_cache.statistics()
        if step == 0:
            assert sm["last_hit"] == 0 and ss["last_hit"] == 0 and sm["last_missed"] > 0 and ss["last_missed"] > 0
        else:
            seen_hit = seen_hit or (sm["last_hit"] > 0 and ss["last_hit"] > 0)
        if step == 2 and sa_tokens >= (1 << 20):
            assert sm["last_missed"] == 0 and ss["last_missed"] == 0, (sm, ss)
    assert seen_hit
    if sa_tokens < (1 << 20):
        # the working set does not fit: blocks used in a step are never evicted in that step, so misses persist
        assert cache.sa_kv_cache.statistics()["last_missed"] > 0


def test_offload_write_through_and_side_stream():
    from hip_attn import HiPOffloadCache, hip_attention_12

    print("[case] offload write-through", flush=True)
    B, TK, H, HKV, D, TQ = 1, 1536, 4, 1, 64, 1
    lens = np.array([1536])
    X, XP = _offloaded_case(77, B, TK, H, HKV, D, lens, TQ)
    A = O.OArgs(sliding_window_size=128, second_stage_k=256, extend_context_length=TK, sink_token_size=32,
                stages=[O.OStage(64, 4, 64, None, 1), O.OStage(64, 4, 16, 512, 1), O.OStage(64, 1, 8, 256, 1)])
    rows = XP.k_cache.shape[0]
    cache = HiPOffloadCache(0, rows, 1 << 18, 1 << 18, HKV, D, torch.bfloat16, torch.device("cuda"))
    # the side stream comes from the probe that looks for a hardware queue of its own; whether it finds one depends
    # on how many streams the process already has, the results do not
    assert isinstance(cache.enable_miss_stream(), bool) and cache.miss_stream is not None
    assert cache.miss_stream != torch.cuda.current_stream()
    _fill(cache, XP)
    q = to_torch(X.q, "bf16")
    for _ in range(2):  # warm both caches, fetching on the side stream
        _, meta = hip_attention_12(q, None, None, _args(XP, A, offload_cache=cache))
        cache.handle_cache_miss(meta)
    # overwrite a stretch of tokens that is resident by now (the sliding window) from the device side
    t0 = int(lens[0]) - 40
    rows_new = torch.from_numpy(XP.block_table[0, t0:t0 + 24]).cuda()
    g = torch.Generator().manual_seed(5)
    k_new = torch.randn((24, HKV, D), generator=g).to(torch.bfloat16).cuda()
    v_new = torch.randn((24, HKV, D), generator=g).to(torch.bfloat16).cuda()
    cache.set_kv_buffer(rows_new, rows_new, k_new, v_new)
    torch.cuda.synchronize()
    assert torch.equal(cache.k_uvm.bank_cpu[rows_new.cpu()].view(torch.int16), k_new.cpu().view(torch.int16))
    kc = to_torch(XP.k_cache, "bf16")
    vc = to_torch(XP.v_cache, "bf16")
    kc[rows_new, 0] = k_new
    vc[rows_new, 0] = v_new
    ctx_res, meta_res = hip_attention_12(q, None, None, _args(XP, A, k_cache=kc, v_cache=vc))
    ctx, meta = hip_attention_12(q, None, None, _args(XP, A, offload_cache=cache))
    torch.cuda.synchronize()
    assert torch.equal(meta.indices, meta_res.indices)
    assert torch.equal(_bits(ctx), _bits(ctx_res))
    cache.flush()
    ctx2, meta2 = hip_attention_12(q, None, None, _args(XP, A, offload_cache=cache))
    assert torch.equal(_bits(ctx2), _bits(ctx_res))
    assert torch.equal(meta2.sa_cache_statistics.cache_miss_counter, meta2.sa_cache_statistics.access_counter)


def test_model_level_manager_prefetches_prefixes_and_orders_async_stores():
    """HiPModelOffloadCache: per-layer pools, stores on a side stream, the next layer's prefix gathered by the device
    from the pinned pool while the current layer runs (model_offload_cache.py:229-452)."""
    from hip_attn import HiPAttentionArgs12, HiPAttentionConfig, HiPModelOffloadCache, hip_attention_12

    print("[case] model-level offload manager", flush=True)
    dev = torch.device("cuda", 0)
    L, HKV, H, D, T = 3, 2, 4, 64, 4096
    cfg = HiPAttentionConfig()
    mgr = HiPModelOffloadCache(max_token_size=T + 64, max_mask_cache_token_size=2048, max_sa_cache_token_size=2048,
                               dtype=torch.bfloat16, head_num=HKV, head_dim=D, layer_num=L, device=dev, hip_config=cfg)
    host, gpu = mgr._calc_allocated_bytes()
    assert host == L * 2 * (T + 65) * HKV * D * 2 and gpu > 0
    g = torch.Generator().manual_seed(5)
    perm = (torch.randperm(T + 60, generator=g)[:T] + 1).to(dev)  # pool rows of the sequence, row 0 left alone
    ks = [torch.randn((T, HKV, D), generator=g).to(torch.bfloat16).to(dev) for _ in range(L)]
    vs = [torch.randn((T, HKV, D), generator=g).to(torch.bfloat16).to(dev) for _ in range(L)]
    prefix, fresh = 3072, 1024
    for layer in range(L):  # the prefix was stored by earlier chunks; one layer asynchronously
        mgr.set_kv_buffer(layer, perm[:prefix], ks[layer][:prefix], vs[layer][:prefix], async_copy=(layer == 1))
    req_to_token = torch.zeros((2, T), dtype=torch.int64, device=dev)
    req_to_token[1] = perm
    pool_idx = torch.tensor([1], device=dev)
    hooks = dict(batch_size=1, req_to_token=req_to_token, req_pool_indices=pool_idx,
                 extend_prefix_lens_cpu=np.array([prefix]), extend_seq_lens_cpu=np.array([fresh]))
    mgr.on_model_start(True, **hooks)
    for layer in range(L):
        mgr.on_layer_start(layer, True, **hooks)
        new_k, new_v = ks[layer][None, prefix:], vs[layer][None, prefix:]
        k, v, extra = mgr.get_fetched_prefix_kv_buffer(layer, 0, new_k, new_v)
        assert extra is None and k.shape == (1, T, HKV, D)
        assert torch.equal(k[0], ks[layer]) and torch.equal(v[0], vs[layer])
        mgr.set_kv_buffer(layer, perm[prefix:], new_k[0], new_v[0], async_copy=True)
        mgr.on_layer_end(layer, True)
    mgr.on_model_end(True)
    # decode against the offloaded layer 1 equals decode against the same rows held densely
    cache, _ = mgr.get_kv_buffer(1)
    q = torch.randn((1, 1, H, D), generator=g).to(torch.bfloat16).to(dev)
    common = dict(sliding_window_size=256, sink_token_size=16, second_stage_k=512,
                  position_ids=torch.tensor([[T - 1]], device=dev))
    from hip_attn import ScanStage12
    stages = [ScanStage12(stage_block_size_q=32, stage_block_stride_q=2, stage_chunk_size=64, stage_k=None, stage_stride=1),
              ScanStage12(stage_block_size_q=32, stage_block_stride_q=2, stage_chunk_size=16, stage_k=2048, stage_stride=1),
              ScanStage12(stage_block_size_q=32, stage_block_stride_q=1, stage_chunk_size=2, stage_k=1024, stage_stride=1)]
    off_args = HiPAttentionArgs12(offload_cache=cache, block_table=perm[None].contiguous(),
                                  cache_seq_lens=torch.tensor([T], device=dev), extend_context_length=T, stages=stages,
                                  **common)
    out_off, meta_off = hip_attention_12(q, None, None, off_args)
    out_res, meta_res = hip_attention_12(q, ks[1][None], vs[1][None], HiPAttentionArgs12(stages=stages, **common))
    assert torch.equal(meta_off.indices, meta_res.indices)
    assert torch.equal(out_off, out_res)


def test_model_level_manager_with_fp8_pools():
    """float8_e5m2 pools are held as bytes (model_offload_cache.py:39-41); stores round wider rows to e5m2 and the
    prefetched prefix comes back as float8_e5m2 with the new chunk's rows behind it."""
    from hip_attn import HiPAttentionConfig, HiPModelOffloadCache

    print("[case] model-level offload manager, fp8 pools", flush=True)
    dev = torch.device("cuda", 0)
    L, HKV, D, T = 2, 2, 64, 1024
    mgr = HiPModelOffloadCache(max_token_size=T + 8, max_mask_cache_token_size=512, max_sa_cache_token_size=512,
                               dtype=torch.float8_e5m2, head_num=HKV, head_dim=D, layer_num=L, device=dev,
                               hip_config=HiPAttentionConfig())
    assert mgr.store_dtype == torch.uint8 and mgr.layer_buffer[0].k_uvm.bank_cpu.dtype == torch.uint8
    g = torch.Generator().manual_seed(9)
    perm = (torch.randperm(T + 4, generator=g)[:T] + 1).to(dev)
    ks = [torch.randn((T, HKV, D), generator=g).to(torch.bfloat16).to(dev) for _ in range(L)]
    vs = [torch.randn((T, HKV, D), generator=g).to(torch.bfloat16).to(dev) for _ in range(L)]
    prefix, fresh = 768, 256
    for layer in range(L):
        mgr.set_kv_buffer(layer, perm[:prefix], ks[layer][:prefix], vs[layer][:prefix], async_copy=(layer == 1))
    req_to_token = torch.zeros((1, T), dtype=torch.int64, device=dev)
    req_to_token[0] = perm
    hooks = dict(batch_size=1, req_to_token=req_to_token, req_pool_indices=torch.tensor([0], device=dev),
                 extend_prefix_lens_cpu=np.array([prefix]), extend_seq_lens_cpu=np.array([fresh]))
    mgr.on_model_start(True, **hooks)
    for layer in range(L):
        mgr.on_layer_start(layer, True, **hooks)
        k, v, _ = mgr.get_fetched_prefix_kv_buffer(layer, 0, ks[layer][None, prefix:], vs[layer][None, prefix:])
        assert k.dtype == torch.float8_e5m2 and k.shape == (1, T, HKV, D)
        assert torch.equal(k[0].view(torch.uint8), ks[layer].to(torch.float8_e5m2).view(torch.uint8))
        assert torch.equal(v[0].view(torch.uint8), vs[layer].to(torch.float8_e5m2).view(torch.uint8))
        mgr.on_layer_end(layer, True)
    mgr.on_model_end(True)


def test_validation_pools_catch_a_corrupted_host_row(monkeypatch):
    """``HIP_OFFLOAD_CACHE_VALIDATION=1``: the manager keeps a resident copy of every layer, checks prefetched prefixes
    against it and hands it to ``forward_paged_hip(offloading_metadata=...)``, which repeats the call on the copy
    (model_offload_cache.py:117-128,211-226, paged_hip.py:95-320)."""
    from hip_attn import HiPAttentionConfig, HiPModelOffloadCache, forward_paged_hip

    print("[case] offload validation pools", flush=True)
    monkeypatch.setenv("HIP_OFFLOAD_CACHE_VALIDATION", "1")
    dev = torch.device("cuda", 0)
    L, HKV, H, D, T = 1, 2, 8, 64, 2048
    cfg = HiPAttentionConfig(json_or_path='{"using_extend": false, "layers": [{"second_stage_k": 256, '
                             '"sliding_window_size": 256}, {"second_stage_k": 256, "sliding_window_size": 256}]}')
    mgr = HiPModelOffloadCache(max_token_size=T + 8, max_mask_cache_token_size=T, max_sa_cache_token_size=T,
                               dtype=torch.bfloat16, head_num=HKV, head_dim=D, layer_num=L, device=dev, hip_config=cfg)
    assert mgr.require_validation
    g = torch.Generator().manual_seed(3)
    perm = (torch.randperm(T + 4, generator=g)[:T] + 1).to(dev)
    ks = torch.randn((T, HKV, D), generator=g).to(torch.bfloat16).to(dev)
    vs = torch.randn((T, HKV, D), generator=g).to(torch.bfloat16).to(dev)
    mgr.set_kv_buffer(0, perm, ks, vs)
    cache, valid = mgr.get_kv_buffer(0)
    assert torch.equal(valid[0][perm], ks) and torch.equal(valid[1][perm], vs)
    # the prefix check of a prefill pass
    req_to_token = perm[None].to(torch.int64).contiguous()
    hooks = dict(batch_size=1, req_to_token=req_to_token, req_pool_indices=torch.tensor([0], device=dev),
                 extend_prefix_lens_cpu=np.array([T - 128]), extend_seq_lens_cpu=np.array([128]))
    mgr.on_model_start(True, **hooks)
    k, v, extra = mgr.get_fetched_prefix_kv_buffer(0, 0, ks[None, T - 128:], vs[None, T - 128:])
    assert extra is not None and torch.equal(k[0], ks)
    mgr.on_model_end(True)
    # a decode step validated against the copy
    q = (torch.randn((1, H, D), generator=g) * 0.5).to(torch.bfloat16).to(dev)
    call = dict(sm_scale=D ** -0.5, batch_size=1, k_cache=None, v_cache=None, offload_cache=cache,
                positions=torch.tensor([T - 1], device=dev), seq_lens=torch.tensor([T], device=dev),
                req_to_tokens=req_to_token, req_pool_indices=torch.tensor([0], device=dev), rope_cos=None, rope_sin=None,
                layer_id=0, logit_cap=0.0, orig_context_len=131072, max_context_len=T, is_prefill=False, hip_config=cfg,
                is_decode=True)
    out, meta = forward_paged_hip(q, offloading_metadata=valid, **call)
    out_plain, _ = forward_paged_hip(q, **call)
    assert torch.equal(out, out_plain)
    # corrupt rows of the host pool inside the sliding window: the validated call must notice
    torch.cuda.synchronize()
    cache.k_uvm.bank_cpu[perm[T - 64:].cpu()] = 0
    cache.v_uvm.bank_cpu[perm[T - 64:].cpu()] = 0
    cache.mask_k_cache.flush()
    cache.sa_kv_cache.flush()
    with pytest.raises(AssertionError):
        forward_paged_hip(q, offloading_metadata=valid, **call)
