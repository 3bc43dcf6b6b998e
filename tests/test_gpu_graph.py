"""A decode step captured in a HIP graph replays to the eager result.

The reference operator must be capturable when ``position_ids`` is given
(``src/hip_attn/v1_2/attention_extend.py:1980-1982``); serving stacks replay the decode step from a graph.
Each graph is replayed several times with eager work and synchronisation in between, on fresh inputs copied
into the captured buffers, and every replay is compared with an eager call on the same inputs.
"""
import numpy as np
import pytest
import torch

from helpers import make_inputs, to_paged
from gpu_utils import to_torch

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16)


@pytest.mark.parametrize("refresh", [False, True])
def test_decode_step_replays_from_a_graph(refresh):
    from hip_attn import HiPAttentionArgs12, hip_attention_12

    print(f"[case] graph replay refresh={refresh}", flush=True)
    B, TK, H, HKV, D = 2, 4096, 8, 2, 128
    lens = np.array([4096, 3000])
    X = make_inputs(90, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", pos=(lens - 1)[:, None])
    XP = to_paged(X, 16, seed=3, seq_lens=lens)
    kc, vc = to_torch(XP.k_cache, "bf16"), to_torch(XP.v_cache, "bf16")
    bt = torch.from_numpy(XP.block_table).cuda()
    sl = torch.from_numpy(XP.cache_seq_lens).cuda()
    pos = torch.from_numpy(np.ascontiguousarray(XP.pos)).cuda()

    def make_args():
        return HiPAttentionArgs12(sliding_window_size=512, second_stage_k=1024, k_cache=kc, v_cache=vc, block_table=bt,
                                  cache_seq_lens=sl, position_ids=pos, extend_context_length=TK,
                                  require_cache_statistics=False)

    g = torch.Generator().manual_seed(7)
    queries = [torch.randn((B, 1, H, D), generator=g).to(torch.bfloat16).cuda() for _ in range(4)]
    q_static = queries[0].clone()
    _, meta0 = hip_attention_12(q_static, None, None, make_args())
    cached = None if refresh else meta0

    # warm up on a side stream, then capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            hip_attention_12(q_static, None, None, make_args(), cached_metadata=cached)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static, meta_static = hip_attention_12(q_static, None, None, make_args(), cached_metadata=cached)
    torch.cuda.synchronize()

    for it, qn in enumerate(queries):
        eager, meta_e = hip_attention_12(qn, None, None, make_args(), cached_metadata=cached)  # eager work in between
        torch.cuda.synchronize()
        q_static.copy_(qn)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(_bits(out_static), _bits(eager)), f"replay {it} differs from the eager step"
        if refresh:
            assert torch.equal(meta_static.indices, meta_e.indices), f"replay {it}: indices differ"
            assert torch.equal(meta_static.ks, meta_e.ks)


def test_graph_survives_many_other_shapes():
    """A captured refresh step reads the cached stage-0 chunk list; calls with more than sixteen other shapes after
    the capture must not free it (the list was handed out during the capture and is therefore kept for good)."""
    from hip_attn import HiPAttentionArgs12, hip_attention_12

    print("[case] graph replay after many other shapes", flush=True)
    B, TK, H, HKV, D = 1, 4096, 8, 2, 128
    X = make_inputs(91, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", pos=np.array([[TK - 1]]))
    XP = to_paged(X, 16, seed=4, seq_lens=np.array([TK]))
    kc, vc = to_torch(XP.k_cache, "bf16"), to_torch(XP.v_cache, "bf16")
    bt = torch.from_numpy(XP.block_table).cuda()
    sl = torch.from_numpy(XP.cache_seq_lens).cuda()
    pos = torch.from_numpy(np.ascontiguousarray(XP.pos)).cuda()

    def make_args(sink=256):
        return HiPAttentionArgs12(sliding_window_size=512, second_stage_k=1024, sink_token_size=sink, k_cache=kc,
                                  v_cache=vc, block_table=bt, cache_seq_lens=sl, position_ids=pos,
                                  extend_context_length=TK, require_cache_statistics=False)

    q_static = to_torch(X.q, "bf16")
    hip_attention_12(q_static, None, None, make_args())  # warm-up: builds and keeps the chunk list
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static, meta_static = hip_attention_12(q_static, None, None, make_args())
    torch.cuda.synchronize()
    eager, meta_e = hip_attention_12(q_static, None, None, make_args())
    for sink in range(16, 16 + 16 * 24, 16):  # 24 other stage-0 lists
        hip_attention_12(q_static, None, None, make_args(sink))
    junk = [torch.full((n,), 0x7FFFFFF, dtype=torch.int32, device="cuda") for n in (4, 8, 16, 32, 64) for _ in range(8)]
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    del junk
    assert torch.equal(meta_static.indices, meta_e.indices)
    assert torch.equal(_bits(out_static), _bits(eager))
