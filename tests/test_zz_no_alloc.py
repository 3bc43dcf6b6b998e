"""``hipattn_bsa_decode_static``: decode attention with its split partials in a device array inside the library.

The entry point exists for callers that cannot allocate device memory around the call (HIP graph capture, tight
serving loops).  It runs the kernels of ``hipattn_bsa_decode_partial`` + ``hipattn_bsa_decode_merge``, so its output
must equal theirs bit for bit; two calls in a row, the second on a smaller problem, share the array, and nothing of the
first may leak into the second.  Everything goes through the C ABI.
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import hip12 as O
from helpers import make_inputs, to_paged
from gpu_utils import assert_context_close, to_torch

pytestmark = pytest.mark.gpu


def _problem(seed, B, lens, TK, H, HKV, D, page):
    from hip_attn import _native as N

    lens = np.asarray(lens)
    X = make_inputs(seed, B=B, TQ=1, TK=TK, H=H, HKV=HKV, D=D, dtype="bf16", pos=(lens - 1)[:, None])
    XP = to_paged(X, page, seed=seed + 1, seq_lens=lens)
    A = O.OArgs(sliding_window_size=512, second_stage_k=1024, extend_context_length=TK)
    octx, ometa = O.hip_attention_12(XP, A)
    q = to_torch(X.q, "bf16")
    kc, vc = to_torch(XP.k_cache, "bf16"), to_torch(XP.v_cache, "bf16")
    bt = torch.from_numpy(XP.block_table).cuda()
    sl = torch.from_numpy(XP.cache_seq_lens).cuda()
    pos = torch.from_numpy(np.ascontiguousarray(XP.pos)).cuda()
    indices = torch.from_numpy(ometa.indices).cuda()
    kse = torch.from_numpy(ometa.ks_start_end).cuda()
    keep = (q, kc, vc, bt, sl, pos, indices, kse)
    qs = N.make_q(q, pos)
    kvs = N.make_kv_paged(kc, vc, bt, sl, TK)
    return dict(qs=qs, kvs=kvs, indices=indices, kse=kse, BK=indices.shape[-1], octx=octx, keep=keep, shape=q.shape, A=A)


def _run_both(P, nsplits):
    from hip_attn import _native as N

    dev = torch.device("cuda", torch.cuda.current_device())
    A = P["A"]
    want = torch.empty(P["shape"], dtype=torch.bfloat16, device=dev)
    N.bsa_decode(P["qs"], P["kvs"], P["indices"], P["kse"], P["BK"], 8, 512, A.sink_token_size, want, dev,
                 nsplits=nsplits, second_stage_k=A.second_stage_k)
    got = torch.full(P["shape"], float("nan"), dtype=torch.bfloat16, device=dev)
    N.bsa_decode_static(P["qs"], P["kvs"], P["indices"], P["kse"], P["BK"], 8, 512, A.sink_token_size, got, dev,
                        nsplits=nsplits, second_stage_k=A.second_stage_k)
    torch.cuda.synchronize()
    return got, want


def test_static_scratch_decode_equals_the_workspace_decode_on_two_calls_in_a_row():
    print("[case] decode without allocation: large call, then a smaller one", flush=True)
    big = _problem(301, B=4, lens=[8192, 5000, 7777, 6100], TK=8192, H=16, HKV=4, D=128, page=16)
    small = _problem(303, B=1, lens=[3000], TK=4096, H=8, HKV=2, D=128, page=16)
    for name, P, nsplits in (("large", big, 0), ("small", small, 0), ("large again, 7 splits", big, 7),
                             ("small, 3 splits", small, 3)):
        print(f"  {name}", flush=True)
        got, want = _run_both(P, nsplits)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"{name}: output differs from the workspace path"
        assert_context_close(got, P["octx"], "bf16")


def test_static_scratch_decode_refuses_what_does_not_fit():
    from hip_attn import _native as N

    print("[case] decode without allocation: size limit", flush=True)
    P = _problem(305, B=1, lens=[3000], TK=4096, H=8, HKV=2, D=128, page=16)
    dev = torch.device("cuda", torch.cuda.current_device())
    out = torch.empty(P["shape"], dtype=torch.bfloat16, device=dev)
    limit = 4 * 1024 * 1024
    too_many = limit // (8 * (128 + 4) * 4) + 1  # splits whose partials no longer fit
    assert too_many <= 1024
    with pytest.raises(N.HipAttnError, match="scratch"):
        N.bsa_decode_static(P["qs"], P["kvs"], P["indices"], P["kse"], P["BK"], 8, 512, 256, out, dev, nsplits=too_many)
    torch.cuda.synchronize()


def test_static_scratch_decode_under_graph_capture_allocates_nothing():
    """What the entry point is for: after one eager call (which looks the array's address up) it is captured into a
    HIP graph and replayed with new queries; device memory does not move across the calls."""
    from hip_attn import _native as N

    print("[case] decode without allocation: captured into a graph, replayed with new queries", flush=True)
    P = _problem(307, B=2, lens=[4096, 3500], TK=4096, H=8, HKV=2, D=128, page=16)
    dev = torch.device("cuda", torch.cuda.current_device())
    A = P["A"]
    q = P["keep"][0]
    out = torch.empty(P["shape"], dtype=torch.bfloat16, device=dev)
    want = torch.empty_like(out)

    def static_call():
        N.bsa_decode_static(P["qs"], P["kvs"], P["indices"], P["kse"], P["BK"], 8, 512, A.sink_token_size, out, dev,
                            nsplits=0, second_stage_k=A.second_stage_k)

    static_call()  # eager: address lookup, code objects loaded
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    torch_before = torch.cuda.memory_allocated()
    static_call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the device's free memory"
    assert torch.cuda.memory_allocated() == torch_before

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        static_call()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_call()
    g = torch.Generator().manual_seed(11)
    for rep in range(3):
        q.copy_(torch.randn(q.shape, generator=g).to(torch.bfloat16))
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        N.bsa_decode(P["qs"], P["kvs"], P["indices"], P["kse"], P["BK"], 8, 512, A.sink_token_size, want, dev,
                     nsplits=0, second_stage_k=A.second_stage_k)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), f"replay {rep} differs from the workspace path"
