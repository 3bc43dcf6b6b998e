"""Helpers shared by the GPU parity tests: move oracle inputs to the device and call the product."""
import numpy as np
import torch

from oracle import hip12 as O


def to_torch(a, dtype, device="cuda"):
    if a is None:
        return None
    if dtype == "bf16":
        return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16).to(device)
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def from_torch(t, dtype):
    t = t.detach().cpu().contiguous()
    if dtype == "bf16":
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def product_args(A: O.OArgs, X: O.OInputs, device="cuda", **extra):
    from hip_attn import HiPAttentionArgs12, ScanStage12

    kw = dict(
        sink_token_size=A.sink_token_size, sliding_window_size=A.sliding_window_size,
        block_size_k=A.block_size_k, second_stage_k=A.second_stage_k,
        stages=[ScanStage12(stage_block_size_q=s.stage_block_size_q, stage_block_stride_q=s.stage_block_stride_q,
                            stage_chunk_size=s.stage_chunk_size, stage_k=s.stage_k, stage_stride=s.stage_stride,
                            stage_extend_backend=getattr(s, "stage_extend_backend", None))
                for s in A.stages],
        model_context_length=A.model_context_length, extend_context_length=A.extend_context_length,
        block_sparse_block_size_q=A.block_sparse_block_size_q, stage_early_terminate=A.stage_early_terminate,
        disable_flashdecode=A.disable_flashdecode, mask_only=A.mask_only, is_causal=A.is_causal,
        position_ids=torch.from_numpy(np.ascontiguousarray(X.pos)).to(device),
    )
    if X.k is None:
        kw.update(k_cache=to_torch(X.k_cache, X.dtype, device), v_cache=to_torch(X.v_cache, X.dtype, device),
                  block_table=torch.from_numpy(X.block_table).to(device),
                  cache_seq_lens=torch.from_numpy(X.cache_seq_lens).to(device))
    if getattr(A, "logit_softcap", None) is not None:
        kw.update(logit_softcap=A.logit_softcap)
    if A.using_extend:
        kw.update(using_extend=True, need_apply_rope=A.need_apply_rope, scan_extend_backend=A.scan_extend_backend,
                  sa_extend_backend=A.sa_extend_backend,
                  rope_cos=to_torch(O.f32_to_bf16_bits(X.rope_cos) if X.dtype == "bf16" else X.rope_cos, X.dtype, device),
                  rope_sin=to_torch(O.f32_to_bf16_bits(X.rope_sin) if X.dtype == "bf16" else X.rope_sin, X.dtype, device))
    kw.update(extra)
    return HiPAttentionArgs12(**kw)


def run_product(X: O.OInputs, A: O.OArgs, cached=None, device="cuda", **extra):
    from hip_attn import hip_attention_12

    q = to_torch(X.q, X.dtype, device)
    k = to_torch(X.k, X.dtype, device)
    v = to_torch(X.v, X.dtype, device)
    args = product_args(A, X, device, **extra)
    ctx, meta = hip_attention_12(q, k, v, args, cached_metadata=cached)
    torch.cuda.synchronize()
    return ctx, meta


def assert_metadata_equal(meta, ometa):
    assert meta.indices.dtype == torch.int64 and meta.ks.dtype == torch.int64
    assert meta.ks_start_end.dtype == torch.int32
    assert np.array_equal(meta.indices.cpu().numpy(), ometa.indices), "indices differ"
    assert np.array_equal(meta.ks.cpu().numpy(), ometa.ks), "ks differ"
    assert np.array_equal(meta.ks_count.cpu().numpy(), ometa.ks_count)
    assert np.array_equal(meta.ks_start_end.cpu().numpy(), ometa.ks_start_end)
    # access statistics, whenever both sides recorded them
    for got, want, name in ((meta.mask_cache_statistics, getattr(ometa, "mask_access", None), "mask"),
                            (meta.sa_cache_statistics, getattr(ometa, "sa_access", None), "attention")):
        if got is None or got.access_counter is None or want is None:
            continue
        a = got.access_counter.cpu().numpy()
        if a.shape != want.shape:
            continue  # oracle ran on the dense tensors, product on a paged copy: flags are indexed differently
        assert np.array_equal(a, want), f"{name} access flags differ in {int((a != want).sum())} entries"


def assert_context_close(ctx, octx, dtype):
    """bf16: 2e-2 abs + 1e-2 rel; f32: 1e-4 (the tolerances the operator is accepted at)."""
    got = O.bf16_bits_to_f32(from_torch(ctx, dtype)) if dtype == "bf16" else from_torch(ctx, dtype)
    ref = O.bf16_bits_to_f32(octx) if dtype == "bf16" else octx
    if dtype == "bf16":
        ok = np.abs(got - ref) <= 2e-2 + 1e-2 * np.abs(ref)
    else:
        ok = np.abs(got - ref) <= 1e-4 + 1e-4 * np.abs(ref)
    assert ok.all(), f"max abs err {np.abs(got - ref).max()}, {int((~ok).sum())} elements out of tolerance"
