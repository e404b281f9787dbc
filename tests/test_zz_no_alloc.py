"""The decode entry point that allocates nothing (mi_attn_decode_static): same kernels and results as mi_attn_decode,
with the per-split partial results in the library's static device array instead of a caller workspace."""

import ctypes
import math

import pytest
import torch

from scaling_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _inputs(B, nq, nkv, d, max_ctx, lens, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, nq, d, generator=g).bfloat16().to(DEV)
    kc = torch.randn(B, max_ctx, nkv, d, generator=g).bfloat16().to(DEV)
    vc = torch.randn(B, max_ctx, nkv, d, generator=g).bfloat16().to(DEV)
    ctx = torch.tensor(lens, dtype=torch.int32, device=DEV)
    return q, kc, vc, ctx


def test_static_scratch_decode_equals_workspace_decode_on_consecutive_calls():
    """Two calls in a row through the C ABI, the second with a smaller input (fewer sequences, heads, shorter
    contexts, fewer splits): the array keeps the first call's contents, and every result must still equal the
    entry point that takes a caller workspace, bit for bit.  Neither call may allocate device memory."""
    lib = _lib.load()
    assert lib.mi_attn_decode_static_scratch_bytes() == 8 << 20
    cases = [(6, 32, 8, 128, 2100, [2100, 1, 777, 2048, 1500, 64], 1), (2, 8, 2, 128, 300, [300, 17], 2),
             (3, 4, 4, 64, 200, [200, 5, 130], 3)]
    for B, nq, nkv, d, max_ctx, lens, seed in cases:
        print(f"case static decode B={B} nq={nq} nkv={nkv} d={d} lens={lens}", flush=True)
        q, kc, vc, ctx = _inputs(B, nq, nkv, d, max_ctx, lens, seed)
        want = ops.decode_attention(q, kc, vc, ctx, softmax_scale=1 / math.sqrt(d))
        out = torch.empty_like(want)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        got = ops.decode_attention(q, kc, vc, ctx, softmax_scale=1 / math.sqrt(d), out=out, static_scratch=True)
        after = torch.cuda.memory_stats()["allocation.all.allocated"]
        torch.cuda.synchronize()
        assert after == before, "the static-scratch call went through torch's allocator"
        assert got.data_ptr() == out.data_ptr() and torch.equal(got, want)
    # explicit split counts: more splits than the library would choose, then a single split (which bypasses the scratch)
    q, kc, vc, ctx = _inputs(2, 16, 2, 128, 1024, [1024, 333], 4)
    for n_splits in (32, 5, 1):
        want = ops.decode_attention(q, kc, vc, ctx, n_splits=n_splits)
        got = ops.decode_attention(q, kc, vc, ctx, n_splits=n_splits, out=torch.empty_like(want), static_scratch=True)
        torch.cuda.synchronize()
        assert torch.equal(got, want), n_splits


def test_static_scratch_decode_rejects_sizes_beyond_the_array():
    """batch 64 x 32 heads x 32 splits x 130 floats = 34 MB > 8 MiB: refused with MI_E_WORKSPACE before any launch."""
    q, kc, vc, ctx = _inputs(64, 32, 8, 128, 64, [64] * 64, 5)
    with pytest.raises(RuntimeError, match="MI_E_WORKSPACE"):
        ops.decode_attention(q, kc, vc, ctx, n_splits=32, out=torch.empty_like(q), static_scratch=True)
    # the same shape with the library's own choice (one split at 512 (sequence, KV head) pairs) needs no scratch and runs
    want = ops.decode_attention(q, kc, vc, ctx)
    got = ops.decode_attention(q, kc, vc, ctx, out=torch.empty_like(q), static_scratch=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_static_scratch_decode_under_graph_capture():
    """The use the entry point exists for: captured into a HIP graph and replayed, with eager work in between."""
    q, kc, vc, ctx = _inputs(4, 32, 8, 128, 900, [900, 512, 31, 700], 6)
    want = ops.decode_attention(q, kc, vc, ctx)
    out = torch.zeros_like(want)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.decode_attention(q, kc, vc, ctx, out=out, static_scratch=True)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.decode_attention(q, kc, vc, ctx, out=out, static_scratch=True)
    for i in range(3):
        out.zero_()
        q2, kc2, vc2, ctx2 = _inputs(2, 8, 2, 128, 300, [300, 17], 7 + i)      # eager work that overwrites the array
        ops.decode_attention(q2, kc2, vc2, ctx2, out=torch.empty_like(q2), static_scratch=True)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i}"
