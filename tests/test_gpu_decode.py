"""GPU parity of the KV-cache decode kernel against the CPU oracle (per-sequence batch-1 reference
semantics: the step output equals the last row of full causal attention over the cached positions)."""

import math

import pytest
import torch

import oracle
from scaling_amd import ops
from tests.parity import check

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _oracle_decode(q, kc, vc, ctx, scale, dtype):
    """q [B,nq,d], caches [B,max,nkv,d] (already containing the new token); one reference call per sequence."""
    B, nq, d = q.shape
    nkv = kc.shape[2]
    outs = []
    for b in range(B):
        n = int(ctx[b])
        qq = q[b].to(dtype).view(1, 1, nq, d)                                   # [s_q=1, b=1, n, d]
        kk = oracle.repeat_kv(kc[b, :n].to(dtype).unsqueeze(1), nq // nkv)      # [s_k, 1, nq, d]
        vv = oracle.repeat_kv(vc[b, :n].to(dtype).unsqueeze(1), nq // nkv)
        o = oracle.multi_head_attention(qq, kk, vv, torch.tensor([0, 1], dtype=torch.int32), True, scale,
                                        softmax_in_fp32=True)                   # [(1 nq), 1, d]
        outs.append(o.view(nq, d))
    return torch.stack(outs)


@pytest.mark.parametrize("B,nq,nkv,d,max_ctx,lens", [
    (3, 8, 2, 128, 300, [1, 137, 300]),
    (2, 4, 4, 64, 128, [128, 5]),
    (4, 32, 8, 128, 1100, [1024, 1025, 33, 1100]),
    (1, 16, 1, 128, 64, [64]),
    # groups of more than 16 query heads (multi-query attention with 32 heads; 24 = one full and one partial chunk)
    (2, 32, 1, 128, 300, [300, 17]),
    (1, 24, 1, 64, 128, [128]),
    # the other head sizes of the attention kernels
    (2, 4, 2, 96, 200, [200, 33]),
    (3, 8, 8, 32, 100, [100, 1, 64]),
    (40, 12, 6, 96, 70, [70, 69, 1, 35] * 10),
    # batch x KV heads >= 192: the 8-wavefront workgroups (a single split writes the output directly)
    (24, 16, 8, 128, 300, [300, 1, 257, 31] * 6),
    (48, 8, 4, 64, 520, [520, 256, 255, 7, 300, 513] * 8),
])
@pytest.mark.parametrize("n_splits", [0, 1, 3])
def test_decode_parity(B, nq, nkv, d, max_ctx, lens, n_splits):
    print(f"case decode B={B} nq={nq} nkv={nkv} d={d} max_ctx={max_ctx} lens={lens} splits={n_splits}", flush=True)
    g = torch.Generator().manual_seed(B * 31 + d)
    q = torch.randn(B, nq, d, generator=g).bfloat16()
    kc = torch.randn(B, max_ctx, nkv, d, generator=g).bfloat16()
    vc = torch.randn(B, max_ctx, nkv, d, generator=g).bfloat16()
    ctx = torch.tensor(lens, dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    ref = _oracle_decode(q, kc, vc, ctx, scale, torch.float32)
    ref_o = _oracle_decode(q, kc, vc, ctx, scale, torch.bfloat16)
    out = ops.decode_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), ctx.to(DEV), softmax_scale=scale, n_splits=n_splits)
    torch.cuda.synchronize()
    check("decode.o", out, ref, ref_o, kind="decode")


def test_decode_append_and_fused_rotary():
    B, nq, nkv, d, max_ctx = 3, 8, 2, 128, 96
    g = torch.Generator().manual_seed(77)
    lens = [10, 96, 1]                       # lengths INCLUDING the appended token
    q = torch.randn(B, nq, d, generator=g).bfloat16()
    k_new = torch.randn(B, nkv, d, generator=g).bfloat16()
    v_new = torch.randn(B, nkv, d, generator=g).bfloat16()
    kc = torch.randn(B, max_ctx, nkv, d, generator=g).bfloat16()
    vc = torch.randn(B, max_ctx, nkv, d, generator=g).bfloat16()
    ctx = torch.tensor(lens, dtype=torch.int32)
    pos = torch.tensor([n - 1 for n in lens], dtype=torch.int64)
    tabs = oracle.rotary_tables(d, max_ctx, 500000, torch.bfloat16)
    hi = oracle.RotaryTables(tabs.cos.float(), tabs.sin.float(), d)
    # reference: rotate the new q/k at their positions, append, attend
    qr, kr = oracle.apply_rotary(q.float().unsqueeze(0), k_new.float().unsqueeze(0), hi, pos.view(1, B), pos.view(1, B))
    qr, kr = qr[0].bfloat16(), kr[0].bfloat16()     # what is stored / consumed after one rounding
    kc_ref, vc_ref = kc.clone(), vc.clone()
    for b in range(B):
        kc_ref[b, lens[b] - 1] = kr[b]
        vc_ref[b, lens[b] - 1] = v_new[b]
    scale = 1 / math.sqrt(d)
    ref = _oracle_decode(qr, kc_ref, vc_ref, ctx, scale, torch.float32)
    ref_o = _oracle_decode(qr, kc_ref, vc_ref, ctx, scale, torch.bfloat16)
    kcd, vcd = kc.to(DEV), vc.to(DEV)
    out = ops.decode_attention(q.to(DEV), kcd, vcd, ctx.to(DEV), k_new.to(DEV), v_new.to(DEV),
                               rotary=(tabs.cos.to(DEV), tabs.sin.to(DEV), pos.to(DEV)), softmax_scale=scale)
    torch.cuda.synchronize()
    check("decode.o(append+rotary)", out, ref, ref_o, kind="decode")
    # the cache was updated in place: only the appended rows changed, and they hold the rotated key
    for b in range(B):
        kd = (kcd[b, lens[b] - 1].float().cpu() - kr[b].float()).abs()
        assert float(kd.max()) <= 2e-2 and float((kd > 0).float().mean()) < 0.02
        assert torch.equal(vcd[b, lens[b] - 1].cpu(), v_new[b])
    mask = torch.ones(B, max_ctx, dtype=torch.bool)
    for b in range(B):
        mask[b, lens[b] - 1] = False
    assert torch.equal(kcd.cpu()[mask], kc[mask]) and torch.equal(vcd.cpu()[mask], vc[mask])


@pytest.mark.parametrize("B,nq,nkv,d", [(3, 8, 2, 128), (2, 4, 4, 64), (32, 32, 8, 128)])
def test_decode_append_and_fused_interleaved_rotary(B, nq, nkv, d):
    """Interleaved-pair rotary of q and of the appended key inside the decode kernels: same bits as the stand-alone
    kernel followed by a plain append, and within the gates of the oracle."""
    print(f"case decode fused interleaved rotary B={B} nq={nq} nkv={nkv} d={d}", flush=True)
    max_ctx = 96
    g = torch.Generator().manual_seed(B + d)
    lens = [(7 * i) % max_ctx + 1 for i in range(B)]
    lens[0] = max_ctx
    q = torch.randn(B, nq, d, generator=g).bfloat16()
    k_new = torch.randn(B, nkv, d, generator=g).bfloat16()
    v_new = torch.randn(B, nkv, d, generator=g).bfloat16()
    kc = torch.randn(B, max_ctx, nkv, d, generator=g).bfloat16()
    vc = torch.randn(B, max_ctx, nkv, d, generator=g).bfloat16()
    ctx = torch.tensor(lens, dtype=torch.int32)
    pos = torch.tensor([n - 1 for n in lens], dtype=torch.int64)
    scale = 1 / math.sqrt(d)
    qr, kr = oracle.apply_rotary_complex(q.unsqueeze(0), k_new.unsqueeze(0), d, max_ctx, 10000.0, pos.view(1, B), pos.view(1, B))
    qr, kr = qr[0], kr[0]                           # fp32 math, one rounding to bf16 (the reference's order)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    for b in range(B):
        kc_ref[b, lens[b] - 1] = kr[b]
        vc_ref[b, lens[b] - 1] = v_new[b]
    ref = _oracle_decode(qr, kc_ref, vc_ref, ctx, scale, torch.float32)
    ref_o = _oracle_decode(qr, kc_ref, vc_ref, ctx, scale, torch.bfloat16)
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, d, 2)[: d // 2].float() / d))
    ang = torch.outer(torch.arange(max_ctx).float(), inv_freq).float()
    real, imag = ang.cos().contiguous().to(DEV), ang.sin().contiguous().to(DEV)
    qd, knd, vnd, ctxd, posd = q.to(DEV), k_new.to(DEV), v_new.to(DEV), ctx.to(DEV), pos.to(DEV)
    kc1, vc1 = kc.to(DEV), vc.to(DEV)
    fused = ops.decode_attention(qd, kc1, vc1, ctxd, knd, vnd, rotary=(real, imag, posd), softmax_scale=scale)
    kc2, vc2 = kc.to(DEV), vc.to(DEV)
    q2 = ops.rotary_embedding_complex(qd, real, imag, posd)
    k2 = ops.rotary_embedding_complex(knd, real, imag, posd)
    sep = ops.decode_attention(q2, kc2, vc2, ctxd, k2, vnd, softmax_scale=scale)
    torch.cuda.synchronize()
    check("decode.o(append+interleaved rotary)", fused, ref, ref_o, kind="decode")
    assert torch.equal(fused, sep) and torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
    for b in range(B):
        kd = (kc1[b, lens[b] - 1].float().cpu() - kr[b].float()).abs()
        assert float(kd.max()) <= 2e-2 and float((kd > 0).float().mean()) < 0.02


def test_decode_equals_last_row_of_prefill_kernel():
    """Cached == uncached: the decode kernel agrees with the last query row of the forward kernel."""
    nq, nkv, d, n = 8, 2, 128, 333
    g = torch.Generator().manual_seed(5)
    q = torch.randn(n, nq, d, generator=g).bfloat16().to(DEV)
    k = torch.randn(n, nkv, d, generator=g).bfloat16().to(DEV)
    v = torch.randn(n, nkv, d, generator=g).bfloat16().to(DEV)
    cu = torch.tensor([0, n], dtype=torch.int32, device=DEV)
    full, _ = ops.attention_forward(q, k, v, cu)
    out = ops.decode_attention(q[n - 1:n].contiguous(), k.unsqueeze(0), v.unsqueeze(0),
                               torch.tensor([n], dtype=torch.int32, device=DEV))
    torch.cuda.synchronize()
    diff = (out[0].float() - full[n - 1].float()).abs()
    assert float(diff.max()) <= 1.6e-2


def test_decode_takes_column_slices_of_a_fused_projection():
    """q, k_new and v_new as strided column slices of one [B, (nq + 2 nkv) d] tensor (what a single q/k/v GEMM
    produces) give bit-identical outputs and cache contents to packed copies of the same values."""
    print("case decode strided operands", flush=True)
    B, nq, nkv, d, max_ctx = 5, 8, 2, 128, 200
    g = torch.Generator().manual_seed(5)
    fused = torch.randn(B, (nq + 2 * nkv) * d, generator=g).bfloat16().to(DEV)
    q = fused[:, :nq * d].view(B, nq, d)
    k = fused[:, nq * d:(nq + nkv) * d].view(B, nkv, d)
    v = fused[:, (nq + nkv) * d:].view(B, nkv, d)
    assert not q.is_contiguous() and q.stride(0) == (nq + 2 * nkv) * d
    ctx = torch.tensor([200, 1, 77, 128, 129], dtype=torch.int32, device=DEV)
    outs, caches = [], []
    for packed in (False, True):
        kc = torch.randn(B, max_ctx, nkv, d, generator=torch.Generator().manual_seed(6)).bfloat16().to(DEV)
        vc = torch.randn(B, max_ctx, nkv, d, generator=torch.Generator().manual_seed(7)).bfloat16().to(DEV)
        args = (q.contiguous(), kc, vc, ctx, k.contiguous(), v.contiguous()) if packed else (q, kc, vc, ctx, k, v)
        outs.append(ops.decode_attention(*args))
        caches.append((kc, vc))
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])
    assert torch.equal(caches[0][0], caches[1][0]) and torch.equal(caches[0][1], caches[1][1])
    for b in range(B):     # the appended rows landed at ctx - 1
        assert torch.equal(caches[0][0][b, int(ctx[b]) - 1], k[b]) and torch.equal(caches[0][1][b, int(ctx[b]) - 1], v[b])
    with pytest.raises(AssertionError):
        ops.decode_attention(fused.view(B, nq + 2 * nkv, d)[:, ::2], caches[0][0], caches[0][1], ctx)   # heads not contiguous


@pytest.mark.parametrize("B,nq,nkv,d,max_ctx,lens", [(3, 8, 2, 128, 300, [1, 137, 300]), (24, 16, 8, 128, 300, [300, 1, 257, 31] * 6),
                                                    (2, 4, 4, 64, 128, [128, 5])])
def test_decode_float16_parity(B, nq, nkv, d, max_ctx, lens):
    """The decode kernels built on the half-precision MFMA (precision: float16), with the in-place append."""
    print(f"case decode f16 B={B} nq={nq} nkv={nkv} d={d} lens={lens}", flush=True)
    g = torch.Generator().manual_seed(B + d)
    q = torch.randn(B, nq, d, generator=g).half()
    kc = torch.randn(B, max_ctx, nkv, d, generator=g).half()
    vc = torch.randn(B, max_ctx, nkv, d, generator=g).half()
    k_new, v_new = torch.randn(B, nkv, d, generator=g).half(), torch.randn(B, nkv, d, generator=g).half()
    ctx = torch.tensor(lens, dtype=torch.int32)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    for b in range(B):
        kc_ref[b, lens[b] - 1] = k_new[b]
        vc_ref[b, lens[b] - 1] = v_new[b]
    scale = 1 / math.sqrt(d)
    ref = _oracle_decode(q, kc_ref, vc_ref, ctx, scale, torch.float32)
    ref_o = _oracle_decode(q, kc_ref, vc_ref, ctx, scale, torch.float16)
    kcd, vcd = kc.to(DEV), vc.to(DEV)
    out = ops.decode_attention(q.to(DEV), kcd, vcd, ctx.to(DEV), k_new.to(DEV), v_new.to(DEV), softmax_scale=scale)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16
    check("decode.f16.o", out, ref, ref_o, kind="decode")
    assert torch.equal(kcd.cpu(), kc_ref) and torch.equal(vcd.cpu(), vc_ref)
