"""GPU parity of the attention core (forward, backward, masks, GQA, fused rotary) against the CPU
oracle, called through the C ABI."""

import math

import pytest
import torch

import oracle
from scaling_amd import ops
from tests import attn_utils as U
from tests.golden import known_answers as KA
from tests.parity import check

pytestmark = pytest.mark.gpu
DEV = "cuda"

# (batch, seq, n_q, n_kv, head_dim, causal, extra cut points)
CASES = [
    (2, 64, 4, 4, 32, True, (32,)),            # the reference's flash-vs-torch test shape (cu = [0,32,64,128])
    (2, 64, 4, 2, 32, False, (32,)),           # ... its GQA variant, bidirectional
    (2, 128, 4, 4, 64, True, ()),              # config 1 attention shape
    (1, 200, 2, 1, 64, True, (3, 77, 78, 150)),  # ragged: seq not a multiple of any tile, tiny documents
    (2, 256, 8, 2, 128, True, (100, 300, 301)),
    (1, 512, 4, 4, 128, False, (130,)),
    (1, 384, 6, 3, 96, True, (129,)),
    (3, 1, 2, 2, 64, True, ()),                # one token per sequence
    # equal-length sequences of whole blocks: the kernels hand out blocks across the sequences (longest first) ...
    (3, 256, 4, 4, 64, True, ()),              # ... forward / dQ (every query head has its own K / V)
    (2, 256, 4, 2, 128, True, ()),             # ... dK/dV (few workgroups)
    (1, 512, 4, 4, 64, True, (100,)),          # ... and two documents that only look equal-length from the host
    # fewer than 8 KV heads: the dK/dV launch splits the query heads of a group over workgroups and sums partials
    (2, 256, 8, 1, 128, True, (100, 300)),     # multi-query attention, 8-way split
    (1, 384, 8, 2, 64, False, (129,)),         # 4-way split, bidirectional
    (1, 320, 12, 4, 96, True, ()),             # group of 3: no split possible, the unsplit kernel
    # documents of different lengths over several blocks: blocks are handed out longest-processing-time first, in an
    # order every workgroup derives from the cumulative lengths (key blocks in dK/dV; query blocks too when n_q = n_kv)
    (1, 1300, 4, 4, 64, True, (100, 450, 451, 1000)),
    (1, 1300, 8, 2, 128, True, (300, 1100)),
    (1, 1100, 4, 4, 64, False, (64, 700)),
    # every token a document of its own (each one an end-of-document token): 300 documents of length 1
    (1, 300, 4, 2, 64, True, tuple(range(1, 300))),
]


@pytest.mark.parametrize("b,s,nq,nkv,d,causal,cuts", CASES)
def test_attention_fwd_bwd_parity(b, s, nq, nkv, d, causal, cuts):
    print(f"case attn b={b} s={s} nq={nq} nkv={nkv} d={d} causal={causal} cuts={cuts}", flush=True)
    q, k, v, do = U.make_qkv(b, s, nq, nkv, d, seed=b * 1000 + s + d)
    cu = U.make_cu(b, s, cuts)
    scale = 1.0 / math.sqrt(d)
    ref = U.oracle_attention(q, k, v, cu, b, s, causal, scale, torch.float32, do)
    ref_o = U.oracle_attention(q, k, v, cu, b, s, causal, scale, torch.bfloat16, do)

    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o = ops.attention(qg, kg, vg, cu.to(DEV), None, causal, scale)
    o.backward(do.to(DEV))
    torch.cuda.synchronize()
    check("attn.o", o, ref[0], ref_o[0], kind="o")
    check("attn.dq", qg.grad, ref[1], ref_o[1], kind="grad")
    check("attn.dk", kg.grad, ref[2], ref_o[2], kind="grad")
    check("attn.dv", vg.grad, ref[3], ref_o[3], kind="grad")


def test_attention_of_no_tokens_is_empty():
    """An empty batch (no tokens at all) is not an error: empty output, empty gradients, no launch."""
    q = torch.zeros(0, 4, 64, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    k = torch.zeros(0, 2, 64, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    v = torch.zeros(0, 2, 64, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    o = ops.attention(q, k, v, torch.zeros(1, dtype=torch.int32, device=DEV), None, True, 0.125)
    assert o.shape == (0, 4, 64)
    o.backward(torch.zeros_like(o))
    assert q.grad.shape == q.shape and k.grad.shape == k.shape and v.grad.shape == v.shape


@pytest.mark.parametrize("b,s,nq,nkv,d,causal,cuts", [
    (2, 128, 4, 4, 64, True, ()),
    (2, 256, 8, 2, 128, True, (100, 300, 301)),
    (1, 512, 4, 4, 128, False, (130,)),
    (1, 384, 6, 3, 96, True, (129,)),
    (2, 256, 8, 1, 128, True, (100, 300)),     # split dK/dV launch + reduce kernel
    (1, 1024, 8, 2, 128, True, (300, 700)),
])
def test_attention_accuracy_mode_meets_the_stated_tolerance(b, s, nq, nkv, d, causal, cuts):
    """MI_ATTN_SPLIT_P (ops.attention(precise=True)): P and dS enter their MFMAs as hi + lo bf16 terms.  Output and all
    three gradients then pass the gates exactly as stated (max-abs <= 2e-2 and mean-relative <= 1e-3 against the fp32
    oracle rounded once to bf16) with no second clause; the default mode's numbers are printed beside them."""
    print(f"case attn precise b={b} s={s} nq={nq} nkv={nkv} d={d} causal={causal} cuts={cuts}", flush=True)
    q, k, v, do = U.make_qkv(b, s, nq, nkv, d, seed=b * 1000 + s + d)
    cu = U.make_cu(b, s, cuts)
    scale = 1.0 / math.sqrt(d)
    ref = U.oracle_attention(q, k, v, cu, b, s, causal, scale, torch.float32, do)
    ref_o = U.oracle_attention(q, k, v, cu, b, s, causal, scale, torch.bfloat16, do)
    for precise in (False, True):
        qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
        o = ops.attention(qg, kg, vg, cu.to(DEV), None, causal, scale, precise=precise)
        o.backward(do.to(DEV))
        torch.cuda.synchronize()
        tag = "precise" if precise else "default"
        for name, got, r, ro in (("o", o, ref[0], ref_o[0]), ("dq", qg.grad, ref[1], ref_o[1]),
                                 ("dk", kg.grad, ref[2], ref_o[2]), ("dv", vg.grad, ref[3], ref_o[3])):
            check(f"attn.{tag}.{name}", got, r, ro, literal=precise, kind="o" if name == "o" else "grad")


@pytest.mark.parametrize("b,s,nq,nkv,d,causal,cuts,rot", [
    (2, 128, 4, 4, 64, True, (), False),
    (2, 256, 8, 2, 128, True, (100, 300, 301), False),
    (1, 384, 6, 3, 96, False, (129,), False),
    (2, 64, 4, 2, 32, True, (32,), False),
    (1, 320, 8, 1, 128, True, (100,), True),        # rotary on the training path, split dK/dV launch
])
def test_attention_float16_fwd_bwd_parity(b, s, nq, nkv, d, causal, cuts, rot):
    """precision: float16 (transformer/context/config.py:28-48): the same kernels built on the half-precision MFMA."""
    print(f"case attn f16 b={b} s={s} nq={nq} nkv={nkv} d={d} causal={causal} cuts={cuts} rotary={rot}", flush=True)
    q, k, v, do = U.make_qkv(b, s, nq, nkv, d, seed=b * 100 + s + d, dtype=torch.float16)
    cu = U.make_cu(b, s, cuts)
    scale, n_rep = 1.0 / math.sqrt(d), nq // nkv
    pos = U.position_ids_from_cu(cu, b * s)
    ids = pos.view(b, s).transpose(0, 1)
    tabs = oracle.rotary_tables(d, s, 10000, torch.float16) if rot else None

    def reference(dtype):
        qq, kk, vv = (t.to(dtype).clone().requires_grad_() for t in (q, k, v))
        q4, k4, v4 = U.to_sbnd(qq, b, s), U.to_sbnd(kk, b, s), U.to_sbnd(vv, b, s)
        if rot:
            q4, k4 = oracle.apply_rotary(q4, k4, oracle.RotaryTables(tabs.cos.to(dtype), tabs.sin.to(dtype), d), ids, ids)
        out = oracle.multi_head_attention(q4, oracle.repeat_kv(k4, n_rep), oracle.repeat_kv(v4, n_rep), cu, causal, scale,
                                          softmax_in_fp32=True)
        o = U.from_bn_s_d(out, b, nq)
        o.backward(do.to(dtype))
        return o.detach(), qq.grad, kk.grad, vv.grad

    ref, ref_o = reference(torch.float32), reference(torch.float16)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    rotary = (tabs.cos.to(DEV), tabs.sin.to(DEV), pos.to(DEV), pos.to(DEV)) if rot else None
    o = ops.attention(qg, kg, vg, cu.to(DEV), None, causal, scale, rotary=rotary)
    o.backward(do.to(DEV))
    torch.cuda.synchronize()
    assert o.dtype == torch.float16 and qg.grad.dtype == torch.float16
    for name, got, r, ro in (("o", o, ref[0], ref_o[0]), ("dq", qg.grad, ref[1], ref_o[1]),
                             ("dk", kg.grad, ref[2], ref_o[2]), ("dv", vg.grad, ref[3], ref_o[3])):
        check(f"attn.f16.{name}", got, r, ro, kind="o" if name == "o" else "grad")


def test_attention_mask_is_bit_exact_on_reference_known_answers():
    """q = k = 0 makes the softmax uniform over the allowed keys; with one-hot values the output row is
    1/count on exactly the allowed key positions, which exposes the kernel's mask predicate."""
    s, b = KA.MASK_SEQ_LEN, 3
    cu = torch.tensor(KA.MASK_CU_SEQLENS, dtype=torch.int32)
    d = 32
    q = torch.zeros(b * s, 1, d, dtype=torch.bfloat16)
    v = torch.zeros(b * s, 1, d, dtype=torch.bfloat16)
    for t in range(b * s):
        v[t, 0, t % s] = 1.0
    for causal, allowed in ((True, KA.MASK_ALLOWED_CAUSAL), (False, KA.MASK_ALLOWED_BIDIRECTIONAL)):
        o, _ = ops.attention_forward(q.to(DEV), q.to(DEV), v.to(DEV), cu.to(DEV), None, causal, 1.0)
        got = (o.float().cpu().view(b, s, d)[:, :, :s] > 0)
        assert torch.equal(got, torch.tensor(allowed, dtype=torch.bool))
        assert torch.equal(~got.unsqueeze(1), oracle.cumulative_seq_lengths_to_dense_attention_mask(cu, s, causal))
        assert not bool((o.float().cpu().view(b, s, d)[:, :, s:] != 0).any())


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_attention_mask_random_documents_bit_exact(seed):
    g = torch.Generator().manual_seed(seed)
    b, s, d = 2, 96, 96
    cuts = sorted(set(int(x) for x in torch.randint(1, b * s, (7,), generator=g)))
    cu = U.make_cu(b, s, cuts)
    q = torch.zeros(b * s, 2, d, dtype=torch.bfloat16)
    v = torch.zeros(b * s, 2, d, dtype=torch.bfloat16)
    for t in range(b * s):
        v[t, :, t % s] = 1.0
    for causal in (True, False):
        o, _ = ops.attention_forward(q.to(DEV), q.to(DEV), v.to(DEV), cu.to(DEV), None, causal, 1.0)
        got = o.float().cpu().view(b, s, 2, d) > 0
        want = ~oracle.cumulative_seq_lengths_to_dense_attention_mask(cu, s, causal)   # [b,1,s,s]
        assert torch.equal(got[:, :, 0, :], want[:, 0]) and torch.equal(got[:, :, 1, :], want[:, 0])


def test_attention_fused_rotary_matches_separate_rotary():
    b, s, nq, nkv, d = 2, 192, 4, 2, 128
    q, k, v, _ = U.make_qkv(b, s, nq, nkv, d, seed=5)
    cu = U.make_cu(b, s, (50, 250))
    pos = U.position_ids_from_cu(cu, b * s)
    tabs = oracle.rotary_tables(d, s, 500000, torch.bfloat16)
    cos, sin = tabs.cos.to(DEV), tabs.sin.to(DEV)
    qd, kd, vd, cud, posd = q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), pos.to(DEV)
    # oracle: rotary (table values as stored, fp32 arithmetic) then attention, everything fp32
    hi = oracle.RotaryTables(tabs.cos.float(), tabs.sin.float(), d)
    ids = pos.view(b, s).transpose(0, 1)
    qr, kr = oracle.apply_rotary(U.to_sbnd(q.float(), b, s), U.to_sbnd(k.float(), b, s), hi, ids, ids)
    ref = U.from_bn_s_d(oracle.multi_head_attention(qr, oracle.repeat_kv(kr, 2), oracle.repeat_kv(U.to_sbnd(v.float(), b, s), 2),
                                                    cu, True, 1 / math.sqrt(d), softmax_in_fp32=True), b, nq)
    qo, ko = oracle.apply_rotary(U.to_sbnd(q, b, s), U.to_sbnd(k, b, s), tabs, ids, ids)
    ref_o = U.from_bn_s_d(oracle.multi_head_attention(qo, oracle.repeat_kv(ko, 2), oracle.repeat_kv(U.to_sbnd(v, b, s), 2),
                                                      cu, True, 1 / math.sqrt(d), softmax_in_fp32=True), b, nq)
    fused, _ = ops.attention_forward(qd, kd, vd, cud, None, True, None, rotary=(cos, sin, posd, posd))
    q2 = ops.rotary_embedding(qd, cos, sin, posd)
    k2 = ops.rotary_embedding(kd, cos, sin, posd)
    sep, _ = ops.attention_forward(q2, k2, vd, cud, None, True, None)
    torch.cuda.synchronize()
    check("attn.fused_rotary", fused, ref, ref_o, kind="rotary")
    check("attn.separate_rotary", sep, ref, ref_o, kind="rotary")
    # same rounding points (rotate in fp32, round once to bf16); only fma contraction may differ
    diff = (fused.float() - sep.float()).abs()
    assert float(diff.max()) <= 2e-2 and float((diff > 0).float().mean()) < 0.02


def _complex_tables(d, rows, base):
    """fp32 [rows, d / 2] real / imaginary parts of freqs_cis (core/nn/rotary.py:45-56)."""
    inv_freq = 1.0 / (float(base) ** (torch.arange(0, d, 2)[: d // 2].float() / d))
    ang = torch.outer(torch.arange(rows).float(), inv_freq).float()
    return ang.cos().contiguous(), ang.sin().contiguous()


@pytest.mark.parametrize("kind,b,s,nq,nkv,d,cuts,p_drop", [
    ("half", 2, 192, 4, 2, 128, (50, 250), 0.0),
    ("half", 1, 320, 8, 1, 128, (100,), 0.0),          # one KV head: dK goes through the partial-sum reduce kernel
    ("half", 2, 96, 4, 4, 64, (), 0.0),
    ("interleaved", 2, 160, 4, 2, 128, (70,), 0.0),
    ("interleaved", 1, 200, 8, 2, 64, (33, 34), 0.0),  # 4-way head split
    ("half", 1, 256, 4, 2, 128, (77,), 0.1),           # rotary together with dropout
])
def test_attention_with_rotary_fwd_bwd_parity(kind, b, s, nq, nkv, d, cuts, p_drop):
    """ops.attention(rotary=...) is rotary -> attention of the reference (attention.py:836-845, 876-888): q is rotated
    inside the forward kernel, k by the stand-alone kernel, and dq / dk are rotated back inside the backward kernels.
    Output and the gradients of the UNROTATED q, k, v against the oracle's rotary followed by its attention."""
    print(f"case attn rotary {kind} b={b} s={s} nq={nq} nkv={nkv} d={d} cuts={cuts} dropout={p_drop}", flush=True)
    q, k, v, do = U.make_qkv(b, s, nq, nkv, d, seed=s + d + nq)
    cu = U.make_cu(b, s, cuts)
    pos = U.position_ids_from_cu(cu, b * s)
    ids = pos.view(b, s).transpose(0, 1)
    scale, n_rep = 1 / math.sqrt(d), nq // nkv
    seed = 1234567 + s
    drop = None
    if p_drop > 0:
        keep, p_eff = U.dropout_keep_mask(seed, nq, b * s, b * s, p_drop)
        drop = dict(dropout_p=p_eff, dropout_keep=torch.stack([keep[:, i * s:(i + 1) * s, i * s:(i + 1) * s] for i in range(b)]))
    if kind == "half":
        tabs = oracle.rotary_tables(d, s, 500000, torch.bfloat16)
        dev_tabs = (tabs.cos.to(DEV), tabs.sin.to(DEV))
    else:
        dev_tabs = tuple(t.to(DEV) for t in _complex_tables(d, s, 10000.0))

    def reference(dtype):
        qq, kk, vv = (t.to(dtype).clone().requires_grad_() for t in (q, k, v))
        q4, k4, v4 = U.to_sbnd(qq, b, s), U.to_sbnd(kk, b, s), U.to_sbnd(vv, b, s)
        if kind == "half":    # table values as stored (bf16), arithmetic in `dtype`
            q4, k4 = oracle.apply_rotary(q4, k4, oracle.RotaryTables(tabs.cos.to(dtype), tabs.sin.to(dtype), d), ids, ids)
        else:
            q4, k4 = oracle.apply_rotary_complex(q4, k4, d, s, 10000.0, ids, ids)
        out = oracle.multi_head_attention(q4, oracle.repeat_kv(k4, n_rep), oracle.repeat_kv(v4, n_rep), cu, True, scale,
                                          softmax_in_fp32=True, **(drop or {}))
        o = U.from_bn_s_d(out, b, nq)
        o.backward(do.to(dtype))
        return o.detach(), qq.grad, kk.grad, vv.grad

    ref, ref_o = reference(torch.float32), reference(torch.bfloat16)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    posd = pos.to(DEV)
    o = ops.attention(qg, kg, vg, cu.to(DEV), None, True, scale, rotary=(*dev_tabs, posd, posd), dropout_p=p_drop, dropout_seed=seed)
    o.backward(do.to(DEV))
    torch.cuda.synchronize()
    for name, got, r, ro in (("o", o, ref[0], ref_o[0]), ("dq", qg.grad, ref[1], ref_o[1]),
                             ("dk", kg.grad, ref[2], ref_o[2]), ("dv", vg.grad, ref[3], ref_o[3])):
        check(f"attn.rotary[{kind}].{name}", got, r, ro, kind="rotary")
    # without autograd the same kernels run (minus the copy of the rotated q): same output bits
    with torch.no_grad():
        o2 = ops.attention(qg, kg, vg, cu.to(DEV), None, True, scale, rotary=(*dev_tabs, posd, posd), dropout_p=p_drop, dropout_seed=seed)
    assert torch.equal(o2, o.detach())


def _cross_length_reference(q, k, v, do, cu_q, cu_k, causal, scale, dtype=torch.float32):
    """Brute force from the mask predicate of the C header, one document at a time: query t of document j may
    attend key u of the same document iff (not causal) or u_local <= t_local + (len_k - len_q); rows without any
    allowed key give zeros.  dtype float32 is the target; bfloat16 follows the reference's rounding points (scores
    and probabilities in bf16 around an fp32 softmax, attention.py:160-211) and gives the error floor.
    Returns o, dq, dk, dv."""
    q, k, v = (t.to(dtype).clone().requires_grad_() for t in (q, k, v))
    n_rep = q.shape[1] // k.shape[1]
    outs = []
    for j in range(cu_q.numel() - 1):
        q0, q1, k0, k1 = int(cu_q[j]), int(cu_q[j + 1]), int(cu_k[j]), int(cu_k[j + 1])
        lq, lk = q1 - q0, k1 - k0
        if lq == 0:
            continue
        kj = k[k0:k1].repeat_interleave(n_rep, dim=1)
        vj = v[k0:k1].repeat_interleave(n_rep, dim=1)
        sc = (torch.einsum("tnd,und->ntu", q[q0:q1], kj) * scale).float()
        allowed = torch.ones(lq, lk, dtype=torch.bool)
        if causal:
            allowed = torch.arange(lk)[None, :] <= torch.arange(lq)[:, None] + (lk - lq)
        sc = sc.masked_fill(~allowed[None], float("-inf"))
        p = torch.softmax(sc, dim=-1)
        p = torch.where(allowed.any(dim=1)[None, :, None], p, torch.zeros_like(p))   # rows with no key: zeros, not NaN
        outs.append(torch.einsum("ntu,und->tnd", p.to(dtype), vj))
    o = torch.cat(outs, dim=0)
    o.backward(do.to(dtype))
    return o.detach(), q.grad, k.grad, v.grad


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("nq,nkv,d", [(4, 2, 128), (2, 2, 64)])
def test_attention_with_separate_key_lengths(causal, nq, nkv, d):
    """Documents whose query and key lengths differ (cu_seqlens_k given): chunked prefill against a longer key
    prefix, single-query documents, more queries than keys (causal: the first rows see nothing and must be zero),
    and an empty document."""
    print(f"case cross-length causal={causal} nq={nq} nkv={nkv} d={d}", flush=True)
    len_q = [5, 64, 1, 130, 0, 10, 257]
    len_k = [70, 64, 33, 200, 0, 4, 300]
    cu_q = torch.tensor([0] + torch.tensor(len_q).cumsum(0).tolist(), dtype=torch.int32)
    cu_k = torch.tensor([0] + torch.tensor(len_k).cumsum(0).tolist(), dtype=torch.int32)
    g = torch.Generator().manual_seed(17 + d)
    q = torch.randn(int(cu_q[-1]), nq, d, generator=g).bfloat16()
    k = torch.randn(int(cu_k[-1]), nkv, d, generator=g).bfloat16()
    v = torch.randn(int(cu_k[-1]), nkv, d, generator=g).bfloat16()
    do = torch.randn(int(cu_q[-1]), nq, d, generator=g).bfloat16()
    scale = 1 / math.sqrt(d)
    ref = _cross_length_reference(q, k, v, do, cu_q, cu_k, causal, scale)
    ref_o = _cross_length_reference(q, k, v, do, cu_q, cu_k, causal, scale, torch.bfloat16)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o = ops.attention(qg, kg, vg, cu_q.to(DEV), cu_k.to(DEV), causal, scale)
    o.backward(do.to(DEV))
    torch.cuda.synchronize()
    check("cross.o", o, ref[0], ref_o[0], kind="o")
    check("cross.dq", qg.grad, ref[1], ref_o[1], kind="grad")
    check("cross.dk", kg.grad, ref[2], ref_o[2], kind="grad")
    check("cross.dv", vg.grad, ref[3], ref_o[3], kind="grad")
    if causal:   # document 5: 10 queries, 4 keys -> queries 0..5 have no key
        a = int(cu_q[5])
        assert torch.count_nonzero(o[a:a + 6]) == 0 and torch.count_nonzero(qg.grad[a:a + 6]) == 0


def test_attention_single_token_documents_return_v_exactly():
    """Every token its own document: each query sees one key, the probability is exactly 1, so O = V (per KV group),
    dV = dO summed over the group, dQ = dK = 0 up to rounding, whatever the tiling does with 700 documents in a 256-query block."""
    T, nq, nkv, d = 700, 8, 2, 128
    g = torch.Generator().manual_seed(21)
    q, k, v, do = (torch.randn(T, n, d, generator=g).bfloat16().to(DEV) for n in (nq, nkv, nkv, nq))
    cu = torch.arange(0, T + 1, dtype=torch.int32, device=DEV)
    qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))
    o = ops.attention(qg, kg, vg, cu, None, True, None)
    o.backward(do)
    torch.cuda.synchronize()
    assert torch.equal(o, v.repeat_interleave(nq // nkv, dim=1))
    # dS = P * (dP - delta) with dP and delta two fp32 evaluations of the same dot product: rounding noise only
    assert qg.grad.float().abs().max().item() <= 1e-5 and kg.grad.float().abs().max().item() <= 1e-5
    dv_ref = do.float().view(T, nkv, nq // nkv, d).sum(dim=2)
    assert torch.allclose(vg.grad.float(), dv_ref, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("flags", [1, 2])
def test_attention_fused_interleaved_rotary_matches_separate_rotary(d, flags):
    """Interleaved-pair ("complex") rotary applied while q / k are loaded: same bits as the stand-alone kernel
    followed by the plain call, and the oracle's complex rotary followed by its attention within the gates."""
    print(f"case fused interleaved rotary d={d} flags={flags}", flush=True)
    b, s, nq, nkv = 2, 320, 4, 2
    q, k, v, _ = U.make_qkv(b, s, nq, nkv, d, seed=9)
    cu = U.make_cu(b, s, (70, 400))
    pos = U.position_ids_from_cu(cu, b * s)
    ids = pos.view(b, s).transpose(0, 1)
    scale = 1 / math.sqrt(d)
    n_rep = nq // nkv
    qr, kr = oracle.apply_rotary_complex(U.to_sbnd(q.float(), b, s), U.to_sbnd(k.float(), b, s), d, s, 10000.0, ids, ids)
    ref = U.from_bn_s_d(oracle.multi_head_attention(qr, oracle.repeat_kv(kr, n_rep), oracle.repeat_kv(U.to_sbnd(v.float(), b, s), n_rep),
                                                    cu, True, scale, softmax_in_fp32=True), b, nq)
    qo, ko = oracle.apply_rotary_complex(U.to_sbnd(q, b, s), U.to_sbnd(k, b, s), d, s, 10000.0, ids, ids)
    ref_o = U.from_bn_s_d(oracle.multi_head_attention(qo, oracle.repeat_kv(ko, n_rep), oracle.repeat_kv(U.to_sbnd(v, b, s), n_rep),
                                                      cu, True, scale, softmax_in_fp32=True), b, nq)
    real, imag = (t.to(DEV) for t in _complex_tables(d, s, 10000.0))
    qd, kd, vd, cud, posd = q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), pos.to(DEV)
    fused, lse_f = ops.attention_forward(qd, kd, vd, cud, None, True, None, rotary=(real, imag, posd, posd), flags=flags)
    q2 = ops.rotary_embedding_complex(qd, real, imag, posd)
    k2 = ops.rotary_embedding_complex(kd, real, imag, posd)
    sep, lse_s = ops.attention_forward(q2, k2, vd, cud, None, True, None, flags=flags)
    torch.cuda.synchronize()
    check("attn.fused_interleaved_rotary", fused, ref, ref_o, kind="rotary")
    assert torch.equal(fused, sep) and torch.equal(lse_f, lse_s)
    # tables of the wrong shape or type are refused before the launch
    with pytest.raises(AssertionError):
        ops.attention_forward(qd, kd, vd, cud, None, True, None, rotary=(real[:, : d // 4].contiguous(), imag[:, : d // 4].contiguous(), posd, posd))


def test_attention_is_bit_reproducible_and_gqa_equals_repeated_heads():
    b, s, nq, nkv, d = 1, 320, 8, 2, 128
    q, k, v, do = U.make_qkv(b, s, nq, nkv, d, seed=9)
    cu = U.make_cu(b, s, (100,)).to(DEV)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    o1, lse1 = ops.attention_forward(qd, kd, vd, cu)
    o2, lse2 = ops.attention_forward(qd, kd, vd, cu)
    assert torch.equal(o1, o2) and torch.equal(lse1, lse2)
    g1 = ops.attention_backward(dod, qd, kd, vd, o1, lse1, cu)
    g2 = ops.attention_backward(dod, qd, kd, vd, o1, lse1, cu)
    assert all(torch.equal(a, c) for a, c in zip(g1, g2))
    # explicit repeat_interleave of the kv heads gives the same output bits
    kr = torch.repeat_interleave(kd, 4, dim=1)
    vr = torch.repeat_interleave(vd, 4, dim=1)
    o3, _ = ops.attention_forward(qd, kr, vr, cu)
    assert torch.equal(o1, o3)
    # log-sum-exp against the closed form on a few rows
    lse_ref = []
    for t in (0, 99, 100, 319):
        lo = 0 if t < 100 else 100
        sc = (k[lo:t + 1, 0].double() @ q[t, 1].double()) / math.sqrt(d)
        lse_ref.append(torch.logsumexp(sc, 0))
    got = lse1[1, [0, 99, 100, 319]].double().cpu()
    assert torch.allclose(got, torch.stack(lse_ref), atol=2e-3)


def test_attention_strided_views_of_fused_qkv():
    """q, k, v as per-head slices of one fused projection output ([tokens, heads, 3*d]), as the
    reference's qkv_in_one layout produces them."""
    b, s, n, d = 2, 96, 4, 64
    g = torch.Generator().manual_seed(13)
    qkv = torch.randn(b * s, n, 3 * d, generator=g).bfloat16()
    cu = U.make_cu(b, s)
    ref = U.oracle_attention(qkv[..., :d], qkv[..., d:2 * d], qkv[..., 2 * d:], cu, b, s, True, 1 / math.sqrt(d))
    ref_o = U.oracle_attention(qkv[..., :d], qkv[..., d:2 * d], qkv[..., 2 * d:], cu, b, s, True, 1 / math.sqrt(d), torch.bfloat16)
    qd = qkv.to(DEV)
    o, _ = ops.attention_forward(qd[..., :d], qd[..., d:2 * d], qd[..., 2 * d:], cu.to(DEV))
    check("attn.o(strided)", o, ref, ref_o, kind="o")


def test_attention_rejects_unsupported_input():
    q = torch.zeros(8, 2, 80, dtype=torch.bfloat16, device=DEV)
    cu = torch.tensor([0, 8], dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="head_dim"):
        ops.attention_forward(q, q, q, cu)
    # float32 runs its own kernels, which take neither dropout nor the fused rotary
    qf = torch.zeros(8, 2, 64, dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError, match="dropout"):
        ops.attention_forward(qf, qf, qf, cu, dropout=(0.1, 3))
    with pytest.raises(RuntimeError, match="rotary"):
        a = ops._fill_attn_args(qf, qf, qf, torch.empty_like(qf), torch.empty(2, 8, device=DEV), cu, None, True, 0.125)
        a.rotary_cos = a.rotary_sin = a.position_ids_q = qf.data_ptr()
        a.rotary_table_rows = 8
        ops.check(ops._lib.load().mi_attn_fwd(ops.ctypes.byref(a)), "mi_attn_fwd")
    qd = torch.zeros(8, 2, 64, dtype=torch.float64, device=DEV)
    with pytest.raises((RuntimeError, TypeError)):
        ops.attention_forward(qd, qd, qd, cu)


@pytest.mark.parametrize("flags", [1, 2])
@pytest.mark.parametrize("rot", [False, True])
def test_attention_forward_tilings_agree_with_oracle(flags, rot):
    """Both forward tilings (one / two query groups per wavefront), with and without fused rotary."""
    b, s, nq, nkv, d = 1, 700, 4, 2, 128
    q, k, v, _ = U.make_qkv(b, s, nq, nkv, d, seed=21)
    cu = U.make_cu(b, s, (130, 131, 555))
    pos = U.position_ids_from_cu(cu, b * s)
    tabs = oracle.rotary_tables(d, s, 500000, torch.bfloat16)
    scale = 1 / math.sqrt(d)
    if rot:
        ids = pos.view(b, s).transpose(0, 1)
        hi = oracle.RotaryTables(tabs.cos.float(), tabs.sin.float(), d)
        qr, kr = oracle.apply_rotary(U.to_sbnd(q.float(), b, s), U.to_sbnd(k.float(), b, s), hi, ids, ids)
        qr = qr.permute(1, 0, 2, 3).reshape(b * s, nq, d).bfloat16()
        kr = kr.permute(1, 0, 2, 3).reshape(b * s, nkv, d).bfloat16()
    else:
        qr, kr = q, k
    ref = U.oracle_attention(qr, kr, v, cu, b, s, True, scale)
    ref_o = U.oracle_attention(qr, kr, v, cu, b, s, True, scale, torch.bfloat16)
    rotary = (tabs.cos.to(DEV), tabs.sin.to(DEV), pos.to(DEV), pos.to(DEV)) if rot else None
    o, _ = ops.attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), None, True, scale, rotary=rotary, flags=flags)
    torch.cuda.synchronize()
    check(f"attn.o(flags={flags},rot={rot})", o, ref, ref_o, kind="rotary" if rot else "o")


def test_attention_medium_multi_tile_backward():
    """Several query / key blocks per head and a GQA group of 4: exercises every loop of the backward."""
    b, s, nq, nkv, d = 1, 1024, 8, 2, 128
    q, k, v, do = U.make_qkv(b, s, nq, nkv, d, seed=33)
    cu = U.make_cu(b, s, (300, 700))
    scale = 1 / math.sqrt(d)
    ref = U.oracle_attention(q, k, v, cu, b, s, True, scale, torch.float32, do)
    ref_o = U.oracle_attention(q, k, v, cu, b, s, True, scale, torch.bfloat16, do)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o = ops.attention(qg, kg, vg, cu.to(DEV), None, True, scale)
    o.backward(do.to(DEV))
    torch.cuda.synchronize()
    check("attn1k.o", o, ref[0], ref_o[0], kind="o")
    check("attn1k.dq", qg.grad, ref[1], ref_o[1], kind="grad")
    check("attn1k.dk", kg.grad, ref[2], ref_o[2], kind="grad")
    check("attn1k.dv", vg.grad, ref[3], ref_o[3], kind="grad")


@pytest.mark.parametrize("name,b,s,nq,nkv,docs", [("config2", 4, 2048, 32, 32, False), ("config3", 1, 8192, 32, 8, True)])
def test_attention_full_size_properties(name, b, s, nq, nkv, docs):
    """At the benchmark sizes the dense oracle does not fit; check size-independent properties:
    sampled rows against an fp64 row-wise evaluation, V = ones -> O = ones, and GQA head sharing."""
    d = 128
    g = torch.Generator().manual_seed(100 + s)
    q = torch.randn(b * s, nq, d, generator=g).bfloat16()
    k = torch.randn(b * s, nkv, d, generator=g).bfloat16()
    v = torch.randn(b * s, nkv, d, generator=g).bfloat16()
    cu = U.random_docs_cu(b * s, 256, 2048, seed=7) if docs else U.make_cu(b, s)
    scale = 1 / math.sqrt(d)
    qd, kd, vd, cud = q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV)
    o, lse = ops.attention_forward(qd, kd, vd, cud, None, True, scale)
    torch.cuda.synchronize()
    starts = cu.tolist()

    def lo_hi(r):
        j = max(i for i, c in enumerate(starts) if c <= r)
        return starts[j], r + 1

    rows = sorted(set([0, 1, 127, 128, 255, 256, b * s - 1] + [int(x) for x in torch.randint(0, b * s, (40,), generator=g)]))
    for head in (0, nq // 2 + 1, nq - 1):
        kvh = head // (nq // nkv)
        ref = U.rows_reference(q, k, v, lo_hi, rows, head, kvh, scale)
        ref_o = U.rows_reference(q, k, v, lo_hi, rows, head, kvh, scale, reference_bf16_order=True)
        check(f"{name}.rows.head{head}", o[rows, head], ref, ref_o, kind="o")
    ones = torch.ones_like(vd)
    o1, _ = ops.attention_forward(qd, kd, ones, cud, None, True, scale)
    assert float((o1.float() - 1).abs().max()) <= 2 ** -7
    assert bool(torch.isfinite(lse).all())


# ---- dropout on the attention probabilities (attention.py:204-207) --------------------------------------------
@pytest.mark.parametrize("b,s,nq,nkv,d,causal,cuts,p", [
    (1, 256, 4, 4, 128, True, (), 0.1),
    (2, 192, 4, 2, 64, True, (100, 250), 0.25),
    (1, 320, 8, 2, 128, False, (77,), 0.1),
    (1, 200, 2, 1, 32, True, (), 0.5),
    (1, 136, 3, 3, 96, True, (9,), 0.05),
])
def test_attention_dropout_matches_oracle_with_the_same_mask(b, s, nq, nkv, d, causal, cuts, p):
    """The kernels' mask is a documented integer function of (seed, head, query, key); the test rebuilds it in
    numpy and hands it to the oracle, so forward and all three gradients are compared element for element."""
    print(f"case attn dropout b={b} s={s} nq={nq} nkv={nkv} d={d} causal={causal} cuts={cuts} p={p}", flush=True)
    seed = 0x1234_5678_9ABC_DEF0 + s
    q, k, v, do = U.make_qkv(b, s, nq, nkv, d, seed=s + nq)
    cu = U.make_cu(b, s, cuts)
    scale = 1.0 / math.sqrt(d)
    keep, p_eff = U.dropout_keep_mask(seed, nq, b * s, b * s, p)
    assert abs(p_eff - p) <= 1.0 / 512
    ref = U.oracle_attention(q, k, v, cu, b, s, causal, scale, torch.float32, do, dropout=(keep, p_eff))
    ref_o = U.oracle_attention(q, k, v, cu, b, s, causal, scale, torch.bfloat16, do, dropout=(keep, p_eff))
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o = ops.attention(qg, kg, vg, cu.to(DEV), None, causal, scale, dropout_p=p, dropout_seed=seed)
    o.backward(do.to(DEV))
    torch.cuda.synchronize()
    for name, got, r, ro in (("o", o, ref[0], ref_o[0]), ("dq", qg.grad, ref[1], ref_o[1]),
                             ("dk", kg.grad, ref[2], ref_o[2]), ("dv", vg.grad, ref[3], ref_o[3])):
        check(f"attn.dropout.{name}", got, r, ro, kind="o" if name == "o" else "grad")
    # the mask really dropped something, the same seed reproduces the result, another seed does not
    plain = ops.attention(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), None, causal, scale)
    assert not torch.equal(plain, o.detach())
    again = ops.attention(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), None, causal, scale, dropout_p=p, dropout_seed=seed)
    other = ops.attention(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), None, causal, scale, dropout_p=p, dropout_seed=seed + 1)
    assert torch.equal(again, o.detach()) and not torch.equal(other, o.detach())


def test_attention_dropout_statistics_and_generator_seed():
    """With V = identity-like one-hot rows the output of a non-causal single document is the dropped probability
    matrix itself, which exposes the keep rate; seeds drawn from the device generator follow torch.manual_seed."""
    print("case attn dropout statistics", flush=True)
    s, d, p = 128, 128, 0.1
    q = torch.zeros(s, 8, d, dtype=torch.bfloat16, device=DEV)      # uniform probabilities 1 / s
    k = torch.zeros(s, 8, d, dtype=torch.bfloat16, device=DEV)
    v = torch.eye(s, d, dtype=torch.bfloat16, device=DEV).unsqueeze(1).expand(s, 8, d).contiguous()
    cu = torch.tensor([0, s], dtype=torch.int32, device=DEV)
    seed = 99
    o = ops.attention(q, k, v, cu, None, False, 1.0, dropout_p=p, dropout_seed=seed)   # o[q, h, k] = keep / (1 - p) / s
    keep, p_eff = U.dropout_keep_mask(seed, 8, s, s, p)
    got_keep = (o.float().cpu() > 0).permute(1, 0, 2)
    assert torch.equal(got_keep, keep)
    kept_value = o.float().max().item()
    assert abs(kept_value - 1.0 / (1.0 - p_eff) / s) < 1e-4
    rate = got_keep.float().mean().item()
    assert abs(rate - (1.0 - p_eff)) < 4 * math.sqrt(p_eff * (1 - p_eff) / got_keep.numel())
    torch.manual_seed(7)
    a = ops.attention(q, k, v, cu, None, False, 1.0, dropout_p=p)
    b2 = ops.attention(q, k, v, cu, None, False, 1.0, dropout_p=p)
    torch.manual_seed(7)
    a2 = ops.attention(q, k, v, cu, None, False, 1.0, dropout_p=p)
    assert torch.equal(a, a2) and not torch.equal(a, b2)


# ---- float32 tensors (the reference's default precision) ---------------------------------------------------------------
@pytest.mark.parametrize("b,s,nq,nkv,d,causal,cuts", [
    (2, 128, 4, 4, 64, True, ()),                 # config 1 attention shape, in config 1's own dtype
    (2, 64, 4, 2, 32, False, (32,)),              # GQA, bidirectional, documents
    (1, 200, 2, 1, 64, True, (3, 77, 78, 150)),   # ragged: not a multiple of the 32-token tiles, tiny documents
    (2, 96, 8, 2, 128, True, (100,)),
    (1, 160, 6, 3, 96, True, (33,)),
    (3, 1, 2, 2, 64, True, ()),                   # one token per sequence
])
def test_attention_float32_fwd_bwd_parity(b, s, nq, nkv, d, causal, cuts):
    """fp32 q / k / v through the fp32 kernels against the oracle in fp32: the stated gates, with no second clause, and
    far inside them (the arithmetic is fp32 on both sides; what differs is the summation order)."""
    print(f"case attn f32 b={b} s={s} nq={nq} nkv={nkv} d={d} causal={causal} cuts={cuts}", flush=True)
    q, k, v, do = U.make_qkv(b, s, nq, nkv, d, seed=7 + s + d, dtype=torch.float32)
    cu = U.make_cu(b, s, cuts)
    scale = 1.0 / math.sqrt(d)
    ref = U.oracle_attention(q, k, v, cu, b, s, causal, scale, torch.float32, do)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o = ops.attention(qg, kg, vg, cu.to(DEV), None, causal, scale)
    assert o.dtype == torch.float32
    o.backward(do.to(DEV))
    torch.cuda.synchronize()
    for name, got, r in (("o", o, ref[0]), ("dq", qg.grad, ref[1]), ("dk", kg.grad, ref[2]), ("dv", vg.grad, ref[3])):
        m = check(f"attn.f32.{name}", got, r, literal=True, max_abs_tol=1e-4, mean_rel_tol=1e-5)
        assert m["clause_abs"] == "literal" and m["clause_rel"] == "literal"
    # bit-reproducible, and GQA equals explicitly repeated heads
    o2, lse2 = ops.attention_forward(qg.detach(), kg.detach(), vg.detach(), cu.to(DEV), None, causal, scale)
    assert torch.equal(o2, o.detach())
    if nq != nkv:
        rep = nq // nkv
        o3, _ = ops.attention_forward(qg.detach(), kg.detach().repeat_interleave(rep, 1).contiguous(),
                                      vg.detach().repeat_interleave(rep, 1).contiguous(), cu.to(DEV), None, causal, scale)
        assert torch.equal(o3, o2)


def test_attention_float32_cross_length_and_rotary():
    """fp32: keys longer than queries (causal diagonal aligned to the end of the keys), and the rotary embedding applied
    by the stand-alone kernel in front of the fp32 core when ops.attention is handed fp32 tables."""
    b, s_q, s_k, nq, nkv, d = 2, 24, 88, 4, 2, 64
    g = torch.Generator().manual_seed(5)
    q = torch.randn(b * s_q, nq, d, generator=g)
    k = torch.randn(b * s_k, nkv, d, generator=g)
    v = torch.randn(b * s_k, nkv, d, generator=g)
    cu_q = torch.arange(0, b * s_q + 1, s_q, dtype=torch.int32)
    cu_k = torch.arange(0, b * s_k + 1, s_k, dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    o = ops.attention(q.to(DEV), k.to(DEV), v.to(DEV), cu_q.to(DEV), cu_k.to(DEV), True, scale)
    allowed = torch.ones(s_q, s_k, dtype=torch.bool).tril(diagonal=s_k - s_q)
    mask = (~allowed).view(1, 1, s_q, s_k).expand(b, 1, s_q, s_k)
    ref = oracle.multi_head_attention(U.to_sbnd(q, b, s_q), oracle.repeat_kv(U.to_sbnd(k, b, s_k), nq // nkv),
                                      oracle.repeat_kv(U.to_sbnd(v, b, s_k), nq // nkv), cu_q, True, scale, mask=mask)
    check("attn.f32.cross.o", o, U.from_bn_s_d(ref, b, nq), literal=True, max_abs_tol=1e-4, mean_rel_tol=1e-5)
    # rotary through ops.attention on fp32 tensors
    s = 96
    q, k, v, do = U.make_qkv(1, s, 4, 2, d, seed=9, dtype=torch.float32)
    cu = U.make_cu(1, s, (40,))
    pos = U.position_ids_from_cu(cu, s)
    tabs = oracle.rotary_tables(d, s, 10000, torch.float32)
    qr, kr = oracle.apply_rotary(U.to_sbnd(q, 1, s), U.to_sbnd(k, 1, s), tabs, pos.view(s, 1), pos.view(s, 1))
    ref = U.oracle_attention(qr.permute(1, 0, 2, 3).reshape(s, 4, d), kr.permute(1, 0, 2, 3).reshape(s, 2, d), v, cu, 1, s, True, scale)
    o = ops.attention(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), None, True, scale,
                      rotary=(tabs.cos.to(DEV), tabs.sin.to(DEV), pos.to(DEV), pos.to(DEV)))
    check("attn.f32.rotary.o", o, ref, literal=True, max_abs_tol=1e-4, mean_rel_tol=1e-5)
