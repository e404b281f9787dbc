"""Pins the oracle's floating-point functions against library routines, closed forms,
brute force and invariants (none of these re-types the oracle's own formula)."""

import math

import pytest
import torch
import torch.nn.functional as F

import oracle


def _cu(b, s, cuts=()):
    cu = sorted(set([i * s for i in range(b + 1)]) | set(cuts))
    return torch.tensor(cu, dtype=torch.int32)


# ------------------------------------------------------------------ masked softmax ---------
def test_masked_softmax_invariants():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 3, 8, 8, generator=g)
    mask = oracle.cumulative_seq_lengths_to_dense_attention_mask(_cu(2, 8, (3, 13)), 8, True)
    p = oracle.masked_softmax(x, mask)
    assert torch.allclose(p.sum(-1), torch.ones(2, 3, 8), atol=1e-6)
    assert torch.all(p[mask.expand_as(p)] == 0)          # exp(-10000 - max) underflows to exactly 0
    ref = torch.softmax(torch.where(mask, torch.tensor(float("-inf")), x), -1)
    assert torch.allclose(p, ref, atol=1e-7)
    # scale multiplies the scores before the fill
    p2 = oracle.masked_softmax(x, mask, scale=2.0)
    assert torch.allclose(p2, torch.softmax(torch.where(mask, torch.tensor(float("-inf")), 2 * x), -1), atol=1e-7)
    # fp32 softmax of bf16 scores: result dtype bf16, value = rounded fp32 softmax
    xb = x.bfloat16()
    pb = oracle.masked_softmax(xb, mask, softmax_in_fp32=True)
    assert pb.dtype == torch.bfloat16
    assert torch.equal(pb, torch.softmax(torch.where(mask, torch.tensor(float("-inf")), xb.float()), -1).bfloat16())


# ------------------------------------------------------------------ attention core ---------
def _sdpa_reference(q, k, v, mask, alpha):
    # q,k,v [s,b,n,d] -> library SDPA on [b,n,s,d]
    qq, kk, vv = (t.permute(1, 2, 0, 3) for t in (q, k, v))
    o = F.scaled_dot_product_attention(qq, kk, vv, attn_mask=~mask, scale=alpha)
    b, n, s, d = o.shape
    return o.reshape(b * n, s, d)


@pytest.mark.parametrize("causal", [True, False])
def test_attention_matches_library_sdpa(causal):
    g = torch.Generator().manual_seed(1)
    s, b, n, d = 16, 2, 3, 8
    q, k, v = (torch.randn(s, b, n, d, generator=g, dtype=torch.float64) for _ in range(3))
    cu = _cu(b, s, (5, 11, 20))
    alpha = 1 / math.sqrt(d)
    out = oracle.multi_head_attention(q, k, v, cu, causal, alpha)
    mask = oracle.cumulative_seq_lengths_to_dense_attention_mask(cu, s, causal)
    assert torch.allclose(out, _sdpa_reference(q, k, v, mask, alpha), atol=1e-12)


def test_attention_brute_force_loops():
    g = torch.Generator().manual_seed(2)
    s, b, n, d = 6, 1, 2, 4
    q, k, v = (torch.randn(s, b, n, d, generator=g, dtype=torch.float64) for _ in range(3))
    cu = torch.tensor([0, 2, 6], dtype=torch.int32)
    out = oracle.multi_head_attention(q, k, v, cu, True, 0.5)
    doc = [0, 0, 1, 1, 1, 1]
    for h in range(n):
        for i in range(s):
            ws, acc = [], [0.0] * d
            for j in range(s):
                if doc[i] == doc[j] and j <= i:
                    ws.append((j, math.exp(0.5 * sum(float(q[i, 0, h, t]) * float(k[j, 0, h, t]) for t in range(d)))))
            z = sum(wt for _, wt in ws)
            for j, wt in ws:
                for t in range(d):
                    acc[t] += wt / z * float(v[j, 0, h, t])
            assert torch.allclose(out[h, i], torch.tensor(acc, dtype=torch.float64), atol=1e-12)


def test_attention_gradcheck_and_gqa_reduction():
    g = torch.Generator().manual_seed(3)
    s, b, nq, nkv, d = 5, 1, 4, 2, 4
    q = torch.randn(s, b, nq, d, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(s, b, nkv, d, generator=g, dtype=torch.float64, requires_grad=True)
    v = torch.randn(s, b, nkv, d, generator=g, dtype=torch.float64, requires_grad=True)
    cu = torch.tensor([0, 2, 5], dtype=torch.int32)

    def f(q_, k_, v_):
        return oracle.multi_head_attention(q_, oracle.repeat_kv(k_, 2), oracle.repeat_kv(v_, 2), cu, True, 0.5)

    assert torch.autograd.gradcheck(f, (q, k, v), atol=1e-8)
    # GQA == MHA on explicitly repeated heads with the kv gradients summed over each group
    kr = torch.repeat_interleave(k.detach(), 2, dim=2).requires_grad_()
    vr = torch.repeat_interleave(v.detach(), 2, dim=2).requires_grad_()
    go = torch.randn(nq, s, d, generator=g, dtype=torch.float64)
    f(q, k, v).backward(go)
    oracle.multi_head_attention(q.detach(), kr, vr, cu, True, 0.5).backward(go)
    assert torch.allclose(k.grad, kr.grad.view(s, b, nkv, 2, d).sum(3), atol=1e-12)
    assert torch.allclose(v.grad, vr.grad.view(s, b, nkv, 2, d).sum(3), atol=1e-12)
    # kv head mapping: query head h reads kv head h // n_rep
    x = torch.arange(nkv).view(1, 1, nkv, 1).float()
    assert oracle.repeat_kv(x, 2).flatten().tolist() == [0, 0, 1, 1]


def test_attention_bf16_rounding_points():
    # scores are rounded to bf16 before the fp32 softmax; probabilities to bf16 before PV
    g = torch.Generator().manual_seed(4)
    s, b, n, d = 8, 1, 1, 16
    q, k, v = (torch.randn(s, b, n, d, generator=g).bfloat16() for _ in range(3))
    cu = _cu(1, s)
    out = oracle.multi_head_attention(q, k, v, cu, True, 0.25, softmax_in_fp32=True)
    assert out.dtype == torch.bfloat16
    scores = (0.25 * (q[:, 0, 0].float() @ k[:, 0, 0].float().T)).bfloat16()
    mask = torch.triu(torch.ones(s, s, dtype=torch.bool), 1)
    p = torch.softmax(scores.float().masked_fill(mask, -10000.0), -1).bfloat16()
    ref = (p.float() @ v[:, 0, 0].float()).bfloat16()
    assert (out[0].float() - ref.float()).abs().max() <= 2 ** -7  # one bf16 ulp at |x| < 2 (BLAS accumulation order)


# ------------------------------------------------------------------ rotary -----------------
def test_rotary_closed_form_and_invariants():
    g = torch.Generator().manual_seed(5)
    s, b, n, d = 10, 2, 3, 8
    tabs = oracle.rotary_tables(d, s, 10000, torch.float64)
    assert tabs.cos.dtype == torch.float64 and tabs.cos.shape == (s, d)
    q = torch.randn(s, b, n, d, generator=g, dtype=torch.float64)
    k = torch.randn(s, b, n, d, generator=g, dtype=torch.float64)
    qr, kr = oracle.apply_rotary(q, k, tabs)
    # textbook: pair (i, i + d/2) rotated by angle p * base^(-2i/d)
    for p in (0, 3, 9):
        for i in range(d // 2):
            th = p * 10000.0 ** (-2.0 * i / d)
            x0, x1 = float(q[p, 1, 2, i]), float(q[p, 1, 2, i + d // 2])
            assert abs(float(qr[p, 1, 2, i]) - (x0 * math.cos(th) - x1 * math.sin(th))) < 1e-5
            assert abs(float(qr[p, 1, 2, i + d // 2]) - (x1 * math.cos(th) + x0 * math.sin(th))) < 1e-5
    # reference invariants: arange ids == no ids; slicing commutes with ids
    ids = torch.arange(s).unsqueeze(1).expand(s, b)
    q2, k2 = oracle.apply_rotary(q, k, tabs, ids, ids)
    assert torch.equal(q2, qr) and torch.equal(k2, kr)
    q3, k3 = oracle.apply_rotary(q[1:], k[1:], tabs, ids[1:], ids[1:])
    assert torch.equal(q3, qr[1:]) and torch.equal(k3, kr[1:])
    # norm preservation and relative-position property
    assert torch.allclose(qr.norm(dim=-1), q.norm(dim=-1), atol=1e-6)
    qa, ka = oracle.apply_rotary(q[:1].expand(s, b, n, d).clone(), k[:1].expand(s, b, n, d).clone(), tabs)
    dots = torch.einsum("sbnd,tbnd->bnst", qa, ka)
    for m in range(1, s - 2):
        assert torch.allclose(dots[..., m, m + 2], dots[..., 0, 2], atol=1e-5)


def test_rotary_partial_and_table_dtype():
    g = torch.Generator().manual_seed(6)
    s, b, n, d = 7, 1, 2, 8
    tabs = oracle.rotary_tables(4, s, 10000, torch.bfloat16)
    assert tabs.cos.dtype == torch.bfloat16  # tables are rounded to the module dtype
    q = torch.randn(s, b, n, d, generator=g).bfloat16()
    qr, _ = oracle.apply_rotary(q, q, tabs)
    assert torch.equal(qr[..., 4:], q[..., 4:])
    assert not torch.equal(qr[1:, ..., :4], q[1:, ..., :4])


def test_rotary_complex_equals_rotate_half_under_permutation():
    s, b, n, d = 10, 2, 2, 8
    g = torch.Generator().manual_seed(7)
    q = torch.randn(s, b, n, d, generator=g)
    tabs = oracle.rotary_tables(d, s, 10000, torch.float32)
    base, _ = oracle.apply_rotary(q, q, tabs)
    perm = torch.cat((torch.arange(0, d, 2), torch.arange(1, d, 2)))  # interleaved -> halves
    qc, _ = oracle.apply_rotary_complex(q[..., torch.argsort(perm)], q[..., torch.argsort(perm)], d, s, 10000.0)
    assert torch.allclose(qc[..., perm], base, atol=1e-5)


# ------------------------------------------------------------------ norms / activations ----
def test_rms_norm_matches_library():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(4, 5, 32, generator=g)
    w = torch.randn(32, generator=g)
    assert torch.allclose(oracle.rms_norm(x, w, 1e-5), F.rms_norm(x, (32,), w, 1e-5), atol=1e-6)
    y = oracle.rms_norm(torch.randn(64, 512, generator=g), torch.ones(512))
    assert abs(float(y.std()) - 1.0) < 0.02  # unit-scale statistic
    xb = x.bfloat16()
    assert oracle.rms_norm(xb, w.bfloat16()).dtype == torch.bfloat16


def test_swiglu_closed_form_gradient():
    g = torch.Generator().manual_seed(9)
    a = torch.randn(6, 11, generator=g, dtype=torch.float64, requires_grad=True)
    gate = torch.randn(6, 11, generator=g, dtype=torch.float64, requires_grad=True)
    do = torch.randn(6, 11, generator=g, dtype=torch.float64)
    out = oracle.swiglu(a, gate)
    assert torch.allclose(out, a / (1 + torch.exp(-a)) * gate, atol=1e-12)
    out.backward(do)
    da, dg = oracle.swiglu_grad(a.detach(), gate.detach(), do)
    assert torch.allclose(a.grad, da, atol=1e-12) and torch.allclose(gate.grad, dg, atol=1e-12)
    assert torch.autograd.gradcheck(oracle.swiglu, (a, gate), atol=1e-8)


# ------------------------------------------------------------------ cached decode ----------
def _tiny_model(spec, n_layers, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    H, d = spec.hidden_size, spec.head_dim
    I = 24

    def w(*shape):
        return torch.randn(*shape, generator=g) * 0.2

    layers = []
    for _ in range(n_layers):
        layers.append({
            "input_layernorm.weight": torch.ones(H), "post_attention_layernorm.weight": torch.ones(H),
            "self_attention.query.weight": w(H, H), "self_attention.key.weight": w(spec.n_kv * d, H),
            "self_attention.value.weight": w(spec.n_kv * d, H), "self_attention.dense.weight": w(H, H),
            "mlp.dense_in.weight": w(I, H), "mlp.siglu_weight.weight": w(I, H), "mlp.dense_out.weight": w(H, I),
        })
    return {"embedding.weight": w(vocab, H), "layers": layers, "final": {"norm.weight": torch.ones(H)},
            "lm_head.weight": w(vocab, H)}


def test_cached_generation_equals_uncached():
    spec = oracle.LayerSpec(hidden_size=16, num_attention_heads=4, num_kv_heads=2, qkv_in_one=False,
                            norm_type="rms", mlp_type="swiglu", rotary_base=10000, sequence_length=32)
    model = _tiny_model(spec, 2, 50, 10)
    prompt = [3, 7, 1, 9, 4]
    tok_u, log_u = oracle.generate_uncached(spec, model, prompt, 6)
    tok_c, log_c = oracle.generate_cached(spec, model, prompt, 6)
    assert tok_u == tok_c
    assert torch.allclose(log_u, log_c, atol=1e-5)


# ---- LM head + cross entropy (losses/cross_entropy.py:18-32, 58-88) -----------------------------------------
def test_cross_entropy_oracle_against_library_and_closed_forms():
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(3, 17, 50, generator=g, dtype=torch.float64)
    targets = torch.randint(0, 50, (3, 17), generator=g)
    weights = torch.rand(3, 17, generator=g, dtype=torch.float64)
    weights[0, :5] = 0
    loss, m = oracle.cross_entropy_loss(logits, targets, weights)
    lib = torch.nn.functional.cross_entropy(logits.reshape(-1, 50), targets.flatten(), reduction="none")
    assert torch.allclose(oracle.token_losses(logits.reshape(-1, 50), targets.flatten()), lib, rtol=1e-12)
    assert torch.allclose(loss, (lib * weights.flatten()).sum() / weights.sum(), rtol=1e-12)
    hits = (logits.reshape(-1, 50).argmax(-1) == targets.flatten()).double()
    mask = (weights.flatten() > 0).double()
    assert torch.allclose(m["accuracy"], (hits * mask).sum() / mask.sum())
    # uniform logits -> log V; a dominant target logit -> 0; ignore_index rows -> 0
    assert torch.allclose(oracle.token_losses(torch.zeros(2, 1000, dtype=torch.float64), torch.tensor([3, 9])),
                          torch.full((2,), math.log(1000.0), dtype=torch.float64))
    peaked = torch.zeros(1, 10, dtype=torch.float64)
    peaked[0, 4] = 100.0
    assert float(oracle.token_losses(peaked, torch.tensor([4]))) < 1e-12
    assert float(oracle.token_losses(torch.randn(1, 10, dtype=torch.float64), torch.tensor([-100]))) == 0.0
    # gradient closed form: d loss / d logits = w / sum(w) * (softmax - onehot); every row sums to zero
    x = logits.clone().requires_grad_()
    oracle.cross_entropy_loss(x, targets, weights)[0].backward()
    p = torch.softmax(logits.reshape(-1, 50), -1)
    p[torch.arange(51), targets.flatten()] -= 1.0
    want = (p * (weights.flatten() / weights.sum()).unsqueeze(-1)).reshape(3, 17, 50)
    assert torch.allclose(x.grad, want, rtol=1e-10, atol=1e-14)
    assert float(x.grad.sum(-1).abs().max()) < 1e-15
    small = torch.randn(4, 6, dtype=torch.float64, generator=g).requires_grad_()
    assert torch.autograd.gradcheck(lambda z: oracle.cross_entropy_loss(z, torch.tensor([0, 5, 2, 2]), torch.tensor([1.0, 0.5, 0.0, 2.0]))[0], (small,))
    # the head is a bias-free projection with weight [vocab, hidden]
    h, w = torch.randn(5, 8, dtype=torch.float64, generator=g), torch.randn(11, 8, dtype=torch.float64, generator=g)
    assert torch.allclose(oracle.lm_head(h, w), h @ w.t())
