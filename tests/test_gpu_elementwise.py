"""GPU parity of the bandwidth-bound kernels (RMSNorm, LayerNorm, SwiGLU, GELU, rotary) against the CPU oracle,
called through the C ABI."""

import os

import pytest
import torch

import oracle
from scaling_amd import _lib, ops
from tests.parity import check

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rand(gen, *shape, dtype=torch.bfloat16, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


@pytest.mark.parametrize("rows,hidden", [(2 * 128, 256), (37, 128), (1024, 4096), (19, 8192), (5, 1000 * 8), (64, 64), (7, 16384)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_parity(rows, hidden, dtype):
    print(f"case rmsnorm rows={rows} hidden={hidden} dtype={dtype}", flush=True)
    if hidden // (8 if dtype == torch.bfloat16 else 4) > 2048:
        pytest.skip("rows wider than 2048 vectors of 16 bytes are outside the kernels' range")
    g = torch.Generator().manual_seed(rows * 7 + hidden)
    x = _rand(g, rows, hidden, dtype=dtype)
    w = (1.0 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    dy = _rand(g, rows, hidden, dtype=dtype)
    xr = x.float().clone().requires_grad_()
    wr = w.float().clone().requires_grad_()
    ref = oracle.rms_norm(xr, wr, 1e-5)
    ref.backward(dy.float())
    xo = x.clone().requires_grad_()
    wo = w.clone().requires_grad_()
    ref_o = oracle.rms_norm(xo, wo, 1e-5)          # the reference's own operation order in `dtype`
    ref_o.backward(dy)

    xg = x.to(DEV).detach().requires_grad_()
    wg = w.to(DEV).detach().requires_grad_()
    y = ops.rms_norm(xg, wg, 1e-5)
    y.backward(dy.to(DEV))
    torch.cuda.synchronize()
    tol = dict(max_abs_tol=2e-2, mean_rel_tol=1e-3) if dtype == torch.bfloat16 else dict(max_abs_tol=1e-4, mean_rel_tol=1e-5)
    check("rmsnorm.y", y, ref, ref_o, literal_rel=True, **tol)
    check("rmsnorm.dx", xg.grad, xr.grad, xo.grad, literal_rel=True, **tol)
    check("rmsnorm.dw", wg.grad, wr.grad, wo.grad, literal_rel=True, **tol)


def test_rmsnorm_bwd_is_bit_reproducible():
    g = torch.Generator().manual_seed(3)
    x, w, dy = _rand(g, 3000, 4096).to(DEV), torch.ones(4096, dtype=torch.bfloat16, device=DEV), _rand(g, 3000, 4096).to(DEV)
    a = ops.rms_norm_backward(x, w, dy, 1e-5)
    b = ops.rms_norm_backward(x, w, dy, 1e-5)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


@pytest.mark.parametrize("shape", [(2, 128, 688), (3, 7, 5), (4, 1000, 14336), (1, 1, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_swiglu_parity(shape, dtype):
    print(f"case swiglu shape={shape} dtype={dtype}", flush=True)
    g = torch.Generator().manual_seed(sum(shape))
    a, gate, do = (_rand(g, *shape, dtype=dtype) for _ in range(3))
    ar, gr = a.float().clone().requires_grad_(), gate.float().clone().requires_grad_()
    ref = oracle.swiglu(ar, gr)
    ref.backward(do.float())
    ao, go = a.clone().requires_grad_(), gate.clone().requires_grad_()
    ref_o = oracle.swiglu(ao, go)
    ref_o.backward(do)
    ag, gg = a.to(DEV).detach().requires_grad_(), gate.to(DEV).detach().requires_grad_()
    out = ops.swiglu(ag, gg)
    out.backward(do.to(DEV))
    torch.cuda.synchronize()
    tol = dict(max_abs_tol=1e-4, mean_rel_tol=1e-5) if dtype == torch.float32 else {}
    check("swiglu.out", out, ref, ref_o, literal_rel=True, **tol)
    check("swiglu.da", ag.grad, ar.grad, ao.grad, literal_rel=True, **tol)
    check("swiglu.dgate", gg.grad, gr.grad, go.grad, literal_rel=True, **tol)
    # closed-form gradient of the oracle agrees with what the kernel returns
    da_cf, dg_cf = oracle.swiglu_grad(a.float(), gate.float(), do.float())
    check("swiglu.da(closed form)", ag.grad, da_cf, ao.grad, literal_rel=True, **tol)


@pytest.mark.parametrize("seq,batch,heads,dim,rot", [(17, 2, 4, 16, 16), (10, 7, 1, 2, 2), (10, 2, 2, 8, 8),
                                                      (64, 2, 8, 128, 128), (33, 1, 3, 64, 32), (16, 2, 2, 128, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("with_ids", [True, False])
def test_rotary_parity(seq, batch, heads, dim, rot, dtype, with_ids):
    print(f"case rotary s={seq} b={batch} n={heads} d={dim} rot={rot} {dtype} ids={with_ids}", flush=True)
    g = torch.Generator().manual_seed(seq + dim)
    tabs = oracle.rotary_tables(rot, seq, 10000, dtype)
    q = _rand(g, seq, batch, heads, dim, dtype=dtype)
    if with_ids:
        ids = torch.randint(0, seq, (seq, batch), generator=g)
    else:
        ids = None
    hi = oracle.RotaryTables(tabs.cos.float(), tabs.sin.float(), rot)   # same (rounded) table values, fp32 arithmetic
    ref, _ = oracle.apply_rotary(q.float(), q.float(), hi, ids, ids)
    ref_o, _ = oracle.apply_rotary(q, q, tabs, ids, ids)
    # kernel layout: tokens = (b s)
    x = q.permute(1, 0, 2, 3).reshape(batch * seq, heads, dim).contiguous().to(DEV)
    pid = None if ids is None else ids.transpose(0, 1).reshape(-1).contiguous().to(DEV)
    out = ops.rotary_embedding(x, tabs.cos.to(DEV), tabs.sin.to(DEV), pid, seq_len_for_null_ids=seq)
    torch.cuda.synchronize()
    got = out.view(batch, seq, heads, dim).permute(1, 0, 2, 3)
    tol = dict(max_abs_tol=1e-5, mean_rel_tol=1e-6) if dtype == torch.float32 else {}
    check("rotary.out", got, ref, ref_o, literal_rel=True, **tol)
    if rot < dim:
        assert torch.equal(got[..., rot:].cpu(), q[..., rot:])


def test_rotary_reference_invariants_and_backward():
    g = torch.Generator().manual_seed(11)
    seq, batch, heads, dim = 17, 2, 4, 16
    tabs = oracle.rotary_tables(dim, seq, 10000, torch.bfloat16)
    cos, sin = tabs.cos.to(DEV), tabs.sin.to(DEV)
    x = _rand(g, batch * seq, heads, dim).to(DEV)
    ids = torch.arange(seq).repeat(batch).to(DEV)
    a = ops.rotary_embedding(x, cos, sin, None, seq_len_for_null_ids=seq)
    b = ops.rotary_embedding(x, cos, sin, ids)
    assert torch.equal(a, b)                       # arange ids == no ids
    xs = x.view(batch, seq, heads, dim)[:, 1:].reshape(-1, heads, dim)
    ids_s = ids.view(batch, seq)[:, 1:].reshape(-1).contiguous()
    c = ops.rotary_embedding(xs, cos, sin, ids_s)
    assert torch.equal(c.view(batch, seq - 1, heads, dim), a.view(batch, seq, heads, dim)[:, 1:])
    # backward == rotation by the negative angle == autograd of the oracle
    xr = x.float().cpu().view(batch, seq, heads, dim).permute(1, 0, 2, 3).clone().requires_grad_()
    hi = oracle.RotaryTables(tabs.cos.float(), tabs.sin.float(), dim)
    out_r, _ = oracle.apply_rotary(xr, xr.detach(), hi)
    go = _rand(g, seq, batch, heads, dim)
    out_r.backward(go.float())
    xg = x.clone().requires_grad_()
    out = ops.rotary_embedding(xg, cos, sin, ids)
    out.backward(go.permute(1, 0, 2, 3).reshape(batch * seq, heads, dim).contiguous().to(DEV))
    torch.cuda.synchronize()
    check("rotary.dx", xg.grad.view(batch, seq, heads, dim).permute(1, 0, 2, 3), xr.grad)


@pytest.mark.parametrize("seq,batch,heads,dim", [(10, 2, 2, 8), (17, 7, 4, 16), (64, 2, 8, 128)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rotary_complex_parity(seq, batch, heads, dim, dtype):
    print(f"case rotary_complex s={seq} b={batch} n={heads} d={dim} {dtype}", flush=True)
    from scaling_amd.config import RotaryConfig
    from scaling_amd.nn import RotaryEmbeddingComplex
    g = torch.Generator().manual_seed(seq * dim)
    q = _rand(g, seq, batch, heads, dim, dtype=dtype)
    k = _rand(g, seq, batch, heads, dim, dtype=dtype)
    ids = torch.randint(0, seq, (seq, batch), generator=g)
    ref_q, ref_k = oracle.apply_rotary_complex(q.float(), k.float(), dim, seq, 10000.0, ids, ids)
    refo_q, _ = oracle.apply_rotary_complex(q, k, dim, seq, 10000.0, ids, ids)     # reference: fp32 math, cast back
    mod = RotaryEmbeddingComplex(RotaryConfig(dimensions=dim, max_seq_length=seq, base=10000), torch.device(DEV))
    got_q, got_k = mod(q.to(DEV), k.to(DEV), ids.to(DEV), ids.to(DEV))
    torch.cuda.synchronize()
    tol = dict(max_abs_tol=1e-5, mean_rel_tol=1e-6) if dtype == torch.float32 else {}
    check("rotary_complex.q", got_q, ref_q, refo_q, literal_rel=True, **tol)
    check("rotary_complex.k", got_k, ref_k, literal_rel=True, **tol)
    # no ids == arange ids (the reference's invariant), and the backward is the inverse rotation
    a, _ = mod(q.to(DEV), k.to(DEV))
    ar = torch.arange(seq).unsqueeze(1).expand(seq, batch).contiguous().to(DEV)
    b_, _ = mod(q.to(DEV), k.to(DEV), ar, ar)
    assert torch.equal(a, b_)
    xr = q.float().clone().requires_grad_()
    out_r, _ = oracle.apply_rotary_complex(xr, xr.detach(), dim, seq, 10000.0, ids, ids)
    go = _rand(g, seq, batch, heads, dim, dtype=dtype)
    out_r.backward(go.float())
    xg = q.to(DEV).detach().requires_grad_()
    out_g, _ = mod(xg, k.to(DEV), ids.to(DEV), ids.to(DEV))
    out_g.backward(go.to(DEV))
    torch.cuda.synchronize()
    check("rotary_complex.dx", xg.grad, xr.grad, literal_rel=True, **tol)


@pytest.mark.parametrize("rows,hidden", [(2 * 128, 256), (37, 128), (1024, 4096), (19, 8192), (5, 1000 * 8), (64, 64), (300, 16)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("with_bias", [True, False])
def test_layernorm_parity(rows, hidden, dtype, with_bias):
    print(f"case layernorm rows={rows} hidden={hidden} dtype={dtype} bias={with_bias}", flush=True)
    g = torch.Generator().manual_seed(rows * 11 + hidden)
    x = (_rand(g, rows, hidden, dtype=torch.float32) + 0.5).to(dtype)       # non-zero mean
    w = (1.0 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    b = (0.1 * torch.randn(hidden, generator=g)).to(dtype) if with_bias else None
    dy = _rand(g, rows, hidden, dtype=dtype)

    def run(cast):
        xs, ws = cast(x).clone().requires_grad_(), cast(w).clone().requires_grad_()
        bs = cast(b).clone().requires_grad_() if with_bias else None
        y = oracle.layer_norm(xs, ws, bs, 1e-5)
        y.backward(cast(dy))
        return y, xs.grad, ws.grad, (bs.grad if with_bias else None)

    ref = run(lambda t: t.float())
    ref_o = run(lambda t: t)                       # torch's own layer_norm in `dtype`
    xg, wg = x.to(DEV).requires_grad_(), w.to(DEV).requires_grad_()
    bg = b.to(DEV).requires_grad_() if with_bias else None
    y = ops.layer_norm(xg, wg, bg, 1e-5)
    y.backward(dy.to(DEV))
    torch.cuda.synchronize()
    tol = dict(max_abs_tol=2e-2, mean_rel_tol=1e-3) if dtype == torch.bfloat16 else dict(max_abs_tol=1e-4, mean_rel_tol=1e-5)
    check("layernorm.y", y, ref[0], ref_o[0], literal_rel=True, **tol)
    check("layernorm.dx", xg.grad, ref[1], ref_o[1], literal_rel=True, **tol)
    check("layernorm.dw", wg.grad, ref[2], ref_o[2], literal_rel=True, **tol)
    if with_bias:
        check("layernorm.db", bg.grad, ref[3], ref_o[3], literal_rel=True, **tol)


@pytest.mark.parametrize("rows,hidden", [(1024, 4096), (19, 8192), (5, 8000), (3000, 2048), (37, 128)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_layernorm_saved_statistics_and_recomputed_backward_agree(rows, hidden, dtype):
    """The backward runs with the statistics the forward saved (what the autograd function does) or
    recomputes them when none are passed: both must match the oracle, and the saved statistics are the row
    mean and 1 / sqrt(biased variance + eps) (torch.native_layer_norm's second and third results)."""
    print(f"case layernorm stats rows={rows} hidden={hidden} dtype={dtype}", flush=True)
    g = torch.Generator().manual_seed(rows + 3 * hidden)
    x = (_rand(g, rows, hidden, dtype=torch.float32) * 1.5 - 2.0).to(dtype)
    w = (1.0 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    b = (0.1 * torch.randn(hidden, generator=g)).to(dtype)
    dy = _rand(g, rows, hidden, dtype=dtype)
    xr, wr, br = x.float().requires_grad_(), w.float().requires_grad_(), b.float().requires_grad_()
    oracle.layer_norm(xr, wr, br, 1e-5).backward(dy.float())
    _, mean_ref, rstd_ref = torch.native_layer_norm(x.float(), [hidden], w.float(), b.float(), 1e-5)

    xg, wg, bg, dyg = x.to(DEV), w.to(DEV), b.to(DEV), dy.to(DEV)
    y, stats = ops.layer_norm_forward(xg, wg, bg, 1e-5, save_stats=True)
    assert torch.equal(y, ops.layer_norm_forward(xg, wg, bg, 1e-5))
    assert stats.shape == (2, rows) and stats.dtype == torch.float32
    assert torch.allclose(stats[0].cpu(), mean_ref.view(-1), rtol=1e-5, atol=1e-6)
    assert torch.allclose(stats[1].cpu(), rstd_ref.view(-1), rtol=1e-5, atol=0)
    tol = dict(max_abs_tol=2e-2, mean_rel_tol=1e-3) if dtype == torch.bfloat16 else dict(max_abs_tol=1e-4, mean_rel_tol=1e-5)
    for name, st in (("saved", stats), ("recomputed", None)):
        dx, dw, db = ops.layer_norm_backward(xg, wg, dyg, 1e-5, True, st)
        torch.cuda.synchronize()
        check(f"layernorm[{name}].dx", dx, xr.grad, literal_rel=True, **tol)
        check(f"layernorm[{name}].dw", dw, wr.grad, literal_rel=True, **tol)
        check(f"layernorm[{name}].db", db, br.grad, literal_rel=True, **tol)
    # half of a pair is refused
    lib = _lib.load()
    ws = torch.empty(lib.mi_layernorm_bwd_workspace_bytes(rows, hidden) // 4, dtype=torch.float32, device=DEV)
    dx = torch.empty_like(xg)
    rc = lib.mi_layernorm_bwd(xg.data_ptr(), wg.data_ptr(), dyg.data_ptr(), stats[0].data_ptr(), None, dx.data_ptr(),
                              dx.data_ptr(), None, ws.data_ptr(), ws.numel() * 4, rows, hidden, 1e-5,
                              _lib.dtype_code(dtype), torch.cuda.current_stream().cuda_stream)
    assert rc == -1 and "mean and rstd" in lib.mi_last_error().decode()   # MI_E_NULL


@pytest.mark.parametrize("shape", [(2, 128, 1024), (3, 7, 5), (4, 1000, 4096), (1, 1, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_gelu_parity(shape, dtype):
    print(f"case gelu shape={shape} dtype={dtype}", flush=True)
    g = torch.Generator().manual_seed(sum(shape) + 1)
    x, dy = (_rand(g, *shape, dtype=dtype, scale=2.0) for _ in range(2))
    xr = x.float().clone().requires_grad_()
    ref = torch.nn.functional.gelu(xr)             # the reference's activation (activation_function.py:13-14)
    ref.backward(dy.float())
    xo = x.clone().requires_grad_()
    ref_o = torch.nn.functional.gelu(xo)
    ref_o.backward(dy)
    xg = x.to(DEV).requires_grad_()
    y = ops.gelu(xg)
    y.backward(dy.to(DEV))
    torch.cuda.synchronize()
    tol = dict(max_abs_tol=1e-5, mean_rel_tol=1e-5) if dtype == torch.float32 else dict(max_abs_tol=2e-2, mean_rel_tol=1e-3)
    check("gelu.y", y, ref, ref_o, literal_rel=True, **tol)
    check("gelu.dx", xg.grad, xr.grad, xo.grad, literal_rel=True, **tol)
    # closed-form spot values: gelu(0) = 0, gelu'(0) = 0.5, gelu(x) -> x for large x
    pts = torch.tensor([0.0, 10.0, -10.0, 1.0], device=DEV)
    assert torch.allclose(ops.gelu_forward(pts), torch.tensor([0.0, 10.0, 0.0, 0.8413447], device=DEV), atol=1e-6)
    assert torch.allclose(ops.gelu_backward(pts, torch.ones_like(pts))[:1], torch.tensor([0.5], device=DEV), atol=1e-7)


def test_layernorm_and_gelu_mlp_reproduce_the_reference_golden(golden_dir):
    """fp32 LayerNorm and GELU-MLP kernels on the activations held by the reference's own test-suite
    (tests/transformer/files/backward_compatibility_checkpoint, gate 3e-3 in test_backwards_compatibility.py:175)."""
    d = os.path.join(golden_dir, "backward_compatibility")
    gt = torch.load(os.path.join(d, "ground_truth.pt"), weights_only=True)
    sd = torch.load(os.path.join(d, "state_dict.pt"), weights_only=True)
    dev = lambda k: sd[k].to(DEV)
    gt = {k: (v.detach() if torch.is_tensor(v) else v) for k, v in gt.items()}
    h0 = gt["hidden_states_embedding"].to(DEV)
    ln1 = ops.layer_norm(h0, dev("transformer.layer0.input_layernorm.weight"), dev("transformer.layer0.input_layernorm.bias"), 1e-5)
    assert float((ln1.cpu() - gt["hidden_states_input_layernorm"]).abs().max()) < 1e-5
    att = gt["hidden_states_attention"].to(DEV)
    ln2 = ops.layer_norm(att, dev("transformer.layer0.post_attention_layernorm.weight"),
                         dev("transformer.layer0.post_attention_layernorm.bias"), 1e-5)
    assert float((ln2.cpu() - gt["hidden_states_post_attention_layernorm"]).abs().max()) < 1e-4
    # mlp block: residual + dense_out(gelu(dense_in(ln2)))
    h = torch.nn.functional.linear(ln2, dev("transformer.layer0.mlp.dense_h_to_4h.weight"), dev("transformer.layer0.mlp.dense_h_to_4h.bias"))
    h = torch.nn.functional.linear(ops.gelu(h), dev("transformer.layer0.mlp.dense_4h_to_h.weight"), dev("transformer.layer0.mlp.dense_4h_to_h.bias"))
    assert float(((att + h).cpu() - gt["hidden_states_mlp"]).abs().max()) < 1e-4
    fin = ops.layer_norm(gt["hidden_states_layer0"].to(DEV), dev("transformer.norm.weight"), dev("transformer.norm.bias"), 1e-5)
    assert float((fin.cpu() - gt["hidden_states_norm"]).abs().max()) < 1e-3


@pytest.mark.parametrize("rows,hidden", [(32, 4096), (5, 256), (33, 8192)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_add_rmsnorm_equals_separate_add_and_norm(rows, hidden, dtype):
    """The fused residual add + RMSNorm of the decode loop is bit-identical to the tensor add followed by the norm
    kernel (the sum is rounded to the tensor dtype before it is normalised), and in-place sums are allowed."""
    print(f"case add_rmsnorm rows={rows} hidden={hidden} dtype={dtype}", flush=True)
    g = torch.Generator().manual_seed(rows + hidden)
    x, r = _rand(g, rows, hidden, dtype=dtype).to(DEV), _rand(g, rows, hidden, dtype=dtype).to(DEV)
    w = (1.0 + 0.1 * torch.randn(hidden, generator=g)).to(dtype).to(DEV)
    total, y = ops.add_rms_norm(x, r, w, 1e-5)
    want_total = x + r
    assert torch.equal(total, want_total)
    assert torch.equal(y, ops.rms_norm_forward(want_total, w, 1e-5))
    ref = oracle.rms_norm((x.float() + r.float()).to(dtype).float().cpu(), w.float().cpu(), 1e-5)
    check("add_rmsnorm.y", y, ref, max_abs_tol=1e-5 if dtype == torch.float32 else 2e-2,
          mean_rel_tol=1e-5 if dtype == torch.float32 else 1e-3)


def test_empty_tensors_pass_through_every_elementwise_op():
    """No rows / no tokens is not an error: outputs of the input's shape, zero parameter gradients, no launch."""
    w = torch.ones(256, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    b = torch.zeros(256, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    x = torch.zeros(0, 256, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    for y in (ops.rms_norm(x, w, 1e-5), ops.layer_norm(x, w, b, 1e-5), ops.swiglu(x, x.clone()), ops.gelu(x)):
        assert y.shape == x.shape
        y.sum().backward()
    assert x.grad.shape == x.shape and float(w.grad.abs().sum()) == 0.0 and float(b.grad.abs().sum()) == 0.0
    total, normed = ops.add_rms_norm(x.detach(), x.detach(), w.detach(), 1e-5)
    assert total.shape == normed.shape == x.shape
    q = torch.zeros(0, 4, 64, dtype=torch.bfloat16, device=DEV)
    tables = torch.zeros(16, 64, dtype=torch.bfloat16, device=DEV)
    assert ops.rotary_embedding(q, tables, tables, torch.zeros(0, dtype=torch.int64, device=DEV)).shape == q.shape
