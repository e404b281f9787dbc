"""GPU parity of the cross-entropy kernel, the chunked LM-head loss and the loss modules against the CPU oracle,
called through the C ABI.  Losses, log-sum-exp and gradients are fp32 arithmetic on the given logits: gates are
1e-5 relative on the fp32 outputs and the bf16 gates of tests/parity.py on gradients stored in bf16."""

import math
import types

import pytest
import torch

import oracle
from scaling_amd import ops
from scaling_amd.config import TransformerArchitectureConfig
from scaling_amd.layer import TransformerLayerIO
from scaling_amd.loss import CrossEntropyLoss, TransformerLMHead
from tests.parity import check

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(rows, vocab, dtype, seed, scale=3.0, pad=0):
    g = torch.Generator().manual_seed(seed)
    store = (torch.randn(rows, vocab + pad, generator=g) * scale).to(dtype)
    logits = store[:, :vocab]
    targets = torch.randint(0, vocab, (rows,), generator=g)
    weights = torch.rand(rows, generator=g) + 0.1
    return store, logits, targets, weights


def _oracle(logits, targets, row_scale):
    x = logits.float().clone().requires_grad_()
    losses = oracle.token_losses(x, targets)
    (losses * row_scale).sum().backward()
    return losses.detach(), x.grad, x.detach().argmax(-1)


# vocab sizes: one 128-bit vector per thread and less, several vectors per thread (register-resident row), the
# config-5 vocabulary, sizes that are not a multiple of the vector width and rows beyond the register path; more rows
# than compute units, so that a workgroup walks several rows (the next row staged through LDS at the large vocabularies)
@pytest.mark.parametrize("rows,vocab", [(7, 128), (33, 1000), (4, 8192), (12, 32000), (6, 128256), (5, 50257), (3, 262144), (2, 3),
                                        (600, 4096), (530, 50000), (777, 128256)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_cross_entropy_parity(rows, vocab, dtype):
    print(f"case cross_entropy rows={rows} vocab={vocab} dtype={dtype}", flush=True)
    _, logits, targets, weights = _case(rows, vocab, dtype, rows * 13 + vocab)
    if rows > 2:
        targets[1] = -100                                   # torch's ignore_index: zero loss, zero gradient
    row_scale = (weights / weights.sum()).float()
    ref_losses, ref_grad, ref_arg = _oracle(logits, targets, row_scale)
    lg = logits.to(DEV)
    dl = torch.empty_like(lg)
    losses, argmax, lse = ops.cross_entropy_forward(lg, targets.to(DEV), row_scale.to(DEV), dl, want_lse=True)
    torch.cuda.synchronize()
    assert torch.allclose(losses.cpu(), ref_losses, rtol=1e-5, atol=1e-5), (losses.cpu() - ref_losses).abs().max()
    assert torch.allclose(lse.cpu(), torch.logsumexp(logits.float(), -1), rtol=1e-5, atol=1e-5)
    assert torch.equal(argmax.cpu().long(), ref_arg)
    if dtype == torch.float32:
        assert torch.allclose(dl.cpu(), ref_grad, rtol=1e-4, atol=1e-7), (dl.cpu() - ref_grad).abs().max()
    else:
        check("cross_entropy.dlogits", dl, ref_grad)
    # the library routine on the same logits
    lib = torch.nn.functional.cross_entropy(logits.float(), targets, reduction="none")
    assert torch.allclose(losses.cpu(), lib, rtol=1e-5, atol=1e-5)
    # the forward-only launch (its own kernel and summation order) agrees; the in-place gradient is bit-identical
    l2, a2 = ops.cross_entropy_forward(lg, targets.to(DEV))
    assert torch.allclose(l2, losses, rtol=2e-6, atol=2e-6) and torch.equal(a2, argmax)
    assert torch.allclose(l2.cpu(), ref_losses, rtol=1e-5, atol=1e-5)
    inplace = lg.clone()
    ops.cross_entropy_forward(inplace, targets.to(DEV), row_scale.to(DEV), inplace)
    assert torch.equal(inplace, dl)


def test_cross_entropy_strided_rows_ties_and_closed_forms():
    print("case cross_entropy strided / ties / closed forms", flush=True)
    store, logits, targets, weights = _case(9, 4096, torch.bfloat16, 5, pad=64)
    logits[3, 100] = logits[3].max() + 1                    # unique maximum
    logits[4, 7] = logits[4, 900] = logits[4].max() + 1     # tie: the first index wins (torch.argmax on CPU)
    targets[4] = 900
    dev_store = store.to(DEV)
    lg = dev_store[:, :4096]
    assert lg.stride(0) == 4160
    losses, argmax = ops.cross_entropy_forward(lg, targets.to(DEV))
    ref_losses, _, ref_arg = _oracle(logits, targets, torch.ones(9))
    assert torch.allclose(losses.cpu(), ref_losses, rtol=1e-5, atol=1e-5)
    assert torch.equal(argmax.cpu().long(), ref_arg) and int(argmax[4]) == 7 and int(argmax[3]) == 100
    # uniform logits: loss = log V exactly, gradient = (1/V - onehot)
    v = 32000
    flat = torch.zeros(4, v, dtype=torch.float32, device=DEV)
    t = torch.tensor([0, 5, v - 1, 17], device=DEV)
    g = torch.empty_like(flat)
    losses, _ = ops.cross_entropy_forward(flat, t, None, g)
    assert torch.allclose(losses.cpu(), torch.full((4,), math.log(v)), rtol=1e-6)
    assert torch.allclose(g.sum(-1).cpu(), torch.zeros(4), atol=1e-5)
    assert abs(float(g[1, 5]) - (1.0 / v - 1.0)) < 1e-6 and abs(float(g[1, 6]) - 1.0 / v) < 1e-9
    # a dominant target logit: loss -> 0, gradient -> 0
    peaked = torch.zeros(2, 1024, dtype=torch.bfloat16, device=DEV)
    peaked[:, 3] = 60.0
    losses, argmax = ops.cross_entropy_forward(peaked, torch.tensor([3, 3], device=DEV))
    assert float(losses.abs().max()) < 1e-6 and argmax.tolist() == [3, 3]


def test_cross_entropy_autograd_and_module():
    print("case cross_entropy autograd / module", flush=True)
    b, s, vocab = 2, 37, 2000
    g = torch.Generator().manual_seed(3)
    act = (torch.randn(b, s, vocab, generator=g) * 2).bfloat16()
    targets = torch.randint(0, vocab, (b, s), generator=g)
    weights = (torch.rand(b, s, generator=g) > 0.3).float() * torch.rand(b, s, generator=g)
    batch = types.SimpleNamespace(target_token_ids=targets, loss_weights=weights)
    ar = act.float().clone().requires_grad_()
    ref_loss, ref_metrics = oracle.cross_entropy_loss(ar, targets, weights)
    (ref_loss * 1.7).backward()
    ag = act.to(DEV).requires_grad_()
    dev_batch = types.SimpleNamespace(target_token_ids=targets.to(DEV), loss_weights=weights.to(DEV))
    loss, metrics_ = CrossEntropyLoss()(TransformerLayerIO(activations=ag, position_ids=None), dev_batch)
    (loss * 1.7).backward()
    torch.cuda.synchronize()
    assert abs(loss.item() - ref_loss.item()) < 1e-5 * abs(ref_loss.item())
    assert abs(float(metrics_["accuracy"]) - float(ref_metrics["accuracy"])) < 1e-6
    check("cross_entropy_module.dlogits", ag.grad, ar.grad)
    # the reference's formula through the library routine (cross_entropy.py:24-30)
    lib = torch.nn.functional.cross_entropy(act.float().reshape(-1, vocab), targets.flatten(), reduction="none")
    lib_loss = torch.sum(lib * weights.flatten()) / weights.sum()
    assert abs(loss.item() - lib_loss.item()) < 1e-5 * abs(lib_loss.item())
    with pytest.raises(NotImplementedError):
        CrossEntropyLoss(umup_config=types.SimpleNamespace(enable=True))


@pytest.mark.parametrize("dtype,chunk", [(torch.bfloat16, 128), (torch.float32, 77), (torch.bfloat16, 4096)])
def test_linear_cross_entropy_matches_unfused_head_and_loss(dtype, chunk):
    print(f"case linear_cross_entropy dtype={dtype} chunk={chunk}", flush=True)
    rows, hidden, vocab = 300, 256, 1000
    g = torch.Generator().manual_seed(11)
    h = torch.randn(rows, hidden, generator=g).to(dtype)
    w = (torch.randn(vocab, hidden, generator=g) * 0.05).to(dtype)
    targets = torch.randint(0, vocab, (rows,), generator=g)
    weights = torch.rand(rows, generator=g)
    hr, wr = h.float().clone().requires_grad_(), w.float().clone().requires_grad_()
    # oracle: logits rounded to the model dtype as the reference's head produces them (lm_head.py:58), then the loss
    logits = oracle.lm_head(hr, wr)
    ref_loss, _ = oracle.cross_entropy_loss(logits, targets, weights)
    ref_loss.backward()
    hg, wg = h.to(DEV).requires_grad_(), w.to(DEV).requires_grad_()
    loss, argmax = ops.linear_cross_entropy(hg, wg, targets.to(DEV), weights.to(DEV), chunk_rows=chunk)
    loss.backward()
    torch.cuda.synchronize()
    tol = 1e-5 if dtype == torch.float32 else 2e-3       # bf16 logits: each is rounded once before the loss
    assert abs(loss.item() - ref_loss.item()) < tol * abs(ref_loss.item()), (loss.item(), ref_loss.item())
    if dtype == torch.float32:
        assert torch.allclose(hg.grad.cpu(), hr.grad, rtol=1e-3, atol=1e-7)
        assert torch.allclose(wg.grad.cpu(), wr.grad, rtol=1e-3, atol=1e-7)
    else:
        # gradients are O(1e-3): compare in relative terms (mean |diff| / mean |ref|), bf16 storage of dlogits
        for name, got, ref in (("dh", hg.grad, hr.grad), ("dw", wg.grad, wr.grad)):
            rel = float((got.float().cpu() - ref).abs().mean() / ref.abs().mean())
            print(f"[parity] linear_cross_entropy.{name}: mean_rel={rel:.3e}", flush=True)
            assert rel < 1e-2, (name, rel)


def test_lm_head_module_loss_equals_head_then_loss():
    print("case lm head module", flush=True)
    cfg = TransformerArchitectureConfig.from_dict(dict(vocab_size=512, hidden_size=128, num_layers=1, num_attention_heads=2,
                                                       precision="bfloat16", sequence_length=64, masked_softmax={"kernel": "hip"},
                                                       norm_type="rms", mlp_type="swiglu", mlp_factor=2.0))
    torch.manual_seed(0)
    head = TransformerLMHead(cfg, device=torch.device(DEV))
    assert list(head.state_dict().keys()) == ["linear.weight"] and head.linear.weight.shape == (512, 128)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 50, 128, generator=g).bfloat16().to(DEV)
    batch = types.SimpleNamespace(target_token_ids=torch.randint(0, 512, (2, 50), generator=g).to(DEV),
                                  loss_weights=torch.ones(2, 50, device=DEV))
    io = TransformerLayerIO(activations=x, position_ids=None)
    fused, m_fused = head.loss(io, batch, chunk_rows=32)
    unfused, m_unfused = CrossEntropyLoss()(head(io), batch)
    assert abs(fused.item() - unfused.item()) < 1e-5 * abs(unfused.item())
    assert float(m_fused["accuracy"]) == float(m_unfused["accuracy"])


def test_cross_entropy_full_size_properties():
    """Config-5 vocabulary at 2048 rows: rows of the gradient sum to zero, the loss of shifted logits is unchanged
    (softmax shift invariance), and the bf16 gradient matches a float64 evaluation on sampled rows."""
    print("case cross_entropy full size", flush=True)
    rows, vocab = 2048, 128256
    g = torch.Generator(device=DEV).manual_seed(0)
    logits = (torch.randn(rows, vocab, generator=g, device=DEV) * 2).bfloat16()
    targets = torch.randint(0, vocab, (rows,), generator=g, device=DEV)
    scale = torch.full((rows,), 1.0 / rows, device=DEV)
    dl = torch.empty_like(logits)
    losses, argmax = ops.cross_entropy_forward(logits, targets, scale, dl)
    sums = dl.float().sum(-1)
    assert float(sums.abs().max()) < 2e-5, float(sums.abs().max())       # bf16 rounding of 128256 terms of ~1e-9
    shifted = (logits.float() + 8.0).bfloat16()           # exact in bf16 only where |x| is small; compare in fp32
    l2, _ = ops.cross_entropy_forward(shifted.float(), targets)
    l1, _ = ops.cross_entropy_forward(shifted.float() - 8.0, targets)
    assert torch.allclose(l1, l2, rtol=1e-5, atol=1e-5)
    for r in (0, 777, rows - 1):
        x = logits[r].double().cpu()
        p = torch.softmax(x, -1)
        p[int(targets[r])] -= 1.0
        ref = (p / rows).float()
        check(f"cross_entropy.full.row{r}", dl[r].cpu(), ref)
        assert abs(float(losses[r]) - float(torch.logsumexp(x, -1) - x[int(targets[r])])) < 1e-4
        assert int(argmax[r]) == int(x.argmax())


def test_cross_entropy_edge_shapes_and_errors():
    print("case cross_entropy edges", flush=True)
    # a vocabulary of one: probability 1, loss 0, zero gradient
    one = torch.randn(4, 1, device=DEV)
    g = torch.empty_like(one)
    losses, argmax = ops.cross_entropy_forward(one, torch.zeros(4, dtype=torch.int64, device=DEV), None, g)
    assert float(losses.abs().max()) == 0.0 and argmax.tolist() == [0] * 4 and float(g.abs().max()) == 0.0
    # no rows
    empty = torch.empty(0, 128, device=DEV, dtype=torch.bfloat16)
    losses, argmax = ops.cross_entropy_forward(empty, torch.empty(0, dtype=torch.int64, device=DEV))
    assert losses.numel() == 0 and argmax.numel() == 0
    # fp16 logits through the register-resident kernel
    gen = torch.Generator().manual_seed(4)
    x = (torch.randn(9, 4096, generator=gen) * 3).half()
    t = torch.randint(0, 4096, (9,), generator=gen)
    dl = torch.empty(9, 4096, dtype=torch.float16, device=DEV)
    losses, argmax = ops.cross_entropy_forward(x.to(DEV), t.to(DEV), None, dl)
    ref = torch.nn.functional.cross_entropy(x.float(), t, reduction="none")
    assert torch.allclose(losses.cpu(), ref, rtol=1e-5, atol=1e-5) and torch.equal(argmax.cpu().long(), x.float().argmax(-1))
    p = torch.softmax(x.float(), -1)
    p[torch.arange(9), t] -= 1.0
    assert torch.allclose(dl.float().cpu(), p, atol=1e-3)
    # host-side checks
    with pytest.raises(AssertionError):
        ops.cross_entropy_forward(x.to(DEV).t(), t.to(DEV))                 # vocabulary dimension not contiguous
    with pytest.raises(RuntimeError):
        ops.cross_entropy_forward(x, t)                                       # CPU tensors: there is no CPU path
