"""Forward + backward parity at the benchmarked shapes.

The dense oracle cannot hold 32 heads x 8192^2 scores, but heads are independent: the kernels run the whole
workload (all heads, the launch shape that is timed) and the oracle is evaluated in fp32 on KV-group slices of the
same tensors (the query heads of one KV head with that KV head), which pins o, dq of those heads and dk, dv of
that KV head (their sum over the group's query heads lies inside the slice)."""

import math

import pytest
import torch

import oracle
from scaling_amd import ops
from tests import attn_utils as U
from tests.parity import check

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _slice_reference(q, k, v, do, cu, b, s, heads, kvh, scale, dtype, rotary=None):
    """Oracle o, dq, dk, dv for query heads `heads` (all reading KV head `kvh`); rotary = (tables, position ids)
    applies the oracle's rotary to q and k first, so the gradients are those of the unrotated inputs."""
    qs, ks, vs = q[:, heads].to(dtype).clone().requires_grad_(), k[:, kvh:kvh + 1].to(dtype).clone().requires_grad_(), \
        v[:, kvh:kvh + 1].to(dtype).clone().requires_grad_()
    q4, k4, v4 = U.to_sbnd(qs, b, s), U.to_sbnd(ks, b, s), U.to_sbnd(vs, b, s)
    if rotary is not None:
        tabs, pos = rotary
        ids = pos.view(b, s).transpose(0, 1)
        t = oracle.RotaryTables(tabs.cos.to(dtype), tabs.sin.to(dtype), tabs.dim)
        q4, k4 = oracle.apply_rotary(q4, k4, t, ids, ids)
    n_rep = len(heads)
    out = oracle.multi_head_attention(q4, oracle.repeat_kv(k4, n_rep), oracle.repeat_kv(v4, n_rep), cu, True, scale,
                                      softmax_in_fp32=True)
    o = U.from_bn_s_d(out, b, n_rep)
    o.backward(do[:, heads].to(dtype))
    return o.detach(), qs.grad, ks.grad[:, 0], vs.grad[:, 0]


@pytest.mark.timeout(600)
@pytest.mark.parametrize("precise", [False, True])
@pytest.mark.parametrize("name,b,s,nq,nkv,docs,rotary", [
    ("headline", 1, 8192, 32, 8, False, False),     # the workload of the headline metric
    ("config2", 4, 2048, 32, 32, False, False),
    ("config3", 1, 8192, 32, 8, True, True),        # packed documents of 256..2048 tokens, rotary base 500000
])
def test_attention_fwd_bwd_full_size_against_oracle_slices(name, b, s, nq, nkv, docs, rotary, precise):
    """precise=True is the accuracy mode (P and dS as hi + lo bf16 terms): held to the gates exactly as stated, except
    with rotary, where q and k are attended with after one rounding to bf16 (as the reference's bf16 path does) while
    the fp32 oracle rotates without rounding."""
    print(f"case full-size attention {name} precise={precise}", flush=True)
    d = 128
    q, k, v, do = U.make_qkv(b, s, nq, nkv, d, seed=200 + s + nq + nkv)
    cu = U.random_docs_cu(b * s, 256, 2048, seed=0) if docs else U.make_cu(b, s)
    scale = 1 / math.sqrt(d)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    rot_ref = None
    if rotary:
        pos = U.position_ids_from_cu(cu, b * s)
        tabs = oracle.rotary_tables(d, s, 500000, torch.bfloat16)
        rot_ref = (tabs, pos)
        o = ops.attention(qg, kg, vg, cu.to(DEV), None, True, scale, rotary=(tabs.cos.to(DEV), tabs.sin.to(DEV), pos.to(DEV), pos.to(DEV)),
                          precise=precise)
    else:
        o = ops.attention(qg, kg, vg, cu.to(DEV), None, True, scale, precise=precise)
    o.backward(do.to(DEV))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(o.float()).all()) and all(bool(torch.isfinite(t.grad.float()).all()) for t in (qg, kg, vg))
    n_rep = nq // nkv
    for kvh in (0, nkv - 1):
        heads = list(range(kvh * n_rep, (kvh + 1) * n_rep))
        ref = _slice_reference(q, k, v, do, cu, b, s, heads, kvh, scale, torch.float32, rot_ref)
        ref_o = _slice_reference(q, k, v, do, cu, b, s, heads, kvh, scale, torch.bfloat16, rot_ref)
        lit = precise and not rotary
        tag = f"{name}.precise" if precise else name
        check(f"{tag}.o[kv{kvh}]", o[:, heads], ref[0], ref_o[0], literal=lit, kind="rotary" if rotary else "o")
        check(f"{tag}.dq[kv{kvh}]", qg.grad[:, heads], ref[1], ref_o[1], literal=lit, kind="rotary" if rotary else "grad")
        check(f"{tag}.dk[kv{kvh}]", kg.grad[:, kvh], ref[2], ref_o[2], literal=lit, kind="rotary" if rotary else "grad")
        check(f"{tag}.dv[kv{kvh}]", vg.grad[:, kvh], ref[3], ref_o[3], literal=lit, kind="rotary" if rotary else "grad")


@pytest.mark.timeout(600)
def test_decode_attention_config5_shape():
    """Decode kernel at the config-5 per-layer shape: batch 32, context 4096 (+ ragged lengths), 32 query / 8 KV
    heads, head_dim 128, head-major cache of 4352 positions as the module allocates it."""
    print("case decode config-5 shape", flush=True)
    B, nq, nkv, d, max_ctx = 32, 32, 8, 128, 4352
    g = torch.Generator().manual_seed(55)
    q = torch.randn(B, nq, d, generator=g).bfloat16()
    kc = torch.randn(B, nkv, max_ctx, d, generator=g).bfloat16().transpose(1, 2)   # viewed [B, ctx, nkv, d]
    vc = torch.randn(B, nkv, max_ctx, d, generator=g).bfloat16().transpose(1, 2)
    lens = [4096] * 24 + [4097, 4351, 4352, 1, 63, 64, 65, 2049]
    ctx = torch.tensor(lens, dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    out = ops.decode_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), ctx.to(DEV), softmax_scale=scale)
    torch.cuda.synchronize()

    def ref_for(rows, dtype):
        outs = []
        for i in rows:
            n = lens[i]
            kk = oracle.repeat_kv(kc[i, :n].to(dtype).unsqueeze(1), nq // nkv)
            vv = oracle.repeat_kv(vc[i, :n].to(dtype).unsqueeze(1), nq // nkv)
            outs.append(oracle.multi_head_attention(q[i].to(dtype).view(1, 1, nq, d), kk, vv, torch.tensor([0, 1], dtype=torch.int32),
                                                    True, scale, softmax_in_fp32=True).view(nq, d))
        return torch.stack(outs)

    rows = list(range(B))
    check("decode.config5.o", out[rows], ref_for(rows, torch.float32), ref_for(rows, torch.bfloat16), kind="decode")


@pytest.mark.timeout(900)
def test_config5_shaped_module_graph_equals_eager_and_oracle_logits():
    """The config-5 architecture (hidden 4096, 32 query / 8 KV heads x 128, SwiGLU 14336, vocabulary 128256, RMSNorm,
    rotary base 500000) cut to 2 layers, batch 32 prompts of 4096 tokens: the HIP-graph decode loop produces the
    eager loop's tokens, and the prefill logits of two sequences match the oracle run on the same weights."""
    print("case config-5 shaped module", flush=True)
    from scaling_amd.config import TransformerArchitectureConfig
    from scaling_amd.inference import TransformerInferenceModule
    batch, prompt, steps = 32, 4096, 6
    cfg = TransformerArchitectureConfig.from_dict(dict(
        vocab_size=128256, hidden_size=4096, num_layers=2, num_attention_heads=32, attention_num_kv_heads=8,
        attention_qkv_in_one=False, norm_type="rms", mlp_type="swiglu", mlp_factor=3.5, attention_bias=False, mlp_bias=False,
        precision="bfloat16", sequence_length=prompt + steps + 16, rotary_embedding_base=500000, weight_tying=False,
        masked_softmax={"kernel": "hip", "softmax_in_fp32": True}))
    torch.manual_seed(0)
    model = TransformerInferenceModule(cfg, device=DEV, init_std=0.02)
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(1, cfg.vocab_size, (batch, prompt), generator=g)
    eager, logits = model.generate(steps, ids)
    graphed = model.generate_graph(steps, ids)
    assert graphed == eager
    # oracle: prefill of two of the sequences, last position only, on the same (bf16-valued) weights: in fp32 (the
    # target) and in the reference's bf16 operation order (the floor)
    def oracle_last_logits(row, dtype):
        spec = oracle.LayerSpec(hidden_size=4096, num_attention_heads=32, num_kv_heads=8, qkv_in_one=False, norm_type="rms",
                                mlp_type="swiglu", layernorm_epsilon=cfg.layernorm.layernorm_epsilon, rotary_base=500000,
                                sequence_length=cfg.sequence_length, causal=True, softmax_in_fp32=True, dtype=dtype)
        sd = {k_: v_.detach().cpu().to(dtype) for k_, v_ in model.state_dict().items()}
        layers = [{k_[len(f"_layers.{i + 1}."):]: v_ for k_, v_ in sd.items() if k_.startswith(f"_layers.{i + 1}.")} for i in range(2)]
        t = oracle.rotary_tables(128, cfg.sequence_length, 500000, torch.bfloat16)   # the module keeps bf16 tables
        tables = oracle.RotaryTables(t.cos.to(dtype), t.sin.to(dtype), t.dim)
        one = ids[row:row + 1]
        with torch.no_grad():
            h = torch.nn.functional.embedding(one, sd["_layers.0.embedding.weight"])
            cu = oracle.get_cumulative_seq_lengths(one)
            pos = oracle.get_position_ids(one)
            for w in layers:
                h = oracle.transformer_layer(spec, w, h, cu, pos, tables=tables)
            h = oracle.final_norm(spec, {"norm.weight": sd["_layers.3.norm.weight"]}, h[:, -1:])
            return torch.nn.functional.linear(h, sd["_layers.4.linear.weight"])[0, 0]

    for row in (0, batch - 1):
        ref = oracle_last_logits(row, torch.float32)
        ref_o = oracle_last_logits(row, torch.bfloat16)
        check(f"config5.prefill_logits[row{row}]", logits[row, 0], ref, ref_o, module_level=True)


@pytest.mark.timeout(900)
def test_layer_config4_against_oracle_on_one_sequence():
    """Config-4 layer (batch 2 x 4096, hidden 4096, GQA 32/8, SwiGLU 14336): output and input gradient of one whole
    sequence against the oracle layer run on that sequence alone (batch rows are independent documents)."""
    print("case config-4 layer against oracle", flush=True)
    from scaling_amd import config as C
    from scaling_amd.layer import TransformerLayer, TransformerLayerIO
    cfg = C.TransformerArchitectureConfig.from_dict(dict(
        vocab_size=128, hidden_size=4096, num_layers=1, num_attention_heads=32, attention_num_kv_heads=8,
        attention_qkv_in_one=False, norm_type="rms", mlp_type="swiglu", mlp_factor=3.5, attention_bias=False, mlp_bias=False,
        precision="bfloat16", sequence_length=4096, rotary_embedding_base=500000,
        masked_softmax={"kernel": "hip", "softmax_in_fp32": True}, weight_tying=False))
    g = torch.Generator().manual_seed(2)

    def init(w):
        w.data.copy_((torch.randn(w.shape, generator=g) * 0.02).to(w.dtype))
        return w

    layer = TransformerLayer(cfg, layer_index=0, init_method=init, device=DEV)
    b, s = 2, 4096
    x = torch.randn(b, s, cfg.hidden_size, generator=g).bfloat16()
    dy = torch.randn(b, s, cfg.hidden_size, generator=g).bfloat16()
    pos = torch.arange(s).repeat(b, 1)
    cu = torch.arange(0, b * s + 1, s, dtype=torch.int32)
    xg = x.to(DEV).requires_grad_()
    out = layer(TransformerLayerIO(activations=xg, position_ids=pos.to(DEV), cumulative_seq_lengths=cu.to(DEV)))
    out.activations.backward(dy.to(DEV))
    torch.cuda.synchronize()

    row = 1

    def oracle_layer(dtype):
        spec = oracle.LayerSpec(hidden_size=4096, num_attention_heads=32, num_kv_heads=8, qkv_in_one=False, norm_type="rms",
                                mlp_type="swiglu", layernorm_epsilon=cfg.layernorm.layernorm_epsilon, rotary_base=500000,
                                sequence_length=4096, causal=True, softmax_in_fp32=True, dtype=dtype)
        w = {k_: v_.detach().cpu().to(dtype) for k_, v_ in layer.state_dict().items()}
        t = oracle.rotary_tables(128, 4096, 500000, torch.bfloat16)
        tables = oracle.RotaryTables(t.cos.to(dtype), t.sin.to(dtype), t.dim)
        xr = x[row:row + 1].to(dtype).clone().requires_grad_()
        y = oracle.transformer_layer(spec, w, xr, cu[:2], pos[:1], tables=tables)
        y.backward(dy[row:row + 1].to(dtype))
        return y.detach(), xr.grad

    ref, ref_o = oracle_layer(torch.float32), oracle_layer(torch.bfloat16)
    check("config4.layer.y", out.activations[row:row + 1], ref[0], ref_o[0], module_level=True)
    check("config4.layer.dx", xg.grad[row:row + 1], ref[1], ref_o[1], module_level=True)
