#!/usr/bin/env python3
"""Benchmark of the transformer-layer hot path on one MI355X.

Headline workload (`config.workload`): attention core forward + backward, GQA 32 query / 8 KV heads,
head_dim 128, one sequence of 8192 tokens, causal, bf16, fp32 softmax.  One step = one forward and
one backward pass over synthetic N(0,1) inputs already resident in HBM.  `value` is
14 * d * n_q * P / time (P = allowed (query, key) pairs per head), i.e. the algorithmic TFLOP/s.

The JSON line also carries
  roofline      the dominant kernel of the step, timed live with HIP events on the launch stream
  cpu_baseline  the reference's operation order (CPU oracle, plain torch) timed on the host cores
                on a bounded sample of the same workload
  extra         the other quantities of the metric: per-kernel attention times, config-2 / config-3
                attention, RMSNorm / SwiGLU / rotary GB/s at the config-4 sizes, decode-attention GB/s
                at the config-5 per-layer shape.
"""

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, vendor figure
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, vendor figure

# HBM bytes per launch of the attention kernels on the headline workload: rocprofv3 FETCH_SIZE and WRITE_SIZE
# (KiB per dispatch, one counter per run), scaled by what the same counters read for a plain 1 GiB device copy
# (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).  Summary and commands: profiles/attention_fwd_bwd_gqa32x8_d128_s8192_hbm_traffic.md
MEASURED_TRAFFIC_KIB = {
    "attn_fwd_kernel": 2.0 * 72101 + 66560,
    "attn_bwd_dkdv_kernel": 2.0 * 703245 + 32788,
    "attn_bwd_dq_kernel": 2.0 * 106432 + 65536,
}


def causal_pairs(cu):
    return sum((b - a) * (b - a + 1) // 2 for a, b in zip(cu[:-1], cu[1:]))


def time_gpu(fn, steps, warmup):
    """Average milliseconds per call, measured with events on the current stream."""
    import torch
    for _ in range(warmup):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def time_gpu_graph(fn, steps, warmup):
    """Average milliseconds per call with the calls replayed from one HIP graph, so that a launch that takes the
    host longer than the kernel takes the GPU (the 20-30 us bandwidth kernels) is still timed on the GPU side.
    Best of three replays; falls back to eager timing if the calls cannot be captured."""
    import torch
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(warmup, 2)):
                fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(steps):
                fn()
        best = float("inf")
        for _ in range(3):
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            start.record()
            graph.replay()
            stop.record()
            torch.cuda.synchronize()
            best = min(best, start.elapsed_time(stop) / steps)
        del graph
        return best
    except Exception as exc:  # noqa: BLE001 - any capture problem: measure eagerly instead
        print(f"[bench] graph timing unavailable ({type(exc).__name__}: {exc}); timing eagerly", file=sys.stderr)
        torch.cuda.synchronize()
        return time_gpu(fn, steps, warmup)


def random_docs_cu(total, lo, hi, seed):
    """Cumulative document lengths: lengths uniform in [lo, hi], the last one truncated so they sum to `total`."""
    import torch
    g = torch.Generator().manual_seed(seed)
    cu = [0]
    while cu[-1] < total:
        cu.append(min(total, cu[-1] + int(torch.randint(lo, hi + 1, (1,), generator=g))))
    return torch.tensor(cu, dtype=torch.int32)


def _rotary_tables(dim, max_seq, base, device):
    """cos / sin tables [max_seq, dim] in bf16 from the product's own RotaryEmbedding module."""
    import torch
    from scaling_amd.config import RotaryConfig
    from scaling_amd.nn import RotaryEmbedding
    return RotaryEmbedding(RotaryConfig(dimensions=dim, max_seq_length=max_seq, base=base), torch.device(device), torch.bfloat16).tables()


def attention_case(b, s, nq, nkv, d, cu_list, steps, warmup, seed=0, rotary=False):
    """Times forward, backward stages and the whole step for one attention workload."""
    import torch
    from scaling_amd import ops
    dev = "cuda"
    g = torch.Generator().manual_seed(seed)
    T = b * s
    q = torch.randn(T, nq, d, generator=g).bfloat16().to(dev)
    k = torch.randn(T, nkv, d, generator=g).bfloat16().to(dev)
    v = torch.randn(T, nkv, d, generator=g).bfloat16().to(dev)
    do = torch.randn(T, nq, d, generator=g).bfloat16().to(dev)
    cu = torch.tensor(cu_list, dtype=torch.int32, device=dev)
    scale = 1.0 / math.sqrt(d)
    pairs = causal_pairs(cu_list)
    rot = None
    if rotary:
        cos_tab, sin_tab = _rotary_tables(d, s, 500000, dev)
        pos = torch.zeros(T, dtype=torch.int64)
        for a_, b_ in zip(cu_list[:-1], cu_list[1:]):
            pos[a_:b_] = torch.arange(b_ - a_)
        pos = pos.to(dev)
        rot = (cos_tab, sin_tab, pos, pos)

    o, lse = ops.attention_forward(q, k, v, cu, None, True, scale)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    from scaling_amd import _lib
    ws = torch.empty(_lib.load().mi_attn_bwd_workspace_bytes_kv(T, T, nq, nkv, d) // 4, dtype=torch.float32, device=dev)
    bufs = (dq, dk, dv, ws)

    def fwd():
        ops.attention_forward(q, k, v, cu, None, True, scale)

    def fwd_rot():
        ops.attention_forward(q, k, v, cu, None, True, scale, rotary=rot)

    def bwd(flags=0):
        ops.attention_backward(do, q, k, v, o, lse, cu, None, True, scale, flags=flags, buffers=bufs)

    def step():
        fwd()
        bwd()

    res = {"pairs_per_head": pairs}
    res["ms_step"] = time_gpu(step, steps, warmup)
    res["ms_step_graph"] = time_gpu_graph(step, steps, warmup)
    res["ms_fwd"] = time_gpu(fwd, steps, warmup)
    res["ms_bwd_delta"] = time_gpu(lambda: bwd(16), steps, 1)
    res["ms_bwd_dkdv"] = time_gpu(lambda: bwd(32), steps, 1)
    res["ms_bwd_dq"] = time_gpu(lambda: bwd(64), steps, 1)
    if rot is not None:
        res["ms_fwd_fused_rotary"] = time_gpu(fwd_rot, steps, warmup)
        # training step with the rotary embedding as ops.attention runs it: k rotated by one stand-alone launch, q
        # while the forward kernel loads it (the rotated q is written out for the backward), dq and dk rotated back
        # inside the backward kernels
        cos_t, sin_t, pos_t, _ = rot

        def step_rotary():
            kr = ops._rotary_launch(k, cos_t, sin_t, pos_t, 0, False)
            o2, lse2, qr = ops.attention_forward(q, kr, v, cu, None, True, scale, rotary=(cos_t, sin_t, pos_t, None), return_rotated_q=True)
            ops.attention_backward(do, qr, kr, v, o2, lse2, cu, None, True, scale, buffers=bufs, rotary=rot)

        res["ms_step_with_rotary"] = time_gpu(step_rotary, steps, warmup)
        res["tflops_step_with_rotary"] = 14 * d * nq * pairs / (res["ms_step_with_rotary"] * 1e-3) / 1e12
    flops_unit = d * nq * pairs
    res["tflops_fwd"] = 4 * flops_unit / (res["ms_fwd"] * 1e-3) / 1e12
    res["tflops_step"] = 14 * flops_unit / (res["ms_step"] * 1e-3) / 1e12
    res["tflops_step_graph"] = 14 * flops_unit / (res["ms_step_graph"] * 1e-3) / 1e12
    res["frac_of_bf16_peak_step"] = res["tflops_step"] / PEAK_BF16_TFLOPS
    return res


def bandwidth_cases(steps, warmup):
    """RMSNorm / SwiGLU / rotary at the config-4 sizes and decode attention at the config-5 layer shape."""
    import torch
    from scaling_amd import ops
    dev = "cuda"
    out = {}
    g = torch.Generator().manual_seed(1)
    N, H, I = 8192, 4096, 14336
    x = torch.randn(N, H, generator=g).bfloat16().to(dev)
    w = torch.ones(H, dtype=torch.bfloat16, device=dev)
    dy = torch.randn(N, H, generator=g).bfloat16().to(dev)
    ms = time_gpu_graph(lambda: ops.rms_norm_forward(x, w, 1e-5), steps, warmup)
    out["rmsnorm_fwd"] = {"ms": ms, "GBs": 2 * N * H * 2 / ms / 1e6}
    ms = time_gpu_graph(lambda: ops.rms_norm_backward(x, w, dy, 1e-5), steps, warmup)
    out["rmsnorm_bwd"] = {"ms": ms, "GBs": 3 * N * H * 2 / ms / 1e6}
    bias = torch.zeros(H, dtype=torch.bfloat16, device=dev)
    ms = time_gpu_graph(lambda: ops.layer_norm_forward(x, w, bias, 1e-5), steps, warmup)
    out["layernorm_fwd"] = {"ms": ms, "GBs": 2 * N * H * 2 / ms / 1e6}
    _, ln_stats = ops.layer_norm_forward(x, w, bias, 1e-5, save_stats=True)   # as the autograd function runs it
    ms = time_gpu_graph(lambda: ops.layer_norm_backward(x, w, dy, 1e-5, True, ln_stats), steps, warmup)
    out["layernorm_bwd"] = {"ms": ms, "GBs": 3 * N * H * 2 / ms / 1e6}
    a = torch.randn(N, I, generator=g).bfloat16().to(dev)
    gate = torch.randn(N, I, generator=g).bfloat16().to(dev)
    dout = torch.randn(N, I, generator=g).bfloat16().to(dev)
    ms = time_gpu_graph(lambda: ops.swiglu_forward(a, gate), steps, warmup)
    out["swiglu_fwd"] = {"ms": ms, "GBs": 3 * N * I * 2 / ms / 1e6}
    ms = time_gpu_graph(lambda: ops.swiglu_backward(a, gate, dout), steps, warmup)
    out["swiglu_bwd"] = {"ms": ms, "GBs": 5 * N * I * 2 / ms / 1e6}
    ms = time_gpu_graph(lambda: ops.gelu_forward(a), steps, warmup)
    out["gelu_fwd"] = {"ms": ms, "GBs": 2 * N * I * 2 / ms / 1e6}
    ms = time_gpu_graph(lambda: ops.gelu_backward(a, dout), steps, warmup)
    out["gelu_bwd"] = {"ms": ms, "GBs": 3 * N * I * 2 / ms / 1e6}
    del a, gate, dout
    rows, vocab = 4096, 128256                      # config-5 vocabulary
    logits = (torch.randn(rows, vocab, generator=torch.Generator(device=dev).manual_seed(2), device=dev) * 2).bfloat16()
    targets = torch.randint(0, vocab, (rows,), device=dev)
    row_scale = torch.full((rows,), 1.0 / rows, device=dev)
    dlogits = torch.empty_like(logits)
    ms = time_gpu_graph(lambda: ops.cross_entropy_forward(logits, targets), steps, warmup)
    out["cross_entropy_fwd"] = {"ms": ms, "GBs": rows * vocab * 2 / ms / 1e6}
    ms = time_gpu_graph(lambda: ops.cross_entropy_forward(logits, targets, row_scale, dlogits), steps, warmup)
    out["cross_entropy_fwd_bwd"] = {"ms": ms, "GBs": 2 * rows * vocab * 2 / ms / 1e6}
    del logits, dlogits
    nq, nkv, d = 32, 8, 128
    qk = torch.randn(N, nq + nkv, d, generator=g).bfloat16().to(dev)
    cos, sin = _rotary_tables(d, 8192, 500000, dev)
    pos = torch.arange(N, dtype=torch.int64, device=dev) % 4096
    ms = time_gpu_graph(lambda: ops.rotary_embedding(qk, cos, sin, pos), steps, warmup)
    out["rotary"] = {"ms": ms, "GBs": (2 * N * (nq + nkv) * d * 2 + 8 * N) / ms / 1e6}
    del qk
    B, ctx, max_ctx = 32, 4096, 4352
    # head-major storage viewed as [batch, token, kv head, d]: the layout scaling_amd.nn.KVCache allocates
    kc = torch.randn(B, nkv, max_ctx, d, generator=g).bfloat16().to(dev).transpose(1, 2)
    vc = torch.randn(B, nkv, max_ctx, d, generator=g).bfloat16().to(dev).transpose(1, 2)
    q1 = torch.randn(B, nq, d, generator=g).bfloat16().to(dev)
    ctx_len = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    wsd = ops.decode_workspace(B, nq, d, max_ctx, dev)
    od = torch.empty_like(q1)
    ms = time_gpu_graph(lambda: ops.decode_attention(q1, kc, vc, ctx_len, workspace=wsd, out=od), steps, warmup)
    out["decode_attention"] = {"ms": ms, "GBs": 2 * B * ctx * nkv * d * 2 / ms / 1e6, "batch": B, "ctx": ctx}
    for v_ in out.values():
        v_["frac_of_hbm_peak"] = v_["GBs"] / PEAK_HBM_GBS
    return out


def layer_case(steps, warmup):
    """Config 4: one transformer layer (pre-RMSNorm, GQA 32/8 x 128, rotary, SwiGLU 14336) forward + backward on
    [2, 4096, 4096] bf16.  The projections run on PyTorch matmul; the time of this library's kernels inside the step
    is the step time minus the time of the same projections alone (forward, input gradient, weight gradient)."""
    import torch
    from scaling_amd import config as C
    from scaling_amd.layer import TransformerLayer, TransformerLayerIO
    dev = "cuda"
    bsz, seq, hidden = 2, 4096, 4096
    cfg = C.TransformerArchitectureConfig.from_dict(dict(
        vocab_size=128256, hidden_size=hidden, num_layers=1, num_attention_heads=32, attention_num_kv_heads=8,
        attention_qkv_in_one=False, norm_type="rms", mlp_type="swiglu", mlp_factor=3.5, attention_bias=False, mlp_bias=False,
        precision="bfloat16", sequence_length=seq, rotary_embedding_base=500000,
        masked_softmax={"kernel": "hip", "softmax_in_fp32": True}, weight_tying=False))
    g = torch.Generator().manual_seed(4)

    def init(w):
        w.data.copy_((torch.randn(w.shape, generator=g) * 0.02).to(w.dtype))
        return w

    layer = TransformerLayer(cfg, layer_index=0, init_method=init, device=dev)
    x = torch.randn(bsz, seq, hidden, generator=g).bfloat16().to(dev).requires_grad_()
    dy = torch.randn(bsz, seq, hidden, generator=g).bfloat16().to(dev)
    pos = torch.arange(seq, device=dev).repeat(bsz, 1)
    cu = torch.arange(0, bsz * seq + 1, seq, dtype=torch.int32, device=dev)

    def step():
        for p_ in layer.parameters():
            p_.grad = None
        x.grad = None
        out = layer(TransformerLayerIO(activations=x, position_ids=pos, cumulative_seq_lengths=cu))
        out.activations.backward(dy)

    ms = time_gpu(step, steps, warmup)
    # the projections alone: y = x W^T, dx = dy W, dW = dy^T x for each of the seven weights
    n_tok = bsz * seq
    shapes = [(hidden, hidden), (1024, hidden), (1024, hidden), (hidden, hidden), (14336, hidden), (14336, hidden), (hidden, 14336)]
    mats = [(torch.randn(n_tok, i, device=dev, dtype=torch.bfloat16), torch.randn(o, i, device=dev, dtype=torch.bfloat16),
             torch.randn(n_tok, o, device=dev, dtype=torch.bfloat16)) for o, i in shapes]

    def gemms():
        for xin, w, dout in mats:
            torch.nn.functional.linear(xin, w)
            torch.matmul(dout, w)
            torch.matmul(dout.t(), xin)

    ms_gemm = time_gpu(gemms, steps, warmup)
    gemm_flop = 3 * 2 * n_tok * sum(o * i for o, i in shapes)
    pairs = bsz * seq * (seq + 1) // 2
    attn_flop = 14 * 128 * 32 * pairs
    return {"ms_step": ms, "tokens_per_s": n_tok / (ms * 1e-3), "ms_projection_gemms_alone": ms_gemm,
            "ms_everything_else": ms - ms_gemm, "share_outside_gemms": (ms - ms_gemm) / ms,
            "tflops_model": (gemm_flop + attn_flop) / (ms * 1e-3) / 1e12,
            "note": "everything else = attention core, rotary, RMSNorm, SwiGLU, residual adds and autograd glue"}


def decode_case(steps, layers=32, batch=32, prompt=4096):
    """Config 5: random-init 8B-class decoder, batch of prompts prefilled, then greedy cached decoding.
    Reports decode tokens/s (batch * steps / decode wall time) and the prefill time."""
    import torch
    from scaling_amd.config import TransformerArchitectureConfig
    from scaling_amd.inference import TransformerInferenceModule
    cfg = TransformerArchitectureConfig.from_dict(dict(
        vocab_size=128256, hidden_size=4096, num_layers=layers, num_attention_heads=32, attention_num_kv_heads=8,
        attention_qkv_in_one=False, norm_type="rms", mlp_type="swiglu", mlp_factor=3.5, attention_bias=False, mlp_bias=False,
        precision="bfloat16", sequence_length=prompt + steps + 16, rotary_embedding_base=500000, weight_tying=False,
        masked_softmax={"kernel": "hip", "softmax_in_fp32": True}))
    torch.manual_seed(0)
    model = TransformerInferenceModule(cfg, device="cuda", init_std=0.02)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(1, cfg.vocab_size, (batch, prompt), generator=g)   # id 0 would split a prompt into documents
    model.generate(2, ids)                       # warm-up: library heuristics, allocator, caches
    torch.cuda.synchronize()
    t0 = time.time()
    model.generate(1, ids)                       # prefill + first token
    torch.cuda.synchronize()
    t_prefill = time.time() - t0
    t0 = time.time()
    model.generate(steps + 1, ids)               # prefill again + steps decode iterations, one launch per kernel
    torch.cuda.synchronize()
    t_eager = max(time.time() - t0 - t_prefill, 1e-9)
    model.generate_graph(4, ids)                 # warm-up of the capture path
    torch.cuda.synchronize()
    t0 = time.time()
    model.generate_graph(steps + 1, ids)         # prefill + steps decode iterations replayed from one HIP graph
    torch.cuda.synchronize()
    t_decode = max(time.time() - t0 - t_prefill, 1e-9)
    out = {"layers": layers, "batch": batch, "prompt": prompt, "decode_steps": steps, "prefill_s": t_prefill,
           "decode_s": t_decode, "decode_tok_per_s": batch * steps / t_decode, "ms_per_decode_step": 1e3 * t_decode / steps,
           "eager_decode_tok_per_s": batch * steps / t_eager, "eager_ms_per_decode_step": 1e3 * t_eager / steps,
           "note": "decode time = (prefill + decode wall time) - prefill wall time; graph capture time is included"}
    del model
    torch.cuda.empty_cache()
    return out


def cpu_baseline(seconds_budget=25.0):
    """The reference's operation order (CPU oracle) on a bounded sample of the headline workload:
    same head_dim / GQA ratio / causal mask / bf16 with fp32 softmax, fewer heads and a shorter sequence."""
    import torch
    import oracle
    cores = os.cpu_count() or 1
    cores = min(cores, 16)
    torch.set_num_threads(cores)
    s, nq, nkv, d = 2048, 4, 1, 128
    g = torch.Generator().manual_seed(0)
    q = torch.randn(s, 1, nq, d, generator=g).bfloat16().requires_grad_()
    k = torch.randn(s, 1, nkv, d, generator=g).bfloat16().requires_grad_()
    v = torch.randn(s, 1, nkv, d, generator=g).bfloat16().requires_grad_()
    do = torch.randn(nq, s, d, generator=g).bfloat16()
    cu = torch.tensor([0, s], dtype=torch.int32)

    def step():
        out = oracle.multi_head_attention(q, oracle.repeat_kv(k, nq // nkv), oracle.repeat_kv(v, nq // nkv), cu, True,
                                          1 / math.sqrt(d), softmax_in_fp32=True)
        out.backward(do)
        q.grad = k.grad = v.grad = None

    step()
    times = []
    t_all = time.time()
    while len(times) < 3 or (time.time() - t_all < seconds_budget / 2 and len(times) < 10):
        t0 = time.time()
        step()
        times.append(time.time() - t0)
    med = sorted(times)[len(times) // 2]
    flops = 14 * d * nq * (s * (s + 1) // 2)
    return {"value": flops / med / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"oracle (reference op order, bf16 + fp32 softmax) attention fwd+bwd, b1 s{s} {nq}q/{nkv}kv d{d} causal, "
                      f"median of {len(times)} runs = {med * 1e3:.1f} ms"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--decode-steps", type=int, default=256, help="greedy decode steps of the config-5 workload")
    ap.add_argument("--decode-only", action="store_true",
                    help="only run the config-5 decode workload (for a kernel trace of the decode step)")
    ap.add_argument("--decode-layers", type=int, default=32, help="layers of the config-5 model")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain 1 GiB device copy (reference point for the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the path; this build uses no collectives, so --gpus must be 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from scaling_amd import _lib
    _lib.require_device()
    torch.cuda.set_device(0)

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        ms = time_gpu(lambda: dst.copy_(src), args.steps, args.warmup)
        print(json.dumps({"calibration": "device copy", "bytes_read": 1 << 30, "bytes_written": 1 << 30, "ms": ms,
                          "GBs": 2 * (1 << 30) / ms / 1e6}))
        return

    if args.decode_only:
        print(json.dumps({"config5_decode": decode_case(args.decode_steps, layers=args.decode_layers)}))
        return

    b, s, nq, nkv, d = 1, 8192, 32, 8, 128
    main_res = attention_case(b, s, nq, nkv, d, [0, s], args.steps, args.warmup)
    flops_unit = d * nq * main_res["pairs_per_head"]
    # dominant kernel of the step and the algorithmic flops it is credited with:
    #   forward 4 (QK^T, PV), dK/dV kernel 8 (S, dP, dV, dK), dQ kernel 2 (dQ; its S / dP are recomputation)
    kernels = {"attn_fwd_kernel": (main_res["ms_fwd"], 4), "attn_bwd_dkdv_kernel": (main_res["ms_bwd_dkdv"], 8),
               "attn_bwd_dq_kernel": (main_res["ms_bwd_dq"], 2)}
    dom = max(kernels, key=lambda n: kernels[n][0])
    dom_ms, dom_mult = kernels[dom]
    achieved = dom_mult * flops_unit / (dom_ms * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": dom, "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": achieved / PEAK_BF16_TFLOPS, "traffic": None,
                "avg_launch_ms": dom_ms}

    extra = {"headline": main_res}
    if not args.no_extra:
        extra["config2_mha_b4_s2048"] = attention_case(4, 2048, 32, 32, 128, [i * 2048 for i in range(5)], args.steps, args.warmup, seed=2)
        cu3 = random_docs_cu(8192, 256, 2048, seed=0).tolist()
        extra["config3_gqa_packed_rotary_s8192"] = attention_case(1, 8192, 32, 8, 128, cu3, args.steps, args.warmup, seed=3, rotary=True)
        extra["config3_gqa_packed_rotary_s8192"]["n_docs"] = len(cu3) - 1
        extra.update(bandwidth_cases(args.steps, args.warmup))
        extra["config4_layer_fwd_bwd_b2_s4096_h4096"] = layer_case(max(5, args.steps // 2), 3)
        extra["config5_decode_8b_b32_ctx4096"] = decode_case(args.decode_steps, layers=args.decode_layers)

    line = {
        "metric": "attn fwd+bwd TFLOP/s (% bf16 MFMA peak); decode tok/s; norm GB/s (% HBM)",
        "value": main_res["tflops_step"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_res["ms_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "attention core fwd+bwd, GQA 32q/8kv, head_dim 128, batch 1 x seq 8192, causal, bf16, fp32 softmax",
                   "pairs_per_head": main_res["pairs_per_head"], "flop_formula": "14*d*n_q*P"},
        "frac_of_bf16_peak": main_res["tflops_step"] / PEAK_BF16_TFLOPS,
        "roofline": roofline,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline()
    line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
