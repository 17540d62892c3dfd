"""Benchmark of the hot path on one MI355X: GPT-2 113M-class (12 x 768, 12 heads, MLP 3072,
vocab 50257, context 1024) forward + backward + AdamW step at B=16, T=1024 in bf16 with fp32
master weights, dropout 0.1, synthetic uniform token ids (BASELINE config 5).

Prints ONE JSON line.  `value` = steps per second of the whole fwd+bwd(+AdamW) step with
tokens and weights resident in HBM.  `roofline` is for the dominant kernel (the MFMA GEMM
behind t_matmul: forward, dX and dW products), measured with HIP events around every GEMM
launch in a second pass over the same steps.  `attn` and `rowwise` report the other kernel
families the metric names.  `cpu_baseline` is the CPU oracle (fp32, torch on the host cores)
on a bounded sample of the same workload."""
import argparse
import importlib
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Measured with rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE on this benchmark (commands, per-kernel table
# and the copy-kernel scale factors: profiles/hbm_traffic__gpt2_b16_t1024_bf16_step.md): 228.3e6 read +
# 69.3e6 written per GEMM launch, averaged over the forward, dX and dW products of a step.
GEMM_TRAFFIC_BYTES_PER_LAUNCH = 237.9e6
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

CFG = dict(V=50257, D=768, L=12, H=12, F=3072, T=1024, B=16)


def step_flops(c):
    """Algorithmic FLOPs of one fwd+bwd: GEMMs 2NMK (x3 for fwd + dX + dW) + causal attention
    (4 + 10) * dh * B * H * T(T+1)/2 per layer; recomputation not counted."""
    N = c["B"] * c["T"]
    D, F, V, L, H = c["D"], c["F"], c["V"], c["L"], c["H"]
    per_layer = 2 * N * D * (3 * D) + 2 * N * D * D + 2 * 2 * N * D * F
    gemm = 3 * (L * per_layer + 2 * N * D * V)
    attn = L * 14 * (D // H) * c["B"] * H * c["T"] * (c["T"] + 1) // 2
    return gemm + attn, gemm, attn


def make_state(torch, lo, c, dev):
    from_seed = torch.Generator().manual_seed(1234 + 4)
    V, D, L, H, F, T = c["V"], c["D"], c["L"], c["H"], c["F"], c["T"]
    dh = D // H
    res = 0.02 / math.sqrt(2 * L)

    def rn(*shape, scale=0.02):
        return (scale * torch.randn(*shape, generator=from_seed)).to(dev)

    master = [[rn(V, D), torch.zeros(V, device=dev)], [rn(T, D)]]
    for _ in range(L):
        master.append([torch.ones(D, device=dev), torch.zeros(D, device=dev), rn(H, 3, dh, D), rn(D, D, scale=res),
                       torch.ones(D, device=dev), torch.zeros(D, device=dev), rn(F, D), torch.zeros(F, device=dev),
                       rn(D, F, scale=res), torch.zeros(D, device=dev)])
    master.append([torch.ones(D, device=dev), torch.zeros(D, device=dev)])
    shadow = [[p.to(torch.bfloat16) for p in grp] for grp in master]
    _, moments = lo.init_adam_w(master)
    # weight decay on matrices only (train_gpt2_triton.py:71: not the 1-D zero-initialised tensors)
    wd_mask = [[p.dim() > 1 for p in grp] for grp in master]
    return master, shadow, moments, wd_mask


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-probe", action="store_true",
                    help="run one plain 1 GiB device copy first (reference reading for FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--steps-only", action="store_true",
                    help="only the timed training steps (for profiling): no per-kernel legs, no CPU leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the path shards by batch: data parallel over more GPUs "
              "needs one gradient exchange per optimizer step, which is not built); --gpus %d is not supported"
              % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    mt = importlib.import_module("pre-tjax_amd.model_triton")
    lo = importlib.import_module("pre-tjax_amd.loss_and_optimizer_triton")
    _lib = importlib.import_module("pre-tjax_amd._lib")
    _lib.lib()  # fail loudly if the HIP library is missing
    dev = "cuda:0"
    torch.cuda.set_device(0)
    c = CFG
    B, T, V = c["B"], c["T"], c["V"]

    master, shadow, moments, wd_mask = make_state(torch, lo, c, dev)
    tok_gen = torch.Generator().manual_seed(99)
    seed_gen = torch.Generator().manual_seed(100)
    n_total = args.warmup + 2 * args.steps
    tokens = torch.randint(0, V, (n_total, B, T + 1), generator=tok_gen).to(dev)
    mask = None   # plain causal mask (unpadded, unpacked synthetic sequences): masked by index in the kernels
    seeds = [lo.sample_p_gen_aux(master, seed_gen) for _ in range(n_total)]
    losses = []

    def step(i):
        grads, (loss, acc, frac) = lo.t_loss_bkwd3_t(shadow, tokens[i], mask, None, True, seeds[i])
        lo.adam_w_in_place(master, grads, 6e-4, (0.9, 0.95), 1e-8, moments, i, 0.1, wd_mask, shadow=shadow)
        losses.append(loss)

    if args.copy_probe:
        src = torch.ones(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.warmup, args.warmup + args.steps):
        step(i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    value = args.steps / dt
    if args.steps_only:
        print(json.dumps({"value": round(value, 4), "unit": "it/s", "ms_per_step": round(ms_per_step, 3),
                          "steps": args.steps, "warmup": args.warmup}))
        return

    # ---- second pass over further steps with HIP events around every GEMM launch ----------
    ev = []
    orig_gemm = _lib.lib().ptj_gemm

    class Timed:
        def __call__(self, *a):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            rc = orig_gemm(*a)
            e.record()
            ev.append((s, e, 2.0 * a[4] * a[5] * a[6]))   # 2*n*m*k
            return rc

    _lib._lib.ptj_gemm = Timed()
    for i in range(args.warmup + args.steps, n_total):
        step(i)
    torch.cuda.synchronize()
    _lib._lib.ptj_gemm = orig_gemm
    gemm_ms = sum(s.elapsed_time(e) for s, e, _ in ev)
    gemm_flops = sum(f for _, _, f in ev)
    n_launch = len(ev)
    total_flops, gemm_alg, attn_alg = step_flops(c)
    achieved = gemm_flops / (gemm_ms * 1e-3) / 1e12

    # ---- attention and row-wise kernels at the workload's shapes (HIP events) ----------------
    def timeit(fn, n=20):
        for _ in range(3):
            fn()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(n):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / n

    H, dh, D, F = c["H"], c["D"] // c["H"], c["D"], c["F"]
    N = B * T
    qkv = torch.randn(B, H, 3, T, dh, device=dev).to(torch.bfloat16)
    dO = torch.randn(B, H, T, dh, device=dev).to(torch.bfloat16)
    q, k, v = qkv.unbind(2)
    o, ms_, ls_ = mt.attn_fwd_t(q, k, v, None, True, 5)
    t_af = timeit(lambda: mt.attn_fwd_t(q, k, v, None, True, 5))
    t_ab = timeit(lambda: mt.attn_bwd_t(dO, q, k, v, o, ms_, ls_, None, True, 5))
    causal = dh * B * H * T * (T + 1) // 2
    attn = {"fwd_ms": round(t_af, 4), "bwd_ms": round(t_ab, 4),
            "fwd_tflops": round(4 * causal / (t_af * 1e-3) / 1e12, 1),
            "bwd_tflops": round(10 * causal / (t_ab * 1e-3) / 1e12, 1),
            "fwd_bwd_tflops": round(14 * causal / ((t_af + t_ab) * 1e-3) / 1e12, 1),
            "peak_tflops": PEAK_BF16_TFLOPS,
            "frac": round(14 * causal / ((t_af + t_ab) * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
            "shape": "B%d H%d T%d dh%d bf16 causal dropout0.1" % (B, H, T, dh)}
    # Row-wise legs: every call works on another set of buffers and the sets together exceed the
    # 256 MB last-level cache, so the rates are HBM rates as in the training step (a leg that
    # re-used one set would run out of cache).
    def timeit_sets(fn, nsets, n=24):
        for i in range(3):
            fn(i % nsets)
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for i in range(n):
            fn(i % nsets)
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / n

    ND, NF = 12, 4                                   # 12 x 3 x 25 MB and 4 x 2 x 100 MB
    xs_ = [torch.randn(N, D, device=dev).to(torch.bfloat16) for _ in range(ND)]
    dys = [torch.randn(N, D, device=dev).to(torch.bfloat16) for _ in range(ND)]
    rss = [torch.randn(N, D, device=dev).to(torch.bfloat16) for _ in range(ND)]
    gam = torch.ones(D, device=dev, dtype=torch.bfloat16)
    xfs = [torch.randn(N, F, device=dev).to(torch.bfloat16) for _ in range(NF)]
    dfs = [torch.randn(N, F, device=dev).to(torch.bfloat16) for _ in range(NF)]
    keeps = [mt.dropout_add_t(xs_[i], rss[i], True, 42, want_keep=True)[1] for i in range(ND)]
    e2 = 2
    rows = {}

    def gbs(nbytes, ms):
        return round(nbytes / (ms * 1e-3) / 1e9, 1)
    rows["layernorm_fwd"] = gbs(2 * N * D * e2, timeit_sets(lambda i: mt.t_layernorm_fwd_t((gam, gam), xs_[i]), ND))
    rows["layernorm_bwd_dx_dgb"] = gbs(3 * N * D * e2,
                                       timeit_sets(lambda i: mt.layernorm_bkwd2_t(dys[i], (gam, gam), xs_[i]), ND))
    # the training step's variants: residual update + norm in one pass (reads x, res; writes y, h,
    # keep bytes), and the norm backward that adds the residual and also writes the dropped copy
    # and its column sums (reads dy, x, res, keep bytes; writes dx, dropped)
    rows["dropout_add_layernorm"] = gbs(4 * N * D * e2 + N * D // 8, timeit_sets(
        lambda i: mt.dropout_add_layernorm_t(xs_[i], rss[i], (gam, gam), True, 42, want_keep=True), ND))
    rows["layernorm_bwd_res_drop_sums"] = gbs(5 * N * D * e2 + N * D // 8, timeit_sets(
        lambda i: mt.layernorm_bkwd2_t(dys[i], (gam, gam), xs_[i], residual=rss[i], drop=(True, 42, keeps[i]),
                                       drop_sum=True), ND))
    rows["gelu_fwd"] = gbs(2 * N * F * e2, timeit_sets(lambda i: mt.t_gelu_fwd_t(xfs[i]), NF))
    rows["gelu_bwd"] = gbs(3 * N * F * e2, timeit_sets(lambda i: mt.t_gelu_bkwd2_t(dfs[i], xfs[i]), NF))
    rows["gelu_bwd_colsum"] = gbs(3 * N * F * e2, timeit_sets(lambda i: mt.t_gelu_bkwd2_colsum_t(dfs[i], xfs[i]), NF))
    rows["dropout_fwd"] = gbs(2 * N * D * e2, timeit_sets(lambda i: mt.t_dropout_fwd_t(xs_[i], True, 42), ND))
    del xfs, dfs
    # the logits as the step holds them: rows padded to a multiple of 64 columns (the LM-head product's
    # output pitch), argmax requested; the gradient goes to a second buffer here (in place the next timed
    # call would read gradients as logits)
    vp = (V + 63) // 64 * 64
    lgbuf = torch.randn(N, vp, device=dev).to(torch.bfloat16)
    lg = lgbuf[:, :V]
    lab = torch.randint(0, V, (N,), device=dev)
    rows["ce_fwd_bwd"] = gbs(2 * N * V * e2 + 8 * N,
                             timeit(lambda: lo.t_avg_cross_entropy_loss_bkwd3_t(lab, lg, want_pred=True), n=8))
    del lg, lgbuf
    rowwise = {"achieved_GBs": rows, "peak_GBs": PEAK_HBM_GBS, "bytes": "algorithmic (minimum traffic), bf16",
               "note": "wrapper calls timed with HIP events (two launches each where a second-stage reduction "
                       "follows); inputs rotate over buffer sets larger than the last-level cache",
               "frac": {kk: round(vv / PEAK_HBM_GBS, 3) for kk, vv in rows.items()}}

    # ---- CPU baseline: the oracle (fp32) on a bounded sample ------------------------------------
    cpu = None
    if not args.no_cpu:
        from oracle import gpt2 as ogpt2
        nthreads = torch.get_num_threads()
        cb = 8                                   # about 15 s of CPU work on 16 host cores
        cparams = [[p.detach().to("cpu") for p in grp] for grp in master]
        cy = tokens[0, :cb].to("cpu")
        cmask = torch.tril(torch.ones(T, T, dtype=torch.bool)).expand(cb, T, T)
        t1 = time.perf_counter()
        ogpt2.grad_loss(cparams, cy, cmask, False)
        cpu_s = time.perf_counter() - t1
        cpu = {"value": round(1.0 / (cpu_s * (B / cb)), 5), "unit": "it/s", "cores": nthreads, "kind": "port",
               "sample": "oracle fwd+bwd (torch fp32 autograd, eval-mode dropout scaling) on %d of %d sequences, "
                         "%.2f s, scaled to the full batch" % (cb, B, cpu_s)}

    out = {
        "metric": "GPT-2 113M fwd+bwd it/s at B16 T1024; attn fwd+bwd TFLOP/s vs MFMA peak",
        "value": round(value, 4), "unit": "it/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE config 5: GPT-2 small 12x768 H12 F3072 V50257 T1024, B=16, bf16 + fp32 "
                               "master weights, dropout 0.1, fwd+bwd+AdamW every step",
                   "global_batch": B, "seq_len": T, "step_tflop": round(total_flops / 1e12, 3),
                   "step_tflops_achieved": round(total_flops / 1e12 * value, 1)},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": GEMM_TRAFFIC_BYTES_PER_LAUNCH,
                     "traffic_note": "HBM bytes per GEMM launch (average over the 147 launches of a step) from rocprofv3 "
                                     "FETCH_SIZE / WRITE_SIZE runs scaled by a 1 GiB copy; algorithmic minimum 145.2e6",
                     "kernel": "gemm_kernel<bf16> (all %d launches of a step: fwd, dX, dW)" % (n_launch // args.steps),
                     "avg_launch_ms": round(gemm_ms / n_launch, 4),
                     "gflop_per_launch": round(gemm_flops / n_launch / 1e9, 2),
                     "gemm_ms_per_step": round(gemm_ms / args.steps, 3)},
        "attn": attn,
        "rowwise": rowwise,
        "cpu_baseline": cpu,
        "final_loss": round(float(losses[-1].item()), 4),
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
