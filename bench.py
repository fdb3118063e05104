#!/usr/bin/env python3
"""Headline benchmark: train tokens/s of the TopK SAE step on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B]

A "step" is one pass of the hot path over one batch of synthetic activations that already sit in
HBM: compute_loss under bf16 autocast (encoder GEMM -> bias + TopK select -> sparse decode + MSE
and its backward) -> loss.backward() (feature index, dW_D / dW_E rows, bias gradients) ->
HipAdam.step() -> zero_grad().  Workload: d_model 4096, d_sae 131072, k 64, fp32 master weights with
bf16 GEMM / gather operands (the reference's default mixed precision), B tokens per step.

Prints ONE JSON line.  `roofline` describes the kernel with the largest share of the step, timed
with HIP events inside the timed region; `cpu_baseline` is the oracle (a CPU restatement of the
reference's eager path) timed on this host on a reduced batch of the same shape.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

D_MODEL, D_SAE, TOP_K = 4096, 131072, 64
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E


def algorithmic_work(B: int) -> dict:
    """Per-launch algorithmic work of every kernel of the step (bytes unless noted)."""
    d, F, k = D_MODEL, D_SAE, TOP_K
    return {
        "encoder_gemm": ("mfma", 2.0 * B * d * F),                       # flop
        "select_topk_row": ("hbm", B * F * 2 + B * k * 8),               # read bf16 pre once, write idx+val
        "sparse_decode_mse_fused": ("hbm", 2 * B * k * d * 2 + 3 * B * d * 4),  # rows for recon and for d val; label, recon, grad
        "sparse_grad_rows[f32 dense]": ("hbm", F * d * 4),               # dW_D: one full fp32 gradient matrix written
        "sparse_grad_rows[bf16 dense]": ("hbm", F * d * 4),              # dW_E^T: likewise
        "adam_step[matrix]": ("hbm", F * d * 30),                        # g,p,m,v read; p,m,v written; bf16 shadow written
        "adam_step[vector]": ("hbm", (F + d) / 2 * 28),                  # the two biases, averaged
        # Adam with the gradient rows rebuilt in registers: p,m,v read; p,m,v written; bf16 shadow written
        "adam_step_sparse_rows[f32 dense]": ("hbm", F * d * 26),
        "adam_step_sparse_rows[bf16 dense]": ("hbm", F * d * 26),
        "build_feature_index": ("hbm", B * k * 16 + F * 12),
        "cast_f32_to_bf16": ("hbm", B * d * 6),
        "col_sum": ("hbm", B * d * 4),
    }


def gpu_step_bench(args):
    import torch
    from __graft_entry__ import load_package

    pkg = load_package()
    from lm_saes_amd import synthetic

    dev = torch.device("cuda:0")
    B = args.batch
    d, F, k = D_MODEL, D_SAE, TOP_K
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                        top_k=k, norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda",
                        dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    # N* recipe: activations G(d, r=64, seed 4); weights drawn on the device (1.07e9 parameters)
    x = synthetic.activations(B, d, 64, seed=4).to(dev)
    with torch.no_grad():
        g = torch.Generator(device=dev).manual_seed(4)
        wt = sae.W_E.t()
        wt.uniform_(-1.0 / d ** 0.5, 1.0 / d ** 0.5, generator=g)
        sae.W_D.copy_(wt / wt.norm(dim=1, keepdim=True))
        sae.b_E.zero_()
        sae.b_D.copy_(x.mean(0))
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, betas=(0.9, 0.999), model=sae,
                       overlap_decoder_update=args.overlap)

    def step():
        with torch.autocast("cuda", dtype=torch.bfloat16):
            loss = sae.compute_loss(batch, return_aux_data=False)
        loss.backward()
        opt.step()
        opt.zero_grad()
        return loss

    if args.calibrate_copy:
        # a plain device copy of known size (1 GiB read + 1 GiB written), for scaling rocprofv3's
        # FETCH_SIZE / WRITE_SIZE counters when they are collected over this command
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    pkg.ops.set_kernel_timer(None)
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    kernels = timer.summary()
    return ms_per_step, kernels, float(loss.item())


def cpu_baseline(sample_batch: int, sample_features: int):
    """Oracle (the reference's eager op sequence on CPU) on a bounded sample of the workload:
    same d_model and k, `sample_features` of the 131072 dictionary features, `sample_batch` tokens.
    Per-step CPU cost is close to linear in the number of features (GEMMs, [B, F] temporaries and
    Adam all scale with F), so the full dictionary would take 131072 / sample_features times longer
    per token; the reported value is the measured one, not an extrapolation."""
    import torch
    from __graft_entry__ import load_oracle, load_package

    oracle = load_oracle()
    load_package()
    from lm_saes_amd import synthetic

    d, F, k = D_MODEL, sample_features, TOP_K
    cores = torch.get_num_threads()
    m = oracle.SAEOracle(d, F, act_fn="topk", top_k=k, sparsity_include_decoder_norm=True)
    with torch.no_grad():
        m.W_E.uniform_(-1.0 / d ** 0.5, 1.0 / d ** 0.5)
        m.W_D.copy_(m.W_E.t())
        m.W_D.div_(m.W_D.norm(dim=1, keepdim=True))
    x = synthetic.activations(sample_batch, d, 64, seed=4)
    batch = {"in": x, "out": x, "tokens": torch.zeros(sample_batch, dtype=torch.long)}
    opt = oracle.make_adam(m, lr=4e-4)
    oracle.train_step(m, opt, batch, amp_dtype=torch.bfloat16)  # warm-up (allocates Adam state)
    t0 = time.perf_counter()
    oracle.train_step(m, opt, batch, amp_dtype=torch.bfloat16)
    dt = time.perf_counter() - t0
    return {
        "value": round(sample_batch / dt, 2), "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"1 warm-up + 1 timed step of the TopK SAE train step at d_model={d} k={k} with {F} of the "
                  f"{D_SAE} features (1/{D_SAE // F} of the dictionary) and B={sample_batch} tokens, fp32 master "
                  f"weights + bf16 autocast on CPU, torch {torch.__version__}, {dt:.1f} s per step",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=4096)
    ap.add_argument("--cpu-sample-batch", type=int, default=512)
    ap.add_argument("--cpu-sample-features", type=int, default=32768)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true", help="also run three 1 GiB device copies (counter calibration)")
    ap.add_argument("--overlap", action="store_true", help="run the decoder Adam pass on a second stream, overlapping the next GEMM")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collectives are part of it); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    ms_per_step, kernels, loss = gpu_step_bench(args)
    B = args.batch
    work = algorithmic_work(B)
    dominant = max(kernels, key=lambda n: kernels[n]["total_ms"])
    bound, per_launch = work.get(dominant, ("hbm", 0.0))
    avg_ms = kernels[dominant]["avg_ms"]
    if bound == "mfma":
        achieved, peak, unit = per_launch / avg_ms / 1e9, PEAK_BF16_TFLOPS, "TFLOP/s"
    else:
        achieved, peak, unit = per_launch / avg_ms / 1e6, PEAK_HBM_GBS, "GB/s"
    roofline = {
        "kernel": dominant, "bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
        "frac": round(achieved / peak, 4), "traffic": None, "avg_ms": round(avg_ms, 4),
        "launches_per_step": kernels[dominant]["calls"] / args.steps,
    }
    per_kernel = {}
    for name, st in kernels.items():
        bnd, w = work.get(name, ("hbm", 0.0))
        rate = w / st["avg_ms"] / (1e9 if bnd == "mfma" else 1e6) if w else None
        per_kernel[name] = {
            "ms_per_step": round(st["total_ms"] / args.steps, 4), "avg_ms": round(st["avg_ms"], 4), "bound": bnd,
            "achieved": None if rate is None else round(rate, 1),
            "frac": None if rate is None else round(rate / (PEAK_BF16_TFLOPS if bnd == "mfma" else PEAK_HBM_GBS), 4),
        }
    out = {
        "metric": "train tokens/s, TopK SAE d=4096 F=131072 k=64 bf16; % MFMA / HBM roofline",
        "value": round(B / (ms_per_step / 1e3), 1),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"topk_sae_train_step d_model={D_MODEL} d_sae={D_SAE} k={TOP_K} batch={B} "
                               "fp32-master/bf16-operands adam", "batch_tokens": B},
        "roofline": roofline,
        "kernels": per_kernel,
        "final_loss": loss,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.cpu_sample_batch, args.cpu_sample_features)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
