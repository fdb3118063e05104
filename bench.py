#!/usr/bin/env python3
"""Headline benchmark: train tokens/s of the TopK SAE step on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--workload NAME]

A "step" is one pass of the hot path over one batch of synthetic activations that already sit in
HBM: compute_loss under bf16 autocast (encoder GEMM -> bias + TopK select -> sparse decode + MSE
and its backward) -> loss.backward() (feature index, dW_D / dW_E rows, bias gradients) ->
HipAdam.step() -> zero_grad().  Default workload: d_model 4096, d_sae 131072, k 64, fp32 master
weights with bf16 GEMM / gather operands (the reference's default mixed precision), 4096 tokens per
step.  `--workload` runs the same step on the other model configurations (BatchTopK with aux-k,
JumpReLU with the tanh penalty, cross-layer transcoder, Lorsa) for profiling; their lines carry their
own workload name.

Prints ONE JSON line.  `roofline` describes the kernel of this library with the largest share of
the step, timed with HIP events inside the timed region; `cpu_baseline` (default workload only) is
the oracle (a CPU restatement of the reference's eager path) timed on this host on a reduced batch
of the same shape.  After the headline's timed region a default run also times the other benchmark
configurations for a few steps each (the reference's CPU configuration in fp32, BatchTopK with aux-k,
JumpReLU dense and sparse, the cross-layer transcoder, Lorsa, a crosscoder) and reports them under
`configs`; they never enter `value`.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

D_MODEL, D_SAE, TOP_K = 4096, 131072, 64
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# Measured HBM bytes per launch of the default workload's kernels are not typed in here: they are read from the table
# "Scaled HBM traffic per launch" of the committed counter summary (two rocprofv3 runs, FETCH_SIZE and WRITE_SIZE, scaled
# by what the same counters read for transfers of known size in the same runs).
HBM_TRAFFIC_FILE = os.path.join("profiles", "train_step_topk_d4096_F131072_k64_B4096_hbm_counters.md")
HBM_TRAFFIC_ROWS = {"encoder_gemm": "encoder_gemm", "adam_step_sparse_rows[f32 dense]": "adam_sparse_rows",
                    "adam_step_sparse_rows[bf16 dense]": "adam_sparse_rows", "sparse_decode_mse_fused": "sparse_decode_mse_fused",
                    "select_topk_row": "select_topk_row"}
# launches that move so little that their duration is the launch / dependency latency, not a bandwidth
LATENCY_BOUND = {"build_feature_index", "adam_step[vector]", "col_sum", "cast_f32_to_bf16", "code_stats", "recon_stats",
                 "grad_sq_nnz", "gather_rows", "row_sum", "row_norm",
                 # one workgroup per token: a radix select over F / 64 keys in LDS (a dozen barriers) and ~k scattered granules
                 "select_topk_row[granule]"}


def measured_traffic_gb(kernel: str):
    """Total HBM GB per launch of `kernel` from the committed counter summary, or None."""
    label = HBM_TRAFFIC_ROWS.get(kernel)
    path = os.path.join(ROOT, HBM_TRAFFIC_FILE)
    if label is None or not os.path.exists(path):
        return None
    in_table = False
    for line in open(path):
        if line.startswith("## "):
            in_table = line.startswith("## Scaled HBM traffic per launch")
        elif in_table and line.startswith("| " + label):
            cells = [c.strip() for c in line.strip().strip("|").split("|")]
            try:
                return float(cells[3])        # kernel | fetched GB | written GB | total GB | ...
            except (IndexError, ValueError):
                return None
    return None


def algorithmic_work(B: int, d: int, F: int, k: int) -> dict:
    """Per-launch algorithmic work of the library's kernels (bytes unless noted) for B tokens of a
    d -> F dictionary with k active features per token."""
    return {
        "encoder_gemm": ("mfma", 2.0 * B * d * F),                       # flop
        "select_topk_row": ("hbm", B * F * 2 + B * k * 8),               # read bf16 pre once, write idx+val
        "select_topk_row[granule]": ("hbm", B * (F // 64) * 4 + B * k * (128 + 8)),   # granule maxima, ~k granules of pre, idx+val
        "select_topk_batch": ("hbm", B * F * 2 + B * k * 8),             # read bf16 pre once, write idx+val
        "sparse_decode_mse_fused": ("hbm", 2 * B * k * d * 2 + 3 * B * d * 4),  # rows for recon and for d val; label, recon, grad
        "sparse_decode_fwd": ("hbm", B * k * d * 2 + B * d * 4),
        "sparse_decode_bwd_dval": ("hbm", B * k * d * 2 + B * d * 4),
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
        "sparse_rows_grad_sq_nnz": ("hbm", B * k * d * 2 + B * k * 12 + F * 24),  # gathered bf16 rows (cache hits), index, partials
        "code_stats": ("hbm", B * k * 8 + B * 12),
        "recon_stats": ("hbm", 2 * B * d * 4),
        "grad_sq_nnz": ("hbm", (F + d) / 2 * 4),
        "gather_rows": ("hbm", B * d * 6),                               # fp32 rows read, bf16 rows written
        "jumprelu_fwd": ("hbm", B * F * 4),                              # bf16 pre read, bf16 acts written
        "jumprelu_bwd": ("hbm", B * F * 6),                              # bf16 pre and d_acts read, bf16 d_pre written
    }


# ---- workloads ------------------------------------------------------------------------------------

def _autocast_step(model, batch, opt, loss_kwargs):
    import torch

    def step():
        with torch.autocast("cuda", dtype=torch.bfloat16):
            loss = model.compute_loss(batch, return_aux_data=False, **loss_kwargs)
        loss.backward()
        opt.step()
        opt.zero_grad()
        return loss
    return step


def _init_sae_on_device(sae, x, d, seed=4):
    import torch

    with torch.no_grad():
        g = torch.Generator(device=x.device).manual_seed(seed)
        wt = sae.W_E.t()
        wt.uniform_(-1.0 / d ** 0.5, 1.0 / d ** 0.5, generator=g)
        sae.W_D.copy_(wt / wt.norm(dim=1, keepdim=True))
        sae.b_E.zero_()
        sae.b_D.copy_(x.mean(0))


def build_topk(pkg, dev, args):
    """The headline workload: TopK SAE d=4096, F=131072, k=64."""
    import torch
    from lm_saes_amd import synthetic

    B, d, F, k = args.batch or 4096, D_MODEL, args.d_sae or D_SAE, TOP_K
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                        top_k=k, norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda",
                        dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    x = synthetic.activations(B, d, 64, seed=4).to(dev)    # activations G(d, r=64, seed 4); weights drawn on the device
    _init_sae_on_device(sae, x, d)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, betas=(0.9, 0.999), model=sae,
                      overlap_decoder_update=args.overlap)
    name = f"topk_sae_train_step d_model={d} d_sae={F} k={k} batch={B} fp32-master/bf16-operands adam"
    return _autocast_step(sae, batch, opt, {}), B, name, (B, d, F, k)


C1 = dict(d=768, F=6144, k=32, B=4096, r=16, seed=0)   # the reference's CPU-runnable configuration: fp32, MSE only


def build_c1_fp32(pkg, dev, args):
    """TopK SAE d=768 -> 6144, k=32, B=4096 in fp32 (no autocast), Adam lr 4e-4: the configuration the CPU path runs
    at full shape, so `cpu_baseline` of this workload is the oracle on exactly the same step."""
    import torch
    from lm_saes_amd import synthetic

    B, d, F, k = C1["B"], C1["d"], C1["F"], C1["k"]
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                        top_k=k, norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda",
                        dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    x = synthetic.activations(B, d, C1["r"], seed=C1["seed"]).to(dev)
    _init_sae_on_device(sae, x, d, seed=C1["seed"])
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, betas=(0.9, 0.999), model=sae)

    def step():
        loss = sae.compute_loss(batch, return_aux_data=False)
        loss.backward()
        opt.step()
        opt.zero_grad()
        return loss
    return step, B, f"topk_sae_train_step d_model={d} d_sae={F} k={k} batch={B} fp32 adam", (B, d, F, k)


def cpu_baseline_c1():
    """The oracle on the full C1 step (same shape, fp32, same optimizer), all host threads."""
    import torch
    from __graft_entry__ import load_oracle, load_package

    oracle = load_oracle()
    load_package()
    from lm_saes_amd import synthetic

    B, d, F, k = C1["B"], C1["d"], C1["F"], C1["k"]
    m = oracle.SAEOracle(d, F, act_fn="topk", top_k=k, sparsity_include_decoder_norm=True)
    with torch.no_grad():
        m.W_E.uniform_(-1.0 / d ** 0.5, 1.0 / d ** 0.5)
        m.W_D.copy_(m.W_E.t())
        m.W_D.div_(m.W_D.norm(dim=1, keepdim=True))
    x = synthetic.activations(B, d, C1["r"], seed=C1["seed"])
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long)}
    opt = oracle.make_adam(m, lr=4e-4)
    oracle.train_step(m, opt, batch)
    n_timed, t0 = 0, time.perf_counter()
    while n_timed < 3 or (time.perf_counter() - t0 < 12.0 and n_timed < 20):
        oracle.train_step(m, opt, batch)
        n_timed += 1
    dt = (time.perf_counter() - t0) / n_timed
    return {"value": round(B / dt, 2), "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"1 warm-up + {n_timed} timed steps of the full step (d_model={d} d_sae={F} k={k} B={B}, fp32) on CPU, "
                      f"torch {torch.__version__}, {dt:.2f} s per step"}


def build_topk_bf16_params(pkg, dev, args):
    """The headline shape with the dictionary itself held in bf16 (cfg.dtype = bfloat16: bf16 parameters,
    gradients and Adam moments, as the reference trains with that dtype).  A secondary figure: the reference's
    default, and the headline, is fp32 parameters under bf16 autocast."""
    import torch
    from lm_saes_amd import synthetic

    B, d, F, k = args.batch or 4096, D_MODEL, args.d_sae or D_SAE, TOP_K
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                        top_k=k, norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda",
                        dtype=torch.bfloat16)
    sae = pkg.SparseAutoEncoder(cfg)
    x = synthetic.activations(B, d, 64, seed=4).to(dev)
    _init_sae_on_device(sae, x, d)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, betas=(0.9, 0.999), model=sae)
    name = f"topk_sae_train_step d_model={d} d_sae={F} k={k} batch={B} bf16-parameters adam"
    return _autocast_step(sae, batch, opt, {}), B, name, (B, d, F, k)


def build_topk_trainer(pkg, dev, args):
    """The headline shape driven through `Trainer.train_one_step`: the step plus what the reference's loop
    adds around it every step (gradient norm over all parameters, the eight logging metrics, LR schedule)."""
    import torch
    from lm_saes_amd import synthetic

    B, d, F, k = args.batch or 4096, D_MODEL, D_SAE, TOP_K
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                        top_k=k, norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda",
                        dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    x = synthetic.activations(B, d, 64, seed=4).to(dev)
    _init_sae_on_device(sae, x, d)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    tcfg = pkg.TrainerConfig(lr=4e-4, total_training_tokens=B * 1_000_000, amp_dtype=torch.bfloat16, l1_coefficient=None,
                             skip_metrics_calculation=False, log_frequency=1000, clip_grad_norm=args.clip, k_warmup_steps=0,
                             lr_warm_up_steps=100)
    trainer = pkg.Trainer(tcfg)
    trainer.prepare(sae, batch)
    name = (f"topk_sae Trainer.train_one_step d_model={d} d_sae={F} k={k} batch={B} fp32-master/bf16-operands adam, "
            f"grad norm + metrics every step, clip_grad_norm={args.clip}")
    return (lambda: trainer.train_one_step(sae, batch)["loss"]), B, name, (B, d, F, k)


def build_activation_stream(pkg, dev, args):
    """Not a train step: one batch drawn from the shuffling batchler (4096 tokens of d_model=4096, fp32 rows in a
    131072-token HBM buffer, handed out as bf16), refills and shuffles included."""
    import torch

    B, d, chunk = args.batch or 4096, D_MODEL, 32768
    src = torch.randn(chunk, d, device=dev)

    def chunks():
        while True:
            yield {"in": src, "tokens": torch.zeros(chunk, dtype=torch.long, device=dev)}

    batchler = pkg.ActivationBatchler(B, buffer_size=131072, buffer_shuffle_config=pkg.BufferShuffleConfig(),
                                      override_dtype=torch.bfloat16)
    it = batchler.process(chunks())
    name = f"activation_batchler batch={B} d_model={d} buffer=131072 tokens fp32 -> bf16"
    return (lambda: next(it)["in"].sum()), B, name, (B, d, D_SAE, TOP_K)


class _FixedDead:
    """Stands in for the trainer's dead-feature statistics: a fixed set of features counts as dead."""

    def __init__(self, is_dead):
        self.is_dead = is_dead

    def update_dead_statistics(self, feature_acts, mask, specs):
        return self.is_dead

    def update_dead_statistics_sparse(self, code, mask):
        return self.is_dead


def build_batchtopk(pkg, dev, args, bf16_params=False):
    """BatchTopK SAE d=2048, F=32768, 8192 tokens, global top 64 x 8192, aux-k on the top 512 dead features."""
    import torch
    from lm_saes_amd import synthetic

    B, d, F, k = args.batch or 8192, 2048, 32768, 64
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="batchtopk",
                        top_k=k, norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda",
                        dtype=torch.bfloat16 if bf16_params else torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    x = synthetic.activations(B, d, 32, seed=4).to(dev)
    _init_sae_on_device(sae, x, d)
    g = torch.Generator(device=dev).manual_seed(5)
    dead = _FixedDead(torch.rand(F, device=dev, generator=g) < 0.1)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, model=sae)
    kw = dict(auxk_coefficient=1.0 / 32, k_aux=512, update_dead_statistics=dead.update_dead_statistics)
    name = (f"batchtopk_sae_train_step d_model={d} d_sae={F} k={k} batch={B} aux-k=512 (10% of features dead) "
            + ("bf16-parameters adam" if bf16_params else "bf16 adam"))
    return _autocast_step(sae, batch, opt, kw), B, name, (B, d, F, k)


def build_batchtopk_bf16_params(pkg, dev, args):
    """The BatchTopK + aux-k workload with the dictionary itself held in bf16 (cfg.dtype = bfloat16): a secondary figure."""
    return build_batchtopk(pkg, dev, args, bf16_params=True)


def build_jumprelu(pkg, dev, args):
    """JumpReLU SAE d=4096, F=131072, 4096 tokens: Gaussian rows with 4 outlier dimensions x50, threshold
    log(0.001), rectangle window 0.001, tanh penalty coefficient 5."""
    import torch

    B, d, F = args.batch or 4096, D_MODEL, D_SAE
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="jumprelu",
                        jumprelu_threshold_window=0.001, norm_activation="inference", sparsity_include_decoder_norm=True,
                        device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    g = torch.Generator(device=dev).manual_seed(4)
    x = torch.randn(B, d, device=dev, generator=g)
    x[:, [7, 1029, 2050, 3071]] *= 50.0
    _init_sae_on_device(sae, x, d)
    with torch.no_grad():
        sae.activation_function.log_jumprelu_threshold.fill_(math.log(0.001))
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    groups = sae.get_parameters()
    opt = pkg.HipAdam([{"params": groups[0]["params"]}, {"params": groups[1]["params"]}], lr=4e-4, model=sae)
    kw = dict(sparsity_loss_type="tanh", l1_coefficient=5.0)
    name = f"jumprelu_sae_train_step d_model={d} d_sae={F} batch={B} window=0.001 tanh-penalty=5 bf16 adam"
    return _autocast_step(sae, batch, opt, kw), B, name, (B, d, F, F // 2)


def build_jumprelu_sparse(pkg, dev, args):
    """The JumpReLU configuration as it looks once trained: the same shapes and data, thresholds raised so that about 64 of
    the 131072 features pass per token (log-threshold log(3.5), window 0.1).  The step then takes its sparse form."""
    import torch

    B, d, F = args.batch or 4096, D_MODEL, D_SAE
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="jumprelu",
                        jumprelu_threshold_window=0.1, norm_activation="inference", sparsity_include_decoder_norm=True,
                        device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    g = torch.Generator(device=dev).manual_seed(4)
    x = torch.randn(B, d, device=dev, generator=g)
    x[:, [7, 1029, 2050, 3071]] *= 50.0
    _init_sae_on_device(sae, x, d)
    with torch.no_grad():
        sae.activation_function.log_jumprelu_threshold.fill_(math.log(3.5))
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    groups = sae.get_parameters()
    opt = pkg.HipAdam([{"params": groups[0]["params"]}, {"params": groups[1]["params"]}], lr=4e-4, model=sae)
    kw = dict(sparsity_loss_type="tanh", l1_coefficient=5.0)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        out = sae.compute_loss(batch, **kw)
    l0 = float(out["sparse_code"].row_nnz.float().mean().item()) if "sparse_code" in out else float("nan")
    name = (f"jumprelu_sae_train_step (sparse form, {l0:.0f} kept-or-window entries per token) d_model={d} d_sae={F} batch={B} "
            f"window=0.1 tanh-penalty=5 bf16 adam")
    return _autocast_step(sae, batch, opt, kw), B, name, (B, d, F, max(1, int(l0) if l0 == l0 else 64))


def build_clt(pkg, dev, args):
    """Cross-layer transcoder: 12 layers, d=768, 12288 features per layer, k=64 per layer, 2048 tokens;
    targets y_j = tanh(A_j x_j) with seeded A_j ~ N(0, 1) / sqrt(768)."""
    import torch
    from lm_saes_amd import synthetic

    B, L, d, F, k = args.batch or 2048, 12, 768, 12288, 64
    hin, hout = [f"in{l}" for l in range(L)], [f"out{l}" for l in range(L)]
    cfg = pkg.CLTConfig(hook_points_in=hin, hook_points_out=hout, d_model=d, expansion_factor=F / d, act_fn="topk", top_k=k,
                        norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda", dtype=torch.float32)
    clt = pkg.CrossLayerTranscoder(cfg)
    clt.init_parameters()
    g = torch.Generator(device=dev).manual_seed(4)
    batch = {"tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    for l in range(L):
        x = synthetic.activations(B, d, 16, seed=4 + l).to(dev)
        A = torch.randn(d, d, device=dev, generator=g) / d ** 0.5
        batch[hin[l]], batch[hout[l]] = x, torch.tanh(x @ A)
    opt = pkg.HipAdam(clt.get_parameters()[0]["params"], lr=4e-4, model=clt)
    name = f"clt_train_step layers={L} d_model={d} d_sae={F} k={k}/layer batch={B} bf16 adam"
    return _autocast_step(clt, batch, opt, {}), B, name, (B, d, F, k)


def build_lorsa(pkg, dev, args, positional="none"):
    """Lorsa: d=768, 16 sequences x 1024 tokens, 64 query/key heads of width 64, 8192 value/output heads
    (128 per query/key head), k=64; target = causal softmax attention of a seeded rank-64 head set."""
    import torch
    from lm_saes_amd import synthetic

    nb, s, d, F, h, dq, k = 16, 1024, 768, 8192, 64, 64, 64
    cfg = pkg.LorsaConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, n_qk_heads=h,
                          d_qk_head=dq, n_ctx=s, rotary_dim=dq, positional_embedding_type=positional, act_fn="topk", top_k=k,
                          norm_activation="inference", device="cuda", dtype=torch.float32)
    m = pkg.LowRankSparseAttention(cfg)
    m.init_parameters()
    g = torch.Generator(device=dev).manual_seed(4)
    x = synthetic.activations(nb * s, d, 64, seed=4).to(dev).view(nb, s, d)
    with torch.no_grad():
        wq, wk = (torch.randn(d, 64, device=dev, generator=g) / d ** 0.5 for _ in range(2))
        wvo = (torch.randn(d, 64, device=dev, generator=g) @ torch.randn(64, d, device=dev, generator=g)) / (8 * d ** 0.5)
        y = torch.nn.functional.scaled_dot_product_attention((x @ wq)[:, None], (x @ wk)[:, None], (x @ wvo)[:, None],
                                                             is_causal=True, scale=1 / 8)[:, 0]
    batch = {"in": x, "out": y.contiguous(), "tokens": torch.zeros(nb, s, dtype=torch.long, device=dev)}
    opt = pkg.HipAdam(m.get_parameters()[0]["params"], lr=4e-4, model=m)
    name = (f"lorsa_train_step d_model={d} sequences={nb}x{s} qk_heads={h}x{dq} ov_heads={F} k={k} "
            + ("rotary " if positional == "rotary" else "") + "bf16 adam")
    return _autocast_step(m, batch, opt, {}), nb * s, name, (nb * s, d, F, k)


def build_lorsa_rotary(pkg, dev, args):
    """The Lorsa workload with rotary embeddings on queries and keys (the reference's default; the benchmarked Lorsa
    configuration has none): a secondary figure."""
    return build_lorsa(pkg, dev, args, positional="rotary")


def build_crosscoder(pkg, dev, args):
    """Crosscoder: 4 heads (hook points) of d=768, 24576 shared features, k=64 per head, 4096 tokens; head h reads
    activations G(768, r=16, seed 20 + h); decoders start as unit-norm rows, encoders as their transposes."""
    import torch
    from lm_saes_amd import synthetic

    B, H, d, F, k = args.batch or 4096, 4, 768, 24576, 64
    hooks = [f"h{i}" for i in range(H)]
    cfg = pkg.CrosscoderConfig(hook_points=hooks, d_model=d, expansion_factor=F / d, act_fn="topk", top_k=k,
                               norm_activation="inference", device="cuda", dtype=torch.float32)
    m = pkg.Crosscoder(cfg)
    batch = {"tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    for i, hp in enumerate(hooks):
        batch[hp] = synthetic.activations(B, d, 16, seed=20 + i).to(dev)
    with torch.no_grad():
        g = torch.Generator(device=dev).manual_seed(4)
        m.W_D.uniform_(-1.0 / d ** 0.5, 1.0 / d ** 0.5, generator=g)
        m.W_D.div_(m.W_D.norm(dim=-1, keepdim=True))
        m.W_D.mul_(0.5 + torch.rand(H, F, 1, device=dev, generator=g))     # the heads' norms differ, so do their selections
        m.init_encoder_with_decoder_transpose()
        m.b_E.zero_()
        m.b_D.copy_(torch.stack([batch[hp].mean(0) for hp in hooks]))
    opt = pkg.HipAdam(m.get_parameters()[0]["params"], lr=4e-4, model=m)
    name = f"crosscoder_train_step heads={H} d_model={d} d_sae={F} k={k} batch={B} bf16 adam"
    return _autocast_step(m, batch, opt, {}), B, name, (B, d, F, k)


WORKLOADS = {"topk": build_topk, "c1_fp32": build_c1_fp32, "topk_bf16_params": build_topk_bf16_params, "topk_trainer": build_topk_trainer, "activation_stream": build_activation_stream, "batchtopk": build_batchtopk, "batchtopk_bf16_params": build_batchtopk_bf16_params, "jumprelu": build_jumprelu, "jumprelu_sparse": build_jumprelu_sparse, "clt": build_clt,
             "lorsa": build_lorsa, "lorsa_rotary": build_lorsa_rotary, "crosscoder": build_crosscoder}

# the other benchmark configurations a default run times after the headline (a few steps each): the five
# benchmarked configurations, the JumpReLU one in both of its forms, and a crosscoder
CONFIG_RUNS = [("c1_topk_fp32", "c1_fp32", 20), ("c2_batchtopk_auxk", "batchtopk", 12), ("c3_jumprelu_dense", "jumprelu", 5),
               ("c3_jumprelu_sparse", "jumprelu_sparse", 10), ("c4_clt", "clt", 8), ("c5_lorsa", "lorsa", 12),
               ("crosscoder", "crosscoder", 12)]


def step_work(workload: str, shape) -> dict:
    """Algorithmic work PER STEP of kernels whose launches differ in shape inside one step of `workload` (label ->
    (bound, flop or bytes)); a kernel's fraction of its roofline is then that work over its time per step."""
    B, d, F, k = shape
    if workload == "clt":
        L = 12
        blocks = L * (L + 1) // 2
        return {"adam_step_sparse_rows[bf16 dense]": ("hbm", 26.0 * (L + blocks) * F * d),
                "sparse_decode_mse_fused": ("hbm", sum(2.0 * B * (j + 1) * k * d * 2 + 3 * B * d * 4 for j in range(L))),
                "encoder_gemm": ("mfma", 2.0 * B * d * F * L)}
    if workload == "crosscoder":
        H = 4
        return {"adam_step_sparse_rows[bf16 dense]": ("hbm", 26.0 * 2 * H * F * d),
                "sparse_decode_mse_fused": ("hbm", H * (2.0 * B * k * d * 2 + 3 * B * d * 4)),
                "encoder_gemm": ("mfma", 2.0 * B * (H * d) * F)}
    if workload in ("batchtopk", "jumprelu_sparse"):
        return {"adam_step_sparse_rows[bf16 dense]": ("hbm", 26.0 * 2 * F * d)}
    if workload in ("lorsa", "lorsa_rotary"):
        nb, s, h, dq, dv = 16, 1024, 64, 64, 128
        pairs = nb * h * s * (s + 1) // 2
        return {"attention_fwd": ("mfma", 2.0 * pairs * (dq + dv)), "attention_bwd": ("mfma", 2.0 * pairs * (3 * dq + 2 * dv))}
    return {}



def gpu_step_bench(args, workload=None, steps=None, warmup=None):
    import torch
    from __graft_entry__ import load_package

    pkg = load_package()
    dev = torch.device("cuda:0")
    workload = workload or args.workload
    steps = steps or args.steps
    warmup = args.warmup if warmup is None else warmup
    step, tokens, name, shape = WORKLOADS[workload](pkg, dev, args)

    if args.calibrate_copy:
        # a plain device copy of known size (1 GiB read + 1 GiB written), for scaling rocprofv3's
        # FETCH_SIZE / WRITE_SIZE counters when they are collected over this command
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    # Two HIP-event records around every library call cost host time (up to 5 % of a step made of many short launches), so
    # the timed region carries them for ONE kernel only, the one the roofline is quoted on: the warm-up steps run with every
    # call timed and name it, and the per-kernel table comes from a few more steps after the timed region.
    probe = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(probe)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    seen = probe.summary()
    dominant = max(seen, key=lambda n: seen[n]["total_ms"]) if seen else None
    timer = pkg.ops.KernelTimer(only=None if dominant is None else {dominant})
    pkg.ops.set_kernel_timer(timer)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    pkg.ops.set_kernel_timer(None)
    ms_per_step = (t1 - t0) * 1e3 / steps
    kernels = {n: dict(st, steps=steps) for n, st in timer.summary().items()}
    if dominant is not None:
        table = pkg.ops.KernelTimer()
        pkg.ops.set_kernel_timer(table)
        n_table = min(steps, 5)
        for _ in range(n_table):
            step()
        torch.cuda.synchronize()
        pkg.ops.set_kernel_timer(None)
        for n, st in table.summary().items():
            kernels.setdefault(n, dict(st, steps=n_table))
    return ms_per_step, kernels, float(loss.item()), tokens, name, shape


def config_run(args, key: str, workload: str, steps: int) -> dict:
    """One of the other benchmark configurations, timed for a few steps in this process: its step time, throughput and
    the library kernel with the largest share of the step (with its fraction of the roofline that bounds it where every
    launch of it does known work)."""
    import gc

    import torch

    batch, d_sae = args.batch, args.d_sae
    args.batch, args.d_sae = 0, 0
    try:
        ms, kernels, loss, tokens, name, shape = gpu_step_bench(args, workload, steps, 2)
    finally:
        args.batch, args.d_sae = batch, d_sae
    gc.collect()
    torch.cuda.empty_cache()
    dominant = max(kernels, key=lambda n: kernels[n]["total_ms"] / kernels[n]["steps"])
    per_step = step_work(workload, shape)
    uniform = workload in ("c1_fp32", "jumprelu")
    bound = frac = None
    if dominant in LATENCY_BOUND:
        bound = "latency"
    elif dominant in per_step:
        bound, w = per_step[dominant]
        rate = w / (kernels[dominant]["total_ms"] / kernels[dominant]["steps"])
        frac = rate / 1e9 / PEAK_BF16_TFLOPS if bound == "mfma" else rate / 1e6 / PEAK_HBM_GBS
    elif uniform and dominant in algorithmic_work(*shape):
        bound, w = algorithmic_work(*shape)[dominant]
        rate = w / kernels[dominant]["avg_ms"]
        frac = rate / 1e9 / (157.3 if workload == "c1_fp32" else PEAK_BF16_TFLOPS) if bound == "mfma" else rate / 1e6 / PEAK_HBM_GBS
    return {"workload": name, "steps": steps, "ms_per_step": round(ms, 4), "tokens_per_s": round(tokens / (ms / 1e3), 1),
            "dominant_kernel": dominant,
            "dominant_ms_per_step": round(kernels[dominant]["total_ms"] / kernels[dominant]["steps"], 4),
            "bound": bound, "frac": None if frac is None else round(frac, 4),
            "kernel_ms_per_step": round(sum(v["total_ms"] / v["steps"] for v in kernels.values()), 4), "final_loss": loss}


def mfma_probe() -> dict:
    """Rate of back-to-back v_mfma_f32_16x16x32_bf16 from registers: the matrix cores' ceiling on this card at
    the clock it grants, next to the published 2.5 PFLOP/s."""
    import torch
    from __graft_entry__ import load_package

    pkg = load_package()
    dev = torch.device("cuda:0")
    pkg.ops.mfma_probe(dev, 4096, 256)   # warm-up
    best = 0.0
    runs = []
    for _ in range(5):
        flop, ms = pkg.ops.mfma_probe(dev, 4096, 8192)
        runs.append(round(flop / ms / 1e9, 1))
        best = max(best, flop / ms / 1e9)
    return {"probe": "v_mfma_f32_16x16x32_bf16 from registers, 4096 workgroups x 4 waves x 8192 x 32 instructions",
            "tflops_best": round(best, 1), "tflops_runs": runs, "published_peak_tflops": 2500.0}


def gemm_operand_probe() -> dict:
    """The headline encoder product (4096 x 4096 x 131072, bf16) timed with random, zero and constant operands: the same
    kernel, launch and memory traffic each time, so what separates the figures is what the data costs the chip in
    switching power, i.e. in clock."""
    import torch
    from __graft_entry__ import load_package

    pkg = load_package()
    dev = torch.device("cuda:0")
    B, d, F = 4096, D_MODEL, D_SAE
    g = torch.Generator(device=dev).manual_seed(4)
    xr = torch.randn(B, d, device=dev, generator=g).bfloat16()
    wr = (torch.randn(F, d, device=dev, generator=g) / d ** 0.5).bfloat16()

    def timed(x, w, n=10):
        for _ in range(3):
            pkg.ops.encoder_gemm(x, w, torch.bfloat16)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(n):
            pkg.ops.encoder_gemm(x, w, torch.bfloat16)
        end.record()
        end.synchronize()
        return start.elapsed_time(end) / n

    cases = [("random", xr, wr), ("x zero", torch.zeros_like(xr), wr), ("both zero", torch.zeros_like(xr), torch.zeros_like(wr)),
             ("both one", torch.ones_like(xr), torch.ones_like(wr)), ("random again", xr, wr)]
    flop = 2.0 * B * d * F
    out = {"probe": f"sae_encoder_gemm {B} x {d} x {F} bf16, 10 launches per case", "published_peak_tflops": PEAK_BF16_TFLOPS, "cases": {}}
    for name, x, w in cases:
        ms = timed(x, w)
        out["cases"][name] = {"ms": round(ms, 3), "tflops": round(flop / ms / 1e9, 1)}
    return out


def cpu_baseline(sample_batch: int, sample_features: int):
    """Oracle (the reference's eager op sequence on CPU) on a bounded sample of the headline workload: the full
    dictionary (d_model, d_sae, k as on the GPU), `sample_batch` tokens per step instead of 4096 (the host cannot
    finish the full batch in the time a default run has); the reported value is measured, not extrapolated."""
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
    # timed steps until about 12 s of CPU work have been spent (at least 3, at most 20)
    n_timed, t0 = 0, time.perf_counter()
    while n_timed < 3 or (time.perf_counter() - t0 < 12.0 and n_timed < 20):
        oracle.train_step(m, opt, batch, amp_dtype=torch.bfloat16)
        n_timed += 1
    dt = (time.perf_counter() - t0) / n_timed
    return {
        "value": round(sample_batch / dt, 2), "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"1 warm-up + {n_timed} timed steps of the TopK SAE train step at d_model={d} k={k} d_sae={F}"
                  + ("" if F == D_SAE else f" ({F} of the {D_SAE} features)")
                  + f" with B={sample_batch} tokens per step (the GPU step has 4096), fp32 master "
                  f"weights + bf16 autocast on CPU, torch {torch.__version__}, {dt:.2f} s per step",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=0, help="tokens per step (0: the workload's own size)")
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="topk")
    ap.add_argument("--d-sae", type=int, default=0,
                    help="dictionary size of the topk workload (0: 131072, the headline; a smaller one keeps the 32-bit "
                         "hardware counters of a profiling run from saturating and is never the headline metric)")
    ap.add_argument("--cpu-sample-batch", type=int, default=512)
    ap.add_argument("--cpu-sample-features", type=int, default=D_SAE,
                    help="dictionary size of the CPU baseline (default: the full 131072 features)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="headline run only: skip the short runs of the other benchmark configurations")
    ap.add_argument("--calibrate-copy", action="store_true", help="also run three 1 GiB device copies (counter calibration)")
    ap.add_argument("--gemm-operand-probe", action="store_true",
                    help="instead of a train step: the headline encoder product with random, zero and constant operands "
                         "(one JSON line)")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="instead of a train step: the rate of register-only bf16 MFMA loops (one JSON line)")
    ap.add_argument("--clip", type=float, default=0.0, help="clip_grad_norm of the topk_trainer workload (0: norm only)")
    ap.add_argument("--overlap", action="store_true", help="run the decoder Adam pass on a second stream, overlapping the next GEMM")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collectives are part of it); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    if args.gemm_operand_probe:
        print(json.dumps(gemm_operand_probe()))
        return
    if args.mfma_probe:
        print(json.dumps(mfma_probe()))
        return

    ms_per_step, kernels, loss, tokens, name, shape = gpu_step_bench(args)
    work = algorithmic_work(*shape)
    if args.workload in ("topk_bf16_params", "batchtopk_bf16_params"):   # bf16 p, m, v read and written; no shadow copy
        work["adam_step_sparse_rows[bf16 dense]"] = ("hbm", shape[1] * shape[2] * 12)
        work["adam_step[vector]"] = ("hbm", (shape[1] + shape[2]) / 2 * 14)
    known = {}     # launches whose work is known although the workload runs other kernels on several shapes
    if args.workload in ("lorsa", "lorsa_rotary"):
        # causal attention of build_lorsa's shape: (query, key) pairs with key <= query, 2 flop per multiply-add;
        # forward = scores + weighted values; backward = scores again, dP, dV, dK, dQ (the algorithmic minimum: the
        # three backward kernels each recompute the scores they need)
        nb, s, h, dq, dv = 16, 1024, 64, 64, 128
        pairs = nb * h * s * (s + 1) // 2
        known = {"attention_fwd": ("mfma", 2.0 * pairs * (dq + dv)), "attention_bwd": ("mfma", 2.0 * pairs * (3 * dq + 2 * dv))}
        work.update(known)
    dominant = max(kernels, key=lambda n: kernels[n]["total_ms"] / kernels[n]["steps"])
    bound, per_launch = work.get(dominant, ("hbm", 0.0))
    avg_ms = kernels[dominant]["avg_ms"]
    if bound == "mfma":
        achieved, peak, unit = per_launch / avg_ms / 1e9, PEAK_BF16_TFLOPS, "TFLOP/s"
    else:
        achieved, peak, unit = per_launch / avg_ms / 1e6, PEAK_HBM_GBS, "GB/s"
    traffic = measured_traffic_gb(dominant) if args.workload in ("topk", "topk_trainer") and not args.d_sae and not args.batch else None
    roofline = {
        "kernel": dominant, "bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
        "frac": round(achieved / peak, 4), "traffic": None if traffic is None else traffic * 1e9,
        "traffic_source": None if traffic is None else HBM_TRAFFIC_FILE, "avg_ms": round(avg_ms, 4),
        "launches_per_step": kernels[dominant]["calls"] / kernels[dominant]["steps"],
    }
    per_kernel = {}
    # one dictionary shape for every launch of a kernel (the aux-k branch of "batchtopk" runs the GEMM and the
    # select on its compact block of dead features as well, CLT and Lorsa on several shapes)
    uniform = args.workload in ("topk", "topk_bf16_params", "topk_trainer", "jumprelu", "activation_stream")
    for kname, st in kernels.items():
        bnd, w = work.get(kname, ("hbm", 0.0)) if uniform or kname in known else ("hbm", 0.0)
        if kname in LATENCY_BOUND:
            bnd, w = "latency", 0.0
        rate = w / st["avg_ms"] / (1e9 if bnd == "mfma" else 1e6) if w else None
        per_kernel[kname] = {
            "ms_per_step": round(st["total_ms"] / st["steps"], 4), "avg_ms": round(st["avg_ms"], 4),
            "launches_per_step": st["calls"] / st["steps"], "bound": bnd,
            "achieved": None if rate is None else round(rate, 1),
            "frac": None if rate is None else round(rate / (PEAK_BF16_TFLOPS if bnd == "mfma" else PEAK_HBM_GBS), 4),
        }
    if not uniform and dominant not in known:
        roofline.update(achieved=None, frac=None)   # launches of different shapes share a label: no single per-launch figure
    headline = args.workload == "topk" and not args.d_sae and not args.batch
    out = {
        "metric": "train tokens/s, TopK SAE d=4096 F=131072 k=64 bf16; % MFMA / HBM roofline" if headline
                  else f"train tokens/s, {args.workload} workload (not the headline metric)",
        "value": round(tokens / (ms_per_step / 1e3), 1),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": name, "batch_tokens": tokens},
        "roofline": roofline,
        "kernels": per_kernel,
        "kernel_ms_per_step": round(sum(v["ms_per_step"] for v in per_kernel.values()), 4),
        "final_loss": loss,
    }
    if headline and not args.no_configs:
        # the other configurations, a few steps each: not part of `value`, measured after its timed region
        import gc

        import torch

        gc.collect()
        torch.cuda.empty_cache()
        out["configs"] = {key: config_run(args, key, workload, steps) for key, workload, steps in CONFIG_RUNS}
    if headline and not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.cpu_sample_batch, args.cpu_sample_features)
        out["cpu_baseline_c1"] = cpu_baseline_c1()   # the configuration the reference's CPU path runs at full shape
    if args.workload == "c1_fp32" and not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_c1()
        out["dtype"] = "f32"
    print(json.dumps(out))


if __name__ == "__main__":
    main()
