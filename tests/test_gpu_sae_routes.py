"""Routes of `SparseAutoEncoder.compute_loss` that the kernels cover beside the plain 2-D TopK step: activations with a
sequence axis ([batch, seq_len, d_model], models/sae.py:288-345), a ReLU dictionary on the JumpReLU kernels, and TopK /
BatchTopK with one of the sparsity penalties (models/sparse_dictionary.py:888-925) formed on the sparse code.  Each against
the oracle (its encoder product takes the kernel's forward values, so that last-bit differences of the two GEMMs cannot
flip a selection), with an assertion on the kernels that ran.
"""

import contextlib
import math

import pytest
import torch

from test_gpu_sae_step import _SubstitutedMatmul, rel_err

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5
GRAD_TOL = 1e-4
BF16_TOL = 2e-2


def make_models(pkg, oracle, dev, act_fn, d, F, k, seed, include_norm=True, window=0.3, log_theta=-1.0):
    from lm_saes_amd import synthetic

    x = synthetic.activations(64, d, 8, seed)
    w = synthetic.sae_weights(d, F, x, seed)
    g = torch.Generator().manual_seed(seed + 1)
    W_D = (w[2] * (0.5 + torch.rand(F, 1, generator=g))).contiguous()
    b_E = 0.02 * torch.randn(F, generator=g)
    w = (w[0], b_E, W_D, w[3])
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn=act_fn, top_k=k,
                        norm_activation="inference", sparsity_include_decoder_norm=include_norm, jumprelu_threshold_window=window,
                        device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    synthetic.load_weights(sae, *[t.to(dev) for t in w])
    ref = oracle.SAEOracle(d, F, act_fn=act_fn, top_k=k, sparsity_include_decoder_norm=include_norm, jumprelu_threshold_window=window)
    synthetic.load_weights(ref, *w)
    if act_fn == "jumprelu":
        with torch.no_grad():
            t = log_theta + 0.3 * torch.randn(F, generator=g)
            sae.activation_function.log_jumprelu_threshold.copy_(t.to(dev))
            ref.activation_function.log_jumprelu_threshold.copy_(t)
    return sae, ref


@contextlib.contextmanager
def kernel_names(pkg):
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    try:
        yield timer.records
    finally:
        torch.cuda.synchronize()
        pkg.ops.set_kernel_timer(None)


def run_both(pkg, dev, sae, ref, batch, kw, amp=False, stats=None):
    """-> (ctx, rctx, kernel names): one loss + backward on each side; the oracle's encoder product takes the GEMM kernel's
    forward values."""
    gb = {k_: v.to(dev) for k_, v in batch.items()}
    kw_g, kw_r = dict(kw), dict(kw)
    if stats is not None:
        kw_g["update_dead_statistics"], kw_r["update_dead_statistics"] = stats
    with kernel_names(pkg) as names, (torch.autocast("cuda", dtype=torch.bfloat16) if amp else contextlib.nullcontext()):
        ctx = sae.compute_loss(gb, **kw_g)
        ctx["loss"].backward()
    names = set(names)
    x2 = gb["in"].reshape(-1, gb["in"].shape[-1]).contiguous()
    if amp:
        pre = pkg.ops.encoder_gemm(pkg.ops.cast_bf16(x2), sae._w_enc_operand(True), torch.bfloat16).cpu()
    else:
        pre = pkg.ops.encoder_gemm(x2, sae._w_enc_operand(False), torch.float32).cpu()

    def encode_sub(x, return_hidden_pre=False, **_):
        lead = x.shape[:-1]
        xx = x.reshape(-1, x.shape[-1]).to(ref.W_E.dtype)
        mm = _SubstitutedMatmul.apply(xx.to(pre.dtype), ref.W_E.to(pre.dtype), pre).reshape(*lead, -1)
        hidden_pre = mm + ref.b_E
        if ref.sparsity_include_decoder_norm:
            hidden_pre = hidden_pre * ref.decoder_norm()
        fa = ref.activation_function(hidden_pre)
        if ref.sparsity_include_decoder_norm:
            fa = fa / ref.decoder_norm()
            hidden_pre = hidden_pre / ref.decoder_norm()
        return (fa, hidden_pre) if return_hidden_pre else fa

    ref.encode = encode_sub
    with (torch.autocast("cpu", dtype=torch.bfloat16) if amp else contextlib.nullcontext()):
        rctx = ref.compute_loss(batch, **kw_r)
    rctx["loss"].backward()
    return ctx, rctx, names


def compare(sae, ref, ctx, rctx, tol, gtol, pkg=None):
    assert torch.equal((ctx["feature_acts"] != 0).cpu(), rctx["feature_acts"] != 0), "selected index sets differ"
    assert ctx["feature_acts"].shape == rctx["feature_acts"].shape and ctx["reconstructed"].shape == rctx["reconstructed"].shape
    assert rel_err(ctx["feature_acts"], rctx["feature_acts"]) < tol
    assert rel_err(ctx["reconstructed"], rctx["reconstructed"]) < tol
    assert abs(ctx["loss"].item() - rctx["loss"].item()) < tol * abs(rctx["loss"].item())
    for key in ("l_rec", "l_s"):
        if rctx.get(key) is not None:
            assert ctx[key] is not None, key
            assert rel_err(ctx[key].float().mean(), rctx[key].float().mean()) < tol, key
    if pkg is not None:
        pkg.optim.fold_row_grad_coef(list(sae.parameters()))
    for name, p in sae.named_parameters():
        want = dict(ref.named_parameters())[name].grad
        assert p.grad is not None, name
        assert rel_err(p.grad, want) < gtol, (name, rel_err(p.grad, want))


# ---- activations with a sequence axis ---------------------------------------------------------------------------------

@pytest.mark.parametrize("act_fn,kw", [("topk", {}), ("batchtopk", {}), ("jumprelu", dict(sparsity_loss_type="tanh", l1_coefficient=0.05)),
                                       ("topk", dict(sparsity_loss_type="tanh", l1_coefficient=0.05))])
@pytest.mark.parametrize("masked", [False, True])
def test_sequence_shaped_activations_take_the_kernel_step(pkg, oracle, dev, act_fn, kw, masked):
    from lm_saes_amd import synthetic

    b, s, d, F, k = 4, 48, 128, 1024, 8
    sae, ref = make_models(pkg, oracle, dev, act_fn, d, F, k, seed=11)
    x = synthetic.activations(b * s, d, 8, seed=12).view(b, s, d)
    batch = {"in": x, "out": x, "tokens": torch.zeros(b, s, dtype=torch.long)}
    if masked:
        batch["mask"] = (torch.rand(b, s, generator=torch.Generator().manual_seed(13)) > 0.25).float()
    ctx, rctx, names = run_both(pkg, dev, sae, ref, batch, kw)
    assert "encoder_gemm" in names and ({"sparse_decode_mse_fused", "jumprelu_fwd"} & names), names
    assert ctx["reconstructed"].shape == (b, s, d) and ctx["feature_acts"].shape == (b, s, F)
    assert ctx["n_tokens"] == rctx["n_tokens"]
    if act_fn == "batchtopk":
        assert int((ctx["feature_acts"] != 0).sum()) == k * b * s
    compare(sae, ref, ctx, rctx, FP32_TOL, GRAD_TOL)


def test_sequence_shaped_activations_with_auxk(pkg, oracle, dev):
    from lm_saes_amd import synthetic

    b, s, d, F, k = 3, 64, 128, 1024, 8
    sae, ref = make_models(pkg, oracle, dev, "topk", d, F, k, seed=21)
    x = synthetic.activations(b * s, d, 8, seed=22).view(b, s, d)
    batch = {"in": x, "out": x, "tokens": torch.zeros(b, s, dtype=torch.long)}
    trainer_stats = pkg.Trainer(pkg.TrainerConfig(total_training_tokens=10 ** 6, auxk_coefficient=0.1, dead_threshold=b * s))
    trainer_stats.tokens_since_last_activation = torch.zeros(F, dtype=torch.int64, device=dev)
    trainer_stats.is_dead = torch.zeros(F, dtype=torch.bool, device=dev)
    rstats = oracle.DeadStatistics(F, dead_threshold=b * s)
    ctx, rctx, names = run_both(pkg, dev, sae, ref, batch, dict(auxk_coefficient=0.1, k_aux=16),
                                stats=(trainer_stats.update_dead_statistics, rstats.update))
    assert "sparse_decode_fwd" in names or "sparse_decode_mse_fused" in names
    assert torch.equal(trainer_stats.is_dead.cpu(), rstats.is_dead)
    assert rel_err(ctx["l_aux"], rctx["l_aux"]) < FP32_TOL
    compare(sae, ref, ctx, rctx, FP32_TOL, GRAD_TOL)


# ---- a ReLU dictionary on the JumpReLU kernels ------------------------------------------------------------------------

@pytest.mark.parametrize("kw", [{}, dict(sparsity_loss_type="power", p=1, l1_coefficient=0.01), dict(sparsity_loss_type="tanh", l1_coefficient=0.02),
                                dict(sparsity_loss_type="tanh-quad", l1_coefficient=0.02, frequency_scale=0.05)])
@pytest.mark.parametrize("include_norm", [False, True])
def test_relu_dictionary_runs_the_activation_kernels(pkg, oracle, dev, kw, include_norm):
    from lm_saes_amd import synthetic

    B, d, F = 96, 128, 1024
    sae, ref = make_models(pkg, oracle, dev, "relu", d, F, 8, seed=31, include_norm=include_norm)
    x = synthetic.activations(B, d, 8, seed=32)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long), "mask": (torch.arange(B) % 5 != 0).float()}
    ctx, rctx, names = run_both(pkg, dev, sae, ref, batch, kw)
    assert {"encoder_gemm", "jumprelu_fwd", "jumprelu_bwd"} <= names, names
    compare(sae, ref, ctx, rctx, FP32_TOL, GRAD_TOL)


def test_relu_dictionary_under_autocast(pkg, oracle, dev):
    from lm_saes_amd import synthetic

    B, d, F = 128, 128, 1024
    sae, ref = make_models(pkg, oracle, dev, "relu", d, F, 8, seed=33)
    x = synthetic.activations(B, d, 8, seed=34)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long)}
    ctx, rctx, names = run_both(pkg, dev, sae, ref, batch, dict(sparsity_loss_type="tanh", l1_coefficient=0.02), amp=True)
    assert {"encoder_gemm", "jumprelu_fwd", "jumprelu_bwd"} <= names, names
    assert abs(ctx["loss"].item() - rctx["loss"].item()) < BF16_TOL * abs(rctx["loss"].item())
    assert rel_err(ctx["reconstructed"], rctx["reconstructed"]) < BF16_TOL
    for name, p in sae.named_parameters():
        assert rel_err(p.grad, dict(ref.named_parameters())[name].grad) < BF16_TOL, name


def test_sparse_relu_dictionary_takes_the_sparse_form(pkg, oracle, dev):
    """A ReLU dictionary whose biases leave a few features active per token: the step's sparse form (threshold select with
    a threshold of zero, sparse decode, factored gradients), with every penalty on the code."""
    from lm_saes_amd import synthetic

    B, d, F = 96, 128, 2048
    for kw in ({}, dict(sparsity_loss_type="power", p=2, l1_coefficient=0.01), dict(sparsity_loss_type="tanh-quad", l1_coefficient=0.02)):
        sae, ref = make_models(pkg, oracle, dev, "relu", d, F, 8, seed=35)
        x = synthetic.activations(B, d, 8, seed=36)
        with torch.no_grad():      # biases that leave about 2 % of the pre-activations positive
            shift = torch.quantile((x @ ref.W_E + ref.b_E).flatten()[:: 7], 0.98).item()
            sae.b_E.sub_(shift)
            ref.b_E.sub_(shift)
        sae.cfg.sparsity_threshold_for_triton_spmm_kernel = 0.9
        batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long)}
        ctx, rctx, names = run_both(pkg, dev, sae, ref, batch, kw)
        assert "sparse_code" in ctx and "sparse_decode_mse_fused" in names and "jumprelu_fwd" not in names, names
        density = (rctx["feature_acts"] != 0).float().mean().item()
        assert 0 < density < 0.1, density
        compare(sae, ref, ctx, rctx, FP32_TOL, GRAD_TOL)


# ---- TopK / BatchTopK with a sparsity penalty ------------------------------------------------------------------------------

PENALTIES = [dict(sparsity_loss_type="tanh", l1_coefficient=0.05, tanh_stretch_coefficient=3.0),
             dict(sparsity_loss_type="power", p=1, l1_coefficient=0.02),
             dict(sparsity_loss_type="power", p=2, l1_coefficient=0.02),
             dict(sparsity_loss_type="tanh-quad", l1_coefficient=0.05, frequency_scale=0.05)]


@pytest.mark.parametrize("kw", PENALTIES, ids=["tanh", "l1", "l2", "tanh-quad"])
@pytest.mark.parametrize("act_fn,include_norm,masked", [("topk", True, False), ("topk", False, True), ("batchtopk", True, True)])
def test_topk_with_a_sparsity_penalty_on_the_sparse_code(pkg, oracle, dev, kw, act_fn, include_norm, masked):
    from lm_saes_amd import synthetic

    B, d, F, k = 160, 128, 1024, 8
    sae, ref = make_models(pkg, oracle, dev, act_fn, d, F, k, seed=41, include_norm=include_norm)
    x = synthetic.activations(B, d, 8, seed=42)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long)}
    if masked:
        batch["mask"] = (torch.rand(B, generator=torch.Generator().manual_seed(43)) > 0.3).float()
    ctx, rctx, names = run_both(pkg, dev, sae, ref, batch, dict(kw, lp_coefficient=0.3))     # an Lp coefficient is ignored for TopK
    assert "sparse_code" in ctx and {"sparse_decode_mse_fused", "build_feature_index"} <= names, names
    assert not ({"jumprelu_fwd", "dense_to_code"} & names), names
    assert rctx["l_p"] is None and ctx["l_p"] is None
    compare(sae, ref, ctx, rctx, FP32_TOL, GRAD_TOL)


def test_topk_with_a_penalty_hands_factored_gradients_to_the_optimizer(pkg, oracle, dev):
    """With HipAdam attached the two weight gradients stay factored and the penalty's decoder-norm term rides along as a
    per-row coefficient; after one step the parameters equal torch's Adam on the oracle's dense gradients."""
    from lm_saes_amd import synthetic

    B, d, F, k = 128, 128, 1024, 8
    sae, ref = make_models(pkg, oracle, dev, "topk", d, F, k, seed=51)
    x = synthetic.activations(B, d, 8, seed=52)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long)}
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=1e-3, model=sae)
    ropt = torch.optim.Adam(ref.parameters(), lr=1e-3)
    kw = dict(sparsity_loss_type="tanh", l1_coefficient=0.05)
    ctx, rctx, names = run_both(pkg, dev, sae, ref, batch, kw, amp=True)
    assert getattr(sae.W_D, "_sparse_grad", None) is not None and getattr(sae.W_D, "_row_grad_coef", None) is not None
    before = {n: p.detach().clone() for n, p in sae.named_parameters()}
    opt.step()
    ropt.step()
    rp = dict(ref.named_parameters())
    for n, p in sae.named_parameters():
        moved, want = (p.detach() - before[n]).cpu(), rp[n].detach() - before[n].cpu()
        # first Adam step: lr * sign(g) wherever the gradient is resolved; both sides must agree where the oracle's
        # gradient is not within rounding of zero
        g = rp[n].grad
        resolved = g.abs() > 1e-2 * g.abs().max()
        assert (moved - want)[resolved].abs().max().item() < 0.05 * 1e-3, n


# ---- gated (GLU) encoder on the sparse step ----------------------------------------------------------------------------------

def make_glu_models(pkg, oracle, dev, act_fn, d, F, k, B, seed):
    from lm_saes_amd import synthetic

    x = synthetic.activations(B, d, 8, seed)
    w = synthetic.sae_weights(d, F, x, seed)
    g = torch.Generator().manual_seed(seed + 1)
    W_D = (w[2] * (0.5 + torch.rand(F, 1, generator=g))).contiguous()
    w = (w[0], 0.02 * torch.randn(F, generator=g), W_D, w[3])
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn=act_fn, top_k=k,
                        norm_activation="inference", sparsity_include_decoder_norm=True, use_glu_encoder=True, device="cuda",
                        dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    synthetic.load_weights(sae, *[t.to(dev) for t in w])
    ref = oracle.SAEOracle(d, F, act_fn=act_fn, top_k=k, sparsity_include_decoder_norm=True, use_glu_encoder=True)
    synthetic.load_weights(ref, *w)
    with torch.no_grad():
        wg, bg = torch.randn(d, F, generator=g) / d ** 0.5, 0.1 * torch.randn(F, generator=g)
        sae.W_E_glu.copy_(wg.to(dev)); sae.b_E_glu.copy_(bg.to(dev))
        ref.W_E_glu.copy_(wg); ref.b_E_glu.copy_(bg)
    return sae, ref, x


@pytest.mark.parametrize("act_fn", ["topk", "batchtopk"])
def test_glu_encoder_takes_the_sparse_step_fp32(pkg, oracle, dev, act_fn):
    """hidden_pre = (x W_E + b_E) * sigmoid(x W_E_glu + b_E_glu) (models/sae.py:326-331) with a token mask: select, fused
    decode + loss and gathered gradient rows for W_E, W_E_glu and W_D; loss, outputs and all six gradients against the
    oracle."""
    d, F, k, B = 64, 512, 8, 96
    sae, ref, x = make_glu_models(pkg, oracle, dev, act_fn, d, F, k, B, seed=71)
    g = torch.Generator().manual_seed(72)
    mask = (torch.rand(B, generator=g) > 0.2).float()
    batch = {"in": x, "out": torch.tanh(x), "tokens": torch.zeros(B), "mask": mask}
    with kernel_names(pkg) as names:
        out = sae.compute_loss({k_: v.to(dev) for k_, v in batch.items()})
        out["loss"].backward()
    names = set(names)
    assert {"sparse_decode_mse_fused", "build_feature_index"} <= names and any(n.startswith("sparse_grad_rows") for n in names), names
    assert "sparse_code" in out
    want = ref.compute_loss(batch)
    want["loss"].backward()
    assert torch.equal((out["feature_acts"] != 0).cpu(), want["feature_acts"] != 0)
    if act_fn == "batchtopk":
        assert len(set((out["feature_acts"] != 0).sum(-1).tolist())) > 1
    for key in ("loss", "feature_acts", "hidden_pre", "reconstructed"):
        assert rel_err(out[key], want[key]) < FP32_TOL, key
    got, exp = dict(sae.named_parameters()), dict(ref.named_parameters())
    assert set(got) == set(exp) and len(got) == 6
    for n, p in exp.items():
        assert got[n].grad is not None and tuple(got[n].grad.shape) == tuple(p.shape), n
        assert rel_err(got[n].grad, p.grad) < GRAD_TOL, (n, rel_err(got[n].grad, p.grad))


def test_glu_encoder_sparse_step_under_autocast(pkg, oracle, dev):
    """bf16 autocast: the sparse step against the module's generic op sequence, whose two encoder products are the same
    kernel launches (the same gated pre-activations, hence the same selection) and whose backward is dense bf16 products."""
    d, F, k, B = 128, 1024, 16, 128
    sae, _, x = make_glu_models(pkg, oracle, dev, "topk", d, F, k, B, seed=73)
    batch = {"in": x.to(dev), "out": torch.tanh(x).to(dev), "tokens": torch.zeros(B, device=dev)}
    with kernel_names(pkg) as names, torch.autocast("cuda", dtype=torch.bfloat16):
        out = sae.compute_loss(batch)
        out["loss"].backward()
    assert "sparse_decode_mse_fused" in set(names)
    fused = {n: p.grad.clone() for n, p in sae.named_parameters()}
    for p in sae.parameters():
        p.grad = None
    with torch.autocast("cuda", dtype=torch.bfloat16):
        want = pkg.SparseDictionary.compute_loss(sae, batch)
    want["loss"].backward()
    assert torch.equal(out["feature_acts"] != 0, want["feature_acts"] != 0)
    # (h n) / n with the norms of the row-norm kernel or of torch.norm: equal to a rounding of the product and the quotient
    assert rel_err(out["hidden_pre"], want["hidden_pre"]) < 1e-6
    assert rel_err(out["reconstructed"], want["reconstructed"]) < BF16_TOL
    assert abs(out["loss"].item() - want["loss"].item()) < BF16_TOL * want["loss"].item()
    for n, p in sae.named_parameters():
        assert rel_err(fused[n], p.grad) < BF16_TOL, (n, rel_err(fused[n], p.grad))


def test_glu_encoder_sparse_step_over_adam_steps(pkg, oracle, dev):
    """Three optimisation steps of the gated dictionary with HipAdam (dense gradient rows from the sparse step; under autocast
    the gate's bf16 operand is re-derived after every update) against torch.optim.Adam on the oracle."""
    d, F, k, B = 64, 512, 8, 96
    sae, ref, x = make_glu_models(pkg, oracle, dev, "topk", d, F, k, B, seed=75)
    batch = {"in": x, "out": torch.tanh(x), "tokens": torch.zeros(B)}
    gb = {k_: v.to(dev) for k_, v in batch.items()}
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=1e-3, model=sae)
    ropt = oracle.make_adam(ref, lr=1e-3)
    for step in range(3):
        out = sae.compute_loss(gb)
        assert "sparse_code" in out
        out["loss"].backward()
        want = ref.compute_loss(batch)
        want["loss"].backward()
        assert rel_err(out["loss"], want["loss"]) < 1e-4, step
        opt.step(); opt.zero_grad()
        ropt.step(); ropt.zero_grad()
        for (n, p), q in zip(sae.named_parameters(), ref.parameters()):
            assert (p.detach().cpu() - q.detach()).abs().max() <= 2e-2 * 1e-3 * (step + 1) + 1e-6 * q.detach().abs().max(), (step, n)
    with torch.autocast("cuda", dtype=torch.bfloat16):      # the bf16 operands follow the updated weights
        sae.compute_loss(gb, return_aux_data=False)
    assert torch.equal(sae._w_glu_operand(True), sae.W_E_glu.detach().t().contiguous().to(torch.bfloat16))
