"""JumpReLU kernels (forward, straight-through backward, tanh / Lp penalty sums) and the JumpReLU train
step of the SAE module against the oracle.

Kernel level: the oracle's STEFunction / JumpReLU under autograd on CPU, composed exactly as the
reference's encoder and loss compose them (scale by the decoder norm, activate, unscale; tanh and Lp
penalties), is differentiated with respect to the pre-activation, bias, threshold and norm.
Step level: SAEOracle with act_fn="jumprelu" against the module's compute_loss.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5
GRAD_TOL = 1e-4
BF16_TOL = 2e-2


def rel_err(got, want):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def oracle_terms(oracle, pre, b, n, log_theta, window, c, pen=None):
    """acts, tanh_tok, lp_tok as the reference composes them (models/sae.py:136-160,
    models/sparse_dictionary.py:893-894, 927-938)."""
    jr = oracle.JumpReLU(window, (pre.shape[1],))
    jr.log_jumprelu_threshold = log_theta
    h = pre + b
    u = h * n if n is not None else h
    acts = jr(u)
    if n is not None:
        acts = acts / n
        hidden_pre = u / n
    else:
        hidden_pre = u
    one = pen if pen is not None else torch.ones_like(b)
    tanh_tok = torch.tanh(c * acts * one).sum(-1)
    lp_tok = (torch.nn.functional.relu(jr.get_jumprelu_threshold() - hidden_pre) * one).sum(-1)
    return acts, tanh_tok, lp_tok


@pytest.mark.parametrize("B,F", [(70, 512), (129, 1024), (64, 2056)])
@pytest.mark.parametrize("with_scale", [True, False])
def test_jumprelu_kernels_fp32(pkg, oracle, dev, B, F, with_scale):
    ops = pkg.ops
    g = torch.Generator().manual_seed(B + F)
    pre = torch.randn(B, F, generator=g).requires_grad_()
    b = (0.1 * torch.randn(F, generator=g)).requires_grad_()
    pen = (0.5 + torch.rand(F, generator=g)).requires_grad_()       # the decoder norm: always weighs the penalties,
    n = pen if with_scale else None                                  # scales the activation only when configured
    log_theta = torch.nn.Parameter(torch.log(0.05 + 0.5 * torch.rand(F, generator=g)))
    window, c = 0.4, 1.7
    acts, tanh_tok, lp_tok = oracle_terms(oracle, pre, b, n, log_theta, window, c, pen=pen)
    d_acts = torch.randn(B, F, generator=g)
    g_tanh, g_lp = torch.rand(B, generator=g), torch.rand(B, generator=g)
    ((acts * d_acts).sum() + (tanh_tok * g_tanh).sum() + (lp_tok * g_lp).sum()).backward()

    to = lambda t: None if t is None else t.detach().to(dev).contiguous()  # noqa: E731
    theta = log_theta.detach().exp()
    a, tt, lt, l0 = ops.jumprelu_fwd(to(pre), to(b), to(n), to(theta), c, pen_norm=to(pen), want_tanh=True, want_lp=True,
                                     want_l0=True)
    assert torch.equal((a > 0).cpu(), acts.detach() > 0) or torch.equal((a != 0).cpu(), acts.detach() != 0)
    assert rel_err(a, acts) < FP32_TOL
    assert rel_err(tt, tanh_tok) < FP32_TOL and rel_err(lt, lp_tok) < FP32_TOL
    assert torch.equal(l0.cpu(), (acts.detach() != 0).sum(-1).float())
    d_pre, d_bias, d_theta, d_norm = ops.jumprelu_bwd(to(pre), to(b), to(n), to(theta), to(d_acts), to(g_tanh), c, to(g_lp),
                                                      window, pen_norm=to(pen), want_norm_grad=True)
    assert rel_err(d_pre, pre.grad) < FP32_TOL
    assert rel_err(d_bias, b.grad) < GRAD_TOL
    assert rel_err(d_theta * theta.to(dev), log_theta.grad) < GRAD_TOL      # chain rule through exp()
    assert (log_theta.grad != 0).float().mean() > 0.5                         # the window did catch entries
    assert rel_err(d_norm, pen.grad) < GRAD_TOL      # penalty terms only: the activation's two norm terms cancel
    # without the penalty terms: plain STE
    pre.grad = b.grad = log_theta.grad = None
    acts2, _, _ = oracle_terms(oracle, pre, b, pen.detach() if with_scale else None, log_theta, window, c)
    (acts2 * d_acts).sum().backward()
    d_pre2, d_bias2, d_theta2, _ = ops.jumprelu_bwd(to(pre), to(b), to(n), to(theta), to(d_acts), None, 0.0, None, window)
    assert rel_err(d_pre2, pre.grad) < FP32_TOL
    assert rel_err(d_theta2 * theta.to(dev), log_theta.grad) < GRAD_TOL


def test_jumprelu_special_cases(pkg, dev):
    """Closed forms of the estimator: no entry inside the window -> zero threshold gradient; non-positive
    inputs never contribute to it; kept entries pass the gradient unchanged, dropped entries block it."""
    ops = pkg.ops
    F = 16
    theta = torch.full((F,), 0.5, device=dev)
    pre = torch.tensor([[2.0] * 8 + [-3.0] * 8, [0.55] * 8 + [0.45] * 8], device=dev)      # row 0 far away, row 1 inside
    d_acts = torch.ones(2, F, device=dev)
    a, _, _, _ = ops.jumprelu_fwd(pre, None, None, theta)
    assert torch.equal(a, torch.where(pre > 0.5, pre, torch.zeros_like(pre)))
    d_pre, d_bias, d_theta, _ = ops.jumprelu_bwd(pre[:1].contiguous(), None, None, theta, d_acts[:1].contiguous(), None, 0.0,
                                                 None, 0.2)
    assert torch.all(d_theta == 0) and torch.equal(d_pre, (pre[:1] > 0.5).float())
    d_pre, d_bias, d_theta, _ = ops.jumprelu_bwd(pre, None, None, theta, d_acts, None, 0.0, None, 0.2)
    assert torch.allclose(d_theta, torch.full((F,), -0.5 / 0.2, device=dev))               # one in-window row: -theta / eps
    assert torch.equal(d_bias, torch.tensor([2.0] * 8 + [0.0] * 8, device=dev))
    neg = torch.full((1, F), -0.01, device=dev)      # within the window of a tiny threshold but not positive
    _, _, d_theta, _ = ops.jumprelu_bwd(neg, None, None, torch.full((F,), 0.001, device=dev), d_acts[:1].contiguous(), None,
                                        0.0, None, 0.1)
    assert torch.all(d_theta == 0)
    with pytest.raises(RuntimeError):
        ops.jumprelu_fwd(torch.zeros(2, 12, device=dev), None, None, torch.zeros(12, device=dev))   # F not a multiple of 8


def test_jumprelu_kernels_bf16(pkg, oracle, dev):
    ops = pkg.ops
    B, F = 96, 1024
    g = torch.Generator().manual_seed(7)
    pre = torch.randn(B, F, generator=g).bfloat16()
    b = 0.1 * torch.randn(F, generator=g)
    n = 0.5 + torch.rand(F, generator=g)
    theta = 0.05 + 0.5 * torch.rand(F, generator=g)
    d_acts = torch.randn(B, F, generator=g).bfloat16()
    pre32 = pre.float().requires_grad_()
    log_theta = torch.nn.Parameter(theta.log())
    acts, _, _ = oracle_terms(oracle, pre32, b, n, log_theta, 0.4, 1.0, pen=n)
    (acts * d_acts.float()).sum().backward()
    a, _, _, _ = ops.jumprelu_fwd(pre.to(dev), b.to(dev), n.to(dev), theta.to(dev))
    assert a.dtype == torch.bfloat16 and rel_err(a, acts) < BF16_TOL
    d_pre, d_bias, d_theta, _ = ops.jumprelu_bwd(pre.to(dev), b.to(dev), n.to(dev), theta.to(dev), d_acts.to(dev), None, 0.0,
                                                 None, 0.4)
    assert d_pre.dtype == torch.bfloat16 and rel_err(d_pre, pre32.grad) < BF16_TOL
    assert rel_err(d_theta * theta.to(dev), log_theta.grad) < GRAD_TOL       # sums are fp32 on both sides


def make_pair(pkg, oracle, dev, d, F, B, seed, include_norm, window):
    from lm_saes_amd import synthetic

    x = synthetic.activations(B, d, 8, seed)
    w = synthetic.sae_weights(d, F, x, seed)
    g = torch.Generator().manual_seed(seed + 1)
    W_D = (w[2] * (0.5 + torch.rand(F, 1, generator=g))).contiguous()
    b_E = 0.02 * torch.randn(F, generator=g)
    w = (w[0], b_E, W_D, w[3])
    log_theta = torch.log(0.02 + 0.3 * torch.rand(F, generator=g))
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="jumprelu",
                        jumprelu_threshold_window=window, norm_activation="inference",
                        sparsity_include_decoder_norm=include_norm, device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    synthetic.load_weights(sae, *[t.to(dev) for t in w])
    ref = oracle.SAEOracle(d, F, act_fn="jumprelu", jumprelu_threshold_window=window,
                           sparsity_include_decoder_norm=include_norm)
    synthetic.load_weights(ref, *w)
    with torch.no_grad():
        sae.activation_function.log_jumprelu_threshold.copy_(log_theta.to(dev))
        ref.activation_function.log_jumprelu_threshold.copy_(log_theta)
    y = x + 0.1 * torch.randn(B, d, generator=g)
    batch = {"in": x, "out": y, "tokens": torch.zeros(B, dtype=torch.long),
             "mask": (torch.rand(B, generator=g) > 0.25).float()}
    return sae, ref, batch


def named_grads(m):
    out = {n: p.grad for n, p in m.named_parameters()}
    return {k.replace("activation_function.", ""): v for k, v in out.items()}


@pytest.mark.parametrize("include_norm", [True, False])
@pytest.mark.parametrize("kw", [dict(), dict(sparsity_loss_type="tanh", l1_coefficient=0.05, tanh_stretch_coefficient=2.0),
                                dict(sparsity_loss_type="tanh", l1_coefficient=0.05, lp_coefficient=0.01)])
def test_jumprelu_step_fp32_matches_oracle(pkg, oracle, dev, include_norm, kw):
    d, F, B = 64, 512, 96
    sae, ref, batch = make_pair(pkg, oracle, dev, d, F, B, seed=11, include_norm=include_norm, window=0.3)
    gb = {k: v.to(dev) for k, v in batch.items()}
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    out = sae.compute_loss(gb, **kw)
    out["loss"].backward()
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    ran = set(timer.summary())
    assert {"encoder_gemm", "jumprelu_fwd", "jumprelu_bwd"} <= ran, ran      # the kernel path, not the generic one
    want = ref.compute_loss(batch, **kw)
    want["loss"].backward()
    assert torch.equal((out["feature_acts"] != 0).cpu(), want["feature_acts"] != 0)
    for key in ("feature_acts", "hidden_pre", "reconstructed", "loss", "l_rec"):
        assert rel_err(out[key], want[key]) < FP32_TOL, key
    for key in ("l_s", "l_p"):
        assert (out[key] is None) == (want[key] is None)
        if want[key] is not None:
            assert rel_err(out[key], want[key]) < FP32_TOL, key
    got, exp = named_grads(sae), named_grads(ref)
    for n in exp:
        assert got[n] is not None, n
        assert rel_err(got[n], exp[n]) < GRAD_TOL, (n, rel_err(got[n], exp[n]))
    assert (exp["log_jumprelu_threshold"] != 0).float().mean() > 0.3


def test_jumprelu_step_bf16_and_adam(pkg, oracle, dev):
    d, F, B = 64, 1024, 128
    sae, ref, batch = make_pair(pkg, oracle, dev, d, F, B, seed=12, include_norm=True, window=0.3)
    gb = {k: v.to(dev) for k, v in batch.items()}
    groups = sae.get_parameters()
    opt = pkg.HipAdam([{"params": groups[0]["params"]}, {"params": groups[1]["params"], "lr": 2e-3}], lr=1e-3, model=sae)
    kw = dict(sparsity_loss_type="tanh", l1_coefficient=0.05)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = sae.compute_loss(gb, **kw)
    assert out["feature_acts"].dtype == torch.bfloat16
    want = ref.compute_loss(batch, **kw)
    assert rel_err(out["loss"], want["loss"]) < BF16_TOL
    assert rel_err(out["l_s"], want["l_s"]) < BF16_TOL
    agree = ((out["feature_acts"] != 0).cpu() == (want["feature_acts"] != 0)).float().mean().item()
    assert agree > 0.995
    out["loss"].backward()
    before = {n: p.detach().clone() for n, p in sae.named_parameters()}
    opt.step()
    for n, p in sae.named_parameters():
        assert torch.isfinite(p).all() and not torch.equal(p, before[n]), n
    # the operands cached for the next step follow the update
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out2 = sae.compute_loss(gb, **kw)
    assert torch.isfinite(out2["loss"]) and out2["loss"].item() != out["loss"].item()


def test_jumprelu_norm_gradient_inside_the_adam_kernel_equals_the_dense_route(pkg, oracle, dev):
    """The gradient that reaches W_D through decoder_norm() is applied as a per-row coefficient inside the Adam
    kernel when the optimiser owns the model; with that switched off it is a dense tensor added to the other
    gradient.  Same bits after several steps, and the gradient norm (which needs the element-wise gradient) agrees."""
    d, F, B = 64, 1024, 128
    kw = dict(sparsity_loss_type="tanh", l1_coefficient=0.05)
    models = []
    for defer in (True, False):
        sae, _, batch = make_pair(pkg, oracle, dev, d, F, B, seed=13, include_norm=True, window=0.3)
        gb = {k: v.to(dev) for k, v in batch.items()}
        groups = sae.get_parameters()
        opt = pkg.HipAdam([{"params": groups[0]["params"]}, {"params": groups[1]["params"], "lr": 2e-3}], lr=1e-3,
                          model=sae, defer_weight_grads=defer)
        norms = []
        for step in range(3):
            with torch.autocast("cuda", dtype=torch.bfloat16):
                out = sae.compute_loss(gb, **kw)
            out["loss"].backward()
            if step == 0:
                assert (getattr(sae.W_D, "_row_grad_coef", None) is not None) == defer
            if step == 2:
                norms.append(pkg.optim.compute_grad_norm([p for g in opt.param_groups for p in g["params"]]))
                assert getattr(sae.W_D, "_row_grad_coef", None) is None      # folded into .grad for the norm
            opt.step()
            opt.zero_grad()
        models.append((sae, norms))
    (a, na), (b, nb) = models
    for (n, p), (_, q) in zip(a.named_parameters(), b.named_parameters()):
        assert torch.equal(p, q), n
    assert torch.equal(na[0], nb[0])


@pytest.mark.parametrize("clip", [0.0, 0.05])
def test_jumprelu_trainer_steps_with_and_without_deferred_terms(pkg, oracle, dev, clip):
    """`Trainer.train_one_step` on a JumpReLU SAE under bf16 autocast (gradient norm every step, clipping on or off):
    the run whose optimiser takes the norm gradient and the bf16 weight gradients inside its kernels ends with the
    bits of the run that gets them as dense fp32 gradients."""
    d, F, B, steps = 64, 1024, 128, 4
    finals = []
    for defer in (True, False):
        sae, _, batch = make_pair(pkg, oracle, dev, d, F, B, seed=14, include_norm=True, window=0.3)
        gb = {k: v.to(dev) for k, v in batch.items()}
        tcfg = pkg.TrainerConfig(lr=1e-3, lr_warm_up_steps=2, lr_cool_down_steps=1, total_training_tokens=B * steps,
                                 amp_dtype=torch.bfloat16, sparsity_loss_type="tanh", l1_coefficient=0.05,
                                 skip_metrics_calculation=True, log_frequency=2, clip_grad_norm=clip, k_warmup_steps=0,
                                 l1_coefficient_warmup_steps=2)
        trainer = pkg.Trainer(tcfg)
        trainer.prepare(sae, gb)
        assert sae.defer_weight_grads          # the trainer's optimiser owns the model
        if not defer:
            sae.defer_weight_grads = False
        norms = []
        for _ in range(steps):
            out = trainer.train_one_step(sae, gb)
            norms.append(float(out["grad_norm_before_clipping"]))
        finals.append(({n: p.detach().clone() for n, p in sae.named_parameters()}, norms))
    (a, na), (b, nb) = finals
    for n in a:
        assert torch.isfinite(a[n]).all()
        assert torch.equal(a[n], b[n]), n
    assert na == nb


# ---- the sparse form of the step: threshold select -> sparse code -> sparse decode / factored gradients ----------

def make_sparse_pair(pkg, oracle, dev, d, F, B, seed, include_norm, window=0.3, theta_lo=1.7, theta_hi=2.3, budget=0.99):
    """Thresholds near 2.0 on pre-activations of unit scale: a few entries per thousand are kept, about as many more
    lie inside the straight-through window."""
    from lm_saes_amd import synthetic

    x = synthetic.activations(B, d, 8, seed)
    w = synthetic.sae_weights(d, F, x, seed)
    g = torch.Generator().manual_seed(seed + 1)
    W_D = (w[2] * (0.5 + torch.rand(F, 1, generator=g))).contiguous()
    w = (w[0], 0.02 * torch.randn(F, generator=g), W_D, w[3])
    log_theta = torch.log(theta_lo + (theta_hi - theta_lo) * torch.rand(F, generator=g))
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="jumprelu",
                        jumprelu_threshold_window=window, norm_activation="inference", sparsity_include_decoder_norm=include_norm,
                        sparsity_threshold_for_triton_spmm_kernel=budget, device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    synthetic.load_weights(sae, *[t.to(dev) for t in w])
    ref = oracle.SAEOracle(d, F, act_fn="jumprelu", jumprelu_threshold_window=window, sparsity_include_decoder_norm=include_norm)
    synthetic.load_weights(ref, *w)
    with torch.no_grad():
        sae.activation_function.log_jumprelu_threshold.copy_(log_theta.to(dev))
        ref.activation_function.log_jumprelu_threshold.copy_(log_theta)
    y = x + 0.1 * torch.randn(B, d, generator=g)
    batch = {"in": x, "out": y, "tokens": torch.zeros(B, dtype=torch.long), "mask": (torch.rand(B, generator=g) > 0.25).float()}
    return sae, ref, batch


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("with_scale", [True, False])
def test_jumprelu_select_lists_kept_and_window_entries(pkg, dev, dtype, with_scale):
    """sae_jumprelu_select_count / _emit against the definition on the CPU: kept = u > theta (value u / s), window =
    |u - theta| < window / 2 and u > 0; every token's entries in ascending feature order; per-token tanh sums and L0."""
    g = torch.Generator().manual_seed(31)
    B, F, window, c = 37, 1024, 0.4, 2.0
    pre = torch.randn(B, F, generator=g).to(dtype)
    b = 0.1 * torch.randn(F, generator=g)
    s = (0.5 + torch.rand(F, generator=g)) if with_scale else None
    theta = 1.5 + torch.rand(F, generator=g)
    got = pkg.ops.jumprelu_select(pre.to(dev), b.to(dev), None if s is None else s.to(dev), theta.to(dev), window, c,
                                  pen_norm=None if s is None else s.to(dev), want_tanh=True)
    code, win, tanh_tok, l0 = got
    h = pre.float() + b
    u = h * s if s is not None else h
    keep = u > theta
    inwin = ((u - theta).abs() < 0.5 * window) & (u > 0)
    listed = keep | inwin
    assert torch.equal(code.row_nnz.cpu().long(), listed.sum(1))
    rows, cols = listed.nonzero(as_tuple=True)
    assert code.n_slots == len(cols) and torch.equal(code.idx.cpu().long(), cols)
    acts = torch.where(keep, (u / s) if s is not None else h, torch.zeros_like(h))
    want_val = acts[rows, cols]
    assert torch.equal(code.val.cpu(), want_val)
    assert torch.equal(win.cpu(), inwin[rows, cols].float())
    assert torch.equal(l0.cpu(), keep.sum(1).float())
    n = s if s is not None else torch.ones(F)
    want_tanh = torch.tanh(c * acts * n).sum(1)
    assert ((tanh_tok.cpu() - want_tanh).abs().max() / want_tanh.abs().max()).item() < 1e-5
    # the budget: more entries than allowed -> None (the caller's dense route); none at all -> None
    assert pkg.ops.jumprelu_select(pre.to(dev), b.to(dev), None, theta.to(dev), window, max_entries=3) is None
    assert pkg.ops.jumprelu_select(pre.to(dev), None, None, (theta + 100).to(dev), window) is None


@pytest.mark.parametrize("with_scale", [True, False])
@pytest.mark.parametrize("B,d,F,theta0", [(70, 64, 1024, 1.5), (300, 128, 4096, 2.5), (33, 64, 64, 0.2)])
def test_jumprelu_margin_route_lists_the_same_entries(pkg, dev, with_scale, B, d, F, theta0):
    """sae_encoder_gemm_jumprelu_margin: the same pre-activations as the plain product, and per granule the largest
    (pre + b) s - theta with product and difference rounded separately; the select that reads only the granules those
    margins allow returns the code of the select that reads every row, bit for bit."""
    g = torch.Generator().manual_seed(B + F)
    x = torch.randn(B, d, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(F, d, generator=g) / d ** 0.5).to(torch.bfloat16).to(dev)
    b = (0.1 * torch.randn(F, generator=g)).to(dev)
    s = (0.5 + torch.rand(F, generator=g)).to(dev) if with_scale else None
    theta = (theta0 + 0.5 * torch.rand(F, generator=g)).to(dev)
    window, c = 0.3, 2.0
    pre, margin = pkg.ops.encoder_gemm_jumprelu_margin(x, w, b, s, theta)
    assert torch.equal(pre, pkg.ops.encoder_gemm(x, w, torch.bfloat16))
    h = pre.float() + b
    u = h * s if s is not None else h
    want_margin = (u - theta).view(B, F // 64, 64).max(dim=2).values
    assert torch.equal(margin, want_margin)
    got = pkg.ops.jumprelu_select(pre, b, s, theta, window, c, pen_norm=s, want_tanh=True, granule_margin=margin)
    ref = pkg.ops.jumprelu_select(pre, b, s, theta, window, c, pen_norm=s, want_tanh=True)
    assert (got is None) == (ref is None)
    if ref is not None:
        (gc, gw, gt, gl), (rc, rw, rt, rl) = got, ref
        assert torch.equal(gc.row_nnz, rc.row_nnz) and torch.equal(gc.row_off, rc.row_off)
        assert torch.equal(gc.idx, rc.idx) and torch.equal(gc.val, rc.val) and torch.equal(gw, rw) and torch.equal(gl, rl)
        assert ((gt - rt).abs().max() / rt.abs().max().clamp_min(1e-30)).item() < 1e-5     # another summation order


@pytest.mark.parametrize("include_norm", [True, False])
@pytest.mark.parametrize("kw", [dict(), dict(sparsity_loss_type="tanh", l1_coefficient=0.05, tanh_stretch_coefficient=2.0)])
def test_sparse_jumprelu_step_fp32_matches_oracle(pkg, oracle, dev, include_norm, kw):
    d, F, B = 64, 4096, 96
    sae, ref, batch = make_sparse_pair(pkg, oracle, dev, d, F, B, seed=21, include_norm=include_norm)
    gb = {k: v.to(dev) for k, v in batch.items()}
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    out = sae.compute_loss(gb, **kw)
    out["loss"].backward()
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    ran = set(timer.records)
    assert "jumprelu_select" in ran and "sparse_decode_mse_fused" in ran and "jumprelu_fwd" not in ran, ran
    want = ref.compute_loss(batch, **kw)
    want["loss"].backward()
    density = (want["feature_acts"] != 0).float().mean().item()
    assert 0 < density < 0.01, density
    assert torch.equal((out["feature_acts"] != 0).cpu(), want["feature_acts"] != 0)
    for key in ("feature_acts", "hidden_pre", "reconstructed", "loss", "l_rec"):
        assert rel_err(out[key], want[key]) < FP32_TOL, key
    if want["l_s"] is not None:
        assert rel_err(out["l_s"], want["l_s"]) < FP32_TOL
    got, exp = named_grads(sae), named_grads(ref)
    for n in exp:
        assert got[n] is not None, n
        assert rel_err(got[n], exp[n]) < GRAD_TOL, (n, rel_err(got[n], exp[n]))
    assert (exp["log_jumprelu_threshold"] != 0).sum() > 20       # window entries exist and carry threshold gradient


def test_sparse_jumprelu_adam_steps_follow_the_oracle_and_fall_back_when_dense(pkg, oracle, dev):
    """Three optimizer steps on the sparse route with the tanh penalty: the factored weight gradients and the decoder-norm
    term go into the Adam kernel (`row_grad_coef`), and the parameters follow torch.optim.Adam on the oracle (fp32: under
    bf16 the first Adam steps, which move every touched weight by +-lr whatever the gradient's size, turn rounding noise on
    near-zero gradient elements into full steps on either side).  One more step under bf16 autocast agrees in its loss.
    Then the thresholds are lowered: the same model takes the dense route again."""
    d, F, B = 64, 4096, 128
    sae, ref, batch = make_sparse_pair(pkg, oracle, dev, d, F, B, seed=23, include_norm=True)
    gb = {k: v.to(dev) for k, v in batch.items()}
    kw = dict(sparsity_loss_type="tanh", l1_coefficient=0.05)
    groups = sae.get_parameters()
    opt = pkg.HipAdam([{"params": groups[0]["params"]}, {"params": groups[1]["params"], "lr": 2e-3}], lr=1e-3, model=sae)
    ropt = oracle.make_adam(ref, lr=1e-3, jumprelu_lr_factor=2.0)
    rp = {k.replace("activation_function.", ""): v for k, v in ref.named_parameters()}
    for step in range(3):
        out = sae.compute_loss(gb, **kw)
        assert "sparse_code" in out, "the sparse route did not run"
        out["loss"].backward()
        assert sae.W_D._sparse_grad is not None and sae.W_D._row_grad_coef is not None and sae.W_D.grad is None
        opt.step(); opt.zero_grad()
        rctx = oracle.train_step(ref, ropt, batch, **kw)
        assert rel_err(out["loss"], rctx["loss"]) < 1e-4, step
        for n, p in sae.named_parameters():
            q = rp[n.replace("activation_function.", "")].detach()
            assert (p.detach().cpu() - q).abs().max() <= 2e-2 * 2e-3 * (step + 1) + 1e-6 * q.abs().max(), (step, n)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = sae.compute_loss(gb, **kw)
    assert "sparse_code" in out
    with torch.autocast("cpu", dtype=torch.bfloat16):
        want = ref.compute_loss(batch, **kw)
    assert rel_err(out["loss"], want["loss"]) < BF16_TOL
    out["loss"].backward()
    opt.step(); opt.zero_grad()
    assert all(torch.isfinite(p).all() for p in sae.parameters())
    with torch.no_grad():
        sae.activation_function.log_jumprelu_threshold.fill_(-3.0)
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        dense = sae.compute_loss(gb, **kw)
    pkg.ops.set_kernel_timer(None)
    assert "jumprelu_fwd" in timer.records and "sparse_code" not in dense
    assert len(timer.records["encoder_gemm"]) == 2      # the probe's encoder product is reused, not recomputed
