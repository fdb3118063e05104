"""End-to-end parity of the fused SAE train step (module API -> HIP kernels) against the oracle.

The encoder GEMM is checked against exact arithmetic in test_gpu_kernels.py.  Its fp32 (or bf16)
rounding differs from the CPU's in the last bits, which can flip a TopK choice between two
near-equal pre-activations; to compare everything downstream on identical selections, the oracle
here takes the GEMM's forward values from the HIP path (its backward stays the matmul's).  A
second test runs the oracle untouched and checks agreement statistically.
"""

import contextlib

import pytest
import torch

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5
BF16_TOL = 2e-2


def rel_err(got, want):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


class _SubstitutedMatmul(torch.autograd.Function):
    """y = x @ W with the forward value supplied; backward is the matmul's own."""

    @staticmethod
    def forward(ctx, x, W, y_given):
        ctx.save_for_backward(x, W)
        return y_given.clone()

    @staticmethod
    def backward(ctx, g):
        x, W = ctx.saved_tensors
        return (g.to(W.dtype) @ W.t()).to(x.dtype), (x.t().to(g.dtype) @ g).to(W.dtype), None


def make_pair(pkg, oracle, dev, d, F, k, B, r, seed, include_norm, mask_frac=0.0, dtype=torch.float32):
    from lm_saes_amd import synthetic

    x = synthetic.activations(B, d, r, seed)
    w = synthetic.sae_weights(d, F, x, seed)
    g = torch.Generator().manual_seed(seed + 1)
    # make the decoder norms and the encoder bias non-trivial so that the fused scale/bias matter
    W_D = w[2] * (0.5 + torch.rand(F, 1, generator=g))
    b_E = 0.02 * torch.randn(F, generator=g)
    w = (w[0], b_E, W_D.contiguous(), w[3])
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                        top_k=k, norm_activation="inference", sparsity_include_decoder_norm=include_norm,
                        device="cuda", dtype=dtype)
    sae = pkg.SparseAutoEncoder(cfg)
    synthetic.load_weights(sae, *[t.to(dev) for t in w])
    ref = oracle.SAEOracle(d, F, act_fn="topk", top_k=k, sparsity_include_decoder_norm=include_norm, dtype=dtype)
    synthetic.load_weights(ref, *w)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long)}
    if mask_frac > 0:
        batch["mask"] = (torch.rand(B, generator=g) > mask_frac).float()
    return sae, ref, batch


def run_both(pkg, oracle, dev, sae, ref, batch, amp, substitute):
    gbatch = {k: v.to(dev) for k, v in batch.items()}
    if amp:
        with torch.autocast("cuda", dtype=torch.bfloat16):
            ctx = sae.compute_loss(gbatch)
    else:
        ctx = sae.compute_loss(gbatch)
    ctx["loss"].backward()

    if substitute:
        # hand the HIP GEMM's forward values to the oracle's encoder matmul
        def encode_sub(x, return_hidden_pre=False, **kw):
            x = x.to(ref.W_E.dtype)
            y_given = sae_pre.to(torch.bfloat16 if amp else torch.float32)
            mm = _SubstitutedMatmul.apply(x.to(y_given.dtype) if amp else x, ref.W_E.to(y_given.dtype) if amp else ref.W_E, y_given)
            hidden_pre = mm + ref.b_E
            if ref.sparsity_include_decoder_norm:
                hidden_pre = hidden_pre * ref.decoder_norm()
            fa = ref.activation_function(hidden_pre)
            if ref.sparsity_include_decoder_norm:
                fa = fa / ref.decoder_norm()
                hidden_pre = hidden_pre / ref.decoder_norm()
            return (fa, hidden_pre) if return_hidden_pre else fa

        # raw GEMM output of the HIP path, recomputed through the C ABI on the same operands
        xg = gbatch["in"]
        if amp:
            sae_pre = pkg.ops.encoder_gemm(pkg.ops.cast_bf16(xg), sae._w_enc_operand(True), torch.bfloat16).cpu()
        else:
            sae_pre = pkg.ops.encoder_gemm(xg.contiguous(), sae._w_enc_operand(False), torch.float32).cpu()
        ref.encode = encode_sub
    if amp:
        with torch.autocast("cpu", dtype=torch.bfloat16):
            rctx = ref.compute_loss(batch)
    else:
        rctx = ref.compute_loss(batch)
    rctx["loss"].backward()
    return ctx, rctx


@pytest.mark.parametrize("include_norm", [False, True])
@pytest.mark.parametrize("masked", [False, True])
def test_fused_step_fp32_matches_oracle(pkg, oracle, dev, include_norm, masked):
    print(f"fused fp32 step include_norm={include_norm} masked={masked}", flush=True)
    sae, ref, batch = make_pair(pkg, oracle, dev, d=256, F=2048, k=16, B=192, r=8, seed=0,
                                include_norm=include_norm, mask_frac=0.25 if masked else 0.0)
    ctx, rctx = run_both(pkg, oracle, dev, sae, ref, batch, amp=False, substitute=True)
    assert torch.equal((ctx["feature_acts"] != 0).cpu(), rctx["feature_acts"] != 0), "selected index sets differ"
    assert rel_err(ctx["feature_acts"], rctx["feature_acts"]) < FP32_TOL
    assert rel_err(ctx["hidden_pre"], rctx["hidden_pre"]) < FP32_TOL
    assert rel_err(ctx["reconstructed"], rctx["reconstructed"]) < FP32_TOL
    assert abs(ctx["loss"].item() - rctx["loss"].item()) / rctx["loss"].item() < FP32_TOL
    assert ctx["n_tokens"] == rctx["n_tokens"]
    for name in ("W_E", "b_E", "W_D", "b_D"):
        got, want = getattr(sae, name).grad, getattr(ref, name).grad
        assert got.shape == want.shape
        assert rel_err(got, want) < FP32_TOL, name


@pytest.mark.parametrize("include_norm", [False, True])
def test_fused_step_bf16_matches_oracle(pkg, oracle, dev, include_norm):
    print(f"fused bf16 step include_norm={include_norm}", flush=True)
    sae, ref, batch = make_pair(pkg, oracle, dev, d=256, F=2048, k=16, B=192, r=8, seed=1, include_norm=include_norm)
    ctx, rctx = run_both(pkg, oracle, dev, sae, ref, batch, amp=True, substitute=True)
    assert torch.equal((ctx["feature_acts"] != 0).cpu(), rctx["feature_acts"] != 0), "selected index sets differ"
    assert rel_err(ctx["feature_acts"], rctx["feature_acts"]) < BF16_TOL
    assert rel_err(ctx["reconstructed"], rctx["reconstructed"]) < BF16_TOL
    assert abs(ctx["loss"].item() - rctx["loss"].item()) / rctx["loss"].item() < BF16_TOL
    for name in ("W_E", "b_E", "W_D", "b_D"):
        got, want = getattr(sae, name).grad, getattr(ref, name).grad
        assert got.dtype == torch.float32 and rel_err(got, want) < BF16_TOL, name


@pytest.mark.parametrize("include_norm", [False, True])
def test_fused_step_with_bf16_parameters_matches_oracle(pkg, oracle, dev, include_norm):
    """cfg.dtype = bfloat16: parameters, gradients and the tensors around the select are bf16 in the reference.
    The select must keep the same set (its arithmetic rounds where the reference's tensors do); the
    reconstruction is compared to bf16 tolerance (the kernel keeps it in fp32, the reference rounds it)."""
    print(f"fused step, bf16 parameters, include_norm={include_norm}", flush=True)
    sae, ref, batch = make_pair(pkg, oracle, dev, d=256, F=2048, k=16, B=192, r=8, seed=7, include_norm=include_norm,
                                dtype=torch.bfloat16)
    assert sae.W_E.dtype == torch.bfloat16 and ref.W_E.dtype == torch.bfloat16
    ctx, rctx = run_both(pkg, oracle, dev, sae, ref, batch, amp=True, substitute=True)
    assert "sparse_code" in ctx, "the fused route was not taken"
    assert torch.equal((ctx["feature_acts"] != 0).cpu(), rctx["feature_acts"] != 0), "selected index sets differ"
    assert torch.equal(ctx["feature_acts"].cpu(), rctx["feature_acts"].float()), "kept values differ"
    assert rel_err(ctx["reconstructed"], rctx["reconstructed"]) < BF16_TOL
    assert abs(ctx["loss"].item() - rctx["loss"].item()) / rctx["loss"].item() < BF16_TOL
    for name in ("W_E", "b_E", "W_D", "b_D"):
        got, want = getattr(sae, name).grad, getattr(ref, name).grad
        assert got.dtype == torch.bfloat16 and got.shape == want.shape
        assert rel_err(got, want) < BF16_TOL, name


def test_bf16_parameters_step_with_adam_follows_torch_adam(pkg, oracle, dev):
    """three steps of fused loss + HipAdam on a bf16 dictionary against the oracle + torch.optim.Adam on CPU bf16
    tensors; factored gradients (no dense dW) and dense ones end at the same bits"""
    finals = []
    for defer in (True, False):
        sae, ref, batch = make_pair(pkg, oracle, dev, d=256, F=2048, k=16, B=192, r=8, seed=8, include_norm=True,
                                    dtype=torch.bfloat16)
        opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, betas=(0.9, 0.999), model=sae, defer_weight_grads=defer)
        gbatch = {k: v.to(dev) for k, v in batch.items()}
        for _ in range(3):
            loss = sae.compute_loss(gbatch, return_aux_data=False)
            loss.backward()
            if defer:
                assert sae.W_D.grad is None and sae.W_D._sparse_grad is not None
            opt.step()
            opt.zero_grad()
        for n, p in sae.named_parameters():
            assert p.dtype == torch.bfloat16 and opt.state[p]["exp_avg"].dtype == torch.bfloat16, n
        finals.append(({n: p.detach().clone() for n, p in sae.named_parameters()}, loss.item()))
    (pa, la), (pb, lb) = finals
    assert la == lb
    for n in pa:
        assert torch.equal(pa[n], pb[n]), n
    # the oracle: same three steps with torch's Adam; selections may differ in a few near-ties (its matmul rounds
    # differently), so the comparison is in tolerance
    ropt = oracle.make_adam(ref, lr=4e-4)
    before = {n: p.detach().clone() for n, p in ref.named_parameters()}
    for _ in range(3):
        rloss = ref.compute_loss(batch)["loss"]
        rloss.backward()
        ropt.step(); ropt.zero_grad()
    assert abs(la - rloss.item()) / rloss.item() < BF16_TOL
    for name in ("W_E", "b_E", "W_D", "b_D"):
        got, want = pa[name].cpu().float(), getattr(ref, name).detach().float()
        assert (want != before[name].float()).any(), name
        # an entry whose gradient differs (a selection flipped at a near-tie) moves the other way: bounded by a few
        # times steps * lr, and rare
        moved = (want - before[name].float()).abs().max().item()
        assert (got - want).abs().max().item() <= 4 * moved, name
        assert ((got - want).abs() > 0.5 * moved).float().mean().item() < 2e-2, name


@pytest.mark.parametrize("clip", [0.0, 0.02])
def test_bf16_parameters_through_the_trainer_shell(pkg, oracle, dev, clip):
    """`Trainer.train_one_step` on a bf16 dictionary: gradient norm every step (and clipping), metrics on; the loss
    goes down and everything stays bf16 and finite.  Factored and dense weight gradients agree on the norm to bf16
    tolerance (the factored one is summed over unrounded rows) and, without clipping, end at the same parameters."""
    d, F, k, B, steps = 256, 2048, 16, 192, 5
    runs = []
    for defer in (True, False):
        sae, _, batch = make_pair(pkg, oracle, dev, d=d, F=F, k=k, B=B, r=8, seed=9, include_norm=True, dtype=torch.bfloat16)
        gb = {kk: v.to(dev) for kk, v in batch.items()}
        gb["mask"] = torch.ones(B, device=dev)
        tcfg = pkg.TrainerConfig(lr=2e-3, lr_warm_up_steps=1, lr_cool_down_steps=1, total_training_tokens=B * steps,
                                 amp_dtype=torch.bfloat16, skip_metrics_calculation=False, log_frequency=1,
                                 clip_grad_norm=clip, k_warmup_steps=0, l1_coefficient_warmup_steps=2)
        trainer = pkg.Trainer(tcfg)
        trainer.prepare(sae, gb)
        if not defer:
            sae.defer_weight_grads = False
        losses, norms = [], []
        for _ in range(steps):
            out = trainer.train_one_step(sae, gb)
            losses.append(float(out["loss"].detach()))
            norms.append(float(out["grad_norm_before_clipping"]))
        for n, p in sae.named_parameters():
            assert p.dtype == torch.bfloat16 and torch.isfinite(p).all(), n
        assert losses[-1] < losses[0]
        runs.append(({n: p.detach().clone() for n, p in sae.named_parameters()}, losses, norms))
    (pa, la, na), (pb, lb, nb) = runs
    assert abs(na[0] - nb[0]) / nb[0] < BF16_TOL
    if clip == 0.0:
        assert la == lb
        for n in pa:
            assert torch.equal(pa[n], pb[n]), n


def test_fused_step_unsubstituted_agrees_statistically(pkg, oracle, dev):
    """No substitution: the two GEMMs round differently, so a few near-tie selections may flip."""
    sae, ref, batch = make_pair(pkg, oracle, dev, d=256, F=2048, k=16, B=192, r=8, seed=2, include_norm=True)
    ctx, rctx = run_both(pkg, oracle, dev, sae, ref, batch, amp=False, substitute=False)
    same = ((ctx["feature_acts"] != 0).cpu() == (rctx["feature_acts"] != 0)).all(dim=-1).float().mean().item()
    assert same > 0.98
    assert abs(ctx["loss"].item() - rctx["loss"].item()) / rctx["loss"].item() < 1e-4


def test_fused_step_then_adam_matches_oracle_adam(pkg, oracle, dev):
    """One full step: fused loss + backward + HipAdam against the oracle's loss + torch.optim.Adam."""
    sae, ref, batch = make_pair(pkg, oracle, dev, d=256, F=2048, k=16, B=192, r=8, seed=3, include_norm=True)
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, betas=(0.9, 0.999), model=sae)
    ropt = oracle.make_adam(ref, lr=4e-4)
    before = {n: p.detach().clone() for n, p in ref.named_parameters()}
    ctx, rctx = run_both(pkg, oracle, dev, sae, ref, batch, amp=False, substitute=True)
    opt.step(); opt.zero_grad()
    ropt.step(); ropt.zero_grad()
    for name in ("W_E", "b_E", "W_D", "b_D"):
        got, want = getattr(sae, name).detach().cpu(), getattr(ref, name).detach()
        moved_ref = (want - before[name]).abs().max().item()
        assert moved_ref > 0
        # Adam's first step is +-lr wherever the gradient is non-zero; entries whose tiny gradient
        # differs in the last bits may move differently, so bound the count, and demand exactness elsewhere
        diff = (got - want).abs()
        assert (diff > 1e-3 * moved_ref).float().mean().item() < 1e-3, name
    # features no token selected keep their exact weights (zero gradient => zero Adam move)
    want, got = ref.W_D.detach(), sae.W_D.detach().cpu()
    unchanged = (want == before["W_D"]).all(dim=1)
    assert unchanged.any() and torch.equal(got[unchanged], before["W_D"][unchanged])


@pytest.mark.parametrize("amp", [False, True])
def test_factored_gradients_match_dense_gradients(pkg, oracle, dev, amp):
    """HipAdam consuming the factored weight gradients (no dense dW in memory) ends at the same
    parameters, moments and derived operands as HipAdam fed dense gradients from autograd."""
    results = []
    for defer in (True, False):
        sae, _, batch = make_pair(pkg, oracle, dev, d=256, F=2048, k=16, B=192, r=8, seed=5, include_norm=True)
        opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, model=sae, defer_weight_grads=defer)
        assert sae.defer_weight_grads == defer
        gbatch = {k: v.to(dev) for k, v in batch.items()}
        for _ in range(3):
            if amp:
                with torch.autocast("cuda", dtype=torch.bfloat16):
                    loss = sae.compute_loss(gbatch, return_aux_data=False)
            else:
                loss = sae.compute_loss(gbatch, return_aux_data=False)
            loss.backward()
            if defer:
                assert sae.W_D.grad is None and sae.W_E.grad is None and sae.W_D._sparse_grad is not None
            else:
                assert sae.W_D.grad is not None and sae.W_E.grad.shape == sae.W_E.shape
            opt.step()
            opt.zero_grad()
            assert sae.W_D.grad is None and getattr(sae.W_D, "_sparse_grad", None) is None
        results.append(({n: p.detach().clone() for n, p in sae.named_parameters()}, loss.item(),
                        {n: opt.state[p]["exp_avg_sq"].clone() for n, p in sae.named_parameters()}))
    (pa, la, va), (pb, lb, vb) = results
    assert la == lb
    for n in pa:
        assert torch.equal(pa[n], pb[n]), n
        assert torch.equal(va[n], vb[n]), n


def test_materialize_grads_and_second_backward(pkg, oracle, dev):
    sae, ref, batch = make_pair(pkg, oracle, dev, d=256, F=2048, k=16, B=192, r=8, seed=6, include_norm=False)
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, model=sae)
    gbatch = {k: v.to(dev) for k, v in batch.items()}
    sae.compute_loss(gbatch)["loss"].backward()
    opt.materialize_grads()
    g1 = {n: p.grad.clone() for n, p in sae.named_parameters()}
    assert g1["W_E"].shape == sae.W_E.shape and g1["W_E"].stride() == sae.W_E.stride()
    opt.zero_grad()
    # two backward passes before a step accumulate, as autograd would
    sae.compute_loss(gbatch)["loss"].backward()
    sae.compute_loss(gbatch)["loss"].backward()
    opt.materialize_grads()
    for n, p in sae.named_parameters():
        assert torch.allclose(p.grad, 2 * g1[n], rtol=1e-6, atol=1e-12), n


def test_overlapped_decoder_update_gives_identical_training(pkg, oracle, dev):
    """Running the decoder's Adam pass on a second stream (overlapping the next step's GEMM) must not
    change a single bit of a multi-step run."""
    results = []
    for overlap in (False, True):
        sae, _, batch = make_pair(pkg, oracle, dev, d=256, F=2048, k=16, B=192, r=8, seed=7, include_norm=True)
        opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, model=sae, overlap_decoder_update=overlap)
        gbatch = {k: v.to(dev) for k, v in batch.items()}
        losses = []
        for _ in range(6):
            with torch.autocast("cuda", dtype=torch.bfloat16):
                loss = sae.compute_loss(gbatch, return_aux_data=False)
            loss.backward()
            opt.step()
            opt.zero_grad()
            losses.append(loss)
        opt.join()
        torch.cuda.synchronize()
        results.append(([l.item() for l in losses], {n: p.detach().clone() for n, p in sae.named_parameters()},
                        sae.decoder_norm().detach().clone()))
    (la, pa, na), (lb, pb, nb) = results
    assert la == lb and la[-1] < la[0]
    for n in pa:
        assert torch.equal(pa[n], pb[n]), n
    assert torch.equal(na, nb)


# ---------------------------------------------------------------------------------------------
# BatchTopK and aux-k through the fused step
# ---------------------------------------------------------------------------------------------

def make_pair_act(pkg, oracle, dev, act_fn, **kw):
    sae, ref, batch = make_pair(pkg, oracle, dev, **kw)
    sae.cfg.act_fn = act_fn
    sae.activation_function = sae.activation_function_factory(None)
    ref.act_fn = act_fn
    ref.activation_function = ref._make_activation()
    return sae, ref, batch


@pytest.mark.parametrize("amp", [False, True])
def test_fused_batchtopk_step_matches_oracle(pkg, oracle, dev, amp):
    print(f"fused batchtopk amp={amp}", flush=True)
    sae, ref, batch = make_pair_act(pkg, oracle, dev, "batchtopk", d=256, F=2048, k=16, B=192, r=8, seed=11,
                                    include_norm=True)
    ctx, rctx = run_both(pkg, oracle, dev, sae, ref, batch, amp=amp, substitute=True)
    tol = BF16_TOL if amp else FP32_TOL
    assert torch.equal((ctx["feature_acts"] != 0).cpu(), rctx["feature_acts"] != 0), "selected index sets differ"
    assert (rctx["feature_acts"] != 0).sum().item() == 16 * 192
    assert (rctx["feature_acts"] != 0).sum(-1).float().std().item() > 0  # rows really differ in length
    assert rel_err(ctx["reconstructed"], rctx["reconstructed"]) < tol
    assert abs(ctx["loss"].item() - rctx["loss"].item()) / rctx["loss"].item() < tol
    for name in ("W_E", "b_E", "W_D", "b_D"):
        assert rel_err(getattr(sae, name).grad, getattr(ref, name).grad) < tol, name


@pytest.mark.parametrize("include_norm", [False, True])
def test_fused_batchtopk_step_with_bf16_parameters_matches_oracle(pkg, oracle, dev, include_norm):
    """BatchTopK with cfg.dtype = bfloat16: the tensors around the batch-wide select are bf16 in the reference, so the
    kept set and the kept values must be identical; reconstruction, loss and gradients to bf16 tolerance."""
    print(f"fused batchtopk step, bf16 parameters, include_norm={include_norm}", flush=True)
    sae, ref, batch = make_pair_act(pkg, oracle, dev, "batchtopk", d=256, F=2048, k=16, B=192, r=8, seed=12,
                                    include_norm=include_norm, dtype=torch.bfloat16)
    assert sae.W_E.dtype == torch.bfloat16 and ref.W_E.dtype == torch.bfloat16
    ctx, rctx = run_both(pkg, oracle, dev, sae, ref, batch, amp=True, substitute=True)
    assert "sparse_code" in ctx, "the fused route was not taken"
    assert (rctx["feature_acts"] != 0).sum().item() == 16 * 192
    assert (rctx["feature_acts"] != 0).sum(-1).float().std().item() > 0  # rows really differ in length
    assert torch.equal((ctx["feature_acts"] != 0).cpu(), rctx["feature_acts"] != 0), "selected index sets differ"
    assert torch.equal(ctx["feature_acts"].cpu(), rctx["feature_acts"].float()), "kept values differ"
    assert rel_err(ctx["reconstructed"], rctx["reconstructed"]) < BF16_TOL
    assert abs(ctx["loss"].item() - rctx["loss"].item()) / rctx["loss"].item() < BF16_TOL
    for name in ("W_E", "b_E", "W_D", "b_D"):
        got, want = getattr(sae, name).grad, getattr(ref, name).grad
        assert got.dtype == torch.bfloat16 and got.shape == want.shape
        assert rel_err(got, want) < BF16_TOL, name


def test_batchtopk_bf16_parameters_adam_steps_factored_equals_dense(pkg, oracle, dev):
    """three steps of the fused BatchTopK loss + HipAdam on a bf16 dictionary: the factored gradients and the dense
    ones end at the same bits, and the loss falls"""
    finals = []
    for defer in (True, False):
        sae, _, batch = make_pair_act(pkg, oracle, dev, "batchtopk", d=256, F=2048, k=16, B=192, r=8, seed=13,
                                      include_norm=True, dtype=torch.bfloat16)
        opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, betas=(0.9, 0.999), model=sae, defer_weight_grads=defer)
        gbatch = {k: v.to(dev) for k, v in batch.items()}
        losses = []
        for _ in range(3):
            loss = sae.compute_loss(gbatch, return_aux_data=False)
            loss.backward()
            if defer:
                assert sae.W_D.grad is None and sae.W_D._sparse_grad is not None
            opt.step()
            opt.zero_grad()
            losses.append(loss.item())
        assert losses[-1] < losses[0]
        finals.append(({n: p.detach().clone() for n, p in sae.named_parameters()}, losses))
    (pa, la), (pb, lb) = finals
    assert la == lb
    for n in pa:
        assert pa[n].dtype == torch.bfloat16 and torch.equal(pa[n], pb[n]), n


@pytest.mark.parametrize("act_fn", ["topk", "batchtopk"])
@pytest.mark.parametrize("include_norm", [False, True])
@pytest.mark.parametrize("route", ["dense", "sparse"])
def test_fused_auxk_step_matches_oracle(pkg, oracle, dev, act_fn, include_norm, route):
    """Both routes of the aux-k term (dead features as a compact dense block / stacked onto the sparse code)."""
    print(f"fused aux-k {act_fn} include_norm={include_norm} route={route}", flush=True)
    B, F, k, k_aux = 192, 2048, 16, 32
    sae, ref, batch = make_pair_act(pkg, oracle, dev, act_fn, d=256, F=F, k=k, B=B, r=8, seed=12, include_norm=include_norm,
                                    mask_frac=0.2)
    sae.aux_dense_block = route == "dense"
    trainer = pkg.Trainer(pkg.TrainerConfig(auxk_coefficient=1 / 32, k_aux=k_aux, dead_threshold=float(B)))
    trainer._initialize_dead_statistics(sae)
    stats = oracle.DeadStatistics(F, dead_threshold=float(B))
    # one earlier batch so that the counters are not all zero
    warm = torch.zeros(B, F); warm[:, ::7] = 1.0
    trainer.update_dead_statistics(warm.to(dev), None, ("batch", "sae"))
    stats.update(warm, None, 1)

    gbatch = {k_: v.to(dev) for k_, v in batch.items()}
    kw = dict(auxk_coefficient=1 / 32, k_aux=k_aux)
    ctx = sae.compute_loss(gbatch, update_dead_statistics=trainer.update_dead_statistics, **kw)
    ctx["loss"].backward()
    # oracle with the HIP GEMM's forward values (see run_both)
    sae_pre = pkg.ops.encoder_gemm(gbatch["in"].contiguous(), sae._w_enc_operand(False), torch.float32).cpu()

    def encode_sub(x, return_hidden_pre=False, **_):
        mm = _SubstitutedMatmul.apply(x, ref.W_E, sae_pre)
        hp = mm + ref.b_E
        if ref.sparsity_include_decoder_norm:
            hp = hp * ref.decoder_norm()
        fa = ref.activation_function(hp)
        if ref.sparsity_include_decoder_norm:
            fa = fa / ref.decoder_norm()
            hp = hp / ref.decoder_norm()
        return (fa, hp) if return_hidden_pre else fa

    ref.encode = encode_sub
    rctx = ref.compute_loss(batch, update_dead_statistics=stats.update, **kw)
    rctx["loss"].backward()

    assert sae._last_aux_route == route
    assert torch.equal(trainer.is_dead.cpu(), stats.is_dead)
    assert torch.equal(trainer.tokens_since_last_activation.cpu(), stats.tokens_since_last_activation)
    assert stats.is_dead.sum().item() > k_aux  # plenty of dead features: the aux select really truncates
    assert rctx["l_aux"].item() > 0
    assert abs(ctx["l_aux"].item() - rctx["l_aux"].item()) / rctx["l_aux"].item() < FP32_TOL
    assert abs(ctx["l_rec"].item() - rctx["l_rec"].item()) / rctx["l_rec"].item() < FP32_TOL
    assert abs(ctx["loss"].item() - rctx["loss"].item()) / rctx["loss"].item() < FP32_TOL
    for name in ("W_E", "b_E", "W_D", "b_D"):
        assert rel_err(getattr(sae, name).grad, getattr(ref, name).grad) < FP32_TOL, name
    assert sae.current_k == k and ref.current_k == k


@pytest.mark.parametrize("act_fn", ["topk", "batchtopk"])
@pytest.mark.parametrize("route", ["dense", "sparse"])
def test_auxk_step_with_bf16_parameters(pkg, oracle, dev, act_fn, route):
    """aux-k on a dictionary held in bf16, on the compact dense block and on the stacked sparse code: the aux selection
    is the reference's bf16 op sequence exactly; losses and gradients agree with the oracle on CPU bf16 tensors to bf16
    tolerance; three Adam steps with factored and with dense gradients end at the same bits."""
    print(f"aux-k step, bf16 parameters, {act_fn}, route={route}", flush=True)
    B, F, k, k_aux = 192, 2048, 16, 32
    kw = dict(auxk_coefficient=1 / 32, k_aux=k_aux)

    def fresh():
        sae, ref, batch = make_pair_act(pkg, oracle, dev, act_fn, d=256, F=F, k=k, B=B, r=8, seed=15, include_norm=True,
                                        dtype=torch.bfloat16)
        sae.aux_dense_block = route == "dense"
        trainer = pkg.Trainer(pkg.TrainerConfig(auxk_coefficient=1 / 32, k_aux=k_aux, dead_threshold=float(B)))
        trainer._initialize_dead_statistics(sae)
        warm = torch.zeros(B, F); warm[:, ::7] = 1.0
        trainer.update_dead_statistics(warm.to(dev), None, ("batch", "sae"))
        stats = oracle.DeadStatistics(F, dead_threshold=float(B))
        stats.update(warm, None, 1)
        return sae, ref, batch, trainer, stats

    sae, ref, batch, trainer, stats = fresh()
    gbatch = {k_: v.to(dev) for k_, v in batch.items()}
    ctx = sae.compute_loss(gbatch, update_dead_statistics=trainer.update_dead_statistics, **kw)
    ctx["loss"].backward()
    assert "sparse_code" in ctx and sae._last_aux_route == route
    # the reference's sequence on bf16 tensors, from the kernel's own product
    pre = pkg.ops.encoder_gemm(pkg.ops.cast_bf16(gbatch["in"].float().contiguous()), sae._w_enc_operand(True), torch.bfloat16).cpu()
    n = sae._decoder_norm_nograd().cpu().bfloat16()
    h1 = (pre + sae.b_E.detach().cpu()) * n
    assert h1.dtype == torch.bfloat16
    dead = trainer.is_dead.cpu()
    dead_pre = (h1 / n) * dead * n
    relu = dead_pre * dead_pre.gt(0).to(dead_pre.dtype)
    kk = min(k_aux, int(dead.sum()))
    assert int(dead.sum()) > k_aux
    want = (oracle.topk(relu, k=kk, dim=-1) if act_fn == "topk" else oracle.topk(relu, k=kk * B, dim=(-2, -1))) / n
    got = ctx["aux_sparse_code"].to_dense().cpu()
    assert torch.equal(got != 0, want != 0), "aux-k kept sets differ"
    assert torch.equal(got, want.float()), "aux-k kept values differ"

    # the oracle on CPU bf16 tensors with the kernel's product handed in (see run_both)
    def encode_sub(x, return_hidden_pre=False, **_):
        mm = _SubstitutedMatmul.apply(x.to(torch.bfloat16), ref.W_E, pre)
        hp = mm + ref.b_E
        hp = hp * ref.decoder_norm()
        fa = ref.activation_function(hp)
        fa = fa / ref.decoder_norm()
        hp = hp / ref.decoder_norm()
        return (fa, hp) if return_hidden_pre else fa

    ref.encode = encode_sub
    rctx = ref.compute_loss(batch, update_dead_statistics=stats.update, **kw)
    rctx["loss"].backward()
    assert torch.equal(trainer.is_dead.cpu(), stats.is_dead)
    assert torch.equal((ctx["feature_acts"] != 0).cpu(), rctx["feature_acts"] != 0), "selected index sets differ"
    assert rctx["l_aux"].item() > 0
    assert abs(ctx["l_aux"].item() - rctx["l_aux"].item()) / rctx["l_aux"].item() < BF16_TOL
    assert abs(ctx["loss"].item() - rctx["loss"].item()) / rctx["loss"].item() < BF16_TOL
    for name in ("W_E", "b_E", "W_D", "b_D"):
        gotg, wantg = getattr(sae, name).grad, getattr(ref, name).grad
        assert gotg.dtype == torch.bfloat16 and gotg.shape == wantg.shape
        assert rel_err(gotg, wantg) < BF16_TOL, name

    finals = []
    for defer in (True, False):
        sae, _, batch, trainer, _ = fresh()
        opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, betas=(0.9, 0.999), model=sae, defer_weight_grads=defer)
        losses = []
        for _ in range(3):
            loss = sae.compute_loss(gbatch, update_dead_statistics=trainer.update_dead_statistics, return_aux_data=False, **kw)
            loss.backward()
            if defer:
                assert sae.W_D.grad is None and sae.W_D._sparse_grad is not None
            opt.step()
            opt.zero_grad()
            losses.append(loss.item())
        finals.append(({nm: p.detach().clone() for nm, p in sae.named_parameters()}, losses))
    (pa, la), (pb, lb) = finals
    assert la == lb and la[-1] < la[0]
    for nm in pa:
        assert pa[nm].dtype == torch.bfloat16 and torch.equal(pa[nm], pb[nm]), nm


@pytest.mark.parametrize("act_fn", ["topk", "batchtopk"])
@pytest.mark.parametrize("amp", [False, True])
def test_auxk_selection_is_the_reference_op_sequence_on_both_routes(pkg, oracle, dev, act_fn, amp):
    """The aux-k term's own selection among the dead features: `hidden_pre * is_dead * decoder_norm` with hidden_pre the
    quotient the encoder returned (models/sparse_dictionary.py:958-970), evaluated op for op on the kernel's GEMM
    output with the oracle's TopK.  The compact dense block and the stacked sparse code must keep exactly that set with
    exactly those values."""
    print(f"aux-k selection {act_fn} amp={amp}", flush=True)
    B, F, k, k_aux = 192, 2048, 16, 32
    codes = {}
    for route in ("dense", "sparse"):
        sae, ref, batch = make_pair_act(pkg, oracle, dev, act_fn, d=256, F=F, k=k, B=B, r=8, seed=14, include_norm=True)
        sae.aux_dense_block = route == "dense"
        trainer = pkg.Trainer(pkg.TrainerConfig(auxk_coefficient=1 / 32, k_aux=k_aux, dead_threshold=float(B)))
        trainer._initialize_dead_statistics(sae)
        warm = torch.zeros(B, F); warm[:, ::7] = 1.0
        trainer.update_dead_statistics(warm.to(dev), None, ("batch", "sae"))
        gbatch = {k_: v.to(dev) for k_, v in batch.items()}
        with (torch.autocast("cuda", dtype=torch.bfloat16) if amp else contextlib.nullcontext()):
            ctx = sae.compute_loss(gbatch, update_dead_statistics=trainer.update_dead_statistics, auxk_coefficient=1 / 32,
                                   k_aux=k_aux)
        assert sae._last_aux_route == route
        codes[route] = ctx["aux_sparse_code"].to_dense().cpu()
        dead = trainer.is_dead.cpu()
    # the reference's sequence on the same GEMM output
    x_op = gbatch["in"].contiguous()
    pre = (pkg.ops.encoder_gemm(pkg.ops.cast_bf16(x_op), sae._w_enc_operand(True), torch.bfloat16) if amp
           else pkg.ops.encoder_gemm(x_op, sae._w_enc_operand(False), torch.float32)).cpu().float()
    n = sae._decoder_norm_nograd().cpu()   # the norms the kernels read (the oracle's differ from them in the last bit)
    hidden_pre = ((pre + sae.b_E.detach().cpu()) * n) / n
    dead_pre = hidden_pre * dead * n
    kk = min(k_aux, int(dead.sum()))
    assert int(dead.sum()) > k_aux
    relu = dead_pre * dead_pre.gt(0).to(dead_pre.dtype)
    want = (oracle.topk(relu, k=kk, dim=-1) if act_fn == "topk" else oracle.topk(relu, k=kk * B, dim=(-2, -1))) / n
    for route in ("dense", "sparse"):
        assert torch.equal(codes[route] != 0, want != 0), f"{route}: kept sets differ"
        assert torch.equal(codes[route], want), f"{route}: kept values differ"


def test_fused_auxk_without_dead_features_is_plain_loss(pkg, oracle, dev):
    sae, ref, batch = make_pair_act(pkg, oracle, dev, "topk", d=256, F=2048, k=16, B=192, r=8, seed=13, include_norm=True)
    trainer = pkg.Trainer(pkg.TrainerConfig(auxk_coefficient=0.5, k_aux=8, dead_threshold=1e9))
    trainer._initialize_dead_statistics(sae)
    gbatch = {k_: v.to(dev) for k_, v in batch.items()}
    ctx = sae.compute_loss(gbatch, auxk_coefficient=0.5, k_aux=8, update_dead_statistics=trainer.update_dead_statistics)
    plain = sae.compute_loss(gbatch)
    assert ctx["l_aux"].item() == 0.0
    assert abs(ctx["loss"].item() - plain["loss"].item()) <= 1e-6 * plain["loss"].item()
