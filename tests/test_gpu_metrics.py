"""Metrics kernels (sparse-code statistics, reconstruction statistics), the factored gradient norm and the
trainer's logging path against the CPU oracles."""

import importlib
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mo():
    import __graft_entry__  # noqa: F401
    return importlib.import_module("oracle.metrics_oracle")


def random_code(pkg, dev, B, F, kmax, seed, ragged=True):
    """A sparse code with ascending distinct indices per token, ragged row lengths, some zero / negative values."""
    g = torch.Generator().manual_seed(seed)
    nnz = torch.randint(0, kmax + 1, (B,), generator=g) if ragged else torch.full((B,), kmax)
    idx = torch.zeros(B, kmax, dtype=torch.int32)
    val = torch.zeros(B, kmax)
    dense = torch.zeros(B, F)
    for b in range(B):
        n = int(nnz[b])
        ids = torch.randperm(F, generator=g)[:n].sort().values
        v = torch.randn(n, generator=g)
        v[torch.rand(n, generator=g) < 0.1] = 0.0
        idx[b, :n] = ids.int(); val[b, :n] = v
        dense[b, ids] = v
    code = pkg.SparseCode(idx.reshape(-1).to(dev), val.reshape(-1).to(dev), (torch.arange(B) * kmax).to(dev),
                          nnz.int().to(dev), B, F)
    return code, dense


@pytest.mark.parametrize("B,F,kmax,masked", [(50, 300, 17, False), (129, 1000, 64, True), (7, 70, 70, True), (64, 4096, 130, False)])
def test_code_stats_kernel_matches_dense_oracle(pkg, mo, dev, B, F, kmax, masked):
    code, dense = random_code(pkg, dev, B, F, kmax, seed=B)
    mask = (torch.rand(B, generator=torch.Generator().manual_seed(1)) > 0.3).float() if masked else None
    freq = torch.zeros(F, device=dev)
    totals = torch.zeros(3, dtype=torch.float64, device=dev)
    l0 = pkg.ops.code_stats(code, tok_w=None if mask is None else mask.to(dev), freq_acc=freq, totals=totals, want_l0=True)
    assert torch.equal(freq.cpu(), mo.act_freq_scores(dense, mask))                         # integer counts: exact
    assert torch.equal(l0.cpu(), (dense > 0).float().sum(-1))
    assert totals[1].item() == (dense > 0).sum().item()
    assert totals[2].item() == mo.l0_sum(dense, mask).item()
    assert totals[0].item() == pytest.approx(dense.double().sum().item(), rel=1e-5, abs=1e-4)
    assert (totals[0] / totals[1]).item() == pytest.approx(mo.mean_feature_act(dense).item(), rel=1e-5)
    # the accumulators are added to, not overwritten
    pkg.ops.code_stats(code, tok_w=None if mask is None else mask.to(dev), freq_acc=freq, totals=totals)
    assert torch.equal(freq.cpu(), 2 * mo.act_freq_scores(dense, mask)) and totals[1].item() == 2 * (dense > 0).sum().item()


@pytest.mark.parametrize("B,d,masked", [(40, 64, False), (257, 768, True), (33, 50, True), (5, 7, False)])
def test_recon_stats_kernel_matches_oracle(pkg, mo, dev, B, d, masked):
    g = torch.Generator().manual_seed(d)
    label = torch.randn(B, d, generator=g) + 0.5
    recon = label + 0.3 * torch.randn(B, d, generator=g) * torch.rand(B, 1, generator=g)
    mask = (torch.rand(B, generator=g) > 0.3).float() if masked else None
    ev, legacy = mo.explained_variance(label.double(), recon.double(), None if mask is None else mask.double())
    err, ratio = mo.l2_norm_error(label.double(), recon.double(), None if mask is None else mask.double())
    mean = label.mean(0) if mask is None else (label * mask[:, None]).sum(0) / mask.sum()
    acc = torch.zeros(4, dtype=torch.float64, device=dev)
    for rep in (1, 2):
        step = pkg.ops.recon_stats(label.to(dev), recon.to(dev), mean.to(dev), acc, tok_w=None if mask is None else mask.to(dev))
        for got, want in zip(step.tolist(), (ev, legacy, err, ratio)):
            assert got == pytest.approx(want.item(), rel=1e-5, abs=1e-6)
        for got, want in zip(acc.tolist(), (ev, legacy, err, ratio)):
            assert got == pytest.approx(rep * want.item(), rel=1e-5, abs=1e-6)
    # closed forms through the kernel: perfect reconstruction, reconstruction = mean
    acc.zero_()
    step = pkg.ops.recon_stats(label.to(dev), label.to(dev), mean.to(dev), acc, tok_w=None if mask is None else mask.to(dev))
    assert step.tolist() == [1.0, 1.0, 0.0, 0.0]
    step = pkg.ops.recon_stats(label.to(dev), mean.expand(B, d).contiguous().to(dev), mean.to(dev), acc,
                               tok_w=None if mask is None else mask.to(dev))
    assert abs(step[0].item()) < 1e-6 and abs(step[1].item()) < 1e-6


@pytest.mark.parametrize("B,d,F,k,dense_dtype", [(64, 128, 512, 8, torch.float32), (96, 256, 300, 16, torch.bfloat16),
                                                 (33, 64, 2048, 4, torch.float32)])
def test_factored_grad_norm_equals_the_dense_one(pkg, oracle, dev, B, d, F, k, dense_dtype):
    g = torch.Generator().manual_seed(F)
    code, _ = random_code(pkg, dev, B, F, k, seed=F + 1)
    fi = pkg.ops.build_feature_index(code)
    coef = torch.randn(B * k, generator=g).to(dev)
    dense_op = torch.randn(B, d, generator=g).to(dev).to(dense_dtype)
    rows, bias = pkg.ops.sparse_grad_rows(fi, coef, dense_op, F, want_bias=True)
    acc = torch.zeros(2, dtype=torch.float64, device=dev)
    bias_out = torch.full((F,), float("nan"), device=dev)
    pkg.ops.sparse_rows_grad_sq_nnz(fi, coef, dense_op, acc, bias_grad_out=bias_out)
    assert acc[1].item() == (rows != 0).sum().item()                                         # same rows, bit for bit
    assert acc[0].item() == pytest.approx(rows.double().pow(2).sum().item(), rel=1e-6)
    assert torch.equal(bias_out, bias)
    want = oracle.compute_grad_norm([rows.cpu()]).item()
    assert (acc[0].sqrt() / acc[1].sqrt()).item() == pytest.approx(want, rel=1e-5)
    assert (rows == 0).all(dim=1).any(), "the case must include features no token used"
    pkg.ops.sparse_rows_grad_sq_nnz(fi, coef, dense_op, acc)                                 # accumulates
    assert acc[1].item() == 2 * (rows != 0).sum().item()


@pytest.mark.parametrize("dense_dtype", [torch.float32, torch.bfloat16])
def test_adam_sparse_rows_with_grad_scale_equals_scaled_dense_gradient(pkg, dev, dense_dtype):
    B, d, F, k = 80, 128, 700, 8
    g = torch.Generator().manual_seed(9)
    code, _ = random_code(pkg, dev, B, F, k, seed=10)
    fi = pkg.ops.build_feature_index(code)
    coef = torch.randn(B * k, generator=g).to(dev)
    dense_op = torch.randn(B, d, generator=g).to(dev).to(dense_dtype)
    scale = torch.tensor([0.37], device=dev)
    p0 = torch.randn(F, d, generator=g).to(dev)
    rows, bias = pkg.ops.sparse_grad_rows(fi, coef, dense_op, F, want_bias=True)
    pa, ma, va = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    pb, mb, vb = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    bias_out = torch.empty(F, device=dev)
    for step in (1, 2):
        pkg.ops.adam_step(pa, rows * scale, ma, va, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, step=step)
        pkg.ops.adam_step_sparse_rows(fi, coef, dense_op, pb, mb, vb, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, step=step,
                                      bias_grad_out=bias_out, grad_scale=scale)
    assert torch.equal(pa, pb) and torch.equal(ma, mb) and torch.equal(va, vb)
    assert torch.equal(bias_out, bias * scale)


def _small_sae(pkg, dev, d, F, k, x, seed, act_fn="topk"):
    from lm_saes_amd import synthetic

    w = synthetic.sae_weights(d, F, x, seed=seed)
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn=act_fn,
                        top_k=k, norm_activation="inference", device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    synthetic.load_weights(sae, *[t.to(dev) for t in w])
    return sae, w


def test_clip_grad_norm_on_factored_gradients_matches_the_oracle(pkg, oracle, dev):
    """Norm before clipping, clipped update and norm after clipping, with the weight gradients never densified."""
    from lm_saes_amd import synthetic

    d, F, k, B = 128, 1024, 8, 96
    x = synthetic.activations(B, d, 8, seed=11)
    sae, w = _small_sae(pkg, dev, d, F, k, x, seed=11)
    ref = oracle.SAEOracle(d, F, act_fn="topk", top_k=k)
    synthetic.load_weights(ref, *w)
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=1e-3, model=sae)
    ropt = oracle.make_adam(ref, lr=1e-3)
    for max_norm in (1e-4, math.inf):
        sae.compute_loss({"in": x.to(dev), "out": x.to(dev), "tokens": torch.zeros(B, device=dev)})["loss"].backward()
        ref.compute_loss({"in": x, "out": x, "tokens": torch.zeros(B)})["loss"].backward()
        assert sae.W_E.grad is None and sae.W_D.grad is None and sae.W_E._sparse_grad is not None
        rgrads = [p.grad for p in ref.parameters()]
        want_before = oracle.clip_grad_norm(rgrads, max_norm).item()
        got_before = pkg.clip_grad_norm(list(sae.parameters()), max_norm)
        assert sae.W_E.grad is None and sae.W_D.grad is None, "clipping must not materialise the weight gradients"
        assert got_before.item() == pytest.approx(want_before, rel=1e-5)
        want_after = oracle.compute_grad_norm(rgrads).item()
        assert pkg.compute_grad_norm(sae.parameters()).item() == pytest.approx(want_after, rel=1e-5)
        if max_norm < 1:
            assert want_after < want_before * 0.9, "the case must actually clip"
        opt.step(); opt.zero_grad(); ropt.step(); ropt.zero_grad()
        for (n, p), q in zip(sae.named_parameters(), ref.parameters()):
            # clipped gradients are tiny and Adam normalises them: compare the moves, which are O(lr)
            assert (p.detach().cpu() - q.detach()).abs().max() <= 2e-2 * 1e-3 + 1e-6 * q.detach().abs().max(), n


@pytest.mark.parametrize("masked,auxk", [(False, False), (True, False), (True, True)])
def test_trainer_log_matches_the_oracle_metrics(pkg, oracle, mo, dev, masked, auxk):
    """`Trainer.fit` with metrics on: what is logged every `log_frequency` steps against the dense oracle
    formulas applied to the oracle model's own step contexts."""
    from lm_saes_amd import synthetic

    d, F, k, B, steps = 128, 1024, 8, 64, 6
    x = synthetic.activations(B * steps, d, 8, seed=21)
    sae, w = _small_sae(pkg, dev, d, F, k, x[:B], seed=21)
    tcfg = pkg.TrainerConfig(lr=1e-3, lr_warm_up_steps=2, lr_cool_down_steps=1, total_training_tokens=B * steps,
                             amp_dtype=torch.float32, l1_coefficient=None, skip_metrics_calculation=False, log_frequency=3,
                             clip_grad_norm=0.0, k_warmup_steps=0, auxk_coefficient=1 / 32 if auxk else None, k_aux=16,
                             dead_threshold=B if auxk else 10_000_000)
    trainer = pkg.Trainer(tcfg)
    logged = []
    trainer.log_sink = lambda step, m: logged.append((step, dict(m)))
    gm = torch.Generator().manual_seed(5)
    masks = [(torch.rand(B, generator=gm) > 0.3).float() if masked else None for _ in range(steps)]
    batches = []
    for i in range(steps):
        b = {"in": x[i * B:(i + 1) * B].to(dev), "out": x[i * B:(i + 1) * B].to(dev), "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
        if masked:
            b["mask"] = masks[i].to(dev)
        batches.append(b)
    trainer.fit(sae, batches)
    assert [s for s, _ in logged] == [3, 6]

    ref = oracle.SAEOracle(d, F, act_fn="topk", top_k=k)
    synthetic.load_weights(ref, *w)
    opt = oracle.make_adam(ref, lr=1e-3)
    dead = oracle.DeadStatistics(F, dead_threshold=B) if auxk else None
    sm = mo.StepMetrics()
    want = []
    for s in range(steps):
        for gparam in opt.param_groups:
            gparam["lr"] = 1e-3 * min(1.0, (s + 1) / 2)
        xb = x[s * B:(s + 1) * B]
        batch = {"in": xb, "out": xb, "tokens": torch.zeros(B)}
        if masked:
            batch["mask"] = masks[s]
        kw = dict(auxk_coefficient=1 / 32, k_aux=16, update_dead_statistics=dead.update) if auxk else {}
        rctx = ref.compute_loss(batch, **kw)
        rctx["loss"].backward()
        grads = [p.grad for p in ref.parameters()]
        gn = oracle.clip_grad_norm(grads, math.inf).item()
        sm.update(feature_acts=rctx["feature_acts"].detach(), label=rctx["label"], reconstructed=rctx["reconstructed"].detach(),
                  mask=batch.get("mask"), n_tokens=rctx["n_tokens"], loss=rctx["loss"].detach(), l_rec=rctx["l_rec"].detach(),
                  l_aux=None if rctx.get("l_aux") is None else rctx["l_aux"].detach(), grad_norm_before_clipping=gn, grad_norm=gn)
        opt.step(); opt.zero_grad()
        if (s + 1) % 3 == 0:
            want.append(sm.compute())
    for (_, got), ref_m in zip(logged, want):
        for key, v in ref_m.items():
            if key.startswith("sparsity/"):
                assert got[key] == v, key
            else:
                assert got[key] == pytest.approx(v, rel=2e-3, abs=1e-6), (key, got[key], v)
        assert got["sparsity/k"] == k and "metrics/decoder_norm" in got and got["details/current_learning_rate"] > 0


def test_deferred_grad_norm_comes_out_of_the_optimizer_step(pkg, oracle, dev):
    """The norm produced as a by-product of HipAdam.step() equals the direct one, and the step itself is unchanged."""
    from lm_saes_amd import synthetic

    d, F, k, B = 128, 1024, 8, 96
    x = synthetic.activations(B, d, 8, seed=41)
    batch = {"in": x.to(dev), "out": x.to(dev), "tokens": torch.zeros(B, device=dev)}
    results = []
    for deferred in (False, True):
        sae, w = _small_sae(pkg, dev, d, F, k, x, seed=41)
        opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=1e-3, model=sae)
        norms = []
        for _ in range(3):
            sae.compute_loss(batch, return_aux_data=False).backward()
            params = list(sae.parameters())
            norms.append(opt.deferred_grad_norm(params) if deferred else pkg.compute_grad_norm(params))
            opt.step(); opt.zero_grad()
        results.append(([n.item() for n in norms], [p.detach().clone() for p in sae.parameters()]))
    (direct, p_direct), (by_product, p_by) = results
    for a, b in zip(direct, by_product):
        assert b == pytest.approx(a, rel=1e-6)
    for a, b in zip(p_direct, p_by):
        assert torch.equal(a, b)
    ref = oracle.SAEOracle(d, F, act_fn="topk", top_k=k)
    synthetic.load_weights(ref, *w)
    ref.compute_loss({"in": x, "out": x, "tokens": torch.zeros(B)})["loss"].backward()
    assert by_product[0] == pytest.approx(oracle.compute_grad_norm([p.grad for p in ref.parameters()]).item(), rel=1e-5)


def test_dense_row_block_adds_to_the_factored_gradient(pkg, dev):
    """`extra` (a densely held block of gradient rows) in the Adam row pass and in the factored norm: equal to the
    same rows added to the materialised gradient."""
    B, d, F, k, n = 64, 128, 600, 8, 37
    g = torch.Generator().manual_seed(17)
    code, _ = random_code(pkg, dev, B, F, k, seed=18)
    fi = pkg.ops.build_feature_index(code)
    coef = torch.randn(B * k, generator=g).to(dev)
    dense_op = torch.randn(B, d, generator=g).to(dev)
    ids = torch.randperm(F, generator=g)[:n].sort().values
    row_map = torch.full((F,), -1, dtype=torch.int32); row_map[ids] = torch.arange(n, dtype=torch.int32)
    block = pkg.ops.DenseRowBlock(row_map.to(dev), torch.randn(n, d, generator=g).to(dev), torch.randn(n, generator=g).to(dev))
    rows, bias = pkg.ops.sparse_grad_rows(fi, coef, dense_op, F, want_bias=True)
    rows_x = rows.clone(); rows_x[ids.to(dev)] = block.rows + rows[ids.to(dev)]      # the block is the accumulator's start value
    bias_x = bias.clone(); bias_x[ids.to(dev)] += block.bias
    p0 = torch.randn(F, d, generator=g).to(dev)
    pa, ma, va = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    pb, mb, vb = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    bias_out = torch.empty(F, device=dev)
    acc = torch.zeros(2, dtype=torch.float64, device=dev)
    pkg.ops.adam_step(pa, rows_x, ma, va, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, step=1)
    pkg.ops.adam_step_sparse_rows(fi, coef, dense_op, pb, mb, vb, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, step=1,
                                  bias_grad_out=bias_out, grad_sq_nnz_acc=acc, extra=block)
    assert (pa - pb).abs().max() <= 2e-6 * 1e-3 + 1e-7 and (ma - mb).abs().max() <= 1e-6 * ma.abs().max()
    assert (bias_out - bias_x).abs().max() <= 1e-5 * bias_x.abs().max()
    assert acc[1].item() == (rows_x != 0).sum().item()
    assert acc[0].item() == pytest.approx(rows_x.double().pow(2).sum().item(), rel=1e-5)
    acc2 = torch.zeros(2, dtype=torch.float64, device=dev)
    pkg.ops.sparse_rows_grad_sq_nnz(fi, coef, dense_op, acc2, extra=block)
    assert acc2[1].item() == acc[1].item() and acc2[0].item() == pytest.approx(acc[0].item(), rel=1e-9)
    with pytest.raises(ValueError):
        pkg.ops.adam_step_sparse_rows(fi, coef, dense_op, pb, mb, vb, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, step=2,
                                      extra=pkg.ops.DenseRowBlock(row_map[:10].to(dev), block.rows, None))
