"""SparseAdam / grad-norm kernels and the trainer shell against the oracle."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_sparse_adam_kernel_matches_oracle(pkg, oracle, dev):
    g = torch.Generator().manual_seed(0)
    n = 5000
    p0 = torch.randn(n, generator=g)
    pr = p0.clone()
    st = oracle.SparseAdamState(pr)
    p, m, v = p0.clone().to(dev), torch.zeros(n, device=dev), torch.zeros(n, device=dev)
    step = torch.zeros(1, device=dev)
    for it in range(5):
        grad = torch.randn(n, generator=g) * (torch.rand(n, generator=g) > 0.6)
        if it == 2:
            grad.zero_()  # skipped entirely: no decay, no step
        oracle.sparse_adam_step(pr, grad, st, lr=1e-2, betas=(0.9, 0.999), eps=1e-8)
        pkg.ops.sparse_adam_step(p, grad.to(dev), m, v, step, lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8)
        assert (p.cpu() - pr).abs().max() <= 4 * 1.2e-7 * p0.abs().max()
    assert step.item() == st.step == 4
    # (a sum of opposite-signed terms may cancel: bound the error by the scale of the tensor)
    assert (m.cpu() - st.exp_avg).abs().max() <= 1e-6 * st.exp_avg.abs().max()
    assert (v.cpu() - st.exp_avg_sq).abs().max() <= 1e-6 * st.exp_avg_sq.abs().max()
    # entries whose gradient was zero in the last step did not move in that step
    before = p.clone()
    grad = torch.zeros(n); grad[::3] = 1.0
    pkg.ops.sparse_adam_step(p, grad.to(dev), m, v, step, lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8)
    moved = (p != before).cpu()
    assert moved[::3].all() and not moved[1::3].any() and not moved[2::3].any()


def test_grad_norm_matches_oracle(pkg, oracle, dev):
    g = torch.Generator().manual_seed(1)
    grads = [torch.randn(300, 17, generator=g) * (torch.rand(300, 17, generator=g) > 0.5), torch.randn(77, generator=g),
             torch.zeros(10)]
    want = oracle.compute_grad_norm(grads).item()
    params = []
    for t in grads:
        p = torch.nn.Parameter(torch.zeros_like(t).to(dev)); p.grad = t.to(dev); params.append(p)
    assert abs(pkg.compute_grad_norm(params).item() - want) < 1e-5 * want
    hand = torch.nn.Parameter(torch.zeros(3, device=dev)); hand.grad = torch.tensor([0.0, 3.0, 4.0], device=dev)
    assert abs(pkg.compute_grad_norm([hand]).item() - 5 / math.sqrt(2)) < 1e-6
    # clipping: same rule as the reference, decided on the device
    norm = pkg.clip_grad_norm([hand], max_norm=1.0)
    assert torch.allclose(hand.grad.cpu(), torch.tensor([0.0, 3.0, 4.0]) / (5 / math.sqrt(2) + 1e-6), rtol=1e-6)
    assert abs(norm.item() - 5 / math.sqrt(2)) < 1e-6
    hand.grad = torch.tensor([0.0, 3.0, 4.0], device=dev)
    pkg.clip_grad_norm([hand], max_norm=math.inf)
    assert torch.equal(hand.grad.cpu(), torch.tensor([0.0, 3.0, 4.0]))


def test_hip_sparse_adam_optimizer_on_module(pkg, oracle, dev):
    from lm_saes_amd import synthetic

    d, F, k, B = 128, 1024, 8, 96
    x = synthetic.activations(B, d, 8, seed=3)
    w = synthetic.sae_weights(d, F, x, seed=3)
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                        top_k=k, norm_activation="inference", device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    synthetic.load_weights(sae, *[t.to(dev) for t in w])
    opt = pkg.HipSparseAdam(sae.get_parameters()[0]["params"], lr=1e-3, model=sae)
    before = {n: p.detach().clone() for n, p in sae.named_parameters()}
    sae.compute_loss({"in": x.to(dev), "out": x.to(dev), "tokens": torch.zeros(B, device=dev)})["loss"].backward()
    grads = {n: p.grad.clone() for n, p in sae.named_parameters()}
    opt.step()
    for n, p in sae.named_parameters():
        moved = (p.detach() - before[n]).abs()
        nz = grads[n] != 0
        big = grads[n].abs() > 1e-3  # first step: lr * sign(g), up to eps / (sqrt(1 - beta2) |g|)
        assert torch.allclose(moved[big], torch.full_like(moved[big], 1e-3), rtol=2e-3), n
        assert (moved[nz] <= 1e-3 * 1.002).all() and big.any(), n
        assert (moved[~nz] == 0).all(), n                                                  # untouched where g == 0
    assert (~(grads["W_D"] != 0)).any()


def test_trainer_fit_follows_the_oracle_loop(pkg, oracle, dev):
    """k annealing, LR warm-up, Adam: a short run tracked step by step against an oracle loop."""
    from lm_saes_amd import synthetic

    d, F, k, B, steps = 128, 1024, 4, 64, 6
    x = synthetic.activations(B * steps, d, 8, seed=5)
    w = synthetic.sae_weights(d, F, x[:B], seed=5)
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                        top_k=k, norm_activation="token-wise", device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    synthetic.load_weights(sae, *[t.to(dev) for t in w])
    tcfg = pkg.TrainerConfig(lr=1e-3, initial_k=16, k_warmup_steps=4, k_cold_booting_steps=1, lr_warm_up_steps=3,
                             lr_cool_down_steps=2, total_training_tokens=B * steps, amp_dtype=torch.float32,
                             l1_coefficient=None, skip_metrics_calculation=True)
    trainer = pkg.Trainer(tcfg)
    seen = []
    batches = [{"in": x[i * B:(i + 1) * B].to(dev), "out": x[i * B:(i + 1) * B].to(dev),
                "tokens": torch.zeros(B, dtype=torch.long, device=dev), "mask": torch.ones(B, device=dev)} for i in range(steps)]
    trainer.fit(sae, batches, on_step=lambda s, ctx: seen.append((s, sae.current_k, trainer.optimizer.param_groups[0]["lr"],
                                                                 ctx["loss"].item())))
    assert trainer.cur_step == steps and trainer.cur_tokens == B * steps

    ref = oracle.SAEOracle(d, F, act_fn="topk", top_k=k, norm_activation="token-wise")
    synthetic.load_weights(ref, *w)
    opt = oracle.make_adam(ref, lr=1e-3)
    total = steps
    lam = lambda s: min(1.0, (s + 1) / 3, 1 / 32 + (1 - 1 / 32) / 2 * max(total - s, 1))  # noqa: E731  constantwithwarmup
    for s in range(steps):
        ref.current_k = oracle.k_schedule(s, top_k=k, initial_k=16, k_cold_booting_steps=1, k_warmup_steps=4)
        for gparam in opt.param_groups:
            gparam["lr"] = 1e-3 * lam(s)
        xb = x[s * B:(s + 1) * B]
        b = ref.normalize_activations({"in": xb, "out": xb, "tokens": torch.zeros(B), "mask": torch.ones(B)})
        rctx = oracle.train_step(ref, opt, b)
        step_no, k_used, lr_used, loss = seen[s]
        assert step_no == s and k_used == ref.current_k
        assert abs(lr_used - 1e-3 * lam(s)) < 1e-12
        assert abs(loss - rctx["loss"].item()) < 2e-3 * rctx["loss"].item(), (s, loss, rctx["loss"].item())
    assert [t[1] for t in seen] == [16, 16, 13, 10, 7, 4]
