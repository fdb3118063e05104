"""Checkpoints cross between the oracle (reference layout on the CPU) and the HIP path in both directions."""

import json

import pytest
import safetensors.torch as safe
import torch

pytestmark = pytest.mark.gpu


def test_reference_layout_checkpoint_trains_on_the_hip_path_and_back(pkg, oracle, dev, tmp_path):
    from lm_saes_amd import synthetic

    d, F, k, B = 128, 1024, 8, 96
    x = synthetic.activations(B, d, 8, seed=31)
    w = synthetic.sae_weights(d, F, x, seed=31)
    ref = oracle.SAEOracle(d, F, act_fn="topk", top_k=k)
    synthetic.load_weights(ref, *w)
    # a directory as the reference writes it: config.json + sae_weights.safetensors with its key names and shapes
    (tmp_path / "config.json").write_text(json.dumps({
        "sae_type": "sae", "d_model": d, "expansion_factor": F / d, "hook_point_in": "in", "hook_point_out": "out",
        "act_fn": "topk", "top_k": k, "norm_activation": "inference"}))
    sd = {n: p.detach().clone().contiguous() for n, p in ref.named_parameters()}
    assert tuple(sd["W_E"].shape) == (d, F) and tuple(sd["W_D"].shape) == (F, d)
    safe.save_file(sd, str(tmp_path / "sae_weights.safetensors"))

    sae = pkg.SparseDictionary.from_pretrained(str(tmp_path), device="cuda", dtype=torch.float32)
    assert sae.W_E.is_cuda and torch.equal(sae.W_E.detach().cpu(), sd["W_E"])
    batch = {"in": x.to(dev), "out": x.to(dev), "tokens": torch.zeros(B, device=dev)}
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=1e-3, model=sae)
    ropt = oracle.make_adam(ref, lr=1e-3)
    for _ in range(3):
        loss = sae.compute_loss(batch, return_aux_data=False)
        loss.backward(); opt.step(); opt.zero_grad()
        rctx = oracle.train_step(ref, ropt, {"in": x, "out": x, "tokens": torch.zeros(B)})
        assert abs(loss.item() - rctx["loss"].item()) < 1e-4 * rctx["loss"].item()

    # back: the HIP-trained weights, saved by the package, loaded into the oracle
    out = tmp_path / "trained"
    sae.save_pretrained(str(out))
    back = safe.load_file(str(out / "sae_weights.safetensors"))
    probe = oracle.SAEOracle(d, F, act_fn="topk", top_k=k)
    probe.load_state_dict({n: back[n] for n, _ in probe.named_parameters()})
    want = probe.compute_loss({"in": x, "out": x, "tokens": torch.zeros(B)})["loss"].item()
    got = sae.compute_loss(batch, return_aux_data=False).item()
    assert abs(got - want) < 1e-5 * want
    for n, p in ref.named_parameters():
        assert (back[n] - p.detach()).abs().max() <= 2e-2 * 3e-3 + 1e-6 * p.detach().abs().max(), n


def _stream(x, B, n, dev):
    for i in range(n):
        rows = x[(i * B) % x.shape[0]:][:B]
        yield {"in": rows.to(dev), "out": rows.to(dev), "tokens": torch.zeros(B, device=dev),
               "mask": torch.ones(B, device=dev)}


def test_trainer_resumes_bit_identically_from_a_complete_checkpoint(pkg, dev, tmp_path):
    """trainer.py:155-307: three steps, a checkpoint, two more steps -- against loading the checkpoint into a fresh
    model + `Trainer.from_checkpoint` and running the same two steps: parameters and moments agree to the bit."""
    from lm_saes_amd import synthetic

    d, F, k, B = 128, 1024, 8, 96
    x = synthetic.activations(5 * B, d, 8, seed=41)
    w = synthetic.sae_weights(d, F, x, seed=41)

    def fresh():
        cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                            top_k=k, norm_activation="inference", device="cuda", dtype=torch.float32)
        m = pkg.SparseAutoEncoder(cfg)
        synthetic.load_weights(m, *[t.to(dev) for t in w])
        return m

    tcfg = pkg.TrainerConfig(total_training_tokens=5 * B, lr=1e-3, lr_warm_up_steps=2, lr_cool_down_steps=2, amp_dtype=None,
                             k_warmup_steps=0, l1_coefficient=None, skip_metrics_calculation=True,
                             exp_result_path=str(tmp_path / "results"))
    sae, tr = fresh(), pkg.Trainer(tcfg)
    batches = list(_stream(x, B, 5, dev))
    tr.prepare(sae, batches[0])
    for b in batches[:3]:
        tr.train_one_step(sae, b)
    ckpt = tr.save_checkpoint(sae, tmp_path / "run")
    for b in batches[3:]:
        tr.train_one_step(sae, b)

    sae2 = pkg.SparseDictionary.from_pretrained(str(ckpt), device="cuda", dtype=torch.float32)
    tr2 = pkg.Trainer.from_checkpoint(sae2, str(ckpt))
    assert tr2.cur_step == 3 and tr2.optimizer.param_groups[0]["lr"] == pytest.approx(1e-3)
    assert tr2.fit(sae2, iter(batches[3:])) is None and tr2.cur_step == 5
    torch.cuda.synchronize()
    for (n, p), q in zip(sae.named_parameters(), sae2.parameters()):
        assert torch.equal(p, q), n
        a, b = tr.optimizer.state[p], tr2.optimizer.state[q]
        assert torch.equal(a["exp_avg"], b["exp_avg"]) and torch.equal(a["exp_avg_sq"], b["exp_avg_sq"]), n
        assert float(a["step"]) == float(b["step"]) == 5.0


def test_adam_state_round_trip_through_torch_adam_continues_bit_identically(pkg, oracle, dev):
    """HipAdam's state after two steps is exported, loaded into a torch.optim.Adam over reference-layout parameters
    (the oracle model: W_E and its moments [d, F] contiguous), exported from there and loaded into a second HipAdam
    on a copy of the weights.  Both HIP models then take the same two steps: parameters and moments stay identical
    to the bit, and torch's Adam accepts the state (it takes a step of its own on the oracle from it)."""
    from lm_saes_amd import synthetic

    d, F, k, B = 128, 1024, 8, 96
    x = synthetic.activations(B, d, 8, seed=43)
    w = synthetic.sae_weights(d, F, x, seed=43)

    def fresh(weights):
        cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                            top_k=k, norm_activation="inference", device="cuda", dtype=torch.float32)
        m = pkg.SparseAutoEncoder(cfg)
        if isinstance(weights, dict):
            m.load_state_dict(weights)
        else:
            synthetic.load_weights(m, *weights)
        return m, pkg.HipAdam(m.get_parameters()[0]["params"], lr=1e-3, model=m)

    def steps(m, opt, n):
        for _ in range(n):
            m.compute_loss(batch, return_aux_data=False).backward()
            opt.step(); opt.zero_grad()

    batch = {"in": x.to(dev), "out": x.to(dev), "tokens": torch.zeros(B, device=dev)}
    a, opt_a = fresh([t.to(dev) for t in w])
    steps(a, opt_a, 2)
    # -> torch.optim.Adam on the oracle (reference layout), by parameter name
    ref = oracle.SAEOracle(d, F, act_fn="topk", top_k=k)
    ref.load_state_dict({n: p.detach().cpu().contiguous() for n, p in a.named_parameters()})
    ropt = oracle.make_adam(ref, lr=1e-3)
    names_a = {id(p): n for n, p in a.named_parameters()}
    names_r = {id(p): n for n, p in ref.named_parameters()}
    order_a = [names_a[id(p)] for g in opt_a.param_groups for p in g["params"]]
    order_r = [names_r[id(p)] for g in ropt.param_groups for p in g["params"]]
    sd_a = opt_a.state_dict()
    by_name = {order_a[i]: st for i, st in sd_a["state"].items()}
    assert by_name["W_E"]["exp_avg"].is_contiguous() and tuple(by_name["W_E"]["exp_avg"].shape) == (d, F)
    ropt.load_state_dict({"state": {i: by_name[n] for i, n in enumerate(order_r)}, "param_groups": ropt.state_dict()["param_groups"]})
    assert all(float(ropt.state[p]["step"]) == 2.0 for p in ref.parameters())
    # <- and back into a second HipAdam
    sd_r = ropt.state_dict()
    back = {order_r[i]: st for i, st in sd_r["state"].items()}
    b, opt_b = fresh({n: p.detach().clone() for n, p in a.named_parameters()})
    order_b = [{id(p): n for n, p in b.named_parameters()}[id(p)] for g in opt_b.param_groups for p in g["params"]]
    opt_b.load_state_dict({"state": {i: back[n] for i, n in enumerate(order_b)}, "param_groups": opt_b.state_dict()["param_groups"]})
    assert opt_b.state[b.W_E]["exp_avg"].stride() == b.W_E.stride()
    steps(a, opt_a, 2); steps(b, opt_b, 2)
    torch.cuda.synchronize()
    for (n, p), q in zip(a.named_parameters(), b.parameters()):
        assert torch.equal(p, q), n
        assert torch.equal(opt_a.state[p]["exp_avg"], opt_b.state[q]["exp_avg"]), n
        assert torch.equal(opt_a.state[p]["exp_avg_sq"], opt_b.state[q]["exp_avg_sq"]), n
        assert float(opt_a.state[p]["step"]) == float(opt_b.state[q]["step"]) == 4.0
    before = {n: p.detach().clone() for n, p in ref.named_parameters()}
    oracle.train_step(ref, ropt, {"in": x, "out": x, "tokens": torch.zeros(B)})
    assert all(torch.isfinite(p).all() and not torch.equal(p.detach(), before[n]) for n, p in ref.named_parameters())
