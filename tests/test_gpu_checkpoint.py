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
