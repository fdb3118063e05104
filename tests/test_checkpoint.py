"""Checkpoint files in the reference's format: the reference's own loading recipe
(tests/unit/test_from_local.py:17-60), round trips, key names, shapes and the search order."""

import json
import os

import pytest
import safetensors
import safetensors.torch as safe
import torch


REF_CONFIG = {  # tests/unit/test_from_local.py:20-28
    "sae_type": "sae", "d_model": 8, "expansion_factor": 2, "hook_point_in": "layer_0", "hook_point_out": "layer_0",
    "device": "cpu", "dtype": "float32",
}


def _reference_style_dir(tmp_path, with_pt=True):
    (tmp_path / "config.json").write_text(json.dumps(REF_CONFIG))
    sd = {"W_E": torch.full((8, 16), 1.0), "b_E": torch.full((16,), 2.0), "W_D": torch.full((16, 8), 3.0), "b_D": torch.full((8,), 4.0)}
    safe.save_file(sd, str(tmp_path / "sae_weights.safetensors"))
    if with_pt:
        torch.save({"sae": sd}, str(tmp_path / "sae_weights.pt"))
    return tmp_path


def test_from_local_reads_a_reference_directory(pkg, tmp_path):
    d = _reference_style_dir(tmp_path)
    model = pkg.SparseDictionary.from_local(str(d))
    assert isinstance(model, pkg.SparseAutoEncoder)
    assert model.W_E.shape == (8, 16) and model.W_D.shape == (16, 8)
    assert torch.equal(model.W_E, torch.ones(8, 16)) and torch.equal(model.b_E, torch.full((16,), 2.0))
    assert torch.equal(model.W_D, torch.full((16, 8), 3.0)) and torch.equal(model.b_D, torch.full((8,), 4.0))
    assert model.cfg.sae_pretrained_name_or_path is None
    # the .pt form, named directly
    model = pkg.SparseDictionary.from_local(str(d / "sae_weights.pt"))
    assert torch.equal(model.W_D, torch.full((16, 8), 3.0))
    # and through from_config, as a config that names pretrained weights does
    cfg = pkg.SparseDictionaryConfig.from_pretrained(str(d))
    assert isinstance(cfg, pkg.SAEConfig) and cfg.sae_pretrained_name_or_path == str(d)
    assert torch.equal(pkg.SparseDictionary.from_config(cfg).b_D, torch.full((8,), 4.0))


def test_round_trip_preserves_values_layout_and_norms(pkg, tmp_path):
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=6, expansion_factor=3, act_fn="relu",
                        norm_activation="dataset-wise")
    sae = pkg.SparseAutoEncoder(cfg)
    g = torch.Generator().manual_seed(0)
    with torch.no_grad():
        for p in sae.parameters():
            p.copy_(torch.randn(p.shape, generator=g))
    sae.set_dataset_average_activation_norm({"in": 3.0, "out": 2.0})
    sae.save_pretrained(str(tmp_path))
    cfg.save_hyperparameters(str(tmp_path))
    on_disk = json.loads((tmp_path / "config.json").read_text())
    assert "sae_pretrained_name_or_path" not in on_disk and "device" not in on_disk and on_disk["sae_type"] == "sae"
    with safetensors.safe_open(str(tmp_path / "sae_weights.safetensors"), framework="pt") as f:
        keys = set(f.keys())
        assert keys == {"W_E", "b_E", "W_D", "b_D", "dataset_average_activation_norm.in", "dataset_average_activation_norm.out"}
        assert "version" in f.metadata()
        w_e = f.get_tensor("W_E")
        assert tuple(w_e.shape) == (6, 18) and w_e.is_contiguous()          # the reference's [d_model, d_sae] row-major
        assert torch.equal(w_e, sae.W_E.detach())
        assert f.get_tensor("dataset_average_activation_norm.in").item() == 3.0
    back = pkg.SparseAutoEncoder.from_pretrained(str(tmp_path))
    assert back.cfg.model_dump() == sae.cfg.model_dump()
    assert back.dataset_average_activation_norm == {"in": 3.0, "out": 2.0}
    for (n, p), q in zip(sae.named_parameters(), back.parameters()):
        assert torch.equal(p, q), n
    # same function after the round trip
    x = torch.randn(5, 6, generator=g)
    assert torch.equal(sae.forward(x), back.forward(x))


def test_search_order_and_errors(pkg, tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(REF_CONFIG))
    with pytest.raises(FileNotFoundError):
        pkg.SparseDictionary.from_local(str(tmp_path))
    os.makedirs(tmp_path / "checkpoints")
    sd = lambda v: {"W_E": torch.full((8, 16), v), "b_E": torch.zeros(16), "W_D": torch.zeros(16, 8), "b_D": torch.zeros(8)}  # noqa: E731
    safe.save_file(sd(1.0), str(tmp_path / "checkpoints" / "final.safetensors"))
    assert pkg.SparseDictionary.from_local(str(tmp_path)).W_E[0, 0] == 1.0
    torch.save({"sae": sd(2.0)}, str(tmp_path / "checkpoints" / "pruned.pt"))
    assert pkg.SparseDictionary.from_local(str(tmp_path)).W_E[0, 0] == 2.0      # pruned before final
    safe.save_file(sd(3.0), str(tmp_path / "sae_weights.safetensors"))
    assert pkg.SparseDictionary.from_local(str(tmp_path)).W_E[0, 0] == 3.0      # sae_weights first
    assert pkg.SparseDictionary.from_local(str(tmp_path / "checkpoints" / "final.safetensors")).W_E[0, 0] == 1.0
    model = pkg.SparseDictionary.from_local(str(tmp_path))
    with pytest.raises(ValueError):
        model.save_checkpoint(str(tmp_path / "weights.bin"))
    with pytest.raises(ValueError):
        pkg.SparseAutoEncoder.from_pretrained("some-org/some-repo:name")
    # strict loading: a missing key is an error unless strict_loading=False
    bad = sd(5.0); del bad["b_D"]
    safe.save_file(bad, str(tmp_path / "sae_weights.safetensors"))
    with pytest.raises(RuntimeError):
        pkg.SparseDictionary.from_local(str(tmp_path))
    assert pkg.SparseDictionary.from_local(str(tmp_path), strict_loading=False).W_E[0, 0] == 5.0


def test_pt_checkpoint_round_trip_and_jumprelu_key(pkg, tmp_path):
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=4, expansion_factor=2, act_fn="jumprelu",
                        norm_activation="inference")
    sae = pkg.SparseAutoEncoder(cfg)
    with torch.no_grad():
        sae.activation_function.log_jumprelu_threshold.fill_(-1.5)
    sae.save_checkpoint(str(tmp_path / "sae_weights.pt"))
    cfg.save_hyperparameters(str(tmp_path))
    blob = torch.load(str(tmp_path / "sae_weights.pt"), weights_only=True)
    assert set(blob) == {"sae", "version"} and "activation_function.log_jumprelu_threshold" in blob["sae"]
    back = pkg.SparseDictionary.from_local(str(tmp_path))
    assert torch.equal(back.activation_function.log_jumprelu_threshold, torch.full((8,), -1.5))


@pytest.mark.parametrize("kind", ["crosscoder", "clt", "lorsa"])
def test_variant_checkpoints_round_trip(pkg, tmp_path, kind):
    if kind == "crosscoder":
        cfg = pkg.CrosscoderConfig(hook_points=["a", "b"], d_model=6, expansion_factor=2, act_fn="topk", top_k=3,
                                   norm_activation="inference")
    elif kind == "clt":
        cfg = pkg.CLTConfig(hook_points_in=["i0", "i1"], hook_points_out=["o0", "o1"], d_model=6, expansion_factor=2,
                            act_fn="topk", top_k=3, norm_activation="inference")
    else:
        cfg = pkg.LorsaConfig(hook_point_in="in", hook_point_out="out", d_model=8, expansion_factor=2, n_qk_heads=2,
                              d_qk_head=4, n_ctx=16, act_fn="topk", top_k=3, norm_activation="inference",
                              positional_embedding_type="rotary", rotary_dim=4)
    model = pkg.SparseDictionary.from_config(cfg)
    g = torch.Generator().manual_seed(1)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=g))
    model.save_pretrained(str(tmp_path))
    cfg.save_hyperparameters(str(tmp_path))
    back = pkg.SparseDictionary.from_pretrained(str(tmp_path))
    assert type(back) is type(model) and back.cfg.model_dump() == cfg.model_dump()
    for (n, p), q in zip(model.named_parameters(), back.parameters()):
        assert torch.equal(p, q), n
    with safetensors.safe_open(str(tmp_path / "sae_weights.safetensors"), framework="pt") as f:
        for k in f.keys():
            if not k.startswith("dataset_average_activation_norm."):
                assert tuple(f.get_tensor(k).shape) == tuple(model.state_dict()[k].shape), k


# ---- trainer checkpoints (trainer.py:155-307) and optimizer-state interchange with torch.optim.Adam ----

def _tiny_sae(pkg, device="cpu"):
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=8, expansion_factor=2, act_fn="topk", top_k=2,
                        norm_activation="inference", device=device, dtype=torch.float32)
    m = pkg.SparseAutoEncoder(cfg)
    g = torch.Generator().manual_seed(3)
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(torch.randn(p.shape, generator=g))
    return m


def test_adam_state_crosses_between_torch_adam_and_hip_adam(pkg):
    """A torch.optim.Adam state dict (moments contiguous in the reference's [d, F] shape for W_E) loads into HipAdam
    with the moments re-laid to the parameter's feature-major strides, and HipAdam's own state dict goes back."""
    m = _tiny_sae(pkg)
    twin = {n: torch.nn.Parameter(p.detach().clone().contiguous()) for n, p in m.named_parameters()}
    topt = torch.optim.Adam(list(twin.values()), lr=1e-3)
    g = torch.Generator().manual_seed(4)
    for _ in range(2):
        for p in twin.values():
            p.grad = torch.randn(p.shape, generator=g)
        topt.step()
    sd = topt.state_dict()
    assert sd["state"][0]["exp_avg"].is_contiguous()
    hopt = pkg.HipAdam(list(m.parameters()), lr=1e-3, model=m)
    hopt.load_state_dict(sd)
    for (n, p), q in zip(m.named_parameters(), twin.values()):
        st = hopt.state[p]
        assert st["exp_avg"].stride() == p.stride() and st["exp_avg_sq"].stride() == p.stride(), n
        assert torch.equal(st["exp_avg"], topt.state[q]["exp_avg"]) and torch.equal(st["exp_avg_sq"], topt.state[q]["exp_avg_sq"])
        assert st["step"].device.type == "cpu" and float(st["step"]) == 2.0
    assert m.W_E.stride() == (1, 8) and hopt.state[m.W_E]["exp_avg"].t().is_contiguous()
    back = hopt.state_dict()
    assert hopt.state[m.W_E]["exp_avg"].stride() == m.W_E.stride()      # exporting left the live state as it was
    assert all(s["exp_avg"].is_contiguous() and s["exp_avg_sq"].is_contiguous() for s in back["state"].values())
    topt2 = torch.optim.Adam([torch.nn.Parameter(p.detach().clone().contiguous()) for p in m.parameters()], lr=1e-3)
    topt2.load_state_dict(back)
    for a, b in zip(topt2.state.values(), topt.state.values()):
        assert torch.equal(a["exp_avg"], b["exp_avg"]) and torch.equal(a["exp_avg_sq"], b["exp_avg_sq"]) and float(a["step"]) == 2.0
    with pytest.raises(ValueError, match="shape"):
        bad = topt.state_dict()
        bad["state"][0]["exp_avg"] = torch.zeros(3, 3)
        pkg.HipAdam(list(m.parameters()), lr=1e-3).load_state_dict(bad)


def test_trainer_checkpoint_file_set_and_resume_state(pkg, tmp_path):
    """The reference's directory layout and the counters a resumed trainer starts from."""
    m = _tiny_sae(pkg)
    cfg = pkg.TrainerConfig(total_training_tokens=40, lr=1e-3, lr_warm_up_steps=2, lr_cool_down_steps=2, amp_dtype=None,
                            k_warmup_steps=0, l1_coefficient=None, n_checkpoints=2, check_point_save_mode="linear",
                            exp_result_path=str(tmp_path / "results"))
    tr = pkg.Trainer(cfg)
    tr._initialize_trainer(m, {"tokens": torch.zeros(4)})
    assert tr.total_training_steps == 10 and tr.checkpoint_thresholds == [5]
    tr._initialize_optimizer(m)
    for _ in range(3):     # the counters and the LR schedule move as in three steps (no kernel runs on the CPU)
        tr.scheduler.step(); tr.cur_step += 1; tr.cur_tokens += 4
    ckpt = tr.save_checkpoint(m, tmp_path / "run")
    assert ckpt == tmp_path / "run" / "checkpoints" / "step_3"
    assert sorted(p.name for p in ckpt.iterdir()) == ["config.json", "optimizer.pt", "sae_weights.safetensors", "scheduler.pt", "trainer.pt"]
    m2 = pkg.SparseDictionary.from_pretrained(str(ckpt), device="cpu", dtype=torch.float32)
    assert all(torch.equal(a, b) for a, b in zip(m.parameters(), m2.parameters()))
    tr2 = pkg.Trainer.from_checkpoint(m2, str(ckpt))
    assert (tr2.cur_step, tr2.cur_tokens, tr2.total_training_steps, tr2.checkpoint_thresholds) == (3, 12, 10, [5])
    assert tr2.cfg.from_pretrained_path == str(ckpt) and tr2.cfg.amp_dtype is None and tr2.cfg.lr == 1e-3
    assert tr2.scheduler.last_epoch == 3 and tr2.optimizer.param_groups[0]["lr"] == tr.optimizer.param_groups[0]["lr"]
    with pytest.raises(ValueError, match="not found"):
        pkg.Trainer.from_checkpoint(m2, str(tmp_path))
    # "log" thresholds as the reference computes them (trainer.py:339-343)
    tr3 = pkg.Trainer(pkg.TrainerConfig(total_training_tokens=4096, n_checkpoints=4, exp_result_path=str(tmp_path / "r3")))
    tr3._initialize_trainer(m, {"tokens": torch.zeros(4)})
    import math
    assert tr3.checkpoint_thresholds == [math.ceil(2 ** (i / 4 * 10)) * 4 for i in (1, 2, 3)]
