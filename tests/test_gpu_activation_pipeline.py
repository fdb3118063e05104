"""Row-gather kernel, cached-activation stream to the GPU, and the initializer's grid search on the fused path."""

import pytest
import torch
from safetensors.torch import save_file

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("N,d,n,src,dst", [(100, 64, 37, torch.float32, torch.float32), (1000, 768, 512, torch.float32, torch.bfloat16),
                                            (64, 4096, 200, torch.bfloat16, torch.bfloat16), (50, 30, 50, torch.bfloat16, torch.float32),
                                            (33, 7, 90, torch.float32, torch.bfloat16)])
def test_gather_rows_kernel(pkg, dev, N, d, n, src, dst):
    g = torch.Generator().manual_seed(N + d)
    table = torch.randn(N, d, generator=g).to(src)
    idx = torch.randint(0, N, (n,), generator=g)
    out = pkg.ops.gather_rows(table.to(dev), idx.to(dev), out_dtype=dst)
    assert out.dtype == dst and torch.equal(out.cpu(), table[idx].to(dst))                       # a copy / a cast: exact
    out = pkg.ops.gather_rows(table.to(dev), idx.to(dev), out_dtype=dst, scale=0.37)
    want = (table[idx].float() * torch.tensor(0.37)).to(dst)
    assert torch.equal(out.cpu(), want)                                                            # one fp32 multiply, one rounding
    with pytest.raises(RuntimeError):
        pkg.ops.gather_rows(table, idx, out_dtype=dst)                                             # CPU tensors are refused


def _write_cache(root, hooks, n_chunks, n_samples, n_ctx, d, seed=0):
    g = torch.Generator().manual_seed(seed)
    want = []
    for c in range(n_chunks):
        tokens = torch.randint(0, 1000, (n_samples, n_ctx), generator=g)
        mask = (torch.rand(n_samples, n_ctx, generator=g) > 0.25).to(torch.int64)
        acts = {hp: torch.randn(n_samples, n_ctx, d, generator=g) for hp in hooks}
        for hp in hooks:
            (root / hp).mkdir(parents=True, exist_ok=True)
            save_file({"activation": acts[hp], "tokens": tokens, "mask": mask, "attention_mask": torch.ones_like(mask)},
                      str(root / hp / f"chunk-{c:08d}.safetensors"))
        want.append((tokens, mask, acts))
    return want


def test_cached_stream_on_the_gpu_equals_the_cpu_stream(pkg, dev, tmp_path):
    hooks = ["in", "out"]
    want = _write_cache(tmp_path, hooks, n_chunks=6, n_samples=4, n_ctx=16, d=64)
    loader = pkg.CachedActivationLoader({hp: tmp_path / hp for hp in hooks}, device="cuda")
    chunks = list(loader.process())
    assert len(chunks) == 6 and all(c["in"].is_cuda and c["tokens"].is_cuda for c in chunks)
    for got, (tokens, mask, acts) in zip(chunks, want):
        assert torch.equal(got["tokens"].cpu(), tokens) and torch.equal(got["out"].cpu(), acts["out"])
    shuffle = pkg.BufferShuffleConfig(perm_seed=5)
    cpu = list(pkg.cached_activation_stream(tmp_path, hooks, batch_size=48, buffer_size=150, buffer_shuffle_config=shuffle, device="cpu",
                                            override_dtype=torch.bfloat16))
    gpu = list(pkg.cached_activation_stream(tmp_path, hooks, batch_size=48, buffer_size=150, buffer_shuffle_config=shuffle, device="cuda",
                                            override_dtype=torch.bfloat16))
    assert len(cpu) == len(gpu) > 3
    for a, b in zip(cpu, gpu):
        assert b["in"].is_cuda and b["in"].dtype == torch.bfloat16
        assert torch.equal(a["in"], b["in"].cpu()) and torch.equal(a["out"], b["out"].cpu()) and torch.equal(a["tokens"], b["tokens"].cpu())
    kept = sum(int(m.sum()) for _, m, _ in want)
    assert sum(b["in"].shape[0] for b in gpu) == kept


def test_trainer_consumes_a_cached_stream(pkg, dev, tmp_path):
    """files -> loader -> mask filter -> batchler -> Trainer.fit on the fused path."""
    from lm_saes_amd import synthetic

    d, F, k, B = 128, 1024, 8, 64
    x = synthetic.activations(8 * 96, d, 8, seed=3)
    (tmp_path / "in").mkdir()
    for c in range(8):
        save_file({"activation": x[c * 96:(c + 1) * 96].reshape(2, 48, d).contiguous(), "tokens": torch.arange(96).reshape(2, 48),
                   "mask": torch.ones(2, 48, dtype=torch.int64), "attention_mask": torch.ones(2, 48, dtype=torch.int64)},
                  str(tmp_path / "in" / f"chunk-{c:08d}.safetensors"))
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="in", d_model=d, expansion_factor=F / d, act_fn="topk", top_k=k,
                        norm_activation="inference", device="cuda", dtype=torch.float32)
    stream = pkg.cached_activation_stream(tmp_path, ["in"], batch_size=B, buffer_size=256, buffer_shuffle_config=pkg.BufferShuffleConfig())
    init = pkg.Initializer(pkg.InitializerConfig(grid_search_init_norm=True, bias_init_method="geometric_median"))
    sae = init.initialize_sae_from_config(cfg, activation_stream=stream)
    trainer = pkg.Trainer(pkg.TrainerConfig(lr=1e-3, lr_warm_up_steps=2, lr_cool_down_steps=1, total_training_tokens=B * 10,
                                            amp_dtype=torch.float32, l1_coefficient=None, log_frequency=5, k_warmup_steps=0))
    losses = []
    trainer.fit(sae, stream, on_step=lambda s, ctx: losses.append(ctx["loss"].item()))
    assert trainer.cur_step == 10 and len(losses) == 10 and losses[-1] < losses[0]
    assert trainer.last_logged is not None and trainer.last_logged["metrics/l0"] == pytest.approx(k)


def test_grid_search_on_the_fused_path_matches_oracle_brute_force(pkg, oracle, dev):
    from lm_saes_amd import synthetic

    d, F, k, B = 128, 1024, 8, 256
    x = synthetic.activations(B, d, 8, seed=7)
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="in", d_model=d, expansion_factor=F / d, act_fn="topk", top_k=k,
                        norm_activation="inference", device="cuda", dtype=torch.float32)
    torch.manual_seed(1)
    init = pkg.Initializer(pkg.InitializerConfig(grid_search_init_norm=True, bias_init_method="geometric_median"))
    sae = init.initialize_sae_from_config(cfg, activation_stream=[{"in": x.to(dev), "tokens": torch.zeros(B, device=dev)}])
    direction = (sae.W_D.detach() / sae.W_D.detach().norm(dim=1, keepdim=True)).cpu()

    def mse(norm):
        ref = oracle.SAEOracle(d, F, act_fn="topk", top_k=k)
        with torch.no_grad():
            ref.W_D.copy_(direction * norm); ref.W_E.copy_(ref.W_D.t()); ref.b_E.zero_(); ref.b_D.copy_(x.mean(0))
            return ref.compute_loss({"in": x, "out": x, "tokens": torch.zeros(B)})["l_rec"].mean().item()

    coarse = min(torch.linspace(0.1, 5.0, 50).numpy().tolist(), key=mse)
    fine = min(torch.linspace(coarse - 0.09, coarse + 0.1, 20).numpy().tolist(), key=mse)
    assert init.best_norm == pytest.approx(fine, abs=0.0101)
    assert mse(init.best_norm) <= mse(fine) * (1 + 1e-4)
    assert torch.allclose(sae.decoder_norm().cpu(), torch.full((F,), init.best_norm), rtol=1e-5)
