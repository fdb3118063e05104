"""Randomized parity sweep over the crosscoder, the cross-layer transcoder and Lorsa: shapes, activation scopes,
masks and positional embeddings are drawn from a seeded generator and every case's loss, outputs and parameter
gradients are checked against the variants' oracle (crosscoder.py:221-469, clt.py:527-709, 837-876,
lorsa.py:683-829), in fp32 and under bf16 autocast (there with the stage-by-stage checks of the fixed-shape tests: the
oracle's bf16 step on the kernels' own selection).  Each case prints its parameters before it runs.

The GEMMs on the two sides add in different orders, so two pre-activations that differ in their last bits may swap
places at the k-th rank: a case whose selections differ in a handful of entries is counted as a flip and its further
comparisons are skipped; flips must stay rare, and a selection that differs by more than that fails."""

import importlib.util
import math
import os
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

_spec = importlib.util.spec_from_file_location("_gpu_variant_checks", os.path.join(os.path.dirname(__file__), "test_gpu_variants.py"))
tv = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(tv)

vo = tv.vo     # the module-scoped fixture of the variants' oracle

N_CASES = 30
MAX_FLIPPED_ENTRIES = 4


def compare(out, want, m, ref, with_hidden_pre=True):
    """True when the whole case was compared, False when the selections differ by a near-tie swap."""
    kept, kept_want = (out["feature_acts"] > 0).cpu(), want["feature_acts"] > 0
    differing = int((kept != kept_want).sum())
    assert differing <= MAX_FLIPPED_ENTRIES, f"{differing} entries selected differently"
    if with_hidden_pre:
        assert tv.rel_err(out["hidden_pre"], want["hidden_pre"]) < tv.FP32_TOL
    if differing:
        return False
    assert tv.rel_err(out["feature_acts"], want["feature_acts"]) < tv.FP32_TOL
    assert tv.rel_err(out["reconstructed"], want["reconstructed"]) < tv.FP32_TOL
    assert tv.rel_err(out["loss"], want["loss"]) < tv.FP32_TOL
    out["loss"].backward(); want["loss"].backward()
    tv.check_grads(m, ref)
    return True


def few_flips(flips, n):
    print(f"{flips} of {n} cases held a near-tie swap", flush=True)
    assert flips <= max(2, n // 4), f"{flips} of {n} cases selected differently from the oracle"


@pytest.mark.parametrize("sweep_seed", [11, 21])
def test_crosscoder_random_shapes(pkg, vo, dev, sweep_seed):
    rng = random.Random(sweep_seed)
    flips = 0
    for n in range(N_CASES):
        H = rng.choice([2, 3, 5]); d = rng.choice([32, 64, 96]); F = rng.choice([128, 384, 640, 1024])
        k = rng.choice([1, 4, 9, 32]); B = rng.choice([1, 17, 64, 130]); masked = rng.random() < 0.4
        seed = rng.randrange(1 << 20)
        print(f"[{n}] crosscoder seed={seed} H={H} d={d} F={F} k={k} B={B} masked={masked}", flush=True)
        m, ref, hooks = tv.make_crosscoder(pkg, vo, dev, H, d, F, k, seed=seed)
        g = torch.Generator().manual_seed(seed + 1)
        batch = {h: torch.randn(B, d, generator=g) for h in hooks}
        batch["tokens"] = torch.zeros(B, dtype=torch.long)
        mask = (torch.rand(B, H, generator=g) > 0.3).float() if masked else None
        if mask is not None and float(mask.sum()) == 0:
            mask[0, 0] = 1.0
        gb = {k_: v.to(dev) for k_, v in batch.items()}
        if mask is not None:
            gb["mask"] = mask.to(dev)
        out = m.compute_loss(gb)
        assert "sparse_codes" in out, "the kernel path did not run"
        want = ref.compute_loss(batch, hooks, mask=mask)
        flips += not compare(out, want, m, ref)
    few_flips(flips, N_CASES)


@pytest.mark.parametrize("sweep_seed", [12, 22])
def test_clt_random_shapes(pkg, vo, dev, sweep_seed):
    rng = random.Random(sweep_seed)
    flips = 0
    for n in range(N_CASES):
        act_fn = rng.choice(["topk", "layertopk", "batchtopk", "batchlayertopk"])
        L = rng.choice([2, 3, 5]); d = rng.choice([32, 64]); F = rng.choice([128, 192, 320]); k = rng.choice([2, 6, 11])
        B = rng.choice([8, 50, 96]); include_norm = rng.random() < 0.6
        seed = rng.randrange(1 << 20)
        print(f"[{n}] clt seed={seed} {act_fn} L={L} d={d} F={F} k={k} B={B} include_norm={include_norm}", flush=True)
        m, ref, hin, hout = tv.make_clt(pkg, vo, dev, act_fn, L, d, F, k, seed=seed, include_norm=include_norm)
        batch = tv.clt_batch(L, B, d, seed=seed + 1)
        gb = {k_: v.to(dev) for k_, v in batch.items()}
        out = m.compute_loss(gb)
        assert "sparse_code" in out, "the kernel path did not run"
        want = ref.compute_loss(batch, hin, hout)
        flips += not compare(out, want, m, ref, with_hidden_pre=False)    # the transcoder's loss reports no hidden_pre
    few_flips(flips, N_CASES)


@pytest.mark.parametrize("sweep_seed", [13, 23])
def test_lorsa_random_shapes(pkg, vo, dev, sweep_seed):
    rng = random.Random(sweep_seed)
    flips = 0
    for n in range(N_CASES):
        d = rng.choice([64, 96]); F = rng.choice([128, 256, 512]); h = rng.choice([2, 4]); dq = rng.choice([16, 32])
        s = rng.choice([8, 16, 40]); b = rng.choice([1, 3]); k = rng.choice([2, 8]); masked = rng.random() < 0.5
        kw = rng.choice([dict(positional_embedding_type="none"),
                         dict(positional_embedding_type="rotary", rotary_dim=16),
                         dict(positional_embedding_type="none", sparsity_include_decoder_norm=False)])
        seed = rng.randrange(1 << 20)
        print(f"[{n}] lorsa seed={seed} d={d} F={F} h={h} dq={dq} s={s} b={b} k={k} masked={masked} {kw}", flush=True)
        m, ref = tv.make_lorsa(pkg, vo, dev, d, F, h, dq, max(s, 16), k, seed=seed, **kw)
        g = torch.Generator().manual_seed(seed + 1)
        batch = {"in": torch.randn(b, s, d, generator=g), "out": torch.randn(b, s, d, generator=g), "tokens": torch.zeros(b, s)}
        mask = (torch.rand(b, s, generator=g) > 0.2).float() if masked else None
        if mask is not None and float(mask.sum()) == 0:
            mask[0, 0] = 1.0
        gb = {k_: v.to(dev) for k_, v in batch.items()}
        if mask is not None:
            gb["mask"] = mask.to(dev)
        out = m.compute_loss(gb)
        assert "sparse_code" in out, "the kernel path did not run"
        want = ref.compute_loss(batch, mask=mask)
        flips += not compare(out, want, m, ref)
    few_flips(flips, N_CASES)


N_BF16_CASES = 12


@pytest.mark.parametrize("sweep_seed", [31, 41, 51])
def test_bf16_steps_over_random_shapes(pkg, vo, dev, sweep_seed):
    rng = random.Random(sweep_seed)
    for n in range(N_BF16_CASES):
        seed = rng.randrange(1 << 20)
        H = rng.choice([2, 3, 4]); d = rng.choice([64, 128]); F = rng.choice([256, 512, 1024]); k = rng.choice([4, 16])
        B = rng.choice([64, 96, 130])
        print(f"[{n}] crosscoder bf16 seed={seed} H={H} d={d} F={F} k={k} B={B}", flush=True)
        tv.crosscoder_bf16_step(pkg, vo, dev, H, d, F, k, B, seed=seed)
    for n in range(N_BF16_CASES):
        seed = rng.randrange(1 << 20)
        act_fn = rng.choice(["topk", "topk", "layertopk", "batchtopk", "batchlayertopk"])
        L = rng.choice([2, 3, 4]); d = rng.choice([64, 128]); F = rng.choice([256, 512]); k = rng.choice([4, 8]); B = rng.choice([64, 96, 160])
        print(f"[{n}] clt bf16 seed={seed} {act_fn} L={L} d={d} F={F} k={k} B={B}", flush=True)
        tv.clt_bf16_step(pkg, vo, dev, act_fn, L, d, F, k, B, seed=seed)
    for n in range(N_BF16_CASES):
        seed = rng.randrange(1 << 20)
        d = rng.choice([64, 128]); h = rng.choice([2, 4, 8]); dv = rng.choice([32, 64, 128]); dq = rng.choice([32, 64])
        s = rng.choice([8, 24, 64, 104]); b = (64 // math.gcd(s, 64)) * rng.choice([1, 2]); dense = rng.random() < 0.5
        kw = rng.choice([dict(positional_embedding_type="none"),
                         dict(positional_embedding_type="rotary", rotary_dim=rng.choice([16, 32, dq]),
                              rotary_adjacent_pairs=rng.random() < 0.5)])
        print(f"[{n}] lorsa bf16 seed={seed} d={d} h={h} dv={dv} dq={dq} s={s} b={b} dense={dense} {kw}", flush=True)
        tv.lorsa_bf16_step(pkg, vo, dev, d, h * dv, h, dq, s, b, dense, seed=seed, **kw)
