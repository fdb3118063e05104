"""Randomized parity sweep over the selection, feature-index and Adam entry points: shapes, dtypes, tie
densities, masks and seeds are drawn from a seeded generator and every case is checked against the oracle (or,
for the Adam rows passes, against the dense route) to the bit.  Each case prints its parameters before it runs.
A time budget bounds the run (a few thousand cases); longer runs of the same generator are a matter of raising it."""

import importlib.util
import os
import random
import time

import pytest
import torch

pytestmark = pytest.mark.gpu

_spec = importlib.util.spec_from_file_location("_gpu_kernel_checks", os.path.join(os.path.dirname(__file__), "test_gpu_kernels.py"))
tk = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(tk)


def quant(t, levels):
    return (t * levels).round() / levels

@pytest.mark.parametrize("sweep_seed", [1, 2])
def test_random_sweep(pkg, oracle, dev, sweep_seed, budget_s=12.0):
    rng = random.Random(sweep_seed)
    t0 = time.time()
    n = 0
    while time.time() - t0 < budget_s:
        n += 1
        kind = rng.choice(['row', 'row', 'row_lowp', 'row_mask', 'batch', 'batch', 'fi_adam', 'adam_lowp'])
        seed = rng.randrange(1 << 30)
        g = torch.Generator().manual_seed(seed)
        if kind.startswith('row'):
            B = rng.choice([1, 3, 8, 17]); F = rng.choice([37, 512, 1000, 4096, 8192, 12288, 24576, 65536, 131072, 50000])
            k = min(F, rng.choice([1, 4, 16, 32, 64, 128, 300]))
            dt = rng.choice([torch.float32, torch.bfloat16])
            ties = rng.choice([0, 0, 4, 64])
            pre = torch.randn(B, F, generator=g)
            if ties: pre = quant(pre, ties)
            if rng.random() < 0.2: pre[:, : F // 2] = -1.0
            pre = pre.to(dt)
            b = 0.1 * torch.randn(F, generator=g) if rng.random() < 0.7 else None
            s = 0.5 + torch.rand(F, generator=g) if rng.random() < 0.7 else None
            print(f'[{n}] {kind} seed={seed} B={B} F={F} k={k} {dt} ties={ties} b={b is not None} s={s is not None}', flush=True)
            if kind == 'row':
                tk.check_select(pkg, oracle, dev, pre, b, s, k, rng.choice([None, None, 0, 64]))
            elif kind == 'row_lowp':
                pre = pre.bfloat16(); bb = (b if b is not None else torch.zeros(F)).bfloat16(); nn = (s if s is not None else torch.ones(F)).bfloat16()
                h1 = (pre + bb) * nn
                want = oracle.topk(h1 * h1.gt(0).to(h1.dtype), k=k, dim=-1) / nn
                got = pkg.ops.select_topk_row(pre.to(dev), bb.float().to(dev), nn.float().to(dev), k, lowp=True).to_dense().cpu()
                assert torch.equal(got, want.float())
            else:
                fm = (torch.rand(F, generator=g) < rng.choice([0.01, 0.2, 0.9])).float()
                if s is None: s = 0.5 + torch.rand(F, generator=g)
                code = pkg.ops.select_topk_row(pre.to(dev), None if b is None else b.to(dev), s.to(dev), k, feat_mask=fm.to(dev))
                h0 = pre.float() + (b if b is not None else 0.0)
                h1 = ((h0 * s) / s * fm) * s
                want = oracle.topk(h1 * h1.gt(0).to(h1.dtype), k=k, dim=-1) / s
                assert torch.equal(code.to_dense().cpu(), want)
        elif kind == 'batch':
            B = rng.choice([2, 5, 16, 33]); F = rng.choice([64, 1000, 4096, 8192, 32768]); k = rng.choice([1, 4, 32, 64])
            k_total = min(B * F, k * B)
            dt = rng.choice([torch.float32, torch.bfloat16]); ties = rng.choice([0, 0, 4, 64])
            pre = torch.randn(B, F, generator=g)
            if ties: pre = quant(pre, ties)
            pre = pre.to(dt)
            b = 0.1 * torch.randn(F, generator=g) if rng.random() < 0.7 else None
            s = 0.5 + torch.rand(F, generator=g) if rng.random() < 0.7 else None
            fm = (torch.rand(F, generator=g) < 0.3).float() if (s is not None and rng.random() < 0.3) else None
            print(f'[{n}] batch seed={seed} B={B} F={F} k_total={k_total} {dt} ties={ties} mask={fm is not None}', flush=True)
            tk.check_batch_select(pkg, oracle, dev, pre, b, s, k_total, fm, k_on_device=rng.random() < 0.3)
        elif kind == 'fi_adam':
            B = rng.choice([16, 64, 300]); d = rng.choice([64, 256, 768, 2048, 4096]); F = rng.choice([96, 256, 1000]); k = rng.choice([3, 8, 16])
            dd = rng.choice([torch.float32, torch.bfloat16])
            print(f'[{n}] fi_adam seed={seed} B={B} d={d} F={F} k={k} {dd}', flush=True)
            code = tk.random_code(pkg, dev, B, F, k, seed=seed)
            fi = pkg.ops.build_feature_index(code)
            dense = torch.randn(B, d, generator=g).to(dd).to(dev); coef = torch.randn(code.n_slots, generator=g).to(dev)
            p0 = torch.randn(F, d, generator=g).to(dev)
            hy = dict(lr=4e-4, beta1=0.9, beta2=0.999, eps=1e-8)
            pa, ma, va = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0); pb, mb, vb = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
            for step in (1, 2):
                rows, _ = pkg.ops.sparse_grad_rows(fi, coef, dense, F, want_bias=True)
                pkg.ops.adam_step(pa, rows, ma, va, step=step, **hy)
                pkg.ops.adam_step_sparse_rows(fi, coef, dense, pb, mb, vb, step=step, **hy)
                assert torch.equal(pa, pb) and torch.equal(ma, mb) and torch.equal(va, vb)
        else:
            B = rng.choice([16, 64, 300]); d = rng.choice([64, 256, 768, 2048, 4096, 5120]); F = rng.choice([96, 256, 1000, 3000]); k = rng.choice([3, 8, 16])
            dd = rng.choice([torch.float32, torch.bfloat16])
            print(f'[{n}] adam_lowp seed={seed} B={B} d={d} F={F} k={k} {dd}', flush=True)
            code = tk.random_code(pkg, dev, B, F, k, seed=seed)
            fi = pkg.ops.build_feature_index(code)
            dense = torch.randn(B, d, generator=g).to(dd).to(dev); coef = torch.randn(code.n_slots, generator=g).to(dev)
            p0 = torch.randn(F, d, generator=g).bfloat16().to(dev)
            hy = dict(lr=4e-4, beta1=0.9, beta2=0.999, eps=1e-8)
            z = lambda: torch.zeros(F, d, dtype=torch.bfloat16, device=dev)
            pa, ma, va, pb, mb, vb = p0.clone(), z(), z(), p0.clone(), z(), z()
            for step in (1, 2, 3):
                rows, _ = pkg.ops.sparse_grad_rows(fi, coef, dense, F, want_bias=True)
                pkg.ops.adam_step(pa, rows.bfloat16(), ma, va, step=step, **hy)
                pkg.ops.adam_step_sparse_rows(fi, coef, dense, pb, mb, vb, step=step, **hy)
                assert torch.equal(pa, pb) and torch.equal(ma, mb) and torch.equal(va, vb)
    assert n > 100
