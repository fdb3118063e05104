"""Pins of the metrics oracle (closed forms, hand cases, scalar loops) and the product's dense metric
formulas against it on the CPU."""

import importlib
import math

import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def mo():
    import __graft_entry__  # noqa: F401  (puts the repository root on sys.path)
    return importlib.import_module("oracle.metrics_oracle")


def test_record_reductions_and_reset(mo):
    r = mo.Record()
    r.update(2.0); r.update(4.0)
    assert r.compute() == 3.0 and r.value is None and r.count == 0
    r = mo.Record("mean"); r.update(torch.tensor([2.0, 6.0]), 4); r.update(torch.tensor([2.0, 2.0]), 4)
    assert torch.equal(r.compute(), torch.tensor([0.5, 1.0]))
    r = mo.Record("max"); [r.update(v) for v in (1.0, 5.0, 3.0)]
    assert r.compute() == 5.0
    r = mo.Record("min"); [r.update(v) for v in (4.0, 2.0, 3.0)]
    assert r.compute() == 2.0
    r = mo.Record("sum"); [r.update(v) for v in (4.0, 2.0)]
    assert r.compute() == 6.0
    with pytest.raises(AssertionError):
        mo.Record().compute()
    r = mo.Record(); r.update(torch.tensor(1.5, dtype=torch.bfloat16))
    assert r.value.dtype == torch.float32


def test_frequency_l0_mean_act_hand_case(mo):
    acts = torch.tensor([[0.0, 2.0, 0.0, 1.0],
                         [3.0, 0.0, 0.0, 1.0],
                         [0.0, 0.0, 0.0, -1.0]])
    assert torch.equal(mo.act_freq_scores(acts, None), torch.tensor([1.0, 1.0, 0.0, 2.0]))
    mask = torch.tensor([1.0, 0.0, 1.0])
    assert torch.equal(mo.act_freq_scores(acts, mask), torch.tensor([0.0, 1.0, 0.0, 1.0]))
    assert mo.l0_sum(acts, None).item() == 4 and mo.l0_sum(acts, mask).item() == 2
    # the sum runs over every entry (the -1 included), the count over the positive ones
    assert mo.mean_feature_act(acts).item() == pytest.approx(6.0 / 4.0)
    th = mo.sparsity_thresholds(torch.tensor([0.5, 0.05, 1e-3, 5e-6, 5e-7, 0.0]))
    assert th == {"sparsity/above_1e-1": 1, "sparsity/above_1e-2": 2, "sparsity/below_1e-5": 3,
                  "sparsity/below_1e-6": 2, "sparsity/below_1e-7": 1}


def test_frequency_against_a_scalar_loop(mo):
    g = torch.Generator().manual_seed(0)
    acts = torch.randn(37, 23, generator=g) * (torch.rand(37, 23, generator=g) > 0.7)
    mask = (torch.rand(37, generator=g) > 0.3).float()
    want = np.zeros(23)
    for b in range(37):
        for f in range(23):
            if mask[b] > 0 and acts[b, f] > 0:
                want[f] += 1
    assert np.array_equal(mo.act_freq_scores(acts, mask).numpy(), want)
    assert mo.l0_sum(acts, mask).item() == want.sum()


def test_explained_variance_closed_forms(mo):
    g = torch.Generator().manual_seed(1)
    label = torch.randn(50, 12, generator=g, dtype=torch.float64) + 3.0
    mask = (torch.rand(50, generator=g) > 0.4).double()
    for m in (None, mask):
        ev, legacy = mo.explained_variance(label, label.clone(), m)
        assert ev.item() == 1.0 and legacy.item() == 1.0
        mean = label.mean(0) if m is None else (label * m[:, None]).sum(0) / m.sum()
        ev, legacy = mo.explained_variance(label, mean.expand_as(label), m)
        assert abs(ev.item()) < 1e-12 and abs(legacy.item()) < 1e-12       # residual = deviation from the mean, token by token
        for c in (0.25, 0.5, 2.0):
            recon = mean + c * (label - mean)
            ev, legacy = mo.explained_variance(label, recon, m)
            assert ev.item() == pytest.approx(1 - (1 - c) ** 2, abs=1e-12)
            assert legacy.item() == pytest.approx(1 - (1 - c) ** 2, abs=1e-12)
    # the two forms differ when the error is uneven across tokens: pooled ratio vs mean of ratios
    label = torch.tensor([[1.0, 0.0], [-1.0, 0.0], [0.0, 3.0], [0.0, -3.0]], dtype=torch.float64)   # mean 0; variances 1,1,9,9
    recon = label.clone(); recon[0, 0] = 0.0                                                          # squared error 1 on token 0
    ev, legacy = mo.explained_variance(label, recon, None)
    assert ev.item() == pytest.approx(1 - (1 / 4) / (20 / 4)) and legacy.item() == pytest.approx(1 - (1 / 1) / 4)


def test_explained_variance_and_l2_against_fp64_loops(mo):
    g = torch.Generator().manual_seed(2)
    B, d = 19, 7
    label = torch.randn(B, d, generator=g, dtype=torch.float64)
    recon = label + 0.3 * torch.randn(B, d, generator=g, dtype=torch.float64)
    mask = (torch.rand(B, generator=g) > 0.3).double()
    n = mask.sum().item()
    mean = [sum(mask[b].item() * label[b, j].item() for b in range(B)) / n for j in range(d)]
    se = [sum((recon[b, j].item() - label[b, j].item()) ** 2 for j in range(d)) for b in range(B)]
    var = [sum((label[b, j].item() - mean[j]) ** 2 for j in range(d)) for b in range(B)]
    nrm = [math.sqrt(sum(label[b, j].item() ** 2 for j in range(d))) for b in range(B)]
    w = [mask[b].item() for b in range(B)]
    ev, legacy = mo.explained_variance(label, recon, mask)
    assert ev.item() == pytest.approx(1 - (sum(w[b] * se[b] for b in range(B)) / n) / (sum(w[b] * var[b] for b in range(B)) / n), rel=1e-12)
    assert legacy.item() == pytest.approx(sum(w[b] * (1 - se[b] / var[b]) for b in range(B)) / n, rel=1e-12)
    err, ratio = mo.l2_norm_error(label, recon, mask)
    e = sum(w[b] * math.sqrt(se[b]) for b in range(B)) / n
    assert err.item() == pytest.approx(e, rel=1e-12)
    assert ratio.item() == pytest.approx(e / (sum(w[b] * nrm[b] for b in range(B)) / n), rel=1e-12)


def test_l2_norm_error_hand_cases(mo):
    label = torch.tensor([[3.0, 4.0], [0.0, 5.0]])
    err, ratio = mo.l2_norm_error(label, torch.zeros_like(label), None)
    assert err.item() == 5.0 and ratio.item() == 1.0                     # recon = 0: the error is the label norm
    recon = torch.tensor([[0.0, 0.0], [0.0, 5.0]])
    err, ratio = mo.l2_norm_error(label, recon, None)
    assert err.item() == 2.5 and ratio.item() == 0.5
    err, ratio = mo.l2_norm_error(label, recon, torch.tensor([0.0, 1.0]))
    assert err.item() == 0.0 and ratio.item() == 0.0


def test_step_metrics_window(mo):
    """Two steps then compute(): means over steps / tokens as Record defines them, then a clean restart."""
    sm = mo.StepMetrics()
    a1 = torch.tensor([[1.0, 0.0], [0.0, 0.0]]); a2 = torch.tensor([[1.0, 2.0], [3.0, 0.0]])
    lab = torch.tensor([[1.0, 1.0], [-1.0, -1.0]])
    for acts, rec, loss in ((a1, lab * 0.5, 2.0), (a2, lab, 4.0)):
        sm.update(feature_acts=acts, label=lab, reconstructed=rec, mask=None, n_tokens=2, loss=torch.tensor(loss),
                  l_rec=torch.tensor(loss), grad_norm_before_clipping=loss, grad_norm=loss / 2)
    out = sm.compute()
    # firing frequency: feature 0 on 3 of 4 tokens, feature 1 on 1 of 4
    assert out["sparsity/above_1e-1"] == 2 and out["sparsity/below_1e-5"] == 0
    assert out["metrics/l0"] == pytest.approx((1 + 3) / 4)
    assert out["metrics/mean_feature_act"] == pytest.approx((1.0 + 2.0) / 2)
    assert out["losses/overall_loss"] == 3.0 and out["losses/mse_loss"] == 3.0
    assert out["metrics/explained_variance"] == pytest.approx((0.75 + 1.0) / 2)
    assert out["metrics/gradient_norm_before_clipping"] == 4.0 and out["metrics/gradient_norm_per_param"] == 2.0
    assert sm.loss.value is None


def test_product_dense_metrics_match_the_oracle_on_cpu(pkg, mo):
    """The metric classes of the package, on a context without a sparse code (generic dense route), CPU tensors."""
    from lm_saes_amd import metrics as pm

    g = torch.Generator().manual_seed(3)
    B, F, d = 33, 40, 9

    class _Model:
        cfg = None
        def parameters(self):
            return []

    ms = [pm.FrequencyMetric(_Model()), pm.LossMetric(_Model()), pm.MeanFeatureActMetric(_Model()),
          pm.ExplainedVarianceMetric(_Model()), pm.L0Metric(_Model()), pm.L2NormErrorMetric(_Model())]
    sm = mo.StepMetrics()
    for step in range(3):
        acts = torch.randn(B, F, generator=g).relu() * (torch.rand(B, F, generator=g) > 0.8)
        label = torch.randn(B, d, generator=g) + 1.0
        recon = label + 0.2 * torch.randn(B, d, generator=g)
        mask = (torch.rand(B, generator=g) > 0.25).float() if step != 1 else None
        n_tokens = B if mask is None else int(mask.sum())
        loss = torch.tensor(1.0 + step)
        ctx = {"feature_acts": acts, "label": label, "reconstructed": recon, "mask": mask, "n_tokens": n_tokens,
               "loss": loss, "l_rec": loss * 0.5, "l_s": None, "l_p": None, "l_aux": loss * 0.25}
        for m in ms:
            ctx.update(m.update(ctx))
        sm.update(feature_acts=acts, label=label, reconstructed=recon, mask=mask, n_tokens=n_tokens, loss=loss,
                  l_rec=loss * 0.5, l_aux=loss * 0.25)
    got = {}
    for m in ms:
        got.update(m.compute())
    want = sm.compute()
    assert set(want) <= set(got)
    for k, v in want.items():
        assert got[k] == pytest.approx(v, rel=1e-6), k


def test_product_record_keeps_device_values(pkg):
    from lm_saes_amd.metrics import Record

    r = Record("max")
    r.update(torch.tensor(2.0)); r.update(torch.tensor(5.0)); r.update(torch.tensor(3.0))
    assert r.compute().item() == 5.0
    r = Record("min")
    r.update(4.0); r.update(torch.tensor(1.0))
    assert float(r.compute()) == 1.0
    with pytest.raises(ValueError):
        Record("median")
