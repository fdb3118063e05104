"""Pins the CPU oracle: the reference's known-answer vectors, closed forms, brute force in fp64.

A check here is chosen so that a plausible slip in the oracle (dropped term, wrong sign or index,
transposed operand, wrong tie rule) fails it; none of them re-types the oracle's own formula.
"""

import json
import math
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_kats.json")))


def fixture_model(oracle, **kw):
    f = KATS["sae_fixture"]
    m = oracle.SAEOracle(f["d_model"], f["d_sae"], act_fn=kw.pop("act_fn", "topk"), top_k=f["top_k"], **kw)
    with torch.no_grad():
        m.W_E.copy_(torch.tensor(f["W_E"]))
        m.b_E.copy_(torch.tensor(f["b_E"]))
        m.W_D.copy_(torch.tensor(f["W_D"]))
        m.b_D.copy_(torch.tensor(f["b_D"]))
    return m


# ---- the reference's own KATs ----------------------------------------------------------------

def test_topk_activation_kat(oracle):
    k = KATS["topk_activation"]
    m = fixture_model(oracle)
    m.current_k = k["k"]
    out = m.activation_function(torch.tensor(k["input"]))
    assert torch.allclose(out, torch.tensor(k["expected"]), atol=k["atol"], rtol=1e-5)


def test_set_norm_kat(oracle):
    k = KATS["set_norm"]
    m = fixture_model(oracle)
    for value, exact in k["decoder_steps"]:
        m.set_decoder_to_fixed_norm(value, force_exact=exact)
        n = m.decoder_norm()
        if exact:
            assert torch.allclose(n, torch.full_like(n, value), atol=k["atol"], rtol=1e-5)
        else:
            assert torch.all(n <= value + k["atol"])
    for value in k["encoder_steps"]:
        m.set_encoder_to_fixed_norm(value)
        n = m.encoder_norm()
        assert torch.allclose(n, torch.full_like(n, value), atol=k["atol"], rtol=1e-5)
    m.transform_to_unit_decoder_norm()
    assert torch.allclose(m.decoder_norm(), torch.ones(4), atol=1e-4)


def test_norms_closed_form(oracle):
    m = fixture_model(oracle)
    # rows of W_D: (1,5) (2,6) (3,7) (4,8); columns of W_E: (1,5) (2,6) (3,7) (4,8)
    want = torch.tensor([26.0, 40.0, 58.0, 80.0]).sqrt()
    assert torch.allclose(m.decoder_norm(), want)
    assert torch.allclose(m.encoder_norm(), want)
    assert torch.allclose(m.decoder_bias_norm(), torch.tensor([math.sqrt(5.0)]))
    assert m.decoder_norm(keepdim=True).shape == (4, 1) and m.encoder_norm(keepdim=True).shape == (1, 4)


def test_compute_norm_factor_kat(oracle):
    k = KATS["compute_norm_factor"]
    x = torch.tensor(k["x"])
    m = fixture_model(oracle, norm_activation="token-wise")
    assert torch.allclose(m.compute_norm_factor(x, "in"), torch.tensor(k["token_wise"]), atol=k["atol"])
    m.norm_activation = "batch-wise"
    assert torch.allclose(m.compute_norm_factor(x, "in"), torch.tensor(k["batch_wise"]), atol=k["atol"])
    m.norm_activation = "dataset-wise"
    m.dataset_average_activation_norm = k["dataset_norms"]
    assert abs(m.compute_norm_factor(x, "in").item() - k["dataset_wise_in"]) < k["atol"]
    assert abs(m.compute_norm_factor(x, "out").item() - k["dataset_wise_out"]) < k["atol"]
    m.norm_activation = "inference"
    assert m.compute_norm_factor(x, "in").item() == 1.0
    out = fixture_model(oracle, norm_activation="token-wise").normalize_activations({"in": x, "tokens": torch.zeros(2)})
    assert torch.allclose(out["in"].norm(dim=-1), torch.full((2,), math.sqrt(2.0)))


# ---- forward / loss against hand arithmetic and fp64 brute force -----------------------------

def test_forward_hand_computed(oracle):
    """x = (1, 1) through the fixture, relu, no norm scaling: every number below is hand arithmetic.
    h = x W_E + b_E = (6+3, 8+2, 10+3, 12+4) = (9, 10, 13, 16); recon = h W_D + b_D."""
    m = fixture_model(oracle, act_fn="relu", sparsity_include_decoder_norm=False)
    x = torch.tensor([[1.0, 1.0]])
    fa, hp = m.encode(x, return_hidden_pre=True)
    assert torch.equal(hp, torch.tensor([[9.0, 10.0, 13.0, 16.0]])) and torch.equal(fa, hp)
    # recon_0 = 9*1 + 10*2 + 13*3 + 16*4 + 1 = 133 ; recon_1 = 9*5 + 10*6 + 13*7 + 16*8 + 2 = 326
    assert torch.equal(m.decode(fa), torch.tensor([[133.0, 326.0]]))
    ctx = m.compute_loss({"in": x, "out": x, "tokens": torch.zeros(1)})
    assert ctx["l_rec"].item() == 132.0 ** 2 + 325.0 ** 2  # sum over d_model, mean over the single token
    # top-2 of h keeps (13, 16): recon = 13*(3,7) + 16*(4,8) + (1,2) = (104, 221)
    mt = fixture_model(oracle, act_fn="topk", sparsity_include_decoder_norm=False)
    assert torch.equal(mt.forward(x), torch.tensor([[104.0, 221.0]]))


def test_decoder_norm_scaling_changes_selection(oracle):
    """With sparsity_include_decoder_norm the ranking is by h * ||W_D row||, the output by h."""
    m = fixture_model(oracle, act_fn="topk", sparsity_include_decoder_norm=True)
    with torch.no_grad():
        m.W_D.copy_(torch.tensor([[10.0, 0.0], [0.0, 10.0], [0.1, 0.0], [0.0, 0.1]]))  # norms 10, 10, .1, .1
    fa, hp = m.encode(torch.tensor([[1.0, 1.0]]), return_hidden_pre=True)
    # h = (9, 10, 13, 16); h*n = (90, 100, 1.3, 1.6) -> features 0 and 1 win although 2 and 3 have larger h
    assert torch.allclose(fa, torch.tensor([[9.0, 10.0, 0.0, 0.0]]), atol=1e-5)
    assert torch.allclose(hp, torch.tensor([[9.0, 10.0, 13.0, 16.0]]), atol=1e-5)


def np_sae_loss(x, y, W_E, b_E, W_D, b_D, k, mask=None, include_norm=True):
    """fp64 loops: per-token TopK SAE reconstruction loss."""
    B, F = x.shape[0], W_E.shape[1]
    n = np.sqrt((W_D ** 2).sum(1))
    tot, wsum = 0.0, 0.0
    recon = np.zeros_like(y)
    for b in range(B):
        h = x[b] @ W_E + b_E
        key = h * n if include_norm else h
        order = sorted(range(F), key=lambda f: (-key[f], f))[:k]
        acts = np.zeros(F)
        for f in order:
            if key[f] > 0:
                acts[f] = h[f]
        recon[b] = acts @ W_D + b_D
        w = 1.0 if mask is None else mask[b]
        tot += w * ((recon[b] - y[b]) ** 2).sum()
        wsum += w
    return tot / wsum, recon


@pytest.mark.parametrize("include_norm", [False, True])
@pytest.mark.parametrize("masked", [False, True])
def test_topk_loss_vs_fp64_brute_force(oracle, include_norm, masked):
    rng = np.random.default_rng(0)
    B, d, F, k = 12, 6, 20, 4
    x = rng.normal(size=(B, d)); y = rng.normal(size=(B, d))
    W_E = rng.normal(size=(d, F)); b_E = 0.1 * rng.normal(size=F)
    W_D = rng.normal(size=(F, d)); b_D = rng.normal(size=d)
    mask = (rng.random(B) > 0.3).astype(np.float64) if masked else None
    want, recon = np_sae_loss(x, y, W_E, b_E, W_D, b_D, k, mask, include_norm)
    m = oracle.SAEOracle(d, F, act_fn="topk", top_k=k, sparsity_include_decoder_norm=include_norm, dtype=torch.float64)
    with torch.no_grad():
        m.W_E.copy_(torch.tensor(W_E)); m.b_E.copy_(torch.tensor(b_E))
        m.W_D.copy_(torch.tensor(W_D)); m.b_D.copy_(torch.tensor(b_D))
    batch = {"in": torch.tensor(x), "out": torch.tensor(y), "tokens": torch.zeros(B)}
    if masked:
        batch["mask"] = torch.tensor(mask)
    ctx = m.compute_loss(batch)
    assert abs(ctx["loss"].item() - want) < 1e-10 * abs(want)
    assert np.allclose(ctx["reconstructed"].detach().numpy(), recon, atol=1e-10)
    assert ctx["n_tokens"] == (int(mask.sum()) if masked else B)
    assert (ctx["feature_acts"] != 0).sum(-1).max().item() <= k


def test_gradients_vs_finite_differences(oracle):
    torch.manual_seed(0)
    d, F, k, B = 5, 12, 3, 7
    m = oracle.SAEOracle(d, F, act_fn="topk", top_k=k, dtype=torch.float64)
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(torch.randn_like(p))
    x = torch.randn(B, d, dtype=torch.float64)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B)}
    m.compute_loss(batch)["loss"].backward()
    eps = 1e-6
    for name in ("W_E", "b_E", "W_D", "b_D"):
        p = getattr(m, name)
        flat = p.data.view(-1)
        for i in (0, flat.numel() // 2, flat.numel() - 1):
            old = flat[i].item()
            flat[i] = old + eps; lp = m.compute_loss(batch)["loss"].item()
            flat[i] = old - eps; lm = m.compute_loss(batch)["loss"].item()
            flat[i] = old
            fd = (lp - lm) / (2 * eps)
            assert abs(fd - p.grad.view(-1)[i].item()) < 1e-5 * max(1.0, abs(fd)), (name, i)


# ---- selection rules ----------------------------------------------------------------------------

def test_topk_tie_rule_and_invariants(oracle):
    x = torch.tensor([[1.0, 2.0, 2.0, 2.0, 0.5, 2.0]])
    out = oracle.topk(x, k=2, dim=-1)
    assert torch.equal(out, torch.tensor([[0.0, 2.0, 2.0, 0.0, 0.0, 0.0]]))  # lowest indices among the tie
    g = torch.Generator().manual_seed(1)
    y = torch.randn(20, 300, generator=g)
    for k in (1, 7, 300):
        o = oracle.topk(y, k=k, dim=-1)
        assert ((o != 0).sum(-1) <= k).all()
        kept_min = torch.where(o != 0, y, torch.full_like(y, float("inf"))).min(-1).values
        drop_max = torch.where(o == 0, y, torch.full_like(y, -float("inf"))).max(-1).values
        assert (kept_min >= drop_max).all() or k == 300
        assert torch.equal(oracle.topk(o, k=k, dim=-1), o)  # idempotent
        # tie-free rows: same set as torch.topk
        want = torch.zeros_like(y).scatter(-1, torch.topk(y, k, dim=-1).indices, 1.0).bool()
        assert torch.equal(o != 0, want & (y != 0))
    _, thr = oracle.topk(y, k=5, dim=-1, return_threshold=True)
    assert torch.equal(thr, torch.topk(y, 5, dim=-1).values[:, -1])


def test_batchtopk_vs_global_sort(oracle):
    rng = np.random.default_rng(2)
    B, F, k = 9, 40, 3
    h = rng.normal(size=(B, F)).astype(np.float32)
    m = oracle.SAEOracle(4, F, act_fn="batchtopk", top_k=k, sparsity_include_decoder_norm=False)
    out = m.activation_function(torch.tensor(h)).numpy()
    r = np.where(h > 0, h, 0.0).reshape(-1)
    order = sorted(range(B * F), key=lambda i: (-r[i], i))[: k * B]
    want = np.zeros(B * F, dtype=np.float32)
    want[order] = r[order]
    assert np.array_equal(out.reshape(-1), want)
    assert (out != 0).sum() == k * B  # enough positives exist
    # 3-D input is flattened over (batch, context) and restored
    out3 = m.activation_function(torch.tensor(h).reshape(3, 3, F))
    assert out3.shape == (3, 3, F) and np.array_equal(out3.reshape(B, F).numpy(), out)


# ---- JumpReLU -----------------------------------------------------------------------------------

def test_jumprelu_forward_backward_vs_numpy(oracle):
    rng = np.random.default_rng(3)
    B, F, eps = 50, 16, 0.5
    x = rng.normal(size=(B, F))
    logt = rng.normal(size=F) * 0.3 - 0.5
    g = rng.normal(size=(B, F))
    theta = np.exp(logt)
    fwd = np.where(x > theta, x, 0.0)
    gx = np.where(x > theta, g, 0.0)
    win = (np.abs(x - theta) < eps / 2) & (x > 0)
    gtheta = (np.where(win, -theta / eps, 0.0) * g).sum(0)
    glog = gtheta * theta
    act = oracle.JumpReLU(eps, (F,), dtype=torch.float64)
    with torch.no_grad():
        act.log_jumprelu_threshold.copy_(torch.tensor(logt))
    xt = torch.tensor(x, requires_grad=True)
    out = act(xt)
    out.backward(torch.tensor(g))
    assert np.allclose(out.detach().numpy(), fwd) and np.allclose(xt.grad.numpy(), gx)
    assert np.allclose(act.log_jumprelu_threshold.grad.numpy(), glog)
    assert win.any() and (~win).any()


def test_jumprelu_special_cases(oracle):
    act = oracle.JumpReLU(0.1, (3,), dtype=torch.float64)
    with torch.no_grad():
        act.log_jumprelu_threshold.fill_(0.0)  # theta = 1
    x = torch.tensor([[1.0, 1.0 + 1e-9, 5.0], [-3.0, 0.2, 0.96]], dtype=torch.float64, requires_grad=True)
    out = act(x)
    assert torch.equal(out.detach(), torch.tensor([[0.0, 1.0 + 1e-9, 5.0], [0.0, 0.0, 0.0]], dtype=torch.float64))  # strict >
    out.sum().backward()
    # window |x - 1| < 0.05: columns 0 and 1 of row 0 and 0.96 of row 1; -theta/eps = -10 each, times theta = 1
    assert torch.allclose(act.log_jumprelu_threshold.grad, torch.tensor([-10.0, -10.0, -10.0], dtype=torch.float64))
    # CLT-style threshold of shape (L, F): the gradient keeps both trailing dims
    act2 = oracle.JumpReLU(2.0, (2, 3), dims_to_keep_in_bwd=(-2, -1), dtype=torch.float64)
    with torch.no_grad():
        act2.log_jumprelu_threshold.fill_(0.0)
    act2(torch.ones(5, 2, 3, dtype=torch.float64) * 1.5).sum().backward()
    assert act2.log_jumprelu_threshold.grad.shape == (2, 3)
    assert torch.allclose(act2.log_jumprelu_threshold.grad, torch.full((2, 3), -2.5, dtype=torch.float64))


# ---- losses -------------------------------------------------------------------------------------

def _dense_model(oracle, act_fn, F=10, d=4, **kw):
    torch.manual_seed(5)
    m = oracle.SAEOracle(d, F, act_fn=act_fn, top_k=3, dtype=torch.float64, **kw)
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(torch.randn_like(p) * 0.5)
    return m


@pytest.mark.parametrize("kind", ["power", "tanh", "tanh-quad"])
def test_sparsity_losses_vs_numpy(oracle, kind):
    m = _dense_model(oracle, "relu")
    B = 6
    x = torch.randn(B, 4, dtype=torch.float64)
    ctx = m.compute_loss({"in": x, "out": x, "tokens": torch.zeros(B)}, sparsity_loss_type=kind, l1_coefficient=0.7,
                         tanh_stretch_coefficient=3.0, frequency_scale=0.05, p=1)
    f = ctx["feature_acts"].detach().numpy()
    n = np.sqrt((m.W_D.detach().numpy() ** 2).sum(1))
    a = f * n
    if kind == "power":
        want = 0.7 * np.abs(a).sum(1).mean()
    elif kind == "tanh":
        want = 0.7 * np.tanh(3.0 * a).sum(1).mean()
    else:
        q = np.tanh(3.0 * a).mean(0)
        want = 0.7 * (q * (1 + q / 0.05)).sum()
    got = (ctx["loss"] - ctx["l_rec"]).item()
    assert abs(got - want) < 1e-10 * max(1.0, abs(want))


def test_lp_loss_vs_numpy(oracle):
    m = _dense_model(oracle, "jumprelu", jumprelu_threshold_window=0.3)
    with torch.no_grad():
        m.activation_function.log_jumprelu_threshold.copy_(torch.linspace(-1, 0.5, 10, dtype=torch.float64))
    x = torch.randn(5, 4, dtype=torch.float64)
    ctx = m.compute_loss({"in": x, "out": x, "tokens": torch.zeros(5)}, lp_coefficient=0.2)
    theta = np.exp(np.linspace(-1, 0.5, 10))
    hp = ctx["hidden_pre"].detach().numpy()
    n = np.sqrt((m.W_D.detach().numpy() ** 2).sum(1))
    want = 0.2 * (np.maximum(theta - hp, 0) * n).sum(1).mean()
    assert abs(ctx["l_p"].item() - want) < 1e-10
    assert abs(ctx["loss"].item() - ctx["l_rec"].item() - want) < 1e-10


def test_auxk_vs_numpy_and_special_cases(oracle):
    F, d, B, k = 12, 4, 8, 2
    m = _dense_model(oracle, "topk", F=F, d=d, sparsity_include_decoder_norm=False)
    m.current_k = k
    x = torch.randn(B, d, dtype=torch.float64)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B)}
    stats = oracle.DeadStatistics(F, dead_threshold=B)  # silent in this batch => dead
    ctx = m.compute_loss(batch, auxk_coefficient=0.25, k_aux=3, update_dead_statistics=stats.update)
    f = ctx["feature_acts"].detach().numpy()
    fired = (f.sum(0) > 0)
    assert np.array_equal(stats.is_dead.numpy(), ~fired)
    assert np.array_equal(stats.tokens_since_last_activation.numpy(), np.where(fired, 0, B))
    hp = ctx["hidden_pre"].detach().numpy()
    W_D = m.W_D.detach().numpy()
    e = (x - ctx["reconstructed"]).detach().numpy()
    kk = min(3, int((~fired).sum()))
    tot = 0.0
    for b in range(B):
        hd = np.where(~fired, hp[b], 0.0)
        order = sorted(range(F), key=lambda j: (-max(hd[j], 0.0), j))[:kk]
        acts = np.zeros(F)
        for j in order:
            if hd[j] > 0:
                acts[j] = hd[j]
        tot += ((e[b] - acts @ W_D) ** 2).sum()
    want = 0.25 * tot / B
    assert kk > 0 and abs(ctx["l_aux"].item() - want) < 1e-10 * max(1.0, want)
    assert m.current_k == k  # restored
    # the residual carries gradient: d l_aux / d b_D is not zero
    m.zero_grad(); ctx["l_aux"].backward(retain_graph=True)
    assert m.b_D.grad.abs().max() > 0
    # no dead feature -> l_aux == 0
    alive = oracle.DeadStatistics(F, dead_threshold=10 ** 9)
    ctx2 = m.compute_loss(batch, auxk_coefficient=0.25, k_aux=3, update_dead_statistics=alive.update)
    assert ctx2["l_aux"].item() == 0.0 and ctx2["loss"].item() == ctx2["l_rec"].item()


def test_auxk_with_decoder_norm_scale_vs_numpy(oracle):
    """The aux-k branch with `sparsity_include_decoder_norm=True` (models/sparse_dictionary.py:958-972): the dead features'
    keys are hidden_pre * n (n = decoder row norms, spread here so that the ranking by h n differs from the ranking by h),
    the kept values are divided by n again, so the aux reconstruction is built from hidden_pre itself.  Scalar loops."""
    F, d, B, k = 12, 4, 9, 2
    m = _dense_model(oracle, "topk", F=F, d=d, sparsity_include_decoder_norm=True)
    with torch.no_grad():
        m.W_D.mul_(torch.linspace(0.2, 3.0, F, dtype=torch.float64)[:, None])
    m.current_k = k
    x = torch.randn(B, d, dtype=torch.float64)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B)}
    stats = oracle.DeadStatistics(F, dead_threshold=B)
    ctx = m.compute_loss(batch, auxk_coefficient=0.5, k_aux=3, update_dead_statistics=stats.update)
    f = ctx["feature_acts"].detach().numpy()
    fired = f.sum(0) > 0
    hp = ctx["hidden_pre"].detach().numpy()
    W_D = m.W_D.detach().numpy()
    n = np.sqrt((W_D ** 2).sum(1))
    e = (x - ctx["reconstructed"]).detach().numpy()
    kk = min(3, int((~fired).sum()))
    tot, by_h_differs = 0.0, False
    for b in range(B):
        key = np.where(~fired, hp[b] * n, 0.0)
        order = sorted(range(F), key=lambda j: (-max(key[j], 0.0), j))[:kk]
        plain = sorted(range(F), key=lambda j: (-max(np.where(~fired, hp[b], 0.0)[j], 0.0), j))[:kk]
        by_h_differs |= set(j for j in order if key[j] > 0) != set(j for j in plain if hp[b][j] > 0 and not fired[j])
        acts = np.zeros(F)
        for j in order:
            if key[j] > 0:
                acts[j] = key[j] / n[j]
        tot += ((e[b] - acts @ W_D) ** 2).sum()
    want = 0.5 * tot / B
    assert kk > 0 and by_h_differs          # the norm scale changes which dead features are picked
    assert abs(ctx["l_aux"].item() - want) < 1e-10 * max(1.0, want)
    assert abs(ctx["loss"].item() - ctx["l_rec"].item() - want) < 1e-10 * max(1.0, want)


def test_dead_statistics_accumulate(oracle):
    st = oracle.DeadStatistics(3, dead_threshold=5)
    a = torch.tensor([[1.0, 0.0, 0.0], [0.0, 0.0, 0.0]])
    st.update(a, None, 1)
    assert st.tokens_since_last_activation.tolist() == [0, 2, 2] and st.is_dead.tolist() == [False, False, False]
    st.update(a, torch.tensor([1.0, 0.0]), 1)  # one valid token
    assert st.tokens_since_last_activation.tolist() == [0, 3, 3]
    st.update(torch.tensor([[0.0, 2.0, 0.0], [0.0, 0.0, 0.0]]), None, 1)
    assert st.tokens_since_last_activation.tolist() == [2, 0, 5] and st.is_dead.tolist() == [False, False, True]


# ---- trainer / optimiser side -------------------------------------------------------------------

def test_k_schedule_hand_table(oracle):
    kw = dict(top_k=10, initial_k=100.0, k_cold_booting_steps=2, k_warmup_steps=9)
    ks = [oracle.k_schedule(s, **kw) for s in (0, 1, 2, 5, 11, 12, 50)]
    assert ks == [100, 100, 100, 70, 10, 10, 10]
    ke = oracle.k_schedule(5, k_schedule_type="exponential", k_exponential_factor=3.0, **kw)
    want = 100 - 90 * (1 - math.exp(-1.0)) / (1 - math.exp(-3.0))
    assert ke == math.ceil(want) and 10 < ke < 70
    assert oracle.l1_warmup(5, 10, 8e-5) == 4e-5 and oracle.l1_warmup(50, 10, 8e-5) == 8e-5
    assert oracle.l1_warmup(5, 10, None) == 1.0


def test_grad_norm_hand_case(oracle):
    g = [torch.tensor([0.0, 3.0, 4.0])]
    assert abs(oracle.compute_grad_norm(g).item() - 5 / math.sqrt(2)) < 1e-6
    g2 = [torch.tensor([3.0, 0.0]), torch.tensor([[4.0], [0.0]])]
    assert abs(oracle.compute_grad_norm(g2).item() - 5 / math.sqrt(2)) < 1e-6
    gs = [torch.tensor([0.0, 3.0, 4.0])]
    oracle.clip_grad_norm(gs, max_norm=1.0)
    assert torch.allclose(gs[0], torch.tensor([0.0, 3.0, 4.0]) / (5 / math.sqrt(2) + 1e-6))
    gs = [torch.tensor([0.0, 3.0, 4.0])]
    oracle.clip_grad_norm(gs, max_norm=100.0)
    assert torch.equal(gs[0], torch.tensor([0.0, 3.0, 4.0]))


def test_sparse_adam_vs_scalar_loop(oracle):
    rng = np.random.default_rng(7)
    n, lr, b1, b2, eps = 9, 0.01, 0.9, 0.999, 1e-8
    p = torch.tensor(rng.normal(size=n)); st = oracle.SparseAdamState(p)
    pr, m, v, t = p.numpy().copy(), np.zeros(n), np.zeros(n), 0
    for step in range(4):
        g = rng.normal(size=n) * (rng.random(n) > 0.4)
        if step == 2:
            g[:] = 0.0  # all-zero gradient: the whole parameter is skipped, the step counter too
        oracle.sparse_adam_step(p, torch.tensor(g), st, lr=lr, betas=(b1, b2), eps=eps)
        if g.any():
            t += 1
            for i in range(n):
                m[i] *= b1; v[i] *= b2
                if g[i] != 0:
                    m[i] += (1 - b1) * g[i]; v[i] += (1 - b2) * g[i] ** 2
                    pr[i] -= lr * math.sqrt(1 - b2 ** t) / (1 - b1 ** t) * m[i] / (math.sqrt(v[i]) + eps)
    assert st.step == t == 3
    assert np.allclose(p.numpy(), pr, atol=1e-12) and np.allclose(st.exp_avg.numpy(), m) and np.allclose(st.exp_avg_sq.numpy(), v)


def test_adam_first_step_closed_form(oracle):
    m = fixture_model(oracle, act_fn="relu", sparsity_include_decoder_norm=False)
    before = {n: p.detach().clone() for n, p in m.named_parameters()}
    opt = oracle.make_adam(m, lr=1e-3)
    x = torch.tensor([[1.0, 1.0]])
    oracle.train_step(m, opt, {"in": x, "out": x, "tokens": torch.zeros(1)})
    for n, p in m.named_parameters():
        moved = (p.detach() - before[n]).abs()
        assert torch.allclose(moved, torch.full_like(moved, 1e-3), rtol=1e-4), n  # bias-corrected: -lr * sign(g)
        assert p.grad is None  # zero_grad(set_to_none)


def test_apply_token_mask(oracle):
    t = torch.arange(12.0).reshape(3, 4)
    assert torch.equal(oracle.apply_token_mask(t, 1, None, "sum"), t.sum(0))
    assert torch.equal(oracle.apply_token_mask(t, 1, None, "mean"), t.mean(0))
    mask = torch.tensor([1.0, 0.0, 1.0])
    assert torch.equal(oracle.apply_token_mask(t, 1, mask, "mean"), (t[0] + t[2]) / 2)
    t3 = torch.arange(24.0).reshape(2, 3, 4)
    m2 = torch.tensor([[1.0, 1.0, 0.0], [0.0, 0.0, 1.0]])
    assert torch.equal(oracle.apply_token_mask(t3, 2, m2, "sum"), t3[0, 0] + t3[0, 1] + t3[1, 2])
    with pytest.raises(AssertionError):
        oracle.apply_token_mask(t, 1, torch.ones(4), "sum")
