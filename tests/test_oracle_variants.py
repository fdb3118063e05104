"""Pins the crosscoder / cross-layer transcoder / Lorsa oracles.

Crosscoder: the reference's own known answers.  CLT and Lorsa: scalar-loop brute force in fp64,
reductions to simpler models (L = 1 -> SAE; one feature per key head width -> ordinary multi-head
attention through torch's library routine) and closed forms (2-D rotation for rotary).
None of the checks re-types the vectorised formula of the oracle.
"""

import json
import math
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_kats.json")))


@pytest.fixture(scope="module")
def vo(oracle):
    import importlib

    return importlib.import_module("oracle.variants_oracle")


def crosscoder_fixture(vo, **kw):
    f = KATS["crosscoder_fixture"]
    m = vo.CrosscoderOracle(2, 2, 4, act_fn=kw.pop("act_fn", "relu"), top_k=2, **kw)
    with torch.no_grad():
        for name in ("W_E", "b_E", "W_D", "b_D"):
            getattr(m, name).copy_(torch.tensor(f[name]))
    return m


# ---- crosscoder: reference KATs -------------------------------------------------------------------

def test_crosscoder_encode_kat(vo):
    k = KATS["crosscoder_encode"]
    m = crosscoder_fixture(vo)
    acts, hidden_pre = m.encode(torch.tensor(k["x"]), return_hidden_pre=True)
    assert torch.allclose(hidden_pre, torch.tensor(k["expected_hidden_pre"]), atol=k["atol"])
    assert torch.all(acts > 0)
    # relu(h * n) / n == h for positive h
    assert torch.allclose(acts, hidden_pre, atol=1e-6)


def test_crosscoder_decode_kat(vo):
    k = KATS["crosscoder_decode"]
    m = crosscoder_fixture(vo)
    assert torch.allclose(m.decode(torch.tensor(k["feature_acts"])), torch.tensor(k["expected"]), atol=k["atol"])


def test_crosscoder_norms_kat(vo):
    k = KATS["crosscoder_norms"]
    m = crosscoder_fixture(vo)
    assert torch.allclose(m.encoder_norm(), torch.tensor(k["encoder_norm"]), atol=k["atol"])
    assert torch.allclose(m.decoder_norm(), torch.tensor(k["decoder_norm"]), atol=k["atol"])
    # tests/unit/test_crosscoder.py:277-293
    assert torch.allclose(m.decoder_bias_norm(), torch.tensor([[0.224], [0.224]]), atol=1e-3)


def test_crosscoder_topk_per_head_brute_force(vo):
    """The selection differs per head because each head scales the shared pre-activation by its own
    decoder norms: brute force picks, per (token, head), the k largest of h * n_head."""
    H, d, F, B, k = 3, 5, 12, 7, 4
    m = vo.init_uniform_(vo.CrosscoderOracle(H, d, F, act_fn="topk", top_k=k, dtype=torch.float64), seed=1)
    x = torch.randn(B, H, d, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    acts, hp = m.encode(x, return_hidden_pre=True)
    W_E, b_E, W_D = m.W_E.detach().numpy(), m.b_E.detach().numpy(), m.W_D.detach().numpy()
    xn = x.numpy()
    for b in range(B):
        acc = np.zeros(F)
        for h in range(H):
            for f in range(F):
                acc[f] += sum(xn[b, h, j] * W_E[h, j, f] for j in range(d)) + b_E[h, f]
        for h in range(H):
            assert np.allclose(hp[b, h].detach().numpy(), acc, atol=1e-12)
            n = np.sqrt((W_D[h] ** 2).sum(-1))
            scaled = np.maximum(acc * n, 0.0)
            keep = sorted(range(F), key=lambda f: (-scaled[f], f))[:k]
            want = np.zeros(F)
            for f in keep:
                want[f] = scaled[f] / n[f]
            assert np.allclose(acts[b, h].detach().numpy(), want, atol=1e-12)


def test_crosscoder_loss_brute_force(vo):
    H, d, F, B = 2, 3, 6, 5
    m = vo.init_uniform_(vo.CrosscoderOracle(H, d, F, act_fn="topk", top_k=2, dtype=torch.float64), seed=3)
    g = torch.Generator().manual_seed(4)
    batch = {f"h{i}": torch.randn(B, d, dtype=torch.float64, generator=g) for i in range(H)}
    out = m.compute_loss(batch, ["h0", "h1"])
    rec = out["reconstructed"].detach().numpy()
    total = 0.0
    for b in range(B):
        for h in range(H):
            total += sum((rec[b, h, j] - batch[f"h{h}"][b, j].item()) ** 2 for j in range(d))
    assert math.isclose(out["loss"].item(), total / (B * H), rel_tol=1e-12)
    # masked mean: only (token, head) cells under the mask count
    mask = torch.tensor([[1, 0], [1, 1], [0, 0], [0, 1], [1, 1]])
    outm = m.compute_loss(batch, ["h0", "h1"], mask=mask)
    tot = sum(sum((rec[b, h, j] - batch[f"h{h}"][b, j].item()) ** 2 for j in range(d))
              for b in range(B) for h in range(H) if mask[b, h])
    assert math.isclose(outm["loss"].item(), tot / mask.sum().item(), rel_tol=1e-12)


# ---- CLT -----------------------------------------------------------------------------------------

def _clt(vo, L=3, d=4, F=8, **kw):
    return vo.init_uniform_(vo.CLTOracle(L, d, F, dtype=torch.float64, **kw), seed=5)


def test_clt_decode_triple_loop(vo):
    L, d, F, B = 3, 4, 8, 5
    m = _clt(vo, L, d, F, act_fn="relu")
    f = torch.rand(B, L, F, dtype=torch.float64, generator=torch.Generator().manual_seed(6))
    y = m.decode(f)
    assert y.shape == (L, B, d)
    for j in range(L):
        for b in range(B):
            for c in range(d):
                acc = m.b_D[j][c].item()
                for i in range(j + 1):
                    for s in range(F):
                        acc += f[b, i, s].item() * m.W_D[j][i, s, c].item()
                assert math.isclose(y[j, b, c].item(), acc, rel_tol=1e-10, abs_tol=1e-12)
    assert torch.equal(m.decode(f, batch_first=True), y.permute(1, 0, 2))


def test_clt_decoder_norm_per_feature_loop(vo):
    L, d, F = 3, 4, 8
    m = _clt(vo, L, d, F)
    n = m.decoder_norm_per_feature()
    for i in range(L):
        for s in range(F):
            sq = sum(m.W_D[j][i, s, c].item() ** 2 for j in range(i, L) for c in range(d))
            assert math.isclose(n[i, s].item(), math.sqrt(sq), rel_tol=1e-12)
    # the constant-one stand-ins of clt.py:801-825
    assert torch.equal(m.decoder_norm(), torch.ones(L * (L + 1) // 2, dtype=torch.float64))
    assert torch.equal(m.decoder_bias_norm(), torch.ones(L, dtype=torch.float64))


def test_clt_encode_loop_and_scaled_hidden_pre(vo):
    L, d, F, B = 3, 4, 8, 4
    m = _clt(vo, L, d, F, act_fn="relu")
    x = torch.randn(B, L, d, dtype=torch.float64, generator=torch.Generator().manual_seed(7))
    acts, hp = m.encode(x, return_hidden_pre=True)
    n = m.decoder_norm_per_feature()
    for b in range(B):
        for i in range(L):
            for s in range(F):
                h = sum(x[b, i, c].item() * m.W_E[i, c, s].item() for c in range(d)) + m.b_E[i, s].item()
                assert math.isclose(hp[b, i, s].item(), h * n[i, s].item(), rel_tol=1e-10, abs_tol=1e-12)  # stays scaled
                assert math.isclose(acts[b, i, s].item(), max(h * n[i, s].item(), 0.0) / n[i, s].item(), rel_tol=1e-10, abs_tol=1e-12)


@pytest.mark.parametrize("act_fn", ["topk", "layertopk", "batchtopk", "batchlayertopk"])
def test_clt_topk_scopes_brute_force(vo, act_fn):
    L, d, F, B, k = 3, 4, 8, 5, 3
    m = _clt(vo, L, d, F, act_fn=act_fn, top_k=k, sparsity_include_decoder_norm=False)
    x = torch.randn(B, L, d, dtype=torch.float64, generator=torch.Generator().manual_seed(8))
    acts, hp = m.encode(x, return_hidden_pre=True)
    h = np.maximum(hp.detach().numpy(), 0.0)
    want = np.zeros_like(h)
    cells = [(b, i, s) for b in range(B) for i in range(L) for s in range(F)]

    def keep_top(group, kk):
        # flattened order of the reference's permute: constant dims first, then the selected dims in the
        # order they are named (utils/math.py:118-135); ties (zeros) go to the lowest flattened index
        for c in sorted(group, key=lambda c: -h[c])[:kk]:
            want[c] = h[c]

    if act_fn == "topk":
        for b in range(B):
            for i in range(L):
                keep_top([(b, i, s) for s in range(F)], k)
    elif act_fn == "layertopk":
        for b in range(B):
            keep_top([(b, i, s) for i in range(L) for s in range(F)], k)
    elif act_fn == "batchtopk":
        for i in range(L):
            keep_top([(b, i, s) for b in range(B) for s in range(F)], k * B)
    else:
        keep_top(cells, k * B)
    # zero-valued picks are indistinguishable from drops, so comparing values is tie-safe
    assert np.allclose(acts.detach().numpy(), want, atol=0)


def test_clt_reduces_to_sae_when_one_layer(vo, oracle):
    d, F, B, k = 6, 16, 9, 3
    m = vo.init_uniform_(vo.CLTOracle(1, d, F, act_fn="topk", top_k=k, dtype=torch.float64), seed=9)
    s = oracle.SAEOracle(d, F, act_fn="topk", top_k=k, dtype=torch.float64)
    with torch.no_grad():
        s.W_E.copy_(m.W_E[0]); s.b_E.copy_(m.b_E[0]); s.W_D.copy_(m.W_D[0][0]); s.b_D.copy_(m.b_D[0])
    g = torch.Generator().manual_seed(10)
    x, y = torch.randn(B, d, dtype=torch.float64, generator=g), torch.randn(B, d, dtype=torch.float64, generator=g)
    out = m.compute_loss({"i": x, "o": y}, ["i"], ["o"])
    ref = s.compute_loss({"in": x, "out": y, "tokens": torch.zeros(B)})
    assert torch.allclose(out["feature_acts"][:, 0], ref["feature_acts"], atol=1e-12)
    assert math.isclose(out["loss"].item(), ref["loss"].item(), rel_tol=1e-12)


def test_clt_loss_and_sparsity_terms(vo):
    L, d, F, B = 3, 4, 8, 5
    m = _clt(vo, L, d, F, act_fn="relu")
    g = torch.Generator().manual_seed(11)
    batch = {f"i{l}": torch.randn(B, d, dtype=torch.float64, generator=g) for l in range(L)}
    batch.update({f"o{l}": torch.randn(B, d, dtype=torch.float64, generator=g) for l in range(L)})
    hin, hout = [f"i{l}" for l in range(L)], [f"o{l}" for l in range(L)]
    out = m.compute_loss(batch, hin, hout, sparsity_loss_type="tanh", tanh_stretch_coefficient=2.0, l1_coefficient=0.3)
    rec, fa, n = out["reconstructed"], out["feature_acts"], m.decoder_norm_per_feature()
    l_rec = sum((rec[l, b, c].item() - batch[f"o{l}"][b, c].item()) ** 2 for l in range(L) for b in range(B) for c in range(d)) / (L * B)
    l_s = sum(0.3 * math.tanh(2.0 * fa[b, l, s].item() * n[l, s].item()) for b in range(B) for l in range(L) for s in range(F)) / (B * L)
    assert math.isclose(out["l_rec"].item(), l_rec, rel_tol=1e-10)
    assert math.isclose(out["loss"].item(), l_rec + l_s, rel_tol=1e-10)
    # tanh-quad: the frequency is averaged over batch AND layers, one value per feature column (clt.py:1075-1081)
    outq = m.compute_loss(batch, hin, hout, sparsity_loss_type="tanh-quad", frequency_scale=0.05)
    tot = 0.0
    for s in range(F):
        q = sum(math.tanh(4.0 * fa[b, l, s].item() * n[l, s].item()) for b in range(B) for l in range(L)) / (B * L)
        tot += q * (1 + q / 0.05)
    assert math.isclose(outq["loss"].item(), l_rec + tot, rel_tol=1e-10)


# ---- Lorsa ---------------------------------------------------------------------------------------

def _lorsa(vo, **kw):
    args = dict(d_model=6, d_sae=8, n_qk_heads=2, d_qk_head=4, n_ctx=8, act_fn="relu", dtype=torch.float64)
    args.update(kw)
    return vo.init_uniform_(vo.LorsaOracle(**args), seed=12)


def test_lorsa_hidden_pre_scalar_loops(vo):
    m = _lorsa(vo, sparsity_include_decoder_norm=False)
    b, s = 2, 5
    x = torch.randn(b, s, 6, dtype=torch.float64, generator=torch.Generator().manual_seed(13))
    acts, hp, pattern = m.encode(x, return_hidden_pre=True, return_attention_pattern=True)
    F, h, dq, group = 8, 2, 4, 4
    for bi in range(b):
        q = [[[sum(x[bi, p, c].item() * m.W_Q[hh, c, e].item() for c in range(6)) + m.b_Q[hh, e].item() for e in range(dq)]
              for hh in range(h)] for p in range(s)]
        kk = [[[sum(x[bi, p, c].item() * m.W_K[hh, c, e].item() for c in range(6)) + m.b_K[hh, e].item() for e in range(dq)]
               for hh in range(h)] for p in range(s)]
        v = [[sum(x[bi, p, c].item() * m.W_V[f, c].item() for c in range(6)) + m.b_V[f].item() for f in range(F)] for p in range(s)]
        for hh in range(h):
            for qp in range(s):
                sc = [sum(q[qp][hh][e] * kk[kp][hh][e] for e in range(dq)) / 2.0 for kp in range(qp + 1)]  # sqrt(4) = 2
                mx = max(sc)
                ex = [math.exp(t - mx) for t in sc]
                z = sum(ex)
                for kp in range(s):
                    want = ex[kp] / z if kp <= qp else 0.0
                    assert math.isclose(pattern[bi, hh, qp, kp].item(), want, rel_tol=1e-10, abs_tol=1e-14)
                for r in range(group):
                    f = hh * group + r
                    want = sum(ex[kp] / z * v[kp][f] for kp in range(qp + 1))
                    assert math.isclose(hp[bi, qp, f].item(), want, rel_tol=1e-9, abs_tol=1e-12)
                    assert math.isclose(acts[bi, qp, f].item(), max(want, 0.0), rel_tol=1e-9, abs_tol=1e-12)


def test_lorsa_matches_library_attention_when_groups_are_heads(vo):
    """With ov_group_size == d_qk_head the hidden pre-activation is ordinary causal multi-head attention:
    torch's scaled_dot_product_attention is the library routine for it."""
    m = _lorsa(vo, d_sae=8, n_qk_heads=2, d_qk_head=4, sparsity_include_decoder_norm=False)
    x = torch.randn(3, 7, 6, dtype=torch.float64, generator=torch.Generator().manual_seed(14))
    _, hp = m.encode(x, return_hidden_pre=True)
    q, k, v = m._compute_qkv(x)
    z = torch.nn.functional.scaled_dot_product_attention(
        q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.reshape(3, 7, 2, 4).permute(0, 2, 1, 3), is_causal=True, scale=0.5)
    assert torch.allclose(hp, z.permute(0, 2, 1, 3).reshape(3, 7, 8), atol=1e-12)


def test_lorsa_decode_and_norm_scaling(vo):
    m = _lorsa(vo, act_fn="topk", top_k=3)
    x = torch.randn(2, 6, 6, dtype=torch.float64, generator=torch.Generator().manual_seed(15))
    acts, hp = m.encode(x, return_hidden_pre=True)
    m2 = _lorsa(vo, act_fn="topk", top_k=3, sparsity_include_decoder_norm=False)
    _, hp_plain = m2.encode(x, return_hidden_pre=True)
    assert torch.allclose(hp, hp_plain, atol=1e-12)      # hidden_pre is handed back unscaled
    n = m.decoder_norm().detach().numpy()
    for bi in range(2):
        for p in range(6):
            scaled = np.maximum(hp_plain[bi, p].detach().numpy() * n, 0.0)
            keep = sorted(range(8), key=lambda f: (-scaled[f], f))[:3]
            want = np.zeros(8)
            for f in keep:
                want[f] = scaled[f] / n[f]
            assert np.allclose(acts[bi, p].detach().numpy(), want, atol=1e-12)
    y = m.decode(acts)
    for c in range(6):
        want = sum(acts[1, 2, f].item() * m.W_O[f, c].item() for f in range(8)) + m.b_D[c].item()
        assert math.isclose(y[1, 2, c].item(), want, rel_tol=1e-10, abs_tol=1e-12)


@pytest.mark.parametrize("adjacent", [True, False])
def test_lorsa_rotary_is_a_plane_rotation(vo, adjacent):
    """Each rotated pair (a, b) at position p becomes (a cos t - b sin t, a sin t + b cos t) with
    t = p / base^(i / (rotary_dim / 2)) for pair i; dims beyond rotary_dim pass through."""
    m = _lorsa(vo, positional_embedding_type="rotary", rotary_dim=2, d_qk_head=4, rotary_base=100, rotary_adjacent_pairs=adjacent)
    x = torch.randn(1, 5, 2, 4, dtype=torch.float64, generator=torch.Generator().manual_seed(16))
    y = m._apply_rotary(x)
    for p in range(5):
        t = p / (100 ** 0.0)
        a, b = x[0, p, 1, 0].item(), x[0, p, 1, 1].item()
        assert math.isclose(y[0, p, 1, 0].item(), a * math.cos(t) - b * math.sin(t), rel_tol=1e-6, abs_tol=1e-7)
        assert math.isclose(y[0, p, 1, 1].item(), a * math.sin(t) + b * math.cos(t), rel_tol=1e-6, abs_tol=1e-7)
        assert torch.equal(y[0, p, :, 2:], x[0, p, :, 2:])
    # four rotated dims: pair frequencies base^0 and base^(1/2); pairing differs between the two conventions
    m4 = _lorsa(vo, positional_embedding_type="rotary", rotary_dim=4, d_qk_head=4, rotary_base=100, rotary_adjacent_pairs=adjacent)
    y4 = m4._apply_rotary(x)
    pairs = [(0, 1), (2, 3)] if adjacent else [(0, 2), (1, 3)]
    for p in range(5):
        for i, (ia, ib) in enumerate(pairs):
            t = p / (100 ** (i / 2))
            a, b = x[0, p, 0, ia].item(), x[0, p, 0, ib].item()
            assert math.isclose(y4[0, p, 0, ia].item(), a * math.cos(t) - b * math.sin(t), rel_tol=1e-6, abs_tol=1e-7)
            assert math.isclose(y4[0, p, 0, ib].item(), a * math.sin(t) + b * math.cos(t), rel_tol=1e-6, abs_tol=1e-7)


def test_lorsa_rotary_scores_depend_on_relative_position_only(vo):
    """Invariant of rotary embeddings with full-width rotation: <rot(q, p), rot(k, r)> depends on p - r."""
    m = _lorsa(vo, positional_embedding_type="rotary", rotary_dim=4, d_qk_head=4)
    g = torch.Generator().manual_seed(17)
    q, k = torch.randn(4, dtype=torch.float64, generator=g), torch.randn(4, dtype=torch.float64, generator=g)
    Q = m._apply_rotary(q.expand(1, 8, 1, 4).clone())[0, :, 0]
    K = m._apply_rotary(k.expand(1, 8, 1, 4).clone())[0, :, 0]
    s = Q @ K.t()
    for off in range(-3, 4):
        diag = torch.diagonal(s, offset=off)
        assert torch.allclose(diag, diag[0].expand_as(diag), atol=1e-5)
