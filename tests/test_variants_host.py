"""Host logic of the crosscoder / CLT / Lorsa modules on CPU: configs, parameter layouts, state-dict
keys, and the dense API path (ReLU / JumpReLU activations, which need no kernel) against the oracle
and the reference's known answers."""

import importlib
import json
import os

import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_kats.json")))


@pytest.fixture(scope="module")
def vo(oracle):
    return importlib.import_module("oracle.variants_oracle")


def copy_params(dst, src):
    s = dict(src.named_parameters())
    s = {k.replace("ln_q_w", "ln_q.w").replace("ln_k_w", "ln_k.w"): v for k, v in s.items()}
    with torch.no_grad():
        for k, p in dst.named_parameters():
            if k.startswith("activation_function"):
                continue
            p.copy_(s[k].to(p.dtype))


# ---- crosscoder ----------------------------------------------------------------------------------

def kat_crosscoder(pkg):
    cfg = pkg.CrosscoderConfig(hook_points=["head0", "head1"], d_model=2, expansion_factor=2, act_fn="relu", top_k=2,
                               norm_activation="token-wise", n_heads=2)
    m = pkg.Crosscoder(cfg)
    f = KATS["crosscoder_fixture"]
    with torch.no_grad():
        for n in ("W_E", "b_E", "W_D", "b_D"):
            getattr(m, n).copy_(torch.tensor(f[n]))
    return m


def test_crosscoder_reference_kats(pkg):
    m = kat_crosscoder(pkg)
    e, d, n = KATS["crosscoder_encode"], KATS["crosscoder_decode"], KATS["crosscoder_norms"]
    acts, hp = m.encode(torch.tensor(e["x"]), return_hidden_pre=True)
    assert torch.allclose(hp, torch.tensor(e["expected_hidden_pre"]), atol=e["atol"])
    assert torch.all(acts > 0)
    assert torch.allclose(m.decode(torch.tensor(d["feature_acts"])), torch.tensor(d["expected"]), atol=d["atol"])
    assert torch.allclose(m.encoder_norm(), torch.tensor(n["encoder_norm"]), atol=n["atol"])
    assert torch.allclose(m.decoder_norm(), torch.tensor(n["decoder_norm"]), atol=n["atol"])
    assert torch.allclose(m.decoder_bias_norm(), torch.tensor([[0.224], [0.224]]), atol=1e-3)
    x = torch.tensor(e["x"])
    assert torch.allclose(m.forward(x), m.decode(m.encode(x)), atol=1e-6)     # tests/unit/test_crosscoder.py:203-227


def test_crosscoder_layout_and_state(pkg):
    m = kat_crosscoder(pkg)
    assert tuple(m.W_E.shape) == (2, 2, 4) and m.W_E.permute(2, 0, 1).is_contiguous()      # feature-major storage
    sd = m.full_state_dict()
    assert set(k for k in sd if not k.startswith("dataset")) == {"W_E", "b_E", "W_D", "b_D"}
    assert sd["W_E"].is_contiguous() and torch.equal(sd["W_E"], torch.tensor(KATS["crosscoder_fixture"]["W_E"]))
    m2 = kat_crosscoder(pkg)
    with torch.no_grad():
        m2.W_E.zero_()
    m2.load_full_state_dict(sd)
    assert torch.equal(m2.W_E, m.W_E)
    # tests/unit/test_crosscoder.py:296-335: fixed-norm setters
    m.set_decoder_to_fixed_norm(2.0, force_exact=True)
    assert torch.allclose(m.decoder_norm(), torch.full((2, 4), 2.0), atol=1e-6)
    m.set_encoder_to_fixed_norm(1.5)
    assert torch.allclose(m.encoder_norm(), torch.full((2, 4), 1.5), atol=1e-6)
    # init: every head gets the same draw, biases zero (crosscoder.py:160-219; tests/unit/test_crosscoder.py:98-117)
    m.init_parameters(encoder_uniform_bound=0.1, decoder_uniform_bound=0.1, init_log_jumprelu_threshold_value=0.0)
    assert torch.equal(m.W_E[0], m.W_E[1]) and torch.equal(m.W_D[0], m.W_D[1])
    assert m.W_E.abs().max() <= 0.1 and m.W_D.abs().max() <= 0.1
    assert torch.all(m.b_E == 0) and torch.all(m.b_D == 0)


def test_crosscoder_dense_loss_matches_oracle(pkg, vo):
    H, d, F, B = 3, 4, 10, 6
    ref = vo.init_uniform_(vo.CrosscoderOracle(H, d, F, act_fn="relu"), seed=21)
    hooks = [f"h{i}" for i in range(H)]
    m = pkg.Crosscoder(pkg.CrosscoderConfig(hook_points=hooks, d_model=d, expansion_factor=F / d, act_fn="relu",
                                            norm_activation="inference"))
    copy_params(m, ref)
    g = torch.Generator().manual_seed(22)
    batch = {h: torch.randn(B, d, generator=g) for h in hooks}
    batch["tokens"] = torch.zeros(B, dtype=torch.long)
    out, want = m.compute_loss(batch), ref.compute_loss(batch, hooks)
    assert torch.allclose(out["loss"], want["loss"], rtol=1e-6)
    out["loss"].backward(); want["loss"].backward()
    for n in ("W_E", "b_E", "W_D", "b_D"):
        assert torch.allclose(getattr(m, n).grad, getattr(ref, n).grad, rtol=1e-5, atol=1e-7), n
    # narrower inputs are zero-padded to d_model (crosscoder.py:554-566)
    narrow = dict(batch); narrow["h1"] = batch["h1"][:, :2]
    x, _, _ = m.prepare_input(narrow)
    assert x.shape == (B, H, d) and torch.all(x[:, 1, 2:] == 0)


# ---- CLT -----------------------------------------------------------------------------------------

def make_clt(pkg, vo, act_fn, L=3, d=4, F=8, k=3, seed=23, **kw):
    ref = vo.init_uniform_(vo.CLTOracle(L, d, F, act_fn=act_fn, top_k=k, **kw), seed=seed)
    hin, hout = [f"i{l}" for l in range(L)], [f"o{l}" for l in range(L)]
    cfg = pkg.CLTConfig(hook_points_in=hin, hook_points_out=hout, d_model=d, expansion_factor=F / d, act_fn=act_fn, top_k=k,
                        norm_activation="inference", **kw)
    m = pkg.CrossLayerTranscoder(cfg)
    copy_params(m, ref)
    return m, ref, hin, hout


def clt_batch(L, B, d, seed):
    g = torch.Generator().manual_seed(seed)
    batch = {f"i{l}": torch.randn(B, d, generator=g) for l in range(L)}
    batch.update({f"o{l}": torch.randn(B, d, generator=g) for l in range(L)})
    batch["tokens"] = torch.zeros(B, dtype=torch.long)
    return batch


def test_clt_layout_and_state(pkg, vo):
    m, ref, _, _ = make_clt(pkg, vo, "relu")
    assert tuple(m.W_E.shape) == (3, 4, 8) and m.W_E.permute(0, 2, 1).is_contiguous()
    keys = set(m.state_dict().keys())
    assert keys == {"W_E", "b_E", "W_D.0", "W_D.1", "W_D.2", "b_D.0", "b_D.1", "b_D.2"}     # ParameterList names of clt.py:160-176
    assert [tuple(w.shape) for w in m.W_D] == [(1, 8, 4), (2, 8, 4), (3, 8, 4)]
    assert m.cfg.n_decoders == 6
    assert torch.allclose(m.decoder_norm_per_feature(), ref.decoder_norm_per_feature(), rtol=1e-6)
    assert torch.allclose(m.decoder_norm_per_feature(layer=1)[1:], torch.stack([w[1].norm(dim=-1) for w in list(ref.W_D)[1:]]))
    m.init_parameters()
    assert m.W_E.abs().max() <= 1 / 8 ** 0.5 and all(w.abs().max() <= 1 / 12 ** 0.5 for w in m.W_D)
    assert torch.all(m.b_E == 0) and all(torch.all(b == 0) for b in m.b_D)


@pytest.mark.parametrize("act_fn,loss_type", [("relu", None), ("relu", "tanh"), ("jumprelu", "tanh-quad"), ("relu", "power"),
                                               ("layertopk", None), ("batchtopk", None), ("batchlayertopk", None)])
def test_clt_dense_loss_matches_oracle(pkg, vo, act_fn, loss_type):
    m, ref, hin, hout = make_clt(pkg, vo, act_fn)
    if act_fn == "jumprelu":
        with torch.no_grad():
            t = torch.linspace(-2.0, -0.5, 24).view(3, 8)
            m.activation_function.log_jumprelu_threshold.copy_(t)
            ref.activation_function.log_jumprelu_threshold.copy_(t)
    batch = clt_batch(3, 7, 4, seed=24)
    kw = dict(sparsity_loss_type=loss_type, l1_coefficient=0.2) if loss_type else {}
    out, want = m.compute_loss(batch, **kw), ref.compute_loss(batch, hin, hout, **kw)
    assert torch.allclose(out["feature_acts"], want["feature_acts"], rtol=1e-5, atol=1e-7)
    assert torch.allclose(out["reconstructed"], want["reconstructed"], rtol=1e-5, atol=1e-6)
    assert torch.allclose(out["loss"], want["loss"], rtol=1e-5)
    out["loss"].backward(); want["loss"].backward()
    rp = dict(ref.named_parameters())
    for n, p in m.named_parameters():
        assert torch.allclose(p.grad, rp[n].grad, rtol=1e-4, atol=1e-6), n


@pytest.mark.parametrize("act_fn", ["relu", "jumprelu"])
def test_clt_standardize_folds_dataset_norms_as_the_reference_does(pkg, vo, act_fn):
    """clt.py:908-937.  Closed form per parameter (W_E untouched; b_E[l] and the threshold / fin(l);
    W_D[to][from] * fin(from) / fout(to); b_D[to] / fout(to)) and the property the fold exists for: the folded
    model on raw activations gives the normalised model's features / fin(l) and reconstruction / fout(l)."""
    import math
    # without the decoder-norm scale around the activation: a threshold on h * norm is not invariant under the
    # fold (the norms change with W_D), in the reference either
    m, _, hin, hout = make_clt(pkg, vo, act_fn, sparsity_include_decoder_norm=False)
    L, d = 3, 4
    if act_fn == "jumprelu":
        with torch.no_grad():
            m.activation_function.log_jumprelu_threshold.copy_(torch.linspace(-2.0, -0.5, 24).view(3, 8))
    norms = {**{h: 1.5 + 0.5 * l for l, h in enumerate(hin)}, **{h: 0.7 + 0.3 * l for l, h in enumerate(hout)}}
    fin = [math.sqrt(d) / norms[h] for h in hin]
    fout = [math.sqrt(d) / norms[h] for h in hout]
    m.cfg.norm_activation = "dataset-wise"
    m.set_dataset_average_activation_norm(norms)
    raw = torch.randn(7, L, d, generator=torch.Generator().manual_seed(5))
    x_n = raw * torch.tensor(fin).view(1, L, 1)
    with torch.no_grad():
        acts_n = m.encode(x_n)
        rec_n = m.decode(acts_n, batch_first=True)
    before = {n: p.detach().clone() for n, p in m.named_parameters()}
    versions = {n: p._version for n, p in m.named_parameters()}
    m.standardize_parameters_of_dataset_norm()
    assert m.cfg.norm_activation == "inference"
    after = dict(m.named_parameters())
    assert torch.equal(after["W_E"], before["W_E"])
    for l in range(L):
        assert torch.allclose(after["b_E"][l], before["b_E"][l] / fin[l])
        assert torch.allclose(after[f"b_D.{l}"], before[f"b_D.{l}"] / fout[l])
        for lf in range(l + 1):
            assert torch.allclose(after[f"W_D.{l}"][lf], before[f"W_D.{l}"][lf] * (fin[lf] / fout[l]))
        if act_fn == "jumprelu":
            n = "activation_function.log_jumprelu_threshold"
            assert torch.allclose(after[n][l].exp(), before[n][l].exp() / fin[l])
    # every touched parameter's version moved, so cached bf16 copies and norms are rebuilt
    assert all(after[n]._version > versions[n] for n in after if n != "W_E")
    with torch.no_grad():
        acts = m.encode(raw)
        rec = m.decode(acts, batch_first=True)
    assert torch.allclose(acts, acts_n / torch.tensor(fin).view(1, L, 1), rtol=1e-5, atol=1e-7)
    assert torch.allclose(rec, rec_n / torch.tensor(fout).view(1, L, 1), rtol=1e-5, atol=1e-6)


# ---- Lorsa ---------------------------------------------------------------------------------------

def make_lorsa(pkg, vo, act_fn="relu", **kw):
    args = dict(d_model=8, d_sae=12, n_qk_heads=3, d_qk_head=4, n_ctx=8)
    okw = dict(kw)
    ref = vo.init_uniform_(vo.LorsaOracle(act_fn=act_fn, top_k=3, **args, **okw), seed=25)
    ckw = dict(kw)
    if ckw.get("use_post_qk_ln"):
        ckw["normalization_type"] = "RMS"
    ckw.setdefault("rotary_dim", 4)
    cfg = pkg.LorsaConfig(hook_point_in="in", hook_point_out="out", d_model=8, expansion_factor=1.5, n_qk_heads=3, d_qk_head=4,
                          n_ctx=8, act_fn=act_fn, top_k=3, norm_activation="inference", **ckw)
    m = pkg.LowRankSparseAttention(cfg)
    copy_params(m, ref)
    return m, ref


@pytest.mark.parametrize("kw", [dict(positional_embedding_type="none"), dict(positional_embedding_type="rotary", rotary_dim=4),
                                dict(positional_embedding_type="rotary", rotary_dim=2, rotary_adjacent_pairs=False),
                                dict(positional_embedding_type="none", use_post_qk_ln=True),
                                dict(positional_embedding_type="none", sparsity_include_decoder_norm=False)])
def test_lorsa_dense_loss_matches_oracle(pkg, vo, kw):
    m, ref = make_lorsa(pkg, vo, **kw)
    assert m.cfg.d_sae == 12 and m.cfg.ov_group_size == 4 and m.cfg.attn_scale == 2.0
    g = torch.Generator().manual_seed(26)
    batch = {"in": torch.randn(2, 6, 8, generator=g), "out": torch.randn(2, 6, 8, generator=g), "tokens": torch.zeros(2, 6)}
    out, want = m.compute_loss(batch), ref.compute_loss(batch)
    assert torch.allclose(out["hidden_pre"], want["hidden_pre"], rtol=1e-5, atol=1e-6)
    assert torch.allclose(out["loss"], want["loss"], rtol=1e-5)
    # the explicit-pattern branch gives the same activations as the fused-attention branch
    acts, pattern = m.encode(batch["in"], return_attention_pattern=True)
    _, _, ref_pattern = ref.encode(batch["in"], return_hidden_pre=True, return_attention_pattern=True)
    assert torch.allclose(acts, want["feature_acts"], rtol=1e-5, atol=1e-6)
    assert torch.allclose(pattern, ref_pattern, rtol=1e-5, atol=1e-7)
    out["loss"].backward(); want["loss"].backward()
    rp = {k.replace("ln_q_w", "ln_q.w").replace("ln_k_w", "ln_k.w"): v for k, v in ref.named_parameters()}
    for n, p in m.named_parameters():
        assert torch.allclose(p.grad, rp[n].grad, rtol=1e-4, atol=1e-6), n


def test_lorsa_aliases_state_and_checkpoint_widening(pkg, vo):
    m, _ = make_lorsa(pkg, vo, positional_embedding_type="none")
    assert m.W_D is m.W_O and torch.equal(m.W_E, m.W_V.T) and m.b_O is m.b_D
    assert {"W_Q", "W_K", "W_V", "W_O", "b_Q", "b_K", "b_V", "b_D"} <= set(m.state_dict().keys())
    # a checkpoint with a single query/key head is repeated to the configured three (lorsa.py:960-980)
    sd = {k: v.clone() for k, v in m.state_dict().items()}
    for k in ("W_Q", "W_K", "b_Q", "b_K"):
        sd[k] = sd[k][:1]
    m.load_full_state_dict(sd)
    assert torch.equal(m.W_Q[0], m.W_Q[2]) and torch.equal(m.b_K[0], m.b_K[1])
    with pytest.raises(NotImplementedError):
        m.set_encoder_to_fixed_norm(1.0)
    n0 = m.decoder_norm().clone()
    hp0 = m.encode(torch.ones(1, 4, 8), return_hidden_pre=True)[1]
    m.transform_to_unit_decoder_norm()        # W_O /= n, W_V *= n, b_V *= n: same reconstruction (lorsa.py:611-617)
    assert torch.allclose(m.decoder_norm(), torch.ones(12), atol=1e-6)
    assert torch.allclose(m.encode(torch.ones(1, 4, 8), return_hidden_pre=True)[1], hp0 * n0, rtol=1e-5, atol=1e-6)


def test_registry_builds_every_model(pkg):
    from lm_saes_amd.config import SAE_TYPE_TO_CONFIG_CLASS, SAE_TYPE_TO_MODEL_CLASS

    assert set(SAE_TYPE_TO_MODEL_CLASS) >= {"sae", "crosscoder", "clt", "lorsa"}
    assert set(SAE_TYPE_TO_CONFIG_CLASS) >= {"sae", "crosscoder", "clt", "lorsa"}
    cfg = pkg.CrosscoderConfig(hook_points=["a", "b"], d_model=4, expansion_factor=2)
    assert isinstance(pkg.SparseDictionary.from_config(cfg), pkg.Crosscoder)
