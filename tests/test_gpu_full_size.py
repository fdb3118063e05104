"""The benchmark configurations at their full sizes.

The CPU oracle cannot finish these shapes in seconds, so the kernel path is checked here through
size-independent properties and against an independent dense recomputation with torch's library
routines ON THE GPU (matmul, topk, sort): given the kernel's own pre-activation, the selection must
be exactly the k largest with lowest-index ties; given the selection, reconstruction, loss and every
gradient must equal what dense GEMMs give; the optimiser move must equal the closed-form first Adam
step.  The small-shape tests elsewhere tie the same kernels to the CPU oracle, and the last three tests of this file
run the oracle itself, with the full dictionaries, on a few tokens (or one sequence) of the full-size steps.
"""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def rel_err(got, want):
    return ((got.double() - want.double()).abs().max() / want.double().abs().max().clamp_min(1e-30)).item()


def dense_mask(code):
    """bool [B, F]: the positions a sparse code holds."""
    B, F = code.n_tokens, code.d_sae
    slots = torch.arange(code.n_slots, device=code.idx.device)
    tok = (torch.searchsorted(code.row_off, slots, right=True) - 1).clamp_(min=0)
    valid = (slots - code.row_off[tok]) < code.row_nnz[tok]
    m = torch.zeros(B * F, dtype=torch.bool, device=code.idx.device)
    m[(tok * F + code.idx.long())[valid]] = True
    return m.view(B, F)


def check_threshold_selection(score, kept, per_row: bool):
    """kept must be the largest entries of `score` (per row, or over the whole batch), ties at the
    threshold going to the lowest (flattened) index."""
    if not per_row:
        score, kept = score.reshape(1, -1), kept.reshape(1, -1)
    lo = score.masked_fill(~kept, float("inf")).min(dim=1).values          # smallest kept
    hi = score.masked_fill(kept, float("-inf")).max(dim=1).values          # largest dropped
    assert torch.all(lo >= hi), "a dropped entry is larger than a kept one"
    assert torch.all(lo > 0), "a non-positive entry was kept"
    tied = lo == hi
    if tied.any():
        n = score.shape[1]
        pos = torch.arange(n, device=score.device).expand_as(score)
        at_t = score == lo[:, None]
        last_kept = torch.where(at_t & kept, pos, torch.full_like(pos, -1)).max(dim=1).values
        first_dropped = torch.where(at_t & ~kept, pos, torch.full_like(pos, n)).min(dim=1).values
        assert torch.all(last_kept[tied] < first_dropped[tied]), "a tie at the threshold did not go to the lowest index"
    return int(tied.sum().item())


def build_sae(pkg, dev, d, F, k, B, r, act_fn="topk", seed=4):
    from lm_saes_amd import synthetic

    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn=act_fn, top_k=k,
                        norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    x = synthetic.activations(B, d, r, seed=seed).to(dev)
    with torch.no_grad():
        g = torch.Generator(device=dev).manual_seed(seed)
        wt = sae.W_E.t()
        wt.uniform_(-1.0 / d ** 0.5, 1.0 / d ** 0.5, generator=g)
        sae.W_D.copy_(wt / wt.norm(dim=1, keepdim=True) * (0.5 + torch.rand(F, 1, device=dev, generator=g)))
        sae.b_E.copy_(0.01 * torch.randn(F, device=dev, generator=g))
        sae.b_D.copy_(x.mean(0))
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    return sae, batch


def own_scores(pkg, sae, x):
    """(h, n): the pre-activation plus bias exactly as the select kernel forms it (the encoder kernel is
    deterministic, so running it again gives the same bits) and the decoder norms it scales by."""
    pre = pkg.ops.encoder_gemm(pkg.ops.cast_bf16(x.contiguous()), sae._w_enc_operand(True), torch.bfloat16)
    return pre.float() + sae.b_E.detach(), sae._decoder_norm_nograd()


def dense_backward(sae, x_bf, kept, val, recon, label, w):
    """Gradients of sum_b w_b |recon_b - label_b|^2 by dense library GEMMs, given the selection `kept`, the kept
    values `val` ([B, F] dense) and bf16-rounded operands (the rounding the kernels' operands carry)."""
    Wd = sae._w_dec_operand(True).float()
    grad_recon = 2.0 * w[:, None] * (recon - label)
    dW_D = val.t() @ grad_recon.bfloat16().float()      # the decoder gradient rows are gathered in bf16 under autocast
    d_pre = (grad_recon @ Wd.t()) * kept
    dW_Et = d_pre.t() @ x_bf.float()
    return dW_D, dW_Et, d_pre.sum(0), grad_recon.sum(0)


def test_headline_shape_step_properties(pkg, dev):
    """TopK SAE d=4096, F=131072, k=64, 4096 tokens, bf16 operands: the benchmark's own configuration."""
    d, F, k, B = 4096, 131072, 64, 4096
    sae, batch = build_sae(pkg, dev, d, F, k, B, r=64)
    x = batch["in"]
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = sae.compute_loss(batch)
    code = out["sparse_code"]
    # --- the code: k entries per row, ascending, in range
    assert torch.all(code.row_nnz == k) and torch.equal(code.row_off, torch.arange(B, device=dev) * k)
    idx = code.idx.view(B, k)
    assert torch.all(idx[:, 1:] > idx[:, :-1]) and idx.min() >= 0 and idx.max() < F
    # --- selection = k largest of the kernel's own scaled pre-activation, lowest index on ties
    hp, n = own_scores(pkg, sae, x)                         # (pre + b_E) as the kernel formed it, [B, F] fp32
    assert rel_err(out["hidden_pre"], hp) < 1e-6
    x_bf = x.bfloat16()
    assert rel_err(hp, x_bf.float() @ sae._w_enc_operand(True).float().t() + sae.b_E.detach()) < 2e-2     # bf16 output rounding
    kept = dense_mask(code)
    ties = check_threshold_selection(hp * n, kept, per_row=True)
    print(f"rows with a tie at the threshold: {ties}", flush=True)
    val = torch.zeros(B, F, device=dev).masked_scatter_(kept, code.val)        # both in (row, ascending index) order
    assert rel_err(val[kept], ((hp * n) / n)[kept]) < 1e-6                      # kept values: scaled, selected, unscaled again
    # --- decode, loss
    Wd = sae._w_dec_operand(True).float()
    recon = val @ Wd + sae.b_D.detach()
    assert rel_err(out["reconstructed"], recon) < 1e-4
    w = torch.full((B,), 1.0 / B, device=dev)
    assert abs(out["loss"].item() - ((recon - x).pow(2).sum(-1) * w).sum().item()) < 1e-4 * out["loss"].item()
    doubled = pkg.ops.sparse_decode_fwd(pkg.ops.SparseCode(code.idx, 2 * code.val, code.row_off, code.row_nnz, B, F),
                                        sae._w_dec_operand(True), sae.b_D.detach())
    assert rel_err(doubled - sae.b_D.detach(), 2 * (out["reconstructed"] - sae.b_D.detach())) < 1e-6   # linear in the values
    # --- backward against dense GEMMs
    out["loss"].backward()
    dW_D, dW_Et, db_E, db_D = dense_backward(sae, x_bf, kept, val, out["reconstructed"], x, w)
    assert rel_err(sae.W_D.grad, dW_D) < 1e-4
    assert rel_err(sae.W_E.grad.t(), dW_Et) < 1e-4
    assert rel_err(sae.b_E.grad, db_E) < 1e-4 and rel_err(sae.b_D.grad, db_D) < 1e-4
    # --- the optimiser consuming factored gradients: closed-form first Adam step, fresh shadows and norms
    g_D, g_Et = sae.W_D.grad.clone(), sae.W_E.grad.t().clone()
    p_D, p_Et = sae.W_D.detach().clone(), sae.W_E.detach().t().clone()
    for p in sae.parameters():
        p.grad = None
    lr, eps = 4e-4, 1e-8
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=lr, eps=eps, model=sae)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        loss = sae.compute_loss(batch, return_aux_data=False)
    loss.backward()
    assert sae.W_D.grad is None and sae.W_D._sparse_grad is not None      # no dense gradient matrix was written
    opt.step()
    for p_new, p_old, g in ((sae.W_D.detach(), p_D, g_D), (sae.W_E.detach().t(), p_Et, g_Et)):
        want = -lr * g / (g.abs() + eps)           # m_hat = g, v_hat = g^2 on the first step
        assert ((p_new - p_old) - want).abs().max().item() < 2e-3 * lr
    assert torch.equal(sae.get_derived_buffer("W_D.bf16"), sae.W_D.detach().bfloat16())
    assert torch.equal(sae.get_derived_buffer("W_E.bf16"), sae.W_E.detach().t().bfloat16())
    assert rel_err(sae.get_derived_buffer("W_D.norm"), sae.W_D.detach().norm(dim=1)) < 1e-6


class _FixedDead:
    def __init__(self, is_dead):
        self.is_dead = is_dead

    def update_dead_statistics(self, feature_acts, mask, specs):
        return self.is_dead

    def update_dead_statistics_sparse(self, code, mask):
        return self.is_dead


def test_batchtopk_auxk_shape_step_properties(pkg, oracle, dev):
    """BatchTopK SAE d=2048, F=32768, 8192 tokens, global top 64 x 8192, aux-k over the top 512 dead features."""
    d, F, k, B, k_aux, alpha = 2048, 32768, 64, 8192, 512, 1 / 32
    sae, batch = build_sae(pkg, dev, d, F, k, B, r=32, act_fn="batchtopk")
    x = batch["in"]
    g = torch.Generator(device=dev).manual_seed(5)
    is_dead = torch.rand(F, device=dev, generator=g) < 0.1
    dead = _FixedDead(is_dead)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = sae.compute_loss(batch, auxk_coefficient=alpha, k_aux=k_aux, update_dead_statistics=dead.update_dead_statistics)
    code = out["sparse_code"]
    assert int(code.row_nnz.sum().item()) == k * B                                  # exactly k x B survive, batch-wide
    assert code.row_nnz.float().std().item() > 0
    hp, n = own_scores(pkg, sae, x)
    kept = dense_mask(code)
    assert int(kept.sum().item()) == k * B
    check_threshold_selection(hp * n, kept, per_row=False)
    # the oracle's own BatchTopK (models/sparse_dictionary.py:761-794 restated: relu mask, then the k B largest over both
    # axes by a stable sort on the CPU) on the kernel's scores: the same set of 524 288 positions, bit for bit
    score_cpu = (hp * n).cpu()
    want_kept = oracle.topk(score_cpu * score_cpu.gt(0).to(score_cpu.dtype), k=k * B, dim=(-2, -1), abs=True) != 0
    assert torch.equal(want_kept, kept.cpu())
    del score_cpu, want_kept
    # rows ascend in index
    val = torch.zeros(B, F, device=dev).masked_scatter_(kept, code.val[: k * B])
    assert rel_err(val[kept], hp[kept]) < 1e-6
    # the aux selection, recomputed densely: the k_aux x B largest of the dead features' scaled pre-activations
    n_dead = int(is_dead.sum().item())
    kk = min(k_aux, n_dead) * B
    dead_score = torch.where(is_dead[None, :], hp * n, torch.zeros_like(hp)).clamp_min(0)
    thr = torch.topk(dead_score.flatten(), kk).values[-1]
    aux_kept = dead_score > thr                                                       # strict: ties at the threshold aside
    Wd = sae._w_dec_operand(True).float()
    recon = val @ Wd + sae.b_D.detach()
    assert rel_err(out["reconstructed"], recon) < 1e-4
    w = torch.full((B,), 1.0 / B, device=dev)
    l_rec = ((recon - x).pow(2).sum(-1) * w).sum()
    aux_val = torch.where(aux_kept, hp, torch.zeros_like(hp))
    resid = (x - recon) - aux_val @ Wd
    l_aux = alpha * (resid.pow(2).sum(-1) * w).sum()
    assert abs(out["l_rec"].item() - l_rec.item()) < 1e-4 * l_rec.item()
    assert abs(out["l_aux"].item() - l_aux.item()) < 1e-3 * l_aux.item()            # a handful of threshold ties may differ
    out["loss"].backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in sae.parameters())
    # gradient of the decoder bias: column sums of d loss / d recon, with the residual carrying gradient
    g_recon = 2.0 * w[:, None] * (recon - x) - 2.0 * alpha * w[:, None] * resid
    assert rel_err(sae.b_D.grad, g_recon.sum(0)) < 1e-3
    # dead features only ever receive aux gradient rows; live unselected features none at all
    untouched = ~(kept.any(0) | (is_dead & (dead_score > 0).any(0)))
    assert torch.all(sae.W_D.grad[untouched] == 0)


def test_reference_cpu_configuration_full_size_against_oracle(pkg, oracle, dev):
    """The configuration the reference's CPU path runs: d=768, F=6144, k=32, 4096 tokens, fp32, one step with
    Adam (lr 4e-4), against the oracle itself (its encoder product takes the kernel's forward values so that
    last-bit differences of the two GEMMs cannot flip a selection)."""
    from lm_saes_amd import synthetic

    d, F, k, B = 768, 6144, 32, 4096
    x = synthetic.activations(B, d, 16, seed=4)
    w = synthetic.sae_weights(d, F, x, seed=4)
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk", top_k=k,
                        norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    synthetic.load_weights(sae, *[t.to(dev) for t in w])
    ref = oracle.SAEOracle(d, F, act_fn="topk", top_k=k, sparsity_include_decoder_norm=True)
    synthetic.load_weights(ref, *w)
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long)}
    gb = {k_: v.to(dev) for k_, v in batch.items()}
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=4e-4, model=sae)
    ropt = oracle.make_adam(ref, lr=4e-4)
    out = sae.compute_loss(gb)
    out["loss"].backward()
    pre = pkg.ops.encoder_gemm(gb["in"].contiguous(), sae._w_enc_operand(False), torch.float32).cpu()

    class Sub(torch.autograd.Function):
        @staticmethod
        def forward(ctx, xx, W):
            ctx.save_for_backward(xx, W)
            return pre.clone()

        @staticmethod
        def backward(ctx, gg):
            xx, W = ctx.saved_tensors
            return gg @ W.t(), xx.t() @ gg

    def encode_sub(xx, return_hidden_pre=False, **_):
        hp = (Sub.apply(xx, ref.W_E) + ref.b_E) * ref.decoder_norm()
        fa = ref.activation_function(hp) / ref.decoder_norm()
        return (fa, hp / ref.decoder_norm()) if return_hidden_pre else fa

    ref.encode = encode_sub
    want = ref.compute_loss(batch)
    want["loss"].backward()
    assert torch.equal((out["feature_acts"] != 0).cpu(), want["feature_acts"] != 0)          # bit-exact index sets
    assert rel_err(out["feature_acts"].cpu(), want["feature_acts"]) < 1e-5
    assert rel_err(out["reconstructed"].cpu(), want["reconstructed"]) < 1e-5
    assert abs(out["loss"].item() - want["loss"].item()) < 1e-5 * want["loss"].item()
    opt.materialize_grads()
    for name in ("W_E", "b_E", "W_D", "b_D"):
        assert rel_err(getattr(sae, name).grad.cpu(), getattr(ref, name).grad) < 1e-5, name
    before = {n_: p.detach().clone() for n_, p in ref.named_parameters()}
    grads = {n_: p.grad.detach().clone() for n_, p in ref.named_parameters()}
    opt.step(); ropt.step()
    for n_, p in sae.named_parameters():
        move, want_move = p.detach().cpu() - before[n_], dict(ref.named_parameters())[n_].detach() - before[n_]
        # the first Adam step is g / (|g| + eps): where |g| is within rounding of zero the two sides may differ in
        # sign, so the move is compared where the gradient is resolved, and bounded by lr everywhere
        resolved = grads[n_].abs() > 1e-3 * grads[n_].abs().max()
        assert (move - want_move)[resolved].abs().max().item() < 2e-3 * 4e-4, n_
        assert move.abs().max().item() <= 4e-4 * (1 + 1e-5), n_


def _amp(on: bool):
    """bf16 autocast (the benchmark configurations' precision: fp32 parameters, bf16 matmul operands) or nothing."""
    import contextlib

    return torch.autocast("cuda", dtype=torch.bfloat16) if on else contextlib.nullcontext()


@pytest.mark.parametrize("amp", [False, True], ids=["fp32", "bf16_autocast"])
def test_clt_shape_fused_step_against_dense_path(pkg, dev, amp):
    """CLT, 12 layers, d=768, 12288 features per layer, k=64 per layer, 2048 tokens: the prefix decode of the
    concatenated sparse code against the module's dense path (78 library GEMMs), forward and backward; in fp32
    (1e-4) and under bf16 autocast as the benchmark runs it (2e-2: the library's matmuls round their bf16 outputs,
    the kernels keep fp32 sums)."""
    from lm_saes_amd import synthetic

    tol_out, tol_loss, tol_grad = (2e-2, 2e-2, 2e-2) if amp else (1e-4, 1e-5, 2e-4)

    L, d, F, k, B = 12, 768, 12288, 64, 2048
    hin, hout = [f"in{l}" for l in range(L)], [f"out{l}" for l in range(L)]
    cfg = pkg.CLTConfig(hook_points_in=hin, hook_points_out=hout, d_model=d, expansion_factor=F / d, act_fn="topk", top_k=k,
                        norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda", dtype=torch.float32)
    torch.manual_seed(0)
    clt = pkg.CrossLayerTranscoder(cfg)
    clt.init_parameters()
    g = torch.Generator(device=dev).manual_seed(4)
    batch = {"tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    for l in range(L):
        x = synthetic.activations(B, d, 16, seed=4 + l).to(dev)
        batch[hin[l]], batch[hout[l]] = x, torch.tanh(x @ (torch.randn(d, d, device=dev, generator=g) / d ** 0.5))
    with _amp(amp):
        out = clt.compute_loss(batch)
    code = out["sparse_code"]
    assert torch.all(code.row_nnz == L * k)
    out["loss"].backward()
    fused = {n_: p.grad.clone() for n_, p in clt.named_parameters()}
    for p in clt.parameters():
        p.grad = None
    # dense path on the kernel's own selection (a second encoder product by the library GEMM would differ in
    # the last bit and could flip near-ties): decode through the 78 dense blocks, autograd for the decoder side
    xs, _, _ = clt.prepare_input(batch)
    label = clt.prepare_label(batch)
    feature_acts = out["feature_acts"].clone().requires_grad_()
    kept = feature_acts.detach() != 0
    assert int(kept.sum().item()) == B * L * k
    clt.sparse_api_decode = False      # the module's dense products: one 2-D library product per output layer
    with _amp(amp):
        recon = clt.decode(feature_acts)
        loss = (recon.float() - label).pow(2).sum(-1).mean()
    assert rel_err(out["reconstructed"], recon) < tol_out
    assert abs(out["loss"].item() - loss.item()) < tol_loss * loss.item()
    loss.backward()
    for n_, p in clt.named_parameters():
        if n_.startswith("W_D") or n_.startswith("b_D"):
            assert rel_err(fused[n_], p.grad) < tol_grad, n_
    # encoder side: TopK passes the gradient of kept entries unchanged (the decoder-norm factors cancel)
    d_pre = feature_acts.grad * kept
    assert rel_err(fused["W_E"], torch.einsum("bld,blf->ldf", xs, d_pre)) < tol_grad
    assert rel_err(fused["b_E"], d_pre.sum(0)) < tol_grad
    # and the values the code holds are the unscaled pre-activations of its own encoder product
    if amp:
        hp = torch.stack([pkg.ops.encoder_gemm(pkg.ops.cast_bf16(xs[:, l].contiguous()), clt._w_enc_operand(True)[l],
                                               torch.bfloat16).float() for l in range(L)], dim=1) + clt.b_E.detach()
    else:
        hp = torch.stack([pkg.ops.encoder_gemm(xs[:, l].contiguous(), clt._w_enc_operand(False)[l], torch.float32)
                          for l in range(L)], dim=1) + clt.b_E.detach()
    assert rel_err(feature_acts.detach()[kept], hp[kept]) < 1e-6
    score = (hp * clt._norm_per_feature_nograd()).view(B * L, F)
    check_threshold_selection(score, kept.view(B * L, F), per_row=True)


def test_lorsa_shape_fused_step_against_dense_path(pkg, dev):
    """Lorsa, d=768, 16 x 1024 tokens, 64 query/key heads of width 64, 8192 value/output heads, k=64, fp32:
    the sparse tail (select, sparse decode, W_O rows, scatter of the value gradients) against the dense path."""
    from lm_saes_amd import synthetic

    nb, s, d, F, h, dq, k = 16, 1024, 768, 8192, 64, 64, 64
    cfg = pkg.LorsaConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, n_qk_heads=h,
                          d_qk_head=dq, n_ctx=s, rotary_dim=dq, positional_embedding_type="none", act_fn="topk", top_k=k,
                          norm_activation="inference", device="cuda", dtype=torch.float32)
    torch.manual_seed(0)
    m = pkg.LowRankSparseAttention(cfg)
    m.init_parameters()
    # both paths scale by the same norm vector (the library's norm and the row-norm kernel may differ in the last
    # bit, which could flip a selection between two nearly equal scores)
    m._decoder_norm_nograd = lambda: m.decoder_norm().detach()
    x = synthetic.activations(nb * s, d, 64, seed=4).to(dev).view(nb, s, d)
    y = torch.roll(x, 1, dims=1) * 0.5
    batch = {"in": x, "out": y, "tokens": torch.zeros(nb, s, dtype=torch.long, device=dev)}
    out = m.compute_loss(batch)
    assert "sparse_code" in out and torch.all(out["sparse_code"].row_nnz == k)
    out["loss"].backward()
    fused = {n_: p.grad.clone() for n_, p in m.named_parameters()}
    for p in m.parameters():
        p.grad = None
    want = pkg.SparseDictionary.compute_loss(m, batch)          # the generic dense op sequence
    assert torch.equal(want["feature_acts"] != 0, out["feature_acts"] != 0)
    assert rel_err(out["reconstructed"], want["reconstructed"]) < 1e-4
    assert abs(out["loss"].item() - want["loss"].item()) < 1e-5 * want["loss"].item()
    want["loss"].backward()
    scale = max(p.grad.abs().max().item() for p in m.parameters())
    for n_, p in m.named_parameters():
        if p.grad.abs().max().item() < 1e-5 * scale:        # analytically zero (key bias): rounding noise on both sides
            continue
        assert rel_err(fused[n_], p.grad) < 2e-4, n_


@pytest.mark.parametrize("rotary", [None, (16, False), (64, True)], ids=["no_rotary", "rotary16_halves", "rotary64_adjacent"])
def test_lorsa_shape_bf16_attention_kernels_against_library_path(pkg, dev, rotary):
    """Lorsa at the benchmark shape under bf16 autocast (d=768, 16 x 1024 tokens, 64 query/key heads of width 64, 8192
    value/output heads in groups of 128, k=64): projections and causal mixing on the GEMM / attention kernels against
    the same module with those stages on torch's library routines (einsum + scaled_dot_product_attention).
    hidden_pre agrees within the bf16 bound; the selection is exactly the k largest of the kernel path's own scores;
    loss and gradients agree within the bound although a few near-tied selections differ between the two paths."""
    from lm_saes_amd import synthetic

    nb, s, d, F, h, dq, k = 16, 1024, 768, 8192, 64, 64, 64
    # with rotary embeddings: the first 16 elements of a head in half-split pairs (the reference's own example,
    # examples/train_pythia_lorsa_topk.py:32-34), or the whole head in adjacent pairs
    pos = dict(positional_embedding_type="none", rotary_dim=dq) if rotary is None else dict(
        positional_embedding_type="rotary", rotary_dim=rotary[0], rotary_adjacent_pairs=rotary[1])
    cfg = pkg.LorsaConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, n_qk_heads=h,
                          d_qk_head=dq, n_ctx=s, act_fn="topk", top_k=k, norm_activation="inference", device="cuda",
                          dtype=torch.float32, **pos)
    torch.manual_seed(0)
    m = pkg.LowRankSparseAttention(cfg)
    m.init_parameters()
    with torch.no_grad():
        for b_ in (m.b_Q, m.b_K, m.b_V):
            b_.normal_(0, 0.05)
    m._decoder_norm_nograd = lambda: m.decoder_norm().detach()
    x = synthetic.activations(nb * s, d, 64, seed=4).to(dev).view(nb, s, d)
    y = torch.roll(x, 1, dims=1) * 0.5
    batch = {"in": x, "out": y, "tokens": torch.zeros(nb, s, dtype=torch.long, device=dev)}
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    with _amp(True):
        out = m.compute_loss(batch)
    out["loss"].backward()
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    assert {"attention_fwd", "attention_bwd"} <= set(timer.records), set(timer.records)
    assert ({"rotary_fwd", "rotary_bwd_t"} <= set(timer.records)) == (rotary is not None)
    fused = {n_: p.grad.clone() for n_, p in m.named_parameters()}
    hp = out["hidden_pre"]
    kept = dense_mask(out["sparse_code"])
    assert torch.all(out["sparse_code"].row_nnz == k)
    check_threshold_selection((hp.view(nb * s, F) * m._decoder_norm_nograd()), kept, per_row=True)
    loss_f = out["loss"].item()
    del out
    for p in m.parameters():
        p.grad = None
    m.use_mix_kernels = False
    with _amp(True):
        want = m.compute_loss(batch)
    assert rel_err(hp, want["hidden_pre"]) < 2e-2
    same = (kept == dense_mask(want["sparse_code"])).all(dim=1).float().mean().item()
    assert same > 0.9, same                                   # near-ties at the k-th place may fall either way
    assert abs(loss_f - want["loss"].item()) < 2e-2 * want["loss"].item()
    want["loss"].backward()
    scale = max(p.grad.abs().max().item() for p in m.parameters())
    errs = {}
    for n_, p in m.named_parameters():
        if p.grad.abs().max().item() < 1e-2 * scale:           # analytically zero (key bias) or below the step's bf16 noise
            continue
        errs[n_] = ((fused[n_].double() - p.grad.double()).norm() / p.grad.double().norm()).item()
    assert all(e < 5e-2 for e in errs.values()), errs


@pytest.mark.parametrize("amp", [False, True], ids=["fp32", "bf16_autocast"])
def test_jumprelu_shape_fused_step_against_dense_path(pkg, dev, amp):
    """JumpReLU SAE d=4096, F=131072, 4096 tokens, threshold 0.001, window 0.001, tanh penalty 5: the fused
    element-wise kernels and the step's own dense products against the generic dense op sequence (library matmuls)
    fed the same encoder product; in fp32 and under bf16 autocast as the benchmark runs it."""
    d, F, B = 4096, 131072, 4096
    tol_loss, tol_grad = (2e-2, 2e-2) if amp else (1e-5, 2e-4)
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="jumprelu",
                        jumprelu_threshold_window=0.001, norm_activation="inference", sparsity_include_decoder_norm=True,
                        device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    g = torch.Generator(device=dev).manual_seed(4)
    x = torch.randn(B, d, device=dev, generator=g)
    x[:, [7, 1029, 2050, 3071]] *= 50.0
    with torch.no_grad():
        wt = sae.W_E.t()
        wt.uniform_(-1.0 / d ** 0.5, 1.0 / d ** 0.5, generator=g)
        sae.W_D.copy_(wt / wt.norm(dim=1, keepdim=True))
        sae.b_E.zero_()
        sae.b_D.copy_(x.mean(0))
        sae.activation_function.log_jumprelu_threshold.fill_(math.log(0.001))
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    kw = dict(sparsity_loss_type="tanh", l1_coefficient=5.0)
    opt = pkg.HipAdam(sae.get_parameters()[0]["params"], lr=1e-4, model=sae) if amp else None   # deferred bf16 gradients, as in the benchmark
    with _amp(amp):
        out = sae.compute_loss(batch, **kw)
    out["loss"].backward()
    if opt is not None:
        pkg.optim.fold_row_grad_coef(list(sae.parameters()))    # what the backward left for the optimiser -> .grad
        sae.defer_weight_grads = False
    fused = {n_: p.grad.clone() for n_, p in sae.named_parameters()}
    acts_mask, loss_f, l_s_f = out["feature_acts"] != 0, out["loss"].item(), out["l_s"].mean().item()
    pre = (out["hidden_pre"] - sae.b_E.detach()).to(torch.bfloat16 if amp else torch.float32)
    del out
    for p in sae.parameters():
        p.grad = None

    class Sub(torch.autograd.Function):      # the kernel's encoder product as the forward value, matmul backward
        @staticmethod
        def forward(ctx, xx, W):
            ctx.save_for_backward(xx, W)
            return pre.clone()

        @staticmethod
        def backward(ctx, gg):
            xx, W = ctx.saved_tensors
            gg = gg.float()
            return gg @ W.t(), xx.t() @ gg

    sae._matmul_enc = lambda xx, W: Sub.apply(xx, W)
    with _amp(amp):
        want = pkg.SparseDictionary.compute_loss(sae, batch, **kw)
    assert torch.equal(want["feature_acts"] != 0, acts_mask)
    assert 0.3 < acts_mask.float().mean().item() < 0.7               # about half of all features fire at this threshold
    assert abs(loss_f - want["loss"].item()) < tol_loss * want["loss"].item()
    assert abs(l_s_f - want["l_s"].mean().item()) < tol_loss * want["l_s"].mean().item()
    want["loss"].backward()
    for n_, p in sae.named_parameters():
        assert rel_err(fused[n_], p.grad) < tol_grad, n_
    assert (fused["activation_function.log_jumprelu_threshold"] != 0).float().mean().item() > 0.5


# ---- the full-size steps against the CPU oracle on a few of their tokens ----------------------------------------------------
# A token's forward pass does not depend on the batch's other tokens (per-token TopK, JumpReLU) or, for Lorsa, on other
# sequences, so the oracle can afford the full dictionaries on a handful of tokens: the step runs on the GPU at its real
# shape and the oracle recomputes some of its rows from the same parameters.

def _copy_to_oracle(ref, model):
    src = dict(model.named_parameters())
    with torch.no_grad():
        for n_, p in ref.named_parameters():
            p.copy_(src[n_].detach().to("cpu", p.dtype))


def test_clt_shape_rows_against_the_oracle(pkg, oracle, dev):
    """C4 in fp32 (12 layers, d=768, 12288 features per layer, k=64, 2048 tokens): 32 of the tokens through the oracle's
    encode (einsum + per-layer TopK) and its 78-block decode.  The two encoder products add in different orders, so an
    entry within rounding of the k-th value may fall either way: such (token, layer) rows are counted and must be rare;
    everything else agrees to fp32 rounding."""
    import importlib

    from lm_saes_amd import synthetic

    vo = importlib.import_module("oracle.variants_oracle")
    L, d, F, k, B = 12, 768, 12288, 64, 2048
    hin, hout = [f"in{l}" for l in range(L)], [f"out{l}" for l in range(L)]
    cfg = pkg.CLTConfig(hook_points_in=hin, hook_points_out=hout, d_model=d, expansion_factor=F / d, act_fn="topk", top_k=k,
                        norm_activation="inference", sparsity_include_decoder_norm=True, device="cuda", dtype=torch.float32)
    torch.manual_seed(0)
    clt = pkg.CrossLayerTranscoder(cfg)
    clt.init_parameters()
    g = torch.Generator(device=dev).manual_seed(4)
    batch = {"tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    for l in range(L):
        x = synthetic.activations(B, d, 16, seed=4 + l).to(dev)
        batch[hin[l]], batch[hout[l]] = x, torch.tanh(x @ (torch.randn(d, d, device=dev, generator=g) / d ** 0.5))
    with torch.no_grad():
        out = clt.compute_loss(batch)
    assert "sparse_code" in out, "the kernel path did not run"
    rows = torch.arange(5, B, 64, device=dev)
    ref = vo.CLTOracle(L, d, F, act_fn="topk", top_k=k, sparsity_include_decoder_norm=True)
    _copy_to_oracle(ref, clt)
    sub = {n_: v[rows].cpu() for n_, v in batch.items()}
    with torch.no_grad():
        want = ref.compute_loss(sub, hin, hout)
    # activations are [tokens, layers, features], reconstructions [layers, tokens, d] (the reference's layouts)
    assert tuple(out["feature_acts"].shape) == (B, L, F) and tuple(out["reconstructed"].shape) == (L, B, d)
    assert tuple(want["feature_acts"].shape) == (len(rows), L, F) and tuple(want["reconstructed"].shape) == (L, len(rows), d)
    got_acts, got_recon = out["feature_acts"][rows].cpu(), out["reconstructed"][:, rows].cpu().transpose(0, 1)
    want_recon = want["reconstructed"].transpose(0, 1)
    same_rows = ((got_acts != 0) == (want["feature_acts"] != 0)).all(-1)            # [32, L]
    assert same_rows.float().mean().item() > 0.99, same_rows.float().mean().item()
    assert rel_err(got_acts[same_rows], want["feature_acts"][same_rows]) < 1e-5
    # a token's reconstruction of layer j reads its layers 0..j: compared where all of those rows hold the same entries
    prefix_ok = same_rows.cumprod(dim=1).bool()                                       # [32, L]
    assert prefix_ok.float().mean().item() > 0.9
    assert rel_err(got_recon[prefix_ok], want_recon[prefix_ok]) < 1e-4


def test_lorsa_shape_sequence_against_the_oracle(pkg, oracle, dev):
    """C5 under bf16 autocast (the attention, GEMM and select kernels): one of the 16 sequences through the fp32 oracle
    (explicit causal softmax per head, dense TopK, dense decode), with the oracle's activation replaced by the kernel
    path's own selection so that entries near the k-th value cannot fall differently; hidden_pre, the kept values and
    the reconstruction agree at the bf16 bound."""
    import importlib

    from lm_saes_amd import synthetic

    vo = importlib.import_module("oracle.variants_oracle")
    nb, s, d, F, h, dq, k = 16, 1024, 768, 8192, 64, 64, 64
    cfg = pkg.LorsaConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, n_qk_heads=h,
                          d_qk_head=dq, n_ctx=s, rotary_dim=dq, positional_embedding_type="none", act_fn="topk", top_k=k,
                          norm_activation="inference", device="cuda", dtype=torch.float32)
    torch.manual_seed(0)
    m = pkg.LowRankSparseAttention(cfg)
    m.init_parameters()
    with torch.no_grad():
        for b_ in (m.b_Q, m.b_K, m.b_V):
            b_.normal_(0, 0.05)
    x = synthetic.activations(nb * s, d, 64, seed=4).to(dev).view(nb, s, d)
    y = torch.roll(x, 1, dims=1) * 0.5
    batch = {"in": x, "out": y, "tokens": torch.zeros(nb, s, dtype=torch.long, device=dev)}
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    with torch.no_grad(), _amp(True):
        out = m.compute_loss(batch)
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    assert "attention_fwd" in timer.records, set(timer.records)
    seq = 11
    ref = vo.LorsaOracle(d_model=d, d_sae=F, n_qk_heads=h, d_qk_head=dq, n_ctx=s, act_fn="topk", top_k=k,
                         positional_embedding_type="none")
    _copy_to_oracle(ref, m)
    for name, width in (("feature_acts", F), ("hidden_pre", F), ("reconstructed", d)):
        assert tuple(out[name].shape) == (nb, s, width), (name, tuple(out[name].shape))
    kept = (out["feature_acts"][seq] != 0).cpu()
    assert torch.all(kept.sum(-1) == k)
    ref.activation_function = lambda hp: hp * kept.to(hp.dtype).reshape(hp.shape)
    sub = {"in": x[seq:seq + 1].cpu(), "out": y[seq:seq + 1].cpu(), "tokens": torch.zeros(1, s, dtype=torch.long)}
    with torch.no_grad():
        want = ref.compute_loss(sub)
    assert rel_err(out["hidden_pre"][seq].cpu(), want["hidden_pre"][0]) < 2e-2
    assert rel_err(out["feature_acts"][seq].cpu(), want["feature_acts"][0]) < 2e-2
    assert rel_err(out["reconstructed"][seq].cpu(), want["reconstructed"][0]) < 2e-2
    # and the kernel's selection is the oracle's own on all but near-tied entries
    hp = want["hidden_pre"][0] * ref.decoder_norm()
    own = torch.zeros_like(kept).scatter_(1, hp.topk(k, dim=-1).indices, True)
    assert (own & kept).sum().item() > 0.9 * kept.sum().item()


def test_jumprelu_shape_rows_against_the_oracle(pkg, oracle, dev):
    """C3 in fp32 (d=4096, F=131072, 4096 tokens, threshold and window 0.001, tanh penalty): 48 of the tokens through the
    oracle with the full dictionary.  A pre-activation within rounding of its threshold may fall either way between the two
    encoder products: such entries are counted (a few of 6 M) and carry values of the threshold's size; activations,
    reconstruction and the per-token penalty agree to fp32 rounding."""
    d, F, B = 4096, 131072, 4096
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="jumprelu",
                        jumprelu_threshold_window=0.001, norm_activation="inference", sparsity_include_decoder_norm=True,
                        device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    g = torch.Generator(device=dev).manual_seed(4)
    x = torch.randn(B, d, device=dev, generator=g)
    x[:, [7, 1029, 2050, 3071]] *= 50.0
    with torch.no_grad():
        wt = sae.W_E.t()
        wt.uniform_(-1.0 / d ** 0.5, 1.0 / d ** 0.5, generator=g)
        sae.W_D.copy_(wt / wt.norm(dim=1, keepdim=True))
        sae.b_E.zero_()
        sae.b_D.copy_(x.mean(0))
        sae.activation_function.log_jumprelu_threshold.fill_(math.log(0.001))
    batch = {"in": x, "out": x, "tokens": torch.zeros(B, dtype=torch.long, device=dev)}
    kw = dict(sparsity_loss_type="tanh", l1_coefficient=5.0)
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    with torch.no_grad():
        out = sae.compute_loss(batch, **kw)
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    assert "jumprelu_fwd" in timer.records, set(timer.records)
    rows = torch.arange(3, B, 86, device=dev)
    assert tuple(out["feature_acts"].shape) == (B, F) and tuple(out["reconstructed"].shape) == (B, d) and tuple(out["l_s"].shape) == (B,)
    got_acts, got_recon, got_ls = out["feature_acts"][rows].cpu(), out["reconstructed"][rows].cpu(), out["l_s"][rows].cpu()
    del out
    ref = oracle.SAEOracle(d, F, act_fn="jumprelu", jumprelu_threshold_window=0.001, sparsity_include_decoder_norm=True)
    _copy_to_oracle(ref, sae)
    sub = {"in": x[rows].cpu(), "out": x[rows].cpu(), "tokens": torch.zeros(len(rows), dtype=torch.long)}
    with torch.no_grad():
        want = ref.compute_loss(sub, **kw)
    differ = (got_acts != 0) != (want["feature_acts"] != 0)
    assert differ.sum().item() <= 1e-5 * differ.numel(), differ.sum().item()
    assert 0.3 < (got_acts != 0).float().mean().item() < 0.7
    # an entry that fell the other way holds a value of the threshold's size on one side and 0 on the other
    both = got_acts - want["feature_acts"]
    assert both[differ].abs().max().item() < 0.05 if differ.any() else True
    assert rel_err(torch.where(differ, 0, got_acts), torch.where(differ, 0, want["feature_acts"])) < 1e-5
    assert rel_err(got_recon, want["reconstructed"]) < 1e-4
    assert rel_err(got_ls, want["l_s"]) < 1e-4
