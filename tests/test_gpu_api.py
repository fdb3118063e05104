"""The module API (`encode` / `decode` / `forward`, the activation callables) and the kernel operators of the
reference's `kernels` package, on the HIP path, against the CPU oracle and dense arithmetic.

The encoder product of `encode()` is the GEMM kernel, the TopK / BatchTopK activations are the select kernels, and
with `cfg.use_triton_kernel` `decode()` switches to the sparse decoder kernel on sparse-enough activations
(models/sae.py:355-367).  A KernelTimer records which library calls ran, so a silent library fallback fails the test.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5
GRAD_TOL = 1e-4


def rel_err(got, want):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def make_pair(pkg, oracle, dev, act_fn, d=64, F=512, k=8, B=96, seed=0, include_norm=True, glu=False, triton=False):
    from lm_saes_amd import synthetic

    x = synthetic.activations(B, d, 8, seed)
    w = synthetic.sae_weights(d, F, x, seed)
    g = torch.Generator().manual_seed(seed + 1)
    W_D = (w[2] * (0.5 + torch.rand(F, 1, generator=g))).contiguous()
    w = (w[0], 0.02 * torch.randn(F, generator=g), W_D, w[3])
    cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn=act_fn, top_k=k,
                        jumprelu_threshold_window=0.3, norm_activation="inference", sparsity_include_decoder_norm=include_norm,
                        use_glu_encoder=glu, use_triton_kernel=triton, device="cuda", dtype=torch.float32)
    sae = pkg.SparseAutoEncoder(cfg)
    synthetic.load_weights(sae, *[t.to(dev) for t in w])
    ref = oracle.SAEOracle(d, F, act_fn=act_fn, top_k=k, jumprelu_threshold_window=0.3,
                           sparsity_include_decoder_norm=include_norm, use_glu_encoder=glu)
    synthetic.load_weights(ref, *w)
    with torch.no_grad():
        if act_fn == "jumprelu":
            t = torch.log(0.02 + 0.3 * torch.rand(F, generator=g))
            sae.activation_function.log_jumprelu_threshold.copy_(t.to(dev))
            ref.activation_function.log_jumprelu_threshold.copy_(t)
        if glu:
            wg, bg = torch.randn(d, F, generator=g) / d ** 0.5, 0.1 * torch.randn(F, generator=g)
            sae.W_E_glu.copy_(wg.to(dev)); sae.b_E_glu.copy_(bg.to(dev))
            ref.W_E_glu.copy_(wg); ref.b_E_glu.copy_(bg)
    return sae, ref, x


def named_grads(m):
    return {n.replace("activation_function.", ""): p.grad for n, p in m.named_parameters()}


@pytest.mark.parametrize("act_fn", ["relu", "jumprelu", "topk", "batchtopk"])
@pytest.mark.parametrize("triton", [False, True])
def test_encode_decode_forward_run_on_the_kernels_and_match_the_oracle(pkg, oracle, dev, act_fn, triton):
    sae, ref, x = make_pair(pkg, oracle, dev, act_fn, seed=3, triton=triton)
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    acts, hidden_pre = sae.encode(x.to(dev), return_hidden_pre=True)
    recon = sae.decode(acts)
    loss = (recon - x.to(dev)).pow(2).sum(-1).mean()
    loss.backward()
    out = sae.forward(x.to(dev))
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    ran = set(timer.records)
    assert "encoder_gemm" in ran, ran
    if act_fn == "topk":
        assert "select_topk_row" in ran, ran
    if act_fn == "batchtopk":
        assert "select_topk_batch" in ran, ran
    want_acts, want_hp = ref.encode(x, return_hidden_pre=True)
    want_recon = ref.decode(want_acts)
    ((want_recon - x).pow(2).sum(-1).mean()).backward()
    assert torch.equal((acts != 0).cpu(), want_acts != 0), "kept sets differ"
    assert rel_err(acts, want_acts) < FP32_TOL and rel_err(hidden_pre, want_hp) < FP32_TOL
    assert rel_err(recon, want_recon) < FP32_TOL and rel_err(out, want_recon) < FP32_TOL
    got, exp = named_grads(sae), named_grads(ref)
    for n, g_ in exp.items():
        if g_ is None:
            continue
        assert got[n] is not None and rel_err(got[n], g_) < GRAD_TOL, (n, rel_err(got[n], g_))
    # the gate of models/sae.py:355-367: max L0 < d_sae * (1 - 0.996) = 2.05 here, so these activations stay dense
    assert "sparse_decode_fwd" not in ran


def test_decode_takes_the_sparse_kernel_below_the_sparsity_gate(pkg, oracle, dev):
    """k = 2 of d_sae = 1024: max L0 = 2 < 1024 * 0.004 = 4.1, so `use_triton_kernel` sends decode() to the sparse
    kernel; same values and gradients as the dense product."""
    sae, ref, x = make_pair(pkg, oracle, dev, "topk", d=64, F=1024, k=2, B=80, seed=5, triton=True)
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    acts = sae.encode(x.to(dev))
    recon = sae.decode(acts)
    (recon - x.to(dev)).pow(2).sum(-1).mean().backward()
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    assert {"sparse_decode_fwd", "dense_to_code", "sparse_decode_bwd_dval", "sparse_grad_rows[f32 dense]"} <= set(timer.records), set(timer.records)
    want_acts = ref.encode(x)
    want_recon = ref.decode(want_acts)
    ((want_recon - x).pow(2).sum(-1).mean()).backward()
    assert torch.equal((acts != 0).cpu(), want_acts != 0)
    assert rel_err(recon, want_recon) < FP32_TOL
    got, exp = named_grads(sae), named_grads(ref)
    for n in ("W_E", "b_E", "W_D", "b_D"):
        assert rel_err(got[n], exp[n]) < GRAD_TOL, (n, rel_err(got[n], exp[n]))
    # an all-zero activation matrix stays on the dense product (the kernel path needs at least one entry)
    zero = torch.zeros(16, 1024, device=dev)
    assert torch.equal(sae.decode(zero), sae.b_D.detach().expand(16, -1))


@pytest.mark.parametrize("loss_type,kw", [("power", dict(p=1)), ("power", dict(p=2)), ("tanh-quad", dict(frequency_scale=0.05)),
                                           ("tanh", dict())])
@pytest.mark.parametrize("act_fn", ["relu", "jumprelu"])
def test_sparsity_losses_match_the_oracle(pkg, oracle, dev, loss_type, kw, act_fn):
    """models/sparse_dictionary.py:888-925: the three sparsity penalties (with the decoder-norm weighting) through
    compute_loss + backward on the GPU."""
    sae, ref, x = make_pair(pkg, oracle, dev, act_fn, seed=7)
    g = torch.Generator().manual_seed(8)
    batch = {"in": x, "out": x + 0.1 * torch.randn(x.shape, generator=g), "tokens": torch.zeros(x.shape[0], dtype=torch.long),
             "mask": (torch.rand(x.shape[0], generator=g) > 0.25).float()}
    args = dict(sparsity_loss_type=loss_type, l1_coefficient=0.05, tanh_stretch_coefficient=2.0, **kw)
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    out = sae.compute_loss({k_: v.to(dev) for k_, v in batch.items()}, **args)
    want = ref.compute_loss(batch, **args)
    out["loss"].backward(); want["loss"].backward()
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    if act_fn == "jumprelu":    # the step's own route: activation kernel each way, five products on the GEMM kernel
        assert {"jumprelu_fwd", "jumprelu_bwd"} <= set(timer.records) and len(timer.records["encoder_gemm"]) == 5, set(timer.records)
    for key in ("loss", "l_rec", "l_s", "feature_acts", "reconstructed"):
        assert rel_err(out[key], want[key]) < FP32_TOL, key
    got, exp = named_grads(sae), named_grads(ref)
    for n, g_ in exp.items():
        if g_ is not None:
            assert got[n] is not None and rel_err(got[n], g_) < GRAD_TOL, (n, rel_err(got[n], g_))


@pytest.mark.parametrize("act_fn", ["relu", "topk"])
def test_glu_encoder_matches_the_oracle(pkg, oracle, dev, act_fn):
    """models/sae.py:326-331: hidden_pre * sigmoid(x @ W_E_glu + b_E_glu); both products on the GEMM kernel."""
    sae, ref, x = make_pair(pkg, oracle, dev, act_fn, seed=9, glu=True)
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    out = sae.compute_loss({"in": x.to(dev), "out": x.to(dev), "tokens": torch.zeros(x.shape[0], device=dev)})
    out["loss"].backward()
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    assert len(timer.records["encoder_gemm"]) >= 2
    want = ref.compute_loss({"in": x, "out": x, "tokens": torch.zeros(x.shape[0])})
    want["loss"].backward()
    assert torch.equal((out["feature_acts"] != 0).cpu(), want["feature_acts"] != 0)
    for key in ("loss", "feature_acts", "hidden_pre", "reconstructed"):
        assert rel_err(out[key], want[key]) < FP32_TOL, key
    got, exp = named_grads(sae), named_grads(ref)
    for n, g_ in exp.items():
        assert got[n] is not None and rel_err(got[n], g_) < GRAD_TOL, (n, rel_err(got[n], g_))


def test_batchtopk_callable_is_the_select_kernel(pkg, oracle, dev):
    """`sae.activation_function` of a BatchTopK model (models/sparse_dictionary.py:761-794): exactly the k * B largest
    positive entries of the batch, ties to the lowest flattened index, 2-D and 3-D inputs, gradient on kept entries."""
    sae, ref, _ = make_pair(pkg, oracle, dev, "batchtopk", F=512, k=8)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(40, 512, generator=g).round(decimals=1)            # one decimal: many exact ties
    xg = x.to(dev).requires_grad_()
    y = sae.activation_function(xg)
    want = ref.activation_function(x)
    assert torch.equal(y.detach().cpu(), want)
    assert int((y != 0).sum()) == 8 * 40
    y.sum().backward()
    assert torch.equal(xg.grad.cpu(), (want != 0).float())
    x3 = x.view(5, 8, 512)
    assert torch.equal(sae.activation_function(x3.to(dev)).cpu(), ref.activation_function(x3))


# ---- the kernel operators ---------------------------------------------------------------------------

@pytest.mark.parametrize("B,F,dtype", [(7, 100, torch.float32), (33, 4096, torch.float32), (5, 5000, torch.bfloat16),
                                       (64, 2048 + 8, torch.bfloat16), (3, 131072, torch.bfloat16)])
def test_dense_to_code_lists_the_nonzeros_in_order(pkg, dev, B, F, dtype):
    g = torch.Generator().manual_seed(B + F)
    x = torch.randn(B, F, generator=g) * (torch.rand(B, F, generator=g) < 0.03)
    x[B // 2] = 0                                   # an empty row
    x[0, 0], x[0, F - 1] = 1.5, -2.0                # first and last column, a negative value
    x[-1, 1] = -0.0                                 # negative zero is zero
    x = x.to(dtype)
    code = pkg.ops.dense_to_code(x.to(dev))
    nz = x != 0
    assert torch.equal(code.row_nnz.cpu().long(), nz.sum(1))
    assert torch.equal(code.row_off.cpu(), torch.cumsum(nz.sum(1), 0) - nz.sum(1))
    rows, cols = nz.nonzero(as_tuple=True)          # row-major order = ascending column inside a row
    assert code.n_slots == max(int(nz.sum()), 1)
    assert torch.equal(code.idx.cpu().long()[: len(cols)], cols)
    assert torch.equal(code.val.cpu()[: len(cols)], x[rows, cols].float())
    assert torch.equal(code.to_dense().cpu(), x.float())
    # a caller-supplied capacity: nothing is read back, the extra slots stay idx 0 / val 0
    code2 = pkg.ops.dense_to_code(x.to(dev), capacity=int(nz.sum()) + 5)
    assert torch.equal(code2.to_dense().cpu(), x.float()) and torch.all(code2.val[-5:] == 0)


def test_get_sparse_representation_has_the_reference_shape(pkg, dev):
    """kernels/kernels.py:14-58: [B, nnz_max] indices / values, each row's non-zeros first (ascending columns), pad behind."""
    x = torch.tensor([[0.0, 2.0, 0.0, -1.0, 0.0], [0.0, 0.0, 0.0, 0.0, 0.0], [3.0, 4.0, 5.0, 0.0, 0.0]])
    idx, val = pkg.kernels.get_sparse_representation(x.to(dev))
    assert idx.dtype == torch.long and idx.cpu().tolist() == [[1, 3, 0], [0, 0, 0], [0, 1, 2]]
    assert val.cpu().tolist() == [[2.0, -1.0, 0.0], [0.0, 0.0, 0.0], [3.0, 4.0, 5.0]]
    idx, val = pkg.kernels.get_sparse_representation(torch.zeros(2, 4, device=dev))
    assert idx.cpu().tolist() == [[0], [0]] and val.cpu().tolist() == [[0.0], [0.0]]


@pytest.mark.parametrize("weight_form", ["d_sae_by_d_model", "as_the_reference_call_site_passes_it"])
def test_decode_with_hip_spmm_kernel_matches_the_dense_product(pkg, dev, weight_form):
    """kernels/entrypoints.py:16-40 and its self-test recipe (:96-150): sparse activations times a decoder weight,
    forward and both gradients, against the dense product in fp64; 2-D and 3-D activations."""
    g = torch.Generator().manual_seed(21)
    B, F, d = 48, 768, 64
    fa = (torch.randn(B, F, generator=g).abs() * (torch.rand(B, F, generator=g) < 0.02)).requires_grad_()
    W = (torch.randn(F, d, generator=g) / d ** 0.5).requires_grad_()
    up = torch.randn(B, d, generator=g)
    (fa.double() @ W.double() * up.double()).sum().backward()
    fa_g = fa.detach().to(dev).requires_grad_()
    W_g = W.detach().to(dev).requires_grad_()
    arg = W_g if weight_form == "d_sae_by_d_model" else W_g.t().contiguous()
    if weight_form != "d_sae_by_d_model":
        arg.retain_grad()
    out = pkg.kernels.decode_with_triton_spmm_kernel(fa_g, arg)
    assert rel_err(out, fa.detach().double() @ W.detach().double()) < FP32_TOL
    (out * up.to(dev)).sum().backward()
    assert rel_err(fa_g.grad, fa.grad * (fa.detach() != 0)) < GRAD_TOL     # the gradient of the stored entries only
    got_W = W_g.grad if weight_form == "d_sae_by_d_model" else arg.grad.t()
    assert rel_err(got_W, W.grad) < GRAD_TOL
    out3 = pkg.kernels.decode_with_hip_spmm_kernel(fa.detach().to(dev).view(4, 12, F), W.detach().to(dev))
    assert tuple(out3.shape) == (4, 12, d) and rel_err(out3.view(B, d), out) < 1e-6


@pytest.mark.parametrize("sparse_grad", [True, False])
def test_encode_with_hip_spmm_kernel_matches_einsum(pkg, dev, sparse_grad):
    """kernels/entrypoints.py:43-90: "bld,lds->bls" + b_E, and its backward with a sparse (TopK-like) or a dense
    incoming gradient: both routes give einsum's gradients."""
    g = torch.Generator().manual_seed(23)
    B, L, d, F = 64, 3, 64, 256
    x = torch.randn(B, L, d, generator=g).requires_grad_()
    W = (torch.randn(L, d, F, generator=g) / d ** 0.5).requires_grad_()
    b = (0.1 * torch.randn(L, F, generator=g)).requires_grad_()
    up = torch.randn(B, L, F, generator=g)
    if sparse_grad:
        up = up * (torch.rand(B, L, F, generator=g) < 0.002)
    want = torch.einsum("bld,lds->bls", x.double(), W.double()) + b.double()
    (want * up.double()).sum().backward()
    xg, Wg, bg = (t.detach().to(dev).requires_grad_() for t in (x, W, b))
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    out = pkg.kernels.encode_with_triton_spmm_kernel(xg, Wg, bg, 0.996)
    (out * up.to(dev)).sum().backward()
    torch.cuda.synchronize()
    pkg.ops.set_kernel_timer(None)
    assert any(n.startswith("sparse_grad_rows") for n in timer.records) == sparse_grad
    assert rel_err(out, want) < FP32_TOL
    for name, got, exp in (("x", xg.grad, x.grad), ("W_E", Wg.grad, W.grad), ("b_E", bg.grad, b.grad)):
        assert rel_err(got, exp) < GRAD_TOL, (name, rel_err(got, exp))
