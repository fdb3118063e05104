"""The module API of the crosscoder, the cross-layer transcoder and Lorsa (`encode` / `decode` / `forward`, and the
generic `compute_loss` built on them) against the variants' CPU oracle, with an assertion that the library's kernels
ran: the encoder products on the GEMM kernel, the selections on the select kernels, `decode` of sparse activations on the
sparse decoder kernels.  fp32 at 1e-5 (gradients 1e-4), bf16 autocast at 2e-2.
"""

import contextlib
import importlib

import pytest
import torch

from test_gpu_variants import (BF16_TOL, FP32_TOL, GRAD_TOL, clt_batch, copy_params, make_clt, make_crosscoder, make_lorsa,
                               rel_err)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def vo(oracle):
    return importlib.import_module("oracle.variants_oracle")


@contextlib.contextmanager
def kernel_names(pkg):
    """Names of the library calls made inside the block (`ops.KernelTimer` records one entry per call)."""
    timer = pkg.ops.KernelTimer()
    pkg.ops.set_kernel_timer(timer)
    try:
        yield timer.records
    finally:
        torch.cuda.synchronize()
        pkg.ops.set_kernel_timer(None)


def amp_ctx(on):
    return torch.autocast("cuda", dtype=torch.bfloat16) if on else contextlib.nullcontext()


def grads_of(module):
    return {n: p.grad.detach().clone() for n, p in module.named_parameters() if p.grad is not None}


def zero_grads(module):
    for p in module.parameters():
        p.grad = None


def check_param_grads(model, ref, tol, names=None):
    rp = dict(ref.named_parameters())
    scale = max(v.grad.abs().max().item() for v in rp.values() if v.grad is not None)
    for n, p in model.named_parameters():
        if names is not None and n not in names:
            continue
        assert p.grad is not None, n
        want = rp[n].grad
        if want.abs().max().item() < 1e-5 * scale:
            assert p.grad.abs().max().item() < 1e-3 * scale, n
            continue
        assert rel_err(p.grad, want) < tol, (n, rel_err(p.grad, want))


# ---- cross-layer transcoder: decode ------------------------------------------------------------------------------

def sparse_acts(B, L, F, k, seed, device="cpu"):
    """[B, L, F] with k positive entries per (token, layer) at seeded places."""
    g = torch.Generator().manual_seed(seed)
    a = torch.zeros(B, L, F)
    idx = torch.rand(B, L, F, generator=g).topk(k, dim=-1).indices
    a.scatter_(-1, idx, torch.rand(B, L, k, generator=g) + 0.1)
    return a.to(device)


@pytest.mark.parametrize("route", ["sparse_kernels", "dense_products"])
@pytest.mark.parametrize("amp", [False, True], ids=["fp32", "bf16_autocast"])
def test_clt_decode_forward_and_backward_against_the_oracle(pkg, vo, dev, route, amp):
    """`CrossLayerTranscoder.decode` (clt.py:630-709), both routes, forward and backward (activations, every decoder
    group, every bias), against the oracle's decode in fp32 on the CPU: fp32 at 1e-5 / 1e-4, bf16 autocast at 2e-2."""
    L, d, F, k, B = 4, 64, 256, 6, 80
    m, ref, _, _ = make_clt(pkg, vo, dev, "topk", L, d, F, k, seed=141)
    m.sparse_api_decode = route == "sparse_kernels"
    acts = sparse_acts(B, L, F, k, seed=142)
    if amp:   # bf16-representable activations: what the products see is then the same on both sides
        acts = acts.bfloat16().float()
    r = torch.randn(L, B, d, generator=torch.Generator().manual_seed(143))
    a_ref = acts.clone().requires_grad_()
    want = ref.decode(a_ref)
    (want * r).sum().backward()
    a_gpu = acts.to(dev).requires_grad_()
    with kernel_names(pkg) as names, amp_ctx(amp):
        got = m.decode(a_gpu)
        (got.float() * r.to(dev)).sum().backward()
    assert ("sparse_decode_fwd" in names) == (route == "sparse_kernels"), set(names)
    tol, gtol = (BF16_TOL, BF16_TOL) if amp else (FP32_TOL, GRAD_TOL)
    assert got.shape == want.shape
    assert rel_err(got, want) < tol
    # the sparse operators return the activation gradient at the non-zero entries only (kernels/kernels.py:563), which is
    # all that a TopK-family or ReLU activation passes on
    want_a_grad = a_ref.grad * (acts != 0) if route == "sparse_kernels" else a_ref.grad
    assert rel_err(a_gpu.grad, want_a_grad) < gtol
    check_param_grads(m, ref, gtol, names={n for n, _ in m.named_parameters() if n.startswith(("W_D", "b_D"))})
    # batch_first puts the layer axis behind the batch
    with torch.no_grad(), amp_ctx(amp):
        assert torch.equal(m.decode(a_gpu.detach(), batch_first=True), got.detach().transpose(0, 1))


@pytest.mark.parametrize("route", ["sparse_kernels", "dense_products"])
def test_clt_decode_backward_under_autocast_at_the_benchmark_shape(pkg, dev, route):
    """12 layers, d = 768, 12288 features per layer, 2048 tokens, 64 active features per (token, layer), bf16 autocast:
    `decode` forward and backward against block-wise fp32 products (one 2-D product per (target, source) pair), every
    decoder block compared on its own at 2e-2.  (The batched product over a permuted view that the reference's dense
    branch uses returned wrong gradients for source layer 0 through the library's bf16 batched GEMM at this size.)"""
    L, d, F, k, B = 12, 768, 12288, 64, 2048
    hin, hout = [f"in{l}" for l in range(L)], [f"out{l}" for l in range(L)]
    cfg = pkg.CLTConfig(hook_points_in=hin, hook_points_out=hout, d_model=d, expansion_factor=F / d, act_fn="topk", top_k=k,
                        norm_activation="inference", device="cuda", dtype=torch.float32)
    torch.manual_seed(0)
    m = pkg.CrossLayerTranscoder(cfg)
    m.init_parameters()
    m.sparse_api_decode = route == "sparse_kernels"
    g = torch.Generator(device=dev).manual_seed(7)
    acts = torch.zeros(B, L, F, device=dev)
    idx = torch.rand(B, L, F, device=dev, generator=g).topk(k, dim=-1).indices
    acts.scatter_(-1, idx, (torch.rand(B, L, k, device=dev, generator=g) + 0.1).bfloat16().float())
    del idx
    r = torch.randn(L, B, d, device=dev, generator=g) / B
    a = acts.clone().requires_grad_()
    with kernel_names(pkg) as names, amp_ctx(True):
        out = m.decode(a)
        (out.float() * r).sum().backward()
    assert ("sparse_decode_fwd" in names) == (route == "sparse_kernels"), set(names)
    got_w = [w.grad.clone() for w in m.W_D]
    got_b = [b.grad.clone() for b in m.b_D]
    got_a = a.grad.clone()
    zero_grads(m)
    del a
    # block-wise fp32 products
    want_a = torch.zeros_like(acts)
    for lt in range(L):
        recon = m.b_D[lt].detach().expand(B, d).clone()
        for lf in range(lt + 1):
            recon += acts[:, lf] @ m.W_D[lt][lf].detach()
            want_w = acts[:, lf].t() @ r[lt]
            e = rel_err(got_w[lt][lf], want_w)
            assert e < BF16_TOL, (lt, lf, e)
            want_a[:, lf] += r[lt] @ m.W_D[lt][lf].detach().t()
        assert rel_err(out[lt], recon) < BF16_TOL, lt
        assert rel_err(got_b[lt], r[lt].sum(0)) < BF16_TOL, lt
    if route == "sparse_kernels":
        want_a = want_a * (acts != 0)
    assert rel_err(got_a, want_a) < BF16_TOL


@pytest.mark.parametrize("act_fn", ["jumprelu", "relu"])
@pytest.mark.parametrize("kw", [dict(sparsity_loss_type="tanh", l1_coefficient=0.3), dict(sparsity_loss_type="power", p=1, l1_coefficient=0.01),
                                dict(sparsity_loss_type="tanh-quad", l1_coefficient=0.1, frequency_scale=0.05), {}],
                         ids=["tanh", "l1", "tanh-quad", "mse"])
def test_clt_threshold_activations_against_the_oracle(pkg, vo, dev, act_fn, kw):
    """A JumpReLU (thresholds [L, F], clt.py:247-257) or ReLU cross-layer transcoder, with each sparsity penalty
    (clt.py:1024-1104): the encoder products on the GEMM kernel, the activation and the tanh sums on the threshold
    kernels layer by layer, the decode as dense products on the GEMM kernel; loss and every gradient, the thresholds'
    included, against the oracle in fp32; under bf16 autocast the loss at 2e-2 and the decoder gradients on the same
    activations at 2e-2."""
    L, d, F, B = 3, 64, 256, 96
    m, ref, hin, hout = make_clt(pkg, vo, dev, act_fn, L, d, F, 4, seed=151)
    if act_fn == "jumprelu":
        with torch.no_grad():
            ref.activation_function.log_jumprelu_threshold.add_(1.0)     # thresholds around 2.7: a minority of the entries fire
        copy_params(m, ref)
    batch = clt_batch(L, B, d, seed=152)
    gb = {k_: v.to(dev) for k_, v in batch.items()}
    with kernel_names(pkg) as names:
        out = m.compute_loss(gb, **kw)
        out["loss"].backward()
    assert {"encoder_gemm", "jumprelu_fwd", "jumprelu_bwd"} <= set(names), set(names)
    assert len(names["encoder_gemm"]) >= 2 * L + L      # L encoder products, L decodes, and their backward products
    want = ref.compute_loss(batch, hin, hout, **kw)
    want["loss"].backward()
    assert torch.equal((out["feature_acts"] != 0).cpu(), want["feature_acts"] != 0)
    density = (want["feature_acts"] != 0).float().mean().item()
    assert 0.001 < density < 0.6, density
    assert rel_err(out["loss"], want["loss"]) < FP32_TOL
    assert rel_err(out["reconstructed"], want["reconstructed"]) < FP32_TOL
    check_param_grads(m, ref, GRAD_TOL)
    # bf16 autocast: the step's loss, and decode's gradients on the fp32 step's activations
    zero_grads(m)
    with amp_ctx(True):
        out16 = m.compute_loss(gb, **kw)
    assert rel_err(out16["loss"], want["loss"]) < BF16_TOL
    acts = want["feature_acts"].detach()
    r = torch.randn(L, B, d, generator=torch.Generator().manual_seed(153))
    zero_grads(ref)
    (ref.decode(acts) * r).sum().backward()
    with amp_ctx(True):
        (m.decode(acts.to(dev)).float() * r.to(dev)).sum().backward()
    check_param_grads(m, ref, BF16_TOL, names={n for n, _ in m.named_parameters() if n.startswith(("W_D", "b_D"))})


# ---- cross-layer transcoder: encode / forward ----------------------------------------------------------------------

@pytest.mark.parametrize("act_fn", ["topk", "layertopk", "batchtopk", "batchlayertopk", "relu", "jumprelu"])
def test_clt_encode_and_forward_on_the_kernels(pkg, vo, dev, act_fn):
    L, d, F, k, B = 3, 64, 256, 5, 64
    m, ref, hin, hout = make_clt(pkg, vo, dev, act_fn, L, d, F, k, seed=161)
    m.cfg.sparsity_threshold_for_csr = 0.2
    batch = clt_batch(L, B, d, seed=162)
    x = torch.stack([batch[h] for h in hin], dim=1)
    want_acts, want_hp = ref.encode(x, return_hidden_pre=True)
    want_out = ref.decode(want_acts)
    r = torch.randn(L, B, d, generator=torch.Generator().manual_seed(163))
    (want_out * r).sum().backward()
    with kernel_names(pkg) as names:
        acts, hp = m.encode(x.to(dev), return_hidden_pre=True)
        out = m.forward(x.to(dev))
        (out * r.to(dev)).sum().backward()
    assert "encoder_gemm" in names, set(names)
    if "topk" in act_fn:
        assert {"select_topk_row", "select_topk_batch"} & set(names), set(names)
        assert "sparse_decode_fwd" in names, set(names)       # k / F = 2 % of the entries: under the gate set above
    assert rel_err(hp, want_hp) < FP32_TOL
    assert torch.equal((acts != 0).cpu(), want_acts != 0)
    assert rel_err(acts, want_acts) < FP32_TOL
    assert rel_err(out, want_out) < FP32_TOL
    check_param_grads(m, ref, GRAD_TOL)


def test_clt_encode_under_autocast(pkg, vo, dev):
    L, d, F, k, B = 3, 64, 256, 5, 64
    m, ref, hin, hout = make_clt(pkg, vo, dev, "topk", L, d, F, k, seed=171)
    batch = clt_batch(L, B, d, seed=172)
    x = torch.stack([batch[h] for h in hin], dim=1)
    _, want_hp = ref.encode(x, return_hidden_pre=True)
    with kernel_names(pkg) as names, amp_ctx(True), torch.no_grad():
        acts, hp = m.encode(x.to(dev), return_hidden_pre=True)
    assert "encoder_gemm" in names
    assert rel_err(hp, want_hp) < BF16_TOL
    assert torch.all((acts != 0).sum(-1) == k)


# ---- crosscoder -----------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("H,d,F,k,B", [(2, 64, 512, 8, 96), (3, 32, 384, 5, 70)])
def test_crosscoder_api_on_the_kernels(pkg, vo, dev, H, d, F, k, B):
    """`encode` = one GEMM-kernel product over the concatenated heads + the select kernel per head; `decode` of its output
    = the sparse decoder kernels over the H decoder blocks; `forward` differentiates through both (crosscoder.py:314-469)."""
    m, ref, hooks = make_crosscoder(pkg, vo, dev, H, d, F, k, seed=181)
    m.cfg.sparsity_threshold_for_triton_spmm_kernel = 0.9
    g = torch.Generator().manual_seed(182)
    x = torch.randn(B, H, d, generator=g)
    r = torch.randn(B, H, d, generator=g)
    want_acts, want_hp = ref.encode(x, return_hidden_pre=True)
    want_out = ref.decode(want_acts)
    (want_out * r).sum().backward()
    with kernel_names(pkg) as names:
        acts, hp = m.encode(x.to(dev), return_hidden_pre=True)
        recon = m.decode(acts)
        out = m.forward(x.to(dev))
        (out * r.to(dev)).sum().backward()
    assert {"encoder_gemm", "select_topk_row", "dense_to_code", "sparse_decode_fwd", "sparse_decode_bwd_dval"} <= set(names), set(names)
    assert rel_err(hp, want_hp) < FP32_TOL
    assert torch.equal((acts != 0).cpu(), want_acts != 0)
    assert rel_err(acts, want_acts) < FP32_TOL
    assert rel_err(recon, want_out) < FP32_TOL and rel_err(out, want_out) < FP32_TOL
    check_param_grads(m, ref, GRAD_TOL)
    # a denser input than the gate allows takes the dense product, with the same result
    m.cfg.sparsity_threshold_for_triton_spmm_kernel = 0.9999
    with kernel_names(pkg) as names, torch.no_grad():
        again = m.decode(acts.detach())
    assert "sparse_decode_fwd" not in names
    assert rel_err(again, want_out) < FP32_TOL
    # bf16 autocast: the summed encoding within the bf16 bound of the oracle's fp32 value
    with amp_ctx(True), torch.no_grad():
        _, hp16 = m.encode(x.to(dev), return_hidden_pre=True)
    assert rel_err(hp16, want_hp) < BF16_TOL


# ---- Lorsa ------------------------------------------------------------------------------------------------------------

def test_lorsa_api_on_the_kernels(pkg, vo, dev):
    """`decode` of sparse activations on the sparse decoder kernels against the oracle (lorsa.py:765-782), forward and
    backward; `encode` under bf16 autocast on the GEMM and attention kernels within the bf16 bound of the oracle."""
    d, F, h, dq, s, b, k = 64, 256, 4, 32, 64, 2, 8
    m, ref = make_lorsa(pkg, vo, dev, d, F, h, dq, s, k, seed=191, positional_embedding_type="none")
    m.cfg.sparsity_threshold_for_triton_spmm_kernel = 0.9
    g = torch.Generator().manual_seed(192)
    x = torch.randn(b, s, d, generator=g)
    r = torch.randn(b, s, d, generator=g)
    want_acts, want_hp = ref.encode(x, return_hidden_pre=True)
    a_ref = want_acts.detach().clone().requires_grad_()
    want_out = ref.decode(a_ref)
    (want_out * r).sum().backward()
    a_gpu = want_acts.detach().to(dev).requires_grad_()
    with kernel_names(pkg) as names:
        out = m.decode(a_gpu)
        (out * r.to(dev)).sum().backward()
    assert {"dense_to_code", "sparse_decode_fwd", "sparse_decode_bwd_dval"} <= set(names), set(names)
    assert rel_err(out, want_out) < FP32_TOL
    assert rel_err(a_gpu.grad, a_ref.grad * (want_acts != 0)) < GRAD_TOL
    assert rel_err(m.W_O.grad, ref.W_O.grad) < GRAD_TOL and rel_err(m.b_D.grad, ref.b_D.grad) < GRAD_TOL
    with kernel_names(pkg) as names, amp_ctx(True), torch.no_grad():
        acts16, hp16 = m.encode(x.to(dev), return_hidden_pre=True)
        m.forward(x.to(dev))
    assert {"encoder_gemm", "attention_fwd", "select_topk_row", "sparse_decode_fwd"} <= set(names), set(names)
    assert rel_err(hp16, want_hp) < BF16_TOL
    assert torch.all((acts16 != 0).sum(-1) == k)


# ---- the dense -> code conversion with an undersized capacity -----------------------------------------------------------

def test_dense_to_code_with_an_undersized_capacity_truncates_inside_the_arrays(pkg, dev):
    """`capacity` below the number of non-zeros: the code keeps the entries that fit (whole leading rows, a cut row, empty
    rows behind it) and every consumer stays inside idx / val."""
    g = torch.Generator().manual_seed(5)
    B, F, d = 40, 128, 32
    x = torch.where(torch.rand(B, F, generator=g) < 0.1, torch.randn(B, F, generator=g), torch.zeros(B, F))
    nnz = (x != 0).sum(1)
    total = int(nnz.sum())
    cap = total // 2
    code = pkg.ops.dense_to_code(x.to(dev), capacity=cap)
    incl = torch.cumsum(nnz, 0)
    want_nnz = torch.minimum(nnz, (cap - (incl - nnz)).clamp_min(0))
    assert torch.equal(code.row_nnz.cpu().long(), want_nnz)
    assert int(code.row_nnz.sum()) == cap and code.n_slots == cap
    dense = code.to_dense().cpu()
    flat_keep = torch.zeros(B * F, dtype=torch.bool)
    flat_keep[(x != 0).flatten().nonzero().flatten()[:cap]] = True
    assert torch.equal(dense, x * flat_keep.view(B, F))
    W = torch.randn(F, d, generator=g)
    out = pkg.ops.sparse_decode_fwd(code, W.to(dev), None)
    assert rel_err(out, (x * flat_keep.view(B, F)) @ W) < 1e-5
    fi = pkg.ops.build_feature_index(code)
    assert int(fi.feat_ptr[-1]) == cap


def test_decode_operator_rejects_an_ambiguous_square_weight(pkg, dev):
    F = 64
    fa = torch.zeros(8, F, device=dev)
    fa[:, 3] = 1.0
    W = torch.randn(F, F, device=dev)
    with pytest.raises(ValueError, match="square"):
        pkg.kernels.decode_with_hip_spmm_kernel(fa, W)
    a = pkg.kernels.decode_with_hip_spmm_kernel(fa, W, transposed=False)
    b = pkg.kernels.decode_with_hip_spmm_kernel(fa, W.t().contiguous(), transposed=True)
    assert torch.equal(a, W[3].expand(8, F)) and torch.equal(b, a)
