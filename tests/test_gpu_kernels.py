"""Kernel-level parity of the HIP path (through the C ABI) against the CPU oracle.

Tolerances (relative to the largest magnitude of the expected tensor):
  fp32 path 1e-5, bf16 path 2e-2; indices bit-exact.
"""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5
BF16_TOL = 2e-2


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def code_to_rows(code):
    """list of (idx list, val list) per token from a SparseCode on any device"""
    idx, val = code.idx.cpu().numpy(), code.val.cpu().numpy()
    off, nnz = code.row_off.cpu().numpy(), code.row_nnz.cpu().numpy()
    return [(idx[o:o + n], val[o:o + n]) for o, n in zip(off, nnz)]


# ---------------------------------------------------------------------------------------------
# encoder GEMM
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("B,d,F", [(256, 64, 256), (300, 128, 1000), (64, 768, 6144), (1, 64, 8), (513, 256, 260), (40, 32, 24), (70, 96, 300), (2100, 64, 520), (300, 32, 9000)])
def test_encoder_gemm_fp32(pkg, dev, B, d, F):
    print(f"gemm fp32 B={B} d={d} F={F}", flush=True)
    g = torch.Generator().manual_seed(B * 7 + F)
    x = torch.randn(B, d, generator=g)
    w = torch.randn(F, d, generator=g) / d ** 0.5
    pre = pkg.ops.encoder_gemm(x.to(dev), w.to(dev), torch.float32)
    want = x.double() @ w.double().t()
    assert rel_err(pre, want) < FP32_TOL


@pytest.mark.parametrize("B,d,F", [(256, 64, 256), (300, 128, 1000), (512, 2048, 4096), (33, 64, 72), (20, 64, 16), (100, 192, 520), (2304, 128, 300)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_encoder_gemm_bf16(pkg, dev, B, d, F, out_dtype):
    print(f"gemm bf16 B={B} d={d} F={F} out={out_dtype}", flush=True)
    g = torch.Generator().manual_seed(B * 11 + F)
    x = torch.randn(B, d, generator=g).bfloat16()
    w = (torch.randn(F, d, generator=g) / d ** 0.5).bfloat16()
    pre = pkg.ops.encoder_gemm(x.to(dev), w.to(dev), out_dtype)
    want = x.double() @ w.double().t()  # exact products of the bf16 operands
    if out_dtype == torch.float32:
        assert rel_err(pre, want) < FP32_TOL
    else:
        # one bf16 rounding of the fp32 accumulator: bit-exact against rounding the fp64 result,
        # except where fp32 accumulation noise straddles a rounding boundary (<= 1 bf16 ulp)
        want_bf = want.float().bfloat16()
        diff = (pre.cpu().float() - want_bf.float()).abs()
        ulp = want_bf.float().abs() * 2 ** -7
        # (+ an absolute floor: near-zero sums keep the fp32 accumulation noise of O(1) terms)
        assert (diff <= ulp + 1e-5 * want.abs().max().item()).all()
        assert (diff == 0).float().mean() > 0.99


@pytest.mark.parametrize("M,K,N", [(256, 64, 256), (264, 128, 1000), (512, 2048, 776), (40, 64, 72), (8, 64, 16), (2304, 192, 520),
                                   (1000, 4096, 200), (776, 8192, 264)])
@pytest.mark.parametrize("a_k_major,b_k_major", [(False, True), (True, False), (True, True)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_gemm_bf16_operand_layouts(pkg, dev, M, K, N, a_k_major, b_k_major, out_dtype):
    """sae_gemm_bf16 with an operand stored [K, rows]: the product of the operands as they lie equals, BIT FOR BIT, the
    K-contiguous kernel's product of their transposed copies (the same fragments reach the matrix cores in the same order),
    and both match the exact product of the bf16 operands.  Shapes with edge tiles in both dimensions, one to 128 slabs of
    K, and long contractions over few tiles (cut into slices for fp32 output, as for the K-contiguous kernel)."""
    print(f"gemm layouts M={M} K={K} N={N} a_k_major={a_k_major} b_k_major={b_k_major} out={out_dtype}", flush=True)
    g = torch.Generator().manual_seed(M * 13 + N + K)
    a = torch.randn(M, K, generator=g).bfloat16()
    b = (torch.randn(N, K, generator=g) / K ** 0.5).bfloat16()
    a_dev, b_dev = a.to(dev), b.to(dev)
    a_arg = a_dev.t().contiguous() if a_k_major else a_dev
    b_arg = b_dev.t().contiguous() if b_k_major else b_dev
    got = pkg.ops.gemm(a_arg, b_arg, out_dtype, a_k_major=a_k_major, b_k_major=b_k_major, copy_when_faster=False)
    plain = pkg.ops.encoder_gemm(a_dev, b_dev, out_dtype)
    assert got.shape == (M, N) and got.dtype == out_dtype
    assert torch.equal(got, plain)
    want = a.double() @ b.double().t()
    assert rel_err(got, want) < (FP32_TOL if out_dtype == torch.float32 else 2 ** -7)
    # into a given output tensor
    out = torch.empty(M, N, dtype=out_dtype, device=dev)
    assert pkg.ops.gemm(a_arg, b_arg, out_dtype, a_k_major=a_k_major, b_k_major=b_k_major, out=out, copy_when_faster=False) is out
    assert torch.equal(out, plain)
    # with the choice between reading across the rows and a transposed copy left to the shape: the same bits
    assert torch.equal(pkg.ops.gemm(a_arg, b_arg, out_dtype, a_k_major=a_k_major, b_k_major=b_k_major), plain)


def test_gemm_bf16_rejects_what_it_cannot_address(pkg, dev):
    a = torch.zeros(64, 12, dtype=torch.bfloat16, device=dev)       # [K, M] with M = 12: not a multiple of 8
    b = torch.zeros(16, 64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        pkg.ops.gemm(a, b, torch.float32, a_k_major=True, copy_when_faster=False)
    with pytest.raises(ValueError, match="contraction"):
        pkg.ops.gemm(b, torch.zeros(16, 128, dtype=torch.bfloat16, device=dev), torch.float32)


def test_encoder_gemm_rejects_bad_shapes(pkg, dev):
    x = torch.randn(8, 40, device=dev)
    w = torch.randn(16, 40, device=dev)
    with pytest.raises(RuntimeError, match="multiple of"):
        pkg.ops.encoder_gemm(x, w, torch.float32)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        pkg.ops.encoder_gemm(x.cpu(), w.cpu(), torch.float32)


# ---------------------------------------------------------------------------------------------
# TopK select
# ---------------------------------------------------------------------------------------------

def oracle_topk_code(oracle, pre, b_enc, scale, k):
    """(idx, val) per row by the oracle's rule: relu mask, k largest, ties -> lowest index."""
    h0 = pre.float() + (b_enc if b_enc is not None else 0.0)
    h1 = h0 * scale if scale is not None else h0
    r = h1 * h1.gt(0).to(h1.dtype)
    a = oracle.topk(r, k=k, dim=-1)
    f = a / scale if scale is not None else a
    rows = []
    for b in range(pre.shape[0]):
        nz = torch.nonzero(a[b] > 0).flatten()
        rows.append((nz.numpy().astype(np.int32), f[b, nz].numpy()))
    return rows


def check_select(pkg, oracle, dev, pre, b_enc, scale, k, cand_cap=None):
    code = pkg.ops.select_topk_row(
        pre.to(dev), None if b_enc is None else b_enc.to(dev), None if scale is None else scale.to(dev), k, cand_cap
    )
    got = code_to_rows(code)
    want = oracle_topk_code(oracle, pre, b_enc, scale, k)
    assert code.row_off.cpu().tolist() == [b * k for b in range(pre.shape[0])]
    for b, ((gi, gv), (wi, wv)) in enumerate(zip(got, want)):
        assert np.array_equal(gi, wi), f"row {b}: indices differ\n got {gi}\nwant {wi}"
        assert np.array_equal(gv, wv), f"row {b}: values differ"
    # unused slots are zero-filled
    idx = code.idx.view(-1, k).cpu()
    val = code.val.view(-1, k).cpu()
    pad = torch.arange(k)[None, :] >= code.row_nnz.cpu()[:, None]
    assert (val[pad] == 0).all() and (idx[pad] == 0).all()
    return code


@pytest.mark.parametrize("B,F,k", [(7, 1000, 5), (16, 4096, 32), (4, 131072, 64), (3, 37, 37), (5, 2048, 512)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_select_topk_row_random(pkg, oracle, dev, B, F, k, dtype):
    print(f"select B={B} F={F} k={k} {dtype}", flush=True)
    g = torch.Generator().manual_seed(F + k)
    pre = torch.randn(B, F, generator=g).to(dtype)
    b_enc = 0.1 * torch.randn(F, generator=g)
    scale = 0.5 + torch.rand(F, generator=g)
    check_select(pkg, oracle, dev, pre, b_enc, scale, k)
    check_select(pkg, oracle, dev, pre, None, None, k)


@pytest.mark.parametrize("cand_cap", [0, 8, 4096])
def test_select_topk_row_paths_agree(pkg, oracle, dev, cand_cap):
    """fast path (candidate list) and general path (row histograms) give the same code"""
    g = torch.Generator().manual_seed(5)
    pre = torch.randn(9, 5000, generator=g)
    check_select(pkg, oracle, dev, pre, None, None, 40, cand_cap)


def test_select_topk_row_reference_kat(pkg, oracle, dev):
    """tests/unit/test_sae.py:92-113 of the reference: TopK(k=2)"""
    pre = torch.tensor([[1.0, 1.5, 3.0, 4.0], [4.0, 3.0, 1.5, 1.0]])
    code = check_select(pkg, oracle, dev, pre, None, None, 2)
    dense = code.to_dense().cpu()
    assert torch.equal(dense, torch.tensor([[0.0, 0.0, 3.0, 4.0], [4.0, 3.0, 0.0, 0.0]]))


@pytest.mark.parametrize("cand_cap", [None, 0])
def test_select_topk_row_ties_and_degenerate_rows(pkg, oracle, dev, cand_cap):
    F, k = 3000, 16
    rows = []
    rows.append(torch.full((F,), 2.0))                      # all equal: lowest k indices win
    rows.append(torch.zeros(F))                             # nothing positive
    rows.append(-torch.ones(F))                             # all negative
    r = torch.zeros(F); r[[5, 77, 2999]] = torch.tensor([1.0, 3.0, 2.0]); rows.append(r)  # fewer than k positives
    r = torch.ones(F); r[100:110] = 5.0; rows.append(r)     # 10 clear winners + 6 of a 2990-way tie
    g = torch.Generator().manual_seed(3)
    r = torch.randint(0, 4, (F,), generator=g).float(); rows.append(r)  # heavy ties on a few levels
    r = torch.randn(F, generator=g).bfloat16().float(); rows.append(r)  # bf16-quantised values
    pre = torch.stack(rows)
    code = check_select(pkg, oracle, dev, pre, None, None, k, cand_cap)
    assert code.row_nnz.cpu().tolist()[:4] == [k, 0, 0, 3]
    assert code.idx.view(-1, k)[0].cpu().tolist() == list(range(k))


def test_select_topk_row_matches_torch_topk_when_tie_free(pkg, dev):
    g = torch.Generator().manual_seed(11)
    pre = torch.randn(32, 8192, generator=g)
    k = 50
    code = pkg.ops.select_topk_row(pre.to(dev), None, None, k)
    want = torch.topk(pre * (pre > 0), k, dim=-1).indices.sort(dim=-1).values
    assert torch.equal(code.idx.view(-1, k).cpu().long(), want)


@pytest.mark.gpu
@pytest.mark.parametrize("B,F,k", [(5, 4096, 16), (16, 24576, 64), (3, 1001, 8), (4, 131072, 64)])
def test_select_topk_row_in_bf16_arithmetic(pkg, oracle, dev, B, F, k):
    """a dictionary held in bf16: bias sum, norm product and final quotient are bf16 tensors in the reference
    (models/sae.py:324-341).  The expected code is that op sequence on CPU bf16 tensors with the oracle's TopK."""
    print(f"select lowp B={B} F={F} k={k}", flush=True)
    g = torch.Generator().manual_seed(F + k + 1)
    pre = torch.randn(B, F, generator=g).bfloat16()
    b_enc = (0.1 * torch.randn(F, generator=g)).bfloat16()
    norm = (0.5 + torch.rand(F, generator=g)).bfloat16()
    h1 = (pre + b_enc) * norm
    want = oracle.topk(h1 * h1.gt(0).to(h1.dtype), k=k, dim=-1) / norm
    assert want.dtype == torch.bfloat16
    code = pkg.ops.select_topk_row(pre.to(dev), b_enc.float().to(dev), norm.float().to(dev), k, lowp=True)
    got = code.to_dense().cpu()
    assert torch.equal(got != 0, want != 0), "kept sets differ"
    assert torch.equal(got, want.float()), "kept values differ"
    # the rounding makes ties at the threshold common; the plain arithmetic keeps another set
    plain = pkg.ops.select_topk_row(pre.to(dev), b_enc.float().to(dev), norm.float().to(dev), k).to_dense().cpu()
    if F >= 24576:
        assert not torch.equal(plain != 0, want != 0)


# ---------------------------------------------------------------------------------------------
# sparse decode, fused loss, d val
# ---------------------------------------------------------------------------------------------

def random_code(pkg, dev, B, F, k, seed, ragged=True):
    g = torch.Generator().manual_seed(seed)
    pre = torch.randn(B, F, generator=g)
    if ragged:
        pre[0] = -1.0                 # an empty token
        pre[1, 3:] = -1.0             # a token with at most 3 active features
    return pkg.ops.select_topk_row(pre.to(dev), None, None, k)


@pytest.mark.parametrize("B,d,F,k", [(10, 64, 512, 8), (33, 768, 2048, 32), (6, 4096, 1024, 64), (4, 8, 16, 3), (5, 16384, 64, 4)])
@pytest.mark.parametrize("w_dtype", [torch.float32, torch.bfloat16])
def test_sparse_decode_fwd(pkg, dev, B, d, F, k, w_dtype):
    print(f"decode B={B} d={d} F={F} k={k} {w_dtype}", flush=True)
    code = random_code(pkg, dev, B, F, k, seed=d + k)
    g = torch.Generator().manual_seed(1)
    w = (torch.randn(F, d, generator=g) / d ** 0.5).to(w_dtype)
    b_dec = torch.randn(d, generator=g)
    recon = pkg.ops.sparse_decode_fwd(code, w.to(dev), b_dec.to(dev))
    want = code.to_dense().cpu().double() @ w.double() + b_dec.double()
    assert rel_err(recon, want) < FP32_TOL
    recon_nb = pkg.ops.sparse_decode_fwd(code, w.to(dev), None)
    assert rel_err(recon_nb, want - b_dec.double()) < FP32_TOL


@pytest.mark.parametrize("B,d,F,k", [(10, 64, 512, 8), (33, 768, 2048, 32), (6, 4096, 1024, 64),
                                     # short rows with long row lists (a cross-layer transcoder's prefix codes)
                                     (20, 768, 4096, 200), (9, 1024, 2048, 131), (12, 256, 1024, 150), (5, 8, 600, 133)])
@pytest.mark.parametrize("w_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("masked", [False, True])
def test_sparse_decode_mse_fused(pkg, dev, B, d, F, k, w_dtype, masked):
    print(f"fused B={B} d={d} F={F} k={k} {w_dtype} masked={masked}", flush=True)
    code = random_code(pkg, dev, B, F, k, seed=d + 3 * k)
    g = torch.Generator().manual_seed(2)
    w = (torch.randn(F, d, generator=g) / d ** 0.5).to(w_dtype)
    b_dec = torch.randn(d, generator=g)
    label = torch.randn(B, d, generator=g)
    if masked:
        mask = (torch.rand(B, generator=g) > 0.3).float()
        tok_w = mask / mask.sum()
    else:
        tok_w = torch.full((B,), 1.0 / B)
    recon, loss_tok, grad_recon, dval = pkg.ops.sparse_decode_mse_fused(
        code, w.to(dev), b_dec.to(dev), label.to(dev), tok_w.to(dev)
    )
    # autograd of the dense restatement in fp64
    fa = code.to_dense().cpu().double().requires_grad_(True)
    wd = w.double()
    rec = fa @ wd + b_dec.double()
    rec.retain_grad()
    loss = (((rec - label.double()) ** 2).sum(-1) * tok_w.double()).sum()
    loss.backward()
    assert rel_err(recon, rec) < FP32_TOL
    assert abs(loss_tok.sum().item() - loss.item()) / loss.item() < FP32_TOL
    assert rel_err(grad_recon, rec.grad) < FP32_TOL
    # d val against the dense gradient gathered at the code's slots
    rows = code_to_rows(code)
    dv = dval.cpu().numpy()
    off = code.row_off.cpu().numpy()
    scale = fa.grad.abs().max().item()
    for b, (ri, _) in enumerate(rows):
        want = fa.grad[b, torch.as_tensor(ri, dtype=torch.long)].numpy()
        got = dv[off[b]: off[b] + len(ri)]
        assert len(ri) == 0 or np.abs(got - want).max() <= FP32_TOL * scale + 1e-30
        assert (dv[off[b] + len(ri): off[b] + k] == 0).all()
    # the stand-alone backward kernel agrees with the fused one
    dval2 = pkg.ops.sparse_decode_bwd_dval(code, grad_recon, w.to(dev))
    assert rel_err(dval2, dval) < 1e-6


# ---------------------------------------------------------------------------------------------
# feature index and gradient rows
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("B,F,k", [(50, 64, 8), (300, 1000, 16), (1024, 512, 32), (7, 10000, 3)])
def test_build_feature_index(pkg, dev, B, F, k):
    print(f"feature index B={B} F={F} k={k}", flush=True)
    code = random_code(pkg, dev, B, F, k, seed=B + F)
    fi = pkg.ops.build_feature_index(code)
    idx = code.idx.cpu().numpy()
    off, nnz = code.row_off.cpu().numpy(), code.row_nnz.cpu().numpy()
    slots = np.concatenate([np.arange(o, o + n) for o, n in zip(off, nnz)]).astype(np.int64)
    feats = idx[slots]
    order = np.argsort(feats, kind="stable")          # ascending feature, then ascending slot
    want_slots = slots[order].astype(np.int32)
    want_ptr = np.concatenate([[0], np.cumsum(np.bincount(feats, minlength=F))]).astype(np.int32)
    assert np.array_equal(fi.feat_ptr.cpu().numpy(), want_ptr)
    n_valid = int(nnz.sum())
    assert np.array_equal(fi.feat_slot.cpu().numpy()[:n_valid], want_slots)
    tok = np.repeat(np.arange(B), nnz).astype(np.int32)
    assert np.array_equal(fi.slot_tok.cpu().numpy()[slots], tok)


def test_build_feature_index_long_segments(pkg, dev):
    """a feature active on every token exercises the bitmap ordering of long segments"""
    B, F, k = 700, 256, 4
    g = torch.Generator().manual_seed(0)
    pre = torch.randn(B, F, generator=g)
    pre[:, 17] = 10.0
    pre[::2, 200] = 9.0
    code = pkg.ops.select_topk_row(pre.to(dev), None, None, k)
    fi = pkg.ops.build_feature_index(code)
    ptr = fi.feat_ptr.cpu().numpy()
    seg = fi.feat_slot.cpu().numpy()[ptr[17]:ptr[18]]
    assert len(seg) == B and np.all(np.diff(seg) > 0)
    seg = fi.feat_slot.cpu().numpy()[ptr[200]:ptr[201]]
    assert len(seg) >= B // 2 and np.all(np.diff(seg) > 0)  # odd tokens may pick it by chance


@pytest.mark.parametrize("B,d,F,k", [(64, 64, 256, 8), (300, 768, 1000, 16), (128, 4096, 512, 4)])
@pytest.mark.parametrize("dense_dtype", [torch.float32, torch.bfloat16])
def test_sparse_grad_rows(pkg, dev, B, d, F, k, dense_dtype):
    print(f"grad rows B={B} d={d} F={F} k={k} {dense_dtype}", flush=True)
    code = random_code(pkg, dev, B, F, k, seed=d + B)
    fi = pkg.ops.build_feature_index(code)
    g = torch.Generator().manual_seed(4)
    dense = torch.randn(B, d, generator=g).to(dense_dtype)
    coef = torch.randn(code.n_slots, generator=g)
    out, bias = pkg.ops.sparse_grad_rows(fi, coef.to(dev), dense.to(dev), F, want_bias=True)
    # dense restatement: C[b, f] = coef at the valid slots; out = C^T @ dense
    import dataclasses
    c_code = dataclasses.replace(code, val=coef.to(dev))
    C = c_code.to_dense().cpu().double()
    want = C.t() @ dense.double()
    assert rel_err(out, want) < FP32_TOL
    assert rel_err(bias, C.sum(0)) < FP32_TOL
    # reproducible: the atomics only decide an order that is then canonicalised
    fi2 = pkg.ops.build_feature_index(code)
    out2, _ = pkg.ops.sparse_grad_rows(fi2, coef.to(dev), dense.to(dev), F)
    assert torch.equal(out, out2)


# ---------------------------------------------------------------------------------------------
# element-wise helpers and Adam
# ---------------------------------------------------------------------------------------------

def test_cast_rownorm_transpose_colsum(pkg, dev):
    g = torch.Generator().manual_seed(9)
    a = torch.randn(301, 520, generator=g)
    assert torch.equal(pkg.ops.cast_bf16(a.to(dev)).cpu(), a.bfloat16())
    assert rel_err(pkg.ops.row_norm(a.to(dev)), a.double().norm(dim=1)) < 1e-6
    assert torch.equal(pkg.ops.transpose(a.to(dev)).cpu(), a.t().contiguous())
    assert rel_err(pkg.ops.col_sum(a.to(dev)), a.double().sum(0)) < 1e-6
    b = torch.randn(77, 13, generator=g)  # odd sizes: scalar tails
    assert torch.equal(pkg.ops.cast_bf16(b.to(dev)).cpu(), b.bfloat16())
    assert rel_err(pkg.ops.row_norm(b.to(dev)), b.double().norm(dim=1)) < 1e-6


@pytest.mark.parametrize("rows,cols", [(256, 192), (301, 520), (64, 8), (8, 64), (77, 13), (1, 1)])
@pytest.mark.parametrize("src_dtype", [torch.float32, torch.bfloat16])
def test_transpose_to_bf16(pkg, dev, rows, cols, src_dtype):
    """bit-exact against cast-then-transpose; the mask zeroes entries; the column sums are those of the masked source"""
    print(f"transpose_to_bf16 {rows}x{cols} {src_dtype}", flush=True)
    g = torch.Generator().manual_seed(rows * 1000 + cols)
    a = torch.randn(rows, cols, generator=g).to(src_dtype)
    out, sums = pkg.ops.transpose_to_bf16(a.to(dev))
    assert sums is None and torch.equal(out.cpu(), a.bfloat16().t().contiguous())
    mask = torch.randn(rows, cols, generator=g)          # about half not positive, some exactly 0
    mask[0, 0] = 0.0
    masked = torch.where(mask > 0, a.float(), torch.zeros(()))
    out, sums = pkg.ops.transpose_to_bf16(a.to(dev), mask=mask.to(dev), col_sums=True)
    assert torch.equal(out.cpu(), masked.bfloat16().t().contiguous())
    assert torch.allclose(sums.cpu().double(), masked.double().sum(0), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("B,n_cols,k", [(5, 100, 7), (64, 3328, 512), (3, 20000, 40), (2, 8192, 1)])
def test_code_to_dense(pkg, oracle, dev, B, n_cols, k):
    """a BatchTopK code (ragged rows, unused tail slots) and a TopK code written out densely, fp32 and bf16"""
    print(f"code_to_dense B={B} n={n_cols} k={k}", flush=True)
    g = torch.Generator().manual_seed(B + n_cols)
    pre = torch.randn(B, n_cols, generator=g)
    pre[0] = -1.0                                        # a token that keeps nothing
    for code in (pkg.ops.select_topk_batch(pre.to(dev), None, None, k * B), pkg.ops.select_topk_row(pre.to(dev), None, None, k)):
        want = code.to_dense().cpu()
        f32, b16 = pkg.ops.code_to_dense(code, n_cols, want_f32=True, want_bf16=True)
        assert torch.equal(f32.cpu(), want)
        assert torch.equal(b16.cpu(), want.bfloat16())
        only_b16 = pkg.ops.code_to_dense(code, n_cols, want_f32=False, want_bf16=True)
        assert only_b16[0] is None and torch.equal(only_b16[1].cpu(), want.bfloat16())
    # indices at or beyond n_cols are dropped
    f32, _ = pkg.ops.code_to_dense(code, n_cols // 2)
    assert torch.equal(f32.cpu(), want[:, : n_cols // 2])


@pytest.mark.parametrize("B,d", [(7, 64), (300, 768), (64, 4096)])
def test_mse_auxk_fused(pkg, dev, B, d):
    """the four outputs against the formulas of the aux-k loss in fp64 (fp32 bar: 1e-5 relative)"""
    g = torch.Generator().manual_seed(B + d)
    recon, label, aux = (torch.randn(B, d, generator=g) for _ in range(3))
    w = torch.rand(B, generator=g) / B
    alpha = 1.0 / 32
    rec_tok, aux_tok, g_aux, grad, grad16 = pkg.ops.mse_auxk_fused(recon.to(dev), label.to(dev), aux.to(dev), w.to(dev), alpha,
                                                                   want_bf16=True)
    R, L, A, W = recon.double(), label.double(), aux.double(), w.double()[:, None]
    r = (L - R) - A
    assert rel_err(rec_tok, (W * (R - L) ** 2).sum(1)) < 1e-5
    assert rel_err(aux_tok, (W * r ** 2).sum(1)) < 1e-5
    assert rel_err(g_aux, -2 * alpha * W * r) < 1e-5
    assert rel_err(grad, 2 * W * (R - L) - 2 * alpha * W * r) < 1e-5
    assert torch.equal(grad16.cpu(), grad.cpu().bfloat16())
    # without an aux reconstruction (no dead feature) and without token weights
    rec_tok, aux_tok, g_aux, grad2, grad16 = pkg.ops.mse_auxk_fused(recon.to(dev), label.to(dev), None, None, alpha)
    assert aux_tok is None and g_aux is None and grad16 is None
    assert rel_err(rec_tok, ((R - L) ** 2).sum(1)) < 1e-5 and rel_err(grad2, 2 * (R - L)) < 1e-5


def test_row_norm_reference_fixture(pkg, dev):
    """decoder norms of the reference's test fixture (tests/unit/test_sae.py:31-55): closed forms"""
    W_D = torch.tensor([[1.0, 5.0], [2.0, 6.0], [3.0, 7.0], [4.0, 8.0]])
    want = torch.tensor([26.0, 40.0, 58.0, 80.0]).sqrt()
    assert torch.allclose(pkg.ops.row_norm(W_D.to(dev)).cpu(), want, rtol=1e-6)


@pytest.mark.parametrize("n,row_len", [(1000, 0), (4096 * 3, 4096), (77, 0), (64 * 128, 128)])
def test_adam_step_matches_torch(pkg, dev, n, row_len):
    g = torch.Generator().manual_seed(n)
    p0 = torch.randn(n, generator=g)
    ref = torch.nn.Parameter(p0.clone())
    opt = torch.optim.Adam([ref], lr=4e-4, betas=(0.9, 0.999))
    p = p0.clone().to(dev)
    m = torch.zeros(n, device=dev)
    v = torch.zeros(n, device=dev)
    shadow = torch.empty(n, dtype=torch.bfloat16, device=dev)
    norms = torch.empty(n // row_len, device=dev) if row_len else None
    for step in range(1, 4):
        grad = torch.randn(n, generator=g) * (torch.rand(n, generator=g) > 0.5)  # exact zeros included
        ref.grad = grad.clone()
        opt.step()
        pkg.ops.adam_step(p, grad.to(dev), m, v, lr=4e-4, beta1=0.9, beta2=0.999, eps=1e-8, step=step,
                          shadow_bf16=shadow, row_norm_out=norms, row_len=row_len)
        # both sides round p to fp32 after an lr-sized move: allow a few ulps of |p|
        assert (p.cpu() - ref.detach()).abs().max() <= 4 * 1.2e-7 * p0.abs().max()
        assert torch.equal(shadow.cpu(), p.cpu().bfloat16())
        if row_len:
            assert rel_err(norms, p.cpu().view(-1, row_len).double().norm(dim=1)) < 1e-6
    st = opt.state[ref]
    assert rel_err(m, st["exp_avg"]) < 1e-6 and rel_err(v, st["exp_avg_sq"]) < 1e-6


def test_adam_step_row_grad_coef_equals_adding_the_term_first(pkg, dev):
    """g + coef[r] * p applied inside the update kernel gives the bits of adding coef[:, None] * p to g beforehand"""
    g0 = torch.Generator().manual_seed(21)
    F, d = 300, 768
    p0 = torch.randn(F, d, generator=g0).to(dev)
    grad = torch.randn(F, d, generator=g0).to(dev)
    coef = (0.1 * torch.randn(F, generator=g0)).to(dev)
    hyper = dict(lr=4e-4, beta1=0.9, beta2=0.999, eps=1e-8)
    pa, ma, va = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    pb, mb, vb = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    na, nb = torch.empty(F, device=dev), torch.empty(F, device=dev)
    for step in (1, 2, 3):
        pkg.ops.adam_step(pa, grad + coef[:, None] * pa, ma, va, step=step, row_norm_out=na, row_len=d, **hyper)
        pkg.ops.adam_step(pb, grad, mb, vb, step=step, row_norm_out=nb, row_len=d, row_grad_coef=coef, **hyper)
        assert torch.equal(pa, pb) and torch.equal(ma, mb) and torch.equal(va, vb) and torch.equal(na, nb)
    pkg.ops.adam_step(pb, grad, mb, vb, step=4, row_len=d, row_grad_coef=coef, **hyper)      # without the norm output
    pkg.ops.adam_step(pa, grad + coef[:, None] * pa, ma, va, step=4, **hyper)
    assert torch.equal(pa, pb)
    with pytest.raises(ValueError):
        pkg.ops.adam_step(pb, grad, mb, vb, step=5, row_grad_coef=coef, **hyper)               # row_len missing
    # a bf16 gradient is widened as it is read: the bits of converting it first (row-wise and flat kernels, odd tail)
    g16 = grad.bfloat16()
    for kwargs in (dict(row_norm_out=nb, row_len=d, row_grad_coef=coef), dict()):
        pkg.ops.adam_step(pb, g16, mb, vb, step=5, **kwargs, **hyper)
        kwargs_a = dict(kwargs, row_norm_out=na) if kwargs else {}
        pkg.ops.adam_step(pa, g16.float(), ma, va, step=5, **kwargs_a, **hyper)
        assert torch.equal(pa, pb) and torch.equal(ma, mb) and torch.equal(va, vb)
    q0 = torch.randn(1003, generator=g0).to(dev)
    gq = torch.randn(1003, generator=g0).to(dev).bfloat16()
    qa, qb = q0.clone(), q0.clone()
    z = lambda: torch.zeros_like(q0)  # noqa: E731
    pkg.ops.adam_step(qa, gq.float(), z(), z(), step=1, **hyper)
    pkg.ops.adam_step(qb, gq, z(), z(), step=1, **hyper)
    assert torch.equal(qa, qb)


@pytest.mark.parametrize("B,d,F,k", [(64, 64, 256, 8), (300, 768, 1000, 16), (128, 4096, 512, 4), (40, 5120, 96, 3)])
@pytest.mark.parametrize("dense_dtype", [torch.float32, torch.bfloat16])
def test_adam_step_sparse_rows_equals_grad_rows_then_adam(pkg, dev, B, d, F, k, dense_dtype):
    """the gradient-free route (rows rebuilt inside the Adam pass) gives the same bits as writing the
    dense gradient rows first and running the plain Adam kernel on them"""
    print(f"adam sparse rows B={B} d={d} F={F} k={k} {dense_dtype}", flush=True)
    code = random_code(pkg, dev, B, F, k, seed=d + B + 1)
    fi = pkg.ops.build_feature_index(code)
    g = torch.Generator().manual_seed(8)
    dense = torch.randn(B, d, generator=g).to(dense_dtype).to(dev)
    coef = torch.randn(code.n_slots, generator=g).to(dev)
    p0 = torch.randn(F, d, generator=g).to(dev)
    hyper = dict(lr=4e-4, beta1=0.9, beta2=0.999, eps=1e-8)
    pa, ma, va = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    pb, mb, vb = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    sha, shb = torch.empty(F, d, dtype=torch.bfloat16, device=dev), torch.empty(F, d, dtype=torch.bfloat16, device=dev)
    na, nb = torch.empty(F, device=dev), torch.empty(F, device=dev)
    bias_b = torch.empty(F, device=dev)
    for step in (1, 2):
        rows, bias_a = pkg.ops.sparse_grad_rows(fi, coef, dense, F, want_bias=True)
        pkg.ops.adam_step(pa, rows, ma, va, step=step, shadow_bf16=sha, row_norm_out=na, row_len=d, **hyper)
        pkg.ops.adam_step_sparse_rows(fi, coef, dense, pb, mb, vb, step=step, shadow_bf16=shb, row_norm_out=nb,
                                      bias_grad_out=bias_b, **hyper)
        assert torch.equal(pa, pb) and torch.equal(ma, mb) and torch.equal(va, vb)
        assert torch.equal(sha, shb) and torch.equal(na, nb) and torch.equal(bias_a, bias_b)
    assert not torch.equal(pa, p0)


@pytest.mark.gpu
@pytest.mark.parametrize("n,row_len", [(4096 * 3, 0), (1003, 0), (512 * 768, 768)])
def test_adam_step_on_bf16_tensors_follows_torch_adam(pkg, dev, n, row_len):
    """bf16 parameter, gradient and moments: the oracle is the library routine itself, torch.optim.Adam on CPU
    bf16 tensors (every element-wise op rounds to bf16).  Tolerance 2e-2 relative (bf16); nearly every element
    agrees to the bit."""
    print(f"adam lowp n={n} row_len={row_len}", flush=True)
    g = torch.Generator().manual_seed(n)
    p0 = torch.randn(n, generator=g).bfloat16()
    ref_p = torch.nn.Parameter(p0.clone())
    opt = torch.optim.Adam([ref_p], lr=1e-2, betas=(0.9, 0.999), eps=1e-8, foreach=False)
    p, m, v = p0.clone().to(dev), torch.zeros(n, dtype=torch.bfloat16, device=dev), torch.zeros(n, dtype=torch.bfloat16, device=dev)
    norm = torch.empty(n // row_len, device=dev) if row_len else None
    for step in range(1, 6):
        grad = (torch.randn(n, generator=g) * 0.1).bfloat16()
        ref_p.grad = grad.clone()
        opt.step()
        pkg.ops.adam_step(p, grad.to(dev), m, v, lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, step=step,
                          row_norm_out=norm, row_len=row_len)
        st = opt.state[ref_p]
        for name, got, want in (("p", p, ref_p.data), ("m", m, st["exp_avg"]), ("v", v, st["exp_avg_sq"])):
            got, want = got.cpu().float(), want.float()
            assert torch.allclose(got, want, rtol=2e-2, atol=1e-6), f"{name} at step {step}"
            assert (got == want).float().mean().item() > 0.97, f"{name} at step {step}: too few identical elements"
    assert not torch.equal(p.cpu(), p0)
    if row_len:
        assert torch.allclose(norm.cpu(), p.cpu().float().view(-1, row_len).norm(dim=1), rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("B,d,F,k", [(64, 64, 256, 8), (300, 768, 1000, 16), (40, 5120, 96, 3)])
def test_adam_step_sparse_rows_on_bf16_tensors_equals_grad_rows_then_adam(pkg, dev, B, d, F, k):
    """bf16 state: rows rebuilt inside the pass == dense rows written out, rounded to bf16, then the plain pass"""
    print(f"adam lowp sparse rows B={B} d={d} F={F} k={k}", flush=True)
    code = random_code(pkg, dev, B, F, k, seed=d + B + 2)
    fi = pkg.ops.build_feature_index(code)
    g = torch.Generator().manual_seed(9)
    dense = torch.randn(B, d, generator=g).bfloat16().to(dev)
    coef = torch.randn(code.n_slots, generator=g).to(dev)
    p0 = torch.randn(F, d, generator=g).bfloat16().to(dev)
    hyper = dict(lr=4e-4, beta1=0.9, beta2=0.999, eps=1e-8)
    z = lambda: torch.zeros(F, d, dtype=torch.bfloat16, device=dev)  # noqa: E731
    pa, ma, va, pb, mb, vb = p0.clone(), z(), z(), p0.clone(), z(), z()
    na, nb, bias_b = torch.empty(F, device=dev), torch.empty(F, device=dev), torch.empty(F, device=dev)
    for step in (1, 2):
        rows, bias_a = pkg.ops.sparse_grad_rows(fi, coef, dense, F, want_bias=True)
        pkg.ops.adam_step(pa, rows.bfloat16(), ma, va, step=step, row_norm_out=na, row_len=d, **hyper)
        pkg.ops.adam_step_sparse_rows(fi, coef, dense, pb, mb, vb, step=step, row_norm_out=nb, bias_grad_out=bias_b, **hyper)
        assert torch.equal(pa, pb) and torch.equal(ma, mb) and torch.equal(va, vb)
        assert torch.equal(na, nb) and torch.equal(bias_a, bias_b)
    assert not torch.equal(pa, p0)
    with pytest.raises(ValueError):
        pkg.ops.adam_step_sparse_rows(fi, coef, dense, pb, mb, vb, step=3, shadow_bf16=z(), **hyper)


# ---------------------------------------------------------------------------------------------
# BatchTopK select
# ---------------------------------------------------------------------------------------------

def oracle_batchtopk_dense(oracle, pre, b_enc, scale, k_total, feat_mask=None):
    """dense [B, F] feature activations by the oracle's rule (global top-k_total, ties -> lowest flat index)"""
    h0 = pre.float() + (b_enc if b_enc is not None else 0.0)
    h1 = h0 * scale if scale is not None else h0
    if feat_mask is not None:
        h1 = ((h1 / scale) * feat_mask) * scale if scale is not None else h1 * feat_mask
    r = h1 * h1.gt(0).to(h1.dtype)
    a = oracle.topk(r, k=min(k_total, r.numel()), dim=(-2, -1)) if k_total > 0 else torch.zeros_like(r)
    return a / scale if scale is not None else a


def check_batch_select(pkg, oracle, dev, pre, b_enc, scale, k_total, feat_mask=None, k_on_device=False):
    to = lambda t: None if t is None else t.to(dev)  # noqa: E731
    if k_on_device:
        code = pkg.ops.select_topk_batch(pre.to(dev), to(b_enc), to(scale), torch.tensor(k_total, dtype=torch.int64, device=dev),
                                         to(feat_mask), capacity=max(k_total, 1))
    else:
        code = pkg.ops.select_topk_batch(pre.to(dev), to(b_enc), to(scale), k_total, to(feat_mask))
    want = oracle_batchtopk_dense(oracle, pre, b_enc, scale, k_total, feat_mask)
    got = code.to_dense().cpu()
    assert torch.equal(got != 0, want != 0), "kept sets differ"
    assert torch.equal(got, want), "kept values differ"
    # structure: offsets are the running sum of the row lengths; indices ascend inside a row
    nnz = code.row_nnz.cpu().long()
    assert torch.equal(code.row_off.cpu(), torch.cumsum(nnz, 0) - nnz)
    assert nnz.sum().item() == (want != 0).sum().item()
    for (ri, _) in code_to_rows(code):
        assert np.all(np.diff(ri) > 0)
    return code


@pytest.mark.parametrize("B,F,k", [(9, 1000, 5), (64, 4096, 32), (8, 32768, 64), (3, 37, 4), (300, 512, 7),
                                   (2, 600064, 50), (2, 600001, 50)])   # more than 64 segments per wave; odd row length
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_select_topk_batch_random(pkg, oracle, dev, B, F, k, dtype):
    print(f"batchtopk B={B} F={F} k={k} {dtype}", flush=True)
    g = torch.Generator().manual_seed(F + k)
    pre = torch.randn(B, F, generator=g).to(dtype)
    b_enc = 0.1 * torch.randn(F, generator=g)
    scale = 0.5 + torch.rand(F, generator=g)
    code = check_batch_select(pkg, oracle, dev, pre, b_enc, scale, k * B)
    assert code.row_nnz.sum().item() == k * B
    check_batch_select(pkg, oracle, dev, pre, None, None, k * B, k_on_device=True)


def test_select_topk_batch_ties_and_degenerate(pkg, oracle, dev):
    B, F = 6, 2000
    g = torch.Generator().manual_seed(0)
    pre = torch.randint(0, 4, (B, F), generator=g).float()      # four levels: the threshold sits inside a huge tie
    for k_total in (1, 17, 3000, 5000, B * F):
        check_batch_select(pkg, oracle, dev, pre, None, None, k_total)
    check_batch_select(pkg, oracle, dev, torch.full((B, F), 2.0), None, None, 2500)   # all equal: first 2500 flat indices
    check_batch_select(pkg, oracle, dev, -torch.ones(B, F), None, None, 100)          # nothing positive
    few = torch.zeros(B, F); few[1, 5] = 1.0; few[4, 1999] = 3.0
    code = check_batch_select(pkg, oracle, dev, few, None, None, 100)                 # fewer positives than k_total
    assert code.row_nnz.cpu().tolist() == [0, 1, 0, 0, 1, 0]
    code = check_batch_select(pkg, oracle, dev, few, None, None, 5000)                # the same with k_total beyond the candidate list
    assert code.row_nnz.cpu().tolist() == [0, 1, 0, 0, 1, 0]
    check_batch_select(pkg, oracle, dev, pre, None, None, 5000, k_on_device=True)     # k_total read on the device, beyond the list
    check_batch_select(pkg, oracle, dev, pre, None, None, 0)                          # k_total = 0 keeps nothing
    bfq = torch.randn(B, F, generator=g).bfloat16()                                   # bf16-quantised: natural ties
    check_batch_select(pkg, oracle, dev, bfq, None, None, 64 * B)
    # more keys at the threshold's level than the candidate list holds (B * F / 64 + 1024): the select then
    # re-reads the matrix; one token alone holds more of them than a wave collects at a time (512)
    wide = torch.randint(0, 3, (40, 8192), generator=g).float()
    wide[7] = 2.0
    for k_total in (50, 9000, 120000):
        check_batch_select(pkg, oracle, dev, wide, None, None, k_total)
    # the list holds them, but one token has more than 512: it is walked twice
    peaked = torch.randn(40, 8192, generator=g)
    peaked[11, 1000:3000] += 10.0
    check_batch_select(pkg, oracle, dev, peaked, None, None, 2500)
    check_batch_select(pkg, oracle, dev, peaked.bfloat16(), None, None, 2500)


def test_select_topk_batch_random_sweep(pkg, oracle, dev):
    """many small random cases against the oracle: shapes around the granule (64 / 32 elements) and list-capacity
    boundaries, quantised values (ties at the threshold), all three k regimes, bias / scale / mask on and off"""
    rng = np.random.default_rng(7)
    g = torch.Generator().manual_seed(7)
    for case in range(60):
        B = int(rng.integers(1, 40))
        F = int(rng.choice([1, 7, 31, 32, 33, 63, 64, 65, 127, 128, 200, 511, 512, 513, 1000, 2048, 4097]))
        dtype = torch.bfloat16 if rng.random() < 0.5 else torch.float32
        levels = int(rng.choice([0, 0, 3, 17]))                        # 0: continuous values
        pre = torch.randn(B, F, generator=g)
        if levels:
            pre = torch.round(pre * levels / 3) * 3 / levels          # few distinct values
        pre = pre.to(dtype)
        b_enc = 0.1 * torch.randn(F, generator=g) if rng.random() < 0.6 else None
        scale = 0.5 + torch.rand(F, generator=g) if rng.random() < 0.6 else None
        mask = (torch.rand(F, generator=g) < 0.5).float() if (scale is not None and rng.random() < 0.3) else None
        k_total = int(rng.choice([0, 1, B, max(1, B * F // 50), B * F // 3, B * F]))
        print(f"sweep case {case}: B={B} F={F} {dtype} levels={levels} k_total={k_total} "
              f"bias={b_enc is not None} scale={scale is not None} mask={mask is not None}", flush=True)
        check_batch_select(pkg, oracle, dev, pre, b_enc, scale, k_total, feat_mask=mask,
                           k_on_device=bool(k_total > 0 and rng.random() < 0.3))


def test_select_topk_batch_feature_mask(pkg, oracle, dev):
    """aux-k form: only masked-in (dead) features compete"""
    B, F = 16, 3000
    g = torch.Generator().manual_seed(4)
    pre = torch.randn(B, F, generator=g)
    b_enc = 0.1 * torch.randn(F, generator=g)
    scale = 0.5 + torch.rand(F, generator=g)
    mask = (torch.rand(F, generator=g) < 0.1).float()
    code = check_batch_select(pkg, oracle, dev, pre, b_enc, scale, 8 * B, feat_mask=mask)
    assert (mask[code.idx.cpu().long()[: code.row_nnz.sum().item()]] == 1).all()
    check_batch_select(pkg, oracle, dev, pre, b_enc, scale, 8 * B, feat_mask=torch.zeros(F))  # nothing is dead


@pytest.mark.gpu
@pytest.mark.parametrize("B,F,k", [(5, 4096, 16), (16, 24576, 64), (3, 1001, 8), (40, 8192, 200), (64, 32768, 32)])
def test_select_topk_batch_in_bf16_arithmetic(pkg, oracle, dev, B, F, k):
    """BatchTopK of a dictionary held in bf16: bias sum, norm product and final quotient are bf16 tensors in the
    reference (models/sae.py:324-341), and the closure's TopK runs over those bf16 values
    (models/sparse_dictionary.py:761-794).  The expected code is that op sequence on CPU bf16 tensors with the oracle's
    TopK over both axes; keys collide by the hundred at the threshold, where the lowest flattened indices are kept."""
    print(f"batch select lowp B={B} F={F} k={k}", flush=True)
    g = torch.Generator().manual_seed(F + k + 2)
    pre = torch.randn(B, F, generator=g).bfloat16()
    b_enc = (0.1 * torch.randn(F, generator=g)).bfloat16()
    norm = (0.5 + torch.rand(F, generator=g)).bfloat16()
    h1 = (pre + b_enc) * norm
    h1 = h1 * h1.gt(0).to(h1.dtype)
    want = oracle.topk(h1, k=k * B, dim=(-2, -1)) / norm
    assert want.dtype == torch.bfloat16
    for k_dev in (False, True):
        kt = torch.tensor(k * B, dtype=torch.int64, device=dev) if k_dev else k * B
        code = pkg.ops.select_topk_batch(pre.to(dev), b_enc.float().to(dev), norm.float().to(dev), kt, lowp=True,
                                         capacity=k * B if k_dev else None)
        got = code.to_dense().cpu()
        assert int(code.row_nnz.sum()) == k * B
        assert torch.equal(got != 0, want != 0), "kept sets differ"
        assert torch.equal(got, want.float()), "kept values differ"
    # the threshold's value is shared: a set of the same size with another tie order exists
    thr = h1[want != 0].float().min()
    if B * F >= 300000:
        assert (h1.float() == thr).sum() > ((want != 0) & (h1.float() == thr)).sum()
    # without bias and scale the arithmetic is the plain one
    plain = pkg.ops.select_topk_batch(pre.to(dev), None, None, k * B)
    lowp = pkg.ops.select_topk_batch(pre.to(dev), None, None, k * B, lowp=True)
    assert torch.equal(plain.to_dense(), lowp.to_dense())
    with pytest.raises(ValueError):
        pkg.ops.select_topk_batch(pre.float().to(dev), None, None, k * B, lowp=True)


@pytest.mark.gpu
@pytest.mark.parametrize("batch_wide", [False, True])
@pytest.mark.parametrize("B,F,k,with_norm", [(5, 4096, 16, True), (16, 24576, 64, True), (3, 1001, 8, True), (12, 8192, 40, False)])
def test_masked_select_in_bf16_arithmetic(pkg, oracle, dev, B, F, k, with_norm, batch_wide):
    """aux-k selection of a dictionary held in bf16: the keys are `hidden_pre * is_dead * decoder_norm` on bf16 tensors,
    hidden_pre being the quotient `encode` returned (models/sae.py:324-341, models/sparse_dictionary.py:958-970).  The
    expected code is that op sequence on CPU bf16 tensors with the oracle's TopK."""
    print(f"masked select lowp B={B} F={F} k={k} norm={with_norm} batch_wide={batch_wide}", flush=True)
    g = torch.Generator().manual_seed(F + k + 3)
    pre = torch.randn(B, F, generator=g).bfloat16()
    b_enc = (0.1 * torch.randn(F, generator=g)).bfloat16()
    norm = (0.5 + torch.rand(F, generator=g)).bfloat16() if with_norm else None
    dead = torch.rand(F, generator=g) < 0.3
    h1 = pre + b_enc
    if with_norm:
        h1 = h1 * norm
        hidden_pre = h1 / norm
        dead_pre = hidden_pre * dead * norm
    else:
        dead_pre = h1 * dead
    assert dead_pre.dtype == torch.bfloat16
    relu = dead_pre * dead_pre.gt(0).to(dead_pre.dtype)
    want = oracle.topk(relu, k=k * B, dim=(-2, -1)) if batch_wide else oracle.topk(relu, k=k, dim=-1)
    if with_norm:
        want = want / norm
    args = (pre.to(dev), b_enc.float().to(dev), None if norm is None else norm.float().to(dev))
    fm = dead.float().to(dev)
    if batch_wide:
        code = pkg.ops.select_topk_batch(*args, k * B, feat_mask=fm, lowp=True)
    else:
        code = pkg.ops.select_topk_row(*args, k, feat_mask=fm, lowp=True)
    got = code.to_dense().cpu()
    assert torch.equal(got != 0, want != 0), "kept sets differ"
    assert torch.equal(got, want.float()), "kept values differ"
    assert not got[:, ~dead].any()


@pytest.mark.gpu
def test_mfma_probe_runs_and_counts_its_flop(pkg, dev):
    flop, ms = pkg.ops.mfma_probe(dev, n_workgroups=64, iters=16)
    assert flop == 2.0 * 16 * 16 * 32 * 32 * 16 * 4 * 64
    assert ms > 0.0
    with pytest.raises(RuntimeError):
        pkg.ops.mfma_probe(dev, n_workgroups=0, iters=16)


@pytest.mark.parametrize("B,d,F", [(300, 128, 520), (256, 64, 256), (70, 192, 1030)])
def test_encoder_gemm_bias_epilogue(pkg, dev, B, d, F):
    """out = bf16(float(bf16(x @ w^T)) + col_bias + row_bias): bit for bit the plain product followed by the sums."""
    g = torch.Generator().manual_seed(B + F)
    x = torch.randn(B, d, generator=g).to(torch.bfloat16).to(dev)
    w = torch.randn(F, d, generator=g).to(torch.bfloat16).to(dev)
    cb = torch.randn(F, generator=g).to(dev)
    rb = torch.randn(B, generator=g).to(dev)
    plain = pkg.ops.encoder_gemm(x, w, torch.bfloat16).float()
    assert torch.equal(pkg.ops.encoder_gemm_bias(x, w, col_bias=cb), (plain + cb).to(torch.bfloat16))
    assert torch.equal(pkg.ops.encoder_gemm_bias(x, w, row_bias=rb), (plain + rb[:, None]).to(torch.bfloat16))
    assert torch.equal(pkg.ops.encoder_gemm_bias(x, w, cb, rb), ((plain + cb) + rb[:, None]).to(torch.bfloat16))
    assert torch.equal(pkg.ops.encoder_gemm_bias(x, w), plain.to(torch.bfloat16))


def test_sparse_decode_fused_accumulates_value_gradients_and_writes_in_place(pkg, dev):
    """sae_sparse_decode_mse_fused_acc: two decoders over prefixes of one code add their value gradients into one
    array (bit for bit the sum of the two separate results, taken in call order) and write their reconstructions and
    per-token losses into slices handed in."""
    g = torch.Generator().manual_seed(77)
    B, d, F, k = 50, 128, 600, 12
    idx = torch.stack([torch.randperm(F, generator=g)[:k].sort().values for _ in range(B)]).to(torch.int32)
    val = torch.rand(B, k, generator=g)
    code = pkg.ops.SparseCode(idx.reshape(-1).to(dev), val.reshape(-1).to(dev), (torch.arange(B) * k).to(dev),
                              torch.full((B,), k, dtype=torch.int32).to(dev), B, F)
    import dataclasses
    nnz_a = torch.randint(0, k + 1, (B,), generator=g).to(torch.int32).to(dev)
    codes = [dataclasses.replace(code, row_nnz=nnz_a), code]
    ws = [torch.randn(F, d, generator=g).to(dev) for _ in range(2)]
    labels = [torch.randn(B, d, generator=g).to(dev) for _ in range(2)]
    tok_w = torch.full((B,), 1.0 / B, device=dev)
    sep = [pkg.ops.sparse_decode_mse_fused(c, w, None, y, tok_w) for c, w, y in zip(codes, ws, labels)]
    recon = torch.empty(2, B, d, device=dev); loss = torch.empty(2, B, device=dev)
    acc = torch.zeros(B * k, device=dev)
    for j, (c, w, y) in enumerate(zip(codes, ws, labels)):
        r, lt, gr, dv = pkg.ops.sparse_decode_mse_fused(c, w, None, y, tok_w, recon_out=recon[j], loss_out=loss[j], dval_acc=acc)
        assert r.data_ptr() == recon[j].data_ptr() and dv.data_ptr() == acc.data_ptr()
        assert torch.equal(gr, sep[j][2]) and torch.equal(recon[j], sep[j][0]) and torch.equal(loss[j], sep[j][1])
    assert torch.equal(acc, sep[0][3] + sep[1][3])


def test_code_to_dense_transposed(pkg, dev):
    """sae_code_to_dense_t: the dense matrix of a sparse code, transposed, in bf16; ragged and empty rows."""
    g = torch.Generator().manual_seed(5)
    B, F, k = 70, 333, 9
    idx = torch.stack([torch.randperm(F, generator=g)[:k].sort().values for _ in range(B)]).to(torch.int32)
    val = torch.randn(B, k, generator=g)
    nnz = torch.randint(0, k + 1, (B,), generator=g).to(torch.int32)
    nnz[3] = 0
    code = pkg.ops.SparseCode(idx.reshape(-1).to(dev), val.reshape(-1).to(dev), (torch.arange(B) * k).to(dev), nnz.to(dev), B, F)
    want = torch.zeros(B, F)
    for r in range(B):
        want[r, idx[r, : nnz[r]].long()] = val[r, : nnz[r]]
    got = pkg.ops.code_to_dense_t(code, F)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (F, B)
    assert torch.equal(got.cpu(), want.t().to(torch.bfloat16))


def test_encoder_gemm_split_k(pkg, dev):
    """A bf16 -> fp32 product with few output tiles and a long contraction is cut along K: the slices' fp32 results summed
    in slice order equal the sum of the separately computed slice products bit for bit, and the product within fp32
    summation error of the unsplit kernel."""
    g = torch.Generator().manual_seed(9)
    B, d, F = 300, 8192, 520
    G = pkg.ops.gemm_split_k(B, d, F)
    assert G == 4 and pkg.ops.gemm_split_k(4096, 4096, 131072) == 1 and pkg.ops.gemm_split_k(300, 1024, 520) == 1
    x = torch.randn(B, d, generator=g).to(torch.bfloat16).to(dev)
    w = torch.randn(F, d, generator=g).to(torch.bfloat16).to(dev)
    got = pkg.ops.encoder_gemm(x, w, torch.float32)
    parts = [pkg.ops.encoder_gemm(x[:, i * d // G:(i + 1) * d // G].contiguous(), w[:, i * d // G:(i + 1) * d // G].contiguous(),
                                  torch.float32) for i in range(G)]
    assert torch.equal(got, torch.stack(parts).sum(0))
    want = x.double() @ w.double().t()
    assert ((got.double() - want).abs().max() / want.abs().max()).item() < 1e-5


@pytest.mark.parametrize("ascending", [True, False])
@pytest.mark.parametrize("G,B,k,F", [(4, 101, 16, 64), (1, 9, 8, 32), (3, 50, 64, 4096), (16, 7, 64, 256)])
def test_union_group_codes(pkg, dev, G, B, k, F, ascending):
    """Every (token, feature) of G stacked codes once, values summed in group order, order of first appearance; rows of
    unequal length, a token with an empty row in every group, and 16 x 64 = 1024 entries per token (the limit).  Rows in
    ascending feature order (what the select kernels write: searched by bisection) and in any order (compared pairwise)."""
    g = torch.Generator().manual_seed(G * 1000 + B)
    idx = torch.stack([torch.randperm(F, generator=g)[:k] for _ in range(G * B)]).to(torch.int32)    # distinct within a row
    val = torch.randn(G * B, k, generator=g)
    nnz = torch.randint(0, k + 1, (G * B,), generator=g, dtype=torch.int32)
    nnz[torch.arange(G) * B + (B - 1)] = 0           # the last token keeps nothing anywhere
    nnz[:B] = k                                      # group 0's rows are full
    if ascending:                                    # the live part of every row in ascending order
        for r in range(G * B):
            idx[r, :int(nnz[r])] = idx[r, :int(nnz[r])].sort().values
    code = pkg.ops.SparseCode(idx.flatten().to(dev), val.flatten().to(dev), (torch.arange(G * B) * k).to(dev), nnz.to(dev), G * B, F)
    got = pkg.ops.union_group_codes(code, G)
    assert got.n_tokens == B and got.d_sae == F and got.row_off.tolist() == [t * G * k for t in range(B)]
    gi, gv, gn = got.idx.view(B, G * k).cpu(), got.val.view(B, G * k).cpu(), got.row_nnz.tolist()
    for t in range(B):
        order, sums = [], {}
        for q in range(G):
            r = q * B + t
            for j in range(int(nnz[r])):
                f = int(idx[r, j])
                if f not in sums:
                    order.append(f)
                    sums[f] = np.float32(0.0)
                sums[f] = np.float32(sums[f] + np.float32(val[r, j]))
        assert gn[t] == len(order), t
        assert gi[t, :gn[t]].tolist() == order, t
        assert np.array_equal(gv[t, :gn[t]].numpy(), np.array([sums[f] for f in order], dtype=np.float32)), t
        assert not gi[t, gn[t]:].any() and not gv[t, gn[t]:].any()
    with pytest.raises(ValueError):
        pkg.ops.union_group_codes(code, G + 1)                       # rows that are not G + 1 groups of equally many tokens
    if G * k == 1024:
        wide = pkg.ops.SparseCode(torch.cat([code.idx, code.idx]), torch.cat([code.val, code.val]),
                                  (torch.arange(2 * G * B) * k).to(dev), torch.cat([code.row_nnz, code.row_nnz]), 2 * G * B, F)
        with pytest.raises(ValueError):
            pkg.ops.union_group_codes(wide, 2 * G)                   # 2048 entries per token
