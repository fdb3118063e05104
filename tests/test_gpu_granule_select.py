"""The granule route of the per-token TopK: the encoder GEMM's per-granule key maxima and the select that reads the
row only where those maxima allow a kept element, against the kernels they stand in for.  Everything here is
integer-exact: the same pre-activations (bit for bit), the same keys, the same kept indices and values."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(B, d, F, seed, dev, scale_kind="random", bias=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, d, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(F, d, generator=g) / d ** 0.5).to(torch.bfloat16).to(dev)
    b = (0.1 * torch.randn(F, generator=g)).to(dev) if bias else None
    s = None
    if scale_kind == "random":
        s = (0.5 + torch.rand(F, generator=g)).to(dev)
    return x, w, b, s


def _keys(pre, b, s):
    h1 = pre.float()
    if b is not None:
        h1 = h1 + b
    if s is not None:
        h1 = h1 * s
    bits = h1.contiguous().view(torch.int32)
    return torch.where(h1 > 0, bits, torch.zeros_like(bits))


@pytest.mark.parametrize("B,d,F", [(300, 128, 1024), (256, 256, 4096), (77, 64, 192), (512, 64, 64)])
@pytest.mark.parametrize("bias,scale_kind", [(True, "random"), (False, None)])
def test_gemm_granule_max_matches_keys_of_its_own_output(pkg, dev, B, d, F, bias, scale_kind):
    x, w, b, s = _inputs(B, d, F, seed=B + F, dev=dev, scale_kind=scale_kind, bias=bias)
    pre, gmax = pkg.ops.encoder_gemm_granule_max(x, w, b, s)
    want_pre = pkg.ops.encoder_gemm(x, w, torch.bfloat16)
    assert torch.equal(pre, want_pre)
    want = _keys(pre, b, s).view(B, F // 64, 64).max(dim=2).values     # positive-float bits order like ints
    assert torch.equal(gmax, want)


CASES = [
    # B, d, F, k
    (128, 128, 2048, 16),
    (300, 128, 8192, 64),
    (64, 64, 64, 8),          # one granule
    (96, 128, 1024, 512),     # the largest k the route takes
    (50, 256, 16384, 100),
]


@pytest.mark.parametrize("B,d,F,k", CASES)
def test_granule_select_equals_row_select(pkg, dev, B, d, F, k):
    x, w, b, s = _inputs(B, d, F, seed=3 * B + k, dev=dev)
    pre, gmax = pkg.ops.encoder_gemm_granule_max(x, w, b, s)
    got = pkg.ops.select_topk_row(pre, b, s, k, granule_max=gmax)
    want = pkg.ops.select_topk_row(pre, b, s, k)
    assert torch.equal(got.row_nnz, want.row_nnz) and torch.equal(got.row_off, want.row_off)
    assert torch.equal(got.idx, want.idx) and torch.equal(got.val, want.val)


@pytest.mark.parametrize("B,d,F,k", [(128, 128, 2048, 16), (300, 128, 8192, 64), (64, 64, 256, 8), (256, 256, 16384, 100)])
def test_granule_route_in_bf16_arithmetic(pkg, dev, B, d, F, k):
    """A dictionary held in bf16: the product's epilogue forms the granule maxima from keys in bf16 arithmetic, and the
    per-token and the batch-wide select that read them return what their full-row forms in that arithmetic return."""
    x, w, b, s = _inputs(B, d, F, seed=5 * B + k, dev=dev)
    b, s = b.bfloat16().float(), s.bfloat16().float()          # the bias and the norms of such a dictionary are bf16 values
    pre, gmax = pkg.ops.encoder_gemm_granule_max(x, w, b, s, lowp=True)
    assert torch.equal(pre, pkg.ops.encoder_gemm(x, w, torch.bfloat16))
    h1 = ((pre + b.bfloat16()) * s.bfloat16()).float()        # bf16 tensors: each operation rounds
    bits = h1.contiguous().view(torch.int32)
    want_max = torch.where(h1 > 0, bits, torch.zeros_like(bits)).view(B, F // 64, 64).max(dim=2).values
    assert torch.equal(gmax, want_max)
    plain_max = pkg.ops.encoder_gemm_granule_max(x, w, b, s)[1]
    assert not torch.equal(gmax, plain_max)                   # the fp32 keys are other numbers
    got = pkg.ops.select_topk_row(pre, b, s, k, granule_max=gmax, lowp=True)
    want = pkg.ops.select_topk_row(pre, b, s, k, lowp=True)
    assert torch.equal(got.row_nnz, want.row_nnz) and torch.equal(got.idx, want.idx) and torch.equal(got.val, want.val)
    if F % 256 == 0:
        got = pkg.ops.select_topk_batch(pre, b, s, k * B, granule_max=gmax, lowp=True)
        want = pkg.ops.select_topk_batch(pre, b, s, k * B, lowp=True)
        assert torch.equal(got.row_nnz, want.row_nnz) and torch.equal(got.row_off, want.row_off)
        n = int(want.row_nnz.sum())
        assert n == k * B and torch.equal(got.idx[:n], want.idx[:n]) and torch.equal(got.val[:n], want.val[:n])


def _granule_max_of(pre, b, s):
    B, F = pre.shape
    return _keys(pre, b, s).view(B, F // 64, 64).max(dim=2).values.contiguous()


def test_granule_select_degenerate_rows(pkg, dev):
    """Rows with no positive entry, with fewer positive entries than k (spread over few granules and over many), rows
    of one repeated value (mass ties: the candidate list overflows and the general kernel redoes the row), and ties
    at the threshold inside and across granules.  The granule maxima are formed here from the same keys."""
    B, F, k = 12, 4096, 32
    g = torch.Generator().manual_seed(11)
    pre = torch.randn(B, F, generator=g)
    pre[0] = -pre[0].abs()                                   # nothing positive
    pre[1] = -pre[1].abs(); pre[1, 5:15] = 1.0               # 10 positives, all equal, one granule
    pre[2] = -pre[2].abs(); pre[2, ::300] = torch.arange(1, 15).float()   # 14 positives over 14 granules
    pre[3] = 0.75                                            # every entry equal: 4096 ties
    pre[4] = -1.0; pre[4, 100:1500] = 2.0                    # 1400 ties: more than the candidate list holds
    pre[5] = pre[5].abs(); pre[5, 64:64 + 40] = 9.0          # 40 ties above everything, one granule: k - 40 more from the rest
    pre[6] = -1.0; pre[6, 0::64] = 3.0                       # one tie per granule, 64 granules: lowest 32 indices win
    pre[7] = -1.0; pre[7, 63::64] = 3.0; pre[7, 10] = 3.0
    pre = pre.to(torch.bfloat16).to(dev)
    b = torch.zeros(F, device=dev)
    s = torch.ones(F, device=dev)
    gmax = _granule_max_of(pre, b, s)
    got = pkg.ops.select_topk_row(pre, b, s, k, granule_max=gmax)
    want = pkg.ops.select_topk_row(pre, b, s, k)
    assert torch.equal(got.row_nnz, want.row_nnz), (got.row_nnz, want.row_nnz)
    assert torch.equal(got.idx, want.idx) and torch.equal(got.val, want.val)
    nnz = got.row_nnz.tolist()
    assert nnz[0] == 0 and nnz[1] == 10 and nnz[2] == 14 and nnz[3] == k and nnz[4] == k
    assert got.idx.view(B, k)[6].tolist() == list(range(0, 64 * k, 64))
    assert got.idx.view(B, k)[3].tolist() == list(range(k))


def test_granule_route_is_what_the_fused_step_runs_and_changes_nothing(pkg, dev):
    from lm_saes_amd import synthetic

    d, F, k, B = 128, 2048, 16, 256
    x = synthetic.activations(B, d, 8, seed=5)
    w = synthetic.sae_weights(d, F, x, seed=5)

    calls = []
    real = pkg.ops.encoder_gemm_granule_max

    def spy(*a, **kw):
        calls.append(1)
        return real(*a, **kw)

    def run(granule):
        cfg = pkg.SAEConfig(hook_point_in="in", hook_point_out="out", d_model=d, expansion_factor=F / d, act_fn="topk",
                            top_k=k, norm_activation="inference", device="cuda", dtype=torch.float32)
        m = pkg.SparseAutoEncoder(cfg)
        synthetic.load_weights(m, *[t.to(dev) for t in w])
        m.granule_select = granule
        batch = {"in": x.to(dev), "out": x.to(dev), "tokens": torch.zeros(B, device=dev)}
        with torch.autocast("cuda", dtype=torch.bfloat16):
            loss = m.compute_loss(batch, return_aux_data=False)
        loss.backward()
        return loss.detach(), {n: p.grad for n, p in m.named_parameters()}

    pkg.ops.encoder_gemm_granule_max = spy
    try:
        la, ga = run(True)
        assert len(calls) == 1
        lb, gb = run(False)
        assert len(calls) == 1
    finally:
        pkg.ops.encoder_gemm_granule_max = real
    assert torch.equal(la, lb)
    for n in ga:
        assert (ga[n] is None) == (gb[n] is None), n
        if ga[n] is not None:
            assert torch.equal(ga[n], gb[n]), n


def test_grouped_gemm_select_and_merge_equal_the_per_layer_route(pkg, dev):
    """L products in one launch, one select over the L * B stacked rows with a bias / scale vector per group, and the
    merge kernel -- against L separate products and selects merged through a sort of (token, layer, feature) keys."""
    from lm_saes_amd.clt import merge_layer_codes

    L, B, d, F, k = 5, 200, 128, 1024, 24
    g = torch.Generator().manual_seed(17)
    x = torch.randn(L, B, d, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(L, F, d, generator=g) / d ** 0.5).to(torch.bfloat16).to(dev)
    b = (0.1 * torch.randn(L, F, generator=g)).to(dev)
    s = (0.5 + torch.rand(L, F, generator=g)).to(dev)
    x[2, 7] = 0          # a token with nothing positive in layer 2 but for the bias
    b[3] = -5.0          # a layer that keeps (almost) nothing
    pre_all, gmax = pkg.ops.encoder_gemm_granule_max(x, w, b, s)
    for l in range(L):
        assert torch.equal(pre_all[l], pkg.ops.encoder_gemm(x[l], w[l], torch.bfloat16))
    stacked = pkg.ops.select_topk_row(pre_all.view(L * B, F), b, s, k, granule_max=gmax.view(L * B, -1), rows_per_group=B)
    codes = [pkg.ops.select_topk_row(pre_all[l], b[l], s[l], k) for l in range(L)]
    for l, c in enumerate(codes):
        assert torch.equal(stacked.row_nnz[l * B:(l + 1) * B], c.row_nnz)
        assert torch.equal(stacked.idx[l * B * k:(l + 1) * B * k], c.idx) and torch.equal(stacked.val[l * B * k:(l + 1) * B * k], c.val)
    got, got_cnt = pkg.ops.merge_layer_codes(stacked, L)
    want, want_cnt = merge_layer_codes(codes)
    assert torch.equal(got_cnt, want_cnt) and torch.equal(got.row_nnz, want.row_nnz)
    assert got.d_sae == want.d_sae == L * F and got.n_tokens == B
    # the two lay their rows out differently (fixed L * k slots per token against packed rows): compare row by row
    gi, gv = got.idx.view(B, L * k), got.val.view(B, L * k)
    nnz = got.row_nnz.tolist()
    off = want.row_off.tolist()
    for t in range(B):
        assert torch.equal(gi[t, :nnz[t]], want.idx[off[t]:off[t] + nnz[t]]), t
        assert torch.equal(gv[t, :nnz[t]], want.val[off[t]:off[t] + nnz[t]]), t
        assert not gi[t, nnz[t]:].any() and not gv[t, nnz[t]:].any()
    assert got.row_off.tolist() == [t * L * k for t in range(B)]


@pytest.mark.parametrize("B,F,groups", [(300, 1024, 1), (64, 8192, 1), (96, 256, 3)])
def test_standalone_granule_max(pkg, dev, B, F, groups):
    g = torch.Generator().manual_seed(B + F)
    pre = torch.randn(B, F, generator=g).to(torch.bfloat16).to(dev)
    b = (0.1 * torch.randn(groups, F, generator=g)).to(dev)
    s = (0.5 + torch.rand(groups, F, generator=g)).to(dev)
    rpg = B // groups
    got = pkg.ops.granule_max(pre, b.view(-1) if groups == 1 else b, s.view(-1) if groups == 1 else s, rows_per_group=0 if groups == 1 else rpg)
    rows_b = b.repeat_interleave(rpg, dim=0)
    rows_s = s.repeat_interleave(rpg, dim=0)
    h1 = (pre.float() + rows_b) * rows_s
    bits = h1.contiguous().view(torch.int32)
    want = torch.where(h1 > 0, bits, torch.zeros_like(bits)).view(B, F // 64, 64).max(dim=2).values
    assert torch.equal(got, want)
    # and with neither bias nor scale
    got0 = pkg.ops.granule_max(pre, None, None)
    h0 = pre.float()
    want0 = torch.where(h0 > 0, h0.contiguous().view(torch.int32), torch.zeros(B, F, dtype=torch.int32, device=dev)).view(B, F // 64, 64).max(dim=2).values
    assert torch.equal(got0, want0)
    k = 16
    a = pkg.ops.select_topk_row(pre, None, None, k, granule_max=got0)
    w = pkg.ops.select_topk_row(pre, None, None, k)
    assert torch.equal(a.idx, w.idx) and torch.equal(a.val, w.val) and torch.equal(a.row_nnz, w.row_nnz)


@pytest.mark.parametrize("B,d,F,k", [(64, 64, 256, 4), (300, 128, 1024, 16), (128, 64, 2048, 100)])
def test_batch_select_with_granule_maxima_equals_batch_select(pkg, dev, B, d, F, k):
    x, w, b, s = _inputs(B, d, F, seed=B + 5 * k, dev=dev)
    pre, gmax = pkg.ops.encoder_gemm_granule_max(x, w, b, s)
    got = pkg.ops.select_topk_batch(pre, b, s, k * B, granule_max=gmax)
    want = pkg.ops.select_topk_batch(pre, b, s, k * B)
    assert torch.equal(got.row_nnz, want.row_nnz) and torch.equal(got.row_off, want.row_off)
    assert torch.equal(got.idx, want.idx) and torch.equal(got.val, want.val)
    # nothing kept, and more asked for than there are positive entries
    zero = pkg.ops.select_topk_batch(pre, b, s, 0, granule_max=gmax)
    assert int(zero.row_nnz.sum()) == 0
    every = pkg.ops.select_topk_batch(pre, b, s, B * F, granule_max=gmax)
    ref = pkg.ops.select_topk_batch(pre, b, s, B * F)
    assert torch.equal(every.row_nnz, ref.row_nnz) and torch.equal(every.idx, ref.idx) and torch.equal(every.val, ref.val)


@pytest.mark.parametrize("H,B,F,k", [(3, 70, 1024, 8), (4, 128, 4096, 32), (2, 33, 512, 64)])
def test_groups_of_scales_over_one_shared_matrix(pkg, dev, H, B, F, k):
    """`n_rows = H * B`: H groups of rows share ONE pre-activation matrix [B, F], each group selecting under a bias / scale
    vector of its own (a crosscoder's heads).  The maxima equal those of the explicitly repeated matrix, and the one stacked
    select equals, bit for bit, H selects of the row kernel."""
    print(f"shared-matrix select H={H} B={B} F={F} k={k}", flush=True)
    g = torch.Generator().manual_seed(H * 1000 + F + k)
    pre = torch.randn(B, F, generator=g).bfloat16().to(dev)
    bias = (0.1 * torch.randn(H, F, generator=g)).to(dev)
    scale = (0.25 + 1.5 * torch.rand(H, F, generator=g)).to(dev)
    gmax = pkg.ops.granule_max(pre, bias, scale, rows_per_group=B, n_rows=H * B)
    want_gmax = pkg.ops.granule_max(pre.repeat(H, 1), bias, scale, rows_per_group=B)
    assert torch.equal(gmax, want_gmax)
    code = pkg.ops.select_topk_row(pre, bias, scale, k, granule_max=gmax, rows_per_group=B, n_rows=H * B)
    assert code.n_tokens == H * B
    for h in range(H):
        want = pkg.ops.select_topk_row(pre, bias[h].contiguous(), scale[h].contiguous(), k)
        sl, rows = slice(h * B * k, (h + 1) * B * k), slice(h * B, (h + 1) * B)
        assert torch.equal(code.idx[sl], want.idx) and torch.equal(code.val[sl], want.val)
        assert torch.equal(code.row_nnz[rows], want.row_nnz) and torch.equal(code.row_off[rows] - h * B * k, want.row_off)
