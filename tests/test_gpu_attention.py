"""The causal attention kernels (grouped value heads, bf16 operands on the matrix cores) through the C ABI against
textbook attention in fp64 with an explicit [s, s] score matrix, on inputs that are exactly representable in bf16.

What separates the kernel from exact arithmetic is then only its own roundings: the probabilities are rounded to
bf16 before they multiply the values (2^-9 relative per term), dS likewise, and the outputs are bf16 tensors
(2^-9).  The bounds below are therefore a few 2^-9 of each tensor's largest element; the log-sum-exp, which
never leaves fp32, is held to 1e-5.  A wrong mask, head mapping, scale or a missing rescale of the running sums is
off by tens of percent.
"""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

OUT_TOL = 8e-3        # bf16 output + bf16 probabilities
GRAD_TOL = 2e-2       # bf16 gradients of sums of products of bf16-rounded factors
LSE_TOL = 1e-5


def bf16r(t):
    return t.to(torch.bfloat16).to(torch.float64)


def rel_max(got, want):
    return ((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def rel_frob(got, want):
    return ((got.double().cpu() - want).norm() / want.norm().clamp_min(1e-30)).item()


def reference(q, k, v, nb, s, h, scale):
    """q, k [T, h dq], v [T, h dv] fp64 leaves -> out [T, h dv], lse [nb, h, s]; causal softmax per (batch, head)."""
    dq, dv = q.shape[1] // h, v.shape[1] // h
    q4, k4, v4 = q.view(nb, s, h, dq), k.view(nb, s, h, dq), v.view(nb, s, h, dv)
    scores = torch.einsum("bqhd,bkhd->bhqk", q4, k4) * scale
    mask = torch.ones(s, s, dtype=torch.bool).tril()
    scores = scores.masked_fill(~mask, float("-inf"))
    lse = torch.logsumexp(scores, dim=-1)
    out = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(scores, dim=-1), v4)
    return out.reshape(nb * s, h * dv), lse


def make_case(nb, s, h, dq, dv, seed):
    g = torch.Generator().manual_seed(seed)
    T = nb * s
    q = bf16r(torch.randn(T, h * dq, generator=g))
    k = bf16r(torch.randn(T, h * dq, generator=g))
    v = bf16r(torch.randn(T, h * dv, generator=g))
    dout = bf16r(torch.randn(T, h * dv, generator=g))
    return q, k, v, dout


CASES = [
    # nb, seq, heads, d_qk, d_v
    (2, 64, 2, 32, 32),
    (1, 40, 3, 32, 64),          # ragged: one partial block
    (2, 72, 2, 64, 64),          # ragged second block
    (1, 200, 2, 64, 128),        # the benchmark's head widths, four key blocks, ragged tail
    (3, 128, 4, 64, 128),        # exactly one workgroup of queries per (sequence, head)
    (1, 8, 1, 64, 32),           # shortest sequence the kernels take
    (2, 136, 4, 64, 128),        # 8 (sequence, head) pairs: the XCD-aware workgroup order; a second workgroup of 8 queries
    (4, 72, 4, 32, 64),          # 16 pairs
    (1, 328, 2, 32, 128),        # three workgroups per head, ragged in both block sizes
    (2, 256, 8, 64, 32),
]


@pytest.mark.parametrize("nb,s,h,dq,dv", CASES)
def test_attention_forward_and_backward_against_fp64(pkg, dev, nb, s, h, dq, dv):
    print(f"attention case nb={nb} seq={s} heads={h} d_qk={dq} d_v={dv}", flush=True)
    q, k, v, dout = make_case(nb, s, h, dq, dv, seed=100 + s + dq + dv)
    scale = 1.0 / math.sqrt(dq)
    ql, kl, vl = q.clone().requires_grad_(), k.clone().requires_grad_(), v.clone().requires_grad_()
    want_out, want_lse = reference(ql, kl, vl, nb, s, h, scale)
    (want_out * dout).sum().backward()

    to_dev = lambda t: t.to(torch.bfloat16).to(dev).contiguous()                # noqa: E731
    gq, gk, gv, gdo = to_dev(q), to_dev(k), to_dev(v), to_dev(dout)
    out, lse = pkg.ops.attention_fwd(gq, gk, gv, nb, s, h, scale)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (nb * s, h * dv)
    assert rel_max(out, want_out.detach()) < OUT_TOL, rel_max(out, want_out.detach())
    assert (lse.double().cpu() - want_lse.detach()).abs().max().item() < LSE_TOL * max(1.0, want_lse.abs().max().item())

    dqt, dkt, dvt = pkg.ops.attention_bwd(gq, gk, gv, out, gdo, lse, nb, s, h, scale)
    torch.cuda.synchronize()
    errs = {"dq": (rel_max(dqt.t(), ql.grad), rel_frob(dqt.t(), ql.grad)),
            "dk": (rel_max(dkt.t(), kl.grad), rel_frob(dkt.t(), kl.grad)),
            "dv": (rel_max(dvt.t(), vl.grad), rel_frob(dvt.t(), vl.grad))}
    assert all(e[0] < GRAD_TOL and e[1] < GRAD_TOL / 2 for e in errs.values()), errs


def test_attention_at_the_benchmark_shape_on_sampled_heads(pkg, dev):
    """16 sequences x 1024 tokens, 64 heads of width 64 / 128 (8192 workgroups per kernel, every XCD slot used): forward
    and the three gradients of a few (sequence, head) pairs against fp64 attention computed on the device."""
    nb, s, h, dq, dv = 16, 1024, 64, 64, 128
    g = torch.Generator(device=dev).manual_seed(11)
    T = nb * s
    q, k, v, do = (torch.randn(T, h * w, device=dev, generator=g).to(torch.bfloat16) for w in (dq, dq, dv, dv))
    scale = 1.0 / math.sqrt(dq)
    out, lse = pkg.ops.attention_fwd(q, k, v, nb, s, h, scale)
    dqt, dkt, dvt = pkg.ops.attention_bwd(q, k, v, out, do, lse, nb, s, h, scale)
    mask = torch.ones(s, s, dtype=torch.bool, device=dev).tril()
    for b, hh in ((0, 0), (7, 33), (15, 63), (3, 8)):
        rows = slice(b * s, (b + 1) * s)
        ql = q[rows, hh * dq:(hh + 1) * dq].double().requires_grad_()
        kl = k[rows, hh * dq:(hh + 1) * dq].double().requires_grad_()
        vl = v[rows, hh * dv:(hh + 1) * dv].double().requires_grad_()
        sc = (ql @ kl.t() * scale).masked_fill(~mask, float("-inf"))
        want = torch.softmax(sc, -1) @ vl
        (want * do[rows, hh * dv:(hh + 1) * dv].double()).sum().backward()
        rel = lambda a, w: ((a.double() - w).abs().max() / w.abs().max()).item()     # noqa: E731
        assert rel(out[rows, hh * dv:(hh + 1) * dv], want.detach()) < OUT_TOL
        assert (lse[b, hh].double() - torch.logsumexp(sc.detach(), -1)).abs().max().item() < 1e-4
        assert rel(dqt[hh * dq:(hh + 1) * dq, rows].t(), ql.grad) < GRAD_TOL
        assert rel(dkt[hh * dq:(hh + 1) * dq, rows].t(), kl.grad) < GRAD_TOL
        assert rel(dvt[hh * dv:(hh + 1) * dv, rows].t(), vl.grad) < GRAD_TOL


def test_attention_is_causal_and_sequences_do_not_mix(pkg, dev):
    """Changing a later position, or another sequence of the batch, leaves every earlier output bit-identical."""
    nb, s, h, dq, dv = 2, 96, 2, 64, 128
    q, k, v, _ = make_case(nb, s, h, dq, dv, seed=7)
    to_dev = lambda t: t.to(torch.bfloat16).to(dev).contiguous()                # noqa: E731
    gq, gk, gv = to_dev(q), to_dev(k), to_dev(v)
    out0, lse0 = pkg.ops.attention_fwd(gq, gk, gv, nb, s, h, 0.125)
    cut = 50
    gk2, gv2 = gk.clone(), gv.clone()
    gk2[cut:s] = 3.0          # later positions of sequence 0
    gv2[cut:s] = -2.0
    gk2[s + 10:] = 1.5        # and a stretch of sequence 1
    out1, lse1 = pkg.ops.attention_fwd(gq, gk2, gv2, nb, s, h, 0.125)
    assert torch.equal(out0[:cut], out1[:cut]) and torch.equal(lse0[0, :, :cut], lse1[0, :, :cut])
    assert torch.equal(out0[s:s + 10], out1[s:s + 10])
    assert not torch.equal(out0[cut:s], out1[cut:s])
    # the first position attends to itself only
    assert torch.equal(out0[0].float(), gv[0].float())


def test_attention_rejects_shapes_it_is_not_built_for(pkg, dev):
    z = torch.zeros(16, 48, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="d_qk"):
        pkg.ops.attention_fwd(z, z, z, 1, 16, 1, 1.0)          # d_qk = 48
    z = torch.zeros(12, 32, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        pkg.ops.attention_fwd(z, z, z, 1, 12, 1, 1.0)
    assert not pkg.ops.attention_shapes_supported(12, 32, 32) and pkg.ops.attention_shapes_supported(1024, 64, 128)


def test_row_sum(pkg, dev):
    g = torch.Generator().manual_seed(3)
    src = torch.randn(37, 1000, generator=g)
    assert rel_max(pkg.ops.row_sum(src.to(dev)), src.double().sum(1)) < 1e-6
    b = src.to(torch.bfloat16)
    assert rel_max(pkg.ops.row_sum(b.to(dev)), b.double().sum(1)) < 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("nb,seq,h,dq,rd,adjacent,with_bias", [(2, 16, 3, 32, 32, True, True), (2, 16, 3, 32, 32, False, True),
                                                           (1, 40, 2, 64, 32, True, False), (3, 8, 5, 64, 48, False, True),
                                                           (2, 24, 4, 16, 16, True, True), (16, 1024, 64, 64, 64, True, True)])
def test_rotary_kernels_follow_the_reference_sequence(pkg, oracle, dev, nb, seq, h, dq, rd, adjacent, with_bias):
    """models/lorsa.py:864-904 under bf16 autocast: the bf16 product plus the fp32 bias is an fp32 tensor, rotated in
    fp32 (x * cos + flip(x) * sin), and the attention rounds it to bf16.  The expected values are that sequence with
    torch on the CPU, its backward torch's autograd through it; both must be reproduced to the bit."""
    import importlib
    vo = importlib.import_module("oracle.variants_oracle")
    print(f"rotary nb={nb} seq={seq} h={h} dq={dq} rd={rd} adjacent={adjacent} bias={with_bias}", flush=True)
    n_ctx = seq + 8
    g = torch.Generator().manual_seed(seq * dq + rd)
    T = nb * seq
    acc = torch.randn(T, h * dq, generator=g)
    bias = 0.3 * torch.randn(h * dq, generator=g) if with_bias else None
    sin, cos = vo.rotary_sin_cos(rd, n_ctx, 10000, adjacent)

    def rotate(x4):      # [b, s, h, dq] fp32, the reference's sequence
        x_rot, x_pass = x4[..., :rd], x4[..., rd:]
        flip = x_rot.clone()
        if adjacent:
            flip[..., ::2] = -x_rot[..., 1::2]
            flip[..., 1::2] = x_rot[..., ::2]
        else:
            n = rd // 2
            flip[..., :n] = -x_rot[..., n:]
            flip[..., n:] = x_rot[..., :n]
        return torch.cat([x_rot * cos[None, :seq, None, :] + flip * sin[None, :seq, None, :], x_pass], dim=-1)

    x = (acc.bfloat16().float() + (bias if with_bias else 0.0)).view(nb, seq, h, dq).requires_grad_(True)
    y = rotate(x)
    want = y.detach().bfloat16().view(T, h * dq)
    got = pkg.ops.rotary_fwd(acc.to(dev), None if bias is None else bias.to(dev), cos.to(dev), sin.to(dev), seq, h, rd, adjacent)
    assert torch.equal(got.cpu(), want)
    # backward: a bf16 gradient with respect to y, held transposed [h dq, T]
    dy = torch.randn(T, h * dq, generator=g).bfloat16()
    y.backward(dy.float().view(nb, seq, h, dq))
    want_dx_t = x.grad.view(T, h * dq).bfloat16().t().contiguous()
    grad_t = dy.t().contiguous().to(dev)
    pkg.ops.rotary_bwd_t(grad_t, cos.t().contiguous().to(dev), sin.t().contiguous().to(dev), seq, h, rd, adjacent)
    assert torch.equal(grad_t.cpu(), want_dx_t)
