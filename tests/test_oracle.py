"""Pins the CPU oracle (oracle/ti_oracle.c) before anything is compared with it.

Checks are chosen so that a plausible mistake in the oracle (dropped term,
transposed operand, wrong rounding mode, extra/missing fp32 rounding, clamp
and round in the wrong order) fails at least one of them:
  * integer accumulation against four independent routes and the literal
    matrices held by upstream tests/test_bmm.py;
  * fp32 epilogues against exact rational arithmetic with a single final
    rounding, and against hand-computed ties / saturation / ReLU cases;
  * LayerNorm-quant against torch's own ops and an fp64 computation.
"""
import json
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _rand_s8(gen, *shape, lo=-128, hi=128):
    return torch.randint(lo, hi, shape, dtype=torch.int8, generator=gen)


# ------------------------------------------------------------------ accumulation

@pytest.mark.parametrize("M,N,K", [(1, 4, 16), (1, 16, 16), (3, 5, 7), (33, 65, 129), (128, 96, 512), (7, 1, 1)])
def test_acc_routes_agree(M, N, K):
    g = torch.Generator().manual_seed(M * 1000 + N * 10 + K)
    a, b = _rand_s8(g, M, K), _rand_s8(g, N, K)
    acc = orc.gemm_acc(a, b)
    assert acc.dtype == torch.int32 and acc.shape == (M, N)
    via_np = a.numpy().astype(np.int64) @ b.numpy().astype(np.int64).T
    via_f64 = (a.double() @ b.double().T).round().long()
    assert np.array_equal(acc.numpy().astype(np.int64), via_np)
    assert torch.equal(acc.long(), via_f64)
    assert torch.equal(acc, orc.gemm_acc_torch(a, b))
    assert torch.equal(acc.long(), orc.gemm_acc_naive64(a, b))


def test_acc_batched_and_extremes():
    g = torch.Generator().manual_seed(7)
    a, b = _rand_s8(g, 5, 9, 48), _rand_s8(g, 5, 11, 48)
    acc = orc.gemm_acc(a, b)
    ref = torch.einsum("bmk,bnk->bmn", a.long(), b.long())
    assert torch.equal(acc.long(), ref)
    # each batch uses its own B: permuting the batches of B changes the result
    assert not torch.equal(acc, orc.gemm_acc(a, b.flip(0)))
    # -128 * -128 * K is the largest product sum
    a = torch.full((2, 4096), -128, dtype=torch.int8)
    assert orc.gemm_acc(a, a)[0, 0].item() == 128 * 128 * 4096
    # transposition sanity: A.B^T, not A^T.B or A.B
    a = torch.tensor([[1, 2], [3, 4]], dtype=torch.int8)
    b = torch.tensor([[5, 6], [7, 8]], dtype=torch.int8)
    assert orc.gemm_acc(a, b).tolist() == [[17, 23], [39, 53]]


def test_literal_fixture_from_upstream_tests():
    with open(os.path.join(GOLDEN, "bmm_literal_16x16.json")) as f:
        fx = json.load(f)
    a = torch.tensor(fx["a"], dtype=torch.int8)[None]
    b_nk = torch.tensor(fx["b_kn"], dtype=torch.int8).t().contiguous()[None]  # upstream passes B^T
    assert orc.bmm_s8t_s8n_s32t(a, b_nk)[0].tolist() == fx["acc"]
    assert orc.bmm_s8t_s8n_s8t(a, b_nk, fx["scale"])[0].tolist() == fx["expected_s8"]
    # the expectation upstream computes itself (tests/test_bmm.py:99-101)
    c_gt = (torch.bmm(a.float(), b_nk.float().transpose(1, 2)) * fx["scale"]).round().clamp(-128, 127)
    assert torch.equal(c_gt.to(torch.int8), orc.bmm_s8t_s8n_s8t(a, b_nk, fx["scale"]))


# ------------------------------------------------------------------ epilogues

def _f32(x):
    return float(np.float32(x))


def _round_to_f32(fr):
    """Correctly rounded (nearest-even) fp32 value of an exact rational."""
    if fr == 0:
        return 0.0
    # numpy rounds a Python float (53 bits) to fp32; go through exact integer scaling
    # instead so there is only one rounding.
    sign = -1 if fr < 0 else 1
    fr = abs(fr)
    e = 0
    while fr >= 2 ** 24:
        fr /= 2
        e += 1
    while fr < 2 ** 23:
        fr *= 2
        e -= 1
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return sign * float(fl) * 2.0 ** e


def test_fp32_epilogue_is_one_fma_of_separately_rounded_bias_term():
    rng = np.random.default_rng(0)
    n = 4000
    acc = torch.from_numpy(rng.integers(-2 ** 23, 2 ** 23, n).astype(np.int32))
    bias = torch.from_numpy(rng.standard_normal(n).astype(np.float32))
    alpha, beta = 0.0037, 0.83
    out = orc.epi_bfp32_ofp32(acc.view(1, n), bias, alpha, beta)[0]
    a32, b32 = np.float32(alpha), np.float32(beta)
    n_differs_from_unfused = 0
    for i in range(n):
        bb = np.float32(b32 * bias[i].numpy())  # first rounding
        exact = Fraction(float(a32)) * int(acc[i]) + Fraction(float(bb))
        assert out[i].item() == _round_to_f32(exact), i
        unfused = np.float32(np.float32(a32 * np.float32(int(acc[i]))) + bb)
        n_differs_from_unfused += int(unfused != out[i].numpy())
    # the check can tell the two forms apart on this data
    assert n_differs_from_unfused > 0


def _rint_half_even(fr):
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return fl


@pytest.mark.parametrize("which", ["b8_o8", "relu_b8_o8", "b32_o32_scaled"])
def test_integer_output_epilogues_are_one_fma_then_one_rint(which):
    """The s8, ReLU-s8 and scaled-s32 epilogues against exact rationals: t = fp32(alpha * f32(acc) + fp32(beta * bias))
    with ONE rounding of the sum (an fma), then round-half-even and the clamp.  The cases are searched for, not drawn:
    only inputs on which a separately rounded product followed by an add would produce a different integer are kept,
    so an oracle that slipped to mul + add fails every one of them."""
    a32, b32 = np.float32(0.0037), np.float32(0.83)
    if which == "b32_o32_scaled":
        rng = np.random.default_rng(5)
        acc = rng.integers(-2 ** 31, 2 ** 31, 400000).astype(np.int64)
        bias = rng.integers(-2 ** 20, 2 ** 20, acc.size).astype(np.int64)
    else:  # every accumulator whose scaled value lands in the int8 range, against a spread of int8 bias values
        acc = np.repeat(np.arange(-36000, 36001, dtype=np.int64), 128)
        bias = np.tile(np.arange(-127, 128, 2, dtype=np.int64)[:128], acc.size // 128)
    accf = acc.astype(np.float32)                        # int32 -> fp32, round to nearest even
    bt = (b32 * bias.astype(np.float32)).astype(np.float32)      # the separately rounded bias term
    fused = (accf.astype(np.float64) * np.float64(a32) + bt.astype(np.float64)).astype(np.float32)
    unfused = ((a32 * accf).astype(np.float32) + bt).astype(np.float32)
    tell = np.nonzero(np.rint(fused.astype(np.float64)) != np.rint(unfused.astype(np.float64)))[0]
    assert tell.size >= 20, tell.size            # the search found inputs that tell the two forms apart
    tell = tell[:300]
    acc_t = torch.from_numpy(acc[tell].astype(np.int32)).view(1, -1)
    if which == "b32_o32_scaled":
        out = orc.epi_b32_o32_scaled(acc_t, torch.from_numpy(bias[tell].astype(np.int32)), float(a32), float(b32))[0]
    else:
        out = orc.epi_b8_o8(acc_t, torch.from_numpy(bias[tell].astype(np.int8)), float(a32), float(b32),
                            relu=which == "relu_b8_o8")[0]
    n_unfused_differs = 0
    for j, i in enumerate(tell):
        bb = Fraction(float(bt[i]))
        t = Fraction(_round_to_f32(Fraction(float(a32)) * Fraction(float(accf[i])) + bb))   # the one rounding of the fma
        if which == "b32_o32_scaled":
            want = max(min(_rint_half_even(t), 2 ** 31 - 1), -2 ** 31)
            other = max(min(int(np.rint(np.float64(unfused[i]))), 2 ** 31 - 1), -2 ** 31)
        else:
            lo = 0 if which == "relu_b8_o8" else -128
            want = max(min(_rint_half_even(t), 127), lo)
            other = max(min(int(np.rint(np.float64(unfused[i]))), 127), lo)
        assert out[j].item() == want, (which, int(acc[i]), int(bias[i]))
        n_unfused_differs += int(other != want)
    assert n_unfused_differs > 0


def test_int_to_float_conversion_rounds_to_nearest_even():
    acc = torch.tensor([2 ** 24 + 1, 2 ** 24 + 3, -(2 ** 24 + 1), 2 ** 31 - 1, -2 ** 31], dtype=torch.int32)
    out = orc.epi_f32t(acc, 1.0)
    assert out.tolist() == [2.0 ** 24, 2.0 ** 24 + 4, -(2.0 ** 24), 2.0 ** 31, -(2.0 ** 31)]


def test_f32t_and_s8t_epilogues_are_one_rounded_multiply():
    # alpha * f32(acc): one fp32 product of the (already rounded) converted accumulator, against exact rationals
    rng = np.random.default_rng(1)
    acc = torch.from_numpy(np.concatenate([rng.integers(-2 ** 31, 2 ** 31, 1500), rng.integers(-40000, 40000, 1500)])
                           .astype(np.int32))
    alpha = 0.0186   # the scale of upstream's literal test (tests/test_bmm.py:99)
    out = orc.epi_f32t(acc, alpha)
    out8 = orc.epi_s8t(acc, alpha)
    a32 = Fraction(float(np.float32(alpha)))
    for i in range(acc.numel()):
        conv = Fraction(float(np.float32(int(acc[i]))))          # int32 -> fp32, first rounding
        want = _round_to_f32(a32 * conv)
        assert out[i].item() == want, i
        t = Fraction(want)
        lo = max(min(t, Fraction(127)), Fraction(-128))           # clamp, then round half to even
        fl = lo.numerator // lo.denominator
        rem = lo - fl
        if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
            fl += 1
        assert out8[i].item() == fl, i


def test_s8_epilogue_identity_ties_and_saturation():
    acc = torch.arange(-140, 141, dtype=torch.int32).view(1, -1)
    n = acc.numel()
    zero_b = torch.zeros(n, dtype=torch.int8)
    ident = orc.epi_b8_o8(acc, zero_b, 1.0, 0.0)
    assert torch.equal(ident, acc.clamp(-128, 127).to(torch.int8))
    assert torch.equal(orc.epi_s8t(acc, 1.0), ident)
    # alpha = 0.5: odd accumulators land on .5 and go to the even neighbour
    half = orc.epi_b8_o8(torch.tensor([[1, 3, 5, 7, -1, -3, -5, 255, 257, -257]], dtype=torch.int32),
                         torch.zeros(10, dtype=torch.int8), 0.5, 0.0)
    assert half.tolist() == [[0, 2, 2, 4, 0, -2, -2, 127, 127, -128]]
    # clamp happens before rounding: 127.5 -> 127 (rounding first would give 128 -> overflow)
    assert orc.epi_s8t(torch.tensor([255, -257, 10 ** 9, -10 ** 9], dtype=torch.int32), 0.5).tolist() == \
        [127, -128, 127, -128]
    # alpha = 0 leaves rne(beta * bias)
    bias = torch.tensor([-128, -3, -1, 0, 1, 3, 127], dtype=torch.int8)
    only_bias = orc.epi_b8_o8(torch.full((1, 7), 12345, dtype=torch.int32), bias, 0.0, 0.5)
    assert only_bias.tolist() == [[-64, -2, 0, 0, 0, 2, 64]]  # -1.5->-2, -.5->-0, .5->0, 1.5->2, 63.5->64
    # per-column bias, shared by all rows
    two_rows = orc.epi_b8_o8(torch.zeros((2, 3), dtype=torch.int32), torch.tensor([1, 2, 3], dtype=torch.int8),
                             1.0, 1.0)
    assert two_rows.tolist() == [[1, 2, 3], [1, 2, 3]]


def test_relu_epilogue():
    acc = torch.tensor([[-300, -1, 0, 1, 3, 253, 255, 1000]], dtype=torch.int32)
    out = orc.epi_b8_o8(acc, torch.zeros(8, dtype=torch.int8), 0.5, 0.0, relu=True)
    assert out.tolist() == [[0, 0, 0, 0, 2, 126, 127, 127]]
    # bias can lift a negative product above zero
    out = orc.epi_b8_o8(torch.tensor([[-4]], dtype=torch.int32), torch.tensor([10], dtype=torch.int8), 1.0, 1.0,
                        relu=True)
    assert out.tolist() == [[6]]


def test_s32_epilogues():
    acc = torch.tensor([[2 ** 31 - 1, -2 ** 31, 5, -7]], dtype=torch.int32)
    bias = torch.tensor([1, -1, 10, 3], dtype=torch.int32)
    # wrapping add, as torch int32 addition does
    assert torch.equal(orc.epi_b32_o32(acc, bias), acc + bias)
    assert orc.epi_b32_o32(acc, bias).tolist() == [[-2 ** 31, 2 ** 31 - 1, 15, -4]]
    small = torch.tensor([[1, 3, -3, 1000]], dtype=torch.int32)
    zb = torch.zeros(4, dtype=torch.int32)
    assert orc.epi_b32_o32_scaled(small, zb, 0.5, 0.0).tolist() == [[0, 2, -2, 500]]
    assert orc.epi_b32_o32_scaled(small, torch.tensor([2, 2, 2, 2], dtype=torch.int32), 1.0, 0.25).tolist() == \
        [[2, 4, -2, 1000]]  # 1.5->2, 3.5->4, -2.5->-2, 1000.5->1000
    big = torch.tensor([[2 ** 30, -2 ** 30]], dtype=torch.int32)
    assert orc.epi_b32_o32_scaled(big, torch.zeros(2, dtype=torch.int32), 4.0, 0.0).tolist() == \
        [[2 ** 31 - 1, -2 ** 31]]


@pytest.mark.parametrize("relu", [False, True])
def test_s8_linear_matches_upstream_test_expectation_within_one_lsb(relu):
    # upstream tests/test_linear_kernels.py:55-84: fp32 nn.Linear with scaled weights,
    # clamp then round; agreement is only promised to +-1 LSB there.
    g = torch.Generator().manual_seed(3)
    x, w = _rand_s8(g, 128, 512, lo=-127, hi=127), _rand_s8(g, 1024, 512, lo=-127, hi=127)
    bias = _rand_s8(g, 1024, lo=-127, hi=127)
    alpha, beta = 0.001, 0.01
    y_gt = torch.nn.functional.linear(x.float(), w.float() * alpha, bias.float() * beta)
    y_gt = y_gt.clamp(0 if relu else -128, 127).round()
    fn = orc.linear_relu_a8_w8_b8_o8 if relu else orc.linear_a8_w8_b8_o8
    y = fn(x, w, bias, alpha, beta)
    assert (y.float() - y_gt).abs().max().item() <= 1
    assert (y.float() != y_gt).float().mean().item() < 0.01


def test_fp32_and_scaled_linear_match_upstream_test_expectation():
    # upstream tests/test_linear_kernels.py:22-51 (atol 0.5 there; fp32 accumulation noise only)
    g = torch.Generator().manual_seed(4)
    x, w = _rand_s8(g, 128, 512, lo=-127, hi=127), _rand_s8(g, 1024, 512, lo=-127, hi=127)
    bias = torch.randn(1024, generator=g)
    y = orc.linear_a8_w8_bfp32_ofp32(x, w, bias, 0.001, 1.0)
    y_gt = (x.double() @ w.double().T) * float(np.float32(0.001)) + bias.double()
    assert torch.allclose(y.double(), y_gt, rtol=1e-6, atol=1e-4)
    ibias = torch.randint(-2 ** 31, 2 ** 31 - 1, (1024,), dtype=torch.int64, generator=g).to(torch.int32)
    y = orc.linear_a8_w8_b32_o32_with_scaling(x, w, ibias, 0.01, 0.0001)
    y_gt = (x.double() @ w.double().T) * 0.01 + ibias.double() * 0.0001
    assert (y.double() - y_gt).abs().max().item() <= 1.0
    y = orc.linear_a8_w8_b32_o32(x, w, ibias)
    assert torch.equal(y, (x.int() @ w.int().T) + ibias)


# ------------------------------------------------------------------ dq_add_layernorm_q

def _torch_dq_add_ln_q(inp, s, res, gamma, beta, eps):
    # upstream torch_int/functional/fused.py:5-12, restated
    r = torch.add(res, inp, alpha=s)
    y = torch.nn.functional.layer_norm(r, r.shape[-1:], gamma, beta, eps)
    return r, y.clamp(-128, 127).round().to(torch.int8)


@pytest.mark.parametrize("shape", [(2, 3, 4), (5, 768), (3, 5120), (4, 1023), (2, 9216), (1, 1)])
def test_ln_q_against_torch_and_fp64(shape):
    g = torch.Generator().manual_seed(sum(shape))
    H = shape[-1]
    inp = torch.randint(-65536, 65536, shape, dtype=torch.int32, generator=g)
    res = torch.randn(shape, generator=g)
    gamma = 1 + 0.02 * torch.randn(H, generator=g)
    beta = 0.02 * torch.randn(H, generator=g)
    gamma, beta = gamma * 20, beta * 20  # spread q over the int8 range
    s, eps = 0.01, 1e-5
    r, q = orc.dq_add_layernorm_q(inp, s, res, gamma, beta, eps)
    r_t, q_t = _torch_dq_add_ln_q(inp, s, res, gamma, beta, eps)
    # r: one fma; torch may or may not fuse -> within 1 ulp
    ulp = torch.abs(r_t) * 2 ** -23 + 1e-30
    assert ((r - r_t).abs() <= ulp).all()
    # and exactly the single-rounding value
    s32 = np.float32(s)
    exact = (inp.double() * float(s32) + res.double())
    assert torch.equal(r, exact.float())  # fp64 holds the fma exactly here (|in| < 2^17)
    assert (q.int() - q_t.int()).abs().max().item() <= 1
    assert (q != q_t).float().mean().item() <= 0.01 + 1.0 / q.numel()
    rd = r.double()
    mu = rd.mean(-1, keepdim=True)
    var = ((rd - mu) ** 2).mean(-1, keepdim=True)
    y64 = (rd - mu) / torch.sqrt(var + eps) * gamma.double() + beta.double()
    q64 = y64.clamp(-128, 127).round().to(torch.int8)
    assert (q.int() - q64.int()).abs().max().item() <= 1
    assert (q != q64).float().mean().item() <= 0.01 + 1.0 / q.numel()


def test_ln_q_invariants():
    H = 640
    gamma = torch.full((H,), 3.0)
    beta = torch.linspace(-140, 140, H)
    # constant row: variance 0, output is rne(clamp(beta))
    inp = torch.full((1, H), 100, dtype=torch.int32)
    res = torch.full((1, H), 0.25)
    r, q = orc.dq_add_layernorm_q(inp, 0.5, res, gamma, beta, 1e-5)
    assert torch.equal(r, torch.full((1, H), 50.25))
    assert torch.equal(q[0], beta.clamp(-128, 127).round().to(torch.int8))
    # gamma = 1, beta = 0 on a symmetric row: q is antisymmetric and sums to 0
    half = torch.arange(1, H // 2 + 1, dtype=torch.int32) * 37
    inp = torch.cat([half, -half]).view(1, H)
    r, q = orc.dq_add_layernorm_q(inp, 1.0, torch.zeros(1, H), torch.ones(H) * 50, torch.zeros(H), 1e-5)
    assert q.int().sum().item() == 0
    assert torch.equal(q[0, : H // 2], -q[0, H // 2:])
    # rows are independent
    g = torch.Generator().manual_seed(1)
    inp = torch.randint(-65536, 65536, (6, H), dtype=torch.int32, generator=g)
    res = torch.randn(6, H, generator=g)
    r_all, q_all = orc.dq_add_layernorm_q(inp, 0.01, res, gamma, beta * 0, 1e-5)
    r_one, q_one = orc.dq_add_layernorm_q(inp[4:5], 0.01, res[4:5], gamma, beta * 0, 1e-5)
    assert torch.equal(r_all[4:5], r_one) and torch.equal(q_all[4:5], q_one)


# ------------------------------------------------------------------ fused chains of the OPT blocks

def test_add_layernorm_q_against_torch():
    # upstream models/opt.py:281-283 + nn/fused.py:13-18, restated with torch ops
    g = torch.Generator().manual_seed(11)
    for shape in [(6, 768), (2, 5120), (3, 1023), (4, 1)]:
        H = shape[-1]
        x, res = torch.randn(shape, generator=g), torch.randn(shape, generator=g) * 2
        gamma = (1 + 0.02 * torch.randn(H, generator=g)) * 30
        beta = torch.randn(H, generator=g)
        r, q = orc.add_layernorm_q(x, res, gamma, beta, 1e-5)
        assert torch.equal(r, res + x)
        ref = torch.nn.functional.layer_norm(res + x, (H,), gamma, beta, 1e-5).round().clamp(-128, 127).to(torch.int8)
        assert (q.int() - ref.int()).abs().max().item() <= 1
        assert (q != ref).float().mean().item() <= 0.01 + 1.0 / q.numel()
        r0, q0 = orc.add_layernorm_q(None, res + x, gamma, beta, 1e-5)
        assert torch.equal(q0, q)  # adding first or passing the sum is the same thing


def test_attn_softmax_q_against_torch():
    # upstream models/opt.py:144-178, restated with torch ops
    neg = torch.finfo(torch.float32).min
    g = torch.Generator().manual_seed(12)
    for (B, H, T, S) in [(2, 3, 8, 8), (1, 2, 5, 131), (2, 2, 16, 512), (1, 1, 3, 1)]:
        scores = torch.randn(B * H, T, S, generator=g) * 8
        mask = torch.zeros(B, 1, T, S)
        mask.masked_fill_(torch.arange(S)[None, :] > torch.arange(S - T, S)[:, None] + (S < T) * T, neg)
        for m in (mask, None):
            q = orc.attn_softmax_q(scores, m, H)
            s = scores.view(B, H, T, S)
            if m is not None:
                s = torch.clamp_min(s + m, neg)
            p = torch.softmax(s.double(), -1)  # fp64 route
            ref = (p * 127).round().to(torch.int8).view(B * H, T, S)
            assert (q.int() - ref.int()).abs().max().item() <= 1
            assert (q != ref).float().mean().item() <= 1e-3 + 1.0 / q.numel()
            assert int(q.min()) >= 0 and int(q.max()) <= 127
            # every row sums to 127 up to rounding of its entries
            assert (q.int().sum(-1) - 127).abs().max().item() <= S // 2 + 1
    # a fully masked row degenerates to the uniform distribution, like softmax of equal inputs
    q = orc.attn_softmax_q(torch.randn(1, 1, 8, generator=g), torch.full((1, 1, 1, 8), neg), 1)
    assert q.tolist() == [[[16] * 8]]  # round(127 / 8) = 16


# ------------------------------------------------------------------ fp16 residual stream

def test_f16_conversion_matches_numpy():
    g = torch.Generator().manual_seed(0)
    x = torch.cat([torch.randn(3000, generator=g) * torch.logspace(-9, 5.2, 3000),
                   torch.tensor([0.0, -0.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e9, -1e9, float("inf"), -float("inf"),
                                 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -14, 2.0 ** -14 * 0.9999, 6.1e-5,
                                 5.96e-8, 1.0009765625, 1.00048828125, 1.00146484375])])   # ties, subnormals, overflow
    bits, back = orc.f16_round_trip(x)
    with np.errstate(over="ignore"):
        ref = x.numpy().astype(np.float16)
    assert np.array_equal(bits.numpy().astype(np.uint16), ref.view(np.uint16))
    assert np.array_equal(back.numpy(), ref.astype(np.float32))


@pytest.mark.parametrize("shape", [(2, 3, 4), (5, 768), (3, 1023), (2, 5120)])
def test_ln_q_f16_against_torch_ops_in_fp32(shape):
    # the GPU chain of ATen ops on fp16 tensors computes in fp32 and rounds every tensor it produces to fp16
    g = torch.Generator().manual_seed(sum(shape))
    H = shape[-1]
    inp = torch.randint(-60000, 60000, shape, dtype=torch.int32, generator=g)
    res = torch.randn(shape, generator=g).half()
    gamma = ((1 + 0.02 * torch.randn(H, generator=g)) * 20).half()
    beta = (0.4 * torch.randn(H, generator=g)).half()
    s = 0.0037
    r, q = orc.dq_add_layernorm_q_f16(inp, s, res, gamma, beta, 1e-5)
    assert r.dtype == torch.float16 and q.dtype == torch.int8
    # torch.add casts the int32 operand to the common dtype (fp16) before the fp32 arithmetic
    r_t = torch.add(res.float(), inp.half().float(), alpha=s).half()
    # identical but for a double-rounding tie now and then (torch's fp32 add is within 1 ulp of the fma)
    assert (r != r_t).float().mean() < 1e-3 and ((r.float() - r_t.float()).abs() <= r_t.float().abs() * 2 ** -10).all()
    y_t = torch.nn.functional.layer_norm(r.float(), (H,), gamma.float(), beta.float(), 1e-5).half()
    q_t = y_t.float().clamp(-128, 127).round().to(torch.int8)
    assert (q.int() - q_t.int()).abs().max() <= 1 and (q != q_t).float().mean() <= 0.01 + 1.0 / q.numel()
    # the add + LayerNormQ chain, with and without the add
    x = torch.randn(shape, generator=g).half()
    r2, q2 = orc.add_layernorm_q_f16(x, res, gamma, beta, 1e-5)
    assert torch.equal(r2, (res.float() + x.float()).half())
    y_t = torch.nn.functional.layer_norm(r2.float(), (H,), gamma.float(), beta.float(), 1e-5).half()
    q_t = y_t.float().clamp(-128, 127).round().to(torch.int8)
    assert (q2.int() - q_t.int()).abs().max() <= 1 and (q2 != q_t).float().mean() <= 0.01 + 1.0 / q2.numel()
    r3, q3 = orc.add_layernorm_q_f16(None, r2, gamma, beta, 1e-5)
    assert torch.equal(r3, r2) and torch.equal(q3, q2)
    # an fp32 addend on the fp16 stream, `residual.add_(x32.to(residual.dtype))`: rounded to fp16 first, so the
    # result is the all-fp16 form on the rounded addend -- and differs from the single rounding of res + x32
    x32 = torch.randn(shape, generator=g) * 3 + 1e-4 * torch.randn(shape, generator=g)
    r4, q4 = orc.add_layernorm_q_f16(x32, res, gamma, beta, 1e-5)
    r5, q5 = orc.add_layernorm_q_f16(x32.half(), res, gamma, beta, 1e-5)
    assert torch.equal(r4, r5) and torch.equal(q4, q5)
    assert torch.equal(r4, res.clone().add_(x32.to(res.dtype)))          # torch's own in-place fp16 add on the CPU
    if res.numel() >= 1000:
        assert not torch.equal(r4, (res.float() + x32).half())


def test_ln_q_f16_rounds_the_normalised_value_to_half_before_the_integer():
    # one row where fp16 rounding of y decides the integer: y = 65.47 -> fp16 65.5 -> 66 (fp32 alone gives 65)
    H = 4
    res = torch.tensor([[1.0, -1.0, 1.0, -1.0]]).half()          # mean 0, variance 1
    gamma = torch.tensor([65.47, 64.47, 1.0, 1.0]).half()
    beta = torch.zeros(H).half()
    _, q = orc.add_layernorm_q_f16(None, res, gamma, beta, 0.0)
    g32 = gamma.float()
    y = (res.float()[0] * g32)
    assert q[0].tolist() == y.half().float().round().to(torch.int8).tolist()
