"""Parity of the HIP kernels with the CPU oracle, through torch_int._CUDA -> C ABI.

Bars: bit-exact for int32 and int8 outputs; fp32 outputs within 1 ulp (in practice 0:
the kernels and the oracle spell the same fma).  Inputs are generated on the CPU from a
seeded generator and copied to the GPU, so both sides see identical bytes.
"""
import json
import os
import sys

import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DEV = "cuda:0"


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _s8(g, *shape, lo=-127, hi=128):
    return torch.randint(lo, hi, shape, dtype=torch.int8, generator=g)


def _scal(g, lo, hi):
    return float(torch.empty(1).uniform_(lo, hi, generator=g).item())


def _ulp_diff(a, b):
    """max distance in units of the last place between two fp32 tensors."""
    ai = a.contiguous().view(torch.int32).long()
    bi = b.contiguous().view(torch.int32).long()
    ai = torch.where(ai < 0, -(ai & 0x7fffffff), ai)
    bi = torch.where(bi < 0, -(bi & 0x7fffffff), bi)
    return (ai - bi).abs().max().item() if a.numel() else 0


@pytest.fixture
def two_launch_split_k():
    """Split-K linears take the two-launch form (raw int32 slices + reduction kernel) even where the one-launch form
    would run, so that the tests that walk through the kernel families still reach those kernels."""
    import torch_int._CUDA as C
    before = C._lib.ti_fused_splitk(0)
    yield
    C._lib.ti_fused_splitk(before)


def _linear_case(C, variant, M, N, K, seed, alpha=None, beta=None):
    g = torch.Generator().manual_seed(seed)
    x, w = _s8(g, M, K), _s8(g, N, K)
    alpha = _scal(g, 1e-4, 1e-2) if alpha is None else alpha
    beta = _scal(g, 1e-4, 1e-2) if beta is None else beta
    if variant == "b32_o32":
        bias = torch.randint(-65535, 65535, (N,), dtype=torch.int32, generator=g)
        ref = orc.linear_a8_w8_b32_o32(x, w, bias)
        out = C.linear_a8_w8_b32_o32(x.to(DEV), w.to(DEV), bias.to(DEV))
    elif variant == "b32_o32_scaled":
        bias = torch.randint(-2 ** 31, 2 ** 31 - 1, (N,), dtype=torch.int64, generator=g).to(torch.int32)
        ref = orc.linear_a8_w8_b32_o32_with_scaling(x, w, bias, alpha, beta)
        out = C.linear_a8_w8_b32_o32_with_scaling(x.to(DEV), w.to(DEV), bias.to(DEV), alpha, beta)
    elif variant == "bfp32_ofp32":
        bias = torch.randn(N, generator=g)
        ref = orc.linear_a8_w8_bfp32_ofp32(x, w, bias, alpha, beta)
        out = C.linear_a8_w8_bfp32_ofp32(x.to(DEV), w.to(DEV), bias.to(DEV), alpha, beta)
    elif variant == "b8_o8":
        bias = _s8(g, N)
        ref = orc.linear_a8_w8_b8_o8(x, w, bias, alpha, beta)
        out = C.linear_a8_w8_b8_o8(x.to(DEV), w.to(DEV), bias.to(DEV), alpha, beta)
    elif variant == "relu_b8_o8":
        bias = _s8(g, N)
        ref = orc.linear_relu_a8_w8_b8_o8(x, w, bias, alpha, beta)
        out = C.linear_relu_a8_w8_b8_o8(x.to(DEV), w.to(DEV), bias.to(DEV), alpha, beta)
    else:
        raise AssertionError(variant)
    out = out.cpu()
    assert out.shape == ref.shape and out.dtype == ref.dtype
    if out.dtype == torch.float32:
        assert _ulp_diff(out, ref) <= 1, f"{variant} {M}x{N}x{K}: {_ulp_diff(out, ref)} ulp"
    else:
        nbad = (out != ref).sum().item()
        assert nbad == 0, f"{variant} {M}x{N}x{K}: {nbad} mismatches"
    return out


VARIANTS = ["b32_o32", "b32_o32_scaled", "bfp32_ofp32", "b8_o8", "relu_b8_o8"]

# (M, N, K): upstream minimum shapes (tests/test_linear_shape.py:9,26), upstream kernel
# test shape (tests/test_linear_kernels.py:8), ragged edges, every tile family.
LINEAR_SHAPES = [
    (1, 4, 16), (1, 16, 16), (128, 1024, 512), (3, 20, 48), (65, 100, 272), (64, 64, 128),
    (130, 260, 400), (257, 513, 1040), (300, 768, 768), (512, 1024, 256),
]


@pytest.mark.parametrize("variant", VARIANTS)
def test_linear_shapes(variant):
    import torch_int._CUDA as C
    for i, (M, N, K) in enumerate(LINEAR_SHAPES):
        _say(f"linear {variant} M={M} N={N} K={K}")
        _linear_case(C, variant, M, N, K, seed=100 + i)


@pytest.mark.parametrize("variant", VARIANTS)
def test_linear_large_tiles(variant):
    # enough 256x256 tiles to select the large-tile kernel, with ragged M and N
    import torch_int._CUDA as C
    for (M, N, K) in [(2048, 5120, 256), (2100, 5000, 272), (4096, 2560, 128), (4000, 2816, 1024), (4090, 2790, 256),
                      (2010, 5120, 384), (1990, 9216, 128), (2040, 5120, 128), (2048, 2560, 640),
                      # 256x128 tiles (widths that 160 and 288 do not divide, or fill worse), 256x160 tiles under 160 tiles of 256x256
                      (2048, 4096, 2048), (1100, 4096, 2048), (1600, 5120, 2048), (1290, 5120, 2176)]:
        _say(f"linear-large {variant} M={M} N={N} K={K}")
        _linear_case(C, variant, M, N, K, seed=7)


def test_every_gemm_kernel_family_is_reached_and_exact(two_launch_split_k):
    # one shape per dispatch branch; the library reports which kernel family it launched
    import ctypes
    import torch_int._CUDA as C
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    expect = [((2048, 5120, 256), "pipe16_256x160"), ((2048, 5120, 192), "pipe16_256x160"),
              ((2000, 9216, 192), "pipe16_256x288"), ((2000, 9216, 384), "pipe16_256x288"),
              ((4096, 2816, 192), "pipe_256x256"),
              ((4096, 2816, 128), "pipe_256x256"), ((1024, 2048, 64), "pipe_128x128"),
              ((2048, 4096, 2048), "pipe16_256x128"), ((1280, 5120, 2048), "pipe16_256x128"), ((1600, 5120, 2048), "pipe16_256x160"),
              ((2048, 2048, 2048), "pipe_128x128"), ((2048, 7168, 2048), "pipe_256x256"), ((2048, 4096, 256), "pipe_128x128"),
              ((512, 5120, 5120), "pipe16_128x80"), ((384, 2560, 1024), "pipe16_128x80"), ((1024, 5120, 5120), "splitk_256x160"),
              ((256, 3200, 11648), "splitk_256x160"), ((1024, 9216, 9216), "splitk_256x288"),
              ((384, 2880, 4608), "splitk_128x80"), ((128, 640, 4096), "splitk_128x80"),
              ((256, 1600, 11648), "splitk_128x160"), ((1024, 4608, 3584), "splitk_128x288"),
              ((768, 3072, 11648), "splitk_256x256"), ((256, 3072, 7744), "splitk_256x256"),  # 128- and 64-byte steps
              ((128, 1024, 4096), "splitk_128x128"), ((256, 2048, 11648), "splitk_128x128"),
              ((512, 3072, 1024), "splitk_128x192"), ((128, 768, 4096), "splitk_128x192"), ((512, 12288, 2048), "pipe16_128x192"),
              ((1024, 12288, 1024), "pipe16_256x192"), ((256, 49152, 1024), "pipe16_256x192"),
              ((16, 5120, 3072), "stream"), ((3, 4608, 16384), "stream"), ((3, 100, 272), "skinny"), ((300, 200, 48), "tile_64x64"),
              ((2100, 5000, 272), "tile_256x256"), ((1024, 2048, 80), "tile_128x128"), ((70, 50, 37), "scalar")]
    for (M, N, K), family in expect:
        for variant in ("b8_o8", "bfp32_ofp32"):
            _say(f"family {family} {variant} M={M} N={N} K={K}")
            _linear_case(C, variant, M, N, K, seed=55)
            assert C._lib.ti_last_kernel().decode() == family, (M, N, K, C._lib.ti_last_kernel())


@pytest.mark.parametrize("variant", VARIANTS)
def test_linear_split_k_and_decode_shapes(variant):
    # few output tiles and a long K: the K loop is split over workgroups (with and without the
    # scratch workspace the Python wrapper provides); M <= 16 with K % 1024 == 0: streaming kernel
    import torch_int._CUDA as C
    for (M, N, K) in [(128, 640, 4096), (100, 520, 2048), (512, 1280, 5120), (40, 256, 8192),
                      (1, 4096, 2048), (4, 4112, 1024), (16, 5120, 3072), (9, 4100, 5120)]:
        _say(f"linear-splitk/decode {variant} M={M} N={N} K={K}")
        _linear_case(C, variant, M, N, K, seed=21)


def test_split_k_matches_unsplit_through_the_c_abi():
    # same call with and without a workspace must give identical bytes
    import torch_int._CUDA as C
    g = torch.Generator().manual_seed(3)
    M, N, K = 128, 640, 4096
    x, w, b = _s8(g, M, K).to(DEV), _s8(g, N, K).to(DEV), _s8(g, N).to(DEV)
    need = C._lib.ti_linear_workspace_bytes(M, N, K)
    assert need > 0
    outs = []
    for ws_bytes in (0, need):
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=DEV)
        out = torch.empty((M, N), dtype=torch.int8, device=DEV)
        rc = C._lib.ti_linear_a8_w8_b8_o8(x.data_ptr(), w.data_ptr(), b.data_ptr(), out.data_ptr(), M, N, K,
                                          0.002, 0.01, ws.data_ptr() if ws_bytes else None, ws_bytes,
                                          torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        outs.append(out.cpu())
    assert torch.equal(outs[0], outs[1])
    assert torch.equal(outs[0], orc.linear_a8_w8_b8_o8(x.cpu(), w.cpu(), b.cpu(), 0.002, 0.01))


def test_linear_opt125m_config():
    # the single-linear benchmark configuration at OPT-125m width: x [4,512,768], W [768,768], bias [768], alpha 1e-3, beta 1e-2, seed 0
    import torch_int._CUDA as C
    _say("linear C1")
    out = _linear_case(C, "b8_o8", 2048, 768, 768, seed=0, alpha=0.001, beta=0.01)
    assert (out == 127).any() and (out == -128).any()  # saturates by design


def test_linear_odd_k_and_bias_shapes():
    import torch_int._CUDA as C
    for (M, N, K) in [(5, 7, 13), (33, 17, 100), (1, 128, 513)]:
        for v in VARIANTS:
            _say(f"linear-odd {v} M={M} N={N} K={K}")
            _linear_case(C, v, M, N, K, seed=11)
    g = torch.Generator().manual_seed(5)
    x, w, b = _s8(g, 8, 32), _s8(g, 16, 32), _s8(g, 16)
    ref = orc.linear_a8_w8_b8_o8(x, w, b, 0.01, 0.5)
    out = C.linear_a8_w8_b8_o8(x.to(DEV), w.to(DEV), b.view(1, 16).to(DEV), 0.01, 0.5)  # [1,N] bias as modules hold it
    assert torch.equal(out.cpu(), ref)
    out = C.linear_a8_w8_b8_o8(x.to(DEV), w.to(DEV), b, 0.01, 0.5)  # CPU bias is moved like upstream does
    assert torch.equal(out.cpu(), ref)
    assert C.linear_a8_w8_b8_o8(x[:0].to(DEV), w.to(DEV), b.to(DEV), 1.0, 1.0).shape == (0, 16)


def test_linear_ties_and_saturation_on_device():
    import torch_int._CUDA as C
    # K = 16 ones against small integers: acc = sum of a row, alpha = 0.5 produces exact .5 ties
    x = torch.zeros(64, 16, dtype=torch.int8)
    x[:, 0] = torch.arange(-32, 32, dtype=torch.int8)
    x[:, 1] = 127
    x[:, 2] = torch.arange(0, 64, dtype=torch.int8)
    w = torch.zeros(16, 16, dtype=torch.int8)
    w[:, 0] = 1
    w[8:, 1] = 2
    w[4:12, 2] = -3
    bias = torch.arange(-8, 8, dtype=torch.int8)
    for alpha, beta in [(0.5, 0.5), (0.5, 0.0), (1.0, 0.0), (0.25, 1.0), (0.0, 0.5)]:
        for fn_name in ["linear_a8_w8_b8_o8", "linear_relu_a8_w8_b8_o8"]:
            _say(f"ties {fn_name} alpha={alpha} beta={beta}")
            ref = getattr(orc, fn_name)(x, w, bias, alpha, beta)
            out = getattr(C, fn_name)(x.to(DEV), w.to(DEV), bias.to(DEV), alpha, beta).cpu()
            assert torch.equal(out, ref)
    ib = bias.to(torch.int32) * 1000
    ref = orc.linear_a8_w8_b32_o32_with_scaling(x, w, ib, 0.5, 0.0005)
    out = C.linear_a8_w8_b32_o32_with_scaling(x.to(DEV), w.to(DEV), ib.to(DEV), 0.5, 0.0005).cpu()
    assert torch.equal(out, ref)
    ref = orc.linear_a8_w8_b32_o32_with_scaling(x, w, ib, 3e7, 1.0)  # saturates int32
    out = C.linear_a8_w8_b32_o32_with_scaling(x.to(DEV), w.to(DEV), ib.to(DEV), 3e7, 1.0).cpu()
    assert torch.equal(out, ref) and (out == 2 ** 31 - 1).any() and (out == -2 ** 31).any()


def test_linear_large_accumulators_round_like_the_oracle():
    # |acc| > 2^24: the int32 -> fp32 conversion is inexact and must round to nearest even
    import torch_int._CUDA as C
    M, N, K = 32, 32, 4096
    x = torch.full((M, K), 127, dtype=torch.int8)
    w = torch.full((N, K), 127, dtype=torch.int8)
    g = torch.Generator().manual_seed(2)
    x[:, :64] = _s8(g, M, 64)
    w[:, 64:128] = _s8(g, N, 64)
    bias = torch.randn(N, generator=g)
    ref = orc.linear_a8_w8_bfp32_ofp32(x, w, bias, 1.0, 1.0)
    assert ref.abs().max() > 2 ** 25
    out = C.linear_a8_w8_bfp32_ofp32(x.to(DEV), w.to(DEV), bias.to(DEV), 1.0, 1.0).cpu()
    assert _ulp_diff(out, ref) == 0
    ib = torch.zeros(N, dtype=torch.int32)
    assert torch.equal(C.linear_a8_w8_b32_o32(x.to(DEV), w.to(DEV), ib.to(DEV)).cpu(),
                       orc.linear_a8_w8_b32_o32(x, w, ib))


# ------------------------------------------------------------------ batched products

def _bmm_case(C, B, M, N, K, seed, prob_lhs=False):
    g = torch.Generator().manual_seed(seed)
    a = _s8(g, B, M, K, lo=0 if prob_lhs else -127)
    b = _s8(g, B, N, K)
    alpha = _scal(g, 1e-3 if prob_lhs else 1e-4, 1e-2)
    ad, bd = a.to(DEV), b.to(DEV)
    ref32 = orc.bmm_s8t_s8n_s32t(a, b)
    assert torch.equal(C.bmm_s8t_s8n_s32t(ad, bd).cpu(), ref32), f"s32t {B}x{M}x{N}x{K}"
    out8 = C.bmm_s8t_s8n_s8t(ad, bd, alpha).cpu()
    assert torch.equal(out8, orc.epi_s8t(ref32, alpha)), f"s8t {B}x{M}x{N}x{K}"
    outf = C.bmm_s8t_s8n_f32t(ad, bd, alpha).cpu()
    assert _ulp_diff(outf, orc.epi_f32t(ref32, alpha)) == 0, f"f32t {B}x{M}x{N}x{K}"


def test_bmm_shapes():
    import torch_int._CUDA as C
    # upstream minimum shapes (tests/test_bmm_shape.py:8,19), kernel test shapes
    # (tests/test_bmm.py:8,114), ragged, decode-like (M=1, src_len not a multiple of 16)
    shapes = [(1, 1, 4, 16), (1, 1, 16, 16), (1, 512, 32, 512), (1, 512, 12288, 512), (3, 70, 50, 96),
              (5, 33, 129, 128), (8, 1, 513, 128), (8, 1, 128, 513), (2, 130, 130, 528), (16, 128, 128, 128),
              (12, 1, 517, 128), (3, 4, 33, 64), (2, 16, 1030, 256), (2, 300, 132, 64), (3, 5, 20, 32)]
    for i, (B, M, N, K) in enumerate(shapes):
        _say(f"bmm B={B} M={M} N={N} K={K}")
        _bmm_case(C, B, M, N, K, seed=200 + i)


def test_bmm_split_k_over_a_long_inner_dimension():
    # upstream's benchmark/bench_bmm.py multiplies [batch, seq, 12288] operands: few output tiles, a long K.  The
    # library then cuts K into slices (all problems' slices in one raw-int32 launch + one reduction; a single problem
    # takes the linears' forms); same bits as the oracle for all three output kinds, ragged shapes included
    import ctypes
    import torch_int._CUDA as C
    lib = C._lib
    lib.ti_last_kernel.restype = ctypes.c_char_p
    for i, (B, M, N, K) in enumerate([(4, 256, 256, 12288), (16, 256, 256, 4096), (8, 512, 512, 2048), (3, 200, 260, 4096),
                                      (1, 512, 512, 12288), (1, 256, 256, 12288), (2, 100, 128, 6144), (5, 64, 384, 8192)]):
        _say(f"bmm, long K: B={B} M={M} N={N} K={K}")
        split = lib.ti_bmm_workspace_bytes(B, M, N, K) > 0
        assert split or i == 2, (B, M, N, K)      # (8 x 512 x 512 x 2048 fills the chip without)
        _bmm_case(C, B, M, N, K, seed=400 + i)
        assert lib.ti_last_kernel().decode().startswith(("splitk_", "fusedk_")) == split, (B, M, N, K, lib.ti_last_kernel())
    # attention-shaped products never split, and a call without the workspace still works
    assert lib.ti_bmm_workspace_bytes(160, 512, 512, 128) == 0 and lib.ti_bmm_workspace_bytes(160, 512, 128, 512) == 0
    g = torch.Generator().manual_seed(409)
    a, b = _s8(g, 4, 256, 4096), _s8(g, 4, 256, 4096)
    out = torch.empty((4, 256, 256), dtype=torch.int8, device=DEV)
    ad, bd = a.to(DEV), b.to(DEV)
    rc = lib.ti_bmm_s8t_s8n_s8t(ad.data_ptr(), bd.data_ptr(), out.data_ptr(), 4, 256, 256, 4096, 0.002,
                                torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and not lib.ti_last_kernel().decode().startswith("splitk_")
    assert torch.equal(out, C.bmm_s8t_s8n_s8t(ad, bd, 0.002))
    assert lib.ti_last_kernel().decode().startswith("splitk_")


def test_large_problems_with_an_inner_dimension_that_16_does_not_divide():
    # the library's kernel for such shapes is one thread per output; from 2^26 products the host functions pad K
    # with zeros and the tiled kernels run (same results: the added products are zero)
    import ctypes
    import torch_int._CUDA as C
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    for i, (B, M, N, K) in enumerate([(8, 256, 128, 1500), (3, 200, 260, 1001)]):
        _say(f"bmm, odd K: B={B} M={M} N={N} K={K}")
        _bmm_case(C, B, M, N, K, seed=300 + i, prob_lhs=i == 0)
        assert C._lib.ti_last_kernel().decode() != "scalar"
    for variant in ("b8_o8", "bfp32_ofp32", "b32_o32", "relu_b8_o8"):
        _say(f"linear, odd K: {variant}")
        _linear_case(C, variant, 512, 640, 1001, seed=310)
        assert C._lib.ti_last_kernel().decode() != "scalar"
    # the zero-padded copy of a weight is made once per weight tensor and version: a second call reuses it, a weight
    # changed in place gets a new one
    g = torch.Generator().manual_seed(312)
    x, w, b = _s8(g, 512, 1001), _s8(g, 640, 1001), _s8(g, 640)
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    for _ in range(2):
        assert torch.equal(C.linear_a8_w8_b8_o8(xd, wd, bd, 0.001, 0.01).cpu(), orc.linear_a8_w8_b8_o8(x, w, b, 0.001, 0.01))
    assert id(wd) in C._padded
    w2 = _s8(g, 640, 1001)
    wd.copy_(w2)
    assert torch.equal(C.linear_a8_w8_b8_o8(xd, wd, bd, 0.001, 0.01).cpu(), orc.linear_a8_w8_b8_o8(x, w2, b, 0.001, 0.01))
    key = id(wd)
    del wd
    assert key not in C._padded
    _linear_case(C, "b8_o8", 70, 50, 37, seed=311)   # small: the one-thread-per-output kernel as it is
    assert C._lib.ti_last_kernel().decode() == "scalar"


def test_bmm_literal_fixture_from_upstream_tests():
    import torch_int._CUDA as C
    with open(os.path.join(GOLDEN, "bmm_literal_16x16.json")) as f:
        fx = json.load(f)
    a = torch.tensor(fx["a"], dtype=torch.int8)[None].to(DEV)
    b_nk = torch.tensor(fx["b_kn"], dtype=torch.int8).t().contiguous()[None].to(DEV)
    assert C.bmm_s8t_s8n_s32t(a, b_nk)[0].cpu().tolist() == fx["acc"]
    assert C.bmm_s8t_s8n_s8t(a, b_nk, fx["scale"])[0].cpu().tolist() == fx["expected_s8"]


@pytest.mark.parametrize("S", [128, 512])
def test_bmm_attention_config(S):
    # the attention-product benchmark configuration at a reduced batch*heads (the full 160 is covered by properties below)
    import torch_int._CUDA as C
    BH, d = 8, 128
    _say(f"attention bmm S={S}")
    _bmm_case(C, BH, S, S, d, seed=31)                  # Q.K^T
    _bmm_case(C, BH, S, d, S, seed=32, prob_lhs=True)   # P.V^T^T


def test_bmm_long_prefill_pv_tile():
    # P.V of a long prefill (N = 128, many row tiles): the 256x128 three-stage kernel, ragged M included
    import ctypes
    import torch_int._CUDA as C
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    for (B, M, K) in [(64, 2048, 256), (70, 1900, 384), (260, 520, 128)]:
        _say(f"long P.V B={B} M={M} N=128 K={K}")
        _bmm_case(C, B, M, 128, K, seed=77, prob_lhs=True)
        assert C._lib.ti_last_kernel().decode() == "pipe16_256x128", (B, M, K)


def test_bmm_full_size_properties():
    # B*H = 160, S = 512, d = 128 (the attention-product benchmark configuration): size-independent checks
    import torch_int._CUDA as C
    g = torch.Generator().manual_seed(9)
    BH, S, d = 160, 512, 128
    q, k = _s8(g, BH, S, d).to(DEV), _s8(g, BH, S, d).to(DEV)
    _say("bmm full-size properties")
    s32 = C.bmm_s8t_s8n_s32t(q, k)
    # (Q K^T)^T = K Q^T
    assert torch.equal(s32.transpose(1, 2), C.bmm_s8t_s8n_s32t(k, q))
    # a checksum of checksums: sum over n of acc[b,m,n] = q[b,m,:] . sum_n k[b,n,:]
    ksum = k.long().sum(1)  # every value below stays far under 2^53, so fp64 is exact
    assert torch.equal(s32.long().sum(2), torch.einsum("bmk,bk->bm", q.double(), ksum.double()).long())
    # batches are independent: the first 3 batches alone give the same slices
    assert torch.equal(C.bmm_s8t_s8n_s32t(q[:3].contiguous(), k[:3].contiguous()), s32[:3])
    # the fp32 and int8 epilogues are pure functions of the accumulator
    alpha = 0.00123
    f = C.bmm_s8t_s8n_f32t(q, k, alpha)
    assert torch.equal(f, s32.float() * alpha)
    o8 = C.bmm_s8t_s8n_s8t(q, k, alpha)
    assert torch.equal(o8, (s32.float() * alpha).clamp(-128, 127).round().to(torch.int8))
    # three full batches against the oracle
    ref = orc.bmm_s8t_s8n_s32t(q[157:].cpu(), k[157:].cpu())
    assert torch.equal(s32[157:].cpu(), ref)
    # P.V at the same size (probabilities [160, 512, 512] x V^T [160, 128, 512]): four tiles per head and more tiles
    # than resident workgroups, so the tiles of a head are dealt to one XCD; every head against an fp64 product on
    # the device (exact: the sums stay far below 2^53), four heads against the oracle
    import ctypes
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    _say("P.V full size")
    prob = torch.randint(0, 128, (BH, S, S), dtype=torch.int8, generator=g).to(DEV)
    vt = _s8(g, BH, d, S).to(DEV)
    pv = C.bmm_s8t_s8n_s8t(prob, vt, 0.0041)
    assert C._lib.ti_last_kernel().decode() == "pipe_128x128"
    exact = torch.einsum("bmk,bnk->bmn", prob.double(), vt.double())
    want = (exact.float() * 0.0041).clamp(-128, 127).round().to(torch.int8)
    assert torch.equal(pv, want)
    heads = [0, 53, 107, 159]
    assert torch.equal(pv[heads].cpu(), orc.bmm_s8t_s8n_s8t(prob[heads].cpu(), vt[heads].cpu(), 0.0041))
    assert torch.equal(C.bmm_s8t_s8n_s32t(prob, vt), exact.to(torch.int32))


# ------------------------------------------------------------------ dq_add_layernorm_q

def _ln_case(C, shape, seed, spread=20.0):
    g = torch.Generator().manual_seed(seed)
    H = shape[-1]
    inp = torch.randint(-65536, 65536, shape, dtype=torch.int32, generator=g)
    res = torch.randn(shape, generator=g)
    gamma = (1 + 0.02 * torch.randn(H, generator=g)) * spread
    beta = 0.02 * torch.randn(H, generator=g) * spread
    s = _scal(g, 1e-4, 1e-2)
    r_ref, q_ref = orc.dq_add_layernorm_q(inp, s, res, gamma, beta, 1e-5)
    r, q = C.dq_add_layernorm_q(inp.to(DEV), s, res.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5)
    assert r.dtype == torch.float32 and q.dtype == torch.int8 and r.shape == shape and q.shape == shape
    assert _ulp_diff(r.cpu(), r_ref) == 0, f"r {shape}"
    nbad = (q.cpu() != q_ref).sum().item()
    assert nbad == 0, f"q {shape}: {nbad} mismatches"
    # and the upstream composition of torch ops, on the GPU, within +-1 LSB
    from torch_int.functional.fused import dq_add_layernorm_q_py
    r_t, q_t = dq_add_layernorm_q_py(inp.to(DEV), s, res.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5)
    assert _ulp_diff(r, r_t) <= 1
    assert (q.int() - q_t.int()).abs().max().item() <= 1
    assert (q != q_t).float().mean().item() <= 0.01 + 1.0 / q.numel()


def test_ln_q_shapes():
    import torch_int._CUDA as C
    # upstream test shape (tests/test_dq_add_ln_q.py:8), OPT widths, odd H, H beyond the register path
    for i, shape in enumerate([(2, 3, 4), (7, 768), (4, 5, 5120), (3, 9216), (2, 12288), (5, 1023), (3, 1),
                               (2, 16384), (2, 20000), (1, 17)]):
        _say(f"ln_q shape={shape}")
        _ln_case(C, shape, seed=300 + i)


def test_ln_q_full_size_and_in_place():
    import torch_int._CUDA as C
    _say("ln_q C4 [4,512,5120]")
    _ln_case(C, (4, 512, 5120), seed=0)
    # r_out may alias the residual (C ABI contract): call the library directly
    g = torch.Generator().manual_seed(1)
    inp = torch.randint(-65536, 65536, (64, 5120), dtype=torch.int32, generator=g)
    res = torch.randn(64, 5120, generator=g)
    gamma, beta = torch.ones(5120) * 30, torch.zeros(5120)
    r_ref, q_ref = orc.dq_add_layernorm_q(inp, 0.003, res, gamma, beta, 1e-5)
    d_in, d_res, d_g, d_b = inp.to(DEV), res.to(DEV), gamma.to(DEV), beta.to(DEV)
    q = torch.empty((64, 5120), dtype=torch.int8, device=DEV)
    rc = C._lib.ti_dq_add_layernorm_q(d_in.data_ptr(), 0.003, d_res.data_ptr(), d_g.data_ptr(), d_b.data_ptr(),
                                      1e-5, d_res.data_ptr(), q.data_ptr(), 64, 5120,
                                      torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert torch.equal(d_res.cpu(), r_ref) and torch.equal(q.cpu(), q_ref)


# ------------------------------------------------------------------ fused chains of the OPT blocks

def test_fused_add_layernorm_q():
    import torch_int._hip_ext as X
    for i, shape in enumerate([(7, 768), (4, 6, 5120), (3, 9216), (5, 1023), (2, 20000), (3, 1)]):
        _say(f"add_layernorm_q shape={shape}")
        g = torch.Generator().manual_seed(400 + i)
        H = shape[-1]
        x, res = torch.randn(shape, generator=g), torch.randn(shape, generator=g) * 3
        gamma = (1 + 0.02 * torch.randn(H, generator=g)) * 25
        beta = 0.5 * torch.randn(H, generator=g)
        r_ref, q_ref = orc.add_layernorm_q(x, res, gamma, beta, 1e-5)
        d_res = res.to(DEV)
        q = X.add_layernorm_q(x.to(DEV), d_res, gamma.to(DEV), beta.to(DEV), 1e-5)
        assert torch.equal(d_res.cpu(), r_ref) and torch.equal(r_ref, res + x)  # residual updated in place
        assert (q.cpu() != q_ref).sum().item() == 0
        _, q_ref2 = orc.add_layernorm_q(None, res, gamma, beta, 1e-5)
        d_res = res.to(DEV)
        q2 = X.add_layernorm_q(None, d_res, gamma.to(DEV), beta.to(DEV), 1e-5)
        assert torch.equal(d_res.cpu(), res) and (q2.cpu() != q_ref2).sum().item() == 0
        # upstream chain (nn/fused.py:13-18) on the GPU: one LSB, rarely
        y = torch.nn.functional.layer_norm(res.to(DEV), (H,), gamma.to(DEV), beta.to(DEV), 1e-5)
        q_t = y.round().clamp(-128, 127).to(torch.int8)
        assert (q2.int() - q_t.int()).abs().max().item() <= 1
        assert (q2 != q_t).float().mean().item() <= 0.01 + 1.0 / q2.numel()


def test_fused_attn_softmax_q():
    import torch_int._hip_ext as X
    neg = torch.finfo(torch.float32).min
    for i, (B, H, T, S) in enumerate([(2, 4, 16, 16), (1, 3, 5, 513), (2, 2, 33, 100), (1, 2, 1, 2049),
                                      (1, 1, 4, 4100), (4, 40, 64, 512)]):
        _say(f"attn_softmax_q B={B} H={H} T={T} S={S}")
        g = torch.Generator().manual_seed(500 + i)
        scores = torch.randn(B * H, T, S, generator=g) * 6
        mask = torch.zeros(B, 1, T, S)
        mask.masked_fill_(torch.arange(S)[None, :] > torch.arange(S - T, S)[:, None], neg)  # causal
        mask[0, 0, :, : S // 7] = neg                                                       # padding
        for m in (mask, None):
            ref = orc.attn_softmax_q(scores, m, H)
            out = X.attn_softmax_q(scores.to(DEV), m.to(DEV) if m is not None else None, H)
            assert out.dtype == torch.int8 and out.shape == scores.shape
            assert (out.cpu() != ref).sum().item() == 0
            # upstream chain (models/opt.py:144-178) on the GPU
            s = scores.to(DEV).view(B, H, T, S)
            if m is not None:
                s = torch.clamp_min(s + m.to(DEV), neg)
            q_t = (torch.softmax(s.view(B * H, T, S), -1) * 127).round().to(torch.int8)
            assert (out.int() - q_t.int()).abs().max().item() <= 1
            assert (out != q_t).float().mean().item() <= 1e-3 + 1.0 / out.numel()
            assert int(out.min()) >= 0


def test_int8_layout_kernels():
    import torch_int._hip_ext as X
    g = torch.Generator().manual_seed(9)
    for (B, T, H, d) in [(4, 512, 40, 128), (2, 37, 4, 64), (1, 1, 3, 24), (3, 5, 7, 20)]:
        _say(f"split/merge heads B={B} T={T} H={H} d={d}")
        t = _s8(g, B, T, H * d).to(DEV)
        ref = t.view(B, T, H, d).transpose(1, 2).contiguous()
        out = X.split_heads(t, B, T, H, d)
        assert out.is_contiguous() and torch.equal(out, ref)
        back = X.merge_heads(out.view(B * H, T, d), B, H, T, d)
        assert back.shape == (B, T, H * d) and torch.equal(back, t)
    # R % 4 == 0 and C % 16 == 0 take the 4 x 4-block kernels: 128 x 128 tiles (the first two), 64 x 64 tiles with
    # and without cut-off edge tiles (the next five and the sliced source below); the rest the byte-by-byte kernel
    for (B, R, C) in [(160, 512, 128), (2, 128, 384), (3, 64, 64), (2, 192, 320), (4, 520, 128), (2, 68, 48), (3, 36, 16), (8, 513, 128), (3, 70, 50), (2, 1, 128), (5, 64, 1),
                      (1, 200, 333)]:
        _say(f"transpose_last2 B={B} R={R} C={C}")
        t = _s8(g, B, R, C).to(DEV)
        out = X.transpose_last2(t)
        assert out.is_contiguous() and torch.equal(out, t.transpose(1, 2).contiguous())
    big = _s8(g, 5, 128, 64).to(DEV)
    part = big[1:]   # contiguous, starts 8192 bytes into the allocation
    assert torch.equal(X.transpose_last2(part), part.transpose(1, 2).contiguous())


def test_stream_kernel_strip_orders_and_ragged_widths():
    # the M <= 16 streaming kernel: grids that are and are not a multiple of 8 (two strip orders), several strips
    # per workgroup with a last partial run of 8, widths that are not a multiple of 16 or of 4 (the prefetched
    # bias and old-output loads are clamped there), every row count class (1, <= 4, <= 16), all output kinds
    import ctypes
    import torch_int._CUDA as C
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator().manual_seed(91)
    for (M, N, K) in [(1, 4100, 1024), (2, 4102, 2048), (16, 4099, 1024), (1, 20500, 1024), (4, 16400, 1024),
                      (13, 8200, 2048), (16, 20480, 1024)]:
        for variant in ("b8_o8", "relu_b8_o8", "bfp32_ofp32", "b32_o32"):
            _say(f"stream {variant} M={M} N={N} K={K}")
            _linear_case(C, variant, M, N, K, seed=91)
            assert C._lib.ti_last_kernel().decode() == ("gemv" if M == 1 else "stream"), (M, N, K, C._lib.ti_last_kernel())
        _say(f"stream += M={M} N={N} K={K}")
        x, w = _s8(g, M, K), _s8(g, N, K)
        bias, resid = torch.randn(N, generator=g), torch.randn(M, N, generator=g) * 3
        ref = orc.linear_a8_w8_bfp32_ofp32_acc(x, w, bias, 0.003, 1.0, resid)
        out = C._linear_a8_w8_bfp32_ofp32_acc(x.to(DEV), w.to(DEV), bias.to(DEV), 0.003, 1.0, resid.to(DEV))
        assert _ulp_diff(out.cpu(), ref) == 0, (M, N, K)
        assert C._lib.ti_last_kernel().decode() == ("gemv" if M == 1 else "stream")


def test_stream_kernel_on_the_view_with_rows_cut_into_parts():
    # one or two rows of activations against few, long weight rows (fc2 of a decode step): the streaming kernel
    # multiplies the view with every row cut into four (two) parts and its epilogue adds the parts of each output.
    # One row otherwise runs on the flat-reading dot-product kernel.  Every output kind, widths with a last partial
    # run of strips or of rows, the shapes next to the rules' limits.
    import ctypes
    import torch_int._CUDA as C
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator().manual_seed(92)
    for (M, N, K, kern) in [(1, 4096, 28672, "stream_parts"), (1, 9216, 36864, "stream_parts"), (1, 4096, 53248, "stream_parts"),
                            (2, 5120, 20480, "stream_parts"), (2, 4112, 10240, "stream_parts"), (2, 16384, 10240, "stream_parts"),
                            (1, 5120, 20480, "gemv"), (1, 4096, 8192, "gemv"), (1, 9232, 12288, "gemv"), (1, 4099, 1024, "gemv"),
                            (1, 4096, 32768, "gemv"), (1, 4097, 49152, "gemv"), (1, 20481, 2048, "gemv"),
                            (1, 4104, 53248, "stream"), (2, 5120, 7168, "stream"), (3, 5120, 20480, "stream"),
                            (2, 4096, 8192, "stream")]:
        for variant in VARIANTS:
            _say(f"stream view {variant} M={M} N={N} K={K}")
            _linear_case(C, variant, M, N, K, seed=92)
            assert C._lib.ti_last_kernel().decode() == kern, (M, N, K, C._lib.ti_last_kernel())
        _say(f"stream view += M={M} N={N} K={K}")
        x, w = _s8(g, M, K), _s8(g, N, K)
        bias, resid = torch.randn(N, generator=g), torch.randn(M, N, generator=g) * 3
        ref = orc.linear_a8_w8_bfp32_ofp32_acc(x, w, bias, 0.003, 1.0, resid)
        out = C._linear_a8_w8_bfp32_ofp32_acc(x.to(DEV), w.to(DEV), bias.to(DEV), 0.003, 1.0, resid.to(DEV))
        assert _ulp_diff(out.cpu(), ref) == 0, (M, N, K)
        assert C._lib.ti_last_kernel().decode() == kern


def test_one_launch_split_k_is_exact_for_every_output_kind():
    # 2 to 4 K slices on a tile of the 16x16-block kernel that divides M: the slices of a tile meet in one XCD's L2 and
    # the wave that arrives last applies the epilogue.  Every tile shape, every epilogue, sampled rows against the
    # oracle and all rows against the two-launch form; called three times in a row (the arrival counters must be back
    # at zero after each call) and on a second stream (which gets counters of its own).
    import ctypes
    import torch_int._CUDA as C
    import torch_int._hip_ext as X
    lib = C._lib
    lib.ti_last_kernel.restype = ctypes.c_char_p
    assert lib.ti_fused_splitk(1) in (0, 1)
    try:
        g = torch.Generator().manual_seed(97)
        side = torch.cuda.Stream()
        for (M, N, K, tile) in [(256, 640, 2048, "128x80"), (256, 2880, 3584, "128x80"), (256, 3200, 7168, "128x160"),
                                (896, 1600, 6144, "128x160"), (128, 4608, 2048, "128x288"), (128, 9216, 2048, "128x288"),
                                (256, 3072, 3584, "128x192"), (128, 12288, 1536, "128x192"),
                                (768, 3840, 9216, "256x160"), (1024, 9216, 2560, "256x288")]:
            x, w = _s8(g, M, K), _s8(g, N, K)
            b8, bf = _s8(g, N), torch.randn(N, generator=g)
            b32 = torch.randint(-65535, 65535, (N,), dtype=torch.int32, generator=g)
            resid = torch.randn(M, N, generator=g) * 3
            alpha, beta = _scal(g, 1e-4, 1e-2), _scal(g, 1e-4, 1e-2)
            xd, wd, b8d, bfd, b32d = x.to(DEV), w.to(DEV), b8.to(DEV), bf.to(DEV), b32.to(DEV)
            rows = torch.arange(M) if M <= 256 else torch.cat([torch.arange(0, 64), torch.arange(M // 2 - 32, M // 2 + 32),
                                                                torch.arange(M - 64, M)])
            acc = orc.gemm_acc(x[rows].contiguous(), w)
            heads_d = 128 if N % 128 == 0 else 64 if N % 64 == 0 else 32
            runs = [
                ("b32_o32", lambda: C.linear_a8_w8_b32_o32(xd, wd, b32d), lambda: orc.epi_b32_o32(acc, b32)),
                ("b32_o32_scaled", lambda: C.linear_a8_w8_b32_o32_with_scaling(xd, wd, b32d, alpha, beta),
                 lambda: orc.epi_b32_o32_scaled(acc, b32, alpha, beta)),
                ("bfp32_ofp32", lambda: C.linear_a8_w8_bfp32_ofp32(xd, wd, bfd, alpha, 1.0),
                 lambda: orc.epi_bfp32_ofp32(acc, bf, alpha, 1.0)),
                ("b8_o8", lambda: C.linear_a8_w8_b8_o8(xd, wd, b8d, alpha, beta), lambda: orc.epi_b8_o8(acc, b8, alpha, beta)),
                ("relu_b8_o8", lambda: C.linear_relu_a8_w8_b8_o8(xd, wd, b8d, alpha, beta),
                 lambda: orc.epi_b8_o8(acc, b8, alpha, beta, relu=True)),
                ("bfp32_ofp32 +=", lambda: C._linear_a8_w8_bfp32_ofp32_acc(xd, wd, bfd, alpha, 1.0, resid.to(DEV)),
                 lambda: resid[rows] + orc.epi_bfp32_ofp32(acc, bf, alpha, 1.0)),
                ("b8_o8 head-major",
                 lambda: X.linear_a8_w8_b8_o8_heads(xd, wd, b8d, alpha, beta, 1, M, N // heads_d, heads_d)
                 .permute(0, 2, 1, 3).reshape(M, N), lambda: orc.epi_b8_o8(acc, b8, alpha, beta)),
            ]
            for name, gpu, ref in runs:
                _say(f"one-launch split-K {name} M={M} N={N} K={K}")
                outs = [gpu() for _ in range(3)]
                # the accumulating epilogue stays with the two-launch form (its reads of the old outputs are cheaper
                # when the whole chip does them in the reduction kernel)
                form = "splitk_" if name.endswith("+=") else "fusedk_"
                assert lib.ti_last_kernel().decode() == form + tile, (M, N, K, lib.ti_last_kernel())
                with torch.cuda.stream(side):
                    side.wait_stream(torch.cuda.current_stream())
                    outs.append(gpu())
                torch.cuda.current_stream().wait_stream(side)
                lib.ti_fused_splitk(0)
                two = gpu()
                assert lib.ti_last_kernel().decode() == "splitk_" + tile, lib.ti_last_kernel()
                lib.ti_fused_splitk(1)
                want = ref()
                for o in outs:
                    assert torch.equal(o, two), (name, M, N, K)
                if name == "bfp32_ofp32 +=":   # one rounding of the sum on the device, as the oracle's fused form does
                    want = orc.linear_a8_w8_bfp32_ofp32_acc(x[rows].contiguous(), w, bf, alpha, 1.0, resid[rows].contiguous())
                assert torch.equal(two[rows.to(DEV)].cpu(), want), (name, M, N, K)
        # a ragged M, or more than four slices, stays with the two-launch form
        for (M, N, K) in [(200, 640, 4096), (128, 640, 4096)]:
            _linear_case(C, "b8_o8", M, N, K, seed=98)
            assert lib.ti_last_kernel().decode().startswith("splitk_"), (M, N, K, lib.ti_last_kernel())
    finally:
        lib.ti_fused_splitk(1)


def test_one_launch_split_k_on_concurrent_streams():
    # three streams issue split-K linears of different shapes without waiting for one another: each stream has its own
    # workspace and its own arrival counters, so every output must equal the two-launch result
    import ctypes
    import torch_int._CUDA as C
    lib = C._lib
    lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator().manual_seed(101)
    cases = []
    for (M, N, K) in [(256, 2880, 3584), (256, 640, 2048), (128, 4608, 2048), (256, 3200, 7168)]:
        x, w, b = _s8(g, M, K).to(DEV), _s8(g, N, K).to(DEV), _s8(g, N).to(DEV)
        before = lib.ti_fused_splitk(0)
        try:
            ref = C.linear_a8_w8_b8_o8(x, w, b, 0.001, 0.01)
        finally:
            lib.ti_fused_splitk(before)
        cases.append((x, w, b, ref))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(3)]
    outs = []
    for it in range(24):
        for si, st in enumerate(streams):
            x, w, b, ref = cases[(it + 2 * si) % len(cases)]
            with torch.cuda.stream(st):
                outs.append((C.linear_a8_w8_b8_o8(x, w, b, 0.001, 0.01), ref, lib.ti_last_kernel().decode()))
    torch.cuda.synchronize()
    assert all(k.startswith("fusedk_") for _, _, k in outs), sorted(set(k for _, _, k in outs))
    assert all(torch.equal(o, r) for o, r, _ in outs)


def test_one_launch_split_k_in_a_graph():
    # a split-K linear captured into a HIP graph (after a warm-up on the capture stream: the first use on a device
    # probes and is not capturable) and replayed with eager split-K launches between the replays
    import ctypes
    import torch_int._CUDA as C
    lib = C._lib
    lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator().manual_seed(99)
    M, N, K = 256, 2880, 3584
    w, b = _s8(g, N, K).to(DEV), _s8(g, N).to(DEV)
    xs = [_s8(g, M, K) for _ in range(3)]
    refs = [orc.linear_a8_w8_b8_o8(x, w.cpu(), b.cpu(), 0.0011, 0.02) for x in xs]
    static_x = xs[0].to(DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            C.linear_a8_w8_b8_o8(static_x, w, b, 0.0011, 0.02)
    side.synchronize()
    assert lib.ti_last_kernel().decode() == "fusedk_128x80", lib.ti_last_kernel()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        static_out = C.linear_a8_w8_b8_o8(static_x, w, b, 0.0011, 0.02)
    for i in (1, 2, 0, 1):
        _say("one-launch split-K graph replay", i)
        eager = C.linear_a8_w8_b8_o8(xs[i].to(DEV), w, b, 0.0011, 0.02)   # eager launch on the current stream
        torch.cuda.synchronize()
        static_x.copy_(xs[i])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_out.cpu(), refs[i]) and torch.equal(eager.cpu(), refs[i]), i


def test_one_launch_split_k_needs_a_256_byte_aligned_workspace():
    # through the C ABI: the waves park and read back 1 KiB regions of the workspace, which must not share a 128-byte
    # line with a neighbour's; a workspace that is only 16-byte aligned takes the two-launch form, same bytes
    import ctypes
    import torch_int._CUDA as C
    lib = C._lib
    lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator().manual_seed(103)
    M, N, K = 256, 2880, 3584
    x, w, b = _s8(g, M, K).to(DEV), _s8(g, N, K).to(DEV), _s8(g, N).to(DEV)
    need = lib.ti_linear_workspace_bytes(M, N, K)
    assert need > 0
    ws = torch.empty(need + 512, dtype=torch.uint8, device=DEV)
    base = (ws.data_ptr() + 255) // 256 * 256
    outs, kernels = [], []
    for off in (0, 16, 128, 256):
        _say(f"one-launch split-K, workspace offset {off}")
        out = torch.empty((M, N), dtype=torch.int8, device=DEV)
        rc = lib.ti_linear_a8_w8_b8_o8(x.data_ptr(), w.data_ptr(), b.data_ptr(), out.data_ptr(), M, N, K, 0.0013, 0.02,
                                       base + off, need, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.ti_last_error()
        kernels.append(lib.ti_last_kernel().decode())
        outs.append(out.cpu())
    assert kernels[0].startswith("fusedk_") and kernels[3].startswith("fusedk_"), kernels
    assert kernels[1].startswith("splitk_") and kernels[2].startswith("splitk_"), kernels
    ref = orc.linear_a8_w8_b8_o8(x.cpu(), w.cpu(), b.cpu(), 0.0013, 0.02)
    for o in outs:
        assert torch.equal(o, ref)
    assert lib.ti_fused_splitk_faulted() == 0


def test_one_launch_split_k_hands_counter_sets_on_to_new_streams():
    # more streams than the eight sets of arrival counters a device has: a stream that has gone idle hands its set
    # on, so every one of twelve streams used one after the other still gets the one-launch form, with exact results
    import ctypes
    import torch_int._CUDA as C
    lib = C._lib
    lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator().manual_seed(105)
    M, N, K = 256, 640, 2048
    x, w, b = _s8(g, M, K).to(DEV), _s8(g, N, K).to(DEV), _s8(g, N).to(DEV)
    ref = orc.linear_a8_w8_b8_o8(x.cpu(), w.cpu(), b.cpu(), 0.001, 0.01)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(12)]
    for i, st in enumerate(streams):
        _say("one-launch split-K on stream", i)
        with torch.cuda.stream(st):
            out = C.linear_a8_w8_b8_o8(x, w, b, 0.001, 0.01)
            out2 = C.linear_a8_w8_b8_o8(x, w, b, 0.001, 0.01)
        kern = lib.ti_last_kernel().decode()
        st.synchronize()
        assert kern.startswith("fusedk_"), (i, kern)
        assert torch.equal(out.cpu(), ref) and torch.equal(out2.cpu(), ref), i
    assert lib.ti_fused_splitk_faulted() == 0


def test_linear_accumulate_into_output(two_launch_split_k):
    # inout += alpha*acc + bias in the GEMM epilogue, through every kernel family the fp32 linear can take
    import ctypes
    import torch_int._CUDA as C
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator().manual_seed(63)
    seen = set()
    for (M, N, K) in [(2048, 5120, 256), (2048, 5120, 64), (2000, 9216, 192), (2000, 9216, 128), (4096, 2816, 128),
                      (2048, 4096, 2048),   # 256x128 tiles
                      (4096, 2816, 1024), (1024, 2048, 64), (1024, 5120, 5120), (1024, 4608, 3584), (256, 3072, 7744),
                      (1024, 9216, 9216), (384, 2880, 4608), (4, 4608, 16384), (256, 3200, 11648), (256, 1600, 11648), (384, 2560, 1024),
                      (128, 640, 4096), (128, 768, 4096), (128, 1024, 4096), (512, 12288, 2048), (1024, 12288, 1024), (16, 5120, 3072), (3, 100, 272), (300, 200, 48), (2100, 5000, 272),
                      (70, 50, 37), (4, 64, 0)]:
        _say(f"linear += M={M} N={N} K={K}")
        x, w = _s8(g, M, K), _s8(g, N, K)
        bias, resid = torch.randn(N, generator=g), torch.randn(M, N, generator=g) * 3
        alpha = _scal(g, 1e-4, 1e-2)
        ref = orc.linear_a8_w8_bfp32_ofp32_acc(x, w, bias, alpha, 1.0, resid)
        inout = resid.to(DEV)
        out = C._linear_a8_w8_bfp32_ofp32_acc(x.to(DEV), w.to(DEV), bias.to(DEV), alpha, 1.0, inout)
        assert out.data_ptr() == inout.data_ptr()
        assert _ulp_diff(out.cpu(), ref) == 0, (M, N, K)
        seen.add(C._lib.ti_last_kernel().decode())
    assert {"pipe16_256x160", "pipe16_256x288", "pipe16_256x128", "pipe16_128x80", "pipe16_128x192", "pipe16_256x192", "pipe_256x256", "pipe_128x128", "splitk_256x256", "splitk_256x160",
            "splitk_256x288", "splitk_128x160", "splitk_128x288", "splitk_128x80", "splitk_128x192", "splitk_128x128", "stream", "skinny", "tile_64x64", "tile_256x256", "scalar"} <= seen, seen
    # the module route: W8A8BFP32OFP32Linear(x, add_to=residual)
    from torch_int.nn.linear import W8A8BFP32OFP32Linear
    m = W8A8BFP32OFP32Linear(256, 320, alpha=0.003)
    m.bias = torch.randn(1, 320, generator=g)
    x = _s8(g, 2, 5, 256)
    resid = torch.randn(2, 5, 320, generator=g)
    ref = orc.linear_a8_w8_bfp32_ofp32_acc(x.view(-1, 256), m.weight, m.bias, 0.003, 1.0, resid)
    m = m.to(DEV)
    r = resid.to(DEV)
    assert m(x.to(DEV), add_to=r) is r and _ulp_diff(r.cpu(), ref) == 0


def test_bmm_rowmajor_rhs_for_decode():
    # P.V on V as the KV cache stores it: [B, M, K] x [B, K, N], any K and N
    import torch_int._hip_ext as X
    g = torch.Generator().manual_seed(41)
    shapes = [(288, 1, 128, 517), (16, 1, 128, 2500), (8, 4, 128, 33), (3, 16, 100, 50), (2, 37, 64, 300),
              (2, 2, 130, 70), (3, 1, 7, 5), (2, 3, 16, 0), (1, 16, 256, 1024)]
    for (B, M, N, K) in shapes:
        _say(f"bmm_s8t_s8t_s8t B={B} M={M} N={N} K={K}")
        a = _s8(g, B, M, K, lo=0)
        b = _s8(g, B, K, N)
        alpha = _scal(g, 2e-4, 4e-3)
        out = X.bmm_s8t_s8t_s8t(a.to(DEV), b.to(DEV), alpha).cpu()
        assert torch.equal(out, orc.bmm_s8t_s8t_s8t(a, b, alpha)), (B, M, N, K)
    # operands that live in a buffer with spare rows after every batch (a KV cache with room to grow)
    for (B, M, S, d, cap) in [(288, 1, 517, 128, 656), (6, 4, 33, 64, 48), (3, 16, 100, 32, 101)]:
        _say(f"batch-strided products B={B} M={M} S={S} d={d} cap={cap}")
        p_, q_ = _s8(g, B, M, S, lo=0), _s8(g, B, M, d)
        kbuf, vbuf = _s8(g, B, cap, d), _s8(g, B, cap, d)
        kd, vd = kbuf.to(DEV)[:, :S], vbuf.to(DEV)[:, :S]
        assert not kd.is_contiguous() or B == 1
        out = X.bmm_s8t_s8t_s8t(p_.to(DEV), vd, 0.002).cpu()
        assert torch.equal(out, orc.bmm_s8t_s8t_s8t(p_, vbuf[:, :S].contiguous(), 0.002))
        sc = X.bmm_s8t_s8n_f32t_strided(q_.to(DEV), kd, 0.003).cpu()
        assert _ulp_diff(sc, orc.bmm_s8t_s8n_f32t(q_, kbuf[:, :S].contiguous(), 0.003)) == 0
    # an operand pair whose rows are not dword aligned takes the byte path
    a, b = _s8(g, 2, 3, 40), _s8(g, 2, 41, 24)
    bd = b.to(DEV)[:, 1:, :].contiguous()
    odd = torch.empty(2 * 40 * 24 + 1, dtype=torch.int8, device=DEV)[1:].view(2, 40, 24)
    odd.copy_(bd)
    assert odd.data_ptr() % 4 != 0
    out = X.bmm_s8t_s8t_s8t(a.to(DEV), odd, 0.001).cpu()
    assert torch.equal(out, orc.bmm_s8t_s8t_s8t(a, b[:, 1:, :].contiguous(), 0.001))


def test_head_major_projection_through_every_kernel_family(two_launch_split_k):
    # the s8 linear whose stores write [bsz, heads, seq, d]: same values as the plain linear, permuted
    import ctypes
    import torch_int._CUDA as C
    import torch_int._hip_ext as X
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator().manual_seed(71)
    seen = set()
    # (bsz, seq, heads, d, K)
    for (B, T, H, d, K) in [(4, 512, 40, 128, 256), (4, 512, 40, 128, 192), (2, 1000, 72, 128, 192), (2, 1000, 72, 128, 256),
                            (8, 512, 22, 128, 128), (8, 512, 22, 128, 192), (2, 512, 16, 128, 64),
                            (2, 512, 40, 128, 5120), (2, 512, 36, 128, 3584), (2, 512, 72, 128, 9216), (1, 384, 90, 32, 4608),
                            (1, 256, 24, 128, 7744), (2, 64, 5, 128, 4096), (1, 256, 25, 128, 11648), (1, 256, 25, 64, 11648), (1, 384, 20, 128, 1024), (1, 128, 6, 128, 4096), (1, 128, 8, 128, 4096), (4, 128, 96, 128, 2048), (2, 512, 96, 128, 1024), (1, 16, 40, 128, 3072), (1, 3, 5, 32, 272),
                            (1, 1, 40, 128, 5120), (1, 1, 40, 128, 20480), (2, 1, 40, 128, 20480), (1, 4, 40, 128, 2048),  # decode rows
                            (3, 100, 5, 48, 48), (3, 700, 39, 128, 272), (2, 35, 3, 16, 37)]:
        M, N = B * T, H * d
        _say(f"head-major linear bsz={B} seq={T} heads={H} d={d} K={K}")
        x, w, b = _s8(g, M, K), _s8(g, N, K), _s8(g, N)
        alpha, beta = _scal(g, 1e-4, 1e-2), _scal(g, 1e-4, 1e-2)
        ref = orc.linear_a8_w8_b8_o8_heads(x, w, b, alpha, beta, B, T, H, d)
        out = X.linear_a8_w8_b8_o8_heads(x.to(DEV), w.to(DEV), b.to(DEV), alpha, beta, B, T, H, d)
        assert out.shape == (B, H, T, d) and out.is_contiguous()
        assert torch.equal(out.cpu(), ref), (B, T, H, d, K)
        seen.add(C._lib.ti_last_kernel().decode())
    assert {"pipe16_256x160", "pipe16_256x288", "pipe16_128x80", "pipe16_128x192", "pipe16_256x192", "pipe_256x256", "pipe_128x128", "splitk_256x256", "splitk_256x160",
            "splitk_256x288", "splitk_128x160", "splitk_128x288", "splitk_128x80", "splitk_128x192", "splitk_128x128", "stream", "gemv", "skinny", "tile_64x64", "tile_256x256", "scalar"} <= seen, seen
    with pytest.raises(RuntimeError):
        X.linear_a8_w8_b8_o8_heads(x.to(DEV), w.to(DEV), b.to(DEV), alpha, beta, 2, 35, 6, 8)   # d not a multiple of 16


def test_grouped_qkv_linear():
    import ctypes
    import torch_int._CUDA as C
    import torch_int._hip_ext as X
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator().manual_seed(29)
    for (M, N, K, n, family) in [(4, 5120, 5120, 3, "stream_group"), (1, 2048, 1024, 3, "gemv_group"),
                                 (1, 5120, 5120, 3, "gemv_group"), (1, 4098, 2048, 2, "gemv_group"),
                                 (16, 1536, 2048, 4, "stream_group"), (9, 4100, 3072, 2, "stream_group"),
                                 (4, 640, 1024, 3, None), (40, 512, 256, 3, None), (3, 100, 272, 1, None)]:
        _say(f"grouped linear M={M} N={N} K={K} n={n}")
        x = _s8(g, M, K)
        ws, bs = [_s8(g, N, K) for _ in range(n)], [_s8(g, N) for _ in range(n)]
        al, be = [_scal(g, 1e-4, 1e-2) for _ in range(n)], [_scal(g, 1e-4, 1e-2) for _ in range(n)]
        ref = orc.linear_a8_w8_b8_o8_group(x, ws, bs, al, be)
        out = X.linear_a8_w8_b8_o8_group(x.to(DEV), [w.to(DEV) for w in ws], [b.to(DEV) for b in bs], al, be)
        assert len(out) == n
        for o, r_ in zip(out, ref):
            assert torch.equal(o.cpu(), r_), (M, N, K)
        if family:
            assert C._lib.ti_last_kernel().decode() == family


def test_grouped_prefill_linears_one_launch():
    # q/k/v-style groups at prefill sizes: plain and head-major stores, the one-launch kernels and the loop
    import ctypes
    import torch_int._CUDA as C
    import torch_int._hip_ext as X
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator().manual_seed(31)
    # (bsz, seq, heads, d, K, problems, family)
    for (B, T, H, d, K, n, family) in [(4, 512, 40, 128, 256, 3, "pipe16_256x160_group"),
                                       (2, 1000, 72, 128, 128, 3, "pipe16_256x288_group"),
                                       (4, 512, 32, 128, 256, 3, "pipe16_256x128_group"),
                                       (1, 500, 32, 128, 384, 3, "pipe16_256x128_group"),
                                       (2, 100, 5, 128, 384, 2, "pipe16_256x160_group"),
                                       (1, 300, 9, 32, 640, 4, "pipe16_256x288_group"),
                                       (3, 171, 10, 16, 128, 3, "pipe16_256x160_group"),
                                       # 512 x 12288: each problem is one round of 128x192 tiles and runs by itself
                                       (1, 512, 96, 128, 2048, 3, None),
                                       (2, 100, 6, 128, 128, 3, None), (2, 60, 5, 128, 128, 3, None),
                                       (2, 100, 5, 128, 192, 3, None)]:
        M, N = B * T, H * d
        _say(f"grouped prefill linear M={M} N={N} K={K} n={n}")
        x = _s8(g, M, K)
        ws, bs = [_s8(g, N, K) for _ in range(n)], [_s8(g, N) for _ in range(n)]
        al, be = [_scal(g, 1e-4, 1e-2) for _ in range(n)], [_scal(g, 1e-4, 1e-2) for _ in range(n)]
        xd, wd, bd = x.to(DEV), [w.to(DEV) for w in ws], [b.to(DEV) for b in bs]
        ref = orc.linear_a8_w8_b8_o8_group(x, ws, bs, al, be)
        out = X.linear_a8_w8_b8_o8_group(xd, wd, bd, al, be)
        if family:
            assert C._lib.ti_last_kernel().decode() == family
        elif N == 12288:
            assert C._lib.ti_last_kernel().decode() == "pipe16_128x192"
        for o, r_ in zip(out, ref):
            assert torch.equal(o.cpu(), r_), (M, N, K)
        out = X.linear_a8_w8_b8_o8_group_heads(xd, wd, bd, al, be, B, T, H, d)
        if family:
            assert C._lib.ti_last_kernel().decode() == family
        assert X.linear_group_is_one_launch(M, N, K, n) == (family is not None)
        for o, r_ in zip(out, ref):
            assert o.shape == (B, H, T, d) and o.is_contiguous()
            assert torch.equal(o.cpu(), r_.view(B, T, H, d).transpose(1, 2)), (M, N, K)


def test_kv_append_kernel():
    import torch_int._hip_ext as X
    g = torch.Generator().manual_seed(17)
    for (B, H, cap, d, S, T) in [(4, 72, 656, 128, 544, 1), (2, 3, 40, 64, 7, 5), (1, 2, 9, 24, 8, 1), (2, 2, 16, 20, 0, 16)]:
        _say(f"kv_append B={B} H={H} cap={cap} d={d} S={S} T={T}")
        kbuf, vbuf = _s8(g, B, H, cap, d), _s8(g, B, H, cap, d)
        kn, vn = _s8(g, B, H, T, d), _s8(g, B, H, T, d)
        kd, vd = kbuf.to(DEV), vbuf.to(DEV)
        X.kv_append(kn.to(DEV), vn.to(DEV), kd, vd, S)
        kbuf[:, :, S:S + T] = kn
        vbuf[:, :, S:S + T] = vn
        assert torch.equal(kd.cpu(), kbuf) and torch.equal(vd.cpu(), vbuf)
    with pytest.raises(RuntimeError):
        X.kv_append(kn.to(DEV), vn.to(DEV), kd, vd, 1)   # 1 + 16 positions do not fit 16


def test_decode_attention_matches_the_separate_kernels_and_the_oracle():
    # one launch = append + Q.K^T + softmax-quant + P.V of a decode step, bit for bit
    import torch_int._hip_ext as X
    import torch_int._CUDA as C
    g = torch.Generator().manual_seed(29)
    neg = torch.finfo(torch.float32).min
    # (batch, heads, cap, d, filled, T, masked)
    cases = [(4, 72, 656, 128, 543, 1, True), (1, 40, 2064, 128, 2047, 1, False), (2, 12, 96, 64, 70, 1, True),
             (2, 5, 48, 128, 0, 1, False), (2, 3, 600, 128, 513, 4, True), (1, 2, 80, 64, 61, 3, False),
             (3, 2, 40, 128, 7, 2, True),
             # head sizes between the two lane layouts (OPT-2.7B: 80): rows of their own length in memory
             (2, 32, 560, 80, 543, 1, True), (1, 3, 700, 80, 650, 1, False), (2, 4, 96, 96, 30, 4, True),
             (1, 5, 64, 48, 17, 2, True), (2, 2, 48, 16, 5, 1, False), (1, 2, 128, 112, 100, 3, True), (1, 3, 80, 32, 0, 1, False)]
    for (B, H, cap, d, S0, T, masked) in cases:
        _say(f"decode_attn B={B} H={H} cap={cap} d={d} filled={S0} T={T} mask={masked}")
        S = S0 + T
        kbuf, vbuf = _s8(g, B * H, cap, d), _s8(g, B * H, cap, d)
        q, kn, vn = _s8(g, B * H, T, d), _s8(g, B * H, T, d), _s8(g, B * H, T, d)
        a_qk, a_pv = _scal(g, 1e-4, 2e-3), _scal(g, 1e-3, 1e-2)
        mask = None
        if masked:   # padding on the left of some batch rows plus causality among the new tokens
            mask = torch.zeros(B, 1, T, S)
            mask[0, :, :, :min(3, S0)] = neg
            for t in range(T):
                mask[:, :, t, S0 + t + 1:] = neg
        ref_ctx, ref_p, ref_k, ref_v = orc.decode_attn_s8(q, kn, vn, kbuf, vbuf, S0, mask, H, a_qk, a_pv)
        kd, vd = kbuf.view(B, H, cap, d).to(DEV), vbuf.view(B, H, cap, d).to(DEV)
        args = (q.view(B, H, T, d).to(DEV), kn.view(B, H, T, d).to(DEV), vn.view(B, H, T, d).to(DEV), kd, vd, S0,
                mask.to(DEV) if masked else None)
        assert X.can_decode_attention(*args)
        ctx, probs = X.decode_attention(*args, a_qk, a_pv, want_probs=True)
        assert torch.equal(probs.cpu(), ref_p), "probabilities"
        assert torch.equal(ctx.cpu(), ref_ctx), "context"
        assert torch.equal(kd.cpu().view(B * H, cap, d), ref_k) and torch.equal(vd.cpu().view(B * H, cap, d), ref_v)
        # and against the kernels it replaces, on the device
        kc = kd.view(B * H, cap, d)[:, :S].contiguous()
        sc = C.bmm_s8t_s8n_f32t(q.to(DEV), kc, a_qk)
        pq = X.attn_softmax_q(sc, args[6], H)
        assert torch.equal(pq, probs)
        assert torch.equal(X.bmm_s8t_s8t_s8t(pq, vd.view(B * H, cap, d)[:, :S], a_pv), ctx)
        ctx2, none = X.decode_attention(*args, a_qk, a_pv)   # same cache rows again, no probabilities wanted
        assert none is None and torch.equal(ctx2, ctx)
    assert not X.can_decode_attention(args[0], args[1], args[2], kd, vd, cap, None)        # no room
    assert not X.can_decode_attention(args[0][:, :, :, :16].contiguous(), args[1], args[2], kd, vd, 0, None)   # q narrower than the cache rows


def test_fused_qk_softmax_matches_the_two_kernels_and_the_oracle():
    # Q.K^T + mask + softmax + quantise in one launch: the bytes of bmm_s8t_s8n_f32t followed by attn_softmax_q
    import torch_int._hip_ext as X
    import torch_int._CUDA as C
    g = torch.Generator().manual_seed(83)
    neg = torch.finfo(torch.float32).min
    # (batch, heads, T, S, mask kind)
    cases = [(4, 40, 512, 512, "causal"), (2, 3, 100, 96, "pad"), (1, 4, 64, 16, None), (2, 2, 70, 272, "causal"),
             (1, 2, 1, 512, None), (3, 1, 130, 144, "pad"), (1, 2, 300, 304, "causal"),
             # exactly 128 / 256 / 512 keys, with and without a mask: the kernels compiled for those facts
             (2, 3, 100, 128, "pad"), (1, 2, 70, 128, None), (2, 2, 33, 256, "causal"), (1, 2, 40, 256, None)]
    for (B, H, T, S, kind) in cases:
        _say(f"qk_softmax B={B} H={H} T={T} S={S} mask={kind}")
        q, k = _s8(g, B * H, T, 128), _s8(g, B * H, S, 128)
        alpha = _scal(g, 2e-4, 2e-3)
        mask = None
        if kind is not None:
            mask = torch.zeros(B, 1, T, S)
            if kind == "causal":
                mask += torch.zeros(T, S).masked_fill(torch.arange(S)[None, :] > torch.arange(T)[:, None] + (S - T), neg)
            mask[0, :, :, :5] = neg      # left padding of the first batch row (adds up with causality, may overflow to -inf)
        ref = orc.attn_softmax_q(orc.bmm_s8t_s8n_f32t(q, k, alpha), mask, H)
        qd, kd, md = q.to(DEV), k.to(DEV), (mask.to(DEV) if mask is not None else None)
        assert X.can_attn_qk_softmax_q(qd, kd, md, B, H)
        out = X.attn_qk_softmax_q(qd, kd, md, alpha, H)
        assert out.shape == (B * H, T, S) and out.dtype == torch.int8
        assert torch.equal(out.cpu(), ref), (B, H, T, S, kind, (out.cpu() != ref).sum().item())
        two = X.attn_softmax_q(C.bmm_s8t_s8n_f32t(qd, kd, alpha), md, H)
        assert torch.equal(out, two)
        # keys read in place from a longer cache buffer (batch stride > S * 128)
        buf = torch.zeros(B * H, S + 48, 128, dtype=torch.int8, device=DEV)
        buf[:, :S] = kd
        assert X.can_attn_qk_softmax_q(qd, buf[:, :S], md, B, H)
        assert torch.equal(X.attn_qk_softmax_q(qd, buf[:, :S], md, alpha, H), out)
    assert not X.can_attn_qk_softmax_q(qd, kd[:, :40], None, B, H)          # S not a multiple of 16
    assert not X.can_attn_qk_softmax_q(qd[:, :, :24].contiguous(), kd[:, :, :24].contiguous(), None, B, H)   # head size 24


def test_fused_prefill_attention_matches_the_chain():
    # Q.K^T + softmax-quant + P.V + head merge in one launch against the oracle's chain of the separate operators
    import torch_int._hip_ext as X
    g = torch.Generator().manual_seed(97)
    neg = torch.finfo(torch.float32).min
    shapes = [(4, 40, 512, 512, "causal"), (2, 3, 100, 128, "pad"), (1, 4, 64, 64, None),
              (2, 2, 70, 256, "causal"), (1, 2, 300, 320, "causal"), (1, 1, 5, 448, None),
              # exactly 128 / 256 / 512 keys without a mask: the kernels compiled for that fact
              (1, 2, 80, 128, None), (1, 2, 64, 256, None), (1, 1, 100, 512, None),
              # 513 to 576 keys: still one sweep (36 blocks of 16 keys in the registers), 576 exactly with / without a mask;
              # key counts that 64 does not divide multiply on with V through a last slice that is partly zeros
              (1, 3, 528, 528, "causal"), (2, 2, 64, 544, "pad"), (1, 2, 576, 576, "causal"), (1, 2, 100, 576, None),
              (1, 2, 130, 560, None), (1, 2, 90, 400, "causal"), (1, 2, 64, 16, None), (1, 1, 70, 208, "pad")]
    # head size 128, and 64 (OPT-125m ... 1.3B) on the same kernel's 64-byte-row form
    others = [(2, 32, 512, 512, "causal", 80), (2, 3, 100, 128, "pad", 80), (1, 2, 300, 320, "causal", 96),
              (1, 1, 5, 448, None, 112), (1, 2, 64, 256, None, 48), (2, 2, 70, 256, "causal", 32), (1, 4, 64, 64, None, 16),
              # the three-sweep kernel (more than 576 keys) and single sweeps with a partly filled last slice at those head sizes
              (2, 32, 1024, 1024, "causal", 80), (1, 3, 200, 784, "pad", 80), (2, 2, 100, 400, "causal", 96),
              (1, 2, 528, 528, "causal", 112), (1, 2, 70, 1040, None, 48), (1, 3, 600, 2048, "causal", 32), (1, 2, 40, 560, "pad", 16)]
    for (B, H, T, S, kind, d) in ([sh + (128,) for sh in shapes] + [sh + (64,) for sh in [(4, 12, 512, 512, "causal")] + shapes[1:]]
                                  + others):
        _say(f"attn_prefill B={B} H={H} T={T} S={S} mask={kind} d={d}")
        q, k, v = _s8(g, B * H, T, d), _s8(g, B * H, S, d), _s8(g, B * H, S, d)
        a_qk, a_pv = _scal(g, 2e-4, 2e-3), _scal(g, 2e-3, 2e-2)
        mask = None
        if kind is not None:
            mask = torch.zeros(B, 1, T, S)
            if kind == "causal":
                mask += torch.zeros(T, S).masked_fill(torch.arange(S)[None, :] > torch.arange(T)[:, None] + (S - T), neg)
            mask[0, :, :, :5] = neg
        probs = orc.attn_softmax_q(orc.bmm_s8t_s8n_f32t(q, k, a_qk), mask, H)
        ref = orc.bmm_s8t_s8t_s8t(probs, v, a_pv).view(B, H, T, d).transpose(1, 2).reshape(B, T, H * d)
        qd, kd, md = q.to(DEV), k.to(DEV), (mask.to(DEV) if mask is not None else None)
        vt = X.transpose_last2(v.to(DEV))
        assert X.can_attn_prefill(qd, kd, vt, md, B, H)
        out = X.attn_prefill(qd, kd, vt, md, a_qk, a_pv, H)
        assert out.shape == (B, T, H * d) and out.dtype == torch.int8
        assert torch.equal(out.cpu(), ref), (B, H, T, S, kind, d, (out.cpu() != ref).sum().item())
        # the probabilities alone (the form that stores them instead of multiplying on)
        assert torch.equal(X.attn_qk_softmax_q(qd, kd, md, a_qk, H).cpu(), probs), (B, H, T, S, kind, d)
    z = lambda *shape: torch.zeros(*shape, dtype=torch.int8, device=DEV)   # noqa: E731
    assert not X.can_attn_prefill(z(2, 64, 128), z(2, 440, 128), z(2, 128, 440), None, 1, 2)   # S % 16 != 0
    assert X.can_attn_prefill(z(2, 64, 80), z(2, 400, 80), z(2, 80, 400), None, 1, 2)          # head size 80, S % 64 != 0
    assert not X.can_attn_prefill(z(2, 64, 72), z(2, 400, 72), z(2, 72, 400), None, 1, 2)      # head size 72


def test_runs_are_deterministic():
    # identical bytes on repeated launches (an LDS race would show up here)
    import torch_int._CUDA as C
    g = torch.Generator().manual_seed(77)
    x, w, b = _s8(g, 1024, 1024).to(DEV), _s8(g, 2048, 1024).to(DEV), _s8(g, 2048).to(DEV)
    first = C.linear_a8_w8_b8_o8(x, w, b, 0.002, 0.01)
    first32 = C.linear_a8_w8_b32_o32(x, w, b.to(torch.int32))
    for _ in range(5):
        assert torch.equal(C.linear_a8_w8_b8_o8(x, w, b, 0.002, 0.01), first)
        assert torch.equal(C.linear_a8_w8_b32_o32(x, w, b.to(torch.int32)), first32)


def test_diag_mfma_loop_runs_and_reports_its_work():
    # the diagnostic loop behind bench.py's measured ceiling: every mode launches, exits and counts its operations
    import torch_int._hip_ext as X
    data = torch.randint(-127, 128, (1 << 20,), dtype=torch.int8, device=DEV)
    sink = torch.zeros(1, dtype=torch.int32, device=DEV)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    for mode in (0, 1, 2):
        _say(f"diag_mfma_loop mode {mode}")
        ops = X.diag_mfma_loop(mode, data, 200, sink)
        torch.cuda.synchronize()
        assert ops == cus * 8 * 200 * 16 * 65536
    with pytest.raises(RuntimeError):
        X.diag_mfma_loop(3, data, 200, sink)
    with pytest.raises(RuntimeError):
        X.diag_mfma_loop(0, data[: 1 << 19], 200, sink)


def test_diag_copy_and_mix_loops_run_and_report_their_work():
    # the copy-rate and instruction-mix diagnostics: every form launches, exits and counts its bytes / operations
    import torch_int._hip_ext as X
    data = torch.randint(-127, 128, (3 << 20,), dtype=torch.int8, device=DEV)
    sink = torch.zeros(1, dtype=torch.int32, device=DEV)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    for mode in (0, 1):
        _say(f"diag_copy_loop mode {mode}")
        assert X.diag_copy_loop(mode, data, 50, sink) == cus * 48 * 1024 * 50
        torch.cuda.synchronize()
    for shape, per_cu in ((0, 8 * 40), (1, 4 * 20)):
        for parts in range(1, 16):
            _say(f"diag_mix_loop shape {shape} parts {parts}")
            assert X.diag_mix_loop(shape, parts, data, 50, sink) == cus * per_cu * 50 * 32768
        torch.cuda.synchronize()
    # the read-rate diagnostic: every mode launches and exits, for fewer strips than workgroups and for more
    for (N, K) in [(16, 1024), (64, 3072), (9216, 2048), (20480, 1024)]:
        mat = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=DEV)
        for mode in range(4):
            _say(f"diag_read_loop mode {mode} {N}x{K}")
            assert X.diag_read_loop(mode, mat, sink) == N * K
        torch.cuda.synchronize()
    with pytest.raises(RuntimeError):
        X.diag_read_loop(2, torch.zeros(24, 1024, dtype=torch.int8, device=DEV), sink)
    assert int(sink.item()) == 0
    for bad in (lambda: X.diag_copy_loop(2, data, 50, sink), lambda: X.diag_mix_loop(2, 15, data, 50, sink),
                lambda: X.diag_mix_loop(0, 16, data, 50, sink), lambda: X.diag_mix_loop(0, 15, data[: 1 << 20], 50, sink)):
        with pytest.raises(RuntimeError):
            bad()


def test_diag_store_loop_fills_the_matrix_and_nothing_else():
    # the store-rate diagnostic writes every element of its [M, N] matrix, for any number of workgroups, and stays
    # inside it (guard rows before and after keep their value)
    import torch_int._hip_ext as X
    for (M, N, wgs, reps) in [(256, 160, 1, 1), (512, 480, 3, 2), (1024, 5120, 256, 1), (768, 320, 1000, 1)]:
        _say(f"diag_store_loop {M}x{N} workgroups {wgs}")
        buf = torch.full((M + 2, N), -3.0, device=DEV)
        out = buf[1:M + 1]
        assert X.diag_store_loop(out, wgs, reps) == M * N * 4 * reps
        torch.cuda.synchronize()
        assert bool((out == 1.0).all()) and bool((buf[0] == -3.0).all()) and bool((buf[M + 1] == -3.0).all())
    with pytest.raises(RuntimeError):
        X.diag_store_loop(torch.empty(100, 160, device=DEV), 1, 1)


def test_ln_q_fp16_residual_stream():
    # dq_add_layernorm_q and add + LayerNormQ with fp16 residual / gamma / beta: bit-exact against the oracle's
    # restatement, and within one LSB of the chain of torch ops on the same fp16 tensors on the device
    import torch_int._CUDA as C
    import torch_int._hip_ext as X
    from torch_int.functional.fused import dq_add_layernorm_q_py
    for i, shape in enumerate([(2, 3, 4), (7, 768), (4, 5, 5120), (3, 9216), (2, 12288), (5, 1023), (3, 1), (2, 16384),
                               (2, 20000), (1, 18), (4, 512, 5120)]):
        _say(f"ln_q fp16 shape={shape}")
        g = torch.Generator().manual_seed(600 + i)
        H = shape[-1]
        inp = torch.randint(-60000, 60000, shape, dtype=torch.int32, generator=g)   # fp16 holds these (see below)
        res = torch.randn(shape, generator=g).half()
        gamma = ((1 + 0.02 * torch.randn(H, generator=g)) * 20).half()
        beta = (0.4 * torch.randn(H, generator=g)).half()
        s = _scal(g, 1e-4, 1e-2)
        r_ref, q_ref = orc.dq_add_layernorm_q_f16(inp, s, res, gamma, beta, 1e-5)
        r, q = C.dq_add_layernorm_q(inp.to(DEV), s, res.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5)
        assert r.dtype == torch.float16 and q.dtype == torch.int8 and r.shape == shape and q.shape == shape
        assert torch.equal(r.cpu().view(torch.int16), r_ref.view(torch.int16)), f"r {shape}"
        assert (q.cpu() != q_ref).sum().item() == 0, f"q {shape}"
        r_t, q_t = dq_add_layernorm_q_py(inp.to(DEV), s, res.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5)
        assert r_t.dtype == torch.float16 and (r != r_t).float().mean().item() <= 1e-3 + 1.0 / r.numel()
        assert (q.int() - q_t.int()).abs().max().item() <= 1
        assert (q != q_t).float().mean().item() <= 0.01 + 1.0 / q.numel()
        # residual.add_(x) + LayerNormQ on the fp16 stream, and LayerNormQ alone
        x = torch.randn(shape, generator=g).half()
        r2_ref, q2_ref = orc.add_layernorm_q_f16(x, res, gamma, beta, 1e-5)
        d_res = res.to(DEV)
        q2 = X.add_layernorm_q(x.to(DEV), d_res, gamma.to(DEV), beta.to(DEV), 1e-5)
        assert torch.equal(d_res.cpu().view(torch.int16), r2_ref.view(torch.int16)) and (q2.cpu() != q2_ref).sum().item() == 0
        q3 = X.add_layernorm_q(None, d_res, gamma.to(DEV), beta.to(DEV), 1e-5)
        assert torch.equal(q3, q2) and torch.equal(d_res.cpu().view(torch.int16), r2_ref.view(torch.int16))
    # int32 values beyond fp16's range become infinity, as in torch's own add: same bits as the oracle, NaN rows -> 0
    inp = torch.tensor([[65519, 65520, -70000, 5], [1, 2, 3, 4]], dtype=torch.int32)
    res4, g4, b4 = torch.randn(2, 4, generator=g).half(), torch.ones(4).half(), torch.zeros(4).half()
    r_ref, q_ref = orc.dq_add_layernorm_q_f16(inp, 0.001, res4, g4, b4, 1e-5)
    r, q = C.dq_add_layernorm_q(inp.to(DEV), 0.001, res4.to(DEV), g4.to(DEV), b4.to(DEV), 1e-5)
    assert torch.isinf(r_ref[0, 1]) and torch.isinf(r_ref[0, 2]) and not torch.isinf(r_ref[0, 0])
    assert torch.equal(r.cpu().view(torch.int16), r_ref.view(torch.int16)) and torch.equal(q.cpu(), q_ref)
    assert torch.equal(r.cpu(), torch.add(res4.to(DEV), inp.to(DEV), alpha=0.001).cpu())
    with pytest.raises(RuntimeError, match="share one dtype"):
        C.dq_add_layernorm_q(inp.to(DEV), 0.001, res4.to(DEV), g4.float().to(DEV), b4.to(DEV), 1e-5)
    # the modules: a LayerNormQ converted with .half(), and an fp16 input of an fp32 layer (promoted first)
    from torch_int.nn.fused import LayerNormQ
    ln = LayerNormQ(768)
    ln.weight, ln.bias = torch.randn(768, generator=g) * 20, torch.randn(768, generator=g)
    x16 = torch.randn(5, 768, generator=g).half()
    q32 = copy_to(ln, DEV)(x16.to(DEV))
    _, ref32 = orc.add_layernorm_q(None, x16.float(), ln.weight, ln.bias, 1e-5)
    assert torch.equal(q32.cpu(), ref32)
    q16 = copy_to(ln, DEV).half()(x16.to(DEV))
    _, ref16 = orc.add_layernorm_q_f16(None, x16, ln.weight.half(), ln.bias.half(), 1e-5)
    assert torch.equal(q16.cpu(), ref16)
    # the decoder layer's residual update on an fp16 stream: an fp32 branch output is rounded to fp16, added in
    # place, and the sum normalised -- one kernel; the bits of `x.add_(add.to(x.dtype))` + LayerNormQ on the device
    for (rows, H) in [(7, 768), (64, 5120), (3, 9216), (5, 1001)]:
        _say(f"fp16 residual += fp32 branch, LayerNormQ rows={rows} H={H}")
        lnh = LayerNormQ(H)
        lnh.weight, lnh.bias = (torch.randn(H, generator=g) * 20).half(), torch.randn(H, generator=g).half()
        lnd = copy_to(lnh, DEV)
        res, add = torch.randn(rows, H, generator=g).half(), torch.randn(rows, H, generator=g) * 2
        r_ref, q_ref = orc.add_layernorm_q_f16(add, res, lnh.weight, lnh.bias, 1e-5)
        rd = res.to(DEV)
        qd = lnd(rd, add=add.to(DEV))
        assert torch.equal(rd.cpu().view(torch.int16), r_ref.view(torch.int16)) and torch.equal(qd.cpu(), q_ref)
        chain = res.to(DEV)
        chain.add_(add.to(DEV).to(chain.dtype))
        assert torch.equal(rd, chain)
        y = torch.nn.functional.layer_norm(chain, (H,), lnd.weight, lnd.bias, 1e-5)
        q_chain = y.round().clamp(-128, 127).to(torch.int8)
        assert (qd.int() - q_chain.int()).abs().max() <= 1 and (qd != q_chain).float().mean() <= 0.01
    # the same update without a LayerNorm after it (the fp32 output of fc2 added to an fp16 stream), any length
    import torch_int._hip_ext as X
    from torch_int.nn.linear import W8A8BFP32OFP32Linear
    for n in (1, 7, 4096, 5 * 5120 + 3):
        res, add = torch.randn(n, generator=g).half(), torch.randn(n, generator=g) * 2
        rd = X.add_rounded_(res.to(DEV), add.to(DEV))
        assert torch.equal(rd.cpu(), res.clone().add_(add.to(res.dtype)))
        off = torch.zeros(n + 1, dtype=torch.float16, device=DEV)[1:]     # a base that is not 8-byte aligned
        off.copy_(res)
        assert torch.equal(X.add_rounded_(off, add.to(DEV)).cpu(), res.clone().add_(add.to(res.dtype)))
    m = W8A8BFP32OFP32Linear(256, 320, alpha=0.003)
    m.bias = torch.randn(1, 320, generator=g)
    x = _s8(g, 2, 5, 256)
    resid = torch.randn(2, 5, 320, generator=g).half()
    ref = resid.clone().add_(orc.linear_a8_w8_bfp32_ofp32(x.view(-1, 256), m.weight, m.bias, 0.003, 1.0)
                             .view(2, 5, 320).to(resid.dtype))
    r = resid.to(DEV)
    assert copy_to(m, DEV)(x.to(DEV), add_to=r) is r and torch.equal(r.cpu(), ref)


def copy_to(module, dev):
    import copy
    return copy.deepcopy(module).to(dev)


def _attn_masks(kind, B, T, S):
    if kind is None:
        return None
    neg = torch.finfo(torch.float32).min
    mask = torch.zeros(B, 1, T, S)
    if kind == "causal":
        mask += torch.zeros(T, S).masked_fill(torch.arange(S)[None, :] > torch.arange(T)[:, None] + (S - T), neg)
    mask[0, :, :, :5] = neg      # left padding of the first batch row (adds up with causality, may overflow to -inf)
    return mask


def test_fused_attention_long_keys_and_head_size_64():
    # more than 576 keys (three sweeps), key counts that are not multiples of 64, head size 64; the bytes of
    # bmm_s8t_s8n_f32t -> attn_softmax_q (-> bmm_s8t_s8n_s8t -> head merge), from the oracle and from the device kernels
    import torch_int._hip_ext as X
    import torch_int._CUDA as C
    g = torch.Generator().manual_seed(131)
    # (batch, heads, T, S, head size, mask kind)
    cases = [(1, 3, 2048, 2048, 128, "causal"), (2, 2, 100, 528, 128, "pad"), (1, 2, 64, 1040, 128, None),
             (1, 2, 700, 1024, 128, "causal"), (1, 1, 17, 4096, 128, None), (2, 3, 512, 512, 64, "causal"),
             (1, 4, 200, 208, 64, "pad"), (1, 2, 1500, 1536, 64, "causal"), (2, 2, 70, 48, 128, "causal"),
             (1, 2, 33, 16, 64, None)]
    for (B, H, T, S, d, kind) in cases:
        _say(f"attn long B={B} H={H} T={T} S={S} d={d} mask={kind}")
        q, k, v = _s8(g, B * H, T, d), _s8(g, B * H, S, d), _s8(g, B * H, S, d)
        a_qk, a_pv = _scal(g, 2e-4, 2e-3), _scal(g, 2e-3, 2e-2)
        mask = _attn_masks(kind, B, T, S)
        probs_ref = orc.attn_softmax_q(orc.bmm_s8t_s8n_f32t(q, k, a_qk), mask, H)
        ctx_ref = orc.bmm_s8t_s8t_s8t(probs_ref, v, a_pv).view(B, H, T, d).transpose(1, 2).reshape(B, T, H * d)
        qd, kd, md = q.to(DEV), k.to(DEV), (mask.to(DEV) if mask is not None else None)
        assert X.can_attn_qk_softmax_q(qd, kd, md, B, H)
        probs = X.attn_qk_softmax_q(qd, kd, md, a_qk, H)
        nbad = (probs.cpu() != probs_ref).sum().item()
        assert nbad == 0, (B, H, T, S, d, kind, nbad)
        assert torch.equal(probs, X.attn_softmax_q(C.bmm_s8t_s8n_f32t(qd, kd, a_qk), md, H))
        vt = X.transpose_last2(v.to(DEV))
        assert X.can_attn_prefill(qd, kd, vt, md, B, H)
        ctx = X.attn_prefill(qd, kd, vt, md, a_qk, a_pv, H)
        assert ctx.shape == (B, T, H * d)
        nbad = (ctx.cpu() != ctx_ref).sum().item()
        assert nbad == 0, (B, H, T, S, d, kind, nbad)
        # keys read in place from a longer cache buffer (batch stride > S * d)
        buf = torch.zeros(B * H, S + 48, d, dtype=torch.int8, device=DEV)
        buf[:, :S] = kd
        assert torch.equal(X.attn_prefill(qd, buf[:, :S], vt, md, a_qk, a_pv, H), ctx)
    z = lambda *shape: torch.zeros(*shape, dtype=torch.int8, device=DEV)   # noqa: E731
    assert X.can_attn_qk_softmax_q(z(2, 8, 64), z(2, 48, 64), None, 1, 2)
    assert not X.can_attn_qk_softmax_q(z(2, 8, 64), z(2, 40, 64), None, 1, 2)      # S not a multiple of 16
    assert not X.can_attn_qk_softmax_q(z(1, 8, 64), z(1, 4112, 64), None, 1, 1)    # more than 4096 keys
    assert X.can_attn_qk_softmax_q(z(2, 8, 32), z(2, 48, 32), None, 1, 2)          # head size 32
    assert X.can_attn_qk_softmax_q(z(2, 8, 32), z(2, 528, 32), None, 1, 2)         # beyond 512 keys as well
    assert not X.can_attn_qk_softmax_q(z(2, 8, 40), z(2, 48, 40), None, 1, 2)      # head size 40


@pytest.mark.parametrize("seed", [3, 4])
def test_fused_attention_random_shapes_against_the_operator_chain(seed):
    # 250 seeded random (batch, heads, T, S, head size, mask) per seed through ti_attn_qk_softmax_q and
    # ti_attn_prefill_s8 - single sweep or three, head sizes 32 ... 128, ragged T, causal / padded / fully masked rows /
    # no mask - against the chain of the separate device kernels (each of which the tests above pin to the oracle)
    import random
    import torch_int._CUDA as C
    import torch_int._hip_ext as X
    g = torch.Generator(device=DEV).manual_seed(seed)
    rnd = random.Random(seed + 2)
    neg = torch.finfo(torch.float32).min
    ran = 0
    for it in range(250):
        D = rnd.choice([128, 64, 64, 80, 96, 32, 112, 48, 16])
        B, H = rnd.choice([1, 2, 3]), rnd.choice([1, 2, 5, 8, 33])
        S = (16 * rnd.randrange(1, 70) if it % 3 == 1 else 16 * rnd.randrange(1, 33) if it % 3 == 2 else
             rnd.choice([64, 128, 256, 512, 1024, 2048]))
        T = S if it % 2 == 0 else rnd.randrange(17, min(S, 700) + 1) if S > 17 else S
        kind = rnd.choice(["causal", "pad", None, "rows_masked"])
        _say(f"random attention {it}: B={B} H={H} T={T} S={S} d={D} mask={kind}")
        q, k, v = (torch.randint(-127, 128, (B * H, n, D), dtype=torch.int8, device=DEV, generator=g) for n in (T, S, S))
        a_qk, a_pv = rnd.uniform(2e-4, 2e-3), rnd.uniform(2e-3, 2e-2)
        mask = None
        if kind is not None:
            mask = torch.zeros(B, 1, T, S, device=DEV)
            if kind == "causal":
                mask.masked_fill_(torch.triu(torch.ones(T, S, dtype=torch.bool, device=DEV), S - T + 1), neg)
            elif kind == "pad":
                mask[:, :, :, : rnd.randrange(0, max(1, S // 3))] = neg
            else:
                mask[:, :, : max(1, T // 4), :] = neg      # fully masked rows: uniform probabilities
        if not X.can_attn_qk_softmax_q(q, k, mask, B, H):
            continue
        ran += 1
        want = X.attn_softmax_q(C.bmm_s8t_s8n_f32t(q, k, a_qk), mask, H)
        assert torch.equal(X.attn_qk_softmax_q(q, k, mask, a_qk, H), want), (B, H, T, S, D, kind)
        vt = X.transpose_last2(v)
        if X.can_attn_prefill(q, k, vt, mask, B, H):
            ctx = X.merge_heads(C.bmm_s8t_s8n_s8t(want, vt, a_pv), B, H, T, D)
            assert torch.equal(X.attn_prefill(q, k, vt, mask, a_qk, a_pv, H), ctx), (B, H, T, S, D, kind)
    assert ran >= 220, ran


def test_attention_mask_classes():
    # the class array of a mask (per batch, 64 query rows, 256 keys: mixed / all zero / all one masked value) against
    # a plain restatement, and the long-prefill kernel with and without it on masks built to sit on the class
    # boundaries: same bytes either way, and those of the oracle
    import ctypes
    import torch_int._CUDA as C
    import torch_int._hip_ext as X
    lib = C._lib
    neg = torch.finfo(torch.float32).min
    B, H, T, S, d = 3, 2, 200, 784, 128            # 4 row blocks (the last one 8 rows), 4 key tiles (the last one 16 keys)
    g = torch.Generator().manual_seed(141)
    mask = torch.zeros(B, 1, T, S)
    mask[0, 0, :64, 256:512] = neg                  # uniform
    mask[0, 0, :64, 512:768] = -1e30                # uniform, exactly on the bound
    mask[0, 0, 64:128, 0:256] = -9.9e29             # uniform but above the bound: mixed
    mask[0, 0, 64:128, 256:512] = neg
    mask[0, 0, 100, 300] = -3e38                    # one value differs: mixed
    mask[0, 0, 128:192, 0:256] = -0.0               # negative zero counts as zero
    mask[0, 0, 128:192, 256:512] = torch.randn(64, 256, generator=g)
    mask[0, 0, 192:, 768:] = neg                    # ragged corner, uniform
    mask[1, 0] = neg                                # everything masked: every row is a uniform distribution
    mask[1, 0, 70:, :300] = 0.0
    mask[2, 0] = torch.zeros(T, S).masked_fill(torch.arange(S)[None, :] > torch.arange(T)[:, None] + (S - T), neg)
    mask[2, 0, :, :7] = neg                         # left padding on top of causality
    n = lib.ti_attn_mask_classes_bytes(B, T, S)
    assert n == B * 4 * 4
    md = mask.to(DEV)
    cls = X.mask_classes(md)
    assert cls is not None and cls.numel() == n and X.mask_classes(md) is cls          # cached per mask tensor
    want = torch.zeros(B, 4, 4, dtype=torch.uint8)
    for b in range(B):
        for i in range(4):
            for j in range(4):
                blk = mask[b, 0, 64 * i:64 * i + 64, 256 * j:256 * j + 256]
                if (blk == 0).all():
                    want[b, i, j] = 1
                elif (blk.view(torch.int32) == blk.view(torch.int32).flatten()[0]).all() and blk.flatten()[0] <= -1e30:
                    want[b, i, j] = 2
    assert torch.equal(cls.cpu().view(B, 4, 4), want), (cls.cpu().view(B, 4, 4), want)
    assert want[0, 0].tolist() == [1, 2, 2, 1] and want[0, 1].tolist() == [0, 0, 1, 1] and want[0, 2].tolist() == [1, 0, 1, 1]
    assert want[0, 3, 3] == 2 and want[1, 0].tolist() == [2, 2, 2, 2] and want[1, 1].tolist() == [0, 0, 2, 2]
    md[0, 0, 0, 0] = 1.0                            # an in-place change makes a new class array
    assert X.mask_classes(md) is not cls and X.mask_classes(md)[0] == 0
    md[0, 0, 0, 0] = 0.0
    cls = X.mask_classes(md)

    q, k, v = _s8(g, B * H, T, d), _s8(g, B * H, S, d), _s8(g, B * H, S, d)
    a_qk, a_pv = 0.0007, 0.011
    probs_ref = orc.attn_softmax_q(orc.bmm_s8t_s8n_f32t(q, k, a_qk), mask, H)
    ctx_ref = orc.bmm_s8t_s8t_s8t(probs_ref, v, a_pv).view(B, H, T, d).transpose(1, 2).reshape(B, T, H * d)
    qd, kd = q.to(DEV), k.to(DEV)
    vt = X.transpose_last2(v.to(DEV))
    stream = torch.cuda.current_stream().cuda_stream
    for classes in (None, cls.data_ptr()):
        _say("attention with mask classes:", classes is not None)
        probs = torch.empty((B * H, T, S), dtype=torch.int8, device=DEV)
        rc = lib.ti_attn_qk_softmax_q_mc(qd.data_ptr(), kd.data_ptr(), md.data_ptr(), classes, probs.data_ptr(), B * H, T, S, d,
                                         T * d, S * d, H, a_qk, stream)
        assert rc == 0, lib.ti_last_error()
        assert (probs.cpu() != probs_ref).sum().item() == 0
        ctx = torch.empty((B, T, H * d), dtype=torch.int8, device=DEV)
        rc = lib.ti_attn_prefill_s8_mc(qd.data_ptr(), kd.data_ptr(), vt.data_ptr(), md.data_ptr(), classes, ctx.data_ptr(),
                                       B * H, T, S, d, T * d, S * d, H, a_qk, a_pv, stream)
        assert rc == 0, lib.ti_last_error()
        assert (ctx.cpu() != ctx_ref).sum().item() == 0
    assert probs_ref[2:4].max() > 0 and (probs_ref[2, 0] == probs_ref[2, 0, 0]).all()   # batch 1, row 0: all keys alike
