"""The entry point that allocates nothing (ti_linear_a8_w8_b8_o8_noalloc) against ti_linear_a8_w8_b8_o8,
both through the C ABI: same bytes, on two calls in a row that share the library's built-in scratch, the second
with a smaller input.  Bar: bit-exact (int8 outputs)."""
import ctypes
import sys

import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _s8(g, *shape):
    return torch.randint(-127, 128, shape, dtype=torch.int8, generator=g)


def _bind(lib):
    vp, i64, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_float
    lib.ti_linear_a8_w8_b8_o8_noalloc.argtypes = [vp, vp, vp, vp, i64, i64, i64, f32, f32, vp]
    lib.ti_linear_a8_w8_b8_o8_noalloc.restype = ctypes.c_int
    lib.ti_last_kernel.restype = ctypes.c_char_p
    return lib


def _both(lib, M, N, K, seed, alpha, beta):
    g = torch.Generator().manual_seed(seed)
    x, w, b = _s8(g, M, K), _s8(g, N, K), _s8(g, N)
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.ti_linear_workspace_bytes(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
    ref = torch.empty((M, N), dtype=torch.int8, device=DEV)
    rc = lib.ti_linear_a8_w8_b8_o8(xd.data_ptr(), wd.data_ptr(), bd.data_ptr(), ref.data_ptr(), M, N, K, alpha, beta,
                                   ws.data_ptr(), need, stream)
    assert rc == 0, lib.ti_last_error()
    kernel_ref = lib.ti_last_kernel().decode()
    out = torch.full((M, N), 77, dtype=torch.int8, device=DEV)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.ti_linear_a8_w8_b8_o8_noalloc(xd.data_ptr(), wd.data_ptr(), bd.data_ptr(), out.data_ptr(), M, N, K,
                                           alpha, beta, stream)
    assert rc == 0, lib.ti_last_error()
    assert lib.ti_last_kernel().decode() == kernel_ref
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(out, ref), f"{M}x{N}x{K}: {(out != ref).sum().item()} bytes differ from ti_linear_a8_w8_b8_o8"
    return x, w, b, out.cpu(), kernel_ref


def test_noalloc_linear_matches_the_workspace_entry_point_twice_in_a_row():
    import torch_int._CUDA as C
    lib = _bind(C._lib)
    assert lib.ti_init() == 0, lib.ti_last_error()
    # first a split-K shape that fills most of the scratch, then a smaller one that reuses its first bytes
    _say("noalloc 512x9216x9216 (split-K, 36 MiB of partial products)")
    x, w, b, out, kern = _both(lib, 512, 9216, 9216, 5, 0.0007, 0.02)
    assert kern.startswith(("splitk", "fusedk")), kern
    rows = torch.arange(0, 512, 7)
    assert torch.equal(out[rows], orc.linear_a8_w8_b8_o8(x[rows], w, b, 0.0007, 0.02, acc_fn=orc.gemm_acc_torch))
    _say("noalloc 128x640x4096 (split-K, smaller)")
    x, w, b, out, kern = _both(lib, 128, 640, 4096, 6, 0.002, 0.01)
    assert kern.startswith(("splitk", "fusedk")), kern
    assert torch.equal(out, orc.linear_a8_w8_b8_o8(x, w, b, 0.002, 0.01))
    # shapes that need no scratch go through unchanged: decode, prefill and an odd K
    for (M, N, K) in [(1, 5120, 5120), (2048, 768, 768), (33, 17, 100)]:
        _say(f"noalloc {M}x{N}x{K}")
        x, w, b, out, kern = _both(lib, M, N, K, 7, 0.001, 0.01)
        assert not kern.startswith("splitk")
        assert torch.equal(out, orc.linear_a8_w8_b8_o8(x, w, b, 0.001, 0.01, acc_fn=orc.gemm_acc_torch))
    # and the split-K shape once more after the others
    _both(lib, 512, 5120, 5120, 8, 0.0007, 0.02)


def test_noalloc_linear_refuses_what_the_scratch_cannot_hold():
    import torch_int._CUDA as C
    lib = _bind(C._lib)
    M, N, K = 1024, 9216, 36864
    assert lib.ti_linear_workspace_bytes(M, N, K) > 40 * 2 ** 20
    t = torch.zeros(16, dtype=torch.int8, device=DEV)
    rc = lib.ti_linear_a8_w8_b8_o8_noalloc(t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), M, N, K, 1.0, 1.0,
                                           None)
    assert rc == 1 and b"scratch" in lib.ti_last_error()
