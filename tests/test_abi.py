"""CPU-side checks of the C-ABI library and the host validation in torch_int._CUDA
(no kernel is launched here)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "torch_int_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ti_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import torch_int._CUDA as C
    lib = ctypes.CDLL(C.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 13
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/torch_int_hip.h but not exported"
    assert C._lib.ti_version() >= 100
    assert C._lib.ti_last_error() == b""


def test_python_module_mirrors_upstream_bindings():
    import torch_int._CUDA as C
    import torch_int.kernels as K
    expected = {"linear_relu_a8_w8_b8_o8", "linear_a8_w8_b32_o32", "linear_a8_w8_bfp32_ofp32",
                "linear_a8_w8_b32_o32_with_scaling", "linear_a8_w8_b8_o8", "dq_add_layernorm_q",
                "bmm_s8t_s8n_s8t", "bmm_s8t_s8n_f32t", "bmm_s8t_s8n_s32t"}  # upstream bindings.cpp:5-20
    assert set(C.__all__) == expected
    for n in expected:
        assert callable(getattr(C, n)) and getattr(K, n) is getattr(C, n)
    # the reference's own import lines work unchanged
    from torch_int._CUDA import bmm_s8t_s8n_s8t, linear_a8_w8_b8_o8  # noqa: F401
    from torch_int.functional.bmm import bmm_i8_o8, bmm_i8_o32  # noqa: F401
    from torch_int.functional.fused import dq_add_layernorm_q_cpp, dq_add_layernorm_q_py  # noqa: F401
    from torch_int.nn.linear import W8A8B8O8Linear, W8A8BFP32OFP32Linear  # noqa: F401


def test_c_abi_rejects_bad_arguments_without_a_device():
    import torch_int._CUDA as C
    lib = C._lib
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    # negative size
    rc = lib.ti_bmm_s8t_s8n_s32t(p, p, p, 1, -1, 4, 16, None)
    assert rc == 1 and b"negative" in lib.ti_last_error()
    # NULL operand with a non-empty problem
    rc = lib.ti_linear_a8_w8_b8_o8(None, p, p, p, 4, 4, 16, 1.0, 1.0, None, 0, None)
    assert rc == 1 and b"NULL" in lib.ti_last_error()
    # misaligned int32 output
    rc = lib.ti_bmm_s8t_s8n_s32t(p, p, p + 1, 1, 1, 4, 16, None)
    assert rc == 2 and b"aligned" in lib.ti_last_error()
    # the no-allocation linear refuses a shape whose split-K scratch exceeds its built-in buffer (before any device call)
    lib.ti_linear_a8_w8_b8_o8_noalloc.argtypes = ([ctypes.c_void_p] * 4 + [ctypes.c_int64] * 3 + [ctypes.c_float] * 2
                                                  + [ctypes.c_void_p])
    rc = lib.ti_linear_a8_w8_b8_o8_noalloc(p, p, p, p, 1024, 9216, 36864, 1.0, 1.0, None)
    assert rc == 1 and b"scratch" in lib.ti_last_error()
    # the diagnostic matrix-pipe loop validates its arguments before touching the device
    lib.ti_diag_mfma_loop.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
                                      ctypes.c_void_p]
    assert lib.ti_diag_mfma_loop(0, p, 64, 100, p, None) == 1 and b"1 MiB" in lib.ti_last_error()
    assert lib.ti_diag_mfma_loop(0, p, 1 << 20, 3, p, None) == 1 and b"even" in lib.ti_last_error()
    lib.ti_diag_store_loop.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                       ctypes.c_void_p]
    assert lib.ti_diag_store_loop(p, 256, 100, 1, 1, None) == 1 and b"multiple of 256" in lib.ti_last_error()
    assert lib.ti_diag_store_loop(p, 256, 160, 0, 1, None) == 1 and b"workgroups" in lib.ti_last_error()
    lib.ti_diag_copy_loop.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
                                      ctypes.c_void_p]
    assert lib.ti_diag_copy_loop(0, p, 1 << 20, 10, p, None) == 1 and b"2 MiB" in lib.ti_last_error()
    assert lib.ti_diag_copy_loop(0, p, 2 << 20, 0, p, None) == 1 and b"iters" in lib.ti_last_error()
    lib.ti_diag_mix_loop.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                     ctypes.c_void_p, ctypes.c_void_p]
    assert lib.ti_diag_mix_loop(0, 15, p, 2 << 20, 10, p, None) == 1 and b"3 MiB" in lib.ti_last_error()
    assert lib.ti_diag_mix_loop(0, 15, p, 3 << 20, 0, p, None) == 1 and b"iters" in lib.ti_last_error()
    lib.ti_diag_read_loop.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
                                      ctypes.c_void_p]
    assert lib.ti_diag_read_loop(4, p, 16, 1024, p, None) == 1 and b"mode" in lib.ti_last_error()
    assert lib.ti_diag_read_loop(2, p, 24, 1024, p, None) == 1 and b"multiple of 16" in lib.ti_last_error()
    assert lib.ti_diag_read_loop(2, p, 16, 1000, p, None) == 1 and b"multiple of 1024" in lib.ti_last_error()
    # beyond the 32-bit tiling limits
    rc = lib.ti_linear_a8_w8_b32_o32(p, p, p, p, 1 << 20, 4, 1 << 20, None, 0, None)
    assert rc == 1 and b"limits" in lib.ti_last_error()
    # batch strides smaller than one matrix; a cache append that does not fit; the row-major product's stride
    i64 = ctypes.c_int64
    lib.ti_bmm_s8t_s8n_f32t_strided.argtypes = [ctypes.c_void_p] * 3 + [i64] * 6 + [ctypes.c_float, ctypes.c_void_p]
    rc = lib.ti_bmm_s8t_s8n_f32t_strided(p, p, p, 2, 1, 4, 16, 8, 64, 1.0, None)
    assert rc == 1 and b"batch strides" in lib.ti_last_error()
    lib.ti_kv_append_s8.argtypes = [ctypes.c_void_p] * 4 + [i64] * 5 + [ctypes.c_void_p]
    rc = lib.ti_kv_append_s8(p, p, p, p, 2, 3, 16, 10, 8, None)
    assert rc == 1 and b"do not fit" in lib.ti_last_error()
    lib.ti_bmm_s8t_s8t_s8t.argtypes = [ctypes.c_void_p] * 3 + [i64] * 5 + [ctypes.c_float, ctypes.c_void_p]
    rc = lib.ti_bmm_s8t_s8t_s8t(p, p, p, 2, 1, 4, 16, 8, 1.0, None)
    assert rc == 1 and b"batch stride" in lib.ti_last_error()
    assert lib.ti_kv_append_s8(None, None, None, None, 0, 1, 16, 8, 0, None) == 0
    # decode attention: shape limits, the pairing of the new rows, alignment; (T, S, head_dim) support query
    lib.ti_decode_attn_s8.argtypes = [ctypes.c_void_p] * 8 + [i64] * 6 + [ctypes.c_float] * 2 + [ctypes.c_void_p]
    lib.ti_decode_attn_supported.argtypes = [i64] * 3
    assert lib.ti_decode_attn_supported(1, 2048, 128) == 1 and lib.ti_decode_attn_supported(4, 2048, 128) == 1
    assert lib.ti_decode_attn_supported(5, 16, 128) == 0 and lib.ti_decode_attn_supported(1, 16, 96) == 1
    assert lib.ti_decode_attn_supported(1, 544, 80) == 1 and lib.ti_decode_attn_supported(1, 16, 40) == 0
    assert lib.ti_decode_attn_supported(1, 16, 144) == 0 and lib.ti_decode_attn_supported(1, 16, 0) == 0
    assert lib.ti_decode_attn_supported(4, 1 << 20, 128) == 0 and lib.ti_decode_attn_supported(1, 0, 128) == 0
    rc = lib.ti_decode_attn_s8(p, p, p, p, p, None, p, None, 4, 5, 128, 64, 32, 2, 1.0, 1.0, None)
    assert rc == 1 and b"unsupported shape" in lib.ti_last_error()
    rc = lib.ti_decode_attn_s8(p, p, None, p, p, None, p, None, 4, 1, 128, 64, 32, 2, 1.0, 1.0, None)
    assert rc == 1 and b"both" in lib.ti_last_error()
    rc = lib.ti_decode_attn_s8(p, p, p, p, p, None, p, None, 4, 1, 128, 16, 32, 2, 1.0, 1.0, None)
    assert rc == 1 and b"do not fit" in lib.ti_last_error()
    rc = lib.ti_decode_attn_s8(p, p, p, p, p, None, p, None, 3, 1, 128, 64, 32, 2, 1.0, 1.0, None)
    assert rc == 1 and b"multiple of heads" in lib.ti_last_error()
    rc = lib.ti_decode_attn_s8(p + 4, p, p, p, p, None, p, None, 4, 1, 128, 64, 32, 2, 1.0, 1.0, None)
    assert rc == 2 and b"aligned" in lib.ti_last_error()
    assert lib.ti_decode_attn_s8(None, None, None, None, None, None, None, None, 0, 1, 128, 64, 32, 2, 1.0, 1.0, None) == 0
    # fused Q.K^T + softmax-quant: shape limits, batch strides, alignment
    lib.ti_attn_qk_softmax_q.argtypes = [ctypes.c_void_p] * 4 + [i64] * 7 + [ctypes.c_float, ctypes.c_void_p]
    lib.ti_attn_qk_softmax_q_supported.argtypes = [i64] * 3
    assert lib.ti_attn_qk_softmax_q_supported(512, 512, 128) == 1 and lib.ti_attn_qk_softmax_q_supported(1, 16, 128) == 1
    assert lib.ti_attn_qk_softmax_q_supported(512, 528, 128) == 1 and lib.ti_attn_qk_softmax_q_supported(512, 40, 128) == 0
    assert lib.ti_attn_qk_softmax_q_supported(512, 512, 64) == 1 and lib.ti_attn_qk_softmax_q_supported(2048, 4096, 64) == 1
    assert lib.ti_attn_qk_softmax_q_supported(512, 4112, 128) == 0 and lib.ti_attn_qk_softmax_q_supported(512, 512, 96) == 1
    # every head size that is a multiple of 16 up to 128, in the single-sweep and the three-sweep kernel alike
    assert lib.ti_attn_qk_softmax_q_supported(512, 528, 96) == 1 and lib.ti_attn_qk_softmax_q_supported(512, 512, 144) == 0
    assert lib.ti_attn_qk_softmax_q_supported(512, 512, 72) == 0 and lib.ti_attn_qk_softmax_q_supported(64, 48, 16) == 1
    lib.ti_attn_prefill_supported.argtypes = [i64] * 3
    assert lib.ti_attn_prefill_supported(512, 512, 80) == 1 and lib.ti_attn_prefill_supported(512, 448, 80) == 1
    assert lib.ti_attn_prefill_supported(512, 400, 80) == 1 and lib.ti_attn_prefill_supported(512, 400, 64) == 1
    assert lib.ti_attn_prefill_supported(512, 1024, 80) == 1 and lib.ti_attn_prefill_supported(512, 1024, 128) == 1
    assert lib.ti_attn_prefill_supported(512, 4112, 80) == 0 and lib.ti_attn_prefill_supported(512, 1024, 8) == 0
    rc = lib.ti_attn_qk_softmax_q(p, p, None, p, 4, 64, 520, 128, 64 * 128, 520 * 128, 2, 1.0, None)
    assert rc == 1 and b"unsupported shape" in lib.ti_last_error()
    rc = lib.ti_attn_qk_softmax_q(p, p, None, p, 4, 64, 64, 128, 64 * 128, 63 * 128, 2, 1.0, None)
    assert rc == 1 and b"batch strides" in lib.ti_last_error()
    rc = lib.ti_attn_qk_softmax_q(p, p + 8, None, p, 4, 64, 64, 128, 64 * 128, 64 * 128, 2, 1.0, None)
    assert rc == 2 and b"aligned" in lib.ti_last_error()
    assert lib.ti_attn_qk_softmax_q(None, None, None, None, 0, 64, 64, 128, 0, 0, 2, 1.0, None) == 0
    lib.ti_attn_prefill_s8.argtypes = [ctypes.c_void_p] * 5 + [i64] * 7 + [ctypes.c_float] * 2 + [ctypes.c_void_p]
    rc = lib.ti_attn_prefill_s8(p, p, p, None, p, 4, 64, 72, 128, 64 * 128, 72 * 128, 2, 1.0, 1.0, None)
    assert rc == 1 and b"multiple of 16" in lib.ti_last_error()
    rc = lib.ti_attn_prefill_s8(p, p, p, None, p, 4, 64, 80, 72, 64 * 72, 80 * 72, 2, 1.0, 1.0, None)
    assert rc == 1 and b"unsupported shape" in lib.ti_last_error()   # head size 72 is not a multiple of 16
    rc = lib.ti_attn_prefill_s8(p, p, None, None, p, 4, 64, 64, 128, 64 * 128, 64 * 128, 2, 1.0, 1.0, None)
    assert rc == 1 and b"vt is NULL" in lib.ti_last_error()
    assert lib.ti_attn_prefill_s8(None, None, None, None, None, 0, 64, 64, 128, 0, 0, 2, 1.0, 1.0, None) == 0
    # grouped head-major linears: head split, group size, per-problem arrays
    pp, fp = ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_float)
    lib.ti_linear_a8_w8_b8_o8_group_heads.argtypes = [ctypes.c_void_p, pp, pp, pp, fp, fp] + [i64] * 6 + [ctypes.c_void_p]
    ptrs, scal = (ctypes.c_void_p * 3)(p, p, p), (ctypes.c_float * 3)(1.0, 1.0, 1.0)
    rc = lib.ti_linear_a8_w8_b8_o8_group_heads(p, ptrs, ptrs, ptrs, scal, scal, 3, 8, 32, 16, 3, 16, None)
    assert rc == 1 and b"multiple of T" in lib.ti_last_error()
    rc = lib.ti_linear_a8_w8_b8_o8_group_heads(p, ptrs, ptrs, ptrs, scal, scal, 5, 8, 32, 16, 4, 16, None)
    assert rc == 1 and b"0 to 4 problems" in lib.ti_last_error()
    rc = lib.ti_linear_a8_w8_b8_o8_group_heads(p, None, ptrs, ptrs, scal, scal, 3, 8, 32, 16, 4, 16, None)
    assert rc == 1 and b"NULL" in lib.ti_last_error()
    assert lib.ti_linear_a8_w8_b8_o8_group_heads(p, ptrs, ptrs, ptrs, scal, scal, 0, 8, 32, 16, 4, 16, None) == 0
    # one decoder layer's decode step from one call: layer description, batch limit, scratch size
    import torch_int._hip_ext as X
    st = X.OptDecodeLayer()
    st.embed, st.heads, st.head_dim, st.ffn = 256, 4, 64, 1024
    need = lib.ti_opt_decoder_layer_decode_scratch_bytes(4, 256, 1024)
    assert need == 5 * 1024 + 4096 + 4096 and lib.ti_opt_decoder_layer_decode_scratch_bytes(0, 256, 1024) == 0
    big = ctypes.create_string_buffer(512)
    pa = (ctypes.addressof(big) + 255) // 256 * 256
    assert lib.ti_opt_decoder_layer_decode(None, p, None, p, p, 4, 64, 10, pa, need, None) == 1
    assert b"no layer" in lib.ti_last_error()
    assert lib.ti_opt_decoder_layer_decode(ctypes.addressof(st), p, None, p, p, 17, 64, 10, pa, need, None) == 1
    assert b"0 to 16" in lib.ti_last_error()
    assert lib.ti_opt_decoder_layer_decode(ctypes.addressof(st), p, None, p, p, 4, 64, 10, pa, need - 1, None) == 1
    assert b"scratch" in lib.ti_last_error()
    assert lib.ti_opt_decoder_layer_decode(ctypes.addressof(st), None, None, p, p, 4, 64, 10, pa, need, None) == 1
    assert b"NULL" in lib.ti_last_error()
    st.head_dim = 80
    assert lib.ti_opt_decoder_layer_decode(ctypes.addressof(st), p, None, p, p, 4, 64, 10, pa, need, None) == 1
    assert b"heads * head_dim" in lib.ti_last_error()
    st.head_dim = 64
    assert lib.ti_opt_decoder_layer_decode(ctypes.addressof(st), None, None, None, None, 0, 64, 10, None, 0, None) == 0
    # ... and a short prefill: token limit, key counts the attention takes, scratch size
    need = lib.ti_opt_decoder_layer_prefill_scratch_bytes(64, 256, 1024)
    assert need == 4 * 64 * 256 + 4 * 64 * 256 + 64 * 1024
    adr = ctypes.addressof(st)
    p16 = (ctypes.addressof(big) + 15) // 16 * 16
    # (arguments that pass: the first step then refuses the description's missing LayerNorm parameters, before any device call)
    assert lib.ti_opt_decoder_layer_prefill(adr, p, None, None, p16, p16, 2, 32, pa, need, None, 0, None) == 1
    assert b"gamma is NULL" in lib.ti_last_error()
    assert lib.ti_opt_decoder_layer_prefill(adr, p, None, None, p16, p16, 8, 1024, pa, need, None, 0, None) == 1
    assert b"4096 tokens" in lib.ti_last_error()
    assert lib.ti_opt_decoder_layer_prefill(adr, p, None, None, p16, p16, 2, 40, pa, need, None, 0, None) == 1
    assert b"multiple of 16" in lib.ti_last_error()
    assert lib.ti_opt_decoder_layer_prefill(adr, p, None, None, p16, p16, 2, 32, pa, need - 1, None, 0, None) == 1
    assert b"scratch" in lib.ti_last_error()
    assert lib.ti_opt_decoder_layer_prefill(None, p, None, None, p16, p16, 2, 32, pa, need, None, 0, None) == 1
    assert lib.ti_opt_decoder_layer_prefill(adr, None, None, None, None, None, 0, 32, None, 0, None, 0, None) == 0
    # empty problems succeed without touching pointers or a device
    assert lib.ti_linear_a8_w8_b8_o8(None, None, None, None, 0, 16, 16, 1.0, 1.0, None, 0, None) == 0
    assert lib.ti_dq_add_layernorm_q(None, 1.0, None, None, None, 1e-5, None, None, 0, 128, None) == 0
    assert lib.ti_last_error() == b""


def test_host_validation_raises_and_never_computes_on_cpu():
    import torch_int._CUDA as C
    x = torch.zeros(4, 16, dtype=torch.int8)
    w = torch.zeros(8, 16, dtype=torch.int8)
    b = torch.zeros(8, dtype=torch.int8)
    with pytest.raises(RuntimeError, match="only run on a HIP"):
        C.linear_a8_w8_b8_o8(x, w, b, 1.0, 1.0)
    with pytest.raises(RuntimeError, match="must be torch.int8"):
        C.linear_a8_w8_b8_o8(x.float(), w, b, 1.0, 1.0)
    with pytest.raises(RuntimeError, match="2-D"):
        C.linear_a8_w8_b8_o8(x[None], w, b, 1.0, 1.0)
    with pytest.raises(RuntimeError, match="only run on a HIP"):
        C.bmm_s8t_s8n_s32t(x[None], w[None])
    with pytest.raises(RuntimeError, match="only run on a HIP"):
        C.dq_add_layernorm_q(torch.zeros(2, 8, dtype=torch.int32), 1.0, torch.zeros(2, 8), torch.ones(8),
                             torch.zeros(8), 1e-5)


def test_split_k_choice_is_sane_at_the_opt_widths():
    # ti_linear_workspace_bytes = splits * M * N * 4 for the split the dispatcher would take (no GPU needed: without
    # a device the cost model prices a 256-CU part).  Pins what the design promises about it: no split for decode
    # (M <= 16) and prefill (M > 1024) shapes or where the unsplit tiles already fill the chip, a slice count that
    # divides K into multiples of 64, and a workspace of at most ten partial copies of the output.
    import torch_int._CUDA as C
    lib = ctypes.CDLL(C.LIB_PATH)
    lib.ti_linear_workspace_bytes.restype = ctypes.c_int64
    lib.ti_linear_workspace_bytes.argtypes = [ctypes.c_int64] * 3
    widths = [(5120, 5120), (20480, 5120), (5120, 20480), (9216, 9216), (36864, 9216), (9216, 36864)]
    for (N, K) in widths:
        for M in (1, 4, 16, 1025, 2048, 8192):
            assert lib.ti_linear_workspace_bytes(M, N, K) == 0, (M, N, K)
        for M in (17, 64, 128, 256, 512, 1024):
            need = lib.ti_linear_workspace_bytes(M, N, K)
            assert need % (M * N * 4) == 0, (M, N, K, need)
            splits = need // (M * N * 4)
            assert splits == 0 or (2 <= splits <= 10 and (K // 64) % splits == 0), (M, N, K, splits)
    # 512 rows of the fc1 widths make 256 tiles of 256x160 / 256x288 on their own: one launch
    assert lib.ti_linear_workspace_bytes(512, 20480, 5120) == 0
    assert lib.ti_linear_workspace_bytes(512, 36864, 9216) == 0
    # 128x80 tiles make 256 of 512 x 5120 outputs and run the whole of a short K in one launch
    assert lib.ti_linear_workspace_bytes(512, 5120, 5120) == 0
    # few output tiles and a long K: split
    for (M, N, K) in [(128, 5120, 5120), (512, 5120, 20480), (1024, 9216, 36864), (128, 36864, 9216)]:
        assert lib.ti_linear_workspace_bytes(M, N, K) >= 2 * M * N * 4, (M, N, K)
    # at least as many slices for 128 rows as for 512 or 1024 at a fixed width (fewer tiles to share the chip)
    for (N, K) in widths:
        got = [lib.ti_linear_workspace_bytes(M, N, K) // (M * N * 4) for M in (128, 512, 1024)]
        assert got[0] >= got[1] and got[0] >= got[2], (N, K, got)
    # OPT-125m widths are too small to be worth a second launch
    assert lib.ti_linear_workspace_bytes(512, 768, 768) == 0


def test_one_launch_split_k_flag_logic():
    # what a GEMM call does for a device state (0 not probed / 1 usable / -1 off) and a misplacement flag:
    # 1 = go on with the one-launch form, 0 = two-launch form, -1 = report the misplacement
    import torch_int._CUDA as C
    lib = ctypes.CDLL(C.LIB_PATH)
    act = lib.ti_selftest_fused_flag_action
    act.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int64]
    assert act(1, 0, 1, 100, 32768) == 1          # usable, nothing flagged
    assert act(0, 0, 1, 100, 32768) == 1          # first use: the probe decides
    assert act(1, 0, 0, 100, 32768) == 0          # switched off by the caller
    assert act(-1, 0, 1, 100, 32768) == 0         # the probe said no
    assert act(1, 0, 1, 32769, 32768) == 0        # more counters than a stream owns
    # a flagged misplacement is reported whatever else holds, also when the form is switched off meanwhile or the
    # call would not have used it
    assert act(1, 1, 1, 100, 32768) == -1
    assert act(1, 1, 0, 100, 32768) == -1
    assert act(1, 1, 1, 1 << 40, 32768) == -1
    assert act(-1, 1, 1, 100, 32768) == -1        # the caller then sees state -1 and reports nothing twice
    # without a device there is nothing to report
    lib.ti_fused_splitk_faulted.restype = ctypes.c_int
    assert lib.ti_fused_splitk_faulted() == 0


def test_one_launch_split_k_stream_slots_are_recycled():
    # eight sets of arrival counters per device: a stream keeps its set, a new stream takes a vacant one, then the
    # set of a stream that has gone idle; with every stream busy it gets none (two-launch form)
    import torch_int._CUDA as C
    lib = ctypes.CDLL(C.LIB_PATH)
    fn = lib.ti_selftest_fused_slot
    fn.argtypes = [ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_uint32), ctypes.c_int, ctypes.c_int64,
                   ctypes.c_uint32, ctypes.POINTER(ctypes.c_int)]
    table, live, fresh = (ctypes.c_int64 * 8)(), ctypes.c_uint32(0), ctypes.c_int(0)

    def slot(stream, busy):
        s = fn(table, ctypes.byref(live), 8, stream, busy, ctypes.byref(fresh))
        return s, fresh.value
    # the null stream (handle 0) is a stream like any other: it must not match an empty slot
    assert slot(0, 0) == (0, 1) and live.value == 1
    assert slot(0, 0) == (0, 0)
    for i in range(1, 8):
        assert slot(1000 + i, 0xFF) == (i, 1)
    assert live.value == 0xFF
    assert slot(1003, 0xFF) == (3, 0)                     # known stream: its own slot, busy or not
    assert slot(2000, 0xFF) == (-1, 1)                    # ninth stream, all busy
    assert slot(2000, 0xFF & ~(1 << 5)) == (5, 1)         # slot 5's stream is idle: handed on
    assert table[5] == 2000 and slot(2000, 0xFF) == (5, 0)
    assert slot(1005, 0xFF) == (-1, 1)                    # the stream that lost its slot is a new one now
    live.value &= ~(1 << 2)                               # a slot given back (probe refused the stream)
    assert slot(3000, 0xFF) == (2, 1)


def test_graph_decoder_refuses_steps_beyond_its_buffers():
    # Int8OPTGraphDecoder.step guards the device-side cache length: after max_new_tokens steps it raises before
    # anything is launched (the recorded attention kernel also clamps the length it reads)
    from torch_int.models.opt import Int8OPTGraphDecoder
    dec = object.__new__(Int8OPTGraphDecoder)
    dec.filled, dec.max_length = 40, 40
    with pytest.raises(RuntimeError, match="max_new_tokens"):
        dec.step(torch.zeros(1, 1, dtype=torch.long))


def test_only_the_256x288_gemm_tiles_spill_registers():
    """The build writes every kernel's register and scratch use (the compiler's own figures) next to the library.
    A kernel that spills still gives the right bits, several times slower, so parity tests cannot see it: only the
    256x288 GEMM tiles, whose 144 accumulator registers per lane leave too few for the operands, are allowed to
    (they are priced with that cost), and every pipelined GEMM and fused attention kernel must fit two waves per
    SIMD (256 registers per lane), which their launch bounds and tilings assume."""
    import json
    import torch_int._CUDA as C
    path = os.path.join(os.path.dirname(C.LIB_PATH), "kernel_resources.json")
    if not os.path.exists(path) or os.path.getmtime(path) + 60 < os.path.getmtime(C.LIB_PATH):
        pytest.skip("no kernel_resources.json from the build of this library")
    kernels = json.load(open(path))["kernels"]
    assert len(kernels) > 300
    spilling = sorted(k for k, v in kernels.items() if v.get("scratch_bytes_per_lane", 0) > 0)
    unexpected = [k for k in spilling if "ILi256ELi288E" not in k]
    assert not unexpected, unexpected
    for k, v in kernels.items():
        if "gemm_pipe" in k or "attn_qk_softmax_q_kernel" in k or "attn_long_kernel" in k:
            assert v["occupancy_waves_per_simd"] >= 2 and v["vgprs"] + v.get("agprs", 0) <= 256, (k, v)
