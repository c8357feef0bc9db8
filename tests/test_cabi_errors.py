"""Error behaviour of the C ABI (include/mllm_hip_qlinear.h): null pointers, unknown enums, shapes the kernels do not
take and misaligned pointers are rejected with the documented negative code BEFORE any device call, so these run
without a GPU.  The pointers below are made-up addresses: a rejected call never reads them.

The reference asserts the same preconditions on the CPU path (mllm/backends/cpu/ops/LinearOp.cpp: K a multiple of the
block size; mllm/backends/cpu/kernels/common/ggml/matmul_ggml.cpp: type pairs it has kernels for)."""
import ctypes as C

import pytest

from mllm_amd import _lib

P = 0x7F0000100000        # "device pointer", aligned to 1 MiB
ODD = P + 2               # breaks every alignment requirement above 2 bytes
BADARG, SHAPE, ALIGN = -1, -2, -3
Q4_0, Q8_0, Q4_K, Q6_K = 0, 1, 2, 3
F32, BF16, IMAGE = 0, 1, 2


def _part(packed=P, bias=None, y=P, N=64):
    return (_lib.GemvPart * 1)(_lib.GemvPart(packed, bias, y, N))


# name -> (valid argument list, [(argument index, bad value, expected code)])
def _cases():
    part = _part()
    cases = {
        "mllm_hip_q_prepack": ([Q4_0, P, 0, P, 64, 64, None],
                               [(0, 7, BADARG), (1, None, BADARG), (3, None, BADARG), (2, 5, BADARG), (5, 48, SHAPE), (4, 0, BADARG)]),
        "mllm_hip_linear_q_gemv": ([Q4_0, P, P, F32, None, P, 1, 64, 64, 0, None],
                                   [(0, 9, BADARG), (1, None, BADARG), (2, None, BADARG), (5, None, BADARG), (3, 5, BADARG),
                                    (6, 0, SHAPE), (8, 48, SHAPE), (9, 3, BADARG), (2, ODD, ALIGN)]),
        "mllm_hip_linear_q_gemv_multi": ([Q4_0, 1, part, P, F32, 1, 64, 0, None],
                                         [(1, 0, BADARG), (1, 5, BADARG), (2, None, BADARG), (3, None, BADARG), (5, 0, SHAPE),
                                          (6, 40, SHAPE), (3, ODD, ALIGN)]),
        "mllm_hip_linear_q_gemv_multi_ws": ([Q8_0, 1, part, P, BF16, 4, 64, 0, P, None],
                                            [(3, None, BADARG), (6, 40, SHAPE), (8, ODD, ALIGN)]),
        # the workspace of stated size: one smaller than the image of eight rows is refused
        "mllm_hip_linear_q_gemv_multi_wsn": ([Q8_0, 1, part, P, BF16, 4, 64, 0, P, 8 * 2 * 40, None],
                                             [(3, None, BADARG), (4, IMAGE, BADARG), (6, 40, SHAPE), (8, ODD, ALIGN),
                                              (9, 8 * 2 * 40 - 1, SHAPE)]),
        # the variant that allocates nothing: rows longer than its static array hold are refused
        "mllm_hip_linear_q_gemv_multi_static": ([Q8_0, 1, part, P, BF16, 4, 64, 0, None],
                                                [(3, None, BADARG), (4, IMAGE, BADARG), (6, 32768 + 32, SHAPE), (6, 40, SHAPE)]),
        "mllm_hip_linear_q": ([Q4_0, P, P, F32, None, P, 16, 64, 64, 0, P, None],
                              [(1, None, BADARG), (2, None, BADARG), (5, None, BADARG), (10, None, BADARG), (8, 50, SHAPE),
                               (6, 0, BADARG)]),
        "mllm_hip_linear_q_gemm": ([Q4_0, P, P, F32, None, P, 16, 64, 64, 0, P, None],
                                   [(0, Q4_K, BADARG), (1, None, BADARG), (2, None, BADARG), (5, None, BADARG), (10, None, BADARG),
                                    (8, 50, SHAPE)]),
        "mllm_hip_linear_q_gemm_short": ([Q8_0, P, P, BF16, None, P, 16, 64, 64, 0, P, None],
                                         [(1, None, BADARG), (5, None, BADARG), (10, None, BADARG), (8, 50, SHAPE), (6, -1, BADARG)]),
        "mllm_hip_q_gemm_prepack": ([Q4_0, P, 0, P, 64, 64, None], [(1, None, BADARG), (3, None, BADARG), (5, 48, SHAPE)]),
        "mllm_hip_quantize_q8_0": ([P, F32, P, P, 4, 64, None], [(0, None, BADARG), (2, None, BADARG), (3, None, BADARG), (5, 48, SHAPE),
                                                                 (1, 4, BADARG)]),
        "mllm_hip_quantize_weight_blocks": ([Q4_0, P, P, 0, 8, 64, None], [(1, None, BADARG), (2, None, BADARG), (5, 33, SHAPE),
                                                                           (0, 5, BADARG)]),
        "mllm_hip_q_dequantize": ([Q8_0, P, P, 8, 64, None], [(1, None, BADARG), (2, None, BADARG), (4, 31, SHAPE)]),
        "mllm_hip_mlp_gate_up_q": ([Q4_0, P, P, P, F32, P, None, 1, 64, 64, 0, None],
                                   [(1, None, BADARG), (2, None, BADARG), (3, None, BADARG), (7, 0, SHAPE), (7, 9, SHAPE),
                                    (8, 48, SHAPE), (9, 48, SHAPE), (0, Q6_K, BADARG)]),
        "mllm_hip_moe_ffn_q": ([Q4_0, P, P, P, P, F32, P, P, P, 4, 64, 64, 8, 2, 0, P, None],
                               [(1, None, BADARG), (4, None, BADARG), (6, None, BADARG), (7, None, BADARG), (8, None, BADARG),
                                (15, None, BADARG), (10, 48, SHAPE), (11, 48, SHAPE), (12, 0, BADARG), (13, 0, BADARG), (12, 3073, SHAPE)]),
        "mllm_hip_moe_ffn_q_gemm": ([Q4_0, P, P, P, P, F32, P, P, P, 4, 64, 64, 8, 2, 0, P, None],
                                    [(2, None, BADARG), (3, None, BADARG), (15, None, BADARG), (10, 48, SHAPE), (11, 48, SHAPE),
                                     (4, ODD, ALIGN), (0, Q4_K, BADARG), (12, 3073, SHAPE)]),
        # the routing pass keeps five int arrays of E entries in 64 KB of LDS
        "mllm_hip_moe_route": ([P, 4, 8, 2, None, None, None, P, None], [(0, None, BADARG), (7, None, BADARG), (2, 3073, SHAPE), (2, 0, BADARG)]),
        "mllm_hip_moe_ffn_kq": ([Q4_K, P, P, P, P, F32, P, P, P, 4, 256, 256, 8, 2, P, None],
                                [(0, Q4_0, BADARG), (1, None, BADARG), (3, None, BADARG), (4, None, BADARG), (6, None, BADARG),
                                 (14, None, BADARG), (10, 128, SHAPE), (11, 320, SHAPE), (9, 40000, SHAPE), (4, ODD, ALIGN)]),
        "mllm_hip_moe_ffn_kq2": ([Q4_K, Q6_K, P, P, P, P, F32, P, P, P, 4, 256, 256, 8, 2, P, None],
                                 [(0, Q4_0, BADARG), (1, Q8_0, BADARG), (2, None, BADARG), (5, None, BADARG), (11, 128, SHAPE),
                                  (12, 320, SHAPE), (10, 40000, SHAPE), (5, ODD, ALIGN)]),
        "mllm_hip_kq_quantize_weight_blocks": ([Q6_K, P, P, 0, 8, 256, None], [(0, Q8_0, BADARG), (1, None, BADARG), (2, None, BADARG),
                                                                              (3, 7, BADARG), (5, 128, SHAPE), (4, 0, BADARG)]),
        "mllm_hip_kq_prepack": ([Q4_K, P, 0, P, 8, 256, None], [(0, Q4_0, BADARG), (1, None, BADARG), (3, None, BADARG), (5, 128, SHAPE)]),
        "mllm_hip_linear_kq": ([Q6_K, P, P, F32, None, P, 1, 8, 256, P, None],
                               [(0, Q8_0, BADARG), (1, None, BADARG), (2, None, BADARG), (5, None, BADARG), (9, ODD, ALIGN),
                                (8, 320, SHAPE), (6, 0, BADARG)]),
        # the workspace of stated size: one smaller than the Q8_K image of eight rows is refused
        "mllm_hip_linear_kq_multi_ws": ([Q4_K, 1, part, P, BF16, 4, 256, P, 8 * 256 + 8 * 36, None],
                                        [(0, Q4_0, BADARG), (1, 0, BADARG), (1, 5, BADARG), (2, None, BADARG), (3, None, BADARG),
                                         (4, IMAGE, BADARG), (5, 0, BADARG), (6, 320, SHAPE), (7, ODD, ALIGN), (8, 8 * 256 + 8 * 36 - 1, BADARG)]),
        "mllm_hip_kq_set_slice_meeting": ([-1, 0], [(0, 2, BADARG), (0, -2, BADARG), (1, 9, BADARG), (1, -1, BADARG)]),
        # switches for comparison runs: anything but 0 and 1 is refused and leaves the setting alone
        "mllm_hip_w8a8_set_decode": ([1], [(0, 2, BADARG), (0, -1, BADARG)]),
        "mllm_hip_w8a8_set_decode_mfma_from": ([5], [(0, 0, BADARG), (0, 34, BADARG)]),
        "mllm_hip_w4a16_set_decode": ([1], [(0, 2, BADARG), (0, -1, BADARG)]),
        "mllm_hip_w4a16_set_decode_mfma_from": ([2], [(0, 0, BADARG), (0, 34, BADARG)]),
        "mllm_hip_moe_gate_set_form": ([1], [(0, 2, BADARG), (0, -1, BADARG)]),
        "mllm_hip_kq_gemm_prepack": ([Q4_K, P, 0, P, 8, 256, None], [(0, Q8_0, BADARG), (1, None, BADARG), (5, 96, SHAPE)]),
        "mllm_hip_linear_kq_gemm": ([Q4_K, P, P, F32, None, P, 16, 8, 256, P, None],
                                    [(0, Q4_0, BADARG), (1, None, BADARG), (5, None, BADARG), (9, None, BADARG), (8, 100, SHAPE)]),
        "mllm_hip_linear_kq_gemm_short": ([Q6_K, P, P, BF16, None, P, 16, 8, 256, P, None],
                                          [(0, Q4_0, BADARG), (2, None, BADARG), (9, None, BADARG), (8, 100, SHAPE)]),
        "mllm_hip_quantize_q8_K": ([P, F32, P, P, P, 2, 256, None], [(0, None, BADARG), (2, None, BADARG), (3, None, BADARG),
                                                                     (4, None, BADARG), (6, 64, SHAPE)]),
        "mllm_hip_per_token_quant_int8": ([P, BF16, P, P, 4, 64, None], [(0, None, BADARG), (2, None, BADARG), (3, None, BADARG),
                                                                        (1, 7, BADARG), (4, 0, BADARG)]),
        "mllm_hip_w8a8_gemm": ([P, P, P, P, None, P, None, 16, 64, 64, None],
                               [(0, None, BADARG), (1, None, BADARG), (2, None, BADARG), (3, None, BADARG), (5, None, BADARG),
                                (7, 0, BADARG), (9, 40, SHAPE), (0, ODD, ALIGN)]),
        "mllm_hip_w8a8_linear": ([P, BF16, P, P, None, P, 16, 64, 64, P, None],
                                 [(0, None, BADARG), (2, None, BADARG), (3, None, BADARG), (5, None, BADARG), (9, None, BADARG),
                                  (1, 9, BADARG), (8, 40, SHAPE)]),
        "mllm_hip_w8a8_linear_packed": ([P, BF16, P, P, None, P, 16, 64, 64, P, None],
                                        [(0, None, BADARG), (2, None, BADARG), (3, None, BADARG), (5, None, BADARG), (9, None, BADARG)]),
        "mllm_hip_w4a16_gemm": ([P, P, P, P, None, P, 16, 64, 256, 128, None],
                                [(0, None, BADARG), (1, None, BADARG), (2, None, BADARG), (5, None, BADARG), (9, 100, SHAPE),
                                 (8, 200, SHAPE)]),
        "mllm_hip_w4a16_from_awq": ([P, P, P, 64, 256, 128, P, P, P, None],
                                    [(0, None, BADARG), (1, None, BADARG), (2, None, BADARG), (6, None, BADARG), (7, None, BADARG),
                                     (8, None, BADARG), (3, 60, SHAPE), (4, 100, SHAPE), (5, 96, SHAPE), (6, ODD, ALIGN)]),
        "mllm_hip_w4a16_gemm_packed": ([P, P, None, P, 16, 64, 256, 128, None],
                                       [(0, None, BADARG), (1, None, BADARG), (3, None, BADARG), (7, 100, SHAPE)]),
        "mllm_hip_rmsnorm": ([P, F32, P, P, 1, 64, C.c_float(1e-6), 0, None, 0, None],
                             [(0, None, BADARG), (2, None, BADARG), (1, 3, BADARG), (4, 0, BADARG)]),
        "mllm_hip_silu_mul": ([P, P, P, F32, 1, 64, None, 0, None], [(0, None, BADARG), (1, None, BADARG), (3, 3, BADARG), (4, 0, BADARG)]),
        "mllm_hip_add": ([P, P, P, F32, 1, 64, None, 0, None], [(0, None, BADARG), (1, None, BADARG), (2, None, BADARG)]),
        "mllm_hip_softmax": ([P, P, 2, 16, None], [(0, None, BADARG), (1, None, BADARG), (2, 0, BADARG)]),
        "mllm_hip_topk": ([P, P, P, 2, 16, 4, 1, 1, None], [(0, None, BADARG), (1, None, BADARG), (2, None, BADARG), (5, 0, SHAPE),
                                                            (5, 17, SHAPE)]),
        "mllm_hip_matmul_batched": ([P, P, P, 0, 2, 4, 4, 4, 16, 16, 16, 0, 0, None],
                                    [(0, None, BADARG), (1, None, BADARG), (2, None, BADARG), (3, 2, BADARG), (3, 7, BADARG),
                                     (4, 0, BADARG), (5, 0, BADARG), (8, -1, BADARG), (10, 8, SHAPE), (0, P + 2, ALIGN)]),
        "mllm_hip_matmul_f32": ([P, P, P, 4, 4, 4, 0, 0, None], [(0, None, BADARG), (1, None, BADARG), (2, None, BADARG), (3, 0, BADARG)]),
    }
    return cases


_CASES = _cases()
_PARAMS = [(name, idx, bad, code) for name, (_, bads) in _CASES.items() for (idx, bad, code) in bads]


@pytest.mark.parametrize("name,idx,bad,code", _PARAMS, ids=["%s-arg%d-%s" % (n, i, b) for n, i, b, _ in _PARAMS])
def test_entry_point_rejects_bad_argument(name, idx, bad, code):
    L = _lib.lib()
    args = list(_CASES[name][0])
    args[idx] = bad
    rc = getattr(L, name)(*args)
    assert rc == code, "%s with argument %d = %r returned %d, expected %d" % (name, idx, bad, rc, code)


def test_size_helpers_return_zero_for_shapes_they_do_not_take():
    L = _lib.lib()
    assert L.mllm_hip_q_packed_bytes(Q4_0, 64, 48) == 0
    assert L.mllm_hip_q_packed_bytes(5, 64, 64) == 0
    assert L.mllm_hip_kq_packed_bytes(Q4_K, 8, 128) == 0
    assert L.mllm_hip_kq_packed_bytes(Q4_0, 8, 256) == 0
    assert L.mllm_hip_q_gemm_packed_bytes(Q4_0, 0, 64) == 0
    assert L.mllm_hip_kq_gemm_packed_bytes(Q8_0, 8, 256) == 0
    assert L.mllm_hip_gemv_workspace_bytes(0, 64) == 0
    assert L.mllm_hip_gemv_workspace_bytes(1, 48) == 0
    assert L.mllm_hip_moe_workspace_bytes(4, 48, 64, 8, 2) == 0
    assert L.mllm_hip_moe_gemm_workspace_bytes(4, 64, 64, 0, 2) == 0
    assert L.mllm_hip_w4a16_packed_bytes(64, 256, 100) == 0
    assert L.mllm_hip_moe_kq_workspace_bytes(4, 128, 256, 8, 2) == 0
    assert L.mllm_hip_kq_workspace_bytes_n(4, 128, 64) == 0
    # room for partial sums only where a row has K slices: 256 elements have none, 4096 have four
    assert 0 <= L.mllm_hip_kq_workspace_bytes_n(4, 256, 64) - L.mllm_hip_kq_workspace_bytes(4, 256) < 256
    assert L.mllm_hip_kq_workspace_bytes_n(4, 4096, 64) >= L.mllm_hip_kq_workspace_bytes(4, 4096) + 4 * 4 * 512
    assert L.mllm_hip_kq_workspace_bytes_n(4, 4096, 0) == L.mllm_hip_kq_workspace_bytes(4, 4096)
