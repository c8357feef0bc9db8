"""Loads the in-tree HIP library through its C ABI (include/mllm_hip_qlinear.h).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmllm_hip_qlinear.so")

_lib = None


class GemvPart(C.Structure):
    """mllm_hip_gemv_part"""
    _fields_ = [("packed", C.c_void_p), ("bias", C.c_void_p), ("y", C.c_void_p), ("N", C.c_int64)]


class GemvFusion(C.Structure):
    """mllm_hip_gemv_fusion"""
    _fields_ = [("residual", C.POINTER(C.c_void_p)), ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class HipQLinearError(RuntimeError):
    pass


_ERRS = {-1: "bad argument", -2: "unsupported shape", -3: "misaligned pointer", -4: "no gfx950 device"}


def check(rc, what):
    if rc != 0:
        msg = _ERRS.get(rc, "hipError_t %d" % rc if rc > 0 else "error %d" % rc)
        raise HipQLinearError("%s failed: %s" % (what, msg))


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HipQLinearError(
                "%s not found: build it with `python -m mllm_amd.build` (hipcc, gfx950)" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        i64, vp, ci = C.c_int64, C.c_void_p, C.c_int
        L.mllm_hip_version.restype = C.c_char_p
        L.mllm_hip_init.argtypes = [ci]
        L.mllm_hip_gemv_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_gemv_workspace_bytes.argtypes = [ci, i64]
        L.mllm_hip_q_packed_bytes.restype = C.c_size_t
        L.mllm_hip_q_packed_bytes.argtypes = [ci, i64, i64]
        L.mllm_hip_q_prepack.argtypes = [ci, vp, ci, vp, i64, i64, vp]
        L.mllm_hip_quantize_weight_blocks.argtypes = [ci, vp, vp, ci, i64, i64, vp]
        L.mllm_hip_linear_q_gemv.argtypes = [ci, vp, vp, ci, vp, vp, ci, i64, i64, ci, vp]
        L.mllm_hip_linear_q_gemv_multi.argtypes = [ci, ci, C.POINTER(GemvPart), vp, ci, ci, i64, ci, vp]
        L.mllm_hip_linear_q_gemv_multi_ws.argtypes = [ci, ci, C.POINTER(GemvPart), vp, ci, ci, i64, ci, vp, vp]
        L.mllm_hip_linear_q_gemv_multi_wsn.argtypes = [ci, ci, C.POINTER(GemvPart), vp, ci, ci, i64, ci, vp, C.c_size_t, vp]
        L.mllm_hip_gemv_splitk_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_gemv_splitk_workspace_bytes.argtypes = [ci, i64, i64]
        L.mllm_hip_gemv_workspace_release.argtypes = [vp]
        L.mllm_hip_gemv_workspace_stats.argtypes = [ci, C.POINTER(ci), C.POINTER(ci), C.POINTER(C.c_longlong), C.POINTER(C.c_longlong)]
        L.mllm_hip_linear_q_gemv_multi_static.argtypes = [ci, ci, C.POINTER(GemvPart), vp, ci, ci, i64, ci, vp]
        L.mllm_hip_linear_q_gemv_fused.argtypes = [ci, ci, C.POINTER(GemvPart), C.POINTER(GemvFusion), vp, ci, ci, i64, ci, vp]
        L.mllm_hip_mlp_gate_up_q.argtypes = [ci, vp, vp, vp, ci, vp, vp, ci, i64, i64, ci, vp]
        L.mllm_hip_mlp_set_tuning.argtypes = [ci]
        L.mllm_hip_gemv_set_path.argtypes = [ci]
        L.mllm_hip_gemv_set_request_order.argtypes = [ci]
        L.mllm_hip_kq_set_path.argtypes = [ci]
        L.mllm_hip_moe_kq_set_path.argtypes = [ci]
        L.mllm_hip_rmsnorm.argtypes = [vp, ci, vp, vp, i64, i64, C.c_float, ci, vp, ci, vp]
        L.mllm_hip_silu.argtypes = [vp, vp, ci, i64, vp]
        L.mllm_hip_add.argtypes = [vp, vp, vp, ci, i64, i64, vp, ci, vp]
        L.mllm_hip_mul.argtypes = [vp, vp, vp, ci, i64, i64, vp, ci, vp]
        L.mllm_hip_silu_mul.argtypes = [vp, vp, vp, ci, i64, i64, vp, ci, vp]
        L.mllm_hip_set_exp_mode.argtypes = [ci]
        L.mllm_hip_softmax.argtypes = [vp, vp, i64, i64, vp]
        L.mllm_hip_topk.argtypes = [vp, vp, vp, i64, i64, ci, ci, ci, vp]
        L.mllm_hip_moe_gate.argtypes = [vp, ci, vp, vp, vp, vp, i64, i64, i64, ci, ci, vp]
        L.mllm_hip_moe_gate_set_form.argtypes = [ci]
        L.mllm_hip_w8a8_set_decode.argtypes = [ci]
        L.mllm_hip_w8a8_set_decode_mfma_from.argtypes = [ci]
        L.mllm_hip_w4a16_set_decode.argtypes = [ci]
        L.mllm_hip_w4a16_set_decode_mfma_from.argtypes = [ci]
        L.mllm_hip_quantize_q8_0.argtypes = [vp, ci, vp, vp, i64, i64, vp]
        L.mllm_hip_kq_gemm_packed_bytes.restype = C.c_size_t
        L.mllm_hip_kq_gemm_packed_bytes.argtypes = [ci, i64, i64]
        L.mllm_hip_kq_gemm_prepack.argtypes = [ci, vp, ci, vp, i64, i64, vp]
        L.mllm_hip_linear_kq_gemm_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_linear_kq_gemm_workspace_bytes.argtypes = [i64, i64]
        L.mllm_hip_linear_kq_gemm.argtypes = [ci, vp, vp, ci, vp, vp, i64, i64, i64, vp, vp]
        L.mllm_hip_linear_q_gemm_short_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_linear_q_gemm_short_workspace_bytes.argtypes = [i64, i64, i64]
        L.mllm_hip_linear_q_gemm_short.argtypes = [ci, vp, vp, ci, vp, vp, i64, i64, i64, ci, vp, vp]
        L.mllm_hip_linear_kq_gemm_short_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_linear_kq_gemm_short_workspace_bytes.argtypes = [i64, i64, i64]
        L.mllm_hip_linear_kq_gemm_short.argtypes = [ci, vp, vp, ci, vp, vp, i64, i64, i64, vp, vp]
        L.mllm_hip_kq_packed_bytes.restype = C.c_size_t
        L.mllm_hip_kq_packed_bytes.argtypes = [ci, i64, i64]
        L.mllm_hip_kq_prepack.argtypes = [ci, vp, ci, vp, i64, i64, vp]
        L.mllm_hip_kq_quantize_weight_blocks.argtypes = [ci, vp, vp, ci, i64, i64, vp]
        L.mllm_hip_linear_kq.argtypes = [ci, vp, vp, ci, vp, vp, i64, i64, i64, vp, vp]
        L.mllm_hip_kq_set_tuning.argtypes = [ci, ci, ci]
        L.mllm_hip_linear_kq_multi.argtypes = [ci, ci, C.POINTER(GemvPart), vp, ci, i64, i64, vp, vp]
        L.mllm_hip_kq_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_kq_workspace_bytes.argtypes = [i64, i64]
        L.mllm_hip_kq_set_slice_meeting.argtypes = [ci, ci]
        L.mllm_hip_kq_workspace_bytes_n.restype = C.c_size_t
        L.mllm_hip_kq_workspace_bytes_n.argtypes = [i64, i64, i64]
        L.mllm_hip_linear_kq_multi_ws.argtypes = [ci, ci, C.POINTER(GemvPart), vp, ci, i64, i64, vp, C.c_size_t, vp]
        L.mllm_hip_kq_dequantize.argtypes = [ci, vp, vp, i64, i64, vp]
        L.mllm_hip_quantize_q8_K.argtypes = [vp, ci, vp, vp, vp, i64, i64, vp]
        L.mllm_hip_q_dequantize.argtypes = [ci, vp, vp, i64, i64, vp]
        L.mllm_hip_q_block_isums.argtypes = [ci, vp, vp, vp, i64, i64, i64, vp]
        L.mllm_hip_probe_copy.argtypes = [vp, vp, C.c_size_t, vp]
        L.mllm_hip_probe_q8_scales.argtypes = [C.c_uint32, C.c_uint32, vp, vp]
        L.mllm_hip_gemv_set_tuning.argtypes = [ci, ci, ci]
        L.mllm_hip_per_token_quant_int8.argtypes = [vp, ci, vp, vp, i64, i64, vp]
        L.mllm_hip_w8a8_gemm.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, vp]
        L.mllm_hip_w8a8_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_w8a8_workspace_bytes.argtypes = [i64, i64]
        L.mllm_hip_w8a8_linear.argtypes = [vp, ci, vp, vp, vp, vp, i64, i64, i64, vp, vp]
        L.mllm_hip_w8a8_set_tuning.argtypes = [ci]
        L.mllm_hip_w8a8_nsplit_set_tuning.argtypes = [ci]
        L.mllm_hip_w8a8_packed_bytes.restype = C.c_size_t
        L.mllm_hip_w8a8_packed_bytes.argtypes = [i64, i64]
        L.mllm_hip_w8a8_prepack.argtypes = [vp, i64, i64, vp, vp]
        L.mllm_hip_w8a8_gemm_packed.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, vp]
        L.mllm_hip_w8a8_linear_packed.argtypes = [vp, ci, vp, vp, vp, vp, i64, i64, i64, vp, vp]
        L.mllm_hip_w4a16_gemm.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, ci, vp]
        L.mllm_hip_w4a16_dequantize.argtypes = [vp, vp, vp, vp, i64, i64, ci, vp]
        L.mllm_hip_w4a16_from_awq.argtypes = [vp, vp, vp, i64, i64, ci, vp, vp, vp, vp]
        L.mllm_hip_w4a16_set_tuning.argtypes = [ci]
        L.mllm_hip_w4a16_packed_set_tuning.argtypes = [ci]
        L.mllm_hip_w4a16_packed_bytes.restype = C.c_size_t
        L.mllm_hip_w4a16_packed_bytes.argtypes = [i64, i64, ci]
        L.mllm_hip_w4a16_prepack.argtypes = [vp, vp, vp, i64, i64, ci, vp, vp]
        L.mllm_hip_w4a16_gemm_packed.argtypes = [vp, vp, vp, vp, i64, i64, i64, ci, vp]
        L.mllm_hip_w4a16_dequantize_packed.argtypes = [vp, vp, i64, i64, ci, vp]
        L.mllm_hip_linear_q_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_linear_q_workspace_bytes.argtypes = [i64, i64]
        L.mllm_hip_linear_q.argtypes = [ci, vp, vp, ci, vp, vp, i64, i64, i64, ci, vp, vp]
        L.mllm_hip_moe_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_moe_workspace_bytes.argtypes = [i64, i64, i64, ci, ci]
        L.mllm_hip_moe_ffn_q.argtypes = [ci, vp, vp, vp, vp, ci, vp, vp, vp, i64, i64, i64, ci, ci, ci, vp, vp]
        L.mllm_hip_q_gemm_packed_bytes.restype = C.c_size_t
        L.mllm_hip_q_gemm_packed_bytes.argtypes = [ci, i64, i64]
        L.mllm_hip_q_gemm_prepack.argtypes = [ci, vp, ci, vp, i64, i64, vp]
        L.mllm_hip_linear_q_gemm_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_linear_q_gemm_workspace_bytes.argtypes = [i64, i64]
        L.mllm_hip_linear_q_gemm.argtypes = [ci, vp, vp, ci, vp, vp, i64, i64, i64, ci, vp, vp]
        L.mllm_hip_moe_gemm_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_moe_gemm_workspace_bytes.argtypes = [i64, i64, i64, ci, ci]
        L.mllm_hip_moe_ffn_q_gemm.argtypes = [ci, vp, vp, vp, vp, ci, vp, vp, vp, i64, i64, i64, ci, ci, ci, vp, vp]
        L.mllm_hip_moe_set_tuning.argtypes = [ci, ci]
        L.mllm_hip_moe_kq_workspace_bytes.restype = C.c_size_t
        L.mllm_hip_moe_kq_workspace_bytes.argtypes = [i64, i64, i64, ci, ci]
        L.mllm_hip_moe_ffn_kq.argtypes = [ci, vp, vp, vp, vp, ci, vp, vp, vp, i64, i64, i64, ci, ci, vp, vp]
        L.mllm_hip_moe_ffn_kq2.argtypes = [ci, ci, vp, vp, vp, vp, ci, vp, vp, vp, i64, i64, i64, ci, ci, vp, vp]
        L.mllm_hip_moe_gemm_set_path.argtypes = [ci]
        L.mllm_hip_moe_route.argtypes = [vp, i64, ci, ci, vp, vp, vp, vp, vp]
        L.mllm_hip_matmul_f32.argtypes = [vp, vp, vp, i64, i64, i64, ci, ci, vp]
        L.mllm_hip_matmul_batched.argtypes = [vp, vp, vp, ci, i64, i64, i64, i64, i64, i64, i64, ci, ci, vp]
        _lib = L
    return _lib


# every symbol include/mllm_hip_qlinear.h declares (checked by the CPU test-suite against the header text)
def exported_symbols():
    import re
    hdr = os.path.join(os.path.dirname(_HERE), "include", "mllm_hip_qlinear.h")
    txt = open(hdr).read()
    return sorted(set(re.findall(r"\b(mllm_hip_[a-z0-9_]+)\s*\(", txt)))
