"""ctypes front-end of the CPU oracle (oracle/qlinear_oracle.c).  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this module; the shipped
package never does.  All arrays are numpy, C-contiguous.

Weight blocks are passed in the reference's array-of-structures layout (mllm/core/DataTypes.hpp:110-121,164-170)
as a uint8 array [N, K/32, 18] (Q4_0) or [N, K/32, 34] (Q8_0); the 2-byte `d` field is an IEEE fp16 bit pattern.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
Q4_0, Q8_0 = 0, 1
SCALE_IEEE, SCALE_X86_REF = 0, 1
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34}

_lib = None
_ref = None


def _p(a, t):
    return a.ctypes.data_as(C.POINTER(t)) if a is not None else None


def lib():
    """Load liboracle.so, building it with the committed Makefile when it is not there yet."""
    global _lib
    if _lib is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            subprocess.check_call(["make", "-C", _HERE, "liboracle.so"])
        L = C.CDLL(so)
        L.orc_fp16_to_fp32.restype = C.c_float
        L.orc_fp16_to_fp32.argtypes = [C.c_uint16]
        L.orc_fp32_to_fp16.restype = C.c_uint16
        L.orc_fp32_to_fp16.argtypes = [C.c_float]
        L.orc_bf16_to_fp32.restype = C.c_float
        L.orc_bf16_to_fp32.argtypes = [C.c_uint16]
        L.orc_fp32_to_bf16.restype = C.c_uint16
        L.orc_fp32_to_bf16.argtypes = [C.c_float]
        L.orc_x86_scale_bits.restype = C.c_uint16
        L.orc_x86_scale_bits.argtypes = [C.c_uint16]
        L.orc_vec_dot.restype = C.c_float
        L.orc_silu.restype = C.c_float
        L.orc_silu.argtypes = [C.c_float]
        L.orc_exp_poly.restype = C.c_float
        L.orc_exp_poly.argtypes = [C.c_float]
        L.orc_linear_q.restype = C.c_int
        L.orc_w4a16_gemm.restype = C.c_int
        L.orc_moe_ffn.restype = C.c_int
        _lib = L
    return _lib


def ref_available():
    return os.path.exists(os.path.join(_HERE, "_ref", "libmllm_ref.so"))


def ref():
    """The reference's own kernels compiled into oracle/_ref (only where `make -C oracle ref` has been run)."""
    global _ref
    if _ref is None:
        L = C.CDLL(os.path.join(_HERE, "_ref", "libmllm_ref.so"))
        L.ref_fp32_to_fp16_bits.restype = C.c_uint16
        L.ref_fp32_to_fp16_bits.argtypes = [C.c_float]
        L.ref_fp16_bits_to_fp32.restype = C.c_float
        L.ref_fp16_bits_to_fp32.argtypes = [C.c_uint16]
        L.ref_scale_store_load.restype = C.c_float
        L.ref_scale_store_load.argtypes = [C.c_uint16]
        _ref = L
    return _ref


# ----------------------------------------------------------------------------- scalar helpers (vectorised in numpy)
def fp16_bits_to_fp32(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)


def x86_scale_bits(bits):
    f = np.vectorize(lambda b: lib().orc_x86_scale_bits(int(b)), otypes=[np.uint16])
    return f(np.asarray(bits, dtype=np.uint16))


def bf16_bits_to_fp32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def fp32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


# ----------------------------------------------------------------------------- Q8_0 activation quantisation
def quantize_rows_q8_0(x):
    """x fp32 [M, K] -> (codes int8 [M, K], scale bit patterns uint16 [M, K/32])."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, K = x.shape
    qs = np.empty((M, K), np.int8)
    d = np.empty((M, K // 32), np.uint16)
    for m in range(M):
        lib().orc_quantize_row_q8_0(_p(x[m], C.c_float), _p(qs[m], C.c_int8), _p(d[m], C.c_uint16), C.c_int(K))
    return qs, d


def dequantize(W, wtype, scale_mode=SCALE_IEEE):
    """W uint8 [N, K/32, blk] -> fp32 [N, K]."""
    W = np.ascontiguousarray(W, dtype=np.uint8)
    N, nb, _ = W.shape
    y = np.empty((N, nb * 32), np.float32)
    for n in range(N):
        lib().orc_dequantize_row(_p(W[n], C.c_uint8), C.c_int(wtype), _p(y[n], C.c_float), C.c_int(nb * 32),
                                 C.c_int(scale_mode))
    return y


def block_isums(W, wtype, xq):
    """exact int32 block dot products [N, M, K/32]."""
    W = np.ascontiguousarray(W, dtype=np.uint8)
    xq = np.ascontiguousarray(xq, dtype=np.int8)
    N, nb, _ = W.shape
    M = xq.shape[0]
    out = np.empty((N, M, nb), np.int32)
    lib().orc_block_isums(_p(W, C.c_uint8), C.c_int(wtype), _p(xq, C.c_int8), C.c_int(M), C.c_int(N),
                          C.c_int(nb * 32), _p(out, C.c_int32))
    return out


def linear_q(x, W, wtype, bias=None, scale_mode=SCALE_X86_REF, return_xq=False):
    """Quantized Linear as the reference CPU path computes it.  x fp32 [M, K]; returns y fp32 [M, N]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    W = np.ascontiguousarray(W, dtype=np.uint8)
    M, K = x.shape
    N, nb, bb = W.shape
    assert nb * 32 == K and bb == BLOCK_BYTES[wtype]
    y = np.empty((M, N), np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    xq = np.empty((M, K), np.int8)
    xd = np.empty((M, nb), np.uint16)
    rc = lib().orc_linear_q(_p(x, C.c_float), _p(W, C.c_uint8), C.c_int(wtype), _p(b, C.c_float), _p(y, C.c_float),
                            C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(scale_mode), _p(xq, C.c_int8),
                            _p(xd, C.c_uint16))
    assert rc == 0, rc
    return (y, xq, xd) if return_xq else y


def linear_q_tiles(x, W, wtype, bias=None, scale_mode=SCALE_X86_REF, threads=8):
    """The same Linear through the AVX2 tile form of the reference's x86 path (tinyBLAS tiles, jobs split over `threads` as
    the op's threads option does); bit-identical to linear_q."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    W = np.ascontiguousarray(W, dtype=np.uint8)
    M, K = x.shape
    N, nb, bb = W.shape
    assert nb * 32 == K and bb == BLOCK_BYTES[wtype]
    y = np.empty((M, N), np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    rc = lib().orc_linear_q_tiles(_p(x, C.c_float), _p(W, C.c_uint8), C.c_int(wtype), _p(b, C.c_float), _p(y, C.c_float),
                                  C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(scale_mode), C.c_int(threads), None)
    assert rc == 0, rc
    return y


# ----------------------------------------------------------------------------- W4A16
def w4a16_dequant(qw, s_bits, zp, group=128):
    """qw uint8 [N, K/2], s uint16 [N, G], zp uint8 [N, ceil(G/2)] -> bf16 bit patterns [N, K]."""
    qw = np.ascontiguousarray(qw, dtype=np.uint8)
    s_bits = np.ascontiguousarray(s_bits, dtype=np.uint16)
    zp = np.ascontiguousarray(zp, dtype=np.uint8)
    N, K = qw.shape[0], qw.shape[1] * 2
    w = np.empty((N, K), np.uint16)
    lib().orc_w4a16_dequant(_p(qw, C.c_uint8), _p(s_bits, C.c_uint16), _p(zp, C.c_uint8), C.c_int(N), C.c_int(K),
                            C.c_int(group), _p(w, C.c_uint16))
    return w


AWQ_ORDER = np.array([0, 2, 4, 6, 1, 3, 5, 7])  # nibble position p of a checkpoint dword holds column 8 j + AWQ_ORDER[p]


def awq_unpack_cols(packed):
    """int32 [R, N/8] -> codes [R, N] in true column order: unpack_cols (pymllm/quantization/methods/awq_marlin.py:202-213)
    followed by the undo_interleave step of awq_to_marlin_zero_points (:248-257)."""
    packed = np.ascontiguousarray(packed).view(np.uint32)
    R, nd = packed.shape
    out = np.zeros((R, nd * 8), np.uint8)
    for i in range(8):
        out[:, i::8] = (packed >> np.uint32(4 * i)) & np.uint32(15)
    undo = np.argsort(AWQ_ORDER)
    return out.reshape(-1, 8)[:, undo].reshape(R, nd * 8)


def awq_unpack(qweight, qzeros, scales_bits):
    """AWQ checkpoint tensors (qweight int32 [K, N/8], qzeros int32 [G, N/8], scales fp16 bits [G, N]) -> the row-major
    tensors of w4a16_dequant / w4a16_gemm: (qw uint8 [N, K/2], scales uint16 [N, G], zeros uint8 [N, ceil(G/2)])."""
    q = awq_unpack_cols(qweight).T  # [N, K]
    z = awq_unpack_cols(qzeros).T  # [N, G]
    if z.shape[1] % 2:
        z = np.concatenate([z, np.zeros((z.shape[0], 1), np.uint8)], axis=1)
    return ((q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8), np.ascontiguousarray(np.asarray(scales_bits, np.uint16).T),
            (z[:, 0::2] | (z[:, 1::2] << 4)).astype(np.uint8))


def w4a16_gemm(a_bits, qw, s_bits, zp, bias_bits=None, group=128):
    """A bf16 bits [M, K] -> C bf16 bits [M, N]."""
    a_bits = np.ascontiguousarray(a_bits, dtype=np.uint16)
    qw = np.ascontiguousarray(qw, dtype=np.uint8)
    s_bits = np.ascontiguousarray(s_bits, dtype=np.uint16)
    zp = np.ascontiguousarray(zp, dtype=np.uint8)
    M, K = a_bits.shape
    N = qw.shape[0]
    c = np.empty((M, N), np.uint16)
    bb = None if bias_bits is None else np.ascontiguousarray(bias_bits, dtype=np.uint16)
    rc = lib().orc_w4a16_gemm(_p(a_bits, C.c_uint16), _p(qw, C.c_uint8), _p(s_bits, C.c_uint16), _p(zp, C.c_uint8),
                              _p(bb, C.c_uint16), _p(c, C.c_uint16), C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(group))
    assert rc == 0, rc
    return c


# ----------------------------------------------------------------------------- W8A8
def per_token_quant_int8(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, K = x.shape
    q = np.empty((M, K), np.int8)
    s = np.empty((M,), np.float32)
    lib().orc_per_token_quant_int8(_p(x, C.c_float), _p(q, C.c_int8), _p(s, C.c_float), C.c_int(M), C.c_int(K))
    return q, s


def w8a8_gemm(xq, x_scale, W, w_scale, bias=None):
    """returns (acc int32 [M, N], y bf16 bits [M, N])."""
    xq = np.ascontiguousarray(xq, dtype=np.int8)
    W = np.ascontiguousarray(W, dtype=np.int8)
    x_scale = np.ascontiguousarray(x_scale, dtype=np.float32)
    w_scale = np.ascontiguousarray(w_scale, dtype=np.float32)
    M, K = xq.shape
    N = W.shape[0]
    acc = np.empty((M, N), np.int32)
    y = np.empty((M, N), np.uint16)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    lib().orc_w8a8_gemm(_p(xq, C.c_int8), _p(x_scale, C.c_float), _p(W, C.c_int8), _p(w_scale, C.c_float),
                        _p(b, C.c_float), _p(acc, C.c_int32), _p(y, C.c_uint16), C.c_int(M), C.c_int(N), C.c_int(K))
    return acc, y


# ----------------------------------------------------------------------------- MoE
def moe_ffn(x, topk_ids, topk_w, Wg, Wu, Wd, wtype, scale_mode=SCALE_X86_REF):
    """x fp32 [T, H]; ids int32 [T, k]; w fp32 [T, k]; Wg/Wu uint8 [E, I, H/32, blk]; Wd uint8 [E, H, I/32, blk]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    ids = np.ascontiguousarray(topk_ids, dtype=np.int32)
    tw = np.ascontiguousarray(topk_w, dtype=np.float32)
    Wg = np.ascontiguousarray(Wg, dtype=np.uint8)
    Wu = np.ascontiguousarray(Wu, dtype=np.uint8)
    Wd = np.ascontiguousarray(Wd, dtype=np.uint8)
    T, H = x.shape
    E, I = Wg.shape[0], Wg.shape[1]
    k = ids.shape[1]
    y = np.empty((T, H), np.float32)
    rc = lib().orc_moe_ffn(_p(x, C.c_float), _p(ids, C.c_int32), _p(tw, C.c_float), _p(Wg, C.c_uint8),
                           _p(Wu, C.c_uint8), _p(Wd, C.c_uint8), C.c_int(wtype), _p(y, C.c_float), C.c_int(T),
                           C.c_int(H), C.c_int(I), C.c_int(E), C.c_int(k), C.c_int(scale_mode))
    assert rc == 0, rc
    return y


def quantize_weight_rows(w, wtype, scale_mode=SCALE_IEEE):
    """fp32 [N, K] -> reference blocks uint8 [N, K/32, 18|34] (offline weight quantizer restatement)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, K = w.shape
    out = np.empty((N, K // 32, 18 if wtype == Q4_0 else 34), np.uint8)
    fn = lib().orc_quantize_row_q4_0 if wtype == Q4_0 else lib().orc_quantize_row_q8_0_blocks
    for n in range(N):
        fn(_p(w[n], C.c_float), _p(out[n], C.c_uint8), C.c_int(K), C.c_int(scale_mode))
    return out


# ----------------------------------------------------------------------------- compiled reference (oracle/_ref)
def ref_quantize_rows_q8_0(x):
    """reference quantize_row_q8_0 -> (codes int8 [M, K], EFFECTIVE scale values fp32 [M, K/32])."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, K = x.shape
    qs = np.empty((M, K), np.int8)
    d = np.empty((M, K // 32), np.float32)
    for m in range(M):
        ref().ref_quantize_row_q8_0(_p(x[m], C.c_float), _p(qs[m], C.c_int8), _p(d[m], C.c_float), C.c_int(K))
    return qs, d


def ref_dequantize(W, wtype):
    W = np.ascontiguousarray(W, dtype=np.uint8)
    N, nb, _ = W.shape
    y = np.empty((N, nb * 32), np.float32)
    for n in range(N):
        ref().ref_dequantize_row(_p(W[n], C.c_uint8), C.c_int(wtype), _p(y[n], C.c_float), C.c_int(nb * 32))
    return y


def ref_linear_q(x, W, wtype, bias=None):
    x = np.ascontiguousarray(x, dtype=np.float32)
    W = np.ascontiguousarray(W, dtype=np.uint8)
    M, K = x.shape
    N = W.shape[0]
    y = np.empty((M, N), np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    ref().ref_linear_q(_p(x, C.c_float), _p(W, C.c_uint8), C.c_int(wtype), _p(b, C.c_float), _p(y, C.c_float),
                       C.c_int(M), C.c_int(N), C.c_int(K))
    return y


def ref_quantize_rows_q4_0(x):
    """reference quantize_row_q4_0 (the offline weight quantizer) -> canonical blocks uint8 [N, K/32, 18]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    N, K = x.shape
    out = np.empty((N, K // 32, 18), np.uint8)
    for n in range(N):
        ref().ref_quantize_row_q4_0(_p(x[n], C.c_float), _p(out[n], C.c_uint8), C.c_int(K))
    return out


# ----------------------------------------------------------------------------- neighbours of Linear in a decoder layer
def exp_poly(x):
    """vexpq_fast_f32 (mllm/backends/cpu/kernels/x86/math.hpp:19-72), elementwise"""
    x = np.ascontiguousarray(x, np.float32)
    L = lib()
    return np.array([L.orc_exp_poly(float(v)) for v in x.ravel()], np.float32).reshape(x.shape)


def silu(x):
    """silu_fp32 over the flattened tensor (x86/silu.cpp:16-56)"""
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty_like(x)
    lib().orc_silu_array(_p(x, C.c_float), _p(y, C.c_float), C.c_int64(x.size))
    return y


def rmsnorm(x, w, eps, add_unit_offset=False):
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    D = x.shape[-1]
    assert w.shape == (D,)
    y = np.empty_like(x)
    lib().orc_rmsnorm(_p(x, C.c_float), _p(w, C.c_float), _p(y, C.c_float), C.c_int64(x.size // D), C.c_int(D),
                      C.c_float(eps), C.c_int(int(add_unit_offset)))
    return y


def softmax(x):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty_like(x)
    n = x.shape[-1]
    lib().orc_softmax_rows(_p(x, C.c_float), _p(y, C.c_float), C.c_int64(x.size // n), C.c_int(n))
    return y


def topk(x, k, largest=True, sorted=True):
    x = np.ascontiguousarray(x, np.float32)
    n = x.shape[-1]
    shape = x.shape[:-1] + (k,)
    v = np.empty(shape, np.float32)
    i = np.empty(shape, np.int32)
    lib().orc_topk_rows(_p(x, C.c_float), _p(v, C.c_float), _p(i, C.c_int32), C.c_int64(x.size // n), C.c_int(n), C.c_int(k),
                        C.c_int(int(largest)), C.c_int(int(sorted)))
    return v, i


def moe_gate(x, w, k, norm=True):
    """returns (ids int32 [M,k], weights fp32 [M,k], scores fp32 [M,E])"""
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    M, H = x.shape
    E = w.shape[0]
    ids = np.empty((M, k), np.int32)
    wt = np.empty((M, k), np.float32)
    sc = np.empty((M, E), np.float32)
    lib().orc_moe_gate(_p(x, C.c_float), _p(w, C.c_float), _p(ids, C.c_int32), _p(wt, C.c_float), _p(sc, C.c_float), C.c_int64(M),
                       C.c_int(H), C.c_int(E), C.c_int(k), C.c_int(int(norm)))
    return ids, wt, sc


# ----------------------------------------------------------------------------- K-quants (Q4_K / Q6_K weights, Q8_K activations)
Q4_K, Q6_K = 2, 3
KBLOCK_BYTES = {Q4_K: 144, Q6_K: 210}


def quantize_rows_q8_K(x):
    """x fp32 [M, K] -> (codes int8 [M, K], scales fp32 [M, K/256], sums of 16 int16 [M, K/16])"""
    x = np.ascontiguousarray(x, np.float32)
    M, K = x.shape
    q = np.empty((M, K), np.int8)
    d = np.empty((M, K // 256), np.float32)
    bs = np.empty((M, K // 16), np.int16)
    for m in range(M):
        lib().orc_quantize_row_q8_K(_p(x[m], C.c_float), _p(q[m], C.c_int8), _p(d[m], C.c_float), _p(bs[m], C.c_int16), C.c_int(K))
    return q, d, bs


def dequantize_k(W, wtype, scale_mode=SCALE_IEEE):
    """W uint8 [N, K/256, 144|210] -> fp32 [N, K]"""
    W = np.ascontiguousarray(W, np.uint8)
    N, nb, bb = W.shape
    assert bb == KBLOCK_BYTES[wtype]
    y = np.empty((N, nb * 256), np.float32)
    fn = lib().orc_dequantize_row_q4_K if wtype == Q4_K else lib().orc_dequantize_row_q6_K
    for n in range(N):
        fn(_p(W[n], C.c_uint8), _p(y[n], C.c_float), C.c_int(nb * 256), C.c_int(scale_mode))
    return y


def linear_kq(x, W, wtype, bias=None, scale_mode=SCALE_X86_REF):
    x = np.ascontiguousarray(x, np.float32)
    W = np.ascontiguousarray(W, np.uint8)
    M, K = x.shape
    N, nb, bb = W.shape
    assert nb * 256 == K and bb == KBLOCK_BYTES[wtype]
    y = np.empty((M, N), np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    lib().orc_linear_kq.restype = C.c_int
    rc = lib().orc_linear_kq(_p(x, C.c_float), _p(W, C.c_uint8), C.c_int(wtype), _p(b, C.c_float), _p(y, C.c_float), C.c_int(M),
                             C.c_int(N), C.c_int(K), C.c_int(scale_mode))
    assert rc == 0, rc
    return y


def moe_ffn_kq(x, topk_ids, topk_w, Wg, Wu, Wd, wtype, scale_mode=SCALE_X86_REF, wtype_down=None):
    """The expert FFN of moe_ffn with Q4_K / Q6_K experts (the formats the shipped Qwen3-MoE recipe quantizes to): per active
    expert three linear_kq calls (each quantizes its input rows to Q8_K), silu over the gathered [cnt, I] tensor and the
    product in between, then acc += per * w in slot order (modeling_qwen3_moe_fa2.hpp:98-100,175-238).  A composition of
    functions pinned on their own (linear_kq, silu); x fp32 [T, H]; Wg/Wu uint8 [E, I, H/256, blk]; Wd uint8 [E, H, I/256, blk];
    slots with an expert id outside [0, E) contribute nothing.  wtype_down: the format of the down projections where it
    differs (the shipped recipe: Q4_K gate / up, Q6_K down, examples/qwen3_moe/quant_cfg_30B_q4_k.json)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    ids = np.ascontiguousarray(topk_ids, dtype=np.int32)
    tw = np.ascontiguousarray(topk_w, dtype=np.float32)
    T, H = x.shape
    E = Wg.shape[0]
    k = ids.shape[1]
    wtype_down = wtype if wtype_down is None else wtype_down
    per = np.zeros((T * k, H), np.float32)
    flat = ids.reshape(-1)
    for e in range(E):
        pos = np.nonzero(flat == e)[0]
        if pos.size == 0:
            continue
        xe = x[pos // k]
        g = linear_kq(xe, Wg[e], wtype, scale_mode=scale_mode)
        u = linear_kq(xe, Wu[e], wtype, scale_mode=scale_mode)
        h = silu(g) * u
        per[pos] = linear_kq(h, Wd[e], wtype_down, scale_mode=scale_mode)
    y = np.zeros((T, H), np.float32)
    per = per.reshape(T, k, H)
    valid = (ids >= 0) & (ids < E)
    for j in range(k):
        y = np.where(valid[:, j:j + 1], y + per[:, j, :] * tw[:, j:j + 1], y).astype(np.float32)
    return y


def kq_block_sums(W, wtype, xq, xbs):
    """exact per-super-block integers: isum int32 [N, M, nb] (and msum for Q4_K, else None)"""
    W = np.ascontiguousarray(W, np.uint8)
    N, nb, bb = W.shape
    M, K = xq.shape
    isum = np.empty((N, M, nb), np.int32)
    msum = np.empty((N, M, nb), np.int32) if wtype == Q4_K else None
    xd = np.ones((M, nb), np.float32)
    L = lib()
    L.orc_vec_dot_q4_K_q8_K.restype = C.c_float
    L.orc_vec_dot_q6_K_q8_K.restype = C.c_float
    for n in range(N):
        for m in range(M):
            if wtype == Q4_K:
                L.orc_vec_dot_q4_K_q8_K(_p(W[n], C.c_uint8), _p(xq[m], C.c_int8), _p(xd[m], C.c_float), _p(xbs[m], C.c_int16),
                                        C.c_int(K), C.c_int(SCALE_IEEE), _p(isum[n, m], C.c_int32), _p(msum[n, m], C.c_int32))
            else:
                L.orc_vec_dot_q6_K_q8_K(_p(W[n], C.c_uint8), _p(xq[m], C.c_int8), _p(xd[m], C.c_float), C.c_int(K),
                                        C.c_int(SCALE_IEEE), _p(isum[n, m], C.c_int32))
    return isum, msum


def ref_quantize_rows_q8_K(x):
    x = np.ascontiguousarray(x, np.float32)
    M, K = x.shape
    q = np.empty((M, K), np.int8)
    d = np.empty((M, K // 256), np.float32)
    bs = np.empty((M, K // 16), np.int16)
    for m in range(M):
        ref().ref_quantize_row_q8_K(_p(x[m], C.c_float), _p(q[m], C.c_int8), _p(d[m], C.c_float), _p(bs[m], C.c_int16), C.c_int(K))
    return q, d, bs


def ref_dequantize_k(W, wtype):
    W = np.ascontiguousarray(W, np.uint8)
    N, nb, bb = W.shape
    y = np.empty((N, nb * 256), np.float32)
    for n in range(N):
        ref().ref_dequantize_row_k(_p(W[n], C.c_uint8), C.c_int(wtype), _p(y[n], C.c_float), C.c_int(nb * 256))
    return y


def ref_linear_kq(x, W, wtype, bias=None):
    x = np.ascontiguousarray(x, np.float32)
    W = np.ascontiguousarray(W, np.uint8)
    M, K = x.shape
    N = W.shape[0]
    y = np.empty((M, N), np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    ref().ref_linear_kq(_p(x, C.c_float), _p(W, C.c_uint8), C.c_int(wtype), _p(b, C.c_float), _p(y, C.c_float), C.c_int(M), C.c_int(N),
                        C.c_int(K))
    return y


def quantize_weight_rows_k(w, wtype, scale_mode=SCALE_IEEE):
    """fp32 [N, K] -> reference super-blocks uint8 [N, K/256, 144|210] (offline K-quant quantizer restatement); the fp16
    fields are stored as scale_mode says (IEEE pattern, or the x86 build's encoding of the pattern as a number)"""
    w = np.ascontiguousarray(w, np.float32)
    N, K = w.shape
    assert K % 256 == 0
    out = np.empty((N, K // 256, KBLOCK_BYTES[wtype]), np.uint8)
    fn = lib().orc_quantize_row_q4_K if wtype == Q4_K else lib().orc_quantize_row_q6_K
    for n in range(N):
        fn(_p(w[n], C.c_float), _p(out[n], C.c_uint8), C.c_int(K), C.c_int(scale_mode))
    return out


def ref_quantize_rows_k(w, wtype):
    """the reference's offline quantizer -> canonical blocks uint8 [N, K/256, 144|210]"""
    w = np.ascontiguousarray(w, np.float32)
    N, K = w.shape
    out = np.empty((N, K // 256, KBLOCK_BYTES[wtype]), np.uint8)
    for n in range(N):
        ref().ref_quantize_row_k(_p(w[n], C.c_float), _p(out[n], C.c_uint8), C.c_int(wtype), C.c_int(K))
    return out
