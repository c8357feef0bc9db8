"""Host-side convenience layer over the C ABI for callers that hold torch tensors on the GPU.

torch is used for device memory and the current stream only; every computation is a call into
libmllm_hip_qlinear.so.  Enumerations mirror include/mllm_hip_qlinear.h.
"""
import ctypes as C

import torch

from . import _lib

Q4_0, Q8_0 = 0, 1
F32, BF16 = 0, 1
SCALE_IEEE, SCALE_X86_REF = 0, 1
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34}


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _xdtype(x):
    if x.dtype == torch.float32:
        return F32
    if x.dtype == torch.bfloat16:
        return BF16
    raise TypeError("activations must be float32 or bfloat16, got %s" % x.dtype)


class PackedQWeight:
    """A Q4_0 / Q8_0 weight [N, K] repacked on the device into the layout the kernels read."""

    def __init__(self, wtype, blocks, weight_scale_mode=SCALE_IEEE, layout="gemv"):
        """blocks: uint8 tensor [N, K/32, 18|34] of reference blocks (host or device).  layout "gemv": the decode kernels'
        structure-of-arrays form; "gemm": the matrix-core operand order of linear_q_gemm."""
        assert blocks.dtype == torch.uint8 and blocks.dim() == 3 and blocks.shape[2] == BLOCK_BYTES[wtype]
        assert layout in ("gemv", "gemm")
        self.wtype, self.N, self.K, self.layout = wtype, blocks.shape[0], blocks.shape[1] * 32, layout
        L = _lib.lib()
        size_fn, pack_fn = ((L.mllm_hip_q_packed_bytes, L.mllm_hip_q_prepack) if layout == "gemv" else
                            (L.mllm_hip_q_gemm_packed_bytes, L.mllm_hip_q_gemm_prepack))
        nbytes = size_fn(wtype, self.N, self.K)
        if nbytes == 0:
            raise _lib.HipQLinearError("unsupported weight shape N=%d K=%d" % (self.N, self.K))
        dev_blocks = blocks.contiguous().cuda()
        self.buf = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        _lib.check(pack_fn(wtype, dev_blocks.data_ptr(), weight_scale_mode, self.buf.data_ptr(), self.N, self.K, _stream()),
                   "prepack")
        torch.cuda.current_stream().synchronize()  # dev_blocks may be released after this

    @classmethod
    def synthetic(cls, wtype, N, K, generator=None, layout="gemv"):
        """Random weight drawn on the device (benchmark pools): codes uniform, fp16 block scales |N(0,0.02)|/7 with the low
        three pattern bits cleared so that the IEEE and the x86 reading of the scale agree.  Goes through prepack."""
        nb = K // 32
        blocks = torch.randint(0, 256, (N, nb, BLOCK_BYTES[wtype]), dtype=torch.uint8, device="cuda", generator=generator)
        if wtype == Q8_0:
            blocks[blocks == 0x80] = 0x81  # int8 codes in [-127, 127]
        s = (torch.randn((N, nb), device="cuda", generator=generator) * 0.02).abs() / 7.0
        bits = s.to(torch.float16).view(torch.int16) & ~7
        blocks[:, :, 0:2] = bits.view(torch.uint8).view(N, nb, 2)
        return cls(wtype, blocks, layout=layout)

    @property
    def ptr(self):
        return self.buf.data_ptr()

    def dequantize(self):
        out = torch.empty((self.N, self.K), dtype=torch.float32, device="cuda")
        _lib.check(_lib.lib().mllm_hip_q_dequantize(self.wtype, self.ptr, out.data_ptr(), self.N, self.K, _stream()),
                   "mllm_hip_q_dequantize")
        return out

    def block_isums(self, codes):
        M = codes.shape[0]
        out = torch.empty((self.N, M, self.K // 32), dtype=torch.int32, device="cuda")
        _lib.check(_lib.lib().mllm_hip_q_block_isums(self.wtype, self.ptr, codes.data_ptr(), out.data_ptr(), M, self.N,
                                                     self.K, _stream()), "mllm_hip_q_block_isums")
        return out


def linear_q_gemv(w, x, bias=None, act_scale_mode=SCALE_X86_REF, out=None):
    """y = Linear(x) with Q4_0/Q8_0 weights (more than eight rows: passes of eight).  x [M, K] fp32/bf16 on the GPU -> y fp32 [M, N]."""
    assert x.is_cuda and x.is_contiguous() and x.dim() == 2 and x.shape[1] == w.K
    M = x.shape[0]
    y = out if out is not None else torch.empty((M, w.N), dtype=torch.float32, device="cuda")
    _lib.check(_lib.lib().mllm_hip_linear_q_gemv(w.wtype, w.ptr, x.data_ptr(), _xdtype(x),
                                                 bias.data_ptr() if bias is not None else None, y.data_ptr(), M, w.N,
                                                 w.K, act_scale_mode, _stream()), "mllm_hip_linear_q_gemv")
    return y


def gemv_workspace(M, K, n_total=None):
    """Workspace for linear_q_gemv_multi with three or more activation rows (also the size of a quantized image of x).
    n_total = rows of all weight matrices of a launch together: room for the partial sums of the K slices as well, which
    lets three to eight rows run as one launch."""
    L = _lib.lib()
    size = L.mllm_hip_gemv_workspace_bytes(M, K) if n_total is None else L.mllm_hip_gemv_splitk_workspace_bytes(M, K, n_total)
    return torch.empty(size, dtype=torch.uint8, device="cuda")


def linear_q_gemv_multi(ws, x, biases=None, act_scale_mode=SCALE_X86_REF, outs=None, workspace=None):
    """Sibling projections (same x, same K) in one launch.  ws: list of PackedQWeight; returns the list of outputs.
    With a workspace (gemv_workspace) and M >= 3, x is quantized once by a small kernel instead of in every workgroup."""
    assert 1 <= len(ws) <= 4 and x.is_cuda and x.is_contiguous() and x.dim() == 2
    M, K = x.shape
    if outs is None:
        outs = [torch.empty((M, w.N), dtype=torch.float32, device="cuda") for w in ws]
    parts = (_lib.GemvPart * len(ws))()
    for i, w in enumerate(ws):
        assert w.K == K and w.wtype == ws[0].wtype
        b = biases[i] if biases is not None else None
        parts[i] = _lib.GemvPart(w.ptr, b.data_ptr() if b is not None else None, outs[i].data_ptr(), w.N)
    _lib.check(_lib.lib().mllm_hip_linear_q_gemv_multi_wsn(ws[0].wtype, len(ws), parts, x.data_ptr(), _xdtype(x), M, K,
                                                           act_scale_mode, _p(workspace),
                                                           workspace.numel() if workspace is not None else 0, _stream()),
               "mllm_hip_linear_q_gemv_multi_wsn")
    return outs


Q8_IMAGE = 2  # MLLM_HIP_Q8_IMAGE


def linear_q_gemv_fused(ws, x, M=None, biases=None, residuals=None, act_scale_mode=SCALE_X86_REF, outs=None, image=False,
                        workspace=None):
    """The decode GEMV with its neighbours folded in: residuals[i] (fp32 [M, N], may be outs[i]) is added to part i;
    with image=True `x` is the Q8_0 image a producer (rmsnorm / silu_mul with want_image) wrote for M rows."""
    assert 1 <= len(ws) <= 4 and x.is_cuda and x.is_contiguous()
    K = ws[0].K
    if not image:
        assert x.dim() == 2 and x.shape[1] == K
        M = x.shape[0]
    assert M is not None
    if outs is None:
        outs = [torch.empty((M, w.N), dtype=torch.float32, device="cuda") for w in ws]
    parts = (_lib.GemvPart * len(ws))()
    res = (C.c_void_p * len(ws))()
    for i, w in enumerate(ws):
        assert w.K == K and w.wtype == ws[0].wtype
        b = biases[i] if biases is not None else None
        parts[i] = _lib.GemvPart(w.ptr, b.data_ptr() if b is not None else None, outs[i].data_ptr(), w.N)
        r = residuals[i] if residuals is not None else None
        if r is not None:
            assert r.dtype == torch.float32 and r.is_contiguous() and tuple(r.shape) == (M, w.N)
        res[i] = r.data_ptr() if r is not None else None
    fu = _lib.GemvFusion(res if residuals is not None else None, _p(workspace), workspace.numel() if workspace is not None else 0)
    _lib.check(_lib.lib().mllm_hip_linear_q_gemv_fused(ws[0].wtype, len(ws), parts, C.byref(fu), x.data_ptr(),
                                                       Q8_IMAGE if image else _xdtype(x), M, K, act_scale_mode, _stream()),
               "mllm_hip_linear_q_gemv_fused")
    return outs


def quantize_weight_blocks(w, wtype, weight_scale_mode=SCALE_IEEE):
    """fp32 [N, K] on the GPU -> reference blocks uint8 [N, K/32, 18|34] (the offline quantizer's output)."""
    assert w.is_cuda and w.is_contiguous() and w.dtype == torch.float32 and w.dim() == 2 and w.shape[1] % 32 == 0
    N, K = w.shape
    out = torch.empty((N, K // 32, BLOCK_BYTES[wtype]), dtype=torch.uint8, device="cuda")
    _lib.check(_lib.lib().mllm_hip_quantize_weight_blocks(wtype, w.data_ptr(), out.data_ptr(), weight_scale_mode, N, K,
                                                          _stream()), "mllm_hip_quantize_weight_blocks")
    return out


def quantize_q8_0(x):
    """x [M, K] -> (codes int8 [M, K], scale patterns int16-viewed-as-uint16 [M, K/32])."""
    assert x.is_cuda and x.is_contiguous() and x.dim() == 2
    M, K = x.shape
    codes = torch.empty((M, K), dtype=torch.int8, device="cuda")
    d = torch.empty((M, K // 32), dtype=torch.int16, device="cuda")
    _lib.check(_lib.lib().mllm_hip_quantize_q8_0(x.data_ptr(), _xdtype(x), codes.data_ptr(), d.data_ptr(), M, K,
                                                 _stream()), "mllm_hip_quantize_q8_0")
    return codes, d


# ----------------------------------------------------------------------------- W8A8 (per-token dynamic int8)
def _p(t):
    return t.data_ptr() if t is not None else None


def per_token_quant_int8(x):
    """x [M, K] fp32/bf16 -> (q int8 [M, K], scale fp32 [M])."""
    assert x.is_cuda and x.is_contiguous() and x.dim() == 2
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.int8, device="cuda")
    s = torch.empty((M,), dtype=torch.float32, device="cuda")
    _lib.check(_lib.lib().mllm_hip_per_token_quant_int8(x.data_ptr(), _xdtype(x), q.data_ptr(), s.data_ptr(), M, K,
                                                        _stream()), "mllm_hip_per_token_quant_int8")
    return q, s


def w8a8_gemm(xq, x_scale, W, w_scale, bias=None, want_acc=False, out=None):
    """xq int8 [M, K], W int8 [N, K] -> bf16 [M, N] (and the int32 accumulators when want_acc)."""
    M, K = xq.shape
    N = W.shape[0]
    assert W.shape[1] == K and xq.is_contiguous() and W.is_contiguous()
    y = out if out is not None else torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    acc = torch.empty((M, N), dtype=torch.int32, device="cuda") if want_acc else None
    _lib.check(_lib.lib().mllm_hip_w8a8_gemm(xq.data_ptr(), _p(x_scale), W.data_ptr(), _p(w_scale), _p(bias),
                                             y.data_ptr(), _p(acc), M, N, K, _stream()), "mllm_hip_w8a8_gemm")
    return (y, acc) if want_acc else y


def w8a8_linear(x, W, w_scale, bias=None, workspace=None, out=None):
    """bf16/fp32 x [M, K] -> bf16 [M, N]: per-token quantization + int8 GEMM, two launches."""
    M, K = x.shape
    N = W.shape[0]
    L = _lib.lib()
    if workspace is None:
        workspace = torch.empty(L.mllm_hip_w8a8_workspace_bytes(M, K), dtype=torch.uint8, device="cuda")
    y = out if out is not None else torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    _lib.check(L.mllm_hip_w8a8_linear(x.data_ptr(), _xdtype(x), W.data_ptr(), w_scale.data_ptr(), _p(bias),
                                      y.data_ptr(), M, N, K, workspace.data_ptr(), _stream()), "mllm_hip_w8a8_linear")
    return y


def w8a8_prepack(W):
    """W int8 [N, K] -> the matrix in MFMA operand order (uint8, mllm_hip_w8a8_packed_bytes long), done once per weight."""
    assert W.is_cuda and W.is_contiguous() and W.dtype == torch.int8 and W.dim() == 2
    N, K = W.shape
    L = _lib.lib()
    packed = torch.empty(L.mllm_hip_w8a8_packed_bytes(N, K), dtype=torch.uint8, device="cuda")
    _lib.check(L.mllm_hip_w8a8_prepack(W.data_ptr(), N, K, packed.data_ptr(), _stream()), "mllm_hip_w8a8_prepack")
    return packed


def w8a8_gemm_packed(xq, x_scale, W_packed, N, w_scale, bias=None, want_acc=False, out=None):
    """As w8a8_gemm, with the weights from w8a8_prepack (N = their row count)."""
    M, K = xq.shape
    L = _lib.lib()
    assert xq.is_contiguous() and W_packed.numel() == L.mllm_hip_w8a8_packed_bytes(N, K)
    y = out if out is not None else torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    acc = torch.empty((M, N), dtype=torch.int32, device="cuda") if want_acc else None
    _lib.check(L.mllm_hip_w8a8_gemm_packed(xq.data_ptr(), _p(x_scale), W_packed.data_ptr(), _p(w_scale), _p(bias),
                                           y.data_ptr(), _p(acc), M, N, K, _stream()), "mllm_hip_w8a8_gemm_packed")
    return (y, acc) if want_acc else y


def w8a8_linear_packed(x, W_packed, N, w_scale, bias=None, workspace=None, out=None):
    """As w8a8_linear, with the weights from w8a8_prepack."""
    M, K = x.shape
    L = _lib.lib()
    assert W_packed.numel() == L.mllm_hip_w8a8_packed_bytes(N, K)
    if workspace is None:
        workspace = torch.empty(L.mllm_hip_w8a8_workspace_bytes(M, K), dtype=torch.uint8, device="cuda")
    y = out if out is not None else torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    _lib.check(L.mllm_hip_w8a8_linear_packed(x.data_ptr(), _xdtype(x), W_packed.data_ptr(), w_scale.data_ptr(), _p(bias),
                                             y.data_ptr(), M, N, K, workspace.data_ptr(), _stream()),
               "mllm_hip_w8a8_linear_packed")
    return y


# ----------------------------------------------------------------------------- W4A16 (group-wise uint4 + zero point)
def w4a16_gemm(a, qw, scales, zeros, bias=None, group=128, out=None):
    """a bf16 [M, K]; qw uint8 [N, K/2]; scales fp16 [N, K/group]; zeros uint8 [N, ceil(K/group/2)] -> bf16 [M, N]."""
    assert a.dtype == torch.bfloat16 and a.is_contiguous() and qw.dtype == torch.uint8 and scales.dtype == torch.float16
    M, K = a.shape
    N = qw.shape[0]
    assert qw.shape[1] * 2 == K
    y = out if out is not None else torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    _lib.check(_lib.lib().mllm_hip_w4a16_gemm(a.data_ptr(), qw.data_ptr(), scales.data_ptr(), zeros.data_ptr(), _p(bias),
                                              y.data_ptr(), M, N, K, group, _stream()), "mllm_hip_w4a16_gemm")
    return y


def w4a16_from_awq(qweight, qzeros, scales, group=128):
    """AWQ checkpoint tensors (qweight int32 [K, N/8], qzeros int32 [K/group, N/8], scales fp16 [K/group, N]) ->
    (qw uint8 [N, K/2], scales fp16 [N, K/group], zeros uint8 [N, ceil(K/group/2)]), the inputs of w4a16_gemm / w4a16_prepack.
    pymllm/quantization/methods/awq_marlin.py:284-410."""
    assert qweight.dtype == torch.int32 and qzeros.dtype == torch.int32 and scales.dtype == torch.float16
    assert qweight.is_contiguous() and qzeros.is_contiguous() and scales.is_contiguous()
    K, N = qweight.shape[0], qweight.shape[1] * 8
    G = K // group
    assert qzeros.shape == (G, N // 8) and scales.shape == (G, N)
    qw = torch.empty((N, K // 2), dtype=torch.uint8, device="cuda")
    s = torch.empty((N, G), dtype=torch.float16, device="cuda")
    z = torch.empty((N, (G + 1) // 2), dtype=torch.uint8, device="cuda")
    _lib.check(_lib.lib().mllm_hip_w4a16_from_awq(qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(), N, K, group,
                                                  qw.data_ptr(), s.data_ptr(), z.data_ptr(), _stream()),
               "mllm_hip_w4a16_from_awq")
    return qw, s, z


def w4a16_prepack(qw, scales, zeros, group=128):
    """Checkpoint tensors -> the packed weight blob of the fast GEMM (uint8), done once per weight."""
    assert qw.dtype == torch.uint8 and scales.dtype == torch.float16 and qw.is_contiguous() and scales.is_contiguous()
    N, K = qw.shape[0], qw.shape[1] * 2
    L = _lib.lib()
    packed = torch.empty(L.mllm_hip_w4a16_packed_bytes(N, K, group), dtype=torch.uint8, device="cuda")
    _lib.check(L.mllm_hip_w4a16_prepack(qw.data_ptr(), scales.data_ptr(), zeros.data_ptr(), N, K, group, packed.data_ptr(),
                                        _stream()), "mllm_hip_w4a16_prepack")
    return packed


def w4a16_gemm_packed(a, packed, N, bias=None, group=128, out=None):
    """a bf16 [M, K] x packed weights (w4a16_prepack) -> bf16 [M, N]."""
    assert a.dtype == torch.bfloat16 and a.is_contiguous()
    M, K = a.shape
    L = _lib.lib()
    assert packed.numel() == L.mllm_hip_w4a16_packed_bytes(N, K, group)
    y = out if out is not None else torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    _lib.check(L.mllm_hip_w4a16_gemm_packed(a.data_ptr(), packed.data_ptr(), _p(bias), y.data_ptr(), M, N, K, group,
                                            _stream()), "mllm_hip_w4a16_gemm_packed")
    return y


def w4a16_dequantize_packed(packed, N, K, group=128):
    w = torch.empty((N, K), dtype=torch.bfloat16, device="cuda")
    _lib.check(_lib.lib().mllm_hip_w4a16_dequantize_packed(packed.data_ptr(), w.data_ptr(), N, K, group, _stream()),
               "mllm_hip_w4a16_dequantize_packed")
    return w


def w4a16_dequantize(qw, scales, zeros, group=128):
    N, K = qw.shape[0], qw.shape[1] * 2
    w = torch.empty((N, K), dtype=torch.bfloat16, device="cuda")
    _lib.check(_lib.lib().mllm_hip_w4a16_dequantize(qw.data_ptr(), scales.data_ptr(), zeros.data_ptr(), w.data_ptr(), N, K,
                                                    group, _stream()), "mllm_hip_w4a16_dequantize")
    return w


# ----------------------------------------------------------------------------- any-M quantized Linear and the MoE FFN
def linear_q(w, x, bias=None, act_scale_mode=SCALE_X86_REF, workspace=None, out=None):
    """Q4_0/Q8_0 Linear for any number of rows: stand-alone Q8_0 activation quantization + MFMA block-dot tiles (up to 16 rows:
    passes of the eight-row GEMV, the same arithmetic)."""
    assert x.is_cuda and x.is_contiguous() and x.dim() == 2 and x.shape[1] == w.K
    M = x.shape[0]
    L = _lib.lib()
    if workspace is None:
        workspace = torch.empty(L.mllm_hip_linear_q_workspace_bytes(M, w.K), dtype=torch.uint8, device="cuda")
    y = out if out is not None else torch.empty((M, w.N), dtype=torch.float32, device="cuda")
    _lib.check(L.mllm_hip_linear_q(w.wtype, w.ptr, x.data_ptr(), _xdtype(x), _p(bias), y.data_ptr(), M, w.N, w.K,
                                   act_scale_mode, workspace.data_ptr(), _stream()), "mllm_hip_linear_q")
    return y


class PackedExperts:
    """E pre-packed [N, K] weight matrices back to back: layout "gemv" for mllm_hip_moe_ffn_q, "gemm" for
    mllm_hip_moe_ffn_q_gemm."""

    def __init__(self, wtype, blocks, weight_scale_mode=SCALE_IEEE, layout="gemv"):
        """blocks: uint8 [E, N, K/32, 18|34] (host or device)."""
        assert blocks.dtype == torch.uint8 and blocks.dim() == 4 and layout in ("gemv", "gemm")
        self.wtype, self.E, self.N, self.K, self.layout = wtype, blocks.shape[0], blocks.shape[1], blocks.shape[2] * 32, layout
        L = _lib.lib()
        size_fn, pack_fn = ((L.mllm_hip_q_packed_bytes, L.mllm_hip_q_prepack) if layout == "gemv" else
                            (L.mllm_hip_q_gemm_packed_bytes, L.mllm_hip_q_gemm_prepack))
        self.stride = size_fn(wtype, self.N, self.K)
        self.buf = torch.empty(self.E * self.stride, dtype=torch.uint8, device="cuda")
        for e in range(self.E):
            dev = blocks[e].contiguous().cuda()
            _lib.check(pack_fn(wtype, dev.data_ptr(), weight_scale_mode, self.buf.data_ptr() + e * self.stride, self.N,
                               self.K, _stream()), "prepack")
            torch.cuda.current_stream().synchronize()

    @classmethod
    def synthetic(cls, wtype, E, N, K, generator=None, layout="gemv"):
        nb = K // 32
        blocks = torch.randint(0, 256, (E, N, nb, BLOCK_BYTES[wtype]), dtype=torch.uint8, device="cuda", generator=generator)
        if wtype == Q8_0:
            blocks[blocks == 0x80] = 0x81
        s = (torch.randn((E, N, nb), device="cuda", generator=generator) * 0.02).abs() / 7.0
        bits = s.to(torch.float16).view(torch.int16) & ~7
        blocks[:, :, :, 0:2] = bits.view(torch.uint8).view(E, N, nb, 2)
        return cls(wtype, blocks, layout=layout)

    @property
    def ptr(self):
        return self.buf.data_ptr()


def moe_ffn_q(gate, up, down, x, topk_ids, topk_w, act_scale_mode=SCALE_X86_REF, workspace=None, out=None):
    """x [T, H]; topk_ids int32 [T, k]; topk_w fp32 [T, k]; gate/up PackedExperts [E, I, H]; down [E, H, I] -> y fp32 [T, H]."""
    T, H = x.shape
    k = topk_ids.shape[1]
    E, I = gate.E, gate.N
    assert gate.K == H and up.N == I and down.N == H and down.K == I and topk_ids.dtype == torch.int32
    L = _lib.lib()
    if workspace is None:
        workspace = torch.empty(L.mllm_hip_moe_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device="cuda")
    y = out if out is not None else torch.empty((T, H), dtype=torch.float32, device="cuda")
    _lib.check(L.mllm_hip_moe_ffn_q(gate.wtype, gate.ptr, up.ptr, down.ptr, x.data_ptr(), _xdtype(x), topk_ids.data_ptr(),
                                    topk_w.data_ptr(), y.data_ptr(), T, H, I, E, k, act_scale_mode, workspace.data_ptr(),
                                    _stream()), "mllm_hip_moe_ffn_q")
    return y


def linear_q_gemm(w, x, bias=None, act_scale_mode=SCALE_X86_REF, workspace=None, out=None, short=False):
    """Q4_0/Q8_0 Linear for many rows on the matrix cores (fp16 operands with the block scales folded in); w in the "gemm"
    layout.  short=True: the entry point for short batches (K cut into ranges that run as separate workgroups)."""
    assert x.is_cuda and x.is_contiguous() and x.dim() == 2 and x.shape[1] == w.K and w.layout == "gemm"
    M = x.shape[0]
    L = _lib.lib()
    if workspace is None:
        size = L.mllm_hip_linear_q_gemm_short_workspace_bytes(M, w.N, w.K) if short else L.mllm_hip_linear_q_gemm_workspace_bytes(M, w.K)
        workspace = torch.empty(size, dtype=torch.uint8, device="cuda")
    y = out if out is not None else torch.empty((M, w.N), dtype=torch.float32, device="cuda")
    fn = L.mllm_hip_linear_q_gemm_short if short else L.mllm_hip_linear_q_gemm
    _lib.check(fn(w.wtype, w.ptr, x.data_ptr(), _xdtype(x), _p(bias), y.data_ptr(), M, w.N, w.K, act_scale_mode, workspace.data_ptr(),
                  _stream()), "mllm_hip_linear_q_gemm")
    return y


def moe_ffn_q_gemm(gate, up, down, x, topk_ids, topk_w, act_scale_mode=SCALE_X86_REF, workspace=None, out=None):
    """As moe_ffn_q on the matrix cores; gate/up/down PackedExperts in the "gemm" layout."""
    T, H = x.shape
    k = topk_ids.shape[1]
    E, I = gate.E, gate.N
    assert gate.K == H and up.N == I and down.N == H and down.K == I and topk_ids.dtype == torch.int32
    assert gate.layout == up.layout == down.layout == "gemm"
    L = _lib.lib()
    if workspace is None:
        workspace = torch.empty(L.mllm_hip_moe_gemm_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device="cuda")
    y = out if out is not None else torch.empty((T, H), dtype=torch.float32, device="cuda")
    _lib.check(L.mllm_hip_moe_ffn_q_gemm(gate.wtype, gate.ptr, up.ptr, down.ptr, x.data_ptr(), _xdtype(x),
                                         topk_ids.data_ptr(), topk_w.data_ptr(), y.data_ptr(), T, H, I, E, k, act_scale_mode,
                                         workspace.data_ptr(), _stream()), "mllm_hip_moe_ffn_q_gemm")
    return y


def moe_route(topk_ids, E):
    T, k = topk_ids.shape
    L = _lib.lib()
    ws = torch.empty(L.mllm_hip_moe_workspace_bytes(T, 32, 32, E, k), dtype=torch.uint8, device="cuda")
    counts = torch.empty(E, dtype=torch.int32, device="cuda")
    offsets = torch.empty(E + 1, dtype=torch.int32, device="cuda")
    sidx = torch.empty(T * k, dtype=torch.int32, device="cuda")
    _lib.check(L.mllm_hip_moe_route(topk_ids.data_ptr(), T, E, k, counts.data_ptr(), offsets.data_ptr(), sidx.data_ptr(),
                                    ws.data_ptr(), _stream()), "mllm_hip_moe_route")
    return counts, offsets, sidx


# ----------------------------------------------------------------------------- the operators around Linear in a layer
def rmsnorm(x, weight, eps, add_unit_offset=False, want_image=False, act_scale_mode=SCALE_X86_REF, out=None):
    """x [..., D] fp32 or bf16, weight fp32 [D].  want_image (rows <= 8): also returns the Q8_0 image of the result for
    linear_q_gemv_fused(..., image=True)."""
    assert x.is_cuda and x.is_contiguous() and weight.dtype == torch.float32 and weight.is_contiguous()
    D = x.shape[-1]
    rows = x.numel() // D
    y = out if out is not None else torch.empty_like(x)
    img = gemv_workspace(rows, D) if want_image else None
    _lib.check(_lib.lib().mllm_hip_rmsnorm(x.data_ptr(), _xdtype(x), weight.data_ptr(), y.data_ptr(), rows, D, eps,
                                           int(add_unit_offset), _p(img), act_scale_mode, _stream()), "mllm_hip_rmsnorm")
    return (y, img) if want_image else y


def _binary(fn, name, a, b, want_image, act_scale_mode):
    assert a.is_cuda and a.is_contiguous() and b.is_contiguous() and a.shape == b.shape and a.dtype == b.dtype
    D = a.shape[-1]
    rows = a.numel() // D
    y = torch.empty_like(a)
    img = gemv_workspace(rows, D) if want_image else None
    _lib.check(fn(a.data_ptr(), b.data_ptr(), y.data_ptr(), _xdtype(a), rows, D, _p(img), act_scale_mode, _stream()), name)
    return (y, img) if want_image else y


def add(a, b, want_image=False, act_scale_mode=SCALE_X86_REF):
    return _binary(_lib.lib().mllm_hip_add, "mllm_hip_add", a, b, want_image, act_scale_mode)


def mul(a, b, want_image=False, act_scale_mode=SCALE_X86_REF):
    return _binary(_lib.lib().mllm_hip_mul, "mllm_hip_mul", a, b, want_image, act_scale_mode)


def silu(x):
    assert x.is_cuda and x.is_contiguous()
    y = torch.empty_like(x)
    _lib.check(_lib.lib().mllm_hip_silu(x.data_ptr(), y.data_ptr(), _xdtype(x), x.numel(), _stream()), "mllm_hip_silu")
    return y


def silu_mul(gate, up, want_image=False, act_scale_mode=SCALE_X86_REF, out=None):
    """silu(gate) * up over [rows, D]; want_image as for rmsnorm."""
    assert gate.is_cuda and gate.is_contiguous() and up.is_contiguous() and gate.shape == up.shape and gate.dtype == up.dtype
    D = gate.shape[-1]
    rows = gate.numel() // D
    y = out if out is not None else torch.empty_like(gate)
    img = gemv_workspace(rows, D) if want_image else None
    _lib.check(_lib.lib().mllm_hip_silu_mul(gate.data_ptr(), up.data_ptr(), y.data_ptr(), _xdtype(gate), rows, D, _p(img),
                                            act_scale_mode, _stream()), "mllm_hip_silu_mul")
    return (y, img) if want_image else y


def mlp_gate_up(wg, wu, x, M=None, image=False, want_h=True, want_image=False, act_scale_mode=SCALE_X86_REF):
    """silu(x Wg^T) * (x Wu^T) for up to eight rows in one launch; `x` activations [M, H] or (image=True) their Q8_0 image.
    Returns h (fp32 [M, I]) and/or the Q8_0 image of h for the down projection."""
    assert wg.K == wu.K and wg.N == wu.N and wg.wtype == wu.wtype and x.is_cuda and x.is_contiguous()
    if not image:
        assert x.dim() == 2 and x.shape[1] == wg.K
        M = x.shape[0]
    assert M is not None and (want_h or want_image)
    h = torch.empty((M, wg.N), dtype=torch.float32, device="cuda") if want_h else None
    img = gemv_workspace(M, wg.N) if want_image else None
    _lib.check(_lib.lib().mllm_hip_mlp_gate_up_q(wg.wtype, wg.ptr, wu.ptr, x.data_ptr(), Q8_IMAGE if image else _xdtype(x), _p(h),
                                                 _p(img), M, wg.N, wg.K, act_scale_mode, _stream()), "mllm_hip_mlp_gate_up_q")
    if want_h and want_image:
        return h, img
    return h if want_h else img


def set_exp_mode(accurate):
    _lib.check(_lib.lib().mllm_hip_set_exp_mode(int(accurate)), "mllm_hip_set_exp_mode")


def softmax(x):
    assert x.is_cuda and x.is_contiguous() and x.dtype == torch.float32
    n = x.shape[-1]
    y = torch.empty_like(x)
    _lib.check(_lib.lib().mllm_hip_softmax(x.data_ptr(), y.data_ptr(), x.numel() // n, n, _stream()), "mllm_hip_softmax")
    return y


def topk(x, k, largest=True, sorted=True):
    assert x.is_cuda and x.is_contiguous() and x.dtype == torch.float32
    n = x.shape[-1]
    v = torch.empty(x.shape[:-1] + (k,), dtype=torch.float32, device="cuda")
    i = torch.empty(x.shape[:-1] + (k,), dtype=torch.int32, device="cuda")
    _lib.check(_lib.lib().mllm_hip_topk(x.data_ptr(), v.data_ptr(), i.data_ptr(), x.numel() // n, n, k, int(largest),
                                        int(sorted), _stream()), "mllm_hip_topk")
    return v, i


def moe_gate(x, gate_weight, k, norm_topk_prob=True, want_scores=False, scores=None):
    """x [M, H] fp32 or bf16, gate_weight fp32 [E, H] -> (ids int32 [M, k], weights fp32 [M, k][, scores fp32 [M, E]]).
    scores: a buffer fp32 [M, E] to use (with one -- want_scores allocates it -- the call takes the two-launch form)"""
    assert x.is_cuda and x.is_contiguous() and x.dim() == 2 and gate_weight.dtype == torch.float32 and gate_weight.is_contiguous()
    M, H = x.shape
    E = gate_weight.shape[0]
    ids = torch.empty((M, k), dtype=torch.int32, device="cuda")
    wt = torch.empty((M, k), dtype=torch.float32, device="cuda")
    sc = scores if scores is not None else (torch.empty((M, E), dtype=torch.float32, device="cuda") if want_scores else None)
    _lib.check(_lib.lib().mllm_hip_moe_gate(x.data_ptr(), _xdtype(x), gate_weight.data_ptr(), ids.data_ptr(), wt.data_ptr(),
                                            _p(sc), M, H, E, k, int(norm_topk_prob), _stream()), "mllm_hip_moe_gate")
    return (ids, wt, sc) if want_scores else (ids, wt)


# ----------------------------------------------------------------------------- K-quants (Q4_K / Q6_K weights, Q8_K activations)
Q4_K, Q6_K = 2, 3
KBLOCK_BYTES = {Q4_K: 144, Q6_K: 210}


def kq_quantize_weight_blocks(w, wtype, weight_scale_mode=SCALE_IEEE):
    """fp32 [N, K] on the GPU -> reference super-blocks uint8 [N, K/256, 144|210] (the offline K-quant quantizers' output)."""
    assert w.is_cuda and w.is_contiguous() and w.dtype == torch.float32 and w.dim() == 2 and w.shape[1] % 256 == 0
    N, K = w.shape
    out = torch.empty((N, K // 256, KBLOCK_BYTES[wtype]), dtype=torch.uint8, device="cuda")
    _lib.check(_lib.lib().mllm_hip_kq_quantize_weight_blocks(wtype, w.data_ptr(), out.data_ptr(), weight_scale_mode, N, K, _stream()),
               "mllm_hip_kq_quantize_weight_blocks")
    return out


class PackedKWeight:
    """Q4_K / Q6_K weight [N, K] repacked on the device.  blocks: uint8 [N, K/256, 144|210] (reference layout)."""

    def __init__(self, wtype, blocks, weight_scale_mode=SCALE_IEEE, layout="gemv"):
        assert blocks.dtype == torch.uint8 and blocks.dim() == 3 and blocks.shape[2] == KBLOCK_BYTES[wtype]
        assert layout in ("gemv", "gemm")
        self.wtype, self.N, self.K, self.layout = wtype, blocks.shape[0], blocks.shape[1] * 256, layout
        L = _lib.lib()
        size, pack = ((L.mllm_hip_kq_packed_bytes, L.mllm_hip_kq_prepack) if layout == "gemv"
                      else (L.mllm_hip_kq_gemm_packed_bytes, L.mllm_hip_kq_gemm_prepack))
        self.buf = torch.empty(size(wtype, self.N, self.K), dtype=torch.uint8, device="cuda")
        src = blocks.contiguous().cuda()
        _lib.check(pack(wtype, src.data_ptr(), weight_scale_mode, self.buf.data_ptr(), self.N, self.K, _stream()), "kq prepack (%s)" % layout)
        torch.cuda.current_stream().synchronize()  # src may be released

    @classmethod
    def synthetic(cls, wtype, N, K, gen, layout="gemv"):
        """random blocks made on the device (bench): every byte uniform, fp16 fields set to a small positive value"""
        bb = KBLOCK_BYTES[wtype]
        blocks = torch.randint(0, 256, (N, K // 256, bb), dtype=torch.uint8, device="cuda", generator=gen)
        for off in ((0, 2) if wtype == Q4_K else (208,)):
            blocks[:, :, off] = 0x00
            blocks[:, :, off + 1] = 0x14  # 0x1400 = 9.8e-4
        return cls(wtype, blocks, layout=layout)

    @property
    def ptr(self):
        return self.buf.data_ptr()

    def dequantize(self):
        w = torch.empty((self.N, self.K), dtype=torch.float32, device="cuda")
        _lib.check(_lib.lib().mllm_hip_kq_dequantize(self.wtype, self.ptr, w.data_ptr(), self.N, self.K, _stream()), "mllm_hip_kq_dequantize")
        return w


class PackedKExperts:
    """E Q4_K / Q6_K matrices [N, K] packed back to back for mllm_hip_moe_ffn_kq.  blocks: uint8 [E, N, K/256, 144|210]."""

    def __init__(self, wtype, blocks, weight_scale_mode=SCALE_IEEE):
        assert blocks.dtype == torch.uint8 and blocks.dim() == 4 and blocks.shape[3] == KBLOCK_BYTES[wtype]
        self.wtype, self.E, self.N, self.K = wtype, blocks.shape[0], blocks.shape[1], blocks.shape[2] * 256
        L = _lib.lib()
        self.stride = L.mllm_hip_kq_packed_bytes(wtype, self.N, self.K)
        self.buf = torch.empty(self.E * self.stride, dtype=torch.uint8, device="cuda")
        for e in range(self.E):
            src = blocks[e].contiguous().cuda()
            _lib.check(L.mllm_hip_kq_prepack(wtype, src.data_ptr(), weight_scale_mode, self.buf.data_ptr() + e * self.stride, self.N,
                                             self.K, _stream()), "kq prepack")
            torch.cuda.current_stream().synchronize()

    @classmethod
    def synthetic(cls, wtype, E, N, K, gen):
        bb = KBLOCK_BYTES[wtype]
        blocks = torch.randint(0, 256, (E, N, K // 256, bb), dtype=torch.uint8, device="cuda", generator=gen)
        for off in ((0, 2) if wtype == Q4_K else (208,)):
            blocks[..., off] = 0x00
            blocks[..., off + 1] = 0x14
        return cls(wtype, blocks)

    @property
    def ptr(self):
        return self.buf.data_ptr()


def moe_ffn_kq(gate, up, down, x, topk_ids, topk_w, workspace=None, out=None):
    """The MoE expert FFN with Q4_K / Q6_K experts (PackedKExperts): x [T, H], topk_ids int32 [T, k], topk_w fp32 [T, k].
    gate and up share a format; down may have the other one (the shipped recipe: Q4_K gate / up, Q6_K down)."""
    T, H = x.shape
    k = topk_ids.shape[1]
    E, I = gate.E, gate.N
    assert gate.K == H and up.N == I and down.N == H and down.K == I and topk_ids.dtype == torch.int32
    assert gate.wtype == up.wtype
    L = _lib.lib()
    if workspace is None:
        workspace = torch.empty(L.mllm_hip_moe_kq_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device="cuda")
    y = out if out is not None else torch.empty((T, H), dtype=torch.float32, device="cuda")
    if down.wtype == gate.wtype:
        _lib.check(L.mllm_hip_moe_ffn_kq(gate.wtype, gate.ptr, up.ptr, down.ptr, x.data_ptr(), _xdtype(x), topk_ids.data_ptr(),
                                         topk_w.data_ptr(), y.data_ptr(), T, H, I, E, k, workspace.data_ptr(), _stream()),
                   "mllm_hip_moe_ffn_kq")
    else:
        _lib.check(L.mllm_hip_moe_ffn_kq2(gate.wtype, down.wtype, gate.ptr, up.ptr, down.ptr, x.data_ptr(), _xdtype(x),
                                          topk_ids.data_ptr(), topk_w.data_ptr(), y.data_ptr(), T, H, I, E, k, workspace.data_ptr(),
                                          _stream()), "mllm_hip_moe_ffn_kq2")
    return y


def kq_workspace(M, K, N_total=0):
    """N_total (the sum of the N of a launch's parts) > 0: with room for the partial sums of K slices that meet in global memory"""
    L = _lib.lib()
    size = L.mllm_hip_kq_workspace_bytes_n(M, K, N_total) if N_total else L.mllm_hip_kq_workspace_bytes(M, K)
    return torch.empty(size, dtype=torch.uint8, device="cuda")


def linear_kq_gemm(w, x, bias=None, out=None, workspace=None, short=False):
    """many rows on the matrix cores; w: PackedKWeight(layout="gemm"); short=True: the entry point for short batches"""
    assert w.layout == "gemm" and x.is_cuda and x.is_contiguous() and x.dim() == 2 and x.shape[1] == w.K
    M = x.shape[0]
    L = _lib.lib()
    y = out if out is not None else torch.empty((M, w.N), dtype=torch.float32, device="cuda")
    if workspace is None:
        size = L.mllm_hip_linear_kq_gemm_short_workspace_bytes(M, w.N, w.K) if short else L.mllm_hip_linear_kq_gemm_workspace_bytes(M, w.K)
        workspace = torch.empty(size, dtype=torch.uint8, device="cuda")
    fn = L.mllm_hip_linear_kq_gemm_short if short else L.mllm_hip_linear_kq_gemm
    _lib.check(fn(w.wtype, w.ptr, x.data_ptr(), _xdtype(x), _p(bias), y.data_ptr(), M, w.N, w.K, workspace.data_ptr(), _stream()),
               "mllm_hip_linear_kq_gemm")
    return y


def linear_kq(w, x, bias=None, out=None, workspace=None):
    """workspace (kq_workspace): from three rows on, x is quantized once by a small kernel instead of in every workgroup;
    with room for partial sums (kq_workspace(M, K, N)), long Q4_K rows are cut into K slices with a workgroup each"""
    assert w.layout == "gemv" and x.is_cuda and x.is_contiguous() and x.dim() == 2 and x.shape[1] == w.K
    M = x.shape[0]
    y = out if out is not None else torch.empty((M, w.N), dtype=torch.float32, device="cuda")
    if workspace is not None and workspace.numel() > _lib.lib().mllm_hip_kq_workspace_bytes(M, w.K):
        return linear_kq_multi([w], x, [bias], [y], workspace=workspace)[0]  # (the entry point that is told the workspace's size)
    _lib.check(_lib.lib().mllm_hip_linear_kq(w.wtype, w.ptr, x.data_ptr(), _xdtype(x), _p(bias), y.data_ptr(), M, w.N, w.K,
                                             _p(workspace), _stream()), "mllm_hip_linear_kq")
    return y


def linear_kq_multi(ws, x, biases=None, outs=None, workspace=None):
    """Sibling projections (same x, same K) in one launch; ws: list of PackedKWeight."""
    assert 1 <= len(ws) <= 4 and x.is_cuda and x.is_contiguous() and x.dim() == 2
    M, K = x.shape
    if outs is None:
        outs = [torch.empty((M, w.N), dtype=torch.float32, device="cuda") for w in ws]
    parts = (_lib.GemvPart * len(ws))()
    for i, w in enumerate(ws):
        assert w.K == K and w.wtype == ws[0].wtype
        b = biases[i] if biases is not None else None
        parts[i] = _lib.GemvPart(w.ptr, b.data_ptr() if b is not None else None, outs[i].data_ptr(), w.N)
    if workspace is not None:
        _lib.check(_lib.lib().mllm_hip_linear_kq_multi_ws(ws[0].wtype, len(ws), parts, x.data_ptr(), _xdtype(x), M, K, workspace.data_ptr(),
                                                          workspace.numel(), _stream()), "mllm_hip_linear_kq_multi_ws")
        return outs
    _lib.check(_lib.lib().mllm_hip_linear_kq_multi(ws[0].wtype, len(ws), parts, x.data_ptr(), _xdtype(x), M, K, None, _stream()),
               "mllm_hip_linear_kq_multi")
    return outs


def quantize_q8_K(x):
    """x [M, K] -> (codes int8 [M, K], d fp32 [M, K/256], sums of 16 int16 [M, K/16])"""
    assert x.is_cuda and x.is_contiguous() and x.dim() == 2
    M, K = x.shape
    codes = torch.empty((M, K), dtype=torch.int8, device="cuda")
    d = torch.empty((M, K // 256), dtype=torch.float32, device="cuda")
    bs = torch.empty((M, K // 16), dtype=torch.int16, device="cuda")
    _lib.check(_lib.lib().mllm_hip_quantize_q8_K(x.data_ptr(), _xdtype(x), codes.data_ptr(), d.data_ptr(), bs.data_ptr(), M, K, _stream()),
               "mllm_hip_quantize_q8_K")
    return codes, d, bs


# ----------------------------------------------------------------------------- MatMul (activation x activation)
_MM_DTYPE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 3}


def matmul(a, b, transpose_a=False, transpose_b=False, out=None):
    """C[..., M, N] = op(a) @ op(b) for fp32 / bf16 / fp16 tensors of rank >= 2, the whole batch in one launch; b may be a
    single matrix shared by every batch entry.  mllm/backends/cpu/ops/MatMulOp.cpp:19-90."""
    assert a.dtype == b.dtype and a.dtype in _MM_DTYPE and a.is_contiguous() and b.is_contiguous()
    M, K = (a.shape[-1], a.shape[-2]) if transpose_a else (a.shape[-2], a.shape[-1])
    N, Kb = (b.shape[-2], b.shape[-1]) if transpose_b else (b.shape[-1], b.shape[-2])
    assert K == Kb
    batch = 1
    for d in a.shape[:-2]:
        batch *= d
    b_batch = 1
    for d in b.shape[:-2]:
        b_batch *= d
    assert b_batch in (1, batch)
    c = out if out is not None else torch.empty(tuple(a.shape[:-2]) + (M, N), dtype=a.dtype, device="cuda")
    _lib.check(_lib.lib().mllm_hip_matmul_batched(a.data_ptr(), b.data_ptr(), c.data_ptr(), _MM_DTYPE[a.dtype], batch, M, N, K,
                                                  M * K, N * K if b_batch == batch and batch > 1 else 0, M * N,
                                                  int(transpose_a), int(transpose_b), _stream()), "mllm_hip_matmul_batched")
    return c
