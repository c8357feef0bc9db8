"""GPU parity of the W8A8 path: per-token int8 activation quantization (bit-exact), int32 accumulators (bit-exact) and the
scaled bf16 output (the epilogue is the same three fp32 operations as the oracle's, so it is compared bit for bit; the
stated bar is rel-L2 <= 1e-3)."""
import numpy as np
import pytest
import torch

from mllm_amd import _lib, qlinear as ql, synth
from oracle import oracle as orc
from gpu_util import announce, bf16_dev, rel_l2, to_dev

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def test_per_token_quant_bit_exact_special_rows():
    rng = synth.rng_for(3, 1)
    a_bits, _, _ = synth.make_w8a8(rng, 40, 8, 512)
    x = synth.bf16_bits_to_fp32(a_bits)
    x[5] = 0                                                              # all-zero row -> absmax clamps to 1e-10
    x[6, :] = np.float32(0.25) * np.arange(512, dtype=np.float32)         # many exact ties after scaling
    x[7, 3] = 1e4                                                         # huge outlier
    announce("per-token quant special rows")
    for dev_x in (to_dev(x), bf16_dev(synth.fp32_to_bf16_bits(x))):
        xf = x if dev_x.dtype == torch.float32 else synth.bf16_bits_to_fp32(synth.fp32_to_bf16_bits(x))
        q, s = ql.per_token_quant_int8(dev_x)
        wq, wsc = orc.per_token_quant_int8(xf)
        assert np.array_equal(q.cpu().numpy(), wq)
        assert np.array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))


@pytest.mark.parametrize("M,K", [(2048, 2048), (7, 100), (3, 8), (5, 6144 + 24)])
def test_per_token_quant_bit_exact(M, K):
    rng = synth.rng_for(3, M + K)
    a_bits, _, _ = synth.make_w8a8(rng, M, 8, K)
    announce("per-token quant", M, K)
    q, s = ql.per_token_quant_int8(bf16_dev(a_bits))
    wq, wsc = orc.per_token_quant_int8(synth.bf16_bits_to_fp32(a_bits))
    assert np.array_equal(q.cpu().numpy(), wq)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))


# the shapes the reference's own int8 GEMM test uses (mllm-kernel/tests/test_int8_scaled_mm_cutlass.py:123-132)
REF_SHAPES = [(1, 64, 32), (1, 2048, 2048), (8, 128, 64), (16, 6144, 2048), (32, 2048, 2048), (93, 6144, 2048),
              (128, 2048, 6144)]


@pytest.mark.parametrize("M,N,K", REF_SHAPES + [(300, 200, 48), (257, 193, 80)])
@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4])
def test_gemm_bit_exact(M, N, K, tile):
    rng = synth.rng_for(3, M * 7 + N + K)
    xq = rng.integers(-127, 128, (M, K), dtype=np.int8)
    W = rng.integers(-127, 128, (N, K), dtype=np.int8)
    xs = ((rng.random(M) + 0.01) * 0.01).astype(np.float32)
    ws = ((rng.random(N) + 0.01) * 0.01).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.01).astype(np.float32)
    L = _lib.lib()
    try:
        assert L.mllm_hip_w8a8_set_tuning(tile) == 0
        announce("w8a8 gemm", M, N, K, "tile", tile)
        y, acc = ql.w8a8_gemm(to_dev(xq), to_dev(xs), to_dev(W), to_dev(ws), None, want_acc=True)
        yb = ql.w8a8_gemm(to_dev(xq), to_dev(xs), to_dev(W), to_dev(ws), to_dev(bias))
    finally:
        L.mllm_hip_w8a8_set_tuning(0)
    wacc, wy = orc.w8a8_gemm(xq, xs, W, ws, None)
    _, wyb = orc.w8a8_gemm(xq, xs, W, ws, bias)
    assert np.array_equal(acc.cpu().numpy(), wacc)
    assert np.array_equal(_bits(y), wy)
    assert np.array_equal(_bits(yb), wyb)
    assert rel_l2(synth.bf16_bits_to_fp32(_bits(y)), synth.bf16_bits_to_fp32(wy)) <= 1e-3


def _pack_reference(W):
    """The packed layout restated with numpy: block (nb, kb) of 32 rows x 32 bytes, lane l = (row l%32, half l/32)."""
    N, K = W.shape
    Np, Kp = (N + 31) // 32 * 32, (K + 127) // 128 * 128
    Wp = np.zeros((Np, Kp), dtype=np.int8)
    Wp[:N, :K] = W
    # [nb][row][kb][half][16] -> [nb][kb][half][row][16]
    return Wp.reshape(Np // 32, 32, Kp // 32, 2, 16).transpose(0, 2, 3, 1, 4).reshape(-1)


# shapes that reach each tile of the weights-from-global kernel: 128x384, 64x384, 128x128, 64x128, and ragged edges
PACKED_SHAPES = REF_SHAPES + [(300, 200, 48), (257, 193, 80), (1536, 6144, 256), (512, 9216, 128), (1024, 3072, 128),
                              (200, 800, 144)]


@pytest.mark.parametrize("M,N,K", PACKED_SHAPES)
def test_gemm_packed_bit_exact(M, N, K):
    rng = synth.rng_for(3, M * 11 + N + K)
    xq = rng.integers(-127, 128, (M, K), dtype=np.int8)
    W = rng.integers(-127, 128, (N, K), dtype=np.int8)
    xs = ((rng.random(M) + 0.01) * 0.01).astype(np.float32)
    ws = ((rng.random(N) + 0.01) * 0.01).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.01).astype(np.float32)
    announce("w8a8 packed gemm", M, N, K)
    Wp = ql.w8a8_prepack(to_dev(W))
    assert np.array_equal(Wp.cpu().numpy().view(np.int8), _pack_reference(W))
    y, acc = ql.w8a8_gemm_packed(to_dev(xq), to_dev(xs), Wp, N, to_dev(ws), None, want_acc=True)
    y1 = ql.w8a8_gemm_packed(to_dev(xq), to_dev(xs), Wp, N, to_dev(ws), None)      # bf16 only: the fast store path
    yb = ql.w8a8_gemm_packed(to_dev(xq), to_dev(xs), Wp, N, to_dev(ws), to_dev(bias))
    wacc, wy = orc.w8a8_gemm(xq, xs, W, ws, None)
    _, wyb = orc.w8a8_gemm(xq, xs, W, ws, bias)
    assert np.array_equal(acc.cpu().numpy(), wacc)
    assert np.array_equal(_bits(y), wy)
    assert np.array_equal(_bits(y1), wy)
    assert np.array_equal(_bits(yb), wyb)


@pytest.mark.parametrize("M,mfma_from", [(1, 5), (2, 5), (3, 5), (5, 33), (8, 33), (1, 1), (2, 2), (3, 2), (5, 5), (8, 5), (13, 5), (16, 5),
                                         (27, 5), (32, 5)])
def test_decode_gemv_packed_bit_exact(M, mfma_from):
    """up to 32 tokens take the GEMV kernels (a block row of the packed matrix per workgroup; dot instructions, or the matrix
    cores from `mfma_from` tokens): the oracle's bits, and the tile kernels' bits; ragged N and K (zero padding of the packed
    layout), rows long enough to pass through LDS in several runs, bias"""
    L = _lib.lib()
    assert L.mllm_hip_w8a8_set_decode_mfma_from(mfma_from) == 0
    try:
        _decode_gemv_cases(L, M)
    finally:
        assert L.mllm_hip_w8a8_set_decode_mfma_from(5) == 0
    assert L.mllm_hip_w8a8_set_decode_mfma_from(0) == -1 and L.mllm_hip_w8a8_set_decode_mfma_from(34) == -1


def _decode_gemv_cases(L, M):
    for N, K in ((9728, 2560), (2560, 9728), (77, 48), (200, 144), (33, 4096 + 16)):
        rng = synth.rng_for(3, 700 + M * 11 + N + K)
        xq = rng.integers(-127, 128, (M, K), dtype=np.int8)
        W = rng.integers(-127, 128, (N, K), dtype=np.int8)
        xs = ((rng.random(M) + 0.01) * 0.01).astype(np.float32)
        ws = ((rng.random(N) + 0.01) * 0.01).astype(np.float32)
        bias = (rng.standard_normal(N) * 0.01).astype(np.float32)
        announce("w8a8 decode gemv", M, N, K)
        Wp = ql.w8a8_prepack(to_dev(W))
        y, acc = ql.w8a8_gemm_packed(to_dev(xq), to_dev(xs), Wp, N, to_dev(ws), None, want_acc=True)
        yb = ql.w8a8_gemm_packed(to_dev(xq), to_dev(xs), Wp, N, to_dev(ws), to_dev(bias))
        wacc, wy = orc.w8a8_gemm(xq, xs, W, ws, None)
        _, wyb = orc.w8a8_gemm(xq, xs, W, ws, bias)
        assert np.array_equal(acc.cpu().numpy(), wacc)
        assert np.array_equal(_bits(y), wy) and np.array_equal(_bits(yb), wyb)
        assert L.mllm_hip_w8a8_set_decode(0) == 0
        try:
            yt = ql.w8a8_gemm_packed(to_dev(xq), to_dev(xs), Wp, N, to_dev(ws), to_dev(bias))
        finally:
            assert L.mllm_hip_w8a8_set_decode(1) == 0
        assert np.array_equal(_bits(yt), wyb)
    assert L.mllm_hip_w8a8_set_decode(2) == -1


def test_full_size_prefill():
    """A bf16 [2048,2048] with outliers, W int8 [6144,2048]: quantization bit-exact on every row; accumulators checked on a
    row sample against the oracle and on ALL rows through the column-sum identity
    sum_n acc[m][n] = sum_k xq[m][k] * (sum_n W[n][k])."""
    rng = synth.rng_for(3)
    M, N, K = 2048, 6144, 2048
    a_bits, W, ws = synth.make_w8a8(rng, M, N, K)
    announce("w8a8 full size")
    xd = bf16_dev(a_bits)
    Wd, wsd = to_dev(W), to_dev(ws)
    q, s = ql.per_token_quant_int8(xd)
    wq, wsc = orc.per_token_quant_int8(synth.bf16_bits_to_fp32(a_bits))
    assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(s.cpu().numpy(), wsc)
    y, acc = ql.w8a8_gemm(q, s, Wd, wsd, None, want_acc=True)
    acc = acc.cpu().numpy()
    colsum = W.astype(np.int64).sum(axis=0)
    assert np.array_equal(acc.astype(np.int64).sum(axis=1), wq.astype(np.int64) @ colsum)
    rows = np.sort(rng.choice(M, 48, replace=False))
    wacc, wy = orc.w8a8_gemm(wq[rows], wsc[rows], W, ws, None)
    assert np.array_equal(acc[rows], wacc)
    assert np.array_equal(_bits(y)[rows], wy)
    # the fused entry point (quantize + GEMM) gives the same bits
    y2 = ql.w8a8_linear(xd, Wd, wsd)
    assert torch.equal(y2.view(torch.int16), y.view(torch.int16))
    # and so does the prepacked-weight path, on every element
    Wp = ql.w8a8_prepack(Wd)
    y3, acc3 = ql.w8a8_gemm_packed(q, s, Wp, N, wsd, None, want_acc=True)
    assert np.array_equal(acc3.cpu().numpy(), acc)
    y4 = ql.w8a8_linear_packed(xd, Wp, N, wsd)
    assert torch.equal(y3.view(torch.int16), y.view(torch.int16))
    assert torch.equal(y4.view(torch.int16), y.view(torch.int16))


def test_argument_errors():
    L = _lib.lib()
    t = torch.zeros(64 * 64, dtype=torch.int8, device="cuda")
    f = torch.zeros(64, device="cuda")
    o = torch.zeros(64 * 64, dtype=torch.bfloat16, device="cuda")
    g = L.mllm_hip_w8a8_gemm
    assert g(t.data_ptr(), f.data_ptr(), t.data_ptr(), f.data_ptr(), None, o.data_ptr(), None, 64, 64, 40, None) == -2
    assert g(None, f.data_ptr(), t.data_ptr(), f.data_ptr(), None, o.data_ptr(), None, 64, 64, 64, None) == -1
    assert g(t.data_ptr(), f.data_ptr(), t.data_ptr(), f.data_ptr(), None, None, None, 64, 64, 64, None) == -1
    assert g(t.data_ptr() + 1, f.data_ptr(), t.data_ptr(), f.data_ptr(), None, o.data_ptr(), None, 8, 8, 64, None) == -3
    assert L.mllm_hip_per_token_quant_int8(None, 1, t.data_ptr(), f.data_ptr(), 4, 64, None) == -1
    assert L.mllm_hip_w8a8_set_tuning(9) == -1
    assert L.mllm_hip_w8a8_prepack(t.data_ptr(), 64, 40, o.data_ptr(), None) == -2
    assert L.mllm_hip_w8a8_prepack(None, 64, 64, o.data_ptr(), None) == -1
    assert L.mllm_hip_w8a8_packed_bytes(33, 130) == 64 * 256
