"""GPU parity of the any-M block-quantized Linear and of the MoE expert FFN against the CPU oracle.

Bars: routing counts exact; first-GEMM activation codes are the bit-exact Q8_0 kernel already covered elsewhere; fp32
outputs rel-L2 <= 1e-3 (summation order differs; the re-quantization of silu(g)*u in front of the down projection can
flip a code by one where the two sides' fp32 values differ in the last bit)."""
import numpy as np
import pytest
import torch

from mllm_amd import _lib, qlinear as ql, synth
from oracle import oracle as orc
from gpu_util import announce, bf16_dev, rel_l2, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M,N,K", [(1, 32, 32), (9, 100, 96), (16, 768, 2048 + 64), (17, 64, 2048), (33, 100, 96), (129, 64, 2048),
                                   (300, 768, 2048 + 64), (512, 2048, 768)])
def test_linear_q_any_m(wtype, M, N, K):
    rng = synth.rng_for(4, M + N + K + wtype)
    W = synth.make_weight(rng, wtype, N, K)
    w = ql.PackedQWeight(wtype, torch.from_numpy(W))
    x = synth.make_x_fp32(rng, M, K)
    bias = rng.standard_normal(N).astype(np.float32)
    announce("linear_q", wtype, M, N, K)
    for mode, omode in ((ql.SCALE_X86_REF, orc.SCALE_X86_REF), (ql.SCALE_IEEE, orc.SCALE_IEEE)):
        y = ql.linear_q(w, to_dev(x), None, mode).cpu().numpy()
        want = orc.linear_q(x, W, wtype, None, omode)
        assert rel_l2(y, want) < 2e-6, (mode, rel_l2(y, want))
    yb = ql.linear_q(w, to_dev(x), to_dev(bias)).cpu().numpy()
    assert rel_l2(yb, orc.linear_q(x, W, wtype, bias)) < 2e-6
    if M <= 8:  # agrees with the decode GEMV
        yg = ql.linear_q_gemv(w, to_dev(x)).cpu().numpy()
        assert rel_l2(yg, orc.linear_q(x, W, wtype)) < 2e-6


GEMM_TOL = 5e-4  # fp16 operands: two roundings of relative error <= 2^-12 each; measured about 2e-4


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M,N,K", [(1, 32, 32), (33, 100, 96), (129, 64, 2048), (300, 768, 2048 + 64), (512, 2048, 768),
                                    (70, 260, 160)])
def test_linear_q_gemm_any_m(wtype, M, N, K):
    rng = synth.rng_for(4, 5 * M + N + K + wtype)
    W = synth.make_weight(rng, wtype, N, K)
    w = ql.PackedQWeight(wtype, torch.from_numpy(W), layout="gemm")
    x = synth.make_x_fp32(rng, M, K)
    bias = rng.standard_normal(N).astype(np.float32)
    announce("linear_q_gemm", wtype, M, N, K)
    for mode, omode in ((ql.SCALE_X86_REF, orc.SCALE_X86_REF), (ql.SCALE_IEEE, orc.SCALE_IEEE)):
        y = ql.linear_q_gemm(w, to_dev(x), None, mode).cpu().numpy()
        want = orc.linear_q(x, W, wtype, None, omode)
        assert rel_l2(y, want) < GEMM_TOL, (mode, rel_l2(y, want))
    yb = ql.linear_q_gemm(w, to_dev(x), to_dev(bias)).cpu().numpy()
    assert rel_l2(yb, orc.linear_q(x, W, wtype, bias)) < GEMM_TOL
    # against the block-dot kernel on the same inputs, and bf16 activations
    wv = ql.PackedQWeight(wtype, torch.from_numpy(W))
    assert rel_l2(y, ql.linear_q(wv, to_dev(x), None, ql.SCALE_IEEE).cpu().numpy()) < GEMM_TOL
    xb = synth.fp32_to_bf16_bits(x)
    y16 = ql.linear_q_gemm(w, bf16_dev(xb)).cpu().numpy()
    assert rel_l2(y16, orc.linear_q(synth.bf16_bits_to_fp32(xb), W, wtype)) < GEMM_TOL
    # the entry point for short batches (K cut into ranges, partial results added in range order): same operands, the fp32
    # sum over K grouped differently; deterministic
    ys = ql.linear_q_gemm(w, to_dev(x), to_dev(bias), short=True)
    assert rel_l2(ys.cpu().numpy(), yb) < 2e-6
    assert torch.equal(ys, ql.linear_q_gemm(w, to_dev(x), to_dev(bias), short=True))


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M,N,K", [(16, 9728, 2560), (128, 2560, 9728), (200, 1024, 640), (256, 6144, 2560), (40, 132, 4096 + 128)])
def test_linear_q_gemm_short_batches(wtype, M, N, K):
    """short prompts: K ranges as separate workgroups + reduction, against the oracle and the unsplit call"""
    rng = synth.rng_for(4, 600 + M + N % 97 + wtype)
    W = synth.make_weight(rng, wtype, N, K)
    w = ql.PackedQWeight(wtype, torch.from_numpy(W), layout="gemm")
    x = synth.make_x_fp32(rng, M, K)
    bias = rng.standard_normal(N).astype(np.float32)
    announce("linear_q_gemm short", wtype, M, N, K)
    assert _lib.lib().mllm_hip_linear_q_gemm_short_workspace_bytes(M, N, K) > _lib.lib().mllm_hip_linear_q_gemm_workspace_bytes(M, K)
    ys = ql.linear_q_gemm(w, to_dev(x), to_dev(bias), short=True).cpu().numpy()
    rows = rng.integers(0, M, 8)
    want = orc.linear_q(x[rows], W, wtype, bias)
    assert rel_l2(ys[rows], want) < GEMM_TOL
    assert rel_l2(ys, ql.linear_q_gemm(w, to_dev(x), to_dev(bias)).cpu().numpy()) < 2e-6


def test_linear_q_gemm_exact_when_operands_fit_fp16():
    """Weights and activations chosen so that dW*qW and dX*qX are exactly representable in fp16 and every partial sum in
    fp32: then the matrix-core path must equal the reference arithmetic bit for bit (a wrong nibble order, scale pairing,
    row or column mapping cannot hide behind a tolerance)."""
    rng = synth.rng_for(4, 99)
    M, N, K = 150, 200, 256
    for wtype in (0, 1):
        W = synth.make_weight(rng, wtype, N, K)
        Wv = W.reshape(N, K // 32, -1)
        Wv[:, :, 0:2] = np.frombuffer(np.float16(2.0 ** rng.integers(-4, -2, (N, K // 32))).tobytes(), dtype=np.uint8).reshape(N, K // 32, 2)
        # activations: integers in [-127, 127] with one +-127 per block, so that d = 1 and the codes are the values
        x = rng.integers(-127, 128, (M, K)).astype(np.float32)
        x[:, ::32] = 127.0
        w = ql.PackedQWeight(wtype, torch.from_numpy(W), layout="gemm")
        announce("linear_q_gemm exact", wtype)
        y = ql.linear_q_gemm(w, to_dev(x), None, ql.SCALE_IEEE).cpu().numpy()
        want = orc.linear_q(x, W, wtype, None, orc.SCALE_IEEE)
        assert np.array_equal(y, want)
        assert np.array_equal(ql.linear_q_gemm(w, to_dev(x), None, ql.SCALE_IEEE, short=True).cpu().numpy(), want)


@pytest.mark.parametrize("wtype", [0, 1])
def test_gemm_layout_reads_x86_written_scales(wtype):
    """A weight file written by the x86 quantizer holds each scale pattern as a half-precision NUMBER.  Both device
    layouts must decode it the same way: same weights through the decode layout (dequantize probe, pinned bit-exactly
    elsewhere) and through the matrix-core layout."""
    rng = synth.rng_for(4, 77 + wtype)
    M, N, K = 40, 96, 256
    W = synth.make_weight(rng, wtype, N, K)
    W[:, :, 0] |= 0x05  # off the grid where both readings agree
    b = W[:, :, 0:2].copy().view(np.uint16)[:, :, 0]
    Wx = W.copy()
    Wx[:, :, 0:2] = b.astype(np.float32).astype(np.float16).view(np.uint16).reshape(N, -1, 1).view(np.uint8)
    x = synth.make_x_fp32(rng, M, K)
    announce("gemm layout x86 scales", wtype)
    wg = ql.PackedQWeight(wtype, torch.from_numpy(Wx), ql.SCALE_X86_REF, layout="gemm")
    y = ql.linear_q_gemm(wg, to_dev(x), None, ql.SCALE_X86_REF).cpu().numpy()
    want = orc.linear_q(x, W, wtype, None, orc.SCALE_X86_REF)  # the oracle applies the x86 reading to the raw patterns
    assert rel_l2(y, want) < GEMM_TOL, rel_l2(y, want)
    wv = ql.PackedQWeight(wtype, torch.from_numpy(Wx), ql.SCALE_X86_REF)
    yv = ql.linear_q(wv, to_dev(x), None, ql.SCALE_X86_REF).cpu().numpy()
    assert rel_l2(yv, want) < 2e-6


def test_route_counts_and_order():
    rng = synth.rng_for(4, 1)
    T, E, k = 512, 128, 8
    ids, _ = synth.make_moe_routing(rng, T, E, k)
    announce("moe route")
    counts, offsets, sidx = ql.moe_route(to_dev(ids), E)
    counts, offsets, sidx = counts.cpu().numpy(), offsets.cpu().numpy(), sidx.cpu().numpy()
    want = np.bincount(ids.reshape(-1), minlength=E)
    assert np.array_equal(counts, want) and counts.sum() == T * k
    assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(want)]))
    assert np.array_equal(np.sort(sidx), np.arange(T * k))             # a permutation of all entries
    flat = ids.reshape(-1)
    assert (np.diff(flat[sidx]) >= 0).all()                              # grouped by ascending expert


def _moe_case(rng, T, H, I, E, k, wtype=0):
    Wg, Wu, Wd = synth.make_moe_weights(rng, E, H, I, wtype)
    ids, w = synth.make_moe_routing(rng, T, E, k)
    g = ql.PackedExperts(wtype, torch.from_numpy(Wg))
    u = ql.PackedExperts(wtype, torch.from_numpy(Wu))
    d = ql.PackedExperts(wtype, torch.from_numpy(Wd))
    return Wg, Wu, Wd, ids, w, g, u, d


@pytest.mark.parametrize("T,H,I,E,k,wtype", [(16, 64, 32, 4, 2, 0), (40, 256, 96, 8, 3, 0), (200, 128, 64, 3, 2, 1),
                                              (1, 64, 64, 4, 4, 0)])
def test_moe_small(T, H, I, E, k, wtype):
    rng = synth.rng_for(4, T + H + I + E)
    Wg, Wu, Wd, ids, w, g, u, d = _moe_case(rng, T, H, I, E, k, wtype)
    x = synth.make_x_fp32(rng, T, H)
    announce("moe small", T, H, I, E, k, wtype)
    y = ql.moe_ffn_q(g, u, d, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
    want = orc.moe_ffn(x, ids, w, Wg, Wu, Wd, wtype)
    assert rel_l2(y, want) < TOL, rel_l2(y, want)
    # permuting the tokens permutes the outputs (row order inside an expert is irrelevant)
    perm = rng.permutation(T)
    y2 = ql.moe_ffn_q(g, u, d, to_dev(x[perm]), to_dev(ids[perm]), to_dev(w[perm])).cpu().numpy()
    assert np.array_equal(y2, y[perm])


@pytest.mark.parametrize("T,H,I,E,k,wtype", [(1, 2048, 768, 128, 8, 0), (8, 2048, 768, 128, 8, 0), (3, 256, 96, 8, 3, 1), (5, 2048, 768, 16, 8, 1),
                                              (2, 64, 32, 4, 4, 0), (7, 128, 1024, 6, 2, 0), (8, 4096, 32, 5, 1, 0),
                                              (20, 2048, 768, 128, 8, 0), (12, 256, 96, 64, 4, 1), (48, 512, 64, 128, 8, 0)])
def test_moe_decode_path(T, H, I, E, k, wtype):
    """few tokens under the default rule: up to eight tokens, or up to one pair per expert, every (token, expert) pair is a GEMV
    row (two launches, Qwen3-30B-A3B dimensions included); the larger cases here run as eight-row tiles;
    fp32 block arithmetic as the CPU path, so close to the oracle; slots with an expert id outside [0, E) add nothing;
    permuting tokens permutes outputs bit for bit; bf16 activations"""
    rng = synth.rng_for(4, 5000 + T + H + I + E)
    Wg, Wu, Wd, ids, w, g, u, d = _moe_case(rng, T, H, I, E, k, wtype)
    x = synth.make_x_fp32(rng, T, H)
    announce("moe decode", T, H, I, E, k, wtype)
    y = ql.moe_ffn_q(g, u, d, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
    want = orc.moe_ffn(x, ids, w, Wg, Wu, Wd, wtype)
    # fp32 summation-order noise (1e-7) in front of the Q8_0 re-quantization of h flips a code now and then: about 5e-5
    assert rel_l2(y, want) < 2e-4, rel_l2(y, want)
    perm = rng.permutation(T)
    y2 = ql.moe_ffn_q(g, u, d, to_dev(x[perm]), to_dev(ids[perm]), to_dev(w[perm])).cpu().numpy()
    assert np.array_equal(y2, y[perm])
    bad = ids.copy()
    bad[0, 0] = E + 3
    if k > 1:
        bad[T - 1, k - 1] = -1
    y3 = ql.moe_ffn_q(g, u, d, to_dev(x), to_dev(bad), to_dev(w)).cpu().numpy()
    assert rel_l2(y3, orc.moe_ffn(x, bad, w, Wg, Wu, Wd, wtype)) < 2e-4
    bits, xb = synth.make_x_bf16(rng, T, H)
    from gpu_util import bf16_dev
    y4 = ql.moe_ffn_q(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
    assert rel_l2(y4, orc.moe_ffn(xb, ids, w, Wg, Wu, Wd, wtype)) < 2e-4


@pytest.mark.parametrize("T,H,I,E,k,wtype", [(16, 64, 32, 4, 2, 0), (40, 256, 96, 8, 3, 0), (200, 128, 64, 3, 2, 1),
                                              (1, 64, 64, 4, 4, 0), (300, 192, 160, 2, 2, 0), (70, 96, 224, 5, 3, 1)])
def test_moe_gemm_small(T, H, I, E, k, wtype):
    """Both forms of the grouped FFN on gemm-packed experts.  Form 0 keeps the reference's block arithmetic (exact integer
    block sums, exact scale products, one fp32 FMA per block): as close to the oracle as the decode kernels (2e-4 leaves
    room for the odd Q8_0 code of h that flips where fp32 sums differ in the last bit).  Form 1 folds the scales into fp16
    operands (1e-3).  Odd block counts (H = 96, I = 224, 160: 3, 7 and 5 blocks) exercise the half-filled last record;
    slots with an expert id outside [0, E) add nothing."""
    rng = synth.rng_for(4, 3 * T + H + I + E)
    Wg, Wu, Wd = synth.make_moe_weights(rng, E, H, I, wtype)
    ids, w = synth.make_moe_routing(rng, T, E, k)
    if T > 1:
        ids[0, 0] = E + 2
        ids[T - 1, k - 1] = -1
    g, u, d = (ql.PackedExperts(wtype, torch.from_numpy(m), layout="gemm") for m in (Wg, Wu, Wd))
    x = synth.make_x_fp32(rng, T, H)
    want = orc.moe_ffn(x, ids, w, Wg, Wu, Wd, wtype)
    L = _lib.lib()
    try:
        for form, tol in ((0, 2e-4), (1, TOL)):
            announce("moe gemm small", T, H, I, E, k, wtype, "form", form)
            assert L.mllm_hip_moe_gemm_set_path(form) == 0
            y = ql.moe_ffn_q_gemm(g, u, d, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
            assert rel_l2(y, want) < tol, (form, rel_l2(y, want))
            perm = rng.permutation(T)
            y2 = ql.moe_ffn_q_gemm(g, u, d, to_dev(x[perm]), to_dev(ids[perm]), to_dev(w[perm])).cpu().numpy()
            assert np.array_equal(y2, y[perm])
            if form == 0:  # tiles of at most sixteen rows in their own form or padded to 32 rows: the same bits
                assert L.mllm_hip_moe_gemm_set_path(2) == 0
                y32 = ql.moe_ffn_q_gemm(g, u, d, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
                assert np.array_equal(y32, y)
    finally:
        L.mllm_hip_moe_gemm_set_path(0)
    assert L.mllm_hip_moe_gemm_set_path(3) == -1


def test_moe_gemm_exact_form_is_the_block_arithmetic():
    """Form 0 against the block-dot kernels of mllm_hip_moe_ffn_q on the same inputs: both compute
    sum_b fp32(dW * dX) * float(int32 block sum) with exact block sums, so they differ by fp32 summation order only; and a
    case built from integers (unit scales, small codes) in which every sum is exact must come out bit for bit."""
    rng = synth.rng_for(4, 7100)
    T, H, I, E, k = 96, 256, 128, 6, 2
    Wg, Wu, Wd = synth.make_moe_weights(rng, E, H, I, 0)
    ids, w = synth.make_moe_routing(rng, T, E, k)
    x = synth.make_x_fp32(rng, T, H)
    gg, ug, dg = (ql.PackedExperts(0, torch.from_numpy(m), layout="gemm") for m in (Wg, Wu, Wd))
    gv, uv, dv = (ql.PackedExperts(0, torch.from_numpy(m)) for m in (Wg, Wu, Wd))
    announce("moe gemm exact form vs block-dot tiles")
    L = _lib.lib()
    try:
        assert L.mllm_hip_moe_set_tuning(1, 1) == 0  # the grouped block-dot tiles
        yv = ql.moe_ffn_q(gv, uv, dv, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
    finally:
        L.mllm_hip_moe_set_tuning(0, 0)
    yg = ql.moe_ffn_q_gemm(gg, ug, dg, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
    assert rel_l2(yg, yv) < 1e-4, rel_l2(yg, yv)
    assert rel_l2(yg, orc.moe_ffn(x, ids, w, Wg, Wu, Wd, 0)) < 2e-4


@pytest.mark.parametrize("T,wtype", [(6, 0), (24, 0), (40, 1), (100, 0)])
def test_moe_pair_row_and_tile_kernels_agree(T, wtype):
    """the per-pair kernels, the eight-row tiles and the grouped 64-row tiles follow the same block arithmetic: forced one way
    or the other by the tuning override they agree to fp32 summation order (plus the odd flipped Q8_0 code of h), and all
    match the oracle; slots with an expert id outside [0, E) add nothing on any of them"""
    L = _lib.lib()
    H, I, E, k = 512, 128, 32, 4
    rng = synth.rng_for(4, 5300 + T)
    Wg, Wu, Wd, ids, w, g, u, d = _moe_case(rng, T, H, I, E, k, wtype)
    ids[0, 0] = E + 3
    ids[T - 1, k - 1] = -1
    x = synth.make_x_fp32(rng, T, H)
    announce("moe pairs vs rows vs tiles", T, wtype)
    ys = {}
    try:
        for name, (pt, rt) in {"pairs": (4096, 1), "rows": (1, 65536), "tiles": (1, 1)}.items():
            assert L.mllm_hip_moe_set_tuning(pt, rt) == 0
            ys[name] = ql.moe_ffn_q(g, u, d, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
    finally:
        L.mllm_hip_moe_set_tuning(0, 0)
    want = orc.moe_ffn(x, ids, w, Wg, Wu, Wd, wtype)
    for name, y in ys.items():
        assert rel_l2(y, want) < 2e-4, (name, rel_l2(y, want))
    assert rel_l2(ys["pairs"], ys["tiles"]) < 2e-4 and rel_l2(ys["rows"], ys["tiles"]) < 2e-4
    assert L.mllm_hip_moe_set_tuning(-1, 0) == -1


@pytest.mark.parametrize("T,H,I,E,k,wtype", [(64, 2048, 768, 128, 8, 0), (100, 2048, 768, 128, 8, 1), (9, 64, 32, 2, 2, 0),
                                              (33, 256, 1024, 7, 3, 1), (150, 4096 + 32, 96, 128, 8, 0)])
def test_moe_row_tiles(T, H, I, E, k, wtype):
    """a few pairs per expert (Qwen3-30B-A3B dimensions at 64 and 100 tokens; one expert with many tiles; ragged last tiles): the
    pairs sorted by expert, eight rows per workgroup; permuting tokens permutes outputs bit for bit; bf16 activations"""
    rng = synth.rng_for(4, 5600 + T + H + I + E)
    Wg, Wu, Wd, ids, w, g, u, d = _moe_case(rng, T, H, I, E, k, wtype)
    x = synth.make_x_fp32(rng, T, H)
    announce("moe row tiles", T, H, I, E, k, wtype)
    L = _lib.lib()
    try:
        assert L.mllm_hip_moe_set_tuning(1, 65536) == 0
        y = ql.moe_ffn_q(g, u, d, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
        perm = rng.permutation(T)
        y2 = ql.moe_ffn_q(g, u, d, to_dev(x[perm]), to_dev(ids[perm]), to_dev(w[perm])).cpu().numpy()
        bits, xb = synth.make_x_bf16(rng, T, H)
        y4 = ql.moe_ffn_q(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
    finally:
        L.mllm_hip_moe_set_tuning(0, 0)
    assert rel_l2(y, orc.moe_ffn(x, ids, w, Wg, Wu, Wd, wtype)) < 2e-4
    assert np.array_equal(y2, y[perm])
    assert rel_l2(y4, orc.moe_ffn(xb, ids, w, Wg, Wu, Wd, wtype)) < 2e-4


def test_moe_gemm_full_size():
    """The full-size case on the matrix-core path."""
    rng = synth.rng_for(4)
    T, H, I, E, k = 512, 2048, 768, 128, 8
    Wg, Wu, Wd = synth.make_moe_weights(rng, E, H, I, 0)
    ids, w = synth.make_moe_routing(rng, T, E, k)
    g, u, d = (ql.PackedExperts(0, torch.from_numpy(m), layout="gemm") for m in (Wg, Wu, Wd))
    bits, xf = synth.make_x_bf16(rng, T, H)
    announce("moe gemm full size")
    y = ql.moe_ffn_q_gemm(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
    want = orc.moe_ffn(xf, ids, w, Wg, Wu, Wd, 0)
    r = rel_l2(y, want)
    assert r < 2e-4, r  # the exact form: the reference's block arithmetic
    y2 = ql.moe_ffn_q_gemm(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
    assert np.array_equal(y, y2)
    try:
        assert _lib.lib().mllm_hip_moe_gemm_set_path(2) == 0  # every tile padded to 32 rows: the same bits
        y32 = ql.moe_ffn_q_gemm(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
        assert np.array_equal(y, y32)
        assert _lib.lib().mllm_hip_moe_gemm_set_path(1) == 0
        y3 = ql.moe_ffn_q_gemm(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
    finally:
        _lib.lib().mllm_hip_moe_gemm_set_path(0)
    assert rel_l2(y3, want) < TOL


def test_moe_full_size():
    """512 tokens, hidden 2048, 128 experts, top-8 (Zipf 1.1), expert intermediate 768, Q4_0, bf16 activations."""
    rng = synth.rng_for(4)
    T, H, I, E, k = 512, 2048, 768, 128, 8
    Wg, Wu, Wd, ids, w, g, u, d = _moe_case(rng, T, H, I, E, k)
    bits, xf = synth.make_x_bf16(rng, T, H)
    announce("moe full size")
    y = ql.moe_ffn_q(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
    want = orc.moe_ffn(xf, ids, w, Wg, Wu, Wd, 0)
    r = rel_l2(y, want)
    assert r < TOL, r
    # two runs give identical bits (no order-dependent accumulation)
    y2 = ql.moe_ffn_q(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
    assert np.array_equal(y, y2)


def test_moe_argument_errors():
    L = _lib.lib()
    t = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p = t.data_ptr()
    f = L.mllm_hip_moe_ffn_q
    assert f(0, p, p, p, p, 0, p, p, p, 4, 48, 32, 2, 1, 1, p, None) == -2     # H % 32
    assert f(0, p, p, p, p, 0, p, p, p, 4, 64, 40, 2, 1, 1, p, None) == -2     # I % 32
    assert f(0, None, p, p, p, 0, p, p, p, 4, 64, 32, 2, 1, 1, p, None) == -1
    assert f(3, p, p, p, p, 0, p, p, p, 4, 64, 32, 2, 1, 1, p, None) == -1
    assert L.mllm_hip_moe_workspace_bytes(4, 48, 32, 2, 1) == 0
    assert L.mllm_hip_linear_q_workspace_bytes(4, 48) == 0
