"""GPU parity of the Q4_0 / Q8_0 decode GEMV against the CPU oracle and the committed golden vectors.

Bars: activation codes, scale patterns, dequantized weights and int32 block sums bit-exact; fp32 outputs rel-L2 <= 1e-3
(the kernel sums the per-block terms in a different order than the CPU's 8-lane accumulators).
"""
import os

import ctypes as C

import numpy as np
import pytest
import torch

from mllm_amd import _lib, qlinear as ql, synth
from oracle import oracle as orc
from gpu_util import announce, bf16_dev, rel_l2, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3  # rel-L2, the bar of the fp32 outputs


def _mode(m):
    return ql.SCALE_X86_REF if m == orc.SCALE_X86_REF else ql.SCALE_IEEE


def test_init_and_version():
    L = _lib.lib()
    assert b"gfx950" in L.mllm_hip_version()
    _lib.check(L.mllm_hip_init(0), "mllm_hip_init")
    assert L.mllm_hip_init(99) == -4


@pytest.mark.parametrize("wname,wtype", [("q4_0", 0), ("q8_0", 1)])
def test_golden_gemv(golden_dir, wname, wtype):
    g = np.load(os.path.join(golden_dir, "gemv_kat.npz"))
    announce("golden gemv", wname)
    w = ql.PackedQWeight(wtype, torch.from_numpy(g[f"{wname}_W"]))
    bias = to_dev(g[f"{wname}_bias"])
    for M in (1, 3, 4, 8):
        x = to_dev(g[f"{wname}_x{M}"])
        y = ql.linear_q_gemv(w, x, None, ql.SCALE_X86_REF).cpu().numpy()
        yb = ql.linear_q_gemv(w, x, bias, ql.SCALE_X86_REF).cpu().numpy()
        assert rel_l2(y, g[f"{wname}_y{M}"]) < 1e-5, M
        assert rel_l2(yb, g[f"{wname}_yb{M}"]) < 1e-5, M


def test_golden_actquant_bit_exact(golden_dir):
    g = np.load(os.path.join(golden_dir, "q8_0_actquant.npz"))
    announce("golden actquant")
    codes, d = ql.quantize_q8_0(to_dev(g["x"]))
    assert np.array_equal(codes.cpu().numpy(), g["qs"])
    d_bits = d.cpu().numpy().view(np.uint16)
    eff = orc.fp16_bits_to_fp32(orc.x86_scale_bits(d_bits))
    assert np.array_equal(eff.view(np.uint32), g["d_eff"].view(np.uint32))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_actquant_bit_exact_vs_oracle(dtype):
    rng = synth.rng_for(1, 11)
    M, K = 8, 9728
    if dtype == "bf16":
        bits, xf = synth.make_x_bf16(rng, M, K)
        xd = bf16_dev(bits)
    else:
        xf = (synth.make_x_fp32(rng, M, K) * rng.uniform(0.001, 50, (M, 1))).astype(np.float32)
        xf[2, 96:128] = 0
        xd = to_dev(xf)
    announce("actquant", dtype, M, K)
    codes, d = ql.quantize_q8_0(xd)
    qs, db = orc.quantize_rows_q8_0(xf)
    assert np.array_equal(codes.cpu().numpy(), qs)
    assert np.array_equal(d.cpu().numpy().view(np.uint16), db)


@pytest.mark.parametrize("wtype", [0, 1])
def test_dequant_and_block_isums_bit_exact(wtype, golden_dir):
    rng = synth.rng_for(1, 12)
    N, K, M = 96, 640, 5
    W = synth.make_weight(rng, wtype, N, K)
    W[:, :, 0] |= 0x05  # scales off the snapped grid: the two decodings of the weight scale now differ
    announce("dequant/isums", wtype)
    for mode in (orc.SCALE_IEEE, orc.SCALE_X86_REF):
        # x86 mode: the file holds the pattern as a half-precision number -> encode it that way for prepack
        Wd = W.copy()
        if mode == orc.SCALE_X86_REF:
            b = W[:, :, 0:2].copy().view(np.uint16)[:, :, 0]
            enc = b.astype(np.float32).astype(np.float16).view(np.uint16)  # half(float(pattern))
            Wd[:, :, 0:2] = enc.reshape(N, -1, 1).view(np.uint8)
        w = ql.PackedQWeight(wtype, torch.from_numpy(Wd), _mode(mode))
        want = orc.dequantize(W, wtype, mode)
        assert np.array_equal(w.dequantize().cpu().numpy().view(np.uint32), want.view(np.uint32)), mode
    g = np.load(os.path.join(golden_dir, "dequant_kat.npz"))
    wg = ql.PackedQWeight(wtype, torch.from_numpy(g["W4" if wtype == 0 else "W8"]))
    assert np.array_equal(wg.dequantize().cpu().numpy(), g["y4" if wtype == 0 else "y8"])
    x = synth.make_x_fp32(rng, M, K)
    qs, _ = orc.quantize_rows_q8_0(x)
    w = ql.PackedQWeight(wtype, torch.from_numpy(W))
    got = w.block_isums(to_dev(qs)).cpu().numpy()
    assert np.array_equal(got, orc.block_isums(W, wtype, qs))


SHAPES = [("c1", 6144, 2048)] + [(k, n, kk) for k, (n, kk) in synth.QWEN3_4B_LAYER.items() if k != "v_proj"]


@pytest.mark.parametrize("name,N,K", SHAPES)
@pytest.mark.parametrize("wtype", [0, 1])
def test_gemv_full_shapes(name, N, K, wtype):
    rng = synth.rng_for(1, 2 * [s[0] for s in SHAPES].index(name) + wtype)  # fixed: the same inputs in every run
    W = synth.make_weight(rng, wtype, N, K)
    w = ql.PackedQWeight(wtype, torch.from_numpy(W))
    bias = rng.standard_normal(N).astype(np.float32)
    for M in (1, 4, 8):
        bits, xf = synth.make_x_bf16(rng, M, K)
        announce("gemv", name, N, K, "wtype", wtype, "M", M)
        for mode in (orc.SCALE_X86_REF, orc.SCALE_IEEE):
            y = ql.linear_q_gemv(w, bf16_dev(bits), None, _mode(mode)).cpu().numpy()
            want = orc.linear_q(xf, W, wtype, None, mode)
            assert rel_l2(y, want) < TOL, (M, mode, rel_l2(y, want))
            assert rel_l2(y, want) < 2e-6, (M, mode, rel_l2(y, want))  # in practice only the summation order differs
        yb = ql.linear_q_gemv(w, to_dev(xf), to_dev(bias), ql.SCALE_X86_REF).cpu().numpy()
        assert rel_l2(yb, orc.linear_q(xf, W, wtype, bias, orc.SCALE_X86_REF)) < 2e-6


@pytest.mark.parametrize("N,K", [(1, 32), (37, 96), (1000, 800), (65, 2048), (7, 4096 + 32)])
@pytest.mark.parametrize("M", [1, 2, 3, 5, 6, 7, 8])
def test_gemv_ragged(N, K, M):
    rng = synth.rng_for(1, N + K + M)
    for wtype in (0, 1):
        W = synth.make_weight(rng, wtype, N, K)
        w = ql.PackedQWeight(wtype, torch.from_numpy(W))
        xf = synth.make_x_fp32(rng, M, K)
        announce("ragged", N, K, M, wtype)
        y = ql.linear_q_gemv(w, to_dev(xf), None, ql.SCALE_X86_REF).cpu().numpy()
        assert rel_l2(y, orc.linear_q(xf, W, wtype, None, orc.SCALE_X86_REF)) < 2e-6


def test_gemv_every_launch_shape():
    """the dot4 kernel in every launch shape it is compiled for (with three rows or more it is the comparison path: path 1)"""
    rng = synth.rng_for(1, 99)
    N, K = 520, 2560
    L = _lib.lib()
    assert L.mllm_hip_gemv_set_path(1) == 0
    try:
        for wtype in (0, 1):
            W = synth.make_weight(rng, wtype, N, K)
            w = ql.PackedQWeight(wtype, torch.from_numpy(W))
            for M in (1, 2, 4, 8):
                xf = synth.make_x_fp32(rng, M, K)
                want = orc.linear_q(xf, W, wtype, None, orc.SCALE_X86_REF)
                xd = to_dev(xf)
                for G in (8, 16, 32, 64):
                    for R in (1, 2, 4):
                        for NW in (1, 4, 16):
                            announce("launch shape", wtype, M, G, R, NW)
                            assert L.mllm_hip_gemv_set_tuning(G, R, NW) == 0
                            y = ql.linear_q_gemv(w, xd, None, ql.SCALE_X86_REF).cpu().numpy()
                            assert rel_l2(y, want) < 2e-6, (wtype, M, G, R, NW)
        # the matrix-core kernel with its own sweep knobs: K slices (second argument) and waves per workgroup (third)
        assert L.mllm_hip_gemv_set_path(0) == 0
        W = synth.make_weight(rng, 0, N, K)
        w = ql.PackedQWeight(0, torch.from_numpy(W))
        for M in (3, 8):
            xf = synth.make_x_fp32(rng, M, K)
            want = orc.linear_q(xf, W, 0, None, orc.SCALE_X86_REF)
            for S in (0, 1, 2, 4):
                for NW in (0, 2, 4, 8):
                    announce("matrix-core launch shape", M, S, NW)
                    assert L.mllm_hip_gemv_set_tuning(0, S, NW) == 0
                    assert rel_l2(ql.linear_q_gemv(w, to_dev(xf), None, ql.SCALE_X86_REF).cpu().numpy(), want) < 2e-6, (M, S, NW)
    finally:
        L.mllm_hip_gemv_set_tuning(0, 0, 0)
        L.mllm_hip_gemv_set_path(0)


def test_gemv_special_inputs():
    """all-zero activations -> bias only; a x20 outlier; a single hot element"""
    rng = synth.rng_for(1, 5)
    N, K = 256, 1024
    W = synth.make_q4_0(rng, N, K)
    w = ql.PackedQWeight(0, torch.from_numpy(W))
    bias = rng.standard_normal(N).astype(np.float32)
    announce("special inputs")
    y0 = ql.linear_q_gemv(w, torch.zeros((2, K), device="cuda"), to_dev(bias)).cpu().numpy()
    assert np.array_equal(y0, np.stack([bias, bias]))
    x = synth.make_x_fp32(rng, 1, K)
    x[0, 17] *= 20
    y = ql.linear_q_gemv(w, to_dev(x)).cpu().numpy()
    assert rel_l2(y, orc.linear_q(x, W, 0)) < 2e-6
    e = np.zeros((1, K), np.float32)
    e[0, 40] = 3.0
    y = ql.linear_q_gemv(w, to_dev(e), None, ql.SCALE_IEEE).cpu().numpy()
    col = orc.dequantize(W, 0)[:, 40] / np.float32(1)  # one hot: y = W[:, 40] * dequant(q8(3.0)) = w * 127 * d
    d = np.float32(np.float16(np.float32(3.0) / np.float32(127)))
    assert np.allclose(y[0], col * (np.float32(127) * d), rtol=1e-6, atol=0)


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M", [9, 16, 21])
def test_gemv_more_than_eight_rows_runs_as_passes(wtype, M):
    """rows beyond eight are passes of eight over the same weights: row by row the bits of an eight-row call"""
    rng = synth.rng_for(1, 800 + M + wtype)
    N, K = 300, 1024
    W = synth.make_weight(rng, wtype, N, K)
    w = ql.PackedQWeight(wtype, torch.from_numpy(W))
    bias = to_dev(rng.standard_normal(N).astype(np.float32))
    xf = synth.make_x_fp32(rng, M, K)
    xd = to_dev(xf)
    announce("gemv passes", wtype, M)
    y = ql.linear_q_gemv(w, xd, bias)
    for m0 in range(0, M, 8):
        assert torch.equal(y[m0:m0 + 8], ql.linear_q_gemv(w, xd[m0:m0 + 8].contiguous(), bias))
    assert rel_l2(y.cpu().numpy(), orc.linear_q(xf, W, wtype, bias.cpu().numpy(), orc.SCALE_X86_REF)) < 2e-6
    r = to_dev(rng.standard_normal((M, N)).astype(np.float32))
    (yr,) = ql.linear_q_gemv_fused([w], xd, biases=[bias], residuals=[r], workspace=ql.gemv_workspace(8, K))
    assert torch.equal(yr, y + r)


@pytest.mark.parametrize("M", [1, 2, 5])
def test_gemv_vocabulary_sized_matrix(M):
    """the lm_head of the reference's Qwen3 recipes: 151936 rows (quant_cfg_30B_q4_k.json lists [151936, 2048]); checked on
    sampled rows, the first and the last ones included"""
    rng = synth.rng_for(1, 950 + M)
    N, K = 151936, 2048
    W = synth.make_weight(rng, 0, N, K)
    w = ql.PackedQWeight(0, torch.from_numpy(W))
    xf = synth.make_x_fp32(rng, M, K)
    announce("gemv vocabulary rows", M)
    y = ql.linear_q_gemv(w, to_dev(xf)).cpu().numpy()
    rows = np.unique(np.concatenate([np.arange(40), np.arange(N - 40, N), rng.integers(0, N, 2000)]))
    want = orc.linear_q(xf, W[rows], 0, None, orc.SCALE_X86_REF)
    assert rel_l2(y[:, rows], want) < 2e-6
    assert np.isfinite(y).all()


def test_gemv_argument_errors():
    L = _lib.lib()
    rng = synth.rng_for(1, 6)
    W = synth.make_q4_0(rng, 8, 64)
    w = ql.PackedQWeight(0, torch.from_numpy(W))
    x = torch.zeros((8, 64), device="cuda")
    y = torch.zeros((8, 8), device="cuda")
    f = L.mllm_hip_linear_q_gemv
    assert f(0, w.ptr, x.data_ptr(), 0, None, y.data_ptr(), 0, 8, 64, 0, None) == -2   # M = 0
    fu = _lib.GemvFusion(None, None)  # an image holds at most eight rows
    part = (_lib.GemvPart * 1)(_lib.GemvPart(w.ptr, None, y.data_ptr(), 8))
    assert L.mllm_hip_linear_q_gemv_fused(0, 1, part, C.byref(fu), x.data_ptr(), ql.Q8_IMAGE, 9, 64, 0, None) == -2
    assert f(0, w.ptr, x.data_ptr(), 0, None, y.data_ptr(), 1, 8, 48, 0, None) == -2   # K % 32
    assert f(5, w.ptr, x.data_ptr(), 0, None, y.data_ptr(), 1, 8, 64, 0, None) == -1   # weight type
    assert f(0, None, x.data_ptr(), 0, None, y.data_ptr(), 1, 8, 64, 0, None) == -1    # null weight
    assert f(0, w.ptr, None, 0, None, y.data_ptr(), 1, 8, 64, 0, None) == -1           # null x
    assert f(0, w.ptr, x.data_ptr(), 7, None, y.data_ptr(), 1, 8, 64, 0, None) == -1   # x dtype
    assert f(0, w.ptr + 4, x.data_ptr(), 0, None, y.data_ptr(), 1, 8, 64, 0, None) == -3  # alignment
    assert L.mllm_hip_q_packed_bytes(0, 8, 48) == 0
    with pytest.raises(_lib.HipQLinearError):
        _lib.check(-2, "probe")


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M", [11, 16, 18, 20, 21, 32])
def test_gemv_groups_of_eight_rows_share_a_launch(wtype, M):
    """more than eight rows, with room in the workspace for every group's partial sums: the groups of eight rows run in one
    launch, a last group of three to seven rows with them (one or two remaining rows as a pass of their own): row by row the
    bits of a call with that group alone and the same kind of workspace (a group of three or four rows alone runs the
    four-row build of the kernel: same bits); cut rows, whole rows, several matrices, ragged N, a last slice that is empty"""
    rng = synth.rng_for(1, 900 + M + wtype)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(900 + M + wtype)
    assert _lib.lib().mllm_hip_gemv_set_path(3) == 0  # this form, not the many-row kernel that nine rows and more take by default
    try:
        _groups_of_eight_rows_share_a_launch(wtype, M, rng, gen)
    finally:
        assert _lib.lib().mllm_hip_gemv_set_path(0) == 0


def _groups_of_eight_rows_share_a_launch(wtype, M, rng, gen):
    for shapes, oracle_too in (([(300, 1024)], True), ([(50, 161 * 32)], True), ([(2560, 9728)], False),
                               ([(4096, 2560), (1024, 2560), (1024, 2560)], False), ([(9728, 2560), (9728, 2560)], False),
                               ([(8200, 97 * 32), (8193, 97 * 32)], False)):
        K = shapes[0][1]
        n_total = sum(n for n, _ in shapes)
        if oracle_too:
            Ws = [synth.make_weight(rng, wtype, n, K) for n, _ in shapes]
            ws = [ql.PackedQWeight(wtype, torch.from_numpy(W)) for W in Ws]
        else:
            ws = [ql.PackedQWeight.synthetic(wtype, n, K, gen) for n, _ in shapes]
        biases = [to_dev(rng.standard_normal(n).astype(np.float32)) for n, _ in shapes]
        for bf16 in (True, False):
            if bf16:
                bits, xf = synth.make_x_bf16(rng, M, K)
                xd = bf16_dev(bits)
            else:
                xf = synth.make_x_fp32(rng, M, K)
                xd = to_dev(xf)
            announce("gemv row groups", wtype, M, shapes, "bf16" if bf16 else "fp32")
            outs = ql.linear_q_gemv_multi(ws, xd, biases, workspace=ql.gemv_workspace(M, K, n_total))
            ws8 = ql.gemv_workspace(8, K, n_total)
            for m0 in range(0, M, 8):
                part = ql.linear_q_gemv_multi(ws, xd[m0:m0 + 8].contiguous(), biases, workspace=ws8)
                for o, pr in zip(outs, part):
                    assert torch.equal(o[m0:m0 + 8], pr), (shapes, m0)
            if oracle_too:
                for W, b, o in zip(Ws, biases, outs):
                    assert rel_l2(o.cpu().numpy(), orc.linear_q(xf, W, wtype, b.cpu().numpy(), orc.SCALE_X86_REF)) < 2e-6
    # with residuals (the fused entry point), the same groups
    K, N = 1024, 300
    w = ql.PackedQWeight.synthetic(wtype, N, K, gen)
    xd = to_dev(synth.make_x_fp32(rng, M, K))
    r = to_dev(rng.standard_normal((M, N)).astype(np.float32))
    (y,) = ql.linear_q_gemv_multi([w], xd, None, workspace=ql.gemv_workspace(M, K, N))
    (yr,) = ql.linear_q_gemv_fused([w], xd, residuals=[r], workspace=ql.gemv_workspace(M, K, N))
    assert torch.equal(yr, y + r)


def test_gemv_groups_run_in_several_launches_when_one_is_refused():
    """all groups of a batch in one launch need room for every group's partial sums and an arrival counter per (workgroup
    column, group): with less of either the groups run as halves (quarters, ...) of the batch per launch, same bits"""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(77)
    rng = synth.rng_for(1, 977)
    assert _lib.lib().mllm_hip_gemv_set_path(3) == 0  # the form of groups of eight rows
    try:
        # 8192 x 8192: rows of 256 blocks are always cut, 128 workgroup columns x 16 groups = 2048 counters > 1024
        for (N, K, M, ws_rows) in ((8192, 8192, 128, 128), (300, 1024, 37, 16), (2560, 9728, 32, 16)):
            w = ql.PackedQWeight.synthetic(0, N, K, gen)
            xd = to_dev(synth.make_x_fp32(rng, M, K))
            announce("gemv row groups in several launches", N, K, M, ws_rows)
            (y,) = ql.linear_q_gemv_multi([w], xd, None, workspace=ql.gemv_workspace(ws_rows, K, N))
            ws8 = ql.gemv_workspace(8, K, N)
            for m0 in range(0, M, 8):
                (part,) = ql.linear_q_gemv_multi([w], xd[m0:m0 + 8].contiguous(), None, workspace=ws8)
                assert torch.equal(y[m0:m0 + 8], part), (N, K, M, m0)
    finally:
        assert _lib.lib().mllm_hip_gemv_set_path(0) == 0


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M", [9, 12, 16, 17, 24, 32, 33, 40, 64, 70])
def test_gemv_many_rows_read_the_weights_once(wtype, M):
    """Nine rows and more with room in the workspace for the image of all rows: one launch quantizes x, one launch of the
    many-row kernel (16 x 16 x 32 integer matrix instruction = one block, 16 or 32 activation rows per workgroup) produces every
    row.  Against the oracle (the reference's arithmetic, 2e-6: the fp32 additions run in another order), against the form of
    groups of eight rows, twice in a row (the arrival counters go back to zero), and row by row the same bits whatever else is
    in the call: cut rows, whole rows, several matrices, ragged N, a last slice that is empty, bias and residual."""
    rng = synth.rng_for(1, 1900 + M + wtype)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1900 + M + wtype)
    L = _lib.lib()
    for shapes, oracle_too in (([(300, 1024)], True), ([(50, 161 * 32)], True), ([(37, 96), (7, 96)], True), ([(65, 32)], True),
                               ([(2560, 9728)], False), ([(4096, 2560), (1024, 2560), (1024, 2560)], False),
                               ([(9728, 2560), (9728, 2560)], False), ([(8200, 97 * 32), (8193, 97 * 32)], False)):
        K = shapes[0][1]
        n_total = sum(n for n, _ in shapes)
        if oracle_too:
            Ws = [synth.make_weight(rng, wtype, n, K) for n, _ in shapes]
            ws = [ql.PackedQWeight(wtype, torch.from_numpy(W)) for W in Ws]
        else:
            ws = [ql.PackedQWeight.synthetic(wtype, n, K, gen) for n, _ in shapes]
        biases = [to_dev(rng.standard_normal(n).astype(np.float32)) for n, _ in shapes]
        wsp = ql.gemv_workspace(M, K, n_total)
        for bf16 in (True, False):
            if bf16:
                bits, xf = synth.make_x_bf16(rng, M, K)
                xd = bf16_dev(bits)
            else:
                xf = synth.make_x_fp32(rng, M, K)
                xd = to_dev(xf)
            announce("gemv many rows", wtype, M, shapes, "bf16" if bf16 else "fp32")
            # by default the kernel takes the launches whose rows stay whole (many row tiles, rows of up to 128 blocks) and leaves
            # the others to the groups of eight rows; the second tuning value 2 makes it take every launch (rows cut into K
            # slices that meet in memory), 1 keeps rows whole wherever they fit
            outs = [torch.full((M, n), float("nan"), device="cuda") for n, _ in shapes]
            ql.linear_q_gemv_multi(ws, xd, biases, outs=outs, workspace=wsp)
            assert L.mllm_hip_gemv_set_tuning(0, 2, 0) == 0
            try:
                forced = [torch.full((M, n), float("nan"), device="cuda") for n, _ in shapes]
                ql.linear_q_gemv_multi(ws, xd, biases, outs=forced, workspace=wsp)
                again = ql.linear_q_gemv_multi(ws, xd, biases, workspace=wsp)  # (the arrival counters are back at zero)
                if M > 9:  # a row's bits do not depend on the other rows of the call
                    tail = ql.linear_q_gemv_multi(ws, xd[M - 9:].contiguous(), biases, workspace=wsp)
                    for o, t in zip(forced, tail):
                        assert torch.equal(o[M - 9:], t)
                assert L.mllm_hip_gemv_set_tuning(0, 1, 0) == 0
                whole = ql.linear_q_gemv_multi(ws, xd, biases, workspace=wsp)
            finally:
                assert L.mllm_hip_gemv_set_tuning(0, 0, 0) == 0
            for o, f, o2, wh in zip(outs, forced, again, whole):
                assert torch.equal(f, o2)
                assert rel_l2(f.cpu().numpy(), o.cpu().numpy()) < 2e-6 and rel_l2(wh.cpu().numpy(), o.cpu().numpy()) < 2e-6
            if oracle_too:
                for W, b, f, wh in zip(Ws, biases, forced, whole):
                    want = orc.linear_q(xf, W, wtype, b.cpu().numpy(), orc.SCALE_X86_REF)
                    assert rel_l2(f.cpu().numpy(), want) < 2e-6 and rel_l2(wh.cpu().numpy(), want) < 2e-6
            assert L.mllm_hip_gemv_set_path(3) == 0
            try:
                eights = ql.linear_q_gemv_multi(ws, xd, biases, workspace=wsp)
            finally:
                assert L.mllm_hip_gemv_set_path(0) == 0
            for o, e in zip(outs, eights):
                assert rel_l2(o.cpu().numpy(), e.cpu().numpy()) < 2e-6  # another kernel: another order of additions of the same terms
            if oracle_too:
                for W, b, o in zip(Ws, biases, outs):
                    assert rel_l2(o.cpu().numpy(), orc.linear_q(xf, W, wtype, b.cpu().numpy(), orc.SCALE_X86_REF)) < 2e-6
    # residuals (the fused entry point)
    K, N = 1024, 300
    w = ql.PackedQWeight.synthetic(wtype, N, K, gen)
    xd = to_dev(synth.make_x_fp32(rng, M, K))
    r = to_dev(rng.standard_normal((M, N)).astype(np.float32))
    wsp = ql.gemv_workspace(M, K, N)
    (y,) = ql.linear_q_gemv_multi([w], xd, None, workspace=wsp)
    (yr,) = ql.linear_q_gemv_fused([w], xd, residuals=[r], workspace=wsp)
    assert torch.equal(yr, y + r)
    # a workspace without room for the image of all rows: the groups of eight rows, as before
    (y8,) = ql.linear_q_gemv_multi([w], xd, None, workspace=ql.gemv_workspace(8, K))
    assert L.mllm_hip_gemv_set_path(3) == 0
    try:
        (y3,) = ql.linear_q_gemv_multi([w], xd, None, workspace=ql.gemv_workspace(8, K))
    finally:
        assert L.mllm_hip_gemv_set_path(0) == 0
    assert torch.equal(y8, y3)
    assert L.mllm_hip_gemv_splitk_workspace_bytes(32, 2560, 19456) >= 32 * 80 * 40 + 2 * 32 * (19456 + 32) * 4


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M", [1, 3, 8])
def test_gemv_multi_equals_single(wtype, M):
    """sibling projections in one launch give exactly the bits of one launch each (q/k/v and gate/up shapes)"""
    rng = synth.rng_for(1, 70 + M + wtype)
    for shapes in ([(4096, 2560), (1024, 2560), (1024, 2560)], [(9728, 2560), (9728, 2560)], [(40, 96), (7, 96), (33, 96), (1, 96)]):
        K = shapes[0][1]
        Ws = [synth.make_weight(rng, wtype, n, K) for n, _ in shapes]
        ws = [ql.PackedQWeight(wtype, torch.from_numpy(W)) for W in Ws]
        biases = [to_dev(rng.standard_normal(n).astype(np.float32)) for n, _ in shapes]
        bits, xf = synth.make_x_bf16(rng, M, K)
        xd = bf16_dev(bits)
        announce("gemv multi", wtype, M, shapes)
        outs = ql.linear_q_gemv_multi(ws, xd, biases)
        for w, W, b, o in zip(ws, Ws, biases, outs):
            single = ql.linear_q_gemv(w, xd, b)
            assert torch.equal(o, single)
            assert rel_l2(o.cpu().numpy(), orc.linear_q(xf, W, wtype, b.cpu().numpy(), orc.SCALE_X86_REF)) < 2e-6
    L = _lib.lib()
    assert L.mllm_hip_linear_q_gemv_multi(0, 5, None, None, 0, 1, 64, 0, None) == -1
    assert L.mllm_hip_linear_q_gemv_multi(0, 0, None, None, 0, 1, 64, 0, None) == -1


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M", [1, 2])
def test_gemv_request_order_does_not_change_the_bits(wtype, M):
    """One or two rows: the kernel that asks for all weights of its first trip at once and the one that asks for all but the
    first block column behind the quantization of x (the default for large launches) compute the same sums in the same
    order: equal bit for bit, whichever the size rule would pick.  Raw activations (fp32, bf16), both scale modes, bias,
    sibling matrices, ragged N, rows of one to 304 blocks, and the quantized image as input."""
    rng = synth.rng_for(1, 430 + M + 10 * wtype)
    L = _lib.lib()
    assert L.mllm_hip_gemv_set_request_order(2) == -1 and L.mllm_hip_gemv_set_request_order(-2) == -1
    for shapes in ([(4096, 2560), (1024, 2560), (1024, 2560)], [(2560, 9728)], [(257, 4096)], [(40, 96), (7, 96), (33, 96)],
                   [(65, 32)], [(300, 2048), (9, 2048)], [(129, 161 * 32)]):
        K = shapes[0][1]
        ws = [ql.PackedQWeight(wtype, torch.from_numpy(synth.make_weight(rng, wtype, n, K))) for n, _ in shapes]
        biases = [to_dev(rng.standard_normal(n).astype(np.float32)) for n, _ in shapes]
        x = synth.make_x_fp32(rng, M, K)
        announce("gemv request order", wtype, M, shapes)
        for xd in (to_dev(x), bf16_dev(synth.fp32_to_bf16_bits(x))):
            for mode in (ql.SCALE_X86_REF, ql.SCALE_IEEE):
                outs = {}
                for order in (0, 1):
                    assert L.mllm_hip_gemv_set_request_order(order) == 0
                    try:
                        outs[order] = ql.linear_q_gemv_multi(ws, xd, biases, mode)
                    finally:
                        assert L.mllm_hip_gemv_set_request_order(-1) == 0
                for a_, b_ in zip(outs[0], outs[1]):
                    assert torch.equal(a_, b_)
        xd = to_dev(x)
        _, img = ql.add(xd, torch.zeros_like(xd), want_image=True)
        outs = {}
        for order in (0, 1):
            assert L.mllm_hip_gemv_set_request_order(order) == 0
            try:
                outs[order] = ql.linear_q_gemv_fused(ws, img, M=M, image=True, biases=biases)
            finally:
                assert L.mllm_hip_gemv_set_request_order(-1) == 0
        for a_, b_ in zip(outs[0], outs[1]):
            assert torch.equal(a_, b_)


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M", [3, 4, 5, 8])
def test_gemv_matrix_core_and_vector_kernels_agree(wtype, M):
    """three to eight rows: the matrix-core kernel (default) and the vector-ALU kernel are two independent implementations of
    the same arithmetic (exact block sums, fp32 scaling); they differ only in the order of the fp32 sums"""
    rng = synth.rng_for(1, 700 + M + 10 * wtype)
    L = _lib.lib()
    for N, K in ((9728, 2560), (2560, 9728), (100, 4096 + 64), (33, 96), (257, 8192)):
        W = synth.make_weight(rng, wtype, N, K)
        w = ql.PackedQWeight(wtype, torch.from_numpy(W))
        bias = to_dev(rng.standard_normal(N).astype(np.float32))
        xf = synth.make_x_fp32(rng, M, K)
        xd = to_dev(xf)
        announce("gemv both kernels", wtype, M, N, K)
        y0 = ql.linear_q_gemv(w, xd, bias)
        _, img = ql.add(xd, torch.zeros_like(xd), want_image=True)
        (y0i,) = ql.linear_q_gemv_fused([w], img, M=M, image=True, biases=[bias])
        assert torch.equal(y0, y0i)  # activations quantized in the kernel or handed over as an image: the same bits
        assert L.mllm_hip_gemv_set_path(1) == 0
        try:
            y1 = ql.linear_q_gemv(w, xd, bias)
        finally:
            assert L.mllm_hip_gemv_set_path(0) == 0
        assert rel_l2(y0.cpu().numpy(), y1.cpu().numpy()) < 2e-6
        assert rel_l2(y0.cpu().numpy(), orc.linear_q(xf, W, wtype, bias.cpu().numpy(), orc.SCALE_X86_REF)) < 2e-6
    assert L.mllm_hip_gemv_set_path(4) == -1


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M", [3, 4, 5, 8])
def test_gemv_k_slices_as_workgroups_give_the_same_bits(wtype, M):
    """With room for partial sums in the workspace the K slices of a row tile are separate workgroups that meet through
    global memory (one launch, every workgroup quantizes its slice of x).  Same partial sums added in the same order as the
    form that keeps the slices in one workgroup (path 2), so the outputs must be equal bit for bit: fp32 and bf16
    activations, both scale modes, bias, several matrices per launch, ragged N, rows whose last slice is empty (161 blocks),
    one to eight slices; and against the oracle."""
    rng = synth.rng_for(1, 900 + M + 10 * wtype)
    L = _lib.lib()
    # Q8_0 at three or four rows: the comparison path (no slice form) is the vector-ALU kernel there, which adds the blocks
    # of a row in another order
    for shapes in ([(9728, 2560), (9728, 2560)], [(2560, 9728)], [(4096, 2560), (1024, 2560), (1024, 2560)], [(2560, 4096)],
                   [(40, 96), (7, 96), (33, 96)], [(65, 32)], [(50, 161 * 32)], [(129, 41 * 32), (16, 41 * 32)],
                   # the longest rows the one-workgroup matrix-core kernel holds (two trips per slice at four rows)
                   [(31, (512 if M <= 4 else 320) * 32)],
                   # whole rows (below), ragged: 97 blocks, the last row tile with one row
                   [(8200, 97 * 32), (8193, 97 * 32)]):
        K = shapes[0][1]
        # (a launch of 1024 row tiles or more with rows of up to 128 blocks keeps its rows whole: one workgroup sums the
        # chains the slices would have summed and adds them in slice order)
        same_bits = not (wtype == 1 and M <= 4)
        Ws = [synth.make_weight(rng, wtype, n, K) for n, _ in shapes]
        ws = [ql.PackedQWeight(wtype, torch.from_numpy(W)) for W in Ws]
        biases = [to_dev(rng.standard_normal(n).astype(np.float32)) for n, _ in shapes]
        x = synth.make_x_fp32(rng, M, K)
        wsp = ql.gemv_workspace(M, K, sum(n for n, _ in shapes))
        announce("gemv k slices as workgroups", wtype, M, shapes)
        for xd in (to_dev(x), bf16_dev(synth.fp32_to_bf16_bits(x))):
            for mode in (ql.SCALE_X86_REF, ql.SCALE_IEEE):
                assert L.mllm_hip_gemv_set_path(2) == 0
                try:
                    one_wg = ql.linear_q_gemv_multi(ws, xd, biases, mode, workspace=wsp)
                finally:
                    assert L.mllm_hip_gemv_set_path(0) == 0
                for rep in range(2):  # twice: the arrival counters must be back at zero after a launch
                    outs = [torch.full((M, n), float("nan"), device="cuda") for n, _ in shapes]
                    ql.linear_q_gemv_multi(ws, xd, biases, mode, outs=outs, workspace=wsp)
                    for f, p in zip(one_wg, outs):
                        if same_bits:
                            assert torch.equal(f, p)
                        else:
                            assert rel_l2(p.cpu().numpy(), f.cpu().numpy()) < 2e-6
        # residual added in the epilogue, and the quantized image as input
        xd = to_dev(x)
        res = [to_dev(rng.standard_normal((M, n)).astype(np.float32)) for n, _ in shapes]
        _, img = ql.add(xd, torch.zeros_like(xd), want_image=True)
        assert L.mllm_hip_gemv_set_path(2) == 0
        try:
            r0 = ql.linear_q_gemv_fused(ws, xd, biases=biases, residuals=res, workspace=wsp)
        finally:
            assert L.mllm_hip_gemv_set_path(0) == 0
        r1 = ql.linear_q_gemv_fused(ws, xd, biases=biases, residuals=res, workspace=wsp)
        r2 = ql.linear_q_gemv_fused(ws, img, M=M, image=True, biases=biases, residuals=res, workspace=wsp)
        for f, p, i in zip(r0, r1, r2):
            assert torch.equal(p, i)
            assert torch.equal(f, p) if same_bits else rel_l2(p.cpu().numpy(), f.cpu().numpy()) < 2e-6
        want = orc.linear_q(x, Ws[0], wtype, biases[0].cpu().numpy(), orc.SCALE_X86_REF)
        got = ql.linear_q_gemv_multi(ws, to_dev(x), biases, ql.SCALE_X86_REF, workspace=wsp)[0].cpu().numpy()
        assert rel_l2(got, want) < 2e-6
    assert L.mllm_hip_gemv_splitk_workspace_bytes(8, 9728, 2560) == 8 * 304 * 40 + 8 * 8 * (2560 + 64) * 4
    assert L.mllm_hip_gemv_splitk_workspace_bytes(8, 96, 100) == 8 * 3 * 40 + 1 * 8 * (100 + 64) * 4
    assert L.mllm_hip_gemv_splitk_workspace_bytes(0, 96, 100) == 0


@pytest.mark.parametrize("wtype", [0, 1])
def test_gemv_k_slices_share_a_workspace_across_launch_shapes(wtype):
    """The columns' arrival counters of a launch lie up to a cache line apart inside the workspace's block of counters, the
    distance depending on how many columns the launch has: launches of different shapes on ONE workspace (32 columns: a
    line per counter; hundreds of columns and several row groups: neighbouring counters) must find every counter at zero
    whatever the launch before used.  Three rounds over the shapes, eight and 24 rows, each output equal bit for bit to the
    form that keeps the slices in one workgroup (eight rows) or to the same call on a workspace of its own (24 rows)."""
    rng = synth.rng_for(1, 977 + wtype)
    L = _lib.lib()
    shapes = [(2560, 9728), (6144, 2560), (100, 161 * 32), (9000, 4096)]
    Ws = [ql.PackedQWeight(wtype, torch.from_numpy(synth.make_weight(rng, wtype, n, k))) for n, k in shapes]
    for M in (8, 24):
        xs = [bf16_dev(synth.fp32_to_bf16_bits(synth.make_x_fp32(rng, M, k))) for _, k in shapes]
        shared = ql.gemv_workspace(M, max(k for _, k in shapes), max(n for n, _ in shapes))
        refs = []
        for w, x, (n, k) in zip(Ws, xs, shapes):
            own = ql.gemv_workspace(M, k, n)
            if M <= 8:
                assert L.mllm_hip_gemv_set_path(2) == 0
            try:
                refs.append(ql.linear_q_gemv_multi([w], x, None, ql.SCALE_X86_REF, workspace=own)[0])
            finally:
                assert L.mllm_hip_gemv_set_path(0) == 0
        announce("gemv k slices, one workspace, several launch shapes", wtype, M)
        for rnd in range(3):
            for w, x, ref in zip(Ws, xs, refs):
                y = torch.full_like(ref, float("nan"))
                ql.linear_q_gemv_multi([w], x, None, ql.SCALE_X86_REF, outs=[y], workspace=shared)
                assert torch.equal(y, ref)


def _counter_stats():
    import ctypes as C
    owned, cap = C.c_int(), C.c_int()
    rec, ref = C.c_longlong(), C.c_longlong()
    assert _lib.lib().mllm_hip_gemv_workspace_stats(0, C.byref(owned), C.byref(cap), C.byref(rec), C.byref(ref)) == 0
    return owned.value, cap.value, rec.value, ref.value


def test_gemv_k_slices_keep_their_kernel_over_more_workspace_addresses_than_counter_blocks():
    """The K-slice kernel keeps one block of arrival counters per workspace ADDRESS.  A caller that walks through more
    addresses than there are blocks must still get that kernel: same bits as the first call (Q8_0 at four rows, where the
    kernels that would otherwise run add the blocks in another order and give other bits), nothing refused, the blocks handed
    out afresh at least once, and about the same time per call.  A released address gives its block back."""
    import time
    rng = synth.rng_for(1, 4242)
    L = _lib.lib()
    M, N, K = 4, 200, 64 * 32
    W = synth.make_weight(rng, 1, N, K)
    w = ql.PackedQWeight(1, torch.from_numpy(W))
    x = to_dev(synth.make_x_fp32(rng, M, K))
    need = L.mllm_hip_gemv_splitk_workspace_bytes(M, K, N)
    stride = (need + 255) // 256 * 256
    _, cap, rec0, ref0 = _counter_stats()
    count = cap + 76
    pool = torch.empty(stride * count, dtype=torch.uint8, device="cuda")
    announce("gemv k slices: workspace addresses", count, "counter blocks", cap)
    first = ql.linear_q_gemv_multi([w], x, workspace=pool[:need])[0]
    want = orc.linear_q(x.cpu().numpy(), W, 1, None, orc.SCALE_X86_REF)
    assert rel_l2(first.cpu().numpy(), want) < 2e-6
    assert L.mllm_hip_gemv_set_path(2) == 0  # without the K-slice kernel: the bits differ (that is what makes this a test)
    try:
        other = ql.linear_q_gemv_multi([w], x, workspace=pool[:need])[0]
    finally:
        assert L.mllm_hip_gemv_set_path(0) == 0
    assert not torch.equal(first, other)
    torch.cuda.synchronize()
    times = []
    for i in range(count):
        wsp = pool[i * stride:i * stride + need]
        t0 = time.perf_counter()
        y = ql.linear_q_gemv_multi([w], x, workspace=wsp)[0]
        times.append(time.perf_counter() - t0)
        assert torch.equal(y, first), i
    torch.cuda.synchronize()
    owned, _, rec1, ref1 = _counter_stats()
    assert ref1 == ref0 and rec1 >= rec0 + 1 and 1 <= owned <= cap
    # the calls after the table was handed out afresh cost what the early ones did (host time per call, median)
    early, late = sorted(times[10:110])[50], sorted(times[-60:])[30]
    assert late < 3 * early + 20e-6, (early, late)
    # release: the address of the last call gives its block back, an unknown address is fine
    assert L.mllm_hip_gemv_workspace_release(wsp.data_ptr()) == 0
    assert _counter_stats()[0] == owned - 1
    assert L.mllm_hip_gemv_workspace_release(wsp.data_ptr()) == 0
    assert L.mllm_hip_gemv_workspace_release(None) == -1


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M", [4, 8])
def test_gemv_k_slices_as_workgroups_take_rows_of_any_length(wtype, M):
    """rows beyond what the one-workgroup kernels hold in LDS (eight rows: about 11 000 elements): the slice form has no such
    limit; against the oracle"""
    rng = synth.rng_for(1, 950 + M + 10 * wtype)
    for N, K in ((31, 512 * 32), (20, 1030 * 32)):
        W = synth.make_weight(rng, wtype, N, K)
        w = ql.PackedQWeight(wtype, torch.from_numpy(W))
        x = synth.make_x_fp32(rng, M, K)
        bias = rng.standard_normal(N).astype(np.float32)
        announce("gemv long rows", wtype, M, N, K)
        (got,) = ql.linear_q_gemv_multi([w], to_dev(x), [to_dev(bias)], ql.SCALE_X86_REF, workspace=ql.gemv_workspace(M, K, N))
        assert rel_l2(got.cpu().numpy(), orc.linear_q(x, W, wtype, bias, orc.SCALE_X86_REF)) < 2e-6


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M", [3, 4, 5, 8])
def test_gemv_prequantized_equals_fused(wtype, M):
    """With a workspace (three rows or more) x is quantized once by a small kernel and the GEMV copies that image: the
    results must be the bits of the fused kernel, for fp32 and bf16 activations, both scale modes, long and ragged rows."""
    rng = synth.rng_for(1, 90 + M + wtype)
    for shapes in ([(9728, 2560), (9728, 2560)], [(2560, 9728)], [(40, 96), (7, 96), (33, 96)], [(65, 32)]):
        K = shapes[0][1]
        Ws = [synth.make_weight(rng, wtype, n, K) for n, _ in shapes]
        ws = [ql.PackedQWeight(wtype, torch.from_numpy(W)) for W in Ws]
        biases = [to_dev(rng.standard_normal(n).astype(np.float32)) for n, _ in shapes]
        x = synth.make_x_fp32(rng, M, K)
        wsp = ql.gemv_workspace(M, K)
        announce("gemv prequantized", wtype, M, shapes)
        for xd in (to_dev(x), bf16_dev(synth.fp32_to_bf16_bits(x))):
            for mode in (ql.SCALE_X86_REF, ql.SCALE_IEEE):
                fused = ql.linear_q_gemv_multi(ws, xd, biases, mode)
                pre = ql.linear_q_gemv_multi(ws, xd, biases, mode, workspace=wsp)
                for f, p in zip(fused, pre):
                    assert torch.equal(f, p)
        want = orc.linear_q(x, Ws[0], wtype, biases[0].cpu().numpy(), orc.SCALE_X86_REF)
        got = ql.linear_q_gemv_multi(ws, to_dev(x), biases, ql.SCALE_X86_REF, workspace=wsp)[0].cpu().numpy()
        assert rel_l2(got, want) < 2e-6
    assert _lib.lib().mllm_hip_gemv_workspace_bytes(8, 2560) == 8 * 80 * 40
    assert _lib.lib().mllm_hip_gemv_workspace_bytes(9, 2560) == 8 * 80 * 40  # more rows run as passes of eight
    assert _lib.lib().mllm_hip_gemv_workspace_bytes(0, 2560) == 0


@pytest.mark.parametrize("wtype", [0, 1])
def test_weight_quantizer_bit_exact_and_round_trip(wtype, golden_dir):
    """The offline quantizer on the GPU: blocks equal to the oracle's byte for byte in both storage conventions (the
    oracle is pinned against the reference's own quantizers), the reference-written golden vectors, and the round trip
    quantize -> prepack -> GEMV against the oracle Linear on the same blocks."""
    rng = synth.rng_for(1, 110 + wtype)
    N, K = 200, 2560
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    w[1, :32] = 0.0
    w[2, :32] = np.float32(-0.5) * np.arange(32) / 31
    w[3, :32] = np.float32(0.5) * np.arange(32) / 31
    w[4, :32] = np.float32(8.0) * np.linspace(-1, 1, 32)
    announce("weight quantizer", wtype)
    for mode, omode in ((ql.SCALE_IEEE, orc.SCALE_IEEE), (ql.SCALE_X86_REF, orc.SCALE_X86_REF)):
        got = ql.quantize_weight_blocks(to_dev(w), wtype, mode).cpu().numpy()
        assert np.array_equal(got, orc.quantize_weight_rows(w, wtype, omode)), mode
    g = np.load(os.path.join(golden_dir, "weight_quantizer_kat.npz"))
    gb = ql.quantize_weight_blocks(to_dev(g["w"]), wtype, ql.SCALE_X86_REF).cpu().numpy()
    if wtype == 0:
        assert np.array_equal(gb[:, :, 2:], g["q4_blocks"][:, :, 2:])
    else:
        assert np.array_equal(gb[:, :, 2:].view(np.int8).reshape(g["w"].shape[0], -1), g["q8_codes"])
    # round trip in the x86 convention end to end
    blocks = ql.quantize_weight_blocks(to_dev(w), wtype, ql.SCALE_X86_REF)
    pw = ql.PackedQWeight(wtype, blocks, ql.SCALE_X86_REF)
    x = synth.make_x_fp32(rng, 2, K)
    y = ql.linear_q_gemv(pw, to_dev(x), None, ql.SCALE_X86_REF).cpu().numpy()
    canon = orc.quantize_weight_rows(w, wtype, orc.SCALE_IEEE)  # raw patterns: the oracle applies the x86 reading itself
    assert rel_l2(y, orc.linear_q(x, canon, wtype, None, orc.SCALE_X86_REF)) < 2e-6
    L = _lib.lib()
    assert L.mllm_hip_quantize_weight_blocks(wtype, None, blocks.data_ptr(), 0, 4, 64, None) == -1
    assert L.mllm_hip_quantize_weight_blocks(wtype, blocks.data_ptr(), blocks.data_ptr(), 0, 4, 48, None) == -2


def test_q8_scale_divisions_equal_ieee_division_for_every_amax():
    """The kernels for three to eight rows form d = amax / 127 and id = 127 / amax from short sequences (a multiply by
    RN(1/127) or v_rcp_f32, one residual, one correction; a wave with an amax outside [2^-100, 2^100] takes the compiler's
    division).  Every fp32 bit pattern from +0 through the positive finite numbers, +inf and the positive NaNs, taken as
    amax, must give the bits of IEEE division (amax is a maximum of magnitudes: never negative)."""
    L = _lib.lib()
    bad = torch.zeros(1, dtype=torch.int64, device="cuda")
    announce("q8 scale divisions, all non-negative bit patterns")
    for first, last in ((0x00000000, 0x3fffffff), (0x40000000, 0x7fffffff)):
        _lib.check(L.mllm_hip_probe_q8_scales(first, last, bad.data_ptr(), None), "mllm_hip_probe_q8_scales")
    torch.cuda.synchronize()
    assert int(bad.item()) == 0
    assert L.mllm_hip_probe_q8_scales(5, 4, bad.data_ptr(), None) == -1  # an empty range is refused
