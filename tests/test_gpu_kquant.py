"""GPU parity of the Q4_K / Q6_K Linear against the CPU oracle (which is pinned bit for bit against the compiled reference
kernels in tests/test_oracle_vs_reference.py).

Bars: Q8_K activation codes, scales and sums of 16, and dequantized weights bit-exact; fp32 outputs rel-L2 <= 1e-3 (the
integer part is exact, the fp32 accumulation order differs from the CPU's eight lanes; measured about 1e-7)."""
import numpy as np
import pytest
import torch

from mllm_amd import _lib, qlinear as ql, synth
from oracle import oracle as orc
from gpu_util import announce, bf16_dev, rel_l2, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_q8_K_quantization_bit_exact(dtype):
    rng = synth.rng_for(7, 1)
    M, K = 7, 2560
    if dtype == "bf16":
        bits, xf = synth.make_x_bf16(rng, M, K)
        x = bf16_dev(bits)
    else:
        xf = synth.make_x_fp32(rng, M, K) * 3
        xf[1, 256:512] = 0                       # an all-zero super-block
        xf[2, :256] = 0.1
        xf[2, 9], xf[2, 200] = -4.5, 4.5         # equal magnitudes, opposite signs: the first one decides
        xf[3, 512:768] = 0.25
        xf[3, 767] = -0.25                       # the LAST element differs in sign only
        xf[4, :256] = 0.1
        xf[4, 16], xf[4, 17] = 5.0, -5.0         # the tie inside one lane's eight elements, positive first
        xf[5, :256] = 0.1
        xf[5, 18], xf[5, 21] = -5.0, 5.0         # ... negative first
        xf[6, 256:512] = 0.1
        xf[6, 256 + 128], xf[6, 256 + 255] = 6.0, -6.0  # the tie across the two 16-lane rows of an odd super-block
        x = to_dev(xf)
    announce("q8_K quantization", dtype)
    q, d, bs = ql.quantize_q8_K(x)
    oq, od, obs = orc.quantize_rows_q8_K(xf)
    assert np.array_equal(q.cpu().numpy(), oq)
    assert np.array_equal(d.cpu().numpy().view(np.uint32), od.view(np.uint32))
    assert np.array_equal(bs.cpu().numpy(), obs)


@pytest.mark.parametrize("wtype", [2, 3])
def test_prepack_and_dequantize_bit_exact(wtype):
    rng = synth.rng_for(7, 10 + wtype)
    N, K = 37, 1280
    W = synth.make_weight(rng, wtype, N, K)
    announce("kq dequantize", wtype)
    w = ql.PackedKWeight(wtype, torch.from_numpy(W))
    assert np.array_equal(w.dequantize().cpu().numpy().view(np.uint32), orc.dequantize_k(W, wtype, orc.SCALE_IEEE).view(np.uint32))
    # blocks written by the x86 build: the fp16 fields hold the pattern as a NUMBER
    Wx = W.copy()
    for off in ((0, 2) if wtype == 2 else (208,)):
        pat = W[:, :, off:off + 2].copy().view(np.uint16).astype(np.float32)
        Wx[:, :, off:off + 2] = pat.astype(np.float16).view(np.uint16).reshape(N, -1, 1).view(np.uint8)
    wx = ql.PackedKWeight(wtype, torch.from_numpy(Wx), weight_scale_mode=ql.SCALE_X86_REF)
    assert np.array_equal(wx.dequantize().cpu().numpy().view(np.uint32), orc.dequantize_k(W, wtype, orc.SCALE_X86_REF).view(np.uint32))


@pytest.mark.parametrize("wtype", [2, 3])
@pytest.mark.parametrize("M,N,K", [(1, 256, 2560), (2, 100, 256), (3, 77, 768), (4, 512, 2048), (8, 130, 9728), (5, 31, 512),
                                   (11, 64, 1024), (20, 48, 2560)])
def test_linear_kq(wtype, M, N, K):
    rng = synth.rng_for(7, 100 + wtype * 1000 + M * 13 + N)
    W = synth.make_weight(rng, wtype, N, K)
    w = ql.PackedKWeight(wtype, torch.from_numpy(W))
    bias = rng.standard_normal(N).astype(np.float32)
    xf = synth.make_x_fp32(rng, M, K)
    announce("linear kq", wtype, M, N, K)
    y = ql.linear_kq(w, to_dev(xf)).cpu().numpy()
    assert rel_l2(y, orc.linear_kq(xf, W, wtype, None, orc.SCALE_X86_REF)) < 2e-6
    yb = ql.linear_kq(w, to_dev(xf), to_dev(bias)).cpu().numpy()
    assert rel_l2(yb, orc.linear_kq(xf, W, wtype, bias, orc.SCALE_X86_REF)) < 2e-6
    bits, xb = synth.make_x_bf16(rng, M, K)
    y2 = ql.linear_kq(w, bf16_dev(bits))
    assert rel_l2(y2.cpu().numpy(), orc.linear_kq(xb, W, wtype, None, orc.SCALE_X86_REF)) < 2e-6
    # with a workspace (x quantized once by its own kernel): the same bits
    ws = ql.kq_workspace(M, K)
    assert torch.equal(ql.linear_kq(w, to_dev(xf), to_dev(bias), workspace=ws), torch.from_numpy(yb).cuda())
    assert torch.equal(ql.linear_kq(w, bf16_dev(bits), workspace=ws), y2)


@pytest.mark.parametrize("wtype", [2, 3])
@pytest.mark.parametrize("M", [1, 4, 8, 13])
def test_linear_kq_multi_equals_single(wtype, M):
    """sibling projections in one launch: per part the bits of the single launch"""
    rng = synth.rng_for(7, 300 + wtype * 10 + M)
    K = 1280
    Ns = [96, 33, 200, 8]
    Ws = [synth.make_weight(rng, wtype, n, K) for n in Ns]
    ws = [ql.PackedKWeight(wtype, torch.from_numpy(W)) for W in Ws]
    biases = [to_dev(rng.standard_normal(n).astype(np.float32)) if i % 2 == 0 else None for i, n in enumerate(Ns)]
    x = to_dev(synth.make_x_fp32(rng, M, K))
    announce("kq multi", wtype, M)
    wsp = ql.kq_workspace(M, K)
    for nparts in (2, 4):
        outs = ql.linear_kq_multi(ws[:nparts], x, biases[:nparts], workspace=wsp if M % 2 else None)
        for w, b, o in zip(ws, biases, outs):
            assert torch.equal(o, ql.linear_kq(w, x, b))


@pytest.mark.parametrize("wtype", [2, 3])
def test_linear_kq_exact_cases(wtype):
    """unit scales and integer activations that quantize to themselves: every product is an integer below 2^24, so the
    result must equal the integer matrix product exactly"""
    rng = synth.rng_for(7, 50 + wtype)
    N, K, M = 64, 512, 4
    W = synth.make_weight(rng, wtype, N, K)
    if wtype == 2:
        W[:, :, 0:2] = np.array([0x00, 0x3c], np.uint8)
        W[:, :, 2:4] = np.array([0x00, 0x3c], np.uint8)
    else:
        W[:, :, 208:210] = np.array([0x00, 0x3c], np.uint8)
        W[:, :, 192:208] = rng.integers(-3, 4, size=(N, K // 256, 16)).astype(np.int8).view(np.uint8)
    x = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    x[:, ::256] = -128.0  # max = -128 -> iscale = 1, d = 1: codes equal the values
    wd = orc.dequantize_k(W, wtype, orc.SCALE_IEEE).astype(np.float64)
    want = x.astype(np.float64) @ wd.T
    assert np.abs(want).max() < 2 ** 24
    announce("linear kq exact", wtype)
    y = ql.linear_kq(ql.PackedKWeight(wtype, torch.from_numpy(W)), to_dev(x)).cpu().numpy()
    assert np.array_equal(y.astype(np.float64), want)


@pytest.mark.parametrize("wtype", [2, 3])
@pytest.mark.parametrize("M,N,K", [(9, 100, 256), (64, 257, 768), (130, 512, 2560), (33, 31, 512), (300, 96, 9728), (512, 300, 1024)])
def test_linear_kq_gemm(wtype, M, N, K):
    """many rows on the matrix cores (fp16 operands with folded scales) against the oracle's integer / fp32 arithmetic"""
    rng = synth.rng_for(7, 700 + wtype * 1000 + M * 13 + N)
    W = synth.make_weight(rng, wtype, N, K)
    wg = ql.PackedKWeight(wtype, torch.from_numpy(W), layout="gemm")
    bias = rng.standard_normal(N).astype(np.float32)
    xf = synth.make_x_fp32(rng, M, K)
    announce("linear kq gemm", wtype, M, N, K)
    want = orc.linear_kq(xf, W, wtype, bias, orc.SCALE_X86_REF)
    y = ql.linear_kq_gemm(wg, to_dev(xf), to_dev(bias)).cpu().numpy()
    err = rel_l2(y, want)
    print("rel-L2 %.2e" % err)
    assert err < TOL
    bits, xb = synth.make_x_bf16(rng, M, K)
    y2 = ql.linear_kq_gemm(wg, bf16_dev(bits)).cpu().numpy()
    assert rel_l2(y2, orc.linear_kq(xb, W, wtype, None, orc.SCALE_X86_REF)) < TOL
    ys = ql.linear_kq_gemm(wg, to_dev(xf), to_dev(bias), short=True).cpu().numpy()  # K ranges as separate workgroups
    assert rel_l2(ys, y) < 2e-6
    # and against the GEMV path (the reference arithmetic itself) on the same device
    yv = ql.linear_kq(ql.PackedKWeight(wtype, torch.from_numpy(W)), to_dev(xf), to_dev(bias)).cpu().numpy()
    assert rel_l2(y, yv) < TOL


@pytest.mark.parametrize("wtype", [2, 3])
def test_linear_kq_gemm_exact_cases(wtype):
    """unit scales, small integer sub-block scales and integer activations that quantize to themselves: every operand is
    an integer that fp16 holds exactly and every partial sum stays below 2^24, so the result must equal the integer
    matrix product exactly (a misplaced code, scale or offset in the packed layout cannot pass)"""
    rng = synth.rng_for(7, 60 + wtype)
    N, K, M = 70, 768, 37
    W = synth.make_weight(rng, wtype, N, K)
    if wtype == 2:
        W[:, :, 0:2] = np.array([0x00, 0x3c], np.uint8)
        W[:, :, 2:4] = np.array([0x00, 0x3c], np.uint8)
    else:
        W[:, :, 208:210] = np.array([0x00, 0x3c], np.uint8)
        W[:, :, 192:208] = rng.integers(-3, 4, size=(N, K // 256, 16)).astype(np.int8).view(np.uint8)
    x = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    x[:, ::256] = -128.0  # max = -128 -> iscale = 1, d = 1: codes equal the values
    wd = orc.dequantize_k(W, wtype, orc.SCALE_IEEE).astype(np.float64)
    assert np.abs(wd).max() <= 2048
    want = x.astype(np.float64) @ wd.T
    assert (np.abs(x).astype(np.float64) @ np.abs(wd).T).max() < 2 ** 24
    announce("linear kq gemm exact", wtype)
    y = ql.linear_kq_gemm(ql.PackedKWeight(wtype, torch.from_numpy(W), layout="gemm"), to_dev(x)).cpu().numpy()
    assert np.array_equal(y.astype(np.float64), want)


@pytest.mark.parametrize("wtype", [2, 3])
@pytest.mark.parametrize("M", [3, 4, 5, 8, 11])
def test_matrix_core_and_dot4_kernels_agree(wtype, M):
    """three to eight rows: the matrix-core kernels (default) and the dot4 kernel are independent implementations of the same
    arithmetic (exact integer sums, fp32 scaling in another order)"""
    rng = synth.rng_for(7, 900 + M + 100 * wtype)
    L = _lib.lib()
    for N, K in ((9728, 2560), (2560, 9728), (77, 768), (130, 4096 + 256), (33, 256)):
        W = synth.make_weight(rng, wtype, N, K)
        w = ql.PackedKWeight(wtype, torch.from_numpy(W))
        bias = to_dev(rng.standard_normal(N).astype(np.float32))
        xf = synth.make_x_fp32(rng, M, K)
        xd = to_dev(xf)
        announce("kq both kernels", wtype, M, N, K)
        assert L.mllm_hip_kq_set_path(2) == 0  # the matrix-core kernel also where the default keeps the dot4 kernel
        try:
            y0 = ql.linear_kq(w, xd, bias)
            assert torch.equal(y0, ql.linear_kq(w, xd, bias, workspace=ql.kq_workspace(M, K)))
            assert L.mllm_hip_kq_set_path(1) == 0
            y1 = ql.linear_kq(w, xd, bias)
        finally:
            assert L.mllm_hip_kq_set_path(0) == 0
        yd = ql.linear_kq(w, xd, bias)  # whatever the default picks per group of eight rows: one of the two, bit for bit
        for lo in range(0, M, 8):
            assert torch.equal(yd[lo:lo + 8], y0[lo:lo + 8]) or torch.equal(yd[lo:lo + 8], y1[lo:lo + 8])
        assert rel_l2(y0.cpu().numpy(), y1.cpu().numpy()) < 2e-6
        assert rel_l2(y0.cpu().numpy(), orc.linear_kq(xf, W, wtype, bias.cpu().numpy(), orc.SCALE_X86_REF)) < 2e-6
    assert L.mllm_hip_kq_set_path(3) == -1


@pytest.mark.parametrize("wtype", [2, 3])
@pytest.mark.parametrize("M", [3, 4, 7, 8, 19])
def test_k_slices_that_meet_in_the_workspace_give_the_same_bits(wtype, M):
    """a workspace with room for partial sums: rows of more than 2560 elements are cut into K slices with a workgroup each, which
    quantize their own part of x and meet through arrival counters; the sum runs in slice order as in the one-workgroup form.
    Ragged N, several parts, bias, fp32 and bf16 activations, every workgroup shape, the workspace used again and again."""
    rng = synth.rng_for(7, 1300 + M + 50 * wtype)
    L = _lib.lib()
    for Ns, K in (((2560,), 9728), ((2560,), 4096), ((77, 130), 4096 + 256), ((33, 16, 50, 200), 3072), ((700, 90), 2560), ((40,), 256)):
        ws = [ql.PackedKWeight(wtype, torch.from_numpy(synth.make_weight(rng, wtype, N, K))) for N in Ns]
        biases = [to_dev(rng.standard_normal(N).astype(np.float32)) if i % 2 == 0 else None for i, N in enumerate(Ns)]
        xf = synth.make_x_fp32(rng, M, K)
        for x in (to_dev(xf), to_dev(xf).to(torch.bfloat16)):
            announce("kq slices meet", wtype, M, Ns, K, x.dtype)
            want = ql.linear_kq_multi(ws, x, biases)                                        # no workspace
            small = ql.linear_kq_multi(ws, x, biases, workspace=ql.kq_workspace(M, K))       # image only
            room = ql.kq_workspace(M, K, sum(Ns))
            assert room.numel() >= ql.kq_workspace(M, K).numel()
            try:
                for mode, waves in ((-1, 0), (-1, 0), (1, 0), (1, 1), (1, 3), (-1, 5), (1, 8), (0, 0)):
                    assert L.mllm_hip_kq_set_slice_meeting(mode, waves) == 0
                    got = ql.linear_kq_multi(ws, x, biases, workspace=room)
                    for a, b, c in zip(want, small, got):
                        assert torch.equal(a, b) and torch.equal(a, c), (mode, waves)
            finally:
                assert L.mllm_hip_kq_set_slice_meeting(-1, 0) == 0
            assert L.mllm_hip_gemv_workspace_release(room.data_ptr()) == 0
    assert L.mllm_hip_kq_set_slice_meeting(2, 0) == -1 and L.mllm_hip_kq_set_slice_meeting(0, 9) == -1
    # a workspace smaller than the image is an error, stated size or not
    p = ws[0].ptr
    part = (_lib.GemvPart * 1)(_lib.GemvPart(p, None, want[0].data_ptr(), 40))
    assert L.mllm_hip_linear_kq_multi_ws(wtype, 1, part, x.data_ptr(), ql._xdtype(x), M, 256, room.data_ptr(), 16, None) == -1


@pytest.mark.parametrize("wtype", [2, 3])
def test_units_in_flight_do_not_change_the_bits(wtype):
    """one or two rows: a lane adds its units in the same order whether the row is requested whole before the quantization of
    x (the default for Q4_K rows of up to 96 / 128 units) or trip by trip (mllm_hip_kq_set_tuning with units in flight)"""
    rng = synth.rng_for(7, 1500 + wtype)
    L = _lib.lib()
    for M in (1, 2):
        for N, K in ((1000, 2560), (300, 4096), (70, 768), (2560, 2560 + 512)):
            w = ql.PackedKWeight(wtype, torch.from_numpy(synth.make_weight(rng, wtype, N, K)))
            x = to_dev(synth.make_x_fp32(rng, M, K)).to(torch.bfloat16)
            announce("kq units in flight", wtype, M, N, K)
            want = ql.linear_kq(w, x)
            try:
                for u in (1, 2, 4):
                    assert L.mllm_hip_kq_set_tuning(0, 0, u) == 0
                    assert torch.equal(want, ql.linear_kq(w, x)), u
            finally:
                assert L.mllm_hip_kq_set_tuning(0, 0, 0) == 0


def test_argument_checks():
    L = _lib.lib()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p = buf.data_ptr()
    assert L.mllm_hip_kq_packed_bytes(2, 4, 100) == 0
    assert L.mllm_hip_kq_packed_bytes(0, 4, 256) == 0
    assert L.mllm_hip_linear_kq(2, p, p, 0, None, p, 1, 4, 100, None, None) == -2
    assert L.mllm_hip_linear_kq(1, p, p, 0, None, p, 1, 4, 256, None, None) == -1
    assert L.mllm_hip_linear_kq(2, p + 16, p, 0, None, p, 1, 4, 256, None, None) == -3
    assert L.mllm_hip_kq_prepack(3, None, 0, p, 4, 256, None) == -1
    assert L.mllm_hip_quantize_q8_K(p, 0, p, p, p, 1, 100, None) == -2
    assert L.mllm_hip_kq_gemm_packed_bytes(2, 4, 100) == 0
    assert L.mllm_hip_kq_gemm_packed_bytes(1, 4, 256) == 0
    assert L.mllm_hip_kq_gemm_packed_bytes(2, 33, 256) == 64 * 256 // 2 + 64 * 4 * 8
    assert L.mllm_hip_linear_kq_gemm(2, p, p, 0, None, p, 16, 4, 100, p, None) == -2
    assert L.mllm_hip_linear_kq_gemm(0, p, p, 0, None, p, 16, 4, 256, p, None) == -1
    assert L.mllm_hip_linear_kq_gemm(2, p, p, 0, None, p, 16, 4, 256, None, None) == -1


@pytest.mark.parametrize("name,wtype", [("q4_k", 2), ("q6_k", 3)])
def test_golden_kquant(golden_dir, name, wtype):
    """against what the compiled reference produced on blocks written by its own offline quantizers"""
    import os
    g = np.load(os.path.join(golden_dir, "kquant_kat.npz"))
    announce("golden kquant", name)
    w = ql.PackedKWeight(wtype, torch.from_numpy(g[f"{name}_W"]))
    assert np.array_equal(w.dequantize().cpu().numpy().view(np.uint32), g[f"{name}_deq"].view(np.uint32))
    for M in (1, 3, 8):
        y = ql.linear_kq(w, to_dev(g[f"{name}_x{M}"]), to_dev(g[f"{name}_bias"])).cpu().numpy()
        assert rel_l2(y, g[f"{name}_y{M}"]) < 1e-5
    q, d, bs = ql.quantize_q8_K(to_dev(g["q8k_x"]))
    assert np.array_equal(q.cpu().numpy(), g["q8k_q"]) and np.array_equal(d.cpu().numpy().view(np.uint32), g["q8k_d"].view(np.uint32))
    assert np.array_equal(bs.cpu().numpy(), g["q8k_bsums"])


@pytest.mark.parametrize("wtype,T,H,I,E,k", [(2, 1, 2048, 768, 16, 8), (3, 1, 2048, 768, 16, 8), (2, 5, 512, 256, 6, 3), (3, 9, 256, 512, 4, 2),
                                            (2, 8, 2048, 768, 128, 8)])
def test_moe_ffn_with_k_quant_experts(wtype, T, H, I, E, k):
    """Q4_K / Q6_K experts (Qwen3-30B-A3B dimensions included): every (token, expert) pair one K-quant GEMV row, SiLU and product,
    down GEMV, weighted sum in slot order, against the oracle's composition of the same Linears; slots with an expert id
    outside [0, E) add nothing; permuting tokens permutes outputs bit for bit; bf16 activations"""
    rng = synth.rng_for(9, 7000 + wtype + T + H + I + E)
    Wg = synth.make_weight(rng, wtype, E * I, H).reshape(E, I, H // 256, -1)
    Wu = synth.make_weight(rng, wtype, E * I, H).reshape(E, I, H // 256, -1)
    Wd = synth.make_weight(rng, wtype, E * H, I).reshape(E, H, I // 256, -1)
    ids, w = synth.make_moe_routing(rng, T, E, k)
    g, u, d = (ql.PackedKExperts(wtype, torch.from_numpy(W)) for W in (Wg, Wu, Wd))
    x = synth.make_x_fp32(rng, T, H)
    announce("moe k-quant", wtype, T, H, I, E, k)
    y = ql.moe_ffn_kq(g, u, d, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
    want = orc.moe_ffn_kq(x, ids, w, Wg, Wu, Wd, wtype)
    assert rel_l2(y, want) < 1e-3, rel_l2(y, want)
    perm = rng.permutation(T)
    y2 = ql.moe_ffn_kq(g, u, d, to_dev(x[perm]), to_dev(ids[perm]), to_dev(w[perm])).cpu().numpy()
    assert np.array_equal(y2, y[perm])
    bad = ids.copy()
    bad[0, 0] = E + 3
    if k > 1:
        bad[T - 1, k - 1] = -1
    y3 = ql.moe_ffn_kq(g, u, d, to_dev(x), to_dev(bad), to_dev(w)).cpu().numpy()
    assert rel_l2(y3, orc.moe_ffn_kq(x, bad, w, Wg, Wu, Wd, wtype)) < 1e-3
    bits, xb = synth.make_x_bf16(rng, T, H)
    y4 = ql.moe_ffn_kq(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
    assert rel_l2(y4, orc.moe_ffn_kq(xb, ids, w, Wg, Wu, Wd, wtype)) < 1e-3


@pytest.mark.parametrize("wtype,T,H,I,E,k", [(2, 40, 512, 256, 6, 3), (3, 33, 256, 512, 4, 2), (2, 96, 2048, 768, 16, 4),
                                            (3, 64, 2048, 768, 8, 2), (2, 9, 256, 256, 3, 1)])
def test_moe_ffn_k_quant_grouped_form_equals_the_pair_form(wtype, T, H, I, E, k):
    """Many pairs per expert: the pairs sorted by expert run as tiles of eight rows on the matrix-core kernels (x and h
    quantized to Q8_K once, tiles gather their rows).  Same arithmetic as one GEMV row per pair (exact integer sums, fp32
    scaling in another order): the two forms agree to 1e-5, both meet the oracle; invalid expert ids add nothing; a permutation
    of the tokens permutes the outputs bit for bit; bf16 activations."""
    rng = synth.rng_for(9, 7100 + wtype + T + H + I + E)
    L = _lib.lib()
    Wg = synth.make_weight(rng, wtype, E * I, H).reshape(E, I, H // 256, -1)
    Wu = synth.make_weight(rng, wtype, E * I, H).reshape(E, I, H // 256, -1)
    Wd = synth.make_weight(rng, wtype, E * H, I).reshape(E, H, I // 256, -1)
    ids, w = synth.make_moe_routing(rng, T, E, k)
    ids[1, 0] = E + 2          # an expert id out of range
    if k > 1:
        ids[T - 1, k - 1] = -1
    g, u, d = (ql.PackedKExperts(wtype, torch.from_numpy(W)) for W in (Wg, Wu, Wd))
    x = synth.make_x_fp32(rng, T, H)
    announce("moe k-quant grouped", wtype, T, H, I, E, k)
    outs = {}
    for path in (1, 2):
        assert L.mllm_hip_moe_kq_set_path(path) == 0
        try:
            outs[path] = ql.moe_ffn_kq(g, u, d, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
            if path == 2:
                perm = rng.permutation(T)
                y2 = ql.moe_ffn_kq(g, u, d, to_dev(x[perm]), to_dev(ids[perm]), to_dev(w[perm])).cpu().numpy()
                bits, xb = synth.make_x_bf16(rng, T, H)
                y4 = ql.moe_ffn_kq(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
        finally:
            assert L.mllm_hip_moe_kq_set_path(0) == 0
    want = orc.moe_ffn_kq(x, ids, w, Wg, Wu, Wd, wtype)
    assert rel_l2(outs[2], want) < 1e-3, rel_l2(outs[2], want)
    assert rel_l2(outs[2], outs[1]) < 1e-5, rel_l2(outs[2], outs[1])
    assert np.array_equal(y2, outs[2][perm])
    assert rel_l2(y4, orc.moe_ffn_kq(xb, ids, w, Wg, Wu, Wd, wtype)) < 1e-3
    assert L.mllm_hip_moe_kq_set_path(4) == -1


@pytest.mark.parametrize("wtype,T,H,I,E,k", [(2, 40, 512, 256, 6, 3), (2, 96, 2048, 768, 16, 4), (2, 200, 1024, 512, 5, 2),
                                            (2, 33, 256, 256, 1, 1), (2, 70, 768, 2048, 9, 4), (2, 300, 256, 512, 64, 8),
                                            (3, 40, 512, 256, 6, 3), (3, 96, 2048, 768, 16, 4), (3, 33, 256, 256, 1, 1),
                                            (3, 70, 768, 2048, 9, 4), ((2, 3), 96, 2048, 768, 16, 4), ((2, 3), 200, 512, 256, 5, 2),
                                            ((3, 2), 64, 256, 512, 4, 2)])
def test_moe_ffn_k_quant_tiles_of_32_rows(wtype, T, H, I, E, k):
    """Four pairs per expert and more: tiles of 32 expert-sorted rows, the weights as the second operand of 32 x 32 matrix
    instructions, integer sub-block sums scaled in int32 (experts with one row, 32, 33 rows, none at all; channel counts that
    end inside a workgroup's 128 or 256).  Same integers as one GEMV row per pair, fp32 scaling in another order: the forms
    agree row by row (see below) and meet the oracle; invalid expert ids add nothing; a permutation of the tokens permutes the outputs bit
    for bit; bf16 activations.  Q6_K: groups of 16 elements on 32 x 32 x 16 instructions, the offset of 32 through the sums
    of 16.  A pair of formats: gate / up in the first, down in the second (the shipped recipe is Q4_K / Q6_K)."""
    wtype, wdown = wtype if isinstance(wtype, tuple) else (wtype, wtype)
    rng = synth.rng_for(9, 7300 + wtype + 5 * wdown + T + H + I + E)
    L = _lib.lib()
    Wg = synth.make_weight(rng, wtype, E * I, H).reshape(E, I, H // 256, -1)
    Wu = synth.make_weight(rng, wtype, E * I, H).reshape(E, I, H // 256, -1)
    Wd = synth.make_weight(rng, wdown, E * H, I).reshape(E, H, I // 256, -1)
    ids, w = synth.make_moe_routing(rng, T, E, k)
    if E > 2:
        ids[1, 0] = E + 2          # an expert id out of range
        if k > 1:
            ids[T - 1, k - 1] = -1
    g, u = (ql.PackedKExperts(wtype, torch.from_numpy(W)) for W in (Wg, Wu))
    d = ql.PackedKExperts(wdown, torch.from_numpy(Wd))
    x = synth.make_x_fp32(rng, T, H)
    announce("moe k-quant tiles of 32 rows", wtype, T, H, I, E, k)
    outs = {}
    for path in (1, 3):
        assert L.mllm_hip_moe_kq_set_path(path) == 0
        try:
            outs[path] = ql.moe_ffn_kq(g, u, d, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
            if path == 3:
                perm = rng.permutation(T)
                y2 = ql.moe_ffn_kq(g, u, d, to_dev(x[perm]), to_dev(ids[perm]), to_dev(w[perm])).cpu().numpy()
                bits, xb = synth.make_x_bf16(rng, T, H)
                y4 = ql.moe_ffn_kq(g, u, d, bf16_dev(bits), to_dev(ids), to_dev(w)).cpu().numpy()
        finally:
            assert L.mllm_hip_moe_kq_set_path(0) == 0
    want = orc.moe_ffn_kq(x, ids, w, Wg, Wu, Wd, wtype, wtype_down=wdown)
    assert rel_l2(outs[3], want) < 1e-3, rel_l2(outs[3], want)
    # row by row against the pair form: the same integers, fp32 sums in another order (about 2e-7); where the last bit of an h
    # value decides a Q8_K code, that one row of the down projection moves by a code step (a few 1e-4 of the row)
    rows = np.linalg.norm(outs[3] - outs[1], axis=1) / np.maximum(np.linalg.norm(outs[1], axis=1), 1e-30)
    assert np.median(rows) < 1e-6 and (rows > 1e-5).mean() <= 0.05 and rel_l2(outs[3], outs[1]) < 2e-4, (np.median(rows), rows.max())
    assert np.array_equal(y2, outs[3][perm])
    assert rel_l2(y4, orc.moe_ffn_kq(xb, ids, w, Wg, Wu, Wd, wtype, wtype_down=wdown)) < 1e-3


def _x86_field_to_pattern(field):
    """what a read on x86 makes of a stored fp16 field: the half-precision number, as an integer"""
    return field.view(np.float16).astype(np.float32).astype(np.uint16)


@pytest.mark.parametrize("wtype", [2, 3])
def test_offline_k_quant_quantizers_byte_exact(wtype, golden_dir):
    """mllm_hip_kq_quantize_weight_blocks against the oracle (pinned byte for byte to the compiled reference quantizers) in both
    storage modes, against the fixture the compiled reference wrote, and through the library's own Linear."""
    import os
    rng = synth.rng_for(7, 300 + wtype)
    N, K = 48, 1024
    w = (rng.standard_normal((N, K)) * 0.04).astype(np.float32)
    w[0, :256] = 0.0
    w[1, :32], w[1, 32:64] = 0.3, -0.3
    w[2, :256] = np.abs(w[2, :256])
    w[3, :512] *= 80
    w[4, :16] = 0.0
    w[5, :256] = np.float32(1e-3) * rng.integers(-8, 8, 256)
    w[6, 0], w[6, 5] = 0.9, -0.9
    w[7, :] = 1e-20                                      # below the all-zero threshold of the Q6_K search, not of the Q4_K one
    announce("offline k-quant quantizer", wtype)
    for mode, omode in ((ql.SCALE_X86_REF, orc.SCALE_X86_REF), (ql.SCALE_IEEE, orc.SCALE_IEEE)):
        got = ql.kq_quantize_weight_blocks(to_dev(w), wtype, mode).cpu().numpy()
        want = orc.quantize_weight_rows_k(w, wtype, omode)
        assert np.array_equal(got, want), (mode, np.argwhere(got != want)[:5])
    # the fixture of the compiled reference: codes and sub-block scales byte for byte, the fp16 fields as an x86 read decodes them
    g = np.load(os.path.join(golden_dir, "kquant_quantizer_kat.npz"))
    ref = g["q4_k_blocks" if wtype == 2 else "q6_k_blocks"]
    gb = ql.kq_quantize_weight_blocks(to_dev(g["w"]), wtype, ql.SCALE_X86_REF).cpu().numpy()
    body = np.ones(gb.shape[2], bool)
    for a, b in ([(0, 2), (2, 4)] if wtype == 2 else [(208, 210)]):
        body[a:b] = False
        assert np.array_equal(_x86_field_to_pattern(gb[:, :, a:b].copy().view(np.uint16)[:, :, 0]), ref[:, :, a:b].copy().view(np.uint16)[:, :, 0])
    assert np.array_equal(gb[:, :, body], ref[:, :, body])
    # quantize -> prepack -> Linear on the GPU equals the oracle's Linear on the oracle's blocks
    blocks = ql.kq_quantize_weight_blocks(to_dev(w), wtype, ql.SCALE_IEEE)
    pw = ql.PackedKWeight(wtype, blocks)
    x = synth.make_x_fp32(rng, 3, K)
    y = ql.linear_kq(pw, to_dev(x)).cpu().numpy()
    assert rel_l2(y, orc.linear_kq(x, orc.quantize_weight_rows_k(w, wtype, orc.SCALE_IEEE), wtype, None, orc.SCALE_IEEE)) < 2e-6
    # and the blocks reproduce the weights to the format's resolution
    deq = pw.dequantize().cpu().numpy()
    assert np.abs(deq - w).max() <= (0.08 if wtype == 2 else 0.05) * np.abs(w).max()
    L = _lib.lib()
    p = blocks.data_ptr()
    assert L.mllm_hip_kq_quantize_weight_blocks(wtype, None, p, 0, 4, 256, None) == -1
    assert L.mllm_hip_kq_quantize_weight_blocks(0, p, p, 0, 4, 256, None) == -1
    assert L.mllm_hip_kq_quantize_weight_blocks(wtype, p, p, 2, 4, 256, None) == -1
    assert L.mllm_hip_kq_quantize_weight_blocks(wtype, p, p, 0, 4, 128, None) == -2
    assert L.mllm_hip_kq_quantize_weight_blocks(wtype, p + 4, p, 0, 4, 256, None) == -3
