"""Pins the oracle without the reference checkout: committed golden vectors (made by tests/golden/make_golden.py from the
reference's compiled kernels) and what the mathematics fixes (closed forms, brute force, special cases)."""
import os

import numpy as np
import pytest

from mllm_amd import synth
from oracle import oracle as orc


def _g(golden_dir, name):
    return np.load(os.path.join(golden_dir, name))


# ------------------------------------------------------------------ golden vectors from the compiled reference
def test_golden_actquant(golden_dir):
    g = _g(golden_dir, "q8_0_actquant.npz")
    qs, d_bits = orc.quantize_rows_q8_0(g["x"])
    assert np.array_equal(qs, g["qs"])
    eff = orc.fp16_bits_to_fp32(orc.x86_scale_bits(d_bits))
    assert np.array_equal(eff.view(np.uint32), g["d_eff"].view(np.uint32))


@pytest.mark.parametrize("wname,wtype", [("q4_0", orc.Q4_0), ("q8_0", orc.Q8_0)])
def test_golden_gemv(golden_dir, wname, wtype):
    g = _g(golden_dir, "gemv_kat.npz")
    W, bias = g[f"{wname}_W"], g[f"{wname}_bias"]
    for M in (1, 3, 4, 8):
        x = g[f"{wname}_x{M}"]
        y = orc.linear_q(x, W, wtype, None, orc.SCALE_X86_REF)
        assert np.array_equal(y.view(np.uint32), g[f"{wname}_y{M}"].view(np.uint32))
        yb = orc.linear_q(x, W, wtype, bias, orc.SCALE_X86_REF)
        assert np.array_equal(yb.view(np.uint32), g[f"{wname}_yb{M}"].view(np.uint32))
        # the IEEE reading of the activation scale is a different function: it must NOT reproduce the x86 vectors
        yi = orc.linear_q(x, W, wtype, None, orc.SCALE_IEEE)
        rel = np.linalg.norm(yi - y) / np.linalg.norm(y)
        assert 1e-5 < rel < 1e-2


def test_golden_x86_scale_grid(golden_dir):
    g = _g(golden_dir, "x86_scale_grid.npz")
    eff = orc.x86_scale_bits(g["bits"])
    got = orc.fp16_bits_to_fp32(eff).view(np.uint32)
    want = g["value_bits"]
    nan = np.isnan(want.view(np.float32))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(got.view(np.float32)[nan]).all()
    # the numpy generator-side snap is the same function
    assert np.array_equal(synth.snap_scale_bits(g["bits"]), eff)


def test_golden_dequant(golden_dir):
    g = _g(golden_dir, "dequant_kat.npz")
    assert np.array_equal(orc.dequantize(g["W4"], orc.Q4_0, orc.SCALE_X86_REF), g["y4"])
    assert np.array_equal(orc.dequantize(g["W8"], orc.Q8_0, orc.SCALE_X86_REF), g["y8"])
    # snapped scales: both readings agree
    assert np.array_equal(orc.dequantize(g["W4"], orc.Q4_0, orc.SCALE_IEEE), g["y4"])


# ------------------------------------------------------------------ fp16 / bf16 conversions vs numpy
def test_golden_weight_quantizers(golden_dir):
    """offline quantizers against vectors written by the reference's own quantize_row_q4_0 / quantize_row_q8_0"""
    g = np.load(os.path.join(golden_dir, "weight_quantizer_kat.npz"))
    w = g["w"]

    def pattern(field):  # an x86 read of the stored field: the half-precision number as an integer
        return field.view(np.float16).astype(np.float32).astype(np.uint16)
    got = orc.quantize_weight_rows(w, orc.Q4_0, orc.SCALE_X86_REF)
    assert np.array_equal(got[:, :, 2:], g["q4_blocks"][:, :, 2:])
    assert np.array_equal(pattern(got[:, :, 0:2].copy().view(np.uint16)[:, :, 0]), g["q4_blocks"][:, :, 0:2].copy().view(np.uint16)[:, :, 0])
    got8 = orc.quantize_weight_rows(w, orc.Q8_0, orc.SCALE_X86_REF)
    assert np.array_equal(got8[:, :, 2:].view(np.int8).reshape(w.shape[0], -1), g["q8_codes"])
    pat8 = pattern(got8[:, :, 0:2].copy().view(np.uint16)[:, :, 0])
    assert np.array_equal(pat8.view(np.float16).astype(np.float32).view(np.uint32), g["q8_d_eff"].view(np.uint32))


def test_fp16_vs_numpy():
    L = orc.lib()
    allb = np.arange(65536, dtype=np.uint16)
    want = allb.view(np.float16).astype(np.float32)
    got = np.array([L.orc_fp16_to_fp32(int(b)) for b in allb], dtype=np.float32)
    ok = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert ok.all()
    rng = np.random.default_rng(0)
    halves = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = ((halves[:-1] + halves[1:]) / 2).astype(np.float32)  # exact ties
    s = np.concatenate([mids, np.nextafter(mids, np.float32(1e9)), np.nextafter(mids, np.float32(0)),
                        (rng.standard_normal(30000) * 0.02).astype(np.float32),
                        np.float32([0, 65504, 65519.996, 65520, 7e4, 1e-8, 2.9802322e-8, 3e-8, 6e-8])])
    s = np.concatenate([s, -s])
    with np.errstate(over="ignore"):
        want = s.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_fp32_to_fp16(float(f)) for f in s], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16_vs_numpy():
    L = orc.lib()
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32),
                        np.float32([1.00390625, 1.01171875, 1.0, 3.3895314e38])])  # ties up/down
    got = np.array([L.orc_fp32_to_bf16(float(f)) for f in x], dtype=np.uint16)
    assert np.array_equal(got, synth.fp32_to_bf16_bits(x))
    import torch
    assert np.array_equal(got.view(np.int16), torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy())


# ------------------------------------------------------------------ Q8_0 activation quantisation: closed form + invariants
def test_actquant_closed_form_and_invariants():
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((16, 1024)) * rng.uniform(0.01, 30, (16, 1))).astype(np.float32)
    x[3, 64:96] = 0
    qs, d = orc.quantize_rows_q8_0(x)
    xb = x.reshape(16, -1, 32)
    amax = np.abs(xb).max(axis=2)
    with np.errstate(divide="ignore", invalid="ignore"):
        idv = np.where(amax != 0, np.float32(127) / amax, np.float32(0)).astype(np.float32)
    want = np.rint(xb * idv[:, :, None]).astype(np.int32).clip(-128, 127).astype(np.int8).reshape(16, -1)
    assert np.array_equal(qs, want)
    assert np.array_equal(d, (amax / np.float32(127)).astype(np.float32).astype(np.float16).view(np.uint16))
    assert np.abs(qs.astype(np.int32)).max() <= 127
    assert (qs[3, 64:96] == 0).all() and d[3, 2] == 0
    # the element carrying amax maps to +-127
    idx = np.abs(xb).argmax(axis=2)
    top = np.take_along_axis(qs.reshape(16, -1, 32), idx[:, :, None], axis=2)[:, :, 0]
    assert (np.abs(top.astype(np.int32))[amax > 0] == 127).all()
    # odd symmetry
    qn, dn = orc.quantize_rows_q8_0(-x)
    assert np.array_equal(qn, -qs) and np.array_equal(dn, d)


# ------------------------------------------------------------------ block dot products: brute force
@pytest.mark.parametrize("wtype", [orc.Q4_0, orc.Q8_0])
def test_linear_vs_double_brute_force(wtype):
    rng = np.random.default_rng(4)
    N, K, M = 40, 512, 5
    W = synth.make_weight(rng, wtype, N, K)
    x = synth.make_x_fp32(rng, M, K)
    bias = rng.standard_normal(N).astype(np.float32)
    for mode in (orc.SCALE_IEEE, orc.SCALE_X86_REF):
        y, xq, xd = orc.linear_q(x, W, wtype, bias, mode, return_xq=True)
        xdb = orc.x86_scale_bits(xd) if mode == orc.SCALE_X86_REF else xd
        xdeq = (xq.reshape(M, -1, 32).astype(np.float64) * orc.fp16_bits_to_fp32(xdb).astype(np.float64)[:, :, None])
        wdeq = orc.dequantize(W, wtype, mode).astype(np.float64)
        want = xdeq.reshape(M, K) @ wdeq.T + bias
        assert np.abs(y - want).max() <= 2e-6 * np.abs(want).max() + 1e-6
    # int32 block sums against int64 numpy
    codes = (wdeq / orc.fp16_bits_to_fp32(W[:, :, 0:2].copy().view(np.uint16)[:, :, 0]).repeat(32, axis=1))
    codes = np.rint(codes).astype(np.int64).reshape(N, -1, 32)
    want_i = np.einsum("nbj,mbj->nmb", codes, xq.reshape(M, -1, 32).astype(np.int64))
    assert np.array_equal(orc.block_isums(W, wtype, xq).astype(np.int64), want_i)


def test_q4_0_nibble_order():
    """element j = low nibble of qs[j], element j+16 = high nibble (quantize_q4.cpp:85-90)."""
    blk = np.zeros((1, 1, 18), np.uint8)
    blk[0, 0, 0:2] = np.array([0x3c00], dtype="<u2").view(np.uint8)  # d = 1.0
    blk[0, 0, 2:] = np.arange(16, dtype=np.uint8) | ((15 - np.arange(16, dtype=np.uint8)) << 4)
    y = orc.dequantize(blk, orc.Q4_0)[0]
    assert np.array_equal(y[:16], np.arange(16) - 8) and np.array_equal(y[16:], (15 - np.arange(16)) - 8)


# ------------------------------------------------------------------ W4A16
def test_w4a16_dequant_table_exhaustive():
    # every (q, zp) pair against a spread of scales, one group per row
    s_bits = np.float16([0.01, 0.0123, 1.0, 3.14e-3, 6.1e-5, 2.5]).view(np.uint16)
    rows = []
    for zp in range(16):
        for si in range(len(s_bits)):
            rows.append((zp, si))
    N, K = len(rows), 128
    q = np.tile(np.arange(16, dtype=np.uint8), (N, 8))
    z = np.array([[r[0]] for r in rows], dtype=np.uint8)
    s = np.array([[s_bits[r[1]]] for r in rows], dtype=np.uint16)
    w = orc.w4a16_dequant(synth.pack_nibbles(q), s, synth.pack_nibbles(z))
    want = (q.astype(np.float32) - z.astype(np.float32)) * s.view(np.float16).astype(np.float32)
    assert np.array_equal(w, synth.fp32_to_bf16_bits(want))


def test_w4a16_gemm_vs_float64():
    rng = np.random.default_rng(6)
    M, N, K = 9, 24, 384
    qw, s, zp, q, z = synth.make_w4a16(rng, N, K)
    a_bits, a = synth.make_x_bf16(rng, M, K)
    bias = synth.fp32_to_bf16_bits(rng.standard_normal(N).astype(np.float32))
    w = synth.bf16_bits_to_fp32(orc.w4a16_dequant(qw, s, zp)).astype(np.float64)
    for b in (None, bias):
        c = orc.w4a16_gemm(a_bits, qw, s, zp, b)
        want = (a.astype(np.float64) @ w.T).astype(np.float32)
        if b is not None:
            want = want + synth.bf16_bits_to_fp32(b)
        wb = synth.fp32_to_bf16_bits(want)
        diff = np.abs(c.astype(np.int32) - wb.astype(np.int32))
        assert diff.max() <= 1 and (diff == 0).mean() > 0.99
    # zero-point equal to the code everywhere -> exact zeros; scale 1, zp 0 -> plain integer matmul
    qz = np.repeat(z, 128, axis=1)
    c0 = orc.w4a16_gemm(a_bits, synth.pack_nibbles(qz), s, zp)
    assert (synth.bf16_bits_to_fp32(c0) == 0).all()


# ------------------------------------------------------------------ W8A8
def test_per_token_quant_closed_form():
    rng = np.random.default_rng(7)
    a_bits, _, _ = synth.make_w8a8(rng, 33, 8, 512)
    x = synth.bf16_bits_to_fp32(a_bits)
    x[5] = 0
    x[6, :] = np.float32(0.5) * np.arange(512, dtype=np.float32) / 2  # many exact ties once scaled
    q, s = orc.per_token_quant_int8(x)
    absmax = np.maximum(np.abs(x).max(axis=1), np.float32(1e-10)).astype(np.float32)
    sc = (absmax / np.float32(127.0)).astype(np.float32)
    want = np.rint((x / sc[:, None]).astype(np.float32)).clip(-128, 127).astype(np.int8)
    assert np.array_equal(s, sc) and np.array_equal(q, want)
    assert (q[5] == 0).all() and s[5] == np.float32(1e-10) / np.float32(127)
    import torch
    xt = torch.from_numpy(x)
    am = torch.clamp(xt.abs().amax(dim=-1, keepdim=True), min=1e-10)
    ts = am / 127.0
    tq = torch.round(xt / ts).clamp(-128, 127).to(torch.int8)
    assert np.array_equal(q, tq.numpy()) and np.array_equal(s, ts[:, 0].numpy())


@pytest.mark.parametrize("M,N,K", [(1, 64, 32), (8, 128, 64), (16, 96, 2048), (33, 40, 6144)])
def test_w8a8_gemm_exact(M, N, K):
    rng = np.random.default_rng(8)
    xq = rng.integers(-127, 128, (M, K), dtype=np.int8)
    W = rng.integers(-127, 128, (N, K), dtype=np.int8)
    xs = ((rng.random(M) + 0.01) * 0.01).astype(np.float32)
    ws = ((rng.random(N) + 0.01) * 0.01).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.01).astype(np.float32)
    acc, y = orc.w8a8_gemm(xq, xs, W, ws, bias)
    want = xq.astype(np.int64) @ W.astype(np.int64).T
    assert np.array_equal(acc.astype(np.int64), want)
    e = (want.astype(np.float32) * (ws[None, :] * xs[:, None])).astype(np.float32) + bias[None, :]
    assert np.array_equal(y, synth.fp32_to_bf16_bits(e))
    # worst case magnitude stays inside int32
    acc2, _ = orc.w8a8_gemm(np.full((1, K), 127, np.int8), xs[:1], np.full((1, K), -127, np.int8), ws[:1])
    assert acc2[0, 0] == -127 * 127 * K


# ------------------------------------------------------------------ MoE
def test_moe_composition_and_invariance():
    rng = np.random.default_rng(9)
    T, H, I, E, k = 16, 64, 32, 4, 2
    Wg, Wu, Wd = synth.make_moe_weights(rng, E, H, I)
    x = synth.make_x_fp32(rng, T, H)
    ids, w = synth.make_moe_routing(rng, T, E, k)
    y = orc.moe_ffn(x, ids, w, Wg, Wu, Wd, orc.Q4_0)
    assert sum((ids == e).sum() for e in range(E)) == T * k
    # token-at-a-time composition (expert batches of one row): row order inside an expert must not matter
    want = np.zeros((T, H), np.float32)
    for t in range(T):
        acc = np.zeros(H, np.float32)
        for j in range(k):
            e = ids[t, j]
            g = orc.linear_q(x[t:t + 1], Wg[e], orc.Q4_0)
            u = orc.linear_q(x[t:t + 1], Wu[e], orc.Q4_0)
            h = orc.silu(g) * u  # the SiLU operator as the x86 build computes it (pinned in test_oracle_layer_ops.py)
            o = orc.linear_q(h, Wd[e], orc.Q4_0)
            acc = acc + o[0] * w[t, j]
        want[t] = acc
    assert np.abs(y - want).max() <= 1e-5 * np.abs(want).max()
    # permuting tokens permutes outputs
    perm = rng.permutation(T)
    y2 = orc.moe_ffn(x[perm], ids[perm], w[perm], Wg, Wu, Wd, orc.Q4_0)
    assert np.array_equal(y2, y[perm])
    # silu special values
    L = orc.lib()
    assert L.orc_silu(0.0) == 0.0 and abs(L.orc_silu(20.0) - 20.0) < 1e-6 and abs(L.orc_silu(-20.0)) < 1e-7


@pytest.mark.parametrize("name,wtype", [("q4_k", 2), ("q6_k", 3)])
def test_golden_kquant(golden_dir, name, wtype):
    """blocks written by the reference's offline quantizers, dequantized values, Q8_K activation quantization and Linear
    outputs as the compiled reference produced them (tests/golden/make_golden.py, kquant)"""
    g = np.load(os.path.join(golden_dir, "kquant_kat.npz"))
    W = g[f"{name}_W"]
    assert np.array_equal(orc.dequantize_k(W, wtype, orc.SCALE_X86_REF).view(np.uint32), g[f"{name}_deq"].view(np.uint32))
    for M in (1, 3, 8):
        y = orc.linear_kq(g[f"{name}_x{M}"], W, wtype, g[f"{name}_bias"], orc.SCALE_X86_REF)
        assert np.array_equal(y.view(np.uint32), g[f"{name}_y{M}"].view(np.uint32))
    q, d, bs = orc.quantize_rows_q8_K(g["q8k_x"])
    assert np.array_equal(q, g["q8k_q"]) and np.array_equal(d.view(np.uint32), g["q8k_d"].view(np.uint32))
    assert np.array_equal(bs, g["q8k_bsums"])


@pytest.mark.parametrize("name,wtype", [("q4_k", 2), ("q6_k", 3)])
def test_golden_kquant_quantizers(golden_dir, name, wtype):
    """the offline Q4_K / Q6_K quantizers against super-blocks the compiled reference wrote (make_golden.py, kquant_quantizer)"""
    g = np.load(os.path.join(golden_dir, "kquant_quantizer_kat.npz"))
    ref = g[f"{name}_blocks"]
    got = orc.quantize_weight_rows_k(g["w"], wtype, orc.SCALE_X86_REF)
    body = np.ones(got.shape[2], bool)
    for a, b in ([(0, 2), (2, 4)] if wtype == 2 else [(208, 210)]):
        body[a:b] = False
        pat = got[:, :, a:b].copy().view(np.uint16)[:, :, 0].view(np.float16).astype(np.float32).astype(np.uint16)  # an x86 read
        assert np.array_equal(pat, ref[:, :, a:b].copy().view(np.uint16)[:, :, 0])
    assert np.array_equal(got[:, :, body], ref[:, :, body])


@pytest.mark.parametrize("wtype", [0, 1])
def test_avx2_tile_form_equals_the_scalar_restatement_bit_for_bit(wtype):
    """orc_linear_q_tiles (the vector instructions, tile shapes and job split of tinyBLAS_Q0_AVX, llamafile_sgemm.cpp:579-790)
    against orc_linear_q (scalar, pinned against the compiled vec_dot_* of the reference): every output goes through the same
    eight lanes, fused multiply-adds and horizontal sum, so the bits must agree for every tile shape of mnpack (rows 1..9
    exercise 4x2, 2x4, 3x2, 2x3, 4x1, ... down to 1x1 with ragged edges), with and without bias, for any thread count."""
    from mllm_amd import synth
    from oracle import oracle as orc
    rng = synth.rng_for(2, 800 + wtype)
    for M, N, K in [(1, 64, 256), (2, 37, 96), (3, 50, 64), (4, 33, 128), (5, 7, 32), (7, 130, 160), (9, 23, 96)]:
        W = synth.make_weight(rng, wtype, N, K)
        x = synth.make_x_fp32(rng, M, K)
        bias = rng.standard_normal(N).astype(np.float32)
        for mode in (orc.SCALE_X86_REF, orc.SCALE_IEEE):
            want = orc.linear_q(x, W, wtype, None, mode)
            for threads in (1, 3, 8):
                got = orc.linear_q_tiles(x, W, wtype, None, mode, threads)
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (M, N, K, mode, threads)
        wb = orc.linear_q(x, W, wtype, bias, orc.SCALE_X86_REF)
        assert np.array_equal(orc.linear_q_tiles(x, W, wtype, bias, orc.SCALE_X86_REF, 4).view(np.uint32), wb.view(np.uint32))


def test_awq_checkpoint_order_known_answer_and_round_trip():
    """A dword whose nibble p holds the value p: the reference reads column c of the run from nibble (0, 4, 1, 5, 2, 6, 3, 7)[c]
    (mllm-kernel/mllm_kernel/cuda/csrc/gemm/marlin/awq_marlin_repack.cuh:108-110), so the columns read 0 4 1 5 2 6 3 7."""
    one = np.array([[0x76543210]], np.uint32).view(np.int32)
    assert orc.awq_unpack_cols(one).tolist() == [[0, 4, 1, 5, 2, 6, 3, 7]]
    # second dword of a row = columns 8..15; value 0xF in nibble 1 only -> column 2 of that run
    two = np.array([[0, 0x000000F0]], np.uint32).view(np.int32)
    assert np.flatnonzero(orc.awq_unpack_cols(two)[0]).tolist() == [10]
    rng = synth.rng_for(2, 77)
    qweight, qzeros, scales, q, z, s = synth.make_awq(rng, 24, 384, 128)
    qw, s2, zp = orc.awq_unpack(qweight, qzeros, scales)
    assert np.array_equal(qw, synth.pack_nibbles(q)) and np.array_equal(zp, synth.pack_nibbles(z)) and np.array_equal(s2, s)
