"""Pins oracle/qlinear_oracle.c against the reference's own compiled kernels (oracle/_ref).

Skipped where oracle/_ref was not built (it needs the reference checkout); tests/test_oracle_golden.py covers the same
ground from committed fixtures there.
"""
import numpy as np
import pytest

from mllm_amd import synth
from oracle import oracle as orc

pytestmark = pytest.mark.skipif(not orc.ref_available(), reason="oracle/_ref not built (reference checkout absent)")


def test_fp16_conversions_match_reference_macros():
    L, R = orc.lib(), orc.ref()
    for b in range(65536):
        a, r = np.float32(L.orc_fp16_to_fp32(b)), np.float32(R.ref_fp16_bits_to_fp32(b))
        assert a.view(np.uint32) == r.view(np.uint32) or (np.isnan(a) and np.isnan(r)), hex(b)
    rng = np.random.default_rng(1)
    halves = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mids = (halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2
    samples = np.concatenate([halves, mids.astype(np.float32), np.nextafter(mids.astype(np.float32), np.float32(1e9)),
                              np.nextafter(mids.astype(np.float32), np.float32(-1e9)),
                              rng.standard_normal(20000).astype(np.float32) * np.float32(0.01),
                              np.float32([65504, 65519.99, 65520, 1e6, 3e-8, 2.9802322e-8, 2.98e-8, 0.0])])
    samples = np.concatenate([samples, -samples])
    for f in samples[::3]:
        assert L.orc_fp32_to_fp16(float(f)) == R.ref_fp32_to_fp16_bits(float(f)), float(f)


def test_x86_scale_roundtrip_exhaustive():
    L, R = orc.lib(), orc.ref()
    changed = 0
    for b in range(65520):
        eff = L.orc_x86_scale_bits(b)
        want = np.float32(R.ref_scale_store_load(b))
        got = np.float32(L.orc_fp16_to_fp32(eff))
        assert got.view(np.uint32) == want.view(np.uint32) or (np.isnan(got) and np.isnan(want)), hex(b)
        changed += eff != b
    assert changed > 50000  # the quirk is real: most patterns do not survive


def _rows(rng, K):
    import importlib.util, os
    spec = importlib.util.spec_from_file_location(
        "make_golden", os.path.join(os.path.dirname(__file__), "golden", "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.actquant_rows(rng, K)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_quantize_row_q8_0_bit_exact(seed):
    rng = np.random.default_rng(seed)
    x = np.concatenate([_rows(rng, 512), rng.standard_normal((64, 512)).astype(np.float32) * 3])
    qs, d_bits = orc.quantize_rows_q8_0(x)
    rqs, rd = orc.ref_quantize_rows_q8_0(x)
    assert np.array_equal(qs, rqs)
    eff = orc.fp16_bits_to_fp32(orc.x86_scale_bits(d_bits))
    assert np.array_equal(eff.view(np.uint32), rd.view(np.uint32))


@pytest.mark.parametrize("wtype", [orc.Q4_0, orc.Q8_0])
def test_dequantize_bit_exact(wtype):
    rng = np.random.default_rng(3)
    W = synth.make_weight(rng, wtype, 16, 256)
    assert np.array_equal(orc.dequantize(W, wtype, orc.SCALE_X86_REF).view(np.uint32),
                          orc.ref_dequantize(W, wtype).view(np.uint32))
    # un-snapped scales: only the x86 reading reproduces the reference, the IEEE reading must differ somewhere
    W2 = W.copy()
    W2[:, :, 0] |= 0x05
    assert np.array_equal(orc.dequantize(W2, wtype, orc.SCALE_X86_REF).view(np.uint32),
                          orc.ref_dequantize(W2, wtype).view(np.uint32))
    assert not np.array_equal(orc.dequantize(W2, wtype, orc.SCALE_IEEE), orc.ref_dequantize(W2, wtype))


@pytest.mark.parametrize("wtype", [orc.Q4_0, orc.Q8_0])
@pytest.mark.parametrize("M", [1, 3, 4, 8])
@pytest.mark.parametrize("bias", [False, True])
def test_linear_bit_exact_vs_reference_vec_dot(wtype, M, bias):
    rng = np.random.default_rng(100 + M)
    N, K = 48, 320
    W = synth.make_weight(rng, wtype, N, K)
    x = synth.make_x_fp32(rng, M, K)
    b = rng.standard_normal(N).astype(np.float32) if bias else None
    y = orc.linear_q(x, W, wtype, b, orc.SCALE_X86_REF)
    r = orc.ref_linear_q(x, W, wtype, b)
    assert np.array_equal(y.view(np.uint32), r.view(np.uint32))


def test_q4_0_weights_from_reference_quantizer():
    """weights written by the reference's own quantize_row_q4_0 (negative scales included) run through the oracle."""
    rng = np.random.default_rng(5)
    Wf = (rng.standard_normal((32, 256)) * 0.05).astype(np.float32)
    W = orc.ref_quantize_rows_q4_0(Wf)
    x = synth.make_x_fp32(rng, 2, 256)
    y = orc.linear_q(x, W, orc.Q4_0, None, orc.SCALE_X86_REF)
    r = orc.ref_linear_q(x, W, orc.Q4_0)
    assert np.array_equal(y.view(np.uint32), r.view(np.uint32))
    # and the quantized Linear approximates the fp32 one
    ref = x @ Wf.T
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 0.15


def _weight_rows(rng, N, K):
    """rows with positive and negative maxima, zero blocks, codes landing exactly on the .5 truncation boundaries"""
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    w[1, :32] = 0.0                                            # all-zero block: d = 0, id = 0, every code 8
    w[2, :32] = np.float32(-0.5) * np.arange(32) / 31          # negative maximum -> positive d
    w[3, :32] = np.float32(0.5) * np.arange(32) / 31           # positive maximum -> negative d (pattern >= 0x8000)
    w[4, :32] = np.float32(8.0) * np.linspace(-1, 1, 32)       # x*id lands on multiples of 1/2: the truncation boundaries
    w[5, :64] = np.float32(1e-6)
    return w


def _x86_field_to_pattern(field):
    """what a read on x86 makes of the stored field: the half-precision number, as an integer"""
    return field.view(np.float16).astype(np.float32).astype(np.uint16)


def test_q4_0_offline_quantizer_bit_exact():
    rng = np.random.default_rng(21)
    w = _weight_rows(rng, 24, 256)
    ref = orc.ref_quantize_rows_q4_0(w)                        # codes + the scale pattern an x86 read yields
    got = orc.quantize_weight_rows(w, orc.Q4_0, orc.SCALE_X86_REF)
    assert np.array_equal(got[:, :, 2:], ref[:, :, 2:])
    assert np.array_equal(_x86_field_to_pattern(got[:, :, 0:2].copy().view(np.uint16)[:, :, 0]),
                          ref[:, :, 0:2].copy().view(np.uint16)[:, :, 0])
    # IEEE storage: the field is the fp16 pattern of max / -8 itself; same codes
    ieee = orc.quantize_weight_rows(w, orc.Q4_0, orc.SCALE_IEEE)
    assert np.array_equal(ieee[:, :, 2:], ref[:, :, 2:])
    blocks = w.reshape(24, -1, 32)
    idx = np.abs(blocks).argmax(axis=2)
    d = np.take_along_axis(blocks, idx[..., None], axis=2)[..., 0] / np.float32(-8)
    assert np.array_equal(ieee[:, :, 0:2].copy().view(np.uint16)[:, :, 0], d.astype(np.float16).view(np.uint16))
    assert ieee[3, 0, 0:2].copy().view(np.uint16)[0] >= 0x8000  # positive maximum: negative d, sign bit in the pattern


def test_q8_0_offline_quantizer_bit_exact():
    rng = np.random.default_rng(22)
    w = _weight_rows(rng, 16, 128)
    codes, d_eff = orc.ref_quantize_rows_q8_0(w)               # reference: codes + effective scale values
    got = orc.quantize_weight_rows(w, orc.Q8_0, orc.SCALE_X86_REF)
    assert np.array_equal(got[:, :, 2:].view(np.int8).reshape(16, -1), codes)
    pat = _x86_field_to_pattern(got[:, :, 0:2].copy().view(np.uint16)[:, :, 0])
    assert np.array_equal(pat.view(np.float16).astype(np.float32).view(np.uint32), d_eff.view(np.uint32))
    ieee = orc.quantize_weight_rows(w, orc.Q8_0, orc.SCALE_IEEE)
    qs, bits = orc.quantize_rows_q8_0(w)
    assert np.array_equal(ieee[:, :, 0:2].copy().view(np.uint16)[:, :, 0], bits)
    assert np.array_equal(ieee[:, :, 2:].view(np.int8).reshape(16, -1), qs)


# ---- K-quants ------------------------------------------------------------------------------------------------------
def test_q8_K_quantizer_bit_exact():
    rng = np.random.default_rng(41)
    x = (rng.standard_normal((6, 1024)) * 3).astype(np.float32)
    x[1, 256:512] = 0                      # an all-zero super-block
    x[2, 0], x[2, 7] = -4.5, 4.5           # equal magnitudes, opposite signs: the FIRST one sets the sign of the scale
    x[2, 1:7] = 0.1
    x[2, 8:256] = 0.1
    x[3, 300] = 1e-30
    q, d, bs = orc.quantize_rows_q8_K(x)
    rq, rd, rbs = orc.ref_quantize_rows_q8_K(x)
    assert np.array_equal(q, rq) and np.array_equal(d.view(np.uint32), rd.view(np.uint32))
    nz = np.repeat(d != 0, 16, axis=1)
    assert np.array_equal(bs[nz], rbs[nz])   # the reference leaves the sums of an all-zero block unwritten
    assert d[2, 0] > 0 and q[2, 0] == -128 and q[2, 7] == 127


@pytest.mark.parametrize("wtype", [2, 3])
def test_kquant_dequantize_and_linear_bit_exact(wtype):
    rng = np.random.default_rng(42 + wtype)
    N, K, M = 24, 1024, 5
    # random blocks, and blocks the reference's own offline quantizer makes from fp32 weights
    for W in (synth.make_weight(rng, wtype, N, K), orc.ref_quantize_rows_k((rng.standard_normal((N, K)) * 0.05).astype(np.float32), wtype)):
        assert np.array_equal(orc.dequantize_k(W, wtype, orc.SCALE_X86_REF).view(np.uint32), orc.ref_dequantize_k(W, wtype).view(np.uint32))
        x = rng.standard_normal((M, K)).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32)
        y = orc.linear_kq(x, W, wtype, bias, orc.SCALE_X86_REF)
        assert np.array_equal(y.view(np.uint32), orc.ref_linear_kq(x, W, wtype, bias).view(np.uint32))
        # the exact integers behind it: brute force from the dequantized codes
        xq, xd, xbs = orc.quantize_rows_q8_K(x)
        isum, msum = orc.kq_block_sums(W, wtype, xq, xbs)
        unit = W.copy()
        if wtype == 2:
            unit[:, :, 0:2] = np.array([0x00, 0x3c], np.uint8)  # d = 1.0
            unit[:, :, 2:4] = 0                                  # dmin = 0: codes * sub-block scales remain
        else:
            unit[:, :, 208:210] = np.array([0x00, 0x3c], np.uint8)
        wq = orc.dequantize_k(unit, wtype, orc.SCALE_IEEE).astype(np.int64).reshape(N, K // 256, 256)
        want = np.einsum("nbk,mbk->nmb", wq, xq.astype(np.int64).reshape(M, K // 256, 256))
        assert np.array_equal(isum, want)


def _kq_weight_rows(rng, N, K):
    w = (rng.standard_normal((N, K)) * 0.04).astype(np.float32)
    w[0, :256] = 0.0                                        # an all-zero super-block
    w[1, :32] = 0.3                                         # a constant positive sub-block (its minimum is clamped to 0)
    w[1, 32:64] = -0.3                                      # a constant negative sub-block: max == min
    w[2, :256] = np.abs(w[2, :256])                         # all positive: every offset is zero
    w[3, :256] *= 50                                        # large values
    w[4, :16] = 0.0                                         # an all-zero group of 16 (Q6_K) inside a live super-block
    w[5, :256] = np.float32(1e-3) * rng.integers(-8, 8, 256)  # few distinct values, many ties in the search
    w[6, 0], w[6, 5] = 0.9, -0.9                            # equal magnitudes, opposite signs: the first one decides
    return w


@pytest.mark.parametrize("wtype", [orc.Q4_K, orc.Q6_K])
def test_k_quant_offline_quantizers_bit_exact(wtype):
    """orc_quantize_row_q4_K / _q6_K against the compiled reference quantizers (quantize_q4.cpp:184-282 with the search of
    :97-168; quantize_q6.cpp:34-106 with quantize.hpp:268-325): every byte of codes and sub-block scales equal, and the fp16
    fields decode -- the way an x86 read decodes them -- to the patterns the reference holds."""
    rng = np.random.default_rng(61 + wtype)
    w = _kq_weight_rows(rng, 20, 768)
    ref = orc.ref_quantize_rows_k(w, wtype)                 # canonical: effective patterns in the fp16 fields
    got = orc.quantize_weight_rows_k(w, wtype, orc.SCALE_X86_REF)
    fields = [(0, 2), (2, 4)] if wtype == orc.Q4_K else [(208, 210)]
    body = np.ones(got.shape[2], bool)
    for a, b in fields:
        body[a:b] = False
        assert np.array_equal(_x86_field_to_pattern(got[:, :, a:b].copy().view(np.uint16)[:, :, 0]),
                              ref[:, :, a:b].copy().view(np.uint16)[:, :, 0])
    assert np.array_equal(got[:, :, body], ref[:, :, body])
    # IEEE storage: the field is the fp16 pattern itself; the codes may differ from the x86 form only in super-blocks whose d
    # or dmin pattern the x86 read rounds (patterns of more than 11 significant bits)
    ieee = orc.quantize_weight_rows_k(w, wtype, orc.SCALE_IEEE)
    same = np.ones(got.shape[:2], bool)
    for a, b in fields:
        pat = ieee[:, :, a:b].copy().view(np.uint16)[:, :, 0]
        rounded = np.array([[orc.lib().orc_x86_scale_bits(int(v)) for v in row] for row in pat], np.uint16)
        same &= rounded == pat
    assert same.any() and (~same).any()
    assert np.array_equal(ieee[same][:, body], ref[same][:, body])
    # and the dequantized values of the blocks reproduce the weights to the formats' resolution
    deq = orc.dequantize_k(ref, wtype)
    err = np.abs(deq - w).max(axis=1) / (np.abs(w).max(axis=1) + 1e-12)
    assert (err < (0.08 if wtype == orc.Q4_K else 0.05)).all(), err
