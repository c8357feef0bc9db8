"""GPU parity of the W4A16 path: dequantized weight table bit-exact; GEMM output rel-L2 <= 1e-3 against the oracle
(the oracle sums in float64, the matrix cores in fp32, and both round once to bf16)."""
import numpy as np
import pytest
import torch

from mllm_amd import _lib, qlinear as ql, synth
from oracle import oracle as orc
from gpu_util import announce, bf16_dev, rel_l2, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _same_values(got_bits, want_bits):
    """bf16 tables equal as numbers; bit patterns may differ only in the sign of a zero (a zero scale: the kernel forms
    fma(q, s, -zp*s) = +0 where the closed form (q - zp) * 0 carries the sign of q - zp)."""
    g, w = synth.bf16_bits_to_fp32(got_bits), synth.bf16_bits_to_fp32(want_bits)
    neq = got_bits != want_bits
    return np.array_equal(g, w) and bool(((g == 0) & (w == 0))[neq].all())


def _dev(qw, s, zp):
    return to_dev(qw), torch.from_numpy(s.view(np.float16).copy()).cuda(), to_dev(zp)


def test_dequant_table_exhaustive():
    """every (q, zp) pair against a spread of scales"""
    s_bits = np.float16([0.01, 0.0123, 1.0, 3.14e-3, 6.1e-5, 2.5, 0.0, 1e-7]).view(np.uint16)
    rows = [(zp, si) for zp in range(16) for si in range(len(s_bits))]
    N, K = len(rows), 256
    q = np.tile(np.arange(16, dtype=np.uint8), (N, 16))
    z = np.array([[r[0], 15 - r[0]] for r in rows], dtype=np.uint8)
    s = np.array([[s_bits[r[1]], s_bits[(r[1] + 3) % len(s_bits)]] for r in rows], dtype=np.uint16)
    announce("w4a16 dequant table")
    got = _bits(ql.w4a16_dequantize(*_dev(synth.pack_nibbles(q), s, synth.pack_nibbles(z))))
    assert _same_values(got, orc.w4a16_dequant(synth.pack_nibbles(q), s, synth.pack_nibbles(z)))


def test_dequant_full_size_bit_exact():
    rng = synth.rng_for(2)
    qw, s, zp, _, _ = synth.make_w4a16(rng, 9728, 2560)
    announce("w4a16 dequant full")
    got = _bits(ql.w4a16_dequantize(*_dev(qw, s, zp)))
    assert np.array_equal(got, orc.w4a16_dequant(qw, s, zp))


@pytest.mark.parametrize("M,N,K,group", [(1, 64, 128, 128), (9, 24, 384, 128), (130, 200, 512, 128), (64, 96, 256, 64),
                                         (257, 193, 1024, 256), (33, 128, 2560, 128)])
@pytest.mark.parametrize("tile", [0, 1, 2, 3])
def test_gemm_vs_oracle(M, N, K, group, tile):
    rng = synth.rng_for(2, M + N + K + group)
    qw, s, zp, _, _ = synth.make_w4a16(rng, N, K, group)
    a_bits, _ = synth.make_x_bf16(rng, M, K)
    bias = synth.fp32_to_bf16_bits((rng.standard_normal(N) * 0.1).astype(np.float32))
    L = _lib.lib()
    try:
        assert L.mllm_hip_w4a16_set_tuning(tile) == 0
        announce("w4a16 gemm", M, N, K, group, "tile", tile)
        d = _dev(qw, s, zp)
        c = _bits(ql.w4a16_gemm(bf16_dev(a_bits), *d, None, group))
        cb = _bits(ql.w4a16_gemm(bf16_dev(a_bits), *d, bf16_dev(bias), group))
    finally:
        L.mllm_hip_w4a16_set_tuning(0)
    want = orc.w4a16_gemm(a_bits, qw, s, zp, None, group)
    wantb = orc.w4a16_gemm(a_bits, qw, s, zp, bias, group)
    assert rel_l2(synth.bf16_bits_to_fp32(c), synth.bf16_bits_to_fp32(want)) <= TOL
    assert rel_l2(synth.bf16_bits_to_fp32(cb), synth.bf16_bits_to_fp32(wantb)) <= TOL
    # almost every element identical, the rest one bf16 ulp apart (different summation order before the single rounding)
    diff = np.abs(c.astype(np.int32) - want.astype(np.int32))
    assert diff.max() <= 1 or rel_l2(synth.bf16_bits_to_fp32(c), synth.bf16_bits_to_fp32(want)) < 1e-4
    assert (diff == 0).mean() > 0.97


# shapes that reach each tile of the weights-from-global kernel (128x384, 64x384, 128x128, 64x128), ragged edges, a K
# that is not a multiple of the 128-element K step, and groups of 64 / 128 / 256
PACKED_SHAPES = [(1, 64, 128, 128), (9, 24, 384, 128), (130, 200, 512, 128), (64, 96, 256, 64), (257, 193, 1024, 256),
                 (33, 128, 2560, 128), (70, 100, 192, 64), (1536, 6144, 256, 128), (512, 9216, 128, 128),
                 (1024, 3072, 128, 64)]


@pytest.mark.parametrize("M,N,K,group", PACKED_SHAPES)
def test_gemm_packed_vs_oracle(M, N, K, group):
    rng = synth.rng_for(2, 3 * M + N + K + group)
    qw, s, zp, _, _ = synth.make_w4a16(rng, N, K, group)
    a_bits, _ = synth.make_x_bf16(rng, M, K)
    bias = synth.fp32_to_bf16_bits((rng.standard_normal(N) * 0.1).astype(np.float32))
    announce("w4a16 packed gemm", M, N, K, group)
    packed = ql.w4a16_prepack(*_dev(qw, s, zp), group)
    table = _bits(ql.w4a16_dequantize_packed(packed, N, K, group))
    assert _same_values(table, orc.w4a16_dequant(qw, s, zp, group))
    c = _bits(ql.w4a16_gemm_packed(bf16_dev(a_bits), packed, N, None, group))
    cb = _bits(ql.w4a16_gemm_packed(bf16_dev(a_bits), packed, N, bf16_dev(bias), group))
    want = orc.w4a16_gemm(a_bits, qw, s, zp, None, group)
    wantb = orc.w4a16_gemm(a_bits, qw, s, zp, bias, group)
    assert rel_l2(synth.bf16_bits_to_fp32(c), synth.bf16_bits_to_fp32(want)) <= TOL
    assert rel_l2(synth.bf16_bits_to_fp32(cb), synth.bf16_bits_to_fp32(wantb)) <= TOL
    diff = np.abs(c.astype(np.int32) - want.astype(np.int32))
    assert diff.max() <= 1 or rel_l2(synth.bf16_bits_to_fp32(c), synth.bf16_bits_to_fp32(want)) < 1e-4
    assert (diff == 0).mean() > 0.97


@pytest.mark.parametrize("M,mfma_from", [(1, 2), (2, 5), (3, 5), (4, 5), (1, 1), (2, 2), (3, 2), (5, 2), (8, 2), (13, 2), (16, 2), (27, 2), (32, 2)])
def test_decode_gemv_packed_vs_oracle_and_tiles(M, mfma_from):
    """a few tokens take the GEMV kernels (a block row of the packed matrix per workgroup; fp32 FMAs up to four tokens, the matrix
    cores from `mfma_from`): the oracle within the GEMM's tolerance, nearly every output the tile kernels' bits; ragged N, K not
    a multiple of 128, groups of 64 / 128 / 256, bias.  (Where the tokens' activations do not fit LDS the tile kernels run.)"""
    L = _lib.lib()
    assert L.mllm_hip_w4a16_set_decode_mfma_from(mfma_from) == 0
    try:
        _decode_gemv_cases(L, M)
    finally:
        assert L.mllm_hip_w4a16_set_decode_mfma_from(2) == 0
    assert L.mllm_hip_w4a16_set_decode_mfma_from(0) == -1 and L.mllm_hip_w4a16_set_decode_mfma_from(34) == -1


def _decode_gemv_cases(L, M):
    for N, K, group in ((9728, 2560, 128), (2560, 9728, 128), (77, 192, 64), (200, 1024, 256), (33, 4096 + 64, 64)):
        rng = synth.rng_for(2, 900 + 3 * M + N + K + group)
        qw, s, zp, _, _ = synth.make_w4a16(rng, N, K, group)
        a_bits, _ = synth.make_x_bf16(rng, M, K)
        bias = synth.fp32_to_bf16_bits((rng.standard_normal(N) * 0.1).astype(np.float32))
        announce("w4a16 decode gemv", M, N, K, group)
        packed = ql.w4a16_prepack(*_dev(qw, s, zp), group)
        c = _bits(ql.w4a16_gemm_packed(bf16_dev(a_bits), packed, N, None, group))
        cb = _bits(ql.w4a16_gemm_packed(bf16_dev(a_bits), packed, N, bf16_dev(bias), group))
        want = orc.w4a16_gemm(a_bits, qw, s, zp, None, group)
        wantb = orc.w4a16_gemm(a_bits, qw, s, zp, bias, group)
        assert rel_l2(synth.bf16_bits_to_fp32(c), synth.bf16_bits_to_fp32(want)) <= TOL
        assert rel_l2(synth.bf16_bits_to_fp32(cb), synth.bf16_bits_to_fp32(wantb)) <= TOL
        assert L.mllm_hip_w4a16_set_decode(0) == 0
        try:
            ct = _bits(ql.w4a16_gemm_packed(bf16_dev(a_bits), packed, N, bf16_dev(bias), group))
        finally:
            assert L.mllm_hip_w4a16_set_decode(1) == 0
        diff = np.abs(cb.astype(np.int32) - ct.astype(np.int32))
        assert diff.max() <= 1 or rel_l2(synth.bf16_bits_to_fp32(cb), synth.bf16_bits_to_fp32(ct)) < 1e-4
        assert (diff == 0).mean() > 0.95
    assert L.mllm_hip_w4a16_set_decode(2) == -1


@pytest.mark.parametrize("tile", [1, 2, 3, 4, 5, 16 + 5])
def test_gemm_packed_every_tile(tile):
    M, N, K, group = 200, 800, 384, 128
    rng = synth.rng_for(2, 77 + tile)
    qw, s, zp, _, _ = synth.make_w4a16(rng, N, K, group)
    a_bits, _ = synth.make_x_bf16(rng, M, K)
    L = _lib.lib()
    packed = ql.w4a16_prepack(*_dev(qw, s, zp), group)
    try:
        assert L.mllm_hip_w4a16_packed_set_tuning(tile) == 0
        announce("w4a16 packed gemm tile", tile)
        c = _bits(ql.w4a16_gemm_packed(bf16_dev(a_bits), packed, N, None, group))
    finally:
        L.mllm_hip_w4a16_packed_set_tuning(0)
    want = orc.w4a16_gemm(a_bits, qw, s, zp, None, group)
    assert rel_l2(synth.bf16_bits_to_fp32(c), synth.bf16_bits_to_fp32(want)) <= TOL


def test_full_size_prefill():
    """A bf16 [2048,2560], W uint4 [9728,2560] g128: a row sample against the oracle, plus linearity on all rows:
    GEMM(2*A) == 2*GEMM(A) exactly (scaling by two commutes with every rounding)."""
    rng = synth.rng_for(2)
    M, N, K = 2048, 9728, 2560
    qw, s, zp, _, _ = synth.make_w4a16(rng, N, K)
    a_bits, a = synth.make_x_bf16(rng, M, K)
    announce("w4a16 full size")
    d = _dev(qw, s, zp)
    c = ql.w4a16_gemm(bf16_dev(a_bits), *d)
    cb = _bits(c)
    rows = np.sort(rng.choice(M, 32, replace=False))
    want = orc.w4a16_gemm(a_bits[rows], qw, s, zp)
    r = rel_l2(synth.bf16_bits_to_fp32(cb[rows]), synth.bf16_bits_to_fp32(want))
    assert r <= TOL, r
    a2 = synth.fp32_to_bf16_bits(a * 2)
    c2 = ql.w4a16_gemm(bf16_dev(a2), *d)
    assert torch.equal(c2.float(), c.float() * 2)
    # (this shape runs 512 full tiles and 192 half-height tiles in the packed kernel's schedule)
    # the prepacked-weight path: table bit-exact, same row sample, same linearity, and close to the plain path everywhere
    packed = ql.w4a16_prepack(*d)
    assert np.array_equal(_bits(ql.w4a16_dequantize_packed(packed, N, K)), orc.w4a16_dequant(qw, s, zp))
    cp = ql.w4a16_gemm_packed(bf16_dev(a_bits), packed, N)
    r = rel_l2(synth.bf16_bits_to_fp32(_bits(cp)[rows]), synth.bf16_bits_to_fp32(want))
    assert r <= TOL, r
    assert torch.equal(ql.w4a16_gemm_packed(bf16_dev(a2), packed, N).float(), cp.float() * 2)
    assert rel_l2(cp.float().cpu().numpy(), c.float().cpu().numpy()) <= 1e-4
    # zero-point equal to every code -> exact zeros
    z_un = rng.integers(0, 16, (64, K // 128), dtype=np.uint8)
    qz = np.repeat(z_un, 128, axis=1)
    dz = _dev(synth.pack_nibbles(qz), s[:64].copy(), synth.pack_nibbles(z_un))
    c0 = ql.w4a16_gemm(bf16_dev(a_bits[:128]), *dz)
    assert (c0.float() == 0).all()


def test_argument_errors():
    L = _lib.lib()
    t = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    g = L.mllm_hip_w4a16_gemm
    p = t.data_ptr()
    assert g(p, p, p, p, None, p, 8, 8, 128, 100, None) == -2     # group not a multiple of 64
    assert g(p, p, p, p, None, p, 8, 8, 192, 128, None) == -2     # K not a multiple of the group
    assert g(None, p, p, p, None, p, 8, 8, 128, 128, None) == -1
    assert g(p, p + 1, p, p, None, p, 8, 8, 128, 128, None) == -3
    assert L.mllm_hip_w4a16_set_tuning(-1) == -1


@pytest.mark.parametrize("N,K,group", [(8, 128, 128), (24, 384, 128), (200, 512, 64), (72, 1000, 200), (9728, 2560, 128)])
def test_awq_checkpoint_unpack_bit_exact_and_gemm(N, K, group):
    """AWQ int32 tensors -> row-major tensors byte for byte (against the known codes and against the oracle's unpack of the
    same dwords), then the packed GEMM on them against the oracle."""
    rng = synth.rng_for(2, N + K + group + 5)
    qweight, qzeros, scales, q, z, s = synth.make_awq(rng, N, K, group)
    announce("w4a16 from awq N=%d K=%d group=%d" % (N, K, group))
    qw_d, s_d, z_d = ql.w4a16_from_awq(torch.from_numpy(qweight).cuda(), torch.from_numpy(qzeros).cuda(),
                                       torch.from_numpy(scales.view(np.float16).copy()).cuda(), group)
    torch.cuda.synchronize()
    assert np.array_equal(qw_d.cpu().numpy(), synth.pack_nibbles(q))
    assert np.array_equal(z_d.cpu().numpy(), synth.pack_nibbles(z))
    assert np.array_equal(_bits(s_d), s)
    oq, osb, oz = orc.awq_unpack(qweight, qzeros, scales)
    assert np.array_equal(qw_d.cpu().numpy(), oq) and np.array_equal(z_d.cpu().numpy(), oz) and np.array_equal(_bits(s_d), osb)
    if group % 64 or N > 1000:
        return
    M = 37
    a_bits, _ = synth.make_x_bf16(rng, M, K)
    packed = ql.w4a16_prepack(qw_d, s_d, z_d, group)
    got = _bits(ql.w4a16_gemm_packed(bf16_dev(a_bits), packed, N, None, group))
    want = orc.w4a16_gemm(a_bits, oq, osb, oz, None, group)
    assert rel_l2(synth.bf16_bits_to_fp32(got), synth.bf16_bits_to_fp32(want)) <= TOL
