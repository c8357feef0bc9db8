"""GPU parity of the operators around Linear (RMSNorm, SiLU, add, mul, SiLU*up, softmax, top-k, MoE gate) and of the decode
GEMV with those neighbours folded in (residual in the epilogue, activations handed over as a quantized image).

Bars: fp32 / bf16 outputs rel-L2 <= 1e-3 against the oracle (measured: 1e-7 .. 1e-6, elementwise work is the same fp32
operation sequence); indices, quantized images and everything derived from stored tensors bit-exact.
"""
import numpy as np
import pytest
import torch

from mllm_amd import _lib, qlinear as ql, synth
from oracle import oracle as orc
from gpu_util import announce, bf16_dev, rel_l2, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _bf16_round(a):
    return orc.bf16_bits_to_fp32(orc.fp32_to_bf16_bits(np.asarray(a, np.float32)))


def _image_fields(img, M, K):
    """splits a quantized image into (codes int8 [MT, K], scales fp32 [MT, nb], n8 int32 [MT, nb])"""
    MT = 1 if M <= 1 else 2 if M <= 2 else 4 if M <= 4 else 8
    nb = K // 32
    mnb = MT * nb
    raw = img.cpu().numpy()
    lo = raw[:mnb * 16].view(np.int8).reshape(mnb, 16)
    hi = raw[mnb * 16:mnb * 32].view(np.int8).reshape(mnb, 16)
    d = raw[mnb * 32:mnb * 36].view(np.float32).reshape(MT, nb)
    n8 = raw[mnb * 36:mnb * 40].view(np.int32).reshape(MT, nb)
    codes = np.concatenate([lo, hi], axis=1).reshape(MT, K)
    return codes, d, n8


def _check_image(img, y_stored, M, K, x86):
    """the image must be the Q8_0 quantization of the stored rows (bit-exact), zero beyond them"""
    codes, d, n8 = _image_fields(img, M, K)
    q, dbits = orc.quantize_rows_q8_0(np.asarray(y_stored, np.float32).reshape(M, K))
    bits = orc.x86_scale_bits(dbits) if x86 else dbits
    assert np.array_equal(codes[:M], q)
    assert np.array_equal(d[:M].view(np.uint32), orc.fp16_bits_to_fp32(bits).view(np.uint32))
    assert np.array_equal(n8[:M], -8 * q.reshape(M, K // 32, 32).astype(np.int32).sum(-1))
    assert not codes[M:].any() and not d[M:].any() and not n8[M:].any()


@pytest.mark.parametrize("rows,D", [(1, 2560), (5, 2560), (3, 128), (64, 4096), (2, 9728), (7, 40), (300, 128)])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_rmsnorm(rows, D, dtype):
    rng = synth.rng_for(6, rows * 7 + D)
    w = (1 + 0.2 * rng.standard_normal(D)).astype(np.float32)
    if dtype == "bf16":
        bits, xf = synth.make_x_bf16(rng, rows, D)
        x = bf16_dev(bits)
    else:
        xf = synth.make_x_fp32(rng, rows, D) * 2.5
        x = to_dev(xf)
    for off in (False, True):
        announce("rmsnorm", rows, D, dtype, off)
        y = ql.rmsnorm(x, to_dev(w), 1e-6, off).float().cpu().numpy()
        want = orc.rmsnorm(xf, w, 1e-6, off)
        if dtype == "f32":
            assert rel_l2(y, want) < 2e-6
        else:  # stored as bf16: equal to the rounded oracle values up to single-ulp flips at rounding boundaries
            assert rel_l2(y, _bf16_round(want)) < TOL


@pytest.mark.parametrize("rows,D", [(1, 2560), (3, 128), (4, 4096), (2, 40)])
def test_rmsnorm_fp32_bit_for_bit(rows, D):
    """x * (w * rms) in the reference's operation order (x86/rmsnorm.cpp:29-47), compared bit for bit: the rows hold small
    integers, so the sum of squares is exact in fp32 whatever the order of its additions and rms is the same number on
    both sides; every difference left would be an operation-order difference in the elementwise part."""
    rng = synth.rng_for(6, 50000 + rows * 7 + D)
    xf = rng.integers(-15, 16, (rows, D)).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(D)).astype(np.float32)
    for off in (False, True):
        announce("rmsnorm bit-exact", rows, D, off)
        y = ql.rmsnorm(to_dev(xf), to_dev(w), 1e-6, off).cpu().numpy()
        want = orc.rmsnorm(xf, w, 1e-6, off)
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("M,K", [(1, 2560), (2, 2560), (3, 4096), (4, 9728), (8, 2560), (1, 96), (6, 32)])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_rmsnorm_writes_the_image_of_what_it_stored(M, K, dtype):
    rng = synth.rng_for(6, 1000 + M * 13 + K)
    w = (1 + 0.2 * rng.standard_normal(K)).astype(np.float32)
    if dtype == "bf16":
        bits, _ = synth.make_x_bf16(rng, M, K)
        x = bf16_dev(bits)
    else:
        x = to_dev(synth.make_x_fp32(rng, M, K))
    for mode, x86 in ((ql.SCALE_X86_REF, True), (ql.SCALE_IEEE, False)):
        announce("rmsnorm image", M, K, dtype, x86)
        y, img = ql.rmsnorm(x, to_dev(w), 1e-6, want_image=True, act_scale_mode=mode)
        assert torch.equal(y, ql.rmsnorm(x, to_dev(w), 1e-6))
        _check_image(img, y.float().cpu().numpy(), M, K, x86)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_elementwise(dtype):
    rng = synth.rng_for(6, 77)
    n = 8 * 1237
    a = (rng.standard_normal(n) * 4).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    if dtype == "bf16":
        a, b = _bf16_round(a), _bf16_round(b)
        da, db = to_dev(a).bfloat16(), to_dev(b).bfloat16()
        rnd = _bf16_round
    else:
        da, db = to_dev(a), to_dev(b)
        rnd = lambda v: v
    announce("elementwise", dtype)
    assert np.array_equal(ql.add(da, db).float().cpu().numpy(), rnd(a + b))
    assert np.array_equal(ql.mul(da, db).float().cpu().numpy(), rnd(a * b))
    s = ql.silu(da).float().cpu().numpy()
    assert rel_l2(s, rnd(orc.silu(a))) < (2e-7 if dtype == "f32" else TOL)
    sm = ql.silu_mul(da.view(1, n), db.view(1, n)).float().cpu().numpy().ravel()
    assert rel_l2(sm, rnd(rnd(orc.silu(a)) * b)) < (2e-7 if dtype == "f32" else TOL)
    # one pass equals the two operators run one after the other, bit for bit
    assert torch.equal(ql.silu_mul(da.view(1, n), db.view(1, n)).view(-1), ql.mul(ql.silu(da), db))
    # the reference's exp is not an accurate exp: the switch to expf moves SiLU by about 1e-4 .. 1e-3
    if dtype == "f32":
        ql.set_exp_mode(1)
        try:
            acc = ql.silu(da).cpu().numpy()
        finally:
            ql.set_exp_mode(0)
        exact = a.astype(np.float64) / (1 + np.exp(-a.astype(np.float64)))
        assert rel_l2(acc, exact) < 2e-7 and 1e-5 < rel_l2(s, exact) < 2e-3


@pytest.mark.parametrize("M,D", [(1, 9728), (4, 9728), (8, 768), (2, 64)])
def test_silu_mul_image(M, D):
    rng = synth.rng_for(6, 2000 + M + D)
    g = to_dev(synth.make_x_fp32(rng, M, D) * 2)
    u = to_dev(synth.make_x_fp32(rng, M, D))
    announce("silu_mul image", M, D)
    y, img = ql.silu_mul(g, u, want_image=True, act_scale_mode=ql.SCALE_X86_REF)
    assert torch.equal(y, ql.silu_mul(g, u))
    _check_image(img, y.cpu().numpy(), M, D, True)
    # the product alone can write the image too (the reference runs SiLU and the product as two operators)
    y2, img2 = ql.mul(ql.silu(g), u, want_image=True)
    assert torch.equal(y2, y)
    _check_image(img2, y.cpu().numpy(), M, D, True)
    y3, img3 = ql.add(g, u, want_image=True, act_scale_mode=ql.SCALE_IEEE)
    _check_image(img3, y3.cpu().numpy(), M, D, False)


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M", [1, 2, 3, 8])
def test_gemv_fused_equals_the_operators_it_replaces(wtype, M):
    """rmsnorm(+image) -> gate/up GEMV from the image -> silu*up(+image) -> down GEMV from the image + residual
    equals rmsnorm -> GEMV -> silu -> mul -> GEMV -> add, bit for bit, and the oracle's chain within tolerance"""
    rng = synth.rng_for(6, 3000 + wtype * 10 + M)
    H, I = 512, 1536
    Wg, Wu, Wd = (synth.make_weight(rng, wtype, I, H), synth.make_weight(rng, wtype, I, H), synth.make_weight(rng, wtype, H, I))
    pg, pu, pd = (ql.PackedQWeight(wtype, torch.from_numpy(W)) for W in (Wg, Wu, Wd))
    xf = synth.make_x_fp32(rng, M, H)
    nw = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    x, w = to_dev(xf), to_dev(nw)
    announce("fused mlp chain", wtype, M)
    # unfused
    h0 = ql.rmsnorm(x, w, 1e-6)
    g0, u0 = ql.linear_q_gemv_multi([pg, pu], h0)
    a0 = ql.mul(ql.silu(g0), u0)
    o0 = ql.add(ql.linear_q_gemv(pd, a0), x)
    # fused
    h1, img = ql.rmsnorm(x, w, 1e-6, want_image=True)
    g1, u1 = ql.linear_q_gemv_fused([pg, pu], img, M=M, image=True)
    a1, img2 = ql.silu_mul(g1, u1, want_image=True)
    (o1,) = ql.linear_q_gemv_fused([pd], img2, M=M, image=True, residuals=[x])
    assert torch.equal(g0, g1) and torch.equal(u0, u1) and torch.equal(a0, a1) and torch.equal(o0, o1)
    # raw activations with a workspace (quantized once per launch from three rows on): the same bits
    (o1w,) = ql.linear_q_gemv_fused([pd], a0, residuals=[x], workspace=ql.gemv_workspace(M, I))
    assert torch.equal(o1w, o0)
    # residual together with a bias, activations not pre-quantized, residual aliasing the output
    bias = to_dev(rng.standard_normal(H).astype(np.float32))
    o2 = x.clone()
    ql.linear_q_gemv_fused([pd], a0, biases=[bias], residuals=[o2], outs=[o2])
    assert torch.equal(o2, ql.add(ql.linear_q_gemv(pd, a0, bias), x))
    # oracle chain
    hn = orc.rmsnorm(xf, nw, 1e-6)
    gn = orc.linear_q(hn, Wg, wtype, None, orc.SCALE_X86_REF)
    un = orc.linear_q(hn, Wu, wtype, None, orc.SCALE_X86_REF)
    an = orc.silu(gn) * un
    on = orc.linear_q(an, Wd, wtype, None, orc.SCALE_X86_REF) + xf
    assert rel_l2(g1.cpu().numpy(), gn) < TOL and rel_l2(a1.cpu().numpy(), an) < TOL and rel_l2(o1.cpu().numpy(), on) < TOL


@pytest.mark.parametrize("wtype", [0, 1])
@pytest.mark.parametrize("M,H,I", [(1, 512, 1536), (2, 512, 96), (3, 2560, 9728), (4, 4096, 512), (5, 96, 64), (8, 2560, 1024), (1, 2560, 9728),
                                   (6, 4096, 256), (7, 5120, 160), (3, 8192, 64)])
def test_mlp_gate_up_one_launch(wtype, M, H, I):
    """gate / up / SiLU / product (/ Q8_0 image of the product) in one launch against the oracle's chain, and the image
    against the Q8_0 quantization of the h the same launch stored (bit-exact); from activations and from rmsnorm's image"""
    rng = synth.rng_for(6, 5000 + wtype * 1000 + M * 10 + H % 7)
    Wg, Wu = synth.make_weight(rng, wtype, I, H), synth.make_weight(rng, wtype, I, H)
    pg, pu = ql.PackedQWeight(wtype, torch.from_numpy(Wg)), ql.PackedQWeight(wtype, torch.from_numpy(Wu))
    xf = synth.make_x_fp32(rng, M, H)
    x = to_dev(xf)
    announce("mlp gate/up one launch", wtype, M, H, I)
    h, img = ql.mlp_gate_up(pg, pu, x, want_image=True)
    gn = orc.linear_q(xf, Wg, wtype, None, orc.SCALE_X86_REF)
    un = orc.linear_q(xf, Wu, wtype, None, orc.SCALE_X86_REF)
    assert rel_l2(h.cpu().numpy(), orc.silu(gn) * un) < TOL
    _check_image(img, h.cpu().numpy(), M, I, True)
    # the separate launches it replaces: same arithmetic, row sums over other lane counts -> equal to fp32 rounding
    g0, u0 = ql.linear_q_gemv_multi([pg, pu], x)
    assert rel_l2(h.cpu().numpy(), ql.silu_mul(g0, u0).cpu().numpy()) < 1e-5
    # only one of the two results asked for; bf16 activations; the image of x handed over
    assert torch.equal(ql.mlp_gate_up(pg, pu, x), h)
    same = lambda a, b: all(np.array_equal(p, q) for p, q in zip(_image_fields(a, M, I), _image_fields(b, M, I)))
    assert same(ql.mlp_gate_up(pg, pu, x, want_h=False, want_image=True), img)
    _, ximg = ql.add(x, torch.zeros_like(x), want_image=True)
    h2, img2 = ql.mlp_gate_up(pg, pu, ximg, M=M, image=True, want_image=True)
    assert torch.equal(h2, h) and same(img2, img)
    xb = x.to(torch.bfloat16)
    hb = ql.mlp_gate_up(pg, pu, xb)
    assert torch.equal(hb, ql.mlp_gate_up(pg, pu, xb.float()))
    # IEEE scales and the accurate exp
    hi, imgi = ql.mlp_gate_up(pg, pu, x, want_image=True, act_scale_mode=ql.SCALE_IEEE)
    _check_image(imgi, hi.cpu().numpy(), M, I, False)
    ql.set_exp_mode(True)
    try:
        ha = ql.mlp_gate_up(pg, pu, x)
    finally:
        ql.set_exp_mode(False)
    g64, u64 = gn.astype(np.float64), un.astype(np.float64)
    assert rel_l2(ha.cpu().numpy(), g64 / (1 + np.exp(-g64)) * u64) < 1e-5


@pytest.mark.parametrize("rows,n", [(1, 128), (512, 128), (5, 16), (7, 13), (3, 1000), (9, 60), (3, 2048), (5, 2049), (3, 4099), (2, 8192),
                                    (3, 12003), (2, 16384), (2, 16391), (1, 40003)])
def test_softmax(rows, n):
    rng = synth.rng_for(6, 4000 + rows + n)
    x = (rng.standard_normal((rows, n)) * 3).astype(np.float32)
    announce("softmax", rows, n)
    y = ql.softmax(to_dev(x)).cpu().numpy()
    want = orc.softmax(x)
    # (the oracle adds a row's terms one after another in fp32: over tens of thousands of terms its own sum is the less exact one)
    assert rel_l2(y, want) < (2e-6 if n <= 16384 else 4e-6)
    assert np.allclose(y.sum(-1), 1.0, atol=1e-5)


def test_topk_reference_test_shapes_and_sort():
    rng = synth.rng_for(6, 5000)
    for shape in [(10,), (1, 10), (5, 10), (2, 5, 10), (1, 4, 8, 16)]:  # tests/cpu/KernelTest.cpp:686
        x = rng.uniform(-10, 10, shape).astype(np.float32)
        announce("topk", shape)
        v, i = ql.topk(to_dev(x), 3)
        wv, wi = orc.topk(x, 3)
        assert v.shape == wv.shape and i.dtype == torch.int32
        assert np.array_equal(i.cpu().numpy(), wi) and np.array_equal(v.cpu().numpy(), wv)
    x = rng.standard_normal((700, 128)).astype(np.float32)
    for k, largest, srt in [(8, True, False), (8, True, True), (5, False, True), (128, True, True), (1, False, False)]:
        announce("topk", k, largest, srt)
        v, i = ql.topk(to_dev(x), k, largest, srt)
        wv, wi = orc.topk(x, k, largest, srt)
        assert np.array_equal(i.cpu().numpy(), wi) and np.array_equal(v.cpu().numpy(), wv)
    # ties are taken lowest index first
    t = np.float32([[1, 3, 3, 2, 3, 0, 3, 3]])
    v, i = ql.topk(to_dev(t), 3)
    assert i.cpu().numpy().tolist() == [[1, 2, 4]]
    long = rng.standard_normal((3, 5000)).astype(np.float32)
    v, i = ql.topk(to_dev(long), 20)
    wv, wi = orc.topk(long, 20)
    assert np.array_equal(i.cpu().numpy(), wi)
    # rows long enough for the workgroup-per-row kernel, with repeated values (ties go lowest index first), both orders
    vocab = np.round(rng.standard_normal((3, 20011)) * 50).astype(np.float32)
    for k, largest, srt in [(20, True, True), (7, False, False), (50, True, False)]:
        announce("topk long rows", k, largest, srt)
        v, i = ql.topk(to_dev(vocab), k, largest, srt)
        wv, wi = orc.topk(vocab, k, largest, srt)
        assert np.array_equal(i.cpu().numpy(), wi) and np.array_equal(v.cpu().numpy(), wv)


@pytest.mark.parametrize("rows,ln", [(5, 257), (3, 1000), (4, 2048), (3, 2051), (2, 8192), (2, 9001), (2, 33000), (1, 151936)])
def test_topk_by_radix_select(rows, ln):
    """rows longer than 256 elements: every selection equals the oracle's (ties lowest index first), whatever the row's length
    (whole 16-byte loads or single elements, keys in registers or read again per pass), k, order and kind of ties"""
    rng = synth.rng_for(6, 5100 + ln)
    smooth = rng.standard_normal((rows, ln)).astype(np.float32)
    coarse = np.round(rng.standard_normal((rows, ln)) * 3).astype(np.float32)  # a few dozen distinct values, signed zeros among them
    coarse[:, ::7] *= -1.0
    flat = np.full((rows, ln), 2.5, np.float32)  # every element ties
    flat[:, ln // 2] = 7.0
    for nm, x in (("smooth", smooth), ("coarse", coarse), ("flat", flat)):
        for k, largest, srt in [(1, True, True), (8, True, False), (50, True, True), (33, False, True), (min(ln, 2048), True, False),
                                (257, False, False)]:
            announce("topk radix", nm, rows, ln, k, largest, srt)
            v, i = ql.topk(to_dev(x), k, largest, srt)
            wv, wi = orc.topk(x, k, largest, srt)
            assert np.array_equal(i.cpu().numpy(), wi)
            assert np.array_equal(v.cpu().numpy().view(np.uint32), wv.view(np.uint32))


@pytest.mark.parametrize("M,H,E,k,dtype", [(512, 2048, 128, 8, "f32"), (1, 2048, 128, 8, "f32"), (7, 256, 60, 4, "f32"),
                                           (33, 2048, 128, 8, "bf16"), (5, 64, 8, 2, "f32")])
def test_moe_gate(M, H, E, k, dtype):
    rng = synth.rng_for(6, 6000 + M + E)
    w = (rng.standard_normal((E, H)) * 0.05).astype(np.float32)
    if dtype == "bf16":
        bits, xf = synth.make_x_bf16(rng, M, H)
        x = bf16_dev(bits)
    else:
        xf = synth.make_x_fp32(rng, M, H)
        x = to_dev(xf)
    for norm in (True, False):
        announce("moe gate", M, H, E, k, dtype, norm)
        ids, wt, sc = ql.moe_gate(x, to_dev(w), k, norm, want_scores=True)
        # the two forms -- logits with the experts spread over the grid and a second launch per token (with a scores buffer),
        # everything in one workgroup per four tokens (without, or forced) -- give the same bits
        L = _lib.lib()
        i1, w1 = ql.moe_gate(x, to_dev(w), k, norm)
        assert L.mllm_hip_moe_gate_set_form(0) == 0
        try:
            i0, w0, s0 = ql.moe_gate(x, to_dev(w), k, norm, want_scores=True)
        finally:
            assert L.mllm_hip_moe_gate_set_form(1) == 0
        assert torch.equal(ids, i1) and torch.equal(wt, w1) and torch.equal(ids, i0) and torch.equal(wt, w0) and torch.equal(sc, s0)
        ids, wt, sc = ids.cpu().numpy(), wt.cpu().numpy(), sc.cpu().numpy()
        oi, ow, osc = orc.moe_gate(xf, w, k, norm)
        assert rel_l2(sc, osc) < 1e-5
        # index work is exact: the selection made on the kernel's own scores is the oracle's selection on those scores
        sv, si = orc.topk(sc, k, True, False)
        assert np.array_equal(ids, si)
        want_w = sv / sv.sum(-1, keepdims=True) if norm else sv
        assert np.max(np.abs(wt - want_w)) < 1e-6
        # end to end the experts agree wherever the oracle's k-th and (k+1)-th scores are further apart than the
        # rounding noise of the logits
        srt = -np.sort(-osc, axis=-1)
        safe = (srt[:, k - 1] - srt[:, k]) > 1e-5 * srt[:, 0] if k < E else np.ones(M, bool)
        assert safe.mean() > 0.9
        assert np.array_equal(ids[safe], oi[safe])
        assert np.max(np.abs(wt[safe] - ow[safe])) < 1e-5


def test_argument_checks():
    L = _lib.lib()
    x = torch.zeros(64, dtype=torch.float32, device="cuda")
    p = x.data_ptr()
    assert L.mllm_hip_rmsnorm(p, 0, p, p, 1, 60, 1e-6, 0, None, 0, None) == -2       # D % 8
    assert L.mllm_hip_rmsnorm(p, 0, p, p, 1, 1 << 15, 1e-6, 0, None, 0, None) == -2  # D too long
    assert L.mllm_hip_rmsnorm(p, 0, p, p, 9, 64, 1e-6, 0, p, 0, None) == -2          # image wants rows <= 8
    assert L.mllm_hip_rmsnorm(p, 0, p, p, 1, 40, 1e-6, 0, p, 0, None) == -2          # image wants D % 32
    assert L.mllm_hip_rmsnorm(p + 4, 0, p, p, 1, 8, 1e-6, 0, None, 0, None) == -3
    assert L.mllm_hip_rmsnorm(None, 0, p, p, 1, 8, 1e-6, 0, None, 0, None) == -1
    assert L.mllm_hip_silu(p, p, 0, 12, None) == -2
    assert L.mllm_hip_add(p, None, p, 0, 1, 8, None, 0, None) == -1
    assert L.mllm_hip_topk(p, p, p, 1, 8, 9, 1, 1, None) == -2
    assert L.mllm_hip_topk(p, p, p, 1, 8, 0, 1, 1, None) == -2
    assert L.mllm_hip_softmax(p, None, 1, 8, None) == -1
    assert L.mllm_hip_moe_gate_set_form(2) == -1
    assert L.mllm_hip_moe_gate(p, 0, p, p, p, None, 1, 12, 4, 2, 1, None) == -2      # H % 8
    assert L.mllm_hip_moe_gate(p, 0, p, p, p, None, 1, 8, 4, 5, 1, None) == -2       # k > E
    assert L.mllm_hip_set_exp_mode(2) == -1
    assert L.mllm_hip_mlp_gate_up_q(0, p, p, p, 0, p, None, 9, 64, 64, 0, None) == -2  # at most eight rows
    assert L.mllm_hip_mlp_gate_up_q(0, p, p, p, 0, p, None, 1, 48, 64, 0, None) == -2  # I % 32
    assert L.mllm_hip_mlp_gate_up_q(0, p, p, p, 0, None, None, 1, 64, 64, 0, None) == -1  # no result asked for
    assert L.mllm_hip_mlp_gate_up_q(2, p, p, p, 0, p, None, 1, 64, 64, 0, None) == -1  # Q4_0 / Q8_0 only
