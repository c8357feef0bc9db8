"""Pins the oracle's restatements of the operators around Linear (RMSNorm, SiLU, softmax, top-k, MoE gate).

The reference's x86 kernels for these need Highway, which its tree does not carry, so they cannot be compiled here; every
function is instead checked against what the mathematics fixes, in float64, with checks chosen so that a dropped term, a
wrong sign or a wrong constant fails: the polynomial exp against exp(x) * exp(n * 2.1219444e-4) (the closed form of the
reference's reduction constants), RMSNorm / softmax / SiLU against their definitions, top-k against numpy's sort and the
properties the reference's own TopK test checks (tests/cpu/TopKKernelTest.hpp:13-70, shapes of tests/cpu/KernelTest.cpp:686)."""
import numpy as np

from oracle import oracle as orc

C2 = float(np.float32(2.12194440e-4))


def _exp_closed_form(x):
    """exp as the reference's constants make it: reduced argument x - n * (ln2_f32 - C2)"""
    x = np.asarray(x, np.float64)
    n = np.floor(x * float(np.float32(1.44269504088896341)) + 0.5)
    ln2f = float(np.float32(0.693147180559945309))
    return np.exp(x - n * ln2f + n * C2) * 2.0 ** n


def test_exp_poly_closed_form():
    x = np.concatenate([np.linspace(-87, 87, 4001), np.linspace(-1, 1, 1001), [0.0, -0.0, 1e-8, -1e-8]]).astype(np.float32)
    got = orc.exp_poly(x).astype(np.float64)
    want = _exp_closed_form(x)
    # fp32 rounding of n * ln2 (up to 86) in the reduction leaves up to |x| * 2^-24 on top of the polynomial's 2e-7
    assert np.all(np.abs(got / want - 1) < 5e-7 + np.abs(x) * 6e-8)
    # and the size of the deviation from exp itself: n * 2.12e-4 relative, i.e. NOT an accurate exp away from 0
    far = orc.exp_poly(np.float32([-10.0]))[0] / np.exp(-10.0) - 1
    assert abs(far - (np.exp(-14 * C2) - 1)) < 1e-6
    assert abs(orc.exp_poly(np.float32([0.0]))[0] - 1.0) < 2e-7
    # clamp: beyond +-88.376 the argument is held
    assert orc.exp_poly(np.float32([-200.0]))[0] == orc.exp_poly(np.float32([-88.3762626647949]))[0]
    assert np.isfinite(orc.exp_poly(np.float32([200.0]))[0])


def test_silu_vector_part_and_tail():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(8 * 13 + 5) * 4).astype(np.float32)
    y = orc.silu(x).astype(np.float64)
    xd = x.astype(np.float64)
    n_vec = x.size - x.size % 8
    want_vec = xd[:n_vec] / (1 + _exp_closed_form(-xd[:n_vec]))
    want_tail = xd[n_vec:] / (1 + np.exp(-xd[n_vec:]))
    assert np.max(np.abs(y[:n_vec] - want_vec)) < 1e-6 * np.max(np.abs(xd))
    assert np.max(np.abs(y[n_vec:] - want_tail)) < 1e-6 * np.max(np.abs(xd))
    assert orc.silu(np.zeros(8, np.float32)).tolist() == [0.0] * 8
    # silu(x) - silu(-x) = x holds for any exp with exp(-t) = 1 / exp(t); the polynomial satisfies it to rounding
    big = np.float32([3.0, -3.0, 0.5, -0.5, 7.0, -7.0, 1.0, -1.0])
    s = orc.silu(big).astype(np.float64)
    assert np.allclose(s[0::2] - s[1::2], big[0::2], rtol=2e-3)


def test_rmsnorm_definition():
    rng = np.random.default_rng(2)
    for D in (8, 128, 2560, 37):  # 37: vectors of eight + a tail of five
        x = rng.standard_normal((5, D)).astype(np.float32) * 3
        w = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
        for off in (False, True):
            y = orc.rmsnorm(x, w, 1e-6, off).astype(np.float64)
            xd, wd = x.astype(np.float64), w.astype(np.float64)
            want = xd / np.sqrt((xd * xd).mean(-1, keepdims=True) + 1e-6) * (wd + (1.0 if off else 0.0))
            assert np.max(np.abs(y - want)) < 2e-6 * np.max(np.abs(want))
    # epsilon matters on a zero row and the weight is applied once
    y = orc.rmsnorm(np.zeros((1, 16), np.float32), np.ones(16, np.float32), 1e-6)
    assert not np.any(y)
    y = orc.rmsnorm(np.full((1, 16), 2.0, np.float32), np.full(16, 3.0, np.float32), 0.0)
    assert np.allclose(y, 3.0, rtol=1e-6)


def test_rmsnorm_operation_order_in_whole_vectors_and_tail():
    """x86/rmsnorm.cpp:29-36,41-47: every whole vector of eight takes x * (w * rms), only the D % 8 tail takes
    x * rms * w.  The two orders differ in the last bit for many elements; both are computed here with numpy's fp32
    scalars (one IEEE rounding per operation, nothing shared with the C restatement)."""
    f = np.float32
    for D in (16, 64, 37, 2560):
        rng = np.random.default_rng(100 + D)
        # small integers: the sum of squares is exact in fp32 in any order, so rms is the same number for everybody
        x = rng.integers(-15, 16, (1, D)).astype(np.float32)
        x[0, -8:] = [3, -5, 7, 9, -11, 13, 14, -15]
        w = (1 + 0.2 * rng.standard_normal(D)).astype(np.float32)
        eps = f(1e-6)
        rms = f(1.0) / np.sqrt(f(np.sum(x.astype(np.float64) ** 2)) / f(D) + eps, dtype=np.float32)
        for off in (False, True):
            ww = w + f(1.0) if off else w
            vec_form = x[0] * (ww * rms)          # fp32 throughout
            tail_form = (x[0] * rms) * ww
            n_vec = D - D % 8
            want = np.concatenate([vec_form[:n_vec], tail_form[n_vec:]])
            got = orc.rmsnorm(x, w, 1e-6, off)[0]
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (D, off)
            # the case must be able to tell the orders apart in the last seven elements of the vector part
            lo, hi = max(0, n_vec - 7), n_vec
            assert np.any(vec_form[lo:hi].view(np.uint32) != tail_form[lo:hi].view(np.uint32)), (D, off)


def test_softmax_definition():
    rng = np.random.default_rng(3)
    for n in (4, 16, 17, 128, 133):
        x = (rng.standard_normal((7, n)) * 3).astype(np.float32)
        y = orc.softmax(x).astype(np.float64)
        d = x.astype(np.float64) - x.max(-1, keepdims=True).astype(np.float64)
        if n <= 16:
            e = np.exp(d)
        else:  # whole vectors of eight through the polynomial, the tail through expf
            nv = n - n % 8
            e = np.concatenate([_exp_closed_form(d[:, :nv]), np.exp(d[:, nv:])], axis=1)
        want = e / e.sum(-1, keepdims=True)
        assert np.max(np.abs(y - want)) < 1e-6
        assert np.allclose(y.sum(-1), 1.0, atol=1e-5)
        assert np.array_equal(np.argmax(y, -1), np.argmax(x, -1))


def test_topk_against_sort_and_reference_test_properties():
    rng = np.random.default_rng(4)
    # shapes and k of the reference's own test; values uniform in [-10, 10) like Tensor::random there
    for shape in [(10,), (1, 10), (5, 10), (2, 5, 10), (1, 4, 8, 16)]:
        x = rng.uniform(-10, 10, shape).astype(np.float32)
        v, i = orc.topk(x, 3)
        assert v.shape == shape[:-1] + (3,) and i.shape == v.shape and v.dtype == np.float32 and i.dtype == np.int32
        assert np.all(v[..., 1:] <= v[..., :-1])
        order = np.argsort(-x, axis=-1, kind="stable")[..., :3]
        assert np.array_equal(i, order)
        assert np.array_equal(v, np.take_along_axis(x, order, -1))
    x = rng.standard_normal((6, 128)).astype(np.float32)
    v, i = orc.topk(x, 8, largest=True, sorted=False)
    want = np.sort(np.argsort(-x, axis=-1, kind="stable")[:, :8], axis=-1)
    assert np.array_equal(i, want) and np.array_equal(v, np.take_along_axis(x, want, -1))
    v, i = orc.topk(x, 5, largest=False, sorted=True)
    want = np.argsort(x, axis=-1, kind="stable")[:, :5]
    assert np.array_equal(i, want)
    # ties: the kept VALUES are fixed, the lowest indices are kept; k == len returns everything
    t = np.float32([[1, 3, 3, 2, 3, 0]])
    v, i = orc.topk(t, 2)
    assert v.tolist() == [[3, 3]] and i.tolist() == [[1, 2]]
    v, i = orc.topk(t, 6, sorted=False)
    assert i.tolist() == [[0, 1, 2, 3, 4, 5]] and np.array_equal(v, t)


def test_moe_gate_composition():
    rng = np.random.default_rng(5)
    M, H, E, k = 9, 64, 32, 4
    x = rng.standard_normal((M, H)).astype(np.float32)
    w = (rng.standard_normal((E, H)) * 0.2).astype(np.float32)
    ids, wt, sc = orc.moe_gate(x, w, k, norm=True)
    logits = x.astype(np.float64) @ w.astype(np.float64).T
    d = logits - logits.max(-1, keepdims=True)
    e = _exp_closed_form(d)
    p = e / e.sum(-1, keepdims=True)
    assert np.max(np.abs(sc - p)) < 2e-6
    want_ids = np.sort(np.argsort(-p, axis=-1, kind="stable")[:, :k], axis=-1)
    assert np.array_equal(ids, want_ids)
    pw = np.take_along_axis(p, want_ids, -1)
    assert np.max(np.abs(wt - pw / pw.sum(-1, keepdims=True))) < 2e-6
    assert np.allclose(wt.sum(-1), 1.0, atol=1e-6)
    _, wt2, _ = orc.moe_gate(x, w, k, norm=False)
    assert np.max(np.abs(wt2 - pw)) < 2e-6


def test_moe_ffn_kq_composition_against_float64_model():
    """The K-quant MoE oracle is a composition of linear_kq and silu (each pinned on its own).  What the composition adds --
    which expert serves which slot, gate against up, the weighted sum -- is checked against a float64 model on the dequantized
    weights; the two differ by the Q8_K activation noise only (under one percent), while a swapped operand, a wrong expert
    or a dropped slot would show as tens of percent.  Slots with an expert id outside [0, E) contribute nothing."""
    from mllm_amd import synth
    rng = synth.rng_for(9, 1)
    for wt in (2, 3):
        T, H, I, E, k = 3, 256, 256, 4, 2
        Wg = synth.make_weight(rng, wt, E * I, H).reshape(E, I, H // 256, -1)
        Wu = synth.make_weight(rng, wt, E * I, H).reshape(E, I, H // 256, -1)
        Wd = synth.make_weight(rng, wt, E * H, I).reshape(E, H, I // 256, -1)
        ids, w = synth.make_moe_routing(rng, T, E, k)
        ids[1, 1] = E + 2
        x = synth.make_x_fp32(rng, T, H)
        y = orc.moe_ffn_kq(x, ids, w, Wg, Wu, Wd, wt)
        Dg = [orc.dequantize_k(Wg[e], wt).astype(np.float64) for e in range(E)]
        Du = [orc.dequantize_k(Wu[e], wt).astype(np.float64) for e in range(E)]
        Dd = [orc.dequantize_k(Wd[e], wt).astype(np.float64) for e in range(E)]
        ref = np.zeros((T, H))
        for t in range(T):
            for j in range(k):
                e = ids[t, j]
                if 0 <= e < E:
                    g, u = Dg[e] @ x[t], Du[e] @ x[t]
                    ref[t] += w[t, j] * (Dd[e] @ (g / (1 + np.exp(-g)) * u))
        assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 0.03
