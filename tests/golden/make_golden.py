"""Writes the golden vectors under tests/golden/ from the reference's own compiled kernels.

Run where the reference checkout is mounted:   make -C oracle ref && python tests/golden/make_golden.py
The vectors are produced by oracle/_ref/libmllm_ref.so (the reference's quantize_q8.cpp, quantize_q4.cpp and vec_dot.cpp
compiled unchanged) on seeded inputs; the inputs are stored next to the outputs so the fixtures are self-contained.

  q8_0_actquant.npz   quantize_row_q8_0: fp32 rows -> int8 codes + effective scale values (special rows included)
  gemv_kat.npz        Q4_0 / Q8_0 Linear (quantize_row_q8_0 + vec_dot_*): N=64, K=256, M in {1,3,4,8}, with/without bias
  x86_scale_grid.npz  what a stored scale pattern reads back as on the x86 build, 4096 sampled patterns
  dequant_kat.npz     dequantize_row_q4_0 / dequantize_row_q8_0 on a few rows
  kquant_kat.npz      Q4_K / Q6_K: blocks made by the reference's own offline quantizers from fp32 weights, their
                      dequantized values, quantize_row_q8_K of the activations, and the Linear outputs (vec_dot_q4_K_q8_K /
                      vec_dot_q6_K_q8_K); written alone with `--only kquant`
  kquant_quantizer_kat.npz  fp32 weights and the super-blocks the reference's offline Q4_K / Q6_K quantizers make of them; written
                      alone with `--only kquant_quantizer`
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from mllm_amd import synth  # noqa: E402
from oracle import oracle as orc  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))


def actquant_rows(rng, K=256):
    rows = []
    rows.append(rng.standard_normal(K).astype(np.float32))                      # plain
    r = rng.standard_normal(K).astype(np.float32); r[32:64] = 0.0; rows.append(r)      # an all-zero block
    r = rng.standard_normal(K).astype(np.float32); r[5] *= 20.0; r[100] *= -20.0; rows.append(r)  # outliers
    r = np.zeros(K, np.float32)                                                  # exact ties: amax = 127 -> id = 1
    r[:] = (rng.integers(-126, 126, K) + 0.5).astype(np.float32); r[::32] = 127.0; rows.append(r)
    r = (rng.standard_normal(K) * 1e-6).astype(np.float32); rows.append(r)       # tiny -> subnormal fp16 scales
    r = (rng.standard_normal(K) * 3e4).astype(np.float32); rows.append(r)        # large
    r = rng.standard_normal(K).astype(np.float32); r[0:32] = -np.abs(r[0:32]); rows.append(r)   # amax on a negative
    r = synth.bf16_bits_to_fp32(synth.fp32_to_bf16_bits(rng.standard_normal(K).astype(np.float32))); rows.append(r)
    return np.stack(rows)


def kquant():
    rk = np.random.default_rng(synth.SEED_BASE + 79)
    N, K = 24, 512
    out = {}
    for name, wtype in (("q4_k", 2), ("q6_k", 3)):
        w = (rk.standard_normal((N, K)) * 0.04).astype(np.float32)
        w[0, :256] = 0.0                      # an all-zero super-block
        w[1, :32] = 0.3                       # a constant sub-block
        W = orc.ref_quantize_rows_k(w, wtype)
        out[f"{name}_W"] = W
        out[f"{name}_deq"] = orc.ref_dequantize_k(W, wtype)
        bias = rk.standard_normal(N).astype(np.float32)
        out[f"{name}_bias"] = bias
        for M in (1, 3, 8):
            x = rk.standard_normal((M, K)).astype(np.float32)
            out[f"{name}_x{M}"] = x
            out[f"{name}_y{M}"] = orc.ref_linear_kq(x, W, wtype, bias)
    x = (rk.standard_normal((4, K)) * 2).astype(np.float32)
    x[1, 256:] = 0.0
    x[2, 3], x[2, 77] = 9.0, -9.0
    q, d, bs = orc.ref_quantize_rows_q8_K(x)
    bs[np.repeat(d == 0, 16, axis=1)] = 0     # the reference leaves the sums of an all-zero block unwritten
    out.update(q8k_x=x, q8k_q=q, q8k_d=d, q8k_bsums=bs)
    np.savez_compressed(os.path.join(OUT, "kquant_kat.npz"), **out)


def kquant_quantizer():
    """inputs and outputs of the reference's offline Q4_K / Q6_K quantizers (quantize_row_q4_K / _q6_K compiled from the
    reference's sources): canonical super-blocks whose fp16 fields hold the patterns an x86 read of the written block yields"""
    rq = np.random.default_rng(synth.SEED_BASE + 80)
    N, K = 16, 512
    w = (rq.standard_normal((N, K)) * 0.04).astype(np.float32)
    w[0, :256] = 0.0                                         # an all-zero super-block
    w[1, :32] = 0.3                                          # constant sub-blocks, positive and negative
    w[1, 32:64] = -0.3
    w[2, :256] = np.abs(w[2, :256])                          # all positive: every offset is zero
    w[3, :256] *= 50
    w[4, :16] = 0.0                                          # an all-zero group of 16 inside a live super-block
    w[5, :256] = np.float32(1e-3) * rq.integers(-8, 8, 256)  # few distinct values
    w[6, 0], w[6, 5] = 0.9, -0.9                             # equal magnitudes, opposite signs
    np.savez_compressed(os.path.join(OUT, "kquant_quantizer_kat.npz"), w=w, q4_k_blocks=orc.ref_quantize_rows_k(w, 2),
                        q6_k_blocks=orc.ref_quantize_rows_k(w, 3))


def main():
    if not orc.ref_available():
        raise SystemExit("oracle/_ref/libmllm_ref.so missing: run `make -C oracle ref` where the reference is mounted")
    if sys.argv[1:] == ["--only", "kquant"]:
        kquant()
        return
    if sys.argv[1:] == ["--only", "kquant_quantizer"]:
        kquant_quantizer()
        return

    rng = np.random.default_rng(synth.SEED_BASE + 77)
    x = actquant_rows(rng)
    qs, d_eff = orc.ref_quantize_rows_q8_0(x)
    np.savez_compressed(os.path.join(OUT, "q8_0_actquant.npz"), x=x, qs=qs, d_eff=d_eff)

    kat = {}
    N, K = 64, 256
    for wname, wtype in (("q4_0", 0), ("q8_0", 1)):
        W = synth.make_weight(rng, wtype, N, K)
        bias = rng.standard_normal(N).astype(np.float32)
        kat[f"{wname}_W"] = W
        kat[f"{wname}_bias"] = bias
        for M in (1, 3, 4, 8):
            xx = synth.make_x_fp32(rng, M, K)
            kat[f"{wname}_x{M}"] = xx
            kat[f"{wname}_y{M}"] = orc.ref_linear_q(xx, W, wtype)
            kat[f"{wname}_yb{M}"] = orc.ref_linear_q(xx, W, wtype, bias)
    np.savez_compressed(os.path.join(OUT, "gemv_kat.npz"), **kat)

    pats = np.unique(np.concatenate([
        rng.integers(0, 65520, 3500).astype(np.uint16),
        np.arange(2040, 2060, dtype=np.uint16), np.arange(4090, 4110, dtype=np.uint16),
        np.arange(0x3bf0, 0x3c10, dtype=np.uint16), np.arange(0x1ff0, 0x2010, dtype=np.uint16),
        np.array([0, 1, 2047, 2048, 2049, 0x7bff, 0x7c00, 0x8000, 65519], dtype=np.uint16)]))
    vals = np.array([orc.ref().ref_scale_store_load(int(b)) for b in pats], dtype=np.float32)
    np.savez_compressed(os.path.join(OUT, "x86_scale_grid.npz"), bits=pats, value_bits=vals.view(np.uint32))

    W4 = synth.make_q4_0(rng, 4, 128)
    W8 = synth.make_q8_0(rng, 4, 128)
    np.savez_compressed(os.path.join(OUT, "dequant_kat.npz"), W4=W4, y4=orc.ref_dequantize(W4, 0), W8=W8,
                        y8=orc.ref_dequantize(W8, 1))
    # offline weight quantizers (quantize_row_q4_0 / quantize_row_q8_0 writing blocks on x86): inputs, the codes, and the
    # scale pattern / value an x86 read of the written block yields
    rq = np.random.default_rng(synth.SEED_BASE + 78)
    w = (rq.standard_normal((12, 128)) * 0.05).astype(np.float32)
    w[1, :32] = 0.0
    w[2, :32] = np.float32(-0.5) * np.arange(32) / 31
    w[3, :32] = np.float32(0.5) * np.arange(32) / 31
    w[4, :32] = np.float32(8.0) * np.linspace(-1, 1, 32)
    q8_codes, q8_d = orc.ref_quantize_rows_q8_0(w)
    np.savez_compressed(os.path.join(OUT, "weight_quantizer_kat.npz"), w=w, q4_blocks=orc.ref_quantize_rows_q4_0(w),
                        q8_codes=q8_codes, q8_d_eff=q8_d)
    kquant()
    kquant_quantizer()
    for f in sorted(os.listdir(OUT)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(OUT, f)))


if __name__ == "__main__":
    main()
