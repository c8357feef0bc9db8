"""Seeded synthetic inputs of the benchmark configurations (numpy only, no GPU, no oracle).

Weight blocks are produced in the reference's array-of-structures layout
(mllm/core/DataTypes.hpp:110-121,164-170): uint8 [N, K/32, 18] for Q4_0 ({fp16 d; u8 qs[16]}, element j in the low
nibble of qs[j], element j+16 in the high nibble, value = nibble - 8) and uint8 [N, K/32, 34] for Q8_0
({fp16 d; i8 qs[32]}).  The `d` field is an IEEE fp16 bit pattern.

Block scales are snapped to the grid the x86 build of the reference can represent in a block: it stores the 16-bit
pattern as a *number* in a half-precision field, i.e. rounded to 11 significant bits.  On that grid the IEEE reading and
the x86 reading of a stored scale agree, so one weight file serves both conventions.
"""
import numpy as np

SEED_BASE = 20260101
QK = 32


def rng_for(config_index, extra=0):
    return np.random.default_rng(SEED_BASE + config_index + 1000 * extra)


def snap_scale_bits(bits):
    """Round 16-bit patterns (taken as integers) to 11 significant bits, nearest even."""
    b = np.asarray(bits, dtype=np.uint32)
    out = b.copy()
    big = b >= 2048
    if big.any():
        bb = b[big]
        p = np.floor(np.log2(bb.astype(np.float64))).astype(np.uint32)
        sh = p - 10
        q = bb >> sh
        rem = bb & ((np.uint32(1) << sh) - 1)
        half = np.uint32(1) << (sh - 1)
        up = (rem > half) | ((rem == half) & ((q & 1) == 1))
        out[big] = (q + up.astype(np.uint32)) << sh
    return out.astype(np.uint16)


def fp32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_fp32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def _scales(rng, shape, sigma):
    s = (np.abs(rng.normal(0.0, sigma, size=shape)) / 7.0).astype(np.float32)
    return snap_scale_bits(s.astype(np.float16).view(np.uint16))


def pack_q4_0(codes, d_bits):
    """codes int in [-8,7] [N, K]; d_bits uint16 [N, K/32] -> uint8 [N, K/32, 18]."""
    N, K = codes.shape
    nb = K // QK
    nibs = (codes.reshape(N, nb, QK) + 8).astype(np.uint8)
    out = np.empty((N, nb, 18), np.uint8)
    out[:, :, 0:2] = np.ascontiguousarray(d_bits, dtype="<u2").reshape(N, nb, 1).view(np.uint8)
    out[:, :, 2:] = nibs[:, :, :16] | (nibs[:, :, 16:] << 4)
    return out


def pack_q8_0(codes, d_bits):
    """codes int8 [N, K]; d_bits uint16 [N, K/32] -> uint8 [N, K/32, 34]."""
    N, K = codes.shape
    nb = K // QK
    out = np.empty((N, nb, 34), np.uint8)
    out[:, :, 0:2] = np.ascontiguousarray(d_bits, dtype="<u2").reshape(N, nb, 1).view(np.uint8)
    out[:, :, 2:] = codes.astype(np.int8).reshape(N, nb, QK).view(np.uint8)
    return out


def make_q4_0(rng, N, K, sigma=0.02):
    codes = rng.integers(-8, 8, size=(N, K), dtype=np.int8)
    return pack_q4_0(codes, _scales(rng, (N, K // QK), sigma))


def make_q8_0(rng, N, K, sigma=0.02):
    codes = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    return pack_q8_0(codes, _scales(rng, (N, K // QK), sigma))


def make_q4_K(rng, N, K, sigma=0.02):
    """random block_q4_K rows, uint8 [N, K/256, 144]: fp16 d and dmin on the grid both scale conventions read alike,
    6-bit scales / mins and nibbles uniform"""
    nb = K // 256
    out = np.empty((N, nb, 144), np.uint8)
    out[:, :, 0:2] = np.ascontiguousarray(_scales(rng, (N, nb), sigma / 8), dtype="<u2").reshape(N, nb, 1).view(np.uint8)
    out[:, :, 2:4] = np.ascontiguousarray(_scales(rng, (N, nb), sigma / 8), dtype="<u2").reshape(N, nb, 1).view(np.uint8)
    out[:, :, 4:] = rng.integers(0, 256, size=(N, nb, 140), dtype=np.uint8)
    return out


def make_q6_K(rng, N, K, sigma=0.02):
    """random block_q6_K rows, uint8 [N, K/256, 210]"""
    nb = K // 256
    out = np.empty((N, nb, 210), np.uint8)
    out[:, :, :208] = rng.integers(0, 256, size=(N, nb, 208), dtype=np.uint8)
    out[:, :, 208:] = np.ascontiguousarray(_scales(rng, (N, nb), sigma / 64), dtype="<u2").reshape(N, nb, 1).view(np.uint8)
    return out


def make_weight(rng, wtype, N, K):
    if wtype == 2:
        return make_q4_K(rng, N, K)
    if wtype == 3:
        return make_q6_K(rng, N, K)
    return make_q4_0(rng, N, K) if wtype == 0 else make_q8_0(rng, N, K)


def make_x_fp32(rng, M, K):
    return rng.standard_normal((M, K), dtype=np.float32)


def make_x_bf16(rng, M, K):
    """returns (bf16 bit patterns uint16 [M, K], the same values as fp32)."""
    bits = fp32_to_bf16_bits(rng.standard_normal((M, K), dtype=np.float32))
    return bits, bf16_bits_to_fp32(bits)


# Qwen3-4B decoder-layer projections: name -> (N out, K in)
QWEN3_4B_LAYER = {
    "q_proj": (4096, 2560),
    "k_proj": (1024, 2560),
    "v_proj": (1024, 2560),
    "o_proj": (2560, 4096),
    "gate_proj": (9728, 2560),
    "up_proj": (9728, 2560),
    "down_proj": (2560, 9728),
}


def gemv_algorithmic_bytes(wtype, M, N, K, x_bytes):
    """weights (18 or 34 bytes per 32-element block) + activations + fp32 outputs."""
    return N * (K // QK) * (18 if wtype == 0 else 34) + M * K * x_bytes + M * N * 4


# ----------------------------------------------------------------------------- W4A16 (group 128, uint4 + zero point)
def pack_nibbles(a):
    """uint8 values in [0,15] [..., L] -> [..., ceil(L/2)], element 2j in the low nibble of byte j."""
    a = np.asarray(a, dtype=np.uint8)
    if a.shape[-1] % 2:
        a = np.concatenate([a, np.zeros(a.shape[:-1] + (1,), np.uint8)], axis=-1)
    return (a[..., 0::2] | (a[..., 1::2] << 4)).astype(np.uint8)


def make_w4a16(rng, N, K, group=128, sigma=0.01):
    """returns (qw uint8 [N, K/2], scale fp16 bits uint16 [N, K/group], zp uint8 [N, ceil(G/2)], q, z unpacked)."""
    G = K // group
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    z = rng.integers(0, 16, size=(N, G), dtype=np.uint8)
    s = np.abs(rng.normal(0.0, sigma, size=(N, G))).astype(np.float32).astype(np.float16).view(np.uint16)
    return pack_nibbles(q), s, pack_nibbles(z), q, z


def pack_awq_cols(codes):
    """codes [R, N] in [0, 15] -> int32 [R, N/8] as an AWQ checkpoint stores them: each run of eight columns reordered to
    (0, 2, 4, 6, 1, 3, 5, 7) and then packed column i of the run into bits 4 i .. 4 i + 3 (the pack_cols of
    pymllm/quantization/methods/awq_marlin.py:188-199 applied to the interleaved columns)."""
    codes = np.asarray(codes, dtype=np.uint32)
    R, N = codes.shape
    assert N % 8 == 0
    inter = codes.reshape(-1, 8)[:, [0, 2, 4, 6, 1, 3, 5, 7]].reshape(R, N)
    out = np.zeros((R, N // 8), np.uint32)
    for i in range(8):
        out |= inter[:, i::8] << np.uint32(4 * i)
    return out.view(np.int32)


def make_awq(rng, N, K, group=128, sigma=0.01):
    """returns (qweight int32 [K, N/8], qzeros int32 [G, N/8], scales fp16 bits [G, N], q [N, K], z [N, G], s bits [N, G])."""
    G = K // group
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    z = rng.integers(0, 16, size=(N, G), dtype=np.uint8)
    s = np.abs(rng.normal(0.0, sigma, size=(N, G))).astype(np.float32).astype(np.float16).view(np.uint16)
    return pack_awq_cols(q.T), pack_awq_cols(z.T), np.ascontiguousarray(s.T), q, z, s


# ----------------------------------------------------------------------------- W8A8
def make_w8a8(rng, M, N, K):
    """A bf16 bits [M, K] ~N(0,1) with 1 % of entries x20; W int8 [N, K]; w_scale fp32 [N]."""
    a = rng.standard_normal((M, K), dtype=np.float32)
    a = np.where(rng.random((M, K)) < 0.01, a * 20.0, a).astype(np.float32)
    a_bits = fp32_to_bf16_bits(a)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    w_scale = ((rng.random(N, dtype=np.float32) + np.float32(0.01)) * np.float32(0.01)).astype(np.float32)
    return a_bits, W, w_scale


# ----------------------------------------------------------------------------- MoE routing
def make_moe_routing(rng, T, E, k, zipf_s=1.1):
    """Zipf(s) expert popularity over a seeded permutation; k distinct experts per token; softmax weights of N(0,1)."""
    p = np.arange(1, E + 1, dtype=np.float64) ** (-zipf_s)
    p = p[rng.permutation(E)]
    p /= p.sum()
    ids = np.empty((T, k), np.int32)
    for t in range(T):
        ids[t] = rng.choice(E, size=k, replace=False, p=p)
    logits = rng.standard_normal((T, k)).astype(np.float32)
    w = np.exp(logits - logits.max(axis=1, keepdims=True))
    w = (w / w.sum(axis=1, keepdims=True)).astype(np.float32)
    return ids, w


def make_moe_weights(rng, E, H, I, wtype=0):
    """(Wg [E, I, H/32, blk], Wu same, Wd [E, H, I/32, blk])."""
    Wg = make_weight(rng, wtype, E * I, H).reshape(E, I, H // QK, -1)
    Wu = make_weight(rng, wtype, E * I, H).reshape(E, I, H // QK, -1)
    Wd = make_weight(rng, wtype, E * H, I).reshape(E, H, I // QK, -1)
    return Wg, Wu, Wd
