"""Synthetic quantized-weight makers for tests and the benchmark (TEST INFRASTRUCTURE ONLY).

The reference has no F32 -> Q4_0/Q4_K/Q6_K quantizer (only dequantizers), so these are
not restatements of reference code paths, with one exception: the block *encoders*
(encode_q4_0_block, encode_q8_0_block, encode_q4_k_block, encode_q6_k_block; the Q5_0 / Q5_K encoders are
written from the layout comments of dequant.go, the reference's tests hold none) follow the
helpers in the reference's own tests, which define the byte layout independently of
dequant.go:
  createQ4_0Block  inference/backend/metal/q4_kernel_test.go:19-38
  createQ8_0Block  inference/backend/metal/q8_0_matmul_test.go:22-35
  createQ4_KBlock  inference/backend/metal/q4k_kernel_test.go:33-79
  createQ6_KBlock  inference/backend/metal/q6k_kernel_test.go:19-70
quantize_q4_0 / quantize_q8_0 use the llama.cpp convention (signed-absmax / -8 for
Q4_0, absmax / 127 for Q8_0). random_q4_k / random_q6_k draw valid blocks at random.
"""
import numpy as np


def _f16_bits(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


# ------------------------------------------------------------------ encoders (layout definition)
def encode_q4_0_block(scale, values32):
    """values32: 32 ints in [0,15]; elt i -> low nibble of byte i (i<16), elt i+16 -> high nibble."""
    v = np.asarray(values32, dtype=np.uint8)
    assert v.size == 32
    out = np.zeros(18, dtype=np.uint8)
    out[0:2] = np.frombuffer(_f16_bits([scale]).tobytes(), dtype=np.uint8)
    out[2:18] = (v[:16] & 0xF) | ((v[16:] & 0xF) << 4)
    return out


def encode_q8_0_block(scale, values32):
    v = np.asarray(values32, dtype=np.int8)
    assert v.size == 32
    out = np.zeros(34, dtype=np.uint8)
    out[0:2] = np.frombuffer(_f16_bits([scale]).tobytes(), dtype=np.uint8)
    out[2:34] = v.view(np.uint8)
    return out


def pack_q4_k_scales(scales8, mins8):
    s = [int(x) for x in scales8]
    m = [int(x) for x in mins8]
    sd = np.zeros(12, dtype=np.uint8)
    for i in range(4):
        sd[i] = (s[i] & 0x3F) | ((s[4 + i] >> 4) << 6)
        sd[4 + i] = (m[i] & 0x3F) | ((m[4 + i] >> 4) << 6)
        sd[8 + i] = (s[4 + i] & 0x0F) | ((m[4 + i] & 0x0F) << 4)
    return sd


def encode_q4_k_block(d, dmin, scales8, mins8, values256):
    v = np.asarray(values256, dtype=np.uint8)
    assert v.size == 256
    out = np.zeros(144, dtype=np.uint8)
    out[0:2] = np.frombuffer(_f16_bits([d]).tobytes(), dtype=np.uint8)
    out[2:4] = np.frombuffer(_f16_bits([dmin]).tobytes(), dtype=np.uint8)
    out[4:16] = pack_q4_k_scales(scales8, mins8)
    for g in range(4):
        lo = v[g * 64:g * 64 + 32] & 0xF
        hi = v[g * 64 + 32:g * 64 + 64] & 0xF
        out[16 + g * 32:16 + g * 32 + 32] = lo | (hi << 4)
    return out


def encode_q6_k_block(d, scales16, values256):
    """values256: signed 6-bit values in [-32,31]."""
    vals = np.asarray(values256, dtype=np.int32) + 32
    assert vals.size == 256
    out = np.zeros(210, dtype=np.uint8)
    for n in range(2):
        for l in range(32):
            v1, v2, v3, v4 = (int(vals[n * 128 + l]), int(vals[n * 128 + l + 32]),
                              int(vals[n * 128 + l + 64]), int(vals[n * 128 + l + 96]))
            out[n * 64 + l] = (v1 & 0xF) | ((v3 & 0xF) << 4)
            out[n * 64 + l + 32] = (v2 & 0xF) | ((v4 & 0xF) << 4)
            out[128 + n * 32 + l] = ((v1 >> 4) & 3) | (((v2 >> 4) & 3) << 2) | (((v3 >> 4) & 3) << 4) | (((v4 >> 4) & 3) << 6)
    out[192:208] = np.asarray(scales16, dtype=np.int8).view(np.uint8)
    out[208:210] = np.frombuffer(_f16_bits([d]).tobytes(), dtype=np.uint8)
    return out


def encode_q5_0_block(scale, values32):
    """values32: 32 ints in [0,31]. Written from the format's description (dequant.go:92-99: [d:f16][qh:4][qs:16],
    the fifth bit of element i is bit i of the little-endian qh), not from the decoder's loop."""
    v = np.asarray(values32, dtype=np.uint32)
    assert v.size == 32
    out = np.zeros(22, dtype=np.uint8)
    out[0:2] = np.frombuffer(_f16_bits([scale]).tobytes(), dtype=np.uint8)
    qh = 0
    for i in range(32):
        qh |= ((int(v[i]) >> 4) & 1) << i
    out[2:6] = np.frombuffer(np.uint32(qh).tobytes(), dtype=np.uint8)
    out[6:22] = ((v[:16] & 0xF) | ((v[16:] & 0xF) << 4)).astype(np.uint8)
    return out


def encode_q5_k_block(d, dmin, scales8, mins8, values256):
    """values256: ints in [0,31]. Layout from dequant.go:411-422: Q4_K's header, then qh[32] where qh[l]
    carries one bit each for the elements l, l+32, ..., l+224 (bit e // 32 of qh[e % 32]), then the nibbles
    in Q4_K's order."""
    v = np.asarray(values256, dtype=np.uint8)
    assert v.size == 256
    out = np.zeros(176, dtype=np.uint8)
    out[0:2] = np.frombuffer(_f16_bits([d]).tobytes(), dtype=np.uint8)
    out[2:4] = np.frombuffer(_f16_bits([dmin]).tobytes(), dtype=np.uint8)
    out[4:16] = pack_q4_k_scales(scales8, mins8)
    for e in range(256):
        out[16 + e % 32] |= ((int(v[e]) >> 4) & 1) << (e // 32)
    for g in range(4):
        lo = v[g * 64:g * 64 + 32] & 0xF
        hi = v[g * 64 + 32:g * 64 + 64] & 0xF
        out[48 + g * 32:48 + g * 32 + 32] = lo | (hi << 4)
    return out


# ------------------------------------------------------------------ bulk synthetic quantizers
def quantize_q4_0(w):
    """w [N,K] float32 -> uint8 [N, K/32*18]. llama.cpp convention: d = signed absmax / -8,
    q = min(15, floor(x/d + 8.5))."""
    w = np.asarray(w, dtype=np.float32)
    n, k = w.shape
    assert k % 32 == 0
    blk = w.reshape(n, k // 32, 32)
    idx = np.abs(blk).argmax(axis=2)
    mx = np.take_along_axis(blk, idx[..., None], axis=2)[..., 0]
    d = mx / -8.0
    inv = np.where(d != 0, 1.0 / np.where(d != 0, d, 1), 0).astype(np.float32)
    q = np.minimum(15, np.floor(blk * inv[..., None] + 8.5)).astype(np.int32).clip(0, 15).astype(np.uint8)
    out = np.zeros((n, k // 32, 18), dtype=np.uint8)
    out[..., 0:2] = d.astype(np.float16).view(np.uint16)[..., None].view(np.uint8).reshape(n, k // 32, 2)
    out[..., 2:18] = q[..., :16] | (q[..., 16:] << 4)
    return out.reshape(n, -1)


def quantize_q8_0(w):
    """w [N,K] float32 -> uint8 [N, K/32*34]. d = absmax/127, q = round(x/d)."""
    w = np.asarray(w, dtype=np.float32)
    n, k = w.shape
    assert k % 32 == 0
    blk = w.reshape(n, k // 32, 32)
    amax = np.abs(blk).max(axis=2)
    d = amax / 127.0
    inv = np.where(d != 0, 1.0 / np.where(d != 0, d, 1), 0).astype(np.float32)
    q = np.rint(blk * inv[..., None]).clip(-127, 127).astype(np.int8)
    out = np.zeros((n, k // 32, 34), dtype=np.uint8)
    out[..., 0:2] = d.astype(np.float16).view(np.uint16)[..., None].view(np.uint8).reshape(n, k // 32, 2)
    out[..., 2:34] = q.view(np.uint8)
    return out.reshape(n, -1)


def random_q4_k(rng, n, k, d_scale=0.02 / 8 / 32):
    """Random valid Q4_K rows [N, K/256*144]: d, dmin = |N(0,1)|*d_scale (f16), 6-bit
    scales/mins uniform, nibbles uniform. The dequantised weights have a std near 0.02."""
    assert k % 256 == 0
    nb = n * (k // 256)
    out = np.zeros((nb, 144), dtype=np.uint8)
    d = (np.abs(rng.standard_normal(nb)) * d_scale + d_scale * 0.1).astype(np.float16)
    dmin = (np.abs(rng.standard_normal(nb)) * d_scale + d_scale * 0.1).astype(np.float16)
    out[:, 0:2] = d.view(np.uint16)[:, None].view(np.uint8).reshape(nb, 2)
    out[:, 2:4] = dmin.view(np.uint16)[:, None].view(np.uint8).reshape(nb, 2)
    out[:, 4:16] = rng.integers(0, 256, size=(nb, 12), dtype=np.uint8)
    out[:, 16:144] = rng.integers(0, 256, size=(nb, 128), dtype=np.uint8)
    return out.reshape(n, -1)


def random_q6_k(rng, n, k, d_scale=0.02 / 18 / 64):
    """Random valid Q6_K rows [N, K/256*210]."""
    assert k % 256 == 0
    nb = n * (k // 256)
    out = np.zeros((nb, 210), dtype=np.uint8)
    out[:, 0:192] = rng.integers(0, 256, size=(nb, 192), dtype=np.uint8)
    out[:, 192:208] = rng.integers(-128, 128, size=(nb, 16), dtype=np.int8).view(np.uint8)
    d = (np.abs(rng.standard_normal(nb)) * d_scale + d_scale * 0.1).astype(np.float16)
    out[:, 208:210] = d.view(np.uint16)[:, None].view(np.uint8).reshape(nb, 2)
    return out.reshape(n, -1)


def quantize_q5_0(w):
    """w [N,K] float32 -> uint8 [N, K/32*22]. llama.cpp convention: d = signed absmax / -16,
    q = min(31, floor(x/d + 16.5))."""
    w = np.asarray(w, dtype=np.float32)
    n, k = w.shape
    assert k % 32 == 0
    nb = k // 32
    blk = w.reshape(n, nb, 32)
    idx = np.abs(blk).argmax(axis=2)
    mx = np.take_along_axis(blk, idx[..., None], axis=2)[..., 0]
    d = mx / -16.0
    inv = np.where(d != 0, 1.0 / np.where(d != 0, d, 1), 0).astype(np.float32)
    q = np.minimum(31, np.floor(blk * inv[..., None] + 16.5)).astype(np.int32).clip(0, 31).astype(np.uint32)
    out = np.zeros((n, nb, 22), dtype=np.uint8)
    out[..., 0:2] = d.astype(np.float16).view(np.uint16)[..., None].view(np.uint8).reshape(n, nb, 2)
    qh = ((q >> 4) << np.arange(32, dtype=np.uint32)).sum(axis=2, dtype=np.uint64).astype(np.uint32)
    out[..., 2:6] = qh[..., None].view(np.uint8).reshape(n, nb, 4)
    out[..., 6:22] = ((q[..., :16] & 0xF) | ((q[..., 16:] & 0xF) << 4)).astype(np.uint8)
    return out.reshape(n, -1)


def random_q5_k(rng, n, k, d_scale=0.02 / 16 / 32):
    """Random valid Q5_K rows [N, K/256*176]."""
    assert k % 256 == 0
    nb = n * (k // 256)
    out = np.zeros((nb, 176), dtype=np.uint8)
    d = (np.abs(rng.standard_normal(nb)) * d_scale + d_scale * 0.1).astype(np.float16)
    dmin = (np.abs(rng.standard_normal(nb)) * d_scale + d_scale * 0.1).astype(np.float16)
    out[:, 0:2] = d.view(np.uint16)[:, None].view(np.uint8).reshape(nb, 2)
    out[:, 2:4] = dmin.view(np.uint16)[:, None].view(np.uint8).reshape(nb, 2)
    out[:, 4:176] = rng.integers(0, 256, size=(nb, 172), dtype=np.uint8)
    return out.reshape(n, -1)


def quantize_bf16(w):
    """w [N,K] float32 -> uint8 [N, K*2]: the upper 16 bits of each float32, rounded to nearest even."""
    u = np.ascontiguousarray(w, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r.view(np.uint8).reshape(w.shape[0], -1)


def random_quant(fmt, rng, n, k, std=0.02):
    """Quantized [N,K] weight of format fmt (1=Q4_0, 2=Q8_0, 3=Q4_K, 4=Q6_K, 5=Q5_0, 6=Q5_K, 7=BF16) with
    dequantised std near `std`."""
    if fmt == 1:
        return quantize_q4_0(rng.standard_normal((n, k), dtype=np.float32) * std)
    if fmt == 2:
        return quantize_q8_0(rng.standard_normal((n, k), dtype=np.float32) * std)
    if fmt == 3:
        return random_q4_k(rng, n, k, d_scale=std / 8 / 32)
    if fmt == 4:
        return random_q6_k(rng, n, k, d_scale=std / 18 / 64)
    if fmt == 5:
        return quantize_q5_0(rng.standard_normal((n, k), dtype=np.float32) * std)
    if fmt == 6:
        return random_q5_k(rng, n, k, d_scale=std / 16 / 32)
    if fmt == 7:
        return quantize_bf16(rng.standard_normal((n, k), dtype=np.float32) * std)
    raise ValueError(fmt)
