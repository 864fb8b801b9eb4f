"""Synthetic quantized-weight makers for tests and the benchmark (TEST INFRASTRUCTURE ONLY).

The reference has no F32 -> Q4_0/Q4_K/Q6_K quantizer (only dequantizers), so these are
not restatements of reference code paths, with one exception: the block *encoders*
(encode_q4_0_block, encode_q8_0_block, encode_q4_k_block, encode_q6_k_block) follow the
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


def random_quant(fmt, rng, n, k, std=0.02):
    """Quantized [N,K] weight of format fmt (1=Q4_0, 2=Q8_0, 3=Q4_K, 4=Q6_K) with
    dequantised std near `std`."""
    if fmt == 1:
        return quantize_q4_0(rng.standard_normal((n, k), dtype=np.float32) * std)
    if fmt == 2:
        return quantize_q8_0(rng.standard_normal((n, k), dtype=np.float32) * std)
    if fmt == 3:
        return random_q4_k(rng, n, k, d_scale=std / 8 / 32)
    if fmt == 4:
        return random_q6_k(rng, n, k, d_scale=std / 18 / 64)
    raise ValueError(fmt)
