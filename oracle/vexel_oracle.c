/*
 * vexel_oracle.c -- CPU restatement of the reference's batched-decode arithmetic.
 *
 * THIS IS TEST INFRASTRUCTURE. It is the checker that the HIP backend is compared
 * against; nothing in the shipped library links, loads or calls it.
 *
 * Every function restates one function of keithballinger/vexel (Go) loop for loop,
 * with the same operation order and the same float32/float64 mix, and cites the
 * file:line it follows (paths relative to the reference root). Floating point
 * follows Go's semantics on amd64: float32 expressions are evaluated in float32
 * with no fused multiply-add (build with -ffp-contract=off, no fast-math), and
 * math.Sqrt/Exp/Pow/Cos/Sin are float64 functions whose result is then rounded
 * to float32. (Go fuses x*y+z on arm64 only; the MI355X host is x86-64.)
 *
 * Pinning status (which independent check pins each function) is listed in
 * tests/test_oracle_*.py; functions with no such check are listed here:
 *   - none of the arithmetic kernels below is unpinned; see the test files.
 *   - vxo_matmul_q4_0 / vxo_sdpa last-ulp summation order: pinned only by
 *     restating the loop order (no reference vector fixes the last ulp).
 *   - the operators of the other architectures (vxo_layernorm, vxo_gelu[_mul], vxo_add_bias,
 *     vxo_scale_buffer, vxo_sdpa[_prefill]_softcap, vxo_rope_with_freqs, vxo_logit_softcap) and
 *     vxo_medusa_forward: pinned in tests/test_oracle_arch_ops.py by the reference's own test
 *     values and float64 closed forms; their last-ulp operation order likewise by restatement only.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define VXO_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* half precision                                                            */
/* ------------------------------------------------------------------------- */

/* inference/pkg/gguf/dequant.go:231-261 (float16ToFloat32). The twin in
 * inference/backend/cpu/cpu.go:962-992 differs only for NaN payloads (it forces
 * the quiet bit); vxo_f16_to_f32_cpu below restates that one. */
VXO_API float vxo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h >> 15) & 1u;
    uint32_t exp = (uint32_t)(h >> 10) & 0x1Fu;
    uint32_t mant = (uint32_t)h & 0x3FFu;
    uint32_t f32;
    if (exp == 0) {
        if (mant == 0) {
            f32 = sign << 31;
        } else {
            exp = 127 - 14;
            while ((mant & 0x400u) == 0) {
                mant <<= 1;
                exp--;
            }
            mant &= 0x3FFu;
            f32 = (sign << 31) | (exp << 23) | (mant << 13);
        }
    } else if (exp == 0x1F) {
        f32 = (sign << 31) | (0xFFu << 23) | (mant << 13);
    } else {
        f32 = (sign << 31) | ((exp + 127 - 15) << 23) | (mant << 13);
    }
    float out;
    memcpy(&out, &f32, 4);
    return out;
}

/* inference/backend/cpu/cpu.go:962-992 */
VXO_API float vxo_f16_to_f32_cpu(uint16_t h) {
    uint32_t sign = (uint32_t)(h >> 15) & 1u;
    uint32_t exp = (uint32_t)(h >> 10) & 0x1Fu;
    uint32_t frac = (uint32_t)h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (frac == 0) {
            bits = sign << 31;
            float z;
            memcpy(&z, &bits, 4);
            return z;
        }
        exp = 1;
        while ((frac & 0x400u) == 0) {
            frac <<= 1;
            exp--; /* wraps in uint32 exactly as the Go code does */
        }
        frac &= 0x3FFu;
    } else if (exp == 31) {
        if (frac == 0) {
            bits = (sign << 31) | 0x7F800000u;
        } else {
            bits = (sign << 31) | 0x7FC00000u | (frac << 13);
        }
        float z;
        memcpy(&z, &bits, 4);
        return z;
    }
    exp = exp + (127 - 15);
    frac = frac << 13;
    bits = (sign << 31) | (exp << 23) | frac;
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

/* float32 -> float16, round to nearest even, as the Metal cast `(half)x` in
 * reshape_paged_kv_f16 (inference/backend/metal/metal_bridge_darwin.m:8641).
 * Overflow goes to infinity, NaN stays NaN (quiet), subnormals are produced. */
VXO_API uint16_t vxo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) { /* inf / nan */
        if (absx > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((absx >> 13) & 0x3FFu));
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx >= 0x477FF000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx < 0x33000001u) { /* <= 2^-25 rounds to zero (ties to even -> 0) */
        return (uint16_t)sign;
    }
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    uint32_t shift;
    uint32_t hexp;
    if (e < -14) { /* subnormal half: value = m * 2^(e-23), unit 2^-24 */
        shift = (uint32_t)(13 + (-14 - e));
        hexp = 0;
    } else {
        shift = 13;
        hexp = (uint32_t)(e + 15);
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    uint32_t out;
    if (hexp == 0) {
        out = q; /* may carry into exponent 1: still correct encoding */
    } else {
        out = ((hexp - 1) << 10) + q; /* q includes the hidden bit (0x400) */
    }
    return (uint16_t)(sign | out);
}

VXO_API void vxo_f32_to_f16_n(const float *x, uint16_t *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = vxo_f32_to_f16(x[i]);
}

VXO_API void vxo_f16_to_f32_n(const uint16_t *x, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = vxo_f16_to_f32(x[i]);
}

/* ------------------------------------------------------------------------- */
/* GGUF block dequantisation (bit-exact targets)                             */
/* ------------------------------------------------------------------------- */

static uint16_t rd_u16(const uint8_t *p) { return (uint16_t)(p[0] | ((uint16_t)p[1] << 8)); }

/* inference/pkg/gguf/dequant.go:16-56. nbytes bounds the input as len(data)
 * does: a block that does not fit leaves its outputs (and all later ones) zero. */
VXO_API void vxo_dequant_q4_0(const uint8_t *data, int64_t nbytes, int64_t n, float *out) {
    const int64_t bs = 32, bb = 18;
    int64_t nblk = (n + bs - 1) / bs;
    memset(out, 0, (size_t)n * sizeof(float));
    for (int64_t b = 0; b < nblk; b++) {
        int64_t off = b * bb;
        if (off + bb > nbytes) break;
        float scale = vxo_f16_to_f32(rd_u16(data + off));
        for (int i = 0; i < 16; i++) {
            uint8_t bv = data[off + 2 + i];
            int64_t idx = b * bs + i;
            if (idx < n) {
                int q = (int)(bv & 0x0F);
                out[idx] = scale * (float)(q - 8);
            }
            idx = b * bs + i + 16;
            if (idx < n) {
                int q = (int)((bv >> 4) & 0x0F);
                out[idx] = scale * (float)(q - 8);
            }
        }
    }
}

/* inference/pkg/gguf/dequant.go:62-90 */
VXO_API void vxo_dequant_q8_0(const uint8_t *data, int64_t nbytes, int64_t n, float *out) {
    const int64_t bs = 32, bb = 34;
    int64_t nblk = (n + bs - 1) / bs;
    memset(out, 0, (size_t)n * sizeof(float));
    for (int64_t b = 0; b < nblk; b++) {
        int64_t off = b * bb;
        if (off + bb > nbytes) break;
        float scale = vxo_f16_to_f32(rd_u16(data + off));
        for (int i = 0; i < 32; i++) {
            int64_t idx = b * bs + i;
            if (idx < n) {
                int8_t q = (int8_t)data[off + 2 + i];
                out[idx] = scale * (float)q;
            }
        }
    }
}

/* inference/pkg/gguf/dequant.go:400-409 (getScaleMinK4) */
VXO_API void vxo_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *mn) {
    if (j < 4) {
        *sc = q[j] & 63;
        *mn = q[j + 4] & 63;
        return;
    }
    *sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
    *mn = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
}

/* inference/pkg/gguf/dequant.go:342-396. d1 = d*float32(sc) and dm1 = dmin*float32(m)
 * are rounded to float32 first; the element is d1*q - dm1 (two roundings). */
VXO_API void vxo_dequant_q4_k(const uint8_t *data, int64_t nbytes, int64_t n, float *out) {
    const int64_t bs = 256, bb = 144;
    int64_t nblk = (n + bs - 1) / bs;
    memset(out, 0, (size_t)n * sizeof(float));
    for (int64_t b = 0; b < nblk; b++) {
        int64_t off = b * bb;
        if (off + bb > nbytes) break;
        float d = vxo_f16_to_f32(rd_u16(data + off));
        float dmin = vxo_f16_to_f32(rd_u16(data + off + 2));
        const uint8_t *scales = data + off + 4;
        const uint8_t *qs = data + off + 16;
        int qoff = 0, is = 0;
        for (int j = 0; j < 256; j += 64) {
            uint8_t sc1, m1, sc2, m2;
            vxo_get_scale_min_k4(is + 0, scales, &sc1, &m1);
            float d1 = d * (float)sc1;
            float dm1 = dmin * (float)m1;
            vxo_get_scale_min_k4(is + 1, scales, &sc2, &m2);
            float d2 = d * (float)sc2;
            float dm2 = dmin * (float)m2;
            for (int l = 0; l < 32; l++) {
                int64_t i1 = b * bs + j + l, i2 = b * bs + j + l + 32;
                if (i1 < n) out[i1] = d1 * (float)(qs[qoff + l] & 0x0F) - dm1;
                if (i2 < n) out[i2] = d2 * (float)(qs[qoff + l] >> 4) - dm2;
            }
            qoff += 32;
            is += 2;
        }
    }
}

/* inference/pkg/gguf/dequant.go:272-331. d*sc*q is evaluated left to right. */
VXO_API void vxo_dequant_q6_k(const uint8_t *data, int64_t nbytes, int64_t n, float *out) {
    const int64_t bs = 256, bb = 210;
    int64_t nblk = (n + bs - 1) / bs;
    memset(out, 0, (size_t)n * sizeof(float));
    for (int64_t b = 0; b < nblk; b++) {
        int64_t off = b * bb;
        if (off + bb > nbytes) break;
        const uint8_t *ql = data + off;
        const uint8_t *qh = data + off + 128;
        const uint8_t *scales = data + off + 192;
        float d = vxo_f16_to_f32(rd_u16(data + off + 208));
        for (int nn = 0; nn < 2; nn++) {
            int qlo = nn * 64, qho = nn * 32, sco = nn * 8;
            int64_t yo = b * bs + nn * 128;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int8_t q1 = (int8_t)((int8_t)((ql[qlo + l] & 0xF) | (((qh[qho + l] >> 0) & 3) << 4)) - 32);
                int8_t q2 = (int8_t)((int8_t)((ql[qlo + l + 32] & 0xF) | (((qh[qho + l] >> 2) & 3) << 4)) - 32);
                int8_t q3 = (int8_t)((int8_t)((ql[qlo + l] >> 4) | (((qh[qho + l] >> 4) & 3) << 4)) - 32);
                int8_t q4 = (int8_t)((int8_t)((ql[qlo + l + 32] >> 4) | (((qh[qho + l] >> 6) & 3) << 4)) - 32);
                float sc0 = (float)(int8_t)scales[sco + is + 0];
                float sc2 = (float)(int8_t)scales[sco + is + 2];
                float sc4 = (float)(int8_t)scales[sco + is + 4];
                float sc6 = (float)(int8_t)scales[sco + is + 6];
                if (yo + l < n) out[yo + l] = d * sc0 * (float)q1;
                if (yo + l + 32 < n) out[yo + l + 32] = d * sc2 * (float)q2;
                if (yo + l + 64 < n) out[yo + l + 64] = d * sc4 * (float)q3;
                if (yo + l + 96 < n) out[yo + l + 96] = d * sc6 * (float)q4;
            }
        }
    }
}

/* inference/pkg/gguf/dequant.go:100-145: q = low nibble | bit j (or j+16) of qh << 4; element (q - 16) * d */
VXO_API void vxo_dequant_q5_0(const uint8_t *data, int64_t nbytes, int64_t n, float *out) {
    const int64_t bs = 32, bb = 22;
    int64_t nblk = (n + bs - 1) / bs;
    memset(out, 0, (size_t)n * sizeof(float));
    for (int64_t b = 0; b < nblk; b++) {
        int64_t off = b * bb;
        if (off + bb > nbytes) break;
        float d = vxo_f16_to_f32(rd_u16(data + off));
        uint32_t qh = (uint32_t)data[off + 2] | ((uint32_t)data[off + 3] << 8) | ((uint32_t)data[off + 4] << 16) |
                      ((uint32_t)data[off + 5] << 24);
        for (int j = 0; j < 16; j++) {
            uint8_t bv = data[off + 6 + j];
            int64_t idx = b * bs + j;
            if (idx < n) {
                uint8_t xh0 = (uint8_t)(((qh >> j) << 4) & 0x10);
                int q = (int)(bv & 0x0F) | (int)xh0;
                out[idx] = (float)(q - 16) * d;
            }
            idx = b * bs + j + 16;
            if (idx < n) {
                uint8_t xh1 = (uint8_t)(((qh >> (j + 16)) << 4) & 0x10);
                int q = (int)(bv >> 4) | (int)xh1;
                out[idx] = (float)(q - 16) * d;
            }
        }
    }
}

/* inference/pkg/gguf/dequant.go:423-500: Q4_K's header and 6-bit scales, then qh[32] (bit 2*group + half of
 * qh[l] is the fifth bit of element 64*group + 32*half + l) and the nibbles. d1 = d*float32(sc) and
 * dm1 = dmin*float32(m) are rounded first; the element is d1*q - dm1. */
VXO_API void vxo_dequant_q5_k(const uint8_t *data, int64_t nbytes, int64_t n, float *out) {
    const int64_t bs = 256, bb = 176;
    int64_t nblk = (n + bs - 1) / bs;
    memset(out, 0, (size_t)n * sizeof(float));
    for (int64_t b = 0; b < nblk; b++) {
        int64_t off = b * bb;
        if (off + bb > nbytes) break;
        float d = vxo_f16_to_f32(rd_u16(data + off));
        float dmin = vxo_f16_to_f32(rd_u16(data + off + 2));
        const uint8_t *scales = data + off + 4;
        const uint8_t *qh = data + off + 16;
        const uint8_t *qs = data + off + 48;
        int qoff = 0, is = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < 256; j += 64) {
            uint8_t sc1, m1, sc2, m2;
            vxo_get_scale_min_k4(is + 0, scales, &sc1, &m1);
            float d1 = d * (float)sc1;
            float dm1 = dmin * (float)m1;
            vxo_get_scale_min_k4(is + 1, scales, &sc2, &m2);
            float d2 = d * (float)sc2;
            float dm2 = dmin * (float)m2;
            for (int l = 0; l < 32; l++) {
                int64_t i1 = b * bs + j + l, i2 = b * bs + j + l + 32;
                uint8_t hb1 = (qh[l] & u1) ? 16 : 0, hb2 = (qh[l] & u2) ? 16 : 0;
                if (i1 < n) out[i1] = d1 * (float)(uint8_t)((qs[qoff + l] & 0x0F) + hb1) - dm1;
                if (i2 < n) out[i2] = d2 * (float)(uint8_t)((qs[qoff + l] >> 4) + hb2) - dm2;
            }
            qoff += 32;
            is += 2;
            u1 = (uint8_t)(u1 << 2);
            u2 = (uint8_t)(u2 << 2);
        }
    }
}

/* inference/pkg/gguf/dequant.go:215-228: the 16 bits are the upper half of the float32 */
VXO_API void vxo_dequant_bf16(const uint8_t *data, int64_t nbytes, int64_t n, float *out) {
    memset(out, 0, (size_t)n * sizeof(float));
    for (int64_t i = 0; i < n; i++) {
        if (i * 2 + 2 > nbytes) break;
        uint32_t u = (uint32_t)rd_u16(data + i * 2) << 16;
        memcpy(out + i, &u, 4);
    }
}

/* inference/pkg/gguf/dequant.go:200-211 */
VXO_API void vxo_dequant_f16(const uint8_t *data, int64_t nbytes, int64_t n, float *out) {
    memset(out, 0, (size_t)n * sizeof(float));
    for (int64_t i = 0; i < n; i++) {
        if (i * 2 + 2 > nbytes) break;
        out[i] = vxo_f16_to_f32(rd_u16(data + i * 2));
    }
}

/* ------------------------------------------------------------------------- */
/* matmuls                                                                   */
/* ------------------------------------------------------------------------- */

/* inference/backend/cpu/cpu.go:106-145 (matMulNaive): C[M,N] = A[M,K] * B[K,N] */
VXO_API void vxo_matmul_f32(const float *a, const float *b, float *out, int m, int n, int k) {
    for (int i = 0; i < m; i++)
        for (int j = 0; j < n; j++) {
            float sum = 0;
            for (int p = 0; p < k; p++) sum += a[(int64_t)i * k + p] * b[(int64_t)p * n + j];
            out[(int64_t)i * n + j] = sum;
        }
}

/* inference/backend/cpu/cpu.go:158-197 (matMulTransposedNaive): C = A * B^T, B is [N,K].
 * This is also the CPU semantics of the Q4_K / Q6_K / Q8_0 matmuls: the CPU backend
 * panics for them (cpu.go:916-945) and the loader dequantises those tensors to F32
 * (inference/runtime/loader.go:216-271) before this loop runs. */
VXO_API void vxo_matmul_t_f32(const float *a, const float *b, float *out, int m, int n, int k) {
    for (int i = 0; i < m; i++)
        for (int j = 0; j < n; j++) {
            float sum = 0;
            for (int p = 0; p < k; p++) sum += a[(int64_t)i * k + p] * b[(int64_t)j * k + p];
            out[(int64_t)i * n + j] = sum;
        }
}

/* inference/backend/cpu/cpu.go:842-911 (MatMulQ4_0): per block, byte ascending,
 * low nibble (position i) then high nibble (position i+16); the dequantised value
 * is float32(q-8)*scale and is multiplied into the running float32 sum. */
VXO_API void vxo_matmul_q4_0(const float *a, const uint8_t *bq, float *out, int m, int n, int k) {
    const int bb = 18;
    int bpr = k / 32;
    for (int i = 0; i < m; i++) {
        const float *arow = a + (int64_t)i * k;
        for (int j = 0; j < n; j++) {
            float sum = 0;
            int64_t rowoff = (int64_t)j * bpr * bb;
            for (int blk = 0; blk < bpr; blk++) {
                int64_t bo = rowoff + (int64_t)blk * bb;
                float scale = vxo_f16_to_f32_cpu(rd_u16(bq + bo));
                int base = blk * 32;
                for (int bi = 0; bi < 16; bi++) {
                    uint8_t bv = bq[bo + 2 + bi];
                    int lo = (int)(bv & 0x0F);
                    float dl = (float)(lo - 8) * scale;
                    sum += arow[base + bi] * dl;
                    int hi = (int)((bv >> 4) & 0x0F);
                    float dh = (float)(hi - 8) * scale;
                    sum += arow[base + bi + 16] * dh;
                }
            }
            out[(int64_t)i * n + j] = sum;
        }
    }
}

/* Semantics of MatMulQ4_K / MatMulQ6_K / MatMulQ8_0 on the reference CPU path:
 * gguf.Dequantize (dequant.go:503-538) then matMulTransposedNaive. fmt: 1=Q4_0
 * (dequantise-then-multiply variant, used only to cross-check), 2=Q8_0, 3=Q4_K, 4=Q6_K.
 * Dequantises one weight row at a time so host memory stays small. */
VXO_API int vxo_matmul_quant_via_dequant(int fmt, const float *a, const uint8_t *bq, float *out,
                                         int m, int n, int k) {
    int64_t row_bytes;
    switch (fmt) {
    case 1: row_bytes = (int64_t)k / 32 * 18; break;
    case 2: row_bytes = (int64_t)k / 32 * 34; break;
    case 3: row_bytes = (int64_t)k / 256 * 144; break;
    case 4: row_bytes = (int64_t)k / 256 * 210; break;
    case 5: row_bytes = (int64_t)k / 32 * 22; break;
    case 6: row_bytes = (int64_t)k / 256 * 176; break;
    case 7: row_bytes = (int64_t)k * 2; break;
    default: return -1;
    }
    float *w = (float *)malloc((size_t)k * sizeof(float));
    if (!w) return -2;
    for (int j = 0; j < n; j++) {
        const uint8_t *row = bq + (int64_t)j * row_bytes;
        switch (fmt) {
        case 1: vxo_dequant_q4_0(row, row_bytes, k, w); break;
        case 2: vxo_dequant_q8_0(row, row_bytes, k, w); break;
        case 3: vxo_dequant_q4_k(row, row_bytes, k, w); break;
        case 4: vxo_dequant_q6_k(row, row_bytes, k, w); break;
        case 5: vxo_dequant_q5_0(row, row_bytes, k, w); break;
        case 6: vxo_dequant_q5_k(row, row_bytes, k, w); break;
        case 7: vxo_dequant_bf16(row, row_bytes, k, w); break;
        }
        for (int i = 0; i < m; i++) {
            const float *arow = a + (int64_t)i * k;
            float sum = 0;
            for (int p = 0; p < k; p++) sum += arow[p] * w[p];
            out[(int64_t)i * n + j] = sum;
        }
    }
    free(w);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* elementwise / normalisation                                               */
/* ------------------------------------------------------------------------- */

/* inference/backend/cpu/cpu.go:200-220 */
VXO_API void vxo_rmsnorm(const float *x, const float *w, float *out, int rows, int cols, float eps) {
    for (int i = 0; i < rows; i++) {
        float ss = 0;
        int64_t off = (int64_t)i * cols;
        for (int j = 0; j < cols; j++) {
            float v = x[off + j];
            ss += v * v;
        }
        float mean = ss / (float)cols;
        float rms = (float)sqrt((double)(mean + eps));
        for (int j = 0; j < cols; j++) out[off + j] = (x[off + j] / rms) * w[j];
    }
}

static void rope_one(float *data, int64_t total_vectors, int heads, int head_dim, int start_pos,
                     int eff_dim, float theta, int neox, const int32_t *positions) {
    int half = eff_dim / 2;
    for (int64_t i = 0; i < total_vectors; i++) {
        int seq_pos = (int)(i / heads);
        int pos = positions ? positions[seq_pos] : start_pos + seq_pos;
        int64_t off = i * head_dim;
        for (int j = 0; j < half; j++) {
            int i0, i1;
            if (neox) {
                i0 = j;
                i1 = j + half;
            } else {
                i0 = j * 2;
                i1 = j * 2 + 1;
            }
            double ex = (double)(2 * j) / (double)eff_dim;
            float freq = (float)(1.0 / pow((double)theta, ex));
            float angle = (float)pos * freq;
            float c = (float)cos((double)angle);
            float s = (float)sin((double)angle);
            float v1 = data[off + i0], v2 = data[off + i1];
            data[off + i0] = v1 * c - v2 * s;
            data[off + i1] = v1 * s + v2 * c;
        }
    }
}

/* inference/backend/cpu/cpu.go:226-303. k may be NULL. */
VXO_API void vxo_rope(float *q, float *k, int head_dim, int num_heads, int num_kv_heads, int seq_len,
                      int start_pos, int rope_dim, float theta, int neox) {
    int eff = rope_dim == 0 ? head_dim : rope_dim;
    rope_one(q, (int64_t)seq_len * num_heads, num_heads, head_dim, start_pos, eff, theta, neox, NULL);
    if (k) rope_one(k, (int64_t)seq_len * num_kv_heads, num_kv_heads, head_dim, start_pos, eff, theta, neox, NULL);
}

/* Same arithmetic with an explicit position per row: row r is rotated exactly as
 * cpu.go:226-303 rotates a one-row call with startPos = positions[r]. This is what
 * the sequential loop in inference/runtime/decode.go:642-650 does to each sequence. */
VXO_API void vxo_rope_positions(float *q, float *k, int head_dim, int num_heads, int num_kv_heads,
                                int rows, const int32_t *positions, int rope_dim, float theta, int neox) {
    int eff = rope_dim == 0 ? head_dim : rope_dim;
    rope_one(q, (int64_t)rows * num_heads, num_heads, head_dim, 0, eff, theta, neox, positions);
    if (k) rope_one(k, (int64_t)rows * num_kv_heads, num_kv_heads, head_dim, 0, eff, theta, neox, positions);
}

/* inference/backend/cpu/backend.go:244-276 (RoPEShift): every K vector rotated by the angle of position `shift`,
 * interleaved pairs over the whole head; shift 0 returns at once. */
VXO_API void vxo_rope_shift(float *k, int head_dim, int num_kv_heads, int num_tokens, int shift, float theta) {
    if (shift == 0) return;
    for (int t = 0; t < num_tokens; t++)
        for (int h = 0; h < num_kv_heads; h++) {
            int64_t offset = (int64_t)t * num_kv_heads * head_dim + (int64_t)h * head_dim;
            for (int j = 0; j < head_dim / 2; j++) {
                int idx = j * 2;
                double ex = (double)(2 * j) / (double)head_dim;
                float freq = (float)(1.0 / pow((double)theta, ex));
                float angle = (float)shift * freq;
                float c = (float)cos((double)angle), sn = (float)sin((double)angle);
                float v1 = k[offset + idx], v2 = k[offset + idx + 1];
                k[offset + idx] = v1 * c - v2 * sn;
                k[offset + idx + 1] = v1 * sn + v2 * c;
            }
        }
}

static void rope_freqs_one(float *data, int64_t total_vectors, int heads, int head_dim, int start_pos,
                           const float *freqs, int neox) {
    int half = head_dim / 2;
    for (int64_t i = 0; i < total_vectors; i++) {
        int pos = start_pos + (int)(i / heads);
        int64_t off = i * head_dim;
        for (int j = 0; j < half; j++) {
            int i0 = neox ? j : 2 * j, i1 = neox ? j + half : 2 * j + 1;
            float angle = (float)pos * freqs[j];
            float c = (float)cos((double)angle), sn = (float)sin((double)angle);
            float v1 = data[off + i0], v2 = data[off + i1];
            data[off + i0] = v1 * c - v2 * sn;
            data[off + i1] = v1 * sn + v2 * c;
        }
    }
}

/* inference/backend/cpu/cpu.go:308-375 (RoPEWithFreqs): RoPE over the whole head with the inverse frequency of
 * pair j read from freqs[j] (head_dim / 2 values) instead of computed from theta. k may be NULL. */
VXO_API void vxo_rope_with_freqs(float *q, float *k, const float *freqs, int head_dim, int num_heads, int num_kv_heads,
                                 int seq_len, int start_pos, int neox) {
    rope_freqs_one(q, (int64_t)seq_len * num_heads, num_heads, head_dim, start_pos, freqs, neox);
    if (k) rope_freqs_one(k, (int64_t)seq_len * num_kv_heads, num_kv_heads, head_dim, start_pos, freqs, neox);
}

/* inference/backend/cpu/cpu.go:378-387 */
VXO_API void vxo_silu(const float *x, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) {
        float v = x[i];
        float sg = 1.0f / (1.0f + (float)exp((double)(-v)));
        out[i] = v * sg;
    }
}

/* inference/backend/cpu/cpu.go:390-400 */
VXO_API void vxo_silu_mul(const float *gate, const float *up, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) {
        float g = gate[i];
        float sg = 1.0f / (1.0f + (float)exp((double)(-g)));
        out[i] = (g * sg) * up[i];
    }
}

/* inference/backend/cpu/cpu.go:404-436 (LayerNorm): mean and variance by sequential float32 sums over the row,
 * 1/sqrt in float64 rounded to float32, then ((x - mean) * invStd) * w + b. */
VXO_API void vxo_layernorm(const float *x, const float *w, const float *b, float *out, int rows, int cols, float eps) {
    for (int i = 0; i < rows; i++) {
        int64_t off = (int64_t)i * cols;
        float sum = 0;
        for (int j = 0; j < cols; j++) sum += x[off + j];
        float mean = sum / (float)cols;
        float vs = 0;
        for (int j = 0; j < cols; j++) {
            float diff = x[off + j] - mean;
            vs += diff * diff;
        }
        float variance = vs / (float)cols;
        float inv_std = 1.0f / (float)sqrt((double)(variance + eps));
        for (int j = 0; j < cols; j++) {
            float normalized = (x[off + j] - mean) * inv_std;
            out[off + j] = normalized * w[j] + b[j];
        }
    }
}

/* The tanh form of GELU as cpu.go:440-454 evaluates it: the untyped constants take float32 beside a float32
 * operand, every product is float32, tanh is taken in float64 of the float32 argument. */
static float gelu_one(float val) {
    const float sqrt_two_pi = 0.7978845608f, coeff = 0.044715f;
    float x3 = val * val * val;
    float inner = coeff * x3;
    float arg = sqrt_two_pi * (val + inner);
    float th = (float)tanh((double)arg);
    return 0.5f * val * (1.0f + th);
}

/* inference/backend/cpu/cpu.go:440-454 */
VXO_API void vxo_gelu(const float *x, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = gelu_one(x[i]);
}

/* inference/backend/cpu/cpu.go:457-473 (GELUMul): gelu(gate) * up */
VXO_API void vxo_gelu_mul(const float *gate, const float *up, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = gelu_one(gate[i]) * up[i];
}

/* inference/backend/cpu/cpu.go:476-487 (AddBias): out[r][c] = x[r][c] + bias[c] */
VXO_API void vxo_add_bias(const float *x, const float *bias, float *out, int rows, int cols) {
    for (int i = 0; i < rows; i++)
        for (int j = 0; j < cols; j++) out[(int64_t)i * cols + j] = x[(int64_t)i * cols + j] + bias[j];
}

/* inference/backend/cpu/cpu.go:558-563 (ScaleBuffer), in place */
VXO_API void vxo_scale_buffer(float *buf, float scale, int64_t n) {
    for (int64_t i = 0; i < n; i++) buf[i] *= scale;
}

/* inference/backend/cpu/cpu.go:490-518 */
VXO_API void vxo_softmax(const float *x, float *out, int rows, int cols) {
    for (int i = 0; i < rows; i++) {
        const float *row = x + (int64_t)i * cols;
        float *orow = out + (int64_t)i * cols;
        float mx = row[0];
        for (int j = 0; j < cols; j++)
            if (row[j] > mx) mx = row[j];
        float sum = 0;
        for (int j = 0; j < cols; j++) {
            float e = (float)exp((double)(row[j] - mx));
            orow[j] = e;
            sum += e;
        }
        float inv = 1.0f / sum;
        for (int j = 0; j < cols; j++) orow[j] *= inv;
    }
}

/* inference/backend/cpu/cpu.go:521-529 */
VXO_API void vxo_add(const float *a, const float *b, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = a[i] + b[i];
}

/* inference/backend/cpu/cpu.go:532-540 */
VXO_API void vxo_mul(const float *a, const float *b, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = a[i] * b[i];
}

/* inference/backend/cpu/cpu.go:543-555: an out-of-range id leaves its row untouched. */
VXO_API void vxo_embedding(const int32_t *ids, int num_tokens, const float *table, float *out,
                           int vocab, int dim) {
    for (int i = 0; i < num_tokens; i++) {
        int id = ids[i];
        if (id < 0 || id >= vocab) continue;
        memcpy(out + (int64_t)i * dim, table + (int64_t)id * dim, (size_t)dim * sizeof(float));
    }
}

/* inference/pkg/sampler/sampler.go:80-91: first index of the strict maximum,
 * starting from -MaxFloat32 (so NaN never wins and all -inf returns 0). */
VXO_API int vxo_argmax(const float *x, int n) {
    float mv = -3.40282346638528859811704183484516925440e+38f;
    int mi = 0;
    for (int i = 0; i < n; i++)
        if (x[i] > mv) {
            mv = x[i];
            mi = i;
        }
    return mi;
}

/* inference/runtime/model.go:336-350 (ApplyFinalLogitSoftCap): float32(float64(cap) * tanh(float64(x) * invCap))
 * with invCap = 1.0 / float64(cap), in place; cap <= 0 changes nothing. */
VXO_API void vxo_logit_softcap(float *logits, int64_t n, float cap) {
    if (cap <= 0) return;
    double inv_cap = 1.0 / (double)cap;
    for (int64_t i = 0; i < n; i++) logits[i] = (float)((double)cap * tanh((double)logits[i] * inv_cap));
}

/* inference/medusa/heads.go:83-117 (Heads.Forward) for one head: intermediate = silu(hidden . FC1) with
 * silu(x) = x / (1 + exp(-x)) (heads.go:20-22), logits = intermediate . FC2; FC1 is [hidden, hidden] and FC2
 * [hidden, vocab], both indexed [in * out_size + out]; every sum runs over the input index in order. */
VXO_API void vxo_medusa_forward(const float *hidden, const float *fc1, const float *fc2, float *intermediate,
                                float *logits, int hidden_size, int vocab_size) {
    for (int i = 0; i < hidden_size; i++) {
        float sum = 0;
        for (int j = 0; j < hidden_size; j++) sum += hidden[j] * fc1[(int64_t)j * hidden_size + i];
        intermediate[i] = sum / (1.0f + (float)exp((double)(-sum)));
    }
    for (int i = 0; i < vocab_size; i++) {
        float sum = 0;
        for (int j = 0; j < hidden_size; j++) sum += intermediate[j] * fc2[(int64_t)j * vocab_size + i];
        logits[i] = sum;
    }
}

/* ------------------------------------------------------------------------- */
/* attention                                                                 */
/* ------------------------------------------------------------------------- */

/* One query head against kv_len (k,v) rows fetched through callbacks-free strided
 * access: k_at(p) = kbase + p*kstride. Body of inference/backend/cpu/cpu.go:589-630. */
static void sdpa_head_capped(const float *qh, float *oh, int kv_len, int head_dim, float scale, float softcap,
                             const float *const *krows, const float *const *vrows, float *scores) {
    for (int p = 0; p < kv_len; p++) {
        const float *kv = krows[p];
        float dot = 0;
        for (int d = 0; d < head_dim; d++) dot += qh[d] * kv[d];
        float score = dot * scale;
        /* cpu.go:735-737, 802-804: the only difference of the soft-capped forms */
        if (softcap > 0) score = softcap * (float)tanh((double)(score / softcap));
        scores[p] = score;
    }
    float mx = scores[0];
    for (int p = 0; p < kv_len; p++)
        if (scores[p] > mx) mx = scores[p];
    float se = 0;
    for (int p = 0; p < kv_len; p++) {
        scores[p] = (float)exp((double)(scores[p] - mx));
        se += scores[p];
    }
    float inv = 1.0f / se;
    for (int p = 0; p < kv_len; p++) scores[p] *= inv;
    for (int d = 0; d < head_dim; d++) oh[d] = 0;
    for (int p = 0; p < kv_len; p++) {
        const float *vv = vrows[p];
        float w = scores[p];
        for (int d = 0; d < head_dim; d++) oh[d] += w * vv[d];
    }
}

static void sdpa_head(const float *qh, float *oh, int kv_len, int head_dim, float scale,
                      const float *const *krows, const float *const *vrows, float *scores) {
    sdpa_head_capped(qh, oh, kv_len, head_dim, scale, 0.0f, krows, vrows, scores);
}

/* inference/backend/cpu/cpu.go:568-632. K/V head-major [numKVHeads, stride/headDim, headDim]. */
VXO_API void vxo_sdpa(const float *q, const float *k, const float *v, float *out, int kv_len,
                      int num_q_heads, int num_kv_heads, int head_dim, float scale, int kv_head_stride) {
    int hpk = num_q_heads / num_kv_heads;
    float *scores = (float *)malloc((size_t)(kv_len > 0 ? kv_len : 1) * sizeof(float));
    const float **kr = (const float **)malloc((size_t)(kv_len > 0 ? kv_len : 1) * sizeof(float *));
    const float **vr = (const float **)malloc((size_t)(kv_len > 0 ? kv_len : 1) * sizeof(float *));
    for (int h = 0; h < num_q_heads; h++) {
        int kvh = h / hpk;
        int64_t base = (int64_t)kvh * kv_head_stride;
        for (int p = 0; p < kv_len; p++) {
            kr[p] = k + base + (int64_t)p * head_dim;
            vr[p] = v + base + (int64_t)p * head_dim;
        }
        sdpa_head(q + (int64_t)h * head_dim, out + (int64_t)h * head_dim, kv_len, head_dim, scale, kr, vr, scores);
    }
    free(scores);
    free(kr);
    free(vr);
}

/* inference/backend/cpu/cpu.go:635-701. Q,K,V,out token-major [seqLen, heads, headDim]. */
VXO_API void vxo_sdpa_prefill(const float *q, const float *k, const float *v, float *out, int seq_len,
                              int num_q_heads, int num_kv_heads, int head_dim, float scale) {
    int hpk = num_q_heads / num_kv_heads;
    float *scores = (float *)malloc((size_t)(seq_len > 0 ? seq_len : 1) * sizeof(float));
    const float **kr = (const float **)malloc((size_t)(seq_len > 0 ? seq_len : 1) * sizeof(float *));
    const float **vr = (const float **)malloc((size_t)(seq_len > 0 ? seq_len : 1) * sizeof(float *));
    for (int qp = 0; qp < seq_len; qp++)
        for (int h = 0; h < num_q_heads; h++) {
            int kvh = h / hpk;
            int64_t qo = ((int64_t)qp * num_q_heads + h) * head_dim;
            int mk = qp + 1;
            for (int p = 0; p < mk; p++) {
                kr[p] = k + ((int64_t)p * num_kv_heads + kvh) * head_dim;
                vr[p] = v + ((int64_t)p * num_kv_heads + kvh) * head_dim;
            }
            sdpa_head(q + qo, out + qo, mk, head_dim, scale, kr, vr, scores);
        }
    free(scores);
    free(kr);
    free(vr);
}

/* inference/backend/cpu/cpu.go:705-765 (SDPASoftCap): SDPA whose scaled scores pass through
 * softcap * tanh(score / softcap) when softcap > 0. */
VXO_API void vxo_sdpa_softcap(const float *q, const float *k, const float *v, float *out, int kv_len,
                              int num_q_heads, int num_kv_heads, int head_dim, float scale, float softcap,
                              int kv_head_stride) {
    int hpk = num_q_heads / num_kv_heads;
    size_t cap = (size_t)(kv_len > 0 ? kv_len : 1);
    float *scores = (float *)malloc(cap * sizeof(float));
    const float **kr = (const float **)malloc(cap * sizeof(float *));
    const float **vr = (const float **)malloc(cap * sizeof(float *));
    for (int h = 0; h < num_q_heads; h++) {
        int64_t base = (int64_t)(h / hpk) * kv_head_stride;
        for (int p = 0; p < kv_len; p++) {
            kr[p] = k + base + (int64_t)p * head_dim;
            vr[p] = v + base + (int64_t)p * head_dim;
        }
        sdpa_head_capped(q + (int64_t)h * head_dim, out + (int64_t)h * head_dim, kv_len, head_dim, scale, softcap, kr,
                         vr, scores);
    }
    free(scores);
    free(kr);
    free(vr);
}

/* inference/backend/cpu/cpu.go:770-841 (SDPAPrefillSoftCap): causal, token-major. */
VXO_API void vxo_sdpa_prefill_softcap(const float *q, const float *k, const float *v, float *out, int seq_len,
                                      int num_q_heads, int num_kv_heads, int head_dim, float scale, float softcap) {
    int hpk = num_q_heads / num_kv_heads;
    size_t cap = (size_t)(seq_len > 0 ? seq_len : 1);
    float *scores = (float *)malloc(cap * sizeof(float));
    const float **kr = (const float **)malloc(cap * sizeof(float *));
    const float **vr = (const float **)malloc(cap * sizeof(float *));
    for (int qp = 0; qp < seq_len; qp++)
        for (int h = 0; h < num_q_heads; h++) {
            int kvh = h / hpk;
            int64_t qo = ((int64_t)qp * num_q_heads + h) * head_dim;
            for (int p = 0; p <= qp; p++) {
                kr[p] = k + ((int64_t)p * num_kv_heads + kvh) * head_dim;
                vr[p] = v + ((int64_t)p * num_kv_heads + kvh) * head_dim;
            }
            sdpa_head_capped(q + qo, out + qo, qp + 1, head_dim, scale, softcap, kr, vr, scores);
        }
    free(scores);
    free(kr);
    free(vr);
}

/* ------------------------------------------------------------------------- */
/* paged KV: scatter and attention through a block table                     */
/* ------------------------------------------------------------------------- */

/* reshape_paged_kv_f32, inference/backend/metal/metal_bridge_darwin.m:8539-8601
 * (interface: inference/backend/backend.go:416-424). */
VXO_API void vxo_reshape_paged_kv_f32(const float *src, float *dst_base, const int32_t *block_idx,
                                      const int32_t *block_off, int num_tokens, int num_kv_heads,
                                      int head_dim, int block_size, int is_value) {
    int64_t hs = (int64_t)num_kv_heads * head_dim;
    int64_t part = (int64_t)block_size * hs;
    for (int t = 0; t < num_tokens; t++)
        for (int64_t r = 0; r < hs; r++) {
            int64_t di = (int64_t)block_idx[t] * 2 * part + (is_value ? part : 0) + (int64_t)block_off[t] * hs + r;
            dst_base[di] = src[(int64_t)t * hs + r];
        }
}

/* reshape_paged_kv_f16, metal_bridge_darwin.m:8607-8642: same addressing, value
 * stored as (half)src, i.e. round to nearest even. */
VXO_API void vxo_reshape_paged_kv_f16(const float *src, uint16_t *dst_base, const int32_t *block_idx,
                                      const int32_t *block_off, int num_tokens, int num_kv_heads,
                                      int head_dim, int block_size, int is_value) {
    int64_t hs = (int64_t)num_kv_heads * head_dim;
    int64_t part = (int64_t)block_size * hs;
    for (int t = 0; t < num_tokens; t++)
        for (int64_t r = 0; r < hs; r++) {
            int64_t di = (int64_t)block_idx[t] * 2 * part + (is_value ? part : 0) + (int64_t)block_off[t] * hs + r;
            dst_base[di] = vxo_f32_to_f16(src[(int64_t)t * hs + r]);
        }
}

/* Paged single-query attention. Addressing follows sdpa_paged_decode_f32/_f16
 * (metal_bridge_darwin.m:11074-11198, 8655-8755): position p lives in physical
 * block bt[p/bs] at token p%bs, K part then V part, [bs, Hkv, D] each. The
 * arithmetic is the CPU backend's SDPA (cpu.go:589-630): float32 dot in d order,
 * exp through float64, weights normalised before the V accumulation. An F16 pool
 * is read as float(half). Deliberately NOT the CPU fallback of
 * inference/runtime/block.go:948-953, which mis-strides K/V when numKVHeads > 1. */
static void paged_query(const float *q, const void *pool, int pool_f16, const int32_t *bt, float *out,
                        int kv_len, int block_size, int num_q_heads, int num_kv_heads, int head_dim,
                        float scale, const uint8_t *extra_mask, int mask_base) {
    int hpk = num_q_heads / num_kv_heads;
    int64_t hs = (int64_t)num_kv_heads * head_dim;
    int64_t part = (int64_t)block_size * hs;
    /* gather the attended rows as float32 once per kv head */
    int cnt = 0;
    int *sel = (int *)malloc((size_t)(kv_len > 0 ? kv_len : 1) * sizeof(int));
    for (int p = 0; p < kv_len; p++) {
        if (extra_mask && p >= mask_base && !extra_mask[p - mask_base]) continue;
        sel[cnt++] = p;
    }
    float *kbuf = (float *)malloc((size_t)(cnt > 0 ? cnt : 1) * head_dim * sizeof(float));
    float *vbuf = (float *)malloc((size_t)(cnt > 0 ? cnt : 1) * head_dim * sizeof(float));
    const float **kr = (const float **)malloc((size_t)(cnt > 0 ? cnt : 1) * sizeof(float *));
    const float **vr = (const float **)malloc((size_t)(cnt > 0 ? cnt : 1) * sizeof(float *));
    float *scores = (float *)malloc((size_t)(cnt > 0 ? cnt : 1) * sizeof(float));
    for (int h = 0; h < num_q_heads; h++) {
        int kvh = h / hpk;
        if (h % hpk == 0) {
            for (int c = 0; c < cnt; c++) {
                int p = sel[c];
                int64_t kb = (int64_t)bt[p / block_size] * 2 * part + (int64_t)(p % block_size) * hs + (int64_t)kvh * head_dim;
                int64_t vb = kb + part;
                for (int d = 0; d < head_dim; d++) {
                    if (pool_f16) {
                        kbuf[(int64_t)c * head_dim + d] = vxo_f16_to_f32(((const uint16_t *)pool)[kb + d]);
                        vbuf[(int64_t)c * head_dim + d] = vxo_f16_to_f32(((const uint16_t *)pool)[vb + d]);
                    } else {
                        kbuf[(int64_t)c * head_dim + d] = ((const float *)pool)[kb + d];
                        vbuf[(int64_t)c * head_dim + d] = ((const float *)pool)[vb + d];
                    }
                }
                kr[c] = kbuf + (int64_t)c * head_dim;
                vr[c] = vbuf + (int64_t)c * head_dim;
            }
        }
        sdpa_head(q + (int64_t)h * head_dim, out + (int64_t)h * head_dim, cnt, head_dim, scale, kr, vr, scores);
    }
    free(sel);
    free(kbuf);
    free(vbuf);
    free(kr);
    free(vr);
    free(scores);
}

/* PagedKVOps.SDPAPagedDecode / SDPAPagedDecodeF16 (backend.go:426-438):
 * kvLen = (numBlocks-1)*blockSize + tokensInLastBlock (metal_bridge_darwin.m:11105). */
VXO_API void vxo_sdpa_paged_decode(const float *q, const void *pool, int pool_f16, const int32_t *bt,
                                   float *out, int num_blocks, int block_size, int num_q_heads,
                                   int num_kv_heads, int head_dim, float scale, int tokens_in_last_block) {
    int kv_len = (num_blocks - 1) * block_size + tokens_in_last_block;
    paged_query(q, pool, pool_f16, bt, out, kv_len, block_size, num_q_heads, num_kv_heads, head_dim, scale, NULL, 0);
}

/* PagedKVOps.SDPAPagedDecodeBatched (backend.go:440-454) = a loop of single-sequence
 * calls (inference/backend/metal/backend.go:2667-2680). Block tables are given as one
 * padded [batch, max_blocks] matrix. seq_lens[i] is the context length of sequence i. */
VXO_API void vxo_sdpa_paged_decode_batched(const float *q, const void *pool, int pool_f16,
                                           const int32_t *bts, float *out, int batch, int max_blocks,
                                           int block_size, int num_q_heads, int num_kv_heads,
                                           int head_dim, float scale, const int32_t *seq_lens) {
    int64_t qs = (int64_t)num_q_heads * head_dim;
    for (int i = 0; i < batch; i++)
        paged_query(q + i * qs, pool, pool_f16, bts + (int64_t)i * max_blocks, out + i * qs, seq_lens[i],
                    block_size, num_q_heads, num_kv_heads, head_dim, scale, NULL, 0);
}

/* PagedKVOps.SDPAPagedDecodeMultiquery (backend.go:459-465; kernel
 * metal_bridge_darwin.m:11205-11311): query i attends to positions 0..kvLens[i]-1.
 * The pool is read in its real element type (the Metal kernel reads an F16 pool as
 * F32, a defect that is not reproduced).
 * Tree verification extension (no reference kernel; mask rule from
 * inference/medusa/tree.go:186-202): when tree_mask != NULL, query i attends to all
 * positions < tree_base and to position tree_base+j iff tree_mask[i*n+j] != 0; kvLens
 * is ignored in that case and n = query_len. */
VXO_API void vxo_sdpa_paged_multiquery(const float *q, const void *pool, int pool_f16, const int32_t *bt,
                                       float *out, const int32_t *kv_lens, int block_size,
                                       int num_q_heads, int num_kv_heads, int head_dim, float scale,
                                       int query_len, const uint8_t *tree_mask, int tree_base) {
    int64_t qs = (int64_t)num_q_heads * head_dim;
    for (int i = 0; i < query_len; i++) {
        if (tree_mask)
            paged_query(q + i * qs, pool, pool_f16, bt, out + i * qs, tree_base + query_len, block_size,
                        num_q_heads, num_kv_heads, head_dim, scale, tree_mask + (int64_t)i * query_len, tree_base);
        else
            paged_query(q + i * qs, pool, pool_f16, bt, out + i * qs, kv_lens[i], block_size, num_q_heads,
                        num_kv_heads, head_dim, scale, NULL, 0);
    }
}
