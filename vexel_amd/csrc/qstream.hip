// Decode-batch GEMM (2 .. 64 activation rows) over quantized weights repacked at load time into the order the matrix
// cores consume them: C[M,N] = A[M,K] * B^T with B [N,K] as backend.go:47-81 (MatMulQ4_0 / Q8_0 / Q4_K / Q6_K) has
// it, the arithmetic of backend/cpu/cpu.go:842-911 up to float32 summation order.
//
// Packed layout (vx_qweight_pack): the matrix is cut into tiles of 16 rows and half chunks of 128 columns. One
// (tile, half chunk) is a unit, units of a tile follow one another along K. The Q4_0 unit, 1152 bytes:
//   bytes [0, 1024): lane l = 16 * g + r of a wave owns 16 bytes, dword j of them the eight 4-bit codes of row r's
//     block 4 * hc + j that lane group g feeds to the matrix core: nibble i of the dword is block element
//     ELT[g][SLOT[i]] (the slot order of the prepared activation tiles, prep_tiles.h), so that two masks, one shift
//     and four packed f16 operations turn the dword into the operand;
//   bytes [1024, 1152): row r's four f16 block scales at 1024 + 8 r.
// Its bytes are a permutation of the GGUF rows' bytes (18 per 32 elements either way), as are the Q8_0 unit's; the
// Q4_K and Q6_K units carry their scales as float32 products (see SQ4_K, SQ6_K). vx_dequantize_packed gives back
// gguf.Dequantize's values bit for bit for every format (pkg/gguf/dequant.go:16-95, 272-409).
//
// Kernel: one workgroup of eight waves per compute unit owns a range of tiles and one K slice. Wave w keeps the
// activation operand of half chunk h0 + w (and h0 + 8 + w) of the slice in registers for the whole pass and streams
// the weight units of those half chunks through them, tile after tile, from a ring of requests that runs ahead of
// the arithmetic: a unit goes from memory to registers with one 16-byte and one 8-byte load per lane (Q4_0) and nowhere
// else. Per 32-column step (Q4_0): 9 vector instructions unpack the codes to exact integers in f16, four
// v_mfma_f32_16x16x32_f16 multiply them with the hi and lo halves of two activation tiles, 8 fused multiply-adds
// apply the block scale. After every RG tiles the eight waves' sums meet in LDS and are added in wave order. A slice
// wider than 16 half chunks is walked in passes of 16 (the sums wait in LDS), which is how the Q|K|V launch
// keeps the whole K in one workgroup and finishes its rows itself (RoPE, K/V store).
// Which tiles and half chunks a workgroup takes depends on (N, K, device, epilogue, format) and on whether the batch
// has up to 32 or up to 64 rows; every sum is added in a fixed order, so a row has the same bits in any batch of
// 2 .. 32 rows, and in any batch of 33 .. 64.
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "common.h"
#include "qgemm_shared.h"

using namespace vx;

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int NW = 8;            // waves per workgroup
constexpr int ACC_TILES = 8;     // tiles whose sums can wait in LDS between the passes of a wide slice

// block element held by slot i of lane group g (the prepared tiles' order), and the slot that nibble j feeds
__host__ __device__ inline int elt_of(int g, int slot) {
    const int base[8] = {0, 2, 16, 18, 1, 3, 17, 19};
    return 4 * g + base[slot];
}
__host__ __device__ inline int slot_of_nibble(int j) { return j < 4 ? 2 * j : 2 * (j - 4) + 1; }

__device__ __forceinline__ half2v as_h2(uint32_t u) {
    half2v v;
    __builtin_memcpy(&v, &u, 4);
    return v;
}
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t k) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(k));
    return r;
}
// A load through the global address space (pointers that arrive inside a by-value kernel argument are generic, and
// a generic load also waits on the LDS counter), and a pointer known to be the same in every lane.
template <class T> __device__ __forceinline__ T gload(const void *p) {
    return *(const __attribute__((address_space(1))) T *)(uintptr_t)p;
}
__device__ __forceinline__ const uint8_t *uniform_ptr(const uint8_t *p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const uint8_t *)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

// Eight nibbles of one dword -> the step's operand: exact integers q - 8 as f16. A nibble under 0x6400's exponent is
// the f16 1024 + q; one four bits higher is 1024 + 16 q, which one fused multiply-add brings to q - 8 as well.
// BIAS: what is subtracted from the code (8 for Q4_0, 0 for Q4_K's unsigned codes).
template <int BIAS> __device__ __forceinline__ half8 unpack_q4(uint32_t w, uint32_t k64) {
    const uint32_t w8 = w >> 8;
    const half2v a = as_h2(and_or(w, 0x000F000Fu, k64)), b = as_h2(and_or(w, 0x00F000F0u, k64));
    const half2v c = as_h2(and_or(w8, 0x000F000Fu, k64)), d = as_h2(and_or(w8, 0x00F000F0u, k64));
    const half2v m1032 = {(_Float16)(-1024.f - BIAS), (_Float16)(-1024.f - BIAS)}, m72 = {(_Float16)(-64.f - BIAS), (_Float16)(-64.f - BIAS)};
    const half2v s16 = {(_Float16)0.0625f, (_Float16)0.0625f};
    // (explicitly fused: the library is built without contraction of a * b + c)
    const half2v h0 = a + m1032, h1 = __builtin_elementwise_fma(b, s16, m72), h2 = c + m1032, h3 = __builtin_elementwise_fma(d, s16, m72);
    half8 r;
    r[0] = h0[0]; r[1] = h0[1]; r[2] = h1[0]; r[3] = h1[1];
    r[4] = h2[0]; r[5] = h2[1]; r[6] = h3[0]; r[7] = h3[1];
    return r;
}

// Eight biased bytes (q + 128, two dwords) -> exact integers q as f16: a byte under 0x64 is the f16 1024 + byte. Byte
// positions 0, 2, 1, 3 of a dword hold consecutive slots, so that each byte permute yields a finished pair.
template <int BIAS> __device__ __forceinline__ half8 unpack_q8(uint32_t w0, uint32_t w1) {
    const uint32_t c64 = 0x64646464u;
    const half2v off = {(_Float16)(1024.f + BIAS), (_Float16)(1024.f + BIAS)};
    const half2v h0 = as_h2(__builtin_amdgcn_perm(w0, c64, 0x00060004u)) - off, h1 = as_h2(__builtin_amdgcn_perm(w0, c64, 0x00070005u)) - off;
    const half2v h2 = as_h2(__builtin_amdgcn_perm(w1, c64, 0x00060004u)) - off, h3 = as_h2(__builtin_amdgcn_perm(w1, c64, 0x00070005u)) - off;
    half8 r;
    r[0] = h0[0]; r[1] = h0[1]; r[2] = h1[0]; r[3] = h1[1];
    r[4] = h2[0]; r[5] = h2[1]; r[6] = h3[0]; r[7] = h3[1];
    return r;
}
__device__ __forceinline__ float half_of(uint32_t w, int hi) {
    _Float16 dh;
    const uint16_t d16 = (uint16_t)(hi ? (w >> 16) : (w & 0xFFFFu));
    __builtin_memcpy(&dh, &d16, 2);
    return (float)dh;
}

// What the kernel needs to know of a packed format: the unit's size, what a lane requests of it (Ring), and how the
// request becomes block j's operand and scale.
struct SQ4_0 {
    static constexpr int UNIT = 1152, SCALES_AT = 1024;
    static constexpr bool TWO_SCALES = false, HAS_MIN = false;
    struct Ring {
        u32x4 c;
        u32x2 s;
    };
    static __device__ __forceinline__ Ring load(const uint8_t *u, int lane, int ln) {
        Ring x;
        x.c = gload<u32x4>(u + lane * 16);
        x.s = gload<u32x2>(u + SCALES_AT + ln * 8);
        return x;
    }
    static __device__ __forceinline__ half8 codes(const Ring &x, int j, uint32_t k64) { return unpack_q4<8>(x.c[j], k64); }
    static __device__ __forceinline__ float scale(const Ring &x, int j) { return half_of(x.s[j >> 1], j & 1); }
    static __device__ __forceinline__ float minimum(const Ring &, int) { return 0.f; }
};
// Q4_K (144-byte super-blocks of 8 sub-blocks of 32, pkg/gguf/dequant.go:333-409): element = d1 * q - m1 with
// d1 = d * sc and m1 = dmin * m per sub-block (both exact float32 products). A half chunk is half a super-block. A
// unit is 1536 bytes: the codes as in the Q4_0 unit (unsigned), then row r's d1[4] at 1024 + 32 r and m1[4] at
// 1040 + 32 r. The m1 term multiplies the activation's block sums (prepared with the tiles): one more FMA per output
// and block. 6 bits per weight against GGUF's 4.5.
struct SQ4_K {
    static constexpr int UNIT = 1536, SCALES_AT = 1024;
    static constexpr bool TWO_SCALES = false, HAS_MIN = true;
    struct Ring {
        u32x4 c;
        float4v d1, m1;
    };
    static __device__ __forceinline__ Ring load(const uint8_t *u, int lane, int ln) {
        Ring x;
        x.c = gload<u32x4>(u + lane * 16);
        x.d1 = gload<float4v>(u + SCALES_AT + ln * 32);
        x.m1 = gload<float4v>(u + SCALES_AT + ln * 32 + 16);
        return x;
    }
    static __device__ __forceinline__ half8 codes(const Ring &x, int j, uint32_t k64) { return unpack_q4<0>(x.c[j], k64); }
    static __device__ __forceinline__ float scale(const Ring &x, int j) { return x.d1[j]; }
    static __device__ __forceinline__ float minimum(const Ring &x, int j) { return x.m1[j]; }
};
// Q8_0: a unit is 2176 bytes, lane l = 16 g + r owns 32 of the first 2048: block j's eight codes at 8 j, as q + 128,
// slot s at byte (s & 4) + {0, 2, 1, 3}[s & 3]; row r's four f16 scales at 2048 + 8 r. 34 bytes per block as in GGUF.
struct SQ8_0 {
    static constexpr int UNIT = 2176, SCALES_AT = 2048;
    static constexpr bool TWO_SCALES = false, HAS_MIN = false;
    struct Ring {
        u32x4 c0, c1;
        u32x2 s;
    };
    static __device__ __forceinline__ Ring load(const uint8_t *u, int lane, int ln) {
        Ring x;
        x.c0 = gload<u32x4>(u + lane * 32);
        x.c1 = gload<u32x4>(u + lane * 32 + 16);
        x.s = gload<u32x2>(u + SCALES_AT + ln * 8);
        return x;
    }
    static __device__ __forceinline__ half8 codes(const Ring &x, int j, uint32_t) {
        return j == 0 ? unpack_q8<128>(x.c0[0], x.c0[1]) : j == 1 ? unpack_q8<128>(x.c0[2], x.c0[3]) : j == 2 ? unpack_q8<128>(x.c1[0], x.c1[1]) : unpack_q8<128>(x.c1[2], x.c1[3]);
    }
    static __device__ __forceinline__ float scale(const Ring &x, int j) { return half_of(x.s[j >> 1], j & 1); }
    static __device__ __forceinline__ float minimum(const Ring &, int) { return 0.f; }
};
// Q5_0 (22-byte blocks, pkg/gguf/dequant.go:100-145: element = float32(q - 16) * d) is packed into Q8_0 units with
// q - 16 as the code: the same kernel, the same product. Q5_K (176-byte super-blocks, dequant.go:411-470: element =
// d1 * q - m1 with 5-bit q) gets a unit of 2560 bytes: the codes one byte each in the Q8_0 unit's order (unsigned),
// then row r's d1[4] at 2048 + 32 r and m1[4] at 2064 + 32 r; its min term as Q4_K's. 10 bits per weight against 5.5.
struct SQ5_K {
    static constexpr int UNIT = 2560, SCALES_AT = 2048;
    static constexpr bool TWO_SCALES = false, HAS_MIN = true;
    struct Ring {
        u32x4 c0, c1;
        float4v d1, m1;
    };
    static __device__ __forceinline__ Ring load(const uint8_t *u, int lane, int ln) {
        Ring x;
        x.c0 = gload<u32x4>(u + lane * 32);
        x.c1 = gload<u32x4>(u + lane * 32 + 16);
        x.d1 = gload<float4v>(u + SCALES_AT + ln * 32);
        x.m1 = gload<float4v>(u + SCALES_AT + ln * 32 + 16);
        return x;
    }
    static __device__ __forceinline__ half8 codes(const Ring &x, int j, uint32_t) {
        return j == 0 ? unpack_q8<0>(x.c0[0], x.c0[1]) : j == 1 ? unpack_q8<0>(x.c0[2], x.c0[3]) : j == 2 ? unpack_q8<0>(x.c1[0], x.c1[1]) : unpack_q8<0>(x.c1[2], x.c1[3]);
    }
    static __device__ __forceinline__ float scale(const Ring &x, int j) { return x.d1[j]; }
    static __device__ __forceinline__ float minimum(const Ring &x, int j) { return x.m1[j]; }
};
// Q6_K (210-byte super-blocks of 256 elements, pkg/gguf/dequant.go:272-331): a half chunk is half a super-block, and
// every 16 of its elements carry a scale of their own, so a 32-column step is two v_mfma_f32_16x16x16_f16 per
// activation half instead of one x32. A unit is 2560 bytes: lane l = 16 g + r owns 32 of the first 2048 — block j's
// codes at 8 j, one byte each (q, 0 .. 63): elements 4 g .. 4 g + 3, then 16 + 4 g .. 16 + 4 g + 3 — and row r's eight
// float32 scales d * sc (exact products; element = scale * float32(q - 32) as the reference rounds it) at 2048 + 32 r,
// scale 2 j + h for elements 16 h .. 16 h + 15 of block j. 10 bits per weight against GGUF's 6.5625.
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ half4v unpack_q6(uint32_t w) {
    const uint32_t c64 = 0x64646464u;
    const half2v off = {(_Float16)1056.f, (_Float16)1056.f};  // 1024 + 32
    const half2v h0 = as_h2(__builtin_amdgcn_perm(w, c64, 0x00060004u)) - off, h1 = as_h2(__builtin_amdgcn_perm(w, c64, 0x00070005u)) - off;
    half4v r;
    r[0] = h0[0]; r[1] = h0[1]; r[2] = h1[0]; r[3] = h1[1];  // elements 0, 2, 1, 3 of the four: the activation halves' order
    return r;
}
struct SQ6_K {
    static constexpr int UNIT = 2560, SCALES_AT = 2048;
    static constexpr bool TWO_SCALES = true, HAS_MIN = false;
    struct Ring {
        u32x4 c0, c1;
        float4v s0, s1;
    };
    static __device__ __forceinline__ Ring load(const uint8_t *u, int lane, int ln) {
        Ring x;
        x.c0 = gload<u32x4>(u + lane * 32);
        x.c1 = gload<u32x4>(u + lane * 32 + 16);
        x.s0 = gload<float4v>(u + SCALES_AT + ln * 32);
        x.s1 = gload<float4v>(u + SCALES_AT + ln * 32 + 16);
        return x;
    }
    // h: which 16 elements of block j
    static __device__ __forceinline__ half4v codes16(const Ring &x, int j, int h) {
        const uint32_t w = j < 2 ? x.c0[2 * j + h] : x.c1[2 * (j - 2) + h];
        return unpack_q6(w);
    }
    static __device__ __forceinline__ float scale16(const Ring &x, int j, int h) { return j < 2 ? x.s0[2 * j + h] : x.s1[2 * (j - 2) + h]; }
    // (unused forms of the one-scale interface)
    static __device__ __forceinline__ half8 codes(const Ring &, int, uint32_t) { return half8{}; }
    static __device__ __forceinline__ float scale(const Ring &, int) { return 0.f; }
    static __device__ __forceinline__ float minimum(const Ring &, int) { return 0.f; }
};

__host__ __device__ inline int q8_byte_of_slot(int slot) {
    const int pos[4] = {0, 2, 1, 3};
    return (slot & 4) + pos[slot & 3];
}

// ------------------------------------------------------------------------------------------------ pack / unpack
// grid = (tiles, half chunks), block = 64: lane l writes its 16 code bytes, lanes 0 .. 15 their row's scales.
__global__ void __launch_bounds__(64) pack_q4_0_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ packed, int n_hc) {
    const int T = blockIdx.x, hc = blockIdx.y, lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const size_t row_bytes = (size_t)n_hc * 4 * 18;
    const uint8_t *row = raw + (size_t)(T * 16 + r) * row_bytes + (size_t)hc * 4 * 18;
    uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ4_0::UNIT;
    uint32_t out[4];
    for (int j = 0; j < 4; j++) {
        const uint8_t *blk = row + j * 18;
        uint32_t w = 0;
        for (int nib = 0; nib < 8; nib++) {
            const int e = elt_of(g, slot_of_nibble(nib));
            const uint32_t q = e < 16 ? (blk[2 + e] & 0xFu) : (blk[2 + e - 16] >> 4);
            w |= q << (4 * nib);
        }
        out[j] = w;
    }
    *(u32x4 *)(u + lane * 16) = (u32x4){out[0], out[1], out[2], out[3]};
    if (g == 0) {
        uint16_t d[4];
        for (int j = 0; j < 4; j++) d[j] = (uint16_t)(row[j * 18] | (row[j * 18 + 1] << 8));
        *(u32x2 *)(u + 1024 + r * 8) = (u32x2){(uint32_t)d[0] | ((uint32_t)d[1] << 16), (uint32_t)d[2] | ((uint32_t)d[3] << 16)};
    }
}

// One thread per element: scale * float32(q - 8) as gguf.DequantizeQ4_0 computes it, read from the packed form.
__global__ void __launch_bounds__(256) dequant_packed_q4_0_kernel(const uint8_t *__restrict__ packed, float *__restrict__ dst, int n,
                                                                  int k) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)n * k) return;
    const int row = (int)(idx / k), col = (int)(idx % k);
    const int T = row >> 4, r = row & 15, hc = col >> 7, j = (col >> 5) & 3, e = col & 31;
    const int n_hc = k >> 7;
    const uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ4_0::UNIT;
    int g = 0, nib = 0;
    for (int gg = 0; gg < 4; gg++)
        for (int i = 0; i < 8; i++)
            if (elt_of(gg, slot_of_nibble(i)) == e) {
                g = gg;
                nib = i;
            }
    const uint32_t w = *(const uint32_t *)(u + (g * 16 + r) * 16 + j * 4);
    const int q = (int)((w >> (4 * nib)) & 0xFu);
    _Float16 d;
    __builtin_memcpy(&d, u + 1024 + r * 8 + j * 2, 2);
    dst[idx] = __fmul_rn((float)d, (float)(q - 8));
}

__global__ void __launch_bounds__(64) pack_q8_0_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ packed, int n_hc) {
    const int T = blockIdx.x, hc = blockIdx.y, lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const size_t row_bytes = (size_t)n_hc * 4 * 34;
    const uint8_t *row = raw + (size_t)(T * 16 + r) * row_bytes + (size_t)hc * 4 * 34;
    uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ8_0::UNIT;
    uint32_t out[8];
    for (int j = 0; j < 4; j++) {
        const uint8_t *blk = row + j * 34;
        uint32_t w[2] = {0, 0};
        for (int slot = 0; slot < 8; slot++) {
            const int at = q8_byte_of_slot(slot);
            w[at >> 2] |= (uint32_t)(uint8_t)(blk[2 + elt_of(g, slot)] ^ 0x80u) << (8 * (at & 3));
        }
        out[2 * j] = w[0];
        out[2 * j + 1] = w[1];
    }
    *(u32x4 *)(u + lane * 32) = (u32x4){out[0], out[1], out[2], out[3]};
    *(u32x4 *)(u + lane * 32 + 16) = (u32x4){out[4], out[5], out[6], out[7]};
    if (g == 0) {
        uint16_t d[4];
        for (int j = 0; j < 4; j++) d[j] = (uint16_t)(row[j * 34] | (row[j * 34 + 1] << 8));
        *(u32x2 *)(u + SQ8_0::SCALES_AT + r * 8) = (u32x2){(uint32_t)d[0] | ((uint32_t)d[1] << 16), (uint32_t)d[2] | ((uint32_t)d[3] << 16)};
    }
}

// Q5_0 rows into Q8_0 units: code q - 16 (dequant.go:100-145: low nibbles and bits 0 .. 15 of qh are elements 0 .. 15,
// high nibbles and bits 16 .. 31 elements 16 .. 31)
__global__ void __launch_bounds__(64) pack_q5_0_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ packed, int n_hc) {
    const int T = blockIdx.x, hc = blockIdx.y, lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const size_t row_bytes = (size_t)n_hc * 4 * 22;
    const uint8_t *row = raw + (size_t)(T * 16 + r) * row_bytes + (size_t)hc * 4 * 22;
    uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ8_0::UNIT;
    uint32_t out[8];
    for (int j = 0; j < 4; j++) {
        const uint8_t *blk = row + j * 22;
        const uint32_t qh = (uint32_t)blk[2] | ((uint32_t)blk[3] << 8) | ((uint32_t)blk[4] << 16) | ((uint32_t)blk[5] << 24);
        uint32_t w[2] = {0, 0};
        for (int slot = 0; slot < 8; slot++) {
            const int e = elt_of(g, slot), at = q8_byte_of_slot(slot);
            const int q = (int)(e < 16 ? (blk[6 + e] & 0xFu) : (blk[6 + e - 16] >> 4)) | (int)(((qh >> e) & 1u) << 4);
            w[at >> 2] |= (uint32_t)(uint8_t)(q - 16 + 128) << (8 * (at & 3));
        }
        out[2 * j] = w[0];
        out[2 * j + 1] = w[1];
    }
    *(u32x4 *)(u + lane * 32) = (u32x4){out[0], out[1], out[2], out[3]};
    *(u32x4 *)(u + lane * 32 + 16) = (u32x4){out[4], out[5], out[6], out[7]};
    if (g == 0) {
        uint16_t d[4];
        for (int j = 0; j < 4; j++) d[j] = (uint16_t)(row[j * 22] | (row[j * 22 + 1] << 8));
        *(u32x2 *)(u + SQ8_0::SCALES_AT + r * 8) = (u32x2){(uint32_t)d[0] | ((uint32_t)d[1] << 16), (uint32_t)d[2] | ((uint32_t)d[3] << 16)};
    }
}

// scale * float32(q) as gguf.DequantizeQ8_0 computes it (pkg/gguf/dequant.go:58-95), read from the packed form.
__global__ void __launch_bounds__(256) dequant_packed_q8_0_kernel(const uint8_t *__restrict__ packed, float *__restrict__ dst, int n,
                                                                  int k) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)n * k) return;
    const int row = (int)(idx / k), col = (int)(idx % k);
    const int T = row >> 4, r = row & 15, hc = col >> 7, j = (col >> 5) & 3, e = col & 31;
    const int n_hc = k >> 7;
    const uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ8_0::UNIT;
    int g = 0, slot = 0;
    for (int gg = 0; gg < 4; gg++)
        for (int i = 0; i < 8; i++)
            if (elt_of(gg, i) == e) {
                g = gg;
                slot = i;
            }
    const int q = (int)(int8_t)(u[(g * 16 + r) * 32 + j * 8 + q8_byte_of_slot(slot)] ^ 0x80u);
    _Float16 d;
    __builtin_memcpy(&d, u + SQ8_0::SCALES_AT + r * 8 + j * 2, 2);
    dst[idx] = __fmul_rn((float)d, (float)q);
}

// Q4_K: scale and min of sub-block j of a super-block (get_scale_min_k4, pkg/gguf/dequant.go:400-409)
__host__ __device__ inline void q4k_scale_min(const uint8_t *q, int j, int *sc, int *mn) {
    if (j < 4) {
        *sc = q[j] & 63;
        *mn = q[j + 4] & 63;
    } else {
        *sc = (q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4);
        *mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}
__global__ void __launch_bounds__(64) pack_q4_k_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ packed, int n_hc) {
    const int T = blockIdx.x, hc = blockIdx.y, lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const size_t row_bytes = (size_t)(n_hc / 2) * 144;
    const uint8_t *sb = raw + (size_t)(T * 16 + r) * row_bytes + (size_t)(hc >> 1) * 144;
    uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ4_K::UNIT;
    uint32_t out[4];
    for (int j = 0; j < 4; j++) {
        const int sbi = 4 * (hc & 1) + j;  // sub-block: pair sbi / 2 of 32 bytes, low or high nibbles
        const uint8_t *qs = sb + 16 + 32 * (sbi >> 1);
        uint32_t w = 0;
        for (int nib = 0; nib < 8; nib++) {
            const int e = elt_of(g, slot_of_nibble(nib));
            const uint32_t q = (sbi & 1) ? (qs[e] >> 4) : (qs[e] & 0xFu);
            w |= q << (4 * nib);
        }
        out[j] = w;
    }
    *(u32x4 *)(u + lane * 16) = (u32x4){out[0], out[1], out[2], out[3]};
    if (g == 0) {
        _Float16 dh, mh;
        const uint16_t d16 = (uint16_t)(sb[0] | (sb[1] << 8)), m16 = (uint16_t)(sb[2] | (sb[3] << 8));
        __builtin_memcpy(&dh, &d16, 2);
        __builtin_memcpy(&mh, &m16, 2);
        float d1[4], m1[4];
        for (int j = 0; j < 4; j++) {
            int sc, mn;
            q4k_scale_min(sb + 4, 4 * (hc & 1) + j, &sc, &mn);
            d1[j] = __fmul_rn((float)dh, (float)sc);
            m1[j] = __fmul_rn((float)mh, (float)mn);
        }
        *(float4v *)(u + SQ4_K::SCALES_AT + r * 32) = (float4v){d1[0], d1[1], d1[2], d1[3]};
        *(float4v *)(u + SQ4_K::SCALES_AT + r * 32 + 16) = (float4v){m1[0], m1[1], m1[2], m1[3]};
    }
}

// d1 * float32(q) - m1 as gguf.DequantizeQ4_K rounds it (pkg/gguf/dequant.go:333-398), from the packed form.
__global__ void __launch_bounds__(256) dequant_packed_q4_k_kernel(const uint8_t *__restrict__ packed, float *__restrict__ dst, int n,
                                                                  int k) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)n * k) return;
    const int row = (int)(idx / k), col = (int)(idx % k);
    const int T = row >> 4, r = row & 15, hc = col >> 7, j = (col >> 5) & 3, e = col & 31;
    const int n_hc = k >> 7;
    const uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ4_K::UNIT;
    int g = 0, nib = 0;
    for (int gg = 0; gg < 4; gg++)
        for (int i = 0; i < 8; i++)
            if (elt_of(gg, slot_of_nibble(i)) == e) {
                g = gg;
                nib = i;
            }
    const uint32_t w = *(const uint32_t *)(u + (g * 16 + r) * 16 + j * 4);
    const int q = (int)((w >> (4 * nib)) & 0xFu);
    float d1, m1;
    __builtin_memcpy(&d1, u + SQ4_K::SCALES_AT + r * 32 + j * 4, 4);
    __builtin_memcpy(&m1, u + SQ4_K::SCALES_AT + r * 32 + 16 + j * 4, 4);
    dst[idx] = __fsub_rn(__fmul_rn(d1, (float)q), m1);
}

// Q5_K (dequant.go:411-470): sub-block sbi's element e is nibble (sbi & 1) of qs[32 (sbi / 2) + e] plus 16 times bit
// sbi of qh[e]
__global__ void __launch_bounds__(64) pack_q5_k_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ packed, int n_hc) {
    const int T = blockIdx.x, hc = blockIdx.y, lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const size_t row_bytes = (size_t)(n_hc / 2) * 176;
    const uint8_t *sb = raw + (size_t)(T * 16 + r) * row_bytes + (size_t)(hc >> 1) * 176;
    uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ5_K::UNIT;
    uint32_t out[8];
    for (int j = 0; j < 4; j++) {
        const int sbi = 4 * (hc & 1) + j;
        const uint8_t *qs = sb + 48 + 32 * (sbi >> 1), *qh = sb + 16;
        uint32_t w[2] = {0, 0};
        for (int slot = 0; slot < 8; slot++) {
            const int e = elt_of(g, slot), at = q8_byte_of_slot(slot);
            const uint32_t q = ((sbi & 1) ? (qs[e] >> 4) : (qs[e] & 0xFu)) + (((qh[e] >> sbi) & 1u) << 4);
            w[at >> 2] |= q << (8 * (at & 3));
        }
        out[2 * j] = w[0];
        out[2 * j + 1] = w[1];
    }
    *(u32x4 *)(u + lane * 32) = (u32x4){out[0], out[1], out[2], out[3]};
    *(u32x4 *)(u + lane * 32 + 16) = (u32x4){out[4], out[5], out[6], out[7]};
    if (g == 0) {
        _Float16 dh, mh;
        const uint16_t d16 = (uint16_t)(sb[0] | (sb[1] << 8)), m16 = (uint16_t)(sb[2] | (sb[3] << 8));
        __builtin_memcpy(&dh, &d16, 2);
        __builtin_memcpy(&mh, &m16, 2);
        float d1[4], m1[4];
        for (int j = 0; j < 4; j++) {
            int sc, mn;
            q4k_scale_min(sb + 4, 4 * (hc & 1) + j, &sc, &mn);
            d1[j] = __fmul_rn((float)dh, (float)sc);
            m1[j] = __fmul_rn((float)mh, (float)mn);
        }
        *(float4v *)(u + SQ5_K::SCALES_AT + r * 32) = (float4v){d1[0], d1[1], d1[2], d1[3]};
        *(float4v *)(u + SQ5_K::SCALES_AT + r * 32 + 16) = (float4v){m1[0], m1[1], m1[2], m1[3]};
    }
}

__global__ void __launch_bounds__(256) dequant_packed_q5_k_kernel(const uint8_t *__restrict__ packed, float *__restrict__ dst, int n,
                                                                  int k) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)n * k) return;
    const int row = (int)(idx / k), col = (int)(idx % k);
    const int T = row >> 4, r = row & 15, hc = col >> 7, j = (col >> 5) & 3, e = col & 31;
    const int n_hc = k >> 7;
    const uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ5_K::UNIT;
    int g = 0, slot = 0;
    for (int gg = 0; gg < 4; gg++)
        for (int i = 0; i < 8; i++)
            if (elt_of(gg, i) == e) {
                g = gg;
                slot = i;
            }
    const int q = (int)u[(g * 16 + r) * 32 + j * 8 + q8_byte_of_slot(slot)];
    float d1, m1;
    __builtin_memcpy(&d1, u + SQ5_K::SCALES_AT + r * 32 + j * 4, 4);
    __builtin_memcpy(&m1, u + SQ5_K::SCALES_AT + r * 32 + 16 + j * 4, 4);
    dst[idx] = __fsub_rn(__fmul_rn(d1, (float)q), m1);
}

// Q6_K code and scale of element e (0 .. 127) of half nn of a super-block (dequant.go:272-331)
__host__ __device__ inline int q6k_code(const uint8_t *sb, int nn, int e) {
    const int j = e >> 5, l = e & 31;
    const uint8_t ql = sb[64 * nn + 32 * (j & 1) + l], qh = sb[128 + 32 * nn + l];
    return (int)(((j & 2) ? (ql >> 4) : (ql & 0xF)) | (((qh >> (2 * j)) & 3) << 4));
}
__global__ void __launch_bounds__(64) pack_q6_k_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ packed, int n_hc) {
    const int T = blockIdx.x, hc = blockIdx.y, lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const size_t row_bytes = (size_t)(n_hc / 2) * 210;
    const uint8_t *sb = raw + (size_t)(T * 16 + r) * row_bytes + (size_t)(hc >> 1) * 210;
    const int nn = hc & 1;
    uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ6_K::UNIT;
    uint32_t out[8];
    for (int j = 0; j < 4; j++)
        for (int h = 0; h < 2; h++) {
            uint32_t w = 0;
            for (int i = 0; i < 4; i++) w |= (uint32_t)q6k_code(sb, nn, 32 * j + 16 * h + 4 * g + i) << (8 * i);
            out[2 * j + h] = w;
        }
    *(u32x4 *)(u + lane * 32) = (u32x4){out[0], out[1], out[2], out[3]};
    *(u32x4 *)(u + lane * 32 + 16) = (u32x4){out[4], out[5], out[6], out[7]};
    if (g == 0) {
        _Float16 dh;
        const uint16_t d16 = (uint16_t)(sb[208] | (sb[209] << 8));
        __builtin_memcpy(&dh, &d16, 2);
        const float d = (float)dh;
        float sc[8];
        for (int i = 0; i < 8; i++) sc[i] = __fmul_rn(d, (float)(int8_t)sb[192 + 8 * nn + i]);
        *(float4v *)(u + SQ6_K::SCALES_AT + r * 32) = (float4v){sc[0], sc[1], sc[2], sc[3]};
        *(float4v *)(u + SQ6_K::SCALES_AT + r * 32 + 16) = (float4v){sc[4], sc[5], sc[6], sc[7]};
    }
}

// d * float32(sc) * float32(q - 32) as gguf.DequantizeQ6_K rounds it (pkg/gguf/dequant.go:272-331), from the packed form.
__global__ void __launch_bounds__(256) dequant_packed_q6_k_kernel(const uint8_t *__restrict__ packed, float *__restrict__ dst, int n,
                                                                  int k) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)n * k) return;
    const int row = (int)(idx / k), col = (int)(idx % k);
    const int T = row >> 4, r = row & 15, hc = col >> 7, j = (col >> 5) & 3, e = col & 31;
    const int n_hc = k >> 7;
    const uint8_t *u = packed + ((size_t)T * n_hc + hc) * SQ6_K::UNIT;
    const int h = e >> 4, g = (e & 15) >> 2, i = e & 3;
    const int q = (int)u[(g * 16 + r) * 32 + j * 8 + h * 4 + i];
    float s;
    __builtin_memcpy(&s, u + SQ6_K::SCALES_AT + r * 32 + (2 * j + h) * 4, 4);
    dst[idx] = __fmul_rn(s, (float)(q - 32));
}

// ------------------------------------------------------------------------------------------------ the GEMM
// First unit of tile T among up to three packed matrices (all arguments the same in every lane). A plain function of
// values: the same selection written over a lambda's captures is compiled into an indexed load of the closure
// object, which then lives in scratch memory.
__device__ __forceinline__ const uint8_t *tile_base(int T, const uint8_t *w0, const uint8_t *w1, const uint8_t *w2, int e0, int e1,
                                                    size_t tile_stride) {
    uint64_t b = (uint64_t)(uintptr_t)w0;
    int local = T;
    if (T >= e0) {
        b = (uint64_t)(uintptr_t)w1;
        local = T - e0;
    }
    if (T >= e1) {
        b = (uint64_t)(uintptr_t)w2;
        local = T - e1;
    }
    return (const uint8_t *)(uintptr_t)(b + (uint64_t)local * tile_stride);
}

struct PackedSegs {  // up to three packed matrices whose rows follow one another in the output
    const uint8_t *w[3];
    int t_end[3];  // tiles before the end of each
};

template <int MT, bool TWO> struct APhase {
    half8 h[4][MT], l[4][MT];
    float4v cs[MT];
};
template <int MT> struct APhase<MT, true> {  // the halves of each operand that belong to the first and the second 16 elements
    half4v h[4][MT][2], l[4][MT][2];
    float4v cs[MT];
};
__device__ __forceinline__ half4v first16(half8 v) { return __builtin_shufflevector(v, v, 0, 1, 4, 5); }
__device__ __forceinline__ half4v second16(half8 v) { return __builtin_shufflevector(v, v, 2, 3, 6, 7); }
struct StreamShape {
    int M, Mpad, N, n_hc, npass, t_end0, t_end1;
    int split_groups;  // (the two-format launch: row groups of the first format)
};

// grid = (row groups, K slices), block = 512. PH: half chunks a wave holds per pass (1 or 2); RG: tiles per
// reduction; EPI: finish Q|K|V rows (one slice).
// The workgroup's share: row group gx of gdx over the tiles [tile_lo, tile_lo + tile_cnt) (of format W), K slice
// blockIdx.y. The LDS areas come from the kernel (red: [2][NW][16 * MT * (16 RG + 4)] floats).
template <class W, int PH, int RG, int MT, bool EPI>
__device__ __forceinline__ void
qstream_body(const uint8_t *__restrict__ pw0, const uint8_t *__restrict__ pw1, const uint8_t *__restrict__ pw2,
             const half8 *__restrict__ a_tiles, const float *__restrict__ a_cscale, const float *__restrict__ a_inv_scale,
             const float *__restrict__ a_bsum, float *__restrict__ partial, const StreamShape &a, const QkvEpi &epi,
             float (*red)[NW][16 * MT * (16 * RG + 4)], float *wait_sums, float *s_fac, const int gx, const int gdx,
             const int tile_lo, const int tile_cnt) {
    constexpr int D = RG * PH;            // requests in flight per wave
    constexpr int TP = 16 * RG + 4;       // floats per row of a wave's block in LDS

    const int tid = threadIdx.x, lane = tid & 63, ln = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int mtiles = a.Mpad >> 4, n_hc = a.n_hc;
    const int gb = tile_cnt / gdx, gr = tile_cnt % gdx;
    const int t0 = tile_lo + gx * gb + min(gx, gr), nt = gb + (gx < gr ? 1 : 0);
    const int sb = n_hc / (int)gridDim.y, sr = n_hc % (int)gridDim.y;
    const int h0 = blockIdx.y * sb + min((int)blockIdx.y, sr), nh = sb + ((int)blockIdx.y < sr ? 1 : 0);

    const size_t tile_stride = (size_t)n_hc * W::UNIT;
    typedef typename W::Ring WHalf;
    // the packed matrices' addresses and tile ends as scalars (the same in every lane)
    // (through readfirstlane: selecting among plain kernel arguments becomes an indexed load of the argument
    // block, copied to scratch memory for it)
    const uint8_t *const w0 = uniform_ptr(pw0), *const w1 = uniform_ptr(pw1), *const w2 = uniform_ptr(pw2);
    const int e0 = __builtin_amdgcn_readfirstlane(a.t_end0), e1 = __builtin_amdgcn_readfirstlane(a.t_end1);
    uint32_t k64;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(k64));

    if (EPI) {
        // row factors with the pending 1/rms of the RMSNorm that fed the activation: whole-wave computations
        for (int r = wave; r < 16 * MT; r += NW) {
            const float f = row_factor(a_inv_scale, epi.rn, r);
            if (lane == 0) s_fac[r] = f;
        }
    }

    int buf = 0;
    for (int pass = 0; pass < a.npass; pass++) {
        const int hp = h0 + pass * NW * PH, nhp = min(nh - pass * NW * PH, NW * PH);  // this pass's half chunks
        // (separate scalars, not arrays: an array indexed in an unrolled loop can end up in scratch memory)
        const bool valid0 = wave < nhp, valid1 = PH > 1 && NW + wave < nhp;
        const int hc0 = hp + min(wave, nhp - 1), hc1 = hp + min(NW + wave, nhp - 1);
        auto ldw = [&](int tile, int p) __attribute__((always_inline)) {
            const uint8_t *u = uniform_ptr(tile_base(t0 + min(tile, nt - 1), w0, w1, w2, e0, e1, tile_stride) + (size_t)(p == 0 ? hc0 : hc1) * W::UNIT);
            return W::load(u, lane, ln);
        };
        APhase<MT, W::TWO_SCALES> A[PH];
        float4v bsum[W::HAS_MIN ? PH : 1][4][MT];
#pragma unroll
        for (int p = 0; p < PH; p++) {
            const int hc = p == 0 ? hc0 : hc1;
            const half8 *base = a_tiles + ((size_t)(hc * 4) * mtiles * 2) * 64 + lane;
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const half8 vh = gload<half8>(base + ((size_t)(j * mtiles + t) * 2 + 0) * 64);
                    const half8 vl = gload<half8>(base + ((size_t)(j * mtiles + t) * 2 + 1) * 64);
                    if constexpr (W::TWO_SCALES) {
                        A[p].h[j][t][0] = first16(vh);
                        A[p].h[j][t][1] = second16(vh);
                        A[p].l[j][t][0] = first16(vl);
                        A[p].l[j][t][1] = second16(vl);
                    } else {
                        A[p].h[j][t] = vh;
                        A[p].l[j][t] = vl;
                    }
                }
#pragma unroll
            for (int t = 0; t < MT; t++)
                A[p].cs[t] = gload<float4v>(a_cscale + (size_t)(hc >> 1) * a.Mpad + t * 16 + 4 * g);
            if constexpr (W::HAS_MIN) {  // the activation's block sums of this half chunk, rows 16 t + 4 g + e
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int t = 0; t < MT; t++) bsum[p][j][t] = gload<float4v>(a_bsum + (size_t)(hc * 4 + j) * a.Mpad + t * 16 + 4 * g);
            }
        }
        WHalf ring[D];
#pragma unroll
        for (int i = 0; i < D; i++) ring[i] = ldw(i / PH, i % PH);

        for (int tb = 0; tb < nt; tb += RG) {
            float4v acc[RG][MT];
#pragma unroll
            for (int r = 0; r < RG; r++) {
#pragma unroll
                for (int m = 0; m < MT; m++) acc[r][m] = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int p = 0; p < PH; p++) {
                    const WHalf x = ring[r * PH + p];
                    ring[r * PH + p] = ldw(tb + RG + r, p);
                    if (p == 0 ? valid0 : valid1) {
                        float4v tmp[MT];
#pragma unroll
                        for (int m = 0; m < MT; m++) tmp[m] = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            if constexpr (W::TWO_SCALES) {
#pragma unroll
                                for (int h = 0; h < 2; h++) {
                                    const half4v wb = W::codes16(x, j, h);
                                    const float d = W::scale16(x, j, h);
                                    float4v P[MT];
#pragma unroll
                                    for (int m = 0; m < MT; m++)
                                        P[m] = __builtin_amdgcn_mfma_f32_16x16x16f16(A[p].h[j][m][h], wb, (float4v){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                                    for (int m = 0; m < MT; m++) P[m] = __builtin_amdgcn_mfma_f32_16x16x16f16(A[p].l[j][m][h], wb, P[m], 0, 0, 0);
#pragma unroll
                                    for (int m = 0; m < MT; m++)
#pragma unroll
                                        for (int e = 0; e < 4; e++) tmp[m][e] = __builtin_fmaf(d, P[m][e], tmp[m][e]);
                                }
                            } else {
                                const half8 wb = W::codes(x, j, k64);
                                const float d = W::scale(x, j);
                                float4v P[MT];
#pragma unroll
                                for (int m = 0; m < MT; m++)
                                    P[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[p].h[j][m], wb, (float4v){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                                for (int m = 0; m < MT; m++) P[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[p].l[j][m], wb, P[m], 0, 0, 0);
#pragma unroll
                                for (int m = 0; m < MT; m++)
#pragma unroll
                                    for (int e = 0; e < 4; e++) tmp[m][e] = __builtin_fmaf(d, P[m][e], tmp[m][e]);
                                if constexpr (W::HAS_MIN) {
                                    const float mn = -W::minimum(x, j);
#pragma unroll
                                    for (int m = 0; m < MT; m++)
#pragma unroll
                                        for (int e = 0; e < 4; e++) tmp[m][e] = __builtin_fmaf(mn, bsum[p][j][m][e], tmp[m][e]);
                                }
                            }
                        }
#pragma unroll
                        for (int m = 0; m < MT; m++)
#pragma unroll
                            for (int e = 0; e < 4; e++) acc[r][m][e] = __builtin_fmaf(A[p].cs[m][e], tmp[m][e], acc[r][m][e]);
                    }
                }
            }
            // the waves' sums of these RG tiles: lane (g, ln) of tile r holds C[16 m + 4 g + e][16 r + ln]
            float *T = &red[buf][wave][0];
#pragma unroll
            for (int r = 0; r < RG; r++)
#pragma unroll
                for (int m = 0; m < MT; m++)
#pragma unroll
                    for (int e = 0; e < 4; e++) T[(m * 16 + 4 * g + e) * TP + r * 16 + ln] = acc[r][m][e];
            __syncthreads();
            const int ntile = min(RG, nt - tb);
            constexpr int F4 = 16 * MT * RG * 4;  // float4 groups of a full block
#pragma unroll
            for (int f0 = 0; f0 < F4; f0 += 64 * NW) {
                const int f = f0 + tid;
                const int ml = f / (RG * 4), nl = (f % (RG * 4)) * 4;
                if (f < F4 && nl < ntile * 16) {
                    float4 c = *(const float4 *)(&red[buf][0][0] + ml * TP + nl);
#pragma unroll
                    for (int w = 1; w < NW; w++) {
                        const float4 d = *(const float4 *)(&red[buf][w][0] + ml * TP + nl);
                        c.x += d.x; c.y += d.y; c.z += d.z; c.w += d.w;
                    }
                    if (!EPI) {
                        if (ml < a.M)
                            *(float4 *)(partial + ((size_t)blockIdx.y * a.M + ml) * a.N + (size_t)(t0 + tb) * 16 + nl) = c;
                    } else {
                        // sums of the earlier passes wait in LDS, [tile][row][16 columns]
                        float4 *ws = (float4 *)(wait_sums + ((size_t)(tb * 16 * MT + ml * RG) * 16 + nl));
                        if (a.npass > 1) {
                            if (pass > 0) {
                                const float4 p = *ws;
                                c.x += p.x; c.y += p.y; c.z += p.z; c.w += p.w;
                            }
                            if (pass + 1 < a.npass) *ws = c;
                        }
                        if (pass + 1 == a.npass && ml < a.M) {
                            // columns n .. n+3 of row m: two RoPE pairs of a Q or K head, or four V values
                            // (the arithmetic of rope_store_partials_kernel)
                            const int m = ml, n = (t0 + tb) * 16 + nl;
                            const float inv = s_fac[ml];
                            const float a0 = __fmul_rn(c.x, inv), b0 = __fmul_rn(c.y, inv), a1 = __fmul_rn(c.z, inv), b1 = __fmul_rn(c.w, inv);
                            const bool is_q = n < epi.qd, is_v = n >= epi.qd + epi.kvd;
                            const int o = is_q ? n : (is_v ? n - epi.qd - epi.kvd : n - epi.qd);
                            float4 r4 = make_float4(a0, b0, a1, b1);
                            if (!is_v) {
                                const float2 *cs = epi.cs_tab + (size_t)m * (epi.head_dim >> 1) + ((o & (epi.head_dim - 1)) >> 1);
                                const float2 c0 = cs[0], c1 = cs[1];
                                r4.x = __fsub_rn(__fmul_rn(a0, c0.x), __fmul_rn(b0, c0.y));
                                r4.y = __fadd_rn(__fmul_rn(a0, c0.y), __fmul_rn(b0, c0.x));
                                r4.z = __fsub_rn(__fmul_rn(a1, c1.x), __fmul_rn(b1, c1.y));
                                r4.w = __fadd_rn(__fmul_rn(a1, c1.y), __fmul_rn(b1, c1.x));
                            }
                            if (is_q) {
                                *(float4 *)(epi.q_out + (size_t)m * epi.qd + o) = r4;
                            } else {
                                const int slot = epi.slots[m], blk = slot / epi.block_size, off = slot - blk * epi.block_size;
                                const size_t part = (size_t)epi.block_size * epi.kvd;
                                const size_t at = (size_t)blk * 2 * part + (size_t)off * epi.kvd + (is_v ? part : 0) + o;
                                if (epi.pool_f16) {
                                    typedef _Float16 half4w __attribute__((ext_vector_type(4)));
                                    const half4w h4 = {(_Float16)r4.x, (_Float16)r4.y, (_Float16)r4.z, (_Float16)r4.w};
                                    *(half4w *)((_Float16 *)epi.pool + at) = h4;
                                } else {
                                    *(float4 *)((float *)epi.pool + at) = r4;
                                }
                            }
                        }
                    }
                }
            }
            buf ^= 1;
        }
    }
}

// grid = (row groups, K slices), block = 512.
template <class W, int PH, int RG, int MT, bool EPI>
__global__ void __launch_bounds__(64 * NW, 1)
qstream_kernel(const uint8_t *__restrict__ pw0, const uint8_t *__restrict__ pw1, const uint8_t *__restrict__ pw2,
               const half8 *__restrict__ a_tiles, const float *__restrict__ a_cscale, const float *__restrict__ a_inv_scale,
               const float *__restrict__ a_bsum, float *__restrict__ partial, const StreamShape a, const QkvEpi epi) {
    __shared__ __attribute__((aligned(16))) float red[2][NW][16 * MT * (16 * RG + 4)];
    __shared__ __attribute__((aligned(16))) float wait_sums[EPI ? ACC_TILES * 16 * 16 * MT : 4];
    __shared__ float s_fac[16 * MT];
    qstream_body<W, PH, RG, MT, EPI>(pw0, pw1, pw2, a_tiles, a_cscale, a_inv_scale, a_bsum, partial, a, epi, red, wait_sums, s_fac,
                                     (int)blockIdx.x, (int)gridDim.x, 0, a.N >> 4);
}

// Two formats in one launch (a Q|K|V group whose V matrix has another format than Q and K, as the Q4_K_M mixes keep
// attn_v in Q6_K): the first a.split_groups row groups take the tiles below a.t_end1 in format W1, the others the
// tiles from there on in format W2; one half chunk per wave, K slices of 8 half chunks, no epilogue.
template <class W1, class W2, int RG, int MT>
__global__ void __launch_bounds__(64 * NW, 1)
qstream_mixed_kernel(const uint8_t *__restrict__ pw0, const uint8_t *__restrict__ pw1, const uint8_t *__restrict__ pw2,
                     const half8 *__restrict__ a_tiles, const float *__restrict__ a_cscale, const float *__restrict__ a_inv_scale,
                     const float *__restrict__ a_bsum, float *__restrict__ partial, const StreamShape a) {
    __shared__ __attribute__((aligned(16))) float red[2][NW][16 * MT * (16 * RG + 4)];
    __shared__ float unused[4];
    const QkvEpi none = {};
    const int split = __builtin_amdgcn_readfirstlane(a.split_groups);
    if ((int)blockIdx.x < split)
        qstream_body<W1, 1, RG, MT, false>(pw0, pw1, pw2, a_tiles, a_cscale, a_inv_scale, a_bsum, partial, a, none, red, unused,
                                           unused, (int)blockIdx.x, split, 0, a.t_end1);
    else
        qstream_body<W2, 1, RG, MT, false>(pw0, pw1, pw2, a_tiles, a_cscale, a_inv_scale, a_bsum, partial, a, none, red, unused,
                                           unused, (int)blockIdx.x - split, (int)gridDim.x - split, a.t_end1, (a.N >> 4) - a.t_end1);
}


// ------------------------------------------------------------------------------------------------ many rows
// More than 64 activation rows (prefill chunks, tree verification) over the same packed units. The activation no
// longer fits the registers, so the roles turn: a wave owns R weight tiles (16 R rows) and keeps their sums for 64
// activation rows (R x 4 tiles of 16 x 16) in registers; the eight waves of a workgroup share the activation tiles of
// those 64 rows, which all threads bring into LDS half chunk by half chunk (double buffered, one barrier each), and
// every wave requests its R units of the next half chunk straight into registers meanwhile. Per 32-column step a
// wave reads 8 operands from LDS for 8 R MFMAs (the form with two tiles a wave reads them for 16 and is bound by LDS
// bandwidth). grid = (groups of 8 R tiles, K slices, groups of 64 rows); the sums of one K slice carry the chunk
// factor of the chunk they are in and move to the next chunk's by a ratio of two powers of two.
__device__ __forceinline__ float pow2_ratio_s(float num, float den) {
    return __uint_as_float(__float_as_uint(num) - __float_as_uint(den) + 0x3F800000u);
}

template <class W, int R>
__global__ void __launch_bounds__(64 * NW, 1)
qtiles_kernel(const uint8_t *__restrict__ pw0, const uint8_t *__restrict__ pw1, const uint8_t *__restrict__ pw2,
              const half8 *__restrict__ a_tiles, const float *__restrict__ a_cscale, const float *__restrict__ a_inv_scale,
              const float *__restrict__ a_bsum, float *__restrict__ out, const float *__restrict__ residual,
              float *__restrict__ partial, const StreamShape a, const int slices, const RowNorm fin, float *__restrict__ fin_rows) {
    constexpr int MT = 4;
    __shared__ half8 a_lds[2][4 * 512];
    typedef typename W::Ring Unit;

    const int tid = threadIdx.x, lane = tid & 63, ln = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // A side job of a launch that leaves K slices' sums (it reads no row factors itself): the activation's pending
    // 1/rms is folded into its plain row factors - finalize_row_norm_kernel's work, by up to eight workgroups of
    // the first K slice per 64 rows, a row per wave and turn - so that whoever consumes the sums reads plain
    // factors instead of adding up the chunks' sums of squares in every one of its waves.
    // Which (tile group, K slice, 64-row group) this workgroup takes. The hardware hands workgroups to the eight dies
    // in turn (linear id % 8), and each die has an L2 of its own: the ids are dealt out so that the row groups of one
    // (tile group, K slice) - which read the same weight units - run on one die, next to each other in its queue;
    // the weights then come from memory once instead of once per row group. (Whole eighths and eight row groups or
    // more only - 512-row prompt chunks: 1.6 - 2 % shorter on the 8B Q8_0 shape; with four row groups, a 256-row tree
    // step, the launch order measured 0.5 - 1.5 % faster. a.split_groups != 0, VEXEL_HIP_TILES_AS_LAUNCHED=1: as launched.)
    int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
    {
        const int X = gridDim.x, Y = gridDim.y, Z = gridDim.z, T = X * Y * Z;
        if (Z >= 8 && T % 8 == 0 && a.split_groups == 0) {
            const int L = bx + X * (by + Y * bz);
            const int S = L / 8 + (T / 8) * (L % 8);  // die-major order
            bz = S % Z;
            const int P = S / Z;
            bx = P % X;
            by = P / X;
        }
    }
    if (fin.sspart && by == 0) {
        const int nx = min((int)gridDim.x, 8);
        if (bx < nx) {
            for (int i = bx + nx * wave; i < 64; i += nx * NW) {
                const int r = bz * 64 + i;
                if (r < a.Mpad) {
                    const float f = row_factor(fin_rows, fin, r);
                    if (lane == 0) fin_rows[r] = f;
                }
            }
        }
    }
    const int n_tiles = a.N >> 4, mtiles = a.Mpad >> 4, n_hc = a.n_hc;
    const int t_own = (bx * NW + wave) * R;                  // first tile this wave writes
    const int t0 = max(min(t_own, n_tiles - R), 0);          // (a wave past the end works on the last tiles and writes nothing)
    const int ks = by, mg = bz, m0 = mg * 16 * MT;
    const int sl_base = slices >> 16, sl_rem = slices & 0xFFFF;
    const int h_begin = ks * sl_base + min(ks, sl_rem), n_half = sl_base + (ks < sl_rem ? 1 : 0);

    const size_t tile_stride = (size_t)n_hc * W::UNIT;
    const uint8_t *const w0 = uniform_ptr(pw0), *const w1 = uniform_ptr(pw1), *const w2 = uniform_ptr(pw2);
    const int e0 = __builtin_amdgcn_readfirstlane(a.t_end0), e1 = __builtin_amdgcn_readfirstlane(a.t_end1);
    const uint8_t *tb[R];
#pragma unroll
    for (int r = 0; r < R; r++) tb[r] = uniform_ptr(tile_base(t0 + r, w0, w1, w2, e0, e1, tile_stride));
    uint32_t k64;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(k64));

    // this thread's piece of a step's activation tiles: tile tid / 128 of the group (hi and lo halves, 64 lanes each);
    // a tile past the padded rows repeats the last one (its products are not stored)
    const int a_tile = min(mg * MT + tid / 128, mtiles - 1);
    const half8 *a_src = a_tiles + ((size_t)a_tile * 2) * 64 + (tid & 127);

    float4v run[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int t = 0; t < MT; t++) run[r][t] = (float4v){0.f, 0.f, 0.f, 0.f};
    if (n_half <= 0) return;

    half8 areg[4];
    // half chunk q of the slice (past the end: the last again): the wave's R units into `dst`, this thread's pieces of
    // the activation tiles into areg
    auto fetch = [&](int q, Unit (&dst)[R]) __attribute__((always_inline)) {
        const int hc = h_begin + min(q, n_half - 1);
#pragma unroll
        for (int r = 0; r < R; r++) dst[r] = W::load(tb[r] + (size_t)hc * W::UNIT, lane, ln);
#pragma unroll
        for (int sp = 0; sp < 4; sp++) areg[sp] = gload<half8>(a_src + (size_t)(hc * 4 + sp) * mtiles * 128);
    };
    auto commit = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int sp = 0; sp < 4; sp++) {
            if constexpr (W::TWO_SCALES)  // elements 0 - 15 of the step (dwords 0, 2) in front of elements 16 - 31
                a_lds[buf][sp * 512 + tid] = __builtin_shufflevector(areg[sp], areg[sp], 0, 1, 4, 5, 2, 3, 6, 7);
            else
                a_lds[buf][sp * 512 + tid] = areg[sp];
        }
    };
    auto load_cs = [&](int chunk, float4v (&cs)[MT]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const int mt = min(mg * MT + t, mtiles - 1);
            cs[t] = gload<float4v>(a_cscale + (size_t)chunk * a.Mpad + mt * 16 + 4 * g);
        }
    };

    float4v cs[MT];
    // One half chunk: the units in `cur` against the tiles in LDS buffer q & 1, while the next half chunk's units go to
    // `nxt` (two sets of registers that swap roles from one half chunk to the next, so nothing is copied).
    auto half_chunk = [&](int q, const Unit (&cur)[R], Unit (&nxt)[R]) __attribute__((always_inline)) {
        const int hc = h_begin + q;
        fetch(q + 1, nxt);
        if (q > 0 && (hc & 1) == 0) {  // a new chunk: the sums move to its activation scale
            float4v cn[MT];
            load_cs(hc >> 1, cn);
#pragma unroll
            for (int t = 0; t < MT; t++) {
                float4v f;
#pragma unroll
                for (int e = 0; e < 4; e++) f[e] = pow2_ratio_s(cs[t][e], cn[t][e]);
#pragma unroll
                for (int r = 0; r < R; r++)
#pragma unroll
                    for (int e = 0; e < 4; e++) run[r][t][e] *= f[e];
                cs[t] = cn[t];
            }
        }
        const half8 *ab = &a_lds[q & 1][0];
#pragma unroll
        for (int sp = 0; sp < 4; sp++) {
            half8 ah[MT], al[MT];
            half4v ah16[MT][2], al16[MT][2];  // (two scales a step) the operand halves of elements 0 - 15 and 16 - 31
            if constexpr (W::TWO_SCALES) {
                // (commit() has put each tile's dwords 0, 2 in front of its dwords 1, 3: the two halves of the 16 bytes
                // a lane reads are the two operands as they stand, no register copies)
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const half8 vh = ab[sp * 512 + (t * 2 + 0) * 64 + lane], vl = ab[sp * 512 + (t * 2 + 1) * 64 + lane];
                    ah16[t][0] = __builtin_shufflevector(vh, vh, 0, 1, 2, 3);
                    ah16[t][1] = __builtin_shufflevector(vh, vh, 4, 5, 6, 7);
                    al16[t][0] = __builtin_shufflevector(vl, vl, 0, 1, 2, 3);
                    al16[t][1] = __builtin_shufflevector(vl, vl, 4, 5, 6, 7);
                }
            } else {
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    ah[t] = ab[sp * 512 + (t * 2 + 0) * 64 + lane];
                    al[t] = ab[sp * 512 + (t * 2 + 1) * 64 + lane];
                }
            }
            float4v bs[MT];
            if constexpr (W::HAS_MIN) {
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const int mt = min(mg * MT + t, mtiles - 1);
                    bs[t] = gload<float4v>(a_bsum + (size_t)(hc * 4 + sp) * a.Mpad + mt * 16 + 4 * g);
                }
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                if constexpr (W::TWO_SCALES) {
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const half4v wb = W::codes16(cur[r], sp, h);
                        const float d = W::scale16(cur[r], sp, h);
                        float4v P[MT];
#pragma unroll
                        for (int t = 0; t < MT; t++)
                            P[t] = __builtin_amdgcn_mfma_f32_16x16x16f16(ah16[t][h], wb, (float4v){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                        for (int t = 0; t < MT; t++) P[t] = __builtin_amdgcn_mfma_f32_16x16x16f16(al16[t][h], wb, P[t], 0, 0, 0);
#pragma unroll
                        for (int t = 0; t < MT; t++)
#pragma unroll
                            for (int e = 0; e < 4; e++) run[r][t][e] = __builtin_fmaf(d, P[t][e], run[r][t][e]);
                    }
                } else {
                    const half8 wb = W::codes(cur[r], sp, k64);
                    const float d = W::scale(cur[r], sp);
                    float4v P[MT];
#pragma unroll
                    for (int t = 0; t < MT; t++) P[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah[t], wb, (float4v){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                    for (int t = 0; t < MT; t++) P[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al[t], wb, P[t], 0, 0, 0);
#pragma unroll
                    for (int t = 0; t < MT; t++)
#pragma unroll
                        for (int e = 0; e < 4; e++) run[r][t][e] = __builtin_fmaf(d, P[t][e], run[r][t][e]);
                    if constexpr (W::HAS_MIN) {
                        const float mn = -W::minimum(cur[r], sp);
#pragma unroll
                        for (int t = 0; t < MT; t++)
#pragma unroll
                            for (int e = 0; e < 4; e++) run[r][t][e] = __builtin_fmaf(mn, bs[t][e], run[r][t][e]);
                    }
                }
            }
        }
        // the next half chunk's activation tiles into the buffer every wave finished with before the previous barrier
        commit((q + 1) & 1);
        __syncthreads();
    };
    Unit ua[R], ub[R];
    fetch(0, ua);
    load_cs(h_begin >> 1, cs);
    commit(0);
    __syncthreads();
    if constexpr (W::HAS_MIN) {
        // (with the block sums' loads in the step the twice-unrolled loop runs out of registers: one set, copied)
        for (int q = 0; q < n_half; q++) {
#pragma unroll
            for (int r = 0; r < R; r++) ub[r] = ua[r];
            half_chunk(q, ub, ua);
        }
    } else {
        for (int q = 0; q < n_half; q += 2) {
            half_chunk(q, ua, ub);
            if (q + 1 < n_half) half_chunk(q + 1, ub, ua);
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int e = 0; e < 4; e++) run[r][t][e] *= cs[t][e];

    // lane (g, ln) of tile (r, t) holds C[m0 + 16 t + 4 g + e][16 (t0 + r) + ln]
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int m = m0 + 16 * t + 4 * g + e;
            if (m >= a.M) continue;
            const float inv = partial ? 1.f : a_inv_scale[m];
#pragma unroll
            for (int r = 0; r < R; r++) {
                if (t0 + r < t_own) continue;
                const int n = 16 * (t0 + r) + ln;
                if (partial) {
                    partial[((size_t)ks * a.M + m) * a.N + n] = run[r][t][e];
                } else {
                    float v = __fmul_rn(run[r][t][e], inv);
                    if (residual) v = __fadd_rn(residual[(size_t)m * a.N + n], v);
                    out[(size_t)m * a.N + n] = v;
                }
            }
        }
}

bool has_min(int fmt) { return fmt == VX_Q4_K || fmt == VX_Q5_K; }
struct TilesPlan {
    int r, s;  // weight tiles a wave, K slices; r == 0: not served
};
// Weight tiles a wave (at most what the format's units leave of the registers: four tiles are 64 more accumulators
// than there are; Q6_K's units and the block sums of the formats with a min term leave room for two) and K slices,
// chosen together by a small cost model in units of about a microsecond: rounds of workgroups over the device x (a
// half chunk's time, which grows with the tiles a wave owns, x half chunks per slice + a fixed part) + the round trip
// of the slices' sums. Depends on the format, the matrix' shape and the number of 64-row groups only.
TilesPlan tiles_plan(int fmt, int n_tiles, int n_hc, int mgroups, int cus) {
    TilesPlan pl = {0, 1};
    const int rmax = (fmt == VX_Q6_K || has_min(fmt)) ? 2 : 3;
    // a tile's time per half chunk relative to Q4_0's: Q6_K issues twice the MFMAs and scale FMAs, a min term adds FMAs
    const float unit = fmt == VX_Q6_K ? 1.9f : (has_min(fmt) ? 1.3f : 1.f);
    float best_cost = 1e30f;
    for (int r = std::min(rmax, n_tiles); r >= 1; r--) {
        const int base = ceil_div(n_tiles, NW * r) * mgroups;
        for (int s = 1; s <= std::min(16, std::max(1, n_hc / 2)); s++) {
            const int rounds = ceil_div(base * s, cus);
            const float sums = s > 1 ? (float)s * 64.f * (float)mgroups * 16.f * (float)n_tiles * 1.0e-6f : 0.f;
            const float cost = (float)rounds * (((float)r * unit + 0.4f) * (float)ceil_div(n_hc, s) + 4.f) + sums;
            if (cost < best_cost) {
                best_cost = cost;
                pl.r = r;
                pl.s = s;
            }
        }
    }
    return pl;
}

struct StreamPlan {
    int g, s, ph, npass;  // row groups, K slices, half chunks per wave and pass, passes; g == 0: not served
};

// The cut of an [n_tiles * 16, n_hc * 128] matrix for a device of `cus` compute units; max_ph: how many half chunks'
// operands a wave's registers hold (2; 1 at four activation tiles). With the epilogue the whole
// K stays in one workgroup (passes of 16 half chunks); otherwise K is sliced so that a slice is one pass, and
// further while a workgroup would own fewer than four tiles and slices stay at least four half chunks wide: every
// workgroup first pulls its slice of the activation (128 bytes per column) through its compute unit's L1, which
// costs as much as the weights of a few tiles. VEXEL_HIP_SPLAN="NxK:G,S;..." overrides the choice (tuning).
StreamPlan stream_plan(int n_tiles, int n_hc, int cus, bool epi, int N, int K, int max_ph) {
    StreamPlan pl = {0, 1, 1, 1};
    if (n_tiles < 1 || n_hc < 1 || (epi && max_ph < 2)) return pl;
    static const char *env = getenv("VEXEL_HIP_SPLAN");
    const int cap = NW * max_ph;  // half chunks a workgroup's registers hold
    int s = epi ? 1 : ceil_div(n_hc, cap), g = 0;
    if (!epi) {
        while (true) {
            const int gg = std::max(1, std::min(cus / s, n_tiles));
            const int nh = ceil_div(n_hc, s);
            if (n_tiles / gg >= 4 || nh < 8 || s * 2 > cus) break;
            s *= 2;
        }
    }
    g = std::max(1, std::min(cus / s, n_tiles));
    if (env && !epi) {
        char key[64];
        snprintf(key, sizeof key, "%dx%d:", N, K);
        const char *p = strstr(env, key);
        int eg = 0, es = 0;
        if (p && sscanf(p + strlen(key), "%d,%d", &eg, &es) == 2 && eg >= 1 && es >= 1 && es <= n_hc && eg <= n_tiles &&
            ceil_div(n_hc, es) <= cap) {
            g = eg;
            s = es;
        }
    }
    const int nh = ceil_div(n_hc, s);
    pl.g = g;
    pl.s = s;
    pl.ph = nh > 8 ? 2 : 1;
    pl.npass = ceil_div(nh, 8 * pl.ph);
    if (!epi && pl.npass != 1) pl.g = 0;
    if (epi && pl.npass > 1 && ceil_div(n_tiles, g) > ACC_TILES) pl.g = 0;
    return pl;
}

struct PackedW {
    void *data;
    int fmt, n, k;
    size_t bytes;  // of the raw matrix (what a write into it is checked against)
};

bool packable(int fmt) { return fmt == VX_Q4_0 || fmt == VX_Q8_0 || fmt == VX_Q6_K || fmt == VX_Q4_K || fmt == VX_Q5_0 || fmt == VX_Q5_K; }
size_t raw_row_bytes(int fmt, int K) {
    switch (fmt) {
    case VX_Q4_0: return (size_t)K / 32 * 18;
    case VX_Q8_0: return (size_t)K / 32 * 34;
    case VX_Q4_K: return (size_t)K / 256 * 144;
    case VX_Q5_0: return (size_t)K / 32 * 22;
    case VX_Q5_K: return (size_t)K / 256 * 176;
    default: return (size_t)K / 256 * 210;
    }
}
int unit_bytes(int fmt) {
    switch (fmt) {
    case VX_Q4_0: return SQ4_0::UNIT;
    case VX_Q8_0: return SQ8_0::UNIT;
    case VX_Q5_0: return SQ8_0::UNIT;
    case VX_Q4_K: return SQ4_K::UNIT;
    case VX_Q5_K: return SQ5_K::UNIT;
    default: return SQ6_K::UNIT;
    }
}
// half chunks whose operands a wave's registers hold beside the format's requests in flight
int max_ph_of(int fmt, int M) { return (M > 32 || fmt == VX_Q6_K || fmt == VX_Q4_K || fmt == VX_Q5_K) ? 1 : 2; }

}  // namespace

namespace vx {

// Registry of packed copies, keyed by the raw matrix' device address (the backend's map stores them type-erased).
static PackedW *find_packed(vx_backend *be, const void *raw) {
    auto it = be->packed.find(raw);
    return it == be->packed.end() ? nullptr : (PackedW *)it->second;
}

void stream_drop_packed(vx_backend *be, const void *raw) {
    auto it = be->packed.find(raw);
    if (it == be->packed.end()) return;
    PackedW *pw = (PackedW *)it->second;
    (void)hipFree(pw->data);
    delete pw;
    be->packed.erase(it);
    be->scratch_gen++;  // a recorded graph may hold the copy's address
}

void stream_written(vx_backend *be, const void *dst, size_t bytes) {
    const char *a = (const char *)dst;
    std::vector<const void *> stale;
    for (auto &kv : be->packed) {
        const PackedW *pw = (const PackedW *)kv.second;
        const char *r = (const char *)kv.first;
        if (a < r + pw->bytes && r < a + bytes) stale.push_back(kv.first);
    }
    if (stale.empty()) return;
    (void)hipStreamSynchronize(be->stream);  // a launch may still read the copies
    for (const void *r : stale) stream_drop_packed(be, r);
}

void stream_drop_all(vx_backend *be) {
    while (!be->packed.empty()) stream_drop_packed(be, be->packed.begin()->first);
}

// Resolves up to three row segments of raw matrices (each a run of registered matrices laid end to end) into packed
// matrices; false when any part has no packed copy.
static bool resolve(vx_backend *be, int fmt, const uint8_t *const *w, const int *n_end, int nseg, int N, int K, PackedSegs *out) {
    if (!packable(fmt) || be->packed.empty()) return false;
    const size_t row_bytes = raw_row_bytes(fmt, K);
    int np = 0, rows_done = 0;
    for (int i = 0; i < nseg && rows_done < N; i++) {
        const int seg_rows = n_end[i] - rows_done;
        if (seg_rows <= 0) continue;
        const uint8_t *p = w[i];
        int left = seg_rows;
        while (left > 0) {
            PackedW *pw = find_packed(be, p);
            if (!pw || pw->fmt != fmt || pw->k != K || pw->n > left || np == 3) return false;
            out->w[np] = (const uint8_t *)pw->data;
            out->t_end[np] = (rows_done + pw->n) / 16;
            np++;
            rows_done += pw->n;
            left -= pw->n;
            p += (size_t)pw->n * row_bytes;
        }
    }
    if (rows_done != N || np == 0) return false;
    for (int i = np; i < 3; i++) {
        out->w[i] = out->w[np - 1];
        out->t_end[i] = N / 16;
    }
    return true;
}

bool stream_gemm_ok(vx_backend *be, int fmt, const uint8_t *const *w, const int *n_end, int nseg, int N, int K, int M, bool epi) {
    static const char *off = getenv("VEXEL_HIP_STREAM_OFF");
    if (off && atoi(off)) return false;
    if (M < 2 || M > 64 || N % 16 != 0 || K % 256 != 0 || N < 16) return false;
    if (epi && M > 32) return false;
    if (has_min(fmt) && M > 32) return false;  // the block sums of four activation tiles do not fit the registers
    // With the epilogue the whole K stays in one workgroup, which walks it in passes of 16 half chunks; every pass
    // starts its requests anew, and for two passes and more the launch takes longer than the wave-private kernel's
    // (7B Q|K|V, 32 rows: 23.8 against 20.9 us). VEXEL_HIP_STREAM_EPI=1 takes it anyway (measurements).
    static const bool epi_any = getenv("VEXEL_HIP_STREAM_EPI") != nullptr;
    if (epi && K / 128 > 16 && !epi_any) return false;
    PackedSegs ps;
    if (!resolve(be, fmt, w, n_end, nseg, N, K, &ps)) return false;
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, be->device) != hipSuccess || cus <= 0) cus = 256;
    return stream_plan(N / 16, K / 128, cus, epi, N, K, max_ph_of(fmt, M)).g > 0;
}

template <class W>
static void launch_stream(vx_backend *be, const StreamPlan &pl, dim3 grid, int mt, bool fin, const PackedSegs &ps, const PrepView &pv,
                          float *partial, const StreamShape &a, const QkvEpi &e) {
#define VX_STREAM_LAUNCH(PH_, RG_, MT_, EPI_)                                                                                  \
    qstream_kernel<W, PH_, RG_, MT_, EPI_><<<grid, 64 * NW, 0, be->stream>>>(ps.w[0], ps.w[1], ps.w[2], pv.tiles, pv.cscale, pv.inv_scale, \
                                                                              pv.bsum, partial, a, e)
    if (mt == 4) {
        if constexpr (!W::HAS_MIN) VX_STREAM_LAUNCH(1, 2, 4, false);  // (refused by stream_gemm_ok for a format with a min term)
    } else if constexpr (W::TWO_SCALES || W::HAS_MIN) {
        if (mt == 2) VX_STREAM_LAUNCH(1, 4, 2, false);
        else VX_STREAM_LAUNCH(1, 4, 1, false);
    } else if (fin) {
        if (pl.ph == 2) {
            if (mt == 2) VX_STREAM_LAUNCH(2, 2, 2, true);
            else VX_STREAM_LAUNCH(2, 2, 1, true);
        } else {
            if (mt == 2) VX_STREAM_LAUNCH(1, 2, 2, true);
            else VX_STREAM_LAUNCH(1, 2, 1, true);
        }
    } else if (pl.ph == 2) {
        if (mt == 2) VX_STREAM_LAUNCH(2, 2, 2, false);
        else VX_STREAM_LAUNCH(2, 2, 1, false);
    } else {
        if (mt == 2) VX_STREAM_LAUNCH(1, 4, 2, false);
        else VX_STREAM_LAUNCH(1, 4, 1, false);
    }
#undef VX_STREAM_LAUNCH
}

// Launches the streaming kernel; the K slices' sums go to be->part_ws as [slice][M][N] (raw: no row factors), or, with
// an epilogue, the finished rows to where it says. *ks_out: the number of slices.
int stream_gemm(vx_backend *be, int fmt, const uint8_t *const *w, const int *n_end, int nseg, int N, int K, int M, int mpad,
                const PrepView &pv, const QkvEpi *epi, int *ks_out) {
    PackedSegs ps;
    if (!resolve(be, fmt, w, n_end, nseg, N, K, &ps)) return VX_ERR_UNSUPPORTED;
    static int cus = 0;
    if (cus == 0 && (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, be->device) != hipSuccess || cus <= 0)) cus = 256;
    const bool fin = epi && epi->q_out;
    const int mt = mpad / 16;
    if (mt != 1 && mt != 2 && mt != 4) return VX_ERR_UNSUPPORTED;
    const int max_ph = max_ph_of(fmt, M);
    const StreamPlan pl = stream_plan(N / 16, K / 128, cus, fin, N, K, max_ph);
    if (pl.g == 0 || (max_ph == 1 && (fin || pl.ph != 1)) || (has_min(fmt) && mt == 4)) return VX_ERR_UNSUPPORTED;
    StreamShape a;
    a.M = M;
    a.Mpad = mpad;
    a.N = N;
    a.n_hc = K / 128;
    a.npass = pl.npass;
    a.t_end0 = ps.t_end[0];
    a.t_end1 = ps.t_end[1];
    a.split_groups = 0;
    const QkvEpi e = fin ? *epi : QkvEpi{};
    float *partial = nullptr;
    if (!fin) {
        int rc = ensure_ws(be, &be->part_ws, &be->part_ws_bytes, (size_t)pl.s * M * N * sizeof(float), "split-K partial sums");
        if (rc) return rc;
        partial = (float *)be->part_ws;
    }
    dim3 grid(pl.g, pl.s);
    if (fmt == VX_Q4_0) launch_stream<SQ4_0>(be, pl, grid, mt, fin, ps, pv, partial, a, e);
    else if (fmt == VX_Q8_0 || fmt == VX_Q5_0) launch_stream<SQ8_0>(be, pl, grid, mt, fin, ps, pv, partial, a, e);
    else if (fmt == VX_Q4_K) launch_stream<SQ4_K>(be, pl, grid, mt, fin, ps, pv, partial, a, e);
    else if (fmt == VX_Q5_K) launch_stream<SQ5_K>(be, pl, grid, mt, fin, ps, pv, partial, a, e);
    else launch_stream<SQ6_K>(be, pl, grid, mt, fin, ps, pv, partial, a, e);
    VX_CHECK_LAUNCH();
    if (ks_out) *ks_out = pl.s;
    return VX_OK;
}


// ---- a Q|K|V group whose V matrix has another format: one launch over both
// Q and K (format fa, rows na) and V (format fb, rows nb) with packed copies; 2 .. 32 rows (the formats with a min term
// hold no more), K in slices of 8 half chunks, the row groups shared out by what a tile of each format costs.
static bool mixed_resolve(vx_backend *be, int fa, const uint8_t *wq, const uint8_t *wk, int nq, int nk, int fb, const uint8_t *wv,
                          int nv, int K, PackedSegs *out) {
    PackedW *pq = find_packed(be, wq), *pk = find_packed(be, wk), *pv = find_packed(be, wv);
    if (!pq || !pk || !pv || pq->fmt != fa || pk->fmt != fa || pv->fmt != fb) return false;
    if (pq->k != K || pk->k != K || pv->k != K || pq->n != nq || pk->n != nk || pv->n != nv) return false;
    out->w[0] = (const uint8_t *)pq->data;
    out->w[1] = (const uint8_t *)pk->data;
    out->w[2] = (const uint8_t *)pv->data;
    out->t_end[0] = nq / 16;
    out->t_end[1] = (nq + nk) / 16;
    out->t_end[2] = (nq + nk + nv) / 16;
    return true;
}

// The row groups of a two-format launch and how many of them the first format takes. A group works in rounds of four
// tiles (a started round costs a whole one), and a round costs what its format's tiles cost (relative to Q4_0's: the
// many-rows kernel's plan uses the same figures): the split with the shortest longer side, then the least work.
static bool mixed_plan(vx_backend *be, int ta, int tb, int slices, int *groups_out, int *ga_out) {
    static int cus = 0;
    if (cus == 0 && (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, be->device) != hipSuccess || cus <= 0)) cus = 256;
    const int groups = std::max(2, std::min(cus / slices, ta + tb));
    auto rounds = [](int tiles, int g) { return (ceil_div(tiles, g) + 3) / 4; };
    float best = 0.f, best_sum = 0.f;
    int best_ga = 0;
    for (int ga = 1; ga < groups; ga++) {
        const int gb = groups - ga;
        if (ga > ta || gb > tb) continue;  // (no group without a tile)
        const float ra = 1.3f * (float)rounds(ta, ga), rb = 1.9f * (float)rounds(tb, gb);
        const float longer = std::max(ra, rb), sum = ra * (float)ga + rb * (float)gb;
        if (best_ga == 0 || longer < best || (longer == best && sum < best_sum)) {
            best = longer;
            best_sum = sum;
            best_ga = ga;
        }
    }
    if (best_ga == 0) return false;
    *groups_out = groups;
    *ga_out = best_ga;
    return true;
}

bool stream_gemm_mixed_ok(vx_backend *be, int fa, const uint8_t *wq, const uint8_t *wk, int nq, int nk, int fb, const uint8_t *wv,
                          int nv, int K, int M) {
    static const char *off = getenv("VEXEL_HIP_STREAM_OFF");
    if (off && atoi(off)) return false;
    static const bool mixed_off = getenv("VEXEL_HIP_MIXED_OFF") != nullptr;  // (measurements: V in a launch of its own)
    if (mixed_off) return false;
    if (!((fa == VX_Q4_K || fa == VX_Q5_K) && fb == VX_Q6_K)) return false;  // (the pairs the K-quant mixes hold)
    if (M < 2 || M > 32 || K % 1024 != 0 || nq % 16 || nk % 16 || nv % 16 || nq < 16 || nk < 16 || nv < 16) return false;
    if (be->packed.empty()) return false;
    PackedSegs ps;
    int groups, ga;
    return mixed_resolve(be, fa, wq, wk, nq, nk, fb, wv, nv, K, &ps) && mixed_plan(be, (nq + nk) / 16, nv / 16, K / 128 / NW, &groups, &ga);
}

int stream_gemm_mixed(vx_backend *be, int fa, const uint8_t *wq, const uint8_t *wk, int nq, int nk, int fb, const uint8_t *wv, int nv,
                      int K, int M, int mpad, const PrepView &pv, int *ks_out) {
    PackedSegs ps;
    if (!mixed_resolve(be, fa, wq, wk, nq, nk, fb, wv, nv, K, &ps)) return VX_ERR_UNSUPPORTED;
    const int N = nq + nk + nv, n_hc = K / 128, slices = n_hc / NW, mt = mpad / 16;
    if (mt != 1 && mt != 2) return VX_ERR_UNSUPPORTED;
    int groups, ga;
    if (!mixed_plan(be, (nq + nk) / 16, nv / 16, slices, &groups, &ga)) return VX_ERR_UNSUPPORTED;
    StreamShape a;
    a.M = M;
    a.Mpad = mpad;
    a.N = N;
    a.n_hc = n_hc;
    a.npass = 1;
    a.t_end0 = ps.t_end[0];
    a.t_end1 = ps.t_end[1];
    a.split_groups = ga;
    int rc = ensure_ws(be, &be->part_ws, &be->part_ws_bytes, (size_t)slices * M * N * sizeof(float), "split-K partial sums");
    if (rc) return rc;
    float *partial = (float *)be->part_ws;
    dim3 grid(groups, slices);
#define VX_MIXED_LAUNCH(W1_, MT_)                                                                                              \
    qstream_mixed_kernel<W1_, SQ6_K, 4, MT_><<<grid, 64 * NW, 0, be->stream>>>(ps.w[0], ps.w[1], ps.w[2], pv.tiles, pv.cscale,    \
                                                                                pv.inv_scale, pv.bsum, partial, a)
    if (fa == VX_Q4_K) {
        if (mt == 2) VX_MIXED_LAUNCH(SQ4_K, 2);
        else VX_MIXED_LAUNCH(SQ4_K, 1);
    } else {
        if (mt == 2) VX_MIXED_LAUNCH(SQ5_K, 2);
        else VX_MIXED_LAUNCH(SQ5_K, 1);
    }
#undef VX_MIXED_LAUNCH
    VX_CHECK_LAUNCH();
    if (ks_out) *ks_out = slices;
    return VX_OK;
}

bool tiles_gemm_ok(vx_backend *be, int fmt, const uint8_t *const *w, const int *n_end, int nseg, int N, int K, int M) {
    static const char *off = getenv("VEXEL_HIP_TILES_OFF");
    if (off && atoi(off)) return false;
    if (M <= 64 || N % 16 != 0 || K % 256 != 0 || N < 16) return false;
    PackedSegs ps;
    return resolve(be, fmt, w, n_end, nseg, N, K, &ps);
}

template <class W>
static void launch_tiles(vx_backend *be, const TilesPlan &pl, dim3 grid, const PackedSegs &ps, const PrepView &pv, float *out,
                         const float *residual, float *partial, const StreamShape &a, int slices, const RowNorm &fin) {
#define VX_TILES_LAUNCH(R_)                                                                                                    \
    qtiles_kernel<W, R_><<<grid, 64 * NW, 0, be->stream>>>(ps.w[0], ps.w[1], ps.w[2], pv.tiles, pv.cscale, pv.inv_scale, pv.bsum, out, \
                                                           residual, partial, a, slices, fin, pv.inv_scale)
    if (pl.r == 3) {
        if constexpr (!W::TWO_SCALES && !W::HAS_MIN) VX_TILES_LAUNCH(3);
    } else if (pl.r == 2) {
        VX_TILES_LAUNCH(2);
    } else {
        VX_TILES_LAUNCH(1);
    }
#undef VX_TILES_LAUNCH
}

// More than 64 rows over packed matrices. One K slice and no request for the slices' sums: the finished rows go to
// out (row factors and the residual applied); otherwise [slice][M][N] sums go to be->part_ws and *ks_out says how many.
int tiles_gemm(vx_backend *be, int fmt, const uint8_t *const *w, const int *n_end, int nseg, int N, int K, int M, int mpad,
               const PrepView &pv, float *out, const float *residual, bool to_partials, int *ks_out, const RowNorm *fin_norm) {
    PackedSegs ps;
    if (!resolve(be, fmt, w, n_end, nseg, N, K, &ps)) return VX_ERR_UNSUPPORTED;
    // (a pending 1/rms is folded in by the launch only where the launch itself reads no row factors)
    if (fin_norm && !to_partials) return VX_ERR_UNSUPPORTED;
    const RowNorm fin = fin_norm ? *fin_norm : RowNorm{nullptr, 0, 0.f, 0.f};
    static int cus = 0;
    if (cus == 0 && (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, be->device) != hipSuccess || cus <= 0)) cus = 256;
    const int n_hc = K / 128, mgroups = ceil_div(mpad, 64);
    TilesPlan pl = tiles_plan(fmt, N / 16, n_hc, mgroups, cus);
    if (const char *env = getenv("VEXEL_HIP_TPLAN")) {  // "r,s" for every shape (tuning)
        int r = 0, s2 = 0;
        const int rmax = (fmt == VX_Q6_K || has_min(fmt)) ? 2 : 3;
        if (sscanf(env, "%d,%d", &r, &s2) == 2 && r >= 1 && r <= rmax && s2 >= 1 && s2 <= std::max(1, n_hc / 2)) pl = {r, s2};
    }
    if (pl.r == 0) return VX_ERR_UNSUPPORTED;
    StreamShape a;
    a.M = M;
    a.Mpad = mpad;
    a.N = N;
    a.n_hc = n_hc;
    a.npass = 1;
    a.t_end0 = ps.t_end[0];
    a.t_end1 = ps.t_end[1];
    static const bool as_launched = getenv("VEXEL_HIP_TILES_AS_LAUNCHED") != nullptr;  // (measurements: no dealing out by die)
    a.split_groups = as_launched ? 1 : 0;
    float *partial = nullptr;
    if (pl.s > 1 || to_partials) {
        int rc = ensure_ws(be, &be->part_ws, &be->part_ws_bytes, (size_t)pl.s * M * N * sizeof(float), "split-K partial sums");
        if (rc) return rc;
        partial = (float *)be->part_ws;
    }
    const int slices = ((n_hc / pl.s) << 16) | (n_hc % pl.s);
    dim3 grid(ceil_div(N / 16, NW * pl.r), pl.s, mgroups);
    switch (fmt) {
    case VX_Q4_0: launch_tiles<SQ4_0>(be, pl, grid, ps, pv, out, residual, partial, a, slices, fin); break;
    case VX_Q8_0:
    case VX_Q5_0: launch_tiles<SQ8_0>(be, pl, grid, ps, pv, out, residual, partial, a, slices, fin); break;
    case VX_Q5_K: launch_tiles<SQ5_K>(be, pl, grid, ps, pv, out, residual, partial, a, slices, fin); break;
    case VX_Q4_K: launch_tiles<SQ4_K>(be, pl, grid, ps, pv, out, residual, partial, a, slices, fin); break;
    default: launch_tiles<SQ6_K>(be, pl, grid, ps, pv, out, residual, partial, a, slices, fin); break;
    }
    VX_CHECK_LAUNCH();
    if (ks_out) *ks_out = pl.s;
    return VX_OK;
}

}  // namespace vx

extern "C" {

int vx_qweight_pack(vx_backend *be, const vx_qweight *w) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(w && w->data, "vx_qweight_pack: null weight");
    VX_REQUIRE(!be->capturing, "vx_qweight_pack during graph capture");
    if (!packable(w->fmt) || w->n < 16 || w->n % 16 != 0 || w->k < 256 || w->k % 256 != 0) return VX_ERR_UNSUPPORTED;
    if (find_packed(be, w->data)) stream_drop_packed(be, w->data);
    const size_t bytes = (size_t)(w->n / 16) * (w->k / 128) * unit_bytes(w->fmt);
    PackedW *pw = new PackedW{nullptr, w->fmt, w->n, w->k, (size_t)w->n * raw_row_bytes(w->fmt, w->k)};
    if (hipMalloc(&pw->data, bytes) != hipSuccess) {
        delete pw;
        set_error("vx_qweight_pack: out of device memory (%zu bytes)", bytes);
        return VX_ERR_OOM;
    }
    if (w->fmt == VX_Q4_0)
        pack_q4_0_kernel<<<dim3(w->n / 16, w->k / 128), 64, 0, be->stream>>>((const uint8_t *)w->data, (uint8_t *)pw->data, w->k / 128);
    else if (w->fmt == VX_Q8_0)
        pack_q8_0_kernel<<<dim3(w->n / 16, w->k / 128), 64, 0, be->stream>>>((const uint8_t *)w->data, (uint8_t *)pw->data, w->k / 128);
    else if (w->fmt == VX_Q5_0)
        pack_q5_0_kernel<<<dim3(w->n / 16, w->k / 128), 64, 0, be->stream>>>((const uint8_t *)w->data, (uint8_t *)pw->data, w->k / 128);
    else if (w->fmt == VX_Q5_K)
        pack_q5_k_kernel<<<dim3(w->n / 16, w->k / 128), 64, 0, be->stream>>>((const uint8_t *)w->data, (uint8_t *)pw->data, w->k / 128);
    else if (w->fmt == VX_Q4_K)
        pack_q4_k_kernel<<<dim3(w->n / 16, w->k / 128), 64, 0, be->stream>>>((const uint8_t *)w->data, (uint8_t *)pw->data, w->k / 128);
    else
        pack_q6_k_kernel<<<dim3(w->n / 16, w->k / 128), 64, 0, be->stream>>>((const uint8_t *)w->data, (uint8_t *)pw->data, w->k / 128);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        (void)hipFree(pw->data);
        delete pw;
        set_error("vx_qweight_pack: launch failed: %s", hipGetErrorString(e));
        return VX_ERR_HIP;
    }
    be->packed[w->data] = pw;
    be->scratch_gen++;  // a graph recorded before streams the GGUF rows: the holder records again
    return VX_OK;
}

int vx_qweight_unpack(vx_backend *be, const vx_qweight *w) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(w && w->data, "vx_qweight_unpack: null weight");
    VX_CHECK_HIP(hipStreamSynchronize(be->stream));  // a launch may still read the copy
    stream_drop_packed(be, w->data);
    return VX_OK;
}

int vx_qweight_is_packed(vx_backend *be, const vx_qweight *w) {
    if (!be || !w || !w->data) return 0;
    PackedW *pw = find_packed(be, w->data);
    return pw && pw->fmt == w->fmt && pw->n == w->n && pw->k == w->k ? 1 : 0;
}

int vx_dequantize_packed(vx_backend *be, const vx_qweight *w, float *dst) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(w && w->data && dst, "vx_dequantize_packed: null pointer");
    PackedW *pw = find_packed(be, w->data);
    VX_REQUIRE(pw && pw->fmt == w->fmt && pw->n == w->n && pw->k == w->k, "vx_dequantize_packed: the matrix has no packed copy");
    const size_t total = (size_t)w->n * w->k;
    if (pw->fmt == VX_Q4_0)
        dequant_packed_q4_0_kernel<<<(unsigned)((total + 255) / 256), 256, 0, be->stream>>>((const uint8_t *)pw->data, dst, w->n, w->k);
    else if (pw->fmt == VX_Q5_K)
        dequant_packed_q5_k_kernel<<<(unsigned)((total + 255) / 256), 256, 0, be->stream>>>((const uint8_t *)pw->data, dst, w->n, w->k);
    else if (pw->fmt == VX_Q8_0 || pw->fmt == VX_Q5_0)
        dequant_packed_q8_0_kernel<<<(unsigned)((total + 255) / 256), 256, 0, be->stream>>>((const uint8_t *)pw->data, dst, w->n, w->k);
    else if (pw->fmt == VX_Q4_K)
        dequant_packed_q4_k_kernel<<<(unsigned)((total + 255) / 256), 256, 0, be->stream>>>((const uint8_t *)pw->data, dst, w->n, w->k);
    else
        dequant_packed_q6_k_kernel<<<(unsigned)((total + 255) / 256), 256, 0, be->stream>>>((const uint8_t *)pw->data, dst, w->n, w->k);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

}  // extern "C"
