// Benchmark support, not part of the backend's C ABI: fills device buffers with synthetic
// data of the shapes the benchmark configs name, without any host round trip:
//   vxs_gaussian_quant  N(0,std) values quantized to Q4_0 / Q8_0 blocks (llama.cpp convention:
//                       Q4_0 d = signed absmax / -8, q = min(15, floor(x/d + 8.5));
//                       Q8_0 d = absmax / 127, q = round(x/d))
//   vxs_gaussian_f16    N(0,std) halves (pre-filled KV cache contents)
// Values come from a counter-based generator (splitmix64 of seed and element index, Box-Muller),
// so a buffer's contents depend only on (seed, index), not on the launch shape.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// two independent standard normals for pair index i
__device__ __forceinline__ float2 normal_pair(uint64_t seed, uint64_t i) {
    uint64_t r = splitmix64(seed ^ splitmix64(i));
    float u1 = ((uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777217.0f);  // (0,1]
    float u2 = (uint32_t)((r >> 8) & 0xFFFFFF) * (1.0f / 16777216.0f);
    float rad = sqrtf(-2.0f * logf(u1));
    float s, c;
    sincosf(6.283185307179586f * u2, &s, &c);
    return make_float2(rad * c, rad * s);
}

// one thread per super-block: random bytes, then f16 headers of about 2^-10 at byte offsets h0 / h1 (h1 < 0: none)
__global__ void random_kquant_kernel(uint8_t *dst, int64_t nblocks, int block_bytes, int h0, int h1, uint64_t seed) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    uint8_t *o = dst + b * block_bytes;
    for (int i = 0; i < block_bytes; i += 2) {  // block sizes are even
        const uint64_t r = splitmix64(seed ^ splitmix64((uint64_t)b * 128 + i / 2));
        o[i] = (uint8_t)r;
        o[i + 1] = (uint8_t)(r >> 8);
    }
    const uint64_t r = splitmix64(seed + 0x5bd1e995ull * (uint64_t)b);
    o[h0] = (uint8_t)r;
    o[h0 + 1] = 0x14;  // 2^-10 * (1 + mantissa)
    if (h1 >= 0) {
        o[h1] = (uint8_t)(r >> 8);
        o[h1 + 1] = 0x10;
    }
}

__global__ void gaussian_q4_0_kernel(uint8_t *dst, int64_t nblocks, float stdv, uint64_t seed) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    float x[32];
    float amax = 0.f, mx = 0.f;
    for (int i = 0; i < 16; i++) {
        float2 p = normal_pair(seed, (uint64_t)b * 16 + i);
        x[2 * i] = p.x * stdv;
        x[2 * i + 1] = p.y * stdv;
    }
    for (int i = 0; i < 32; i++)
        if (fabsf(x[i]) > amax) {
            amax = fabsf(x[i]);
            mx = x[i];
        }
    float d = mx / -8.0f;
    float id = d != 0.f ? 1.0f / d : 0.f;
    uint8_t *o = dst + b * 18;
    _Float16 dh = (_Float16)d;
    uint16_t bits;
    __builtin_memcpy(&bits, &dh, 2);
    o[0] = (uint8_t)(bits & 0xFF);
    o[1] = (uint8_t)(bits >> 8);
    for (int i = 0; i < 16; i++) {
        int q0 = (int)fminf(15.f, floorf(x[i] * id + 8.5f));
        int q1 = (int)fminf(15.f, floorf(x[i + 16] * id + 8.5f));
        q0 = q0 < 0 ? 0 : q0;
        q1 = q1 < 0 ? 0 : q1;
        o[2 + i] = (uint8_t)(q0 | (q1 << 4));
    }
}

__global__ void gaussian_q8_0_kernel(uint8_t *dst, int64_t nblocks, float stdv, uint64_t seed) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    float x[32];
    float amax = 0.f;
    for (int i = 0; i < 16; i++) {
        float2 p = normal_pair(seed, (uint64_t)b * 16 + i);
        x[2 * i] = p.x * stdv;
        x[2 * i + 1] = p.y * stdv;
    }
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(x[i]));
    float d = amax / 127.0f;
    float id = d != 0.f ? 1.0f / d : 0.f;
    uint8_t *o = dst + b * 34;
    _Float16 dh = (_Float16)d;
    uint16_t bits;
    __builtin_memcpy(&bits, &dh, 2);
    o[0] = (uint8_t)(bits & 0xFF);
    o[1] = (uint8_t)(bits >> 8);
    for (int i = 0; i < 32; i++) {
        int q = (int)rintf(x[i] * id);
        q = q < -127 ? -127 : (q > 127 ? 127 : q);
        o[2 + i] = (uint8_t)(int8_t)q;
    }
}

__global__ void gaussian_f16_kernel(_Float16 *dst, int64_t npairs, float stdv, uint64_t seed) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= npairs) return;
    float2 p = normal_pair(seed, (uint64_t)i);
    dst[2 * i] = (_Float16)(p.x * stdv);
    dst[2 * i + 1] = (_Float16)(p.y * stdv);
}

}  // namespace

// Plain 16-byte-per-lane copy: a kernel of known traffic (bytes read = bytes written = n16*16) against
// which hardware counters are calibrated.
__global__ void plain_copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, int64_t n16) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}

extern "C" {

// Copies `bytes` (a multiple of 16) with plain_copy_kernel. Returns 0 or a hipError_t value.
int vxs_plain_copy(void *dst, const void *src, int64_t bytes) {
    const int64_t n16 = bytes / 16;
    if (n16 <= 0) return 0;
    plain_copy_kernel<<<(unsigned)((n16 + 255) / 256), 256>>>((const uint4 *)src, (uint4 *)dst, n16);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return (int)hipDeviceSynchronize();
}

// fmt: 3 = Q4_K (144-byte super-blocks), 4 = Q6_K (210-byte): uniformly random codes and sub-block scales
// under small finite f16 super-block scales. Timing input only: the values follow no distribution a
// quantizer would produce.
int vxs_random_kquant(int fmt, void *dst, int64_t nblocks, uint64_t seed) {
    if (nblocks <= 0) return 0;
    if (fmt != 3 && fmt != 4) return -1;
    random_kquant_kernel<<<(unsigned)((nblocks + 255) / 256), 256>>>((uint8_t *)dst, nblocks, fmt == 3 ? 144 : 210,
                                                                      fmt == 3 ? 0 : 208, fmt == 3 ? 2 : -1, seed);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return (int)hipDeviceSynchronize();
}

// fmt: 1 = Q4_0, 2 = Q8_0. Returns 0 or a hipError_t value.
int vxs_gaussian_quant(int fmt, void *dst, int64_t nblocks, float stdv, uint64_t seed) {
    if (nblocks <= 0) return 0;
    unsigned grid = (unsigned)((nblocks + 255) / 256);
    if (fmt == 1)
        gaussian_q4_0_kernel<<<grid, 256>>>((uint8_t *)dst, nblocks, stdv, seed);
    else if (fmt == 2)
        gaussian_q8_0_kernel<<<grid, 256>>>((uint8_t *)dst, nblocks, stdv, seed);
    else
        return -1;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return (int)hipDeviceSynchronize();
}

// n must be even.
int vxs_gaussian_f16(void *dst, int64_t n, float stdv, uint64_t seed) {
    if (n <= 0) return 0;
    int64_t npairs = n / 2;
    unsigned grid = (unsigned)((npairs + 255) / 256);
    gaussian_f16_kernel<<<grid, 256>>>((_Float16 *)dst, npairs, stdv, seed);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return (int)hipDeviceSynchronize();
}

}  // extern "C"
