// Quantized GEMM for decode batches (2 <= M, one or two activation tiles per workgroup), wave-private form
// (included by qgemm.hip inside its anonymous namespace).
//
// One workgroup of NW waves per compute unit owns 16*R weight rows and one K slice; each wave takes whole
// 256-column chunks of the slice (chunk c_begin + wave, + NW, ...) for ALL of the workgroup's rows. Why this cut:
// at 32 activation rows a step of 32 columns needs 4 KB of activation operand (hi and lo halves) against 288
// bytes of Q4_0 weights per 16-row tile, so the activation operand, not the weight stream, is what a compute unit
// has to move. Waves that split K between them read every activation element once per compute unit, and the more
// rows a wave covers per step the more MFMAs each operand load feeds. Nothing is shared between the waves until
// the end, so the main loop has no workgroup barrier:
//   * the activation tiles of a step (MFMA-ready as the prepare kernels leave them) go from global memory (L2)
//     straight into registers, three steps ahead of their use (seven where a step has four MFMA tile pairs or
//     fewer and passes quickly), once per step for all R weight tiles;
//   * the wave's weight bytes are staged four steps at a time: global -> registers (requested a whole stage ahead,
//     in flight while the previous stage is computed) -> the wave's own LDS region, laid out one row after the
//     other so that lane (row, g) of a tile finds its four code bytes with one read;
//   * per tile and step: unpack the codes to exact integer f16 values, v_mfma_f32_16x16x32_f16 for the hi and the
//     lo halves of each activation tile, one fused multiply-add per output with the block scale.
// The accumulators stay in the units of the current chunk's activation scale: at a chunk boundary they are
// multiplied by the ratio of the two chunks' factors (powers of two, exact) instead of keeping a second set of
// per-chunk sums. At the end the waves' sums are added in wave order through LDS and go to the split-K partial
// sums (or, with one slice, to the output). Which chunks a wave takes and the order of every addition depend on
// (N, K, R, NW, slices) only, so a row has the same bits in any batch.
//
// Requirements checked by the host: N >= 16*R and a multiple of 16, every boundary between weight segments a
// multiple of 16*R, K a multiple of 256, 16-byte aligned rows. A last row group that would run past N is moved
// back to end at N and writes only the rows the groups before it do not own.

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
template <int BYTES> struct PieceOf;
template <> struct PieceOf<8> { typedef u32x2 type; };
template <> struct PieceOf<16> { typedef u32x4 type; };

constexpr int WSS = 4;     // steps per stage

// Per format: how a stage (WSS steps of one chunk) of a weight row is brought into LDS and read back.
//   PIECE / NP: a row's stage is NP pieces of PIECE bytes; src_off(h, col): where piece col of stage h starts
//   inside the row's chunk; PITCH: bytes between rows in LDS (16 rows x 4 lane groups read conflict-free when
//   PITCH/4 is 4 mod 8); GI / GROWS: GI load instructions of 64 lanes cover GROWS whole rows.
struct WQ4_0 {
    static constexpr int CHUNK_BYTES = 144, PIECE = 8, NP = 9, PITCH = 80, GI = 1, GROWS = 7;
    static constexpr bool HAS_MIN = false;
    static __host__ __device__ size_t row_bytes(int K) { return (size_t)K / 32 * 18; }
    static __device__ __forceinline__ int src_off(int h, int col) { return 72 * h + 8 * col; }
    struct Raw { uint32_t a, b, d; };
    // row: the lane's weight row in the stage; sp: step inside the stage (a compile-time constant after unrolling)
    static __device__ __forceinline__ Raw read(const uint8_t *row, int sp, int g) {
        const int byte = 18 * sp + 2;  // the block's 16 code bytes; lane group g takes bytes 4g..4g+3
        const uint32_t *p = (const uint32_t *)(row + (byte & ~3)) + g;
        Raw x;
        x.a = p[0];
        x.b = (byte & 3) ? p[1] : 0u;
        x.d = *(const uint16_t *)(row + 18 * sp);
        return x;
    }
    static __device__ __forceinline__ StepW unpack(const Raw &x, int sp, int) {
        const uint32_t w = ((18 * sp + 2) & 3) ? __builtin_amdgcn_alignbyte(x.b, x.a, 2u) : x.a;
        const half2v off = {(_Float16)1032.f, (_Float16)1032.f};  // 1024 + 8
        const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu, c64 = 0x64646464u;
        StepW r;  // byte b next to a 0x64 byte is the f16 1024 + b
        r.b = pack8(as_h2(__builtin_amdgcn_perm(lo, c64, 0x00060004u)) - off, as_h2(__builtin_amdgcn_perm(hi, c64, 0x00060004u)) - off,
                    as_h2(__builtin_amdgcn_perm(lo, c64, 0x00070005u)) - off, as_h2(__builtin_amdgcn_perm(hi, c64, 0x00070005u)) - off);
        r.d = h2f((uint16_t)x.d);
        r.dm = 0.f;
        return r;
    }
};

struct WQ8_0 {
    static constexpr int CHUNK_BYTES = 272, PIECE = 8, NP = 17, PITCH = 144, GI = 2, GROWS = 7;
    static constexpr bool HAS_MIN = false;
    static __host__ __device__ size_t row_bytes(int K) { return (size_t)K / 32 * 34; }
    static __device__ __forceinline__ int src_off(int h, int col) { return 136 * h + 8 * col; }
    struct Raw { uint32_t a0, a1, b0, b1, d; };
    static __device__ __forceinline__ Raw read(const uint8_t *row, int sp, int g) {
        const int byte = 34 * sp + 2;  // elements 4g..4g+3; 16+4g.. are 16 bytes on
        const uint32_t *p = (const uint32_t *)(row + (byte & ~3)) + g;
        Raw x;
        x.a0 = p[0];
        x.b0 = p[4];
        x.a1 = (byte & 3) ? p[1] : 0u;
        x.b1 = (byte & 3) ? p[5] : 0u;
        x.d = *(const uint16_t *)(row + 34 * sp);
        return x;
    }
    static __device__ __forceinline__ StepW unpack(const Raw &x, int sp, int) {
        const bool sh = ((34 * sp + 2) & 3) != 0;
        const uint32_t w0 = (sh ? __builtin_amdgcn_alignbyte(x.a1, x.a0, 2u) : x.a0) ^ 0x80808080u;
        const uint32_t w1 = (sh ? __builtin_amdgcn_alignbyte(x.b1, x.b0, 2u) : x.b0) ^ 0x80808080u;
        const half2v off = {(_Float16)1152.f, (_Float16)1152.f};  // 1024 + 128
        const uint32_t c64 = 0x64646464u;
        StepW r;
        r.b = pack8(as_h2(__builtin_amdgcn_perm(w0, c64, 0x00060004u)) - off, as_h2(__builtin_amdgcn_perm(w1, c64, 0x00060004u)) - off,
                    as_h2(__builtin_amdgcn_perm(w0, c64, 0x00070005u)) - off, as_h2(__builtin_amdgcn_perm(w1, c64, 0x00070005u)) - off);
        r.d = h2f((uint16_t)x.d);
        r.dm = 0.f;
        return r;
    }
};

// Q4_K: a stage is the super-block's 16-byte header (d, dmin, the twelve scale bytes) and half of its 128 code
// bytes; steps 2i and 2i+1 are the low and the high nibbles of code bytes 32i..32i+31.
struct WQ4_K {
    static constexpr int CHUNK_BYTES = 144, PIECE = 16, NP = 5, PITCH = 80, GI = 1, GROWS = 12;
    static constexpr bool HAS_MIN = true;
    static __host__ __device__ size_t row_bytes(int K) { return (size_t)K / 256 * 144; }
    static __device__ __forceinline__ int src_off(int h, int col) { return col == 0 ? 0 : 64 * h + 16 * col; }
    struct Raw { uint32_t w0, w1, hd, s0, s1, s2; };
    static __device__ __forceinline__ Raw read(const uint8_t *row, int sp, int g) {
        const uint32_t *sb = (const uint32_t *)row;
        const uint32_t *qp = sb + 4 + 8 * (sp >> 1);
        Raw r;
        r.w0 = qp[g];
        r.w1 = qp[4 + g];
        r.hd = sb[0];
        r.s0 = sb[1];
        r.s1 = sb[2];
        r.s2 = sb[3];
        return r;
    }
    static __device__ __forceinline__ StepW unpack(const Raw &x, int, int j) {
        PQ4_K::Raw y = {x.w0, x.w1, x.hd, x.s0, x.s1, x.s2};
        return PQ4_K::unpack(y, j);
    }
};

// BF16 (pkg/gguf/dequant.go:215-228): no blocks and no scales. A bf16 value's eight significant bits fit f16's eleven,
// so its conversion to f16 is exact wherever the value lies inside f16's range. The weights are converted times 64
// (added to the exponent field; 1/64 is the step's scale): exact for magnitudes from 2^-23 to 1023, an absolute error
// below 2^-31 under that, and a wrong (saturated) value from 1024 up, which weight matrices do not hold.
// A stage is the row's 128 elements, 256 bytes.
struct WBF16 {
    static constexpr int CHUNK_BYTES = 512, PIECE = 16, NP = 16, PITCH = 272, GI = 1, GROWS = 4;
    static constexpr bool HAS_MIN = false;
    static __host__ __device__ size_t row_bytes(int K) { return (size_t)K * 2; }
    static __device__ __forceinline__ int src_off(int h, int col) { return 256 * h + 16 * col; }
    struct Raw { uint32_t a0, a1, b0, b1; };  // elements 4g..4g+3 and 16+4g..16+4g+3 of the step
    static __device__ __forceinline__ Raw read(const uint8_t *row, int sp, int g) {
        const uint32_t *p = (const uint32_t *)(row + 64 * sp) + 2 * g;
        Raw x;
        x.a0 = p[0];
        x.a1 = p[1];
        x.b0 = p[8];
        x.b1 = p[9];
        return x;
    }
    static __device__ __forceinline__ half2v cvt2(uint32_t lo_bits, uint32_t hi_bits) {  // two bf16 patterns in the high halves
        return __builtin_bit_cast(half2v, __builtin_amdgcn_cvt_pkrtz(__uint_as_float(lo_bits), __uint_as_float(hi_bits)));
    }
    static __device__ __forceinline__ StepW unpack(const Raw &x, int, int) {
        constexpr uint32_t E = 6u << 23;  // times 64 (a zero becomes 2^-121 and converts to zero)
        auto lo = [](uint32_t w) { return (w << 16) + E; };
        auto hi = [](uint32_t w) { return (w & 0xFFFF0000u) + E; };
        StepW r;  // slot order {4g, 4g+2, 16+4g, 16+4g+2, 4g+1, 4g+3, 16+4g+1, 16+4g+3}
        r.b = pack8(cvt2(lo(x.a0), lo(x.a1)), cvt2(lo(x.b0), lo(x.b1)), cvt2(hi(x.a0), hi(x.a1)), cvt2(hi(x.b0), hi(x.b1)));
        r.d = 1.f / 64.f;
        r.dm = 0.f;
        return r;
    }
};

// ratio of two chunk factors (positive powers of two): the difference of their exponent fields
__device__ __forceinline__ float pow2_ratio(float num, float den) {
    return __uint_as_float(__float_as_uint(num) - __float_as_uint(den) + 0x3F800000u);
}

template <class W, int R, int MT> struct WaveGeom {
    static constexpr int ROWS = 16 * R;
    static constexpr int TP = ROWS + 4;  // floats per row of the transposed block: rows 4 apart land 16 banks apart
    static constexpr int W_BYTES = ROWS * W::PITCH + 16;
    static constexpr int T_BYTES = 16 * MT * TP * 4;
    static constexpr int REGION = ((W_BYTES > T_BYTES ? W_BYTES : T_BYTES) + 15) / 16 * 16;
};

// grid = (ceil(N / (16 R)), K slices, groups of MT activation tiles); block = 64 NW.
template <class W, int R, int MT, int NW>
__global__ void __launch_bounds__(64 * NW, 1) qgemm_wave_kernel(Segs segs, PrepView pv, float *__restrict__ out,
                                                               const float *__restrict__ residual, float *__restrict__ partial,
                                                               int M, int Mpad, int N, int K, int n_slices, int flags,
                                                               QkvEpi epi) {
    typedef WaveGeom<W, R, MT> G;
    constexpr int ROWS = G::ROWS;
    // steps an activation load runs ahead of its use: a step of few tiles is short, so its operand must be
    // requested more steps ahead to cover the same latency (the ring's size divides the eight steps of a chunk)
    constexpr int AD = MT >= 4 ? 1 : (R * MT <= 4 ? 7 : 3);  // (four tiles a step: two ring slots are 64 registers)
    constexpr int NG = (ROWS + W::GROWS - 1) / W::GROWS;  // load groups per stage
    constexpr int LAST_ROWS = ROWS - (NG - 1) * W::GROWS;
    constexpr int REGION = G::REGION;
    typedef typename PieceOf<W::PIECE>::type piece_t;
    __shared__ __attribute__((aligned(16))) uint8_t w_lds[NW][REGION];

    const int tid = threadIdx.x, lane = tid & 63, ln = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same for all lanes: keeps chunk arithmetic scalar
    const int n_own = blockIdx.x * ROWS;                        // first row this workgroup writes
    const int n0 = min(n_own, N - ROWS);
    const int ks = blockIdx.y, mg = blockIdx.z, m0 = mg * 16 * MT, mtiles = Mpad / 16;
    const size_t row_bytes = W::row_bytes(K);
    const int sl_base = n_slices >> 16, sl_rem = n_slices & 0xFFFF;  // chunks per slice, slices with one more
    const int c_begin = ks * sl_base + min(ks, sl_rem);
    const int c_end = c_begin + sl_base + (ks < sl_rem ? 1 : 0);
    const int my_n = (c_end - c_begin - wave + NW - 1) / NW;  // chunks of this wave: c_begin + wave + NW i

    // the workgroup's rows lie in one segment
    const uint8_t *wg_rows;
    {
        const int e0 = segs.n_end[0], e1 = segs.n_end[1];
        const uint8_t *base = n0 < e0 ? segs.w[0] : (n0 < e1 ? segs.w[1] : segs.w[2]);
        const int local = n0 < e0 ? n0 : (n0 < e1 ? n0 - e0 : n0 - e1);
        wg_rows = base + (size_t)local * row_bytes;
    }
    uint8_t *const region = &w_lds[wave][0];

    // which piece of a load group this lane moves (instruction j of the group): row in the group, column. Lanes
    // beyond the group's rows repeat the first piece (same source, same destination).
    uint32_t voff[W::GI], voff_last[W::GI], hinc[W::GI], hinc_last[W::GI];
    int loff[W::GI], loff_last[W::GI];
#pragma unroll
    for (int j = 0; j < W::GI; j++) {
        const int pc = j * 64 + lane;
        const int lrow = pc / W::NP, lcol = pc % W::NP;
        const bool ok = lrow < W::GROWS, ok_l = lrow < LAST_ROWS;
        const int row = ok ? lrow : 0, col = ok ? lcol : 0, row_l = ok_l ? lrow : 0, col_l = ok_l ? lcol : 0;
        voff[j] = (uint32_t)(row * row_bytes) + W::src_off(0, col);
        voff_last[j] = (uint32_t)(row_l * row_bytes) + W::src_off(0, col_l);
        hinc[j] = (uint32_t)(W::src_off(1, col) - W::src_off(0, col));
        hinc_last[j] = (uint32_t)(W::src_off(1, col_l) - W::src_off(0, col_l));
        loff[j] = row * W::PITCH + col * W::PIECE;
        loff_last[j] = row_l * W::PITCH + col_l * W::PIECE;
    }

    float4v run[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int t = 0; t < MT; t++) run[r][t] = (float4v){0.f, 0.f, 0.f, 0.f};

    if (my_n > 0) {
        piece_t st[NG * W::GI];
        // Stage q of this wave: chunk c_begin + wave + NW (q / 2), half q % 2; past the end the last one again.
        auto fetch = [&](int q) __attribute__((always_inline)) {
            const int qq = min(q, 2 * my_n - 1);
            const int chunk = c_begin + wave + NW * (qq >> 1), h = qq & 1;
            const uint8_t *src = wg_rows + (size_t)chunk * W::CHUNK_BYTES;
#pragma unroll
            for (int i = 0; i < NG; i++)
#pragma unroll
                for (int j = 0; j < W::GI; j++) {
                    const uint32_t vo = i == NG - 1 ? voff_last[j] + (h ? hinc_last[j] : 0u) : voff[j] + (h ? hinc[j] : 0u);
                    st[i * W::GI + j] = *(const piece_t *)(src + (size_t)i * W::GROWS * row_bytes + vo);
                }
        };
        auto commit = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < NG; i++)
#pragma unroll
                for (int j = 0; j < W::GI; j++)
                    *(piece_t *)(region + i * W::GROWS * W::PITCH + (i == NG - 1 ? loff_last[j] : loff[j])) = st[i * W::GI + j];
        };
        struct StepA { half8 h[MT], l[MT]; };
        // the wave's q-th step (q counts through its chunks, eight steps each); past its last step the last again
        const int q_last = 8 * my_n - 1;
        auto load_a = [&](int q) __attribute__((always_inline)) {
            const int qq = min(q, q_last);
            const int s = (c_begin + wave + NW * (qq >> 3)) * 8 + (qq & 7);
            StepA a;
            const half8 *p = pv.tiles + ((size_t)(s * mtiles + mg * MT) * 2) * 64 + lane;
#pragma unroll
            for (int t = 0; t < MT; t++) {
                a.h[t] = p[(t * 2 + 0) * 64];
                a.l[t] = p[(t * 2 + 1) * 64];
            }
            return a;
        };
        auto load_cs = [&](int chunk, float4v (&cs)[MT]) __attribute__((always_inline)) {
#pragma unroll
            for (int t = 0; t < MT; t++) cs[t] = *(const float4v *)(pv.cscale + (size_t)chunk * Mpad + m0 + t * 16 + 4 * g);
        };
        const uint8_t *const lane_row = region + ln * W::PITCH;  // this lane's row of tile 0
        // one step: every weight tile of the stage's step sp against the activation tiles a
        auto compute = [&](const StepA &a, int s, int sp, int j) __attribute__((always_inline)) {
            float4v bs[MT];
            if (W::HAS_MIN) {
#pragma unroll
                for (int t = 0; t < MT; t++) bs[t] = *(const float4v *)(pv.bsum + (size_t)s * Mpad + m0 + t * 16 + 4 * g);
            }
            typename W::Raw raw = W::read(lane_row, sp, g);
#pragma unroll
            for (int r = 0; r < R; r++) {
                const StepW w = W::unpack(raw, sp, j);
                if (r + 1 < R) raw = W::read(lane_row + (r + 1) * 16 * W::PITCH, sp, g);
                float4v acc[MT];
#pragma unroll
                for (int t = 0; t < MT; t++)
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h[t], w.b, (float4v){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                for (int t = 0; t < MT; t++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.l[t], w.b, acc[t], 0, 0, 0);
#pragma unroll
                for (int t = 0; t < MT; t++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if (W::HAS_MIN)
                            run[r][t][e] = __builtin_fmaf(-w.dm, bs[t][e], __builtin_fmaf(w.d, acc[t][e], run[r][t][e]));
                        else
                            run[r][t][e] = __builtin_fmaf(w.d, acc[t][e], run[r][t][e]);
                    }
            }
        };

        // Loads come back in issue order, so anything a step waits for must be older than the prefetches around
        // it: the chunk factors of the next chunk are requested at the top of the current one.
        float4v cs[MT], cs_next[MT], cs_prev[MT];
        load_cs(c_begin + wave, cs);
        fetch(0);
        StepA ar[AD + 1];  // step q's tiles sit in ar[q % (AD + 1)] (eight steps per chunk keep the slots in phase)
        static_assert(8 % (AD + 1) == 0, "the ring must stay in phase with the chunks");
#pragma unroll
        for (int i = 0; i < AD; i++) ar[i] = load_a(i);
        ar[AD] = ar[AD - 1];
        for (int ci = 0; ci < my_n; ci++) {
            const int chunk = c_begin + wave + NW * ci;
            load_cs(c_begin + wave + NW * min(ci + 1, my_n - 1), cs_next);
            if (ci > 0) {
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    float4v f;
#pragma unroll
                    for (int e = 0; e < 4; e++) f[e] = pow2_ratio(cs_prev[t][e], cs[t][e]);
#pragma unroll
                    for (int r = 0; r < R; r++)
#pragma unroll
                        for (int e = 0; e < 4; e++) run[r][t][e] *= f[e];
                }
            }
#pragma unroll
            for (int t = 0; t < MT; t++) cs_prev[t] = cs[t];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                commit();
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                __builtin_amdgcn_wave_barrier();

                const int s = chunk * 8 + h * WSS, q = ci * 8 + h * WSS;
#pragma unroll
                for (int sp = 0; sp < WSS; sp++) {
                    const int j = h * WSS + sp;
                    // the slot of the step before this one is free: the tiles AD steps on go there; the next
                    // stage's weights are requested right behind the first of them
                    ar[(j + AD) % (AD + 1)] = load_a(q + sp + AD);
                    if (sp == 0) fetch(2 * ci + h + 1);
                    __builtin_amdgcn_sched_barrier(0);
                    compute(ar[j % (AD + 1)], s + sp, sp, j);
                    __builtin_amdgcn_sched_barrier(0);
                }
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                __builtin_amdgcn_wave_barrier();

            }
#pragma unroll
            for (int t = 0; t < MT; t++) cs[t] = cs_next[t];
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int e = 0; e < 4; e++) run[r][t][e] *= cs_prev[t][e];
    }

    // The waves' sums, added in wave order. Lane (g, ln) of tile (r, t) holds C[m0 + 16t + 4g + e][n0 + 16r + ln];
    // each wave lays its block out in its own region as [m][n] rows of ROWS + 4 floats, then every thread adds
    // the NW regions for a float4 of the output.
    constexpr int TP = G::TP;
    const bool vec = (flags & 1) != 0;
    __syncthreads();  // every wave is done with its region
    {
        float *T = (float *)region;
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int e = 0; e < 4; e++) T[(t * 16 + 4 * g + e) * TP + r * 16 + ln] = run[r][t][e];
    }
    // Q|K|V rows finished here: the row factors (with the pending 1/rms of the RMSNorm that fed the activation) are
    // whole-wave computations, one row at a time
    __shared__ float s_fac[16 * MT];
    if (epi.q_out) {
        for (int r = wave; r < 16 * MT; r += NW) {
            const float f = row_factor(pv.inv_scale, epi.rn, m0 + r);
            if (lane == 0) s_fac[r] = f;
        }
    }
    __syncthreads();
    constexpr int F4 = 16 * MT * ROWS / 4;  // float4 groups of the block
    constexpr int NT = 64 * NW;
#pragma unroll
    for (int i = 0; i < (F4 + NT - 1) / NT; i++) {
        const int f = i * NT + tid;
        if (F4 % NT != 0 && f >= F4) break;
        const int ml = f / (ROWS / 4), nl = (f % (ROWS / 4)) * 4;
        float4 c = *(const float4 *)((const float *)&w_lds[0][0] + ml * TP + nl);
#pragma unroll
        for (int w = 1; w < NW; w++) {
            const float4 d = *(const float4 *)((const float *)&w_lds[w][0] + ml * TP + nl);
            c.x += d.x; c.y += d.y; c.z += d.z; c.w += d.w;
        }
        const int m = m0 + ml, n = n0 + nl;
        if (m >= M || n < n_own) continue;
        if (epi.q_out) {
            // columns n .. n+3 of row m: two RoPE pairs of a Q or K head, or four V values (the arithmetic of
            // rope_store_partials_kernel, which does this for launches that leave partial sums)
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
                continue;
            }
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
            continue;
        }
        if (partial) {
            *(float4 *)(partial + ((size_t)ks * M + m) * N + n) = c;
            continue;
        }
        const float inv = pv.inv_scale[m];
        float v[4] = {__fmul_rn(c.x, inv), __fmul_rn(c.y, inv), __fmul_rn(c.z, inv), __fmul_rn(c.w, inv)};
        float *dst = out + (size_t)m * N + n;
        const float *rs = residual ? residual + (size_t)m * N + n : nullptr;
        if (vec) {
            if (rs) {
                const float4 q = *(const float4 *)rs;
                v[0] = __fadd_rn(q.x, v[0]); v[1] = __fadd_rn(q.y, v[1]); v[2] = __fadd_rn(q.z, v[2]); v[3] = __fadd_rn(q.w, v[3]);
            }
            *(float4 *)dst = make_float4(v[0], v[1], v[2], v[3]);
        } else {
            for (int e = 0; e < 4; e++) dst[e] = rs ? __fadd_rn(rs[e], v[e]) : v[e];
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The same arithmetic for many activation rows (prompt chunks, candidate trees), cut the other way: the eight
// waves of a workgroup take 16*R weight rows EACH (128*R rows per workgroup) and walk the K slice together, against
// 16*MT activation rows whose tiles the workgroup brings into LDS once per half chunk for all eight. Per step a
// wave unpacks its R weight tiles once and feeds R*MT MFMA pairs from them, so the unpack and the weight staging
// are spread over MT*16 rows instead of 32, and an activation tile is fetched from L2 once per 128*R weight rows.
// Weight staging (global -> registers -> the wave's own LDS rows) is the wave-private kernel's; the activation
// tiles are double-buffered in LDS with one workgroup barrier per half chunk.
// grid = (ceil(N / (128 R)), K slices, ceil(Mpad / (16 MT))); block = 512.
template <class W, int R, int MT>
__global__ void __launch_bounds__(512, 1) qgemm_rows_kernel(Segs segs, PrepView pv, float *__restrict__ out,
                                                           const float *__restrict__ residual, float *__restrict__ partial,
                                                           int M, int Mpad, int N, int K, int n_slices) {
    constexpr int NW = 8, ROWS = 16 * R;
    constexpr int NG = (ROWS + W::GROWS - 1) / W::GROWS;
    constexpr int LAST_ROWS = ROWS - (NG - 1) * W::GROWS;
    constexpr int W_BYTES = (ROWS * W::PITCH + 16 + 15) / 16 * 16;
    constexpr int A_HALF = WSS * MT * 2 * 64;  // half8 pieces of a half chunk's activation tiles
    static_assert(MT * 2 * 64 == 512, "one piece per thread and step");
    typedef typename PieceOf<W::PIECE>::type piece_t;
    __shared__ __attribute__((aligned(16))) uint8_t w_lds[NW][W_BYTES];
    __shared__ half8 a_lds[2][A_HALF];

    const int tid = threadIdx.x, lane = tid & 63, ln = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_own = (blockIdx.x * NW + wave) * ROWS;  // first row this wave writes
    const int n0 = max(min(n_own, N - ROWS), 0);         // (a wave past the matrix' end works on its last rows and writes nothing)
    const int ks = blockIdx.y, mg = blockIdx.z, m0 = mg * 16 * MT, mtiles = Mpad / 16;
    const size_t row_bytes = W::row_bytes(K);
    const int sl_base = n_slices >> 16, sl_rem = n_slices & 0xFFFF;
    const int c_begin = ks * sl_base + min(ks, sl_rem);
    const int c_end = c_begin + sl_base + (ks < sl_rem ? 1 : 0);
    const int n_half = 2 * (c_end - c_begin);

    const uint8_t *wg_rows;
    {
        const int e0 = segs.n_end[0], e1 = segs.n_end[1];
        const uint8_t *base = n0 < e0 ? segs.w[0] : (n0 < e1 ? segs.w[1] : segs.w[2]);
        const int local = n0 < e0 ? n0 : (n0 < e1 ? n0 - e0 : n0 - e1);
        wg_rows = base + (size_t)local * row_bytes;
    }
    uint8_t *const region = &w_lds[wave][0];
    uint32_t voff[W::GI], voff_last[W::GI], hinc[W::GI], hinc_last[W::GI];
    int loff[W::GI], loff_last[W::GI];
#pragma unroll
    for (int j = 0; j < W::GI; j++) {
        const int pc = j * 64 + lane;
        const int lrow = pc / W::NP, lcol = pc % W::NP;
        const bool ok = lrow < W::GROWS, ok_l = lrow < LAST_ROWS;
        const int row = ok ? lrow : 0, col = ok ? lcol : 0, row_l = ok_l ? lrow : 0, col_l = ok_l ? lcol : 0;
        voff[j] = (uint32_t)(row * row_bytes) + W::src_off(0, col);
        voff_last[j] = (uint32_t)(row_l * row_bytes) + W::src_off(0, col_l);
        hinc[j] = (uint32_t)(W::src_off(1, col) - W::src_off(0, col));
        hinc_last[j] = (uint32_t)(W::src_off(1, col_l) - W::src_off(0, col_l));
        loff[j] = row * W::PITCH + col * W::PIECE;
        loff_last[j] = row_l * W::PITCH + col_l * W::PIECE;
    }
    // this thread's piece of a step's activation tiles: tile tid / 128 of the group (hi and lo halves, 64 lanes each);
    // a tile past the padded rows repeats the last one (its products are not stored)
    const int a_tile = min(mg * MT + tid / 128, mtiles - 1);
    const half8 *a_src = pv.tiles + ((size_t)a_tile * 2) * 64 + (tid & 127);

    float4v run[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int t = 0; t < MT; t++) run[r][t] = (float4v){0.f, 0.f, 0.f, 0.f};

    piece_t st[NG * W::GI];
    half8 areg[WSS];
    // half chunk q of the slice: chunk c_begin + q / 2, half q % 2 (past the end: the last again)
    auto fetch = [&](int q) __attribute__((always_inline)) {
        const int qq = min(q, n_half - 1);
        const int chunk = c_begin + (qq >> 1), h = qq & 1;
        const uint8_t *src = wg_rows + (size_t)chunk * W::CHUNK_BYTES;
#pragma unroll
        for (int i = 0; i < NG; i++)
#pragma unroll
            for (int j = 0; j < W::GI; j++) {
                const uint32_t vo = i == NG - 1 ? voff_last[j] + (h ? hinc_last[j] : 0u) : voff[j] + (h ? hinc[j] : 0u);
                st[i * W::GI + j] = *(const piece_t *)(src + (size_t)i * W::GROWS * row_bytes + vo);
            }
        const int s0 = chunk * 8 + h * WSS;
#pragma unroll
        for (int sp = 0; sp < WSS; sp++) areg[sp] = a_src[(size_t)(s0 + sp) * mtiles * 128];
    };
    auto commit = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NG; i++)
#pragma unroll
            for (int j = 0; j < W::GI; j++)
                *(piece_t *)(region + i * W::GROWS * W::PITCH + (i == NG - 1 ? loff_last[j] : loff[j])) = st[i * W::GI + j];
#pragma unroll
        for (int sp = 0; sp < WSS; sp++) a_lds[buf][sp * 512 + tid] = areg[sp];
    };
    auto load_cs = [&](int chunk, float4v (&cs)[MT]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const int mt = min(mg * MT + t, mtiles - 1);
            cs[t] = *(const float4v *)(pv.cscale + (size_t)chunk * Mpad + mt * 16 + 4 * g);
        }
    };
    const uint8_t *const lane_row = region + ln * W::PITCH;

    if (n_half > 0) {
        float4v cs[MT], cs_prev[MT];
        fetch(0);
        load_cs(c_begin, cs);
        commit(0);
        __syncthreads();
        for (int q = 0; q < n_half; q++) {
            const int chunk = c_begin + (q >> 1), h = q & 1;
            fetch(q + 1);
            if (h == 0 && q > 0) {
                // a new chunk: the sums move to its activation scale
                float4v cn[MT];
                load_cs(chunk, cn);
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    float4v f;
#pragma unroll
                    for (int e = 0; e < 4; e++) f[e] = pow2_ratio(cs[t][e], cn[t][e]);
#pragma unroll
                    for (int r = 0; r < R; r++)
#pragma unroll
                        for (int e = 0; e < 4; e++) run[r][t][e] *= f[e];
                    cs[t] = cn[t];
                }
            }
            const half8 *ab = &a_lds[q & 1][0];
#pragma unroll
            for (int sp = 0; sp < WSS; sp++) {
                const int j = h * WSS + sp, s = chunk * 8 + j;
                half8 ah[MT], al[MT];
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    ah[t] = ab[sp * 512 + (t * 2 + 0) * 64 + lane];
                    al[t] = ab[sp * 512 + (t * 2 + 1) * 64 + lane];
                }
                float4v bs[MT];
                if (W::HAS_MIN) {
#pragma unroll
                    for (int t = 0; t < MT; t++) {
                        const int mt = min(mg * MT + t, mtiles - 1);
                        bs[t] = *(const float4v *)(pv.bsum + (size_t)s * Mpad + mt * 16 + 4 * g);
                    }
                }
                typename W::Raw raw = W::read(lane_row, sp, g);
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const StepW w = W::unpack(raw, sp, j);
                    if (r + 1 < R) raw = W::read(lane_row + (r + 1) * 16 * W::PITCH, sp, g);
                    float4v acc[MT];
#pragma unroll
                    for (int t = 0; t < MT; t++)
                        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah[t], w.b, (float4v){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                    for (int t = 0; t < MT; t++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al[t], w.b, acc[t], 0, 0, 0);
#pragma unroll
                    for (int t = 0; t < MT; t++)
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            if (W::HAS_MIN)
                                run[r][t][e] = __builtin_fmaf(-w.dm, bs[t][e], __builtin_fmaf(w.d, acc[t][e], run[r][t][e]));
                            else
                                run[r][t][e] = __builtin_fmaf(w.d, acc[t][e], run[r][t][e]);
                        }
                }
            }
            // the next half chunk: this wave's weights into its own rows (it is done reading them), the activation
            // tiles into the buffer that every wave finished with before the previous barrier
            commit((q + 1) & 1);
            __syncthreads();
        }
#pragma unroll
        for (int t = 0; t < MT; t++) cs_prev[t] = cs[t];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int e = 0; e < 4; e++) run[r][t][e] *= cs_prev[t][e];
    }

    // lane (g, ln) of tile (r, t) holds C[m0 + 16t + 4g + e][n0 + 16r + ln]
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int m = m0 + 16 * t + 4 * g + e;
            if (m >= M) continue;
            const float inv = partial ? 1.f : pv.inv_scale[m];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int n = n0 + 16 * r + ln;
                if (n < n_own) continue;
                if (partial) {
                    partial[((size_t)ks * M + m) * N + n] = run[r][t][e];
                } else {
                    float v = __fmul_rn(run[r][t][e], inv);
                    if (residual) v = __fadd_rn(residual[(size_t)m * N + n], v);
                    out[(size_t)m * N + n] = v;
                }
            }
        }
}
