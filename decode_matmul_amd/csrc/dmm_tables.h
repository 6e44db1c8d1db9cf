// Decode tables in the LDS, the scalar decode of one code, the standalone decoder and the
// catch-all operator kernel.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ decode tables in LDS
struct DecodeTables {
    u4_t grid[256];   // row i: 8 halves of grid[i][0..7]
    u4_t sign[128];   // row s: 8 halves, +-1.0, dim d negative iff bit d of (s | parity(s) << 7)
};

__device__ __forceinline__ u4_t sign_row(uint32_t s7)
{
    const uint32_t s8 = s7 | ((__builtin_popcount(s7) & 1u) << 7);
    u4_t r;
#pragma unroll
    for (int i = 0; i < 4; i++)   // +-1.0 = 0x3C00 with the sign bit of dim 2i (low half) / 2i+1 (high half)
        r[i] = 0x3C003C00u | (((s8 >> (2 * i)) & 1u) << 15) | (((s8 >> (2 * i + 1)) & 1u) << 31);
    return r;
}

// Fill the tables with `nthreads` threads (tid in [0, nthreads)).  grid16 tells whether the
// global grid pointer may be read 16 bytes at a time.
template <bool kAligned>
__device__ __forceinline__ void stage_tables(DecodeTables &t, const void *grid, int tid, int nthreads)
{
    for (int i = tid; i < 256; i += nthreads) {
        if (kAligned) {
            t.grid[i] = reinterpret_cast<const u4_t *>(grid)[i];
        } else {
            const uint16_t *g = reinterpret_cast<const uint16_t *>(grid) + i * 8;
            u4_t r;
#pragma unroll
            for (int j = 0; j < 4; j++) r[j] = (uint32_t)g[2 * j] | ((uint32_t)g[2 * j + 1] << 16);
            t.grid[i] = r;
        }
    }
    for (int i = tid; i < 128; i += nthreads) t.sign[i] = sign_row((uint32_t)i);
}

__device__ __forceinline__ h2_t as_h2(uint32_t v) { return __builtin_bit_cast(h2_t, v); }
__device__ __forceinline__ uint32_t as_u32(h2_t v) { return __builtin_bit_cast(uint32_t, v); }

// Decode one code (low 16 bits of c) into 8 halves = 4 packed registers.
__device__ __forceinline__ u4_t decode8(uint32_t c, const DecodeTables &t)
{
    u4_t g = t.grid[c & 0xFFu];
    u4_t s = t.sign[(c >> 8) & 0x7Fu];
    uint32_t db = ((c & 0x8000u) * 0x10001u) | 0x34003400u;   // packed (+-0.25, +-0.25)
    h2_t d = as_h2(db);
    u4_t w;
#pragma unroll
    for (int i = 0; i < 4; i++) w[i] = as_u32(__builtin_elementwise_fma(as_h2(g[i]), as_h2(s[i]), d));
    return w;
}

// Two codes packed in one 32-bit word (low half = first code).
__device__ __forceinline__ void decode8x2(uint32_t w, const DecodeTables &t, u4_t &w0, u4_t &w1)
{
    u4_t g0 = t.grid[w & 0xFFu];
    u4_t s0 = t.sign[(w >> 8) & 0x7Fu];
    u4_t g1 = t.grid[(w >> 16) & 0xFFu];
    u4_t s1 = t.sign[(w >> 24) & 0x7Fu];
    uint32_t db = (w & 0x80008000u) | 0x34003400u;            // delta of code 0 | delta of code 1 << 16
    h2_t d0 = as_h2((db & 0xFFFFu) * 0x10001u);
    h2_t d1 = as_h2((db >> 16) * 0x10001u);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        w0[i] = as_u32(__builtin_elementwise_fma(as_h2(g0[i]), as_h2(s0[i]), d0));
        w1[i] = as_u32(__builtin_elementwise_fma(as_h2(g1[i]), as_h2(s1[i]), d1));
    }
}

// ------------------------------------------------------------------ standalone decoder
// Flat: code i -> halves [8i, 8i+8).  kAligned: each thread takes 8 codes with one
// 16-byte load and issues eight 16-byte stores; otherwise one code per thread.
template <bool kAligned>
__global__ __launch_bounds__(256) void decode_kernel(const uint16_t *__restrict__ codes,
                                                     const void *__restrict__ grid,
                                                     uint16_t *__restrict__ W, int64_t n_codes)
{
    __shared__ DecodeTables tab;
    stage_tables<kAligned>(tab, grid, threadIdx.x, 256);
    __syncthreads();
    if (kAligned) {
        // a wave covers 64 consecutive 32-bit words per step: loads are 256 B per wave,
        // stores 2 KiB per wave, both contiguous.
        const int64_t n_words = n_codes >> 1;
        const uint32_t *cw = reinterpret_cast<const uint32_t *>(codes);
        u4_t *out = reinterpret_cast<u4_t *>(W);
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * 256) {
            u4_t w0, w1;
            decode8x2(cw[i], tab, w0, w1);
            out[2 * i] = w0;
            out[2 * i + 1] = w1;
        }
        if ((n_codes & 1) && blockIdx.x == 0 && threadIdx.x == 0)
            out[n_codes - 1] = decode8(codes[n_codes - 1], tab);
    } else {
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_codes; i += (int64_t)gridDim.x * 256) {
            u4_t w = decode8(codes[i], tab);
            uint16_t *o = W + i * 8;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                o[2 * j] = (uint16_t)(w[j] & 0xFFFFu);
                o[2 * j + 1] = (uint16_t)(w[j] >> 16);
            }
        }
    }
}

// ------------------------------------------------------------------ generic operator path
// One wave per output row n, lanes stride over the row's codes, dot products on the
// vector ALU with fp32 accumulation, DPP/shuffle reduction across the wave.  Handles any
// M, N, K % 8 == 0 and 2-byte alignment; M is processed in chunks of kMC rows of x.
constexpr int kGenericMC = 4;

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__global__ __launch_bounds__(256) void generic_kernel(const uint16_t *__restrict__ x,
                                                      const uint16_t *__restrict__ codes,
                                                      const void *__restrict__ grid, float scale,
                                                      uint16_t *__restrict__ y, int64_t M, int64_t N,
                                                      int64_t K)
{
    __shared__ DecodeTables tab;
    stage_tables<false>(tab, grid, threadIdx.x, 256);
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t kc = K >> 3;
    for (int64_t n = (int64_t)blockIdx.x * 4 + wave; n < N; n += (int64_t)gridDim.x * 4) {
        const uint16_t *crow = codes + n * kc;
        for (int64_t m0 = 0; m0 < M; m0 += kGenericMC) {
            float acc[kGenericMC] = {};
            for (int64_t j = lane; j < kc; j += kWave) {
                u4_t w = decode8(crow[j], tab);
                float wf[8];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    h2_t p = as_h2(w[i]);
                    wf[2 * i] = (float)p[0];
                    wf[2 * i + 1] = (float)p[1];
                }
#pragma unroll
                for (int mm = 0; mm < kGenericMC; mm++) {
                    if (m0 + mm < M) {
                        const uint16_t *xr = x + (m0 + mm) * K + j * 8;
#pragma unroll
                        for (int d = 0; d < 8; d++) {
                            half_t xv = __builtin_bit_cast(half_t, xr[d]);
                            acc[mm] = __builtin_fmaf((float)xv, wf[d], acc[mm]);
                        }
                    }
                }
            }
#pragma unroll
            for (int mm = 0; mm < kGenericMC; mm++) {
                float s = wave_sum(acc[mm]);
                if (lane == 0 && m0 + mm < M) {
                    half_t h = (half_t)(s * scale);
                    y[(m0 + mm) * N + n] = __builtin_bit_cast(uint16_t, h);
                }
            }
        }
    }
}
