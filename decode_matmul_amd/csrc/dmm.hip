// libdmm: decode+matmul for MI355X (gfx950, CDNA4).  Kernels and the C ABI of include/dmm.h.
//
// The weight matrix arrives as 16-bit codes, one per 8 consecutive weights along K
// (format: /root/reference/test_decode_matmul.py:29-55,
//          /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:45-65).
// Decoding one code is: one 16-byte LDS read of the grid row, one 16-byte LDS read of a
// (+-1.0 x 8) sign row indexed by the seven sign bits (the parity-implied eighth sign is
// baked into that table), one integer op for the packed +-0.25, and four packed-half FMAs
//     w = g * s + delta          (g * +-1 is exact, so this is the flip-then-add of the
//                                 reference with a single rounding)
// whose result registers are, unchanged, the 8-halves-per-lane operand of the
// 16x16x32 / 32x32x16 half MFMA.  Nothing decoded ever goes back through memory on the
// matrix-vector path.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "dmm.h"

namespace dmm {

typedef _Float16 half_t;
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u4_t __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// ------------------------------------------------------------------ decode tables in LDS
struct DecodeTables {
    u4_t grid[256];   // row i: 8 halves of grid[i][0..7]
    u4_t sign[128];   // row s: 8 halves, +-1.0, dim d negative iff bit d of (s | parity(s) << 7)
};

__device__ __forceinline__ u4_t sign_row(uint32_t s7)
{
    uint32_t s8 = s7 | ((__builtin_popcount(s7) & 1u) << 7);
    u4_t r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t lo = ((s8 >> (2 * i)) & 1u) ? 0xBC00u : 0x3C00u;
        uint32_t hi = ((s8 >> (2 * i + 1)) & 1u) ? 0xBC00u : 0x3C00u;
        r[i] = lo | (hi << 16);
    }
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

// ------------------------------------------------------------------ matrix-vector path (M <= 16*MT)
// Workgroup = W waves, owns 16*R consecutive rows of W for the whole of K; the waves split
// K in interleaved 256-wide steps.  In one step a lane (row r = lane%16 of each 16-row
// tile, quarter q = lane/16) loads 8 consecutive codes (16 bytes) of its row, decodes them
// one at a time and feeds each as the A operand (16 rows x 32 k: this lane supplies the 8
// k of its quarter) of v_mfma_f32_16x16x32_f16.  The B operand is x: column c = lane%16 is
// row m = c of x, same 8 k.  Any k order works as long as A and B agree, so the 32 k of
// MFMA number t in a step are {64*q + 8*t .. +8 : q = 0..3} rather than 32 consecutive k;
// that is what lets the code load be one 16-byte load per lane.  For M = 1 only column 0
// carries data, the other 15 columns cost nothing extra: the matrix unit has the
// headroom and the kernel is bound by the code bytes coming from HBM.
// Accumulator layout: lane holds rows 4*q + i (i = 0..3) of column c, i.e.
// y[m = c][n = n0 + 4*q + i] - four consecutive halves of a row of y.
template <int R, int W, int MT>
struct GemvShared {
    DecodeTables tab;
    f4_t red[W][R * MT][kWave];
};

template <int R, int W, int MT>
__global__ __launch_bounds__(64 * W) void gemv_kernel(const uint16_t *__restrict__ x,
                                                      const uint16_t *__restrict__ codes,
                                                      const void *__restrict__ grid, float scale,
                                                      uint16_t *__restrict__ y, int M, int N, int K)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    GemvShared<R, W, MT> &sh = *reinterpret_cast<GemvShared<R, W, MT> *>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int c16 = lane & 15;   // row within a 16-row tile (A) / column m within an m-tile (B)
    const int q = lane >> 4;     // k quarter
    const int n_steps = K >> 8;  // 256 k per step
    const int64_t row_bytes = (int64_t)K >> 2;  // K/8 codes * 2 bytes
    const int row0 = blockIdx.x * (16 * R);

    // per-tile code pointers; rows past N are clamped (their results are never stored)
    const unsigned char *cptr[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        int row = row0 + 16 * r + c16;
        row = row < N ? row : N - 1;
        cptr[r] = reinterpret_cast<const unsigned char *>(codes) + row * row_bytes + q * 16;
    }
    // x pointers: lane's column c16 is row m of x (per m-tile), its quarter starts at 64*q.
    // Columns past M read row 0: whatever they compute is never stored, and identical
    // addresses within a quarter cost no extra bytes.
    const unsigned char *xptr[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        int m = 16 * mt + c16;
        m = m < M ? m : 0;
        xptr[mt] = reinterpret_cast<const unsigned char *>(x) + ((int64_t)m * K + 64 * q) * 2;
    }

    // first step's code loads go out before the tables are built
    u4_t cw[R];
    int step = wave;
    if (step < n_steps) {
#pragma unroll
        for (int r = 0; r < R; r++) cw[r] = *reinterpret_cast<const u4_t *>(cptr[r] + (int64_t)step * 64);
    }

    stage_tables<true>(sh.tab, grid, tid, 64 * W);
    __syncthreads();

    f4_t acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[r][mt] = f4_t{0.f, 0.f, 0.f, 0.f};

    for (; step < n_steps; step += W) {
        // x for this step: 8 x 16 bytes per lane and m-tile (64 halves of the lane's quarter)
        u4_t xb[MT][8];
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int t = 0; t < 8; t++)
                xb[mt][t] = *reinterpret_cast<const u4_t *>(xptr[mt] + (int64_t)step * 512 + t * 16);
        // next step's codes
        u4_t cn[R];
        const int next = step + W;
        if (next < n_steps) {
#pragma unroll
            for (int r = 0; r < R; r++) cn[r] = *reinterpret_cast<const u4_t *>(cptr[r] + (int64_t)next * 64);
        }
#pragma unroll
        for (int t2 = 0; t2 < 4; t2++) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                u4_t w0, w1;
                decode8x2(cw[r][t2], sh.tab, w0, w1);
                h8_t a0 = __builtin_bit_cast(h8_t, w0);
                h8_t a1 = __builtin_bit_cast(h8_t, w1);
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    acc[r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        a0, __builtin_bit_cast(h8_t, xb[mt][2 * t2]), acc[r][mt], 0, 0, 0);
                    acc[r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        a1, __builtin_bit_cast(h8_t, xb[mt][2 * t2 + 1]), acc[r][mt], 0, 0, 0);
                }
            }
        }
        if (next < n_steps) {
#pragma unroll
            for (int r = 0; r < R; r++) cw[r] = cn[r];
        }
    }

    // cross-wave (split-K) reduction through LDS, then scale, round to half and store
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) sh.red[wave][r * MT + mt][lane] = acc[r][mt];
    __syncthreads();
    for (int idx = tid; idx < R * MT * kWave; idx += 64 * W) {
        const int l = idx & 63;
        const int tile = idx >> 6;
        const int r = tile / MT, mt = tile % MT;
        f4_t s = sh.red[0][tile][l];
#pragma unroll
        for (int w = 1; w < W; w++) s += sh.red[w][tile][l];
        const int m = 16 * mt + (l & 15);
        const int n = row0 + 16 * r + 4 * (l >> 4);
        if (m < M && n < N) {   // N % 4 == 0, so the four rows are in range together
            h4_t o;
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = (half_t)(s[i] * scale);
            *reinterpret_cast<h4_t *>(y + (int64_t)m * N + n) = o;
        }
    }
}

// ------------------------------------------------------------------ matrix-matrix path
// Block tile 128 (n) x 128 (m) x 64 (k), 4 waves as 2 x 2, each wave 64 x 64 with
// v_mfma_f32_32x32x16_f16 (A = decoded W rows, B = x rows, fp32 accumulate).  Per k tile
// every thread decodes four codes of one W row into LDS and copies 64 bytes of x into LDS;
// the global loads of tile k+1 are issued before the MFMAs of tile k.
constexpr int kGemmBN = 128, kGemmBM = 128, kGemmBK = 64;
constexpr int kGemmLd = kGemmBK + 8;   // halves per LDS row: 144 B keeps 16-byte alignment, staggers banks

struct GemmShared {
    DecodeTables tab;
    uint16_t w[kGemmBN][kGemmLd];
    uint16_t x[kGemmBM][kGemmLd];
};

__global__ __launch_bounds__(256) void gemm_kernel(const uint16_t *__restrict__ x,
                                                   const uint16_t *__restrict__ codes,
                                                   const void *__restrict__ grid, float scale,
                                                   uint16_t *__restrict__ y, int M, int N, int K)
{
    __shared__ GemmShared sh;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wn = wave & 1, wm = wave >> 1;
    const int n0 = blockIdx.x * kGemmBN;
    const int m0 = blockIdx.y * kGemmBM;
    const int k_tiles = K / kGemmBK;
    const int64_t kc = K >> 3;

    stage_tables<true>(sh.tab, grid, tid, 256);

    // W staging: thread -> row tid/2, codes 4*(tid%2) .. +3 of the k tile (8 bytes)
    const int w_row = tid >> 1, w_half = tid & 1;
    int wr = n0 + w_row;
    wr = wr < N ? wr : N - 1;
    const uint16_t *wsrc = codes + (int64_t)wr * kc + w_half * 4;
    // x staging: thread -> row tid/2, 32 halves (64 bytes) starting at 32*(tid%2)
    int xr = m0 + w_row;
    const bool x_in = xr < M;
    xr = x_in ? xr : M - 1;
    const uint16_t *xsrc = x + (int64_t)xr * K + w_half * 32;

    u2_t cw = *reinterpret_cast<const u2_t *>(wsrc);
    u4_t xv[4];
#pragma unroll
    for (int i = 0; i < 4; i++) xv[i] = reinterpret_cast<const u4_t *>(xsrc)[i];

    f16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    const int l32 = lane & 31, kq = lane >> 5;
    __syncthreads();   // tables ready

    for (int kt = 0; kt < k_tiles; kt++) {
        // registers -> LDS (decode W on the way)
        {
            u4_t w0, w1, w2, w3;
            decode8x2(cw[0], sh.tab, w0, w1);
            decode8x2(cw[1], sh.tab, w2, w3);
            u4_t *dst = reinterpret_cast<u4_t *>(&sh.w[w_row][w_half * 32]);
            dst[0] = w0; dst[1] = w1; dst[2] = w2; dst[3] = w3;
            u4_t *xd = reinterpret_cast<u4_t *>(&sh.x[w_row][w_half * 32]);
            const u4_t zero = u4_t{0u, 0u, 0u, 0u};
#pragma unroll
            for (int i = 0; i < 4; i++) xd[i] = x_in ? xv[i] : zero;
        }
        __syncthreads();
        if (kt + 1 < k_tiles) {
            cw = *reinterpret_cast<const u2_t *>(wsrc + (int64_t)(kt + 1) * 8);
#pragma unroll
            for (int i = 0; i < 4; i++)
                xv[i] = reinterpret_cast<const u4_t *>(xsrc + (int64_t)(kt + 1) * kGemmBK)[i];
        }
#pragma unroll
        for (int ks = 0; ks < kGemmBK / 16; ks++) {
            h8_t a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                a[i] = *reinterpret_cast<const h8_t *>(&sh.w[wn * 64 + i * 32 + l32][ks * 16 + kq * 8]);
                b[i] = *reinterpret_cast<const h8_t *>(&sh.x[wm * 64 + i * 32 + l32][ks * 16 + kq * 8]);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // D layout of 32x32: element e of lane: row (n) = 8*(e/4) + 4*(lane/32) + e%4, column (m) = lane%32
    const bool n_vec = (N & 3) == 0;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int m = m0 + wm * 64 + j * 32 + l32;
            if (m >= M) continue;
#pragma unroll
            for (int e4 = 0; e4 < 4; e4++) {
                const int n = n0 + wn * 64 + i * 32 + 8 * e4 + 4 * kq;
                uint16_t o[4];
#pragma unroll
                for (int e = 0; e < 4; e++)
                    o[e] = __builtin_bit_cast(uint16_t, (half_t)(acc[i][j][4 * e4 + e] * scale));
                uint16_t *dst = y + (int64_t)m * N + n;
                if (n_vec && n + 3 < N) {
                    u2_t v;
                    v[0] = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
                    v[1] = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
                    *reinterpret_cast<u2_t *>(dst) = v;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < N) dst[e] = o[e];
                }
            }
        }
}

// ------------------------------------------------------------------ host side
thread_local hipEvent_t tls_start = nullptr;
thread_local hipEvent_t tls_stop = nullptr;

template <typename Kern, typename... Args>
int launch(Kern kernel, dim3 grid, dim3 block, size_t shmem, hipStream_t stream, Args... args)
{
    if (tls_start && tls_stop)
        hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, tls_start, tls_stop, 0, args...);
    else
        hipLaunchKernelGGL(kernel, grid, block, shmem, stream, args...);
    return (int)hipGetLastError();
}

inline bool aligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

int check_common(const void *x, const void *codes, const void *grid, const void *y, int64_t M,
                 int64_t N, int64_t K)
{
    if (M < 0 || N < 0 || K < 0 || (K & 7)) return DMM_ERR_BAD_SHAPE;
    if (M == 0 || N == 0) return DMM_OK;   // nothing to write; pointers may be NULL
    if (!y || !grid) return DMM_ERR_NULL_POINTER;
    if (K > 0 && (!x || !codes)) return DMM_ERR_NULL_POINTER;
    if (!aligned(x, 2) || !aligned(codes, 2) || !aligned(grid, 2) || !aligned(y, 2)) return DMM_ERR_MISALIGNED;
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return DMM_ERR_TOO_LARGE;
    return DMM_OK;
}

bool gemv_ok(const void *x, const void *codes, const void *grid, const void *y, int64_t M, int64_t N,
             int64_t K)
{
    return M >= 1 && M <= 32 && K >= 256 && (K & 255) == 0 && (N & 3) == 0 && aligned(x, 16) &&
           aligned(codes, 16) && aligned(grid, 16) && aligned(y, 8);
}

bool gemm_ok(const void *x, const void *codes, const void *grid, const void *, int64_t M, int64_t N,
             int64_t K)
{
    return M >= 1 && N >= 1 && K >= 64 && (K & 63) == 0 && aligned(x, 16) && aligned(codes, 16) &&
           aligned(grid, 16) && M <= 65535LL * kGemmBM;
}

template <int R, int W, int MT>
int launch_gemv(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                int64_t N, int64_t K, hipStream_t stream)
{
    const size_t shmem = sizeof(GemvShared<R, W, MT>);
    static bool attr_done = false;   // benign race: every thread sets the same value
    if (!attr_done && shmem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_kernel<R, W, MT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return (int)e;
        attr_done = true;
    }
    const int64_t blocks = (N + 16 * R - 1) / (16 * R);
    return launch(gemv_kernel<R, W, MT>, dim3((unsigned)blocks), dim3(64 * W), shmem, stream,
                  (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)M, (int)N,
                  (int)K);
}

int run_gemv(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
             int64_t N, int64_t K, hipStream_t stream)
{
    if (M <= 16) return launch_gemv<2, 8, 1>(x, codes, grid, scale, y, M, N, K, stream);
    return launch_gemv<2, 8, 2>(x, codes, grid, scale, y, M, N, K, stream);
}

int run_gemm(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
             int64_t N, int64_t K, hipStream_t stream)
{
    dim3 g((unsigned)((N + kGemmBN - 1) / kGemmBN), (unsigned)((M + kGemmBM - 1) / kGemmBM));
    return launch(gemm_kernel, g, dim3(256), 0, stream, (const uint16_t *)x, (const uint16_t *)codes, grid,
                  scale, (uint16_t *)y, (int)M, (int)N, (int)K);
}

// y = 0 when K == 0 (empty sum), any M, N.
__global__ void zero_kernel(uint16_t *y, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        y[i] = 0;
}

int run_generic(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                int64_t N, int64_t K, hipStream_t stream)
{
    if (K == 0) {
        int64_t n = M * N;
        unsigned blocks = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
        return launch(zero_kernel, dim3(blocks), dim3(256), 0, stream, (uint16_t *)y, n);
    }
    int64_t blocks = (N + 3) / 4;
    if (blocks > 65535 * 16) blocks = 65535 * 16;
    return launch(generic_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint16_t *)x,
                  (const uint16_t *)codes, grid, scale, (uint16_t *)y, M, N, K);
}

}  // namespace dmm

using namespace dmm;

extern "C" {

int dmm_version(void) { return (0 << 16) | 1; }

const char *dmm_status_string(int status)
{
    switch (status) {
        case DMM_OK: return "ok";
        case DMM_ERR_NULL_POINTER: return "a required pointer is NULL";
        case DMM_ERR_BAD_SHAPE: return "bad shape: sizes must be non-negative and K a multiple of 8";
        case DMM_ERR_MISALIGNED: return "a pointer does not meet the required alignment";
        case DMM_ERR_TOO_LARGE: return "a dimension is too large for the launch";
        case DMM_ERR_UNSUPPORTED: return "this explicit path does not support the given shape or alignment";
        default: break;
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "unknown status";
}

int dmm_set_kernel_events(void *start_event, void *stop_event)
{
    if ((start_event == nullptr) != (stop_event == nullptr)) return DMM_ERR_NULL_POINTER;
    tls_start = (hipEvent_t)start_event;
    tls_stop = (hipEvent_t)stop_event;
    return DMM_OK;
}

int dmm_decode_f16(const void *codes, const void *grid, void *W, int64_t N, int64_t K, void *stream)
{
    if (N < 0 || K < 0 || (K & 7)) return DMM_ERR_BAD_SHAPE;
    const int64_t n_codes = N * (K >> 3);
    if (n_codes == 0) return DMM_OK;
    if (!codes || !grid || !W) return DMM_ERR_NULL_POINTER;
    if (!aligned(codes, 2) || !aligned(grid, 2) || !aligned(W, 2)) return DMM_ERR_MISALIGNED;
    const bool wide = aligned(codes, 4) && aligned(grid, 16) && aligned(W, 16);
    const int64_t work = wide ? (n_codes + 1) / 2 : n_codes;
    int64_t blocks = (work + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    if (wide)
        return launch(decode_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                      (const uint16_t *)codes, grid, (uint16_t *)W, n_codes);
    return launch(decode_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                  (const uint16_t *)codes, grid, (uint16_t *)W, n_codes);
}

int dmm_generic_f16(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                    int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    return run_generic(x, codes, grid, scale, y, M, N, K, (hipStream_t)stream);
}

int dmm_gemv_f16(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                 int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    if (!gemv_ok(x, codes, grid, y, M, N, K)) return DMM_ERR_UNSUPPORTED;
    return run_gemv(x, codes, grid, scale, y, M, N, K, (hipStream_t)stream);
}

int dmm_gemm_f16(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                 int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    if (!gemm_ok(x, codes, grid, y, M, N, K)) return DMM_ERR_UNSUPPORTED;
    return run_gemm(x, codes, grid, scale, y, M, N, K, (hipStream_t)stream);
}

int dmm_decode_matmul_f16(const void *x, const void *codes, const void *grid, float scale, void *y,
                          int64_t M, int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    hipStream_t s = (hipStream_t)stream;
    if (gemv_ok(x, codes, grid, y, M, N, K)) return run_gemv(x, codes, grid, scale, y, M, N, K, s);
    if (gemm_ok(x, codes, grid, y, M, N, K)) return run_gemm(x, codes, grid, scale, y, M, N, K, s);
    return run_generic(x, codes, grid, scale, y, M, N, K, s);
}

}  // extern "C"
