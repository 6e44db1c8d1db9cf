// Matrix-vector kernels on 8-bit operands: fp8 weights times bf8 terms of x on the scaled MFMA,
// with x in registers (M = 1..4) or staged through the LDS in chunks (M = 1, any K).
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ streaming matrix-vector path, 8-bit operands
// The streaming kernel above is bound by the LDS: two 16-byte table gathers per code.  When
// every grid value is exactly representable in 8 bits (fp8 e4m3: 4 significant bits - the E8P
// grid of half-odd values is), the same product can be formed with 8-byte gathers, which the
// LDS serves at twice the rate, by running the matrix unit on 8-bit operands:
//   * weights.  w = s g + d, s = +-1 per dim, d = +-1/4 per code.  The grid table holds rows of
//     8 fp8 bytes, the sign table rows of 8 flag bytes (0x80 = flipped); one exclusive or per
//     4 weights applies the signs, and the 8 bytes of a code are a quarter of the A operand of
//     v_mfma_f32_16x16x128_f8f6f4 (four codes = 32 consecutive k per lane; twice the time of the
//     16x16x32 form for four times the work) as they are.  d is left out of the decode and added by the
//     matrix unit instead: sum_k d x[k] = sum over codes of (8 d) * (mean of the code's 8 x
//     values), one more MFMA (the 16-bit 16x16x32 form) per 16 rows x 256 k, into an
//     accumulator of its own, whose A operand is +-2.0 per code, made from the code words
//     themselves (the shift bit is the sign bit of a half), and whose B operand is the means as
//     two halves, hi + lo (22 bits of the fp32 sum of the 8 values), in two columns;
//   * x.  A half with a zero low byte IS a bf8 (e5m2) number in its high byte.  Cutting x after
//     its top byte, subtracting, scaling what is left by 8 and repeating gives
//     x = t0 + t1 / 8 + t2 / 64 + t3 / 512 exactly for every normal x (3 significant bits per
//     term, 11 in a half); the four terms sit in four B columns - at batch 1 the other 15
//     columns of the 16-wide tile are idle anyway - and the four result columns are added, with
//     those weights, at the end.
// s g + d is exact in half for every fp8 g and the terms of x add up to x (subnormal x may lose
// bits below 2^-24 * 4), so nothing is lost in the operands, and the products are exact in the
// fp32 accumulators.  Two things remain: the means (hi + lo drops what lies 22 bits below the
// leading one of a mean) and the matrix unit's adder, which aligns the products of a group to
// the largest of them.  Measured against the fp64 reference on the benchmark's inputs: 98 %
// of the outputs are the correctly rounded ones and the 99th percentile of the error is 0.57
// half ulps (the 16-bit kernel: 0.5, the output rounding alone); with 100-fold outliers in x
// 2.6 ulps; x with few significant bits: every output correctly rounded.  All of it a
// hundredth of the operator's tolerance of 1e-2 or less.  A grid with a value fp8 cannot hold is found while the table is built
// (convert, convert back, compare), an x that is not finite while it is split; every workgroup
// then runs the 16-bit kernel above instead: same launch, same result as that kernel gives.
// LDS map: [0, 32K) sign rows (128 x 32 copies x 8 B), [32K, 96K) grid rows (256 x 32 copies x
// 8 B; a lane reads copy lane % 32, conflict-free for any codes), partial sums, then the terms
// of x (column m * 4 + t, pitch K + 16 bytes) and the means (rows 2 m: hi, 2 m + 1: lo; K / 8
// halves each, pitch K / 4 + 16 bytes).
typedef __attribute__((address_space(3))) const u2_t lds_u2_t;
__device__ __forceinline__ u2_t lds_read8(uint32_t byte_addr)
{
    return *reinterpret_cast<lds_u2_t *>(byte_addr);
}

// Partial sums of a row block, two parities: one float4 per (wave, tile, quarter, x row), the term
// columns already added by the wave.
__host__ __device__ constexpr int q8_red_bytes(int R, int W, int M) { return 2 * W * R * 4 * M * 16; }
// terms of x (4 rows of K bytes per x row), the per-code means of x as two halves each (hi + lo:
// 2 rows of K / 8 halves per x row), and one word per wave for the vote on the grid
__host__ __device__ constexpr int64_t q8_x_bytes(int64_t M, int64_t K)
{
    return 4 * M * (K + 16) + 2 * M * (K / 4 + 16) + 64;
}

// the 8 sign flags of a sign-row index as bytes: dims 0-3 in [0], 4-7 in [1]
__device__ __forceinline__ u2_t sign_bytes(uint32_t s7)
{
    const uint32_t s8 = s7 | ((__builtin_popcount(s7) & 1u) << 7);
    u2_t r;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const uint32_t n = (s8 >> (4 * i)) & 0xFu;
        r[i] = ((n & 1u) << 7) | ((n & 2u) << 14) | ((n & 4u) << 21) | ((n & 8u) << 28);
    }
    return r;
}

// a grid row as 8 fp8 bytes; exact: every value survives the round trip
__device__ __forceinline__ u2_t grid_row_fp8(const u4_t &row, bool &exact)
{
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const h2_t h = as_h2(row[i]);
        f[2 * i] = (float)h[0];
        f[2 * i + 1] = (float)h[1];
    }
    u2_t r;
    exact = true;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        int p = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * i], f[4 * i + 1], 0, false);
        p = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * i + 2], f[4 * i + 3], p, true);
        r[i] = (uint32_t)p;
        // (no short circuit: eight compares in a row beat eight branches)
        exact = exact & (__builtin_amdgcn_cvt_f32_fp8(p, 0) == f[4 * i]) & (__builtin_amdgcn_cvt_f32_fp8(p, 1) == f[4 * i + 1]) &
                (__builtin_amdgcn_cvt_f32_fp8(p, 2) == f[4 * i + 2]) & (__builtin_amdgcn_cvt_f32_fp8(p, 3) == f[4 * i + 3]);
    }
    return r;
}

// A half as four bf8 terms, h = t0 + t1 / 8 + t2 / 64 + t3 / 512: a term is the top byte of what
// is left, and what is left after it is scaled by 8 (exact, and it keeps the remainder as far
// above the subnormal range as h itself was), so every normal h is split without loss.
// 8 halves (one 16-byte piece of x) at a time: term t of the 8 as 8 bytes in t[t].  Returns
// whether all 8 are finite (if not, the caller hands the launch to the 16-bit kernel: an
// infinity must meet the whole weight, not its two parts one after the other).
__device__ __forceinline__ bool split_piece_bf8(const u4_t &v, u2_t (&t)[4])
{
    bool finite = true;
#pragma unroll
    for (int i = 0; i < 4; i++) finite = finite && (v[i] & 0x7C00u) != 0x7C00u && (v[i] & 0x7C000000u) != 0x7C000000u;
    const h2_t eight = h2_t{(half_t)8.0f, (half_t)8.0f};
    u4_t r = v;
#pragma unroll
    for (int term = 0; term < 4; term++) {
        const u4_t hi = r & 0xFF00FF00u;
        t[term][0] = __builtin_amdgcn_perm(hi[1], hi[0], 0x07050301u);   // the high bytes of halves 0..3
        t[term][1] = __builtin_amdgcn_perm(hi[3], hi[2], 0x07050301u);   // and of halves 4..7
        if (term < 3) {
#pragma unroll
            for (int i = 0; i < 4; i++) r[i] = as_u32((as_h2(r[i]) - as_h2(hi[i])) * eight);
        }
    }
    return finite;
}

// The mean of the 8 halves of a piece (fp32 sum, times 1/8) as two halves, hi + lo: 22 of the
// fp32 sum's 24 bits.  Low half of the result: hi.
__device__ __forceinline__ uint32_t piece_mean_hi_lo(const u4_t &v)
{
    const h2_t ones = h2_t{(half_t)1.0f, (half_t)1.0f};
    float r = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) r = __builtin_amdgcn_fdot2(as_h2(v[i]), ones, r, false);
    r *= 0.125f;
    const half_t hi = (half_t)r;
    const half_t lo = (half_t)(r - (float)hi);
    return as_u32(h2_t{hi, lo});
}

struct Q8Gather {
    u2_t g0, s0, g1, s1;
};

// lane_base = (lane % 32) * 8; the tables start at LDS address 0
__device__ __forceinline__ void q8_gather(Q8Gather &o, uint32_t w, uint32_t lane_base)
{
    const uint32_t w7 = w & 0x7FFF7FFFu;                 // sign-row index must not see the shift bit
    o.g0 = lds_read8(__builtin_amdgcn_perm(w, lane_base, 0x0C0C0400u) + kSSignBytes);
    o.s0 = lds_read8(__builtin_amdgcn_perm(w7, lane_base, 0x0C0C0500u));
    o.g1 = lds_read8(__builtin_amdgcn_perm(w, lane_base, 0x0C0C0600u) + kSSignBytes);
    o.s1 = lds_read8(__builtin_amdgcn_perm(w7, lane_base, 0x0C0C0700u));
}

__device__ __forceinline__ long q8_pack(uint32_t lo, uint32_t hi)
{
    return (long)(((unsigned long)hi << 32) | (unsigned long)lo);
}

// One 256-wide k step for the first nv (uniform, 1 <= nv <= R) of R row tiles; same item order
// as stream_step.  xaddr: this lane's x terms of the step (16 bytes per word pair: the B
// operands of its two codes), x8addr: the means of its 8 codes (8 halves: hi or lo, by column).
template <int R>
__device__ __forceinline__ void q8_step(const u4_t (&cw)[R], uint32_t xaddr, uint32_t x8addr, uint32_t lane_base,
                                        f4_t (&acc)[R][2], f4_t (&accd)[R], int nv)
{
    // All 16 table gathers of a tile's step and the reads of x go out before the first MFMA
    // (8-byte results: 48 registers), so the wave meets the LDS latency once per step and tile,
    // not once per word; with two tiles the reads of x serve both.
    u4_t xq[4];
    xq[0] = lds_read16(xaddr);
    xq[1] = lds_read16(xaddr + 16);
    xq[2] = lds_read16(xaddr + 32);
    xq[3] = lds_read16(xaddr + 48);
    const u4_t x8 = lds_read16(x8addr);
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (r > 0 && r >= nv) break;   // tiles past nv: nothing to do (uniform)
        Q8Gather g[4];
#pragma unroll
        for (int t2 = 0; t2 < 4; t2++) q8_gather(g[t2], cw[r][t2], lane_base);
        // two words = four codes = 32 consecutive k of the lane's 64: one 16x16x128 MFMA (32
        // bytes per lane and operand, A fp8, B bf8, no scaling), which does four times the work
        // of the 16x16x32 form in twice its time
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const Q8Gather &b0 = g[2 * h], &b1 = g[2 * h + 1];
            const i8_t a = i8_t{(int)(b0.g0[0] ^ b0.s0[0]), (int)(b0.g0[1] ^ b0.s0[1]), (int)(b0.g1[0] ^ b0.s1[0]),
                                (int)(b0.g1[1] ^ b0.s1[1]), (int)(b1.g0[0] ^ b1.s0[0]), (int)(b1.g0[1] ^ b1.s0[1]),
                                (int)(b1.g1[0] ^ b1.s1[0]), (int)(b1.g1[1] ^ b1.s1[1])};
            const u4_t &x0 = xq[2 * h], &x1 = xq[2 * h + 1];
            const i8_t xb = i8_t{(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
            acc[r][h] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, xb, acc[r][h], 0 /* A: fp8 */, 1 /* B: bf8 */, 0, 0, 0, 0);
        }
        // the shift term, in 16-bit arithmetic: +-2.0 per code (a code word with everything but its
        // shift bits replaced by the bits of 2.0) against the means
        const u4_t a8 = (cw[r] & 0x80008000u) | 0x40004000u;
        accd[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8_t, a8), __builtin_bit_cast(h8_t, x8), accd[r], 0, 0, 0);
    }
}

template <int R, int W, int D, bool kPacked>
__global__ __launch_bounds__(64 * W) void gemv_q8_kernel(const uint16_t *__restrict__ x,
                                                         const uint16_t *__restrict__ codes,
                                                         const void *__restrict__ grid, float scale,
                                                         uint16_t *__restrict__ y, int M, int N, int K,
                                                         int tiles_q, int tiles_r)
{
    static_assert(R == 1 || R == 2, "a partial row block is handled as one tile");
    static_assert(W == 16, "the table staging below assumes 1024 threads");
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];
    f4_t *red = reinterpret_cast<f4_t *>(smem_raw + kSTablesBytes);   // two parities, see q8_red_bytes
    const int red_par = q8_red_bytes(R, W, M) / 32;                    // float4 per parity
    unsigned char *xt = smem_raw + kSTablesBytes + q8_red_bytes(R, W, M);
    // the means: rows 2 m (hi) and 2 m + 1 (lo) of K / 8 halves; the shift term has an accumulator of
    // its own, where they sit in columns 4 m and 4 m + 1
    const int xt_pitch = K + 16, x8_pitch = (K >> 2) + 16;
    unsigned char *x8t = xt + 4 * M * xt_pitch;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15;
    const int q = lane >> 4;
    const int n_steps = K >> 8;
    const int row_bytes = K >> 2;
    const uint32_t lane_base = (uint32_t)(lane & 31) * 8u;

    // ---- prologue: the loads with nothing queued in front of them first (grid rows, the first
    // pieces of x), then the code stream, then the tables and the terms of x while the code
    // loads fly.  The three kinds of staging go to different waves - grid rows to waves 0-3 (one
    // row per thread), sign rows to waves 4-7, x to everybody - because every instruction of
    // the prologue is paid once per wave that runs it, needed or not.
    u4_t grow = u4_t{0u, 0u, 0u, 0u};
    if (wave < 4) grow = reinterpret_cast<const u4_t *>(grid)[tid];
    const int row_chunks = K >> 3;                     // 16-byte pieces per row of x
    const int n_pieces = M * row_chunks;               // x is [M][K] contiguous: piece p sits at x + 16 p
    u4_t xnext = tid < n_pieces ? reinterpret_cast<const u4_t *>(x)[tid] : u4_t{0u, 0u, 0u, 0u};

    const int n_sw = wave < n_steps ? (n_steps - wave + W - 1) / W : 0;   // k steps of this wave per row block
    const int t0 = (int)blockIdx.x * tiles_q + ((int)blockIdx.x < tiles_r ? (int)blockIdx.x : tiles_r);
    const int t1 = t0 + tiles_q + ((int)blockIdx.x < tiles_r ? 1 : 0);
    const int nb_wg = (t1 - t0 + R - 1) / R;

    const int n_tiles_all = (N + 15) >> 4;
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(codes), 0, (int)((int64_t)(kPacked ? n_tiles_all * 16 : N) * row_bytes), 0x00020000);
    int voff[R];
#pragma unroll
    for (int r = 0; r < R; r++) voff[r] = kPacked ? lane * 16 + r * n_steps * 1024 : (16 * r + c16) * row_bytes + q * 16;
    constexpr int kOut = (int)0x80000000;
    int pf_blk = 0, pf_j = 0;
    auto issue = [&](u4_t (&cwd)[R]) {
        const bool ok = pf_blk < nb_wg && n_sw > 0;
        const int tb = t0 + pf_blk * R;
        const int soff = !ok ? kOut
                         : kPacked ? (tb * n_steps + wave + pf_j * W) * 1024
                                   : tb * 16 * row_bytes + (wave + pf_j * W) * 64;
#pragma unroll
        for (int r = 0; r < R; r++)   // tiles of a partial block that belong to the next workgroup: no access
            cwd[r] = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff[r], (r == 0 || tb + r < t1) ? soff : kOut, 0);
        if (++pf_j >= n_sw) { pf_j = 0; pf_blk++; }
    };

    u4_t cw[D][R];
#pragma unroll
    for (int d = 0; d < D; d++) issue(cw[d]);

    bool fits = true;   // stays true while x is finite and the grid fits fp8
    if (wave >= 4 && wave < 8) {
        // sign rows: 128 rows of 16 slots (16 bytes = two copies each); thread t of these 256 writes
        // 8 slots of row t / 2 (16 neighbouring lanes hit 16 different slot positions)
        const int t = tid - 256, row = t >> 1;
        const u2_t sb = sign_bytes((uint32_t)row);
        const uint32_t sg = lds_addr(smem_raw) + (uint32_t)((row * 16 + (t & 1) * 8 + (row & 7)) * 16);   // slot i ^ (row % 8)
#pragma unroll
        for (int i = 0; i < 8; i++) lds_write16(sg ^ (uint32_t)(i * 16), u4_t{sb[0], sb[1], sb[0], sb[1]});
    }
    __builtin_amdgcn_sched_barrier(0);   // keep the sign rows ahead of the waits for the loads

    // x -> its four terms, and the means of every 8 values -> theirs.  One piece per thread and
    // trip, the next one already on its way.
    {
        int m = 0, c = tid;
        for (int p = tid; p < n_pieces; p += 64 * W) {
            const u4_t v = xnext;
            if (p + 64 * W < n_pieces) xnext = reinterpret_cast<const u4_t *>(x)[p + 64 * W];
            while (c >= row_chunks) { c -= row_chunks; m++; }
            u2_t t[4];
            fits = split_piece_bf8(v, t) && fits;
            const uint32_t mb = piece_mean_hi_lo(v);
#pragma unroll
            for (int term = 0; term < 4; term++) *reinterpret_cast<u2_t *>(xt + (m * 4 + term) * xt_pitch + c * 8) = t[term];
            reinterpret_cast<uint16_t *>(x8t + (2 * m) * x8_pitch)[c] = (uint16_t)mb;
            reinterpret_cast<uint16_t *>(x8t + (2 * m + 1) * x8_pitch)[c] = (uint16_t)(mb >> 16);
            c += 64 * W;
        }
    }
    if (wave < 4) {
        // grid rows: thread tid converts row tid and writes its 16 slots (two copies each)
        bool exact;
        const u2_t g8 = grid_row_fp8(grow, exact);
        fits = fits && exact;
        const uint32_t gg = lds_addr(smem_raw) + (uint32_t)(kSSignBytes + (tid * 16 + (tid & 15)) * 16);   // slot i ^ (tid % 16)
#pragma unroll
        for (int i = 0; i < 16; i++) lds_write16(gg ^ (uint32_t)(i * 16), u4_t{g8[0], g8[1], g8[0], g8[1]});
    }
    // the vote: every wave publishes whether one of its rows or pieces failed, in a word of its own (so
    // nothing needs clearing first), and after the barrier every wave reads all of them
    uint32_t *votes = reinterpret_cast<uint32_t *>(x8t + 2 * M * x8_pitch);
    const bool wave_bad = __builtin_amdgcn_ballot_w64(!fits) != 0;
    if (lane == 0) votes[wave] = wave_bad ? 1u : 0u;
    __syncthreads();
    if (__builtin_amdgcn_ballot_w64(votes[lane & (W - 1)] != 0) != 0) {
        // a grid value does not fit 8 bits, or x is not finite: the 16-bit kernel takes over (it
        // builds its own tables)
        gemv_stream_body<R, W, 2, kPacked, 4>(x, codes, grid, scale, y, M, N, K, tiles_q, tiles_r);
        return;
    }

    // B operand addresses of this lane: column c16 = 4 m + term (column 0 for the idle ones)
    const int col = c16 < 4 * M ? c16 : 0;
    const int row8 = (c16 < 4 * M && (c16 & 3) < 2) ? 2 * (c16 >> 2) + (c16 & 3) : 0;   // hi or lo of x row c16 / 4
    const uint32_t xlane = lds_addr(xt) + (uint32_t)(col * xt_pitch + q * 64);
    const uint32_t x8lane = lds_addr(x8t) + (uint32_t)(row8 * x8_pitch + q * 16);

    f4_t acc[R][2];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r][0] = acc[r][1] = f4_t{0.f, 0.f, 0.f, 0.f};
    // weights of this lane's column: 8^-t with t = c16 % 4 for the terms of x, 1 for the two halves
    // of the means; columns that hold nothing count as zero
    const float x_weight = c16 < 4 * M ? __builtin_bit_cast(float, 0x3F800000u - ((uint32_t)(c16 & 3) * 3u << 23)) : 0.f;
    const float mean_weight = (c16 < 4 * M && (c16 & 3) < 2) ? 1.f : 0.f;
    f4_t accd[R];   // the shift term
#pragma unroll
    for (int r = 0; r < R; r++) accd[r] = f4_t{0.f, 0.f, 0.f, 0.f};

    auto finish_block = [&](int blk) {
        f4_t *rp = red + (blk & 1) * red_par;
#pragma unroll
        for (int r = 0; r < R; r++) {
            // the four term columns of an x row are added first, each with the weight of its term:
            // lane 4 m gets columns 4 m .. 4 m + 3
            f4_t v = (acc[r][0] + acc[r][1]) * x_weight + accd[r] * mean_weight;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                v[e] = dpp_shr_add<0x101>(v[e]);   // row_shl:1
                v[e] = dpp_shr_add<0x102>(v[e]);   // row_shl:2
            }
            if ((c16 & 3) == 0 && c16 < 4 * M) rp[(wave * R + r) * 4 * M + q * M + (c16 >> 2)] = v;
            acc[r][0] = acc[r][1] = accd[r] = f4_t{0.f, 0.f, 0.f, 0.f};
        }
        __syncthreads();
        for (int p = wave; p < R * M; p += W) {
            const int r = p / M, m = p - r * M;
            f4_t v = f4_t{0.f, 0.f, 0.f, 0.f};
            if (c16 < W) v = rp[(c16 * R + r) * 4 * M + q * M + m];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = row_sum16(v[e]);
            const int tile = t0 + blk * R + r;
            const int n = tile * 16 + 4 * q;
            if (c16 == 15 && tile < t1 && n < N) {   // N % 4 == 0, so the four rows are in range together
                h4_t o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = (half_t)(v[e] * scale);
                *reinterpret_cast<h4_t *>(y + (int64_t)m * N + n) = o;
            }
        }
    };

    if (n_sw == 0) {
        for (int blk = 0; blk < nb_wg; blk++) finish_block(blk);
        return;
    }

    const int n_items = nb_wg * n_sw;
    int blk = 0, j = 0;
    for (int i0 = 0; i0 < n_items; i0 += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (i0 + d < n_items) {
                const uint32_t step = (uint32_t)(wave + j * W);
                const int nv = t1 - (t0 + blk * R);   // tiles of this block that are ours (uniform)
                q8_step<R>(cw[d], xlane + step * 256u, x8lane + step * 64u, lane_base, acc, accd, nv);
                if (++j >= n_sw) {
                    j = 0;
                    finish_block(blk);
                    blk++;
                }
            }
            issue(cw[d]);
        }
    }
}

// ------------------------------------------------------------------ batch 1 on 8-bit operands, x staged in chunks
// gemv_q8_kernel's arithmetic (fp8 weights by two 8-byte gathers and two exclusive ors per code, x
// as four bf8 terms, the shift term through the per-code means) for ONE row of x of any length: the
// terms of x are staged 4096 values (16 k steps, one per wave) at a time into two LDS buffers taken
// in turn, the chunk after the current one being split while the current one is multiplied, so
//   * the launch starts multiplying after 512 pieces of x have been split, not after all of them,
//     and the rest of the splitting runs beside the code stream;
//   * the LDS holds 37 KB of x however long x is (K = 28672 needs 129 KB in one piece).
// A workgroup walks its tiles in groups of up to T; within a group it goes chunk by chunk, and
// in a chunk wave w does k step 16 c + w of every tile of the group with the same two registers
// of B operands.  One barrier per chunk hands the x buffers over; the partial sums of the T tiles
// meet once per group.  The code stream is one load per tile in flight per wave, refilled as soon
// as the tile's step of the chunk is done.
// LDS map: tables as in gemv_q8_kernel, partial sums [16 waves][T * 16 + 1] float4, two x buffers
// (4 term rows of 4096 + 16 bytes, 2 rows of means of 1024 + 16 bytes), one flag word.
constexpr int kQcChunkK = 4096;
constexpr int kQcTermPitch = kQcChunkK + 16, kQcMeanPitch = kQcChunkK / 4 + 16;
constexpr int kQcXBuf = 4 * kQcTermPitch + 2 * kQcMeanPitch;
__host__ __device__ constexpr int qc_red_bytes(int T) { return 16 * (T * 16 + 1) * 16; }
__host__ __device__ constexpr int qc_lds_bytes(int T) { return kSTablesBytes + qc_red_bytes(T) + 2 * kQcXBuf + 128; }

// the four bf8 terms of a piece of x (8 halves) and the mean of the 8 as hi + lo halves; returns
// whether all 8 are finite (their fp32 sum is finite exactly when they all are)
__device__ __forceinline__ bool qc_split_piece(const u4_t &v, u2_t (&t)[4], uint32_t &mean_hi_lo)
{
    const h2_t ones = h2_t{(half_t)1.0f, (half_t)1.0f};
    float r = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) r = __builtin_amdgcn_fdot2(as_h2(v[i]), ones, r, false);
    const bool finite = (__builtin_bit_cast(uint32_t, r) & 0x7F800000u) != 0x7F800000u;
    r *= 0.125f;
    const half_t hi = (half_t)r;
    const half_t lo = (half_t)(r - (float)hi);
    mean_hi_lo = as_u32(h2_t{hi, lo});
    const h2_t eight = h2_t{(half_t)8.0f, (half_t)8.0f};
    u4_t rem = v;
#pragma unroll
    for (int term = 0; term < 4; term++) {
        t[term][0] = __builtin_amdgcn_perm(rem[1], rem[0], 0x07050301u);   // the high bytes of halves 0..3
        t[term][1] = __builtin_amdgcn_perm(rem[3], rem[2], 0x07050301u);   // and of halves 4..7
        if (term < 3) {
#pragma unroll
            for (int i = 0; i < 4; i++) rem[i] = as_u32((as_h2(rem[i]) - as_h2(rem[i] & 0xFF00FF00u)) * eight);
        }
    }
    return finite;
}

template <int T, int DC, bool kPacked>
__global__ __launch_bounds__(1024) void gemv_q8c_kernel(const uint16_t *__restrict__ x,
                                                        const uint16_t *__restrict__ codes,
                                                        const void *__restrict__ grid, float scale,
                                                        uint16_t *__restrict__ y, int N, int K, int tiles_q, int tiles_r)
{
    constexpr int W = 16;
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];
    f4_t *red = reinterpret_cast<f4_t *>(smem_raw + kSTablesBytes);
    unsigned char *xbuf = smem_raw + kSTablesBytes + qc_red_bytes(T);
    // [0 .. 15]: one prologue vote per wave.  [16], [17]: "an x staged later is not finite", the word of chunk gc
    // being 16 + gc % 2: the stagers of chunk gc + 1 write the word nobody reads before the next barrier,
    // while slower waves may still be reading the word of chunk gc.  A word once set ends the loop for
    // every wave at the barrier that follows, so neither is ever cleared.
    uint32_t *flags = reinterpret_cast<uint32_t *>(xbuf + 2 * kQcXBuf);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15;
    const int q = lane >> 4;
    const int n_steps = K >> 8;
    const int n_chunks = (n_steps + W - 1) / W;
    const int row_bytes = K >> 2;
    const int n_pieces = K >> 3;
    const uint32_t lane_base = (uint32_t)(lane & 31) * 8u;

    // ---- prologue: grid rows to waves 8-11, sign rows to waves 12-15, the first chunk of x to waves 0-7
    u4_t grow = u4_t{0u, 0u, 0u, 0u};
    if (wave >= 8 && wave < 12) grow = reinterpret_cast<const u4_t *>(grid)[tid - 512];
    u4_t xpiece = u4_t{0u, 0u, 0u, 0u};
    if (wave < 8 && tid < n_pieces) xpiece = reinterpret_cast<const u4_t *>(x)[tid];

    // this workgroup's tiles [t0, t1), walked in n_groups groups of up to T tiles whose sizes differ by
    // at most one (7 tiles with T = 3: 3 + 2 + 2, not 3 + 3 + 1: a group of one leaves a wave a single
    // load in flight)
    const int t0 = (int)blockIdx.x * tiles_q + ((int)blockIdx.x < tiles_r ? (int)blockIdx.x : tiles_r);
    const int t1 = t0 + tiles_q + ((int)blockIdx.x < tiles_r ? 1 : 0);
    const int n_groups = (t1 - t0 + T - 1) / T;
    // (t1 - t0) / n_groups without a division, which would stand between the kernel's start and its first loads:
    // with T = 3 the groups of two or more are of 2 or 3 tiles, of 3 only if all are
    static_assert(T == 3, "the group sizes below are those of T = 3");
    const int g_base = n_groups <= 1 ? t1 - t0 : (t1 - t0 == 3 * n_groups ? 3 : 2);
    const int g_rem = n_groups <= 1 ? 0 : t1 - t0 - g_base * n_groups;
    const int total = n_groups * n_chunks;   // chunks to go through, over all groups

    const int n_tiles_all = (N + 15) >> 4;
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(codes), 0, (int)((int64_t)(kPacked ? n_tiles_all * 16 : N) * row_bytes), 0x00020000);
    const int voff = kPacked ? lane * 16 : c16 * row_bytes + q * 16;
    constexpr int kOut = (int)0x80000000;
    // Scalar byte offset of the code word of (group g, chunk c, tile 0 of the group) for this wave, or the
    // out-of-range offset when the group or the wave's step of the chunk does not exist; tile t of the
    // group lies t * tile_stride further on.  Out of range: zeros, no memory access.
    const int tile_stride = kPacked ? n_steps * 1024 : 16 * row_bytes;
    auto chunk_offset = [&](int g, int c, int &gn) {
        const int gt0 = t0 + g * g_base + (g < g_rem ? g : g_rem), step = c * W + wave;
        gn = g < n_groups && step < n_steps ? g_base + (g < g_rem ? 1 : 0) : 0;
        return kPacked ? (gt0 * n_steps + step) * 1024 : gt0 * tile_stride + step * 64;
    };
    auto issue = [&](u4_t &cwd, int base, int gn, int t) {
        cwd = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff, t < gn ? base + t * tile_stride : kOut, 0);
    };
    // the ring: DC chunks deep, one slot per tile of the group
    u4_t cw[DC][T];
    {
        int g = 0, c = 0;
#pragma unroll
        for (int d = 0; d < DC; d++) {
            int gn;
            const int base = chunk_offset(g, c, gn);
#pragma unroll
            for (int t = 0; t < T; t++) issue(cw[d][t], base, gn, t);
            if (++c == n_chunks) { c = 0; g++; }
        }
    }

    // one piece of x -> its terms and means in buffer `buf` (piece p of the chunk); returns finite
    auto stage_piece = [&](const u4_t &v, int buf, int p) {
        u2_t tm[4];
        uint32_t mb;
        const bool fin = qc_split_piece(v, tm, mb);
        unsigned char *xb = xbuf + buf * kQcXBuf;
#pragma unroll
        for (int term = 0; term < 4; term++) *reinterpret_cast<u2_t *>(xb + term * kQcTermPitch + p * 8) = tm[term];
        reinterpret_cast<uint16_t *>(xb + 4 * kQcTermPitch)[p] = (uint16_t)mb;
        reinterpret_cast<uint16_t *>(xb + 4 * kQcTermPitch + kQcMeanPitch)[p] = (uint16_t)(mb >> 16);
        return fin;
    };

    bool fits = true;   // stays true while x is finite and the grid fits fp8
    if (wave >= 12) {
        // sign rows: 128 rows of 16 slots (16 bytes = two copies each); thread t of these 256 writes
        // 8 slots of row t / 2 (16 neighbouring lanes hit 16 different slot positions)
        const int t = tid - 768, row = t >> 1;
        if (t < 2) flags[16 + t] = 0u;
        const u2_t sb = sign_bytes((uint32_t)row);
        // slot i ^ (row % 8) of the thread's eight: one exclusive or per address
        const uint32_t sg = lds_addr(smem_raw) + (uint32_t)((row * 16 + (t & 1) * 8 + (row & 7)) * 16);
#pragma unroll
        for (int i = 0; i < 8; i++) lds_write16(sg ^ (uint32_t)(i * 16), u4_t{sb[0], sb[1], sb[0], sb[1]});
    } else if (wave >= 8) {
        bool exact;
        const u2_t g8 = grid_row_fp8(grow, exact);
        fits = exact;
        const int r = tid - 512;
        const uint32_t gg = lds_addr(smem_raw) + (uint32_t)(kSSignBytes + (r * 16 + (r & 15)) * 16);   // slot i ^ (r % 16)
#pragma unroll
        for (int i = 0; i < 16; i++) lds_write16(gg ^ (uint32_t)(i * 16), u4_t{g8[0], g8[1], g8[0], g8[1]});
    } else {
        fits = stage_piece(xpiece, 0, tid);
    }
    // the vote: every wave publishes whether something of its own failed, in a word of its own (so
    // nothing needs clearing first), and after the barrier every wave reads all of them
    {
        const bool wave_bad = __builtin_amdgcn_ballot_w64(!fits) != 0;
        if (lane == 0) flags[wave] = wave_bad ? 1u : 0u;
    }
    __syncthreads();
    // a grid value that does not fit 8 bits, or (here or in a later chunk) an x that is not finite: the
    // 16-bit kernel does the whole call over, at the end of this function
    bool hand_over = __builtin_amdgcn_ballot_w64(flags[lane & (W - 1)] != 0) != 0;

    // B operands of this lane: columns 0 .. 7 = term c16 % 4 of the first or the second MFMA's 32 bytes
    // of the wave's k step, columns 8 and 9 = the means (hi, lo); the other columns repeat 2 .. 7.
    // Wave w always does step w of a chunk, so the address only depends on the buffer.
    const bool mean_col = c16 == 8 || c16 == 9;
    const uint32_t xlane = lds_addr(xbuf) + (mean_col ? (uint32_t)(4 * kQcTermPitch + (c16 - 8) * kQcMeanPitch + q * 16 + wave * 64)
                                                      : (uint32_t)((c16 & 3) * kQcTermPitch + q * 64 + ((c16 >> 2) & 1) * 32 + wave * 256));

    f4_t acc[T][2], accd[T];
#pragma unroll
    for (int t = 0; t < T; t++) acc[t][0] = acc[t][1] = accd[t] = f4_t{0.f, 0.f, 0.f, 0.f};
    const float d_scale = c16 == 0 ? 1.f : c16 == 1 ? 8.f : 0.f;

    // With one or two chunks all of x stays resident once staged (chunk c in buffer c); longer x goes
    // through the two buffers in turn and is staged again for every group.
    const bool resident = n_chunks <= 2;
    int g = 0, c = 0;            // group and chunk of the chunk being multiplied
    int pg = 0, pc = 0;          // ... of the chunk DC further on, whose code words refill the slots
#pragma unroll
    for (int d = 0; d < DC; d++)
        if (++pc == n_chunks) { pc = 0; pg++; }
    bool barrier_in_group = true;   // the prologue's

    // one chunk; kSlot: its ring slot (static).  Every path issues exactly T code loads (tiles and
    // steps that do not exist load nothing and get zeros), so the wait counters stay exact.
    auto chunk = [&](auto slot_tag, int gc) {
        constexpr int kSlot = decltype(slot_tag)::value;
        const bool exists = DC == 1 || gc < total;   // only a second chunk of an unrolled pair may lie past the end
        const int gn = g_base + (g < g_rem ? 1 : 0);
        const int ntg = exists ? gn : 0;                          // tiles of this group (uniform)
        const bool last_c = c + 1 == n_chunks;
        const int xb_cur = resident ? c : gc & 1;
        // the chunk after this one: if its x is not in LDS yet, half of the waves split it while everybody
        // multiplies, waves 0-7 and 8-15 taking turns
        const int ng = last_c ? g + 1 : g, nc = last_c ? 0 : c + 1;
        const bool stage_next = exists && gc + 1 < total && (!resident || gc + 1 < n_chunks);
        const bool stager = stage_next && wave < 8;   // the waves the arbiter prefers: they are through their steps first
        const int sp = tid & 511;
        if (stager) {
            const int p = nc * 512 + sp;
            xpiece = p < n_pieces ? reinterpret_cast<const u4_t *>(x)[p] : u4_t{0u, 0u, 0u, 0u};
        }
        const bool step_ok = exists && c * W + wave < n_steps;
        int p_gn;                                                 // the refills: chunk DC further on
        const int p_base = chunk_offset(pg, pc, p_gn);
        u4_t x0 = u4_t{0u, 0u, 0u, 0u}, x1 = x0;
        if (step_ok) {
            const uint32_t xa = xlane + (uint32_t)(xb_cur * kQcXBuf);
            x0 = lds_read16(xa);
            x1 = lds_read16(xa + 16);
        }
        const i8_t xb = i8_t{(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
#pragma unroll
        for (int t = 0; t < T; t++) {
            if (step_ok && t < ntg) {   // uniform
                Q8Gather gt[4];
#pragma unroll
                for (int t2 = 0; t2 < 4; t2++) q8_gather(gt[t2], cw[kSlot][t][t2], lane_base);
                u4_t a8;   // +-2.0 per code, the shift term's A operand: the code words' shift bits over the bits of 2.0
#pragma unroll
                for (int i = 0; i < 4; i++) a8[i] = bfi(0x80008000u, cw[kSlot][t][i], 0x40004000u);
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const Q8Gather &b0 = gt[2 * h], &b1 = gt[2 * h + 1];
                    const i8_t a = i8_t{(int)(b0.g0[0] ^ b0.s0[0]), (int)(b0.g0[1] ^ b0.s0[1]), (int)(b0.g1[0] ^ b0.s1[0]),
                                        (int)(b0.g1[1] ^ b0.s1[1]), (int)(b1.g0[0] ^ b1.s0[0]), (int)(b1.g0[1] ^ b1.s0[1]),
                                        (int)(b1.g1[0] ^ b1.s1[0]), (int)(b1.g1[1] ^ b1.s1[1])};
                    acc[t][h] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, xb, acc[t][h], 0 /* A: fp8 */, 1 /* B: bf8 */, 0, 0, 0, 0);
                }
                accd[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8_t, a8), __builtin_bit_cast(h8_t, x0), accd[t], 0, 0, 0);
            }
            issue(cw[kSlot][t], p_base, p_gn, t);                  // the slot's next code word
        }
        if (stager && !stage_piece(xpiece, resident ? nc : (gc + 1) & 1, sp)) flags[16 + ((gc + 1) & 1)] = 1u;
        if (!exists) return;
        const bool group_end = last_c;
        if (group_end) {
            // `red` still holds the sums of the group before while its reducers read them: a barrier has
            // to lie between their read and this write
            if (!barrier_in_group) __syncthreads();
            // the group's partial sums: 4 columns per (wave, tile, quarter) - term t of the first MFMAs
            // (column t) plus term t of the second (column 4 + t); the shift term's columns 8 and 9 ride
            // in slots 0 and 1, the second times 8 to meet the weight 1/8 it gets from the reducer
#pragma unroll
            for (int t = 0; t < T; t++) {
                if (t >= ntg) break;
                f4_t v;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    v[e] = dpp_shl_add<4>(acc[t][0][e], acc[t][1][e]) + dpp_shl_add<8>(0.f, accd[t][e]) * d_scale;
                if (c16 < 4) red[wave * (T * 16 + 1) + (t * 4 + q) * 4 + c16] = v;
                acc[t][0] = acc[t][1] = accd[t] = f4_t{0.f, 0.f, 0.f, 0.f};
            }
        }
        barrier_in_group = !group_end && (barrier_in_group || stage_next);
        if (stage_next || group_end) {
            __syncthreads();   // hands the x buffers over and / or gathers the group's partial sums
            if (stage_next && __builtin_amdgcn_ballot_w64(flags[16 + ((gc + 1) & 1)] != 0) != 0) hand_over = true;
        }
        if (group_end && !hand_over && wave < ntg) {
            // wave t adds up tile t: lane (w, quarter) takes wave w's 4 columns with their weights 8^-c,
            // then the 16 lanes of a row are added with DPP shifts
            const f4_t *src = red + c16 * (T * 16 + 1) + (wave * 4 + q) * 4;
            f4_t v = src[0];
#pragma unroll
            for (int cc = 1; cc < 4; cc++) v += src[cc] * __builtin_bit_cast(float, 0x3F800000u - ((uint32_t)cc * 3u << 23));
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = row_sum16(v[e]);
            const int gt0 = t0 + g * g_base + (g < g_rem ? g : g_rem);
            const int n = (gt0 + wave) * 16 + 4 * q;
            if (c16 == 15 && n < N) {   // N % 4 == 0, so the four rows are in range together
                h4_t o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = (half_t)(v[e] * scale);
                *reinterpret_cast<h4_t *>(y + n) = o;
            }
        }
        if (++c == n_chunks) { c = 0; g++; }
        if (++pc == n_chunks) { pc = 0; pg++; }
    };

    for (int gc = 0; gc < total && !hand_over; gc += DC) {
        chunk(std::integral_constant<int, 0>{}, gc);
        if constexpr (DC > 1) {
            if (!hand_over) chunk(std::integral_constant<int, 1>{}, gc + 1);
        }
    }
    if (hand_over) {
        __syncthreads();   // everybody has read the flags before the LDS is laid out anew
        gemv_stream_body<1, W, 2, kPacked, 4>(x, codes, grid, scale, y, 1, N, K, tiles_q, tiles_r);
    }
}
