// Small-batch matrix-vector kernel with x in registers.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ small-batch matrix-vector path
// A few rows of x whose M * K does not fit in LDS beside the tables.  Same tables, same decode,
// same persistent workgroups as the streaming kernel; the difference is where B comes from: a
// wave fetches the x slice of its 256-wide k step from global memory (L2) together with the
// codes.  Because vector-memory results return in order, x and codes of a step travel as ONE
// prefetch unit (x first, then the codes), D units deep: an x load never waits behind codes that
// are needed later than it is.  All loads are raw buffer loads whose offset is out of range past
// the end (zeros, no memory access), so no branch surrounds them and the wait counters stay
// exact.
//
// How the x of a step reaches the lanes.  A lane's eight B fragments of a step are 128
// consecutive bytes of ITS row of x, so loading them fragment by fragment makes every load
// instruction touch 64 different cache lines for 16 bytes each, eight times over - at M = 16
// that cost as much as everything else in the kernel together.  Instead the slice of the step
// (16 rows x 512 bytes, fewer rows for M <= 8) is loaded in XI instructions whose 32 lanes per
// row take 512 consecutive bytes, written as loaded to an 8 KB piece of LDS that belongs to the
// wave alone, and read back in fragment order; the 16-byte pieces of row m are exchanged by
// m % 16 so that both the writes and the reads are free of bank conflicts without padding.  No
// other wave touches the piece while the wave is in its k steps, so this takes no barrier; at
// the end of a row block the same pieces carry the partial sums to the waves that add them up
// (a barrier before and one after).
//
// More than 16 rows of x: a row block is walked once per 16 rows (a pass), the accumulators
// being one tile of x wide, so the codes come from HBM once and from the caches after that.
template <int R>
__device__ __forceinline__ void regx_step(const u4_t (&cw)[R], const u4_t (&xb)[8], uint32_t lane_base,
                                          uint32_t quarter_bits, f4_t (&acc)[R][2], int nv)
{
    constexpr int kItems = 4 * R;
    StreamGather buf[2];
    stream_gather(buf[0], cw[0][0], lane_base, quarter_bits);
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int t2 = i / R, r = i % R;
        if (i + 1 < kItems) {
            const int nt2 = (i + 1) / R, nr = (i + 1) % R;
            if (nr == 0 || nr < nv) stream_gather(buf[(i + 1) & 1], cw[nr][nt2], lane_base, quarter_bits);
        }
        if (r == 0 || r < nv) {   // tiles past nv (uniform) belong to the next workgroup
            const StreamGather &b = buf[i & 1];
            const h8_t a0 = stream_finish<false>(b.g0, b.s0, b.dd);
            acc[r][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, __builtin_bit_cast(h8_t, xb[2 * t2]), acc[r][0], 0, 0, 0);
            const h8_t a1 = stream_finish<true>(b.g1, b.s1, b.dd);
            acc[r][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, __builtin_bit_cast(h8_t, xb[2 * t2 + 1]), acc[r][1], 0, 0, 0);
        }
    }
}

constexpr int kRegxPiece = 8192;   // LDS bytes of a wave's own piece: 16 rows x 512 bytes

// R: row tiles per block; W: waves; D: prefetch units in flight; XI: load instructions per slice
// (two rows each), 2, 4 or 8 for up to 4, 8 or 16 rows of x per pass (more than 16 rows: 8)
template <int R, int W, int D, bool kPacked, int XI>
__global__ __launch_bounds__(64 * W) void gemv_regx_kernel(const uint16_t *__restrict__ x,
                                                           const uint16_t *__restrict__ codes,
                                                           const void *__restrict__ grid, float scale,
                                                           uint16_t *__restrict__ y, int M, int N, int K,
                                                           int tiles_q, int tiles_r)
{
    static_assert(R >= 1 && R <= 4, "row tiles per block");
    static_assert(XI == 2 || XI == 4 || XI == 8, "4, 8 or 16 rows of x per pass");
    static_assert(R * kWave * 16 <= kRegxPiece, "the partial sums of a row block go through the wave's piece");
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15;
    const int q = lane >> 4;
    const int n_steps = K >> 8;
    const int row_bytes = K >> 2;
    const uint32_t lane_base = (uint32_t)c16 * 16u;
    const uint32_t quarter_bits = 0x34003400u;

    const u4_t grow = reinterpret_cast<const u4_t *>(grid)[tid & 255];

    const int n_sw = wave < n_steps ? (n_steps - wave + W - 1) / W : 0;
    // contiguous, balanced range of 16-row tiles per workgroup, as in the streaming kernel
    const int t0 = (int)blockIdx.x * tiles_q + ((int)blockIdx.x < tiles_r ? (int)blockIdx.x : tiles_r);
    const int t1 = t0 + tiles_q + ((int)blockIdx.x < tiles_r ? 1 : 0);
    const int nb_wg = (t1 - t0 + R - 1) / R;

    // row-major or packed codes, addressed as in the streaming kernel
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(codes), 0, (int)((int64_t)(kPacked ? ((N + 15) >> 4) * 16 : N) * row_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t xrsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(x), 0, M * K * 2, 0x00020000);
    constexpr int kOut = (int)0x80000000;
    int voff[R];
#pragma unroll
    for (int r = 0; r < R; r++) voff[r] = kPacked ? lane * 16 + r * n_steps * 1024 : (16 * r + c16) * row_bytes + q * 16;
    // load i of a step is piece lane % 32 of row 2 i + lane / 32 of the slice; pass p adds 16 p rows.
    // Rows past M lie past the end of the buffer: zeros, no memory access.
    int xcoff[XI];
#pragma unroll
    for (int i = 0; i < XI; i++) xcoff[i] = ((2 * i + (lane >> 5)) * K + (lane & 31) * 8) * 2;
    const int n_pass = (M + 15) >> 4;
    const int pass_bytes = 32 * K;
    // the wave's piece of LDS: row m at m * 512, its piece p in slot p ^ (m % 16).  Writes: row 2 i + h,
    // piece lane % 32, h = lane / 32, i.e. (xs_w ^ 32 i) + 1024 i.  Reads: row c16, piece 8 q + t, i.e.
    // xs_r ^ 16 t; lanes whose row is never written (c16 >= 2 XI) read row c16 % (2 XI): their columns
    // of the product are not stored.
    const uint32_t xs_piece = lds_addr(smem_raw) + (uint32_t)(kSTablesBytes + wave * kRegxPiece);
    const uint32_t xs_w = xs_piece + (uint32_t)((lane >> 5) * 512 + (((lane & 31) ^ (lane >> 5)) << 4));
    const int xr_row = c16 & (2 * XI - 1);
    const uint32_t xs_r = xs_piece + (uint32_t)(xr_row * 512 + (((8 * q) ^ xr_row) << 4));

    struct Unit {
        u4_t cw[R];
        u4_t xs[XI];   // the slice as loaded
    };
    // the prefetch walks blocks, passes and steps in the order the main loop uses them
    int pf_blk = 0, pf_pass = 0, pf_j = 0;
    auto issue = [&](Unit &u) {
        const bool ok = pf_blk < nb_wg && n_sw > 0;
        const int step = wave + pf_j * W;
        const int xs_off = ok ? step * 512 + pf_pass * pass_bytes : kOut;
        const int tb = t0 + pf_blk * R;
        const int soff = !ok ? kOut : kPacked ? (tb * n_steps + step) * 1024 : tb * 16 * row_bytes + step * 64;
#pragma unroll
        for (int i = 0; i < XI; i++) u.xs[i] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xcoff[i], xs_off, 0);
#pragma unroll
        for (int r = 0; r < R; r++)
            u.cw[r] = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff[r], (r == 0 || tb + r < t1) ? soff : kOut, 0);
        if (++pf_j >= n_sw) {
            pf_j = 0;
            if (++pf_pass >= n_pass) { pf_pass = 0; pf_blk++; }
        }
    };

    Unit ring[D];
#pragma unroll
    for (int d = 0; d < D; d++) issue(ring[d]);

    // tables (sign rows need no load; grid rows from the fetch above)
    {
        constexpr int kPerRow = 64 * W / 128, kCopies = 16 / kPerRow;
        u4_t *sg = reinterpret_cast<u4_t *>(smem_raw);
        const int srow = tid / kPerRow, sc0 = (tid % kPerRow) * kCopies;
        const u4_t sv = sign_row((uint32_t)srow);
#pragma unroll
        for (int i = 0; i < kCopies; i++) sg[srow * 16 + ((sc0 + i + srow) & 15)] = sv;   // 16 lanes, 16 bank groups
        constexpr int kCopiesPer = 4096 / (64 * W);
        u4_t *gg = reinterpret_cast<u4_t *>(smem_raw + kSSignBytes);
        const int row = tid & 255, c0 = (tid >> 8) * kCopiesPer;
#pragma unroll
        for (int i = 0; i < kCopiesPer; i++) gg[row * 16 + ((c0 + i + tid) & 15)] = grow;   // 16 lanes, 16 bank groups
    }
    __syncthreads();

    f4_t acc[R][2];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r][0] = acc[r][1] = f4_t{0.f, 0.f, 0.f, 0.f};

    // end of a pass over a row block: every wave leaves its partial sums in its own piece (row tile
    // r at lane l: byte (r * 64 + l) * 16), one barrier, then the first R waves add up one row tile
    // each and store it; a second barrier, because the pieces take the x of the next pass next
    auto finish_block = [&](int blk, int pass) {
        f4_t *own = reinterpret_cast<f4_t *>(smem_raw + kSTablesBytes + wave * kRegxPiece);
#pragma unroll
        for (int r = 0; r < R; r++) {
            own[r * kWave + lane] = acc[r][0] + acc[r][1];
            acc[r][0] = acc[r][1] = f4_t{0.f, 0.f, 0.f, 0.f};
        }
        __syncthreads();
        for (int r = wave; r < R; r += W) {
            const f4_t *src = reinterpret_cast<const f4_t *>(smem_raw + kSTablesBytes) + r * kWave + lane;
            f4_t sacc = src[0];
#pragma unroll
            for (int w = 1; w < W; w++) sacc += src[w * (kRegxPiece / 16)];
            const int m = 16 * pass + c16;
            const int rt = t0 + blk * R + r;
            const int n = rt * 16 + 4 * q;
            if (m < M && rt < t1 && n < N) {   // N % 4 == 0, so the four rows are in range together
                h4_t o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = (half_t)(sacc[e] * scale);
                *reinterpret_cast<h4_t *>(y + (int64_t)m * N + n) = o;
            }
        }
        __syncthreads();
    };

    if (n_sw == 0) {
        for (int blk = 0; blk < nb_wg; blk++)
            for (int pass = 0; pass < n_pass; pass++) finish_block(blk, pass);
        return;
    }
    const int n_items = nb_wg * n_pass * n_sw;
    int blk = 0, pass = 0, j = 0;
    for (int i0 = 0; i0 < n_items; i0 += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (i0 + d < n_items) {
                // the slice through the wave's piece: in as loaded, out as fragments
#pragma unroll
                for (int i = 0; i < XI; i++) lds_write16((xs_w ^ (uint32_t)(32 * i)) + (uint32_t)(1024 * i), ring[d].xs[i]);
                u4_t xf[8];
#pragma unroll
                for (int t = 0; t < 8; t++) xf[t] = lds_read16(xs_r ^ (uint32_t)(16 * t));
                regx_step<R>(ring[d].cw, xf, lane_base, quarter_bits, acc, t1 - (t0 + blk * R));
                if (++j >= n_sw) {
                    j = 0;
                    finish_block(blk, pass);
                    if (++pass >= n_pass) { pass = 0; blk++; }
                }
            }
            issue(ring[d]);
        }
    }
}
