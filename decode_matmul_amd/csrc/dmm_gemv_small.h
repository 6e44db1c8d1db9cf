// Small-batch matrix-vector kernel with x in registers.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ small-batch matrix-vector path
// M <= 32 when x does not fit in LDS beside the tables (M * K too large).  Same tables, same
// decode, same persistent workgroups and split-K as the streaming kernel; the difference is
// where B comes from: x is read from global memory (L2) into registers, one 256-wide step at
// a time.  Because vector-memory results return in order, x and codes of a step travel as ONE
// prefetch unit (x first, then the codes), D units deep: an x load never waits behind codes
// that are needed later than it is.  All loads are raw buffer loads whose offset is out of
// range past the end (zeros, no memory access), so no branch surrounds them and the wait
// counters stay exact.  MT = number of 16-row tiles of x (M <= 16 * MT).
//
// How the x of a step reaches the lanes.  A lane's eight B fragments of a step are 128
// consecutive bytes of ITS row of x, so loading them fragment by fragment makes every load
// instruction touch 64 different cache lines for 16 bytes each, eight times over - at M = 16
// that cost as much as everything else in the kernel together.  With XI > 0 (M <= 2 XI <= 16)
// the slice of the step (M rows x 512 bytes) is instead loaded in XI instructions whose 32
// lanes per row take 512 consecutive bytes, written as loaded to an 8 KB piece of LDS that
// belongs to the wave alone, and read back in fragment order; the 16-byte pieces of row m are
// exchanged by m % 16 so that both the writes and the reads are free of bank conflicts without
// padding.  No other wave touches the piece while the wave is in its k steps, so this takes no
// barrier; at the end of a row block the same pieces carry the partial sums to the waves
// that add them up (a barrier before and one after).  XI = 0: fragment loads (M = 17 .. 32).
template <int R, int MT>
__device__ __forceinline__ void regx_step(const u4_t (&cw)[R], const u4_t (&xb)[MT][8], uint32_t lane_base,
                                          uint32_t quarter_bits, f4_t (&acc)[R][MT][2], int nv)
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
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
                acc[r][mt][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, __builtin_bit_cast(h8_t, xb[mt][2 * t2]), acc[r][mt][0], 0, 0, 0);
            const h8_t a1 = stream_finish<true>(b.g1, b.s1, b.dd);
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
                acc[r][mt][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, __builtin_bit_cast(h8_t, xb[mt][2 * t2 + 1]), acc[r][mt][1], 0, 0, 0);
        }
    }
}

constexpr int kRegxPiece = 8192;   // LDS bytes of a wave's own piece (XI > 0): 16 rows x 512 bytes

template <int R, int W, int MT, int D, bool kPacked, int XI = 0>
__global__ __launch_bounds__(64 * W) void gemv_regx_kernel(const uint16_t *__restrict__ x,
                                                           const uint16_t *__restrict__ codes,
                                                           const void *__restrict__ grid, float scale,
                                                           uint16_t *__restrict__ y, int M, int N, int K,
                                                           int tiles_q, int tiles_r)
{
    static_assert(R >= 1 && R <= 4, "row tiles per block");
    static_assert(XI == 0 || (MT == 1 && (XI == 2 || XI == 4 || XI == 8)), "coalesced x: one tile of x, 4, 8 or 16 rows");
    static_assert(XI == 0 || R * kWave * 16 <= kRegxPiece, "the partial sums of a row block go through the wave's piece");
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];
    typedef f4_t red_t[W][R * MT][kWave];
    red_t *red = reinterpret_cast<red_t *>(smem_raw + kSTablesBytes);   // red[parity] (XI == 0)

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
    int voff[R], xoff[MT];
#pragma unroll
    for (int r = 0; r < R; r++) voff[r] = kPacked ? lane * 16 + r * n_steps * 1024 : (16 * r + c16) * row_bytes + q * 16;
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        const int m = 16 * mt + c16;
        xoff[mt] = m < M ? (m * K + 64 * q) * 2 : kOut;   // columns past M: zeros, no memory access
    }
    // XI > 0: load i of a step is piece lane % 32 of row 2 i + lane / 32 of the slice
    constexpr int kXs = XI > 0 ? XI : 1;
    int xcoff[kXs];
#pragma unroll
    for (int i = 0; i < kXs; i++) {
        const int m = 2 * i + (lane >> 5);
        xcoff[i] = m < M ? (m * K + (lane & 31) * 8) * 2 : kOut;   // rows past M: zeros, no memory access
    }
    // the wave's piece of LDS: row m at m * 512, its piece p in slot p ^ (m % 16).  Writes: row 2 i + h,
    // piece lane % 32, h = lane / 32, i.e. (xs_w ^ 32 i) + 1024 i.  Reads: row c16, piece 8 q + t, i.e.
    // xs_r ^ 16 t; lanes whose row is never written (c16 >= 2 XI) read row c16 % (2 XI): their columns
    // of the product are not stored.
    const uint32_t xs_piece = lds_addr(smem_raw) + (uint32_t)(kSTablesBytes + wave * kRegxPiece);
    const uint32_t xs_w = xs_piece + (uint32_t)((lane >> 5) * 512 + (((lane & 31) ^ (lane >> 5)) << 4));
    const int xr_row = XI > 0 ? c16 & (2 * XI - 1) : c16;
    const uint32_t xs_r = xs_piece + (uint32_t)(xr_row * 512 + (((8 * q) ^ xr_row) << 4));

    struct Unit {
        u4_t cw[R];
        u4_t xb[XI > 0 ? 1 : MT][XI > 0 ? XI : 8];   // XI > 0: the slice as loaded; else the fragments
    };
    int pf_blk = 0, pf_j = 0;
    auto issue = [&](Unit &u) {
        const bool ok = pf_blk < nb_wg && n_sw > 0;
        const int step = wave + pf_j * W;
        const int xs_off = ok ? step * 512 : kOut;
        const int tb = t0 + pf_blk * R;
        const int soff = !ok ? kOut : kPacked ? (tb * n_steps + step) * 1024 : tb * 16 * row_bytes + step * 64;
        if constexpr (XI > 0) {
#pragma unroll
            for (int i = 0; i < XI; i++) u.xb[0][i] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xcoff[i], xs_off, 0);
        } else {
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int t = 0; t < 8; t++)
                    u.xb[mt][t] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xoff[mt] + t * 16, xs_off, 0);
        }
#pragma unroll
        for (int r = 0; r < R; r++)
            u.cw[r] = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff[r], (r == 0 || tb + r < t1) ? soff : kOut, 0);
        if (++pf_j >= n_sw) { pf_j = 0; pf_blk++; }
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

    f4_t acc[R][MT][2];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[r][mt][0] = acc[r][mt][1] = f4_t{0.f, 0.f, 0.f, 0.f};

    // end of a row block: partial sums to LDS (double-buffered per block), one barrier, then
    // the first R * MT waves add up one (row tile, m tile) each and store it
    auto finish_block = [&](int blk) {
        const int par = blk & 1;
        // XI > 0: wave w's sums of row tile r at lane l sit at piece w, byte (r * 64 + l) * 16
        f4_t *own = reinterpret_cast<f4_t *>(smem_raw + kSTablesBytes + wave * kRegxPiece);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                if constexpr (XI > 0) own[r * kWave + lane] = acc[r][mt][0] + acc[r][mt][1];
                else red[par][wave][r * MT + mt][lane] = acc[r][mt][0] + acc[r][mt][1];
                acc[r][mt][0] = acc[r][mt][1] = f4_t{0.f, 0.f, 0.f, 0.f};
            }
        __syncthreads();
        for (int tile = wave; tile < R * MT; tile += W) {
            f4_t sacc;
            if constexpr (XI > 0) {
                const f4_t *src = reinterpret_cast<const f4_t *>(smem_raw + kSTablesBytes) + tile * kWave + lane;
                sacc = src[0];
#pragma unroll
                for (int w = 1; w < W; w++) sacc += src[w * (kRegxPiece / 16)];
            } else {
                sacc = red[par][0][tile][lane];
#pragma unroll
                for (int w = 1; w < W; w++) sacc += red[par][w][tile][lane];
            }
            const int r = tile / MT, mt = tile % MT;
            const int m = 16 * mt + c16;
            const int rt = t0 + blk * R + r;
            const int n = rt * 16 + 4 * q;
            if (m < M && rt < t1 && n < N) {   // N % 4 == 0, so the four rows are in range together
                h4_t o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = (half_t)(sacc[e] * scale);
                *reinterpret_cast<h4_t *>(y + (int64_t)m * N + n) = o;
            }
        }
        // the pieces take the x of the next row block next: not before the sums have been read
        if constexpr (XI > 0) __syncthreads();
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
                if constexpr (XI > 0) {
                    // the slice through the wave's piece: in as loaded, out as fragments
#pragma unroll
                    for (int i = 0; i < XI; i++) lds_write16((xs_w ^ (uint32_t)(32 * i)) + (uint32_t)(1024 * i), ring[d].xb[0][i]);
                    u4_t xf[1][8];
#pragma unroll
                    for (int t = 0; t < 8; t++) xf[0][t] = lds_read16(xs_r ^ (uint32_t)(16 * t));
                    regx_step<R, 1>(ring[d].cw, xf, lane_base, quarter_bits, acc, t1 - (t0 + blk * R));
                } else {
                    regx_step<R, MT>(ring[d].cw, ring[d].xb, lane_base, quarter_bits, acc, t1 - (t0 + blk * R));
                }
                if (++j >= n_sw) {
                    j = 0;
                    finish_block(blk);
                    blk++;
                }
            }
            issue(ring[d]);
        }
    }
}
