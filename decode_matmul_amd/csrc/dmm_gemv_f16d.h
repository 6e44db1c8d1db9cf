// Up to 32 rows of x on 16-bit operands with x taken a k step at a time and every tile of a workgroup in registers.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ 16-bit operands, x by the k step, resident accumulators
// The streaming kernel keeps all of x in the LDS beside the tables, which stops at M * (2 K + 16) = 64 KB:
// four rows of K = 8192, two of K = 28672 no longer fit, and such calls went to the small-batch kernel with its
// eight waves, its row blocks of four tiles and its x slices fetched again for every block.  This kernel has
// the streaming kernel's tables, decode and MFMA (one code = two 16-byte gathers, four packed FMAs, one
// v_mfma_f32_16x16x32_f16 whose B column m is row m of x) and the loop order of the batch-1 kernel on 8-bit
// operands:
//   * a chunk of x is W = 16 k steps (8 for nine to sixteen rows of x), one per wave, and a wave only ever needs its own: the slice of its k step (up
//     to 2 XI rows of 512 bytes) is loaded in XI instructions whose 32 lanes per row take 512 consecutive bytes,
//     written as loaded into a piece of LDS that belongs to the wave alone and read back as the eight B
//     operands of a tile step (the 16-byte pieces of row m exchanged by m, so that writes and reads meet no
//     bank conflict), which then serve every tile of the workgroup.  No wave touches another's piece, so x
//     takes no barrier; the slice of the next chunk is asked for before the tile steps of this one.
//   * chunk outside, tiles inside: the accumulators of all NT tiles of the workgroup's share stay in registers
//     for the whole launch (one per tile: a second one to alternate the MFMAs between bought nothing, and
//     with one the sums do not depend on how many tiles a workgroup has), and the code stream is a ring of D
//     loads per wave over the items (chunk, tile).
//   * at the end every wave leaves its accumulators' columns 0 .. 2 XI - 1 (the rows of x) in its own piece,
//     and after the launch's one other barrier wave t adds tile t up over the W waves by DPP and stores y.
// Any grid of finite halves, any x: the arithmetic is the streaming kernel's (fp32 sums of exact products),
// only the order of the sums differs.
// LDS map: tables [0, 96K), then W pieces of XI KB.
__host__ __device__ constexpr int fd_lds_bytes(int XI, int W = 16) { return kSTablesBytes + W * XI * 1024; }

// One tile's 256-wide k step: 8 codes of the lane -> 16 gathers, 32 packed FMAs, 8 MFMAs into acc.  kAhead: the
// gathers of a code word are issued before the arithmetic of the word before it (17 more registers, which the
// instances with many tiles do not have).
template <bool kAhead, int CG>
__device__ __forceinline__ void fd_tile_step(const u4_t &cw, uint32_t lane_base, uint32_t quarter_bits,
                                             const u4_t (&xb)[CG][8], f4_t (&acc)[CG])
{
    StreamGather buf[kAhead ? 2 : 1];
    stream_gather(buf[0], cw[0], lane_base, quarter_bits);
#pragma unroll
    for (int t2 = 0; t2 < 4; t2++) {
        if (kAhead && t2 + 1 < 4) stream_gather(buf[(t2 + 1) & 1], cw[t2 + 1], lane_base, quarter_bits);
        const StreamGather &b = buf[kAhead ? t2 & 1 : 0];
        const h8_t a0 = stream_finish<false>(b.g0, b.s0, b.dd);
#pragma unroll
        for (int g = 0; g < CG; g++)
            acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, __builtin_bit_cast(h8_t, xb[g][2 * t2]), acc[g], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        const h8_t a1 = stream_finish<true>(b.g1, b.s1, b.dd);
#pragma unroll
        for (int g = 0; g < CG; g++)
            acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, __builtin_bit_cast(h8_t, xb[g][2 * t2 + 1]), acc[g], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (!kAhead && t2 + 1 < 4) stream_gather(buf[0], cw[t2 + 1], lane_base, quarter_bits);
    }
}

// XI: load instructions per slice of x, two rows each: 2 for up to four rows, 4 for up to eight, 8 for up to sixteen.
// W: waves, i.e. k steps per chunk: 16, or 8 where sixteen pieces of 8 KB would not fit beside the tables.
// CG: groups of sixteen rows of x (1, or 2 for 17 to 32 rows): one decode of a code feeds an MFMA per group, the
// slices of the groups go through the wave's piece one after the other, and so do the sums at the end.
template <int NT, int U, int D, bool kPacked, int XI, int W = 16, int CG = 1>
__global__ __launch_bounds__(64 * W) void gemv_f16d_kernel(const uint16_t *__restrict__ x,
                                                         const uint16_t *__restrict__ codes,
                                                         const void *__restrict__ grid, float scale,
                                                         uint16_t *__restrict__ y, int M, int N, int K, int tiles_q,
                                                         int tiles_r)
{
    constexpr int CM = 2 * XI;          // columns of the product that can hold a row of x
    constexpr int kPiece = XI * 1024;   // bytes of a wave's own piece: CM rows x 512 bytes
    static_assert((W == 16 && (XI == 2 || XI == 4)) || (W == 8 && XI == 8), "up to four, eight or sixteen rows of x");
    static_assert(CG == 1 || (CG == 2 && XI == 8), "a second group of rows only beside a full first one");
    static_assert(fd_lds_bytes(XI, W) <= 160 * 1024, "tables and pieces have to fit the LDS");
    // sixteen waves: 8 tiles, or 6 with eight rows of x, leave no registers for it
    constexpr bool kAhead = W == 8 || (NT < 8 && !(NT >= 6 && XI == 4));
    static_assert((U * NT) % D == 0, "the ring has to divide the unrolled loop");
    static_assert(NT * 4 * CM * 16 <= kPiece, "the partial sums of the end go through the wave's piece");
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15;
    const int q = lane >> 4;
    const int n_steps = K >> 8;
    const int n_chunks = (n_steps + W - 1) / W;
    const int row_bytes = K >> 2;
    const uint32_t lane_base = (uint32_t)c16 * 16u;
    const uint32_t quarter_bits = 0x34003400u;

    // ---- prologue: the grid row of the first 256 threads and the wave's slice of the first chunk, then one code word
    const u4_t grow = tid < 256 ? reinterpret_cast<const u4_t *>(grid)[tid] : u4_t{0u, 0u, 0u, 0u};
    // load i of a slice is piece lane % 32 (16 bytes) of row 2 i + lane / 32; rows past M lie past the end of the
    // buffer (zeros, no memory access), and so does the slice of a k step that does not exist
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(x), 0, M * K * 2, 0x00020000);
    constexpr int kOut = (int)0x80000000;
    // load i: 4 i K bytes further on, in the scalar offset (recomputed where it is used: a register less to hold)
    auto x_voff = [&]() { return (((int)threadIdx.x >> 5 & 1) * K + ((int)threadIdx.x & 31) * 8) * 2; };
    auto x_soff = [&](int c, int i) { return c * W + wave < n_steps ? (c * W + wave) * 512 + i * 4 * K : kOut; };   // i: pair of rows
    u4_t xv[CG][XI];
#pragma unroll
    for (int g = 0; g < CG; g++)
#pragma unroll
        for (int i = 0; i < XI; i++) xv[g][i] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, x_voff(), x_soff(0, g * 8 + i), 0);
    // the wave's piece: row m at m * 512, its piece p in slot p ^ m.  Writes: row 2 i + h, piece lane % 32,
    // h = lane / 32, i.e. (xs_w ^ 32 i) + 1024 i.  Reads: row c16, piece 8 q + t, i.e. xs_r ^ 16 t; lanes whose row
    // is never written (c16 >= CM) read row c16 % CM: their columns of the product are not stored.
    const uint32_t piece = lds_addr(smem_raw) + (uint32_t)(kSTablesBytes + wave * kPiece);
    auto xs_w = [&]() { return piece + (uint32_t)((lane >> 5) * 512 + (((lane & 31) ^ (lane >> 5)) << 4)); };
    const int xr_row = c16 & (CM - 1);
    const uint32_t xs_r = piece + (uint32_t)(xr_row * 512 + (((8 * q) ^ xr_row) << 4));

    const int t0 = (int)blockIdx.x * tiles_q + ((int)blockIdx.x < tiles_r ? (int)blockIdx.x : tiles_r);
    const int nt = tiles_q + ((int)blockIdx.x < tiles_r ? 1 : 0);   // <= NT (the host's business)

    const int n_tiles_all = (N + 15) >> 4;
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(codes), 0, (int)((int64_t)(kPacked ? n_tiles_all * 16 : N) * row_bytes), 0x00020000);
    const int voff = kPacked ? lane * 16 : c16 * row_bytes + q * 16;
    const int tile_stride = kPacked ? n_steps * 1024 : 16 * row_bytes;
    const int step_stride = kPacked ? 1024 : 64;
    const int tile0_off = t0 * tile_stride;
    // the code word of (chunk c, tile t) for this wave; out of range when the tile or the step does not exist
    auto issue = [&](u4_t &cwd, int c, int t) {
        const int step = c * W + wave;
        const bool ok = t < nt && step < n_steps;
        cwd = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff, ok ? tile0_off + t * tile_stride + step * step_stride : kOut, 0);
    };
    u4_t cw[D];
    // one item ahead of the prologue's work, the rest of the ring after it (a code load queued ahead of the
    // grid load delays the tables by the time the memory pipeline takes it apart)
    issue(cw[0], 0, 0);

    stream_stage_signs<64 * W>(smem_raw, tid);
    __builtin_amdgcn_sched_barrier(0);   // keep the sign rows ahead of the waits for the loads
    stream_stage_grid<64 * W>(smem_raw, grow, tid);
#pragma unroll
    for (int d = 1; d < D; d++) issue(cw[d], d / NT, d % NT);
    __syncthreads();

    f4_t acc[NT][CG];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int g = 0; g < CG; g++) acc[t][g] = f4_t{0.f, 0.f, 0.f, 0.f};

    for (int c0 = 0; c0 < n_chunks; c0 += U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = c0 + u;
            const bool step_ok = (U == 1 || c < n_chunks) && c * W + wave < n_steps;
            // the slice through the wave's piece: in as loaded, out as the B operands of the eight MFMAs
            // (the LDS serves a wave's instructions in order: the second group's slice may follow the first one's reads)
            u4_t xb[CG][8];
#pragma unroll
            for (int g = 0; g < CG; g++) {
#pragma unroll
                for (int i = 0; i < XI; i++) lds_write16((xs_w() ^ (uint32_t)(32 * i)) + (uint32_t)(1024 * i), xv[g][i]);
#pragma unroll
                for (int i = 0; i < 8; i++) xb[g][i] = lds_read16(xs_r ^ (uint32_t)(16 * i));
#pragma unroll
                for (int i = 0; i < XI; i++)
                    xv[g][i] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, x_voff(), x_soff(c + 1, g * 8 + i), 0);
            }
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int slot = (u * NT + t) % D;
                if (step_ok && t < nt) fd_tile_step<kAhead, CG>(cw[slot], lane_base, quarter_bits, xb, acc[t]);
                issue(cw[slot], c + (t + D) / NT, (t + D) % NT);   // the item D further on
            }
        }
    }
    // the sums of every tile into the wave's own piece, a group of rows at a time: cell (tile, quarter, column) at
    // slot cell ^ wave, so that the 16 lanes of a reader, one per wave, meet no bank conflict
#pragma unroll
    for (int g = 0; g < CG; g++) {
        if (g > 0) __syncthreads();   // the readers of the group before are done with the pieces
#pragma unroll
        for (int t = 0; t < NT; t++)
            if (t < nt && c16 < CM)
                lds_write16(piece + (uint32_t)(((((t * 4 + q) * CM + c16) ^ wave)) << 4), __builtin_bit_cast(u4_t, acc[t][g]));
        __syncthreads();
        if (wave < nt) {
            // wave t adds up tile t: lane (w, quarter) takes wave w's sums of the quarter's four rows for each
            // row of x (nothing where there is no wave w), then the 16 lanes of a row are added with DPP shifts
            const uint32_t src = lds_addr(smem_raw) + (uint32_t)(kSTablesBytes + (c16 & (W - 1)) * kPiece);
            const int n = (t0 + wave) * 16 + 4 * q;
#pragma unroll
            for (int m = 0; m < CM; m++) {
                f4_t v = __builtin_bit_cast(f4_t, lds_read16(src + (uint32_t)(((((wave * 4 + q) * CM + m) ^ (c16 & (W - 1)))) << 4)));
                if (W < 16 && c16 >= W) v = f4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = row_sum16(v[e]);
                if (c16 == 15 && g * 16 + m < M && n < N) {   // N % 4 == 0, so the four rows are in range together
                    h4_t o;
#pragma unroll
                    for (int e = 0; e < 4; e++) o[e] = (half_t)(v[e] * scale);
                    *reinterpret_cast<h4_t *>(y + (int64_t)(g * 16 + m) * N + n) = o;
                }
            }
        }
    }
}
