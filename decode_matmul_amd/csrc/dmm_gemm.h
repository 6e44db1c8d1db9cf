// Matrix-matrix kernels (prefill): the LDS-tiled kernel, the kernel that decodes weights straight
// into MFMA operand registers, and the split-K reduction.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ matrix-matrix path
// Block tile BN (n) x BM (m) x 64 (k) with WN x WM waves, each wave TN x TM tiles of
// v_mfma_f32_32x32x16_f16 (A = decoded W rows, B = x rows, fp32 accumulate).  A wide n keeps
// x re-reads down (x is fetched once per BN output columns) and a tall m amortises the decode.
//
// The k loop is software-pipelined three deep so that the matrix unit never waits for
// staging: while the MFMAs of tile kt run out of LDS buffer kt%2, the same waves decode tile
// kt+1 (whose codes and x already sit in registers) into buffer (kt+1)%2 - a quarter of that
// work after each group of MFMAs, in the matrix unit's shadow - and the global loads of tiles
// kt+2 .. kt+4 are in flight.  One barrier per k tile.  LDS rows are 144 bytes apart (9 bank groups),
// so the 16 lanes the LDS serves per clock - 16 consecutive rows at the same k - hit 16
// different groups.
constexpr int kGemmBK = 64;
constexpr int kGemmLd = kGemmBK + 8;   // halves per LDS row

template <int WN, int WM, int TN, int TM>
struct GemmCfg {
    static constexpr int kThreads = 64 * WN * WM;
    static constexpr int kBN = WN * TN * 32;
    static constexpr int kBM = WM * TM * 32;
    static constexpr int kTPR = kThreads / kBN;            // threads sharing one W row (1 or 2)
    static constexpr int kCPT = 8 / kTPR;                  // codes per thread per k tile
    static constexpr int kXPT = kBM * 8 / kThreads;        // 16-byte pieces of x per thread per k tile
    static constexpr int kXTPR = 8 / kXPT;                 // threads sharing one x row
    static_assert(kTPR == 1 || kTPR == 2, "one or two threads per W row");
    static_assert(kXPT >= 1 && kXPT <= 8 && 8 % kXPT == 0, "x pieces per thread");
    struct Shared {
        DecodeTables tab;
        uint16_t w[2][kBN][kGemmLd];
        uint16_t x[2][kBM][kGemmLd];
    };
};

// decode of one code with the packed delta taken from the low / high half of dd
template <bool kHi>
__device__ __forceinline__ u4_t gemm_decode(uint32_t code, uint32_t dd, const DecodeTables &t)
{
    const u4_t g = t.grid[code & 0xFFu];
    const u4_t sg = t.sign[(code >> 8) & 0x7Fu];
    u4_t r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = pk_fma_bcast<kHi>(g[i], sg[i], dd);
    return r;
}

template <int WN, int WM, int TN, int TM>
__global__ __launch_bounds__(64 * WN * WM) void gemm_kernel(const uint16_t *__restrict__ x,
                                                            const uint16_t *__restrict__ codes,
                                                            const void *__restrict__ grid, float scale,
                                                            uint16_t *__restrict__ y, int M, int N, int K, int y_vec)
{
    typedef GemmCfg<WN, WM, TN, TM> C;
    extern __shared__ __attribute__((aligned(16))) unsigned char gemm_smem[];
    typename C::Shared &sh = *reinterpret_cast<typename C::Shared *>(gemm_smem);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave % WN, wm = wave / WN;
    const int n0 = blockIdx.x * C::kBN;
    const int m0 = blockIdx.y * C::kBM;
    const int k_tiles = K / kGemmBK;
    const int64_t kc = K >> 3;

    stage_tables<true>(sh.tab, grid, tid, C::kThreads);

    // W staging: thread -> row tid / kTPR, kCPT codes of the k tile
    const int w_row = tid / C::kTPR, w_part = tid % C::kTPR;
    int wr = n0 + w_row;
    wr = wr < N ? wr : N - 1;
    const uint16_t *wsrc = codes + (int64_t)wr * kc + w_part * C::kCPT;
    // x staging: thread -> row tid / kXTPR, kXPT pieces of 8 halves
    const int x_row = tid / C::kXTPR, x_part = tid % C::kXTPR;
    int xr = m0 + x_row;
    const bool x_in = xr < M;
    xr = x_in ? xr : M - 1;
    const uint16_t *xsrc = x + (int64_t)xr * K + x_part * C::kXPT * 8;

    struct Stage {
        uint32_t cw[C::kCPT / 2];
        u4_t xv[C::kXPT];
    };
    auto load_tile = [&](Stage &st, int kt) {
        kt = kt < k_tiles ? kt : k_tiles - 1;    // past the end: reload the last tile (never used)
        const uint32_t *wp = reinterpret_cast<const uint32_t *>(wsrc + (int64_t)kt * 8);
        if (C::kCPT == 8) {
            const u4_t v = *reinterpret_cast<const u4_t *>(wp);
#pragma unroll
            for (int i = 0; i < C::kCPT / 2; i++) st.cw[i] = v[i];
        } else {
            const u2_t v = *reinterpret_cast<const u2_t *>(wp);
#pragma unroll
            for (int i = 0; i < C::kCPT / 2; i++) st.cw[i] = v[i];
        }
#pragma unroll
        for (int i = 0; i < C::kXPT; i++) st.xv[i] = reinterpret_cast<const u4_t *>(xsrc + (int64_t)kt * kGemmBK)[i];
    };
    // One quarter (q = 0..3) of a thread's staging work for LDS buffer `buf`, in two halves:
    // the table gathers are issued before a group of MFMAs, the packed FMAs and the LDS writes
    // run after it, in the matrix unit's shadow.
    constexpr int kCq = C::kCPT / 4;             // codes per quarter: 1 or 2
    struct Gathered {
        u4_t g[kCq], sg[kCq];
    };
    auto stage_gather = [&](Gathered &o, const Stage &st, int q) {
#pragma unroll
        for (int c = 0; c < kCq; c++) {
            const int ci = q * kCq + c;          // code index within the thread's kCPT
            const uint32_t code = (ci & 1) ? st.cw[ci >> 1] >> 16 : st.cw[ci >> 1];
            o.g[c] = sh.tab.grid[code & 0xFFu];
            o.sg[c] = sh.tab.sign[(code >> 8) & 0x7Fu];
        }
    };
    auto stage_finish = [&](const Gathered &o, const Stage &st, int buf, int q) {
#pragma unroll
        for (int c = 0; c < kCq; c++) {
            const int ci = q * kCq + c;
            const uint32_t dd = (st.cw[ci >> 1] & 0x80008000u) | 0x34003400u;
            u4_t wv;
#pragma unroll
            for (int i = 0; i < 4; i++)
                wv[i] = (ci & 1) ? pk_fma_bcast<true>(o.g[c][i], o.sg[c][i], dd) : pk_fma_bcast<false>(o.g[c][i], o.sg[c][i], dd);
            *reinterpret_cast<u4_t *>(&sh.w[buf][w_row][(w_part * C::kCPT + ci) * 8]) = wv;
        }
        const u4_t zero = u4_t{0u, 0u, 0u, 0u};
        if (C::kXPT >= 4) {
#pragma unroll
            for (int i = 0; i < C::kXPT / 4; i++) {
                const int pi = q * (C::kXPT / 4) + i;
                *reinterpret_cast<u4_t *>(&sh.x[buf][x_row][(x_part * C::kXPT + pi) * 8]) = x_in ? st.xv[pi] : zero;
            }
        } else if (q < C::kXPT) {
            *reinterpret_cast<u4_t *>(&sh.x[buf][x_row][(x_part * C::kXPT + q) * 8]) = x_in ? st.xv[q] : zero;
        }
    };

    // ring of four stages: tile kt+1 is staged out of ring[(kt+1)%4] while tile kt+4 is fetched
    // into ring[kt%4], so a global load has three tiles of MFMAs to arrive
    Stage ring[4];
#pragma unroll
    for (int i = 0; i < 4; i++) load_tile(ring[i], i);

    f16_t acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    const int l32 = lane & 31, kq = lane >> 5;
    __syncthreads();   // tables ready
#pragma unroll
    for (int q = 0; q < 4; q++) {
        Gathered gq;
        stage_gather(gq, ring[0], q);
        stage_finish(gq, ring[0], 0, q);
    }
    __syncthreads();   // tile 0 staged

    // Compute tile kt from buffer `buf` while staging tile kt+1 (registers sn) into the other
    // buffer and fetching tile kt+4 into sf.  Operand fragments are double-buffered in
    // registers: those of k step ks+1 are requested before the MFMAs of step ks are issued.
    auto read_frags = [&](h8_t (&a)[TN], h8_t (&b)[TM], int buf, int ks) {
#pragma unroll
        for (int i = 0; i < TN; i++)
            a[i] = *reinterpret_cast<const h8_t *>(&sh.w[buf][(wn * TN + i) * 32 + l32][ks * 16 + kq * 8]);
#pragma unroll
        for (int j = 0; j < TM; j++)
            b[j] = *reinterpret_cast<const h8_t *>(&sh.x[buf][(wm * TM + j) * 32 + l32][ks * 16 + kq * 8]);
    };
    auto tile = [&](int kt, int buf, const Stage &sn, Stage &sf) {
        const bool staging = kt + 1 < k_tiles;
        load_tile(sf, kt + 4);
        h8_t a[2][TN], b[2][TM];
        read_frags(a[0], b[0], buf, 0);
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            if (ks < 3) read_frags(a[(ks + 1) & 1], b[(ks + 1) & 1], buf, ks + 1);
            Gathered gq;
            if (staging) stage_gather(gq, sn, ks);
#pragma unroll
            for (int i = 0; i < TN; i++)
#pragma unroll
                for (int j = 0; j < TM; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ks & 1][i], b[ks & 1][j], acc[i][j], 0, 0, 0);
            if (staging) stage_finish(gq, sn, buf ^ 1, ks);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    };

    for (int kt = 0; kt < k_tiles; kt += 4) {
        tile(kt, 0, ring[1], ring[0]);
        if (kt + 1 < k_tiles) tile(kt + 1, 1, ring[2], ring[1]);
        if (kt + 2 < k_tiles) tile(kt + 2, 0, ring[3], ring[2]);
        if (kt + 3 < k_tiles) tile(kt + 3, 1, ring[0], ring[3]);
    }

    // D layout of 32x32: element e of lane: row (n) = 8*(e/4) + 4*(lane/32) + e%4, column (m) = lane%32
    const bool n_vec = (N & 3) == 0 && y_vec != 0;   // 8-byte stores need an 8-byte aligned y
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++) {
            const int m = m0 + (wm * TM + j) * 32 + l32;
            if (m >= M) continue;
#pragma unroll
            for (int e4 = 0; e4 < 4; e4++) {
                const int n = n0 + (wn * TN + i) * 32 + 8 * e4 + 4 * kq;
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

// ------------------------------------------------------------------ matrix-matrix path, weights in registers
// Block tile 256 (n) x 128 (m) x 64 (k), four waves, each wave 64 rows of W (two 32-row tiles)
// against all 128 rows of x (four 32-row tiles): 8 accumulators of v_mfma_f32_32x32x16_f16.
//
// The LDS is the scarce resource of the staged kernel above (table gathers with bank
// conflicts, W tile written and read back, operand fragments read by every wave).  Here
//   * a wave decodes ITS 64 rows straight into A-operand registers - a lane's 8 bytes of a
//     row are the 4 codes it feeds to the 4 MFMA k steps of the tile, any k order works as
//     long as A and B agree - so W never touches the LDS and no decode is done twice;
//   * the tables are the conflict-free 16-copy ones of the matrix-vector kernels (256-byte
//     row pitch, lane reads copy lane % 16, address = one v_perm_b32);
//   * only x goes through the LDS (coalesced global loads, rows 144 bytes apart, double
//     buffered, one barrier per k tile), read as B fragments once per wave and k step.
// Per k tile and wave: 32 MFMAs (1024 matrix-unit clocks) against 36 LDS instructions and
// about 64 VALU operations, so the matrix unit is the bound.  Tile kt+1 is decoded and its x
// written while the MFMAs of tile kt run; global loads are four tiles ahead.
// w = g * s + d, d = low (kHi false) or high half of dd for both lanes, as plain vector code:
// the compiler folds the broadcast into the op_sel bits and its scheduler sees a VALU
// instruction (it cannot classify inline assembly)
template <bool kHi>
__device__ __forceinline__ h8_t gemm_finish(const u4_t &g, const u4_t &sg, uint32_t dd)
{
    const h2_t dv = as_h2(dd);
    const h2_t d = kHi ? h2_t{dv[1], dv[1]} : h2_t{dv[0], dv[0]};
    u4_t r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = as_u32(__builtin_elementwise_fma(as_h2(g[i]), as_h2(sg[i]), d));
    return __builtin_bit_cast(h8_t, r);
}

constexpr int kGrBN = 256, kGrBK = 64, kGrLd = kGrBK + 8;
constexpr int kGrTN = 2;
__host__ __device__ constexpr int gr_smem_bytes(int TM) { return kSTablesBytes + 2 * (32 * TM) * kGrLd * 2; }

// TM = 32-row tiles of x per workgroup (block tile 256 x 32 TM): 4 for prefill, 2 and 1 for
// shorter x.  kSplit: blockIdx.z picks a contiguous share of the k tiles and the block writes
// fp32 partial sums to part[z][M][N] instead of y (summed, scaled and rounded by
// splitk_reduce_kernel), so that short x still fills the chip with workgroups.
template <int TM, bool kSplit, bool kPacked>
__global__ __launch_bounds__(256) void gemm_reg_kernel(const uint16_t *__restrict__ x,
                                                       const uint16_t *__restrict__ codes,
                                                       const void *__restrict__ grid, float scale,
                                                       uint16_t *__restrict__ y, float *__restrict__ part,
                                                       int M, int N, int K, int splits, int y_vec)
{
    constexpr int kBM = 32 * TM;
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, kq = lane >> 5;
    const uint32_t lane_base = (uint32_t)(lane & 15) * 16u;
    const uint32_t quarter_bits = 0x34003400u;
    // Workgroups go to the 8 XCDs round robin by linear id, so with m fastest the workgroups
    // of one XCD share a few x row blocks (which then stay in that XCD's L2) and stream the codes.
    const int m0 = blockIdx.x * kBM;
    const int n0 = blockIdx.y * kGrBN;
    const int row_bytes = K >> 2;
    constexpr int kOut = (int)0x80000000;
    // this block's k tiles: [kt_lo, kt_lo + k_tiles)
    int kt_lo = 0, k_tiles = K / kGrBK;
    if (kSplit) {
        const int z = blockIdx.z, tq = k_tiles / splits, tr = k_tiles % splits;
        kt_lo = z * tq + (z < tr ? z : tr);
        k_tiles = tq + (z < tr ? 1 : 0);
    }

    // tables: thread tid owns grid row tid (16 copies) and 8 of the 2048 sign slots
    {
        const u4_t grow = reinterpret_cast<const u4_t *>(grid)[tid];
        u4_t *gg = reinterpret_cast<u4_t *>(smem_raw + kSSignBytes);
        u4_t *sg = reinterpret_cast<u4_t *>(smem_raw);
#pragma unroll
        for (int i = 0; i < 8; i++) sg[tid + i * 256] = sign_row((uint32_t)((tid + i * 256) >> 4));
#pragma unroll
        for (int i = 0; i < 16; i++) gg[tid * 16 + ((i + tid) & 15)] = grow;   // 16 lanes, 16 bank groups
    }

    // global sources.  Codes: lane (row l32 of tile i, half kq) reads 8 bytes = codes 4 kq .. 4 kq + 3
    // of the k tile.  x: load p of thread tid is piece tid % 8 (16 bytes) of row 32 p + tid / 8, so
    // that 8 lanes cover one 128-byte line.  Both as raw buffer
    // loads: rows past N / M and tiles past the end get zeros without a memory access.
    // Packed codes (pack_kernel): the 16 bytes of (row, k tile) sit at
    // (((row / 16) * (K / 256) + kt / 4) * 64 + (kt % 4) * 16 + row % 16) * 16, so the per-tile part
    // of the offset is kt * 256 and a wave's load is two runs of 256 consecutive bytes instead
    // of 32 pieces of 16.
    const int n_pad = ((N + 15) >> 4) << 4;
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(codes), 0, (int)((int64_t)(kPacked ? n_pad : N) * row_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t xrsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(x), 0, (int)((int64_t)M * K * 2), 0x00020000);
    // Row-major codes travel four k tiles at a time: lane (row, half kq) loads the 32 bytes of its row that
    // hold tiles 4 j + 2 kq and 4 j + 2 kq + 1 whole, so the two lanes of a row take 64 consecutive bytes
    // (half a cache line per visit, not 16 bytes of it), and one v_permlane32_swap per word hands lanes
    // l and l + 32 the halves they need of each other's tiles.  Tiles past the end of the block's share read
    // whatever follows in the row (zeros past the end of the matrix); their x is zero, so they add nothing.
    constexpr bool kWide = !kPacked;
    int cvoff[kGrTN];
#pragma unroll
    for (int i = 0; i < kGrTN; i++) {
        const int n = n0 + wave * 64 + i * 32 + l32;
        if (kPacked) cvoff[i] = n < n_pad ? (n >> 4) * (K >> 8) * 1024 + (n & 15) * 16 + kq * 8 : kOut;
        else cvoff[i] = n < N ? n * row_bytes + kq * 32 : kOut;
    }
    // rows r and r + 8 share a group of 16 lanes: with the 144-byte pitch their 16 pieces fall in
    // 16 different bank groups, so the LDS writes below are conflict-free like the fragment reads
    const int x_row = ((tid >> 7) << 4) + ((tid >> 4) & 7) + (((tid >> 3) & 1) << 3), x_piece = tid & 7;
    int xvoff[TM];
#pragma unroll
    for (int p = 0; p < TM; p++) {
        const int m = m0 + 32 * p + x_row;
        xvoff[p] = m < M ? (m * K + x_piece * 8) * 2 : kOut;
    }

    struct Stage {
        u2_t cw[kGrTN];
        u4_t xv[TM];
    };
    auto load_codes = [&](Stage &st, int kt) {   // kt counts this block's tiles (packed codes: one tile at a time)
        const int coff = kt < k_tiles ? (kt_lo + kt) * 256 : kOut;
#pragma unroll
        for (int i = 0; i < kGrTN; i++) st.cw[i] = __builtin_amdgcn_raw_buffer_load_b64(crsrc, cvoff[i], coff, 0);
    };
    // the codes of four tiles (row-major codes): w[row tile][h] holds, once swapped, tile h of the four in
    // words 0 and 1 and tile h + 2 in words 2 and 3
    struct CodeTrip {
        u4_t w[kGrTN][2];
    };
    auto load_trip = [&](CodeTrip &ct, int kt) {   // kt: the first of the four tiles, counted within the block
        const int coff = kt < k_tiles ? (kt_lo + kt) * 16 : kOut;
#pragma unroll
        for (int i = 0; i < kGrTN; i++)
#pragma unroll
            for (int h = 0; h < 2; h++) ct.w[i][h] = __builtin_amdgcn_raw_buffer_load_b128(crsrc, cvoff[i] + 16 * h, coff, 0);
    };
    auto swap_trip = [&](CodeTrip &ct) {
#pragma unroll
        for (int i = 0; i < kGrTN; i++)
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int w = 0; w < 2; w++) {
                    const u2_t r = __builtin_amdgcn_permlane32_swap(ct.w[i][h][w], ct.w[i][h][w + 2], false, false);
                    ct.w[i][h][w] = r[0];
                    ct.w[i][h][w + 2] = r[1];
                }
    };
    auto load_x = [&](Stage &st, int kt, int p) {
        const int xoff = kt < k_tiles ? (kt_lo + kt) * 128 : kOut;
        st.xv[p] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xvoff[p], xoff, 0);
    };
    auto load_tile = [&](Stage &st, int kt) {
        if constexpr (!kWide) load_codes(st, kt);
#pragma unroll
        for (int p = 0; p < TM; p++) load_x(st, kt, p);
    };
    unsigned char *xs = smem_raw + kSTablesBytes;                       // [2][kBM][kGrLd] halves
    const uint32_t xs_w = (uint32_t)(x_row * kGrLd + x_piece * 8) * 2u;                      // this thread's write slot (p = 0)
    const uint32_t xs_r = lds_addr(xs) + (uint32_t)(l32 * kGrLd + kq * 32) * 2u;             // this lane's B fragments
    constexpr uint32_t kXBuf = kBM * kGrLd * 2;

    CodeTrip cur, nxt;   // row-major codes: the four tiles being decoded and the four after them
    if constexpr (kWide) load_trip(nxt, 0);
    Stage ring[4];
#pragma unroll
    for (int i = 0; i < 4; i++) load_tile(ring[i], i);

    f16_t acc[kGrTN][TM];
#pragma unroll
    for (int i = 0; i < kGrTN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    // A fragments of one k tile: [tile i][k step s], a decoded code each
    u4_t afr[2][kGrTN][4];
    auto x_store = [&](const Stage &st, int buf, int p) {
        *reinterpret_cast<u4_t *>(xs + xs_w + buf * kXBuf + p * (32 * kGrLd * 2)) = st.xv[p];
    };
    // The decode runs as a stream of units, one per k step: unit u of a tile is word u / 2 of
    // row tile u % 2 (two codes = two k steps of that row tile).  A step gathers the table
    // rows of its unit and finishes (packed FMAs) the unit gathered one step earlier, so no
    // step waits for its own gathers.
    StreamGather g[2];
    // unit u of tile kI of the four in `ct` (row-major codes) or of the tile in `st` (packed codes)
    auto unit_gather = [&](StreamGather &o, const Stage &st, const CodeTrip &ct, int kI, int u) {
        const uint32_t cwd = kWide ? ct.w[u & 1][kI & 1][2 * (kI >> 1) + (u >> 1)] : st.cw[u & 1][u >> 1];
        stream_gather(o, cwd, lane_base, quarter_bits);
    };
    auto unit_finish = [&](const StreamGather &o, int abuf, int u) {
        afr[abuf][u & 1][2 * (u >> 1)] = __builtin_bit_cast(u4_t, gemm_finish<false>(o.g0, o.s0, o.dd));
        afr[abuf][u & 1][2 * (u >> 1) + 1] = __builtin_bit_cast(u4_t, gemm_finish<true>(o.g1, o.s1, o.dd));
    };

    __syncthreads();   // tables ready
    if constexpr (kWide) swap_trip(nxt);
#pragma unroll
    for (int u = 0; u < 4; u++) {
        unit_gather(g[u & 1], ring[0], nxt, 0, u);
        if (u < 3) unit_finish(g[u & 1], 0, u);   // unit 3 is finished by the first step of the loop
    }
    if constexpr (kWide) {
        cur = nxt;
        load_trip(nxt, 4);
    }
#pragma unroll
    for (int p = 0; p < TM; p++) x_store(ring[0], 0, p);
    __syncthreads();   // x tile 0 staged

    auto read_b = [&](u4_t (&b)[TM], int buf, int s) {
#pragma unroll
        for (int j = 0; j < TM; j++) b[j] = lds_read16(xs_r + buf * kXBuf + (uint32_t)(j * 32 * kGrLd * 2 + s * 16));
    };
    u4_t b[2][TM];   // the x fragments of the current and the next MFMA step
    read_b(b[0], 0, 0);
    // MFMAs of tile kt (A = afr[buf], B from x buffer buf) while tile kt+1 (registers sn) is
    // decoded into afr[buf ^ 1] and its x written to buffer buf ^ 1, and tile kt+4 is fetched
    // into sf.  Past the last tile sn holds zeros (out-of-range loads): decoding and storing
    // them is harmless and keeps every step one straight line of code, which the scheduling
    // hints below then weave into groups of one MFMA, LDS reads and VALU: with one wave per
    // SIMD nothing else hides the non-matrix instructions.
    constexpr int kMfma = kGrTN * TM;                       // MFMAs per k step
    constexpr int kDsPer = (TM + 4 + kMfma - 1) / kMfma;    // LDS reads per MFMA group
    constexpr int kValuPer = (24 + kMfma - 1) / kMfma;      // VALU per MFMA group
    // kNext (row-major codes): which of its four tiles tile kt+1 is; 0 = the first of the four after
    // the current ones, which then become the current ones while the loads of the four after them start
    auto tile = [&](int kt, int buf, const Stage &sn, Stage &sf, auto next_tag) {
        constexpr int kNext = decltype(next_tag)::value;
        if constexpr (kWide && kNext == 0) swap_trip(nxt);
        const CodeTrip &ct = kNext == 0 ? nxt : cur;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            // the global loads of tile kt+4 spread over the steps, woven between the MFMAs too
            if (!kWide && s == 0) load_codes(sf, kt + 4);
            if (TM == 4 && (s == 1 || s == 2)) {
                load_x(sf, kt + 4, 2 * s - 2);
                load_x(sf, kt + 4, 2 * s - 1);
            }
            if (TM < 4 && s >= 1 && s <= TM) load_x(sf, kt + 4, s - 1);
            // unit 3 of the CURRENT tile was gathered in the last step of the previous tile
            unit_finish(g[(s + 1) & 1], s == 0 ? buf : buf ^ 1, (s + 3) & 3);
            unit_gather(g[s & 1], sn, ct, kNext, s);
            if (s < 3) read_b(b[(s + 1) & 1], buf, s + 1);
            else read_b(b[0], buf ^ 1, 0);   // step 0 of tile kt + 1: its x is in place since the barrier
            if (kWide && kNext == 0 && s == 3) {
                cur = nxt;
                load_trip(nxt, kt + 5);   // tile kt + 1 is the first of the new current four
            }
#pragma unroll
            for (int i = 0; i < kGrTN; i++)
#pragma unroll
                for (int j = 0; j < TM; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8_t, afr[buf][i][s]),
                                                                       __builtin_bit_cast(h8_t, b[s & 1][j]), acc[i][j], 0, 0, 0);
            // the x of tile kt + 1 goes to the other buffer in steps 0 .. 2, ahead of the barrier
            if (TM == 4) {
                if (s == 0) x_store(sn, buf ^ 1, 0);
                if (s == 1) {
                    x_store(sn, buf ^ 1, 1);
                    x_store(sn, buf ^ 1, 2);
                }
                if (s == 2) x_store(sn, buf ^ 1, 3);
            } else if (s < TM) {
                x_store(sn, buf ^ 1, s);
            }
#pragma unroll
            for (int r = 0; r < kMfma; r++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);          // MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, kDsPer, 0);     // LDS reads
                __builtin_amdgcn_sched_group_barrier(0x002, kValuPer, 0);   // VALU
                if (s < 3 && (r == 1 || r == kMfma / 2)) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // global load
                if (kWide && kNext == 0 && s == 3 && r < 2 * kGrTN) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            }
            if (TM == 4 ? s < 3 : s < TM) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);   // LDS writes
            if (TM == 4 && s == 1) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            __builtin_amdgcn_sched_barrier(0);
            // The tile's one barrier lies between steps 2 and 3, not at its end, so that no tile starts by
            // waiting for an LDS read behind a barrier: buffer buf ^ 1 was last read in step 2 of the tile
            // before (the fragments of its step 3), ahead of that tile's barrier, and is read again in step 3.
            if (s == 2) __syncthreads();
        }
    };

    // Four tiles per trip with no way out in between: a path that left the loop body early
    // would reach the loop head with the newest loads still pending on registers the body
    // reuses, and the wait the compiler places there for that path (all loads done) would
    // be paid by every trip.  The up to three tiles left over run after the loop.
    int kt = 0;
    typedef std::integral_constant<int, 0> N0;
    typedef std::integral_constant<int, 1> N1;
    typedef std::integral_constant<int, 2> N2;
    typedef std::integral_constant<int, 3> N3;
    for (; kt + 4 <= k_tiles; kt += 4) {
        tile(kt, 0, ring[1], ring[0], N1{});
        tile(kt + 1, 1, ring[2], ring[1], N2{});
        tile(kt + 2, 0, ring[3], ring[2], N3{});
        tile(kt + 3, 1, ring[0], ring[3], N0{});
    }
    if (kt < k_tiles) tile(kt, 0, ring[1], ring[0], N1{});
    if (kt + 1 < k_tiles) tile(kt + 1, 1, ring[2], ring[1], N2{});
    if (kt + 2 < k_tiles) tile(kt + 2, 0, ring[3], ring[2], N3{});

    // D layout of 32x32: element e of lane: row (n) = 8*(e/4) + 4*(lane/32) + e%4, column (m) = lane%32
    const bool n_vec = (N & 3) == 0 && (kSplit || y_vec != 0);   // 8-byte stores need an 8-byte aligned y
#pragma unroll
    for (int i = 0; i < kGrTN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++) {
            const int m = m0 + j * 32 + l32;
            if (m >= M) continue;
#pragma unroll
            for (int e4 = 0; e4 < 4; e4++) {
                const int n = n0 + wave * 64 + i * 32 + 8 * e4 + 4 * kq;
                if (kSplit) {
                    float *dst = part + ((int64_t)blockIdx.z * M + m) * N + n;
                    if (n_vec && n + 3 < N) {
                        *reinterpret_cast<f4_t *>(dst) =
                            f4_t{acc[i][j][4 * e4], acc[i][j][4 * e4 + 1], acc[i][j][4 * e4 + 2], acc[i][j][4 * e4 + 3]};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (n + e < N) dst[e] = acc[i][j][4 * e4 + e];
                    }
                    continue;
                }
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

// y = half(scale * sum_z part[z]) over M * N elements; the order of the sum is fixed, so the
// result does not depend on how the blocks were scheduled.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ part, uint16_t *__restrict__ y,
                                                            int64_t mn, int splits, float scale)
{
    const int64_t i4 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i4 >= mn) return;
    if (i4 + 3 < mn && (mn & 3) == 0) {
        f4_t sacc = *reinterpret_cast<const f4_t *>(part + i4);
        for (int z = 1; z < splits; z++) sacc += *reinterpret_cast<const f4_t *>(part + (int64_t)z * mn + i4);
        u2_t v;
        v[0] = (uint32_t)__builtin_bit_cast(uint16_t, (half_t)(sacc[0] * scale)) |
               ((uint32_t)__builtin_bit_cast(uint16_t, (half_t)(sacc[1] * scale)) << 16);
        v[1] = (uint32_t)__builtin_bit_cast(uint16_t, (half_t)(sacc[2] * scale)) |
               ((uint32_t)__builtin_bit_cast(uint16_t, (half_t)(sacc[3] * scale)) << 16);
        *reinterpret_cast<u2_t *>(y + i4) = v;
    } else {
        for (int64_t i = i4; i < mn && i < i4 + 4; i++) {
            float sacc = part[i];
            for (int z = 1; z < splits; z++) sacc += part[(int64_t)z * mn + i];
            y[i] = __builtin_bit_cast(uint16_t, (half_t)(sacc * scale));
        }
    }
}
