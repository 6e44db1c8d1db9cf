// Matrix-vector kernels on 16-bit operands (M <= 32): shared helpers and the streaming kernel.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ matrix-vector paths (M <= 32)
// A workgroup owns 16*R consecutive rows of W for the whole of K; its W waves split K in
// interleaved 256-wide steps.  In one step a lane (row r = lane%16 of each 16-row tile,
// quarter q = lane/16) loads 8 consecutive codes (16 bytes) of its row, decodes them one at a
// time and feeds each as the A operand (16 rows x 32 k: this lane supplies the 8 k of its
// quarter) of v_mfma_f32_16x16x32_f16.  The B operand is x: column c = lane%16 is row m = c of
// x, same 8 k.  Any k order works as long as A and B agree, so the 32 k of MFMA number t in a
// step are {64*q + 8*t .. +8 : q = 0..3} rather than 32 consecutive k; that is what lets the
// code load be one 16-byte load per lane.  For M = 1 only column 0 carries data, the other 15
// columns cost nothing extra: the matrix unit has the headroom.
// Accumulator layout: lane holds rows 4*q + i (i = 0..3) of column c, i.e.
// y[m = c][n = n0 + 4*q + i] - four consecutive halves of a row of y.
typedef __attribute__((address_space(3))) const u4_t lds_u4_t;

// 32-bit LDS byte address of a pointer into shared memory
__device__ __forceinline__ uint32_t lds_addr(const void *p)
{
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}

__device__ __forceinline__ u4_t lds_read16(uint32_t byte_addr)
{
    return *reinterpret_cast<lds_u4_t *>(byte_addr);
}

typedef __attribute__((address_space(3))) u4_t lds_u4_rw_t;
__device__ __forceinline__ void lds_write16(uint32_t byte_addr, const u4_t &v)
{
    *reinterpret_cast<lds_u4_rw_t *>(byte_addr) = v;
}

// w = g * s + d with d taken from the low (kHi = false) or high half of dd for both lanes
template <bool kHi>
__device__ __forceinline__ uint32_t pk_fma_bcast(uint32_t g, uint32_t s, uint32_t dd)
{
    uint32_t r;
    if (kHi)
        asm("v_pk_fma_f16 %0, %1, %2, %3 op_sel:[0,0,1] op_sel_hi:[1,1,1]" : "=v"(r) : "v"(g), "v"(s), "v"(dd));
    else
        asm("v_pk_fma_f16 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[1,1,0]" : "=v"(r) : "v"(g), "v"(s), "v"(dd));
    return r;
}

// ------------------------------------------------------------------ streaming matrix-vector path
// The batch-1 path proper (small M, x small enough to live in LDS).  Two facts shape it: HBM
// answers in a few microseconds under load, so a CU must keep tens of KB of code bytes
// outstanding at all times, and vector-memory results return in order, so any x load queued
// behind the code prefetch would stall until the whole prefetch had landed.  Hence:
//   * x is copied once per workgroup into LDS (row pitch 2K + 16 bytes, so the rows read
//     together fall in different bank groups) and B operands are read from there;
//   * the code stream is a ring of D register buffers per wave, refilled with raw buffer
//     loads: the per-lane part of the address never changes, everything that moves (row
//     block, k step) is in the scalar offset, and past the end that offset is out of range,
//     which the hardware answers with zeros - no branch around any vector-memory
//     instruction, so the wait counters stay exact and D * R loads per wave stay in flight;
//   * workgroups are persistent (one per CU) and walk over row blocks, so the tables and x
//     are staged once and the prefetch runs across row-block boundaries;
//   * the LDS serves 16 lanes of a 16-byte gather per clock, so the decode tables hold 16
//     copies of every row (row pitch 256 bytes, lane reads copy lane % 16): conflict-free for
//     any codes.  A table address is one v_perm_b32: a byte of the code word placed above
//     the lane's copy offset.
// LDS map: [0, 32K) sign rows (128 x 256 B), [32K, 96K) grid rows (256 x 256 B),
//          then 2 x (W x R x 4 x M) float4 partial sums (double-buffered per row block), then x.

constexpr int kSSignBytes = 128 * 256;
constexpr int kSGridBytes = 256 * 256;
constexpr int kSTablesBytes = kSSignBytes + kSGridBytes;

__host__ __device__ constexpr int stream_red_bytes(int R, int W, int M) { return 2 * W * R * 4 * M * 16; }

// Table staging.  Every instruction of the prologue is paid once per wave that runs it, so the
// two tables go to different waves instead of a share of each to every thread: the first 256
// threads (waves 0-3) fetch one grid row each and write its 16 copies, the next 256 (waves 4-7)
// compute the sign rows (thread t: row t / 2, 8 of its 16 copies; needs no load, so it runs
// while the loads are in flight).  16 neighbouring lanes always write 16 different copy
// positions, i.e. 16 bank groups.
template <int kNThreads>
__device__ __forceinline__ void stream_stage_signs(unsigned char *smem, int tid)
{
    static_assert(kNThreads >= 512, "staging assumes at least 8 waves");
    if (tid < 256 || tid >= 512) return;
    const int t = tid - 256, row = t >> 1;
    const u4_t sv = sign_row((uint32_t)row);
    // slot i ^ (row % 8) of the thread's eight: one exclusive or per address
    const uint32_t sg = lds_addr(smem) + (uint32_t)((row * 16 + (t & 1) * 8 + (row & 7)) * 16);
#pragma unroll
    for (int i = 0; i < 8; i++) lds_write16(sg ^ (uint32_t)(i * 16), sv);
}

template <int kNThreads>
__device__ __forceinline__ void stream_stage_grid(unsigned char *smem, const u4_t &grow, int tid)
{
    if (tid >= 256) return;
    const uint32_t gg = lds_addr(smem) + (uint32_t)(kSSignBytes + (tid * 16 + (tid & 15)) * 16);   // slot i ^ (tid % 16)
#pragma unroll
    for (int i = 0; i < 16; i++) lds_write16(gg ^ (uint32_t)(i * 16), grow);
}

// Sum over each row of 16 lanes, result in lane 15 of the row (all 64 lanes must be active).
template <int kCtrl>
__device__ __forceinline__ float dpp_shr_add(float v)
{
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xF, 0xF, true));
}
__device__ __forceinline__ float row_sum16(float v)
{
    v = dpp_shr_add<0x118>(v);   // row_shr:8, lanes shifted in from outside the row read 0
    v = dpp_shr_add<0x114>(v);   // row_shr:4
    v = dpp_shr_add<0x112>(v);   // row_shr:2
    return dpp_shr_add<0x111>(v);   // row_shr:1
}

// (a & m) | (b & ~m) in one instruction
__device__ __forceinline__ uint32_t bfi(uint32_t m, uint32_t a, uint32_t b)
{
    uint32_t r;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(r) : "s"(m), "v"(a), "v"(b));
    return r;
}

struct StreamGather {
    u4_t g0, s0, g1, s1;
    uint32_t dd;
};

// lane_base = (lane % 16) * 16; the tables start at LDS address 0
__device__ __forceinline__ void stream_gather(StreamGather &o, uint32_t w, uint32_t lane_base, uint32_t quarter_bits)
{
    const uint32_t w7 = w & 0x7FFF7FFFu;                 // sign-row index must not see the shift bit
    o.g0 = lds_read16(__builtin_amdgcn_perm(w, lane_base, 0x0C0C0400u) + kSSignBytes);
    o.s0 = lds_read16(__builtin_amdgcn_perm(w7, lane_base, 0x0C0C0500u));
    o.g1 = lds_read16(__builtin_amdgcn_perm(w, lane_base, 0x0C0C0600u) + kSSignBytes);
    o.s1 = lds_read16(__builtin_amdgcn_perm(w7, lane_base, 0x0C0C0700u));
    o.dd = bfi(0x7FFF7FFFu, quarter_bits, w);            // (+-0.25, +-0.25): signs from the shift bits
}

template <bool kHi>
__device__ __forceinline__ h8_t stream_finish(const u4_t &g, const u4_t &sg, uint32_t dd)
{
    u4_t r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = pk_fma_bcast<kHi>(g[i], sg[i], dd);
    return __builtin_bit_cast(h8_t, r);
}

// One 256-wide k step for the first nv (uniform, 1 <= nv <= R) of R row tiles.  Items (word
// t2 of row tile r) run t2-major; the gathers of item i+1 are issued before the math of item i.
// Tiles past nv are skipped by uniform branches around their gathers and their math.
//
// The B operand.  A lane's 8 codes of the step feed 8 MFMAs (i = 0 .. 7), and MFMA i needs the
// 16-byte piece i of the lane quarter's 128 bytes of x in the lanes of ONE column per x row.
// JP = 1: column m holds row m (M <= 16) and every MFMA reads its piece, 8 wave-wide LDS reads
// per step, a third of the kernel's LDS traffic for one useful lane in 16.  JP = 4 (M <= 4):
// column 4 m + j holds piece 4 s + j of row m in register set s, so TWO reads fetch the whole
// step; MFMA i multiplies by set i / 4, and since its other columns hold the pieces of other
// MFMAs, MFMA i adds into accumulator i % 4, of which only the columns 4 m + i % 4 are ever
// looked at (finish_block adds column 4 m + j of accumulator j over j).  Lanes of columns past
// 4 M read zeros.
template <int JP>
struct StreamB {
    static constexpr int kAcc = JP == 1 ? 2 : JP;   // accumulators per row tile
};

template <int R, int JP>
__device__ __forceinline__ void stream_step(const u4_t (&cw)[R], uint32_t xaddr, uint32_t lane_base,
                                            uint32_t quarter_bits, f4_t (&acc)[R][StreamB<JP>::kAcc], int nv)
{
    constexpr int kItems = 4 * R;
    StreamGather buf[2];
    constexpr int kSets = JP == 1 ? 4 : 8 / JP;
    u4_t xb[kSets];
    if constexpr (JP == 1) {
        xb[0] = lds_read16(xaddr);
        xb[1] = lds_read16(xaddr + 16);
    } else {
#pragma unroll
        for (int s = 0; s < kSets; s++) xb[s] = lds_read16(xaddr + s * JP * 16);
    }
    stream_gather(buf[0], cw[0][0], lane_base, quarter_bits);
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int t2 = i / R, r = i % R;
        if (i + 1 < kItems) {
            const int nt2 = (i + 1) / R, nr = (i + 1) % R;
            if (nr == 0) {
                if constexpr (JP == 1) {
                    xb[(nt2 & 1) * 2] = lds_read16(xaddr + nt2 * 32);
                    xb[(nt2 & 1) * 2 + 1] = lds_read16(xaddr + nt2 * 32 + 16);
                }
                stream_gather(buf[(i + 1) & 1], cw[nr][nt2], lane_base, quarter_bits);
            } else if (nr < nv) {
                stream_gather(buf[(i + 1) & 1], cw[nr][nt2], lane_base, quarter_bits);
            }
        }
        if (r == 0 || r < nv) {
            // 4 packed FMAs, MFMA, 4 packed FMAs, MFMA: the second group and the next item's
            // address math run in the shadow of the matrix unit
            const StreamGather &b = buf[i & 1];
            constexpr int kA = StreamB<JP>::kAcc;
            const int i0 = 2 * t2, i1 = 2 * t2 + 1;
            const u4_t &b0 = JP == 1 ? xb[(t2 & 1) * 2] : xb[i0 / JP];
            const u4_t &b1 = JP == 1 ? xb[(t2 & 1) * 2 + 1] : xb[i1 / JP];
            const h8_t a0 = stream_finish<false>(b.g0, b.s0, b.dd);
            acc[r][i0 % kA] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, __builtin_bit_cast(h8_t, b0), acc[r][i0 % kA], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            const h8_t a1 = stream_finish<true>(b.g1, b.s1, b.dd);
            acc[r][i1 % kA] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, __builtin_bit_cast(h8_t, b1), acc[r][i1 % kA], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// v + (the value of the lane kShl places up the row of 16)
template <int kShl>
__device__ __forceinline__ float dpp_shl_add(float v, float w)
{
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, w), 0x100 + kShl, 0xF, 0xF, true));
}

// bytes of the LDS copy of x: M padded rows and 128 bytes of zeros behind them (the B operand
// of the columns that hold no x)
__host__ __device__ constexpr int64_t stream_x_bytes(int64_t M, int64_t K) { return M * (2 * K + 16) + 128; }

template <int R, int W, int D, bool kPacked, int JP>
__device__ __forceinline__ void gemv_stream_body(const uint16_t *__restrict__ x, const uint16_t *__restrict__ codes,
                                                 const void *__restrict__ grid, float scale,
                                                 uint16_t *__restrict__ y, int M, int N, int K, int tiles_q,
                                                 int tiles_r)
{
    static_assert(R == 1 || R == 2, "a partial row block is handled as one tile");
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];
    f4_t *red = reinterpret_cast<f4_t *>(smem_raw + kSTablesBytes);   // [2][W][R][4 * M]
    const int red_par = W * R * 4 * M;                                 // float4 per parity
    unsigned char *xs = smem_raw + kSTablesBytes + stream_red_bytes(R, W, M);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: offsets derived from it live in SGPRs
    const int c16 = lane & 15;
    const int q = lane >> 4;
    const int n_steps = K >> 8;
    const int row_bytes = K >> 2;
    const int x_pitch = 2 * K + 16;
    const uint32_t lane_base = (uint32_t)c16 * 16u;
    const uint32_t quarter_bits = 0x34003400u;

    // ---- prologue: this thread's grid row and its share of x first (short latency, nothing
    // queued in front of them), then the first D items of the code stream; the tables and the
    // LDS copy of x are built while the code loads fly ---------------------------------------
    const u4_t grow = tid < 256 ? reinterpret_cast<const u4_t *>(grid)[tid] : u4_t{0u, 0u, 0u, 0u};   // waves 0-3 stage the grid
    const int row_chunks = K >> 3;                     // 16-byte pieces per row of x
    const int n_pieces = M * row_chunks;               // x is [M][K] contiguous: piece p sits at x + 16 p
    // pieces of x per thread fetched up front, before the code loads are queued: vector-memory results
    // return in order, so a piece asked for later arrives behind the whole first burst of codes.  One
    // row of x: up to four pieces (all of it for K <= 32768); more rows: up to six (all of x for M <= 4 at
    // K = 11008).
    constexpr int kXPer = 6, kXPer1 = 4;
    u4_t xv[kXPer];
#pragma unroll
    for (int u = 0; u < kXPer; u++) {
        const int p = u * 64 * W + tid;
        xv[u] = p < n_pieces && (u < kXPer1 || M > 1) ? reinterpret_cast<const u4_t *>(x)[p] : u4_t{0u, 0u, 0u, 0u};
    }

    const int n_sw = wave < n_steps ? (n_steps - wave + W - 1) / W : 0;   // k steps of this wave per row block
    // this workgroup's share of the 16-row tiles: a contiguous range, tiles_q tiles plus one
    // more for the first tiles_r workgroups (quotient and remainder of tiles / workgroups, from
    // the host), walked R tiles (one row block) at a time; the last block may be partial
    const int t0 = (int)blockIdx.x * tiles_q + ((int)blockIdx.x < tiles_r ? (int)blockIdx.x : tiles_r);
    const int t1 = t0 + tiles_q + ((int)blockIdx.x < tiles_r ? 1 : 0);
    const int nb_wg = (t1 - t0 + R - 1) / R;

    // Row-major codes [N][K/8]: a lane's 16 bytes are 8 codes of its row, a wave's load touches
    // 16 rows x 64 bytes.  Packed codes (pack_kernel): the same 16 bytes sit at
    // ((tile * n_steps + step) * 64 + lane) * 16, so a wave's load is 1 KB of consecutive bytes.
    const int n_tiles_all = (N + 15) >> 4;
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(codes), 0, (int)((int64_t)(kPacked ? n_tiles_all * 16 : N) * row_bytes), 0x00020000);
    // per-lane byte offset inside a row block (never changes) ...
    int voff[R];
#pragma unroll
    for (int r = 0; r < R; r++) voff[r] = kPacked ? lane * 16 + r * n_steps * 1024 : (16 * r + c16) * row_bytes + q * 16;
    // ... and the scalar part: first tile and k step of the next item to prefetch.  Rows past N
    // land past the end of the buffer by themselves (row-major) or are zero padding (packed);
    // items past the end get an offset no buffer reaches.
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
    stream_stage_signs<64 * W>(smem_raw, tid);
    __builtin_amdgcn_sched_barrier(0);   // keep the sign rows ahead of the waits for the loads

    // x -> LDS (row m at m * x_pitch): the pieces fetched above, then whatever is left
    if (M == 1) {
#pragma unroll
        for (int u = 0; u < kXPer1; u++) {
            const int c = u * 64 * W + tid;
            if (c < row_chunks) reinterpret_cast<u4_t *>(xs)[c] = xv[u];
        }
        for (int c = kXPer1 * 64 * W + tid; c < row_chunks; c += 64 * W)
            reinterpret_cast<u4_t *>(xs)[c] = reinterpret_cast<const u4_t *>(x)[c];
    } else {
        int m = 0, c = tid;   // piece p = m * row_chunks + c
#pragma unroll
        for (int u = 0; u < kXPer; u++) {
            while (c >= row_chunks) { c -= row_chunks; m++; }
            if (m < M) reinterpret_cast<u4_t *>(xs + m * x_pitch)[c] = xv[u];
            c += 64 * W;
        }
        for (int p = kXPer * 64 * W + tid; p < n_pieces; p += 64 * W) {
            while (c >= row_chunks) { c -= row_chunks; m++; }
            reinterpret_cast<u4_t *>(xs + m * x_pitch)[c] = reinterpret_cast<const u4_t *>(x)[p];
            c += 64 * W;
        }
    }
    if (tid >= 64 * W - 8) reinterpret_cast<u4_t *>(xs + M * x_pitch)[tid - (64 * W - 8)] = u4_t{0u, 0u, 0u, 0u};
    stream_stage_grid<64 * W>(smem_raw, grow, tid);
    __syncthreads();

    // B operand address of this lane.  JP = 1: row m = c16 (row 0 for columns past M), quarter
    // q.  JP = 4: column c16 = 4 m + j reads piece j (and 4 + j) of row m's quarter; columns past
    // 4 M read the zeros behind x, at every step (their step stride is 0).
    constexpr int kAcc = StreamB<JP>::kAcc;
    const bool col_live = JP == 1 || c16 / JP < M;
    const uint32_t xlane = JP == 1    ? lds_addr(xs) + (uint32_t)((c16 < M ? c16 : 0) * x_pitch + q * 128)
                           : col_live ? lds_addr(xs) + (uint32_t)((c16 / JP) * x_pitch + q * 128 + (c16 % JP) * 16)
                                      : lds_addr(xs) + (uint32_t)(M * x_pitch);
    const uint32_t xstride = col_live ? 512u : 0u;

    f4_t acc[R][kAcc];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int a = 0; a < kAcc; a++) acc[r][a] = f4_t{0.f, 0.f, 0.f, 0.f};

    // publish this wave's partial sums of a finished row block, meet the other waves, add up
    // and store
    auto finish_block = [&](int blk) {
        f4_t *rp = red + (blk & 1) * red_par;
        if constexpr (JP == 1) {
            if (c16 < M) {
#pragma unroll
                for (int r = 0; r < R; r++) rp[(wave * R + r) * 4 * M + q * M + c16] = acc[r][0] + acc[r][1];
            }
        } else {
            // column 4 m + j of accumulator j, added over j into the lane of column 4 m
#pragma unroll
            for (int r = 0; r < R; r++) {
                f4_t v = acc[r][0];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    v[e] = dpp_shl_add<1>(v[e], acc[r][1][e]);
                    v[e] = dpp_shl_add<2>(v[e], acc[r][2][e]);
                    v[e] = dpp_shl_add<3>(v[e], acc[r][3][e]);
                }
                if (c16 % JP == 0 && c16 / JP < M) rp[(wave * R + r) * 4 * M + q * M + c16 / JP] = v;
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int a = 0; a < kAcc; a++) acc[r][a] = f4_t{0.f, 0.f, 0.f, 0.f};
        __syncthreads();
        // (row tile r, x row m) pairs go round the waves; lane (w = lane % 16, quarter lane / 16)
        // fetches ONE partial sum, wave w's, and the 16 of a row of lanes are added with DPP
        // shifts: a single LDS round trip instead of a chain of W dependent ones
        for (int p = wave; p < R * M; p += W) {
            const int r = M == 1 ? p : p / M, m = p - r * M;
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
        // no k step for this wave (K shorter than the workgroup is wide): it still meets the
        // others at every row block's barrier, contributing zeros
        for (int blk = 0; blk < nb_wg; blk++) finish_block(blk);
        return;
    }

    const int n_items = nb_wg * n_sw;
    int blk = 0, j = 0;
    for (int i0 = 0; i0 < n_items; i0 += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (i0 + d < n_items) {
                const uint32_t xa = xlane + __umul24((uint32_t)(wave + j * W), xstride);
                const int nv = t1 - (t0 + blk * R);   // tiles of this block that are ours (uniform)
                stream_step<R, JP>(cw[d], xa, lane_base, quarter_bits, acc, nv);
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

template <int R, int W, int D, bool kPacked, int JP>
__global__ __launch_bounds__(64 * W) void gemv_stream_kernel(const uint16_t *__restrict__ x,
                                                             const uint16_t *__restrict__ codes,
                                                             const void *__restrict__ grid, float scale,
                                                             uint16_t *__restrict__ y, int M, int N, int K,
                                                             int tiles_q, int tiles_r)
{
    gemv_stream_body<R, W, D, kPacked, JP>(x, codes, grid, scale, y, M, N, K, tiles_q, tiles_r);
}
