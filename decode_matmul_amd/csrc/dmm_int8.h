// The reference's integer operator (int8 x, int64 codebook, int32 out): exact kernels on the int8
// MFMA and the catch-all.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ the reference's integer operator
// out[m,n] = sum_k x[m,k] * W[n,k] in int32, W decoded to int8 from the packed int64 table
// exactly as /root/reference/test_decode_matmul.py:29-55 (value = +-byte, then +1 or -1, kept
// in int8).  Codes may be in the layout the reference's kernel reads
// (/root/reference/test_decode_matmul.py:101-109: 16-row x 4-column tiles of 64 codes ordered
// [row % 8][column % 4][row / 8]) or plain row-major.  One wave per output row, integer
// arithmetic throughout, so the result is exact for any K (the sum wraps in int32 like the
// reference's accumulator).  A correctness path, not a tuned one (no matrix unit).
__device__ __forceinline__ int64_t tiled_code_index(int64_t n, int64_t j, int64_t kc)
{
    return ((n >> 4) * (kc >> 2) + (j >> 2)) * 64 + (n & 7) * 8 + (j & 3) * 2 + ((n >> 3) & 1);
}

__device__ __forceinline__ int wave_sum_i32(int v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Weights of one code, exactly as the reference's scalar decode: +-byte, then +1 or -1, kept in int8.
__device__ __forceinline__ void int8_decode_exact(uint64_t abs, uint32_t c, int (&w)[8])
{
    uint32_t s8 = (c >> 8) & 0x7Fu;
    s8 |= (__builtin_popcount(s8) & 1u) << 7;
    const int shift = (c >> 15) & 1;
#pragma unroll
    for (int d = 0; d < 8; d++) {
        int8_t v = (int8_t)(abs & 0xFFu);
        if ((s8 >> d) & 1u) v = (int8_t)(-v);
        v = (int8_t)(shift ? v - 1 : v + 1);
        w[d] = v;
        abs >>= 8;
    }
}

// kFast: every byte of the table is 2 mod 4 (the E8P table is: 4 x a half-odd value).  Then
// negating a byte flips its upper six bits, adding 1 sets its lowest bit and subtracting 1
// turns the low bits 10 into 01 - the whole decode is one exclusive or with a mask that depends
// only on the code's high byte (/root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:45-65
// uses the same property), and the 8 products of a code are two 4-way int8 dot products.
// Otherwise (kFast false) the scalar decode above, byte by byte.  x8: x and K allow 8-byte loads.
// Rows n_first, n_first + n_stride, ... below n_end, one wave each.
template <bool kFast>
__device__ __forceinline__ void int8_rows(const int8_t *__restrict__ x, const uint16_t *__restrict__ codes,
                                          const uint64_t *table, const uint64_t *masks, int32_t *__restrict__ out,
                                          int64_t M, int64_t N, int64_t K, int tiled, bool x8, int64_t n_first,
                                          int64_t n_stride, int64_t n_end)
{
    const int lane = threadIdx.x & 63;
    const int64_t kc = K >> 3;
    constexpr int kMC = 8;
    for (int64_t n = n_first; n < n_end; n += n_stride) {
        for (int64_t m0 = 0; m0 < M; m0 += kMC) {
            int acc[kMC] = {};
            for (int64_t j = lane; j < kc; j += kWave) {
                const uint32_t c = codes[tiled ? tiled_code_index(n, j, kc) : n * kc + j];
                if (kFast) {
                    const uint64_t w8 = table[c & 0xFFu] ^ masks[c >> 8];
                    const int wlo = (int)(uint32_t)w8, whi = (int)(uint32_t)(w8 >> 32);
#pragma unroll
                    for (int mm = 0; mm < kMC; mm++) {
                        if (m0 + mm < M) {
                            const int8_t *xr = x + (m0 + mm) * K + j * 8;
                            int xlo, xhi;
                            if (x8) {
                                const u2_t v = *reinterpret_cast<const u2_t *>(xr);
                                xlo = (int)v[0];
                                xhi = (int)v[1];
                            } else {
                                xlo = (int)((uint32_t)(uint8_t)xr[0] | (uint32_t)(uint8_t)xr[1] << 8 |
                                            (uint32_t)(uint8_t)xr[2] << 16 | (uint32_t)(uint8_t)xr[3] << 24);
                                xhi = (int)((uint32_t)(uint8_t)xr[4] | (uint32_t)(uint8_t)xr[5] << 8 |
                                            (uint32_t)(uint8_t)xr[6] << 16 | (uint32_t)(uint8_t)xr[7] << 24);
                            }
                            acc[mm] = __builtin_amdgcn_sdot4(xlo, wlo, acc[mm], false);
                            acc[mm] = __builtin_amdgcn_sdot4(xhi, whi, acc[mm], false);
                        }
                    }
                } else {
                    int w[8];
                    int8_decode_exact(table[c & 0xFFu], c, w);
#pragma unroll
                    for (int mm = 0; mm < kMC; mm++) {
                        if (m0 + mm < M) {
                            const int8_t *xr = x + (m0 + mm) * K + j * 8;
#pragma unroll
                            for (int d = 0; d < 8; d++) acc[mm] += (int)xr[d] * w[d];
                        }
                    }
                }
            }
#pragma unroll
            for (int mm = 0; mm < kMC; mm++) {
                const int sum = wave_sum_i32(acc[mm]);
                if (lane == 0 && m0 + mm < M) out[(m0 + mm) * N + n] = sum;
            }
        }
    }
}

__global__ __launch_bounds__(256) void int8_kernel(const int8_t *__restrict__ x, const uint16_t *__restrict__ codes,
                                                   const int64_t *__restrict__ codebook_abs,
                                                   int32_t *__restrict__ out, int64_t M, int64_t N, int64_t K,
                                                   int tiled, int x8)
{
    __shared__ uint64_t table[256];
    __shared__ uint64_t masks[256];
    __shared__ int slow[4];
    const uint64_t abs = (uint64_t)codebook_abs[threadIdx.x];
    table[threadIdx.x] = abs;
    {
        // mask of high byte t: sign bits t & 0x7F (the eighth by parity), shift t >> 7
        uint32_t s8 = threadIdx.x & 0x7Fu;
        s8 |= (__builtin_popcount(s8) & 1u) << 7;
        uint64_t mk = (threadIdx.x >> 7) ? 0x0303030303030303ull : 0x0101010101010101ull;
#pragma unroll
        for (int d = 0; d < 8; d++)
            if ((s8 >> d) & 1u) mk ^= 0xFCull << (8 * d);
        masks[threadIdx.x] = mk;
    }
    const bool bad = (abs & 0x0303030303030303ull) != 0x0202020202020202ull;
    const bool wave_bad = __builtin_amdgcn_ballot_w64(bad) != 0;
    if ((threadIdx.x & 63) == 0) slow[threadIdx.x >> 6] = wave_bad ? 1 : 0;
    __syncthreads();
    const int64_t n_first = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6), n_stride = (int64_t)gridDim.x * 4;
    if (slow[0] | slow[1] | slow[2] | slow[3])
        int8_rows<false>(x, codes, table, masks, out, M, N, K, tiled, false, n_first, n_stride, N);
    else
        int8_rows<true>(x, codes, table, masks, out, M, N, K, tiled, x8 != 0, n_first, n_stride, N);
}

// ------------------------------------------------------------------ the integer operator on the matrix unit
// K a multiple of 256, a table whose bytes are all 2 mod 4 (see int8_rows): the
// small-batch kernel's structure (persistent workgroups over contiguous ranges of 16-row tiles,
// k steps of 256 dealt to 8 waves, the x slice of a step fetched from L2 with the codes as one
// prefetch unit - in whole lines, four rows of 256 bytes per load instruction - and turned into
// fragments through a 4 KB piece of LDS that belongs to the wave alone, the 16-byte pieces of row m
// exchanged by m % 16 so that neither the writes nor the reads meet a bank conflict; the same pieces
// carry the partial sums at the end of a row block) with the decode done in bytes - one 8-byte gather of
// the table entry by the code's low byte, one of the mask by its high byte, exclusive or - and
// v_mfma_i32_16x16x64_i8: a lane's 8 codes of a step are the A operands of four MFMAs (two codes =
// 16 k each), B is 16 bytes of x per lane and MFMA.  Both tables hold 32 copies of every 8-byte
// row (row pitch 256 B, lane reads copy lane % 32: no bank conflicts for any codes).  Exact:
// int8 products, int32 sums (which wrap like the reference's accumulator).
// Codes row-major, or in the reference's tile order (/root/reference/test_decode_matmul.py:101-109):
// there 16 bytes hold codes (row g, columns c .. c + 3) interleaved with row g + 8's, so lanes g
// and g + 8 load the same two pieces and each keeps its halves (one v_perm per two codes).
// A table with any other byte is found while the tables are built, and the workgroup then does
// its rows with the scalar decode instead.  More than 16 rows of x: a row block is walked once
// per 16 rows (a pass), so the codes come from HBM once and from the caches after that.
typedef int i4_t __attribute__((ext_vector_type(4)));
constexpr int kI8TableBytes = 256 * 256;   // one table: 256 rows x 32 copies x 8 bytes

constexpr int kI8xPiece = 4096;   // LDS bytes of a wave's own piece: 16 rows x 256 bytes

// kSlice: the x of a step through the wave's piece as above (pays from about 8 rows of x on); else
// every lane loads its own four fragments, which for a row or two of x is the cheaper way
template <int R, int W, int D, bool kTiled, bool kSlice>
__global__ __launch_bounds__(64 * W) void int8x_kernel(const int8_t *__restrict__ x, const uint16_t *__restrict__ codes,
                                                       const int64_t *__restrict__ codebook_abs,
                                                       int32_t *__restrict__ out, int M, int N, int K, int tiles_q,
                                                       int tiles_r)
{
    static_assert(W == 8, "the table staging below assumes 512 threads");
    static_assert(R * kWave * 16 <= kI8xPiece, "the partial sums of a row block go through the wave's piece");
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15;
    const int q = lane >> 4;
    const int n_steps = K >> 8;
    const int row_bytes = K >> 2;
    const uint32_t lane_base = (uint32_t)(lane & 31) * 8u;          // grid rows: [0, 64K)
    const uint32_t lane_base2 = lane_base | 0x10000u;               // mask rows: [64K, 128K)

    uint64_t entry = 0;
    if (tid < 256) entry = (uint64_t)codebook_abs[tid];

    const int n_sw = wave < n_steps ? (n_steps - wave + W - 1) / W : 0;
    const int t0 = (int)blockIdx.x * tiles_q + ((int)blockIdx.x < tiles_r ? (int)blockIdx.x : tiles_r);
    const int t1 = t0 + tiles_q + ((int)blockIdx.x < tiles_r ? 1 : 0);
    const int nb_wg = (t1 - t0 + R - 1) / R;

    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(codes), 0, (int)((int64_t)(kTiled ? ((N + 15) >> 4) * 16 : N) * row_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t xrsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(x), 0, M * K, 0x00020000);
    constexpr int kOut = (int)0x80000000;
    // per-lane byte offsets inside a row block.  Row-major: row 16 r + c16, 16 bytes at quarter q.
    // Tiled: the tile row of the block is 16 rows x K / 4 bytes as well, a tile (4 code columns) is
    // 128 bytes, and lane (g = c16 % 8, quarter q) reads 16 bytes at g * 16 of tiles 2 q and 2 q + 1
    // of the step's 8.
    int voff[R];
#pragma unroll
    for (int r = 0; r < R; r++)
        voff[r] = kTiled ? r * 16 * row_bytes + q * 256 + (c16 & 7) * 16 : (16 * r + c16) * row_bytes + q * 16;
    // load i of a step is piece lane % 16 (16 bytes) of row 4 i + lane / 16 of the slice; pass p adds
    // 16 p rows; rows past M lie past the end of the buffer: zeros, no memory access
    int xcoff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) xcoff[i] = kSlice ? (4 * i + q) * K + c16 * 16 : c16 * K + 64 * q + 16 * i;
    const int n_pass = (M + 15) >> 4;
    const int pass_bytes = 16 * K;
    // the wave's piece of LDS: row m at m * 256, its piece p in slot p ^ m.  Writes: row 4 i + h, piece
    // lane % 16, h = lane / 16, i.e. (xs_w ^ 64 i) + 1024 i.  Reads: row c16, piece 4 q + t, i.e. xs_r ^ 16 t.
    const uint32_t xs_piece = lds_addr(smem_raw) + (uint32_t)(2 * kI8TableBytes + wave * kI8xPiece);
    const uint32_t xs_w = xs_piece + (uint32_t)(q * 256 + ((c16 ^ q) << 4));
    const uint32_t xs_r = xs_piece + (uint32_t)(c16 * 256 + (((4 * q) ^ c16) << 4));
    const uint32_t half_sel = (c16 & 8) ? 0x07060302u : 0x05040100u;   // tiled: which row of the pair is ours

    struct Unit {
        u4_t cw[R][kTiled ? 2 : 1];
        u4_t xs[4];   // the slice as loaded, or the lane's four fragments
    };
    int pf_blk = 0, pf_pass = 0, pf_j = 0;
    auto issue = [&](Unit &u) {
        const bool ok = pf_blk < nb_wg && n_sw > 0;
        const int step = wave + pf_j * W;
        const int xs_off = ok ? step * 256 + pf_pass * pass_bytes : kOut;
        const int tb = t0 + pf_blk * R;
        const int soff = !ok ? kOut : kTiled ? tb * 16 * row_bytes + step * 1024 : tb * 16 * row_bytes + step * 64;
#pragma unroll
        for (int i = 0; i < 4; i++) u.xs[i] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xcoff[i], xs_off, 0);
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int so = (r == 0 || tb + r < t1) ? soff : kOut;
            u.cw[r][0] = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff[r], so, 0);
            if (kTiled) u.cw[r][kTiled ? 1 : 0] = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff[r] + 128, so, 0);
        }
        if (++pf_j >= n_sw) {
            pf_j = 0;
            if (++pf_pass >= n_pass) { pf_pass = 0; pf_blk++; }
        }
    };

    Unit ring[D];
#pragma unroll
    for (int d = 0; d < D; d++) issue(ring[d]);

    // tables: threads 0 .. 255 write the 32 copies of table entry tid (16 slots of two copies),
    // threads 256 .. 511 those of the mask of high byte tid - 256
    bool bad = false;
    {
        uint64_t v = entry;
        if (tid < 256) {
            bad = (entry & 0x0303030303030303ull) != 0x0202020202020202ull;
        } else {
            const uint32_t t = (uint32_t)tid - 256u;
            uint32_t s8 = t & 0x7Fu;
            s8 |= (__builtin_popcount(s8) & 1u) << 7;
            v = (t >> 7) ? 0x0303030303030303ull : 0x0101010101010101ull;
#pragma unroll
            for (int d = 0; d < 8; d++)
                if ((s8 >> d) & 1u) v ^= 0xFCull << (8 * d);
        }
        const uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
        // tid >= 256 lands in the mask table; slot i ^ (tid % 16): 16 lanes, 16 bank groups, one exclusive or per address
        const uint32_t rowp = lds_addr(smem_raw) + (uint32_t)((tid * 16 + (tid & 15)) * 16);
#pragma unroll
        for (int i = 0; i < 16; i++) lds_write16(rowp ^ (uint32_t)(i * 16), u4_t{lo, hi, lo, hi});
    }
    // the vote on the table: one word per wave in the area of the pieces, read by everybody after the barrier
    uint32_t *votes = reinterpret_cast<uint32_t *>(smem_raw + 2 * kI8TableBytes);
    const bool wave_bad = __builtin_amdgcn_ballot_w64(bad) != 0;
    if (lane == 0) votes[wave] = wave_bad ? 1u : 0u;
    __syncthreads();
    const bool any_bad = __builtin_amdgcn_ballot_w64(votes[lane & (W - 1)] != 0) != 0;
    __syncthreads();   // the votes are read before the first slice of x overwrites them
    if (any_bad) {
        // scalar decode for this workgroup's rows; the raw table goes where the pieces would
        uint64_t *table = reinterpret_cast<uint64_t *>(smem_raw + 2 * kI8TableBytes);
        if (tid < 256) table[tid] = entry;
        __syncthreads();
        const int64_t n_end = (int64_t)t1 * 16 < N ? (int64_t)t1 * 16 : N;
        int8_rows<false>(x, codes, table, table, out, M, N, K, kTiled ? 1 : 0, false, (int64_t)t0 * 16 + wave, W, n_end);
        return;
    }

    i4_t acc[R][2];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r][0] = acc[r][1] = i4_t{0, 0, 0, 0};

    // end of a pass over a row block: every wave leaves its partial sums in its own piece (row tile
    // r at lane l: byte (r * 64 + l) * 16), one barrier, the first R waves add up one row tile each
    // and store it, and a second barrier, because the pieces take the x of the next pass next
    auto finish_block = [&](int blk, int pass) {
        i4_t *own = reinterpret_cast<i4_t *>(smem_raw + 2 * kI8TableBytes + wave * kI8xPiece);
#pragma unroll
        for (int r = 0; r < R; r++) {
            own[r * kWave + lane] = acc[r][0] + acc[r][1];
            acc[r][0] = acc[r][1] = i4_t{0, 0, 0, 0};
        }
        __syncthreads();
        for (int r = wave; r < R; r += W) {
            const i4_t *src = reinterpret_cast<const i4_t *>(smem_raw + 2 * kI8TableBytes) + r * kWave + lane;
            i4_t sacc = src[0];
#pragma unroll
            for (int w = 1; w < W; w++) sacc += src[w * (kI8xPiece / 16)];
            const int rt = t0 + blk * R + r;
            const int n = rt * 16 + 4 * q;
            const int m = 16 * pass + c16;
            if (m < M && rt < t1 && n < N)   // N % 4 == 0, so the four rows are in range together
                *reinterpret_cast<i4_t *>(out + (int64_t)m * N + n) = sacc;
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
                const Unit &u = ring[d];
                const int nv = t1 - (t0 + blk * R);   // tiles of this block that are ours (uniform)
                u4_t xf[4];
                if constexpr (kSlice) {
                    // the slice through the wave's piece: in as loaded, out as fragments
#pragma unroll
                    for (int i = 0; i < 4; i++) lds_write16((xs_w ^ (uint32_t)(64 * i)) + (uint32_t)(1024 * i), u.xs[i]);
#pragma unroll
                    for (int t = 0; t < 4; t++) xf[t] = lds_read16(xs_r ^ (uint32_t)(16 * t));
                } else {
#pragma unroll
                    for (int t = 0; t < 4; t++) xf[t] = u.xs[t];
                }
#pragma unroll
                for (int r = 0; r < R; r++) {
                    if (r > 0 && r >= nv) break;
                    u4_t cw;   // the lane's 8 codes of the step, two per word
                    if (kTiled) {
                        const u4_t &a = u.cw[r][0], &b = u.cw[r][kTiled ? 1 : 0];
                        cw = u4_t{__builtin_amdgcn_perm(a[1], a[0], half_sel), __builtin_amdgcn_perm(a[3], a[2], half_sel),
                                  __builtin_amdgcn_perm(b[1], b[0], half_sel), __builtin_amdgcn_perm(b[3], b[2], half_sel)};
                    } else {
                        cw = u.cw[r][0];
                    }
                    u2_t g[8], m[8];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const uint32_t w = cw[i];
                        g[2 * i] = lds_read8(__builtin_amdgcn_perm(w, lane_base, 0x0C0C0400u));
                        m[2 * i] = lds_read8(__builtin_amdgcn_perm(w, lane_base2, 0x0C020500u));
                        g[2 * i + 1] = lds_read8(__builtin_amdgcn_perm(w, lane_base, 0x0C0C0600u));
                        m[2 * i + 1] = lds_read8(__builtin_amdgcn_perm(w, lane_base2, 0x0C020700u));
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const i4_t a = i4_t{(int)(g[2 * i][0] ^ m[2 * i][0]), (int)(g[2 * i][1] ^ m[2 * i][1]),
                                            (int)(g[2 * i + 1][0] ^ m[2 * i + 1][0]), (int)(g[2 * i + 1][1] ^ m[2 * i + 1][1])};
                        acc[r][i & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, __builtin_bit_cast(i4_t, xf[i]), acc[r][i & 1], 0, 0, 0);
                    }
                }
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


// ------------------------------------------------------------------ the integer operator, up to eight rows, resident sums
// int8x_kernel's tables and byte decode in the loop order of the batch-1 half-precision kernels: sixteen
// waves, chunk (16 k steps, one per wave) outside and tiles inside, the int32 sums of all NT <= 8 row tiles
// of the workgroup's share in registers from start to end, a ring of D code loads per wave over the items
// (chunk, tile), one of them ahead of the prologue's work.  A wave fetches the x of its own k step - up
// to 8 rows of 256 bytes, two load instructions of four whole lines each - through a 2 KB piece of LDS
// that is its own (pieces of row m exchanged by m: no bank conflicts) into the four B operands of a tile
// step, and keeps them for every tile; the slice of the next chunk is asked for before the tile steps of
// this one.  No barrier between the one after the tables and the end, where the sums go through the same
// pieces, four tiles at a time (the 128 KB of tables leave 32 KB).  Nine to sixteen rows of x: eight waves with
// pieces of sixteen rows (four load instructions per slice), a chunk of 8 k steps.  Exact like int8x_kernel; a
// table with a byte that is not 2 mod 4 goes to the scalar decode.
template <int kCtrl>
__device__ __forceinline__ int dpp_shr_add_i(int v)
{
    return v + __builtin_amdgcn_update_dpp(0, v, kCtrl, 0xF, 0xF, true);
}
// sum over each row of 16 lanes, result in lane 15 of the row
__device__ __forceinline__ int row_sum16_i(int v)
{
    v = dpp_shr_add_i<0x118>(v);
    v = dpp_shr_add_i<0x114>(v);
    v = dpp_shr_add_i<0x112>(v);
    return dpp_shr_add_i<0x111>(v);
}

// W = 16 waves with pieces of 8 rows of x (2 KB), or 8 waves with pieces of 16 rows (4 KB): 32 KB either way
__host__ __device__ constexpr int i8d_piece_bytes(int W) { return W == 16 ? 2048 : 4096; }

// CG: groups of sixteen rows of x (1, or 2 for 17 to 32 rows on eight waves): one decode of a code feeds an MFMA per
// group, the slices of the groups go through the wave's piece one after the other, and so do the sums at the end.
template <int NT, int U, int D, bool kTiled, int W = 16, int CG = 1>
__global__ __launch_bounds__(64 * W) void int8d_kernel(const int8_t *__restrict__ x, const uint16_t *__restrict__ codes,
                                                     const int64_t *__restrict__ codebook_abs,
                                                     int32_t *__restrict__ out, int M, int N, int K, int tiles_q,
                                                     int tiles_r)
{
    static_assert(W == 16 || W == 8, "sixteen waves for up to 8 rows of x, eight for up to 16");
    static_assert(CG == 1 || (CG == 2 && W == 8), "a second group of rows only beside a full first one");
    constexpr int kPiece = i8d_piece_bytes(W);
    constexpr int XR = kPiece / 256;   // rows of x a piece holds = columns of the product that are stored
    constexpr int XL = XR / 4;         // load instructions per slice, four rows each
    static_assert((U * NT) % D == 0, "the ring has to divide the unrolled loop");
    static_assert(NT <= 8, "the sums of the end go through the pieces four tiles at a time, twice at most");
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15;
    const int q = lane >> 4;
    const int n_steps = K >> 8;
    const int n_chunks = (n_steps + W - 1) / W;
    const int row_bytes = K >> 2;
    const uint32_t lane_base = (uint32_t)(lane & 31) * 8u;          // grid rows: [0, 64K)
    const uint32_t lane_base2 = lane_base | 0x10000u;               // mask rows: [64K, 128K)

    uint64_t entry = 0;
    if (tid < 256) entry = (uint64_t)codebook_abs[tid];

    // the wave's slice of the first chunk: load i is piece lane % 16 (16 bytes) of row 4 i + lane / 16; rows
    // past M lie past the end of the buffer (zeros, no memory access), and so does a k step that does not exist
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(x), 0, M * K, 0x00020000);
    constexpr int kOut = (int)0x80000000;
    const int xcoff = q * K + c16 * 16;
    auto x_soff = [&](int c, int i) { return c * W + wave < n_steps ? (c * W + wave) * 256 + i * 4 * K : kOut; };
    u4_t xv[CG][XL];   // load i of group g: rows 16 g + 4 i ..
#pragma unroll
    for (int g = 0; g < CG; g++)
#pragma unroll
        for (int i = 0; i < XL; i++) xv[g][i] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xcoff, x_soff(0, 4 * g + i), 0);
    // the wave's piece: row m at m * 256, its piece p in slot p ^ m.  Writes: row 4 i + h, piece lane % 16,
    // h = lane / 16, i.e. (xs_w ^ 64 i) + 1024 i.  Reads: row c16 % XR, piece 4 q + t, i.e. xs_r ^ 16 t (with 8-row
    // pieces columns 8 .. 15 of the product repeat 0 .. 7 and are not stored).
    const uint32_t piece = lds_addr(smem_raw) + (uint32_t)(2 * kI8TableBytes + wave * kPiece);
    const uint32_t xs_w = piece + (uint32_t)(q * 256 + ((c16 ^ q) << 4));
    const int xr_row = c16 & (XR - 1);
    const uint32_t xs_r = piece + (uint32_t)(xr_row * 256 + (((4 * q) ^ xr_row) << 4));

    const int t0 = (int)blockIdx.x * tiles_q + ((int)blockIdx.x < tiles_r ? (int)blockIdx.x : tiles_r);
    const int nt = tiles_q + ((int)blockIdx.x < tiles_r ? 1 : 0);   // <= NT (the host's business)

    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(codes), 0, (int)((int64_t)(kTiled ? ((N + 15) >> 4) * 16 : N) * row_bytes), 0x00020000);
    // row-major: row c16 of the tile, 16 bytes at quarter q.  Tiled: the tile row is 16 rows x K / 4 bytes as
    // well, a tile (4 code columns) is 128 bytes, and lane (g = c16 % 8, quarter q) reads 16 bytes at g * 16 of
    // tiles 2 q and 2 q + 1 of the step's 8.
    const int voff = kTiled ? q * 256 + (c16 & 7) * 16 : c16 * row_bytes + q * 16;
    const int tile_stride = 16 * row_bytes;
    const int step_stride = kTiled ? 1024 : 64;
    const int tile0_off = t0 * tile_stride;
    const uint32_t half_sel = (c16 & 8) ? 0x07060302u : 0x05040100u;   // tiled: which row of the pair is ours
    constexpr int kCw = kTiled ? 2 : 1;
    auto issue = [&](u4_t (&cwd)[kCw], int c, int t) {
        const int step = c * W + wave;
        const bool ok = t < nt && step < n_steps;
        const int so = ok ? tile0_off + t * tile_stride + step * step_stride : kOut;
        cwd[0] = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff, so, 0);
        if (kTiled) cwd[kCw - 1] = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff + 128, so, 0);
    };
    u4_t cw[D][kCw];
    issue(cw[0], 0, 0);

    // tables: threads 0 .. 255 write the 32 copies of table entry tid (16 slots of two copies),
    // threads 256 .. 511 those of the mask of high byte tid - 256
    bool bad = false;
    if (tid < 512) {
        uint64_t v = entry;
        if (tid < 256) {
            bad = (entry & 0x0303030303030303ull) != 0x0202020202020202ull;
        } else {
            const uint32_t t = (uint32_t)tid - 256u;
            uint32_t s8 = t & 0x7Fu;
            s8 |= (__builtin_popcount(s8) & 1u) << 7;
            v = (t >> 7) ? 0x0303030303030303ull : 0x0101010101010101ull;
#pragma unroll
            for (int d = 0; d < 8; d++)
                if ((s8 >> d) & 1u) v ^= 0xFCull << (8 * d);
        }
        const uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
        const uint32_t rowp = lds_addr(smem_raw) + (uint32_t)((tid * 16 + (tid & 15)) * 16);
#pragma unroll
        for (int i = 0; i < 16; i++) lds_write16(rowp ^ (uint32_t)(i * 16), u4_t{lo, hi, lo, hi});
    }
#pragma unroll
    for (int d = 1; d < D; d++) issue(cw[d], d / NT, d % NT);
    // the vote on the table: one word per wave in the area of the pieces, read by everybody after the barrier
    uint32_t *votes = reinterpret_cast<uint32_t *>(smem_raw + 2 * kI8TableBytes);
    const bool wave_bad = __builtin_amdgcn_ballot_w64(bad) != 0;
    if (lane == 0) votes[wave] = wave_bad ? 1u : 0u;
    __syncthreads();
    const bool any_bad = __builtin_amdgcn_ballot_w64(votes[lane & (W - 1)] != 0) != 0;
    __syncthreads();   // the votes are read before the first slice of x overwrites them
    if (any_bad) {
        // scalar decode for this workgroup's rows; the raw table goes where the pieces would
        uint64_t *table = reinterpret_cast<uint64_t *>(smem_raw + 2 * kI8TableBytes);
        if (tid < 256) table[tid] = entry;
        __syncthreads();
        const int64_t n_end = (int64_t)(t0 + nt) * 16 < N ? (int64_t)(t0 + nt) * 16 : N;
        int8_rows<false>(x, codes, table, table, out, M, N, K, kTiled ? 1 : 0, false, (int64_t)t0 * 16 + wave, W, n_end);
        return;
    }

    i4_t acc[NT][CG];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int g = 0; g < CG; g++) acc[t][g] = i4_t{0, 0, 0, 0};

    for (int c0 = 0; c0 < n_chunks; c0 += U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = c0 + u;
            const bool step_ok = (U == 1 || c < n_chunks) && c * W + wave < n_steps;
            // the slice through the wave's piece: in as loaded, out as the B operands of the four MFMAs
            // (the LDS serves a wave's instructions in order: the second group's slice may follow the first one's reads)
            u4_t xb[CG][4];
#pragma unroll
            for (int g = 0; g < CG; g++) {
#pragma unroll
                for (int i = 0; i < XL; i++) lds_write16((xs_w ^ (uint32_t)(64 * i)) + (uint32_t)(1024 * i), xv[g][i]);
#pragma unroll
                for (int t = 0; t < 4; t++) xb[g][t] = lds_read16(xs_r ^ (uint32_t)(16 * t));
#pragma unroll
                for (int i = 0; i < XL; i++)
                    xv[g][i] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xcoff, x_soff(c + 1, 4 * g + i), 0);
            }
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int slot = (u * NT + t) % D;
                if (step_ok && t < nt) {
                    u4_t w4;   // the lane's 8 codes of the step, two per word
                    if (kTiled) {
                        const u4_t &a = cw[slot][0], &b = cw[slot][kCw - 1];
                        w4 = u4_t{__builtin_amdgcn_perm(a[1], a[0], half_sel), __builtin_amdgcn_perm(a[3], a[2], half_sel),
                                  __builtin_amdgcn_perm(b[1], b[0], half_sel), __builtin_amdgcn_perm(b[3], b[2], half_sel)};
                    } else {
                        w4 = cw[slot][0];
                    }
                    u2_t g[8], m[8];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const uint32_t w = w4[i];
                        g[2 * i] = lds_read8(__builtin_amdgcn_perm(w, lane_base, 0x0C0C0400u));
                        m[2 * i] = lds_read8(__builtin_amdgcn_perm(w, lane_base2, 0x0C020500u));
                        g[2 * i + 1] = lds_read8(__builtin_amdgcn_perm(w, lane_base, 0x0C0C0600u));
                        m[2 * i + 1] = lds_read8(__builtin_amdgcn_perm(w, lane_base2, 0x0C020700u));
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const i4_t a = i4_t{(int)(g[2 * i][0] ^ m[2 * i][0]), (int)(g[2 * i][1] ^ m[2 * i][1]),
                                            (int)(g[2 * i + 1][0] ^ m[2 * i + 1][0]), (int)(g[2 * i + 1][1] ^ m[2 * i + 1][1])};
#pragma unroll
                        for (int g2 = 0; g2 < CG; g2++)
                            acc[t][g2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, __builtin_bit_cast(i4_t, xb[g2][i]), acc[t][g2], 0, 0, 0);
                    }
                }
                issue(cw[slot], c + (t + D) / NT, (t + D) % NT);   // the item D further on
            }
        }
    }
    // the sums, four tiles at a time, through the wave's own piece: cell (tile % 4, quarter, column) at slot
    // cell ^ wave, so that the 16 lanes of a reader, one per wave, meet no bank conflict; wave w adds up
    // XR / (W / 4) columns of tile w % 4 of the four (lanes of waves that do not exist add nothing)
#pragma unroll
    for (int g = 0; g < CG; g++) {
#pragma unroll
        for (int r0 = 0; r0 < NT; r0 += 4) {
            if (r0 > 0 && r0 >= nt) break;          // uniform
            if (g > 0 || r0 > 0) __syncthreads();   // the readers of the round before are done with the pieces
#pragma unroll
            for (int t = r0; t < r0 + 4 && t < NT; t++)
                if (t < nt && c16 < XR)
                    lds_write16(piece + (uint32_t)((((((t & 3) * 4 + q) * XR + c16) ^ wave)) << 4), __builtin_bit_cast(u4_t, acc[t][g]));
            __syncthreads();
            const int tw = wave & 3;
            if (r0 + tw < nt) {
                constexpr int kCols = XR / (W / 4);   // 2 with sixteen waves, 8 with eight
                const int sw = c16 & (W - 1);
                const uint32_t src = lds_addr(smem_raw) + (uint32_t)(2 * kI8TableBytes + sw * kPiece);
                const int n = (t0 + r0 + tw) * 16 + 4 * q;
#pragma unroll
                for (int j = 0; j < kCols; j++) {
                    const int m = kCols * (wave >> 2) + j;
                    i4_t v = __builtin_bit_cast(i4_t, lds_read16(src + (uint32_t)(((((tw * 4 + q) * XR + m) ^ sw)) << 4)));
                    if (W < 16 && c16 >= W) v = i4_t{0, 0, 0, 0};
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = row_sum16_i(v[e]);
                    if (c16 == 15 && 16 * g + m < M && n < N)   // N % 4 == 0, so the four rows are in range together
                        *reinterpret_cast<i4_t *>(out + (int64_t)(16 * g + m) * N + n) = v;
                }
            }
        }
    }
}

// ------------------------------------------------------------------ the integer operator, many rows of x
// Block tile 256 (n) x 128 (m), eight waves in two groups of four.  A group is a complete
// 256 x 128 x 64 pipeline - one wave per SIMD, each 64 rows of W (two 32-row tiles) x all 128 rows
// of x = 8 accumulators of v_mfma_i32_32x32x32_i8 - and the two groups take the even and the odd k
// tiles of the same output tile, so that every SIMD holds two waves working on different k tiles:
// while one waits for its table gathers or its x fragments the other's MFMAs run.  At the end each
// group hands the other the partial sums of one of its two row tiles through the LDS (the tables'
// space, by then free) and stores the other one.
// Like the half-precision gemm_reg_kernel, every wave decodes its own rows straight into A
// operands - here that is two 8-byte gathers and two exclusive ors per code (int8x_kernel's
// tables), eight codes per lane and k tile - and only x goes through the LDS: four buffers (two
// per group) of 128 rows x 64 bytes, the 16-byte pieces of a row exchanged by (row / 4) % 4 so
// that the 16 lanes the LDS serves per clock hit 16 different bank groups without padding (the
// tables take 128 KB of the 160).  Lane (row, half h = lane / 32) takes codes 4 h .. 4 h + 3 of its
// row's 8 in the k tile (8 consecutive bytes; in the reference's tile order, the 16 bytes of the
// pair of rows, of which one v_perm per two codes keeps ours) and pairs them with bytes 32 h ..
// 32 h + 31 of the x rows.
// The decode runs one k tile ahead of the MFMAs as a stream of units (the two codes of one row tile
// and MFMA step): a step gathers the table rows of two units and finishes (exclusive ors) the two
// gathered a step earlier, and scheduling hints weave that between the step's eight MFMAs.  Global
// loads run three of the group's k tiles ahead in a ring of registers; one barrier per pair of k
// tiles (one of either group).
// A table with a byte that is not 2 mod 4: the workgroup does its tile with the scalar decode.
typedef int i16_t __attribute__((ext_vector_type(16)));
constexpr int kI8gBN = 256, kI8gBM = 128, kI8gBK = 64;
constexpr int kI8gXBuf = kI8gBM * kI8gBK;                       // one x tile, unpadded
constexpr int kI8gSmem = 2 * kI8TableBytes + 4 * kI8gXBuf;      // 160 KB

template <bool kTiled>
__global__ __launch_bounds__(512) void int8g_kernel(const int8_t *__restrict__ x, const uint16_t *__restrict__ codes,
                                                    const int64_t *__restrict__ codebook_abs,
                                                    int32_t *__restrict__ out, int M, int N, int K)
{
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];
    unsigned char *xs = smem_raw + 2 * kI8TableBytes;   // x tiles: [group][buffer]
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2, w4 = wave & 3;            // group (k tile parity) and place along n
    const int gtid = tid & 255;
    const int l32 = lane & 31, kq = lane >> 5;
    const uint32_t lane_base = (uint32_t)(lane & 31) * 8u;   // grid rows: [0, 64K)
    const uint32_t lane_base2 = lane_base | 0x10000u;        // mask rows: [64K, 128K)
    const int m0 = blockIdx.x * kI8gBM;
    const int n0 = blockIdx.y * kI8gBN;
    const int row_bytes = K >> 2;
    const int k_tiles = K / kI8gBK;
    const int g_tiles = (k_tiles + 1) >> 1;              // tiles per group (the odd group's last may not exist)
    constexpr int kOut = (int)0x80000000;

    // global sources, as raw buffer loads (rows past N / M and tiles past the end: zeros, no access)
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(codes), 0, (int)((int64_t)(kTiled ? ((N + 15) >> 4) * 16 : N) * row_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t xrsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(x), 0, (int)((int64_t)M * K), 0x00020000);
    // codes of row tile i (32 rows): row-major 8 bytes at row * K / 4 + kt * 16 + 8 h; tiled: tile
    // (row / 16, 2 kt + h) of 128 bytes, 16 bytes at (row % 8) * 16
    int cvoff[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int n = n0 + w4 * 64 + i * 32 + l32;
        if (kTiled) cvoff[i] = n < N ? (n >> 4) * 16 * row_bytes + kq * 128 + (n & 7) * 16 : kOut;
        else cvoff[i] = n < N ? n * row_bytes + kq * 8 : kOut;
    }
    const uint32_t half_sel = (l32 & 8) ? 0x07060302u : 0x05040100u;   // tiled: which row of the pair is ours
    // x: thread gtid of a group loads piece gtid % 4 (16 bytes) of rows gtid / 4 and gtid / 4 + 64 of the
    // group's tile; in the LDS piece p of row r sits at r * 64 + (p ^ (r / 4) % 4) * 16
    int xvoff[2];
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const int m = m0 + (gtid >> 2) + 64 * p;
        xvoff[p] = m < M ? m * K + (gtid & 3) * 16 : kOut;
    }
    unsigned char *xg = xs + grp * 2 * kI8gXBuf;   // this group's two buffers
    unsigned char *xw_ptr = xg + (gtid >> 2) * 64 + (((gtid & 3) ^ ((gtid >> 4) & 3)) << 4);
    const uint32_t swz = (uint32_t)(l32 >> 2) & 3u;
    const uint32_t xr_addr = lds_addr(xg) + (uint32_t)(l32 * 64);
    const uint32_t xr_off[2] = {(((uint32_t)kq * 2u) ^ swz) << 4, (((uint32_t)kq * 2u + 1u) ^ swz) << 4};

    struct Stage {
        u4_t cw[2];   // row-major: only the low 8 bytes are loaded
        u4_t xv[2];
    };
    auto load = [&](Stage &st, int t) {   // t: the group's tile, k tile 2 t + grp
        const int kt = 2 * t + grp;
        const int ok = kt < k_tiles;
        const int coff = ok ? (kTiled ? kt * 256 : kt * 16) : kOut;
        const int xoff = ok ? kt * kI8gBK : kOut;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if (kTiled) {
                st.cw[i] = __builtin_amdgcn_raw_buffer_load_b128(crsrc, cvoff[i], coff, 0);
            } else {
                const u2_t v = __builtin_amdgcn_raw_buffer_load_b64(crsrc, cvoff[i], coff, 0);
                st.cw[i] = u4_t{v[0], v[1], 0u, 0u};
            }
        }
#pragma unroll
        for (int p = 0; p < 2; p++) st.xv[p] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xvoff[p], xoff, 0);
    };
    auto stage_x = [&](const Stage &st, int buf) {
#pragma unroll
        for (int p = 0; p < 2; p++) *reinterpret_cast<u4_t *>(xw_ptr + buf * kI8gXBuf + p * 64 * 64) = st.xv[p];
    };
    Stage ring[3];
#pragma unroll
    for (int d = 0; d < 3; d++) load(ring[d], d);

    // tables: threads 0 .. 255 write the 32 copies of table entry tid, threads 256 .. 511 those of
    // the mask of high byte tid - 256 (the mask table follows the grid table: row tid either way)
    const uint64_t entry = tid < 256 ? (uint64_t)codebook_abs[tid] : 0x0202020202020202ull;
    {
        uint64_t v = entry;
        if (tid >= 256) {
            const uint32_t t = (uint32_t)tid - 256u;
            uint32_t s8 = t & 0x7Fu;
            s8 |= (__builtin_popcount(s8) & 1u) << 7;
            v = (t >> 7) ? 0x0303030303030303ull : 0x0101010101010101ull;
#pragma unroll
            for (int d = 0; d < 8; d++)
                if ((s8 >> d) & 1u) v ^= 0xFCull << (8 * d);
        }
        u4_t *rowp = reinterpret_cast<u4_t *>(smem_raw) + tid * 16;
        const u4_t vv = u4_t{(uint32_t)v, (uint32_t)(v >> 32), (uint32_t)v, (uint32_t)(v >> 32)};
#pragma unroll
        for (int i = 0; i < 16; i++) rowp[(i + tid) & 15] = vv;   // 16 lanes, 16 bank groups
    }
    // the vote on the table (one word per wave in the x area, read by everybody after the barrier)
    {
        uint32_t *votes = reinterpret_cast<uint32_t *>(xs);
        const bool bad = (entry & 0x0303030303030303ull) != 0x0202020202020202ull;
        const bool wave_bad = __builtin_amdgcn_ballot_w64(bad) != 0;
        if (lane == 0) votes[wave] = wave_bad ? 1u : 0u;
        __syncthreads();
        const bool any_bad = (votes[0] | votes[1] | votes[2] | votes[3]) != 0;   // the table is in waves 0 - 3
        __syncthreads();   // the votes are read before x overwrites them
        if (any_bad) {
            uint64_t *table = reinterpret_cast<uint64_t *>(xs);
            if (tid < 256) table[tid] = entry;
            __syncthreads();
            const int64_t n_end = (int64_t)n0 + kI8gBN < N ? (int64_t)n0 + kI8gBN : N;
            const int64_t mc = M - m0 < kI8gBM ? M - m0 : kI8gBM;
            int8_rows<false>(x + (int64_t)m0 * K, codes, table, table, out + (int64_t)m0 * N, mc, N, K, kTiled ? 1 : 0,
                             false, (int64_t)n0 + wave, 8, n_end);
            return;
        }
    }

    i16_t acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0;

    // unit u of a tile: the two codes (8 weights each) of row tile u % 2 and MFMA step u / 2
    struct Unit {
        u2_t g[2], k[2];
    };
    i4_t afr[2][2][2];   // A operands: [buffer][row tile][MFMA step]
    auto unit_gather = [&](Unit &o, const Stage &st, int u) {
        const int i = u & 1, s2 = u >> 1;
        const uint32_t w = kTiled ? __builtin_amdgcn_perm(st.cw[i][2 * s2 + 1], st.cw[i][2 * s2], half_sel) : st.cw[i][s2];
        o.g[0] = lds_read8(__builtin_amdgcn_perm(w, lane_base, 0x0C0C0400u));
        o.k[0] = lds_read8(__builtin_amdgcn_perm(w, lane_base2, 0x0C020500u));
        o.g[1] = lds_read8(__builtin_amdgcn_perm(w, lane_base, 0x0C0C0600u));
        o.k[1] = lds_read8(__builtin_amdgcn_perm(w, lane_base2, 0x0C020700u));
    };
    auto unit_finish = [&](const Unit &o, int abuf, int u) {
        afr[abuf][u & 1][u >> 1] = i4_t{(int)(o.g[0][0] ^ o.k[0][0]), (int)(o.g[0][1] ^ o.k[0][1]),
                                        (int)(o.g[1][0] ^ o.k[1][0]), (int)(o.g[1][1] ^ o.k[1][1])};
    };
    Unit ga[2], gb[2];   // units 0, 1 (MFMA step 0) and 2, 3 (step 1) in flight

    auto read_b = [&](u4_t (&b)[4], int buf, int s2) {
#pragma unroll
        for (int j = 0; j < 4; j++) b[j] = lds_read16(xr_addr + (uint32_t)(buf * kI8gXBuf + j * 32 * 64) + xr_off[s2]);
    };
    stage_x(ring[0], 0);
    unit_gather(ga[0], ring[0], 0);
    unit_gather(ga[1], ring[0], 1);
    unit_finish(ga[0], 0, 0);
    unit_finish(ga[1], 0, 1);
    unit_gather(gb[0], ring[0], 2);
    unit_gather(gb[1], ring[0], 3);
    __syncthreads();   // x tile 0 of either group staged

    // MFMAs of the group's tile t (A = afr[buf], B from the group's x buffer buf).  Step 0 finishes the
    // tile's own second pair of units (gathered in the last step of the tile before), gathers the first
    // pair of tile t + 1 (registers sn), writes the x of tile t + 1 to buffer buf ^ 1 and fetches tile
    // t + 3 into sf; step 1 finishes that pair into afr[buf ^ 1] and gathers the second.  Each step
    // reads its own x fragments as it starts: the SIMD's other wave covers the wait.
    auto tile = [&](int t, int buf, const Stage &sn, Stage &sf) {
        u4_t b[4];
        read_b(b, buf, 0);
        unit_finish(gb[0], buf, 2);
        unit_finish(gb[1], buf, 3);
        unit_gather(ga[0], sn, 0);
        unit_gather(ga[1], sn, 1);
        stage_x(sn, buf ^ 1);
        load(sf, t + 3);
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(afr[buf][i][0], __builtin_bit_cast(i4_t, b[j]), acc[i][j], 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 8; r++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                // MFMA
            if (r < 4) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);     // LDS reads
            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);                // VALU
            if (r == 4) __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);    // LDS writes
            if (r >= 4) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);    // global loads
        }
        __builtin_amdgcn_sched_barrier(0);
        read_b(b, buf, 1);
        unit_finish(ga[0], buf ^ 1, 0);
        unit_finish(ga[1], buf ^ 1, 1);
        unit_gather(gb[0], sn, 2);
        unit_gather(gb[1], sn, 3);
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(afr[buf][i][1], __builtin_bit_cast(i4_t, b[j]), acc[i][j], 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 8; r++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                // MFMA
            if (r < 4) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);     // LDS reads
            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);                // VALU
        }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    };

    // both groups make the same number of trips (the barriers are the workgroup's); six tiles per trip
    // so that ring slot and x buffer are compile-time constants
    int t = 0;
    for (; t + 6 <= g_tiles; t += 6) {
        tile(t, 0, ring[1], ring[0]);
        tile(t + 1, 1, ring[2], ring[1]);
        tile(t + 2, 0, ring[0], ring[2]);
        tile(t + 3, 1, ring[1], ring[0]);
        tile(t + 4, 0, ring[2], ring[1]);
        tile(t + 5, 1, ring[0], ring[2]);
    }
    if (t < g_tiles) tile(t, 0, ring[1], ring[0]);
    if (t + 1 < g_tiles) tile(t + 1, 1, ring[2], ring[1]);
    if (t + 2 < g_tiles) tile(t + 2, 0, ring[0], ring[2]);
    if (t + 3 < g_tiles) tile(t + 3, 1, ring[1], ring[0]);
    if (t + 4 < g_tiles) tile(t + 4, 0, ring[2], ring[1]);

    // The two groups hold partial sums of the same 256 x 128 outputs.  Group g keeps row tile g of
    // each of its waves' two and gets the other group's sums for it through the LDS: wave (g, w4)
    // leaves row tile 1 - g in slot (g, w4), 16 KB of the tables' space, and adds slot (1 - g, w4).
    {
        int *slot_w = reinterpret_cast<int *>(smem_raw) + (grp * 4 + w4) * 4096 + lane;
        const int *slot_r = reinterpret_cast<const int *>(smem_raw) + ((1 - grp) * 4 + w4) * 4096 + lane;
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) slot_w[(j * 16 + e) * 64] = grp == 0 ? acc[1][j][e] : acc[0][j][e];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int v = slot_r[(j * 16 + e) * 64];
                if (grp == 0) acc[0][j][e] += v;
                else acc[1][j][e] += v;
            }
    }

    // D layout of 32x32: element e of lane: row (n) = 8 * (e / 4) + 4 * (lane / 32) + e % 4, column (m) = lane % 32
    const bool n_vec = (N & 3) == 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int m = m0 + j * 32 + l32;
        if (m >= M) continue;
#pragma unroll
        for (int e4 = 0; e4 < 4; e4++) {
            const int n = n0 + w4 * 64 + grp * 32 + 8 * e4 + 4 * kq;
            int32_t *dst = out + (int64_t)m * N + n;
            i4_t v;
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = grp == 0 ? acc[0][j][4 * e4 + e] : acc[1][j][4 * e4 + e];
            if (n_vec && n + 3 < N) {
                *reinterpret_cast<i4_t *>(dst) = v;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < N) dst[e] = v[e];
            }
        }
    }
}

__global__ void zero_i32_kernel(int32_t *y, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        y[i] = 0;
}
