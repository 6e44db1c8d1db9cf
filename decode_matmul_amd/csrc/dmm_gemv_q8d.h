// Batch 1 on 8-bit operands with every tile of a workgroup in registers from start to end.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ batch 1, 8-bit operands, resident accumulators
// gemv_q8c_kernel's arithmetic (fp8 weights by two 8-byte gathers and two exclusive ors per code, x as
// four bf8 terms staged 4096 values at a time, the shift term through the per-code means) for
// workgroups of up to NT tiles, arranged so that the k loop is decode and nothing else:
//   * ONE accumulator (four registers) per tile.  The three MFMAs of a tile's k step - fp8 x bf8 for
//     each half of the step's 256 k, 16-bit for the shift term - take B operands of their own whose
//     idle columns are zero, and all add into columns 0 .. 3 of the same accumulator: column t is
//     term t of x (weight 8^-t), and the two halves of the per-code means ride in columns 0 and 1,
//     the low half times 8 to meet the weight of its column.  So the accumulators of all NT tiles
//     stay in registers for the whole launch, the workgroup goes through x once (chunk outside,
//     tiles inside, whatever the number of tiles), the five B operand reads of a chunk serve every
//     tile, and nothing is added up, published or waited for until the very end.
//   * The code stream is a ring of D loads per wave over the items (chunk, tile) in that order, D
//     dividing the U * NT items of the U-fold unrolled chunk loop, so slots and accumulators are
//     static registers; an item is asked for D items ahead of its use.  Tiles past the workgroup's
//     share and steps past K are out-of-range offsets: zeros, no memory access, no decode.
//   * At the end every wave leaves columns 0 .. 3 of its accumulators in the LDS - in the x buffer that
//     the last chunk does not use and the free space behind it, so nobody has to be waited for first -
//     and after the launch's one closing barrier wave t adds tile t up: four columns with their weights,
//     then the 16 waves by DPP.
// The hand-over to the 16-bit kernel (a grid fp8 cannot hold, an x that is not finite) is the
// chunked kernel's.
// LDS map: tables [0, 96K), 16 vote words and 2 words for what the stagers find, two x buffers (4 term
// rows, 2 rows of means, 64 zero bytes for the B operands' idle columns; chunk c sits in buffer
// (n_chunks - 1 - c) % 2, the last one in buffer 0), and from buffer 1 on the partial sums of the end.
constexpr int kQdXBuf = kQcXBuf + 64;
constexpr int kQdRedWave = 4 * 4 * 16 + 16;        // 4 quarters x 4 columns of float4, padded: lane w of a reader hits bank group w
constexpr int kQdRedTile = 16 * kQdRedWave;
constexpr int kQdMaxTiles = 8;
__host__ __device__ constexpr int qd_lds_bytes()
{
    return kSTablesBytes + 128 + kQdXBuf + (kQdXBuf > kQdMaxTiles * kQdRedTile ? kQdXBuf : kQdMaxTiles * kQdRedTile);
}

// qc_split_piece with the low half of the mean times 8 (exact: it lies 11 bits below the high half)
__device__ __forceinline__ bool qd_split_piece(const u4_t &v, u2_t (&t)[4], uint32_t &mean_hi_lo8)
{
    const h2_t ones = h2_t{(half_t)1.0f, (half_t)1.0f};
    float r = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) r = __builtin_amdgcn_fdot2(as_h2(v[i]), ones, r, false);
    const bool finite = (__builtin_bit_cast(uint32_t, r) & 0x7F800000u) != 0x7F800000u;
    r *= 0.125f;
    const half_t hi = (half_t)r;
    const half_t lo = (half_t)((r - (float)hi) * 8.f);
    mean_hi_lo8 = as_u32(h2_t{hi, lo});
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

// One tile's 256-wide k step: 8 code words of the lane -> 16 gathers, 16 exclusive ors, 3 MFMAs into acc.
__device__ __forceinline__ void qd_tile_step(const u4_t &cw, uint32_t lane_base, const i8_t &xb0, const i8_t &xb1,
                                             const h8_t &xm, f4_t &acc)
{
    Q8Gather gt[4];
#pragma unroll
    for (int t2 = 0; t2 < 4; t2++) q8_gather(gt[t2], cw[t2], lane_base);
    u4_t a8;   // +-2.0 per code, the shift term's A operand: the code words' shift bits over the bits of 2.0
#pragma unroll
    for (int i = 0; i < 4; i++) a8[i] = bfi(0x80008000u, cw[i], 0x40004000u);
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const Q8Gather &b0 = gt[2 * h], &b1 = gt[2 * h + 1];
        const i8_t a = i8_t{(int)(b0.g0[0] ^ b0.s0[0]), (int)(b0.g0[1] ^ b0.s0[1]), (int)(b0.g1[0] ^ b0.s1[0]),
                            (int)(b0.g1[1] ^ b0.s1[1]), (int)(b1.g0[0] ^ b1.s0[0]), (int)(b1.g0[1] ^ b1.s0[1]),
                            (int)(b1.g1[0] ^ b1.s1[0]), (int)(b1.g1[1] ^ b1.s1[1])};
        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, h == 0 ? xb0 : xb1, acc, 0 /* A: fp8 */, 1 /* B: bf8 */, 0, 0, 0, 0);
        if (h == 0) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8_t, a8), xm, acc, 0, 0, 0);
    }
}

template <int NT, int U, int D, bool kPacked>
__global__ __launch_bounds__(1024) void gemv_q8d_kernel(const uint16_t *__restrict__ x,
                                                        const uint16_t *__restrict__ codes,
                                                        const void *__restrict__ grid, float scale,
                                                        uint16_t *__restrict__ y, int N, int K, int tiles_q, int tiles_r)
{
    constexpr int W = 16;
    static_assert((U * NT) % D == 0, "the ring has to divide the unrolled loop");
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];
    static_assert(NT <= kQdMaxTiles, "the partial sums of the end are sized for kQdMaxTiles tiles");
    uint32_t *flags = reinterpret_cast<uint32_t *>(smem_raw + kSTablesBytes);   // [0 .. 15]: one vote per wave; [16], [17]: the stagers' finds
    unsigned char *xbuf = smem_raw + kSTablesBytes + 128;

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
    // x through a buffer resource: a wave with nothing to stage asks for an out-of-range piece and gets
    // zeros, so every wave issues the same loads and the wait counters stay exact
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(x), 0, K * 2, 0x00020000);
    constexpr int kOut = (int)0x80000000;
    const int sp = tid & 511;
    u4_t xpiece = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, sp * 16, wave < 8 ? 0 : kOut, 0);

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
    // The first items of the code stream.  The memory pipeline of a compute unit takes a row-major code
    // load apart in about 64 clocks (16 rows, 16 pages) and serves loads in the order they were issued,
    // so every code load that goes out ahead of the prologue's own loads (grid rows, x) delays the tables
    // by that much, and a wave that asks for more than the pipeline holds blocks at the issue and writes
    // no tables meanwhile.  One item per wave goes out here, the rest of the ring after the wave's share
    // of the prologue's work, ahead of the barrier: they are back when the barrier opens.
    constexpr int kFirst = 1;
#pragma unroll
    for (int d = 0; d < kFirst; d++) issue(cw[d], d / NT, d % NT);

    // one piece of x -> its terms and means in buffer `buf` (piece p of the chunk); returns finite
    auto stage_piece = [&](const u4_t &v, int buf, int p) {
        u2_t tm[4];
        uint32_t mb;
        const bool fin = qd_split_piece(v, tm, mb);
        unsigned char *xb = xbuf + buf * kQdXBuf;
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
        const u2_t sb = sign_bytes((uint32_t)row);
        const uint32_t sg = lds_addr(smem_raw) + (uint32_t)((row * 16 + (t & 1) * 8 + (row & 7)) * 16);
#pragma unroll
        for (int i = 0; i < 8; i++) lds_write16(sg ^ (uint32_t)(i * 16), u4_t{sb[0], sb[1], sb[0], sb[1]});
        // the zero bytes behind each x buffer, and the stagers' two words
        if (t < 8) *reinterpret_cast<u4_t *>(xbuf + (t >> 2) * kQdXBuf + kQcXBuf + (t & 3) * 16) = u4_t{0u, 0u, 0u, 0u};
        if (t == 8) flags[16] = flags[17] = 0u;
    } else if (wave >= 8) {
        bool exact;
        const u2_t g8 = grid_row_fp8(grow, exact);
        fits = exact;
        const int r = tid - 512;
        const uint32_t gg = lds_addr(smem_raw) + (uint32_t)(kSSignBytes + (r * 16 + (r & 15)) * 16);   // slot i ^ (r % 16)
#pragma unroll
        for (int i = 0; i < 16; i++) lds_write16(gg ^ (uint32_t)(i * 16), u4_t{g8[0], g8[1], g8[0], g8[1]});
    } else {
        fits = stage_piece(xpiece, (n_chunks - 1) & 1, sp);   // pieces past the end of x are zeros
    }
#pragma unroll
    for (int d = kFirst; d < D; d++) issue(cw[d], d / NT, d % NT);
    {
        const bool wave_bad = __builtin_amdgcn_ballot_w64(!fits) != 0;
        if (lane == 0) flags[wave] = wave_bad ? 1u : 0u;
    }
    __syncthreads();
    bool hand_over = __builtin_amdgcn_ballot_w64(flags[lane & (W - 1)] != 0) != 0;

    // B operands of this lane (offsets inside an x buffer): columns 0 .. 3 read term c16 of the wave's k step
    // (32 bytes per MFMA half), columns 0 and 1 the two halves of the means; every other column the zeros
    const uint32_t xb_lds = lds_addr(xbuf);
    const uint32_t xt_off = xb_lds + (c16 < 4 ? (uint32_t)(c16 * kQcTermPitch + q * 64 + wave * 256) : (uint32_t)kQcXBuf);
    const uint32_t xm_off = xb_lds + (c16 < 2 ? (uint32_t)(4 * kQcTermPitch + c16 * kQcMeanPitch + q * 16 + wave * 64) : (uint32_t)kQcXBuf);

    f4_t acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = f4_t{0.f, 0.f, 0.f, 0.f};

    for (int c0 = 0; c0 < n_chunks && !hand_over; c0 += U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = c0 + u;
            const bool exists = U == 1 || c < n_chunks;
            // the chunk after this one is split by waves 0-7 while everybody multiplies this one
            const bool stage_next = exists && c + 1 < n_chunks;
            xpiece = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, sp * 16, stage_next && wave < 8 ? (c + 1) * 8192 : kOut, 0);
            const bool step_ok = exists && c * W + wave < n_steps;
            i8_t xb0 = i8_t{0, 0, 0, 0, 0, 0, 0, 0}, xb1 = xb0;
            h8_t xm = __builtin_bit_cast(h8_t, u4_t{0u, 0u, 0u, 0u});
            if (step_ok) {
                const uint32_t bo = (uint32_t)(((n_chunks - 1 - c) & 1) * kQdXBuf);
                const u4_t r0 = lds_read16(xt_off + bo), r1 = lds_read16(xt_off + bo + 16);
                const u4_t r2 = lds_read16(xt_off + bo + 32), r3 = lds_read16(xt_off + bo + 48);
                xm = __builtin_bit_cast(h8_t, lds_read16(xm_off + bo));
                xb0 = i8_t{(int)r0[0], (int)r0[1], (int)r0[2], (int)r0[3], (int)r1[0], (int)r1[1], (int)r1[2], (int)r1[3]};
                xb1 = i8_t{(int)r2[0], (int)r2[1], (int)r2[2], (int)r2[3], (int)r3[0], (int)r3[1], (int)r3[2], (int)r3[3]};
            }
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int slot = (u * NT + t) % D;
                if (step_ok && t < nt) qd_tile_step(cw[slot], lane_base, xb0, xb1, xm, acc[t]);
                issue(cw[slot], c + (t + D) / NT, (t + D) % NT);   // the item D further on
            }
            if (stage_next && wave < 8 && !stage_piece(xpiece, (n_chunks - 2 - c) & 1, sp)) flags[16 + (c & 1)] = 1u;
            if (stage_next) {
                __syncthreads();   // hands the x buffer over
                if (__builtin_amdgcn_ballot_w64(flags[16 + (c & 1)] != 0) != 0) hand_over = true;
            }
        }
    }
    // columns 0 .. 3 of every accumulator into the LDS, [tile][wave][quarter][column], from x buffer 1 on: the
    // chunk that sat there has been read by everybody before the barrier that handed the last chunk over
    const uint32_t red = lds_addr(xbuf) + (uint32_t)kQdXBuf;
    if (!hand_over) {
#pragma unroll
        for (int t = 0; t < NT; t++)
            if (t < nt && c16 < 4)
                lds_write16(red + (uint32_t)(t * kQdRedTile + wave * kQdRedWave + (q * 4 + c16) * 16), __builtin_bit_cast(u4_t, acc[t]));
    }
    __syncthreads();   // the launch's closing barrier: every partial sum is there (or everybody has read the flags)
    if (hand_over) {
        gemv_stream_body<1, W, 2, kPacked, 4>(x, codes, grid, scale, y, 1, N, K, tiles_q, tiles_r);
        return;
    }
    if (wave < nt) {
        // wave t adds up tile t: lane (w, quarter) takes wave w's 4 columns with their weights 8^-c, then
        // the 16 lanes of a row are added with DPP shifts
        const uint32_t src = red + (uint32_t)(wave * kQdRedTile + c16 * kQdRedWave + q * 64);
        f4_t v = __builtin_bit_cast(f4_t, lds_read16(src));
#pragma unroll
        for (int cc = 1; cc < 4; cc++)
            v += __builtin_bit_cast(f4_t, lds_read16(src + cc * 16)) * __builtin_bit_cast(float, 0x3F800000u - ((uint32_t)cc * 3u << 23));
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = row_sum16(v[e]);
        const int n = (t0 + wave) * 16 + 4 * q;
        if (c16 == 15 && n < N) {   // N % 4 == 0, so the four rows are in range together
            h4_t o;
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = (half_t)(v[e] * scale);
            *reinterpret_cast<h4_t *>(y + n) = o;
        }
    }
}
