// One to four rows of x on 16-bit operands with x taken in chunks and every tile of a workgroup in registers.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ 16-bit operands, chunked x, resident accumulators
// The streaming kernel keeps all of x in the LDS beside the tables, which stops at M * (2 K + 16) = 64 KB:
// four rows of K = 8192, two of K = 28672 no longer fit, and such calls went to the small-batch kernel with its
// eight waves and its x slices from L2.  This kernel has the streaming kernel's tables, decode and MFMA (one
// code = two 16-byte gathers, four packed FMAs, one v_mfma_f32_16x16x32_f16 whose B column m is row m of x) and
// the loop order of the batch-1 kernel on 8-bit operands:
//   * x goes through ONE LDS buffer 4096 values (16 k steps, one per wave) at a time.  At the start of a chunk
//     a wave reads the B operands of its k step - 8 registers sets, one per MFMA of a tile step - and keeps
//     them for every tile of the workgroup; after the barrier that follows nobody reads the buffer any more,
//     and all waves copy the next chunk into it (loaded from global memory before the tile steps, written
//     after them) ahead of the barrier that opens the next chunk.  Two barriers per chunk, none per tile.
//   * chunk outside, tiles inside: the accumulators of all NT tiles of the workgroup's share stay in registers
//     for the whole launch (one per tile: a second one to alternate the MFMAs between bought nothing, and
//     with one the sums do not depend on how many tiles a workgroup has), and the code stream is a ring of D
//     loads per wave over the items (chunk, tile).
//   * at the end every wave leaves columns 0 .. 3 of its accumulators (rows 0 .. 3 of x) in the LDS, where the
//     x buffer was, and after one barrier wave t adds tile t up over the 16 waves by DPP and stores y.
// Any grid of finite halves, any x: the arithmetic is the streaming kernel's (fp32 sums of exact products),
// only the order of the sums differs.
// LDS map: tables [0, 96K), then the x buffer (4 rows of 8192 + 16 bytes: rows read together fall into
// different bank groups), which the partial sums of the end reuse.
constexpr int kFdRows = 4;
constexpr int kFdPitch = 4096 * 2 + 16;
constexpr int kFdXBytes = kFdRows * kFdPitch;
constexpr int kFdRedWave = 4 * 4 * 16 + 16;        // 4 quarters x 4 columns of float4, padded: lane w of a reader hits bank group w
constexpr int kFdRedTile = 16 * kFdRedWave;
constexpr int kFdMaxTiles = 8;
__host__ __device__ constexpr int fd_lds_bytes()
{
    return kSTablesBytes + (kFdXBytes > kFdMaxTiles * kFdRedTile ? kFdXBytes : kFdMaxTiles * kFdRedTile);
}

// One tile's 256-wide k step: 8 codes of the lane -> 16 gathers, 32 packed FMAs, 8 MFMAs into acc.
__device__ __forceinline__ void fd_tile_step(const u4_t &cw, uint32_t lane_base, uint32_t quarter_bits,
                                             const u4_t (&xb)[8], f4_t &acc)
{
    StreamGather buf[2];
    stream_gather(buf[0], cw[0], lane_base, quarter_bits);
#pragma unroll
    for (int t2 = 0; t2 < 4; t2++) {
        if (t2 + 1 < 4) stream_gather(buf[(t2 + 1) & 1], cw[t2 + 1], lane_base, quarter_bits);
        const StreamGather &b = buf[t2 & 1];
        const h8_t a0 = stream_finish<false>(b.g0, b.s0, b.dd);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, __builtin_bit_cast(h8_t, xb[2 * t2]), acc, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        const h8_t a1 = stream_finish<true>(b.g1, b.s1, b.dd);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, __builtin_bit_cast(h8_t, xb[2 * t2 + 1]), acc, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <int NT, int U, int D, bool kPacked>
__global__ __launch_bounds__(1024) void gemv_f16d_kernel(const uint16_t *__restrict__ x,
                                                         const uint16_t *__restrict__ codes,
                                                         const void *__restrict__ grid, float scale,
                                                         uint16_t *__restrict__ y, int M, int N, int K, int tiles_q,
                                                         int tiles_r)
{
    constexpr int W = 16;
    static_assert((U * NT) % D == 0, "the ring has to divide the unrolled loop");
    static_assert(NT <= kFdMaxTiles, "the partial sums of the end are sized for kFdMaxTiles tiles");
    extern __shared__ __attribute__((aligned(256))) unsigned char smem_raw[];
    unsigned char *xbuf = smem_raw + kSTablesBytes;

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

    // ---- prologue: the grid row of the first 256 threads and the first chunk of x, then one code word
    const u4_t grow = tid < 256 ? reinterpret_cast<const u4_t *>(grid)[tid] : u4_t{0u, 0u, 0u, 0u};
    // a chunk of x is up to 4 rows of 512 pieces (16 bytes); thread tid copies piece tid % 512 of rows
    // tid / 512 and tid / 512 + 2.  Rows past M are not asked for (an offset out of range: zeros, no memory
    // access); pieces past K are whatever follows in x - no k step past K is ever multiplied.
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(x), 0, M * K * 2, 0x00020000);
    constexpr int kOut = (int)0x80000000;
    const int xrow = wave >> 3;                       // uniform: 0 or 1 (+ 2 for the second piece)
    const int xvoff = (tid & 511) * 16;
    auto x_soff = [&](int u, int c, bool on) { return on && xrow + 2 * u < M ? ((xrow + 2 * u) * K + c * 4096) * 2 : kOut; };
    const uint32_t xw = lds_addr(xbuf) + (uint32_t)(xrow * kFdPitch + (tid & 511) * 16);
    u4_t xv[2];
#pragma unroll
    for (int u = 0; u < 2; u++) xv[u] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xvoff, x_soff(u, 0, true), 0);

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
    // grid and x loads delays the tables by the time the memory pipeline takes it apart)
    issue(cw[0], 0, 0);

    stream_stage_signs<64 * W>(smem_raw, tid);
    __builtin_amdgcn_sched_barrier(0);   // keep the sign rows ahead of the waits for the loads
#pragma unroll
    for (int u = 0; u < 2; u++)
        if (xrow + 2 * u < M) lds_write16(xw + (uint32_t)(2 * u * kFdPitch), xv[u]);
    stream_stage_grid<64 * W>(smem_raw, grow, tid);
#pragma unroll
    for (int d = 1; d < D; d++) issue(cw[d], d / NT, d % NT);
    __syncthreads();

    // B operand address of this lane: column c16 is row c16 of x (columns past M read row 0; their
    // columns of the product are never looked at), quarter q, the wave's k step of the chunk
    const uint32_t xlane = lds_addr(xbuf) + (uint32_t)((c16 < M ? c16 : 0) * kFdPitch + wave * 512 + q * 128);

    f4_t acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = f4_t{0.f, 0.f, 0.f, 0.f};

    for (int c0 = 0; c0 < n_chunks; c0 += U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = c0 + u;
            const bool exists = U == 1 || c < n_chunks;
            const bool step_ok = exists && c * W + wave < n_steps;
            u4_t xb[8];
#pragma unroll
            for (int i = 0; i < 8; i++) xb[i] = step_ok ? lds_read16(xlane + (uint32_t)(i * 16)) : u4_t{0u, 0u, 0u, 0u};
            if (exists) __syncthreads();   // everybody has its operands: the buffer is free for the next chunk
            const bool stage_next = exists && c + 1 < n_chunks;
#pragma unroll
            for (int v = 0; v < 2; v++) xv[v] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xvoff, x_soff(v, c + 1, stage_next), 0);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int slot = (u * NT + t) % D;
                if (step_ok && t < nt) fd_tile_step(cw[slot], lane_base, quarter_bits, xb, acc[t]);
                issue(cw[slot], c + (t + D) / NT, (t + D) % NT);   // the item D further on
            }
            if (stage_next) {
#pragma unroll
                for (int v = 0; v < 2; v++)
                    if (xrow + 2 * v < M) lds_write16(xw + (uint32_t)(2 * v * kFdPitch), xv[v]);
                __syncthreads();   // the next chunk is in
            }
        }
    }
    // columns 0 .. 3 of every tile's sum into the LDS, [tile][wave][quarter][column], where the x buffer was:
    // nobody has read that since the barrier after the last chunk's operand reads
    const uint32_t red = lds_addr(xbuf);
#pragma unroll
    for (int t = 0; t < NT; t++)
        if (t < nt && c16 < 4)
            lds_write16(red + (uint32_t)(t * kFdRedTile + wave * kFdRedWave + (q * 4 + c16) * 16), __builtin_bit_cast(u4_t, acc[t]));
    __syncthreads();
    if (wave < nt) {
        // wave t adds up tile t: lane (w, quarter) takes wave w's sums of the quarter's four rows for each
        // row of x, then the 16 lanes of a row are added with DPP shifts
        const uint32_t src = red + (uint32_t)(wave * kFdRedTile + c16 * kFdRedWave + q * 64);
        const int n = (t0 + wave) * 16 + 4 * q;
#pragma unroll
        for (int m = 0; m < 4; m++) {
            f4_t v = __builtin_bit_cast(f4_t, lds_read16(src + (uint32_t)(m * 16)));
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = row_sum16(v[e]);
            if (c16 == 15 && m < M && n < N) {   // N % 4 == 0, so the four rows are in range together
                h4_t o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = (half_t)(v[e] * scale);
                *reinterpret_cast<h4_t *>(y + (int64_t)m * N + n) = o;
            }
        }
    }
}
