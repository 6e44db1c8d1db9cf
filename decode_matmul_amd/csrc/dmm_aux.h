// Offline repack of the codes and the plain read probe.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ offline repack for the streaming kernel
// packed[((tile * n_steps + step) * 64 + lane) * 8 + e] = codes[16 tile + lane % 16][32 step + 8 (lane / 16) + e]
// (16-bit units; rows past N are zeros).  One thread moves one 16-byte piece.
__global__ __launch_bounds__(256) void pack_kernel(const uint16_t *__restrict__ codes, u4_t *__restrict__ packed,
                                                   int64_t N, int64_t K, int64_t pieces)
{
    const int64_t n_steps = K >> 8, kc = K >> 3;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < pieces; i += (int64_t)gridDim.x * 256) {
        const int64_t lane = i & 63, chunk = i >> 6;
        const int64_t step = chunk % n_steps, tile = chunk / n_steps;
        const int64_t n = tile * 16 + (lane & 15);
        u4_t v = u4_t{0u, 0u, 0u, 0u};
        if (n < N) v = *reinterpret_cast<const u4_t *>(codes + n * kc + step * 32 + (lane >> 4) * 8);
        packed[i] = v;
    }
}

// ------------------------------------------------------------------ plain read of a code matrix
// What the memory system gives a kernel that only reads: the batch-1 kernels' launch shape (one
// workgroup of 16 waves per compute unit over contiguous ranges of 16-row tiles, a wave's load 16
// rows x 64 bytes, the waves of a workgroup dealing out the 256-wide k steps) with two loads in flight
// per wave and an exclusive or in place of the decode.  The yardstick the benchmark prints beside the
// batch-1 kernels; `sink` is written only if the bytes happen to cancel (never for random codes),
// which keeps the loads alive.
__global__ __launch_bounds__(1024) void read_probe_kernel(const uint16_t *__restrict__ codes, uint32_t *__restrict__ sink,
                                                          int N, int K, int tiles_q, int tiles_r)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c16 = lane & 15, q = lane >> 4;
    const int n_steps = K >> 8, row_bytes = K >> 2;
    const int t0 = (int)blockIdx.x * tiles_q + ((int)blockIdx.x < tiles_r ? (int)blockIdx.x : tiles_r);
    const int t1 = t0 + tiles_q + ((int)blockIdx.x < tiles_r ? 1 : 0);
    const __amdgpu_buffer_rsrc_t crsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(codes), 0, (int)((int64_t)N * row_bytes), 0x00020000);
    const int voff = c16 * row_bytes + q * 16;
    u4_t acc = u4_t{0u, 0u, 0u, 0u};
    for (int tile = t0; tile < t1; tile++)
        for (int step = wave; step < n_steps; step += 32) {
            const u4_t a = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff, tile * 16 * row_bytes + step * 64, 0);
            const u4_t b = __builtin_amdgcn_raw_buffer_load_b128(crsrc, voff, step + 16 < n_steps ? tile * 16 * row_bytes + (step + 16) * 64 : (int)0x80000000, 0);
            acc ^= a ^ b;
        }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9E3779B9u && N < 0) sink[0] = acc[0];
}
