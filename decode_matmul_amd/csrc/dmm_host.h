// The library scratch memory and the host side: launch plumbing, per-device set-up, argument
// checks, dispatch and the operator on host memory.
// Part of libdmm: included by dmm.hip inside namespace dmm, in this order; not a
// translation unit of its own.

// ------------------------------------------------------------------ scratch memory of the library
// The one buffer the library owns: split-K partial sums for dmm_decode_matmul_noalloc_f16, whose
// callers cannot allocate.  In host code the array's name is a stand-in, not a device address;
// dmm_init asks the runtime for the address once per device and the launches pass that.
constexpr int64_t kScratchBytes = 16ll << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// ------------------------------------------------------------------ host side
thread_local hipEvent_t tls_start = nullptr;
thread_local hipEvent_t tls_stop = nullptr;

template <typename T>
struct same_type { typedef T type; };

// Enqueue one kernel; the status is what the launch call itself returns (no look at the
// thread's last-error state, which may hold somebody else's stale error).  kFirst / kLast:
// whether this launch opens / closes the span the timing events bracket (an operator call
// that takes two kernels records start before the first and stop after the second).
template <bool kFirst = true, bool kLast = true, typename... KArgs>
int launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t shmem, hipStream_t stream,
           typename same_type<KArgs>::type... args)
{
    void *argv[] = {(void *)&args...};
    if (tls_start && tls_stop)
        return (int)hipExtLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, argv, shmem, stream,
                                       kFirst ? tls_start : nullptr, kLast ? tls_stop : nullptr, 0);
    return (int)hipLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, argv, shmem, stream);
}

inline bool aligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// ---- per-device state, set up by dmm_init --------------------------------------------------
constexpr int kMaxDevices = 64;
constexpr int kLdsMax = 160 * 1024;

struct DeviceState {
    std::atomic<int> ready{0};
    int cus = 256;
    void *scratch = nullptr;   // this device's copy of `scratch`
};
DeviceState g_dev[kMaxDevices];
std::mutex g_init_mutex;

// Every kernel that needs more dynamic LDS than the default limit, or whose table addressing
// assumes that its dynamic LDS starts at LDS address 0 (true exactly when the kernel has no
// static LDS, which dmm_init verifies from the function's attributes).
struct KernelInfo {
    const void *fn;
    int dynamic_lds;   // bytes to allow; 0 = default limit is enough
    bool lds_base0;
};

template <typename... KArgs>
KernelInfo kinfo(void (*k)(KArgs...), int lds, bool base0) { return KernelInfo{reinterpret_cast<const void *>(k), lds, base0}; }

const std::vector<KernelInfo> &kernel_table()
{
    static const std::vector<KernelInfo> t = {
#define DMM_BOTH_LAYOUTS(X) X(false), X(true)
#define DMM_K_STREAM(P) kinfo(gemv_stream_kernel<1, 16, 2, P, 4>, kLdsMax, true), kinfo(gemv_stream_kernel<1, 16, 2, P, 1>, kLdsMax, true)
        DMM_BOTH_LAYOUTS(DMM_K_STREAM),
#define DMM_K_Q8(P) kinfo(gemv_q8_kernel<1, 16, 2, P>, kLdsMax, true), kinfo(gemv_q8_kernel<1, 16, 3, P>, kLdsMax, true), kinfo(gemv_q8c_kernel<3, 1, P>, kLdsMax, true)
        DMM_BOTH_LAYOUTS(DMM_K_Q8),
#define DMM_K_Q8D(P)                                                                                             \
    kinfo(gemv_q8d_kernel<1, 2, 2, P>, kLdsMax, true), kinfo(gemv_q8d_kernel<2, 1, 2, P>, kLdsMax, true),         \
        kinfo(gemv_q8d_kernel<3, 1, 3, P>, kLdsMax, true), kinfo(gemv_q8d_kernel<4, 1, 2, P>, kLdsMax, true),     \
        kinfo(gemv_q8d_kernel<6, 1, 3, P>, kLdsMax, true), kinfo(gemv_q8d_kernel<8, 1, 2, P>, kLdsMax, true)
        DMM_BOTH_LAYOUTS(DMM_K_Q8D),
#define DMM_K_F16D_XI(P, XI)                                                                                      \
    kinfo(gemv_f16d_kernel<2, 1, 2, P, XI>, kLdsMax, true), kinfo(gemv_f16d_kernel<3, 1, 3, P, XI>, kLdsMax, true),     \
        kinfo(gemv_f16d_kernel<4, 1, 2, P, XI>, kLdsMax, true), kinfo(gemv_f16d_kernel<6, 1, 3, P, XI>, kLdsMax, true), \
        kinfo(gemv_f16d_kernel<8, 1, 2, P, XI>, kLdsMax, true)
#define DMM_K_F16D_W8(P)                                                                                         \
    kinfo(gemv_f16d_kernel<2, 1, 2, P, 8, 8>, kLdsMax, true), kinfo(gemv_f16d_kernel<3, 1, 3, P, 8, 8>, kLdsMax, true),   \
        kinfo(gemv_f16d_kernel<4, 1, 2, P, 8, 8>, kLdsMax, true), kinfo(gemv_f16d_kernel<6, 1, 3, P, 8, 8>, kLdsMax, true), \
        kinfo(gemv_f16d_kernel<8, 1, 2, P, 8, 8>, kLdsMax, true)
#define DMM_K_F16D_W8G2(P)                                                                                       \
    kinfo(gemv_f16d_kernel<2, 1, 2, P, 8, 8, 2>, kLdsMax, true), kinfo(gemv_f16d_kernel<3, 1, 3, P, 8, 8, 2>, kLdsMax, true),   \
        kinfo(gemv_f16d_kernel<4, 1, 2, P, 8, 8, 2>, kLdsMax, true), kinfo(gemv_f16d_kernel<6, 1, 3, P, 8, 8, 2>, kLdsMax, true), \
        kinfo(gemv_f16d_kernel<8, 1, 2, P, 8, 8, 2>, kLdsMax, true)
#define DMM_K_F16D(P) DMM_K_F16D_XI(P, 2), DMM_K_F16D_XI(P, 4), DMM_K_F16D_W8(P), DMM_K_F16D_W8G2(P)
        DMM_BOTH_LAYOUTS(DMM_K_F16D),
#define DMM_K_REGX_XI(P, XI)                                                                                      \
    kinfo(gemv_regx_kernel<1, 8, 2, P, XI>, kLdsMax, true), kinfo(gemv_regx_kernel<2, 8, 2, P, XI>, kLdsMax, true),     \
        kinfo(gemv_regx_kernel<3, 8, 2, P, XI>, kLdsMax, true), kinfo(gemv_regx_kernel<4, 8, 2, P, XI>, kLdsMax, true)
#define DMM_K_REGX(P) DMM_K_REGX_XI(P, 2), DMM_K_REGX_XI(P, 4), DMM_K_REGX_XI(P, 8)
        DMM_BOTH_LAYOUTS(DMM_K_REGX),
#define DMM_K_GREG(P)                                                                                        \
    kinfo(gemm_reg_kernel<1, false, P>, gr_smem_bytes(1), true), kinfo(gemm_reg_kernel<2, false, P>, gr_smem_bytes(2), true), \
        kinfo(gemm_reg_kernel<4, false, P>, gr_smem_bytes(4), true), kinfo(gemm_reg_kernel<1, true, P>, gr_smem_bytes(1), true), \
        kinfo(gemm_reg_kernel<2, true, P>, gr_smem_bytes(2), true), kinfo(gemm_reg_kernel<4, true, P>, gr_smem_bytes(4), true)
        DMM_BOTH_LAYOUTS(DMM_K_GREG),
        kinfo(gemm_kernel<4, 2, 2, 2>, (int)sizeof(GemmCfg<4, 2, 2, 2>::Shared), false),
#define DMM_K_I8X_S(T, S)                                                                                    \
    kinfo(int8x_kernel<1, 8, 2, T, S>, kLdsMax, true), kinfo(int8x_kernel<2, 8, 2, T, S>, kLdsMax, true),              \
        kinfo(int8x_kernel<3, 8, 2, T, S>, kLdsMax, true), kinfo(int8x_kernel<4, 8, 2, T, S>, kLdsMax, true)
#define DMM_K_I8D(T)                                                                                         \
    kinfo(int8d_kernel<2, 1, 2, T>, kLdsMax, true), kinfo(int8d_kernel<3, 1, 3, T>, kLdsMax, true),                \
        kinfo(int8d_kernel<4, 1, 2, T>, kLdsMax, true), kinfo(int8d_kernel<6, 1, 3, T>, kLdsMax, true),            \
        kinfo(int8d_kernel<8, 1, 2, T>, kLdsMax, true)
#define DMM_K_I8D8(T)                                                                                        \
    kinfo(int8d_kernel<2, 1, 2, T, 8>, kLdsMax, true), kinfo(int8d_kernel<3, 1, 3, T, 8>, kLdsMax, true),          \
        kinfo(int8d_kernel<4, 1, 2, T, 8>, kLdsMax, true), kinfo(int8d_kernel<6, 1, 3, T, 8>, kLdsMax, true),      \
        kinfo(int8d_kernel<8, 1, 2, T, 8>, kLdsMax, true)
#define DMM_K_I8D8G2(T)                                                                                      \
    kinfo(int8d_kernel<2, 1, 2, T, 8, 2>, kLdsMax, true), kinfo(int8d_kernel<3, 1, 3, T, 8, 2>, kLdsMax, true),    \
        kinfo(int8d_kernel<4, 1, 2, T, 8, 2>, kLdsMax, true), kinfo(int8d_kernel<6, 1, 3, T, 8, 2>, kLdsMax, true), \
        kinfo(int8d_kernel<8, 1, 2, T, 8, 2>, kLdsMax, true)
#define DMM_K_I8X(T) DMM_K_I8X_S(T, false), DMM_K_I8X_S(T, true), DMM_K_I8D(T), DMM_K_I8D8(T), DMM_K_I8D8G2(T), kinfo(int8g_kernel<T>, kI8gSmem, true)
        DMM_BOTH_LAYOUTS(DMM_K_I8X),
#undef DMM_K_I8X
#undef DMM_K_I8D
#undef DMM_K_I8D8
#undef DMM_K_I8D8G2
#undef DMM_K_I8X_S
#undef DMM_K_GREG
#undef DMM_K_REGX
#undef DMM_K_REGX_XI
#undef DMM_K_F16D
#undef DMM_K_F16D_W8
#undef DMM_K_F16D_W8G2
#undef DMM_K_F16D_XI
#undef DMM_K_Q8D
#undef DMM_K_Q8
#undef DMM_K_STREAM
#undef DMM_BOTH_LAYOUTS
    };
    return t;
}

// One-time set-up of a device (the current one must be `dev`): compute-unit count, dynamic-LDS
// limits, the check that the table kernels have no static LDS, and the address of `scratch`.
int init_current_device(int dev)
{
    DeviceState &ds = g_dev[dev];
    if (ds.ready.load(std::memory_order_acquire)) return DMM_OK;
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (ds.ready.load(std::memory_order_acquire)) return DMM_OK;
    int v = 0;
    hipError_t e = hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return (int)e;
    ds.cus = v > 0 ? v : 256;
    for (const KernelInfo &k : kernel_table()) {
        if (k.lds_base0) {
            hipFuncAttributes attr;
            e = hipFuncGetAttributes(&attr, k.fn);
            if (e != hipSuccess) return (int)e;
            if (attr.sharedSizeBytes != 0) return DMM_ERR_INTERNAL;
        }
        if (k.dynamic_lds > 0) {
            e = hipFuncSetAttribute(k.fn, hipFuncAttributeMaxDynamicSharedMemorySize, k.dynamic_lds);
            if (e != hipSuccess) return (int)e;
        }
    }
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    ds.scratch = p;
    ds.ready.store(1, std::memory_order_release);
    return DMM_OK;
}

// Called by every entry point that launches, after its argument checks.  A first call on a
// device does the set-up unless the stream is being captured into a graph, where host-side
// set-up has no business: such a caller runs dmm_init beforehand.
int ensure_ready(hipStream_t stream, const DeviceState **out = nullptr)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return DMM_ERR_TOO_LARGE;
    if (!g_dev[dev].ready.load(std::memory_order_acquire)) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (stream && hipStreamIsCapturing(stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
            return DMM_ERR_NOT_INITIALIZED;
        if (int st = init_current_device(dev)) return st;
    }
    if (out) *out = &g_dev[dev];
    return DMM_OK;
}

// compute units of the current device (after ensure_ready)
int cu_count()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    return g_dev[dev].cus;
}

int check_common(const void *x, const void *codes, const void *grid, const void *y, int64_t M,
                 int64_t N, int64_t K)
{
    if (M < 0 || N < 0 || K < 0 || (K & 7)) return DMM_ERR_BAD_SHAPE;
    if (M == 0 || N == 0) return DMM_OK;   // nothing to write; pointers may be NULL
    if (!y || !grid) return DMM_ERR_NULL_POINTER;
    if (K > 0 && (!x || !codes)) return DMM_ERR_NULL_POINTER;
    if (!aligned(x, 2) || !aligned(codes, 2) || !aligned(grid, 2) || !aligned(y, 2)) return DMM_ERR_MISALIGNED;
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return DMM_ERR_TOO_LARGE;
    return DMM_OK;
}

// what the matrix-vector kernels can take at all: any number of rows of x goes through the small-batch
// kernel 16 at a time (the operator sends more than 32 there only when that beats the matrix-matrix kernel)
bool gemv_rows_ok(const void *x, const void *codes, const void *grid, const void *y, int64_t M, int64_t N,
                  int64_t K)
{
    return M >= 1 && M <= 4096 && M * K < (1LL << 30) && K >= 256 && (K & 255) == 0 && K <= (1 << 23) &&
           N * (K >> 2) < (1LL << 31) && (N & 3) == 0 && aligned(x, 16) && aligned(codes, 16) && aligned(grid, 16) &&
           aligned(y, 8);
}

// the domain of the explicit matrix-vector entry points
bool gemv_ok(const void *x, const void *codes, const void *grid, const void *y, int64_t M, int64_t N,
             int64_t K)
{
    return gemv_rows_ok(x, codes, grid, y, M, N, K) && M <= 32;
}

bool gemm_ok(const void *x, const void *codes, const void *grid, const void *, int64_t M, int64_t N,
             int64_t K)
{
    return M >= 1 && N >= 1 && K >= 64 && (K & 63) == 0 && aligned(x, 16) && aligned(codes, 16) &&
           aligned(grid, 16) && M <= 65535LL * 128;
}

template <int R, int W, int D, bool kPacked = false>
int launch_gemv_stream(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                       int64_t N, int64_t K, hipStream_t stream)
{
    const size_t shmem = (size_t)kSTablesBytes + stream_red_bytes(R, W, (int)M) + (size_t)stream_x_bytes(M, K);
    const int64_t n_tiles = (N + 15) / 16;
    const int64_t wgs = n_tiles < cu_count() ? n_tiles : cu_count();
    if (M <= 4)   // four pieces of x per LDS read
        return launch(gemv_stream_kernel<R, W, D, kPacked, 4>, dim3((unsigned)wgs), dim3(64 * W), shmem, stream,
                      (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)M, (int)N,
                      (int)K, (int)(n_tiles / wgs), (int)(n_tiles % wgs));
    return launch(gemv_stream_kernel<R, W, D, kPacked, 1>, dim3((unsigned)wgs), dim3(64 * W), shmem, stream,
                  (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)M, (int)N, (int)K,
                  (int)(n_tiles / wgs), (int)(n_tiles % wgs));
}

// tables, partial sums and x fit in the 160 KB of LDS, and every byte offset of the code
// matrix fits the 31 bits the buffer addressing is used with
template <int R, int W>
bool gemv_q8_ok(int64_t M, int64_t N, int64_t K)
{
    return M <= 4 && (int64_t)kSTablesBytes + q8_red_bytes(R, W, (int)M) + q8_x_bytes(M, K) <= kLdsMax &&
           N * (K >> 2) < (1LL << 31);
}

template <int R, int W, int D, bool kPacked = false>
int launch_gemv_q8(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                   int64_t N, int64_t K, hipStream_t stream)
{
    // the 8-bit layout is the larger one, so the 16-bit kernel it may hand over to fits as well
    const size_t shmem = (size_t)kSTablesBytes + q8_red_bytes(R, W, (int)M) + (size_t)q8_x_bytes(M, K);
    const int64_t n_tiles = (N + 15) / 16;
    const int64_t wgs = n_tiles < cu_count() ? n_tiles : cu_count();
    return launch(gemv_q8_kernel<R, W, D, kPacked>, dim3((unsigned)wgs), dim3(64 * W), shmem, stream,
                  (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)M, (int)N, (int)K,
                  (int)(n_tiles / wgs), (int)(n_tiles % wgs));
}

// the chunked 8-bit kernel: one row of x of any length the 16-bit kernel could take over (its x in LDS)
bool gemv_q8c_ok(int64_t M, int64_t N, int64_t K)
{
    return M == 1 && (int64_t)kSTablesBytes + stream_red_bytes(1, 16, 1) + stream_x_bytes(1, K) <= kLdsMax &&
           N * (K >> 2) < (1LL << 31);
}

// groups of up to three tiles, one code load per tile in flight per wave (four tiles per group spill
// registers; two chunks in flight per wave were no faster)
template <bool kPacked>
int launch_gemv_q8c(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t N, int64_t K,
                    hipStream_t stream)
{
    constexpr int T = 3;
    size_t shmem = (size_t)kSTablesBytes + stream_red_bytes(1, 16, 1) + (size_t)stream_x_bytes(1, K);   // the 16-bit hand-over
    if (shmem < (size_t)qc_lds_bytes(T)) shmem = qc_lds_bytes(T);
    const int64_t n_tiles = (N + 15) / 16;
    const int64_t wgs = n_tiles < cu_count() ? n_tiles : cu_count();
    return launch(gemv_q8c_kernel<T, 1, kPacked>, dim3((unsigned)wgs), dim3(1024), shmem, stream, (const uint16_t *)x,
                  (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)N, (int)K, (int)(n_tiles / wgs),
                  (int)(n_tiles % wgs));
}

// the resident-accumulator form: up to 8 tiles per workgroup, instantiated for 1, 2, 3, 4, 6 and 8.  The ring
// is two loads deep wherever two divides the tiles (measured as graph launches, two against four deep, us:
// 8192 -> 28672 13.72 / 13.90, 28672 -> 8192 13.60 / 14.21, 8192 -> 8192 6.20 / 6.58, 8192 -> 16384 8.49 / 8.84,
// 4096 -> 16384 5.88 / 6.23; eight deep 15.90 at 8192 -> 28672), three for three and six tiles (six tiles, two /
// three / six deep: 8192 -> 24576 12.55 / 12.16 / 14.23, 4096 -> 22016 8.06 / 7.60 / 8.64)
inline bool gemv_q8d_ok(int64_t N) { return (N + 15) / 16 <= 8 * (int64_t)cu_count(); }

template <int NT, int U, int D, bool kPacked>
int launch_gemv_q8d_inst(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t N, int64_t K,
                         hipStream_t stream)
{
    size_t shmem = (size_t)kSTablesBytes + stream_red_bytes(1, 16, 1) + (size_t)stream_x_bytes(1, K);   // the 16-bit hand-over
    if (shmem < (size_t)qd_lds_bytes()) shmem = qd_lds_bytes();
    const int64_t n_tiles = (N + 15) / 16;
    const int64_t wgs = n_tiles < cu_count() ? n_tiles : cu_count();
    return launch(gemv_q8d_kernel<NT, U, D, kPacked>, dim3((unsigned)wgs), dim3(1024), shmem, stream, (const uint16_t *)x,
                  (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)N, (int)K, (int)(n_tiles / wgs),
                  (int)(n_tiles % wgs));
}

template <bool kPacked>
int launch_gemv_q8d(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t N, int64_t K,
                    hipStream_t stream)
{
    const int64_t n_tiles = (N + 15) / 16, cus = cu_count();
    const int64_t share = n_tiles <= cus ? 1 : (n_tiles + cus - 1) / cus;   // most tiles a workgroup gets
    switch (share) {
        case 1: return launch_gemv_q8d_inst<1, 2, 2, kPacked>(x, codes, grid, scale, y, N, K, stream);
        case 2: return launch_gemv_q8d_inst<2, 1, 2, kPacked>(x, codes, grid, scale, y, N, K, stream);
        case 3: return launch_gemv_q8d_inst<3, 1, 3, kPacked>(x, codes, grid, scale, y, N, K, stream);
        case 4: return launch_gemv_q8d_inst<4, 1, 2, kPacked>(x, codes, grid, scale, y, N, K, stream);
        case 5:
        case 6: return launch_gemv_q8d_inst<6, 1, 3, kPacked>(x, codes, grid, scale, y, N, K, stream);
        default: return launch_gemv_q8d_inst<8, 1, 2, kPacked>(x, codes, grid, scale, y, N, K, stream);
    }
}

// the same loop order on 16-bit operands, for up to 32 rows of x of any length (a wave fetches the x of its
// k steps itself; from nine rows on eight waves instead of sixteen, from seventeen on two MFMAs per code): up to
// 8 tiles per workgroup
inline bool gemv_f16d_ok(int64_t M, int64_t N, int64_t K)
{
    return M >= 1 && M <= 32 && (N + 15) / 16 <= 8 * (int64_t)cu_count() && N * (K >> 2) < (1LL << 31) && M * K * 2 < (1LL << 31);
}

template <int NT, int U, int D, bool kPacked>
int launch_gemv_f16d_inst(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M, int64_t N,
                          int64_t K, hipStream_t stream)
{
    const int64_t n_tiles = (N + 15) / 16;
    const int64_t wgs = n_tiles < cu_count() ? n_tiles : cu_count();
    if (M <= 4)
        return launch(gemv_f16d_kernel<NT, U, D, kPacked, 2>, dim3((unsigned)wgs), dim3(1024), (size_t)fd_lds_bytes(2), stream,
                      (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)M, (int)N, (int)K,
                      (int)(n_tiles / wgs), (int)(n_tiles % wgs));
    if (M > 16)
        return launch(gemv_f16d_kernel<NT, U, D, kPacked, 8, 8, 2>, dim3((unsigned)wgs), dim3(512), (size_t)fd_lds_bytes(8, 8), stream,
                      (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)M, (int)N, (int)K,
                      (int)(n_tiles / wgs), (int)(n_tiles % wgs));
    if (M > 8)
        return launch(gemv_f16d_kernel<NT, U, D, kPacked, 8, 8>, dim3((unsigned)wgs), dim3(512), (size_t)fd_lds_bytes(8, 8), stream,
                      (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)M, (int)N, (int)K,
                      (int)(n_tiles / wgs), (int)(n_tiles % wgs));
    return launch(gemv_f16d_kernel<NT, U, D, kPacked, 4>, dim3((unsigned)wgs), dim3(1024), (size_t)fd_lds_bytes(4), stream,
                  (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)M, (int)N, (int)K,
                  (int)(n_tiles / wgs), (int)(n_tiles % wgs));
}

template <bool kPacked>
int launch_gemv_f16d(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M, int64_t N,
                     int64_t K, hipStream_t stream)
{
    const int64_t n_tiles = (N + 15) / 16, cus = cu_count();
    const int64_t share = n_tiles <= cus ? 1 : (n_tiles + cus - 1) / cus;   // most tiles a workgroup gets
    switch (share) {
        case 1:
        case 2: return launch_gemv_f16d_inst<2, 1, 2, kPacked>(x, codes, grid, scale, y, M, N, K, stream);
        case 3: return launch_gemv_f16d_inst<3, 1, 3, kPacked>(x, codes, grid, scale, y, M, N, K, stream);
        case 4: return launch_gemv_f16d_inst<4, 1, 2, kPacked>(x, codes, grid, scale, y, M, N, K, stream);
        case 5:
        case 6: return launch_gemv_f16d_inst<6, 1, 3, kPacked>(x, codes, grid, scale, y, M, N, K, stream);
        default: return launch_gemv_f16d_inst<8, 1, 2, kPacked>(x, codes, grid, scale, y, M, N, K, stream);
    }
}

template <int R, int W>
bool gemv_stream_ok(int64_t M, int64_t N, int64_t K)
{
    return M <= 16 && (int64_t)kSTablesBytes + stream_red_bytes(R, W, (int)M) + stream_x_bytes(M, K) <= kLdsMax &&
           N * (K >> 2) < (1LL << 31);
}

// the x of a step goes through one 8 KB piece of LDS per wave, which also carries the partial sums
template <int R, int W, int D, bool kPacked, int XI>
int launch_gemv_regx(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                     int64_t N, int64_t K, hipStream_t stream)
{
    const size_t shmem = (size_t)kSTablesBytes + W * kRegxPiece;
    const int64_t n_tiles = (N + 15) / 16;
    const int64_t wgs = n_tiles < cu_count() ? n_tiles : cu_count();
    return launch(gemv_regx_kernel<R, W, D, kPacked, XI>, dim3((unsigned)wgs), dim3(64 * W), shmem, stream,
                  (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)M, (int)N, (int)K,
                  (int)(n_tiles / wgs), (int)(n_tiles % wgs));
}

// dmm_set_choice: what a benchmark that checks the operator's choices forces instead (-1: nothing).
// [0]: more than 16 rows of x (0 passes of the small-batch kernel, 1 matrix-matrix kernel, 2 split K);
// [1]: the integer operator on more than 16 rows (1 passes of the matrix-vector kernel, 2 matrix-matrix);
// [2]: up to eight rows of x (0 never the 16-bit kernel with resident sums, 1 wherever it can run).
// A forced kernel that cannot take the call leaves the choice to the library.
std::atomic<int> g_choice[4] = {{-1}, {-1}, {-1}, {-1}};

// Whether the operator may pick the 8-bit kernel: dmm_set_gemv_8bit, or DMM_GEMV_8BIT=0 in the
// environment (read once, at the first call that needs it) for hosts that cannot call it.
std::atomic<int> g_gemv_q8{-1};

inline bool gemv_q8_enabled()
{
    int on = g_gemv_q8.load(std::memory_order_relaxed);
    if (on < 0) {
        const char *e = getenv("DMM_GEMV_8BIT");
        on = (e && e[0] == '0') ? 0 : 1;
        int expected = -1;
        if (!g_gemv_q8.compare_exchange_strong(expected, on)) on = expected;   // a setter came first
    }
    return on == 1;
}

// The 8-bit kernels.  One row of x: the chunked kernel.  Two to four rows: one row tile at a time, the
// code stream three loads deep per wave when a workgroup has more than two row tiles to walk
// through, two deep for shorter launches (where a larger first burst only delays the first tile).
template <bool kPacked>
int run_gemv_q8(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                int64_t N, int64_t K, hipStream_t stream)
{
    if (M == 1 && gemv_q8d_ok(N)) return launch_gemv_q8d<kPacked>(x, codes, grid, scale, y, N, K, stream);
    if (M == 1) return launch_gemv_q8c<kPacked>(x, codes, grid, scale, y, N, K, stream);
    const int64_t n_tiles = (N + 15) / 16;
    if (n_tiles > 2 * cu_count()) return launch_gemv_q8<1, 16, 3, kPacked>(x, codes, grid, scale, y, M, N, K, stream);
    return launch_gemv_q8<1, 16, 2, kPacked>(x, codes, grid, scale, y, M, N, K, stream);
}

// whether an 8-bit kernel can take the shape at all (grid and x permitting, which the kernel finds out)
bool gemv_8bit_ok(int64_t M, int64_t N, int64_t K) { return M == 1 ? gemv_q8c_ok(M, N, K) : gemv_q8_ok<1, 16>(M, N, K); }

// The choice among the matrix-vector kernels.  The 8-bit kernels where they apply and pay.  One row of x:
// from more than one row tile per workgroup on, and with one tile on a long x (measured as launches of one
// HIP graph on rotating code buffers, 8-bit against 16-bit kernel, us per launch: 8192 -> 28672 13.7 / 16.6,
// 28672 -> 8192 14.0 / 16.2, 8192 -> 10240 6.9 / 8.7, 8192 -> 8192 6.2 / 7.2, 8192 -> 4352 5.9 / 6.8, 4096 -> 8192
// 4.7 / 5.3, 4096 -> 4352 4.4 / 5.2, 11008 -> 8192 7.6 / 8.2, 11008 -> 4352 7.0 / 7.7, 28672 -> 4096 10.4 / 11.0;
// but with one tile per workgroup 4096 -> 4096 4.22 / 4.21, 8192 -> 4096 4.97 / 4.89, 11008 -> 4096 5.98 / 5.48).
// Two to four rows only beyond eight tiles per workgroup (below, the 16-bit kernel with resident sums is faster).
// A grid that does not fit fp8 costs them a second table
// build, and the 16-bit kernel's y is the correctly rounded one.  Otherwise the 16-bit streaming kernel,
// one tile at a time; the small-batch kernel when x does not fit the LDS.
enum GemvKind { kGemvQ8, kGemvStream, kGemvF16d, kGemvRegx };

// 17 .. 32 rows of x: is this a shape for the 16-bit kernel with resident sums (two to eight tiles per workgroup,
// K of 2048 or more)?
inline bool rows32_resident(int64_t N, int64_t K, int64_t cus)
{
    const int64_t n_tiles = (N + 15) / 16;
    return n_tiles > cus && n_tiles <= 8 * cus && K >= 2048;
}

GemvKind pick_gemv(int64_t M, int64_t N, int64_t K)
{
    const int64_t n_tiles = (N + 15) / 16, cus = cu_count();
    const int64_t share = n_tiles <= cus ? 1 : (n_tiles + cus - 1) / cus;   // most tiles a workgroup gets
    if (M == 1 && (n_tiles > cus || K >= 16384) && gemv_q8_enabled() && gemv_8bit_ok(M, N, K)) return kGemvQ8;
    // Two to sixteen rows on up to eight tiles per workgroup, and one row on two to eight: the 16-bit kernel that keeps
    // every tile's sums in registers and has each wave fetch the x of its own k steps.  It beats what served
    // before it at every such shape measured (graph launches, us, this kernel / before: M = 2 4096 -> 11008
    // 6.2 / 7.2, 8192 -> 8192 6.45 / 7.40, 8192 -> 10240 8.0 / 9.6, 8192 -> 28672 17.3 / 18.6, 28672 -> 8192 16.6 / 20.3,
    // 2048 -> 16384 5.25 / 7.02, 256 -> 32768 6.45 / 13.66; M = 4 8192 -> 28672 16.9 / 22.7, 28672 -> 8192 17.7 / 20.9;
    // M = 8 8192 -> 10240 9.6 / 10.7, 8192 -> 28672 18.4 / 24.2, 4096 -> 22016 10.6 / 12.8; one row with the 8-bit
    // kernels off: 8192 -> 28672 16.6 / 18.0, 4096 -> 22016 9.3 / 11.3), the 8-bit kernel for two to four rows
    // included (M = 2 4096 -> 22016 9.5 / 10.4, 4096 -> 32000 10.1 / 11.75; M = 4 3072 -> 32768 9.7 / 11.8).  With
    // one tile per workgroup it is behind for one row (11008 -> 4096 6.03 / 5.63) and 1 - 7 % ahead for two to eight
    // (M = 2 4096 -> 4096 4.01 / 4.22, M = 4 11008 -> 4096 6.29 / 6.63, M = 8 7.95 / 8.34); nine to sixteen rows run it on
    // eight waves with pieces of sixteen rows, ahead at every share (M = 16 4096 -> 4096 6.68 / 7.02, 4096 -> 11008
    // 8.8 / 10.1, 8192 -> 28672 23.0 / 27.6).
    const int force = g_choice[2].load(std::memory_order_relaxed);
    // Seventeen to 32 rows: the same kernel with two MFMAs per code where a workgroup has two to eight tiles and
    // K is not short, else two passes of the small-batch kernel (graph launches, us, this kernel / passes, M = 32:
    // 4096 -> 11008 13.1 / 14.4, 4096 -> 22016 18.0 / 23.6, 8192 -> 10240 18.4 / 21.6, 8192 -> 28672 30.0 / 45.0,
    // 28672 -> 8192 41.4 / 48.1; but 4096 -> 4096 10.7 / 9.4, 1024 -> 16384 10.3 / 9.1, and level at 8192 -> 4096 and
    // 11008 -> 4096)
    if (M > 16) {
        if (force == 1 && gemv_f16d_ok(M, N, K)) return kGemvF16d;
        return force != 0 && rows32_resident(N, K, cus) && gemv_f16d_ok(M, N, K) ? kGemvF16d : kGemvRegx;
    }
    if (force == 1 && gemv_f16d_ok(M, N, K)) return kGemvF16d;
    if (force != 0 && (share >= 2 || M >= 2) && gemv_f16d_ok(M, N, K)) return kGemvF16d;
    // Beyond eight tiles per workgroup: two to four rows on 8-bit operands where their x fits the LDS
    if (M >= 2 && n_tiles > 4 * cus && gemv_q8_enabled() && gemv_8bit_ok(M, N, K)) return kGemvQ8;
    // Otherwise the 16-bit streaming kernel, one tile at a time, or the small-batch kernel when x does not fit the
    // LDS - and for two to four rows on a launch of one tile per workgroup with a short x, and for four rows,
    // where its eight waves start sooner than the streaming kernel's sixteen with their x in the LDS (M = 2
    // 4096 -> 4096 4.77 / 4.47, 11008 -> 4096 6.27 / 6.51; M = 4 4096 -> 4096 5.13 / 4.47)
    const bool small_first = M == 4 || (M >= 2 && M <= 4 && n_tiles <= cus && K <= 4096);
    if (!small_first && gemv_stream_ok<1, 16>(M, N, K)) return kGemvStream;
    return kGemvRegx;
}

// Row tiles per block of the small-batch kernels (half precision and integer): the workgroup's whole share
// of tiles when that is one to four, else the size (<= 4) that needs the fewest blocks - the x slice of a
// k step is fetched once per row block and pass.
inline int small_batch_row_block(int64_t n_tiles, int64_t cus, int64_t *blocks = nullptr)
{
    const int64_t share = n_tiles <= cus ? 1 : (n_tiles + cus - 1) / cus;   // most tiles a workgroup gets
    int best = 1;
    for (int r = 2; r <= 4; r++)
        if ((share + r - 1) / r < (share + best - 1) / best) best = r;
    if (blocks) *blocks = (share + best - 1) / best;
    return best;
}

// XI: load instructions per slice of x, two rows each
template <bool kPacked, int XI>
int run_gemv_regx_r(int r, const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                    int64_t N, int64_t K, hipStream_t stream)
{
    switch (r) {
        case 1: return launch_gemv_regx<1, 8, 2, kPacked, XI>(x, codes, grid, scale, y, M, N, K, stream);
        case 2: return launch_gemv_regx<2, 8, 2, kPacked, XI>(x, codes, grid, scale, y, M, N, K, stream);
        case 3: return launch_gemv_regx<3, 8, 2, kPacked, XI>(x, codes, grid, scale, y, M, N, K, stream);
        default: return launch_gemv_regx<4, 8, 2, kPacked, XI>(x, codes, grid, scale, y, M, N, K, stream);
    }
}

// The small-batch kernel reads the x slice of a k step once per row block and pass, so the row
// block should be the workgroup's whole share of tiles when that is 1 .. 4 tiles, and otherwise
// the size that needs the fewest blocks.
template <bool kPacked>
int run_gemv_regx(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                  int64_t N, int64_t K, hipStream_t stream)
{
    const int best = small_batch_row_block((N + 15) / 16, cu_count());
    return M <= 4 ? run_gemv_regx_r<kPacked, 2>(best, x, codes, grid, scale, y, M, N, K, stream)
         : M <= 8 ? run_gemv_regx_r<kPacked, 4>(best, x, codes, grid, scale, y, M, N, K, stream)
                  : run_gemv_regx_r<kPacked, 8>(best, x, codes, grid, scale, y, M, N, K, stream);
}

template <bool kPacked>
int run_gemv(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
             int64_t N, int64_t K, hipStream_t stream)
{
    switch (pick_gemv(M, N, K)) {
        case kGemvQ8: return run_gemv_q8<kPacked>(x, codes, grid, scale, y, M, N, K, stream);
        case kGemvF16d: return launch_gemv_f16d<kPacked>(x, codes, grid, scale, y, M, N, K, stream);
        case kGemvStream: return launch_gemv_stream<1, 16, 2, kPacked>(x, codes, grid, scale, y, M, N, K, stream);
        default: return run_gemv_regx<kPacked>(x, codes, grid, scale, y, M, N, K, stream);
    }
}

template <int TM, bool kSplit, bool kPacked>
int launch_gemm_reg_tm(const void *x, const void *codes, const void *grid, float scale, void *y, float *part,
                       int64_t M, int64_t N, int64_t K, int splits, hipStream_t stream)
{
    dim3 g((unsigned)((M + 32 * TM - 1) / (32 * TM)), (unsigned)((N + kGrBN - 1) / kGrBN), (unsigned)splits);
    return launch<true, !kSplit>(gemm_reg_kernel<TM, kSplit, kPacked>, g, dim3(256), gr_smem_bytes(TM), stream,
                                 (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, part, (int)M,
                                 (int)N, (int)K, splits, aligned(y, 8) ? 1 : 0);
}

// rows of x per block: 32, 64 or 128
inline int gemm_reg_tm(int64_t M) { return M <= 32 ? 1 : M <= 64 ? 2 : 4; }

template <bool kPacked = false>
int launch_gemm_reg(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                    int64_t N, int64_t K, hipStream_t stream)
{
    switch (gemm_reg_tm(M)) {
        case 1: return launch_gemm_reg_tm<1, false, kPacked>(x, codes, grid, scale, y, nullptr, M, N, K, 1, stream);
        case 2: return launch_gemm_reg_tm<2, false, kPacked>(x, codes, grid, scale, y, nullptr, M, N, K, 1, stream);
        default: return launch_gemm_reg_tm<4, false, kPacked>(x, codes, grid, scale, y, nullptr, M, N, K, 1, stream);
    }
}

// How many ways to split K so that the blocks about fill the chip: as many as fit the CU count
// without starting a second round, each with at least 4 k tiles, and no more than the
// workspace holds partial sums for.  1 = no split.
int splitk_plan(int64_t M, int64_t N, int64_t K, int64_t workspace_bytes, int cus)
{
    const int tm = gemm_reg_tm(M);
    const int64_t tiles = ((M + 32 * tm - 1) / (32 * tm)) * ((N + kGrBN - 1) / kGrBN);
    int64_t splits = cus / tiles;
    const int64_t k_tiles = K / kGrBK;
    if (splits > k_tiles / 4) splits = k_tiles / 4;
    if (splits > 64) splits = 64;
    const int64_t per_split = M * N * 4;
    if (per_split > 0 && splits * per_split > workspace_bytes) splits = workspace_bytes / per_split;
    return splits < 2 ? 1 : (int)splits;
}

template <bool kPacked = false>
int launch_gemm_splitk(const void *x, const void *codes, const void *grid, float scale, void *y, void *workspace,
                       int splits, int64_t M, int64_t N, int64_t K, hipStream_t stream)
{
    float *part = reinterpret_cast<float *>(workspace);
    int st;
    switch (gemm_reg_tm(M)) {
        case 1: st = launch_gemm_reg_tm<1, true, kPacked>(x, codes, grid, scale, y, part, M, N, K, splits, stream); break;
        case 2: st = launch_gemm_reg_tm<2, true, kPacked>(x, codes, grid, scale, y, part, M, N, K, splits, stream); break;
        default: st = launch_gemm_reg_tm<4, true, kPacked>(x, codes, grid, scale, y, part, M, N, K, splits, stream); break;
    }
    if (st != 0) return st;
    const int64_t mn = M * N;
    const int64_t blocks = (mn + 1023) / 1024;
    return launch<false, true>(splitk_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const float *)part,
                               (uint16_t *)y, mn, splits, scale);
}

// the register-operand kernel addresses codes and x through 31-bit buffer offsets
bool gemm_reg_ok(int64_t M, int64_t N, int64_t K)
{
    return N * (K >> 2) < (1LL << 31) && M * K * 2 < (1LL << 31) && N <= 65535LL * kGrBN;
}

// Smallest M that takes the split-K path when a workspace is given (up to M = 16 the
// matrix-vector kernels are as fast or faster).
constexpr int kSplitKMinM = 17;

// What passes of the small-batch kernel cost, us: 2 for the launch, the code bytes once at 5.5 TB/s on 256
// compute units (the first pass reads them from HBM), and per 16 rows of x about 0.9, the code bytes at
// 3.8 TB/s (from the caches) and K / 6000 (every workgroup streams its rows of x whole).  Graph launches, us,
// M = 64 / 128 / 256: 4096 -> 4096 14.5 / 24.4 / 44.2, 4096 -> 11008 22.8 / 39.7 / 73.8, 11008 -> 4096 28.4 / 51.4 /
// 97.7, 8192 -> 8192 30.9 / 55.1 / 107.5.
inline double passes_cost_us(int64_t M, int64_t N, int64_t K, int cus)
{
    const double mb = 1e-6 * (double)N * (double)(K >> 2) * (256.0 / cus);
    return 2.0 + mb / 5.5 + (double)((M + 15) / 16) * (0.9 + mb / 3.8 + (double)K / 6000.0);
}

bool passes_beat_gemm(int64_t M, int64_t N, int64_t K, int cus);

// A workspace is there, and so the choice of splitting K.  17 .. 32 rows of x where the small-batch kernel
// serves: its two passes beat the split and its second launch while the busiest workgroup has no more than 68 KB of codes
// (graph launches, us, split / passes, M = 32: 4096 -> 11008 16.8 / 14.9, 8192 -> 8192 19.7 / 18.3, but 8192 ->
// 8448 18.9 / 22.0, 4096 -> 17408 19.1 / 22.3, 8192 -> 10240 22.4 / 22.0, 8192 -> 28672 31.7 / 42.0).  More rows:
// the split costs about 14 us + 0.085 per row + 0.3 per MB of codes, and the passes have to beat that by a
// twentieth, and the matrix-matrix kernel too (M = 48: 4096 -> 4096 18.0 / 11.9, 4096 -> 11008 20.0 / 18.6, 8192 -> 8192
// 23.6 / 24.3; M = 64: 20.6 / 14.5, 21.3 / 22.8, 23.5 / 30.9; M = 128: 26.5 / 24.4, 28.1 / 39.7, 33.7 / 55.1) -
// only where that was measured, up to 128 rows on 2 MB of codes or more.  Such a shape asks for no
// workspace and ignores one.
inline bool passes_beat_splitk(int64_t M, int64_t N, int64_t K, int cus)
{
    if (K < 256 || (K & 255) || (N & 3)) return false;
    if (M <= 32) {
        // the kernel with resident sums serves (one launch, every code decoded once): it wins up to K = 12288 or so
        // (graph launches, us, split / that kernel, M = 32: 4096 -> 22016 22.1 / 18.4, 8192 -> 10240 21.9 / 18.7,
        // 8192 -> 28672 34.6 / 30.9, but 16384 -> 8192 24.0 / 27.2, 28672 -> 8192 34.1 / 41.8)
        if (g_choice[2].load(std::memory_order_relaxed) != 0 && rows32_resident(N, K, cus)) return K <= 12288;
        const int64_t share = ((N + 15) / 16 + cus - 1) / cus;   // row tiles of the busiest workgroup
        return share * 4 * K <= (68 << 10);
    }
    if (M > 128 || N * (K >> 2) < (2 << 20)) return false;
    const double t_split = 14.0 + 0.085 * (double)M + 0.3e-6 * (double)N * (double)(K >> 2) * (256.0 / cus);
    return passes_cost_us(M, N, K, cus) * 1.05 < t_split && passes_beat_gemm(M, N, K, cus);
}

bool splitk_ok(const void *x, const void *codes, const void *grid, const void *y, int64_t M, int64_t N,
               int64_t K)
{
    return M >= kSplitKMinM && gemm_ok(x, codes, grid, y, M, N, K) && gemm_reg_ok(M, N, K) && aligned(y, 8);
}

// The register-operand kernel where its offsets fit, else the LDS-staged one (256 x 128, 8 waves)
int run_gemm(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
             int64_t N, int64_t K, hipStream_t stream)
{
    if (gemm_reg_ok(M, N, K)) return launch_gemm_reg(x, codes, grid, scale, y, M, N, K, stream);
    typedef GemmCfg<4, 2, 2, 2> C;
    dim3 g((unsigned)((N + C::kBN - 1) / C::kBN), (unsigned)((M + C::kBM - 1) / C::kBM));
    return launch(gemm_kernel<4, 2, 2, 2>, g, dim3(C::kThreads), sizeof(typename C::Shared), stream,
                  (const uint16_t *)x, (const uint16_t *)codes, grid, scale, (uint16_t *)y, (int)M, (int)N, (int)K,
                  aligned(y, 8) ? 1 : 0);
}

// y = 0 when K == 0 (empty sum), any M, N.
__global__ void zero_kernel(uint16_t *y, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        y[i] = 0;
}

int run_generic(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                int64_t N, int64_t K, hipStream_t stream)
{
    if (K == 0) {
        int64_t n = M * N;
        unsigned blocks = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
        return launch(zero_kernel, dim3(blocks), dim3(256), 0, stream, (uint16_t *)y, n);
    }
    int64_t blocks = (N + 3) / 4;
    if (blocks > 65535 * 16) blocks = 65535 * 16;
    return launch(generic_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint16_t *)x,
                  (const uint16_t *)codes, grid, scale, (uint16_t *)y, M, N, K);
}

template <int R, bool kTiled, bool kSlice>
int launch_int8x_s(const void *x, const void *codes, const void *cb, void *out, int64_t M, int64_t N, int64_t K,
                   hipStream_t stream)
{
    constexpr int W = 8, D = 2;
    const size_t shmem = (size_t)2 * kI8TableBytes + W * kI8xPiece;
    const int64_t n_tiles = (N + 15) / 16;
    const int64_t wgs = n_tiles < cu_count() ? n_tiles : cu_count();
    return launch(int8x_kernel<R, W, D, kTiled, kSlice>, dim3((unsigned)wgs), dim3(64 * W), shmem, stream,
                  (const int8_t *)x, (const uint16_t *)codes, (const int64_t *)cb, (int32_t *)out, (int)M, (int)N, (int)K,
                  (int)(n_tiles / wgs), (int)(n_tiles % wgs));
}

// More than 8 rows of x: the slice of a step goes through the LDS (graph launches, us, fragment loads /
// slice: M = 16 28672 -> 8192 20.5 / 17.1, 11008 -> 4096 9.3 / 7.5; M = 64 67.0 / 54.1, 25.4 / 16.9; but
// M = 1 13.9 / 17.0, 6.5 / 7.6, and level at M = 8).
template <int R, bool kTiled>
int launch_int8x(const void *x, const void *codes, const void *cb, void *out, int64_t M, int64_t N, int64_t K,
                 hipStream_t stream)
{
    return M > 8 ? launch_int8x_s<R, kTiled, true>(x, codes, cb, out, M, N, K, stream)
                 : launch_int8x_s<R, kTiled, false>(x, codes, cb, out, M, N, K, stream);
}

// Which kernel the integer operator takes for 16-byte aligned buffers.  More than 16 rows of x are
// passes of the matrix-vector kernel (16 rows each, the codes from the caches after the first) or one
// launch of the matrix-matrix kernel; the cheaper estimate wins.  A pass costs each wave its k steps
// (K / 256 over 8 waves, per row block) at 0.35 us + 0.27 us per row tile of the block; the
// matrix-matrix kernel K * 5.2 ns per round of one 256 x 128 tile per CU when few CUs have a tile,
// rising to K * 8.8 ns with all of them busy (the clock drops).  Graph launches, us, passes /
// matrix-matrix: 4096 x 4096 M = 256 28.5 / 30.3, M = 384 40.7 / 30.6; 11008 -> 4096 M = 256 60.1 / 63.5,
// M = 384 86.3 / 64.1; 8192 -> 28672 M = 32 32.6 / 49.2, M = 64 54.7 / 48.7; 28672 -> 8192 M = 128
// 111.5 / 148.7, M = 192 158.0 / 149.5.
enum Int8Kind { kInt8Scalar, kInt8Gemv, kInt8Gemm };
Int8Kind pick_int8(int64_t M, int64_t N, int64_t K, int cus)
{
    if (M < 1 || N < 1 || K < 256 || (K & 255) || (N & 3) || N * (K >> 2) >= (1LL << 31) || K > (1 << 17) ||
        M * K >= (1LL << 31))
        return kInt8Scalar;
    if (M > 16) {
        int64_t tiles = ((M + kI8gBM - 1) / kI8gBM) * ((N + kI8gBN - 1) / kI8gBN);
        double t_gemm = 5.0;
        for (; tiles > 0; tiles -= cus) {
            const double fill = tiles >= cus ? 1.0 : (double)tiles / (double)cus;
            t_gemm += (double)K * (0.0052 + 0.0036 * fill * fill);
        }
        int64_t blocks = 1;
        const int r = small_batch_row_block((N + 15) / 16, cus, &blocks);
        const double t_pass = (double)(blocks * (((K >> 8) + 7) / 8)) * (0.35 + 0.27 * r);
        const double t_gemv = 3.0 + (double)N * (double)(K >> 2) / (27344.0 * cus) /* 7 TB/s on 256 units */ + (double)((M + 15) / 16) * t_pass;
        if (t_gemm < 0.95 * t_gemv) return kInt8Gemm;   // the estimate of the passes runs high for long K
    }
    return kInt8Gemv;
}

template <bool kTiled>
int launch_int8g(const void *x, const void *codes, const void *cb, void *out, int64_t M, int64_t N, int64_t K,
                 hipStream_t stream)
{
    dim3 g((unsigned)((M + kI8gBM - 1) / kI8gBM), (unsigned)((N + kI8gBN - 1) / kI8gBN));
    return launch(int8g_kernel<kTiled>, g, dim3(512), kI8gSmem, stream, (const int8_t *)x, (const uint16_t *)codes,
                  (const int64_t *)cb, (int32_t *)out, (int)M, (int)N, (int)K);
}

// Up to 32 rows of x with two to eight row tiles per compute unit: the kernel with resident sums (graph
// launches, us, row-block kernel / this one: M = 1 4096 -> 11008 6.9 / 5.6, 8192 -> 8192 7.5 / 6.4, 8192 -> 28672
// 18.3 / 16.2, 28672 -> 8192 17.1 / 15.2; M = 8 7.1 / 6.0, 8.1 / 6.6, 19.2 / 18.3, 18.6 / 17.7; M = 16 7.7 / 6.7, 8.7 / 8.1,
// 20.4 / 20.0, 20.0 / 19.0; M = 32 10.4 / 9.3, 12.3 / 11.3, 30.4 / 24.6, 32.1 / 26.8)
inline bool int8d_ok(int64_t M, int64_t N, int cus)
{
    const int64_t n_tiles = (N + 15) / 16;
    return M >= 1 && M <= 32 && n_tiles > cus && n_tiles <= 8 * (int64_t)cus;
}

template <int NT, int U, int D, bool kTiled>
int launch_int8d_inst(const void *x, const void *codes, const void *cb, void *out, int64_t M, int64_t N, int64_t K,
                      hipStream_t stream)
{
    const size_t shmem = (size_t)2 * kI8TableBytes + 16 * i8d_piece_bytes(16);   // = 8 * i8d_piece_bytes(8)
    const int64_t n_tiles = (N + 15) / 16;
    const int64_t wgs = cu_count();   // int8d_ok: more tiles than that, and at most NT each
    if (M > 16)
        return launch(int8d_kernel<NT, U, D, kTiled, 8, 2>, dim3((unsigned)wgs), dim3(512), shmem, stream, (const int8_t *)x,
                      (const uint16_t *)codes, (const int64_t *)cb, (int32_t *)out, (int)M, (int)N, (int)K,
                      (int)(n_tiles / wgs), (int)(n_tiles % wgs));
    if (M > 8)
        return launch(int8d_kernel<NT, U, D, kTiled, 8>, dim3((unsigned)wgs), dim3(512), shmem, stream, (const int8_t *)x,
                      (const uint16_t *)codes, (const int64_t *)cb, (int32_t *)out, (int)M, (int)N, (int)K,
                      (int)(n_tiles / wgs), (int)(n_tiles % wgs));
    return launch(int8d_kernel<NT, U, D, kTiled, 16>, dim3((unsigned)wgs), dim3(1024), shmem, stream, (const int8_t *)x,
                  (const uint16_t *)codes, (const int64_t *)cb, (int32_t *)out, (int)M, (int)N, (int)K,
                  (int)(n_tiles / wgs), (int)(n_tiles % wgs));
}

template <bool kTiled>
int launch_int8d(const void *x, const void *codes, const void *cb, void *out, int64_t M, int64_t N, int64_t K,
                 hipStream_t stream)
{
    const int64_t n_tiles = (N + 15) / 16;
    const int cus = cu_count();
    switch ((int)((n_tiles + cus - 1) / cus)) {
        case 2: return launch_int8d_inst<2, 1, 2, kTiled>(x, codes, cb, out, M, N, K, stream);
        case 3: return launch_int8d_inst<3, 1, 3, kTiled>(x, codes, cb, out, M, N, K, stream);
        case 4: return launch_int8d_inst<4, 1, 2, kTiled>(x, codes, cb, out, M, N, K, stream);
        case 5:
        case 6: return launch_int8d_inst<6, 1, 3, kTiled>(x, codes, cb, out, M, N, K, stream);
        default: return launch_int8d_inst<8, 1, 2, kTiled>(x, codes, cb, out, M, N, K, stream);
    }
}

// does the matrix-vector route of the integer operator take the kernel with resident sums?  g_choice[3]: 0 never,
// 1 wherever it can run
// ... from K = 1024 on for up to 16 rows (from 512 on for up to 8 rows on at most four tiles per compute unit) and
// from K = 4096 on for 17 to 32: with fewer k steps than waves the row-block kernel is ahead (us, row blocks / this
// kernel: M = 16 32768 x 512 6.8 / 8.0, M = 8 32768 x 512 6.6 / 7.1, M = 32 8192 x 512 5.1 / 6.6, 8192 x 2048 6.6 / 7.1;
// but M = 8 16384 x 512 5.1 / 4.7, M = 16 16384 x 1024 6.3 / 5.8, M = 32 11008 x 4096 10.1 / 9.3, 28672 x 8192 30.8 / 24.9)
inline bool int8_takes_resident(int64_t M, int64_t N, int64_t K, int cus)
{
    const int force = g_choice[3].load(std::memory_order_relaxed);
    const int64_t share = ((N + 15) / 16 + cus - 1) / cus;
    const int64_t k_min = M > 16 ? 4096 : M <= 8 && share <= 4 ? 512 : 1024;
    return int8d_ok(M, N, cus) && force != 0 && (force == 1 || K >= k_min);
}

// any number of rows of x, 16 per pass
template <bool kTiled>
int run_int8x(const void *x, const void *codes, const void *cb, void *out, int64_t M, int64_t N, int64_t K,
              hipStream_t stream)
{
    if (int8_takes_resident(M, N, K, cu_count())) return launch_int8d<kTiled>(x, codes, cb, out, M, N, K, stream);
    switch (small_batch_row_block((N + 15) / 16, cu_count())) {
        case 1: return launch_int8x<1, kTiled>(x, codes, cb, out, M, N, K, stream);
        case 2: return launch_int8x<2, kTiled>(x, codes, cb, out, M, N, K, stream);
        case 3: return launch_int8x<3, kTiled>(x, codes, cb, out, M, N, K, stream);
        default: return launch_int8x<4, kTiled>(x, codes, cb, out, M, N, K, stream);
    }
}

// CU count for the pure queries (kernel names, workspace size), which must answer without a
// device: the current device's if it has been set up, else the MI355X's 256
int cu_count_or_default()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    return g_dev[dev].ready.load(std::memory_order_acquire) ? g_dev[dev].cus : 256;
}

// More than 32 rows of x, passes of the small-batch kernel or the matrix-matrix kernel: the latter costs about
// K * 6.9 ns (x tiles of up to 64 rows) or K * 10.4 ns (128 rows) per round of one 256-row tile per CU, however
// few of its tiles exist.  The cheaper estimate wins.  Graph launches, us, matrix-matrix / passes: M = 64 11008 ->
// 4096 75.7 / 28.4, 28672 -> 8192 186.7 / 95.6, 8192 -> 28672 57.7 / 79.6; M = 128 4096 -> 11008 49.1 / 39.7, 8192 ->
// 8192 87.9 / 55.1; M = 256 4096 -> 4096 47.9 / 44.2, 4096 -> 11008 49.5 / 73.8, 11008 -> 4096 125.2 / 97.7,
// 8192 -> 8192 88.7 / 107.5.
bool passes_beat_gemm(int64_t M, int64_t N, int64_t K, int cus)
{
    const int tm = gemm_reg_tm(M);
    const int64_t tiles = ((M + 32 * tm - 1) / (32 * tm)) * ((N + kGrBN - 1) / kGrBN);
    const double t_gemm = 3.0 + (double)((tiles + cus - 1) / cus) * (double)K * (tm == 4 ? 0.0104 : 0.0069);
    return passes_cost_us(M, N, K, cus) < t_gemm;
}

// the operator's dispatch once the arguments are checked and the device is ready
int dispatch_f16(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M, int64_t N,
                 int64_t K, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    const int force = M > 16 ? g_choice[0].load(std::memory_order_relaxed) : -1;
    if (force == 0 && gemv_rows_ok(x, codes, grid, y, M, N, K))
        return M <= 32 ? run_gemv<false>(x, codes, grid, scale, y, M, N, K, s)
                       : run_gemv_regx<false>(x, codes, grid, scale, y, M, N, K, s);
    if (force == 1 && gemm_ok(x, codes, grid, y, M, N, K)) return run_gemm(x, codes, grid, scale, y, M, N, K, s);
    if (workspace && workspace_bytes > 0 && splitk_ok(x, codes, grid, y, M, N, K) &&
        (force == 2 || !(passes_beat_splitk(M, N, K, cu_count()) && gemv_rows_ok(x, codes, grid, y, M, N, K)))) {
        const int splits = splitk_plan(M, N, K, workspace_bytes, cu_count());
        if (splits >= 2) return launch_gemm_splitk(x, codes, grid, scale, y, workspace, splits, M, N, K, s);
    }
    if (gemv_ok(x, codes, grid, y, M, N, K)) return run_gemv<false>(x, codes, grid, scale, y, M, N, K, s);
    if (gemv_rows_ok(x, codes, grid, y, M, N, K) && passes_beat_gemm(M, N, K, cu_count()))
        return run_gemv_regx<false>(x, codes, grid, scale, y, M, N, K, s);
    if (gemm_ok(x, codes, grid, y, M, N, K)) return run_gemm(x, codes, grid, scale, y, M, N, K, s);
    return run_generic(x, codes, grid, scale, y, M, N, K, s);
}

// ------------------------------------------------------------------ the operator on host memory
// The reference's own CPU path is a scalar decode and a triple loop (/root/reference/test_decode_matmul.py:29-71);
// this is the same thing for the half-precision form, in plain C++ for tensors that live in host
// memory: no GPU is involved and no GPU call is made.  Not a fallback: device pointers never come
// here, the entry points below are separate ones.  One rounding per weight (the fp32 sum of a half
// and +-1/4 is exact), fp32 sums over k in ascending order, rows of W spread over host threads.
inline void host_decode_row(const uint16_t *codes, const half_t *grid, int64_t kc, half_t *w)
{
    for (int64_t j = 0; j < kc; j++) {
        const uint32_t c = codes[j];
        const uint32_t idx = c & 0xFFu, s7 = (c >> 8) & 0x7Fu;
        const uint32_t s8 = s7 | ((uint32_t)(__builtin_popcount(s7) & 1) << 7);
        const float shift = (c & 0x8000u) ? -0.25f : 0.25f;
        for (int d = 0; d < 8; d++) {
            const float g = (float)grid[idx * 8 + d];
            w[j * 8 + d] = (half_t)(((s8 >> d) & 1u ? -g : g) + shift);
        }
    }
}

// Rows [0, n_rows) split over host threads; body(n0, n1) must not throw.  Threads cost about 50 us
// each to start, so only work of 2^24 multiply-adds or more (several milliseconds on one core) gets
// any, and never more than one per 2^22.  If a thread cannot be started the rows it was to
// take run on the calling thread.
template <typename F>
void host_parallel_rows(int64_t n_rows, int64_t work_per_row, F body) noexcept
{
    const int64_t work = n_rows * work_per_row;
    unsigned threads = std::thread::hardware_concurrency();
    if (threads == 0) threads = 1;
    if (threads > 16) threads = 16;
    if ((int64_t)threads > (work >> 22)) threads = (unsigned)(work >> 22);
    if ((int64_t)threads > n_rows) threads = (unsigned)n_rows;
    if (work < (1 << 24) || threads < 2) {
        body(0, n_rows);
        return;
    }
    std::thread pool[16];
    unsigned started = 0;
    for (unsigned t = 1; t < threads; t++) {
        try {
            pool[started] = std::thread([=] { body(n_rows * t / threads, n_rows * (t + 1) / threads); });
        } catch (...) {   // std::system_error: no more threads to be had
            body(n_rows * t / threads, n_rows);
            break;
        }
        started++;
    }
    body(0, n_rows / threads);
    for (unsigned t = 0; t < started; t++) pool[t].join();
}
