// libdmm: decode+matmul for MI355X (gfx950, CDNA4).  Kernels and the C ABI of include/dmm.h.
//
// The weight matrix arrives as 16-bit codes, one per 8 consecutive weights along K
// (format: /root/reference/test_decode_matmul.py:29-55,
//          /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:45-65).
// Decoding one code is: one 16-byte LDS read of the grid row, one 16-byte LDS read of a
// (+-1.0 x 8) sign row indexed by the seven sign bits (the parity-implied eighth sign is
// baked into that table), one integer op for the packed +-0.25, and four packed-half FMAs
//     w = g * s + delta          (g * +-1 is exact, so this is the flip-then-add of the
//                                 reference with a single rounding)
// whose result registers are, unchanged, the 8-halves-per-lane operand of the
// 16x16x32 / 32x32x16 half MFMA.  Nothing decoded ever goes back through memory on the
// matrix-vector path.
//
// This file is the one translation unit of the library: shared types, then the kernel files
// beside it (each included once, inside namespace dmm, in dependency order), then the
// extern "C" entry points.
//   dmm_tables.h      decode tables, decode of one code, standalone decoder, catch-all operator
//   dmm_gemv_f16.h    matrix-vector helpers and the streaming kernel on 16-bit operands
//   dmm_gemv_q8.h     matrix-vector kernels on 8-bit operands (fp8 weights, bf8 terms of x)
//   dmm_gemv_q8d.h    batch 1 on 8-bit operands, every tile of a workgroup in registers
//   dmm_gemv_small.h  small-batch kernel with x in registers
//   dmm_gemm.h        matrix-matrix kernels and the split-K reduction
//   dmm_int8.h        the reference's integer operator
//   dmm_aux.h         offline repack, read probe
//   dmm_host.h        library scratch memory, launch plumbing, set-up, checks and dispatch
#include <hip/hip_runtime.h>
#include <atomic>
#include <mutex>
#include <thread>
#include <type_traits>
#include <vector>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "dmm.h"

namespace dmm {

typedef _Float16 half_t;
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
typedef int i8_t __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

#include "dmm_tables.h"
#include "dmm_gemv_f16.h"
#include "dmm_gemv_q8.h"
#include "dmm_gemv_q8d.h"
#include "dmm_gemv_f16d.h"
#include "dmm_gemv_small.h"
#include "dmm_gemm.h"
#include "dmm_int8.h"
#include "dmm_aux.h"
#include "dmm_host.h"

}  // namespace dmm

using namespace dmm;

extern "C" {

int dmm_version(void) { return (0 << 16) | 2; }

const char *dmm_status_string(int status)
{
    switch (status) {
        case DMM_OK: return "ok";
        case DMM_ERR_NULL_POINTER: return "a required pointer is NULL";
        case DMM_ERR_BAD_SHAPE: return "bad shape: sizes must be non-negative and K a multiple of 8";
        case DMM_ERR_MISALIGNED: return "a pointer does not meet the required alignment";
        case DMM_ERR_TOO_LARGE: return "a dimension is too large for the launch";
        case DMM_ERR_UNSUPPORTED: return "this explicit path does not support the given shape or alignment";
        case DMM_ERR_NOT_INITIALIZED:
            return "first call on this device while its stream is being captured: call dmm_init before capturing";
        case DMM_ERR_INTERNAL: return "a table kernel was built with static LDS (library build error)";
        case DMM_ERR_SCRATCH_TOO_SMALL:
            return "the split-K partial sums of this shape exceed the library's 16 MiB scratch buffer: use "
                   "dmm_decode_matmul_ws_f16 with a workspace of dmm_workspace_bytes, or dmm_decode_matmul_f16";
        case DMM_ERR_HOST_MEMORY: return "host memory for a decoded row could not be allocated";
        default: break;
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "unknown status";
}

int dmm_init(int device)
{
    int cur = 0;
    hipError_t e = hipGetDevice(&cur);
    if (e != hipSuccess) return (int)e;
    if (device < 0) device = cur;
    if (device >= kMaxDevices) return DMM_ERR_TOO_LARGE;
    if (device != cur) {
        e = hipSetDevice(device);
        if (e != hipSuccess) return (int)e;
    }
    const int st = init_current_device(device);
    if (device != cur) (void)hipSetDevice(cur);
    return st;
}

int dmm_set_kernel_events(void *start_event, void *stop_event)
{
    if ((start_event == nullptr) != (stop_event == nullptr)) return DMM_ERR_NULL_POINTER;
    tls_start = (hipEvent_t)start_event;
    tls_stop = (hipEvent_t)stop_event;
    return DMM_OK;
}

int dmm_decode_f16(const void *codes, const void *grid, void *W, int64_t N, int64_t K, void *stream)
{
    if (N < 0 || K < 0 || (K & 7)) return DMM_ERR_BAD_SHAPE;
    const int64_t n_codes = N * (K >> 3);
    if (n_codes == 0) return DMM_OK;
    if (!codes || !grid || !W) return DMM_ERR_NULL_POINTER;
    if (!aligned(codes, 2) || !aligned(grid, 2) || !aligned(W, 2)) return DMM_ERR_MISALIGNED;
    if (int st = ensure_ready((hipStream_t)stream)) return st;
    const bool wide = aligned(codes, 4) && aligned(grid, 16) && aligned(W, 16);
    const int64_t work = wide ? (n_codes + 1) / 2 : n_codes;
    int64_t blocks = (work + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    if (wide)
        return launch(decode_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                      (const uint16_t *)codes, grid, (uint16_t *)W, n_codes);
    return launch(decode_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                  (const uint16_t *)codes, grid, (uint16_t *)W, n_codes);
}

int dmm_generic_f16(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                    int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    if ((st = ensure_ready((hipStream_t)stream))) return st;
    return run_generic(x, codes, grid, scale, y, M, N, K, (hipStream_t)stream);
}

int dmm_gemv_f16(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                 int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    if (!gemv_ok(x, codes, grid, y, M, N, K)) return DMM_ERR_UNSUPPORTED;
    if ((st = ensure_ready((hipStream_t)stream))) return st;
    return run_gemv<false>(x, codes, grid, scale, y, M, N, K, (hipStream_t)stream);
}

int dmm_set_gemv_8bit(int enabled)
{
    const int before = gemv_q8_enabled() ? 1 : 0;
    g_gemv_q8.store(enabled ? 1 : 0, std::memory_order_relaxed);
    return before;
}

int dmm_set_choice(int which, int value)
{
    if (which < 0 || which > 3 || value < -1 || value > 2) return DMM_ERR_BAD_SHAPE;
    return g_choice[which].exchange(value, std::memory_order_relaxed);
}

const char *dmm_integer_kernel_name(int64_t M, int64_t N, int64_t K)
{
    switch (pick_int8(M, N, K, cu_count_or_default())) {
        case kInt8Gemm: return "dmm::int8g_kernel";
        case kInt8Gemv: return int8_takes_resident(M, N, K, cu_count_or_default()) ? "dmm::int8d_kernel" : "dmm::int8x_kernel";
        default: return "dmm::int8_kernel";
    }
}

const char *dmm_gemv_kernel_name(int64_t M, int64_t N, int64_t K)
{
    if (M < 1 || M > 32 || N < 1 || K < 256 || (K & 255) || (N & 3) || N * (K >> 2) >= (1LL << 31)) return "";
    switch (pick_gemv(M, N, K)) {
        case kGemvStream: return "dmm::gemv_stream_kernel";
        case kGemvF16d: return "dmm::gemv_f16d_kernel";
        case kGemvQ8: return M > 1 ? "dmm::gemv_q8_kernel" : gemv_q8d_ok(N) ? "dmm::gemv_q8d_kernel" : "dmm::gemv_q8c_kernel";
        default: return "dmm::gemv_regx_kernel";
    }
}

int dmm_gemv_8bit_f16(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                      int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    if (!gemv_ok(x, codes, grid, y, M, N, K) || !gemv_8bit_ok(M, N, K)) return DMM_ERR_UNSUPPORTED;
    if ((st = ensure_ready((hipStream_t)stream))) return st;
    return run_gemv_q8<false>(x, codes, grid, scale, y, M, N, K, (hipStream_t)stream);
}

int64_t dmm_packed_bytes(int64_t N, int64_t K)
{
    if (N < 0 || K < 256 || (K & 255)) return 0;
    return ((N + 15) / 16) * 16 * (K >> 2);
}

int dmm_pack_codes(const void *codes, void *packed, int64_t N, int64_t K, void *stream)
{
    if (N < 0 || K < 0 || (K & 7)) return DMM_ERR_BAD_SHAPE;
    if (K < 256 || (K & 255)) return DMM_ERR_UNSUPPORTED;
    if (N == 0) return DMM_OK;
    if (!codes || !packed) return DMM_ERR_NULL_POINTER;
    if (!aligned(codes, 16) || !aligned(packed, 16)) return DMM_ERR_MISALIGNED;
    if (int st = ensure_ready((hipStream_t)stream)) return st;
    const int64_t pieces = dmm_packed_bytes(N, K) / 16;
    int64_t blocks = (pieces + 255) / 256;
    if (blocks > 65535 * 16) blocks = 65535 * 16;
    return launch(pack_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)codes,
                  (u4_t *)packed, N, K, pieces);
}

int dmm_gemv_packed_f16(const void *x, const void *packed, const void *grid, float scale, void *y, int64_t M,
                        int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, packed, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    // the matrix-vector kernels' domain, with the padded size in place of N * K / 4; same choice
    // of kernel as for row-major codes
    if (!gemv_ok(x, packed, grid, y, M, N, K) || dmm_packed_bytes(N, K) >= (1LL << 31)) return DMM_ERR_UNSUPPORTED;
    if ((st = ensure_ready((hipStream_t)stream))) return st;
    return run_gemv<true>(x, packed, grid, scale, y, M, N, K, (hipStream_t)stream);
}

int dmm_decode_matmul_packed_f16(const void *x, const void *packed, const void *grid, float scale, void *y,
                                 int64_t M, int64_t N, int64_t K, void *workspace, int64_t workspace_bytes,
                                 void *stream)
{
    int st = check_common(x, packed, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    if (workspace_bytes < 0) return DMM_ERR_BAD_SHAPE;
    if (workspace && workspace_bytes > 0 && !aligned(workspace, 16)) return DMM_ERR_MISALIGNED;
    const int64_t pbytes = dmm_packed_bytes(N, K);
    if (pbytes == 0 || pbytes >= (1LL << 31)) return DMM_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    const bool mm_ok = gemm_ok(x, packed, grid, y, M, N, K) && gemm_reg_ok(M, ((N + 15) / 16) * 16, K);
    const bool mv_ok = gemv_ok(x, packed, grid, y, M, N, K);
    const bool rows_ok = gemv_rows_ok(x, packed, grid, y, M, N, K);   // more than 32 rows, 16 at a time
    if (!mm_ok && !rows_ok) return DMM_ERR_UNSUPPORTED;
    if ((st = ensure_ready(s))) return st;
    if (workspace && workspace_bytes > 0 && mm_ok && M >= kSplitKMinM && aligned(y, 8) &&
        !(passes_beat_splitk(M, N, K, cu_count()) && rows_ok)) {
        const int splits = splitk_plan(M, N, K, workspace_bytes, cu_count());
        if (splits >= 2) return launch_gemm_splitk<true>(x, packed, grid, scale, y, workspace, splits, M, N, K, s);
    }
    if (mv_ok) return run_gemv<true>(x, packed, grid, scale, y, M, N, K, s);
    if (rows_ok && (!mm_ok || passes_beat_gemm(M, N, K, cu_count())))
        return run_gemv_regx<true>(x, packed, grid, scale, y, M, N, K, s);
    return launch_gemm_reg<true>(x, packed, grid, scale, y, M, N, K, s);
}

int dmm_gemm_f16(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                 int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    if (!gemm_ok(x, codes, grid, y, M, N, K)) return DMM_ERR_UNSUPPORTED;
    if ((st = ensure_ready((hipStream_t)stream))) return st;
    return run_gemm(x, codes, grid, scale, y, M, N, K, (hipStream_t)stream);
}

int dmm_decode_matmul_i8(const void *x, const void *codes, const void *codebook_abs, void *out, int64_t M,
                         int64_t N, int64_t K, int tiled, void *stream)
{
    if (M < 0 || N < 0 || K < 0 || (K & 7)) return DMM_ERR_BAD_SHAPE;
    if (tiled && ((N & 15) || (K & 31))) return DMM_ERR_BAD_SHAPE;   // the tile is 16 rows x 4 codes
    if (M == 0 || N == 0) return DMM_OK;
    if (!out || !codebook_abs) return DMM_ERR_NULL_POINTER;
    if (K > 0 && (!x || !codes)) return DMM_ERR_NULL_POINTER;
    if (!aligned(codes, 2) || !aligned(codebook_abs, 8) || !aligned(out, 4)) return DMM_ERR_MISALIGNED;
    if (int st = ensure_ready((hipStream_t)stream)) return st;
    if (K == 0) {
        const int64_t n = M * N;
        const unsigned blocks = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
        return launch(zero_i32_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (int32_t *)out, n);
    }
    // the matrix-unit kernels (K <= 2^17: their weights are odd, so |w| <= 127 and no sum of K
    // products leaves int32 - nothing depends on what the matrix unit does on overflow)
    Int8Kind kind =
        aligned(x, 16) && aligned(codes, 16) && aligned(out, 16) ? pick_int8(M, N, K, cu_count()) : kInt8Scalar;
    if (kind != kInt8Scalar && M > 16) {   // both matrix-unit kernels can take it: a benchmark may force one
        const int force = g_choice[1].load(std::memory_order_relaxed);
        if (force == 1) kind = kInt8Gemv;
        if (force == 2) kind = kInt8Gemm;
    }
    if (kind == kInt8Gemm)
        return tiled ? launch_int8g<true>(x, codes, codebook_abs, out, M, N, K, (hipStream_t)stream)
                     : launch_int8g<false>(x, codes, codebook_abs, out, M, N, K, (hipStream_t)stream);
    if (kind == kInt8Gemv)   // 16 rows of x per pass of the one launch
        return tiled ? run_int8x<true>(x, codes, codebook_abs, out, M, N, K, (hipStream_t)stream)
                     : run_int8x<false>(x, codes, codebook_abs, out, M, N, K, (hipStream_t)stream);
    int64_t blocks = (N + 3) / 4;
    if (blocks > 65535 * 16) blocks = 65535 * 16;
    return launch(int8_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const int8_t *)x,
                  (const uint16_t *)codes, (const int64_t *)codebook_abs, (int32_t *)out, M, N, K, tiled ? 1 : 0,
                  aligned(x, 8) ? 1 : 0);
}

int64_t dmm_workspace_bytes(int64_t M, int64_t N, int64_t K)
{
    if (M < 1 || N < 1 || K < kGrBK || (K & 63) || M < kSplitKMinM || M > 65535LL * 128 || !gemm_reg_ok(M, N, K))
        return 0;
    // the small-batch kernel takes it, without a workspace (unless a benchmark forces the split)
    if (passes_beat_splitk(M, N, K, cu_count_or_default()) && g_choice[0].load(std::memory_order_relaxed) != 2) return 0;
    const int splits = splitk_plan(M, N, K, INT64_MAX, cu_count_or_default());
    return splits >= 2 ? (int64_t)splits * M * N * 4 : 0;
}

int dmm_decode_matmul_ws_f16(const void *x, const void *codes, const void *grid, float scale, void *y,
                             int64_t M, int64_t N, int64_t K, void *workspace, int64_t workspace_bytes,
                             void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    if (workspace_bytes < 0) return DMM_ERR_BAD_SHAPE;
    if (workspace && workspace_bytes > 0 && !aligned(workspace, 16)) return DMM_ERR_MISALIGNED;
    if ((st = ensure_ready((hipStream_t)stream))) return st;
    return dispatch_f16(x, codes, grid, scale, y, M, N, K, workspace, workspace_bytes, (hipStream_t)stream);
}

int dmm_decode_host_f16(const void *codes, const void *grid, void *W, int64_t N, int64_t K)
{
    if (N < 0 || K < 0 || (K & 7)) return DMM_ERR_BAD_SHAPE;
    if (N == 0 || K == 0) return DMM_OK;
    if (!codes || !grid || !W) return DMM_ERR_NULL_POINTER;
    if (!aligned(codes, 2) || !aligned(grid, 2) || !aligned(W, 2)) return DMM_ERR_MISALIGNED;
    const int64_t kc = K >> 3;
    host_parallel_rows(N, K, [=](int64_t n0, int64_t n1) {
        for (int64_t n = n0; n < n1; n++)
            host_decode_row((const uint16_t *)codes + n * kc, (const half_t *)grid, kc, (half_t *)W + n * K);
    });
    return DMM_OK;
}

int dmm_decode_matmul_host_f16(const void *x, const void *codes, const void *grid, float scale, void *y, int64_t M,
                               int64_t N, int64_t K)
{
    const int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    const int64_t kc = K >> 3;
    const half_t *xh = (const half_t *)x;
    half_t *yh = (half_t *)y;
    std::atomic<int> failed{0};
    std::atomic<int> *failed_p = &failed;
    host_parallel_rows(N, K * (M + 1), [=](int64_t n0, int64_t n1) {
        half_t *w = (half_t *)malloc((size_t)K * sizeof(half_t));   // one decoded row
        if (!w) {
            failed_p->store(1, std::memory_order_relaxed);
            return;
        }
        for (int64_t n = n0; n < n1; n++) {
            host_decode_row((const uint16_t *)codes + n * kc, (const half_t *)grid, kc, w);
            for (int64_t m = 0; m < M; m++) {
                float acc = 0.f;
                for (int64_t k = 0; k < K; k++) acc += (float)xh[m * K + k] * (float)w[k];
                yh[m * N + n] = (half_t)(acc * scale);
            }
        }
        free(w);
    });
    return failed.load(std::memory_order_relaxed) ? DMM_ERR_HOST_MEMORY : DMM_OK;
}

int dmm_read_probe(const void *codes, void *sink, int64_t N, int64_t K, void *stream)
{
    if (N < 1 || K < 256 || (K & 255) || N * (K >> 2) >= (1LL << 31)) return DMM_ERR_UNSUPPORTED;
    if (!codes || !sink) return DMM_ERR_NULL_POINTER;
    if (!aligned(codes, 16) || !aligned(sink, 4)) return DMM_ERR_MISALIGNED;
    if (int st = ensure_ready((hipStream_t)stream)) return st;
    const int64_t n_tiles = (N + 15) / 16;
    const int64_t wgs = n_tiles < cu_count() ? n_tiles : cu_count();
    return launch(read_probe_kernel, dim3((unsigned)wgs), dim3(1024), 0, (hipStream_t)stream, (const uint16_t *)codes,
                  (uint32_t *)sink, (int)N, (int)K, (int)(n_tiles / wgs), (int)(n_tiles % wgs));
}

int64_t dmm_noalloc_scratch_bytes(void) { return kScratchBytes; }

int dmm_decode_matmul_noalloc_f16(const void *x, const void *codes, const void *grid, float scale, void *y,
                                  int64_t M, int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    // what dmm_decode_matmul_ws_f16 would like as a workspace must fit the library's buffer
    const int64_t want = splitk_ok(x, codes, grid, y, M, N, K) ? dmm_workspace_bytes(M, N, K) : 0;
    if (want > kScratchBytes) return DMM_ERR_SCRATCH_TOO_SMALL;
    const DeviceState *ds = nullptr;
    if ((st = ensure_ready((hipStream_t)stream, &ds))) return st;
    return dispatch_f16(x, codes, grid, scale, y, M, N, K, want > 0 ? ds->scratch : nullptr, want, (hipStream_t)stream);
}

int dmm_decode_matmul_f16(const void *x, const void *codes, const void *grid, float scale, void *y,
                          int64_t M, int64_t N, int64_t K, void *stream)
{
    int st = check_common(x, codes, grid, y, M, N, K);
    if (st != DMM_OK || M == 0 || N == 0) return st;
    if ((st = ensure_ready((hipStream_t)stream))) return st;
    return dispatch_f16(x, codes, grid, scale, y, M, N, K, nullptr, 0, (hipStream_t)stream);
}

}  // extern "C"
