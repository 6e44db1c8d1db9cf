/* dmm.h - C ABI of the MI355X (gfx950) decode+matmul library, libdmm.so.
 *
 * This is the boundary a host binding (the PyTorch extension in
 * decode_matmul_amd/csrc/torch_binding.cpp, a ctypes stub, cgo, ...) binds to.
 * Plain pointers and sizes only.  Every pointer is a DEVICE pointer unless a comment
 * says otherwise.  The library never allocates, frees or retains caller memory, never
 * synchronises the device and never terminates the process: every entry point enqueues
 * its kernels on the caller's stream and returns a status code.
 *
 * Host work outside the launches happens once per device, in dmm_init: the compute-unit
 * count is read, the kernels' dynamic-LDS limits are raised (hipFuncSetAttribute) and the
 * library's one device buffer is located.  An entry point called on a device that has not
 * been initialised does this itself first - except when its stream is being captured into
 * a HIP graph, where it returns DMM_ERR_NOT_INITIALIZED instead: call dmm_init (or make one
 * eager call) before capturing.  After that every entry point only enqueues kernels and
 * can be captured.
 *
 * The choice between kernels depends on the device's compute-unit count.  The queries that
 * predict it without touching a device (dmm_workspace_bytes, dmm_gemv_kernel_name,
 * dmm_integer_kernel_name) assume 256 compute units until dmm_init (or a first call) has read
 * the real count on the calling thread's device: on any other part they are exact only after
 * that.  The choice itself was fitted on the 256-unit MI355X.
 *
 * Code format (one 16-bit code per 8 consecutive weights along K), as defined by
 * /root/reference/test_decode_matmul.py:29-55 and
 * /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:45-65:
 *   bits 0-7   grid row                     bits 8-14  sign flips of dims 0-6
 *   dim 7 sign parity of bits 8-14          bit 15     set: shift -1/4, clear: +1/4
 *   w[d] = half( (sign_d ? -grid[row][d] : grid[row][d]) + shift )   (flip, then one add)
 *   W[n, 8*j + d] = decode(codes[n, j])[d]
 */
#ifndef DMM_H
#define DMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes.  0 = success.  Negative = the call was rejected on the host before any
 * launch.  Positive = a hipError_t reported by the HIP runtime for the launch. */
enum {
    DMM_OK = 0,
    DMM_ERR_NULL_POINTER = -1,  /* a required pointer is NULL                          */
    DMM_ERR_BAD_SHAPE = -2,     /* M, N or K negative, K not a multiple of 8, or a
                                   shape constraint of the entry point is violated      */
    DMM_ERR_MISALIGNED = -3,    /* a pointer misses the alignment the entry point asks  */
    DMM_ERR_TOO_LARGE = -4,     /* a dimension exceeds what the launch can index        */
    DMM_ERR_UNSUPPORTED = -5,   /* explicit-path entry point called outside its domain  */
    DMM_ERR_NOT_INITIALIZED = -6, /* first call on a device made under stream capture     */
    DMM_ERR_INTERNAL = -7,      /* the library was built wrongly (a table kernel has
                                   static LDS); no kernel was launched                  */
    DMM_ERR_SCRATCH_TOO_SMALL = -8, /* dmm_decode_matmul_noalloc_f16: the shape's partial
                                   sums exceed the library's scratch buffer             */
    DMM_ERR_HOST_MEMORY = -9    /* dmm_decode_matmul_host_f16: malloc of a row failed   */
};

/* Library version, (major << 16) | minor. */
int dmm_version(void);

/* Human-readable text for a status code returned by this library (static storage). */
const char *dmm_status_string(int status);

/* One-time set-up of a device (device < 0: the current one); see the note on host work
 * above.  Idempotent and thread-safe; restores the current device before it returns.  The
 * reference does the corresponding host work on every call
 * (cudaGetDeviceProperties, /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:217-218). */
int dmm_init(int device);

/* Standalone decoder: codes [N, K/8] row-major -> W half [N, K] row-major.
 * Replaces the decode half of the fused reference kernel
 * (decode8weights, /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:45-65) in the
 * half-precision form of the same code; it is the bit-exact gate of the library and the
 * front half of the decode-then-dense-GEMM comparison.
 *   codes  uint16/int16 bits, 2-byte aligned         grid  half [256,8], 2-byte aligned
 *   W      half, 2-byte aligned (16-byte alignment of all three enables the wide path) */
int dmm_decode_f16(const void *codes, const void *grid, void *W,
                   int64_t N, int64_t K, void *stream);

/* The operator: y[M,N] = half( scale * sum_k x[m,k] * W[n,k] ), W decoded on the fly,
 * fp32 accumulation.  Replaces the host wrapper and kernel launch of
 * /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:178-234 (operator
 * `decode_matmul`), in the half-precision form: x half [M,K], codes [N,K/8], grid half
 * [256,8], scalar scale, y half [M,N], all row-major and contiguous.  The only shape
 * demand is K % 8 == 0 (the reference's M%8, N%16, K%2048 demands,
 * decode_matmul_cuda.cu:195-207, do not apply).  Chooses the kernel from M, the shape and
 * the pointer alignments; y is fully overwritten (no caller zeroing).  A few dozen to a few
 * hundred rows of x give the matrix-matrix kernel too few tiles to fill the chip; without a
 * workspace (below) such a call runs as passes of the small-batch kernel, 16 rows of x each,
 * where a cost estimate says that is faster. */
int dmm_decode_matmul_f16(const void *x, const void *codes, const void *grid, float scale,
                          void *y, int64_t M, int64_t N, int64_t K, void *stream);

/* The operator with a caller-provided workspace.  No counterpart in the reference (its one
 * kernel accumulates split-K partial sums with atomics into the zero-initialised output,
 * /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:95,172,210-215, which an fp16 output
 * cannot take).  When x is short (17 <= M, up to a few hundred rows) one block per output
 * tile leaves most of the chip idle; with a workspace the K dimension is split over several
 * blocks per tile, each writes fp32 partial sums to the workspace and a second small kernel
 * adds them in a fixed order (results stay bit-reproducible), scales and rounds into y.
 *   dmm_workspace_bytes  the size that lets the call split as far as it would like to
 *                        (0: this shape never uses a workspace - among others up to 32 rows
 *                        of x on up to 17 MB of codes, which the small-batch kernel serves
 *                        faster); any smaller size is legal and only limits the split.
 *   workspace            device memory, 16-byte aligned, owned by the caller; it must not be
 *                        used by another call that may run at the same time (other stream).
 *                        NULL or workspace_bytes == 0: identical to dmm_decode_matmul_f16. */
int64_t dmm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int dmm_decode_matmul_ws_f16(const void *x, const void *codes, const void *grid, float scale,
                             void *y, int64_t M, int64_t N, int64_t K, void *workspace,
                             int64_t workspace_bytes, void *stream);

/* The operator for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same result as dmm_decode_matmul_ws_f16 with a workspace of dmm_workspace_bytes(M, N, K),
 * bit for bit, but the split-K partial sums go to a buffer inside the library: a 16 MiB
 * static device array (dmm_noalloc_scratch_bytes), one copy per GPU the library runs on,
 * held until the process ends.  The call allocates nothing and frees nothing.  A shape whose
 * preferred workspace exceeds the buffer is rejected with DMM_ERR_SCRATCH_TOO_SMALL (nothing is
 * launched): this is a hard limit - serving such a shape with fewer splits would break the
 * bit-identity with the full workspace.  It concerns a band of middle-sized M only (M <= 64 is
 * always accepted, and so is every M large enough to fill the chip without a split): on 256
 * compute units the rejected M are 113 .. 1024 for N x K = 4096 x 4096, 65 .. 1024 for 4096 x 11008,
 * 77 .. 256 for 11008 x 4096, 65 .. 512 for 8192 x 8192 and 8192 x 28672, 69 .. 384 for
 * 10240 x 8192, 74 .. 128 for 28672 x 8192 (not every M inside a band: ask
 * dmm_workspace_bytes(M, N, K) <= dmm_noalloc_scratch_bytes()).  Shapes that use no
 * workspace (M <= 16, or too few k tiles to split) run exactly as dmm_decode_matmul_f16.  Every partial sum is written before it is read, so the buffer
 * needs no clearing between calls; but all calls on one GPU share it: two such calls that
 * may overlap (different streams, or graphs replayed concurrently) race. */
int64_t dmm_noalloc_scratch_bytes(void);
int dmm_decode_matmul_noalloc_f16(const void *x, const void *codes, const void *grid, float scale,
                                  void *y, int64_t M, int64_t N, int64_t K, void *stream);

/* Explicit paths of the operator, for tests and measurement.  Same arguments.  Each
 * returns DMM_ERR_UNSUPPORTED outside its domain instead of falling back:
 *   dmm_gemv_f16     M <= 32, K % 256 == 0, N % 4 == 0, 16-byte aligned x/codes/grid,
 *                    8-byte aligned y.  Decoded registers feed the MFMA unit directly;
 *                    HBM-bound on the code bytes N*K/4 (more than 16 rows of x: every
 *                    workgroup walks its rows of W once per 16 rows of x, so the codes come
 *                    from HBM once and from the caches after that).
 *   dmm_gemm_f16     K % 64 == 0, 16-byte aligned x/codes/grid.  Decoded tiles staged in
 *                    LDS, fp16 MFMA with fp32 accumulate.
 *   dmm_generic_f16  any K % 8 == 0, 2-byte alignment: wave-per-row dot products with a
 *                    DPP wave reduction.  The catch-all. */
int dmm_gemv_f16(const void *x, const void *codes, const void *grid, float scale,
                 void *y, int64_t M, int64_t N, int64_t K, void *stream);
/*   dmm_gemv_8bit_f16  the matrix-vector kernels on 8-bit MFMA operands, which dmm_gemv_f16 and
 *                    the operator pick for M = 1 on launches of more than one 16-row tile per
 *                    compute unit (from one on when K >= 16384) and for M = 2 .. 4 on launches of
 *                    more than eight (below that a 16-bit kernel is faster).  Weights as fp8 (e4m3) bytes - exact when
 *                    every grid value has at most 4 significant bits in fp8's range, as the E8P
 *                    grid does - and x as four bf8 (e5m2) terms that add up to it exactly; the
 *                    +-1/4 shift of a code is added through the per-code means of x (two halves,
 *                    hi + lo, times +-2 in a 16-bit MFMA of their own).  Nothing is lost in the
 *                    operands; the 8-bit MFMA aligns the products of a group to the largest of
 *                    them, so y is not always the 16-bit kernel's bit for bit: 98 % of the
 *                    outputs are the correctly rounded ones and the rest are one half ulp off
 *                    (99th percentile of the error 0.57 ulps; the tolerance of the operator is
 *                    1e-2, thousands of ulps).  A grid that does not fit fp8, or an x that is not
 *                    finite, is detected inside the launch and served by the 16-bit kernel: same
 *                    call, same status.  dmm_set_gemv_8bit(0), or DMM_GEMV_8BIT=0 in the
 *                    environment, keeps the operator off these kernels.  Domain: that of
 *                    dmm_gemv_f16 with M <= 4; at M = 1 the terms of x go through the LDS 4096
 *                    values at a time, so K is only limited by the 16-bit kernel the launch may
 *                    hand over to (K <= 31488); at M = 2 .. 4 the terms of x and of its means have
 *                    to fit the LDS beside the tables and the partial sums (4 M (K + 16) +
 *                    2 M (K / 4 + 16) bytes: K <= 6656 / 4352 / 3072).  DMM_ERR_UNSUPPORTED
 *                    outside.  No counterpart in the reference (its kernel multiplies int8 by
 *                    int8). */
int dmm_gemv_8bit_f16(const void *x, const void *codes, const void *grid, float scale,
                      void *y, int64_t M, int64_t N, int64_t K, void *stream);
/* Process-wide switch for the 8-bit kernel in the operator's choice (explicit calls of
 * dmm_gemv_8bit_f16 are not affected): 0 keeps batch 1 on the 16-bit kernel, whose y is the
 * correctly rounded fp32-accumulated product; non-zero (the default, unless DMM_GEMV_8BIT=0 is
 * set in the environment) allows the 8-bit one.  Returns the previous setting.  Takes effect
 * for calls made after it returns.  No counterpart in the reference. */
int dmm_set_gemv_8bit(int enabled);
/* Which matrix-vector kernel the operator runs for a shape with aligned pointers, as a profiler's
 * kernel trace names it without the template arguments ("dmm::gemv_q8d_kernel" - one row of x on
 * 8-bit operands, up to eight row tiles per compute unit -, "dmm::gemv_q8c_kernel" - the same for
 * more tiles -, "dmm::gemv_q8_kernel", "dmm::gemv_stream_kernel", "dmm::gemv_f16d_kernel" - up to 32
 * rows on 16-bit operands, up to eight row tiles per compute unit -, "dmm::gemv_regx_kernel"; ""
 * outside dmm_gemv_f16's domain).  For
 * benchmarks that report per kernel.  Static storage.  No counterpart in the reference. */
const char *dmm_gemv_kernel_name(int64_t M, int64_t N, int64_t K);
int dmm_gemm_f16(const void *x, const void *codes, const void *grid, float scale,
                 void *y, int64_t M, int64_t N, int64_t K, void *stream);
int dmm_generic_f16(const void *x, const void *codes, const void *grid, float scale,
                    void *y, int64_t M, int64_t N, int64_t K, void *stream);

/* Offline repack for the batch-1 kernel (the counterpart of the reference's `transpose_tile`,
 * /root/reference/test_decode_matmul.py:101-109, which pre-tiles the codes for ITS kernel's
 * fragment loads).  In the packed form the 16 bytes a lane loads sit at
 *   ((tile * (K / 256) + step) * 64 + lane) * 16,   tile = n / 16, step = k / 256,
 *   lane = n % 16 + 16 * (k % 256 / 64),
 * so a wave's load is 1 KB of consecutive bytes instead of 16 rows x 64 bytes; rows are padded
 * with zeros to a multiple of 16.  Same arithmetic in the same order as the row-major call:
 * results are bit-identical.  K % 256 == 0 is required (DMM_ERR_UNSUPPORTED otherwise).
 *   dmm_packed_bytes     size of the packed buffer (0 if the shape cannot be packed)
 *   dmm_pack_codes       codes [N, K/8] row-major -> packed; both 16-byte aligned, distinct
 *   dmm_decode_matmul_packed_f16  the operator on packed codes, any M: the matrix-vector
 *                        kernels for M <= 32, the register-operand MFMA kernel above (its code
 *                        loads become two runs of 256 consecutive bytes per wave), split-K when
 *                        a workspace is given (same rules as dmm_decode_matmul_ws_f16; NULL, 0
 *                        for none).  16-byte aligned x, packed, grid; DMM_ERR_UNSUPPORTED for
 *                        what the packed kernels do not cover (K % 256, unaligned pointers,
 *                        packed size of 2 GiB or more).
 *   dmm_gemv_packed_f16  explicit matrix-vector path on packed codes; domain: that of
 *                        dmm_gemv_f16 (M <= 32, N % 4 == 0, aligned pointers). */
int64_t dmm_packed_bytes(int64_t N, int64_t K);
int dmm_pack_codes(const void *codes, void *packed, int64_t N, int64_t K, void *stream);
int dmm_decode_matmul_packed_f16(const void *x, const void *packed, const void *grid, float scale,
                                 void *y, int64_t M, int64_t N, int64_t K, void *workspace,
                                 int64_t workspace_bytes, void *stream);
int dmm_gemv_packed_f16(const void *x, const void *packed, const void *grid, float scale,
                        void *y, int64_t M, int64_t N, int64_t K, void *stream);

/* The reference's operator itself, in integers:
 *   out int32 [M,N] = x int8 [M,K]  @  decode(codes, codebook_abs) int8 [N,K] ^T
 * Replaces `decode_matmul(x, weights_compressed, codebook_abs)` of
 * /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:178-234 with its dtypes (int8, int16,
 * int64 -> int32).  codebook_abs is the packed table of
 * /root/reference/test_decode_matmul.py:74-86 (byte d of entry i = dim d, as int8).  tiled != 0:
 * codes are in the layout the reference's kernel reads, `transpose_tile` of
 * /root/reference/test_decode_matmul.py:101-109 (needs N % 16 == 0 and K % 32 == 0, as
 * decode_matmul_cuda.cu:196-197 does); tiled == 0: plain row-major [N, K/8].  None of the
 * reference's other shape demands (M % 8, K % 2048, K >= 4096) apply.  Exact integer
 * arithmetic (int32 sums wrap); `out` is fully overwritten.  With K % 256 == 0, N % 4 == 0 and
 * 16-byte aligned x, codes and out the call runs on the int8 matrix unit - 16 rows of x per
 * launch of a matrix-vector kernel, or one launch of a matrix-matrix kernel when x has many rows
 * (a table with a byte that is not 2 mod 4 - the E8P table has none - is noticed inside
 * the launch and served by the scalar decode); anything else takes the scalar kernel, one wave
 * per output row. */
int dmm_decode_matmul_i8(const void *x, const void *codes, const void *codebook_abs, void *out,
                         int64_t M, int64_t N, int64_t K, int tiled, void *stream);

/* Which kernel dmm_decode_matmul_i8 takes for this shape when x, codes and out are 16-byte
 * aligned: "dmm::int8g_kernel" (matrix-matrix, many rows of x), "dmm::int8x_kernel"
 * (matrix-vector, 16 rows of x per pass), "dmm::int8d_kernel" (matrix-vector, up to 32 rows of x
 * with two to eight 16-row tiles of W per compute unit, every tile's sums in registers) or
 * "dmm::int8_kernel" (scalar).  For tests and
 * benchmarks; no counterpart in the reference. */
const char *dmm_integer_kernel_name(int64_t M, int64_t N, int64_t K);

/* For benchmarks that check the operator's choices against the alternatives, as launches of one
 * HIP graph: forces a kernel where the library would choose, process-wide, for calls made after it
 * returns.  which = 0: the half-precision operator on more than 16 rows of x (value 0: passes of the
 * small-batch kernel, 16 rows each; 1: the matrix-matrix kernel; 2: split K, where a workspace is
 * given - dmm_workspace_bytes then answers for the split as well).  which = 1: the integer
 * operator on more than 16 rows (1: passes of the matrix-vector kernel, 2: the matrix-matrix
 * kernel).  which = 2: up to 32 rows of x (0: never the 16-bit kernel that keeps every tile's
 * sums in registers, 1: wherever it can run).  which = 3: the same for the integer operator's kernel
 * of that kind (up to 32 rows).  value -1: the library's own choice (the default).  A forced
 * kernel that cannot take a call (shape, alignment) leaves that call to the library's choice;
 * results do not depend on the setting beyond what the kernels' own summation orders differ by
 * (the integer operator: not at all).  Returns the previous value (>= -1), or DMM_ERR_BAD_SHAPE for arguments out of
 * range.  No counterpart in the reference. */
int dmm_set_choice(int which, int value);

/* Kernel timing hook for benchmarks.  While a (start, stop) pair of hipEvent_t handles is
 * set on the calling thread, the dominant kernel of each operator call records `start`
 * immediately before and `stop` immediately after itself on the GPU timeline, so
 * hipEventElapsedTime(start, stop) is that kernel's own duration, as a profiler's kernel
 * trace reports it.  Pass NULL, NULL to clear.  No counterpart in the reference, whose
 * only timer (/root/reference/test_decode_matmul.py:8-22) brackets the whole call. */
int dmm_set_kernel_events(void *start_event, void *stop_event);

/* The operator and the decoder on HOST memory (every pointer a host pointer): the counterpart of the
 * reference's CPU path, its scalar `decode` and its triple-loop matmul
 * (/root/reference/test_decode_matmul.py:29-71), in the half-precision form.  Plain C++ on the host's
 * cores, no GPU call; for hosts without a GPU and for checking small cases.  These are separate
 * entry points, not a fallback: the device entry points never come here, and a device pointer
 * passed here is dereferenced as host memory.  Same code format, same one rounding per weight,
 * fp32 sums over k in ascending order, y = half(scale * sum); blocking (returns when y is written). */
int dmm_decode_host_f16(const void *codes, const void *grid, void *W, int64_t N, int64_t K);
int dmm_decode_matmul_host_f16(const void *x, const void *codes, const void *grid, float scale,
                               void *y, int64_t M, int64_t N, int64_t K);

/* Yardstick for benchmarks: a kernel that only READS a row-major code matrix [N, K/8] with the
 * batch-1 kernels' launch shape and access pattern (16 rows x 64 bytes per wave load) and does no
 * decoding; timed with dmm_set_kernel_events like any other call, it shows what the memory system
 * gives a launch of this size.  `sink`: 4 bytes of device memory that the kernel never writes in
 * practice.  K % 256 == 0, 16-byte aligned codes, N * K / 4 below 2 GiB (DMM_ERR_UNSUPPORTED
 * otherwise).  No counterpart in the reference. */
int dmm_read_probe(const void *codes, void *sink, int64_t N, int64_t K, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DMM_H */
