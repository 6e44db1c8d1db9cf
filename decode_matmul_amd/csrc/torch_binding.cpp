// PyTorch-ROCm operator over the C ABI of libdmm.so.  Host code only: no device code is
// compiled here, the kernels live in dmm.hip and the dmm_*.h files it includes, behind include/dmm.h.
//
// Mirrors the operator boundary of the reference,
// /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:178-239: one module, a function
// `decode_matmul`, inputs checked with TORCH_CHECK (-> Python RuntimeError), output
// allocated by the op on x's device, launch on the current stream under a DeviceGuard.
// Differences, all deliberate: half precision with a scale (x half, codes 16-bit, grid half
// [256,8], scale float -> half); no shape demands beyond K % 8 == 0; no device
// synchronisation and no exit() on error (a non-zero status becomes an exception); the
// GIL is released around the launch.
#include <torch/extension.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include "dmm.h"

namespace {

#define DMM_CHECK_DEVICE(t) TORCH_CHECK((t).is_cuda(), #t " must be a GPU tensor")
#define DMM_CHECK_CONTIGUOUS(t) TORCH_CHECK((t).is_contiguous(), #t " must be contiguous")
#define DMM_CHECK_INPUT(t)       \
    do {                         \
        DMM_CHECK_DEVICE(t);     \
        DMM_CHECK_CONTIGUOUS(t); \
    } while (false)

bool is_code_dtype(const torch::Tensor &t)
{
    return t.scalar_type() == torch::kInt16 || t.scalar_type() == torch::kUInt16;
}

void check_status(int st, const char *what)
{
    TORCH_CHECK(st == DMM_OK, what, " failed: ", dmm_status_string(st), " (status ", st, ")");
}

// allow_cpu: the operator and the decoder also take tensors in host memory (all of them there), which
// go to the library's host route; every other operation is GPU-only
void check_codes_grid(const torch::Tensor &codes, const torch::Tensor &grid, bool allow_cpu = false)
{
    if (allow_cpu && codes.is_cpu()) {
        DMM_CHECK_CONTIGUOUS(codes);
        DMM_CHECK_CONTIGUOUS(grid);
    } else {
        DMM_CHECK_INPUT(codes);
        DMM_CHECK_INPUT(grid);
    }
    TORCH_CHECK(is_code_dtype(codes), "codes must be int16 or uint16");
    TORCH_CHECK(grid.scalar_type() == torch::kHalf, "grid must be float16");
    TORCH_CHECK(codes.dim() == 2, "codes must be [N, K/8]");
    TORCH_CHECK(grid.dim() == 2 && grid.size(0) == 256 && grid.size(1) == 8, "grid must be [256, 8]");
    TORCH_CHECK(codes.device() == grid.device(), "codes and grid must be on the same device");
}

enum class Path { kAuto, kGemv, kGemm, kGeneric };

torch::Tensor run(const torch::Tensor &x, const torch::Tensor &codes, const torch::Tensor &grid,
                  double scale, Path path)
{
    if (x.is_cpu()) {
        DMM_CHECK_CONTIGUOUS(x);
    } else {
        DMM_CHECK_INPUT(x);
    }
    check_codes_grid(codes, grid, true);
    TORCH_CHECK(x.scalar_type() == torch::kHalf, "x must be float16");
    TORCH_CHECK(x.dim() == 2, "x must be [M, K]");
    TORCH_CHECK(x.device() == codes.device(), "x and codes must be on the same device");
    TORCH_CHECK(x.size(-1) == codes.size(-1) * 8, "x.size(-1) must be 8 * codes.size(-1)");

    const int64_t M = x.size(-2);
    const int64_t N = codes.size(-2);
    const int64_t K = x.size(-1);

    if (x.is_cpu()) {
        // tensors in host memory: the library's host route (the reference's CPU path,
        // test_decode_matmul.py:58-71, in the half-precision form); no GPU call is made
        TORCH_CHECK(path == Path::kAuto, "the named kernel paths are GPU paths; CPU tensors take path 'auto'");
        torch::Tensor y = torch::empty({M, N}, x.options().requires_grad(false));
        int st;
        {
            pybind11::gil_scoped_release nogil;
            st = dmm_decode_matmul_host_f16(x.data_ptr(), codes.data_ptr(), grid.data_ptr(), static_cast<float>(scale),
                                            y.data_ptr(), M, N, K);
        }
        check_status(st, "decode_matmul (host)");
        return y;
    }

    c10::DeviceGuard guard(x.device());
    torch::Tensor y = torch::empty({M, N}, x.options().requires_grad(false));
    hipStream_t stream = c10::hip::getCurrentHIPStream(x.device().index()).stream();
    // split-K workspace for short x, from torch's caching allocator: stream-ordered, so calls
    // on different streams never share one
    torch::Tensor workspace;
    const int64_t ws_bytes = path == Path::kAuto ? dmm_workspace_bytes(M, N, K) : 0;
    if (ws_bytes > 0) workspace = torch::empty({ws_bytes}, x.options().dtype(torch::kUInt8).requires_grad(false));

    int st;
    {
        pybind11::gil_scoped_release nogil;
        const void *xp = x.data_ptr(), *cp = codes.data_ptr(), *gp = grid.data_ptr();
        void *yp = y.data_ptr();
        const float sc = static_cast<float>(scale);
        switch (path) {
            case Path::kGemv: st = dmm_gemv_f16(xp, cp, gp, sc, yp, M, N, K, stream); break;
            case Path::kGemm: st = dmm_gemm_f16(xp, cp, gp, sc, yp, M, N, K, stream); break;
            case Path::kGeneric: st = dmm_generic_f16(xp, cp, gp, sc, yp, M, N, K, stream); break;
            default:
                st = dmm_decode_matmul_ws_f16(xp, cp, gp, sc, yp, M, N, K, ws_bytes > 0 ? workspace.data_ptr() : nullptr,
                                              ws_bytes, stream);
                break;
        }
    }
    check_status(st, "decode_matmul");
    return y;
}

torch::Tensor decode_matmul(torch::Tensor x, torch::Tensor codes, torch::Tensor grid, double scale)
{
    return run(x, codes, grid, scale, Path::kAuto);
}

torch::Tensor decode_matmul_path(torch::Tensor x, torch::Tensor codes, torch::Tensor grid, double scale,
                                 const std::string &path)
{
    Path p;
    if (path == "auto") p = Path::kAuto;
    else if (path == "gemv") p = Path::kGemv;
    else if (path == "gemm") p = Path::kGemm;
    else if (path == "generic") p = Path::kGeneric;
    else TORCH_CHECK(false, "unknown path '", path, "' (auto, gemv, gemm, generic)");
    return run(x, codes, grid, scale, p);
}

torch::Tensor decode(torch::Tensor codes, torch::Tensor grid)
{
    check_codes_grid(codes, grid, true);
    const int64_t N = codes.size(0);
    const int64_t K = codes.size(1) * 8;
    if (codes.is_cpu()) {   // host memory: the library's host decoder, no GPU call
        torch::Tensor W = torch::empty({N, K}, grid.options().requires_grad(false));
        int st;
        {
            pybind11::gil_scoped_release nogil;
            st = dmm_decode_host_f16(codes.data_ptr(), grid.data_ptr(), W.data_ptr(), N, K);
        }
        check_status(st, "decode (host)");
        return W;
    }
    c10::DeviceGuard guard(codes.device());
    torch::Tensor W = torch::empty({N, K}, grid.options().requires_grad(false));
    hipStream_t stream = c10::hip::getCurrentHIPStream(codes.device().index()).stream();
    int st;
    {
        pybind11::gil_scoped_release nogil;
        st = dmm_decode_f16(codes.data_ptr(), grid.data_ptr(), W.data_ptr(), N, K, stream);
    }
    check_status(st, "decode");
    return W;
}

// Offline repack for the batch-1 kernel: codes [N, K/8] -> packed [ceil(N/16)*16, K/8] (same
// dtype; rows past N are zero padding), and the operator on packed codes.
torch::Tensor pack_codes(torch::Tensor codes)
{
    DMM_CHECK_INPUT(codes);
    TORCH_CHECK(is_code_dtype(codes) && codes.dim() == 2, "codes must be int16 or uint16 [N, K/8]");
    const int64_t N = codes.size(0), K = codes.size(1) * 8;
    TORCH_CHECK(K >= 256 && K % 256 == 0, "packing needs K % 256 == 0");
    c10::DeviceGuard guard(codes.device());
    torch::Tensor packed = torch::empty({(N + 15) / 16 * 16, K / 8}, codes.options().requires_grad(false));
    hipStream_t stream = c10::hip::getCurrentHIPStream(codes.device().index()).stream();
    int st;
    {
        pybind11::gil_scoped_release nogil;
        st = dmm_pack_codes(codes.data_ptr(), packed.data_ptr(), N, K, stream);
    }
    check_status(st, "pack_codes");
    return packed;
}

torch::Tensor decode_matmul_packed(torch::Tensor x, torch::Tensor packed, torch::Tensor grid, double scale, int64_t N)
{
    DMM_CHECK_INPUT(x);
    check_codes_grid(packed, grid);
    TORCH_CHECK(x.scalar_type() == torch::kHalf && x.dim() == 2, "x must be float16 [M, K]");
    TORCH_CHECK(x.device() == packed.device(), "x and packed must be on the same device");
    TORCH_CHECK(x.size(-1) == packed.size(-1) * 8, "x.size(-1) must be 8 * packed.size(-1)");
    TORCH_CHECK(N >= 0 && packed.size(0) == (N + 15) / 16 * 16, "packed must have ceil(N / 16) * 16 rows");
    const int64_t M = x.size(0), K = x.size(1);
    c10::DeviceGuard guard(x.device());
    torch::Tensor y = torch::empty({M, N}, x.options().requires_grad(false));
    hipStream_t stream = c10::hip::getCurrentHIPStream(x.device().index()).stream();
    torch::Tensor workspace;
    const int64_t ws_bytes = dmm_workspace_bytes(M, N, K);
    if (ws_bytes > 0) workspace = torch::empty({ws_bytes}, x.options().dtype(torch::kUInt8).requires_grad(false));
    int st;
    {
        pybind11::gil_scoped_release nogil;
        st = dmm_decode_matmul_packed_f16(x.data_ptr(), packed.data_ptr(), grid.data_ptr(), static_cast<float>(scale),
                                          y.data_ptr(), M, N, K, ws_bytes > 0 ? workspace.data_ptr() : nullptr,
                                          ws_bytes, stream);
    }
    check_status(st, "decode_matmul_packed");
    return y;
}

// The reference's own signature: int8 x, int16 codes (tiled like its kernel reads them, or
// row-major), int64[256] table -> int32 (decode_matmul_cuda.cu:178-234).
torch::Tensor decode_matmul_int8(torch::Tensor x, torch::Tensor weights_compressed, torch::Tensor codebook_abs,
                                 bool tiled)
{
    DMM_CHECK_INPUT(x);
    DMM_CHECK_INPUT(weights_compressed);
    DMM_CHECK_INPUT(codebook_abs);
    TORCH_CHECK(x.scalar_type() == torch::kInt8, "x must be int8");
    TORCH_CHECK(is_code_dtype(weights_compressed), "weights_compressed must be int16 or uint16");
    TORCH_CHECK(codebook_abs.scalar_type() == torch::kInt64 && codebook_abs.numel() == 256,
                "codebook_abs must be int64[256]");
    TORCH_CHECK(x.dim() == 2 && weights_compressed.dim() == 2, "x must be [M, K], weights_compressed [N, K/8]");
    TORCH_CHECK(x.size(-1) == weights_compressed.size(-1) << 3, "x.size(-1) must be 8 * weights_compressed.size(-1)");
    TORCH_CHECK(x.device() == weights_compressed.device() && x.device() == codebook_abs.device(),
                "all tensors must be on the same device");
    const int64_t M = x.size(-2), N = weights_compressed.size(-2), K = x.size(-1);
    c10::DeviceGuard guard(x.device());
    torch::Tensor out = torch::empty({M, N}, x.options().dtype(torch::kInt32).requires_grad(false));
    hipStream_t stream = c10::hip::getCurrentHIPStream(x.device().index()).stream();
    int st;
    {
        pybind11::gil_scoped_release nogil;
        st = dmm_decode_matmul_i8(x.data_ptr(), weights_compressed.data_ptr(), codebook_abs.data_ptr(),
                                  out.data_ptr(), M, N, K, tiled ? 1 : 0, stream);
    }
    check_status(st, "decode_matmul_int8");
    return out;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("decode_matmul", &decode_matmul, "Fused decode + matrix multiplication (half precision)",
          pybind11::arg("x"), pybind11::arg("codes"), pybind11::arg("grid"), pybind11::arg("scale"));
    m.def("decode_matmul_path", &decode_matmul_path, "decode_matmul through one named kernel path",
          pybind11::arg("x"), pybind11::arg("codes"), pybind11::arg("grid"), pybind11::arg("scale"),
          pybind11::arg("path"));
    m.def("decode_matmul_int8", &decode_matmul_int8,
          "The reference's integer operator: int8 x, int16 codes, int64[256] table -> int32",
          pybind11::arg("x"), pybind11::arg("weights_compressed"), pybind11::arg("codebook_abs"),
          pybind11::arg("tiled") = true);
    m.def("pack_codes", &pack_codes, "codes [N, K/8] -> the batch-1 kernel's packed layout", pybind11::arg("codes"));
    m.def("decode_matmul_packed", &decode_matmul_packed, "decode_matmul on packed codes (K % 256 == 0)",
          pybind11::arg("x"), pybind11::arg("packed"), pybind11::arg("grid"), pybind11::arg("scale"), pybind11::arg("N"));
    m.def("decode", &decode, "Decode codes [N, K/8] to the dense half matrix [N, K]",
          pybind11::arg("codes"), pybind11::arg("grid"));
}
