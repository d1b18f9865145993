// C ABI: prefill matmul Y[n x rows] (+)= X[n x cols] . W^T over raw GGUF block rows (see include/msq.h; reference
// host code src/kernels/quant.mm:159-248, kernels src/kernels/quant_mm.metal:81-185).
//
// The reference multiplies fp16 activations by weight tiles dequantized to fp16 and, from n >= 512, dequantizes the
// whole matrix to fp16 once and runs a dense GEMM (quant.mm:204-221). Here the second route serves every n: with
// 8 TB/s of HBM the fp16 copy of an attention projection (7168 x 1536: 22 MB) is written and read back in a few
// microseconds, after which the product is a plain fp16 x fp16 -> fp32 GEMM, which is left to rocBLAS (MFMA kernels
// tuned per shape). The fp16 copies of X and W live in scratch the library owns and grows on demand; like the
// reference's (docs/modules/quant.md:265-268) it is shared by all calls, so calls must be enqueued on one stream at a
// time, and a call that has to grow it synchronises that stream and allocates (never inside a stream capture).
#include <rocblas/rocblas.h>

#include <mutex>

#include "msq_deq.cuh"
#include "msq_host.h"

namespace msq {
namespace {

__global__ __launch_bounds__(256) void f32_to_f16_kernel(const float4* __restrict__ src, uint2* __restrict__ dst, size_t n4) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n4) return;
  const float4 v = src[i];
  dst[i] = uint2{pack_h2(v.x, v.y), pack_h2(v.z, v.w)};
}

struct Scratch {
  void* p = nullptr;
  size_t bytes = 0;
};
std::mutex g_mu;
Scratch g_x16, g_w16;
rocblas_handle g_blas = nullptr;

// at least `bytes` of device memory in s (>= 64 MiB like the reference's, quant.mm:176-183); growing waits for the
// stream first, since enqueued work may still use the old allocation
int reserve(Scratch& s, size_t bytes, hipStream_t st) {
  if (s.bytes >= bytes) return MSQ_OK;
  MSQ_HIP(hipStreamSynchronize(st));
  if (s.p) MSQ_HIP(hipFree(s.p));
  s.p = nullptr;
  s.bytes = 0;
  const size_t want = std::max(bytes, (size_t)64 << 20);
  MSQ_HIP(hipMalloc(&s.p, want));
  s.bytes = want;
  return MSQ_OK;
}

int launch_f32_to_f16(hipStream_t st, const float* X, uint16_t* X16, size_t count) {
  const size_t n4 = count / 4;
  if (n4 == 0) return MSQ_OK;
  hipLaunchKernelGGL(f32_to_f16_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, st, (const float4*)X, (uint2*)X16, n4);
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

int launch_deq_f16(hipStream_t st, int t, const uint8_t* W, uint16_t* out, int64_t n_elems) {
  const int64_t nchunks = n_elems / 8;
  const dim3 grid((unsigned)((nchunks + 255) / 256)), block(256);
  switch (t) {
#define MSQ_DEQH(T) case T: hipLaunchKernelGGL((dequant_kernel<T, uint16_t>), grid, block, 0, st, W, out, nchunks); break;
    MSQ_DEQH(MSQ_F32) MSQ_DEQH(MSQ_BF16) MSQ_DEQH(MSQ_Q8_0) MSQ_DEQH(MSQ_IQ4_NL) MSQ_DEQH(MSQ_IQ1_S) MSQ_DEQH(MSQ_IQ2_XXS)
    MSQ_DEQH(MSQ_Q6_K) MSQ_DEQH(MSQ_Q5_K)
#undef MSQ_DEQH
    default: return MSQ_ERR_UNSUPPORTED;
  }
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

bool mm_type_ok(int t) {
  switch (t) {
    case MSQ_F32: case MSQ_F16: case MSQ_BF16: case MSQ_Q8_0: case MSQ_Q5_K: case MSQ_Q6_K: case MSQ_IQ1_S: case MSQ_IQ2_XXS:
    case MSQ_IQ4_NL: return true;
    default: return false;
  }
}

// Y[n][rows] (+)= X16[n][x_stride] . W16[rows][cols]^T. In rocBLAS' column-major terms: C (rows x n, ld rows) =
// op(A) B with A = W16 seen as cols x rows (ld cols), transposed, and B = X16 seen as cols x n (ld x_stride).
int gemm_f16(hipStream_t st, const uint16_t* W16, const uint16_t* X16, float* Y, int n, int rows, int cols, int x_stride,
             bool accumulate) {
  if (!g_blas) {
    if (rocblas_create_handle(&g_blas) != rocblas_status_success) {
      g_blas = nullptr;
      return fail(MSQ_ERR_HIP, "macseek quant: matmul: rocblas_create_handle failed");
    }
    rocblas_set_pointer_mode(g_blas, rocblas_pointer_mode_host);
  }
  if (rocblas_set_stream(g_blas, st) != rocblas_status_success) return fail(MSQ_ERR_HIP, "macseek quant: matmul: rocblas_set_stream failed");
  const float alpha = 1.f, beta = accumulate ? 1.f : 0.f;
  const rocblas_status rs = rocblas_gemm_ex(g_blas, rocblas_operation_transpose, rocblas_operation_none, rows, n, cols, &alpha, W16,
                                            rocblas_datatype_f16_r, cols, X16, rocblas_datatype_f16_r, x_stride, &beta, Y,
                                            rocblas_datatype_f32_r, rows, Y, rocblas_datatype_f32_r, rows, rocblas_datatype_f32_r,
                                            rocblas_gemm_algo_standard, 0, 0);
  if (rs != rocblas_status_success) return fail(MSQ_ERR_HIP, "macseek quant: matmul: rocblas_gemm_ex failed (%d)", (int)rs);
  return MSQ_OK;
}

int matmul_h(hipStream_t st, int t, const MsqBuffer* W, int rows, int cols, const uint16_t* X16, float* Y, int n, bool accumulate,
             int x_stride) {
  const uint16_t* w16 = (const uint16_t*)bptr(W);
  if (t != MSQ_F16) {  // F16 weights are the GEMM operand as they are
    const int rc = reserve(g_w16, (size_t)rows * cols * 2, st);
    if (rc != MSQ_OK) return rc;
    const int rd = launch_deq_f16(st, t, bptr(W), (uint16_t*)g_w16.p, (int64_t)rows * cols);
    if (rd != MSQ_OK) return rd;
    w16 = (const uint16_t*)g_w16.p;
  }
  return gemm_f16(st, w16, X16, Y, n, rows, cols, x_stride, accumulate);
}

}  // namespace
}  // namespace msq

using namespace msq;

extern "C" {

int msq_f32_to_f16(void* stream, const MsqBuffer* X, const MsqBuffer* X16, size_t count) {
  if (count % 4) return fail(MSQ_ERR_UNSUPPORTED, "macseek quant: f32_to_f16 unsupported (count %zu not a multiple of 4)", count);
  if (count == 0) return MSQ_OK;
  if (!buf_ok(X, count * 4) || !buf_ok(X16, count * 2) || ((uintptr_t)bptr(X) & 15) || ((uintptr_t)bptr(X16) & 7))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: f32_to_f16: buffer missing, too small or misaligned");
  return launch_f32_to_f16((hipStream_t)stream, (const float*)bptr(X), (uint16_t*)bptr_mut(X16), count);
}

int msq_matmul_h(void* stream, int t, const MsqBuffer* W, int rows, int cols, const MsqBuffer* X16, const MsqBuffer* Y, int n,
                 int accumulate, int x_stride) {
  if (!mm_type_ok(t) || rows < 1 || cols < 1 || cols % 128 || n < 1 || (x_stride && x_stride < cols)) return unsupported("matmul", t, rows, cols);
  const int xs = x_stride ? x_stride : cols;
  if (!buf_ok(W, msq_type_row_bytes(t, cols) * (size_t)rows) || !buf_ok(X16, ((size_t)(n - 1) * xs + cols) * 2) ||
      !buf_ok(Y, (size_t)n * rows * 4) || ((uintptr_t)bptr(X16) & 1) || ((uintptr_t)bptr(Y) & 3))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: matmul: buffer missing, too small or misaligned (type %s rows %d cols %d n %d)",
                msq_type_name_of(t), rows, cols, n);
  std::lock_guard<std::mutex> lock(g_mu);
  return matmul_h((hipStream_t)stream, t, W, rows, cols, (const uint16_t*)bptr(X16), (float*)bptr_mut(Y), n, accumulate != 0, xs);
}

int msq_matmul(void* stream, int t, const MsqBuffer* W, int rows, int cols, const MsqBuffer* X, const MsqBuffer* Y, int n,
               int accumulate) {
  if (!mm_type_ok(t) || rows < 1 || cols < 1 || cols % 128 || n < 1) return unsupported("matmul", t, rows, cols);
  if (!buf_ok(W, msq_type_row_bytes(t, cols) * (size_t)rows) || !buf_ok(X, (size_t)n * cols * 4) || !buf_ok(Y, (size_t)n * rows * 4) ||
      ((uintptr_t)bptr(X) & 15) || ((uintptr_t)bptr(Y) & 3))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: matmul: buffer missing, too small or misaligned (type %s rows %d cols %d n %d)",
                msq_type_name_of(t), rows, cols, n);
  hipStream_t st = (hipStream_t)stream;
  std::lock_guard<std::mutex> lock(g_mu);
  const int rc = reserve(g_x16, (size_t)n * cols * 2, st);
  if (rc != MSQ_OK) return rc;
  const int rx = launch_f32_to_f16(st, (const float*)bptr(X), (uint16_t*)g_x16.p, (size_t)n * cols);
  if (rx != MSQ_OK) return rx;
  return matmul_h(st, t, W, rows, cols, (const uint16_t*)g_x16.p, (float*)bptr_mut(Y), n, accumulate != 0, cols);
}

}  // extern "C"
