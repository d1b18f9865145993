// C ABI: prefill matmul Y[n x rows] (+)= X[n x cols] . W^T over raw GGUF block rows (see include/msq.h; reference
// host code src/kernels/quant.mm:159-248, kernels src/kernels/quant_mm.metal:81-185).
//
// The reference multiplies fp16 activations by weight tiles dequantized to fp16 inside its GEMM kernel and, from
// n >= 512, dequantizes the whole matrix to fp16 once and runs a dense GEMM (quant.mm:204-221). The same two routes
// exist here; the switch between them sits where they were measured to cross (use_fused, tile_ok below). Fused route:
// mm_fused_kernel (msq_mm.cuh) decodes each weight tile straight into matrix-core fragments -- no fp16 copy of W or X,
// nothing allocated, the call only enqueues; for large matrices of four formats at 65 to 256 tokens mm_tile_kernel
// does the same with both operands staged through LDS (F32 activations are first rounded to fp16 rows in a
// file-scope device buffer, which calls share like the partial sums); when the tiles alone would not fill the device K is cut into slices whose
// partial sums go to a file-scope device buffer and are added in order by a second launch (no floating-point atomics:
// results repeat bit for bit; calls on this route share the buffer and must be enqueued on one stream at a time).
// Materialising route: the bit-exact dequantizer writes
// W as fp16 into library-owned scratch (22 MB for a 7168 x 1536 projection, a few microseconds at 8 TB/s) and the
// product is a plain fp16 x fp16 -> fp32 GEMM left to rocBLAS. That scratch only grows: a larger request allocates a
// new block and the old one stays alive until the process ends (work already enqueued may still read it), so growing
// never waits for the stream; it does allocate, so the first call of a larger shape must not be inside a stream
// capture, and like the reference's scratch (docs/modules/quant.md:265-268) it is shared by all calls: calls on this
// route must be enqueued on one stream at a time.
#include <rocblas/rocblas.h>

#include <cstdlib>
#include <mutex>
#include <vector>

#include "msq_deq.cuh"
#include "msq_host.h"
#include "msq_mm.cuh"

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
std::vector<void*> g_retired;  // outgrown blocks: kept until the process ends
rocblas_handle g_blas = nullptr;
// Which calls the fused kernel serves. The reference switches to dequantize-then-GEMM at 512 tokens (quant.mm:204); here
// the switch sits where the two routes were measured to cross on MI355X: the fused kernel wins up to 128 tokens on every
// matrix tried (Q6_K 1536x7168 at 128 tokens: 22.5 us against 36 us; 16 tokens: 11 against 30) and up to 256 tokens on
// matrices of at most 2048 rows and on every Q6_K / Q5_K matrix (4096x4096 at 192 tokens: 32 us against 44); above, the
// materialising route is ahead (IQ4_NL 7168x4096 at 512 tokens: 63 us against 124). MSQ_MM_FUSED_MAX = N makes the
// switch "up to N tokens" for every matrix (0: never fused).
int fused_forced() {
  static const int forced = [] { const char* e = getenv("MSQ_MM_FUSED_MAX"); return e && *e ? atoi(e) : -1; }();
  return forced;
}
bool use_fused(int t, int n, int rows) {
  const int forced = fused_forced();
  if (forced >= 0) return n <= forced;
  return n <= 128 || (n <= 256 && (rows <= 2048 || t == MSQ_Q6_K || t == MSQ_Q5_K));
}

// at least `bytes` of device memory in s (>= 64 MiB like the reference's, quant.mm:176-183)
int reserve(Scratch& s, size_t bytes, hipStream_t st) {
  if (s.bytes >= bytes) return MSQ_OK;
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
    return fail(MSQ_ERR_SCRATCH, "macseek quant: matmul: the fp16 scratch has to grow, which cannot happen inside a stream capture "
                                 "(run the shape once before capturing)");
  void* p = nullptr;
  const size_t want = std::max(bytes, (size_t)64 << 20);
  MSQ_HIP(hipMalloc(&p, want));
  if (s.p) g_retired.push_back(s.p);
  s.p = p;
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

// Partial sums of the fused kernel's K slices: a file-scope device array, so the fused route allocates nothing and can
// be captured. Every GPU holds its own copy; its address is looked up once per device (hipGetSymbolAddress) by
// msq_init() or the first call. Calls of the fused route share it: like the reference's module scratch
// (docs/modules/quant.md:265-268) they must be enqueued on one stream at a time.
constexpr size_t kMmPartialBytes = (size_t)32 << 20;
__device__ __align__(256) float g_mm_partials[kMmPartialBytes / 4];
float* g_mm_partials_ptr[16] = {};
float* mm_partials() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
  std::lock_guard<std::mutex> lock(g_mu);
  if (!g_mm_partials_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_mm_partials)) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    g_mm_partials_ptr[dev] = (float*)p;
  }
  return g_mm_partials_ptr[dev];
}

// K slices per tile at most: MSQ_MM_SPLITK (experiments; 1 keeps every sum inside one workgroup), 0 / unset lets the
// launcher choose
int splitk_limit() {
  static const int v = [] { const char* e = getenv("MSQ_MM_SPLITK"); return e && *e ? atoi(e) : 0; }();
  return v;
}

// token counts that take the tile kernel (MSQ_MM_TILE_MIN / MSQ_MM_TILE_MAX: experiments; a huge minimum switches it off)
long tile_min_tokens() {
  static const long v = [] { const char* e = getenv("MSQ_MM_TILE_MIN"); return e && *e ? atol(e) : 65L; }();
  return v;
}
long tile_max_tokens() {
  static const long v = [] { const char* e = getenv("MSQ_MM_TILE_MAX"); return e && *e ? atol(e) : 256L; }();
  return v;
}

template <class F, bool X_F32>
int launch_mm_t(hipStream_t st, MmArgs a) {
  const long cus = device_info().cus;
  const uint32_t nstages = a.cols / kMmKStage;
  auto go = [&](auto wv_tag, auto tm_tag) -> int {
    constexpr int WV = decltype(wv_tag)::value, TM = decltype(tm_tag)::value;
    const size_t lds = (size_t)F::LDS_WORDS * 4 + 2 * (size_t)16 * TM * kMmPitch;
    const int rc = allow_large_lds(mm_fused_kernel<F, WV, TM, X_F32>, lds);
    if (rc != MSQ_OK) return rc;
    const long gx = (a.rows + 16 * WV - 1) / (16 * WV), gy = (a.n + 16 * TM - 1) / (16 * TM);
    // Few tiles: the K range is cut into slices (at least two stages each) until there are about two workgroups per CU;
    // a workgroup's K loop is a chain of stage latencies, so a call is as slow as its longest chain. The slices of a tile
    // leave their sums in the partial buffer (as many slices as it holds) and a second launch adds them in order.
    const size_t cnt = (size_t)a.n * a.rows;
    long kz = std::min<long>((2 * cus + gx * gy - 1) / (gx * gy), std::max<long>(1, nstages / 2));
    kz = std::min<long>(kz, (long)(kMmPartialBytes / (cnt * 4)));
    if (splitk_limit() > 0) kz = std::min<long>(kz, splitk_limit());
    float* partials = kz > 1 ? mm_partials() : nullptr;
    if (!partials) kz = 1;
    a.slice_stages = (uint32_t)((nstages + kz - 1) / kz);
    kz = (nstages + a.slice_stages - 1) / a.slice_stages;
    a.partials = kz > 1 ? partials : nullptr;
    hipLaunchKernelGGL((mm_fused_kernel<F, WV, TM, X_F32>), dim3((unsigned)gx, (unsigned)gy, (unsigned)kz), dim3(64 * WV), lds, st, a.X, a.W, a.Y,
                       a.n, a.rows, a.cols, a.x_stride, a.row_bytes, a.accumulate, a.slice_stages, a.partials);
    if (a.partials)
      hipLaunchKernelGGL(mm_reduce_kernel, dim3((unsigned)((cnt + 255) / 256)), dim3(256), 0, st, (const float*)a.partials, a.Y, cnt,
                         (uint32_t)kz, a.accumulate);
    MSQ_HIP(hipGetLastError());
    return MSQ_OK;
  };
  // token tiles per workgroup: what the call's tokens need, at most eight; eight waves when that still leaves a
  // workgroup per CU, four otherwise
  auto wgs = [&](long wv, long tm) { return ((a.rows + 16 * wv - 1) / (16 * wv)) * ((a.n + 16 * tm - 1) / (16 * tm)); };
  using I1 = std::integral_constant<int, 1>; using I2 = std::integral_constant<int, 2>;
  using I4 = std::integral_constant<int, 4>; using I8 = std::integral_constant<int, 8>;
  if (a.n > 64) return wgs(8, 8) >= cus ? go(I8{}, I8{}) : go(I4{}, I8{});
  if (a.n > 32) return go(I4{}, I4{});
  if (a.n > 16) return go(I4{}, I2{});
  return go(I4{}, I1{});
}
template <bool X_F32>
int launch_mm(hipStream_t st, int t, const MmArgs& a) {
  switch (t) {
    case MSQ_F32: return launch_mm_t<FragF32H, X_F32>(st, a);
    case MSQ_F16: return launch_mm_t<FragDense16<MSQ_F16>, X_F32>(st, a);
    case MSQ_BF16: return launch_mm_t<FragBF16H, X_F32>(st, a);
    case MSQ_Q8_0: return launch_mm_t<FragQ8_0, X_F32>(st, a);
    case MSQ_Q5_K: return launch_mm_t<FragQ5K, X_F32>(st, a);
    case MSQ_Q6_K: return launch_mm_t<FragQ6K, X_F32>(st, a);
    case MSQ_IQ4_NL: return launch_mm_t<FragIQ4NL, X_F32>(st, a);
    case MSQ_IQ1_S: return launch_mm_t<FragIQ1S, X_F32>(st, a);
    case MSQ_IQ2_XXS: return launch_mm_t<FragIQ2XXS, X_F32>(st, a);
  }
  return unsupported("matmul", t, (int)a.rows, (int)a.cols);
}

// The tile kernel (fp16 activations in memory): eight waves of one row tile each, 128 rows x 128 or 256 tokens per
// workgroup (256 when the call has the tokens: a decoded fragment then feeds sixteen matrix instructions), one
// workgroup per CU, K cut into slices of whole weight stages until every CU has one.
template <class F, int TM, int XK>
int launch_tile_c(hipStream_t st, MmArgs a) {
  constexpr int WV = 8, RT = 1;
  constexpr int P = ((F::WS_BYTES + 14 + 15) / 16) | 1, NPI = (16 * WV * RT * P + 64 * WV - 1) / (64 * WV);
  const long cus = device_info().cus;
  const uint32_t nstages = a.cols / XK, xpw = 256 / XK;
  const size_t lds = (size_t)F::LDS_WORDS * 4 + 2 * (size_t)16 * TM * XK * 2 + 2 * (size_t)NPI * 64 * WV * 16 +
                     (NPI * 64 * WV > 16 * WV * RT * P ? 0 : 16);  // (a fragment read may end a few bytes past its row's pieces)
  const int rc = allow_large_lds(mm_tile_kernel<F, WV, RT, TM, XK>, lds);
  if (rc != MSQ_OK) return rc;
  const long gx = (a.rows + 16 * WV * RT - 1) / (16 * WV * RT), gy = (a.n + 16 * TM - 1) / (16 * TM);
  const size_t cnt = (size_t)a.n * a.rows;
  const long wstages = (nstages + xpw - 1) / xpw;  // weight stages (256 columns) of a row
  long kz = std::min<long>(std::max<long>(1, cus / (gx * gy)), std::max<long>(1, wstages / 2));
  kz = std::min<long>(kz, std::max<long>(1, (long)(kMmPartialBytes / (cnt * 4))));
  if (splitk_limit() > 0) kz = std::min<long>(kz, splitk_limit());
  float* partials = kz > 1 ? mm_partials() : nullptr;
  if (!partials) kz = 1;
  const long per = (wstages + kz - 1) / kz;
  a.slice_stages = (uint32_t)(per * xpw);
  kz = (wstages + per - 1) / per;
  a.partials = kz > 1 ? partials : nullptr;
  hipLaunchKernelGGL((mm_tile_kernel<F, WV, RT, TM, XK>), dim3((unsigned)gx, (unsigned)gy, (unsigned)kz), dim3(64 * WV), lds, st, a.X, a.W, a.Y,
                     a.n, a.rows, a.cols, a.x_stride, a.row_bytes, a.accumulate, a.slice_stages, a.partials);
  if (a.partials)
    hipLaunchKernelGGL(mm_reduce_kernel, dim3((unsigned)((cnt + 255) / 256)), dim3(256), 0, st, (const float*)a.partials, a.Y, cnt, (uint32_t)kz,
                       a.accumulate);
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}
template <class F>
int launch_tile_t(hipStream_t st, const MmArgs& a) {
  return a.n >= 192 ? launch_tile_c<F, 16, 64>(st, a) : launch_tile_c<F, 8, 128>(st, a);
}
int launch_tile(hipStream_t st, int t, const MmArgs& a) {
  switch (t) {
    case MSQ_Q8_0: return launch_tile_t<FragQ8_0>(st, a);
    case MSQ_IQ4_NL: return launch_tile_t<FragIQ4NL>(st, a);
    case MSQ_IQ1_S: return launch_tile_t<FragIQ1S>(st, a);
    case MSQ_IQ2_XXS: return launch_tile_t<FragIQ2XXS>(st, a);
  }
  return unsupported("matmul", t, (int)a.rows, (int)a.cols);
}
// Which calls take it, from what was measured against the two other routes on MI355X: the codebook formats, Q8_0 and
// IQ4_NL, matrices of twelve million weights and more, 65 to 256 tokens (IQ2_XXS 4096x7168 at 128 tokens: 30 us against
// 35 fused / 53 materialised; Q8_0 4096x4096 at 256: 33 against 45 / 34; beyond 256 tokens the dense GEMM on the
// materialised matrix is ahead, and on smaller matrices the kernel above; Q6_K and Q5_K gain 6 % at best and stay
// with the two other routes). MSQ_MM_TILE_MIN / _MAX / _ELEMS move the bounds. Also required: the matrix and the
// activations each below 4 GiB (a buffer descriptor spans them), activation rows on 16-byte boundaries.
bool tile_ok(int t, int n, int rows, int cols, size_t x_stride, const void* X16) {
  switch (t) {
    case MSQ_Q8_0: case MSQ_IQ4_NL: case MSQ_IQ1_S: case MSQ_IQ2_XXS: break;
    default: return false;
  }
  static const long min_elems = [] { const char* e = getenv("MSQ_MM_TILE_ELEMS"); return e && *e ? atol(e) : 12000000L; }();
  const size_t lim = ((size_t)1 << 32) - 64;
  if (fused_forced() >= 0 && n > fused_forced()) return false;
  return n >= tile_min_tokens() && n <= tile_max_tokens() && (long)rows * cols >= min_elems &&
         (size_t)rows * msq_type_row_bytes(t, cols) < lim && ((size_t)(n - 1) * x_stride + cols) * 2 < lim && x_stride % 8 == 0 &&
         ((uintptr_t)X16 & 15) == 0;
}

// fp16 copy of the activations for the tile kernel: a file-scope device array (nothing allocated, capturable) while
// it is large enough, the growing scratch above otherwise. Like the partial sums it is shared by the calls of a device.
constexpr size_t kMmX16Bytes = (size_t)16 << 20;
__device__ __align__(256) uint16_t g_mm_x16[kMmX16Bytes / 2];
uint16_t* g_mm_x16_ptr[16] = {};
uint16_t* mm_x16() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
  std::lock_guard<std::mutex> lock(g_mu);
  if (!g_mm_x16_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_mm_x16)) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    g_mm_x16_ptr[dev] = (uint16_t*)p;
  }
  return g_mm_x16_ptr[dev];
}

// more tokens than the fused kernel takes: W as fp16 in scratch (F16 weights are the GEMM operand as they are), then the dense GEMM
int matmul_big(hipStream_t st, int t, const MsqBuffer* W, int rows, int cols, const uint16_t* X16, float* Y, int n, bool accumulate,
               int x_stride) {
  const uint16_t* w16 = (const uint16_t*)bptr(W);
  if (t != MSQ_F16) {
    const int rc = reserve(g_w16, (size_t)rows * cols * 2, st);
    if (rc != MSQ_OK) return rc;
    const int rd = launch_deq_f16(st, t, bptr(W), (uint16_t*)g_w16.p, (int64_t)rows * cols);
    if (rd != MSQ_OK) return rd;
    w16 = (const uint16_t*)g_w16.p;
  }
  return gemm_f16(st, w16, X16, Y, n, rows, cols, x_stride, accumulate);
}

}  // namespace

void matmul_partials_setup() { (void)mm_partials(); (void)mm_x16(); }

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
  // (a row is whole blocks: for the 256-weight formats a multiple of 128 columns is not enough)
  if (!mm_type_ok(t) || rows < 1 || cols < 1 || cols % 128 || cols % msq_type_block_elems(t) || n < 1 || (x_stride && x_stride < cols))
    return unsupported("matmul", t, rows, cols);
  const int xs = x_stride ? x_stride : cols;
  if (!buf_ok(W, msq_type_row_bytes(t, cols) * (size_t)rows) || !buf_ok(X16, ((size_t)(n - 1) * xs + cols) * 2) ||
      !buf_ok(Y, (size_t)n * rows * 4) || ((uintptr_t)bptr(X16) & 1) || ((uintptr_t)bptr(Y) & 3))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: matmul: buffer missing, too small or misaligned (type %s rows %d cols %d n %d)",
                msq_type_name_of(t), rows, cols, n);
  hipStream_t st = (hipStream_t)stream;
  if (tile_ok(t, n, rows, cols, (size_t)xs, bptr(X16))) {
    const MmArgs a{bptr(X16), bptr(W), (float*)bptr_mut(Y), (uint32_t)n, (uint32_t)rows, (uint32_t)cols, (uint32_t)xs,
                   (uint32_t)msq_type_row_bytes(t, cols), accumulate ? 1u : 0u};
    return launch_tile(st, t, a);
  }
  if (use_fused(t, n, rows)) {
    const MmArgs a{bptr(X16), bptr(W), (float*)bptr_mut(Y), (uint32_t)n, (uint32_t)rows, (uint32_t)cols, (uint32_t)xs,
                   (uint32_t)msq_type_row_bytes(t, cols), accumulate ? 1u : 0u};
    return launch_mm<false>(st, t, a);
  }
  std::lock_guard<std::mutex> lock(g_mu);
  return matmul_big(st, t, W, rows, cols, (const uint16_t*)bptr(X16), (float*)bptr_mut(Y), n, accumulate != 0, xs);
}

int msq_matmul(void* stream, int t, const MsqBuffer* W, int rows, int cols, const MsqBuffer* X, const MsqBuffer* Y, int n,
               int accumulate) {
  if (!mm_type_ok(t) || rows < 1 || cols < 1 || cols % 128 || cols % msq_type_block_elems(t) || n < 1) return unsupported("matmul", t, rows, cols);
  if (!buf_ok(W, msq_type_row_bytes(t, cols) * (size_t)rows) || !buf_ok(X, (size_t)n * cols * 4) || !buf_ok(Y, (size_t)n * rows * 4) ||
      ((uintptr_t)bptr(X) & 15) || ((uintptr_t)bptr(Y) & 3))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: matmul: buffer missing, too small or misaligned (type %s rows %d cols %d n %d)",
                msq_type_name_of(t), rows, cols, n);
  hipStream_t st = (hipStream_t)stream;
  if (tile_ok(t, n, rows, cols, (size_t)cols, nullptr)) {
    // the activations as fp16 rows first (one pass over X; every workgroup of the tile kernel then fetches half the bytes)
    const size_t xbytes = (size_t)n * cols * 2;
    uint16_t* x16 = xbytes <= kMmX16Bytes ? mm_x16() : nullptr;
    std::unique_lock<std::mutex> lock(g_mu, std::defer_lock);
    if (!x16) {
      lock.lock();
      const int rc = reserve(g_x16, xbytes, st);
      if (rc != MSQ_OK) return rc;
      x16 = (uint16_t*)g_x16.p;
    }
    const int rx = launch_f32_to_f16(st, (const float*)bptr(X), x16, (size_t)n * cols);
    if (rx != MSQ_OK) return rx;
    const MmArgs a{x16, bptr(W), (float*)bptr_mut(Y), (uint32_t)n, (uint32_t)rows, (uint32_t)cols, (uint32_t)cols,
                   (uint32_t)msq_type_row_bytes(t, cols), accumulate ? 1u : 0u};
    return launch_tile(st, t, a);
  }
  if (use_fused(t, n, rows)) {
    const MmArgs a{bptr(X), bptr(W), (float*)bptr_mut(Y), (uint32_t)n, (uint32_t)rows, (uint32_t)cols, (uint32_t)cols,
                   (uint32_t)msq_type_row_bytes(t, cols), accumulate ? 1u : 0u};
    return launch_mm<true>(st, t, a);  // X is rounded to fp16 on its way into LDS
  }
  std::lock_guard<std::mutex> lock(g_mu);
  const int rc = reserve(g_x16, (size_t)n * cols * 2, st);
  if (rc != MSQ_OK) return rc;
  const int rx = launch_f32_to_f16(st, (const float*)bptr(X), (uint16_t*)g_x16.p, (size_t)n * cols);
  if (rx != MSQ_OK) return rx;
  return matmul_big(st, t, W, rows, cols, (const uint16_t*)g_x16.p, (float*)bptr_mut(Y), n, accumulate != 0, cols);
}

}  // extern "C"
