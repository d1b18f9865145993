// C ABI: small-N matvec (see include/msq.h; reference host code src/kernels/quant.mm:129-156).
#include <algorithm>
#include <cstdlib>

#include "msq_host.h"
#include "msq_mvn.cuh"

namespace msq {
namespace {

template <class F>
int launch_mvn(hipStream_t st, MvnArgs a) {
  const int cus = device_info().cus;
  a.nsteps = a.cols / 32u;
  const uint32_t ks = std::min<uint32_t>(16u, a.nsteps);
  a.steps_per_wave = (a.nsteps + ks - 1) / ks;
  const uint32_t waves = (a.nsteps + a.steps_per_wave - 1) / a.steps_per_wave;
  const size_t lds = (size_t)waves * 16 * 17 * 4;  // dynamic LDS: the partial results (the table is a static array)
  // resident workgroups per CU (the kernel takes up to 128 registers per lane: 16 waves per CU); a persistent
  // workgroup keeps its activation fragments across tiles, a later one would stage them again
  const int wg_per_cu = std::max(1, 16 / (int)waves);
  const long grid = std::min<long>(a.ntiles, (long)cus * wg_per_cu);
  hipLaunchKernelGGL((mvn_kernel<F>), dim3((unsigned)grid), dim3(64 * waves), lds, st, a);
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

}  // namespace
}  // namespace msq

using namespace msq;

extern "C" int msq_matvec_n(void* stream, int t, const MsqBuffer* W, int rows, int cols, const MsqBuffer* X,
                            const MsqBuffer* Y, int n, int accumulate, int groups) {
  if (n == 1) return msq_matvec(stream, t, W, rows, cols, X, Y, accumulate, groups, nullptr);
  const int be = msq_type_block_elems(t);
  const int colmul = be == 1 ? 256 : be;
  if (!msq_matvec_supported(t) || n < 1 || n > 16 || rows < 1 || cols < 1 || cols % colmul || groups < 1 || rows % groups)
    return unsupported("matvec_n", t, rows, cols);
  const size_t rb = msq_type_row_bytes(t, cols);
  const size_t xs = (size_t)cols * groups;
  if (!buf_ok(W, rb * (size_t)rows) || !buf_ok(X, xs * n * 4) || !buf_ok(Y, (size_t)rows * n * 4))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: matvec_n: buffer missing or too small (type %s rows %d cols %d n %d)",
                msq_type_name_of(t), rows, cols, n);
  const int rpg = rows / groups;
  const double mb = (double)rb * rows / 1e6;
  // From nine tokens on (two passes of the dot-product kernel below) the K-quant and codebook formats go through the
  // fused matrix-core kernel of msq_matmul, as the reference's small-N operator hands its larger n to its matmul kernel
  // (quant.mm:133): Q6_K 2304x5120 at 12 tokens 17.3 -> 11.1 us, IQ1_S 4096x7168 at 16 tokens 24.9 -> 16.7, Q5_K
  // 1280x5120 at 16 tokens 13.7 -> 9.7; at eight tokens only Q6_K matrices of 5 to 12 MB gain (1536x7168: 11.3 -> 10.8).
  // IQ4_NL, Q8_0 and the dense types stay below (IQ4_NL 7168x4096 at 16 tokens: 20.6 us here, 26.4 there). That route
  // sums its K slices through a buffer inside the library: such calls must be enqueued on one stream at a time.
  {
    const bool kq = t == MSQ_Q6_K || t == MSQ_Q5_K || t == MSQ_IQ1_S || t == MSQ_IQ2_XXS;
    const bool mm = groups == 1 && cols % 128 == 0 && ((kq && n >= 9) || (t == MSQ_Q6_K && n == 8 && mb >= 5.0 && mb <= 12.0));
    static const bool off = [] { const char* e = getenv("MSQ_MVN_MM"); return e && *e == '0'; }();
    if (mm && !off && !((uintptr_t)bptr(X) & 15)) return msq_matmul(stream, t, W, rows, cols, X, Y, n, accumulate);
  }
  // Two kernels serve 2 <= n <= 8 (and what the rule above leaves). The dot-product kernel (weights fetched in contiguous runs, decoded once for up to eight
  // tokens, dot2 chains per token) wins wherever its shape fits: measured on MI355X at n = 16, IQ4_NL 7168x4096 takes
  // 20.7 us there and 25.4 us through the MFMA kernel, Q8_0 4096x7168 28.8 and 29.6 us, Q6_K 1536x7168 14.4 and 42.9 us.
  {
    const int rc = matvec_tok((hipStream_t)stream, t, bptr(W), rows, cols, (const float*)bptr(X), (float*)bptr_mut(Y), n, accumulate, groups);
    if (rc != MSQ_ERR_UNSUPPORTED) return rc;
  }
  // Rows too wide for the dot-product kernel (or for its activation staging in LDS): a few tokens over a small matrix
  // are served faster as n decode matvecs (the matrix stays in the caches after the first) than by the MFMA kernel: a
  // matvec launch costs about 3 us + 1 us per 1.5 MB of weights, an MFMA launch about 20 us + 1 us per MB (one 16-row
  // tile per workgroup pass, K split over its waves).
  const bool few = n * (3.0 + mb / 1.5) < 20.0 + mb;
  if (t == MSQ_F32 || (groups > 1 && rpg % 16) || few) {  // served as n decode matvecs
    for (int i = 0; i < n; i++) {
      const MsqBuffer xi{X->dev, X->off + (size_t)i * xs * 4, xs * 4}, yi{Y->dev, Y->off + (size_t)i * rows * 4, (size_t)rows * 4};
      const int rc = msq_matvec(stream, t, W, rows, cols, &xi, &yi, accumulate, groups, nullptr);
      if (rc != MSQ_OK) return rc;
    }
    return MSQ_OK;
  }
  MvnArgs a{};
  a.W = bptr(W); a.X = (const float*)bptr(X); a.Y = (float*)bptr_mut(Y);
  a.rows = (uint32_t)rows; a.cols = (uint32_t)cols; a.row_bytes = (uint32_t)rb; a.n = (uint32_t)n;
  a.x_stride = (uint32_t)xs; a.y_stride = (uint32_t)rows;
  a.rows_per_group = (uint32_t)rpg; a.x_group_stride = (uint32_t)cols; a.accumulate = accumulate ? 1u : 0u;
  a.ntiles = (uint32_t)((rows + 15) / 16);
  hipStream_t st = (hipStream_t)stream;
  switch (t) {
    case MSQ_IQ1_S: return launch_mvn<FragIQ1S>(st, a);
    case MSQ_IQ2_XXS: return launch_mvn<FragIQ2XXS>(st, a);
    case MSQ_Q8_0: return launch_mvn<FragQ8_0>(st, a);
    case MSQ_IQ4_NL: return launch_mvn<FragIQ4NL>(st, a);
    case MSQ_Q6_K: return launch_mvn<FragQ6K>(st, a);
    case MSQ_Q5_K: return launch_mvn<FragQ5K>(st, a);
    case MSQ_F16: return launch_mvn<FragDense16<MSQ_F16>>(st, a);
    case MSQ_BF16: return launch_mvn<FragDense16<MSQ_BF16>>(st, a);
  }
  return unsupported("matvec_n", t, rows, cols);
}
