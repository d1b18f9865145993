// Host-side helpers shared by the C-ABI translation units: error reporting, buffer checks, device facts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "../../include/msq.h"
#include "msq_types.h"

namespace msq {

extern thread_local char g_err[512];

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}
// reference message shape: "macseek quant: <what> unsupported (type T rows R cols C)" (src/kernels/quant.mm:34-37)
inline int unsupported(const char* what, int t, int rows, int cols) {
  return fail(MSQ_ERR_UNSUPPORTED, "macseek quant: %s unsupported (type %s rows %d cols %d)", what, msq_type_name_of(t), rows, cols);
}
inline int hip_fail(hipError_t e, const char* where) {
  return fail(MSQ_ERR_HIP, "macseek quant: HIP error in %s: %s", where, hipGetErrorString(e));
}
#define MSQ_HIP(expr)                                        \
  do {                                                       \
    hipError_t e_ = (expr);                                  \
    if (e_ != hipSuccess) return ::msq::hip_fail(e_, #expr); \
  } while (0)

// LDS of one CU; a kernel that takes more than 64 KB of it as dynamic LDS has to be told so. The limit granted so far
// is kept per kernel (keyed by the kernel's address: instantiations of one template share their function type) and
// per device.
constexpr int kMaxLds = 160 * 1024;
int grant_large_lds(const void* kernel, size_t lds);  // msq_matvec.hip
template <class K>
int allow_large_lds(K kernel, size_t lds) {
  return lds > 64 * 1024 ? grant_large_lds((const void*)kernel, lds) : MSQ_OK;
}
inline const uint8_t* bptr(const MsqBuffer* b) { return (const uint8_t*)b->dev + b->off; }
inline uint8_t* bptr_mut(const MsqBuffer* b) { return (uint8_t*)b->dev + b->off; }
inline bool buf_ok(const MsqBuffer* b, size_t need) { return b && b->dev && b->size >= need; }

struct DeviceInfo { int ok, cus; };
const DeviceInfo& device_info();  // cached facts of the current device (CU count, gfx950 check)

// looks up this device's copy of the static MoE scratch (msq_moe.hip); called by msq_init() and by the entry point
int static_scratch_setup(float** out);
void matmul_partials_setup();     // msq_matmul.hip: looks up the current device's partial-sum buffer
void prefill_side_stream_setup();  // msq_prefill.hip: creates the current device's side stream and its two events

// small-N matvec through the dot-product kernels (msq_matvec.hip); MSQ_ERR_UNSUPPORTED, without a message, when the
// shape does not fit them
int matvec_tok(hipStream_t st, int t, const uint8_t* W, int rows, int cols, const float* X, float* Y, int n, int accumulate,
               int groups, const MsqMvCfg* cfg = nullptr, const float* norm_w = nullptr, float eps = 0.f);

}  // namespace msq
