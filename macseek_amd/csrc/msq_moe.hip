// C ABI: fused one-token MoE layer (see include/msq.h; reference host code src/kernels/quant.mm:252-369).
#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "msq_host.h"
#include "msq_moe.cuh"

namespace msq {

// ---- msq_moe_decode_static: the h scratch of the one-token layer in memory the library's code object carries, for
// callers that cannot allocate. Every device that loads the library holds its own copy of the array; host code never
// uses the array's name as an address (it is only a handle for hipGetSymbolAddress), but the per-device pointer that
// static_scratch_setup() looks up once, with that device current.
constexpr int kStaticMaxInter = 4096;  // largest expert intermediate size the static scratch serves
static __device__ __align__(256) float g_moe_static_scratch[(kMaxRouted + 1) * kStaticMaxInter * 3 / 2];  // fp32 h + fp16 h
constexpr int kStaticMaxDevices = 64;
static float* g_static_ptr[kStaticMaxDevices];
static std::mutex g_static_mu;

int static_scratch_setup(float** out) {
  int dev = 0;
  MSQ_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kStaticMaxDevices) return fail(MSQ_ERR_ARGUMENT, "macseek quant: device ordinal %d is beyond the static scratch table", dev);
  std::lock_guard<std::mutex> lock(g_static_mu);
  if (!g_static_ptr[dev]) {
    void* p = nullptr;
    MSQ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_moe_static_scratch)));
    if (!p) return fail(MSQ_ERR_HIP, "macseek quant: hipGetSymbolAddress returned no address for the static MoE scratch");
    g_static_ptr[dev] = (float*)p;
  }
  if (out) *out = g_static_ptr[dev];
  return MSQ_OK;
}

namespace {

bool routed_type_ok(int t) { return t == MSQ_IQ1_S || t == MSQ_IQ2_XXS; }
bool shared_type_ok(int t) { return t == MSQ_Q6_K || t == MSQ_Q8_0 || t == MSQ_IQ2_XXS || t == MSQ_IQ1_S; }

template <class DR, class DS>
int launch_gu_t(dim3 g, dim3 b, size_t lds, hipStream_t st, const MoeArgs& a) {
  if (const int rc = allow_large_lds(moe_gu_kernel<DR, DS>, lds)) return rc;
  hipLaunchKernelGGL((moe_gu_kernel<DR, DS>), g, b, lds, st, a.table, a);
  return MSQ_OK;
}
template <class DR, class DS>
int launch_down_t(dim3 g, dim3 b, size_t lds, hipStream_t st, const MoeArgs& a) {
  if (b.x <= 768) {
    if (const int rc = allow_large_lds(moe_down_kernel<DR, DS, 768>, lds)) return rc;
    hipLaunchKernelGGL((moe_down_kernel<DR, DS, 768>), g, b, lds, st, a.table, a);
  } else {
    if (const int rc = allow_large_lds(moe_down_kernel<DR, DS, 1024>, lds)) return rc;
    hipLaunchKernelGGL((moe_down_kernel<DR, DS, 1024>), g, b, lds, st, a.table, a);
  }
  return MSQ_OK;
}
// launch-shape knobs for experiments (the reference exposes MACSEEK_MOE_* the same way, quant.mm:274-276)
int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return v && *v ? atoi(v) : dflt;
}
// The staged activations follow the partial sums in dynamic LDS when everything (with the kernel's static tables) fits
// the CU's LDS. gate/up: x in the routed decoder's form for the routed workgroups, in the shared decoder's form for
// the others (one region, sized for the larger); down: the routed h rows in DR's form, then the shared row in DS's.
template <class DR, class DS, bool DOWN>
size_t place_x(MoeArgs& a, size_t lds, uint32_t cols_r, uint32_t cols_s) {
  const size_t static_lds = 4 * (size_t)(DOWN ? DR::LDS_WORDS + DS::LDS_WORDS
                                              : std::max<int>(DR::LDS_WORDS, DS::LDS_WORDS));
  const size_t wr = cols_r ? x_stage_words<DR>(cols_r) : 0, ws = cols_s ? x_stage_words<DS>(cols_s) : 0;
  const size_t words = DOWN ? wr + ws : std::max(wr, ws);
  const size_t at = (lds + 15) / 16 * 16, end = at + words * 4;
  a.xs_off = (uint32_t)(at / 4);
  a.stage_x = end + static_lds + 64 <= (size_t)kMaxLds ? 1u : 0u;
  return a.stage_x ? end : lds;
}
// The down kernel (rows of `inter` columns: one wave per row, a dozen rows per wave and launch) keeps the fp16 form of
// the IQ1_S decoder: the integer form's larger tables and activation quantization cost its prologue more than its
// shorter decode saves there.
template <class D> struct DownDec { using T = D; };
template <> struct DownDec<DecIQ1SQ> { using T = DecIQ1S; };
template <> struct DownDec<DecIQ2XXSQ> { using T = DecIQ2XXS; };
template <> struct DownDec<DecQ6KQ> { using T = DecQ6K; };
// dispatch over (routed type, shared type); cols_r / cols_s: activations the routed / shared part stages (0 = none)
// returns MSQ_OK, a launch's error, or MSQ_ERR_UNSUPPORTED (without a message) when no kernel serves the type pair
template <bool DOWN>
int dispatch(int tr, int ts, dim3 g, dim3 b, size_t part_bytes, uint32_t cols_r, uint32_t cols_s, hipStream_t st, MoeArgs& a) {
#define MSQ_MOE_CASE(TR, DRT, TS, DST)                                                            \
  if (tr == TR && ts == TS) {                                                                     \
    if constexpr (DOWN) {                                                                         \
      using R = typename DownDec<DRT>::T;                                                         \
      using S = typename DownDec<DST>::T;                                                         \
      const size_t lds = place_x<R, S, true>(a, part_bytes, cols_r, cols_s);                      \
      return launch_down_t<R, S>(g, b, lds, st, a);                                               \
    } else {                                                                                      \
      const size_t lds = place_x<DRT, DST, false>(a, part_bytes, cols_r, cols_s);                 \
      return launch_gu_t<DRT, DST>(g, b, lds, st, a);                                             \
    }                                                                                             \
  }
  MSQ_MOE_CASE(MSQ_IQ1_S, DecIQ1SQ, MSQ_Q6_K, DecQ6KQ)
  MSQ_MOE_CASE(MSQ_IQ1_S, DecIQ1SQ, MSQ_Q8_0, DecQ8_0)
  MSQ_MOE_CASE(MSQ_IQ1_S, DecIQ1SQ, MSQ_IQ2_XXS, DecIQ2XXSQ)
  MSQ_MOE_CASE(MSQ_IQ1_S, DecIQ1SQ, MSQ_IQ1_S, DecIQ1SQ)
  MSQ_MOE_CASE(MSQ_IQ2_XXS, DecIQ2XXSQ, MSQ_Q6_K, DecQ6KQ)
  MSQ_MOE_CASE(MSQ_IQ2_XXS, DecIQ2XXSQ, MSQ_Q8_0, DecQ8_0)
  MSQ_MOE_CASE(MSQ_IQ2_XXS, DecIQ2XXSQ, MSQ_IQ2_XXS, DecIQ2XXSQ)
  MSQ_MOE_CASE(MSQ_IQ2_XXS, DecIQ2XXSQ, MSQ_IQ1_S, DecIQ1SQ)
#undef MSQ_MOE_CASE
  return MSQ_ERR_UNSUPPORTED;
}

int moe_decode_impl(hipStream_t st, const MsqMoeDecodeArgs* p, const MsqBuffer* table, int part, bool need_table) {
  if (!p) return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_decode: null arguments");
  const int dim = p->dim ? p->dim : MSQ_EXPERT_DIM, inter = p->inter ? p->inter : MSQ_EXPERT_INTER;
  if (p->n_routed < 0 || p->n_routed > kMaxRouted) return unsupported("moe_decode n_routed", p->t_gate_up, p->n_routed, 0);
  const bool shared_part = part == MSQ_PART_SHARED_GU || part == MSQ_PART_SHARED || part == MSQ_PART_SHARED_DOWN;
  if (part < MSQ_PART_ALL || part > MSQ_PART_DOWN) return unsupported("moe_decode part", p->t_gate_up, part, 0);
  if (shared_part && !p->has_shared) return MSQ_OK;
  if (p->n_routed + (p->has_shared ? 1 : 0) == 0) return MSQ_OK;
  if (!routed_type_ok(p->t_gate_up) || !routed_type_ok(p->t_down) || (p->has_shared && !shared_type_ok(p->t_shared)))
    return unsupported("moe_decode type combo", p->t_gate_up, 0, 0);
  if (dim < 256 || inter < 256 || dim % 256 || inter % 256 || dim > 32768 || inter > 32768)
    return unsupported("moe_decode expert shape", p->t_gate_up, inter, dim);
  if (!buf_ok(&p->scratch, msq_moe_decode_scratch_bytes(inter)))
    return fail(MSQ_ERR_SCRATCH, "macseek quant: moe_decode scratch too small unsupported (type %s rows 0 cols 0)",
                msq_type_name_of(p->t_gate_up));
  // which pieces this call runs (reference: quant.mm:329-334)
  const bool gu_r = part == MSQ_PART_ALL || part == MSQ_PART_AFTER_SHARED_GU || part == MSQ_PART_ROUTED || part == MSQ_PART_GU;
  const bool gu_s = p->has_shared && (part == MSQ_PART_ALL || part == MSQ_PART_SHARED_GU || part == MSQ_PART_SHARED ||
                                      part == MSQ_PART_GU);
  const bool d_r = part == MSQ_PART_ALL || part == MSQ_PART_AFTER_SHARED_GU || part == MSQ_PART_ROUTED || part == MSQ_PART_DOWN;
  const bool d_s = p->has_shared && (part == MSQ_PART_ALL || part == MSQ_PART_AFTER_SHARED_GU || part == MSQ_PART_SHARED ||
                                     part == MSQ_PART_SHARED_DOWN || part == MSQ_PART_DOWN);
  const int nr = p->n_routed;
  const bool routed_live = nr > 0;
  if (!buf_ok(&p->x, (size_t)dim * 4) || !buf_ok(&p->y, (size_t)dim * 4))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_decode: x / y missing or too small");
  if (routed_live && gu_r && !buf_ok(&p->weights, (size_t)nr * 4))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_decode: routing weights missing or too small");
  const int ts = p->has_shared ? p->t_shared : MSQ_Q8_0;  // placeholder decoder when there is no shared expert
  MoeArgs a{};
  a.x = (const float*)bptr(&p->x); a.h = (float*)bptr_mut(&p->scratch); a.y = (float*)bptr_mut(&p->y);
  a.wts = p->weights.dev ? (const float*)bptr(&p->weights) : nullptr;
  a.n_routed = (uint32_t)nr; a.dim = (uint32_t)dim; a.inter = (uint32_t)inter;
  a.rb_gu_r = (uint32_t)msq_type_row_bytes(p->t_gate_up, dim); a.rb_d_r = (uint32_t)msq_type_row_bytes(p->t_down, inter);
  a.rb_gu_s = (uint32_t)msq_type_row_bytes(ts, dim); a.rb_d_s = (uint32_t)msq_type_row_bytes(ts, inter);
  if (routed_live && (gu_r || d_r)) {
    if (need_table) {
      if (!buf_ok(table, (size_t)kMaxRouted * 24)) return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_decode: table missing or too small");
      // (the kernels read the table through the scalar cache, which ignores an address's low bits)
      if ((uintptr_t)bptr(table) & 7) return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_decode: table not 8-byte aligned");
      a.table = (const uint64_t*)bptr(table);
    } else {
      for (int i = 0; i < nr; i++) {
        const MsqExpertSlot& s = p->slot[i];
        if (!buf_ok(&s.gate, (size_t)a.rb_gu_r * inter) || !buf_ok(&s.up, (size_t)a.rb_gu_r * inter) ||
            !buf_ok(&s.down, (size_t)a.rb_d_r * dim))
          return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_decode: routed slot %d missing or too small", i);
        a.gate[i] = bptr(&s.gate); a.up[i] = bptr(&s.up); a.down[i] = bptr(&s.down);
      }
    }
  }
  if (p->has_shared) {
    const MsqExpertSlot& s = p->shared;
    if (!buf_ok(&s.gate, (size_t)a.rb_gu_s * inter) || !buf_ok(&s.up, (size_t)a.rb_gu_s * inter) ||
        !buf_ok(&s.down, (size_t)a.rb_d_s * dim))
      return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_decode: shared expert missing or too small");
    a.sgate = bptr(&s.gate); a.sup = bptr(&s.up); a.sdown = bptr(&s.down);
  }
  // h also as scaled fp16, behind the fp32 rows, when the down kernel's decoder pair takes its activations in that form
  // (kHalfH in msq_moe.cuh: both decoders of the instantiation, the placeholder of a layer without shared expert included)
  auto x32_type = [](int t) { return t == MSQ_IQ1_S || t == MSQ_IQ2_XXS; };
  if (x32_type(p->t_down) && x32_type(ts)) a.h16 = (_Float16*)(a.h + (size_t)(kMaxRouted + 1) * inter);
  const int cus = device_info().cus;

  // 1) gate + up + SwiGLU -> h
  static const int env_gu_wgs = env_int("MSQ_MOE_GU_WGS", 1), env_d_wgs = env_int("MSQ_MOE_D_WGS", 1);
  static const int env_gu_rsg = env_int("MSQ_MOE_GU_RSG", 0), env_d_rsg = env_int("MSQ_MOE_D_RSG", 0);
  const int n_gu_r = (gu_r && routed_live) ? nr : 0;
  if (n_gu_r > 0 || gu_s) {
    const int units = dim / 32;
    const int ks = (units + 63) / 64;
    int rw = p->gu_rsg > 0 ? p->gu_rsg : env_gu_rsg > 0 ? env_gu_rsg : std::max(1, 16 / ks);
    if (rw * ks > 16) rw = std::max(1, 16 / ks);
    const int threads = 64 * rw * ks;
    a.ks = (uint32_t)ks;
    a.run_routed = n_gu_r > 0; a.run_shared = gu_s;
    const size_t part_bytes = (size_t)kMoeChunkRows * 2 * (4 * ks + 1) * 4;
    // persistent workgroups, dealt to the routed experts and the shared expert in proportion to their bytes
    const long rows_r = (long)n_gu_r * inter, rows_s = gu_s ? inter : 0;
    const long total = std::max<long>(2, (long)cus * std::max(1, env_gu_wgs));
    // ... weighted by the decode work per byte (IQ2_XXS takes two 16-byte table lookups and sign flips per 8 weights:
    // the layer of 6 IQ1_S + 1 IQ2_XXS experts is fastest with its bytes counted 1.4 times)
    static const int env_iq2_cost = env_int("MSQ_MOE_IQ2_COST", 140);  // percent
    auto cost = [](int t) { return t == MSQ_IQ2_XXS ? 0.01 * env_iq2_cost : 1.0; };
    const double br = (double)n_gu_r * a.rb_gu_r * cost(p->t_gate_up), bs = gu_s ? (double)a.rb_gu_s * cost(ts) : 0.0;
    long g_s = gu_s ? std::max<long>(1, (long)(total * bs / (br + bs) + 0.5)) : 0;
    long g_r = n_gu_r ? std::max<long>(1, total - g_s) : 0;
    if (g_r) { a.rows_per_wg_r = (uint32_t)((rows_r + g_r - 1) / g_r); g_r = (rows_r + a.rows_per_wg_r - 1) / a.rows_per_wg_r; }
    if (g_s) { a.rows_per_wg_s = (uint32_t)((rows_s + g_s - 1) / g_s); g_s = (rows_s + a.rows_per_wg_s - 1) / a.rows_per_wg_s; }
    a.grid_routed = (uint32_t)g_r;
    const int rc = dispatch<false>(p->t_gate_up, ts, dim3((unsigned)(g_r + g_s)), dim3(threads), part_bytes, g_r ? (uint32_t)dim : 0u,
                                   g_s ? (uint32_t)dim : 0u, st, a);
    if (rc == MSQ_ERR_UNSUPPORTED) return unsupported("moe_decode type combo", p->t_gate_up, 0, 0);
    if (rc != MSQ_OK) return rc;
    MSQ_HIP(hipGetLastError());
  }
  // 2) down for all experts, accumulated into y
  const bool run_d_r = d_r && routed_live;
  if (run_d_r || d_s) {
    const int units = inter / 32;
    const int ks = (units + 63) / 64;
    const int ne = run_d_r ? nr : 1;
    const int wpg = ne * ks;
    if (wpg > 16) return unsupported("moe_decode inter too large for the down kernel", p->t_down, dim, inter);
    // at most 12 waves where a row-group fits them: 170 registers per lane instead of 128 (the 1024-thread
    // instantiations of some decoder pairs spill a few registers; they remain for row-groups of 13 to 16 waves)
    const int max_waves = wpg <= 12 ? 12 : 16;
    int rw = p->d_rsg > 0 ? p->d_rsg : env_d_rsg > 0 ? env_d_rsg : std::max(1, max_waves / wpg);
    if (rw * wpg > max_waves) rw = std::max(1, max_waves / wpg);
    const int threads = 64 * rw * wpg;
    a.ks = (uint32_t)ks;
    a.run_routed = run_d_r; a.run_shared = d_s;
    const size_t slots = 4 * ((size_t)(run_d_r ? nr * ks : 0) + (d_s ? ks : 0));
    const size_t part_bytes = (size_t)kMoeChunkRows * (slots + 1) * 4;
    const long total = std::max<long>(1, (long)cus * std::max(1, env_d_wgs));
    a.rows_per_wg = (uint32_t)((dim + total - 1) / total);
    const long grid = (dim + a.rows_per_wg - 1) / a.rows_per_wg;
    const int rc = dispatch<true>(p->t_down, ts, dim3((unsigned)grid), dim3(threads), part_bytes, (uint32_t)((run_d_r ? nr : 0) * inter),
                                  d_s ? (uint32_t)inter : 0u, st, a);
    if (rc == MSQ_ERR_UNSUPPORTED) return unsupported("moe_decode type combo", p->t_down, 0, 0);
    if (rc != MSQ_OK) return rc;
    MSQ_HIP(hipGetLastError());
  }
  return MSQ_OK;
}

}  // namespace
}  // namespace msq

using namespace msq;

extern "C" {

size_t msq_moe_decode_scratch_bytes(int inter) {
  // h of the routed experts and the shared one as fp32, then the same values as fp16 (MoeArgs::h16)
  return (sizeof(float) + sizeof(_Float16)) * (size_t)(kMaxRouted + 1) * (size_t)(inter > 0 ? inter : MSQ_EXPERT_INTER);
}
int msq_moe_decode(void* stream, const MsqMoeDecodeArgs* a) {
  return moe_decode_impl((hipStream_t)stream, a, nullptr, MSQ_PART_ALL, false);
}
int msq_moe_decode_table(void* stream, const MsqMoeDecodeArgs* a, const MsqBuffer* table) {
  return moe_decode_impl((hipStream_t)stream, a, table, MSQ_PART_ALL, true);
}
int msq_moe_decode_table_part(void* stream, const MsqMoeDecodeArgs* a, const MsqBuffer* table, int part) {
  return moe_decode_impl((hipStream_t)stream, a, table, part, true);
}
int msq_moe_decode_static_max_inter(void) { return kStaticMaxInter; }
int msq_moe_decode_static(void* stream, const MsqMoeDecodeArgs* a) {
  if (!a) return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_decode_static: null arguments");
  const int inter = a->inter ? a->inter : MSQ_EXPERT_INTER;
  if (inter > kStaticMaxInter)
    return fail(MSQ_ERR_SCRATCH, "macseek quant: moe_decode_static: inter %d exceeds the static scratch limit of %d; use msq_moe_decode "
                "with caller scratch", inter, kStaticMaxInter);
  float* h = nullptr;
  if (const int rc = static_scratch_setup(&h)) return rc;
  MsqMoeDecodeArgs b = *a;
  b.scratch.dev = h;
  b.scratch.off = 0;
  b.scratch.size = sizeof(float) * (size_t)(kMaxRouted + 1) * kStaticMaxInter * 3 / 2;
  return moe_decode_impl((hipStream_t)stream, &b, nullptr, MSQ_PART_ALL, false);
}

}  // extern "C"
