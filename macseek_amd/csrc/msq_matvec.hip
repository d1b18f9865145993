// C ABI: library bring-up, geometry queries, decode matvec and dequantization (see include/msq.h).
#include <algorithm>
#include <map>
#include <mutex>
#include <utility>

#include "msq_deq.cuh"
#include "msq_host.h"
#include "msq_mv.cuh"
#include "msq_mvq.cuh"

namespace msq {

thread_local char g_err[512] = "";

const DeviceInfo& device_info() {
  static const DeviceInfo info = [] {
    DeviceInfo d{0, 256};
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) {
      d.cus = p.multiProcessorCount > 0 ? p.multiProcessorCount : 256;
      d.ok = strncmp(p.gcnArchName, "gfx950", 6) == 0;
    }
    return d;
  }();
  return info;
}

int grant_large_lds(const void* kernel, size_t lds) {
  static std::mutex mu;
  static std::map<std::pair<const void*, int>, size_t> granted;
  int dev = 0;
  MSQ_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  size_t& g = granted[{kernel, dev}];
  if (lds > g) {
    MSQ_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    g = lds;
  }
  return MSQ_OK;
}

// Plain streaming read: every workgroup walks contiguous 16 KiB chunks grid-stride, one 128-bit load per lane per step.
__global__ __launch_bounds__(1024) void bw_probe_kernel(const uint4* __restrict__ src, size_t n16, uint32_t* __restrict__ sink) {
  uint4 acc = {0, 0, 0, 0};
  const size_t chunk = 1024;  // uint4 per workgroup step
  for (size_t base = (size_t)blockIdx.x * chunk; base < n16; base += (size_t)gridDim.x * chunk) {
    const size_t i = base + threadIdx.x;
    if (i < n16) { const uint4 v = src[i]; acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w; }
  }
  const uint32_t r = acc.x ^ acc.y ^ acc.z ^ acc.w;
  if (r == 0x9E3779B9u) sink[blockIdx.x & 1023] = r;  // practically never true: keeps the loads alive without a store stream
}

namespace {

// Launch shape of the decode matvec. units = cols / UNIT columns-slices per row; a wave covers 64 * iters of them.
struct MvShape { int iters, ks, rw, rpw, unit; int per_cu = 1; bool stage_w = false, free_shape = false; };  // per_cu: persistent workgroups per CU, stage_w: weight rows through LDS (mv_tok_kernel), free_shape: no part of the shape was imposed by the caller

int mv_unit(int t) { return msq_type_block_elems(t) == 1 ? 8 : 32; }

bool mv_shape(int t, int rows, int cols, int groups, const MsqMvCfg* cfg, MvShape* s) {
  const int unit = mv_unit(t);
  const int units = cols / unit;
  int iters = 1;
  while (iters < 4 && units > 64 * 16 * iters) iters *= 2;
  int ks = (units + 64 * iters - 1) / (64 * iters);
  if (cfg && cfg->ks > 0) {  // a wider K split than needed only adds idle waves; a narrower one needs more iters
    ks = cfg->ks;
    while (iters < 4 && units > 64 * ks * iters) iters *= 2;
  }
  if (ks > 16 || units > 64 * ks * iters) return false;
  // the codebook formats stage a table of up to 32 KB per workgroup: one 16-wave workgroup per CU, each wave a run of
  // rows long enough for its register ring; the others run several small workgroups per CU
  const bool table = t == MSQ_IQ1_S || t == MSQ_IQ2_XXS;
  int rw = std::max(1, (table ? 16 : 8) / ks);
  if (cfg && cfg->rsg > 0) rw = cfg->rsg;
  if (rw * ks > 16) rw = std::max(1, 16 / ks);
  const int rpg = rows / groups;
  int rpw;
  if (table) {  // about one tile per CU
    const long per_cu = ((long)rows + device_info().cus - 1) / device_info().cus;
    rpw = (int)std::min<long>(64, std::max<long>(1, (per_cu + rw - 1) / rw));
  } else {  // rows per wave per tile: enough tiles to fill the chip a few times over, at most 8 rows per wave
    rpw = 8;
    while (rpw > 1 && (long)rows / (rw * rpw) < 2048) rpw /= 2;
  }
  if (cfg && cfg->nr > 0) rpw = std::min(cfg->nr, 64);
  if (groups > 1) {  // every tile must stay inside one block-diagonal group
    while (rpw > 1 && rpg % (rw * rpw)) rpw /= 2;
    while (rw > 1 && rpg % (rw * rpw)) rw /= 2;
    if (rpg % (rw * rpw)) return false;
  }
  *s = {iters, ks, rw, rpw, unit};
  return true;
}

// static LDS of the matvec kernels of decoder D: the codebook table (an array of at least four words)
template <class D>
constexpr size_t kStaticLds = (D::LDS_WORDS > 0 ? D::LDS_WORDS : 4) * 4 + 64;

// LDS layout behind the partial sums: the four partial sums of a fused norm, then the padded activation
// rows the workgroup stages, `tokens` of them, when all of it fits under `limit` bytes (else the activations are read
// straight from device memory; refused with a fused norm or when the kernel has no such path).
bool place_x_row(MvArgs& a, size_t& lds, int tokens = 1, size_t limit = 64 * 1024, bool required = false) {
  size_t at = (lds + 15) / 16 * 16;
  if (a.norm_w) { a.norm_off = (uint32_t)(at / 4); at += 16; }
  a.xs_off = (uint32_t)(at / 4);
  const size_t end = at + (size_t)xlds_words(a.cols) * 4 * tokens;
  a.stage_x = end <= limit ? 1u : 0u;
  if (a.stage_x) lds = end;
  return a.stage_x || !(a.norm_w || required);
}

template <class D>
int launch_mv(hipStream_t st, const MvShape& s, MvArgs& a) {
  const int threads = 64 * s.rw * s.ks;
  const int tile_rows = s.rw * s.rpw;
  a.units = a.cols / D::UNIT;
  a.ks = s.ks;
  a.rpw = s.rpw;
  a.ntiles = (a.rows + tile_rows - 1) / tile_rows;
  size_t lds = (size_t)tile_rows * s.ks * 4;  // dynamic LDS: partial sums, staged activations (the table is static)
  if ((D::STAGE_X || a.norm_w) && !place_x_row(a, lds, 1, 64 * 1024 - kStaticLds<D>)) return MSQ_ERR_UNSUPPORTED;
  // persistent workgroups: as many as can be resident, never more than there are tiles
  const int wg_per_cu = std::max(1, std::min(2048 / threads, (int)((size_t)kMaxLds / (lds + kStaticLds<D>))));
  const int grid = (int)std::min<long>(a.ntiles, (long)device_info().cus * wg_per_cu);
  if (a.norm_w) {
    if constexpr (requires { D::STAGES; }) return MSQ_ERR_UNSUPPORTED;  // codebook formats: as in the reference (quant.mm:110)
    else {
      switch (s.iters) {
        case 1: hipLaunchKernelGGL((mv_kernel<D, 1, true>), dim3(grid), dim3(threads), lds, st, a); break;
        case 2: hipLaunchKernelGGL((mv_kernel<D, 2, true>), dim3(grid), dim3(threads), lds, st, a); break;
        default: hipLaunchKernelGGL((mv_kernel<D, 4, true>), dim3(grid), dim3(threads), lds, st, a); break;
      }
      MSQ_HIP(hipGetLastError());
      return MSQ_OK;
    }
  }
  if constexpr (requires { D::STAGES; }) {  // codebook formats: ring kernel (one unit per lane, matrix below 4 GiB)
    if (s.iters == 1 && (uint64_t)a.rows * a.row_bytes < (1ull << 32)) {
      hipLaunchKernelGGL((mv_ring_kernel<D>), dim3(grid), dim3(threads), lds, st, a);
      MSQ_HIP(hipGetLastError());
      return MSQ_OK;
    }
  }
  switch (s.iters) {
    case 1: hipLaunchKernelGGL((mv_kernel<D, 1>), dim3(grid), dim3(threads), lds, st, a); break;
    case 2: hipLaunchKernelGGL((mv_kernel<D, 2>), dim3(grid), dim3(threads), lds, st, a); break;
    default: hipLaunchKernelGGL((mv_kernel<D, 4>), dim3(grid), dim3(threads), lds, st, a); break;
  }
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

int env_knob_early(const char* name, int dflt) {
  const char* v = getenv(name);
  return v && *v ? atoi(v) : dflt;
}
// Launch shape of the small-N matvec: workgroups of at most 8 waves (the kernel keeps T activation slices per lane
// and is built for 512 threads), one or two units per lane.
bool mv_tok_shape(int t, int rows, int cols, int groups, int n, int token_groups, const MsqMvCfg* cfg, MvShape* s) {
  const int unit = mv_unit(t);
  const int units = cols / unit;
  int iters = 1;
  while (iters < 2 && units > 64 * 8 * iters) iters *= 2;
  int ks = (units + 64 * iters - 1) / (64 * iters);
  if (cfg && cfg->ks > 0) {
    ks = cfg->ks;
    iters = units > 64 * ks ? 2 : 1;
  }
  if (ks > 8 || units > 64 * ks * iters) return false;
  int rw = std::max(1, 8 / ks);
  if (cfg && cfg->rsg > 0) rw = cfg->rsg;
  if (rw * ks > 8) return false;
  // rows per wave per tile: one workgroup per CU, one tile each, is what measures fastest (a wave prefetches along its
  // run of rows; every tile ends in a workgroup-wide reduction)
  // One token, a matrix without a codebook table that is large (48 MB: the launch is bound by the bytes a CU keeps in
  // flight, and a wave still walks a long run of rows) or dense and at least 8 MB (nothing to decode): two workgroups
  // per CU. Measured, one / two workgroups: Q6_K 129280x5120 165 / 132 us, Q6_K 25600x6144 43.6 / 29.9, F16 5120x5120
  // 13.7 / 11.2, BF16 4096x1280 6.75 / 5.2; the block formats between 5 and 35 MB lose up to 1.5 us with two.
  const bool table = t == MSQ_IQ1_S || t == MSQ_IQ2_XXS;
  static const int env_wgs = env_knob_early("MSQ_MV_WGS", 0);
  const bool free_shape = !(cfg && (cfg->nr > 0 || cfg->rsg > 0 || cfg->ks > 0));
  const double bytes = (double)msq_type_row_bytes(t, cols) * rows;
  const bool two = !table && (bytes >= 48e6 || (unit == 8 && bytes >= 8e6));
  const int per_cu = (n == 1 && free_shape) ? (env_wgs > 0 ? env_wgs : two ? 2 : 1) : 1;
  const long wgs = std::max(1, per_cu * device_info().cus / token_groups);
  int rpw = (int)std::min<long>(32, std::max<long>(1, (rows + wgs * rw - 1) / (wgs * rw)));
  if (cfg && cfg->nr > 0) rpw = std::min(cfg->nr, 64);
  const int rpg = rows / groups;
  if (groups > 1) {  // every tile must stay inside one block-diagonal group
    while (rpw > 1 && rpg % (rw * rpw)) rpw--;
    while (rw > 1 && rpg % (rw * rpw)) rw /= 2;
    if (rpg % (rw * rpw)) return false;
  }
  // Weight rows through LDS (mv_tok_kernel) where it measures faster: Q6_K (five loads per lane and row otherwise) from
  // 12 MB, Q8_0 (three) from 40 MB -- ring / through LDS: Q6_K 8192x5120 12.3 / 12.0 us, 65536x5120 71.9 / 57.0, Q8_0
  // 8192x5120 12.9 / 12.2, 65536x5120 82.4 / 67.5. Q5_K and IQ4_NL, whose 16-byte reads from LDS cost five words and four
  // shifts each, lose 10 to 17 %; the codebook formats are bound by their table lookups. MSQ_MV_STAGEW = 0 / 1 imposes
  // the choice.
  static const int env_sw = env_knob_early("MSQ_MV_STAGEW", -1);
  const bool stage_w = n == 1 && free_shape &&
                       (env_sw >= 0 ? env_sw > 0 : (t == MSQ_Q6_K && bytes >= 12e6) || (t == MSQ_Q8_0 && bytes >= 40e6));
  *s = {iters, ks, rw, rpw, unit, per_cu, stage_w, free_shape};
  return true;
}

// n = 1: the prefetching kernel pays from two full rows per wave and CU on (below that mv_kernel does the same with
// less ceremony). Large codebook matrices are bound by decode arithmetic and do better in the 16-wave ring kernel
// (measured: IQ1_S 4096x7168 7.5 against 8.6 us, 8192 rows 9.9 against 10.1 us, 16384 rows 20.3 against 14.7 us).
// An imposed shape with nr >= 2 and at most 8 waves names the prefetching kernel outright.
bool tok_serves_single(int t, int rows, int cols, const MvShape& s, const MsqMvCfg* cfg) {
  if (cfg && cfg->nr > 0) return s.rpw >= 2;
  const bool table = t == MSQ_IQ1_S || t == MSQ_IQ2_XXS;
  if (table && (double)msq_type_row_bytes(t, cols) * rows > 10e6) return false;
  return s.rpw >= 2 && (long)rows >= 2L * device_info().cus * s.rw;
}

template <class D, int T>
int launch_mv_tok(hipStream_t st, const MvShape& s_, const MvTokArgs& ta_) {
  MvTokArgs ta = ta_;  // (the launch may reshape rows into pairs: the caller's arguments stay as they are)
  MvArgs& a = ta.m;
  MvShape s = s_;
  // One token, rows whose units fill a whole number of waves and at most half of another (5120 or 7168 columns of a
  // block format: 2.5 and 3.5 waves): two rows are launched as one of twice the units, which leaves no lane idle
  // (mv_tok_kernel, PAIR). One group, an even number of rows, a row's units a multiple of 16. Measured, rows one by
  // one / in pairs: Q6_K 129280x5120 113.2 / 99.8 us, 1536x7168 6.41 / 6.10, 2304x5120 6.61 / 6.29, Q8_0 2304x5120
  // 6.67 / 6.52; the codebook formats, bound by their lookups, lose 1 % and keep the one-row form. MSQ_MV_PAIR = 0 / 2:
  // never / every format.
  bool pair = false;
  {
    static const int env_pair = env_knob_early("MSQ_MV_PAIR", -1);
    const int u = (int)(a.cols / D::UNIT), k1 = (u + 63) / 64, k2 = (2 * u + 63) / 64;
    pair = s.iters == 1 && s.free_shape && (D::LDS_WORDS == 0 || env_pair == 2) && !a.norm_w && env_pair != 0 && a.rows % 2 == 0 && a.rows_per_group >= a.rows && u % 16 == 0 &&
           k2 < 2 * k1 && k2 <= 8;
    if (pair) {
      a.rows /= 2;
      a.rows_per_group = a.rows;
      a.row_bytes *= 2;
      s.ks = k2;
      s.rw = std::max(1, 8 / k2);
      const long wgs = std::max<long>(1, s.per_cu * device_info().cus / (((long)ta.n + T - 1) / T));
      s.rpw = (int)std::min<long>(32, std::max<long>(1, (a.rows + wgs * s.rw - 1) / (wgs * s.rw)));
    }
  }
  const int threads = 64 * s.rw * s.ks;
  const int tile_rows = s.rw * s.rpw;
  a.units = (pair ? 2 : 1) * (a.cols / D::UNIT);
  a.ks = s.ks;
  a.rpw = s.rpw;
  a.ntiles = (a.rows + tile_rows - 1) / tile_rows;
  size_t lds = (size_t)tile_rows * s.ks * 4 * T * 4;  // dynamic LDS: partial sums, staged activations (the table is static)
  const int gy = ((int)ta.n + T - 1) / T;
  if (tok_stages_x<D, T>() || a.norm_w) {
    // one workgroup per CU: all of its LDS (decoders that stage only in the four-token kernel read directly when a round does not fit)
    if (!place_x_row(a, lds, tok_round<D, T>(), kMaxLds - kStaticLds<D>, D::STAGE_X)) return MSQ_ERR_UNSUPPORTED;
  }
  const bool sw = tok_stages_w<D, 1, T>() && s.iters == 1 && s.stage_w && !a.norm_w;
  if (sw) {  // the waves' weight-row buffers
    lds = (lds + 15) / 16 * 16;
    a.w_off = (uint32_t)(lds / 4);
    lds += (size_t)(threads / 64) * 4 * wspan_loads<D>() * 1024;  // four slots per wave
  }
  auto launch = [&](auto kernel, dim3 grid) {
    allow_large_lds(kernel, lds);
    hipLaunchKernelGGL(kernel, grid, dim3(threads), lds, st, a.W, a.rows, a.row_bytes, a.units, a.ks, a.rpw, a.ntiles, a.rows_per_group, a.x, a.cols, ta);
  };
  if (a.norm_w) {  // fused input norm (single token)
    if constexpr (T != 1 || requires { D::STAGES; }) return MSQ_ERR_UNSUPPORTED;
    else {
      const dim3 gxn((unsigned)std::min<long>(a.ntiles, std::max(1, device_info().cus)));
      if (s.iters == 1) launch(mv_tok_kernel<D, 1, 1, true>, gxn);
      else if constexpr (D::UNIT == 8) launch(mv_tok_kernel<D, 2, 1, true>, gxn);
      else return MSQ_ERR_UNSUPPORTED;
      MSQ_HIP(hipGetLastError());
      return MSQ_OK;
    }
  }
  // persistent workgroups, one per CU over all token groups (two for a large matrix: MvShape::per_cu)
  const int per_cu = (T == 1 && !a.norm_w && (lds + kStaticLds<D>) * s.per_cu <= (size_t)kMaxLds) ? s.per_cu : 1;
  const int gx = (int)std::min<long>(a.ntiles, std::max(1, per_cu * device_info().cus / gy));
  const dim3 grid((unsigned)gx, (unsigned)gy);
  if (sw) {
    if constexpr (tok_stages_w<D, 1, T>()) {
      if (pair) launch(mv_tok_kernel<D, 1, T, false, true, true>, grid);
      else launch(mv_tok_kernel<D, 1, T, false, true>, grid);
    }
  } else if (s.iters == 1) {
    if (pair) launch(mv_tok_kernel<D, 1, T, false, false, true>, grid);
    else launch(mv_tok_kernel<D, 1, T>, grid);
  } else if constexpr (D::UNIT == 8) launch(mv_tok_kernel<D, 2, T>, grid);
  else return MSQ_ERR_UNSUPPORTED;  // two block-format units per lane and T activation slices do not fit the registers
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

template <int T>
int launch_mv_tok_t(hipStream_t st, int t, const MvShape& s, MvTokArgs& ta) {
  if constexpr (T == 1) {  // one token: the block formats' integer decoders (msq_mvq.cuh)
    switch (t) {
      case MSQ_IQ1_S: return launch_mv_tok<DecIQ1SM, 1>(st, s, ta);
      case MSQ_IQ2_XXS: return launch_mv_tok<DecIQ2XXSM, 1>(st, s, ta);
      case MSQ_IQ4_NL: return launch_mv_tok<DecIQ4NLQ, 1>(st, s, ta);
      case MSQ_Q6_K: return launch_mv_tok<DecQ6KQ, 1>(st, s, ta);
      case MSQ_Q5_K: return launch_mv_tok<DecQ5KQ, 1>(st, s, ta);
    }
  }
  switch (t) {
    case MSQ_IQ1_S: return launch_mv_tok<DecIQ1S, T>(st, s, ta);
    case MSQ_IQ2_XXS: return launch_mv_tok<DecIQ2XXS, T>(st, s, ta);
    case MSQ_IQ4_NL: return launch_mv_tok<DecIQ4NL, T>(st, s, ta);
    case MSQ_Q6_K: return launch_mv_tok<DecQ6K, T>(st, s, ta);
    case MSQ_Q5_K: return launch_mv_tok<DecQ5K, T>(st, s, ta);
    case MSQ_F32: return launch_mv_tok<DecDense<MSQ_F32>, T>(st, s, ta);
    case MSQ_F16: return launch_mv_tok<DecDense<MSQ_F16>, T>(st, s, ta);
    case MSQ_BF16: return launch_mv_tok<DecDense<MSQ_BF16>, T>(st, s, ta);
  }
  return MSQ_ERR_UNSUPPORTED;
}

bool mv_type_ok(int t) {
  switch (t) {
    case MSQ_F32: case MSQ_F16: case MSQ_BF16: case MSQ_Q8_0: case MSQ_Q5_K: case MSQ_Q6_K: case MSQ_IQ1_S:
    case MSQ_IQ2_XXS: case MSQ_IQ4_NL: return true;
    default: return false;
  }
}
// Launch-shape overrides from the environment, on top of the caller's MsqMvCfg (reference: MACSEEK_MV_NR / _RSG / _KS,
// quant.mm:78-83, and MACSEEK_MVN_NR / _SG for the small-N form, quant.mm:141): MSQ_MV_NR / MSQ_MV_RSG / MSQ_MV_KS for
// one token, MSQ_MVN_NR / MSQ_MVN_RSG / MSQ_MVN_KS for several. Returns null when nothing is imposed.
int env_knob(const char* name) {
  const char* v = getenv(name);
  return v && *v ? atoi(v) : 0;
}
const MsqMvCfg* effective_cfg(const MsqMvCfg* cfg, bool several, MsqMvCfg* store) {
  static const int e1[3] = {env_knob("MSQ_MV_NR"), env_knob("MSQ_MV_RSG"), env_knob("MSQ_MV_KS")};
  static const int en[3] = {env_knob("MSQ_MVN_NR"), env_knob("MSQ_MVN_RSG"), env_knob("MSQ_MVN_KS")};
  const int* e = several ? en : e1;
  *store = cfg ? *cfg : MsqMvCfg{0, 0, 0};
  if (e[0] > 0) store->nr = e[0];
  if (e[1] > 0) store->rsg = e[1];
  if (e[2] > 0) store->ks = e[2];
  return (store->nr > 0 || store->rsg > 0 || store->ks > 0) ? store : nullptr;
}
// column granularity the kernels need: dense types use a virtual 256 block like the reference (quant.mm:31-32)
int mv_col_multiple(int t) { return msq_type_block_elems(t) == 1 ? 256 : msq_type_block_elems(t); }

}  // namespace
}  // namespace msq

namespace msq {

// Small-N matvec through the dot-product kernels. Returns MSQ_ERR_UNSUPPORTED without an error message when the shape
// does not fit them (the caller then takes another path). Arguments are already validated.
int matvec_tok(hipStream_t st, int t, const uint8_t* W, int rows, int cols, const float* X, float* Y, int n, int accumulate,
               int groups, const MsqMvCfg* cfg, const float* norm_w, float eps) {
  MsqMvCfg several;
  if (n > 1) cfg = effective_cfg(cfg, true, &several);
  // tokens per pass over the weights: one, two, four or eight (Q8_0 keeps fp32 activations, 32 registers per token: four at most)
  // ... and groups of four also for more tokens over a small matrix (below 8 MB): every workgroup then fetches four
  // tokens' activations instead of eight, and the second group finds the weights in the caches (Q5_K 512x7168 at 8 / 16
  // tokens: 10.4 / 11.1 -> 7.3 / 8.8 us; BF16 384x7168 6.1 / 6.7 -> 5.2 / 6.2; the 9 MB and 16 MB matrices lose at 16)
  static const int env_t = env_knob("MSQ_MVN_T");
  const bool small = (double)msq_type_row_bytes(t, cols) * rows < 8e6;
  const int T = n <= 2 ? n : (t == MSQ_Q8_0 || n <= 4 || env_t == 4 || (small && env_t != 8)) ? 4 : 8;
  MvShape s;
  if (!mv_tok_shape(t, rows, cols, groups, n, (n + T - 1) / T, cfg, &s)) return MSQ_ERR_UNSUPPORTED;
  if (n == 1 && !tok_serves_single(t, rows, cols, s, cfg)) return MSQ_ERR_UNSUPPORTED;
  MvTokArgs ta{};
  MvArgs& a = ta.m;
  a.W = W; a.x = X; a.y = Y;
  a.rows = (uint32_t)rows; a.cols = (uint32_t)cols; a.row_bytes = (uint32_t)msq_type_row_bytes(t, cols);
  a.rows_per_group = (uint32_t)(rows / groups); a.x_group_stride = (uint32_t)cols; a.accumulate = accumulate ? 1u : 0u;
  ta.n = (uint32_t)n; ta.x_stride = (uint32_t)((size_t)cols * groups); ta.y_stride = (uint32_t)rows;
  a.norm_w = norm_w; a.eps = eps;
  if (n == 1) return t == MSQ_Q8_0 ? launch_mv_tok<DecQ8_0, 1>(st, s, ta) : launch_mv_tok_t<1>(st, t, s, ta);
  if (t == MSQ_Q8_0) return T == 2 ? launch_mv_tok<DecQ8_0, 2>(st, s, ta) : launch_mv_tok<DecQ8_0, 4>(st, s, ta);
  return T == 2 ? launch_mv_tok_t<2>(st, t, s, ta) : T == 4 ? launch_mv_tok_t<4>(st, t, s, ta) : launch_mv_tok_t<8>(st, t, s, ta);
}

}  // namespace msq

using namespace msq;

extern "C" {

int msq_init(void) {
  g_err[0] = 0;
  const DeviceInfo& d = device_info();
  if (!d.ok) return fail(MSQ_ERR_HIP, "macseek quant: no gfx950 device is current");
  prefill_side_stream_setup();
  matmul_partials_setup();
  return static_scratch_setup(nullptr);
}
const char* msq_last_error(void) { return g_err; }
int msq_device_ok(void) { return device_info().ok; }

int msq_block_elems(int t) { return msq_type_block_elems(t); }
size_t msq_block_bytes(int t) { return msq_type_block_bytes(t); }
size_t msq_row_bytes(int t, int64_t cols) { return msq_type_row_bytes(t, cols); }
const char* msq_type_name(int t) { return msq_type_name_of(t); }

int msq_matvec_supported(int t) { return mv_type_ok(t) ? 1 : 0; }

int msq_matvec_cfg(int t, int rows, int cols, MsqMvCfg* out) {
  MvShape s;
  if (!out) return fail(MSQ_ERR_ARGUMENT, "macseek quant: matvec_cfg: null output");
  if (!mv_type_ok(t) || rows < 1 || cols < 1 || cols % mv_col_multiple(t)) return unsupported("matvec_cfg", t, rows, cols);
  MsqMvCfg env;
  const MsqMvCfg* cfg = effective_cfg(nullptr, false, &env);
  const bool tok = mv_tok_shape(t, rows, cols, 1, 1, 1, cfg, &s) && tok_serves_single(t, rows, cols, s, cfg);  // as msq_matvec decides
  if (!tok && !mv_shape(t, rows, cols, 1, cfg, &s)) return unsupported("matvec_cfg", t, rows, cols);
  out->nr = s.rpw; out->rsg = s.rw; out->ks = s.ks;
  return MSQ_OK;
}

// msq_matvec and msq_matvec_rmsnorm (norm_w != nullptr: the activations are normalized on the way in; the kernel is the
// one msq_matvec picks for the matrix, so the two agree bit for bit on a pre-normalized input)
static int matvec_impl(void* stream, const char* what, int t, const MsqBuffer* W, int rows, int cols, const MsqBuffer* x,
                       const MsqBuffer* y, int accumulate, int groups, const MsqMvCfg* cfg, const float* norm_w, float eps) {
  const size_t rb = msq_type_row_bytes(t, cols);
  if (!buf_ok(W, rb * (size_t)rows) || !buf_ok(x, (size_t)cols * groups * 4) || !buf_ok(y, (size_t)rows * 4))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: %s: buffer missing or too small (type %s rows %d cols %d)", what,
                msq_type_name_of(t), rows, cols);
  hipStream_t st = (hipStream_t)stream;
  MsqMvCfg imposed;
  cfg = effective_cfg(cfg, false, &imposed);
  {  // shapes with several rows per wave (chosen for matrices of more than a row per wave and CU, or imposed by cfg) go
     // through the prefetching kernel; a shape names its kernel, so row chunks launched with the shape of the whole
     // matrix repeat its bits
    const int rc = matvec_tok(st, t, bptr(W), rows, cols, (const float*)bptr(x), (float*)bptr_mut(y), 1, accumulate, groups, cfg,
                              norm_w, eps);
    if (rc != MSQ_ERR_UNSUPPORTED) return rc;
  }
  MvShape s;
  if (!mv_shape(t, rows, cols, groups, cfg, &s)) return unsupported("matvec launch shape", t, rows, cols);
  MvArgs a{};
  a.W = bptr(W); a.x = (const float*)bptr(x); a.y = (float*)bptr_mut(y);
  a.rows = (uint32_t)rows; a.cols = (uint32_t)cols; a.row_bytes = (uint32_t)rb;
  a.rows_per_group = (uint32_t)(rows / groups); a.x_group_stride = (uint32_t)cols; a.accumulate = accumulate ? 1u : 0u;
  a.norm_w = norm_w; a.eps = eps;
  int rc = MSQ_ERR_UNSUPPORTED;
  switch (t) {
    case MSQ_IQ1_S: rc = launch_mv<DecIQ1SM>(st, s, a); break;
    case MSQ_IQ2_XXS: rc = launch_mv<DecIQ2XXSM>(st, s, a); break;
    case MSQ_Q8_0: rc = launch_mv<DecQ8_0>(st, s, a); break;
    case MSQ_IQ4_NL: rc = launch_mv<DecIQ4NLQ>(st, s, a); break;
    case MSQ_Q6_K: rc = launch_mv<DecQ6KQ>(st, s, a); break;
    case MSQ_Q5_K: rc = launch_mv<DecQ5KQ>(st, s, a); break;
    case MSQ_F32: rc = launch_mv<DecDense<MSQ_F32>>(st, s, a); break;
    case MSQ_F16: rc = launch_mv<DecDense<MSQ_F16>>(st, s, a); break;
    case MSQ_BF16: rc = launch_mv<DecDense<MSQ_BF16>>(st, s, a); break;
  }
  return rc == MSQ_ERR_UNSUPPORTED ? unsupported(what, t, rows, cols) : rc;
}

int msq_matvec(void* stream, int t, const MsqBuffer* W, int rows, int cols, const MsqBuffer* x, const MsqBuffer* y,
               int accumulate, int groups, const MsqMvCfg* cfg) {
  if (!mv_type_ok(t) || rows < 1 || cols < 1 || cols % mv_col_multiple(t) || groups < 1 || rows % groups)
    return unsupported("matvec", t, rows, cols);
  return matvec_impl(stream, "matvec", t, W, rows, cols, x, y, accumulate, groups, cfg, nullptr, 0.f);
}

int msq_matvec_rmsnorm(void* stream, int t, const MsqBuffer* W, int rows, int cols, const MsqBuffer* x, const MsqBuffer* norm_w,
                       float eps, const MsqBuffer* y, int tiles_per_tg) {
  (void)tiles_per_tg;  // the reference's amortisation knob for the norm prologue; workgroups here are persistent
  if (!mv_type_ok(t) || t == MSQ_IQ1_S || t == MSQ_IQ2_XXS || rows < 1 || cols < 1 || cols % mv_col_multiple(t))
    return unsupported("matvec_rmsnorm", t, rows, cols);
  if (!buf_ok(norm_w, (size_t)cols * 4))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: matvec_rmsnorm: norm weights missing or too small (cols %d)", cols);
  return matvec_impl(stream, "matvec_rmsnorm", t, W, rows, cols, x, y, 0, 1, nullptr, (const float*)bptr(norm_w), eps);
}

int msq_rmsnorm(void* stream, const MsqBuffer* x, const MsqBuffer* w, const MsqBuffer* y, int rows, int dim, float eps,
                int in_stride, int out_stride) {
  if (rows < 0 || dim < 1 || (in_stride && in_stride < dim) || (out_stride && out_stride < dim))
    return unsupported("rmsnorm", MSQ_F32, rows, dim);
  if (rows == 0) return MSQ_OK;
  const int is = in_stride ? in_stride : dim, os = out_stride ? out_stride : dim;
  const bool has_w = w && w->dev;
  if (!buf_ok(x, ((size_t)(rows - 1) * is + dim) * 4) || !buf_ok(y, ((size_t)(rows - 1) * os + dim) * 4) ||
      (has_w && !buf_ok(w, (size_t)dim * 4)))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: rmsnorm: buffer missing or too small (rows %d dim %d)", rows, dim);
  hipLaunchKernelGGL(rmsnorm_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, (const float*)bptr(x),
                     has_w ? (const float*)bptr(w) : nullptr, (float*)bptr_mut(y), (uint32_t)dim, eps, (uint32_t)is, (uint32_t)os);
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

int msq_bw_probe(void* stream, const MsqBuffer* src, size_t bytes, const MsqBuffer* sink) {
  if (!buf_ok(src, bytes) || !buf_ok(sink, 4096) || bytes % 16 || ((uintptr_t)bptr(src) & 15))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: bw_probe: buffer missing, too small or misaligned");
  if (bytes == 0) return MSQ_OK;
  const size_t n16 = bytes / 16;
  const long grid = std::min<long>((long)((n16 + 1023) / 1024), (long)device_info().cus * 2);
  hipLaunchKernelGGL(bw_probe_kernel, dim3((unsigned)grid), dim3(1024), 0, (hipStream_t)stream, (const uint4*)bptr(src), n16,
                     (uint32_t*)bptr_mut(sink));
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

int msq_dequant(void* stream, int t, const MsqBuffer* W, int64_t n, const MsqBuffer* out) {
  const int be = msq_type_block_elems(t);
  if (!be || n < 0 || n % be || n % 8) return unsupported("dequant", t, 0, (int)n);
  if (n == 0) return MSQ_OK;
  if (!buf_ok(W, msq_type_row_bytes(t, n)) || !buf_ok(out, (size_t)n * 4))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: dequant: buffer missing or too small");
  const uint8_t* src = bptr(W);
  float* dst = (float*)bptr_mut(out);
  const int64_t nchunks = n / 8;
  const dim3 grid((unsigned)((nchunks + 255) / 256)), block(256);
  hipStream_t st = (hipStream_t)stream;
  switch (t) {
#define MSQ_DEQ(T) case T: hipLaunchKernelGGL((dequant_kernel<T>), grid, block, 0, st, src, dst, nchunks); break;
    MSQ_DEQ(MSQ_F32) MSQ_DEQ(MSQ_F16) MSQ_DEQ(MSQ_BF16) MSQ_DEQ(MSQ_Q8_0) MSQ_DEQ(MSQ_IQ4_NL) MSQ_DEQ(MSQ_IQ1_S)
    MSQ_DEQ(MSQ_IQ2_XXS) MSQ_DEQ(MSQ_Q6_K) MSQ_DEQ(MSQ_Q5_K)
#undef MSQ_DEQ
    default: return unsupported("dequant", t, 0, (int)n);
  }
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

}  // extern "C"
