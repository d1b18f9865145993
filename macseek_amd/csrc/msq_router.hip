// C ABI: MoE router (top-6 selection) and the expert-sorted routing lists the prefill grouped GEMM consumes
// (see include/msq.h; reference host code src/kernels/arch.hpp:79-97, kernels src/kernels/arch_router.metal:26-183,
// CPU twin tests/ref/arch_ref.cpp:97-130).
//
// score = sqrt(softplus(logit)), key = score + bias, the six experts with the largest keys (ties: lowest id), weight =
// score / (sum of the six scores + 1e-20) * route_scale. The scores are computed in double precision and rounded where
// the reference's CPU twin rounds (fp64 runs at a quarter of the fp32 rate on this device and a token has 384 experts),
// so expert ids and weights repeat that twin's bits rather than being close to them.
#include <algorithm>

#include "msq_device.cuh"
#include "msq_host.h"

namespace msq {
namespace {

constexpr int kTopK = MSQ_MAX_ROUTED;
constexpr int kMaxEpl = 8;  // experts per lane: n_exp <= 512

// Wave-wide maximum / minimum, returned in every lane: the DPP steps of wave_sum with the lane's own value standing in
// where a step has no source lane.
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_fmax(float v) {
  const int b = __builtin_bit_cast(int, v);
  return fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, CTRL, ROW_MASK, 0xF, false)));
}
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ int dpp_imin(int v) {
  return min(v, __builtin_amdgcn_update_dpp(v, v, CTRL, ROW_MASK, 0xF, false));
}
__device__ __forceinline__ float wave_max_f(float v) {
  v = dpp_fmax<0xB1>(v); v = dpp_fmax<0x4E>(v); v = dpp_fmax<0x141>(v); v = dpp_fmax<0x140>(v);
  v = dpp_fmax<0x142, 0xA>(v); v = dpp_fmax<0x143, 0xC>(v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ int wave_min_i(int v) {
  v = dpp_imin<0xB1>(v); v = dpp_imin<0x4E>(v); v = dpp_imin<0x141>(v); v = dpp_imin<0x140>(v);
  v = dpp_imin<0x142, 0xA>(v); v = dpp_imin<0x143, 0xC>(v);
  return __builtin_amdgcn_readlane(v, 63);
}

struct alignas(16) RouterRec { double score; float key; float logit; };

// score and key of one expert, rounded where the reference's CPU twin rounds (tests/ref/arch_ref.cpp:100-105)
__device__ __forceinline__ void score_key(float logit, float bias, double& sc, float& key) {
  const double x = (double)logit;
  const double sp = x > 20.0 ? x : log1p(exp(x));
  sc = sqrt(sp);
  key = (float)sc + bias;
}

// One wave selects the top six experts of one token from the keys and scores its lanes hold (lane l: experts l + 64 i)
// and writes ids / weights.
__device__ __forceinline__ void select6(float (&key)[kMaxEpl], const double (&sc)[kMaxEpl], uint32_t epl, float route_scale,
                                        uint32_t lane, int* __restrict__ ids, float* __restrict__ wts) {
  int sel_e[kTopK];
  double sel_s[kTopK];
  double sum = 0.0;  // the six scores are added in selection order, as the reference adds them
#pragma unroll
  for (int k = 0; k < kTopK; k++) {
    float bk = -INFINITY;
    double bs = 0.0;
    int be = 0x7fffffff;
#pragma unroll
    for (uint32_t i = 0; i < kMaxEpl; i++)  // ascending expert id, strict comparison: the lane's lowest id among equals
      if (i < epl && key[i] > bk) { bk = key[i]; bs = sc[i]; be = (int)(lane + 64u * i); }
    const float m = wave_max_f(bk);
    const int win = wave_min_i(bk == m ? be : 0x7fffffff);
    if (win == 0x7fffffff) {  // fewer than six comparable keys (NaN logits): expert 0 with weight 0
      sel_e[k] = 0;
      sel_s[k] = 0.0;
      continue;
    }
#pragma unroll
    for (uint32_t i = 0; i < kMaxEpl; i++)
      if ((int)(lane + 64u * i) == win) key[i] = -INFINITY;
    const int src = __builtin_amdgcn_readfirstlane(win) & 63;  // the winner's lane holds its score in bs
    const uint64_t bits = __builtin_bit_cast(uint64_t, bs);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)bits, src);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(bits >> 32), src);
    sel_e[k] = win;
    sel_s[k] = __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
    sum += sel_s[k];
  }
  if (lane < (uint32_t)kTopK) {
#pragma unroll
    for (int k = 0; k < kTopK; k++)
      if (lane == (uint32_t)k) { ids[k] = sel_e[k]; wts[k] = (float)(sel_s[k] / (sum + 1e-20) * (double)route_scale); }
  }
}

// logits [n][n_exp] -> ids [n][6], weights [n][6]; one wave per token, four per workgroup.
__global__ __launch_bounds__(256) void router_topk_kernel(const float* __restrict__ logits, const float* __restrict__ bias,
                                                          int* __restrict__ ids, float* __restrict__ wts, uint32_t n_tokens,
                                                          uint32_t n_exp, float route_scale) {
  const uint32_t lane = threadIdx.x & 63u, t = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (t >= n_tokens) return;  // whole waves leave; no barrier follows
  const float* row = logits + (size_t)t * n_exp;
  const uint32_t epl = n_exp >> 6;
  double sc[kMaxEpl];
  float key[kMaxEpl];
#pragma unroll
  for (uint32_t i = 0; i < kMaxEpl; i++) {
    sc[i] = 0.0;
    key[i] = -INFINITY;
    if (i < epl) score_key(row[lane + 64u * i], bias[lane + 64u * i], sc[i], key[i]);
  }
  select6(key, sc, epl, route_scale, lane, ids + (size_t)t * kTopK, wts + (size_t)t * kTopK);
}

// Decode: logits = W[n_exp][dim] . x[dim] and the selection in one launch. A workgroup is four waves, each taking one
// expert row and leaving the expert's logit, score and key in scratch; the workgroup that finishes last (device-scope
// counter, one increment per workgroup: n_exp / 4 of them contend, not n_exp) selects from the keys, then re-arms the
// counter. W is F32 (QT = MSQ_F32) or BF16. No bit of the result depends on which workgroup is last.
template <int QT>
__global__ __launch_bounds__(256) void router_fused_kernel(const float* __restrict__ x, const void* __restrict__ W, uint32_t dim,
                                                           uint32_t n_exp, const float* __restrict__ bias, float* logits,
                                                           RouterRec* recs, uint32_t* counter, int* __restrict__ ids,
                                                           float* __restrict__ wts, float route_scale) {
  __shared__ uint32_t last;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, e = blockIdx.x * 4u + wave;
  // the row's weights are requested U vectors per lane at a time before any is used: with one wave per row the loop is
  // otherwise a chain of memory latencies
  constexpr uint32_t U = 8;
  float acc = 0.f;
  if constexpr (QT == MSQ_F32) {
    const float4* wr = (const float4*)((const float*)W + (size_t)e * dim);
    const float4* xv = (const float4*)x;
    const uint32_t nv = dim / 4u;
    for (uint32_t c0 = 0; c0 < nv; c0 += 64u * U) {
      float4 a[U], b[U];
#pragma unroll
      for (uint32_t u = 0; u < U; u++) { const uint32_t c = min(c0 + 64u * u + lane, nv - 1u); a[u] = wr[c]; b[u] = xv[c]; }
#pragma unroll
      for (uint32_t u = 0; u < U; u++)
        if (c0 + 64u * u + lane < nv) acc += a[u].x * b[u].x + a[u].y * b[u].y + a[u].z * b[u].z + a[u].w * b[u].w;
    }
  } else {
    const uint4* wr = (const uint4*)((const uint16_t*)W + (size_t)e * dim);
    const float4* xv = (const float4*)x;
    const uint32_t nv = dim / 8u;
    for (uint32_t c0 = 0; c0 < nv; c0 += 64u * U) {
      uint4 a[U];
      float4 b0[U], b1[U];
#pragma unroll
      for (uint32_t u = 0; u < U; u++) {
        const uint32_t c = min(c0 + 64u * u + lane, nv - 1u);
        a[u] = wr[c]; b0[u] = xv[2 * c]; b1[u] = xv[2 * c + 1];
      }
#pragma unroll
      for (uint32_t u = 0; u < U; u++)
        if (c0 + 64u * u + lane < nv)
          acc += __builtin_bit_cast(float, a[u].x << 16) * b0[u].x + __builtin_bit_cast(float, a[u].x & 0xFFFF0000u) * b0[u].y +
                 __builtin_bit_cast(float, a[u].y << 16) * b0[u].z + __builtin_bit_cast(float, a[u].y & 0xFFFF0000u) * b0[u].w +
                 __builtin_bit_cast(float, a[u].z << 16) * b1[u].x + __builtin_bit_cast(float, a[u].z & 0xFFFF0000u) * b1[u].y +
                 __builtin_bit_cast(float, a[u].w << 16) * b1[u].z + __builtin_bit_cast(float, a[u].w & 0xFFFF0000u) * b1[u].w;
    }
  }
  const float v = wave_sum(acc);
  if (lane == 0) {
    double sc;
    float key;
    score_key(v, bias[e], sc, key);
    // Hand-over to the selecting workgroup. Writer side: the three results are device-scope atomic stores (they are
    // written through to the level of the memory system that all XCDs share, never parked in this XCD's L2), the
    // wave waits until the memory system has acknowledged them (vmcnt(0)), and only then, after the workgroup
    // barrier, is the counter incremented: a store that is acknowledged is visible to every device-scope load, so no
    // record can be observed older than the count that announces it. This is the effect of a release fence without its
    // price: a device-scope release writes back the whole L2 of this workgroup's XCD (measured: the launch takes
    // 19 us with plain stores and a fence, 15 us with atomic stores and a fence, less without the fence). Reader side:
    // the workgroup that draws the last count passes an acquire fence (cheap: it drops cached lines, writes nothing)
    // and reads the records with device-scope atomic loads.
    uint64_t* r = (uint64_t*)(recs + e);
    __hip_atomic_store(logits + e, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(r, __builtin_bit_cast(uint64_t, sc), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(r + 1, (uint64_t)__builtin_bit_cast(uint32_t, key) | ((uint64_t)__builtin_bit_cast(uint32_t, v) << 32),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __syncthreads();
  if (tid == 0) {
    const uint32_t prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = prev == gridDim.x - 1u ? 1u : 0u;
  }
  __syncthreads();
  if (!last) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  // Selection in two levels. Six rounds of "wave-wide best, then remove it" by one wave over all experts is a chain of
  // twelve DPP reductions plus a six-way local maximum per round, run by a wave that has its SIMD to itself: 3 us.
  // Here each of the four waves picks the six best of its quarter of the experts (two per lane at most: the local
  // maximum is one comparison), leaves them in LDS, and wave 0 picks the six best of those 24 (one per lane). The six
  // best overall are among the six best of their quarters, and "greater key, then lower expert id" is a total order, so
  // the result is the one-level selection's.
  __shared__ float c_key[4 * kTopK];
  __shared__ int c_id[4 * kTopK];
  __shared__ double c_sc[4 * kTopK];
  const uint32_t quarter = n_exp >> 2;  // experts of this wave: quarter * wave + {lane, lane + 64}
  {
    float key[2];
    double sc[2];
#pragma unroll
    for (uint32_t i = 0; i < 2; i++) {
      key[i] = -INFINITY;
      sc[i] = 0.0;
      if (lane + 64u * i < quarter) {  // device-scope loads: the records were written by other CUs during this launch
        const uint64_t* r = (const uint64_t*)(recs + quarter * wave + lane + 64u * i);
        const uint64_t s64 = __hip_atomic_load(r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint64_t k64 = __hip_atomic_load(r + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sc[i] = __builtin_bit_cast(double, s64);
        key[i] = __builtin_bit_cast(float, (uint32_t)k64);
      }
    }
#pragma unroll
    for (int k = 0; k < kTopK; k++) {
      // the lane's best: strict comparisons from -inf up, so NaN and -inf keys are never candidates and the lower id
      // wins among equals
      float bk = -INFINITY;
      bool second = false, any = false;
      if (key[0] > bk) { bk = key[0]; any = true; }
      if (key[1] > bk) { bk = key[1]; second = true; any = true; }
      const int be = any ? (int)(quarter * wave + lane + (second ? 64u : 0u)) : 0x7fffffff;
      const float m = wave_max_f(bk);
      const int win = wave_min_i(bk == m ? be : 0x7fffffff);
      if (win != 0x7fffffff && be == win) {  // one lane
        c_key[wave * kTopK + k] = bk;
        c_id[wave * kTopK + k] = win;
        c_sc[wave * kTopK + k] = second ? sc[1] : sc[0];
        if (second) key[1] = -INFINITY; else key[0] = -INFINITY;
      }
      if (win == 0x7fffffff && lane == 0) { c_key[wave * kTopK + k] = -INFINITY; c_id[wave * kTopK + k] = 0x7fffffff; c_sc[wave * kTopK + k] = 0.0; }
    }
  }
  __syncthreads();
  if (wave == 0) {
    float ck = lane < 4u * kTopK ? c_key[lane] : -INFINITY;
    const int ce = lane < 4u * kTopK ? c_id[lane] : 0x7fffffff;
    const double cs = lane < 4u * kTopK ? c_sc[lane] : 0.0;
    int sel_e[kTopK];
    double sel_s[kTopK];
    double sum = 0.0;  // the six scores are added in selection order, as the reference adds them
#pragma unroll
    for (int k = 0; k < kTopK; k++) {
      const float m = wave_max_f(ck);
      const int win = wave_min_i((ck == m && ce != 0x7fffffff) ? ce : 0x7fffffff);
      if (win == 0x7fffffff) {  // fewer than six comparable keys (NaN logits): expert 0 with weight 0
        sel_e[k] = 0;
        sel_s[k] = 0.0;
        continue;
      }
      const uint64_t holder = __builtin_amdgcn_ballot_w64(ce == win);
      const int src = (int)__builtin_ctzll(holder);
      if (ce == win) ck = -INFINITY;
      const uint64_t bits = __builtin_bit_cast(uint64_t, cs);
      const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)bits, src);
      const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(bits >> 32), src);
      sel_e[k] = win;
      sel_s[k] = __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
      sum += sel_s[k];
    }
    if (lane < (uint32_t)kTopK) {
#pragma unroll
      for (int k = 0; k < kTopK; k++)
        if (lane == (uint32_t)k) { ids[k] = sel_e[k]; wts[k] = (float)(sel_s[k] / (sum + 1e-20) * (double)route_scale); }
    }
    if (lane == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Routing lists: one wave per expert e. A first pass over the ids counts the entries of lower experts (the expert's
// offset) and its own; a second pass writes its entries in entry order, positions from ballots. No atomics: the
// lists are the same on every run, sorted by (expert, entry index).
__global__ __launch_bounds__(256) void route_lists_kernel(const int* __restrict__ ids, const float* __restrict__ w,
                                                          uint32_t n_entries, uint32_t n_exp, uint32_t* __restrict__ counts,
                                                          uint32_t* __restrict__ offsets, uint32_t* __restrict__ entry,
                                                          uint32_t* __restrict__ tok, float* __restrict__ lw,
                                                          uint32_t* __restrict__ slot_of) {
  const uint32_t lane = threadIdx.x & 63u;
  const int e = (int)(blockIdx.x * 4u + (threadIdx.x >> 6));
  if (e >= (int)n_exp) return;  // whole waves leave; no barrier follows
  constexpr uint32_t U = 16;  // ids fetched per lane before they are used: the loop is bound by load latency otherwise
  uint32_t lt = 0, eq = 0;
  for (uint32_t i0 = 0; i0 < n_entries; i0 += 64u * U) {
    int id[U];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      const uint32_t i = i0 + 64u * u + lane;
      id[u] = ids[min(i, n_entries - 1u)];
      if (i >= n_entries) id[u] = -1;
    }
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      lt += (id[u] >= 0 && id[u] < e) ? 1u : 0u;
      eq += id[u] == e ? 1u : 0u;
    }
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) { lt += __shfl_xor(lt, m, 64); eq += __shfl_xor(eq, m, 64); }
  if (lane == 0) {
    counts[e] = eq;
    offsets[e] = lt;
    if (e == (int)n_exp - 1) offsets[n_exp] = lt + eq;
  }
  if (eq == 0) return;
  uint32_t base = lt;
  const uint64_t below = (1ull << lane) - 1ull;
  for (uint32_t i0 = 0; i0 < n_entries; i0 += 64u * U) {
    int id[U];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      const uint32_t i = i0 + 64u * u + lane;
      id[u] = ids[min(i, n_entries - 1u)];
      if (i >= n_entries) id[u] = -1;
    }
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      const uint32_t i = i0 + 64u * u + lane;
      const bool m = id[u] == e;
      const uint64_t bits = __ballot(m);
      if (m) {
        const uint32_t pos = base + (uint32_t)__popcll(bits & below);
        entry[pos] = i;
        tok[pos] = i / (uint32_t)kTopK;
        lw[pos] = w[i];
        slot_of[i] = pos;
      }
      base += (uint32_t)__popcll(bits);
    }
  }
}

bool exp_ok(int n_exp) { return n_exp >= 64 && n_exp <= 64 * kMaxEpl && n_exp % 64 == 0; }

}  // namespace
}  // namespace msq

using namespace msq;

extern "C" {

int msq_router_topk(void* stream, const MsqBuffer* logits, const MsqBuffer* bias, const MsqBuffer* ids, const MsqBuffer* w,
                    int n_tokens, int n_exp, float route_scale) {
  if (!exp_ok(n_exp) || n_tokens < 0) return unsupported("router_topk", MSQ_F32, n_tokens, n_exp);
  if (n_tokens == 0) return MSQ_OK;
  if (!buf_ok(logits, (size_t)n_tokens * n_exp * 4) || !buf_ok(bias, (size_t)n_exp * 4) ||
      !buf_ok(ids, (size_t)n_tokens * kTopK * 4) || !buf_ok(w, (size_t)n_tokens * kTopK * 4))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: router_topk: buffer missing or too small (tokens %d experts %d)", n_tokens, n_exp);
  hipLaunchKernelGGL(router_topk_kernel, dim3((unsigned)((n_tokens + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                     (const float*)bptr(logits), (const float*)bptr(bias), (int*)bptr_mut(ids), (float*)bptr_mut(w),
                     (uint32_t)n_tokens, (uint32_t)n_exp, route_scale);
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

// scratch: logits f32 [n_exp] (padded to 256 bytes), {score f64, key f32, logit f32} [n_exp], then the counter in a
// 256-byte line of its own
size_t msq_router_scratch_bytes(int n_exp) { return ((size_t)n_exp * 4 + 255) / 256 * 256 + (size_t)n_exp * 16 + 256; }

int msq_router_fused(void* stream, int wtype, const MsqBuffer* x, const MsqBuffer* W, const MsqBuffer* bias,
                     const MsqBuffer* scratch, const MsqBuffer* ids, const MsqBuffer* w, int dim, int n_exp, float route_scale) {
  if (!exp_ok(n_exp) || dim < 8 || dim % 8 || (wtype != MSQ_F32 && wtype != MSQ_BF16)) return unsupported("router_fused", wtype, n_exp, dim);
  const size_t esz = wtype == MSQ_F32 ? 4 : 2;
  if (!buf_ok(x, (size_t)dim * 4) || !buf_ok(W, (size_t)n_exp * dim * esz) || !buf_ok(bias, (size_t)n_exp * 4) ||
      !buf_ok(ids, kTopK * 4) || !buf_ok(w, kTopK * 4) || ((uintptr_t)bptr(x) & 15) || ((uintptr_t)bptr(W) & 15))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: router_fused: buffer missing, too small or not 16-byte aligned (experts %d dim %d)", n_exp, dim);
  if (!buf_ok(scratch, msq_router_scratch_bytes(n_exp)) || ((uintptr_t)bptr(scratch) & 15))
    return fail(MSQ_ERR_SCRATCH, "macseek quant: router_fused scratch too small unsupported (type %s rows %d cols %d)",
                msq_type_name_of(wtype), n_exp, dim);
  float* logits = (float*)bptr_mut(scratch);
  RouterRec* recs = (RouterRec*)(bptr_mut(scratch) + ((size_t)n_exp * 4 + 255) / 256 * 256);
  uint32_t* counter = (uint32_t*)(bptr_mut(scratch) + msq_router_scratch_bytes(n_exp) - 256);
  const dim3 grid((unsigned)(n_exp / 4)), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (wtype == MSQ_F32)
    hipLaunchKernelGGL((router_fused_kernel<MSQ_F32>), grid, block, 0, st, (const float*)bptr(x), (const void*)bptr(W),
                       (uint32_t)dim, (uint32_t)n_exp, (const float*)bptr(bias), logits, recs, counter, (int*)bptr_mut(ids),
                       (float*)bptr_mut(w), route_scale);
  else
    hipLaunchKernelGGL((router_fused_kernel<MSQ_BF16>), grid, block, 0, st, (const float*)bptr(x), (const void*)bptr(W),
                       (uint32_t)dim, (uint32_t)n_exp, (const float*)bptr(bias), logits, recs, counter, (int*)bptr_mut(ids),
                       (float*)bptr_mut(w), route_scale);
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

int msq_route_lists(void* stream, const MsqBuffer* ids, const MsqBuffer* w, int n_tokens, int n_exp, const MsqRouteLists* L) {
  if (n_exp < 1 || n_tokens < 0 || !L) return unsupported("route_lists", MSQ_F32, n_tokens, n_exp);
  const size_t n_entries = (size_t)n_tokens * kTopK;
  if (n_tokens > L->max_tokens || n_entries >= (1ull << 31))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: route_lists: %d tokens exceed the lists' capacity of %d", n_tokens, L->max_tokens);
  if (!buf_ok(&L->counts, (size_t)n_exp * 4) || !buf_ok(&L->offsets, (size_t)(n_exp + 1) * 4))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: route_lists: counts / offsets missing or too small (experts %d)", n_exp);
  if (n_tokens > 0 && (!buf_ok(ids, n_entries * 4) || !buf_ok(w, n_entries * 4) || !buf_ok(&L->entry, n_entries * 4) ||
                       !buf_ok(&L->tok, n_entries * 4) || !buf_ok(&L->w, n_entries * 4) || !buf_ok(&L->slot_of, n_entries * 4)))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: route_lists: buffer missing or too small (tokens %d)", n_tokens);
  hipLaunchKernelGGL(route_lists_kernel, dim3((unsigned)((n_exp + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                     n_tokens ? (const int*)bptr(ids) : nullptr, n_tokens ? (const float*)bptr(w) : nullptr, (uint32_t)n_entries,
                     (uint32_t)n_exp, (uint32_t*)bptr_mut(&L->counts), (uint32_t*)bptr_mut(&L->offsets),
                     n_tokens ? (uint32_t*)bptr_mut(&L->entry) : nullptr, n_tokens ? (uint32_t*)bptr_mut(&L->tok) : nullptr,
                     n_tokens ? (float*)bptr_mut(&L->w) : nullptr, n_tokens ? (uint32_t*)bptr_mut(&L->slot_of) : nullptr);
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}

}  // extern "C"
