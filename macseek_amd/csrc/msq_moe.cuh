// Fused batch-1 MoE layer (reference operators: ms::q::encode_moe_decode / _table / _table_part,
// src/kernels/quant.mm:266-369; reference kernels q_moe_gu / q_moe_down, src/kernels/quant_moe.metal:50-147):
//   moe_gu_kernel  : h[e][r] = silu(min(gate_e[r].x, 10)) * clamp(up_e[r].x, -10, 10) * w_e   for all experts
//   moe_down_kernel: y[r] += sum_e down_e[r] . h[e]   (routed experts in slot order, then the shared expert)
// Expert e < n_routed is a routed expert (decoder DR); the shared expert (decoder DS, weight 1) keeps its h row at
// index n_routed. Expert matrices are reached either through pointers passed by value or through a device-resident
// table of 6 x {gate, up, down} 64-bit addresses that the host may fill after the launch was enqueued.
//
// Both kernels are persistent: about one 16-wave workgroup per CU, so the codebook tables are staged into LDS and the
// activations into registers once per CU. Every wave owns a contiguous run of rows and a fixed K slice, streams its
// rows with the next group's loads in flight while the current group is decoded, and parks per-row partial sums in
// LDS; a workgroup synchronises only once per chunk of rows, to add the K-split / per-expert partials in a fixed
// order and run the epilogue.
#pragma once
#include <type_traits>

#include "msq_device.cuh"
#include "msq_iq1s.cuh"
#include "msq_iq2xxsq.cuh"
#include "msq_q6kq.cuh"

namespace msq {

constexpr int kMaxRouted = 6;
constexpr int kMoeChunkRows = 128;  // rows a workgroup finishes between two synchronisations
// The down kernel multiplies h by this power of two before it is rounded to fp16 pairs and divides the row sums by it:
// |h| <= 100 |w| (the clamps of SwiGLU), so routing weights up to 5 keep 128 h inside the fp16 range, and h down to
// 5e-7 stays out of its denormals.
constexpr float kHScale = 128.f;

// Field order: the scalar cache fetches the argument block line by line (64 bytes), one miss after the other, so what
// a kernel needs before its first weight row can be requested sits together at the front -- gate/up finds it in the
// first line (the block starts 8 bytes into the segment, behind the table address), down in the first two -- and the
// by-value expert addresses, unused when a table is passed, at the end.
struct MoeArgs {
  const float* x;        // [dim]
  uint32_t dim, inter;
  uint32_t ks;           // K-split waves
  uint32_t n_routed;     // h row of the shared expert
  uint32_t run_routed;   // experts this launch computes: routed ones (0 or 1) ...
  uint32_t run_shared;   // ... and / or the shared one
  // activations staged through LDS (padded rows of XLds): word offset in dynamic LDS, or read straight from device
  // memory when stage_x is 0 (rows too long for LDS)
  uint32_t xs_off, stage_x;
  uint32_t grid_routed;  // gate/up: workgroups [0, grid_routed) take routed rows, the rest shared rows
  uint32_t rows_per_wg_r, rb_gu_r, rows_per_wg_s;  // gate/up: virtual rows (expert * inter + row) per workgroup; row bytes
  uint32_t rb_gu_s;      // row bytes: shared gate/up
  uint32_t rows_per_wg;  // down: rows of y per workgroup
  uint32_t rb_d_r, rb_d_s;  // row bytes: routed down, shared down
  const uint8_t* sdown;
  float* y;              // [dim], accumulated
  // Second copy of h as fp16, scaled by kHScale and rounded by the gate/up kernel: the form in which the down kernel's
  // X32 decoders multiply it (half the bytes for every workgroup of the down kernel to stage, and no conversion there).
  // Null when the down kernel's decoder pair does not read it (kHalfH).
  _Float16* h16;
  float* h;              // scratch: [(n_routed + 1)][inter]
  const uint8_t *sgate, *sup;
  const float* wts;      // [n_routed] routing weights (device memory)
  const uint64_t* table; // kMaxRouted x {gate, up, down} device addresses, or null to use the arrays below
  const uint8_t* gate[kMaxRouted];
  const uint8_t* up[kMaxRouted];
  const uint8_t* down[kMaxRouted];
};

// h value i of the layer: fp32 for the caller's eyes, and the fp16 form that the down kernel would otherwise make of it
__device__ __forceinline__ void store_h(const MoeArgs& a, size_t i, float v) {
  a.h[i] = v;
  if (a.h16) a.h16[i] = (_Float16)(v * kHScale);
}
// Whether the down kernel with decoders DR / DS reads h in the fp16 form (a property of the decoder pair, so that the
// kernel holds one form only; the host passes MoeArgs::h16 by the same rule).
template <class DR, class DS>
constexpr bool kHalfH = std::is_same_v<typename DR::X, X32> && std::is_same_v<typename DS::X, X32>;
// the lane's slice (unit u) of the h row that starts at column col0 of the staged rows hs / of the rows in device memory
template <class D, bool HALF, bool ROT = false>
__device__ __forceinline__ typename D::X load_h_staged(const uint32_t* hs, uint32_t col0, uint32_t u) {
  if constexpr (HALF && ROT) return load_x32_half_rot(hs, (col0 >> 5) + u);
  else if constexpr (HALF) return load_x32_half(hs + xhalf_words(col0) + 20u * u);
  else return D::load_x(XLds{(const float*)hs + xlds_words(col0)}, u, kHScale);
}
template <class D, bool HALF>
__device__ __forceinline__ typename D::X load_h_direct(const MoeArgs& a, uint32_t col0, uint32_t u) {
  if constexpr (HALF) return load_x32_half((const uint32_t*)a.h16 + (col0 >> 1) + 16u * u);
  else return D::load_x(a.h + col0, u, kHScale);
}

__device__ __forceinline__ float swiglu(float g, float u, float w) {  // quant_moe.metal:23-27
  g = fminf(g, 10.f);
  u = fminf(fmaxf(u, -10.f), 10.f);
  return g / (1.f + expf(-g)) * u * w;
}

// the register batch in which a decoder with quantized activations holds its table items between request and store
template <class D> struct TblRegsOf { struct type {}; };
template <class D> requires requires { typename D::TblRegs; } struct TblRegsOf<D> { using type = typename D::TblRegs; };

// Rows a wave keeps in flight per prefetch group: as many as fit about 24 registers of raw block bytes per buffer.
template <class D>
constexpr int rows_in_flight(int matrices) {
  const int words = (int)(sizeof(typename D::Raw) / 4) * matrices;
  return words <= 6 ? 4 : words <= 12 ? 2 : 1;
}

// 32-bit words of LDS that the staged activations of a row of `cols` columns take for decoder D
template <class D>
__host__ __device__ constexpr uint32_t x_stage_words(uint32_t cols) {
  if constexpr (requires { D::QUANT_X; }) return xq_words(cols);
  else return xlds_words(cols);
}
// the lane's activation slice of unit u from a staged row (at word offset `at` of `base`), or from device memory
template <class D>
__device__ __forceinline__ typename D::X load_x_staged(const uint32_t* base, uint32_t u) {
  if constexpr (requires { D::QUANT_X; }) return D::load_x(XQLds{base}, u);
  else return D::load_x(XLds{(const float*)base}, u);
}

// Entry i of the expert address table, read through the scalar cache (the index is wave-uniform): one request per wave
// instead of one per lane, and its result does not queue behind the vector loads in flight.
__device__ __forceinline__ const void* table_entry(const uint64_t* table, uint32_t i) {
  typedef const __attribute__((address_space(4))) uint64_t* cptr_t;
  return (const void*)((cptr_t)(uintptr_t)table)[i];
}

__device__ __forceinline__ uint32_t uniform(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ const void* uniform(const void* p) {
  const uint64_t v = (uint64_t)p;
  return (const void*)((uint64_t)uniform((uint32_t)v) | ((uint64_t)uniform((uint32_t)(v >> 32)) << 32));
}

// gate + up + SwiGLU over the virtual rows [wg * per, ...) of one kind of expert (routed: e * inter + r; shared: r).
template <class D, int RPW>
__device__ __forceinline__ void moe_gu_run_direct(const MoeArgs& a, const uint64_t* table, uint32_t* tbl, uint32_t* smem, const bool shared, const uint32_t wg) {
  float* part = (float*)smem;
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = uniform(tid >> 6), nwaves = blockDim.x >> 6;
  const uint32_t KS = a.ks, ks = wave % KS, rw = wave / KS, RW = nwaves / KS;
  const uint32_t units = a.dim / D::UNIT;
  const uint32_t row_bytes = shared ? a.rb_gu_s : a.rb_gu_r;
  const uint32_t total = (shared ? 1u : a.n_routed) * a.inter;
  const uint32_t per = shared ? a.rows_per_wg_s : a.rows_per_wg_r;
  const uint32_t wg_begin = wg * per, wg_end = min(total, wg_begin + per);

  const uint32_t u0 = ks * 64u + lane;
  const bool valid = u0 < units;
  const uint32_t unit = valid ? u0 : units - 1;
  const uint32_t PSTRIDE = 4 * KS + 1;  // partial sums per (row, matrix): 4 sixteen-lane rows per K-split wave, padded

  // address of virtual row v of the gate (which = 0) or up (1) matrices
  auto row_ptr = [&](uint32_t v, int which) -> gptr_t {
    const uint32_t e = shared ? 0u : v / a.inter, r = v - e * a.inter;
    const uint8_t* base;
    if (shared) base = which ? a.sup : a.sgate;
    else if (table) base = (const uint8_t*)table[3 * e + which];
    else base = which ? a.up[e] : a.gate[e];
    return as_global(base) + (size_t)r * row_bytes;
  };

  typename D::X xr;
  bool first = true;
  for (uint32_t c0 = wg_begin; c0 < wg_end; c0 += kMoeChunkRows) {
    const uint32_t c1 = min(wg_end, c0 + kMoeChunkRows), n = c1 - c0;
    // rows of this chunk are dealt to the row-waves in contiguous runs
    const uint32_t run = (n + RW - 1) / RW;
    const uint32_t w0 = min(c0 + rw * run, c1), w1 = min(w0 + run, c1);
    typename D::Raw cg[RPW], cu[RPW], ng[RPW], nu[RPW];
    if (w0 < w1) {
#pragma unroll
      for (int j = 0; j < RPW; j++) {
        const uint32_t v = min(w0 + j, w1 - 1);
        cg[j] = D::load(row_ptr(v, 0), unit);
        cu[j] = D::load(row_ptr(v, 1), unit);
      }
    }
    if (first) {  // tables and activations arrive while the first weight rows are in flight
      if constexpr (requires { D::QUANT_X; }) {  // quantized activations (no table)
        if (a.stage_x) {
          stage_xq<2>(smem + a.xs_off, a.x, a.dim, tid, blockDim.x);
          __syncthreads();
          xr = D::load_x(XQLds{smem + a.xs_off}, unit);
        } else {
          xr = D::load_x(a.x, unit);
          __syncthreads();
        }
      } else {
        const CopyJob jobs[3] = {tbl_job_of<D>(0, 0u, true), tbl_job_of<D>(1, 0u, true),
                                 {(const uint4*)a.x, (uint32_t)(smem - tbl) + a.xs_off, a.stage_x ? a.dim / 4u : 0u, 3u}};
        copy_jobs<4>(tbl, jobs, tid, blockDim.x);
        if (a.stage_x) {
          __syncthreads();
          xr = D::load_x(XLds{(const float*)(smem + a.xs_off)}, unit);
        } else {
          xr = D::load_x(a.x, unit);
          __syncthreads();
        }
      }
      first = false;
    }
    for (uint32_t r0 = w0; r0 < w1; r0 += RPW) {
      const bool more = r0 + RPW < w1;
      if (more) {
#pragma unroll
        for (int j = 0; j < RPW; j++) {
          const uint32_t v = min(r0 + RPW + j, w1 - 1);
          ng[j] = D::load(row_ptr(v, 0), unit);
          nu[j] = D::load(row_ptr(v, 1), unit);
        }
      }
      float acc[2 * RPW];  // value 2 j + m: row j of the group, m = 0 gate, 1 up
#pragma unroll
      for (int j = 0; j < RPW; j++) {
        const float g = dec_dot<D>(cg[j], xr, tbl, unit), u = dec_dot<D>(cu[j], xr, tbl, unit);
        acc[2 * j] = valid ? g : 0.f;
        acc[2 * j + 1] = valid ? u : 0.f;
        asm volatile("" ::: "memory");  // one row pair's table lookups live at a time (register pressure)
      }
      row16_fold<2 * RPW>(acc, lane);
      {
        const uint32_t k = group8_sel<2 * RPW>(lane), j = k >> 1, m = k & 1u;
        if (!(lane & 8u) && r0 + j < w1) part[((r0 + j - c0) * 2 + m) * PSTRIDE + ks * 4 + (lane >> 4)] = acc[0];
      }
      if (more) {
#pragma unroll
        for (int j = 0; j < RPW; j++) { cg[j] = ng[j]; cu[j] = nu[j]; }
      }
    }
    __syncthreads();
    // thread q sums the partials of (row q / 2, matrix q % 2); gate and up then meet in the even lane
    for (uint32_t q0 = 0; q0 < 2 * n; q0 += blockDim.x) {
      const uint32_t q = q0 + tid;
      float sum = 0.f;
      if (q < 2 * n) sum = sum_in_order(part + q * PSTRIDE, 4 * KS);
      const float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sum), 0xB1, 0xF, 0xF, false));
      if (q < 2 * n && !(q & 1u)) {
        const uint32_t v = c0 + (q >> 1);
        const uint32_t e = shared ? 0u : v / a.inter, r = v - e * a.inter;
        const uint32_t he = shared ? a.n_routed : e;
        store_h(a, (size_t)he * a.inter + r, swiglu(sum, other, shared ? 1.f : a.wts[e]));
      }
    }
    __syncthreads();
  }
}

// Same computation for the codebook decoders (those with lookup() / partial() stages), arranged for memory-level
// parallelism: a wave keeps the block bytes of NR row pairs in flight in a register ring -- a slot is refilled with the
// row pair NR places ahead as soon as its bytes have been consumed -- so that about NR x 2 x (slice of a row) bytes per
// wave are outstanding at any time, which is what it takes to keep HBM busy at batch 1. The refills are range-checked
// buffer loads issued unconditionally (an empty descriptor past the end of the wave's run), so every wait in the loop
// names an exact number of loads that may stay in flight. Table lookups run one decoder stage ahead of the dot
// products (two alternating lookup buffers), so LDS latency overlaps the math as well.
template <class D>
__device__ __forceinline__ void moe_gu_run_ring(const MoeArgs& a, const uint64_t* table, uint32_t* tbl, uint32_t* smem, const bool shared, const uint32_t wg) {
  constexpr int NR = 4;  // row pairs in flight per wave
  constexpr int NS = D::STAGES;
  float* part = (float*)smem;
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = uniform(tid >> 6), nwaves = blockDim.x >> 6;
  const uint32_t KS = a.ks, ks = wave % KS, rw = wave / KS, RW = nwaves / KS;
  const uint32_t PSTRIDE = 4 * KS + 1;
  const uint32_t units = a.dim / D::UNIT;
  const uint32_t row_bytes = shared ? a.rb_gu_s : a.rb_gu_r;
  const uint32_t mat_bytes = a.inter * row_bytes;
  const uint32_t total = (shared ? 1u : a.n_routed) * a.inter;
  const uint32_t per = shared ? a.rows_per_wg_s : a.rows_per_wg_r;
  const uint32_t wg_begin = wg * per, wg_end = min(total, wg_begin + per);

  const uint32_t u0 = ks * 64u + lane;
  const bool valid = u0 < units;
  const uint32_t unit = valid ? u0 : units - 1;  // lanes past the row shadow the last unit; their activations are zero
  const typename D::Off off = D::offsets(unit);

  typename D::X xr;
  bool first = true;
  // The loads of the prologue (grid items, activations) need nothing but kernel arguments: they are requested before
  // the expert addresses are looked up, and stored to LDS after the first weight rows have been requested.
  [[maybe_unused]] typename TblRegsOf<D>::type tr;
  [[maybe_unused]] XqBatch<2> xb;
  if constexpr (requires { D::QUANT_X; }) {
    tr = D::issue_tables(tid, blockDim.x);
    if (a.stage_x) xb = xq_issue<2>(a.x, a.dim >> 2, tid, blockDim.x);
  }
  for (uint32_t c0 = wg_begin; c0 < wg_end; c0 += kMoeChunkRows) {
    const uint32_t c1 = min(wg_end, c0 + kMoeChunkRows), n = c1 - c0;
    const uint32_t run = uniform((n + RW - 1) / RW);  // divisions run on the vector unit: bring the results back
    const uint32_t w0 = min(c0 + rw * run, c1), w1 = min(w0 + run, c1);

    // cursor of the next row pair to fetch: expert pe, row pr of it, matrix bases pg / pu (all wave-uniform)
    uint32_t pv = uniform(w0), pe = 0, pr = pv;
    const void *pg = nullptr, *pu = nullptr;
    auto set_expert = [&]() {
      if (shared) { pg = a.sgate; pu = a.sup; }
      else if (table) { pg = table_entry(table, 3 * pe); pu = table_entry(table, 3 * pe + 1); }
      else { pg = a.gate[pe]; pu = a.up[pe]; }
      pg = uniform(pg); pu = uniform(pu);  // buffer descriptors live in scalar registers
    };
    if (w0 < w1) {
      if (!shared) { pe = uniform(w0 / a.inter); pr = uniform(w0 - pe * a.inter); }
      set_expert();
    }
    typename D::Raw rg[NR], ru[NR];
    auto fetch = [&](int s) {  // loads of row pair pv into slot s (nothing is read once pv has passed w1), then advance
      const uint32_t bytes = pv < w1 ? mat_bytes : 0u;
      const uint32_t soff = pr * row_bytes;
      rg[s] = D::fetch(make_rsrc(pg, bytes), off, soff);
      ru[s] = D::fetch(make_rsrc(pu, bytes), off, soff);
      pv++; pr++;
      if (!shared && pr == a.inter && pv < w1) { pr = 0; pe++; set_expert(); }
    };
    // Half of the ring is requested before the tables and activations, the other half behind them: loads return in
    // order, so with the whole ring ahead the prologue's small reads wait for four row pairs, and with none ahead the
    // first rows start a memory trip late (gate/up of the one-token layer: 16.9 us with 4 or 0 pairs first, 16.6 / 16.4
    // with 3 / 1, 16.0 with 2)
#pragma unroll
    for (int s = 0; s < NR / 2; s++) fetch(s);
    if (first) {  // tables and activations arrive while the first weight rows are in flight
      if constexpr (requires { D::QUANT_X; }) {
        if (a.stage_x) {
          D::finish_tables(tbl, tr, tid, blockDim.x);
          stage_xq<2>(smem + a.xs_off, a.x, a.dim, tid, blockDim.x, &xb);
          __syncthreads();
          xr = D::load_x(XQLds{smem + a.xs_off}, unit);
        } else {
          D::finish_tables(tbl, tr, tid, blockDim.x);
          xr = D::load_x(a.x, unit);
          __syncthreads();
        }
      } else {
        const CopyJob jobs[3] = {tbl_job_of<D>(0, 0u, true), tbl_job_of<D>(1, 0u, true),
                                 {(const uint4*)a.x, (uint32_t)(smem - tbl) + a.xs_off, a.stage_x ? a.dim / 4u : 0u, 3u}};
        copy_jobs<4>(tbl, jobs, tid, blockDim.x);
        if (a.stage_x) {
          __syncthreads();
          xr = D::load_x(XLds{(const float*)(smem + a.xs_off)}, unit);
        } else {
          xr = D::load_x(a.x, unit);
          __syncthreads();
        }
      }
      if (!valid) xr = typename D::X{};
      first = false;
    }
#pragma unroll
    for (int s = NR / 2; s < NR; s++) fetch(s);
    if constexpr (requires { D::HAS_PRE; }) {
      // Three steps per row pair (gate and up together, four interleaved chains): table reads of the pair two places
      // ahead, entry reads of the next pair, arithmetic of this one. Pairs past the end of the run decode the zeros that
      // their empty buffer descriptors returned (every address stays inside the tables, and a zero block scale makes
      // the result zero).
      const uint32_t lanec = (lane & 1u) * 0x80808080u;
      typename D::Pre pg_[2], pu_[2];    // [pair & 1]
      typename D::Look lg[2], lu[2];
      pg_[0] = D::pre(rg[0], tbl); pu_[0] = D::pre(ru[0], tbl);
      pg_[1] = D::pre(rg[1], tbl); pu_[1] = D::pre(ru[1], tbl);
      D::lookup(rg[0], pg_[0], tbl, lanec, lg[0]); D::lookup(ru[0], pu_[0], tbl, lanec, lu[0]);
      static_assert(NS == 1 && NR % 2 == 0 && NR >= 4, "two row pairs per fold, table reads two pairs ahead");
      for (uint32_t r0 = w0; r0 < w1; r0 += NR) {
#pragma unroll
        for (int half = 0; half < NR / 2; half++) {
          float acc[4];  // value 2 j + m: row pair j of this half, m = 0 gate, 1 up
#pragma unroll
          for (int j = 0; j < 2; j++) {
            const int s = half * 2 + j, s1 = (s + 1) % NR, s2 = (s + 2) % NR, b = s & 1;
            D::lookup(rg[s1], pg_[b ^ 1], tbl, lanec, lg[b ^ 1]);
            D::lookup(ru[s1], pu_[b ^ 1], tbl, lanec, lu[b ^ 1]);
            pg_[b] = D::pre(rg[s2], tbl);
            pu_[b] = D::pre(ru[s2], tbl);
            // (scheduling barriers: left alone, the compiler moves a pair's entry reads next to their use)
            __builtin_amdgcn_sched_barrier(0);
            D::partial2(rg[s], lg[b], ru[s], lu[b], xr, acc[2 * j], acc[2 * j + 1]);
            __builtin_amdgcn_sched_barrier(0);
            fetch(s);  // the slot is free again: fetch the row pair NR places ahead
          }
          const uint32_t rb = r0 + half * 2;
          if (rb < w1) {
            row16_fold<4>(acc, lane);
            const uint32_t k = group8_sel<4>(lane), j = k >> 1, m = k & 1u;
            if (!(lane & 8u) && rb + j < w1) part[((rb + j - c0) * 2 + m) * PSTRIDE + ks * 4 + (lane >> 4)] = acc[0];
          }
        }
      }
    } else {
    typename D::Look lk[2];  // stage t of a row pair uses lk[t & 1]; 2 NS stages per row pair keep the parity fixed
    if (w0 < w1) lk[0] = D::lookup(rg[0], 0, tbl);
    for (uint32_t r0 = w0; r0 < w1; r0 += NR) {
#pragma unroll
      for (int half = 0; half < 2; half++) {
        float acc[NR];  // value 2 j + m: row pair j of this half, m = 0 gate, 1 up
#pragma unroll
        for (int j = 0; j < NR / 2; j++) {
          const int s = half * (NR / 2) + j;
          const uint32_t row = r0 + s;
          float g = 0.f, u = 0.f;
          if (row < w1) {  // wave-uniform; no global loads inside, so the loads in flight stay countable
            const bool more = row + 1 < w1;
#pragma unroll
            for (int t = 0; t < 2 * NS; t++) {
              const bool up = t >= NS;
              const int st = up ? t - NS : t;
              // issue the next stage's table reads, then consume this stage's
              if (t + 1 < 2 * NS) lk[(t + 1) & 1] = D::lookup(t + 1 >= NS ? ru[s] : rg[s], t + 1 >= NS ? t + 1 - NS : t + 1, tbl);
              else if (more) lk[0] = D::lookup(rg[(s + 1) % NR], 0, tbl);
              if (up) { u = D::partial(ru[s], lk[t & 1], xr, st, u); asm volatile("" : "+v"(u)); }
              else { g = D::partial(rg[s], lk[t & 1], xr, st, g); asm volatile("" : "+v"(g)); }
            }
          }
          acc[2 * j] = g;
          acc[2 * j + 1] = u;
          fetch(s);  // the slot is free again: fetch the row pair NR places ahead
        }
        const uint32_t rb = r0 + half * (NR / 2);
        if (rb < w1) {
          row16_fold<NR>(acc, lane);
          const uint32_t k = group8_sel<NR>(lane), j = k >> 1, m = k & 1u;
          if (!(lane & 8u) && rb + j < w1) part[((rb + j - c0) * 2 + m) * PSTRIDE + ks * 4 + (lane >> 4)] = acc[0];
        }
      }
    }
    }
    __syncthreads();
    // thread q sums the partials of (row q / 2, matrix q % 2); gate and up then meet in the even lane
    for (uint32_t q0 = 0; q0 < 2 * n; q0 += blockDim.x) {
      const uint32_t q = q0 + tid;
      float sum = 0.f;
      if (q < 2 * n) sum = sum_in_order(part + q * PSTRIDE, 4 * KS);
      const float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sum), 0xB1, 0xF, 0xF, false));
      if (q < 2 * n && !(q & 1u)) {
        const uint32_t v = c0 + (q >> 1);
        const uint32_t e = shared ? 0u : v / a.inter, r = v - e * a.inter;
        const uint32_t he = shared ? a.n_routed : e;
        store_h(a, (size_t)he * a.inter + r, swiglu(sum, other, shared ? 1.f : a.wts[e]));
      }
    }
    __syncthreads();
  }
}

template <class D>
__device__ __forceinline__ void moe_gu_run(const MoeArgs& a, const uint64_t* table, uint32_t* tbl, uint32_t* smem, const bool shared, const uint32_t wg) {
  if constexpr (requires { D::STAGES; }) moe_gu_run_ring<D>(a, table, tbl, smem, shared, wg);
  else moe_gu_run_direct<D, rows_in_flight<D>(2)>(a, table, tbl, smem, shared, wg);
}

// table: MoeArgs::table once more, as an argument of its own in first place: built with kernel-argument preload it is
// in scalar registers when the wave starts, and the expert addresses are requested one memory trip earlier.
template <class DR, class DS>
__global__ __launch_bounds__(1024) void moe_gu_kernel(const uint64_t* table, const MoeArgs a) {
  // The codebook table is a static array: its LDS address is a compile-time constant that goes into the offset field
  // of the lookups (with a table in dynamic LDS every lookup address ends in an addition of the base). Partial sums and
  // the staged activations follow in dynamic LDS.
  constexpr int TBL = DR::LDS_WORDS > DS::LDS_WORDS ? DR::LDS_WORDS : DS::LDS_WORDS;
  __shared__ __attribute__((aligned(16))) uint32_t tbl[TBL > 0 ? TBL : 4];
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  if (blockIdx.x < a.grid_routed) moe_gu_run<DR>(a, table, tbl, smem, false, blockIdx.x);
  else moe_gu_run<DS>(a, table, tbl, smem, true, blockIdx.x - a.grid_routed);
}

// down: workgroup = RW row-groups x (NE expert-waves x KS K-split waves). In a row-group, wave (e, ks) owns routed
// expert e's K-slice ks of the row-group's rows; the shared expert's rows are dealt over the same waves (wave e takes
// rows e, e + E, ...). Per row the partial sums are added in the fixed order (expert 0 ks 0.., expert 1 .., shared ks 0..).
// Codebook decoders stream their rows through register rings of range-checked buffer loads (see moe_gu_run_ring): the
// first rows of both the routed and the shared matrix are requested before the tables and activations are staged.
template <class D, int NR, class F>
__device__ __forceinline__ void down_rows_ring(const uint32_t* tbl, const typename D::X& x, const uint32_t lane, uint32_t first,
                                                const uint32_t step, const uint32_t end, typename D::Raw (&ring)[NR], F&& fetch,
                                                float* part_col, const uint32_t pstride, const uint32_t c0) {
  // rows first, first + step, ... < end; ring[s] already holds row first + s * step; fetch(s) refills slot s
  constexpr int NS = D::STAGES;
  typename D::Look lk[2];
  if (first < end) lk[0] = D::lookup(ring[0], 0, tbl);
  for (uint32_t r0 = first; r0 < end; r0 += NR * step) {
#pragma unroll
    for (int half = 0; half < NR / 4; half++) {
      float acc[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int s = half * 4 + j;
        const uint32_t row = r0 + s * step;
        float v = 0.f;
        if (row < end) {  // wave-uniform; no global loads inside
          const bool more = row + step < end;
#pragma unroll
          for (int t = 0; t < NS; t++) {
            const int cur = (s * NS + t) & 1;
            if (t + 1 < NS) lk[cur ^ 1] = D::lookup(ring[s], t + 1, tbl);
            else if (more) lk[cur ^ 1] = D::lookup(ring[(s + 1) % NR], 0, tbl);
            v = D::partial(ring[s], lk[cur], x, t, v);
            asm volatile("" : "+v"(v));
          }
        }
        acc[j] = v;
        fetch(s);
      }
      const uint32_t rb = r0 + half * 4 * step;
      if (rb < end) {
        row16_fold<4>(acc, lane);
        const uint32_t r = rb + group8_sel<4>(lane) * step;
        if (!(lane & 8u) && r < end) part_col[(r - c0) * pstride + (lane >> 4)] = acc[0];
      }
    }
  }
}

// MAXT: largest workgroup the instantiation is launched with (768 threads leave 170 registers per lane, 1024 only 128)
template <class DR, class DS, int MAXT>
__global__ __launch_bounds__(MAXT) void moe_down_kernel(const uint64_t* table, const MoeArgs a) {
  constexpr bool RING_R = requires { DR::STAGES; }, RING_S = requires { DS::STAGES; };
  constexpr bool HALF = kHalfH<DR, DS>;
  constexpr int RPW = rows_in_flight<DR>(1);
  constexpr int NR = 4, NSH = 4;  // ring depth: routed rows, shared rows
  constexpr int TBL = DR::LDS_WORDS + DS::LDS_WORDS;
  __shared__ __attribute__((aligned(16))) uint32_t tbl[TBL > 0 ? TBL : 4];  // static: see moe_gu_kernel
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  uint32_t* tbl_r = tbl;
  uint32_t* tbl_s = tbl + DR::LDS_WORDS;
  float* part = (float*)smem;

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = uniform(tid >> 6), nwaves = blockDim.x >> 6;
  const uint32_t KS = a.ks;
  const uint32_t NE = a.run_routed ? a.n_routed : 0u;       // routed experts computed here
  const uint32_t E = max(NE, 1u);
  const uint32_t wpg = E * KS;                              // waves per row-group
  const uint32_t RW = uniform(small_div(nwaves, wpg)), rg = uniform(small_div(wave, wpg)), wl = wave - rg * wpg;
  const uint32_t e = uniform(small_div(wl, KS)), ks = wl - e * KS;
  const uint32_t slots = 4 * (NE * KS + (a.run_shared ? KS : 0u));  // partial sums per row: 4 per contributing wave
  const uint32_t PSTRIDE = slots + 1;

  const uint32_t u0 = ks * 64u + lane;
  const uint32_t units_r = a.inter / DR::UNIT, units_s = a.inter / DS::UNIT;
  const bool valid_r = NE && u0 < units_r, valid_s = a.run_shared && u0 < units_s;
  const uint32_t unit_r = u0 < units_r ? u0 : units_r - 1, unit_s = u0 < units_s ? u0 : units_s - 1;
  const void* Dr_ = nullptr;
  if (NE) Dr_ = uniform(table ? table_entry(table, 3 * e + 2) : (const void*)a.down[e]);
  const gptr_t Dr = as_global(Dr_), Dsh = as_global(a.sdown);

  const auto off_r = [&] { if constexpr (RING_R) return DR::offsets(unit_r); else return 0; }();
  const auto off_s = [&] { if constexpr (RING_S) return DS::offsets(unit_s); else return 0; }();

  const uint32_t wg_begin = blockIdx.x * a.rows_per_wg, wg_end = min(a.dim, wg_begin + a.rows_per_wg);
  typename DR::X xr;
  typename DS::X xs;
  bool first = true;
  for (uint32_t c0 = wg_begin; c0 < wg_end; c0 += kMoeChunkRows) {
    const uint32_t c1 = min(wg_end, c0 + kMoeChunkRows), n = c1 - c0;
    const uint32_t run = uniform(small_div(n + RW - 1, RW));
    const uint32_t w0 = uniform(min(c0 + rg * run, c1)), w1 = uniform(min(w0 + run, c1));

    // Codebook pairs that take h as fp16: tables and h rows come by loads that write LDS themselves, requested ahead of
    // everything else (no registers are held for them, and they return -- loads return in order -- ahead of the first
    // weight rows' trip to HBM instead of behind it); what does not fill a group of 64 items goes through one register.
    constexpr bool DMA = RING_R && RING_S && HALF && MAXT <= 768;  // (the 1024-thread instantiations have no registers to spare)
    [[maybe_unused]] u32x4 rest[4];
    [[maybe_unused]] uint32_t rest_at[4] = {0u, 0u, 0u, 0u};  // LDS word offset + 1 of the thread's leftover item, 0: none
    if constexpr (DMA) {
      if (first && a.stage_x) {
        const uint32_t lo = NE ? 0u : a.n_routed * a.inter;
        const uint32_t hi = (a.run_shared ? a.n_routed + 1u : a.n_routed) * a.inter;
        const CopyJob jobs[5] = {tbl_job_of<DR>(0, 0u, NE), tbl_job_of<DR>(1, 0u, NE), tbl_job_of<DS>(0, DR::LDS_WORDS, a.run_shared),
                                 tbl_job_of<DS>(1, DR::LDS_WORDS, a.run_shared),
                                 {(const uint4*)(a.h16 + lo), (uint32_t)(smem - tbl) + a.xs_off, (hi - lo) / 8u, 0u}};
        auto same = [](uint32_t i) { return i; };
#pragma unroll
        for (int j = 0; j < 5; j++) {
          if (jobs[j].n16 == 0) continue;
          const uint32_t done = j == 4 ? lds_dma_groups(tbl + jobs[j].dst, jobs[j].src, jobs[j].n16, wave, nwaves, lane, xhalf_rot_src)
                                       : lds_dma_groups(tbl + jobs[j].dst, jobs[j].src, jobs[j].n16, wave, nwaves, lane, same);
          if (j < 4 && done + tid < jobs[j].n16) {  // (the h rows are whole groups: inter is a multiple of 256)
            rest[j] = *(const u32x4*)(jobs[j].src + done + tid);
            rest_at[j] = jobs[j].dst + 4u * (done + tid) + 1u;
          }
        }
      }
    }
    // the value of y that this thread adds to in the epilogue, requested ahead of the rows (14.3 -> 14.15 us)
    float yq = 0.f;
    if (!DMA && tid < n) yq = a.y[c0 + tid];
    // ---- request the first rows of both matrices
    typename DR::Raw cur[RING_R ? 1 : RPW], nxt[RING_R ? 1 : RPW];
    uint32_t pv = w0;  // routed ring cursor
    typename DR::Raw rr[NR];
    typename DS::Raw rs[NSH];
    uint32_t sv = w0 + e;  // shared ring cursor
    auto fetch_r = [&](int s) {
      if constexpr (RING_R) {
        rr[s] = DR::fetch(make_rsrc(Dr_, (NE && pv < w1) ? a.dim * a.rb_d_r : 0u), off_r, pv * a.rb_d_r);
        pv++;
      }
    };
    auto fetch_s = [&](int s) {
      if constexpr (RING_S) {
        rs[s] = DS::fetch(make_rsrc(a.sdown, (a.run_shared && sv < w1) ? a.dim * a.rb_d_s : 0u), off_s, sv * a.rb_d_s);
        sv += E;
      }
    };
    if constexpr (RING_R) {
#pragma unroll
      for (int s = 0; s < NR; s++) fetch_r(s);
    } else if (NE && w0 < w1) {
#pragma unroll
      for (int j = 0; j < RPW; j++) cur[j] = DR::load(Dr + (size_t)min(w0 + j, w1 - 1) * a.rb_d_r, unit_r);
    }
    if constexpr (DMA) yq = a.y[c0 + min(tid, n - 1u)];  // (every wave: the wait below counts the loads behind the copy)
    if (DMA && first && a.stage_x) {
      wait_vm<NR * DR::FETCH_LOADS + 1>();  // everything older than the routed ring and y: the copy
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (rest_at[j]) *(u32x4*)(tbl + rest_at[j] - 1u) = rest[j];
      const uint32_t lo = NE ? 0u : a.n_routed * a.inter;
      const uint32_t* hs = smem + a.xs_off;
      __syncthreads();
      if (NE) xr = load_h_staged<DR, HALF, true>(hs, e * a.inter, unit_r);
      if (a.run_shared) xs = load_h_staged<DS, HALF, true>(hs, a.n_routed * a.inter - lo, unit_s);
      if (!valid_r) xr = typename DR::X{};
      if (!valid_s) xs = typename DS::X{};
      first = false;
    }
    if (first) {
      // h rows this launch reads: the routed ones [0, NE), then the shared one at n_routed (NE is 0 or n_routed)
      const uint32_t lo = NE ? 0u : a.n_routed * a.inter;
      const uint32_t hi = (a.run_shared ? a.n_routed + 1u : a.n_routed) * a.inter;
      const CopyJob jobs[5] = {tbl_job_of<DR>(0, 0u, NE), tbl_job_of<DR>(1, 0u, NE),
                               tbl_job_of<DS>(0, DR::LDS_WORDS, a.run_shared), tbl_job_of<DS>(1, DR::LDS_WORDS, a.run_shared),
                               HALF ? CopyJob{(const uint4*)(a.h16 + lo), (uint32_t)(smem - tbl) + a.xs_off,
                                              a.stage_x ? (hi - lo) / 8u : 0u, 2u}
                                    : CopyJob{(const uint4*)(a.h + lo), (uint32_t)(smem - tbl) + a.xs_off,
                                              a.stage_x ? (hi - lo) / 4u : 0u, 3u}};
      copy_jobs<(MAXT <= 768 ? 8 : 4)>(tbl, jobs, tid, blockDim.x);
      if (a.stage_x) {
        const uint32_t* hs = smem + a.xs_off;
        __syncthreads();
        if (NE) xr = load_h_staged<DR, HALF>(hs, e * a.inter, unit_r);
        if (a.run_shared) xs = load_h_staged<DS, HALF>(hs, a.n_routed * a.inter - lo, unit_s);
      } else {
        if (NE) xr = load_h_direct<DR, HALF>(a, e * a.inter, unit_r);
        if (a.run_shared) xs = load_h_direct<DS, HALF>(a, a.n_routed * a.inter, unit_s);
        __syncthreads();
      }
      if (!valid_r) xr = typename DR::X{};
      if (!valid_s) xs = typename DS::X{};
      first = false;
    }
    // the shared expert's first rows are requested only now: they are not needed before the routed rows are done, and
    // requested with the routed ones they lengthen the queue that the prologue's copy waits behind
    if constexpr (RING_S) {
#pragma unroll
      for (int s = 0; s < NSH; s++) fetch_s(s);
    }
    // ---- routed expert e, rows w0 .. w1
    if (NE) {
      if constexpr (RING_R) {
        down_rows_ring<DR, NR>(tbl_r, xr, lane, w0, 1u, w1, rr, fetch_r, part + 4 * (e * KS + ks), PSTRIDE, c0);
      } else {
        for (uint32_t r0 = w0; r0 < w1; r0 += RPW) {
          const bool more = r0 + RPW < w1;
          if (more) {
#pragma unroll
            for (int j = 0; j < RPW; j++) nxt[j] = DR::load(Dr + (size_t)min(r0 + RPW + j, w1 - 1) * a.rb_d_r, unit_r);
          }
          float acc[RPW];
#pragma unroll
          for (int j = 0; j < RPW; j++) {
            acc[j] = dec_dot<DR>(cur[j], xr, tbl_r, unit_r);  // lanes past the row hold zero activations
            asm volatile("" ::: "memory");
          }
          row16_fold<RPW>(acc, lane);
          {
            const uint32_t j = group8_sel<RPW>(lane);
            if (!(lane & 8u) && r0 + j < w1) part[(r0 + j - c0) * PSTRIDE + 4 * (e * KS + ks) + (lane >> 4)] = acc[0];
          }
          if (more) {
#pragma unroll
            for (int j = 0; j < RPW; j++) cur[j] = nxt[j];
          }
        }
      }
    }
    // ---- shared expert: the row-group's waves with K-slice ks take rows w0 + e, w0 + e + E, ...
    if (a.run_shared) {
      if constexpr (RING_S) {
        down_rows_ring<DS, NSH>(tbl_s, xs, lane, w0 + e, E, w1, rs, fetch_s, part + 4 * (NE * KS + ks), PSTRIDE, c0);
      } else {
        for (uint32_t r0 = w0 + e; r0 < w1; r0 += 2 * E) {
          const uint32_t r1 = r0 + E;
          const typename DS::Raw ra = DS::load(Dsh + (size_t)r0 * a.rb_d_s, unit_s);
          const typename DS::Raw rb = DS::load(Dsh + (size_t)min(r1, w1 - 1) * a.rb_d_s, unit_s);
          float acc[2] = {dec_dot<DS>(ra, xs, tbl_s, unit_s), dec_dot<DS>(rb, xs, tbl_s, unit_s)};
          row16_fold<2>(acc, lane);
          const uint32_t r = group8_sel<2>(lane) ? r1 : r0;
          if (!(lane & 8u) && r < w1) part[(r - c0) * PSTRIDE + 4 * (NE * KS + ks) + (lane >> 4)] = acc[0];
        }
      }
    }
    __syncthreads();
    for (uint32_t t = tid; t < n; t += blockDim.x) {
      const float s = sum_in_order(part + t * PSTRIDE, slots);
      a.y[c0 + t] = (t == tid ? yq : a.y[c0 + t]) + s * (1.f / kHScale);
    }
    __syncthreads();
  }
}

}  // namespace msq
