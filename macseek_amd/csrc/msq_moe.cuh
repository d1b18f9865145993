// Fused batch-1 MoE layer (reference operators: ms::q::encode_moe_decode / _table / _table_part,
// src/kernels/quant.mm:266-369; reference kernels q_moe_gu / q_moe_down, src/kernels/quant_moe.metal:50-147):
//   moe_gu_kernel  : h[e][r] = silu(min(gate_e[r].x, 10)) * clamp(up_e[r].x, -10, 10) * w_e   for all experts
//   moe_down_kernel: y[r] += sum_e down_e[r] . h[e]   (routed experts in slot order, then the shared expert)
// Expert e < n_routed is a routed expert (decoder DR); the shared expert (decoder DS, weight 1) keeps its h row at
// index n_routed. Expert matrices are reached either through pointers passed by value or through a device-resident
// table of 6 x {gate, up, down} 64-bit addresses that the host may fill after the launch was enqueued.
#pragma once
#include "msq_device.cuh"

namespace msq {

constexpr int kMaxRouted = 6;

struct MoeArgs {
  const float* x;        // [dim]
  float* h;              // scratch: [(n_routed + 1)][inter]
  float* y;              // [dim], accumulated
  const float* wts;      // [n_routed] routing weights (device memory)
  const uint64_t* table; // kMaxRouted x {gate, up, down} device addresses, or null to use the arrays below
  const uint8_t* gate[kMaxRouted];
  const uint8_t* up[kMaxRouted];
  const uint8_t* down[kMaxRouted];
  const uint8_t *sgate, *sup, *sdown;
  uint32_t n_routed;     // h row of the shared expert
  uint32_t run_routed;   // experts this launch computes: routed ones (0 or n_routed) ...
  uint32_t run_shared;   // ... and / or the shared one
  uint32_t dim, inter;
  uint32_t rb_gu_r, rb_d_r, rb_gu_s, rb_d_s;  // row bytes: routed gate/up, routed down, shared gate/up, shared down
  uint32_t ks, rpw;      // K-split waves, rows per wave per tile
  uint32_t tiles_per_expert;  // gate/up: row tiles per expert
  uint32_t grid_routed;       // gate/up: workgroups [0, grid_routed) take routed tiles, the rest shared tiles
  uint32_t ntiles;            // down: row tiles
};

__device__ __forceinline__ float swiglu(float g, float u, float w) {  // quant_moe.metal:23-27
  g = fminf(g, 10.f);
  u = fminf(fmaxf(u, -10.f), 10.f);
  return g / (1.f + expf(-g)) * u * w;
}

// gate + up + SwiGLU for the experts [e0, e0 + ne) of one kind; workgroup `wg` of `nwg` walks their row tiles.
template <class D>
__device__ __forceinline__ void moe_gu_run(const MoeArgs& a, uint32_t* smem, bool shared, uint32_t wg, uint32_t nwg) {
  uint32_t* tbl = smem;
  float* part = (float*)(smem + D::LDS_WORDS);
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, nwaves = blockDim.x >> 6;
  const uint32_t KS = a.ks, ks = wave % KS, rw = wave / KS, RW = nwaves / KS;
  const uint32_t tile_rows = RW * a.rpw;
  const uint32_t units = a.dim / D::UNIT;
  const uint32_t row_bytes = shared ? a.rb_gu_s : a.rb_gu_r;
  const uint32_t n_exp = shared ? 1u : a.n_routed;

  D::fill_lds(tbl, (int)tid, (int)blockDim.x);
  const uint32_t u0 = ks * 64u + lane;
  const bool valid = u0 < units;
  const uint32_t unit = valid ? u0 : units - 1;
  const typename D::X xr = D::load_x(a.x, unit);
  if (D::LDS_WORDS) __syncthreads();

  const uint32_t ntiles = n_exp * a.tiles_per_expert;
  for (uint32_t tile = wg; tile < ntiles; tile += nwg) {
    const uint32_t e = tile / a.tiles_per_expert;
    const uint32_t tile_row0 = (tile - e * a.tiles_per_expert) * tile_rows;
    const uint8_t *G, *U;
    if (shared) { G = a.sgate; U = a.sup; }
    else if (a.table) { G = (const uint8_t*)a.table[3 * e]; U = (const uint8_t*)a.table[3 * e + 1]; }
    else { G = a.gate[e]; U = a.up[e]; }
    const uint32_t row0 = tile_row0 + rw * a.rpw;
    for (uint32_t j = 0; j < a.rpw; j++) {
      const uint32_t row = min(row0 + j, a.inter - 1);
      const size_t off = (size_t)row * row_bytes;
      const typename D::Raw rg = D::load(G + off, unit), ru = D::load(U + off, unit);
      float ag = dec_dot<D>(rg, xr, tbl, unit), au = dec_dot<D>(ru, xr, tbl, unit);
      ag = wave_sum(valid ? ag : 0.f);
      au = wave_sum(valid ? au : 0.f);
      if (lane == 0) {
        part[((rw * a.rpw + j) * 2 + 0) * KS + ks] = ag;
        part[((rw * a.rpw + j) * 2 + 1) * KS + ks] = au;
      }
    }
    __syncthreads();
    if (tid < tile_rows) {
      const uint32_t row = tile_row0 + tid;
      if (row < a.inter) {
        float g = 0.f, u = 0.f;
        for (uint32_t k = 0; k < KS; k++) { g += part[(tid * 2) * KS + k]; u += part[(tid * 2 + 1) * KS + k]; }
        const uint32_t he = shared ? a.n_routed : e;
        a.h[(size_t)he * a.inter + row] = swiglu(g, u, shared ? 1.f : a.wts[e]);
      }
    }
    __syncthreads();
  }
}

template <class DR, class DS>
__global__ __launch_bounds__(1024) void moe_gu_kernel(const MoeArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  if (blockIdx.x < a.grid_routed) moe_gu_run<DR>(a, smem, false, blockIdx.x, a.grid_routed);
  else moe_gu_run<DS>(a, smem, true, blockIdx.x - a.grid_routed, gridDim.x - a.grid_routed);
}

// down: workgroup = RW row-groups x (NE expert-waves x KS K-split waves). In a row-group, wave (e, ks) owns routed
// expert e's K-slice ks of every row of the tile; afterwards the same waves share out the shared expert's rows.
// Per row the partial sums are added in the fixed order (expert 0 ks 0.., expert 1 .., shared ks 0..).
template <class DR, class DS>
__global__ __launch_bounds__(1024) void moe_down_kernel(const MoeArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  constexpr int TBL = DR::LDS_WORDS + DS::LDS_WORDS;
  uint32_t* tbl_r = smem;
  uint32_t* tbl_s = smem + DR::LDS_WORDS;
  float* part = (float*)(smem + TBL);

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, nwaves = blockDim.x >> 6;
  const uint32_t KS = a.ks;
  const uint32_t NE = a.run_routed ? a.n_routed : 0u;       // routed experts computed here
  const uint32_t wpg = max(NE, 1u) * KS;                    // waves per row-group
  const uint32_t RW = nwaves / wpg, rg = wave / wpg, wl = wave % wpg;
  const uint32_t e = wl / KS, ks = wl % KS;
  const uint32_t tile_rows = RW * a.rpw;
  const uint32_t slots = NE * KS + (a.run_shared ? KS : 0u);  // partial sums per row

  if (NE) DR::fill_lds(tbl_r, (int)tid, (int)blockDim.x);
  if (a.run_shared) DS::fill_lds(tbl_s, (int)tid, (int)blockDim.x);

  const uint32_t u0 = ks * 64u + lane;
  const uint32_t units_r = a.inter / DR::UNIT, units_s = a.inter / DS::UNIT;
  const bool valid_r = NE && u0 < units_r, valid_s = a.run_shared && u0 < units_s;
  const uint32_t unit_r = u0 < units_r ? u0 : units_r - 1, unit_s = u0 < units_s ? u0 : units_s - 1;
  typename DR::X xr;
  typename DS::X xs;
  const uint8_t* Dr = nullptr;
  if (NE) {
    xr = DR::load_x(a.h + (size_t)e * a.inter, unit_r);
    Dr = a.table ? (const uint8_t*)a.table[3 * e + 2] : a.down[e];
  }
  if (a.run_shared) xs = DS::load_x(a.h + (size_t)a.n_routed * a.inter, unit_s);
  if (TBL) __syncthreads();

  for (uint32_t tile = blockIdx.x; tile < a.ntiles; tile += gridDim.x) {
    const uint32_t row0 = tile * tile_rows + rg * a.rpw;
    if (NE) {
#pragma unroll 4
      for (uint32_t j = 0; j < a.rpw; j++) {
        const uint32_t row = min(row0 + j, a.dim - 1);
        const typename DR::Raw r = DR::load(Dr + (size_t)row * a.rb_d_r, unit_r);
        float acc = dec_dot<DR>(r, xr, tbl_r, unit_r);
        acc = wave_sum(valid_r ? acc : 0.f);
        if (lane == 0) part[(rg * a.rpw + j) * slots + e * KS + ks] = acc;
      }
    }
    if (a.run_shared) {
      // the row-group's waves with K-slice ks take the shared expert's rows e, e + E, ... of the tile
      const uint32_t E = max(NE, 1u);
#pragma unroll 2
      for (uint32_t j = e; j < a.rpw; j += E) {
        const uint32_t row = min(row0 + j, a.dim - 1);
        const typename DS::Raw r = DS::load(a.sdown + (size_t)row * a.rb_d_s, unit_s);
        float acc = dec_dot<DS>(r, xs, tbl_s, unit_s);
        acc = wave_sum(valid_s ? acc : 0.f);
        if (lane == 0) part[(rg * a.rpw + j) * slots + NE * KS + ks] = acc;
      }
    }
    __syncthreads();
    if (tid < tile_rows) {
      const uint32_t row = tile * tile_rows + tid;
      if (row < a.dim) {
        float s = 0.f;
        for (uint32_t k = 0; k < slots; k++) s += part[tid * slots + k];
        a.y[row] += s;
      }
    }
    __syncthreads();
  }
}

}  // namespace msq
