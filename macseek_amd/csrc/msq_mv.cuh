// Decode matvec (n = 1): y[r] (+)= W[r] . x over raw GGUF block rows (reference operator: ms::q::encode_matvec,
// src/kernels/quant.mm:70-95; reference kernel q_mv, src/kernels/quant_mv.metal:7-39).
//
// Workgroup = RW row-waves x KS K-split waves. A lane owns ITERS units of D::UNIT columns at fixed column positions
// and keeps their activations in registers for the whole kernel; a wave walks the rows of its tile, so weights are
// the only HBM stream. Workgroups are persistent (grid-stride over row tiles) so codebook tables are staged into LDS
// once per workgroup. K-split partial sums meet in LDS and are added in a fixed order.
#pragma once
#include "msq_device.cuh"

namespace msq {

struct MvArgs {
  const uint8_t* W;
  const float* x;
  float* y;
  uint32_t rows, cols, row_bytes;
  uint32_t rows_per_group;  // block-diagonal: rows in each group (== rows when groups == 1)
  uint32_t x_group_stride;  // elements between the inputs of consecutive groups
  uint32_t accumulate;
  uint32_t units;   // cols / D::UNIT
  uint32_t ks;      // waves splitting K
  uint32_t rpw;     // rows per wave per tile
  uint32_t ntiles;  // ceil(rows / (RW * rpw))
};

template <class D, int ITERS>
__global__ __launch_bounds__(1024) void mv_kernel(const MvArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  uint32_t* tbl = smem;
  float* part = (float*)(smem + D::LDS_WORDS);

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, nwaves = blockDim.x >> 6;
  const uint32_t KS = a.ks, ks = wave % KS, rw = wave / KS, RW = nwaves / KS;
  const uint32_t tile_rows = RW * a.rpw;

  D::fill_lds(tbl, (int)tid, (int)blockDim.x);

  uint32_t unit[ITERS];
  bool valid[ITERS];
#pragma unroll
  for (int i = 0; i < ITERS; i++) {
    const uint32_t u = (ks * ITERS + i) * 64u + lane;
    valid[i] = u < a.units;
    unit[i] = valid[i] ? u : a.units - 1;  // idle lanes shadow the last unit; their result is dropped
  }
  typename D::X xr[ITERS];
  uint32_t cur_group = 0xFFFFFFFFu;
  if (D::LDS_WORDS) __syncthreads();

  for (uint32_t tile = blockIdx.x; tile < a.ntiles; tile += gridDim.x) {
    const uint32_t tile_row0 = tile * tile_rows;
    const uint32_t group = tile_row0 / a.rows_per_group;  // a tile never straddles two groups (host guarantees)
    if (group != cur_group) {
      const float* xg = a.x + (size_t)group * a.x_group_stride;
#pragma unroll
      for (int i = 0; i < ITERS; i++) xr[i] = D::load_x(xg, unit[i]);
      cur_group = group;
    }
    const uint32_t row0 = tile_row0 + rw * a.rpw;
    for (uint32_t j = 0; j < a.rpw; j++) {
      const uint32_t row = min(row0 + j, a.rows - 1);
      const uint8_t* wr = a.W + (size_t)row * a.row_bytes;
      typename D::Raw raw[ITERS];
#pragma unroll
      for (int i = 0; i < ITERS; i++) raw[i] = D::load(wr, unit[i]);
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < ITERS; i++) {
        const float v = dec_dot<D>(raw[i], xr[i], tbl, unit[i]);
        acc += valid[i] ? v : 0.f;
      }
      acc = wave_sum(acc);
      if (KS == 1) {
        if (lane == 0 && row0 + j < a.rows) a.y[row0 + j] = a.accumulate ? a.y[row0 + j] + acc : acc;
      } else if (lane == 0) {
        part[(rw * a.rpw + j) * KS + ks] = acc;
      }
    }
    if (KS > 1) {
      __syncthreads();
      if (tid < tile_rows) {
        const uint32_t row = tile_row0 + tid;
        if (row < a.rows) {
          float s = 0.f;
          for (uint32_t k = 0; k < KS; k++) s += part[tid * KS + k];
          a.y[row] = a.accumulate ? a.y[row] + s : s;
        }
      }
      __syncthreads();
    }
  }
}

}  // namespace msq
