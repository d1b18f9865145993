// Decode matvec (n = 1): y[r] (+)= W[r] . x over raw GGUF block rows (reference operator: ms::q::encode_matvec,
// src/kernels/quant.mm:70-95; reference kernel q_mv, src/kernels/quant_mv.metal:7-39).
//
// Workgroup = RW row-waves x KS K-split waves. A lane owns ITERS units of D::UNIT columns at fixed column positions
// and keeps their activations in registers for the whole kernel; a wave walks the rows of its tile, so weights are
// the only HBM stream. Workgroups are persistent (grid-stride over row tiles) so codebook tables are staged into LDS
// once per workgroup. K-split partial sums meet in LDS and are added in a fixed order.
#pragma once
#include <array>

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
  // fused input RMSNorm (NORM kernels only): x is replaced by x * rsqrt(mean(x^2) + eps) * norm_w
  const float* norm_w;
  float eps;
  uint32_t norm_off;  // word offset in dynamic LDS of the norm's four partial sums
  // Activations staged through LDS (always for NORM kernels): word offset in dynamic LDS of the padded row
  // (xlds_words(cols) words), and whether the plain kernels stage at all (rows too long for LDS are read directly)
  uint32_t xs_off;
  uint32_t stage_x;
  uint32_t w_off;     // word offset in dynamic LDS of the waves' weight-row buffers (token kernel, one token of a block format)
};

// The lane's activation slices of one row, from the workgroup's padded LDS copy (staged here, all threads must call)
// or straight from device memory.
template <class D, int ITERS>
__device__ __forceinline__ void load_x_row(const MvArgs& a, float* xs, const float* xg, const uint32_t (&unit)[ITERS],
                                           typename D::X (&xr)[ITERS], uint32_t tid, uint32_t nt) {
  if (D::STAGE_X && a.stage_x) {
    __syncthreads();  // readers of the previous row are done
    const float* src[1] = {xg};
    stage_x_rows<1>(xs, src, 1u, 0u, a.cols, tid, nt);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < ITERS; i++) xr[i] = D::load_x(XLds{xs}, unit[i]);
  } else {
#pragma unroll
    for (int i = 0; i < ITERS; i++) xr[i] = D::load_x(xg, unit[i]);
  }
}

// ---------------------------------------------------------------------------------------------------- RMSNorm
// scale = 1 / sqrt(mean(x^2) + eps) of one row, computed by a workgroup with a reduction whose order does not depend
// on the workgroup's size: four virtual waves, virtual lane v (0..255) adds x[v], x[v + 256], ... with fused
// multiply-adds, a DPP wave sum per virtual wave, then (s0 + s1) + (s2 + s3). The standalone norm kernel and the
// matvec kernels with a fused norm both call this, so "norm, then matvec" and the fused call produce the same bits
// (reference contract: src/kernels/quant.hpp:20-23; reduction being replayed there: src/kernels/quant_mv.metal:72-86).
// `red` is four floats of LDS; all threads of the workgroup must call (it synchronises).
__device__ __forceinline__ float rms_scale(const float* __restrict__ x, uint32_t dim, float eps, float* red, uint32_t lane,
                                           uint32_t wave, uint32_t nwaves) {
  for (uint32_t v = wave; v < 4u; v += nwaves) {
    float ss = 0.f;
    // eight elements are requested before the first is used (one at a time the loop is a chain of memory latencies);
    // indices past the end repeat the last element and are left out of the sum, so the order of additions stays
    for (uint32_t i0 = v * 64u + lane; i0 < dim; i0 += 8u * 256u) {
      float t[8];
#pragma unroll
      for (int k = 0; k < 8; k++) t[k] = x[min(i0 + 256u * k, dim - 1u)];
#pragma unroll
      for (int k = 0; k < 8; k++)
        if (i0 + 256u * k < dim) ss = __builtin_fmaf(t[k], t[k], ss);
    }
    ss = wave_sum(ss);
    if (lane == 0) red[v] = ss;
  }
  __syncthreads();
  const float total = (red[0] + red[1]) + (red[2] + red[3]);
  return 1.0f / __builtin_sqrtf(total / (float)dim + eps);
}

// y[row] = (x[row] * scale) * w (w may be null): reference ms::arch::encode_rmsnorm (src/kernels/arch.hpp:127-130,
// kernel arch_rmsnorm, src/kernels/arch_sample.metal:216-233). One workgroup of 256 threads per row; y may alias x.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* x, const float* __restrict__ w, float* y, uint32_t dim,
                                                      float eps, uint32_t in_stride, uint32_t out_stride) {
  __shared__ float red[4];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const float* xr = x + (size_t)blockIdx.x * in_stride;
  float* yr = y + (size_t)blockIdx.x * out_stride;
  const float r = rms_scale(xr, dim, eps, red, lane, wave, 4u);
  for (uint32_t i0 = tid; i0 < dim; i0 += 4u * 256u) {  // four elements in flight per thread
    float xv[4], wv[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const uint32_t i = min(i0 + 256u * k, dim - 1u);
      xv[k] = xr[i];
      wv[k] = w ? w[i] : 1.f;
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const uint32_t i = i0 + 256u * k;
      if (i < dim) { const float v = xv[k] * r; yr[i] = w ? v * wv[k] : v; }
    }
  }
}

// Prologue of the NORM matvec kernels: the normalized activations of the (single) input row go to LDS as fp32 (padded
// layout of XLds), from where load_x() converts them exactly as it would from device memory.
__device__ __forceinline__ void stage_normed_x(const MvArgs& a, uint32_t* smem, float* xs, uint32_t tid, uint32_t lane, uint32_t wave,
                                               uint32_t nwaves) {
  float* red = (float*)(smem + a.norm_off);
  const float r = rms_scale(a.x, a.cols, a.eps, red, lane, wave, nwaves);
  const uint32_t nt = nwaves * 64u;
  for (uint32_t i0 = tid; i0 < a.cols; i0 += 4u * nt) {  // four elements in flight per thread
    float xv[4], wv[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const uint32_t i = min(i0 + nt * k, a.cols - 1u);
      xv[k] = a.x[i];
      wv[k] = a.norm_w[i];
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const uint32_t i = i0 + nt * k;
      if (i < a.cols) { const float v = xv[k] * r; xs[i + (i >> 5) * 4u] = v * wv[k]; }
    }
  }
  __syncthreads();
}

template <class D, int ITERS, bool NORM = false>
__global__ __launch_bounds__(1024) void mv_kernel(const MvArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  // the codebook table is a static array: its LDS address is a compile-time constant, which saves the addition of a base
  // in every lookup address; partial sums (and staged activations) follow in dynamic LDS
  __shared__ __attribute__((aligned(16))) uint32_t tbl[D::LDS_WORDS > 0 ? D::LDS_WORDS : 4];
  float* part = (float*)smem;

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
  float* xs = (float*)(smem + a.xs_off);
  if constexpr (NORM) stage_normed_x(a, smem, xs, tid, lane, wave, nwaves);  // synchronises (one group only)
  else if (D::LDS_WORDS) __syncthreads();

  for (uint32_t tile = blockIdx.x; tile < a.ntiles; tile += gridDim.x) {
    const uint32_t tile_row0 = tile * tile_rows;
    // a tile never straddles two groups (host guarantees)
    const uint32_t group = a.rows_per_group >= a.rows ? 0u : tile_row0 / a.rows_per_group;
    if (group != cur_group) {
      if constexpr (NORM) {
#pragma unroll
        for (int i = 0; i < ITERS; i++) xr[i] = D::load_x(XLds{xs}, unit[i]);
      } else {
        load_x_row<D, ITERS>(a, xs, a.x + (size_t)group * a.x_group_stride, unit, xr, tid, blockDim.x);
      }
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
          const float s = sum_in_order(part + tid * KS, KS);
          a.y[row] = a.accumulate ? a.y[row] + s : s;
        }
      }
      __syncthreads();
    }
  }
}

// The same matvec with one unit per lane, arranged like the MoE decode kernels: a wave keeps the block bytes of NR rows
// in flight in a register ring that is refilled unconditionally (codebook decoders: range-checked buffer loads with an
// empty descriptor past the end of the wave's rows; the others: the last row again), the first NR rows before the
// tables and activations are staged; codebook table lookups run one decoder stage ahead of the dot products. With a handful of rows
// per wave per launch it is the latency of the first loads, not bandwidth, that such a launch spends its time on.
template <class D>
__global__ __launch_bounds__(1024) void mv_ring_kernel(const MvArgs a) {
  constexpr bool BUFFER = requires { D::STAGES; };  // codebook decoders: buffer loads and staged table lookups
  constexpr int NR = 4;
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  // the codebook table is a static array: its LDS address is a compile-time constant, which saves the addition of a base
  // in every lookup address; partial sums (and staged activations) follow in dynamic LDS
  __shared__ __attribute__((aligned(16))) uint32_t tbl[D::LDS_WORDS > 0 ? D::LDS_WORDS : 4];
  float* part = (float*)smem;

  const uint32_t tid = threadIdx.x, lane = tid & 63u, nwaves = blockDim.x >> 6;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  const uint32_t KS = a.ks, ks = wave % KS, rw = wave / KS, RW = nwaves / KS;
  const uint32_t tile_rows = RW * a.rpw;
  const uint32_t u0 = ks * 64u + lane;
  const bool valid = u0 < a.units;
  const uint32_t unit = valid ? u0 : a.units - 1;  // lanes past the row shadow the last unit with zero activations
  const auto off = [&] { if constexpr (BUFFER) return D::offsets(unit); else return 0; }();
  const uint32_t mat_bytes = a.rows * a.row_bytes;  // buffer loads: < 4 GiB (host-checked)

  typename D::X xr;
  uint32_t cur_group = 0xFFFFFFFFu;
  bool first = true;
  for (uint32_t tile = blockIdx.x; tile < a.ntiles; tile += gridDim.x) {
    const uint32_t tile_row0 = tile * tile_rows;
    const uint32_t row0 = tile_row0 + rw * a.rpw, row1 = min(row0 + a.rpw, a.rows);
    uint32_t pv = row0;
    typename D::Raw ring[NR];
    auto fetch = [&](int s) {
      if constexpr (BUFFER) ring[s] = D::fetch(make_rsrc(a.W, pv < row1 ? mat_bytes : 0u), off, pv * a.row_bytes);
      else ring[s] = D::load(as_global(a.W) + (size_t)min(pv, a.rows - 1) * a.row_bytes, unit);  // past the end: the last row again
      pv++;
    };
#pragma unroll
    for (int s = 0; s < NR; s++) fetch(s);
    if (first) {
      D::fill_lds(tbl, (int)tid, (int)blockDim.x);
      first = false;
      if (D::LDS_WORDS) __syncthreads();
    }
    // a tile never straddles two groups (host guarantees)
    const uint32_t group = a.rows_per_group >= a.rows ? 0u : tile_row0 / a.rows_per_group;
    if (group != cur_group) {
      const uint32_t units1[1] = {unit};
      typename D::X x1[1];
      load_x_row<D, 1>(a, (float*)(smem + a.xs_off), a.x + (size_t)group * a.x_group_stride, units1, x1, tid, blockDim.x);
      xr = x1[0];
      if (!valid) xr = typename D::X{};
      cur_group = group;
    }
    auto lk = [&] { if constexpr (BUFFER) return std::array<typename D::Look, 2>{}; else return 0; }();
    if constexpr (BUFFER) { if (row0 < row1) lk[0] = D::lookup(ring[0], 0, tbl); }
    for (uint32_t r0 = row0; r0 < row1; r0 += NR) {
#pragma unroll
      for (int s = 0; s < NR; s++) {
        const uint32_t row = r0 + s;
        if (row < row1) {  // wave-uniform; no global loads inside
          float v = 0.f;
          if constexpr (BUFFER) {
            constexpr int NS = D::STAGES;
            const bool more = row + 1 < row1;
#pragma unroll
            for (int t = 0; t < NS; t++) {
              const int cur = (s * NS + t) & 1;
              if (t + 1 < NS) lk[cur ^ 1] = D::lookup(ring[s], t + 1, tbl);
              else if (more) lk[cur ^ 1] = D::lookup(ring[(s + 1) % NR], 0, tbl);
              v = D::partial(ring[s], lk[cur], xr, t, v);
              asm volatile("" : "+v"(v));
            }
          } else {
            v = dec_dot<D>(ring[s], xr, tbl, unit);
          }
          v = wave_sum(valid ? v : 0.f);
          if (KS == 1) {
            if (lane == 0) a.y[row] = a.accumulate ? a.y[row] + v : v;
          } else if (lane == 0) {
            part[(row - tile_row0) * KS + ks] = v;
          }
        }
        fetch(s);
      }
    }
    if (KS > 1) {
      __syncthreads();
      if (tid < tile_rows) {
        const uint32_t row = tile_row0 + tid;
        if (row < a.rows) {
          const float sum = sum_in_order(part + tid * KS, KS);
          a.y[row] = a.accumulate ? a.y[row] + sum : sum;
        }
      }
      __syncthreads();
    }
  }
}

// Small-N form of mv_kernel: T tokens per pass over the weights (reference operator: ms::q::encode_matvec_n,
// src/kernels/quant.mm:129-156; reference kernel q_mvn, src/kernels/quant_mv.metal:148-202). A lane keeps the
// activation slices of T tokens; a weight unit is fetched once and its decode is shared by the T dot products (the T
// calls of dec_dot are inlined over the same raw bytes, so only the dot2 chains differ). blockIdx.y picks the token
// group: groups beyond the first find the weights in the caches. Lanes are laid out over a row exactly as in
// mv_kernel, so every load is a contiguous run over the wave.
struct MvTokArgs {
  MvArgs m;
  uint32_t n;                    // tokens
  uint32_t x_stride, y_stride;   // elements between the activation / output rows of consecutive tokens
};

// Tokens whose activation rows a workgroup stages in LDS per round (a decoder with a large table leaves less room).
template <class D, int T>
constexpr int tok_round() {
  constexpr int g = D::LDS_WORDS * 4 > 16 * 1024 ? 2 : 4;
  return T < g ? T : g;
}

// Whether the T-token kernel of decoder D takes its activations through LDS: the decoders with STAGE_X always; the other
// block formats in the four-token instantiation. Their lane slices are short runs (Q6_K: four runs of 32 bytes per
// token), read straight from device memory for one or two tokens; at four tokens one staged round is faster (Q6_K
// 1536x7168 8.9 -> 8.5 us, Q5_K 512x7168 7.0 -> 6.5), at eight the two rounds cost more than they save (11.3 -> 12.7).
template <class D, int T>
constexpr bool tok_stages_x() { return D::STAGE_X || (T == 4 && D::UNIT == 32); }

// Whether the T-token kernel of decoder D copies its weight rows through LDS (one token of a block format; see the kernel),
// the bytes of a wave's slice of a row (its 64 units' blocks; fewer at the end of the row), and the 16-byte pieces per
// lane that cover a slice at any alignment.
template <class D, int ITERS, int T>
constexpr bool tok_stages_w() {
  if constexpr (requires { D::BLOCK; }) return T == 1 && ITERS == 1;
  else return false;
}
template <class D>
__host__ __device__ constexpr uint32_t wspan_bytes() {
  if constexpr (requires { D::BLOCK; }) return (64u / D::UPB) * D::BLOCK;
  else return 0u;
}
template <class D>
__host__ __device__ constexpr uint32_t wspan_loads() { return (wspan_bytes<D>() + 14u + 1023u) / 1024u; }
template <class D>
__device__ __forceinline__ uint32_t wspan_len(uint32_t units, uint32_t ks) {
  if constexpr (requires { D::BLOCK; }) {
    constexpr uint32_t SB = 64u / D::UPB;
    const uint32_t nblk = units / D::UPB, b0 = ks * SB;
    return (min(b0 + SB, nblk) - b0) * D::BLOCK;
  } else return 0u;
}

template <int N>
__device__ __forceinline__ void wait_rows() { wait_vm<N>(); }
// the same for a count that is a constant only after unrolling (0 .. 9)
__device__ __forceinline__ void wait_rows_n(int n) {
  switch (n) {
    case 0: wait_rows<0>(); break;
    case 1: wait_rows<1>(); break;
    case 2: wait_rows<2>(); break;
    case 3: wait_rows<3>(); break;
    case 4: wait_rows<4>(); break;
    case 5: wait_rows<5>(); break;
    case 6: wait_rows<6>(); break;
    case 7: wait_rows<7>(); break;
    case 8: wait_rows<8>(); break;
    case 9: wait_rows<9>(); break;
    default: wait_rows<0>(); break;
  }
}

// Decoders with STAGE_X take the activations through LDS (contiguous loads, tok_round() tokens per round); with the
// others every lane reads its slices from device memory, all T tokens' loads in flight at once.
// PAIR (with SW): the launch treats two consecutive rows as one row of twice the units -- rows are contiguous in memory,
// so a wave's slice of 64 units may run from the end of one row into the next -- which leaves no lane idle when a row's
// units fill a whole number of waves and a half (5120 columns: five waves per row pair instead of twice three). rows_,
// row_bytes_, units_, ks_ and the tile shape then describe the pairs; the two rows' 16-lane sums are told apart when
// the partial sums are added (a row's units must be a multiple of 16 for that).
template <class D, int ITERS, int T, bool NORM = false, bool SW = false, bool PAIR = false>
__global__ __launch_bounds__(512) void mv_tok_kernel(const uint8_t* W_, uint32_t rows_, uint32_t row_bytes_, uint32_t units_, uint32_t ks_,
                                                     uint32_t rpw_, uint32_t ntiles_, uint32_t rows_per_group_, const float* x_,
                                                     uint32_t cols_, const MvTokArgs ta) {
  constexpr bool STAGE = tok_stages_x<D, T>();
  constexpr bool STAGE_W = SW && tok_stages_w<D, ITERS, T>();  // weight rows through LDS: the launch's choice (large matrices)
  constexpr int WL = STAGE_W ? (int)wspan_loads<D>() : 1;
  // What the first loads need comes as leading arguments (W_ .. cols_: the fields of the same names in ta.m, delivered
  // in scalar registers with the wave when the file is built with kernel-argument preload) and is used under those
  // names below; the rest is read from the argument block.
  const MvArgs& a = ta.m;
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  // the codebook table is a static array: its LDS address is a compile-time constant, which saves the addition of a base
  // in every lookup address; partial sums (and staged activations) follow in dynamic LDS
  __shared__ __attribute__((aligned(16))) uint32_t tbl[D::LDS_WORDS > 0 ? D::LDS_WORDS : 4];
  float* part = (float*)smem;  // [row of tile][ks][16-lane row of the wave][T]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, nwaves = blockDim.x >> 6;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  // (the quotients come from the vector unit: brought back to scalar registers, the wave's row offsets are scalar too)
  const uint32_t KS = ks_, rw = (uint32_t)__builtin_amdgcn_readfirstlane((int)small_div(wave, KS)), ks = wave - rw * KS;
  const uint32_t RW = (uint32_t)__builtin_amdgcn_readfirstlane((int)small_div(nwaves, KS));
  const uint32_t tile_rows = RW * rpw_;
  const uint32_t t0 = blockIdx.y * T;

  // One token of one group: its activations are requested before anything else, so that they come back ahead of the
  // table and the weight rows (loads return in order) and are in LDS, converted, when the first rows arrive.
  constexpr bool EARLY_X = T == 1 && STAGE && !NORM;
  constexpr int XK = 4;
  [[maybe_unused]] u32x4 xe[XK];
  [[maybe_unused]] bool early = false;
  if constexpr (EARLY_X) {
    const uint32_t n4 = cols_ >> 2;
    early = blockIdx.y == 0 && rows_per_group_ >= rows_ && n4 <= XK * blockDim.x;
    if (early) {
#pragma unroll
      for (int k = 0; k < XK; k++) xe[k] = ((const u32x4*)x_)[min(tid + k * blockDim.x, n4 - 1u)];
    }
  }
  D::fill_lds(tbl, (int)tid, (int)blockDim.x);

  uint32_t unit[ITERS];
  bool valid[ITERS];
#pragma unroll
  for (int i = 0; i < ITERS; i++) {
    const uint32_t u = (ks * ITERS + i) * 64u + lane;
    valid[i] = u < units_;
    unit[i] = valid[i] ? u : units_ - 1;  // idle lanes shadow the last unit; their result is dropped
  }
  uint32_t xu[ITERS];  // the unit of the activations that goes with unit[i] (second row of a pair: the same columns again)
#pragma unroll
  for (int i = 0; i < ITERS; i++) xu[i] = PAIR && unit[i] >= (units_ >> 1) ? unit[i] - (units_ >> 1) : unit[i];
  typename D::X xr[T][ITERS];
  uint32_t cur_group = 0xFFFFFFFFu;
  float* xs = (float*)(smem + a.xs_off);
  if constexpr (NORM) stage_normed_x(a, smem, xs, tid, lane, wave, nwaves);  // synchronises (one token, one group)
  else if (D::LDS_WORDS) __syncthreads();
  const uint32_t roww = xlds_words(cols_);

  for (uint32_t tile = blockIdx.x; tile < ntiles_; tile += gridDim.x) {
    const uint32_t tile_row0 = tile * tile_rows;
    // a tile never straddles two groups (host guarantees)
    const uint32_t group = rows_per_group_ >= rows_ ? 0u : tile_row0 / rows_per_group_;
    const uint32_t row0 = tile_row0 + rw * rpw_;
    const uint32_t last = min(min(row0 + rpw_, rows_) - 1u, rows_ - 1u);  // last row of this wave's run
    // The wave's first NR rows are on their way while the activations are staged; a slot is refilled with the row NR
    // places ahead as soon as its bytes are consumed. Rows are reached through a buffer descriptor over the wave's run
    // (BufRow): the row offset is a scalar, the lane offsets are loop constants, and a refill past the end of the run
    // takes an empty descriptor (zeros, no memory access) instead of a branch around the load, so that every wait names
    // an exact number of loads that may stay in flight.
    // One token keeps four rows in flight per wave (large matrices are bound by the bytes a CU has in flight, and a
    // second workgroup per CU, mv_tok_shape, adds to them); several tokens, whose activation slices fill the registers, two.
    constexpr int NR = T == 1 ? 4 : 2;
    const uint32_t run_rows = row0 <= last ? last - row0 + 1u : 0u;
    // ---- one token of a block format, large matrix: the wave's slice of a row -- the consecutive blocks of its 64 units,
    // one contiguous run of bytes -- is fetched as aligned 16-byte pieces, consecutive lanes consecutive pieces (one to
    // three loads per lane and row, each cache line requested once), straight into a slot of the wave's own LDS ring
    // (loads with an LDS destination), and read from there by the decoder's load(). A lane's pieces of a block lie in
    // the same few cache lines as its neighbours', and fetched lane by lane every one of a decoder's three to six loads
    // asks for all lines of the slice again; the vector cache then holds several requests per line in its queue, and
    // that queue, not memory, bounds the launch (Q6_K 129280x5120 with the arithmetic taken out: 133 us with Q6_K's
    // five loads per lane, 107 with three of them, 89 with one, 85 with two loads of consecutive 16-byte pieces -- the
    // speed of a plain read).
    // The compiler does not know that such a load writes LDS: the waits for a slot's loads (wait_rows) and the order of
    // slot reads and refills are written out below. Loads complete in order, so "at most k row requests outstanding"
    // means every older one has landed; other loads and stores in flight only make a wait stricter.
    [[maybe_unused]] typename D::Raw ring[STAGE_W ? 1 : NR][ITERS];
    [[maybe_unused]] typename D::Raw raw[2];
    [[maybe_unused]] uint32_t span_at = 0, w_low = 0;  // the slice's byte offset in a row; low address bits of the run's first slice
    [[maybe_unused]] rsrc_t w_rs, w_none;
    [[maybe_unused]] uint8_t* wbuf = nullptr;
    if constexpr (STAGE_W) {
      constexpr uint32_t SB = 64u / D::UPB;  // blocks of the wave's 64 units
      const uint32_t nblk = units_ / D::UPB, b0 = ks * SB;
      span_at = b0 * D::BLOCK;
      const uint32_t span_len = (min(b0 + SB, nblk) - b0) * D::BLOCK;
      const uint64_t first = (uint64_t)(uintptr_t)W_ + (uint64_t)min(row0, last) * row_bytes_ + span_at;
      w_low = (uint32_t)first & 15u;
      const uint32_t covered = run_rows ? (w_low + (run_rows - 1u) * row_bytes_ + span_len + 15u) & ~15u : 0u;
      w_rs = make_rsrc((const void*)(uintptr_t)(first & ~15ull), covered);
      w_none = make_rsrc((const void*)(uintptr_t)(first & ~15ull), 0u);
      wbuf = (uint8_t*)(smem + a.w_off) + wave * (NR * WL * 1024u);
    }
    // request row j of the run into slot s (past the end of the run: zeros, no memory access)
    auto request = [&](int s, uint32_t j) {
      typedef __attribute__((address_space(3))) void* lds_ptr_t;
      const uint32_t so = w_low + j * row_bytes_;                   // bytes from the descriptor's base to the slice
      const uint32_t top = ((so & 15u) + wspan_len<D>(units_, ks) - 1u) & ~15u;  // offset of the slice's last piece
      asm volatile("" ::: "memory");  // behind the reads of the slot's previous row
#pragma unroll
      for (int k = 0; k < WL; k++)  // lane l's piece lands at the given LDS address + 16 l
        __builtin_amdgcn_raw_ptr_buffer_load_lds(j < run_rows ? w_rs : w_none, (lds_ptr_t)(wbuf + (s * WL + k) * 1024u), 16,
                                                 (int)min(16u * lane + 1024u * k, top), (int)(so & ~15u), 0, 0);
    };
    auto take = [&](int s, uint32_t j) {  // the lane's block bytes of row j, which slot s holds
      return D::load(LdsRow::of(wbuf + s * WL * 1024u, ((w_low + j * row_bytes_) & 15u) - span_at), unit[0]);
    };
    const uint8_t* run_base = W_ + (size_t)min(row0, last) * row_bytes_;
    auto fetch = [&](typename D::Raw (&slot)[ITERS], uint32_t j) {  // row j of the wave's run; past its end: zeros, no memory access
      const BufRow wr = {make_rsrc(run_base, j < run_rows ? run_rows * row_bytes_ : 0u), j * row_bytes_, 0u};
#pragma unroll
      for (int i = 0; i < ITERS; i++) slot[i] = D::load(wr, unit[i]);
    };
    // Half of the ring is requested ahead of the activations, the other half behind them: loads return in order, so with
    // the whole ring ahead the activations of a small matrix wait for four rows.
    constexpr int AHEAD = NR / 2;
#pragma unroll
    for (int s = 0; s < AHEAD; s++) {
      if constexpr (STAGE_W) request(s, s);
      else fetch(ring[s], s);
    }
    if (group != cur_group) {
      // tokens past the last repeat it; their results are never stored
      auto x_of = [&](int t) { return x_ + (size_t)min(t0 + t, ta.n - 1) * ta.x_stride + (size_t)group * a.x_group_stride; };
      constexpr int G = tok_round<D, T>();  // tokens staged per round (the host has made room for G padded rows)
      bool staged = false;
      if constexpr (EARLY_X) {
        if (early && cur_group == 0xFFFFFFFFu) {  // (group 0, token 0: the row requested at the top)
#pragma unroll
          for (int k = 0; k < XK; k++) {
            const uint32_t i = tid + k * blockDim.x;
            if (i < (cols_ >> 2)) *(u32x4*)(xs + 4u * i + (i >> 3) * 4u) = xe[k];
          }
          __syncthreads();
#pragma unroll
          for (int i = 0; i < ITERS; i++) xr[0][i] = D::load_x(XLds{xs}, xu[i]);
          staged = true;
        }
      }
      if (!staged) {
#pragma unroll
      for (int t = 0; t < T; t++) {
        if constexpr (NORM) {
#pragma unroll
          for (int i = 0; i < ITERS; i++) xr[t][i] = D::load_x(XLds{xs}, xu[i]);
        } else if constexpr (!STAGE) {
#pragma unroll
          for (int i = 0; i < ITERS; i++) xr[t][i] = D::load_x(x_of(t), xu[i]);
        } else if (!D::STAGE_X && !a.stage_x) {  // (rows too long for a round of G in LDS: read directly, as for few tokens)
#pragma unroll
          for (int i = 0; i < ITERS; i++) xr[t][i] = D::load_x(x_of(t), xu[i]);
        } else {
          if (t % G == 0) {
            __syncthreads();  // readers of the previous round are done
            const float* src[G];
#pragma unroll
            for (int k = 0; k < G; k++) src[k] = x_of(t + k);
            stage_x_rows<G>(xs, src, G, roww, cols_, tid, blockDim.x);
            __syncthreads();
          }
#pragma unroll
          for (int i = 0; i < ITERS; i++) xr[t][i] = D::load_x(XLds{xs + (t % G) * roww}, xu[i]);
        }
      }
      }
      cur_group = group;
    }
#pragma unroll
    for (int s = AHEAD; s < NR; s++) {
      if constexpr (STAGE_W) request(s, s);
      else fetch(ring[s], s);
    }
    // RF rows' results are folded over the lanes together (a fold takes up to eight values): afterwards lane l holds
    // value k = group8_sel(l), row k / T of the group and token k % T, summed over l's 16-lane row
    constexpr int RF = NR * T <= 8 ? NR : 2 * T <= 8 ? 2 : 1;
    if constexpr (STAGE_W) {  // row 0 to registers
      wait_rows<(NR - 1) * WL>();
      raw[0] = take(0, 0);
    }
    // A round = the NR rows the ring holds. Rounds with more rows behind them refill every slot (with an empty descriptor
    // past the end of the run); the last round requests nothing, so a short run pays for no loads it does not need.
    auto round = [&]<bool REFILL>(uint32_t j0) {
#pragma unroll
      for (int f = 0; f < NR; f += RF) {
        float acc[RF * T];
#pragma unroll
        for (int q = 0; q < RF; q++) {
          const int s = f + q;
#pragma unroll
          for (int t = 0; t < T; t++) acc[q * T + t] = 0.f;
          if constexpr (STAGE_W) {
            // the next row moves to the other register set while this one is multiplied; this row's slot, whose bytes
            // the multiplication has consumed, is then requested again
            if (REFILL || s + 1 < NR) {  // (a constant: the loops are unrolled)
              wait_rows_n((REFILL ? NR - 2 : NR - 2 - s) * WL);  // row requests behind the next row's
              raw[(s + 1) & 1] = take((s + 1) % NR, j0 + s + 1);
            }
            if (j0 + s < rpw_) {
              const float v = dec_dot<D>(raw[s & 1], xr[0][0], tbl, unit[0]);
              acc[q] = valid[0] ? v : 0.f;
            }
            if constexpr (REFILL) request(s, j0 + s + NR);
          } else {
            if (j0 + s < rpw_) {  // wave-uniform; no load inside (a row past the run is not decoded)
#pragma unroll
              for (int t = 0; t < T; t++) {
#pragma unroll
                for (int i = 0; i < ITERS; i++) {
                  const float v = dec_dot<D>(ring[s][i], xr[t][i], tbl, unit[i]);
                  acc[q * T + t] += valid[i] ? v : 0.f;
                }
              }
            }
            if constexpr (REFILL) fetch(ring[s], j0 + s + NR);
          }
        }
        row16_fold<RF * T>(acc, lane);
        const uint32_t k = group8_sel<RF * T>(lane), j = j0 + f + k / T;
        if (!(lane & 8u) && j < rpw_) part[(((rw * rpw_ + j) * KS + ks) * 4 + (lane >> 4)) * T + k % T] = acc[0];
      }
    };
    uint32_t j0 = 0;
    for (; j0 + NR < rpw_; j0 += NR) round.template operator()<true>(j0);
    round.template operator()<false>(j0);
    __syncthreads();
    if constexpr (PAIR) {  // pair r / 2, its first or second units / 32 sixteen-lane sums
      const uint32_t G = units_ >> 5;
      for (uint32_t idx = tid; idx < 2u * tile_rows * T; idx += blockDim.x) {
        const uint32_t r = idx % (2u * tile_rows), t = idx / (2u * tile_rows), row = 2u * tile_row0 + r;
        if (row < 2u * rows_ && t0 + t < ta.n) {
          const float s = sum_in_order(part + ((r >> 1) * 4 * KS + (r & 1u) * G) * T + t, G, T);
          float* y = a.y + (size_t)(t0 + t) * ta.y_stride + row;
          *y = a.accumulate ? *y + s : s;
        }
      }
    } else
    for (uint32_t idx = tid; idx < tile_rows * T; idx += blockDim.x) {
      const uint32_t r = idx % tile_rows, t = idx / tile_rows, row = tile_row0 + r;  // consecutive lanes: consecutive rows
      if (row < rows_ && t0 + t < ta.n) {
        const float s = sum_in_order(part + r * 4 * KS * T + t, 4 * KS, T);
        float* y = a.y + (size_t)(t0 + t) * ta.y_stride + row;
        *y = a.accumulate ? *y + s : s;
      }
    }
    __syncthreads();
  }
}

}  // namespace msq
