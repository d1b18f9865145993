// Small-N matvec for speculative verify: Y[t][r] (+)= W[r] . X[t], t < n <= 16 (reference operator:
// ms::q::encode_matvec_n, src/kernels/quant.mm:129-156; reference kernels q_mvn, src/kernels/quant_mv.metal:148-202,
// and for n >= 8 the tile matmul q_mm, src/kernels/quant_mm.metal:81-115).
//
// One weight read serves all n tokens through the matrix cores: a 16-row tile of W is the B operand, the (up to 16)
// tokens are the A operand. A workgroup is KS waves that split K; each wave keeps the activations of its K steps in
// registers as MFMA A fragments for the whole launch and walks the row tiles (persistent grid), so weights are the
// only HBM stream. Per tile the KS partial 16 x 16 results meet in LDS and are added in a fixed order.
#pragma once
#include "msq_mfma.cuh"

namespace msq {

struct MvnArgs {
  const uint8_t* W;
  const float* X;
  float* Y;
  uint32_t rows, cols, row_bytes, n;
  uint32_t x_stride, y_stride;   // elements between activation / output rows of consecutive tokens
  uint32_t rows_per_group, x_group_stride;
  uint32_t accumulate;
  uint32_t col0, col0_bytes;     // first column this launch covers and its byte offset in a row (K chunking)
  uint32_t nsteps;               // K steps this launch covers
  uint32_t steps_per_wave;
  uint32_t ntiles;               // ceil(rows / 16)
  int qtype;
};

// byte offset of column `col` (a multiple of 256) inside a row
inline size_t msq_type_row_bytes_of_cols(const MvnArgs& a, uint32_t col) { return msq_type_row_bytes(a.qtype, col); }

template <class F>
__global__ __launch_bounds__(1024) void mvn_kernel(const MvnArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  uint32_t* tbl = smem;
  float* red = (float*)(smem + F::LDS_WORDS);  // [wave][token][17]

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6)), nwaves = blockDim.x >> 6;
  const uint32_t m16 = lane & 15u, q = lane >> 4;  // A: token m16; B: weight row m16; both: chunk q of the K step
  const uint32_t S = a.steps_per_wave, s0 = wave * S;

  F::fill_lds(tbl, (int)tid, (int)blockDim.x);

  // activations of this wave's K steps, as A fragments (token m16, chunk q); bf16 math splits x into hi + lo
  uint32_t xa[kMvnMaxSteps][4];
  uint32_t xb[F::BF16_MATH ? kMvnMaxSteps : 1][4];
  auto load_x = [&](uint32_t group) {
#pragma unroll
    for (int i = 0; i < kMvnMaxSteps; i++) {
      const uint32_t step = s0 + i;
      if ((uint32_t)i < S && step < a.nsteps && m16 < a.n) {
        const float* xs = a.X + (size_t)m16 * a.x_stride + (size_t)group * a.x_group_stride + a.col0 + 32u * step;
        float v[8];
#pragma unroll
        for (int p = 0; p < 8; p++) v[p] = xs[F::col_of(q, p)];
#pragma unroll
        for (int p = 0; p < 4; p++) {
          if constexpr (F::BF16_MATH) {
            const uint32_t h0 = bf16_rne(v[2 * p]), h1 = bf16_rne(v[2 * p + 1]);
            const float r0 = v[2 * p] - __builtin_bit_cast(float, h0 << 16), r1 = v[2 * p + 1] - __builtin_bit_cast(float, h1 << 16);
            xa[i][p] = h0 | (h1 << 16);
            xb[i][p] = bf16_rne(r0) | (bf16_rne(r1) << 16);
          } else {
            xa[i][p] = pack_h2(v[2 * p], v[2 * p + 1]);
          }
        }
      } else {
#pragma unroll
        for (int p = 0; p < 4; p++) { xa[i][p] = 0u; if constexpr (F::BF16_MATH) xb[i][p] = 0u; }
      }
    }
  };
  uint32_t cur_group = 0xFFFFFFFFu;
  if (F::LDS_WORDS) __syncthreads();

  const uint32_t ones[4] = {0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
  for (uint32_t tile = blockIdx.x; tile < a.ntiles; tile += gridDim.x) {
    const uint32_t group = (tile * 16u) / a.rows_per_group;  // a tile never straddles two groups (host guarantees)
    if (group != cur_group) { load_x(group); cur_group = group; }
    const uint32_t row = min(tile * 16u + m16, a.rows - 1);
    const uint8_t* wr = a.W + (size_t)row * a.row_bytes + a.col0_bytes;
    f4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < kMvnMaxSteps; i++) {
      const uint32_t step = s0 + i;
      if ((uint32_t)i < S && step < a.nsteps) {  // wave-uniform
        const f4_t zero = {0.f, 0.f, 0.f, 0.f};
        const FragOut f = F::get(wr, step, q, tbl);
        if constexpr (requires(float& s) { F::get_scales(wr, step, s, s); }) {
          // half-step scale groups: chunks 0-1 and chunks 2-3 go through separate MFMAs
          float sa, sb;
          F::get_scales(wr, step, sa, sb);
          uint32_t ha[4], hb[4];
#pragma unroll
          for (int p = 0; p < 4; p++) { ha[p] = q < 2 ? f.h[p] : 0u; hb[p] = q < 2 ? 0u : f.h[p]; }
          const f4_t pa = mfma_f16(xa[i], ha, zero), pb = mfma_f16(xa[i], hb, zero);
          acc += sa * pa + sb * pb;
        } else if constexpr (F::BF16_MATH) {
          f4_t p = mfma_bf16(xa[i], f.h, zero);
          p = mfma_bf16(xb[i], f.h, p);
          acc += f.scale * p;
        } else {
          const f4_t p = mfma_f16(xa[i], f.h, zero);
          acc += f.scale * p;
          if constexpr (F::HAS_ADD) acc += f.add * mfma_f16(xa[i], ones, zero);  // per-token sum of the step's x
        }
      }
    }
    // acc[i] = partial of (token 4 q + i, weight row tile * 16 + m16)
#pragma unroll
    for (int i = 0; i < 4; i++) red[(wave * 16u + 4u * q + i) * 17u + m16] = acc[i];
    __syncthreads();
    for (uint32_t idx = tid; idx < 16u * a.n; idx += blockDim.x) {
      const uint32_t t = idx >> 4, r = idx & 15u, orow = tile * 16u + r;
      if (orow < a.rows) {
        float s = 0.f;
        for (uint32_t w = 0; w < nwaves; w++) s += red[(w * 16u + t) * 17u + r];
        float* y = a.Y + (size_t)t * a.y_stride + orow;
        *y = a.accumulate ? *y + s : s;
      }
    }
    __syncthreads();
  }
}

}  // namespace msq
