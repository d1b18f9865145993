// Small-N matvec for speculative verify: Y[t][r] (+)= W[r] . X[t], t < n <= 16 (reference operator:
// ms::q::encode_matvec_n, src/kernels/quant.mm:129-156; reference kernels q_mvn, src/kernels/quant_mv.metal:148-202,
// and for n >= 8 the tile matmul q_mm, src/kernels/quant_mm.metal:81-115).
//
// One weight read serves all n tokens through the matrix cores: a 16-row tile of W is the B operand, the (up to 16)
// tokens are the A operand. A workgroup is KS waves that split K; a wave takes its K steps eight at a time: the weight
// fragments of all eight are requested before the first MFMA, the activations are MFMA A fragments in registers (kept
// for the whole launch when a wave has at most eight steps); the workgroups walk the row tiles (persistent grid). Per
// tile the KS partial 16 x 16 results meet in LDS and are added in a fixed order. msq_matvec_n uses this kernel for
// rows too wide for the dot-product kernel (mv_tok_kernel) and for many tokens over large matrices.
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
  uint32_t nsteps;               // K steps of 32 columns
  uint32_t steps_per_wave;
  uint32_t ntiles;               // ceil(rows / 16)
};

template <class F>
__global__ __launch_bounds__(1024) void mvn_kernel(const MvnArgs a) {
  constexpr int MS = kMvnSubSteps;
  constexpr bool HALF_SCALES = requires(const uint8_t* r, float& s) { F::get_scales(r, 0u, s, s); };
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  __shared__ __attribute__((aligned(16))) uint32_t tbl[F::LDS_WORDS > 0 ? F::LDS_WORDS : 4];  // static: a known address
  float* red = (float*)smem;  // [wave][token][17]

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6)), nwaves = blockDim.x >> 6;
  const uint32_t m16 = lane & 15u, q = lane >> 4;  // A: token m16; B: weight row m16; both: chunk q of the K step
  const uint32_t S = a.steps_per_wave, s0 = wave * S;

  F::fill_lds(tbl, (int)tid, (int)blockDim.x);

  // activations of MS of this wave's K steps at a time, as A fragments (token m16, chunk q); bf16 math splits x into
  // hi + lo. A wave with at most MS steps keeps them for the whole launch.
  uint32_t xa[MS][4];
  uint32_t xb[F::BF16_MATH ? MS : 1][4];
  auto load_x = [&](uint32_t group, uint32_t c0) {
    // all requests first, then the conversions (scheduling barrier in between): left to itself the scheduler pairs
    // each step's loads with their conversion and waits for every step separately. No branch around the loads either
    // (a wait after a conditional load waits for everything in flight): lanes past the last token repeat it -- their
    // output rows are never stored -- and steps past the end repeat the last one, which the MFMA loop skips.
    float4 raw[MS][2];
#pragma unroll
    for (int i = 0; i < MS; i++) {
      const uint32_t step = min(s0 + c0 + i, a.nsteps - 1);
      const float* xs = a.X + (size_t)min(m16, a.n - 1) * a.x_stride + (size_t)group * a.x_group_stride + 32u * step;
      // the chunk's 8 columns as two 128-bit loads (col_of is 8 q + p, or for IQ4_NL 4 q + p / 2 + 16 (p % 2))
      const bool natural = F::col_of(1, 1) == 9u;
      raw[i][0] = *(const float4*)(xs + (natural ? 8u * q : 4u * q));
      raw[i][1] = *(const float4*)(xs + (natural ? 8u * q + 4u : 4u * q + 16u));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < MS; i++) {
      const float4 lo = raw[i][0], hi = raw[i][1];
      float v[8];
      if (F::col_of(1, 1) == 9u) {
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
      } else {
        v[0] = lo.x; v[1] = hi.x; v[2] = lo.y; v[3] = hi.y; v[4] = lo.z; v[5] = hi.z; v[6] = lo.w; v[7] = hi.w;
      }
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
    }
  };
  uint32_t cur_group = 0xFFFFFFFFu;
  if (F::LDS_WORDS) __syncthreads();

  const uint32_t ones[4] = {0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
  for (uint32_t tile = blockIdx.x; tile < a.ntiles; tile += gridDim.x) {
    const uint32_t group = (tile * 16u) / a.rows_per_group;  // a tile never straddles two groups (host guarantees)
    const uint32_t row = min(tile * 16u + m16, a.rows - 1);
    const gptr_t wr = as_global(a.W) + (size_t)row * a.row_bytes;
    f4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t c0 = 0; c0 < S; c0 += MS) {
      // all of the sub-chunk's weight fragments are requested (and decoded as they arrive) before the first MFMA:
      // a wave's steps are independent, and fetched one at a time each would cost a full memory latency
      // activations first: their raw fp32 form takes twice the registers of the packed fragments, and requested
      // after the weights they would be fetched and waited for one step at a time
      if (S > MS || group != cur_group) {
        load_x(group, c0);
        cur_group = group;
        __builtin_amdgcn_sched_barrier(0);
      }
      FragOut fr[MS];
      float sa[HALF_SCALES ? MS : 1], sb[HALF_SCALES ? MS : 1];
#pragma unroll
      for (int i = 0; i < MS; i++) {
        const uint32_t step = min(s0 + c0 + i, a.nsteps - 1);  // past the end: the last step again, never multiplied
        fr[i] = F::get(wr, step, q, tbl);
        if constexpr (HALF_SCALES) F::get_scales(wr, step, sa[i], sb[i]);
      }
#pragma unroll
      for (int i = 0; i < MS; i++) {
        const uint32_t step = s0 + c0 + i;
        if (c0 + i < S && step < a.nsteps) {  // wave-uniform
          const f4_t zero = {0.f, 0.f, 0.f, 0.f};
          const FragOut& f = fr[i];
          if constexpr (HALF_SCALES) {
            // half-step scale groups: chunks 0-1 and chunks 2-3 go through separate MFMAs
            uint32_t ha[4], hb[4];
#pragma unroll
            for (int p = 0; p < 4; p++) { ha[p] = q < 2 ? f.h[p] : 0u; hb[p] = q < 2 ? 0u : f.h[p]; }
            const f4_t pa = mfma_f16(xa[i], ha, zero), pb = mfma_f16(xa[i], hb, zero);
            acc += sa[i] * pa + sb[i] * pb;
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
