// Prefill matmul Y[n x rows] (+)= X[n x cols] . W^T with the dequantization fused into the GEMM tiles (reference
// operator: ms::q::encode_matmul / encode_matmul_h, src/kernels/quant.mm:159-248; reference kernel q_mm,
// src/kernels/quant_mm.metal:87-115). Numerics are the reference's: activations and weights rounded to fp16, fp32
// accumulation (quant.hpp:36-39).
//
// A workgroup of WV waves owns 16 WV weight rows x 16 TM tokens of one K slice (blockIdx.z). A workgroup's K loop is a
// chain of stage latencies and a small matrix has few tiles, so the host cuts K into slices until the device holds about
// two workgroups per CU; every slice leaves its tile in a partial-sum buffer and mm_reduce_kernel adds the slices in
// their order (no floating-point atomics: the result does not depend on which slice finishes first). A wave owns one 16-row tile of W: per K step
// (32 columns) it decodes the lane's eight weights into exact fp16 payloads + fp32 scale (the fragment decoders of
// msq_mfma.cuh), rounds scale * payload (+ add) to fp16 once (v_fma_mix: fp32 arithmetic, one rounding -- the value
// the reference's dequantized tile holds) and feeds TM matrix instructions, one per token tile. The activation tile
// [16 TM tokens][128 columns] is staged in LDS for all waves, double-buffered, one barrier per 128 columns;
// F32 activations are rounded to fp16 on their way into LDS, so no fp16 copy of X or W is ever materialised.
#pragma once
#include "msq_mfma.cuh"

namespace msq {

struct MmArgs {
  const void* X;       // activations [n][x_stride]: fp16, or fp32 (X_F32)
  const uint8_t* W;    // raw block rows
  float* Y;            // [n][rows]
  uint32_t n, rows, cols, x_stride, row_bytes, accumulate;
  uint32_t slice_stages;  // 128-column stages per K slice (blockIdx.z picks the slice)
  float* partials;        // several K slices: slice z leaves its tile in partials[z][n][rows] and a second kernel adds the
                          // slices in order (null: one slice, written to Y directly)
};

// F32 and BF16 weight rows as fp16 payloads (the matmul multiplies every type as fp16)
struct FragF32H {
  static constexpr bool BF16_MATH = false, HAS_ADD = false, PLAIN = true;
  static constexpr int LDS_WORDS = 0;
  __device__ static void fill_lds(uint32_t*, int, int) {}
  __device__ static uint32_t col_of(uint32_t q, uint32_t p) { return 8u * q + p; }
  template <class P>
  __device__ static FragOut get(P row, uint32_t step, uint32_t q, const uint32_t*) {
    const u128_a2 a = ld128(row + 128u * step + 32u * q), b = ld128(row + 128u * step + 32u * q + 16);
    auto f = [](uint32_t v) { return __builtin_bit_cast(float, v); };
    FragOut o;
    o.h[0] = pack_h2(f(a.x), f(a.y)); o.h[1] = pack_h2(f(a.z), f(a.w));
    o.h[2] = pack_h2(f(b.x), f(b.y)); o.h[3] = pack_h2(f(b.z), f(b.w));
    o.scale = 1.f; o.add = 0.f;
    return o;
  }
};
struct FragBF16H {
  static constexpr bool BF16_MATH = false, HAS_ADD = false, PLAIN = true;
  static constexpr int LDS_WORDS = 0;
  __device__ static void fill_lds(uint32_t*, int, int) {}
  __device__ static uint32_t col_of(uint32_t q, uint32_t p) { return 8u * q + p; }
  template <class P>
  __device__ static FragOut get(P row, uint32_t step, uint32_t q, const uint32_t*) {
    const u128_a2 v = ld128(row + 64u * step + 16u * q);
    auto two = [](uint32_t w) { return pack_h2(__builtin_bit_cast(float, w << 16), __builtin_bit_cast(float, w & 0xFFFF0000u)); };
    FragOut o;
    o.h[0] = two(v.x); o.h[1] = two(v.y); o.h[2] = two(v.z); o.h[3] = two(v.w);
    o.scale = 1.f; o.add = 0.f;
    return o;
  }
};

// fp16(scale * payload + add) for both halves of a payload word: fp32 arithmetic on the fp16 payloads, one rounding
__device__ __forceinline__ uint32_t scale_round_h2(uint32_t h, float scale, float add) {
  uint32_t r;
  asm("v_fma_mixlo_f16 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(h), "v"(scale), "v"(add));
  asm("v_fma_mixhi_f16 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(r) : "v"(h), "v"(scale), "v"(add));
  return r;
}

constexpr int kMmKStage = 128, kMmPitch = kMmKStage * 2 + 16;  // bytes per staged token row

// WV waves (16 weight rows each) x TM token tiles per workgroup
template <class F, int WV, int TM, bool X_F32>
__global__ __launch_bounds__(64 * WV) void mm_fused_kernel(const void* X_, const uint8_t* W_, float* Y_, uint32_t n_, uint32_t rows_,
                                                           uint32_t cols_, uint32_t x_stride_, uint32_t row_bytes_, uint32_t accumulate_,
                                                           uint32_t slice_stages_, float* partials_) {
  // (the fields of MmArgs one by one: built with kernel-argument preload the leading fourteen words are in scalar
  // registers when the wave starts, instead of one trip to memory away)
  const MmArgs a{X_, W_, Y_, n_, rows_, cols_, x_stride_, row_bytes_, accumulate_, slice_stages_, partials_};
  constexpr int NT = 64 * WV, TOK = 16 * TM, ABUF = TOK * kMmPitch;
  constexpr int GRAN = TOK * (kMmKStage / 8);           // 16-byte granules (8 halves) per stage
  constexpr int AG = (GRAN + NT - 1) / NT;              // per thread
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  uint32_t* tbl = smem;
  uint8_t* abuf = (uint8_t*)(smem + F::LDS_WORDS);
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  const uint32_t n16 = lane & 15u, q = lane >> 4;
  const uint32_t row = (blockIdx.x * WV + wave) * 16u + n16;
  const uint32_t m0 = blockIdx.y * TOK;
  const gptr_t wrow = as_global(a.W) + (size_t)min(row, a.rows - 1) * a.row_bytes;
  const uint32_t nstages = a.cols / kMmKStage;
  const uint32_t st0 = blockIdx.z * a.slice_stages, st1 = min(st0 + a.slice_stages, nstages);  // this workgroup's K slice

  // activation stage loader: granule g = (token g / 16, columns 8 (g % 16) ..); tokens past n repeat the last one
  u32x4 pa[AG][X_F32 ? 2 : 1];
  auto a_issue = [&](uint32_t st) {
#pragma unroll
    for (int i = 0; i < AG; i++) {
      const uint32_t g = min(tid + i * NT, (uint32_t)GRAN - 1u);
      const uint32_t tok = min(m0 + (g >> 4), a.n - 1), col = st * kMmKStage + (g & 15u) * 8u;
      if constexpr (X_F32) {
        const MSQ_GLOBAL float* p = (const MSQ_GLOBAL float*)a.X + (size_t)tok * a.x_stride + col;
        pa[i][0] = *(const MSQ_GLOBAL u32x4*)p;
        pa[i][1] = *(const MSQ_GLOBAL u32x4*)(p + 4);
      } else {
        // rows of fp16 activations are only 2-byte aligned in general (any x_stride)
        const u128_a2 v = ld128(as_global((const uint16_t*)a.X + (size_t)tok * a.x_stride + col));
        pa[i][0] = u32x4{v.x, v.y, v.z, v.w};
      }
    }
  };
  auto a_store = [&](uint32_t buf) {
#pragma unroll
    for (int i = 0; i < AG; i++) {
      const uint32_t g = tid + i * NT;
      if (g >= (uint32_t)GRAN) continue;
      u32x4 v;
      if constexpr (X_F32) {
        auto f = [](uint32_t w) { return __builtin_bit_cast(float, w); };
        v = u32x4{pack_h2(f(pa[i][0].x), f(pa[i][0].y)), pack_h2(f(pa[i][0].z), f(pa[i][0].w)),
                  pack_h2(f(pa[i][1].x), f(pa[i][1].y)), pack_h2(f(pa[i][1].z), f(pa[i][1].w))};
      } else {
        v = pa[i][0];
      }
      uint8_t* dst = abuf + buf * ABUF + (g >> 4) * kMmPitch;
      const uint32_t c0 = (g & 15u) * 8u;  // first of the granule's eight columns inside the stage
      if constexpr (requires { F::pos_of(0u); }) {
        // position p of chunk q in a step stands for column col_of(q, p): every column is stored where its fragment
        // reads it (pos_of is the inverse of col_of)
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 8; e++)
          *(uint16_t*)(dst + 2u * ((c0 & ~31u) + F::pos_of((c0 & 31u) + e))) = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
      } else {
        *(u32x4*)(dst + 2u * c0) = v;
      }
    }
  };

  a_issue(st0);
  F::fill_lds(tbl, (int)tid, NT);
  a_store(0);
  __syncthreads();

  f4_t acc[TM];
#pragma unroll
  for (int t = 0; t < TM; t++) acc[t] = f4_t{0.f, 0.f, 0.f, 0.f};
  uint32_t touch = 0;

  for (uint32_t st = st0; st < st1; st++) {
    const uint32_t sn = st + 1 < st1 ? st + 1 : st;  // the last stage fetches itself again: no branch around the loads
    const uint32_t buf = (st - st0) & 1u;
    a_issue(sn);
    // the next stage's weight bytes are touched now (a lane per 32 bytes of its row's stage), so that the fragment
    // loads of that stage, which sit right in front of their decode, find them in the nearest cache
    {
      const uint32_t stage_bytes = a.row_bytes / nstages;  // rows are whole blocks: every stage has the same byte count
      const uint32_t off = min(sn * stage_bytes + 32u * q, a.row_bytes - 4u) & ~3u;
      touch ^= *(const MSQ_GLOBAL uint32_t*)(wrow - ((uintptr_t)wrow & 3u) + off);
      if (stage_bytes > 128u) touch ^= *(const MSQ_GLOBAL uint32_t*)(wrow - ((uintptr_t)wrow & 3u) + (min(off + 128u, a.row_bytes - 4u) & ~3u));
    }
    const uint8_t* arow = abuf + buf * ABUF + n16 * kMmPitch + 16u * q;
    // the four steps' fragments first: their loads are then in flight together (one trip to memory per stage)
    constexpr int NS = kMmKStage / 32;
    uint32_t h[NS][4];
    {
      FragOut f[NS];
      float sc[NS];
#pragma unroll
      for (int js = 0; js < NS; js++) {
        const uint32_t step = st * NS + js;
        f[js] = F::get(wrow, step, q, tbl);
        sc[js] = f[js].scale;
        if constexpr (requires(float& s) { F::get_scales(wrow, step, s, s); }) {  // two scale groups per step (Q6_K)
          float sa, sb;
          F::get_scales(wrow, step, sa, sb);
          sc[js] = q < 2 ? sa : sb;
        }
      }
#pragma unroll
      for (int js = 0; js < NS; js++) {
#pragma unroll
        for (int p = 0; p < 4; p++) {
          if constexpr (requires { F::PLAIN; }) h[js][p] = f[js].h[p];
          else h[js][p] = scale_round_h2(f[js].h[p], sc[js], F::HAS_ADD ? f[js].add : 0.f);
        }
      }
    }
#pragma unroll
    for (int js = 0; js < NS; js++) {
#pragma unroll
      for (int t = 0; t < TM; t++) {
        const uint4 av = *(const uint4*)(arow + t * 16 * kMmPitch + 64u * js);
        const uint32_t x[4] = {av.x, av.y, av.z, av.w};
        acc[t] = mfma_f16(x, h[js], acc[t]);
      }
    }
    a_store(buf ^ 1u);  // the other buffer was last read one stage ago, before the previous barrier
    __syncthreads();
  }

  if (touch == 0x9E3779B9u && a.n == 0) a.Y[0] = 0.f;  // never true: keeps the touching loads
  // D: lane holds weight row n16 (column of D), tokens 4 q + i of every tile
  if (row < a.rows) {
#pragma unroll
    for (int t = 0; t < TM; t++) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t tok = m0 + 16u * t + 4u * q + i;
        if (tok < a.n) {
          float* y = a.Y + (size_t)tok * a.rows + row;
          if (a.partials) a.partials[((size_t)blockIdx.z * a.n + tok) * a.rows + row] = acc[t][i];
          else *y = a.accumulate ? *y + acc[t][i] : acc[t][i];
        }
      }
    }
  }
}

// The same product for more tokens, block formats only, activations as fp16 rows in memory. The kernel above fetches a
// lane's weight bytes straight from memory: sixteen rows per load instruction, a row per lane, so every load asks the
// vector cache for sixteen or more lines, and its waves wait for every LDS read in front of the matrix instruction that
// uses it. Here
//  * weights and activations both come by loads that write LDS directly (no registers, no conversion, no address
//    arithmetic per stage for the activations): the weight bytes of a weight stage (256 columns of the workgroup's
//    16 WV RT rows) as consecutive aligned 16-byte pieces over consecutive lanes, every cache line asked for once; the
//    activations of a stage ([16 TM tokens][XK columns]) one stage ahead, the 16-byte chunks of a token's row stored
//    at slot (chunk ^ f(token)), so that the sixteen tokens of a fragment read hit sixteen different bank groups
//    without padding;
//  * the fragment decoders read the weight bytes from LDS (load_raw / finish); a decoded fragment feeds TM matrix
//    instructions -- decoding costs about 37 vector instructions per fragment, a matrix instruction takes the time of
//    3.5, so TM = 16 where the call has the tokens. Measured with TM = 16: the LDS is busy 88 % of the time (one
//    16-byte-per-lane activation read per matrix instruction), the matrix cores about half of it;
//  * the K loop is pipelined by hand: the bytes of step j + 2 and the activation fragments of the next half step are
//    read from LDS and the weights of step j + 1 decoded while the matrix cores work on step j; scheduling barriers
//    keep the compiler from moving the reads back next to their use; the requests to memory are dealt over the steps
//    (the load unit takes one every sixteen cycles or so: a wave that issues them in one go waits there).
// The loads that write LDS are hidden from the compiler (lds_dma16): the waits for them are explicit (wait_vm).
template <class F, int WV, int RT, int TM, int XK>
__global__ __launch_bounds__(64 * WV) void mm_tile_kernel(const void* X_, const uint8_t* W_, float* Y_, uint32_t n_, uint32_t rows_,
                                                          uint32_t cols_, uint32_t x_stride_, uint32_t row_bytes_, uint32_t accumulate_,
                                                          uint32_t slice_stages_, float* partials_) {
  const MmArgs a{X_, W_, Y_, n_, rows_, cols_, x_stride_, row_bytes_, accumulate_, slice_stages_, partials_};
  constexpr int NT = 64 * WV, TOK = 16 * TM, ROWS = 16 * WV * RT;
  constexpr int CPT = XK / 8;                 // 16-byte chunks per token and stage
  constexpr int XBUF = TOK * XK * 2;
  constexpr int NS = XK / 32;                 // K steps per stage
  constexpr int XPW = 256 / XK;               // stages per weight stage
  constexpr int TH = TM < 8 ? TM : 8, UPS = TM / TH;  // token tiles per unit of the pipeline, units per K step
  static_assert((XK == 64 || XK == 128) && TM % TH == 0, "");
  // 16-byte pieces per row and weight stage: the stage's bytes at any 2-byte alignment inside their first piece; an odd
  // count, so that the sixteen rows of a tile start in sixteen different groups of four banks
  constexpr int P = ((F::WS_BYTES + 14 + 15) / 16) | 1;
  constexpr int NPI = (ROWS * P + NT - 1) / NT;  // weight pieces per thread and weight stage
  constexpr int WBUF = NPI * NT * 16;
  constexpr int XPI = TOK * CPT / NT;            // activation pieces per thread and stage
  static_assert(TOK * CPT % NT == 0, "every thread requests the same number of pieces");
  constexpr bool PAIR = requires { F::pos_of(0u); };
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  uint32_t* tbl = smem;
  uint8_t* abuf = (uint8_t*)(smem + F::LDS_WORDS);
  uint8_t* wbuf = abuf + 2 * XBUF;
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  const uint32_t n16 = lane & 15u, q = lane >> 4;
  const uint32_t row0 = blockIdx.x * ROWS, m0 = blockIdx.y * TOK;
  const uint32_t nstages = a.cols / XK;
  const uint32_t st0 = blockIdx.z * a.slice_stages, st1 = min(st0 + a.slice_stages, nstages);  // st0: a whole number of weight stages
  // slot of chunk c in the row of token t: the LDS has 32 banks of four bytes, rows are one or two times 128 bytes
  // apart, so all rows start in the same bank; eight consecutive lanes (tokens) of a 16-byte read are served together and
  // have to hit eight different 16-byte groups: the token's low three bits go into the slot
  auto swz = [](uint32_t t) { return CPT == 16 ? (t & 15u) : (t & 7u); };

  // ---- activations: piece i = k NT + tid is slot i % CPT of token i / CPT (host: rows 16-byte aligned, below 4 GiB)
  const rsrc_t xrs = make_rsrc(a.X, ((a.n - 1) * a.x_stride + a.cols) * 2u);
  uint32_t xoff[XPI];
#pragma unroll
  for (int k = 0; k < XPI; k++) {
    const uint32_t i = (uint32_t)k * NT + tid, t = i / CPT;
    xoff[k] = min(m0 + t, a.n - 1) * a.x_stride * 2u + 16u * ((i % CPT) ^ swz(t));  // tokens past n repeat the last one
  }
  auto x_request = [&](uint32_t st, uint32_t buf, int k0, int k1) {
#pragma unroll
    for (int k = k0; k < k1; k++)
      lds_dma16(xrs, abuf + buf * XBUF + ((uint32_t)k * NT + wave * 64u) * 16u, xoff[k], st * (XK * 2u));
  };
  // ---- weights: piece i = k NT + tid is 16-byte piece i % P of row i / P
  const uintptr_t wa = (uintptr_t)a.W;
  const uint32_t wmis = (uint32_t)wa & 15u;
  const uint32_t wbytes = (wmis + a.rows * a.row_bytes + 15u) & ~15u;  // (below 4 GiB: the host sends larger matrices elsewhere)
  const rsrc_t wrs = make_rsrc((const void*)(wa - wmis), wbytes);      // whole aligned pieces: no piece straddles the end
  uint32_t woff[NPI], wpc[NPI];
#pragma unroll
  for (int k = 0; k < NPI; k++) {
    const uint32_t i = (uint32_t)k * NT + tid, rl = i / P, r = row0 + rl;
    woff[k] = rl < (uint32_t)ROWS && r < a.rows ? wmis + r * a.row_bytes : ~0u;  // rows past the end: zeros, no traffic
    wpc[k] = (i % P) * 16u;
  }
  auto w_request = [&](uint32_t ws, uint32_t buf) {  // (past a row's last block this fetches bytes nobody reads)
#pragma unroll
    for (int k = 0; k < NPI; k++) {
      const uint32_t v = woff[k] + ws * (uint32_t)F::WS_BYTES;
      lds_dma16(wrs, wbuf + buf * WBUF + ((uint32_t)k * NT + wave * 64u) * 16u, woff[k] == ~0u ? wbytes : (v & ~15u) + wpc[k], 0u);
    }
  };
  uint32_t myoff[RT];
  const uint8_t* lbase[RT];
#pragma unroll
  for (int rt = 0; rt < RT; rt++) {
    const uint32_t rl = (wave * RT + rt) * 16u + n16;
    myoff[rt] = wmis + min(row0 + rl, a.rows - 1) * a.row_bytes;
    lbase[rt] = wbuf + rl * (uint32_t)(P * 16);
  }

  x_request(st0, 0, 0, XPI);
  w_request(st0 / XPW, 0);
  F::fill_lds(tbl, (int)tid, NT);
  wait_vm<0>();
  __syncthreads();

  f4_t acc[RT][TM];
#pragma unroll
  for (int rt = 0; rt < RT; rt++)
#pragma unroll
    for (int t = 0; t < TM; t++) acc[rt][t] = f4_t{0.f, 0.f, 0.f, 0.f};

  for (uint32_t st = st0; st < st1; st++) {
    const uint32_t rel = st - st0, buf = rel & 1u, ws = st / XPW, sub = st % XPW, wb = (rel / XPW) & 1u;
    // the targets of this stage's requests were last read before the barrier that ended the previous stage (the
    // weight buffer before the one that ended the previous weight stage)
    const uint32_t stn = st + 1 < st1 ? st + 1 : st;  // (the last stage fetches itself again: the waits stay the same)
    const uint8_t* arow = abuf + buf * XBUF + n16 * (XK * 2u);
    LdsRow lrow[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) lrow[rt] = LdsRow::of(lbase[rt] + wb * WBUF, (myoff[rt] + ws * (uint32_t)F::WS_BYTES) & 15u);
    const uint32_t sl0 = sub * NS;  // first K step of this stage inside the weight stage
    decltype(F::load_raw(lrow[0], 0u, 0u)) raw[2][RT];
    uint4 bx[2][TH];
    uint32_t h[2][RT][4];
    auto fetch_w = [&](int slot, int js) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) raw[slot][rt] = F::load_raw(lrow[rt], sl0 + js, q);
    };
    auto fetch_x = [&](int slot, int js, int u) {
#pragma unroll
      for (int t = 0; t < TH; t++) {
        const uint8_t* tr = arow + (u * TH + t) * 16 * (XK * 2);
        if constexpr (PAIR) {
          // positions (2 i, 2 i + 1) of chunk q stand for columns (4 q + i, 16 + 4 q + i) of the step: two 8-byte reads,
          // interleaved when they are used
          const uint32_t c1 = 4u * js + (q >> 1), at = 8u * (q & 1u);
          const uint2 lo = *(const uint2*)(tr + 16u * (c1 ^ swz(n16)) + at), hi = *(const uint2*)(tr + 16u * ((c1 + 2u) ^ swz(n16)) + at);
          bx[slot][t] = uint4{lo.x, lo.y, hi.x, hi.y};
        } else {
          bx[slot][t] = *(const uint4*)(tr + 16u * ((4u * js + q) ^ swz(n16)));
        }
      }
    };
    auto decode = [&](int hs, int slot, int js) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        const FragOut f = F::finish(raw[slot][rt], sl0 + js, q, tbl);
#pragma unroll
        for (int p = 0; p < 4; p++) h[hs][rt][p] = scale_round_h2(f.h[p], f.scale, F::HAS_ADD ? f.add : 0.f);
      }
    };
    fetch_w(0, 0);
    fetch_x(0, 0, 0);
    if (NS > 1) fetch_w(1, 1);
    __builtin_amdgcn_sched_barrier(0);
    decode(0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int g = 0; g < NS * UPS; g++) {  // unit g: token tiles u TH .. of K step js
      const int js = g / UPS, u = g % UPS;
      if (u == 0 && js + 2 < NS) fetch_w(js & 1, js + 2);
      if (g + 1 < NS * UPS) fetch_x((g + 1) & 1, (g + 1) / UPS, (g + 1) % UPS);
      if (u == 0) {
        constexpr int XA = NS > 1 ? (XPI + NS - 2) / (NS - 1) : XPI;  // activations over the first steps, weights with the last
        if (js < NS - 1 || NS == 1) x_request(stn, buf ^ 1u, js * XA, (js + 1) * XA < XPI ? (js + 1) * XA : XPI);
        if (js == NS - 1 && sub == 0) w_request(ws + 1, wb ^ 1u);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (u == 0 && js + 1 < NS) decode((js + 1) & 1, (js + 1) & 1, js + 1);
#pragma unroll
      for (int t = 0; t < TH; t++) {
        const uint4 av = bx[g & 1][t];
        uint32_t x[4] = {av.x, av.y, av.z, av.w};
        if constexpr (PAIR) {
          x[0] = __builtin_amdgcn_perm(av.z, av.x, 0x05040100u); x[1] = __builtin_amdgcn_perm(av.z, av.x, 0x07060302u);
          x[2] = __builtin_amdgcn_perm(av.w, av.y, 0x05040100u); x[3] = __builtin_amdgcn_perm(av.w, av.y, 0x07060302u);
        }
#pragma unroll
        for (int rt = 0; rt < RT; rt++) acc[rt][u * TH + t] = mfma_f16(x, h[js & 1][rt], acc[rt][u * TH + t]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // the next stage's activations have to be there; the weight stage requested behind them in the first stage of a
    // weight stage may stay in flight over the next stage
    if (sub == 0) wait_vm<NPI>();
    else wait_vm<0>();
    __syncthreads();
  }
  wait_vm<0>();  // a weight stage may still be on its way into this workgroup's LDS: not past the end of the kernel

  // D: lane holds weight row n16 of its tile (column of D), tokens 4 q + i of every token tile
#pragma unroll
  for (int rt = 0; rt < RT; rt++) {
    const uint32_t row = row0 + (wave * RT + rt) * 16u + n16;
    if (row >= a.rows) continue;
    float* out = a.partials ? a.partials + (size_t)blockIdx.z * a.n * a.rows : a.Y;
    const bool add = !a.partials && a.accumulate;
#pragma unroll
    for (int t = 0; t < TM; t++) {
      float old[4];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t tok = m0 + 16u * t + 4u * q + i;
        old[i] = add && tok < a.n ? out[(size_t)tok * a.rows + row] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t tok = m0 + 16u * t + 4u * q + i;
        if (tok < a.n) out[(size_t)tok * a.rows + row] = old[i] + acc[rt][t][i];
      }
    }
  }
}

// Y (+)= partials[0] + partials[1] + ... in that order, element by element
__global__ __launch_bounds__(256) void mm_reduce_kernel(const float* __restrict__ partials, float* __restrict__ Y, size_t count,
                                                        uint32_t slices, uint32_t accumulate) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float s = 0.f;
  for (uint32_t z0 = 0; z0 < slices; z0 += 8u) {  // eight slices requested before the first is added
    float t[8];
#pragma unroll
    for (uint32_t k = 0; k < 8u; k++) t[k] = partials[(size_t)min(z0 + k, slices - 1u) * count + i];
#pragma unroll
    for (uint32_t k = 0; k < 8u; k++)
      if (z0 + k < slices) s += t[k];
  }
  Y[i] = accumulate ? Y[i] + s : s;
}

}  // namespace msq
