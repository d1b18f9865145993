// Prefill MoE: grouped GEMM over experts on the matrix cores (reference operator: ms::q::encode_moe_prefill,
// src/kernels/quant.mm:433-612; reference kernels q_moe_gather / q_moe_rgu / q_moe_rdown / q_moe_reduce,
// src/kernels/quant_moe_prefill.metal:22-29,190-239,275-303,330-344).
//
//   gather : Xg[i] = fp16(X[tok[i]]) for the expert-sorted entries, then Xg[total + t] = fp16(X[t]) (shared expert)
//   gate/up: H[i][r] = fp16(silu(min(Xg_e[i].Wg[r], 10)) * clamp(Xg_e[i].Wu[r], -10, 10) * wt[i])
//   down   : Z[i][c] = H_e[i] . Wd[c]   (fp32, one row per entry)
//   reduce : Y[t] += Z[total + t] + sum_k Z[slot_of[t][k]]   in that fixed order
//
// GEMM work item = (token tile of up to 16 entries of one expert, chunk of weight-row tiles). A workgroup is up to 16
// waves that split K; each wave keeps the token tile's activations of its K steps in registers as MFMA A fragments,
// and the workgroup walks the 16-row weight tiles of its chunk. A tile's raw block bytes (16 contiguous rows) are
// copied into LDS with fully coalesced 128-bit loads, one tile ahead through registers, and decoded from there into
// B fragments; weights stay exact (fp16 payloads, fp32 scales applied to the MFMA result). The K-split partial tiles
// meet in LDS and are added in wave order, so results do not depend on scheduling.
#pragma once
#include <type_traits>

#include "msq_mfma.cuh"

namespace msq {

struct PfArgs {
  const uint16_t* A;        // activations fp16 [(total + n) x K]: Xg (gate/up) or H (down)
  uint16_t* H;              // gate/up output fp16 [(total + n) x inter]
  float* Z;                 // down output fp32 [(total + n) x dim]
  const float* wt;          // routing weight per entry [total]
  const uint64_t* ptrs;     // (n_exp + 1) x {gate, up, down} device addresses (the shared expert is entry n_exp)
  const uint32_t* offs;     // n_exp + 2 entry offsets
  const uint32_t* tiles;    // token tiles: pairs {expert index, first entry of the tile inside the expert}
  uint32_t ntiles;          // token tiles this launch covers
  uint32_t total;           // routed entries: entries at or beyond use weight 1 (shared expert)
  uint32_t K, N;            // gate/up: K = dim, N = inter; down: K = inter, N = dim
  uint32_t row_bytes;
  uint32_t nsteps, steps_per_wave;
  uint32_t chunk_tiles;     // weight-row tiles per work item
  uint32_t nchunks;         // ceil(N / 16 / chunk_tiles)
  uint32_t staged;          // 1: weight tiles go through LDS staging
};

constexpr int kPfStageGranules = 3;  // 16-byte granules per thread per matrix the staging path can hold (48 KiB / 1024 threads)

template <class F, bool GU, bool STAGED>
__global__ __launch_bounds__(1024) void moe_pf_gemm_kernel(const PfArgs a) {
  constexpr int NM = GU ? 2 : 1;
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  uint32_t* tbl = smem;
  float* red = (float*)(smem + F::LDS_WORDS);  // [NM][wave][token][17]
  const uint32_t tid = threadIdx.x, lane = tid & 63u, nthreads = blockDim.x;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6)), nwaves = nthreads >> 6;
  uint8_t* stage = (uint8_t*)(red + NM * nwaves * 16 * 17);  // [NM][tile window]
  const uint32_t m16 = lane & 15u, q = lane >> 4;
  const uint32_t S = a.steps_per_wave, s0 = wave * S;
  const uint32_t tile_bytes = 16u * a.row_bytes;
  const uint32_t window = (tile_bytes + 15u + 15u) & ~15u;  // staged window per matrix, rounded to granules

  F::fill_lds(tbl, (int)tid, (int)nthreads);

  const uint32_t item = blockIdx.x;
  const uint32_t mt = item / a.nchunks, rc = item - mt * a.nchunks;
  const uint32_t e = a.tiles[2 * mt], t0 = a.tiles[2 * mt + 1];
  const uint32_t base = a.offs[e] + t0;                       // first entry (row of A / H / Z) of the token tile
  const uint32_t mtok = min(16u, a.offs[e + 1] - base);
  gptr_t W[NM];
  if (GU) { W[0] = as_global((const void*)a.ptrs[3 * e]); W[NM - 1] = as_global((const void*)a.ptrs[3 * e + 1]); }
  else W[0] = as_global((const void*)a.ptrs[3 * e + 2]);

  // A fragments of this wave's K steps: token m16 of the tile, chunk q
  uint32_t xa[kMvnMaxSteps][4];
#pragma unroll
  for (int i = 0; i < kMvnMaxSteps; i++) {
    const uint32_t step = s0 + i;
    uint4 v = {0u, 0u, 0u, 0u};
    if ((uint32_t)i < S && step < a.nsteps && m16 < mtok) {
      const uint16_t* xs = a.A + (size_t)(base + m16) * a.K + 32u * step;
      v = *(const uint4*)(xs + 8u * q);  // every format used here keeps the natural column order (col_of = 8 q + p)
    }
    xa[i][0] = v.x; xa[i][1] = v.y; xa[i][2] = v.z; xa[i][3] = v.w;
  }

  const uint32_t ntile_rows = (a.N + 15u) / 16u;
  const uint32_t tile_first = rc * a.chunk_tiles, tile_last = min(ntile_rows, tile_first + a.chunk_tiles);
  // staging: thread i owns granules i, i + nthreads, ... of each matrix' aligned window
  uint4 pf[NM][kPfStageGranules];
  auto issue = [&](uint32_t tile) {
#pragma unroll
    for (int m = 0; m < NM; m++) {
      const gptr_t start = W[m] + (size_t)tile * tile_bytes;
      const uint32_t shift = (uint32_t)((uintptr_t)start & 15u);
      // the last tile of a matrix may be short: never read beyond the last row's granule
      const uint32_t rows_here = min(16u, a.N - tile * 16u);
      const uint32_t valid = shift + rows_here * a.row_bytes;
#pragma unroll
      for (int g = 0; g < kPfStageGranules; g++) {
        const uint32_t gi = tid + g * nthreads;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (16u * gi < valid) v = *(const MSQ_GLOBAL u32x4*)(start - shift + 16u * gi);
        pf[m][g] = uint4{v.x, v.y, v.z, v.w};
      }
    }
  };
  if (STAGED && tile_first < tile_last) issue(tile_first);
  __syncthreads();  // tables ready

  const uint32_t ones[4] = {0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
  for (uint32_t tile = tile_first; tile < tile_last; tile++) {
    std::conditional_t<STAGED, const uint8_t*, gptr_t> wr[NM];
    if constexpr (STAGED) {
#pragma unroll
      for (int m = 0; m < NM; m++) {
#pragma unroll
        for (int g = 0; g < kPfStageGranules; g++) {
          const uint32_t gi = tid + g * nthreads;
          if (16u * gi < window) ((uint4*)(stage + (size_t)m * window))[gi] = pf[m][g];
        }
        const uint32_t shift = (uint32_t)((uintptr_t)(W[m] + (size_t)tile * tile_bytes) & 15u);
        wr[m] = stage + (size_t)m * window + shift + m16 * a.row_bytes;
      }
      if (tile + 1 < tile_last) issue(tile + 1);  // next tile's bytes travel while this one is decoded
      __syncthreads();
    } else {
      const uint32_t row = min(tile * 16u + m16, a.N - 1);
#pragma unroll
      for (int m = 0; m < NM; m++) wr[m] = W[m] + (size_t)row * a.row_bytes;
    }
    f4_t acc[NM];
#pragma unroll
    for (int m = 0; m < NM; m++) acc[m] = f4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < kMvnMaxSteps; i++) {
      const uint32_t step = s0 + i;
      if ((uint32_t)i < S && step < a.nsteps) {  // wave-uniform
        const f4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < NM; m++) {
          const FragOut f = F::get(wr[m], step, q, tbl);
          if constexpr (requires(float& s) { F::get_scales(wr[m], step, s, s); }) {
            float sa, sb;
            F::get_scales(wr[m], step, sa, sb);
            uint32_t ha[4], hb[4];
#pragma unroll
            for (int p = 0; p < 4; p++) { ha[p] = q < 2 ? f.h[p] : 0u; hb[p] = q < 2 ? 0u : f.h[p]; }
            acc[m] += sa * mfma_f16(xa[i], ha, zero) + sb * mfma_f16(xa[i], hb, zero);
          } else {
            acc[m] += f.scale * mfma_f16(xa[i], f.h, zero);
            if constexpr (F::HAS_ADD) acc[m] += f.add * mfma_f16(xa[i], ones, zero);
          }
        }
      }
    }
#pragma unroll
    for (int m = 0; m < NM; m++)
#pragma unroll
      for (int i = 0; i < 4; i++) red[((m * nwaves + wave) * 16u + 4u * q + i) * 17u + m16] = acc[m][i];
    __syncthreads();
    for (uint32_t idx = tid; idx < 16u * mtok; idx += nthreads) {
      const uint32_t t = idx >> 4, r = idx & 15u, orow = tile * 16u + r;
      if (orow < a.N) {
        float s[NM];
#pragma unroll
        for (int m = 0; m < NM; m++) {
          s[m] = 0.f;
          for (uint32_t w = 0; w < nwaves; w++) s[m] += red[((m * nwaves + w) * 16u + t) * 17u + r];
        }
        const uint32_t entry = base + t;
        if constexpr (GU) {
          float g = fminf(s[0], 10.f), u = fminf(fmaxf(s[NM - 1], -10.f), 10.f);
          const float w = entry < a.total ? a.wt[entry] : 1.f;
          const float h = g / (1.f + expf(-g)) * u * w;
          a.H[(size_t)entry * a.N + orow] = __builtin_bit_cast(uint16_t, (_Float16)h);
        } else {
          a.Z[(size_t)entry * a.N + orow] = s[0];
        }
      }
    }
    __syncthreads();
  }
}

// ------------------------------------------------------------------------------------------------ block GEMM
// Grouped GEMM for the 256-weight codebook formats (block fragments, see msq_mfma.cuh). A work item is one expert's
// block of up to 48 entries (T <= 3 token tiles) times a chunk of weight rows; the item's waves own different
// weight-row tiles and walk K block by block (256 columns): the activation block [48][256] fp16 is staged in LDS for
// all waves, every wave decodes the fragments of its own rows once per block and reuses each of them for all T token
// tiles, accumulates the block in the matrix cores and applies the fp32 block scale once. Weights are decoded exactly
// once per (item, row), no lane loads a weight byte twice, and the next block's bytes are in flight during a block.
// Table lookups run one fragment pair ahead of the pair being multiplied.
struct PfBlkArgs {
  const uint16_t* A;        // fp16 activations [entries][K]
  const uint64_t* ptrs;     // per expert: gate, up, down addresses
  const uint32_t* offs;     // per expert: first entry
  const uint32_t* items;    // per item: expert, first entry of the block inside the expert, entries in the block
  const float* wt;          // per routed entry: routing weight
  uint16_t* H;              // gate/up output [entries][N] fp16
  float* Z;                 // down output [entries][N] fp32
  uint32_t nitems, total;
  uint32_t K, N, row_bytes, nblocks;
  uint32_t row_chunks;      // chunks of pf_blk_rows() weight rows
  uint32_t chunks_per_wg;   // consecutive row chunks one workgroup takes, one after the other
  uint32_t row_groups;      // workgroups per item: row_chunks / chunks_per_wg, rounded up
};

constexpr int kPfBlkTokens = 48, kPfBigTokens = 112, kPfBigTiles = kPfBigTokens / 16, kPfBlkPitch = 256 * 2 + 16;
// waves per workgroup by token tiles per item: four per SIMD for up to three tiles, three for more (registers)
constexpr int pf_blk_waves(int T) { return T > 3 ? 12 : 16; }
// weight-row tiles per wave: two fragments per K step (gate + up of one tile, or two tiles of the down matrix) keep the
// register count low enough for three or four waves per SIMD, which is what overlaps decode, matrix and LDS work
constexpr int pf_blk_rt(bool gu, int) { return gu ? 1 : 2; }
constexpr int pf_blk_rows(bool gu, int T) { return pf_blk_waves(T) * pf_blk_rt(gu, T) * 16; }  // weight rows per work item
// activation staging: double-buffered for up to three token tiles, a single buffer (two barriers per block) for seven
template <class B>
constexpr size_t pf_blk_lds(int T) { return (size_t)B::LDS_WORDS * 4 + (T > 3 ? 1 : 2) * (size_t)(T > 3 ? kPfBigTokens : kPfBlkTokens) * kPfBlkPitch; }

// Where the 16 bytes of step j of chunk q (columns blk_col_of(q, j) .. + 7 of a block) sit in a token's staged row: the
// chunks in the order 0, 2, 1, 3. A 16-byte LDS read serves the lanes in four groups of sixteen -- {0-7, 24-31},
// {8-15, 16-23}, {32-39, 56-63}, {40-47, 48-55}, measured -- so a group holds tokens 0-7 of one chunk and tokens 8-15 of
// its neighbour (lane = 16 q + token); rows are 33 sixteen-byte units apart, token n starts in bank group n mod 16, and the
// two halves of a group only miss each other when the neighbouring chunks are a multiple of 256 bytes apart (in column
// order they are 128 apart and every read took two passes).
__device__ __forceinline__ uint32_t pf_lds_at(uint32_t q, uint32_t j) { return 16u * (16u * (q & 1u) + 8u * (q >> 1) + j); }

template <class B, bool GU, int T>
__device__ __forceinline__ void pf_block_body(const PfBlkArgs& a) {
  constexpr int WAVES = pf_blk_waves(T), NT = 64 * WAVES;
  constexpr int NM = GU ? 2 : 1, RT = pf_blk_rt(GU, T), R = RT * NM, PITCH = kPfBlkPitch;
  constexpr bool DB = T <= 3;  // two activation buffers
  constexpr int ABUF = (DB ? kPfBlkTokens : kPfBigTokens) * PITCH;
  constexpr int PPS = R / 2, NP = 8 * PPS;  // fragment pairs per K step, per block
  static_assert(R == 2 || R == 4, "fragments are processed in pairs");
  static_assert(T <= 3 || T == kPfBigTiles, "the single-buffer variant is sized for kPfBigTokens");
  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  uint32_t* tbl = smem;
  uint8_t* abuf = (uint8_t*)(smem + B::LDS_WORDS);  // [2][T * 16 tokens][PITCH]
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  const uint32_t n16 = lane & 15u, q = lane >> 4;

  // consecutive workgroups land on different XCDs: the row chunks of one item stay on one XCD (shared L2 for its
  // activations), and items are dealt round-robin over the XCDs
  const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
  const uint32_t item = (slot / a.row_groups) * 8u + xcd, rc0 = (slot % a.row_groups) * a.chunks_per_wg;
  if (item >= a.nitems) return;
  const uint32_t e = a.items[3 * item], t0 = a.items[3 * item + 1], cnt = a.items[3 * item + 2];
  const uint32_t base = a.offs[e] + t0;
  // A workgroup takes chunks_per_wg consecutive row chunks of its item, one after the other: the first trip to memory
  // (about 4.5 us before the first block can be multiplied, 17 % of a down-projection workgroup's life) is paid once, and
  // the next chunk's first block is requested during the last block of the one before, where a single chunk would
  // fetch its last block again
  // (built into the down projection of the small items only: the other variants have no registers to spare for it)
  constexpr bool MULTI = !GU && T <= 3;
  const uint32_t nch = MULTI ? min(a.chunks_per_wg, a.row_chunks - rc0) : 1u;

  // a weight row = the expert's matrix (a scalar address) + the lane's row offset (32 bits: a matrix is far below 4 GiB)
  gptr_t wbase[NM];
  uint32_t woff[RT], row_of[RT];
#pragma unroll
  for (int m = 0; m < NM; m++) wbase[m] = as_global((const void*)a.ptrs[3 * e + (GU ? m : 2)]);
#pragma unroll
  for (int jt = 0; jt < RT; jt++) {
    row_of[jt] = ((rc0 * WAVES + wave) * RT + jt) * 16u + n16;
    woff[jt] = min(row_of[jt], a.N - 1) * a.row_bytes;
  }
  auto wrow = [&](int r, uint32_t off) { return wbase[r % NM] + (size_t)(woff[r / NM] + off); };

  // activation chunk loader: T * 512 granules of 16 bytes (token g / 32, column g % 32) over the workgroup's threads
  constexpr int AG = (T * 512 + NT - 1) / NT;
  u32x4 pa[AG];  // (a plain vector type: the HIP struct type keeps the array in scratch memory)
  auto a_issue = [&](uint32_t kc) {
#pragma unroll
    for (int i = 0; i < AG; i++) {
      // rows past the block's last entry repeat it (their products are never stored): no branch around the load, so
      // the number of loads in flight stays known to every wait that follows
      const uint32_t g = min(tid + i * NT, T * 512u - 1u);
      const uint32_t tok = min(g >> 5, cnt - 1);
      pa[i] = *(const u32x4*)(a.A + (size_t)(base + tok) * a.K + kc * 256u + (g & 31u) * 8u);
    }
  };
  auto a_store = [&](uint32_t buf) {
#pragma unroll
    for (int i = 0; i < AG; i++) {
      const uint32_t g = tid + i * NT;
      if (g < T * 512u) *(u32x4*)(abuf + buf * ABUF + (g >> 5) * PITCH + pf_lds_at((g >> 3) & 3u, g & 7u)) = pa[i];
    }
  };

  typename B::Raw cur[R], nxt[R];
#pragma unroll
  for (int r = 0; r < R; r++) cur[r] = B::load(wrow(r, 0u), q);
  a_issue(0);
  B::fill_lds(tbl, (int)tid, NT);
  a_store(0);
  __syncthreads();

  uint32_t kb = 0;  // blocks done so far (double buffering: block kb sits in buffer kb % 2)
  for (uint32_t c = 0; c < nch; c++) {
  const bool more = c + 1 < nch;
  f4_t acc[T][R];
#pragma unroll
  for (int t = 0; t < T; t++)
#pragma unroll
    for (int r = 0; r < R; r++) acc[t][r] = f4_t{0.f, 0.f, 0.f, 0.f};

  for (uint32_t kc = 0; kc < a.nblocks; kc++, kb++) {
    // the block requested during this one: the chunk's next, or the first of the workgroup's next chunk, or (nothing left)
    // this one again: no branch around the loads
    const bool lastb = kc + 1 == a.nblocks;
    const uint32_t kn = !lastb ? kc + 1 : more ? 0u : kc;
    // (the host lets a workgroup take several chunks only when all chunks are whole: the next chunk's rows are then the
    // same number of bytes further for every lane)
    const uint32_t wn = kn * (uint32_t)B::BLOCK_BYTES + (c + (lastb && more ? 1u : 0u)) * ((uint32_t)(WAVES * RT * 16) * a.row_bytes);
    const uint8_t* arow = abuf + (DB ? (kb & 1u) * ABUF : 0u) + n16 * PITCH;
    if constexpr (T > 3) {
      // many token tiles: a step's fragments are all decoded first, then every tile's activation fragment (read from
      // LDS two tiles ahead of its use) feeds one matrix instruction per fragment
      uint32_t af[3][4];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        // the next block's bytes are requested a few at a time between the steps: requested all at once by all waves
        // right after the barrier, they queue up in the texture addresser and hold the waves at issue
        if (j == 1) {
          __builtin_amdgcn_sched_barrier(0);  // keep the requests here: the scheduler would sink them to their first use
          a_issue(kn);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (j >= 2 && j - 2 < R) {
          __builtin_amdgcn_sched_barrier(0);
          nxt[j - 2] = B::load(wrow(j - 2, wn), q);
          __builtin_amdgcn_sched_barrier(0);
        }
        typename B::Look lk[R];
#pragma unroll
        for (int r = 0; r < R; r++) lk[r] = B::lookup(cur[r], j, tbl, n16);
#pragma unroll
        for (int u = 0; u < 2; u++) {
          const uint4 av = *(const uint4*)(arow + u * 16 * PITCH + pf_lds_at(q, j));
          af[u][0] = av.x; af[u][1] = av.y; af[u][2] = av.z; af[u][3] = av.w;
        }
        uint32_t h[R][4];
#pragma unroll
        for (int r = 0; r < R; r++) B::finish(cur[r], j, lk[r], h[r]);
#pragma unroll
        for (int t = 0; t < T; t++) {
          const uint32_t(&x)[4] = af[t % 3];
          if (t + 2 < T) {
            const uint4 av = *(const uint4*)(arow + (t + 2) * 16 * PITCH + pf_lds_at(q, j));
            uint32_t(&y)[4] = af[(t + 2) % 3];
            y[0] = av.x; y[1] = av.y; y[2] = av.z; y[3] = av.w;
          }
          if (16u * t < cnt) {  // (uniform) a block of fewer entries leaves its last tiles out
#pragma unroll
            for (int r = 0; r < R; r++) acc[t][r] = mfma_f16(x, h[r], acc[t][r]);
          }
        }
      }
    } else {
    // table reads run one fragment pair ahead where registers allow (pair p = 2 j + half uses lk[p & 1]: fragments
    // 2 half, 2 half + 1 of step j): the one-tile variant has four waves per SIMD to hide them behind instead, the
    // three-tile variant six matrix instructions per pair
    constexpr bool AHEAD = T == 2;
    typename B::Look lk[2][2];
    if (AHEAD) {
      lk[0][0] = B::lookup(cur[0], 0, tbl, n16);
      lk[0][1] = B::lookup(cur[1], 0, tbl, n16);
    }
    uint32_t af[T][4];
#pragma unroll
    for (int p = 0; p < NP; p++) {
      const int j = p / PPS, r0 = 2 * (p % PPS);
      // the next block's bytes are requested a few at a time between the fragment pairs: requested all at once by
      // all waves right after the barrier, they queue up in the texture addresser and hold the waves at issue
      if (p == 1) {
        __builtin_amdgcn_sched_barrier(0);  // keep the requests here: the scheduler would sink them to their first use
        a_issue(kn);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (p % 2 == 0 && p >= 2 && p / 2 - 1 < R) {
        __builtin_amdgcn_sched_barrier(0);
        nxt[p / 2 - 1] = B::load(wrow(p / 2 - 1, wn), q);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (p % PPS == 0) {  // activations of step j, read with the fragments' column mapping
#pragma unroll
        for (int t = 0; t < T; t++) {
          const uint4 av = *(const uint4*)(arow + t * 16 * PITCH + pf_lds_at(q, j));
          af[t][0] = av.x; af[t][1] = av.y; af[t][2] = av.z; af[t][3] = av.w;
        }
      }
      if (!AHEAD) {
        lk[p & 1][0] = B::lookup(cur[r0], j, tbl, n16);
        lk[p & 1][1] = B::lookup(cur[r0 + 1], j, tbl, n16);
      } else if (p + 1 < NP) {  // table reads of the next pair
        const int jn = (p + 1) / PPS, rn = 2 * ((p + 1) % PPS);
        lk[(p + 1) & 1][0] = B::lookup(cur[rn], jn, tbl, n16);
        lk[(p + 1) & 1][1] = B::lookup(cur[rn + 1], jn, tbl, n16);
      }
      uint32_t h[2][4];
      B::finish(cur[r0], j, lk[p & 1][0], h[0]);
      B::finish(cur[r0 + 1], j, lk[p & 1][1], h[1]);
#pragma unroll
      for (int t = 0; t < T; t++) {
        const uint32_t(&x)[4] = af[t];
        acc[t][r0] = mfma_f16(x, h[0], acc[t][r0]);
        acc[t][r0 + 1] = mfma_f16(x, h[1], acc[t][r0 + 1]);
      }
    }
    }
    // the other activation buffer was last read one block ago, before the previous barrier: free to refill (with a
    // single buffer every wave has to be done with the block first)
    if (!DB) __syncthreads();
    a_store(DB ? (kb & 1u) ^ 1u : 0u);
#pragma unroll
    for (int r = 0; r < R; r++) cur[r] = nxt[r];
    __syncthreads();
  }

  float wts[T][4];  // routing weights of the lane's entries, fetched together ahead of the epilogue's math
#pragma unroll
  for (int t = 0; t < T; t++)
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t entry = base + min(16u * t + 4u * q + i, cnt - 1);
      wts[t][i] = GU && entry < a.total ? a.wt[entry] : 1.f;
    }
  __builtin_amdgcn_sched_barrier(0);  // all requests first: sunk to their uses they would be waited for one by one
#pragma unroll
  for (int t = 0; t < T; t++) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t tok = 16u * t + 4u * q + i;
      if (tok >= cnt) continue;
      const uint32_t entry = base + tok;
#pragma unroll
      for (int jt = 0; jt < RT; jt++) {
        if (row_of[jt] >= a.N) continue;
        if constexpr (GU) {
          const float g = fminf(acc[t][2 * jt][i], 10.f), u = fminf(fmaxf(acc[t][2 * jt + 1][i], -10.f), 10.f);
          const float hv = g / (1.f + expf(-g)) * u * wts[t][i];
          a.H[(size_t)entry * a.N + row_of[jt]] = __builtin_bit_cast(uint16_t, (_Float16)hv);
        } else {
          a.Z[(size_t)entry * a.N + row_of[jt]] = acc[t][jt][i];
        }
      }
    }
  }
  // the next chunk: its first block is in `cur` and in LDS already
#pragma unroll
  for (int jt = 0; jt < RT; jt++) row_of[jt] += WAVES * RT * 16;
  }
}

// Kernel variants: T = 3 takes the items of up to three token tiles in one launch, largest first (each runs the body
// built for its tile count; one launch has one tail of half-idle CUs); T = 7 the blocks of 49 to 112 entries that the
// popular experts are cut into (their weights are then decoded once per 112 entries; 12 waves, one activation buffer).
template <class B, bool GU, int T>
__global__ __launch_bounds__(64 * pf_blk_waves(T)) void moe_pf_block_kernel(const PfBlkArgs a) {
  if constexpr (T > 3) {
    pf_block_body<B, GU, T>(a);
  } else {
    const uint32_t item = ((blockIdx.x >> 3) / a.row_groups) * 8u + (blockIdx.x & 7u);
    if (item >= a.nitems) return;
    const uint32_t cnt = a.items[3 * item + 2];
    if (cnt > 32) pf_block_body<B, GU, 3>(a);
    else if (cnt > 16) pf_block_body<B, GU, 2>(a);
    else pf_block_body<B, GU, 1>(a);
  }
}

// ------------------------------------------------------------------------------------------------ scratch header
// The header of the prefill scratch (expert addresses, entry offsets, the shared expert's token tiles, the work items
// of the block GEMM) is built on the device. What only the host knows travels in kernel arguments: a raw image
//   word 0 n_exp | 1 has_shared | 2 n_tokens | 3 total | 4, 5 base address | 6 address mode | 7 unused
//   words 8 .. 8 + n_exp: entry offsets offs[0 .. n_exp]
//   then 3 addresses per expert (gate, up, down; the shared expert last): mode 0 one word each, (address - base) / 4;
//   mode 1 two words each
// cut into pieces of kHdrChunkWords (the argument block holds 4 KB). Every launch stores its piece behind the header;
// the last one then expands the image: addresses and offsets as the GEMM kernels read them, and the work items --
// an expert of m entries gives m / 112 blocks of 112 entries and one of m % 112 -- grouped by the token tiles a block
// fills, seven-tile blocks first, one-tile blocks last, inside a group in expert order (a counting sort over seven
// buckets: nothing in it depends on timing, so the table is the same on every run).
constexpr int kHdrChunkWords = 960, kHdrRawHead = 8, kHdrThreads = 1024;
struct HdrChunk { uint32_t w[kHdrChunkWords]; };
struct HdrBuild {
  uint32_t* raw;        // the image, behind the header
  uint64_t* ptrs;       // (n_exp + 1) x {gate, up, down}
  uint32_t* offs;       // n_exp + 2
  uint32_t* tiles;      // shared expert: {n_exp, first token} per 16 tokens
  uint32_t* items;      // routed items, then the shared expert's
  uint32_t build;       // 1: this launch holds the image's last piece and expands it
};
__host__ __device__ constexpr uint32_t pf_item_bucket(uint32_t cnt) { return 7u - (cnt + 15u) / 16u; }  // cnt in 1..112

// exclusive prefix of v over the workgroup's threads; total = sum over all; wsum: 17 words of LDS
__device__ __forceinline__ uint32_t hdr_scan(uint32_t v, uint32_t* wsum, uint32_t tid, uint32_t& total) {
  const uint32_t lane = tid & 63u, wave = tid >> 6;
  uint32_t inc = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t t = (uint32_t)__shfl_up((int)inc, d, 64);
    if (lane >= (uint32_t)d) inc += t;
  }
  if (lane == 63u) wsum[wave] = inc;
  __syncthreads();
  if (tid == 0) {
    uint32_t run = 0;
    for (uint32_t w = 0; w < kHdrThreads / 64; w++) { const uint32_t t = wsum[w]; wsum[w] = run; run += t; }
    wsum[kHdrThreads / 64] = run;
  }
  __syncthreads();
  total = wsum[kHdrThreads / 64];
  const uint32_t r = wsum[wave] + inc - v;
  __syncthreads();
  return r;
}

__global__ __launch_bounds__(kHdrThreads) void moe_pf_header_kernel(const HdrBuild b, const HdrChunk c, uint32_t word0, uint32_t nwords) {
  __shared__ uint32_t wsum[kHdrThreads / 64 + 1];
  const uint32_t tid = threadIdx.x;
  for (uint32_t i = tid; i < nwords; i += kHdrThreads) b.raw[word0 + i] = c.w[i];
  if (!b.build) return;
  __syncthreads();  // the image's earlier pieces were stored by earlier launches, the last one just now
  const uint32_t* raw = b.raw;
  const uint32_t ne = raw[0], has_shared = raw[1], n = raw[2], total = raw[3], mode = raw[6];
  const uint64_t base = (uint64_t)raw[4] | ((uint64_t)raw[5] << 32);
  const uint32_t* roffs = raw + kHdrRawHead;
  const uint32_t* rp = roffs + ne + 1;
  for (uint32_t i = tid; i < 3u * (ne + has_shared); i += kHdrThreads)
    b.ptrs[i] = mode ? ((uint64_t)rp[2 * i] | ((uint64_t)rp[2 * i + 1] << 32)) : base + 4ull * rp[i];
  for (uint32_t i = tid; i <= ne; i += kHdrThreads) b.offs[i] = roffs[i];
  if (tid == 0) b.offs[ne + 1] = total + n;
  if (has_shared)
    for (uint32_t i = tid; i < (n + 15u) / 16u; i += kHdrThreads) { b.tiles[2 * i] = ne; b.tiles[2 * i + 1] = 16u * i; }
  // routed items: this thread's experts [j0, j1)
  const uint32_t per = (ne + kHdrThreads - 1) / kHdrThreads, j0 = min(ne, tid * per), j1 = min(ne, j0 + per);
  uint32_t cnt[7] = {0, 0, 0, 0, 0, 0, 0};
  for (uint32_t j = j0; j < j1; j++) {
    const uint32_t m = roffs[j + 1] - roffs[j], r = m % 112u;
    cnt[0] += m / 112u;
    if (r) {
      const uint32_t bk = pf_item_bucket(r);
#pragma unroll
      for (int k = 0; k < 7; k++) cnt[k] += bk == (uint32_t)k;
    }
  }
  uint32_t at[7], first = 0;  // where this thread's items of each bucket start
#pragma unroll
  for (int k = 0; k < 7; k++) {
    uint32_t tot;
    at[k] = first + hdr_scan(cnt[k], wsum, tid, tot);
    first += tot;
  }
  for (uint32_t j = j0; j < j1; j++) {
    const uint32_t m = roffs[j + 1] - roffs[j], q = m / 112u, r = m % 112u;
    for (uint32_t k = 0; k < q; k++) {
      uint32_t* it = b.items + 3 * (size_t)at[0]++;
      it[0] = j; it[1] = 112u * k; it[2] = 112u;
    }
    if (r) {
      const uint32_t bk = pf_item_bucket(r);
      uint32_t pos = 0;
#pragma unroll
      for (int k = 0; k < 7; k++)
        if (bk == (uint32_t)k) pos = at[k]++;
      uint32_t* it = b.items + 3 * (size_t)pos;
      it[0] = j; it[1] = 112u * q; it[2] = r;
    }
  }
  // the shared expert's items follow: blocks of 112 tokens, then the rest
  if (has_shared) {
    const uint32_t q = n / 112u, r = n % 112u;
    for (uint32_t k = tid; k < q + (r ? 1u : 0u); k += kHdrThreads) {
      uint32_t* it = b.items + 3 * (size_t)(first + k);
      it[0] = ne; it[1] = 112u * k; it[2] = k < q ? 112u : r;
    }
  }
}

// Xg[i] = fp16(X[src(i)]): i < total gathers token tok[i]; rows total .. total + n - 1 are the tokens themselves. One
// workgroup per row, eight elements (one 16-byte store) per thread and pass.
template <bool X_BF16>
__global__ __launch_bounds__(256) void moe_pf_gather_kernel(const void* __restrict__ X, uint16_t* __restrict__ Xg,
                                                            const int* __restrict__ tok, uint32_t total, uint32_t nrows,
                                                            uint32_t dim) {
  const uint32_t i = blockIdx.x;
  if (i >= nrows) return;
  const uint32_t src = i < total ? (uint32_t)tok[i] : i - total;
  auto f = [](uint32_t w) { return __builtin_bit_cast(float, w); };
  for (uint32_t c8 = threadIdx.x; c8 < dim / 8; c8 += blockDim.x) {
    u32x4 o;
    if constexpr (X_BF16) {
      const u32x4 b = ((const u32x4*)((const uint16_t*)X + (size_t)src * dim))[c8];
      o = u32x4{pack_h2(f(b.x << 16), f(b.x & 0xFFFF0000u)), pack_h2(f(b.y << 16), f(b.y & 0xFFFF0000u)),
                pack_h2(f(b.z << 16), f(b.z & 0xFFFF0000u)), pack_h2(f(b.w << 16), f(b.w & 0xFFFF0000u))};
    } else {
      const u32x4* p = (const u32x4*)((const float*)X + (size_t)src * dim) + 2 * (size_t)c8;
      const u32x4 lo = p[0], hi = p[1];
      o = u32x4{pack_h2(f(lo.x), f(lo.y)), pack_h2(f(lo.z), f(lo.w)), pack_h2(f(hi.x), f(hi.y)), pack_h2(f(hi.z), f(hi.w))};
    }
    ((u32x4*)(Xg + (size_t)i * dim))[c8] = o;
  }
}

// Y[t] += Z[total + t] (shared) + sum_k Z[slot_of[t][k]] in fixed k order; tokens without any entry are left alone
__global__ __launch_bounds__(256) void moe_pf_reduce_kernel(const float* __restrict__ Z, float* __restrict__ Y,
                                                            const int* __restrict__ slot_of, uint32_t n, uint32_t total,
                                                            uint32_t dim, uint32_t k_per_token, uint32_t has_shared) {
  const uint32_t t = blockIdx.y;
  if (t >= n) return;
  for (uint32_t c4 = blockIdx.x * blockDim.x + threadIdx.x; c4 < dim / 4; c4 += gridDim.x * blockDim.x) {
    float4 s = has_shared ? ((const float4*)(Z + (size_t)(total + t) * dim))[c4] : make_float4(0.f, 0.f, 0.f, 0.f);
    bool any = has_shared != 0;
    for (uint32_t k = 0; k < k_per_token; k++) {
      const int i = slot_of[t * k_per_token + k];
      if (i >= 0) {
        const float4 z = ((const float4*)(Z + (size_t)i * dim))[c4];
        s.x += z.x; s.y += z.y; s.z += z.z; s.w += z.w;
        any = true;
      }
    }
    if (!any) continue;
    float4* y = (float4*)(Y + (size_t)t * dim) + c4;
    float4 o = *y;
    o.x += s.x; o.y += s.y; o.z += s.z; o.w += s.w;
    *y = o;
  }
}

}  // namespace msq
