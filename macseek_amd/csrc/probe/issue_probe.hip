// NOT part of libmsq.so: a measurement tool of the benchmark, built into a shared object of its own (libmsq_probe.so)
// that only `bench.py --workload issue_probe` loads.
//
// Instruction-issue probes: how fast one SIMD of this device issues the instruction kinds the decode and prefill
// kernels are built from, alone and mixed, at a chosen number of waves per SIMD. The design decisions that rest on
// these figures (vector-issue ceiling of a table decode, whether matrix-core work hides behind vector work) can be
// re-measured with `bench.py --workload issue_probe`.
//
// Every kernel runs `iters` iterations of a fixed instruction group per wave and writes nothing unless an impossible
// value appears, so the measured time is issue + execution of the group only. Groups:
//   VALU   32 independent full-rate vector ops (v_dot2_f32_f16 and v_and_or_b32 alternating, four chains each)
//   MFMA16 8 x v_mfma_f32_16x16x32_f16, four independent accumulators
//   MFMA4  8 x v_mfma_scale_f32_16x16x128_f8f6f4 with fp4 A and fp6 B operands (block-scaled), four accumulators
//   MFMA8  8 x the same instruction with fp8 A and B operands
//   LDS    16 x ds_read_b32 at per-lane pseudo-random addresses inside a 8 KB table (+ one v_xor per value read)
//   VINT   32 x v_and_or_b32 (integer only: nothing that could share hardware with the matrix cores)
//   VPK    32 x v_pk_mul_f16 (packed fp16 arithmetic, four chains)
//   VFMA   32 x v_fma_f32 (four chains)
// and the mixes VALU+MFMA16, VALU+MFMA4, VALU+LDS, VALU+LDS+MFMA4, VINT+MFMA16, VPK+MFMA16, VFMA+MFMA16 (groups
// interleaved 4 : 1 in program order).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace msq {

typedef _Float16 ph8_t __attribute__((ext_vector_type(8)));
typedef _Float16 ph2_t __attribute__((ext_vector_type(2)));
typedef float pf4_t __attribute__((ext_vector_type(4)));
typedef int pi8_t __attribute__((ext_vector_type(8)));

enum { P_VALU = 1, P_MFMA16 = 2, P_MFMA4 = 4, P_MFMA8 = 8, P_LDS = 16, P_VINT = 32, P_VPK = 64, P_VFMA = 128 };

template <int MASK>
__global__ __launch_bounds__(1024) void issue_probe_kernel(uint32_t* sink, uint32_t iters, uint32_t seed) {
  __shared__ uint32_t tbl[2048];
  const uint32_t tid = threadIdx.x;
  for (uint32_t i = tid; i < 2048; i += blockDim.x) tbl[i] = i * seed;
  __syncthreads();
  // vector state
  float f[4] = {0.f, 0.f, 0.f, 0.f};
  uint32_t u[4] = {tid, tid * 3u, tid * 5u, tid * 7u};
  const uint32_t w = 0x3c003c00u | tid, xs = seed | 0x38003800u;
  // matrix state
  ph8_t ha = {1, 2, 3, 4, 5, 6, 7, 8}, hb = {1, 1, 1, 1, 1, 1, 1, 1};
  pi8_t qa = {(int)(tid * 0x01010101u), (int)seed, 3, 4, 5, 6, 7, 8}, qb = {(int)seed, 2, (int)tid, 4, 5, 6, 7, 8};
  pf4_t c[4] = {};
  const int sc = 0x7f7f7f7f;
  // LDS state
  uint32_t off[4] = {(tid * 2654435761u >> 19) & 0x1FFCu, (tid * 40503u >> 3) & 0x1FFCu, (tid * 9973u) & 0x1FFCu, (tid * 31u + 64u) & 0x1FFCu};
  uint32_t ld = 0, lv[2] = {0, 0};

  for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
    for (int g = 0; g < 8; g++) {
      if constexpr (MASK & P_VALU) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          if (j & 1) {
            u[(g + j) & 3] = (u[(g + j) & 3] & 0x00FFF0F0u) | u[(g + j + 1) & 3];  // one v_and_or_b32
            asm volatile("" : "+v"(u[(g + j) & 3]));
          } else {
            f[(g + j) & 3] = __builtin_amdgcn_fdot2(__builtin_bit_cast(ph2_t, w), __builtin_bit_cast(ph2_t, xs), f[(g + j) & 3], false);
            asm volatile("" : "+v"(f[(g + j) & 3]));
          }
        }
      }
      if constexpr (MASK & P_VINT) {  // integer-only vector group: no dot-product unit involved
#pragma unroll
        for (int j = 0; j < 4; j++) {
          u[(g + j) & 3] = (u[(g + j) & 3] & 0x00FFF0F0u) | u[(g + j + 1) & 3];
          asm volatile("" : "+v"(u[(g + j) & 3]));
        }
      }
      if constexpr (MASK & P_VPK) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const ph2_t r = __builtin_bit_cast(ph2_t, u[(g + j) & 3]) * __builtin_bit_cast(ph2_t, w);  // one v_pk_mul_f16
          u[(g + j) & 3] = __builtin_bit_cast(uint32_t, r);
          asm volatile("" : "+v"(u[(g + j) & 3]));
        }
      }
      if constexpr (MASK & P_VFMA) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          f[(g + j) & 3] = __builtin_fmaf(f[(g + j) & 3], __builtin_bit_cast(float, xs), __builtin_bit_cast(float, w));
          asm volatile("" : "+v"(f[(g + j) & 3]));
        }
      }
      if constexpr (MASK & P_LDS) {
#pragma unroll
        for (int j = 0; j < 2; j++) {  // the values read one group ago are consumed now (one v_xor each)
          ld ^= lv[j];
          asm volatile("" : "+v"(off[(2 * g + j) & 3]));
          lv[j] = *(const uint32_t*)((const uint8_t*)tbl + off[(2 * g + j) & 3]);
        }
      }
      if constexpr (MASK & P_MFMA16) c[g & 3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ha, hb, c[g & 3], 0, 0, 0);
      if constexpr (MASK & P_MFMA4) c[g & 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(qa, qb, c[g & 3], 4, 2, 0, sc, 0, sc);
      if constexpr (MASK & P_MFMA8) c[g & 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(qa, qb, c[g & 3], 0, 0, 0, sc, 0, sc);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float total = f[0] + f[1] + f[2] + f[3];
#pragma unroll
  for (int i = 0; i < 4; i++) total += c[i][0] + c[i][1] + c[i][2] + c[i][3];
  const uint32_t all = u[0] ^ u[1] ^ u[2] ^ u[3] ^ ld ^ lv[0] ^ lv[1];
  if (total == 1.2345e-30f || all == 0xFEDCBA98u) sink[blockIdx.x] = all;  // never true: keeps both results live
}

template <int MASK>
static void launch_probe(hipStream_t st, int grid, int block, uint32_t* sink, uint32_t iters) {
  hipLaunchKernelGGL(issue_probe_kernel<MASK>, dim3((unsigned)grid), dim3((unsigned)block), 0, st, sink, iters, 0x9E3779B9u);
}

}  // namespace msq

using namespace msq;

// mask ORs the groups above (1 VALU, 2 MFMA16, 4 MFMA4, 8 MFMA8, 16 LDS, 32 VINT, 64 VPK, 128 VFMA); sink holds at least
// 4 * grid bytes of device memory. Returns 0, -1 for a bad launch shape or an unknown mix, or the HIP error code.
extern "C" int msq_probe_issue(void* stream, int mask, int grid, int block, int iters, void* sink, size_t sink_bytes) {
  if (grid < 1 || block < 64 || block > 1024 || block % 64 || iters < 1 || !sink || sink_bytes < (size_t)grid * 4) return -1;
  hipStream_t st = (hipStream_t)stream;
  uint32_t* s = (uint32_t*)sink;
  switch (mask) {
    case P_VALU: launch_probe<P_VALU>(st, grid, block, s, iters); break;
    case P_MFMA16: launch_probe<P_MFMA16>(st, grid, block, s, iters); break;
    case P_MFMA4: launch_probe<P_MFMA4>(st, grid, block, s, iters); break;
    case P_MFMA8: launch_probe<P_MFMA8>(st, grid, block, s, iters); break;
    case P_LDS: launch_probe<P_LDS>(st, grid, block, s, iters); break;
    case P_VALU | P_MFMA16: launch_probe<P_VALU | P_MFMA16>(st, grid, block, s, iters); break;
    case P_VALU | P_MFMA4: launch_probe<P_VALU | P_MFMA4>(st, grid, block, s, iters); break;
    case P_VALU | P_LDS: launch_probe<P_VALU | P_LDS>(st, grid, block, s, iters); break;
    case P_VINT: launch_probe<P_VINT>(st, grid, block, s, iters); break;
    case P_VINT | P_MFMA16: launch_probe<P_VINT | P_MFMA16>(st, grid, block, s, iters); break;
    case P_VPK: launch_probe<P_VPK>(st, grid, block, s, iters); break;
    case P_VPK | P_MFMA16: launch_probe<P_VPK | P_MFMA16>(st, grid, block, s, iters); break;
    case P_VFMA: launch_probe<P_VFMA>(st, grid, block, s, iters); break;
    case P_VFMA | P_MFMA16: launch_probe<P_VFMA | P_MFMA16>(st, grid, block, s, iters); break;
    case P_VALU | P_LDS | P_MFMA4: launch_probe<P_VALU | P_LDS | P_MFMA4>(st, grid, block, s, iters); break;
    default: return -1;
  }
  return (int)hipGetLastError();
}
