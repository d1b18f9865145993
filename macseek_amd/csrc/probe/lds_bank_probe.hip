// Which lanes of a wave does the LDS serve together? Probe for bench.py --workload lds_bank_probe (libmsq_probe.so, no
// part of the library). Every lane of every wave reads the same address again and again: lane l at 256 l + 16 slot[l]
// (its own 256-byte row, i.e. its own bank period of 64 banks x 4 bytes), so two lanes touch the same banks exactly when
// their slots are equal, and a pattern of slots that costs no more than distinct slots tells which lanes are never
// served in the same pass. Eight waves keep the LDS saturated (a single wave issues a read every 16 cycles or so and
// hides everything but the worst conflicts).
#include <hip/hip_runtime.h>

#include <cstdint>

namespace msq {

template <int W>
__global__ __launch_bounds__(512) void lds_bank_probe_kernel(const uint32_t* __restrict__ addr, unsigned long long* __restrict__ out, int iters) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  for (uint32_t i = threadIdx.x; i < 65536u / 4u; i += 512u) ((uint32_t*)smem)[i] = i;
  __syncthreads();
  const uint32_t a = addr[threadIdx.x & 63u];
  uint32_t acc = 0;
  const unsigned long long t0 = __builtin_readcyclecounter();
  for (int it = 0; it < iters; it++) {
    uint4 v[16];
#pragma unroll
    for (int k = 0; k < 16; k++) {  // sixteen independent reads, one wait
      if constexpr (W == 16) asm volatile("ds_read_b128 %0, %1" : "=v"(v[k]) : "v"(a));
      else if constexpr (W == 8) asm volatile("ds_read_b64 %0, %1" : "=v"(*(uint2*)&v[k]) : "v"(a));
      else asm volatile("ds_read_b32 %0, %1" : "=v"(v[k].x) : "v"(a));
    }
    asm volatile("s_waitcnt lgkmcnt(0)");
#pragma unroll
    for (int k = 0; k < 16; k++) acc ^= v[k].x;
  }
  const unsigned long long t1 = __builtin_readcyclecounter();
  if (threadIdx.x == 0) out[0] = t1 - t0;
  if (acc == 0x12345678u) out[1] = acc;  // keeps the reads
}

}  // namespace msq

// One workgroup of eight waves; addr: 64 byte addresses (one per lane, below 64 KB, aligned to `width`); out: two
// 64-bit words, out[0] = cycles of wave 0 for iters x 16 reads per wave.
extern "C" int msq_probe_lds_bank(void* stream, int width, const void* addr, void* out, int iters) {
  if (!addr || !out || iters < 1) return -1;
  hipStream_t st = (hipStream_t)stream;
  auto go = [&](auto k) {
    if (hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, 65536) != hipSuccess) return -2;
    hipLaunchKernelGGL(k, dim3(1), dim3(512), 65536, st, (const uint32_t*)addr, (unsigned long long*)out, iters);
    return hipGetLastError() == hipSuccess ? 0 : -3;
  };
  switch (width) {
    case 16: return go(msq::lds_bank_probe_kernel<16>);
    case 8: return go(msq::lds_bank_probe_kernel<8>);
    case 4: return go(msq::lds_bank_probe_kernel<4>);
  }
  return -1;
}
