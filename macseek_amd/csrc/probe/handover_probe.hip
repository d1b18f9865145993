// NOT part of libmsq.so: a measurement tool of the benchmark (libmsq_probe.so, `bench.py --workload handover_probe`).
//
// What an in-kernel, device-wide hand-over costs on this eight-XCD part -- the step a single-launch MoE layer would
// need between its gate/up half (256 workgroups write h) and its down half (every workgroup reads all of h), against
// the kernel boundary that the two-launch layer uses. Every workgroup of a one-workgroup-per-CU launch
//   1. stores its share of an h-sized array with device-scope stores and waits until they are acknowledged   (stamp 1)
//   2. announces itself: one device-scope atomic add, either on one counter for the whole device (flat) or on its
//      XCD's counter, whose last arrival adds to the device's counter (two-level)                               (stamp 2)
//   3. polls the device's counter until every workgroup has arrived -- a bounded wait: it gives up after
//      `max_polls` reads and the launch reports that                                                          (stamp 3)
//   4. reads the whole array (28 KB, the fp16 form of seven h rows of 2048) with device-scope loads            (stamp 4)
// and leaves its four stamps (100 MHz wall clock, relative to its own start) in `out`. Counters only grow, launch k
// waits for (k + 1) arrivals per workgroup, so nothing is reset between launches.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace msq {

__device__ unsigned long long g_hp_device[2];   // [mode]
__device__ unsigned long long g_hp_xcd[2][8 * 16];  // one counter per XCD, 128 bytes apart

__global__ __launch_bounds__(1024) void handover_probe_kernel(uint32_t* h, uint32_t h_words, uint32_t two_level, uint32_t epoch,
                                                              uint32_t max_polls, uint64_t* out, uint32_t* sink) {
  __shared__ uint32_t ok;
  const uint32_t tid = threadIdx.x, wg = blockIdx.x, nwg = gridDim.x;
  const uint64_t t0 = wall_clock64();
  // 1. this workgroup's share of h
  const uint32_t per = (h_words + nwg - 1) / nwg;
  for (uint32_t i = tid; i < per; i += blockDim.x) {
    const uint32_t at = wg * per + i;
    if (at < h_words) __hip_atomic_store(h + at, epoch * 977u + at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const uint64_t t1 = wall_clock64();
  uint64_t t2 = 0, t3 = 0;
  if (tid == 0) {
    // 2. arrival
    const unsigned long long want = (unsigned long long)nwg * (epoch + 1ull);
    if (two_level) {
      const uint32_t x = wg & 7u, members = (nwg - x + 7u) / 8u;  // workgroups are dealt round-robin over the XCDs
      const unsigned long long old = __hip_atomic_fetch_add(&g_hp_xcd[1][x * 16], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (old + 1ull == (unsigned long long)members * (epoch + 1ull))
        __hip_atomic_fetch_add(&g_hp_device[1], (unsigned long long)members, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      __hip_atomic_fetch_add(&g_hp_device[0], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    t2 = wall_clock64();
    // 3. bounded wait for the others
    uint32_t polls = 0, good = 1;
    while (__hip_atomic_load(&g_hp_device[two_level ? 1 : 0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) {
      if (++polls >= max_polls) { good = 0; break; }
      __builtin_amdgcn_s_sleep(1);
    }
    ok = good;
    t3 = wall_clock64();
  }
  __syncthreads();
  // 4. all of h, device-scope loads (two 8-byte loads per thread and pass)
  uint64_t acc = 0;
  const unsigned long long* p = (const unsigned long long*)h;
  const uint32_t n8 = h_words / 2;
  for (uint32_t i = tid; i < n8; i += 2 * blockDim.x) {
    const unsigned long long a = __hip_atomic_load(p + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long b = __hip_atomic_load(p + (i + blockDim.x < n8 ? i + blockDim.x : i), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    acc += a ^ b;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const uint64_t t4 = wall_clock64();
  if (acc == 0x123456789ull) sink[wg] = 1;  // practically never: keeps the loads alive
  if (tid == 0) {
    uint64_t* o = out + 5 * (size_t)wg;
    o[0] = t1 - t0; o[1] = t2 - t0; o[2] = t3 - t0; o[3] = t4 - t0; o[4] = ok;
  }
}

}  // namespace msq

// h: device memory of h_words 32-bit words; out: 5 x grid 64-bit words; sink: grid 32-bit words. `epoch` must count the
// launches of a mode (0 flat, 1 two-level) since the library was loaded. Returns 0 or the HIP error code.
extern "C" int msq_probe_handover(void* stream, int grid, void* h, uint32_t h_words, int two_level, uint32_t epoch, uint32_t max_polls,
                                  void* out, void* sink) {
  if (grid < 1 || !h || !out || !sink) return -1;
  hipLaunchKernelGGL(msq::handover_probe_kernel, dim3((unsigned)grid), dim3(1024), 0, (hipStream_t)stream, (uint32_t*)h, h_words,
                     two_level ? 1u : 0u, epoch, max_polls, (uint64_t*)out, (uint32_t*)sink);
  return (int)hipGetLastError();
}
