// The C++ shim (include/macseek_amd/quant.hpp) driven the way the reference's own tests drive ms::q
// (tests/test_quant_matvec.mm:31-47): build inputs, encode on an Enc, wait, compare. Known answers only, so the
// program needs nothing but the library: Q8_0 blocks with d = 1/8 and quants j - 16 against an exact host dot, the
// same through encode_matvec_n, and the abort-on-misuse contract in a child process.
#include <hip/hip_runtime.h>
#include <sys/wait.h>
#include <unistd.h>

#include <cmath>
#include <cstring>
#include <vector>

#include "macseek_amd/arch.hpp"
#include "macseek_amd/gguf.hpp"
#include "macseek_amd/quant.hpp"

#define HIP_OK(e) do { hipError_t r_ = (e); if (r_ != hipSuccess) { fprintf(stderr, "HIP: %s\n", hipGetErrorString(r_)); return 2; } } while (0)

static ms::Buffer upload(const void* p, size_t n) {
  void* d = nullptr;
  if (hipMalloc(&d, n) != hipSuccess || hipMemcpy(d, p, n, hipMemcpyHostToDevice) != hipSuccess) abort();
  return ms::Buffer{d, 0, n};
}

int main() {
  namespace mq = ms::q;
  const int rows = 48, cols = 512, n = 3;
  std::vector<uint8_t> W((size_t)rows * mq::row_bytes(mq::QType::Q8_0, cols));
  std::vector<float> x((size_t)cols * n), want((size_t)rows * n, 0.f);
  for (size_t i = 0; i < x.size(); i++) x[i] = (float)((int)(i * 7 % 13) - 6) * 0.25f;  // exact in fp16
  for (int r = 0; r < rows; r++)
    for (int b = 0; b < cols / 32; b++) {
      uint8_t* blk = W.data() + ((size_t)r * (cols / 32) + b) * 34;
      const uint16_t d = 0x3000;  // fp16 0.125
      memcpy(blk, &d, 2);
      for (int j = 0; j < 32; j++) blk[2 + j] = (uint8_t)(int8_t)((j + r + b) % 33 - 16);
      for (int t = 0; t < n; t++)
        for (int j = 0; j < 32; j++) want[(size_t)t * rows + r] += 0.125f * (float)((j + r + b) % 33 - 16) * x[(size_t)t * cols + b * 32 + j];
    }
  ms::Buffer bw = upload(W.data(), W.size()), bx = upload(x.data(), x.size() * 4);
  std::vector<float> zero((size_t)rows * n, 0.f), got((size_t)rows * n);
  ms::Buffer by = upload(zero.data(), zero.size() * 4);
  ms::Enc e;
  int fails = 0;
  mq::encode_matvec(e, mq::QType::Q8_0, bw, rows, cols, bx, by);  // n = 1: first activation row
  HIP_OK(hipStreamSynchronize((hipStream_t)e.stream));
  HIP_OK(hipMemcpy(got.data(), by.buf, rows * 4, hipMemcpyDeviceToHost));
  for (int r = 0; r < rows; r++) if (std::fabs(got[r] - want[r]) > 1e-4f * (1.f + std::fabs(want[r]))) fails++;
  printf("  encode_matvec   Q8_0 [%d -> %d] %s\n", cols, rows, fails ? "FAIL" : "ok");
  mq::encode_matvec_n(e, mq::QType::Q8_0, bw, rows, cols, bx, by, n);
  HIP_OK(hipStreamSynchronize((hipStream_t)e.stream));
  HIP_OK(hipMemcpy(got.data(), by.buf, got.size() * 4, hipMemcpyDeviceToHost));
  int f2 = 0;
  for (size_t i = 0; i < got.size(); i++) if (std::fabs(got[i] - want[i]) > 1e-4f * (1.f + std::fabs(want[i]))) f2++;
  printf("  encode_matvec_n Q8_0 [%d -> %d] n=%d %s\n", cols, rows, n, f2 ? "FAIL" : "ok");
  fails += f2;
  if (mq::matvec_cfg(mq::QType::Q8_0, rows, cols).ks < 1) fails++;
  {  // ms::arch router shim: known answers (ties go to the lower expert id; equal logits share the scale equally)
    namespace ma = ms::arch;
    const int nt = 2, E = ma::kExperts;
    std::vector<float> logits((size_t)nt * E, -30.f), bias(E, 0.f);
    const int pick[6] = {300, 200, 50, 100, 20, 10};
    const float val[6] = {30.f, 25.f, 0.f, 0.f, -1.f, -2.f};
    for (int k = 0; k < 6; k++) logits[pick[k]] = val[k];
    for (int i = 0; i < E; i++) logits[E + i] = 0.f;
    ms::Buffer bl = upload(logits.data(), logits.size() * 4), bb = upload(bias.data(), bias.size() * 4);
    std::vector<uint32_t> z(512, 0);
    ms::Buffer ids = upload(z.data(), nt * 24), wts = upload(z.data(), nt * 24);
    ma::RouteLists L;
    L.counts = upload(z.data(), E * 4); L.offsets = upload(z.data(), (E + 1) * 4);
    L.entry = upload(z.data(), nt * 24); L.tok = upload(z.data(), nt * 24); L.w = upload(z.data(), nt * 24);
    L.slot_of = upload(z.data(), nt * 24); L.max_tokens = nt;
    ma::encode_router_topk(e, bl, bb, ids, wts, nt);
    ma::encode_route_lists(e, ids, wts, nt, L);
    HIP_OK(hipStreamSynchronize((hipStream_t)e.stream));
    int gid[12]; float gw[12]; uint32_t off[385], slot[12], ent[12];
    HIP_OK(hipMemcpy(gid, ids.buf, 48, hipMemcpyDeviceToHost)); HIP_OK(hipMemcpy(gw, wts.buf, 48, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(off, L.offsets.buf, 385 * 4, hipMemcpyDeviceToHost)); HIP_OK(hipMemcpy(slot, L.slot_of.buf, 48, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(ent, L.entry.buf, 48, hipMemcpyDeviceToHost));
    int f3 = 0;
    float sum0 = 0.f;
    for (int k = 0; k < 6; k++) { f3 += gid[k] != pick[k]; f3 += gid[6 + k] != k; f3 += std::fabs(gw[6 + k] - 0.25f) > 1e-6f; sum0 += gw[k]; }
    f3 += std::fabs(sum0 - 1.5f) > 1e-5f;
    f3 += off[E] != 12;
    for (int i = 0; i < 12; i++) f3 += ent[slot[i]] != (uint32_t)i;
    printf("  ms::arch router_topk + route_lists %s\n", f3 ? "FAIL" : "ok");
    fails += f3;
  }
  {  // ms::Gguf shim: a two-tensor file written here (GGUF v3, default alignment 32)
    std::vector<uint8_t> f;
    auto put = [&](const void* p, size_t n) { f.insert(f.end(), (const uint8_t*)p, (const uint8_t*)p + n); };
    auto u32 = [&](uint32_t v) { put(&v, 4); };
    auto u64 = [&](uint64_t v) { put(&v, 8); };
    auto str = [&](const char* s) { u64(strlen(s)); put(s, strlen(s)); };
    u32(0x46554747u); u32(3); u64(1); u64(2);
    str("general.architecture"); u32(8); str("deepseek41");
    str("deepseek41.expert_count"); u32(4); u32(384);
    str("w"); u32(2); u64(32); u64(2); u32(8); u64(0);  // Q8_0 [32, 2]
    while (f.size() % 32) f.push_back(0);
    const size_t data_off = f.size();
    for (int i = 0; i < 68; i++) f.push_back((uint8_t)(i * 3 + 1));
    const char* path = "/tmp/msq_shim_test.gguf";
    FILE* fp = fopen(path, "wb");
    int f4 = fp == nullptr;
    if (fp) { f4 += fwrite(f.data(), 1, f.size(), fp) != f.size(); fclose(fp); }
    if (!f4) {
      ms::Gguf g(path);
      const ms::TensorInfo t = g.at("w");
      uint8_t back[68];
      f4 += g.get_str("general.architecture") != "deepseek41" || g.get_i64("deepseek41.expert_count") != 384;
      f4 += t.type != 8 || t.ne[0] != 32 || t.ne[1] != 2 || t.nbytes != 68 || t.offset != data_off || t.row_bytes() != 34;
      f4 += g.read(t, back, 68) != 68 || memcmp(back, f.data() + data_off, 68) != 0;
      f4 += g.tensors().size() != 1 || g.alignment() != 32;
    }
    remove(path);
    printf("  ms::Gguf parse + read %s\n", f4 ? "FAIL" : "ok");
    fails += f4;
  }
  // misuse aborts like the reference (src/kernels/quant.mm:34-37): cols not a multiple of the block size
  fflush(stdout);
  const pid_t pid = fork();
  if (pid == 0) {
    fclose(stderr);
    ms::Enc e2;
    mq::encode_matvec(e2, mq::QType::Q6_K, bw, 4, 300, bx, by);
    _exit(0);
  }
  int st = 0;
  waitpid(pid, &st, 0);
  const bool aborted = WIFSIGNALED(st) && WTERMSIG(st) == SIGABRT;
  printf("  misuse aborts: %s\n", aborted ? "ok" : "FAIL");
  fails += !aborted;
  printf(fails ? "FAILED (%d)\n" : "all OK\n", fails);
  return fails ? 1 : 0;
}
