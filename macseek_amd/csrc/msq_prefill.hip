// C ABI: prefill MoE (see include/msq.h; reference host code src/kernels/quant.mm:372-612).
#include <algorithm>
#include <array>
#include <cstdlib>
#include <cstring>
#include <vector>

#include <mutex>

#include "msq_host.h"
#include "msq_prefill.cuh"

namespace msq {
namespace {

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
// header: addresses | offsets | the shared expert's token tiles | work items | raw image (see moe_pf_header_kernel)
struct HdrLayout { size_t ptrs, offs, tiles, items, raw, bytes; };
HdrLayout header_layout(int total, int n, int n_exp) {
  HdrLayout h;
  const size_t tiles = (size_t)n / 16 + 2;                                          // the shared expert's
  const size_t items = 2 * ((size_t)n_exp + 1) + (size_t)total / kPfBigTokens + (size_t)n / kPfBigTokens;  // m / 112 blocks + a rest per expert
  const size_t raw_words = kHdrRawHead + ((size_t)n_exp + 1) + 6 * ((size_t)n_exp + 1);
  h.ptrs = 0;
  h.offs = 24 * (size_t)(n_exp + 1);
  h.tiles = h.offs + 4 * (size_t)(n_exp + 2);
  h.items = h.tiles + 8 * tiles;
  h.raw = h.items + 12 * items;
  h.bytes = align256(h.raw + 4 * raw_words);
  return h;
}
size_t header_bytes(int total, int n, int n_exp) { return header_layout(total, n, n_exp).bytes; }
bool routed_ok(int t) { return t == MSQ_IQ1_S || t == MSQ_IQ2_XXS; }
bool shared_ok(int t) { return t == MSQ_Q6_K || t == MSQ_Q8_0 || t == MSQ_IQ2_XXS || t == MSQ_IQ1_S; }

template <class F, bool GU>
int launch_gemm_t(hipStream_t st, PfArgs a, int cus) {
  const uint32_t waves = (a.nsteps + a.steps_per_wave - 1) / a.steps_per_wave;
  const uint32_t threads = 64 * waves;
  constexpr int NM = GU ? 2 : 1;
  const size_t window = ((size_t)16 * a.row_bytes + 30) & ~(size_t)15;
  const size_t base_lds = (size_t)F::LDS_WORDS * 4 + (size_t)NM * waves * 16 * 17 * 4;
  a.staged = (window <= (size_t)threads * kPfStageGranules * 16 && base_lds + NM * window <= 150 * 1024) ? 1u : 0u;
  const size_t lds = base_lds + (a.staged ? NM * window : 0);
  const uint32_t ntile_rows = (a.N + 15) / 16;
  // enough work items to fill the chip a few times, at least 8 weight tiles per item to amortise the A fragments
  uint32_t nchunks = std::max<uint32_t>(1, std::min<uint32_t>((4u * (uint32_t)cus + a.ntiles - 1) / a.ntiles, (ntile_rows + 7) / 8));
  a.chunk_tiles = (ntile_rows + nchunks - 1) / nchunks;
  a.nchunks = (ntile_rows + a.chunk_tiles - 1) / a.chunk_tiles;
  static bool attr_set = false;  // per instantiation: allow more than 64 KiB of dynamic LDS
  if (!attr_set) {
    MSQ_HIP(hipFuncSetAttribute((const void*)moe_pf_gemm_kernel<F, GU, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    MSQ_HIP(hipFuncSetAttribute((const void*)moe_pf_gemm_kernel<F, GU, false>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    attr_set = true;
  }
  if (a.staged) hipLaunchKernelGGL((moe_pf_gemm_kernel<F, GU, true>), dim3(a.ntiles * a.nchunks), dim3(threads), lds, st, a);
  else hipLaunchKernelGGL((moe_pf_gemm_kernel<F, GU, false>), dim3(a.ntiles * a.nchunks), dim3(threads), lds, st, a);
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}
template <class B, bool GU, int T>
int launch_block_tt(hipStream_t st, PfBlkArgs a) {
  if (!a.nitems) return MSQ_OK;
  const uint32_t rows_per_item = pf_blk_rows(GU, T);
  a.row_chunks = (a.N + rows_per_item - 1) / rows_per_item;
  static bool attr_set = false;  // per instantiation: allow more than 64 KiB of dynamic LDS
  if (!attr_set) {
    MSQ_HIP(hipFuncSetAttribute((const void*)moe_pf_block_kernel<B, GU, T>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    attr_set = true;
  }
  // two row chunks per workgroup while that leaves three workgroups and more per CU (MSQ_MOEP_CHUNKS imposes a count)
  static const int env_ch = [] { const char* e = getenv("MSQ_MOEP_CHUNKS"); return e && *e ? atoi(e) : 0; }();
  const uint32_t items8 = ((a.nitems + 7) / 8) * 8;
  uint32_t ch = env_ch > 0 ? (uint32_t)env_ch : ((size_t)items8 * ((a.row_chunks + 1) / 2) >= (size_t)3 * device_info().cus ? 2u : 1u);
  ch = std::max(1u, std::min(ch, a.row_chunks));
  if (a.N % rows_per_item || GU || T > 3) ch = 1;  // (a ragged last chunk clamps its rows: the chunks are then not a fixed stride apart)
  a.chunks_per_wg = ch;
  a.row_groups = (a.row_chunks + ch - 1) / ch;
  const uint32_t grid = items8 * a.row_groups;
  hipLaunchKernelGGL((moe_pf_block_kernel<B, GU, T>), dim3(grid), dim3(64 * pf_blk_waves(T)), pf_blk_lds<B>(T), st, a);
  MSQ_HIP(hipGetLastError());
  return MSQ_OK;
}
// A second stream of the library's own, per device, and the two events that fork work onto it and join it back. The
// routed experts' work falls into two classes that never meet before the final reduction: the popular experts' blocks
// (gate/up, then down of the same entries) and the small items (likewise). Each launch has one workgroup per CU and
// ends in a round that leaves CUs idle (the blocks' last round fills less than half of them); as two pipelines on two
// streams, each class starts on the CUs the other leaves idle, and no class waits for the other's gate/up before its
// own down. Fork and join are event dependencies, so a stream capture records them like any other (the objects are created
// outside of captures: by msq_init() or by the first call that is not being captured; until then calls stay on one stream).
struct SideStream { hipStream_t stream = nullptr; hipEvent_t fork = nullptr, join = nullptr; bool ok = false; };
std::mutex g_side_mu;
SideStream g_side[16];
// The device's side stream, or null when this call has to stay on the caller's stream: the fork is switched off, the
// objects do not exist yet and `st` is being captured, or the side stream still belongs to a stream capture that `st`
// is not part of (work forked from a capturing stream pulls the side stream into that capture until the capture ends;
// an eager call, or a call under another capture, must not enqueue into it). Call with g_side_mu held.
SideStream* side_stream(hipStream_t st) {
  static const bool off = [] { const char* e = getenv("MSQ_MOEP_ONE_STREAM"); return e && *e && atoi(e) != 0; }();
  int dev = 0;
  if (off || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
  SideStream& s = g_side[dev];
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  unsigned long long cid = 0;
  if (st && hipStreamGetCaptureInfo(st, &cs, &cid) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  if (!s.ok) {
    if (cs != hipStreamCaptureStatusNone) return nullptr;
    if (hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&s.fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&s.join, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    s.ok = true;
  }
  hipStreamCaptureStatus ss = hipStreamCaptureStatusNone;
  unsigned long long sid = 0;
  if (hipStreamGetCaptureInfo(s.stream, &ss, &sid) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  if (ss != hipStreamCaptureStatusNone && !(cs == hipStreamCaptureStatusActive && ss == hipStreamCaptureStatusActive && cid == sid))
    return nullptr;
  return &s;
}

// items are sorted by size, largest first: n6 blocks of more than 48 entries, n3 items of three token tiles, n2 of two,
// then the one-tile items; which: kBig (the blocks), kSmall (everything up to three tiles, one launch: one tail of
// half-idle CUs instead of two) or both; skip: profiling mask (see msq_moe_prefill)
enum { kBig = 1, kSmall = 2 };
template <class B, bool GU>
int launch_block_t(hipStream_t st, PfBlkArgs a, uint32_t n6, uint32_t n3, uint32_t n2, int skip, int which) {
  const uint32_t* items = a.items;
  const uint32_t n = a.nitems;
  int rc;
  a.items = items; a.nitems = n6;
  if ((which & kBig) && !(skip & 256) && (rc = launch_block_tt<B, GU, kPfBigTiles>(st, a))) return rc;
  if (!(which & kSmall)) return MSQ_OK;
  const uint32_t lo = (skip & 128) ? n6 + n3 + n2 : n6, hi = (skip & 64) ? n6 + n3 + n2 : n;
  a.items = items + 3 * (size_t)lo; a.nitems = hi > lo ? hi - lo : 0u;
  return launch_block_tt<B, GU, 3>(st, a);
}
bool block_path(int t) { return t == MSQ_IQ1_S || t == MSQ_IQ2_XXS; }
template <bool GU>
int launch_block(int t, hipStream_t st, const PfBlkArgs& a, uint32_t n6, uint32_t n3, uint32_t n2, int skip, int which) {
  return t == MSQ_IQ1_S ? launch_block_t<BlkIQ1S, GU>(st, a, n6, n3, n2, skip, which)
                        : launch_block_t<BlkIQ2XXS, GU>(st, a, n6, n3, n2, skip, which);
}

template <bool GU>
int launch_gemm(int t, hipStream_t st, const PfArgs& a, int cus) {
  switch (t) {  // the codebook formats never come here (block_path)
    case MSQ_Q6_K: return launch_gemm_t<FragQ6K, GU>(st, a, cus);
    case MSQ_Q8_0: return launch_gemm_t<FragQ8_0, GU>(st, a, cus);
  }
  return unsupported("moe_prefill types", t, 0, 0);
}

}  // namespace

void prefill_side_stream_setup() {
  std::lock_guard<std::mutex> lock(g_side_mu);
  (void)side_stream(nullptr);
}

}  // namespace msq

using namespace msq;

extern "C" {

size_t msq_moe_prefill_scratch_bytes(int total, int n, int n_exp, int dim, int inter) {
  if (dim <= 0) dim = MSQ_EXPERT_DIM;
  if (inter <= 0) inter = MSQ_EXPERT_INTER;
  const size_t rows = (size_t)std::max(total, 0) + (size_t)std::max(n, 0);
  return header_bytes(std::max(total, 0), std::max(n, 0), std::max(n_exp, 0)) + align256(rows * dim * 2) +
         align256(rows * inter * 2) + align256(rows * dim * 4);
}

int msq_moe_prefill(void* stream, const MsqMoePrefillArgs* p) {
  if (!p) return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_prefill: null arguments");
  const int n = p->n_tokens, ne = p->n_exp;
  if (n <= 0) return MSQ_OK;
  const int dim = p->dim ? p->dim : MSQ_EXPERT_DIM, inter = p->inter ? p->inter : MSQ_EXPERT_INTER;
  if (ne < 0 || (ne > 0 && (!p->slots || !p->offs))) return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_prefill: slots / offs missing");
  const int total = ne > 0 ? p->offs[ne] : 0;
  if (!routed_ok(p->t_gate_up) || !routed_ok(p->t_down) || (p->has_shared && !shared_ok(p->t_shared)))
    return unsupported("moe_prefill types", p->t_gate_up, 0, 0);
  if (dim < 256 || inter < 256 || dim % 256 || inter % 256 || dim > 8192 || inter > 8192)
    return unsupported("moe_prefill expert shape", p->t_gate_up, inter, dim);
  if (total < 0 || p->k_per_token < 0) return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_prefill: negative counts");
  for (int j = 0; j < ne; j++)
    if (p->offs[j + 1] < p->offs[j] || p->offs[0] != 0) return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_prefill: offs not ascending from 0");
  if (!buf_ok(&p->scratch, msq_moe_prefill_scratch_bytes(total, n, ne, dim, inter)))
    return fail(MSQ_ERR_SCRATCH, "macseek quant: moe_prefill scratch too small unsupported (type %s rows %d cols %d)",
                msq_type_name_of(p->t_gate_up), total, n);
  const size_t xbytes = (size_t)n * dim * (p->x_is_bf16 ? 2 : 4);
  if (!buf_ok(&p->X, xbytes) || !buf_ok(&p->Y, (size_t)n * dim * 4))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_prefill: X / Y missing or too small");
  if (((uintptr_t)bptr(&p->X) & 15) || ((uintptr_t)bptr(&p->Y) & 15) || ((uintptr_t)bptr(&p->scratch) & 255))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_prefill: X / Y not 16-byte aligned or scratch not 256-byte aligned");
  if (total > 0 && (!buf_ok(&p->tok, (size_t)total * 4) || !buf_ok(&p->wt, (size_t)total * 4)))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_prefill: tok / wt missing or too small");
  if (p->k_per_token > 0 && !buf_ok(&p->slot_of, (size_t)n * p->k_per_token * 4))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_prefill: slot_of missing or too small");
  const size_t rb_gu = msq_type_row_bytes(p->t_gate_up, dim), rb_d = msq_type_row_bytes(p->t_down, inter);
  const size_t rb_sgu = msq_type_row_bytes(p->t_shared, dim), rb_sd = msq_type_row_bytes(p->t_shared, inter);
  for (int j = 0; j < ne; j++) {
    const MsqExpertSlot& s = p->slots[j];
    if (!buf_ok(&s.gate, rb_gu * inter) || !buf_ok(&s.up, rb_gu * inter) || !buf_ok(&s.down, rb_d * dim))
      return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_prefill: expert slot %d missing or too small", j);
  }
  if (p->has_shared && (!buf_ok(&p->shared.gate, rb_sgu * inter) || !buf_ok(&p->shared.up, rb_sgu * inter) ||
                        !buf_ok(&p->shared.down, rb_sd * dim)))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: moe_prefill: shared expert missing or too small");

  hipStream_t st = (hipStream_t)stream;
  const int cus = device_info().cus;
  // PROFILING ONLY (wrong output): MSQ_MOEP_SKIP bit mask 1 gather, 2 routed gate/up, 4 shared gate/up, 8 routed down,
  // 16 shared down, 32 reduce; of the block GEMMs' work 64 the one-tile items, 128 the two- and three-tile
  // items, 256 the blocks of the popular experts -- read on every call (reference: MACSEEK_MOEP_SKIP,
  // src/kernels/quant.mm:520-522)
  const char* skip_env = getenv("MSQ_MOEP_SKIP");
  const int skip = skip_env && *skip_env ? atoi(skip_env) : 0;
  // ---- header. The host only counts the work items per class (the launches' grids); the tables themselves are built
  // on the device from a raw image that travels in kernel arguments (moe_pf_header_kernel): nothing is read from host
  // memory after this call returns, the call never waits for the stream, and a stream capture records the values.
  const HdrLayout hl = header_layout(total, n, ne);
  const uint32_t nt_shared = p->has_shared ? (uint32_t)((n + 15) / 16) : 0u;
  uint32_t ni_routed = 0, ni_shared = 0;
  uint32_t nc_routed[3] = {0, 0, 0}, nc_shared[3] = {0, 0, 0};  // items of more than 48 entries / three tiles / two tiles
  auto count = [](int m, uint32_t& ni, uint32_t* nc) {  // an expert of m entries: m / 112 blocks of 112 and one of m % 112
    const uint32_t q = (uint32_t)(m / kPfBigTokens), r = (uint32_t)(m % kPfBigTokens);
    ni += q + (r ? 1u : 0u);
    nc[0] += q + (r > 48 ? 1u : 0u); nc[1] += r > 32 && r <= 48; nc[2] += r > 16 && r <= 32;
  };
  for (int j = 0; j < ne; j++) count(p->offs[j + 1] - p->offs[j], ni_routed, nc_routed);
  if (p->has_shared) count(n, ni_shared, nc_shared);
  uint8_t* sc = bptr_mut(&p->scratch);
  {
    const int nptr = 3 * (ne + (p->has_shared ? 1 : 0));
    std::vector<uint64_t> ptrs((size_t)nptr);
    for (int j = 0; j < ne; j++) {
      ptrs[3 * j] = (uint64_t)(uintptr_t)bptr(&p->slots[j].gate);
      ptrs[3 * j + 1] = (uint64_t)(uintptr_t)bptr(&p->slots[j].up);
      ptrs[3 * j + 2] = (uint64_t)(uintptr_t)bptr(&p->slots[j].down);
    }
    if (p->has_shared) {
      ptrs[3 * ne] = (uint64_t)(uintptr_t)bptr(&p->shared.gate);
      ptrs[3 * ne + 1] = (uint64_t)(uintptr_t)bptr(&p->shared.up);
      ptrs[3 * ne + 2] = (uint64_t)(uintptr_t)bptr(&p->shared.down);
    }
    // addresses as one word each, (address - lowest address) / 4, when they all lie within 16 GiB of the lowest and
    // are 4 bytes apart (expert matrices are 4-byte aligned); else in full
    uint64_t base = nptr ? *std::min_element(ptrs.begin(), ptrs.end()) : 0;
    bool rel = true;
    for (uint64_t v : ptrs) rel = rel && !((v - base) & 3) && ((v - base) >> 2) <= 0xFFFFFFFFull;
    std::vector<uint32_t> raw;
    raw.reserve(kHdrRawHead + (size_t)ne + 1 + (rel ? 1 : 2) * (size_t)nptr);
    raw.insert(raw.end(), {(uint32_t)ne, p->has_shared ? 1u : 0u, (uint32_t)n, (uint32_t)total, (uint32_t)base, (uint32_t)(base >> 32),
                           rel ? 0u : 1u, 0u});
    for (int j = 0; j < ne; j++) raw.push_back((uint32_t)p->offs[j]);
    raw.push_back((uint32_t)total);
    for (uint64_t v : ptrs) {
      if (rel) raw.push_back((uint32_t)((v - base) >> 2));
      else { raw.push_back((uint32_t)v); raw.push_back((uint32_t)(v >> 32)); }
    }
    HdrBuild hb{};
    hb.raw = (uint32_t*)(sc + hl.raw); hb.ptrs = (uint64_t*)(sc + hl.ptrs); hb.offs = (uint32_t*)(sc + hl.offs);
    hb.tiles = (uint32_t*)(sc + hl.tiles); hb.items = (uint32_t*)(sc + hl.items);
    for (size_t w0 = 0; w0 < raw.size(); w0 += kHdrChunkWords) {
      HdrChunk c;
      const uint32_t nw = (uint32_t)std::min<size_t>(kHdrChunkWords, raw.size() - w0);
      memcpy(c.w, raw.data() + w0, 4 * (size_t)nw);
      hb.build = w0 + nw == raw.size() ? 1u : 0u;
      hipLaunchKernelGGL(moe_pf_header_kernel, dim3(1), dim3(kHdrThreads), 0, st, hb, c, (uint32_t)w0, nw);
    }
    MSQ_HIP(hipGetLastError());
  }
  const size_t hbytes = hl.bytes;
  const size_t rows = (size_t)total + n;
  uint16_t* Xg = (uint16_t*)(sc + hbytes);
  uint16_t* H = (uint16_t*)((uint8_t*)Xg + align256(rows * dim * 2));
  float* Z = (float*)((uint8_t*)H + align256(rows * inter * 2));
  const uint64_t* d_ptrs = (const uint64_t*)(sc + hl.ptrs);
  const uint32_t* d_offs = (const uint32_t*)(sc + hl.offs);
  const uint32_t* d_tiles = (const uint32_t*)(sc + hl.tiles);
  const uint32_t* d_items = (const uint32_t*)(sc + hl.items);
  const bool any_routed = total > 0;

  // 1) gather + convert
  const uint32_t grows = (uint32_t)(total + (p->has_shared ? n : 0));
  if (grows > 0 && !(skip & 1)) {
    const dim3 grid(grows), block(256);
    const int* tok = total > 0 ? (const int*)bptr(&p->tok) : nullptr;
    if (p->x_is_bf16) hipLaunchKernelGGL((moe_pf_gather_kernel<true>), grid, block, 0, st, (const void*)bptr(&p->X), Xg, tok, (uint32_t)total, grows, (uint32_t)dim);
    else hipLaunchKernelGGL((moe_pf_gather_kernel<false>), grid, block, 0, st, (const void*)bptr(&p->X), Xg, tok, (uint32_t)total, grows, (uint32_t)dim);
    MSQ_HIP(hipGetLastError());
  }
  PfArgs a{};
  a.H = H; a.Z = Z; a.wt = total > 0 ? (const float*)bptr(&p->wt) : nullptr;
  a.ptrs = d_ptrs; a.offs = d_offs; a.total = (uint32_t)total;
  auto steps = [&](uint32_t K) {
    a.K = K; a.nsteps = K / 32;
    const uint32_t ks = std::min<uint32_t>(16u, a.nsteps);
    a.steps_per_wave = (a.nsteps + ks - 1) / ks;
  };
  PfBlkArgs b{};
  b.H = H; b.Z = Z; b.wt = a.wt; b.ptrs = d_ptrs; b.offs = d_offs; b.total = (uint32_t)total;
  // one GEMM over the routed experts or over the shared expert: block kernel for the codebook formats, else the
  // token-tile kernel
  auto gemm = [&](auto gu_tag, int type, bool shared, const uint16_t* A, uint32_t K, uint32_t N, size_t row_bytes,
                  hipStream_t gs, int which) -> int {
    constexpr bool GU = decltype(gu_tag)::value;
    if (block_path(type)) {
      b.A = A; b.K = K; b.N = N; b.nblocks = K / 256; b.row_bytes = (uint32_t)row_bytes;
      b.items = d_items + (shared ? 3 * (size_t)ni_routed : 0); b.nitems = shared ? ni_shared : ni_routed;
      const uint32_t* nc = shared ? nc_shared : nc_routed;
      return launch_block<GU>(type, gs, b, nc[0], nc[1], nc[2], skip, which);
    }
    a.A = A; a.N = N; steps(K); a.row_bytes = (uint32_t)row_bytes;
    // (the token-tile kernel only ever serves a Q6_K / Q8_0 shared expert: routed experts are codebook formats)
    a.tiles = d_tiles; a.ntiles = shared ? nt_shared : 0u;
    if (!a.ntiles) return MSQ_OK;
    return launch_gemm<GU>(type, gs, a, cus);
  };
  int rc;
  const bool routed_gu = any_routed && !(skip & 2), routed_dn = any_routed && !(skip & 8);
  const int both = kBig | kSmall;
  // The routed experts' two item classes as two pipelines (see SideStream) when both exist and a side stream does
  bool forked = false;
  if ((routed_gu || routed_dn) && block_path(p->t_gate_up) && block_path(p->t_down) && nc_routed[0] > 0 &&
      ni_routed > nc_routed[0] && !(skip & 256) && (skip & (64 | 128)) != (64 | 128)) {
    std::lock_guard<std::mutex> lock(g_side_mu);
    SideStream* s = side_stream(st);
    if (s && hipEventRecord(s->fork, st) == hipSuccess && hipStreamWaitEvent(s->stream, s->fork, 0) == hipSuccess) {
      forked = true;
      rc = routed_gu ? gemm(std::true_type{}, p->t_gate_up, false, Xg, (uint32_t)dim, (uint32_t)inter, rb_gu, s->stream, kBig) : MSQ_OK;
      if (rc == MSQ_OK && routed_dn) rc = gemm(std::false_type{}, p->t_down, false, H, (uint32_t)inter, (uint32_t)dim, rb_d, s->stream, kBig);
      // whatever happened above, the side stream is joined back before anything else can fail: a caller's capture is
      // never left with an unjoined stream
      const hipError_t ej = hipEventRecord(s->join, s->stream);
      const hipError_t ew = ej == hipSuccess ? hipStreamWaitEvent(st, s->join, 0) : ej;
      if (rc == MSQ_OK && ew != hipSuccess) rc = hip_fail(ew, "joining the side stream");
      if (rc == MSQ_OK && routed_gu) rc = gemm(std::true_type{}, p->t_gate_up, false, Xg, (uint32_t)dim, (uint32_t)inter, rb_gu, st, kSmall);
      if (rc == MSQ_OK && nt_shared && !(skip & 4)) rc = gemm(std::true_type{}, p->t_shared, true, Xg, (uint32_t)dim, (uint32_t)inter, rb_sgu, st, both);
      if (rc == MSQ_OK && routed_dn) rc = gemm(std::false_type{}, p->t_down, false, H, (uint32_t)inter, (uint32_t)dim, rb_d, st, kSmall);
      if (rc == MSQ_OK && nt_shared && !(skip & 16)) rc = gemm(std::false_type{}, p->t_shared, true, H, (uint32_t)inter, (uint32_t)dim, rb_sd, st, both);
      if (rc != MSQ_OK) return rc;
    } else {
      (void)hipGetLastError();
    }
  }
  if (!forked) {
    // 2) gate + up + SwiGLU -> H
    if (routed_gu && (rc = gemm(std::true_type{}, p->t_gate_up, false, Xg, (uint32_t)dim, (uint32_t)inter, rb_gu, st, both))) return rc;
    if (nt_shared && !(skip & 4) && (rc = gemm(std::true_type{}, p->t_shared, true, Xg, (uint32_t)dim, (uint32_t)inter, rb_sgu, st, both))) return rc;
    // 3) down -> Z
    if (routed_dn && (rc = gemm(std::false_type{}, p->t_down, false, H, (uint32_t)inter, (uint32_t)dim, rb_d, st, both))) return rc;
    if (nt_shared && !(skip & 16) && (rc = gemm(std::false_type{}, p->t_shared, true, H, (uint32_t)inter, (uint32_t)dim, rb_sd, st, both))) return rc;
  }
  // 4) ordered reduction into Y
  if ((any_routed || nt_shared) && !(skip & 32)) {
    const dim3 grid((dim / 4 + 255) / 256, (unsigned)n), block(256);
    hipLaunchKernelGGL(moe_pf_reduce_kernel, grid, block, 0, st, (const float*)Z, (float*)bptr_mut(&p->Y),
                       p->k_per_token > 0 ? (const int*)bptr(&p->slot_of) : nullptr, (uint32_t)n, (uint32_t)total, (uint32_t)dim,
                       (uint32_t)(any_routed ? p->k_per_token : 0), (uint32_t)(p->has_shared ? 1 : 0));
    MSQ_HIP(hipGetLastError());
  }
  return MSQ_OK;
}

}  // extern "C"
