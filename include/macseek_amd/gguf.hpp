// C++20 shim: the reference's GGUF reader (ms::Gguf, src/gguf/gguf.hpp:38-96) and per-layer expert layout
// (ms::ExpertLayout::from_gguf, src/store/experts.hpp:35-42) over the libmsq C ABI. Same member names for what the
// quant / MoE path needs; file descriptors are not exposed (reads go through read() / load_tensor()).
#pragma once
#include <string>
#include <vector>

#include "quant.hpp"

namespace ms {

struct TensorInfo {  // reference: gguf.hpp:40-51
  std::string name;
  int type = 0, n_dims = 0;
  int64_t ne[4] = {1, 1, 1, 1};
  uint64_t nbytes = 0;
  int split = 0;
  uint64_t offset = 0;
  int index = -1;
  int64_t nelements() const { return ne[0] * ne[1] * ne[2] * ne[3]; }
  uint64_t row_bytes() const { return msq_gguf_type_bytes(type, (uint64_t)ne[0]); }
};

class Gguf {
 public:
  explicit Gguf(const std::string& path) { q::detail::check(msq_gguf_open(path.c_str(), &g_)); }
  ~Gguf() { msq_gguf_close(g_); }
  Gguf(const Gguf&) = delete;
  Gguf& operator=(const Gguf&) = delete;

  int64_t get_i64(const std::string& key, int64_t dflt = 0) const { return msq_gguf_get_i64(g_, key.c_str(), dflt); }
  double get_f64(const std::string& key, double dflt = 0) const { return msq_gguf_get_f64(g_, key.c_str(), dflt); }
  std::string get_str(const std::string& key, const std::string& dflt = "") const {
    const char* s = msq_gguf_get_str(g_, key.c_str(), nullptr);
    return s ? s : dflt;
  }
  std::vector<int64_t> get_arr_i64(const std::string& key) const {
    std::vector<int64_t> v((size_t)std::max<int64_t>(0, msq_gguf_arr_len(g_, key.c_str())));
    if (!v.empty()) v.resize((size_t)std::max<int64_t>(0, msq_gguf_arr_i64(g_, key.c_str(), v.data(), (int64_t)v.size())));
    return v;
  }
  std::vector<std::string> get_arr_str(const std::string& key) const {
    std::vector<std::string> v;
    for (int64_t i = 0; i < msq_gguf_arr_len(g_, key.c_str()); i++) {
      const char* s = msq_gguf_arr_str(g_, key.c_str(), i);
      if (!s) break;
      v.emplace_back(s);
    }
    return v;
  }

  std::vector<TensorInfo> tensors() const {
    std::vector<TensorInfo> v;
    for (int i = 0; i < msq_gguf_n_tensors(g_); i++) v.push_back(info(i));
    return v;
  }
  bool find(const std::string& name, TensorInfo* out) const {
    const int i = msq_gguf_find(g_, name.c_str());
    if (i < 0) return false;
    if (out) *out = info(i);
    return true;
  }
  TensorInfo at(const std::string& name) const {  // aborts if missing, like the reference
    TensorInfo t;
    if (!find(name, &t)) { fprintf(stderr, "gguf: tensor %s is missing\n", name.c_str()); abort(); }
    return t;
  }
  int n_splits() const { return msq_gguf_n_splits(g_); }
  uint32_t alignment() const { return msq_gguf_alignment(g_); }
  uint32_t version() const { return msq_gguf_version(g_); }
  const MsqGguf* handle() const { return g_; }

  // tensor bytes into host memory / device memory (enqueued on e's stream)
  long long read(const TensorInfo& t, void* dst, uint64_t len, uint64_t byte_off = 0) const { return msq_gguf_read(g_, t.index, byte_off, dst, len); }
  void load_tensor(Enc& e, const TensorInfo& t, const Buffer& dst) const {
    const MsqBuffer d = dst.c();
    q::detail::check(msq_gguf_load_tensor(e.stream, g_, t.index, 0, t.nbytes, &d));
  }

 private:
  TensorInfo info(int i) const {
    MsqGgufTensor m{};
    q::detail::check(msq_gguf_tensor(g_, i, &m));
    TensorInfo t;
    t.name = m.name; t.type = m.type; t.n_dims = m.n_dims; t.nbytes = m.nbytes; t.split = m.split; t.offset = m.offset; t.index = i;
    for (int d = 0; d < 4; d++) t.ne[d] = m.ne[d];
    return t;
  }
  MsqGguf* g_ = nullptr;
};

// reference: ExpertLayout::from_gguf for one layer, and resident placement of that layer in a device arena: fills
// `slots` (n_experts entries) with views for q::MoeDecodeArgs::slot / q::MoePrefillArgs::slots.
inline MsqExpertLayout expert_layout(const Gguf& g, int layer) {
  MsqExpertLayout L{};
  q::detail::check(msq_gguf_expert_layout(g.handle(), layer, &L));
  return L;
}
inline std::vector<q::ExpertSlot> place_experts(Enc& e, const Gguf& g, int layer, const Buffer& arena) {
  const MsqExpertLayout L = expert_layout(g, layer);
  std::vector<MsqExpertSlot> raw((size_t)L.n_experts);
  const MsqBuffer a = arena.c();
  q::detail::check(msq_gguf_place_experts(e.stream, g.handle(), layer, &a, raw.data(), L.n_experts));
  std::vector<q::ExpertSlot> out;
  for (const MsqExpertSlot& s : raw)
    out.push_back(q::ExpertSlot{Buffer{s.gate.dev, s.gate.off, s.gate.size}, Buffer{s.up.dev, s.up.off, s.up.size},
                                Buffer{s.down.dev, s.down.off, s.down.size}});
  return out;
}

}  // namespace ms
