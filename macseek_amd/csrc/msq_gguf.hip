// C ABI: GGUF reader and resident expert placement -- the on-disk format on the input side of the kernels (see
// include/msq.h; reference: ms::Gguf, src/gguf/gguf.hpp:38-96 and src/gguf/gguf.cpp; ExpertLayout::from_gguf,
// src/store/experts.hpp:35-42, src/store/experts.mm:36-56).
//
// The file format is the public GGUF container (versions 2 and 3): header {magic "GGUF", u32 version, u64 tensor count,
// u64 key-value count}, typed key-value pairs, tensor table {name, dims, ggml type, offset into the data section}, then
// the data section at the next multiple of general.alignment (32 unless stated). A model may be split over files named
// *-0000N-of-0000M.gguf; tensors are reported with absolute offsets in their split, metadata merged (first wins).
//
// Placement: the reference streams experts from SSD into a cache arena; an MI355X holds all of them (288 GB of HBM), so
// a layer's experts are copied once, each matrix at a 256-byte aligned offset of a caller-owned device arena, and the
// kernels then take MsqExpertSlot views of it.
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <string>
#include <unordered_map>
#include <vector>

#include "msq_host.h"

namespace msq {
namespace {

struct TypeRow { int t; const char* name; uint32_t blck, bytes; };
// ggml type table (ids, elements per block, bytes per block): src/gguf/gguf.cpp:17-30
const TypeRow kTypes[] = {
    {0, "F32", 1, 4},       {1, "F16", 1, 2},       {2, "Q4_0", 32, 18},    {3, "Q4_1", 32, 20},     {6, "Q5_0", 32, 22},
    {7, "Q5_1", 32, 24},    {8, "Q8_0", 32, 34},    {9, "Q8_1", 32, 36},    {10, "Q2_K", 256, 84},   {11, "Q3_K", 256, 110},
    {12, "Q4_K", 256, 144}, {13, "Q5_K", 256, 176}, {14, "Q6_K", 256, 210}, {15, "Q8_K", 256, 292},  {16, "IQ2_XXS", 256, 66},
    {17, "IQ2_XS", 256, 74}, {18, "IQ3_XXS", 256, 98}, {19, "IQ1_S", 256, 50}, {20, "IQ4_NL", 32, 18}, {21, "IQ3_S", 256, 110},
    {22, "IQ2_S", 256, 82}, {23, "IQ4_XS", 256, 136}, {24, "I8", 1, 1},     {25, "I16", 1, 2},       {26, "I32", 1, 4},
    {27, "I64", 1, 8},      {28, "F64", 1, 8},      {29, "IQ1_M", 256, 56}, {30, "BF16", 1, 2},      {34, "TQ1_0", 256, 54},
    {35, "TQ2_0", 256, 66}, {39, "MXFP4", 32, 17},
};
const TypeRow* type_row(int t) {
  for (const TypeRow& r : kTypes)
    if (r.t == t) return &r;
  return nullptr;
}

enum Kv : uint32_t { U8 = 0, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 };

// One metadata value. Scalars land in i (every integer and bool kind), f (both float kinds) or s; an array keeps its
// elements in the one list that fits its element kind.
struct Value {
  uint32_t type = U8, arr_type = U8;
  int64_t i = 0;
  double f = 0;
  std::string s;
  std::vector<int64_t> ints;
  std::vector<double> floats;
  std::vector<std::string> strings;
  std::vector<Value> nested;
  size_t size() const { return type == ARR ? ints.size() + floats.size() + strings.size() + nested.size() : 0; }
};

struct Tensor {
  std::string name;
  int type = 0, n_dims = 0;
  int64_t ne[4] = {1, 1, 1, 1};
  uint64_t nbytes = 0, offset = 0;
  int split = 0;
};

struct File {
  std::string path;
  int fd = -1;
  uint64_t size = 0, data_off = 0;
};

// Reads len bytes at file offset off; returns how many arrived (fewer only at the end of the file) or -1 on an error.
long long read_at(int fd, void* dst, size_t len, uint64_t off) {
  char* out = (char*)dst;
  size_t left = len;
  for (;;) {
    if (left == 0) return (long long)len;
    const ssize_t r = pread(fd, out, left, (off_t)off);
    if (r > 0) { out += r; off += (uint64_t)r; left -= (size_t)r; continue; }
    if (r == 0) return (long long)(len - left);
    if (errno != EINTR) return -1;
  }
}

// Sequential reader over a file descriptor with a refillable window (headers of real models run to tens of MB of
// tokenizer strings; tensor data is never read through it).
struct Reader {
  int fd;
  uint64_t pos = 0, size;
  std::vector<uint8_t> buf;
  uint64_t buf_off = 0;
  bool ok = true;
  Reader(int fd_, uint64_t size_) : fd(fd_), size(size_) {}
  bool fill(size_t need) {
    if (pos >= buf_off && pos + need <= buf_off + buf.size()) return true;
    if (pos + need > size) return ok = false;
    const size_t want = (size_t)std::min<uint64_t>(std::max<uint64_t>(need, 1u << 20), size - pos);
    buf.resize(want);
    buf_off = pos;
    if (read_at(fd, buf.data(), want, pos) != (long long)want) return ok = false;
    return true;
  }
  template <class T>
  T get() {
    T v{};
    if (!ok || !fill(sizeof(T))) return v;
    memcpy(&v, buf.data() + (pos - buf_off), sizeof(T));
    pos += sizeof(T);
    return v;
  }
  std::string str() {
    const uint64_t n = get<uint64_t>();
    if (!ok || n > size - pos || !fill((size_t)n)) { ok = false; return {}; }
    std::string s((const char*)buf.data() + (pos - buf_off), (size_t)n);
    pos += n;
    return s;
  }
};

bool read_scalar(Reader& r, uint32_t t, Value& v) {
  switch (t) {
    case U8: v.i = r.get<uint8_t>(); break;
    case I8: v.i = r.get<int8_t>(); break;
    case U16: v.i = r.get<uint16_t>(); break;
    case I16: v.i = r.get<int16_t>(); break;
    case U32: v.i = r.get<uint32_t>(); break;
    case I32: v.i = r.get<int32_t>(); break;
    case BOOL: v.i = r.get<uint8_t>() != 0; break;
    case U64: v.i = (int64_t)r.get<uint64_t>(); break;
    case I64: v.i = r.get<int64_t>(); break;
    case F32: v.f = r.get<float>(); break;
    case F64: v.f = r.get<double>(); break;
    case STR: v.s = r.str(); break;
    default: return false;
  }
  if (t != F32 && t != F64 && t != STR) v.f = (double)v.i;  // integers are mirrored into f, as the reference does
  return r.ok;
}

bool read_value(Reader& r, uint32_t t, Value& v, int depth) {
  v.type = t;
  if (t != ARR) return read_scalar(r, t, v);
  if (depth > 4) return false;
  v.arr_type = r.get<uint32_t>();
  const uint64_t n = r.get<uint64_t>();
  if (!r.ok || n > r.size) return false;
  for (uint64_t k = 0; k < n; k++) {
    Value e;
    if (!read_value(r, v.arr_type, e, depth + 1)) return false;
    if (v.arr_type == ARR) v.nested.push_back(std::move(e));
    else if (v.arr_type == STR) v.strings.push_back(std::move(e.s));
    else if (v.arr_type == F32 || v.arr_type == F64) v.floats.push_back(e.f);
    else v.ints.push_back(e.i);
  }
  return true;
}

// "*-0000N-of-0000M.gguf" -> all M split paths; anything else -> the path itself (src/gguf/gguf.hpp:60)
std::vector<std::string> expand_splits(const std::string& path) {
  const size_t n = path.size();
  // suffix layout: -NNNNN-of-MMMMM.gguf (5 digits each)
  if (n >= 20 && path.compare(n - 5, 5, ".gguf") == 0 && path.compare(n - 14, 4, "-of-") == 0 && path[n - 20] == '-') {
    bool digits = true;
    for (size_t k = 0; k < 5; k++) digits = digits && isdigit((unsigned char)path[n - 19 + k]) && isdigit((unsigned char)path[n - 10 + k]);
    if (digits) {
      const int m = atoi(path.substr(n - 10, 5).c_str());
      if (m >= 1 && m < 100000) {
        std::vector<std::string> out;
        for (int k = 1; k <= m; k++) {
          char num[8];
          snprintf(num, sizeof num, "%05d", k);
          out.push_back(path.substr(0, n - 19) + num + path.substr(n - 14));
        }
        return out;
      }
    }
  }
  return {path};
}

}  // namespace
}  // namespace msq

using namespace msq;

struct MsqGguf {
  std::vector<File> files;
  std::unordered_map<std::string, Value> kv;
  std::vector<std::string> kv_order;
  std::vector<Tensor> tensors;
  std::unordered_map<std::string, size_t> tindex;
  uint32_t align = 32, version = 0;
  std::string err;

  ~MsqGguf() {
    for (File& f : files)
      if (f.fd >= 0) close(f.fd);
  }
  bool parse(int split) {
    File& f = files[split];
    f.fd = open(f.path.c_str(), O_RDONLY);
    if (f.fd < 0) { err = "cannot open " + f.path; return false; }
    struct stat st;
    if (fstat(f.fd, &st) != 0) { err = "cannot stat " + f.path; return false; }
    f.size = (uint64_t)st.st_size;
    Reader r(f.fd, f.size);
    const uint32_t magic = r.get<uint32_t>();
    const uint32_t ver = r.get<uint32_t>();
    if (!r.ok || magic != 0x46554747u) { err = f.path + ": not a GGUF file"; return false; }
    if (ver < 2 || ver > 3) { err = f.path + ": unsupported GGUF version " + std::to_string(ver); return false; }
    if (split == 0) version = ver;
    const uint64_t nt = r.get<uint64_t>(), nkv = r.get<uint64_t>();
    if (!r.ok || nt > f.size || nkv > f.size) { err = f.path + ": bad header counts"; return false; }
    uint32_t file_align = 32;
    for (uint64_t k = 0; k < nkv; k++) {
      std::string key = r.str();
      const uint32_t t = r.get<uint32_t>();
      Value v;
      if (!r.ok || !read_value(r, t, v, 0)) { err = f.path + ": bad metadata value for key '" + key + "'"; return false; }
      if (key == "general.alignment") {
        if (v.i < 1 || v.i > (1 << 20) || (v.i & (v.i - 1))) { err = f.path + ": general.alignment is not a power of two between 1 and 2^20"; return false; }
        file_align = (uint32_t)v.i;
      }
      if (!kv.count(key)) {  // merged across splits: the first occurrence wins
        kv_order.push_back(key);
        kv.emplace(std::move(key), std::move(v));
      }
    }
    if (split == 0) align = file_align;
    const size_t first = tensors.size();
    for (uint64_t k = 0; k < nt; k++) {
      Tensor t;
      t.name = r.str();
      t.n_dims = (int)r.get<uint32_t>();
      if (!r.ok || t.n_dims < 0 || t.n_dims > 4) { err = f.path + ": bad tensor table"; return false; }
      for (int d = 0; d < t.n_dims; d++) t.ne[d] = (int64_t)r.get<uint64_t>();
      t.type = (int)r.get<uint32_t>();
      t.offset = r.get<uint64_t>();
      t.split = split;
      if (!r.ok) { err = f.path + ": truncated tensor table"; return false; }
      const TypeRow* row = type_row(t.type);
      uint64_t nel = 1;
      bool fits = true;
      for (int d = 0; d < 4; d++) {
        if (t.ne[d] < 0 || (t.ne[d] > 0 && nel > (UINT64_MAX / 512) / (uint64_t)t.ne[d])) fits = false;  // x 292 bytes per block below
        else nel *= (uint64_t)t.ne[d];
      }
      if (!fits) { err = f.path + ": tensor '" + t.name + "' has dimensions whose product overflows"; return false; }
      if (!row || t.ne[0] % row->blck) { err = f.path + ": tensor '" + t.name + "' has an unknown type or a ragged row"; return false; }
      t.nbytes = nel / row->blck * row->bytes;
      tensors.push_back(std::move(t));
    }
    f.data_off = (r.pos + file_align - 1) / file_align * file_align;
    for (size_t k = first; k < tensors.size(); k++) {
      Tensor& t = tensors[k];
      if (t.offset > f.size) { err = f.path + ": tensor '" + t.name + "' runs past the end of the file"; return false; }
      t.offset += f.data_off;  // absolute in its split
      if (t.offset > f.size || t.nbytes > f.size - t.offset) { err = f.path + ": tensor '" + t.name + "' runs past the end of the file"; return false; }
      tindex.emplace(t.name, k);
    }
    return true;
  }
  const Value* find_kv(const char* key) const {
    auto it = kv.find(key);
    return it == kv.end() ? nullptr : &it->second;
  }
};

namespace {
const Tensor* tensor_at(const MsqGguf* g, int i) { return g && i >= 0 && (size_t)i < g->tensors.size() ? &g->tensors[i] : nullptr; }

// file range -> device memory through two pinned staging buffers (the pread of one chunk overlaps the copy of the other)
int copy_file_to_device(hipStream_t st, int fd, uint64_t off, uint64_t len, uint8_t* dst) {
  constexpr size_t kChunk = 8u << 20;
  static thread_local void* stage[2] = {nullptr, nullptr};
  hipEvent_t done[2] = {nullptr, nullptr};
  for (int k = 0; k < 2; k++) {
    if (!stage[k]) MSQ_HIP(hipHostMalloc(&stage[k], kChunk, hipHostMallocDefault));
    MSQ_HIP(hipEventCreateWithFlags(&done[k], hipEventDisableTiming));
  }
  int rc = MSQ_OK;
  uint64_t pos = 0;
  for (int k = 0; pos < len && rc == MSQ_OK; k ^= 1) {
    const size_t n = (size_t)std::min<uint64_t>(kChunk, len - pos);
    if (hipEventSynchronize(done[k]) != hipSuccess) rc = fail(MSQ_ERR_HIP, "macseek quant: gguf: hipEventSynchronize failed");
    else if (read_at(fd, stage[k], n, off + pos) != (long long)n) rc = fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf: short read at offset %llu", (unsigned long long)(off + pos));
    else if (hipMemcpyAsync(dst + pos, stage[k], n, hipMemcpyHostToDevice, st) != hipSuccess || hipEventRecord(done[k], st) != hipSuccess)
      rc = fail(MSQ_ERR_HIP, "macseek quant: gguf: host to device copy failed");
    pos += n;
  }
  // the staging buffers are reused by the next call: wait for the copies that read them
  for (int k = 0; k < 2; k++) {
    if (hipEventSynchronize(done[k]) != hipSuccess && rc == MSQ_OK) rc = fail(MSQ_ERR_HIP, "macseek quant: gguf: hipEventSynchronize failed");
    hipEventDestroy(done[k]);
  }
  return rc;
}

constexpr uint64_t kPlaceAlign = 256;
uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }
const char* const kExpertNames[3] = {"ffn_gate_exps", "ffn_up_exps", "ffn_down_exps"};

// the three stacked expert tensors of a layer (blk.L.ffn_{gate,up,down}_exps.weight: [cols, rows, n_experts])
int expert_tensors(const MsqGguf* g, int layer, const Tensor* out[3], int64_t* n_exp) {
  if (!g) return fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf: null handle");
  for (int k = 0; k < 3; k++) {
    const std::string name = "blk." + std::to_string(layer) + "." + kExpertNames[k] + ".weight";
    auto it = g->tindex.find(name);
    if (it == g->tindex.end()) return fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf: tensor %s is missing", name.c_str());
    out[k] = &g->tensors[it->second];
    const int64_t e = out[k]->ne[2];
    if (out[k]->n_dims != 3 || e < 1 || out[k]->nbytes % (uint64_t)e || (k && e != *n_exp))
      return fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf: bad expert tensor %s", name.c_str());  // reference: experts.mm:46
    *n_exp = e;
  }
  return MSQ_OK;
}
}  // namespace

extern "C" {

int msq_gguf_open(const char* path, MsqGguf** out) {
  if (!path || !out) return fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf_open: null argument");
  *out = nullptr;
  MsqGguf* g = new MsqGguf();
  for (const std::string& p : expand_splits(path)) g->files.push_back(File{p});
  for (size_t s = 0; s < g->files.size(); s++)
    if (!g->parse((int)s)) {
      const int rc = fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf_open: %s", g->err.c_str());
      delete g;
      return rc;
    }
  *out = g;
  return MSQ_OK;
}
void msq_gguf_close(MsqGguf* g) { delete g; }

int msq_gguf_n_splits(const MsqGguf* g) { return g ? (int)g->files.size() : 0; }
int msq_gguf_n_tensors(const MsqGguf* g) { return g ? (int)g->tensors.size() : 0; }
int msq_gguf_n_kv(const MsqGguf* g) { return g ? (int)g->kv_order.size() : 0; }
uint32_t msq_gguf_alignment(const MsqGguf* g) { return g ? g->align : 0; }
uint32_t msq_gguf_version(const MsqGguf* g) { return g ? g->version : 0; }
const char* msq_gguf_split_path(const MsqGguf* g, int split) { return g && split >= 0 && (size_t)split < g->files.size() ? g->files[split].path.c_str() : nullptr; }
uint64_t msq_gguf_data_offset(const MsqGguf* g, int split) { return g && split >= 0 && (size_t)split < g->files.size() ? g->files[split].data_off : 0; }
int msq_gguf_split_count_of_path(const char* path) { return path ? (int)expand_splits(path).size() : 0; }

uint64_t msq_gguf_type_bytes(int type, uint64_t n_elems) {
  const TypeRow* r = type_row(type);
  return r ? n_elems / r->blck * r->bytes : 0;
}
const char* msq_gguf_type_name(int type) {
  const TypeRow* r = type_row(type);
  return r ? r->name : "?";
}

int msq_gguf_tensor(const MsqGguf* g, int index, MsqGgufTensor* out) {
  const Tensor* t = tensor_at(g, index);
  if (!t || !out) return fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf_tensor: index %d out of range", index);
  out->name = t->name.c_str();
  out->type = t->type;
  out->n_dims = t->n_dims;
  for (int d = 0; d < 4; d++) out->ne[d] = t->ne[d];
  out->nbytes = t->nbytes;
  out->split = t->split;
  out->offset = t->offset;
  return MSQ_OK;
}
int msq_gguf_find(const MsqGguf* g, const char* name) {
  if (!g || !name) return -1;
  auto it = g->tindex.find(name);
  return it == g->tindex.end() ? -1 : (int)it->second;
}

const char* msq_gguf_key(const MsqGguf* g, int index) { return g && index >= 0 && (size_t)index < g->kv_order.size() ? g->kv_order[index].c_str() : nullptr; }
int msq_gguf_kv_type(const MsqGguf* g, const char* key, int* arr_type) {
  const Value* v = g && key ? g->find_kv(key) : nullptr;
  if (!v) return -1;
  if (arr_type) *arr_type = v->type == ARR ? (int)v->arr_type : -1;
  return (int)v->type;
}
int64_t msq_gguf_get_i64(const MsqGguf* g, const char* key, int64_t dflt) {
  const Value* v = g && key ? g->find_kv(key) : nullptr;
  if (!v || v->type == STR || v->type == ARR) return dflt;
  return (v->type == F32 || v->type == F64) ? (int64_t)v->f : v->i;
}
double msq_gguf_get_f64(const MsqGguf* g, const char* key, double dflt) {
  const Value* v = g && key ? g->find_kv(key) : nullptr;
  return (!v || v->type == STR || v->type == ARR) ? dflt : v->f;
}
const char* msq_gguf_get_str(const MsqGguf* g, const char* key, const char* dflt) {
  const Value* v = g && key ? g->find_kv(key) : nullptr;
  return v && v->type == STR ? v->s.c_str() : dflt;
}
int64_t msq_gguf_arr_len(const MsqGguf* g, const char* key) {
  const Value* v = g && key ? g->find_kv(key) : nullptr;
  return v && v->type == ARR ? (int64_t)v->size() : -1;
}
int64_t msq_gguf_arr_i64(const MsqGguf* g, const char* key, int64_t* out, int64_t cap) {
  const Value* v = g && key ? g->find_kv(key) : nullptr;
  if (!v || v->type != ARR) return -1;
  int64_t n = 0;
  if (!v->ints.empty()) { for (; n < (int64_t)v->ints.size() && n < cap; n++) out[n] = v->ints[n]; }
  else { for (; n < (int64_t)v->floats.size() && n < cap; n++) out[n] = (int64_t)v->floats[n]; }
  return n;
}
int64_t msq_gguf_arr_f64(const MsqGguf* g, const char* key, double* out, int64_t cap) {
  const Value* v = g && key ? g->find_kv(key) : nullptr;
  if (!v || v->type != ARR) return -1;
  int64_t n = 0;
  if (!v->floats.empty()) { for (; n < (int64_t)v->floats.size() && n < cap; n++) out[n] = v->floats[n]; }
  else { for (; n < (int64_t)v->ints.size() && n < cap; n++) out[n] = (double)v->ints[n]; }
  return n;
}
const char* msq_gguf_arr_str(const MsqGguf* g, const char* key, int64_t index) {
  const Value* v = g && key ? g->find_kv(key) : nullptr;
  return v && v->type == ARR && index >= 0 && (size_t)index < v->strings.size() ? v->strings[(size_t)index].c_str() : nullptr;
}
// element `index` of a nested array (an array of arrays of integers): its length, and up to cap values
int64_t msq_gguf_arr_nested_i64(const MsqGguf* g, const char* key, int64_t index, int64_t* out, int64_t cap) {
  const Value* v = g && key ? g->find_kv(key) : nullptr;
  if (!v || v->type != ARR || index < 0 || (size_t)index >= v->nested.size()) return -1;
  const Value& e = v->nested[(size_t)index];
  int64_t n = 0;
  for (; n < (int64_t)e.ints.size() && n < cap; n++) out[n] = e.ints[n];
  return (int64_t)e.ints.size();
}

int64_t msq_gguf_read(const MsqGguf* g, int tensor, uint64_t byte_off, void* dst, uint64_t len) {
  const Tensor* t = tensor_at(g, tensor);
  if (!t || !dst || byte_off > t->nbytes || len > t->nbytes - byte_off) {
    fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf_read: bad tensor index or range");
    return -1;
  }
  return read_at(g->files[t->split].fd, dst, (size_t)len, t->offset + byte_off);
}

int msq_gguf_load_tensor(void* stream, const MsqGguf* g, int tensor, uint64_t byte_off, uint64_t len, const MsqBuffer* dst) {
  const Tensor* t = tensor_at(g, tensor);
  if (!t || byte_off > t->nbytes || len > t->nbytes - byte_off) return fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf_load_tensor: bad tensor index or range");
  if (len == 0) return MSQ_OK;
  if (!buf_ok(dst, len)) return fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf_load_tensor: destination missing or too small");
  return copy_file_to_device((hipStream_t)stream, g->files[t->split].fd, t->offset + byte_off, len, bptr_mut(dst));
}

int msq_gguf_expert_layout(const MsqGguf* g, int layer, MsqExpertLayout* out) {
  const Tensor* t[3];
  int64_t ne = 0;
  const int rc = expert_tensors(g, layer, t, &ne);
  if (rc != MSQ_OK) return rc;
  if (!out) return fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf_expert_layout: null output");
  out->n_experts = (int)ne;
  uint64_t per_expert = 0;
  for (int k = 0; k < 3; k++) {
    out->type[k] = t[k]->type;
    out->cols[k] = t[k]->ne[0];
    out->rows[k] = t[k]->ne[1];
    out->stride[k] = t[k]->nbytes / (uint64_t)ne;  // the per-expert slab (reference: experts.mm:49)
    out->tensor[k] = (int)(t[k] - g->tensors.data());
    per_expert += align_up(out->stride[k], kPlaceAlign);
  }
  out->arena_bytes = per_expert * (uint64_t)ne;
  return MSQ_OK;
}

int msq_gguf_place_experts(void* stream, const MsqGguf* g, int layer, const MsqBuffer* arena, MsqExpertSlot* slots, int n_slots) {
  MsqExpertLayout L;
  const int rc = msq_gguf_expert_layout(g, layer, &L);
  if (rc != MSQ_OK) return rc;
  if (!slots || n_slots < L.n_experts) return fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf_place_experts: %d slots for %d experts", n_slots, L.n_experts);
  if (!buf_ok(arena, L.arena_bytes) || ((uintptr_t)bptr(arena) % kPlaceAlign))
    return fail(MSQ_ERR_ARGUMENT, "macseek quant: gguf_place_experts: arena missing, smaller than %llu bytes or not 256-byte aligned",
                (unsigned long long)L.arena_bytes);
  // matrix-major: all gate slabs, then up, then down; every slab at a 256-byte aligned offset. A slab whose length is a
  // multiple of 256 makes the tensor one contiguous copy.
  uint64_t base = 0;
  for (int k = 0; k < 3; k++) {
    const uint64_t pitch = align_up(L.stride[k], kPlaceAlign);
    const Tensor& t = g->tensors[L.tensor[k]];
    if (pitch == L.stride[k]) {
      const int rcc = copy_file_to_device((hipStream_t)stream, g->files[t.split].fd, t.offset, t.nbytes, bptr_mut(arena) + base);
      if (rcc != MSQ_OK) return rcc;
    }
    for (int e = 0; e < L.n_experts; e++) {
      const uint64_t off = base + pitch * (uint64_t)e;
      if (pitch != L.stride[k]) {
        const int rcc = copy_file_to_device((hipStream_t)stream, g->files[t.split].fd, t.offset + L.stride[k] * (uint64_t)e, L.stride[k], bptr_mut(arena) + off);
        if (rcc != MSQ_OK) return rcc;
      }
      MsqBuffer* b = k == 0 ? &slots[e].gate : k == 1 ? &slots[e].up : &slots[e].down;
      *b = MsqBuffer{arena->dev, arena->off + off, L.stride[k]};
    }
    base += pitch * (uint64_t)L.n_experts;
  }
  return MSQ_OK;
}

}  // extern "C"
