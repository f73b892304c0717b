// GGUF reader of include/arcz_gguf.h: POSIX mmap, one pass over the header with a bounds-checked cursor.
#include "../../include/arcz_gguf.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace {
std::string g_gguf_err;

struct Tensor {
  std::string name;
  uint32_t type = 0, ndim = 0;
  uint64_t dims[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  uint64_t offset = 0, nbytes = 0;
};
struct Value {
  enum Kind { INT, BOOL, FLOAT, STRING, OTHER } kind = OTHER;  // (BOOL: an integer to get_int, nothing to get_float, as src/gguf.h:151-166)
  int64_t i = 0;
  double f = 0.0;
  std::string s;
};
}  // namespace

struct arcz_gguf {
  int fd = -1;
  const uint8_t* base = nullptr;
  uint64_t size = 0, pos = 0, data_start = 0, align = 32;
  uint32_t version = 0;
  uint64_t n_kv = 0;
  std::unordered_map<std::string, Value> kv;
  std::vector<Tensor> tensors;
  std::unordered_map<std::string, size_t> index;

  ~arcz_gguf() {
    if (base) munmap((void*)base, size);
    if (fd >= 0) close(fd);
  }
  void need(uint64_t n) const {
    if (n > size - pos) throw std::runtime_error("truncated (a field of " + std::to_string(n) + " bytes at offset " + std::to_string(pos) + ")");
  }
  template <class T> T rd() {
    need(sizeof(T));
    T v;
    memcpy(&v, base + pos, sizeof(T));
    pos += sizeof(T);
    return v;
  }
  std::string rd_str() {
    const uint64_t n = rd<uint64_t>();
    need(n);
    std::string s((const char*)base + pos, (size_t)n);
    pos += n;
    return s;
  }
  static int scalar_size(uint32_t t) {
    switch (t) {
      case 0: case 1: case 7: return 1;
      case 2: case 3: return 2;
      case 4: case 5: case 6: return 4;
      case 10: case 11: case 12: return 8;
      default: return 0;
    }
  }
  Value rd_value(uint32_t t, int depth) {
    Value v;
    switch (t) {
      case 0: v.kind = Value::INT; v.i = rd<uint8_t>(); break;
      case 1: v.kind = Value::INT; v.i = rd<int8_t>(); break;
      case 2: v.kind = Value::INT; v.i = rd<uint16_t>(); break;
      case 3: v.kind = Value::INT; v.i = rd<int16_t>(); break;
      case 4: v.kind = Value::INT; v.i = rd<uint32_t>(); break;
      case 5: v.kind = Value::INT; v.i = rd<int32_t>(); break;
      case 6: v.kind = Value::FLOAT; v.f = rd<float>(); break;
      case 7: v.kind = Value::BOOL; v.i = rd<uint8_t>() != 0; break;
      case 8: v.kind = Value::STRING; v.s = rd_str(); break;
      case 10: v.kind = Value::INT; v.i = (int64_t)rd<uint64_t>(); break;
      case 11: v.kind = Value::INT; v.i = rd<int64_t>(); break;
      case 12: v.kind = Value::FLOAT; v.f = rd<double>(); break;
      case 9: {  // an array: skipped, element by element where the elements have no fixed size
        if (depth > 4) throw std::runtime_error("metadata arrays nested too deep");
        const uint32_t et = rd<uint32_t>();
        const uint64_t n = rd<uint64_t>();
        const int es = scalar_size(et);
        if (es) {
          if (n > (size - pos) / (uint64_t)es) throw std::runtime_error("truncated (array of " + std::to_string(n) + " elements)");
          pos += n * (uint64_t)es;
        } else {
          if (n > size - pos) throw std::runtime_error("truncated (array of " + std::to_string(n) + " elements)");
          for (uint64_t i = 0; i < n; ++i) rd_value(et, depth + 1);
        }
        break;
      }
      default: throw std::runtime_error("unknown metadata type " + std::to_string(t));
    }
    return v;
  }
  void parse() {
    if (rd<uint32_t>() != 0x46554747u) throw std::runtime_error("not a GGUF file");
    version = rd<uint32_t>();
    if (version < 2) throw std::runtime_error("unsupported GGUF version " + std::to_string(version));
    const uint64_t nt = rd<uint64_t>();
    n_kv = rd<uint64_t>();
    // (a key-value pair takes at least 12 bytes, a tensor entry 24: counts the file cannot hold are refused before
    //  anything is allocated for them; src/gguf.h:311-318)
    if (n_kv > (size - pos) / 12 || nt > (size - pos) / 24 || n_kv > 1000000 || nt > 1000000)
      throw std::runtime_error("bad tensor / key count (" + std::to_string(nt) + " / " + std::to_string(n_kv) + ")");
    for (uint64_t i = 0; i < n_kv; ++i) {
      std::string key = rd_str();
      const uint32_t t = rd<uint32_t>();
      kv[key] = rd_value(t, 0);
    }
    tensors.resize(nt);
    for (uint64_t i = 0; i < nt; ++i) {
      Tensor& t = tensors[i];
      t.name = rd_str();
      t.ndim = rd<uint32_t>();
      if (t.ndim > 8) throw std::runtime_error("bad dimension count for " + t.name);
      for (uint32_t d = 0; d < t.ndim; ++d) t.dims[d] = rd<uint64_t>();
      t.type = rd<uint32_t>();
      t.offset = rd<uint64_t>();
      index[t.name] = i;
    }
    auto it = kv.find("general.alignment");
    const int64_t a = it != kv.end() && (it->second.kind == Value::INT || it->second.kind == Value::BOOL) ? it->second.i : 32;
    if (a <= 0 || a > (1 << 20) || (a & (a - 1))) throw std::runtime_error("bad alignment " + std::to_string(a));
    align = (uint64_t)a;
    data_start = (pos + align - 1) / align * align;
    if (nt > 0 && data_start > size) throw std::runtime_error("truncated (no tensor data)");
    for (Tensor& t : tensors) {
      int blk = 0, bytes = 0;
      if (!arcz_ggml_block_info(t.type, &blk, &bytes)) throw std::runtime_error("unsupported ggml type " + std::to_string(t.type) + " (" + t.name + ")");
      uint64_t n = 1;
      for (uint32_t d = 0; d < t.ndim; ++d) {
        if (t.dims[d] != 0 && n > UINT64_MAX / t.dims[d]) throw std::runtime_error("tensor too large: " + t.name);
        n *= t.dims[d];
      }
      if (t.ndim == 0 || t.dims[0] % (uint64_t)blk) throw std::runtime_error("row length of " + t.name + " is no multiple of its block");
      if (n / (uint64_t)blk > UINT64_MAX / (uint64_t)bytes) throw std::runtime_error("tensor too large: " + t.name);
      t.nbytes = n / (uint64_t)blk * (uint64_t)bytes;
      if (t.offset > size - data_start || t.nbytes > size - data_start - t.offset) throw std::runtime_error("tensor out of range: " + t.name);
    }
  }
};

extern "C" {

int arcz_ggml_block_info(uint32_t type, int* blk, int* bytes) {
  int b = 0, n = 0;
  switch (type) {
    case 0: b = 1; n = 4; break;                    // F32
    case 1: case 30: case 25: b = 1; n = 2; break;  // F16, BF16, I16
    case 24: b = 1; n = 1; break;                   // I8
    case 26: b = 1; n = 4; break;                   // I32
    case 2: b = 32; n = 18; break;                  // Q4_0
    case 3: b = 32; n = 20; break;                  // Q4_1
    case 6: b = 32; n = 22; break;                  // Q5_0
    case 7: b = 32; n = 24; break;                  // Q5_1
    case 8: b = 32; n = 34; break;                  // Q8_0
    case 10: b = 256; n = 84; break;                // Q2_K
    case 11: b = 256; n = 110; break;               // Q3_K
    case 12: b = 256; n = 144; break;               // Q4_K
    case 13: b = 256; n = 176; break;               // Q5_K
    case 14: b = 256; n = 210; break;               // Q6_K
    case 20: b = 32; n = 18; break;                 // IQ4_NL
    case 21: b = 256; n = 110; break;               // IQ3_S
    case 23: b = 256; n = 136; break;               // IQ4_XS
    // types the matmul path does not take (make_weight refuses them) but a model file may hold: sized, so that the
    // directory of such a file still parses
    case 16: b = 256; n = 66; break;                // IQ2_XXS
    case 17: b = 256; n = 74; break;                // IQ2_XS
    case 22: b = 256; n = 82; break;                // IQ2_S
    case 18: b = 256; n = 98; break;                // IQ3_XXS
    case 19: b = 256; n = 50; break;                // IQ1_S
    case 29: b = 256; n = 56; break;                // IQ1_M
    case 39: b = 32; n = 17; break;                 // MXFP4
    case 43: b = 32; n = 33; break;                 // MXFP8
    case 42: b = 64; n = 18; break;                 // Q2_0
    case 0x41523447u: b = 128; n = 66; break;       // AR4_128
    default: return 0;
  }
  if (blk) *blk = b;
  if (bytes) *bytes = n;
  return 1;
}

const char* arcz_gguf_error(void) { return g_gguf_err.c_str(); }

arcz_gguf* arcz_gguf_open(const char* path) {
  arcz_gguf* g = new arcz_gguf();
  try {
    g->fd = open(path, O_RDONLY);
    if (g->fd < 0) throw std::runtime_error("cannot open the file");
    struct stat st;
    if (fstat(g->fd, &st) != 0 || st.st_size <= 0) throw std::runtime_error("cannot read the file's size");
    g->size = (uint64_t)st.st_size;
    void* p = mmap(nullptr, g->size, PROT_READ, MAP_PRIVATE, g->fd, 0);
    if (p == MAP_FAILED) throw std::runtime_error("mmap failed");
    g->base = (const uint8_t*)p;
    g->parse();
  } catch (const std::exception& ex) {
    g_gguf_err = std::string("gguf: ") + (path ? path : "(null)") + ": " + ex.what();
    delete g;
    return nullptr;
  }
  return g;
}
void arcz_gguf_close(arcz_gguf* g) { delete g; }

uint32_t arcz_gguf_version(const arcz_gguf* g) { return g->version; }
size_t arcz_gguf_n_kv(const arcz_gguf* g) { return (size_t)g->n_kv; }
size_t arcz_gguf_n_tensors(const arcz_gguf* g) { return g->tensors.size(); }
uint64_t arcz_gguf_alignment(const arcz_gguf* g) { return g->align; }

int arcz_gguf_kv_i64(const arcz_gguf* g, const char* key, int64_t* out) {
  auto it = g->kv.find(key);
  if (it == g->kv.end() || (it->second.kind != Value::INT && it->second.kind != Value::BOOL)) return 0;
  if (out) *out = it->second.i;
  return 1;
}
int arcz_gguf_kv_f64(const arcz_gguf* g, const char* key, double* out) {
  auto it = g->kv.find(key);
  if (it == g->kv.end() || (it->second.kind != Value::INT && it->second.kind != Value::FLOAT)) return 0;
  if (out) *out = it->second.kind == Value::INT ? (double)it->second.i : it->second.f;
  return 1;
}
const char* arcz_gguf_kv_str(const arcz_gguf* g, const char* key) {
  auto it = g->kv.find(key);
  return it == g->kv.end() || it->second.kind != Value::STRING ? nullptr : it->second.s.c_str();
}

int arcz_gguf_tensor(const arcz_gguf* g, size_t i, const char** name, uint32_t* type, uint32_t* ndim, uint64_t dims[8],
                     const void** data, uint64_t* nbytes) {
  if (i >= g->tensors.size()) return -1;
  const Tensor& t = g->tensors[i];
  if (name) *name = t.name.c_str();
  if (type) *type = t.type;
  if (ndim) *ndim = t.ndim;
  if (dims) memcpy(dims, t.dims, sizeof(t.dims));
  if (data) *data = g->base + g->data_start + t.offset;
  if (nbytes) *nbytes = t.nbytes;
  return 0;
}
long arcz_gguf_find(const arcz_gguf* g, const char* name) {
  auto it = g->index.find(name);
  return it == g->index.end() ? -1 : (long)it->second;
}

}  // extern "C"
