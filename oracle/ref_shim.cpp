// Thin extern "C" window onto the reference's own CPU code (src/quants.h), compiled from the reference tree where it
// lies (see oracle/Makefile: -I$(REF)).  TEST INFRASTRUCTURE ONLY: it exists to validate oracle/arcz_oracle.c and,
// optionally, to time the reference's CPU path; the output goes to oracle/_ref/ and is never committed.
// Nothing of the reference is copied here: every function below only forwards to the header's functions.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <variant>
#include <vector>
#include "src/gguf.h"
#include "src/quants.h"

extern "C" {
float ref_fp16_to_f32(uint16_t h) { return fp16_to_f32(h); }
uint16_t ref_f32_to_fp16(float x) { return f32_to_fp16(x); }
int ref_sb_bytes(uint32_t type) { return gguf_sb_bytes(type); }
int ref_dequant_row(uint32_t type, const uint8_t* row, int K, float* out) {
  try { dequant_row(type, row, K, out); } catch (...) { return -1; }
  return 0;
}
// q[256], sc[8], mn[8], sc6[16], d8[8], d, dmin of one superblock
int ref_decode_sb(uint32_t type, const uint8_t* p, int16_t* q, int32_t* sc, int32_t* mn, int32_t* sc6, float* d8,
                  float* d, float* dmin) {
  DecodedSB o;
  try { decode_sb(type, p, o); } catch (...) { return -1; }
  for (int i = 0; i < 256; ++i) q[i] = o.q[i];
  for (int i = 0; i < 8; ++i) { sc[i] = o.sc[i]; mn[i] = o.mn[i]; d8[i] = o.d8[i]; }
  for (int i = 0; i < 16; ++i) sc6[i] = o.sc6[i];
  *d = o.d;
  *dmin = o.dmin;
  return 0;
}
void ref_quantize_act_cpu(const float* x, int M, int K, int8_t* aq, float* asc, uint16_t* absum, int act32) {
  quantize_act_cpu(x, M, K, aq, asc, absum, act32 != 0);
}
void ref_quantize_rows_q8_0(const float* src, int N, int K, uint8_t* out) {
  const std::vector<uint8_t> v = quantize_rows_q8_0(src, N, K);
  memcpy(out, v.data(), v.size());
}
void ref_quantize_rows_q4_0(const float* src, int N, int K, uint8_t* out) {
  const std::vector<uint8_t> v = quantize_rows_q4_0(src, N, K);
  memcpy(out, v.data(), v.size());
}
// the reference's GPU raw form of one superblock (src/quants.h gpu_raw_sb), to compare layouts in tests
int ref_raw_padded_sb_bytes(uint32_t type) { return raw_padded_sb_bytes(type); }
void ref_gpu_raw_sb(uint32_t type, const uint8_t* src, uint8_t* dst) { gpu_raw_sb(type, src, dst); }
// the reference's GGUF reader (GgufFile, src/gguf.h:93-361), to pin the library's own reader on the same files
static std::string g_ref_gguf_err;
const char* ref_gguf_error(void) { return g_ref_gguf_err.c_str(); }
void* ref_gguf_open(const char* path) {
  try {
    return new GgufFile(path);
  } catch (const std::exception& e) {
    g_ref_gguf_err = e.what();
  } catch (...) {
    g_ref_gguf_err = "unknown exception";
  }
  return nullptr;
}
void ref_gguf_close(void* g) { delete (GgufFile*)g; }
int64_t ref_gguf_n_tensors(void* g) { return (int64_t)((GgufFile*)g)->tensors.size(); }
int64_t ref_gguf_n_kv(void* g) { return (int64_t)((GgufFile*)g)->kv.size(); }
// entry i of the directory; name into name[cap]; data: the mapped address of the tensor's first byte
int ref_gguf_tensor(void* g, int64_t i, char* name, int cap, uint32_t* type, uint32_t* ndim, uint64_t* dims,
                    const uint8_t** data, uint64_t* nbytes) {
  const GgufFile* f = (const GgufFile*)g;
  if (i < 0 || (size_t)i >= f->tensors.size()) return -1;
  const GgufTensor& t = f->tensors[(size_t)i];
  snprintf(name, (size_t)cap, "%s", t.name.c_str());
  *type = t.type;
  *ndim = (uint32_t)t.dims.size();
  for (size_t d = 0; d < t.dims.size() && d < 8; ++d) dims[d] = t.dims[d];
  *data = t.data;
  *nbytes = t.nbytes;
  return 0;
}
int64_t ref_gguf_find(void* g, const char* name) {
  const GgufFile* f = (const GgufFile*)g;
  auto it = f->tensor_index.find(name);
  return it == f->tensor_index.end() ? -1 : (int64_t)it->second;
}
int ref_gguf_has(void* g, const char* key) { return ((GgufFile*)g)->has(key) ? 1 : 0; }
int64_t ref_gguf_get_int(void* g, const char* key, int64_t def) { return ((GgufFile*)g)->get_int(key, def); }
double ref_gguf_get_float(void* g, const char* key, double def) { return ((GgufFile*)g)->get_float(key, def); }
int ref_gguf_get_str(void* g, const char* key, char* out, int cap) {
  const GgufFile* f = (const GgufFile*)g;
  auto it = f->kv.find(key);
  if (it == f->kv.end() || !std::get_if<std::string>(&it->second)) return 0;
  snprintf(out, (size_t)cap, "%s", f->get_str(key).c_str());
  return 1;
}
int ref_ggml_block_info(uint32_t type, int* blk, int* bytes) {
  try { ggml_block_info(type, *blk, *bytes); } catch (...) { return 0; }
  return 1;
}
}
