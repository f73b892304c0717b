// C ABI of include/arcz_engine.h over the Engine class (engine_hip.h).
#include <algorithm>
#include "../../include/arcz_engine.h"
#include "../../include/arcz_gguf.h"

#include <string>

#include "engine_hip.h"

struct arcz_engine { Engine* e; };
struct arcz_weight { GpuWeight w; };
struct arcz_moe_layer { Engine::MoeLayer L; };

namespace {
std::string g_err;
template <class F> int guarded(F&& f) {
  try {
    f();
    return ARCZ_OK;
  } catch (const std::exception& ex) {
    g_err = ex.what();
    fprintf(stderr, "arcz engine: %s\n", ex.what());
    return ARCZ_E_ENGINE;
  }
}
}  // namespace

extern "C" {

const char* arcz_engine_error(void) { return g_err.c_str(); }

arcz_engine* arcz_engine_create(int max_chunk, int max_k) {
  Engine* e = nullptr;
  if (guarded([&] { e = new Engine(max_chunk, max_k); }) != ARCZ_OK) return nullptr;
  return new arcz_engine{e};
}
void arcz_engine_destroy(arcz_engine* e) {
  if (!e) return;
  guarded([&] { delete e->e; });
  delete e;
}

arcz_weight* arcz_weight_upload(arcz_engine* e, uint32_t type, int N, int K, const void* gguf, size_t bytes) {
  arcz_weight* w = new arcz_weight;
  if (guarded([&] { w->w = e->e->make_weight(type, (const uint8_t*)gguf, bytes, N, K); }) != ARCZ_OK) {
    delete w;
    return nullptr;
  }
  return w;
}
// Engine::make_weight from a tensor of a GGUF file (zero/engine_load.h:157-196): a matrix [N][K] (dims K, N) or an expert
// tensor [NE][N][K] (dims K, N, NE), taken as it lies in the file.
static GpuWeight weight_from_gguf(Engine& E, const arcz_gguf* g, const char* name, int* ne_out) {
  const long i = arcz_gguf_find(g, name);
  if (i < 0) throw std::runtime_error(std::string("missing tensor ") + name);
  uint32_t type = 0, nd = 0;
  uint64_t dims[8], nbytes = 0;
  const void* data = nullptr;
  arcz_gguf_tensor(g, (size_t)i, nullptr, &type, &nd, dims, &data, &nbytes);
  if (nd < 2 || nd > 3 || dims[0] > (1u << 30) || dims[1] > (1u << 30) || (nd == 3 && dims[2] > 65536))
    throw std::runtime_error(std::string("tensor ") + name + " is no matrix or expert tensor");
  const int K = (int)dims[0], N = (int)dims[1], NE = nd == 3 ? (int)dims[2] : 1;
  if (ne_out) *ne_out = NE;
  return E.make_weight(type, (const uint8_t*)data, (size_t)nbytes, N, K, (size_t)NE * N);
}
arcz_weight* arcz_weight_upload_gguf(arcz_engine* e, const arcz_gguf* g, const char* name) {
  arcz_weight* w = new arcz_weight();
  if (guarded([&] { w->w = weight_from_gguf(*e->e, g, name, nullptr); }) != ARCZ_OK) {
    delete w;
    return nullptr;
  }
  return w;
}
arcz_moe_layer* arcz_moe_layer_upload_gguf(arcz_engine* e, const arcz_gguf* g, const char* gate, const char* up,
                                           const char* down, int NU) {
  arcz_moe_layer* L = new arcz_moe_layer();
  if (guarded([&] {
        int ne[3];
        Engine& E = *e->e;
        // the geometry first (the layer's buffers are sized from it), then the three tensors
        const long ig = arcz_gguf_find(g, gate);
        if (ig < 0) throw std::runtime_error(std::string("missing tensor ") + gate);
        uint32_t nd = 0;
        uint64_t dims[8];
        arcz_gguf_tensor(g, (size_t)ig, nullptr, nullptr, &nd, dims, nullptr, nullptr);
        if (nd != 3) throw std::runtime_error(std::string("tensor ") + gate + " is no expert tensor");
        if (dims[0] > (1u << 30) || dims[1] > (1u << 30) || dims[2] > 65536)  // (before they become ints)
          throw std::runtime_error(std::string("tensor ") + gate + ": dimensions out of range");
        const int Ed = (int)dims[0], F = (int)dims[1], NE = (int)dims[2];
        // the three tensors as they lie in the file: shapes checked here, rows and columns padded in make_moe_layer
        uint32_t types[3];
        const uint8_t* data[3];
        const char* names[3] = {gate, up, down};
        for (int i = 0; i < 3; ++i) {
          const long it = arcz_gguf_find(g, names[i]);
          if (it < 0) throw std::runtime_error(std::string("missing tensor ") + names[i]);
          uint32_t ndi = 0;
          uint64_t di[8], nb = 0;
          const void* p = nullptr;
          arcz_gguf_tensor(g, (size_t)it, nullptr, &types[i], &ndi, di, &p, &nb);
          const uint64_t k = i == 2 ? (uint64_t)F : (uint64_t)Ed, n = i == 2 ? (uint64_t)Ed : (uint64_t)F;
          if (ndi != 3 || di[0] != k || di[1] != n || di[2] != (uint64_t)NE)
            throw std::runtime_error("the expert tensors' shapes do not belong to one layer");
          int blk = 0, bytes = 0;
          if (!arcz_ggml_block_info(types[i], &blk, &bytes) || k % (uint64_t)blk || nb != (uint64_t)NE * n * (k / (uint64_t)blk) * (uint64_t)bytes)
            throw std::runtime_error(std::string("tensor ") + names[i] + ": its bytes do not match its shape");
          data[i] = (const uint8_t*)p;
        }
        L->L = E.make_moe_layer(types, data, NE, NU, Ed, F);
      }) != ARCZ_OK) {
    delete L;
    return nullptr;
  }
  return L;
}

int arcz_weight_free(arcz_engine* e, arcz_weight* w) {
  if (!w) return ARCZ_OK;
  const int r = guarded([&] { e->e->free_weight(w->w); });
  delete w;
  return r;
}
arcz_mem* arcz_weight_raw(const arcz_weight* w) { return w ? w->w.raw : nullptr; }
int arcz_weight_k(const arcz_weight* w) { return w ? w->w.K : 0; }
int arcz_weight_set_softcap(arcz_weight* w, float cap) {
  if (!w || !(cap >= 0.0f)) return ARCZ_E_ENGINE;
  w->w.softcap = cap;
  return ARCZ_OK;
}

int arcz_engine_quantize(arcz_engine* e, arcz_mem* x, int ldx, int K, int Mp, int T, int act32) {
  return guarded([&] { e->e->quantize_rows(x, ldx, K, Mp, T, act32); });
}
int arcz_engine_rmsnorm_quant(arcz_engine* e, arcz_mem* x, int row_off, arcz_mem* w, int K, int Mp, int T, int act32,
                              float eps, arcz_mem* hout) {
  return guarded([&] { e->e->rmsnorm_quant(x, row_off, w, K, Mp, T, act32, eps, hout); });
}
int arcz_engine_add_norm_quant(arcz_engine* e, arcz_mem* x, arcz_mem* t, arcz_mem* w, int K, int T, int Mp, float s,
                               arcz_mem* w2, int norm2, int act32, float eps) {
  return guarded([&] { e->e->add_norm_quant(x, t, w, K, T, Mp, s, w2, norm2 != 0, act32, eps); });
}
int arcz_engine_swiglu_quant(arcz_engine* e, arcz_mem* gu, int F, int Mp, int T, int act32, int fused, int gelu) {
  return guarded([&] { e->e->swiglu_quant(gu, F, Mp, T, act32, fused, gelu); });
}
int arcz_engine_set_activations(arcz_engine* e, const int8_t* aq, const float* asc, const int16_t* absum, int K, int Mp,
                                int T) {
  return guarded([&] { e->e->set_activations(aq, asc, absum, K, Mp, T); });
}
int arcz_engine_two_pass(arcz_engine* e, int on) {
  return guarded([&] {
    e->e->set_two_pass(on != 0);
    e->e->q2_nofuse_ = on == 2;
  });
}
arcz_mem* arcz_engine_residual(arcz_engine* e, int which) {
  cl_mem b[3] = {e->e->aq2_, e->e->asc2_, e->e->absum2_};
  return which >= 0 && which < 3 ? b[which] : nullptr;
}
arcz_mem* arcz_engine_aq(arcz_engine* e) { return e->e->aq_; }
arcz_mem* arcz_engine_asc(arcz_engine* e) { return e->e->asc_; }
arcz_mem* arcz_engine_absum(arcz_engine* e) { return e->e->absum_; }

int arcz_engine_matmul(arcz_engine* e, const char* name, arcz_weight* w, int Mp, arcz_mem* C, int ldc, int c_off, int acc,
                       int act32) {
  return guarded([&] {
    if (!w) throw std::runtime_error("matmul: no weight");
    e->e->matmul(name ? name : "matmul", w->w, Mp, C, ldc, c_off, acc, act32 != 0);
  });
}

int arcz_engine_gemv_gu(arcz_engine* e, arcz_weight* g, arcz_weight* u, int Mp, arcz_mem* C) {
  int taken = 0;
  const int r = guarded([&] {
    if (!g || !u) throw std::runtime_error("gemv_gu: no weight");
    taken = e->e->gemv_gu(g->w, u->w, Mp, C) ? 1 : 0;
  });
  return r != ARCZ_OK ? r : taken;
}

int arcz_engine_matmul_noalloc(arcz_engine* e, const char* name, arcz_weight* w, int Mp, arcz_mem* C, int ldc, int c_off,
                               int acc, int act32) {
  return guarded([&] {
    if (!w) throw std::runtime_error("matmul_noalloc: no weight");
    e->e->matmul_noalloc(name ? name : "matmul", w->w, Mp, C, ldc, c_off, acc, act32 != 0);
  });
}

arcz_moe_layer* arcz_moe_layer_upload(arcz_engine* e, uint32_t type, const void* gate, size_t gate_bytes, const void* up,
                                      size_t up_bytes, const void* down, size_t down_bytes, int NE, int NU, int E, int F) {
  arcz_moe_layer* L = new arcz_moe_layer;
  if (guarded([&] {
        // (the tensors are read for NE x rows x K values of the type: fewer bytes than that would be read past their end)
        int blk = 0, bb = 0;
        if (!arcz_ggml_block_info(type, &blk, &bb) || NE <= 0 || E <= 0 || F <= 0 || E % blk || F % blk)
          throw std::runtime_error("moe layer upload: type " + std::to_string(type) + " with E = " + std::to_string(E) +
                                   ", F = " + std::to_string(F));
        const size_t want_gu = (size_t)NE * F * (size_t)(E / blk) * bb, want_d = (size_t)NE * E * (size_t)(F / blk) * bb;
        if (gate_bytes != want_gu || up_bytes != want_gu || down_bytes != want_d)
          throw std::runtime_error("moe layer upload: the tensors hold " + std::to_string(gate_bytes) + " / " +
                                   std::to_string(up_bytes) + " / " + std::to_string(down_bytes) + " bytes, the shape takes " +
                                   std::to_string(want_gu) + " / " + std::to_string(want_gu) + " / " + std::to_string(want_d));
        L->L = e->e->make_moe_layer(type, (const uint8_t*)gate, (const uint8_t*)up, (const uint8_t*)down, NE, NU, E, F);
      }) != ARCZ_OK) {
    delete L;
    return nullptr;
  }
  return L;
}
int arcz_moe_layer_dims(const arcz_moe_layer* L, int* E, int* F) {
  if (!L) return ARCZ_E_ENGINE;
  if (E) *E = L->L.E;
  if (F) *F = L->L.F;
  return ARCZ_OK;
}
int arcz_engine_layer_moe(arcz_engine* e, arcz_moe_layer* L, arcz_mem* logits, int ldl, arcz_mem* x, int T, int Mp) {
  return guarded([&] { e->e->layer_moe(L->L, logits, ldl, x, T, Mp); });
}
int arcz_engine_layer_moe_sh(arcz_engine* e, arcz_moe_layer* L, arcz_mem* logits, int ldl, arcz_mem* x, int T, int Mp,
                             arcz_mem* sh) {
  return guarded([&] { e->e->layer_moe(L->L, logits, ldl, x, T, Mp, sh); });
}
int arcz_moe_layer_set_routing(arcz_engine* e, arcz_moe_layer* L, const float* escale, const float* ebias, float rscale) {
  return guarded([&] { e->e->set_moe_routing(L->L, escale, ebias, rscale); });
}
int arcz_moe_layer_free(arcz_engine* e, arcz_moe_layer* L) {
  if (!L) return ARCZ_OK;
  const int r = guarded([&] {
    e->e->free_moe_layer(L->L);
  });
  delete L;
  return r;
}
arcz_mem* arcz_engine_moe_sgate(arcz_engine* e) { return e->e->sgate_; }
int arcz_engine_moe_route(arcz_engine* e, arcz_moe_layer* L, arcz_mem* logits, int ldl, int T, int tm) {
  return guarded([&] { e->e->moe_route(L->L, logits, ldl, T, tm); });
}
arcz_mem* arcz_engine_moe_buffer(arcz_engine* e, int which) {
  Engine& E = *e->e;
  cl_mem b[13] = {E.mids_, E.mwts_, E.moffs_, E.mtiles_, E.mtstart_, E.stok_, E.swt_, E.minv_, E.mh_, E.mhq_, E.mhsc_, E.my_,
                  E.mhbs_};
  return which >= 0 && which < 13 ? b[which] : nullptr;
}
int arcz_engine_moe_slots(arcz_engine* e) { return e->e->slots_; }

int arcz_engine_self_check(void) {
  return guarded([&] {
    const std::string r = engine_self_check();
    if (!r.empty()) throw std::runtime_error(r);
  });
}

void arcz_engine_profile(arcz_engine* e, int on) { e->e->profile = on != 0; }
int arcz_engine_profile_collect(arcz_engine* e) {
  return guarded([&] { e->e->collect_profile(); });
}
int arcz_engine_profile_get(arcz_engine* e, const char* name, double* ms, int* launches) {
  auto it = e->e->prof_ms.find(name);
  if (it == e->e->prof_ms.end()) return -1;
  if (ms) *ms = it->second;
  if (launches) *launches = e->e->prof_n[name];
  return ARCZ_OK;
}
int arcz_engine_profile_stats(arcz_engine* e, const char* name, double* min_ms, double* median_ms) {
  auto it = e->e->prof_each.find(name);
  if (it == e->e->prof_each.end() || it->second.empty()) return -1;
  std::vector<double> v = it->second;
  std::sort(v.begin(), v.end());
  if (min_ms) *min_ms = v.front();
  if (median_ms) *median_ms = v.size() % 2 ? v[v.size() / 2] : 0.5 * (v[v.size() / 2 - 1] + v[v.size() / 2]);
  return ARCZ_OK;
}
void arcz_engine_profile_reset(arcz_engine* e) { e->e->prof_ms.clear(); e->e->prof_n.clear(); e->e->prof_each.clear(); }
uint64_t arcz_engine_rd_bytes(arcz_engine* e) { return e->e->rd_bytes; }

}  // extern "C"
