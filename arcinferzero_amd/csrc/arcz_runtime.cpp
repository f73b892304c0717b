// HIP backend behind include/arcz_hip.h: buffers, one stream, ahead-of-time kernel variants looked up by the
// reference's (which, defs, name) key, checked launches, events.  It replaces the reference's zero/clrt.h +
// zero/ze_min.h (hipMalloc / hipModuleLaunchKernel / one hipStream_t).
#include "../../include/arcz_hip.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>
#include <string>
#include <vector>

#include "arcz_scratch.h"
#include "kernel_table.h"

struct arcz_mem {
  char* ptr;
  size_t size;
  bool owner;
  arcz_mem* parent = nullptr;  // a view's owner (the root of a chain of views)
};
struct arcz_kernel {
  hipFunction_t fn;
  const KernelSpec* spec;
  std::string symbol;
  std::vector<int> hidden;  // the -D values that ride along as trailing int arguments
  unsigned lds = 0;         // dynamic LDS bytes of every launch (-DLDS)
};
struct arcz_event {
  hipEvent_t start, stop;
  bool pair;
};
struct arcz_list {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  uint64_t launches = 0;  // kernels recorded
  std::set<arcz_mem*> owners;  // the allocations its kernels' buffer arguments lie in: not to be freed while it lives
};

namespace {
struct Runtime {
  bool up = false;
  int device = 0;
  hipStream_t stream = nullptr;
  hipDeviceProp_t prop;
  std::string name;
  std::set<arcz_mem*> mems;
  size_t device_bytes = 0;
  std::map<std::string, std::vector<hipModule_t>> modules;  // a module may be several code objects
  std::map<std::string, arcz_kernel*> kernels;
  int (*oom_hook)(void) = nullptr;
  long fake_oom = 0, allocs = 0;
  uint64_t launches = 0;
  std::string err;
  arcz_mem* scratch = nullptr;  // non-owning handle onto the device's static scratch array (arcz_scratch.hip)
  bool recording = false;       // between arcz_record_begin and arcz_record_end: launches go into a list, not to the GPU
  std::set<arcz_mem*> rec_owners;  // ... and the allocations their buffer arguments lie in
  uint64_t rec_launches = 0;
  std::set<arcz_list*> lists;
};
Runtime R;

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  R.err = buf;
  fprintf(stderr, "arcz: %s\n", buf);
  return code;
}
#define HIP_TRY(x)                                                                                          \
  do {                                                                                                      \
    hipError_t e_ = (x);                                                                                    \
    if (e_ != hipSuccess) return fail(ARCZ_E_DEVICE, "%s failed: %s", #x, hipGetErrorString(e_));           \
  } while (0)

// While a list is being recorded the stream takes nothing but kernel launches: what allocates, frees, copies to or from
// the host, waits or times is refused, with the recording left as it is.
#define NOT_WHILE_RECORDING(what, ret)                                                                       \
  do {                                                                                                      \
    if (R.recording) {                                                                                      \
      fail(ARCZ_E_RECORDING, "%s while a launch list is being recorded (refused; run the sequence once before " \
                             "recording it, so that every buffer it needs exists)", what);                  \
      return ret;                                                                                           \
    }                                                                                                       \
  } while (0)

bool out_of_bounds(const char* what, const arcz_mem* b, size_t off, size_t n) {
  if (b && R.mems.count(const_cast<arcz_mem*>(b)) && off <= b->size && n <= b->size - off) return false;
  fail(ARCZ_E_BOUNDS, "%s of %zu bytes at offset %zu past the end of a %zu-byte buffer (refused)", what, n, off,
       b && R.mems.count(const_cast<arcz_mem*>(b)) ? b->size : (size_t)0);
  return true;
}
}  // namespace

extern "C" {

// the code objects, linked in by kernel_blobs.S
extern const unsigned char arcz_blob_ops[], arcz_blob_decode[], arcz_blob_decode_q80[], arcz_blob_decode_q40[], arcz_blob_decode_q4k[],
    arcz_blob_decode_q5k[], arcz_blob_decode_q6k[], arcz_blob_decode_iq4xs[], arcz_blob_decode_iq3s[], arcz_blob_decode_iq4nl[], arcz_blob_decode_mxfp4[], arcz_blob_decode_q3k[], arcz_blob_decode_iq3xxs[], arcz_blob_decode_mm[], arcz_blob_gemm[], arcz_blob_moe[];

static std::vector<const unsigned char*> blobs_of(const std::string& which);

int arcz_init(int device) {
  if (R.up) return ARCZ_OK;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return fail(ARCZ_E_DEVICE, "no HIP device");
  if (device < 0 || device >= n) return fail(ARCZ_E_DEVICE, "device %d of %d", device, n);
  HIP_TRY(hipSetDevice(device));
  HIP_TRY(hipGetDeviceProperties(&R.prop, device));
  R.name = std::string(R.prop.gcnArchName) + " " + R.prop.name;
  if (R.name.rfind("gfx950", 0) != 0 && !getenv("ARCZ_ANY_ARCH"))
    return fail(ARCZ_E_DEVICE, "device %d is %s: the kernels are built for gfx950 only", device, R.name.c_str());
  HIP_TRY(hipStreamCreate(&R.stream));
  R.device = device;
  // Everything a later call could otherwise make the HIP runtime allocate for is done here, so that the entry point
  // that must not allocate (arcz_engine_matmul_noalloc) finds it in place: the address of the static scratch array on
  // this device (asked for once, with the device current) behind a non-owning handle, and the code objects loaded.
  void* sp = nullptr;
  size_t sb = 0;
  const char* serr = "";
  if (arcz_scratch_setup(device, &sp, &sb, &serr) != 0) {
    hipStreamDestroy(R.stream);
    R.stream = nullptr;
    return fail(ARCZ_E_DEVICE, "the static device scratch has no address on device %d: %s", device, serr);
  }
  R.scratch = new arcz_mem{(char*)sp, sb, false};
  R.mems.insert(R.scratch);
  for (const char* w : {"ops", "decode", "gemm", "moe"}) {
    std::vector<hipModule_t> mods;
    for (const unsigned char* blob : blobs_of(w)) {
      hipModule_t mod;
      hipError_t e = hipModuleLoadData(&mod, blob);
      if (e != hipSuccess) {
        for (hipModule_t m : mods) hipModuleUnload(m);
        for (auto& kv : R.modules)
          for (hipModule_t m : kv.second) hipModuleUnload(m);
        R.modules.clear();
        R.mems.erase(R.scratch);
        delete R.scratch;
        R.scratch = nullptr;
        hipStreamDestroy(R.stream);
        R.stream = nullptr;
        return fail(ARCZ_E_BUILD, "module %s does not load: %s", w, hipGetErrorString(e));
      }
      mods.push_back(mod);
    }
    R.modules.emplace(w, mods);
  }
  R.up = true;
  return ARCZ_OK;
}

arcz_mem* arcz_scratch_mem(void) { return R.up ? R.scratch : nullptr; }

void arcz_shutdown(void) {
  if (!R.up) return;
  if (R.recording) {  // (an open recording is dropped)
    hipGraph_t g = nullptr;
    if (hipStreamEndCapture(R.stream, &g) == hipSuccess && g) hipGraphDestroy(g);
    (void)hipGetLastError();
    R.recording = false;
  }
  hipStreamSynchronize(R.stream);
  for (arcz_list* l : R.lists) {
    hipGraphExecDestroy(l->exec);
    hipGraphDestroy(l->graph);
    delete l;
  }
  R.lists.clear();
  for (auto& kv : R.kernels) delete kv.second;
  R.kernels.clear();
  for (auto& kv : R.modules)
    for (hipModule_t m : kv.second) hipModuleUnload(m);
  R.modules.clear();
  for (arcz_mem* m : R.mems) {
    if (m->owner) hipFree(m->ptr);
    delete m;
  }
  R.mems.clear();
  R.scratch = nullptr;  // (its handle went with the others; the array itself stays with the device)
  R.device_bytes = 0;
  hipStreamDestroy(R.stream);
  R.stream = nullptr;
  R.up = false;
}

const char* arcz_last_error(void) { return R.err.c_str(); }
const char* arcz_device_name(void) { return R.name.c_str(); }
int arcz_device_cus(void) { return R.up ? R.prop.multiProcessorCount : 0; }
size_t arcz_device_mem(void) { return R.up ? R.prop.totalGlobalMem : 0; }
size_t arcz_device_bytes(void) { return R.device_bytes; }

arcz_mem* arcz_alloc(size_t bytes) {
  if (!R.up) { fail(ARCZ_E_DEVICE, "arcz_alloc before arcz_init"); return nullptr; }
  NOT_WHILE_RECORDING("arcz_alloc", nullptr);
  const size_t n = bytes < 64 ? 64 : bytes;
  void* p = nullptr;
  hipError_t e = hipSuccess;
  ++R.allocs;
  for (int attempt = 0; attempt <= 8; ++attempt) {
    const bool fake = R.fake_oom > 0 && attempt == 0 && R.allocs % R.fake_oom == 0;
    e = fake ? hipErrorOutOfMemory : hipMalloc(&p, n);
    if (e == hipSuccess) break;
    if (!fake) (void)hipGetLastError();
    if (e != hipErrorOutOfMemory) break;
    if (!(R.oom_hook && R.oom_hook())) break;  // nothing was freed: give up (clrt.h:474-487)
  }
  if (e != hipSuccess || !p) {
    fail(ARCZ_E_OOM, "allocation of %zu bytes failed: %s", n, hipGetErrorString(e));
    return nullptr;
  }
  arcz_mem* m = new arcz_mem{(char*)p, bytes, true};
  R.mems.insert(m);
  R.device_bytes += bytes;
  return m;
}

arcz_mem* arcz_view(arcz_mem* parent, size_t offset, size_t bytes) {
  if (!parent || !R.mems.count(parent) || offset > parent->size || bytes > parent->size - offset) {
    fail(ARCZ_E_SUBBUFFER, "view of %zu bytes at %zu past its parent's end", bytes, offset);
    return nullptr;
  }
  arcz_mem* m = new arcz_mem{parent->ptr + offset, bytes, false, parent->owner ? parent : parent->parent};
  R.mems.insert(m);
  return m;
}

int arcz_free(arcz_mem* m) {
  if (!m) return ARCZ_OK;
  if (m == R.scratch) return fail(ARCZ_E_ARG_VALUE, "arcz_free of the library's static scratch");
  if (!R.mems.count(m)) return fail(ARCZ_E_ARG_VALUE, "arcz_free of a handle that is not live");
  if (m->owner) NOT_WHILE_RECORDING("arcz_free", ARCZ_E_RECORDING);
  if (m->owner) {
    // (the caller frees views before their parents, zero/engine.h:251-252; a view that is still live would name freed
    //  memory: refused, nothing is freed)
    for (const arcz_mem* v : R.mems)
      if (v->parent == m) return fail(ARCZ_E_ARG_VALUE, "arcz_free of a buffer that still has live views");
    // (a recorded list keeps the device addresses of the buffers its kernels were given: it would read and write
    //  freed memory.  Refused, nothing is freed: free the list first)
    if (arcz_mem_listed(m)) return fail(ARCZ_E_ARG_VALUE, "arcz_free of a buffer that a live launch list names");
    HIP_TRY(hipStreamSynchronize(R.stream));
    HIP_TRY(hipFree(m->ptr));
    R.device_bytes -= m->size;
  }
  R.mems.erase(m);
  delete m;
  return ARCZ_OK;
}

int arcz_mem_listed(const arcz_mem* m) {
  if (!m || !R.mems.count(const_cast<arcz_mem*>(m))) return 0;
  arcz_mem* o = m->owner ? const_cast<arcz_mem*>(m) : m->parent;
  for (const arcz_list* l : R.lists)
    if (l->owners.count(o)) return 1;
  return 0;
}
size_t arcz_mem_size(const arcz_mem* m) { return m && R.mems.count(const_cast<arcz_mem*>(m)) ? m->size : 0; }
void* arcz_mem_ptr(const arcz_mem* m) { return m && R.mems.count(const_cast<arcz_mem*>(m)) ? m->ptr : nullptr; }

int arcz_h2d(arcz_mem* dst, size_t offset, const void* src, size_t bytes) {
  if (out_of_bounds("write", dst, offset, bytes)) return ARCZ_E_BOUNDS;
  if (!bytes) return ARCZ_OK;
  NOT_WHILE_RECORDING("arcz_h2d", ARCZ_E_RECORDING);
  HIP_TRY(hipMemcpyAsync(dst->ptr + offset, src, bytes, hipMemcpyHostToDevice, R.stream));
  HIP_TRY(hipStreamSynchronize(R.stream));
  return ARCZ_OK;
}
int arcz_d2h(void* dst, const arcz_mem* src, size_t offset, size_t bytes) {
  if (out_of_bounds("read", src, offset, bytes)) return ARCZ_E_BOUNDS;
  if (!bytes) return ARCZ_OK;
  NOT_WHILE_RECORDING("arcz_d2h", ARCZ_E_RECORDING);
  HIP_TRY(hipMemcpyAsync(dst, src->ptr + offset, bytes, hipMemcpyDeviceToHost, R.stream));
  HIP_TRY(hipStreamSynchronize(R.stream));
  return ARCZ_OK;
}
int arcz_d2d(arcz_mem* dst, size_t dst_offset, const arcz_mem* src, size_t src_offset, size_t bytes) {
  if (out_of_bounds("copy (source)", src, src_offset, bytes) || out_of_bounds("copy (destination)", dst, dst_offset, bytes))
    return ARCZ_E_BOUNDS;
  if (!bytes) return ARCZ_OK;
  NOT_WHILE_RECORDING("arcz_d2d", ARCZ_E_RECORDING);
  HIP_TRY(hipMemcpyAsync(dst->ptr + dst_offset, src->ptr + src_offset, bytes, hipMemcpyDeviceToDevice, R.stream));
  return ARCZ_OK;
}

// zrt::host_alloc / mem_free of a host pointer (clrt.h:445-452, 160): pinned host memory the device can copy to and from at
// full rate; allocated, never registered over existing memory.
void* arcz_host_alloc(size_t bytes) {
  if (!R.up) { fail(ARCZ_E_DEVICE, "arcz_host_alloc before arcz_init"); return nullptr; }
  NOT_WHILE_RECORDING("arcz_host_alloc", nullptr);
  void* p = nullptr;
  const hipError_t e = hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocDefault);
  if (e != hipSuccess || !p) {
    (void)hipGetLastError();
    fail(ARCZ_E_OOM, "pinned host allocation of %zu bytes failed: %s", bytes, hipGetErrorString(e));
    return nullptr;
  }
  return p;
}
int arcz_host_free(void* p) {
  if (!p) return ARCZ_OK;
  NOT_WHILE_RECORDING("arcz_host_free", ARCZ_E_RECORDING);
  HIP_TRY(hipHostFree(p));
  return ARCZ_OK;
}

static arcz_kernel* fill_kernel();

int arcz_fill(arcz_mem* dst, const void* pattern, size_t ps, size_t offset, size_t bytes) {
  if (out_of_bounds("fill", dst, offset, bytes)) return ARCZ_E_BOUNDS;
  if (!bytes) return ARCZ_OK;
  if ((ps != 1 && ps != 2 && ps != 4) || bytes % ps || offset % ps)
    return fail(ARCZ_E_BOUNDS, "fill pattern of %zu bytes over %zu bytes at %zu", ps, bytes, offset);
  uint32_t v = 0;
  memcpy(&v, pattern, ps);
  if (ps == 1) v |= v << 8;
  if (ps <= 2) v |= v << 16;
  if (bytes % 4 == 0 && offset % 4 == 0) {
    // a small kernel rather than a memset node (the call still waits for the stream, as the reference's fill does,
    // clrt.h:703-710: the pattern is the caller's; it is not a call for a stream that is being captured)
    arcz_kernel* k = fill_kernel();
    if (!k) return ARCZ_E_BUILD;
    void* p = dst->ptr + offset;
    size_t n = bytes / 4;
    void* params[3] = {&p, &v, &n};
    const unsigned blocks = (unsigned)((n + 255) / 256);
    HIP_TRY(hipModuleLaunchKernel(k->fn, blocks, 1, 1, 256, 1, 1, 0, R.stream, params, nullptr));
    if (R.recording) {  // (recorded as the kernel it is; nothing to wait for)
      ++R.rec_launches;
      R.rec_owners.insert(dst->owner ? dst : dst->parent);
      return ARCZ_OK;
    }
  } else {
    NOT_WHILE_RECORDING("arcz_fill of a range that is not whole words", ARCZ_E_RECORDING);  // (no memset nodes in a list)
    if (ps == 1) HIP_TRY(hipMemsetAsync(dst->ptr + offset, (int)(v & 0xFF), bytes, R.stream));
    else HIP_TRY(hipMemsetD16Async((hipDeviceptr_t)(dst->ptr + offset), (unsigned short)(v & 0xFFFF), bytes / 2, R.stream));
  }
  HIP_TRY(hipStreamSynchronize(R.stream));
  return ARCZ_OK;
}

// ---- kernels

static std::vector<const unsigned char*> blobs_of(const std::string& which) {
  if (which == "ops") return {arcz_blob_ops};
  if (which == "decode") return {arcz_blob_decode, arcz_blob_decode_q80, arcz_blob_decode_q40, arcz_blob_decode_q4k, arcz_blob_decode_q5k, arcz_blob_decode_q6k, arcz_blob_decode_iq4xs, arcz_blob_decode_iq3s, arcz_blob_decode_iq4nl, arcz_blob_decode_mxfp4, arcz_blob_decode_q3k, arcz_blob_decode_iq3xxs, arcz_blob_decode_mm};
  if (which == "gemm") return {arcz_blob_gemm};
  if (which == "moe") return {arcz_blob_moe};
  return {};
}

// "-DQT=12 -DGROWS=2 -cl-whatever" -> {QT: 12, GROWS: 2}; a -D without a value is 1
static std::map<std::string, long> parse_defs(const char* defs) {
  std::map<std::string, long> out;  // (SOFTCAP, RSCALE: the bit pattern of the float value)
  const std::string s = defs ? defs : "";
  size_t i = 0;
  while (i < s.size()) {
    while (i < s.size() && s[i] == ' ') ++i;
    size_t j = i;
    while (j < s.size() && s[j] != ' ') ++j;
    const std::string tok = s.substr(i, j - i);
    if (tok.size() > 2 && tok[0] == '-' && tok[1] == 'D') {
      const size_t eq = tok.find('=');
      const std::string name = tok.substr(2, eq == std::string::npos ? std::string::npos : eq - 2);
      if ((name == "SOFTCAP" || name == "RSCALE") && eq != std::string::npos) {
        const float f = strtof(tok.c_str() + eq + 1, nullptr);
        uint32_t bits;
        memcpy(&bits, &f, 4);
        out[name] = (long)bits;
      } else {
        out[name] = eq == std::string::npos ? 1 : strtol(tok.c_str() + eq + 1, nullptr, 0);
      }
    }
    i = j;
  }
  return out;
}

arcz_kernel* arcz_kernel_get(const char* which, const char* defs, const char* name) {
  if (!R.up) { fail(ARCZ_E_DEVICE, "arcz_kernel_get before arcz_init"); return nullptr; }
  const std::string w = which ? which : "", d = defs ? defs : "", nm = name ? name : "";
  const std::string key = w + d + "|" + nm;  // the reference's cache key (engine_setup.h:318)
  auto it = R.kernels.find(key);
  if (it != R.kernels.end()) return it->second;
  const std::map<std::string, long> dv = parse_defs(defs);
  const KernelSpec* spec = nullptr;
  for (const KernelSpec& s : kKernelTable)
    if (!spec && w == s.which && nm == s.name && (!s.requires_def || dv.count(s.requires_def))) spec = &s;
  if (!spec) { fail(ARCZ_E_BUILD, "no kernel %s in module %s", nm.c_str(), w.c_str()); return nullptr; }
  std::string symbol = nm;
  for (int i = 0; spec->variant[i]; ++i) {
    auto f = dv.find(spec->variant[i]);
    if (f == dv.end()) { fail(ARCZ_E_BUILD, "%s: -D%s is required", nm.c_str(), spec->variant[i]); return nullptr; }
    symbol += (i == 0 ? "__" : "_") + std::string(spec->variant[i]) + std::to_string(f->second);
  }
  std::vector<int> hidden;
  unsigned lds = 0;
  for (int i = 0; spec->hidden[i].name; ++i) {
    auto f = dv.find(spec->hidden[i].name);
    if (f == dv.end() && spec->hidden[i].required) {
      fail(ARCZ_E_BUILD, "%s: -D%s is required", nm.c_str(), spec->hidden[i].name);
      return nullptr;
    }
    const int v = f == dv.end() ? spec->hidden[i].def : (int)f->second;
    if (std::string(spec->hidden[i].name) == "LDS") {
      if (v < 0 || v > 65536) { fail(ARCZ_E_BUILD, "%s: %d bytes of LDS", nm.c_str(), v); return nullptr; }
      lds = (unsigned)v;
    } else {
      hidden.push_back(v);
    }
  }
  auto mi = R.modules.find(w);
  if (mi == R.modules.end()) {
    const std::vector<const unsigned char*> blobs = blobs_of(w);
    if (blobs.empty()) { fail(ARCZ_E_BUILD, "no module %s", w.c_str()); return nullptr; }
    std::vector<hipModule_t> mods;
    for (const unsigned char* blob : blobs) {
      hipModule_t mod;
      hipError_t e = hipModuleLoadData(&mod, blob);
      if (e != hipSuccess) { fail(ARCZ_E_BUILD, "module %s does not load: %s", w.c_str(), hipGetErrorString(e)); return nullptr; }
      mods.push_back(mod);
    }
    mi = R.modules.emplace(w, mods).first;
  }
  hipFunction_t fn = nullptr;
  for (hipModule_t mod : mi->second) {
    if (hipModuleGetFunction(&fn, mod, symbol.c_str()) == hipSuccess) break;
    (void)hipGetLastError();
    fn = nullptr;
  }
  if (!fn) {
    fail(ARCZ_E_BUILD, "module %s has no variant %s (defs \"%s\")", w.c_str(), symbol.c_str(), d.c_str());
    return nullptr;
  }
  arcz_kernel* k = new arcz_kernel{fn, spec, symbol, hidden, lds};
  R.kernels[key] = k;
  return k;
}

static arcz_kernel* fill_kernel() { return arcz_kernel_get("ops", "", "fill32"); }

const char* arcz_kernel_symbol(const arcz_kernel* k) { return k ? k->symbol.c_str() : ""; }

int arcz_launch(arcz_kernel* k, unsigned dim, const size_t* global, const size_t* local, const void* const* args,
                const size_t* sizes, unsigned nargs, arcz_event** event) {
  if (event) *event = nullptr;
  if (!R.up || !k) return fail(ARCZ_E_DEVICE, "arcz_launch without a runtime or kernel");
  if (dim < 1 || dim > 3) return fail(ARCZ_E_GLOBAL_SIZE, "%s: %u dimensions", k->symbol.c_str(), dim);
  unsigned gs[3] = {1, 1, 1}, ls[3] = {1, 1, 1};
  for (unsigned d = 0; d < dim; ++d) {
    if (global[d] == 0) return ARCZ_OK;  // nothing to run (clrt.h:942)
    if (global[d] > 0xFFFFFFFFull)
      return fail(ARCZ_E_GLOBAL_SIZE, "%s: global size %zu past 32 bits (refused)", k->symbol.c_str(), global[d]);
    gs[d] = (unsigned)global[d];
  }
  if (local) {
    for (unsigned d = 0; d < dim; ++d) ls[d] = (unsigned)local[d];
  } else {
    ls[0] = 256;
    while (ls[0] > 1 && gs[0] % ls[0]) --ls[0];
  }
  for (unsigned d = 0; d < 3; ++d)
    if (ls[d] == 0 || gs[d] % ls[d])
      return fail(ARCZ_E_WORK_GROUP, "%s: global size %u x %u x %u is not a multiple of the work-group %u x %u x %u",
                  k->symbol.c_str(), gs[0], gs[1], gs[2], ls[0], ls[1], ls[2]);
  if ((size_t)ls[0] * ls[1] * ls[2] > 1024 || (k->spec->local_x && ls[0] * ls[1] * ls[2] != (unsigned)k->spec->local_x))
    return fail(ARCZ_E_WORK_GROUP, "%s: work-group %u x %u x %u (the kernel is written for %d threads)",
                k->symbol.c_str(), ls[0], ls[1], ls[2], k->spec->local_x ? k->spec->local_x : 1024);
  // arguments: count, sizes, pointers
  const size_t nsig = strlen(k->spec->args);
  if (nargs != nsig)
    return fail(ARCZ_E_ARG_INDEX, "%s takes %zu arguments, %u given", k->symbol.c_str(), nsig, nargs);
  unsigned char store[64][8];
  void* params[64 + 8];
  if (nsig + k->hidden.size() > 64) return fail(ARCZ_E_ARG_INDEX, "%s: too many arguments", k->symbol.c_str());
  for (unsigned i = 0; i < nargs; ++i) {
    const char c = k->spec->args[i];
    const size_t want = (c == 'p' || c == 'z') ? 8 : 4;
    if (sizes[i] != want || !args[i])
      return fail(ARCZ_E_ARG_SIZE, "%s: argument %u has %zu bytes, the kernel takes %zu", k->symbol.c_str(), i, sizes[i], want);
    memcpy(store[i], args[i], want);
    if (c == 'p') {
      arcz_mem* m;
      memcpy(&m, args[i], 8);
      if (m) {
        if (!R.mems.count(m))
          return fail(ARCZ_E_ARG_VALUE, "%s: argument %u is not a live buffer", k->symbol.c_str(), i);
        memcpy(store[i], &m->ptr, 8);
        if (R.recording) R.rec_owners.insert(m->owner ? m : m->parent);
      }
    }
    params[i] = store[i];
  }
  for (size_t h = 0; h < k->hidden.size(); ++h) params[nargs + h] = &k->hidden[h];
  arcz_event* ev = nullptr;
  if (event) NOT_WHILE_RECORDING("arcz_launch with an event", ARCZ_E_RECORDING);
  if (event) {
    ev = new arcz_event{nullptr, nullptr, true};
    HIP_TRY(hipEventCreate(&ev->start));
    HIP_TRY(hipEventCreate(&ev->stop));
    HIP_TRY(hipEventRecord(ev->start, R.stream));
  }
  hipError_t e = hipModuleLaunchKernel(k->fn, gs[0] / ls[0], gs[1] / ls[1], gs[2] / ls[2], ls[0], ls[1], ls[2], k->lds,
                                       R.stream, params, nullptr);
  if (e != hipSuccess) {
    if (ev) { hipEventDestroy(ev->start); hipEventDestroy(ev->stop); delete ev; }
    return fail(ARCZ_E_DEVICE, "launch of %s (global %u x %u x %u, local %u x %u x %u) failed: %s", k->symbol.c_str(),
                gs[0], gs[1], gs[2], ls[0], ls[1], ls[2], hipGetErrorString(e));
  }
  if (R.recording) ++R.rec_launches;  // (it runs when the list runs)
  else ++R.launches;
  if (ev) {
    HIP_TRY(hipEventRecord(ev->stop, R.stream));
    *event = ev;
  }
  return ARCZ_OK;
}

int arcz_sync(void) {
  if (!R.up) return fail(ARCZ_E_DEVICE, "arcz_sync before arcz_init");
  NOT_WHILE_RECORDING("arcz_sync", ARCZ_E_RECORDING);
  HIP_TRY(hipStreamSynchronize(R.stream));
  return ARCZ_OK;
}

double arcz_event_ms(arcz_event* e) {
  if (!e || !e->pair) return -1.0;
  if (hipEventSynchronize(e->stop) != hipSuccess) return -1.0;
  float ms = 0;
  if (hipEventElapsedTime(&ms, e->start, e->stop) != hipSuccess) return -1.0;
  return ms;
}
void arcz_event_release(arcz_event* e) {
  if (!e) return;
  hipEventDestroy(e->start);
  if (e->pair) hipEventDestroy(e->stop);
  delete e;
}
arcz_event* arcz_event_record(void) {
  if (!R.up) return nullptr;
  NOT_WHILE_RECORDING("arcz_event_record", nullptr);
  arcz_event* ev = new arcz_event{nullptr, nullptr, false};
  if (hipEventCreate(&ev->start) != hipSuccess || hipEventRecord(ev->start, R.stream) != hipSuccess) {
    delete ev;
    return nullptr;
  }
  return ev;
}
double arcz_event_elapsed_ms(arcz_event* start, arcz_event* stop) {
  if (!start || !stop) return -1.0;
  if (hipEventSynchronize(stop->start) != hipSuccess) return -1.0;
  float ms = 0;
  if (hipEventElapsedTime(&ms, start->start, stop->start) != hipSuccess) return -1.0;
  return ms;
}

// ---- recorded launch lists.  The reference can record its kernels into regular command lists and hand the GPU a
// whole list at a time (ARC_BATCH, zero/clrt.h:170-265: 700 small kernels took 2.56 us each appended one by one and
// 0.66 us replayed from a list); here the stream is captured into a HIP graph.  Between begin and end arcz_launch
// (and a whole-word arcz_fill) add to the list and nothing reaches the GPU; the list then runs as one submission, as
// often as wanted, on the same buffers with whatever they hold at that time.
int arcz_record_begin(void) {
  if (!R.up) return fail(ARCZ_E_DEVICE, "arcz_record_begin before arcz_init");
  NOT_WHILE_RECORDING("arcz_record_begin", ARCZ_E_RECORDING);
  // (thread-local mode: calls of other threads that are unsafe under capture do not break this one)
  HIP_TRY(hipStreamBeginCapture(R.stream, hipStreamCaptureModeThreadLocal));
  R.recording = true;
  R.rec_launches = 0;
  R.rec_owners.clear();
  return ARCZ_OK;
}
int arcz_record_end(arcz_list** out) {
  if (out) *out = nullptr;
  if (!R.up || !R.recording) return fail(ARCZ_E_RECORDING, "arcz_record_end without arcz_record_begin");
  R.recording = false;
  hipGraph_t g = nullptr;
  hipError_t e = hipStreamEndCapture(R.stream, &g);
  if (e != hipSuccess || !g) {
    (void)hipGetLastError();
    return fail(ARCZ_E_DEVICE, "the recording did not end in a list: %s", hipGetErrorString(e));
  }
  if (!out || R.rec_launches == 0) {  // (abandoned, or empty: nothing to keep)
    hipGraphDestroy(g);
    return out ? fail(ARCZ_E_RECORDING, "nothing was recorded") : ARCZ_OK;
  }
  hipGraphExec_t x = nullptr;
  e = hipGraphInstantiate(&x, g, nullptr, nullptr, 0);
  if (e != hipSuccess || !x) {
    (void)hipGetLastError();
    hipGraphDestroy(g);
    return fail(ARCZ_E_DEVICE, "the recorded list does not instantiate: %s", hipGetErrorString(e));
  }
  arcz_list* l = new arcz_list{g, x, R.rec_launches, R.rec_owners};
  R.rec_owners.clear();
  R.lists.insert(l);
  *out = l;
  return ARCZ_OK;
}
int arcz_recording(void) { return R.recording ? 1 : 0; }
int arcz_list_run(arcz_list* l) {
  if (!R.up || !l || !R.lists.count(l)) return fail(ARCZ_E_ARG_VALUE, "arcz_list_run of a handle that is not a live list");
  NOT_WHILE_RECORDING("arcz_list_run", ARCZ_E_RECORDING);
  HIP_TRY(hipGraphLaunch(l->exec, R.stream));
  R.launches += l->launches;
  return ARCZ_OK;
}
uint64_t arcz_list_launches(const arcz_list* l) { return l && R.lists.count(const_cast<arcz_list*>(l)) ? l->launches : 0; }
int arcz_list_free(arcz_list* l) {
  if (!l) return ARCZ_OK;
  if (!R.lists.count(l)) return fail(ARCZ_E_ARG_VALUE, "arcz_list_free of a handle that is not a live list");
  NOT_WHILE_RECORDING("arcz_list_free", ARCZ_E_RECORDING);
  HIP_TRY(hipStreamSynchronize(R.stream));  // (a run of it may still be in flight)
  hipGraphExecDestroy(l->exec);
  hipGraphDestroy(l->graph);
  R.lists.erase(l);
  delete l;
  return ARCZ_OK;
}

void arcz_set_oom_hook(int (*hook)(void)) { R.oom_hook = hook; }
void arcz_set_fake_oom(long n) { R.fake_oom = n; R.allocs = 0; }
uint64_t arcz_launch_count(void) { return R.launches; }

}  // extern "C"
