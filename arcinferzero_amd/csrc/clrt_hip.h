// The OpenCL-subset names the reference engine is written against (zero/clrt.h), on top of the C ABI of
// include/arcz_hip.h.  Engine code that says clCreateBuffer / clSetKernelArg / clEnqueueNDRangeKernel / CL_CHECK /
// set_args compiles against this header unchanged; underneath there is hipMalloc, hipModuleLaunchKernel and one
// stream instead of Level Zero.
#pragma once
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/arcz_hip.h"

typedef int cl_int;
typedef unsigned cl_uint;
typedef unsigned cl_bool;
typedef unsigned long cl_ulong;
typedef cl_ulong cl_mem_flags;
typedef cl_ulong cl_map_flags;
typedef cl_uint cl_buffer_create_type;
typedef arcz_mem* cl_mem;
typedef arcz_event* cl_event;
typedef struct _arcz_queue* cl_command_queue;
typedef struct _arcz_context* cl_context;
struct cl_buffer_region { size_t origin, size; };

// cl_kernel: the backend's kernel handle plus the argument values set so far (clSetKernelArg keeps them per kernel,
// zero/clrt.h:47-57; a launch sends them all).
struct ArczKernelArgs {
  arcz_kernel* k = nullptr;
  std::string name;
  struct Arg { size_t sz = 0; unsigned char v[8] = {}; };
  std::vector<Arg> args;
};
typedef ArczKernelArgs* cl_kernel;

#define CL_SUCCESS 0
#define CL_TRUE 1
#define CL_FALSE 0
#define CL_MEM_READ_WRITE (1 << 0)
#define CL_MEM_WRITE_ONLY (1 << 1)
#define CL_MEM_READ_ONLY (1 << 2)
#define CL_MEM_COPY_HOST_PTR (1 << 5)
#define CL_BUFFER_CREATE_TYPE_REGION 0x1220
#define CL_MAP_READ (1 << 0)
#define CL_MAP_WRITE (1 << 1)
#define CL_MAP_WRITE_INVALIDATE_REGION (1 << 2)

// cl_program: what ClRt::build returns.  The reference compiles OpenCL C with an option string at run time
// (zero/clrt.h:1189-1281); here the kernels are compiled ahead of time, so a "program" is the module's name and the
// option string, and ClRt::kernel looks the variant up.
struct ArczProgram {
  std::string which, opts;
};
typedef ArczProgram* cl_program;

// Any failure ends the process with a message, unless the owner asked for exceptions (the reference's CL_CHECK,
// zero/clrt.h:85-93, and soft_fail, :1050).
namespace arcz {
inline bool& soft_fail() { static bool v = false; return v; }
inline void check(int err, const char* what, const char* file, int line) {
  if (err == CL_SUCCESS) return;
  char msg[640];
  snprintf(msg, sizeof msg, "%s failed with %d at %s:%d: %s", what, err, file, line, arcz_last_error());
  if (soft_fail()) throw std::runtime_error(msg);
  fprintf(stderr, "arcz: %s\n", msg);
  fflush(stderr);
  _Exit(1);
}
}  // namespace arcz
#define CL_CHECK(x) arcz::check((x), #x, __FILE__, __LINE__)

// zrt::oom_throws (zero/clrt.h:148-168, 474-487): what an allocation does once the out-of-memory hook has given up --
// the reference never hands a failed allocation back to its caller: it ends the process with the sizes that say why,
// or, while this thread-local switch is set (a model being placed that the caller can still load elsewhere), throws.
namespace zrt {
inline thread_local bool oom_throws = false;
}  // namespace zrt

inline cl_int clFinish(cl_command_queue) { return arcz_sync(); }
inline cl_int clFlush(cl_command_queue) { return CL_SUCCESS; }
inline cl_mem clCreateBuffer(cl_context, cl_mem_flags flags, size_t n, void* host, cl_int* err) {
  cl_mem m = arcz_alloc(n);
  // (out of memory -- the hook was called and could free nothing more, or there is none -- as against a call before
  //  arcz_init or inside a recording, which come back as errors: told apart by the runtime's message)
  if (!m && strncmp(arcz_last_error(), "allocation of", 13) == 0) {
    char msg[256];
    snprintf(msg, sizeof msg, "device allocation of %.1f MB failed (%.2f GiB allocated): %s", n / 1e6,
             arcz_device_bytes() / 1073741824.0, arcz_last_error());
    if (zrt::oom_throws) throw std::runtime_error(msg);
    fprintf(stderr, "arcz: %s\n", msg);
    fflush(stderr);
    _Exit(1);
  }
  cl_int e = m ? CL_SUCCESS : ARCZ_E_OOM;
  if (m && (flags & CL_MEM_COPY_HOST_PTR) && host) e = arcz_h2d(m, 0, host, n);
  if (err) *err = e;
  return m;
}
inline cl_mem clCreateSubBuffer(cl_mem parent, cl_mem_flags, cl_buffer_create_type, const void* region, cl_int* err) {
  const cl_buffer_region* r = (const cl_buffer_region*)region;
  cl_mem m = arcz_view(parent, r->origin, r->size);
  if (err) *err = m ? CL_SUCCESS : ARCZ_E_SUBBUFFER;
  return m;
}
inline cl_int clReleaseMemObject(cl_mem m) { return arcz_free(m); }
inline cl_int clEnqueueReadBuffer(cl_command_queue, cl_mem b, cl_bool, size_t off, size_t n, void* host, cl_uint,
                                  const cl_event*, cl_event* ev) {
  if (ev) *ev = nullptr;
  return arcz_d2h(host, b, off, n);
}
inline cl_int clEnqueueWriteBuffer(cl_command_queue, cl_mem b, cl_bool, size_t off, size_t n, const void* host, cl_uint,
                                   const cl_event*, cl_event* ev) {
  if (ev) *ev = nullptr;
  return arcz_h2d(b, off, host, n);
}
inline cl_int clEnqueueCopyBuffer(cl_command_queue, cl_mem src, cl_mem dst, size_t so, size_t doff, size_t n, cl_uint,
                                  const cl_event*, cl_event* ev) {
  if (ev) *ev = nullptr;
  return arcz_d2d(dst, doff, src, so, n);
}
inline cl_int clEnqueueFillBuffer(cl_command_queue, cl_mem b, const void* pattern, size_t ps, size_t off, size_t n,
                                  cl_uint, const cl_event*, cl_event* ev) {
  if (ev) *ev = nullptr;
  return arcz_fill(b, pattern, ps, off, n);
}
// clEnqueueMapBuffer / clEnqueueUnmapMemObject (zero/clrt.h:711-743): a pinned host copy of [off, off + n) of b -- read
// from the device when mapped for reading, written back when a map for writing is released.
namespace arcz {
struct Map { cl_mem m; size_t off, n; void* host; cl_map_flags flags; };
inline std::vector<Map>& maps() { static std::vector<Map> v; return v; }
}  // namespace arcz
inline void* clEnqueueMapBuffer(cl_command_queue, cl_mem b, cl_bool, cl_map_flags flags, size_t off, size_t n, cl_uint,
                                const cl_event*, cl_event* ev, cl_int* err) {
  if (ev) *ev = nullptr;
  if (!b || off > arcz_mem_size(b) || n > arcz_mem_size(b) - off) {  // (refused as the transfers refuse it)
    if (err) *err = ARCZ_E_BOUNDS;
    return nullptr;
  }
  void* h = arcz_host_alloc(n);
  if (!h) {
    if (err) *err = ARCZ_E_OOM;
    return nullptr;
  }
  if (flags & CL_MAP_READ) {
    const cl_int e = arcz_d2h(h, b, off, n);
    if (e != CL_SUCCESS) {
      arcz_host_free(h);
      if (err) *err = e;
      return nullptr;
    }
  }
  arcz::maps().push_back({b, off, n, h, flags});
  if (err) *err = CL_SUCCESS;
  return h;
}
inline cl_int clEnqueueUnmapMemObject(cl_command_queue, cl_mem b, void* p, cl_uint, const cl_event*, cl_event* ev) {
  if (ev) *ev = nullptr;
  auto& mp = arcz::maps();
  for (size_t i = 0; i < mp.size(); ++i)
    if (mp[i].host == p && mp[i].m == b) {
      cl_int e = CL_SUCCESS;
      if (mp[i].flags & (CL_MAP_WRITE | CL_MAP_WRITE_INVALIDATE_REGION)) e = arcz_h2d(b, mp[i].off, p, mp[i].n);
      arcz_host_free(p);
      mp.erase(mp.begin() + (long)i);
      return e;
    }
  return ARCZ_E_BOUNDS;  // (not a live map of b)
}
inline cl_int clReleaseProgram(cl_program p) { delete p; return CL_SUCCESS; }

inline cl_int clSetKernelArg(cl_kernel k, cl_uint i, size_t sz, const void* v) {
  if (!k || sz > 8 || !v) return ARCZ_E_ARG_SIZE;
  if (k->args.size() <= i) k->args.resize(i + 1);
  k->args[i].sz = sz;
  memcpy(k->args[i].v, v, sz);
  return CL_SUCCESS;
}
inline cl_int clEnqueueNDRangeKernel(cl_command_queue, cl_kernel k, cl_uint dim, const size_t*, const size_t* g,
                                     const size_t* l, cl_uint, const cl_event*, cl_event* ev) {
  const void* ptrs[64];
  size_t sizes[64];
  const size_t n = k->args.size();
  if (n > 64) return ARCZ_E_ARG_INDEX;
  for (size_t i = 0; i < n; ++i) { ptrs[i] = k->args[i].v; sizes[i] = k->args[i].sz; }
  return arcz_launch(k->k, dim, g, l, ptrs, sizes, (unsigned)n, ev);
}
inline cl_int clReleaseEvent(cl_event e) { arcz_event_release(e); return CL_SUCCESS; }
inline cl_int clReleaseKernel(cl_kernel k) { delete k; return CL_SUCCESS; }

// set_args(k, first index, values...) (zero/clrt.h:1363-1367)
inline void set_args(cl_kernel, cl_uint) {}
template <class T, class... Rest>
inline void set_args(cl_kernel k, cl_uint i, const T& v, const Rest&... rest) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "kernel arguments are 4 or 8 bytes");
  CL_CHECK(clSetKernelArg(k, i, sizeof(T), &v));
  set_args(k, i + 1, rest...);
}

// ClRt: start-up and kernel lookup (zero/clrt.h:1025-1333).  build() + kernel() of the reference compile a program
// per option string; here both are one lookup in the ahead-of-time variants.
struct ClRt {
  std::string device_id;
  bool soft_fail = false;
  cl_context ctx = (cl_context)1;
  cl_command_queue queue = (cl_command_queue)1;
  bool init(bool = false) {
    if (arcz_init(0) != ARCZ_OK) return false;
    device_id = arcz_device_name();
    return true;
  }
  // build(src, opts) + kernel(prog, name) (zero/clrt.h:1189, 1282).  `src` is the module's name ("ops", "decode",
  // "gemm", "moe") where the reference passes the text of its .cl file; options that are not -D are ignored.  An
  // unknown module is reported by kernel(), as a failed build is in the reference.
  cl_program build(const std::string& src, const std::string& opts) { return new ArczProgram{src, opts}; }
  cl_kernel kernel(cl_program prog, const char* name) { return kernel(prog->which, prog->opts, name); }
  cl_kernel kernel(const std::string& which, const std::string& defs, const std::string& name) {
    arcz_kernel* h = arcz_kernel_get(which.c_str(), defs.c_str(), name.c_str());
    if (!h) {
      const std::string msg = "no kernel " + which + " " + defs + " | " + name + ": " + arcz_last_error();
      if (soft_fail || arcz::soft_fail()) throw std::runtime_error(msg);
      fprintf(stderr, "arcz: %s\n", msg.c_str());
      _Exit(1);
    }
    cl_kernel k = new ArczKernelArgs;
    k->k = h;
    k->name = name;
    return k;
  }
  cl_mem buffer(cl_mem_flags flags, size_t n, const void* host = nullptr) {
    cl_int err;
    cl_mem m = clCreateBuffer(ctx, flags | (host ? CL_MEM_COPY_HOST_PTR : 0), n, const_cast<void*>(host), &err);
    CL_CHECK(err);
    return m;
  }
  static double event_ms(cl_event e) { return arcz_event_ms(e); }
};
