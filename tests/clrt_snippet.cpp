// A short program in the style of the reference's engine code (zero/engine_setup.h:317-362, zero/engine_load.h): the
// OpenCL-subset names of zero/clrt.h -- clCreateBuffer, ClRt::build, ClRt::kernel, set_args, clEnqueueNDRangeKernel,
// CL_CHECK, clEnqueueMapBuffer / clEnqueueUnmapMemObject, clEnqueueReadBuffer -- compiled against clrt_hip.h instead.
// Built by the library's Makefile (target clrt_snippet); tests/test_gpu_runtime.py runs it on the GPU and reads its
// exit status (0 = every check held).
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "clrt_hip.h"

#define EXPECT(c)                                                   \
  do {                                                              \
    if (!(c)) {                                                     \
      fprintf(stderr, "clrt_snippet: %s failed (line %d)\n", #c, __LINE__); \
      return 1;                                                     \
    }                                                               \
  } while (0)

int main() {
  ClRt cl;
  cl.soft_fail = true;
  if (!cl.init()) {
    fprintf(stderr, "clrt_snippet: no GPU runtime: %s\n", arcz_last_error());
    return 2;
  }
  printf("device %s\n", cl.device_id.c_str());
  cl_int err = 0;
  cl_mem buf = clCreateBuffer(cl.ctx, CL_MEM_READ_WRITE, 4096, nullptr, &err);
  CL_CHECK(err);
  // a program per (module, option string), a kernel by name: options that are not -D are ignored
  cl_program p = cl.build("ops", "-cl-std=CL3.0 -cl-mad-enable");
  cl_kernel k = cl.kernel(p, "fill32");
  const uint32_t v = 0xABCD1234u;
  const size_t n = 1024;
  set_args(k, 0, buf, v, n);
  size_t gws = 1024, lws = 256;
  CL_CHECK(clEnqueueNDRangeKernel(cl.queue, k, 1, nullptr, &gws, &lws, 0, nullptr, nullptr));
  CL_CHECK(clFinish(cl.queue));
  // mapped for reading: the device's bytes
  uint32_t* m = (uint32_t*)clEnqueueMapBuffer(cl.queue, buf, CL_TRUE, CL_MAP_READ, 0, 4096, 0, nullptr, nullptr, &err);
  EXPECT(m && err == CL_SUCCESS);
  for (size_t i = 0; i < n; ++i) EXPECT(m[i] == v);
  m[5] = 0;  // (a read map is not written back)
  CL_CHECK(clEnqueueUnmapMemObject(cl.queue, buf, m, 0, nullptr, nullptr));
  // mapped for writing, a sub-range: written back when released
  uint32_t* w = (uint32_t*)clEnqueueMapBuffer(cl.queue, buf, CL_TRUE, CL_MAP_WRITE, 1024, 512, 0, nullptr, nullptr, &err);
  EXPECT(w && err == CL_SUCCESS);
  for (int i = 0; i < 128; ++i) w[i] = (uint32_t)i;
  CL_CHECK(clEnqueueUnmapMemObject(cl.queue, buf, w, 0, nullptr, nullptr));
  std::vector<uint32_t> back(1024);
  CL_CHECK(clEnqueueReadBuffer(cl.queue, buf, CL_TRUE, 0, 4096, back.data(), 0, nullptr, nullptr));
  for (int i = 0; i < 1024; ++i) EXPECT(back[i] == (i >= 256 && i < 384 ? (uint32_t)(i - 256) : v));
  // refused: a map past the end, the release of something that is no map
  EXPECT(clEnqueueMapBuffer(cl.queue, buf, CL_TRUE, CL_MAP_READ, 4000, 200, 0, nullptr, nullptr, &err) == nullptr && err == -30);
  EXPECT(clEnqueueUnmapMemObject(cl.queue, buf, back.data(), 0, nullptr, nullptr) == -30);
  // the matmul kernels by the reference's option strings; an unknown kernel throws under soft_fail as a failed build does
  cl_program pd = cl.build("decode", "-cl-std=CL3.0 -cl-mad-enable -DQT=12 -DGROWS=2");
  cl_kernel kd = cl.kernel(pd, "gemv_v");
  EXPECT(kd && kd->k);
  bool thrown = false;
  try {
    cl.kernel(pd, "no_such_kernel");
  } catch (const std::runtime_error&) {
    thrown = true;
  }
  EXPECT(thrown);
  // an allocation that fails after the out-of-memory hook has given up throws while zrt::oom_throws is set (it ends
  // the process otherwise, as the reference's does): the runtime's test switch makes the next allocation fail
  arcz_set_fake_oom(1);
  zrt::oom_throws = true;
  thrown = false;
  try {
    clCreateBuffer(cl.ctx, CL_MEM_READ_WRITE, 1 << 20, nullptr, &err);
  } catch (const std::runtime_error& e) {
    thrown = strstr(e.what(), "device allocation of") != nullptr;
  }
  arcz_set_fake_oom(0);
  zrt::oom_throws = false;
  EXPECT(thrown);
  cl_mem after = clCreateBuffer(cl.ctx, CL_MEM_READ_WRITE, 1 << 20, nullptr, &err);
  EXPECT(after && err == CL_SUCCESS);
  CL_CHECK(clReleaseMemObject(after));
  clReleaseKernel(k);
  clReleaseKernel(kd);
  clReleaseProgram(p);
  clReleaseProgram(pd);
  CL_CHECK(clReleaseMemObject(buf));
  printf("clrt_snippet ok\n");
  return 0;
}
