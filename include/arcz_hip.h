/*
 * arcz_hip.h -- the C ABI of the HIP backend that stands where the reference engine's runtime layer stands
 * (zero/clrt.h: an OpenCL-subset API on Level Zero, and zero/ze_min.h: the Level Zero loader).
 *
 * One process, one GPU, one in-order stream, one calling thread per device (the reference's rule, zero/clrt.h:47-57:
 * kernel objects carry no hidden state here, but the stream and the error text are per process).
 * Every call returns 0 on success or a negative status (the OpenCL numbers the reference returns where it returns
 * one); no C++ exception crosses this boundary.  arcz_last_error() gives the text of the last failure.
 *
 * Each entry point names the reference interface it replaces (paths relative to the reference tree).
 */
#ifndef ARCZ_HIP_H
#define ARCZ_HIP_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define ARCZ_OK 0
#define ARCZ_E_DEVICE (-2)         /* no device / HIP call failed (the reference ends the process: CL_CHECK, clrt.h:85-93) */
#define ARCZ_E_OOM (-4)            /* CL_MEM_OBJECT_ALLOCATION_FAILURE: after the out-of-memory hook gave up */
#define ARCZ_E_BUILD (-11)         /* CL_BUILD_PROGRAM_FAILURE: no such module / kernel variant */
#define ARCZ_E_SUBBUFFER (-13)     /* CL_MISALIGNED_SUB_BUFFER_OFFSET: a view past its parent (clrt.h:754-757) */
#define ARCZ_E_BOUNDS (-30)        /* CL_INVALID_VALUE: a transfer past a buffer's end is refused (clrt.h:676-681) */
#define ARCZ_E_ARG_INDEX (-49)     /* CL_INVALID_ARG_INDEX: wrong number of arguments for the kernel */
#define ARCZ_E_ARG_VALUE (-50)     /* CL_INVALID_ARG_VALUE: a pointer argument that is no live buffer */
#define ARCZ_E_ARG_SIZE (-51)      /* CL_INVALID_ARG_SIZE (clrt.h:900-903) */
#define ARCZ_E_WORK_GROUP (-54)    /* CL_INVALID_WORK_GROUP_SIZE: global not a multiple of local (clrt.h:973-981) */
#define ARCZ_E_RECORDING (-59)     /* CL_INVALID_OPERATION: a call that a launch list being recorded cannot hold, or a list call out of place */
#define ARCZ_E_GLOBAL_SIZE (-63)   /* CL_INVALID_GLOBAL_WORK_SIZE: a size past 32 bits (clrt.h:943-947) */

typedef struct arcz_mem arcz_mem;       /* the reference's cl_mem = ZMem {ptr, size, owner} (clrt.h:41-46) */
typedef struct arcz_kernel arcz_kernel; /* the reference's cl_kernel = ZKernel (clrt.h:47-57) */
typedef struct arcz_event arcz_event;   /* the reference's cl_event of a launch (clrt.h:982-983) */

/* Starts the runtime on GPU `device` (once per process; again = no-op): device, one stream, the embedded code
 * objects loaded, the address of the library's static device scratch taken.  Replaces ClRt::init (clrt.h:1064-1103).  0 or ARCZ_E_DEVICE. */
int arcz_init(int device);
/* Frees every live buffer, module and the stream (the reference's ClRt destructor path). */
void arcz_shutdown(void);
const char* arcz_last_error(void);
/* Device name ("gfx950 ..."), compute units, bytes of device memory: ClRt::device_id / clGetDeviceInfo (clrt.h:1025-1028). */
const char* arcz_device_name(void);
int arcz_device_cus(void);
size_t arcz_device_mem(void);

/* clCreateBuffer (clrt.h:744-751): device memory, at least 64 bytes, 256-byte aligned; NULL + error text on failure.
 * An allocation that fails calls the out-of-memory hook and is retried up to 8 times (clrt.h:474-487). */
arcz_mem* arcz_alloc(size_t bytes);
/* clCreateSubBuffer (clrt.h:752-762): a non-owning view; NULL if it would pass the parent's end. */
arcz_mem* arcz_view(arcz_mem* parent, size_t offset, size_t bytes);
/* clReleaseMemObject (clrt.h:763-769): waits for the stream, then frees (an owner) or forgets (a view).  The
 * caller frees views before their parents (zero/engine.h:251-252): an owner that still has live views is refused
 * (ARCZ_E_ARG_VALUE, nothing freed). */
int arcz_free(arcz_mem* m);
size_t arcz_mem_size(const arcz_mem* m);
/* The device address of a buffer (for interop with another runtime on the same device; not used by the engine). */
void* arcz_mem_ptr(const arcz_mem* m);
/* Bytes held by live owner buffers (zrt::Dev::device_bytes, clrt.h:766). */
size_t arcz_device_bytes(void);

/* clEnqueueWriteBuffer / ReadBuffer / CopyBuffer / FillBuffer (clrt.h:664-715): synchronous; a range past the end
 * of a buffer is refused with ARCZ_E_BOUNDS and nothing is touched. */
int arcz_h2d(arcz_mem* dst, size_t offset, const void* src, size_t bytes);
int arcz_d2h(void* dst, const arcz_mem* src, size_t offset, size_t bytes);
int arcz_d2d(arcz_mem* dst, size_t dst_offset, const arcz_mem* src, size_t src_offset, size_t bytes);
int arcz_fill(arcz_mem* dst, const void* pattern, size_t pattern_bytes, size_t offset, size_t bytes);

/* zrt::host_alloc and zrt::mem_free of such a pointer (clrt.h:445-452, 160): pinned host memory, the staging behind
 * clEnqueueMapBuffer / clEnqueueUnmapMemObject (clrt.h:711-743).  NULL + error text on failure. */
void* arcz_host_alloc(size_t bytes);
int arcz_host_free(void* p);

/* Engine::kernel(which, defs, name) (zero/engine_setup.h:317-362) over ClRt::build + ClRt::kernel
 * (clrt.h:1189-1307): `which` names the module ("ops", "decode", "gemm", "moe"), `defs` is the reference's -D string
 * and `name` the kernel.  The reference compiles one program per -D string at run time; here every variant is
 * compiled ahead of time: the -D names a kernel is specialized on select the variant, the rest become trailing
 * integer arguments the launch appends, and options that are not -D are ignored.  NULL + error text if there is no
 * such variant (the reference's soft_fail behaviour, clrt.h:1050).  Handles are cached: the same key gives the same
 * handle; they are freed by arcz_shutdown. */
arcz_kernel* arcz_kernel_get(const char* which, const char* defs, const char* name);
const char* arcz_kernel_symbol(const arcz_kernel* k);

/* clSetKernelArg + clEnqueueNDRangeKernel (clrt.h:877-909, 936-1022).  args[i] points at the value of argument i,
 * sizes[i] is its size.  An 8-byte value that is a live arcz_mem* becomes that buffer's device address
 * (clrt.h:880-886); any other non-null 8-byte value where the kernel takes a pointer is refused.  `global` are
 * OpenCL global sizes: a dimension of 0 is success without a launch; past 32 bits ARCZ_E_GLOBAL_SIZE; not a
 * multiple of `local` ARCZ_E_WORK_GROUP; local == NULL picks a size that divides.  The count and sizes of the
 * arguments are checked against the kernel's signature before anything is launched.  With `event` non-null the
 * launch is bracketed by timestamps (arcz_event_ms). */
int arcz_launch(arcz_kernel* k, unsigned dim, const size_t* global, const size_t* local, const void* const* args,
                const size_t* sizes, unsigned nargs, arcz_event** event);
/* clFinish (clrt.h:662). */
int arcz_sync(void);
/* ClRt::event_ms (clrt.h:1315-1321): device time of the launch in ms (waits for it); clReleaseEvent (clrt.h:1032-1035). */
double arcz_event_ms(arcz_event* e);
void arcz_event_release(arcz_event* e);
/* Timestamps on the stream without a launch of their own: a pair brackets any sequence of launches. */
arcz_event* arcz_event_record(void);
double arcz_event_elapsed_ms(arcz_event* start, arcz_event* stop);

/* Recorded launch lists: the reference's ARC_BATCH (clrt.h:170-265 -- kernels recorded into regular command lists and
 * handed to the GPU a list at a time instead of one by one), here a HIP graph captured from the stream.  Between
 * arcz_record_begin and arcz_record_end, arcz_launch without an event (and arcz_fill of whole words, which is a kernel)
 * add to the list and nothing runs; every call that allocates, frees, copies, waits or times returns
 * ARCZ_E_RECORDING (NULL where it returns a handle) and leaves the recording as it is -- so run a sequence once
 * before recording it, so that every buffer it needs exists.  arcz_record_end(NULL) drops the recording.
 * arcz_list_run submits the whole list (in stream order with everything else); it works on the buffers named when it
 * was recorded, with what they hold when it runs, so new input goes into the same buffers.  A list must be freed
 * before the buffers it names: arcz_free of an allocation that a live list names (directly or through a view) is
 * refused with ARCZ_E_ARG_VALUE and frees nothing.  arcz_mem_listed: 1 if a live list names the buffer's allocation
 * (what the owner of internal workspaces asks before it replaces one). */
typedef struct arcz_list arcz_list;
int arcz_record_begin(void);
int arcz_record_end(arcz_list** out);
int arcz_recording(void);
int arcz_list_run(arcz_list* l);
uint64_t arcz_list_launches(const arcz_list* l);
int arcz_list_free(arcz_list* l);
int arcz_mem_listed(const arcz_mem* m);

/* zrt::oom_hook (clrt.h:148-168): called when an allocation fails; returns nonzero if it freed something. */
void arcz_set_oom_hook(int (*hook)(void));
/* Test switch, the reference's ARC_FAKE_OOM (clrt.h:989-996): every n-th allocation "fails" once; 0 = off. */
void arcz_set_fake_oom(long every_nth);
/* Launch count since start (the reference's ARC_LAUNCH_STATS, clrt.h:770-782). */
uint64_t arcz_launch_count(void);

#ifdef __cplusplus
}
#endif
#endif
