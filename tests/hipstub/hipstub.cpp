// Stand-in for the HIP runtime on a machine without a GPU: enough of its host API for libsptmm's launch paths
// (shape checks, launch-shape model, batching, stream capture, the timing loops) to run end to end on the CPU.
// Launches are counted and the first bytes of their first argument are read; nothing runs.  "Device" memory is
// host memory.  Linked into the test driver with -rdynamic, so that the library's own references to the runtime
// resolve here first.  Test infrastructure: nothing in the product links or loads it.
#include <hip/hip_runtime_api.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

static std::atomic<long> g_launches{0};
static thread_local dim3 g_grid, g_block;
static thread_local size_t g_shmem;
static thread_local hipStream_t g_stream;
static std::atomic<unsigned long> g_sink{0};
static bool g_capturing = false;

extern "C" long hipstub_launches() { return g_launches.load(); }

extern "C" {
void **__hipRegisterFatBinary(const void *) { static void *h[4]; return h; }
void __hipUnregisterFatBinary(void **) {}
void __hipRegisterFunction(void **, const void *, char *, const char *, unsigned, void *, void *, void *, void *, int *) {}
void __hipRegisterVar(void **, void *, char *, char *, int, size_t, int, int) {}
hipError_t __hipPushCallConfiguration(dim3 grid, dim3 block, size_t shmem, hipStream_t st)
{
    g_grid = grid, g_block = block, g_shmem = shmem, g_stream = st;
    return hipSuccess;
}
hipError_t __hipPopCallConfiguration(dim3 *grid, dim3 *block, size_t *shmem, hipStream_t *st)
{
    *grid = g_grid, *block = g_block, *shmem = g_shmem, *st = g_stream;
    return hipSuccess;
}
hipError_t hipLaunchKernel(const void *f, dim3 grid, dim3 block, void **args, size_t shmem, hipStream_t)
{
    // touch the first argument (every kernel of the library takes at least a pointer's worth)
    unsigned long s = 0;
    if (args && args[0])
        for (size_t i = 0; i < sizeof(void *); ++i) s += ((const unsigned char *)args[0])[i];
    g_sink += s + grid.x + block.x + shmem + (unsigned long)(size_t)f;
    ++g_launches;
    return hipSuccess;
}
hipError_t hipGetSymbolAddress(void **p, const void *)
{
    static unsigned char image[1 << 20];  // stands for every __device__ variable of the library
    *p = image;
    return hipSuccess;
}
hipError_t hipGetLastError() { return hipSuccess; }
hipError_t hipPeekAtLastError() { return hipSuccess; }
const char *hipGetErrorString(hipError_t) { return "stub"; }
hipError_t hipGetDeviceCount(int *n) { *n = 1; return hipSuccess; }
hipError_t hipGetDevice(int *d) { *d = 0; return hipSuccess; }
hipError_t hipSetDevice(int) { return hipSuccess; }
hipError_t hipDeviceGetAttribute(int *v, hipDeviceAttribute_t a, int)
{
    *v = a == hipDeviceAttributeMultiprocessorCount ? 256 : a == hipDeviceAttributeMaxSharedMemoryPerBlock ? 160 * 1024 : 0;
    return hipSuccess;
}
hipError_t hipGetDevicePropertiesR0600(hipDeviceProp_t *p, int)
{
    memset(p, 0, sizeof *p);
    strcpy(p->name, "stub");
    strcpy(p->gcnArchName, "gfx950");
    p->multiProcessorCount = 256, p->warpSize = 64, p->sharedMemPerBlock = 160 * 1024;
    return hipSuccess;
}
hipError_t hipMalloc(void **p, size_t n) { *p = malloc(n ? n : 16); return *p ? hipSuccess : hipErrorOutOfMemory; }
hipError_t hipFree(void *p) { free(p); return hipSuccess; }
hipError_t hipMemcpy(void *d, const void *s, size_t n, hipMemcpyKind) { memcpy(d, s, n); return hipSuccess; }
hipError_t hipMemset(void *d, int v, size_t n) { memset(d, v, n); return hipSuccess; }
hipError_t hipDeviceSynchronize() { return hipSuccess; }
hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned) { *s = (hipStream_t)malloc(8); return hipSuccess; }
hipError_t hipStreamDestroy(hipStream_t s) { free(s); return hipSuccess; }
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipSuccess; }
hipError_t hipEventCreate(hipEvent_t *e) { *e = (hipEvent_t)malloc(8); return hipSuccess; }
hipError_t hipEventCreateWithFlags(hipEvent_t *e, unsigned) { *e = (hipEvent_t)malloc(8); return hipSuccess; }
hipError_t hipEventDestroy(hipEvent_t e) { free(e); return hipSuccess; }
hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float *ms, hipEvent_t, hipEvent_t) { *ms = 1.0f; return hipSuccess; }
hipError_t hipFuncGetAttributes(hipFuncAttributes *a, const void *) { memset(a, 0, sizeof *a); a->numRegs = 64; return hipSuccess; }
hipError_t hipFuncSetAttribute(const void *, hipFuncAttribute, int) { return hipSuccess; }
hipError_t hipStreamBeginCapture(hipStream_t, hipStreamCaptureMode) { g_capturing = true; return hipSuccess; }
hipError_t hipStreamEndCapture(hipStream_t, hipGraph_t *g) { g_capturing = false; *g = (hipGraph_t)malloc(8); return hipSuccess; }
hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus *s) { *s = g_capturing ? hipStreamCaptureStatusActive : hipStreamCaptureStatusNone; return hipSuccess; }
hipError_t hipGraphInstantiate(hipGraphExec_t *e, hipGraph_t, hipGraphNode_t *, char *, size_t) { *e = (hipGraphExec_t)malloc(8); return hipSuccess; }
hipError_t hipGraphLaunch(hipGraphExec_t, hipStream_t) { return hipSuccess; }
hipError_t hipGraphExecDestroy(hipGraphExec_t e) { free(e); return hipSuccess; }
hipError_t hipGraphDestroy(hipGraph_t g) { free(g); return hipSuccess; }
}
