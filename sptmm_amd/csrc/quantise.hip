// Activation rows quantised in a launch of their own, for sptmm_gemv_q8_ws beyond four rows: the quantising list kernels
// redo the rows' quantisation in every workgroup (each reads all the rows twice), which at eight rows costs more than the
// GEMV itself (K=6912 N=2560, M=8, one call: 18.9 us against 8.1 us for the int8 GEMV); here one workgroup per row does it
// once, and the int8 kernels scale their sums by the rows' 1/s on the way out (QUANT = 2 in lists.hpp).
// Same arithmetic as the fused kernels, value for value (Quantiser): a = max(max|x|, 1e-5), s = 127 / a,
// q = rint(x * s), 1/s = a / 127.
#include "lists.hpp"

namespace sptmm {

__global__ void __launch_bounds__(1024) quantise_rows_kernel(const unsigned short *X, int kind, int M, int K, int8_t *Xq, float *inv, int threads)
{
    typedef Quantiser<1> Q;
    __shared__ float wave_max[16];
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = threads >> 6;
    const int items = K / 16;
    u32 mb[1] = {0u};
    for (int item = tid; item < items; item += threads) {
        uint4 r[2];
        Q::load(X, M, K, row, item, r);
        Q::absmax(r, mb);
    }
    float mx = Q::magnitude(mb[0], kind);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if (lane == 0) wave_max[wave] = mx;
    __syncthreads();
    float a = 0.f;
    for (int w = 0; w < waves; ++w) a = fmaxf(a, wave_max[w]);
    a = fmaxf(a, 1e-5f);
    const float sc[1] = {127.0f / a};
    if (tid == 0) inv[row] = a / 127.0f;
    for (int item = tid; item < items; item += threads) {
        uint4 r[2], q[1];
        Q::load(X, M, K, row, item, r);
        Q::quantise(r, kind, sc, q);
        reinterpret_cast<uint4 *>(Xq + (size_t)row * K)[item] = q[0];
    }
}

int launch_quantise_rows(const void *X, int kind, int M, int K, void *Xq, float *inv, void *stream)
{
    if (M < 1 || K < 16 || K % 16) return fail(SPTMM_ERR_INVALID, "quantise_rows: M >= 1 and K a positive multiple of 16");
    const int items = K / 16;
    const int waves = items >= 1024 ? 16 : items >= 256 ? 4 : 1;
    hipLaunchKernelGGL(quantise_rows_kernel, dim3(M), dim3(64 * waves), 0, (hipStream_t)stream, (const unsigned short *)X, kind, M, K, (int8_t *)Xq, inv,
                       64 * waves);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : fail(SPTMM_ERR_HIP, "quantise_rows_kernel launch: %s (%d)", hipGetErrorString(e), (int)e);
}

// ---- scratch for callers that cannot allocate (sptmm_gemv_q8_static): the workspace of sptmm_gemv_q8_ws, in the library's
// own device image.  Every GPU the library runs on holds its copy of the array until the process ends, each at its own
// address; `scratch` is only the host-side name of the symbol -- what kernels and copies take is the device address
// looked up below, once per device.
constexpr size_t SCRATCH_BYTES = 512 * 1024 + 4096;  // the int8 activation values (M x K, some 524,000 of them at most), then the rows' 1/s
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[SCRATCH_BYTES];  // (no kernel names it: kept for the look-up)
constexpr int SCRATCH_DEVICES = 64;
static std::atomic<void *> scratch_ptr[SCRATCH_DEVICES];

size_t scratch_bytes() { return SCRATCH_BYTES; }

// with `device` current: look up and keep the address of this device's copy of the array
int scratch_init(int device)
{
    if (device < 0 || device >= SCRATCH_DEVICES) return SPTMM_OK;  // (no slot to keep it in: scratch_of says so when asked)
    void *ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return fail(SPTMM_ERR_HIP, "hipGetSymbolAddress(scratch): %s (%d)", hipGetErrorString(e), (int)e);
    scratch_ptr[device].store(ptr, std::memory_order_release);
    return SPTMM_OK;
}

// the device address of `device`'s copy (looked up now if sptmm_device_init has not run for it; `device` must be current)
int scratch_of(int device, void **ptr)
{
    if (device < 0 || device >= SCRATCH_DEVICES) return fail(SPTMM_ERR_UNSUPPORTED, "static scratch is kept for devices 0..%d", SCRATCH_DEVICES - 1);
    void *p = scratch_ptr[device].load(std::memory_order_acquire);
    if (!p) {
        if (int rc = scratch_init(device)) return rc;
        p = scratch_ptr[device].load(std::memory_order_acquire);
    }
    *ptr = p;
    return SPTMM_OK;
}

}  // namespace sptmm
