// Cross-lane helpers of a 64-lane wavefront shared by the list kernels and the i2s kernels.
#pragma once
#include <hip/hip_runtime.h>

namespace sptmm {

template <int CTRL> __device__ __forceinline__ int dpp(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false); }
template <int CTRL> __device__ __forceinline__ float dpp(float v) { return __builtin_bit_cast(float, dpp<CTRL>(__builtin_bit_cast(int, v))); }
__device__ __forceinline__ int swz16(int v) { return __builtin_amdgcn_ds_swizzle(v, 0x401f); }  // lane ^ 16
__device__ __forceinline__ int swz8(int v) { return __builtin_amdgcn_ds_swizzle(v, 0x201f); }   // lane ^ 8
__device__ __forceinline__ int swz4(int v) { return __builtin_amdgcn_ds_swizzle(v, 0x101f); }   // lane ^ 4
__device__ __forceinline__ float swz16(float v) { return __builtin_bit_cast(float, swz16(__builtin_bit_cast(int, v))); }
__device__ __forceinline__ float swz8(float v) { return __builtin_bit_cast(float, swz8(__builtin_bit_cast(int, v))); }
__device__ __forceinline__ float swz4(float v) { return __builtin_bit_cast(float, swz4(__builtin_bit_cast(int, v))); }

// Sum over groups of 2^logL consecutive lanes (logL >= 2); every lane of a group ends with the group's total.
template <typename T>
__device__ __forceinline__ T lanes_sum(T v, int logL)
{
    v += dpp<0xB1>(v);                   // quad_perm [1,0,3,2]
    v += dpp<0x4E>(v);                   // quad_perm [2,3,0,1]
    if (logL >= 3) v += dpp<0x141>(v);   // row_half_mirror
    if (logL >= 4) v += dpp<0x140>(v);   // row_mirror
    if (logL >= 5) v += swz16(v);
    if (logL >= 6) v += __shfl_xor(v, 32, 64);
    return v;
}

}  // namespace sptmm
