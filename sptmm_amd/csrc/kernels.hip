// gfx950 kernels of the SpTMM engine and their launchers.
//
// All three kernels are HBM-bound gather/unpack work: no multiplies on the
// list paths, packed-integer dot4 on the i2s path, no MFMA anywhere.  Common
// shape: the activation tile is staged once per workgroup in LDS (every column
// reuses it), each 64-lane wavefront streams its slice of the weight stream
// with 16-byte per-lane loads that are contiguous across the wavefront, and
// split-K partials are folded across lanes, then (when a column spans several
// wavefronts) through a small LDS buffer.  No atomics.
#include <hip/hip_runtime.h>

#include <atomic>

#include "internal.hpp"

namespace sptmm {

typedef unsigned int u32;

// ------------------------------------------------------------------ helpers
template <typename Act> struct Acc { typedef float type; };
template <> struct Acc<int8_t> { typedef int type; };

template <typename Act, int MT> struct alignas(sizeof(Act) * MT) Row { Act v[MT]; };

// acc[m] (+|-)= X[m][idx] for the MT rows interleaved at lds[idx*MT .. idx*MT+MT)
template <typename Act, int MT, bool NEG>
__device__ __forceinline__ void gather(const Act *lds, u32 idx, typename Acc<Act>::type (&acc)[MT])
{
    typedef typename Acc<Act>::type A;
    Row<Act, MT> r = reinterpret_cast<const Row<Act, MT> *>(lds)[idx];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if (NEG)
            acc[m] -= (A)r.v[m];
        else
            acc[m] += (A)r.v[m];
    }
}

// MODE 0: fields are absolute u16 row indices.  MODE 1 / 2: fields are 8- /
// 16-bit gaps added to a running row index.  Consumes the low NBYTES of `d`.
template <typename Act, int MT, int MODE, bool NEG, int NBYTES>
__device__ __forceinline__ void consume(const Act *lds, u32 d, u32 &run, typename Acc<Act>::type (&acc)[MT])
{
    if (MODE == 1) {
#pragma unroll
        for (int b = 0; b < NBYTES; ++b) {
            run += (d >> (8 * b)) & 0xffu;
            gather<Act, MT, NEG>(lds, run, acc);
        }
    } else {
#pragma unroll
        for (int h = 0; h < NBYTES / 2; ++h) {
            u32 f = h ? (d >> 16) : (d & 0xffffu);
            if (MODE == 2) {
                run += f;
                f = run;
            }
            gather<Act, MT, NEG>(lds, f, acc);
        }
    }
}

template <typename Act, int MT, int MODE, bool NEG>
__device__ __forceinline__ void consume16(const Act *lds, const uint4 &v, u32 &run, typename Acc<Act>::type (&acc)[MT])
{
    consume<Act, MT, MODE, NEG, 4>(lds, v.x, run, acc);
    consume<Act, MT, MODE, NEG, 4>(lds, v.y, run, acc);
    consume<Act, MT, MODE, NEG, 4>(lds, v.z, run, acc);
    consume<Act, MT, MODE, NEG, 4>(lds, v.w, run, acc);
}

// 4 rows x 4 consecutive k (one dword per row) -> 4 dwords, dword j = the 4 rows at k+j
__device__ __forceinline__ void transpose4x4(u32 r0, u32 r1, u32 r2, u32 r3, u32 &o0, u32 &o1, u32 &o2, u32 &o3)
{
    u32 a = __builtin_amdgcn_perm(r1, r0, 0x05010400u), b = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
    u32 c = __builtin_amdgcn_perm(r3, r2, 0x05010400u), d = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    o0 = __builtin_amdgcn_perm(c, a, 0x05040100u);
    o1 = __builtin_amdgcn_perm(c, a, 0x07060302u);
    o2 = __builtin_amdgcn_perm(d, b, 0x05040100u);
    o3 = __builtin_amdgcn_perm(d, b, 0x07060302u);
}

// Stage rows [m0, m0+MT) of X (row-major [M][K]) into LDS as [K+1][MT]; rows
// past M and the extra slot K read as zero.
template <typename Act, int MT>
__device__ __forceinline__ void stage_x(Act *lds, const Act *X, int M, int K, int m0)
{
    const int tid = threadIdx.x, nt = blockDim.x;
    if constexpr (MT == 1) {
        const int per = 16 / (int)sizeof(Act);
        const uint4 *src = reinterpret_cast<const uint4 *>(X + (size_t)m0 * K);
        uint4 *dst = reinterpret_cast<uint4 *>(lds);
        for (int i = tid; i < K / per; i += nt) dst[i] = src[i];
    } else if constexpr (sizeof(Act) == 1 && (MT == 4 || MT == 8)) {
        const u32 *x32 = reinterpret_cast<const u32 *>(X);
        const int kq = K / 4;  // dwords per row
        for (int q = tid; q < kq; q += nt) {
            u32 r[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) r[m] = (m0 + m < M) ? x32[(size_t)(m0 + m) * kq + q] : 0u;
            u32 o[4];
            transpose4x4(r[0], r[1], r[2], r[3], o[0], o[1], o[2], o[3]);
            if constexpr (MT == 4) {
                reinterpret_cast<uint4 *>(lds)[q] = make_uint4(o[0], o[1], o[2], o[3]);
            } else {
                u32 p[4];
                transpose4x4(r[MT - 4], r[MT - 3], r[MT - 2], r[MT - 1], p[0], p[1], p[2], p[3]);
                reinterpret_cast<uint4 *>(lds)[2 * q] = make_uint4(o[0], p[0], o[1], p[1]);
                reinterpret_cast<uint4 *>(lds)[2 * q + 1] = make_uint4(o[2], p[2], o[3], p[3]);
            }
        }
    } else {
        for (int i = tid; i < K * MT; i += nt) {
            int k = i / MT, m = i % MT;
            lds[i] = (m0 + m < M) ? X[(size_t)(m0 + m) * K + k] : (Act)0;
        }
    }
    if (tid < MT) lds[(size_t)K * MT + tid] = (Act)0;
}

template <typename T>
__device__ __forceinline__ T lanes_sum(T v, int L)
{
    for (int off = L >> 1; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;  // valid in the first lane of every group of L lanes
}

struct ListParams {
    const uint8_t *w;
    const void *X;
    void *C;
    int M, K, N;
    int n_lane, tasks, L, G, W;
    int iters;  // tasks each wavefront walks: ceil(tasks / (gridDim.x * waves))
};

constexpr int LISTS_MAX_WAVES = 8;  // 512 threads: two wavefronts per SIMD, 256 VGPRs each

// ------------------------------------------------- index-list / gap-stream GEMV
// One task = one wavefront's share of the stream: G columns x L lanes, or one
// 64-lane part of a column.  A workgroup stages the activation tile once and its
// wavefronts then walk tasks blockIdx.x*waves + wave, + gridDim.x*waves, ...
// blockIdx.y selects the tile of MT activation rows.
template <typename Act, int MT, int MODE>
__global__ void __launch_bounds__(64 * LISTS_MAX_WAVES) lists_kernel(ListParams p)
{
    typedef typename Acc<Act>::type A;
    constexpr int ESZ = (MODE == 1) ? 1 : 2;   // bytes per stream entry
    constexpr int E16 = 16 / ESZ;              // entries per 16-byte load
    constexpr int RB = 4;                      // rounds per prefetch block
    constexpr int HDR = MODE ? 256 : 0;        // restart indices of a gap-stream task
    extern __shared__ __align__(16) unsigned char smem[];
    Act *lds = reinterpret_cast<Act *>(smem);
    A *part = reinterpret_cast<A *>(smem + (((size_t)(p.K + 1) * MT * sizeof(Act) + 15) & ~(size_t)15));

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int m0 = blockIdx.y * MT;
    const size_t task_bytes = HDR + (size_t)128 * ESZ * p.n_lane;
    const int R = p.n_lane / E16, nb = R / RB;
    int task = blockIdx.x * waves + wave;
    const int task_step = gridDim.x * waves;

    // the first block of the first task goes in flight before X is staged
    uint4 bp[RB], bq[RB], cp[RB], cq[RB];
    {
        const uint4 *wp = reinterpret_cast<const uint4 *>(p.w + (size_t)(task < p.tasks ? task : 0) * task_bytes + HDR) + lane;
        if (nb > 0) {
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                bp[i] = wp[(2 * i) * 64];
                bq[i] = wp[(2 * i + 1) * 64];
            }
        }
    }

    stage_x<Act, MT>(lds, reinterpret_cast<const Act *>(p.X), p.M, p.K, m0);
    __syncthreads();

    A *C = reinterpret_cast<A *>(p.C);
    for (int it = 0; it < p.iters; ++it, task += task_step) {
        const bool active = task < p.tasks;
        const uint8_t *tb = p.w + (size_t)(active ? task : 0) * task_bytes;
        const uint4 *wp = reinterpret_cast<const uint4 *>(tb + HDR) + lane;
        u32 runp = 0, runq = 0;
        if (MODE) {
            const unsigned short *rs = reinterpret_cast<const unsigned short *>(tb);
            runp = rs[lane];
            runq = rs[64 + lane];
        }
        if (it > 0 && nb > 0) {
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                bp[i] = wp[(2 * i) * 64];
                bq[i] = wp[(2 * i + 1) * 64];
            }
        }
        A acc[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = (A)0;

        for (int b = 0; b < nb; b += 2) {
            if (b + 1 < nb) {
#pragma unroll
                for (int i = 0; i < RB; ++i) {
                    cp[i] = wp[(2 * ((b + 1) * RB + i)) * 64];
                    cq[i] = wp[(2 * ((b + 1) * RB + i) + 1) * 64];
                }
            }
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                consume16<Act, MT, MODE, false>(lds, bp[i], runp, acc);
                consume16<Act, MT, MODE, true>(lds, bq[i], runq, acc);
            }
            if (b + 2 < nb) {
#pragma unroll
                for (int i = 0; i < RB; ++i) {
                    bp[i] = wp[(2 * ((b + 2) * RB + i)) * 64];
                    bq[i] = wp[(2 * ((b + 2) * RB + i) + 1) * 64];
                }
            }
            if (b + 1 < nb) {
#pragma unroll
                for (int i = 0; i < RB; ++i) {
                    consume16<Act, MT, MODE, false>(lds, cp[i], runp, acc);
                    consume16<Act, MT, MODE, true>(lds, cq[i], runq, acc);
                }
            }
        }
        for (int r = nb * RB; r < R; ++r) {
            uint4 vp = wp[(2 * r) * 64], vq = wp[(2 * r + 1) * 64];
            consume16<Act, MT, MODE, false>(lds, vp, runp, acc);
            consume16<Act, MT, MODE, true>(lds, vq, runq, acc);
        }
        // ragged tail: at most one round each of 8, 4, 2 (and 1) bytes per lane
        {
            const uint8_t *t = tb + HDR + (size_t)R * 2048;
            const int rem = p.n_lane - R * E16;
            if (rem & (8 / ESZ)) {
                uint2 vp = reinterpret_cast<const uint2 *>(t)[lane], vq = reinterpret_cast<const uint2 *>(t + 512)[lane];
                consume<Act, MT, MODE, false, 4>(lds, vp.x, runp, acc);
                consume<Act, MT, MODE, false, 4>(lds, vp.y, runp, acc);
                consume<Act, MT, MODE, true, 4>(lds, vq.x, runq, acc);
                consume<Act, MT, MODE, true, 4>(lds, vq.y, runq, acc);
                t += 1024;
            }
            if (rem & (4 / ESZ)) {
                u32 vp = reinterpret_cast<const u32 *>(t)[lane], vq = reinterpret_cast<const u32 *>(t + 256)[lane];
                consume<Act, MT, MODE, false, 4>(lds, vp, runp, acc);
                consume<Act, MT, MODE, true, 4>(lds, vq, runq, acc);
                t += 512;
            }
            if (rem & (2 / ESZ)) {
                u32 vp = reinterpret_cast<const unsigned short *>(t)[lane], vq = reinterpret_cast<const unsigned short *>(t + 128)[lane];
                consume<Act, MT, MODE, false, 2>(lds, vp, runp, acc);
                consume<Act, MT, MODE, true, 2>(lds, vq, runq, acc);
                t += 256;
            }
            if (MODE == 1 && (rem & 1)) {
                u32 vp = t[lane], vq = t[64 + lane];
                consume<Act, MT, MODE, false, 1>(lds, vp, runp, acc);
                consume<Act, MT, MODE, true, 1>(lds, vq, runq, acc);
            }
        }

#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = lanes_sum(acc[m], p.L);

        if (p.W == 1) {
            if (active && (lane & (p.L - 1)) == 0) {
                const int col = task * p.G + lane / p.L;
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    if (m0 + m < p.M) C[(size_t)(m0 + m) * p.N + col] = acc[m];
            }
        } else {
            // second pass: the W wavefronts of a column meet in a small LDS buffer
            if (lane == 0) {
#pragma unroll
                for (int m = 0; m < MT; ++m) part[wave * MT + m] = acc[m];
            }
            __syncthreads();
            if (active && lane == 0 && (wave % p.W) == 0) {
                const int col = task / p.W;
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    A s = (A)0;
                    for (int w = 0; w < p.W; ++w) s += part[(wave + w) * MT + m];
                    if (m0 + m < p.M) C[(size_t)(m0 + m) * p.N + col] = s;
                }
            }
            __syncthreads();
        }
    }
}

// ------------------------------------------------------------------- i2s GEMV
struct I2sParams {
    const uint4 *w;
    const int8_t *X;
    int *C;
    int M, K, Kp, N, rounds;
};

// Workgroup = 16 columns; wavefront `wave` takes rounds wave, wave+waves, ...;
// in a round lane (col%16)*4 + q reads 64 weights (rows 256*r + 64*q ...) of its column.
// Codes 1..3 are used as they are in dot4; the "-2" of the decode
// (bitnet_kernels.cuh:70) becomes one subtraction of 2*sum(X row) at the end.
template <int MT>
__global__ void __launch_bounds__(1024) i2s_kernel(I2sParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t *lx = reinterpret_cast<int8_t *>(smem);                       // [MT][Kp]
    int *part = reinterpret_cast<int *>(smem + (size_t)MT * p.Kp);      // [waves][16][MT]
    int *sums = part + (blockDim.x >> 6) * 16 * MT;                      // [waves][MT]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const int grp = blockIdx.x, m0 = blockIdx.y * MT;
    constexpr int RPB = 4;

    uint4 wv[RPB];
#pragma unroll
    for (int i = 0; i < RPB; ++i) {
        int r = wave + i * waves;
        wv[i] = (r < p.rounds) ? p.w[((size_t)grp * p.rounds + r) * 64 + lane] : make_uint4(0, 0, 0, 0);
    }

    // stage X rows (zero beyond M and beyond K) and accumulate the row sums on the way
    int rs[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        rs[m] = 0;
        const uint4 *src = reinterpret_cast<const uint4 *>(p.X + (size_t)(m0 + m) * p.K);
        uint4 *dst = reinterpret_cast<uint4 *>(lx + (size_t)m * p.Kp);
        for (int i = tid; i < p.Kp / 16; i += blockDim.x) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (m0 + m < p.M && i < p.K / 16) v = src[i];
            dst[i] = v;
            rs[m] = __builtin_amdgcn_sdot4((int)v.x, 0x01010101, rs[m], false);
            rs[m] = __builtin_amdgcn_sdot4((int)v.y, 0x01010101, rs[m], false);
            rs[m] = __builtin_amdgcn_sdot4((int)v.z, 0x01010101, rs[m], false);
            rs[m] = __builtin_amdgcn_sdot4((int)v.w, 0x01010101, rs[m], false);
        }
        rs[m] = lanes_sum(rs[m], 64);
        if (lane == 0) sums[wave * MT + m] = rs[m];
    }
    __syncthreads();

    int acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0;
    const int q = lane & 3;

    for (int r0 = wave;; r0 += RPB * waves) {
#pragma unroll
        for (int i = 0; i < RPB; ++i) {
            const int r = r0 + i * waves;
            if (r < p.rounds) {
                const u32 words[4] = {wv[i].x, wv[i].y, wv[i].z, wv[i].w};
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    const uint4 *xr = reinterpret_cast<const uint4 *>(lx + (size_t)m * p.Kp + 256 * r + 64 * q);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint4 x = xr[j];
                        const u32 wd = words[j];
                        acc[m] = __builtin_amdgcn_sdot4((int)x.x, (int)(wd & 0x03030303u), acc[m], false);
                        acc[m] = __builtin_amdgcn_sdot4((int)x.y, (int)((wd >> 2) & 0x03030303u), acc[m], false);
                        acc[m] = __builtin_amdgcn_sdot4((int)x.z, (int)((wd >> 4) & 0x03030303u), acc[m], false);
                        acc[m] = __builtin_amdgcn_sdot4((int)x.w, (int)((wd >> 6) & 0x03030303u), acc[m], false);
                    }
                }
            }
        }
        if (r0 + RPB * waves >= p.rounds) break;
#pragma unroll
        for (int i = 0; i < RPB; ++i) {
            int r = r0 + (RPB + i) * waves;
            wv[i] = (r < p.rounds) ? p.w[((size_t)grp * p.rounds + r) * 64 + lane] : make_uint4(0, 0, 0, 0);
        }
    }

#pragma unroll
    for (int m = 0; m < MT; ++m) {
        acc[m] = lanes_sum(acc[m], 4);
        if (q == 0) part[(wave * 16 + (lane >> 2)) * MT + m] = acc[m];
    }
    __syncthreads();
    for (int t = tid; t < 16 * MT; t += blockDim.x) {
        const int col = t / MT, m = t % MT;
        int s = 0, sx = 0;
        for (int w = 0; w < waves; ++w) {
            s += part[(w * 16 + col) * MT + m];
            sx += sums[w * MT + m];
        }
        if (m0 + m < p.M) p.C[(size_t)(m0 + m) * p.N + grp * 16 + col] = s - 2 * sx;
    }
}

__global__ void __launch_bounds__(256) copy_kernel(uint4 *dst, const uint4 *src, size_t n16)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

// ------------------------------------------------------------------ launchers
static int hip_fail(hipError_t e, const char *what)
{
    return fail(SPTMM_ERR_HIP, "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
}

// Dynamic LDS above the default cap has to be granted per kernel once.
static int grant_lds(const void *kern, size_t lds, std::atomic<size_t> &granted)
{
    if (lds <= granted.load(std::memory_order_relaxed)) return SPTMM_OK;
    hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
    granted.store(lds, std::memory_order_relaxed);
    return SPTMM_OK;
}

template <typename Act, int MT, int MODE>
static int launch_lists_t(const GemvArgs &a, hipStream_t st)
{
    // Wavefronts per workgroup: fill the CUs with one workgroup each, and when a
    // CU gets more than LISTS_MAX_WAVES tasks pick the count that wastes the
    // fewest wavefront slots over the task loop.
    const int cus = a.compute_units > 0 ? a.compute_units : 256;
    int wpb = a.W, best = 1 << 30;
    for (int w = a.W; w <= LISTS_MAX_WAVES; w += a.W) {
        int blocks = (a.tasks + w - 1) / w;
        int grid = blocks < cus ? blocks : cus;
        int iters = (blocks + grid - 1) / grid;
        int cost = iters * w;
        if (cost < best || (cost == best && w > wpb)) {
            best = cost;
            wpb = w;
        }
    }
    const int blocks = (a.tasks + wpb - 1) / wpb;
    const int grid_x = blocks < cus ? blocks : cus;
    const int iters = (blocks + grid_x - 1) / grid_x;
    ListParams p{(const uint8_t *)a.w, a.X, a.C, a.M, a.K, a.N, a.n_lane, a.tasks, a.L, a.G, a.W, iters};
    size_t lds = (((size_t)(a.K + 1) * MT * sizeof(Act) + 15) & ~(size_t)15) + (size_t)wpb * MT * sizeof(typename Acc<Act>::type);
    if ((int)lds > a.lds_limit) return fail(SPTMM_ERR_UNSUPPORTED, "activation tile of %zu bytes exceeds the LDS limit %d", lds, a.lds_limit);
    auto kern = lists_kernel<Act, MT, MODE>;
    static std::atomic<size_t> lds_granted{48 * 1024};
    if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted)) return rc;
    dim3 grid(grid_x, (a.M + MT - 1) / MT), block(64 * wpb);
    hipLaunchKernelGGL(kern, grid, block, lds, st, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : hip_fail(e, "lists_kernel launch");
}

template <typename Act, int MODE>
static int launch_lists_m(const GemvArgs &a, hipStream_t st)
{
    const size_t row = (size_t)(a.K + 1) * sizeof(Act) + 64;
    if constexpr (sizeof(Act) == 1) {
        if (a.M >= 5 && row * 8 <= (size_t)a.lds_limit) return launch_lists_t<Act, 8, MODE>(a, st);
    }
    if (a.M >= 2 && row * 4 <= (size_t)a.lds_limit) return launch_lists_t<Act, 4, MODE>(a, st);
    return launch_lists_t<Act, 1, MODE>(a, st);
}

template <int MODE>
static int launch_lists_a(const GemvArgs &a, ActType act, hipStream_t st)
{
    switch (act) {
    case ACT_I8: return launch_lists_m<int8_t, MODE>(a, st);
    case ACT_F16: return launch_lists_m<_Float16, MODE>(a, st);
    case ACT_F32: return launch_lists_m<float, MODE>(a, st);
    }
    return fail(SPTMM_ERR_INVALID, "unknown activation type");
}

int launch_u16(const GemvArgs &a, ActType act, void *stream) { return launch_lists_a<0>(a, act, (hipStream_t)stream); }

int launch_delta(const GemvArgs &a, ActType act, void *stream)
{
    if (a.delta_bits == 8) return launch_lists_a<1>(a, act, (hipStream_t)stream);
    return launch_lists_a<2>(a, act, (hipStream_t)stream);
}

template <int MT>
static int launch_i2s_t(const GemvArgs &a, hipStream_t st, int waves)
{
    const int Kp = i2s_padded_k(a.K);
    I2sParams p{(const uint4 *)a.w, (const int8_t *)a.X, (int *)a.C, a.M, a.K, Kp, a.N, Kp / 256};
    size_t lds = (size_t)MT * Kp + (size_t)waves * 16 * MT * 4 + (size_t)waves * MT * 4;
    auto kern = i2s_kernel<MT>;
    static std::atomic<size_t> lds_granted{48 * 1024};
    if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted)) return rc;
    dim3 grid(a.N / 16, (a.M + MT - 1) / MT), block(64 * waves);
    hipLaunchKernelGGL(kern, grid, block, lds, st, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : hip_fail(e, "i2s_kernel launch");
}

int launch_i2s(const GemvArgs &a, void *stream)
{
    const int Kp = i2s_padded_k(a.K), rounds = Kp / 256, groups = a.N / 16;
    int rpw = groups >= 2 * a.compute_units ? 4 : (groups >= a.compute_units ? 2 : 1);
    int waves = (rounds + rpw - 1) / rpw;
    waves = waves < 1 ? 1 : (waves > 16 ? 16 : waves);
    const size_t extra = (size_t)waves * 17 * 4;
    hipStream_t st = (hipStream_t)stream;
    if (a.M >= 5 && (size_t)8 * Kp + extra * 8 <= (size_t)a.lds_limit) return launch_i2s_t<8>(a, st, waves);
    if (a.M >= 2 && (size_t)4 * Kp + extra * 4 <= (size_t)a.lds_limit) return launch_i2s_t<4>(a, st, waves);
    if ((size_t)Kp + extra > (size_t)a.lds_limit) return fail(SPTMM_ERR_UNSUPPORTED, "K too large for the LDS activation tile");
    return launch_i2s_t<1>(a, st, waves);
}

int launch_copy(void *dst, const void *src, size_t bytes, void *stream)
{
    if (bytes % 16) return fail(SPTMM_ERR_INVALID, "copy size must be a multiple of 16 bytes");
    size_t n16 = bytes / 16;
    int blocks = (int)((n16 + 255) / 256 < 256 * 64 ? (n16 + 255) / 256 : 256 * 64);
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint4 *)dst, (const uint4 *)src, n16);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : hip_fail(e, "copy_kernel launch");
}

}  // namespace sptmm
