// gfx950 kernels of the SpTMM engine and their launchers.
//
// All three kernels are HBM-bound gather/unpack work: no multiplies on the
// list paths, packed-integer dot4 on the i2s path, no MFMA anywhere.  Common
// shape: the activation tile is staged once per workgroup in LDS (every column
// reuses it), each 64-lane wavefront streams its slice of the weight stream
// with 16-byte per-lane loads that are contiguous across the wavefront, and
// split-K partials are folded across lanes with DPP, then (when a column spans
// several wavefronts) through a small LDS buffer.  No atomics.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdlib>

#include "internal.hpp"

namespace sptmm {

typedef unsigned int u32;

// ------------------------------------------------------------------ helpers
template <typename Act> struct Acc { typedef float type; };
template <> struct Acc<int8_t> { typedef int type; };

// Bytes one row index occupies in the LDS activation tile.  Every layout keeps
// "dword address mod 32 == row index mod 32" at 4 bytes per index, which is the
// rule the host-side scheduler of the u16 stream relies on to keep the 32 lanes
// of a half-wavefront on 32 different LDS banks.
template <typename Act, int MT> __host__ __device__ constexpr int slot_bytes()
{
    return sizeof(Act) == 1 ? (MT == 1 ? 4 : MT)        // int8: one int32 (M=1), or MT packed bytes
           : sizeof(Act) == 2 ? (MT == 1 ? 4 : 2 * MT)  // fp16: one fp32 (M=1), or MT halves
                              : 4 * MT;                 // fp32
}
__host__ __device__ constexpr int ilog2(int v) { return v <= 1 ? 0 : 1 + ilog2(v >> 1); }

template <typename T, int N> struct alignas(sizeof(T) * N) Vec { T v[N]; };

// acc[m] (+|-)= X[m][k] for the slot at byte offset `addr` of the tile
template <typename Act, int MT, bool NEG>
__device__ __forceinline__ void gather(const unsigned char *lds, u32 addr, typename Acc<Act>::type (&acc)[MT])
{
    if constexpr (sizeof(Act) == 1 && MT == 1) {
        int v = *reinterpret_cast<const int *>(lds + addr);
        acc[0] = NEG ? acc[0] - v : acc[0] + v;
    } else if constexpr (sizeof(Act) == 1) {
        Vec<int, MT / 4> r = *reinterpret_cast<const Vec<int, MT / 4> *>(lds + addr);
#pragma unroll
        for (int m = 0; m < MT; ++m)  // dot4 with a one-hot (+1 or -1) selector: no unpacking
            acc[m] = __builtin_amdgcn_sdot4(r.v[m / 4], (NEG ? 0xff : 0x01) << (8 * (m % 4)), acc[m], false);
    } else if constexpr (sizeof(Act) == 2 && MT > 1) {
        Vec<_Float16, MT> r = *reinterpret_cast<const Vec<_Float16, MT> *>(lds + addr);
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = NEG ? acc[m] - (float)r.v[m] : acc[m] + (float)r.v[m];
    } else {
        Vec<float, MT> r = *reinterpret_cast<const Vec<float, MT> *>(lds + addr);
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = NEG ? acc[m] - r.v[m] : acc[m] + r.v[m];
    }
}

// MODE 0: fields are u16 row indices (already multiplied by 4 when PRE).
// MODE 1 / 2: fields are 8- / 16-bit gaps added to a running row index.
// Consumes the low NBYTES of `d`.
template <typename Act, int MT, int MODE, bool PRE, bool NEG, int NBYTES>
__device__ __forceinline__ void consume(const unsigned char *lds, u32 d, u32 &run, typename Acc<Act>::type (&acc)[MT])
{
    constexpr int SH = ilog2(slot_bytes<Act, MT>());
    if constexpr (MODE == 1) {
#pragma unroll
        for (int b = 0; b < NBYTES; ++b) {
            run += (d >> (8 * b)) & 0xffu;
            gather<Act, MT, NEG>(lds, run << SH, acc);
        }
    } else {
#pragma unroll
        for (int h = 0; h < NBYTES / 2; ++h) {
            u32 f = h ? (d >> 16) : (d & 0xffffu);
            if constexpr (MODE == 2) {
                run += f;
                gather<Act, MT, NEG>(lds, run << SH, acc);
            } else {
                gather<Act, MT, NEG>(lds, f << (PRE ? SH - 2 : SH), acc);
            }
        }
    }
}

template <typename Act, int MT, int MODE, bool PRE, bool NEG>
__device__ __forceinline__ void consume16(const unsigned char *lds, const uint4 &v, u32 &run, typename Acc<Act>::type (&acc)[MT])
{
    consume<Act, MT, MODE, PRE, NEG, 4>(lds, v.x, run, acc);
    consume<Act, MT, MODE, PRE, NEG, 4>(lds, v.y, run, acc);
    consume<Act, MT, MODE, PRE, NEG, 4>(lds, v.z, run, acc);
    consume<Act, MT, MODE, PRE, NEG, 4>(lds, v.w, run, acc);
}

// 4 rows x 4 consecutive k (one dword per row) -> 4 dwords, dword j = the 4 rows at k+j
__device__ __forceinline__ void transpose4x4(u32 r0, u32 r1, u32 r2, u32 r3, u32 (&o)[4])
{
    u32 a = __builtin_amdgcn_perm(r1, r0, 0x05010400u), b = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
    u32 c = __builtin_amdgcn_perm(r3, r2, 0x05010400u), d = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    o[0] = __builtin_amdgcn_perm(c, a, 0x05040100u);
    o[1] = __builtin_amdgcn_perm(c, a, 0x07060302u);
    o[2] = __builtin_amdgcn_perm(d, b, 0x05040100u);
    o[3] = __builtin_amdgcn_perm(d, b, 0x07060302u);
}

__device__ __forceinline__ u32 comp(const uint4 &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }
__device__ __forceinline__ u32 f2u(float f) { return __builtin_bit_cast(u32, f); }
__device__ __forceinline__ float h2f(u32 d, int hi) { return (float)__builtin_bit_cast(_Float16, (unsigned short)(hi ? d >> 16 : d & 0xffffu)); }

// Staging of the activation tile, in items of 16 consecutive k for all MT rows.
// load() pulls an item into registers (rows past M read as zero); store()
// converts / transposes it into the tile.  Split so that the global loads of X
// can be issued ahead of the weight-stream loads and consumed behind them.
template <typename Act, int MT> struct Stager {
    static constexpr int NLOAD = MT * (int)sizeof(Act);  // 16-byte loads per item
    static constexpr int XI = NLOAD >= 8 ? 1 : 2;       // items per thread staged ahead of the stream (more fall to a loop)

    static __device__ __forceinline__ void load(const Act *X, int M, int K, int m0, int item, uint4 (&r)[NLOAD])
    {
        constexpr int PER = (int)sizeof(Act);  // 16-byte chunks per row per item
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < PER; ++j)
                r[m * PER + j] = (m0 + m < M)
                                     ? reinterpret_cast<const uint4 *>(X + (size_t)(m0 + m) * K)[(size_t)item * PER + j]
                                     : make_uint4(0, 0, 0, 0);
    }

    static __device__ __forceinline__ void store(unsigned char *lds, int item, const uint4 (&r)[NLOAD])
    {
        uint4 *t = reinterpret_cast<uint4 *>(lds);
        if constexpr (sizeof(Act) == 1 && MT == 1) {  // 16 bytes -> 16 sign-extended dwords
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int d = (int)comp(r[0], j);
                t[4 * item + j] = make_uint4((u32)((d << 24) >> 24), (u32)((d << 16) >> 24), (u32)((d << 8) >> 24), (u32)(d >> 24));
            }
        } else if constexpr (sizeof(Act) == 1) {  // [k][MT bytes]
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32 o[4], q[4];
                transpose4x4(comp(r[0], j), comp(r[1], j), comp(r[2], j), comp(r[3], j), o);
                if constexpr (MT == 4) {
                    t[4 * item + j] = make_uint4(o[0], o[1], o[2], o[3]);
                } else {
                    transpose4x4(comp(r[4], j), comp(r[5], j), comp(r[6], j), comp(r[7], j), q);
                    t[2 * (4 * item + j)] = make_uint4(o[0], q[0], o[1], q[1]);
                    t[2 * (4 * item + j) + 1] = make_uint4(o[2], q[2], o[3], q[3]);
                }
            }
        } else if constexpr (sizeof(Act) == 2 && MT == 1) {  // 16 halves -> 16 floats
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32 d0 = comp(r[j / 2], (2 * j) % 4), d1 = comp(r[j / 2], (2 * j + 1) % 4);
                t[4 * item + j] = make_uint4(f2u(h2f(d0, 0)), f2u(h2f(d0, 1)), f2u(h2f(d1, 0)), f2u(h2f(d1, 1)));
            }
        } else if constexpr (sizeof(Act) == 2) {  // MT == 4: [k][4 halves]; r[2m+h] = row m, halves 8h..8h+7
#pragma unroll
            for (int i = 0; i < 8; ++i) {  // k = 16*item + 2i, 2i+1
                u32 d[4];
#pragma unroll
                for (int m = 0; m < 4; ++m) d[m] = comp(r[2 * m + i / 4], i % 4);
                t[8 * item + i] = make_uint4((d[0] & 0xffffu) | (d[1] << 16), (d[2] & 0xffffu) | (d[3] << 16),
                                             (d[0] >> 16) | (d[1] & 0xffff0000u), (d[2] >> 16) | (d[3] & 0xffff0000u));
            }
        } else if constexpr (MT == 1) {  // fp32 copy
#pragma unroll
            for (int j = 0; j < 4; ++j) t[4 * item + j] = r[j];
        } else {  // fp32, MT == 4: [k][4 floats]; r[4m+j] = row m, k = 16*item + 4j ..
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    t[16 * item + 4 * j + i] = make_uint4(comp(r[j], i), comp(r[4 + j], i), comp(r[8 + j], i), comp(r[12 + j], i));
        }
    }
};

template <int CTRL> __device__ __forceinline__ int dpp(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false); }
template <int CTRL> __device__ __forceinline__ float dpp(float v) { return __builtin_bit_cast(float, dpp<CTRL>(__builtin_bit_cast(int, v))); }
__device__ __forceinline__ int swz16(int v) { return __builtin_amdgcn_ds_swizzle(v, 0x401f); }  // lane ^ 16
__device__ __forceinline__ float swz16(float v) { return __builtin_bit_cast(float, swz16(__builtin_bit_cast(int, v))); }

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

struct ListParams {
    const uint8_t *w;
    const void *X;
    void *C;
    int M, K, N;
    int n_lane, tasks, logL, W;
    int iters;  // tasks each wavefront walks: ceil(tasks / (gridDim.x * waves))
};

constexpr int LISTS_MAX_WAVES = 8;  // 512 threads: two wavefronts per SIMD, 256 VGPRs each

// One round of a task's stream: 16 bytes per lane of the +1 list and of the -1 list.
struct Round {
    uint4 p, q;
};
// The stream is read exactly once per GEMV: non-temporal loads keep it from
// pushing the activation vector (re-read by every workgroup) out of L2.
typedef u32 v4u __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 stream_load(const uint4 *p)
{
#ifdef SPTMM_NO_NT
    return *p;
#else
    v4u t = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
#endif
}
__device__ __forceinline__ Round load_round(const uint4 *wp, int r)
{
    Round x;
    x.p = stream_load(wp + (2 * r) * 64);
    x.q = stream_load(wp + (2 * r + 1) * 64);
    return x;
}

template <typename Act, int MT, int MODE, bool PRE>
struct ListsBody {
    typedef typename Acc<Act>::type A;
    typedef Stager<Act, MT> St;
    static constexpr int ESZ = (MODE == 1) ? 1 : 2;   // bytes per stream entry
    static constexpr int E16 = 16 / ESZ;              // entries per 16-byte load
    static constexpr int HDR = MODE ? 256 : 0;        // restart indices of a gap-stream task
    static constexpr int SLOT = slot_bytes<Act, MT>();
    static constexpr int CH = 4;                      // rounds per chunk of the generic path
#ifndef SPTMM_EARLY
#define SPTMM_EARLY 2
#endif
    static constexpr int EARLY = SPTMM_EARLY;         // rounds requested before the activation tile is complete

    static __device__ __forceinline__ void eat(const unsigned char *smem, const Round &x, u32 &runp, u32 &runq, A (&acc)[MT])
    {
        consume16<Act, MT, MODE, PRE, false>(smem, x.p, runp, acc);
        consume16<Act, MT, MODE, PRE, true>(smem, x.q, runq, acc);
    }

    // RF > 0: the task has exactly RF full rounds and all of them live in
    // registers, loaded and consumed in straight-line code (so every wait on the
    // stream is for one round only).  RF == 0: any number of rounds, walked in
    // double-buffered chunks of CH.
    template <int RF>
    static __device__ __forceinline__ void run(const ListParams &p, unsigned char *smem)
    {
        constexpr int NB = RF > 0 ? RF : 2 * CH;
        A *part = reinterpret_cast<A *>(smem + (((size_t)(p.K + 1) * SLOT + 15) & ~(size_t)15));
        const int tid = threadIdx.x, nt = blockDim.x;
        const int lane = tid & 63, wave = tid >> 6, waves = nt >> 6;
        const int m0 = blockIdx.y * MT;
        const size_t task_bytes = HDR + (size_t)128 * ESZ * p.n_lane;
        const int R = p.n_lane / E16, nchunk = R / CH;
        int task = blockIdx.x * waves + wave;
        const int task_step = gridDim.x * waves;
        const Act *X = reinterpret_cast<const Act *>(p.X);

        // 1. every wavefront's activation loads enter the memory pipeline ahead of
        //    any stream load of the workgroup ...
        const int items = p.K / 16;
        uint4 xr[St::XI][St::NLOAD];
#pragma unroll
        for (int i = 0; i < St::XI; ++i) {
            const int item = tid + i * nt;
            St::load(X, p.M, p.K, m0, item < items ? item : items - 1, xr[i]);
        }
#ifdef SPTMM_XBARRIER
        __builtin_amdgcn_s_barrier();
#endif

        // 2. ... then the first rounds of the first task's stream ...
        Round buf[NB];
        {
            const uint4 *wp = reinterpret_cast<const uint4 *>(p.w + (size_t)(task < p.tasks ? task : 0) * task_bytes + HDR) + lane;
            if constexpr (RF > 0) {
#pragma unroll
                for (int i = 0; i < (RF < EARLY ? RF : EARLY); ++i) buf[i] = load_round(wp, i);
            } else {
                if (nchunk > 0) {
#pragma unroll
                    for (int i = 0; i < CH; ++i) buf[i] = load_round(wp, i);
                }
                if (nchunk > 1) {
#pragma unroll
                    for (int i = 0; i < CH; ++i) buf[CH + i] = load_round(wp, CH + i);
                }
            }
        }

        // 3. ... and the tile is written while the stream is still in flight.
#pragma unroll
        for (int i = 0; i < St::XI; ++i)
            if (tid + i * nt < items) St::store(smem, tid + i * nt, xr[i]);
        if constexpr (RF > EARLY) {
            const uint4 *wp = reinterpret_cast<const uint4 *>(p.w + (size_t)(task < p.tasks ? task : 0) * task_bytes + HDR) + lane;
#pragma unroll
            for (int i = EARLY; i < RF; ++i) buf[i] = load_round(wp, i);
        }
        for (int item = tid + St::XI * nt; item < items; item += nt) {
            uint4 r[St::NLOAD];
            St::load(X, p.M, p.K, m0, item, r);
            St::store(smem, item, r);
        }
        if (tid < SLOT / 4) reinterpret_cast<u32 *>(smem + (size_t)p.K * SLOT)[tid] = 0u;  // slot K reads as zero
        __syncthreads();

        A *C = reinterpret_cast<A *>(p.C);
        const int L = 1 << p.logL;
        for (int it = 0; it < p.iters; ++it, task += task_step) {
            const bool active = task < p.tasks;
            const uint8_t *tb = p.w + (size_t)(active ? task : 0) * task_bytes;
            const uint4 *wp = reinterpret_cast<const uint4 *>(tb + HDR) + lane;
            u32 runp = 0, runq = 0;
            if constexpr (MODE != 0) {
                const unsigned short *rs = reinterpret_cast<const unsigned short *>(tb);
                runp = rs[lane];
                runq = rs[64 + lane];
            }
            A acc[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) acc[m] = (A)0;

            if constexpr (RF > 0) {
                if (it > 0) {
#pragma unroll
                    for (int i = 0; i < RF; ++i) buf[i] = load_round(wp, i);
                }
#pragma unroll
                for (int i = 0; i < RF; ++i) eat(smem, buf[i], runp, runq, acc);
            } else {
                if (it > 0) {
                    if (nchunk > 0) {
#pragma unroll
                        for (int i = 0; i < CH; ++i) buf[i] = load_round(wp, i);
                    }
                    if (nchunk > 1) {
#pragma unroll
                        for (int i = 0; i < CH; ++i) buf[CH + i] = load_round(wp, CH + i);
                    }
                }
                int c = 0;
                for (; c + 3 < nchunk; c += 2) {  // steady state: eat a chunk, refill it two chunks ahead
#pragma unroll
                    for (int i = 0; i < CH; ++i) eat(smem, buf[i], runp, runq, acc);
#pragma unroll
                    for (int i = 0; i < CH; ++i) buf[i] = load_round(wp, (c + 2) * CH + i);
#pragma unroll
                    for (int i = 0; i < CH; ++i) eat(smem, buf[CH + i], runp, runq, acc);
#pragma unroll
                    for (int i = 0; i < CH; ++i) buf[CH + i] = load_round(wp, (c + 3) * CH + i);
                }
                const int left = nchunk - c;  // 0..3 chunks, the first two already in registers
                if (left >= 1) {
#pragma unroll
                    for (int i = 0; i < CH; ++i) eat(smem, buf[i], runp, runq, acc);
                }
                if (left == 3) {
#pragma unroll
                    for (int i = 0; i < CH; ++i) buf[i] = load_round(wp, (c + 2) * CH + i);
                }
                if (left >= 2) {
#pragma unroll
                    for (int i = 0; i < CH; ++i) eat(smem, buf[CH + i], runp, runq, acc);
                }
                if (left == 3) {
#pragma unroll
                    for (int i = 0; i < CH; ++i) eat(smem, buf[i], runp, runq, acc);
                }
                for (int r = nchunk * CH; r < R; ++r) {
                    Round x = load_round(wp, r);
                    eat(smem, x, runp, runq, acc);
                }
            }
            // ragged tail: at most one round each of 8, 4, 2 (and 1) bytes per lane
            const int rem = p.n_lane - R * E16;
            if (rem) {
                const uint8_t *t = tb + HDR + (size_t)R * 2048;
                if (rem & (8 / ESZ)) {
                    uint2 vp = reinterpret_cast<const uint2 *>(t)[lane], vq = reinterpret_cast<const uint2 *>(t + 512)[lane];
                    consume<Act, MT, MODE, PRE, false, 4>(smem, vp.x, runp, acc);
                    consume<Act, MT, MODE, PRE, false, 4>(smem, vp.y, runp, acc);
                    consume<Act, MT, MODE, PRE, true, 4>(smem, vq.x, runq, acc);
                    consume<Act, MT, MODE, PRE, true, 4>(smem, vq.y, runq, acc);
                    t += 1024;
                }
                if (rem & (4 / ESZ)) {
                    u32 vp = reinterpret_cast<const u32 *>(t)[lane], vq = reinterpret_cast<const u32 *>(t + 256)[lane];
                    consume<Act, MT, MODE, PRE, false, 4>(smem, vp, runp, acc);
                    consume<Act, MT, MODE, PRE, true, 4>(smem, vq, runq, acc);
                    t += 512;
                }
                if (rem & (2 / ESZ)) {
                    u32 vp = reinterpret_cast<const unsigned short *>(t)[lane], vq = reinterpret_cast<const unsigned short *>(t + 128)[lane];
                    consume<Act, MT, MODE, PRE, false, 2>(smem, vp, runp, acc);
                    consume<Act, MT, MODE, PRE, true, 2>(smem, vq, runq, acc);
                    t += 256;
                }
                if constexpr (MODE == 1) {
                    if (rem & 1) {
                        u32 vp = t[lane], vq = t[64 + lane];
                        consume<Act, MT, MODE, PRE, false, 1>(smem, vp, runp, acc);
                        consume<Act, MT, MODE, PRE, true, 1>(smem, vq, runq, acc);
                    }
                }
            }

#pragma unroll
            for (int m = 0; m < MT; ++m) acc[m] = lanes_sum(acc[m], p.logL);

            if (p.W == 1) {
                if (active && (lane & (L - 1)) == 0) {
                    const int col = (task << (6 - p.logL)) + (lane >> p.logL);
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
                if (active && lane == 0 && (wave & (p.W - 1)) == 0) {
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
};

// ------------------------------------------------- index-list / gap-stream GEMV
// One task = one wavefront's share of the stream: 64/L columns x L lanes, or one
// 64-lane part of a column.  A workgroup stages the activation tile once and its
// wavefronts then walk tasks blockIdx.x*waves + wave, + gridDim.x*waves, ...
// blockIdx.y selects the tile of MT activation rows.  FIXED kernels carry the
// straight-line bodies for tasks of 1, 2, 3, 4, 6 or 8 rounds; other sizes (and
// all kernels built without FIXED) take the chunked loop.
template <typename Act, int MT, int MODE, bool PRE, bool FIXED>
__global__ void __launch_bounds__(64 * LISTS_MAX_WAVES) lists_kernel(ListParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    typedef ListsBody<Act, MT, MODE, PRE> B;
    if constexpr (FIXED) {
        switch (p.n_lane / B::E16) {
        case 1: B::template run<1>(p, smem); return;
        case 2: B::template run<2>(p, smem); return;
        case 3: B::template run<3>(p, smem); return;
        case 4: B::template run<4>(p, smem); return;
        case 6: B::template run<6>(p, smem); return;
        case 8: B::template run<8>(p, smem); return;
        default: break;
        }
    }
    B::template run<0>(p, smem);
}

// Several independent GEMVs of one shape in one launch: blockIdx.z picks the
// (stream, activations, output) triple, everything else is the kernel above.
constexpr int BATCH_MAX = 32;
struct BatchPtrs {
    const uint8_t *w[BATCH_MAX];
    const void *X[BATCH_MAX];
    void *C[BATCH_MAX];
};

template <typename Act, int MT, int MODE, bool PRE, bool FIXED>
__global__ void __launch_bounds__(64 * LISTS_MAX_WAVES) lists_kernel_batched(ListParams p, BatchPtrs b)
{
    extern __shared__ __align__(16) unsigned char smem[];
    typedef ListsBody<Act, MT, MODE, PRE> B;
    p.w = b.w[blockIdx.z];
    p.X = b.X[blockIdx.z];
    p.C = b.C[blockIdx.z];
    if constexpr (FIXED) {
        switch (p.n_lane / B::E16) {
        case 1: B::template run<1>(p, smem); return;
        case 2: B::template run<2>(p, smem); return;
        case 3: B::template run<3>(p, smem); return;
        case 4: B::template run<4>(p, smem); return;
        case 6: B::template run<6>(p, smem); return;
        case 8: B::template run<8>(p, smem); return;
        default: break;
        }
    }
    B::template run<0>(p, smem);
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
        rs[m] = lanes_sum(rs[m], 6);
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
        acc[m] = lanes_sum(acc[m], 2);
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

template <typename Act, int MT, int MODE, bool PRE>
static int launch_lists_t(const GemvArgs &a, hipStream_t st)
{
    // Wavefronts per workgroup: fill the CUs with one workgroup each, and when a
    // CU gets more than LISTS_MAX_WAVES tasks pick the count that wastes the
    // fewest wavefront slots over the task loop.
    const int cus = a.compute_units > 0 ? a.compute_units : 256;
    static const int tune_wpb = getenv("SPTMM_WAVES_PER_WG") ? atoi(getenv("SPTMM_WAVES_PER_WG")) : 0;
    static const int tune_wgs = getenv("SPTMM_WGS_PER_CU") ? atoi(getenv("SPTMM_WGS_PER_CU")) : 1;
    const int slots = cus * (tune_wgs > 0 ? tune_wgs : 1);  // workgroups resident at once
    int wpb = a.W, best = 1 << 30;
    for (int w = a.W; w <= LISTS_MAX_WAVES; w += a.W) {
        int blocks = (a.tasks + w - 1) / w;
        int grid = blocks < slots ? blocks : slots;
        int iters = (blocks + grid - 1) / grid;
        int cost = iters * w;
        if (cost < best || (cost == best && w > wpb)) {
            best = cost;
            wpb = w;
        }
    }
    if (tune_wpb > 0 && tune_wpb <= LISTS_MAX_WAVES && tune_wpb % a.W == 0) wpb = tune_wpb;
    const int blocks = (a.tasks + wpb - 1) / wpb;
    const int grid_x = blocks < slots ? blocks : slots;
    const int iters = (blocks + grid_x - 1) / grid_x;
    ListParams p{(const uint8_t *)a.w, a.X, a.C, a.M, a.K, a.N, a.n_lane, a.tasks, ilog2(a.L), a.W, iters};
    constexpr int SLOT = slot_bytes<Act, MT>();
    size_t lds = (((size_t)(a.K + 1) * SLOT + 15) & ~(size_t)15) + (size_t)wpb * MT * sizeof(typename Acc<Act>::type);
    if ((int)lds > a.lds_limit) return fail(SPTMM_ERR_UNSUPPORTED, "activation tile of %zu bytes exceeds the LDS limit %d", lds, a.lds_limit);
    // straight-line bodies for the int8 paths of the u16 and 8-bit gap streams
    constexpr bool FIXED = sizeof(Act) == 1 && MODE != 2;
    dim3 grid(grid_x, (a.M + MT - 1) / MT), block(64 * wpb);
    if (a.batch) {
        if constexpr (sizeof(Act) == 1) {
            auto kern = lists_kernel_batched<Act, MT, MODE, PRE, FIXED>;
            static std::atomic<size_t> lds_granted_b{48 * 1024};
            if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted_b)) return rc;
            for (int first = 0; first < a.batch; first += BATCH_MAX) {
                BatchPtrs b{};
                const int n = a.batch - first < BATCH_MAX ? a.batch - first : BATCH_MAX;
                for (int i = 0; i < n; ++i) {
                    b.w[i] = (const uint8_t *)a.batch_w[first + i];
                    b.X[i] = a.batch_X[first + i];
                    b.C[i] = a.batch_C[first + i];
                }
                grid.z = n;
                hipLaunchKernelGGL(kern, grid, block, lds, st, p, b);
                hipError_t e = hipGetLastError();
                if (e != hipSuccess) return hip_fail(e, "lists_kernel_batched launch");
            }
            return SPTMM_OK;
        } else {
            return fail(SPTMM_ERR_UNSUPPORTED, "batched launches take int8 activations");
        }
    }
    auto kern = lists_kernel<Act, MT, MODE, PRE, FIXED>;
    static std::atomic<size_t> lds_granted{48 * 1024};
    if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted)) return rc;
    hipLaunchKernelGGL(kern, grid, block, lds, st, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : hip_fail(e, "lists_kernel launch");
}

template <typename Act, int MODE, bool PRE>
static int launch_lists_m(const GemvArgs &a, hipStream_t st)
{
    const size_t lim = (size_t)a.lds_limit - 256;
    if constexpr (sizeof(Act) == 1) {
        if (a.M >= 5 && (size_t)(a.K + 1) * slot_bytes<Act, 8>() <= lim) return launch_lists_t<Act, 8, MODE, PRE>(a, st);
    }
    if (a.M >= 2 && (size_t)(a.K + 1) * slot_bytes<Act, 4>() <= lim) return launch_lists_t<Act, 4, MODE, PRE>(a, st);
    return launch_lists_t<Act, 1, MODE, PRE>(a, st);
}

template <int MODE, bool PRE>
static int launch_lists_a(const GemvArgs &a, ActType act, hipStream_t st)
{
    switch (act) {
    case ACT_I8: return launch_lists_m<int8_t, MODE, PRE>(a, st);
    case ACT_F16: return launch_lists_m<_Float16, MODE, PRE>(a, st);
    case ACT_F32: return launch_lists_m<float, MODE, PRE>(a, st);
    }
    return fail(SPTMM_ERR_INVALID, "unknown activation type");
}

int launch_u16(const GemvArgs &a, ActType act, void *stream)
{
    if (a.index_shift == 2) return launch_lists_a<0, true>(a, act, (hipStream_t)stream);
    return launch_lists_a<0, false>(a, act, (hipStream_t)stream);
}

int launch_delta(const GemvArgs &a, ActType act, void *stream)
{
    if (a.delta_bits == 8) return launch_lists_a<1, false>(a, act, (hipStream_t)stream);
    return launch_lists_a<2, false>(a, act, (hipStream_t)stream);
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
