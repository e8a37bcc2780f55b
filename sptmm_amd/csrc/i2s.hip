// i2s (2-bit packed dense ternary) GEMV, the copy kernel, and the dispatch of the
// list-stream launchers that live in their own translation units.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdlib>

#include "internal.hpp"
#include "lanes.hpp"

namespace sptmm {

typedef unsigned int u32;

// ------------------------------------------------------------------- i2s GEMV
struct I2sParams {
    const uint4 *w;
    const int8_t *X;
    int *C;
    int M, K, Kp, N, rounds;
    int threads;  // blockDim.x as an argument (the built-in costs two memory round trips in a row at kernel start)
};

// Workgroup = 16 columns; wavefront `wave` takes rounds wave, wave+waves, ...;
// in a round lane q*16 + col%16 reads 64 weights (rows 256*r + 64*q ...) of its column.
// Codes 1..3 are used as they are in dot4; the "-2" of the decode
// (bitnet_kernels.cuh:70) becomes one subtraction of 2*sum(X row) at the end.
template <int MT>
__device__ __forceinline__ void i2s_body(const I2sParams &p, unsigned char *smem)
{
    int8_t *lx = reinterpret_cast<int8_t *>(smem);                       // [MT][Kp]
    int *part = reinterpret_cast<int *>(smem + (size_t)MT * p.Kp);      // [waves][16][MT]
    int *sums = part + (p.threads >> 6) * 16 * MT;                      // [waves][MT]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = p.threads >> 6;
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
        for (int i = tid; i < p.Kp / 16; i += p.threads) {
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
    const int q = lane >> 4;

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
        acc[m] += swz16(acc[m]);               // the four quarters of a column sit 16 lanes apart
        acc[m] += __shfl_xor(acc[m], 32, 64);
        if (q == 0) part[(wave * 16 + lane) * MT + m] = acc[m];
    }
    __syncthreads();
    for (int t = tid; t < 16 * MT; t += p.threads) {
        const int col = t / MT, m = t % MT;
        int s = 0, sx = 0;
        for (int w = 0; w < waves; ++w) {
            s += part[(w * 16 + col) * MT + m];
            sx += sums[w * MT + m];
        }
        if (m0 + m < p.M) p.C[(size_t)(m0 + m) * p.N + grp * 16 + col] = s - 2 * sx;
    }
}

template <int MT>
__global__ void __launch_bounds__(1024) i2s_kernel(I2sParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    i2s_body<MT>(p, smem);
}

// Several independent GEMVs of one shape in one launch: blockIdx.z picks the (stream, X, C) triple.
constexpr int I2S_BATCH_MAX = 32;
struct I2sBatch {
    const uint4 *w[I2S_BATCH_MAX];
    const int8_t *X[I2S_BATCH_MAX];
    int *C[I2S_BATCH_MAX];
};

template <int MT>
__global__ void __launch_bounds__(1024) i2s_kernel_batched(I2sParams p, I2sBatch b)
{
    extern __shared__ __align__(16) unsigned char smem[];
    p.w = b.w[blockIdx.z];
    p.X = b.X[blockIdx.z];
    p.C = b.C[blockIdx.z];
    i2s_body<MT>(p, smem);
}

// The same product on the matrix unit, for any number of activation rows (tiles of 16 on blockIdx.y).
// One v_mfma_i32_16x16x64_i8 multiplies 16 rows x 64 k of X with 64 k x 16 columns of W: lane
// g*16 + i hands over X[row i][16 k of k-block g] as A and, for column i, the 16 codes of the same k as B
// -- one 32-bit word of the stream, spread to bytes by four shift-and-mask pairs (codes 1..3 as they
// are).  A second product against a B of all ones gives the row sums of X in the same register layout,
// so the "-2" of the decode is D - 2*D1 per lane.
//
// The wavefronts of a workgroup split K, so no two of them want the same X bytes.  Each reads the
// X of its round with coalesced loads (lane = 16 bytes of one row, 16 lanes = 256 consecutive bytes) and
// turns it into operand order -- 16 lanes = the same 16 k of 16 rows -- through a 4 KiB LDS patch of
// its own: written and read back by the same wavefront, so no barrier; 16-byte units are placed at
// (k16, row ^ k16) so that neither the writes (lanes differ in k16) nor the reads (lanes differ in row)
// meet on a bank.  Reading the operands straight from global memory costs the texture unit a cache
// line per lane and was three times slower.  XJ = ceil(rows / 4): loads of rows nobody stores are left out.
typedef int v4i __attribute__((ext_vector_type(4)));
typedef u32 v4u __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32 comp4(const uint4 &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }

// CT = column tiles (of 16) a wavefront multiplies with the same X operands: what a workgroup reads
// of X (rows x K bytes, from L2) is shared by 16 CT columns, and with 16 rows and CT = 1 that traffic is
// four times the weight stream's and sets the time.
template <int XJ, int CT> struct I2sRound {
    uint4 w[CT];   // 64 codes of this lane's column in each tile
    uint4 x[XJ];   // 16 bytes of row 4j + lane/16 at k = 256 r + 16 (lane % 16)
};

// Every load is unconditional (a load behind a branch makes each later wait on the stream a wait for
// everything in flight).  A round past the end reads 16 hot bytes of X in place of weights and is never
// multiplied; rows past M read row M-1 (their products land in result rows nobody stores); the k
// past K of the last round read the last 16 k of the row (their weights are padding, code 2 = zero,
// and a zero weight takes any activation: 2x - 2x).
template <int XJ, int CT>
__device__ __forceinline__ I2sRound<XJ, CT> i2s_load_round(const I2sParams &p, const uint4 *const (&wbase)[CT], const int8_t *const (&xrow)[XJ], int r,
                                                          int lane)
{
    I2sRound<XJ, CT> o;
    const bool real = r < p.rounds;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
        const uint4 *src = real ? wbase[c] + (size_t)r * 64 + lane : reinterpret_cast<const uint4 *>(p.X);
        const v4u t = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(src));
        o.w[c] = make_uint4(t.x, t.y, t.z, t.w);
    }
    int k = 256 * (real ? r : p.rounds - 1) + 16 * (lane & 15);
    k = k < p.K ? k : p.K - 16;
#pragma unroll
    for (int j = 0; j < XJ; ++j) o.x[j] = *reinterpret_cast<const uint4 *>(xrow[j] + k);
    return o;
}

template <int XJ, int CT>
__device__ __forceinline__ void i2s_mfma_round(const I2sRound<XJ, CT> &o, unsigned char *patch, const u32 (&woff)[XJ], const u32 (&roff)[4],
                                               v4i (&D)[CT], v4i &D1)
{
#pragma unroll
    for (int j = 0; j < XJ; ++j) *reinterpret_cast<uint4 *>(patch + woff[j]) = o.x[j];
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
    uint4 xa[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) xa[j] = *reinterpret_cast<const uint4 *>(patch + roff[j]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const v4i a = {(int)xa[j].x, (int)xa[j].y, (int)xa[j].z, (int)xa[j].w};
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            const u32 wd = comp4(o.w[c], j);
            const v4i b = {(int)(wd & 0x03030303u), (int)((wd >> 2) & 0x03030303u), (int)((wd >> 4) & 0x03030303u), (int)((wd >> 6) & 0x03030303u)};
            D[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, D[c], 0, 0, 0);
        }
        D1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, ones, D1, 0, 0, 0);
    }
}

template <int XJ, int CT>
__device__ __forceinline__ void i2s_mfma_body(const I2sParams &p, unsigned char *smem)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = p.threads >> 6;
    const int m0 = blockIdx.y * 16, groups = p.N / 16;
    unsigned char *patch = smem + (size_t)wave * (CT > 4 ? CT : 4) * 1024;  // this wavefront's 16 rows x 256 k (and its sums at the end)
    const int8_t *xrow[XJ];
    u32 woff[XJ], roff[4];
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const int rt = 4 * j + (lane >> 4), row = m0 + rt, c = lane & 15;
        xrow[j] = p.X + (size_t)(row < p.M ? row : p.M - 1) * p.K;
        woff[j] = (u32)(c * 16 + (rt ^ c)) * 16u;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int c = 4 * (lane >> 4) + j;  // this lane's word j holds rows 256 r + 64 (lane / 16) + 16 j ..
        roff[j] = (u32)(c * 16 + ((lane & 15) ^ c)) * 16u;
    }
    const uint4 *wbase[CT];  // a tile past the last group repeats the last one (and is not stored)
#pragma unroll
    for (int c = 0; c < CT; ++c) {
        const int g = blockIdx.x * CT + c;
        wbase[c] = p.w + (size_t)(g < groups ? g : groups - 1) * p.rounds * 64;
    }
    constexpr int DEPTH = CT >= 8 ? 2 : CT >= 4 ? 3 : 4;  // rounds in flight per wavefront
    const int T = (p.rounds + waves - 1) / waves;   // steps every wavefront makes; step t of this one is round wave + t*waves

    v4i D[CT], D1 = {0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < CT; ++c) D[c] = v4i{0, 0, 0, 0};
    I2sRound<XJ, CT> buf[DEPTH];
#pragma unroll
    for (int i = 0; i < DEPTH; ++i) buf[i] = i2s_load_round<XJ, CT>(p, wbase, xrow, wave + i * waves, lane);
    int base = 0;
    for (; base + DEPTH < T; base += DEPTH) {
#pragma unroll
        for (int i = 0; i < DEPTH; ++i) {
            if (wave + (base + i) * waves < p.rounds) i2s_mfma_round<XJ, CT>(buf[i], patch, woff, roff, D, D1);  // (uniform per wavefront)
            buf[i] = i2s_load_round<XJ, CT>(p, wbase, xrow, wave + (base + DEPTH + i) * waves, lane);
        }
    }
#pragma unroll
    for (int i = 0; i < DEPTH; ++i)
        if (wave + (base + i) * waves < p.rounds) i2s_mfma_round<XJ, CT>(buf[i], patch, woff, roff, D, D1);
    // lane g*16 + j holds rows 4g .. 4g+3 of column j of every tile; the wavefronts' sums meet in their patches
    int *part = reinterpret_cast<int *>(patch);
#pragma unroll
    for (int c = 0; c < CT; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) part[c * 256 + (4 * (lane >> 4) + r) * 16 + (lane & 15)] = D[c][r] - 2 * D1[r];
    __syncthreads();
    for (int t = tid; t < 256 * CT; t += p.threads) {
        int s = 0;
        for (int w = 0; w < waves; ++w) s += reinterpret_cast<const int *>(smem + (size_t)w * (CT > 4 ? CT : 4) * 1024)[t];
        const int m = m0 + ((t & 255) >> 4), g = blockIdx.x * CT + (t >> 8);
        if (m < p.M && g < groups) p.C[(size_t)m * p.N + g * 16 + (t & 15)] = s;
    }
}

template <int XJ, int CT>
__global__ void __launch_bounds__(512) i2s_mfma_kernel(I2sParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    i2s_mfma_body<XJ, CT>(p, smem);
}

template <int XJ, int CT>
__global__ void __launch_bounds__(512) i2s_mfma_kernel_batched(I2sParams p, I2sBatch b)
{
    extern __shared__ __align__(16) unsigned char smem[];
    p.w = b.w[blockIdx.z];
    p.X = b.X[blockIdx.z];
    p.C = b.C[blockIdx.z];
    i2s_mfma_body<XJ, CT>(p, smem);
}

__global__ void __launch_bounds__(256) copy_kernel(uint4 *dst, const uint4 *src, size_t n16)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

// Streaming read of a buffer with the list kernels' own load instruction (16 bytes per lane,
// non-temporal), every lane folding what it reads into one word that is written at the end:
// the ceiling the GEMV kernels can be held against.
// (`threads`: every thread of the launch, as an argument like the GEMV kernels' block and grid sizes.)
__global__ void __launch_bounds__(512) read_kernel(const v4u *src, size_t n16, u32 *sink, size_t threads)
{
    v4u a = {0, 0, 0, 0};
    const size_t stride = threads;
    size_t i = (size_t)blockIdx.x * 512 + threadIdx.x;
    for (; i + 3 * stride < n16; i += 4 * stride) {
        v4u x0 = __builtin_nontemporal_load(src + i), x1 = __builtin_nontemporal_load(src + i + stride);
        v4u x2 = __builtin_nontemporal_load(src + i + 2 * stride), x3 = __builtin_nontemporal_load(src + i + 3 * stride);
        a ^= x0 ^ x1 ^ x2 ^ x3;
    }
    for (; i < n16; i += stride) a ^= __builtin_nontemporal_load(src + i);
    const u32 v = a.x ^ a.y ^ a.z ^ a.w;
    if (v == 0x9e3779b9u) sink[0] = v;  // (practically never: keeps the loads alive without a store per lane)
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

template <int MT>
static int launch_i2s_t(const GemvArgs &a, hipStream_t st, int waves)
{
    const int Kp = i2s_padded_k(a.K);
    I2sParams p{(const uint4 *)a.w, (const int8_t *)a.X, (int *)a.C, a.M, a.K, Kp, a.N, Kp / 256, 64 * waves};
    size_t lds = (size_t)MT * Kp + (size_t)waves * 16 * MT * 4 + (size_t)waves * MT * 4;
    dim3 grid(a.N / 16, (a.M + MT - 1) / MT), block(64 * waves);
    if (a.batch) {
        auto kern = i2s_kernel_batched<MT>;
        static std::atomic<size_t> lds_granted_b{48 * 1024};
        if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted_b)) return rc;
        for (int first = 0; first < a.batch; first += I2S_BATCH_MAX) {
            I2sBatch b{};
            const int n = a.batch - first < I2S_BATCH_MAX ? a.batch - first : I2S_BATCH_MAX;
            for (int i = 0; i < n; ++i) {
                b.w[i] = (const uint4 *)a.batch_w[first + i];
                b.X[i] = (const int8_t *)a.batch_X[first + i];
                b.C[i] = (int *)a.batch_C[first + i];
            }
            grid.z = n;
            hipLaunchKernelGGL(kern, grid, block, lds, st, p, b);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return hip_fail(e, "i2s_kernel_batched launch");
        }
        return SPTMM_OK;
    }
    auto kern = i2s_kernel<MT>;
    static std::atomic<size_t> lds_granted{48 * 1024};
    if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted)) return rc;
    hipLaunchKernelGGL(kern, grid, block, lds, st, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : hip_fail(e, "i2s_kernel launch");
}

template <int XJ, int CT>
static int launch_i2s_mfma_t(const GemvArgs &a, hipStream_t st, int waves)
{
    const int Kp = i2s_padded_k(a.K), groups = a.N / 16;
    I2sParams p{(const uint4 *)a.w, (const int8_t *)a.X, (int *)a.C, a.M, a.K, Kp, a.N, Kp / 256, 64 * waves};
    const size_t lds = (size_t)waves * (CT > 4 ? CT : 4) * 1024;
    dim3 grid((groups + CT - 1) / CT, (a.M + 15) / 16), block(64 * waves);
    static std::atomic<size_t> lds_granted{48 * 1024}, lds_granted_b{48 * 1024};
    if (a.batch) {
        auto kern = i2s_mfma_kernel_batched<XJ, CT>;
        if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted_b)) return rc;
        for (int first = 0; first < a.batch; first += I2S_BATCH_MAX) {
            I2sBatch b{};
            const int n = a.batch - first < I2S_BATCH_MAX ? a.batch - first : I2S_BATCH_MAX;
            for (int i = 0; i < n; ++i) {
                b.w[i] = (const uint4 *)a.batch_w[first + i];
                b.X[i] = (const int8_t *)a.batch_X[first + i];
                b.C[i] = (int *)a.batch_C[first + i];
            }
            grid.z = n;
            hipLaunchKernelGGL(kern, grid, block, lds, st, p, b);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return hip_fail(e, "i2s_mfma_kernel_batched launch");
        }
        return SPTMM_OK;
    }
    auto kern = i2s_mfma_kernel<XJ, CT>;
    if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted)) return rc;
    hipLaunchKernelGGL(kern, grid, block, lds, st, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : hip_fail(e, "i2s_mfma_kernel launch");
}

static int launch_i2s_mfma(const GemvArgs &a, hipStream_t st)
{
    const int tune_waves = a.plan.waves_per_wg, tune_ct = a.plan.i2s_ct;
    const int rounds = i2s_padded_k(a.K) / 256, groups = a.N / 16;
    const int rows = a.M < 16 ? a.M : 16, xj = (rows + 3) / 4;  // loads of X rows per round: four rows each
    // Column tiles per wavefront and wavefronts per workgroup, measured on MI355X (K=6912 N=2560 and K=13824
    // N=5120, 1 to 16 rows).  A batched launch fills the chip along blockIdx.z and does best with the most
    // reuse of X: 4 tiles, 4 wavefronts -- 8 tiles from nine rows on, where X traffic from L2 still sets the time
    // (K=13824 N=5120, 16 rows, 32 GEMVs per launch: 3.36 -> 3.01 us per GEMV; 8 rows: level).  A lone launch needs
    // its workgroups to cover the compute units first: the most tiles that still leave ~160 workgroups, 8 wavefronts each.
    int ct = 1, waves = 8;
    if (a.batch >= 4) {
        ct = xj >= 3 ? 8 : 4;
        waves = 4;
        // ... as long as the launch still has workgroups enough: four per compute unit, eight where a workgroup's share
        // of K is short (K=2560, 32 GEMVs per launch: N=640 4 -> 1 tiles 0.200 -> 0.154 us per GEMV, N=2560 4 -> 2 tiles
        // 0.379 -> 0.355 us; N=6912 stays at 4: 0.82 against 0.89 / 1.05 us)
        const long cus = a.compute_units > 0 ? a.compute_units : 256;
        if (xj >= 3) {
            // Nine rows and more: the reuse of X counts for more than the number of workgroups.  Short K goes to two
            // wavefronts per workgroup, and tiles are given up only while the launch has fewer than six wavefronts per
            // compute unit (32 GEMVs of 16 rows per launch, (tiles, wavefronts) -> us per GEMV: K=2560 N=2560 (2,4) 0.59,
            // (4,2) 0.43; K=2560 N=3840 (4,4) 0.84 as chosen before, (8,2) 0.59; K=6912 N=2560 (8,4) 0.92, (4,2) 0.89;
            // K=4096 N=4096 (8,4) 0.87, (8,2) 0.82; K=13824 N=5120 stays at (8,4): 2.99 against 3.12 for (8,2))
            waves = rounds >= 40 ? 4 : 2;
            while (ct > 1 && (long)a.batch * (groups / ct) * waves < 6 * cus) ct /= 2;
            if (ct == 1) waves = 4;
        } else {
            const long need = cus * (rounds >= 16 ? 4 : 8);
            while (ct > 1 && (long)a.batch * (groups / ct) < need) ct /= 2;
        }
    } else {
        while (ct < 4 && groups / (2 * ct) >= 160) ct *= 2;
    }
    if (tune_ct == 1 || tune_ct == 2 || tune_ct == 4 || (tune_ct == 8 && xj >= 2)) ct = tune_ct;
    if (waves > rounds) waves = rounds;
    if (tune_waves > 0 && tune_waves <= 8) waves = tune_waves;
#define I2S_CASE(XJ, CT) \
    if (xj == XJ && ct == CT) return launch_i2s_mfma_t<XJ, CT>(a, st, waves)
    I2S_CASE(1, 1); I2S_CASE(1, 2); I2S_CASE(1, 4);
    I2S_CASE(2, 1); I2S_CASE(2, 2); I2S_CASE(2, 4);
    I2S_CASE(3, 1); I2S_CASE(3, 2); I2S_CASE(3, 4);
    I2S_CASE(4, 1); I2S_CASE(4, 2); I2S_CASE(4, 4);
    I2S_CASE(2, 8); I2S_CASE(3, 8); I2S_CASE(4, 8);
#undef I2S_CASE
    return fail(SPTMM_ERR_INVALID, "no i2s kernel for %d rows", a.M);
}

int launch_i2s(const GemvArgs &a, void *stream)
{
    const int Kp = i2s_padded_k(a.K), rounds = Kp / 256, groups = a.N / 16;
    int rpw = groups >= 2 * a.compute_units ? 4 : (groups >= a.compute_units ? 2 : 1);
    int waves = (rounds + rpw - 1) / rpw;
    waves = waves < 1 ? 1 : (waves > 16 ? 16 : waves);
    const size_t extra = (size_t)waves * 17 * 4;
    hipStream_t st = (hipStream_t)stream;
    // One activation row launched alone stays on the vector unit (dot4 on the codes as they are); with more
    // rows, or many GEMVs per launch, the matrix-unit kernel is ahead (M=4: 5.0 -> 3.5 us alone, 1.8 -> 0.8 us batched).
    const int mfma_from = tuning().i2s_mfma_from;
    if (a.M >= mfma_from || a.batch >= 4) return launch_i2s_mfma(a, st);
    if ((size_t)Kp + extra > (size_t)a.lds_limit) return launch_i2s_mfma(a, st);  // (K beyond the one-row LDS tile)
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

int launch_read(const void *src, size_t bytes, void *sink, int workgroups, void *stream)
{
    if (bytes % 16) return fail(SPTMM_ERR_INVALID, "read size must be a multiple of 16 bytes");
    if (workgroups < 1) workgroups = 256 * 4;
    hipLaunchKernelGGL(read_kernel, dim3(workgroups), dim3(512), 0, (hipStream_t)stream, (const v4u *)src, bytes / 16, (u32 *)sink,
                       (size_t)workgroups * 512);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : hip_fail(e, "read_kernel launch");
}

int launch_u16(const GemvArgs &a, ActType act, void *stream)
{
    if (a.ragged) return a.index_shift == 2 ? launch_ragged_u16_scaled(a, act, stream) : launch_ragged_u16_plain(a, act, stream);
    return a.index_shift == 2 ? launch_u16_scaled(a, act, stream) : launch_u16_plain(a, act, stream);
}

int launch_delta(const GemvArgs &a, ActType act, void *stream)
{
    if (a.ragged) return a.delta_bits == 8 ? launch_ragged_runs8(a, act, stream) : launch_ragged_runs16(a, act, stream);
    return a.delta_bits == 8 ? launch_runs8(a, act, stream) : launch_runs16(a, act, stream);
}

}  // namespace sptmm
