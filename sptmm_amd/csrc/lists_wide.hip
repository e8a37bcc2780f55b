// Kernels for the wide streams (wide.cpp): activation tiles with 16-byte slots -- 16 int8 rows or
// 8 fp16 rows per row index -- staged K-tile by K-tile, so that the index stream is read once for up
// to 16 rows whatever K is (the reference re-reads it per row, main.cu:567).
//
// Per workgroup and K-tile ("phase"): stage the tile, walk the phase's tasks, add the column sums
// into C (phase 0 stores, later phases add to what the same lane stored before).  Tried and dropped:
// two smaller tiles in the LDS with some wavefronts staging the next K-tile while the others gather
// (K = 13824, 16 rows: 25.2 against 24.4 us alone, 23.1 against 21.1 us in batched launches -- the extra
// K-tile costs more than the overlap returns), deeper rings with fewer wavefronts (slower throughout).
//
// Sums on the matrix unit: one gathered slot (16 bytes = all rows of one index) is a lane's A operand
// of a 16x16 matrix instruction, and the B operand is a constant selector with a single 1 (-1 for the
// minus list) per lane that routes byte b of every k-block to output column b.  The instruction's
// own sum over k then adds the slots of lanes i, i+16, i+32, i+48 -- which the stream gives to one
// column -- so one instruction takes 64 entries of all rows.  Nothing is multiplied by anything but
// 0 and +-1; int8 sums are exact in int32.
#include "lists.hpp"

namespace sptmm {

struct WideParams {
    const uint8_t *w;
    const void *X;
    void *C;
    int M, K, N, k_tile, phases, tasks, logL, iters;
    int threads, grid_x;  // blockDim.x and gridDim.x as arguments (the built-ins cost two memory round trips in a row at kernel start)
    u32 offset[16], stride[16];
    int n_min[16];
};

// position of row r (relative to the K-tile) in the tile: staging writes 16 consecutive rows per lane, and
// this spreads the 16 lanes the LDS serves per pass over its 16 bank groups
__device__ __forceinline__ u32 wide_pos(u32 r) { return r ^ ((r >> 4) & 15u); }

template <typename Act> struct WideSums {
    static constexpr bool I8 = sizeof(Act) == 1;
    static constexpr int ROWS = I8 ? 16 : 8;
    static constexpr int SLOT = 16;
    static constexpr int NACC = 2;  // independent accumulation chains
    typedef typename Acc<Act>::type A;
    typedef Vec<u32, 4> Raw;
    v4i D[NACC], Bp, Bn;
    v4f Df[NACC];
    v8h Bpf, Bnf;

    static __device__ __forceinline__ Raw load(const unsigned char *lds, u32 addr) { return *reinterpret_cast<const Raw *>(lds + addr); }

    __device__ __forceinline__ void init()
    {
        const int j = threadIdx.x & 15;  // output column = activation row this lane's selector picks
        if constexpr (I8) {
            const u32 one = 1u << (8 * (j & 3)), neg = 0xffu << (8 * (j & 3));
            Bp = v4i{j < 4 ? (int)one : 0, (j >> 2) == 1 ? (int)one : 0, (j >> 2) == 2 ? (int)one : 0, (j >> 2) == 3 ? (int)one : 0};
            Bn = v4i{j < 4 ? (int)neg : 0, (j >> 2) == 1 ? (int)neg : 0, (j >> 2) == 2 ? (int)neg : 0, (j >> 2) == 3 ? (int)neg : 0};
#pragma unroll
            for (int x = 0; x < NACC; ++x) D[x] = v4i{0, 0, 0, 0};
        } else {
#pragma unroll
            for (int y = 0; y < 8; ++y) {
                Bpf[y] = y == j ? (_Float16)1.0f : (_Float16)0.0f;
                Bnf[y] = y == j ? (_Float16)-1.0f : (_Float16)0.0f;
            }
#pragma unroll
            for (int x = 0; x < NACC; ++x) Df[x] = v4f{0.f, 0.f, 0.f, 0.f};
        }
    }
    template <bool NEG, int NE> __device__ __forceinline__ void accum_n(const Raw *r)
    {
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            if constexpr (I8) {
                const v4i a = {(int)r[e].v[0], (int)r[e].v[1], (int)r[e].v[2], (int)r[e].v[3]};
                D[e % NACC] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, NEG ? Bn : Bp, D[e % NACC], 0, 0, 0);
            } else {
                const v8h a = __builtin_bit_cast(v8h, r[e]);
                Df[e % NACC] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, NEG ? Bnf : Bpf, Df[e % NACC], 0, 0, 0);
            }
        }
    }
    __device__ __forceinline__ void pin() {}
    // result register r of this lane: the sum over lanes i, i+16, i+32, i+48 (i = 4 (lane / 16) + r) of activation row lane % 16
    __device__ __forceinline__ A reg(int r) const
    {
        if constexpr (I8)
            return D[0][r] + D[1][r];
        else
            return Df[0][r] + Df[1][r];
    }
};

// fp16 rows summed on the VALU: the path of a workgroup whose tile holds an Inf or NaN (the matrix
// instruction would turn 0 x Inf into NaN for every row and partner lane of the operand)
struct WidePlain {
    static constexpr int SLOT = 16;
    typedef Vec<u32, 4> Raw;
    float acc[8];
    static __device__ __forceinline__ Raw load(const unsigned char *lds, u32 addr) { return *reinterpret_cast<const Raw *>(lds + addr); }
    __device__ __forceinline__ void init()
    {
#pragma unroll
        for (int m = 0; m < 8; ++m) acc[m] = 0.f;
    }
    template <bool NEG, int NE> __device__ __forceinline__ void accum_n(const Raw *r)
    {
#pragma unroll
        for (int e = 0; e < NE; ++e)
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                const float v = h2f(r[e].v[m / 2], m & 1);
                acc[m] = NEG ? acc[m] - v : acc[m] + v;
            }
    }
    __device__ __forceinline__ void pin()
    {
#pragma unroll
        for (int m = 0; m < 8; ++m) asm volatile("" : "+v"(acc[m]));
    }
};

// item = 16 consecutive k of all rows -> 16 slots of 16 bytes, slot of row k at position k ^ (item & 15)
template <typename Act> struct WideStager {
    static constexpr int ROWS = WideSums<Act>::ROWS;
    static __device__ __forceinline__ void load(const Act *X, int M, int K, int m0, int k, uint4 (&r)[16])
    {
        constexpr int PER = (int)sizeof(Act);  // 16-byte loads per row and item
#pragma unroll
        for (int m = 0; m < ROWS; ++m)
#pragma unroll
            for (int j = 0; j < PER; ++j)
                r[m * PER + j] = (m0 + m < M) ? reinterpret_cast<const uint4 *>(X + (size_t)(m0 + m) * K + k)[j] : make_uint4(0, 0, 0, 0);
    }
    static __device__ __forceinline__ void store(unsigned char *lds, int item, const uint4 (&r)[16])
    {
        uint4 *t = reinterpret_cast<uint4 *>(lds) + 16 * item;
        const u32 rho = (u32)item & 15u;
        if constexpr (sizeof(Act) == 1) {
            // 16 rows x 16 k bytes: 4 x 4 blocks of 4 x 4 byte transpositions
#pragma unroll
            for (int j = 0; j < 4; ++j) {  // k = 4j .. 4j+3
                u32 o[4][4];
#pragma unroll
                for (int R = 0; R < 4; ++R) transpose4x4(comp(r[4 * R], j), comp(r[4 * R + 1], j), comp(r[4 * R + 2], j), comp(r[4 * R + 3], j), o[R]);
#pragma unroll
                for (int q = 0; q < 4; ++q) t[(u32)(4 * j + q) ^ rho] = make_uint4(o[0][q], o[1][q], o[2][q], o[3][q]);
            }
        } else {
            // 8 rows x 16 k halves; r[2m + h] = row m, halves 8h .. 8h+7
#pragma unroll
            for (int d = 0; d < 8; ++d) {  // k = 2d, 2d+1
                u32 w[8];
#pragma unroll
                for (int m = 0; m < 8; ++m) w[m] = comp(r[2 * m + d / 4], d % 4);
                t[(u32)(2 * d) ^ rho] = make_uint4(__builtin_amdgcn_perm(w[1], w[0], 0x05040100u), __builtin_amdgcn_perm(w[3], w[2], 0x05040100u),
                                                   __builtin_amdgcn_perm(w[5], w[4], 0x05040100u), __builtin_amdgcn_perm(w[7], w[6], 0x05040100u));
                t[(u32)(2 * d + 1) ^ rho] = make_uint4(__builtin_amdgcn_perm(w[1], w[0], 0x07060302u), __builtin_amdgcn_perm(w[3], w[2], 0x07060302u),
                                                       __builtin_amdgcn_perm(w[5], w[4], 0x07060302u), __builtin_amdgcn_perm(w[7], w[6], 0x07060302u));
            }
        }
    }
};


template <typename Act, int MODE, int RING_ = 4> struct WideBody {
    typedef Flavour<MODE> Fl;
    typedef WideSums<Act> Sm;
    typedef typename Acc<Act>::type A;
    static constexpr int ESZ = Fl::ESZ, E16 = 16 / ESZ, HDR = Fl::HDR;
    static constexpr bool GAPS = Fl::GAP8 || Fl::GAP16;
    static constexpr int ROWS = Sm::ROWS;
    static constexpr int RING = RING_;  // rounds of a task's stream in flight per wavefront
    static constexpr bool TWIN = sizeof(Act) == 2;

    template <class S> static __device__ __forceinline__ void eat(const unsigned char *smem, const Round &x, u32 &runp, u32 &runq, S &acc)
    {
        consume16<S, MODE, true, false>(smem, x.p, runp, acc);
        consume16<S, MODE, true, true>(smem, x.q, runq, acc);
        acc.pin();
        if constexpr (GAPS) asm volatile("" : "+v"(runp), "+v"(runq));
    }

    // all n entries per lane and sign of the task at tb, through a ring of RING rounds in flight
    template <class S> static __device__ __forceinline__ void walk(const unsigned char *smem, const uint8_t *tb, int lane, int n, S &acc)
    {
        const uint4 *wp = reinterpret_cast<const uint4 *>(tb + HDR) + lane;
        u32 runp = 0, runq = 0;
        if constexpr (GAPS) {
            const unsigned short *rs = reinterpret_cast<const unsigned short *>(tb);
            runp = (u32)rs[lane] << (Fl::GAP8 ? 0 : 4);
            runq = (u32)rs[64 + lane] << (Fl::GAP8 ? 0 : 4);
        }
        const int R = n / E16, rem = n - R * E16;
        Round buf[RING];
        if (R > 0) {
#pragma unroll
            for (int i = 0; i < RING; ++i) buf[i] = load_round(wp, i < R ? i : R - 1);
        }
        uint2 t8p = make_uint2(0, 0), t8q = make_uint2(0, 0);
        u32 t4p = 0, t4q = 0, t2p = 0, t2q = 0, t1p = 0, t1q = 0;
        if (rem) {
            const uint8_t *t = tb + HDR + (size_t)R * 2048;
            if (rem & (8 / ESZ)) {
                t8p = reinterpret_cast<const uint2 *>(t)[lane];
                t8q = reinterpret_cast<const uint2 *>(t + 512)[lane];
                t += 1024;
            }
            if (rem & (4 / ESZ)) {
                t4p = reinterpret_cast<const u32 *>(t)[lane];
                t4q = reinterpret_cast<const u32 *>(t + 256)[lane];
                t += 512;
            }
            if (rem & (2 / ESZ)) {
                t2p = reinterpret_cast<const unsigned short *>(t)[lane];
                t2q = reinterpret_cast<const unsigned short *>(t + 128)[lane];
                t += 256;
            }
            if constexpr (ESZ == 1) {
                if (rem & 1) {
                    t1p = t[lane];
                    t1q = t[64 + lane];
                }
            }
        }
        int base = 0;
        for (; base + 2 * RING <= R; base += RING) {
#pragma unroll
            for (int i = 0; i < RING; ++i) {
                eat(smem, buf[i], runp, runq, acc);
                buf[i] = load_round(wp, base + RING + i);
            }
        }
        if (R - base > RING) {
#pragma unroll
            for (int i = 0; i < RING; ++i) {
                eat(smem, buf[i], runp, runq, acc);
                const int r = base + RING + i;
                buf[i] = load_round(wp, r < R ? r : R - 1);
            }
            base += RING;
        }
#pragma unroll
        for (int i = 0; i < RING; ++i)
            if (base + i < R) eat(smem, buf[i], runp, runq, acc);
        if (rem) {
            if (rem & (8 / ESZ)) {
                consume<S, MODE, true, false, 4>(smem, t8p.x, runp, acc);
                consume<S, MODE, true, false, 4>(smem, t8p.y, runp, acc);
                consume<S, MODE, true, true, 4>(smem, t8q.x, runq, acc);
                consume<S, MODE, true, true, 4>(smem, t8q.y, runq, acc);
            }
            if (rem & (4 / ESZ)) {
                consume<S, MODE, true, false, 4>(smem, t4p, runp, acc);
                consume<S, MODE, true, true, 4>(smem, t4q, runq, acc);
            }
            if (rem & (2 / ESZ)) {
                consume<S, MODE, true, false, 2>(smem, t2p, runp, acc);
                consume<S, MODE, true, true, 2>(smem, t2q, runq, acc);
            }
            if constexpr (ESZ == 1) {
                if (rem & 1) {
                    consume<S, MODE, true, false, 1>(smem, t1p, runp, acc);
                    consume<S, MODE, true, true, 1>(smem, t1q, runq, acc);
                }
            }
        }
    }

    // C[m][col] = (or +=, behind the first phase) v.  An element is written by the same WAVEFRONT in every phase (a task
    // keeps its wavefront), by the same lane as long as the phases sum on the same unit; where an fp16 tile holds a
    // non-finite value and the phase sums on the vector unit, another lane of that wavefront writes it.  Either way the
    // earlier store is complete and in L2 before the later load: every phase but the first starts with a workgroup
    // barrier, which waits for the wavefront's outstanding stores (the compute unit's own cache writes through), and
    // the load is an agent-scope atomic, served by L2.  (An agent-scope atomic store as well costs 5-7 % of a batched
    // 16-row launch at K=13824 and adds nothing to that.)
    static __device__ __forceinline__ void put(const WideParams &p, void *C, int m, int col, A v, bool first)
    {
        A *c = reinterpret_cast<A *>(C) + (size_t)m * p.N + col;
        if (!first) v += __hip_atomic_load(c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *c = v;
    }

    // (w, Xv, C: the launch's stream, activations and output; a batched launch picks them per blockIdx.z and leaves
    // the parameter block itself untouched, so that it stays in scalar registers)
    static __device__ __forceinline__ void run(const WideParams &p, const uint8_t *w, const void *Xv, void *C, unsigned char *smem)
    {
        const int tid = threadIdx.x, nt = p.threads, lane = tid & 63, wave = tid >> 6, waves = nt >> 6;
        const int m0 = blockIdx.y * ROWS;
        const Act *X = reinterpret_cast<const Act *>(Xv);
        const int logL = p.logL, q = lane >> 4, row = lane & 15;
        for (int ph = 0; ph < p.phases; ++ph) {
            const int k0 = ph * p.k_tile, kt = p.K - k0 < p.k_tile ? p.K - k0 : p.k_tile;
            if (ph > 0) __syncthreads();  // everybody is done gathering from the previous tile
            u32 xmax = 0u;
            for (int item = tid; item < kt / 16; item += nt) {
                uint4 r[16];
                WideStager<Act>::load(X, p.M, p.K, m0, k0 + 16 * item, r);
                WideStager<Act>::store(smem, item, r);
                if constexpr (TWIN) {
#pragma unroll
                    for (int j = 0; j < 16; ++j) xmax = pk_absmax16(xmax, r[j]);
                }
            }
            for (int i = tid; i < 64 * 4; i += nt) reinterpret_cast<u32 *>(smem + (size_t)kt * 16)[i] = 0u;  // rows kt .. kt+63 read as zero
            u32 *nf_flags = reinterpret_cast<u32 *>(smem + (size_t)(p.k_tile + 64) * 16);
            if constexpr (TWIN) {
                const bool any = __builtin_amdgcn_ballot_w64(pk_nonfinite16(xmax)) != 0;
                if (lane == 0) nf_flags[wave] = any ? 1u : 0u;
            }
            __syncthreads();
            bool plain = false;  // workgroup-uniform
            if constexpr (TWIN) {
                u32 f = 0u;
                for (int w = 0; w < waves; ++w) f |= nf_flags[w];
                plain = __builtin_amdgcn_readfirstlane(f) != 0u;
            }

            const uint8_t *sub = w + p.offset[ph];
            const unsigned short *counts = reinterpret_cast<const unsigned short *>(sub + RAGGED_PREAMBLE);
            const uint8_t *tasks_base = sub + ((size_t)16 + 2 * (size_t)p.tasks + 255) / 256 * 256;
            int task = blockIdx.x * waves + wave;
            for (int it = 0; it < p.iters; ++it, task += p.grid_x * waves) {
                if (task >= p.tasks) break;  // (uniform per wavefront; no barrier inside the loop)
                const int n = __builtin_amdgcn_readfirstlane((int)counts[task]);
                const uint8_t *tb = tasks_base + (size_t)task * p.stride[ph];
                const int cbase = task << (6 - logL);
                if (TWIN && plain) {
                    if constexpr (TWIN) {
                        WidePlain acc;
                        acc.init();
                        walk(smem, tb, lane, n, acc);
                        // a column's lanes: {i + 16 g}, i over L/4 consecutive values -> fold g (lane bits 4, 5), then the low bits of i
#pragma unroll
                        for (int m = 0; m < 8; ++m) {
                            float v = acc.acc[m];
                            v += swz16(v);
                            v += __shfl_xor(v, 32, 64);
                            for (int b = 1; b < (1 << (logL - 2)); b <<= 1) v += __shfl_xor(v, b, 64);
                            if (lane < 16 && (lane & ((1 << (logL - 2)) - 1)) == 0 && m0 + m < p.M) put(p, C, m0 + m, cbase + (lane >> (logL - 2)), v, ph == 0);
                        }
                    }
                } else {
                    Sm acc;
                    acc.init();
                    walk(smem, tb, lane, n, acc);
                    // register r: rows i = 4q + r of the result = lanes i + 16 g; a column owns L/4 consecutive i
                    A v0 = acc.reg(0), v1 = acc.reg(1), v2 = acc.reg(2), v3 = acc.reg(3);
                    const bool row_ok = row < ROWS && m0 + row < p.M;
                    if (logL == 3) {  // two i per column: columns 2q and 2q+1
                        if (row_ok) {
                            put(p, C, m0 + row, cbase + 2 * q, v0 + v1, ph == 0);
                            put(p, C, m0 + row, cbase + 2 * q + 1, v2 + v3, ph == 0);
                        }
                    } else {
                        A v = (v0 + v1) + (v2 + v3);
                        if (logL >= 5) v += swz16(v);
                        if (logL >= 6) v += __shfl_xor(v, 32, 64);
                        const bool writer = logL == 4 ? true : logL == 5 ? !(q & 1) : q == 0;
                        const int col = logL == 4 ? q : logL == 5 ? q >> 1 : 0;
                        if (row_ok && writer) put(p, C, m0 + row, cbase + col, v, ph == 0);
                    }
                }
            }
        }
    }
};

// MAXW = most wavefronts per workgroup (the register budget follows from it), RING = rounds in flight per wavefront
template <typename Act, int MODE, int RING, int MAXW>
__global__ void __launch_bounds__(64 * MAXW) wide_kernel(WideParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    WideBody<Act, MODE, RING>::run(p, p.w, p.X, p.C, smem);
}

template <typename Act, int MODE, int RING, int MAXW>
__global__ void __launch_bounds__(64 * MAXW) wide_kernel_batched(WideParams p, BatchPtrs b)
{
    extern __shared__ __align__(16) unsigned char smem[];
    WideBody<Act, MODE, RING>::run(p, b.w[blockIdx.z], b.X[blockIdx.z], b.C[blockIdx.z], smem);
}

template <typename Act, int MODE, int RING, int MAXW>
static int launch_wide_v(const GemvArgs &a, const WideHeader &h, hipStream_t st)
{
    constexpr int ROWS = WideSums<Act>::ROWS;
    const int tune_wpb = a.plan.waves_per_wg;
    const int cus = a.compute_units > 0 ? a.compute_units : 256;
    const size_t lds = (size_t)(h.k_tile + 64) * 16 + 64;
    if ((int)lds > a.lds_limit) return fail(SPTMM_ERR_UNSUPPORTED, "the stream's K-tile of %d rows needs %zu bytes of LDS, the device grants %d", h.k_tile, lds, a.lds_limit);
    // one workgroup per compute unit (the tile fills the LDS), as many wavefronts as it takes to hold a task each
    const int per_cu = (size_t)a.lds_limit >= 2 * lds ? 2 : 1;  // workgroups whose tiles fit a compute unit together
    int wpb = (a.tasks + cus * per_cu - 1) / (cus * per_cu);
    wpb = wpb < 4 ? 4 : wpb > MAXW / per_cu ? MAXW / per_cu : wpb;
    // The walk keeps the matrix unit busy (one instruction per entry), and a wavefront count that does not divide by
    // the four SIMDs leaves some of them a third more work: batched launches, which are free to regroup their tasks,
    // take a multiple of four (config 4, M=16, 10 -> 12 wavefronts: gap stream 17.9 -> 14.7 us per GEMV, u16 16.2 -> 16.0).
    if (a.batch >= 4 && wpb % 4 && (wpb + 3) / 4 * 4 <= MAXW / per_cu) wpb = (wpb + 3) / 4 * 4;
    // ... and the largest workgroup does better still: fewer workgroups stage the tile (the activation rows come out of
    // L2 once per workgroup and K-tile) and four wavefronts per SIMD hide more of the gathers' latency (same shape, 12 ->
    // 16 wavefronts: u16 15.9 -> 15.4 us per GEMV, gap stream 14.2 -> 12.7 us; a lone u16 GEMV 27.9 -> 24.4 us HBM-cold
    // on 160 of the 256 compute units, a lone gap-stream GEMV 23.8 -> 24.4 us, so that one keeps the smaller workgroups)
    if ((a.batch >= 4 || MODE == 0) && wpb >= 8) wpb = MAXW / per_cu;  // (shapes with tasks enough to fill the chip that way)
    // A batched launch takes the largest workgroup whatever its task count: it fills the chip along blockIdx.z, and a
    // workgroup of four wavefronts staged a whole tile for four tasks (8 GEMVs per launch, 16 rows: K=5376 N=3840 S=2016
    // 4 -> 16 wavefronts gap stream 6.04 -> 2.66 us per GEMV, u16 4.69 -> 3.05; K=9728 N=6400 S=512 u16 2.71 -> 1.96;
    // K=2048 N=3840 S=1088, two tiles per compute unit, 4 -> 8: 2.62 -> 1.87)
    if (a.batch >= 4) {
        wpb = MAXW / per_cu;
        // (as long as its workgroups cover three quarters of the compute units: K=12800 N=256, 8 GEMVs of 64 tasks: 16 -> 8
        // wavefronts 2.47 -> 1.90 us per GEMV, K=6656 N=512 1.51 -> 1.09; K=6912 N=1792, 224 workgroups of 16, is best left so)
        while (wpb > 8 && (long)a.batch * ((a.tasks + wpb - 1) / wpb) * 4 < 3L * cus * per_cu) wpb -= 4;
    }
    if (tune_wpb > 0 && tune_wpb <= MAXW) wpb = tune_wpb;
    const int blocks = (a.tasks + wpb - 1) / wpb;
    int grid_x = blocks < cus * per_cu ? blocks : cus * per_cu;
    // A batched launch fills the chip along blockIdx.z, and every workgroup pays 2.5 us per K-tile for staging before
    // it walks (about 7 us per task): fewer workgroups with up to 16 tasks per wavefront, as long as the launch's
    // workgroups still come in full rounds over the compute units (config 4, M=16, 7 GEMVs per launch: 1 / 2 / 4 / 8
    // tasks per wavefront 21.2 / 20.1 / 18.4 / 17.4 us per GEMV; 6 -- one and a fifth rounds -- 23.7 us).
    if (a.batch >= 4 && blocks <= cus * per_cu) {
        double best = 1e30;
        int pick = 1;
        for (int bi = 1; bi <= 16 && bi <= blocks; ++bi) {
            const long total = (long)a.batch * ((blocks + bi - 1) / bi), slots = (long)cus * per_cu;
            const double cost = (double)((total + slots - 1) / slots) * (2.5 + 7.0 * bi);
            if (cost < best - 1e-9) best = cost, pick = bi;
        }
        grid_x = (blocks + pick - 1) / pick;
    }
    WideParams p{};
    p.w = (const uint8_t *)a.w, p.X = a.X, p.C = a.C;
    p.M = a.M, p.K = a.K, p.N = a.N, p.k_tile = h.k_tile, p.phases = h.phases, p.tasks = a.tasks, p.logL = ilog2(a.L);
    p.iters = (blocks + grid_x - 1) / grid_x;
    p.threads = 64 * wpb, p.grid_x = grid_x;
    for (int i = 0; i < h.phases; ++i) p.offset[i] = h.offset[i], p.stride[i] = h.stride[i], p.n_min[i] = h.n_min[i];
    dim3 grid(grid_x, (a.M + ROWS - 1) / ROWS), block(64 * wpb);
    static std::atomic<size_t> lds_granted{48 * 1024}, lds_granted_b{48 * 1024};
    if (a.batch) {
        auto kern = wide_kernel_batched<Act, MODE, RING, MAXW>;
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
            if (e != hipSuccess) return hip_fail(e, "wide_kernel_batched launch");
        }
        return SPTMM_OK;
    }
    auto kern = wide_kernel<Act, MODE, RING, MAXW>;
    if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted)) return rc;
    hipLaunchKernelGGL(kern, grid, block, lds, st, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : hip_fail(e, "wide_kernel launch");
}

template <typename Act, int MODE>
static int launch_wide_t(const GemvArgs &a, const WideHeader &h, hipStream_t st)
{
    // fp16 rows on 8-bit gaps: 16 gathered slots of 16 bytes per stream dword do not fit 128 registers (152 bytes of scratch
    // per lane at 16 wavefronts); 12 wavefronts, 168 registers: K=13824 N=5120, M=8, one GEMV per launch 26.1 -> 22.2 us,
    // batched launches level (13.2 against 13.3 us)
    if constexpr (sizeof(Act) == 2 && MODE == 1)
        return launch_wide_v<Act, MODE, 4, 12>(a, h, st);
    else
        return launch_wide_v<Act, MODE, 4, 16>(a, h, st);
}

int launch_wide(const GemvArgs &a, const WideHeader &h, ActType act, void *stream)
{
    hipStream_t st = (hipStream_t)stream;
    if (act == ACT_F32) return fail(SPTMM_ERR_UNSUPPORTED, "wide streams take int8 or fp16 activations");
    const int mode = h.kind == SPTMM_KIND_U16 ? 0 : h.bits == 8 ? 1 : 2;
    if (act == ACT_I8) {
        if (mode == 0) return launch_wide_t<int8_t, 0>(a, h, st);
        if (mode == 1) return launch_wide_t<int8_t, 1>(a, h, st);
        return launch_wide_t<int8_t, 2>(a, h, st);
    }
    if (mode == 0) return launch_wide_t<_Float16, 0>(a, h, st);
    if (mode == 1) return launch_wide_t<_Float16, 1>(a, h, st);
    return launch_wide_t<_Float16, 2>(a, h, st);
}

}  // namespace sptmm
