// Device code and launch templates shared by the list-stream translation units
// (u16 lists and run gap streams, balanced or ragged).  Each .hip file that
// includes this header instantiates the kernels of one stream flavour, so the
// flavours compile in parallel.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <type_traits>

#include "internal.hpp"
#include "lanes.hpp"

namespace sptmm {


typedef unsigned int u32;

// ------------------------------------------------------------------ helpers
template <typename Act> struct Acc { typedef float type; };
template <> struct Acc<int8_t> { typedef int type; };
// int8 activations kept as they are, one byte per row index, in the tile of a single activation row
// (gap streams whose visiting order was scheduled for such a tile: LDS bank = (row / 4) mod 32).
// The gather address is the running row itself and the tile is a quarter of the int32 one.
struct i8row { int8_t v; };
template <> struct Acc<i8row> { typedef int type; };
template <typename Act> constexpr bool is_byte_rows() { return std::is_same<Act, i8row>::value; }

// Bytes one row index occupies in the LDS activation tile.  Every layout keeps
// "dword address mod 32 == row index mod 32" at 4 bytes per index, which is the
// rule the host-side scheduler of the u16 stream relies on to keep the 32 lanes
// of a half-wavefront on 32 different LDS banks.
template <typename Act, int MT> __host__ __device__ constexpr int slot_bytes()
{
    return is_byte_rows<Act>() ? 1                      // int8, one row, one byte per index
           : sizeof(Act) == 1 ? (MT == 1 ? 4 : MT)      // int8: one int32 (M=1), or MT packed bytes
           : sizeof(Act) == 2 ? (MT == 1 ? 4 : 2 * MT)  // fp16: one fp32 (M=1), or MT halves
                              : 4 * MT;                 // fp32
}
__host__ __device__ constexpr int ilog2(int v) { return v <= 1 ? 0 : 1 + ilog2(v >> 1); }

template <typename T, int N> struct alignas(sizeof(T) * N) Vec { T v[N]; };
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// The running sums of one lane: acc[m] (+|-)= X[m][k] for every gathered row k.
//
// int8 activations with MT > 1 (MX): a gathered slot holds the MT rows of one index as packed
// bytes, and adding bytes into per-row int32 sums on the VALU costs one instruction per entry
// and row however it is arranged (masked 16-bit fields: 4 per four rows; SDWA byte adds and
// 16-bit-field tiles measured slower) -- from M = 4 that, not HBM, set the time.  The matrix unit
// does the same adds: four entries (MT = 8: two) are the 16 bytes a lane hands to one
// v_mfma_i32_16x16x64_i8 as the A operand, and the B operand is a constant selector of 0 / 1
// (-1 for the minus list) that routes every byte to the int32 of its (lane, row) in the 16x16
// result.  Nothing is contracted -- each output sums one lane's own bytes of one row -- the
// instruction is used as 256 byte-to-int32 adders, on a unit this kernel otherwise leaves idle.
//
// PLAIN = true: fp16 rows summed on the VALU whatever MT (one convert and one add per entry and
// row).  The matrix-unit sums multiply every byte of an operand row with 0 or +-1, so one Inf or
// NaN among the gathered values turns the sums of the other rows and of the three partner lanes
// into NaN (0 x Inf); a workgroup whose tile holds a non-finite value therefore sums this way.
// MERGED (eight-row tiles whose columns take 32 or 64 lanes, a property of the launch): one result tile where two are
// needed otherwise -- half the matrix instructions, and 12 registers less in kernels that are held to 128.
template <typename Act, int MT, bool PLAIN = false, bool MERGED = false> struct Sums {
    typedef typename Acc<Act>::type A;
    typedef Act act_type;
    static constexpr int ROWS = MT;
    static constexpr int SLOT = slot_bytes<Act, MT>();
    static_assert(!PLAIN || sizeof(Act) == 2, "only fp16 tiles have a VALU twin");
    static constexpr bool MX = sizeof(Act) == 1 && MT > 1;  // sums on the matrix unit
    static constexpr bool MXF = sizeof(Act) == 2 && MT > 1 && !PLAIN;  // the same for fp16 rows: v_mfma_f32_16x16x32_f16, two entries x
                                                                       // four rows (MT = 4) or one entry x eight rows (MT = 8) per
                                                                       // operand, selector of 0 / +-1.0
    static constexpr int NW = MX ? MT / 4 : 1;              // dwords per gathered slot (int8)
    static_assert(!MERGED || (MT == 8 && !PLAIN), "merged result tiles belong to eight-row tiles on the matrix unit");
    static constexpr int ND = (MX || MXF) && !MERGED ? MT / 4 : 1;  // result tiles
    v4i D[ND], Bp[ND], Bn[ND];                              // MX: 16x16 int32 result tiles and the +1 / -1 selectors
    static constexpr bool merged = MERGED;                  // one result tile sums lanes i, i+16 (, i+32, i+48)
    v4f Df[ND];                                             // MXF: the fp32 result tiles ...
    v8h Bpf[ND], Bnf[ND];                                   // ... and their selectors
    A acc[MT];

    // sum of the four registers a lane holds of result tile x
    __device__ __forceinline__ A tile_sum(int x) const
    {
        if constexpr (MXF)
            return (Df[x][0] + Df[x][1]) + (Df[x][2] + Df[x][3]);
        else
            return (A)(D[x][0] + D[x][1] + D[x][2] + D[x][3]);
    }

    // logL: log2 of the lanes that share a column (the matrix-unit sums of eight-row tiles depend on it)
    __device__ __forceinline__ void init(int logL = 0)
    {
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = (A)0;
        if constexpr (MX) {
            // Selector held by lane j + 16 g (k-block g, output column j): 1 where the byte of the A operand
            // at the same (g, byte) position is to be added into column j.  MT = 4: A = 4 entries x 4 rows,
            // column 4 g + row.  MT = 8: A = 2 entries x 8 rows, tile x takes k-blocks 2x and 2x + 1, column
            // 8 (g & 1) + row.
            const int l = threadIdx.x & 63, g = l >> 4, j = l & 15;
            const u32 b = 1u << (8 * (j & 3));
#pragma unroll
            for (int x = 0; x < ND; ++x) {
                u32 e, o;
                if constexpr (MT == 4) {
                    e = o = (j >> 2) == g ? b : 0u;
                } else {
                    // Two result tiles keep every lane's sums apart (tile x: k-blocks 2x, 2x+1 -> column 8 (g & 1) + row).
                    // When lanes i and i+16 belong to one column anyway (32 lanes per column: k-blocks 0, 1 -> columns
                    // 0..7, k-blocks 2, 3 -> 8..15; 64 lanes: all four -> 0..7) one tile does, with half the instructions.
                    const bool on = merged ? (x == 0 && (j >> 3) == (logL == 5 ? g >> 1 : 0)) : ((g >> 1) == x && (j >> 3) == (g & 1));
                    e = on && !(j & 4) ? b : 0u;
                    o = on && (j & 4) ? b : 0u;
                }
                Bp[x] = v4i{(int)e, (int)o, (int)e, (int)o};
                Bn[x] = v4i{(int)(e * 255u), (int)(o * 255u), (int)(e * 255u), (int)(o * 255u)};
                D[x] = v4i{0, 0, 0, 0};
            }
        } else if constexpr (MXF) {
            // lane j + 16 g holds rows 8 g .. 8 g + 7 of selector column j.  MT = 4: the operand is two entries x four
            // rows, column 4 g + row.  MT = 8: one entry x eight rows; tiles and columns as for eight int8 rows.
            const int l = threadIdx.x & 63, g = l >> 4, j = l & 15;
#pragma unroll
            for (int x = 0; x < ND; ++x) {
#pragma unroll
                for (int y = 0; y < 8; ++y) {
                    bool on;
                    if constexpr (MT == 4)
                        on = (j >> 2) == g && (y & 3) == (j & 3);
                    else
                        on = (merged ? (x == 0 && (j >> 3) == (logL == 5 ? g >> 1 : 0)) : ((g >> 1) == x && (j >> 3) == (g & 1))) && y == (j & 7);
                    Bpf[x][y] = on ? (_Float16)1.0f : (_Float16)0.0f;
                    Bnf[x][y] = on ? (_Float16)-1.0f : (_Float16)0.0f;
                }
                Df[x] = v4f{0.f, 0.f, 0.f, 0.f};
            }
        }
    }

    // What one slot of the tile holds (all MT rows of one index), as read from LDS.
    typedef typename std::conditional<is_byte_rows<Act>(), Vec<int8_t, 1>, typename std::conditional<sizeof(Act) == 1, Vec<u32, NW>,
                                      typename std::conditional<sizeof(Act) == 2 && (MT > 1), Vec<_Float16, MT>, Vec<float, MT>>::type>::type>::type Raw;

    // the slot at byte offset `addr` of the tile
    static __device__ __forceinline__ Raw load(const unsigned char *lds, u32 addr) { return *reinterpret_cast<const Raw *>(lds + addr); }

    // NE gathered slots of one sign
    template <bool NEG, int NE> __device__ __forceinline__ void accum_n(const Raw *r)
    {
        if constexpr (MX) {
            constexpr int PER = 16 / MT;  // entries per A operand; a short tail is filled with zero bytes
#pragma unroll
            for (int e = 0; e < NE; e += PER) {
                v4i a;
                if constexpr (MT == 4)
                    a = v4i{(int)r[e].v[0], e + 1 < NE ? (int)r[e + 1 < NE ? e + 1 : e].v[0] : 0, e + 2 < NE ? (int)r[e + 2 < NE ? e + 2 : e].v[0] : 0,
                            e + 3 < NE ? (int)r[e + 3 < NE ? e + 3 : e].v[0] : 0};
                else
                    a = v4i{(int)r[e].v[0], (int)r[e].v[1], e + 1 < NE ? (int)r[e + 1 < NE ? e + 1 : e].v[0] : 0,
                            e + 1 < NE ? (int)r[e + 1 < NE ? e + 1 : e].v[1] : 0};
                D[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, NEG ? Bn[0] : Bp[0], D[0], 0, 0, 0);
                if constexpr (ND > 1) D[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, NEG ? Bn[1] : Bp[1], D[1], 0, 0, 0);
            }
        } else if constexpr (MXF && MT == 8) {
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                v8h a;
#pragma unroll
                for (int m = 0; m < 8; ++m) a[m] = r[e].v[m];
                Df[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, NEG ? Bnf[0] : Bpf[0], Df[0], 0, 0, 0);
                if constexpr (ND > 1) Df[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, NEG ? Bnf[1] : Bpf[1], Df[1], 0, 0, 0);
            }
        } else if constexpr (MXF) {
#pragma unroll
            for (int e = 0; e < NE; e += 2) {
                v8h a;
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    a[m] = r[e].v[m];
                    a[4 + m] = e + 1 < NE ? r[e + 1 < NE ? e + 1 : e].v[m] : (_Float16)0.0f;
                }
                Df[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, NEG ? Bnf[0] : Bpf[0], Df[0], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                if constexpr (sizeof(Act) == 1) {
                    acc[0] = NEG ? acc[0] - (int)r[e].v[0] : acc[0] + (int)r[e].v[0];
                } else {
#pragma unroll
                    for (int m = 0; m < MT; ++m) acc[m] = NEG ? acc[m] - (float)r[e].v[m] : acc[m] + (float)r[e].v[m];
                }
            }
        }
    }

    // Pin the sums once per round.  Integer adds may be reassociated freely, and without
    // this the compiler keeps every gathered value of every round alive to sum them in
    // one tree at the end.  (The matrix-unit sums are chained by their accumulator.)
    __device__ __forceinline__ void pin()
    {
        if constexpr (!MX && !MXF) {
#pragma unroll
            for (int m = 0; m < MT; ++m) asm volatile("" : "+v"(acc[m]));
        }
    }
};

// Stream flavours (MODE):
//   0  u16 row indices (already multiplied by 4 when PRE)
//   1  signed 8-bit gaps in rows; each lane walks a contiguous run of the sorted list in the
//      order the host scheduled (256-byte task header: first row of every lane and sign)
//   2  unsigned 16-bit gaps, runs walked in ascending order
// VAR (template flag of the kernels): ragged tasks.  The stream starts with a
// table of per-task entry counts and the tasks sit at a fixed stride; lists
// shorter than their task's count are padded with entries on the zero rows
// behind the tile.
template <int MODE> struct Flavour {
    static constexpr bool GAP8 = MODE == 1;
    static constexpr bool GAP16 = MODE == 2;
    static constexpr int HDR = MODE == 0 ? 0 : 256;
    static constexpr int ESZ = GAP8 ? 1 : 2;  // bytes per stream entry
};
constexpr int RAGGED_PREAMBLE = 16;  // {magic, tasks, n_max, n_min} in front of the u16 count table

// run += sign-extended byte B of d, in one SDWA add.  The sum goes to a register of its own: with byte rows
// it is the gather address as it stands, and an add in place would cost a copy per entry.
template <int B> __device__ __forceinline__ void add_signed_byte(u32 &run, u32 d)
{
    u32 next;
    if constexpr (B == 0)
        asm("v_add_u32_sdwa %0, sext(%1), %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0 src1_sel:DWORD" : "=v"(next) : "v"(d), "v"(run));
    else if constexpr (B == 1)
        asm("v_add_u32_sdwa %0, sext(%1), %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1 src1_sel:DWORD" : "=v"(next) : "v"(d), "v"(run));
    else if constexpr (B == 2)
        asm("v_add_u32_sdwa %0, sext(%1), %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2 src1_sel:DWORD" : "=v"(next) : "v"(d), "v"(run));
    else
        asm("v_add_u32_sdwa %0, sext(%1), %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3 src1_sel:DWORD" : "=v"(next) : "v"(d), "v"(run));
    run = next;
}

// the byte at an absolute LDS address
typedef __attribute__((address_space(3))) const unsigned char *lds_ptr;
template <class Raw> __device__ __forceinline__ Raw lds_byte(u32 addr)
{
    Raw r;
    r.v[0] = *reinterpret_cast<__attribute__((address_space(3))) const int8_t *>((lds_ptr)(size_t)addr);
    return r;
}
__device__ __forceinline__ u32 lds_address(const unsigned char *p) { return (u32)(size_t)(lds_ptr)p; }

// `run` is the current row of a gap stream: the row index itself with 8-bit gaps,
// the byte offset of the row's slot in the tile with 16-bit gaps.  fetch() turns
// the low NBYTES of `d` into tile reads; the adds follow separately so that the
// compiler is free to keep several reads in flight.
template <class S, int MODE, bool PRE, int NBYTES>
__device__ __forceinline__ void fetch(const unsigned char *lds, u32 d, u32 &run, typename S::Raw *r)
{
    constexpr int SH = ilog2(S::SLOT);
    if constexpr (Flavour<MODE>::GAP8 && S::SLOT == 1) {
        // byte rows: `run` is the LDS address of the row's byte itself (the tile's own address is in it)
        add_signed_byte<0>(run, d);
        r[0] = lds_byte<typename S::Raw>(run);
        if constexpr (NBYTES > 1) {
            add_signed_byte<1>(run, d);
            r[1] = lds_byte<typename S::Raw>(run);
        }
        if constexpr (NBYTES > 2) {
            add_signed_byte<2>(run, d);
            r[2] = lds_byte<typename S::Raw>(run);
            add_signed_byte<3>(run, d);
            r[3] = lds_byte<typename S::Raw>(run);
        }
    } else if constexpr (Flavour<MODE>::GAP8) {
        add_signed_byte<0>(run, d);
        r[0] = S::load(lds, run << SH);
        if constexpr (NBYTES > 1) {
            add_signed_byte<1>(run, d);
            r[1] = S::load(lds, run << SH);
        }
        if constexpr (NBYTES > 2) {
            add_signed_byte<2>(run, d);
            r[2] = S::load(lds, run << SH);
            add_signed_byte<3>(run, d);
            r[3] = S::load(lds, run << SH);
        }
    } else {
#pragma unroll
        for (int h = 0; h < NBYTES / 2; ++h) {
            u32 f = h ? (d >> 16) : (d & 0xffffu);
            if constexpr (Flavour<MODE>::GAP16) {
                run += f << SH;
                r[h] = S::load(lds, run);
            } else {
                r[h] = S::load(lds, f << (PRE ? SH - 2 : SH));
            }
        }
    }
}

template <class S, int MODE, bool PRE, bool NEG, int NBYTES>
__device__ __forceinline__ void consume(const unsigned char *lds, u32 d, u32 &run, S &acc)
{
    constexpr int NE = NBYTES / Flavour<MODE>::ESZ;
    typename S::Raw r[NE];
    fetch<S, MODE, PRE, NBYTES>(lds, d, run, r);
    acc.template accum_n<NEG, NE>(r);
}

template <class S, int MODE, bool PRE, bool NEG>
__device__ __forceinline__ void consume16(const unsigned char *lds, const uint4 &v, u32 &run, S &acc)
{
    constexpr int NE = 4 / Flavour<MODE>::ESZ;  // entries per dword
    typename S::Raw r[4 * NE];
    fetch<S, MODE, PRE, 4>(lds, v.x, run, r);
    fetch<S, MODE, PRE, 4>(lds, v.y, run, r + NE);
    fetch<S, MODE, PRE, 4>(lds, v.z, run, r + 2 * NE);
    fetch<S, MODE, PRE, 4>(lds, v.w, run, r + 3 * NE);
    acc.template accum_n<NEG, 4 * NE>(r);
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

// The same with the two output pairs exchanged where `odd`: o[0], o[1] = k+2, k+3 and o[2], o[3] = k, k+1.
// The byte selectors come from registers, so the exchange costs no instruction.
__device__ __forceinline__ void transpose4x4_swap(u32 r0, u32 r1, u32 r2, u32 r3, bool odd, u32 (&o)[4])
{
    const u32 s0 = odd ? 0x07030602u : 0x05010400u, s1 = odd ? 0x05010400u : 0x07030602u;
    u32 a = __builtin_amdgcn_perm(r1, r0, s0), b = __builtin_amdgcn_perm(r1, r0, s1);
    u32 c = __builtin_amdgcn_perm(r3, r2, s0), d = __builtin_amdgcn_perm(r3, r2, s1);
    o[0] = __builtin_amdgcn_perm(c, a, 0x05040100u);
    o[1] = __builtin_amdgcn_perm(c, a, 0x07060302u);
    o[2] = __builtin_amdgcn_perm(d, b, 0x05040100u);
    o[3] = __builtin_amdgcn_perm(d, b, 0x07060302u);
}
__device__ __forceinline__ void swap_if(bool c, u32 &a, u32 &b)
{
    const u32 x = c ? b : a, y = c ? a : b;
    a = x;
    b = y;
}

__device__ __forceinline__ u32 comp(const uint4 &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }
__device__ __forceinline__ u32 f2u(float f) { return __builtin_bit_cast(u32, f); }
__device__ __forceinline__ float h2f(u32 d, int hi) { return (float)__builtin_bit_cast(_Float16, (unsigned short)(hi ? d >> 16 : d & 0xffffu)); }

// Running maxima of |x| as 16-bit patterns, two per register: for fp16 and bf16 alike, clearing
// the sign bit leaves patterns that order like the magnitudes they encode (Inf and NaN on top).
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32 pk_absmax16(u32 mx, u32 d)
{
    return __builtin_bit_cast(u32, __builtin_elementwise_max(__builtin_bit_cast(u16x2, mx), __builtin_bit_cast(u16x2, d & 0x7fff7fffu)));
}
__device__ __forceinline__ u32 pk_absmax16(u32 mx, const uint4 &v) { return pk_absmax16(pk_absmax16(pk_absmax16(pk_absmax16(mx, v.x), v.y), v.z), v.w); }
// either half holds the pattern of an fp16 Inf or NaN
__device__ __forceinline__ bool pk_nonfinite16(u32 mx) { return (mx & 0xffffu) >= 0x7c00u || (mx >> 16) >= 0x7c00u; }

// Byte offset, inside a task's rounds, of entry j of `lane` for `sign` (0 = +1 list): full rounds of
// 16 bytes per lane and sign, then at most one round each of 8, 4, 2 (and 1) bytes per lane.
template <int ESZ> __device__ __forceinline__ u32 entry_offset(int n_lane, int sign, int lane, int j)
{
    constexpr int E16 = 16 / ESZ;
    const int full = n_lane / E16;
    if (j < full * E16) return (u32)(j / E16) * 2048u + (u32)sign * 1024u + (u32)lane * 16u + (u32)(j % E16) * ESZ;
    u32 base = (u32)full * 2048u;
    const int rem = n_lane - full * E16;
    int first = full * E16;
#pragma unroll
    for (int w = 8; w >= ESZ; w /= 2) {
        const int cnt = w / ESZ;
        if (rem & cnt) {
            if (j < first + cnt) return base + (u32)sign * 64u * w + (u32)lane * w + (u32)(j - first) * ESZ;
            first += cnt;
            base += 128u * w;
        }
    }
    return base;
}

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
        if constexpr (is_byte_rows<Act>()) {
            t[item] = r[0];
        } else if constexpr (sizeof(Act) == 1 && MT == 1) {  // 16 bytes -> 16 sign-extended dwords
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int d = (int)comp(r[0], j);
                t[4 * item + j] = make_uint4((u32)((d << 24) >> 24), (u32)((d << 16) >> 24), (u32)((d << 8) >> 24), (u32)(d >> 24));
            }
        } else if constexpr (sizeof(Act) == 1 && MT == 4) {  // [k][4 bytes]
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32 o[4];
                transpose4x4(comp(r[0], j), comp(r[1], j), comp(r[2], j), comp(r[3], j), o);
                t[4 * item + j] = make_uint4(o[0], o[1], o[2], o[3]);
            }
        } else if constexpr (sizeof(Act) == 1) {  // [k][8 bytes]
            // An item is 128 bytes of the tile, so the lanes of a 16-byte write all start on the same bank
            // and the write takes eight passes (counted: three quarters of this kernel's LDS conflict
            // cycles at K = 13824).  Lane `item` therefore writes its eight 16-byte chunks in the order
            // c ^ (item & 7): eight neighbouring lanes then cover eight different chunks.  Bit 0 of the
            // order is an exchange of byte selectors in the transposition, bits 1-2 a conditional
            // exchange of the loaded dwords.
            const u32 rho = (u32)item & 7u;
            u32 x[8][4];
#pragma unroll
            for (int m = 0; m < 8; ++m) {
#pragma unroll
                for (int j = 0; j < 4; ++j) x[m][j] = comp(r[m], j);
                swap_if(rho & 2u, x[m][0], x[m][1]);
                swap_if(rho & 2u, x[m][2], x[m][3]);
                swap_if(rho & 4u, x[m][0], x[m][2]);
                swap_if(rho & 4u, x[m][1], x[m][3]);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {  // x[m][j] = dword j ^ (rho >> 1) of row m
                u32 o[4], q[4];
                transpose4x4_swap(x[0][j], x[1][j], x[2][j], x[3][j], rho & 1u, o);
                transpose4x4_swap(x[4][j], x[5][j], x[6][j], x[7][j], rho & 1u, q);
                t[8 * item + ((2 * j) ^ rho)] = make_uint4(o[0], q[0], o[1], q[1]);
                t[8 * item + ((2 * j + 1) ^ rho)] = make_uint4(o[2], q[2], o[3], q[3]);
            }
        } else if constexpr (sizeof(Act) == 2 && MT == 1) {  // 16 halves -> 16 floats
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32 d0 = comp(r[j / 2], (2 * j) % 4), d1 = comp(r[j / 2], (2 * j + 1) % 4);
                t[4 * item + j] = make_uint4(f2u(h2f(d0, 0)), f2u(h2f(d0, 1)), f2u(h2f(d1, 0)), f2u(h2f(d1, 1)));
            }
        } else if constexpr (sizeof(Act) == 2 && MT == 8) {  // [k][8 halves]; r[2m+h] = row m, halves 8h..8h+7
#pragma unroll
            for (int i = 0; i < 8; ++i) {  // k = 16*item + 2i, 2i+1
                u32 d[8];
#pragma unroll
                for (int m = 0; m < 8; ++m) d[m] = comp(r[2 * m + i / 4], i % 4);
                t[16 * item + 2 * i] = make_uint4((d[0] & 0xffffu) | (d[1] << 16), (d[2] & 0xffffu) | (d[3] << 16),
                                                  (d[4] & 0xffffu) | (d[5] << 16), (d[6] & 0xffffu) | (d[7] << 16));
                t[16 * item + 2 * i + 1] = make_uint4((d[0] >> 16) | (d[1] & 0xffff0000u), (d[2] >> 16) | (d[3] & 0xffff0000u),
                                                      (d[4] >> 16) | (d[5] & 0xffff0000u), (d[6] >> 16) | (d[7] & 0xffff0000u));
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

struct ListParams {
    const uint8_t *w;
    const void *X;
    void *C;
    int M, K, N;
    int n_lane, tasks, logL, W;  // n_lane: entries per lane per sign (ragged streams: the smallest over all tasks)
    int task_stride;             // ragged streams: bytes between tasks
    int counts_bytes;            // ragged streams: bytes of the count table (with its preamble) in front of the tasks
    int iters;  // tasks each wavefront walks: ceil(tasks / (gridDim.x * waves))
    int quant;      // quantising kernels: X holds 1 = fp16, 2 = bf16 values
    float w_scale;  // quantising kernels: factor applied to every output
    int stones;     // 8-bit gap streams of tile positions: the tile keeps 16 zero slots behind every 96 rows
    // blockDim.x and gridDim.x, handed over as arguments: the built-ins are read from the dispatch's implicit arguments
    // with a vector load whose address waits for a scalar load, two memory round trips in a row before the kernel's
    // first activation or stream load is issued; these arrive with the other arguments in one
    int threads, grid_x;
    const float *inv;  // kernels for rows quantised beforehand: the rows' 1/s (a / 127), applied to every output
};

// rows of the activation tile in front of its 64 trailing zero rows
static inline int lists_tile_rows(const GemvArgs &a) { return a.stones ? stone_tile_rows(a.K) : a.K; }

constexpr int LISTS_MAX_WAVES = 8;  // 512 threads: two wavefronts per SIMD, 256 VGPRs each
// Multi-row int8 tiles do several times the arithmetic per stream byte, and a large K leaves
// room for one workgroup per CU only, so that workgroup has to bring the wavefronts that fill
// the four SIMDs itself: 1024 threads, four wavefronts per SIMD, 128 VGPRs each.
// The same for four fp32 rows (16-byte slots, a tile as large as eight int8 rows' twice over: headline shape, M=4, 32 GEMVs
// per launch, 8 -> 16 wavefronts: u16 3.66 -> 3.58 us per GEMV, gap stream 3.48 -> 3.26).  Eight fp16 rows stay at 512
// threads: their gathers of 16 entries x 16 bytes do not fit 128 registers (up to 272 bytes of scratch per lane).
// Kernels that run at 128 registers keep a ring of four rounds and no straight-line body beyond four.
template <typename Act, int MT> constexpr bool lists_short_of_registers() { return (MT == 8 && sizeof(Act) == 1) || (MT == 4 && sizeof(Act) == 4); }
template <typename Act, int MT, bool QUANT> constexpr int lists_max_waves()
{
    return ((sizeof(Act) == 1 && MT >= 4) || lists_short_of_registers<Act, MT>()) && !QUANT ? 16 : LISTS_MAX_WAVES;
}

// LDS a workgroup of `waves` wavefronts keeps behind the activation tile: the per-wavefront sums of
// columns that span wavefronts, and for fp16 tiles summed on the matrix unit one flag per wavefront.
template <typename Act, int MT> constexpr size_t lists_behind_tile(int waves)
{
    return (size_t)waves * MT * 4 + (sizeof(Act) == 2 && MT > 1 ? (size_t)waves * 4 : 0);
}

// One round of a task's stream: 16 bytes per lane of the +1 list and of the -1 list.
struct Round {
    uint4 p, q;
};
// The stream is read exactly once per GEMV: non-temporal loads keep it from
// pushing the activation vector (re-read by every workgroup) out of L2.
typedef u32 v4u __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 stream_load(const uint4 *p)
{
    v4u t = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ Round load_round(const uint4 *wp, int r)
{
    Round x;
    x.p = stream_load(wp + (2 * r) * 64);
    x.q = stream_load(wp + (2 * r + 1) * 64);
    return x;
}

// Activation quantisation in front of the integer GEMV (per row: s = 127 / max(|x|, 1e-5),
// q = clamp(rint(x * s), -127, 127)) for the kernels that take fp16 / bf16 rows and
// hand back floats.  Item = 16 consecutive k of all MT rows, as in Stager.
template <int MT> struct Quantiser {
    static constexpr int HOLD = MT <= 4 ? 2 : 0;  // items a thread keeps in registers between the two passes (the rest is read twice)

    // 2 x 16 bytes per row: the item's 16 values of row m0 + m (rows past M read as zero)
    static __device__ __forceinline__ void load(const unsigned short *X, int M, int K, int m0, int item, uint4 (&r)[2 * MT])
    {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                r[2 * m + j] = (m0 + m < M) ? reinterpret_cast<const uint4 *>(X + (size_t)(m0 + m) * K)[(size_t)item * 2 + j]
                                            : make_uint4(0, 0, 0, 0);
    }
    // running maxima of |x| per row, as packed bit patterns
    static __device__ __forceinline__ void absmax(const uint4 (&r)[2 * MT], u32 (&mx)[MT])
    {
#pragma unroll
        for (int m = 0; m < MT; ++m) mx[m] = pk_absmax16(pk_absmax16(mx[m], r[2 * m]), r[2 * m + 1]);
    }
    static __device__ __forceinline__ float magnitude(u32 packed, int kind)
    {
        const u32 bits = (packed >> 16) > (packed & 0xffffu) ? packed >> 16 : packed & 0xffffu;
        return kind == 2 ? __builtin_bit_cast(float, bits << 16) : (float)__builtin_bit_cast(_Float16, (unsigned short)bits);
    }
    template <int KIND> static __device__ __forceinline__ float value(u32 d, int hi)
    {
        if constexpr (KIND == 2) return __builtin_bit_cast(float, hi ? d & 0xffff0000u : d << 16);
        return (float)__builtin_bit_cast(_Float16, (unsigned short)(hi ? d >> 16 : d & 0xffffu));
    }
    // -> the 16 int8 of every row, packed as the int8 kernels' own activation loads would deliver them.
    // No clamp: |x| <= a and s = 127 / a keep |x * s| below 127.5.
    template <int KIND> static __device__ __forceinline__ void quantise_as(const uint4 (&r)[2 * MT], const float (&s)[MT], uint4 (&q)[MT])
    {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            u32 w[4] = {0, 0, 0, 0};
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int v = (int)__builtin_rintf(value<KIND>(comp(r[2 * m + e / 8], (e / 2) % 4), e & 1) * s[m]);
                w[e / 4] |= ((u32)v & 0xffu) << (8 * (e % 4));
            }
            q[m] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
    static __device__ __forceinline__ void quantise(const uint4 (&r)[2 * MT], int kind, const float (&s)[MT], uint4 (&q)[MT])
    {
        if (kind == 2)
            quantise_as<2>(r, s, q);
        else
            quantise_as<1>(r, s, q);
    }
};

// QUANT: 0 int8 / float rows as they come; 1 fp16 / bf16 rows quantised to int8 while the tile is staged, floats out;
// 2 int8 rows quantised beforehand (ListParams::inv holds the rows' 1/s), floats out
template <typename Act, int MT, int MODE, bool PRE, bool VAR, int QUANT = 0, bool MERGED = false>
struct ListsBody {
    typedef Sums<Act, MT, false, MERGED> SumsT;
    typedef typename Acc<Act>::type A;
    typedef Stager<Act, MT> St;
    static constexpr int SLOT_OF = slot_bytes<Act, MT>();
    typedef Flavour<MODE> Fl;
    static constexpr int ESZ = Fl::ESZ;               // bytes per stream entry
    static constexpr int E16 = 16 / ESZ;              // entries per 16-byte load
    static constexpr int HDR = Fl::HDR;               // first rows of a gap-stream task
    static constexpr bool GAPS = Fl::GAP8 || Fl::GAP16;
    static constexpr int ZROWS = 64;                  // zero slots behind the tile (row K, and the padding rows)
    static constexpr int SH = ilog2(SLOT_OF);
    static constexpr int SLOT = SLOT_OF;
    // (four int8 rows also run 16 wavefronts per workgroup at 128 registers: their ragged kernels and the ones on 16-bit gaps
    // keep the ring of four as well -- with eight they spilled 170-180 bytes per lane)
    static constexpr bool TIGHT = lists_short_of_registers<Act, MT>() || (sizeof(Act) == 1 && !is_byte_rows<Act>() && MT == 4 && (VAR || Fl::GAP16));
    static constexpr int XMAX = VAR ? (TIGHT ? 1 : 2) : 0;  // ragged tasks on the straight-line path: full rounds beyond RF a task may have
    static constexpr int RING = TIGHT ? 4 : 8;      // rounds in flight on the generic path (8-row kernels run 10-16 wavefronts per CU and are short of registers)
    static constexpr int EARLY = MT >= 4 ? 4 : 2;     // rounds requested before the activation tile is complete (multi-row tiles take longer to stage)

    static __device__ __forceinline__ void eat(const unsigned char *smem, const Round &x, u32 &runp, u32 &runq, SumsT &acc)
    {
        consume16<SumsT, MODE, PRE, false>(smem, x.p, runp, acc);
        consume16<SumsT, MODE, PRE, true>(smem, x.q, runq, acc);
        acc.pin();  // (and the running rows)
        if constexpr (GAPS) asm volatile("" : "+v"(runp), "+v"(runq));
    }

    // fp16 tiles summed on the matrix unit have a VALU twin for workgroups whose tile holds an Inf or NaN
    static constexpr bool TWIN = SumsT::MXF;
    typedef Sums<Act, MT, TWIN> Plain;

    // One task summed on the VALU with a single round in flight (the twin's path: rare, so small rather than fast).
    static __device__ __forceinline__ void walk_plain(const unsigned char *smem, const uint8_t *tb, int lane, int n_lane, u32 runp, u32 runq,
                                                      Plain &acc)
    {
        const uint4 *wp = reinterpret_cast<const uint4 *>(tb + HDR) + lane;
        const int R = n_lane / E16;
#pragma unroll 1
        for (int r = 0; r < R; ++r) {
            const Round x = load_round(wp, r);
            consume16<Plain, MODE, PRE, false>(smem, x.p, runp, acc);
            consume16<Plain, MODE, PRE, true>(smem, x.q, runq, acc);
        }
#pragma unroll 1
        for (int j = R * E16; j < n_lane; ++j) {
            const uint8_t *ep = tb + HDR + entry_offset<ESZ>(n_lane, 0, lane, j), *eq = tb + HDR + entry_offset<ESZ>(n_lane, 1, lane, j);
            const u32 fp = ESZ == 1 ? (u32)*ep : (u32)*reinterpret_cast<const unsigned short *>(ep);
            const u32 fq = ESZ == 1 ? (u32)*eq : (u32)*reinterpret_cast<const unsigned short *>(eq);
            consume<Plain, MODE, PRE, false, ESZ>(smem, fp, runp, acc);
            consume<Plain, MODE, PRE, true, ESZ>(smem, fq, runq, acc);
        }
    }

    // Per-lane sums of a task -> column totals: folded over the L lanes of a column, then written (one
    // wavefront per column or less) or left in `part` for the second pass (columns that span wavefronts).
    static __device__ __forceinline__ void store_lane_sums(const ListParams &p, A (&v)[MT], A *part, const float (&back)[MT], bool active,
                                                           int task, int lane, int wave, int m0)
    {
        A *C = reinterpret_cast<A *>(p.C);
        float *Cf = reinterpret_cast<float *>(p.C);  // quantising kernels: acc / s * w_scale
        const int L = 1 << p.logL;
#pragma unroll
        for (int m = 0; m < MT; ++m) v[m] = lanes_sum(v[m], p.logL);
        if (p.W == 1) {
            if (active && (lane & (L - 1)) == 0) {
                const int col = (task << (6 - p.logL)) + (lane >> p.logL);
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    if (m0 + m < p.M) {
                        if constexpr (QUANT != 0)
                            Cf[(size_t)(m0 + m) * p.N + col] = (float)v[m] * back[m] * p.w_scale;
                        else
                            C[(size_t)(m0 + m) * p.N + col] = v[m];
                    }
            }
        } else if (lane == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m) part[wave * MT + m] = v[m];
        }
    }

    // RF > 0: the task has exactly RF full rounds (ragged: RF to RF + XMAX) and
    // all of them live in registers, loaded and consumed in straight-line code
    // (so every wait on the stream is for one round only).  RF == 0: any number
    // of rounds, through a ring of RING rounds in flight.  RF == -1: no full round at all
    // (ragged: up to XMAX), only the tail.
    // SL > 0 (u16 lists, one int8 row, straight-line bodies): 1 << SL wavefronts of a workgroup share a task -- wavefront
    // j of them takes the rounds j, j + (1 << SL), ... (RF counts the rounds of ONE wavefront), the first one the tail as
    // well, and their per-column sums meet in LDS.  The launch then has 1 << SL times the wavefronts, each with that
    // fraction of the gathers left to do once the last bytes of its rounds have arrived.
    template <int RF, int SL = 0>
    static __device__ __forceinline__ void run(const ListParams &p, unsigned char *smem)
    {
        static_assert(SL == 0 || (RF > 0 && MODE == 0 && !VAR && QUANT != 1 && MT == 1 && sizeof(Act) == 1), "shared tasks: u16 lists, one int8 row");
        constexpr int NR = RF > 0 ? RF : 0;               // full rounds of the straight-line body (RF == -1: none, tails only)
        constexpr int NB = RF > 0 ? RF : RF == 0 ? RING : 1;
        // stepping-stone streams: item i (16 rows) goes to item i + i/6 of the tile, every seventh item stays zero
        const bool stones = Fl::GAP8 && VAR && p.stones;  // (only ragged 8-bit gap streams come with zero slots: nothing of this in the other kernels)
        const int tile_rows = stones ? STONE_BLOCK * ((p.K + STONE_ROWS - 1) / STONE_ROWS) : p.K;
        auto place = [&](int item) { return stones ? item + item / (STONE_ROWS / 16) : item; };
        A *part = reinterpret_cast<A *>(smem + (size_t)(tile_rows + ZROWS) * SLOT);
        const int tid = threadIdx.x, nt = p.threads;
        const int lane = tid & 63, wave = tid >> 6, waves = nt >> 6;
        const int m0 = blockIdx.y * MT;
        const size_t task_bytes = VAR ? (size_t)p.task_stride : HDR + (size_t)128 * ESZ * p.n_lane;
        const uint8_t *const tasks_base = p.w + (VAR ? p.counts_bytes : 0);
        const unsigned short *const counts = reinterpret_cast<const unsigned short *>(p.w + RAGGED_PREAMBLE);
        // ragged: tasks differ in length; p.n_lane is the shortest, which is all the prologue may assume
        const int R0 = p.n_lane / E16;
        int task = (blockIdx.x * waves + wave) >> SL;
        const int roff = wave & ((1 << SL) - 1);  // which of the task's wavefronts this one is
        const int task_step = (p.grid_x * waves) >> SL;
        const Act *X = reinterpret_cast<const Act *>(p.X);
        typedef Quantiser<MT> Q;
        const unsigned short *Xq = reinterpret_cast<const unsigned short *>(p.X);
        // quantising kernels: behind the per-wavefront sums, one row maximum per wavefront and the rows' 1/s
        float *qmax = reinterpret_cast<float *>(part + LISTS_MAX_WAVES * MT), *qinv = qmax + LISTS_MAX_WAVES * MT;

        // 1. every wavefront's activation loads enter the memory pipeline ahead of
        //    any stream load of the workgroup ...
        const int items = p.K / 16;
        uint4 xr[QUANT == 1 ? 1 : St::XI][St::NLOAD];
        uint4 xq[QUANT == 1 && Q::HOLD > 0 ? Q::HOLD : 1][2 * MT];
        if constexpr (QUANT == 1) {
#pragma unroll
            for (int i = 0; i < Q::HOLD; ++i) {
                const int item = tid + i * nt;
                Q::load(Xq, p.M, p.K, m0, item < items ? item : items - 1, xq[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < St::XI; ++i) {
                const int item = tid + i * nt;
                St::load(X, p.M, p.K, m0, item < items ? item : items - 1, xr[i]);
            }
        }
        u32 xmax = 0u;  // TWIN: largest |x| pattern this thread has staged
        // ragged: the first task's entry count travels with the activation loads, so it is there
        // long before the tile is; every later count is asked for one task ahead
        int n_ahead = p.n_lane;
        if constexpr (VAR) n_ahead = counts[task < p.tasks ? task : 0];

        // 2. ... then the first rounds of the first task's stream (gap streams: and the rows its lanes start from) ...
        Round buf[NB];
        u32 headp = 0, headq = 0;
        {
            const uint8_t *tb = tasks_base + (size_t)(task < p.tasks ? task : 0) * task_bytes;
            const uint4 *wp = reinterpret_cast<const uint4 *>(tb + HDR) + lane;
            if constexpr (GAPS) {
                headp = reinterpret_cast<const unsigned short *>(tb)[lane];
                headq = reinterpret_cast<const unsigned short *>(tb)[64 + lane];
            }
            if constexpr (RF > 0) {
#pragma unroll
                for (int i = 0; i < (RF < EARLY ? RF : EARLY); ++i) buf[i] = load_round(wp, (i << SL) + roff);
            } else if (RF == 0 && R0 > 0) {
#pragma unroll
                for (int i = 0; i < EARLY; ++i) buf[i] = load_round(wp, i < R0 ? i : R0 - 1);
            }
        }

        // 3. ... and the tile is written while the stream is still in flight.
        if constexpr (QUANT == 1) {
            // row maxima: own items (held, and beyond them re-read later), wavefront, workgroup
            u32 mb[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) mb[m] = 0u;
#pragma unroll
            for (int i = 0; i < Q::HOLD; ++i) Q::absmax(xq[i], mb);  // (a clamped duplicate changes no maximum)
            for (int item = tid + Q::HOLD * nt; item < items; item += nt) {
                uint4 r[2 * MT];
                Q::load(Xq, p.M, p.K, m0, item, r);
                Q::absmax(r, mb);
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                float mx = Q::magnitude(mb[m], p.quant);
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
                if (lane == 0) qmax[wave * MT + m] = mx;
            }
            __syncthreads();
            float sc[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                float a = 0.f;
                for (int w = 0; w < waves; ++w) a = fmaxf(a, qmax[w * MT + m]);
                a = fmaxf(a, 1e-5f);
                sc[m] = 127.0f / a;
                if (tid == 0) qinv[m] = a / 127.0f;
            }
#pragma unroll
            for (int i = 0; i < Q::HOLD; ++i)
                if (tid + i * nt < items) {
                    Q::quantise(xq[i], p.quant, sc, xr[0]);
                    St::store(smem, place(tid + i * nt), xr[0]);
                }
            for (int item = tid + Q::HOLD * nt; item < items; item += nt) {
                uint4 r[2 * MT];
                Q::load(Xq, p.M, p.K, m0, item, r);
                Q::quantise(r, p.quant, sc, xr[0]);
                St::store(smem, place(item), xr[0]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < St::XI; ++i)
                if (tid + i * nt < items) St::store(smem, place(tid + i * nt), xr[i]);
            if constexpr (TWIN) {
#pragma unroll
                for (int i = 0; i < St::XI; ++i)
#pragma unroll
                    for (int j = 0; j < St::NLOAD; ++j) xmax = pk_absmax16(xmax, xr[i][j]);
            }
        }
        if constexpr (RF > EARLY) {
            const uint4 *wp = reinterpret_cast<const uint4 *>(tasks_base + (size_t)(task < p.tasks ? task : 0) * task_bytes + HDR) + lane;
#pragma unroll
            for (int i = EARLY; i < RF; ++i) buf[i] = load_round(wp, (i << SL) + roff);
        } else if constexpr (RF == 0) {
            if (R0 > 0) {
                const uint4 *wp = reinterpret_cast<const uint4 *>(tasks_base + (size_t)(task < p.tasks ? task : 0) * task_bytes + HDR) + lane;
#pragma unroll
                for (int i = EARLY; i < RING; ++i) buf[i] = load_round(wp, i < R0 ? i : R0 - 1);
            }
        }
        if constexpr (QUANT != 1) {
            for (int item = tid + St::XI * nt; item < items; item += nt) {
                uint4 r[St::NLOAD];
                St::load(X, p.M, p.K, m0, item, r);
                St::store(smem, place(item), r);
                if constexpr (TWIN) {
#pragma unroll
                    for (int j = 0; j < St::NLOAD; ++j) xmax = pk_absmax16(xmax, r[j]);
                }
            }
        }
        // rows K.. read as zero
        for (int i = tid; i < ZROWS * SLOT / 4; i += nt)
            reinterpret_cast<u32 *>(smem + (size_t)tile_rows * SLOT)[i] = 0u;
        if (stones) {
            // the zero slots inside the tile: the last item of every block, and what the last block holds beyond row K-1
            constexpr int DW = 4 * SLOT;                // dwords per item
            constexpr int BI = STONE_BLOCK / 16;        // items per block
            const int blocks = tile_rows / STONE_BLOCK;
            u32 *t32 = reinterpret_cast<u32 *>(smem);
            for (int i = tid; i < blocks * DW; i += nt) t32[((i / DW + 1) * BI - 1) * DW + i % DW] = 0u;
            const int first_free = place(items - 1) + 1, past = blocks * BI - 1;  // items of the last block without rows
            for (int i = tid; i < (past - first_free) * DW; i += nt) t32[first_free * DW + i] = 0u;
        }
        // TWIN: one flag per wavefront behind the per-wavefront sums, folded by every thread after the barrier
        u32 *nf_flags = reinterpret_cast<u32 *>(part + waves * MT);
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

        A *C = reinterpret_cast<A *>(p.C);
        float *Cf = reinterpret_cast<float *>(p.C);  // quantising kernels: acc / s * w_scale
        float back[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) back[m] = QUANT == 1 ? qinv[m] : QUANT == 2 ? (m0 + m < p.M ? p.inv[m0 + m] : 0.f) : 0.f;
        // rows quantised beforehand, matrix-unit epilogues: lane l writes row l & (MT - 1); its 1/s is fetched once, here
        float inv_lane = 0.f;
        if constexpr (QUANT == 2) inv_lane = m0 + (lane & (MT - 1)) < p.M ? p.inv[m0 + (lane & (MT - 1))] : 0.f;
        for (int it = 0; it < p.iters; ++it, task += task_step) {
            const bool active = task < p.tasks;
            const uint8_t *tb = tasks_base + (size_t)(active ? task : 0) * task_bytes;
            const uint4 *wp = reinterpret_cast<const uint4 *>(tb + HDR) + lane;
            u32 runp = 0, runq = 0;
            int n_lane = p.n_lane;
            // AHEAD: while a task is walked, the next one's first rows and rounds are requested into the registers that
            // come free, so a wavefront that walks several tasks never waits with nothing in flight.  Four int8 rows
            // on gap streams only (tasks of one length, straight-line path), where it pays: headline shape, 32 GEMVs per
            // launch, 10 tasks per wavefront 2.00 -> 1.88 us per GEMV; and eight int8 rows with one result tile, which leaves
            // the registers for it (K=13824 N=5120 split_k=64, 14 GEMVs per launch: 8.9 -> 8.45 us; with two result tiles the
            // kernel spilled and lost, 2.09 -> 2.29 us).  Measured and left out: four fp16 rows (2.18 -> 2.56 us), byte rows
            // (1.70 -> 1.79 us), u16 lists (3.2 -> 13.6 us at M=4).
            constexpr bool AHEAD = RF != 0 && !VAR && !QUANT && (MT == 4 || (MT == 8 && MERGED)) && sizeof(Act) == 1 && MODE != 0;
            const int task_next = task + task_step;
            const uint8_t *tb_next = tasks_base + (size_t)(task_next < p.tasks ? task_next : 0) * task_bytes;
            if constexpr (GAPS) {
                if ((!AHEAD || (TWIN && plain)) && it > 0) {
                    headp = reinterpret_cast<const unsigned short *>(tb)[lane];
                    headq = reinterpret_cast<const unsigned short *>(tb)[64 + lane];
                }
                runp = headp << (Fl::GAP8 ? 0 : SH);
                runq = headq << (Fl::GAP8 ? 0 : SH);
                if constexpr (is_byte_rows<Act>()) runp += lds_address(smem), runq += lds_address(smem);
            }
            if constexpr (VAR) {
                n_lane = __builtin_amdgcn_readfirstlane(n_ahead);
                const int nxt = task + task_step;
                n_ahead = counts[nxt < p.tasks ? nxt : 0];
            }
            const int R = n_lane / E16, rem = SL > 0 && roff != 0 ? 0 : n_lane - R * E16;  // (R: rounds of the whole task)
            if (TWIN && plain) {
                Plain pacc;
                pacc.init();
                walk_plain(smem, tb, lane, n_lane, runp, runq, pacc);
                store_lane_sums(p, pacc.acc, part, back, active, task, lane, wave, m0);
            } else {
            SumsT acc;
            acc.init(p.logL);

            if constexpr (RF != 0) {
                if (!AHEAD && it > 0) {
#pragma unroll
                    for (int i = 0; i < NR; ++i) buf[i] = load_round(wp, (i << SL) + roff);
                }
            } else {
                // ring of RING rounds, loads clamped to the task's last round so that they stay unconditional
                if (it > 0) {
                    if (R > 0) {
#pragma unroll
                        for (int i = 0; i < RING; ++i) buf[i] = load_round(wp, i < R ? i : R - 1);
                    }
                } else if (VAR) {  // this task may be longer than the shortest one the prologue assumed
#pragma unroll
                    for (int i = 0; i < RING; ++i)
                        if (i >= R0 && i < R) buf[i] = load_round(wp, i);
                }
            }
            Round xb[XMAX > 0 ? XMAX : 1];
            if constexpr (RF != 0 && XMAX > 0) {
#pragma unroll
                for (int x = 0; x < XMAX; ++x)
                    if (NR + x < R) xb[x] = load_round(wp, NR + x);
            }
            // ragged tail, requested now and eaten last: at most one round each of 8, 4, 2 (and 1) bytes per lane
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
            if constexpr (RF == 0) {
                int base = 0;
                for (; base + 2 * RING <= R; base += RING) {  // steady state: eat a round, refill its slot RING rounds ahead
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
                for (int i = 0; i < RING; ++i) {
                    if (base + i < R) eat(smem, buf[i], runp, runq, acc);
                }
            } else {
                if (AHEAD && it + 1 < p.iters) {
                    if constexpr (GAPS) {
                        headp = reinterpret_cast<const unsigned short *>(tb_next)[lane];
                        headq = reinterpret_cast<const unsigned short *>(tb_next)[64 + lane];
                    }
                    const uint4 *wn = reinterpret_cast<const uint4 *>(tb_next + HDR) + lane;
#pragma unroll
                    for (int i = 0; i < NR; ++i) {
                        eat(smem, buf[i], runp, runq, acc);
                        buf[i] = load_round(wn, i);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NR; ++i) eat(smem, buf[i], runp, runq, acc);
                }
                if constexpr (XMAX > 0) {
#pragma unroll
                    for (int x = 0; x < XMAX; ++x)
                        if (NR + x < R) eat(smem, xb[x], runp, runq, acc);
                }
            }
            if (rem) {
                if (rem & (8 / ESZ)) {
                    consume<SumsT, MODE, PRE, false, 4>(smem, t8p.x, runp, acc);
                    consume<SumsT, MODE, PRE, false, 4>(smem, t8p.y, runp, acc);
                    consume<SumsT, MODE, PRE, true, 4>(smem, t8q.x, runq, acc);
                    consume<SumsT, MODE, PRE, true, 4>(smem, t8q.y, runq, acc);
                }
                if (rem & (4 / ESZ)) {
                    consume<SumsT, MODE, PRE, false, 4>(smem, t4p, runp, acc);
                    consume<SumsT, MODE, PRE, true, 4>(smem, t4q, runq, acc);
                }
                if (rem & (2 / ESZ)) {
                    consume<SumsT, MODE, PRE, false, 2>(smem, t2p, runp, acc);
                    consume<SumsT, MODE, PRE, true, 2>(smem, t2q, runq, acc);
                }
                if constexpr (ESZ == 1) {
                    if (rem & 1) {
                        consume<SumsT, MODE, PRE, false, 1>(smem, t1p, runp, acc);
                        consume<SumsT, MODE, PRE, true, 1>(smem, t1q, runq, acc);
                    }
                }
            }

            if constexpr (SumsT::MX || SumsT::MXF) {
                // Result tile x, lane l, register r: the sum of source lane 16 g + 4 (l >> 4) + r and row m, where
                // MT = 4: g = (l >> 2) & 3, m = l & 3;  MT = 8: g = 2 x + ((l >> 3) & 1), m = l & 7.
                // The four registers are neighbouring lanes of one column; the rest of a column's L lanes is
                // spread over lane bits 4, 5 (the quarter) and, from L = 32, the bits that hold g.
                constexpr int ND = SumsT::ND;
                const int logL = p.logL;
                if constexpr (MERGED) {
                    {
                        // one tile: lane l, register r = rows i = 4 (l >> 4) + r, result column j = l & 15 holds activation
                        // row j & 7 of the task's column j >> 3; the 16 i are the column's lanes i, i+16 (, i+32, i+48)
                        A v = acc.tile_sum(0);
                        v += swz16(v);
                        v += __shfl_xor(v, 32, 64);
                        const int m = lane & 7;
                        if (p.W == 1) {
                            if (active && lane < (logL == 5 ? 16 : 8) && m0 + m < p.M) {
                                const int col = (task << (6 - logL)) + (lane >> 3);
                                if constexpr (QUANT != 0)
                                    Cf[(size_t)(m0 + m) * p.N + col] = (float)v * (QUANT == 1 ? qinv[m] : inv_lane) * p.w_scale;
                                else
                                    C[(size_t)(m0 + m) * p.N + col] = v;
                            }
                        } else if (lane < MT) {
                            part[wave * MT + lane] = v;
                        }
                    }
                } else {
                A t[ND];
#pragma unroll
                for (int x = 0; x < ND; ++x) {
                    t[x] = acc.tile_sum(x);
                    t[x] += swz16(t[x]);
                    if (logL >= 4) t[x] += __shfl_xor(t[x], 32, 64);
                    if (logL >= 5) t[x] += MT == 4 ? swz4(t[x]) : swz8(t[x]);
                }
                if constexpr (MT == 4) {
                    if (logL >= 6) t[0] += swz8(t[0]);
                } else {
                    if (logL >= 6) t[0] += t[1];
                }
                const int m = lane & (MT - 1);
                int col[ND];
                bool writer;
                if constexpr (MT == 4) {
                    const int g = (lane >> 2) & 3;
                    writer = logL == 3 ? !(lane & 16) : logL == 4 ? lane < 16 : logL == 5 ? (lane < 16 && !(lane & 4)) : lane < 4;
                    col[0] = logL == 3 ? 2 * g + (lane >> 5) : logL == 4 ? g : logL == 5 ? g >> 1 : 0;
                } else {
                    const int g = (lane >> 3) & 1;
                    writer = logL == 3 ? !(lane & 16) : logL == 4 ? lane < 16 : lane < 8;
                    col[0] = logL == 3 ? 2 * g + (lane >> 5) : logL == 4 ? g : 0;
                    col[1] = logL == 3 ? 4 + 2 * g + (lane >> 5) : logL == 4 ? 2 + g : 1;
                }
                if (p.W == 1) {
                    if (active && writer && m0 + m < p.M) {
                        const int cbase = task << (6 - logL);
                        const float bk = QUANT == 1 ? qinv[m] : QUANT == 2 ? inv_lane : 0.f;
#pragma unroll
                        for (int x = 0; x < ND; ++x) {
                            if (x > 0 && logL >= 6) break;  // one column per task: tile 1 is already in t[0]
                            if constexpr (QUANT != 0)
                                Cf[(size_t)(m0 + m) * p.N + cbase + col[x]] = (float)t[x] * bk * p.w_scale;
                            else
                                C[(size_t)(m0 + m) * p.N + cbase + col[x]] = t[x];
                        }
                    }
                } else if (lane < MT) {
                    part[wave * MT + lane] = t[0];
                }
                }  // two-tile epilogue
            } else if constexpr (SL > 0) {
                // the task's wavefronts leave their column sums side by side (8 columns per wavefront at most); the first adds them up
                const int G = 64 >> p.logL;
                A v = lanes_sum(acc.acc[0], p.logL);
                if ((lane & ((1 << p.logL) - 1)) == 0) part[wave * 8 + (lane >> p.logL)] = v;
                __syncthreads();
                if (active && roff == 0 && lane < G) {
                    A sum = (A)0;
#pragma unroll
                    for (int w = 0; w < (1 << SL); ++w) sum += part[(wave + w) * 8 + lane];
                    if constexpr (QUANT != 0)
                        Cf[(size_t)m0 * p.N + (task << (6 - p.logL)) + lane] = (float)sum * back[0] * p.w_scale;
                    else
                        C[(size_t)m0 * p.N + (task << (6 - p.logL)) + lane] = sum;
                }
                if (it + 1 < p.iters) __syncthreads();  // (the next task's sums go to the same place)
            } else {
                store_lane_sums(p, acc.acc, part, back, active, task, lane, wave, m0);
            }
            }  // matrix-unit / plain sums
            if (SL == 0 && p.W != 1) {
                // second pass: the W wavefronts of a column meet in a small LDS buffer
                __syncthreads();
                if (active && lane == 0 && (wave & (p.W - 1)) == 0) {
                    const int col = task / p.W;
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        A s = (A)0;
                        for (int w = 0; w < p.W; ++w) s += part[(wave + w) * MT + m];
                        if (m0 + m < p.M) {
                            if constexpr (QUANT != 0)
                                Cf[(size_t)(m0 + m) * p.N + col] = (float)s * back[m] * p.w_scale;
                            else
                                C[(size_t)(m0 + m) * p.N + col] = s;
                        }
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
// blockIdx.y selects the tile of MT activation rows.  RF > 0: every task has
// exactly RF full rounds (straight-line body); RF == 0: any length (ring).
template <typename Act, int MT, int MODE, bool PRE, bool VAR, int RF, int QUANT = 0, bool MERGED = false>
__global__ void __launch_bounds__((64 * lists_max_waves<Act, MT, QUANT == 1>())) lists_kernel(ListParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    ListsBody<Act, MT, MODE, PRE, VAR, QUANT, MERGED>::template run<RF>(p, smem);
}

// One int8 row on u16 lists with 1 << SL wavefronts per task (see ListsBody::run): up to 16 wavefronts per workgroup.
template <bool PRE, int RF, int SL, int QUANT = 0>
__global__ void __launch_bounds__(1024) lists_kernel_shared(ListParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    ListsBody<int8_t, 1, 0, PRE, false, QUANT, false>::template run<RF, SL>(p, smem);
}

// Several independent GEMVs of one shape in one launch: blockIdx.z picks the
// (stream, activations, output) triple, everything else is the kernel above.
constexpr int BATCH_MAX = 32;
struct BatchPtrs {
    const uint8_t *w[BATCH_MAX];
    const void *X[BATCH_MAX];
    void *C[BATCH_MAX];
};

template <typename Act, int MT, int MODE, bool PRE, bool VAR, int RF, bool MERGED = false>
__global__ void __launch_bounds__((64 * lists_max_waves<Act, MT, false>())) lists_kernel_batched(ListParams p, BatchPtrs b)
{
    extern __shared__ __align__(16) unsigned char smem[];
    p.w = b.w[blockIdx.z];
    p.X = b.X[blockIdx.z];
    p.C = b.C[blockIdx.z];
    ListsBody<Act, MT, MODE, PRE, VAR, 0, MERGED>::template run<RF>(p, smem);
}

// ------------------------------------------------------------------ launchers
static inline int hip_fail(hipError_t e, const char *what)
{
    return fail(SPTMM_ERR_HIP, "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
}

// Dynamic LDS above the default cap has to be granted per kernel once.
static inline int grant_lds(const void *kern, size_t lds, std::atomic<size_t> &granted)
{
    if (lds <= granted.load(std::memory_order_relaxed)) return SPTMM_OK;
    hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
    granted.store(lds, std::memory_order_relaxed);
    return SPTMM_OK;
}

template <typename Act, int MT, int MODE, bool PRE, bool VAR, int RF, bool MERGED = false>
static int launch_lists_rf(const GemvArgs &a, hipStream_t st)
{
    // Launch shape: g workgroups resident per CU, w wavefronts each.  A wavefront asks for its
    // next task's stream only when it is done with the current one, so what hides the memory
    // latency is the number of tasks in flight per CU, R = g*w.  The loop over tasks costs
    // iterations * max(R, R_lat) in units of one task's streaming time at the CU's share of the
    // HBM bandwidth (R_lat = tasks needed in flight to cover ~2 us of latency at 8 TB/s over the
    // CUs, i.e. ~62 KB per CU); R is bounded by the kernel's register footprint and the LDS the
    // tiles take.  Measured on MI355X, K=2560 N=13824 split_k=32: one workgroup per CU 11.4 us,
    // two 6.3 us; the headline shape has 5 tasks per CU and stays at one workgroup of 5.
    const int cus = a.compute_units > 0 ? a.compute_units : 256;
    // launch-shape overrides: the stream's plan for this kind of call, else what sptmm_device_init read from the environment
    const int tune_wpb = a.plan.waves_per_wg, tune_wgs = a.plan.wgs_per_cu, tune_tpw = a.plan.tasks_per_wave;
    constexpr int SLOT = slot_bytes<Act, MT>();
    const size_t tile = (size_t)(lists_tile_rows(a) + 64) * SLOT;
    // batched launches fill the CU with several workgroups where two tiles fit; then the smaller ones do better
    const bool roomy = a.batch && 2 * (tile + lists_behind_tile<Act, MT>(LISTS_MAX_WAVES)) <= (size_t)a.lds_limit;
    const int max_waves = a.quant || roomy ? LISTS_MAX_WAVES : lists_max_waves<Act, MT, false>();
    static std::atomic<int> vgprs{0};  // of the single-GEMV kernel of this instantiation
    int regs = vgprs.load(std::memory_order_relaxed);
    if (!regs) {
        hipFuncAttributes fa;
        hipError_t e = hipFuncGetAttributes(&fa, reinterpret_cast<const void *>(lists_kernel<Act, MT, MODE, PRE, VAR, RF, 0, MERGED>));
        if (e != hipSuccess) return hip_fail(e, "hipFuncGetAttributes");
        regs = fa.numRegs > 0 ? fa.numRegs : 128;
        vgprs.store(regs, std::memory_order_relaxed);
    }
    const int waves_per_simd = std::max(1, std::min(8, 512 / ((regs + 7) / 8 * 8)));
    const double task_kb = (VAR ? a.task_stride : Flavour<MODE>::HDR + 128 * Flavour<MODE>::ESZ * a.n_lane) / 1024.0;
    const double r_lat = 62.0 / (task_kb > 0.25 ? task_kb : 0.25);
    int wpb = a.W, wgs = 1;
    double best = 1e30;
    for (int g = 1; g <= (a.batch ? 1 : 3); ++g) {
        if (tune_wgs > 0 && g != tune_wgs) continue;
        for (int w = a.W; w <= max_waves; w += a.W) {
            if (g > 1 && g * w > 4 * waves_per_simd) continue;  // the register file of the CU's 4 SIMDs
            if (g > 1 && g * (tile + lists_behind_tile<Act, MT>(w)) > (size_t)a.lds_limit) continue;
            const int blocks = (a.tasks + w - 1) / w;
            const int grid = blocks < cus * g ? blocks : cus * g;
            const int iters = (blocks + grid - 1) / grid;
            // tasks a compute unit has in flight: in the full passes, and in the last one, which the workgroups may not fill
            const double r = std::min((double)g * w, (double)grid * w / cus);
            const int full = blocks / grid, rest = blocks - full * grid;
            const double r_rest = (double)rest * w / cus;
            // + each workgroup stages the tile once; a bubble per extra pass; when latency-bound, spread over more CUs
            // (where the latency term leaves several workgroup sizes level, four or five wavefronts: a lone launch of few
            // tasks does better in a few such workgroups than in one or two wavefronts on every compute unit -- K=4352
            // N=512 S=992, 128 tasks: 3.64 -> 3.20 us in workgroups of five; K=6400 N=2048 S=1952, gap stream: 4.39 -> 3.94)
            const double cost = full * (r > r_lat ? r : r_lat) + (rest ? (r_rest > r_lat ? r_rest : r_lat) : 0.0) + 0.05 * g + 0.25 * (iters - 1) +
                                0.001 * (w < 4 ? 4.5 - w : w - 4.5);
            if (cost < best - 1e-9) {
                best = cost;
                wpb = w;
                wgs = g;
            }
        }
    }
    // byte rows, batched: the tile is a quarter of the others' and the chip is filled along blockIdx.z; small workgroups
    // of four wavefronts, many per CU, do best (32 GEMVs per launch, 8 -> 4 wavefronts: K=6912 N=2560 1.65 -> 1.54 us
    // per GEMV, K=2560 N=2560 0.72 -> 0.65, K=13824 N=5120 6.8 -> 6.3; sparse streams with zero slots 0.36-0.86 ->
    // 0.33-0.81 us)
    if (is_byte_rows<Act>() && a.batch && a.W == 1) wpb = 4;
    // u16 lists on one- and four-row int8 tiles, batched, more tasks than the headline shape's 1280: eight wavefronts
    // (K=13824 N=5120: M=1 12.9 -> 12.3 us per GEMV, M=4 13.5 -> 12.6; K=2560 N=6912, M=4: 3.2 -> 3.0 us)
    if (MODE == 0 && MT <= 4 && sizeof(Act) == 1 && !is_byte_rows<Act>() && a.batch >= 4 && a.W == 1 && a.tasks >= 1536 && max_waves >= 8) wpb = 8;
    // ... and for the other shapes of those launches: what streams is the number of wavefronts a compute unit holds, and the
    // tile decides how many workgroups fit one.  At least 24 wavefronts per compute unit, in workgroups of at least four
    // (the latency model above counts tasks in flight and would take two or three wavefronts per 46 KB tile).  16 GEMVs per
    // launch, model's pick -> this: K=11520 N=2816 S=1536 M=1 1.67 -> 1.39 us per GEMV, M=4 2.04 -> 1.43; K=6400 N=2048
    // S=1952 1.54 -> 1.29, M=4 1.77 -> 1.35; K=4352 N=512 S=992 0.38 -> 0.29; K=4096 N=4352 S=1856 2.76 -> 2.44.
    else if (MODE == 0 && MT <= 4 && sizeof(Act) == 1 && !is_byte_rows<Act>() && a.batch >= 4 && a.W == 1 && max_waves >= 8) {
        // Four or eight, which the four SIMDs share evenly: four where six or more tiles fit a compute unit, eight where
        // four or fewer do (K=4096 N=4352 S=1856, 5 -> 4 wavefronts: 2.76 -> 2.38 us; K=8704 N=3328 S=1408, 6 -> 8: 1.93 -> 1.68).
        const int by_lds = std::max(1, (int)((size_t)a.lds_limit / (tile + lists_behind_tile<Act, MT>(LISTS_MAX_WAVES))));
        if (by_lds >= 6) wpb = 4;
        else if (by_lds <= 4) wpb = 8;
    }
    // eight-row tiles keep the matrix unit busy: a batched launch takes a wavefront count the four SIMDs share evenly
    // (K=13824 N=5120, M=8, 10 -> 12 wavefronts: gap stream 48 -> 55 % of HBM peak, u16 lists level)
    // -- and the largest workgroup does best: four wavefronts per SIMD, fewer workgroups staging (same shape, 12 -> 16
    // wavefronts: gap stream 9.95 -> 9.46 us per GEMV, u16 lists 14.0 -> 13.8 us)
    // (also where two tiles would fit a compute unit: the registers of an eight-row kernel allow 16 wavefronts per CU either
    // way, and one workgroup of 16 stages the tile once -- K=6912 N=2560, M=8, 8 -> 16 wavefronts: u16 3.65 -> 3.40 us, gap
    // stream level at 2.14-2.40 us from box to box)
    if (MT == 8 && a.batch >= 4 && a.W == 1 && !a.quant) {
        wpb = lists_max_waves<Act, MT, false>() / 4 * 4;
        // ... as long as the launch still has two workgroups per compute unit: a narrow matrix takes smaller ones
        // (K=12800 N=256, 64 tasks, 16 GEMVs per launch: 16 -> 4 wavefronts 1.43 -> 0.95 us per GEMV; K=6656 N=512: 0.78 -> 0.62)
        while (wpb > 4 && (long)a.batch * ((a.tasks + wpb - 1) / wpb) < 2L * cus) wpb -= 4;
    }
    // four-row tiles on gap streams, batched, tile small enough for several workgroups per CU: four wavefronts for
    // int8 rows (K=2560 N=640 0.32 -> 0.29 us per GEMV, M=2 on the headline shape 1.76 -> 1.67; level elsewhere), eight
    // for fp16 rows (headline shape 57 -> 64 % of HBM peak, K=2560 N=6912 61 -> 66 %; with the 55 KB tile of K=13824
    // five do better)
    if (MT == 4 && MODE != 0 && a.batch >= 4 && a.W == 1 && tile <= 40 * 1024 && max_waves >= 8) wpb = sizeof(Act) == 1 ? 4 : 8;
    // ... four int8 rows on tiles of more than 30 KB: two workgroups or fewer per compute unit would leave it eight
    // wavefronts; the largest workgroup instead (16 GEMVs per launch: K=11520 N=2816 S=1536 1.85 -> 1.05 us per GEMV,
    // K=8704 N=3328 S=1408 1.75 -> 1.13)
    if (MT == 4 && MODE != 0 && sizeof(Act) == 1 && a.batch >= 4 && a.W == 1 && tile > 30 * 1024) wpb = lists_max_waves<Act, MT, false>();
    // four fp16 rows (sums on the matrix unit, 56 KB tile at K=6912), batched: eight wavefronts as well
    // (headline shape, 5 -> 8: u16 lists 69 -> 81 % of HBM peak, gap stream 39 -> 53 %)
    if (MT == 4 && sizeof(Act) == 2 && a.batch >= 4 && a.W == 1 && max_waves >= 8) wpb = 8;
    // four fp32 rows (16-byte slots like eight int8 rows, sums on the VALU), batched: the largest workgroup, and tasks per
    // wavefront by the search below (headline shape, 32 GEMVs: 5 wavefronts x 2 tasks 6.75 us per GEMV, 8 x 4 4.10,
    // 8 x 10 -- two full rounds -- 3.73 us = 71 % of HBM peak; gap stream 4.13 -> 3.46 us)
    if (MT == 4 && sizeof(Act) == 4 && a.batch >= 4 && a.W == 1) wpb = max_waves;
    // tiles of 32 KB or more under anything but the one-row int8 kernels: eight wavefronts, and tasks per wavefront by the
    // search below (the kernels with rules of their own above keep their workgroup size)
    const bool big_tile = tile >= 32 * 1024 && !(MT == 1 && sizeof(Act) == 1) && a.batch >= 4 && a.W == 1 && !a.quant;
    if (big_tile && MT != 8 && !(MT == 4 && sizeof(Act) == 4) && !(MT == 4 && MODE != 0 && sizeof(Act) == 1)) wpb = std::min(8, max_waves);
    // eight fp16 rows, batched, three tiles or more to a compute unit: workgroups of four wavefronts, with the tasks per
    // wavefront the search below gives them (32 GEMVs per launch, K=2560: N=6912 gap stream 4.09 -> 3.39 us per GEMV,
    // N=13824 7.81 -> 6.46 and u16 lists 8.64 -> 7.43, N=3840 2.25 -> 1.95 and 2.29 -> 2.11; K=4096, two tiles: eight stay ahead)
    if (MT == 8 && sizeof(Act) == 2 && a.batch >= 4 && a.W == 1 && !a.quant && 3 * (tile + lists_behind_tile<Act, MT>(4)) <= (size_t)a.lds_limit) wpb = 4;
    if (tune_wpb > 0 && tune_wpb <= (a.quant ? LISTS_MAX_WAVES : lists_max_waves<Act, MT, false>()) && tune_wpb % a.W == 0) wpb = tune_wpb;
    const int slots = cus * wgs;  // workgroups resident at once
    const int blocks = (a.tasks + wpb - 1) / wpb;
    // one GEMV per launch: no more workgroups than the chip holds at once; a batched launch fills the chip along
    // blockIdx.z and starts from one task per wavefront
    int grid_x = a.batch >= 8 || blocks < slots ? blocks : slots;
    int iters = (blocks + grid_x - 1) / grid_x;
    // A batched launch has workgroups enough to fill the chip along blockIdx.z, and every workgroup
    // pays for staging the tile: two tasks per wavefront halve that (measured: gap streams 1.88 -> 1.72 us
    // per GEMV, four-row tiles 2.83 -> 2.76; nothing for the one-row u16 kernel, which waits on HBM only).
    constexpr bool WIDE_SLOT = MT == 8 || (MT == 4 && sizeof(Act) == 4);  // 16 bytes per index
    // ... and so is any tile of 32 KB or more, whatever the rows (float rows at K=13824, 32 GEMVs per launch, two tasks per
    // wavefront -> this search: gap stream fp16 M=1 8.3 -> 6.45 us per GEMV, fp32 M=4 32.0 -> 22.4; u16 lists fp16 M=4
    // 17.6 -> 12.7, fp32 M=4 52 -> 36; int8 M=4 on u16 lists at K=11008-13568 7.3 -> 6.5 and 9.0 -> 8.3) -- except under
    // the one-row int8 kernels, which wait on HBM alone and do best with one task per wavefront up to 55 KB tiles.
    if ((WIDE_SLOT || (MT == 4 && MODE != 0) || big_tile) && a.batch >= 4 && wgs == 1) {
        // Multi-row tiles are expensive to stage (eight rows of K=13824: 110 KB, ~2.5 us against ~4 us per task) and their
        // walks are bound by the LDS and the matrix unit rather than by HBM: up to 16 tasks per wavefront, chosen so that the
        // launch's workgroups come in full rounds over the workgroups the chip holds at once (cost per round: staging
        // + tasks per wavefront x one task's walk, in rough microseconds; only the ratio matters).  Measured, per GEMV:
        // K=13824 N=5120 split_k=64, M=8, 8 u16 GEMVs per launch, 2 / 4 / 8 tasks per wavefront 17.6 / 15.9 / 15.2 us
        // (12 tasks -- one and a third rounds -- 18.9 us); 14 gap-stream GEMVs, 8 / 12 tasks 10.1 / 9.8 us (10 tasks: 2.35
        // rounds, 10.9 us); K=6912 N=2560 split_k=32, M=4, 32 gap-stream GEMVs, 2 / 5 / 10 tasks 2.18 / 2.01 / 1.94 us
        // (int8 rows), 2.50 / 2.19 / 2.05 us (fp16 rows); K=13824, four fp16 rows, 2 / 12 tasks 16.1 / 11.6 us.
        // u16 lists on four-row tiles of int8 or fp16 rows wait on HBM and gain nothing from more than two tasks.
        const size_t per_wg = tile + lists_behind_tile<Act, MT>(wpb);
        const int by_lds = (int)((size_t)a.lds_limit / per_wg), by_regs = 4 * waves_per_simd / wpb;
        const int resident = std::max(1, std::min(by_lds, by_regs));
        const long at_once = (long)cus * resident;
        const int row_tiles = (a.M + MT - 1) / MT;
        // (the two costs as measured on a 110 KB tile with 8.6 KB tasks, and on a 28 KB tile with 8.4 KB tasks; other
        // shapes in proportion to their tile and task bytes)
        const double stage = (WIDE_SLOT ? 2.5 / 110.0 : 2.0 / 28.0) * ((double)tile / 1024.0);
        const double walk = (WIDE_SLOT ? 4.0 / 8.6 : 5.7 / 8.4) * task_kb;
        double best = 1e30;
        int pick = iters;
        for (int t = 1; t <= 16 && t <= blocks; ++t) {
            const long total = (long)a.batch * row_tiles * ((blocks + t - 1) / t);
            // Workgroups of four wavefronts on small tiles sit four or five to a CU and share its throughput: what counts is
            // the number of workgroups per CU, each costing a quarter of a task's walk to stage (hidden behind the others)
            // plus its tasks, and the last one's length (K=6912 N=2560, M=4, 32 GEMVs: 1 / 2 / 4 / 5 / 8 / 10 tasks 2.04 /
            // 1.82 / 1.77 / 1.76 / 1.80 / 1.83 us; K=2560 N=6912: 2.15 / 1.86 / 1.85 / 1.89 / 1.92 / 2.10 us).
            const double cost = MT == 4 && sizeof(Act) == 1 && wpb == 4 ? (double)((total + cus - 1) / cus) * (0.25 + t) + 0.5 * t
                                                                         : (double)((total + at_once - 1) / at_once) * (stage + walk * t);
            if (cost < best - 1e-9) best = cost, pick = t;
        }
        grid_x = (blocks + pick - 1) / pick;
        iters = (blocks + grid_x - 1) / grid_x;
    } else if (a.batch >= 8 && iters == 1 && blocks >= 2 && (long)a.batch * ((blocks + 1) / 2) >= 2L * cus &&  // (still two workgroups per compute unit)
               !(MODE == 0 && (MT == 1 || (MT == 4 && sizeof(Act) == 1))) &&
               !(is_byte_rows<Act>() && !VAR && task_kb >= 8.0 && tile <= (size_t)(task_kb * 1024.0))) {
        // (byte rows whose task is 8 KB or more and no smaller than the tile: one task per wavefront, 1.54 against 1.63 us
        // on the headline shape; shorter tasks and larger tiles do better with two)
        grid_x = (blocks + 1) / 2;
        iters = 2;
    }
    if (tune_tpw > 0 && a.batch) {
        grid_x = (blocks + tune_tpw - 1) / tune_tpw;
        iters = (blocks + grid_x - 1) / grid_x;
    }
    ListParams p{(const uint8_t *)a.w, a.X, a.C, a.M, a.K, a.N, VAR ? a.n_min : a.n_lane, a.tasks, ilog2(a.L), a.W,
                 a.task_stride, a.counts_bytes, iters, a.quant, a.w_scale, a.stones, 64 * wpb, grid_x};
    size_t lds = tile + lists_behind_tile<Act, MT>(wpb);
    if ((int)lds > a.lds_limit) return fail(SPTMM_ERR_UNSUPPORTED, "activation tile of %zu bytes exceeds the LDS limit %d", lds, a.lds_limit);
    dim3 grid(grid_x, (a.M + MT - 1) / MT), block(64 * wpb);
    if (a.batch) {
        {
            auto kern = lists_kernel_batched<Act, MT, MODE, PRE, VAR, RF, MERGED>;
            static std::atomic<size_t> lds_granted_b{48 * 1024};
            if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted_b)) return rc;
            for (int first = 0; first < a.batch; first += BATCH_MAX) {
                BatchPtrs b{};
                const int n = a.batch - first < BATCH_MAX ? a.batch - first : BATCH_MAX;
                for (int i = 0; i < n; ++i) {
                    b.w[i] = (const uint8_t *)a.batch_w[first + i] + a.batch_w_skip;
                    b.X[i] = a.batch_X[first + i];
                    b.C[i] = a.batch_C[first + i];
                }
                grid.z = n;
                hipLaunchKernelGGL(kern, grid, block, lds, st, p, b);
                hipError_t e = hipGetLastError();
                if (e != hipSuccess) return hip_fail(e, "lists_kernel_batched launch");
            }
            return SPTMM_OK;
        }
    }
    if (a.inv) {
        // rows quantised beforehand (sptmm_gemv_i8_scaled, sptmm_gemv_q8_ws): the int8 kernel, its sums scaled on the way out
        if constexpr (sizeof(Act) == 1) {
            auto kern = lists_kernel<Act, MT, MODE, PRE, VAR, RF, 2, MERGED>;
            p.inv = a.inv;
            static std::atomic<size_t> lds_granted_p{48 * 1024};
            if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted_p)) return rc;
            hipLaunchKernelGGL(kern, grid, block, lds, st, p);
            hipError_t e = hipGetLastError();
            return e == hipSuccess ? SPTMM_OK : hip_fail(e, "lists_kernel (rows quantised beforehand) launch");
        } else {
            return fail(SPTMM_ERR_INVALID, "rows quantised beforehand go through the int8 kernels");
        }
    }
    if (a.quant) {
        if constexpr (sizeof(Act) == 1 && !is_byte_rows<Act>()) {  // (quantising launches never take the byte tile: no such kernels are built)
            auto kern = lists_kernel<Act, MT, MODE, PRE, VAR, RF, 1, MERGED>;
            // + room for the per-wavefront sums of a full workgroup, the row maxima and the rows' 1/s
            lds = tile + (size_t)(2 * LISTS_MAX_WAVES + 1) * MT * 4;
            if ((int)lds > a.lds_limit) return fail(SPTMM_ERR_UNSUPPORTED, "activation tile of %zu bytes exceeds the LDS limit %d", lds, a.lds_limit);
            static std::atomic<size_t> lds_granted_q{48 * 1024};
            if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted_q)) return rc;
            hipLaunchKernelGGL(kern, grid, block, lds, st, p);
            hipError_t e = hipGetLastError();
            return e == hipSuccess ? SPTMM_OK : hip_fail(e, "lists_kernel (quantising) launch");
        } else {
            return fail(SPTMM_ERR_INVALID, "quantising launches go through the int8 kernels");
        }
    }
    auto kern = lists_kernel<Act, MT, MODE, PRE, VAR, RF, 0, MERGED>;
    static std::atomic<size_t> lds_granted{48 * 1024};
    if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, lds_granted)) return rc;
    hipLaunchKernelGGL(kern, grid, block, lds, st, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : hip_fail(e, "lists_kernel launch");
}

// A lone GEMV of one int8 row on u16 lists whose tasks are 2, 4, 6 or 8 rounds long: 1 << SL wavefronts per task.
// wpb wavefronts per workgroup (a multiple of 1 << SL), every workgroup resident.
template <bool PRE, int RF, int SL>
static int launch_lists_shared(const GemvArgs &a, int wpb, hipStream_t st)
{
    const size_t tile = (size_t)(a.K + 64) * 4, lds = tile + (size_t)wpb * 8 * 4;
    if ((int)lds > a.lds_limit) return fail(SPTMM_ERR_UNSUPPORTED, "activation tile of %zu bytes exceeds the LDS limit %d", lds, a.lds_limit);
    const int per_wg = wpb >> SL;  // tasks a workgroup holds at once
    const int blocks = (a.tasks + per_wg - 1) / per_wg;
    const int cus = a.compute_units > 0 ? a.compute_units : 256;
    const int slots = cus * std::max(1, std::min(16 / wpb, (int)((size_t)a.lds_limit / lds)));
    const int grid_x = blocks < slots ? blocks : slots;
    const int iters = (blocks + grid_x - 1) / grid_x;
    ListParams p{(const uint8_t *)a.w, a.X, a.C, a.M, a.K, a.N, a.n_lane, a.tasks, ilog2(a.L), a.W,
                 0, 0, iters, 0, a.w_scale, 0, 64 * wpb, grid_x};
    p.inv = a.inv;
    // (a row quantised beforehand: the same kernel with its sums scaled on the way out)
    auto kern = a.inv ? lists_kernel_shared<PRE, RF, SL, 2> : lists_kernel_shared<PRE, RF, SL, 0>;
    static std::atomic<size_t> lds_granted{48 * 1024}, lds_granted_p{48 * 1024};
    if (int rc = grant_lds(reinterpret_cast<const void *>(kern), lds, a.inv ? lds_granted_p : lds_granted)) return rc;
    hipLaunchKernelGGL(kern, dim3(grid_x), dim3(64 * wpb), lds, st, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPTMM_OK : hip_fail(e, "lists_kernel_shared launch");
}

// -> true and *rc when the launch went out with shared tasks
template <typename Act, int MT, int MODE, bool PRE, bool VAR>
static bool try_shared(const GemvArgs &a, hipStream_t st, int *rc)
{
    if constexpr (std::is_same<Act, int8_t>::value && MT == 1 && MODE == 0 && !VAR) {
        if (a.batch || a.quant || a.W != 1 || a.M != 1) return false;
        const int rounds = a.n_lane / 8, cus = a.compute_units > 0 ? a.compute_units : 256;
        int sl = a.plan.share_log, wpb = a.plan.waves_per_wg;
        if (sl < 0 || rounds < 2 || rounds > 8) return false;
        if (sl == 0) {
            // two wavefronts per task where the doubled launch is at most ten wavefronts per compute unit, in workgroups that
            // hold a compute unit's share of the tasks.  One GEMV per launch, HBM-cold, without -> with (K=6912 N=2560):
            // S=4096 split_k 32 (1280 tasks of 8 rounds) 5.62 -> 5.37 us, S=4160 5.87 -> 5.63, S=2048 split_k 16 (640 tasks
            // of 8 rounds) 4.87 -> 3.88, S=1024 (4 rounds) 3.70 -> 3.12; K=2560 N=2560 S=1536 3.53 -> 3.51; beyond ten
            // wavefronts per compute unit nothing (K=2560 N=6912, 1728 tasks: 5.39 -> 5.43), four wavefronts per task lose
            // (headline 6.3-7.4 us).
            if (rounds % 2 || 2 * (long)a.tasks > 10L * cus) return false;
            sl = 1;
            if (wpb <= 0) wpb = std::max(4, (int)((2L * a.tasks + cus - 1) / cus + 1) / 2 * 2);
        }
        if (rounds % (1 << sl)) return false;
        if (wpb <= 0) wpb = 8;
        if (wpb > 16 || wpb % (1 << sl)) return false;
        const int rf = rounds >> sl;
#define SHARED_CASE(RF_, SL_) \
    if (rf == RF_ && sl == SL_) return *rc = launch_lists_shared<PRE, RF_, SL_>(a, wpb, st), true
        SHARED_CASE(4, 1); SHARED_CASE(3, 1); SHARED_CASE(2, 1); SHARED_CASE(1, 1);
        SHARED_CASE(2, 2); SHARED_CASE(1, 2);
#undef SHARED_CASE
    }
    return false;
}

// Straight-line bodies exist for tasks
// with 1, 2, 3, 4, 6 or 8 full rounds (ragged streams: for the shortest
// task, when the longest has at most XMAX more); everything else takes the ring.
// Eight-row tiles whose columns take 32 or 64 lanes run the kernels with one result tile (MERGED).
template <typename Act, int MT, int MODE, bool PRE, bool VAR, int RF>
static int launch_lists_g(const GemvArgs &a, hipStream_t st)
{
    if constexpr (MT == 8) {
        if (a.L >= 32) return launch_lists_rf<Act, MT, MODE, PRE, VAR, RF, true>(a, st);
    }
    return launch_lists_rf<Act, MT, MODE, PRE, VAR, RF, false>(a, st);
}

template <typename Act, int MT, int MODE, bool PRE, bool VAR>
static int launch_lists_t(const GemvArgs &a, hipStream_t st)
{
    {
        int rc = SPTMM_OK;
        if (try_shared<Act, MT, MODE, PRE, VAR>(a, st, &rc)) return rc;
        constexpr int E16 = 16 / Flavour<MODE>::ESZ;
        int rf = (VAR ? a.n_min : a.n_lane) / E16;
        if constexpr (VAR) {
            rf = rf >= 8 ? 8 : rf >= 6 ? 6 : rf == 5 ? 4 : rf;
            if (a.n_max / E16 - rf > ListsBody<Act, MT, MODE, PRE, VAR>::XMAX) rf = 0;
        }
        // Eight-row kernels are short of registers (1024-thread workgroups, 128 VGPRs): beyond four rounds the
        // ring of four does better than a straight-line body that holds six or eight (K=13824 M=8: 15.4 -> 14.4 us).
        if (lists_short_of_registers<Act, MT>() && rf > 4) rf = 9;
        // four int8 rows on 16-bit gaps: straight-line bodies of four rounds and more spill (96-508 bytes per lane at 128 registers)
        constexpr bool UP_TO_THREE = sizeof(Act) == 1 && MT == 4 && MODE == 2;
        if (UP_TO_THREE && rf > 3) rf = 9;  // no straight-line body of that length: falls through to the ring
        switch (rf) {
        case 0:
            if ((VAR ? a.n_max : a.n_lane) / E16 <= ListsBody<Act, MT, MODE, PRE, VAR>::XMAX) return launch_lists_g<Act, MT, MODE, PRE, VAR, -1>(a, st);
            break;
        case 1: return launch_lists_g<Act, MT, MODE, PRE, VAR, 1>(a, st);
        case 2: return launch_lists_g<Act, MT, MODE, PRE, VAR, 2>(a, st);
        case 3: return launch_lists_g<Act, MT, MODE, PRE, VAR, 3>(a, st);
        case 4:
            if constexpr (!UP_TO_THREE) return launch_lists_g<Act, MT, MODE, PRE, VAR, 4>(a, st);
            break;
        case 6:
            if constexpr (!lists_short_of_registers<Act, MT>() && !UP_TO_THREE) return launch_lists_g<Act, MT, MODE, PRE, VAR, 6>(a, st);
            break;
        case 8:
            if constexpr (!lists_short_of_registers<Act, MT>() && !UP_TO_THREE) return launch_lists_g<Act, MT, MODE, PRE, VAR, 8>(a, st);
            break;
        default: break;
        }
    }
    return launch_lists_g<Act, MT, MODE, PRE, VAR, 0>(a, st);
}

template <typename Act, int MODE, bool PRE, bool VAR>
static int launch_lists_m(const GemvArgs &a, hipStream_t st)
{
    // a tile of `mt` rows fits when it leaves room for what the largest workgroup keeps behind it: the
    // per-wavefront sums, and for quantising launches the row maxima and scales as well
    auto fits = [&](size_t slot, int mt, size_t behind) {
        const size_t extra = a.quant ? (size_t)(2 * LISTS_MAX_WAVES + 1) * mt * 4 : behind;
        return (size_t)(lists_tile_rows(a) + 64) * slot + extra <= (size_t)a.lds_limit;
    };
    if constexpr (sizeof(Act) <= 2) {  // int8 and fp16 rows; four fp32 rows already fill a 16-byte slot
        if (a.M >= 5 && fits(slot_bytes<Act, 8>(), 8, lists_behind_tile<Act, 8>(lists_max_waves<Act, 8, false>())))
            return launch_lists_t<Act, 8, MODE, PRE, VAR>(a, st);
    }
    if (a.M >= 2 && fits(slot_bytes<Act, 4>(), 4, lists_behind_tile<Act, 4>(lists_max_waves<Act, 4, false>())))
        return launch_lists_t<Act, 4, MODE, PRE, VAR>(a, st);
    return launch_lists_t<Act, 1, MODE, PRE, VAR>(a, st);
}

template <int MODE, bool PRE, bool VAR>
static int launch_lists_a(const GemvArgs &a, ActType act, hipStream_t st)
{
    switch (act) {
    case ACT_I8:
        if constexpr (MODE == 1) {
            if (a.byte_rows && a.M == 1 && !a.quant) return launch_lists_t<i8row, 1, MODE, PRE, VAR>(a, st);
        }
        return launch_lists_m<int8_t, MODE, PRE, VAR>(a, st);
    case ACT_F16: return launch_lists_m<_Float16, MODE, PRE, VAR>(a, st);
    case ACT_F32: return launch_lists_m<float, MODE, PRE, VAR>(a, st);
    }
    return fail(SPTMM_ERR_INVALID, "unknown activation type");
}

}  // namespace sptmm
