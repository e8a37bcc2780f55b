// Internal declarations shared by the host format builders, the kernels'
// launchers and the C ABI.  Not installed.
#pragma once
#include <cstdarg>
#include <cstddef>
#include <cstdint>

#include "../../include/sptmm.h"

namespace sptmm {

int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// ---- geometry of the wave64 streams --------------------------------------
// One "task" is the work of one 64-lane wavefront: G = 64/L columns, L lanes
// per column (L = min(split_k, 64)); when split_k > 64 a column is spread over
// W = split_k/64 wavefronts ("parts") of the same workgroup.
struct Geometry {
    int N, half;      // columns, entries per sign per column (S/2)
    int split_k;      // lanes cooperating on one column
    int L, G, W;      // lanes per column in a wave, columns per wave, waves per column
    int n_lane;       // entries per lane per sign
    int tasks;        // wavefront tasks in the whole matrix
};

int make_geometry(int N, int S, int split_k, int max_split, Geometry *g);

// Byte offset, inside one task, of slot `j` (0 <= j < n_lane) of `lane` for
// sign `sign` (0 = +1 list, 1 = -1 list) when every entry is `esz` bytes and
// the widest per-lane load is 16 bytes.  Entries are stored in rounds: full
// rounds of 16 bytes per lane (both signs, 2 KiB per round), then at most one
// round each of 8, 4, 2 and (esz==1) 1 bytes per lane.
size_t slot_offset(int n_lane, int esz, int sign, int lane, int j);

// u16 stream fields are row indices shifted left by this many bits (2 when 4*K fits 16 bits).
int u16_index_shift(int K);

// striped gap stream (formats.cpp): stride between tasks, smallest / largest per-task entry count
struct StripedPlan;
int striped_plan(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, StripedPlan *pl);

// i2s tiling: 16 columns x 4 lanes per wave-load, 16 bytes (64 weights) per lane.
inline int i2s_padded_k(int K) { return (K + 255) / 256 * 256; }

// ---- validation shared by packers and uploaders -----------------------------
int check_shape(int K, int N, int S);

// ---- device-side launchers (kernels.hip) --------------------------------------
struct GemvArgs {
    const void *w;      // device stream
    const void *X;      // device activations, row-major [M][K]
    void *C;            // device output, row-major [M][N]
    int M, K, N, half, split_k, n_lane, tasks, L, G, W;
    int delta_bits;
    int delta_layout;   // 1 = contiguous runs, 2 = striped by row mod 32
    int task_stride;    // striped: bytes between tasks
    int n_min;          // striped: smallest per-task entry count
    int n_max;          // striped: largest per-task entry count
    int index_shift;    // u16 stream: fields are row << index_shift
    int compute_units;
    int lds_limit;
    // batched launch (u16 / gap streams, int8): `batch` GEMVs of this shape, one (w, X, C) triple each
    int batch = 0;
    const void *const *batch_w = nullptr;
    const void *const *batch_X = nullptr;
    void *const *batch_C = nullptr;
};
enum ActType { ACT_I8 = 0, ACT_F16 = 1, ACT_F32 = 2 };

int launch_u16(const GemvArgs &a, ActType act, void *stream);
int launch_u16_scaled(const GemvArgs &a, ActType act, void *stream);   // lists_u16_scaled.hip
int launch_u16_plain(const GemvArgs &a, ActType act, void *stream);    // lists_u16_plain.hip
int launch_runs8(const GemvArgs &a, ActType act, void *stream);        // lists_runs8.hip
int launch_runs16(const GemvArgs &a, ActType act, void *stream);       // lists_runs16.hip
int launch_striped(const GemvArgs &a, ActType act, void *stream);      // lists_striped.hip
int launch_delta(const GemvArgs &a, ActType act, void *stream);
int launch_i2s(const GemvArgs &a, void *stream);
int launch_copy(void *dst, const void *src, size_t bytes, void *stream);

}  // namespace sptmm
