// Internal declarations shared by the host format builders, the kernels'
// launchers and the C ABI.  Not installed.
#pragma once
#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <exception>
#include <algorithm>
#include <new>
#include <thread>
#include <vector>

#include "../../include/sptmm.h"

namespace sptmm {

int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Body of an entry point that allocates on the host: no C++ exception may cross the C ABI.
template <class F> int guarded(F body) noexcept
{
    try {
        return body();
    } catch (const std::bad_alloc &) {
        return fail(SPTMM_ERR_NOMEM, "out of host memory");
    } catch (const std::exception &e) {
        return fail(SPTMM_ERR_INVALID, "%s", e.what());
    } catch (...) {
        return fail(SPTMM_ERR_INVALID, "unexpected exception");
    }
}

// f(i) for i in [0, n) on up to 16 worker threads (one below 64 items); the first exception any
// worker meets is rethrown on the calling thread.
template <class F> void parallel_for(int n, F f)
{
    unsigned hw = std::thread::hardware_concurrency();
    int nt = (int)std::min<unsigned>(hw ? hw : 1, 16);
    if (n < 64) nt = 1;
    std::vector<std::thread> th;
    std::vector<std::exception_ptr> err(nt);
    for (int t = 0; t < nt; ++t)
        th.emplace_back([=, &err] {
            try {
                int i0 = (int)((long)n * t / nt), i1 = (int)((long)n * (t + 1) / nt);
                for (int i = i0; i < i1; ++i) f(i);
            } catch (...) {
                err[t] = std::current_exception();
            }
        });
    for (auto &t : th) t.join();
    for (auto &e : err)
        if (e) std::rethrow_exception(e);
}

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

// One scheduling domain of the u16 stream = the 32 lanes of a half-wavefront,
// which the LDS serves in one pass when they hit 32 different banks (bank = row
// index mod 32 in every tile layout).  `owners` columns share the domain, each
// with `lanes` lanes (owners*lanes == 32) and lanes*n cells.  schedule() fills
// cell[owner][slot*lanes + lane], choosing the entries of a slot bank by bank,
// fullest bank first.  An owner with fewer than lanes*n entries gets the rest as
// padding that may sit on any bank: zero rows zero_base + ((bank - zero_base) mod 32)
// behind the activation tile.
struct Domain {
    int owners = 0, lanes = 0, n = 0;
    int banks = 32;  // owners * lanes; 16 for the 16-byte slots of the wide tiles (the LDS serves 16 lanes of a b128 read per pass)
    int zero_base = 0;
    std::vector<std::vector<uint16_t>> entries;  // per owner
    std::vector<std::vector<uint16_t>> cell;     // per owner: [slot][lane] -> row
};
void schedule(Domain &d);

// Gap streams with 8-bit gaps store them SIGNED, so a lane may visit the rows of
// its run in any order whose steps stay within -128..127.  schedule_runs() picks
// those orders for the 32 lanes of a half-wavefront together: at every step each
// lane chooses among the oldest `window` rows it has not visited yet, and the
// choices are matched to distinct LDS banks (row mod 32) as far as possible.
// rows[l]: ascending, all of the same length n; rows >= zero_row are padding (the
// same zero slot for every lane, never a conflict).  order[l][j] = row that lane l
// visits at step j.  Returns false when some run has a sorted gap above 127 (no
// 8-bit stream exists then).
struct RunDomain {
    int n = 0, zero_row = 0;
    int lanes = 32;  // lanes scheduled together = banks (row mod lanes) they are spread over; 16 for the wide tiles
    int shift = 0;   // bank = (row >> shift) mod lanes: 2 for tiles of one byte per row
    std::vector<uint16_t> rows[32];
    std::vector<uint16_t> order[32];
};
bool schedule_runs(RunDomain &d, int window = 16);  // (window 8: 1.30 LDS passes per step on the headline matrix, 16: 1.24, 24: 1.25)
// One task of an 8-bit gap stream (header + rounds at `task`): rows[sign][lane] = what the lane
// visits, ascending, n each.  False when a sorted gap exceeds 127.
bool write_task_runs8(uint8_t *task, int n, int zero_row, const std::vector<uint16_t> (&rows)[2][64], int bank_shift = 0);

// Geometry of a ragged stream (tasks carry their own entry count): as
// make_geometry, with half = n_lane = 0.
int make_ragged_geometry(int N, int split_k, int max_split, Geometry *g);
// ragged u16 stream: fields are row << this (2 when 4*(K+64) fits 16 bits)
int ragged_index_shift(int K);
// ragged streams open with a 16-byte preamble {u32 magic, tasks, n_max, n_min} and one u16 entry
// count per task; the tasks follow at the next multiple of 256 bytes
constexpr uint32_t RAGGED_MAGIC = 0x52545053u;  // "SPTR"
// 8-bit gap streams of sparse matrices ("stepping stones"): the activation tile keeps 16 zero slots behind every 96
// rows, the stream holds tile positions instead of rows, and a gap of more than 127 positions is walked over zero
// slots, each an entry that adds nothing.  Any 127 consecutive positions hold a zero slot.  The period of 112 slots
// moves the zero slots of successive blocks to other LDS banks (a period of 128 would keep them all on the same ones,
// and lanes that wait on zero slots for the rest of their task would queue there).
constexpr uint32_t RAGGED_MAGIC_STONES = 0x53545053u;  // "SPTS"
constexpr int STONE_ROWS = 96, STONE_BLOCK = 112;
inline int stone_blocks(int K) { return (K + STONE_ROWS - 1) / STONE_ROWS; }
inline int stone_tile_rows(int K) { return STONE_BLOCK * stone_blocks(K); }                 // positions of the tile (zero slots included)
inline int stone_pos(int row) { return row + (STONE_BLOCK - STONE_ROWS) * (row / STONE_ROWS); }
// the row at a position, -1 for a zero slot (rows >= K of a last, partial block are zero slots as well: the caller checks)
inline int stone_row(int pos) { return pos % STONE_BLOCK >= STONE_ROWS ? -1 : STONE_ROWS * (pos / STONE_BLOCK) + pos % STONE_BLOCK; }
inline size_t ragged_counts_bytes(int tasks) { return ((size_t)16 + 2 * (size_t)tasks + 255) / 256 * 256; }

// Wide streams (wide.cpp): what the 512-byte header in front of the K-tiles' sub-streams says.
struct WideHeader {
    int phases = 0, k_tile = 0, K = 0, N = 0, kind = 0, bits = 0, split_k = 0;
    uint32_t offset[16] = {0}, stride[16] = {0};
    int n_min[16] = {0}, n_max[16] = {0};
};
int wide_parse_header(const void *packed, WideHeader *out);

// i2s tiling: 16 columns x 4 lanes per wave-load, 16 bytes (64 weights) per lane.
inline int i2s_padded_k(int K) { return (K + 255) / 256 * 256; }

// ---- validation shared by packers and uploaders -----------------------------
int check_shape(int K, int N, int S);

// The launch shape of one kind of call on one stream, where it is not left to the launchers' own model: every field 0 =
// the model's choice.  Mirrors sptmm_plan (sptmm.h) field for field.
struct Plan {
    int waves_per_wg = 0;    // wavefronts per workgroup (list and wide kernels; i2s: of the matrix-unit kernel)
    int wgs_per_cu = 0;      // workgroups per compute unit of a lone list launch
    int tasks_per_wave = 0;  // tasks per wavefront of a batched list launch
    int share_log = 0;       // a lone GEMV (one int8 row, u16 lists): 1 << this many wavefronts per task; -1: never
    int i2s_ct = 0;          // column tiles per wavefront of the i2s matrix-unit kernel
    int reserved[3] = {0, 0, 0};
};
static_assert(sizeof(Plan) == sizeof(sptmm_plan), "Plan mirrors sptmm_plan");
// Which of a stream's plans a call takes: by its activation rows (1, 2-4, 5-8, more) and by whether it is a batched launch.
constexpr int PLAN_SLOTS = 8;
inline int plan_slot(int M, bool batched) { return 2 * (M <= 1 ? 0 : M <= 4 ? 1 : M <= 8 ? 2 : 3) + (batched ? 1 : 0); }

// Process-wide launch-shape overrides for tuning runs, under a stream's own plan.  Filled from the environment by
// sptmm_device_init -- once per call of it, never on a launch path -- and by nothing else.
struct Tuning {
    Plan plan;               // SPTMM_WAVES_PER_WG, SPTMM_WGS_PER_CU, SPTMM_TASKS_PER_WAVE, SPTMM_SHARE_LOG, SPTMM_I2S_CT
    int i2s_mfma_from = 2;   // SPTMM_I2S_MFMA_FROM: rows from which a lone i2s launch takes the matrix-unit kernel
};
const Tuning &tuning();
void tuning_reload();  // reads the environment (formats.cpp)

// ---- device-side launchers (i2s.hip and the lists_*.hip files) --------------------------------------
struct GemvArgs {
    const void *w;      // device stream
    const void *X;      // device activations, row-major [M][K]
    void *C;            // device output, row-major [M][N]
    int M, K, N, half, split_k, n_lane, tasks, L, G, W;
    int delta_bits;
    int index_shift;    // u16 stream: fields are row << index_shift
    int ragged;         // the stream starts with a table of per-task entry counts; the next four fields apply
    int task_stride;    // bytes between tasks
    int counts_bytes;   // bytes of the count table, preamble included
    int n_min, n_max;   // smallest / largest per-task entry count
    int compute_units;
    int lds_limit;
    int byte_rows = 0;    // 8-bit gap stream scheduled for a tile of one byte per row (int8, one activation row)
    int stones = 0;       // 8-bit gap stream of tile positions with zero slots behind every 96 rows (RAGGED_MAGIC_STONES)
    int quant = 0;        // 1 / 2: X holds fp16 / bf16 rows, quantised to int8 in the kernel; C receives floats
    float w_scale = 1.f;  // quantising launches: factor applied to every output
    const float *inv = nullptr;  // int8 rows quantised by an earlier launch: the rows' 1/s on the device; C receives floats (lone list launches, M > 4)
    // batched launch (u16 / gap streams, int8): `batch` GEMVs of this shape, one (w, X, C) triple each
    int batch = 0;
    const void *const *batch_w = nullptr;
    size_t batch_w_skip = 0;  // bytes in front of every batch_w[i] that the kernels do not read (a count table they need not look at)
    const void *const *batch_X = nullptr;
    void *const *batch_C = nullptr;
    Plan plan;            // launch-shape overrides: the stream's plan for this kind of call over the process-wide ones
};
enum ActType { ACT_I8 = 0, ACT_F16 = 1, ACT_F32 = 2 };

int launch_u16(const GemvArgs &a, ActType act, void *stream);
int launch_u16_scaled(const GemvArgs &a, ActType act, void *stream);   // lists_u16_scaled.hip
int launch_u16_plain(const GemvArgs &a, ActType act, void *stream);    // lists_u16_plain.hip
int launch_runs8(const GemvArgs &a, ActType act, void *stream);        // lists_runs8.hip
int launch_runs16(const GemvArgs &a, ActType act, void *stream);       // lists_runs16.hip
int launch_ragged_u16_scaled(const GemvArgs &a, ActType act, void *stream);  // lists_ragged_u16_scaled.hip
int launch_ragged_u16_plain(const GemvArgs &a, ActType act, void *stream);   // lists_ragged_u16_plain.hip
int launch_ragged_runs8(const GemvArgs &a, ActType act, void *stream);       // lists_ragged_runs8.hip
int launch_ragged_runs16(const GemvArgs &a, ActType act, void *stream);      // lists_ragged_runs16.hip
int launch_delta(const GemvArgs &a, ActType act, void *stream);
int launch_wide(const GemvArgs &a, const WideHeader &h, ActType act, void *stream);  // lists_wide.hip
int launch_i2s(const GemvArgs &a, void *stream);
int launch_quantise_rows(const void *X, int kind, int M, int K, void *Xq, float *inv, void *stream);  // quantise.hip
size_t scratch_bytes();                     // the library's static device scratch (quantise.hip): its size,
int scratch_init(int device);               // the look-up of its address on the current device (sptmm_device_init),
int scratch_of(int device, void **ptr);     // and that address
int launch_copy(void *dst, const void *src, size_t bytes, void *stream);
int launch_read(const void *src, size_t bytes, void *sink, int workgroups, void *stream);

}  // namespace sptmm
