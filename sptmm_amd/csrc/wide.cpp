// "Wide" streams: u16 lists / gap streams for activation tiles with 16-byte slots (16 int8 rows, or
// 8 fp16 rows, per row index), cut into K-tiles so that such a tile fits the LDS.  The reference reads
// its index lists once per activation row (main.cu:567); the kernels for these streams read them once
// for up to 16 rows whatever K is.  Host-only code: dense int8 {-1,0,+1} matrix <-> stream.
//
// Stream layout
//   512-byte header: u32 {magic "SPTW", phases P, k_tile KT, K, N, kind, gap bits, split_k}, then per
//   phase p < 16: u32 {offset, stride, n_min, n_max} (offset of the phase's sub-stream from the start
//   of the stream, a multiple of 256).
//   Phase p covers the rows [p*KT, min(K, (p+1)*KT)) of the matrix and is laid out like a ragged
//   stream of that sub-matrix: a 16-byte preamble {magic, tasks, n_max, n_min}, one u16 entry count
//   per task, zero fill to a multiple of 256; then task t at t*stride (gap streams: 256 bytes of u16
//   first positions [sign][lane]; then the rounds of n_t entries per lane and sign, as in every
//   other stream).
//
// Two things differ from the ragged streams of ragged.cpp:
//   * Rows are stored as POSITIONS in the tile: pos(r) = r ^ ((r >> 4) & 15) for the row r relative to
//     the K-tile.  Staging writes 16 consecutive rows per lane, and with this placement the 16 lanes
//     the LDS serves per pass of a 16-byte write fall on 16 different bank groups.  A position stays
//     inside its aligned block of 16 rows.  Zero rows (padding) sit at positions kt .. kt+63.
//   * A column's L lanes of a wavefront are the lanes {i + 16 g}: i in [c*L/4, (c+1)*L/4), g in 0..3
//     (c = the column's index inside the task).  One 16x16 matrix instruction then adds up the
//     gathered slots of lanes i, i+16, i+32, i+48, which must therefore belong to one column.
//     The LDS serves a 16-byte read in four passes of 16 lanes, each lane on the bank group position
//     mod 16 -- but not 16 consecutive lanes.  Measured on gfx950 (one quad of lanes made to read another
//     quad's addresses: free exactly when both are served together): the passes are the lanes
//     {0-3, 12-15, 20-23, 24-27}, {4-11, 16-19, 28-31}, and the same two sets + 32.  Those are the
//     scheduling domains: inside each, the positions of a slot should fall on 16 different bank groups.
#include <algorithm>
#include <cstring>
#include <vector>

#include "internal.hpp"

namespace sptmm {

namespace {

constexpr uint32_t WIDE_MAGIC = 0x57545053u;  // "SPTW"
constexpr int WIDE_MAX_PHASES = 16;
constexpr size_t WIDE_HEADER_BYTES = 512;

inline int wide_pos(int r) { return r ^ ((r >> 4) & 15); }

struct WidePhase {
    int k0 = 0, kt = 0;                          // rows [k0, k0 + kt) of the matrix
    std::vector<std::vector<uint16_t>> pos[2];   // [sign][column]: ascending positions
    std::vector<int> n_task;
    int n_min = 0, n_max = 0;
    size_t offset = 0, stride = 0, counts_bytes = 0, bytes = 0, read_bytes = 0;
};

struct WidePlan {
    Geometry g;
    int K = 0, N = 0, kind = 0, bits = 0, esz = 2, hdr = 0, KT = 0;
    std::vector<WidePhase> ph;
    size_t total = 0, read_bytes = 0;
    uint64_t nnz = 0;
};

int ceil_div(int a, int b) { return (a + b - 1) / b; }

// physical lane of virtual lane u (0 .. L-1) of column c_in_task
inline int wide_lane(int L, int c_in_task, int u) { return c_in_task * (L / 4) + u / 4 + 16 * (u % 4); }

// The 16 lanes the LDS serves in pass d of a 16-byte read (see the header of this file).
inline int pass_lane(int d, int j)
{
    static const int lower[2][16] = {{0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27},
                                     {4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31}};
    return lower[d & 1][j] + 32 * (d >> 1);
}
// column (inside its task) that owns a lane
inline int lane_owner(int L, int lane) { return (lane & 15) / (L / 4); }

int check_wide_shape(int K, int N, int kind, int split_k, int k_tile)
{
    if (K <= 0 || N <= 0) return fail(SPTMM_ERR_INVALID, "K and N must be positive");
    if (K % 16) return fail(SPTMM_ERR_INVALID, "K mod 16 should be 0");
    if (N % 16) return fail(SPTMM_ERR_INVALID, "N mod 16 should be 0");
    if (K >= 65536) return fail(SPTMM_ERR_INVALID, "K should fit an unsigned 16-bit row index");
    if (kind != SPTMM_KIND_U16 && kind != SPTMM_KIND_DELTA) return fail(SPTMM_ERR_INVALID, "wide streams are u16 lists or gap streams");
    if (split_k != 8 && split_k != 16 && split_k != 32 && split_k != 64) return fail(SPTMM_ERR_INVALID, "Wrong split size (wide streams: 8, 16, 32 or 64)");
    if (k_tile <= 0 || k_tile % 16 || k_tile + 64 > 16383) return fail(SPTMM_ERR_INVALID, "k_tile must be a positive multiple of 16 below 16320");
    if ((K + k_tile - 1) / k_tile > WIDE_MAX_PHASES) return fail(SPTMM_ERR_UNSUPPORTED, "more than %d K-tiles", WIDE_MAX_PHASES);
    return SPTMM_OK;
}

// bits_req: 0 = 8 when every gap fits a signed byte else 16; 8 or 16 = exactly that (gap streams only)
int wide_plan(const int8_t *W, int K, int N, int kind, int split_k, int k_tile, int bits_req, WidePlan *pl)
{
    if (int rc = check_wide_shape(K, N, kind, split_k, k_tile)) return rc;
    if (int rc = make_ragged_geometry(N, split_k, 64, &pl->g)) return rc;
    if (!W) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (kind == SPTMM_KIND_U16 ? bits_req != 0 : (bits_req != 0 && bits_req != 8 && bits_req != 16))
        return fail(SPTMM_ERR_INVALID, "delta bits must be 0 (choose), 8 or 16");
    const Geometry &g = pl->g;
    const int P = (K + k_tile - 1) / k_tile;
    pl->K = K, pl->N = N, pl->kind = kind, pl->KT = k_tile;
    pl->ph.assign(P, WidePhase());
    for (int p = 0; p < P; ++p) {
        pl->ph[p].k0 = p * k_tile;
        pl->ph[p].kt = std::min(k_tile, K - p * k_tile);
        pl->ph[p].pos[0].assign(N, {});
        pl->ph[p].pos[1].assign(N, {});
    }
    std::vector<int> bad(N, 0);
    parallel_for(N, [&](int c) {
        const int8_t *w = W + (size_t)c * K;
        for (int r = 0; r < K; ++r) {
            if (w[r] == 0) continue;
            if (w[r] != 1 && w[r] != -1) {
                bad[c] = 1;
                continue;
            }
            const int p = r / k_tile;
            pl->ph[p].pos[w[r] == 1 ? 0 : 1][c].push_back((uint16_t)wide_pos(r - p * k_tile));
        }
        for (int p = 0; p < P; ++p)
            for (int sign = 0; sign < 2; ++sign) std::sort(pl->ph[p].pos[sign][c].begin(), pl->ph[p].pos[sign][c].end());
    });
    pl->nnz = 0;
    for (int c = 0; c < N; ++c)
        if (bad[c]) return fail(SPTMM_ERR_INVALID, "column %d holds a weight outside {-1,0,1}", c);

    const int L = g.L;
    bool fits8 = true;
    for (WidePhase &ph : pl->ph) {
        ph.n_task.assign(g.tasks, 1);
        for (int t = 0; t < g.tasks; ++t) {
            int n = 1;
            for (int sign = 0; sign < 2; ++sign)
                for (int cc = 0; cc < g.G; ++cc) {
                    const int cnt = (int)ph.pos[sign][t * g.G + cc].size();
                    if (kind == SPTMM_KIND_U16) {
                        // dealt round-robin over the four 16-lane domains, L/4 lanes of the column in each
                        for (int d = 0; d < 4; ++d) n = std::max(n, ceil_div((cnt + 3 - d) / 4, L / 4));
                    } else {
                        n = std::max(n, ceil_div(cnt, L));
                    }
                }
            ph.n_task[t] = n;
        }
        ph.n_max = *std::max_element(ph.n_task.begin(), ph.n_task.end());
        ph.n_min = *std::min_element(ph.n_task.begin(), ph.n_task.end());
        if (ph.n_max > 65535) return fail(SPTMM_ERR_UNSUPPORTED, "more than 65535 entries per lane");
        for (int sign = 0; sign < 2; ++sign)
            for (int c = 0; c < N; ++c) {
                const std::vector<uint16_t> &e = ph.pos[sign][c];
                pl->nnz += e.size();
                if (kind != SPTMM_KIND_DELTA || !fits8) continue;
                // every in-run gap, and the step from a list's last position to the zero row kt in the lane where
                // the list ends, has to fit a signed byte
                const int n = ph.n_task[c / g.G], cnt = (int)e.size();
                for (int i = 1; i < cnt; ++i)
                    if (i % n && e[i] - e[i - 1] > 127) fits8 = false;
                if (cnt % n && ph.kt - e[cnt - 1] > 127) fits8 = false;
            }
    }
    if (kind == SPTMM_KIND_U16) {
        pl->bits = 0, pl->esz = 2, pl->hdr = 0;
    } else {
        if (bits_req == 8 && !fits8) return fail(SPTMM_ERR_UNSUPPORTED, "a gap does not fit 8 bits (signed)");
        pl->bits = bits_req ? bits_req : (fits8 ? 8 : 16);
        pl->esz = pl->bits / 8, pl->hdr = 256;
    }
    size_t at = WIDE_HEADER_BYTES;
    pl->read_bytes = WIDE_HEADER_BYTES;
    for (WidePhase &ph : pl->ph) {
        ph.counts_bytes = ragged_counts_bytes(g.tasks);
        ph.stride = pl->hdr + (size_t)128 * pl->esz * ph.n_max;
        ph.bytes = (ph.counts_bytes + ph.stride * g.tasks + 255) / 256 * 256;
        ph.offset = at;
        at += ph.bytes;
        ph.read_bytes = 16 + 2 * (size_t)g.tasks;
        for (int n : ph.n_task) ph.read_bytes += pl->hdr + (size_t)128 * pl->esz * n;
        pl->read_bytes += ph.read_bytes;
    }
    if (at > 0xffffffffull) return fail(SPTMM_ERR_UNSUPPORTED, "stream larger than 4 GiB");
    pl->total = at;
    return SPTMM_OK;
}

void put_header(const WidePlan &pl, uint8_t *out)
{
    uint32_t *h = (uint32_t *)out;
    h[0] = WIDE_MAGIC, h[1] = (uint32_t)pl.ph.size(), h[2] = (uint32_t)pl.KT, h[3] = (uint32_t)pl.K, h[4] = (uint32_t)pl.N;
    h[5] = (uint32_t)pl.kind, h[6] = (uint32_t)pl.bits, h[7] = (uint32_t)pl.g.split_k;
    for (size_t p = 0; p < pl.ph.size(); ++p) {
        h[8 + 4 * p] = (uint32_t)pl.ph[p].offset, h[9 + 4 * p] = (uint32_t)pl.ph[p].stride;
        h[10 + 4 * p] = (uint32_t)pl.ph[p].n_min, h[11 + 4 * p] = (uint32_t)pl.ph[p].n_max;
    }
}

void put_counts(const WidePlan &pl, const WidePhase &ph, uint8_t *base)
{
    uint32_t *pre = (uint32_t *)base;
    pre[0] = RAGGED_MAGIC, pre[1] = (uint32_t)pl.g.tasks, pre[2] = (uint32_t)ph.n_max, pre[3] = (uint32_t)ph.n_min;
    uint16_t *counts = (uint16_t *)(base + 16);
    for (int t = 0; t < pl.g.tasks; ++t) counts[t] = (uint16_t)ph.n_task[t];
}

void pack_phase_u16(const WidePlan &pl, const WidePhase &ph, uint8_t *stream)
{
    const Geometry &g = pl.g;
    const int Lq = g.L / 4;  // lanes of a column in one 16-lane domain
    uint8_t *base = stream + ph.counts_bytes;
    parallel_for(g.tasks, [&](int task) {
        const int n = ph.n_task[task];
        uint8_t *t = base + (size_t)task * ph.stride;
        for (int sign = 0; sign < 2; ++sign) {
            // a column's positions, ordered by bank group, are dealt round-robin over the four domains
            std::vector<std::vector<uint16_t>> sorted(g.G);
            for (int o = 0; o < g.G; ++o) {
                sorted[o] = ph.pos[sign][task * g.G + o];
                std::stable_sort(sorted[o].begin(), sorted[o].end(), [](uint16_t x, uint16_t y) { return (x & 15) < (y & 15); });
            }
            for (int d = 0; d < 4; ++d) {
                // the pass's 16 lanes, grouped by the column that owns them: L/4 of every column
                std::vector<std::vector<int>> lanes_of(g.G);
                for (int j = 0; j < 16; ++j) lanes_of[lane_owner(g.L, pass_lane(d, j))].push_back(pass_lane(d, j));
                Domain dom;
                dom.banks = 16, dom.owners = g.G, dom.lanes = Lq, dom.n = n, dom.zero_base = ph.kt;
                dom.entries.resize(g.G);
                for (int o = 0; o < g.G; ++o)
                    for (size_t i = d; i < sorted[o].size(); i += 4) dom.entries[o].push_back(sorted[o][i]);
                schedule(dom);
                for (int o = 0; o < g.G; ++o)
                    for (int slot = 0; slot < n; ++slot)
                        for (int l = 0; l < Lq; ++l)
                            *(uint16_t *)(t + slot_offset(n, 2, sign, lanes_of[o][l], slot)) = (uint16_t)(dom.cell[o][(size_t)slot * Lq + l] << 2);
            }
        }
    });
}

// Virtual lane u of a column owns entries [u*n, (u+1)*n) of the sorted positions; where the list ends
// the lane steps to the zero row kt and stays there (gap 0), and the lanes behind it start on kt.
bool pack_phase_gaps(const WidePlan &pl, const WidePhase &ph, uint8_t *stream)
{
    const Geometry &g = pl.g;
    uint8_t *base = stream + ph.counts_bytes;
    std::vector<int> bad(g.tasks, 0);
    parallel_for(g.tasks, [&](int task) {
        const int n = ph.n_task[task];
        uint8_t *t = base + (size_t)task * ph.stride;
        for (int sign = 0; sign < 2; ++sign) {
            std::vector<uint16_t> run[64];
            for (int o = 0; o < g.G; ++o) {
                const std::vector<uint16_t> &e = ph.pos[sign][task * g.G + o];
                const int cnt = (int)e.size();
                for (int u = 0; u < g.L; ++u) {
                    std::vector<uint16_t> &r = run[wide_lane(g.L, o, u)];
                    r.resize(n);
                    for (int i = 0; i < n; ++i) r[i] = u * n + i < cnt ? e[u * n + i] : (uint16_t)ph.kt;
                }
            }
            if (pl.esz == 1) {
                for (int d = 0; d < 4; ++d) {
                    RunDomain rd;
                    rd.lanes = 16, rd.n = n, rd.zero_row = ph.kt;
                    for (int l = 0; l < 16; ++l) rd.rows[l] = run[pass_lane(d, l)];
                    if (!schedule_runs(rd)) {
                        bad[task] = 1;
                        return;
                    }
                    for (int l = 0; l < 16; ++l) {
                        const int lane = pass_lane(d, l);
                        *(uint16_t *)(t + sign * 128 + lane * 2) = rd.order[l][0];
                        for (int j = 0; j < n; ++j)
                            t[256 + slot_offset(n, 1, sign, lane, j)] = (uint8_t)(int8_t)(j ? (int)rd.order[l][j] - (int)rd.order[l][j - 1] : 0);
                    }
                }
            } else {
                for (int lane = 0; lane < 64; ++lane) {
                    const std::vector<uint16_t> &r = run[lane];
                    *(uint16_t *)(t + sign * 128 + lane * 2) = r[0];
                    for (int i = 0; i < n; ++i) *(uint16_t *)(t + 256 + slot_offset(n, 2, sign, lane, i)) = (uint16_t)(i ? r[i] - r[i - 1] : 0);
                }
            }
        }
    });
    for (int t = 0; t < g.tasks; ++t)
        if (bad[t]) return false;
    return true;
}

}  // namespace

int wide_parse_header(const void *packed, WideHeader *out)
{
    const uint32_t *h = (const uint32_t *)packed;
    if (h[0] != WIDE_MAGIC || h[1] < 1 || h[1] > (uint32_t)WIDE_MAX_PHASES) return fail(SPTMM_ERR_INVALID, "not a wide stream");
    out->phases = (int)h[1], out->k_tile = (int)h[2], out->K = (int)h[3], out->N = (int)h[4], out->kind = (int)h[5], out->bits = (int)h[6];
    out->split_k = (int)h[7];
    for (int p = 0; p < out->phases; ++p) {
        out->offset[p] = h[8 + 4 * p], out->stride[p] = h[9 + 4 * p];
        out->n_min[p] = (int)h[10 + 4 * p], out->n_max[p] = (int)h[11 + 4 * p];
    }
    return SPTMM_OK;
}

}  // namespace sptmm

using namespace sptmm;

extern "C" {

int sptmm_wide_k_tile(int K, int lds_bytes)
{
    // the largest K-tile whose (k_tile + 64) 16-byte slots, with 256 bytes to spare, fit `lds_bytes`, K cut into equal parts
    if (K <= 0 || K % 16 || lds_bytes < 4096) return fail(SPTMM_ERR_INVALID, "K must be a positive multiple of 16 and the LDS at least 4 KiB");
    const int cap = std::min(((lds_bytes - 256) / 16 - 64) / 16 * 16, 16304);
    const int P = (K + cap - 1) / cap;
    return ((K + P - 1) / P + 15) / 16 * 16;
}

size_t sptmm_pack_wide_bytes(const int8_t *W, int K, int N, int kind, int split_k, int k_tile, int *bits, size_t *read_bytes, uint64_t *nnz)
{
    size_t total = 0;
    const int rc = guarded([&]() -> int {
        WidePlan pl;
        if (int prc = wide_plan(W, K, N, kind, split_k, k_tile, bits ? *bits : 0, &pl)) return prc;
        if (bits) *bits = pl.bits;
        if (read_bytes) *read_bytes = pl.read_bytes;
        if (nnz) *nnz = pl.nnz;
        total = pl.total;
        return SPTMM_OK;
    });
    return rc == SPTMM_OK ? total : 0;
}

int sptmm_pack_wide(const int8_t *W, int K, int N, int kind, int split_k, int k_tile, int bits, void *out)
{
    return guarded([&]() -> int {
        WidePlan pl;
        if (int rc = wide_plan(W, K, N, kind, split_k, k_tile, bits, &pl)) return rc;
        if (!out) return fail(SPTMM_ERR_INVALID, "null pointer");
        uint8_t *o = (uint8_t *)out;
        memset(o, 0, pl.total);
        put_header(pl, o);
        for (const WidePhase &ph : pl.ph) {
            if (kind == SPTMM_KIND_U16)
                pack_phase_u16(pl, ph, o + ph.offset);
            else if (!pack_phase_gaps(pl, ph, o + ph.offset))
                return fail(SPTMM_ERR_INVALID, "a gap does not fit 8 bits (signed)");
            put_counts(pl, ph, o + ph.offset);
        }
        return SPTMM_OK;
    });
}

int sptmm_unpack_wide(const void *packed, int K, int N, int8_t *W)
{
    return guarded([&]() -> int {
        if (!packed || !W) return fail(SPTMM_ERR_INVALID, "null pointer");
        WideHeader h;
        if (int rc = wide_parse_header(packed, &h)) return rc;
        if (h.K != K || h.N != N) return fail(SPTMM_ERR_INVALID, "the stream holds a %d x %d matrix", h.K, h.N);
        if (int rc = check_wide_shape(K, N, h.kind, h.split_k, h.k_tile)) return rc;
        if ((K + h.k_tile - 1) / h.k_tile != h.phases) return fail(SPTMM_ERR_INVALID, "phase count does not match the K-tile");
        Geometry g;
        if (int rc = make_ragged_geometry(N, h.split_k, 64, &g)) return rc;
        const bool gaps = h.kind == SPTMM_KIND_DELTA;
        if (gaps ? (h.bits != 8 && h.bits != 16) : h.bits != 0) return fail(SPTMM_ERR_INVALID, "bad gap width");
        const int esz = gaps ? h.bits / 8 : 2, hdr = gaps ? 256 : 0;
        memset(W, 0, (size_t)K * N);
        std::vector<int> bad(g.tasks, 0);
        for (int p = 0; p < h.phases; ++p) {
            const int k0 = p * h.k_tile, kt = std::min(h.k_tile, K - k0);
            const uint8_t *sub = (const uint8_t *)packed + h.offset[p];
            const uint32_t *pre = (const uint32_t *)sub;
            if (pre[0] != RAGGED_MAGIC || pre[1] != (uint32_t)g.tasks || pre[2] != (uint32_t)h.n_max[p] || pre[3] != (uint32_t)h.n_min[p] ||
                h.stride[p] != (uint32_t)(hdr + 128 * esz * h.n_max[p]))
                return fail(SPTMM_ERR_INVALID, "phase %d: corrupt count table", p);
            const uint16_t *counts = (const uint16_t *)(sub + 16);
            const uint8_t *base = sub + ragged_counts_bytes(g.tasks);
            parallel_for(g.tasks, [&](int task) {
                const int n = counts[task];
                if (n < h.n_min[p] || n > h.n_max[p]) {
                    bad[task] = 1;
                    return;
                }
                const uint8_t *t = base + (size_t)task * h.stride[p];
                for (int sign = 0; sign < 2; ++sign)
                    for (int lane = 0; lane < 64; ++lane) {
                        const int i = lane & 15, c = task * g.G + i / (g.L / 4);
                        int run = gaps ? *(const uint16_t *)(t + sign * 128 + lane * 2) : 0;
                        for (int j = 0; j < n; ++j) {
                            const uint8_t *cell = t + hdr + slot_offset(n, esz, sign, lane, j);
                            int posn;
                            if (!gaps) {
                                posn = *(const uint16_t *)cell >> 2;
                            } else {
                                run += esz == 1 ? (int)(int8_t)*cell : (int)*(const uint16_t *)cell;
                                posn = run;
                            }
                            if (posn < 0 || posn >= kt + 64) {
                                bad[task] = 1;
                                return;
                            }
                            if (posn >= kt) continue;  // padding
                            int8_t &w = W[(size_t)c * K + k0 + wide_pos(posn)];  // (the placement is its own inverse)
                            if (w != 0) bad[task] = 1;
                            w = sign ? (int8_t)-1 : (int8_t)1;
                        }
                    }
            });
        }
        for (int t = 0; t < g.tasks; ++t)
            if (bad[t]) return fail(SPTMM_ERR_INVALID, "task %d: corrupt wide stream", t);
        return SPTMM_OK;
    });
}

}  // extern "C"
