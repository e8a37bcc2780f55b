// Ragged ternary matrices: columns that differ in their number of nonzeros and
// whose +1 / -1 counts need not match (what a quantised model tensor looks like;
// the benchmark generator of main.cu:246-276 only makes exactly S/2 per sign,
// main.cu:90, and its unused "VCSC" arrays, main.cu:461-488, sketch per-column
// counts).  Host-only code: dense int8 {-1,0,+1} matrix -> u16 / gap stream whose
// tasks carry their own entry count.
//
// Stream layout: a 16-byte preamble {u32 magic, tasks, n_max, n_min}, one u16
// entry count n_t per task, zero fill to a multiple of 256 bytes; then task t at
// t * stride, laid out exactly as in the balanced streams (gap streams: 256 bytes
// of u16 first rows [sign][lane]; then the rounds of n_t entries per lane and
// sign).  n_t = the longest list of the task divided over its lanes, rounded up;
// shorter lists are padded with entries on the zero rows K..K+63 that every
// activation tile keeps behind row K-1.  stride = header + 128 * entry_bytes * n_max.
#include <algorithm>
#include <cstring>
#include <exception>
#include <thread>
#include <vector>

#include "internal.hpp"

namespace sptmm {

namespace {

struct RaggedPlan {
    Geometry g;
    int K = 0, kind = 0, bits = 0, esz = 2, hdr = 0, shift = 0;
    int bank_shift = 0;  // 8-bit gap streams: LDS bank = (row >> bank_shift) mod 32 (2: tiles of one byte per row)
    bool stones = false; // 8-bit gap stream of tile positions, long gaps walked over the tile's zero slots
    std::vector<std::vector<uint16_t>> rows[2];  // [sign][column]: ascending row lists
    std::vector<int> n_task;
    int n_min = 0, n_max = 0;
    size_t stride = 0, counts_bytes = 0, read_bytes = 0;
    uint64_t nnz = 0;
};

int ceil_div(int a, int b) { return (a + b - 1) / b; }

// The zero slot a walk at position `cur` steps to next on its way up: the farthest one within 127 positions.
int stone_ahead(int cur)
{
    const int t = cur + 127;
    return t % STONE_BLOCK >= STONE_ROWS ? t : STONE_BLOCK * (t / STONE_BLOCK) - 1;
}

// Stepping-stone stream: the positions the 64 lanes of one sign of a task visit, in ascending order and without padding.
// Lane v of a column owns entries [v*n0, (v+1)*n0) of the column's sorted list (n0 = the task's longest list divided over
// its lanes); wherever two of them lie more than 127 positions apart, zero slots are put between them.  -> longest run
int stone_runs(const RaggedPlan &pl, int task, int sign, int n0, std::vector<uint16_t> (&run)[64])
{
    const Geometry &g = pl.g;
    size_t longest = 0;
    for (int lane = 0; lane < 64; ++lane) {
        const std::vector<uint16_t> &e = pl.rows[sign][task * g.G + lane / g.L];
        const int cnt = (int)e.size(), first = (lane % g.L) * n0;
        std::vector<uint16_t> &r = run[lane];
        r.clear();
        for (int i = first; i < first + n0 && i < cnt; ++i) {
            const int p = stone_pos(e[i]);
            if (!r.empty())
                while (p - (int)r.back() > 127) r.push_back((uint16_t)stone_ahead(r.back()));
            r.push_back((uint16_t)p);
        }
        longest = std::max(longest, r.size());
    }
    return (int)longest;
}

// u16 stream, 64 lanes per column: the column's entries, ordered by bank, are dealt round-robin
// over its nd half-wavefronts; half-wavefront d gets this many of cnt
int dealt(int cnt, int nd, int d) { return (cnt + nd - 1 - d) / nd; }

int check_ragged_shape(int K, int N)
{
    if (K <= 0 || N <= 0) return fail(SPTMM_ERR_INVALID, "K and N must be positive");
    if (K % 16) return fail(SPTMM_ERR_INVALID, "K mod 16 should be 0");
    if (N % 16) return fail(SPTMM_ERR_INVALID, "N mod 16 should be 0");
    if (K + 64 > 65535) return fail(SPTMM_ERR_INVALID, "K + 64 should fit an unsigned 16-bit row index");
    return SPTMM_OK;
}

// bits_req: 0 = 8 when every gap fits a byte else 16; 8 or 16 = exactly that (gap streams only)
int ragged_plan(const int8_t *W, int K, int N, int kind, int split_k, int bits_req, RaggedPlan *pl)
{
    if (int rc = check_ragged_shape(K, N)) return rc;
    if (kind != SPTMM_KIND_U16 && kind != SPTMM_KIND_DELTA) return fail(SPTMM_ERR_INVALID, "ragged streams are u16 lists or gap streams");
    if (int rc = make_ragged_geometry(N, split_k, kind == SPTMM_KIND_U16 ? 256 : 64, &pl->g)) return rc;
    if (!W) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (kind == SPTMM_KIND_U16 ? bits_req != 0 : (bits_req != 0 && bits_req != 8 && bits_req != 16))
        return fail(SPTMM_ERR_INVALID, "delta bits must be 0 (choose), 8 or 16");
    const Geometry &g = pl->g;
    pl->K = K;
    pl->kind = kind;
    pl->rows[0].assign(N, {});
    pl->rows[1].assign(N, {});
    std::vector<int> bad(N, 0);
    parallel_for(N, [&](int c) {
        const int8_t *w = W + (size_t)c * K;
        for (int r = 0; r < K; ++r) {
            if (w[r] == 1)
                pl->rows[0][c].push_back((uint16_t)r);
            else if (w[r] == -1)
                pl->rows[1][c].push_back((uint16_t)r);
            else if (w[r] != 0)
                bad[c] = 1;
        }
    });
    pl->nnz = 0;
    for (int c = 0; c < N; ++c) {
        if (bad[c]) return fail(SPTMM_ERR_INVALID, "column %d holds a weight outside {-1,0,1}", c);
        pl->nnz += pl->rows[0][c].size() + pl->rows[1][c].size();
    }

    pl->n_task.assign(g.tasks, 1);
    for (int t = 0; t < g.tasks; ++t) {
        int n = 1;
        for (int sign = 0; sign < 2; ++sign) {
            if (g.W > 1 || (kind == SPTMM_KIND_U16 && g.L == 64)) {
                const int c = t / g.W, part = t % g.W, cnt = (int)pl->rows[sign][c].size();
                for (int h = 0; h < 2; ++h) n = std::max(n, ceil_div(dealt(cnt, 2 * g.W, 2 * part + h), 32));
            } else {
                for (int cc = 0; cc < g.G; ++cc) n = std::max(n, ceil_div((int)pl->rows[sign][t * g.G + cc].size(), g.L));
            }
        }
        pl->n_task[t] = n;
    }
    pl->n_max = *std::max_element(pl->n_task.begin(), pl->n_task.end());
    pl->n_min = *std::min_element(pl->n_task.begin(), pl->n_task.end());

    if (kind == SPTMM_KIND_U16) {
        pl->bits = 0;
        pl->esz = 2;
        pl->hdr = 0;
        pl->shift = ragged_index_shift(K);
    } else {
        // every in-run gap, and the step from a list's last row to the zero row K in the lane where the
        // list ends, has to fit the gap width
        bool fits8 = true;
        for (int sign = 0; sign < 2 && fits8; ++sign)
            for (int c = 0; c < N && fits8; ++c) {
                const std::vector<uint16_t> &e = pl->rows[sign][c];
                const int n = pl->n_task[c / g.G], cnt = (int)e.size();
                for (int i = 1; i < cnt; ++i)
                    if (i % n && e[i] - e[i - 1] > 127) fits8 = false;
                if (cnt % n && K - e[cnt - 1] > 127) fits8 = false;
            }
        pl->hdr = 256;
        pl->shift = 0;
        pl->bits = bits_req ? bits_req : (fits8 ? 8 : 16);
        if (!fits8 && bits_req != 16) {
            // Some gap is too long for a signed byte: walk it over zero slots of the tile (the task grows by the longest
            // detour of its lanes) where that takes fewer bytes than 16-bit gaps, or where 8 bits were asked for.
            if (stone_tile_rows(K) + 64 > 65535) {
                if (bits_req == 8) return fail(SPTMM_ERR_UNSUPPORTED, "a gap does not fit 8 bits (signed), and K is too large for a tile with zero slots");
            } else {
                std::vector<int> with_stones(g.tasks, 1);
                if (g.W > 1) return fail(SPTMM_ERR_UNSUPPORTED, "gap streams take at most 64 lanes per column");
                parallel_for(g.tasks, [&](int t) {
                    std::vector<uint16_t> run[64];
                    for (int sign = 0; sign < 2; ++sign) with_stones[t] = std::max(with_stones[t], stone_runs(*pl, t, sign, pl->n_task[t], run));
                });
                size_t bytes8 = 0, bytes16 = 0;
                for (int t = 0; t < g.tasks; ++t) bytes8 += 256 + (size_t)128 * with_stones[t], bytes16 += 256 + (size_t)256 * pl->n_task[t];
                if (bits_req == 8 || bytes8 < bytes16) {
                    pl->stones = true;
                    pl->bits = 8;
                    pl->n_task = with_stones;
                    pl->n_max = *std::max_element(pl->n_task.begin(), pl->n_task.end());
                    pl->n_min = *std::min_element(pl->n_task.begin(), pl->n_task.end());
                }
            }
        }
        pl->esz = pl->bits / 8;
    }
    pl->stride = pl->hdr + (size_t)128 * pl->esz * pl->n_max;
    if (pl->n_max > 65535) return fail(SPTMM_ERR_UNSUPPORTED, "more than 65535 entries per lane");
    pl->counts_bytes = ragged_counts_bytes(g.tasks);
    pl->read_bytes = 16 + 2 * (size_t)g.tasks;
    for (int n : pl->n_task) pl->read_bytes += pl->hdr + (size_t)128 * pl->esz * n;
    return SPTMM_OK;
}

void put_counts(const RaggedPlan &pl, uint8_t *base)
{
    uint32_t *pre = (uint32_t *)base;
    pre[0] = pl.stones ? RAGGED_MAGIC_STONES : RAGGED_MAGIC;
    pre[1] = (uint32_t)pl.g.tasks;
    pre[2] = (uint32_t)pl.n_max;
    pre[3] = (uint32_t)pl.n_min;
    uint16_t *counts = (uint16_t *)(base + 16);
    for (int t = 0; t < pl.g.tasks; ++t) counts[t] = (uint16_t)pl.n_task[t];
}

void pack_u16(const RaggedPlan &pl, uint8_t *stream)
{
    const Geometry &g = pl.g;
    uint8_t *base = stream + pl.counts_bytes;
    auto put = [&](int task, int lane, int slot, int sign, uint16_t row) {
        uint8_t *t = base + (size_t)task * pl.stride;
        *(uint16_t *)(t + pl.hdr + slot_offset(pl.n_task[task], 2, sign, lane, slot)) = (uint16_t)(row << pl.shift);
    };
    if (g.L == 64) {
        parallel_for(g.N, [&](int c) {
            const int nd = 2 * g.W;
            for (int sign = 0; sign < 2; ++sign) {
                std::vector<uint16_t> e = pl.rows[sign][c];
                std::stable_sort(e.begin(), e.end(), [](uint16_t x, uint16_t y) { return (x & 31) < (y & 31); });
                for (int d = 0; d < nd; ++d) {
                    const int task = c * g.W + d / 2;
                    Domain dom;
                    dom.owners = 1;
                    dom.lanes = 32;
                    dom.n = pl.n_task[task];
                    dom.zero_base = pl.K;
                    dom.entries.resize(1);
                    for (size_t i = d; i < e.size(); i += nd) dom.entries[0].push_back(e[i]);
                    schedule(dom);
                    for (int slot = 0; slot < dom.n; ++slot)
                        for (int l = 0; l < 32; ++l) put(task, 32 * (d % 2) + l, slot, sign, dom.cell[0][(size_t)slot * 32 + l]);
                }
            }
        });
    } else {
        // columns that share a half-wavefront are scheduled together: one column when L == 32, else 32/L
        const int group = g.L >= 32 ? 1 : 32 / g.L;
        parallel_for(g.N / group, [&](int gi) {
            for (int sign = 0; sign < 2; ++sign) {
                const int task = gi * group / g.G;
                Domain dom;
                dom.owners = group;
                dom.lanes = g.L;
                dom.n = pl.n_task[task];
                dom.zero_base = pl.K;
                dom.entries.resize(group);
                for (int o = 0; o < group; ++o) dom.entries[o] = pl.rows[sign][gi * group + o];
                schedule(dom);
                for (int o = 0; o < group; ++o) {
                    const int c = gi * group + o, l0 = (c % g.G) * g.L;
                    for (int slot = 0; slot < dom.n; ++slot)
                        for (int l = 0; l < g.L; ++l) put(task, l0 + l, slot, sign, dom.cell[o][(size_t)slot * g.L + l]);
                }
            }
        });
    }
    put_counts(pl, stream);
}

// Lane v of a column owns entries [v*n, (v+1)*n) of the sorted list; where the list ends the lane
// steps to the zero row K and stays there (gap 0), and the lanes behind it start on K.  16-bit
// gaps follow the sorted order; 8-bit gaps are signed and follow the bank-aware order.
// False when the scheduler refused some task's runs (a step that does not fit a signed byte): that task's stream is
// then unwritten and the whole stream must not be used.
bool pack_gaps(const RaggedPlan &pl, uint8_t *stream)
{
    const Geometry &g = pl.g;
    uint8_t *base = stream + pl.counts_bytes;
    std::vector<uint8_t> bad(g.tasks, 0);
    parallel_for(g.tasks, [&](int task) {
        const int n = pl.n_task[task];
        uint8_t *t = base + (size_t)task * pl.stride;
        std::vector<uint16_t> rows[2][64];
        if (pl.stones) {
            // runs of positions; a lane that is done (or owns nothing) steps to the zero slots behind its block and stays
            int n0 = 1;
            for (int sign = 0; sign < 2; ++sign)
                for (int cc = 0; cc < g.G; ++cc) n0 = std::max(n0, ceil_div((int)pl.rows[sign][task * g.G + cc].size(), g.L));
            for (int sign = 0; sign < 2; ++sign) {
                stone_runs(pl, task, sign, n0, rows[sign]);
                for (int lane = 0; lane < 64; ++lane) {
                    std::vector<uint16_t> &r = rows[sign][lane];
                    // (one of the block's 16 zero slots per lane: they lie on different banks)
                    const int rest = (r.empty() ? STONE_ROWS : STONE_BLOCK * (r.back() / STONE_BLOCK) + STONE_ROWS) + (lane & 15);
                    r.resize(n, (uint16_t)rest);
                }
            }
            if (!write_task_runs8(t, n, 65535, rows, pl.bank_shift)) bad[task] = 1;
            return;
        }
        for (int sign = 0; sign < 2; ++sign)
            for (int lane = 0; lane < 64; ++lane) {
                const std::vector<uint16_t> &e = pl.rows[sign][task * g.G + lane / g.L];
                const int cnt = (int)e.size(), first = (lane % g.L) * n;
                std::vector<uint16_t> &r = rows[sign][lane];
                r.resize(n);
                for (int i = 0; i < n; ++i) r[i] = first + i < cnt ? e[first + i] : (uint16_t)pl.K;
            }
        if (pl.esz == 1) {
            if (!write_task_runs8(t, n, pl.K, rows, pl.bank_shift)) bad[task] = 1;  // (the plan has checked that every gap fits)
        } else {
            for (int sign = 0; sign < 2; ++sign)
                for (int lane = 0; lane < 64; ++lane) {
                    const std::vector<uint16_t> &r = rows[sign][lane];
                    *(uint16_t *)(t + sign * 128 + lane * 2) = r[0];
                    for (int i = 0; i < n; ++i) *(uint16_t *)(t + pl.hdr + slot_offset(n, 2, sign, lane, i)) = (uint16_t)(i ? r[i] - r[i - 1] : 0);
                }
        }
    });
    put_counts(pl, stream);
    for (uint8_t b : bad)
        if (b) return false;
    return true;
}

}  // namespace
}  // namespace sptmm

using namespace sptmm;

extern "C" {

int sptmm_generate_ternary_iid(int K, int N, uint32_t seed, double p_pos, double p_neg, int8_t *W)
{
    return guarded([&]() -> int {
        if (int rc = check_ragged_shape(K, N)) return rc;
        if (!W) return fail(SPTMM_ERR_INVALID, "null pointer");
        if (!(p_pos >= 0.0) || !(p_neg >= 0.0) || p_pos + p_neg > 1.0) return fail(SPTMM_ERR_INVALID, "probabilities must be >= 0 and sum to at most 1");
        const uint32_t t_pos = (uint32_t)(p_pos * 16777216.0), t_neg = (uint32_t)((p_pos + p_neg) * 16777216.0);
        parallel_for(N, [&](int c) {
            uint32_t st = seed ^ (0x9E3779B9u * (uint32_t)(c + 1));
            if (!st) st = 1u;
            int8_t *w = W + (size_t)c * K;
            for (int r = 0; r < K; ++r) {
                st ^= st << 13;
                st ^= st >> 17;
                st ^= st << 5;
                const uint32_t u = st >> 8;
                w[r] = u < t_pos ? (int8_t)1 : (u < t_neg ? (int8_t)-1 : (int8_t)0);
            }
        });
        return SPTMM_OK;
    });
}

int sptmm_dense_from_i2s_words(const uint32_t *words, int K, int N, int8_t *W)
{
    return guarded([&]() -> int {
        if (K <= 0 || N <= 0 || K % 16) return fail(SPTMM_ERR_INVALID, "K must be a positive multiple of 16");
        if (!words || !W) return fail(SPTMM_ERR_INVALID, "null pointer");
        for (int c = 0; c < N; ++c)
            for (int g16 = 0; g16 < K / 16; ++g16) {
                int8_t *w = W + (size_t)c * K + 16 * g16;
                sptmm_i2s_decode_word(words[(size_t)c * (K / 16) + g16], w);
                for (int e = 0; e < 16; ++e)
                    if (w[e] < -1 || w[e] > 1) return fail(SPTMM_ERR_INVALID, "column %d, row %d: code 0 is not a ternary weight", c, 16 * g16 + e);
            }
        return SPTMM_OK;
    });
}

size_t sptmm_pack_ragged_bytes(const int8_t *W, int K, int N, int kind, int split_k, int *bits, size_t *read_bytes, int *n_min,
                               int *n_max, uint64_t *nnz)
{
    // the planner allocates and starts threads: nothing it throws may cross the C ABI (0 = failure, message set)
    size_t total = 0;
    const int rc = guarded([&]() -> int {
        RaggedPlan pl;
        if (int prc = ragged_plan(W, K, N, kind, split_k, bits ? *bits : 0, &pl)) return prc;
        if (bits) *bits = pl.bits;
        if (read_bytes) *read_bytes = pl.read_bytes;
        if (n_min) *n_min = pl.n_min;
        if (n_max) *n_max = pl.n_max;
        if (nnz) *nnz = pl.nnz;
        total = pl.counts_bytes + pl.stride * pl.g.tasks;
        return SPTMM_OK;
    });
    return rc == SPTMM_OK ? total : 0;
}

int sptmm_pack_ragged(const int8_t *W, int K, int N, int kind, int split_k, int bits, void *out)
{
    return sptmm_pack_ragged_rows(W, K, N, kind, split_k, bits, 0, out);
}

int sptmm_pack_ragged_rows(const int8_t *W, int K, int N, int kind, int split_k, int bits, int rows, void *out)
{
    return guarded([&]() -> int {
        if (rows < 0) return fail(SPTMM_ERR_INVALID, "rows must be 0 (any) or the activation rows per call");
        RaggedPlan pl;
        if (int rc = ragged_plan(W, K, N, kind, split_k, bits, &pl)) return rc;
        pl.bank_shift = rows == 1 ? 2 : 0;
        if (!out) return fail(SPTMM_ERR_INVALID, "null pointer");
        memset(out, 0, pl.counts_bytes + pl.stride * pl.g.tasks);
        if (kind == SPTMM_KIND_U16)
            pack_u16(pl, (uint8_t *)out);
        else if (!pack_gaps(pl, (uint8_t *)out))
            return fail(SPTMM_ERR_INVALID, "a run of the gap stream has a step that does not fit a signed byte");
        return SPTMM_OK;
    });
}

int sptmm_unpack_ragged(const void *packed, int K, int N, int kind, int split_k, int bits, int8_t *W)
{
    return guarded([&]() -> int {
        if (int rc = check_ragged_shape(K, N)) return rc;
        if (kind != SPTMM_KIND_U16 && kind != SPTMM_KIND_DELTA) return fail(SPTMM_ERR_INVALID, "ragged streams are u16 lists or gap streams");
        Geometry g;
        if (int rc = make_ragged_geometry(N, split_k, kind == SPTMM_KIND_U16 ? 256 : 64, &g)) return rc;
        if (!packed || !W) return fail(SPTMM_ERR_INVALID, "null pointer");
        const bool gaps = kind == SPTMM_KIND_DELTA;
        if (gaps ? (bits != 8 && bits != 16) : bits != 0) return fail(SPTMM_ERR_INVALID, "delta bits must be 8 or 16 (0 for u16 lists)");
        const int esz = gaps ? bits / 8 : 2, hdr = gaps ? 256 : 0, sh = gaps ? 0 : ragged_index_shift(K);
        const uint32_t *pre = (const uint32_t *)packed;
        const uint32_t n_max = pre[2];
        const bool stones = gaps && bits == 8 && pre[0] == RAGGED_MAGIC_STONES;
        if ((pre[0] != RAGGED_MAGIC && !stones) || pre[1] != (uint32_t)g.tasks || n_max < 1 || n_max > 65535 || pre[3] < 1 || pre[3] > n_max)
            return fail(SPTMM_ERR_INVALID, "not a ragged stream of this shape");
        const int tile_rows = stones ? stone_tile_rows(K) : K;
        const uint16_t *counts = (const uint16_t *)((const uint8_t *)packed + 16);
        const uint8_t *base = (const uint8_t *)packed + ragged_counts_bytes(g.tasks);
        const size_t stride = hdr + (size_t)128 * esz * n_max;
        memset(W, 0, (size_t)K * N);
        std::vector<int> bad(g.tasks, 0);
        parallel_for(N / g.G, [&](int ci) {  // all tasks of the columns ci*G .. ci*G+G-1
            for (int part = 0; part < g.W; ++part) {
                const int task = ci * g.W + part;
                const uint8_t *t = base + (size_t)task * stride;
                const uint32_t n = counts[task];
                if (n < pre[3] || n > n_max) {
                    bad[task] = 1;
                    continue;
                }
                for (int sign = 0; sign < 2; ++sign)
                    for (int lane = 0; lane < 64; ++lane) {
                        const int col = g.W > 1 ? ci : ci * g.G + lane / g.L;
                        int row = gaps ? *(const uint16_t *)(t + sign * 128 + lane * 2) : 0;
                        for (int i = 0; i < (int)n; ++i) {
                            const uint8_t *cell = t + hdr + slot_offset((int)n, esz, sign, lane, i);
                            const int f = esz == 1 ? (gaps ? (int)(int8_t)*cell : (int)*cell) : (int)*(const uint16_t *)cell;
                            row = gaps ? row + f : f >> sh;
                            if (row < 0 || row >= tile_rows + 64) {
                                bad[task] = 1;
                                continue;
                            }
                            const int r = stones ? (row < tile_rows ? stone_row(row) : K) : row;
                            if (r < 0 || r >= K) continue;  // padding, or a zero slot on the way over a long gap
                            int8_t &w = W[(size_t)col * K + r];
                            if (w) bad[task] = 1;  // a row may appear once per column
                            w = sign ? (int8_t)-1 : (int8_t)1;
                        }
                    }
            }
        });
        for (int t = 0; t < g.tasks; ++t)
            if (bad[t]) return fail(SPTMM_ERR_INVALID, "corrupt ragged stream (task %d)", t);
        return SPTMM_OK;
    });
}

}  // extern "C"
