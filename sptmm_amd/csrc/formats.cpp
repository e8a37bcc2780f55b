// Host side of the SpTMM engine: seeded weight generator and the builders of
// the three device streams.  Pure C++ (no GPU), so it is unit-testable on any
// machine.  The streams are laid out for 64-lane wavefronts: every per-lane
// load of a wavefront touches one contiguous, naturally aligned block.
#include <algorithm>
#include <array>
#include <cstdio>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <thread>
#include <vector>

#include "internal.hpp"

namespace sptmm {

namespace {
Tuning g_tuning;
}
const Tuning &tuning() { return g_tuning; }
void tuning_reload()
{
    auto knob = [](const char *name, int otherwise) {
        const char *v = getenv(name);
        return v && *v ? atoi(v) : otherwise;
    };
    Tuning t;
    t.plan.waves_per_wg = knob("SPTMM_WAVES_PER_WG", 0);
    t.plan.wgs_per_cu = knob("SPTMM_WGS_PER_CU", 0);
    t.plan.tasks_per_wave = knob("SPTMM_TASKS_PER_WAVE", 0);
    t.plan.share_log = knob("SPTMM_SHARE_LOG", 0);
    t.plan.i2s_ct = knob("SPTMM_I2S_CT", 0);
    t.i2s_mfma_from = knob("SPTMM_I2S_MFMA_FROM", 2);
    g_tuning = t;
}


static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

int check_shape(int K, int N, int S)
{
    // main.cu:85-91
    if (K <= 0 || N <= 0 || S <= 0) return fail(SPTMM_ERR_INVALID, "K, N and S must be positive");
    if (K % 16) return fail(SPTMM_ERR_INVALID, "K mod 16 should be 0");
    if (N % 16) return fail(SPTMM_ERR_INVALID, "N mod 16 should be 0");
    if (K >= 65536) return fail(SPTMM_ERR_INVALID, "K should fit an unsigned 16-bit row index");
    if (S % 2) return fail(SPTMM_ERR_INVALID, "S mod 2 must be 0 so that the +1 and -1 lists have the same size");
    if (K <= S) return fail(SPTMM_ERR_INVALID, "K should be bigger than S");
    return SPTMM_OK;
}

int make_geometry(int N, int S, int split_k, int max_split, Geometry *g)
{
    bool ok = false;
    for (int s = 8; s <= max_split; s *= 2) ok |= (s == split_k);
    if (!ok) return fail(SPTMM_ERR_INVALID, "Wrong split size");
    if (N <= 0 || S <= 0) return fail(SPTMM_ERR_INVALID, "N and S must be positive");
    int half = S / 2;
    if (half % split_k) return fail(SPTMM_ERR_INVALID, "Wrong SPLIT Size: (S/2) %% split_k != 0");
    g->N = N;
    g->half = half;
    g->split_k = split_k;
    g->L = std::min(split_k, 64);
    g->G = 64 / g->L;
    g->W = std::max(1, split_k / 64);
    g->n_lane = half / split_k;
    if (N % g->G) return fail(SPTMM_ERR_INVALID, "N must be a multiple of %d for split_k=%d", g->G, split_k);
    g->tasks = N / g->G * g->W;
    return SPTMM_OK;
}

int make_ragged_geometry(int N, int split_k, int max_split, Geometry *g)
{
    bool ok = false;
    for (int s = 8; s <= max_split; s *= 2) ok |= (s == split_k);
    if (!ok) return fail(SPTMM_ERR_INVALID, "Wrong split size");
    if (N <= 0) return fail(SPTMM_ERR_INVALID, "N must be positive");
    g->N = N;
    g->half = 0;
    g->split_k = split_k;
    g->L = std::min(split_k, 64);
    g->G = 64 / g->L;
    g->W = std::max(1, split_k / 64);
    g->n_lane = 0;
    if (N % g->G) return fail(SPTMM_ERR_INVALID, "N must be a multiple of %d for split_k=%d", g->G, split_k);
    g->tasks = N / g->G * g->W;
    return SPTMM_OK;
}

size_t slot_offset(int n_lane, int esz, int sign, int lane, int j)
{
    const int e16 = 16 / esz;
    const int full = n_lane / e16;
    if (j < full * e16) return (size_t)(j / e16) * 2048 + (size_t)sign * 1024 + (size_t)lane * 16 + (size_t)(j % e16) * esz;
    size_t base = (size_t)full * 2048;
    int rem = n_lane - full * e16, first = full * e16;
    for (int w = 8; w >= esz; w /= 2) {
        int cnt = w / esz;
        if (rem & cnt) {
            if (j < first + cnt) return base + (size_t)sign * 64 * w + (size_t)lane * w + (size_t)(j - first) * esz;
            first += cnt;
            base += (size_t)128 * w;
        }
    }
    return (size_t)-1;  // unreachable for j < n_lane
}

// Which (task, lane, slot) holds entry i of column c.  u16 lists interleave a
// column over its split_k lanes (entry i -> lane i % split_k, the assignment of
// main.cu:343-374); gap streams give each lane a contiguous run.
struct Place {
    int task, lane, slot;
};
static inline Place place(const Geometry &g, int c, int i, bool contiguous)
{
    int v = contiguous ? i / g.n_lane : i % g.split_k;  // virtual lane 0..split_k-1
    int slot = contiguous ? i % g.n_lane : i / g.split_k;
    Place p;
    if (g.W > 1) {
        p.task = c * g.W + v / 64;
        p.lane = v % 64;
    } else {
        p.task = c / g.G;
        p.lane = (c % g.G) * g.L + v;
    }
    p.slot = slot;
    return p;
}

static inline uint32_t xorshift32(uint32_t &s)
{
    s ^= s << 13;
    s ^= s >> 17;
    s ^= s << 5;
    return s;
}

}  // namespace sptmm

using namespace sptmm;

extern "C" {

const char *sptmm_last_error(void) { return g_err; }
const char *sptmm_version(void) { return "sptmm-mi355x 0.1 (gfx950)"; }

int sptmm_lists_from_dense(const int8_t *W, int K, int N, int S, uint16_t *pos, uint16_t *neg)
{
    return guarded([&]() -> int {
        if (int rc = check_shape(K, N, S)) return rc;
        if (!W || !pos || !neg) return fail(SPTMM_ERR_INVALID, "null pointer");
        const int half = S / 2;
        std::vector<int> bad(N, 0);
        parallel_for(N, [&](int c) {
            const int8_t *w = W + (size_t)c * K;
            int np = 0, nn = 0;
            for (int r = 0; r < K; ++r) {
                if (w[r] == 1) {
                    if (np < half) pos[(size_t)c * half + np] = (uint16_t)r;
                    ++np;
                } else if (w[r] == -1) {
                    if (nn < half) neg[(size_t)c * half + nn] = (uint16_t)r;
                    ++nn;
                } else if (w[r] != 0) {
                    bad[c] = 1;
                }
            }
            if (np != half || nn != half) bad[c] = 1;
        });
        for (int c = 0; c < N; ++c)
            if (bad[c]) return fail(SPTMM_ERR_INVALID, "W matrix corrupt: column %d is not ternary with S/2 entries per sign", c);
        return SPTMM_OK;
    });
}

int sptmm_generate_ternary(int K, int N, int S, int8_t *W, uint16_t *pos, uint16_t *neg)
{
    return guarded([&]() -> int {
        if (int rc = check_shape(K, N, S)) return rc;
        if (!pos || !neg) return fail(SPTMM_ERR_INVALID, "null pointer");
        const int half = S / 2;
        parallel_for(N, [&](int c) {
            std::vector<int8_t> local;
            int8_t *w;
            if (W) {
                w = W + (size_t)c * K;
            } else {
                local.resize(K);
                w = local.data();
            }
            std::fill(w, w + half, (int8_t)-1);
            std::fill(w + half, w + S, (int8_t)1);
            std::fill(w + S, w + K, (int8_t)0);
            uint32_t st = 0xCAFEBABEu ^ (uint32_t)c;
            for (uint32_t i = (uint32_t)K - 1; i > 0; --i) std::swap(w[i], w[xorshift32(st) % (i + 1)]);
            uint16_t *p = pos + (size_t)c * half, *q = neg + (size_t)c * half;
            for (int r = 0; r < K; ++r) {
                if (w[r] > 0) *p++ = (uint16_t)r;
                if (w[r] < 0) *q++ = (uint16_t)r;
            }
        });
        return SPTMM_OK;
    });
}

int sptmm_make_x_i8(uint32_t seed, size_t count, int8_t *X)
{
    if (!X) return fail(SPTMM_ERR_INVALID, "null pointer");
    uint32_t st = seed ? seed : 1u;
    for (size_t i = 0; i < count; ++i) X[i] = (int8_t)((int)(xorshift32(st) % 255u) - 127);
    return SPTMM_OK;
}

// float -> IEEE half bits, round to nearest even
static uint16_t half_bits(float x)
{
    uint32_t b;
    memcpy(&b, &x, 4);
    const uint32_t sign = (b >> 16) & 0x8000u;
    const int32_t e = (int32_t)((b >> 23) & 0xff) - 127 + 15;
    uint32_t m = b & 0x7fffffu;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        m |= 0x800000u;
        const uint32_t shift = (uint32_t)(14 - e);
        uint32_t h = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (h & 1))) ++h;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((uint32_t)e << 10) | (m >> 13);
    const uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) ++h;
    return (uint16_t)(sign | h);
}

int sptmm_make_x_normal(uint32_t seed, size_t count, float *X32, uint16_t *X16)
{
    if (!X32 && !X16) return fail(SPTMM_ERR_INVALID, "null pointer");
    uint32_t st = seed ? seed : 1u;
    for (size_t i = 0; i < count; i += 2) {
        const double u1 = (xorshift32(st) + 1.0) / 4294967297.0, u2 = xorshift32(st) / 4294967296.0;
        const double r = std::sqrt(-2.0 * std::log(u1));
        const float a = (float)(r * std::cos(6.283185307179586 * u2)), b = (float)(r * std::sin(6.283185307179586 * u2));
        if (X32) X32[i] = a;
        if (X16) X16[i] = half_bits(a);
        if (i + 1 < count) {
            if (X32) X32[i + 1] = b;
            if (X16) X16[i + 1] = half_bits(b);
        }
    }
    return SPTMM_OK;
}

// ------------------------------------------------------------------ u16 stream
// Stored fields are row indices, multiplied by 4 (the byte offset of the row's
// 4-byte LDS slot) whenever 4*K still fits 16 bits.
size_t sptmm_pack_u16_bytes(int N, int S, int split_k)
{
    Geometry g;
    if (make_geometry(N, S, split_k, 256, &g)) return 0;
    return (size_t)g.tasks * 256 * g.n_lane;
}

}  // extern "C"

namespace sptmm {

void schedule(Domain &d)
{
    const int no = d.owners, Lo = d.lanes, n = d.n, NB = d.banks, mask = d.banks - 1;
    std::vector<std::array<std::vector<uint16_t>, 32>> pool(no);
    std::vector<int> wild(no);  // padding cells of each owner, free to take any bank
    for (int o = 0; o < no; ++o) {
        for (uint16_t k : d.entries[o]) pool[o][k & mask].push_back(k);
        wild[o] = n * Lo - (int)d.entries[o].size();
    }
    d.cell.assign(no, std::vector<uint16_t>((size_t)n * Lo));
    std::vector<int> need(no);
    std::vector<std::vector<uint16_t>> pick(no);
    for (int slot = 0; slot < n; ++slot) {
        int open = 0;
        for (int o = 0; o < no; ++o) {
            need[o] = Lo;
            pick[o].clear();
            open += Lo;
        }
        while (open > 0) {  // one sweep = one more entry allowed per bank
            int order[32], total[32];
            for (int b = 0; b < NB; ++b) {
                order[b] = b;
                total[b] = 0;
                for (int o = 0; o < no; ++o) total[b] += (int)pool[o][b].size();
            }
            std::sort(order, order + NB, [&](int x, int y) { return total[x] != total[y] ? total[x] > total[y] : x < y; });
            for (int i = 0; i < NB && open > 0; ++i) {
                const int b = order[i];
                int who = -1;
                for (int o = 0; o < no; ++o)
                    if (need[o] > 0 && !pool[o][b].empty() && (who < 0 || pool[o][b].size() > pool[who][b].size())) who = o;
                if (who < 0) {  // no real entry left for this bank: a padding cell goes here
                    for (int o = 0; o < no; ++o)
                        if (need[o] > 0 && wild[o] > 0 && (who < 0 || wild[o] > wild[who])) who = o;
                    if (who < 0) continue;
                    pick[who].push_back((uint16_t)(d.zero_base + ((b - d.zero_base) & mask)));
                    --wild[who];
                } else {
                    pick[who].push_back(pool[who][b].back());
                    pool[who][b].pop_back();
                }
                --need[who];
                --open;
            }
        }
        for (int o = 0; o < no; ++o) {
            std::sort(pick[o].begin(), pick[o].end(), [mask](uint16_t x, uint16_t y) { return (x & mask) != (y & mask) ? (x & mask) < (y & mask) : x < y; });
            for (int l = 0; l < Lo; ++l) d.cell[o][(size_t)slot * Lo + l] = pick[o][l];
        }
    }
}

bool schedule_runs(RunDomain &d, int window)
{
    const int n = d.n, NL = d.lanes, mask = d.lanes - 1, sh = d.shift;  // lanes of the domain = banks it spreads over
    struct Lane {
        std::vector<char> seen;   // visited entries
        int lo = 0, cur = -1;     // oldest entry not visited yet; row visited last
        std::vector<int> cand;    // this step's candidates (entry indices), most urgent bank first
        int pick = -1;
    } lane[32];
    int demand[32] = {0};         // rows still to visit, per bank, over the whole domain
    for (int l = 0; l < NL; ++l) {
        if ((int)d.rows[l].size() != n) return false;
        for (int i = 1; i < n; ++i)
            if (d.rows[l][i] - d.rows[l][i - 1] > 127) return false;
        for (int i = 0; i < n; ++i)
            if (d.rows[l][i] < d.zero_row) ++demand[(d.rows[l][i] >> sh) & mask];
        lane[l].seen.assign(n, 0);
        d.order[l].assign(n, 0);
    }
    auto fits = [](int step) { return step >= -128 && step <= 127; };
    // Kuhn's augmenting paths, lanes to banks, every bank taking up to `cap` lanes
    struct Matcher {
        Lane *lane;
        RunDomain &d;
        int cap = 1, mask = 31, sh = 0;
        int owners[32][32], count[32];
        bool tried[32];
        bool place(int l)
        {
            for (int i : lane[l].cand) {
                const int row = d.rows[l][i];
                if (row >= d.zero_row) {  // padding: every lane's padding is the same address
                    lane[l].pick = i;
                    return true;
                }
                const int b = (row >> sh) & mask;
                if (tried[b]) continue;
                tried[b] = true;
                if (count[b] < cap) {
                    owners[b][count[b]++] = l;
                    lane[l].pick = i;
                    return true;
                }
                for (int k = 0; k < count[b]; ++k)
                    if (place(owners[b][k])) {
                        owners[b][k] = l;
                        lane[l].pick = i;
                        return true;
                    }
            }
            return false;
        }
    } m{lane, d};
    m.mask = mask;
    m.sh = sh;

    double credit = 0.0;
    for (int step = 0; step < n; ++step) {
        // A bank asked for more often than there are steps left has to be served more than once
        // per step at some point; doing that at an even rate costs the fewest passes overall.
        double q = 1.0;
        for (int b = 0; b < NL; ++b) q = std::max(q, (double)demand[b] / (n - step));
        credit += q;
        const int cap = std::max(1, (int)credit);  // e.g. q = 1.3: one step in three serves every bank twice
        credit -= cap;
        for (int l = 0; l < NL; ++l) {
            Lane &L = lane[l];
            const std::vector<uint16_t> &r = d.rows[l];
            L.cand.clear();
            L.pick = -1;
            int prev = -1;  // last unvisited entry before i
            for (int i = L.lo, taken = 0; i < n && taken < window; ++i) {
                if (L.seen[i]) continue;
                ++taken;
                int next = i + 1;
                while (next < n && L.seen[next]) ++next;
                // a pick must be in reach, must leave its unvisited neighbours in reach of each other,
                // and must leave the oldest unvisited entry in reach of itself
                bool ok = L.cur < 0 || fits(r[i] - L.cur);
                if (ok && prev >= 0 && next < n) ok = fits(r[next] - r[prev]);
                const int lo2 = i == L.lo ? next : L.lo;
                if (ok && lo2 < n) ok = fits(r[lo2] - r[i]);
                if (ok) L.cand.push_back(i);
                prev = i;
            }
            if (L.cand.empty()) return false;  // cannot happen while the sorted gaps fit; kept as a guard
            std::stable_sort(L.cand.begin(), L.cand.end(), [&](int x, int y) {
                const int dx = r[x] >= d.zero_row ? -1 : demand[(r[x] >> sh) & mask], dy = r[y] >= d.zero_row ? -1 : demand[(r[y] >> sh) & mask];
                return dx > dy;
            });
        }
        m.cap = cap;
        for (int b = 0; b < NL; ++b) m.count[b] = 0;
        int load[32] = {0};
        bool placed[32];
        for (int l = 0; l < NL; ++l) {
            for (int b = 0; b < NL; ++b) m.tried[b] = false;
            placed[l] = m.place(l);
        }
        for (int b = 0; b < NL; ++b) load[b] = m.count[b];
        for (int l = 0; l < NL; ++l) {
            Lane &L = lane[l];
            if (!placed[l]) {  // no bank with room: join the least loaded one
                int best = L.cand[0];
                for (int i : L.cand)
                    if (load[(d.rows[l][i] >> sh) & mask] < load[(d.rows[l][best] >> sh) & mask]) best = i;
                L.pick = best;
                ++load[(d.rows[l][best] >> sh) & mask];
            }
            L.seen[L.pick] = 1;
            L.cur = d.rows[l][L.pick];
            if (L.cur < d.zero_row) --demand[(L.cur >> sh) & mask];
            d.order[l][step] = (uint16_t)L.cur;
            while (L.lo < n && L.seen[L.lo]) ++L.lo;
        }
    }
    return true;
}

int u16_index_shift(int K) { return 4 * K <= 65535 ? 2 : 0; }
int ragged_index_shift(int K) { return 4 * (K + 64) <= 65536 ? 2 : 0; }

// Cells of the stream that belong to (column c, sign): calls f(task, lane, slot, i) for i = 0..half-1
// in a fixed enumeration order: part-major, then half-wavefront, then slot, then lane.
template <class F>
void for_cells(const Geometry &g, int c, F f)
{
    int i = 0;
    if (g.L == 64) {
        for (int part = 0; part < g.W; ++part)
            for (int h = 0; h < 2; ++h)
                for (int slot = 0; slot < g.n_lane; ++slot)
                    for (int l = 0; l < 32; ++l) f(c * g.W + part, 32 * h + l, slot, i++);
    } else {
        const int task = c / g.G, l0 = (c % g.G) * g.L;
        for (int slot = 0; slot < g.n_lane; ++slot)
            for (int l = 0; l < g.L; ++l) f(task, l0 + l, slot, i++);
    }
}

}  // namespace sptmm

extern "C" {

int sptmm_choose_split_k(int kind, int N, int S, int compute_units)
{
    // Measured on MI355X over the decoder-layer shapes, K = 2560 ... 13824, N = 128 ... 13824: a lane does best with
    // some 30 to 70 entries per sign (fewer and the per-task overhead shows, more and too few tasks are in flight),
    // and a launch wants at least two tasks per compute unit -- small N pays for that with shorter lanes, down to 24
    // entries: below that a lone launch gains nothing any more and a batched one, which fills the chip with other
    // GEMVs, loses (K=2560 N=640 S=1536, split 32 / 64: alone 3.52 / 3.77 us HBM-cold, 32 per launch 0.33 / 0.41 us
    // per GEMV; K=3072 N=768 S=256, split 8 / 16: 3.64 / 3.69 and 0.19 / 0.26 us).
    const int max_split = kind == SPTMM_KIND_U16 ? 256 : 64;
    if ((kind != SPTMM_KIND_U16 && kind != SPTMM_KIND_DELTA) || N <= 0 || S <= 0 || S % 2) return fail(SPTMM_ERR_INVALID, "no split for this kind or shape");
    const int half = S / 2, cus = compute_units > 0 ? compute_units : 256;
    auto valid = [&](int s) { return s <= max_split && half % s == 0 && N % (s >= 64 ? 1 : 64 / s) == 0; };
    auto tasks = [&](int s) { return (long)N * s / 64; };
    int pick = 0;
    for (int s = 8; s <= max_split; s *= 2)
        if (valid(s)) {
            pick = s;  // (the largest valid one if none gets the lanes short enough)
            if (half / s <= 72) break;
        }
    if (!pick) return fail(SPTMM_ERR_INVALID, "Wrong SPLIT Size: no split_k in 8..%d divides S/2 = %d with N = %d", max_split, half, N);
    while (tasks(pick) < 2L * cus && valid(2 * pick) && half / (2 * pick) >= 24) pick *= 2;
    return pick;
}

int sptmm_pack_u16(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, void *out)
{
    return guarded([&]() -> int {
        if (int rc = check_shape(K, N, S)) return rc;
        Geometry g;
        if (int rc = make_geometry(N, S, split_k, 256, &g)) return rc;
        if (!out || !pos || !neg) return fail(SPTMM_ERR_INVALID, "null pointer");
        for (size_t i = 0, n = (size_t)N * g.half; i < n; ++i)
            if (pos[i] >= K || neg[i] >= K) return fail(SPTMM_ERR_INVALID, "row index out of range");
        const int sh = u16_index_shift(K);
        const size_t task_bytes = (size_t)256 * g.n_lane;
        uint8_t *base = (uint8_t *)out;
        auto put = [&](int task, int lane, int slot, int sign, uint16_t k) {
            *(uint16_t *)(base + task * task_bytes + slot_offset(g.n_lane, 2, sign, lane, slot)) = (uint16_t)(k << sh);
        };
        // groups of columns that share half-wavefronts: one column when L >= 32, else 32/L columns
        const int group = g.L >= 32 ? 1 : 32 / g.L;
        parallel_for(N / group, [&](int gi) {
            for (int sign = 0; sign < 2; ++sign) {
                const uint16_t *lists = sign ? neg : pos;
                if (g.L == 64) {
                    // deal the column's entries, bank by bank, round-robin over its 2*W half-wavefronts
                    const int c = gi, nd = 2 * g.W;
                    std::vector<uint16_t> e(lists + (size_t)c * g.half, lists + (size_t)(c + 1) * g.half);
                    std::stable_sort(e.begin(), e.end(), [](uint16_t x, uint16_t y) { return (x & 31) < (y & 31); });
                    std::vector<Domain> dom(nd);
                    for (int d = 0; d < nd; ++d) {
                        dom[d].owners = 1;
                        dom[d].lanes = 32;
                        dom[d].n = g.n_lane;
                        dom[d].entries.resize(1);
                    }
                    for (int i = 0; i < g.half; ++i) dom[i % nd].entries[0].push_back(e[i]);
                    for (int d = 0; d < nd; ++d) {
                        schedule(dom[d]);
                        for (int slot = 0; slot < g.n_lane; ++slot)
                            for (int l = 0; l < 32; ++l)
                                put(c * g.W + d / 2, 32 * (d % 2) + l, slot, sign, dom[d].cell[0][(size_t)slot * 32 + l]);
                    }
                } else {
                    Domain d;
                    d.owners = group;
                    d.lanes = g.L >= 32 ? 32 : g.L;
                    d.n = g.n_lane;
                    d.entries.resize(group);
                    for (int o = 0; o < group; ++o) {
                        const int c = gi * group + o;
                        d.entries[o].assign(lists + (size_t)c * g.half, lists + (size_t)(c + 1) * g.half);
                    }
                    schedule(d);
                    for (int o = 0; o < group; ++o) {
                        const int c = gi * group + o, task = c / g.G, l0 = (c % g.G) * g.L;
                        for (int slot = 0; slot < g.n_lane; ++slot)
                            for (int l = 0; l < d.lanes; ++l) put(task, l0 + l, slot, sign, d.cell[o][(size_t)slot * d.lanes + l]);
                    }
                }
            }
        });
        return SPTMM_OK;
    });
}

int sptmm_unpack_u16(const void *packed, int K, int N, int S, int split_k, uint16_t *pos, uint16_t *neg)
{
    return guarded([&]() -> int {
        if (int rc = check_shape(K, N, S)) return rc;
        Geometry g;
        if (int rc = make_geometry(N, S, split_k, 256, &g)) return rc;
        if (!packed || !pos || !neg) return fail(SPTMM_ERR_INVALID, "null pointer");
        const int sh = u16_index_shift(K);
        const size_t task_bytes = (size_t)256 * g.n_lane;
        const uint8_t *base = (const uint8_t *)packed;
        parallel_for(N, [&](int c) {
            for (int sign = 0; sign < 2; ++sign) {
                uint16_t *lst = (sign ? neg : pos) + (size_t)c * g.half;
                for_cells(g, c, [&](int task, int lane, int slot, int i) {
                    lst[i] = (uint16_t)(*(const uint16_t *)(base + task * task_bytes + slot_offset(g.n_lane, 2, sign, lane, slot)) >> sh);
                });
                std::sort(lst, lst + g.half);
            }
        });
        return SPTMM_OK;
    });
}

// ---------------------------------------------------------------- gap streams
// Task layout: 256-byte header of first rows, u16 [sign][lane], then the gap
// rounds.  The first gap of every lane is stored as 0 (the header holds the first
// row), so a lane's walk is "row = first; row += gap; gather".  A lane owns a
// contiguous run of the sorted list.  16-bit gaps are unsigned and follow the
// sorted order; 8-bit gaps are signed and follow the order schedule_runs() picks,
// which keeps the lanes of a half-wavefront on different LDS banks.
int sptmm_delta_bits(const uint16_t *pos, const uint16_t *neg, int N, int S, int split_k)
{
    return guarded([&]() -> int {
        Geometry g;
        if (int rc = make_geometry(N, S, split_k, 64, &g)) return rc;
        if (!pos || !neg) return fail(SPTMM_ERR_INVALID, "null pointer");
        for (int sign = 0; sign < 2; ++sign) {
            const uint16_t *l = sign ? neg : pos;
            for (int c = 0; c < N; ++c)
                for (int i = 1; i < g.half; ++i) {
                    if (i % g.n_lane == 0) continue;  // run start: absolute
                    size_t o = (size_t)c * g.half + i;
                    if (l[o] <= l[o - 1]) return fail(SPTMM_ERR_INVALID, "row lists must be strictly ascending");
                    if (l[o] - l[o - 1] > 127) return 16;
                }
        }
        return 8;
    });
}

size_t sptmm_pack_delta_bytes(int N, int S, int split_k, int bits)
{
    Geometry g;
    if (make_geometry(N, S, split_k, 64, &g)) return 0;
    if (bits != 8 && bits != 16) return 0;
    return (size_t)g.tasks * (256 + (size_t)64 * 2 * g.n_lane * (bits / 8));
}

}  // extern "C"

namespace sptmm {

bool write_task_runs8(uint8_t *task, int n, int zero_row, const std::vector<uint16_t> (&rows)[2][64], int bank_shift)
{
    for (int sign = 0; sign < 2; ++sign)
        for (int h = 0; h < 2; ++h) {
            RunDomain d;
            d.n = n;
            d.zero_row = zero_row;
            d.shift = bank_shift;
            for (int l = 0; l < 32; ++l) d.rows[l] = rows[sign][32 * h + l];
            if (!schedule_runs(d)) return false;
            for (int l = 0; l < 32; ++l) {
                const int lane = 32 * h + l;
                *(uint16_t *)(task + sign * 128 + lane * 2) = d.order[l][0];
                for (int j = 0; j < n; ++j)
                    task[256 + slot_offset(n, 1, sign, lane, j)] = (uint8_t)(int8_t)(j ? (int)d.order[l][j] - (int)d.order[l][j - 1] : 0);
            }
        }
    return true;
}

}  // namespace sptmm

extern "C" {

static int delta_walk(bool pack, void *packed, uint16_t *pos, uint16_t *neg, int K, int N, int S, int split_k, int bits, int bank_shift = 0)
{
    if (int rc = check_shape(K, N, S)) return rc;
    Geometry g;
    if (int rc = make_geometry(N, S, split_k, 64, &g)) return rc;
    if (bits != 8 && bits != 16) return fail(SPTMM_ERR_INVALID, "delta bits must be 8 or 16");
    if (!packed || !pos || !neg) return fail(SPTMM_ERR_INVALID, "null pointer");
    const int esz = bits / 8;
    const size_t task_bytes = 256 + (size_t)128 * g.n_lane * esz;
    uint8_t *base = (uint8_t *)packed;
    std::vector<int> bad(N, 0);
    if (pack && bits == 8) {
        for (int sign = 0; sign < 2; ++sign) {
            const uint16_t *l = sign ? neg : pos;
            for (size_t i = 1, e = (size_t)N * g.half; i < e; ++i)
                if (i % g.n_lane && l[i] <= l[i - 1]) return fail(SPTMM_ERR_INVALID, "row lists must be strictly ascending");
        }
        parallel_for(g.tasks, [&](int t) {
            std::vector<uint16_t> rows[2][64];
            for (int sign = 0; sign < 2; ++sign)
                for (int lane = 0; lane < 64; ++lane) {
                    const uint16_t *lst = (sign ? neg : pos) + (size_t)(t * g.G + lane / g.L) * g.half + (size_t)(lane % g.L) * g.n_lane;
                    rows[sign][lane].assign(lst, lst + g.n_lane);
                }
            if (!write_task_runs8(base + (size_t)t * task_bytes, g.n_lane, K, rows, bank_shift)) bad[t * g.G] = 1;
        });
        for (int c = 0; c < N; ++c)
            if (bad[c]) return fail(SPTMM_ERR_INVALID, "column %d: a gap does not fit 8 bits (signed)", c);
        return SPTMM_OK;
    }
    parallel_for(N, [&](int c) {
        for (int sign = 0; sign < 2; ++sign) {
            uint16_t *lst = (sign ? neg : pos) + (size_t)c * g.half;
            int run = 0;
            for (int i = 0; i < g.half; ++i) {
                Place p = place(g, c, i, true);
                uint8_t *task = base + p.task * task_bytes;
                uint16_t *restart = (uint16_t *)(task + sign * 128 + p.lane * 2);
                uint8_t *cell = task + 256 + slot_offset(g.n_lane, esz, sign, p.lane, p.slot);
                if (pack) {
                    unsigned gap = 0;
                    if (p.slot == 0) {
                        *restart = lst[i];
                    } else {
                        gap = (unsigned)lst[i] - lst[i - 1];
                        if (lst[i] <= lst[i - 1]) bad[c] = 1;
                    }
                    if (esz == 1)
                        *cell = (uint8_t)gap;
                    else
                        *(uint16_t *)cell = (uint16_t)gap;
                } else {
                    const int gap = esz == 1 ? (int)(int8_t)*cell : (int)*(uint16_t *)cell;
                    run = p.slot == 0 ? *restart + gap : run + gap;
                    if (run < 0 || run >= K) bad[c] = 1;
                    lst[i] = (uint16_t)run;
                }
            }
            if (!pack) std::sort(lst, lst + g.half);  // 8-bit streams visit a run in scheduled order
        }
    });
    for (int c = 0; c < N; ++c)
        if (bad[c]) return fail(SPTMM_ERR_INVALID, pack ? "column %d: list not ascending" : "column %d: corrupt gap stream", c);
    return SPTMM_OK;
}

int sptmm_pack_delta(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, int bits, void *out)
{
    return sptmm_pack_delta_rows(pos, neg, K, N, S, split_k, bits, 0, out);
}

int sptmm_pack_delta_rows(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, int bits, int rows, void *out)
{
    return guarded([&]() -> int {
        if (rows < 0) return fail(SPTMM_ERR_INVALID, "rows must be 0 (any) or the activation rows per call");
        // shape first: the scan below trusts N and S
        if (int rc = check_shape(K, N, S)) return rc;
        Geometry g;
        if (int rc = make_geometry(N, S, split_k, 64, &g)) return rc;
        if (!out || !pos || !neg) return fail(SPTMM_ERR_INVALID, "null pointer");
        for (size_t i = 0, n = (size_t)N * g.half; i < n; ++i)
            if (pos[i] >= K || neg[i] >= K) return fail(SPTMM_ERR_INVALID, "row index out of range");
        return delta_walk(true, out, (uint16_t *)pos, (uint16_t *)neg, K, N, S, split_k, bits, rows == 1 ? 2 : 0);
    });
}

int sptmm_unpack_delta(const void *packed, int K, int N, int S, int split_k, int bits, uint16_t *pos, uint16_t *neg)
{
    return guarded([&]() -> int {
        return delta_walk(false, (void *)packed, pos, neg, K, N, S, split_k, bits);
    });
}

// ------------------------------------------------------------------------ i2s
uint32_t sptmm_i2s_pack_word(const int8_t w16[16])
{
    uint32_t word = 0;
    for (int e = 0; e < 16; ++e) word |= ((uint32_t)(w16[e] + 2) & 3u) << (8 * (e & 3) + 2 * (e >> 2));
    return word;
}

void sptmm_i2s_decode_word(uint32_t word, int8_t w16[16])
{
    for (int e = 0; e < 16; ++e) w16[e] = (int8_t)((int)((word >> (8 * (e & 3) + 2 * (e >> 2))) & 3u) - 2);
}

size_t sptmm_pack_i2s_bytes(int K, int N)
{
    if (K <= 0 || N <= 0 || K % 16 || N % 16) return 0;
    return (size_t)N * i2s_padded_k(K) / 4;
}

// Word index of rows [16*g16, 16*g16+16) of column c: tiles of 16 columns x 256
// rows (1 KiB); inside a tile lane = quarter*16 + c%16, 4 words per lane -- the order in which
// a 16x16x64 matrix instruction takes its B operand (column = lane mod 16, k-block = lane / 16).
static inline size_t i2s_word_index(int Kp, int c, int g16)
{
    int rounds = Kp / 256, r = g16 / 16, q = (g16 % 16) / 4, j = g16 % 4;
    return ((size_t)(c / 16) * rounds + r) * 256 + (size_t)(q * 16 + c % 16) * 4 + j;
}

int sptmm_pack_i2s(const int8_t *W, int K, int N, void *out)
{
    return guarded([&]() -> int {
        if (K <= 0 || N <= 0 || K % 16 || N % 16) return fail(SPTMM_ERR_INVALID, "K and N must be positive multiples of 16");
        if (!W || !out) return fail(SPTMM_ERR_INVALID, "null pointer");
        const int Kp = i2s_padded_k(K);
        uint32_t *o = (uint32_t *)out;
        std::vector<int> bad(N, 0);
        parallel_for(N, [&](int c) {
            for (int g16 = 0; g16 < Kp / 16; ++g16) {
                int8_t w16[16] = {0};
                if (g16 * 16 < K) {
                    memcpy(w16, W + (size_t)c * K + 16 * g16, 16);
                    for (int e = 0; e < 16; ++e)
                        if (w16[e] < -1 || w16[e] > 1) bad[c] = 1;
                }
                o[i2s_word_index(Kp, c, g16)] = sptmm_i2s_pack_word(w16);
            }
        });
        for (int c = 0; c < N; ++c)
            if (bad[c]) return fail(SPTMM_ERR_INVALID, "column %d holds a weight outside {-1,0,1}", c);
        return SPTMM_OK;
    });
}

int sptmm_unpack_i2s(const void *packed, int K, int N, int8_t *W)
{
    return guarded([&]() -> int {
        if (K <= 0 || N <= 0 || K % 16 || N % 16) return fail(SPTMM_ERR_INVALID, "K and N must be positive multiples of 16");
        if (!W || !packed) return fail(SPTMM_ERR_INVALID, "null pointer");
        const int Kp = i2s_padded_k(K);
        const uint32_t *p = (const uint32_t *)packed;
        for (int c = 0; c < N; ++c)
            for (int g16 = 0; g16 < K / 16; ++g16) sptmm_i2s_decode_word(p[i2s_word_index(Kp, c, g16)], W + (size_t)c * K + 16 * g16);
        return SPTMM_OK;
    });
}

}  // extern "C"
