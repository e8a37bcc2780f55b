// C ABI over the device side: weight upload, GEMV dispatch by kind, and thin
// memory / stream / event helpers.  See include/sptmm.h for the contract.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

#include "internal.hpp"

using namespace sptmm;

struct sptmm_weights {
    sptmm_winfo info;
    Geometry geo;      // unused for i2s
    void *dev;         // the stream
    size_t bytes;
    int device;
    int compute_units;
    int lds_limit;
    int task_stride = 0, counts_bytes = 0;  // ragged streams
    int n_min = 0, n_max = 0;
    int index_shift = 0;  // u16 streams: fields are row << index_shift
    bool byte_rows = false;  // 8-bit gap stream scheduled for a tile of one byte per row
    bool stones = false;     // 8-bit gap stream of tile positions (zero slots behind every 96 rows of the tile)
    bool wide = false;    // wide stream (K-tiled, 16-byte slots): `wh` describes it
    WideHeader wh;
    Plan plans[PLAN_SLOTS];  // the stream's own launch shapes, by kind of call (plan_slot); zeros: the launchers' model
};

namespace {

int hip_fail(hipError_t e, const char *what)
{
    return fail(SPTMM_ERR_HIP, "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
}
#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e_ = (expr);                         \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

struct DevCaps {
    int cus = 0, lds = 0;
};

int device_caps(DevCaps *c)
{
    static thread_local int cached_dev = -1;
    static thread_local DevCaps cached;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev != cached_dev) {
        int v = 0;
        HIP_TRY(hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev));
        cached.cus = v;
        HIP_TRY(hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev));
        cached.lds = v;
        cached_dev = dev;
    }
    *c = cached;
    return SPTMM_OK;
}

// split_k = 0 in an upload call: the library's own choice for this device
int resolve_split(int kind, int N, int S, int *split_k)
{
    if (*split_k != 0) return SPTMM_OK;
    DevCaps caps;
    if (int rc = device_caps(&caps)) return rc;
    const int s = sptmm_choose_split_k(kind, N, S, caps.cus);
    if (s < 0) return s;
    *split_k = s;
    return SPTMM_OK;
}
// the same for an arbitrary ternary matrix: S = twice the mean nonzeros per column and sign, rounded to a multiple of 512
int resolve_split_dense(const int8_t *W, int K, int N, int kind, int *split_k)
{
    if (*split_k != 0 || kind == SPTMM_KIND_I2S) return SPTMM_OK;
    if (!W || K <= 0 || N <= 0) return fail(SPTMM_ERR_INVALID, "bad matrix");
    size_t nnz = 0;
    for (size_t i = 0, n = (size_t)K * N; i < n; ++i) nnz += W[i] != 0;
    long S = (long)((nnz / (size_t)N + 511) / 512 * 512);
    if (S < 512) S = 512;
    return resolve_split(kind, (N + 15) / 16 * 16, (int)S, split_k);
}

// balanced lists -> the dense matrix (column n at W + n*K); SPTMM_ERR_INVALID for a row index beyond K
int dense_from_lists(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, std::vector<int8_t> *W)
{
    if (!pos || !neg) return fail(SPTMM_ERR_INVALID, "null pointer");
    W->assign((size_t)K * N, 0);
    for (int sign = 0; sign < 2; ++sign) {
        const uint16_t *l = sign ? neg : pos;
        for (int c = 0; c < N; ++c)
            for (int i = 0; i < S / 2; ++i) {
                const uint16_t r = l[(size_t)c * (S / 2) + i];
                if (r >= K) return fail(SPTMM_ERR_INVALID, "row index %d out of range in column %d", (int)r, c);
                (*W)[(size_t)c * K + r] = sign ? (int8_t)-1 : (int8_t)1;
            }
    }
    return SPTMM_OK;
}

// Streams declared for more than eight activation rows per call are wide streams: the ordinary ones serve such calls
// in passes of eight rows and read the lists once per pass.
constexpr int ROWS_PER_PASS = 8;

int finish_upload(sptmm_weights *w, const std::vector<uint8_t> &host, sptmm_weights **out)
{
    DevCaps caps;
    if (int rc = device_caps(&caps)) {
        delete w;
        return rc;
    }
    hipError_t e = hipGetDevice(&w->device);
    if (e == hipSuccess) e = hipMalloc(&w->dev, host.size());
    if (e != hipSuccess) {
        delete w;
        return hip_fail(e, "hipMalloc(weight stream)");
    }
    e = hipMemcpy(w->dev, host.data(), host.size(), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(w->dev);
        delete w;
        return hip_fail(e, "hipMemcpy(weight stream)");
    }
    w->bytes = host.size();
    if (!w->info.stream_bytes) w->info.stream_bytes = host.size();
    w->compute_units = caps.cus;
    w->lds_limit = caps.lds;
    *out = w;
    return SPTMM_OK;
}

// what the launchers need to know of one GEMV on `w`
void fill_args(const sptmm_weights *w, const void *X, int M, void *C, GemvArgs *out)
{
    GemvArgs a{};
    a.w = w->dev;
    a.X = X;
    a.C = C;
    a.M = M;
    a.K = w->info.K;
    a.N = w->info.N;
    a.half = w->geo.half;
    a.split_k = w->geo.split_k;
    a.n_lane = w->geo.n_lane;
    a.tasks = w->geo.tasks;
    a.L = w->geo.L;
    a.G = w->geo.G;
    a.W = w->geo.W;
    a.delta_bits = w->info.delta_bits;
    a.task_stride = w->task_stride;
    a.counts_bytes = w->counts_bytes;
    a.n_min = w->n_min;
    a.n_max = w->n_max;
    a.index_shift = w->index_shift;
    a.byte_rows = w->byte_rows;
    a.stones = w->stones;
    a.ragged = w->info.ragged;
    a.compute_units = w->compute_units;
    a.lds_limit = w->lds_limit;
    // A ragged stream whose tasks all hold the same number of entries, and whose tile keeps no zero slots, is laid out
    // behind its count table exactly like a stream of balanced lists (the packers share slot_offset()): it runs on the
    // kernels for tasks of one length -- no table look-ups, straight-line bodies of the exact length (K=6912 N=2560, 864
    // entries per list, 32 GEMVs per launch: 0.81 -> 0.75 us per GEMV).
    if (!w->wide && a.ragged && a.n_min == a.n_max && !a.stones && w->info.kind != SPTMM_KIND_I2S) {
        a.ragged = 0;
        a.n_lane = a.n_max;
        a.w = (const uint8_t *)w->dev + w->counts_bytes;
        a.batch_w_skip = (size_t)w->counts_bytes;  // (the list launchers add it to every stream of a batch)
    }
    *out = a;
}

int gemv_common(const sptmm_weights *w, const void *X, int M, void *C, void *stream, ActType act, int batch = 0,
                const void *const *bw = nullptr, const void *const *bx = nullptr, void *const *bc = nullptr, int quant = 0,
                float w_scale = 1.f, const float *inv = nullptr)
{
    if (!w || !X || !C) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (M < 1) return fail(SPTMM_ERR_INVALID, "M must be at least 1");
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev != w->device) return fail(SPTMM_ERR_INVALID, "the weights live on device %d but device %d is current", w->device, dev);
    GemvArgs a;
    fill_args(w, X, M, C, &a);
    {
        // the stream's plan for this kind of call over the process-wide overrides over the launchers' model
        const Plan &mine = w->plans[plan_slot(M, batch > 0)], &all = tuning().plan;
        a.plan.waves_per_wg = mine.waves_per_wg ? mine.waves_per_wg : all.waves_per_wg;
        a.plan.wgs_per_cu = mine.wgs_per_cu ? mine.wgs_per_cu : all.wgs_per_cu;
        a.plan.tasks_per_wave = mine.tasks_per_wave ? mine.tasks_per_wave : all.tasks_per_wave;
        a.plan.share_log = mine.share_log ? mine.share_log : all.share_log;
        a.plan.i2s_ct = mine.i2s_ct ? mine.i2s_ct : all.i2s_ct;
    }
    a.quant = quant;
    a.w_scale = w_scale;
    a.inv = inv;
    a.batch = batch;
    a.batch_w = bw;
    a.batch_X = bx;
    a.batch_C = bc;
    if (w->wide) {
        if (quant || inv) return fail(SPTMM_ERR_UNSUPPORTED, "the quantising GEMV takes the ordinary u16 or gap streams");
        return launch_wide(a, w->wh, act, stream);
    }
    switch (w->info.kind) {
    case SPTMM_KIND_U16: return launch_u16(a, act, stream);
    case SPTMM_KIND_DELTA: return launch_delta(a, act, stream);
    case SPTMM_KIND_I2S:
        if (act != ACT_I8) return fail(SPTMM_ERR_UNSUPPORTED, "the i2s kernel takes int8 activations only");
        return launch_i2s(a, stream);
    }
    return fail(SPTMM_ERR_INVALID, "corrupt weights object");
}

}  // namespace

extern "C" {

int sptmm_device_init(int device, sptmm_devinfo *out)
{
    return guarded([&]() -> int {
        int count = 0;
        hipError_t e = hipGetDeviceCount(&count);
        if (e != hipSuccess || count == 0) return fail(SPTMM_ERR_HIP, "no HIP device available (%s)", hipGetErrorString(e));
        if (device < 0 || device >= count) return fail(SPTMM_ERR_INVALID, "device %d out of range (have %d)", device, count);
        HIP_TRY(hipSetDevice(device));
        tuning_reload();  // the launch-shape overrides of tuning runs: read here, never on a launch path
        // this device's copy of the static scratch (sptmm_gemv_q8_static); a failed look-up is reported by that call, not here
        (void)scratch_init(device);
        if (out) {
            hipDeviceProp_t pr;
            HIP_TRY(hipGetDeviceProperties(&pr, device));
            memset(out, 0, sizeof *out);
            strncpy(out->name, pr.name, sizeof out->name - 1);
            strncpy(out->arch, pr.gcnArchName, sizeof out->arch - 1);
            out->compute_units = pr.multiProcessorCount;
            out->wave_size = pr.warpSize;
            out->lds_bytes_per_workgroup = (int)pr.sharedMemPerBlock;
            out->l2_bytes = pr.l2CacheSize;
            out->hbm_bytes = pr.totalGlobalMem;
            out->peak_hbm_gbps = 8000.0;  // MI355X HBM3E, published
        }
        return SPTMM_OK;
    });
}

int sptmm_weights_upload_u16(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, sptmm_weights **out)
{
    return sptmm_weights_upload_u16_rows(pos, neg, K, N, S, split_k, 0, out);
}

int sptmm_weights_upload_u16_rows(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, int rows, sptmm_weights **out)
{
    return guarded([&]() -> int {
        if (!out) return fail(SPTMM_ERR_INVALID, "null pointer");
        if (rows < 0) return fail(SPTMM_ERR_INVALID, "rows must be 0 (any) or the activation rows per call");
        if (int rc = check_shape(K, N, S)) return rc;
        if (rows > ROWS_PER_PASS && (split_k == 0 || split_k <= 64)) {
            std::vector<int8_t> W;
            if (int rc = dense_from_lists(pos, neg, K, N, S, &W)) return rc;
            if (int rc = sptmm_weights_upload_wide(W.data(), K, N, SPTMM_KIND_U16, split_k, out)) return rc;
            (*out)->info.S = S;
            return SPTMM_OK;
        }
        if (int rc = resolve_split(SPTMM_KIND_U16, N, S, &split_k)) return rc;
        Geometry g;
        if (int rc = make_geometry(N, S, split_k, 256, &g)) return rc;
        std::vector<uint8_t> host(sptmm_pack_u16_bytes(N, S, split_k));
        if (int rc = sptmm_pack_u16(pos, neg, K, N, S, split_k, host.data())) return rc;
        sptmm_weights *w = new (std::nothrow) sptmm_weights();
        if (!w) return fail(SPTMM_ERR_NOMEM, "out of host memory");
        w->info = sptmm_winfo{SPTMM_KIND_U16, K, N, S, split_k, 0, 0, 0, (uint64_t)S * N};
        w->index_shift = u16_index_shift(K);
        w->geo = g;
        return finish_upload(w, host, out);
    });
}

int sptmm_weights_upload_delta(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, sptmm_weights **out)
{
    return sptmm_weights_upload_delta_rows(pos, neg, K, N, S, split_k, 0, out);
}

int sptmm_weights_upload_delta_rows(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, int rows, sptmm_weights **out)
{
    return guarded([&]() -> int {
        if (!out) return fail(SPTMM_ERR_INVALID, "null pointer");
        if (rows < 0) return fail(SPTMM_ERR_INVALID, "rows must be 0 (any) or the activation rows per call");
        if (int rc = check_shape(K, N, S)) return rc;
        if (rows > ROWS_PER_PASS) {
            std::vector<int8_t> W;
            if (int rc = dense_from_lists(pos, neg, K, N, S, &W)) return rc;
            if (int rc = sptmm_weights_upload_wide(W.data(), K, N, SPTMM_KIND_DELTA, split_k, out)) return rc;
            (*out)->info.S = S;
            return SPTMM_OK;
        }
        if (int rc = resolve_split(SPTMM_KIND_DELTA, N, S, &split_k)) return rc;
        Geometry g;
        if (int rc = make_geometry(N, S, split_k, 64, &g)) return rc;
        int bits = sptmm_delta_bits(pos, neg, N, S, split_k);
        if (bits < 0) return bits;
        if (bits == 16 && K + 64 <= 65535 && (size_t)K * N <= ((size_t)1 << 30)) {  // (the detour builder wants the dense matrix: 1 GiB at most)
            // Some gap is too long for a byte (the reference narrows every gap to u8 unchecked, main.cu:376-394).  The
            // builder for arbitrary matrices can walk long gaps over zero slots of the tile; take its stream where
            // that is smaller than 16-bit gaps throughout.
            std::vector<int8_t> W;
            if (int rc = dense_from_lists(pos, neg, K, N, S, &W)) return rc;
            sptmm_weights *alt = nullptr;
            if (sptmm_weights_upload_dense_rows(W.data(), K, N, SPTMM_KIND_DELTA, split_k, rows, &alt) == SPTMM_OK) {
                if (alt->info.delta_bits == 8) {
                    alt->info.S = S;
                    *out = alt;
                    return SPTMM_OK;
                }
                sptmm_weights_free(alt);
            }
        }
        std::vector<uint8_t> host(sptmm_pack_delta_bytes(N, S, split_k, bits));
        if (int rc = sptmm_pack_delta_rows(pos, neg, K, N, S, split_k, bits, rows, host.data())) return rc;
        sptmm_weights *w = new (std::nothrow) sptmm_weights();
        if (!w) return fail(SPTMM_ERR_NOMEM, "out of host memory");
        w->info = sptmm_winfo{SPTMM_KIND_DELTA, K, N, S, split_k, bits, 0, 0, (uint64_t)S * N};
        w->geo = g;
        w->byte_rows = bits == 8 && rows == 1;
        w->info.row_bytes = bits == 8 ? (rows == 1 ? 1 : 4) : 0;
        return finish_upload(w, host, out);
    });
}

int sptmm_weights_upload_i2s(const int8_t *W, int K, int N, sptmm_weights **out)
{
    return guarded([&]() -> int {
        if (!out) return fail(SPTMM_ERR_INVALID, "null pointer");
        size_t bytes = sptmm_pack_i2s_bytes(K, N);
        if (!bytes) return fail(SPTMM_ERR_INVALID, "K and N must be positive multiples of 16");
        std::vector<uint8_t> host(bytes);
        if (int rc = sptmm_pack_i2s(W, K, N, host.data())) return rc;
        sptmm_weights *w = new (std::nothrow) sptmm_weights();
        if (!w) return fail(SPTMM_ERR_NOMEM, "out of host memory");
        w->info = sptmm_winfo{SPTMM_KIND_I2S, K, N, 0, 0, 0, 0, 0, 0};
        w->geo = Geometry{};
        return finish_upload(w, host, out);
    });
}

int sptmm_weights_upload_dense(const int8_t *W, int K, int N, int kind, int split_k, sptmm_weights **out)
{
    return sptmm_weights_upload_dense_rows(W, K, N, kind, split_k, 0, out);
}

int sptmm_weights_upload_dense_rows(const int8_t *W, int K, int N, int kind, int split_k, int rows, sptmm_weights **out)
{
    return guarded([&]() -> int {
        if (!out) return fail(SPTMM_ERR_INVALID, "null pointer");
        if (rows < 0) return fail(SPTMM_ERR_INVALID, "rows must be 0 (any) or the activation rows per call");
        if (kind == SPTMM_KIND_I2S) return sptmm_weights_upload_i2s(W, K, N, out);
        if (rows > ROWS_PER_PASS && (split_k == 0 || split_k <= 64)) return sptmm_weights_upload_wide(W, K, N, kind, split_k, out);
        if (int rc = resolve_split_dense(W, K, N, kind, &split_k)) return rc;
        int bits = 0, n_min = 0, n_max = 0;
        size_t read_bytes = 0;
        uint64_t nnz = 0;
        const size_t bytes = sptmm_pack_ragged_bytes(W, K, N, kind, split_k, &bits, &read_bytes, &n_min, &n_max, &nnz);
        if (!bytes) return SPTMM_ERR_INVALID;  // message set by the planner
        std::vector<uint8_t> host(bytes);
        if (int rc = sptmm_pack_ragged_rows(W, K, N, kind, split_k, bits, rows, host.data())) return rc;
        sptmm_weights *w = new (std::nothrow) sptmm_weights();
        if (!w) return fail(SPTMM_ERR_NOMEM, "out of host memory");
        w->info = sptmm_winfo{kind, K, N, 0, split_k, bits, read_bytes, 1, nnz};
        if (int rc = make_ragged_geometry(N, split_k, 256, &w->geo)) {
            delete w;
            return rc;
        }
        w->counts_bytes = (int)ragged_counts_bytes(w->geo.tasks);
        w->task_stride = (int)((bytes - w->counts_bytes) / w->geo.tasks);
        w->n_min = n_min;
        w->n_max = n_max;
        w->index_shift = kind == SPTMM_KIND_U16 ? ragged_index_shift(K) : 0;
        w->byte_rows = kind == SPTMM_KIND_DELTA && bits == 8 && rows == 1;
        w->info.row_bytes = kind == SPTMM_KIND_DELTA && bits == 8 ? (rows == 1 ? 1 : 4) : 0;
        w->stones = kind == SPTMM_KIND_DELTA && bits == 8 && *(const uint32_t *)host.data() == RAGGED_MAGIC_STONES;
        w->info.stones = w->stones ? 1 : 0;
        return finish_upload(w, host, out);
    });
}

int sptmm_weights_upload_wide(const int8_t *W, int K, int N, int kind, int split_k, sptmm_weights **out)
{
    return guarded([&]() -> int {
        if (!out) return fail(SPTMM_ERR_INVALID, "null pointer");
        DevCaps caps;
        if (int rc = device_caps(&caps)) return rc;
        const int k_tile = sptmm_wide_k_tile(K, caps.lds);
        if (k_tile < 0) return k_tile;
        if (split_k > 64) return fail(SPTMM_ERR_INVALID, "wide streams take split_k 8, 16, 32 or 64 (or 0: the library's pick), not %d", split_k);
        const bool pick = split_k == 0;
        if (int rc = resolve_split_dense(W, K, N, kind, &split_k)) return rc;
        // the automatic choice is the ordinary streams'; wide tiles do best with at most 32 lanes per column (K=13824 N=5120,
        // 16 rows, 7 GEMVs per launch, split_k 32 / 64: u16 15.7 / 22.4 us per GEMV, gap stream 13.0 / 21.5)
        if (pick && split_k > 32) split_k = 32;
        int bits = 0;
        size_t read_bytes = 0;
        uint64_t nnz = 0;
        const size_t bytes = sptmm_pack_wide_bytes(W, K, N, kind, split_k, k_tile, &bits, &read_bytes, &nnz);
        if (!bytes) return SPTMM_ERR_INVALID;  // message set by the planner
        std::vector<uint8_t> host(bytes);
        if (int rc = sptmm_pack_wide(W, K, N, kind, split_k, k_tile, bits, host.data())) return rc;
        sptmm_weights *w = new (std::nothrow) sptmm_weights();
        if (!w) return fail(SPTMM_ERR_NOMEM, "out of host memory");
        w->info = sptmm_winfo{kind, K, N, 0, split_k, bits, read_bytes, 1, nnz, k_tile};
        w->wide = true;
        if (int rc = wide_parse_header(host.data(), &w->wh)) {
            delete w;
            return rc;
        }
        if (int rc = make_ragged_geometry(N, split_k, 64, &w->geo)) {
            delete w;
            return rc;
        }
        return finish_upload(w, host, out);
    });
}

int sptmm_weights_clone(const sptmm_weights *w, sptmm_weights **out)
{
    return guarded([&]() -> int {
        if (!w || !out) return fail(SPTMM_ERR_INVALID, "null pointer");
        sptmm_weights *c = new (std::nothrow) sptmm_weights(*w);
        if (!c) return fail(SPTMM_ERR_NOMEM, "out of host memory");
        c->dev = nullptr;
        hipError_t e = hipMalloc(&c->dev, w->bytes);
        if (e == hipSuccess) e = hipMemcpy(c->dev, w->dev, w->bytes, hipMemcpyDeviceToDevice);
        // a device-to-device copy need not be complete when hipMemcpy returns, and the streams this library
        // hands out do not order against the null stream: the copy is finished before the clone is handed back
        if (e == hipSuccess) e = hipDeviceSynchronize();
        if (e != hipSuccess) {
            if (c->dev) (void)hipFree(c->dev);
            delete c;
            return hip_fail(e, "clone weight stream");
        }
        *out = c;
        return SPTMM_OK;
    });
}

void sptmm_weights_free(sptmm_weights *w)
{
    if (!w) return;
    (void)hipFree(w->dev);
    delete w;
}

int sptmm_weights_info(const sptmm_weights *w, sptmm_winfo *out)
{
    if (!w || !out) return fail(SPTMM_ERR_INVALID, "null pointer");
    *out = w->info;
    return SPTMM_OK;
}

size_t sptmm_weights_bytes(const sptmm_weights *w) { return w ? w->bytes : 0; }

// ---- weight files: a fixed little-endian header, then the device stream as it is ----
namespace {
struct FileHeader {
    char magic[8];            // "SPTMMW1\0"
    uint32_t header_bytes;    // sizeof(FileHeader)
    uint32_t version;         // 2 (1: i2s tiles in the older lane order, column-major inside a tile; re-tiled on load)
    int32_t kind, K, N, S, split_k, delta_bits, ragged;
    int32_t half, L, G, W, n_lane, tasks;
    int32_t task_stride, counts_bytes, n_min, n_max;
    int32_t index_shift;      // u16 lists: fields are row << index_shift; 8-bit gap streams: 2 when the visiting order was scheduled for
                              // tiles of one byte per row (LDS bank = (row >> 2) mod 32), else 0
    uint64_t nnz, read_bytes, stream_bytes;
    uint64_t fnv1a;           // of the header (this field zero), the plans (version 3) and the stream
};
static_assert(sizeof(FileHeader) == 8 + 4 + 4 + 7 * 4 + 6 * 4 + 5 * 4 + 4 * 8, "file header has no padding");
// version 3: the stream's launch plans follow the header (PLAN_SLOTS x 8 int32), then the stream
typedef int32_t FilePlans[PLAN_SLOTS][8];
static_assert(sizeof(FilePlans) == sizeof(Plan) * PLAN_SLOTS, "a plan is eight int32");
const char FILE_MAGIC[8] = {'S', 'P', 'T', 'M', 'M', 'W', '1', 0};

uint64_t fnv1a(const uint8_t *p, size_t n, uint64_t h = 1469598103934665603ull)
{
    for (size_t i = 0; i < n; ++i) h = (h ^ p[i]) * 1099511628211ull;
    return h;
}

uint64_t file_checksum(FileHeader h, const FilePlans *plans, const std::vector<uint8_t> &stream)
{
    h.fnv1a = 0;
    uint64_t x = fnv1a((const uint8_t *)&h, sizeof h);
    if (plans) x = fnv1a((const uint8_t *)plans, sizeof(FilePlans), x);
    return fnv1a(stream.data(), stream.size(), x);
}
}  // namespace

int sptmm_weights_save(const sptmm_weights *w, const char *path)
{
    return guarded([&]() -> int {
        if (!w || !path) return fail(SPTMM_ERR_INVALID, "null pointer");
        std::vector<uint8_t> host(w->bytes);
        HIP_TRY(hipMemcpy(host.data(), w->dev, w->bytes, hipMemcpyDeviceToHost));
        FileHeader h{};
        memcpy(h.magic, FILE_MAGIC, 8);
        h.header_bytes = (uint32_t)sizeof h;
        h.version = 3;
        FilePlans plans;
        memcpy(plans, w->plans, sizeof plans);
        const sptmm_winfo &i = w->info;
        const Geometry &g = w->geo;
        // ragged: 0 balanced, 1 ragged, 2 wide (K-tiled; the stream's own 512-byte header holds the tiles' offsets and counts)
        h.kind = i.kind, h.K = i.K, h.N = i.N, h.S = i.S, h.split_k = i.split_k, h.delta_bits = i.delta_bits, h.ragged = w->wide ? 2 : i.ragged;
        h.half = g.half, h.L = g.L, h.G = g.G, h.W = g.W, h.n_lane = g.n_lane, h.tasks = g.tasks;
        h.task_stride = w->task_stride, h.counts_bytes = w->counts_bytes, h.n_min = w->n_min, h.n_max = w->n_max;
        h.index_shift = i.kind == SPTMM_KIND_DELTA ? (w->byte_rows ? 2 : 0) : w->index_shift;
        h.nnz = i.nnz, h.read_bytes = i.stream_bytes, h.stream_bytes = w->bytes;
        h.fnv1a = file_checksum(h, &plans, host);
        FILE *f = fopen(path, "wb");
        if (!f) return fail(SPTMM_ERR_INVALID, "cannot open %s for writing", path);
        const bool ok = fwrite(&h, sizeof h, 1, f) == 1 && fwrite(plans, sizeof plans, 1, f) == 1 && fwrite(host.data(), 1, host.size(), f) == host.size();
        if (fclose(f) != 0 || !ok) return fail(SPTMM_ERR_INVALID, "short write to %s", path);
        return SPTMM_OK;
    });
}

int sptmm_weights_load(const char *path, sptmm_weights **out)
{
    return guarded([&]() -> int {
        if (!path || !out) return fail(SPTMM_ERR_INVALID, "null pointer");
        FILE *f = fopen(path, "rb");
        if (!f) return fail(SPTMM_ERR_INVALID, "cannot open %s", path);
        FileHeader h{};
        std::vector<uint8_t> host;
        int rc = SPTMM_OK;
        FilePlans plans = {};
        if (fread(&h, sizeof h, 1, f) != 1 || memcmp(h.magic, FILE_MAGIC, 8) != 0 || h.header_bytes != sizeof h || h.version < 1 || h.version > 3 ||
            (h.version == 3 && fread(plans, sizeof plans, 1, f) != 1))
            rc = fail(SPTMM_ERR_INVALID, "%s is not a weight file of this library", path);
        // every field the kernels index with is checked against the stream size before anything is uploaded
        if (!rc) {
            Geometry g{};
            size_t want = 0;
            if (h.kind == SPTMM_KIND_I2S) {
                want = sptmm_pack_i2s_bytes(h.K, h.N);
            } else if (h.kind == SPTMM_KIND_U16 || h.kind == SPTMM_KIND_DELTA) {
                const int max_split = h.kind == SPTMM_KIND_U16 ? 256 : 64;
                const bool gaps = h.kind == SPTMM_KIND_DELTA;
                if (gaps ? (h.delta_bits != 8 && h.delta_bits != 16) : h.delta_bits != 0) {
                    rc = fail(SPTMM_ERR_INVALID, "%s: bad gap width", path);
                } else if (h.ragged == 2) {
                    // wide stream: shape and geometry here, the K-tiles' tables once the stream is in memory
                    if (h.K <= 0 || h.N <= 0 || h.K % 16 || h.N % 16 || h.K >= 65536 || h.split_k > 64 || make_ragged_geometry(h.N, h.split_k, 64, &g) ||
                        h.index_shift != 0 || h.task_stride != 0 || h.counts_bytes != 0 || h.stream_bytes < 1024 || h.stream_bytes > 0xffffffffull)
                        rc = fail(SPTMM_ERR_INVALID, "%s: inconsistent wide stream header", path);
                    else
                        want = (size_t)h.stream_bytes;
                } else if (h.ragged) {
                    const int esz = gaps ? h.delta_bits / 8 : 2;
                    if (h.K <= 0 || h.N <= 0 || h.K % 16 || h.N % 16 || h.K + 64 > 65535 || make_ragged_geometry(h.N, h.split_k, max_split, &g) ||
                        h.n_min < 1 || h.n_max < h.n_min || h.n_max > 65535 || h.counts_bytes != (int)ragged_counts_bytes(g.tasks) ||
                        h.task_stride != (gaps ? 256 : 0) + 128 * esz * h.n_max ||
                        (gaps ? (h.index_shift != 0 && !(h.index_shift == 2 && h.delta_bits == 8)) : h.index_shift != ragged_index_shift(h.K)))
                        rc = fail(SPTMM_ERR_INVALID, "%s: inconsistent ragged stream header", path);
                    else
                        want = (size_t)h.counts_bytes + (size_t)h.task_stride * g.tasks;
                } else {
                    if (check_shape(h.K, h.N, h.S) || make_geometry(h.N, h.S, h.split_k, max_split, &g) ||
                        (gaps ? (h.index_shift != 0 && !(h.index_shift == 2 && h.delta_bits == 8)) : h.index_shift != u16_index_shift(h.K)))
                        rc = fail(SPTMM_ERR_INVALID, "%s: inconsistent stream header", path);
                    else
                        want = gaps ? sptmm_pack_delta_bytes(h.N, h.S, h.split_k, h.delta_bits) : sptmm_pack_u16_bytes(h.N, h.S, h.split_k);
                }
                if (!rc && (g.half != h.half || g.L != h.L || g.G != h.G || g.W != h.W || g.n_lane != h.n_lane || g.tasks != h.tasks))
                    rc = fail(SPTMM_ERR_INVALID, "%s: geometry does not match the shape", path);
            } else {
                rc = fail(SPTMM_ERR_INVALID, "%s: unknown stream kind %d", path, h.kind);
            }
            if (!rc && (want == 0 || want != h.stream_bytes)) rc = fail(SPTMM_ERR_INVALID, "%s: stream size does not match the shape", path);
        }
        if (!rc) {
            host.resize(h.stream_bytes);
            if (fread(host.data(), 1, host.size(), f) != host.size() || fgetc(f) != EOF)
                rc = fail(SPTMM_ERR_INVALID, "%s: truncated or oversized file", path);
            else if (file_checksum(h, h.version == 3 ? &plans : nullptr, host) != h.fnv1a)
                rc = fail(SPTMM_ERR_INVALID, "%s: checksum mismatch", path);
        }
        fclose(f);
        if (rc) return rc;
        if (h.version == 1 && h.kind == SPTMM_KIND_I2S) {
            // version 1 kept the 16-byte unit of (column c, quarter q) at position 4c + q of its 1 KiB tile; now 16q + c
            std::vector<uint8_t> tile(1024);
            for (size_t t = 0; t + 1024 <= host.size(); t += 1024) {
                memcpy(tile.data(), host.data() + t, 1024);
                for (int c = 0; c < 16; ++c)
                    for (int q = 0; q < 4; ++q) memcpy(host.data() + t + (size_t)(16 * q + c) * 16, tile.data() + (size_t)(4 * c + q) * 16, 16);
            }
        }
        WideHeader wh;
        if (h.ragged == 2) {
            // every offset, stride and count the kernel follows is checked against the stream and the device's LDS
            DevCaps caps;
            if (int crc = device_caps(&caps)) return crc;
            const int esz = h.kind == SPTMM_KIND_U16 ? 2 : h.delta_bits / 8, hdr = h.kind == SPTMM_KIND_DELTA ? 256 : 0;
            if (wide_parse_header(host.data(), &wh)) return fail(SPTMM_ERR_INVALID, "%s: not a wide stream", path);
            bool ok = wh.K == h.K && wh.N == h.N && wh.kind == h.kind && wh.bits == h.delta_bits && wh.split_k == h.split_k && wh.k_tile > 0 &&
                      wh.k_tile % 16 == 0 && wh.k_tile + 64 <= 16383 && wh.phases == (h.K + wh.k_tile - 1) / wh.k_tile;
            if (ok && (size_t)(wh.k_tile + 64) * 16 + 64 > (size_t)caps.lds)
                return fail(SPTMM_ERR_UNSUPPORTED, "%s: K-tiles of %d rows were packed for a larger LDS than this device's %d bytes", path, wh.k_tile, caps.lds);
            const size_t table = ragged_counts_bytes(h.tasks);
            for (int p = 0; ok && p < wh.phases; ++p) {
                const size_t off = wh.offset[p], stride = wh.stride[p];
                ok = off >= 512 && off % 256 == 0 && wh.n_min[p] >= 1 && wh.n_max[p] >= wh.n_min[p] && wh.n_max[p] <= 65535 &&
                     stride == hdr + (size_t)128 * esz * wh.n_max[p] && off + table + stride * h.tasks <= host.size();
                if (!ok) break;
                const uint32_t *pre = (const uint32_t *)(host.data() + off);
                const uint16_t *counts = (const uint16_t *)(host.data() + off + 16);
                ok = pre[0] == RAGGED_MAGIC && pre[1] == (uint32_t)h.tasks && pre[2] == (uint32_t)wh.n_max[p] && pre[3] == (uint32_t)wh.n_min[p];
                for (int t = 0; ok && t < h.tasks; ++t) ok = counts[t] >= wh.n_min[p] && counts[t] <= wh.n_max[p];
            }
            if (!ok) return fail(SPTMM_ERR_INVALID, "%s: corrupt wide stream tables", path);
        } else if (h.ragged && (h.kind == SPTMM_KIND_U16 || h.kind == SPTMM_KIND_DELTA)) {
            // the per-task counts are what the kernel trusts most: keep them inside [n_min, n_max]
            const uint32_t *pre = (const uint32_t *)host.data();
            const uint16_t *counts = (const uint16_t *)(host.data() + 16);
            const bool stones = h.kind == SPTMM_KIND_DELTA && h.delta_bits == 8 && pre[0] == RAGGED_MAGIC_STONES && stone_tile_rows(h.K) + 64 <= 65535;
            bool ok = (pre[0] == RAGGED_MAGIC || stones) && pre[1] == (uint32_t)h.tasks && pre[2] == (uint32_t)h.n_max && pre[3] == (uint32_t)h.n_min;
            for (int t = 0; ok && t < h.tasks; ++t) ok = counts[t] >= h.n_min && counts[t] <= h.n_max;
            if (!ok) return fail(SPTMM_ERR_INVALID, "%s: corrupt count table", path);
        }
        sptmm_weights *w = new (std::nothrow) sptmm_weights();
        if (!w) return fail(SPTMM_ERR_NOMEM, "out of host memory");
        w->info = sptmm_winfo{h.kind, h.K, h.N, h.S, h.split_k, h.delta_bits, h.read_bytes, h.ragged ? 1 : 0, h.nnz};
        w->geo = Geometry{h.N, h.half, h.split_k, h.L, h.G, h.W, h.n_lane, h.tasks};
        memcpy(w->plans, plans, sizeof plans);  // (values a kernel cannot take are ignored at launch)
        if (h.ragged == 2) {
            w->wide = true;
            w->wh = wh;
            w->info.k_tile = wh.k_tile;
            return finish_upload(w, host, out);
        }
        w->task_stride = h.task_stride;
        w->counts_bytes = h.counts_bytes;
        w->n_min = h.n_min;
        w->n_max = h.n_max;
        w->index_shift = h.kind == SPTMM_KIND_DELTA ? 0 : h.index_shift;
        w->byte_rows = h.kind == SPTMM_KIND_DELTA && h.index_shift == 2;
        w->info.row_bytes = h.kind == SPTMM_KIND_DELTA && h.delta_bits == 8 ? (w->byte_rows ? 1 : 4) : 0;
        w->stones = h.ragged && h.kind == SPTMM_KIND_DELTA && h.delta_bits == 8 && *(const uint32_t *)host.data() == RAGGED_MAGIC_STONES;
        w->info.stones = w->stones ? 1 : 0;
        return finish_upload(w, host, out);
    });
}

int sptmm_weights_set_plan(sptmm_weights *w, int M, int batched, const sptmm_plan *plan)
{
    if (!w || !plan) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (M < 1) return fail(SPTMM_ERR_INVALID, "M must be at least 1");
    memcpy(&w->plans[plan_slot(M, batched != 0)], plan, sizeof(Plan));
    return SPTMM_OK;
}

int sptmm_weights_get_plan(const sptmm_weights *w, int M, int batched, sptmm_plan *out)
{
    if (!w || !out) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (M < 1) return fail(SPTMM_ERR_INVALID, "M must be at least 1");
    memcpy(out, &w->plans[plan_slot(M, batched != 0)], sizeof(Plan));
    return SPTMM_OK;
}

int sptmm_weights_tune(sptmm_weights *w, int M, int batch, int act, double *us_model, double *us_tuned)
{
    return guarded([&]() -> int {
        if (!w) return fail(SPTMM_ERR_INVALID, "null pointer");
        if (M < 1 || batch < 0) return fail(SPTMM_ERR_INVALID, "M must be at least 1 and batch at least 0");
        // act 3 / 4: the quantising GEMV on fp16 / bf16 rows (sptmm_gemv_q8), lone launches on ordinary streams
        const bool q8 = act == 3 || act == 4;
        if ((act < ACT_I8 || act > ACT_F32) && !q8) return fail(SPTMM_ERR_INVALID, "act must be 0 (int8), 1 (fp16), 2 (fp32), 3 or 4 (fp16 / bf16 rows quantised in the kernel)");
        if (q8 && (batch > 0 || w->wide || w->info.kind == SPTMM_KIND_I2S))
            return fail(SPTMM_ERR_UNSUPPORTED, "the quantising GEMV is launched alone, on u16 or gap streams");
        if (w->info.kind == SPTMM_KIND_I2S && act != ACT_I8) return fail(SPTMM_ERR_UNSUPPORTED, "the i2s kernel takes int8 activations only");
        const bool batched = batch > 0, lists = w->info.kind != SPTMM_KIND_I2S && !w->wide;
        const int slot = plan_slot(M, batched);
        // device copies to rotate over: enough for ~300 MB (more than the last-level cache holds), in whole batches
        const int per = batched ? std::min(batch, 32) : 1;
        const int by_bytes = (int)std::min<size_t>(64, (300u << 20) / std::max<size_t>(w->bytes, 1) + 1);
        const int groups = std::max(batched ? 1 : 2, (by_bytes + per - 1) / per);
        const int n = groups * per;
        std::vector<sptmm_weights *> owned;
        std::vector<const sptmm_weights *> ws{w};
        void *X = nullptr, *C = nullptr, *stream = nullptr;
        hipEvent_t e0 = nullptr, e1 = nullptr;
        int rc = SPTMM_OK;
        auto cleanup = [&] {
            for (sptmm_weights *c : owned) sptmm_weights_free(c);
            if (X) (void)hipFree(X);
            if (C) (void)hipFree(C);
            if (e0) (void)hipEventDestroy(e0);
            if (e1) (void)hipEventDestroy(e1);
            if (stream) (void)hipStreamDestroy((hipStream_t)stream);
        };
        for (int i = 1; i < n && rc == SPTMM_OK; ++i) {
            sptmm_weights *c = nullptr;
            rc = sptmm_weights_clone(w, &c);
            if (rc == SPTMM_OK) owned.push_back(c), ws.push_back(c);
        }
        const size_t xbytes = (size_t)M * w->info.K * (act == ACT_I8 ? 1 : act == ACT_F32 ? 4 : 2), cbytes = (size_t)4 * M * w->info.N * per;
        if (rc == SPTMM_OK) rc = sptmm_malloc(&X, xbytes);
        if (rc == SPTMM_OK) rc = sptmm_malloc(&C, cbytes);
        if (rc == SPTMM_OK) rc = sptmm_memset(X, 0, xbytes);
        if (rc == SPTMM_OK) rc = sptmm_stream_create(&stream);
        if (rc == SPTMM_OK && (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)) rc = fail(SPTMM_ERR_HIP, "hipEventCreate");
        if (rc != SPTMM_OK) {
            cleanup();
            return rc;
        }
        std::vector<const void *> xs(per, X);
        std::vector<void *> cs(per);
        for (int i = 0; i < per; ++i) cs[i] = (int32_t *)C + (size_t)i * M * w->info.N;
        // `passes` walks over all the copies: one GEMV per launch, or one batched launch per group of `per`
        auto walk = [&](int passes) -> int {
            for (int p = 0; p < passes; ++p)
                for (int g = 0; g < groups; ++g) {
                    const int r = batched ? sptmm_gemv_batched(ws.data() + (size_t)g * per, xs.data(), cs.data(), per, M, act, stream)
                                  : q8    ? gemv_common(ws[g], X, M, C, stream, ACT_I8, 0, nullptr, nullptr, nullptr, act == 3 ? SPTMM_X_F16 : SPTMM_X_BF16, 1.0f)
                                          : gemv_common(ws[g], X, M, C, stream, (ActType)act);
                    if (r != SPTMM_OK) return r;
                }
            return SPTMM_OK;
        };
        // microseconds per GEMV under `plan`: best of three timed loops after a pass of warm-up
        auto time_plan = [&](const Plan &plan, double *us) -> int {
            w->plans[slot] = plan;
            for (sptmm_weights *c : owned) c->plans[slot] = plan;
            const int passes = std::max(2, (batched ? 16 : 64) / groups);
            if (int r = walk(1)) return r;
            double best = 1e30;
            for (int rep = 0; rep < 3; ++rep) {
                float ms = 0.f;
                HIP_TRY(hipEventRecord(e0, (hipStream_t)stream));
                if (int r = walk(passes)) return r;
                HIP_TRY(hipEventRecord(e1, (hipStream_t)stream));
                HIP_TRY(hipEventSynchronize(e1));
                HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
                best = std::min(best, (double)ms * 1000.0 / ((double)passes * n));
            }
            *us = best;
            return SPTMM_OK;
        };
        const Plan before = w->plans[slot];
        Plan best{};
        double t_model = 0, t_best = 0;
        rc = time_plan(best, &t_model);
        t_best = t_model;
        // one dimension at a time, each from the best plan so far
        struct Dim {
            int Plan::*field;
            std::vector<int> values;
        };
        std::vector<Dim> dims;
        if (w->info.kind == SPTMM_KIND_I2S) {
            dims.push_back({&Plan::i2s_ct, {1, 2, 4, 8}});
            dims.push_back({&Plan::waves_per_wg, {1, 2, 4, 8}});
        } else if (w->wide) {
            dims.push_back({&Plan::waves_per_wg, {4, 6, 8, 10, 12, 16}});
        } else if (batched) {
            dims.push_back({&Plan::waves_per_wg, {2, 4, 5, 6, 8, 10, 12, 16}});
            dims.push_back({&Plan::tasks_per_wave, {1, 2, 3, 4, 5, 6, 8, 10, 12, 16}});
        } else {
            dims.push_back({&Plan::waves_per_wg, {2, 4, 5, 6, 8, 10, 12, 16}});
            dims.push_back({&Plan::wgs_per_cu, {1, 2, 3}});
            if (lists && w->info.kind == SPTMM_KIND_U16 && M == 1 && act == ACT_I8) dims.push_back({&Plan::share_log, {-1, 1, 2}});
        }
        for (const Dim &d : dims)
            for (int v : d.values) {
                if (rc != SPTMM_OK) break;
                Plan p = best;
                p.*(d.field) = v;
                double t = 0;
                rc = time_plan(p, &t);
                if (rc == SPTMM_OK && t < t_best) t_best = t, best = p;
            }
        if (rc == SPTMM_OK) {
            // The model's shape stays unless the search found something at least 2 % faster, and still is when both are timed
            // again side by side: the model's first timing is the first work the search puts on the device, and on its own it
            // read up to a tenth slow (the same shape "found" again as a plan the launcher ignores: 3.83 against 3.40 us).
            if (t_best < 0.98 * t_model) {
                double model_again = 0, again = 0;
                rc = time_plan(Plan{}, &model_again);
                if (rc == SPTMM_OK) rc = time_plan(best, &again);
                if (rc == SPTMM_OK) {
                    t_model = std::min(t_model, model_again);
                    if (again >= 0.98 * t_model) best = Plan{}, t_best = t_model;
                    else t_best = std::min(t_best, again);
                }
            } else {
                best = Plan{}, t_best = t_model;
            }
        }
        w->plans[slot] = rc == SPTMM_OK ? best : before;
        if (us_model) *us_model = t_model;
        if (us_tuned) *us_tuned = t_best;
        cleanup();
        return rc;
    });
}

int sptmm_gemv_i8(const sptmm_weights *w, const int8_t *X, int M, int32_t *C, void *stream)
{
    return gemv_common(w, X, M, C, stream, ACT_I8);
}

int sptmm_gemv_batched(const sptmm_weights *const *ws, const void *const *X, void *const *C, int count, int M, int act,
                       void *stream)
{
    return guarded([&]() -> int {
        if (!ws || !X || !C || count < 1) return fail(SPTMM_ERR_INVALID, "bad argument");
        if (act < ACT_I8 || act > ACT_F32) return fail(SPTMM_ERR_INVALID, "act must be 0 (int8), 1 (fp16) or 2 (fp32)");
        if (M < 1) return fail(SPTMM_ERR_INVALID, "M must be at least 1");
        std::vector<const void *> wp(count), xp(count);
        std::vector<void *> cp(count);
        for (int i = 0; i < count; ++i) {
            if (!ws[i] || !X[i] || !C[i]) return fail(SPTMM_ERR_INVALID, "null pointer in batch entry %d", i);
            const sptmm_winfo &a = ws[0]->info, &b = ws[i]->info;
            if (a.kind != b.kind || a.K != b.K || a.N != b.N || a.S != b.S || a.split_k != b.split_k || a.delta_bits != b.delta_bits ||
                a.ragged != b.ragged || a.k_tile != b.k_tile || a.row_bytes != b.row_bytes || a.stones != b.stones || ws[0]->wide != ws[i]->wide ||
                (ws[0]->wide && memcmp(&ws[0]->wh, &ws[i]->wh, sizeof(WideHeader)) != 0) || ws[0]->task_stride != ws[i]->task_stride ||
                ws[0]->n_min != ws[i]->n_min)
                return fail(SPTMM_ERR_INVALID, "batch entry %d differs in kind or shape from entry 0", i);
            wp[i] = ws[i]->dev;
            xp[i] = X[i];
            cp[i] = C[i];
        }
        return gemv_common(ws[0], X[0], M, C[0], stream, (ActType)act, count, wp.data(), xp.data(), cp.data());
    });
}

int sptmm_gemv_i8_batched(const sptmm_weights *const *ws, const int8_t *const *X, int32_t *const *C, int count, int M,
                          void *stream)
{
    return sptmm_gemv_batched(ws, (const void *const *)X, (void *const *)C, count, M, ACT_I8, stream);
}

int sptmm_gemv_q8(const sptmm_weights *w, const uint16_t *X, int x_type, int M, float w_scale, float *Y, void *stream)
{
    if (x_type != SPTMM_X_F16 && x_type != SPTMM_X_BF16) return fail(SPTMM_ERR_INVALID, "x_type must be SPTMM_X_F16 or SPTMM_X_BF16");
    if (w && w->info.kind == SPTMM_KIND_I2S) return fail(SPTMM_ERR_UNSUPPORTED, "the quantising GEMV takes u16 or gap streams");
    return gemv_common(w, X, M, Y, stream, ACT_I8, 0, nullptr, nullptr, nullptr, x_type, w_scale);
}

int sptmm_gemv_i8_scaled(const sptmm_weights *w, const int8_t *Xq, const float *inv, int M, float w_scale, float *Y, void *stream)
{
    if (!inv) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (w && (w->info.kind == SPTMM_KIND_I2S || w->wide)) return fail(SPTMM_ERR_UNSUPPORTED, "scaled sums come from the ordinary u16 or gap streams");
    return gemv_common(w, Xq, M, Y, stream, ACT_I8, 0, nullptr, nullptr, nullptr, 0, w_scale, inv);
}

static bool q8_fused(int M, int K) { return M == 1 || (M <= 4 && (long)M * K <= 32768); }
// workspace of sptmm_gemv_q8_ws: the int8 rows, then (256-byte aligned) the rows' 1/s
static size_t q8_rows_bytes(int M, int K) { return ((size_t)M * K + 255) / 256 * 256; }

// the rows quantised into `workspace` (int8 rows, then their 1/s), then the int8 GEMV scaling its sums by them
static int q8_two_launches(const sptmm_weights *w, const uint16_t *X, int x_type, int M, float w_scale, float *Y, void *workspace, void *stream)
{
    float *inv = reinterpret_cast<float *>((uint8_t *)workspace + q8_rows_bytes(M, w->info.K));
    if (int rc = launch_quantise_rows(X, x_type, M, w->info.K, workspace, inv, stream)) return rc;
    return gemv_common(w, workspace, M, Y, stream, ACT_I8, 0, nullptr, nullptr, nullptr, 0, w_scale, inv);
}

size_t sptmm_gemv_q8_workspace_bytes(const sptmm_weights *w, int M)
{
    if (!w || M < 1) return 0;
    return q8_rows_bytes(M, w->info.K) + ((size_t)M * sizeof(float) + 255) / 256 * 256;
}

int sptmm_gemv_q8_ws(const sptmm_weights *w, const uint16_t *X, int x_type, int M, float w_scale, float *Y, void *workspace, size_t workspace_bytes,
                     void *stream)
{
    if (x_type != SPTMM_X_F16 && x_type != SPTMM_X_BF16) return fail(SPTMM_ERR_INVALID, "x_type must be SPTMM_X_F16 or SPTMM_X_BF16");
    if (!w || !X || !Y) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (M < 1) return fail(SPTMM_ERR_INVALID, "M must be at least 1");
    if (w->info.kind == SPTMM_KIND_I2S || w->wide) return fail(SPTMM_ERR_UNSUPPORTED, "the quantising GEMV takes the ordinary u16 or gap streams");
    // The fused launch quantises all the rows again in every workgroup, each reading M x K values twice: up to 32 K values
    // that is the faster way (K=6912, 4 rows: 8.8 us against 6.2 + 3 in two launches), beyond them it is not (K=6912, 8 rows:
    // 19.0 against 11.8 us; K=13824, 4 rows: 30.7 us fused).  One row always goes the fused way.
    if (q8_fused(M, w->info.K)) return gemv_common(w, X, M, Y, stream, ACT_I8, 0, nullptr, nullptr, nullptr, x_type, w_scale);
    const size_t need = sptmm_gemv_q8_workspace_bytes(w, M);
    if (!workspace || workspace_bytes < need)
        return fail(SPTMM_ERR_INVALID, "workspace of %zu bytes, %zu needed (sptmm_gemv_q8_workspace_bytes)", workspace ? workspace_bytes : (size_t)0, need);
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev != w->device) return fail(SPTMM_ERR_INVALID, "the weights live on device %d but device %d is current", w->device, dev);
    return q8_two_launches(w, X, x_type, M, w_scale, Y, workspace, stream);
}

int sptmm_gemv_q8_static(const sptmm_weights *w, const uint16_t *X, int x_type, int M, float w_scale, float *Y, void *stream)
{
    if (x_type != SPTMM_X_F16 && x_type != SPTMM_X_BF16) return fail(SPTMM_ERR_INVALID, "x_type must be SPTMM_X_F16 or SPTMM_X_BF16");
    if (!w || !X || !Y) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (M < 1) return fail(SPTMM_ERR_INVALID, "M must be at least 1");
    if (w->info.kind == SPTMM_KIND_I2S || w->wide) return fail(SPTMM_ERR_UNSUPPORTED, "the quantising GEMV takes the ordinary u16 or gap streams");
    if (q8_fused(M, w->info.K)) return gemv_common(w, X, M, Y, stream, ACT_I8, 0, nullptr, nullptr, nullptr, x_type, w_scale);  // (no scratch in that launch)
    const size_t need = sptmm_gemv_q8_workspace_bytes(w, M);
    if (need > scratch_bytes())
        return fail(SPTMM_ERR_UNSUPPORTED, "%d rows of K = %d need %zu bytes of scratch, the static array holds %zu: use sptmm_gemv_q8_ws", M, w->info.K,
                    need, scratch_bytes());
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev != w->device) return fail(SPTMM_ERR_INVALID, "the weights live on device %d but device %d is current", w->device, dev);
    void *ptr = nullptr;
    if (int rc = scratch_of(dev, &ptr)) return rc;
    return q8_two_launches(w, X, x_type, M, w_scale, Y, ptr, stream);
}

int sptmm_gemv_f16(const sptmm_weights *w, const uint16_t *X, int M, float *C, void *stream)
{
    return gemv_common(w, X, M, C, stream, ACT_F16);
}

int sptmm_gemv_f32(const sptmm_weights *w, const float *X, int M, float *C, void *stream)
{
    return gemv_common(w, X, M, C, stream, ACT_F32);
}

int sptmm_malloc(void **p, size_t bytes)
{
    if (!p) return fail(SPTMM_ERR_INVALID, "null pointer");
    HIP_TRY(hipMalloc(p, bytes ? bytes : 16));
    return SPTMM_OK;
}
int sptmm_free(void *p)
{
    HIP_TRY(hipFree(p));
    return SPTMM_OK;
}
int sptmm_memcpy_h2d(void *d, const void *s, size_t n)
{
    HIP_TRY(hipMemcpy(d, s, n, hipMemcpyHostToDevice));
    return SPTMM_OK;
}
int sptmm_memcpy_d2h(void *d, const void *s, size_t n)
{
    HIP_TRY(hipMemcpy(d, s, n, hipMemcpyDeviceToHost));
    return SPTMM_OK;
}
int sptmm_memset(void *d, int v, size_t n)
{
    HIP_TRY(hipMemset(d, v, n));
    HIP_TRY(hipStreamSynchronize(nullptr));  // complete on return, whatever stream the caller launches on next
    return SPTMM_OK;
}
int sptmm_stream_create(void **s)
{
    if (!s) return fail(SPTMM_ERR_INVALID, "null pointer");
    hipStream_t st;
    HIP_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    *s = st;
    return SPTMM_OK;
}
int sptmm_stream_destroy(void *s)
{
    HIP_TRY(hipStreamDestroy((hipStream_t)s));
    return SPTMM_OK;
}
int sptmm_stream_sync(void *s)
{
    HIP_TRY(hipStreamSynchronize((hipStream_t)s));
    return SPTMM_OK;
}
int sptmm_device_sync(void)
{
    HIP_TRY(hipDeviceSynchronize());
    return SPTMM_OK;
}
int sptmm_event_create(void **ev)
{
    if (!ev) return fail(SPTMM_ERR_INVALID, "null pointer");
    hipEvent_t e;
    HIP_TRY(hipEventCreate(&e));
    *ev = e;
    return SPTMM_OK;
}
int sptmm_event_destroy(void *ev)
{
    HIP_TRY(hipEventDestroy((hipEvent_t)ev));
    return SPTMM_OK;
}
int sptmm_event_record(void *ev, void *s)
{
    HIP_TRY(hipEventRecord((hipEvent_t)ev, (hipStream_t)s));
    return SPTMM_OK;
}
int sptmm_event_sync(void *ev)
{
    HIP_TRY(hipEventSynchronize((hipEvent_t)ev));
    return SPTMM_OK;
}
int sptmm_event_elapsed_us(void *a, void *b, double *us)
{
    if (!us) return fail(SPTMM_ERR_INVALID, "null pointer");
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, (hipEvent_t)a, (hipEvent_t)b));
    *us = (double)ms * 1000.0;
    return SPTMM_OK;
}
int sptmm_stream_wait_event(void *s, void *ev)
{
    if (!ev) return fail(SPTMM_ERR_INVALID, "null pointer");
    HIP_TRY(hipStreamWaitEvent((hipStream_t)s, (hipEvent_t)ev, 0));
    return SPTMM_OK;
}
struct sptmm_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

int sptmm_graph_begin(void *stream)
{
    if (!stream) return fail(SPTMM_ERR_INVALID, "capture needs a stream made by sptmm_stream_create");
    HIP_TRY(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return SPTMM_OK;
}

int sptmm_graph_end(void *stream, void **graph)
{
    return guarded([&]() -> int {
        if (!stream || !graph) return fail(SPTMM_ERR_INVALID, "null pointer");
        sptmm_graph *g = new (std::nothrow) sptmm_graph();
        if (!g) return fail(SPTMM_ERR_NOMEM, "out of host memory");
        hipError_t e = hipStreamEndCapture((hipStream_t)stream, &g->graph);
        if (e == hipSuccess && !g->graph) e = hipErrorStreamCaptureInvalidated;
        if (e == hipSuccess) e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
        if (e != hipSuccess) {
            if (g->graph) (void)hipGraphDestroy(g->graph);
            delete g;
            return hip_fail(e, "ending the capture");
        }
        *graph = g;
        return SPTMM_OK;
    });
}

int sptmm_graph_launch(void *graph, void *stream)
{
    if (!graph) return fail(SPTMM_ERR_INVALID, "null pointer");
    HIP_TRY(hipGraphLaunch(((sptmm_graph *)graph)->exec, (hipStream_t)stream));
    return SPTMM_OK;
}

int sptmm_graph_destroy(void *graph)
{
    if (!graph) return SPTMM_OK;
    sptmm_graph *g = (sptmm_graph *)graph;
    hipError_t e1 = hipGraphExecDestroy(g->exec), e2 = hipGraphDestroy(g->graph);
    delete g;
    if (e1 != hipSuccess) return hip_fail(e1, "hipGraphExecDestroy");
    if (e2 != hipSuccess) return hip_fail(e2, "hipGraphDestroy");
    return SPTMM_OK;
}

}  // extern "C"

namespace {
int measure_gemv(const sptmm_weights *const *ws, int n_ws, int act, const void *X, int M, void *C, int iters, int mode,
                 void *stream, double *us_per_call)
{
    if (!ws || n_ws < 1 || !X || !C || iters < 1 || !us_per_call) return fail(SPTMM_ERR_INVALID, "bad argument");
    if (act < 0 || act > 4 || mode < 0 || mode > 4) return fail(SPTMM_ERR_INVALID, "bad act or mode");
    if (mode == 4 && act > ACT_F32) return fail(SPTMM_ERR_UNSUPPORTED, "timing over several streams takes int8, fp16 or fp32 activations");
    if (mode == 3 && act > ACT_F32) return fail(SPTMM_ERR_UNSUPPORTED, "batched timing takes int8, fp16 or fp32 activations");
    // act 3 / 4: the quantising GEMV on fp16 / bf16 rows (w_scale 1)
    auto launch = [&](const sptmm_weights *w) {
        return act >= 3 ? sptmm_gemv_q8(w, (const uint16_t *)X, act == 3 ? SPTMM_X_F16 : SPTMM_X_BF16, M, 1.0f, (float *)C, stream)
                        : gemv_common(w, X, M, C, stream, (ActType)act);
    };
    if (!stream) return fail(SPTMM_ERR_INVALID, "sptmm_measure_gemv needs a stream made by sptmm_stream_create");
    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    constexpr int NSTREAMS = 4;
    hipStream_t side[NSTREAMS] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t side_done[NSTREAMS] = {nullptr, nullptr, nullptr, nullptr};
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    int rc = SPTMM_OK;
    float ms = 0.f;
    auto bail = [&](hipError_t e, const char *what) { rc = hip_fail(e, what); };
#define M_TRY(expr)                        \
    do {                                   \
        hipError_t e_ = (expr);            \
        if (e_ != hipSuccess) {            \
            bail(e_, #expr);               \
            goto done;                     \
        }                                  \
    } while (0)
    M_TRY(hipEventCreate(&e0));
    M_TRY(hipEventCreate(&e1));
    if (mode == 2) {
        // one rotation over the weight copies becomes one graph; replay it iters/n_ws times
        M_TRY(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        for (int i = 0; i < n_ws && rc == SPTMM_OK; ++i) rc = launch(ws[i]);
        hipError_t ce = hipStreamEndCapture(st, &graph);
        if (rc != SPTMM_OK) goto done;
        M_TRY(ce);
        M_TRY(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        const int reps = (iters + n_ws - 1) / n_ws;
        M_TRY(hipGraphLaunch(exec, st));  // warm the executable graph
        M_TRY(hipStreamSynchronize(st));
        M_TRY(hipEventRecord(e0, st));
        for (int r = 0; r < reps; ++r) M_TRY(hipGraphLaunch(exec, st));
        M_TRY(hipEventRecord(e1, st));
        M_TRY(hipEventSynchronize(e1));
        M_TRY(hipEventElapsedTime(&ms, e0, e1));
        *us_per_call = (double)ms * 1000.0 / ((double)reps * n_ws);
    } else if (mode == 3) {
        // one launch per rotation: all n_ws GEMVs in a single batched dispatch, outputs side by side in C
        std::vector<const void *> xs(n_ws, X);
        std::vector<void *> cs(n_ws);
        for (int i = 0; i < n_ws; ++i) cs[i] = (int32_t *)C + (size_t)i * M * ws[0]->info.N;  // 4 bytes per output, int32 or float
        const int reps = (iters + n_ws - 1) / n_ws;
        M_TRY(hipEventRecord(e0, st));
        for (int r = 0; r < reps; ++r) {
            rc = sptmm_gemv_batched(ws, xs.data(), cs.data(), n_ws, M, act, st);
            if (rc != SPTMM_OK) goto done;
        }
        M_TRY(hipEventRecord(e1, st));
        M_TRY(hipEventSynchronize(e1));
        M_TRY(hipEventElapsedTime(&ms, e0, e1));
        *us_per_call = (double)ms * 1000.0 / ((double)reps * n_ws);
    } else if (mode == 4) {
        // still one GEMV per launch, but launch i goes to stream i % 4 (default priority, like every stream here): independent
        // GEMVs then overlap the ramp and the tail of their neighbours.  Outputs of the four streams side by side in C.
        for (int s = 0; s < NSTREAMS; ++s) {
            M_TRY(hipStreamCreateWithFlags(&side[s], hipStreamNonBlocking));
            M_TRY(hipEventCreateWithFlags(&side_done[s], hipEventDisableTiming));
        }
        M_TRY(hipEventRecord(e0, st));
        for (int s = 0; s < NSTREAMS; ++s) M_TRY(hipStreamWaitEvent(side[s], e0, 0));
        for (int i = 0; i < iters; ++i) {
            const int s = i % NSTREAMS;
            rc = gemv_common(ws[i % n_ws], X, M, (int32_t *)C + (size_t)s * M * ws[0]->info.N, side[s], (ActType)act);
            if (rc != SPTMM_OK) goto done;
        }
        for (int s = 0; s < NSTREAMS; ++s) {
            M_TRY(hipEventRecord(side_done[s], side[s]));
            M_TRY(hipStreamWaitEvent(st, side_done[s], 0));
        }
        M_TRY(hipEventRecord(e1, st));
        M_TRY(hipEventSynchronize(e1));
        M_TRY(hipEventElapsedTime(&ms, e0, e1));
        *us_per_call = (double)ms * 1000.0 / iters;
    } else {
        M_TRY(hipEventRecord(e0, st));
        for (int i = 0; i < iters; ++i) {
            rc = launch(ws[i % n_ws]);
            if (rc != SPTMM_OK) goto done;
            if (mode == 1) M_TRY(hipStreamSynchronize(st));
        }
        M_TRY(hipEventRecord(e1, st));
        M_TRY(hipEventSynchronize(e1));
        M_TRY(hipEventElapsedTime(&ms, e0, e1));
        *us_per_call = (double)ms * 1000.0 / iters;
    }
done:
#undef M_TRY
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    for (int s = 0; s < NSTREAMS; ++s) {
        if (side[s]) {
            (void)hipStreamSynchronize(side[s]);
            (void)hipStreamDestroy(side[s]);
        }
        if (side_done[s]) (void)hipEventDestroy(side_done[s]);
    }
    (void)hipStreamSynchronize(st);
    return rc;
}
}  // namespace

namespace {
bool same_batch_shape(const sptmm_weights *a, const sptmm_weights *b)
{
    const sptmm_winfo &x = a->info, &y = b->info;
    return x.kind == y.kind && x.K == y.K && x.N == y.N && x.S == y.S && x.split_k == y.split_k && x.delta_bits == y.delta_bits &&
           x.ragged == y.ragged && x.k_tile == y.k_tile && x.row_bytes == y.row_bytes && x.stones == y.stones && a->wide == b->wide &&
           (!a->wide || memcmp(&a->wh, &b->wh, sizeof(WideHeader)) == 0) && a->task_stride == b->task_stride && a->n_min == b->n_min;
}

int measure_sequence(const sptmm_step *steps, int n, int reps, int mode, void *stream, double *us)
{
    if (!steps || n < 1 || reps < 1 || !us) return fail(SPTMM_ERR_INVALID, "bad argument");
    if (mode < 0 || mode > 4) return fail(SPTMM_ERR_INVALID, "mode must be 0..4");
    if (!stream) return fail(SPTMM_ERR_INVALID, "sptmm_measure_sequence needs a stream made by sptmm_stream_create");
    int widest = 1;
    for (int i = 0, run = 0; i < n; ++i) {
        if (!steps[i].w || !steps[i].X_dev || !steps[i].C_dev || steps[i].M < 1 || steps[i].act < ACT_I8 || steps[i].act > ACT_F32)
            return fail(SPTMM_ERR_INVALID, "bad step %d", i);
        if (i > 0 && steps[i].stage < steps[i - 1].stage) return fail(SPTMM_ERR_INVALID, "stages must not decrease (step %d)", i);
        run = i > 0 && steps[i].stage == steps[i - 1].stage ? run + 1 : 1;
        widest = std::max(widest, run);
    }
    constexpr int MAX_SIDE = 7;
    if (widest > MAX_SIDE + 1) return fail(SPTMM_ERR_UNSUPPORTED, "at most %d steps per stage", MAX_SIDE + 1);
    const bool fork = mode == 2 || mode == 3, graphed = mode == 1 || mode == 2;
    hipStream_t st = (hipStream_t)stream;
    hipStream_t side[MAX_SIDE] = {};
    hipEvent_t forked = nullptr, joined[MAX_SIDE] = {}, e0 = nullptr, e1 = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    int rc = SPTMM_OK;
    float ms = 0.f;
    auto bail = [&](hipError_t e, const char *what) { rc = hip_fail(e, what); };
#define M_TRY(expr)                        \
    do {                                   \
        hipError_t e_ = (expr);            \
        if (e_ != hipSuccess) {            \
            bail(e_, #expr);               \
            goto done;                     \
        }                                  \
    } while (0)
    // one pass over the steps: stage by stage, in array order
    auto pass = [&]() -> int {
        for (int i = 0; i < n;) {
            int j = i + 1;
            while (j < n && steps[j].stage == steps[i].stage) ++j;
            if (fork && j - i > 1) {
                hipError_t e = hipEventRecord(forked, st);
                for (int b = 1; b < j - i && e == hipSuccess; ++b) e = hipStreamWaitEvent(side[b - 1], forked, 0);
                if (e != hipSuccess) return hip_fail(e, "forking the stage");
                for (int b = 0; b < j - i; ++b) {
                    const sptmm_step &s = steps[i + b];
                    if (int r = gemv_common(s.w, s.X_dev, s.M, s.C_dev, b ? side[b - 1] : st, (ActType)s.act)) return r;
                }
                for (int b = 1; b < j - i && e == hipSuccess; ++b) {
                    e = hipEventRecord(joined[b - 1], side[b - 1]);
                    if (e == hipSuccess) e = hipStreamWaitEvent(st, joined[b - 1], 0);
                }
                if (e != hipSuccess) return hip_fail(e, "joining the stage");
            } else {
                for (int b = i; b < j;) {
                    int c = b + 1;
                    if (mode == 4)
                        while (c < j && c - b < 32 && steps[c].M == steps[b].M && steps[c].act == steps[b].act && same_batch_shape(steps[b].w, steps[c].w)) ++c;
                    if (c - b > 1) {
                        const sptmm_weights *ws[32];
                        const void *xs[32];
                        void *cs[32];
                        for (int k = b; k < c; ++k) ws[k - b] = steps[k].w, xs[k - b] = steps[k].X_dev, cs[k - b] = steps[k].C_dev;
                        if (int r = sptmm_gemv_batched(ws, xs, cs, c - b, steps[b].M, steps[b].act, st)) return r;
                    } else {
                        const sptmm_step &s = steps[b];
                        if (int r = gemv_common(s.w, s.X_dev, s.M, s.C_dev, st, (ActType)s.act)) return r;
                    }
                    b = c;
                }
            }
            i = j;
        }
        return SPTMM_OK;
    };
    M_TRY(hipEventCreate(&e0));
    M_TRY(hipEventCreate(&e1));
    if (fork) {
        M_TRY(hipEventCreateWithFlags(&forked, hipEventDisableTiming));
        for (int b = 0; b < widest - 1; ++b) {
            M_TRY(hipStreamCreateWithFlags(&side[b], hipStreamNonBlocking));
            M_TRY(hipEventCreateWithFlags(&joined[b], hipEventDisableTiming));
        }
    }
    if (graphed) {
        M_TRY(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        rc = pass();
        hipError_t ce = hipStreamEndCapture(st, &graph);
        if (rc != SPTMM_OK) goto done;
        M_TRY(ce);
        M_TRY(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        M_TRY(hipGraphLaunch(exec, st));
        M_TRY(hipStreamSynchronize(st));
        M_TRY(hipEventRecord(e0, st));
        for (int r = 0; r < reps; ++r) M_TRY(hipGraphLaunch(exec, st));
    } else {
        rc = pass();
        if (rc != SPTMM_OK) goto done;
        M_TRY(hipStreamSynchronize(st));
        M_TRY(hipEventRecord(e0, st));
        for (int r = 0; r < reps; ++r) {
            rc = pass();
            if (rc != SPTMM_OK) goto done;
        }
    }
    M_TRY(hipEventRecord(e1, st));
    M_TRY(hipEventSynchronize(e1));
    M_TRY(hipEventElapsedTime(&ms, e0, e1));
    *us = (double)ms * 1000.0 / reps;
done:
#undef M_TRY
    if (rc != SPTMM_OK) {
        // a capture that failed half way is ended so that the stream is usable again
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) {
            hipGraph_t dead = nullptr;
            (void)hipStreamEndCapture(st, &dead);
            if (dead) (void)hipGraphDestroy(dead);
        }
        (void)hipGetLastError();
    }
    (void)hipStreamSynchronize(st);
    for (int b = 0; b < MAX_SIDE; ++b) {
        if (side[b]) {
            (void)hipStreamSynchronize(side[b]);
            (void)hipStreamDestroy(side[b]);
        }
        if (joined[b]) (void)hipEventDestroy(joined[b]);
    }
    if (forked) (void)hipEventDestroy(forked);
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    return rc;
}
}  // namespace

extern "C" {

int sptmm_measure_sequence(const sptmm_step *steps, int n_steps, int reps, int mode, void *stream, double *us_per_sequence)
{
    return guarded([&]() -> int { return measure_sequence(steps, n_steps, reps, mode, stream, us_per_sequence); });
}

int sptmm_measure_gemv(const sptmm_weights *const *ws, int n_ws, int act, const void *X, int M, void *C, int iters,
                       int mode, void *stream, double *us_per_call)
{
    return guarded([&]() -> int { return measure_gemv(ws, n_ws, act, X, M, C, iters, mode, stream, us_per_call); });
}

int sptmm_read_kernel(const void *src, size_t bytes, size_t stride_bytes, int regions, void *sink, int workgroups, int launches,
                      void *stream, double *us_per_launch)
{
    if (!src || !sink || launches < 1 || regions < 1 || !us_per_launch) return fail(SPTMM_ERR_INVALID, "bad argument");
    if (stride_bytes % 16) return fail(SPTMM_ERR_INVALID, "region stride must be a multiple of 16 bytes");
    if (!stream) return fail(SPTMM_ERR_INVALID, "sptmm_read_kernel needs a stream made by sptmm_stream_create");
    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0, e1;
    HIP_TRY(hipEventCreate(&e0));
    if (hipError_t ce = hipEventCreate(&e1); ce != hipSuccess) {
        (void)hipEventDestroy(e0);
        return hip_fail(ce, "hipEventCreate");
    }
    auto region = [&](int i) { return (const uint8_t *)src + (size_t)(i % regions) * stride_bytes; };
    int rc = launch_read(region(0), bytes, sink, workgroups, stream);  // untimed first launch
    hipError_t e = hipEventRecord(e0, st);
    for (int i = 0; i < launches && rc == SPTMM_OK; ++i) rc = launch_read(region(i + 1), bytes, sink, workgroups, stream);
    if (e == hipSuccess) e = hipEventRecord(e1, st);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != SPTMM_OK) return rc;
    if (e != hipSuccess) return hip_fail(e, "timing the read kernel");
    *us_per_launch = (double)ms * 1000.0 / launches;
    return SPTMM_OK;
}

int sptmm_copy_kernel(void *dst, const void *src, size_t bytes, void *stream)
{
    if (!dst || !src) return fail(SPTMM_ERR_INVALID, "null pointer");
    return launch_copy(dst, src, bytes, stream);
}

}  // extern "C"
