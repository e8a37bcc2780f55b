// C ABI over the device side: weight upload, GEMV dispatch by kind, and thin
// memory / stream / event helpers.  See include/sptmm.h for the contract.
#include <hip/hip_runtime.h>

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

int gemv_common(const sptmm_weights *w, const void *X, int M, void *C, void *stream, ActType act, int batch = 0,
                const void *const *bw = nullptr, const void *const *bx = nullptr, void *const *bc = nullptr)
{
    if (!w || !X || !C) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (M < 1) return fail(SPTMM_ERR_INVALID, "M must be at least 1");
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
    a.ragged = w->info.ragged;
    a.compute_units = w->compute_units;
    a.lds_limit = w->lds_limit;
    a.batch = batch;
    a.batch_w = bw;
    a.batch_X = bx;
    a.batch_C = bc;
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
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0) return fail(SPTMM_ERR_HIP, "no HIP device available (%s)", hipGetErrorString(e));
    if (device < 0 || device >= count) return fail(SPTMM_ERR_INVALID, "device %d out of range (have %d)", device, count);
    HIP_TRY(hipSetDevice(device));
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
}

int sptmm_weights_upload_u16(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, sptmm_weights **out)
{
    if (!out) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (int rc = check_shape(K, N, S)) return rc;
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
}

int sptmm_weights_upload_delta(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, sptmm_weights **out)
{
    if (!out) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (int rc = check_shape(K, N, S)) return rc;
    Geometry g;
    if (int rc = make_geometry(N, S, split_k, 64, &g)) return rc;
    int bits = sptmm_delta_bits(pos, neg, N, S, split_k);
    if (bits < 0) return bits;
    std::vector<uint8_t> host(sptmm_pack_delta_bytes(N, S, split_k, bits));
    if (int rc = sptmm_pack_delta(pos, neg, K, N, S, split_k, bits, host.data())) return rc;
    sptmm_weights *w = new (std::nothrow) sptmm_weights();
    if (!w) return fail(SPTMM_ERR_NOMEM, "out of host memory");
    w->info = sptmm_winfo{SPTMM_KIND_DELTA, K, N, S, split_k, bits, 0, 0, (uint64_t)S * N};
    w->geo = g;
    return finish_upload(w, host, out);
}

int sptmm_weights_upload_i2s(const int8_t *W, int K, int N, sptmm_weights **out)
{
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
}

int sptmm_weights_upload_dense(const int8_t *W, int K, int N, int kind, int split_k, sptmm_weights **out)
{
    if (!out) return fail(SPTMM_ERR_INVALID, "null pointer");
    if (kind == SPTMM_KIND_I2S) return sptmm_weights_upload_i2s(W, K, N, out);
    int bits = 0, n_min = 0, n_max = 0;
    size_t read_bytes = 0;
    uint64_t nnz = 0;
    const size_t bytes = sptmm_pack_ragged_bytes(W, K, N, kind, split_k, &bits, &read_bytes, &n_min, &n_max, &nnz);
    if (!bytes) return SPTMM_ERR_INVALID;  // message set by the planner
    std::vector<uint8_t> host(bytes);
    if (int rc = sptmm_pack_ragged(W, K, N, kind, split_k, bits, host.data())) return rc;
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
    return finish_upload(w, host, out);
}

int sptmm_weights_clone(const sptmm_weights *w, sptmm_weights **out)
{
    if (!w || !out) return fail(SPTMM_ERR_INVALID, "null pointer");
    sptmm_weights *c = new (std::nothrow) sptmm_weights(*w);
    if (!c) return fail(SPTMM_ERR_NOMEM, "out of host memory");
    hipError_t e = hipMalloc(&c->dev, w->bytes);
    if (e == hipSuccess) e = hipMemcpy(c->dev, w->dev, w->bytes, hipMemcpyDeviceToDevice);
    if (e != hipSuccess) {
        delete c;
        return hip_fail(e, "clone weight stream");
    }
    *out = c;
    return SPTMM_OK;
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

int sptmm_gemv_i8(const sptmm_weights *w, const int8_t *X, int M, int32_t *C, void *stream)
{
    return gemv_common(w, X, M, C, stream, ACT_I8);
}

int sptmm_gemv_i8_batched(const sptmm_weights *const *ws, const int8_t *const *X, int32_t *const *C, int count, int M,
                          void *stream)
{
    if (!ws || !X || !C || count < 1) return fail(SPTMM_ERR_INVALID, "bad argument");
    if (M < 1) return fail(SPTMM_ERR_INVALID, "M must be at least 1");
    std::vector<const void *> wp(count), xp(count);
    std::vector<void *> cp(count);
    for (int i = 0; i < count; ++i) {
        if (!ws[i] || !X[i] || !C[i]) return fail(SPTMM_ERR_INVALID, "null pointer in batch entry %d", i);
        const sptmm_winfo &a = ws[0]->info, &b = ws[i]->info;
        if (b.kind == SPTMM_KIND_I2S) return fail(SPTMM_ERR_UNSUPPORTED, "batched launches take u16 or gap streams");
        if (a.kind != b.kind || a.K != b.K || a.N != b.N || a.S != b.S || a.split_k != b.split_k || a.delta_bits != b.delta_bits ||
            a.ragged != b.ragged || ws[0]->task_stride != ws[i]->task_stride ||
            ws[0]->n_min != ws[i]->n_min)
            return fail(SPTMM_ERR_INVALID, "batch entry %d differs in kind or shape from entry 0", i);
        wp[i] = ws[i]->dev;
        xp[i] = X[i];
        cp[i] = C[i];
    }
    return gemv_common(ws[0], X[0], M, C[0], stream, ACT_I8, count, wp.data(), xp.data(), cp.data());
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
int sptmm_measure_gemv(const sptmm_weights *const *ws, int n_ws, int act, const void *X, int M, void *C, int iters,
                       int mode, void *stream, double *us_per_call)
{
    if (!ws || n_ws < 1 || !X || !C || iters < 1 || !us_per_call) return fail(SPTMM_ERR_INVALID, "bad argument");
    if (act < ACT_I8 || act > ACT_F32 || mode < 0 || mode > 3) return fail(SPTMM_ERR_INVALID, "bad act or mode");
    if (mode == 3 && act != ACT_I8) return fail(SPTMM_ERR_UNSUPPORTED, "batched timing takes int8 activations");
    if (!stream) return fail(SPTMM_ERR_INVALID, "sptmm_measure_gemv needs a stream made by sptmm_stream_create");
    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0 = nullptr, e1 = nullptr;
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
        for (int i = 0; i < n_ws && rc == SPTMM_OK; ++i) rc = gemv_common(ws[i], X, M, C, st, (ActType)act);
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
        std::vector<const int8_t *> xs(n_ws, (const int8_t *)X);
        std::vector<int32_t *> cs(n_ws);
        for (int i = 0; i < n_ws; ++i) cs[i] = (int32_t *)C + (size_t)i * M * ws[0]->info.N;
        const int reps = (iters + n_ws - 1) / n_ws;
        M_TRY(hipEventRecord(e0, st));
        for (int r = 0; r < reps; ++r) {
            rc = sptmm_gemv_i8_batched(ws, xs.data(), cs.data(), n_ws, M, st);
            if (rc != SPTMM_OK) goto done;
        }
        M_TRY(hipEventRecord(e1, st));
        M_TRY(hipEventSynchronize(e1));
        M_TRY(hipEventElapsedTime(&ms, e0, e1));
        *us_per_call = (double)ms * 1000.0 / ((double)reps * n_ws);
    } else {
        M_TRY(hipEventRecord(e0, st));
        for (int i = 0; i < iters; ++i) {
            rc = gemv_common(ws[i % n_ws], X, M, C, st, (ActType)act);
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
    (void)hipStreamSynchronize(st);
    return rc;
}

int sptmm_copy_kernel(void *dst, const void *src, size_t bytes, void *stream)
{
    if (!dst || !src) return fail(SPTMM_ERR_INVALID, "null pointer");
    return launch_copy(dst, src, bytes, stream);
}

}  // extern "C"
