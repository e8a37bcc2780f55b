// rcr -- bench driver with the command line of the reference benchmark
// (main.cu:38-49 flags, main.cu:813-832 banner, one bare "ms per call" float per
// selected method as at main.cu:1459/1845/1962), running on the C ABI of
// libsptmm.so.  No HIP headers here.
//
//   ./rcr -row_split3_small 32 -M=1 -K=6912 -N=2560 -S=4096 -iter=100000
//   ./rcr -row_split_delta2 32 -M=1 -K=6912 -N=2560 -S=4096 -iter=100000
//   ./rcr -i2s -M=1 -K=6912 -N=2560 -S=4096 -iter=100000
//
// Unlike the reference, any shape that passes its own validity rules runs (there
// is no table of compiled-in shapes), activations are seeded, and results are
// checked: every method's device output is compared with a gather-sum over the
// same lists computed here on the host ("# check=PASS"), and that host loop is
// timed on the cores this process may use ("# cpu: ...").  -cpu_only runs the
// host side alone (no device needed): the CPU line, and the gather-sum checked
// against the plain dense product of the same matrix.  -cu_blas runs the dense
// int8 product of the same matrix through rocBLAS, loaded when the flag is given.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <chrono>
#include <iostream>
#include <string>
#include <thread>
#include <vector>

#include <dlfcn.h>
#include <sched.h>

#include "../../include/sptmm.h"

namespace {

struct Flags {
    bool cu_blas = false, i2s = false, check = true, help = false;
    bool cpu = true;        // time the host gather-sum and print the "# cpu:" line
    bool cpu_only = false;  // host side only: no device is touched
    uint64_t row_split3_small = 0, row_split_delta2 = 0;
    uint64_t M = 32, K = 3072, N = 768, S = 256, L = 1;  // defaults of main.cu:43-47
    uint32_t iter = 10;
    // additions of this build
    uint64_t cold = 0;      // rotate over this many device copies of the stream (0 = one copy, as the reference)
    uint64_t seed = 0;      // activation seed (0 = 0xC0FFEE ^ M)
    std::string act = "i8"; // i8 | f16 | f32
};

[[noreturn]] void strict_fail(const char *msg)
{
    // STRICT_ASSERT of macro.cuh:66
    fprintf(stderr, "%s\n", msg);
    abort();
}

#define CHECK_SPTMM(expr)                                                                          \
    do {                                                                                           \
        int rc_ = (expr);                                                                          \
        if (rc_ == SPTMM_ERR_INVALID) strict_fail(sptmm_last_error());                             \
        if (rc_ != SPTMM_OK) {                                                                     \
            fprintf(stderr, "HIP error at %s:%d code=%d \"%s\" (%s)\n", __FILE__, __LINE__, rc_,   \
                    #expr, sptmm_last_error());                                                    \
            exit(EXIT_FAILURE);                                                                    \
        }                                                                                          \
    } while (0)

bool parse_bool(const std::string &v, bool *out)
{
    if (v == "true" || v == "1" || v == "t" || v == "yes" || v == "y") return *out = true, true;
    if (v == "false" || v == "0" || v == "f" || v == "no" || v == "n") return *out = false, true;
    return false;
}

// gflags grammar as the reference's README uses it: one or two dashes, "-flag value" or
// "-flag=value"; booleans also as "-flag" / "-noflag".  Unknown flag: message + exit 1.
void parse(int argc, char **argv, Flags &f)
{
    struct Spec {
        const char *name;
        int kind;  // 0 bool, 1 u64, 2 u32, 3 string
        void *dst;
    } specs[] = {
        {"cu_blas", 0, &f.cu_blas}, {"i2s", 0, &f.i2s}, {"check", 0, &f.check}, {"help", 0, &f.help}, {"cpu", 0, &f.cpu}, {"cpu_only", 0, &f.cpu_only},
        {"row_split3_small", 1, &f.row_split3_small}, {"row_split_delta2", 1, &f.row_split_delta2},
        {"M", 1, &f.M}, {"K", 1, &f.K}, {"N", 1, &f.N}, {"S", 1, &f.S}, {"L", 1, &f.L},
        {"iter", 2, &f.iter}, {"cold", 1, &f.cold}, {"seed", 1, &f.seed}, {"act", 3, &f.act},
    };
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "--") break;
        if (a.size() < 2 || a[0] != '-') {
            fprintf(stderr, "ERROR: unexpected argument '%s'\n", a.c_str());
            exit(1);
        }
        a = a.substr(a[1] == '-' ? 2 : 1);
        std::string name = a, val;
        bool has_val = false;
        size_t eq = a.find('=');
        if (eq != std::string::npos) {
            name = a.substr(0, eq);
            val = a.substr(eq + 1);
            has_val = true;
        }
        Spec *sp = nullptr;
        bool negated = false;
        for (auto &s : specs)
            if (name == s.name) sp = &s;
        if (!sp && name.rfind("no", 0) == 0)
            for (auto &s : specs)
                if (s.kind == 0 && name.substr(2) == s.name) sp = &s, negated = true;
        if (!sp) {
            fprintf(stderr, "ERROR: unknown command line flag '%s'\n", name.c_str());
            exit(1);
        }
        if (sp->kind == 0) {
            bool b = !negated;
            if (has_val && (negated || !parse_bool(val, &b))) {
                fprintf(stderr, "ERROR: illegal value '%s' specified for bool flag '%s'\n", val.c_str(), sp->name);
                exit(1);
            }
            *(bool *)sp->dst = b;
            continue;
        }
        if (!has_val) {
            if (i + 1 >= argc) {
                fprintf(stderr, "ERROR: flag '%s' is missing its argument\n", sp->name);
                exit(1);
            }
            val = argv[++i];
        }
        if (sp->kind == 3) {
            *(std::string *)sp->dst = val;
            continue;
        }
        char *end = nullptr;
        unsigned long long v = strtoull(val.c_str(), &end, 0);
        if (val.empty() || *end || val[0] == '-' || (sp->kind == 2 && v > 0xffffffffull)) {
            fprintf(stderr, "ERROR: illegal value '%s' specified for %s flag '%s'\n", val.c_str(),
                    sp->kind == 1 ? "uint64" : "uint32", sp->name);
            exit(1);
        }
        if (sp->kind == 1)
            *(uint64_t *)sp->dst = v;
        else
            *(uint32_t *)sp->dst = (uint32_t)v;
    }
}

float half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    uint32_t b;
    if (e == 0) {
        if (!m) {
            b = sign;
        } else {  // subnormal: value = m * 2^-24
            float v = (float)m * 5.9604644775390625e-8f;
            memcpy(&b, &v, 4);
            b |= sign;
        }
    } else if (e == 31) {
        b = sign | 0x7f800000u | (m << 13);
    } else {
        b = sign | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &b, 4);
    return f;
}

// cores this process may run on
int affinity_cores()
{
    cpu_set_t set;
    CPU_ZERO(&set);
    if (sched_getaffinity(0, sizeof set, &set) != 0) return 1;
    const int n = CPU_COUNT(&set);
    return n > 0 ? n : 1;
}

// body(c0, c1) over [0, n) split statically across `threads` threads
template <class F> void over_columns(int n, int threads, F body)
{
    if (threads <= 1) {
        body(0, n);
        return;
    }
    std::vector<std::thread> th;
    for (int t = 0; t < threads; ++t) th.emplace_back([=] { body((int)((long)n * t / threads), (int)((long)n * (t + 1) / threads)); });
    for (auto &t : th) t.join();
}

// All threads meet here between repetitions of a timed loop (the workers live for the whole loop, so that no
// repetition pays for starting them).
struct SpinBarrier {
    explicit SpinBarrier(int n) : n_(n) {}
    void wait()
    {
        const int gen = gen_.load(std::memory_order_acquire);
        if (count_.fetch_add(1, std::memory_order_acq_rel) + 1 == n_) {
            count_.store(0, std::memory_order_relaxed);
            gen_.fetch_add(1, std::memory_order_release);
        } else {
            int spins = 0;
            while (gen_.load(std::memory_order_acquire) == gen)
                if (++spins > 2000) std::this_thread::yield();
        }
    }
    const int n_;
    std::atomic<int> count_{0}, gen_{0};
};

// `reps` calls of body(c0, c1) over [0, n) on `threads` persistent threads; microseconds of every call (barrier to barrier)
template <class F> std::vector<double> timed_over_columns(int n, int threads, int max_reps, double budget_s, F body)
{
    typedef std::chrono::steady_clock clk;
    std::vector<double> t;
    SpinBarrier bar(threads);
    std::atomic<bool> stop{false};
    auto worker = [&](int id) {
        const int c0 = (int)((long)n * id / threads), c1 = (int)((long)n * (id + 1) / threads);
        const auto begin = clk::now();
        for (int rep = -3;; ++rep) {  // three warm-ups
            bar.wait();
            const auto t0 = clk::now();
            if (stop.load(std::memory_order_acquire)) break;
            body(c0, c1);
            bar.wait();
            if (id == 0) {
                const auto t1 = clk::now();
                if (rep >= 0) t.push_back(std::chrono::duration<double, std::micro>(t1 - t0).count());
                if ((int)t.size() >= max_reps || ((int)t.size() >= 3 && std::chrono::duration<double>(t1 - begin).count() > budget_s))
                    stop.store(true, std::memory_order_release);
            }
        }
    };
    std::vector<std::thread> th;
    for (int i = 1; i < threads; ++i) th.emplace_back(worker, i);
    worker(0);
    for (auto &x : th) x.join();
    return t;
}

// The reference kernel's sum on the host (main.cu:577-593): C[m][n] = sum X[m][pos(n)] - sum X[m][neg(n)],
// int32 for int8 rows, double for float rows.  X is [M][K] of T; out is [M][N].
template <class T, class A, class Conv>
void host_gather_columns(const T *X, int M, int K, int N, int half, const uint16_t *pos, const uint16_t *neg, int c0, int c1, A *out, Conv conv)
{
    for (int m = 0; m < M; ++m) {
        const T *x = X + (size_t)m * K;
        for (int c = c0; c < c1; ++c) {
            const uint16_t *p = pos + (size_t)c * half, *q = neg + (size_t)c * half;
            A acc = 0;
            for (int i = 0; i < half; ++i) acc += (A)conv(x[p[i]]) - (A)conv(x[q[i]]);
            out[(size_t)m * N + c] = acc;
        }
    }
}

// the textbook product with the dense matrix (column n at W + n*K): the host's own second opinion on the lists
template <class T, class A, class Conv>
void host_dense_product(const T *X, int M, int K, int N, const int8_t *W, int threads, A *out, Conv conv)
{
    over_columns(N, threads, [=](int c0, int c1) {
        for (int m = 0; m < M; ++m)
            for (int c = c0; c < c1; ++c) {
                const int8_t *w = W + (size_t)c * K;
                A acc = 0;
                for (int k = 0; k < K; ++k) acc += (A)conv(X[(size_t)m * K + k]) * (A)w[k];
                out[(size_t)m * N + c] = acc;
            }
    });
}

// The dense int8 product through rocBLAS, loaded at run time (no link-time dependency): what main.cu:842-873 asks of
// cuBLAS, in the layouts this build has -- X row-major [M][K], W column-major [K][N], C row-major [M][N], which in the
// library's column-major terms is C^T [N x M] = W^T [N x K] * X^T [K x M].  (The reference's own line only runs in an
// all-column-major build and passes a null weight pointer, main.cu:836, 863.)
struct DenseBlas {
    typedef int (*create_fn)(void **);
    typedef int (*destroy_fn)(void *);
    typedef int (*set_stream_fn)(void *, void *);
    typedef int (*gemm_ex_fn)(void *, int, int, int, int, int, const void *, const void *, int, int, const void *, int, int, const void *,
                              const void *, int, int, void *, int, int, int, int, int32_t, uint32_t);
    void *so = nullptr, *handle = nullptr;
    create_fn create = nullptr;
    destroy_fn destroy = nullptr;
    set_stream_fn set_stream = nullptr;
    gemm_ex_fn gemm_ex = nullptr;

    bool open(void *stream, std::string *why)
    {
        for (const char *name : {"librocblas.so.5", "librocblas.so", "/opt/rocm/lib/librocblas.so"})
            if ((so = dlopen(name, RTLD_NOW | RTLD_LOCAL))) break;
        if (!so) return *why = std::string("cannot load rocBLAS: ") + dlerror(), false;
        create = (create_fn)dlsym(so, "rocblas_create_handle");
        destroy = (destroy_fn)dlsym(so, "rocblas_destroy_handle");
        set_stream = (set_stream_fn)dlsym(so, "rocblas_set_stream");
        gemm_ex = (gemm_ex_fn)dlsym(so, "rocblas_gemm_ex");
        if (!create || !destroy || !set_stream || !gemm_ex) return *why = "rocBLAS lacks rocblas_gemm_ex", false;
        if (int rc = create(&handle)) return *why = "rocblas_create_handle: status " + std::to_string(rc), false;
        if (int rc = set_stream(handle, stream)) return *why = "rocblas_set_stream: status " + std::to_string(rc), false;
        return true;
    }
    // rocblas_operation_transpose = 112, _none = 111; rocblas_datatype_i8_r = 160, _i32_r = 162; rocblas_gemm_algo_standard = 0
    int product(const void *W_d, const void *X_d, void *C_d, int M, int K, int N) const
    {
        const int32_t alpha = 1, beta = 0;
        return gemm_ex(handle, 112, 111, N, M, K, &alpha, W_d, 160, K, X_d, 160, K, &beta, C_d, 162, N, C_d, 162, N, 162, 0, 0, 0);
    }
    void close()
    {
        if (handle) destroy(handle);
        handle = nullptr;
    }
};

struct Method {
    const char *label;
    sptmm_weights *w;
    std::vector<unsigned char> result;  // device output copied back (int32 or float)
};

}  // namespace

int main(int argc, char **argv)
{
    Flags f;
    parse(argc, argv, f);
    if (f.help) {
        printf("matrix multiply speed check\n"
               "  -row_split3_small <splitK>  SpTMM over u16 index lists (8,16,32,64,128,256)\n"
               "  -row_split_delta2 <splitK>  SpTMM-delta over 8/16-bit gap streams (8,16,32,64)\n"
               "  -i2s                        2-bit packed dense-ternary baseline\n"
               "  -cu_blas                    the dense int8 product of the same matrix through rocBLAS (loaded at run time)\n"
               "  -M -K -N -S -L -iter        shape, nonzeros per column, iterations\n"
               "  -act i8|f16|f32  -seed <n>  -cold <copies>  -nocheck  -nocpu (no host timing)\n"
               "  -cpu_only                   host side only: CPU line and the lists checked against the dense product\n");
        return 0;
    }
    const int M = (int)f.M, K = (int)f.K, N = (int)f.N, S = (int)f.S;
    const int act = f.act == "i8" ? 0 : f.act == "f16" ? 1 : f.act == "f32" ? 2 : -1;
    if (act < 0) strict_fail("act must be i8, f16 or f32");
    if (f.M < 1 || f.M > (1u << 20)) strict_fail("M out of range");

    // host side first (needs no GPU): shape rules of main.cu:85-91 and the seeded ternary matrix
    const bool any = f.row_split3_small || f.row_split_delta2 || f.i2s || f.cu_blas;
    std::vector<uint16_t> pos, neg;
    std::vector<int8_t> dense;
    if (any) {
        pos.resize((size_t)N * (size_t)std::max(S / 2, 0));
        neg.resize(pos.size());
        if ((f.i2s || f.cu_blas || f.cpu_only) && K > 0 && N > 0) dense.resize((size_t)K * N);
        CHECK_SPTMM(sptmm_generate_ternary(K, N, S, dense.empty() ? nullptr : dense.data(), pos.data(), neg.data()));
        if (f.row_split3_small && !sptmm_pack_u16_bytes(N, S, (int)f.row_split3_small)) strict_fail("Wrong split size");
        if (f.row_split_delta2 && !sptmm_pack_delta_bytes(N, S, (int)f.row_split_delta2, 8)) strict_fail("Wrong split size");
    }

    // activations (make_X, main.cu:784-797; seeded here)
    const uint32_t seed = f.seed ? (uint32_t)f.seed : (0xC0FFEEu ^ (uint32_t)M);
    const size_t xcount = (size_t)M * K, esz = act == 0 ? 1 : act == 1 ? 2 : 4;
    std::vector<unsigned char> xhost(xcount * esz);
    if (act == 0) {
        CHECK_SPTMM(sptmm_make_x_i8(seed, xcount, (int8_t *)xhost.data()));
    } else {
        // ~N(0,1), Box-Muller over the same seeded stream
        CHECK_SPTMM(sptmm_make_x_normal(seed, xcount, act == 2 ? (float *)xhost.data() : nullptr, act == 1 ? (uint16_t *)xhost.data() : nullptr));
    }

    // The host's own result: the reference kernel's gather-sum over the lists this process holds (exact int32 for int8
    // rows, double for float rows) -- what every device result below is compared with -- timed on one thread and on
    // every core this process may use.
    const int cores = affinity_cores(), half = S / 2;
    std::vector<int32_t> host_i;
    std::vector<double> host_f;
    auto host_sum = [&](int c0, int c1) {  // columns [c0, c1)
        if (act == 0)
            host_gather_columns((const int8_t *)xhost.data(), M, K, N, half, pos.data(), neg.data(), c0, c1, host_i.data(), [](int8_t v) { return (int)v; });
        else if (act == 1)
            host_gather_columns((const uint16_t *)xhost.data(), M, K, N, half, pos.data(), neg.data(), c0, c1, host_f.data(),
                                [](uint16_t v) { return (double)half_to_float(v); });
        else
            host_gather_columns((const float *)xhost.data(), M, K, N, half, pos.data(), neg.data(), c0, c1, host_f.data(), [](float v) { return (double)v; });
    };
    std::string cpu_line;
    if (any && (f.check || f.cpu || f.cpu_only)) {
        (act == 0 ? host_i.resize((size_t)M * N) : host_f.resize((size_t)M * N));
        over_columns(N, cores, host_sum);
        if (f.cpu || f.cpu_only) {
            // steady clock, 3 warm-ups, median and minimum of up to 50 repetitions (at least 3; about a second per thread
            // count), columns split statically over threads that live for the whole loop
            auto time_it = [&](int threads, double *median, double *best, int *reps) {
                std::vector<double> t = timed_over_columns(N, threads, 50, 1.0, host_sum);
                std::sort(t.begin(), t.end());
                *median = t[t.size() / 2], *best = t[0], *reps = (int)t.size();
            };
            double med_n = 0, min_n = 0, med_1 = 0, min_1 = 0;
            int reps_n = 0, reps_1 = 0;
            time_it(cores, &med_n, &min_n, &reps_n);
            time_it(1, &med_1, &min_1, &reps_1);
            const double bytes = 2.0 * S * N + (double)M * K * esz + 4.0 * M * N;
            char buf[512];
            snprintf(buf, sizeof buf,
                     "# cpu: us/call threads=%d median=%.1f min=%.1f reps=%d (%.1f GB/s); threads=1 median=%.1f min=%.1f reps=%d (host "
                     "gather-sum over the u16 lists, main.cu:577-593)",
                     cores, med_n, min_n, reps_n, bytes / med_n / 1e3, med_1, min_1, reps_1);
            cpu_line = buf;
        }
    }

    auto banner = [&] {
        std::cout << "make_X done" << std::endl;
        printf("Compiled on %s at %s\n", __DATE__, __TIME__);
        std::cout << "Start: "
                  << "M=" << f.M << " K=" << f.K << " N=" << f.N << " ITER=" << f.iter << " S=" << f.S << " ("
                  << (100.0 - 100.0 * ((float)f.S / (float)f.K)) << "% Sparsity)"
                  << " L=" << f.L << " B=" << 8 << " X_MAJOR=ROW W_MAJOR=COL C_MAJOR=ROW" << std::endl;
    };
    if (f.cpu_only) {
        // no device: the CPU line, and the lists' gather-sum against the dense product of the same matrix
        banner();
        if (!any) strict_fail("cpu_only needs a method (-row_split3_small, -row_split_delta2 or -i2s)");
        bool pass;
        double worst = 0;
        if (act == 0) {
            std::vector<int32_t> d((size_t)M * N);
            host_dense_product((const int8_t *)xhost.data(), M, K, N, dense.data(), cores, d.data(), [](int8_t v) { return (int)v; });
            pass = d == host_i;
        } else {
            std::vector<double> d((size_t)M * N);
            if (act == 1)
                host_dense_product((const uint16_t *)xhost.data(), M, K, N, dense.data(), cores, d.data(), [](uint16_t v) { return (double)half_to_float(v); });
            else
                host_dense_product((const float *)xhost.data(), M, K, N, dense.data(), cores, d.data(), [](float v) { return (double)v; });
            for (size_t j = 0; j < d.size(); ++j)
                worst = std::max(worst, std::fabs(d[j] - host_f[j]) / std::max(std::fabs(d[j]), std::sqrt((double)S)));
            pass = worst <= 1e-9;
        }
        printf("%s\n", cpu_line.c_str());
        printf("# check=%s (host gather-sum == host dense product; no device used)\n", pass ? "PASS" : "FAIL");
        return pass ? 0 : 2;
    }

    sptmm_devinfo dev;
    CHECK_SPTMM(sptmm_device_init(0, &dev));
    void *x_d = nullptr, *c_d = nullptr, *stream = nullptr;
    CHECK_SPTMM(sptmm_malloc(&x_d, xhost.size()));
    CHECK_SPTMM(sptmm_memcpy_h2d(x_d, xhost.data(), xhost.size()));
    CHECK_SPTMM(sptmm_malloc(&c_d, sizeof(int) * (size_t)M * N));
    CHECK_SPTMM(sptmm_memset(c_d, 0, sizeof(int) * (size_t)M * N));
    CHECK_SPTMM(sptmm_stream_create(&stream));
    banner();

    std::vector<Method> done;
    if (f.cu_blas) {
        // first of the methods, as at main.cu:841
        if (act != 0) strict_fail("cu_blas takes int8 activations");
        DenseBlas blas;
        std::string why;
        if (!blas.open(stream, &why)) {
            fprintf(stderr, "%s\n", why.c_str());
            exit(EXIT_FAILURE);
        }
        void *w_d = nullptr, *e0 = nullptr, *e1 = nullptr;
        CHECK_SPTMM(sptmm_malloc(&w_d, dense.size()));
        CHECK_SPTMM(sptmm_memcpy_h2d(w_d, dense.data(), dense.size()));
        CHECK_SPTMM(sptmm_event_create(&e0));
        CHECK_SPTMM(sptmm_event_create(&e1));
        auto call = [&] {
            if (int rc = blas.product(w_d, x_d, c_d, M, K, N)) {
                fprintf(stderr, "rocblas_gemm_ex: status %d (int8 x int8 -> int32, m=%d n=%d k=%d)\n", rc, N, M, K);
                exit(EXIT_FAILURE);
            }
        };
        CHECK_SPTMM(sptmm_memset(c_d, 0xff, sizeof(int) * (size_t)M * N));
        for (int i = 0; i < 3; ++i) call();  // (the first call loads the library's kernels)
        CHECK_SPTMM(sptmm_stream_sync(stream));
        Method m{"cu_blas", nullptr, std::vector<unsigned char>(sizeof(int) * (size_t)M * N)};
        CHECK_SPTMM(sptmm_memcpy_d2h(m.result.data(), c_d, m.result.size()));
        const int iters = (int)std::max<uint32_t>(f.iter, 1);
        double us_sync = 0, us_b2b = 0;
        // reference protocol: call + synchronize per iteration (main.cu:852-869)
        CHECK_SPTMM(sptmm_event_record(e0, stream));
        for (int i = 0; i < iters; ++i) {
            call();
            CHECK_SPTMM(sptmm_stream_sync(stream));
        }
        CHECK_SPTMM(sptmm_event_record(e1, stream));
        CHECK_SPTMM(sptmm_event_sync(e1));
        CHECK_SPTMM(sptmm_event_elapsed_us(e0, e1, &us_sync));
        // (printf: libraries loaded at run time may have changed std::cout's precision; %g is what the stream prints by default)
        printf("%g\n", (double)(float)(us_sync / iters / 1000.0));
        fflush(stdout);
        CHECK_SPTMM(sptmm_event_record(e0, stream));
        for (int i = 0; i < iters; ++i) call();
        CHECK_SPTMM(sptmm_event_record(e1, stream));
        CHECK_SPTMM(sptmm_event_sync(e1));
        CHECK_SPTMM(sptmm_event_elapsed_us(e0, e1, &us_b2b));
        const double bytes = (double)K * N + (double)M * K + 4.0 * M * N;
        printf("# cu_blas: us/call sync_each=%.3f back_to_back=%.3f (%.1f GB/s, %.1f%% of %.0f) bytes=%.0f rocBLAS int8 x int8 -> int32, dense\n",
               us_sync / iters, us_b2b / iters, bytes / (us_b2b / iters) / 1e3, bytes / (us_b2b / iters) / 1e3 / dev.peak_hbm_gbps * 100.0,
               dev.peak_hbm_gbps, bytes);
        done.push_back(std::move(m));
        blas.close();
        sptmm_event_destroy(e0);
        sptmm_event_destroy(e1);
        sptmm_free(w_d);
    }

    auto run = [&](const char *label, sptmm_weights *w, bool timed) {
        sptmm_winfo wi;
        CHECK_SPTMM(sptmm_weights_info(w, &wi));
        const int a = wi.kind == SPTMM_KIND_I2S ? 0 : act;
        if (wi.kind == SPTMM_KIND_I2S && act != 0) strict_fail("i2s takes int8 activations");
        // one checked call first
        CHECK_SPTMM(sptmm_memset(c_d, 0xff, sizeof(int) * (size_t)M * N));
        if (a == 0)
            CHECK_SPTMM(sptmm_gemv_i8(w, (const int8_t *)x_d, M, (int32_t *)c_d, stream));
        else if (a == 1)
            CHECK_SPTMM(sptmm_gemv_f16(w, (const uint16_t *)x_d, M, (float *)c_d, stream));
        else
            CHECK_SPTMM(sptmm_gemv_f32(w, (const float *)x_d, M, (float *)c_d, stream));
        CHECK_SPTMM(sptmm_stream_sync(stream));
        Method m{label, w, std::vector<unsigned char>(sizeof(int) * (size_t)M * N)};
        CHECK_SPTMM(sptmm_memcpy_d2h(m.result.data(), c_d, m.result.size()));
        if (timed) {
            const int iters = (int)std::max<uint32_t>(f.iter, 1);
            double us_sync = 0, us_b2b = 0, us_cold = 0;
            const sptmm_weights *one[1] = {w};
            // reference protocol: launch + synchronize per iteration (main.cu:1456)
            CHECK_SPTMM(sptmm_measure_gemv(one, 1, a, x_d, M, c_d, iters, 1, stream, &us_sync));
            printf("%g\n", (double)(float)(us_sync / 1000.0));
            fflush(stdout);
            const int warm = std::min(iters, 200);
            CHECK_SPTMM(sptmm_measure_gemv(one, 1, a, x_d, M, c_d, warm, 0, stream, &us_b2b));
            CHECK_SPTMM(sptmm_measure_gemv(one, 1, a, x_d, M, c_d, iters, 0, stream, &us_b2b));
            const double bytes = (double)wi.stream_bytes + (double)M * K * esz + 4.0 * M * N;
            printf("# %s: us/call sync_each=%.3f back_to_back=%.3f (%.1f GB/s, %.1f%% of %.0f)", label, us_sync, us_b2b,
                   bytes / us_b2b / 1e3, bytes / us_b2b / 1e3 / dev.peak_hbm_gbps * 100.0, dev.peak_hbm_gbps);
            if (f.cold > 1) {
                std::vector<sptmm_weights *> copies{w};
                for (uint64_t i = 1; i < f.cold; ++i) {
                    sptmm_weights *c = nullptr;
                    CHECK_SPTMM(sptmm_weights_clone(w, &c));
                    copies.push_back(c);
                }
                std::vector<const sptmm_weights *> cc(copies.begin(), copies.end());
                CHECK_SPTMM(sptmm_measure_gemv(cc.data(), (int)cc.size(), a, x_d, M, c_d, (int)cc.size() * 2, 0, stream, &us_cold));
                CHECK_SPTMM(sptmm_measure_gemv(cc.data(), (int)cc.size(), a, x_d, M, c_d, iters, 0, stream, &us_cold));
                printf(" cold[%d copies]=%.3f (%.1f GB/s, %.1f%%)", (int)cc.size(), us_cold, bytes / us_cold / 1e3,
                       bytes / us_cold / 1e3 / dev.peak_hbm_gbps * 100.0);
                if (a == 0) {
                    // the same copies, up to 32 GEMVs per launch (sptmm_gemv_i8_batched)
                    const int nb = (int)std::min<size_t>(cc.size(), 32);
                    void *cb = nullptr;
                    double us_bat = 0;
                    CHECK_SPTMM(sptmm_malloc(&cb, sizeof(int) * (size_t)M * N * nb));
                    CHECK_SPTMM(sptmm_measure_gemv(cc.data(), nb, 0, x_d, M, cb, 2 * nb, 3, stream, &us_bat));
                    CHECK_SPTMM(sptmm_measure_gemv(cc.data(), nb, 0, x_d, M, cb, std::max(iters, nb), 3, stream, &us_bat));
                    CHECK_SPTMM(sptmm_free(cb));
                    printf(" batched[%d per launch]=%.3f (%.1f GB/s, %.1f%%)", nb, us_bat, bytes / us_bat / 1e3,
                           bytes / us_bat / 1e3 / dev.peak_hbm_gbps * 100.0);
                }
                for (size_t i = 1; i < copies.size(); ++i) sptmm_weights_free(copies[i]);
            }
            printf(" bytes=%.0f kind=%d split_k=%d delta_bits=%d\n", bytes, wi.kind, wi.split_k, wi.delta_bits);
        }
        done.push_back(std::move(m));
    };

    if (f.row_split3_small > 0) {
        sptmm_weights *w = nullptr;
        CHECK_SPTMM(sptmm_weights_upload_u16(pos.data(), neg.data(), K, N, S, (int)f.row_split3_small, &w));
        run("sptmm", w, true);
    }
    if (f.row_split_delta2 > 0) {
        sptmm_weights *w = nullptr;
        // the gap stream is packed for the number of activation rows of this run (M = 1 with int8 rows: the GEMV stream)
        CHECK_SPTMM(sptmm_weights_upload_delta_rows(pos.data(), neg.data(), K, N, S, (int)f.row_split_delta2, act == 0 ? M : 0, &w));
        run("sptmm-delta", w, true);
    }
    if (f.i2s) {
        sptmm_weights *w = nullptr;
        CHECK_SPTMM(sptmm_weights_upload_i2s(dense.data(), K, N, &w));
        run("i2s", w, true);
    }

    int status = 0;
    if (!cpu_line.empty()) printf("%s\n", cpu_line.c_str());
    if (any && f.check) {
        // every method's device output against the host gather-sum: bit-exact for int8 rows, within 1e-3 of
        // max(|ref|, sqrt(S)) for float rows (fp32 sums on the device, double on the host)
        bool pass = !done.empty();
        double worst = 0;
        for (const Method &m : done) {
            if (act == 0) {
                pass &= memcmp(m.result.data(), host_i.data(), m.result.size()) == 0;
            } else {
                const float *g = (const float *)m.result.data();
                for (size_t j = 0; j < (size_t)M * N; ++j) {
                    const double scale = std::max<double>(std::fabs(host_f[j]), std::sqrt((double)S));
                    worst = std::max(worst, std::fabs((double)g[j] - host_f[j]) / scale);
                }
                pass &= worst <= 1e-3;
            }
        }
        printf("# check=%s (", pass ? "PASS" : "FAIL");
        for (size_t i = 0; i < done.size(); ++i) printf("%s%s %s host", i ? "; " : "", done[i].label, act == 0 ? "==" : "~");
        if (act != 0) printf("; max rel diff %.2e", worst);
        printf(")\n");
        if (!pass) status = 2;
    }
    for (auto &m : done) sptmm_weights_free(m.w);
    sptmm_stream_destroy(stream);
    sptmm_free(x_d);
    sptmm_free(c_d);
    return status;
}
