// Host-side stress of libsptmm's launch paths against the HIP stand-in (hipstub.cpp): every stream kind through
// every protocol of sptmm_measure_gemv and sptmm_measure_sequence, `launches` launches per loop (argv[1]), from one
// thread and then from four at once.  Nothing here grows with the number of launches issued: the process must end
// with status 0 however many are queued (and, built with -fsanitize=address,undefined, without a report).
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>

#include "../../include/sptmm.h"

extern "C" long hipstub_launches();

#define OK(x)                                                                  \
    do {                                                                       \
        int rc_ = (x);                                                         \
        if (rc_) {                                                             \
            fprintf(stderr, "%s -> %d %s\n", #x, rc_, sptmm_last_error());    \
            exit(1);                                                           \
        }                                                                      \
    } while (0)

static void hammer(int K, int N, int S, int split, int launches)
{
    std::vector<uint16_t> pos((size_t)N * S / 2), neg(pos.size());
    std::vector<int8_t> W((size_t)K * N);
    OK(sptmm_generate_ternary(K, N, S, W.data(), pos.data(), neg.data()));
    sptmm_weights *u = nullptr, *d = nullptr, *i2 = nullptr, *rag = nullptr, *wide = nullptr;
    OK(sptmm_weights_upload_u16(pos.data(), neg.data(), K, N, S, split, &u));
    OK(sptmm_weights_upload_delta_rows(pos.data(), neg.data(), K, N, S, split, 1, &d));
    OK(sptmm_weights_upload_i2s(W.data(), K, N, &i2));
    OK(sptmm_weights_upload_dense(W.data(), K, N, SPTMM_KIND_U16, split, &rag));
    OK(sptmm_weights_upload_wide(W.data(), K, N, SPTMM_KIND_DELTA, 32, &wide));
    void *x = nullptr, *c = nullptr, *st = nullptr;
    OK(sptmm_malloc(&x, (size_t)16 * K * 4));
    OK(sptmm_malloc(&c, (size_t)4 * 16 * N * 40));
    OK(sptmm_stream_create(&st));
    for (sptmm_weights *w : {u, d, i2, rag, wide}) {
        std::vector<const sptmm_weights *> ws;
        std::vector<sptmm_weights *> owned;
        ws.push_back(w);
        for (int i = 1; i < 40; ++i) {
            sptmm_weights *cl = nullptr;
            OK(sptmm_weights_clone(w, &cl));
            owned.push_back(cl);
            ws.push_back(cl);
        }
        double us = 0;
        for (int m : {1, 4, 8, 16})
            for (int mode : {0, 1, 2, 3, 4}) {
                const int n_ws = mode == 3 ? (m == 1 ? 40 : 32) : 40;
                OK(sptmm_measure_gemv(ws.data(), n_ws, 0, x, m, c, launches, mode, st, &us));
            }
        if (w == u || w == d || w == rag) {
            OK(sptmm_measure_gemv(ws.data(), 8, 1, x, 4, c, launches / 4, 3, st, &us));
            OK(sptmm_measure_gemv(ws.data(), 8, 2, x, 4, c, launches / 4, 0, st, &us));
            OK(sptmm_measure_gemv(ws.data(), 8, 3, x, 4, c, launches / 4, 0, st, &us));
        }
        if (w == u || w == d || w == rag) {
            // the quantising GEMV: fused, with a workspace of the caller's, on the library's static device array
            void *ws = nullptr;
            const size_t ws_bytes = sptmm_gemv_q8_workspace_bytes(w, 16);
            OK(sptmm_malloc(&ws, ws_bytes));
            for (int i = 0; i < launches / 8; ++i) {
                const int m = 1 + i % 16;
                OK(sptmm_gemv_q8(w, (const uint16_t *)x, SPTMM_X_F16, m, 0.5f, (float *)c, st));
                OK(sptmm_gemv_q8_ws(w, (const uint16_t *)x, SPTMM_X_BF16, m, 0.5f, (float *)c, ws, ws_bytes, st));
                OK(sptmm_gemv_q8_static(w, (const uint16_t *)x, SPTMM_X_F16, m, 0.5f, (float *)c, st));
            }
            OK(sptmm_free(ws));
        }
        std::vector<sptmm_step> steps;
        for (int i = 0; i < 28; ++i) steps.push_back(sptmm_step{ws[i], x, c, 1 + i % 4 * 5, 0, i / 3});
        for (int mode = 0; mode <= 4; ++mode) OK(sptmm_measure_sequence(steps.data(), (int)steps.size(), launches / 28, mode, st, &us));
        for (sptmm_weights *o : owned) sptmm_weights_free(o);
    }
    for (sptmm_weights *w : {u, d, i2, rag, wide}) sptmm_weights_free(w);
    OK(sptmm_stream_destroy(st));
    OK(sptmm_free(x));
    OK(sptmm_free(c));
}

int main(int argc, char **argv)
{
    const int launches = argc > 1 ? atoi(argv[1]) : 20000;
    sptmm_devinfo info;
    OK(sptmm_device_init(0, &info));
    hammer(6912, 2560, 4096, 32, launches);
    hammer(2560, 640, 1536, 32, launches);
    printf("single thread: %ld launches\n", hipstub_launches());
    std::vector<std::thread> th;
    for (int t = 0; t < 4; ++t) th.emplace_back([=] { hammer(512 + 256 * t, 64 + 16 * t, 128, 16, launches / 2); });
    for (auto &t : th) t.join();
    printf("four threads: %ld launches in all\n", hipstub_launches());
    return 0;
}
