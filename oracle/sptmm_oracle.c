/*
 * sptmm_oracle.c -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, single-purpose CPU restatement of the reference benchmark's
 * arithmetic (Ogiwara-CostlierRain464/SpTMM).  It exists so that the tests, the
 * smoke check and the CPU-baseline leg of the benchmark have something
 * independent to compare the HIP path against.  Nothing in the shipped library
 * or the bench driver links, loads or calls this file.
 *
 * Every function names the reference lines it restates.  The reference holds
 * no golden vectors and never reads a result back, so the functions are pinned
 * from outside instead (see tests/test_oracle.py):
 *   - orc_xorshift32      : published Marsaglia 13/17/5 sequence for seed 1
 *   - orc_gen_column      : independent numpy restatement + swap KATs + invariants
 *   - list/layout/delta   : closed-form bijection / cumsum identities
 *   - orc_sptmm_*, i2s    : brute-force dense int64 matmul in numpy
 * Parity status: no function here is "parity unpinned".
 *
 * Conventions: W is K x N, stored column-major (reference "rcr" build:
 * W_MAJOR = MAJOR_COL, macro.cuh:58), X is M x K row-major, C is M x N
 * row-major.  Index lists are [N][S/2] with the column's entries contiguous.
 */
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* macro.cuh:69-76 -- Marsaglia xorshift, shifts 13 / 17 / 5, 32-bit state. */
uint32_t orc_xorshift32(uint32_t *state)
{
    uint32_t v = *state;
    v ^= v << 13;
    v ^= v >> 17;
    v ^= v << 5;
    *state = v;
    return v;
}

/*
 * main.cu:246-265 -- one ternary column.  Rows [0,S/2) start as -1, rows
 * [S/2,S) as +1, the rest 0; then a descending Fisher-Yates pass
 * (i = K-1 .. 1, j = rng % (i+1) with unsigned arithmetic, swap even if i==j)
 * seeded with 0xCAFEBABE ^ col.
 */
void orc_gen_column(int K, int S, uint32_t col, int8_t *w)
{
    int half = S / 2;
    memset(w, 0, (size_t)K);
    for (int r = 0; r < half; ++r) w[r] = -1;
    for (int r = half; r < S; ++r) w[r] = 1;
    uint32_t st = 0xCAFEBABEu ^ col;
    for (int i = K - 1; i > 0; --i) {
        uint32_t j = orc_xorshift32(&st) % (uint32_t)(i + 1);
        int8_t t = w[i];
        w[i] = w[j];
        w[j] = t;
    }
}

/*
 * main.cu:267-276 -- ascending row lists of the +1 and the -1 entries of one
 * column.  Returns 0 when both lists hold exactly S/2 entries (the
 * reference's "W matrix corrupt" assert), 1 otherwise.
 */
int orc_lists_from_column(const int8_t *w, int K, int half, uint16_t *pos, uint16_t *neg)
{
    int np = 0, nn = 0;
    for (int r = 0; r < K; ++r) {
        if (w[r] == 1) {
            if (np < half) pos[np] = (uint16_t)r;
            ++np;
        } else if (w[r] == -1) {
            if (nn < half) neg[nn] = (uint16_t)r;
            ++nn;
        }
    }
    return !(np == half && nn == half);
}

/*
 * main.cu:246-276 for all N columns.  W (column-major, K*N bytes) may be NULL
 * when only the lists are wanted.  Returns the number of corrupt columns (0).
 */
int orc_generate(int K, int N, int S, int8_t *W, uint16_t *pos, uint16_t *neg)
{
    int half = S / 2, bad = 0;
    int8_t *tmp = (int8_t *)malloc((size_t)K);
    for (int c = 0; c < N; ++c) {
        int8_t *w = W ? W + (size_t)c * K : tmp;
        orc_gen_column(K, S, (uint32_t)c, w);
        bad += orc_lists_from_column(w, K, half, pos + (size_t)c * half, neg + (size_t)c * half);
    }
    free(tmp);
    return bad;
}

/*
 * main.cu:343-374 -- the "P_div" re-layout, P in {8,16,32}: a pure
 * permutation out[chunk][col][lane] = list[col][chunk*P + lane], i.e. flat
 * offset chunk*(P*N) + col*P + lane.  Needs half % P == 0.
 */
void orc_split_layout(const uint16_t *list, int N, int half, int P, uint16_t *out)
{
    int chunks = half / P;
    for (int ch = 0; ch < chunks; ++ch)
        for (int c = 0; c < N; ++c)
            for (int l = 0; l < P; ++l)
                out[(size_t)ch * P * N + (size_t)c * P + l] = list[(size_t)c * half + ch * P + l];
}

/*
 * main.cu:376-394 -- gaps of a sorted list, first entry absolute, narrowed to
 * one byte exactly as the reference does (a gap above 255 wraps).  Returns how
 * many entries did not fit, so callers can tell when the reference's format
 * would have been silently wrong.
 */
int orc_delta8(const uint16_t *list, int N, int half, uint8_t *d)
{
    int wrapped = 0;
    for (int c = 0; c < N; ++c) {
        const uint16_t *l = list + (size_t)c * half;
        uint8_t *o = d + (size_t)c * half;
        for (int i = 0; i < half; ++i) {
            unsigned g = i ? (unsigned)(l[i] - l[i - 1]) : l[0];
            if (g > 255u) ++wrapped;
            o[i] = (uint8_t)g;
        }
    }
    return wrapped;
}

/* Same gaps kept at 16 bits (what a correct encoder falls back to). */
void orc_delta16(const uint16_t *list, int N, int half, uint16_t *d)
{
    for (int c = 0; c < N; ++c)
        for (int i = 0; i < half; ++i) {
            const uint16_t *l = list + (size_t)c * half;
            d[(size_t)c * half + i] = (uint16_t)(i ? l[i] - l[i - 1] : l[0]);
        }
}

/*
 * main.cu:400-413 -- "div256" layout of a delta stream:
 * out[chunk][col][r] = d[col][chunk*256 + r] for chunk*256 + r < half; the
 * tail of the last chunk is left untouched (callers pre-zero it).
 */
void orc_delta_div256(const uint8_t *d, int N, int half, uint8_t *out)
{
    int chunks = (half + 255) / 256;
    for (int ch = 0; ch < chunks; ++ch)
        for (int c = 0; c < N; ++c)
            for (int r = 0; r < 256; ++r) {
                int src = ch * 256 + r;
                if (src < half) out[((size_t)ch * N + c) * 256 + r] = d[(size_t)c * half + src];
            }
}

/*
 * main.cu:577-593 -- the SpTMM sum itself on the plain lists:
 * C[m][col] = sum_i X[m][pos[col][i]] - sum_i X[m][neg[col][i]], int32.
 */
void orc_sptmm_i8(const int8_t *X, int M, int K, const uint16_t *pos, const uint16_t *neg, int N,
                  int half, int32_t *C)
{
    for (int m = 0; m < M; ++m) {
        const int8_t *x = X + (size_t)m * K;
        for (int c = 0; c < N; ++c) {
            const uint16_t *p = pos + (size_t)c * half, *q = neg + (size_t)c * half;
            int32_t acc = 0;
            for (int i = 0; i < half; ++i) acc += x[p[i]] - x[q[i]];
            C[(size_t)m * N + c] = acc;
        }
    }
}

/*
 * main.cu:556-594 walked the way the kernel walks it: one block per
 * 32/SPLIT columns, lane = ty*SPLIT + tx, each lane strides the P_div layout
 * by SPLIT*N from offset 32*block + lane, partials folded with the
 * shuffle-down tree (width SPLIT), lane tx==0 stores.  Checks the layout and
 * the kernel's indexing together.
 */
void orc_sptmm_split_i8(const int8_t *X, int M, int K, const uint16_t *pos_div, const uint16_t *neg_div,
                        int N, int half, int split, int32_t *C)
{
    int cols_per_warp = 32 / split;
    int blocks = N / cols_per_warp;
    for (int m = 0; m < M; ++m) {
        const int8_t *x = X + (size_t)m * K;
        for (int b = 0; b < blocks; ++b) {
            int32_t part[32];
            for (int lane = 0; lane < 32; ++lane) {
                int32_t acc = 0;
                size_t end = (size_t)(half / split) * split * N;
                for (size_t i = (size_t)lane; i < end; i += (size_t)split * N) {
                    acc += x[pos_div[(size_t)32 * b + i]];
                    acc -= x[neg_div[(size_t)32 * b + i]];
                }
                part[lane] = acc;
            }
            for (int off = split / 2; off > 0; off /= 2)
                for (int lane = 0; lane < 32; ++lane) {
                    int tx = lane % split;
                    if (tx + off < split) part[lane] += part[lane + off];
                    /* lanes beyond the segment keep their own value (shfl_down semantics) */
                }
            for (int ty = 0; ty < cols_per_warp; ++ty)
                C[(size_t)m * N + b * cols_per_warp + ty] = part[ty * split];
        }
    }
}

/*
 * main.cu:644-675 (and 728-762 for the ragged tail) -- SpTMM-delta read from
 * the div256 layout: per column, 256-byte chunks at offset 256*col +
 * chunk*256*N; inside a chunk eight groups of 32 consecutive gaps get an
 * inclusive prefix sum carried in 16-bit arithmetic, plus the running carry
 * of the previous group's last lane; the resulting row index gathers X.
 */
void orc_sptmm_delta_i8(const int8_t *X, int M, int K, const uint8_t *dpos256, const uint8_t *dneg256,
                        int N, int half, int32_t *C)
{
    int chunks = (half + 255) / 256;
    for (int m = 0; m < M; ++m) {
        const int8_t *x = X + (size_t)m * K;
        for (int c = 0; c < N; ++c) {
            uint16_t carry_p = 0, carry_n = 0;
            int32_t acc = 0;
            for (int ch = 0; ch < chunks; ++ch) {
                const uint8_t *bp = dpos256 + (size_t)256 * c + (size_t)ch * 256 * N;
                const uint8_t *bn = dneg256 + (size_t)256 * c + (size_t)ch * 256 * N;
                for (int g = 0; g < 256; g += 32) {
                    uint16_t run_p = 0, run_n = 0, last_p = carry_p, last_n = carry_n;
                    for (int lane = 0; lane < 32; ++lane) {
                        int e = ch * 256 + g + lane;
                        if (e >= half) break;
                        run_p = (uint16_t)(run_p + bp[g + lane]);
                        run_n = (uint16_t)(run_n + bn[g + lane]);
                        uint16_t ip = (uint16_t)(run_p + carry_p), in = (uint16_t)(run_n + carry_n);
                        acc += x[ip];
                        acc -= x[in];
                        last_p = ip;
                        last_n = in;
                    }
                    carry_p = last_p;
                    carry_n = last_n;
                }
            }
            C[(size_t)m * N + c] = acc;
        }
    }
}

/*
 * main.cu:176-192 -- one i2s word: 16 ternary weights w[e] in {-1,0,1}, code =
 * w + 2, element e placed at bit 8*(e%4) + 2*(e/4).
 */
uint32_t orc_i2s_pack_word(const int8_t *w16)
{
    uint32_t word = 0;
    for (int e = 0; e < 16; ++e) {
        uint32_t code = (uint32_t)(w16[e] + 2) & 3u;
        word |= code << (8 * (e % 4) + 2 * (e / 4));
    }
    return word;
}

/*
 * bitnet_kernels.cuh:52-72 -- decode: for i in 0..3 the four bytes of
 * (word >> 2i) & 0x03030303 are codes of elements 4i..4i+3; subtract 2.
 */
void orc_i2s_decode_word(uint32_t word, int8_t *w16)
{
    for (int i = 0; i < 4; ++i) {
        uint32_t t = (word >> (2 * i)) & 0x03030303u;
        for (int b = 0; b < 4; ++b) w16[4 * i + b] = (int8_t)((int)((t >> (8 * b)) & 0xffu) - 2);
    }
}

/*
 * main.cu:194-196 -- plain packed order: the word for rows 16g..16g+15 of
 * column col sits at word index col*(K/16) + g.  (The reference fills every g
 * with one placeholder word; here the real matrix is packed.)
 */
void orc_i2s_pack(const int8_t *W, int K, int N, uint32_t *out)
{
    int words = K / 16;
    for (int c = 0; c < N; ++c)
        for (int g = 0; g < words; ++g) out[(size_t)c * words + g] = orc_i2s_pack_word(W + (size_t)c * K + 16 * g);
}

/*
 * bitnet_kernels.cuh:86-110 -- decode + 4 x dp4a per word, int32 accumulate,
 * C row stride N (the reference's stride K at line 108 is its bug, not a
 * contract).  Reads the plain packed order above.
 */
void orc_i2s_gemv(const int8_t *X, int M, int K, const uint32_t *packed, int N, int32_t *C)
{
    int words = K / 16;
    for (int m = 0; m < M; ++m)
        for (int c = 0; c < N; ++c) {
            int32_t acc = 0;
            for (int g = 0; g < words; ++g) {
                int8_t w16[16];
                orc_i2s_decode_word(packed[(size_t)c * words + g], w16);
                const int8_t *x = X + (size_t)m * K + 16 * g;
                for (int e = 0; e < 16; ++e) acc += (int32_t)x[e] * w16[e];
            }
            C[(size_t)m * N + c] = acc;
        }
}

/* Brute force C = X * W on the dense column-major matrix (textbook matmul). */
void orc_dense_i8(const int8_t *X, int M, int K, const int8_t *W, int N, int32_t *C)
{
    for (int m = 0; m < M; ++m)
        for (int c = 0; c < N; ++c) {
            int32_t acc = 0;
            const int8_t *x = X + (size_t)m * K, *w = W + (size_t)c * K;
            for (int r = 0; r < K; ++r) acc += (int32_t)x[r] * w[r];
            C[(size_t)m * N + c] = acc;
        }
}

/*
 * Seeded int8 activations, uniform on [-127,127]: xorshift32 stream seeded
 * with `seed`, value = r % 255 - 127.  (The reference's make_X, main.cu:784-797,
 * is unseeded; the benchmark definition asks for a seeded uniform draw.)
 */
void orc_make_x_i8(uint32_t seed, size_t n, int8_t *X)
{
    uint32_t st = seed ? seed : 1u;
    for (size_t i = 0; i < n; ++i) X[i] = (int8_t)((int)(orc_xorshift32(&st) % 255u) - 127);
}

/* ---- multi-threaded gather-sum: the CPU baseline the benchmark reports ---- */
typedef struct {
    const int8_t *X;
    const uint16_t *pos, *neg;
    int32_t *C;
    int M, K, N, half, c0, c1;
} orc_job;

static void *orc_worker(void *arg)
{
    orc_job *j = (orc_job *)arg;
    for (int m = 0; m < j->M; ++m) {
        const int8_t *x = j->X + (size_t)m * j->K;
        for (int c = j->c0; c < j->c1; ++c) {
            const uint16_t *p = j->pos + (size_t)c * j->half, *q = j->neg + (size_t)c * j->half;
            int32_t acc = 0;
            for (int i = 0; i < j->half; ++i) acc += x[p[i]] - x[q[i]];
            j->C[(size_t)m * j->N + c] = acc;
        }
    }
    return NULL;
}

/* main.cu:577-593 semantics, columns statically split over `threads` pthreads. */
void orc_sptmm_i8_mt(const int8_t *X, int M, int K, const uint16_t *pos, const uint16_t *neg, int N,
                     int half, int32_t *C, int threads)
{
    if (threads < 1) threads = 1;
    if (threads > 256) threads = 256;
    pthread_t tid[256];
    orc_job job[256];
    for (int t = 0; t < threads; ++t) {
        job[t] = (orc_job){X, pos, neg, C, M, K, N, half, (int)((long)N * t / threads),
                           (int)((long)N * (t + 1) / threads)};
        pthread_create(&tid[t], NULL, orc_worker, &job[t]);
    }
    for (int t = 0; t < threads; ++t) pthread_join(tid[t], NULL);
}
