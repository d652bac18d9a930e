/*
 * CPU oracle for the tile-kernel path: a plain C restatement of the arithmetic
 * the reference's kernels perform.  TEST INFRASTRUCTURE ONLY: it is the checker
 * for the HIP kernels and the timed CPU baseline; nothing shipped routes
 * through it.
 *
 * What each function follows in the reference (paths relative to the reference
 * root):
 *   oracle_gemm_f16        include/cell/compute/gemm.hpp:42-52 (C(i,j) += A(i,k)·B(k,j),
 *                          f16 operands, f32 accumulate) and the host check
 *                          tests/cpp/cell/test_single_wmma.cu:16-29 (naive_gemm).
 *                          A row-major [M,K], B column-major [K,N] (= Bᵀ stored [N,K]).
 *   oracle_b2b_gemm_f16    examples/cpp/02_fused_two_gemms/fused_gemm.hpp:152-175
 *                          (acc = A·B; acc rounded to f16; D = acc·C) with the operand
 *                          layouts of examples/cpp/02_fused_two_gemms/util.hpp:20-28
 *                          (A, D row-major; B, C column-major).
 *   oracle_attention_f16   softmax(scale·Q·K)·V, the function computed blockwise by
 *                          src/kernels/flash_attn.cu:237-306; K is column-major [K,N]
 *                          (= [N,K] row-major), V is column-major [N,P] (the reference
 *                          boundary, pytiledcuda/__init__.py:17-30) or row-major [N,P].
 *   oracle_attention_blocked_f32
 *                          the block-wise online-softmax recurrence of
 *                          tests/python/test_flash_attn.py:27-75 restated (running max
 *                          starts at 0, no scale unless given), in f32.
 *   oracle_lstm_f16        no counterpart in the reference snapshot (only Makefile:3 names
 *                          a test_lstm_cell); standard LSTM cell, gate order i,f,g,o over
 *                          concat(x_t, h_{t-1}).  PARITY UNPINNED by the reference; pinned
 *                          by closed forms in tests/test_oracle.py.
 *   oracle_fill_uniform / oracle_fill_normal
 *                          seeded input generation (the reference uses unseeded rand(),
 *                          tests/cpp/cell/test_gemm.cu:16-21); a counter-based splitmix64
 *                          stream so every consumer sees identical bits.
 *
 * Pinning: tests/test_oracle.py checks every function against closed forms, brute
 * force on tiny inputs, numpy float64 restatements and invariants (see that file).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---------- fp16 <-> fp32, bit exact, round-to-nearest-even ---------- */
static inline float h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t f;
    if (exp == 0) {
        if (man == 0) {
            f = sign;
        } else { /* subnormal */
            int e = -1;
            do { man <<= 1; ++e; } while (!(man & 0x400u));
            man &= 0x3ffu;
            f = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        f = sign | 0x7f800000u | (man << 13);
    } else {
        f = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float out;
    memcpy(&out, &f, 4);
    return out;
}

static inline uint16_t f2h(float x) {
    uint32_t f;
    memcpy(&f, &x, 4);
    uint32_t sign = (f >> 16) & 0x8000u;
    uint32_t fexp = (f >> 23) & 0xffu;
    uint32_t man = f & 0x7fffffu;
    if (fexp == 255) return (uint16_t)(sign | 0x7c00u | (man ? 0x200u : 0));
    int e = (int)fexp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        int shift = 14 - e;
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1))) ++half_man;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half_man = man >> 13;
    uint32_t rem = man & 0x1fffu;
    uint16_t h = (uint16_t)(sign | ((uint32_t)e << 10) | half_man);
    if (rem > 0x1000u || (rem == 0x1000u && (half_man & 1))) ++h; /* may carry into exp: correct */
    return h;
}

void oracle_h2f(const uint16_t* src, float* dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = h2f(src[i]);
}
void oracle_f2h(const float* src, uint16_t* dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = f2h(src[i]);
}

/* ---------- seeded generators ---------- */
static inline uint64_t splitmix64_at(uint64_t seed, uint64_t i) {
    uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* element i = lo + (hi-lo) * u, u = top 24 bits / 2^24, rounded to fp16 */
void oracle_fill_uniform(uint16_t* dst, int64_t n, uint64_t seed, float lo, float hi) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        float u = (float)(splitmix64_at(seed, (uint64_t)i) >> 40) * (1.0f / 16777216.0f);
        dst[i] = f2h(lo + (hi - lo) * u);
    }
}

/* Box-Muller in double on counters 2i, 2i+1; rounded to fp16 */
void oracle_fill_normal(uint16_t* dst, int64_t n, uint64_t seed, float mean, float stddev) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        double u1 = ((double)(splitmix64_at(seed, 2 * (uint64_t)i) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
        double u2 = (double)(splitmix64_at(seed, 2 * (uint64_t)i + 1) >> 11) * (1.0 / 9007199254740992.0);
        double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
        dst[i] = f2h((float)((double)mean + (double)stddev * z));
    }
}

/* ---------- GEMM ---------- */
/* f32 dot product of two f32 rows with 16 independent partial sums (fixed order). */
static inline float dot_f32(const float* a, const float* b, int64_t k) {
    float p[16] = {0};
    int64_t i = 0;
    for (; i + 16 <= k; i += 16)
        for (int j = 0; j < 16; ++j) p[j] += a[i + j] * b[i + j];
    float s = 0.f;
    for (; i < k; ++i) s += a[i] * b[i];
    for (int j = 0; j < 16; ++j) s += p[j];
    return s;
}

/* C[M,N] (f32, row-major) = A[M,K] (f16 row-major) · B (f16 column-major [K,N], i.e. Bt[N,K]).
 * Rows [m0, m1) only, so a caller can time or check a bounded sample. */
void oracle_gemm_f16_rows(const uint16_t* A, const uint16_t* Bt, float* C, int64_t M, int64_t N,
                          int64_t K, int64_t m0, int64_t m1) {
    (void)M;
    float* Bf = (float*)malloc(sizeof(float) * (size_t)N * (size_t)K);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < N * K; ++i) Bf[i] = h2f(Bt[i]);
#pragma omp parallel
    {
        float* arow = (float*)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(dynamic, 4)
        for (int64_t m = m0; m < m1; ++m) {
            for (int64_t k = 0; k < K; ++k) arow[k] = h2f(A[m * K + k]);
            for (int64_t n = 0; n < N; ++n) C[m * N + n] = dot_f32(arow, Bf + n * K, K);
        }
        free(arow);
    }
    free(Bf);
}

void oracle_gemm_f16(const uint16_t* A, const uint16_t* Bt, float* C, int64_t M, int64_t N, int64_t K) {
    oracle_gemm_f16_rows(A, Bt, C, M, N, K, 0, M);
}

/* sequential-k variant (the reference's naive_gemm order) for tiny cross-checks */
void oracle_gemm_f16_naive(const uint16_t* A, const uint16_t* Bt, float* C, int64_t M, int64_t N, int64_t K) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            float s = 0.f;
            for (int64_t k = 0; k < K; ++k) s += h2f(A[m * K + k]) * h2f(Bt[n * K + k]);
            C[m * N + n] = s;
        }
}

/* ---------- back-to-back GEMM ---------- */
/* D[M,P] f32 = f16round(A[M,K]·B[K,N]) · C[N,P];  A row-major, B column-major (Bt[N,K]),
 * C column-major (Ct[P,N]).  batch independent problems laid out back to back. */
void oracle_b2b_gemm_f16(const uint16_t* A, const uint16_t* Bt, const uint16_t* Ct, float* D, int64_t M,
                         int64_t N, int64_t K, int64_t P, int64_t batch) {
    for (int64_t b = 0; b < batch; ++b) {
        const uint16_t* Ab = A + b * M * K;
        const uint16_t* Bb = Bt + b * N * K;
        const uint16_t* Cb = Ct + b * P * N;
        float* Db = D + b * M * P;
        float* Bf = (float*)malloc(sizeof(float) * (size_t)(N * K));
        float* Cf = (float*)malloc(sizeof(float) * (size_t)(P * N));
        for (int64_t i = 0; i < N * K; ++i) Bf[i] = h2f(Bb[i]);
        for (int64_t i = 0; i < P * N; ++i) Cf[i] = h2f(Cb[i]);
#pragma omp parallel
        {
            float* arow = (float*)malloc(sizeof(float) * (size_t)K);
            float* acc = (float*)malloc(sizeof(float) * (size_t)N);
#pragma omp for schedule(static)
            for (int64_t m = 0; m < M; ++m) {
                for (int64_t k = 0; k < K; ++k) arow[k] = h2f(Ab[m * K + k]);
                for (int64_t n = 0; n < N; ++n) acc[n] = h2f(f2h(dot_f32(arow, Bf + n * K, K)));
                for (int64_t p = 0; p < P; ++p) Db[m * P + p] = dot_f32(acc, Cf + p * N, N);
            }
            free(arow);
            free(acc);
        }
        free(Bf);
        free(Cf);
    }
}

/* ---------- attention ---------- */
/* O[M,P] f32 = softmax_rows(scale · Q[M,K]·Kmat) · V per batch item.
 * Q row-major [M,K]; Kn = keys stored [N,K] row-major (the reference's column-major [K,N]);
 * v_col_major != 0: V stored [P,N] (reference boundary); else V stored [N,P].
 * Scores in f32, exp/sum in f64, output accumulation in f64. Rows [m0,m1) of each batch item. */
void oracle_attention_f16_rows(const uint16_t* Q, const uint16_t* Kn, const uint16_t* V, float* O, int64_t batch,
                               int64_t M, int64_t N, int64_t K, int64_t P, float scale, int v_col_major,
                               int64_t m0, int64_t m1) {
    for (int64_t b = 0; b < batch; ++b) {
        const uint16_t* Qb = Q + b * M * K;
        const uint16_t* Kb = Kn + b * N * K;
        const uint16_t* Vb = V + b * N * P;
        float* Ob = O + b * M * P;
        float* Kf = (float*)malloc(sizeof(float) * (size_t)(N * K));
        float* Vf = (float*)malloc(sizeof(float) * (size_t)(N * P)); /* [N,P] row-major */
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < N * K; ++i) Kf[i] = h2f(Kb[i]);
#pragma omp parallel for schedule(static)
        for (int64_t n = 0; n < N; ++n)
            for (int64_t p = 0; p < P; ++p) Vf[n * P + p] = h2f(v_col_major ? Vb[p * N + n] : Vb[n * P + p]);
#pragma omp parallel
        {
            float* q = (float*)malloc(sizeof(float) * (size_t)K);
            double* s = (double*)malloc(sizeof(double) * (size_t)N);
            double* o = (double*)malloc(sizeof(double) * (size_t)P);
#pragma omp for schedule(dynamic, 4)
            for (int64_t m = m0; m < m1; ++m) {
                for (int64_t k = 0; k < K; ++k) q[k] = h2f(Qb[m * K + k]);
                double mx = -INFINITY;
                for (int64_t n = 0; n < N; ++n) {
                    s[n] = (double)scale * (double)dot_f32(q, Kf + n * K, K);
                    if (s[n] > mx) mx = s[n];
                }
                double sum = 0.0;
                for (int64_t n = 0; n < N; ++n) { s[n] = exp(s[n] - mx); sum += s[n]; }
                for (int64_t p = 0; p < P; ++p) o[p] = 0.0;
                for (int64_t n = 0; n < N; ++n) {
                    const double w = s[n];
                    const float* v = Vf + n * P;
                    for (int64_t p = 0; p < P; ++p) o[p] += w * (double)v[p];
                }
                for (int64_t p = 0; p < P; ++p) Ob[m * P + p] = (float)(o[p] / sum);
            }
            free(q); free(s); free(o);
        }
        free(Kf);
        free(Vf);
    }
}

void oracle_attention_f16(const uint16_t* Q, const uint16_t* Kn, const uint16_t* V, float* O, int64_t batch,
                          int64_t M, int64_t N, int64_t K, int64_t P, float scale, int v_col_major) {
    oracle_attention_f16_rows(Q, Kn, V, O, batch, M, N, K, P, scale, v_col_major, 0, M);
}

/* Blockwise recurrence, f32 throughout, running max initialised to 0 and the output
 * renormalised every block, as the reference's test restates it.  Inputs f32:
 * Q[M,K], Kmat[K,N] row-major, V[N,P] row-major. tn = block length along N. */
void oracle_attention_blocked_f32(const float* Q, const float* Kmat, const float* V, float* O, int64_t M,
                                  int64_t N, int64_t K, int64_t P, int64_t tn, float scale) {
    float* w = (float*)malloc(sizeof(float) * (size_t)tn);
    float* ev = (float*)malloc(sizeof(float) * (size_t)P);
    for (int64_t m = 0; m < M; ++m) {
        float prev_max = 0.f, prev_sum = 0.f;
        float* o = O + m * P;
        for (int64_t p = 0; p < P; ++p) o[p] = 0.f;
        for (int64_t n0 = 0; n0 < N; n0 += tn) {
            float cur_max = -INFINITY;
            for (int64_t j = 0; j < tn; ++j) {
                float s = 0.f;
                for (int64_t k = 0; k < K; ++k) s += Q[m * K + k] * Kmat[k * N + n0 + j];
                w[j] = s * scale;
                if (w[j] > cur_max) cur_max = w[j];
            }
            float cur_sum = 0.f;
            for (int64_t j = 0; j < tn; ++j) { w[j] = expf(w[j] - cur_max); cur_sum += w[j]; }
            for (int64_t p = 0; p < P; ++p) {
                float s = 0.f;
                for (int64_t j = 0; j < tn; ++j) s += w[j] * V[(n0 + j) * P + p];
                ev[p] = s;
            }
            float new_max = cur_max > prev_max ? cur_max : prev_max;
            float renorm_prev = expf(prev_max - new_max);
            float renorm_cur = expf(cur_max - new_max);
            float new_sum = renorm_prev * prev_sum + renorm_cur * cur_sum;
            for (int64_t p = 0; p < P; ++p)
                o[p] = (o[p] * prev_sum * renorm_prev + renorm_cur * ev[p]) / new_sum;
            prev_sum = new_sum;
            prev_max = new_max;
        }
    }
    free(w);
    free(ev);
}

/* ---------- LSTM ---------- */
static inline float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

/* x[T,B,I] f16; W[4H, I+H] f16 row-major, rows grouped i,f,g,o; bias[4H] f16;
 * h0[B,H] f16 (may be NULL = 0), c0[B,H] f32 (may be NULL = 0).
 * h_all[T,B,H] f32 = h_t BEFORE rounding to f16 (the recurrence consumes f16-rounded h, as the
 * device keeps h in f16); c_out[B,H] f32 = c_T; c stays f32 throughout.
 * Batch rows [b0,b1) only (rows are independent). */
void oracle_lstm_f16_rows(const uint16_t* x, const uint16_t* W, const uint16_t* bias, const uint16_t* h0,
                          const float* c0, float* h_all, float* c_out, int64_t T, int64_t B, int64_t I,
                          int64_t H, int64_t b0, int64_t b1) {
    const int64_t KK = I + H;
    float* Wf = (float*)malloc(sizeof(float) * (size_t)(4 * H * KK));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < 4 * H * KK; ++i) Wf[i] = h2f(W[i]);
#pragma omp parallel
    {
        float* xh = (float*)malloc(sizeof(float) * (size_t)KK);
        float* c = (float*)malloc(sizeof(float) * (size_t)H);
        float* hn = (float*)malloc(sizeof(float) * (size_t)H);
#pragma omp for schedule(dynamic, 1)
        for (int64_t b = b0; b < b1; ++b) {
            for (int64_t j = 0; j < H; ++j) {
                xh[I + j] = h0 ? h2f(h0[b * H + j]) : 0.f;
                c[j] = c0 ? c0[b * H + j] : 0.f;
            }
            for (int64_t t = 0; t < T; ++t) {
                const uint16_t* xt = x + (t * B + b) * I;
                for (int64_t k = 0; k < I; ++k) xh[k] = h2f(xt[k]);
                for (int64_t j = 0; j < H; ++j) {
                    float gi = dot_f32(xh, Wf + (0 * H + j) * KK, KK) + h2f(bias[0 * H + j]);
                    float gf = dot_f32(xh, Wf + (1 * H + j) * KK, KK) + h2f(bias[1 * H + j]);
                    float gg = dot_f32(xh, Wf + (2 * H + j) * KK, KK) + h2f(bias[2 * H + j]);
                    float go = dot_f32(xh, Wf + (3 * H + j) * KK, KK) + h2f(bias[3 * H + j]);
                    float cn = sigmoidf_(gf) * c[j] + sigmoidf_(gi) * tanhf(gg);
                    c[j] = cn;
                    hn[j] = sigmoidf_(go) * tanhf(cn);
                }
                for (int64_t j = 0; j < H; ++j) {
                    h_all[(t * B + b) * H + j] = hn[j];
                    xh[I + j] = h2f(f2h(hn[j]));
                }
            }
            for (int64_t j = 0; j < H; ++j) c_out[b * H + j] = c[j];
        }
        free(xh); free(c); free(hn);
    }
    free(Wf);
}

void oracle_lstm_f16(const uint16_t* x, const uint16_t* W, const uint16_t* bias, const uint16_t* h0,
                     const float* c0, float* h_all, float* c_out, int64_t T, int64_t B, int64_t I, int64_t H) {
    oracle_lstm_f16_rows(x, W, bias, h0, c0, h_all, c_out, T, B, I, H, 0, B);
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
