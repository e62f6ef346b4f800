/* Plain-C restatement of lmms-engine's Muon step arithmetic.  TEST INFRASTRUCTURE ONLY.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this
 * library; the product never does.  It is independent of torch: bf16 is carried as
 * uint16_t bit patterns and every rounding is spelled out, so it pins the torch
 * restatement in oracle/muon_oracle.py (tests/test_oracle.py compares the two).
 *
 * Follows /root/reference/src/lmms_engine/utils/muon_utils.py:
 *   orc_mmt            matmul_transpose_assign + mmt_kernel   :95-119, :28-92
 *   orc_newton_schulz  fast_newtonschulz                      :129-156
 *   orc_momentum       muon_update's two lerp_ calls          :188-189
 *   orc_scale_update   apply_scaling + SingelDeviceWork tail  :167-175, :324-325
 *   orc_adamw          adam_update + Adam branch              :178-183, :468-477
 *
 * Build: gcc -O2 -fopenmp -ffp-contract=off -shared -fPIC (oracle/Makefile).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = ((uint32_t)h) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even fp32 -> bf16, NaN kept quiet */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

uint16_t orc_f32_to_bf16(float f) { return f32_to_bf16(f); }
float orc_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

/* out (M x M) = bf(X Xt), X (M x K) bf16 row-major, fp32 accumulation in k order,
 * upper triangle computed and mirrored. */
void orc_mmt(const uint16_t* X, int M, int K, uint16_t* out) {
    float* Xf = (float*)malloc(sizeof(float) * (size_t)M * K);
    for (size_t i = 0; i < (size_t)M * K; ++i) Xf[i] = bf16_to_f32(X[i]);
#pragma omp parallel for schedule(dynamic, 4)
    for (int i = 0; i < M; ++i) {
        for (int j = i; j < M; ++j) {
            const float* a = Xf + (size_t)i * K;
            const float* b = Xf + (size_t)j * K;
            float acc = 0.f;
            for (int k = 0; k < K; ++k) acc += a[k] * b[k];
            uint16_t r = f32_to_bf16(acc);
            out[(size_t)i * M + j] = r;
            out[(size_t)j * M + i] = r;
        }
    }
    free(Xf);
}

/* G (rows x cols) fp32 row-major -> out (rows x cols) bf16.  (a,b,c) passed as doubles
 * and narrowed to fp32 like a python scalar meeting a bf16 tensor. */
void orc_newton_schulz(const float* G, int rows, int cols, int steps, double a_, double b_, double c_,
                       uint16_t* out) {
    const int transposed = rows > cols;
    const int M = transposed ? cols : rows;
    const int K = transposed ? rows : cols;
    const float a = (float)a_, b = (float)b_, c = (float)c_;
    size_t MK = (size_t)M * K, MM = (size_t)M * M;
    uint16_t* X = (uint16_t*)malloc(2 * MK);
    uint16_t* Xn = (uint16_t*)malloc(2 * MK);
    uint16_t* A = (uint16_t*)malloc(2 * MM);
    uint16_t* A2 = (uint16_t*)malloc(2 * MM);
    float* Bf = (float*)malloc(4 * MM);
    float* Xf = (float*)malloc(4 * MK);
    /* X = bf(G), viewed transposed when rows > cols (:138-140) */
    for (int i = 0; i < M; ++i)
        for (int k = 0; k < K; ++k)
            X[(size_t)i * K + k] = f32_to_bf16(transposed ? G[(size_t)k * cols + i] : G[(size_t)i * cols + k]);
    /* n = bf(sqrt(sum bf(x)^2)) with fp32 accumulation; d = bf(n + 1e-7)  (:146) */
    double ss = 0.0; /* exact-ish sum; the bf16 rounding of the root absorbs ordering noise */
    for (size_t i = 0; i < MK; ++i) {
        float v = bf16_to_f32(X[i]);
        ss += (double)v * v;
    }
    float n = bf16_to_f32(f32_to_bf16((float)sqrt(ss)));
    float d = bf16_to_f32(f32_to_bf16(n + (float)1e-7));
    for (size_t i = 0; i < MK; ++i) X[i] = f32_to_bf16(bf16_to_f32(X[i]) / d);
    for (int s = 0; s < steps; ++s) {
        orc_mmt(X, M, K, A);   /* :149 */
        orc_mmt(A, M, M, A2);  /* :150 */
        for (size_t i = 0; i < MM; ++i) { /* B = bf(bf(b A) + bf(c A2))  :151 */
            float t1 = bf16_to_f32(f32_to_bf16(b * bf16_to_f32(A[i])));
            float t2 = bf16_to_f32(f32_to_bf16(c * bf16_to_f32(A2[i])));
            Bf[i] = bf16_to_f32(f32_to_bf16(t1 + t2));
        }
        for (size_t i = 0; i < MK; ++i) Xf[i] = bf16_to_f32(X[i]);
#pragma omp parallel for schedule(static)
        for (int i = 0; i < M; ++i) { /* X = bf(bf(a X) + bf(B X))  :152 */
            float* acc = (float*)calloc((size_t)K, sizeof(float));
            for (int m = 0; m < M; ++m) {
                float bim = Bf[(size_t)i * M + m];
                const float* xr = Xf + (size_t)m * K;
                for (int k = 0; k < K; ++k) acc[k] += bim * xr[k];
            }
            for (int k = 0; k < K; ++k) {
                float bx = bf16_to_f32(f32_to_bf16(acc[k]));
                float ax = bf16_to_f32(f32_to_bf16(a * Xf[(size_t)i * K + k]));
                Xn[(size_t)i * K + k] = f32_to_bf16(ax + bx);
            }
            free(acc);
        }
        uint16_t* t = X; X = Xn; Xn = t;
    }
    for (int i = 0; i < M; ++i)
        for (int k = 0; k < K; ++k) {
            uint16_t v = X[(size_t)i * K + k];
            if (transposed) out[(size_t)k * cols + i] = v; else out[(size_t)i * cols + k] = v;
        }
    free(X); free(Xn); free(A); free(A2); free(Bf); free(Xf);
}

/* fp32 grad g (read-only), fp32 momentum m (in place), writes the fp32 update u.
 * ATen lerp: |w|<0.5 -> s + w(e-s); else e - (e-s)(1-w); evaluated with one fma. */
void orc_momentum(const float* g, float* m, float* u, size_t n, double beta_, int nesterov) {
    const float w1 = (float)(1.0 - beta_); /* 1-beta computed in double by python, then narrowed */
    const float w2 = (float)beta_;
    for (size_t i = 0; i < n; ++i) {
        float mi = m[i], gi = g[i];
        float mn = (fabsf(w1) < 0.5f) ? fmaf(w1, gi - mi, mi) : fmaf(w1 - 1.0f, gi - mi, gi);
        m[i] = mn;
        if (nesterov) {
            /* g.lerp_(m, beta): start=g, end=m */
            u[i] = (fabsf(w2) < 0.5f) ? fmaf(w2, mn - gi, gi) : fmaf(w2 - 1.0f, mn - gi, mn);
        } else {
            u[i] = mn;
        }
    }
}

/* o = bf(O*s); p = p*(1-lr*wd); p = p + (-lr)*o, fp32 param, bf16 O; writes o back. */
void orc_scale_update_f32(float* p, uint16_t* O, size_t n, double scale_, double lr_, double wd_) {
    const float s = (float)scale_;
    const float decay = (float)(1.0 - lr_ * wd_);
    const float alpha = (float)(-lr_);
    for (size_t i = 0; i < n; ++i) {
        uint16_t ob = f32_to_bf16(bf16_to_f32(O[i]) * s);
        O[i] = ob;
        float pv = p[i] * decay;
        p[i] = pv + alpha * bf16_to_f32(ob);
    }
}

/* same with a bf16 param: each in-place op rounds to bf16. */
void orc_scale_update_bf16(uint16_t* p, uint16_t* O, size_t n, double scale_, double lr_, double wd_) {
    const float s = (float)scale_;
    const float decay = (float)(1.0 - lr_ * wd_);
    const float alpha = (float)(-lr_);
    for (size_t i = 0; i < n; ++i) {
        uint16_t ob = f32_to_bf16(bf16_to_f32(O[i]) * s);
        O[i] = ob;
        float pv = bf16_to_f32(f32_to_bf16(bf16_to_f32(p[i]) * decay));
        p[i] = f32_to_bf16(pv + alpha * bf16_to_f32(ob));
    }
}

/* fp32 AdamW fallback, step already incremented. */
void orc_adamw_f32(float* p, const float* g, float* e1, float* e2, size_t n, int step, double lr_, double b1_,
                   double b2_, double eps_, double wd_) {
    const float w1 = (float)(1.0 - b1_), w2 = (float)(1.0 - b2_);
    /* tensor / python scalar on a GPU: a multiplication by the scalar's reciprocal, taken in double and narrowed */
    const float r1 = (float)(1.0 / (1.0 - pow(b1_, step))), r2 = (float)(1.0 / (1.0 - pow(b2_, step)));
    const float eps = (float)eps_;
    const float decay = (float)(1.0 - lr_ * wd_);
    const float alpha = (float)(-lr_);
    for (size_t i = 0; i < n; ++i) {
        float gi = g[i];
        float a = (fabsf(w1) < 0.5f) ? fmaf(w1, gi - e1[i], e1[i]) : fmaf(w1 - 1.0f, gi - e1[i], gi);
        float g2 = gi * gi;
        float b = (fabsf(w2) < 0.5f) ? fmaf(w2, g2 - e2[i], e2[i]) : fmaf(w2 - 1.0f, g2 - e2[i], g2);
        e1[i] = a;
        e2[i] = b;
        float upd = (a * r1) / (sqrtf(b * r2) + eps);
        float pv = p[i] * decay;
        p[i] = pv + alpha * upd;
    }
}
