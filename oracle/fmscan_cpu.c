/*
 * CPU restatement of the Factorization-Memory scan (test infrastructure, not
 * product: only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
 * bench.py load this library; nothing under fm_amd/ or fm/ does).
 *
 * Two families, both sequential along the sequence and independent across
 * rows (b, m, d), as the reference's kernel is per block (reference
 * fm/scan/fm_scan.cuh:62-64) and its PyTorch loop per time step
 * (fm/scan/fm_pytorch.py:35-38):
 *
 *   fmscan_oracle_*_f64   double in, double out: the checker.
 *   fmscan_cpu_*          storage dtype in/out (float32, float16 or bfloat16), float32
 *                         arithmetic, OpenMP over rows: the timed CPU baseline.
 *
 * Formulas (the same for both):
 *   forward   h[t] = g[t] h[t-1] + u[t], u = (1-g) x (plain: x), h[-1] = h0 or 0
 *             fm_pytorch.py:22,37; fm_scan.cuh:110,116,121-131
 *   backward  delta[t] = G[t] + g[t+1] delta[t+1], delta[L] = first_prop_grad or 0
 *             fm_scan.cuh:86-88,103-108,121
 *             token_grad[t] = (1 - g[t]) delta[t]          (plain: delta[t])   :184-185
 *             gate_grad[t]  = (h[t-1] - x[t]) delta[t]     (plain: h[t-1] delta[t])   :188-208
 *             h[-1] = h0; h0 == NULL reproduces the kernel, which reads
 *             first_prop_grad there (:196 with :380).
 *
 * Pinned by tests/test_oracle.py against oracle/fm_scan_oracle.py, which is
 * itself pinned by exact rational arithmetic, closed forms and finite differences.
 */
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* output row r = (b*M + m)*D + d -> gate row b*M + m, token row b*D + d (fm_scan.cuh:76-82) */
static inline void map_row(int64_t r, int64_t M, int64_t D, int64_t* grow, int64_t* xrow) {
    *grow = r / D;
    *xrow = (*grow / M) * D + (r - *grow * D);
}

/* ---------------------------------------------------------------- float64 checker */

void fmscan_oracle_forward_f64(const double* g, const double* x, const double* h0, double* out,
                               int64_t B, int64_t M, int64_t D, int64_t L, int plain) {
    const int64_t rows = B * M * D;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        int64_t gr, xr;
        map_row(r, M, D, &gr, &xr);
        const double* gp = g + gr * L;
        const double* xp = x + xr * L;
        double* op = out + r * L;
        double h = h0 ? h0[r] : 0.0;
        for (int64_t t = 0; t < L; ++t) {
            const double u = plain ? xp[t] : (1.0 - gp[t]) * xp[t];
            h = gp[t] * h + u;
            op[t] = h;
        }
    }
}

void fmscan_oracle_backward_f64(const double* g, const double* G, const double* fpg, double* dtok,
                                const double* h, const double* x, double* dgate, const double* h0,
                                int64_t B, int64_t M, int64_t D, int64_t L, int plain) {
    const int64_t rows = B * M * D;
    const double* hm1 = h0 ? h0 : fpg;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        int64_t gr, xr;
        map_row(r, M, D, &gr, &xr);
        const double* gp = g + gr * L;
        const double* xp = x ? x + xr * L : 0;
        const double* Gp = G + r * L;
        const double* hp = h + r * L;
        double* dx = dtok + r * L;
        double* dg = dgate + r * L;
        double from_future = fpg ? fpg[r] : 0.0; /* g[t+1] * delta[t+1] */
        for (int64_t t = L - 1; t >= 0; --t) {
            const double delta = Gp[t] + from_future;
            const double hprev = t > 0 ? hp[t - 1] : (hm1 ? hm1[r] : 0.0);
            if (plain) {
                dx[t] = delta;
                dg[t] = hprev * delta;
            } else {
                dx[t] = (1.0 - gp[t]) * delta;
                dg[t] = (hprev - xp[t]) * delta;
            }
            from_future = gp[t] * delta;
        }
    }
}

/* ------------------------------------------------ storage-dtype port (timed baseline) */

#define FMSCAN_CPU_F32 0
#define FMSCAN_CPU_F16 1
#define FMSCAN_CPU_BF16 2

static inline float bf16_to_f32(uint16_t v) {
    uint32_t u = (uint32_t)v << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint16_t f32_to_bf16(float f) { /* round to nearest even; NaN kept quiet */
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* IEEE binary16 <-> binary32 in integer arithmetic (the host compiler has no _Float16) */
static inline float f16_to_f32(uint16_t v) {
    const uint32_t sign = (uint32_t)(v & 0x8000u) << 16;
    uint32_t exp = (v >> 10) & 0x1fu, man = v & 0x3ffu, u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else { /* subnormal: normalise */
            int sh = 0;
            while (!(man & 0x400u)) { man <<= 1; ++sh; }
            u = sign | ((uint32_t)(113 - sh) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint16_t f32_to_f16(float f) { /* round to nearest even */
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (a > 0x7f800000u ? 0x200u : 0u));
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* rounds to infinity */
    if (a < 0x38800000u) {                                    /* subnormal or zero in binary16 */
        if (a < 0x33000000u) return sign;                     /* below half the smallest subnormal */
        const int e = (int)(a >> 23);
        const uint32_t m = (a & 0x7fffffu) | 0x800000u;
        const int shift = 126 - e; /* 14..24 */
        uint32_t r = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (r & 1u))) ++r;
        return (uint16_t)(sign | r);
    }
    uint32_t r = a - 0x38000000u; /* rebias */
    r += 0xfffu + ((r >> 13) & 1u);
    return (uint16_t)(sign | (r >> 13));
}

static inline float ld_f32(const float* p, int64_t i) { return p[i]; }
static inline void st_f32(float* p, int64_t i, float v) { p[i] = v; }
static inline float ld_bf16(const uint16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
static inline void st_bf16(uint16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }
static inline float ld_f16(const uint16_t* p, int64_t i) { return f16_to_f32(p[i]); }
static inline void st_f16(uint16_t* p, int64_t i, float v) { p[i] = f32_to_f16(v); }

#define LD(T, p, i) LOAD((const T*)(p), i)
#define ST(T, p, i, v) STORE((T*)(p), i, v)

#define DEFINE_PORT(T, SUF)                                                                        \
    static void forward_##SUF(const T* g, const T* x, const T* h0, T* out, int64_t M, int64_t D,   \
                              int64_t L, int64_t rows, int plain) {                                \
        _Pragma("omp parallel for schedule(static)")                                               \
        for (int64_t r = 0; r < rows; ++r) {                                                       \
            int64_t gr, xr;                                                                        \
            map_row(r, M, D, &gr, &xr);                                                            \
            const T* gp = g + gr * L;                                                              \
            const T* xp = x + xr * L;                                                              \
            T* op = out + r * L;                                                                   \
            float h = h0 ? LD(T, h0, r) : 0.0f;                                                    \
            for (int64_t t = 0; t < L; ++t) {                                                      \
                const float gt = LD(T, gp, t), xt = LD(T, xp, t);                                  \
                const float u = plain ? xt : (1.0f - gt) * xt;                                     \
                h = gt * h + u;                                                                    \
                ST(T, op, t, h);                                                                   \
            }                                                                                      \
        }                                                                                          \
    }                                                                                              \
    static void backward_##SUF(const T* g, const T* G, const T* fpg, T* dtok, const T* h,          \
                               const T* x, T* dgate, const T* h0, int64_t M, int64_t D, int64_t L, \
                               int64_t rows, int plain) {                                          \
        const T* hm1 = h0 ? h0 : fpg;                                                              \
        _Pragma("omp parallel for schedule(static)")                                               \
        for (int64_t r = 0; r < rows; ++r) {                                                       \
            int64_t gr, xr;                                                                        \
            map_row(r, M, D, &gr, &xr);                                                            \
            const T* gp = g + gr * L;                                                              \
            const T* xp = x ? x + xr * L : 0;                                                      \
            const T* Gp = G + r * L;                                                               \
            const T* hp = h + r * L;                                                               \
            T* dx = dtok + r * L;                                                                  \
            T* dg = dgate + r * L;                                                                 \
            float from_future = fpg ? LD(T, fpg, r) : 0.0f;                                        \
            float hnext = L > 1 ? LD(T, hp, L - 2) : 0.0f; /* h[t-1], read one step ahead */       \
            for (int64_t t = L - 1; t >= 0; --t) {                                                 \
                const float gt = LD(T, gp, t);                                                     \
                const float delta = LD(T, Gp, t) + from_future;                                    \
                const float hprev = t > 0 ? hnext : (hm1 ? LD(T, hm1, r) : 0.0f);                  \
                if (t > 1) hnext = LD(T, hp, t - 2);                                               \
                if (plain) {                                                                       \
                    ST(T, dx, t, delta);                                                           \
                    ST(T, dg, t, hprev * delta);                                                   \
                } else {                                                                           \
                    ST(T, dx, t, (1.0f - gt) * delta);                                             \
                    ST(T, dg, t, (hprev - LD(T, xp, t)) * delta);                                  \
                }                                                                                  \
                from_future = gt * delta;                                                          \
            }                                                                                      \
        }                                                                                          \
    }

#define LOAD ld_f32
#define STORE st_f32
DEFINE_PORT(float, f32)
#undef LOAD
#undef STORE
#define LOAD ld_bf16
#define STORE st_bf16
DEFINE_PORT(uint16_t, bf16)
#undef LOAD
#undef STORE
#define LOAD ld_f16
#define STORE st_f16
DEFINE_PORT(uint16_t, f16)
#undef LOAD
#undef STORE

/* float32 -> binary16 bit patterns with the port's own rounding (for its conversion test) */
void fmscan_cpu_round_f16(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = f32_to_f16(in[i]);
}

static void set_threads(int nthreads) {
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#else
    (void)nthreads;
#endif
}

int fmscan_cpu_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* returns 0, or -3 for a dtype other than float32 (0) / float16 (1) / bfloat16 (2) */
int fmscan_cpu_forward(const void* g, const void* x, const void* h0, void* out, int64_t B, int64_t M,
                       int64_t D, int64_t L, int dtype, int plain, int nthreads) {
    set_threads(nthreads);
    if (dtype == FMSCAN_CPU_F32)
        forward_f32((const float*)g, (const float*)x, (const float*)h0, (float*)out, M, D, L, B * M * D, plain);
    else if (dtype == FMSCAN_CPU_BF16)
        forward_bf16((const uint16_t*)g, (const uint16_t*)x, (const uint16_t*)h0, (uint16_t*)out, M, D, L,
                     B * M * D, plain);
    else if (dtype == FMSCAN_CPU_F16)
        forward_f16((const uint16_t*)g, (const uint16_t*)x, (const uint16_t*)h0, (uint16_t*)out, M, D, L,
                    B * M * D, plain);
    else
        return -3;
    return 0;
}

int fmscan_cpu_backward(const void* g, const void* G, const void* fpg, void* dtok, const void* h,
                        const void* x, void* dgate, const void* h0, int64_t B, int64_t M, int64_t D,
                        int64_t L, int dtype, int plain, int nthreads) {
    set_threads(nthreads);
    if (dtype == FMSCAN_CPU_F32)
        backward_f32((const float*)g, (const float*)G, (const float*)fpg, (float*)dtok, (const float*)h,
                     (const float*)x, (float*)dgate, (const float*)h0, M, D, L, B * M * D, plain);
    else if (dtype == FMSCAN_CPU_BF16)
        backward_bf16((const uint16_t*)g, (const uint16_t*)G, (const uint16_t*)fpg, (uint16_t*)dtok,
                      (const uint16_t*)h, (const uint16_t*)x, (uint16_t*)dgate, (const uint16_t*)h0, M, D, L,
                      B * M * D, plain);
    else if (dtype == FMSCAN_CPU_F16)
        backward_f16((const uint16_t*)g, (const uint16_t*)G, (const uint16_t*)fpg, (uint16_t*)dtok,
                     (const uint16_t*)h, (const uint16_t*)x, (uint16_t*)dgate, (const uint16_t*)h0, M, D, L,
                     B * M * D, plain);
    else
        return -3;
    return 0;
}
