/*
 * oracle_c.c -- plain-C restatement of what Julia Base computes on `Array` for the ops of the
 * array-kernel path.  TEST INFRASTRUCTURE ONLY: it serves as the timed CPU baseline ("port") of
 * bench.py and is cross-checked against the NumPy oracle in tests/test_oracle.py.  Nothing in the
 * product links or calls it.
 *
 * The reference (AMDGPU.jl) defines every op of the path as "equal to Julia Base on Array"
 * (test/runtests.jl:77-82); Julia itself is not available here, so these loops restate Base:
 *   - sum / mapreduce over a whole array: pairwise reduction with 1024-element sequential
 *     blocks (Base.mapreduce_impl), the entry the GPU op of src/kernels/mapreduce.jl:86 replaces;
 *   - mapreduce(abs2, +, A; dims): column-major loops in the order of Base._mapreducedim!;
 *   - findmax(A; dims=1): sequential scan with Base's isless rule (first maximum, NaN wins);
 *   - accumulate(+, x) eltype-preserving (src/kernels/accumulate.jl:1-8 semantics) and cumsum
 *     along dim 1;
 *   - the two benchmark broadcasts (src/broadcast.jl:3-35);
 *   - volumerhs: loop nest of perf/volumerhs.jl:42-176, one element at a time.
 * With -fopenmp the independent outer loops run on all cores (Julia Base itself is single-threaded;
 * `threads` = 1 reproduces that).
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define PAIRWISE_BLOCK 1024

static double pairwise_f32(const float* a, int64_t lo, int64_t hi) {   /* [lo, hi) */
    if (hi - lo <= PAIRWISE_BLOCK) {
        float s = 0.0f;                     /* Base accumulates Float32 in Float32 */
        for (int64_t i = lo; i < hi; ++i) s += a[i];
        return (double)s;
    }
    int64_t mid = lo + ((hi - lo) >> 1);
    return (double)((float)pairwise_f32(a, lo, mid) + (float)pairwise_f32(a, mid, hi));
}

/* sum(x::Vector{Float32}) -> Float32 (returned widened) */
double orc_sum_f32(const float* x, int64_t n, int threads) {
    if (n == 0) return 0.0;
    if (threads <= 1) return pairwise_f32(x, 0, n);
    double parts[256];
    if (threads > 256) threads = 256;
    int64_t per = (n + threads - 1) / threads;
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int t = 0; t < threads; ++t) {
        int64_t lo = t * per, hi = lo + per < n ? lo + per : n;
        parts[t] = lo < hi ? pairwise_f32(x, lo, hi) : 0.0;
    }
    float s = 0.0f;
    for (int t = 0; t < threads; ++t) s += (float)parts[t];
    return (double)s;
}

/* sum(x::Vector{Int32}) -> Int64 (Base.add_sum widens) */
int64_t orc_sum_i32(const int32_t* x, int64_t n, int threads) {
    int64_t s = 0;
#pragma omp parallel for num_threads(threads) reduction(+ : s) schedule(static)
    for (int64_t i = 0; i < n; ++i) s += (int64_t)x[i];
    return s;
}

/* Base.max on Float32: NaN propagates, max(-0.0, 0.0) == 0.0 */
static float max_f32(float a, float b) {
    if (isnan(a)) return a;
    if (isnan(b)) return b;
    if (a == b) return signbit(a) ? b : a;
    return a > b ? a : b;
}

/* maximum(x::Vector{Float32}); n >= 1.  Threads reduce contiguous shares, combined in order (max is associative). */
float orc_maximum_f32(const float* x, int64_t n, int threads) {
    if (threads < 1) threads = 1;
    if (threads > 256) threads = 256;
    float parts[256];
    int64_t per = (n + threads - 1) / threads;
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int t = 0; t < threads; ++t) {
        int64_t lo = t * per, hi = lo + per < n ? lo + per : n;
        float m = -INFINITY;
        for (int64_t i = lo; i < hi; ++i) m = max_f32(m, x[i]);
        parts[t] = m;
    }
    float m = parts[0];
    for (int t = 1; t < threads; ++t) m = max_f32(m, parts[t]);
    return m;
}

/* mapreduce(abs2, +, A; dims=1) on an m x n column-major matrix -> out[n] */
void orc_abs2sum_dims1_f32(const float* A, int64_t m, int64_t n, float* out, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int64_t j = 0; j < n; ++j) {
        const float* c = A + j * m;
        float s = 0.0f;
        for (int64_t i = 0; i < m; ++i) s += c[i] * c[i];
        out[j] = s;
    }
}

/* mapreduce(abs2, +, A; dims=2) -> out[m]; Base walks columns and accumulates into R */
void orc_abs2sum_dims2_f32(const float* A, int64_t m, int64_t n, float* out, int threads) {
#pragma omp parallel num_threads(threads)
    {
#pragma omp for schedule(static)
        for (int64_t i = 0; i < m; ++i) out[i] = 0.0f;
        /* each thread owns a band of rows so the accumulation order per row matches Base */
#ifdef _OPENMP
        int t = omp_get_thread_num(), nt = omp_get_num_threads();
#else
        int t = 0, nt = 1;
#endif
        int64_t per = (m + nt - 1) / nt, lo = t * per, hi = lo + per < m ? lo + per : m;
        for (int64_t j = 0; j < n; ++j) {
            const float* c = A + j * m;
            for (int64_t i = lo; i < hi; ++i) out[i] += c[i] * c[i];
        }
    }
}

/* findmax(A; dims=1): first maximum under isless (NaN greatest, -0.0 < 0.0); idx = 1-based row */
void orc_findmax_dims1_f32(const float* A, int64_t m, int64_t n, float* vals, int64_t* rows, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int64_t j = 0; j < n; ++j) {
        const float* c = A + j * m;
        float best = c[0];
        int64_t bi = 0;
        for (int64_t i = 1; i < m; ++i) {
            float v = c[i];
            int less;   /* isless(best, v) */
            if (isnan(best) || isnan(v)) less = !isnan(best) && isnan(v);
            else if (best == v) less = signbit(best) && !signbit(v);
            else less = best < v;
            if (less) { best = v; bi = i; }
        }
        vals[j] = best;
        rows[j] = bi + 1;
    }
}

/* accumulate(+, x::Vector{Int32}) -> Vector{Int32}, wrapping */
void orc_cumsum_i32(const int32_t* x, int64_t n, int32_t* out) {
    uint32_t s = 0;
    for (int64_t i = 0; i < n; ++i) { s += (uint32_t)x[i]; out[i] = (int32_t)s; }
}

/* cumsum(B; dims=1) on an m x n column-major Float32 matrix */
void orc_cumsum_dims1_f32(const float* B, int64_t m, int64_t n, float* out, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int64_t j = 0; j < n; ++j) {
        float s = 0.0f;
        for (int64_t i = 0; i < m; ++i) { s += B[j * m + i]; out[j * m + i] = s; }
    }
}

/* cumsum(B; dims=2) on an m x n column-major Float32 matrix: row i runs over the columns, stride m.  Walked
 * column by column (cache-friendly), threads split the rows. */
void orc_cumsum_dims2_f32(const float* B, int64_t m, int64_t n, float* out, int threads) {
#pragma omp parallel num_threads(threads)
    {
        int t = 0, nt = 1;
#ifdef _OPENMP
        t = omp_get_thread_num();
        nt = omp_get_num_threads();
#endif
        int64_t per = (m + nt - 1) / nt, lo = t * per, hi = lo + per < m ? lo + per : m;
        for (int64_t j = 0; j < n; ++j)
            for (int64_t i = lo; i < hi; ++i) out[j * m + i] = (j == 0 ? 0.0f : out[(j - 1) * m + i]) + B[j * m + i];
    }
}

/* z .= a .* x .+ y .* exp.(w) */
void orc_bcast_axpby_exp_f32(float a, const float* x, const float* y, const float* w, float* z, int64_t n, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int64_t i = 0; i < n; ++i) z[i] = a * x[i] + y[i] * expf(w[i]);
}

/* C .= A .+ r .* c   (A, C: m x n; r: 1 x n; c: m x 1) */
void orc_bcast_rowcol_f32(const float* A, const float* r, const float* c, float* C, int64_t m, int64_t n, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int64_t j = 0; j < n; ++j)
        for (int64_t i = 0; i < m; ++i) C[j * m + i] = A[j * m + i] + r[j] * c[i];
}

/* volumerhs!, Float32, N = 4: loop nest of perf/volumerhs.jl:61-174 */
enum { NQ = 5, NP = 125, NSTATE = 5, NVGEO = 14 };
void orc_volumerhs_f32(float* rhs, const float* Q, const float* vgeo, float gravity, const float* D, int64_t nelem, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int64_t e = 0; e < nelem; ++e) {
        const float* q = Q + e * NSTATE * NP;
        const float* vg = vgeo + e * NVGEO * NP;
        float r[NSTATE][NP];
        float F[NSTATE][NP], G[NSTATE][NP], H[NSTATE][NP];
        memset(r, 0, sizeof r);
        for (int node = 0; node < NP; ++node) {
            float rho = q[node], U = q[NP + node], V = q[2 * NP + node], W = q[3 * NP + node], E = q[4 * NP + node];
            float MJ = vg[9 * NP + node], z = vg[13 * NP + node];
            float xix = vg[node], etx = vg[NP + node], zex = vg[2 * NP + node];
            float xiy = vg[3 * NP + node], ety = vg[4 * NP + node], zey = vg[5 * NP + node];
            float xiz = vg[6 * NP + node], etz = vg[7 * NP + node], zez = vg[8 * NP + node];
            float rinv = 1.0f / rho, r2inv = 1.0f / (2.0f * rho);
            float P = 0.4f * (E - (U * U + V * V + W * W) * r2inv - rho * gravity * z);
            float fx[5] = {U, rinv * U * U + P, rinv * U * V, rinv * U * W, rinv * U * (E + P)};
            float fy[5] = {V, rinv * V * U, rinv * V * V + P, rinv * V * W, rinv * V * (E + P)};
            float fz[5] = {W, rinv * W * U, rinv * W * V, rinv * W * W + P, rinv * W * (E + P)};
            for (int s = 0; s < NSTATE; ++s) {
                F[s][node] = MJ * (xix * fx[s] + xiy * fy[s] + xiz * fz[s]);
                G[s][node] = MJ * (etx * fx[s] + ety * fy[s] + etz * fz[s]);
                H[s][node] = MJ * (zex * fx[s] + zey * fy[s] + zez * fz[s]);
            }
            r[3][node] -= MJ * rho * gravity;
        }
        for (int s = 0; s < NSTATE; ++s)
            for (int k = 0; k < NQ; ++k)
                for (int j = 0; j < NQ; ++j)
                    for (int i = 0; i < NQ; ++i) {
                        float acc = 0.0f;
                        for (int n = 0; n < NQ; ++n) {
                            acc += D[n + NQ * i] * F[s][n + NQ * j + NQ * NQ * k];
                            acc += D[n + NQ * j] * G[s][i + NQ * n + NQ * NQ * k];
                            acc += D[n + NQ * k] * H[s][i + NQ * j + NQ * NQ * n];
                        }
                        r[s][i + NQ * j + NQ * NQ * k] += acc;
                    }
        for (int s = 0; s < NSTATE; ++s)
            for (int node = 0; node < NP; ++node)
                rhs[e * NSTATE * NP + s * NP + node] += vg[10 * NP + node] * r[s][node];
    }
}

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
