/* CPU restatement of the NCN layer in plain C -- TEST INFRASTRUCTURE ONLY.
 *
 * Nothing in the shipped package links or loads this file.  It is a second, independent checker next to
 * oracle/ncn_oracle.py (used by tests/) and the CPU baseline that bench.py times on the host cores.  It follows the
 * reference's definition line by line, one (batch entry, head, group) at a time, scalar loops, no tricks:
 *
 *   index map          torch_ref/ncn_pytorch.py:12-41     slot o of group g at stage l is row ((g + o s_l) mod G) n + o,
 *                                                          s_0 = 0, s_l = 2^(l-1) mod G, G = N / n
 *   one stage forward  torch_ref/ncn_pytorch.py:45-99     n steps; step j uses the pre-step row x_j for every row:
 *                                                          s_i = <x_i,Wi> + <x_j,Wj>, T = alpha x_i + (1-alpha) s_i x_j,
 *                                                          xa' = m xa + (1-m) F(T), x' = m x + (1-m) xa'
 *   W per head         torch_ref/ncn_pytorch.py:60-61     Wi = W[c Ec : (c+1) Ec], Wj = W[E + c Ec : E + (c+1) Ec]
 *   one-step inverse   torch_ref/ncn_pytorch_invertible.py:87-113
 *   backward           the closed form of ncn_triton/ncn_triton.py:176-246 (cross-checked with
 *                      ncn_cuda/ncn_bwd_cuda_kernel.cu:124-216): invert a step, recompute T, apply the step's
 *                      vector-Jacobian product; gradients of W summed over batch, groups and rows
 *   tables, lengths    ncn_triton/ncn_triton_old.py:53-96: `table` [N] gives the position of slot o of group g at entry
 *                      g n + o (instead of the stride map), `ctx_len` [batch] the live slots of a batch entry: groups
 *                      below the length run as usual, the group it cuts runs on its live rows with as many steps,
 *                      rows past the length pass through (y = x, dx = dy; this build's choice, the reference leaves
 *                      them unwritten)
 *   activations        ncn_fwd_cuda_kernel.cu:86-95 (0 tanh, 1 relu, 2 sigmoid, other linear), 3 = leaky relu with
 *                      slope 0.01 (ncn_triton/ncn_triton.py:22-28)
 *
 * Pinning: tests/test_oracle_c.py checks the double build against the float64 vectors the reference's own CPU code
 * produced (tests/golden, 1e-12), the float build against its float32 vectors and against the vectors of the
 * reference's Triton kernels, and both against oracle/ncn_oracle.py on random shapes.  relu and sigmoid, which no
 * vector of the reference covers, are held to the Python oracle there, which pins them by what the mathematics fixes
 * (tests/test_oracle_properties.py).  Parity unpinned, as in the Python oracle: the pass-through of rows past a length.
 *
 * Built twice from this one file: -DREAL=float (suffix _f32, what the baseline times) and -DREAL=double (_f64).
 * Groups are independent, so the loops over them are OpenMP-parallel; dW is summed per thread in double and the
 * threads' sums are added in thread order.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#ifndef REAL
#define REAL float
#endif
#ifndef SUFFIX
#define SUFFIX _f32
#endif
#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define NAME(base) CAT(base, SUFFIX)

#define MAX_N 64
#define MAX_EC 128

typedef REAL real;

/* libm in the precision of the build: tanhf / expf for float, tanh / exp for double */
#define REAL_IS_FLOAT (sizeof(real) == sizeof(float))
static real real_tanh(real t) { return REAL_IS_FLOAT ? (real)tanhf((float)t) : (real)tanh((double)t); }
static real real_exp(real t) { return REAL_IS_FLOAT ? (real)expf((float)t) : (real)exp((double)t); }

static real act_f(real t, int code) {
    if (code == 0) return real_tanh(t);
    if (code == 1) return t > 0 ? t : 0;
    if (code == 2) return 1 / (1 + real_exp(-t));
    if (code == 3) return t >= 0 ? t : (real)0.01 * t;
    return t;
}

static real act_df(real t, real f, int code) {
    if (code == 0) return 1 - f * f;
    if (code == 1) return f > 0 ? 1 : 0;
    if (code == 2) return f * (1 - f);
    if (code == 3) return t >= 0 ? 1 : (real)0.01;
    return 1;
}

/* 2^(stage-1) mod groups, 0 for stage 0 (Python integers in the reference) */
static int64_t stage_stride(int64_t stage, int64_t groups) {
    if (stage == 0) return 0;
    uint64_t r = 1 % (uint64_t)groups, b = 2 % (uint64_t)groups;
    for (uint64_t e = (uint64_t)stage - 1; e; e >>= 1) {
        if (e & 1) r = r * b % (uint64_t)groups;
        b = b * b % (uint64_t)groups;
    }
    return (int64_t)r;
}

static int64_t row_of(int64_t g, int64_t o, int64_t stride, int64_t groups, int64_t n) {
    return ((g + o * stride) % groups) * n + o;
}

/* one step forward on a gathered group: x, a are [n][ec] */
static void step_forward(real* x, real* a, const real* wi, const real* wj, int n, int ec, int j, real alpha, real m,
                         int code) {
    real xj[MAX_EC];
    memcpy(xj, x + (size_t)j * ec, sizeof(real) * ec);
    real ej = 0;
    for (int f = 0; f < ec; ++f) ej += xj[f] * wj[f];
    for (int i = 0; i < n; ++i) {
        real* xi = x + (size_t)i * ec;
        real* ai = a + (size_t)i * ec;
        real s = ej;
        for (int f = 0; f < ec; ++f) s += xi[f] * wi[f];
        for (int f = 0; f < ec; ++f) {
            const real t = alpha * xi[f] + (1 - alpha) * s * xj[f];
            ai[f] = m * ai[f] + (1 - m) * act_f(t, code);
            xi[f] = m * xi[f] + (1 - m) * ai[f];
        }
    }
}

/* undo one step: y, b hold the step's outputs and become its inputs; s_out[n], df_out[n][ec] if wanted */
static void step_inverse(real* y, real* b, const real* wi, const real* wj, int n, int ec, int j, real alpha, real m,
                         int code, real* s_out, real* df_out) {
    for (int i = 0; i < n * ec; ++i) y[i] = (y[i] - (1 - m) * b[i]) / m;
    const real* xj = y + (size_t)j * ec;
    real ej = 0;
    for (int f = 0; f < ec; ++f) ej += xj[f] * wj[f];
    for (int i = 0; i < n; ++i) {
        const real* xi = y + (size_t)i * ec;
        real* bi = b + (size_t)i * ec;
        real s = ej;
        for (int f = 0; f < ec; ++f) s += xi[f] * wi[f];
        if (s_out) s_out[i] = s;
        for (int f = 0; f < ec; ++f) {
            const real t = alpha * xi[f] + (1 - alpha) * s * xj[f];
            const real fv = act_f(t, code);
            if (df_out) df_out[(size_t)i * ec + f] = act_df(t, fv, code);
            bi[f] = (bi[f] - (1 - m) * fv) / m;
        }
    }
}

/* positions of the n slots of group g, and how many of them are live for a batch entry of length len */
static int group_rows(int64_t* pos, int64_t g, int64_t stride, int64_t groups, int n, const int32_t* table, int64_t len) {
    for (int o = 0; o < n; ++o) pos[o] = table ? (int64_t)table[g * n + o] : row_of(g, o, stride, groups, n);
    const int64_t live = len - g * n;
    return live >= n ? n : (live > 0 ? (int)live : 0);
}

static void gather(const real* src, real* dst, int64_t base, const int64_t* pos, int rows, int ec, int64_t E) {
    for (int o = 0; o < rows; ++o) memcpy(dst + (size_t)o * ec, src + base + pos[o] * E, sizeof(real) * ec);
}

static void scatter(real* dst, const real* src, int64_t base, const int64_t* pos, int rows, int ec, int64_t E) {
    for (int o = 0; o < rows; ++o) memcpy(dst + base + pos[o] * E, src + (size_t)o * ec, sizeof(real) * ec);
}

/* slots rows .. n-1 of a group: dst = src (or zeros when src is NULL) */
static void pass_through(real* dst, const real* src, int64_t base, const int64_t* pos, int rows, int n, int ec,
                         int64_t E) {
    for (int o = rows; o < n; ++o) {
        if (src) memmove(dst + base + pos[o] * E, src + base + pos[o] * E, sizeof(real) * ec);
        else memset(dst + base + pos[o] * E, 0, sizeof(real) * ec);
    }
}

static int64_t entry_len(const int32_t* ctx_len, int64_t b, int64_t N) {
    if (!ctx_len) return N;
    const int64_t v = ctx_len[b];
    return v < 0 ? 0 : (v > N ? N : v);
}

static int bad_shape(int64_t batch, int64_t N, int64_t E, int C, int n) {
    return batch < 1 || N < 1 || E < 1 || C < 1 || n < 1 || n > MAX_N || N % n || E % C || E / C > MAX_EC;
}

/* One stage, x, xa -> y, ya (may alias).  Returns 0, or -1 for a shape this file does not handle. */
int NAME(ncn_ref_stage_forward)(const real* x, const real* xa, real* y, real* ya, const real* W, int64_t batch,
                                int64_t N, int64_t E, int C, int n, int64_t stage, real alpha, real m, int code,
                                int inverse, const int32_t* table, const int32_t* ctx_len) {
    if (bad_shape(batch, N, E, C, n)) return -1;
    const int ec = (int)(E / C);
    const int64_t groups = N / n, stride = stage_stride(stage, groups);
    const int64_t work = batch * C * groups;
#pragma omp parallel for schedule(static)
    for (int64_t w = 0; w < work; ++w) {
        const int64_t g = w % groups, c = (w / groups) % C, b = w / (groups * C);
        const int64_t base = b * N * E + c * ec;
        real gx[MAX_N * MAX_EC], ga[MAX_N * MAX_EC];
        int64_t pos[MAX_N];
        const int rows = group_rows(pos, g, stride, groups, n, table, entry_len(ctx_len, b, N));
        gather(x, gx, base, pos, rows, ec, E);
        gather(xa, ga, base, pos, rows, ec, E);
        const real* wi = W + c * ec;
        const real* wj = W + E + c * ec;
        if (!inverse)
            for (int j = 0; j < rows; ++j) step_forward(gx, ga, wi, wj, rows, ec, j, alpha, m, code);
        else
            for (int j = rows - 1; j >= 0; --j) step_inverse(gx, ga, wi, wj, rows, ec, j, alpha, m, code, 0, 0);
        pass_through(y, x, base, pos, rows, n, ec, E);      /* before the scatter: y may be x */
        pass_through(ya, xa, base, pos, rows, n, ec, E);
        scatter(y, gx, base, pos, rows, ec, E);
        scatter(ya, ga, base, pos, rows, ec, E);
    }
    return 0;
}

/* Reversible backward of one stage from its outputs y, ya and the gradients dy, dya (dya may be NULL = zeros):
 * x_rec, xa_rec (may be NULL) get the stage's inputs, dx, dxa the gradients, dW[2E] (double) the weight gradient. */
int NAME(ncn_ref_stage_backward)(const real* y, const real* ya, const real* dy, const real* dya, const real* W,
                                 real* x_rec, real* xa_rec, real* dx, real* dxa, double* dW, int64_t batch, int64_t N,
                                 int64_t E, int C, int n, int64_t stage, real alpha, real m, int code,
                                 const int32_t* table, const int32_t* ctx_len) {
    if (bad_shape(batch, N, E, C, n)) return -1;
    const int ec = (int)(E / C);
    const int64_t groups = N / n, stride = stage_stride(stage, groups);
    const int64_t work = batch * C * groups;
    int threads = 1;
#ifdef _OPENMP
    threads = omp_get_max_threads();
#endif
    double* acc = (double*)calloc((size_t)threads * 2 * E, sizeof(double));
    if (!acc) return -2;
#pragma omp parallel
    {
        int tid = 0;
#ifdef _OPENMP
        tid = omp_get_thread_num();
#endif
        double* mine = acc + (size_t)tid * 2 * E;
#pragma omp for schedule(static)
        for (int64_t w = 0; w < work; ++w) {
            const int64_t g = w % groups, c = (w / groups) % C, b = w / (groups * C);
            const int64_t base = b * N * E + c * ec;
            real gy[MAX_N * MAX_EC], gb[MAX_N * MAX_EC], gg[MAX_N * MAX_EC], gh[MAX_N * MAX_EC], df[MAX_N * MAX_EC];
            real s[MAX_N], r[MAX_N], dxj[MAX_EC];
            int64_t pos[MAX_N];
            const int rows = group_rows(pos, g, stride, groups, n, table, entry_len(ctx_len, b, N));
            gather(y, gy, base, pos, rows, ec, E);
            gather(ya, gb, base, pos, rows, ec, E);
            gather(dy, gg, base, pos, rows, ec, E);
            if (dya) gather(dya, gh, base, pos, rows, ec, E);
            else memset(gh, 0, sizeof(real) * n * ec);
            const real* wi = W + c * ec;
            const real* wj = W + E + c * ec;
            double* dwi = mine + c * ec;
            double* dwj = mine + E + c * ec;
            for (int j = rows - 1; j >= 0; --j) {
                step_inverse(gy, gb, wi, wj, rows, ec, j, alpha, m, code, s, df);   /* gy, gb: the step's inputs now */
                const real* xj = gy + (size_t)j * ec;
                for (int f = 0; f < ec; ++f) dxj[f] = 0;
                real rsum = 0;
                for (int i = 0; i < rows; ++i) {
                    const real* xi = gy + (size_t)i * ec;
                    real* gi = gg + (size_t)i * ec;
                    real* hi = gh + (size_t)i * ec;
                    real* ui = df + (size_t)i * ec;                               /* dF -> u in place */
                    real ri = 0;
                    for (int f = 0; f < ec; ++f) {
                        ui[f] *= (1 - m) * (1 - m) * gi[f] + (1 - m) * hi[f];     /* u = dL/dT */
                        ri += ui[f] * xj[f];
                    }
                    r[i] = ri;
                    rsum += ri;
                    for (int f = 0; f < ec; ++f) {
                        dwi[f] += (double)((1 - alpha) * ri * xi[f]);
                        dxj[f] += (1 - alpha) * ri * wj[f] + (1 - alpha) * s[i] * ui[f];
                        const real gnew = m * gi[f] + alpha * ui[f] + (1 - alpha) * ri * wi[f];
                        hi[f] = m * (1 - m) * gi[f] + m * hi[f];
                        gi[f] = gnew;
                    }
                }
                for (int f = 0; f < ec; ++f) {
                    dwj[f] += (double)((1 - alpha) * rsum * xj[f]);
                    gg[(size_t)j * ec + f] += dxj[f];
                }
            }
            pass_through(dx, dy, base, pos, rows, n, ec, E);
            pass_through(dxa, dya, base, pos, rows, n, ec, E);
            if (x_rec) pass_through(x_rec, y, base, pos, rows, n, ec, E);
            if (xa_rec) pass_through(xa_rec, ya, base, pos, rows, n, ec, E);
            scatter(dx, gg, base, pos, rows, ec, E);
            scatter(dxa, gh, base, pos, rows, ec, E);
            if (x_rec) scatter(x_rec, gy, base, pos, rows, ec, E);
            if (xa_rec) scatter(xa_rec, gb, base, pos, rows, ec, E);
        }
    }
    for (int64_t k = 0; k < 2 * E; ++k) {
        double sum = 0;
        for (int t = 0; t < threads; ++t) sum += acc[(size_t)t * 2 * E + k];
        dW[k] = sum;
    }
    free(acc);
    return 0;
}

int NAME(ncn_ref_threads)(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
