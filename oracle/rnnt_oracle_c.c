/*
 * rnnt_oracle_c.c -- plain C restatement (float64 arithmetic, OpenMP over the sequences of a batch)
 * of the compact-layout RNN-T loss and gradient.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/ and bench.py's cpu_baseline leg load
 * the library built from it; the shipped package never does and has no CPU path.
 *
 * It follows the same reference lines as oracle/rnnt_oracle.py (paths relative to the
 * CompactWarpRNNTLoss checkout):
 *   cwarp_cuda.cpp:72-77                row offsets = exclusive cumsum of lx*(ly+1)
 *   cwarp_cuda_gather_kernel.cu:29-42   blank / label log-probability of each row
 *   cwarp_cuda_rnnt_kernel.cu:22-29     log_sum_exp = max + log1p(exp(-|a-b|))
 *   cwarp_cuda_rnnt_kernel.cu:59-125    alpha recursion
 *   cwarp_cuda_rnnt_kernel.cu:165-231   beta recursion
 *   cwarp_cuda_rnnt_kernel.cu:286-307   gradient w.r.t. the blank log-probability (t == T-1, u < U left 0)
 *   cwarp_cuda_rnnt_kernel.cu:321-331   gradient w.r.t. the label log-probability
 *   cwarp_cuda_rnnt_kernel.cu:345-366   cost = -beta[0][0], mean of the two likelihoods above 0.1 % mismatch
 *   cwarp_cuda_rnnt_kernel.cu:518-519   per-sequence rescale by grad_out
 *   cwarp_cuda_gather_kernel.cu:62-73   scatter into (R,V), label written after blank
 * plus, in fused mode, the log-softmax the reference's callers apply first (test/test.py:19-20) and
 * its chain rule: d/dx[r,v] = softmax(x_r)[v] * gamma_r + G[r,0] [v==blank] + G[r,1] [v==label].
 *
 * Pinned in tests/test_oracle_pins.py against the NumPy oracle (itself pinned by brute-force path
 * enumeration, closed forms and finite differences) on random ragged batches of both modes.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static double lse2(double a, double b) {
    if (a == -INFINITY && b == -INFINITY) return -INFINITY;
    const double mx = a > b ? a : b, mn = a > b ? b : a;
    return mx + log1p(exp(mn - mx));
}

int rnnt_oracle_c_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/*
 * x (R,V) fp32 row-major; lx, ly (N) int32; y labels: padded (y_stride >= 0: label u of sequence n at
 * y[n*y_stride+u]) or concatenated (y_stride < 0); fused != 0: x holds logits, else log-probs.
 * grad_out (N) or NULL (= ones).  Outputs: costs (N) fp64; G (R,2) fp64 or NULL; grad (R,V) fp32 or
 * NULL.  Returns 0, or 1 when the lengths do not add up to R, 2 when out of memory.
 */
int rnnt_oracle_c_loss_grad(const float* x, int64_t R, int64_t V, const int32_t* lx, const int32_t* ly,
                            const int32_t* y, int64_t y_stride, int32_t N, int32_t blank, int fused,
                            const double* grad_out, double* costs, double* G, float* grad) {
    int64_t* off = (int64_t*)malloc(sizeof(int64_t) * (size_t)(N + 1));
    int64_t* loff = (int64_t*)malloc(sizeof(int64_t) * (size_t)(N + 1));
    if (!off || !loff) { free(off); free(loff); return 2; }
    off[0] = 0; loff[0] = 0;
    for (int n = 0; n < N; ++n) {
        off[n + 1] = off[n] + (int64_t)lx[n] * ((int64_t)ly[n] + 1);
        loff[n + 1] = loff[n] + ly[n];
    }
    if (off[N] != R) { free(off); free(loff); return 1; }
    int failed = 0;
#pragma omp parallel for schedule(dynamic, 1)
    for (int n = 0; n < N; ++n) {
        const int T = lx[n], U = ly[n], Up = U + 1;
        const int64_t cells = (int64_t)T * Up;
        const float* xs = x + off[n] * V;
        const int32_t* lab = y + (y_stride >= 0 ? (int64_t)n * y_stride : loff[n]);
        double* buf = (double*)malloc(sizeof(double) * (size_t)cells * 5);
        if (!buf) {
#pragma omp atomic write
            failed = 1;
            continue;
        }
        double *lse = buf, *B = buf + cells, *L = buf + 2 * cells, *a = buf + 3 * cells, *b = buf + 4 * cells;
        for (int64_t r = 0; r < cells; ++r) {
            const float* row = xs + r * V;
            double l = 0.0;
            if (fused) {
                double m = row[0];
                for (int64_t v = 1; v < V; ++v) if (row[v] > m) m = row[v];
                double s = 0.0;
                for (int64_t v = 0; v < V; ++v) s += exp((double)row[v] - m);
                l = m + log(s);
            }
            lse[r] = l;
            const int u = (int)(r % Up);
            B[r] = (double)row[blank] - l;
            L[r] = u < U ? (double)row[lab[u]] - l : 0.0;
        }
        /* alpha */
        for (int t = 0; t < T; ++t)
            for (int u = 0; u < Up; ++u) {
                const int64_t i = (int64_t)t * Up + u;
                if (t == 0 && u == 0) { a[i] = 0.0; continue; }
                const double skip = t > 0 ? a[i - Up] + B[i - Up] : -INFINITY;
                const double emit = u > 0 ? a[i - 1] + L[i - 1] : -INFINITY;
                a[i] = lse2(skip, emit);
            }
        /* beta */
        for (int t = T - 1; t >= 0; --t)
            for (int u = U; u >= 0; --u) {
                const int64_t i = (int64_t)t * Up + u;
                if (t == T - 1 && u == U) { b[i] = B[i]; continue; }
                const double skip = t < T - 1 ? b[i + Up] + B[i] : -INFINITY;
                const double emit = u < U ? b[i + 1] + L[i] : -INFINITY;
                b[i] = lse2(skip, emit);
            }
        const double b00 = b[0];
        {
            const double fa = a[cells - 1] + B[cells - 1];
            double fb = b00;
            const double larger = fa > fb ? fa : fb;
            if (fabs(fa - fb) / fabs(larger) > 1e-3) fb = 0.5 * (fa + fb);
            costs[n] = -fb;
        }
        const double go = grad_out ? grad_out[n] : 1.0;
        for (int64_t r = 0; r < cells; ++r) {
            const int t = (int)(r / Up), u = (int)(r % Up);
            double gb = 0.0, gl = 0.0;
            if (t < T - 1) gb = -exp(a[r] + b[r + Up] + B[r] - b00);
            else if (u == U) gb = -exp(a[r] + B[r] - b00);
            if (u < U) gl = -exp(a[r] + b[r + 1] + L[r] - b00);
            if (G) { G[2 * (off[n] + r)] = gb; G[2 * (off[n] + r) + 1] = gl; }
            if (grad) {
                float* g = grad + (off[n] + r) * V;
                const float* row = xs + r * V;
                if (fused) {
                    const double gamma = -(gb + gl);
                    for (int64_t v = 0; v < V; ++v) g[v] = (float)(exp((double)row[v] - lse[r]) * gamma * go);
                    g[blank] = (float)((exp((double)row[blank] - lse[r]) * gamma + gb) * go);
                    if (u < U) {
                        const int32_t k = lab[u];
                        const double base = exp((double)row[k] - lse[r]) * gamma + (k == blank ? gb : 0.0);
                        g[k] = (float)((base + gl) * go);
                    }
                } else {
                    memset(g, 0, sizeof(float) * (size_t)V);
                    g[blank] = (float)(gb * go);
                    if (u < U) g[lab[u]] = (float)(gl * go);
                }
            }
        }
        free(buf);
    }
    free(off);
    free(loff);
    return failed ? 2 : 0;
}
