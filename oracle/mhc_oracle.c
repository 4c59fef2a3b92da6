/*
 * CPU oracle for the mHC layer, plain C, double precision: forward and ANALYTIC backward.
 *
 * TEST INFRASTRUCTURE ONLY - nothing in the product library links or loads this file.  It is
 * the loop-level restatement that the HIP kernels' backward algebra is checked against; the
 * oracle's own forward/backward are pinned (tests/test_oracle_*.py) against the PyTorch
 * restatement's autograd, fp64 finite differences and the golden vectors under tests/golden.
 *
 * What it follows in the reference (paths under the reference tree):
 *   forward, dynamic H : src/python/benchmarks/bench_layer.py:123-145 (NaiveMHCLayerDynamic.forward)
 *                        with MHCLayer's weight layout phi_concat [D, nC], rows
 *                        [pre(n) | post(n) | res(n*n, row-major i*n+j)]
 *                        (src/python/mhc/ops.py:173-177, src/csrc/include/utils.cuh:59-89)
 *   forward, static H  : bench_layer.py:59-71 (NaiveMHCLayer.forward)
 *   Sinkhorn-Knopp     : bench_layer.py:48-53 / :112-117 - exp, then T x (row-normalise,
 *                        column-normalise), eps added to every denominator
 *   loop shape         : src/csrc/tests/test_mhc_layer.cu:38-126
 *   backward algebra   : mix/aggregate  src/csrc/tests/test_stream_ops_backward.cu:81-127
 *                        RMSNorm        src/csrc/tests/test_rmsnorm_backward.cu:17-39
 *                        projection     src/python/mhc/ops.py:276-351 (from d_tilde down)
 *                        Sinkhorn       exact reverse sweep through all T iterations (the
 *                        reference's own kernel is an approximation and is not followed)
 *
 * Layouts: x, y, dy, dx [B, n, C] row-major; f, df [B, C]; phi, dphi [D, nC], D = n*n + 2n;
 * bias, dbias [D]; alpha, dalpha [3] = (pre, post, res); w, dw [C].
 * f_inject != NULL selects the kernel-level view (f is an input; dw is not touched, df is
 * written when non-NULL).
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define MAXN 32

static double sigmoid_d(double v) { return 1.0 / (1.0 + exp(-v)); }

/* Sinkhorn forward on exp(t).  Keeps every iterate's scalings: rho[t][r], s[t][c]. */
static void sk_forward(const double *tl, int n, int T, double eps, double *E, double *M,
                       double *rho, double *s)
{
    for (int k = 0; k < n * n; k++) { E[k] = exp(tl[k]); M[k] = E[k]; }
    for (int t = 0; t < T; t++) {
        for (int r = 0; r < n; r++) {
            double sum = 0.0;
            for (int c = 0; c < n; c++) sum += M[r * n + c];
            sum += eps;
            if (rho) rho[t * n + r] = sum;
            for (int c = 0; c < n; c++) M[r * n + c] /= sum;
        }
        for (int c = 0; c < n; c++) {
            double sum = 0.0;
            for (int r = 0; r < n; r++) sum += M[r * n + c];
            sum += eps;
            if (s) s[t * n + c] = sum;
            for (int r = 0; r < n; r++) M[r * n + c] /= sum;
        }
    }
}

/* Exact reverse sweep.  Every iterate is diag(u) E diag(v); the stored scalings rebuild them.
 * In: dM (grad of the final iterate).  Out: dE (grad of exp(t)). */
static void sk_backward(const double *E, const double *M, const double *rho, const double *s,
                        int n, int T, const double *dM, double *dE)
{
    double u[MAXN], v[MAXN], Out[MAXN * MAXN], R[MAXN * MAXN], dOut[MAXN * MAXN], dR[MAXN * MAXN];
    for (int r = 0; r < n; r++) { u[r] = 1.0; v[r] = 1.0; }
    for (int t = 0; t < T; t++)
        for (int r = 0; r < n; r++) { u[r] /= rho[t * n + r]; v[r] /= s[t * n + r]; }
    memcpy(dOut, dM, sizeof(double) * n * n);
    (void)M;
    for (int t = T - 1; t >= 0; t--) {
        /* Out = diag(u) E diag(v) (after column step t); R = Out * s_c (before it) */
        for (int r = 0; r < n; r++)
            for (int c = 0; c < n; c++) {
                Out[r * n + c] = u[r] * E[r * n + c] * v[c];
                R[r * n + c] = Out[r * n + c] * s[t * n + c];
            }
        for (int c = 0; c < n; c++) {
            double dot = 0.0;
            for (int k = 0; k < n; k++) dot += dOut[k * n + c] * Out[k * n + c];
            for (int r = 0; r < n; r++) dR[r * n + c] = (dOut[r * n + c] - dot) / s[t * n + c];
        }
        for (int r = 0; r < n; r++) {
            double dot = 0.0;
            for (int k = 0; k < n; k++) dot += dR[r * n + k] * R[r * n + k];
            for (int c = 0; c < n; c++) dOut[r * n + c] = (dR[r * n + c] - dot) / rho[t * n + r];
        }
        for (int r = 0; r < n; r++) { u[r] *= rho[t * n + r]; v[r] *= s[t * n + r]; }
    }
    memcpy(dE, dOut, sizeof(double) * n * n);
}

/* Per-sample coefficients from logits t[D]: Hpre, Hpost, E, M (+ scalings). */
static void coefficients(const double *t, int n, int T, double eps, double *Hpre, double *Hpost,
                         double *E, double *M, double *rho, double *s)
{
    for (int i = 0; i < n; i++) {
        Hpre[i] = sigmoid_d(t[i]);
        Hpost[i] = 2.0 * sigmoid_d(t[n + i]);
    }
    sk_forward(t + 2 * n, n, T, eps, E, M, rho, s);
}

/* Mix/aggregate/RMSNorm forward of one sample.  Returns q (inner rms); a, f are [C] scratch. */
static double sample_forward(const double *x, const double *w, const double *f_inject, int n,
                             int C, double eps, const double *Hpre, const double *Hpost,
                             const double *M, double *a, double *f, double *y)
{
    double ssq = 0.0;
    for (int c = 0; c < C; c++) {
        double acc = 0.0;
        for (int i = 0; i < n; i++) acc += Hpre[i] * x[i * C + c];
        a[c] = acc;
        ssq += acc * acc;
    }
    double q = sqrt(ssq / C + eps);
    for (int c = 0; c < C; c++) f[c] = f_inject ? f_inject[c] : a[c] / q * w[c];
    for (int i = 0; i < n; i++)
        for (int c = 0; c < C; c++) {
            double acc = 0.0;
            for (int j = 0; j < n; j++) acc += M[i * n + j] * x[j * C + c];
            y[i * C + c] = acc + Hpost[i] * f[c];
        }
    return q;
}

/* Mix/aggregate/RMSNorm backward of one sample.  dx is written (not accumulated);
 * dw is accumulated; dM [n*n], dHpre, dHpost [n] are written. */
static void sample_backward(const double *x, const double *G, const double *w, int injected,
                            int n, int C, double q, const double *Hpre, const double *Hpost,
                            const double *M, const double *a, const double *f, double *dx,
                            double *df_out, double *dw, double *dM, double *dHpre, double *dHpost,
                            double *da /* [C] scratch */)
{
    for (int i = 0; i < n; i++) {
        for (int j = 0; j < n; j++) {
            double acc = 0.0;
            for (int c = 0; c < C; c++) acc += G[i * C + c] * x[j * C + c];
            dM[i * n + j] = acc;
        }
        double acc = 0.0;
        for (int c = 0; c < C; c++) acc += G[i * C + c] * f[c];
        dHpost[i] = acc;
    }
    double s1 = 0.0;
    for (int c = 0; c < C; c++) {
        double df = 0.0;
        for (int i = 0; i < n; i++) df += Hpost[i] * G[i * C + c];
        if (df_out) df_out[c] = df;
        if (injected) {
            da[c] = 0.0;
        } else {
            dw[c] += df * a[c] / q;
            da[c] = df * w[c]; /* g' for now */
            s1 += da[c] * a[c];
        }
    }
    if (!injected)
        for (int c = 0; c < C; c++) da[c] = da[c] / q - a[c] * s1 / ((double)C * q * q * q);
    for (int j = 0; j < n; j++) {
        double acc = 0.0;
        for (int c = 0; c < C; c++) {
            double mix = 0.0;
            for (int i = 0; i < n; i++) mix += M[i * n + j] * G[i * C + c];
            dx[j * C + c] = mix + Hpre[j] * da[c];
            acc += da[c] * x[j * C + c];
        }
        dHpre[j] = acc;
    }
}

/* ------------------------------------------------------------------------------------------
 * dynamic H
 * ---------------------------------------------------------------------------------------- */
int mhc_oracle_dynamic_forward(const double *x, const double *w, const double *phi,
                               const double *bias, const double *alpha, const double *f_inject,
                               int B, int n, int C, int T, double eps, double *y,
                               double *Hpre_out, double *Hpost_out, double *M_out)
{
    if (n < 1 || n > MAXN) return 1;
    int nC = n * C, D = n * n + 2 * n;
    double *a = malloc(sizeof(double) * C), *f = malloc(sizeof(double) * C);
    double *t = malloc(sizeof(double) * D);
    double Hpre[MAXN], Hpost[MAXN], E[MAXN * MAXN], M[MAXN * MAXN];
    for (int b = 0; b < B; b++) {
        const double *xb = x + (size_t)b * nC;
        double ssq = 0.0;
        for (int k = 0; k < nC; k++) ssq += xb[k] * xb[k];
        double r = sqrt(ssq / nC + eps);
        for (int d = 0; d < D; d++) {
            double acc = 0.0;
            for (int k = 0; k < nC; k++) acc += (xb[k] / r) * phi[(size_t)d * nC + k];
            double al = d < n ? alpha[0] : (d < 2 * n ? alpha[1] : alpha[2]);
            t[d] = al * acc + bias[d];
        }
        coefficients(t, n, T, eps, Hpre, Hpost, E, M, NULL, NULL);
        sample_forward(xb, w, f_inject ? f_inject + (size_t)b * C : NULL, n, C, eps, Hpre, Hpost,
                       M, a, f, y + (size_t)b * nC);
        if (Hpre_out) memcpy(Hpre_out + b * n, Hpre, sizeof(double) * n);
        if (Hpost_out) memcpy(Hpost_out + b * n, Hpost, sizeof(double) * n);
        if (M_out) memcpy(M_out + (size_t)b * n * n, M, sizeof(double) * n * n);
    }
    free(a); free(f); free(t);
    return 0;
}

int mhc_oracle_dynamic_backward(const double *x, const double *dy, const double *w,
                                const double *phi, const double *bias, const double *alpha,
                                const double *f_inject, int B, int n, int C, int T, double eps,
                                double *dx, double *df, double *dw, double *dphi, double *dbias,
                                double *dalpha)
{
    if (n < 1 || n > MAXN) return 1;
    int nC = n * C, D = n * n + 2 * n;
    double *a = malloc(sizeof(double) * C), *f = malloc(sizeof(double) * C);
    double *da = malloc(sizeof(double) * C), *yb = malloc(sizeof(double) * nC);
    double *t = malloc(sizeof(double) * D), *p = malloc(sizeof(double) * D);
    double *dt = malloc(sizeof(double) * D), *dP = malloc(sizeof(double) * D);
    double *rho = malloc(sizeof(double) * (T > 0 ? T : 1) * n);
    double *s = malloc(sizeof(double) * (T > 0 ? T : 1) * n);
    double Hpre[MAXN], Hpost[MAXN], E[MAXN * MAXN], M[MAXN * MAXN];
    double dM[MAXN * MAXN], dE[MAXN * MAXN], dHpre[MAXN], dHpost[MAXN];
    if (dw) memset(dw, 0, sizeof(double) * C);
    memset(dphi, 0, sizeof(double) * (size_t)D * nC);
    memset(dbias, 0, sizeof(double) * D);
    dalpha[0] = dalpha[1] = dalpha[2] = 0.0;
    for (int b = 0; b < B; b++) {
        const double *xb = x + (size_t)b * nC;
        const double *Gb = dy + (size_t)b * nC;
        double ssq = 0.0;
        for (int k = 0; k < nC; k++) ssq += xb[k] * xb[k];
        double r = sqrt(ssq / nC + eps);
        for (int d = 0; d < D; d++) {
            double acc = 0.0;
            for (int k = 0; k < nC; k++) acc += xb[k] * phi[(size_t)d * nC + k];
            p[d] = acc / r; /* x_norm . phi_d */
            double al = d < n ? alpha[0] : (d < 2 * n ? alpha[1] : alpha[2]);
            t[d] = al * p[d] + bias[d];
        }
        coefficients(t, n, T, eps, Hpre, Hpost, E, M, rho, s);
        double q = sample_forward(xb, w, f_inject ? f_inject + (size_t)b * C : NULL, n, C, eps,
                                  Hpre, Hpost, M, a, f, yb);
        sample_backward(xb, Gb, w, f_inject != NULL, n, C, q, Hpre, Hpost, M, a, f,
                        dx + (size_t)b * nC, df ? df + (size_t)b * C : NULL, dw, dM, dHpre,
                        dHpost, da);
        sk_backward(E, M, rho, s, n, T, dM, dE);
        for (int i = 0; i < n; i++) {
            dt[i] = dHpre[i] * Hpre[i] * (1.0 - Hpre[i]);
            dt[n + i] = dHpost[i] * Hpost[i] * (1.0 - Hpost[i] / 2.0);
        }
        for (int k = 0; k < n * n; k++) dt[2 * n + k] = dE[k] * E[k];
        /* t = alpha * p + bias, p = (x . phi_d) / r */
        double corr = 0.0; /* sum_d dt_d alpha_d p_d */
        for (int d = 0; d < D; d++) {
            int g = d < n ? 0 : (d < 2 * n ? 1 : 2);
            dbias[d] += dt[d];
            dalpha[g] += dt[d] * p[d];
            dP[d] = dt[d] * alpha[g] / r; /* grad wrt raw dot product x . phi_d */
            corr += dt[d] * alpha[g] * p[d];
        }
        /* d/dx of p_d = phi_d / r - (x . phi_d) x / (nC r^3) */
        double cx = corr / ((double)nC * r * r);
        for (int k = 0; k < nC; k++) {
            double acc = 0.0;
            for (int d = 0; d < D; d++) acc += dP[d] * phi[(size_t)d * nC + k];
            dx[(size_t)b * nC + k] += acc - cx * xb[k];
        }
        for (int d = 0; d < D; d++)
            for (int k = 0; k < nC; k++) dphi[(size_t)d * nC + k] += dP[d] * xb[k];
    }
    free(a); free(f); free(da); free(yb); free(t); free(p); free(dt); free(dP); free(rho); free(s);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * static H: logits[D] shared by all samples (same row order as the dynamic bias vector)
 * ---------------------------------------------------------------------------------------- */
int mhc_oracle_static_forward(const double *x, const double *w, const double *logits,
                              const double *f_inject, int B, int n, int C, int T, double eps,
                              double *y, double *Hpre_out, double *Hpost_out, double *M_out)
{
    if (n < 1 || n > MAXN) return 1;
    int nC = n * C;
    double *a = malloc(sizeof(double) * C), *f = malloc(sizeof(double) * C);
    double Hpre[MAXN], Hpost[MAXN], E[MAXN * MAXN], M[MAXN * MAXN];
    coefficients(logits, n, T, eps, Hpre, Hpost, E, M, NULL, NULL);
    for (int b = 0; b < B; b++)
        sample_forward(x + (size_t)b * nC, w, f_inject ? f_inject + (size_t)b * C : NULL, n, C,
                       eps, Hpre, Hpost, M, a, f, y + (size_t)b * nC);
    if (Hpre_out) memcpy(Hpre_out, Hpre, sizeof(double) * n);
    if (Hpost_out) memcpy(Hpost_out, Hpost, sizeof(double) * n);
    if (M_out) memcpy(M_out, M, sizeof(double) * n * n);
    free(a); free(f);
    return 0;
}

int mhc_oracle_static_backward(const double *x, const double *dy, const double *w,
                               const double *logits, const double *f_inject, int B, int n, int C,
                               int T, double eps, double *dx, double *df, double *dw,
                               double *dlogits)
{
    if (n < 1 || n > MAXN) return 1;
    int nC = n * C, D = n * n + 2 * n;
    double *a = malloc(sizeof(double) * C), *f = malloc(sizeof(double) * C);
    double *da = malloc(sizeof(double) * C), *yb = malloc(sizeof(double) * nC);
    double *rho = malloc(sizeof(double) * (T > 0 ? T : 1) * n);
    double *s = malloc(sizeof(double) * (T > 0 ? T : 1) * n);
    double Hpre[MAXN], Hpost[MAXN], E[MAXN * MAXN], M[MAXN * MAXN];
    double dM[MAXN * MAXN], dE[MAXN * MAXN], dHpre[MAXN], dHpost[MAXN];
    double dMs[MAXN * MAXN], dHpres[MAXN], dHposts[MAXN];
    memset(dMs, 0, sizeof dMs); memset(dHpres, 0, sizeof dHpres); memset(dHposts, 0, sizeof dHposts);
    if (dw) memset(dw, 0, sizeof(double) * C);
    coefficients(logits, n, T, eps, Hpre, Hpost, E, M, rho, s);
    for (int b = 0; b < B; b++) {
        const double *xb = x + (size_t)b * nC;
        double q = sample_forward(xb, w, f_inject ? f_inject + (size_t)b * C : NULL, n, C, eps,
                                  Hpre, Hpost, M, a, f, yb);
        sample_backward(xb, dy + (size_t)b * nC, w, f_inject != NULL, n, C, q, Hpre, Hpost, M, a,
                        f, dx + (size_t)b * nC, df ? df + (size_t)b * C : NULL, dw, dM, dHpre,
                        dHpost, da);
        for (int k = 0; k < n * n; k++) dMs[k] += dM[k];
        for (int i = 0; i < n; i++) { dHpres[i] += dHpre[i]; dHposts[i] += dHpost[i]; }
    }
    sk_backward(E, M, rho, s, n, T, dMs, dE);
    for (int i = 0; i < n; i++) {
        dlogits[i] = dHpres[i] * Hpre[i] * (1.0 - Hpre[i]);
        dlogits[n + i] = dHposts[i] * Hpost[i] * (1.0 - Hpost[i] / 2.0);
    }
    for (int k = 0; k < n * n; k++) dlogits[2 * n + k] = dE[k] * E[k];
    (void)D;
    free(a); free(f); free(da); free(yb); free(rho); free(s);
    return 0;
}

/* ------------------------------------------------------------------------------------------------
 * Stand-alone operators (loop-level restatements of the reference's own CPU references).
 *   Sinkhorn-Knopp, threshold form: src/csrc/tests/test_sinkhorn_knopp.cu:16-47 - no exp, T x (every
 *     row divided by its sum if the sum exceeds eps, then every column likewise), any rows x cols.
 *     The backward is the exact reverse sweep of that recursion (a row / column that was not
 *     divided passes its gradient through unchanged).
 *   RMSNorm: src/csrc/tests/test_rmsnorm.cu:17-30 (forward) and
 *     src/csrc/tests/test_rmsnorm_backward.cu:17-39 (backward from the saved rms).
 * Pinned in tests/test_oracle_math.py: one-iteration closed forms on a non-square matrix, the
 * PyTorch restatement, torch.nn.functional.rms_norm and central differences.
 * ---------------------------------------------------------------------------------------------- */
int mhc_oracle_sinkhorn_plain_forward(const double *inp, double *out, int rows, int cols, int T, double eps) {
    memcpy(out, inp, sizeof(double) * (size_t)rows * cols);
    for (int t = 0; t < T; t++) {
        for (int r = 0; r < rows; r++) {
            double s = 0.0;
            for (int c = 0; c < cols; c++) s += out[r * cols + c];
            if (s > eps)
                for (int c = 0; c < cols; c++) out[r * cols + c] /= s;
        }
        for (int c = 0; c < cols; c++) {
            double s = 0.0;
            for (int r = 0; r < rows; r++) s += out[r * cols + c];
            if (s > eps)
                for (int r = 0; r < rows; r++) out[r * cols + c] /= s;
        }
    }
    return 0;
}

int mhc_oracle_sinkhorn_plain_backward(const double *grad_out, const double *inp, double *d_inp, int rows,
                                       int cols, int T, double eps) {
    const size_t sz = (size_t)rows * cols;
    /* iterates: A[t] = input of iteration t, R[t] = after the row step; sums kept per iteration */
    double *A = (double *)malloc(sizeof(double) * sz * (size_t)(T + 1));
    double *R = (double *)malloc(sizeof(double) * sz * (size_t)(T > 0 ? T : 1));
    double *rs = (double *)malloc(sizeof(double) * (size_t)rows * (size_t)(T > 0 ? T : 1));
    double *cs = (double *)malloc(sizeof(double) * (size_t)cols * (size_t)(T > 0 ? T : 1));
    if (!A || !R || !rs || !cs) { free(A); free(R); free(rs); free(cs); return 1; }
    memcpy(A, inp, sizeof(double) * sz);
    for (int t = 0; t < T; t++) {
        const double *a = A + sz * t;
        double *rr = R + sz * t, *o = A + sz * (t + 1);
        for (int r = 0; r < rows; r++) {
            double s = 0.0;
            for (int c = 0; c < cols; c++) s += a[r * cols + c];
            rs[t * rows + r] = s;
            for (int c = 0; c < cols; c++) rr[r * cols + c] = s > eps ? a[r * cols + c] / s : a[r * cols + c];
        }
        for (int c = 0; c < cols; c++) {
            double s = 0.0;
            for (int r = 0; r < rows; r++) s += rr[r * cols + c];
            cs[t * cols + c] = s;
            for (int r = 0; r < rows; r++) o[r * cols + c] = s > eps ? rr[r * cols + c] / s : rr[r * cols + c];
        }
    }
    double *d = d_inp;
    memcpy(d, grad_out, sizeof(double) * sz);
    for (int t = T - 1; t >= 0; t--) {
        const double *o = A + sz * (t + 1), *rr = R + sz * t;
        for (int c = 0; c < cols; c++) {   /* o = rr / s: d_rr = (d_o - sum_k d_o o) / s */
            const double s = cs[t * cols + c];
            if (!(s > eps)) continue;
            double dot = 0.0;
            for (int r = 0; r < rows; r++) dot += d[r * cols + c] * o[r * cols + c];
            for (int r = 0; r < rows; r++) d[r * cols + c] = (d[r * cols + c] - dot) / s;
        }
        for (int r = 0; r < rows; r++) {
            const double s = rs[t * rows + r];
            if (!(s > eps)) continue;
            double dot = 0.0;
            for (int c = 0; c < cols; c++) dot += d[r * cols + c] * rr[r * cols + c];
            for (int c = 0; c < cols; c++) d[r * cols + c] = (d[r * cols + c] - dot) / s;
        }
    }
    free(A); free(R); free(rs); free(cs);
    return 0;
}

int mhc_oracle_rmsnorm_forward(const double *inp, const double *w, double *out, double *rms, int rows, int C,
                               double eps) {
    for (int i = 0; i < rows; i++) {
        double ss = 0.0;
        for (int j = 0; j < C; j++) ss += inp[(size_t)i * C + j] * inp[(size_t)i * C + j];
        const double r = sqrt(ss / (double)C + eps);
        if (rms) rms[i] = r;
        for (int j = 0; j < C; j++) out[(size_t)i * C + j] = inp[(size_t)i * C + j] / r * w[j];
    }
    return 0;
}

int mhc_oracle_rmsnorm_backward(const double *grad, const double *inp, const double *w, const double *rms,
                                double *d_inp, double *d_w, int rows, int C) {
    for (int j = 0; j < C; j++) d_w[j] = 0.0;
    for (int i = 0; i < rows; i++) {
        const double r = rms[i], rinv = 1.0 / r;
        double dot = 0.0;
        for (int j = 0; j < C; j++) dot += grad[(size_t)i * C + j] * w[j] * inp[(size_t)i * C + j];
        const double corr = dot / ((double)C * r * r);
        for (int j = 0; j < C; j++) {
            d_inp[(size_t)i * C + j] = grad[(size_t)i * C + j] * w[j] * rinv - inp[(size_t)i * C + j] * corr * rinv;
            d_w[j] += grad[(size_t)i * C + j] * inp[(size_t)i * C + j] * rinv;
        }
    }
    return 0;
}
