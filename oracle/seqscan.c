/*
 * ORACLE (test infrastructure, not part of the product).
 *
 * The recurrences of the scan operator written as the plain sequential loops
 * that define them, evaluated in double precision from fp32 inputs.  This is
 * the "truth" both the GPU kernels and the torch tree scan (oracle/ref_scan.py)
 * are measured against.  Formulas as the reference states them:
 *   forward            accelerated_scan/warp.py:71-74,  scalar.py:28-45
 *   reverse            accelerated_scan/ref.py:100-102,116-118 (used at tests/test_eq.py:77-78)
 *   backward (real)    accelerated_scan/scalar.py:48-86, tests/test_eq.py:77-80
 *   backward (complex) accelerated_scan/complex.py:79-92,113-115,141-147
 * Rows are independent; OpenMP runs them in parallel.
 */
#include <math.h>
#include <stdint.h>

/* out[r,t] = g[r,t] * out[r,t-1] + x[r,t]   (reverse: t+1 in place of t-1) */
void seq_forward_f32(const float* g, const float* x, double* out, int64_t rows, int64_t T, int reverse) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* gr = g + r * T;
        const float* xr = x + r * T;
        double* o = out + r * T;
        double s = 0.0;
        if (!reverse) {
            for (int64_t t = 0; t < T; ++t) {
                s = (double)gr[t] * s + (double)xr[t];
                o[t] = s;
            }
        } else {
            for (int64_t t = T - 1; t >= 0; --t) {
                s = (double)gr[t] * s + (double)xr[t];
                o[t] = s;
            }
        }
    }
}

/*
 * Adjoint of the forward recurrence for an incoming gradient dout:
 *   a[t]  = dout[t] + g[t+1] * a[t+1],  a[T] = 0
 *   dx[t] = a[t]
 *   dg[t] = a[t] * state[t-1],          state[-1] = 0
 * `state` is the forward output (fp32, as the product kernel receives it).
 */
void seq_backward_f32(const float* g, const float* state, const float* dout, double* dg, double* dx,
                      int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* gr = g + r * T;
        const float* sr = state + r * T;
        const float* dr = dout + r * T;
        double* dgr = dg + r * T;
        double* dxr = dx + r * T;
        double a = 0.0;
        for (int64_t t = T - 1; t >= 0; --t) {
            const double gnext = (t + 1 < T) ? (double)gr[t + 1] : 1.0;
            a = (double)dr[t] + gnext * a;
            dxr[t] = a;
            dgr[t] = a * ((t > 0) ? (double)sr[t - 1] : 0.0);
        }
    }
}

/* Complex versions; arrays are interleaved (re, im). */
void seq_forward_c64(const float* g, const float* x, double* out, int64_t rows, int64_t T, int reverse) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* gr = g + 2 * r * T;
        const float* xr = x + 2 * r * T;
        double* o = out + 2 * r * T;
        double sr = 0.0, si = 0.0;
        for (int64_t k = 0; k < T; ++k) {
            const int64_t t = reverse ? T - 1 - k : k;
            const double a = gr[2 * t], b = gr[2 * t + 1];
            const double nr = a * sr - b * si + (double)xr[2 * t];
            const double ni = a * si + b * sr + (double)xr[2 * t + 1];
            sr = nr;
            si = ni;
            o[2 * t] = sr;
            o[2 * t + 1] = si;
        }
    }
}

/*
 *   a[t]  = dout[t] + conj(g[t+1]) * a[t+1]
 *   dx[t] = a[t]
 *   dg[t] = a[t] * conj(state[t-1])
 */
void seq_backward_c64(const float* g, const float* state, const float* dout, double* dg, double* dx,
                      int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* gr = g + 2 * r * T;
        const float* sr = state + 2 * r * T;
        const float* dr = dout + 2 * r * T;
        double* dgr = dg + 2 * r * T;
        double* dxr = dx + 2 * r * T;
        double ar = 0.0, ai = 0.0;
        for (int64_t t = T - 1; t >= 0; --t) {
            double cr = 1.0, ci = 0.0; /* conj(g[t+1]) */
            if (t + 1 < T) {
                cr = gr[2 * (t + 1)];
                ci = -(double)gr[2 * (t + 1) + 1];
            }
            const double nr = (double)dr[2 * t] + cr * ar - ci * ai;
            const double ni = (double)dr[2 * t + 1] + cr * ai + ci * ar;
            ar = nr;
            ai = ni;
            dxr[2 * t] = ar;
            dxr[2 * t + 1] = ai;
            double pr = 0.0, pi = 0.0; /* conj(state[t-1]) */
            if (t > 0) {
                pr = sr[2 * (t - 1)];
                pi = -(double)sr[2 * (t - 1) + 1];
            }
            dgr[2 * t] = ar * pr - ai * pi;
            dgr[2 * t + 1] = ar * pi + ai * pr;
        }
    }
}

/*
 * Scans that start from a given state (one per row), for sequences processed in
 * chunks.  The reference always starts from zero (warp.cuh:76, scalar.py:28,
 * complex.py:32-33); these restate the same recurrences with x[-1] = init[r]:
 *   forward :  out[r,-1] = init[r]   (reverse: out[r,T] = init[r])
 *   backward:  dg[r,0]  = a[0] * conj(init[r]),   dinit[r] = conj(g[r,0]) * a[0]
 * Pinned by tests/test_oracle.py: equality with the zero-start functions above
 * for init = 0, the chunking identity (a scan cut in two, the second half
 * started from the first half's last state, equals the uncut scan, values and
 * gradients), and torch autograd through the plain loop in float64.
 */
void seq_forward_from_f32(const float* g, const float* x, const float* init, double* out, int64_t rows, int64_t T,
                          int reverse) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* gr = g + r * T;
        const float* xr = x + r * T;
        double* o = out + r * T;
        double s = init ? (double)init[r] : 0.0;
        for (int64_t k = 0; k < T; ++k) {
            const int64_t t = reverse ? T - 1 - k : k;
            s = (double)gr[t] * s + (double)xr[t];
            o[t] = s;
        }
    }
}

void seq_backward_from_f32(const float* g, const float* state, const float* init, const float* dout, double* dg,
                           double* dx, double* dinit, int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* gr = g + r * T;
        const float* sr = state + r * T;
        const float* dr = dout + r * T;
        double* dgr = dg + r * T;
        double* dxr = dx + r * T;
        const double x0 = init ? (double)init[r] : 0.0;
        double a = 0.0;
        for (int64_t t = T - 1; t >= 0; --t) {
            const double gnext = (t + 1 < T) ? (double)gr[t + 1] : 1.0;
            a = (double)dr[t] + gnext * a;
            dxr[t] = a;
            dgr[t] = a * ((t > 0) ? (double)sr[t - 1] : x0);
        }
        if (dinit) dinit[r] = (T > 0) ? (double)gr[0] * a : 0.0;
    }
}

void seq_forward_from_c64(const float* g, const float* x, const float* init, double* out, int64_t rows, int64_t T,
                          int reverse) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* gr = g + 2 * r * T;
        const float* xr = x + 2 * r * T;
        double* o = out + 2 * r * T;
        double sr = init ? (double)init[2 * r] : 0.0, si = init ? (double)init[2 * r + 1] : 0.0;
        for (int64_t k = 0; k < T; ++k) {
            const int64_t t = reverse ? T - 1 - k : k;
            const double a = gr[2 * t], b = gr[2 * t + 1];
            const double nr = a * sr - b * si + (double)xr[2 * t];
            const double ni = a * si + b * sr + (double)xr[2 * t + 1];
            sr = nr;
            si = ni;
            o[2 * t] = sr;
            o[2 * t + 1] = si;
        }
    }
}

void seq_backward_from_c64(const float* g, const float* state, const float* init, const float* dout, double* dg,
                           double* dx, double* dinit, int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* gr = g + 2 * r * T;
        const float* sr = state + 2 * r * T;
        const float* dr = dout + 2 * r * T;
        double* dgr = dg + 2 * r * T;
        double* dxr = dx + 2 * r * T;
        const double x0r = init ? (double)init[2 * r] : 0.0, x0i = init ? (double)init[2 * r + 1] : 0.0;
        double ar = 0.0, ai = 0.0;
        for (int64_t t = T - 1; t >= 0; --t) {
            double cr = 1.0, ci = 0.0; /* conj(g[t+1]) */
            if (t + 1 < T) {
                cr = gr[2 * (t + 1)];
                ci = -(double)gr[2 * (t + 1) + 1];
            }
            const double nr = (double)dr[2 * t] + cr * ar - ci * ai;
            const double ni = (double)dr[2 * t + 1] + cr * ai + ci * ar;
            ar = nr;
            ai = ni;
            dxr[2 * t] = ar;
            dxr[2 * t + 1] = ai;
            double pr = x0r, pi = -x0i; /* conj(state[t-1]) */
            if (t > 0) {
                pr = sr[2 * (t - 1)];
                pi = -(double)sr[2 * (t - 1) + 1];
            }
            dgr[2 * t] = ar * pr - ai * pi;
            dgr[2 * t + 1] = ar * pi + ai * pr;
        }
        if (dinit) {
            /* conj(g[0]) * a[0] */
            const double cr = (T > 0) ? (double)gr[0] : 0.0, ci = (T > 0) ? -(double)gr[1] : 0.0;
            dinit[2 * r] = cr * ar - ci * ai;
            dinit[2 * r + 1] = cr * ai + ci * ar;
        }
    }
}

/*
 * Scans whose gates are the sigmoid of stored pre-activations, gradient with
 * respect to the pre-activations (no counterpart in the reference, which is
 * handed finished gates):
 *   gate[t] = 1 / (1 + exp(-z[t])),  out[t] = gate[t] * out[t-1] + x[t],  out[-1] = init
 *   dz[t]   = a[t] * state[t-1] * gate[t] * (1 - gate[t]),  dinit = gate[0] * a[0]
 * Pinned by tests/test_oracle.py: torch autograd through the plain float64 loop
 * with torch.sigmoid, the zero-start functions above on gates rounded to fp32,
 * and closed forms (z = 0 gives the geometric series of ratio 1/2).
 */
static double sigmoid64(double z) { return 1.0 / (1.0 + exp(-z)); }

void seq_forward_sigmoid_f32(const float* z, const float* x, const float* init, double* out, int64_t rows,
                             int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        double s = init ? (double)init[r] : 0.0;
        for (int64_t t = 0; t < T; ++t) {
            s = sigmoid64((double)z[r * T + t]) * s + (double)x[r * T + t];
            out[r * T + t] = s;
        }
    }
}

void seq_backward_sigmoid_f32(const float* z, const float* state, const float* init, const float* dout, double* dz,
                              double* dx, double* dinit, int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* zr = z + r * T;
        const float* sr = state + r * T;
        const double x0 = init ? (double)init[r] : 0.0;
        double a = 0.0;
        for (int64_t t = T - 1; t >= 0; --t) {
            const double gnext = (t + 1 < T) ? sigmoid64((double)zr[t + 1]) : 1.0;
            a = (double)dout[r * T + t] + gnext * a;
            dx[r * T + t] = a;
            const double gate = sigmoid64((double)zr[t]);
            dz[r * T + t] = a * ((t > 0) ? (double)sr[t - 1] : x0) * gate * (1.0 - gate);
        }
        if (dinit) dinit[r] = (T > 0) ? sigmoid64((double)zr[0]) * a : 0.0;
    }
}

/*
 * Scans whose gates are the exponential of stored logarithms (no counterpart
 * in the reference, which is handed finished gates):
 *   gate[t] = exp(z[t]),  out[t] = gate[t] * out[t-1] + x[t],  out[-1] = init
 *   a[t] = dout[t] + gate[t+1] * a[t+1],  dx = a,
 *   dz[t] = a[t] * state[t-1] * gate[t],  dinit = gate[0] * a[0]
 * Pinned by tests/test_oracle.py: torch autograd through the plain float64 loop
 * with torch.exp, the zero-start functions above on gates formed in float64,
 * and closed forms (constant z = log q gives the geometric series of ratio q;
 * x = delta at 0 gives exp of the running sum of z).
 */
void seq_forward_exp_f32(const float* z, const float* x, const float* init, double* out, int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        double s = init ? (double)init[r] : 0.0;
        for (int64_t t = 0; t < T; ++t) {
            s = exp((double)z[r * T + t]) * s + (double)x[r * T + t];
            out[r * T + t] = s;
        }
    }
}

void seq_backward_exp_f32(const float* z, const float* state, const float* init, const float* dout, double* dz,
                          double* dx, double* dinit, int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* zr = z + r * T;
        const float* sr = state + r * T;
        const double x0 = init ? (double)init[r] : 0.0;
        double a = 0.0;
        for (int64_t t = T - 1; t >= 0; --t) {
            const double gnext = (t + 1 < T) ? exp((double)zr[t + 1]) : 1.0;
            a = (double)dout[r * T + t] + gnext * a;
            dx[r * T + t] = a;
            dz[r * T + t] = a * ((t > 0) ? (double)sr[t - 1] : x0) * exp((double)zr[t]);
        }
        if (dinit) dinit[r] = (T > 0) ? exp((double)zr[0]) * a : 0.0;
    }
}

/*
 * Gated interpolation (no counterpart in the reference): the gate is the
 * sigmoid of a stored pre-activation and the token its complement times a
 * stored value,
 *   a[t] = 1 / (1 + exp(-z[t])),  out[t] = a[t] * out[t-1] + (1 - a[t]) * v[t],  out[-1] = init
 *   g[t] = dout[t] + a[t+1] * g[t+1]
 *   dv[t] = g[t] * (1 - a[t]),  dz[t] = g[t] * (state[t-1] - v[t]) * a[t] * (1 - a[t]),  dinit = a[0] * g[0]
 * 1 - a is taken as 1 / (1 + exp(z)), which keeps its relative accuracy for
 * large z.  Pinned by tests/test_oracle.py: torch autograd through the plain
 * float64 loop with torch.sigmoid and torch.lerp, the sigmoid functions above
 * on tokens (1 - sigmoid(z)) * v formed in float64, and closed forms (constant
 * v gives out = v for init = v; z = 0 gives the running average with weights
 * 2^-(k+1)).
 */
void seq_forward_lerp_f32(const float* z, const float* v, const float* init, double* out, int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        double s = init ? (double)init[r] : 0.0;
        for (int64_t t = 0; t < T; ++t) {
            const double zt = (double)z[r * T + t];
            s = sigmoid64(zt) * s + sigmoid64(-zt) * (double)v[r * T + t];
            out[r * T + t] = s;
        }
    }
}

void seq_backward_lerp_f32(const float* z, const float* v, const float* state, const float* init, const float* dout,
                           double* dz, double* dv, double* dinit, int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* zr = z + r * T;
        const float* vr = v + r * T;
        const float* sr = state + r * T;
        const double x0 = init ? (double)init[r] : 0.0;
        double g = 0.0;
        for (int64_t t = T - 1; t >= 0; --t) {
            const double gnext = (t + 1 < T) ? sigmoid64((double)zr[t + 1]) : 1.0;
            g = (double)dout[r * T + t] + gnext * g;
            const double a = sigmoid64((double)zr[t]), rest = sigmoid64(-(double)zr[t]);
            dv[r * T + t] = g * rest;
            dz[r * T + t] = g * (((t > 0) ? (double)sr[t - 1] : x0) - (double)vr[t]) * a * rest;
        }
        if (dinit) dinit[r] = (T > 0) ? sigmoid64((double)zr[0]) * g : 0.0;
    }
}

/*
 * Exponential gate with a variance-preserving input scale (no counterpart in
 * the reference; the update of RG-LRU / Hawk-style layers): the gate is the
 * exponential of a stored logarithm z <= 0 and the token the stored value
 * times sqrt(1 - gate^2),
 *   a[t] = exp(z[t]),  b[t] = sqrt(1 - a[t]^2),  out[t] = a[t] * out[t-1] + b[t] * v[t],  out[-1] = init
 *   g[t] = dout[t] + a[t+1] * g[t+1]
 *   dv[t] = g[t] * b[t],  dz[t] = g[t] * (a[t] * state[t-1] - v[t] * a[t]^2 / b[t]),  dinit = a[0] * g[0]
 * 1 - a^2 is taken as -expm1(2 z), which keeps its relative accuracy for z
 * close to 0 (clamped at 0 for z > 0).  Pinned by tests/test_oracle.py: torch
 * autograd through the plain float64 loop with torch.exp, torch.expm1 and
 * torch.sqrt, the exponential-gate functions above on tokens b * v formed in
 * float64 plus the chain rule, and closed forms (a = 0.6 gives b = 0.8; a
 * constant value c tends to c * sqrt((1 + a) / (1 - a)); z = -800 returns the values).
 */
static double expnorm_scale(double z) {
    const double m = -expm1(2.0 * z);
    return m > 0.0 ? sqrt(m) : 0.0;
}

void seq_forward_expnorm_f32(const float* z, const float* v, const float* init, double* out, int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        double s = init ? (double)init[r] : 0.0;
        for (int64_t t = 0; t < T; ++t) {
            const double zt = (double)z[r * T + t];
            s = exp(zt) * s + expnorm_scale(zt) * (double)v[r * T + t];
            out[r * T + t] = s;
        }
    }
}

void seq_backward_expnorm_f32(const float* z, const float* v, const float* state, const float* init, const float* dout,
                              double* dz, double* dv, double* dinit, int64_t rows, int64_t T) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* zr = z + r * T;
        const float* vr = v + r * T;
        const float* sr = state + r * T;
        const double x0 = init ? (double)init[r] : 0.0;
        double g = 0.0;
        for (int64_t t = T - 1; t >= 0; --t) {
            const double gnext = (t + 1 < T) ? exp((double)zr[t + 1]) : 1.0;
            g = (double)dout[r * T + t] + gnext * g;
            const double a = exp((double)zr[t]), b = expnorm_scale((double)zr[t]);
            dv[r * T + t] = g * b;
            dz[r * T + t] = g * (a * ((t > 0) ? (double)sr[t - 1] : x0) - (double)vr[t] * a * a / b);
        }
        if (dinit) dinit[r] = (T > 0) ? exp((double)zr[0]) * g : 0.0;
    }
}
