/* C restatement of the five benchmark expressions, one IEEE operation per
 * source operation.  TEST INFRASTRUCTURE: used only to pin numpy_oracle.py
 * (tests/test_oracle.py); never linked into the product.
 *
 * Built with -ffp-contract=off -fno-fast-math so that a*b+c is a rounded
 * multiply followed by a rounded add, which is what the reference's CPU backend
 * does when it applies numpy.multiply and numpy.add as separate nodes
 * (delayrepay/cpu.py:19-26).  Float expressions are written with explicit float
 * temporaries so no operation is carried out in double.
 */
#include <math.h>
#include <stddef.h>

/* z = a*x + y, a as float (weak Python scalar; delayarray.py:473-474) */
void dro_saxpy_f32(float a, const float* x, const float* y, float* z, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        float t = a * x[i];
        z[i] = t + y[i];
    }
}

/* ((c[d]*x + c[d-1])*x + ...)*x + c[0] */
void dro_horner_f32(const float* c, int degree, const float* x, float* y, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        float t = c[degree] * x[i];
        float acc = t + c[degree - 1];
        for (int k = degree - 2; k >= 0; k--) {
            t = acc * x[i];
            acc = t + c[k];
        }
        y[i] = acc;
    }
}

/* one Jacobi sweep src -> dst on the interior of an h x w grid; boundary copied;
 * association ((up + down) + left) + right, then 0.25f * sum */
void dro_jacobi_sweep_f32(const float* src, float* dst, size_t h, size_t w)
{
    for (size_t i = 0; i < h; i++)
        for (size_t j = 0; j < w; j++) {
            if (i == 0 || j == 0 || i == h - 1 || j == w - 1) {
                dst[i * w + j] = src[i * w + j];
                continue;
            }
            float s = src[(i - 1) * w + j] + src[(i + 1) * w + j];
            s = s + src[i * w + j - 1];
            s = s + src[i * w + j + 1];
            dst[i * w + j] = 0.25f * s;
        }
}

/* Black-Scholes call and put, double, the fixed operation order of the config */
void dro_black_scholes_f64(const double* S, const double* K, const double* T, double r,
                           double sigma, double* call, double* put, size_t n)
{
    const double inv_sqrt2 = 0.7071067811865476;
    const double drift = r + 0.5 * sigma * sigma;
    const double neg_r = -r;
    for (size_t i = 0; i < n; i++) {
        double sqT = sqrt(T[i]);
        double vs = sigma * sqT;
        double d1 = (log(S[i] / K[i]) + drift * T[i]) / vs;
        double d2 = d1 - vs;
        double N1 = 0.5 * (1 + erf(d1 * inv_sqrt2));
        double N2 = 0.5 * (1 + erf(d2 * inv_sqrt2));
        double disc = K[i] * exp(neg_r * T[i]);
        call[i] = S[i] * N1 - disc * N2;
        put[i] = disc * (1 - N2) - S[i] * (1 - N1);
    }
}

/* terms (x-y)*(x-y)*w written out, so the caller can sum them its own way */
void dro_sumsq_terms_f64(const double* x, const double* y, const double* w, double* t, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        double d = x[i] - y[i];
        double q = d * d;
        t[i] = q * w[i];
    }
}
