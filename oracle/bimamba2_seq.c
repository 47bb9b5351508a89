/* Scalar C restatement of the bidirectional SSD forward:  y = SS(x) + flip(SS(flip(x))) + D*x  [* silu(z)].
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/libbimamba2_seq.so and called from tests/ to pin the torch
 * oracle (oracle/bimamba2_oracle.py) with code in another language that shares nothing with it.
 *
 * Follows: formula README.md:13-17 of the reference; dt preprocessing order (+bias, softplus with the
 * x > 20 identity, clamp) src/ssd/bi/ssd_chunk_state.py:70-82 and src/ssd/bi/softplus.py:8-17; D then z
 * order src/ssd/bi/ssd_chunk_scan.py:168-189; flip applies to x, dt, B, C and D*x is added once
 * tests/fixtures/fwd.py:58-70.
 *
 * All arrays are contiguous doubles: x,z,out (B,L,H,P); dt (B,L,H); A (H); Bm,Cm (B,L,G,N);
 * D (H) or (H,P) or NULL; dt_bias (H) or NULL; final_f, final_b (B,H,P,N) or NULL.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

static double dt_prime(double dt, double bias, int softplus, double lo, double hi) {
    double v = dt + bias;
    if (softplus) v = v > 20.0 ? v : log1p(exp(v));
    if (v < lo) v = lo;
    if (v > hi) v = hi;
    return v;
}

int bimamba2_seq_forward(int nb, int L, int H, int P, int G, int N,
                         const double *x, const double *dt, const double *A, const double *Bm,
                         const double *Cm, const double *D, int D_has_hdim, const double *z,
                         const double *dt_bias, int dt_softplus, double dt_min, double dt_max,
                         double *out, double *out_x, double *final_f, double *final_b) {
    if (H % G) return -1;
    double *state = (double *)malloc(sizeof(double) * (size_t)P * N);
    double *y = (double *)malloc(sizeof(double) * (size_t)L * P);
    if (!state || !y) return -2;
    int hpg = H / G;
    for (int b = 0; b < nb; ++b)
        for (int h = 0; h < H; ++h) {
            int g = h / hpg;
            memset(y, 0, sizeof(double) * (size_t)L * P);
            for (int dir = 0; dir < 2; ++dir) {
                memset(state, 0, sizeof(double) * (size_t)P * N);
                for (int step = 0; step < L; ++step) {
                    int t = dir == 0 ? step : L - 1 - step;
                    double dtp = dt_prime(dt[((size_t)b * L + t) * H + h], dt_bias ? dt_bias[h] : 0.0,
                                          dt_softplus, dt_min, dt_max);
                    double dec = exp(dtp * A[h]);
                    const double *xt = x + (((size_t)b * L + t) * H + h) * P;
                    const double *bt = Bm + (((size_t)b * L + t) * G + g) * N;
                    const double *ct = Cm + (((size_t)b * L + t) * G + g) * N;
                    for (int p = 0; p < P; ++p) {
                        double acc = 0.0;
                        for (int n = 0; n < N; ++n) {
                            double s = dec * state[p * N + n] + dtp * xt[p] * bt[n];
                            state[p * N + n] = s;
                            acc += s * ct[n];
                        }
                        y[(size_t)t * P + p] += acc;
                    }
                }
                double *fin = dir == 0 ? final_f : final_b;
                if (fin) memcpy(fin + ((size_t)b * H + h) * P * N, state, sizeof(double) * (size_t)P * N);
            }
            for (int t = 0; t < L; ++t)
                for (int p = 0; p < P; ++p) {
                    size_t idx = (((size_t)b * L + t) * H + h) * P + p;
                    double v = y[(size_t)t * P + p];
                    if (D) v += (D_has_hdim ? D[h * P + p] : D[h]) * x[idx];
                    if (out_x) out_x[idx] = v;
                    if (z) v *= z[idx] / (1.0 + exp(-z[idx]));
                    out[idx] = v;
                }
        }
    free(state);
    free(y);
    return 0;
}
