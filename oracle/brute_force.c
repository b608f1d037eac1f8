/* fp64 brute-force restatement of the two attention definitions, scalar loops only.
 *
 * TEST INFRASTRUCTURE ONLY.  Built into oracle/libbrute_force.so by oracle/Makefile and
 * loaded by tests/ to pin the eager-PyTorch oracle; never linked into the product.
 *
 * The formulas are taken from the mathematics, not from the tensor program:
 *   - half-layout RoPE as a complex multiplication (x[d] + i x[d+D/2]) * (cos + i sin)
 *     (what fused-rope/rope_attn_pytorch.py:52-84 of the reference computes),
 *   - softmax attention row by row with a running maximum (reference :111-155),
 *   - Co-RoPE scores per (i, j, d) as written in the reference README.md:154-172 and
 *     corope-exp/corope_attn_gqa_pytorch.py:58-78: the key pair is rotated by the angle
 *     delta_ij * w_d where delta_ij = sum_{j < t <= i} sigmoid(s * q_leader[i] . k[t]).
 */
#include <math.h>
#include <stdlib.h>

#define IDX4(b, h, n, d, H, N, D) ((((long)(b) * (H) + (h)) * (N) + (n)) * (D) + (d))

/* q, k, v: (B,H,N,D); cosv, sinv: (N, D/2); o: (B,H,N,D); lse: (B,H,N) natural log. */
int bf_rope_attn_fwd(const double *q, const double *k, const double *v,
                     const double *cosv, const double *sinv,
                     int B, int H, int N, int D, int causal, double sm_scale,
                     double *o, double *lse)
{
    int half = D / 2;
    double *qr = (double *)malloc(sizeof(double) * D);
    double *kr = (double *)malloc(sizeof(double) * (long)N * D);
    double *sc = (double *)malloc(sizeof(double) * N);
    if (!qr || !kr || !sc) return -1;
    for (int b = 0; b < B; b++)
        for (int h = 0; h < H; h++) {
            for (int n = 0; n < N; n++)
                for (int d = 0; d < half; d++) {
                    double re = k[IDX4(b, h, n, d, H, N, D)], im = k[IDX4(b, h, n, d + half, H, N, D)];
                    double c = cosv[(long)n * half + d], s = sinv[(long)n * half + d];
                    kr[(long)n * D + d] = re * c - im * s;
                    kr[(long)n * D + d + half] = re * s + im * c;
                }
            for (int i = 0; i < N; i++) {
                for (int d = 0; d < half; d++) {
                    double re = q[IDX4(b, h, i, d, H, N, D)], im = q[IDX4(b, h, i, d + half, H, N, D)];
                    double c = cosv[(long)i * half + d], s = sinv[(long)i * half + d];
                    qr[d] = re * c - im * s;
                    qr[d + half] = re * s + im * c;
                }
                int last = causal ? i : N - 1;
                double mx = -INFINITY;
                for (int j = 0; j <= last; j++) {
                    double acc = 0.0;
                    for (int d = 0; d < D; d++) acc += qr[d] * kr[(long)j * D + d];
                    sc[j] = acc * sm_scale;
                    if (sc[j] > mx) mx = sc[j];
                }
                double den = 0.0;
                for (int j = 0; j <= last; j++) { sc[j] = exp(sc[j] - mx); den += sc[j]; }
                for (int d = 0; d < D; d++) {
                    double acc = 0.0;
                    for (int j = 0; j <= last; j++) acc += sc[j] * v[IDX4(b, h, j, d, H, N, D)];
                    o[IDX4(b, h, i, d, H, N, D)] = acc / den;
                }
                lse[((long)b * H + h) * N + i] = mx + log(den);
            }
        }
    free(qr); free(kr); free(sc);
    return 0;
}

/* q: (B,Hq,N,D); k, v: (B,Hkv,N,D); inv_freq: (D/2); o: (B,Hq,N,D); delta_out (optional): (B,Hkv,N,N). */
int bf_corope_gqa_fwd(const double *q, const double *k, const double *v, const double *inv_freq,
                      int B, int Hq, int Hkv, int N, int D, double sm_scale,
                      double *o, double *delta_out)
{
    if (Hkv <= 0 || Hq % Hkv) return -2;
    int G = Hq / Hkv, half = D / 2;
    double *delta = (double *)malloc(sizeof(double) * N);
    double *sc = (double *)malloc(sizeof(double) * N);
    if (!delta || !sc) return -1;
    for (int b = 0; b < B; b++)
        for (int hq = 0; hq < Hq; hq++) {
            int kv = hq / G, lead = kv * G;
            for (int i = 0; i < N; i++) {
                /* mileage difference: walk left from the diagonal, accumulating the leader's gates */
                double run = 0.0;
                for (int j = i; j >= 0; j--) {
                    delta[j] = run;
                    double dot = 0.0;
                    for (int d = 0; d < D; d++)
                        dot += q[IDX4(b, lead, i, d, Hq, N, D)] * k[IDX4(b, kv, j, d, Hkv, N, D)];
                    run += 1.0 / (1.0 + exp(-dot * sm_scale));
                }
                if (delta_out && hq == lead)
                    for (int j = 0; j < N; j++)
                        delta_out[(((long)b * Hkv + kv) * N + i) * N + j] = j <= i ? delta[j] : 0.0;
                double mx = -INFINITY;
                for (int j = 0; j <= i; j++) {
                    double acc = 0.0;
                    for (int d = 0; d < half; d++) {
                        double ang = delta[j] * inv_freq[d], c = cos(ang), s = sin(ang);
                        double k1 = k[IDX4(b, kv, j, d, Hkv, N, D)], k2 = k[IDX4(b, kv, j, d + half, Hkv, N, D)];
                        double q1 = q[IDX4(b, hq, i, d, Hq, N, D)], q2 = q[IDX4(b, hq, i, d + half, Hq, N, D)];
                        /* Re( conj(q1 + i q2) * (k1 + i k2) * e^{-i ang} ) */
                        double re = q1 * k1 + q2 * k2, im = q1 * k2 - q2 * k1;
                        acc += re * c + im * s;
                    }
                    sc[j] = acc * sm_scale;
                    if (sc[j] > mx) mx = sc[j];
                }
                double den = 0.0;
                for (int j = 0; j <= i; j++) { sc[j] = exp(sc[j] - mx); den += sc[j]; }
                for (int d = 0; d < D; d++) {
                    double acc = 0.0;
                    for (int j = 0; j <= i; j++) acc += sc[j] * v[IDX4(b, kv, j, d, Hkv, N, D)];
                    o[IDX4(b, hq, i, d, Hq, N, D)] = acc / den;
                }
            }
        }
    free(delta); free(sc);
    return 0;
}
