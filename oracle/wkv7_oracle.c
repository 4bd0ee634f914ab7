/* CPU oracle for the RWKV-7 WKV7 recurrence: fp64, token by token, with a
 * hand-derived reverse pass.  TEST INFRASTRUCTURE ONLY: nothing in the shipped
 * package links or loads this file; it exists so that the full benchmark shape
 * (B=8,T=1024,H=12,C=64) can be checked in seconds.
 *
 * The forward loop follows the reference's ground-truth recurrence,
 * tests/test_attn.py:13-17 (same at wind_rwkv/rwkv7/time_mixer.py:11-15):
 *     decay_t = exp(-exp(w_t))
 *     S_t = S_{t-1} * decay_t[None,:] + (S_{t-1} a_t) b_t^T + v_t k_t^T
 *     y_t = S_t q_t
 * with the initial / final state of the autograd Function (rwkv7_attn.py:20-29).
 *
 * The reverse pass is the textbook adjoint of that loop (not taken from the
 * reference, which never differentiates the loop by hand):
 *     G_t    += dy_t q_t^T                     (G_t = dL/dS_t)
 *     dq_t    = S_t^T dy_t
 *     ddecay  = sum_i G_t[i,:] * S_{t-1}[i,:]  -> dw_t = ddecay * decay_t * (-exp(w_t))
 *     du_t    = G_t b_t          db_t = G_t^T u_t        (u_t = S_{t-1} a_t)
 *     dv_t    = G_t k_t          dk_t = G_t^T v_t
 *     da_t    = S_{t-1}^T du_t
 *     G_{t-1} = G_t * decay_t[None,:] + du_t a_t^T
 * Pinning: tests compare it with torch.autograd on oracle/seq_ref.py:wkv7_seq and
 * with finite differences.
 *
 * Layout: q,w,k,v,a,b,y,dy and the six gradients are [B,T,H,C] row-major doubles;
 * s0,sT,dsT,ds0 are [B,H,C,C] with S[i,j] = value row i, key column j.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define IDX(bi, t, hi) ((((size_t)(bi) * T + (t)) * H + (hi)) * C)

/* Forward for one (batch, head).  If states != NULL it receives S_0..S_T ((T+1)*C*C doubles). */
static void head_forward(int T, int H, int C, int bi, int hi,
                         const double *q, const double *w, const double *k, const double *v,
                         const double *a, const double *b, const double *s0,
                         double *y, double *sT, double *states)
{
    size_t CC = (size_t)C * C;
    double *S = (double *)malloc(CC * sizeof(double));
    double *u = (double *)malloc(C * sizeof(double));
    double *dec = (double *)malloc(C * sizeof(double));
    memcpy(S, s0 + ((size_t)bi * H + hi) * CC, CC * sizeof(double));
    if (states) memcpy(states, S, CC * sizeof(double));
    for (int t = 0; t < T; t++) {
        size_t o = IDX(bi, t, hi);
        for (int j = 0; j < C; j++) dec[j] = exp(-exp(w[o + j]));
        for (int i = 0; i < C; i++) {
            double acc = 0;
            for (int j = 0; j < C; j++) acc += S[i * C + j] * a[o + j];
            u[i] = acc;
        }
        for (int i = 0; i < C; i++) {
            double yi = 0;
            for (int j = 0; j < C; j++) {
                double s = S[i * C + j] * dec[j] + u[i] * b[o + j] + v[o + i] * k[o + j];
                S[i * C + j] = s;
                yi += s * q[o + j];
            }
            y[o + i] = yi;
        }
        if (states) memcpy(states + (size_t)(t + 1) * CC, S, CC * sizeof(double));
    }
    memcpy(sT + ((size_t)bi * H + hi) * CC, S, CC * sizeof(double));
    free(S); free(u); free(dec);
}

int wkv7_oracle_forward(int B, int T, int H, int C,
                        const double *q, const double *w, const double *k, const double *v,
                        const double *a, const double *b, const double *s0,
                        double *y, double *sT)
{
    if (B <= 0 || T <= 0 || H <= 0 || C <= 0) return 1;
#pragma omp parallel for schedule(dynamic)
    for (int bh = 0; bh < B * H; bh++)
        head_forward(T, H, C, bh / H, bh % H, q, w, k, v, a, b, s0, y, sT, NULL);
    return 0;
}

int wkv7_oracle_backward(int B, int T, int H, int C,
                         const double *q, const double *w, const double *k, const double *v,
                         const double *a, const double *b, const double *s0,
                         const double *dy, const double *dsT,
                         double *dq, double *dw, double *dk, double *dv, double *da, double *db,
                         double *ds0)
{
    if (B <= 0 || T <= 0 || H <= 0 || C <= 0) return 1;
    size_t CC = (size_t)C * C;
    int fail = 0;
#pragma omp parallel for schedule(dynamic)
    for (int bh = 0; bh < B * H; bh++) {
        int bi = bh / H, hi = bh % H;
        double *states = (double *)malloc((size_t)(T + 1) * CC * sizeof(double));
        double *G = (double *)malloc(CC * sizeof(double));
        double *u = (double *)malloc(C * sizeof(double));
        double *du = (double *)malloc(C * sizeof(double));
        double *dec = (double *)malloc(C * sizeof(double));
        if (!states || !G || !u || !du || !dec) {
#pragma omp atomic write
            fail = 1;
        }
        else {
            /* recompute the forward pass and keep every state S_0..S_T */
            {
                double *S = G; /* reuse */
                memcpy(S, s0 + ((size_t)bi * H + hi) * CC, CC * sizeof(double));
                memcpy(states, S, CC * sizeof(double));
                for (int t = 0; t < T; t++) {
                    size_t o = IDX(bi, t, hi);
                    for (int j = 0; j < C; j++) dec[j] = exp(-exp(w[o + j]));
                    for (int i = 0; i < C; i++) {
                        double acc = 0;
                        for (int j = 0; j < C; j++) acc += S[i * C + j] * a[o + j];
                        u[i] = acc;
                    }
                    for (int i = 0; i < C; i++)
                        for (int j = 0; j < C; j++)
                            S[i * C + j] = S[i * C + j] * dec[j] + u[i] * b[o + j] + v[o + i] * k[o + j];
                    memcpy(states + (size_t)(t + 1) * CC, S, CC * sizeof(double));
                }
            }
            memcpy(G, dsT + ((size_t)bi * H + hi) * CC, CC * sizeof(double));
            for (int t = T - 1; t >= 0; t--) {
                size_t o = IDX(bi, t, hi);
                const double *Sp = states + (size_t)t * CC;       /* S_{t-1} */
                const double *Sc = states + (size_t)(t + 1) * CC; /* S_t */
                for (int j = 0; j < C; j++) dec[j] = exp(-exp(w[o + j]));
                for (int i = 0; i < C; i++) {
                    double acc = 0;
                    for (int j = 0; j < C; j++) acc += Sp[i * C + j] * a[o + j];
                    u[i] = acc;
                }
                for (int i = 0; i < C; i++)
                    for (int j = 0; j < C; j++) G[i * C + j] += dy[o + i] * q[o + j];
                for (int j = 0; j < C; j++) {
                    double aq = 0, ad = 0, ab = 0, ak = 0;
                    for (int i = 0; i < C; i++) {
                        double g = G[i * C + j];
                        aq += Sc[i * C + j] * dy[o + i];
                        ad += g * Sp[i * C + j];
                        ab += g * u[i];
                        ak += g * v[o + i];
                    }
                    dq[o + j] = aq;
                    dw[o + j] = ad * dec[j] * (-exp(w[o + j]));
                    db[o + j] = ab;
                    dk[o + j] = ak;
                }
                for (int i = 0; i < C; i++) {
                    double au = 0, av = 0;
                    for (int j = 0; j < C; j++) {
                        au += G[i * C + j] * b[o + j];
                        av += G[i * C + j] * k[o + j];
                    }
                    du[i] = au;
                    dv[o + i] = av;
                }
                for (int j = 0; j < C; j++) {
                    double acc = 0;
                    for (int i = 0; i < C; i++) acc += Sp[i * C + j] * du[i];
                    da[o + j] = acc;
                }
                for (int i = 0; i < C; i++)
                    for (int j = 0; j < C; j++)
                        G[i * C + j] = G[i * C + j] * dec[j] + du[i] * a[o + j];
            }
            memcpy(ds0 + ((size_t)bi * H + hi) * CC, G, CC * sizeof(double));
        }
        free(states); free(G); free(u); free(du); free(dec);
    }
    return fail;
}
