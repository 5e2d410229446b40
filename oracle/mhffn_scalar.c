/* Scalar C restatement of the multi-head FFN, forward and backward, in double precision.
 * TEST INFRASTRUCTURE ONLY: it pins oracle/mhffn_oracle.py by brute force (no BLAS, no vector
 * library, one multiply-add at a time) and is never linked into or called by the shipped library.
 *
 * Forward follows models/flashmhf/modeling_mhffnmoe.py:418-427 (s0=s1=s2=1) element by element;
 * backward follows kernels/triton/flash_mlp_moe.py:401-414 with the R factor of :534-536 and :720-729.
 *
 * Layouts (row-major, contiguous): Q,O,dO,dQ [B,H,S,dh]; K,U,V,dK,dU,dV [Hk,E,de,dh]; R,dR [B,H,S,E].
 * q-head h reads kuv-head h / (H/Hk)  (modeling_mhffnmoe.py:246-251).
 */
#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

static double sigmoid_(double x) { return 1.0 / (1.0 + exp(-x)); }

void mhffn_scalar_forward(const double* Q, const double* K, const double* U, const double* V,
                          const double* R, double* O,
                          int B, int H, int Hk, int S, int dh, int E, int de)
{
    const int G = H / Hk;
    for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h)
    for (int t = 0; t < S; ++t) {
        const size_t row = ((size_t)b * H + h) * S + t;
        const double* q = Q + row * dh;
        double* o = O + row * dh;
        for (int c = 0; c < dh; ++c) o[c] = 0.0;
        for (int e = 0; e < E; ++e) {
            const size_t wbase = (((size_t)(h / G) * E + e) * de) * dh;
            const double r = R[row * E + e];
            for (int j = 0; j < de; ++j) {
                const double* kj = K + wbase + (size_t)j * dh;
                const double* uj = U + wbase + (size_t)j * dh;
                const double* vj = V + wbase + (size_t)j * dh;
                double m = 0.0, n = 0.0;
                for (int c = 0; c < dh; ++c) { m += q[c] * kj[c]; n += q[c] * uj[c]; }
                const double a = m * sigmoid_(m) * n;
                for (int c = 0; c < dh; ++c) o[c] += r * a * vj[c];
            }
        }
    }
}

void mhffn_scalar_backward(const double* Q, const double* K, const double* U, const double* V,
                           const double* R, const double* dO,
                           double* dQ, double* dK, double* dU, double* dV, double* dR,
                           int B, int H, int Hk, int S, int dh, int E, int de)
{
    const int G = H / Hk;
    const size_t wsz = (size_t)Hk * E * de * dh;
    memset(dK, 0, wsz * sizeof(double));
    memset(dU, 0, wsz * sizeof(double));
    memset(dV, 0, wsz * sizeof(double));
    for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h)
    for (int t = 0; t < S; ++t) {
        const size_t row = ((size_t)b * H + h) * S + t;
        const double* q = Q + row * dh;
        const double* g = dO + row * dh;
        double* dq = dQ + row * dh;
        for (int c = 0; c < dh; ++c) dq[c] = 0.0;
        for (int e = 0; e < E; ++e) {
            const size_t wbase = (((size_t)(h / G) * E + e) * de) * dh;
            const double r = R[row * E + e];
            double dr = 0.0;
            for (int j = 0; j < de; ++j) {
                const size_t w = wbase + (size_t)j * dh;
                double m = 0.0, n = 0.0, da = 0.0;
                for (int c = 0; c < dh; ++c) { m += q[c] * K[w + c]; n += q[c] * U[w + c]; da += g[c] * V[w + c]; }
                const double sg = sigmoid_(m), s = m * sg;
                dr += da * s * n;
                const double dn = r * da * s;
                const double dm = r * da * n * (sg + s * (1.0 - sg));
                const double pa = r * s * n;
                for (int c = 0; c < dh; ++c) {
                    dq[c] += dm * K[w + c] + dn * U[w + c];
                    dK[w + c] += dm * q[c];
                    dU[w + c] += dn * q[c];
                    dV[w + c] += pa * g[c];
                }
            }
            dR[row * E + e] = dr;
        }
    }
}
