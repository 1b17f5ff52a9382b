/*
 * TEST INFRASTRUCTURE -- CPU oracle of the RBF-scaled geometric attention forward.
 * Not part of the product; the product path never links or calls this file.
 *
 * Follows:
 *   README.md:40                                   multiplier 1 + exp(-|rq-rk|^2 / (2 sigma_h^2))
 *   old/old_scripts/attn/geometric_attn.py:183-236 scale 1/sqrt(d) applied to S before the geometric
 *                                                  factor (:186), -inf for masked pairs (:196-201),
 *                                                  rows with l == 0 -> O = 0 (:233), L = m + log l (:236)
 *   tests/attn/geo_attn.py:194-210                 dense structure: S = QK^T/sqrt(d); dists; rbfs;
 *                                                  where(mask, -inf, .); softmax; P V
 * Padded queries are masked as well as padded keys (geometric_attn.py:196).
 *
 * Q, K, V are floats (the caller passes bf16-rounded values when checking a
 * bf16 kernel).  `rows` selects query rows (NULL = all); output row r of
 * (z,h) is written at ((z*H + h)*nrows + r).  Everything is evaluated in
 * double and returned in double.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

void geo_attn_oracle_f64(const float* Q, const float* K, const float* V /*[Z,H,N,d]*/,
                         const float* coords /*[Z,N,3]*/, const float* sigma /*[H]*/,
                         const uint8_t* key_pad /*[Z,N] or NULL*/,
                         int Z, int H, int N, int d,
                         const int* rows, int nrows,
                         double* O /*[Z,H,nrows,d]*/, double* L /*[Z,H,nrows]*/)
{
    const double scale = 1.0 / sqrt((double)d);
    #pragma omp parallel
    {
        double* s = (double*)malloc(sizeof(double) * (size_t)N);
        #pragma omp for collapse(3) schedule(dynamic, 4)
        for (int z = 0; z < Z; ++z)
        for (int h = 0; h < H; ++h)
        for (int rr = 0; rr < nrows; ++rr) {
            const int i = rows ? rows[rr] : rr;
            const size_t zh = (size_t)z * H + h;
            const float* q = Q + (zh * N + i) * d;
            const float* c = coords + (size_t)z * N * 3;
            const uint8_t* m = key_pad ? key_pad + (size_t)z * N : NULL;
            double* o = O + (zh * nrows + rr) * d;
            for (int t = 0; t < d; ++t) o[t] = 0.0;
            const double two_s2 = 2.0 * (double)sigma[h] * (double)sigma[h];
            double mx = -INFINITY;
            const int qpad = m && m[i];
            for (int j = 0; j < N; ++j) {
                if (qpad || (m && m[j])) { s[j] = -INFINITY; continue; }
                const float* kk = K + (zh * N + j) * d;
                double dot = 0.0;
                for (int t = 0; t < d; ++t) dot += (double)q[t] * (double)kk[t];
                const double dx = (double)c[3*i] - c[3*j], dy = (double)c[3*i+1] - c[3*j+1], dz = (double)c[3*i+2] - c[3*j+2];
                const double d2 = dx*dx + dy*dy + dz*dz;
                s[j] = dot * scale * (1.0 + exp(-d2 / two_s2));
                if (s[j] > mx) mx = s[j];
            }
            if (mx == -INFINITY) { L[zh * nrows + rr] = -INFINITY; continue; }
            double l = 0.0;
            for (int j = 0; j < N; ++j) {
                if (s[j] == -INFINITY) continue;
                const double p = exp(s[j] - mx);
                l += p;
                const float* v = V + (zh * N + j) * d;
                for (int t = 0; t < d; ++t) o[t] += p * (double)v[t];
            }
            for (int t = 0; t < d; ++t) o[t] /= l;
            L[zh * nrows + rr] = mx + log(l);
        }
        free(s);
    }
}

/*
 * The logits of the reference's executable kernel and of its dense PyTorch
 * statement (tests/attn/geo_attn.py:194-210, old/old_scripts/attn/geometric_attn.py:193-201):
 *   S     = Q K^T / sqrt(d)
 *   rbfs  = exp(-dists^2 / (2 spreads^2))
 *   mask  = mask_i | mask_j | rbfs < min_rbf | rbfs > max_rbf
 *   rbfs  = 2 (rbfs - min_rbf)/(max_rbf - min_rbf) - 1
 *   S     = where(mask, -inf, S + b * rbfs * |S|);  P = softmax(S);  out = P V
 * Rows without any unmasked pair give O = 0, L = -inf (kernel :233-236).
 */
void geo_attn_legacy_oracle_f64(const float* Q, const float* K, const float* V /*[Z,H,N,d]*/,
                                const float* coords /*[Z,N,3]*/, const float* sigma /*[H]*/, const float* beta /*[H]*/,
                                const uint8_t* key_pad /*[Z,N] or NULL*/,
                                int Z, int H, int N, int d, double min_rbf, double max_rbf,
                                const int* rows, int nrows,
                                double* O /*[Z,H,nrows,d]*/, double* L /*[Z,H,nrows]*/)
{
    const double scale = 1.0 / sqrt((double)d);
    #pragma omp parallel
    {
        double* s = (double*)malloc(sizeof(double) * (size_t)N);
        #pragma omp for collapse(3) schedule(dynamic, 4)
        for (int z = 0; z < Z; ++z)
        for (int h = 0; h < H; ++h)
        for (int rr = 0; rr < nrows; ++rr) {
            const int i = rows ? rows[rr] : rr;
            const size_t zh = (size_t)z * H + h;
            const float* q = Q + (zh * N + i) * d;
            const float* c = coords + (size_t)z * N * 3;
            const uint8_t* m = key_pad ? key_pad + (size_t)z * N : NULL;
            double* o = O + (zh * nrows + rr) * d;
            for (int t = 0; t < d; ++t) o[t] = 0.0;
            const double two_s2 = 2.0 * (double)sigma[h] * (double)sigma[h];
            double mx = -INFINITY;
            const int qpad = m && m[i];
            for (int j = 0; j < N; ++j) {
                s[j] = -INFINITY;
                if (qpad || (m && m[j])) continue;
                const double dx = (double)c[3*i] - c[3*j], dy = (double)c[3*i+1] - c[3*j+1], dz = (double)c[3*i+2] - c[3*j+2];
                const double rbf = exp(-(dx*dx + dy*dy + dz*dz) / two_s2);
                if (rbf < min_rbf || rbf > max_rbf) continue;
                const float* kk = K + (zh * N + j) * d;
                double dot = 0.0;
                for (int t = 0; t < d; ++t) dot += (double)q[t] * (double)kk[t];
                const double S = dot * scale;
                const double rn = 2.0 * (rbf - min_rbf) / (max_rbf - min_rbf) - 1.0;
                s[j] = S + (double)beta[h] * rn * fabs(S);
                if (s[j] > mx) mx = s[j];
            }
            if (mx == -INFINITY) { L[zh * nrows + rr] = -INFINITY; continue; }
            double l = 0.0;
            for (int j = 0; j < N; ++j) {
                if (s[j] == -INFINITY) continue;
                const double p = exp(s[j] - mx);
                l += p;
                const float* v = V + (zh * N + j) * d;
                for (int t = 0; t < d; ++t) o[t] += p * (double)v[t];
            }
            for (int t = 0; t < d; ++t) o[t] /= l;
            L[zh * nrows + rr] = mx + log(l);
        }
        free(s);
    }
}
