/*
 * TEST INFRASTRUCTURE -- CPU oracle of the anisotropic (C-beta scaled, learnable
 * wavenumber) Wavefunction Embedding.  Not part of the product; the product path
 * never links or calls this file.
 *
 * Follows, in meaning (paths under the reference root):
 *   tests/wf_embed/wf_embed_aniso_learnCB_learnK.py:117-163      (wf_embedding_torch: `out`)
 *   utils/model_utils/wf_embedding/anisotropic/cb_scaling/learnable_wavenumbers/cuda/
 *       wf_embedding_kernel.cu:141-206                            (pair mask, d_k and d_cb terms)
 *
 *   R       = a_i - a_j ; dist = |R| ; R_unit = R / dist             test :127-134
 *   distsB  = R_unit . (b_j * cb_k)                                   test :142-144
 *   phase   = (dist - distsB) * k_k                                   test :146-149
 *   masked  = mask_i | mask_j | dist == 0 ; mag = 1/dist              test :152-155
 *   out[i,2k] = sum_j mag cos(phase), out[i,2k+1] = sum_j mag sin(phase)   test :158-168
 *   real = mag cos, imag = mag sin, A = R_unit . b_j, u = dist - cb_k A     kernel :156-181
 *   d_k [i,2k] = sum_j -imag u        d_k [i,2k+1] = sum_j real u           kernel :187-188
 *   d_cb[i,2k] = sum_j  imag k_k A    d_cb[i,2k+1] = sum_j -real k_k A      kernel :193-194
 *
 * Everything is evaluated in double from the float inputs.  `rows` selects observers
 * (NULL = all), output row r of batch z is written at index (z*nrows + r).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

void we_aniso_oracle_f64(const float* ca /*[Z,N,3]*/, const float* cbv /*[Z,N,3]*/,
                         const float* cbm /*[K]*/, const float* wn /*[K]*/,
                         const uint8_t* mask /*[Z,N] or NULL*/, int Z, int N, int K,
                         const int* rows, int nrows,
                         double* out /*[Z,nrows,2K]*/, double* d_cb, double* d_k)
{
    #pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int z = 0; z < Z; ++z)
    for (int rr = 0; rr < nrows; ++rr) {
        const int i = rows ? rows[rr] : rr;
        const float* a = ca + (size_t)z * N * 3;
        const float* b = cbv + (size_t)z * N * 3;
        const uint8_t* m = mask ? mask + (size_t)z * N : NULL;
        double* o  = out  + ((size_t)z * nrows + rr) * 2 * K;
        double* gc = d_cb + ((size_t)z * nrows + rr) * 2 * K;
        double* gk = d_k  + ((size_t)z * nrows + rr) * 2 * K;
        for (int k = 0; k < 2 * K; ++k) { o[k] = 0.0; gc[k] = 0.0; gk[k] = 0.0; }
        if (m && m[i]) continue;
        for (int j = 0; j < N; ++j) {
            if (m && m[j]) continue;
            const double Rx = (double)a[3*i] - a[3*j], Ry = (double)a[3*i+1] - a[3*j+1], Rz = (double)a[3*i+2] - a[3*j+2];
            const double dist = sqrt(Rx*Rx + Ry*Ry + Rz*Rz);
            if (dist == 0.0) continue;
            const double mag = 1.0 / dist;
            const double A = (Rx * b[3*j] + Ry * b[3*j+1] + Rz * b[3*j+2]) * mag;
            for (int k = 0; k < K; ++k) {
                const double kk = wn[k];
                const double u = dist - A * (double)cbm[k];
                const double phase = u * kk;
                const double real = mag * cos(phase), imag = mag * sin(phase);
                o[2*k]    += real;            o[2*k+1]  += imag;
                gk[2*k]   += -imag * u;       gk[2*k+1] += real * u;
                gc[2*k]   += imag * kk * A;   gc[2*k+1] += -real * kk * A;
            }
        }
    }
}
