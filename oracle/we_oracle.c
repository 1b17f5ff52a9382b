/*
 * TEST INFRASTRUCTURE -- CPU oracle of the isotropic Wavefunction Embedding.
 * Not part of the product; the product path never links or calls this file.
 * PARITY UNPINNED: we_oracle_hash5 (the dropout hash at the end of this file; see its comment).  Everything else is
 * pinned by tests/test_oracle_we.py and tests/test_oracle_we_dropout.py.
 *
 * Follows, line by line in meaning:
 *   tests/wf_embed/wf_embed.py:91-129                    (wf_embedding_torch, mag_type 1)
 *   isotropic/cuda/wf_embedding_kernel.cu:181-250        (valid rule, sums = real*dists)
 *   isotropic/triton_old/wf_embedding.py:163-198         (explicit-mask statement of the sums)
 * under utils/model_utils/wf_embedding/.
 *
 *   dist_ij  = sqrt(sum_c (x_ic - x_jc)^2)                       wf_embed.py:100
 *   phase    = dist_ij * k                                        wf_embed.py:103
 *   masked   = mask_i | mask_j | dist_ij == 0                     wf_embed.py:106
 *   mag      = 1 / (masked ? inf : dist_ij)                       wf_embed.py:112
 *   out[i,2k]   = sum_j mag cos(phase), out[i,2k+1] = sum_j mag sin(phase)   wf_embed.py:119-127
 *   cos_sums[i,k] = sum_j !masked cos(phase), sin_sums likewise   kernel.cu:224-238 (real*dists = cos)
 *
 * Two flavours: *_f64 evaluates everything in double; *_f32 evaluates each
 * term in float exactly as the PyTorch statement would (sqrtf, float product,
 * cosf/sinf, float divide) and accumulates the float terms in double.
 * `rows` selects observers (NULL = all rows 0..nrows-1 of each batch item), so
 * that long sequences can be checked on a sample: rows are independent.
 * Output row r of batch z is written at index (z*nrows + r).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

#define TILE_K 64

void we_oracle_f64(const float* coords /*[Z,N,3]*/, const float* wn /*[K]*/,
                   const uint8_t* mask /*[Z,N] or NULL*/, int Z, int N, int K,
                   const int* rows, int nrows,
                   double* out /*[Z,nrows,2K]*/, double* cs /*[Z,nrows,K]*/, double* ss)
{
    #pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int z = 0; z < Z; ++z)
    for (int rr = 0; rr < nrows; ++rr) {
        const int i = rows ? rows[rr] : rr;
        const float* c = coords + (size_t)z * N * 3;
        const uint8_t* m = mask ? mask + (size_t)z * N : NULL;
        double* o = out + ((size_t)z * nrows + rr) * 2 * K;
        double* pc = cs + ((size_t)z * nrows + rr) * K;
        double* ps = ss + ((size_t)z * nrows + rr) * K;
        for (int k = 0; k < K; ++k) { o[2*k] = o[2*k+1] = pc[k] = ps[k] = 0.0; }
        if (m && m[i]) continue;
        const double xi = c[3*i], yi = c[3*i+1], zi = c[3*i+2];
        for (int j = 0; j < N; ++j) {
            if (m && m[j]) continue;
            const double dx = xi - c[3*j], dy = yi - c[3*j+1], dz = zi - c[3*j+2];
            const double d2 = dx*dx + dy*dy + dz*dz;
            if (d2 == 0.0) continue;
            const double d = sqrt(d2), inv = 1.0 / d;
            for (int k = 0; k < K; ++k) {
                const double ph = d * (double)wn[k];
                const double co = cos(ph), si = sin(ph);
                o[2*k] += co * inv; o[2*k+1] += si * inv; pc[k] += co; ps[k] += si;
            }
        }
    }
}

void we_oracle_f32(const float* coords, const float* wn, const uint8_t* mask, int Z, int N, int K,
                   const int* rows, int nrows, float* out, float* cs, float* ss)
{
    #pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int z = 0; z < Z; ++z)
    for (int rr = 0; rr < nrows; ++rr) {
        const int i = rows ? rows[rr] : rr;
        const float* c = coords + (size_t)z * N * 3;
        const uint8_t* m = mask ? mask + (size_t)z * N : NULL;
        float* o = out + ((size_t)z * nrows + rr) * 2 * K;
        float* pc = cs + ((size_t)z * nrows + rr) * K;
        float* ps = ss + ((size_t)z * nrows + rr) * K;
        double* acc = (double*)calloc((size_t)4 * K, sizeof(double));
        if (!(m && m[i])) {
            const float xi = c[3*i], yi = c[3*i+1], zi = c[3*i+2];
            for (int j = 0; j < N; ++j) {
                if (m && m[j]) continue;
                const float dx = xi - c[3*j], dy = yi - c[3*j+1], dz = zi - c[3*j+2];
                /* torch: sum over the last dim of the squared differences, in float */
                const float d2 = (dx*dx + dy*dy) + dz*dz;
                const float d = sqrtf(d2);
                if (d == 0.0f) continue;
                const float inv = 1.0f / d;
                for (int k = 0; k < K; ++k) {
                    const float ph = d * wn[k];
                    const float co = cosf(ph), si = sinf(ph);
                    acc[4*k]   += (double)(inv * co);
                    acc[4*k+1] += (double)(inv * si);
                    acc[4*k+2] += (double)co;
                    acc[4*k+3] += (double)si;
                }
            }
        }
        for (int k = 0; k < K; ++k) {
            o[2*k] = (float)acc[4*k]; o[2*k+1] = (float)acc[4*k+1];
            pc[k] = (float)acc[4*k+2]; ps[k] = (float)acc[4*k+3];
        }
        free(acc);
    }
}

/*
 * The reference's other source weights (isotropic/cuda/wf_embedding_kernel.cu:192-206;
 * dense statement tests/wf_embed/wf_embed.py:108-116):
 *   mag_type 0: m = 1   1: m = 1/d   2: m = 1/log2(d)   3: m = 1/sqrt(d)
 *   out = sum_j m cos, m sin ;  cos_sums, sin_sums = sum_j (m d) cos, (m d) sin   kernel.cu:237-238
 */
void we_oracle_mag_f64(const float* coords, const float* wn, const uint8_t* mask, int Z, int N, int K,
                       int mag_type, const int* rows, int nrows,
                       double* out, double* cs, double* ss)
{
    #pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int z = 0; z < Z; ++z)
    for (int rr = 0; rr < nrows; ++rr) {
        const int i = rows ? rows[rr] : rr;
        const float* c = coords + (size_t)z * N * 3;
        const uint8_t* m = mask ? mask + (size_t)z * N : NULL;
        double* o = out + ((size_t)z * nrows + rr) * 2 * K;
        double* pc = cs + ((size_t)z * nrows + rr) * K;
        double* ps = ss + ((size_t)z * nrows + rr) * K;
        for (int k = 0; k < K; ++k) { o[2*k] = o[2*k+1] = pc[k] = ps[k] = 0.0; }
        if (m && m[i]) continue;
        const double xi = c[3*i], yi = c[3*i+1], zi = c[3*i+2];
        for (int j = 0; j < N; ++j) {
            if (m && m[j]) continue;
            const double dx = xi - c[3*j], dy = yi - c[3*j+1], dz = zi - c[3*j+2];
            const double d2 = dx*dx + dy*dy + dz*dz;
            if (d2 == 0.0) continue;
            const double d = sqrt(d2);
            double w = 1.0;
            if (mag_type == 1) w = 1.0 / d;
            if (mag_type == 2) w = 1.0 / log2(d);
            if (mag_type == 3) w = 1.0 / sqrt(d);
            for (int k = 0; k < K; ++k) {
                const double ph = d * (double)wn[k];
                const double co = cos(ph), si = sin(ph);
                o[2*k] += co * w; o[2*k+1] += si * w; pc[k] += co * w * d; ps[k] += si * w * d;
            }
        }
    }
}

/*
 * The reference kernel's in-kernel dropout (isotropic/cuda/wf_embedding_kernel.cu):
 *   hash5(a, b, c, d, seed)                                              kernel.cu:27-41
 *       h = seed
 *       h ^= a * 0x85ebca6b + 0x9e3779b9;  h ^= b * 0xc2b2ae35 + 0x165667b1
 *       h ^= c * 0x27d4eb2f + 0xd6e8feb8;  h ^= d * 0x85ebca6b + 0x1b873593      (32-bit unsigned arithmetic)
 *       h = (h ^ (h >> 16)) * 0x85ebca6b;  h ^= h >> 13;  h = (h ^ (h >> 16)) * 0xc2b2ae35;  h ^= h >> 16
 *     (the reference's own hash: its last line resembles MurmurHash3's 32-bit finalizer but has one more shift-xor
 *      before the second multiply, so no published known answer applies.  Constants and order are restated from the
 *      source; only the reference's CUDA kernel could tell a typing slip in them: PARITY UNPINNED for the hash.
 *      The 32-bit arithmetic, the keep test and the sums are pinned in tests/test_oracle_we_dropout.py.)
 *   keep(z, i, j, k) = float(hash5(z, i, j, k, seed)) / float(UINT32_MAX) >= dropout_p          kernel.cu:43-46
 *   real = keep * real / (1 - dropout_p), imag likewise; the sums take real * dists, imag * dists   kernel.cu:227-238
 * The sums over sources are taken in double; mask, zero-distance rule and weights as we_oracle_mag_f64.
 */
uint32_t we_oracle_hash5(int a, int b, int c, int d, uint32_t seed)
{
    uint32_t h = seed;
    h ^= ((uint32_t)a * 0x85ebca6bu) + 0x9e3779b9u;
    h ^= ((uint32_t)b * 0xc2b2ae35u) + 0x165667b1u;
    h ^= ((uint32_t)c * 0x27d4eb2fu) + 0xd6e8feb8u;
    h ^= ((uint32_t)d * 0x85ebca6bu) + 0x1b873593u;
    h = (h ^ (h >> 16)) * 0x85ebca6bu;
    h ^= (h >> 13);
    h = (h ^ (h >> 16)) * 0xc2b2ae35u;
    h ^= (h >> 16);
    return h;
}

int we_oracle_dropout_keep(int z, int i, int j, int k, uint32_t seed, float dropout_p)
{
    const uint32_t h = we_oracle_hash5(z, i, j, k, seed);
    const float normalized = (float)h / (float)UINT32_MAX;
    return normalized >= dropout_p;
}

void we_oracle_dropout_f64(const float* coords, const float* wn, const uint8_t* mask, int Z, int N, int K,
                           int mag_type, float dropout_p, uint32_t seed, const int* rows, int nrows,
                           double* out, double* cs, double* ss)
{
    const double scale = 1.0 / (1.0 - (double)dropout_p);
    #pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int z = 0; z < Z; ++z)
    for (int rr = 0; rr < nrows; ++rr) {
        const int i = rows ? rows[rr] : rr;
        const float* c = coords + (size_t)z * N * 3;
        const uint8_t* m = mask ? mask + (size_t)z * N : NULL;
        double* o = out + ((size_t)z * nrows + rr) * 2 * K;
        double* pc = cs + ((size_t)z * nrows + rr) * K;
        double* ps = ss + ((size_t)z * nrows + rr) * K;
        for (int k = 0; k < K; ++k) { o[2*k] = o[2*k+1] = pc[k] = ps[k] = 0.0; }
        if (m && m[i]) continue;
        const double xi = c[3*i], yi = c[3*i+1], zi = c[3*i+2];
        for (int j = 0; j < N; ++j) {
            if (m && m[j]) continue;
            const double dx = xi - c[3*j], dy = yi - c[3*j+1], dz = zi - c[3*j+2];
            const double d2 = dx*dx + dy*dy + dz*dz;
            if (d2 == 0.0) continue;
            const double d = sqrt(d2);
            double w = 1.0;
            if (mag_type == 1) w = 1.0 / d;
            if (mag_type == 2) w = 1.0 / log2(d);
            if (mag_type == 3) w = 1.0 / sqrt(d);
            for (int k = 0; k < K; ++k) {
                if (dropout_p != 0.0f && !we_oracle_dropout_keep(z, i, j, k, seed, dropout_p)) continue;
                const double ph = d * (double)wn[k];
                const double co = cos(ph) * scale, si = sin(ph) * scale;
                o[2*k] += co * w; o[2*k+1] += si * w; pc[k] += co * w * d; ps[k] += si * w * d;
            }
        }
    }
}
