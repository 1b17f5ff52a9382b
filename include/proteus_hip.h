/*
 * proteus_hip.h -- C ABI of libproteus_hip.so (gfx950 / MI355X).
 *
 * Operators of jaimec00/proteusAI behind plain pointers and sizes:
 *   - the Wavefunction Embedding (WE) forward, isotropic and anisotropic, and
 *   - the RBF-scaled geometric flash-attention forward.
 *
 * Conventions shared by every entry point
 *   - All pointers are DEVICE pointers owned by the caller; the library borrows
 *     them for the duration of the launch and keeps nothing.  Tensor outputs are
 *     fully overwritten (no reliance on zero-initialisation, no atomics).  The one
 *     exception are the per-head scalars d_sigma and d_beta of proteus_geo_attn_bwd:
 *     they are ACCUMULATED into with atomic adds and must be zeroed by the caller.
 *   - All tensors are dense and contiguous in the stated layout.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     Launches are asynchronous; no entry point synchronises.
 *   - Return value: 0 = launched; < 0 = argument error found BEFORE any HIP call
 *     (so it can be exercised on a machine without a GPU); > 0 = a hipError_t
 *     reported by the launch.  proteus_strerror() names any of them.
 */
#ifndef PROTEUS_HIP_H
#define PROTEUS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes (negative = argument errors) ---- */
#define PROTEUS_OK                 0
#define PROTEUS_ERR_NULL_POINTER  -1   /* a required pointer is NULL              */
#define PROTEUS_ERR_BAD_SHAPE     -2   /* Z, N, K, H <= 0 or above the limits     */
#define PROTEUS_ERR_BAD_HEAD_DIM  -3   /* d_head is not 32, 64 or 128             */
#define PROTEUS_ERR_BAD_LAYOUT    -4   /* unknown coords_layout value             */
#define PROTEUS_ERR_BAD_ALIGNMENT -5   /* a pointer is not aligned as required    */
#define PROTEUS_ERR_BAD_TUNING    -6   /* unknown tuning/variant selector         */
#define PROTEUS_ERR_UNSUPPORTED   -7   /* legacy option not implemented           */
#define PROTEUS_ERR_TOO_LARGE     -8   /* beyond the fixed capacity of an entry point that allocates nothing */
#define PROTEUS_ERR_BAD_OPERAND_TYPE -9 /* operand_type is neither PROTEUS_OPERAND_BF16 nor PROTEUS_OPERAND_F16 (dtype: neither PROTEUS_DTYPE_*) */

/* 16-bit type of Q, K, V (and dO) where an entry point takes an operand_type */
#define PROTEUS_OPERAND_BF16 0
#define PROTEUS_OPERAND_F16  1

/* element type of the tensors of proteus_add_layernorm_fwd and of dO in proteus_geo_attn_delta */
#define PROTEUS_DTYPE_F32  0
#define PROTEUS_DTYPE_BF16 1
#define PROTEUS_DTYPE_F16  2   /* proteus_geo_attn_delta only */

/* ---- coordinate layouts accepted by proteus_we_fwd ---- */
#define PROTEUS_COORDS_SOA 0   /* [Z,3,N]: what the reference's wrapper hands its kernel */
#define PROTEUS_COORDS_AOS 1   /* [Z,N,3]: what the Python module receives               */

/* ---- limits ---- */
#define PROTEUS_WE_MAX_N   (1 << 22)
#define PROTEUS_WE_MAX_K   4096
#define PROTEUS_ATTN_MAX_N (1 << 20)
#define PROTEUS_WE_BWD_STATIC_MAX_K 512   /* most wavenumbers proteus_we_bwd_static takes */

/*
 * Library version (major*10000 + minor*100 + patch) as a number that only grows.  PROTEUS_VERSION is the version this
 * header describes; a caller built against it should refuse a library whose proteus_version() differs in
 * major*10000 + minor*100 (argument lists have changed between minors: since 210 the beta-weighted forward and every
 * backward entry point take `int operand_type` before `tuning` / `stream`; a caller built against an older header
 * would pass its tuning selector there).  The Python binding checks for an exact match when it loads the library.
 */
#define PROTEUS_VERSION 301
int proteus_version(void);

/* Human-readable text for a return code of any entry point. */
const char* proteus_strerror(int code);

/*
 * Isotropic Wavefunction Embedding forward (magnitude 1/|r|, no dropout).
 *
 * Replaces the reference's native entry `wf_embedding_kernel.forward(coords,
 * wavenumbers, out, cos_sums, sin_sums, magnitude_type, dropout_p, rng_seed)`
 *   utils/model_utils/wf_embedding/isotropic/cuda/wf_embedding_if.cpp:20-77
 * and the launcher + kernel it calls
 *   utils/model_utils/wf_embedding/isotropic/cuda/wf_embedding_kernel.cu:49-344
 * for magnitude_type == 1 and dropout_p == 0 (the only values the module passes,
 *   utils/model_utils/wf_embedding/wf_embedding.py:44).
 *
 * Semantics, for batch z, observer i, wavenumber k, with
 *   valid(i,j) = !mask[z,i] && !mask[z,j] && |r_i - r_j|^2 != 0 :
 *     out[z,i,2k]     = sum_j valid * cos(k_k r_ij) / r_ij
 *     out[z,i,2k+1]   = sum_j valid * sin(k_k r_ij) / r_ij
 *     cos_sums[z,i,k] = sum_j valid * cos(k_k r_ij)
 *     sin_sums[z,i,k] = sum_j valid * sin(k_k r_ij)
 *   A masked observer's rows are all zero.
 *
 * Difference from the reference: padding is an explicit byte mask (non-zero =
 * padded) instead of the sentinel x == 12345 baked into the coordinates
 * (isotropic/cuda/wf_embedding.py:29, wf_embedding_kernel.cu:154); a genuine
 * coordinate of 12345.0 is therefore NOT masked here.
 *
 *   coords       [Z,3,N] or [Z,N,3] f32, per coords_layout
 *   wavenumbers  [K] f32 (any sign)
 *   mask         [Z,N] u8, non-zero = padded; may be NULL (nothing padded)
 *   out          [Z,N,2K] f32     cos_sums, sin_sums  [Z,N,K] f32, or BOTH NULL: then they are
 *                not computed (inference: nothing is kept for the backward; a faster kernel)
 *   tuning       0 = automatic; otherwise a variant selector (see
 *                proteus_we_num_variants / proteus_we_variant_name)
 */
int proteus_we_fwd(const float* coords, int coords_layout,
                   const float* wavenumbers, const uint8_t* mask,
                   float* out, float* cos_sums, float* sin_sums,
                   int Z, int N, int K, int tuning, void* stream);

/* Validation half of proteus_we_fwd: same checks, no HIP call, no launch. */
int proteus_we_fwd_check(const float* coords, int coords_layout,
                         const float* wavenumbers, const uint8_t* mask,
                         const float* out, const float* cos_sums, const float* sin_sums,
                         int Z, int N, int K, int tuning);

int         proteus_we_num_variants(void);
const char* proteus_we_variant_name(int tuning);

/*
 * proteus_we_fwd with the source weight m(r) of the reference's other
 * `magnitude_type` values (isotropic/cuda/wf_embedding_kernel.cu:192-206):
 *   0: m = 1    1: m = 1/r (the same as proteus_we_fwd)    2: m = 1/log2(r)    3: m = 1/sqrt(r)
 *     out[z,i,2k], out[z,i,2k+1] = sum_j valid * m cos(k_k r), sum_j valid * m sin(k_k r)
 *     cos_sums, sin_sums         = sum_j valid * m r cos(k_k r), ... sin   (kernel.cu:237-238)
 * Any other magnitude_type returns PROTEUS_ERR_UNSUPPORTED.  The reference's
 * in-kernel dropout is proteus_we_dropout_fwd.
 */
int proteus_we_legacy_fwd(const float* coords, int coords_layout,
                          const float* wavenumbers, const uint8_t* mask,
                          float* out, float* cos_sums, float* sin_sums,
                          int Z, int N, int K, int magnitude_type, void* stream);

/*
 * The forward with the reference kernel's in-kernel dropout: the native entry's dropout_p and rng_seed
 * (isotropic/cuda/wf_embedding_if.cpp:20-25; kernel.cu:27-46 the hash, :227-232 its use).  The term of
 * (batch item z, observer i, source j, wavenumber k) is kept iff
 *     float(hash5(z, i, j, k, rng_seed)) / float(UINT32_MAX) >= dropout_p
 * and what is kept is divided by 1 - dropout_p; cos_sums / sin_sums carry the same mask and factor (they are what the
 * backward for the wavenumbers contracts, so the gradient is that of the masked sum).  The hash is integer
 * arithmetic: the mask is the reference's to the bit for the same seed (its wrapper draws a fresh seed per call,
 * isotropic/cuda/wf_embedding.py:48-49; here the caller passes it).  i and j are token indices, k the index of
 * the wavenumber.
 *   magnitude_type 0 .. 3 as proteus_we_legacy_fwd; cos_sums and sin_sums are required
 *   dropout_p      0 <= dropout_p < 1 (else PROTEUS_ERR_BAD_SHAPE); 0 keeps every term
 * proteus_we_dropout_threshold: the smallest value of the hash that is kept for a given dropout_p (host only).
 */
int proteus_we_dropout_fwd(const float* coords, int coords_layout,
                           const float* wavenumbers, const uint8_t* mask,
                           float* out, float* cos_sums, float* sin_sums,
                           int Z, int N, int K, int magnitude_type, float dropout_p, uint32_t rng_seed, void* stream);
int proteus_we_dropout_fwd_check(const float* coords, int coords_layout,
                                 const float* wavenumbers, const uint8_t* mask,
                                 const float* out, const float* cos_sums, const float* sin_sums,
                                 int Z, int N, int K, int magnitude_type, float dropout_p);
uint32_t proteus_we_dropout_threshold(float dropout_p);

/*
 * Anisotropic (C-beta scaled, learnable wavenumber) Wavefunction Embedding
 * forward: the variant WaveFunctionEmbedding(anisotropic=True) calls
 *   utils/model_utils/wf_embedding/wf_embedding.py:41-42.
 *
 * Replaces the reference's native entry `wf_embedding_kernel.forward(coordsA,
 * coordsB, cb_magnitudes, wavenumbers, out, d_cb, d_k)`
 *   anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding.py:57-61
 * and its kernel
 *   anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding_kernel.cu:30-224
 * (paths under utils/model_utils/wf_embedding/).
 *
 * Semantics, for observer i, source j, index k, with R = a_i - a_j, r = |R|,
 * A = (b_j . R)/r, u = r - cb_k A, phase = u k_k, over the pairs with both
 * tokens unpadded and r != 0:
 *     out [z,i,2k] = sum_j cos(phase)/r          out [z,i,2k+1] = sum_j sin(phase)/r
 *     d_k [z,i,2k] = sum_j -sin(phase) u / r     d_k [z,i,2k+1] = sum_j  cos(phase) u / r
 *     d_cb[z,i,2k] = sum_j  sin(phase) k_k A / r d_cb[z,i,2k+1] = sum_j -cos(phase) k_k A / r
 *   A masked observer's rows are all zero.  Padding is an explicit byte mask,
 *   as in proteus_we_fwd (the reference bakes x == 12345 into coordsA, :36).
 *
 *   coordsA, coordsB  [Z,3,N] or [Z,N,3] f32, both per coords_layout
 *                     (positions; per-token C-beta direction vectors)
 *   cb_magnitudes, wavenumbers  [K] f32
 *   mask              [Z,N] u8, non-zero = padded; may be NULL
 *   out, d_cb, d_k    [Z,N,2K] f32, 16-byte aligned.  d_cb and d_k may both be NULL (not one of them): then only
 *                     the embedding is computed, with two running sums per wavenumber instead of six.
 */
int proteus_we_aniso_fwd(const float* coordsA, const float* coordsB, int coords_layout,
                         const float* cb_magnitudes, const float* wavenumbers, const uint8_t* mask,
                         float* out, float* d_cb, float* d_k,
                         int Z, int N, int K, int tuning, void* stream);

/* Validation half of proteus_we_aniso_fwd: same checks, no HIP call. */
int proteus_we_aniso_fwd_check(const float* coordsA, const float* coordsB, int coords_layout,
                               const float* cb_magnitudes, const float* wavenumbers, const uint8_t* mask,
                               const float* out, const float* d_cb, const float* d_k,
                               int Z, int N, int K, int tuning);

int         proteus_we_aniso_num_variants(void);
const char* proteus_we_aniso_variant_name(int tuning);

/*
 * Backward of the wavefunction embedding: the contraction of dO with what the
 * forward kept.  Replaces the tensor expressions of
 *   isotropic/cuda/wf_embedding.py:64-83
 *     d_wavenumbers[k] = sum_{z,n} dO[z,n,2k+1] cos_sums[z,n,k] - dO[z,n,2k] sin_sums[z,n,k]
 *   anisotropic/cb_scaling/learnable_wavenumbers/cuda/wf_embedding.py:65-79
 *     g_cb[k] = sum_{z,n} dO[z,n,2k] d_cb[z,n,2k] + dO[z,n,2k+1] d_cb[z,n,2k+1]   (g_k likewise from d_k)
 *
 *   d_out [Z,N,2K] f32 (8-byte aligned); cos_sums, sin_sums [Z,N,K]; d_cb, d_k [Z,N,2K];
 *   outputs [K] f32, fully overwritten.  In the anisotropic call a gradient that is not
 *   wanted is skipped by passing NULL for both its partials and its output.
 *   workspace: device memory of at least proteus_we_bwd_workspace_bytes(Z, N, K) bytes,
 *   owned by the caller, overwritten; calls that share one workspace must not overlap.
 *   Deterministic (no atomics); bound by HBM: 16 / 24 bytes per (token, wavenumber).
 */
size_t proteus_we_bwd_workspace_bytes(int Z, int N, int K);

int proteus_we_bwd(const float* d_out, const float* cos_sums, const float* sin_sums,
                   float* d_wavenumbers, float* workspace, size_t workspace_bytes,
                   int Z, int N, int K, void* stream);
int proteus_we_bwd_check(const float* d_out, const float* cos_sums, const float* sin_sums,
                         const float* d_wavenumbers, const float* workspace, size_t workspace_bytes,
                         int Z, int N, int K);

/*
 * proteus_we_bwd for callers that cannot allocate device memory or hand over a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  Same kernels and the same,
 * bit-identical result as proteus_we_bwd; the partial sums live in a 2 MiB array in
 * the library's own device image instead of a workspace, which every GPU the library
 * runs on holds until the process ends.  Calls no hipMalloc / hipFree.
 *   K > PROTEUS_WE_BWD_STATIC_MAX_K returns PROTEUS_ERR_TOO_LARGE (before any HIP call).
 *   The GPU that is current at the call must be the one `stream` belongs to.
 *   All calls on one GPU share that GPU's array: calls that overlap there (two
 *   streams, two threads) race; serialise them.  Nothing has to be cleared between calls.
 *   The first call made with a given GPU current looks the array's address up (hipGetSymbolAddress, under a mutex)
 *   and may load the library's device image: make that first call per GPU outside stream capture; every later call
 *   only launches its two kernels and can be captured.
 */
int proteus_we_bwd_static(const float* d_out, const float* cos_sums, const float* sin_sums,
                          float* d_wavenumbers, int Z, int N, int K, void* stream);

int proteus_we_aniso_bwd(const float* d_out, const float* d_cb, const float* d_k,
                         float* g_cb, float* g_k, float* workspace, size_t workspace_bytes,
                         int Z, int N, int K, void* stream);
int proteus_we_aniso_bwd_check(const float* d_out, const float* d_cb, const float* d_k,
                               const float* g_cb, const float* g_k,
                               const float* workspace, size_t workspace_bytes, int Z, int N, int K);

/*
 * RBF-scaled geometric flash-attention forward.
 *
 * Replaces the Triton launch `_attn_fwd[grid](...)` made by
 *   old/old_scripts/attn/geometric_attn.py:552-607 (kernel :57-260)
 * with the logits of README.md:40:
 *     s_ij = (q_i . k_j)/sqrt(d) * (1 + exp(-|r_i - r_j|^2 / (2 sigma_h^2)))
 *     s_ij = -inf where key j is padded
 *     O_i  = softmax_j(s_ij) V_j ;  L_i = logsumexp_j(s_ij)
 *   Padded query rows and rows without any valid key give O = 0, L = -inf
 *   (geometric_attn.py:196,233-236).
 *
 *   Q, K, V      [Z,H,N,d_head] bf16 (raw uint16 bit patterns), 16-byte aligned; d_head = 32, 64 or 128
 *                (the reference's kernel takes any d_k >= 16, geometric_attn.py:597; its test runs 32,
 *                tests/attn/geo_attn.py:15-17), anything else returns PROTEUS_ERR_BAD_HEAD_DIM
 *   coords       [Z,N,3] f32
 *   sigma        [H] f32, > 0 (not checked on the device)
 *   key_pad_mask [Z,N] u8, non-zero = padded; may be NULL
 *   O            [Z,H,N,d_head] f32, 16-byte aligned
 *   L            [Z,H,N] f32; may be NULL (then not written)
 *   tuning       0 = automatic; otherwise a variant selector
 */
int proteus_geo_attn_fwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                         const float* coords, const float* sigma,
                         const uint8_t* key_pad_mask,
                         float* O, float* L,
                         int Z, int H, int N, int d_head, int tuning, void* stream);

/* Validation half of proteus_geo_attn_fwd: same checks, no HIP call. */
int proteus_geo_attn_fwd_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                               const float* coords, const float* sigma,
                               const uint8_t* key_pad_mask,
                               const float* O, const float* L,
                               int Z, int H, int N, int d_head, int tuning);

/*
 * proteus_geo_attn_fwd with a caller-provided workspace (d_head = 64).  The reference's launch gives every (batch,
 * head, query tile) item one program whose key loop is as long as the sequence
 * (old/old_scripts/attn/geometric_attn.py:586-599): a padded batch lasts as long as its longest sequence, and a batch
 * with fewer items than the chip has workgroup slots leaves most of it idle.  With a workspace the key loop of an item
 * may be cut into parts that go to several workgroups, whose partial results meet in the workspace (the last of an
 * item's parts to finish adds them up, in a fixed order: the result does not depend on which one that is).  Same result
 * as proteus_geo_attn_fwd up to the rounding of the probabilities (a part re-bases its softmax reference where the whole
 * item would not).
 *   strides      as proteus_geo_attn_fwd_strided, or NULL for contiguous [Z,H,N,d_head] tensors
 *   key_pad_mask may be NULL
 *   workspace    device memory, 256-byte aligned, workspace_bytes >= proteus_geo_attn_fwd_workspace_bytes(Z, H, N,
 *                d_head, tuning); not initialised by the caller, nothing kept in it between calls; calls that share
 *                one workspace must not overlap.  NULL / too small, or a shape for which
 *                proteus_geo_attn_fwd_workspace_bytes returns 0: the call is proteus_geo_attn_fwd[_strided].
 *   tuning       0 = automatic: the split-items schedule (9) for a padded batch with N >= 1024 and at least 8192
 *                    (item, key tile) steps in the full batch, and for an unpadded batch with N > 2048 and fewer than 512
 *                    items (the size function answers for the shape alone, as if either could be the case);
 *                9 = split items wherever possible (d_head = 64, Z <= 256, fewer than 2^30 steps): when the live items
 *                    are fewer than the chip's workgroup slots, the longest are cut along the keys into equal parts
 *                    until the parts fill the slots; parts are handed out longest first;
 *                8 = the balanced schedule wherever possible (same limits): all (item, key tile) steps as one line, cut
 *                    into equal shares for a persistent grid of two workgroups per compute unit;
 *                proteus_geo_attn_fwd_workspace_bytes returns 0 where the given tuning takes neither
 * Launches (both schedules): a plan kernel (last unpadded token of every query tile, arrival counters) and the grid,
 * which falls back to direct vector-ALU distances, whole items in turn, if a query tile's tokens lie too far apart
 * for the matrix-core distances.
 */
size_t proteus_geo_attn_fwd_workspace_bytes(int Z, int H, int N, int d_head, int tuning);
int proteus_geo_attn_fwd_ws(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const int64_t* strides,
                            const float* coords, const float* sigma, const uint8_t* key_pad_mask,
                            float* O, float* L, void* workspace, size_t workspace_bytes,
                            int Z, int H, int N, int d_head, int tuning, void* stream);
int proteus_geo_attn_fwd_ws_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const int64_t* strides,
                                  const float* coords, const float* sigma, const uint8_t* key_pad_mask,
                                  const float* O, const float* L, const void* workspace, size_t workspace_bytes,
                                  int Z, int H, int N, int d_head, int tuning);

/*
 * The same kernel with the logits of the reference's Triton kernel instead of
 * the README multiplier (old/old_scripts/attn/geometric_attn.py:193-201, launch
 * :588-599; dense statement tests/attn/geo_attn.py:194-210):
 *     rbf   = exp(-|r_i - r_j|^2 / (2 sigma_h^2))
 *     s_ij  = S_ij + beta_h * (2 (rbf - min_rbf)/(max_rbf - min_rbf) - 1) * |S_ij|,   S_ij = q_i.k_j/sqrt(d)
 *     s_ij  = -inf where key j or query i is padded or rbf is outside [min_rbf, max_rbf]
 *   beta [H] f32; requires max_rbf > min_rbf.
 *   operand_type: PROTEUS_OPERAND_F16 reads Q, K, V as fp16 and runs the products on v_mfma_f32_32x32x16_f16, as
 *   the reference does (it casts to fp16, geometric_attn.py:567-569); PROTEUS_OPERAND_BF16 as proteus_geo_attn_fwd.
 *   Everything else as proteus_geo_attn_fwd.
 */
int proteus_geo_attn_legacy_fwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                const float* coords, const float* sigma, const float* beta,
                                const uint8_t* key_pad_mask,
                                float* O, float* L,
                                int Z, int H, int N, int d_head,
                                float min_rbf, float max_rbf, int operand_type, int tuning, void* stream);

/*
 * Backward of both attention forwards: dQ, dK, dV, d sigma (and d beta).
 *
 * Replaces the Triton launch `_attn_bwd[grid](...)` of
 *   old/old_scripts/attn/geometric_attn.py:627-648 (kernel :262-543).
 * The caller passes what the reference's wrapper computes around that launch (:609-660):
 * dO cast to the operand type, D = rowsum(O * dO), the forward's L, and dQ/dK/dV/d_sigma/d_beta
 * buffers.  beta == NULL selects the README logits (proteus_geo_attn_fwd), otherwise the
 * logits and pair mask of proteus_geo_attn_legacy_fwd.
 *
 *   Q, K, V, dO   [Z,H,N,d_head] (raw uint16), 16-byte aligned; d_head = 32, 64 or 128; bf16, or fp16 with
 *                 operand_type = PROTEUS_OPERAND_F16 (legacy logits only: beta != NULL, else PROTEUS_ERR_BAD_OPERAND_TYPE)
 *   coords [Z,N,3] f32; sigma [H] f32; beta [H] f32 or NULL; key_pad_mask [Z,N] u8 or NULL
 *   L, D          [Z,H,N] f32
 *   dQ, dK, dV    [Z,H,N,d_head] f32, 16-byte aligned, fully overwritten (zeros at padded tokens)
 *   d_sigma       [H] f32, ACCUMULATED into with atomic adds (as the reference does, :541-543):
 *                 zero it first; may be NULL.  d_beta likewise (legacy logits only).
 */
int proteus_geo_attn_bwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                         const float* coords, const float* sigma, const float* beta,
                         const uint8_t* key_pad_mask, const float* L, const float* D,
                         float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
                         int Z, int H, int N, int d_head, float min_rbf, float max_rbf, int operand_type, void* stream);

/* Validation half of proteus_geo_attn_bwd: same checks, no HIP call. */
int proteus_geo_attn_bwd_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                               const float* coords, const float* sigma, const float* beta,
                               const uint8_t* key_pad_mask, const float* L, const float* D,
                               const float* dQ, const float* dK, const float* dV,
                               const float* d_sigma, const float* d_beta,
                               int Z, int H, int N, int d_head, float min_rbf, float max_rbf, int operand_type);

/*
 * The same forward and backward on tensors that are not contiguous [Z,H,N,d_head].
 *
 * The reference's Triton launches take every tensor's strides
 * (old/old_scripts/attn/geometric_attn.py:588-599, :627-648); these entry
 * points take the (batch, head, token) strides in ELEMENTS, the head dimension
 * being contiguous:
 *   forward   strides[12] : Q, K, V, O
 *   backward  strides[21] : Q, K, V, dO, dQ, dK, dV
 * so that slices of a fused [Z,N,3,H,d] projection are read in place and O or the
 * gradients are written in the memory order their consumer wants (e.g. [Z,N,H,d]).
 * Per tensor: token stride >= d_head, no negative stride, batch / head stride 0 only for
 * Z == 1 / H == 1 (else PROTEUS_ERR_BAD_LAYOUT); every stride a multiple of 16 bytes
 * (PROTEUS_ERR_BAD_ALIGNMENT); N * token stride below 2^31 bytes (forward) or
 * 2^30 elements (backward) (PROTEUS_ERR_BAD_SHAPE).  coords, sigma, beta, the mask, L and D stay
 * contiguous.  Everything else is as for proteus_geo_attn_fwd / proteus_geo_attn_bwd.
 */
int proteus_geo_attn_fwd_strided(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                 const int64_t* strides,
                                 const float* coords, const float* sigma, const uint8_t* key_pad_mask,
                                 float* O, float* L,
                                 int Z, int H, int N, int d_head, int tuning, void* stream);
int proteus_geo_attn_fwd_strided_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                       const int64_t* strides,
                                       const float* coords, const float* sigma, const uint8_t* key_pad_mask,
                                       const float* O, const float* L,
                                       int Z, int H, int N, int d_head, int tuning);
int proteus_geo_attn_legacy_fwd_strided(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                                        const int64_t* strides,
                                        const float* coords, const float* sigma, const float* beta,
                                        const uint8_t* key_pad_mask,
                                        float* O, float* L,
                                        int Z, int H, int N, int d_head,
                                        float min_rbf, float max_rbf, int operand_type, int tuning, void* stream);
int proteus_geo_attn_bwd_strided(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                 const int64_t* strides,
                                 const float* coords, const float* sigma, const float* beta,
                                 const uint8_t* key_pad_mask, const float* L, const float* D,
                                 float* dQ, float* dK, float* dV, float* d_sigma, float* d_beta,
                                 int Z, int H, int N, int d_head, float min_rbf, float max_rbf, int operand_type, void* stream);
int proteus_geo_attn_bwd_strided_check(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* dO,
                                       const int64_t* strides,
                                       const float* coords, const float* sigma, const float* beta,
                                       const uint8_t* key_pad_mask, const float* L, const float* D,
                                       const float* dQ, const float* dK, const float* dV,
                                       const float* d_sigma, const float* d_beta,
                                       int Z, int H, int N, int d_head, float min_rbf, float max_rbf, int operand_type);

/*
 * D = rowsum(O * dO), the term the attention backward subtracts from dP.  Replaces the torch expression
 * `D = torch.sum(O*dO, dim=3)` of the reference's backward wrapper (old/old_scripts/attn/geometric_attn.py:618);
 * its result is the `D` argument of proteus_geo_attn_bwd.  One launch, HBM-bound, no workspace.
 *   O        f32, rows of d_head elements contiguous and 16-byte aligned
 *   dO       dO_dtype = PROTEUS_DTYPE_F32, _BF16 or _F16 (what autograd hands over, before any cast); rows of d_head
 *            elements contiguous, starting on multiples of 4 elements
 *   strides  NULL: both tensors contiguous [Z,H,N,d_head]; else 6 element strides, (batch, head, token) of O then of
 *            dO, each a multiple of 4 and non-negative, token strides >= d_head
 *   D        f32 [Z,H,N] contiguous
 */
int proteus_geo_attn_delta(const float* O, const void* dO, const int64_t* strides, float* D,
                           int Z, int H, int N, int d_head, int dO_dtype, void* stream);
int proteus_geo_attn_delta_check(const float* O, const void* dO, const int64_t* strides, const float* D,
                                 int Z, int H, int N, int d_head, int dO_dtype);

int         proteus_geo_attn_num_variants(void);
const char* proteus_geo_attn_variant_name(int tuning);

/*
 * Residual add + LayerNorm of the post-LN encoder layer, inference forward:
 *   out[r, :] = LayerNorm(x[r, :] + res[r, :]) * gamma + beta        over the last dimension D
 * Replaces the torch expressions `self.attn_norm(q + self.dropout(attn))` and `self.ffn_norm(q + self.dropout(ffn))`
 * of old/old_scripts/encoder.py:36-39 with dropout inactive (nn.LayerNorm(d_model), old/old_scripts/encoder.py:27,31),
 * evaluated as torch does: the sum rounded to the tensors' type, mean and biased variance in fp32, eps under the
 * square root.  One launch, HBM-bound, no workspace.
 *   x, out        [rows, D] contiguous, dtype PROTEUS_DTYPE_F32 or PROTEUS_DTYPE_BF16 (all tensors of one type)
 *   res           [rows, D] or NULL (plain LayerNorm)
 *   gamma, beta   [D] or NULL (no scale / no shift)
 *   D             a multiple of 4 (f32) or 8 (bf16), at most 2048 (f32) or 4096 (bf16); pointers 16-byte aligned
 *   out may be x or res (every row is read completely before it is written)
 */
int proteus_add_layernorm_fwd(const void* x, const void* res, const void* gamma, const void* beta, void* out,
                              long rows, int D, float eps, int dtype, void* stream);
int proteus_add_layernorm_fwd_check(const void* x, const void* res, const void* gamma, const void* beta, const void* out,
                                    long rows, int D, float eps, int dtype);

#ifdef __cplusplus
}
#endif
#endif /* PROTEUS_HIP_H */
