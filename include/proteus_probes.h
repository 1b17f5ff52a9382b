/*
 * C ABI of libproteus_probes.so: measurement probes for gfx950, NOT part of the product library.
 *
 * Instruction-rate, accuracy and co-issue micro-benchmarks that state, from measurement, the denominators of the
 * issue models the benchmark reports beside the kernels' times.  Nothing in libproteus_hip.so or the Python operators
 * depends on them; bench.py and the test of the hardware sin/cos error load this library.  No counterpart in the
 * reference.  Return codes as in proteus_hip.h (0, < 0 argument error, > 0 hipError_t).
 */
#ifndef PROTEUS_PROBES_H
#define PROTEUS_PROBES_H

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Instruction-rate probe used to state the roofline denominator of the WE
 * kernel.  Runs `iters` rounds of 64 independent chains of one VALU
 * instruction per lane on `blocks` x 256 threads and writes one float per
 * thread to `sink` (blocks * 256 floats; so the work cannot be removed).  The
 * caller times the launch; lane-ops issued = blocks*256*iters*64.  No
 * counterpart in the reference.
 *   op: 0 v_fma_f32, 1 v_mul_f32, 2 v_add_f32 (second operand a scalar register),
 *       3 v_sin_f32, 4 v_cos_f32, 5 v_exp_f32, 6 v_rsq_f32, 7 v_fract_f32;
 *       8 v_fmac_f32 and 9 v_add_f32 with vector-register operands only.
 */
int proteus_probe_valu_rate(int op, int blocks, int iters, float* sink, void* stream);

/*
 * Accuracy probe of the hardware sin/cos path used by the WE kernel:
 * s[i] = v_sin_f32(y), c[i] = v_cos_f32(y) with x in revolutions and
 * y = fract(x[i]) if use_fract else x[i] (the instructions accept |y| <= 256),
 * and q[i] = refined sqrt path r = r2*rsq(r2) applied to x[i].
 */
int proteus_probe_sincos(const float* x, float* s, float* c, float* q, int n, int use_fract, void* stream);

/*
 * Co-issue probe behind the attention forward's issue model (no counterpart in the reference).  Every wave runs
 * `iters` loop trips of eight "slots"; a slot is what the attention kernel's inner loop issues per 32x32x16 bf16
 * matrix product: that product and the softmax work of two scores (2 fused multiply-adds, 2 exp2, 1 pack to bf16,
 * 1 packed row-sum add).  mode 0: the matrix products only; 1: the vector work only; 2: both.  Modes 3-6 replace
 * the vector work, to tell which kind of vector instruction runs beside a matrix product: 3: twelve ordinary fused
 * multiply-adds per slot, alone; 4: those with the products; 5: four exp2 per slot, alone; 6: those with the
 * products.  `blocks`
 * workgroups of 256 threads (512 on a 256-CU chip = two waves per SIMD, the attention kernel's occupancy);
 * sink [blocks*256] f32 receives values that keep the work alive.  Time the launch with events.
 */
int proteus_probe_mfma_softmax_slot(int mode, int blocks, int iters, float* sink, void* stream);

/*
 * Do transcendental and ordinary vector instructions of different waves of one SIMD overlap?  `blocks` workgroups of
 * 4 * waves_per_simd waves, one per compute unit (each asks for 96 KB of LDS), so every SIMD holds waves_per_simd
 * waves; on each SIMD the first k_trans of them run iters_trans links of 64 independent v_sin_f32 chains and the
 * others iters_valu links of 64 independent v_fmac_f32 chains (vector-register operands only).  Time the launch with
 * k_trans = waves_per_simd or iters_valu = 0 (transcendentals alone), with k_trans = 0 or iters_trans = 0 (ordinary
 * alone) and with both: were nothing to overlap, the mixed launch would take the sum of the other two.
 *   sink   [blocks * 256 * waves_per_simd] f32, keeps the work alive
 *   census [blocks * 4] u32: per workgroup and SIMD, (waves placed there << 16) | waves that took the transcendental
 *          role; the placement the probe relies on (waves_per_simd waves of a workgroup per SIMD) is checked from it
 */
int proteus_probe_trans_valu_mix(int waves_per_simd, int k_trans, int blocks, int iters_trans, int iters_valu,
                                 float* sink, unsigned* census, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PROTEUS_PROBES_H */
