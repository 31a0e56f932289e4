/* C interface of libkeops_calibrate.so, the benchmark's loop-only calibration kernels (keops_calibrate.hip).
 * Not part of the product library libkeops_hip.so nor of its ABI (include/keops_hip.h). */
#ifndef KEOPS_CALIBRATE_H
#define KEOPS_CALIBRATE_H
#ifdef __cplusplus
extern "C" {
#endif

/*
 * Loop-only calibration of the instruction issue rates the roofline fractions are held against: runs a grid of
 * `blocks` workgroups of 4 wavefronts, each wavefront issuing `iters` rounds of `chains` independent dependency
 * chains, and returns the elapsed time in ms and the counted instructions per wavefront.
 *   kind 0: v_fmac_f32 only (8 per chain and round); kind 1: the 9-instruction mix of a Gaussian pair (3 sub,
 *   mul, 2 fma, mul, v_exp_f32, fma); kind 2: the same without v_exp_f32; kind 3: v_mfma_f32_32x32x16_bf16
 *   (4 per chain and round); kind 4: v_mfma_f32_32x32x16_f16; kind 5: two chains of the bf16 instruction (8 per round)
 *   with `chains` independent v_fmac_f32 after every matrix instruction (what fits beside a saturated matrix pipe).
 *   chains: 1, 2, 4, 8 (kinds 0-2), 1, 2, 4 (kinds 3, 4, 6) or 0, 1, 2, 4, 8 (kind 5); kind 6: v_mfma_i32_32x32x32_i8
 *   (4 per chain and round); kind 7: two chains of 16 matrix instructions per round whose operands change with every
 *   instruction (16 A x 16 B register sets of random data, as when tiles stream through a kernel), chains = 0: the
 *   bf16 instruction, 1: f16, 2: signed bytes; kind 8: the inner loop of the signed-byte nearest-neighbour filter
 *   without its memory traffic (per round two query sets of two dependent v_mfma_i32_32x32x32_i8 and the minimum
 *   over the 16 results of a set), chains = 0: minima over the results, 1: over registers that no matrix instruction
 *   writes, 2: no vector work; kind 9: the contraction loop of the high-dimensional chunked kernel on its own
 *   (workgroups of 8 wavefronts, 32 rows of 256 components per wavefront in registers as hi and lo half-precision
 *   operands, 32-row tiles streamed through LDS, 48 v_mfma_f32_32x32x16_f16 per round and wavefront, no vector
 *   work), chains = 0: every operand the same constant, 1: random operands with the magnitudes of real data.
 *   kind 10: the Gaussian pair with every operation rounded on its own (12 instructions), `chains` = 1, 2, 4 pairs
 *   advanced statement by statement (11, 12: one / two pairs with log2(e) in a scalar register); kind 11: written-out
 *   instruction sequences at the rate of one kind of instruction each, `chains` = sequence 0 .. 12 (keops_valu_seq_loop);
 *   kind 12: the stream of the Gaussian sweep alone (workgroups of 8 wavefronts: 4 v_mfma_f32_32x32x16_bf16 per 32
 *   pairs, v_exp_f32 and `chains` = 1, 4, 8 v_fmac_f32 per pair; counted: the v_exp_f32).
 * Measurement aid without counterpart in the reference; used by bench.py --valu-calibration / --mfma-calibration.
 * Returns 0, or a negative code (bad arguments, device, allocation, events, kind or chains out of range).
 */
int keops_calibrate(int device_id, int kind, int chains, int blocks, int iters, double* ms, double* instr_per_wave);

/*
 * One v_mfma_f32_32x32x16_bf16 on operands given bit for bit (bfloat16 patterns): out[i * 32 + j] = acc0 +
 * sum_k a[i][k] b[j][k] for a_bits[32][16], b_bits[32][16] (host arrays), as the matrix core adds it.  The tests use it
 * to pin the model of that adder which the error bound of the matrix-core exponents rests on.  Returns 0 or a negative
 * code.
 */
int keops_calibrate_mfma_probe(int device_id, const unsigned short* a_bits, const unsigned short* b_bits, float acc0, float* out);

#ifdef __cplusplus
}
#endif
#endif /* KEOPS_CALIBRATE_H */
