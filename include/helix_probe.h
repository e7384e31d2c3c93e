/*
 * helix_probe.h -- C ABI of the measurement aids built beside the kernel-template libraries.
 *
 * Not part of the template ABI (helix_abi.h) and without a counterpart in the reference: the reference reports
 * TFLOP/s only; here every rate is also quoted against what the part can do, and the matrix pipes of this part
 * run against a power limit on random operands, so the attainable ceiling is measured next to the datasheet one.
 */
#ifndef HELIX_PROBE_H
#define HELIX_PROBE_H

#ifdef __cplusplus
extern "C" {
#endif

#define HELIX_PROBE_API __attribute__((visibility("default")))

/* Runs a loop of v_mfma_f32_16x16x32_f16 and nothing else on every compute unit: 256 workgroups of eight waves,
 * each wave the 4 x 8 accumulator tiles and the two k-steps of operand fragments of the 64 x 128 wave tile the
 * 256 x 256 x 64 GEMM tile uses, operands held in registers (read once from a buffer of seeded values in
 * [-0.17, 0.17), standard deviation 0.1, or of zeros).  `warmup` untimed launches, then `launches` launches of
 * `loops` iterations between two HIP events on the default stream.
 *   *seconds_per_launch : mean duration;  *flop_per_launch : 2 * 16 * 16 * 32 per MFMA, summed over the launch.
 * Allocates its operand buffer (about 50 MB) for the duration of the call.  Returns 0 or a hipError_t value. */
HELIX_PROBE_API int helix_mfma_probe(int zero_operands, int warmup, int launches, int loops, double* seconds_per_launch,
                                     double* flop_per_launch);

#ifdef __cplusplus
}
#endif

#endif /* HELIX_PROBE_H */
