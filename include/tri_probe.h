/* tri_probe.h - calibration kernels for one MI355X (libtri_probe.so). Not part of the attention operator's boundary
 * (include/tri_attn.h) and without a counterpart in the reference: bench.py --ceiling uses them to measure what the
 * matrix pipe sustains on this box. Status codes are those of tri_attn.h. */
#ifndef TRI_PROBE_H
#define TRI_PROBE_H
#ifdef __cplusplus
extern "C" {
#endif

/* Calibration helper with no counterpart in the reference: `workgroups` workgroups of 512 threads each run
 * iters x 64 bf16 32x32x16 MFMAs per wave on the caller's operand bits (operands: 16 * 512 * 16 bytes of
 * device memory read as bf16 values, e.g. random normals; out: workgroups * 512 floats).
 * mode 0: operands in registers; 1: every A operand read from LDS; 2: every LDS read feeds two MFMAs;
 * 3: the fp32 instruction (v_mfma_f32_32x32x2_f32), operands in registers.
 * Flops per launch = workgroups * 8 * iters * 64 * 32768 (mode 3: * 4096). Used by bench.py --ceiling. */
int tri_probe_mfma(int mode, int workgroups, int iters, const void* operands, float* out, void* stream);

/* Calibration, no counterpart in the reference: does vector-ALU work of one wave run in the shadow of another wave's
 * MFMAs on the same SIMD? Waves 0-3 of each 512-thread workgroup issue 16 MFMAs per loop trip (matrix 0:
 * v_mfma_f32_32x32x16_bf16, 1: v_mfma_f32_32x32x2_f32), waves 4-7 work on 32 values per lane per trip (valu 0: one fma
 * each, 1: one exp2 each, 2: fma + max + exp2 each). who: 1 = the matrix waves only, 2 = the vector waves only, 3 = both;
 * 4 = waves 0-3 do both kinds of work themselves (two values' vector work after each matrix step), waves 4-7 nothing.
 * operands: 10 * 512 * 16 bytes; out: workgroups * 512 floats. Used by bench.py --ceiling. */
int tri_probe_coexec(int matrix, int valu, int who, int workgroups, int iters, const void* operands, float* out,
                          void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TRI_PROBE_H */
