/* Measurement aids of the gfx950 quantized-matmul library: libloken_probes.so, a library of its own
 * that only the benchmark loads (loken_amd/probes.py). No counterpart in the reference and no
 * product path calls them: they give the measured denominators reported beside the nominal
 * MI355X peaks. Status codes as in loken_gfx950.h. */
#ifndef LOKEN_PROBES_H
#define LOKEN_PROBES_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* `workgroups` workgroups of 256 threads that end at once: the floor of one launch. */
int lk_probe_empty(int workgroups, void* stream);
/* Reads `bytes` (a multiple of 16, 16-byte aligned) from `src` and writes nothing. pattern 1, 2,
 * 4, 8: grid-strided, that many 16-byte loads per thread in flight; 0: every workgroup walks its
 * own contiguous share. `sink` is 4 bytes of device memory (never written in practice). */
int lk_probe_read(const void* src, int64_t bytes, int workgroups, int pattern, void* sink, void* stream);
/* Register-resident matrix-unit loop: each of a workgroup's four matrix waves issues `iters` x 4
 * independent instructions of `kind` (0 v_mfma_i32_32x32x32_i8, 1 v_mfma_f32_32x32x16_f16,
 * 2 v_mfma_i32_16x16x64_i8, 3 v_mfma_i32_32x32x16_i8). valu_per_mfma (a multiple of 8) independent f32 fmas ride along per
 * matrix instruction: in the same wave (mode 0), or in four further waves, one beside each matrix
 * wave on its SIMD (mode 1). *ops (nullable, host memory) receives the matrix operations launched. */
int lk_probe_mfma(int kind, int workgroups, int iters, int valu_per_mfma, int mode, void* sink, double* ops,
                  void* stream);

/* How vector instructions issue beside matrix instructions. A wave runs iters x 4 slots; a slot is
 * one matrix instruction of `kind` (0 v_mfma_f32_32x32x16_f16, 1 v_mfma_i32_32x32x32_i8,
 * 2 v_mfma_i32_16x16x64_i8, 3 none) into one of four independent accumulator tiles and `valu`
 * (0, 4, 8, 12, 16, 24 or 32) f32 fmas, on registers of their own (dep 0) or reading the tile whose
 * instruction was issued two slots earlier (dep 1). kind 4 is the tile kernels' item: two chained
 * f16 instructions from a zero accumulator with `valu` (4, 8, 12, 16) fmas of the previous item's
 * result behind each. waves_per_simd 1 or 2 (workgroups of 256 or 512 threads). Nothing in the
 * kernels waits on an instruction in flight. */
int lk_probe_overlap(int kind, int valu, int dep, int waves_per_simd, int workgroups, int iters, void* sink,
                     void* stream);

#ifdef __cplusplus
}
#endif
#endif
