/*
 * samfast_bench - measurement and tuning aids exported by libsamfast.so beside the path's C ABI
 * (include/samfast.h).  Nothing here has a counterpart in the reference and nothing here is needed
 * to run the path: bench.py and the tests use these entry points to time bare matrix-instruction
 * loops and to switch kernel variants inside one process.
 */
#ifndef SAMFAST_BENCH_H
#define SAMFAST_BENCH_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Kernel variants are chosen by knobs, each named like the environment variable that gives its
 * initial value (read once per process): SAMFAST_GEMM_TM, SAMFAST_GEMM_WG3, SAMFAST_GEMM_TILE,
 * SAMFAST_GEMM_SMALL_BELOW, SAMFAST_GEMM_PERSIST, SAMFAST_GEMM_PERSIST_SKEW, SAMFAST_GEMM_PERSIST_PRIO,
 * SAMFAST_GEMM_SPLITK,
 * SAMFAST_ATTN_WAVES, SAMFAST_ATTN_WINDOW_ROWS, SAMFAST_SPARSE_PERSIST.  This
 * call sets one (`unset` != 0: back to "not given", `value` ignored).  Every variant of a kernel
 * returns the same bits; the knobs only move time.  Returns SAMFAST_E_INVALID for an unknown name.
 */
int samfast_bench_set_knob(const char* name, int value, int unset);

/*
 * Measurement aid, no counterpart in the reference: one launch of a kernel that does nothing
 * but matrix instructions on operands held in registers (no global loads, no LDS, no barriers)
 * - the rate a GEMM or attention kernel built from the same instruction can approach at best
 * on the same kind of data.  instruction 0 = v_mfma_i32_32x32x32_i8, 1 =
 * v_mfma_f32_32x32x16_bf16.  `operands` holds 4 (A, B) pairs of 16 bytes for each of 256 lanes
 * (8 * 256 * 16 bytes, [pair][A|B][lane]); their values decide what the multipliers toggle.
 * `workgroups` of 256 threads run `iters` rounds of 8 independent instructions per wavefront
 * (workgroups * iters <= 2^27, about a second of GPU time; more returns SAMFAST_E_INVALID);
 * *host_ops_out (may be NULL) receives the arithmetic operations of the launch.  `scratch_out`
 * (>= 1 KiB) receives nothing in practice (see the kernel).  Timing is the caller's (events on `stream`).
 */
int samfast_bench_mfma_ceiling(
    int instruction, const void* operands, int workgroups, int iters,
    int64_t* host_ops_out, void* scratch_out, void* stream);

/*
 * Measurement aid, no counterpart in the reference: how much vector work runs in the shadow of
 * another wavefront's matrix instructions on the same SIMD.  Workgroups of 512 threads, one per
 * CU: wavefronts 0-3 run `mfma_rounds` rounds of eight independent v_mfma_f32_32x32x16_bf16 on
 * operands held in registers, wavefronts 4-7 (their SIMD partners) `vector_rounds` rounds of 64
 * independent vector instructions - vector_kind 0: v_fma_f32, 1: v_exp_f32 + v_mul_f32.  Either
 * count may be 0, which times one side alone; workgroups * (mfma_rounds + vector_rounds) <= 2^27.  `operands`: at least 8 KiB (two 16-byte vectors for
 * each of 256 lanes); `scratch_out`: 2 KiB the kernel may write.  bench.py --mfma-ceiling uses it.
 */
int samfast_bench_mfma_valu_overlap(
    int vector_kind, const void* operands, int workgroups, int mfma_rounds, int vector_rounds,
    void* scratch_out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SAMFAST_BENCH_H */
