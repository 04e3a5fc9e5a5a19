/* espetero_ceilings.h -- measured machine ceilings for the attention path's two rooflines
 * (libespetero_ceilings.so, built from espetero_amd/csrc/ceilings.hip; gfx950 only).
 *
 * No counterpart among the reference's kernels; its documentation holds its kernels against
 * measured limits of the machine rather than data-sheet figures (docs/kernel-guidelines.md:19-27:
 * a measured stream bandwidth and a measured MMA rate). The first two calls produce the same two
 * figures on an MI355X, the third the ceiling of the prefill kernels' own step; bench.py reports them (--workload hbm_read_ceiling, mfma_issue_ceiling, prefill_step_ceiling)
 * and states every roofline fraction against the data-sheet peak and against them.
 * Conventions as in espetero_attn.h: device pointers, work enqueued on `stream`, 0 or an error
 * code (1 bad argument, 2 unsupported, 3 launch failure). start_event / stop_event: two
 * hipEvent_t (or both NULL) that take the kernel's own begin and end.
 */
#ifndef ESPETERO_CEILINGS_H
#define ESPETERO_CEILINGS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A plain streaming read: n_pages pages of page_bytes (a multiple of 4096) from `base`, page i of the
 * launch being pages[i] (device array; NULL: page i itself, i.e. address order), 16 bytes per lane per
 * load, two pages in flight per wavefront, `workgroups` workgroups of 4 wavefronts. nontemporal: the
 * loads carry the streaming hint the decode kernel's K / V loads carry. sink: one device word. */
int esp_ceiling_hbm_read(const void* base, const int32_t* pages, int32_t n_pages, int32_t page_bytes, int32_t nontemporal,
                         int32_t workgroups, uint32_t* sink, void* stream, void* start_event, void* stop_event);

/* The matrix cores under a wavefront that also issues vector arithmetic: every wavefront runs
 * iters x 32 v_mfma_f32_32x32x16_bf16 (four accumulator chains), and per matrix instruction
 * valu_per_mfma fp32 fused multiply-adds plus exp_per_mfma (v_exp_f32 + one add), no memory access.
 * random_data: the matrix operands are random 16-bit floats, as an attention pass has them (1), or the
 * constant 1.0 (0): the multipliers draw more power on random operands and the clock, and with it the
 * ceiling, settles lower - the figure a kernel with real data can be held against is the one with 1.
 * Supported: exp_per_mfma 0 with valu_per_mfma 0, 1, 2, 3, 4, 6; exp_per_mfma 1 with 0 .. 5.
 * Workgroups of 4 wavefronts, at most two per compute unit. out: workgroups * 256 floats.
 * Flops of a launch: workgroups * 4 * iters * 32 * 32768. */
int esp_ceiling_mfma_issue(int32_t valu_per_mfma, int32_t exp_per_mfma, int32_t random_data, int32_t workgroups, int32_t iters, float* out, void* stream,
                           void* start_event, void* stop_event);

/* The prefill kernels' key step as a bare instruction stream, one ingredient more per stage: 0 = 32
 * v_mfma_f32_32x32x16_bf16 per step in chains of 8 with operands in registers; 1 = + every A operand read from
 * LDS a group ahead; 2 = + a workgroup barrier per step; 3 = + the softmax's share of vector work behind the
 * matrix instructions of two of the four groups; 4 = + every wavefront staging 8 KB per step from `src` (a
 * device buffer of at least 4 MB + 64 KB, cache resident) straight into LDS. rows: 1 = 32 query rows per wavefront,
 * two workgroups per compute unit (the kernels as built); 2 = 64 rows, every operand read feeding two matrix
 * instructions, one workgroup per compute unit (stages 1, 3, 4 only). What stage 4 reaches is the ceiling of
 * that kernel design; the difference between stages is what each ingredient costs. clk (NULL or 2 * workgroups
 * 64-bit words): cycles and 100 MHz ticks each workgroup was alive; cycles / ticks * 100 MHz is the clock the
 * part ran at. out: workgroups * 256 floats. Flops of a launch: workgroups * 4 * iters * 32 * rows * 32768. */
int esp_ceiling_prefill_step(int32_t stage, int32_t rows, int32_t random_data, int32_t workgroups, int32_t iters, float* out, const void* src,
                             unsigned long long* clk, void* stream, void* start_event, void* stop_event);

/* The key step of the 256-dim prefill kernel as bare instruction streams, in three shapes of the workgroup. Per step a
 * compute unit multiplies 64 keys with 128 query rows of one head (the flops of 256 v_mfma_f32_32x32x16), every A operand
 * read from LDS, with 32 scores per row of softmax arithmetic and one barrier. shape: 0 = 4 wavefronts x 32 rows, one per
 * SIMD (the kernel as built); 1 = 8 wavefronts as 4 pairs, each wavefront taking half of the step's keys through Q K^T and
 * the softmax, handing its packed P to its partner through LDS and multiplying all 64 keys' P with its half of the dims;
 * 2 = 8 wavefronts x 16 rows on v_mfma_f32_16x16x32, each a whole head. loads: 0 = none, 1 = the step's 64 KB staged from
 * `src` (a device buffer of at least 8 MB + 64 KB, cache resident) straight into LDS behind the barrier, 2 (shape 0 only) =
 * one load behind each of the step's first 16 matrix instructions, 3 (shape 0 only) = a second barrier in mid-step and
 * every wavefront's loads one by one beside two groups of matrix instructions that are its own (never two wavefronts
 * loading at a time). 4, 5, 6 (shape 0 only) = 0, 2, 1 with the operand reads issued one by one, each behind the matrix
 * instruction that frees its register, instead of a group's eight in a row. One workgroup per compute unit. clk as above.
 * out: workgroups * 512 floats. Flops of a launch: workgroups * iters * 256 * 32768. */
int esp_ceiling_prefill_step256(int32_t shape, int32_t loads, int32_t workgroups, int32_t iters, float* out, const void* src, unsigned long long* clk,
                                void* stream, void* start_event, void* stop_event);

#ifdef __cplusplus
}
#endif
#endif /* ESPETERO_CEILINGS_H */
