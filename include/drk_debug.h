/*
 * drk_debug.h -- diagnostic and tuning switches of libdrk_kv.so.  They are process-wide,
 * not thread-safe, and no part of the drop-in surface: tests use them to hold the kernels
 * against each other, the benchmark to time single kernels and to sweep launch shapes.
 * A product caller never needs this header.
 */
#ifndef DRK_DEBUG_H
#define DRK_DEBUG_H

#include "drk_kv.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Diagnostic: route every decode / prefill through the portable kernel (any
 * geometry, any storage type) instead of the tiled one, so that tests can
 * check the two against each other.  Process-wide, not thread-safe. */
void drk_debug_force_portable_decode(int on);
/* Diagnostic: which kernel produces the decode partials when the geometry allows
 * a choice: 0 = automatic (the persistent stream kernel), 2 = the fixed-split
 * tiled kernel (16-bit pages only), 3 = same as 0.  Process-wide. */
void drk_debug_set_decode_kernel(int which);
/* Diagnostic: workgroups of the persistent decode grid; 0 restores the default (512; 1024 for
 * 8-bit pages of head_dim 128). */
void drk_debug_set_stream_workgroups(int n);
/* Measurement aid: the persistent decode kernel leaves after its prologue (the scan of the branch
 * lengths and the workgroup's unit descriptors, one table read each) without reading a page or
 * writing a result -- the launch then costs what every launch pays before its first tile.
 * Outputs are garbage while this is on. */
void drk_debug_set_stream_descriptors_only(int on);
/* Diagnostic: context splits of the shared-prefix pass (default 64, at most 256; 0 restores the
 * default).  Changes drk_decode_shared_workspace_bytes. */
void drk_debug_set_shared_splits(int n);
/* Tuning: the shared-prefix pass for at most 64 rows per kv head and head_dim 128 runs on the
 * producer / consumer kernel (1, the default) or on the kernel every wave stages in (0). */
void drk_debug_set_prefix_stream(int on);
/* Diagnostic: 1 = drk_paged_decode_attention_shared never takes the grouped kernel (one launch over
 * shared and private tiles) but always the prefix pass + tail kernel pair; 0 = the library's choice. */
void drk_debug_set_grouped_decode(int mode);
/* The arithmetic that deals the fork-tree kernel's grid to its units, for tests on the CPU (no device call).
 * drk_debug_grouped_grid: the workgroups launched for group_units tiles of shared ranges and an upper bound of
 * tail_units_upper tail tiles (all kv heads counted), for a kernel whose descriptor table holds descriptor_table units.
 * drk_debug_grouped_region_split: out = {Gs, Us, Ut} -- workgroups [0, Gs) take runs of Us units of the shared ranges,
 * the others runs of Ut units of the tails (tail_runs = tails with at least one tile, all kv heads counted). */
int drk_debug_grouped_grid(int kvh, int group_units, int tail_units_upper, int descriptor_table);
void drk_debug_grouped_region_split(int group_units, int tail_units, int tail_runs, int grid, int descriptor_table, int out[3]);
/* Measurement aid for benchmarks: while on, the decode entry points launch the kernels that read the
 * pages and leave their partial results unmerged (no merge kernel: out is not written), so that an event
 * pair the caller records around a call brackets the dominant kernel(s) alone.  Process-wide. */
void drk_debug_set_skip_merge(int on);
/* Diagnostic: extra dynamic LDS bytes per decode workgroup (lowers occupancy). */
void drk_debug_set_decode_lds_pad(int bytes);
/* Tuning: which prefill chunks run with the context split over the chip (they must stand behind 2 048 tokens
 * or more): negative = the library's cost rule (default); 0 = none; n = every chunk of up to n rows. */
void drk_debug_set_prefill_split(int max_rows);
/* head_dim 256 chunk kernel: 0 = never cut the walks of the last round of workgroups into pieces (what it does
 * without a workspace); 1 (default) = cut them when a piece is eight tiles or more and the workspace
 * drk_prefill_workspace_bytes reports is passed; 2 = whenever a last round exists (tests). */
void drk_debug_set_prefill_pieces(int mode);
/* head_dim 256 chunk kernel on 16-bit pages: 1 (default) = eight waves per workgroup, a score wave (K Q^T, softmax)
 * and a value wave (V^T P^T) per 32 rows; 0 = four waves, each does both products of its 32 rows.  Same walks,
 * same pieces, same bits. */
void drk_debug_set_prefill_d256_waves(int mode);
/* Mass passes (drk_paged_prefill_attention_mass[_lse]): 1 (default) = the kernel that takes 256 rows per workgroup
 * and, on 16-bit pages, its K tiles straight into LDS (blocks of 16 * 2^k tokens; the two-walk call up to
 * 8 184 / 6 136 logical blocks of context at head_dim 128 / 256; 8-bit pages: the one-walk call at head_dim 128,
 * codes staged through registers); 0 = the register-staging kernel, which also serves every other case. */
void drk_debug_set_prefill_mass_direct(int on);
/* The one-walk mass kernels cut every walk into parts (ranges of tiles) when a chunk has few walks, so that a
 * short frame behind a long context fills the chip: 0 (default) = the library's rule (256 or 512 workgroups, a
 * part no shorter than eight tiles); n > 0 = n parts per walk, whatever their length (tests). */
void drk_debug_set_prefill_mass_parts(int parts);
/* Tuning: which causal chunks of head_dim 128 run on the two-phase chunk kernels (eight waves, 256 rows per
 * workgroup): 0 = none (the four-wave kernel); 1 = the library's rule (default: chunks long enough to give
 * most CUs a workgroup); 2 = every chunk the geometry allows; 3 = as 2, and 16-bit pages too go through
 * registers on their way into LDS (the kernel 8-bit pages always use) instead of straight from global memory.
 * Head_dim 256 on 16-bit pages: 1 and 2 = the direct-to-LDS kernel with one wave per SIMD, 0 and 3 = the four-wave
 * kernel that stages through registers. */
void drk_debug_set_prefill_two_phase(int mode);
/* Tuning: 16-byte chunks one workgroup moves per (layer, K|V) in the copying append, in
 * extract / inject, and in the quantising append (0 = default: 256, 512, 1024). */
void drk_debug_set_append_chunks(int copy_chunks, int flat_chunks, int quant_chunks);
/* Tuning: the quantising append takes 32 source bytes per thread (1, the default) or 16 (0: the
 * kernel it shares with the copying append; always used for head_dim 8). */
void drk_debug_set_quant_append_pairs(int on);
/* Self-check of the int8 scale arithmetic: the quantising kernels find a row's fp16 scale and its
 * reciprocal with one multiply and one residual correction per division; this runs that form and
 * the full IEEE divisions over every input that can occur (all bf16 and fp16 magnitudes, all fp16
 * scales) and adds the number of disagreements to *d_mismatches (device memory, 4 bytes, zeroed
 * by the caller).  Asynchronous on `stream`. */
int drk_debug_check_int8_scale_math(unsigned *d_mismatches, void *stream);

/* ---- probes: what the part reaches on its own (bench.py reports them beside the kernels) ---- */
/* Measurement aid (precedent tools/probe_bw.cu:74-97): sustained GB/s of a plain
 * 128-bit streaming read of `bytes` of device memory on the default stream,
 * 5 warm-up + `iters` timed passes; d_sink is 4 bytes of device memory.
 * Synchronises. */
int drk_probe_read_bandwidth(const void *d_ptr, size_t bytes, int iters, void *d_sink, float *gbps);
/* Same, with the decode kernels' access pattern: aligned granules of granule_bytes (a multiple of
 * 4096; 4096 = one 16-token K or V run of one kv head at head_dim 128, 16-bit) read in a
 * scattered order over the largest power-of-two number of granules that fits in `bytes`. */
int drk_probe_read_bandwidth_permuted(const void *d_ptr, size_t bytes, int granule_bytes, int iters,
                                      void *d_sink, float *gbps);
/* Measurement aid: dense bf16 TFLOP/s a registers-only v_mfma_f32_32x32x16_bf16 loop sustains
 * (8 waves per CU, four independent accumulator chains per wave, no memory traffic): the rate
 * the matrix cores of the part reach on their own.  d_sink is 4 bytes of device memory.
 * Synchronises. */
int drk_probe_mfma_rate(int iters, void *d_sink, float *tflops);
/* Measurement aid: how much of one wave's matrix products hides another wave's vector work on
 * the same SIMD.  One workgroup of eight waves per CU; waves 4-7 issue 32x32x16 bf16 products,
 * waves 0-3 a softmax-like mix of vector instructions (exp, fma, max3, pack), balanced to the
 * same issue time.  Reports the milliseconds of a launch with only the matrix waves working,
 * only the vector waves, and both: perfect overlap gives both = max, none gives the sum.
 * d_sink is 4 bytes of device memory.  Synchronises. */
int drk_probe_mfma_valu_coexec(int iters, void *d_sink, float *ms_mfma, float *ms_valu, float *ms_both);
/* Measurement aid: the same question for two waves that take turns, as the halves of a two-phase
 * prefill workgroup do: between two workgroup barriers waves 0-3 issue 32 products while waves 4-7
 * issue vector instructions of ONE kind (about 16 clocks' worth per product), then the roles swap.
 * op: 0 v_exp_f32, 1 v_fma_f32, 2 v_dot2_f32_bf16, 3 v_cvt_pk_bf16_f32, 4 v_max3_f32,
 * 5 v_cmp_gt_f32 (writes vcc), 6 v_permlane32_swap_b32, 7 s_nop 3.  Reports the milliseconds of a
 * launch with only the products, only the vector turns, and both; (both - products) / vectors is
 * the share of the vector time that stays visible.  d_sink is 4 bytes of device memory.  Synchronises. */
int drk_probe_phase_coexec(int op, int iters, void *d_sink, float *ms_products, float *ms_vectors, float *ms_both);

#ifdef __cplusplus
}
#endif
#endif /* DRK_DEBUG_H */
