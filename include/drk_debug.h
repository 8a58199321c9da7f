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
/* Diagnostic for benchmarks: while on, every decode launch (up to 256 per
 * session; switching it on starts a new session) records a HIP event on its
 * stream right before and right after the split-K partial kernel; the merge
 * kernel is outside the pair.  drk_debug_decode_kernel_times waits for the pairs
 * recorded so far and returns their elapsed milliseconds.  Launch back to back
 * (no host sync in between) so that the queue stays busy and the pairs bracket
 * the kernel tightly.  Process-wide. */
void drk_debug_time_decode_kernel(int on);
int  drk_debug_decode_kernel_times(float *ms, int cap, int *count);
/* Diagnostic: extra dynamic LDS bytes per decode workgroup (lowers occupancy). */
void drk_debug_set_decode_lds_pad(int bytes);
/* Tuning: which prefill chunks run with the context split over the chip (they must stand behind 2 048 tokens
 * or more): negative = the library's cost rule (default); 0 = none; n = every chunk of up to n rows. */
void drk_debug_set_prefill_split(int max_rows);
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

#ifdef __cplusplus
}
#endif
#endif /* DRK_DEBUG_H */
