/*
 * morphkv_diag -- tuning switches and measurement hooks of libmorphkv.so.
 *
 * Nothing here has a counterpart in the reference and nothing here is needed to
 * use the library: these entries pin a kernel variant for A/B runs and tests,
 * time individual launches with HIP events, and calibrate the matrix pipe.  The
 * switches are process-global and not thread-safe; production callers leave
 * them alone.  The reference-facing boundary is morphkv.h.
 */
#ifndef MORPHKV_DIAG_H
#define MORPHKV_DIAG_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Which phase-1 kernel
 * mkv_paged_attn_decode launches.  0 = by GQA group size (matrix cores when
 * Hq/Hkv >= 4, vector ALU otherwise), 1 = vector ALU, 2 = matrix cores. */
int mkv_set_decode_variant(int32_t variant);

/* Experiments and tests: pin the prefill kernel's workgroup shape.  Bits 0-7:
 * 0 = by the call (eight waves / 256 query rows per workgroup from 2048-token
 * chunks, or from 256-row chunks over at least 512 cached tokens, where that grid
 * still covers the chip; four waves / 128 rows otherwise),
 * 4 or 8 = always that shape.  Bits 8-9: 0 = a workgroup takes two query tiles
 * of its sequence unless the grid would be too small, 1 = always two, 2 = always
 * one. */
int mkv_set_prefill_variant(int32_t waves);

/* ---- measurement ---------------------------------------------------------- */
/* Kernel ids for mkv_prof_*. */
#define MKV_K_APPEND_DECODE   0
#define MKV_K_APPEND_PREFILL  1
#define MKV_K_ATTN_PHASE1     2
#define MKV_K_ATTN_PHASE2     3
#define MKV_K_MIGRATE         4
#define MKV_K_PREFILL_ATTN    5
#define MKV_K_FILL_ZERO       6
#define MKV_K_SWAP            7
#define MKV_K_ROPE_STORE      8
#define MKV_K_COUNT           9
/* Calibration of the matrix pipe (no counterpart in the reference): `iters` rounds of the prefill
 * kernel's 64 matrix instructions per wave (v_mfma_f32_16x16x32_f16) on 512 workgroups of four
 * waves, with nothing else in the loop.  mode 0: operands in registers, constant within an operand; 1: operands in
 * registers taken from data; 2: operands read from LDS in the prefill kernel's fragment pattern.
 * data: at least 64 KiB of fp16 values, 16-byte aligned; sink: 512 KiB scratch.  *flops (host,
 * may be NULL) receives the floating-point operations of the launch. */
int mkv_diag_mfma_loop(int32_t mode, int32_t iters, const void* data, void* sink, double* flops,
                       void* stream);

/* What the memory system gives a gather of 4 KiB slabs (no counterpart in the reference): `workgroups`
 * workgroups of 256 threads read slabs_per_wg slabs each, loads_in_flight (1, 2, 4, 8) per thread at a
 * time, workgroups_per_cu (1 ... 8) resident per CU; the slab is a hash of (workgroup, i) over
 * slabs_in_buf (a power of two) slabs of buffer a or b (4 KiB aligned, slabs_in_buf * 4096 bytes each).
 * by_xcd = 0: the buffer is one bit of the hash; by_xcd != 0: workgroups on XCD x (= workgroup id mod 8)
 * read b when bit x of xcd_mask is set, else a.  sink: 4 bytes of device scratch.  Reads only. */
int mkv_diag_slab_gather(const void* a, const void* b, uint64_t slabs_in_buf, int32_t workgroups,
                         int32_t slabs_per_wg, int32_t loads_in_flight, int32_t workgroups_per_cu, int32_t by_xcd,
                         uint32_t xcd_mask, void* sink, void* stream);

/* Per-workgroup time stamps of the attention kernels.  buf: device memory of
 * max_workgroups * MKV_TIMELINE_POINTS int64, zeroed by the caller; NULL switches
 * the stamps off.  While set, every launch of the prefill kernel and of the decode
 * phase-1 kernels whose grid has at most max_workgroups workgroups makes thread 0
 * of workgroup w (linear id, x fastest) store the GPU's constant-rate 100 MHz
 * counter into buf[w * MKV_TIMELINE_POINTS + k] at point k of its life -- prefill:
 * 0 entry, 1 first key tile staged, 2 key tiles done, 3 output written, 4-6 the
 * same three for the workgroup's second query tile; decode: 0 entry, 1 before the
 * block loop, 2 blocks done, 3 output stored.  Later launches overwrite earlier
 * ones: set it around ONE launch and synchronise. */
#define MKV_TIMELINE_POINTS 8
int mkv_diag_timeline(void* buf, int64_t max_workgroups);

/* The rule mkv_arena_pair_grow uses to tell memory groups apart (no counterpart in the reference),
 * on rates supplied by the caller: rates[i] is the two-stream fill rate of chunk i beside an anchor
 * chunk, self_rate the anchor's own (its two halves side by side).  same[i] = 1 where chunk i is judged
 * to lie in the anchor's group.  Host-only: runs without a GPU. */
int mkv_diag_split_by_rate(const double* rates, int64_t n, double self_rate, uint8_t* same);

/* When enabled, every launch of the kernels above is bracketed by a
 * hipEvent pair on its stream; mkv_prof_collect synchronises those events and
 * returns the launch count and summed duration since the last reset. */
int mkv_prof_enable(int32_t on);
int mkv_prof_reset(void);
int mkv_prof_collect(int32_t kernel_id, int64_t* launches, double* total_ms);

#ifdef __cplusplus
}
#endif
#endif /* MORPHKV_DIAG_H */
