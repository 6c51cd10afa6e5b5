/*
 * aluminum_amd - test and benchmark support of the C-ABI library.
 *
 * Nothing declared here replaces an interface of the reference and nothing
 * here is needed to use the combine engine: these entry points let tests and
 * benchmarks produce seeded inputs in device memory and check the library's
 * 16-bit float conversions on their own.  The boundary proper is
 * aluminum_amd.h.
 */
#ifndef ALUMINUM_AMD_SUPPORT_H
#define ALUMINUM_AMD_SUPPORT_H

#include "aluminum_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Input distributions of the counter-based generator. */
typedef enum {
  ALAMD_DIST_UNIFORM_PM1 = 0, ALAMD_DIST_UNIFORM_09_11 = 1, ALAMD_DIST_UNIFORM_01 = 2,
  ALAMD_DIST_FULLRANGE = 3, ALAMD_DIST_BOOL01 = 4, ALAMD_DIST_NORMAL = 5,
  ALAMD_DIST_SMALLINT = 6
} alamd_dist;

/* dst[i] = value of element (idx0 + i) of stream `seed` under `dist`: a pure
 * integer hash followed by correctly rounded fp64 operations, so a host
 * implementation of the same formula yields the same bits.  (Stands in for
 * gen_data, test/test_utils.hpp:157-256, whose libstdc++ distributions are
 * not reproducible on a device.) */
int alamd_fill(void *dst, size_t count, int dtype, int dist, uint64_t seed,
               uint64_t idx0, void *stream);
/* The library's own fp32 -> fp16 / bf16 narrowing and the exact widening,
 * as used inside the combine kernels (exposed so that all 2^32 inputs can be
 * checked). */
int alamd_narrow_f32(void *dst16, const float *src, size_t count, int dtype, void *stream);
int alamd_widen_f32(float *dst, const void *src16, size_t count, int dtype, void *stream);
/* The sizes the launch planners cut their work by, for comparisons on a given
 * machine (they exist for measurements, not for production code).  The
 * settings are process-wide atomics: a call that runs while one changes sees
 * the old or the new value of each.  Value 0 restores the default.  Names:
 * launch_bytes, two_step_min_total_bytes, two_step_min_outputs,
 * two_step_piece_bytes, ring_piece_bytes, spread_launch_bytes,
 * spread_hbm_chunk_tiles, spread_hbm_launch_chunks, spread_cache_chunk_tiles,
 * spread_cache_launch_chunks (chunk lengths in units of 16 KiB);
 * stream_wgs_per_cu (one-wave workgroups per CU of a fold / tree launch; 0:
 * the library's choice by size, rank count and outputs), fold_front3_ranks
 * (rank count from which a fold asks for three streams up front instead of
 * two; 0: 12); block_shape_from_bytes and block_shape_below_bytes (a fold /
 * tree launch that reads and writes at least the first and less than the
 * second in all may work in tiles of 16 KiB with every load issued up front
 * instead of streaming; defaults 32 MiB and 384 MiB, between which the library
 * also looks at outputs, rank count and how evenly the tiles deal out over
 * the CUs; with other values every launch in the window does); halo_load_policy (the cache policy of the grid loads of a halo
 * pack: 0 plain, 1 nt, 2 sc1, 3 sc0 sc1, 4 sc0 sc1 nt).  Piece sizes below
 * 64 KiB are refused.  Results never depend on them, only speed. */
int alamd_tune(const char *name, size_t value);
size_t alamd_tuned(const char *name);
/* The number of kernel launches that alamd_combine makes for one output of
 * `count` elements folded from P ranks under a fold order (the launch planner's
 * own answer under the current settings; 0 for arguments it would refuse), so
 * that a benchmark can turn a call's duration into a launch's. */
size_t alamd_planned_launches(int P, size_t count, int dtype);
/* Polls after which a wait inside a chained in-place Reduce_scatterv launch
 * gives up (0 restores the default, 2^24): lets a test make waits expire
 * without anything being wrong with the device.  ALAMD_CHAIN_POLLS_NONE: every
 * wait that the tiling calls for gives up without looking at its flag, whether
 * the neighbouring tile has loaded or not - the same outcome on every device
 * and at every speed; every kernel still runs to its end.  Not synchronised
 * against running calls, like alamd_tune: a test's setting, made while
 * nothing else uses the library. */
#define ALAMD_CHAIN_POLLS_NONE 0xffffffffu
int alamd_set_chain_poll_limit(unsigned polls);
#ifdef __cplusplus
}
#endif
#endif
