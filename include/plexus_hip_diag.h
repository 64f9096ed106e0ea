/*
 * plexus_hip_diag.h -- measurement probes of libplexus_hip.so.  Not part of the GCN-layer path and not needed by a
 * caller of it: the benchmark uses them to measure what the memory system gives to the path's access patterns.
 */
#ifndef PLEXUS_HIP_DIAG_H
#define PLEXUS_HIP_DIAG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Performs about n_gathers reads of uniformly random rows
 * (D fp32 each, D in {16, 32, 64, 128, 256}) of `table` with the SpMM's load shape and nothing else, so that
 * timing it gives the memory system's ceiling for this access pattern on a table of this size.
 * *gathers_done receives the exact count. */
int plx_diag_random_gather_f32(const float *table, int64_t rows, int64_t ld, int64_t D, int64_t n_gathers, int64_t *gathers_done,
                               float *sink, void *stream);

/* plx_spmm_csr_f32 (include/plexus_hip.h) restricted to one of the two parts a product with a hub pass is made of, so
 * that each can be timed by itself: parts = 1 runs the row kernel (with the sums of the split rows that are not hub
 * rows), 2 the hub pass, 3 both (the product).  With parts != 3 the rows of Y that belong to the other part are left
 * as they are.  A plan without a hub pass does everything in part 1. */
struct plx_spmm_plan;
int plx_diag_spmm_parts_f32(const struct plx_spmm_plan *plan, const float *val, const float *H, int64_t ldh, int64_t D, float *Y,
                            int64_t ldy, void *workspace, size_t workspace_bytes, int parts, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PLEXUS_HIP_DIAG_H */
