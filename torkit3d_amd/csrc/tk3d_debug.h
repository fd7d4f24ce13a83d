/*
 * tk3d_debug.h - entry points for the tests and the benchmark only.
 *
 * They are exported by libtk3d.so but are no part of the operator boundary (tk3d.h):
 * nothing a caller of the library needs is here. They exist so that a test can aim an
 * input at one particular kernel whatever the dispatcher would choose for its shape, so
 * that the benchmark can count the work a launch executed, and so that the error bound
 * the matrix-core pre-filters rely on is checked against the hardware.
 * Conventions are those of tk3d.h (device pointers, no allocation, no synchronisation).
 */
#ifndef TK3D_DEBUG_H
#define TK3D_DEBUG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Routes of tk3d_debug_chamfer_forward_route_f32. */
enum {
    TK3D_CHAMFER_ROUTE_EXACT = 1,   /* chamfer_forward_kernel: every pair in the canonical form */
    TK3D_CHAMFER_ROUTE_VECTOR = 2,  /* chamfer_forward_filter_kernel (key clouds >= 512)        */
    TK3D_CHAMFER_ROUTE_MATRIX4 = 3, /* chamfer_forward_mfma_kernel, four query blocks per wave  */
    TK3D_CHAMFER_ROUTE_MATRIX2 = 4, /* chamfer_forward_mfma_kernel, two query blocks per wave   */
    TK3D_CHAMFER_ROUTE_MATRIX_SLICED = 5 /* ... with every key cloud cut into slices of 1024    */
};

/* tk3d_chamfer_distance_forward_f32 through one named kernel. TK3D_ERR_UNSUPPORTED when the
 * kernel does not take the shape (VECTOR: a key cloud under 512 points; MATRIX: the longer
 * cloud under 1024 points or an empty cloud). */
int tk3d_debug_chamfer_forward_route_f32(const float *xyz1, const float *xyz2, int64_t B,
                                         int64_t N1, int64_t N2, float *dist1, int64_t *idx1,
                                         float *dist2, int64_t *idx2, int route, void *stream);

/* tk3d_chamfer_distance_forward_ws_f32 with the sorted path forced (as `always` does in the
 * size function), stage by stage and with its work counted.
 * `stages`: 1 the launches that sort the clouds and build the key terms, 2 the pruned sweep
 * (on a workspace that stage 1 has filled for the same clouds), 4 the hand-over check; 7 is
 * the whole call.
 * `counters`: NULL, or device memory for four uint64 words, cleared by the call itself; the
 * sweep then runs in a counting build and leaves in counters[0] the number of (tile of 32 keys,
 * block of 32 queries) matrix instructions it issued, in counters[1] the number of waves that
 * swept, in counters[2] the queries that took an exact scan and in counters[3] the clouds handed
 * to the sweep of all pairs. */
int tk3d_debug_chamfer_forward_sorted_counted_f32(const float *xyz1, const float *xyz2,
                                                  int64_t B, int64_t N1, int64_t N2,
                                                  float *dist1, int64_t *idx1, float *dist2,
                                                  int64_t *idx2, void *workspace,
                                                  size_t workspace_bytes,
                                                  unsigned long long *counters, int stages,
                                                  void *stream);

/* One v_mfma_f32_32x32x16_f16 on caller-supplied terms: key_terms [T][32][16] and query_terms
 * [T][32][16] hold fp16 bit patterns (uint16), scores [T][32 keys][32 queries] receives
 * sum_i key[k][i] * query[q][i] as the instruction accumulates it from zero. */
int tk3d_debug_mfma_dot16_f16(const uint16_t *key_terms, const uint16_t *query_terms, int64_t T,
                              float *scores, void *stream);

/* The pre-filter score of the chamfer kernels for centred, scaled points: keys [T][32][3] and
 * queries [T][32][3] are split into fp16 terms exactly as the kernels stage them
 * (chamfer_key_terms / chamfer_query_terms) and multiplied by the matrix instruction;
 * scores [T][32 keys][32 queries] approximates |k|^2 - 2 q.k. */
int tk3d_debug_chamfer_scores_f32(const float *keys, const float *queries, int64_t T,
                                  float *scores, void *stream);

/* tk3d_knn_distance_f32 through the pre-filtered kernel (knn_filter_kernel_f32, scores on
 * the matrix cores) whatever the launch size; k <= 16 and at least 256 keys. */
int tk3d_debug_knn_filter_f32(const float *query, const float *key, int64_t B, int64_t N1,
                              int64_t N2, int64_t k, float *distance, int64_t *index,
                              void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TK3D_DEBUG_H */
