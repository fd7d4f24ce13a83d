/*
 * tk3d.h - C ABI of the MI355X (gfx950) point-cloud operator library.
 *
 * One entry point per kernel family of the reference extension torkit3d._C
 * (torkit3d/csrc/torkit3d.cpp:13-21). Each function below names the reference
 * interface it replaces. The reference passes at::Tensor objects and allocates
 * its outputs; here every argument is a plain device pointer, a size or a scalar:
 *
 *   - all pointers are DEVICE pointers on the current HIP device, 16-byte aligned
 *     or better is not required (natural alignment of the element type is);
 *   - tensors are dense row-major: xyz [B,N,3], features [B,C,N], indices int64;
 *   - outputs are caller-allocated and fully overwritten (no pre-zeroing needed);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     kernels are enqueued on it and the call returns without synchronising;
 *   - nothing is allocated or freed, nothing throws;
 *   - the return value is TK3D_OK (0), a negative TK3D_ERR_* argument error
 *     (nothing was launched), or a positive hipError_t from the launch.
 *
 * `_f32` entry points take float data, `_f64` double data (the reference
 * instantiates both through AT_DISPATCH_FLOATING_TYPES).
 *
 * Distances are squared Euclidean, evaluated for key k and query q as
 *   fma(dz,dz, fma(dy,dy, dx*dx)),  dx = k.x - q.x, ...
 * which is what the reference kernels compute under nvcc's default contraction.
 */
#ifndef TK3D_H
#define TK3D_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TK3D_VERSION 100 /* major*10000 + minor*100 + patch */

enum {
    TK3D_OK = 0,
    TK3D_ERR_NULL_POINTER = -1,  /* a required pointer is NULL              */
    TK3D_ERR_BAD_SIZE = -2,      /* negative size, or a product overflows   */
    TK3D_ERR_BAD_K = -3,         /* k / num_samples outside the legal range */
    TK3D_ERR_BAD_VERSION = -4,   /* knn `version` not 0 or 1                */
    TK3D_ERR_WORKSPACE = -5,     /* workspace missing or too small          */
    TK3D_ERR_UNSUPPORTED = -6    /* shape beyond what the kernels index     */
};

/* Library version (TK3D_VERSION of the build). */
int tk3d_version(void);

/* Static, human-readable text for a return code of this library (negative codes)
 * or of the HIP runtime (positive codes). Never NULL. */
const char *tk3d_error_string(int code);

/* ---- chamfer / nearest-neighbour distance ---------------------------------
 * Replaces chamfer_distance_forward_cuda
 * (torkit3d/csrc/include/chamfer_distance.h:6-8, cuda/chamfer_distance_kernel.cu:91-151).
 * dist1[b,i] = min_j d2(xyz1[b,i], xyz2[b,j]), idx1[b,i] = the lowest such j;
 * dist2/idx2 likewise with the clouds swapped. An empty or all-NaN opposite
 * cloud gives (+inf, -1) in fp32. B, N1, N2 may be 0. The fp32 call may enqueue up
 * to three kernels and keeps partial results in idx1 / idx2 (8-byte aligned, as any
 * int64 array is) while they run; all four outputs are final when the last one ends. */
int tk3d_chamfer_distance_forward_f32(const float *xyz1, const float *xyz2,
                                      int64_t B, int64_t N1, int64_t N2,
                                      float *dist1, int64_t *idx1, float *dist2,
                                      int64_t *idx2, void *stream);
int tk3d_chamfer_distance_forward_f64(const double *xyz1, const double *xyz2,
                                      int64_t B, int64_t N1, int64_t N2,
                                      double *dist1, int64_t *idx1, double *dist2,
                                      int64_t *idx2, void *stream);

/* The same operation (chamfer_distance_kernel.cu:91-151) for callers that can lend
 * scratch memory. With `workspace` (256-byte aligned device memory of at least
 * tk3d_chamfer_distance_forward_workspace_bytes(B, N1, N2, 1) bytes, contents irrelevant
 * before and after) both clouds are first sorted along a space-filling curve, and a wave
 * then sweeps only the key tiles that can hold a nearest neighbour of its queries; three
 * kernels are enqueued (five when a cloud has more than 16384 points). Results are
 * bit-identical to tk3d_chamfer_distance_forward_f32 for
 * every input. The size function returns 0 for shapes the path cannot serve (a cloud of
 * more than 65536 points, B = 0) and, with always = 0, also for shapes where it is not
 * the faster route (small or very unequal clouds): callers that pass on that size, and a
 * null workspace when it is 0, get the faster route for every shape. With a null, short
 * or misaligned workspace the call is tk3d_chamfer_distance_forward_f32. */
size_t tk3d_chamfer_distance_forward_workspace_bytes(int64_t B, int64_t N1, int64_t N2,
                                                     int always);
int tk3d_chamfer_distance_forward_ws_f32(const float *xyz1, const float *xyz2,
                                         int64_t B, int64_t N1, int64_t N2,
                                         float *dist1, int64_t *idx1, float *dist2,
                                         int64_t *idx2, void *workspace,
                                         size_t workspace_bytes, void *stream);

/* chamfer_distance_forward_cuda on channel-first clouds xyz1 [B,3,N1], xyz2 [B,3,N2], read
 * in place: what the reference's chamfer_distance / nn_distance with transpose=True compute
 * after copying both clouds to [B,N,3] (torkit3d/ops/chamfer_distance.py:52-55,68-70).
 * Outputs as above. `workspace` may be NULL; with the workspace of the call above (fp32,
 * both clouds of at most 16384 points) the sorted path is taken. */
int tk3d_chamfer_distance_forward_bcn_f32(const float *xyz1, const float *xyz2,
                                          int64_t B, int64_t N1, int64_t N2,
                                          float *dist1, int64_t *idx1, float *dist2,
                                          int64_t *idx2, void *workspace,
                                          size_t workspace_bytes, void *stream);
int tk3d_chamfer_distance_forward_bcn_f64(const double *xyz1, const double *xyz2,
                                          int64_t B, int64_t N1, int64_t N2,
                                          double *dist1, int64_t *idx1, double *dist2,
                                          int64_t *idx2, void *stream);

/* Replaces chamfer_distance_backward_cuda
 * (chamfer_distance.h:10-16, chamfer_distance_kernel.cu:200-274).
 * grad_xyz1[b,i] = 2*gd1[b,i]*(x1[b,i]-x2[b,idx1[b,i]])
 *                  - sum over {j: idx2[b,j]==i} 2*gd2[b,j]*(x2[b,j]-x1[b,i]),
 * and symmetrically for grad_xyz2. Index entries outside [0,N) contribute nothing. */
int tk3d_chamfer_distance_backward_f32(const float *grad_dist1,
                                       const float *grad_dist2, const float *xyz1,
                                       const float *xyz2, const int64_t *idx1,
                                       const int64_t *idx2, int64_t B, int64_t N1,
                                       int64_t N2, float *grad_xyz1,
                                       float *grad_xyz2, void *stream);
int tk3d_chamfer_distance_backward_f64(const double *grad_dist1,
                                       const double *grad_dist2,
                                       const double *xyz1, const double *xyz2,
                                       const int64_t *idx1, const int64_t *idx2,
                                       int64_t B, int64_t N1, int64_t N2,
                                       double *grad_xyz1, double *grad_xyz2,
                                       void *stream);

/* ---- k nearest neighbours --------------------------------------------------
 * Replaces knn_distance_cuda
 * (torkit3d/csrc/include/knn_distance.h:7-11, cuda/knn_distance_kernel.cu:187-298).
 * distance/index are [B,N1,k]: the k smallest squared distances and their key
 * indices in the slot order of the reference's MinK structure
 * (torkit3d/csrc/include/mink.cuh:61-89), not sorted. Requires 1 <= k <= N2.
 * `version` (0 or 1) selects between two kernels in the reference that return
 * identical results; it is validated and otherwise ignored. */
int tk3d_knn_distance_f32(const float *query, const float *key, int64_t B,
                          int64_t N1, int64_t N2, int64_t k, int version,
                          float *distance, int64_t *index, void *stream);
int tk3d_knn_distance_f64(const double *query, const double *key, int64_t B,
                          int64_t N1, int64_t N2, int64_t k, int version,
                          double *distance, int64_t *index, void *stream);

/* KNN on [B,3,N] clouds (query [B,3,N1], key [B,3,N2]), the layout the reference's
 * models hold: knn_points(..., transpose=True) copies both clouds to [B,N,3] before the
 * call (torkit3d/ops/knn_points.py:40-45). Same result as tk3d_knn_distance_* on the
 * transposed clouds, without the copies, for k <= 64. Returns TK3D_ERR_UNSUPPORTED (nothing
 * launched) for k > 64: the caller then copies as the reference does. */
int tk3d_knn_distance_bcn_f32(const float *query, const float *key, int64_t B,
                              int64_t N1, int64_t N2, int64_t k, int version,
                              float *distance, int64_t *index, void *stream);
int tk3d_knn_distance_bcn_f64(const double *query, const double *key, int64_t B,
                              int64_t N1, int64_t N2, int64_t k, int version,
                              double *distance, int64_t *index, void *stream);

/* 3 nearest neighbours and their interpolation weights in one launch. Fuses what
 * FeatureInterpolator.forward does in Python (torkit3d/layers/pointnet2.py:125-130):
 * knn_points(query, key, 3), then 1/clamp(d2, min=eps), a sum and a division as
 * four torch kernels. distance and index are exactly tk3d_knn_distance_* with k = 3
 * (squared distances, MinK slot order); weight[b,i,s] = inv[s] / (inv[0]+inv[1]+inv[2])
 * with inv[s] = 1 / max(distance[b,i,s], eps), eps rounded to the data type.
 * channels_first = 0: query [B,N1,3], key [B,N2,3]; 1: query [B,3,N1], key [B,3,N2]
 * (the reference's models hold [B,3,N]). Outputs are [B,N1,3]. Requires N2 >= 3. */
int tk3d_three_nn_f32(const float *query, const float *key, int channels_first,
                      int64_t B, int64_t N1, int64_t N2, double eps, float *distance,
                      int64_t *index, float *weight, void *stream);
int tk3d_three_nn_f64(const double *query, const double *key, int channels_first,
                      int64_t B, int64_t N1, int64_t N2, double eps,
                      double *distance, int64_t *index, double *weight, void *stream);

/* ---- ball query --------------------------------------------------------------
 * Replaces ball_query_cuda
 * (torkit3d/csrc/include/ball_query.h:6-10, cuda/ball_query_kernel.cu:105-173).
 * index[b,i,:] = the first max_neighbors key indices j (ascending) with
 * d2(key[b,j], query[b,i]) < r*r, r = radius converted to the data type; slots
 * after the last hit repeat the first hit; a row with no hit is all -1. */
int tk3d_ball_query_f32(const float *query, const float *key, int64_t B,
                        int64_t N1, int64_t N2, float radius,
                        int64_t max_neighbors, int64_t *index, void *stream);
int tk3d_ball_query_f64(const double *query, const double *key, int64_t B,
                        int64_t N1, int64_t N2, float radius,
                        int64_t max_neighbors, int64_t *index, void *stream);

/* Ball query on [B,3,N] clouds (query [B,3,N1], key [B,3,N2]), the layout the
 * reference's models hold: ball_query(..., transpose=True) is the Python default and
 * copies both clouds to [B,N,3] before the call (torkit3d/ops/ball_query.py:17-38).
 * Same result as tk3d_ball_query_* on the transposed clouds, without the copies. */
int tk3d_ball_query_bcn_f32(const float *query, const float *key, int64_t B,
                            int64_t N1, int64_t N2, float radius,
                            int64_t max_neighbors, int64_t *index, void *stream);
int tk3d_ball_query_bcn_f64(const double *query, const double *key, int64_t B,
                            int64_t N1, int64_t N2, float radius,
                            int64_t max_neighbors, int64_t *index, void *stream);

/* ---- farthest point sampling ---------------------------------------------------
 * Replaces sample_farthest_points_cuda
 * (torkit3d/csrc/include/sample_farthest_points.h:6-8,
 *  cuda/sample_farthest_points_kernel.cu:106-165).
 * index[b,0] = 0; index[b,i] = the point farthest from {index[b,0..i-1]}.
 * Exact ties for the maximum are resolved as the reference kernel resolves them
 * (its per-thread scan and shared-memory tree, block size = the power of two
 * >= N capped at 512). Requires 1 <= num_samples <= N. A point with a NaN
 * coordinate is never selected and an infinite one, once selected, is selected at
 * every later step, as in the reference.
 *
 * Clouds too large for the register-resident kernel (more than 16384 points in fp32,
 * 8192 in fp64) need a device workspace of
 * tk3d_sample_farthest_points_workspace_bytes(B, N, elem_size) bytes, 8-byte aligned
 * (0 when none is needed; then `workspace` may be NULL), and are sampled with one
 * kernel launch per selection step, i.e. num_samples launches per call. */
size_t tk3d_sample_farthest_points_workspace_bytes(int64_t B, int64_t N,
                                                   size_t elem_size);
int tk3d_sample_farthest_points_f32(const float *points, int64_t B, int64_t N,
                                    int64_t num_samples, int64_t *index,
                                    void *workspace, size_t workspace_bytes,
                                    void *stream);
int tk3d_sample_farthest_points_f64(const double *points, int64_t B, int64_t N,
                                    int64_t num_samples, int64_t *index,
                                    void *workspace, size_t workspace_bytes,
                                    void *stream);

/* tk3d_sample_farthest_points_f32 for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops with a frozen memory pool, harnesses that
 * forbid hipMalloc): no counterpart in the reference. The workspace of the large-cloud
 * path is a fixed array of TK3D_FPS_STATIC_WORKSPACE_BYTES in the library's device image
 * (each GPU the library runs on holds its copy until the process ends). Same result as
 * tk3d_sample_farthest_points_f32. Returns TK3D_ERR_WORKSPACE when
 * tk3d_sample_farthest_points_workspace_bytes(B, N, 4) exceeds that size (8 MiB: e.g. one
 * cloud of 2 million points, or 64 clouds of 32000); clouds of up to 16384 points need
 * no workspace at any batch size. Calls no hipMalloc / hipFree. The first call on a GPU
 * looks the array's address up (hipGetSymbolAddress), and the first call on a GPU for each
 * kernel shape (points per lane: the size class of the cloud) asks the runtime once to
 * allow that kernel's LDS size (hipFuncSetAttribute): both are host calls that stream
 * capture does not record, so make one call per device and cloud-size class outside
 * capture. Return value as everywhere in this header: 0, a negative TK3D_ERR_*, or the
 * positive hipError_t of a runtime call that failed (then nothing further was launched).
 * All calls on one GPU share the array: calls that overlap in time on the same
 * GPU (different streams or threads) race and must be serialised by the caller. */
#define TK3D_FPS_STATIC_WORKSPACE_BYTES (8u << 20)
int tk3d_sample_farthest_points_static_f32(const float *points, int64_t B, int64_t N,
                                           int64_t num_samples, int64_t *index,
                                           void *stream);

/* Farthest point sampling on either point layout, optionally returning the sampled
 * coordinates as well. Fuses what the reference's models do around the op in
 * Python: sample_farthest_points(points, K, transpose=True) copies a [B,3,N] cloud
 * to [B,N,3] first (torkit3d/ops/sample_farthest_points.py:28-30) and
 * batch_index_select(points, index, dim=2) gathers the picks afterwards
 * (torkit3d/nn/functional.py:34-69, models/segmentation/pointnet2.py:89-90).
 * channels_first = 0: points [B,N,3], sampled [B,K,3];
 * channels_first = 1: points [B,3,N], sampled [B,3,K].
 * `sampled` may be NULL. `index` is identical to tk3d_sample_farthest_points_*. */
int tk3d_sample_farthest_points_gather_f32(const float *points, int channels_first,
                                           int64_t B, int64_t N,
                                           int64_t num_samples, int64_t *index,
                                           float *sampled, void *workspace,
                                           size_t workspace_bytes, void *stream);
int tk3d_sample_farthest_points_gather_f64(const double *points, int channels_first,
                                           int64_t B, int64_t N,
                                           int64_t num_samples, int64_t *index,
                                           double *sampled, void *workspace,
                                           size_t workspace_bytes, void *stream);

/* ---- group points (gather) -------------------------------------------------------
 * Replaces group_points_forward_cuda / group_points_backward_cuda
 * (torkit3d/csrc/include/group_points.h:6-13, cuda/group_points_kernel.cu:8-114).
 * forward:  output[b,c,m,s] = input[b,c,index[b,m,s]]          output [B,C,N2,K]
 * backward: grad_input[b,c,index[b,m,s]] += grad_output[b,c,m,s] grad_input [B,C,N1]
 * An index outside [0,N1) reads as 0 / contributes nothing (the reference
 * asserts on the device). */
int tk3d_group_points_forward_f32(const float *input, const int64_t *index,
                                  int64_t B, int64_t C, int64_t N1, int64_t N2,
                                  int64_t K, float *output, void *stream);
int tk3d_group_points_forward_f64(const double *input, const int64_t *index,
                                  int64_t B, int64_t C, int64_t N1, int64_t N2,
                                  int64_t K, double *output, void *stream);
int tk3d_group_points_backward_f32(const float *grad_output, const int64_t *index,
                                   int64_t B, int64_t C, int64_t N1, int64_t N2,
                                   int64_t K, float *grad_input, void *stream);
int tk3d_group_points_backward_f64(const double *grad_output,
                                   const int64_t *index, int64_t B, int64_t C,
                                   int64_t N1, int64_t N2, int64_t K,
                                   double *grad_input, void *stream);

/* Grouping for a PointNet++ set-abstraction layer in one output tensor. Fuses what
 * SetAbstraction.forward does in Python (torkit3d/layers/pointnet2.py:46-58):
 * group_points(feature), group_points(xyz), subtract the centre, torch.cat - the
 * concatenation alone re-reads and re-writes the grouped features.
 *   output[b, c,   m, s] = feature[b, c, index[b,m,s]]              c < C
 *   output[b, C+a, m, s] = xyz[b, a, index[b,m,s]] - centre[b,a,m]  a < 3
 * feature [B,C,N1] (may be NULL when C == 0), xyz [B,3,N1], centre [B,3,N2],
 * index [B,N2,K], output [B,C+3,N2,K].
 * backward: grad_feature[b,c,j] = sum of grad_output[b,c,m,s] over index[b,m,s] == j,
 * grad_xyz the same over channels C..C+2; either may be NULL (not wanted). The
 * gradient of `centre` is minus the sum of channels C..C+2 over s. */
int tk3d_group_points_concat_forward_f32(const float *feature, const float *xyz,
                                         const float *centre, const int64_t *index,
                                         int64_t B, int64_t C, int64_t N1, int64_t N2,
                                         int64_t K, float *output, void *stream);
int tk3d_group_points_concat_forward_f64(const double *feature, const double *xyz,
                                         const double *centre, const int64_t *index,
                                         int64_t B, int64_t C, int64_t N1, int64_t N2,
                                         int64_t K, double *output, void *stream);
int tk3d_group_points_concat_backward_f32(const float *grad_output, const int64_t *index,
                                          int64_t B, int64_t C, int64_t N1, int64_t N2,
                                          int64_t K, float *grad_feature,
                                          float *grad_xyz, void *stream);
int tk3d_group_points_concat_backward_f64(const double *grad_output, const int64_t *index,
                                          int64_t B, int64_t C, int64_t N1, int64_t N2,
                                          int64_t K, double *grad_feature,
                                          double *grad_xyz, void *stream);

/* ---- feature interpolation ----------------------------------------------------------
 * Replaces interpolate_forward_cuda / interpolate_backward_cuda
 * (torkit3d/csrc/include/interpolate.h:7-16, cuda/interpolate_kernel.cu:49-201).
 * forward:  output[b,c,n] = sum_{i<K} input[b,c,index[b,n,i]] * weight[b,n,i]
 * backward: grad_input[b,c,index[b,n,i]] += grad_output[b,c,n] * weight[b,n,i]
 * The reference accepts K == 3 only; this library takes 1 <= K <= 8. */
int tk3d_interpolate_forward_f32(const float *input, const int64_t *index,
                                 const float *weight, int64_t B, int64_t C,
                                 int64_t N1, int64_t N2, int64_t K, float *output,
                                 void *stream);
int tk3d_interpolate_forward_f64(const double *input, const int64_t *index,
                                 const double *weight, int64_t B, int64_t C,
                                 int64_t N1, int64_t N2, int64_t K, double *output,
                                 void *stream);
int tk3d_interpolate_backward_f32(const float *grad_output, const int64_t *index,
                                  const float *weight, int64_t B, int64_t C,
                                  int64_t N1, int64_t N2, int64_t K,
                                  float *grad_input, void *stream);
int tk3d_interpolate_backward_f64(const double *grad_output, const int64_t *index,
                                  const double *weight, int64_t B, int64_t C,
                                  int64_t N1, int64_t N2, int64_t K,
                                  double *grad_input, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TK3D_H */
