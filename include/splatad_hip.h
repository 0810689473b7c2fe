/*
 * C ABI of libsplatad_hip.so: the MI355X (gfx950) kernels behind the operator
 * interface of carlinds/splatad's rendering path.
 *
 * Conventions (they replace the pybind11/torch::Tensor boundary of the
 * reference, gsplat/cuda/csrc/ext.cpp:4-52 and bindings.h:123-468):
 *   - every pointer is a DEVICE pointer to contiguous row-major memory unless
 *     its name ends in _host; optional tensors are passed as NULL;
 *   - the caller allocates every output and every workspace (sizes from the
 *     *_workspace_bytes queries); the library never allocates or frees device
 *     memory;
 *   - all work is enqueued on `stream` (a hipStream_t); the only host
 *     waits are inside the *_count entry points, which copy one integer back
 *     to the host (the reference does the same through Tensor::item():
 *     rasterization.cu:154,465, projection.cu:1421);
 *   - return value 0 = success, negative = error; splatad_last_error() gives a
 *     thread-local message (the reference raises through TORCH_CHECK,
 *     bindings.h:9-13).
 * dtypes: float = IEEE binary32; radii are int32 for cameras and float for
 * lidars; isect ids int64; flatten ids / offsets / last ids int32; camera and
 * gaussian ids int64; masks are one byte per element.
 */
#ifndef SPLATAD_HIP_H
#define SPLATAD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *splatad_stream_t; /* hipStream_t */

const char *splatad_last_error(void);
int splatad_abi_version(void);

/* ---- projection ------------------------------------------------------- */

/* fully_fused_projection_fwd_tensor, projection.cu:966-1045 (kernel :605-751).
 * Exactly one of covars or (quats, scales) is non-NULL.  compensations may be
 * NULL.  Rows of culled Gaussians are written as zeros. */
int splatad_projection_fwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                           const float *quats, const float *scales, const float *velocities,
                           const float *viewmats, const float *Ks, uint32_t image_width,
                           uint32_t image_height, const float *linear_velocity,
                           const float *angular_velocity, const float *rolling_shutter_time,
                           float eps2d, float near_plane, float far_plane, float radius_clip,
                           int32_t *radii, float *means2d, float *depths, float *conics,
                           float *compensations, float *pix_vels, splatad_stream_t stream);

/* fully_fused_projection_packed_fwd_tensor, projection.cu:1355-1464, as a
 * two-call protocol: _count projects into the workspace and returns nnz on the
 * host, _fill compacts into [nnz,...] outputs ordered by (camera, gaussian). */
size_t splatad_projection_packed_workspace_bytes(uint32_t C, uint32_t N);
int splatad_projection_packed_count(uint32_t C, uint32_t N, const float *means,
                                    const float *covars, const float *quats, const float *scales,
                                    const float *velocities, const float *viewmats,
                                    const float *Ks, uint32_t image_width, uint32_t image_height,
                                    const float *linear_velocity, const float *angular_velocity,
                                    const float *rolling_shutter_time, float eps2d,
                                    float near_plane, float far_plane, float radius_clip,
                                    int calc_compensations, void *workspace, int64_t *nnz_host,
                                    splatad_stream_t stream);
/* The same counting call for a caller that goes on to intersect the packed rows with a
 * camera tile grid (rendering.py:278-309 of the reference: projection, then isect_tiles with the
 * same rows): it also counts the tiles the kept rows meet, rasterization.cu:44-62, and returns
 * both numbers with its one wait, so that splatad_isect_tiles_prepare can replace
 * splatad_isect_tiles_count and its wait. */
int splatad_projection_packed_count_tiles(uint32_t C, uint32_t N, const float *means,
                                          const float *covars, const float *quats, const float *scales,
                                          const float *velocities, const float *viewmats,
                                          const float *Ks, uint32_t image_width, uint32_t image_height,
                                          const float *linear_velocity, const float *angular_velocity,
                                          const float *rolling_shutter_time, float eps2d,
                                          float near_plane, float far_plane, float radius_clip,
                                          int calc_compensations, uint32_t tile_size,
                                          uint32_t tile_width, uint32_t tile_height, void *workspace,
                                          void *isect_workspace, int64_t *nnz_host,
                                          int64_t *n_isects_host, splatad_stream_t stream);
/* With isect_workspace (splatad_isect_workspace_bytes(C * N, C, tile_width * tile_height) bytes,
 * may be NULL) the counting call above also enqueues, before it waits, the first stages of the
 * tile intersection on the dense rows in its workspace, and this call completes it for the
 * packed rows: the lists it writes are those of splatad_isect_tiles_count / _fill on the packed
 * outputs of splatad_projection_packed_fill (tiles_per_gauss [nnz] included), without the wait.
 * Both workspaces must be untouched since the counting call; `lists` is
 * splatad_isect_lists_bytes(C * N, n_isects) bytes of scratch.
 * beside_stream (may be NULL): another stream of the caller's, which this call makes wait for
 * the point where the binning is done and the segment sort starts; work the caller enqueues there
 * afterwards (that needs the projection only: splatad_projection_packed_fill,
 * splatad_view_colors_fwd_packed) runs beside the sort, whose long workgroups leave part of the
 * GPU idle.  Nothing waits for that stream: the caller joins it.  (A cross-stream wait costs
 * the host about 10 us on this runtime, four kernel launches; here it rides on the fork the
 * sort makes anyway.)
 * beside_work (may be NULL): called once before this call returns, with beside_context and a
 * stream on which the caller may enqueue such work from inside the callback; it runs beside the
 * sort and has completed, as far as `stream` is concerned, when this call returns (the sort's own
 * fork and join carry it: no further cross-stream wait).  When there is nothing to sort the
 * stream handed over is `stream` itself.  A non-zero return value becomes this call's. */
typedef int (*splatad_beside_fn)(void *context, splatad_stream_t stream);
int splatad_isect_tiles_fill_packed(uint32_t C, uint32_t N, uint32_t tile_size, uint32_t tile_width,
                                    uint32_t tile_height, int64_t n_isects,
                                    const void *packed_workspace, void *isect_workspace, void *lists,
                                    int32_t *tiles_per_gauss, int64_t *isect_ids,
                                    int32_t *flatten_ids, int32_t *tile_offsets,
                                    splatad_stream_t beside_stream, splatad_beside_fn beside_work,
                                    void *beside_context, splatad_stream_t stream);
/* opacities [N] and row_opacities [nnz] (both or neither): the kept rows' opacity for the
 * compositing, opacities[gaussian] times the row's compensation when compensations are
 * computed (rendering.py:311-314 of the reference does this with a gather and a product). */
int splatad_projection_packed_fill(uint32_t C, uint32_t N, int64_t nnz, const void *workspace,
                                   int32_t *indptr, int64_t *camera_ids, int64_t *gaussian_ids,
                                   int32_t *radii, float *means2d, float *depths, float *conics,
                                   float *compensations, float *pix_vels, const float *opacities,
                                   float *row_opacities, splatad_stream_t stream);

/* fully_fused_lidar_projection_fwd_tensor, projection.cu:2631-2714 (kernel :2268-2417). */
int splatad_lidar_projection_fwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                                 const float *quats, const float *scales, const float *velocities,
                                 const float *viewmats, float min_elevation, float max_elevation,
                                 float min_azimuth, float max_azimuth,
                                 const float *linear_velocity, const float *angular_velocity,
                                 const float *rolling_shutter_time, float eps2d, float near_plane,
                                 float far_plane, float radius_clip, float *radii, float *means2d,
                                 float *depths, float *conics, float *compensations,
                                 float *pix_vels, float *depth_compensations,
                                 splatad_stream_t stream);

/* fully_fused_projection_bwd_tensor, projection.cu:1047-1155 (kernel :753-964).
 * v_covars xor (v_quats, v_scales); v_viewmats and v_velocities may be NULL.
 * Unpacked input (camera_ids == NULL): every row of v_means, v_covars, v_quats,
 * v_scales and v_velocities is stored, summed over the sensors in a fixed order
 * (no atomics: the same bits on every run); only v_viewmats is accumulated into and
 * must be zero-filled by the caller.  Packed input: all gradient outputs must be
 * zero-filled by the caller.  The same holds for splatad_lidar_projection_bwd, whose
 * input is always unpacked.  v_velocities is an extension: the reference computes and
 * drops it (projection.cu:874-877). */
int splatad_projection_bwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                           const float *quats, const float *scales, const float *velocities,
                           const float *viewmats, const float *Ks, uint32_t image_width,
                           uint32_t image_height, const float *linear_velocity,
                           const float *angular_velocity, const float *rolling_shutter_time,
                           float eps2d, const int64_t *camera_ids, const int64_t *gaussian_ids,
                           int64_t nnz, const int32_t *radii, const float *conics,
                           const float *compensations, const float *v_means2d,
                           const float *v_depths, const float *v_conics,
                           const float *v_compensations, const float *v_pix_vels, int sparse_grad,
                           float *v_means, float *v_covars, float *v_quats, float *v_scales,
                           float *v_viewmats, float *v_velocities, splatad_stream_t stream);

/* fully_fused_lidar_projection_bwd_tensor, projection.cu:2716-2826 (kernel :2419-2629). */
int splatad_lidar_projection_bwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                                 const float *quats, const float *scales, const float *velocities,
                                 const float *viewmats, const float *linear_velocity,
                                 const float *angular_velocity, const float *rolling_shutter_time,
                                 float eps2d, const float *radii, const float *conics,
                                 const float *compensations, const float *v_means2d,
                                 const float *v_depths, const float *v_conics,
                                 const float *v_compensations, const float *v_pix_vels,
                                 const float *v_depth_compensations, float *v_means,
                                 float *v_covars, float *v_quats, float *v_scales,
                                 float *v_viewmats, float *v_velocities, splatad_stream_t stream);

/* ---- spherical harmonics ------------------------------------------------ */

/* compute_sh_fwd_tensor / compute_sh_bwd_tensor, sh.cu:408-468.  n = number of
 * directions, K = number of bases in coeffs.  Masked-out rows are zero.
 * v_coeffs must be zero-filled; v_dirs may be NULL. */
int splatad_sh_fwd(uint32_t n, uint32_t K, uint32_t degree, const float *dirs,
                   const float *coeffs, const uint8_t *masks, float *colors,
                   splatad_stream_t stream);
int splatad_sh_bwd(uint32_t n, uint32_t K, uint32_t degree, const float *dirs,
                   const float *coeffs, const uint8_t *masks, const float *v_colors,
                   float *v_coeffs, float *v_dirs, splatad_stream_t stream);

/* View-dependent colours of the rendering pipeline in one launch: the block of
 * gsplat/rendering.py:325-351 (inverse of the view matrices, viewing directions, visibility
 * masks, spherical_harmonics(), max(c + 1/2, 0) and, optionally, the depth as fourth channel).
 * Row e is (sensor e / N, Gaussian e % N) for n == C * N, or (camera_ids[e], gaussian_ids[e])
 * for packed input; its direction is means[g] minus the sensor position -A^-1 t of
 * viewmats[c] = [A | t] (last row (0, 0, 0, 1), as the projection kernels assume); it is
 * active when radii[e][0] > 0 and inactive rows evaluate to max(1/2, 0).  coeffs is [N, K, 3]
 * (coeffs_per_sensor == 0) or [C, N, K, 3] (== 1).  colors has 3 channels, or 4 with depths.
 * _bwd takes the forward's colors (a channel passes its gradient only where it is positive)
 * and writes one row per e: v_coeffs [n, K, 3] (zero-filled by the caller) and, unless NULL,
 * v_dirs [n, 3]; the caller sums rows that share a Gaussian.  With scatter_coeffs != 0 the
 * kernel does that sum for the coefficients itself: v_coeffs then has the layout of coeffs
 * ([N, K, 3] or [C, N, K, 3]), cleared by the caller, and every row's gradients are added, with
 * atomics, at the coefficient row it read. */
int splatad_view_colors_fwd(uint32_t n, uint32_t C, uint32_t N, uint32_t K, uint32_t degree,
                            const float *means, const float *viewmats, const int64_t *camera_ids,
                            const int64_t *gaussian_ids, const int32_t *radii, const float *coeffs,
                            int coeffs_per_sensor, const float *depths, float *colors,
                            splatad_stream_t stream);
/* _fwd over dense [C, N] rows that stand in for their packed rows: an active row e writes its
 * colours to row remap[e] (+ remap_offsets[e / 256] where remap_offsets is not NULL: positions
 * kept as a place inside a group of 256 rows plus the group's place) of `colors` (its position
 * among the kept rows), inactive rows write nothing; depths, if given, is indexed by e as well.  Same values as _fwd on the packed rows
 * (one dependent load less per row).  _packed takes the rows, positions and depths from the
 * workspace of splatad_projection_packed_count[_tiles]: colors is [nnz, 3], or [nnz, 4]
 * with_depth. */
int splatad_view_colors_fwd_remapped(uint32_t C, uint32_t N, uint32_t K, uint32_t degree,
                                     const float *means, const float *viewmats, const int32_t *radii,
                                     const int32_t *remap, const int32_t *remap_offsets,
                                     const float *coeffs, int coeffs_per_sensor, const float *depths,
                                     float *colors, splatad_stream_t stream);
int splatad_view_colors_fwd_packed(uint32_t C, uint32_t N, uint32_t K, uint32_t degree,
                                   const float *means, const float *viewmats,
                                   const void *packed_workspace, const float *coeffs,
                                   int coeffs_per_sensor, int with_depth, float *colors,
                                   splatad_stream_t stream);
int splatad_view_colors_bwd(uint32_t n, uint32_t C, uint32_t N, uint32_t K, uint32_t degree,
                            const float *means, const float *viewmats, const int64_t *camera_ids,
                            const int64_t *gaussian_ids, const int32_t *radii, const float *coeffs,
                            int coeffs_per_sensor, uint32_t channels, const float *colors,
                            const float *v_colors, int scatter_coeffs, float *v_coeffs,
                            float *v_dirs, splatad_stream_t stream);

/* ---- tile intersection, sort, offsets ----------------------------------- */

/* isect_tiles_tensor (rasterization.cu:92-216) and isect_lidar_tiles_tensor
 * (:397-529) as a two-call protocol.  total = C*N (camera_ids NULL) or nnz
 * (packed, camera_ids given).  _count writes tiles_per_gauss and returns
 * n_isects on the host; _fill writes isect_ids/flatten_ids, sorted by
 * (camera, tile, depth bits) with ties in emission order when sort != 0, in
 * emission order otherwise.  Depths must be non-negative (sign bit clear).
 * For lidars tile_width/tile_height are the azimuth/elevation tile counts and
 * elev_boundaries has tile_height+1 entries.
 *
 * Memory: `workspace` is splatad_isect_workspace_bytes(total, C, n_tiles) bytes
 * and is shared by the two calls: with sort != 0, _count also enqueues the first
 * stages of the binning (they do not depend on n_isects) behind the counting
 * kernel, so that the GPU has work while the host sizes the outputs, and _fill
 * continues from what they left there (_count reads depths for that: where a tile
 * meets very many Gaussians the binning also cuts the depth axis into slabs, at
 * quantiles of a sample of the depths; depths may be NULL when sort == 0).  Pass
 * both calls the same sort flag, inputs and stream, and leave the workspace
 * untouched in between.  `lists` is
 * splatad_isect_lists_bytes(total, n_isects) bytes of scratch for _fill alone.
 * _count waits for the counting kernel only (the kernel writes n_isects into a
 * pinned host word leased from a small per-device pool that is kept for the life of the
 * process, and the host spins on it), not for the work enqueued behind it.
 *
 * tile_offsets may be NULL; with sort != 0 it receives the [C, tile_height,
 * tile_width] table that splatad_isect_offset_encode would derive from isect_ids
 * (the binning knows every tile's first intersection before the sort runs). */
size_t splatad_isect_workspace_bytes(uint64_t total, uint32_t C, uint32_t n_tiles);
size_t splatad_isect_lists_bytes(uint64_t total, int64_t n_isects);
int splatad_isect_tiles_count(uint64_t total, uint32_t N, const int64_t *camera_ids,
                              const float *means2d, const int32_t *radii, const float *depths,
                              uint32_t C, uint32_t tile_size, uint32_t tile_width, uint32_t tile_height,
                              int sort, int32_t *tiles_per_gauss, void *workspace,
                              int64_t *n_isects_host, splatad_stream_t stream);
/* splatad_isect_tiles_count for a caller that knows n_isects already (from
 * splatad_projection_packed_count_tiles on the same rows and tile grid): enqueues the same work,
 * returns no number and waits for nothing.  _fill follows with that n_isects, which must be
 * the number _count would have returned.  tiles_per_gauss may be NULL when sort != 0: the rows'
 * tile counts are then not made (the sorted lists do not need them). */
int splatad_isect_tiles_prepare(uint64_t total, uint32_t N, const int64_t *camera_ids,
                                const float *means2d, const int32_t *radii, const float *depths,
                                uint32_t C, uint32_t tile_size, uint32_t tile_width,
                                uint32_t tile_height, int sort, int32_t *tiles_per_gauss,
                                void *workspace, splatad_stream_t stream);
/* _fill for dense [C, N] rows that stand in for their packed rows: `remap` [C * N] holds each
 * kept row's position among the kept rows (what flatten_ids must name); tiles_out, if not NULL,
 * receives the kept rows' tile counts at those positions.  remap_offsets (may be NULL): as for
 * splatad_view_colors_fwd_remapped, row e's position is remap[e] + remap_offsets[e / 256].
 * beside_stream, beside_work: see splatad_isect_tiles_fill_packed. */
int splatad_isect_tiles_fill_remapped(uint64_t total, uint32_t N, const float *means2d,
                                      const int32_t *radii, const float *depths, uint32_t C,
                                      uint32_t tile_size, uint32_t tile_width, uint32_t tile_height,
                                      int64_t n_isects, const int32_t *tiles_per_gauss,
                                      const int32_t *remap, const int32_t *remap_offsets,
                                      void *workspace, void *lists, int32_t *tiles_out, int64_t *isect_ids, int32_t *flatten_ids,
                                      int32_t *tile_offsets, splatad_stream_t beside_stream,
                                      splatad_beside_fn beside_work, void *beside_context,
                                      splatad_stream_t stream);
int splatad_isect_tiles_fill(uint64_t total, uint32_t N, const int64_t *camera_ids,
                             const float *means2d, const int32_t *radii, const float *depths,
                             uint32_t C, uint32_t tile_size, uint32_t tile_width,
                             uint32_t tile_height, int sort, int64_t n_isects,
                             const int32_t *tiles_per_gauss, void *workspace, void *lists,
                             int64_t *isect_ids, int32_t *flatten_ids, int32_t *tile_offsets,
                             splatad_stream_t stream);
/* splatad_isect_tiles_fill with work of the caller's beside the sort: beside_work (may be NULL)
 * is called once before the call returns, with beside_context and a stream; what the callback
 * enqueues there must need nothing that is enqueued on `stream` after this call began (the
 * projection's outputs are fine: the colour cache of splatad_view_colors_cache, say), runs
 * beside the sort, and has completed as far as `stream` is concerned when the call returns.  No
 * counterpart in the reference; see splatad_isect_tiles_fill_packed for the mechanism. */
int splatad_isect_tiles_fill_beside(uint64_t total, uint32_t N, const int64_t *camera_ids,
                                    const float *means2d, const int32_t *radii, const float *depths,
                                    uint32_t C, uint32_t tile_size, uint32_t tile_width,
                                    uint32_t tile_height, int sort, int64_t n_isects,
                                    const int32_t *tiles_per_gauss, void *workspace, void *lists,
                                    int64_t *isect_ids, int32_t *flatten_ids, int32_t *tile_offsets,
                                    splatad_beside_fn beside_work, void *beside_context,
                                    splatad_stream_t stream);
int splatad_isect_lidar_tiles_count(uint64_t total, uint32_t N, const int64_t *camera_ids,
                                    const float *means2d, const float *radii, const float *depths,
                                    uint32_t C, const float *elev_boundaries, float tile_azim_resolution,
                                    float min_azim, uint32_t tile_width, uint32_t tile_height,
                                    int sort, int32_t *tiles_per_gauss, void *workspace,
                                    int64_t *n_isects_host, splatad_stream_t stream);
int splatad_isect_lidar_tiles_fill(uint64_t total, uint32_t N, const int64_t *camera_ids,
                                   const float *means2d, const float *radii, const float *depths,
                                   uint32_t C, const float *elev_boundaries,
                                   float tile_azim_resolution, float min_azim,
                                   uint32_t tile_width, uint32_t tile_height, int sort,
                                   int64_t n_isects, const int32_t *tiles_per_gauss,
                                   void *workspace, void *lists, int64_t *isect_ids,
                                   int32_t *flatten_ids, int32_t *tile_offsets,
                                   splatad_stream_t stream);

/* isect_offset_encode_tensor, rasterization.cu:264-285 (kernel :218-262). */
int splatad_isect_offset_encode(int64_t n_isects, const int64_t *isect_ids, uint32_t C,
                                uint32_t n_tiles, int32_t *offsets, splatad_stream_t stream);

/* ---- lidar point binning -------------------------------------------- */

/* map_points_to_lidar_tiles_tensor, rasterization.cu:658-770 (kernel :596-656; op declared
 * in bindings.h next to isect_lidar_tiles).  One key (camera << 32 | tile) and one id per
 * point; points2d is [C, N, 2] (camera_ids NULL, N given) or packed [total, 2] with
 * camera_ids [total].  With sort != 0 the keys ascend and equal keys keep the point order;
 * that mode needs a workspace of splatad_map_points_to_lidar_tiles_workspace_bytes(total,
 * C, n_tiles_azim * n_tiles_elev) bytes and at most 36864 (sensor, tile) pairs. */
size_t splatad_map_points_to_lidar_tiles_workspace_bytes(uint64_t total, uint32_t C,
                                                         uint32_t n_tiles);
int splatad_map_points_to_lidar_tiles(uint64_t total, uint32_t N, const int64_t *camera_ids,
                                      const float *points2d, uint32_t C,
                                      const float *elev_boundaries, float tile_azim_resolution,
                                      float min_azim, uint32_t n_tiles_azim,
                                      uint32_t n_tiles_elev, int sort, void *workspace,
                                      int64_t *tile_ids, int32_t *flatten_ids,
                                      splatad_stream_t stream);

/* splatad_map_points_to_lidar_tiles for callers that cannot allocate (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments without the workspace: the counter table of the sorted mode lives in
 * a static device array of the library (about 2 MiB per GPU, held until the process ends), and
 * the call allocates nothing, on the device or on the host.  Limits, beyond which it returns an
 * error and launches nothing: total <= splatad_map_points_to_lidar_tiles_noalloc_max_points()
 * (4 194 304 points) and C * n_tiles_azim * n_tiles_elev <=
 * splatad_map_points_to_lidar_tiles_noalloc_max_tiles() (16 384).  Results are identical to
 * splatad_map_points_to_lidar_tiles.  All calls on one GPU share that GPU's array: calls that
 * overlap on one GPU (different streams, different threads) race; calls in stream order do not,
 * and nothing has to be cleared between them.  The first sorted call on a device also does the
 * library's one-time setup for that device (kernel attributes, the address of the static
 * array): make one call outside any capture before capturing calls into a HIP graph; after
 * that a call enqueues kernels only. */
uint64_t splatad_map_points_to_lidar_tiles_noalloc_max_points(void);
uint32_t splatad_map_points_to_lidar_tiles_noalloc_max_tiles(void);
int splatad_map_points_to_lidar_tiles_noalloc(uint64_t total, uint32_t N,
                                              const int64_t *camera_ids, const float *points2d,
                                              uint32_t C, const float *elev_boundaries,
                                              float tile_azim_resolution, float min_azim,
                                              uint32_t n_tiles_azim, uint32_t n_tiles_elev,
                                              int sort, int64_t *tile_ids, int32_t *flatten_ids,
                                              splatad_stream_t stream);

/* points_mapping_offset_encode_tensor, rasterization.cu:576-594 (kernel :531-574). */
int splatad_points_mapping_offset_encode(int64_t n_points, const int64_t *point_ids, uint32_t C,
                                         uint32_t n_tiles, int32_t *offsets,
                                         splatad_stream_t stream);

/* populate_image_from_points_tensor, rasterization.cu:807-833 (kernel :772-805).  points is
 * [.., 5]; image [C, image_height, image_width, 5] is written completely (zeros where no
 * point lands). */
int splatad_populate_image_from_points(uint32_t C, int64_t n_points, const float *points,
                                       uint32_t image_width, uint32_t image_height,
                                       uint32_t tile_width, uint32_t tile_height,
                                       uint32_t grid_w, uint32_t grid_h,
                                       const int32_t *tile_offsets, const int32_t *flatten_ids,
                                       float *image, splatad_stream_t stream);

/* ---- rasterization ------------------------------------------------------ */

/* rasterize_to_pixels_fwd_tensor, rasterization.cu:1520-2018 (kernel
 * :1360-1518).  Any channel count >= 1 is accepted (wide inputs are rendered in
 * passes).  backgrounds may be NULL.  tile_batches may be NULL; otherwise it receives,
 * per (camera, tile), the number of entries of the tile's list that were staged (whole
 * batches, until every pixel of the tile had saturated, clipped to the list's length; a
 * diagnostic: it tells how much of the sorted lists a frame really reads).  tile_cycles may be
 * NULL; otherwise it receives, per (camera, tile), the shader clock cycles the tile's workgroup
 * ran for (a diagnostic: the spread tells how far the slowest tiles set the kernel's duration;
 * with channels in several passes, the last pass's). */
int splatad_rasterize_to_pixels_fwd(uint32_t C, int64_t n_isects, uint32_t channels,
                                    const float *means2d, const float *conics,
                                    const float *colors, const float *opacities,
                                    const float *pix_vels, const float *rolling_shutter_time,
                                    const float *backgrounds, uint32_t image_width,
                                    uint32_t image_height, uint32_t tile_size,
                                    uint32_t tile_width, uint32_t tile_height,
                                    const int32_t *tile_offsets, const int32_t *flatten_ids,
                                    float *render_colors, float *render_alphas,
                                    int32_t *last_ids, int32_t *tile_batches,
                                    int64_t *tile_cycles, splatad_stream_t stream);

/* Prepares the colour cache of splatad_rasterize_to_pixels_fwd_sh (no counterpart in the
 * reference): `cache`, splatad_view_colors_cache_bytes(n) bytes, gets a NaN in every float of
 * its n rows, and -- only where the lists will be consumed deeply -- the colours of all visible
 * rows, as splatad_view_colors_fwd makes them, because then nearly every row is needed and a
 * row per lane beforehand is cheaper than rows evaluated as the tiles reach them.  The test:
 * sum over the visible rows of opacities[Gaussian] x tiles met (estimated from radii and
 * tile_size), divided by the C x tile_width x tile_height tiles; below min_opacity_per_tile the
 * colours are made here (0 = never, infinity = always), with the row's depth (depths may be
 * NULL: zero) as fourth float, which the compositing kernel renders as its fourth channel.
 * opacities is [N], one per Gaussian; the other arguments as for splatad_view_colors_fwd. */
size_t splatad_view_colors_cache_bytes(uint64_t n_rows);
int splatad_view_colors_cache(uint32_t n, uint32_t C, uint32_t N, uint32_t K, uint32_t degree,
                              const float *means, const float *viewmats, const int64_t *camera_ids,
                              const int64_t *gaussian_ids, const int32_t *radii, const float *coeffs,
                              int coeffs_per_sensor, const float *depths, const float *opacities,
                              uint32_t tile_size, uint32_t tile_width, uint32_t tile_height,
                              float min_opacity_per_tile, float *cache, splatad_stream_t stream);

/* Steps 3 and 5 of rasterization() in one kernel (gsplat/rendering.py:325-347 and 362-391 of
 * the reference: view directions, spherical harmonics, max(c + 1/2, 0), then
 * rasterize_to_pixels): the compositing kernel evaluates the colour of every list entry it
 * stages from `coeffs` ([N, K, 3], or [C, N, K, 3] with coeffs_per_sensor != 0), `means` [N, 3]
 * and the sensor positions in `viewmats` [C, 4, 4], with the instructions of
 * splatad_view_colors_fwd, so the images equal those of the two calls bit for bit.  It reads
 * the coefficients of the entries that tiles reach before they saturate instead of those of
 * every visible Gaussian, beside arithmetic that leaves the memory idle.  Rows (what
 * flatten_ids index: means2d, conics, opacities, pix_vels, depths) are dense [C, N] with
 * gaussian_ids == NULL, or packed [nnz] with gaussian_ids [nnz] naming each row's Gaussian (the
 * camera of a row is that of the tile that lists it).  Renders 3 channels, or 4 with `depths`
 * (not NULL) as the last one.  color_cache: 16 bytes per row, as splatad_view_colors_cache
 * leaves them (every float a NaN, or the row's colour and depth; the workgroups that first
 * stage a row without a colour leave it there for the tiles that list the Gaussian later); what
 * it holds afterwards is of no use to the caller.  Forward only; last_ids may be NULL (nobody
 * will run a backward pass from this call), which spares the kernel their bookkeeping. */
int splatad_rasterize_to_pixels_fwd_sh(uint32_t C, uint32_t N, int64_t n_isects, uint32_t K,
                                       uint32_t degree, const float *means, const float *viewmats,
                                       const float *coeffs, int coeffs_per_sensor,
                                       const int64_t *gaussian_ids, const float *depths,
                                       float *color_cache, const float *means2d,
                                       const float *conics, const float *opacities,
                                       const float *pix_vels, const float *rolling_shutter_time,
                                       const float *backgrounds, uint32_t image_width,
                                       uint32_t image_height, uint32_t tile_size,
                                       uint32_t tile_width, uint32_t tile_height,
                                       const int32_t *tile_offsets, const int32_t *flatten_ids,
                                       float *render_colors, float *render_alphas,
                                       int32_t *last_ids, splatad_stream_t stream);

/* Diagnostic without a counterpart in the reference: lane utilisation of the compositing loop
 * of splatad_rasterize_to_pixels_fwd on the same inputs (nothing is rendered).  Adds to eight
 * counters in stats (zero them first): [0] (wavefront, Gaussian) iterations of the inner loop,
 * [1] pixels that composited their Gaussian, summed over the iterations, [2] pixels still
 * alive, [3] iterations in which no pixel composited, [4] list entries tested against a
 * wavefront's footprint, [5] entries that passed the test, [6] (stored, not added) pixels per
 * lane of the kernel that ran, so that an iteration offers 64 * [6] pixels, [7] pixels with
 * alpha >= 1/255. */
int splatad_rasterize_to_pixels_lane_stats(uint32_t C, int64_t n_isects, const float *means2d,
                                           const float *conics, const float *opacities,
                                           const float *pix_vels,
                                           const float *rolling_shutter_time,
                                           uint32_t image_width, uint32_t image_height,
                                           uint32_t tile_size, uint32_t tile_width,
                                           uint32_t tile_height, const int32_t *tile_offsets,
                                           const int32_t *flatten_ids, unsigned long long *stats,
                                           splatad_stream_t stream);

/* rasterize_to_pixels_bwd_tensor, rasterization.cu:3091-3726 (kernel
 * :2833-3089).  Gradient outputs must be zero-filled; v_means2d_abs may be NULL.
 *
 * workspace (both backward entry points): optional scratch of
 * splatad_rasterize_bwd_workspace_bytes(total, channels, lidar) bytes, 16-byte
 * aligned, contents irrelevant; total = number of projected Gaussians (C * N, or
 * nnz for packed input), i.e. the rows of means2d.  With it the kernels add up the
 * gradients of a Gaussian in one 64-byte-aligned record of the workspace, where the
 * atomics of one Gaussian share a memory request, and a second kernel adds the
 * records into the v_* arrays: about twice as fast as accumulating into the arrays
 * directly, which is what happens with workspace == NULL. */
size_t splatad_rasterize_bwd_workspace_bytes(uint64_t total, uint32_t channels, int lidar);
int splatad_rasterize_to_pixels_bwd(uint32_t C, int64_t n_isects, uint32_t channels,
                                    const float *means2d, const float *conics,
                                    const float *colors, const float *opacities,
                                    const float *pix_vels, const float *rolling_shutter_time,
                                    const float *backgrounds, uint32_t image_width,
                                    uint32_t image_height, uint32_t tile_size,
                                    uint32_t tile_width, uint32_t tile_height,
                                    const int32_t *tile_offsets, const int32_t *flatten_ids,
                                    const float *render_alphas, const int32_t *last_ids,
                                    const float *v_render_colors, const float *v_render_alphas,
                                    float *v_means2d_abs, float *v_means2d, float *v_conics,
                                    float *v_colors, float *v_opacities, float *v_pix_vels,
                                    uint64_t total, void *workspace, size_t workspace_bytes,
                                    splatad_stream_t stream);

/* The backward pass of splatad_rasterize_to_pixels_fwd_sh (which has no counterpart in the
 * reference): splatad_rasterize_to_pixels_bwd with `colors` = the colour cache that call left
 * behind ([rows, 4], of which `channels` = 4 are composited; for 3 channels hand over a
 * contiguous [rows, 3] copy).  Rows that no tile staged hold NaN there; no pixel composited
 * them, their gradient is zero, and the kernel takes their colour as zero.  v_colors then goes
 * to splatad_view_colors_bwd.  v_depths (may be NULL; with channels = 4 only): [rows] floats,
 * cleared by the caller, that receive the gradient of the fourth channel, the depth, instead
 * of v_colors[.., 3] -- the contiguous array the projection's backward call takes. */
int splatad_rasterize_to_pixels_bwd_sh(uint32_t C, int64_t n_isects, uint32_t channels,
                                    const float *means2d, const float *conics,
                                    const float *colors, const float *opacities,
                                    const float *pix_vels, const float *rolling_shutter_time,
                                    const float *backgrounds, uint32_t image_width,
                                    uint32_t image_height, uint32_t tile_size,
                                    uint32_t tile_width, uint32_t tile_height,
                                    const int32_t *tile_offsets, const int32_t *flatten_ids,
                                    const float *render_alphas, const int32_t *last_ids,
                                    const float *v_render_colors, const float *v_render_alphas,
                                    float *v_means2d_abs, float *v_means2d, float *v_conics,
                                    float *v_colors, float *v_depths, float *v_opacities,
                                    float *v_pix_vels, uint64_t total, void *workspace,
                                    size_t workspace_bytes, splatad_stream_t stream);

/* rasterize_to_points_fwd_tensor, rasterization.cu:2221-2831 (kernel
 * :2021-2219).  Outputs of inactive points (range <= 0) are zero.
 * alpha_sum_until_points may be NULL when compute_alpha_sum_until_points == 0.
 * tile_batches, tile_cycles: optional diagnostics as in splatad_rasterize_to_pixels_fwd.
 *
 * range_channel (both directions; NULL for the reference's layout): the reference's
 * callers concatenate the Gaussians' ranges behind their features first
 * (gsplat/rendering.py:746 and :779, torch.cat of lidar_features and depths), a copy of the
 * whole feature tensor per frame.  With range_channel given, `colors` keeps its
 * channels - 1 feature values per Gaussian and the last channel (depth_channel_idx
 * must be channels - 1, channels >= 2) is read from range_channel[total]; all
 * [.., channels] image-side arrays are as before.  In the backward call v_colors
 * then has channels - 1 values per Gaussian too and the last channel's gradient
 * goes to v_range[total] (zero-filled like the others; NULL exactly when
 * range_channel is). */
int splatad_rasterize_to_points_fwd(uint32_t C, int64_t n_isects, uint32_t channels,
                                    const float *means2d, const float *conics,
                                    const float *colors, const float *range_channel,
                                    const float *opacities, const float *pix_vels,
                                    const float *depth_compensations,
                                    const float *backgrounds, const float *raster_pts,
                                    uint32_t image_width, uint32_t image_height,
                                    uint32_t tile_width, uint32_t tile_height,
                                    uint32_t tile_grid_width, uint32_t tile_grid_height,
                                    int compute_alpha_sum_until_points, float threshold,
                                    const int32_t *tile_offsets, const int32_t *flatten_ids,
                                    uint32_t depth_channel_idx, float *render_colors,
                                    float *render_alphas, float *alpha_sum_until_points,
                                    int32_t *last_ids, float *median_depths,
                                    int32_t *tile_batches, int64_t *tile_cycles,
                                    splatad_stream_t stream);

/* rasterize_to_points_bwd_tensor, rasterization.cu:4056-4851 (kernel :3728-4054). */
int splatad_rasterize_to_points_bwd(uint32_t C, int64_t n_isects, uint32_t channels,
                                    const float *means2d, const float *conics,
                                    const float *colors, const float *range_channel,
                                    const float *opacities, const float *pix_vels,
                                    const float *depth_compensations,
                                    const float *backgrounds, const float *raster_pts,
                                    uint32_t image_width, uint32_t image_height,
                                    uint32_t tile_width, uint32_t tile_height,
                                    uint32_t tile_grid_width, uint32_t tile_grid_height,
                                    int compute_alpha_sum_until_points, float threshold,
                                    const int32_t *tile_offsets, const int32_t *flatten_ids,
                                    uint32_t depth_channel_idx, const float *render_alphas,
                                    const int32_t *last_ids, const float *v_render_colors,
                                    const float *v_render_alphas,
                                    const float *v_alpha_sum_until_points, float *v_means2d_abs,
                                    float *v_means2d, float *v_conics, float *v_colors,
                                    float *v_range, float *v_opacities, float *v_pix_vels,
                                    float *v_depth_compensations, uint64_t total, void *workspace,
                                    size_t workspace_bytes, splatad_stream_t stream);

/* ---- unfused projection operators ------------------------------------ */
/* Every operator streams [C, N, ...] (or [N, ...]) rows; gradients of a forward input are
 * written completely unless stated otherwise. */

/* quat_scale_to_covar_preci_{fwd,bwd}_tensor, projection.cu:161-228 (kernels :18-159).
 * covars / precis are [N, 3, 3], or [N, 6] upper triangles with triu != 0; either may be
 * NULL (not computed / no gradient given). */
int splatad_quat_scale_to_covar_preci_fwd(uint32_t N, const float *quats, const float *scales,
                                          int triu, float *covars, float *precis,
                                          splatad_stream_t stream);
int splatad_quat_scale_to_covar_preci_bwd(uint32_t N, const float *quats, const float *scales,
                                          const float *v_covars, const float *v_precis, int triu,
                                          float *v_quats, float *v_scales, splatad_stream_t stream);

/* world_to_cam_{fwd,bwd}_tensor, projection.cu:386-599.  The backward outputs v_means [N, 3],
 * v_covars [N, 3, 3], v_viewmats [C, 4, 4] are accumulated into (zero-fill them) and may each
 * be NULL. */
int splatad_world_to_cam_fwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                             const float *viewmats, float *means_c, float *covars_c,
                             splatad_stream_t stream);
int splatad_world_to_cam_bwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                             const float *viewmats, const float *v_means_c,
                             const float *v_covars_c, float *v_means, float *v_covars,
                             float *v_viewmats, splatad_stream_t stream);

/* persp_proj_{fwd,bwd}_tensor, projection.cu:230-384: means [C, N, 3], covars [C, N, 3, 3] ->
 * means2d [C, N, 2], covars2d [C, N, 2, 2]. */
int splatad_persp_proj_fwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                           const float *Ks, uint32_t width, uint32_t height, float *means2d,
                           float *covars2d, splatad_stream_t stream);
int splatad_persp_proj_bwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                           const float *Ks, uint32_t width, uint32_t height,
                           const float *v_means2d, const float *v_covars2d, float *v_means,
                           float *v_covars, splatad_stream_t stream);

/* compute_pix_velocity_{fwd,bwd}_tensor, projection.cu:2118-2266: p_view and velocities are
 * [C, N, 3] in the sensor frame; vel is [C, N, 2]. */
int splatad_compute_pix_velocity_fwd(uint32_t C, uint32_t N, const float *p_view,
                                     const float *lin_vel, const float *ang_vel,
                                     const float *velocities, const float *Ks, uint32_t width,
                                     uint32_t height, float *vel, splatad_stream_t stream);
int splatad_compute_pix_velocity_bwd(uint32_t C, uint32_t N, const float *p_view,
                                     const float *lin_vel, const float *ang_vel,
                                     const float *velocities, const float *Ks, uint32_t width,
                                     uint32_t height, const float *v_vel, float *v_p_view,
                                     float *v_velocities, splatad_stream_t stream);

/* lidar_proj_{fwd,bwd}_tensor, projection.cu:1841-1988: means2d (azimuth, elevation in degrees)
 * [C, N, 2], covars2d [C, N, 2, 2], depth_compensations [C, N, 2]. */
int splatad_lidar_proj_fwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                           float eps2d, float *means2d, float *covars2d,
                           float *depth_compensations, splatad_stream_t stream);
int splatad_lidar_proj_bwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                           float eps2d, const float *v_means2d, const float *v_covars2d,
                           const float *v_depth_compensations, float *v_means, float *v_covars,
                           splatad_stream_t stream);

/* compute_lidar_velocity_{fwd,bwd}_tensor, projection.cu:1990-2116: vel is [C, N, 3]
 * (azimuth rate, elevation rate in degrees, range rate). */
int splatad_compute_lidar_velocity_fwd(uint32_t C, uint32_t N, const float *p_view,
                                       const float *lin_vel, const float *ang_vel,
                                       const float *velocities, float *vel,
                                       splatad_stream_t stream);
int splatad_compute_lidar_velocity_bwd(uint32_t C, uint32_t N, const float *p_view,
                                       const float *lin_vel, const float *ang_vel,
                                       const float *velocities, const float *v_vel,
                                       float *v_p_view, float *v_velocities,
                                       splatad_stream_t stream);

/* ---- (Gaussian, pixel) index lists -------------------------------------- */

/* rasterize_to_indices_in_range_tensor, rasterization.cu:1003-1092 (kernel :839-1001)
 * and rasterize_to_indices_in_range_lidar_tensor, :1270-1358 (kernel :1100-1268).
 *
 * The reference runs its kernel twice inside one op, with a host read of the number of
 * pairs in between to size the outputs.  Here the two passes are two entry points so that
 * the caller owns every allocation:
 *   *_count  counts the pairs of every pixel for batches [range_start, range_end) of each
 *            tile's list (a batch is as many Gaussians as a tile has pixels), writes the
 *            exclusive prefix sums to chunk_starts [C * H * W] (int64, row-major pixels,
 *            sensor by sensor) and the number of pairs to *n_elems (device memory);
 *   *_fill   writes gaussian_ids [n_elems] (index in [0, N)) and indices [n_elems]
 *            (pixel + sensor * H * W), front to back within a pixel, with the same arguments
 *            and the chunk_starts of the counting call.
 * transmittances [C, H, W] is the transmittance reached before range_start.  range_end
 * beyond the longest list is allowed (values above 2^32 - 1 are clamped).  workspace is
 * splatad_rasterize_to_indices_workspace_bytes(C, W, H) of scratch. */
size_t splatad_rasterize_to_indices_workspace_bytes(uint32_t C, uint32_t image_width,
                                                    uint32_t image_height);
int splatad_rasterize_to_indices_in_range_count(
    int64_t range_start, int64_t range_end, uint32_t C, uint32_t N, int64_t n_isects,
    const float *transmittances, const float *means2d, const float *conics,
    const float *opacities, const float *pix_vels, const float *rolling_shutter_time,
    uint32_t image_width, uint32_t image_height, uint32_t tile_size, uint32_t tile_width,
    uint32_t tile_height, const int32_t *tile_offsets, const int32_t *flatten_ids,
    void *workspace, size_t workspace_bytes, int64_t *chunk_starts, int64_t *n_elems,
    splatad_stream_t stream);
int splatad_rasterize_to_indices_in_range_fill(
    int64_t range_start, int64_t range_end, uint32_t C, uint32_t N, int64_t n_isects,
    const float *transmittances, const float *means2d, const float *conics,
    const float *opacities, const float *pix_vels, const float *rolling_shutter_time,
    uint32_t image_width, uint32_t image_height, uint32_t tile_size, uint32_t tile_width,
    uint32_t tile_height, const int32_t *tile_offsets, const int32_t *flatten_ids,
    const int64_t *chunk_starts, int64_t *gaussian_ids, int64_t *indices,
    splatad_stream_t stream);
/* Lidar: pix_vels is [C, N, 3], raster_pts [C, H, W, 4] = azimuth, elevation (degrees),
 * range, time; tile_width x tile_height points per tile (at most 256), grid of
 * tile_grid_width x tile_grid_height tiles. */
int splatad_rasterize_to_indices_in_range_lidar_count(
    int64_t range_start, int64_t range_end, uint32_t C, uint32_t N, int64_t n_isects,
    const float *transmittances, const float *means2d, const float *conics,
    const float *opacities, const float *pix_vels, const float *raster_pts,
    uint32_t image_width, uint32_t image_height, uint32_t tile_width, uint32_t tile_height,
    uint32_t tile_grid_width, uint32_t tile_grid_height, const int32_t *tile_offsets,
    const int32_t *flatten_ids, void *workspace, size_t workspace_bytes,
    int64_t *chunk_starts, int64_t *n_elems, splatad_stream_t stream);
int splatad_rasterize_to_indices_in_range_lidar_fill(
    int64_t range_start, int64_t range_end, uint32_t C, uint32_t N, int64_t n_isects,
    const float *transmittances, const float *means2d, const float *conics,
    const float *opacities, const float *pix_vels, const float *raster_pts,
    uint32_t image_width, uint32_t image_height, uint32_t tile_width, uint32_t tile_height,
    uint32_t tile_grid_width, uint32_t tile_grid_height, const int32_t *tile_offsets,
    const int32_t *flatten_ids, const int64_t *chunk_starts, int64_t *gaussian_ids,
    int64_t *indices, splatad_stream_t stream);

/* ---- densification helper --------------------------------------------- */

/* compute_relocation_tensor, gsplat/cuda/csrc/relocation.cu:32-56 (kernel :4-30; op
 * declared in bindings.h).  ratios are int32 in [1, n_max]; binoms is [n_max, n_max]. */
int splatad_compute_relocation(uint32_t N, const float *opacities, const float *scales,
                               const int32_t *ratios, const float *binoms, int32_t n_max,
                               float *new_opacities, float *new_scales, splatad_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SPLATAD_HIP_H */
