/* C ABI of libgsrast.so: the gfx950 Gaussian rasterizer behind CityGS-X's
 * diff_gaussian_rasterization / simple_knn operator API.
 *
 * Conventions
 *   - Every pointer is a device pointer unless its comment says "host".
 *   - The library never allocates or frees device memory.  Outputs are caller
 *     allocated; scratch comes either from a resize callback (render forward,
 *     like the reference's std::function<char*(size_t)> buffers) or from a
 *     workspace whose size a *_workspace_bytes() query returns.
 *   - stream is a hipStream_t (NULL = the default stream).  Calls are
 *     asynchronous except where stated.
 *   - Return value 0 = success; otherwise gs_last_error() (thread local)
 *     describes the failure.
 *   - debug != 0 synchronises the stream after every launch and reports the
 *     first HIP error (cuda_rasterizer/auxiliary.h:220-227).
 *   - Matrices are the (4,4) row-major tensors CityGS-X passes
 *     (scene/cameras.py:124-140): p_view = [p,1] @ viewmatrix.
 *
 * Reference paths: CR/ = submodule_cityx/diff-gaussian-rasterization/cuda_rasterizer/,
 * DGR/ = submodule_cityx/diff-gaussian-rasterization/, KNN/ = submodule_cityx/simple-knn/.
 */
#ifndef GSRAST_H_INCLUDED
#define GSRAST_H_INCLUDED

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* gs_stream_t;

/* Grows a caller-owned byte buffer to at least nbytes and returns its device
 * address (host callback).  Replaces std::function<char*(size_t)> of
 * CR/rasterizer.h:38-40,131-133 / DGR/rasterize_points.cu:31-37. */
typedef char* (*gs_resize_fn)(size_t nbytes, void* user);

/* Message for the last non-zero return on this thread (host string). */
const char* gs_last_error(void);

/* Replaces GetBlockXY (DGR/rasterize_points.cu:858-861): tile width, tile
 * height and 1-D block size, i.e. (16, 16, 256).  Host pointers. */
int gs_get_block_xy(int* block_x, int* block_y, int* one_dim_block);

/* Replaces Rasterizer::markVisible (CR/rasterizer.h:30-35,
 * CR/rasterizer_impl.cu:147-159): present[i] = (view-space z > 0). */
int gs_mark_visible(int P, const float* means3D, const float* viewmatrix, const float* projmatrix,
                    uint8_t* present, gs_stream_t stream);

/* Replaces Rasterizer::visible_filter (CR/rasterizer.h:40-57,
 * CR/rasterizer_impl.cu:517-573): radii only.  Either scales+rotations or
 * cov3D_precomp may be NULL.  No scratch buffers are needed. */
int gs_visible_filter(int P, int M, int width, int height, const float* means3D, const float* scales,
                      float scale_modifier, const float* rotations, const float* cov3D_precomp,
                      const float* viewmatrix, const float* projmatrix, float tan_fovx, float tan_fovy,
                      int prefiltered, int* radii, int debug, gs_stream_t stream);

/* Replaces Rasterizer::preprocessForward (CR/rasterizer.h:61-84,
 * CR/rasterizer_impl.cu:336-425).  Shapes: means2D (P,2), depths (P), radii
 * (P) int32, cov3D (P,6), conic_opacity (P,4), rgb (P,3), clamped (P,3) bytes.
 * Every output element is written (zeros for culled Gaussians), so outputs
 * need no initialisation.  cov3D may be NULL (not stored): gs_preprocess_backward
 * then forms the covariances again from scales and rotations.  shs == NULL or M == 0: colour is left zero, as in
 * the reference (its SH call is commented out, CR/forward.cu:243-250);
 * otherwise shs is (P,M,3) and rgb/clamped follow CR/forward.cu:21-72 at
 * degree D.  tiles_touched (P) uint32 is optional (NULL to skip): the tile
 * rectangle area of each surviving Gaussian (CR/forward.cu:258).
 * prefiltered is accepted and ignored (the reference traps the GPU when a
 * prefiltered Gaussian is culled, CR/auxiliary.h:210-214).
 * dcolor_ddir (no counterpart in the reference; NULL to skip): (P,3,3), in SH
 * mode the derivative of every surviving Gaussian's three colour channels with
 * respect to the unit view direction, [axis][channel] (rows of culled
 * Gaussians are not written).  It is all that gs_preprocess_backward needs the
 * coefficients for: a caller that keeps it (36 bytes per Gaussian) saves the
 * backward call the 192-byte coefficient rows.
 * blend_records (no counterpart in the reference; NULL to skip): (P,16) floats, 16-byte aligned: the blend
 * kernels' operand records, one 64-byte record per Gaussian, (x, y, conic.x, conic.y) (conic.w, opacity, r, g)
 * (b, map0, map1, map2) (map3, map4, depth, 0).  This call writes the record of every surviving Gaussian in
 * full: the five geometry channels are the ones gs_all_map_forward gives for the same means3D, scales (as
 * passed here), rotations, viewmatrix and cam_pos, bit for bit.  A caller that blends with exactly those
 * channels hands the records to gs_render_forward (gs_render_options.blend_records) and gs_render_backward and
 * saves them the pass that packs the same records from the separate arrays. */
int gs_preprocess_forward(float* means2D, float* depths, int* radii, float* cov3D, float* conic_opacity,
                          float* rgb, uint8_t* clamped, uint32_t* tiles_touched, int P, int D, int M, int width,
                          int height, const float* means3D, const float* scales, const float* rotations,
                          const float* shs, const float* opacities, float scale_modifier, const float* viewmatrix,
                          const float* projmatrix, const float* cam_pos, float tan_fovx, float tan_fovy,
                          int prefiltered, int debug, float* dcolor_ddir, float* blend_records,
                          gs_stream_t stream);

/* Replaces Rasterizer::preprocessBackward (CR/rasterizer.h:86-111,
 * CR/rasterizer_impl.cu:427-489) together with the tensor repacking of
 * PreprocessGaussiansBackwardCUDA (DGR/rasterize_points.cu:181-194):
 * dL_dconic_opacity is the packed (P,4) gradient [conic.x, conic.y, conic.w,
 * opacity]; dL_dmean2D has mean2D_stride (2 or 3) floats per row.  Outputs
 * dL_dmean3D (P,3), dL_dscale (P,3), dL_drot (P,4), dL_dopacity (P) are fully
 * written.  dL_dsh: NULL in reference-compatible mode; (P,M,3) in SH mode,
 * where dL_dcolor (P,3) and clamped are read.  dL_dcov3D (P,6) is optional
 * (NULL: kept in registers).  cov3D: what gs_preprocess_forward stored, or NULL with
 * scales and rotations given (the covariances are then formed again, the same bits).
 * dcolor_ddir: NULL, or what gs_preprocess_forward
 * left for the same inputs and camera; shs is then not read and may be NULL.
 * Same results either way, bit for bit. */
int gs_preprocess_backward(const int* radii, const float* cov3D, const uint8_t* clamped, int P, int D, int M,
                           int width, int height, const float* means3D, const float* scales,
                           const float* rotations, const float* shs, float scale_modifier,
                           const float* viewmatrix, const float* projmatrix, const float* campos, float tan_fovx,
                           float tan_fovy, const float* dL_dmean2D, int mean2D_stride,
                           const float* dL_dconic_opacity, const float* dL_dcolor, float* dL_dmean3D,
                           float* dL_dcov3D, float* dL_dscale, float* dL_drot, float* dL_dsh, float* dL_dopacity,
                           int debug, const float* dcolor_ddir, gs_stream_t stream);

/* No counterpart in the reference: per-call options of gs_render_forward (NULL = all defaults).  A field below
 * zero keeps its default; struct_bytes is sizeof(gs_render_options) as the caller compiled it.
 * gs_render_forward builds the per-tile lists by bucketing the instances by tile (a counting sort) and sorting
 * each tile's list on its own: lists of up to 2048 records in registers, longer ones by a radix sort on the depth
 * bits that one workgroup runs inside its CU (up to 16384 records at once; a longer list is first split by its
 * leading depth bits into parts that fit).  A tile grid of more than 30000 tiles takes the reference's own route instead: (tile | depth) keys
 * (rasterizer_impl.cu:74-117), one radix sort over all of them (:675-684), identifyTileRanges (:122-144).  All
 * give the same lists bit for bit.
 * tile_sort_small_limit lowers the list length that is sorted in registers (default and maximum 2048; 0 = the
 * view takes the reference's route) and tile_sort_block_records the number of records the per-tile radix sort
 * holds at once (default and maximum 16384; 0 or below = default), so that small scenes can exercise every route.
 * The library keeps no such setting between calls. */
typedef struct gs_render_options {
  uint32_t struct_bytes;
  int32_t tile_sort_small_limit;
  int32_t tile_sort_block_records;
  int32_t expected_longest_list;
  /* What the caller expects of the view, typically the previous view's figures with a margin (0 = no idea).
   * With expected_instances > 0 (and a gs_render_result to report into) gs_render_forward does not wait for the
   * instance count before it goes on: it sizes the binning buffer for expected_instances, launches the list
   * kernels and the blend right behind the counting kernels, and lets a device-side check turn them into no-ops
   * if the view has more instances than that or a list longer than expected_longest_list (0 = any length; a
   * figure of at most 2048 spares the launch of the radix sort's kernels); in that case the lists are built
   * again the ordinary way, so the result never depends on the expectation, only the time does. */
  int64_t expected_instances;
  /* The blend kernels' operand records of this view's Gaussians as gs_preprocess_forward wrote them (their
   * geometry channels must be the all_map this call is given; with render_geo == 0 they are not read), or NULL:
   * the call then packs
   * them itself when the view has more than 0.8 instances per Gaussian.  The same pointer goes to
   * gs_render_backward; the records must stay as they are until that call has run. */
  const float* blend_records;
} gs_render_options;

/* What gs_render_forward reports besides the instance count (optional, NULL to skip; struct_bytes as above):
 * the longest per-tile list (0 on the radix route), whether the list kernels ran ahead of the host, and
 * binning_capacity: the instance count the arrays inside the binning buffer are laid out for, which is the
 * instance count itself unless the kernels ran ahead.  gs_render_backward and gs_binning_state_layout take it. */
typedef struct gs_render_result {
  uint32_t struct_bytes;
  int32_t longest_list;
  int64_t binning_capacity;
  int32_t launched_ahead;
  int32_t reserved;
} gs_render_result;

/* Replaces Rasterizer::renderForward (CR/rasterizer.h:130-160,
 * CR/rasterizer_impl.cu:586-846): tile count -> prefix sum -> host read-back of
 * the instance count (the call blocks on the stream there, as the reference
 * does at :653) -> key emission -> 64-bit radix sort on 32+bits(tiles) bits
 * -> tile ranges -> blend -> per-tile statistics.
 * out_color (3,H,W) is written in full: pixels of tiles with compute_locally == 0 read 0, as in the reference,
 * whose binding allocates the images zero-filled (rasterize_points.cu:303-307); so are out_all_map (5,H,W) and
 * out_plane_depth (1,H,W) when render_geo != 0 (they are not touched otherwise: pass them zero-filled, as the
 * reference leaves them) and out_max_weight_depth when given.  A Gaussian whose colour or geometry channels are
 * not finite reaches exactly the pixels that blend it (CR/forward.cu:381-407).
 * out_observe (P) int32 is cleared by the call
 * (the reference's binding allocates it zeroed, rasterize_points.cu:305) and then counted;
 * n_render / n_consider / n_contrib are (tiles) int32, fully written.
 * *num_rendered (host) receives the instance count R.  A view may have up to 2^31-2 instances (positions are
 * 32-bit, as in the reference, whose prefix sum wraps beyond that: here the call fails instead); a view that takes
 * the radix sort over all keys (a grid of more than 30000 tiles, or tile_sort_small_limit = 0) up to 2^30-2, the
 * capacity of that sort (gs_sort_max_pairs).
 * out_max_weight_depth (H*W, optional, NULL to skip) has no counterpart in the reference: per pixel the view-space
 * depth (depths[g]) of the Gaussian that blends with the largest weight alpha * T, the front-most among equals, 0
 * where nothing blends; asking for it changes no other output.
 * elapsed_ms (host, optional): if non-NULL the call times key emission + sort
 * + blend with events and blocks until done (the forward_render_time the
 * reference stores at CR/rasterizer_impl.cu:754-755).
 * The geometry buffer is asked for 8 bytes per Gaussian (tile counts and their prefix sum) plus the prefix sum's
 * workspace (the reference's holds the preprocess outputs as well, CR/rasterizer_impl.cu:160-188; here those are
 * the caller's tensors).  The binning buffer is asked for 64 bytes per Gaussian beyond what
 * gs_binning_state_layout reports when this call packs the blend kernels' operand records itself (a view with
 * more than 0.8 instances per Gaussian and no blend_records from the caller). */
int gs_render_forward(gs_resize_fn geometryBuffer, void* geometry_user, gs_resize_fn binningBuffer,
                      void* binning_user, gs_resize_fn imageBuffer, void* image_user, int P,
                      const float* background, int width, int height, float focal_x, float focal_y, float cx,
                      float cy, const float* viewmatrix, const float* cam_pos, const float* all_map,
                      const float* means2D, const float* depths, const int* radii, const float* conic_opacity,
                      const float* rgb, const uint8_t* compute_locally, float* out_color, int* n_render,
                      int* n_consider, int* n_contrib, int* out_observe, float* out_all_map,
                      float* out_plane_depth, float* out_max_weight_depth, int render_geo, int debug,
                      int* num_rendered, float* elapsed_ms, const gs_render_options* options,
                      gs_render_result* result, gs_stream_t stream);

/* Replaces Rasterizer::renderBackward (CR/rasterizer.h:162-187,
 * CR/rasterizer_impl.cu:850-932) plus the repacking of
 * RenderGaussiansBackwardCUDA (DGR/rasterize_points.cu:428-440).  The three
 * buffers are the ones gs_render_forward filled (the geometry buffer is read
 * too: it holds the per-Gaussian instance offsets and, for a view with more than 0.8 instances per Gaussian, one
 * 64-byte record per visible Gaussian with the values of means2D, conic_opacity, rgb and all_maps that the forward
 * call was given, which the kernel then reads instead of those arrays: pass the forward call's arrays, as the
 * reference does).  Gradient outputs are
 * fully written and need no initialisation: dL_dmean2D (P,2), dL_dmean2D_abs
 * (P,3), dL_dconic_opacity (P,4) packed [x, y, w, opacity], dL_dcolor (P,3),
 * dL_dall_map (P,5).  Where the reference adds every pixel's contribution
 * with global float atomics, this implementation writes one 64-byte record
 * per (tile, Gaussian) instance into instance_grads, a caller-provided scratch
 * of gs_render_backward_workspace_bytes(R) bytes, and sums each Gaussian's
 * records in a second kernel (no atomics, run-to-run deterministic).
 * elapsed_ms as above (backward_render_time, CR/rasterizer_impl.cu:924-926).
 * binning_capacity: gs_render_result.binning_capacity of the forward call (0 or R if it did not run ahead).
 * blend_records: gs_render_options.blend_records of the forward call (NULL if that call was given none). */
size_t gs_render_backward_workspace_bytes(int R);
int gs_render_backward(int P, int R, const float* background, int width, int height, float tan_fovx,
                       float tan_fovy, const char* geom_buffer, const char* binning_buffer,
                       const char* img_buffer, const uint8_t* compute_locally, const float* dL_dpix,
                       const float* dL_dout_all_map, const float* dL_dout_plane_depth, float* dL_dmean2D,
                       float* dL_dmean2D_abs, float* dL_dconic_opacity, float* dL_dcolor, float* dL_dall_map,
                       const float* means2D, const float* conic_opacity, const float* rgb, const float* all_maps,
                       const float* all_map_pixels, int render_geo, int debug, float* instance_grads,
                       size_t instance_grads_bytes, float* elapsed_ms, int64_t binning_capacity,
                       const float* blend_records, gs_stream_t stream);

/* Replaces SimpleKNN::knn / distCUDA2 (KNN/simple_knn.h:17, KNN/simple_knn.cu:185-221,
 * KNN/spatial.cu:17-35): mean_dists[i] = mean squared distance from point i
 * to its three nearest other points (a point with fewer than three finite
 * distances reads FLT_MAX for the missing ones, as in the reference).  The
 * result is the exact one, so it does not depend on how the points are
 * ordered inside the call (a Hilbert curve here, Morton codes in the
 * reference).  points (P,3).  The reference allocates its temporaries
 * internally; here the caller passes a workspace of gs_knn_workspace_bytes(P)
 * bytes. */
size_t gs_knn_workspace_bytes(int P);
int gs_knn_dist2(int P, const float* points, float* mean_dists, void* workspace, size_t workspace_bytes,
                 gs_stream_t stream);

/* Replaces the caller-side torch code that builds the per-Gaussian geometry channels between the two
 * rasterizer ops (gaussian_renderer/__init__.py:1501-1518: quaternion_to_matrix(normalize(rotations)),
 * axis of the smallest scale as normal, flipped towards the camera, rotated by viewmatrix[:3,:3];
 * distance = |normal . p_cam|).  all_map (P,5) = [normal_cam(3), 1, distance].  `scales` only has to order
 * like the activated scales (the reference takes the argmin of exp(scales)).
 * The backward entry returns what autograd derives from those lines: dL/dmeans3D (P,3) and
 * dL/drotations (P,4, with respect to the unnormalised quaternions); scales get no gradient.
 * Every output element is written. */
int gs_all_map_forward(int P, const float* means3D, const float* scales, const float* rotations,
                       const float* viewmatrix, const float* campos, float* all_map, gs_stream_t stream);
int gs_all_map_backward(int P, const float* means3D, const float* scales, const float* rotations,
                        const float* viewmatrix, const float* campos, const float* dL_dall_map,
                        float* dL_dmeans3D, float* dL_drotations, gs_stream_t stream);

/* Replaces the body of generate_neural_gaussians (gaussian_renderer/__init__.py:789-899) in the reference's
 * default configuration (arguments/__init__.py:94-124: feat_dim 32, no feature bank, no appearance embedding, no
 * distance or level inputs, dist2level 'round'; the options further down add to it), on the anchors already
 * selected by visible_mask (:794-798):
 *   x = [feat, (anchor - campos) / |anchor - campos|]                                   (:801-828)
 *   neural_opacity = mlp_opacity(x), mask = neural_opacity > 0                          (:841-858)
 *   color = mlp_color(x), scale_rot = mlp_cov(x), and for the selected offsets, in (anchor, offset) order,
 *   xyz = anchor + offset * scaling[:3], scaling = scaling[3:] * sigmoid(scale_rot[:3]),
 *   rot = normalize(scale_rot[3:7])                                                     (:866-896)
 * mlp_params: 12 device pointers, {W1 (32x35; see input_flags), b1 (32), W2 (out x 32), b2 (out)} of mlp_opacity (out = n_offsets,
 * Tanh), mlp_color (3 n_offsets, Sigmoid) and mlp_cov (7 n_offsets), as nn.Linear stores them
 * (scene/gaussian_model.py:131-149).  anchor (N,3), feat (N,32), offsets (N,n_offsets,3), scaling (N,6) = the
 * activated get_scaling, campos (3).  n_offsets must satisfy gs_neural_supported().
 * opacity_scale (N floats, or NULL for none) serves dist2level 'progressive' (:844-848): neural_opacity =
 * mlp_opacity(x) * opacity_scale[anchor], where the caller passes _prog_ratio with 1 for the anchors outside
 * transition_mask; it must be positive wherever the product is (the reference's lies in (0, 1]).  With it the
 * call also writes opacity_tanh (N*n_offsets): the MLP's output before the factor, which gs_neural_backward takes
 * back (1 - tanh^2 of a saturated unit cannot be recovered from the product); NULL without opacity_scale.
 * input_flags / level serve the MLPs' optional inputs (:824-829, :839-877; scene/gaussian_model.py:118-149):
 * bit 0 / 1 / 2 (add_opacity_dist / add_color_dist / add_cov_dist) = that MLP takes the distance
 * |anchor - campos| as input column 35, bit 3 (add_level) = all three take level[anchor] (N floats) as their last
 * input column; an MLP's W1 is then 32 x 36 or 32 x 37, and so is its gradient.  0 and NULL otherwise.  The
 * distance carries a gradient to the anchor, the level none.
 *
 * Step 1, gs_neural_opacity_forward: writes neural_opacity (N*n_offsets), mask (u8, N*n_offsets) and
 * first (u32, N: selected offsets of all earlier anchors), and returns their number in *num_selected (the host
 * waits for it, as the reference does at the boolean indexing :858).  workspace: gs_neural_workspace_bytes().
 * Step 2, gs_neural_gaussians_forward, with the same workspace (it holds the rearranged weights): writes the
 * rows of xyz (S,3), color (S,3), opacity (S), scaling_out (S,3), rot (S,4) and aux (S,4: the three sigmoids of
 * the scale and |scale_rot[3:7]|, kept for the backward pass).
 * gs_neural_backward: gradients of the five (S,.) outputs -> d_anchor (N,3), d_feat (N,32),
 * d_offsets (N,n_offsets,3), d_scaling (N,6) and d_mlp_params (12 pointers shaped like mlp_params); every
 * element is written.  neural_opacity itself is treated as not differentiated (the reference only uses it
 * detached, scene/gaussian_model.py:1183).  workspace: gs_neural_backward_workspace_bytes(). */
int gs_neural_supported(int n_offsets);
size_t gs_neural_workspace_bytes(int64_t num_anchors, int n_offsets);
int gs_neural_opacity_forward(int64_t num_anchors, int n_offsets, const float* anchor, const float* feat,
                              const float* campos, const float* const* mlp_params, const float* opacity_scale,
                              const float* level, int input_flags, float* neural_opacity, float* opacity_tanh,
                              uint8_t* mask, uint32_t* first, void* workspace, size_t workspace_bytes,
                              int64_t* num_selected, gs_stream_t stream);
int gs_neural_gaussians_forward(int64_t num_anchors, int n_offsets, int64_t num_selected, const float* anchor,
                                const float* feat, const float* offsets, const float* scaling, const float* campos,
                                const float* level, const float* neural_opacity, const uint32_t* first,
                                const void* workspace, size_t workspace_bytes, float* xyz, float* color,
                                float* opacity, float* scaling_out, float* rot, float* aux, gs_stream_t stream);
size_t gs_neural_backward_workspace_bytes(int64_t num_anchors, int n_offsets);
int gs_neural_backward(int64_t num_anchors, int n_offsets, int64_t num_selected, const float* anchor,
                       const float* feat, const float* offsets, const float* scaling, const float* campos,
                       const float* const* mlp_params, const float* opacity_scale, const float* level,
                       int input_flags, const float* neural_opacity, const float* opacity_tanh,
                       const uint32_t* first, const float* color, const float* rot, const float* aux,
                       const float* dL_dxyz, const float* dL_dcolor,
                       const float* dL_dopacity, const float* dL_dscaling, const float* dL_drot, float* d_anchor,
                       float* d_feat, float* d_offsets, float* d_scaling, float* const* d_mlp_params,
                       void* workspace, size_t workspace_bytes, gs_stream_t stream);

/* Replaces pixelwise_l1_with_mask and pixelwise_ssim_with_mask (utils/loss_utils.py:88-132, 11x11 Gaussian
 * window of create_window :27-43, zero padding; called at gaussian_renderer/loss_distribution.py:267-279).
 * img1, img2 and the maps are (channels, height, width) float32; pixel_mask u8[height*width] (0/1) or NULL
 * for all ones.  l1_map = |img1-img2| * mask, ssim_map = SSIM * mask.  d_mu / d_xx / d_xy (each the size
 * of a map, or all three NULL when no backward pass will follow) receive the partial derivatives the
 * backward entry needs.  gs_ssim_l1_backward writes dL/dimg1 for upstream gradients dL_dl1_map and
 * dL_dssim_map (either may be NULL = zero); img2 is treated as constant (it is the ground truth). */
int gs_ssim_l1_forward(int channels, int height, int width, const float* img1, const float* img2,
                       const uint8_t* pixel_mask, float* l1_map, float* ssim_map, float* d_mu, float* d_xx,
                       float* d_xy, gs_stream_t stream);
int gs_ssim_l1_backward(int channels, int height, int width, const float* img1, const float* img2,
                        const uint8_t* pixel_mask, const float* dL_dl1_map, const float* dL_dssim_map,
                        const float* d_mu, const float* d_xx, const float* d_xy, float* dL_dimg1,
                        gs_stream_t stream);

/* Replaces the body of GaussianModel.training_statis (scene/gaussian_model.py:1181-1205), the per-view
 * update of the densification statistics.  num_anchors anchors with n_offsets offsets each;
 * anchor_visible_mask u8[num_anchors]; offset_selection_mask u8[num_candidates] and opacity
 * f32[num_candidates] over the candidates of the visible anchors in anchor order (num_candidates =
 * visible anchors x n_offsets); update_filter u8[num_selected] and viewspace_grad f32[num_selected][grad_stride]
 * (columns 0 and 1 are used) over the selected candidates in order.  Updated in place:
 * opacity_accum f32[num_anchors], anchor_demon f32[num_anchors], offset_gradient_accum and offset_denom
 * f32[num_anchors*n_offsets].  Masks are bytes holding 0 or 1 (torch.bool).  Indices that the masks would
 * send past num_candidates / num_selected (inconsistent inputs) are ignored rather than read.
 * workspace: gs_training_stats_workspace_bytes(num_anchors, num_candidates) bytes. */
size_t gs_training_stats_workspace_bytes(int64_t num_anchors, int64_t num_candidates);
int gs_training_stats(int64_t num_anchors, int n_offsets, int64_t num_candidates, int64_t num_selected,
                      const uint8_t* anchor_visible_mask, const uint8_t* offset_selection_mask,
                      const uint8_t* update_filter, const float* viewspace_grad, int grad_stride,
                      const float* opacity, float* opacity_accum, float* anchor_demon,
                      float* offset_gradient_accum, float* offset_denom, void* workspace, size_t workspace_bytes,
                      gs_stream_t stream);

/* Replaces `gaussians.max_radii2D[visibility_filter] = torch.max(gaussians.max_radii2D[visibility_filter],
 * radii[visibility_filter])` (densification.py:71-73): the running maximum of the screen-space radius of every
 * Gaussian, over the views that saw it.  radii int32[n], visibility_filter u8[n] (0/1), max_radii2D float[n]. */
int gs_max_radii_update(int64_t n, const int* radii, const uint8_t* visibility_filter, float* max_radii2D,
                        gs_stream_t stream);

/* Replaces optimizer.step() of the reference's torch.optim.Adam(lr=0.0, eps=1e-15) with per-group learning
 * rates (scene/gaussian_model.py:574, stepped at train_internal.py:404-417) for `count` tensors in one
 * launch: update rule of torch 2.0.0 with betas (beta1, beta2), no weight decay, no amsgrad.
 * params / grads / exp_avg / exp_avg_sq: host arrays of `count` device pointers (float32, sizes[i] elements
 * each); hyper-parameters are doubles, as the Python floats of that optimizer are; lrs[i] and steps[i] (the step number after this update, >= 1) per tensor; grad_scale multiplies
 * every gradient first (1/bsz of train_internal.py:407-410; 1.0 for none).  params, exp_avg and
 * exp_avg_sq are updated in place; grads are only read.  Tensors with sizes[i] <= 0 are skipped. */
int gs_adam_step(int count, float* const* params, const float* const* grads, float* const* exp_avg,
                 float* const* exp_avg_sq, const long long* sizes, const double* lrs, const int* steps, double beta1,
                 double beta2, double eps, float grad_scale, gs_stream_t stream);

/* ---- Stage-level entry points: the individual steps of renderForward, exposed
 * so each can be checked and profiled on its own. ---- */

/* updateTileTouched (CR/rasterizer_impl.cu:264-288). */
int gs_tile_count(int P, int width, int height, const int* radii, const float* means2D,
                  const uint8_t* compute_locally, uint32_t* tiles_touched, gs_stream_t stream);

/* cub::DeviceScan::InclusiveSum as called at CR/rasterizer_impl.cu:648 (uint32). */
size_t gs_scan_workspace_bytes(int64_t n);
int gs_inclusive_sum(int64_t n, const uint32_t* in, uint32_t* out, void* workspace, size_t workspace_bytes,
                     gs_stream_t stream);

/* No counterpart in the reference: gs_inclusive_sum for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  Same result as gs_inclusive_sum,
 * no workspace argument: the scan's spine (one word per 2048 elements) lives in a static device array inside the
 * library, 256 KiB, which every GPU the library runs on holds until the process ends.  n may be at most
 * gs_inclusive_sum_static_max() = 2^27 elements; a larger n is refused with an error.  The call allocates and
 * frees nothing.  The first call on a device looks the array's device address up (a mutex, hipGetDevice and
 * hipGetSymbolAddress: not a sequence to record into a graph), so make one call per device outside any capture
 * before relying on it there.  Every call on a GPU shares
 * that GPU's array: the call itself writes every word it later reads, so nothing has to be cleared between
 * calls, but calls that overlap on one GPU (two streams, two threads) race on it and must be serialised by
 * the caller.  in and out may be the same array. */
int64_t gs_inclusive_sum_static_max(void);
int gs_inclusive_sum_static(int64_t n, const uint32_t* in, uint32_t* out, gs_stream_t stream);

/* duplicateWithKeys (CR/rasterizer_impl.cu:74-117). offsets = inclusive sum of tiles_touched. */
int gs_duplicate_with_keys(int P, int width, int height, const float* means2D, const float* depths,
                           const uint32_t* offsets, const int* radii, const uint8_t* compute_locally,
                           uint64_t* keys, uint32_t* values, gs_stream_t stream);

/* cub::DeviceRadixSort::SortPairs on bits [0, end_bit) (CR/rasterizer_impl.cu:679-684,
 * KNN/simple_knn.cu:210-213): stable.  The input arrays are clobbered; the
 * sorted pairs land in keys_out / vals_out.  At most gs_sort_max_pairs() = 2^30-2 pairs (the look-back words of a
 * pass carry 30-bit counts beside their two flag bits); more is refused with an error before anything is launched. */
int64_t gs_sort_max_pairs(void);
size_t gs_sort_workspace_bytes(int64_t n);
/* No counterpart in the reference.  A pass of the sort waits, with a bounded number of polls, for the digit counts
 * of earlier tiles; if a wait ever ran out the sort sets a word in its workspace (at byte
 * gs_sort_workspace_error_offset() of the 256-byte aligned workspace) instead of hanging, and its output is not
 * sorted.  Three ways to learn of it:
 *   gs_sort_status waits for the stream and returns 1 (with an error message) if the last sort that used this
 *   workspace set the word, else 0;
 *   gs_sort_check_async enqueues a one-thread kernel that raises a process-wide sticky fault word in pinned host
 *   memory if the word is set, and waits for nothing;
 *   gs_pending_fault returns 1 (with a message) if the fault word is raised, and lowers it.
 * gs_render_forward (radix route) and gs_knn_dist2 enqueue that check themselves after their sorts, and
 * gs_render_forward, gs_render_backward and gs_knn_dist2 fail on entry while the fault word is raised (lowering
 * it): a sort that gave up is therefore reported by the next of these calls made after its kernels have run, and
 * by the same call when debug != 0 or elapsed_ms is given (both wait for the stream). */
size_t gs_sort_workspace_error_offset(void);
int gs_sort_status(const void* workspace, gs_stream_t stream);
int gs_sort_check_async(const void* workspace, gs_stream_t stream);
int gs_pending_fault(void);
int gs_sort_pairs_u64(int64_t n, uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out,
                      int end_bit, void* workspace, size_t workspace_bytes, gs_stream_t stream);
int gs_sort_pairs_u32(int64_t n, uint32_t* keys_in, uint32_t* keys_out, uint32_t* vals_in, uint32_t* vals_out,
                      int end_bit, void* workspace, size_t workspace_bytes, gs_stream_t stream);

/* getHigherMsb (CR/rasterizer_impl.cu:39-54); host function. */
uint32_t gs_higher_msb(uint32_t n);

/* memset + identifyTileRanges (CR/rasterizer_impl.cu:687-697). ranges is (tiles,2) uint32. */
int gs_identify_tile_ranges(int64_t L, const uint64_t* keys_sorted, int tiles, uint32_t* ranges,
                            gs_stream_t stream);

/* FORWARD::render + get_n_render + 2x reduce_data_per_block
 * (CR/forward.cu:264-437, CR/rasterizer_impl.cu:219-262). */
int gs_render_tiles_forward(int P, int width, int height, float focal_x, float focal_y, float cx, float cy,
                            const uint32_t* ranges, const uint32_t* point_list, const float* means2D,
                            const float* rgb, const float* all_map, const float* conic_opacity,
                            const uint8_t* compute_locally, const float* background, int render_geo,
                            float* final_T, uint32_t* n_contrib_px, uint32_t* n_contrib2loss_px, float* out_color,
                            int* out_observe, float* out_all_map, float* out_plane_depth, int* n_render,
                            int* n_consider, int* n_contrib, gs_stream_t stream);

/* BACKWARD::render (CR/backward.cu:324-567) on explicit arrays.  emission_sorted[k] is the index, in
 * key-emission order, of the instance at sorted position k (the permutation the sort applied);
 * point_offsets is the inclusive prefix sum of tiles touched; instance_grads is (R,16) float scratch. */
int gs_render_tiles_backward(int P, int width, int height, float tan_fovx, float tan_fovy,
                             const float* background, const uint32_t* ranges, const uint32_t* point_list,
                             const float* means2D, const float* conic_opacity, const float* rgb,
                             const float* all_maps, const float* all_map_pixels, const float* final_T,
                             const uint32_t* n_contrib_px, const uint8_t* compute_locally, const float* dL_dpix,
                             const float* dL_dout_all_map, const float* dL_dout_plane_depth, int render_geo,
                             const uint32_t* emission_sorted, const uint32_t* point_offsets,
                             float* instance_grads, float* dL_dmean2D, float* dL_dmean2D_abs,
                             float* dL_dconic_opacity, float* dL_dcolor, float* dL_dall_map, gs_stream_t stream);

/* A test hook, not part of the path (no counterpart in the reference, nothing in the library calls it; it is
 * exported so that the test suite can check the inline-assembly reductions on their own): runs the two cross-lane
 * reductions of the blend kernels on one 64-lane wave.  in is (64,16) floats;
 * out_wave (16) receives the sums over all 64 lanes, out_rows (4,16) the sums
 * over each 16-lane row.  Synchronises the stream. */
int gs_selftest_reductions(const float* in, float* out_wave, float* out_rows, gs_stream_t stream);

/* Optional per-stage GPU timing, the role of the reference's MyTimerOnGPU
 * (CR/timers.cu:11-79; stage names at CR/rasterizer_impl.cu:385-752): while
 * enabled, each stage of the composite entry points (preprocess_fwd,
 * tile_count, bucket_scatter, tile_sort, or on the radix route inclusive_sum,
 * duplicate_with_keys, sort_pairs, identify_tile_ranges; pack_operands; render_fwd,
 * render_bwd, preprocess_bwd; knn_dist2 and its phases knn_minmax, knn_keys,
 * knn_sort, knn_gather, knn_boxes, knn_box_mean_dist)
 * is bracketed by an event pair on its stream.  Nothing is synchronised until
 * gs_stage_timing_collect, which waits for the recorded events and writes one
 * line per stage, "name total_ms launches", into report (host buffer), then
 * clears the records.  Process wide; safe to use while other threads are inside entry points (a stage's pair
 * is filed under a lock once both events are recorded).  Apart from this switch, the pinned words that carry
 * instance counts to the host and the sticky fault word of the radix sort, the library holds no state between
 * calls. */
int gs_stage_timing_enable(int enable);
int gs_stage_timing_collect(char* report, size_t report_bytes);

/* Byte offsets of the arrays inside the buffers gs_render_forward fills
 * (the role of ImageState / BinningState::fromChunk, CR/rasterizer_impl.cu:182-205),
 * relative to the 256-byte-aligned start of each buffer.  Host pointers.  R of gs_binning_state_layout is the
 * forward call's binning_capacity (the instance count unless its kernels ran ahead of the host). */
int gs_image_state_layout(int width, int height, size_t* accum_alpha, size_t* n_contrib, size_t* n_contrib2loss,
                          size_t* ranges, size_t* total_bytes);
int gs_binning_state_layout(int64_t R, int width, int height, size_t* point_list, size_t* point_list_keys,
                            size_t* point_list_unsorted, size_t* point_list_keys_unsorted, size_t* total_bytes);
int gs_geometry_state_layout(int P, size_t* tiles_touched, size_t* point_offsets, size_t* total_bytes);

#ifdef __cplusplus
}
#endif
#endif /* GSRAST_H_INCLUDED */
