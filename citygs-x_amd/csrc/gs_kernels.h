// Internal launch interface between the C-ABI layer (api.hip) and the kernel
// translation units.  All pointers are device pointers unless noted.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace gs {

struct PreprocessFwdArgs {
  int P, D, M, W, H;
  const float *means3D, *scales, *rotations, *opacities, *shs;
  float scale_modifier;
  const float *viewmatrix, *projmatrix, *campos;
  float tanx, tany;
  int* radii;
  float *means2D, *depths, *cov3D, *conic_opacity, *rgb;
  uint8_t* clamped;
  uint32_t* tiles_touched;  // optional
  // optional (P,3,3): derivative of the three colour channels with respect to the unit view direction,
  // [axis][channel], written for Gaussians that survive culling (SH mode); the backward kernel takes it in place of
  // the coefficients
  float* dcolor_ddir = nullptr;
  // optional (P,16): the blend kernels' operand records (see launch_pack_blend_operands) of the surviving
  // Gaussians, complete: the geometry channels are formed from means3D, scales, rotations, viewmatrix and campos
  // as launch_all_map_fwd forms them
  float* blend_records = nullptr;
};

struct PreprocessBwdArgs {
  int P, D, M, W, H;
  const float* means3D;
  const int* radii;
  const float* shs;
  const uint8_t* clamped;
  const float *scales, *rotations;
  float scale_modifier;
  const float *cov3D, *viewmatrix, *projmatrix, *campos;
  float tanx, tany;
  const float* dL_dmean2D;
  int mean2D_stride;               // 2 or 3 floats per row
  const float* dL_dconic_opacity;  // (P,4) packed [x, y, w, opacity]
  const float* dL_dcolor;          // (P,3), SH mode only
  float *dL_dmean3D, *dL_dcov3D /*optional*/, *dL_dsh /*optional*/, *dL_dscale, *dL_drot, *dL_dopacity /*optional*/;
  const float* dcolor_ddir = nullptr;  // optional: what the forward kernel left (PreprocessFwdArgs::dcolor_ddir)
};

// Brackets a stage with an event pair on its stream while stage timing is enabled (gs_stage_timing_enable; the
// role of the reference's MyTimerOnGPU, cuda_rasterizer/timers.cu:11-79); costs one relaxed load otherwise.  The
// pairs are read by gs_stage_timing_collect.  `stage` must be a string literal (it is kept by pointer).
struct StageScope {
  hipStream_t s;
  const char* name;
  hipEvent_t a = nullptr, b = nullptr;
  StageScope(const char* stage, hipStream_t stream);
  ~StageScope();
  StageScope(const StageScope&) = delete;
  StageScope& operator=(const StageScope&) = delete;
};

int launch_preprocess_fwd(const PreprocessFwdArgs& a, hipStream_t stream);
int launch_preprocess_bwd(const PreprocessBwdArgs& a, hipStream_t stream);
int launch_visible_filter(int P, const float* means, const float* scales, float mod, const float* rots,
                          const float* cov_pre, const float* V, const float* PM, int W, int H, float tanx,
                          float tany, int* radii, hipStream_t stream);
int launch_mark_visible(int P, const float* means, const float* V, uint8_t* present, hipStream_t stream);

// ---- binning ----
// (Gaussian, tile) instances a view may have (positions are 32-bit, counts are handed to the caller as int), and
// the count the kernels report in place of a larger, wrapped-around one
constexpr uint32_t GS_MAX_INSTANCES = 0x7FFFFFFEu;
constexpr uint32_t GS_TOO_MANY_INSTANCES = 0x7FFFFFFFu;
int launch_tile_count(int P, int W, int H, const int* radii, const float* means2D, const uint8_t* compute_locally,
                      uint32_t* tiles_touched, hipStream_t stream,
                      uint32_t* zero_words = nullptr, int64_t zero_count = 0, int* zero_per_gaussian = nullptr);
size_t scan_temp_bytes(int64_t n);
// device word of a scan's workspace that is 1 after a scan whose exact total exceeds GS_MAX_INSTANCES, else 0
const uint32_t* scan_overflow_word(const void* temp, int64_t n);
int launch_exclusive_sum_u8(int64_t n, const uint8_t* in, uint32_t* out, void* temp, hipStream_t stream,
                            uint32_t* total_out = nullptr);
// total_out, when given, is a host-visible word that receives the grand total as well (GS_TOO_MANY_INSTANCES if
// the exact total exceeds GS_MAX_INSTANCES; the 32-bit sums themselves wrap around like the reference's)
// (launch_tile_count and launch_bucket_count: zero_per_gaussian, when given, is an array of P words that the
// counting kernel clears on the way)
int launch_inclusive_sum(int64_t n, const uint32_t* in, uint32_t* out, void* temp, hipStream_t stream,
                         uint32_t* total_out = nullptr);
int launch_exclusive_sum(int64_t n, const uint32_t* in, uint32_t* out, void* temp, hipStream_t stream);
// the inclusive sum with its spine in a static device array instead of a workspace: allocates nothing, takes at
// most static_scan_max_elements() elements, and calls that overlap on one GPU share (and race on) the array
int64_t static_scan_max_elements();
int launch_inclusive_sum_static(int64_t n, const uint32_t* in, uint32_t* out, hipStream_t stream);
int launch_duplicate_with_keys(int P, int W, int H, const float* means2D, const float* depths,
                               const uint32_t* offsets, const int* radii, const uint8_t* compute_locally,
                               uint64_t* keys, uint32_t* values, uint32_t* emission /*optional*/,
                               hipStream_t stream);
// ---- binning by tile: counting sort by tile + per-tile sorts (tile_bucket.hip, tile_radix.hip) ----
constexpr int TILE_SORT_SMALL = 2048;  // longest list the register sort takes; longer ones go to the radix sort
int bucket_max_tiles();
size_t bucket_table_bytes(int T);
// tiles_touched per Gaussian, the workgroup-by-tile table, ranges (2 words per tile), the lists of tiles with more
// than small_limit records (0 = TILE_SORT_SMALL) for the radix sort's kernels, and in three host-visible words the
// number of instances (word 0, written last), the longest list (word 1) and the numbers of tiles in those lists
// (word 2: larger kernel's << 16 | smaller kernel's).  block_limit (0 = the maximum): the records the radix sort
// holds in one block, see launch_tile_sort.
// cap_instances / cap_longest: what kernels launched ahead of the host's decision were sized for; the ranges kernel
// leaves 1 in bucket_fits_word(table) if the view has at most that many instances and no longer list, else 0
int launch_bucket_count(int P, int W, int H, const int* radii, const float* means2D, const uint8_t* compute_locally,
                        uint32_t* tiles_touched, void* table, uint32_t* ranges, uint32_t small_limit,
                        uint32_t block_limit, uint32_t* host_words, int* zero_per_gaussian, uint32_t cap_instances,
                        uint32_t cap_longest, uint32_t* clear_word, hipStream_t stream);
const uint32_t* bucket_fits_word(const void* table, int T);
// records: one 16-byte record (Gaussian, emission index, depth bits, 0) per instance, grouped by tile in any
// order.  Also writes point_offsets (the inclusive prefix sum of tiles_touched).
// ahead_of_host: the kernel checks bucket_fits_word itself and does nothing if the view does not fit what it was
// launched for.
int launch_bucket_scatter(int P, int W, int H, const float* means2D, const float* depths,
                          const uint32_t* tiles_touched, uint32_t* point_offsets, const int* radii,
                          const uint8_t* compute_locally, void* table, const uint32_t* ranges, void* records,
                          bool ahead_of_host, hipStream_t stream);
// scratch: 24 bytes per instance, used for lists of more than block_limit records
int launch_tile_sort(int T, uint32_t longest, uint32_t radix_tiles, uint32_t small_limit, uint32_t block_limit,
                     const uint32_t* ranges, const void* table, const void* records, void* scratch, int64_t capacity,
                     uint64_t* keys, uint32_t* emission, uint32_t* point_list, bool ahead_of_host,
                     hipStream_t stream);
int tile_radix_mid_records();    // records one workgroup of the radix sort's smaller kernel holds (4096)
int tile_radix_block_records();  // ... and of its larger kernel (16384): longer lists are sorted in blocks
int launch_tile_radix_sort(int T, bool mid, bool lng, const uint32_t* ranges, const uint32_t* tile_lists,
                           const uint32_t* counts, uint32_t block_limit, const void* records, void* parted,
                           uint64_t* ping, uint64_t* pong, uint64_t* keys, uint32_t* emission, uint32_t* point_list,
                           const uint32_t* fits_word, hipStream_t stream);
// What the blend kernels read of a Gaussian, in one 64-byte record per Gaussian: (x, y, A, B), (C, opacity, r, g),
// (b, map0, map1, map2), (map3, map4, depth, 0); all_map and depths may be null (zeros).  Records of Gaussians with
// radius 0 are left as they are (no tile lists them).
// valid_word (optional): set to 1 by the kernel.
int launch_pack_blend_operands(int P, const int* radii, const float* means2D, const float* conic_opacity,
                               const float* rgb, const float* all_map, const float* depths, float* packed,
                               uint32_t* valid_word, hipStream_t stream);
int launch_fill_u32(int64_t n, uint32_t value, uint32_t* p, hipStream_t stream);
int launch_gather_u32(int64_t n, const uint32_t* index, const uint32_t* table, uint32_t* out, hipStream_t stream);
int launch_ssim_l1_fwd(int C, int H, int W, const float* img1, const float* img2, const uint8_t* mask,
                       float* l1_map, float* ssim_map, float* d_mu, float* d_xx, float* d_xy, hipStream_t stream);
int launch_ssim_l1_bwd(int C, int H, int W, const float* img1, const float* img2, const uint8_t* mask,
                       const float* g_l1, const float* g_ssim, const float* d_mu, const float* d_xx,
                       const float* d_xy, float* dimg1, hipStream_t stream);
size_t train_stats_temp_bytes(long long A, long long Vk);
int launch_train_stats(long long A, int k, long long Vk, long long M, const uint8_t* visible,
                       const uint8_t* selected, const uint8_t* update_filter, const float* grad, int grad_stride,
                       const float* opacity, float* opacity_accum, float* anchor_demon, float* grad_accum,
                       float* denom, void* temp, hipStream_t stream);
int launch_max_radii(long long n, const int* radii, const uint8_t* visible, float* max_radii, hipStream_t stream);
constexpr int ADAM_MAX_TENSORS = 24;  // tensors per launch (more are split over several launches)
int launch_adam(int count, float* const* params, const float* const* grads, float* const* exp_avg,
                float* const* exp_avg_sq, const long long* sizes, const double* lrs, const int* steps, double beta1,
                double beta2, double eps, float grad_scale, hipStream_t stream);
// ---- neural-Gaussian generation (n_offsets = k) ----
bool neural_supported(int k);
size_t neural_packed_floats(int k);
size_t neural_partial_floats(int k, int64_t N);
// input_flags: bit 0 / 1 / 2 = the opacity / color / cov MLP takes the distance as input column 35, bit 3 = all
// three take the anchor's level as their last input column (W1 is then 32 x 36 or 32 x 37); level (N) is read
// only with bit 3
int launch_neural_pack(int k, const float* const* params, int input_flags, float* packed, hipStream_t stream);
// opacity_scale (N, optional): per-anchor factor on the opacity MLP's output; opacity_tanh (N*k, with opacity_scale):
// the output before the factor, which the backward pass needs
int launch_neural_opacity(int64_t N, int k, const float* anchor, const float* feat, const float* level,
                          const float* campos, const float* packed, const float* opacity_scale,
                          float* neural_opacity, float* opacity_tanh, uint8_t* mask, uint8_t* counts,
                          hipStream_t stream);
int launch_neural_gaussians(int64_t N, int k, const float* anchor, const float* feat, const float* level,
                            const float* offsets, const float* scaling, const float* campos, const float* packed,
                            const float* neural_opacity, const uint32_t* first, float* xyz, float* color,
                            float* opacity, float* scal, float* rot, float* aux, hipStream_t stream);
int launch_neural_backward(int64_t N, int k, const float* anchor, const float* feat, const float* level,
                           int input_flags, const float* offsets, const float* scaling, const float* campos, const float* packed,
                           const float* neural_opacity, const float* opacity_scale, const float* opacity_tanh,
                           const uint32_t* first, const float* color_out, const float* rot_out, const float* aux,
                           const float* g_xyz, const float* g_color, const float* g_opacity, const float* g_scal,
                           const float* g_rot, float* d_anchor, float* d_feat, float* d_offsets, float* d_scaling,
                           float* const* d_params, float* slot_grads, float* partials, hipStream_t stream);
size_t neural_slot_grad_floats(int k, int64_t N);
int launch_all_map_fwd(int P, const float* means, const float* scales, const float* rots, const float* V,
                       const float* campos, float* out, hipStream_t stream);
int launch_all_map_bwd(int P, const float* means, const float* scales, const float* rots, const float* V,
                       const float* campos, const float* grad_out, float* dmeans, float* drots,
                       hipStream_t stream);
// already_zero: the caller cleared `ranges` itself; gather_*: also write gather_out[i] = gather_table[gather_index[i]]
// sort_error / fault_word: also raise the host-visible fault word if the sort's error word is set
int launch_tile_ranges(int64_t L, const uint64_t* keys_sorted, int T, uint32_t* ranges, hipStream_t stream,
                       bool already_zero = false, const uint32_t* gather_index = nullptr,
                       const uint32_t* gather_table = nullptr, uint32_t* gather_out = nullptr,
                       const uint32_t* sort_error = nullptr, uint32_t* fault_word = nullptr);

// ---- radix sort (stable, LSD, 8-bit digits) ----
size_t sort_temp_bytes(int64_t n);
int64_t sort_max_pairs();  // 2^30 - 2
// device word of a sort's workspace that is nonzero after a sort in which a bounded wait of the look-back ran out
// (the order of the output is then not to be trusted)
const uint32_t* sort_error_word(const void* temp);
size_t sort_error_word_offset();  // its byte offset in the workspace
// one-thread kernel: stores 1 (system scope) to the host-visible fault_word if *error_word is nonzero
int launch_sort_fault_report(const uint32_t* error_word, uint32_t* fault_word, hipStream_t stream);
// Sorts on key bits [0, end_bit), ping-ponging between the (a) and (b) arrays
// starting from (a).  With an odd number of 8-bit passes the sorted result
// lands in (b), with an even number back in (a): sort_result_in_b() tells.
constexpr int SORT_DIGIT_BITS = 9;  // 44-bit tile|depth keys take 5 passes (8-bit digits would need 6)
inline int sort_num_passes(int end_bit) { return (end_bit + SORT_DIGIT_BITS - 1) / SORT_DIGIT_BITS; }
inline bool sort_result_in_b(int end_bit) { return (sort_num_passes(end_bit) & 1) != 0; }
int launch_sort_pairs_u64(int64_t n, uint64_t* keys_a, uint64_t* keys_b, uint32_t* vals_a, uint32_t* vals_b,
                          int end_bit, void* temp, hipStream_t stream);
int launch_sort_pairs_u32(int64_t n, uint32_t* keys_a, uint32_t* keys_b, uint32_t* vals_a, uint32_t* vals_b,
                          int end_bit, void* temp, hipStream_t stream);

// ---- tile render ----
struct RenderFwdArgs {
  int P, W, H;
  float fx, fy, cx, cy;
  const uint32_t* ranges;      // (T,2)
  const uint32_t* point_list;  // (R)
  const float *means2D, *rgb, *all_map, *conic_opacity;
  const uint8_t* compute_locally;
  const float* bg;
  int render_geo;
  float* final_T;
  uint32_t *n_contrib_px, *n_contrib2loss_px;
  float* out_color;
  int* out_observe;
  float *out_all_map, *out_plane_depth;
  int *n_render, *n_consider, *n_contrib_tile;
  const float* depths = nullptr;            // only read when out_max_weight_depth is given
  float* out_max_weight_depth = nullptr;    // optional (H*W)
  // optional device word: the kernel was launched before the host knew whether the per-tile lists would be
  // built by the kernels queued ahead of it; it does nothing if the word is 0
  const uint32_t* fits_word = nullptr;
  // optional (R): per sorted instance, which of the tile's sixteen 4x4 pixel blocks the Gaussian can touch (bit
  // 4 * wave + row), as found by the kernel's own list building; the backward blend reads it instead of testing
  // again
  uint16_t* block_hits = nullptr;
  // optional (P,4) 16-byte words: pack_blend_operands' records; the kernel then fetches a Gaussian's operands as
  // one 64-byte line instead of gathering them from means2D, conic_opacity, rgb, all_map (and depths)
  const float* packed = nullptr;
};
int launch_render_fwd(const RenderFwdArgs& a, hipStream_t stream);

struct RenderBwdArgs {
  int P, W, H;
  float fx, fy;
  const float* bg;
  const uint32_t *ranges, *point_list;
  const float *means2D, *conic_opacity, *rgb, *all_map, *all_map_pixels, *final_T;
  const uint32_t* n_contrib_px;
  const uint8_t* compute_locally;
  const float *dL_dpix, *dL_dout_all_map, *dL_dout_plane_depth;
  int render_geo;
  // Per-instance gradient records: instance_grads[e] (16 floats) for the instance with emission index e;
  // emission_sorted[k] = emission index of the instance at sorted position k; point_offsets = inclusive
  // prefix sum of tiles touched, i.e. Gaussian i owns emission indices [point_offsets[i-1], point_offsets[i]).
  const uint32_t* emission_sorted;
  const uint32_t* point_offsets;
  float* instance_grads;  // (R,16) scratch, fully written by the blend kernel
  const uint16_t* block_hits = nullptr;  // optional (R): left by the forward blend (RenderFwdArgs::block_hits)
  const float* packed = nullptr;         // optional (P,4) 16-byte words: see RenderFwdArgs::packed
  // optional device word beside `packed`: non-zero if the forward call did pack the records (it decides per view)
  const uint32_t* packed_valid = nullptr;
  // outputs, fully written by the per-Gaussian reduction
  float* dL_dmean2D;         // (P,2)
  float* dL_dmean2D_abs;     // (P,3)
  float* dL_dconic_opacity;  // (P,4) packed [x, y, w, opacity]
  float* dL_dcolors;         // (P,3)
  float* dL_dall_map;        // (P,5)
};
int launch_render_bwd(const RenderBwdArgs& a, hipStream_t stream);

int launch_reduce_selftest(const float* in, float* out_wave, float* out_rows, hipStream_t stream);

// ---- k-nearest-neighbour mean squared distance ----
size_t knn_temp_bytes(int P);
// fault_word (host-visible, optional): raised if the Morton sort's bounded wait ran out
int launch_knn_dist2(int P, const float* points, float* mean_dist2, void* temp, uint32_t* fault_word,
                     hipStream_t stream);

}  // namespace gs
