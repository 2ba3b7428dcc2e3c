// Densification statistics of one rendered view, the body of GaussianModel.training_statis
// (scene/gaussian_model.py:1181-1205, called per view at train_internal.py:376-392), without its chain of
// boolean-mask gathers and scatters.  With A anchors of k offsets each, V visible anchors, S selected neural
// Gaussians among the V*k candidates:
//   opacity_accum[a] += sum_j max(opacity[rank(a)*k + j], 0);  anchor_demon[a] += 1      for visible a
//   slot (a, j) is hit when a is visible, offset_selection_mask[i] is set at i = rank(a)*k + j, and
//   update_filter[r] is set at r = rank2(i);  then
//   offset_gradient_accum[a*k+j] += |grad[r, 0:2]|;  offset_denom[a*k+j] += 1
// where rank / rank2 count the set entries of anchor_visible_mask / offset_selection_mask before a / i:
// exactly what "x[mask] = y" enumerates.  Two exclusive scans of the masks give the ranks; one kernel with
// a thread per slot then does all four updates.
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

// IDX: 32-bit indices whenever every count fits (64-bit division per thread is what this kernel would
// otherwise spend most of its time on)
template <typename IDX>
__global__ void __launch_bounds__(GS_BLOCK_1D)
train_stats_kernel(IDX slots, int k, IDX Vk, IDX M, const uint8_t* __restrict__ visible,
                   const uint32_t* __restrict__ rank_visible, const uint8_t* __restrict__ selected,
                   const uint32_t* __restrict__ rank_selected, const uint8_t* __restrict__ update_filter,
                   const float* __restrict__ grad, int grad_stride, const float* __restrict__ opacity,
                   float* __restrict__ opacity_accum, float* __restrict__ anchor_demon,
                   float* __restrict__ grad_accum, float* __restrict__ denom) {
  const IDX s = (IDX)blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (s >= slots) return;
  const IDX a = s / (IDX)k;
  const int j = (int)(s - a * (IDX)k);
  if (!visible[a]) return;
  const IDX first = (IDX)rank_visible[a] * (IDX)k;  // the anchor's first candidate
  if (j == 0) {
    float sum = 0.f;
    for (int q = 0; q < k; q++) {
      if (first + q < Vk) {
        const float o = opacity[first + q];
        sum += o < 0.f ? 0.f : o;
      }
    }
    opacity_accum[a] += sum;
    anchor_demon[a] += 1.0f;
  }
  const IDX i = first + (IDX)j;
  if (i >= Vk || !selected[i]) return;
  const IDX r = rank_selected[i];
  if (r >= M || !update_filter[r]) return;
  const float gx = grad[(size_t)r * grad_stride], gy = grad[(size_t)r * grad_stride + 1];
  grad_accum[s] += sqrtf(gx * gx + gy * gy);
  denom[s] += 1.0f;
}

// The same for n_offsets <= 256, the case that matters: a workgroup owns whole anchors (256 / k of them), every
// thread fetches its own candidate's opacity, and the anchor's first thread adds the k values from LDS in
// candidate order, instead of walking k dependent global loads.
template <typename IDX>
__global__ void __launch_bounds__(GS_BLOCK_1D)
train_stats_anchor_kernel(IDX A, int k, int anchors_per_block, IDX Vk, IDX M, const uint8_t* __restrict__ visible,
                          const uint32_t* __restrict__ rank_visible, const uint8_t* __restrict__ selected,
                          const uint32_t* __restrict__ rank_selected, const uint8_t* __restrict__ update_filter,
                          const float* __restrict__ grad, int grad_stride, const float* __restrict__ opacity,
                          float* __restrict__ opacity_accum, float* __restrict__ anchor_demon,
                          float* __restrict__ grad_accum, float* __restrict__ denom) {
  __shared__ float s_op[GS_BLOCK_1D];
  const int local_a = (int)threadIdx.x / k;
  const int j = (int)threadIdx.x - local_a * k;
  const IDX a = (IDX)blockIdx.x * (IDX)anchors_per_block + (IDX)local_a;
  const bool live = local_a < anchors_per_block && a < A && visible[a];
  IDX i = 0;
  bool have = false;
  float o = 0.f;
  if (live) {
    i = (IDX)rank_visible[a] * (IDX)k + (IDX)j;
    have = i < Vk;
    if (have) {
      o = opacity[i];
      o = o < 0.f ? 0.f : o;
    }
  }
  s_op[threadIdx.x] = o;
  __syncthreads();
  if (!live) return;
  if (j == 0) {
    float sum = 0.f;
    for (int q = 0; q < k; q++) sum += s_op[threadIdx.x + q];
    opacity_accum[a] += sum;
    anchor_demon[a] += 1.0f;
  }
  if (!have || !selected[i]) return;
  const IDX r = rank_selected[i];
  if (r >= M || !update_filter[r]) return;
  const float gx = grad[(size_t)r * grad_stride], gy = grad[(size_t)r * grad_stride + 1];
  const size_t slot = (size_t)a * k + j;
  grad_accum[slot] += sqrtf(gx * gx + gy * gy);
  denom[slot] += 1.0f;
}

}  // namespace

size_t train_stats_temp_bytes(long long A, long long Vk) {
  return align_up((size_t)(A > 0 ? A : 1) * 4, 256) + align_up((size_t)(Vk > 0 ? Vk : 1) * 4, 256) +
         align_up(scan_temp_bytes(A > Vk ? A : Vk), 256);
}

// gaussians.max_radii2D[visibility_filter] = max(gaussians.max_radii2D[visibility_filter], radii[visibility_filter])
// (densification.py:71-73, add_densification_stats' companion in the Gaussian-splatting training loop).
namespace {
__global__ void __launch_bounds__(GS_BLOCK_1D)
max_radii_kernel(long long n, const int* __restrict__ radii, const uint8_t* __restrict__ visible,
                 float* __restrict__ max_radii) {
  const long long i = (long long)blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (i < n && visible[i]) max_radii[i] = fmaxf(max_radii[i], (float)radii[i]);
}
}  // namespace

int launch_max_radii(long long n, const int* radii, const uint8_t* visible, float* max_radii, hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(max_radii_kernel, dim3((unsigned)((n + GS_BLOCK_1D - 1) / GS_BLOCK_1D)), dim3(GS_BLOCK_1D), 0,
                     stream, n, radii, visible, max_radii);
  return 0;
}

int launch_train_stats(long long A, int k, long long Vk, long long M, const uint8_t* visible,
                       const uint8_t* selected, const uint8_t* update_filter, const float* grad, int grad_stride,
                       const float* opacity, float* opacity_accum, float* anchor_demon, float* grad_accum,
                       float* denom, void* temp, hipStream_t stream) {
  if (A <= 0 || k <= 0) return 0;
  char* base = (char*)temp;
  uint32_t* rank_visible = (uint32_t*)base;
  base += align_up((size_t)A * 4, 256);
  uint32_t* rank_selected = (uint32_t*)base;
  base += align_up((size_t)(Vk > 0 ? Vk : 1) * 4, 256);
  launch_exclusive_sum_u8(A, visible, rank_visible, base, stream);
  if (Vk > 0) launch_exclusive_sum_u8(Vk, selected, rank_selected, base, stream);
  const long long slots = A * k;
  if (k <= GS_BLOCK_1D && slots < 0x7FFFFFFFll && Vk < 0x7FFFFFFFll && M < 0x7FFFFFFFll) {
    const int apb = GS_BLOCK_1D / k;
    hipLaunchKernelGGL(train_stats_anchor_kernel<uint32_t>, dim3((unsigned)((A + apb - 1) / apb)), dim3(GS_BLOCK_1D), 0,
                       stream, (uint32_t)A, k, apb, (uint32_t)Vk, (uint32_t)M, visible, rank_visible, selected,
                       rank_selected, update_filter, grad, grad_stride, opacity, opacity_accum, anchor_demon,
                       grad_accum, denom);
    return 0;
  }
  const dim3 grid((unsigned)((slots + GS_BLOCK_1D - 1) / GS_BLOCK_1D));
  if (slots < 0x7FFFFFFFll - GS_BLOCK_1D && Vk < 0x7FFFFFFFll && M < 0x7FFFFFFFll)
    hipLaunchKernelGGL(train_stats_kernel<uint32_t>, grid, dim3(GS_BLOCK_1D), 0, stream, (uint32_t)slots, k,
                       (uint32_t)Vk, (uint32_t)M, visible, rank_visible, selected, rank_selected, update_filter, grad,
                       grad_stride, opacity, opacity_accum, anchor_demon, grad_accum, denom);
  else
    hipLaunchKernelGGL(train_stats_kernel<unsigned long long>, grid, dim3(GS_BLOCK_1D), 0, stream,
                       (unsigned long long)slots, k, (unsigned long long)Vk, (unsigned long long)M, visible,
                       rank_visible, selected, rank_selected, update_filter, grad, grad_stride, opacity, opacity_accum,
                       anchor_demon, grad_accum, denom);
  return 0;
}

}  // namespace gs
