// Mean squared distance to the three nearest neighbours of every point
// (simple-knn/simple_knn.cu:185-221, distCUDA2): global bounding box, 30-bit
// Morton codes, stable sort by code, bounding boxes of runs of 1024 sorted
// points, then an exact search that visits only boxes closer than the current
// third-best distance.  The search is exhaustive within that bound, so the
// three distances equal a brute-force search whatever the visiting order.
#include <float.h>

#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

constexpr int KNN_BOX = 1024;  // simple-knn/simple_knn.cu:12
constexpr int KNN_GROUP = 64;  // boxes per group (one group test replaces this many box tests)
constexpr int KNN_LEAF = 64;   // points per leaf box inside a box (one leaf test replaces this many distances)
constexpr int KNN_TWIG = 16;   // points per twig box inside a leaf (the finest level)
constexpr int MM_BLOCKS = 512;
constexpr int MM_THREADS = 256;

struct KnnLayout {
  size_t partial, minmax, codes_a, codes_b, idx_a, idx_b, sorted_pts, boxes, groups, leaves, twigs, sort_temp, total;
};

KnnLayout knn_layout(int P) {
  KnnLayout L;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    size_t o = off;
    off += align_up(bytes, 256);
    return o;
  };
  const size_t n = (size_t)(P > 0 ? P : 1);
  const size_t nb = (n + KNN_BOX - 1) / KNN_BOX;
  L.partial = take(sizeof(float) * 6 * MM_BLOCKS);
  L.minmax = take(sizeof(float) * 6);
  L.codes_a = take(sizeof(uint32_t) * n);
  L.codes_b = take(sizeof(uint32_t) * n);
  L.idx_a = take(sizeof(uint32_t) * n);
  L.idx_b = take(sizeof(uint32_t) * n);
  L.sorted_pts = take(sizeof(float4) * n);
  L.boxes = take(sizeof(float) * 6 * nb);
  L.leaves = take(sizeof(float) * 6 * ((n + KNN_LEAF - 1) / KNN_LEAF));
  L.twigs = take(sizeof(float) * 6 * ((n + KNN_TWIG - 1) / KNN_TWIG));
  L.groups = take(sizeof(float) * 6 * ((nb + KNN_GROUP - 1) / KNN_GROUP));
  L.sort_temp = take(sort_temp_bytes((int64_t)n));
  L.total = off;
  return L;
}

__device__ __forceinline__ void reduce6(float* v, float (*s)[MM_THREADS / GS_WAVE], float* out) {
  // v[0..2] min, v[3..5] max
#pragma unroll
  for (int d = GS_WAVE / 2; d >= 1; d >>= 1) {
#pragma unroll
    for (int k = 0; k < 3; k++) {
      v[k] = fminf(v[k], __shfl_xor(v[k], d, GS_WAVE));
      v[3 + k] = fmaxf(v[3 + k], __shfl_xor(v[3 + k], d, GS_WAVE));
    }
  }
  const int lane = threadIdx.x & (GS_WAVE - 1), wave = threadIdx.x / GS_WAVE;
  if (lane == 0) {
#pragma unroll
    for (int k = 0; k < 6; k++) s[k][wave] = v[k];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int k = 0; k < 3; k++) {
      float mn = s[k][0], mx = s[3 + k][0];
      for (int w = 1; w < MM_THREADS / GS_WAVE; w++) {
        mn = fminf(mn, s[k][w]);
        mx = fmaxf(mx, s[3 + k][w]);
      }
      out[k] = mn;
      out[3 + k] = mx;
    }
  }
}

// Reduction identity is 0 for both min and max (simple-knn/simple_knn.cu:191).
__global__ void __launch_bounds__(MM_THREADS) minmax_partial_kernel(int P, const float* __restrict__ pts,
                                                                     float* __restrict__ partial) {
  __shared__ float s[6][MM_THREADS / GS_WAVE];
  float v[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int i = blockIdx.x * MM_THREADS + threadIdx.x; i < P; i += MM_BLOCKS * MM_THREADS) {
#pragma unroll
    for (int k = 0; k < 3; k++) {
      const float c = pts[3 * (size_t)i + k];
      v[k] = fminf(v[k], c);
      v[3 + k] = fmaxf(v[3 + k], c);
    }
  }
  reduce6(v, s, partial + 6 * blockIdx.x);
}

__global__ void __launch_bounds__(MM_THREADS) minmax_final_kernel(const float* __restrict__ partial,
                                                                   float* __restrict__ minmax) {
  __shared__ float s[6][MM_THREADS / GS_WAVE];
  float v[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int b = threadIdx.x; b < MM_BLOCKS; b += MM_THREADS) {
#pragma unroll
    for (int k = 0; k < 3; k++) {
      v[k] = fminf(v[k], partial[6 * b + k]);
      v[3 + k] = fmaxf(v[3 + k], partial[6 * b + 3 + k]);
    }
  }
  reduce6(v, s, minmax);
}

__device__ __forceinline__ uint32_t spread10(uint32_t x) {  // simple-knn/simple_knn.cu:45-52
  x = (x | (x << 16)) & 0x030000FF;
  x = (x | (x << 8)) & 0x0300F00F;
  x = (x | (x << 4)) & 0x030C30C3;
  x = (x | (x << 2)) & 0x09249249;
  return x;
}

__global__ void __launch_bounds__(GS_BLOCK_1D) morton_kernel(int P, const float* __restrict__ pts,
                                                             const float* __restrict__ minmax,
                                                             uint32_t* __restrict__ codes, uint32_t* __restrict__ idx) {
  const int i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (i >= P) return;
  uint32_t c[3];
#pragma unroll
  for (int k = 0; k < 3; k++) {
    const float mn = minmax[k], mx = minmax[3 + k];
    c[k] = spread10(f2u_sat(((pts[3 * (size_t)i + k] - mn) / (mx - mn)) * (float)((1 << 10) - 1)));
  }
  codes[i] = c[0] | (c[1] << 1) | (c[2] << 2);
  idx[i] = (uint32_t)i;
}

__global__ void __launch_bounds__(GS_BLOCK_1D) gather_points_kernel(int P, const float* __restrict__ pts,
                                                                    const uint32_t* __restrict__ idx,
                                                                    float4* __restrict__ sorted_pts) {
  const int i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (i >= P) return;
  const size_t g = idx[i];
  sorted_pts[i] = make_float4(pts[3 * g], pts[3 * g + 1], pts[3 * g + 2], 0.f);
}

// simple-knn/simple_knn.cu:78-117: one workgroup per run of 1024 sorted points.
__global__ void __launch_bounds__(MM_THREADS) box_minmax_kernel(int P, const float4* __restrict__ sorted_pts,
                                                                float* __restrict__ boxes) {
  __shared__ float s[6][MM_THREADS / GS_WAVE];
  float v[6] = {FLT_MAX, FLT_MAX, FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
  const int start = blockIdx.x * KNN_BOX;
  for (int t = threadIdx.x; t < KNN_BOX; t += MM_THREADS) {
    const int i = start + t;
    if (i < P) {
      const float4 p = sorted_pts[i];
      v[0] = fminf(v[0], p.x); v[1] = fminf(v[1], p.y); v[2] = fminf(v[2], p.z);
      v[3] = fmaxf(v[3], p.x); v[4] = fmaxf(v[4], p.y); v[5] = fmaxf(v[5], p.z);
    }
  }
  reduce6(v, s, boxes + 6 * blockIdx.x);
}

// Bounding box of every run of KNN_GROUP consecutive boxes: lets the search discard that many boxes with
// one test.  (Not in the reference, which tests every box for every point; the result is the same set of
// three nearest neighbours, because a group's box bounds its members' boxes from below.)
__global__ void __launch_bounds__(GS_WAVE) box_group_kernel(int nboxes, const float* __restrict__ boxes,
                                                            float* __restrict__ groups) {
  const int b = blockIdx.x * KNN_GROUP + threadIdx.x;
  float v[6] = {FLT_MAX, FLT_MAX, FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
  if (threadIdx.x < KNN_GROUP && b < nboxes) {
#pragma unroll
    for (int c = 0; c < 6; c++) v[c] = boxes[6 * b + c];
  }
#pragma unroll
  for (int d = GS_WAVE / 2; d >= 1; d >>= 1) {
#pragma unroll
    for (int c = 0; c < 3; c++) {
      v[c] = fminf(v[c], __shfl_xor(v[c], d, GS_WAVE));
      v[3 + c] = fmaxf(v[3 + c], __shfl_xor(v[3 + c], d, GS_WAVE));
    }
  }
  if (threadIdx.x == 0) {
#pragma unroll
    for (int c = 0; c < 6; c++) groups[6 * blockIdx.x + c] = v[c];
  }
}

// Bounding box of every run of KNN_LEAF consecutive sorted points (one wave each) and, inside it, of every run
// of KNN_TWIG points (a 16-lane row each): the two finest levels of the search.  Like the groups, additions that
// prune work without changing which neighbours are found.
__global__ void __launch_bounds__(GS_BLOCK_1D) leaf_minmax_kernel(int P, const float4* __restrict__ sorted_pts,
                                                                  float* __restrict__ leaves,
                                                                  float* __restrict__ twigs) {
  static_assert(KNN_LEAF == GS_WAVE && KNN_TWIG == 16, "a leaf is a wave, a twig a row of 16 lanes");
  const int i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  float v[6] = {FLT_MAX, FLT_MAX, FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
  if (i < P) {
    const float4 p = sorted_pts[i];
    v[0] = v[3] = p.x; v[1] = v[4] = p.y; v[2] = v[5] = p.z;
  }
#pragma unroll
  for (int d = 1; d < GS_WAVE; d <<= 1) {
#pragma unroll
    for (int c = 0; c < 3; c++) {
      v[c] = fminf(v[c], __shfl_xor(v[c], d, GS_WAVE));
      v[3 + c] = fmaxf(v[3 + c], __shfl_xor(v[3 + c], d, GS_WAVE));
    }
    if (d == KNN_TWIG / 2) {
      const int twig = i / KNN_TWIG;
      if ((threadIdx.x & (KNN_TWIG - 1)) == 0 && twig * KNN_TWIG < P) {
#pragma unroll
        for (int c = 0; c < 6; c++) twigs[6 * (size_t)twig + c] = v[c];
      }
    }
  }
  const int leaf = i / KNN_LEAF;
  if ((threadIdx.x & (GS_WAVE - 1)) == 0 && leaf * KNN_LEAF < P) {
#pragma unroll
    for (int c = 0; c < 6; c++) leaves[6 * (size_t)leaf + c] = v[c];
  }
}

__device__ __forceinline__ float box_dist2(const float4& p, const float* bx) {  // simple_knn.cu:119-129
  float diff[3] = {0.f, 0.f, 0.f};
  const float pc[3] = {p.x, p.y, p.z};
#pragma unroll
  for (int c = 0; c < 3; c++)
    if (pc[c] < bx[c] || pc[c] > bx[3 + c]) diff[c] = fminf(fabsf(pc[c] - bx[c]), fabsf(pc[c] - bx[3 + c]));
  return (diff[0] * diff[0] + diff[1] * diff[1]) + diff[2] * diff[2];
}

// Keeps the three smallest of {knn[0..2], dist(ref, p)} in ascending order (simple_knn.cu:131-145 inserts by
// compare-and-swap; the minimum / maximum form leaves the same three values).  A NaN distance (a point with a NaN
// coordinate) is never inserted, as with the reference's `knn[j] > dist`.
__device__ __forceinline__ void update3(const float4& ref, const float4& p, float* knn) {
  const float dx = p.x - ref.x, dy = p.y - ref.y, dz = p.z - ref.z;
  float dist = (dx * dx + dy * dy) + dz * dz;
  dist = dist == dist ? dist : FLT_MAX;
  const float a0 = fminf(knn[0], dist), r0 = fmaxf(knn[0], dist);
  const float a1 = fminf(knn[1], r0), r1 = fmaxf(knn[1], r0);
  knn[0] = a0;
  knn[1] = a1;
  knn[2] = fminf(knn[2], r1);
}

// simple-knn/simple_knn.cu:147-183.  The reference seeds a rejection radius from the three nearest of a point's six
// neighbours in Morton order and then walks all boxes, skipping those farther away than that radius or than the
// third-best distance so far.  Here a point first looks at the other points of its own 64-point leaf (its nearest
// neighbours in Morton order, and the same leaf for every lane of a wave), which makes the third-best distance a
// tight bound from the start, and then walks groups of boxes, boxes, leaves and 16-point twigs with the reference's test
// (simple_knn.cu:161-171) against that bound.  The search is exhaustive within a bound that only ever shrinks to a
// distance actually found, so the three distances are those of a brute-force search whatever the order.
__global__ void __launch_bounds__(GS_BLOCK_1D) box_mean_dist_kernel(int P, const float4* __restrict__ sorted_pts,
                                                                    const uint32_t* __restrict__ idx,
                                                                    const float* __restrict__ boxes, int nboxes,
                                                                    const float* __restrict__ groups,
                                                                    const float* __restrict__ leaves,
                                                                    const float* __restrict__ twigs,
                                                                    float* __restrict__ out) {
  const int k = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (k >= P) return;
  const float4 p = sorted_pts[k];
  float best[3] = {FLT_MAX, FLT_MAX, FLT_MAX};
  // The lanes of a wave are the points of one leaf, so they walk the tree together: a node is opened when any
  // lane is within its bound of it, which keeps the walk's control flow and the loads of nodes and points
  // wave-uniform.  A lane then also sees points that its own test would have skipped; update3 only ever inserts
  // true distances, so that changes nothing.
  const int own = __builtin_amdgcn_readfirstlane(k / KNN_LEAF);
  {
    const int l0 = own * KNN_LEAF, le = min(P, l0 + KNN_LEAF);
    for (int i = l0; i < le; i++) {
      // (the point itself would contribute distance 0)
      const float4 q = sorted_pts[i];
      float keep[3] = {best[0], best[1], best[2]};
      update3(p, q, best);
      if (i == k) {
        best[0] = keep[0];
        best[1] = keep[1];
        best[2] = keep[2];
      }
    }
  }
  const int ngroups = (nboxes + KNN_GROUP - 1) / KNN_GROUP;
  for (int gi = 0; gi < ngroups; gi++) {
    // a group that is too far away holds no box that is near enough
    const float gd = box_dist2(p, groups + 6 * gi);
    if (!__any(!(gd > best[2]))) continue;
    const int b_end = min(nboxes, (gi + 1) * KNN_GROUP);
    for (int b = gi * KNN_GROUP; b < b_end; b++) {
      const float dist = box_dist2(p, boxes + 6 * b);
      if (!__any(!(dist > best[2]))) continue;
      const int e = min(P, (b + 1) * KNN_BOX);
      for (int l0 = b * KNN_BOX; l0 < e; l0 += KNN_LEAF) {
        if (l0 / KNN_LEAF == own) continue;
        const float ld = box_dist2(p, leaves + 6 * (size_t)(l0 / KNN_LEAF));
        if (!__any(!(ld > best[2]))) continue;
        const int le = min(e, l0 + KNN_LEAF);
        for (int t0 = l0; t0 < le; t0 += KNN_TWIG) {
          const float td = box_dist2(p, twigs + 6 * (size_t)(t0 / KNN_TWIG));
          if (!__any(!(td > best[2]))) continue;
          const int te = min(le, t0 + KNN_TWIG);
          for (int i = t0; i < te; i++) update3(p, sorted_pts[i], best);
        }
      }
    }
  }
  out[idx[k]] = ((best[0] + best[1]) + best[2]) / 3.0f;
}

}  // namespace

size_t knn_temp_bytes(int P) { return knn_layout(P).total; }

int launch_knn_dist2(int P, const float* points, float* mean_dist2, void* temp, uint32_t* fault_word,
                     hipStream_t stream) {
  if (P <= 0) return 0;
  const KnnLayout L = knn_layout(P);
  char* base = (char*)temp;
  float* partial = (float*)(base + L.partial);
  float* minmax = (float*)(base + L.minmax);
  uint32_t* codes_a = (uint32_t*)(base + L.codes_a);
  uint32_t* codes_b = (uint32_t*)(base + L.codes_b);
  uint32_t* idx_a = (uint32_t*)(base + L.idx_a);
  uint32_t* idx_b = (uint32_t*)(base + L.idx_b);
  float4* sorted_pts = (float4*)(base + L.sorted_pts);
  float* boxes = (float*)(base + L.boxes);
  float* groups = (float*)(base + L.groups);
  float* leaves = (float*)(base + L.leaves);
  float* twigs = (float*)(base + L.twigs);
  void* sort_temp = base + L.sort_temp;
  const int blocks = (P + GS_BLOCK_1D - 1) / GS_BLOCK_1D;
  const int nboxes = (P + KNN_BOX - 1) / KNN_BOX;

  // (the per-phase scopes only record events while stage timing is enabled)
  {
    StageScope _t("knn_minmax", stream);
    hipLaunchKernelGGL(minmax_partial_kernel, dim3(MM_BLOCKS), dim3(MM_THREADS), 0, stream, P, points, partial);
    hipLaunchKernelGGL(minmax_final_kernel, dim3(1), dim3(MM_THREADS), 0, stream, partial, minmax);
  }
  {
    StageScope _t("knn_morton", stream);
    hipLaunchKernelGGL(morton_kernel, dim3(blocks), dim3(GS_BLOCK_1D), 0, stream, P, points, minmax, codes_a, idx_a);
  }
  const int end_bit = 32;  // 4 passes (even): the sorted pairs come back in the (a) arrays
  {
    StageScope _t("knn_sort", stream);
    if (launch_sort_pairs_u32(P, codes_a, codes_b, idx_a, idx_b, end_bit, sort_temp, stream)) return 1;
    launch_sort_fault_report(sort_error_word(sort_temp), fault_word, stream);
  }
  const uint32_t* idx_sorted = sort_result_in_b(end_bit) ? idx_b : idx_a;
  {
    StageScope _t("knn_gather", stream);
    hipLaunchKernelGGL(gather_points_kernel, dim3(blocks), dim3(GS_BLOCK_1D), 0, stream, P, points, idx_sorted,
                       sorted_pts);
  }
  {
    StageScope _t("knn_boxes", stream);
    hipLaunchKernelGGL(box_minmax_kernel, dim3(nboxes), dim3(MM_THREADS), 0, stream, P, sorted_pts, boxes);
    hipLaunchKernelGGL(leaf_minmax_kernel, dim3(blocks), dim3(GS_BLOCK_1D), 0, stream, P, sorted_pts, leaves, twigs);
    hipLaunchKernelGGL(box_group_kernel, dim3((nboxes + KNN_GROUP - 1) / KNN_GROUP), dim3(GS_WAVE), 0, stream, nboxes,
                       boxes, groups);
  }
  {
    StageScope _t("knn_box_mean_dist", stream);
    hipLaunchKernelGGL(box_mean_dist_kernel, dim3(blocks), dim3(GS_BLOCK_1D), 0, stream, P, sorted_pts, idx_sorted,
                       boxes, nboxes, groups, leaves, twigs, mean_dist2);
  }
  return 0;
}

}  // namespace gs
