// Mean squared distance to the three nearest neighbours of every point
// (simple-knn/simple_knn.cu:185-221, distCUDA2): global bounding box, a 30-bit
// key along a space-filling curve, stable sort by key, bounding boxes of runs
// of 1024 sorted points, then an exact search that visits only boxes closer
// than the current third-best distance.  The search is exhaustive within that
// bound, so the three distances equal a brute-force search whatever the order
// of the points and whatever the visiting order.  That leaves the curve free:
// the reference sorts by Morton code on a grid stretched to the bounding box
// (simple_knn.cu:54-76); here the key is the Hilbert index on a grid with
// cubic cells.  The Morton curve jumps (a run of consecutive points can lie in
// two far-apart places, and its bounding box then spans everything between
// them), the Hilbert curve does not, and runs along it are compact: a wave
// opens 38 instead of 68 sixteen-point runs per leaf on a 200 x 200 x 30 m
// slab of a million uniform points.
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

// (The reference reduces from 0, simple-knn/simple_knn.cu:191, which makes its grid include the origin; the keys
// here are only a means of ordering, so the grid is the points' own bounding box.)
__global__ void __launch_bounds__(MM_THREADS) minmax_partial_kernel(int P, const float* __restrict__ pts,
                                                                     float* __restrict__ partial) {
  __shared__ float s[6][MM_THREADS / GS_WAVE];
  float v[6] = {FLT_MAX, FLT_MAX, FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
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
  float v[6] = {FLT_MAX, FLT_MAX, FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
  for (int b = threadIdx.x; b < MM_BLOCKS; b += MM_THREADS) {
#pragma unroll
    for (int k = 0; k < 3; k++) {
      v[k] = fminf(v[k], partial[6 * b + k]);
      v[3 + k] = fmaxf(v[3 + k], partial[6 * b + 3 + k]);
    }
  }
  reduce6(v, s, minmax);
}

__device__ __forceinline__ uint32_t spread10(uint32_t x) {  // every bit of a 10-bit number to every third place
  x = (x | (x << 16)) & 0x030000FF;
  x = (x | (x << 8)) & 0x0300F00F;
  x = (x | (x << 4)) & 0x030C30C3;
  x = (x | (x << 2)) & 0x09249249;
  return x;
}

// Index of grid cell (x, y, z), 10 bits each, along the three-dimensional Hilbert curve (Skilling's transform:
// undo the curve's rotations and reflections level by level, Gray-code, interleave).  Consecutive indices are
// neighbouring cells.
__device__ __forceinline__ uint32_t hilbert30(uint32_t x, uint32_t y, uint32_t z) {
  uint32_t X[3] = {x, y, z};
#pragma unroll
  for (uint32_t Q = 1u << 9; Q > 1u; Q >>= 1) {
    const uint32_t low = Q - 1u;
#pragma unroll
    for (int i = 0; i < 3; i++) {
      if (X[i] & Q) {
        X[0] ^= low;
      } else {
        const uint32_t t = (X[0] ^ X[i]) & low;
        X[0] ^= t;
        X[i] ^= t;
      }
    }
  }
  X[1] ^= X[0];
  X[2] ^= X[1];
  uint32_t t = 0u;
#pragma unroll
  for (uint32_t Q = 1u << 9; Q > 1u; Q >>= 1)
    if (X[2] & Q) t ^= Q - 1u;
  return (spread10(X[0] ^ t) << 2) | (spread10(X[1] ^ t) << 1) | spread10(X[2] ^ t);
}

__global__ void __launch_bounds__(GS_BLOCK_1D) curve_key_kernel(int P, const float* __restrict__ pts,
                                                                const float* __restrict__ minmax,
                                                                uint32_t* __restrict__ codes, uint32_t* __restrict__ idx) {
  const int i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (i >= P) return;
  // cubic cells: the longest side of the bounding box takes the 1024 steps
  const float side = fmaxf(fmaxf(minmax[3] - minmax[0], minmax[4] - minmax[1]), minmax[5] - minmax[2]);
  uint32_t c[3];
#pragma unroll
  for (int k = 0; k < 3; k++)
    c[k] = min(f2u_sat(((pts[3 * (size_t)i + k] - minmax[k]) / side) * (float)((1 << 10) - 1)), (1u << 10) - 1u);
  codes[i] = hilbert30(c[0], c[1], c[2]);
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

// A node's bounding box: lo = minimum corner, hi = maximum corner.  An absent node is an inverted box, infinitely far
// from everything.
struct NodeBox {
  float lo[3], hi[3];
};

__device__ __forceinline__ NodeBox load_box(const float* __restrict__ bx, bool exists) {
  NodeBox n = {{FLT_MAX, FLT_MAX, FLT_MAX}, {-FLT_MAX, -FLT_MAX, -FLT_MAX}};
  if (exists) {
    const float2 a = *(const float2*)(bx), b = *(const float2*)(bx + 2), c = *(const float2*)(bx + 4);
    n.lo[0] = a.x; n.lo[1] = a.y; n.lo[2] = b.x;
    n.hi[0] = b.y; n.hi[1] = c.x; n.hi[2] = c.y;
  }
  return n;
}

// lane `from`'s box, in every lane (`from` is wave-uniform)
__device__ __forceinline__ NodeBox box_of_lane(const NodeBox& n, int from) {
  NodeBox r;
#pragma unroll
  for (int k = 0; k < 3; k++) {
    r.lo[k] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, n.lo[k]), from));
    r.hi[k] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, n.hi[k]), from));
  }
  return r;
}

// Squared distance between two axis-aligned boxes (0 where they overlap), and between a point and a box
// (simple_knn.cu:119-129 for the latter): lower bounds of the distance between any point of the one and any point
// of the other, also as rounded here and in update3 (differences, squares and the two additions are monotone, and
// the additions associate the same way).
__device__ __forceinline__ float boxes_dist2(const float* q, const NodeBox& n) {
  float gap[3];
#pragma unroll
  for (int k = 0; k < 3; k++) gap[k] = fmaxf(0.f, fmaxf(n.lo[k] - q[3 + k], q[k] - n.hi[k]));
  return (gap[0] * gap[0] + gap[1] * gap[1]) + gap[2] * gap[2];
}

__device__ __forceinline__ float point_box_dist2(const float4& p, const NodeBox& n) {
  const float pc[3] = {p.x, p.y, p.z};
  float gap[3];
#pragma unroll
  for (int k = 0; k < 3; k++) gap[k] = fmaxf(0.f, fmaxf(n.lo[k] - pc[k], pc[k] - n.hi[k]));
  return (gap[0] * gap[0] + gap[1] * gap[1]) + gap[2] * gap[2];
}

// Keeps the three smallest of {knn[0..2], dist(ref, p)} in ascending order (simple_knn.cu:131-145 inserts by
// compare-and-swap; minimum and medians leave the same three values).  A NaN distance (a point with a NaN
// coordinate) is never inserted, as with the reference's `knn[j] > dist`: the minimum with FLT_MAX turns it into a
// value that changes nothing.
__device__ __forceinline__ void update3(const float4& ref, const float4& p, float* knn, bool skip = false) {
  const float dx = p.x - ref.x, dy = p.y - ref.y, dz = p.z - ref.z;
  float dist = fminf((dx * dx + dy * dy) + dz * dz, FLT_MAX);
  dist = skip ? FLT_MAX : dist;
  const float n0 = fminf(knn[0], dist);
  const float n1 = __builtin_amdgcn_fmed3f(knn[0], knn[1], dist);
  const float n2 = __builtin_amdgcn_fmed3f(knn[1], knn[2], dist);
  knn[0] = n0;
  knn[1] = n1;
  knn[2] = n2;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int d = GS_WAVE / 2; d >= 1; d >>= 1) v = fmaxf(v, __shfl_xor(v, d, GS_WAVE));
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}

// simple-knn/simple_knn.cu:147-183.  The reference gives every point a thread that seeds a rejection radius from
// the point's neighbours in sorted order and then walks all boxes, skipping those farther away than that radius or
// than the third-best distance so far (simple_knn.cu:161-171).  Here a wave owns a leaf, 64 consecutive points
// along the curve, and walks the tree for all of them at once:
//   * every point first meets the points of its own leaf and of the two leaves next to it along the curve, which
//     gives it a third-best distance to start from;
//   * 64 nodes of a level (groups of boxes, boxes, 16-point twigs) are tested in one step, a lane each, against
//     the leaf's bounding box and the largest third-best distance of the wave; a box or twig that passes is then
//     tested by every lane for its own point and its own third-best distance, the reference's test, and opened
//     if any lane needs it (the first test alone would open everything between the two ends of a leaf whose
//     points lie in two places, where the curve leaves the occupied part of the grid and comes back elsewhere);
//   * the points of the twigs that are opened go to LDS 64 at a time and every lane measures its distance to each.
// A lane then also sees points that its own test would have skipped; only true distances are ever inserted, and
// nothing nearer than a point's third-best distance is ever skipped, so the three distances are those of a
// brute-force search whatever the order.
__global__ void __launch_bounds__(GS_BLOCK_1D) box_mean_dist_kernel(int P, const float4* __restrict__ sorted_pts,
                                                                    const uint32_t* __restrict__ idx,
                                                                    const float* __restrict__ boxes, int nboxes,
                                                                    const float* __restrict__ groups,
                                                                    const float* __restrict__ leaves,
                                                                    const float* __restrict__ twigs,
                                                                    float* __restrict__ out) {
  constexpr int TWIGS_PER_BOX = KNN_BOX / KNN_TWIG, TWIGS_PER_LEAF = KNN_LEAF / KNN_TWIG;
  constexpr int TWIGS_PER_STEP = GS_WAVE / KNN_TWIG;
  static_assert(TWIGS_PER_BOX == GS_WAVE && KNN_GROUP == GS_WAVE, "a lane tests one node of a level");
  __shared__ float4 s_pts[GS_BLOCK_1D / GS_WAVE][GS_WAVE];
  const int lane = threadIdx.x & (GS_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / GS_WAVE);
  const int own = blockIdx.x * (GS_BLOCK_1D / GS_WAVE) + wave;  // this wave's leaf
  if (own * KNN_LEAF >= P) return;                              // (whole waves only: no workgroup barrier below)
  const int k = own * KNN_LEAF + lane;
  const int n_own = min(KNN_LEAF, P - own * KNN_LEAF);
  // lanes past the last point keep step with a copy of it and store nothing
  const float4 p = sorted_pts[min(k, P - 1)];
  // a point with a non-finite coordinate has no finite distance to anything: its result never changes
  const bool searching = k < P && fabsf(p.x) < __builtin_inff() && fabsf(p.y) < __builtin_inff() &&
                         fabsf(p.z) < __builtin_inff();
  float best[3] = {FLT_MAX, FLT_MAX, FLT_MAX};
  float4* mine = s_pts[wave];
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  // The leaf itself and the leaves before and after it along the curve come first, unconditionally: they hold
  // most of the neighbours, and the third-best distance they leave is the bound for everything that follows
  // (the reference seeds its rejection radius from a point's neighbours in sorted order too,
  // simple_knn.cu:153-160).
  const int nleaves = (P + KNN_LEAF - 1) / KNN_LEAF;
#pragma unroll
  for (int side = -1; side <= 1; side++) {
    const int other = own + side;
    if (other < 0 || other >= nleaves) continue;  // wave-uniform
    const int at = other * KNN_LEAF + lane;
    // a slot without a point holds one that is infinitely far away
    mine[lane] = side == 0 ? p
                 : at < P  ? sorted_pts[at]
                           : make_float4(__builtin_inff(), __builtin_inff(), __builtin_inff(), 0.f);
    wave_sync();
    const int n = side == 0 ? n_own : KNN_LEAF;
    for (int i = 0; i < n; i++) update3(p, mine[i], best, side == 0 && i == lane);  // (not its own neighbour)
    wave_sync();
  }

  float q[6];  // the leaf's bounding box
#pragma unroll
  for (int c = 0; c < 6; c++) q[c] = leaves[6 * (size_t)own + c];
  // (a margin of a few units in the last place: the node test and the point distances round differently)
  constexpr float MARGIN = 1.0f + 0x1p-20f;
  float reach = wave_max(searching ? best[2] : 0.f) * MARGIN;

  const int own_box = own / (KNN_BOX / KNN_LEAF);
  // does any lane need a node, by the reference's test (simple_knn.cu:161-171) for its own point?
  auto needed = [&](const NodeBox& n) {
    const float d = point_box_dist2(p, n);
    return (gs_ballot(searching) & gs_ballot(!(d > best[2]))) != 0ull;
  };
  auto open_box = [&](int b) {
    const int t = b * TWIGS_PER_BOX + lane;
    const NodeBox mine_t = load_box(twigs + 6 * (size_t)t, (size_t)t * KNN_TWIG < (size_t)P);
    uint64_t near = gs_ballot(!(boxes_dist2(q, mine_t) > reach));
    // (the twigs of the three leaves met at the start are not met again)
    const int met = (own - 1) * TWIGS_PER_LEAF - b * TWIGS_PER_BOX;
    const int met_lo = max(met, 0), met_hi = min(met + 3 * TWIGS_PER_LEAF, TWIGS_PER_BOX);
    if (met_lo < met_hi) near &= ~(((1ull << (met_hi - met_lo)) - 1ull) << met_lo);
    uint64_t todo = 0ull;
    while (near != 0ull) {
      const int c = (int)__builtin_ctzll(near);
      near &= near - 1ull;
      if (needed(box_of_lane(mine_t, c))) todo |= 1ull << c;
    }
    while (todo != 0ull) {
      int tw[TWIGS_PER_STEP], n = 0;
#pragma unroll
      for (int e = 0; e < TWIGS_PER_STEP; e++) {
        tw[e] = -1;
        if (todo != 0ull) {
          tw[e] = (int)__builtin_ctzll(todo);
          todo &= todo - 1ull;
          n++;
        }
      }
      const int part = lane / KNN_TWIG;
      const int sel = part == 0 ? tw[0] : part == 1 ? tw[1] : part == 2 ? tw[2] : tw[3];
      const size_t at = ((size_t)b * TWIGS_PER_BOX + (size_t)max(sel, 0)) * KNN_TWIG + (size_t)(lane % KNN_TWIG);
      // a slot without a point holds one that is infinitely far away
      float4 cand = make_float4(__builtin_inff(), __builtin_inff(), __builtin_inff(), 0.f);
      if (sel >= 0 && at < (size_t)P) cand = sorted_pts[at];
      mine[lane] = cand;
      wave_sync();
      const int m = n * KNN_TWIG;
      for (int i = 0; i < m; i++) update3(p, mine[i], best);
      wave_sync();
    }
    reach = wave_max(searching ? best[2] : 0.f) * MARGIN;
  };

  open_box(own_box);
  const int ngroups = (nboxes + KNN_GROUP - 1) / KNN_GROUP;
  for (int g0 = 0; g0 < ngroups; g0 += GS_WAVE) {
    const int g = g0 + lane;
    uint64_t gm = gs_ballot(!(boxes_dist2(q, load_box(groups + 6 * (size_t)g, g < ngroups)) > reach));
    while (gm != 0ull) {
      const int gi = g0 + (int)__builtin_ctzll(gm);
      gm &= gm - 1ull;
      const int b = gi * KNN_GROUP + lane;
      const NodeBox mine_b = load_box(boxes + 6 * (size_t)b, b < nboxes);
      uint64_t bm = gs_ballot(!(boxes_dist2(q, mine_b) > reach));
      if (gi == own_box / KNN_GROUP) bm &= ~(1ull << (own_box % KNN_GROUP));
      while (bm != 0ull) {
        const int c = (int)__builtin_ctzll(bm);
        bm &= bm - 1ull;
        if (needed(box_of_lane(mine_b, c))) open_box(gi * KNN_GROUP + c);
      }
    }
  }
  if (k < P) out[idx[k]] = ((best[0] + best[1]) + best[2]) / 3.0f;
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
    StageScope _t("knn_keys", stream);
    hipLaunchKernelGGL(curve_key_kernel, dim3(blocks), dim3(GS_BLOCK_1D), 0, stream, P, points, minmax, codes_a, idx_a);
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
