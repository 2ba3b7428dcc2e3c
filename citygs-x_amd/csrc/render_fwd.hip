// Per-tile front-to-back alpha blending (cuda_rasterizer/forward.cu:264-437)
// with the per-tile statistics of cuda_rasterizer/rasterizer_impl.cu:219-262
// folded into the same kernel.
//
// One 256-thread workgroup per 16x16 tile; each 64-lane wave owns an 8x8
// quadrant and each 16-lane row of a wave a 4x4 pixel block.  The tile's
// depth-sorted Gaussians are staged through LDS in batches of 256 (index,
// centre, conic+opacity, colour, the five geometry channels, the culling
// parameters and the exponent below which alpha < 1/255 is certain).
// Per batch a wave tests, for each of its four rows, which Gaussians' alpha >= 1/255
// ellipses (slightly inflated) can reach the row's 4x4 block, and compacts the
// slot numbers of those that can into a byte list per row in LDS (a lane's
// place in the list is the number of hits in the lanes below it); the four rows
// then walk their own lists concurrently, entry n of each in pass n,
// so one pass of the loop blends up to four different Gaussians and a
// Gaussian that cannot touch a block costs that row nothing.  Pixels keep
// their own front-to-back order, which is all the blend needs.  A row stops
// when its 16 pixels have saturated; a batch is not fetched once all have.
// The same hits, 16 bits per sorted instance, are left for the backward pass.
// Registers decide how many waves a SIMD holds here (72 allow seven), and a
// kernel that spills to scratch memory starts its waves much more slowly, so
// index arithmetic is kept from being hoisted across the blend loop.
//
// The per-pixel arithmetic keeps a fixed operation order, so contributor
// counts and images match a CPU evaluation bit for bit; exp() is gs_expf.
// out_observe increments are counted per row with a ballot, summed per
// workgroup in LDS and added once per (tile, Gaussian).
#include <type_traits>

#include "gs_common.h"
#include "gs_kernels.h"
#include "render_common.h"

namespace gs {

namespace {

constexpr int BATCH = GS_TILE_PIX;

// The value itself, but opaque to the optimizer from here on: what is computed from it stays behind this point
// instead of being hoisted out of the batch loop, where every hoisted LDS address holds a register through the
// blend loop (the kernel has none to spare: one more costs a wave per SIMD, or scratch memory).
__device__ __forceinline__ int not_hoisted(int x) {
  asm volatile("" : "+v"(x));
  return x;
}

// MAX_DEPTH adds one output with no counterpart in the reference: per pixel, the view-space depth of the Gaussian
// that blends with the largest weight alpha * T (the front-most one among equals; 0 where nothing blends).  It
// leaves every other output as it is.
template <bool RENDER_GEO, bool MAX_DEPTH>
__global__ void __launch_bounds__(GS_TILE_PIX) __attribute__((amdgpu_waves_per_eu(7)))
render_fwd_kernel(const uint2* __restrict__ ranges, const uint32_t* __restrict__ point_list, int W, int H, float fx,
                  float fy, float cx, float cy, const float2* __restrict__ means2D, const float* __restrict__ rgb,
                  const float* __restrict__ all_map, const float4* __restrict__ conic_opacity,
                  const uint8_t* __restrict__ compute_locally, const float* __restrict__ bg,
                  float* __restrict__ final_T, uint32_t* __restrict__ n_contrib_px,
                  uint32_t* __restrict__ n_contrib2loss_px, float* __restrict__ out_color,
                  int* __restrict__ out_observe, float* __restrict__ out_all_map,
                  float* __restrict__ out_plane_depth, int* __restrict__ n_render, int* __restrict__ n_consider,
                  int* __restrict__ n_contrib_tile, const float* __restrict__ depths,
                  float* __restrict__ out_max_weight_depth, const uint32_t* __restrict__ fits_word,
                  uint16_t* __restrict__ block_hits) {
  constexpr bool render_geo = RENDER_GEO;
  // launched ahead of the host's decision on how the per-tile lists are built: nothing to do if they were not
  if (fits_word != nullptr && *fits_word == 0u) return;
  __shared__ float s_depth[MAX_DEPTH ? BATCH : 1];
  __shared__ float2 s_xy[BATCH];
  __shared__ float4 s_co[BATCH];
  __shared__ float2 s_cull[BATCH];  // packed_cull_params
  __shared__ float s_floor[BATCH];
  __shared__ float s_rgb[GS_N_RGB][BATCH];
  __shared__ float s_map[GS_N_MAP][BATCH];
  // observation counts of slots 2w and 2w + 1 in the low and high half of word w (a count is at most 256)
  __shared__ uint32_t s_obs[BATCH / 2];
  // the four rows' lists of every wave: the slots of the batch that can touch the row's block, one byte each, in
  // depth order; bytes behind a list's end are 0
  __shared__ __attribute__((aligned(16))) uint32_t s_idx[GS_TILE_PIX / GS_WAVE][4][BATCH / 4];
  // what the backward pass is left: byte `wave` of word p holds that wave's four row bits for slot 2p (low
  // half) and slot 2p + 1 (high half)
  __shared__ uint32_t s_hits[BATCH / 2];
  __shared__ int s_done[GS_TILE_PIX / GS_WAVE];
  __shared__ int s_bad[GS_TILE_PIX / GS_WAVE];
  __shared__ int s_red[2][GS_TILE_PIX / GS_WAVE];

  const int tid = threadIdx.x;
  const RowThread rt = row_thread(blockIdx.x, blockIdx.y);
  const int lane = rt.lane, wave = rt.wave, row = rt.row;
  const uint32_t tile = blockIdx.y * gridDim.x + blockIdx.x;
  const uint2 range = ranges[tile];
  if (tid == 0) n_render[tile] = (int)(range.y - range.x);
  const uint32_t px = rt.px, py = rt.py;
  const bool inside = px < (uint32_t)W && py < (uint32_t)H;
  const size_t pid = (size_t)W * py + px;
  if (!compute_locally[tile]) {
    // A tile that is not computed here reads zero in every image, as in the reference, whose binding
    // allocates the images zero-filled (rasterize_points.cu:303-307) and whose kernel returns before writing.
    if (inside) {
      const size_t HW = (size_t)H * W;
#pragma unroll
      for (int ch = 0; ch < GS_N_RGB; ch++) out_color[ch * HW + pid] = 0.f;
      if (render_geo) {
#pragma unroll
        for (int ch = 0; ch < GS_N_MAP; ch++) out_all_map[ch * HW + pid] = 0.f;
        out_plane_depth[pid] = 0.f;
      }
      if (MAX_DEPTH) out_max_weight_depth[pid] = 0.f;
    }
    if (tid == 0) {
      n_consider[tile] = 0;
      n_contrib_tile[tile] = 0;
    }
    return;
  }
  const float pfx = (float)px, pfy = (float)py;
  const float rayx = (pfx - cx) / fx, rayy = (pfy - cy) / fy;
  // pixels that still blend, as a lane mask (wave-uniform, so it lives in scalar registers)
  uint64_t alive = gs_ballot(inside);
  const int row_shift = 16 * row;

  int todo = (int)(range.y - range.x);
  const int rounds = (todo + BATCH - 1) / BATCH;

  float T = 1.0f;
  uint32_t last = 0, n2l = 0;
  float C[GS_N_RGB] = {0.f, 0.f, 0.f};
  float Mp[GS_N_MAP] = {0.f, 0.f, 0.f, 0.f, 0.f};
  float best_w = 0.f, best_depth = 0.f;

  for (int i = 0; i < rounds; i++, todo -= BATCH) {
    const uint64_t alive_mask = alive;
    if (lane == 0) s_done[wave] = alive_mask == 0ull;
    __syncthreads();
    if (s_done[0] && s_done[1] && s_done[2] && s_done[3]) break;

    const int count = todo < BATCH ? todo : BATCH;
    // A lane for which a Gaussian does not count blends it with weight 0, which is exact as long as the
    // Gaussian's colour and geometry channels are finite; a batch that holds a non-finite one is walked by
    // the variant of the loop that selects instead (below).
    bool finite = true;
    const int ts = not_hoisted(tid);
    if (ts < count) {
      const uint32_t g = point_list[range.x + (uint32_t)i * BATCH + ts];
      const float2 xy = means2D[g];
      const float4 co = conic_opacity[g];
      float pfl;
      s_xy[ts] = xy;
      s_co[ts] = co;
      s_cull[ts] = pack_cull_params(cull_params(co, pfl));
      s_floor[ts] = pfl;
      const float c0 = rgb[3 * (size_t)g], c1 = rgb[3 * (size_t)g + 1], c2 = rgb[3 * (size_t)g + 2];
      s_rgb[0][ts] = c0;
      s_rgb[1][ts] = c1;
      s_rgb[2][ts] = c2;
      float mag = fmaxf(fmaxf(fabsf(c0), fabsf(c1)), fabsf(c2));
      finite = c0 == c0 && c1 == c1 && c2 == c2;
      if (render_geo) {
#pragma unroll
        for (int ch = 0; ch < GS_N_MAP; ch++) {
          const float v = all_map[5 * (size_t)g + ch];
          s_map[ch][ts] = v;
          mag = fmaxf(mag, fabsf(v));
          finite = finite && v == v;
        }
      }
      finite = finite && mag < __builtin_inff();
      if (MAX_DEPTH) s_depth[ts] = depths[g];
    }
    {
      const uint64_t bad_m = gs_ballot(!finite);
      if (lane == 0) s_bad[wave] = bad_m != 0ull;
    }
    if (ts < BATCH / 2) {
      s_obs[ts] = 0u;
      s_hits[ts] = 0u;
    }
    static_assert(sizeof(s_idx) == 16 * GS_TILE_PIX, "four words of the lists per thread");
    *reinterpret_cast<uint4*>(&s_idx[0][0][0] + 4 * ts) = make_uint4(0u, 0u, 0u, 0u);
    __syncthreads();
    const bool select_blend = (s_bad[0] | s_bad[1] | s_bad[2] | s_bad[3]) != 0;

    if (alive_mask != 0ull) {
      // Per-row lists.  A wave looks at 64 slots at a time, lane = slot: the lanes whose Gaussian can touch row
      // r's 4x4 block append their slot numbers to the row's list, in lane order (a lane's place is the number of
      // set bits below its own).
      uint32_t len0 = 0u, len1 = 0u, len2 = 0u, len3 = 0u;  // the lists' lengths (wave-uniform)
      const int tb = not_hoisted(tid);
      const int lane_b = tb & (GS_WAVE - 1), wave_b = tb / GS_WAVE;
#pragma unroll
      for (int k = 0; k < BATCH / GS_WAVE; k++) {
        if (k * GS_WAVE >= count) break;  // (the last batch of a list is rarely full)
        const int jj = k * GS_WAVE + lane_b;
        const bool valid = jj < count;
        const uint64_t valid_m = gs_ballot(valid);
        const float2 mu = s_xy[valid ? jj : 0];
        const float4 cq = s_co[valid ? jj : 0];
        const float4 cp = unpack_cull_params(s_cull[valid ? jj : 0], s_floor[valid ? jj : 0]);
        // (the four tests first, in one straight line and unconditionally, so that what they have in common is
        // computed once; masks of single comparisons, combined in scalar registers)
        uint64_t hit_m[4];
        bool hits[4];
        ellipse_hits_quadrant(mu, cq, cp, rt.qx0, rt.qy0, hits);
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const bool row_alive = ((alive_mask >> (16 * r)) & 0xFFFFull) != 0ull;
          hit_m[r] = (row_alive ? valid_m : 0ull) & gs_ballot(hits[r]);
        }
        uint32_t rows_hit = 0u;
        auto list_row = [&](auto row_tag, const uint32_t len) {
          constexpr int r = decltype(row_tag)::value;
          const uint64_t b = hit_m[r];
          const uint32_t below = __builtin_amdgcn_mbcnt_hi((uint32_t)(b >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)b, 0u));
          if (__builtin_amdgcn_inverse_ballot_w64(b)) {
            reinterpret_cast<uint8_t*>(&s_idx[0][0][0])[(uint32_t)((wave_b * 4 + r) * BATCH) + len + below] = (uint8_t)jj;
            rows_hit |= 1u << r;
          }
          return len + (uint32_t)__popcll(b);
        };
        len0 = list_row(std::integral_constant<int, 0>{}, len0);
        len1 = list_row(std::integral_constant<int, 1>{}, len1);
        len2 = list_row(std::integral_constant<int, 2>{}, len2);
        len3 = list_row(std::integral_constant<int, 3>{}, len3);
        if (block_hits != nullptr) {
          // an even lane stores its own four bits and its odd neighbour's: one byte, no other wave's
          const uint32_t neighbour = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)rows_hit, 0xB1, 0xF, 0xF, false);
          if ((lane_b & 1) == 0)
            reinterpret_cast<uint8_t*>(&s_hits[0])[(4 * (lane_b >> 1) + wave_b) + k * (4 * GS_WAVE / 2)] =
                (uint8_t)(rows_hit | (neighbour << 4));
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

      // SELECT: a lane that does not blend keeps its sums by a select instead of adding a product with weight 0
      // (0 * NaN and 0 * inf are NaN): the reference only lets a non-finite colour reach the pixels that blend
      // it (cuda_rasterizer/forward.cu:381-407).  Same bits for finite inputs.
      len0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)len0);
      len1 = (uint32_t)__builtin_amdgcn_readfirstlane((int)len1);
      len2 = (uint32_t)__builtin_amdgcn_readfirstlane((int)len2);
      len3 = (uint32_t)__builtin_amdgcn_readfirstlane((int)len3);
      const uint32_t row_len = row == 0 ? len0 : (row == 1 ? len1 : (row == 2 ? len2 : len3));
      auto walk = [&, len0, len1, len2, len3, row_len](auto select_tag) {
      constexpr bool SELECT = decltype(select_tag)::value;
      uint32_t my_len = row_len;
      uint32_t passes = max(max(len0, len1), max(len2, len3));  // wave-uniform
      uint32_t word = 0u;  // four entries of the list
      for (uint32_t n = 0; n < passes; n++) {
        if ((n & 3u) == 0u) word = s_idx[wave][row][n >> 2];
        const uint64_t has_m = gs_ballot(n < my_len);
        // (slot 0 behind the end of the list: its data are this batch's)
        const int j = (int)__builtin_amdgcn_ubfe(word, (n & 3u) * 8u, 8u);

        // Straight-line: every lane evaluates its row's Gaussian; a lane for which it does not count blends
        // with weight 0, which leaves its sums unchanged bit for bit (fma(c, 0, C) == C).  The tests are kept as
        // lane masks of single comparisons and combined in scalar registers.
        const float2 xy = s_xy[j];
        const float4 co = s_co[j];
        const float dx = xy.x - pfx, dy = xy.y - pfy;
        const float power = -0.5f * (co.x * dx * dx + co.z * dy * dy) - co.y * dx * dy;
        const float floor_j = s_floor[j];
        const uint64_t in_m = has_m & alive & gs_ballot(!(power > 0.0f)) & gs_ballot(!(power < floor_j));
        if (in_m == 0ull) continue;
        const float alpha = fminf(0.99f, co.w * gs_expf_core(power));
        const uint64_t pass_m = in_m & gs_ballot(!(alpha < 1.0f / 255.0f));
        const float test_T = T * (1 - alpha);
        const uint64_t stop_m = pass_m & gs_ballot(test_T < 0.0001f);
        const uint64_t bmask = pass_m & ~stop_m;
        if (bmask != 0ull) {
          const bool blend = __builtin_amdgcn_inverse_ballot_w64(bmask);
          n2l += blend ? 1u : 0u;
          // weight once, then one fused multiply-add per channel
          const float w = blend ? alpha * T : 0.f;
#pragma unroll
          for (int ch = 0; ch < GS_N_RGB; ch++) {
            const float sum = __builtin_fmaf(s_rgb[ch][j], w, C[ch]);
            C[ch] = (!SELECT || blend) ? sum : C[ch];
          }
          if (render_geo) {
#pragma unroll
            for (int ch = 0; ch < GS_N_MAP; ch++) {
              const float sum = __builtin_fmaf(s_map[ch][j], w, Mp[ch]);
              Mp[ch] = (!SELECT || blend) ? sum : Mp[ch];
            }
          }
          if (MAX_DEPTH) {
            const bool better = w > best_w;  // w is 0 for a lane that does not blend
            best_depth = better ? s_depth[j] : best_depth;
            best_w = better ? w : best_w;
          }
          const uint64_t omask = bmask & gs_ballot(T > 0.5f);
          if (omask != 0ull) {
            const uint32_t cnt = (uint32_t)__popc((uint32_t)(omask >> row_shift) & 0xFFFFu);
            if (rt.l16 == 0 && cnt != 0u) atomicAdd(&s_obs[j >> 1], cnt << (16 * (j & 1)));
          }
          T = blend ? test_T : T;
          last = blend ? (uint32_t)(i * BATCH + j + 1) : last;
        }
        if (stop_m != 0ull) {
          alive &= ~stop_m;
          // a row whose 16 pixels have all saturated drops the rest of its list
          if (((uint32_t)(alive >> row_shift) & 0xFFFFu) == 0u) my_len = 0u;
          passes = 0u;
          if (((uint32_t)alive & 0xFFFFu) != 0u) passes = len0;
          if (((uint32_t)(alive >> 16) & 0xFFFFu) != 0u) passes = max(passes, len1);
          if (((uint32_t)(alive >> 32) & 0xFFFFu) != 0u) passes = max(passes, len2);
          if (((uint32_t)(alive >> 48) & 0xFFFFu) != 0u) passes = max(passes, len3);
        }
      }
      };
      if (select_blend) walk(std::true_type{});
      else walk(std::false_type{});
    }
    __syncthreads();
    const int tf = not_hoisted(tid);
    if (tf < count) {
      const uint32_t c = (s_obs[tf >> 1] >> (16 * (tf & 1))) & 0xFFFFu;
      if (c != 0u) atomicAdd(&out_observe[point_list[range.x + (uint32_t)i * BATCH + tf]], (int)c);
      // for the backward pass: which of the tile's sixteen rows listed this slot (a row that had saturated has an
      // empty list, and nothing behind a row's last contributor is looked at there)
      if (block_hits != nullptr) {
        const uint32_t x = s_hits[tf >> 1] >> (4 * (tf & 1));
        block_hits[range.x + (uint32_t)i * BATCH + tf] =
            (uint16_t)((x & 0xFu) | ((x >> 4) & 0xF0u) | ((x >> 8) & 0xF00u) | ((x >> 12) & 0xF000u));
      }
    }
  }

  if (inside) {
    const size_t HW = (size_t)H * W;
    final_T[pid] = T;
    n_contrib_px[pid] = last;
    n_contrib2loss_px[pid] = n2l;
#pragma unroll
    for (int ch = 0; ch < GS_N_RGB; ch++) out_color[ch * HW + pid] = C[ch] + T * bg[ch];
    if (render_geo) {
#pragma unroll
      for (int ch = 0; ch < GS_N_MAP; ch++) out_all_map[ch * HW + pid] = Mp[ch];
      const float den_f = (Mp[0] * rayx + Mp[1] * rayy) + Mp[2];
      out_plane_depth[pid] = (float)((double)Mp[4] / -((double)den_f + 1.0e-8));
    }
    if (MAX_DEPTH) out_max_weight_depth[pid] = best_depth;
  }

  // per-tile integer sums of the two per-pixel counters
  int a = inside ? (int)last : 0, b = inside ? (int)n2l : 0;
#pragma unroll
  for (int d = GS_WAVE / 2; d >= 1; d >>= 1) {
    a += __shfl_xor(a, d, GS_WAVE);
    b += __shfl_xor(b, d, GS_WAVE);
  }
  __syncthreads();
  if (lane == 0) {
    s_red[0][wave] = a;
    s_red[1][wave] = b;
  }
  __syncthreads();
  if (tid == 0) {
    n_consider[tile] = s_red[0][0] + s_red[0][1] + s_red[0][2] + s_red[0][3];
    n_contrib_tile[tile] = s_red[1][0] + s_red[1][1] + s_red[1][2] + s_red[1][3];
  }
}

}  // namespace

template <bool GEO, bool MAXD>
static void launch_render_fwd_variant(const RenderFwdArgs& a, hipStream_t stream) {
  const dim3 grid((a.W + GS_TILE_X - 1) / GS_TILE_X, (a.H + GS_TILE_Y - 1) / GS_TILE_Y, 1);
  hipLaunchKernelGGL((render_fwd_kernel<GEO, MAXD>), grid, dim3(GS_TILE_PIX), 0, stream, (const uint2*)a.ranges,
                     a.point_list, a.W, a.H, a.fx, a.fy, a.cx, a.cy, (const float2*)a.means2D, a.rgb, a.all_map,
                     (const float4*)a.conic_opacity, a.compute_locally, a.bg, a.final_T, a.n_contrib_px,
                     a.n_contrib2loss_px, a.out_color, a.out_observe, a.out_all_map, a.out_plane_depth, a.n_render,
                     a.n_consider, a.n_contrib_tile, a.depths, a.out_max_weight_depth, a.fits_word, a.block_hits);
}

int launch_render_fwd(const RenderFwdArgs& a, hipStream_t stream) {
  const bool maxd = a.out_max_weight_depth != nullptr;
  if (a.render_geo) {
    if (maxd) launch_render_fwd_variant<true, true>(a, stream);
    else launch_render_fwd_variant<true, false>(a, stream);
  } else {
    if (maxd) launch_render_fwd_variant<false, true>(a, stream);
    else launch_render_fwd_variant<false, false>(a, stream);
  }
  return 0;
}

}  // namespace gs
