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
// place in the list is the number of hits in the lanes below it).  A pixel
// blends about a quarter of its block's list, so the lists are walked 32
// entries at a time in two steps: every lane marks, one bit per entry, the
// entries that can reach its own pixel (a fused quadratic form against a
// limit, eleven instructions an entry), then blends its marked entries in
// order, the k-th marked one in pass k, whichever entry that is for the other
// lanes; a chunk takes as many blend passes as its busiest pixel has marks.
// Pixels keep their own front-to-back order, which is all the blend needs.
// A row stops when its 16 pixels have saturated; a batch is not fetched once
// all have.  The rows' hits, 16 bits per sorted instance, are left for the
// backward pass.
// Registers decide how many waves a SIMD holds here (80 allow six), and a
// kernel that spills to scratch memory starts its waves much more slowly, so
// index arithmetic is kept from being hoisted across the blend loop.
//
// The per-pixel arithmetic keeps a fixed operation order, so contributor
// counts and images match a CPU evaluation bit for bit; exp() is gs_expf.
// out_observe increments are counted per lane in LDS, two 16-bit counts a
// word, and added once per (tile, Gaussian).
#include <type_traits>

#include "gs_common.h"
#include "gs_kernels.h"
#include "render_common.h"

namespace gs {

namespace {

constexpr int BATCH = GS_TILE_PIX;
constexpr int CHUNK = 32;  // entries of a list marked, then blended, at a time: one bit each in a register

// The exponent of a Gaussian at offset (dx, dy) from its centre (cuda_rasterizer/forward.cu:366).
__device__ __forceinline__ float gauss_power(const float4 co, const float dx, const float dy) {
  return -0.5f * (co.x * dx * dx + co.z * dy * dy) - co.y * dx * dy;
}

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
__global__ void __launch_bounds__(GS_TILE_PIX) __attribute__((amdgpu_waves_per_eu(MAX_DEPTH ? 5 : 6)))
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
                  uint16_t* __restrict__ block_hits, const float4* __restrict__ packed) {
  constexpr bool render_geo = RENDER_GEO;
  // launched ahead of the host's decision on how the per-tile lists are built: nothing to do if they were not
  if (fits_word != nullptr && *fits_word == 0u) return;
  __shared__ float s_depth[MAX_DEPTH ? BATCH : 1];
  // a slot's geometry, (x, y, A, B) and (C, mark limit, opacity, exponent floor), and its channels, (r, g, b, map0)
  // and (map1 .. map4), in four arrays of 16-byte elements: one address per slot serves them all, and lanes
  // that read different slots spread over all the banks
  __shared__ float4 s_geo0[BATCH];
  __shared__ float4 s_geo1[BATCH];
  __shared__ float4 s_col0[BATCH];
  __shared__ float4 s_col1[RENDER_GEO ? BATCH : 1];
  // block_test_params
  __shared__ float4 s_cull[BATCH];
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
      // A Gaussian's operands: one 64-byte record where the caller had them packed (a single line of memory,
      // every byte of it used), else gathered from the five arrays.  (Each route loads and then stages by itself:
      // with the loaded values merged across the two routes the compiler splits the gathers into single words.)
      auto stage = [&](const float2 xy, const float4 co, const float c0, const float c1, const float c2,
                       const float (&m)[GS_N_MAP], const float depth_g) {
        // (the marking step evaluates the quadratic form with fused operations, the blend the exponent with one
        // rounding per operation: the mark limit's margin covers both, and the blend tests the exponent itself
        // again)
        float pfl, mark_limit;
        s_cull[ts] = block_test_params(co, xy, (float)(blockIdx.x * GS_TILE_X), (float)(blockIdx.y * GS_TILE_Y), pfl,
                                       mark_limit);
        s_geo0[ts] = make_float4(xy.x, xy.y, co.x, co.y);
        s_geo1[ts] = make_float4(co.z, mark_limit, co.w, pfl);
        float mag = fmaxf(fmaxf(fabsf(c0), fabsf(c1)), fabsf(c2));
        bool fin = c0 == c0 && c1 == c1 && c2 == c2;
        if (render_geo) {
#pragma unroll
          for (int ch = 0; ch < GS_N_MAP; ch++) {
            mag = fmaxf(mag, fabsf(m[ch]));
            fin = fin && m[ch] == m[ch];
          }
        }
        s_col0[ts] = make_float4(c0, c1, c2, m[0]);
        if constexpr (RENDER_GEO) s_col1[ts] = make_float4(m[1], m[2], m[3], m[4]);
        if (MAX_DEPTH) s_depth[ts] = depth_g;
        return fin && mag < __builtin_inff();
      };
      if (packed != nullptr) {
        const float4* rec = packed + 4 * (size_t)g;
        const float4 r0 = rec[0], r1 = rec[1], r2 = rec[2];
        float m[GS_N_MAP] = {r2.y, r2.z, r2.w, 0.f, 0.f};
        float depth_g = 0.f;
        if (render_geo || MAX_DEPTH) {
          const float4 r3 = rec[3];
          m[3] = r3.x, m[4] = r3.y, depth_g = r3.z;
        }
        finite = stage(make_float2(r0.x, r0.y), make_float4(r0.z, r0.w, r1.x, r1.y), r1.z, r1.w, r2.x, m, depth_g);
      } else {
        const float2 xy = means2D[g];
        const float4 co = conic_opacity[g];
        const float c0 = rgb[3 * (size_t)g], c1 = rgb[3 * (size_t)g + 1], c2 = rgb[3 * (size_t)g + 2];
        float m[GS_N_MAP] = {0.f, 0.f, 0.f, 0.f, 0.f};
        if (render_geo) {
#pragma unroll
          for (int ch = 0; ch < GS_N_MAP; ch++) m[ch] = all_map[5 * (size_t)g + ch];
        }
        finite = stage(xy, co, c0, c1, c2, m, MAX_DEPTH ? depths[g] : 0.f);
      }
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
        const int js = valid ? jj : 0;
        const float4 geo0 = s_geo0[js];
        const float2 mu = make_float2(geo0.x, geo0.y);
        const float4 cq = make_float4(geo0.z, geo0.w, s_geo1[js].x, 0.f);
        const float4 cu = s_cull[js];
        // (the four tests first, in one straight line and unconditionally, so that what they have in common is
        // computed once; masks of single comparisons, combined in scalar registers)
        uint64_t hit_m[4];
        bool hits[4];
        ellipse_hits_quadrant(mu, cq, cu.x, cu.y, cu.z, rt.qx0, rt.qy0, hits);
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
      // Of a 4x4 block's list a single pixel blends about a quarter, so the lists are walked a chunk of 32 entries
      // at a time, in two steps.  First every lane marks, one bit per entry, the entries whose exponent lies in
      // its window (the cheap part of a blend: centre, conic, two comparisons).  Then each lane blends its own
      // marked entries in order, the k-th marked one in pass k, whichever entry that is for its neighbours: a
      // chunk takes as many passes as its busiest pixel has marks.  A pixel's entries keep their order, which is
      // all the blend needs.
      float done = __builtin_amdgcn_inverse_ballot_w64(alive) ? 0.f : 1.f;  // 1: this pixel has saturated (or lies outside)
      const uint8_t* const my_list = reinterpret_cast<const uint8_t*>(&s_idx[wave][row][0]);
      for (uint32_t base = 0; base < passes; base += CHUNK) {
        uint32_t marks = 0u;
        const uint32_t words = min((uint32_t)CHUNK / 4u, (passes - base + 3u) / 4u);
        // (last entry first: a mark is shifted in at bit 0, as the carry of marks + marks, so entry e of the chunk
        // ends at bit e)
        for (int q = (int)words - 1; q >= 0; q--) {
          const uint32_t word = s_idx[wave][row][(base >> 2) + (uint32_t)q];  // (zero, slot 0, behind the list's end)
#pragma unroll
          for (int u = 3; u >= 0; u--) {
            const int j = (int)__builtin_amdgcn_ubfe(word, 8u * u, 8u);
            const float4 g0 = s_geo0[j];
            const float2 g1 = *reinterpret_cast<const float2*>(&s_geo1[j]);  // C and the mark limit
            const float dx = g0.x - pfx, dy = g0.y - pfy;
            const float form = __builtin_fmaf(g1.x * dy, dy, __builtin_fmaf(g0.z, dx, g0.w * (dy + dy)) * dx);
            // marked unless the form exceeds the limit (so a NaN marks, as the blend's own tests let it through)
            asm("v_cmp_ngt_f32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc"
                : "+v"(marks)
                : "v"(form), "v"(g1.y)
                : "vcc");
          }
        }
        {
          const uint32_t mine = my_len > base ? my_len - base : 0u;  // entries of the chunk that are in the list
          marks = mine >= (uint32_t)CHUNK ? marks : (marks & ((1u << mine) - 1u));
          marks = (done != 0.f) ? 0u : marks;
        }
        // (the slot of a lane's next marked entry is fetched one pass ahead)
        uint32_t slot_next = my_list[base + ((uint32_t)__builtin_ctz(marks | 0x80000000u))];
        // (tested at the bottom: the ballot cannot be copied, so a loop tested at the top is not rotated and pays
        // a register copy per accumulator and pass)
        if (gs_ballot(marks != 0u) != 0ull) do {
          const bool active = marks != 0u;
          const int j = active ? (int)slot_next : 0;  // (slot 0's data are this batch's)
          marks &= marks - 1u;
          slot_next = my_list[base + ((uint32_t)__builtin_ctz(marks | 0x80000000u))];
          const float4 g0 = s_geo0[j], g1 = s_geo1[j];
          const float2 xy = make_float2(g0.x, g0.y);
          const float4 co = make_float4(g0.z, g0.w, g1.x, g1.z);
          const float floor_j = g1.w;
          float c[GS_N_RGB + GS_N_MAP] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          {
            const float4 c0 = s_col0[j];
            c[0] = c0.x, c[1] = c0.y, c[2] = c0.z, c[3] = c0.w;
            if constexpr (RENDER_GEO) {
              const float4 c1 = s_col1[j];
              c[4] = c1.x, c[5] = c1.y, c[6] = c1.z, c[7] = c1.w;
            }
          }
          float depth_j = 0.f;
          if (MAX_DEPTH) depth_j = s_depth[j];

          const float power = gauss_power(co, xy.x - pfx, xy.y - pfy);
          const float alpha = fminf(0.99f, co.w * gs_expf_core(power));
          // alpha as far as this lane is concerned: 0 unless it has an entry in this pass and the exponent lies
          // in the window
          float a = alpha;
          a = (power > 0.0f) ? 0.f : a;
          a = (power < floor_j) ? 0.f : a;
          a = active ? a : 0.f;
          a = (a < 1.0f / 255.0f) ? 0.f : a;            // (NaN stays: the reference blends it too)
          const bool counts = a != 0.f;                  // alpha >= 1/255 and everything above
          const float test_T = T * (1 - alpha);          // (of use where the entry counts: a == alpha there)
          const bool stops = counts && test_T < 0.0001f;
          const bool blend = counts && !stops;
          // weight once, then one fused multiply-add per channel; w == 0 where the entry does not blend
          const float w = blend ? alpha * T : 0.f;
          done = stops ? 1.f : done;
          marks = stops ? 0u : marks;
          n2l += blend ? 1u : 0u;
#pragma unroll
          for (int ch = 0; ch < GS_N_RGB; ch++) {
            const float sum = __builtin_fmaf(c[ch], w, C[ch]);
            C[ch] = (!SELECT || blend) ? sum : C[ch];
          }
          if (render_geo) {
#pragma unroll
            for (int ch = 0; ch < GS_N_MAP; ch++) {
              const float sum = __builtin_fmaf(c[GS_N_RGB + ch], w, Mp[ch]);
              Mp[ch] = (!SELECT || blend) ? sum : Mp[ch];
            }
          }
          if (MAX_DEPTH) {
            const bool better = w > best_w;  // w is 0 for a lane that does not blend
            best_depth = better ? depth_j : best_depth;
            best_w = better ? w : best_w;
          }
          // observation count of the entry: one for a lane that blends it with T > 0.5
          if (blend && T > 0.5f) atomicAdd(&s_obs[j >> 1], 1u << (16 * (j & 1)));
          T = blend ? test_T : T;
          last = blend ? (uint32_t)(i * BATCH + j + 1) : last;
        } while (gs_ballot(marks != 0u) != 0ull);
        // a row whose 16 pixels have all saturated drops the rest of its list
        alive = gs_ballot(done == 0.f);
        if (((uint32_t)(alive >> row_shift) & 0xFFFFu) == 0u) my_len = 0u;
        uint32_t left = 0u;
        if (((uint32_t)alive & 0xFFFFu) != 0u) left = len0;
        if (((uint32_t)(alive >> 16) & 0xFFFFu) != 0u) left = max(left, len1);
        if (((uint32_t)(alive >> 32) & 0xFFFFu) != 0u) left = max(left, len2);
        if (((uint32_t)(alive >> 48) & 0xFFFFu) != 0u) left = max(left, len3);
        passes = left;
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
                     a.n_consider, a.n_contrib_tile, a.depths, a.out_max_weight_depth, a.fits_word, a.block_hits,
                     (const float4*)a.packed);
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
