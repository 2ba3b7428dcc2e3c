// Backward of the per-tile blend (cuda_rasterizer/backward.cu:324-567): each
// pixel replays its Gaussians back to front from the stored final
// transmittance and contributor count, and per-Gaussian gradients are summed
// over pixels.
//
// Workgroup = one 16x16 tile = four 64-lane waves; a wave owns an 8x8 quadrant
// and each of its 16-lane rows a 4x4 pixel block.  Gaussians are staged in LDS
// 128 at a time, in back-to-front order, and worked on 64 at a time:
//   * a wave ballots, for each of its rows, which of the 64 Gaussians can touch
//     the row's block (the forward kernel's own answer, 16 bits per instance,
//     when the caller hands them on; otherwise the inflated alpha >= 1/255
//     ellipse is tested against the block again) and lie in front of the
//     row's deepest contributor, and compacts their slot numbers into a byte
//     list per row; the four rows then walk their own lists concurrently
//     (entry n of each in pass n), so one pass of the loop handles up to four
//     Gaussians;
//   * the 16 partial sums of a Gaussian (mean2D x/y, |mean2D| x/y, conic
//     x/y/w, opacity, colour 3, map 5) are reduced over the row's 16 lanes by
//     a transposing DPP reduction (15 additions instead of 64) that leaves
//     component q in lane q; rows of the wave that are at the same Gaussian
//     are merged, and the sums go into the wave's own 16x64 accumulator in
//     LDS with a plain read-add-write (no atomics: an LDS float atomic costs
//     about three cycles per active lane here, and the kernel was bound by
//     them);
//   * then the four waves' accumulators are added in wave order and every
//     (tile, Gaussian) instance's 16 sums are stored as one 64-byte record, at
//     the instance's index in emission order (the order key emission wrote
//     them: all instances of a Gaussian are consecutive there).  No global
//     atomics either.
// A second kernel then sums, for every Gaussian, its consecutive records and
// writes the five gradient tensors: a streaming pass.  Every sum is taken in a
// fixed order, so the gradients are the same bits from run to run.  (The
// reference issues 16 global float atomics per pixel and Gaussian,
// cuda_rasterizer/backward.cu:510-563.)
// The per-pixel arithmetic follows the CPU statement's operation for operation
// (transmittance, reciprocal, weights, the derivative of the exponent), with
// three exceptions: the order in which pixels are summed; the factors that are
// constant per Gaussian (W/2, H/2, the opacity and -1/2 of the geometric
// gradients), which multiply the sums instead of every term; and the blend of
// everything behind a Gaussian, which the reference
// keeps per channel and this kernel keeps as its dot product with the upstream
// gradients (one recurrence instead of eight: see `behind_dot`).  Gradients
// therefore agree with a CPU evaluation to rounding (rel. L2 of the order of
// 1e-7 on the test scenes), not bit for bit.
#include <type_traits>

#include "gs_common.h"
#include "gs_kernels.h"
#include "render_common.h"

namespace gs {

namespace {

constexpr int BATCH = GS_TILE_PIX / 2;  // Gaussians staged in LDS per round
constexpr int SUB = GS_WAVE;        // Gaussians whose sums are in the accumulators at a time: one ballot's worth
constexpr int NV = 16;
constexpr int WAVES = GS_TILE_PIX / GS_WAVE;
static_assert(SUB * 4 == GS_TILE_PIX, "a thread hands over a quarter of one record of the sub-batch");

// HITS: the forward blend left, per sorted instance, which 4x4 blocks of the tile the Gaussian can touch; without
// it the same test is made again here.
template <bool RENDER_GEO, bool HITS>
__global__ void __launch_bounds__(GS_TILE_PIX) __attribute__((amdgpu_waves_per_eu(5)))
render_bwd_kernel(const uint2* __restrict__ ranges, const uint32_t* __restrict__ point_list, int W, int H, float fx,
                  float fy, const float* __restrict__ bg, const float2* __restrict__ means2D,
                  const float4* __restrict__ conic_opacity, const float* __restrict__ rgb,
                  const float* __restrict__ all_map, const float* __restrict__ all_map_pixels,
                  const float* __restrict__ final_Ts, const uint32_t* __restrict__ n_contrib_px,
                  const uint8_t* __restrict__ compute_locally, const float* __restrict__ dL_dpix,
                  const float* __restrict__ dL_dout_all_map, const float* __restrict__ dL_dout_plane_depth,
                  const uint32_t* __restrict__ emission_sorted, float4* __restrict__ instance_grads,
                  const uint16_t* __restrict__ block_hits, const float4* __restrict__ packed_records,
                  const uint32_t* __restrict__ packed_valid) {
  // (whether the forward call packed the records is its decision per view: a word beside them says)
  const float4* packed = (packed_records != nullptr && (packed_valid == nullptr || *packed_valid != 0u))
                             ? packed_records : nullptr;
  constexpr bool render_geo = RENDER_GEO;
  __shared__ uint32_t s_emis[BATCH];
  __shared__ float4 s_xyf[BATCH];  // centre x, y; the power floor; unused
  __shared__ float4 s_co[BATCH];
  __shared__ float4 s_cp[HITS ? 1 : BATCH];
  __shared__ uint16_t s_hits[HITS ? BATCH : 1];
  // colour, then the five geometry channels: eight floats per Gaussian, read as two 16-byte words
  __shared__ float4 s_chan[BATCH][RENDER_GEO ? 2 : 1];
  // one accumulator per wave; +1: the 16 components of one Gaussian fall in 16 different banks
  __shared__ float s_acc[WAVES][NV][SUB + 1];
  // the four rows' lists of every wave: the slots of the sub-batch that can touch the row's block and are not
  // behind its deepest contributor, one byte each, in walking order; bytes behind a list's end are 0
  __shared__ __attribute__((aligned(16))) uint32_t s_idx[GS_TILE_PIX / GS_WAVE][4][SUB / 4];
  __shared__ int s_max[GS_TILE_PIX / GS_WAVE];
  __shared__ int s_bad[GS_TILE_PIX / GS_WAVE];

  const int tid = threadIdx.x;
  const RowThread rt = row_thread(blockIdx.x, blockIdx.y);
  const int lane = rt.lane, wave = rt.wave, row = rt.row, l16 = rt.l16;
  const uint32_t tile = blockIdx.y * gridDim.x + blockIdx.x;
  const uint32_t px = rt.px, py = rt.py;
  const bool inside = px < (uint32_t)W && py < (uint32_t)H;
  const size_t pid = (size_t)W * py + px;
  const size_t HW = (size_t)H * W;
  const float pfx = (float)px, pfy = (float)py;
  const float rayx = (float)(((double)pfx - W * 0.5) / (double)fx);
  const float rayy = (float)(((double)pfy - H * 0.5) / (double)fy);
  const uint2 range = ranges[tile];
  const int total = (int)(range.y - range.x);
  if (!compute_locally[tile]) {
    // normally an empty range; if the forward pass binned this tile under a wider mask its records are zeros
    for (int p = tid; p < total; p += GS_TILE_PIX) {
      float4* rec = instance_grads + 4 * (size_t)emission_sorted[range.x + (uint32_t)p];
      const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
      rec[0] = z; rec[1] = z; rec[2] = z; rec[3] = z;
    }
    return;
  }

  const float T_final = inside ? final_Ts[pid] : 0.f;
  float T = T_final;
  const int last_contributor = inside ? (int)n_contrib_px[pid] : 0;

  // deepest contributor of each row, of this wave and of the whole tile: nothing behind it is ever touched
  int row_last = last_contributor;
#pragma unroll
  for (int d = 8; d >= 1; d >>= 1) row_last = max(row_last, __shfl_xor(row_last, d, GS_WAVE));
  int row_last_of[4];
#pragma unroll
  for (int r = 0; r < 4; r++) row_last_of[r] = __builtin_amdgcn_readlane(row_last, 16 * r);
  const int wave_last = max(max(row_last_of[0], row_last_of[1]), max(row_last_of[2], row_last_of[3]));
  if (lane == 0) s_max[wave] = wave_last;
  __syncthreads();
  const int tile_last = max(max(s_max[0], s_max[1]), max(s_max[2], s_max[3]));
  // Every instance record of the tile is written exactly once: the ones behind the deepest contributor
  // get zeros here, the others are written at the end of their batch.
  for (int p = tile_last + tid; p < total; p += GS_TILE_PIX) {
    float4* rec = instance_grads + 4 * (size_t)emission_sorted[range.x + (uint32_t)p];
    const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
    rec[0] = z; rec[1] = z; rec[2] = z; rec[3] = z;
  }
  if (tile_last == 0) return;

  float gpix[GS_N_RGB] = {0.f, 0.f, 0.f}, gmap[GS_N_MAP] = {0.f, 0.f, 0.f, 0.f, 0.f};
  if (inside) {
#pragma unroll
    for (int ch = 0; ch < GS_N_RGB; ch++) gpix[ch] = dL_dpix[ch * HW + pid];
    if (render_geo) {
#pragma unroll
      for (int ch = 0; ch < GS_N_MAP; ch++) gmap[ch] = dL_dout_all_map[ch * HW + pid];
      const float nx = all_map_pixels[pid], ny = all_map_pixels[HW + pid], nz = all_map_pixels[2 * HW + pid];
      const float dist = all_map_pixels[4 * HW + pid];
      const float tmp = (float)((double)((nx * rayx + ny * rayy) + nz) + 1.0e-8);
      const float gd = dL_dout_plane_depth[pid];
      gmap[GS_N_MAP - 1] += (-gd / tmp);
      gmap[0] += gd * (dist / (tmp * tmp) * rayx);
      gmap[1] += gd * (dist / (tmp * tmp) * rayy);
      gmap[2] += gd * (dist / (tmp * tmp));
    }
  }
  float bg_dot = 0.f;
#pragma unroll
  for (int ch = 0; ch < GS_N_RGB; ch++) bg_dot += bg[ch] * gpix[ch];

  const float bg_term = T_final * bg_dot;
  // dL/dalpha of a Gaussian needs sum_ch (c_ch - b_ch) g_ch, with b the blend of everything behind it and g the
  // upstream gradients of the eight channels.  The reference keeps b per channel (accum_rec,
  // cuda_rasterizer/backward.cu:463-472: b <- alpha c + (1 - alpha) b at every step); the sum is linear in b, so
  // here the pixel keeps the one number B = sum_ch b_ch g_ch instead, which obeys the same recurrence with
  // S = sum_ch c_ch g_ch in place of c: the term is S - B, and B <- alpha S + (1 - alpha) B.  Same value, eight
  // multiply-adds per step instead of forty operations; it is rounded differently (an error of the order of
  // eps |c| |g| per term where the per-channel form has eps |c - b| |g|), well inside the stated tolerance.
  float behind_dot = 0.f;

  // Positions are 0-based indices into the tile's list; the walk starts at the tile's deepest contributor.
  // Slot j of batch i holds position start - (i*BATCH + j).
  const int start = tile_last - 1;
  const int rounds = (start + 1 + BATCH - 1) / BATCH;

  // thread tid hands over components 4*part .. 4*part+3 of the sub-batch's slot tid / 4 and clears them
  const int my_slot = tid >> 2, my_part = tid & 3;
#pragma unroll
  for (int w = 0; w < WAVES; w++) {
#pragma unroll
    for (int e = 0; e < 4; e++) s_acc[w][4 * my_part + e][my_slot] = 0.f;
  }

  for (int i = 0; i < rounds; i++) {
    const int first_pos = start - i * BATCH;  // position in slot 0
    const int count = first_pos + 1 < BATCH ? first_pos + 1 : BATCH;
    // (the barrier that ends the previous batch's last sub-batch has let every wave finish with the staged data)
    // (a lane for which a Gaussian does not count takes part with alpha = 0, which is exact as long as the
    // Gaussian's colour and geometry channels are finite; a batch holding a non-finite one is walked by the
    // variant of the loop that leaves such a lane's recurrence state alone instead)
    bool finite = true;
    if (tid < count) {
      const uint32_t k_sorted = range.x + (uint32_t)(first_pos - tid);
      const uint32_t g = point_list[k_sorted];
      // A Gaussian's operands: one 64-byte record where the forward call packed them (a single line of memory,
      // every byte of it used), else gathered from the four arrays.  (Each route loads and then stages by itself:
      // with the loaded values merged across the two routes the compiler splits the gathers into single words.)
      auto stage = [&](const float2 xy, const float4 co, const float c0, const float c1, const float c2,
                       const float (&m)[GS_N_MAP]) {
        s_emis[tid] = emission_sorted[k_sorted];
        s_co[tid] = co;
        float pfl, mark_limit;
        const float4 cp = block_test_params(co, xy, (float)(blockIdx.x * GS_TILE_X), (float)(blockIdx.y * GS_TILE_Y),
                                            pfl, mark_limit);
        if (HITS) s_hits[tid] = block_hits[k_sorted];
        else s_cp[tid] = cp;
        s_xyf[tid] = make_float4(xy.x, xy.y, pfl, 0.f);
        float mag = fmaxf(fmaxf(fabsf(c0), fabsf(c1)), fabsf(c2));
        bool fin = c0 == c0 && c1 == c1 && c2 == c2;
        if (render_geo) {
#pragma unroll
          for (int ch = 0; ch < GS_N_MAP; ch++) {
            mag = fmaxf(mag, fabsf(m[ch]));
            fin = fin && m[ch] == m[ch];
          }
          s_chan[tid][RENDER_GEO ? 1 : 0] = make_float4(m[1], m[2], m[3], m[4]);
        }
        s_chan[tid][0] = make_float4(c0, c1, c2, m[0]);
        return fin && mag < __builtin_inff();
      };
      if (packed != nullptr) {
        const float4* rec = packed + 4 * (size_t)g;
        const float4 r0 = rec[0], r1 = rec[1], r2 = rec[2];
        float m[GS_N_MAP] = {r2.y, r2.z, r2.w, 0.f, 0.f};
        if (render_geo) {
          const float4 r3 = rec[3];
          m[3] = r3.x, m[4] = r3.y;
        }
        finite = stage(make_float2(r0.x, r0.y), make_float4(r0.z, r0.w, r1.x, r1.y), r1.z, r1.w, r2.x, m);
      } else {
        const float2 xy = means2D[g];
        const float4 co = conic_opacity[g];
        const float c0 = rgb[3 * (size_t)g], c1 = rgb[3 * (size_t)g + 1], c2 = rgb[3 * (size_t)g + 2];
        float m[GS_N_MAP] = {0.f, 0.f, 0.f, 0.f, 0.f};
        if (render_geo) {
#pragma unroll
          for (int ch = 0; ch < GS_N_MAP; ch++) m[ch] = all_map[5 * (size_t)g + ch];
        }
        finite = stage(xy, co, c0, c1, c2, m);
      }
    }
    {
      const uint64_t bad_m = gs_ballot(!finite);
      if (lane == 0) s_bad[wave] = bad_m != 0ull;
    }
    __syncthreads();
    const bool select_state = (s_bad[0] | s_bad[1] | s_bad[2] | s_bad[3]) != 0;

    for (int base = 0; base < count; base += SUB) {
      // Per-row lists: lane = slot of the sub-batch; the lanes whose Gaussian counts for row r append their slot
      // numbers to the row's list, in lane order (a lane's place is the number of set bits below its own).
      uint32_t len0, len1, len2, len3;  // the lists' lengths (wave-uniform)
      {
        static_assert(sizeof(s_idx[0]) == 4 * GS_WAVE, "a wave clears its own lists, one word per lane");
        (&s_idx[wave][0][0])[lane] = 0u;
        const int jj = base + lane;
        const bool valid = jj < count;
        const uint64_t valid_m = gs_ballot(valid);  // (masks of single comparisons, combined in scalar registers)
        float2 mu = make_float2(0.f, 0.f);
        float4 cq = make_float4(0.f, 0.f, 0.f, 0.f), cp = cq;
        uint32_t nibble = 0u;
        if (HITS) {
          nibble = (uint32_t)s_hits[valid ? jj : 0] >> (4 * wave);
        } else {
          const float4 xyf = s_xyf[valid ? jj : 0];
          mu = make_float2(xyf.x, xyf.y);
          cq = s_co[valid ? jj : 0];
          cp = s_cp[valid ? jj : 0];
        }
        uint64_t hit_m[4];
        bool hits[4] = {false, false, false, false};
        if (!HITS) ellipse_hits_quadrant(mu, cq, cp.x, cp.y, cp.z, rt.qx0, rt.qy0, hits);
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const bool touches = HITS ? ((nibble >> r) & 1u) != 0u : hits[r];
          hit_m[r] = valid_m & gs_ballot((first_pos - jj) < row_last_of[r]) & gs_ballot(touches);
        }
        auto list_row = [&](auto row_tag) {
          constexpr int r = decltype(row_tag)::value;
          const uint64_t b = hit_m[r];
          const uint32_t below = __builtin_amdgcn_mbcnt_hi((uint32_t)(b >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)b, 0u));
          if (__builtin_amdgcn_inverse_ballot_w64(b)) reinterpret_cast<uint8_t*>(&s_idx[wave][r][0])[below] = (uint8_t)lane;
          return (uint32_t)__builtin_amdgcn_readfirstlane((int)__popcll(b));
        };
        len0 = list_row(std::integral_constant<int, 0>{});
        len1 = list_row(std::integral_constant<int, 1>{});
        len2 = list_row(std::integral_constant<int, 2>{});
        len3 = list_row(std::integral_constant<int, 3>{});
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const uint32_t my_len = row == 0 ? len0 : (row == 1 ? len1 : (row == 2 ? len2 : len3));
      const uint32_t passes = max(max(len0, len1), max(len2, len3));  // wave-uniform
      // The passes in which two rows of the wave are at the same Gaussian (their sums are merged before they go
      // to the accumulator) are known as soon as the lists are: bit n of meet_m = entry n of two lists is the
      // same slot.  Lane n looks at entry n of the four lists.
      uint64_t meet_m;
      {
        const uint8_t* lists = reinterpret_cast<const uint8_t*>(&s_idx[wave][0][0]);
        const uint32_t e0 = lists[lane], e1 = lists[SUB + lane], e2 = lists[2 * SUB + lane], e3 = lists[3 * SUB + lane];
        const bool v0 = (uint32_t)lane < len0, v1 = (uint32_t)lane < len1, v2 = (uint32_t)lane < len2,
                   v3 = (uint32_t)lane < len3;
        meet_m = gs_ballot((v0 && v1 && e0 == e1) || (v0 && v2 && e0 == e2) || (v0 && v3 && e0 == e3) ||
                           (v1 && v2 && e1 == e2) || (v1 && v3 && e1 == e3) || (v2 && v3 && e2 == e3));
      }

      // SELECT: a lane for which the Gaussian does not count takes the Gaussian's colour and geometry channels
      // as 0 (its step then still only rotates the recurrence state: alpha = 0 with a finite colour), so that a
      // non-finite channel only reaches the pixels that blended it in the forward pass, as in the reference
      // (cuda_rasterizer/backward.cu:463-472).  Same bits for finite inputs.
      auto walk = [&, my_len, passes, meet_m](auto select_tag) {
        constexpr bool SELECT = decltype(select_tag)::value;
        uint32_t word = 0u;  // four entries of the list
        for (uint32_t n = 0; n < passes; n++) {
          if ((n & 3u) == 0u) word = s_idx[wave][row][n >> 2];
          const bool has = n < my_len;
          const uint64_t has_m = gs_ballot(has);
          // (slot 0 behind the end of the list: its data are this sub-batch's)
          const int ja = (int)__builtin_amdgcn_ubfe(word, (n & 3u) * 8u, 8u);  // slot of the accumulators
          const int j = base + ja;                                             // slot of the batch
          const int pos = first_pos - j;
          // Straight-line from here on: every lane evaluates its row's Gaussian, and a lane for which the
          // Gaussian does not count (behind the pixel's last contributor, outside the power window, alpha
          // below 1/255) takes part with alpha = 0, G = 0.  Such a step leaves T unchanged (T * 1/(1-0)),
          // contributes zeros to every sum and leaves the recurrence state as it is
          // (fma(0, c, 1 * accum) == accum), so results are those of skipping it.
          // Same tests as the forward pass, on the same bits.
          const float4 xy = s_xyf[j];
          const float4 co = s_co[j];
          const float dx = xy.x - pfx, dy = xy.y - pfy;
          const float power = -0.5f * (co.x * dx * dx + co.z * dy * dy) - co.y * dx * dy;
          // never true for pixels outside the image (last_contributor = 0)
          const float floor_j = xy.z;
          // (lane masks of single comparisons, combined in scalar registers: no short-circuit branches in the loop)
          const uint64_t in_m = has_m & gs_ballot(pos < last_contributor) & gs_ballot(!(power > 0.0f)) &
                                gs_ballot(!(power < floor_j));
          if (in_m == 0ull) continue;  // wave-uniform
          const float G_raw = gs_expf_core(power);
          const float alpha_raw = fminf(0.99f, co.w * G_raw);
          const uint64_t active_m = in_m & gs_ballot(!(alpha_raw < 1.0f / 255.0f));
          if (active_m == 0ull) continue;  // wave-uniform
          const bool active = __builtin_amdgcn_inverse_ballot_w64(active_m);
          const float alpha = active ? alpha_raw : 0.f;
          const float G = active ? G_raw : 0.f;

          float v[NV];
          // The transmittance follows the CPU statement's operation sequence exactly (IEEE reciprocal):
          // upstream gradients of the geometry channels can be many orders of magnitude larger than the
          // result (plane depth divides by a blended normal that may be nearly perpendicular to the ray), so
          // T, which multiplies them, decides how far a gradient can drift.  What follows dL/dalpha is
          // products only.
          const float rcp1ma = gs_rcp_normal(1.f - alpha);  // alpha <= 0.99: the bits of 1.f / (1.f - alpha)
          T = T * rcp1ma;
          const float w = alpha * T;
          const float oma = 1.f - alpha;
          float colour_dot = 0.0f;  // S
          {
            const float4 c4 = s_chan[j][0];
            const float c[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
            for (int ch = 0; ch < GS_N_RGB; ch++) {
              colour_dot = __builtin_fmaf((!SELECT || active) ? c[ch] : 0.f, gpix[ch], colour_dot);
              v[8 + ch] = w * gpix[ch];
            }
            if (render_geo) {
              const float4 m4 = s_chan[j][RENDER_GEO ? 1 : 0];
              const float m[GS_N_MAP] = {c4.w, m4.x, m4.y, m4.z, m4.w};
#pragma unroll
              for (int ch = 0; ch < GS_N_MAP; ch++) {
                colour_dot = __builtin_fmaf((!SELECT || active) ? m[ch] : 0.f, gmap[ch], colour_dot);
                v[11 + ch] = w * gmap[ch];
              }
            } else {
#pragma unroll
              for (int ch = 0; ch < GS_N_MAP; ch++) v[11 + ch] = 0.f;
            }
          }
          float dL_dalpha = colour_dot - behind_dot;
          behind_dot = __builtin_fmaf(alpha, colour_dot, oma * behind_dot);  // (alpha = 0: unchanged)
          dL_dalpha = __builtin_fmaf(dL_dalpha, T, -(bg_term * rcp1ma));
          dL_dalpha = active ? dL_dalpha : 0.f;
          // The per-Gaussian factors of the geometric gradients stay out of the pixel sums: with
          // q = G dL/dalpha, u = conic (dx, dy), a pixel's terms are dL/dmean = -opacity q u,
          // dL/dconic = -opacity/2 q (dx dx, dx dy, dy dy) and dL/dopacity = q
          // (cuda_rasterizer/backward.cu:520-541), so the row sums q u, q (dx dx, dx dy, dy dy) and q, and the
          // thread that hands a record over multiplies by -opacity, |opacity| (the sums of absolute values,
          // formed inside the row reduction) and -opacity/2.  (The factors W/2 and H/2 from pixel to normalised
          // coordinates are applied once per Gaussian by the reduction kernel.)
          const float q = G * dL_dalpha;
          const float ux = __builtin_fmaf(co.y, dy, co.x * dx), uy = __builtin_fmaf(co.y, dx, co.z * dy);
          v[0] = q * ux;
          v[1] = q * uy;
          const float qx = q * dx;
          v[4] = qx * dx;
          v[5] = qx * dy;
          v[6] = (q * dy) * dy;
          v[7] = q;
          // lane q of the row now receives the row's total of component q
          float tot = row_transpose_reduce16_abs23(v);
          // Rows of this wave that are at the same Gaussian in this pass are merged, and the lowest of them
          // adds the sum to the wave's own accumulator with a plain read-add-write: rows that write hold
          // different Gaussians, so their addresses differ.  (An LDS float atomic takes about three cycles per
          // active lane on this hardware, thirteen times the read-add-write.)
          bool writes = has;
          if ((meet_m >> n) & 1ull) {  // wave-uniform, uncommon
            const int key = has ? ja : -1 - row;
            const int k0 = __builtin_amdgcn_readlane(key, 0), k1 = __builtin_amdgcn_readlane(key, 16);
            const int k2 = __builtin_amdgcn_readlane(key, 32), k3 = __builtin_amdgcn_readlane(key, 48);
            constexpr uint64_t R0 = 0xFFFFull, R1 = R0 << 16, R2 = R0 << 32, R3 = R0 << 48;
            const uint64_t eq16 = (k0 == k1 ? R0 | R1 : 0ull) | (k2 == k3 ? R2 | R3 : 0ull);
            const uint64_t eq32 = (k0 == k2 ? R0 | R2 : 0ull) | (k1 == k3 ? R1 | R3 : 0ull);
            const uint64_t eq48 = (k0 == k3 ? R0 | R3 : 0ull) | (k1 == k2 ? R1 | R2 : 0ull);
            const uint64_t follower = (k1 == k0 ? R1 : 0ull) | ((k2 == k0 || k2 == k1) ? R2 : 0ull) |
                                      ((k3 == k0 || k3 == k1 || k3 == k2) ? R3 : 0ull);
            const float t16 = __shfl_xor(tot, 16, GS_WAVE), t32 = __shfl_xor(tot, 32, GS_WAVE);
            const float t48 = __shfl_xor(tot, 48, GS_WAVE);
            tot += __builtin_amdgcn_inverse_ballot_w64(eq16) ? t16 : 0.f;
            tot += __builtin_amdgcn_inverse_ballot_w64(eq32) ? t32 : 0.f;
            tot += __builtin_amdgcn_inverse_ballot_w64(eq48) ? t48 : 0.f;
            writes = has && !__builtin_amdgcn_inverse_ballot_w64(follower);
          }
          if (writes && tot != 0.f) s_acc[wave][l16][ja] += tot;
        }
      };
      if (select_state) walk(std::true_type{});
      else walk(std::false_type{});
      __syncthreads();
      // a thread stores a quarter of a record: the four waves' sums of four components, added in wave order;
      // it leaves zeros behind for the next sub-batch
      {
        float c[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          c[e] = s_acc[0][4 * my_part + e][my_slot];
          s_acc[0][4 * my_part + e][my_slot] = 0.f;
#pragma unroll
          for (int w = 1; w < WAVES; w++) {
            c[e] += s_acc[w][4 * my_part + e][my_slot];
            s_acc[w][4 * my_part + e][my_slot] = 0.f;
          }
        }
        if (base + my_slot < count) {
          const float opacity = s_co[base + my_slot].w;
          if (my_part == 0) {  // mean2D x, y and their sums of absolute values
            c[0] *= -opacity; c[1] *= -opacity; c[2] *= fabsf(opacity); c[3] *= fabsf(opacity);
          } else if (my_part == 1) {  // conic x, y, w; the fourth component is the opacity gradient itself
            const float h = -0.5f * opacity;
            c[0] *= h; c[1] *= h; c[2] *= h;
          }
          instance_grads[4 * (size_t)s_emis[base + my_slot] + my_part] = make_float4(c[0], c[1], c[2], c[3]);
        }
      }
      __syncthreads();
    }
  }
}

// Sums the instance records of every Gaussian (consecutive in emission order) into the gradient
// tensors.  Record layout: [mean2D.x, mean2D.y, |mean2D|.x, |mean2D|.y, conic.x, conic.y, conic.w,
// opacity, rgb(3), map(5)].  Every output element is written.
__global__ void __launch_bounds__(GS_BLOCK_1D)
reduce_instances_kernel(int P, const uint32_t* __restrict__ point_offsets, const float4* __restrict__ instance_grads,
                        float ddelx_dx, float ddely_dy, int render_geo, float2* __restrict__ dL_dmean2D, float* __restrict__ dL_dmean2D_abs,
                        float4* __restrict__ dL_dconic_opacity, float* __restrict__ dL_dcolors,
                        float* __restrict__ dL_dall_map) {
  const int i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  const int lane = threadIdx.x & (GS_WAVE - 1);
  const bool live = i < P;
  const uint32_t b = (!live || i == 0) ? 0u : point_offsets[i - 1], e = live ? point_offsets[i] : 0u;
  const uint32_t n = e - b;
  float4 a0 = make_float4(0.f, 0.f, 0.f, 0.f), a1 = a0, a2 = a0, a3 = a0;
  auto add = [](float4& a, const float4& r) { a.x += r.x; a.y += r.y; a.z += r.z; a.w += r.w; };
  // A Gaussian with many instances (in a street-level view one can cover thousands of tiles) is summed by the
  // whole wave: lane l takes records l, l + 64, ..., then the 64 partial sums are added across the lanes in a fixed
  // order.  Everything else is summed by its own thread, record after record.
  constexpr uint32_t MANY = 32;
  constexpr uint32_t REC_CHUNK = GS_WAVE, REC_STRIDE4 = 5;
  __shared__ float4 s_rec[GS_BLOCK_1D / GS_WAVE][REC_CHUNK * REC_STRIDE4];
  uint64_t many = gs_ballot(n > MANY);
  const uint64_t many_in_wave = many;
  while (many != 0ull) {
    const int owner = (int)__builtin_ctzll(many);
    many &= many - 1ull;
    const uint32_t ob = __shfl(b, owner, GS_WAVE), on = __shfl(n, owner, GS_WAVE);
    float4 p0 = make_float4(0.f, 0.f, 0.f, 0.f), p1 = p0, p2 = p0, p3 = p0;
    for (uint32_t k = (uint32_t)lane; k < on; k += GS_WAVE) {
      const float4* rec = instance_grads + 4 * (size_t)(ob + k);
      add(p0, rec[0]); add(p1, rec[1]); add(p2, rec[2]); add(p3, rec[3]);
    }
#pragma unroll
    for (int d = GS_WAVE / 2; d >= 1; d >>= 1) {
      float4* parts[4] = {&p0, &p1, &p2, &p3};
#pragma unroll
      for (int q = 0; q < 4; q++) {
        parts[q]->x += __shfl_xor(parts[q]->x, d, GS_WAVE);
        parts[q]->y += __shfl_xor(parts[q]->y, d, GS_WAVE);
        parts[q]->z += __shfl_xor(parts[q]->z, d, GS_WAVE);
        parts[q]->w += __shfl_xor(parts[q]->w, d, GS_WAVE);
      }
    }
    if (lane == owner) { a0 = p0; a1 = p1; a2 = p2; a3 = p3; }
  }
  if (many_in_wave != 0ull) {
    // (a wave that holds such a Gaussian reads the others' records directly: rare)
    if (live && n <= MANY) {
      for (uint32_t k = b; k < e; k++) {
        const float4* rec = instance_grads + 4 * (size_t)k;
        add(a0, rec[0]); add(a1, rec[1]); add(a2, rec[2]); add(a3, rec[3]);
      }
    }
  } else {
    // The records of a wave's 64 Gaussians are one contiguous run.  It is fetched 64 records at a time with
    // whole-wave 16-byte loads (the four lanes of a record share its 64-byte line), parked in LDS (records
    // padded to five 16-byte words: neither access pattern has bank conflicts) and every lane then adds up its own
    // records from there, in order.  With every lane loading its own records directly, a line passed through
    // the first-level cache once per 16-byte part.
    float4* mine = s_rec[threadIdx.x / GS_WAVE];
    const uint32_t run_begin = (uint32_t)__builtin_amdgcn_readfirstlane((int)b);
    uint32_t run_end = e;
#pragma unroll
    for (int d = GS_WAVE / 2; d >= 1; d >>= 1) run_end = max(run_end, (uint32_t)__shfl_xor((int)run_end, d, GS_WAVE));
    run_end = (uint32_t)__builtin_amdgcn_readfirstlane((int)run_end);
    for (uint32_t c = run_begin; c < run_end; c += REC_CHUNK) {
      float4 v[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const uint32_t idx = (uint32_t)(j * GS_WAVE + lane), r = c + (idx >> 2);
        v[j] = r < run_end ? instance_grads[4 * (size_t)r + (idx & 3u)] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const uint32_t idx = (uint32_t)(j * GS_WAVE + lane);
        mine[(idx >> 2) * REC_STRIDE4 + (idx & 3u)] = v[j];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const uint32_t lo = max(b, c), hi = min(e, c + REC_CHUNK);
      for (uint32_t k = lo; k < hi; k++) {
        const float4* rec = mine + (k - c) * REC_STRIDE4;
        add(a0, rec[0]); add(a1, rec[1]); add(a2, rec[2]); add(a3, rec[3]);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  }
  if (!live) return;
  // records hold the mean2D sums per pixel unit: d(pixel offset)/d(normalised coordinate) = W/2, H/2
  dL_dmean2D[i] = make_float2(a0.x * ddelx_dx, a0.y * ddely_dy);
  dL_dmean2D_abs[3 * (size_t)i] = a0.z * ddelx_dx;
  dL_dmean2D_abs[3 * (size_t)i + 1] = a0.w * ddely_dy;
  dL_dmean2D_abs[3 * (size_t)i + 2] = 0.f;
  dL_dconic_opacity[i] = a1;
  dL_dcolors[3 * (size_t)i] = a2.x;
  dL_dcolors[3 * (size_t)i + 1] = a2.y;
  dL_dcolors[3 * (size_t)i + 2] = a2.z;
  if (dL_dall_map) {
    float* m = dL_dall_map + 5 * (size_t)i;
    m[0] = render_geo ? a2.w : 0.f;
    m[1] = render_geo ? a3.x : 0.f;
    m[2] = render_geo ? a3.y : 0.f;
    m[3] = render_geo ? a3.z : 0.f;
    m[4] = render_geo ? a3.w : 0.f;
  }
}

}  // namespace

int launch_render_bwd(const RenderBwdArgs& a, hipStream_t stream) {
  const dim3 grid((a.W + GS_TILE_X - 1) / GS_TILE_X, (a.H + GS_TILE_Y - 1) / GS_TILE_Y, 1);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(GS_TILE_PIX), 0, stream, (const uint2*)a.ranges, a.point_list, a.W, a.H,
                       a.fx, a.fy, a.bg, (const float2*)a.means2D, (const float4*)a.conic_opacity, a.rgb, a.all_map,
                       a.all_map_pixels, a.final_T, a.n_contrib_px, a.compute_locally, a.dL_dpix, a.dL_dout_all_map,
                       a.dL_dout_plane_depth, a.emission_sorted, (float4*)a.instance_grads, a.block_hits,
                       (const float4*)a.packed, a.packed_valid);
  };
  if (a.render_geo) {
    if (a.block_hits) go(render_bwd_kernel<true, true>);
    else go(render_bwd_kernel<true, false>);
  } else {
    if (a.block_hits) go(render_bwd_kernel<false, true>);
    else go(render_bwd_kernel<false, false>);
  }
  hipLaunchKernelGGL(reduce_instances_kernel, dim3((a.P + GS_BLOCK_1D - 1) / GS_BLOCK_1D), dim3(GS_BLOCK_1D), 0,
                     stream, a.P, a.point_offsets, (const float4*)a.instance_grads, (float)(0.5 * a.W),
                     (float)(0.5 * a.H), a.render_geo,
                     (float2*)a.dL_dmean2D, a.dL_dmean2D_abs, (float4*)a.dL_dconic_opacity, a.dL_dcolors,
                     a.dL_dall_map);
  return 0;
}

}  // namespace gs
