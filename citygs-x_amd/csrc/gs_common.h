// Shared host/device definitions for the gfx950 Gaussian rasterizer library.
//
// Arithmetic policy: every kernel is compiled with -ffp-contract=off, so each
// fp32 operation rounds once exactly as written; fused multiply-adds appear
// only where __builtin_fmaf is spelled out.  Division and sqrt are the
// correctly rounded ones (hipcc default).  This is what makes radii, tile
// rectangles, depth keys and contributor counts reproducible bit for bit on a
// CPU.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define GS_TILE_X 16      // cuda_rasterizer/config.h:17
#define GS_TILE_Y 16      // cuda_rasterizer/config.h:19
#define GS_TILE_PIX 256
#define GS_BLOCK_1D 256   // cuda_rasterizer/config.h:21
#define GS_N_RGB 3        // cuda_rasterizer/config.h:15
#define GS_N_MAP 5        // cuda_rasterizer/config.h:24
#define GS_WAVE 64

namespace gs {

// Lane mask of a predicate.  Takes the bool itself: the int-taking __ballot makes the compiler materialise the
// predicate as 0/1 in a vector register and compare it again.
__device__ __forceinline__ uint64_t gs_ballot(bool p) { return __builtin_amdgcn_ballot_w64(p); }

void set_error(const char* fmt, ...);
int check_launch(const char* what, hipStream_t stream, bool sync);

#define GS_HIP_TRY(expr)                                                            \
  do {                                                                              \
    hipError_t _e = (expr);                                                         \
    if (_e != hipSuccess) {                                                         \
      gs::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
      return 1;                                                                     \
    }                                                                               \
  } while (0)

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// ------------------------------------------------------------ device math --

__device__ __forceinline__ int f2i_sat(float v) {
  // float -> int32: truncate toward zero, clamp to the int32 range, NaN -> 0.  That is what the conversion
  // instruction does by itself; as C++ (three comparisons around a cast, whose out-of-range cases the language
  // leaves undefined) it came out as three nested branches per conversion.
  int r;
  asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(v));
  return r;
}

// Workgroups go to the eight XCDs in turn (workgroup b of a launch runs on XCD b % 8), and each XCD has its own L2.
// This renumbers them so that the workgroups of one XCD hold consecutive indices (XCD 0 the first eighth, and so
// on, each in launch order): work items that are neighbours in memory then share an L2.  A bijection on [0, n).
__device__ __forceinline__ uint32_t xcd_contiguous_index(uint32_t b, uint32_t n) {
  constexpr uint32_t XCDS = 8;
  const uint32_t x = b % XCDS, rest = n % XCDS;
  return x * (n / XCDS) + (x < rest ? x : rest) + b / XCDS;
}

__device__ __forceinline__ uint32_t f2u_sat(float v) {
  // float -> uint32: truncate, clamp to [0, 2^32 - 1], NaN -> 0 (the conversion instruction's own behaviour)
  uint32_t r;
  asm("v_cvt_u32_f32 %0, %1" : "=v"(r) : "v"(v));
  return r;
}

// Store for data that is written once and not read again on the GPU for a long while (gradients of leaf
// parameters on their way to the optimizer): it goes out past the caches, so it does not evict what the next
// kernel reads.
__device__ __forceinline__ void store_streaming(float4* p, const float4& v) {
  typedef float v4f __attribute__((ext_vector_type(4)));
  const v4f w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<v4f*>(p));
}

// exp() of the blending loops: n = rint(x*log2e), r = x - n*ln2 (two-constant
// split), degree-6 polynomial, scale by 2^n.  Only IEEE operations and explicit
// FMAs, so a CPU evaluates the same bits.  x < -87 -> 0, x > 88 -> +inf.
__device__ __forceinline__ float gs_expf(float x) {
  if (!(x == x)) return x;
  if (x < -87.0f) return 0.0f;
  if (x > 88.0f) return __builtin_inff();
  float n = __builtin_rintf(x * 1.44269504088896341f);
  float r = __builtin_fmaf(n, -0.693145751953125f, x);
  r = __builtin_fmaf(n, -1.42860682030941723212e-6f, r);
  float p = 1.9875691500e-4f;
  p = __builtin_fmaf(p, r, 1.3981999507e-3f);
  p = __builtin_fmaf(p, r, 8.3334519073e-3f);
  p = __builtin_fmaf(p, r, 4.1665795894e-2f);
  p = __builtin_fmaf(p, r, 1.6666665459e-1f);
  p = __builtin_fmaf(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  p = __builtin_fmaf(p, r2, r);
  p = p + 1.0f;
  return __builtin_ldexpf(p, (int)n);
}

// Same routine without the range checks, for callers that guarantee -87 <= x <= 0
// (or NaN, which propagates); returns the same bits as gs_expf there.
__device__ __forceinline__ float gs_expf_core(float x) {
  float n = __builtin_rintf(x * 1.44269504088896341f);
  float r = __builtin_fmaf(n, -0.693145751953125f, x);
  r = __builtin_fmaf(n, -1.42860682030941723212e-6f, r);
  float p = 1.9875691500e-4f;
  p = __builtin_fmaf(p, r, 1.3981999507e-3f);
  p = __builtin_fmaf(p, r, 8.3334519073e-3f);
  p = __builtin_fmaf(p, r, 4.1665795894e-2f);
  p = __builtin_fmaf(p, r, 1.6666665459e-1f);
  p = __builtin_fmaf(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  p = __builtin_fmaf(p, r2, r);
  p = p + 1.0f;
  return __builtin_ldexpf(p, (int)n);
}

// 1.0f / d for a normal d whose reciprocal is normal too: the operation sequence of the IEEE division
// without its scaling and special-case steps, which change nothing in that range.  Same bits, four
// instructions fewer.
__device__ __forceinline__ float gs_rcp_normal(float d) {
  const float r0 = __builtin_amdgcn_rcpf(d);
  const float r = __builtin_fmaf(__builtin_fmaf(-d, r0, 1.0f), r0, r0);
  const float q = __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
  return __builtin_fmaf(__builtin_fmaf(-d, q, 1.0f), r, q);
}

// Column-major 3x3 with the product evaluated term by term, left to right
// (the semantics of the reference's matrix type,
// third_party/glm/glm/detail/type_mat3x3.inl:486-518).
struct M3 {
  float m[3][3];  // m[col][row]
};

__device__ __forceinline__ M3 m3_cols(float a0, float a1, float a2, float b0, float b1, float b2,
                                      float c0, float c1, float c2) {
  M3 r;
  r.m[0][0] = a0; r.m[0][1] = a1; r.m[0][2] = a2;
  r.m[1][0] = b0; r.m[1][1] = b1; r.m[1][2] = b2;
  r.m[2][0] = c0; r.m[2][1] = c1; r.m[2][2] = c2;
  return r;
}

__device__ __forceinline__ M3 m3_mul(const M3& A, const M3& B) {
  M3 R;
#pragma unroll
  for (int c = 0; c < 3; c++)
#pragma unroll
    for (int r = 0; r < 3; r++)
      R.m[c][r] = (A.m[0][r] * B.m[c][0] + A.m[1][r] * B.m[c][1]) + A.m[2][r] * B.m[c][2];
  return R;
}

__device__ __forceinline__ M3 m3_T(const M3& A) {
  M3 R;
#pragma unroll
  for (int c = 0; c < 3; c++)
#pragma unroll
    for (int r = 0; r < 3; r++) R.m[c][r] = A.m[r][c];
  return R;
}

__device__ __forceinline__ float dot3(const float* a, const float* b) {
  return (a[0] * b[0] + a[1] * b[1]) + a[2] * b[2];
}

// Row-vector transforms by a 4x4 matrix stored row-major
// (cuda_rasterizer/auxiliary.h:112-151).
__device__ __forceinline__ void xform4x3(const float* p, const float* M, float* o) {
#pragma unroll
  for (int k = 0; k < 3; k++) o[k] = ((M[k] * p[0] + M[4 + k] * p[1]) + M[8 + k] * p[2]) + M[12 + k];
}
__device__ __forceinline__ void xform4x4(const float* p, const float* M, float* o) {
#pragma unroll
  for (int k = 0; k < 4; k++) o[k] = ((M[k] * p[0] + M[4 + k] * p[1]) + M[8 + k] * p[2]) + M[12 + k];
}
__device__ __forceinline__ void xformVec4x3T(const float* v, const float* M, float* o) {
#pragma unroll
  for (int k = 0; k < 3; k++) o[k] = (M[4 * k] * v[0] + M[4 * k + 1] * v[1]) + M[4 * k + 2] * v[2];
}

// cuda_rasterizer/auxiliary.h:52-55 (double intermediates).
__device__ __forceinline__ float ndc2pix(float v, int S) {
  return (float)((((double)v + 1.0) * (double)S - 1.0) * 0.5);
}

struct Rect {
  uint32_t x0, y0, x1, y1;
};

// cuda_rasterizer/auxiliary.h:66-76: tile rectangle [min,max) of a splat with
// integer radius, clamped to the grid.
__device__ __forceinline__ Rect get_rect(float px, float py, int radius, uint32_t gx, uint32_t gy) {
  const float rf = (float)radius;
  Rect r;
  r.x0 = min(gx, (uint32_t)max(0, f2i_sat((px - rf) / (float)GS_TILE_X)));
  r.y0 = min(gy, (uint32_t)max(0, f2i_sat((py - rf) / (float)GS_TILE_Y)));
  r.x1 = min(gx, (uint32_t)max(0, f2i_sat((((px + rf) + (float)GS_TILE_X) - 1.0f) / (float)GS_TILE_X)));
  r.y1 = min(gy, (uint32_t)max(0, f2i_sat((((py + rf) + (float)GS_TILE_Y) - 1.0f) / (float)GS_TILE_Y)));
  return r;
}

// Walks the tile rectangles of a wave's 64 Gaussians (one per lane; `live` = the lane has one) and calls
// visit(payload_of_owner, tile, rank) for every tile of a rectangle that is computed locally, rank = number of
// such tiles before it in the rectangle's row-major order (the order duplicateWithKeys emits them,
// cuda_rasterizer/rasterizer_impl.cu:95-112).  Returns, to the owner lane, its rectangle's count of local tiles.
// A rectangle of more than GS_BIG_RECT tiles is walked by the whole wave, 64 tiles at a time, instead of by its
// owner alone: a street-level view has Gaussians that cover thousands of tiles, and one lane looping over them
// would hold up everybody.  `mine` is whatever visit needs of the owning Gaussian (a struct of 32-bit words); for a
// big rectangle it is handed from the owner lane to all lanes while the wave is still convergent.  Every lane of
// the wave must call this (it uses ballots and cross-lane reads).
#define GS_BIG_RECT 16
// The rectangles of more than GS_BIG_RECT tiles among the wave's 64, one after the other, each by the whole wave:
// 64 tiles per step, ranks by ballot.  Returns, to the owner lane of such a rectangle, its count of local tiles
// (0 to every other lane).
template <typename Payload, typename Mask, typename Visit>
__device__ __forceinline__ uint32_t walk_wave_big_rects(uint32_t area, const Rect& rc, uint32_t w, uint32_t gx,
                                                        const Payload& mine, Mask is_local, Visit visit) {
  static_assert(sizeof(Payload) % 4 == 0, "payload of 32-bit words");
  const int lane = threadIdx.x & (GS_WAVE - 1);
  uint32_t count = 0;
  uint64_t big = __ballot(area > GS_BIG_RECT);
  while (big != 0ull) {
    const int owner = (int)__builtin_ctzll(big);
    big &= big - 1ull;
    const uint32_t ox0 = __shfl(rc.x0, owner, GS_WAVE), oy0 = __shfl(rc.y0, owner, GS_WAVE);
    const uint32_t ow = __shfl(w, owner, GS_WAVE), on = __shfl(area, owner, GS_WAVE);
    Payload theirs;
    {
      const uint32_t* src = reinterpret_cast<const uint32_t*>(&mine);
      uint32_t* dst = reinterpret_cast<uint32_t*>(&theirs);
#pragma unroll
      for (int k = 0; k < (int)(sizeof(Payload) / 4); k++) dst[k] = __shfl(src[k], owner, GS_WAVE);
    }
    uint32_t before = 0;
    for (uint32_t q0 = 0; q0 < on; q0 += GS_WAVE) {
      const uint32_t q = q0 + (uint32_t)lane;
      const uint32_t ry = q / ow, rx = q - ry * ow;
      const uint32_t tile = (oy0 + ry) * gx + (ox0 + rx);
      const bool local = q < on && is_local(tile);
      const uint64_t bits = __ballot(local);
      if (local) visit(theirs, tile, before + (uint32_t)__popcll(bits & ((1ull << lane) - 1ull)));
      before += (uint32_t)__popcll(bits);
    }
    if (lane == owner) count = before;
  }
  return count;
}

template <typename Payload, typename Mask, typename Visit>
__device__ __forceinline__ uint32_t walk_wave_rects(bool live, const Rect& rc, uint32_t gx, const Payload& mine,
                                                    Mask is_local, Visit visit) {
  const uint32_t w = live ? rc.x1 - rc.x0 : 0u, h = live ? rc.y1 - rc.y0 : 0u;
  const uint32_t area = w * h;
  uint32_t count = walk_wave_big_rects(area, rc, w, gx, mine, is_local, visit);
  if (area != 0u && area <= GS_BIG_RECT) {
    for (uint32_t y = rc.y0; y < rc.y1; y++)
      for (uint32_t x = rc.x0; x < rc.x1; x++) {
        const uint32_t tile = y * gx + x;
        if (is_local(tile)) {
          visit(mine, tile, count);
          count++;
        }
      }
  }
  return count;
}

// Inclusive scans over the 64 lanes of a wave by DPP moves: four shifts inside the 16-lane rows, then the last
// lane of rows 0 and 2 goes to rows 1 and 3 and lane 31 to rows 2 and 3 (a lane without a source takes the
// identity, 0).  All 64 lanes must be active.
#define GS_WAVE_SCAN_STEP(OP, CTRL, ROWS) \
  v = OP(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROWS, 0xF, false))
__device__ __forceinline__ uint32_t gs_scan_add_op(uint32_t a, uint32_t b) { return a + b; }
__device__ __forceinline__ uint32_t gs_scan_max_op(uint32_t a, uint32_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint32_t wave_scan_add(uint32_t v) {
  GS_WAVE_SCAN_STEP(gs_scan_add_op, 0x111, 0xF);  // row_shr:1
  GS_WAVE_SCAN_STEP(gs_scan_add_op, 0x112, 0xF);  // row_shr:2
  GS_WAVE_SCAN_STEP(gs_scan_add_op, 0x114, 0xF);  // row_shr:4
  GS_WAVE_SCAN_STEP(gs_scan_add_op, 0x118, 0xF);  // row_shr:8
  GS_WAVE_SCAN_STEP(gs_scan_add_op, 0x142, 0xA);  // row_bcast:15 into rows 1 and 3
  GS_WAVE_SCAN_STEP(gs_scan_add_op, 0x143, 0xC);  // row_bcast:31 into rows 2 and 3
  return v;
}
__device__ __forceinline__ uint32_t wave_scan_max(uint32_t v) {
  GS_WAVE_SCAN_STEP(gs_scan_max_op, 0x111, 0xF);
  GS_WAVE_SCAN_STEP(gs_scan_max_op, 0x112, 0xF);
  GS_WAVE_SCAN_STEP(gs_scan_max_op, 0x114, 0xF);
  GS_WAVE_SCAN_STEP(gs_scan_max_op, 0x118, 0xF);
  GS_WAVE_SCAN_STEP(gs_scan_max_op, 0x142, 0xA);
  GS_WAVE_SCAN_STEP(gs_scan_max_op, 0x143, 0xC);
  return v;
}
#undef GS_WAVE_SCAN_STEP

// A pointer into LDS typed as such: volatile accesses through a plain pointer come out as flat loads and stores.
typedef __attribute__((address_space(3))) uint32_t lds_word;

// walk_wave_rects for a wave all of whose tiles are computed locally (no tile mask), with the work spread evenly:
// the rectangles of at most GS_BIG_RECT tiles are laid end to end (a prefix sum of their areas over the lanes) and
// lane l of round k takes instance 64 k + l of that sequence, whichever Gaussian it belongs to, instead of every
// lane looping over its own rectangle while the lanes with smaller ones wait.  The owner of an instance is found
// through `heads` (64 words of LDS of the wave's own): every owner enters its lane number at the place of its
// first instance, and a running maximum over the places carries it to the instances behind.  What visit needs of
// the owner comes by cross-lane reads.  rank = the instance's place in its rectangle's row-major order, which
// with every tile local is the rank walk_wave_rects gives.  Larger rectangles are walked as there.
template <typename Payload, typename Visit>
__device__ __forceinline__ uint32_t walk_wave_rects_flat(bool live, const Rect& rc, uint32_t gx, const Payload& mine,
                                                         lds_word* heads, Visit visit) {
  static_assert(sizeof(Payload) % 4 == 0, "payload of 32-bit words");
  static_assert(GS_BIG_RECT <= 16, "areas and ranks are packed into 5 and 11 bits");
  const int lane = threadIdx.x & (GS_WAVE - 1);
  const uint32_t w = live ? rc.x1 - rc.x0 : 0u, h = live ? rc.y1 - rc.y0 : 0u;
  const uint32_t area = w * h;
  (void)walk_wave_big_rects(area, rc, w, gx, mine, [](uint32_t) { return true; }, visit);
  const uint32_t small = area <= GS_BIG_RECT ? area : 0u;
  const uint32_t incl = wave_scan_add(small), excl = incl - small;
  const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)incl, GS_WAVE - 1);
  // what an instance needs of its owner: the rectangle's corner, and in one word its width (5 bits), the place of
  // its first instance (11 bits) and m = floor(2^15 / width) + 1, with which (q m) >> 15 = q / width for q < 16
  const uint32_t corner = rc.x0 | (rc.y0 << 16);
  const uint32_t m = w != 0u ? (uint32_t)(32768.0f / (float)w) + 1u : 0u;  // (exact: w <= 16)
  const uint32_t shape = w | (excl << 5) | (m << 16);
  volatile lds_word* vheads = heads;
  uint32_t carried = 0;  // owner of the last instance of the previous round, plus one
  for (uint32_t base = 0; base < total; base += GS_WAVE) {
    vheads[lane] = 0u;
    __builtin_amdgcn_wave_barrier();
    if (small != 0u && excl >= base && excl < base + GS_WAVE) vheads[excl - base] = (uint32_t)lane + 1u;
    __builtin_amdgcn_wave_barrier();
    uint32_t owner1 = wave_scan_max(vheads[lane]);
    __builtin_amdgcn_wave_barrier();
    owner1 = owner1 > carried ? owner1 : carried;
    carried = (uint32_t)__builtin_amdgcn_readlane((int)owner1, GS_WAVE - 1);
    const int src_lane = (int)owner1 - 1;  // (at least 0: the first instance of the sequence is a head)
    const uint32_t o_corner = __shfl(corner, src_lane, GS_WAVE), o_shape = __shfl(shape, src_lane, GS_WAVE);
    Payload theirs;
    {
      const uint32_t* src = reinterpret_cast<const uint32_t*>(&mine);
      uint32_t* dst = reinterpret_cast<uint32_t*>(&theirs);
#pragma unroll
      for (int k = 0; k < (int)(sizeof(Payload) / 4); k++) dst[k] = __shfl(src[k], src_lane, GS_WAVE);
    }
    const uint32_t slot = base + (uint32_t)lane;
    if (slot < total) {
      const uint32_t ow = o_shape & 31u, q = slot - ((o_shape >> 5) & 2047u);
      const uint32_t ry = (q * (o_shape >> 16)) >> 15, rx = q - ry * ow;
      visit(theirs, ((o_corner >> 16) + ry) * gx + ((o_corner & 0xFFFFu) + rx), q);
    }
  }
  return area;
}

}  // namespace gs
