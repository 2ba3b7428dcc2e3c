// CPU oracle for the CityGS-X differentiable Gaussian rasterizer path.
//
// TEST INFRASTRUCTURE ONLY.  Nothing in the product (the HIP library and the
// Python operator modules built on it) may link, import or call this file; it
// exists so tests, the smoke check and the benchmark's CPU-baseline leg have an
// independent statement of what the reference computes.
//
// Every function restates the arithmetic of the reference rasterizer op by op
// in IEEE fp32 (one rounding per operation, no FMA contraction: build with
// -ffp-contract=off), keeping the reference's double-precision sites.  Citations
// use  CR/ = submodule_cityx/diff-gaussian-rasterization/cuda_rasterizer/,
//      DGR/ = submodule_cityx/diff-gaussian-rasterization/,
//      KNN/ = submodule_cityx/simple-knn/.
//
// Four deliberate, documented choices where the reference leaves the bits open
// (its CUDA binary contracts FMAs and calls the device expf):
//   * exp() in the blending loops is orc_expf below, a fixed Cody-Waite +
//     degree-6 polynomial routine built from fmaf and IEEE ops only, so the
//     same bits come out on any IEEE machine;
//   * float->int conversions saturate (NaN -> 0) like the GPU's conversion
//     instruction does (CR/forward.cu:254, CR/auxiliary.h:66-76);
//   * the per-pixel colour / map accumulation "C += c * alpha * T"
//     (CR/forward.cu:403-407) is evaluated as w = alpha*T; C = fma(c, w, C):
//     the form a contracting compiler produces, one rounding per channel.  It
//     only touches float image values (tolerance 1e-4), never a decision;
//   * likewise in the backward replay the "colour behind" recurrence and the
//     dL/dalpha accumulation (CR/backward.cu:497-521) are written with the
//     FMAs a contracting compiler forms from those source lines:
//     behind = fma(last_alpha, last_c, (1-last_alpha)*behind);
//     dL_dalpha = fma(c - behind, g, dL_dalpha);
//     and the two divisions by (1 - alpha) of CR/backward.cu:488,534 share one
//     reciprocal: inv = 1/(1-alpha); T *= inv;
//     dL_dalpha = fma(dL_dalpha, T, -(T_final*bg_dot)*inv).
//     Algebraically the reference's expressions, with the rounding order fixed.
//
// oracle_all_map_* restate caller-side torch code (floating-point sums whose order torch leaves open):
// pinned to rounding against a float64 torch evaluation with autograd, not bit for bit.
//
// Parity pins (tests/test_oracle_*.py): closed forms, an independent torch
// restatement with autograd, brute force on tiny inputs, numpy/scipy library
// routines.  The reference holds no golden vectors for this path.
//   parity unpinned: none.

#include <algorithm>
#include <cfloat>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <numeric>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

constexpr int TILE_X = 16;  // CR/config.h:17
constexpr int TILE_Y = 16;  // CR/config.h:19
constexpr int N_RGB = 3;    // CR/config.h:15
constexpr int N_MAP = 5;    // CR/config.h:24
constexpr int KNN_BOX = 1024;  // KNN/simple_knn.cu:12

// ---------------------------------------------------------------- helpers --

inline int f2i_sat(float v) {
  if (!(v == v)) return 0;
  if (v >= 2147483648.0f) return INT32_MAX;
  if (v <= -2147483648.0f) return INT32_MIN;
  return (int)v;
}

inline uint32_t f2u_sat(float v) {
  if (!(v == v)) return 0u;
  if (v >= 4294967296.0f) return UINT32_MAX;
  if (v <= 0.0f) return 0u;
  return (uint32_t)v;
}

inline uint32_t float_bits(float v) {
  uint32_t u;
  std::memcpy(&u, &v, 4);
  return u;
}

// exp for the alpha-blending loops (CR/forward.cu:390, CR/backward.cu:484).
// n = rint(x*log2e); r = x - n*ln2 (two-constant split); degree-6 polynomial
// in r; scale by 2^n through the exponent field.  Below -87 the result is 0,
// above 88 it is +inf, so no subnormal is ever produced.
inline float orc_expf(float x) {
  if (!(x == x)) return x;
  if (x < -87.0f) return 0.0f;
  if (x > 88.0f) return INFINITY;
  float n = nearbyintf(x * 1.44269504088896341f);
  float r = fmaf(n, -0.693145751953125f, x);
  r = fmaf(n, -1.42860682030941723212e-6f, r);
  float p = 1.9875691500e-4f;
  p = fmaf(p, r, 1.3981999507e-3f);
  p = fmaf(p, r, 8.3334519073e-3f);
  p = fmaf(p, r, 4.1665795894e-2f);
  p = fmaf(p, r, 1.6666665459e-1f);
  p = fmaf(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  p = fmaf(p, r2, r);
  p = p + 1.0f;
  int e = (int)n;
  uint32_t sb = (uint32_t)(e + 127) << 23;
  float s;
  std::memcpy(&s, &sb, 4);
  return p * s;
}

// 3x3 matrix with glm's storage and product (column vectors, m[col][row];
// DGR/third_party/glm/glm/detail/type_mat3x3.inl:486-518).
struct M3 {
  float m[3][3];
};

inline M3 m3_cols(float a0, float a1, float a2, float b0, float b1, float b2, float c0, float c1,
                  float c2) {
  M3 r;
  r.m[0][0] = a0; r.m[0][1] = a1; r.m[0][2] = a2;
  r.m[1][0] = b0; r.m[1][1] = b1; r.m[1][2] = b2;
  r.m[2][0] = c0; r.m[2][1] = c1; r.m[2][2] = c2;
  return r;
}

inline M3 m3_mul(const M3& A, const M3& B) {
  M3 R;
  for (int c = 0; c < 3; c++)
    for (int r = 0; r < 3; r++)
      R.m[c][r] = (A.m[0][r] * B.m[c][0] + A.m[1][r] * B.m[c][1]) + A.m[2][r] * B.m[c][2];
  return R;
}

inline M3 m3_T(const M3& A) {
  M3 R;
  for (int c = 0; c < 3; c++)
    for (int r = 0; r < 3; r++) R.m[c][r] = A.m[r][c];
  return R;
}

inline float dot3(const float* a, const float* b) { return (a[0] * b[0] + a[1] * b[1]) + a[2] * b[2]; }

// Row-vector point transforms (CR/auxiliary.h:112-131).  M is the 4x4 torch
// tensor as CityGS-X passes it, flattened row-major.
inline void xform4x3(const float* p, const float* M, float* o) {
  for (int k = 0; k < 3; k++) o[k] = ((M[k] * p[0] + M[4 + k] * p[1]) + M[8 + k] * p[2]) + M[12 + k];
}
inline void xform4x4(const float* p, const float* M, float* o) {
  for (int k = 0; k < 4; k++) o[k] = ((M[k] * p[0] + M[4 + k] * p[1]) + M[8 + k] * p[2]) + M[12 + k];
}
// CR/auxiliary.h:143-151
inline void xformVec4x3T(const float* v, const float* M, float* o) {
  for (int k = 0; k < 3; k++) o[k] = (M[4 * k] * v[0] + M[4 * k + 1] * v[1]) + M[4 * k + 2] * v[2];
}

// CR/auxiliary.h:52-55 (double intermediates).
inline float ndc2pix(float v, int S) { return (float)((((double)v + 1.0) * (double)S - 1.0) * 0.5); }

struct Rect {
  uint32_t x0, y0, x1, y1;
};

// CR/auxiliary.h:66-76.
inline Rect get_rect(float px, float py, int radius, uint32_t gx, uint32_t gy) {
  float rf = (float)radius;
  Rect r;
  r.x0 = std::min(gx, (uint32_t)std::max(0, f2i_sat((px - rf) / (float)TILE_X)));
  r.y0 = std::min(gy, (uint32_t)std::max(0, f2i_sat((py - rf) / (float)TILE_Y)));
  // "p.x + max_radius + BLOCK_X - 1" associates left to right in fp32.
  r.x1 = std::min(gx, (uint32_t)std::max(0, f2i_sat((((px + rf) + (float)TILE_X) - 1.0f) / (float)TILE_X)));
  r.y1 = std::min(gy, (uint32_t)std::max(0, f2i_sat((((py + rf) + (float)TILE_Y) - 1.0f) / (float)TILE_Y)));
  return r;
}

// CR/forward.cu:119-153.  Raw (un-normalised) quaternion (r,x,y,z).
inline void cov3d_from_scale_rot(const float* scale, float mod, const float* q, float* out6, M3* M_out,
                                 M3* R_out) {
  M3 S = m3_cols(1, 0, 0, 0, 1, 0, 0, 0, 1);
  S.m[0][0] = mod * scale[0];
  S.m[1][1] = mod * scale[1];
  S.m[2][2] = mod * scale[2];
  float r = q[0], x = q[1], y = q[2], z = q[3];
  M3 R = m3_cols(1.f - 2.f * (y * y + z * z), 2.f * (x * y - r * z), 2.f * (x * z + r * y),
                 2.f * (x * y + r * z), 1.f - 2.f * (x * x + z * z), 2.f * (y * z - r * x),
                 2.f * (x * z - r * y), 2.f * (y * z + r * x), 1.f - 2.f * (x * x + y * y));
  M3 M = m3_mul(S, R);
  M3 Sig = m3_mul(m3_T(M), M);
  if (out6) {
    out6[0] = Sig.m[0][0]; out6[1] = Sig.m[0][1]; out6[2] = Sig.m[0][2];
    out6[3] = Sig.m[1][1]; out6[4] = Sig.m[1][2]; out6[5] = Sig.m[2][2];
  }
  if (M_out) *M_out = M;
  if (R_out) *R_out = R;
}

struct Cov2DCtx {
  M3 T, W, Vrk;
  float t[3];  // clamped view-space mean
  float txtz, tytz, limx, limy;
  float a, b, c;
};

// CR/forward.cu:75-114 (same recomputation at CR/backward.cu:92-127).
inline void cov2d(const float* mean, float fx, float fy, float tanx, float tany, const float* c6,
                  const float* V, Cov2DCtx& o) {
  xform4x3(mean, V, o.t);
  o.limx = 1.3f * tanx;
  o.limy = 1.3f * tany;
  o.txtz = o.t[0] / o.t[2];
  o.tytz = o.t[1] / o.t[2];
  o.t[0] = fminf(o.limx, fmaxf(-o.limx, o.txtz)) * o.t[2];
  o.t[1] = fminf(o.limy, fmaxf(-o.limy, o.tytz)) * o.t[2];
  const float tz = o.t[2];
  M3 J = m3_cols(fx / tz, 0.0f, -(fx * o.t[0]) / (tz * tz), 0.0f, fy / tz, -(fy * o.t[1]) / (tz * tz), 0, 0,
                 0);
  o.W = m3_cols(V[0], V[4], V[8], V[1], V[5], V[9], V[2], V[6], V[10]);
  o.T = m3_mul(o.W, J);
  o.Vrk = m3_cols(c6[0], c6[1], c6[2], c6[1], c6[3], c6[4], c6[2], c6[4], c6[5]);
  M3 cov = m3_mul(m3_mul(m3_T(o.T), m3_T(o.Vrk)), o.T);
  o.a = cov.m[0][0] + 0.3f;
  o.b = cov.m[0][1];
  o.c = cov.m[1][1] + 0.3f;
}

// Real SH basis constants (CR/auxiliary.h:23-40).
constexpr float kC0 = 0.28209479177387814f;
constexpr float kC1 = 0.4886025119029199f;
constexpr float kC2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                          -1.0925484305920792f, 0.5462742152960396f};
constexpr float kC3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                          0.3731763325901154f,  -0.4570457994644658f, 1.445305721320277f,
                          -0.5900435899266435f};

// CR/forward.cu:21-72.  sh is (M,3) for this Gaussian; deg in 0..3.
inline void sh_to_rgb(int deg, const float* mean, const float* campos, const float* sh, float* rgb,
                      uint8_t* clamped) {
  float d[3] = {mean[0] - campos[0], mean[1] - campos[1], mean[2] - campos[2]};
  float len = sqrtf(dot3(d, d));
  float x = d[0] / len, y = d[1] / len, z = d[2] / len;
  for (int ch = 0; ch < 3; ch++) {
    auto c = [&](int k) { return sh[3 * k + ch]; };
    float res = kC0 * c(0);
    if (deg > 0) {
      res = ((res - kC1 * y * c(1)) + kC1 * z * c(2)) - kC1 * x * c(3);
      if (deg > 1) {
        float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
        res = ((((res + kC2[0] * xy * c(4)) + kC2[1] * yz * c(5)) +
                kC2[2] * (2.0f * zz - xx - yy) * c(6)) +
               kC2[3] * xz * c(7)) +
              kC2[4] * (xx - yy) * c(8);
        if (deg > 2) {
          res = ((((((res + kC3[0] * y * (3.0f * xx - yy) * c(9)) + kC3[1] * xy * z * c(10)) +
                    kC3[2] * y * (4.0f * zz - xx - yy) * c(11)) +
                   kC3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy) * c(12)) +
                  kC3[4] * x * (4.0f * zz - xx - yy) * c(13)) +
                 kC3[5] * z * (xx - yy) * c(14)) +
                kC3[6] * x * (xx - 3.0f * yy) * c(15);
        }
      }
    }
    res += 0.5f;
    clamped[ch] = res < 0.0f;
    rgb[ch] = fmaxf(res, 0.0f);
  }
}

// Geometry part shared by preprocess and the visibility prefilter
// (CR/forward.cu:183-239 and :562-616).  Returns radius (>0) when the Gaussian
// survives; writes cov6 when it is computed from scale/rotation.
struct GeomOut {
  float depth, px, py, conic[3];
  int radius;
};

inline bool geom_forward(const float* mean, const float* scale, float mod, const float* rot,
                         const float* cov_pre, const float* V, const float* PM, int W, int H, float tanx,
                         float tany, float fx, float fy, uint32_t gx, uint32_t gy, float* cov6_store,
                         GeomOut& g) {
  float ph[4], pv[3];
  xform4x4(mean, PM, ph);
  float pw = 1.0f / (ph[3] + 0.0000001f);
  float pproj[3] = {ph[0] * pw, ph[1] * pw, ph[2] * pw};
  xform4x3(mean, V, pv);
  if (pv[2] <= 0.0f) return false;  // CR/auxiliary.h:208
  float local6[6];
  const float* c6;
  if (cov_pre) {
    c6 = cov_pre;
  } else {
    float* dst = cov6_store ? cov6_store : local6;
    cov3d_from_scale_rot(scale, mod, rot, dst, nullptr, nullptr);
    c6 = dst;
  }
  Cov2DCtx cc;
  cov2d(mean, fx, fy, tanx, tany, c6, V, cc);
  float det = cc.a * cc.c - cc.b * cc.b;
  if (det == 0.0f) return false;
  float det_inv = 1.f / det;
  g.conic[0] = cc.c * det_inv;
  g.conic[1] = -cc.b * det_inv;
  g.conic[2] = cc.a * det_inv;
  float mid = 0.5f * (cc.a + cc.c);
  float root = sqrtf(fmaxf(0.1f, mid * mid - det));
  float l1 = mid + root, l2 = mid - root;
  float rad_f = ceilf(3.f * sqrtf(fmaxf(l1, l2)));
  g.px = ndc2pix(pproj[0], W);
  g.py = ndc2pix(pproj[1], H);
  g.radius = f2i_sat(rad_f);
  Rect rc = get_rect(g.px, g.py, g.radius, gx, gy);
  if ((rc.x1 - rc.x0) * (rc.y1 - rc.y0) == 0) return false;
  g.depth = pv[2];
  return true;
}

inline void grid_of(int W, int H, uint32_t& gx, uint32_t& gy) {
  gx = (uint32_t)((W + TILE_X - 1) / TILE_X);
  gy = (uint32_t)((H + TILE_Y - 1) / TILE_Y);
}

}  // namespace

extern "C" {

int oracle_num_threads() {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void oracle_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}

void oracle_expf(int n, const float* x, float* y) {
  for (int i = 0; i < n; i++) y[i] = orc_expf(x[i]);
}

// CR/rasterizer_impl.cu:39-54.
uint32_t oracle_higher_msb(uint32_t n) {
  uint32_t msb = sizeof(n) * 4;
  uint32_t step = msb;
  while (step > 1) {
    step /= 2;
    if (n >> msb)
      msb += step;
    else
      msb -= step;
  }
  if (n >> msb) msb++;
  return msb;
}

// CR/rasterizer_impl.cu:58-70, CR/auxiliary.h:193-218.
void oracle_mark_visible(int P, const float* means, const float* V, const float* PM, uint8_t* present) {
  (void)PM;
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; i++) {
    float pv[3];
    xform4x3(means + 3 * i, V, pv);
    present[i] = pv[2] > 0.0f;
  }
}

// CR/forward.cu:156-259 with the SH colour step (CR/forward.cu:21-72) switched
// back on when shs != NULL and M > 0.  Outputs must arrive zero-filled
// (DGR/rasterize_points.cu:92-104); culled Gaussians leave them untouched.
// tiles_touched (optional) is the full-grid rectangle area, the value the
// commented line CR/forward.cu:258 would store.
void oracle_preprocess_fwd(int P, int D, int M, const float* means, const float* scales, float mod,
                           const float* rots, const float* opac, const float* shs, const float* V,
                           const float* PM, const float* campos, int W, int H, float tanx, float tany,
                           int* radii, float* means2D, float* depths, float* cov3D, float* conic_opacity,
                           float* rgb, uint8_t* clamped, uint32_t* tiles_touched) {
  const float fy = H / (2.0f * tany);  // CR/rasterizer_impl.cu:371-372
  const float fx = W / (2.0f * tanx);
  uint32_t gx, gy;
  grid_of(W, H, gx, gy);
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; i++) {
    radii[i] = 0;
    if (tiles_touched) tiles_touched[i] = 0;
    GeomOut g;
    if (!geom_forward(means + 3 * i, scales + 3 * i, mod, rots + 4 * i, nullptr, V, PM, W, H, tanx, tany, fx,
                      fy, gx, gy, cov3D + 6 * i, g))
      continue;
    if (shs && M > 0) sh_to_rgb(D, means + 3 * i, campos, shs + (size_t)i * M * 3, rgb + 3 * i, clamped + 3 * i);
    depths[i] = g.depth;
    radii[i] = g.radius;
    means2D[2 * i] = g.px;
    means2D[2 * i + 1] = g.py;
    conic_opacity[4 * i + 0] = g.conic[0];
    conic_opacity[4 * i + 1] = g.conic[1];
    conic_opacity[4 * i + 2] = g.conic[2];
    conic_opacity[4 * i + 3] = opac[i];
    if (tiles_touched) {
      Rect rc = get_rect(g.px, g.py, g.radius, gx, gy);
      tiles_touched[i] = (rc.x1 - rc.x0) * (rc.y1 - rc.y0);
    }
  }
}

// CR/forward.cu:545-620.  scales/rots or cov_pre may be NULL.
void oracle_visible_filter(int P, const float* means, const float* scales, float mod, const float* rots,
                           const float* cov_pre, const float* V, const float* PM, int W, int H, float tanx,
                           float tany, int* radii) {
  const float fy = H / (2.0f * tany);
  const float fx = W / (2.0f * tanx);
  uint32_t gx, gy;
  grid_of(W, H, gx, gy);
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; i++) {
    radii[i] = 0;
    GeomOut g;
    if (geom_forward(means + 3 * i, scales ? scales + 3 * i : nullptr, mod, rots ? rots + 4 * i : nullptr,
                     cov_pre ? cov_pre + 6 * i : nullptr, V, PM, W, H, tanx, tany, fx, fy, gx, gy, nullptr, g))
      radii[i] = g.radius;
  }
}

// CR/rasterizer_impl.cu:264-288.
void oracle_tiles_touched(int P, int W, int H, const int* radii, const float* means2D,
                          const uint8_t* compute_locally, uint32_t* tiles_touched) {
  uint32_t gx, gy;
  grid_of(W, H, gx, gy);
#pragma omp parallel for schedule(dynamic, 4096)
  for (int i = 0; i < P; i++) {
    uint32_t cnt = 0;
    if (radii[i] > 0) {
      Rect rc = get_rect(means2D[2 * i], means2D[2 * i + 1], radii[i], gx, gy);
      for (uint32_t y = rc.y0; y < rc.y1; y++)
        for (uint32_t x = rc.x0; x < rc.x1; x++)
          if (compute_locally[y * gx + x]) cnt++;
    }
    tiles_touched[i] = cnt;
  }
}

// cub::DeviceScan::InclusiveSum as used at CR/rasterizer_impl.cu:648 (uint32,
// wrap-around addition).
void oracle_inclusive_sum(int P, const uint32_t* in, uint32_t* out) {
  uint32_t acc = 0;
  for (int i = 0; i < P; i++) {
    acc += in[i];
    out[i] = acc;
  }
}

// CR/rasterizer_impl.cu:74-117.
void oracle_duplicate_with_keys(int P, int W, int H, const float* means2D, const float* depths,
                                const uint32_t* offsets, const int* radii, const uint8_t* compute_locally,
                                uint64_t* keys, uint32_t* values) {
  uint32_t gx, gy;
  grid_of(W, H, gx, gy);
#pragma omp parallel for schedule(dynamic, 4096)
  for (int i = 0; i < P; i++) {
    if (radii[i] > 0) {
      uint32_t off = (i == 0) ? 0 : offsets[i - 1];
      Rect rc = get_rect(means2D[2 * i], means2D[2 * i + 1], radii[i], gx, gy);
      for (uint32_t y = rc.y0; y < rc.y1; y++)
        for (uint32_t x = rc.x0; x < rc.x1; x++)
          if (compute_locally[y * gx + x]) {
            uint64_t key = (uint64_t)(y * gx + x);
            key <<= 32;
            key |= float_bits(depths[i]);
            keys[off] = key;
            values[off] = (uint32_t)i;
            off++;
          }
    }
  }
}

// cub::DeviceRadixSort::SortPairs(keys, values, n, 0, end_bit) as used at
// CR/rasterizer_impl.cu:679-684: stable, compares only bits [0, end_bit).
void oracle_sort_pairs(int64_t n, const uint64_t* keys_in, const uint32_t* vals_in, uint64_t* keys_out,
                       uint32_t* vals_out, int end_bit) {
  std::vector<uint32_t> perm((size_t)n);
  std::iota(perm.begin(), perm.end(), 0u);
  const uint64_t mask = end_bit >= 64 ? ~0ull : ((1ull << end_bit) - 1ull);
  std::stable_sort(perm.begin(), perm.end(),
                   [&](uint32_t a, uint32_t b) { return (keys_in[a] & mask) < (keys_in[b] & mask); });
  for (int64_t i = 0; i < n; i++) {
    keys_out[i] = keys_in[perm[i]];
    vals_out[i] = vals_in[perm[i]];
  }
}

// 32-bit key variant (KNN/simple_knn.cu:210-213).
void oracle_sort_pairs_u32(int64_t n, const uint32_t* keys_in, const uint32_t* vals_in, uint32_t* keys_out,
                           uint32_t* vals_out) {
  std::vector<uint32_t> perm((size_t)n);
  std::iota(perm.begin(), perm.end(), 0u);
  std::stable_sort(perm.begin(), perm.end(), [&](uint32_t a, uint32_t b) { return keys_in[a] < keys_in[b]; });
  for (int64_t i = 0; i < n; i++) {
    keys_out[i] = keys_in[perm[i]];
    vals_out[i] = vals_in[perm[i]];
  }
}

// CR/rasterizer_impl.cu:122-144 preceded by the memset at :687.  ranges is
// (T,2) uint32.
void oracle_tile_ranges(int64_t L, const uint64_t* keys, int T, uint32_t* ranges) {
  std::memset(ranges, 0, sizeof(uint32_t) * 2 * (size_t)T);
  for (int64_t i = 0; i < L; i++) {
    uint32_t cur = (uint32_t)(keys[i] >> 32);
    if (i == 0)
      ranges[2 * cur] = 0;
    else {
      uint32_t prev = (uint32_t)(keys[i - 1] >> 32);
      if (cur != prev) {
        ranges[2 * prev + 1] = (uint32_t)i;
        ranges[2 * cur] = (uint32_t)i;
      }
    }
    if (i == L - 1) ranges[2 * cur + 1] = (uint32_t)L;
  }
}

// CR/forward.cu:264-437, one pixel at a time (no batching: the block-level
// early exit and shared-memory staging change work, not results).
// focal/cx/cy as computed at DGR/rasterize_points.cu:328-342.
void oracle_render_fwd(int W, int H, float tanx, float tany, const uint32_t* ranges, const uint32_t* point_list,
                       const float* means2D, const float* rgb, const float* all_map,
                       const float* conic_opacity, const uint8_t* compute_locally, const float* bg,
                       int render_geo, float* final_T, uint32_t* n_contrib, uint32_t* n_contrib2loss,
                       float* out_color, int* out_observe, float* out_all_map, float* out_plane_depth) {
  const float fy = H / (2.0f * tany);
  const float fx = W / (2.0f * tanx);
  const float cx = (float)(W * 0.5f), cy = (float)(H * 0.5f);
  uint32_t gx, gy;
  grid_of(W, H, gx, gy);
  const size_t HW = (size_t)H * W;
  const int T = (int)(gx * gy);
#pragma omp parallel for schedule(dynamic, 1)
  for (int tile = 0; tile < T; tile++) {
    if (!compute_locally[tile]) continue;
    const uint32_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
    const int tx0 = (tile % (int)gx) * TILE_X, ty0 = (tile / (int)gx) * TILE_Y;
    for (int ly = 0; ly < TILE_Y; ly++)
      for (int lx = 0; lx < TILE_X; lx++) {
        const int px = tx0 + lx, py = ty0 + ly;
        if (px >= W || py >= H) continue;
        const size_t pid = (size_t)W * py + px;
        const float pfx = (float)px, pfy = (float)py;
        const float rayx = (pfx - cx) / fx, rayy = (pfy - cy) / fy;
        float Tr = 1.0f;
        uint32_t contributor = 0, last = 0, n2l = 0;
        float C[N_RGB] = {0, 0, 0};
        float Mp[N_MAP] = {0, 0, 0, 0, 0};
        for (uint32_t k = r0; k < r1; k++) {
          contributor++;
          const uint32_t g = point_list[k];
          const float dx = means2D[2 * g] - pfx, dy = means2D[2 * g + 1] - pfy;
          const float* co = conic_opacity + 4 * (size_t)g;
          const float power = -0.5f * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
          if (power > 0.0f) continue;
          const float alpha = fminf(0.99f, co[3] * orc_expf(power));
          if (alpha < 1.0f / 255.0f) continue;
          const float test_T = Tr * (1 - alpha);
          if (test_T < 0.0001f) break;
          n2l++;
          // weight first, then one fused multiply-add per channel (see the header note on accumulation)
          const float wgt = alpha * Tr;
          for (int ch = 0; ch < N_RGB; ch++) C[ch] = fmaf(rgb[3 * (size_t)g + ch], wgt, C[ch]);
          if (render_geo)
            for (int ch = 0; ch < N_MAP; ch++) Mp[ch] = fmaf(all_map[5 * (size_t)g + ch], wgt, Mp[ch]);
          if (Tr > 0.5f) {
#pragma omp atomic
            out_observe[g] += 1;
          }
          Tr = test_T;
          last = contributor;
        }
        final_T[pid] = Tr;
        n_contrib[pid] = last;
        n_contrib2loss[pid] = n2l;
        for (int ch = 0; ch < N_RGB; ch++) out_color[ch * HW + pid] = C[ch] + Tr * bg[ch];
        if (render_geo) {
          for (int ch = 0; ch < N_MAP; ch++) out_all_map[ch * HW + pid] = Mp[ch];
          const float den_f = (Mp[0] * rayx + Mp[1] * rayy) + Mp[2];
          out_plane_depth[pid] = (float)((double)Mp[4] / -((double)den_f + 1.0e-8));
        }
      }
  }
}

// No counterpart in the reference (an additional output of the blend, defined here): per pixel the view-space
// depth of the Gaussian that blends with the largest weight alpha * T, the front-most among equal weights, 0 where
// nothing blends.  Same walk, tests and arithmetic as oracle_render_fwd (CR/forward.cu:330-437).
void oracle_max_weight_depth(int W, int H, const uint32_t* ranges, const uint32_t* point_list, const float* means2D,
                             const float* conic_opacity, const float* depths, const uint8_t* compute_locally,
                             float* out) {
  uint32_t gx, gy;
  grid_of(W, H, gx, gy);
  const int T = (int)(gx * gy);
#pragma omp parallel for schedule(dynamic, 1)
  for (int tile = 0; tile < T; tile++) {
    if (!compute_locally[tile]) continue;
    const uint32_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
    const int tx0 = (tile % (int)gx) * TILE_X, ty0 = (tile / (int)gx) * TILE_Y;
    for (int ly = 0; ly < TILE_Y; ly++)
      for (int lx = 0; lx < TILE_X; lx++) {
        const int px = tx0 + lx, py = ty0 + ly;
        if (px >= W || py >= H) continue;
        const float pfx = (float)px, pfy = (float)py;
        float Tr = 1.0f, best_w = 0.0f, best_d = 0.0f;
        for (uint32_t k = r0; k < r1; k++) {
          const uint32_t g = point_list[k];
          const float dx = means2D[2 * g] - pfx, dy = means2D[2 * g + 1] - pfy;
          const float* co = conic_opacity + 4 * (size_t)g;
          const float power = -0.5f * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
          if (power > 0.0f) continue;
          const float alpha = fminf(0.99f, co[3] * orc_expf(power));
          if (alpha < 1.0f / 255.0f) continue;
          const float test_T = Tr * (1 - alpha);
          if (test_T < 0.0001f) break;
          const float wgt = alpha * Tr;
          if (wgt > best_w) {
            best_w = wgt;
            best_d = depths[g];
          }
          Tr = test_T;
        }
        out[(size_t)W * py + px] = best_d;
      }
  }
}

// CR/rasterizer_impl.cu:219-262, launched :731-752.  Outputs arrive zeroed
// (DGR/rasterize_points.cu:315-317); non-local tiles keep n_consider and
// n_contrib at zero, n_render is written for every tile.
void oracle_tile_stats(int W, int H, const uint32_t* ranges, const uint32_t* n_contrib_px,
                       const uint32_t* n_contrib2loss_px, const uint8_t* compute_locally, int* n_render,
                       int* n_consider, int* n_contrib) {
  uint32_t gx, gy;
  grid_of(W, H, gx, gy);
  for (uint32_t t = 0; t < gx * gy; t++) {
    n_render[t] = (int)(ranges[2 * t + 1] - ranges[2 * t]);
    if (!compute_locally[t]) continue;
    int s1 = 0, s2 = 0;
    const int tx0 = (int)(t % gx) * TILE_X, ty0 = (int)(t / gx) * TILE_Y;
    for (int ly = 0; ly < TILE_Y; ly++)
      for (int lx = 0; lx < TILE_X; lx++) {
        int px = tx0 + lx, py = ty0 + ly;
        if (px >= W || py >= H) continue;
        s1 += (int)n_contrib_px[(size_t)W * py + px];
        s2 += (int)n_contrib2loss_px[(size_t)W * py + px];
      }
    n_consider[t] = s1;
    n_contrib[t] = s2;
  }
}

// CR/backward.cu:324-567.  Per-pixel arithmetic in fp32 as written there; the
// per-Gaussian sums (atomicAdd targets in the reference) are accumulated in
// double and rounded once, which makes this the order-independent tolerance
// oracle.  Gradient outputs (fp32): dL_dmean2D (P,3), dL_dmean2D_abs (P,3),
// dL_dconic (P,4) laid out as the (P,2,2) tensor of DGR/rasterize_points.cu:394
// [x, y, unused, w], dL_dopacity (P), dL_dcolors (P,3), dL_dall_map (P,5).
void oracle_render_bwd(int P, int W, int H, float tanx, float tany, const float* bg, const uint32_t* ranges,
                       const uint32_t* point_list, const float* means2D, const float* conic_opacity,
                       const float* rgb, const float* all_map, const float* all_map_pixels,
                       const float* final_T, const uint32_t* n_contrib, const uint8_t* compute_locally,
                       const float* dL_dpix, const float* dL_dout_all_map, const float* dL_dout_plane_depth,
                       int render_geo, float* dL_dmean2D, float* dL_dmean2D_abs, float* dL_dconic,
                       float* dL_dopacity, float* dL_dcolors, float* dL_dall_map) {
  const float fy = H / (2.0f * tany);
  const float fx = W / (2.0f * tanx);
  uint32_t gx, gy;
  grid_of(W, H, gx, gy);
  const size_t HW = (size_t)H * W;
  const int T = (int)(gx * gy);
  // 16 accumulators per Gaussian: mean2D.xy, abs.xy, conic x,y,w, opacity, rgb(3), map(5)
  std::vector<double> acc((size_t)P * 16, 0.0);
  const float ddelx_dx = (float)(0.5 * W), ddely_dy = (float)(0.5 * H);
#pragma omp parallel for schedule(dynamic, 1)
  for (int tile = 0; tile < T; tile++) {
    if (!compute_locally[tile]) continue;
    const uint32_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
    const int tx0 = (tile % (int)gx) * TILE_X, ty0 = (tile / (int)gx) * TILE_Y;
    for (int ly = 0; ly < TILE_Y; ly++)
      for (int lx = 0; lx < TILE_X; lx++) {
        const int px = tx0 + lx, py = ty0 + ly;
        if (px >= W || py >= H) continue;
        const size_t pid = (size_t)W * py + px;
        const float pfx = (float)px, pfy = (float)py;
        const float rayx = (float)(((double)pfx - W * 0.5) / (double)fx);
        const float rayy = (float)(((double)pfy - H * 0.5) / (double)fy);
        const float T_final = final_T[pid];
        float Tr = T_final;
        uint32_t contributor = r1 - r0;
        const int last_contributor = (int)n_contrib[pid];
        float accum_rec[N_RGB] = {0, 0, 0}, accum_map[N_MAP] = {0, 0, 0, 0, 0};
        float gpix[N_RGB], gmap[N_MAP] = {0, 0, 0, 0, 0};
        for (int ch = 0; ch < N_RGB; ch++) gpix[ch] = dL_dpix[ch * HW + pid];
        if (render_geo) {
          for (int ch = 0; ch < N_MAP; ch++) gmap[ch] = dL_dout_all_map[ch * HW + pid];
          const float nx = all_map_pixels[pid], ny = all_map_pixels[HW + pid], nz = all_map_pixels[2 * HW + pid];
          const float dist = all_map_pixels[4 * HW + pid];
          const float tmp = (float)((double)((nx * rayx + ny * rayy) + nz) + 1.0e-8);
          const float gd = dL_dout_plane_depth[pid];
          gmap[N_MAP - 1] += (-gd / tmp);
          gmap[0] += gd * (dist / (tmp * tmp) * rayx);
          gmap[1] += gd * (dist / (tmp * tmp) * rayy);
          gmap[2] += gd * (dist / (tmp * tmp));
        }
        float last_alpha = 0;
        float last_color[N_RGB] = {0, 0, 0}, last_map[N_MAP] = {0, 0, 0, 0, 0};
        for (uint32_t k = r1; k-- > r0;) {
          contributor--;
          if ((int64_t)contributor >= (int64_t)last_contributor) continue;
          const uint32_t g = point_list[k];
          const float dx = means2D[2 * g] - pfx, dy = means2D[2 * g + 1] - pfy;
          const float* co = conic_opacity + 4 * (size_t)g;
          const float power = -0.5f * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
          if (power > 0.0f) continue;
          const float G = orc_expf(power);
          const float alpha = fminf(0.99f, co[3] * G);
          if (alpha < 1.0f / 255.0f) continue;
          const float inv1ma = 1.f / (1.f - alpha);
          Tr = Tr * inv1ma;
          const float w = alpha * Tr;
          double* a = acc.data() + (size_t)g * 16;
          float dL_dalpha = 0.0f;
          for (int ch = 0; ch < N_RGB; ch++) {
            const float c = rgb[3 * (size_t)g + ch];
            accum_rec[ch] = fmaf(last_alpha, last_color[ch], (1.f - last_alpha) * accum_rec[ch]);
            last_color[ch] = c;
            dL_dalpha = fmaf(c - accum_rec[ch], gpix[ch], dL_dalpha);
            const double v = (double)(w * gpix[ch]);
#pragma omp atomic
            a[8 + ch] += v;
          }
          if (render_geo)
            for (int ch = 0; ch < N_MAP; ch++) {
              const float c = all_map[5 * (size_t)g + ch];
              accum_map[ch] = fmaf(last_alpha, last_map[ch], (1.f - last_alpha) * accum_map[ch]);
              last_map[ch] = c;
              dL_dalpha = fmaf(c - accum_map[ch], gmap[ch], dL_dalpha);
              const double v = (double)(w * gmap[ch]);
#pragma omp atomic
              a[11 + ch] += v;
            }
          last_alpha = alpha;
          float bg_dot = 0;
          for (int ch = 0; ch < N_RGB; ch++) bg_dot += bg[ch] * gpix[ch];
          dL_dalpha = fmaf(dL_dalpha, Tr, -((T_final * bg_dot) * inv1ma));
          const float dL_dG = co[3] * dL_dalpha;
          const float gdx = G * dx, gdy = G * dy;
          const float dG_ddelx = -gdx * co[0] - gdy * co[1];
          const float dG_ddely = -gdy * co[2] - gdx * co[1];
          const float mx = dL_dG * dG_ddelx * ddelx_dx, my = dL_dG * dG_ddely * ddely_dy;
          const double vals[8] = {(double)mx,
                                  (double)my,
                                  (double)fabsf(mx),
                                  (double)fabsf(my),
                                  (double)(-0.5f * gdx * dx * dL_dG),
                                  (double)(-0.5f * gdx * dy * dL_dG),
                                  (double)(-0.5f * gdy * dy * dL_dG),
                                  (double)(G * dL_dalpha)};
          for (int q = 0; q < 8; q++) {
#pragma omp atomic
            a[q] += vals[q];
          }
        }
      }
  }
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; i++) {
    const double* a = acc.data() + (size_t)i * 16;
    dL_dmean2D[3 * i] = (float)a[0];
    dL_dmean2D[3 * i + 1] = (float)a[1];
    dL_dmean2D[3 * i + 2] = 0.0f;
    dL_dmean2D_abs[3 * i] = (float)a[2];
    dL_dmean2D_abs[3 * i + 1] = (float)a[3];
    dL_dmean2D_abs[3 * i + 2] = 0.0f;
    dL_dconic[4 * i] = (float)a[4];
    dL_dconic[4 * i + 1] = (float)a[5];
    dL_dconic[4 * i + 2] = 0.0f;
    dL_dconic[4 * i + 3] = (float)a[6];
    dL_dopacity[i] = (float)a[7];
    for (int ch = 0; ch < 3; ch++) dL_dcolors[3 * i + ch] = (float)a[8 + ch];
    for (int ch = 0; ch < 5; ch++) dL_dall_map[5 * i + ch] = (float)a[11 + ch];
  }
}

// CR/backward.cu:69-199 then :271-321 with :203-266 (BACKWARD::preprocess,
// :570-634), plus the SH colour backward that the reference left as a stub
// (CR/backward.cu:21-64): derivative of CR/forward.cu:21-72 with the clamp
// mask and the direction normalisation (CR/auxiliary.h:161-171).
// dL_dconic is (P,4) laid out [x, y, unused, w] (the (P,2,2) tensor of
// DGR/rasterize_points.cu:181-189).  dL_dmean2D is (P,3).  Outputs arrive
// zeroed.  dL_dsh may be NULL (reference-compatible mode: no SH).
void oracle_preprocess_bwd(int P, int D, int M, const float* means, const int* radii, const float* shs,
                           const uint8_t* clamped, const float* scales, const float* rots, float mod,
                           const float* cov3D, const float* V, const float* PM, int W, int H, float tanx,
                           float tany, const float* campos, const float* dL_dmean2D, const float* dL_dconic,
                           const float* dL_dcolor, float* dL_dmean3D, float* dL_dcov3D, float* dL_dsh,
                           float* dL_dscale, float* dL_drot) {
  const float h_y = H / (2.0f * tany);
  const float h_x = W / (2.0f * tanx);
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; i++) {
    if (!(radii[i] > 0)) continue;
    const float* mean = means + 3 * i;
    // ---- conic -> cov2D -> cov3D and mean (CR/backward.cu:69-199)
    Cov2DCtx cc;
    cov2d(mean, h_x, h_y, tanx, tany, cov3D + 6 * i, V, cc);
    const float gcx = dL_dconic[4 * i], gcy = dL_dconic[4 * i + 1], gcz = dL_dconic[4 * i + 3];
    const float x_mul = (cc.txtz < -cc.limx || cc.txtz > cc.limx) ? 0.f : 1.f;
    const float y_mul = (cc.tytz < -cc.limy || cc.tytz > cc.limy) ? 0.f : 1.f;
    const float a = cc.a, b = cc.b, c = cc.c;
    const float denom = a * c - b * b;
    float dL_da = 0, dL_db = 0, dL_dc = 0;
    const float denom2inv = 1.0f / ((denom * denom) + 0.0000001f);
    const M3& T = cc.T;
    const M3& Vr = cc.Vrk;
    float* gc = dL_dcov3D + 6 * i;
    if (denom2inv != 0) {
      dL_da = denom2inv * ((-c * c * gcx + 2 * b * c * gcy) + (denom - a * c) * gcz);
      dL_dc = denom2inv * ((-a * a * gcz + 2 * a * b * gcy) + (denom - a * c) * gcx);
      dL_db = denom2inv * 2 * ((b * c * gcx - (denom + 2 * b * b) * gcy) + a * b * gcz);
      gc[0] = (T.m[0][0] * T.m[0][0] * dL_da + T.m[0][0] * T.m[1][0] * dL_db) + T.m[1][0] * T.m[1][0] * dL_dc;
      gc[3] = (T.m[0][1] * T.m[0][1] * dL_da + T.m[0][1] * T.m[1][1] * dL_db) + T.m[1][1] * T.m[1][1] * dL_dc;
      gc[5] = (T.m[0][2] * T.m[0][2] * dL_da + T.m[0][2] * T.m[1][2] * dL_db) + T.m[1][2] * T.m[1][2] * dL_dc;
      gc[1] = (2 * T.m[0][0] * T.m[0][1] * dL_da + (T.m[0][0] * T.m[1][1] + T.m[0][1] * T.m[1][0]) * dL_db) +
              2 * T.m[1][0] * T.m[1][1] * dL_dc;
      gc[2] = (2 * T.m[0][0] * T.m[0][2] * dL_da + (T.m[0][0] * T.m[1][2] + T.m[0][2] * T.m[1][0]) * dL_db) +
              2 * T.m[1][0] * T.m[1][2] * dL_dc;
      gc[4] = (2 * T.m[0][2] * T.m[0][1] * dL_da + (T.m[0][1] * T.m[1][2] + T.m[0][2] * T.m[1][1]) * dL_db) +
              2 * T.m[1][1] * T.m[1][2] * dL_dc;
    } else {
      for (int k = 0; k < 6; k++) gc[k] = 0;
    }
    // rows of (T Vrk): u0[k] = sum_j T[0][j] Vrk[k][j], u1 likewise
    float u0[3], u1[3];
    for (int k = 0; k < 3; k++) {
      u0[k] = (T.m[0][0] * Vr.m[k][0] + T.m[0][1] * Vr.m[k][1]) + T.m[0][2] * Vr.m[k][2];
      u1[k] = (T.m[1][0] * Vr.m[k][0] + T.m[1][1] * Vr.m[k][1]) + T.m[1][2] * Vr.m[k][2];
    }
    float dT0[3], dT1[3];
    for (int k = 0; k < 3; k++) {
      dT0[k] = 2 * u0[k] * dL_da + u1[k] * dL_db;
      dT1[k] = 2 * u1[k] * dL_dc + u0[k] * dL_db;
    }
    const M3& Wm = cc.W;
    const float dJ00 = (Wm.m[0][0] * dT0[0] + Wm.m[0][1] * dT0[1]) + Wm.m[0][2] * dT0[2];
    const float dJ02 = (Wm.m[2][0] * dT0[0] + Wm.m[2][1] * dT0[1]) + Wm.m[2][2] * dT0[2];
    const float dJ11 = (Wm.m[1][0] * dT1[0] + Wm.m[1][1] * dT1[1]) + Wm.m[1][2] * dT1[2];
    const float dJ12 = (Wm.m[2][0] * dT1[0] + Wm.m[2][1] * dT1[1]) + Wm.m[2][2] * dT1[2];
    const float tz = 1.f / cc.t[2];
    const float tz2 = tz * tz;
    const float tz3 = tz2 * tz;
    float dt[3];
    dt[0] = x_mul * -h_x * tz2 * dJ02;
    dt[1] = y_mul * -h_y * tz2 * dJ12;
    dt[2] = ((-h_x * tz2 * dJ00 - h_y * tz2 * dJ11) + (2 * h_x * cc.t[0]) * tz3 * dJ02) +
            (2 * h_y * cc.t[1]) * tz3 * dJ12;
    float gm[3];
    xformVec4x3T(dt, V, gm);  // assignment, CR/backward.cu:198

    // ---- mean2D -> mean3D through the projection (CR/backward.cu:296-312)
    float mh[4];
    xform4x4(mean, PM, mh);
    const float m_w = 1.0f / (mh[3] + 0.0000001f);
    const float mul1 = (((PM[0] * mean[0] + PM[4] * mean[1]) + PM[8] * mean[2]) + PM[12]) * m_w * m_w;
    const float mul2 = (((PM[1] * mean[0] + PM[5] * mean[1]) + PM[9] * mean[2]) + PM[13]) * m_w * m_w;
    const float g2x = dL_dmean2D[3 * i], g2y = dL_dmean2D[3 * i + 1];
    gm[0] += (PM[0] * m_w - PM[3] * mul1) * g2x + (PM[1] * m_w - PM[3] * mul2) * g2y;
    gm[1] += (PM[4] * m_w - PM[7] * mul1) * g2x + (PM[5] * m_w - PM[7] * mul2) * g2y;
    gm[2] += (PM[8] * m_w - PM[11] * mul1) * g2x + (PM[9] * m_w - PM[11] * mul2) * g2y;

    // ---- colour -> SH and view direction (north-star SH mode only)
    if (shs && M > 0 && dL_dsh) {
      const float* sh = shs + (size_t)i * M * 3;
      float* gsh = dL_dsh + (size_t)i * M * 3;
      float d0[3] = {mean[0] - campos[0], mean[1] - campos[1], mean[2] - campos[2]};
      const float len = sqrtf(dot3(d0, d0));
      const float x = d0[0] / len, y = d0[1] / len, z = d0[2] / len;
      float gr[3];
      for (int ch = 0; ch < 3; ch++) gr[ch] = dL_dcolor[3 * i + ch] * (clamped[3 * i + ch] ? 0.f : 1.f);
      float dRdx[3] = {0, 0, 0}, dRdy[3] = {0, 0, 0}, dRdz[3] = {0, 0, 0};
      auto S = [&](int k, int ch) { return sh[3 * k + ch]; };
      auto put = [&](int k, float basis) {
        for (int ch = 0; ch < 3; ch++) gsh[3 * k + ch] = basis * gr[ch];
      };
      put(0, kC0);
      if (D > 0) {
        put(1, -kC1 * y);
        put(2, kC1 * z);
        put(3, -kC1 * x);
        for (int ch = 0; ch < 3; ch++) {
          dRdx[ch] = -kC1 * S(3, ch);
          dRdy[ch] = -kC1 * S(1, ch);
          dRdz[ch] = kC1 * S(2, ch);
        }
        if (D > 1) {
          const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
          put(4, kC2[0] * xy);
          put(5, kC2[1] * yz);
          put(6, kC2[2] * (2.f * zz - xx - yy));
          put(7, kC2[3] * xz);
          put(8, kC2[4] * (xx - yy));
          for (int ch = 0; ch < 3; ch++) {
            dRdx[ch] += kC2[0] * y * S(4, ch) + kC2[2] * 2.f * -x * S(6, ch) + kC2[3] * z * S(7, ch) +
                        kC2[4] * 2.f * x * S(8, ch);
            dRdy[ch] += kC2[0] * x * S(4, ch) + kC2[1] * z * S(5, ch) + kC2[2] * 2.f * -y * S(6, ch) +
                        kC2[4] * 2.f * -y * S(8, ch);
            dRdz[ch] += kC2[1] * y * S(5, ch) + kC2[2] * 2.f * 2.f * z * S(6, ch) + kC2[3] * x * S(7, ch);
          }
          if (D > 2) {
            put(9, kC3[0] * y * (3.f * xx - yy));
            put(10, kC3[1] * xy * z);
            put(11, kC3[2] * y * (4.f * zz - xx - yy));
            put(12, kC3[3] * z * (2.f * zz - 3.f * xx - 3.f * yy));
            put(13, kC3[4] * x * (4.f * zz - xx - yy));
            put(14, kC3[5] * z * (xx - yy));
            put(15, kC3[6] * x * (xx - 3.f * yy));
            for (int ch = 0; ch < 3; ch++) {
              dRdx[ch] += kC3[0] * S(9, ch) * 3.f * 2.f * xy + kC3[1] * S(10, ch) * yz +
                          kC3[2] * S(11, ch) * -2.f * xy + kC3[3] * S(12, ch) * -3.f * 2.f * xz +
                          kC3[4] * S(13, ch) * (-3.f * xx + 4.f * zz - yy) + kC3[5] * S(14, ch) * 2.f * xz +
                          kC3[6] * S(15, ch) * 3.f * (xx - yy);
              dRdy[ch] += kC3[0] * S(9, ch) * 3.f * (xx - yy) + kC3[1] * S(10, ch) * xz +
                          kC3[2] * S(11, ch) * (-3.f * yy + 4.f * zz - xx) + kC3[3] * S(12, ch) * -3.f * 2.f * yz +
                          kC3[4] * S(13, ch) * -2.f * xy + kC3[5] * S(14, ch) * -2.f * yz +
                          kC3[6] * S(15, ch) * -3.f * 2.f * xy;
              dRdz[ch] += kC3[1] * S(10, ch) * xy + kC3[2] * S(11, ch) * 4.f * 2.f * yz +
                          kC3[3] * S(12, ch) * 3.f * (2.f * zz - xx - yy) + kC3[4] * S(13, ch) * 4.f * 2.f * xz +
                          kC3[5] * S(14, ch) * (xx - yy);
            }
          }
        }
      }
      const float gdir[3] = {dot3(dRdx, gr), dot3(dRdy, gr), dot3(dRdz, gr)};
      // d(normalize(v))/dv applied to gdir (CR/auxiliary.h:161-171)
      const float s2 = dot3(d0, d0);
      const float inv32 = 1.0f / sqrtf(s2 * s2 * s2);
      gm[0] += ((s2 - d0[0] * d0[0]) * gdir[0] - d0[1] * d0[0] * gdir[1] - d0[2] * d0[0] * gdir[2]) * inv32;
      gm[1] += (-d0[0] * d0[1] * gdir[0] + (s2 - d0[1] * d0[1]) * gdir[1] - d0[2] * d0[1] * gdir[2]) * inv32;
      gm[2] += (-d0[0] * d0[2] * gdir[0] - d0[1] * d0[2] * gdir[1] + (s2 - d0[2] * d0[2]) * gdir[2]) * inv32;
    }
    dL_dmean3D[3 * i] = gm[0];
    dL_dmean3D[3 * i + 1] = gm[1];
    dL_dmean3D[3 * i + 2] = gm[2];

    // ---- cov3D -> scale, rotation (CR/backward.cu:203-266)
    if (scales) {
      M3 Mm, R;
      cov3d_from_scale_rot(scales + 3 * i, mod, rots + 4 * i, nullptr, &Mm, &R);
      const float s[3] = {mod * scales[3 * i], mod * scales[3 * i + 1], mod * scales[3 * i + 2]};
      M3 dSig = m3_cols(gc[0], 0.5f * gc[1], 0.5f * gc[2], 0.5f * gc[1], gc[3], 0.5f * gc[4], 0.5f * gc[2],
                        0.5f * gc[4], gc[5]);
      M3 M2;
      for (int cI = 0; cI < 3; cI++)
        for (int rI = 0; rI < 3; rI++) M2.m[cI][rI] = 2.0f * Mm.m[cI][rI];
      M3 dM = m3_mul(M2, dSig);
      M3 Rt = m3_T(R);
      M3 dMt = m3_T(dM);
      dL_dscale[3 * i] = dot3(Rt.m[0], dMt.m[0]);
      dL_dscale[3 * i + 1] = dot3(Rt.m[1], dMt.m[1]);
      dL_dscale[3 * i + 2] = dot3(Rt.m[2], dMt.m[2]);
      for (int k = 0; k < 3; k++) {
        dMt.m[0][k] *= s[0];
        dMt.m[1][k] *= s[1];
        dMt.m[2][k] *= s[2];
      }
      const float r = rots[4 * i], x = rots[4 * i + 1], y = rots[4 * i + 2], z = rots[4 * i + 3];
      float* gq = dL_drot + 4 * i;
      gq[0] = (2 * z * (dMt.m[0][1] - dMt.m[1][0]) + 2 * y * (dMt.m[2][0] - dMt.m[0][2])) +
              2 * x * (dMt.m[1][2] - dMt.m[2][1]);
      gq[1] = ((2 * y * (dMt.m[1][0] + dMt.m[0][1]) + 2 * z * (dMt.m[2][0] + dMt.m[0][2])) +
               2 * r * (dMt.m[1][2] - dMt.m[2][1])) -
              4 * x * (dMt.m[2][2] + dMt.m[1][1]);
      gq[2] = ((2 * x * (dMt.m[1][0] + dMt.m[0][1]) + 2 * r * (dMt.m[2][0] - dMt.m[0][2])) +
               2 * z * (dMt.m[1][2] + dMt.m[2][1])) -
              4 * y * (dMt.m[2][2] + dMt.m[0][0]);
      gq[3] = ((2 * r * (dMt.m[0][1] - dMt.m[1][0]) + 2 * x * (dMt.m[2][0] + dMt.m[0][2])) +
               2 * y * (dMt.m[1][2] + dMt.m[2][1])) -
              4 * z * (dMt.m[1][1] + dMt.m[0][0]);
    }
  }
}

// KNN/simple_knn.cu:185-221 (distCUDA2): mean of the squared distances to
// the three nearest other points.
void oracle_knn_dist2(int P, const float* pts, float* out) {
  if (P <= 0) return;
  float mn[3] = {0, 0, 0}, mx[3] = {0, 0, 0};  // reduce init {0,0,0}, KNN/simple_knn.cu:191
  for (int i = 0; i < P; i++)
    for (int k = 0; k < 3; k++) {
      mn[k] = fminf(mn[k], pts[3 * i + k]);
      mx[k] = fmaxf(mx[k], pts[3 * i + k]);
    }
  auto prep = [](uint32_t x) {  // KNN/simple_knn.cu:45-52
    x = (x | (x << 16)) & 0x030000FF;
    x = (x | (x << 8)) & 0x0300F00F;
    x = (x | (x << 4)) & 0x030C30C3;
    x = (x | (x << 2)) & 0x09249249;
    return x;
  };
  std::vector<uint32_t> code(P), idx(P), code_s(P), idx_s(P);
#pragma omp parallel for schedule(static)
  for (int i = 0; i < P; i++) {
    uint32_t c[3];
    for (int k = 0; k < 3; k++)
      c[k] = prep(f2u_sat(((pts[3 * i + k] - mn[k]) / (mx[k] - mn[k])) * (float)((1 << 10) - 1)));
    code[i] = c[0] | (c[1] << 1) | (c[2] << 2);
    idx[i] = (uint32_t)i;
  }
  oracle_sort_pairs_u32(P, code.data(), idx.data(), code_s.data(), idx_s.data());
  const int nb = (P + KNN_BOX - 1) / KNN_BOX;
  std::vector<float> bmin((size_t)nb * 3), bmax((size_t)nb * 3);
  for (int b = 0; b < nb; b++) {  // KNN/simple_knn.cu:78-117
    float lo[3] = {FLT_MAX, FLT_MAX, FLT_MAX}, hi[3] = {-FLT_MAX, -FLT_MAX, -FLT_MAX};
    for (int i = b * KNN_BOX; i < std::min(P, (b + 1) * KNN_BOX); i++)
      for (int k = 0; k < 3; k++) {
        lo[k] = fminf(lo[k], pts[3 * idx_s[i] + k]);
        hi[k] = fmaxf(hi[k], pts[3 * idx_s[i] + k]);
      }
    for (int k = 0; k < 3; k++) {
      bmin[3 * b + k] = lo[k];
      bmax[3 * b + k] = hi[k];
    }
  }
  auto upd = [](const float* ref, const float* p, float* knn) {  // KNN/simple_knn.cu:131-145
    float d[3] = {p[0] - ref[0], p[1] - ref[1], p[2] - ref[2]};
    float dist = (d[0] * d[0] + d[1] * d[1]) + d[2] * d[2];
    for (int j = 0; j < 3; j++)
      if (knn[j] > dist) {
        float t = knn[j];
        knn[j] = dist;
        dist = t;
      }
  };
#pragma omp parallel for schedule(dynamic, 256)
  for (int k = 0; k < P; k++) {  // KNN/simple_knn.cu:147-183
    const float* p = pts + 3 * idx_s[k];
    float best[3] = {FLT_MAX, FLT_MAX, FLT_MAX};
    for (int i = std::max(0, k - 3); i <= std::min(P - 1, k + 3); i++) {
      if (i == k) continue;
      upd(p, pts + 3 * idx_s[i], best);
    }
    const float reject = best[2];
    best[0] = best[1] = best[2] = FLT_MAX;
    for (int b = 0; b < nb; b++) {
      float diff[3] = {0, 0, 0};  // KNN/simple_knn.cu:119-129
      for (int c = 0; c < 3; c++)
        if (p[c] < bmin[3 * b + c] || p[c] > bmax[3 * b + c])
          diff[c] = fminf(fabsf(p[c] - bmin[3 * b + c]), fabsf(p[c] - bmax[3 * b + c]));
      const float dist = (diff[0] * diff[0] + diff[1] * diff[1]) + diff[2] * diff[2];
      if (dist > reject || dist > best[2]) continue;
      for (int i = b * KNN_BOX; i < std::min(P, (b + 1) * KNN_BOX); i++) {
        if (i == k) continue;
        upd(p, pts + 3 * idx_s[i], best);
      }
    }
    out[idx_s[k]] = ((best[0] + best[1]) + best[2]) / 3.0f;
  }
}

// Morton code of one point, exposed for known-answer tests
// (KNN/simple_knn.cu:45-61).
uint32_t oracle_morton(const float* p, const float* mn, const float* mx) {
  uint32_t c[3];
  for (int k = 0; k < 3; k++) {
    uint32_t x = f2u_sat(((p[k] - mn[k]) / (mx[k] - mn[k])) * (float)((1 << 10) - 1));
    x = (x | (x << 16)) & 0x030000FF;
    x = (x | (x << 8)) & 0x0300F00F;
    x = (x | (x << 4)) & 0x030C30C3;
    x = (x | (x << 2)) & 0x09249249;
    c[k] = x;
  }
  return c[0] | (c[1] << 1) | (c[2] << 2);
}


// ---------------------------------------------------------------------------
// Per-Gaussian geometry channels handed to the blend ("all_map"): the caller's
// torch code at gaussian_renderer/__init__.py:1501-1518, restated per Gaussian.
//   R = quaternion_to_matrix(normalize(q))      (pytorch3d 0.3.0, environment.yml:156:
//        two_s = 2 / (q.q); row-major 3x3 with (r,i,j,k) = q;  F.normalize divides by max(|q|, 1e-12))
//   n = column argmin(scales) of R, negated where n . (campos - mean) < 0
//   local = n @ V[:3,:3];  p = mean @ V[:3,:3] + V[3,:3];  out = [local, 1, |local . p|]
// The reference takes the argmin over exp(scales); exp is monotone, so this is the argmin of the
// scales themselves (first minimum on ties).  torch's reductions and matmul leave the summation
// order open; sums here run left to right, so agreement with torch is to rounding, not bitwise.
static inline int allmap_min_axis(const float* s) {
  int a = 0;
  if (s[1] < s[a]) a = 1;
  if (s[2] < s[a]) a = 2;
  return a;
}

// column `c` of quaternion_to_matrix for a (not necessarily unit) quaternion q = (r,i,j,k)
static inline void allmap_column(const float* q, int c, float two_s, float* n) {
  const float r = q[0], i = q[1], j = q[2], k = q[3];
  if (c == 0) {
    n[0] = 1.0f - two_s * (j * j + k * k);
    n[1] = two_s * (i * j + k * r);
    n[2] = two_s * (i * k - j * r);
  } else if (c == 1) {
    n[0] = two_s * (i * j - k * r);
    n[1] = 1.0f - two_s * (i * i + k * k);
    n[2] = two_s * (j * k + i * r);
  } else {
    n[0] = two_s * (i * k + j * r);
    n[1] = two_s * (j * k - i * r);
    n[2] = 1.0f - two_s * (i * i + j * j);
  }
}

void oracle_all_map_fwd(int P, const float* means, const float* scales, const float* rots, const float* V,
                        const float* campos, float* out) {
#pragma omp parallel for schedule(static)
  for (int g = 0; g < P; g++) {
    const float* q0 = rots + 4 * (size_t)g;
    const float* m = means + 3 * (size_t)g;
    const float len = sqrtf(((q0[0] * q0[0] + q0[1] * q0[1]) + q0[2] * q0[2]) + q0[3] * q0[3]);
    const float den = fmaxf(len, 1e-12f);
    const float q[4] = {q0[0] / den, q0[1] / den, q0[2] / den, q0[3] / den};
    const float two_s = 2.0f / (((q[0] * q[0] + q[1] * q[1]) + q[2] * q[2]) + q[3] * q[3]);
    float n[3];
    allmap_column(q, allmap_min_axis(scales + 3 * (size_t)g), two_s, n);
    const float tc[3] = {campos[0] - m[0], campos[1] - m[1], campos[2] - m[2]};
    if ((n[0] * tc[0] + n[1] * tc[1]) + n[2] * tc[2] < 0.0f) {
      n[0] = -n[0]; n[1] = -n[1]; n[2] = -n[2];
    }
    float loc[3], pc[3];
    for (int k = 0; k < 3; k++) {
      loc[k] = (n[0] * V[k] + n[1] * V[4 + k]) + n[2] * V[8 + k];
      pc[k] = ((m[0] * V[k] + m[1] * V[4 + k]) + m[2] * V[8 + k]) + V[12 + k];
    }
    float* o = out + 5 * (size_t)g;
    o[0] = loc[0]; o[1] = loc[1]; o[2] = loc[2];
    o[3] = 1.0f;
    o[4] = fabsf((loc[0] * pc[0] + loc[1] * pc[1]) + loc[2] * pc[2]);
  }
}

// Gradient of the above with respect to means and (unnormalised) rotations: what autograd derives
// from the same torch lines.  scales only choose the axis and the flip only a sign: no gradient.
void oracle_all_map_bwd(int P, const float* means, const float* scales, const float* rots, const float* V,
                        const float* campos, const float* gout, float* dmeans, float* drots) {
#pragma omp parallel for schedule(static)
  for (int g = 0; g < P; g++) {
    const float* q0 = rots + 4 * (size_t)g;
    const float* m = means + 3 * (size_t)g;
    const float* go = gout + 5 * (size_t)g;
    const float len = sqrtf(((q0[0] * q0[0] + q0[1] * q0[1]) + q0[2] * q0[2]) + q0[3] * q0[3]);
    const float den = fmaxf(len, 1e-12f);
    const float q[4] = {q0[0] / den, q0[1] / den, q0[2] / den, q0[3] / den};
    const float two_s = 2.0f / (((q[0] * q[0] + q[1] * q[1]) + q[2] * q[2]) + q[3] * q[3]);
    const int c = allmap_min_axis(scales + 3 * (size_t)g);
    float n[3];
    allmap_column(q, c, two_s, n);
    const float tc[3] = {campos[0] - m[0], campos[1] - m[1], campos[2] - m[2]};
    const bool flip = (n[0] * tc[0] + n[1] * tc[1]) + n[2] * tc[2] < 0.0f;
    const float sgn = flip ? -1.0f : 1.0f;
    float loc[3], pc[3];
    for (int k = 0; k < 3; k++) {
      loc[k] = sgn * ((n[0] * V[k] + n[1] * V[4 + k]) + n[2] * V[8 + k]);
      pc[k] = ((m[0] * V[k] + m[1] * V[4 + k]) + m[2] * V[8 + k]) + V[12 + k];
    }
    const float s = (loc[0] * pc[0] + loc[1] * pc[1]) + loc[2] * pc[2];
    const float gs = go[4] * (s > 0.0f ? 1.0f : (s < 0.0f ? -1.0f : 0.0f));  // d|s| = sign(s)
    float gl[3], gp[3];
    for (int k = 0; k < 3; k++) {
      gl[k] = go[k] + gs * pc[k];
      gp[k] = gs * loc[k];
    }
    float gn[3];
    for (int a = 0; a < 3; a++) {
      gn[a] = sgn * ((gl[0] * V[4 * a] + gl[1] * V[4 * a + 1]) + gl[2] * V[4 * a + 2]);
      dmeans[3 * (size_t)g + a] = (gp[0] * V[4 * a] + gp[1] * V[4 * a + 1]) + gp[2] * V[4 * a + 2];
    }
    // column c of R as a function of (r,i,j,k) and two_s = 2/(q.q)
    const float r = q[0], i = q[1], j = q[2], k = q[3], ts = two_s;
    float gq[4], gts;
    if (c == 0) {
      gq[0] = ts * (k * gn[1] - j * gn[2]);
      gq[1] = ts * (j * gn[1] + k * gn[2]);
      gq[2] = ts * ((-2.0f * j * gn[0] + i * gn[1]) - r * gn[2]);
      gq[3] = ts * ((-2.0f * k * gn[0] + r * gn[1]) + i * gn[2]);
      gts = (-(j * j + k * k) * gn[0] + (i * j + k * r) * gn[1]) + (i * k - j * r) * gn[2];
    } else if (c == 1) {
      gq[0] = ts * (-k * gn[0] + i * gn[2]);
      gq[1] = ts * ((j * gn[0] - 2.0f * i * gn[1]) + r * gn[2]);
      gq[2] = ts * (i * gn[0] + k * gn[2]);
      gq[3] = ts * ((-r * gn[0] - 2.0f * k * gn[1]) + j * gn[2]);
      gts = ((i * j - k * r) * gn[0] - (i * i + k * k) * gn[1]) + (j * k + i * r) * gn[2];
    } else {
      gq[0] = ts * (j * gn[0] - i * gn[1]);
      gq[1] = ts * ((k * gn[0] - r * gn[1]) - 2.0f * i * gn[2]);
      gq[2] = ts * ((r * gn[0] + k * gn[1]) - 2.0f * j * gn[2]);
      gq[3] = ts * (i * gn[0] + j * gn[1]);
      gts = ((i * k + j * r) * gn[0] + (j * k - i * r) * gn[1]) - (i * i + j * j) * gn[2];
    }
    // d two_s / dq = -two_s^2 q
    const float w = -(ts * ts) * gts;
    for (int a = 0; a < 4; a++) gq[a] += w * q[a];
    // F.normalize backward: q_hat = q0 / max(|q0|, eps)
    float* dq = drots + 4 * (size_t)g;
    if (len > 1e-12f) {
      const float dot = ((q[0] * gq[0] + q[1] * gq[1]) + q[2] * gq[2]) + q[3] * gq[3];
      for (int a = 0; a < 4; a++) dq[a] = (gq[a] - q[a] * dot) / len;
    } else {
      for (int a = 0; a < 4; a++) dq[a] = gq[a] / den;
    }
  }
}


// ---------------------------------------------------------------------------
// Per-pixel masked L1 and SSIM maps of the training loss: pixelwise_l1_with_mask and
// pixelwise_ssim_with_mask (utils/loss_utils.py:88-132), window from create_window (:27-43): an 11x11
// Gaussian (sigma 1.5) applied per channel with zero padding of 5.  `win` holds the 11 normalised 1-D
// weights as float32 (the caller builds them as gaussian() does); the 2-D window is their float32 outer
// product, as torch's mm gives it.  Convolutions are summed row by row, left to right, in float32; torch's
// conv2d leaves that order open, so agreement with torch is to rounding.
static void ssim_stats(int H, int W, const float* a, const float* b, const float* w2, int y, int x, float* st) {
  float m1 = 0.f, m2 = 0.f, e11 = 0.f, e22 = 0.f, e12 = 0.f;
  for (int dy = -5; dy <= 5; dy++) {
    const int yy = y + dy;
    if (yy < 0 || yy >= H) continue;
    for (int dx = -5; dx <= 5; dx++) {
      const int xx = x + dx;
      if (xx < 0 || xx >= W) continue;
      const float wt = w2[(dy + 5) * 11 + (dx + 5)];
      const float p = a[(size_t)yy * W + xx], q = b[(size_t)yy * W + xx];
      m1 += wt * p;
      m2 += wt * q;
      e11 += wt * (p * p);
      e22 += wt * (q * q);
      e12 += wt * (p * q);
    }
  }
  st[0] = m1; st[1] = m2; st[2] = e11; st[3] = e22; st[4] = e12;
}

void oracle_ssim_l1_fwd(int C, int H, int W, const float* img1, const float* img2, const uint8_t* mask,
                        const float* win, float* l1_map, float* ssim_map) {
  float w2[121];
  for (int i = 0; i < 11; i++)
    for (int j = 0; j < 11; j++) w2[i * 11 + j] = win[i] * win[j];
  const float C1 = (float)(0.01 * 0.01), C2 = (float)(0.03 * 0.03);
#pragma omp parallel for collapse(2) schedule(static)
  for (int c = 0; c < C; c++)
    for (int y = 0; y < H; y++) {
      const float* a = img1 + (size_t)c * H * W;
      const float* b = img2 + (size_t)c * H * W;
      for (int x = 0; x < W; x++) {
        float st[5];
        ssim_stats(H, W, a, b, w2, y, x, st);
        const float mu1 = st[0], mu2 = st[1];
        const float mu1_sq = mu1 * mu1, mu2_sq = mu2 * mu2, mu12 = mu1 * mu2;
        const float s1 = st[2] - mu1_sq, s2 = st[3] - mu2_sq, s12 = st[4] - mu12;
        const float v = ((2 * mu12 + C1) * (2 * s12 + C2)) / ((mu1_sq + mu2_sq + C1) * (s1 + s2 + C2));
        const float mk = mask ? (float)(mask[(size_t)y * W + x] != 0) : 1.0f;
        const size_t o = ((size_t)c * H + y) * W + x;
        ssim_map[o] = v * mk;
        l1_map[o] = fabsf(a[(size_t)y * W + x] - b[(size_t)y * W + x]) * mk;
      }
    }
}

// d(sum(g_l1 * l1_map) + sum(g_ssim * ssim_map)) / d img1, by the adjoint of the statements above: the three
// partial derivatives of the SSIM value with respect to the window means of x, x*x and x*y, weighted by
// mask and upstream gradient, are spread back through the (symmetric) window.
void oracle_ssim_l1_bwd(int C, int H, int W, const float* img1, const float* img2, const uint8_t* mask,
                        const float* win, const float* g_l1, const float* g_ssim, float* dimg1) {
  float w2[121];
  for (int i = 0; i < 11; i++)
    for (int j = 0; j < 11; j++) w2[i * 11 + j] = win[i] * win[j];
  const float C1 = (float)(0.01 * 0.01), C2 = (float)(0.03 * 0.03);
  const size_t HW = (size_t)H * W;
  std::vector<float> d_mu((size_t)C * HW), d_e11((size_t)C * HW), d_e12((size_t)C * HW);
#pragma omp parallel for collapse(2) schedule(static)
  for (int c = 0; c < C; c++)
    for (int y = 0; y < H; y++) {
      const float* a = img1 + (size_t)c * HW;
      const float* b = img2 + (size_t)c * HW;
      for (int x = 0; x < W; x++) {
        float st[5];
        ssim_stats(H, W, a, b, w2, y, x, st);
        const float mu1 = st[0], mu2 = st[1];
        const float A1 = 2 * (mu1 * mu2) + C1, B1 = (mu1 * mu1 + mu2 * mu2) + C1;
        const float s12 = st[4] - mu1 * mu2;
        const float A2 = 2 * s12 + C2, B2 = ((st[2] - mu1 * mu1) + (st[3] - mu2 * mu2)) + C2;
        const float S = (A1 * A2) / (B1 * B2);
        const float mk = mask ? (float)(mask[(size_t)y * W + x] != 0) : 1.0f;
        const size_t o = (size_t)c * HW + (size_t)y * W + x;
        const float gw = g_ssim[o] * mk;
        d_mu[o] = gw * ((2 * mu2 * (A2 - A1)) / (B1 * B2) - S * (2 * mu1 / B1) + S * (2 * mu1 / B2));
        d_e11[o] = gw * (-S / B2);
        d_e12[o] = gw * (2 * A1 / (B1 * B2));
      }
    }
#pragma omp parallel for collapse(2) schedule(static)
  for (int c = 0; c < C; c++)
    for (int y = 0; y < H; y++)
      for (int x = 0; x < W; x++) {
        float cm = 0.f, c11 = 0.f, c12 = 0.f;
        for (int dy = -5; dy <= 5; dy++) {
          const int yy = y + dy;
          if (yy < 0 || yy >= H) continue;
          for (int dx = -5; dx <= 5; dx++) {
            const int xx = x + dx;
            if (xx < 0 || xx >= W) continue;
            const float wt = w2[(dy + 5) * 11 + (dx + 5)];
            const size_t q = (size_t)c * HW + (size_t)yy * W + xx;
            cm += wt * d_mu[q];
            c11 += wt * d_e11[q];
            c12 += wt * d_e12[q];
          }
        }
        const size_t o = (size_t)c * HW + (size_t)y * W + x;
        const float p = img1[o], q2 = img2[o];
        const float mk = mask ? (float)(mask[(size_t)y * W + x] != 0) : 1.0f;
        const float d = p - q2;
        const float sg = d > 0.f ? 1.0f : (d < 0.f ? -1.0f : 0.0f);
        dimg1[o] = ((cm + 2 * p * c11) + q2 * c12) + g_l1[o] * mk * sg;
      }
}


// ---------------------------------------------------------------------------
// Neural-Gaussian generation, generate_neural_gaussians (gaussian_renderer/__init__.py:789-899) in the
// reference's default configuration (arguments/__init__.py:94-124: feat_dim 32, no feature bank, no
// appearance embedding, no distance / level inputs, dist2level 'round'): per visible anchor
//   x = [feat(32), (anchor - campos)/|anchor - campos| (3)]
//   neural_opacity = tanh(W2o relu(W1o x + b1o) + b2o)            (k values)       :841-853
//     (dist2level 'progressive': times prog, the anchor's _prog_ratio or 1 outside transition_mask, :844-848;
//      prog = NULL stands for no factor)
//   color = sigmoid(W2c relu(W1c x + b1c) + b2c)                  (k x 3)          :866-870
//   scale_rot = W2v relu(W1v x + b1v) + b2v                       (k x 7)          :873-877
// and for every (anchor, offset) with neural_opacity > 0, in that order (:856-858, :886):
//   xyz = anchor + offset * scaling[0:3];  scaling = scaling[3:6] * sigmoid(scale_rot[0:3]);
//   rot = scale_rot[3:7] / max(|scale_rot[3:7]|, 1e-12);  color;  opacity = neural_opacity   (:889-896)
// MLPs as nn.Linear: W1 (32 x 35), b1 (32), W2 (out x 32), b2 (out), row-major [out][in]
// (scene/gaussian_model.py:131-149).  `scaling` is the activated one, get_scaling (N x 6).
// Sums run left to right in float32; torch's matmul leaves the order open: agreement to rounding.
struct MlpView {
  const float *W1, *b1, *W2, *b2;
  int out;
  int in;         // input width: 35, +1 with the distance, +1 with the level
  bool has_dist;  // column 35 is the distance |anchor - campos|
  bool has_level; // the last column is the anchor's level
};

// input_flags: bit 0 / 1 / 2 = the opacity / color / cov MLP takes the distance (add_opacity_dist,
// add_color_dist, add_cov_dist, :839-877), bit 3 = all three take the level (add_level, :824-829)
static MlpView mlp_view(const float* W1, const float* b1, const float* W2, const float* b2, int out, int m,
                        int input_flags) {
  const bool d = (input_flags >> m) & 1, l = (input_flags >> 3) & 1;
  return MlpView{W1, b1, W2, b2, out, 35 + (d ? 1 : 0) + (l ? 1 : 0), d, l};
}

static void mlp_forward(const MlpView& m, const float* x, float* hidden, float* out) {
  for (int h = 0; h < 32; h++) {
    float a = m.b1[h];
    for (int i = 0; i < m.in; i++) a += m.W1[h * m.in + i] * x[i];
    hidden[h] = a > 0.f ? a : 0.f;
  }
  for (int o = 0; o < m.out; o++) {
    float a = m.b2[o];
    for (int h = 0; h < 32; h++) a += m.W2[o * 32 + h] * hidden[h];
    out[o] = a;
  }
}

// x = [feat, view direction, distance, level] (37 values; cat_local_view, :824-829)
static void neural_input(const float* anchor, const float* feat, const float* campos, float level, float* x,
                         float* dist) {
  for (int i = 0; i < 32; i++) x[i] = feat[i];
  const float v[3] = {anchor[0] - campos[0], anchor[1] - campos[1], anchor[2] - campos[2]};
  const float d = sqrtf((v[0] * v[0] + v[1] * v[1]) + v[2] * v[2]);
  x[32] = v[0] / d; x[33] = v[1] / d; x[34] = v[2] / d;
  x[35] = d;
  x[36] = level;
  *dist = d;
}

// the columns an MLP takes of x, in its own order
static void mlp_input(const MlpView& m, const float* x, float* xm) {
  for (int i = 0; i < 35; i++) xm[i] = x[i];
  int c = 35;
  if (m.has_dist) xm[c++] = x[35];
  if (m.has_level) xm[c++] = x[36];
}

// dense per-slot results: neural_opacity (N*k), mask (N*k), color (N*k*3, after sigmoid), scale_rot (N*k*7)
void oracle_neural_mlp_fwd(int N, int k, const float* anchor, const float* feat, const float* campos,
                           const float* W1o, const float* b1o, const float* W2o, const float* b2o,
                           const float* W1c, const float* b1c, const float* W2c, const float* b2c,
                           const float* W1v, const float* b1v, const float* W2v, const float* b2v,
                           const float* prog, const float* level, int input_flags, float* neural_opacity,
                           uint8_t* mask, float* color, float* scale_rot) {
  const MlpView mo = mlp_view(W1o, b1o, W2o, b2o, k, 0, input_flags),
                mc = mlp_view(W1c, b1c, W2c, b2c, 3 * k, 1, input_flags),
                mv = mlp_view(W1v, b1v, W2v, b2v, 7 * k, 2, input_flags);
#pragma omp parallel for schedule(static)
  for (int a = 0; a < N; a++) {
    float x[37], xm[37], dist, hid[32];
    neural_input(anchor + 3 * (size_t)a, feat + 32 * (size_t)a, campos, level ? level[a] : 0.f, x, &dist);
    std::vector<float> out(7 * k);
    mlp_input(mo, x, xm);
    mlp_forward(mo, xm, hid, out.data());
    for (int j = 0; j < k; j++) {
      const float t = prog ? tanhf(out[j]) * prog[a] : tanhf(out[j]);
      neural_opacity[(size_t)a * k + j] = t;
      mask[(size_t)a * k + j] = t > 0.f;
    }
    mlp_input(mc, x, xm);
    mlp_forward(mc, xm, hid, out.data());
    for (int j = 0; j < 3 * k; j++) color[(size_t)a * 3 * k + j] = 1.0f / (1.0f + expf(-out[j]));
    mlp_input(mv, x, xm);
    mlp_forward(mv, xm, hid, out.data());
    for (int j = 0; j < 7 * k; j++) scale_rot[(size_t)a * 7 * k + j] = out[j];
  }
}

// compaction and post-processing; returns the number of selected Gaussians
int oracle_neural_compact(int N, int k, const float* anchor, const float* offsets, const float* scaling,
                          const float* neural_opacity, const uint8_t* mask, const float* color,
                          const float* scale_rot, float* xyz, float* col, float* opacity, float* scal, float* rot) {
  size_t r = 0;
  for (int a = 0; a < N; a++)
    for (int j = 0; j < k; j++) {
      const size_t s = (size_t)a * k + j;
      if (!mask[s]) continue;
      const float* sc = scaling + 6 * (size_t)a;
      for (int c = 0; c < 3; c++) {
        xyz[3 * r + c] = anchor[3 * (size_t)a + c] + offsets[3 * s + c] * sc[c];
        col[3 * r + c] = color[3 * s + c];
        scal[3 * r + c] = sc[3 + c] * (1.0f / (1.0f + expf(-scale_rot[7 * s + c])));
      }
      opacity[r] = neural_opacity[s];
      const float* q = scale_rot + 7 * s + 3;
      const float len = sqrtf(((q[0] * q[0] + q[1] * q[1]) + q[2] * q[2]) + q[3] * q[3]);
      const float den = fmaxf(len, 1e-12f);
      for (int c = 0; c < 4; c++) rot[4 * r + c] = q[c] / den;
      r++;
    }
  return (int)r;
}

// Backward of both steps.  Upstream gradients are given for the compacted outputs (S rows each); results:
// d_anchor (N,3), d_feat (N,32), d_offsets (N*k,3), d_scaling (N,6) and the twelve weight gradients
// (accumulated in double, returned as float32).  neural_opacity itself (the dense output) is taken as
// non-differentiated, as the reference only uses it detached (scene/gaussian_model.py:1183).
void oracle_neural_bwd(int N, int k, const float* anchor, const float* feat, const float* offsets,
                       const float* scaling, const float* campos,
                       const float* W1o, const float* b1o, const float* W2o, const float* b2o,
                       const float* W1c, const float* b1c, const float* W2c, const float* b2c,
                       const float* W1v, const float* b1v, const float* W2v, const float* b2v, const float* prog,
                       const float* level, int input_flags, const float* g_xyz, const float* g_col, const float* g_opacity, const float* g_scal,
                       const float* g_rot, float* d_anchor, float* d_feat, float* d_offsets, float* d_scaling,
                       float* dW1o, float* db1o, float* dW2o, float* db2o, float* dW1c, float* db1c, float* dW2c,
                       float* db2c, float* dW1v, float* db1v, float* dW2v, float* db2v) {
  const MlpView ms[3] = {mlp_view(W1o, b1o, W2o, b2o, k, 0, input_flags),
                         mlp_view(W1c, b1c, W2c, b2c, 3 * k, 1, input_flags),
                         mlp_view(W1v, b1v, W2v, b2v, 7 * k, 2, input_flags)};
  float* dW1s[3] = {dW1o, dW1c, dW1v};
  float* db1s[3] = {db1o, db1c, db1v};
  float* dW2s[3] = {dW2o, dW2c, dW2v};
  float* db2s[3] = {db2o, db2c, db2v};
  std::vector<std::vector<double>> aW1(3), ab1(3), aW2(3), ab2(3);
  for (int m = 0; m < 3; m++) {
    aW1[m].assign(32 * (size_t)ms[m].in, 0.0); ab1[m].assign(32, 0.0);
    aW2[m].assign((size_t)ms[m].out * 32, 0.0); ab2[m].assign(ms[m].out, 0.0);
  }
  size_t r = 0;
  for (int a = 0; a < N; a++) {
    float x[37], xm[3][37], dist, hid[3][32];
    neural_input(anchor + 3 * (size_t)a, feat + 32 * (size_t)a, campos, level ? level[a] : 0.f, x, &dist);
    std::vector<float> out[3], gout[3];
    for (int m = 0; m < 3; m++) {
      out[m].resize(ms[m].out);
      gout[m].assign(ms[m].out, 0.f);
      mlp_input(ms[m], x, xm[m]);
      mlp_forward(ms[m], xm[m], hid[m], out[m].data());
    }
    const float* sc = scaling + 6 * (size_t)a;
    float da[3] = {0.f, 0.f, 0.f}, dsc[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; j++) {
      const size_t s = (size_t)a * k + j;
      for (int c = 0; c < 3; c++) d_offsets[3 * s + c] = 0.f;
      const float th = tanhf(out[0][j]);
      const float pf = prog ? prog[a] : 1.0f;
      const float t = prog ? th * pf : th;
      if (!(t > 0.f)) continue;
      // opacity = tanh(pre) * prog
      gout[0][j] = g_opacity[r] * ((1.0f - th * th) * pf);
      for (int c = 0; c < 3; c++) {
        const float cs = 1.0f / (1.0f + expf(-out[1][3 * j + c]));
        gout[1][3 * j + c] = g_col[3 * r + c] * (cs * (1.0f - cs));
        // xyz = anchor + offset * sc[c]
        da[c] += g_xyz[3 * r + c];
        d_offsets[3 * s + c] = g_xyz[3 * r + c] * sc[c];
        dsc[c] += g_xyz[3 * r + c] * offsets[3 * s + c];
        // scaling = sc[3+c] * sigmoid(sr[c])
        const float sg = 1.0f / (1.0f + expf(-out[2][7 * j + c]));
        dsc[3 + c] += g_scal[3 * r + c] * sg;
        gout[2][7 * j + c] = g_scal[3 * r + c] * sc[3 + c] * (sg * (1.0f - sg));
      }
      // rot = q / max(|q|, eps)
      const float* q = out[2].data() + 7 * j + 3;
      const float len = sqrtf(((q[0] * q[0] + q[1] * q[1]) + q[2] * q[2]) + q[3] * q[3]);
      const float* gr = g_rot + 4 * r;
      if (len > 1e-12f) {
        float qh[4], dot = 0.f;
        for (int c = 0; c < 4; c++) { qh[c] = q[c] / len; dot += qh[c] * gr[c]; }
        for (int c = 0; c < 4; c++) gout[2][7 * j + 3 + c] = (gr[c] - qh[c] * dot) / len;
      } else {
        for (int c = 0; c < 4; c++) gout[2][7 * j + 3 + c] = gr[c] / 1e-12f;
      }
      r++;
    }
    // through the three MLPs
    float dx[36];  // features, view direction, distance (the level is an integer-valued buffer)
    for (int i = 0; i < 36; i++) dx[i] = 0.f;
    for (int m = 0; m < 3; m++) {
      float dh[32];
      for (int h = 0; h < 32; h++) dh[h] = 0.f;
      for (int o = 0; o < ms[m].out; o++) {
        const float g = gout[m][o];
        if (g == 0.f) continue;
        ab2[m][o] += g;
        for (int h = 0; h < 32; h++) {
          aW2[m][(size_t)o * 32 + h] += (double)g * hid[m][h];
          dh[h] += ms[m].W2[o * 32 + h] * g;
        }
      }
      for (int h = 0; h < 32; h++) {
        if (!(hid[m][h] > 0.f)) continue;  // ReLU
        ab1[m][h] += dh[h];
        const int in = ms[m].in;
        for (int i = 0; i < in; i++) {
          aW1[m][h * in + i] += (double)dh[h] * xm[m][i];
          if (i < 35 || (i == 35 && ms[m].has_dist)) dx[i] += ms[m].W1[h * in + i] * dh[h];
        }
      }
    }
    for (int i = 0; i < 32; i++) d_feat[32 * (size_t)a + i] = dx[i];
    // view direction v/|v|: d v = (g - n (n.g)) / |v|
    const float nv[3] = {x[32], x[33], x[34]};
    const float ng = (nv[0] * dx[32] + nv[1] * dx[33]) + nv[2] * dx[34];
    // and the distance |v|: d v = n * g
    for (int c = 0; c < 3; c++)
      d_anchor[3 * (size_t)a + c] = (da[c] + (dx[32 + c] - nv[c] * ng) / dist) + nv[c] * dx[35];
    for (int c = 0; c < 6; c++) d_scaling[6 * (size_t)a + c] = dsc[c];
  }
  for (int m = 0; m < 3; m++) {
    for (int i = 0; i < 32 * ms[m].in; i++) dW1s[m][i] = (float)aW1[m][i];
    for (int i = 0; i < 32; i++) db1s[m][i] = (float)ab1[m][i];
    for (size_t i = 0; i < (size_t)ms[m].out * 32; i++) dW2s[m][i] = (float)aW2[m][i];
    for (int i = 0; i < ms[m].out; i++) db2s[m][i] = (float)ab2[m][i];
  }
}

}  // extern "C"
