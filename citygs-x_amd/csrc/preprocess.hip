// Per-Gaussian streaming kernels: frustum cull, 3D/2D covariance, conic,
// radius, pixel centre, SH colour, tile-rectangle count; the visibility
// prefilter; and the backward of all of it.
//
// Arithmetic follows cuda_rasterizer/forward.cu:75-259 and
// cuda_rasterizer/backward.cu:69-321 operation by operation (see gs_common.h
// for the rounding policy).  One thread per Gaussian; every output element is
// written by the kernel (zeros for culled Gaussians), so callers may hand in
// uninitialised buffers.
#include "all_map_common.h"
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

__constant__ const float kC0 = 0.28209479177387814f;
__constant__ const float kC1 = 0.4886025119029199f;
__constant__ const float kC2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                                   -1.0925484305920792f, 0.5462742152960396f};
__constant__ const float kC3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                                   0.3731763325901154f,  -0.4570457994644658f, 1.445305721320277f,
                                   -0.5900435899266435f};

struct CamParams {
  float V[16];
  float PM[16];
  float campos[3];
};

__device__ __forceinline__ void load_cam(const float* __restrict__ V, const float* __restrict__ PM,
                                         const float* __restrict__ campos, CamParams& c) {
#pragma unroll
  for (int k = 0; k < 16; k++) {
    c.V[k] = V[k];
    c.PM[k] = PM[k];
  }
  if (campos) {
    c.campos[0] = campos[0];
    c.campos[1] = campos[1];
    c.campos[2] = campos[2];
  } else {
    c.campos[0] = c.campos[1] = c.campos[2] = 0.f;
  }
}

// cuda_rasterizer/forward.cu:119-153.  q = (r,x,y,z), not normalised.
__device__ __forceinline__ void cov3d_from_scale_rot(const float* s_in, float mod, const float* q, float* out6,
                                                     M3* M_out, M3* R_out) {
  M3 S = m3_cols(1.f, 0.f, 0.f, 0.f, 1.f, 0.f, 0.f, 0.f, 1.f);
  S.m[0][0] = mod * s_in[0];
  S.m[1][1] = mod * s_in[1];
  S.m[2][2] = mod * s_in[2];
  const float r = q[0], x = q[1], y = q[2], z = q[3];
  M3 R = m3_cols(1.f - 2.f * (y * y + z * z), 2.f * (x * y - r * z), 2.f * (x * z + r * y),
                 2.f * (x * y + r * z), 1.f - 2.f * (x * x + z * z), 2.f * (y * z - r * x),
                 2.f * (x * z - r * y), 2.f * (y * z + r * x), 1.f - 2.f * (x * x + y * y));
  M3 M = m3_mul(S, R);
  M3 Sig = m3_mul(m3_T(M), M);
  out6[0] = Sig.m[0][0]; out6[1] = Sig.m[0][1]; out6[2] = Sig.m[0][2];
  out6[3] = Sig.m[1][1]; out6[4] = Sig.m[1][2]; out6[5] = Sig.m[2][2];
  if (M_out) *M_out = M;
  if (R_out) *R_out = R;
}

struct Cov2DCtx {
  M3 T, W, Vrk;
  float t[3];
  float txtz, tytz, limx, limy;
  float a, b, c;
};

// cuda_rasterizer/forward.cu:75-114.
__device__ __forceinline__ void cov2d(const float* mean, float fx, float fy, float tanx, float tany,
                                      const float* c6, const float* V, Cov2DCtx& o) {
  xform4x3(mean, V, o.t);
  o.limx = 1.3f * tanx;
  o.limy = 1.3f * tany;
  o.txtz = o.t[0] / o.t[2];
  o.tytz = o.t[1] / o.t[2];
  o.t[0] = fminf(o.limx, fmaxf(-o.limx, o.txtz)) * o.t[2];
  o.t[1] = fminf(o.limy, fmaxf(-o.limy, o.tytz)) * o.t[2];
  const float tz = o.t[2];
  M3 J = m3_cols(fx / tz, 0.0f, -(fx * o.t[0]) / (tz * tz), 0.0f, fy / tz, -(fy * o.t[1]) / (tz * tz), 0.f,
                 0.f, 0.f);
  o.W = m3_cols(V[0], V[4], V[8], V[1], V[5], V[9], V[2], V[6], V[10]);
  o.T = m3_mul(o.W, J);
  o.Vrk = m3_cols(c6[0], c6[1], c6[2], c6[1], c6[3], c6[4], c6[2], c6[4], c6[5]);
  M3 cov = m3_mul(m3_mul(m3_T(o.T), m3_T(o.Vrk)), o.T);
  o.a = cov.m[0][0] + 0.3f;
  o.b = cov.m[0][1];
  o.c = cov.m[1][1] + 0.3f;
}

struct GeomOut {
  float depth, px, py, conic[3];
  int radius;
  Rect rect;
};

// Geometry of cuda_rasterizer/forward.cu:183-239.  cov6 receives the 3D
// covariance as soon as the Gaussian is in front of the camera.  Returns
// false when the Gaussian is dropped; in_front tells whether cov6 is valid.
__device__ __forceinline__ bool geom_forward(const float* mean, const float* scale, float mod, const float* rot,
                                             const float* cov_pre, const CamParams& cam, int W, int H, float tanx,
                                             float tany, float fx, float fy, uint32_t gx, uint32_t gy, float* cov6,
                                             bool& in_front, GeomOut& g) {
  float ph[4], pv[3];
  xform4x4(mean, cam.PM, ph);
  const float pw = 1.0f / (ph[3] + 0.0000001f);
  const float pprojx = ph[0] * pw, pprojy = ph[1] * pw;
  xform4x3(mean, cam.V, pv);
  in_front = pv[2] > 0.0f;
  if (!in_front) return false;  // cuda_rasterizer/auxiliary.h:208
  if (cov_pre) {
#pragma unroll
    for (int k = 0; k < 6; k++) cov6[k] = cov_pre[k];
  } else {
    cov3d_from_scale_rot(scale, mod, rot, cov6, nullptr, nullptr);
  }
  Cov2DCtx cc;
  cov2d(mean, fx, fy, tanx, tany, cov6, cam.V, cc);
  const float det = cc.a * cc.c - cc.b * cc.b;
  if (det == 0.0f) return false;
  const float det_inv = 1.f / det;
  g.conic[0] = cc.c * det_inv;
  g.conic[1] = -cc.b * det_inv;
  g.conic[2] = cc.a * det_inv;
  const float mid = 0.5f * (cc.a + cc.c);
  const float root = sqrtf(fmaxf(0.1f, mid * mid - det));
  const float l1 = mid + root, l2 = mid - root;
  const float rad_f = ceilf(3.f * sqrtf(fmaxf(l1, l2)));
  g.px = ndc2pix(pprojx, W);
  g.py = ndc2pix(pprojy, H);
  g.radius = f2i_sat(rad_f);
  g.rect = get_rect(g.px, g.py, g.radius, gx, gy);
  if ((g.rect.x1 - g.rect.x0) * (g.rect.y1 - g.rect.y0) == 0) return false;
  g.depth = pv[2];
  return true;
}

// cuda_rasterizer/forward.cu:21-72 for one colour channel; c[k] = coefficient k.
__device__ __forceinline__ float sh_channel(int deg, float x, float y, float z, const float* c) {
  float res = kC0 * c[0];
  if (deg > 0) {
    res = ((res - kC1 * y * c[1]) + kC1 * z * c[2]) - kC1 * x * c[3];
    if (deg > 1) {
      const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
      res = ((((res + kC2[0] * xy * c[4]) + kC2[1] * yz * c[5]) + kC2[2] * (2.0f * zz - xx - yy) * c[6]) +
             kC2[3] * xz * c[7]) +
            kC2[4] * (xx - yy) * c[8];
      if (deg > 2) {
        res = ((((((res + kC3[0] * y * (3.0f * xx - yy) * c[9]) + kC3[1] * xy * z * c[10]) +
                  kC3[2] * y * (4.0f * zz - xx - yy) * c[11]) +
                 kC3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy) * c[12]) +
                kC3[4] * x * (4.0f * zz - xx - yy) * c[13]) +
               kC3[5] * z * (xx - yy) * c[14]) +
              kC3[6] * x * (xx - 3.0f * yy) * c[15];
      }
    }
  }
  return res + 0.5f;
}

// 192-byte rows (16 SH coefficients x 3 channels) of the 64 Gaussians of a wave, moved between global memory
// and LDS with whole-wave 16-byte accesses over the wave's contiguous 12 KB, so every fetched line is used
// completely; a lane then reads or writes its own row in LDS.  Rows are padded to 13 x 16 bytes, which keeps
// both access patterns free of bank conflicts.
constexpr int SH_ROW4 = 13;
constexpr int SH_WAVE_ROWS4 = GS_WAVE * SH_ROW4;

__device__ __forceinline__ void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Basis values of the 16 SH terms for direction (x, y, z) (those of degrees above D are 0) and, when shv is
// given, the derivatives of the three colour channels with respect to the direction,
// dR_[axis][channel] = sum_k d basis_k / d axis * coefficient(k, channel): the derivative of
// cuda_rasterizer/forward.cu:21-72, evaluated in the order of the reference's 3DGS backward.  shv = the row of
// 16 x 3 coefficients, flat.  The forward kernel evaluates this once and the backward kernel takes its nine
// numbers, or evaluates it itself when it is handed the coefficients instead: same code, same bits.
template <bool WITH_DERIVATIVE>
__device__ __forceinline__ void sh_basis_and_direction_derivative(int D, float x, float y, float z, const float* shv,
                                                                  float* basis, float* dRdx, float* dRdy,
                                                                  float* dRdz) {
#pragma unroll
  for (int k = 0; k < 16; k++) basis[k] = 0.f;
#pragma unroll
  for (int ch = 0; ch < 3; ch++) dRdx[ch] = dRdy[ch] = dRdz[ch] = 0.f;
#define SHV(k, ch) (WITH_DERIVATIVE ? shv[3 * (k) + (ch)] : 0.f)
  basis[0] = kC0;
  if (D > 0) {
    basis[1] = -kC1 * y;
    basis[2] = kC1 * z;
    basis[3] = -kC1 * x;
#pragma unroll
    for (int ch = 0; ch < 3; ch++) {
      dRdx[ch] = -kC1 * SHV(3, ch);
      dRdy[ch] = -kC1 * SHV(1, ch);
      dRdz[ch] = kC1 * SHV(2, ch);
    }
    if (D > 1) {
      const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
      basis[4] = kC2[0] * xy;
      basis[5] = kC2[1] * yz;
      basis[6] = kC2[2] * (2.f * zz - xx - yy);
      basis[7] = kC2[3] * xz;
      basis[8] = kC2[4] * (xx - yy);
#pragma unroll
      for (int ch = 0; ch < 3; ch++) {
        dRdx[ch] += kC2[0] * y * SHV(4, ch) + kC2[2] * 2.f * -x * SHV(6, ch) + kC2[3] * z * SHV(7, ch) +
                    kC2[4] * 2.f * x * SHV(8, ch);
        dRdy[ch] += kC2[0] * x * SHV(4, ch) + kC2[1] * z * SHV(5, ch) + kC2[2] * 2.f * -y * SHV(6, ch) +
                    kC2[4] * 2.f * -y * SHV(8, ch);
        dRdz[ch] += kC2[1] * y * SHV(5, ch) + kC2[2] * 2.f * 2.f * z * SHV(6, ch) + kC2[3] * x * SHV(7, ch);
      }
      if (D > 2) {
        basis[9] = kC3[0] * y * (3.f * xx - yy);
        basis[10] = kC3[1] * xy * z;
        basis[11] = kC3[2] * y * (4.f * zz - xx - yy);
        basis[12] = kC3[3] * z * (2.f * zz - 3.f * xx - 3.f * yy);
        basis[13] = kC3[4] * x * (4.f * zz - xx - yy);
        basis[14] = kC3[5] * z * (xx - yy);
        basis[15] = kC3[6] * x * (xx - 3.f * yy);
#pragma unroll
        for (int ch = 0; ch < 3; ch++) {
          dRdx[ch] += kC3[0] * SHV(9, ch) * 3.f * 2.f * xy + kC3[1] * SHV(10, ch) * yz +
                      kC3[2] * SHV(11, ch) * -2.f * xy + kC3[3] * SHV(12, ch) * -3.f * 2.f * xz +
                      kC3[4] * SHV(13, ch) * (-3.f * xx + 4.f * zz - yy) + kC3[5] * SHV(14, ch) * 2.f * xz +
                      kC3[6] * SHV(15, ch) * 3.f * (xx - yy);
          dRdy[ch] += kC3[0] * SHV(9, ch) * 3.f * (xx - yy) + kC3[1] * SHV(10, ch) * xz +
                      kC3[2] * SHV(11, ch) * (-3.f * yy + 4.f * zz - xx) + kC3[3] * SHV(12, ch) * -3.f * 2.f * yz +
                      kC3[4] * SHV(13, ch) * -2.f * xy + kC3[5] * SHV(14, ch) * -2.f * yz +
                      kC3[6] * SHV(15, ch) * -3.f * 2.f * xy;
          dRdz[ch] += kC3[1] * SHV(10, ch) * xy + kC3[2] * SHV(11, ch) * 4.f * 2.f * yz +
                      kC3[3] * SHV(12, ch) * 3.f * (2.f * zz - xx - yy) + kC3[4] * SHV(13, ch) * 4.f * 2.f * xz +
                      kC3[5] * SHV(14, ch) * (xx - yy);
        }
      }
    }
  }
#undef SHV
}

// The same evaluation, one coefficient at a time: B[k] is everything of term k but the coefficient (the products
// in sh_channel associate from the left, so term k = B[k] * c[k] is the same rounding), and sh_accumulate<K> is
// the step of the running sum that takes in coefficient K.  Coefficients of degrees above `deg` are left out.
__device__ __forceinline__ void sh_basis(float x, float y, float z, float* B) {
  const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
  B[0] = kC0;
  B[1] = kC1 * y;
  B[2] = kC1 * z;
  B[3] = kC1 * x;
  B[4] = kC2[0] * xy;
  B[5] = kC2[1] * yz;
  B[6] = kC2[2] * (2.0f * zz - xx - yy);
  B[7] = kC2[3] * xz;
  B[8] = kC2[4] * (xx - yy);
  B[9] = kC3[0] * y * (3.0f * xx - yy);
  B[10] = kC3[1] * xy * z;
  B[11] = kC3[2] * y * (4.0f * zz - xx - yy);
  B[12] = kC3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy);
  B[13] = kC3[4] * x * (4.0f * zz - xx - yy);
  B[14] = kC3[5] * z * (xx - yy);
  B[15] = kC3[6] * x * (xx - 3.0f * yy);
}

template <int K>
__device__ __forceinline__ float sh_accumulate(int deg, float res, const float* B, float c) {
  constexpr int degree_of = K == 0 ? 0 : K < 4 ? 1 : K < 9 ? 2 : 3;
  if (deg < degree_of) return res;
  if (K == 0) return B[0] * c;
  if (K == 1 || K == 3) return res - B[K] * c;
  return res + B[K] * c;
}

// The 192-byte SH rows of a wave's 64 Gaussians, a third at a time: the 64-byte thirds of all rows are fetched with
// whole-wave 16-byte loads (four lanes share a 64-byte line and use all of it), parked in LDS (rows of four 16-byte
// words padded to five, which keeps both access patterns free of bank conflicts) and read back row-wise, a lane its
// own 16 floats, which it folds into the three running sums before the next third arrives.  A lane that loads its
// own row directly issues twelve 16-byte loads 192 bytes apart from its neighbours': every line then passes through
// the first-level cache four times.
constexpr int SH_THIRD4 = 5;

template <int PHASE>
__device__ __forceinline__ void sh_third_fetch(const float4* __restrict__ wave_rows, uint64_t need, int lane,
                                               float4* v) {
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int idx = j * GS_WAVE + lane, row = idx >> 2, part = idx & 3;
    v[j] = ((need >> row) & 1ull) ? wave_rows[row * 12 + 4 * PHASE + part] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
}

template <int PHASE, bool KEEP>
__device__ __forceinline__ void sh_third_fold(int deg, const float* B, const float4* v, float4* lds, int lane,
                                              float* res, float* keep) {
  wave_sync_lds();  // (everyone has read the previous third)
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int idx = j * GS_WAVE + lane, row = idx >> 2, part = idx & 3;
    lds[row * SH_THIRD4 + part] = v[j];
  }
  wave_sync_lds();
  float f[16];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const float4 w = lds[lane * SH_THIRD4 + k];
    f[4 * k] = w.x; f[4 * k + 1] = w.y; f[4 * k + 2] = w.z; f[4 * k + 3] = w.w;
  }
  if constexpr (KEEP) {  // (the caller also wants the row itself)
#pragma unroll
    for (int e = 0; e < 16; e++) keep[16 * PHASE + e] = f[e];
  }
  // flat element 16 * PHASE + e of the row is coefficient (16 * PHASE + e) / 3 of channel (16 * PHASE + e) % 3
#define GS_SH_STEP(E)                                                                                         \
  res[(16 * PHASE + E) % 3] = sh_accumulate<(16 * PHASE + E) / 3>(deg, res[(16 * PHASE + E) % 3], B, f[E]);
  GS_SH_STEP(0) GS_SH_STEP(1) GS_SH_STEP(2) GS_SH_STEP(3) GS_SH_STEP(4) GS_SH_STEP(5) GS_SH_STEP(6) GS_SH_STEP(7)
  GS_SH_STEP(8) GS_SH_STEP(9) GS_SH_STEP(10) GS_SH_STEP(11) GS_SH_STEP(12) GS_SH_STEP(13) GS_SH_STEP(14)
  GS_SH_STEP(15)
#undef GS_SH_STEP
}


// rows whose bit in `need` is clear are not fetched (their LDS rows read as zero)
__device__ __forceinline__ void wave_rows_load(const float4* __restrict__ g4, uint64_t need, float4* lds, int lane) {
  float4 v[12];
#pragma unroll
  for (int j = 0; j < 12; j++) {
    const int idx = j * GS_WAVE + lane;
    const int row = idx / 12;
    v[j] = ((need >> row) & 1ull) ? g4[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int j = 0; j < 12; j++) {
    const int idx = j * GS_WAVE + lane;
    const int row = idx / 12;
    lds[row * SH_ROW4 + (idx - row * 12)] = v[j];
  }
  wave_sync_lds();
}

// stores the first `rows` rows, streaming: SH coefficient gradients exist only when the coefficients are leaf
// parameters, and then the optimizer is their next reader; the position, scale and rotation gradients can feed
// the caller's backward pass at once and are stored normally
__device__ __forceinline__ void wave_rows_store(float4* __restrict__ g4, int rows, const float4* lds, int lane) {
  wave_sync_lds();
#pragma unroll
  for (int j = 0; j < 12; j++) {
    const int idx = j * GS_WAVE + lane;
    const int row = idx / 12;
    if (row < rows) store_streaming(g4 + idx, lds[row * SH_ROW4 + (idx - row * 12)]);
  }
}

// DERIV: also leave, per surviving Gaussian, the derivative of its colour with respect to the view direction
// (nine numbers), which is all the backward kernel needs the coefficients for.
// RECORDS: also write the blend kernels' operand record of every surviving Gaussian, (x, y, conic.x, conic.y)
// (conic.w, opacity, r, g) (b, map0, map1, map2) (map3, map4, depth, 0), the geometry channels formed here by the
// all_map kernel's own operations on the same inputs; a wave's 64 records leave through LDS as contiguous lines.
// (six waves per SIMD; five with the records: six would spill there, and a kernel that spills starts its waves slowly)
template <bool DERIV, bool RECORDS>
__global__ void __launch_bounds__(GS_BLOCK_1D) __attribute__((amdgpu_waves_per_eu(RECORDS ? 5 : 6)))
preprocess_fwd_kernel(int P, int D, int M, const float* __restrict__ means, const float* __restrict__ scales,
                      float mod, const float* __restrict__ rots, const float* __restrict__ opac,
                      const float* __restrict__ shs, const float* __restrict__ Vg, const float* __restrict__ PMg,
                      const float* __restrict__ camg, int W, int H, float tanx, float tany, float fx, float fy,
                      uint32_t gx, uint32_t gy, int* __restrict__ radii, float2* __restrict__ means2D,
                      float* __restrict__ depths, float* __restrict__ cov3D, float4* __restrict__ conic_opacity,
                      float* __restrict__ rgb, uint8_t* __restrict__ clamped, uint32_t* __restrict__ tiles_touched,
                      float* __restrict__ dcolor_ddir, float* __restrict__ blend_records) {
  __shared__ float4 s_sh[GS_BLOCK_1D / GS_WAVE][GS_WAVE * SH_THIRD4];
  // RECORDS: what the record takes of the geometry, parked per lane while the colour is evaluated (held in
  // registers it would make the kernel spill; fetched again at the end it would keep every wave waiting for loads)
  __shared__ float s_keep[RECORDS ? GS_BLOCK_1D / GS_WAVE : 1][RECORDS ? 12 * GS_WAVE : 1];
  const int slot = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  const bool live = slot < P;
  const int i = live ? slot : P - 1;  // lanes past the end keep step with a copy of the last Gaussian and store nothing
  CamParams cam;
  load_cam(Vg, PMg, camg, cam);
  const float mean[3] = {means[3 * (size_t)i], means[3 * (size_t)i + 1], means[3 * (size_t)i + 2]};
  const float sc[3] = {scales[3 * (size_t)i], scales[3 * (size_t)i + 1], scales[3 * (size_t)i + 2]};
  const float4 q4 = reinterpret_cast<const float4*>(rots)[i];
  const float q[4] = {q4.x, q4.y, q4.z, q4.w};
  float cov6[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  GeomOut g;
  bool in_front;
  const bool ok = geom_forward(mean, sc, mod, q, nullptr, cam, W, H, tanx, tany, fx, fy, gx, gy, cov6, in_front, g);
  if (live) {
    if (cov3D != nullptr) {  // (a caller that hands scales and rotations to the backward pass needs no copy)
      float2* c6v = reinterpret_cast<float2*>(cov3D + 6 * (size_t)i);  // 24-byte rows are 8-byte aligned
      c6v[0] = make_float2(cov6[0], cov6[1]);
      c6v[1] = make_float2(cov6[2], cov6[3]);
      c6v[2] = make_float2(cov6[4], cov6[5]);
    }
    radii[i] = ok ? g.radius : 0;
    depths[i] = ok ? g.depth : 0.f;
    means2D[i] = ok ? make_float2(g.px, g.py) : make_float2(0.f, 0.f);
    conic_opacity[i] = ok ? make_float4(g.conic[0], g.conic[1], g.conic[2], opac[i]) : make_float4(0.f, 0.f, 0.f, 0.f);
    if (tiles_touched) tiles_touched[i] = ok ? (g.rect.x1 - g.rect.x0) * (g.rect.y1 - g.rect.y0) : 0u;
  }
  if (RECORDS && ok) {  // (culled Gaussians have no record)
    float chan[5];
    AllMapGeom ag;
    all_map_geom(mean, sc, q4, cam.V, cam.campos, ag);
    all_map_channels(ag, chan);
    float* keep = s_keep[threadIdx.x / GS_WAVE] + (threadIdx.x & (GS_WAVE - 1));
    keep[0 * GS_WAVE] = g.px;
    keep[1 * GS_WAVE] = g.py;
    keep[2 * GS_WAVE] = g.conic[0];
    keep[3 * GS_WAVE] = g.conic[1];
    keep[4 * GS_WAVE] = g.conic[2];
    keep[5 * GS_WAVE] = opac[i];
    keep[6 * GS_WAVE] = g.depth;
#pragma unroll
    for (int k = 0; k < 5; k++) keep[(7 + k) * GS_WAVE] = chan[k];
  }

  float col[3] = {0.f, 0.f, 0.f};
  uint8_t clm[3] = {0, 0, 0};
  if (shs != nullptr && M > 0) {  // wave-uniform
    const float dx = mean[0] - cam.campos[0], dy = mean[1] - cam.campos[1], dz = mean[2] - cam.campos[2];
    const float dv[3] = {dx, dy, dz};
    const float len = sqrtf(dot3(dv, dv));
    const float x = dx / len, y = dy / len, z = dz / len;
    if (M == 16) {
      // colours only for Gaussians that survive culling: the rows of the others are not fetched
      const int lane = threadIdx.x & (GS_WAVE - 1);
      const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / GS_WAVE);
      const uint64_t need = gs_ballot(ok && live);
      const float4* wave_rows =
          reinterpret_cast<const float4*>(shs) + 12 * ((size_t)blockIdx.x * GS_BLOCK_1D + (size_t)wave * GS_WAVE);
      float B[16];
      sh_basis(x, y, z, B);
      float res[3] = {0.f, 0.f, 0.f};
      float4 va[4], vb[4];
      sh_third_fetch<0>(wave_rows, need, lane, va);
      sh_third_fetch<1>(wave_rows, need, lane, vb);
      float row[DERIV ? 48 : 1];
      sh_third_fold<0, DERIV>(D, B, va, s_sh[wave], lane, res, row);
      sh_third_fetch<2>(wave_rows, need, lane, va);
      sh_third_fold<1, DERIV>(D, B, vb, s_sh[wave], lane, res, row);
      sh_third_fold<2, DERIV>(D, B, va, s_sh[wave], lane, res, row);
      if (ok) {
#pragma unroll
        for (int ch = 0; ch < 3; ch++) {
          const float r = res[ch] + 0.5f;
          clm[ch] = r < 0.0f;
          col[ch] = fmaxf(r, 0.0f);
        }
      }
      if (DERIV) {
        // the wave's 64 x 9 numbers leave as nine runs of consecutive floats (through the LDS rows the
        // coefficients came in by); rows of culled Gaussians hold zeros
        float basis[16], dR[3][3];
        sh_basis_and_direction_derivative<true>(D, x, y, z, row, basis, dR[0], dR[1], dR[2]);
        float* lds = reinterpret_cast<float*>(s_sh[wave]);
        wave_sync_lds();
#pragma unroll
        for (int a = 0; a < 3; a++) {
#pragma unroll
          for (int ch = 0; ch < 3; ch++) lds[9 * lane + 3 * a + ch] = ok ? dR[a][ch] : 0.f;
        }
        wave_sync_lds();
        const size_t wave_first = (size_t)blockIdx.x * GS_BLOCK_1D + (size_t)wave * GS_WAVE;
        const size_t rows_left = (size_t)P > wave_first ? (size_t)P - wave_first : 0;
        float* out = dcolor_ddir + 9 * wave_first;
#pragma unroll
        for (int j = 0; j < 9; j++) {
          const size_t e = (size_t)j * GS_WAVE + (size_t)lane;
          if (e < 9 * rows_left) out[e] = lds[e];
        }
      }
    } else if (ok) {
      float c[3][16];
      const float* sh = shs + (size_t)i * M * 3;
#pragma unroll
      for (int k = 0; k < 16; k++) {
        const bool have = k < M;
        c[0][k] = have ? sh[3 * k] : 0.f;
        c[1][k] = have ? sh[3 * k + 1] : 0.f;
        c[2][k] = have ? sh[3 * k + 2] : 0.f;
      }
#pragma unroll
      for (int ch = 0; ch < 3; ch++) {
        const float res = sh_channel(D, x, y, z, c[ch]);
        clm[ch] = res < 0.0f;
        col[ch] = fmaxf(res, 0.0f);
      }
      if (DERIV && live) {
        float row[48], basis[16], dR[3][3];
#pragma unroll
        for (int k = 0; k < 16; k++) {
          row[3 * k] = c[0][k]; row[3 * k + 1] = c[1][k]; row[3 * k + 2] = c[2][k];
        }
        sh_basis_and_direction_derivative<true>(D, x, y, z, row, basis, dR[0], dR[1], dR[2]);
        float* dd = dcolor_ddir + 9 * (size_t)i;
#pragma unroll
        for (int a = 0; a < 3; a++) {
#pragma unroll
          for (int ch = 0; ch < 3; ch++) dd[3 * a + ch] = dR[a][ch];
        }
      }
    }
  }
  if (RECORDS) {
    // lane l stores 16-byte word (l & 3) of record 16 k + (l >> 2) in round k; in LDS a record's four words sit
    // 65 words apart, so that neither the writes, record-major, nor the reads, word-minor, pile up on a few banks
    constexpr int WORD_STRIDE = GS_WAVE + 1;
    static_assert(4 * WORD_STRIDE <= GS_WAVE * SH_THIRD4, "the records are staged where the coefficient rows were");
    const int lane = threadIdx.x & (GS_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / GS_WAVE);
    const uint64_t ok_m = gs_ballot(ok && live);
    if (ok_m != 0ull) {
      float4* mine = s_sh[wave];
      wave_sync_lds();  // (everyone has read what the buffer last held)
      const float* keep = s_keep[wave] + lane;
      mine[0 * WORD_STRIDE + lane] = make_float4(keep[0 * GS_WAVE], keep[1 * GS_WAVE], keep[2 * GS_WAVE], keep[3 * GS_WAVE]);
      mine[1 * WORD_STRIDE + lane] = make_float4(keep[4 * GS_WAVE], keep[5 * GS_WAVE], col[0], col[1]);
      mine[2 * WORD_STRIDE + lane] = make_float4(col[2], keep[7 * GS_WAVE], keep[8 * GS_WAVE], keep[9 * GS_WAVE]);
      mine[3 * WORD_STRIDE + lane] = make_float4(keep[10 * GS_WAVE], keep[11 * GS_WAVE], keep[6 * GS_WAVE], 0.f);
      wave_sync_lds();
      float4* out = reinterpret_cast<float4*>(blend_records) +
                    4 * ((size_t)blockIdx.x * GS_BLOCK_1D + (size_t)wave * GS_WAVE);  // the wave's first record
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const int rec = 16 * k + (lane >> 2);
        if ((ok_m >> rec) & 1ull) out[64 * k + lane] = mine[(lane & 3) * WORD_STRIDE + rec];
      }
    }
  }
  if (!live) return;
  rgb[3 * (size_t)i] = col[0];
  rgb[3 * (size_t)i + 1] = col[1];
  rgb[3 * (size_t)i + 2] = col[2];
  clamped[3 * (size_t)i] = clm[0];
  clamped[3 * (size_t)i + 1] = clm[1];
  clamped[3 * (size_t)i + 2] = clm[2];
}

// cuda_rasterizer/forward.cu:545-620.
__global__ void __launch_bounds__(GS_BLOCK_1D)
visible_filter_kernel(int P, const float* __restrict__ means, const float* __restrict__ scales, float mod,
                      const float* __restrict__ rots, const float* __restrict__ cov_pre,
                      const float* __restrict__ Vg, const float* __restrict__ PMg, int W, int H, float tanx,
                      float tany, float fx, float fy, uint32_t gx, uint32_t gy, int* __restrict__ radii) {
  const int i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (i >= P) return;
  CamParams cam;
  load_cam(Vg, PMg, nullptr, cam);
  const float mean[3] = {means[3 * (size_t)i], means[3 * (size_t)i + 1], means[3 * (size_t)i + 2]};
  float sc[3] = {0.f, 0.f, 0.f}, q[4] = {0.f, 0.f, 0.f, 0.f};
  if (!cov_pre) {
    sc[0] = scales[3 * (size_t)i]; sc[1] = scales[3 * (size_t)i + 1]; sc[2] = scales[3 * (size_t)i + 2];
    q[0] = rots[4 * (size_t)i]; q[1] = rots[4 * (size_t)i + 1]; q[2] = rots[4 * (size_t)i + 2];
    q[3] = rots[4 * (size_t)i + 3];
  }
  float cov6[6];
  GeomOut g;
  bool in_front;
  const bool ok = geom_forward(mean, sc, mod, q, cov_pre ? cov_pre + 6 * (size_t)i : nullptr, cam, W, H, tanx,
                               tany, fx, fy, gx, gy, cov6, in_front, g);
  radii[i] = ok ? g.radius : 0;
}

// cuda_rasterizer/rasterizer_impl.cu:58-70.
__global__ void __launch_bounds__(GS_BLOCK_1D)
mark_visible_kernel(int P, const float* __restrict__ means, const float* __restrict__ Vg,
                    uint8_t* __restrict__ present) {
  const int i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (i >= P) return;
  float V[16];
#pragma unroll
  for (int k = 0; k < 16; k++) V[k] = Vg[k];
  const float mean[3] = {means[3 * (size_t)i], means[3 * (size_t)i + 1], means[3 * (size_t)i + 2]};
  float pv[3];
  xform4x3(mean, V, pv);
  present[i] = pv[2] > 0.0f;
}

// Backward of the geometry and colour steps, one pass per Gaussian:
// cuda_rasterizer/backward.cu:69-199 (conic -> cov2D -> cov3D and mean),
// :296-312 (mean2D -> mean3D), :203-266 (cov3D -> scale, rotation) and the SH
// colour derivative (derivative of cuda_rasterizer/forward.cu:21-72, direction
// normalisation as cuda_rasterizer/auxiliary.h:161-171).  The 3D-covariance
// gradient stays in registers.  dL_dconic_opacity is packed [x, y, w, opacity].
// SAVED: the forward kernel's derivative of the colours with respect to the view direction is given, and the
// coefficient rows are not read.
template <bool SAVED>
__global__ void __launch_bounds__(GS_BLOCK_1D)
preprocess_bwd_kernel(int P, int D, int M, const float* __restrict__ means, const int* __restrict__ radii,
                      const float* __restrict__ shs, const uint8_t* __restrict__ clamped,
                      const float* __restrict__ scales, const float* __restrict__ rots, float mod,
                      const float* __restrict__ cov3D, const float* __restrict__ Vg, const float* __restrict__ PMg,
                      const float* __restrict__ camg, float h_x, float h_y, float tanx, float tany,
                      const float* __restrict__ dL_dmean2D, int mean2D_stride,
                      const float4* __restrict__ dL_dconic_opacity, const float* __restrict__ dL_dcolor,
                      float* __restrict__ dL_dmean3D, float* __restrict__ dL_dcov3D_out, float* __restrict__ dL_dsh,
                      float* __restrict__ dL_dscale, float* __restrict__ dL_drot, float* __restrict__ dL_dopacity,
                      const float* __restrict__ dcolor_ddir) {
  __shared__ float4 s_rows[GS_BLOCK_1D / GS_WAVE][SH_WAVE_ROWS4];
  const int lane = threadIdx.x & (GS_WAVE - 1), wave = threadIdx.x / GS_WAVE;
  const int raw_i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  const bool in_range = raw_i < P;
  const int i = in_range ? raw_i : P - 1;  // lanes past the end shadow the last Gaussian and store nothing
  const bool sh_mode = (SAVED || shs != nullptr) && M > 0 && (dL_dsh != nullptr);
  const bool sh_staged = sh_mode && M == 16;  // coefficient rows and their gradients go through LDS
  const float4 gco = dL_dconic_opacity[i];
  if (dL_dopacity && in_range) dL_dopacity[i] = gco.w;  // passthrough, rasterize_points.cu:191-194
  float gm[3] = {0.f, 0.f, 0.f}, gs_[3] = {0.f, 0.f, 0.f}, gq[4] = {0.f, 0.f, 0.f, 0.f};
  float gc[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const bool live = in_range && radii[i] > 0;
  const size_t wave_first = (size_t)blockIdx.x * GS_BLOCK_1D + (size_t)wave * GS_WAVE;
  float4* my_row = s_rows[wave] + lane * SH_ROW4;
  // (the coefficients are only needed for the colours' derivative with respect to the view direction; a caller
  // that kept the forward pass's nine numbers per Gaussian saves this kernel the 192-byte rows)
  if (sh_staged && !SAVED) {
    const uint64_t need = __ballot(live);
    if (need != 0ull)
      wave_rows_load(reinterpret_cast<const float4*>(shs) + wave_first * 12, need, s_rows[wave], lane);
  }
  if (live) {
    CamParams cam;
    load_cam(Vg, PMg, camg, cam);
    const float mean[3] = {means[3 * (size_t)i], means[3 * (size_t)i + 1], means[3 * (size_t)i + 2]};
    float c6[6];
    if (cov3D != nullptr) {
      const float2* c6v = reinterpret_cast<const float2*>(cov3D + 6 * (size_t)i);
      const float2 a = c6v[0], b = c6v[1], c = c6v[2];
      c6[0] = a.x; c6[1] = a.y; c6[2] = b.x; c6[3] = b.y; c6[4] = c.x; c6[5] = c.y;
    } else {
      // the forward pass's own operations on the same inputs: the same bits it would have stored
      const float sc[3] = {scales[3 * (size_t)i], scales[3 * (size_t)i + 1], scales[3 * (size_t)i + 2]};
      const float4 q4 = reinterpret_cast<const float4*>(rots)[i];
      const float q[4] = {q4.x, q4.y, q4.z, q4.w};
      M3 unused_m, unused_r;
      cov3d_from_scale_rot(sc, mod, q, c6, &unused_m, &unused_r);
    }
    Cov2DCtx cc;
    cov2d(mean, h_x, h_y, tanx, tany, c6, cam.V, cc);
    const float gcx = gco.x, gcy = gco.y, gcz = gco.z;
    const float x_mul = (cc.txtz < -cc.limx || cc.txtz > cc.limx) ? 0.f : 1.f;
    const float y_mul = (cc.tytz < -cc.limy || cc.tytz > cc.limy) ? 0.f : 1.f;
    const float a = cc.a, b = cc.b, c = cc.c;
    const float denom = a * c - b * b;
    float dL_da = 0.f, dL_db = 0.f, dL_dc = 0.f;
    const float denom2inv = 1.0f / ((denom * denom) + 0.0000001f);
    const M3& T = cc.T;
    const M3& Vr = cc.Vrk;
    if (denom2inv != 0.f) {
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
    }
    float u0[3], u1[3];
#pragma unroll
    for (int k = 0; k < 3; k++) {
      u0[k] = (T.m[0][0] * Vr.m[k][0] + T.m[0][1] * Vr.m[k][1]) + T.m[0][2] * Vr.m[k][2];
      u1[k] = (T.m[1][0] * Vr.m[k][0] + T.m[1][1] * Vr.m[k][1]) + T.m[1][2] * Vr.m[k][2];
    }
    float dT0[3], dT1[3];
#pragma unroll
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
    xformVec4x3T(dt, cam.V, gm);

    const float* PM = cam.PM;
    float mh[4];
    xform4x4(mean, PM, mh);
    const float m_w = 1.0f / (mh[3] + 0.0000001f);
    const float mul1 = (((PM[0] * mean[0] + PM[4] * mean[1]) + PM[8] * mean[2]) + PM[12]) * m_w * m_w;
    const float mul2 = (((PM[1] * mean[0] + PM[5] * mean[1]) + PM[9] * mean[2]) + PM[13]) * m_w * m_w;
    const float g2x = dL_dmean2D[(size_t)mean2D_stride * i], g2y = dL_dmean2D[(size_t)mean2D_stride * i + 1];
    gm[0] += (PM[0] * m_w - PM[3] * mul1) * g2x + (PM[1] * m_w - PM[3] * mul2) * g2y;
    gm[1] += (PM[4] * m_w - PM[7] * mul1) * g2x + (PM[5] * m_w - PM[7] * mul2) * g2y;
    gm[2] += (PM[8] * m_w - PM[11] * mul1) * g2x + (PM[9] * m_w - PM[11] * mul2) * g2y;

    if (sh_mode) {
      const float* sh = shs + (size_t)i * M * 3;
      float* gsh = dL_dsh + (size_t)i * M * 3;
      // the Gaussian's coefficients, in registers; 16-coefficient rows (192 bytes) move as twelve 16-byte words
      float shv[48];
      if (!SAVED) {
        if (M == 16) {
#pragma unroll
          for (int j = 0; j < 12; j++) {
            const float4 v = my_row[j];
            shv[4 * j] = v.x;
            shv[4 * j + 1] = v.y;
            shv[4 * j + 2] = v.z;
            shv[4 * j + 3] = v.w;
          }
        } else {
#pragma unroll
          for (int e = 0; e < 48; e++) shv[e] = e < 3 * M ? sh[e] : 0.f;
        }
      }
      const float d0[3] = {mean[0] - cam.campos[0], mean[1] - cam.campos[1], mean[2] - cam.campos[2]};
      const float s2 = dot3(d0, d0);
      const float len = sqrtf(s2);
      const float x = d0[0] / len, y = d0[1] / len, z = d0[2] / len;
      float gr[3];
#pragma unroll
      for (int ch = 0; ch < 3; ch++) gr[ch] = dL_dcolor[3 * (size_t)i + ch] * (clamped[3 * (size_t)i + ch] ? 0.f : 1.f);
      float basis[16];
      float dRdx[3], dRdy[3], dRdz[3];
      if (SAVED) {
        sh_basis_and_direction_derivative<false>(D, x, y, z, nullptr, basis, dRdx, dRdy, dRdz);
        const float* dd = dcolor_ddir + 9 * (size_t)i;
#pragma unroll
        for (int ch = 0; ch < 3; ch++) {
          dRdx[ch] = dd[ch];
          dRdy[ch] = dd[3 + ch];
          dRdz[ch] = dd[6 + ch];
        }
      } else {
        sh_basis_and_direction_derivative<true>(D, x, y, z, shv, basis, dRdx, dRdy, dRdz);
      }
      if (M == 16) {
#pragma unroll
        for (int j = 0; j < 12; j++)
          my_row[j] = make_float4(basis[(4 * j) / 3] * gr[(4 * j) % 3], basis[(4 * j + 1) / 3] * gr[(4 * j + 1) % 3],
                                basis[(4 * j + 2) / 3] * gr[(4 * j + 2) % 3], basis[(4 * j + 3) / 3] * gr[(4 * j + 3) % 3]);
      } else {
        for (int k = 0; k < M; k++) {
          const float bk = k < 16 ? basis[k] : 0.f;
          gsh[3 * k] = bk * gr[0];
          gsh[3 * k + 1] = bk * gr[1];
          gsh[3 * k + 2] = bk * gr[2];
        }
      }
      const float gdir[3] = {dot3(dRdx, gr), dot3(dRdy, gr), dot3(dRdz, gr)};
      const float inv32 = 1.0f / sqrtf(s2 * s2 * s2);
      gm[0] += ((s2 - d0[0] * d0[0]) * gdir[0] - d0[1] * d0[0] * gdir[1] - d0[2] * d0[0] * gdir[2]) * inv32;
      gm[1] += (-d0[0] * d0[1] * gdir[0] + (s2 - d0[1] * d0[1]) * gdir[1] - d0[2] * d0[1] * gdir[2]) * inv32;
      gm[2] += (-d0[0] * d0[2] * gdir[0] - d0[1] * d0[2] * gdir[1] + (s2 - d0[2] * d0[2]) * gdir[2]) * inv32;
    }

    if (scales) {
      const float sc[3] = {scales[3 * (size_t)i], scales[3 * (size_t)i + 1], scales[3 * (size_t)i + 2]};
      const float4 q4 = reinterpret_cast<const float4*>(rots)[i];
      const float q[4] = {q4.x, q4.y, q4.z, q4.w};
      M3 Mm, R;
      float tmp6[6];
      cov3d_from_scale_rot(sc, mod, q, tmp6, &Mm, &R);
      const float s[3] = {mod * sc[0], mod * sc[1], mod * sc[2]};
      M3 dSig = m3_cols(gc[0], 0.5f * gc[1], 0.5f * gc[2], 0.5f * gc[1], gc[3], 0.5f * gc[4], 0.5f * gc[2],
                        0.5f * gc[4], gc[5]);
      M3 M2;
#pragma unroll
      for (int cI = 0; cI < 3; cI++)
#pragma unroll
        for (int rI = 0; rI < 3; rI++) M2.m[cI][rI] = 2.0f * Mm.m[cI][rI];
      M3 dM = m3_mul(M2, dSig);
      M3 Rt = m3_T(R);
      M3 dMt = m3_T(dM);
      gs_[0] = dot3(Rt.m[0], dMt.m[0]);
      gs_[1] = dot3(Rt.m[1], dMt.m[1]);
      gs_[2] = dot3(Rt.m[2], dMt.m[2]);
#pragma unroll
      for (int k = 0; k < 3; k++) {
        dMt.m[0][k] *= s[0];
        dMt.m[1][k] *= s[1];
        dMt.m[2][k] *= s[2];
      }
      const float r = q[0], x = q[1], y = q[2], z = q[3];
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
  } else if (sh_mode && in_range) {
    float* gsh = dL_dsh + (size_t)i * M * 3;
    if (M == 16) {
#pragma unroll
      for (int j = 0; j < 12; j++) my_row[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
      for (int k = 0; k < 3 * M; k++) gsh[k] = 0.f;
    }
  }
  if (sh_staged) {
    const long long left = (long long)P - (long long)wave_first;
    if (left > 0)
      wave_rows_store(reinterpret_cast<float4*>(dL_dsh) + wave_first * 12, left < GS_WAVE ? (int)left : GS_WAVE,
                      s_rows[wave], lane);
  }
  if (!in_range) return;
  dL_dmean3D[3 * (size_t)i] = gm[0];
  dL_dmean3D[3 * (size_t)i + 1] = gm[1];
  dL_dmean3D[3 * (size_t)i + 2] = gm[2];
  if (dL_dscale) {
    dL_dscale[3 * (size_t)i] = gs_[0];
    dL_dscale[3 * (size_t)i + 1] = gs_[1];
    dL_dscale[3 * (size_t)i + 2] = gs_[2];
  }
  if (dL_drot) reinterpret_cast<float4*>(dL_drot)[i] = make_float4(gq[0], gq[1], gq[2], gq[3]);
  if (dL_dcov3D_out) {
#pragma unroll
    for (int k = 0; k < 6; k++) dL_dcov3D_out[6 * (size_t)i + k] = gc[k];
  }
}

}  // namespace

int launch_preprocess_fwd(const PreprocessFwdArgs& a, hipStream_t stream) {
  if (a.P <= 0) return 0;
  const uint32_t gx = (a.W + GS_TILE_X - 1) / GS_TILE_X, gy = (a.H + GS_TILE_Y - 1) / GS_TILE_Y;
  const float fy = a.H / (2.0f * a.tany);  // cuda_rasterizer/rasterizer_impl.cu:371-372
  const float fx = a.W / (2.0f * a.tanx);
  const int blocks = (a.P + GS_BLOCK_1D - 1) / GS_BLOCK_1D;
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(GS_BLOCK_1D), 0, stream, a.P, a.D, a.M, a.means3D, a.scales,
                       a.scale_modifier, a.rotations, a.opacities, a.shs, a.viewmatrix, a.projmatrix, a.campos, a.W,
                       a.H, a.tanx, a.tany, fx, fy, gx, gy, a.radii, (float2*)a.means2D, a.depths, a.cov3D,
                       (float4*)a.conic_opacity, a.rgb, a.clamped, a.tiles_touched, a.dcolor_ddir, a.blend_records);
  };
  const bool deriv = a.dcolor_ddir != nullptr && a.shs != nullptr && a.M > 0;
  if (a.blend_records != nullptr) {
    if (deriv) go(preprocess_fwd_kernel<true, true>);
    else go(preprocess_fwd_kernel<false, true>);
  } else {
    if (deriv) go(preprocess_fwd_kernel<true, false>);
    else go(preprocess_fwd_kernel<false, false>);
  }
  return 0;
}

int launch_visible_filter(int P, const float* means, const float* scales, float mod, const float* rots,
                          const float* cov_pre, const float* V, const float* PM, int W, int H, float tanx,
                          float tany, int* radii, hipStream_t stream) {
  if (P <= 0) return 0;
  const uint32_t gx = (W + GS_TILE_X - 1) / GS_TILE_X, gy = (H + GS_TILE_Y - 1) / GS_TILE_Y;
  const float fy = H / (2.0f * tany);
  const float fx = W / (2.0f * tanx);
  const int blocks = (P + GS_BLOCK_1D - 1) / GS_BLOCK_1D;
  hipLaunchKernelGGL(visible_filter_kernel, dim3(blocks), dim3(GS_BLOCK_1D), 0, stream, P, means, scales, mod, rots,
                     cov_pre, V, PM, W, H, tanx, tany, fx, fy, gx, gy, radii);
  return 0;
}

int launch_mark_visible(int P, const float* means, const float* V, uint8_t* present, hipStream_t stream) {
  if (P <= 0) return 0;
  const int blocks = (P + GS_BLOCK_1D - 1) / GS_BLOCK_1D;
  hipLaunchKernelGGL(mark_visible_kernel, dim3(blocks), dim3(GS_BLOCK_1D), 0, stream, P, means, V, present);
  return 0;
}

int launch_preprocess_bwd(const PreprocessBwdArgs& a, hipStream_t stream) {
  if (a.P <= 0) return 0;
  const float h_y = a.H / (2.0f * a.tany);
  const float h_x = a.W / (2.0f * a.tanx);
  const int blocks = (a.P + GS_BLOCK_1D - 1) / GS_BLOCK_1D;
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(GS_BLOCK_1D), 0, stream, a.P, a.D, a.M, a.means3D, a.radii, a.shs,
                       a.clamped, a.scales, a.rotations, a.scale_modifier, a.cov3D, a.viewmatrix, a.projmatrix,
                       a.campos, h_x, h_y, a.tanx, a.tany, a.dL_dmean2D, a.mean2D_stride,
                       (const float4*)a.dL_dconic_opacity, a.dL_dcolor, a.dL_dmean3D, a.dL_dcov3D, a.dL_dsh,
                       a.dL_dscale, a.dL_drot, a.dL_dopacity, a.dcolor_ddir);
  };
  if (a.dcolor_ddir != nullptr) go(preprocess_bwd_kernel<true>);
  else go(preprocess_bwd_kernel<false>);
  return 0;
}

}  // namespace gs
