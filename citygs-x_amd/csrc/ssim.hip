// Per-pixel masked L1 and SSIM maps of the training loss and their backward pass:
// pixelwise_l1_with_mask / pixelwise_ssim_with_mask (utils/loss_utils.py:88-132; window: create_window,
// :27-43; called per view at gaussian_renderer/loss_distribution.py:267-279).  The reference runs five
// grouped 11x11 convolutions plus about fifteen elementwise kernels forward and their autograd mirror
// backward; here each direction is one kernel.
//
// A 256-thread workgroup owns a 32x16 block of one channel.  It stages the 42x26 neighbourhood of both
// images in LDS (zeros outside the image = the convolution's zero padding; all of a thread's loads go out before
// its first LDS write, so a block waits for memory once) and runs the Gaussian window as a horizontal then a
// vertical 11-tap pass over the five products (x, y, xx, yy, xy).  The kernel is bound by instruction issue, so
// the passes are blocked in registers: a thread of the horizontal pass produces four adjacent columns from the
// 14 staged values they share, a thread of the vertical pass two adjacent rows from 12 rows of partial sums
// (every staged value is read about three times instead of eleven), and a tap is one fused multiply-add.  Then
// the SSIM value and, for the backward pass, its three partial derivatives with respect to the window means of
// x, xx and xy (already times the mask).  Backward: those three maps times the upstream gradient are spread back
// through the same (symmetric) window by the same two passes, and
//   dL/dx = conv(d_mu) + 2 x conv(d_xx) + y conv(d_xy) + g_l1 * mask * sign(x - y).
// 20 bytes per pixel and channel forward (+12 for the derivative maps), 36 backward.
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

constexpr int SBX = 32, SBY = 16;   // block of output pixels
constexpr int SR = 5;               // window radius
constexpr int STX = SBX + 2 * SR;   // staged tile: 42 columns
constexpr int STY = SBY + 2 * SR;   //              26 rows
constexpr int SPITCH = STX + 1;     // odd row pitch
constexpr int SS_THREADS = 256;
constexpr int STAGE_ROUNDS = (STX * STY + SS_THREADS - 1) / SS_THREADS;
constexpr int HG = 4;               // adjacent columns per thread of the horizontal pass
constexpr int VG = 2;               // adjacent rows per thread of the vertical pass
static_assert(STY * (SBX / HG) <= SS_THREADS, "one round of the horizontal pass");
static_assert((SBX * SBY) / VG == SS_THREADS, "one thread per pair of output rows");

struct SsimWindow {
  float w[2 * SR + 1];
};

// Horizontal pass: s_h[q][r][c] = sum_t w[t] * product_q(r, c + t) for the STY staged rows and the SBX output
// columns; product(r, c, v) fills the NQ quantities at staged position (r, c).
template <int NQ, typename F>
__device__ __forceinline__ void horizontal_pass(const SsimWindow& win, float (*s_h)[STY][SBX], F&& product) {
  const int item = threadIdx.x;
  if (item >= STY * (SBX / HG)) return;
  const int r = item / (SBX / HG), c0 = (item - r * (SBX / HG)) * HG;
  float v[HG + 2 * SR][NQ];
#pragma unroll
  for (int i = 0; i < HG + 2 * SR; i++) product(r, c0 + i, v[i]);
#pragma unroll
  for (int o = 0; o < HG; o++) {
    float acc[NQ];
#pragma unroll
    for (int q = 0; q < NQ; q++) acc[q] = 0.f;
#pragma unroll
    for (int t = 0; t < 2 * SR + 1; t++) {
#pragma unroll
      for (int q = 0; q < NQ; q++) acc[q] = __builtin_fmaf(win.w[t], v[o + t][q], acc[q]);
    }
#pragma unroll
    for (int q = 0; q < NQ; q++) s_h[q][r][c0 + o] = acc[q];
  }
}

// Vertical pass for output rows ty and ty + 1 of column tx: out[o][q] = sum_t w[t] * s_h[q][ty + o + t][tx].
template <int NQ>
__device__ __forceinline__ void vertical_pass(const SsimWindow& win, const float (*s_h)[STY][SBX], int ty, int tx,
                                              float (*out)[NQ]) {
  float v[VG + 2 * SR][NQ];
#pragma unroll
  for (int i = 0; i < VG + 2 * SR; i++) {
#pragma unroll
    for (int q = 0; q < NQ; q++) v[i][q] = s_h[q][ty + i][tx];
  }
#pragma unroll
  for (int o = 0; o < VG; o++) {
#pragma unroll
    for (int q = 0; q < NQ; q++) out[o][q] = 0.f;
#pragma unroll
    for (int t = 0; t < 2 * SR + 1; t++) {
#pragma unroll
      for (int q = 0; q < NQ; q++) out[o][q] = __builtin_fmaf(win.w[t], v[o + t][q], out[o][q]);
    }
  }
}

__global__ void __launch_bounds__(SS_THREADS)
ssim_l1_fwd_kernel(int H, int W, const float* __restrict__ img1, const float* __restrict__ img2,
                   const uint8_t* __restrict__ mask, SsimWindow win, float* __restrict__ l1_map,
                   float* __restrict__ ssim_map, float* __restrict__ d_mu, float* __restrict__ d_xx,
                   float* __restrict__ d_xy) {
  __shared__ float s_a[STY][SPITCH];
  __shared__ float s_b[STY][SPITCH];
  __shared__ float s_h[5][STY][SBX];
  // Workgroups go to the eight XCDs in turn; dealt out this way an XCD holds a contiguous run of blocks, so the
  // halo that neighbouring blocks share is fetched into one second-level cache once, not into up to eight.
  const uint32_t blocks_xy = gridDim.x * gridDim.y;
  const uint32_t b = xcd_contiguous_index(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z),
                                          blocks_xy * gridDim.z);
  const uint32_t bz = b / blocks_xy, by = (b % blocks_xy) / gridDim.x, bx = b % gridDim.x;
  const size_t plane = (size_t)bz * H * W;
  const int x0 = bx * SBX, y0 = by * SBY;
  {
    float va[STAGE_ROUNDS], vb[STAGE_ROUNDS];
#pragma unroll
    for (int k = 0; k < STAGE_ROUNDS; k++) {
      const int e = threadIdx.x + k * SS_THREADS;
      const int r = e / STX, c = e - r * STX;
      const int y = y0 + r - SR, x = x0 + c - SR;
      const bool in = e < STX * STY && y >= 0 && y < H && x >= 0 && x < W;
      va[k] = in ? img1[plane + (size_t)y * W + x] : 0.f;
      vb[k] = in ? img2[plane + (size_t)y * W + x] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < STAGE_ROUNDS; k++) {
      const int e = threadIdx.x + k * SS_THREADS;
      const int r = e / STX, c = e - r * STX;
      if (e < STX * STY) {
        s_a[r][c] = va[k];
        s_b[r][c] = vb[k];
      }
    }
  }
  __syncthreads();
  horizontal_pass<5>(win, s_h, [&](int r, int c, float* v) {
    const float p = s_a[r][c], q = s_b[r][c];
    v[0] = p; v[1] = q; v[2] = p * p; v[3] = q * q; v[4] = p * q;
  });
  __syncthreads();
  const int tx = threadIdx.x % SBX, ty = (threadIdx.x / SBX) * VG;
  const int x = x0 + tx;
  if (x >= W) return;
  float st2[VG][5];
  vertical_pass<5>(win, s_h, ty, tx, st2);
  const float C1 = (float)(0.01 * 0.01), C2 = (float)(0.03 * 0.03);
#pragma unroll
  for (int o = 0; o < VG; o++) {
    const int y = y0 + ty + o;
    if (y >= H) break;
    const float* st = st2[o];
    const float mu1 = st[0], mu2 = st[1];
    const float mu1_sq = mu1 * mu1, mu2_sq = mu2 * mu2, mu12 = mu1 * mu2;
    const float s1 = st[2] - mu1_sq, s2 = st[3] - mu2_sq, s12 = st[4] - mu12;
    const float A1 = 2 * mu12 + C1, A2 = 2 * s12 + C2, B1 = (mu1_sq + mu2_sq) + C1, B2 = (s1 + s2) + C2;
    const float S = (A1 * A2) / (B1 * B2);
    const float mk = mask ? (float)(mask[(size_t)y * W + x] != 0) : 1.0f;
    const size_t oidx = plane + (size_t)y * W + x;
    const float p = s_a[ty + o + SR][tx + SR], q = s_b[ty + o + SR][tx + SR];
    ssim_map[oidx] = S * mk;
    l1_map[oidx] = fabsf(p - q) * mk;
    if (d_mu != nullptr) {
      d_mu[oidx] = mk * ((2 * mu2 * (A2 - A1)) / (B1 * B2) - S * (2 * mu1 / B1) + S * (2 * mu1 / B2));
      d_xx[oidx] = mk * (-S / B2);
      d_xy[oidx] = mk * (2 * A1 / (B1 * B2));
    }
  }
}

__global__ void __launch_bounds__(SS_THREADS)
ssim_l1_bwd_kernel(int H, int W, const float* __restrict__ img1, const float* __restrict__ img2,
                   const uint8_t* __restrict__ mask, SsimWindow win, const float* __restrict__ g_l1,
                   const float* __restrict__ g_ssim, const float* __restrict__ d_mu,
                   const float* __restrict__ d_xx, const float* __restrict__ d_xy, float* __restrict__ dimg1) {
  __shared__ float s_d[3][STY][SPITCH];
  __shared__ float s_h[3][STY][SBX];
  // Workgroups go to the eight XCDs in turn; dealt out this way an XCD holds a contiguous run of blocks, so the
  // halo that neighbouring blocks share is fetched into one second-level cache once, not into up to eight.
  const uint32_t blocks_xy = gridDim.x * gridDim.y;
  const uint32_t b = xcd_contiguous_index(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z),
                                          blocks_xy * gridDim.z);
  const uint32_t bz = b / blocks_xy, by = (b % blocks_xy) / gridDim.x, bx = b % gridDim.x;
  const size_t plane = (size_t)bz * H * W;
  const int x0 = bx * SBX, y0 = by * SBY;
  {
    float vg[STAGE_ROUNDS], v0[STAGE_ROUNDS], v1[STAGE_ROUNDS], v2[STAGE_ROUNDS];
#pragma unroll
    for (int k = 0; k < STAGE_ROUNDS; k++) {
      const int e = threadIdx.x + k * SS_THREADS;
      const int r = e / STX, c = e - r * STX;
      const int y = y0 + r - SR, x = x0 + c - SR;
      const bool in = e < STX * STY && y >= 0 && y < H && x >= 0 && x < W;
      const size_t o = plane + (size_t)(in ? y : 0) * W + (in ? x : 0);
      vg[k] = in && g_ssim ? g_ssim[o] : 0.f;
      v0[k] = in ? d_mu[o] : 0.f;
      v1[k] = in ? d_xx[o] : 0.f;
      v2[k] = in ? d_xy[o] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < STAGE_ROUNDS; k++) {
      const int e = threadIdx.x + k * SS_THREADS;
      const int r = e / STX, c = e - r * STX;
      if (e < STX * STY) {
        s_d[0][r][c] = vg[k] * v0[k];
        s_d[1][r][c] = vg[k] * v1[k];
        s_d[2][r][c] = vg[k] * v2[k];
      }
    }
  }
  __syncthreads();
  horizontal_pass<3>(win, s_h, [&](int r, int c, float* v) {
    v[0] = s_d[0][r][c]; v[1] = s_d[1][r][c]; v[2] = s_d[2][r][c];
  });
  __syncthreads();
  const int tx = threadIdx.x % SBX, ty = (threadIdx.x / SBX) * VG;
  const int x = x0 + tx;
  if (x >= W) return;
  float cv2[VG][3];
  vertical_pass<3>(win, s_h, ty, tx, cv2);
#pragma unroll
  for (int i = 0; i < VG; i++) {
    const int y = y0 + ty + i;
    if (y >= H) break;
    const float* cv = cv2[i];
    const size_t o = plane + (size_t)y * W + x;
    const float p = img1[o], q = img2[o];
    const float mk = mask ? (float)(mask[(size_t)y * W + x] != 0) : 1.0f;
    const float d = p - q;
    const float sg = d > 0.f ? 1.0f : (d < 0.f ? -1.0f : 0.0f);
    const float gl = g_l1 ? g_l1[o] : 0.f;
    dimg1[o] = ((cv[0] + 2 * p * cv[1]) + q * cv[2]) + gl * mk * sg;
  }
}

SsimWindow make_window() {
  // create_window (utils/loss_utils.py:27-43): exp in double, stored as float32, divided by the float32 sum
  SsimWindow w;
  float sum = 0.f;
  for (int i = 0; i < 2 * SR + 1; i++) {
    w.w[i] = (float)exp(-(double)((i - SR) * (i - SR)) / (2.0 * 1.5 * 1.5));
    sum += w.w[i];
  }
  for (int i = 0; i < 2 * SR + 1; i++) w.w[i] = w.w[i] / sum;
  return w;
}

}  // namespace

int launch_ssim_l1_fwd(int C, int H, int W, const float* img1, const float* img2, const uint8_t* mask,
                       float* l1_map, float* ssim_map, float* d_mu, float* d_xx, float* d_xy, hipStream_t stream) {
  if (C <= 0 || H <= 0 || W <= 0) return 0;
  const dim3 grid((W + SBX - 1) / SBX, (H + SBY - 1) / SBY, C);
  hipLaunchKernelGGL(ssim_l1_fwd_kernel, grid, dim3(SS_THREADS), 0, stream, H, W, img1, img2, mask, make_window(), l1_map,
                     ssim_map, d_mu, d_xx, d_xy);
  return 0;
}

int launch_ssim_l1_bwd(int C, int H, int W, const float* img1, const float* img2, const uint8_t* mask,
                       const float* g_l1, const float* g_ssim, const float* d_mu, const float* d_xx,
                       const float* d_xy, float* dimg1, hipStream_t stream) {
  if (C <= 0 || H <= 0 || W <= 0) return 0;
  const dim3 grid((W + SBX - 1) / SBX, (H + SBY - 1) / SBY, C);
  hipLaunchKernelGGL(ssim_l1_bwd_kernel, grid, dim3(SS_THREADS), 0, stream, H, W, img1, img2, mask, make_window(), g_l1,
                     g_ssim, d_mu, d_xx, d_xy, dimg1);
  return 0;
}

}  // namespace gs
