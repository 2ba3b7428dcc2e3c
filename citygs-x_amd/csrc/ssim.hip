// Per-pixel masked L1 and SSIM maps of the training loss and their backward pass:
// pixelwise_l1_with_mask / pixelwise_ssim_with_mask (utils/loss_utils.py:88-132; window: create_window,
// :27-43; called per view at gaussian_renderer/loss_distribution.py:267-279).  The reference runs five
// grouped 11x11 convolutions plus about fifteen elementwise kernels forward and their autograd mirror
// backward; here each direction is one kernel.
//
// A 256-thread workgroup owns a 16x16 block of one channel.  It stages the 26x26 neighbourhood of both
// images in LDS (zeros outside the image = the convolution's zero padding), runs the Gaussian window as a
// horizontal then a vertical 11-tap pass over the five products (x, y, xx, yy, xy), evaluates the SSIM value
// and, for the backward pass, its three partial derivatives with respect to the window means of x, xx and
// xy (already times the mask).  Backward: those three maps times the upstream gradient are spread back
// through the same (symmetric) window by the same two passes, and
//   dL/dx = conv(d_mu) + 2 x conv(d_xx) + y conv(d_xy) + g_l1 * mask * sign(x - y).
// 20 bytes per pixel and channel forward (+12 for the derivative maps), 36 backward.
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

constexpr int SB = 16;            // block edge
constexpr int SR = 5;             // window radius
constexpr int ST = SB + 2 * SR;   // staged tile edge (26)

struct SsimWindow {
  float w[2 * SR + 1];
};

// rows of `nq` quantities: horizontal pass from the staged tile(s) into s_h[q][ST][SB]
template <int NQ, typename F>
__device__ __forceinline__ void horizontal_pass(const SsimWindow& win, float (*s_h)[ST][SB], F&& product) {
  for (int item = threadIdx.x; item < ST * SB; item += SB * SB) {
    const int r = item / SB, c = item - r * SB;
    float acc[NQ];
#pragma unroll
    for (int q = 0; q < NQ; q++) acc[q] = 0.f;
#pragma unroll
    for (int t = 0; t < 2 * SR + 1; t++) {
      float v[NQ];
      product(r, c + t, v);
#pragma unroll
      for (int q = 0; q < NQ; q++) acc[q] += win.w[t] * v[q];
    }
#pragma unroll
    for (int q = 0; q < NQ; q++) s_h[q][r][c] = acc[q];
  }
}

template <int NQ>
__device__ __forceinline__ void vertical_pass(const SsimWindow& win, const float (*s_h)[ST][SB], int ty, int tx,
                                              float* out) {
#pragma unroll
  for (int q = 0; q < NQ; q++) out[q] = 0.f;
#pragma unroll
  for (int t = 0; t < 2 * SR + 1; t++) {
#pragma unroll
    for (int q = 0; q < NQ; q++) out[q] += win.w[t] * s_h[q][ty + t][tx];
  }
}

__global__ void __launch_bounds__(SB * SB)
ssim_l1_fwd_kernel(int H, int W, const float* __restrict__ img1, const float* __restrict__ img2,
                   const uint8_t* __restrict__ mask, SsimWindow win, float* __restrict__ l1_map,
                   float* __restrict__ ssim_map, float* __restrict__ d_mu, float* __restrict__ d_xx,
                   float* __restrict__ d_xy) {
  __shared__ float s_a[ST][ST + 1];
  __shared__ float s_b[ST][ST + 1];
  __shared__ float s_h[5][ST][SB];
  const size_t plane = (size_t)blockIdx.z * H * W;
  const int x0 = blockIdx.x * SB, y0 = blockIdx.y * SB;
  for (int e = threadIdx.x; e < ST * ST; e += SB * SB) {
    const int r = e / ST, c = e - r * ST;
    const int y = y0 + r - SR, x = x0 + c - SR;
    const bool in = y >= 0 && y < H && x >= 0 && x < W;
    s_a[r][c] = in ? img1[plane + (size_t)y * W + x] : 0.f;
    s_b[r][c] = in ? img2[plane + (size_t)y * W + x] : 0.f;
  }
  __syncthreads();
  horizontal_pass<5>(win, s_h, [&](int r, int c, float* v) {
    const float p = s_a[r][c], q = s_b[r][c];
    v[0] = p; v[1] = q; v[2] = p * p; v[3] = q * q; v[4] = p * q;
  });
  __syncthreads();
  const int ty = threadIdx.x / SB, tx = threadIdx.x - ty * SB;
  const int y = y0 + ty, x = x0 + tx;
  if (y >= H || x >= W) return;
  float st[5];
  vertical_pass<5>(win, s_h, ty, tx, st);
  const float C1 = (float)(0.01 * 0.01), C2 = (float)(0.03 * 0.03);
  const float mu1 = st[0], mu2 = st[1];
  const float mu1_sq = mu1 * mu1, mu2_sq = mu2 * mu2, mu12 = mu1 * mu2;
  const float s1 = st[2] - mu1_sq, s2 = st[3] - mu2_sq, s12 = st[4] - mu12;
  const float A1 = 2 * mu12 + C1, A2 = 2 * s12 + C2, B1 = (mu1_sq + mu2_sq) + C1, B2 = (s1 + s2) + C2;
  const float S = (A1 * A2) / (B1 * B2);
  const float mk = mask ? (float)(mask[(size_t)y * W + x] != 0) : 1.0f;
  const size_t o = plane + (size_t)y * W + x;
  const float p = s_a[ty + SR][tx + SR], q = s_b[ty + SR][tx + SR];
  ssim_map[o] = S * mk;
  l1_map[o] = fabsf(p - q) * mk;
  if (d_mu != nullptr) {
    d_mu[o] = mk * ((2 * mu2 * (A2 - A1)) / (B1 * B2) - S * (2 * mu1 / B1) + S * (2 * mu1 / B2));
    d_xx[o] = mk * (-S / B2);
    d_xy[o] = mk * (2 * A1 / (B1 * B2));
  }
}

__global__ void __launch_bounds__(SB * SB)
ssim_l1_bwd_kernel(int H, int W, const float* __restrict__ img1, const float* __restrict__ img2,
                   const uint8_t* __restrict__ mask, SsimWindow win, const float* __restrict__ g_l1,
                   const float* __restrict__ g_ssim, const float* __restrict__ d_mu,
                   const float* __restrict__ d_xx, const float* __restrict__ d_xy, float* __restrict__ dimg1) {
  __shared__ float s_d[3][ST][ST + 1];
  __shared__ float s_h[3][ST][SB];
  const size_t plane = (size_t)blockIdx.z * H * W;
  const int x0 = blockIdx.x * SB, y0 = blockIdx.y * SB;
  for (int e = threadIdx.x; e < ST * ST; e += SB * SB) {
    const int r = e / ST, c = e - r * ST;
    const int y = y0 + r - SR, x = x0 + c - SR;
    const bool in = y >= 0 && y < H && x >= 0 && x < W;
    const size_t o = plane + (size_t)(in ? y : 0) * W + (in ? x : 0);
    const float g = in && g_ssim ? g_ssim[o] : 0.f;
    s_d[0][r][c] = in ? g * d_mu[o] : 0.f;
    s_d[1][r][c] = in ? g * d_xx[o] : 0.f;
    s_d[2][r][c] = in ? g * d_xy[o] : 0.f;
  }
  __syncthreads();
  horizontal_pass<3>(win, s_h, [&](int r, int c, float* v) {
    v[0] = s_d[0][r][c]; v[1] = s_d[1][r][c]; v[2] = s_d[2][r][c];
  });
  __syncthreads();
  const int ty = threadIdx.x / SB, tx = threadIdx.x - ty * SB;
  const int y = y0 + ty, x = x0 + tx;
  if (y >= H || x >= W) return;
  float cv[3];
  vertical_pass<3>(win, s_h, ty, tx, cv);
  const size_t o = plane + (size_t)y * W + x;
  const float p = img1[o], q = img2[o];
  const float mk = mask ? (float)(mask[(size_t)y * W + x] != 0) : 1.0f;
  const float d = p - q;
  const float sg = d > 0.f ? 1.0f : (d < 0.f ? -1.0f : 0.0f);
  const float gl = g_l1 ? g_l1[o] : 0.f;
  dimg1[o] = ((cv[0] + 2 * p * cv[1]) + q * cv[2]) + gl * mk * sg;
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
  const dim3 grid((W + SB - 1) / SB, (H + SB - 1) / SB, C);
  hipLaunchKernelGGL(ssim_l1_fwd_kernel, grid, dim3(SB * SB), 0, stream, H, W, img1, img2, mask, make_window(), l1_map,
                     ssim_map, d_mu, d_xx, d_xy);
  return 0;
}

int launch_ssim_l1_bwd(int C, int H, int W, const float* img1, const float* img2, const uint8_t* mask,
                       const float* g_l1, const float* g_ssim, const float* d_mu, const float* d_xx,
                       const float* d_xy, float* dimg1, hipStream_t stream) {
  if (C <= 0 || H <= 0 || W <= 0) return 0;
  const dim3 grid((W + SB - 1) / SB, (H + SB - 1) / SB, C);
  hipLaunchKernelGGL(ssim_l1_bwd_kernel, grid, dim3(SB * SB), 0, stream, H, W, img1, img2, mask, make_window(), g_l1,
                     g_ssim, d_mu, d_xx, d_xy, dimg1);
  return 0;
}

}  // namespace gs
