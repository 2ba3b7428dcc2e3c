// Neural-Gaussian generation: the three anchor MLPs, the opacity selection and the post-processing of
// generate_neural_gaussians (gaussian_renderer/__init__.py:789-899) in its default configuration
// (feat_dim 32, inputs [feat, view direction], scene/gaussian_model.py:131-149), forward and backward.
//
// One wave owns 32 anchors.  Both layers run on the fp32 matrix cores (v_mfma_f32_32x32x2_f32) in the
// transposed form D[unit][anchor] = W[unit][:] . X[:][anchor]: the anchors sit on the 32 columns, so the
// hidden layer comes out of layer 1 with lane = anchor, register = hidden unit, which is exactly the B
// operand layer 2 wants.  Nothing of the hidden layer ever leaves the registers.  Operand layout of the
// instruction, with l the lane, half = l / 32:  A lane l -> A[l % 32][half], B lane l -> B[half][l % 32],
// result register i of lane l -> D[8 * (i / 4) + 4 * half + i % 4][l % 32].  The order in which the inner
// dimension is walked is free as long as both operands agree, so every inner index below is permuted to
// whatever the lanes already hold.
//
// The weights are rearranged once per call into those per-step operand orders ("packed" buffer); the kernels
// then read them with index step * 64 + lane.
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {
namespace {

constexpr int NG_WAVES = 4;          // waves per block
constexpr int NG_THREADS = 64 * NG_WAVES;
constexpr int NG_ANCHORS = 32;       // anchors per wave tile
constexpr int NG_W1_STEPS = 18;      // 36 input slots: 32 features, 3 view components, 1 constant for the bias
constexpr int NG_W1_SIZE = NG_W1_STEPS * 64;
constexpr int NG_TILE = 1024;        // one 32x32 operand tile
constexpr int SX_STRIDE = 37;
constexpr int SG_STRIDE = 33;

typedef float v16f __attribute__((ext_vector_type(16)));

__host__ __device__ constexpr int even_up(int v) { return (v + 1) & ~1; }
__host__ __device__ constexpr int hrow(int half, int i) { return 8 * (i >> 2) + 4 * half + (i & 3); }

// input slot a lane of the given half supplies at layer-1 step s: 16 consecutive features per half, then the
// view direction and the constant
__host__ __device__ constexpr int xslot(int half, int s) { return s < 16 ? 16 * half + s : 32 + 2 * (s - 16) + half; }

template <int K>
struct Shape {
  static_assert(K >= 1 && K <= 32, "n_offsets between 1 and 32");
  static constexpr int OUT0 = K, OUT1 = 3 * K, OUT2 = 7 * K;
  static constexpr int T0 = 1, T1 = (OUT1 + 31) / 32, T2 = (OUT2 + 31) / 32;
  static constexpr int TILES = T0 + T1 + T2;
  static constexpr int APG = 64 / K;                       // anchors per 64-lane slot group
  static constexpr int GROUPS = (NG_ANCHORS + APG - 1) / APG;
  // rows of the per-tile output-gradient matrix, each MLP's block padded to an even count
  static constexpr int G0 = 0, G1 = even_up(OUT0), G2 = G1 + even_up(OUT1), GROWS = G2 + even_up(OUT2);
  __host__ __device__ static constexpr int out(int m) { return m == 0 ? OUT0 : m == 1 ? OUT1 : OUT2; }
  __host__ __device__ static constexpr int tiles(int m) { return m == 0 ? T0 : m == 1 ? T1 : T2; }
  __host__ __device__ static constexpr int first_tile(int m) { return m == 0 ? 0 : m == 1 ? T0 : T0 + T1; }
  __host__ __device__ static constexpr int grow(int m) { return m == 0 ? G0 : m == 1 ? G1 : G2; }
};

// offsets (in floats) of the packed operand arrays
struct PackLayout {
  int w1, w2, b2, w2t, w1t, w1tv, total;
};
__host__ __device__ inline PackLayout pack_layout(int tiles) {
  PackLayout L;
  L.w1 = 0;                           // [3][18*64]  layer-1 A operand: W1[h][xslot], bias in slot 35
  L.w2 = 3 * NG_W1_SIZE;              // [tiles][16*64] layer-2 A operand: W2[row][hrow(half, s)]
  L.b2 = L.w2 + tiles * NG_TILE;      // [tiles][32]
  L.w2t = L.b2 + tiles * 32;          // [tiles][32 rows][32]  W2 rows, zero padded (A operand of dH = W2^T G)
  L.w1t = L.w2t + tiles * NG_TILE;    // [3][16*64]  W1[hrow(half, s)][i], i < 32   (A operand of dX)
  L.w1tv = L.w1t + 3 * NG_TILE;       // [3][16*64]  W1[hrow(half, s)][32 + i], i < 3, else 0
  L.total = L.w1tv + 3 * NG_TILE;
  return L;
}

struct MlpParams {
  const float* p[12];  // W1, b1, W2, b2 of the opacity, color and cov MLPs
};
struct MlpGrads {
  float* p[12];
};

template <int K>
__global__ void __launch_bounds__(256) neural_pack_kernel(MlpParams w, float* __restrict__ packed) {
  using S = Shape<K>;
  const PackLayout L = pack_layout(S::TILES);
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= L.total) return;
  float v = 0.0f;
  if (e < L.w2) {
    const int m = e / NG_W1_SIZE, r = e % NG_W1_SIZE, s = r >> 6, half = (r >> 5) & 1, h = r & 31;
    const int slot = xslot(half, s);
    v = slot < 35 ? w.p[4 * m][h * 35 + slot] : w.p[4 * m + 1][h];
  } else if (e < L.w1t) {
    // the three per-tile arrays
    const int which = e < L.b2 ? 0 : e < L.w2t ? 1 : 2;
    const int rel = e - (which == 0 ? L.w2 : which == 1 ? L.b2 : L.w2t);
    const int per = which == 1 ? 32 : NG_TILE;
    const int t = rel / per, r = rel % per;
    const int m = t < S::T0 ? 0 : t < S::T0 + S::T1 ? 1 : 2;
    const int lt = t - S::first_tile(m), out = S::out(m);
    const float* W2 = w.p[4 * m + 2];
    if (which == 0) {
      const int s = r >> 6, half = (r >> 5) & 1, row = 32 * lt + (r & 31);
      v = row < out ? W2[row * 32 + hrow(half, s)] : 0.0f;
    } else if (which == 1) {
      const int row = 32 * lt + r;
      v = row < out ? w.p[4 * m + 3][row] : 0.0f;
    } else {
      const int row = 32 * lt + (r >> 5), h = r & 31;
      v = row < out ? W2[row * 32 + h] : 0.0f;
    }
  } else {
    const bool view = e >= L.w1tv;
    const int rel = e - (view ? L.w1tv : L.w1t);
    const int m = rel / NG_TILE, r = rel % NG_TILE, s = r >> 6, half = (r >> 5) & 1, i = r & 31;
    const float* W1 = w.p[4 * m];
    if (!view) v = W1[hrow(half, s) * 35 + i];
    else v = i < 3 ? W1[hrow(half, s) * 35 + 32 + i] : 0.0f;
  }
  packed[e] = v;
}

__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }

// The 18 layer-1 B operands of this lane: its anchor's features of its half, the view direction and the constant.
// Also returns the unit view direction and the distance (every lane computes both).
__device__ __forceinline__ void load_x(float (&xb)[NG_W1_STEPS], float (&nv)[3], float& dist, bool valid, int64_t a,
                                       int half, const float* __restrict__ anchor, const float* __restrict__ feat,
                                       const float cam[3]) {
  if (valid) {
    const float4* f = (const float4*)(feat + a * 32 + 16 * half);
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const float4 v = f[q];
      xb[4 * q] = v.x; xb[4 * q + 1] = v.y; xb[4 * q + 2] = v.z; xb[4 * q + 3] = v.w;
    }
    const float vx = anchor[a * 3] - cam[0], vy = anchor[a * 3 + 1] - cam[1], vz = anchor[a * 3 + 2] - cam[2];
    dist = sqrtf((vx * vx + vy * vy) + vz * vz);
    nv[0] = vx / dist; nv[1] = vy / dist; nv[2] = vz / dist;
  } else {
#pragma unroll
    for (int q = 0; q < 16; q++) xb[q] = 0.0f;
    nv[0] = nv[1] = nv[2] = 0.0f;
    dist = 1.0f;
  }
  xb[16] = half ? nv[1] : nv[0];
  xb[17] = half ? 1.0f : nv[2];
}

// relu(W1 x + b1) for the wave's 32 anchors; w1 indexed step * 64 + lane
__device__ __forceinline__ v16f hidden_layer(const float* w1, const float (&xb)[NG_W1_STEPS], int lane) {
  v16f acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int s = 0; s < NG_W1_STEPS; s++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w1[s * 64 + lane], xb[s], acc, 0, 0, 0);
#pragma unroll
  for (int i = 0; i < 16; i++) acc[i] = acc[i] > 0.0f ? acc[i] : 0.0f;
  return acc;
}

// one 32-row tile of W2 h + b2; w2 indexed step * 64 + lane, b2 by row
__device__ __forceinline__ v16f output_tile(const float* w2, const float* b2, const v16f& h, int lane, int half) {
  v16f acc;
#pragma unroll
  for (int i = 0; i < 16; i++) acc[i] = b2[hrow(half, i)];
#pragma unroll
  for (int s = 0; s < 16; s++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w2[s * 64 + lane], h[s], acc, 0, 0, 0);
  return acc;
}

// number of set bits of `bits` in lanes [lo, hi)
__device__ __forceinline__ int count_lanes(unsigned long long bits, int lo, int hi) {
  const unsigned long long upto_hi = hi >= 64 ? ~0ull : ((1ull << hi) - 1ull);
  const unsigned long long upto_lo = (1ull << lo) - 1ull;
  return __popcll(bits & upto_hi & ~upto_lo);
}

// ---------------------------------------------------------------------------------------------------------
// Step 1: the opacity MLP.  neural_opacity = tanh(.), mask = neural_opacity > 0, and per anchor the number of
// selected offsets (input of the scan that places every anchor's Gaussians).
template <int K>
__global__ void __launch_bounds__(NG_THREADS)
neural_opacity_kernel(int64_t N, int ntiles, const float* __restrict__ anchor, const float* __restrict__ feat,
                      const float* __restrict__ campos, const float* __restrict__ packed,
                      float* __restrict__ neural_opacity, uint8_t* __restrict__ mask, uint8_t* __restrict__ counts) {
  using S = Shape<K>;
  const PackLayout L = pack_layout(S::TILES);
  __shared__ float sW1[NG_W1_SIZE];
  __shared__ float sW2[NG_TILE];
  __shared__ float sB2[32];
  __shared__ float sOp[NG_WAVES][NG_ANCHORS * K];
  for (int e = threadIdx.x; e < NG_W1_SIZE; e += NG_THREADS) sW1[e] = packed[L.w1 + e];
  for (int e = threadIdx.x; e < NG_TILE; e += NG_THREADS) sW2[e] = packed[L.w2 + e];
  if (threadIdx.x < 32) sB2[threadIdx.x] = packed[L.b2 + threadIdx.x];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, al = lane & 31;
  const float cam[3] = {campos[0], campos[1], campos[2]};
  float* op = sOp[wave];
  for (int tile = blockIdx.x * NG_WAVES + wave; tile < ntiles; tile += gridDim.x * NG_WAVES) {
    const int64_t a = (int64_t)tile * NG_ANCHORS + al;
    float xb[NG_W1_STEPS], nv[3], dist;
    load_x(xb, nv, dist, a < N, a, half, anchor, feat, cam);
    const v16f h = hidden_layer(sW1, xb, lane);
    const v16f o = output_tile(sW2, sB2, h, lane, half);
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int row = hrow(half, i);
      if (row < K) op[al * K + row] = tanhf(o[i]);
    }
    wave_sync();
#pragma unroll
    for (int g = 0; g < S::GROUPS; g++) {
      const int idx = g * S::APG * K + lane;  // slot within the tile
      const int64_t slot_anchor = (int64_t)tile * NG_ANCHORS + idx / K;
      const bool ok = lane < S::APG * K && idx < NG_ANCHORS * K && slot_anchor < N;
      const float t = ok ? op[idx] : 0.0f;
      const bool sel = t > 0.0f;
      const unsigned long long bits = __ballot(sel);
      if (ok) {
        const int64_t slot = (int64_t)tile * NG_ANCHORS * K + idx;
        neural_opacity[slot] = t;
        mask[slot] = sel ? 1 : 0;
        if (idx % K == 0) counts[slot_anchor] = (uint8_t)count_lanes(bits, lane, lane + K);
      }
    }
    wave_sync();
  }
}

// ---------------------------------------------------------------------------------------------------------
// Step 2: the color and cov MLPs and the post-processing, written straight to each selected Gaussian's row
// (first[a] = number of selected offsets of all anchors before a).
template <int K>
__global__ void __launch_bounds__(NG_THREADS)
neural_gaussians_kernel(int64_t N, int ntiles, const float* __restrict__ anchor, const float* __restrict__ feat,
                        const float* __restrict__ offsets, const float* __restrict__ scaling,
                        const float* __restrict__ campos, const float* __restrict__ packed,
                        const float* __restrict__ neural_opacity, const uint32_t* __restrict__ first,
                        float* __restrict__ xyz, float* __restrict__ color, float* __restrict__ opacity,
                        float* __restrict__ scal, float* __restrict__ rot, float* __restrict__ aux) {
  using S = Shape<K>;
  const PackLayout L = pack_layout(S::TILES);
  constexpr int NT = S::T1 + S::T2;              // tiles of the two MLPs of this kernel
  constexpr int ROWS = 32 * S::T1 + S::OUT2;     // rows kept: color tiles whole, cov rows up to 7K
  __shared__ float sW1[2][NG_W1_SIZE];
  __shared__ float sW2[NT][NG_TILE];
  __shared__ float sB2[NT * 32];
  __shared__ float sOut[NG_WAVES][ROWS * SG_STRIDE];
  for (int e = threadIdx.x; e < 2 * NG_W1_SIZE; e += NG_THREADS) (&sW1[0][0])[e] = packed[L.w1 + NG_W1_SIZE + e];
  for (int e = threadIdx.x; e < NT * NG_TILE; e += NG_THREADS) (&sW2[0][0])[e] = packed[L.w2 + S::T0 * NG_TILE + e];
  for (int e = threadIdx.x; e < NT * 32; e += NG_THREADS) sB2[e] = packed[L.b2 + S::T0 * 32 + e];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, al = lane & 31;
  const float cam[3] = {campos[0], campos[1], campos[2]};
  float* out = sOut[wave];
  for (int tile = blockIdx.x * NG_WAVES + wave; tile < ntiles; tile += gridDim.x * NG_WAVES) {
    const int64_t a = (int64_t)tile * NG_ANCHORS + al;
    float xb[NG_W1_STEPS], nv[3], dist;
    load_x(xb, nv, dist, a < N, a, half, anchor, feat, cam);
    {
      const v16f h = hidden_layer(sW1[0], xb, lane);
#pragma unroll
      for (int t = 0; t < S::T1; t++) {
        const v16f o = output_tile(sW2[t], sB2 + 32 * t, h, lane, half);
#pragma unroll
        for (int i = 0; i < 16; i++) out[(32 * t + hrow(half, i)) * SG_STRIDE + al] = o[i];
      }
    }
    {
      const v16f h = hidden_layer(sW1[1], xb, lane);
#pragma unroll
      for (int t = 0; t < S::T2; t++) {
        const v16f o = output_tile(sW2[S::T1 + t], sB2 + 32 * (S::T1 + t), h, lane, half);
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int row = 32 * t + hrow(half, i);
          if (row < S::OUT2) out[(32 * S::T1 + row) * SG_STRIDE + al] = o[i];
        }
      }
    }
    wave_sync();
#pragma unroll 1
    for (int g = 0; g < S::GROUPS; g++) {
      const int idx = g * S::APG * K + lane;
      const int ax = idx / K, j = idx % K;
      const int64_t sa = (int64_t)tile * NG_ANCHORS + ax;
      const bool ok = lane < S::APG * K && ax < NG_ANCHORS && sa < N;
      const int64_t slot = sa * K + j;
      const float t = ok ? neural_opacity[slot] : 0.0f;
      const bool sel = t > 0.0f;
      const unsigned long long bits = __ballot(sel);
      if (sel) {
        const int64_t r = (int64_t)first[sa] + count_lanes(bits, lane - j, lane);
        const float* sc = scaling + sa * 6;
        const float* cv = out + (32 * S::T1 + 7 * j) * SG_STRIDE + ax;
        float sg[3];
#pragma unroll
        for (int c = 0; c < 3; c++) {
          xyz[r * 3 + c] = anchor[sa * 3 + c] + offsets[slot * 3 + c] * sc[c];
          color[r * 3 + c] = sigmoidf(out[(3 * j + c) * SG_STRIDE + ax]);
          sg[c] = sigmoidf(cv[c * SG_STRIDE]);
          scal[r * 3 + c] = sc[3 + c] * sg[c];
        }
        opacity[r] = t;
        const float q0 = cv[3 * SG_STRIDE], q1 = cv[4 * SG_STRIDE], q2 = cv[5 * SG_STRIDE], q3 = cv[6 * SG_STRIDE];
        const float len = sqrtf(((q0 * q0 + q1 * q1) + q2 * q2) + q3 * q3);
        const float den = fmaxf(len, 1e-12f);
        *(float4*)(rot + r * 4) = make_float4(q0 / den, q1 / den, q2 / den, q3 / den);
        *(float4*)(aux + r * 4) = make_float4(sg[0], sg[1], sg[2], len);
      }
    }
    wave_sync();
  }
}

// ---------------------------------------------------------------------------------------------------------
// Backward.  Per wave tile: the gradients of the selected Gaussians become the pre-activation gradients G of
// the three output layers (a GROWS x 32 matrix in LDS, zero for unselected offsets); then per MLP
//   H = relu(W1 x + b1) (recomputed), dH = W2^T G, dHpre = dH where H > 0, dX += W1^T dHpre,
//   dW2 += G H^T, [dW1 | db1] += dHpre [x | 1]^T, db2 += row sums of G,
// with the weight gradients kept in matrix-core accumulators over all tiles of the wave and reduced over the
// block at the end (one partial set per block; a second kernel adds the blocks in a fixed order).
template <int K>
struct BwdLds {
  using S = Shape<K>;
  float g[S::GROWS * SG_STRIDE];
  float hd[2 * 32 * SG_STRIDE];  // H, then dHpre; also the staging area of the final block reduction
  float x[NG_ANCHORS * SX_STRIDE];
  float c[64 * 9];
  float da[NG_ANCHORS * 3];
};

// floats of one block's partial weight gradients: W2 tiles, then W1 (3 MLPs x 2 column tiles), then b2 rows
template <int K>
__host__ __device__ constexpr int partial_floats() {
  return (Shape<K>::TILES + 6) * NG_TILE + ((Shape<K>::GROWS + 63) / 64) * 64;
}

template <int K>
__global__ void __launch_bounds__(NG_THREADS)
neural_backward_kernel(int64_t N, int ntiles, const float* __restrict__ anchor, const float* __restrict__ feat,
                       const float* __restrict__ offsets, const float* __restrict__ scaling,
                       const float* __restrict__ campos, const float* __restrict__ packed,
                       const float* __restrict__ neural_opacity, const uint32_t* __restrict__ first,
                       const float* __restrict__ color_out, const float* __restrict__ rot_out,
                       const float* __restrict__ aux, const float* __restrict__ g_xyz,
                       const float* __restrict__ g_color, const float* __restrict__ g_opacity,
                       const float* __restrict__ g_scal, const float* __restrict__ g_rot,
                       float* __restrict__ d_anchor, float* __restrict__ d_feat, float* __restrict__ d_offsets,
                       float* __restrict__ d_scaling, float* __restrict__ partials) {
  using S = Shape<K>;
  const PackLayout L = pack_layout(S::TILES);
  constexpr int B2N = (S::GROWS + 63) / 64;
  __shared__ BwdLds<K> lds[NG_WAVES];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, al = lane & 31;
  const float cam[3] = {campos[0], campos[1], campos[2]};
  BwdLds<K>& W = lds[wave];
  // rows that pad a block of G to an even count are read by the dH products and never written below
  for (int e = lane; e < S::GROWS * SG_STRIDE; e += 64) W.g[e] = 0.0f;
  wave_sync();

  v16f accW2[S::TILES], accW1[3][2];
  float accB2[B2N];
#pragma unroll
  for (int t = 0; t < S::TILES; t++)
#pragma unroll
    for (int i = 0; i < 16; i++) accW2[t][i] = 0.0f;
#pragma unroll
  for (int m = 0; m < 3; m++)
#pragma unroll
    for (int i = 0; i < 16; i++) accW1[m][0][i] = accW1[m][1][i] = 0.0f;
#pragma unroll
  for (int q = 0; q < B2N; q++) accB2[q] = 0.0f;

  for (int tile = blockIdx.x * NG_WAVES + wave; tile < ntiles; tile += gridDim.x * NG_WAVES) {
    const int64_t a = (int64_t)tile * NG_ANCHORS + al;
    const bool valid = a < N;
    float xb[NG_W1_STEPS], nv[3], dist;
    load_x(xb, nv, dist, valid, a, half, anchor, feat, cam);
#pragma unroll
    for (int s = 0; s < NG_W1_STEPS; s++) W.x[al * SX_STRIDE + xslot(half, s)] = xb[s];

    // ---- per offset: output gradients -> G, direct gradients of offsets, scaling and anchor
#pragma unroll 1
    for (int g = 0; g < S::GROUPS; g++) {
      const int idx = g * S::APG * K + lane;
      const int ax = idx / K, j = idx % K;
      const int64_t sa = (int64_t)tile * NG_ANCHORS + ax;
      const bool in_group = lane < S::APG * K && ax < NG_ANCHORS;
      const bool ok = in_group && sa < N;
      const int64_t slot = sa * K + j;
      const float t = ok ? neural_opacity[slot] : 0.0f;
      const bool sel = t > 0.0f;
      const unsigned long long bits = __ballot(sel);
      float go = 0.0f, gc[3] = {0.0f, 0.0f, 0.0f}, gv[7] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
      float con[9] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f}, dof[3] = {0.0f, 0.0f, 0.0f};
      if (sel) {
        const int64_t r = (int64_t)first[sa] + count_lanes(bits, lane - j, lane);
        const float* sc = scaling + sa * 6;
        go = g_opacity[r] * (1.0f - t * t);
        const float4 ax4 = *(const float4*)(aux + r * 4);
        const float sg[3] = {ax4.x, ax4.y, ax4.z};
#pragma unroll
        for (int c = 0; c < 3; c++) {
          const float cs = color_out[r * 3 + c];
          gc[c] = g_color[r * 3 + c] * (cs * (1.0f - cs));
          const float gx = g_xyz[r * 3 + c], gs = g_scal[r * 3 + c];
          con[c] = gx;
          dof[c] = gx * sc[c];
          con[3 + c] = gx * offsets[slot * 3 + c];
          con[6 + c] = gs * sg[c];
          gv[c] = gs * sc[3 + c] * (sg[c] * (1.0f - sg[c]));
        }
        const float len = ax4.w;
        const float4 gr = *(const float4*)(g_rot + r * 4);
        if (len > 1e-12f) {
          const float4 qh = *(const float4*)(rot_out + r * 4);
          const float dot = ((qh.x * gr.x + qh.y * gr.y) + qh.z * gr.z) + qh.w * gr.w;
          gv[3] = (gr.x - qh.x * dot) / len; gv[4] = (gr.y - qh.y * dot) / len;
          gv[5] = (gr.z - qh.z * dot) / len; gv[6] = (gr.w - qh.w * dot) / len;
        } else {
          gv[3] = gr.x / 1e-12f; gv[4] = gr.y / 1e-12f; gv[5] = gr.z / 1e-12f; gv[6] = gr.w / 1e-12f;
        }
      }
      if (in_group) {
        W.g[(S::G0 + j) * SG_STRIDE + ax] = go;
#pragma unroll
        for (int c = 0; c < 3; c++) W.g[(S::G1 + 3 * j + c) * SG_STRIDE + ax] = gc[c];
#pragma unroll
        for (int c = 0; c < 7; c++) W.g[(S::G2 + 7 * j + c) * SG_STRIDE + ax] = gv[c];
#pragma unroll
        for (int c = 0; c < 9; c++) W.c[lane * 9 + c] = con[c];
      }
      if (ok) {
#pragma unroll
        for (int c = 0; c < 3; c++) d_offsets[slot * 3 + c] = dof[c];
      }
      wave_sync();
      // sums over the offsets of an anchor, in offset order
      for (int item = lane; item < S::APG * 9; item += 64) {
        const int ga = item / 9, comp = item % 9;
        const int ax2 = g * S::APG + ga;
        const int64_t sa2 = (int64_t)tile * NG_ANCHORS + ax2;
        if (ax2 < NG_ANCHORS && sa2 < N) {
          float sum = 0.0f;
#pragma unroll
          for (int jj = 0; jj < K; jj++) sum += W.c[(ga * K + jj) * 9 + comp];
          if (comp < 3) W.da[ax2 * 3 + comp] = sum;
          else d_scaling[sa2 * 6 + (comp - 3)] = sum;
        }
      }
      wave_sync();
    }

    // ---- through the MLPs
    v16f dxf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, dxv = dxf;
#pragma unroll
    for (int m = 0; m < 3; m++) {
      const v16f h = hidden_layer(packed + L.w1 + m * NG_W1_SIZE, xb, lane);
      v16f dh = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int lt = 0; lt < S::tiles(m); lt++) {
        const int rows = S::out(m) - 32 * lt < 32 ? S::out(m) - 32 * lt : 32;
        const float* w2t = packed + L.w2t + (S::first_tile(m) + lt) * NG_TILE;
        const float* gt = W.g + (S::grow(m) + 32 * lt) * SG_STRIDE;
#pragma unroll
        for (int s = 0; s < (rows + 1) / 2; s++)
          dh = __builtin_amdgcn_mfma_f32_32x32x2f32(w2t[s * 64 + lane], gt[(2 * s + half) * SG_STRIDE + al], dh, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 16; i++) dh[i] = h[i] > 0.0f ? dh[i] : 0.0f;
      const float* w1t = packed + L.w1t + m * NG_TILE;
      const float* w1tv = packed + L.w1tv + m * NG_TILE;
#pragma unroll
      for (int s = 0; s < 16; s++) {
        dxf = __builtin_amdgcn_mfma_f32_32x32x2f32(w1t[s * 64 + lane], dh[s], dxf, 0, 0, 0);
        dxv = __builtin_amdgcn_mfma_f32_32x32x2f32(w1tv[s * 64 + lane], dh[s], dxv, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 16; i++) {
        W.hd[hrow(half, i) * SG_STRIDE + al] = h[i];
        W.hd[(32 + hrow(half, i)) * SG_STRIDE + al] = dh[i];
      }
      wave_sync();
      // weight gradients: the inner dimension is the 32 anchors of the tile
#pragma unroll
      for (int lt = 0; lt < S::tiles(m); lt++) {
        const int last = S::out(m) - 32 * lt - 1;  // rows past the last one repeat it; their results are dropped
        const float* gt = W.g + (S::grow(m) + 32 * lt + (al < last ? al : last)) * SG_STRIDE;
#pragma unroll
        for (int s = 0; s < 16; s++)
          accW2[S::first_tile(m) + lt] = __builtin_amdgcn_mfma_f32_32x32x2f32(
              gt[2 * s + half], W.hd[al * SG_STRIDE + 2 * s + half], accW2[S::first_tile(m) + lt], 0, 0, 0);
      }
#pragma unroll
      for (int s = 0; s < 16; s++) {
        const float dhv = W.hd[(32 + al) * SG_STRIDE + 2 * s + half];
        accW1[m][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(dhv, W.x[(2 * s + half) * SX_STRIDE + al], accW1[m][0], 0, 0, 0);
        accW1[m][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(dhv, W.x[(2 * s + half) * SX_STRIDE + 32 + (al & 3)],
                                                          accW1[m][1], 0, 0, 0);
      }
      wave_sync();
    }
#pragma unroll
    for (int q = 0; q < B2N; q++) {
      const int row = q * 64 + lane;
      if (row < S::GROWS) {
        float sum = 0.0f;
#pragma unroll
        for (int c = 0; c < NG_ANCHORS; c++) sum += W.g[row * SG_STRIDE + c];
        accB2[q] += sum;
      }
    }

    // ---- per anchor results
    if (valid) {
#pragma unroll
      for (int q = 0; q < 4; q++)
        *(float4*)(d_feat + a * 32 + 8 * q + 4 * half) = make_float4(dxf[4 * q], dxf[4 * q + 1], dxf[4 * q + 2], dxf[4 * q + 3]);
      if (half == 0) {
        const float ng = (nv[0] * dxv[0] + nv[1] * dxv[1]) + nv[2] * dxv[2];
#pragma unroll
        for (int c = 0; c < 3; c++) d_anchor[a * 3 + c] = W.da[al * 3 + c] + (dxv[c] - nv[c] * ng) / dist;
      }
    }
    wave_sync();
  }

  // ---- reduce the four waves' accumulators, one 32x32 tile at a time, through each wave's staging area
  float* out = partials + (size_t)blockIdx.x * partial_floats<K>();
  constexpr int NACC = S::TILES + 6;
#pragma unroll
  for (int t = 0; t < NACC; t++) {
    const v16f& acc = t < S::TILES ? accW2[t] : accW1[(t - S::TILES) >> 1][(t - S::TILES) & 1];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; i++) W.hd[hrow(half, i) * 32 + al] = acc[i];
    __syncthreads();
    for (int e = threadIdx.x; e < NG_TILE; e += NG_THREADS)
      out[t * NG_TILE + e] = ((lds[0].hd[e] + lds[1].hd[e]) + lds[2].hd[e]) + lds[3].hd[e];
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < B2N; q++) W.hd[q * 64 + lane] = accB2[q];
  __syncthreads();
  for (int e = threadIdx.x; e < B2N * 64; e += NG_THREADS)
    out[NACC * NG_TILE + e] = ((lds[0].hd[e] + lds[1].hd[e]) + lds[2].hd[e]) + lds[3].hd[e];
}

// Adds the blocks' partial sets in block order and writes the twelve weight gradients.
template <int K>
__global__ void __launch_bounds__(256)
neural_weight_reduce_kernel(int nblocks, const float* __restrict__ partials, MlpGrads d) {
  using S = Shape<K>;
  constexpr int PER_MLP_1 = 32 * 35 + 32;
  constexpr int TOTAL = 3 * PER_MLP_1 + 33 * (S::OUT0 + S::OUT1 + S::OUT2);
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= TOTAL) return;
  int src;      // index inside a partial set
  float* dst;
  if (e < 3 * PER_MLP_1) {
    const int m = e / PER_MLP_1, r = e % PER_MLP_1;
    if (r < 32 * 35) {
      const int h = r / 35, i = r % 35;
      src = (S::TILES + 2 * m + (i >= 32)) * NG_TILE + h * 32 + (i & 31);
      dst = d.p[4 * m] + r;
    } else {
      const int h = r - 32 * 35;
      src = (S::TILES + 2 * m + 1) * NG_TILE + h * 32 + 3;
      dst = d.p[4 * m + 1] + h;
    }
  } else {
    int r = e - 3 * PER_MLP_1;
    int m = 0;
    while (r >= 33 * S::out(m)) { r -= 33 * S::out(m); m++; }
    const int out = S::out(m);
    if (r < 32 * out) {
      const int row = r / 32, h = r % 32;
      src = (S::first_tile(m) + row / 32) * NG_TILE + (row % 32) * 32 + h;
      dst = d.p[4 * m + 2] + r;
    } else {
      const int row = r - 32 * out;
      src = (S::TILES + 6) * NG_TILE + S::grow(m) + row;
      dst = d.p[4 * m + 3] + row;
    }
  }
  float sum = 0.0f;
  for (int b = 0; b < nblocks; b++) sum += partials[(size_t)b * partial_floats<K>() + src];
  *dst = sum;
}

int blocks_for(int ntiles, int per_cu) {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  const int want = (ntiles + NG_WAVES - 1) / NG_WAVES;
  const int cap = cus * per_cu;
  return want < cap ? want : cap;
}

template <int K>
struct Launcher {
  using S = Shape<K>;
  static void pack(const float* const* params, float* packed, hipStream_t stream) {
    MlpParams w;
    for (int i = 0; i < 12; i++) w.p[i] = params[i];
    const int total = pack_layout(S::TILES).total;
    hipLaunchKernelGGL(neural_pack_kernel<K>, dim3((total + 255) / 256), dim3(256), 0, stream, w, packed);
  }
  static void opacity(int64_t N, const float* anchor, const float* feat, const float* campos, const float* packed,
                      float* neural_opacity, uint8_t* mask, uint8_t* counts, hipStream_t stream) {
    const int ntiles = (int)((N + NG_ANCHORS - 1) / NG_ANCHORS);
    hipLaunchKernelGGL(neural_opacity_kernel<K>, dim3(blocks_for(ntiles, 4)), dim3(NG_THREADS), 0, stream, N, ntiles,
                       anchor, feat, campos, packed, neural_opacity, mask, counts);
  }
  static void gaussians(int64_t N, const float* anchor, const float* feat, const float* offsets, const float* scaling,
                        const float* campos, const float* packed, const float* neural_opacity, const uint32_t* first,
                        float* xyz, float* color, float* opacity, float* scal, float* rot, float* aux,
                        hipStream_t stream) {
    const int ntiles = (int)((N + NG_ANCHORS - 1) / NG_ANCHORS);
    hipLaunchKernelGGL(neural_gaussians_kernel<K>, dim3(blocks_for(ntiles, 2)), dim3(NG_THREADS), 0, stream, N, ntiles,
                       anchor, feat, offsets, scaling, campos, packed, neural_opacity, first, xyz, color, opacity,
                       scal, rot, aux);
  }
  static int backward_blocks(int64_t N) { return blocks_for((int)((N + NG_ANCHORS - 1) / NG_ANCHORS), 1); }
  static void backward(int64_t N, const float* anchor, const float* feat, const float* offsets, const float* scaling,
                       const float* campos, const float* packed, const float* neural_opacity, const uint32_t* first,
                       const float* color_out, const float* rot_out, const float* aux, const float* g_xyz,
                       const float* g_color, const float* g_opacity, const float* g_scal, const float* g_rot,
                       float* d_anchor, float* d_feat, float* d_offsets, float* d_scaling, float* const* d_params,
                       float* partials, hipStream_t stream) {
    const int ntiles = (int)((N + NG_ANCHORS - 1) / NG_ANCHORS);
    const int nblocks = backward_blocks(N);
    hipLaunchKernelGGL(neural_backward_kernel<K>, dim3(nblocks), dim3(NG_THREADS), 0, stream, N, ntiles, anchor, feat,
                       offsets, scaling, campos, packed, neural_opacity, first, color_out, rot_out, aux, g_xyz,
                       g_color, g_opacity, g_scal, g_rot, d_anchor, d_feat, d_offsets, d_scaling, partials);
    MlpGrads d;
    for (int i = 0; i < 12; i++) d.p[i] = d_params[i];
    const int total = 3 * (32 * 35 + 32) + 33 * (S::OUT0 + S::OUT1 + S::OUT2);
    hipLaunchKernelGGL(neural_weight_reduce_kernel<K>, dim3((total + 255) / 256), dim3(256), 0, stream, nblocks,
                       partials, d);
  }
};

}  // namespace

// n_offsets values the kernels are instantiated for
#define NG_FOR_EACH_K(X) X(1) X(2) X(3) X(4) X(5) X(6) X(8) X(10) X(12) X(16)

bool neural_supported(int k) {
  switch (k) {
#define X(KK) case KK:
    NG_FOR_EACH_K(X)
#undef X
    return true;
    default: return false;
  }
}

size_t neural_packed_floats(int k) {
  switch (k) {
#define X(KK) case KK: return (size_t)pack_layout(Shape<KK>::TILES).total;
    NG_FOR_EACH_K(X)
#undef X
    default: return 0;
  }
}

size_t neural_partial_floats(int k, int64_t N) {
  switch (k) {
#define X(KK) case KK: return (size_t)partial_floats<KK>() * (size_t)Launcher<KK>::backward_blocks(N);
    NG_FOR_EACH_K(X)
#undef X
    default: return 0;
  }
}

int launch_neural_pack(int k, const float* const* params, float* packed, hipStream_t stream) {
  switch (k) {
#define X(KK) case KK: Launcher<KK>::pack(params, packed, stream); return 0;
    NG_FOR_EACH_K(X)
#undef X
    default: return 1;
  }
}

int launch_neural_opacity(int64_t N, int k, const float* anchor, const float* feat, const float* campos,
                          const float* packed, float* neural_opacity, uint8_t* mask, uint8_t* counts,
                          hipStream_t stream) {
  if (N <= 0) return 0;
  switch (k) {
#define X(KK) case KK: Launcher<KK>::opacity(N, anchor, feat, campos, packed, neural_opacity, mask, counts, stream); return 0;
    NG_FOR_EACH_K(X)
#undef X
    default: return 1;
  }
}

int launch_neural_gaussians(int64_t N, int k, const float* anchor, const float* feat, const float* offsets,
                            const float* scaling, const float* campos, const float* packed,
                            const float* neural_opacity, const uint32_t* first, float* xyz, float* color,
                            float* opacity, float* scal, float* rot, float* aux, hipStream_t stream) {
  if (N <= 0) return 0;
  switch (k) {
#define X(KK) case KK: Launcher<KK>::gaussians(N, anchor, feat, offsets, scaling, campos, packed, neural_opacity, first, xyz, color, opacity, scal, rot, aux, stream); return 0;
    NG_FOR_EACH_K(X)
#undef X
    default: return 1;
  }
}

int launch_neural_backward(int64_t N, int k, const float* anchor, const float* feat, const float* offsets,
                           const float* scaling, const float* campos, const float* packed,
                           const float* neural_opacity, const uint32_t* first, const float* color_out,
                           const float* rot_out, const float* aux, const float* g_xyz, const float* g_color,
                           const float* g_opacity, const float* g_scal, const float* g_rot, float* d_anchor,
                           float* d_feat, float* d_offsets, float* d_scaling, float* const* d_params, float* partials,
                           hipStream_t stream) {
  if (N <= 0) return 0;
  switch (k) {
#define X(KK) case KK: Launcher<KK>::backward(N, anchor, feat, offsets, scaling, campos, packed, neural_opacity, first, color_out, rot_out, aux, g_xyz, g_color, g_opacity, g_scal, g_rot, d_anchor, d_feat, d_offsets, d_scaling, d_params, partials, stream); return 0;
    NG_FOR_EACH_K(X)
#undef X
    default: return 1;
  }
}

}  // namespace gs
