// Neural-Gaussian generation: the three anchor MLPs, the opacity selection and the post-processing of
// generate_neural_gaussians (gaussian_renderer/__init__.py:789-899) for feat_dim 32 (inputs [feat, view
// direction] and, where the model asks for them, the distance and the anchor's level,
// scene/gaussian_model.py:118-149), forward and backward.
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

constexpr int NG_WAVES = 4;          // waves per block of the forward kernels
constexpr int NG_THREADS = 64 * NG_WAVES;
constexpr int NG_ANCHORS = 32;       // anchors per wave tile
constexpr int NG_W1_STEPS = 19;      // 38 input slots: 32 features, 3 view components, 1 constant for the bias,
                                     // the distance and the level (zero weights where an MLP does not take them)
constexpr int NG_SLOTS = 2 * NG_W1_STEPS;
constexpr int NG_TILE = 1024;        // one 32x32 accumulator tile
constexpr int WS = 33;               // row stride of the weight arrays in LDS (conflict-free both ways)
constexpr int SX_STRIDE = 39;
constexpr int SG_STRIDE = 33;
constexpr int NG_SLOT_GRADS = 11;    // pre-activation gradients per offset: 1 opacity, 3 color, 7 cov

typedef float v16f __attribute__((ext_vector_type(16)));

__host__ __device__ constexpr int even_up(int v) { return (v + 1) & ~1; }
__host__ __device__ constexpr int hrow(int half, int i) { return 8 * (i >> 2) + 4 * half + (i & 3); }

// input slot a lane of the given half supplies at layer-1 step s: 16 consecutive features per half, then the
// view direction and the constant, then the distance (half 0) and the level (half 1)
__host__ __device__ constexpr int xslot(int half, int s) { return s < 16 ? 16 * half + s : 32 + 2 * (s - 16) + half; }

template <int K>
struct Shape {
  static_assert(K >= 1 && K <= 32, "n_offsets between 1 and 32");
  static constexpr int OUT0 = K, OUT1 = 3 * K, OUT2 = 7 * K;
  static constexpr int T0 = 1, T1 = (OUT1 + 31) / 32, T2 = (OUT2 + 31) / 32;
  static constexpr int TILES = T0 + T1 + T2;
  static constexpr int APG = 64 / K;                       // anchors per 64-lane slot group
  static constexpr int GROUPS = (NG_ANCHORS + APG - 1) / APG;
  // row numbering shared by the output-layer weights and the output-gradient matrix: the three MLPs' output
  // units one after the other, each block padded to an even count
  static constexpr int G0 = 0, G1 = even_up(OUT0), G2 = G1 + even_up(OUT1), GROWS = G2 + even_up(OUT2);
  static constexpr int BWD_WAVES = GROWS <= 110 ? 4 : 2;   // waves per block of the backward kernel (LDS)
  __host__ __device__ static constexpr int out(int m) { return m == 0 ? OUT0 : m == 1 ? OUT1 : OUT2; }
  __host__ __device__ static constexpr int tiles(int m) { return m == 0 ? T0 : m == 1 ? T1 : T2; }
  __host__ __device__ static constexpr int first_tile(int m) { return m == 0 ? 0 : m == 1 ? T0 : T0 + T1; }
  __host__ __device__ static constexpr int grow(int m) { return m == 0 ? G0 : m == 1 ? G1 : G2; }
};

// The weights as the kernels keep them in LDS (offsets in floats): W1 transposed with the bias as input slot 35,
// [m][slot][WS]; W2 by output row, [row][WS], pad rows zero; b2 by output row.  With the odd row stride both
// the row-wise and the column-wise operand reads of the forward and backward products are conflict-free.
struct PackLayout {
  int w1t, w2, b2, total;
};
__host__ __device__ constexpr PackLayout pack_layout(int grows) {
  return PackLayout{0, 3 * NG_SLOTS * WS, 3 * NG_SLOTS * WS + grows * WS, 3 * NG_SLOTS * WS + grows * WS + grows};
}

// W1 of MLP m has in[m] columns: 32 features, 3 view components, then the distance (column dist_col[m], or -1)
// and the level (column level_col[m], or -1)
struct MlpInputs {
  int in[3], dist_col[3], level_col[3];
};
// input_flags: bit m = MLP m (opacity, color, cov) takes the distance, bit 3 = all take the level
MlpInputs mlp_inputs(int input_flags) {
  MlpInputs q;
  for (int m = 0; m < 3; m++) {
    const bool d = (input_flags >> m) & 1, l = (input_flags >> 3) & 1;
    q.dist_col[m] = d ? 35 : -1;
    q.level_col[m] = l ? 35 + (d ? 1 : 0) : -1;
    q.in[m] = 35 + (d ? 1 : 0) + (l ? 1 : 0);
  }
  return q;
}
struct MlpParams {
  const float* p[12];  // W1, b1, W2, b2 of the opacity, color and cov MLPs
  MlpInputs q;
};
struct MlpGrads {
  float* p[12];
  MlpInputs q;
};

template <int K>
__global__ void __launch_bounds__(256) neural_pack_kernel(MlpParams w, float* __restrict__ packed) {
  using S = Shape<K>;
  constexpr PackLayout L = pack_layout(S::GROWS);
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= L.total) return;
  float v = 0.0f;
  if (e < L.w2) {
    const int m = e / (NG_SLOTS * WS), r = e % (NG_SLOTS * WS), slot = r / WS, h = r % WS;
    if (h < 32) {
      const int col = slot < 35 ? slot : slot == 36 ? w.q.dist_col[m] : slot == 37 ? w.q.level_col[m] : -1;
      v = slot == 35 ? w.p[4 * m + 1][h] : col >= 0 ? w.p[4 * m][h * w.q.in[m] + col] : 0.0f;
    }
  } else {
    const bool bias = e >= L.b2;
    const int rel = e - (bias ? L.b2 : L.w2);
    const int row = bias ? rel : rel / WS, h = bias ? 0 : rel % WS;
    const int m = row < S::G1 ? 0 : row < S::G2 ? 1 : 2;
    const int o = row - S::grow(m);
    if (o < S::out(m) && h < 32) v = bias ? w.p[4 * m + 3][o] : w.p[4 * m + 2][o * 32 + h];
  }
  packed[e] = v;
}

__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// hardware exp2 and reciprocal: about 1e-6 relative, far inside what float32 MLP outputs carry
__device__ __forceinline__ float sigmoidf(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

// The 19 layer-1 B operands of this lane: its anchor's features of its half, the view direction, the constant,
// the distance and the level.
// Also returns the unit view direction and the distance (every lane computes both).
struct XOperand {
  float4 f[4];
  float ax, ay, az, level;
};
__device__ __forceinline__ XOperand fetch_x(bool valid, int64_t a, int half, const float* __restrict__ anchor,
                                            const float* __restrict__ feat, const float* __restrict__ level) {
  XOperand x;
  if (valid) {
    const float4* f = (const float4*)(feat + a * 32 + 16 * half);
#pragma unroll
    for (int q = 0; q < 4; q++) x.f[q] = f[q];
    x.ax = anchor[a * 3]; x.ay = anchor[a * 3 + 1]; x.az = anchor[a * 3 + 2];
    x.level = level != nullptr ? level[a] : 0.0f;
  } else {
#pragma unroll
    for (int q = 0; q < 4; q++) x.f[q] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    x.ax = x.ay = x.az = x.level = 0.0f;
  }
  return x;
}
__device__ __forceinline__ void unpack_x(float (&xb)[NG_W1_STEPS], float (&nv)[3], float& dist, const XOperand& x,
                                         bool valid, int half, const float cam[3]) {
#pragma unroll
  for (int q = 0; q < 4; q++) {
    xb[4 * q] = x.f[q].x; xb[4 * q + 1] = x.f[q].y; xb[4 * q + 2] = x.f[q].z; xb[4 * q + 3] = x.f[q].w;
  }
  if (valid) {
    const float vx = x.ax - cam[0], vy = x.ay - cam[1], vz = x.az - cam[2];
    dist = sqrtf((vx * vx + vy * vy) + vz * vz);
    nv[0] = vx / dist; nv[1] = vy / dist; nv[2] = vz / dist;
  } else {
    nv[0] = nv[1] = nv[2] = 0.0f;
    dist = 1.0f;
  }
  xb[16] = half ? nv[1] : nv[0];
  xb[17] = half ? 1.0f : nv[2];
  xb[18] = half ? x.level : dist;
}

// relu(W1 x + b1) for the wave's 32 anchors; w1t = this MLP's [slot][WS] array
__device__ __forceinline__ v16f hidden_layer(const float* w1t, const float (&xb)[NG_W1_STEPS], int al, int half) {
  v16f acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const float* lo = w1t + half * 16 * WS + al;  // slots 16 half + s
  const float* hi = w1t + (32 + half) * WS + al;  // slots 32 + half, 34 + half
#pragma unroll
  for (int s = 0; s < 16; s++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(lo[s * WS], xb[s], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(hi[0], xb[16], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(hi[2 * WS], xb[17], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(hi[4 * WS], xb[18], acc, 0, 0, 0);
#pragma unroll
  for (int i = 0; i < 16; i++) acc[i] = acc[i] > 0.0f ? acc[i] : 0.0f;
  return acc;
}

// rows [32 lt, 32 lt + 32) of W2 h + b2 of an MLP with `out` output units; w2, b2 = the MLP's first row
template <int OUT>
__device__ __forceinline__ v16f output_tile(const float* w2, const float* b2, int lt, const v16f& h, int al, int half) {
  const int row = 32 * lt + al;
  const bool full = 32 * lt + 32 <= OUT;  // uniform
  const bool live = full || row < OUT;
  const float* wr = w2 + (live ? row : OUT - 1) * WS + 4 * half;
  v16f acc;
#pragma unroll
  for (int i = 0; i < 16; i++) {
    const int r = 32 * lt + hrow(half, i);
    acc[i] = b2[r < OUT ? r : OUT - 1];
  }
#pragma unroll
  for (int s = 0; s < 16; s++) {
    const float v = wr[8 * (s >> 2) + (s & 3)];
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(live ? v : 0.0f, h[s], acc, 0, 0, 0);
  }
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
                      const float* __restrict__ level,
                      const float* __restrict__ campos, const float* __restrict__ packed,
                      const float* __restrict__ opacity_scale, float* __restrict__ neural_opacity,
                      float* __restrict__ opacity_tanh, uint8_t* __restrict__ mask, uint8_t* __restrict__ counts) {
  using S = Shape<K>;
  constexpr PackLayout L = pack_layout(S::GROWS);
  __shared__ float sW1[NG_SLOTS * WS];
  __shared__ float sW2[S::G1 * WS];
  __shared__ float sB2[S::G1];
  __shared__ float sOp[NG_WAVES][NG_ANCHORS * K];
  for (int e = threadIdx.x; e < NG_SLOTS * WS; e += NG_THREADS) sW1[e] = packed[L.w1t + e];
  for (int e = threadIdx.x; e < S::G1 * WS; e += NG_THREADS) sW2[e] = packed[L.w2 + e];
  for (int e = threadIdx.x; e < S::G1; e += NG_THREADS) sB2[e] = packed[L.b2 + e];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, al = lane & 31;
  const float cam[3] = {campos[0], campos[1], campos[2]};
  float* op = sOp[wave];
  for (int tile = blockIdx.x * NG_WAVES + wave; tile < ntiles; tile += gridDim.x * NG_WAVES) {
    const int64_t a = (int64_t)tile * NG_ANCHORS + al;
    float xb[NG_W1_STEPS], nv[3], dist;
    unpack_x(xb, nv, dist, fetch_x(a < N, a, half, anchor, feat, level), a < N, half, cam);
    const v16f h = hidden_layer(sW1, xb, al, half);
    const v16f o = output_tile<S::OUT0>(sW2, sB2, 0, h, al, half);
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
      const float th = ok ? op[idx] : 0.0f;
      const float t = (ok && opacity_scale != nullptr) ? th * opacity_scale[slot_anchor] : th;
      const bool sel = t > 0.0f;
      const unsigned long long bits = __ballot(sel);
      if (ok) {
        const int64_t slot = (int64_t)tile * NG_ANCHORS * K + idx;
        neural_opacity[slot] = t;
        // the backward pass needs 1 - tanh^2 of a saturated unit to the last bit: t / scale would not give it
        if (opacity_tanh != nullptr) opacity_tanh[slot] = th;
        mask[slot] = sel ? 1 : 0;
        if (idx % K == 0) counts[slot_anchor] = (uint8_t)count_lanes(bits, lane, lane + K);
      }
    }
    wave_sync();
  }
}

// ---------------------------------------------------------------------------------------------------------
// Step 2: the color and cov MLPs and the post-processing, written straight to each selected Gaussian's row
// (first[a] = number of selected offsets of all anchors before a).  Everything an offset needs from memory
// is requested before the matrix products start, so the loads complete behind them.
template <int K>
__global__ void __launch_bounds__(NG_THREADS, 2)
neural_gaussians_kernel(int64_t N, int ntiles, const float* __restrict__ anchor, const float* __restrict__ feat,
                        const float* __restrict__ level, const float* __restrict__ offsets, const float* __restrict__ scaling,
                        const float* __restrict__ campos, const float* __restrict__ packed,
                        const float* __restrict__ neural_opacity, const uint32_t* __restrict__ first,
                        float* __restrict__ xyz, float* __restrict__ color, float* __restrict__ opacity,
                        float* __restrict__ scal, float* __restrict__ rot, float* __restrict__ aux) {
  using S = Shape<K>;
  constexpr PackLayout L = pack_layout(S::GROWS);
  constexpr int WROWS = S::GROWS - S::G1;        // output rows of the two MLPs of this kernel
  constexpr int ROWS = S::OUT1 + S::OUT2;        // result rows kept per anchor: 3K color, 7K cov
  constexpr int GEO = 10;                        // per anchor: position, scaling (6), row base
  __shared__ float sW1[2 * NG_SLOTS * WS];
  __shared__ float sW2[WROWS * WS];
  __shared__ float sB2[WROWS];
  __shared__ float sOut[NG_WAVES][ROWS * SG_STRIDE];
  __shared__ float sGeo[NG_WAVES][NG_ANCHORS * GEO];
  for (int e = threadIdx.x; e < 2 * NG_SLOTS * WS; e += NG_THREADS) sW1[e] = packed[L.w1t + NG_SLOTS * WS + e];
  for (int e = threadIdx.x; e < WROWS * WS; e += NG_THREADS) sW2[e] = packed[L.w2 + S::G1 * WS + e];
  for (int e = threadIdx.x; e < WROWS; e += NG_THREADS) sB2[e] = packed[L.b2 + S::G1 + e];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, al = lane & 31;
  const float cam[3] = {campos[0], campos[1], campos[2]};
  float* out = sOut[wave];
  float* geo = sGeo[wave];
  // What a tile reads from memory.  Per anchor (lane = anchor; the two halves share the work): features, position,
  // scaling, row base.  Per offset (lane = offset within a 64-slot group): opacity and offset vector.  The next
  // tile's set is requested before the current tile's per-offset work, so it arrives behind it.
  XOperand xo;
  float p_sc[3], s_t[S::GROUPS], s_of[S::GROUPS][3];
  uint32_t p_first = 0;
  auto fetch_tile = [&](int t) {
    const int64_t a = (int64_t)t * NG_ANCHORS + al;
    xo = fetch_x(a < N, a, half, anchor, feat, level);
#pragma unroll
    for (int c = 0; c < 3; c++) p_sc[c] = a < N ? scaling[a * 6 + 3 * half + c] : 0.0f;
    p_first = a < N ? first[a] : 0u;
#pragma unroll
    for (int g = 0; g < S::GROUPS; g++) {
      const int idx = g * S::APG * K + lane;
      const int64_t sa = (int64_t)t * NG_ANCHORS + idx / K;
      const bool ok = lane < S::APG * K && idx < NG_ANCHORS * K && sa < N;
      const int64_t slot = (int64_t)t * NG_ANCHORS * K + idx;
      s_t[g] = ok ? neural_opacity[slot] : 0.0f;
#pragma unroll
      for (int c = 0; c < 3; c++) s_of[g][c] = ok ? offsets[slot * 3 + c] : 0.0f;
    }
  };
  const int stride = gridDim.x * NG_WAVES;
  int tile = blockIdx.x * NG_WAVES + wave;
  if (tile < ntiles) fetch_tile(tile);
  for (; tile < ntiles; tile += stride) {
    const int64_t a = (int64_t)tile * NG_ANCHORS + al;
    float xb[NG_W1_STEPS], nv[3], dist;
    unpack_x(xb, nv, dist, xo, a < N, half, cam);
    if (half == 0) {
      geo[al * GEO] = xo.ax; geo[al * GEO + 1] = xo.ay; geo[al * GEO + 2] = xo.az;
      geo[al * GEO + 9] = __uint_as_float(p_first);
    }
#pragma unroll
    for (int c = 0; c < 3; c++) geo[al * GEO + 3 + 3 * half + c] = p_sc[c];
    {
      const v16f h = hidden_layer(sW1, xb, al, half);
#pragma unroll
      for (int t = 0; t < S::T1; t++) {
        const v16f o = output_tile<S::OUT1>(sW2, sB2, t, h, al, half);
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int row = 32 * t + hrow(half, i);
          if (row < S::OUT1) out[row * SG_STRIDE + al] = o[i];
        }
      }
    }
    {
      const v16f h = hidden_layer(sW1 + NG_SLOTS * WS, xb, al, half);
#pragma unroll
      for (int t = 0; t < S::T2; t++) {
        const v16f o = output_tile<S::OUT2>(sW2 + (S::G2 - S::G1) * WS, sB2 + (S::G2 - S::G1), t, h, al, half);
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int row = 32 * t + hrow(half, i);
          if (row < S::OUT2) out[(S::OUT1 + row) * SG_STRIDE + al] = o[i];
        }
      }
    }
    wave_sync();
    // this tile's per-offset inputs move to fresh registers so the next tile's loads can start now
    float c_t[S::GROUPS], c_of[S::GROUPS][3];
#pragma unroll
    for (int g = 0; g < S::GROUPS; g++) {
      c_t[g] = s_t[g];
#pragma unroll
      for (int c = 0; c < 3; c++) c_of[g][c] = s_of[g][c];
    }
    if (tile + stride < ntiles) fetch_tile(tile + stride);
#pragma unroll
    for (int g = 0; g < S::GROUPS; g++) {
      const int idx = g * S::APG * K + lane;
      const int ax = idx / K, j = idx % K;
      const float t = c_t[g];
      const bool sel = t > 0.0f;
      const unsigned long long bits = __ballot(sel);
      if (sel) {
        const float* ga = geo + ax * GEO;
        const int64_t r = (int64_t)__float_as_uint(ga[9]) + count_lanes(bits, lane - j, lane);
        const float* cv = out + (S::OUT1 + 7 * j) * SG_STRIDE + ax;
        float sg[3];
#pragma unroll
        for (int c = 0; c < 3; c++) {
          xyz[r * 3 + c] = ga[c] + c_of[g][c] * ga[3 + c];
          color[r * 3 + c] = sigmoidf(out[(3 * j + c) * SG_STRIDE + ax]);
          sg[c] = sigmoidf(cv[c * SG_STRIDE]);
          scal[r * 3 + c] = ga[6 + c] * sg[c];
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
// Backward, first kernel: everything that is per offset.  The gradients of a selected Gaussian's five outputs
// become the 11 pre-activation gradients of its offset's output units (zero for unselected offsets), written
// as one record per offset; the direct gradients of offsets, scaling and anchor (xyz = anchor + offset * scaling)
// are finished here, the per-anchor sums running over an anchor's offsets in order.
template <int K>
__global__ void __launch_bounds__(NG_THREADS)
neural_offset_backward_kernel(int64_t N, int ntiles, const float* __restrict__ offsets,
                              const float* __restrict__ scaling, const float* __restrict__ neural_opacity,
                              const float* __restrict__ opacity_scale, const float* __restrict__ opacity_tanh,
                              const uint32_t* __restrict__ first, const float* __restrict__ color_out,
                              const float* __restrict__ rot_out, const float* __restrict__ aux,
                              const float* __restrict__ g_xyz, const float* __restrict__ g_color,
                              const float* __restrict__ g_opacity, const float* __restrict__ g_scal,
                              const float* __restrict__ g_rot, float* __restrict__ slot_grads,
                              float* __restrict__ d_anchor, float* __restrict__ d_offsets,
                              float* __restrict__ d_scaling) {
  using S = Shape<K>;
  __shared__ float sC[NG_WAVES][64 * 9];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = blockIdx.x * NG_WAVES + wave;
  if (tile >= ntiles) return;  // no workgroup barrier below
  float* con_s = sC[wave];
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
    float grad[NG_SLOT_GRADS] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    float con[9] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f}, dof[3] = {0.0f, 0.0f, 0.0f};
    if (sel) {
      const int64_t r = (int64_t)first[sa] + count_lanes(bits, lane - j, lane);
      const float* sc = scaling + sa * 6;
      // opacity = tanh(.) * scale (scale > 0 wherever an offset is selected): d/d pre = scale * (1 - tanh^2)
      const float ps = opacity_scale != nullptr ? opacity_scale[sa] : 1.0f;
      const float th = opacity_scale != nullptr ? opacity_tanh[slot] : t;
      grad[0] = g_opacity[r] * ((1.0f - th * th) * ps);
      const float4 ax4 = *(const float4*)(aux + r * 4);
      const float sg[3] = {ax4.x, ax4.y, ax4.z};
#pragma unroll
      for (int c = 0; c < 3; c++) {
        const float cs = color_out[r * 3 + c];
        grad[1 + c] = g_color[r * 3 + c] * (cs * (1.0f - cs));
        const float gx = g_xyz[r * 3 + c], gs = g_scal[r * 3 + c];
        con[c] = gx;
        dof[c] = gx * sc[c];
        con[3 + c] = gx * offsets[slot * 3 + c];
        con[6 + c] = gs * sg[c];
        grad[4 + c] = gs * sc[3 + c] * (sg[c] * (1.0f - sg[c]));
      }
      const float len = ax4.w;
      const float4 gr = *(const float4*)(g_rot + r * 4);
      if (len > 1e-12f) {
        const float4 qh = *(const float4*)(rot_out + r * 4);
        const float dot = ((qh.x * gr.x + qh.y * gr.y) + qh.z * gr.z) + qh.w * gr.w;
        grad[7] = (gr.x - qh.x * dot) / len; grad[8] = (gr.y - qh.y * dot) / len;
        grad[9] = (gr.z - qh.z * dot) / len; grad[10] = (gr.w - qh.w * dot) / len;
      } else {
        grad[7] = gr.x / 1e-12f; grad[8] = gr.y / 1e-12f; grad[9] = gr.z / 1e-12f; grad[10] = gr.w / 1e-12f;
      }
    }
    if (ok) {
#pragma unroll
      for (int c = 0; c < NG_SLOT_GRADS; c++) slot_grads[slot * NG_SLOT_GRADS + c] = grad[c];
#pragma unroll
      for (int c = 0; c < 3; c++) d_offsets[slot * 3 + c] = dof[c];
    }
#pragma unroll
    for (int c = 0; c < 9; c++) con_s[lane * 9 + c] = con[c];
    wave_sync();
    for (int item = lane; item < S::APG * 9; item += 64) {
      const int ga = item / 9, comp = item % 9;
      const int ax2 = g * S::APG + ga;
      const int64_t sa2 = (int64_t)tile * NG_ANCHORS + ax2;
      if (ax2 < NG_ANCHORS && sa2 < N) {
        float sum = 0.0f;
#pragma unroll
        for (int jj = 0; jj < K; jj++) sum += con_s[(ga * K + jj) * 9 + comp];
        if (comp < 3) d_anchor[sa2 * 3 + comp] = sum;
        else d_scaling[sa2 * 6 + (comp - 3)] = sum;
      }
    }
    wave_sync();
  }
}

// ---------------------------------------------------------------------------------------------------------
// Backward, second kernel: through the MLPs.  Per wave tile, with G the GROWS x 32 matrix of the tile's
// pre-activation output gradients, and per MLP
//   H = relu(W1 x + b1) (recomputed), dH = W2^T G, dHpre = dH where H > 0, dX += W1^T dHpre,
//   dW2 += G H^T, [dW1 | db1] += dHpre [x | 1]^T, db2 += row sums of G,
// the weight gradients staying in matrix-core accumulators over all tiles of the wave; they are reduced over the
// block at the end (one partial set per block; a last kernel adds the blocks in a fixed order).  The next tile's
// features and gradient records are requested before the current tile's products start.
template <int K>
struct BwdLds {
  using S = Shape<K>;
  float g[S::GROWS * SG_STRIDE];
  float hd[2 * 32 * SG_STRIDE];  // H, then dHpre; also the staging area of the final block reduction
  float x[NG_ANCHORS * SX_STRIDE];
};

// floats of one block's partial weight gradients: W2 tiles, then W1 (3 MLPs x 2 column tiles), then b2 rows
template <int K>
__host__ __device__ constexpr int partial_floats() {
  return (Shape<K>::TILES + 6) * NG_TILE + ((Shape<K>::GROWS + 63) / 64) * 64;
}

template <int K>
__global__ void __launch_bounds__(64 * Shape<K>::BWD_WAVES)
neural_mlp_backward_kernel(int64_t N, int ntiles, const float* __restrict__ anchor, const float* __restrict__ feat,
                           const float* __restrict__ level, const float* __restrict__ campos, const float* __restrict__ packed,
                           const float* __restrict__ slot_grads, float* __restrict__ d_anchor,
                           float* __restrict__ d_feat, float* __restrict__ partials) {
  using S = Shape<K>;
  constexpr PackLayout L = pack_layout(S::GROWS);
  constexpr int NW = S::BWD_WAVES, NT = 64 * NW;
  constexpr int B2N = (S::GROWS + 63) / 64;
  constexpr int TILE_FLOATS = NG_ANCHORS * K * NG_SLOT_GRADS;
  constexpr int NQ = (TILE_FLOATS / 4 + 63) / 64;  // float4 loads per lane and tile
  __shared__ BwdLds<K> lds[NW];
  __shared__ float sW1[3 * NG_SLOTS * WS];
  __shared__ float sW2[S::GROWS * WS];
  // W1's view-direction columns (c = 0..2) and distance column (c = 3) as [m][c][h]
  __shared__ __align__(16) float sWview[12 * 32];
  __shared__ unsigned short sWhere[TILE_FLOATS];  // where in G each float of a tile's records goes
  for (int e = threadIdx.x; e < 3 * NG_SLOTS * WS; e += NT) sW1[e] = packed[L.w1t + e];
  for (int e = threadIdx.x; e < S::GROWS * WS; e += NT) sW2[e] = packed[L.w2 + e];
  for (int e = threadIdx.x; e < 12 * 32; e += NT) {
    const int c = (e / 32) % 4;
    sWview[e] = packed[L.w1t + ((e / 128) * NG_SLOTS + (c < 3 ? 32 + c : 36)) * WS + e % 32];
  }
  for (int e = threadIdx.x; e < TILE_FLOATS; e += NT) {
    const int slot = e / NG_SLOT_GRADS, comp = e % NG_SLOT_GRADS, ax = slot / K, j = slot % K;
    const int row = comp == 0 ? S::G0 + j : comp < 4 ? S::G1 + 3 * j + (comp - 1) : S::G2 + 7 * j + (comp - 4);
    sWhere[e] = (unsigned short)(row * SG_STRIDE + ax);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, al = lane & 31;
  const float cam[3] = {campos[0], campos[1], campos[2]};
  BwdLds<K>& W = lds[wave];
  // rows that pad a block of G to an even count are read by the dH products and never written below
  for (int e = lane; e < S::GROWS * SG_STRIDE; e += 64) W.g[e] = 0.0f;
  __syncthreads();

  // weight-gradient accumulators: the W2 tiles, the 32 feature columns of W1 per MLP, and one tile that holds the
  // six remaining columns of W1 (view direction, bias, distance, level) of all three MLPs as its rows 6 m + c
  v16f accW2[S::TILES], accW1[3], accWx;
  float accB2[B2N];
#pragma unroll
  for (int t = 0; t < S::TILES; t++)
#pragma unroll
    for (int i = 0; i < 16; i++) accW2[t][i] = 0.0f;
#pragma unroll
  for (int m = 0; m < 3; m++) {
#pragma unroll
    for (int i = 0; i < 16; i++) accW1[m][i] = 0.0f;
  }
#pragma unroll
  for (int i = 0; i < 16; i++) accWx[i] = 0.0f;
#pragma unroll
  for (int q = 0; q < B2N; q++) accB2[q] = 0.0f;

  const int64_t total_floats = N * K * NG_SLOT_GRADS;
  const int stride = gridDim.x * NW;
  int tile = blockIdx.x * NW + wave;
  XOperand xo;
  float4 gq[NQ];
  float da[3] = {0.0f, 0.0f, 0.0f};  // the anchor's direct gradient, as the first kernel left it
  auto fetch_tile = [&](int t) {
    const int64_t a = (int64_t)t * NG_ANCHORS + al;
    xo = fetch_x(a < N, a, half, anchor, feat, level);
    if (a < N && half == 0) {
#pragma unroll
      for (int c = 0; c < 3; c++) da[c] = d_anchor[a * 3 + c];
    }
    const int64_t base = (int64_t)t * TILE_FLOATS;
#pragma unroll
    for (int q = 0; q < NQ; q++) {
      const int e = (q * 64 + lane) * 4;
      // the buffer is padded, so a float4 that straddles the end is readable; its tail is dropped below
      gq[q] = (e < TILE_FLOATS && base + e < total_floats) ? *(const float4*)(slot_grads + base + e)
                                                           : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
  };
  if (tile < ntiles) fetch_tile(tile);
  for (; tile < ntiles; tile += stride) {
    const int64_t a = (int64_t)tile * NG_ANCHORS + al;
    const bool valid = a < N;
    float nv[3], dist;
    const float da_now[3] = {da[0], da[1], da[2]};
    {
      float xb[NG_W1_STEPS];
      unpack_x(xb, nv, dist, xo, valid, half, cam);
#pragma unroll
      for (int s = 0; s < NG_W1_STEPS; s++) W.x[al * SX_STRIDE + xslot(half, s)] = xb[s];
      const int64_t left = total_floats - (int64_t)tile * TILE_FLOATS;
      const int nvalid = left < TILE_FLOATS ? (int)left : TILE_FLOATS;  // floats of this tile that exist
#pragma unroll
      for (int q = 0; q < NQ; q++) {
        const int e = (q * 64 + lane) * 4;
        if (e < TILE_FLOATS) {
          const float v[4] = {gq[q].x, gq[q].y, gq[q].z, gq[q].w};
#pragma unroll
          for (int c = 0; c < 4; c++) W.g[sWhere[e + c]] = e + c < nvalid ? v[c] : 0.0f;
        }
      }
    }
    wave_sync();

    v16f dxf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    // this half's share of the gradient of the view direction (0..2) and of the distance (3)
    float dv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const float* xrow = W.x + al * SX_STRIDE;
#pragma unroll
    for (int m = 0; m < 3; m++) {
      // the next tile's loads go out before the last and longest MLP, late enough to keep their registers
      // free until then and early enough to land behind its products
      if (m == 2 && tile + stride < ntiles) fetch_tile(tile + stride);
      const float* w1t = sW1 + m * NG_SLOTS * WS;
      v16f h = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      {
        const float* lo = w1t + half * 16 * WS + al;
        const float* hi = w1t + (32 + half) * WS + al;
#pragma unroll
        for (int s = 0; s < 16; s++) h = __builtin_amdgcn_mfma_f32_32x32x2f32(lo[s * WS], xrow[16 * half + s], h, 0, 0, 0);
        h = __builtin_amdgcn_mfma_f32_32x32x2f32(hi[0], xrow[32 + half], h, 0, 0, 0);
        h = __builtin_amdgcn_mfma_f32_32x32x2f32(hi[2 * WS], xrow[34 + half], h, 0, 0, 0);
        h = __builtin_amdgcn_mfma_f32_32x32x2f32(hi[4 * WS], xrow[36 + half], h, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 16; i++) h[i] = h[i] > 0.0f ? h[i] : 0.0f;
      }
      __builtin_amdgcn_sched_barrier(0);
      v16f dh = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      {
        // dH = W2^T G over this MLP's rows (pad row included: zero on both sides)
        const float* w2r = sW2 + (S::grow(m) + half) * WS + al;
        const float* gr = W.g + (S::grow(m) + half) * SG_STRIDE + al;
#pragma unroll
        for (int s = 0; s < even_up(S::out(m)) / 2; s++)
          dh = __builtin_amdgcn_mfma_f32_32x32x2f32(w2r[2 * s * WS], gr[2 * s * SG_STRIDE], dh, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 16; i++) dh[i] = h[i] > 0.0f ? dh[i] : 0.0f;
      __builtin_amdgcn_sched_barrier(0);
      {
        // dX += W1^T dHpre: the 32 feature rows on the matrix cores, the 3 view rows and the distance row as plain
        // sums over the 16 hidden units this lane holds (the other 16 sit in the lane of the other half)
        const float* wf = w1t + al * WS + 4 * half;
#pragma unroll
        for (int s = 0; s < 16; s++)
          dxf = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[8 * (s >> 2) + (s & 3)], dh[s], dxf, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const float4 w = *(const float4*)(sWview + (m * 4 + c) * 32 + 8 * q + 4 * half);
            dv[c] = __builtin_fmaf(w.x, dh[4 * q], dv[c]);
            dv[c] = __builtin_fmaf(w.y, dh[4 * q + 1], dv[c]);
            dv[c] = __builtin_fmaf(w.z, dh[4 * q + 2], dv[c]);
            dv[c] = __builtin_fmaf(w.w, dh[4 * q + 3], dv[c]);
          }
      }
      __builtin_amdgcn_sched_barrier(0);
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
        __builtin_amdgcn_sched_barrier(0);
      }
      const float* dhrow = W.hd + (32 + al) * SG_STRIDE;
#pragma unroll 4
      for (int s = 0; s < 16; s++) {
        const float dhv = dhrow[2 * s + half];
        const float* xr = W.x + (2 * s + half) * SX_STRIDE;
        accW1[m] = __builtin_amdgcn_mfma_f32_32x32x2f32(dhv, xr[al], accW1[m], 0, 0, 0);
        // rows 6 m .. 6 m + 5 of the shared tile take this MLP's view, bias, distance and level columns, the
        // other rows add zero
        const float xv = xr[32 + (al % 6)];
        accWx = __builtin_amdgcn_mfma_f32_32x32x2f32((al / 6) == m ? xv : 0.0f, dhv, accWx, 0, 0, 0);
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
#pragma unroll
    for (int c = 0; c < 4; c++) dv[c] += __shfl_xor(dv[c], 32);
    if (valid) {
#pragma unroll
      for (int q = 0; q < 4; q++)
        *(float4*)(d_feat + a * 32 + 8 * q + 4 * half) = make_float4(dxf[4 * q], dxf[4 * q + 1], dxf[4 * q + 2], dxf[4 * q + 3]);
      if (half == 0) {
        // the view direction n = v / |v| adds (g - n (n.g)) / |v| to the anchor's direct gradient, the distance
        // |v| adds n g
        const float ng = (nv[0] * dv[0] + nv[1] * dv[1]) + nv[2] * dv[2];
#pragma unroll
        for (int c = 0; c < 3; c++)
          d_anchor[a * 3 + c] = (da_now[c] + (dv[c] - nv[c] * ng) / dist) + nv[c] * dv[3];
      }
    }
    wave_sync();
  }

  // ---- reduce the waves' accumulators, one 32x32 tile at a time, through each wave's staging area
  float* out = partials + (size_t)blockIdx.x * partial_floats<K>();
  constexpr int NACC = S::TILES + 4;
#pragma unroll
  for (int t = 0; t < NACC; t++) {
    const v16f& acc = t < S::TILES ? accW2[t] : t < S::TILES + 3 ? accW1[t - S::TILES] : accWx;
    float* dst = out + (t < S::TILES ? t : S::TILES + 2 * (t - S::TILES)) * NG_TILE;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; i++) W.hd[hrow(half, i) * 32 + al] = acc[i];
    __syncthreads();
    for (int e = threadIdx.x; e < NG_TILE; e += NT) {
      float sum = lds[0].hd[e];
#pragma unroll
      for (int w = 1; w < NW; w++) sum += lds[w].hd[e];
      if (t < S::TILES + 3) {
        dst[e] = sum;
      } else if (e < 18 * 32) {
        // row 6 m + c, column h of the shared tile -> input slot 32 + c of W1 of MLP m: element h * 32 + c of
        // its second tile
        const int row = e >> 5, h = e & 31;
        out[(S::TILES + 2 * (row / 6) + 1) * NG_TILE + h * 32 + (row % 6)] = sum;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < B2N; q++) W.hd[q * 64 + lane] = accB2[q];
  __syncthreads();
  for (int e = threadIdx.x; e < B2N * 64; e += NT) {
    float sum = lds[0].hd[e];
#pragma unroll
    for (int w = 1; w < NW; w++) sum += lds[w].hd[e];
    out[(S::TILES + 6) * NG_TILE + e] = sum;
  }
}

// Adds the blocks' partial sets and writes the twelve weight gradients.  16 threads share an output element:
// each adds every 16th block's value, then the 16 sums are added in thread order (a fixed order for a given
// launch geometry, so results repeat bit for bit).
template <int K>
__global__ void __launch_bounds__(256)
neural_weight_reduce_kernel(int nblocks, const float* __restrict__ partials, MlpGrads d) {
  using S = Shape<K>;
  const int per1[3] = {32 * d.q.in[0] + 32, 32 * d.q.in[1] + 32, 32 * d.q.in[2] + 32};
  const int first_layers = per1[0] + per1[1] + per1[2];
  const int TOTAL = first_layers + 33 * (S::OUT0 + S::OUT1 + S::OUT2);
  __shared__ float s_part[16][17];
  const int el = threadIdx.x & 15, part = threadIdx.x >> 4;
  const int e = blockIdx.x * 16 + el;
  int src = 0;  // index inside a partial set
  float* dst = nullptr;
  if (e < TOTAL) {
    if (e < first_layers) {
      int m = 0, r = e;
      while (r >= per1[m]) { r -= per1[m]; m++; }
      const int in = d.q.in[m];
      if (r < 32 * in) {
        // column i of W1: a feature (first tile), or input slot 32 + c of the second tile: c = 0..2 the view
        // direction, 4 the distance, 5 the level (3 is the bias)
        const int h = r / in, i = r % in;
        const int c = i < 35 ? i - 32 : i == d.q.dist_col[m] ? 4 : 5;
        src = i < 32 ? (S::TILES + 2 * m) * NG_TILE + h * 32 + i : (S::TILES + 2 * m + 1) * NG_TILE + h * 32 + c;
        dst = d.p[4 * m] + r;
      } else {
        const int h = r - 32 * in;
        src = (S::TILES + 2 * m + 1) * NG_TILE + h * 32 + 3;
        dst = d.p[4 * m + 1] + h;
      }
    } else {
      int r = e - first_layers;
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
  }
  float sum = 0.0f;
  if (e < TOTAL)
    for (int b = part; b < nblocks; b += 16) sum += partials[(size_t)b * partial_floats<K>() + src];
  s_part[part][el] = sum;
  __syncthreads();
  if (part == 0 && e < TOTAL) {
    float total = s_part[0][el];
#pragma unroll
    for (int q = 1; q < 16; q++) total += s_part[q][el];
    *dst = total;
  }
}

int blocks_for(int ntiles, int waves_per_block, int per_cu) {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  const int want = (ntiles + waves_per_block - 1) / waves_per_block;
  const int cap = cus * per_cu;
  return want < cap ? want : cap;
}

template <int K>
struct Launcher {
  using S = Shape<K>;
  static void pack(const float* const* params, int input_flags, float* packed, hipStream_t stream) {
    MlpParams w;
    for (int i = 0; i < 12; i++) w.p[i] = params[i];
    w.q = mlp_inputs(input_flags);
    const int total = pack_layout(S::GROWS).total;
    hipLaunchKernelGGL(neural_pack_kernel<K>, dim3((total + 255) / 256), dim3(256), 0, stream, w, packed);
  }
  static void opacity(int64_t N, const float* anchor, const float* feat, const float* level, const float* campos,
                      const float* packed, const float* opacity_scale, float* neural_opacity, float* opacity_tanh,
                      uint8_t* mask, uint8_t* counts, hipStream_t stream) {
    const int ntiles = (int)((N + NG_ANCHORS - 1) / NG_ANCHORS);
    hipLaunchKernelGGL(neural_opacity_kernel<K>, dim3(blocks_for(ntiles, NG_WAVES, 4)), dim3(NG_THREADS), 0, stream,
                       N, ntiles, anchor, feat, level, campos, packed, opacity_scale, neural_opacity, opacity_tanh, mask,
                       counts);
  }
  static void gaussians(int64_t N, const float* anchor, const float* feat, const float* level, const float* offsets,
                        const float* scaling, const float* campos, const float* packed, const float* neural_opacity, const uint32_t* first,
                        float* xyz, float* color, float* opacity, float* scal, float* rot, float* aux,
                        hipStream_t stream) {
    const int ntiles = (int)((N + NG_ANCHORS - 1) / NG_ANCHORS);
    hipLaunchKernelGGL(neural_gaussians_kernel<K>, dim3(blocks_for(ntiles, NG_WAVES, 2)), dim3(NG_THREADS), 0, stream,
                       N, ntiles, anchor, feat, level, offsets, scaling, campos, packed, neural_opacity, first, xyz,
                       color, opacity, scal, rot, aux);
  }
  static int backward_blocks(int64_t N) {
    return blocks_for((int)((N + NG_ANCHORS - 1) / NG_ANCHORS), S::BWD_WAVES, 1);
  }
  static void backward(int64_t N, const float* anchor, const float* feat, const float* level, int input_flags,
                       const float* offsets, const float* scaling, const float* campos, const float* packed, const float* neural_opacity,
                       const float* opacity_scale, const float* opacity_tanh, const uint32_t* first,
                       const float* color_out, const float* rot_out, const float* aux, const float* g_xyz,
                       const float* g_color, const float* g_opacity, const float* g_scal, const float* g_rot,
                       float* d_anchor, float* d_feat, float* d_offsets, float* d_scaling, float* const* d_params,
                       float* slot_grads, float* partials, hipStream_t stream) {
    const int ntiles = (int)((N + NG_ANCHORS - 1) / NG_ANCHORS);
    hipLaunchKernelGGL(neural_offset_backward_kernel<K>, dim3((ntiles + NG_WAVES - 1) / NG_WAVES), dim3(NG_THREADS), 0,
                       stream, N, ntiles, offsets, scaling, neural_opacity, opacity_scale, opacity_tanh, first, color_out,
                       rot_out, aux, g_xyz, g_color, g_opacity, g_scal, g_rot, slot_grads, d_anchor, d_offsets, d_scaling);
    const int nblocks = backward_blocks(N);
    hipLaunchKernelGGL(neural_mlp_backward_kernel<K>, dim3(nblocks), dim3(64 * S::BWD_WAVES), 0, stream, N, ntiles,
                       anchor, feat, level, campos, packed, slot_grads, d_anchor, d_feat, partials);
    MlpGrads d;
    for (int i = 0; i < 12; i++) d.p[i] = d_params[i];
    d.q = mlp_inputs(input_flags);
    const int total = 32 * (d.q.in[0] + d.q.in[1] + d.q.in[2]) + 96 + 33 * (S::OUT0 + S::OUT1 + S::OUT2);
    hipLaunchKernelGGL(neural_weight_reduce_kernel<K>, dim3((total + 15) / 16), dim3(256), 0, stream, nblocks,
                       partials, d);
  }
};

}  // namespace

// n_offsets values the kernels are instantiated for
#define NG_FOR_EACH_K(X) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14) X(15) X(16)

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
#define X(KK) case KK: return (size_t)pack_layout(Shape<KK>::GROWS).total;
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

// floats of the per-offset gradient records, padded so a 16-byte read at the end stays inside
size_t neural_slot_grad_floats(int k, int64_t N) { return (size_t)N * (size_t)k * NG_SLOT_GRADS + 4; }

int launch_neural_pack(int k, const float* const* params, int input_flags, float* packed, hipStream_t stream) {
  switch (k) {
#define X(KK) case KK: Launcher<KK>::pack(params, input_flags, packed, stream); return 0;
    NG_FOR_EACH_K(X)
#undef X
    default: return 1;
  }
}

int launch_neural_opacity(int64_t N, int k, const float* anchor, const float* feat, const float* level,
                          const float* campos, const float* packed, const float* opacity_scale,
                          float* neural_opacity, float* opacity_tanh, uint8_t* mask, uint8_t* counts,
                          hipStream_t stream) {
  if (N <= 0) return 0;
  switch (k) {
#define X(KK)                                                                                                 \
  case KK:                                                                                                    \
    Launcher<KK>::opacity(N, anchor, feat, level, campos, packed, opacity_scale, neural_opacity, opacity_tanh, \
                          mask, counts, stream);                                                              \
    return 0;
    NG_FOR_EACH_K(X)
#undef X
    default: return 1;
  }
}

int launch_neural_gaussians(int64_t N, int k, const float* anchor, const float* feat, const float* level,
                            const float* offsets, const float* scaling, const float* campos, const float* packed,
                            const float* neural_opacity, const uint32_t* first, float* xyz, float* color,
                            float* opacity, float* scal, float* rot, float* aux, hipStream_t stream) {
  if (N <= 0) return 0;
  switch (k) {
#define X(KK)                                                                                                \
  case KK:                                                                                                   \
    Launcher<KK>::gaussians(N, anchor, feat, level, offsets, scaling, campos, packed, neural_opacity, first, \
                            xyz, color, opacity, scal, rot, aux, stream);                                    \
    return 0;
    NG_FOR_EACH_K(X)
#undef X
    default: return 1;
  }
}

int launch_neural_backward(int64_t N, int k, const float* anchor, const float* feat, const float* level,
                           int input_flags, const float* offsets, const float* scaling, const float* campos, const float* packed,
                           const float* neural_opacity, const float* opacity_scale, const float* opacity_tanh,
                           const uint32_t* first, const float* color_out, const float* rot_out, const float* aux,
                           const float* g_xyz, const float* g_color, const float* g_opacity, const float* g_scal,
                           const float* g_rot, float* d_anchor, float* d_feat, float* d_offsets, float* d_scaling,
                           float* const* d_params, float* slot_grads, float* partials, hipStream_t stream) {
  if (N <= 0) return 0;
  switch (k) {
#define X(KK)                                                                                              \
  case KK:                                                                                                 \
    Launcher<KK>::backward(N, anchor, feat, level, input_flags, offsets, scaling, campos, packed,          \
                           neural_opacity, opacity_scale, opacity_tanh, first, color_out, rot_out, aux,    \
                           g_xyz, g_color,                                                                 \
                           g_opacity, g_scal, g_rot, d_anchor, d_feat, d_offsets, d_scaling, d_params,     \
                           slot_grads, partials, stream);                                                  \
    return 0;
    NG_FOR_EACH_K(X)
#undef X
    default: return 1;
  }
}

}  // namespace gs
