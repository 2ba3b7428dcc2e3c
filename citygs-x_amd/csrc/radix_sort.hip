// Stable least-significant-digit radix sort of (key, uint32 value) pairs with
// 8-bit digits, for 64-bit (tile|depth) keys and 32-bit Morton keys.  Replaces
// the library sort the reference calls at cuda_rasterizer/rasterizer_impl.cu:679-684
// and simple-knn/simple_knn.cu:210-213; stability and the [0, end_bit) bit range
// are part of the contract because tie order decides blending order.
//
// Single-sweep organisation: one kernel reads the keys once and builds the
// digit histograms of every pass; one tiny kernel turns them into exclusive
// digit bases; then each pass is ONE kernel that reads every pair once and
// writes it once.  Inside a pass a 4096-pair tile
//   1. takes a ticket (atomic counter), so tile numbers follow start order;
//   2. ranks its keys: per wave, lanes holding equal digits are matched with
//      eight ballots, and a per-wave running counter per digit in LDS gives
//      each key its rank in wave order (stable);
//   3. publishes its 256 digit counts (flag "aggregate") and looks back over
//      the preceding tiles, adding aggregates until it meets a tile whose
//      inclusive prefix is already published, then publishes its own prefix;
//   4. regroups its pairs by digit in LDS and writes each digit run to
//      consecutive addresses.
// A tile only ever waits for tiles with smaller tickets, which have already
// started, so the wait always ends; the spin is bounded anyway and raises an
// error flag instead of hanging.
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

constexpr int SORT_THREADS = 256;
constexpr int SORT_WAVES = SORT_THREADS / GS_WAVE;
constexpr int SORT_ITEMS = 16;
constexpr int SORT_TILE = SORT_THREADS * SORT_ITEMS;
constexpr int RADIX = 256;
constexpr int MAX_PASSES = 8;
constexpr int HIST_ITEMS = 16;  // keys per thread in the histogram kernel

constexpr uint32_t FLAG_AGGREGATE = 1u << 30;
constexpr uint32_t FLAG_PREFIX = 2u << 30;
constexpr uint32_t VALUE_MASK = (1u << 30) - 1u;
constexpr int SPIN_LIMIT = 1 << 22;

// Control block in the workspace: [hist: MAX_PASSES*256][ticket: MAX_PASSES][error: 1][pad to 16]
// followed by the tile states [passes][ntiles][256].
constexpr size_t CTRL_WORDS = MAX_PASSES * RADIX + 16;

template <typename K>
__device__ __forceinline__ uint32_t digit_of(K key, int shift, uint32_t mask) {
  return (uint32_t)(key >> shift) & mask;
}

__global__ void sort_clear_kernel(int64_t nwords, uint32_t* __restrict__ p) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < nwords) p[i] = 0u;
}

template <typename K>
__global__ void __launch_bounds__(SORT_THREADS)
sort_histogram_kernel(int64_t n, const K* __restrict__ keys, int passes, int end_bit, uint32_t* __restrict__ hist) {
  __shared__ uint32_t s_h[MAX_PASSES][RADIX];
  for (int p = 0; p < passes; p++) s_h[p][threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * (SORT_THREADS * HIST_ITEMS);
#pragma unroll 4
  for (int k = 0; k < HIST_ITEMS; k++) {
    const int64_t idx = base + (int64_t)k * SORT_THREADS + threadIdx.x;
    if (idx < n) {
      const K key = keys[idx];
      for (int p = 0; p < passes; p++) {
        const int shift = 8 * p;
        const int bits = end_bit - shift >= 8 ? 8 : end_bit - shift;
        atomicAdd(&s_h[p][digit_of(key, shift, (1u << bits) - 1u)], 1u);
      }
    }
  }
  __syncthreads();
  for (int p = 0; p < passes; p++) {
    const uint32_t c = s_h[p][threadIdx.x];
    if (c) atomicAdd(&hist[p * RADIX + threadIdx.x], c);
  }
}

// One workgroup per pass: counts -> exclusive bases, in place.
__global__ void __launch_bounds__(RADIX) sort_digit_bases_kernel(uint32_t* __restrict__ hist) {
  __shared__ uint32_t s_w[RADIX / GS_WAVE];
  uint32_t* h = hist + blockIdx.x * RADIX;
  const int lane = threadIdx.x & (GS_WAVE - 1), wave = threadIdx.x / GS_WAVE;
  const uint32_t v = h[threadIdx.x];
  uint32_t inc = v;
#pragma unroll
  for (int d = 1; d < GS_WAVE; d <<= 1) {
    const uint32_t o = __shfl_up(inc, d, GS_WAVE);
    if (lane >= d) inc += o;
  }
  if (lane == GS_WAVE - 1) s_w[wave] = inc;
  __syncthreads();
  uint32_t base = 0;
  for (int w = 0; w < wave; w++) base += s_w[w];
  h[threadIdx.x] = base + inc - v;
}

template <typename K>
__global__ void __launch_bounds__(SORT_THREADS)
sort_onesweep_kernel(int64_t n, const K* __restrict__ keys_in, K* __restrict__ keys_out,
                     const uint32_t* __restrict__ vals_in, uint32_t* __restrict__ vals_out, int shift, uint32_t mask,
                     const uint32_t* __restrict__ digit_base, uint32_t* __restrict__ ticket,
                     uint32_t* __restrict__ tile_state, uint32_t* __restrict__ error_flag) {
  __shared__ uint32_t s_wcount[SORT_WAVES][RADIX];
  __shared__ uint32_t s_dbase[RADIX];
  __shared__ uint32_t s_gbase[RADIX];
  __shared__ uint32_t s_scan[SORT_WAVES];
  __shared__ uint32_t s_tile;
  __shared__ K s_keys[SORT_TILE];
  __shared__ uint32_t s_vals[SORT_TILE];

  const int tid = threadIdx.x, lane = tid & (GS_WAVE - 1), wave = tid / GS_WAVE;
  if (tid == 0) s_tile = atomicAdd(ticket, 1u);
#pragma unroll
  for (int w = 0; w < SORT_WAVES; w++) s_wcount[w][tid] = 0;
  __syncthreads();
  const uint32_t tile = s_tile;
  const int64_t tile_start = (int64_t)tile * SORT_TILE;
  const int64_t wave_start = tile_start + (int64_t)wave * (GS_WAVE * SORT_ITEMS);
  const int64_t remaining = n - tile_start;
  const int tile_count = remaining < SORT_TILE ? (int)remaining : SORT_TILE;

  K key[SORT_ITEMS];
  uint32_t val[SORT_ITEMS];
  uint16_t rank[SORT_ITEMS];
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const int64_t idx = wave_start + (int64_t)k * GS_WAVE + lane;
    const bool valid = idx < n;
    key[k] = valid ? keys_in[idx] : (K)0;
    val[k] = valid ? vals_in[idx] : 0u;
  }
  const uint64_t lt_mask = (1ull << lane) - 1ull;
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const int64_t idx = wave_start + (int64_t)k * GS_WAVE + lane;
    const bool valid = idx < n;
    const uint32_t d = digit_of(key[k], shift, mask);
    uint64_t same = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; b++) {
      const bool bit = (d >> b) & 1u;
      const uint64_t vote = __ballot(valid && bit);
      same &= bit ? vote : ~vote;
    }
    uint32_t r = 0;
    if (valid) {
      const uint32_t before = s_wcount[wave][d];
      r = before + (uint32_t)__popcll(same & lt_mask);
      __builtin_amdgcn_wave_barrier();
      if ((same & lt_mask) == 0ull) s_wcount[wave][d] = before + (uint32_t)__popcll(same);
    }
    __builtin_amdgcn_wave_barrier();
    rank[k] = (uint16_t)r;
  }
  __syncthreads();

  // thread tid owns digit tid
  uint32_t total = 0;
  {
    uint32_t run = 0;
#pragma unroll
    for (int w = 0; w < SORT_WAVES; w++) {
      const uint32_t c = s_wcount[w][tid];
      s_wcount[w][tid] = run;
      run += c;
    }
    total = run;
  }
  uint32_t* my_state = tile_state + (size_t)tile * RADIX + tid;
  __hip_atomic_store(my_state, (tile == 0 ? FLAG_PREFIX : FLAG_AGGREGATE) | total, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);

  // digit prefix inside the tile (needed for the LDS regrouping); overlaps with the look-back latency
  uint32_t inc = total;
#pragma unroll
  for (int dd = 1; dd < GS_WAVE; dd <<= 1) {
    const uint32_t o = __shfl_up(inc, dd, GS_WAVE);
    if (lane >= dd) inc += o;
  }
  if (lane == GS_WAVE - 1) s_scan[wave] = inc;
  __syncthreads();
  uint32_t wbase = 0;
#pragma unroll
  for (int w = 0; w < SORT_WAVES; w++)
    if (w < wave) wbase += s_scan[w];
  const uint32_t ex = wbase + inc - total;

  // decoupled look-back over the preceding tiles
  uint32_t before_tiles = 0;
  if (tile != 0) {
    int64_t prev = (int64_t)tile - 1;
    int spins = 0;
    for (;;) {
      const uint32_t s = __hip_atomic_load(tile_state + (size_t)prev * RADIX + tid, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
      const uint32_t flag = s & ~VALUE_MASK;
      if (flag == 0u) {
        if (++spins > SPIN_LIMIT) {
          *error_flag = 1u;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
        continue;
      }
      before_tiles += s & VALUE_MASK;
      if (flag == FLAG_PREFIX) break;
      prev--;  // an aggregate: keep walking back (prev >= 0 because tile 0 always publishes a prefix)
    }
    __hip_atomic_store(my_state, FLAG_PREFIX | ((before_tiles + total) & VALUE_MASK), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  }
  s_dbase[tid] = ex;
  s_gbase[tid] = digit_base[tid] + before_tiles - ex;
  __syncthreads();

#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const int64_t idx = wave_start + (int64_t)k * GS_WAVE + lane;
    if (idx < n) {
      const uint32_t d = digit_of(key[k], shift, mask);
      const uint32_t pos = s_dbase[d] + s_wcount[wave][d] + (uint32_t)rank[k];
      s_keys[pos] = key[k];
      s_vals[pos] = val[k];
    }
  }
  __syncthreads();

#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const int p = k * SORT_THREADS + tid;
    if (p < tile_count) {
      const K kk = s_keys[p];
      const uint32_t dst = s_gbase[digit_of(kk, shift, mask)] + (uint32_t)p;
      keys_out[dst] = kk;
      vals_out[dst] = s_vals[p];
    }
  }
}

struct SortLayout {
  size_t ctrl_words, state_words, total_bytes;
  int ntiles;
};

SortLayout sort_layout(int64_t n) {
  SortLayout L;
  const int64_t nt = (n + SORT_TILE - 1) / SORT_TILE;
  L.ntiles = (int)(nt > 0 ? nt : 1);
  L.ctrl_words = CTRL_WORDS;
  L.state_words = (size_t)MAX_PASSES * L.ntiles * RADIX;
  L.total_bytes = align_up((L.ctrl_words + L.state_words) * sizeof(uint32_t), 256);
  return L;
}

template <typename K>
int sort_pairs_impl(int64_t n, K* keys_a, K* keys_b, uint32_t* vals_a, uint32_t* vals_b, int end_bit, void* temp,
                    hipStream_t stream) {
  if (n <= 0) return 0;
  if (n >= (int64_t)VALUE_MASK) {
    set_error("radix sort: %lld pairs exceed the supported 2^30-2", (long long)n);
    return 1;
  }
  const int passes = sort_num_passes(end_bit);
  if (passes > MAX_PASSES) {
    set_error("radix sort: end_bit %d needs more than %d passes", end_bit, MAX_PASSES);
    return 1;
  }
  const SortLayout L = sort_layout(n);
  uint32_t* ctrl = (uint32_t*)temp;
  uint32_t* hist = ctrl;
  uint32_t* tickets = ctrl + MAX_PASSES * RADIX;
  uint32_t* error_flag = tickets + MAX_PASSES;
  uint32_t* states = ctrl + L.ctrl_words;
  const int64_t clear_words = (int64_t)(L.ctrl_words + (size_t)passes * L.ntiles * RADIX);
  hipLaunchKernelGGL(sort_clear_kernel, dim3((unsigned)((clear_words + 255) / 256)), dim3(256), 0, stream, clear_words,
                     ctrl);
  const int hist_blocks = (int)((n + SORT_THREADS * HIST_ITEMS - 1) / (SORT_THREADS * HIST_ITEMS));
  hipLaunchKernelGGL(sort_histogram_kernel<K>, dim3(hist_blocks), dim3(SORT_THREADS), 0, stream, n, keys_a, passes,
                     end_bit, hist);
  hipLaunchKernelGGL(sort_digit_bases_kernel, dim3(passes), dim3(RADIX), 0, stream, hist);
  K* kin = keys_a;
  K* kout = keys_b;
  uint32_t* vin = vals_a;
  uint32_t* vout = vals_b;
  for (int p = 0; p < passes; p++) {
    const int shift = 8 * p;
    const int bits = end_bit - shift >= 8 ? 8 : end_bit - shift;
    const uint32_t mask = (1u << bits) - 1u;
    hipLaunchKernelGGL(sort_onesweep_kernel<K>, dim3(L.ntiles), dim3(SORT_THREADS), 0, stream, n, kin, kout, vin, vout,
                       shift, mask, hist + p * RADIX, tickets + p, states + (size_t)p * L.ntiles * RADIX, error_flag);
    K* tk = kin; kin = kout; kout = tk;
    uint32_t* tv = vin; vin = vout; vout = tv;
  }
  return 0;
}

}  // namespace

size_t sort_temp_bytes(int64_t n) { return sort_layout(n).total_bytes; }

int launch_sort_pairs_u64(int64_t n, uint64_t* keys_a, uint64_t* keys_b, uint32_t* vals_a, uint32_t* vals_b,
                          int end_bit, void* temp, hipStream_t stream) {
  return sort_pairs_impl<uint64_t>(n, keys_a, keys_b, vals_a, vals_b, end_bit, temp, stream);
}

int launch_sort_pairs_u32(int64_t n, uint32_t* keys_a, uint32_t* keys_b, uint32_t* vals_a, uint32_t* vals_b,
                          int end_bit, void* temp, hipStream_t stream) {
  return sort_pairs_impl<uint32_t>(n, keys_a, keys_b, vals_a, vals_b, end_bit, temp, stream);
}

}  // namespace gs
