// Stable least-significant-digit radix sort of (key, uint32 value) pairs with
// 8-bit digits, for 64-bit (tile|depth) keys and 32-bit Morton keys.  Replaces
// the library sort the reference calls at cuda_rasterizer/rasterizer_impl.cu:679-684
// and simple-knn/simple_knn.cu:210-213; stability and the [0, end_bit) bit range
// are part of the contract because tie order decides blending order.
//
// Per pass: (1) each 2048-key tile counts its digits into table[digit][tile],
// (2) an exclusive scan over the table gives every (digit, tile) its global
// base, (3) each tile ranks its keys (wave-level match by ballot, running
// per-wave digit counters), regroups them by digit in LDS and writes runs of
// equal digits to consecutive addresses.
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

constexpr int SORT_THREADS = 256;
constexpr int SORT_WAVES = SORT_THREADS / GS_WAVE;
constexpr int SORT_ITEMS = 8;
constexpr int SORT_TILE = SORT_THREADS * SORT_ITEMS;
constexpr int RADIX = 256;

template <typename K>
__device__ __forceinline__ uint32_t digit_of(K key, int shift, uint32_t mask) {
  return (uint32_t)(key >> shift) & mask;
}

template <typename K>
__global__ void __launch_bounds__(SORT_THREADS)
sort_count_kernel(int64_t n, const K* __restrict__ keys, int shift, uint32_t mask, uint32_t* __restrict__ table,
                  int ntiles) {
  __shared__ uint32_t s_hist[RADIX];
  s_hist[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * SORT_TILE;
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const int64_t idx = base + (int64_t)k * SORT_THREADS + threadIdx.x;
    if (idx < n) atomicAdd(&s_hist[digit_of(keys[idx], shift, mask)], 1u);
  }
  __syncthreads();
  table[(size_t)threadIdx.x * ntiles + blockIdx.x] = s_hist[threadIdx.x];
}

template <typename K>
__global__ void __launch_bounds__(SORT_THREADS)
sort_scatter_kernel(int64_t n, const K* __restrict__ keys_in, K* __restrict__ keys_out,
                    const uint32_t* __restrict__ vals_in, uint32_t* __restrict__ vals_out, int shift, uint32_t mask,
                    const uint32_t* __restrict__ table, int ntiles) {
  __shared__ uint32_t s_wcount[SORT_WAVES][RADIX];
  __shared__ uint32_t s_dbase[RADIX];
  __shared__ uint32_t s_gbase[RADIX];
  __shared__ uint32_t s_scan[SORT_WAVES];
  __shared__ K s_keys[SORT_TILE];
  __shared__ uint32_t s_vals[SORT_TILE];

  const int tid = threadIdx.x, lane = tid & (GS_WAVE - 1), wave = tid / GS_WAVE;
  const int64_t tile_start = (int64_t)blockIdx.x * SORT_TILE;
  const int64_t wave_start = tile_start + (int64_t)wave * (GS_WAVE * SORT_ITEMS);
  const int64_t remaining = n - tile_start;
  const int tile_count = remaining < SORT_TILE ? (int)remaining : SORT_TILE;

#pragma unroll
  for (int w = 0; w < SORT_WAVES; w++) s_wcount[w][tid] = 0;
  __syncthreads();

  K key[SORT_ITEMS];
  uint32_t val[SORT_ITEMS];
  uint32_t rank[SORT_ITEMS];
  uint32_t dig[SORT_ITEMS];
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
    dig[k] = d;
    // lanes of this wave holding the same digit
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
    rank[k] = r;
  }
  __syncthreads();

  // thread tid owns digit tid: per-wave offsets, block-level digit prefix, global base
  {
    uint32_t run = 0;
#pragma unroll
    for (int w = 0; w < SORT_WAVES; w++) {
      const uint32_t c = s_wcount[w][tid];
      s_wcount[w][tid] = run;
      run += c;
    }
    const uint32_t total = run;
    // exclusive scan of totals over the 256 digits
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
    s_dbase[tid] = ex;
    s_gbase[tid] = table[(size_t)tid * ntiles + blockIdx.x] - ex;
  }
  __syncthreads();

#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const int64_t idx = wave_start + (int64_t)k * GS_WAVE + lane;
    if (idx < n) {
      const uint32_t pos = s_dbase[dig[k]] + s_wcount[wave][dig[k]] + rank[k];
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

template <typename K>
int sort_pairs_impl(int64_t n, K* keys_a, K* keys_b, uint32_t* vals_a, uint32_t* vals_b, int end_bit, void* temp,
                    hipStream_t stream) {
  if (n <= 0) return 0;
  if (n >= (1ll << 31)) {
    set_error("radix sort: %lld pairs exceed the supported 2^31-1", (long long)n);
    return 1;
  }
  const int ntiles = (int)((n + SORT_TILE - 1) / SORT_TILE);
  uint32_t* table = (uint32_t*)temp;
  const size_t table_bytes = align_up((size_t)RADIX * ntiles * sizeof(uint32_t), 256);
  void* scan_temp = (char*)temp + table_bytes;
  const int passes = sort_num_passes(end_bit);
  K* kin = keys_a;
  K* kout = keys_b;
  uint32_t* vin = vals_a;
  uint32_t* vout = vals_b;
  for (int p = 0; p < passes; p++) {
    const int shift = 8 * p;
    const int bits = end_bit - shift >= 8 ? 8 : end_bit - shift;
    const uint32_t mask = (1u << bits) - 1u;
    hipLaunchKernelGGL(sort_count_kernel<K>, dim3(ntiles), dim3(SORT_THREADS), 0, stream, n, kin, shift, mask, table,
                       ntiles);
    launch_exclusive_sum((int64_t)RADIX * ntiles, table, table, scan_temp, stream);
    hipLaunchKernelGGL(sort_scatter_kernel<K>, dim3(ntiles), dim3(SORT_THREADS), 0, stream, n, kin, kout, vin, vout,
                       shift, mask, table, ntiles);
    K* tk = kin; kin = kout; kout = tk;
    uint32_t* tv = vin; vin = vout; vout = tv;
  }
  return 0;
}

}  // namespace

size_t sort_temp_bytes(int64_t n) {
  const int64_t ntiles = (n + SORT_TILE - 1) / SORT_TILE;
  const size_t table_bytes = align_up((size_t)RADIX * (ntiles > 0 ? ntiles : 1) * sizeof(uint32_t), 256);
  return table_bytes + scan_temp_bytes((int64_t)RADIX * (ntiles > 0 ? ntiles : 1));
}

int launch_sort_pairs_u64(int64_t n, uint64_t* keys_a, uint64_t* keys_b, uint32_t* vals_a, uint32_t* vals_b,
                          int end_bit, void* temp, hipStream_t stream) {
  return sort_pairs_impl<uint64_t>(n, keys_a, keys_b, vals_a, vals_b, end_bit, temp, stream);
}

int launch_sort_pairs_u32(int64_t n, uint32_t* keys_a, uint32_t* keys_b, uint32_t* vals_a, uint32_t* vals_b,
                          int end_bit, void* temp, hipStream_t stream) {
  return sort_pairs_impl<uint32_t>(n, keys_a, keys_b, vals_a, vals_b, end_bit, temp, stream);
}

}  // namespace gs
