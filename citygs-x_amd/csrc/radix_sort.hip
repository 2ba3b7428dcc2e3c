// Stable least-significant-digit radix sort of (key, uint32 value) pairs with
// 9-bit digits, for 64-bit (tile|depth) keys and 32-bit Morton keys.  Replaces
// the library sort the reference calls at cuda_rasterizer/rasterizer_impl.cu:679-684
// and simple-knn/simple_knn.cu:210-213; stability and the [0, end_bit) bit range
// are part of the contract because tie order decides blending order.
//
// Single-sweep organisation: one kernel reads the keys once and builds the
// digit histograms of every pass; one tiny kernel turns them into exclusive
// digit bases; then each pass is ONE kernel that reads every pair once and
// writes it once.  Inside a pass a 4096-pair tile
//   1. takes a ticket (atomic counter), so tile numbers follow start order;
//   2. ranks its keys: per wave, lanes holding equal digits find each other
//      through a lane mask per digit in LDS, and a per-wave running counter
//      per digit gives each key its rank in wave order (stable);
//   3. publishes its 512 digit counts and finds how many keys of each digit
//      precede it with a two-level look-back (below);
//   4. regroups its pairs by digit in LDS and writes each digit run to
//      consecutive addresses.
// Look-back: tiles form groups of 16.  A tile adds the counts of the tiles
// before it in its own group (these need no prefix, only the counts, so
// nothing chains), then walks back over whole groups: a group entry is
// either the group's sum ("aggregate", published by the group's last tile as
// soon as the 16 counts exist) or the inclusive prefix up to the group's end
// (published by the same tile after its own walk).  One round trip to memory
// therefore advances the prefix frontier by 16 groups = 256 tiles, instead of
// one tile per round trip in a plain chain.
// A tile only ever waits for tiles with smaller tickets, which have already
// started, so the wait always ends; the spin is bounded anyway and raises an
// error flag instead of hanging.
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

constexpr int RADIX = 1 << SORT_DIGIT_BITS;
constexpr int SORT_THREADS = RADIX;  // one thread per digit value
constexpr int SORT_WAVES = SORT_THREADS / GS_WAVE;
constexpr int SORT_ITEMS = 8;
constexpr int SORT_TILE = SORT_THREADS * SORT_ITEMS;
constexpr int MAX_PASSES = 8;
constexpr int HIST_ITEMS = 16;  // keys per thread in the histogram kernel

constexpr uint32_t FLAG_AGGREGATE = 1u << 30;
constexpr uint32_t FLAG_PREFIX = 2u << 30;
constexpr uint32_t VALUE_MASK = (1u << 30) - 1u;
constexpr int SPIN_LIMIT = 1 << 22;
constexpr int GROUP = 16;           // tiles per look-back group
constexpr int GROUP_LOOKBACK = 16;  // group entries fetched per round trip

// Control block in the workspace: [hist: MAX_PASSES*256][ticket: MAX_PASSES][error: 1][pad to 16]
// followed by the tile counts [passes][ntiles][256] and the group entries [passes][ngroups][256].
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
  K keyv[HIST_ITEMS];  // all loads in flight before the first key is counted
#pragma unroll
  for (int k = 0; k < HIST_ITEMS; k++) {
    const int64_t idx = base + (int64_t)k * SORT_THREADS + threadIdx.x;
    keyv[k] = idx < n ? keys[idx] : (K)0;
  }
#pragma unroll
  for (int k = 0; k < HIST_ITEMS; k++) {
    const int64_t idx = base + (int64_t)k * SORT_THREADS + threadIdx.x;
    const bool valid = idx < n;
    const K key = keyv[k];
    for (int p = 0; p < passes; p++) {
      const int shift = SORT_DIGIT_BITS * p;
      const int bits = end_bit - shift >= SORT_DIGIT_BITS ? SORT_DIGIT_BITS : end_bit - shift;
      const uint32_t d = digit_of(key, shift, (1u << bits) - 1u);
      // A digit shared by the whole wave (float exponent bits, unused high bits) would serialise the LDS
      // atomic 64 ways: one lane adds the wave's count instead.
      const uint64_t vm = __ballot(valid);
      const uint32_t d0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
      if (vm != 0ull && __ballot(valid && d == d0) == vm && (vm & 1ull)) {
        if ((threadIdx.x & (GS_WAVE - 1)) == 0) atomicAdd(&s_h[p][d0], (uint32_t)__popcll(vm));
      } else if (valid) {
        atomicAdd(&s_h[p][d], 1u);
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

// Sums the entries [first, last] of a 256-wide state array for digit `tid`, newest first, W entries per round
// trip, until an entry flagged FLAG_PREFIX has been added (or `first` has been passed).  Entries not yet
// published (flag 0) are polled.  Returns false when the bounded spin ran out.
template <int W>
__device__ __forceinline__ bool look_back(const uint32_t* __restrict__ state, int64_t first, int64_t last, int tid,
                                          uint32_t& sum) {
  int64_t prev = last;
  int spins = 0;
  bool finished = prev < first;
  while (!finished) {
    uint32_t s[W];
#pragma unroll
    for (int i = 0; i < W; i++) {
      const int64_t t = prev - i;
      // before `first` there is nothing: reads as a published prefix of 0, which ends the walk
      s[i] = t >= first ? __hip_atomic_load(state + (size_t)t * RADIX + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                        : FLAG_PREFIX;
    }
    int consumed = 0;
#pragma unroll
    for (int i = 0; i < W; i++) {
      if (finished || consumed != i) continue;  // stopped at an entry that is not published yet
      const uint32_t flag = s[i] & ~VALUE_MASK;
      if (flag == 0u) continue;
      sum += s[i] & VALUE_MASK;
      consumed = i + 1;
      if (flag == FLAG_PREFIX) finished = true;
    }
    prev -= consumed;
    if (!finished && consumed < W) {
      if (++spins > SPIN_LIMIT) return false;
      __builtin_amdgcn_s_sleep(1);
    }
  }
  return true;
}

// Adds up the counts of the earlier tiles of the group, fetched into `earlier` beforehand; entries that had not
// been published at the time of the fetch are polled.  Returns false when the bounded spin ran out.
__device__ __forceinline__ bool level1_sum(const uint32_t* earlier, const uint32_t* __restrict__ tile_state,
                                           uint32_t tile, int tid, uint32_t& sum) {
  uint32_t missing = 0;
#pragma unroll
  for (int i = 0; i < GROUP - 1; i++) {
    sum += earlier[i] & VALUE_MASK;
    if ((earlier[i] & ~VALUE_MASK) == 0u) missing |= 1u << i;
  }
  for (int spins = 0; missing != 0u;) {
    const int i = __builtin_ctz(missing);
    const uint32_t v = __hip_atomic_load(tile_state + (size_t)(tile - 1 - i) * RADIX + tid, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
    if ((v & ~VALUE_MASK) != 0u) {
      sum += v & VALUE_MASK;
      missing &= missing - 1u;
    } else if (++spins > SPIN_LIMIT) {
      return false;
    } else {
      __builtin_amdgcn_s_sleep(1);
    }
  }
  return true;
}

template <typename K>
__global__ void __launch_bounds__(SORT_THREADS)
sort_onesweep_kernel(int64_t n, const K* __restrict__ keys_in, K* __restrict__ keys_out,
                     const uint32_t* __restrict__ vals_in, uint32_t* __restrict__ vals_out, int shift, uint32_t mask,
                     const uint32_t* __restrict__ digit_base, uint32_t* __restrict__ ticket,
                     uint32_t* __restrict__ tile_state, uint32_t* __restrict__ group_state, int ntiles,
                     uint32_t* __restrict__ error_flag) {
  __shared__ uint32_t s_wcount[SORT_WAVES][RADIX];
  __shared__ uint32_t s_gbase[RADIX];
  __shared__ uint32_t s_scan[SORT_WAVES];
  __shared__ uint32_t s_tile;
  // regrouping buffer: the lane masks of the ranking first, then the keys, then the values
  constexpr size_t BUF_BYTES = sizeof(K) * SORT_TILE > sizeof(unsigned long long) * SORT_WAVES * RADIX
                                   ? sizeof(K) * SORT_TILE
                                   : sizeof(unsigned long long) * SORT_WAVES * RADIX;
  __shared__ __attribute__((aligned(16))) unsigned char s_buf[BUF_BYTES];
  K* s_keys = reinterpret_cast<K*>(s_buf);
  unsigned long long (*s_mask)[RADIX] = reinterpret_cast<unsigned long long (*)[RADIX]>(s_buf);

  const int tid = threadIdx.x, lane = tid & (GS_WAVE - 1), wave = tid / GS_WAVE;
  if (tid == 0) s_tile = atomicAdd(ticket, 1u);
#pragma unroll
  for (int w = 0; w < SORT_WAVES; w++) {
    s_wcount[w][tid] = 0;
    s_mask[w][tid] = 0ull;
  }
  s_gbase[tid] = 0u;  // first the tile's digit histogram, later the global bases
  __syncthreads();
  const uint32_t tile = s_tile;
  const int64_t tile_start = (int64_t)tile * SORT_TILE;
  const int64_t wave_start = tile_start + (int64_t)wave * (GS_WAVE * SORT_ITEMS);
  const int64_t remaining = n - tile_start;
  const int tile_count = remaining < SORT_TILE ? (int)remaining : SORT_TILE;

  K key[SORT_ITEMS];
  uint32_t val[SORT_ITEMS];
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const int64_t idx = wave_start + (int64_t)k * GS_WAVE + lane;
    const bool valid = idx < n;
    key[k] = valid ? keys_in[idx] : (K)0;
    val[k] = valid ? vals_in[idx] : 0u;
  }

  // The tile's digit counts first, by plain LDS atomics, so that they can be published before the (longer)
  // ranking: the later tiles of the group and the group's closing tile wait for nothing else, and this
  // tile's own look-back loads travel while it ranks and regroups.
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const bool valid = wave_start + (int64_t)k * GS_WAVE + lane < n;
    const uint32_t d = digit_of(key[k], shift, mask);
    // a digit shared by the whole wave would serialise 64 ways: one lane adds the count
    const uint64_t vm = __ballot(valid);
    const uint32_t d0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
    if (vm != 0ull && __ballot(valid && d == d0) == vm && (vm & 1ull)) {
      if (lane == 0) atomicAdd(&s_gbase[d0], (uint32_t)__popcll(vm));
    } else if (valid) {
      atomicAdd(&s_gbase[d], 1u);
    }
  }
  __syncthreads();
  const uint32_t total = s_gbase[tid];  // thread tid owns digit tid
  __hip_atomic_store(tile_state + (size_t)tile * RADIX + tid, FLAG_AGGREGATE | total, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
  // Look-back, level 1, issue: the counts of the earlier tiles of the own group
  const int64_t group = tile / GROUP;
  const int in_group = (int)(tile % GROUP);
  const bool closes_group = in_group == GROUP - 1;  // an incomplete last group is never looked at
  uint32_t earlier[GROUP - 1];
#pragma unroll
  for (int i = 0; i < GROUP - 1; i++)
    earlier[i] = i < in_group ? __hip_atomic_load(tile_state + (size_t)(tile - 1 - i) * RADIX + tid, __ATOMIC_RELAXED,
                                                  __HIP_MEMORY_SCOPE_AGENT)
                              : FLAG_AGGREGATE;
  uint32_t before_tiles = 0;
  bool ok = true;
  // The closing tile of a group resolves level 1 at once and publishes the group's sum: every later group
  // is waiting for it.  The other tiles come back to their loads after the regrouping.
  if (closes_group) {
    ok = level1_sum(earlier, tile_state, tile, tid, before_tiles);
    __hip_atomic_store(group_state + (size_t)group * RADIX + tid,
                       (group == 0 ? FLAG_PREFIX : FLAG_AGGREGATE) | ((before_tiles + total) & VALUE_MASK),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // Ranking.  LDS operations of one wave execute in program order, which the two steps below rely on; none
  // of them waits for an earlier one's result, so all items are in flight together.
  // Step 1: the lanes of the wave that hold the same digit find each other through a 64-bit lane mask per
  // digit: every lane ORs its bit in, reads the mask back, and clears it for the next item.
  // (typed as LDS pointers: through plain pointers these volatile accesses come out as flat loads and stores,
  // which are slower and wait on the memory counters as well)
  typedef __attribute__((address_space(3))) unsigned long long lds_mask;
  typedef __attribute__((address_space(3))) uint32_t lds_u32;
  volatile lds_mask* vmask = (lds_mask*)&s_mask[wave][0];
  volatile lds_u32* vcount = (lds_u32*)&s_wcount[wave][0];
  const unsigned long long lane_bit = 1ull << lane;
  const unsigned long long lt_mask = lane_bit - 1ull;
  uint32_t match[SORT_ITEMS];  // rank in the wave | valid << 17; later the place in the regrouped tile
  constexpr int HALF = SORT_ITEMS / 2;  // two batches keep fewer masks live in registers
#pragma unroll
  for (int h = 0; h < 2; h++) {
    unsigned long long same[HALF];
#pragma unroll
    for (int j = 0; j < HALF; j++) {
      const int k = h * HALF + j;
      const bool valid = wave_start + (int64_t)k * GS_WAVE + lane < n;
      const uint32_t d = digit_of(key[k], shift, mask);
      if (valid) atomicOr(&s_mask[wave][d], lane_bit);
      __builtin_amdgcn_wave_barrier();
      same[j] = valid ? vmask[d] : 0ull;
      __builtin_amdgcn_wave_barrier();
      if (valid) vmask[d] = 0ull;
      __builtin_amdgcn_wave_barrier();
    }
    // Step 2: a per-wave running count per digit turns the place among the matching lanes into a rank in
    // wave order (stable): all lanes read the count, the first of the matching lanes adds their number.
#pragma unroll
    for (int j = 0; j < HALF; j++) {
      const int k = h * HALF + j;
      const bool valid = same[j] != 0ull;
      const uint32_t d = digit_of(key[k], shift, mask);
      const unsigned long long lower = same[j] & lt_mask;
      const uint32_t before = valid ? vcount[d] : 0u;
      __builtin_amdgcn_wave_barrier();
      if (valid && lower == 0ull) atomicAdd(&s_wcount[wave][d], (uint32_t)__popcll(same[j]));
      __builtin_amdgcn_wave_barrier();
      match[k] = (before + (uint32_t)__popcll(lower)) | (valid ? 1u << 17 : 0u);
    }
  }
  __syncthreads();

  uint32_t wcount[SORT_WAVES];
#pragma unroll
  for (int w = 0; w < SORT_WAVES; w++) wcount[w] = s_wcount[w][tid];

  // digit prefix inside the tile, then regroup the keys by digit in LDS
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
  {
    // s_wcount[w][d] becomes the place in the regrouped tile of wave w's first key with digit d
    uint32_t run = ex;
#pragma unroll
    for (int w = 0; w < SORT_WAVES; w++) {
      s_wcount[w][tid] = run;
      run += wcount[w];
    }
  }
  __syncthreads();

#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const uint32_t d = digit_of(key[k], shift, mask);
    const bool valid = match[k] & (1u << 17);
    const uint32_t pos = s_wcount[wave][d] + (match[k] & 0xFFFFu);
    if (valid) s_keys[pos] = key[k];
    match[k] = valid ? pos : 0xFFFFFFFFu;  // now: place in the regrouped tile, or none
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const int p = k * SORT_THREADS + tid;
    key[k] = p < tile_count ? s_keys[p] : (K)0;  // from here on: the key at regrouped place p
  }

  // Look-back, level 1, use (the closing tile has done it already)
  if (!closes_group) ok = level1_sum(earlier, tile_state, tile, tid, before_tiles);
  // level 2: whole groups
  if (group != 0) {
    ok = look_back<GROUP_LOOKBACK>(group_state, 0, group - 1, tid, before_tiles) && ok;
    if (closes_group)
      __hip_atomic_store(group_state + (size_t)group * RADIX + tid, FLAG_PREFIX | ((before_tiles + total) & VALUE_MASK),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (!ok) *error_flag = 1u;
  s_gbase[tid] = digit_base[tid] + before_tiles - ex;
  __syncthreads();  // also: every read of s_keys above is complete, the buffer can take the values

  uint32_t dst[SORT_ITEMS];
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const int p = k * SORT_THREADS + tid;
    dst[k] = s_gbase[digit_of(key[k], shift, mask)] + (uint32_t)p;
    if (p < tile_count) keys_out[dst[k]] = key[k];
  }
  uint32_t* s_vals = reinterpret_cast<uint32_t*>(s_keys);
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++)
    if (match[k] != 0xFFFFFFFFu) s_vals[match[k]] = val[k];
  __syncthreads();
#pragma unroll
  for (int k = 0; k < SORT_ITEMS; k++) {
    const int p = k * SORT_THREADS + tid;
    if (p < tile_count) vals_out[dst[k]] = s_vals[p];
  }
}

struct SortLayout {
  size_t ctrl_words, state_words, total_bytes;
  int ntiles, ngroups;
};

SortLayout sort_layout(int64_t n) {
  SortLayout L;
  const int64_t nt = (n + SORT_TILE - 1) / SORT_TILE;
  L.ntiles = (int)(nt > 0 ? nt : 1);
  L.ctrl_words = CTRL_WORDS;
  L.ngroups = (L.ntiles + GROUP - 1) / GROUP;
  L.state_words = (size_t)MAX_PASSES * (L.ntiles + L.ngroups) * RADIX;
  L.total_bytes = align_up((L.ctrl_words + L.state_words) * sizeof(uint32_t), 256);
  return L;
}

template <typename K>
int sort_pairs_impl(int64_t n, K* keys_a, K* keys_b, uint32_t* vals_a, uint32_t* vals_b, int end_bit, void* temp,
                    hipStream_t stream) {
  if (n <= 0) return 0;
  if (n > sort_max_pairs()) {
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
  uint32_t* group_states = states + (size_t)passes * L.ntiles * RADIX;
  const int64_t clear_words = (int64_t)(L.ctrl_words + (size_t)passes * (L.ntiles + L.ngroups) * RADIX);
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
    const int shift = SORT_DIGIT_BITS * p;
    const int bits = end_bit - shift >= SORT_DIGIT_BITS ? SORT_DIGIT_BITS : end_bit - shift;
    const uint32_t mask = (1u << bits) - 1u;
    hipLaunchKernelGGL(sort_onesweep_kernel<K>, dim3(L.ntiles), dim3(SORT_THREADS), 0, stream, n, kin, kout, vin, vout,
                       shift, mask, hist + p * RADIX, tickets + p, states + (size_t)p * L.ntiles * RADIX,
                       group_states + (size_t)p * L.ngroups * RADIX, L.ntiles, error_flag);
    K* tk = kin; kin = kout; kout = tk;
    uint32_t* tv = vin; vin = vout; vout = tv;
  }
  return 0;
}

}  // namespace

size_t sort_temp_bytes(int64_t n) { return sort_layout(n).total_bytes; }

// A look-back word carries a 30-bit count beside its two flag bits, and a count can be the whole input.
int64_t sort_max_pairs() { return (int64_t)VALUE_MASK - 1; }

size_t sort_error_word_offset() { return (size_t)(MAX_PASSES * RADIX + MAX_PASSES) * sizeof(uint32_t); }
const uint32_t* sort_error_word(const void* temp) {
  return (const uint32_t*)((const char*)temp + sort_error_word_offset());
}

namespace {
__global__ void sort_fault_report_kernel(const uint32_t* __restrict__ error_word, uint32_t* __restrict__ fault_word) {
  if (*error_word != 0u) __hip_atomic_store(fault_word, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
}  // namespace

// Raises the host-visible fault word if the sort that last used the workspace gave up waiting.
int launch_sort_fault_report(const uint32_t* error_word, uint32_t* fault_word, hipStream_t stream) {
  if (error_word == nullptr || fault_word == nullptr) return 0;
  hipLaunchKernelGGL(sort_fault_report_kernel, dim3(1), dim3(1), 0, stream, error_word, fault_word);
  return 0;
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
