// Binning by tile without a global sort.  The list the rasterizer needs is "instances ordered by (tile, depth
// bits), ties in emission order" (cuda_rasterizer/rasterizer_impl.cu:74-144, :675-697: duplicateWithKeys, a stable
// radix sort on the (tile << 32 | depth) key, identifyTileRanges).  The tile part of that key takes few values
// and every tile's list is short, so the same list comes out of
//   1. a counting sort by tile: per-workgroup tile histograms in LDS, a prefix over workgroups and tiles (which
//      is also the table of tile ranges), and a scatter of every instance into its tile's segment, in any order;
//   2. one workgroup per tile sorting its segment in registers by (depth bits, emission index): the emission index
//      is unique, so the order does not depend on how the scatter happened to fill the segment, and it is the
//      order a stable sort on the depth bits would leave.
// No pass over all instances per digit, no look-back chain.  Lists of up to 2048 records are sorted in registers
// by a bitonic network (below); longer ones by a radix sort on the depth bits that stays inside the CU
// (tile_radix.hip).  The ranges kernel sorts the tiles into those classes.
#include <atomic>

#include "gs_common.h"
#include "gs_kernels.h"
#include "tile_lists.h"

namespace gs {
namespace {

constexpr int BK_THREADS = 1024;        // counting and scatter kernels
constexpr int BK_MAX_BLOCKS = 256;
constexpr int BK_MIN_PER_BLOCK = 4096;  // Gaussians per workgroup, at least
constexpr int BK_BATCH = 4;             // Gaussians a thread loads ahead

__host__ __device__ inline int bucket_per_block(int P) {
  // a multiple of four, so that a thread's four consecutive Gaussians start at a 16-byte boundary of every
  // per-Gaussian array of words
  const int per = ((P + BK_MAX_BLOCKS - 1) / BK_MAX_BLOCKS + 3) & ~3;
  return per < BK_MIN_PER_BLOCK ? BK_MIN_PER_BLOCK : per;
}
__host__ __device__ inline int bucket_blocks(int P) {
  const int per = bucket_per_block(P);
  return (P + per - 1) / per;
}

// Which chunk of Gaussians a workgroup takes: a tile's records lie in chunk order, so with chunk = workgroup index
// the records that share a 64-byte line would come from eight different L2s, each of which writes its part of
// the line back on its own.  Dealt out by xcd_contiguous_index, neighbours in memory meet in one L2.
__device__ __forceinline__ int chunk_of_workgroup(int b, int n) { return (int)xcd_contiguous_index(b, n); }

// 1a. Per Gaussian the number of tiles it touches (rasterizer_impl.cu:264-288), per workgroup the number of
// instances of every tile.  The workgroup's Gaussians are a contiguous chunk; the scatter walks the same chunk.
__global__ void __launch_bounds__(BK_THREADS)
bucket_count_kernel(int P, int per_block, uint32_t gx, uint32_t gy, const int* __restrict__ radii,
                    const float2* __restrict__ means2D, const uint8_t* __restrict__ compute_locally,
                    uint32_t* __restrict__ tiles_touched, uint32_t* __restrict__ table,
                    uint32_t* __restrict__ block_sums, int* __restrict__ zero_per_gaussian) {
  extern __shared__ uint32_t s_hist[];
  __shared__ uint32_t s_sum[BK_THREADS / GS_WAVE];
  __shared__ uint32_t s_heads[BK_THREADS];
  uint32_t my_sum = 0;  // tiles touched by this thread's Gaussians
  const uint32_t T = gx * gy;
  uint8_t* s_local = reinterpret_cast<uint8_t*>(s_hist + T);  // the tile mask, read once per visited tile
  int masked = 0;
  for (uint32_t t = threadIdx.x; t < T; t += BK_THREADS) {
    s_hist[t] = 0u;
    const uint8_t c = compute_locally[t];
    s_local[t] = c;
    masked |= c == 0 ? 1 : 0;
  }
  // (also the barrier behind the loop) without a tile mask the rectangles are walked with the work spread evenly
  const bool all_local = __syncthreads_or(masked) == 0;
  lds_word* heads = (lds_word*)s_heads + (threadIdx.x / GS_WAVE) * GS_WAVE;
  const int chunk = chunk_of_workgroup(blockIdx.x, gridDim.x);
  const int first = chunk * per_block;
  const int last = first + per_block < P ? first + per_block : P;
  // four Gaussians per round: their loads go out together, then each is walked (the loop bounds are the same
  // for every thread of the workgroup, because the walk is a wave-wide operation)
  struct None { uint32_t unused; } none = {0u};
  for (int base = first; base < last; base += BK_BATCH * BK_THREADS) {
    int r[BK_BATCH];
    float2 p[BK_BATCH];
#pragma unroll
    for (int q = 0; q < BK_BATCH; q++) {
      const int i = base + (int)threadIdx.x + q * BK_THREADS;
      r[q] = i < last ? radii[i] : 0;
      p[q] = i < last ? means2D[i] : make_float2(0.0f, 0.0f);
    }
#pragma unroll
    for (int q = 0; q < BK_BATCH; q++) {
      const int i = base + (int)threadIdx.x + q * BK_THREADS;
      const bool live = i < last && r[q] > 0;
      const Rect rc = live ? get_rect(p[q].x, p[q].y, r[q], gx, gy) : Rect{0u, 0u, 0u, 0u};
      const uint32_t cnt =
          all_local ? walk_wave_rects_flat(live, rc, gx, none, heads,
                                           [&](const None&, uint32_t tile, uint32_t) { atomicAdd(&s_hist[tile], 1u); })
                    : walk_wave_rects(
                          live, rc, gx, none, [&](uint32_t tile) { return s_local[tile] != 0; },
                          [&](const None&, uint32_t tile, uint32_t) { atomicAdd(&s_hist[tile], 1u); });
      if (i < last) {
        tiles_touched[i] = cnt;
        my_sum += cnt;
        // an array of one word per Gaussian that the caller wants cleared on the way (saves a launch)
        if (zero_per_gaussian != nullptr) zero_per_gaussian[i] = 0;
      }
    }
  }
#pragma unroll
  for (int d = GS_WAVE / 2; d >= 1; d >>= 1) my_sum += __shfl_xor(my_sum, d, GS_WAVE);
  if ((threadIdx.x & (GS_WAVE - 1)) == 0) s_sum[threadIdx.x / GS_WAVE] = my_sum;
  __syncthreads();
  uint32_t* row = table + (size_t)chunk * T;
  for (uint32_t t = threadIdx.x; t < T; t += BK_THREADS) row[t] = s_hist[t];
  // the workgroup's share of the prefix sum over the Gaussians (the scatter kernel finishes it)
  if (threadIdx.x == 0) {
    uint32_t all = 0;
    for (int w = 0; w < BK_THREADS / GS_WAVE; w++) all += s_sum[w];
    block_sums[chunk] = all;
  }
}

// 1b. Per tile: the workgroups' counts become exclusive prefixes in place, their sum goes to totals.  A workgroup
// takes 32 tiles (one 128-byte row segment) by 8 runs of consecutive workgroup rows; a thread holds its run in
// registers, the runs' sums meet in LDS.
constexpr int COL_TILES = 32, COL_RUNS = 8, COL_RUN_MAX = BK_MAX_BLOCKS / COL_RUNS;
__global__ void __launch_bounds__(COL_TILES * COL_RUNS)
bucket_columns_kernel(int nblocks, uint32_t T, uint32_t* __restrict__ table, uint32_t* __restrict__ totals) {
  __shared__ uint32_t s_sum[COL_RUNS][COL_TILES];
  const int tx = threadIdx.x % COL_TILES, run = threadIdx.x / COL_TILES;
  const uint32_t t = blockIdx.x * COL_TILES + tx;
  const int len = (nblocks + COL_RUNS - 1) / COL_RUNS;  // <= COL_RUN_MAX
  const int b0 = run * len;
  uint32_t c[COL_RUN_MAX];
  uint32_t sum = 0;
#pragma unroll
  for (int k = 0; k < COL_RUN_MAX; k++) {
    const int b = b0 + k;
    c[k] = (k < len && b < nblocks && t < T) ? table[(size_t)b * T + t] : 0u;
    sum += c[k];
  }
  s_sum[run][tx] = sum;
  __syncthreads();
  uint32_t before = 0, all = 0;
#pragma unroll
  for (int r = 0; r < COL_RUNS; r++) {
    const uint32_t v = s_sum[r][tx];
    if (r < run) before += v;
    all += v;
  }
  if (t >= T) return;
#pragma unroll
  for (int k = 0; k < COL_RUN_MAX; k++) {
    const int b = b0 + k;
    if (k < len && b < nblocks) table[(size_t)b * T + t] = before;
    before += c[k];
  }
  if (run == 0) totals[t] = all;
}

__device__ __forceinline__ uint32_t wave_inclusive_scan_u32(uint32_t v, int lane) {
#pragma unroll
  for (int d = 1; d < GS_WAVE; d <<= 1) {
    const uint32_t o = __shfl_up(v, d, GS_WAVE);
    if (lane >= d) v += o;
  }
  return v;
}

// 1c. One workgroup: exclusive prefix of the tile totals = the tile ranges (rasterizer_impl.cu:122-144 leaves
// (0, 0) for a tile without instances).  Tiles whose lists are too long for the register sort are entered in two
// lists for the radix sort's kernels: lists of more than small_limit and at most mid_limit records ascending from
// tile_lists[0], longer ones descending from tile_lists[T - 1]; tile_lists[T] = (number of the longer ones << 16
// | number of the others) (T is at most 30000).  The lists beyond block_limit records, which are split before they
// are sorted and take several times as long, are entered a second time in a list of their own, so that the larger
// kernel can start with them: their number in tile_lists[T + 1], the tiles ascending from tile_lists[T + 2].  The longest list, that word and then the number of instances are
// stored where the host can read them (host_words[1], [2] and [0]; the host polls word 0, so it is written last).
__global__ void __launch_bounds__(1024)
bucket_ranges_kernel(uint32_t T, uint32_t small_limit, uint32_t mid_limit, uint32_t block_limit,
                     const uint32_t* __restrict__ totals,
                     uint32_t* __restrict__ ranges, uint32_t* __restrict__ tile_lists,
                     uint32_t* __restrict__ block_sums, int nblocks, uint32_t* __restrict__ host_words,
                     uint32_t cap_instances, uint32_t cap_longest, uint32_t* __restrict__ fits_word,
                     uint32_t* __restrict__ clear_word) {
  constexpr int ITEMS = 4;  // consecutive tiles per thread: the usual grids (up to 4096 tiles) take one round
  __shared__ uint32_t s_wave[16], s_wave_class[16], s_wave_split[16], s_max[16];
  __shared__ double s_exact[16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  {
    // the counting workgroups' sums of tiles touched (at most BK_MAX_BLOCKS <= 1024 of them) become exclusive
    // prefixes in place
    const uint32_t b = (int)threadIdx.x < nblocks ? block_sums[threadIdx.x] : 0u;
    const uint32_t inc = wave_inclusive_scan_u32(b, lane);
    if (lane == 63) s_wave[wave] = inc;
    __syncthreads();
    uint32_t base = 0;
#pragma unroll
    for (int w = 0; w < 16; w++)
      if (w < wave) base += s_wave[w];
    if ((int)threadIdx.x < nblocks) block_sums[threadIdx.x] = base + inc - b;
    __syncthreads();
  }
  uint32_t carry = 0, carry_class = 0, carry_split = 0, longest = 0;
  double exact = 0.0;  // the number of instances without the 32-bit wrap-around of the prefix sums
  for (uint32_t start = 0; start < T; start += 1024 * ITEMS) {
    const uint32_t t0 = start + threadIdx.x * ITEMS;
    uint32_t v[ITEMS], c[ITEMS], sum = 0, sum_class = 0, sum_split = 0;
#pragma unroll
    for (int q = 0; q < ITEMS; q++) v[q] = t0 + q < T ? totals[t0 + q] : 0u;
#pragma unroll
    for (int q = 0; q < ITEMS; q++) {
      c[q] = v[q] > mid_limit ? 0x10000u : (v[q] > small_limit ? 1u : 0u);
      sum_split += v[q] > block_limit ? 1u : 0u;
      longest = v[q] > longest ? v[q] : longest;
      exact += (double)v[q];
      sum += v[q];
      sum_class += c[q];
    }
    const uint32_t inc = wave_inclusive_scan_u32(sum, lane);
    // (a wave without a long list, the usual case, has nothing to scan)
    const uint32_t inc_class = __ballot(sum_class != 0u) != 0ull ? wave_inclusive_scan_u32(sum_class, lane) : 0u;
    const uint32_t inc_split = __ballot(sum_split != 0u) != 0ull ? wave_inclusive_scan_u32(sum_split, lane) : 0u;
    if (lane == 63) {
      s_wave[wave] = inc;
      s_wave_class[wave] = inc_class;
      s_wave_split[wave] = inc_split;
    }
    __syncthreads();
    uint32_t base = 0, all = 0, base_class = 0, all_class = 0, base_split = 0, all_split = 0;
#pragma unroll
    for (int w = 0; w < 16; w++) {
      const uint32_t s = s_wave[w], sc = s_wave_class[w], ss = s_wave_split[w];
      if (w < wave) {
        base += s;
        base_class += sc;
        base_split += ss;
      }
      all += s;
      all_class += sc;
      all_split += ss;
    }
    __syncthreads();
    uint32_t begin = carry + base + inc - sum, begin_class = carry_class + base_class + inc_class - sum_class;
    uint32_t begin_split = carry_split + base_split + inc_split - sum_split;
#pragma unroll
    for (int q = 0; q < ITEMS; q++) {
      if (t0 + q < T) {
        ranges[2 * (t0 + q)] = v[q] ? begin : 0u;
        ranges[2 * (t0 + q) + 1] = v[q] ? begin + v[q] : 0u;
        if (c[q] == 1u) tile_lists[begin_class & 0xFFFFu] = t0 + q;
        if (c[q] == 0x10000u) tile_lists[T - 1u - (begin_class >> 16)] = t0 + q;
        if (v[q] > block_limit) tile_lists[T + 2u + begin_split] = t0 + q;
      }
      begin += v[q];
      begin_class += c[q];
      begin_split += v[q] > block_limit ? 1u : 0u;
    }
    carry += all;
    carry_class += all_class;
    carry_split += all_split;
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    const uint32_t o = __shfl_xor(longest, d, GS_WAVE);
    longest = o > longest ? o : longest;
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) exact += __shfl_xor(exact, d, GS_WAVE);
  if (lane == 0) {
    s_max[wave] = longest;
    s_exact[wave] = exact;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t m = 0;
    double all = 0.0;
    for (int w = 0; w < 16; w++) {
      m = s_max[w] > m ? s_max[w] : m;
      all += s_exact[w];
    }
    tile_lists[T] = carry_class;
    tile_lists[T + 1u] = carry_split;
    if (clear_word != nullptr) *clear_word = 0u;  // (a word the caller wants cleared on the way: saves a launch)
    // more instances than 32-bit positions can address: the host must not go on with the wrapped count
    const uint32_t reported = all > (double)GS_MAX_INSTANCES ? GS_TOO_MANY_INSTANCES : carry;
    // Kernels launched ahead of the host's decision (buffers sized from the caller's expectation) look at this
    // word and do nothing unless the view fits what they were launched for.
    *fits_word = (reported <= cap_instances && m <= cap_longest) ? 1u : 0u;
    __hip_atomic_store(host_words + 1, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __hip_atomic_store(host_words + 2, carry_class, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __hip_atomic_store(host_words, reported, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// 1d. Every instance goes to its tile's segment: segment start (ranges) + instances of earlier workgroups
// (table) + a place among this workgroup's own, handed out by an LDS counter.  The record is one 16-byte store
// (Gaussian, emission index, depth bits, 0) (rasterizer_impl.cu:74-117 writes the same instances in emission
// order); the per-tile sorts read the depth bits and look the other two up once a record's place is known, inside
// the tile's own segment.  The kernel also finishes the prefix sum
// over the Gaussians' tile counts (rasterizer_impl.cu:648) for its own chunk, which is where the emission
// indices come from: a thread owns four consecutive Gaussians, the workgroup scans the threads' sums, and the
// inclusive sums go to point_offsets on the way (the backward pass reads them).
// fits_word (optional): the kernel was launched before the host knew the instance count; it does nothing unless
// bucket_ranges_kernel found that the view fits the buffers it was launched with.
__global__ void __launch_bounds__(BK_THREADS)
bucket_scatter_kernel(int P, int per_block, uint32_t gx, uint32_t gy, const float2* __restrict__ means2D,
                      const float* __restrict__ depths, const uint32_t* __restrict__ tiles_touched,
                      const uint32_t* __restrict__ block_prefix, uint32_t* __restrict__ point_offsets,
                      const int* __restrict__ radii, const uint8_t* __restrict__ compute_locally,
                      const uint32_t* __restrict__ table, const uint32_t* __restrict__ ranges,
                      TileRecord* __restrict__ records, const uint32_t* __restrict__ fits_word,
                      int vector_loads) {
  extern __shared__ uint32_t s_next[];
  __shared__ uint32_t s_wave[BK_THREADS / GS_WAVE];
  __shared__ uint32_t s_heads[BK_THREADS];
  if (fits_word != nullptr && *fits_word == 0u) return;
  const uint32_t T = gx * gy;
  uint8_t* s_local = reinterpret_cast<uint8_t*>(s_next + T);
  const int chunk = chunk_of_workgroup(blockIdx.x, gridDim.x);
  const uint32_t* row = table + (size_t)chunk * T;
  int masked = 0;
  for (uint32_t t = threadIdx.x; t < T; t += BK_THREADS) {
    s_next[t] = ranges[2 * t] + row[t];
    const uint8_t c = compute_locally[t];
    s_local[t] = c;
    masked |= c == 0 ? 1 : 0;
  }
  const bool all_local = __syncthreads_or(masked) == 0;  // (as in the counting kernel; also the barrier)
  const int lane = threadIdx.x & (GS_WAVE - 1), wave = threadIdx.x / GS_WAVE;
  lds_word* heads = (lds_word*)s_heads + wave * GS_WAVE;
  const int first = chunk * per_block;
  const int last = first + per_block < P ? first + per_block : P;
  struct Owner { uint32_t first, depth_bits, id; };
  uint32_t carry = block_prefix[chunk];  // instances of the Gaussians before this round
  for (int base = first; base < last; base += BK_BATCH * BK_THREADS) {
    const int i0 = base + (int)threadIdx.x * BK_BATCH;
    int r[BK_BATCH];
    float2 p[BK_BATCH];
    uint32_t tt[BK_BATCH], dbits[BK_BATCH], sum = 0;
    static_assert(BK_BATCH == 4, "a thread's Gaussians are loaded as four-word vectors");
    const bool whole = vector_loads != 0 && i0 + BK_BATCH <= last;
    if (whole) {
      // (i0 is a multiple of four and the host found every array 16-byte aligned: 16-byte loads)
      const int4 rv = *reinterpret_cast<const int4*>(radii + i0);
      const uint4 tv = *reinterpret_cast<const uint4*>(tiles_touched + i0);
      const uint4 dv = *reinterpret_cast<const uint4*>(depths + i0);
      const float4 m01 = *reinterpret_cast<const float4*>(means2D + i0);
      const float4 m23 = *reinterpret_cast<const float4*>(means2D + i0 + 2);
      r[0] = rv.x; r[1] = rv.y; r[2] = rv.z; r[3] = rv.w;
      tt[0] = tv.x; tt[1] = tv.y; tt[2] = tv.z; tt[3] = tv.w;
      dbits[0] = dv.x; dbits[1] = dv.y; dbits[2] = dv.z; dbits[3] = dv.w;
      p[0] = make_float2(m01.x, m01.y); p[1] = make_float2(m01.z, m01.w);
      p[2] = make_float2(m23.x, m23.y); p[3] = make_float2(m23.z, m23.w);
    } else {
#pragma unroll
      for (int q = 0; q < BK_BATCH; q++) {
        const int i = i0 + q;
        r[q] = i < last ? radii[i] : 0;
        p[q] = i < last ? means2D[i] : make_float2(0.0f, 0.0f);
        dbits[q] = i < last ? __float_as_uint(depths[i]) : 0u;
        tt[q] = i < last ? tiles_touched[i] : 0u;
      }
    }
#pragma unroll
    for (int q = 0; q < BK_BATCH; q++) sum += tt[q];
    const uint32_t inc = wave_inclusive_scan_u32(sum, lane);
    if (lane == GS_WAVE - 1) s_wave[wave] = inc;
    __syncthreads();
    uint32_t before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < BK_THREADS / GS_WAVE; w++) {
      const uint32_t v = s_wave[w];
      if (w < wave) before += v;
      all += v;
    }
    __syncthreads();
    uint32_t run = carry + before + inc - sum;  // emission index of this thread's first instance
    carry += all;
#pragma unroll
    for (int q = 0; q < BK_BATCH; q++) {
      const int i = i0 + q;
      const bool live = i < last && r[q] > 0;
      const Rect rc = live ? get_rect(p[q].x, p[q].y, r[q], gx, gy) : Rect{0u, 0u, 0u, 0u};
      const Owner mine = {run, dbits[q], (uint32_t)i};
      run += tt[q];
      tt[q] = run;  // from here on: the inclusive sum
      const auto emit = [&](const Owner& o, uint32_t tile, uint32_t rank) {
        const uint32_t e = o.first + rank;
        const uint32_t pos = atomicAdd(&s_next[tile], 1u);
        records[pos] = make_uint4(o.id, e, o.depth_bits, 0u);
      };
      if (all_local) walk_wave_rects_flat(live, rc, gx, mine, heads, emit);
      else walk_wave_rects(live, rc, gx, mine, [&](uint32_t tile) { return s_local[tile] != 0; }, emit);
    }
    if (whole) {
      *reinterpret_cast<uint4*>(point_offsets + i0) = make_uint4(tt[0], tt[1], tt[2], tt[3]);
    } else {
#pragma unroll
      for (int q = 0; q < BK_BATCH; q++)
        if (i0 + q < last) point_offsets[i0 + q] = tt[q];
    }
  }
}

// 1d'. The same scatter for a view in which a workgroup walks its chunk of Gaussians in one round (at most
// BK_BATCH * BK_THREADS of them) and its instances fit the LDS: the records are staged in LDS, ordered by tile (the
// counting kernels' table gives the workgroup's own count per tile: the next workgroup's prefix minus its own), and
// written out tile by tile, so that the records a workgroup adds to one tile's segment leave as one run, all
// workgroups at about the same time.  Every 16-byte record written on its own costs the memory a 64-byte write;
// runs that meet in the L2 cost their bytes.  A workgroup with more than `cap` instances stores directly, as the
// kernel above does.
// Dynamic LDS: 9 bytes per tile and 12 bytes per staged record.
__global__ void __launch_bounds__(BK_THREADS)
bucket_scatter_staged_kernel(int P, int per_block, int nblocks, uint32_t gx, uint32_t gy,
                             const float2* __restrict__ means2D, const float* __restrict__ depths,
                             const uint32_t* __restrict__ tiles_touched, const uint32_t* __restrict__ block_prefix,
                             uint32_t* __restrict__ point_offsets, const int* __restrict__ radii,
                             const uint8_t* __restrict__ compute_locally, const uint32_t* __restrict__ table,
                             const uint32_t* __restrict__ totals, const uint32_t* __restrict__ ranges,
                             TileRecord* __restrict__ records, const uint32_t* __restrict__ fits_word,
                             int vector_loads, uint32_t cap) {
  extern __shared__ uint32_t s_mem[];
  __shared__ uint32_t s_wave[BK_THREADS / GS_WAVE], s_wave_tiles[BK_THREADS / GS_WAVE];
  __shared__ uint32_t s_heads[BK_THREADS];
  if (fits_word != nullptr && *fits_word == 0u) return;
  const uint32_t T = gx * gy;
  uint32_t* s_next = s_mem;         // [T] where the workgroup's first record of a tile goes in memory
  uint32_t* s_cursor = s_mem + T;   // [T] next free place of a tile: in the staging arrays, or in memory
  uint32_t* stage_g = s_cursor + T; // [cap] x 3: Gaussian, emission index, depth bits
  uint32_t* stage_e = stage_g + cap;
  uint32_t* stage_z = stage_e + cap;
  uint8_t* s_local = reinterpret_cast<uint8_t*>(stage_z + cap);
  const int lane = threadIdx.x & (GS_WAVE - 1), wave = threadIdx.x / GS_WAVE;
  const int chunk = chunk_of_workgroup(blockIdx.x, gridDim.x);
  const uint32_t* row = table + (size_t)chunk * T;
  const uint32_t* next_row = chunk + 1 < nblocks ? table + (size_t)(chunk + 1) * T : totals;
  const int first = chunk * per_block;
  const int last = first + per_block < P ? first + per_block : P;
  // (the workgroup's Gaussians are asked for first: their latency passes behind the set-up of the tiles)
  const int i0 = first + (int)threadIdx.x * BK_BATCH;
  int r[BK_BATCH];
  float2 p[BK_BATCH];
  uint32_t tt[BK_BATCH], dbits[BK_BATCH], sum = 0;
  static_assert(BK_BATCH == 4, "a thread's Gaussians are loaded as four-word vectors");
  const bool whole = vector_loads != 0 && i0 + BK_BATCH <= last;
  if (whole) {
    const int4 rv = *reinterpret_cast<const int4*>(radii + i0);
    const uint4 tv = *reinterpret_cast<const uint4*>(tiles_touched + i0);
    const uint4 dv = *reinterpret_cast<const uint4*>(depths + i0);
    const float4 m01 = *reinterpret_cast<const float4*>(means2D + i0);
    const float4 m23 = *reinterpret_cast<const float4*>(means2D + i0 + 2);
    r[0] = rv.x; r[1] = rv.y; r[2] = rv.z; r[3] = rv.w;
    tt[0] = tv.x; tt[1] = tv.y; tt[2] = tv.z; tt[3] = tv.w;
    dbits[0] = dv.x; dbits[1] = dv.y; dbits[2] = dv.z; dbits[3] = dv.w;
    p[0] = make_float2(m01.x, m01.y); p[1] = make_float2(m01.z, m01.w);
    p[2] = make_float2(m23.x, m23.y); p[3] = make_float2(m23.z, m23.w);
  } else {
#pragma unroll
    for (int q = 0; q < BK_BATCH; q++) {
      const int i = i0 + q;
      r[q] = i < last ? radii[i] : 0;
      p[q] = i < last ? means2D[i] : make_float2(0.0f, 0.0f);
      dbits[q] = i < last ? __float_as_uint(depths[i]) : 0u;
      tt[q] = i < last ? tiles_touched[i] : 0u;
    }
  }
  int masked = 0;
  constexpr int TILES_AHEAD = 4;  // tiles a thread has in flight: a usual grid is set up with one memory latency
  for (uint32_t t0 = threadIdx.x; t0 < T; t0 += TILES_AHEAD * BK_THREADS) {
    uint32_t before[TILES_AHEAD], upto[TILES_AHEAD], begin[TILES_AHEAD];
    uint8_t c[TILES_AHEAD];
#pragma unroll
    for (int u = 0; u < TILES_AHEAD; u++) {
      const uint32_t t = t0 + (uint32_t)u * BK_THREADS;
      before[u] = t < T ? row[t] : 0u;
      upto[u] = t < T ? next_row[t] : 0u;
      begin[u] = t < T ? ranges[2 * t] : 0u;
      c[u] = t < T ? compute_locally[t] : (uint8_t)1;
    }
#pragma unroll
    for (int u = 0; u < TILES_AHEAD; u++) {
      const uint32_t t = t0 + (uint32_t)u * BK_THREADS;
      if (t < T) {
        s_next[t] = begin[u] + before[u];
        s_cursor[t] = upto[u] - before[u];  // the workgroup's own instances of the tile
        s_local[t] = c[u];
        masked |= c[u] == 0 ? 1 : 0;
      }
    }
  }
  const bool all_local = __syncthreads_or(masked) == 0;
  // exclusive prefix of the counts over the tiles, in place: a thread owns `per` consecutive tiles
  const uint32_t per = (T + BK_THREADS - 1) / BK_THREADS, t_first = threadIdx.x * per;
  uint32_t own = 0;
  for (uint32_t k = 0; k < per; k++)
    if (t_first + k < T) own += s_cursor[t_first + k];
  const uint32_t own_inc = wave_inclusive_scan_u32(own, lane);
  // (the prefix sum over the Gaussians' tile counts shares the barrier)
#pragma unroll
  for (int q = 0; q < BK_BATCH; q++) sum += tt[q];
  const uint32_t inc = wave_inclusive_scan_u32(sum, lane);
  if (lane == GS_WAVE - 1) {
    s_wave_tiles[wave] = own_inc;
    s_wave[wave] = inc;
  }
  __syncthreads();
  uint32_t tiles_before = 0, total = 0, before = 0;
#pragma unroll
  for (int w = 0; w < BK_THREADS / GS_WAVE; w++) {
    const uint32_t v = s_wave_tiles[w];
    if (w < wave) {
      tiles_before += v;
      before += s_wave[w];
    }
    total += v;
  }
  const bool staged = total <= cap;  // (the same for the whole workgroup)
  {
    uint32_t run = tiles_before + own_inc - own;
    for (uint32_t k = 0; k < per; k++)
      if (t_first + k < T) {
        const uint32_t v = s_cursor[t_first + k];
        s_cursor[t_first + k] = staged ? run : s_next[t_first + k];
        run += v;
      }
  }
  __syncthreads();
  lds_word* heads = (lds_word*)s_heads + wave * GS_WAVE;
  struct Owner { uint32_t first, depth_bits, id; };
  {
    uint32_t run = block_prefix[chunk] + before + inc - sum;  // emission index of this thread's first instance
#pragma unroll
    for (int q = 0; q < BK_BATCH; q++) {
      const int i = i0 + q;
      const bool live = i < last && r[q] > 0;
      const Rect rc = live ? get_rect(p[q].x, p[q].y, r[q], gx, gy) : Rect{0u, 0u, 0u, 0u};
      const Owner mine = {run, dbits[q], (uint32_t)i};
      run += tt[q];
      tt[q] = run;  // from here on: the inclusive sum
      const auto emit = [&](const Owner& o, uint32_t tile, uint32_t rank) {
        const uint32_t e = o.first + rank;
        const uint32_t pos = atomicAdd(&s_cursor[tile], 1u);
        if (staged) {
          stage_g[pos] = o.id;
          stage_e[pos] = e;
          stage_z[pos] = o.depth_bits;
        } else {
          records[pos] = make_uint4(o.id, e, o.depth_bits, 0u);
        }
      };
      if (all_local) walk_wave_rects_flat(live, rc, gx, mine, heads, emit);
      else walk_wave_rects(live, rc, gx, mine, [&](uint32_t tile) { return s_local[tile] != 0; }, emit);
    }
    if (whole) {
      *reinterpret_cast<uint4*>(point_offsets + i0) = make_uint4(tt[0], tt[1], tt[2], tt[3]);
    } else {
#pragma unroll
      for (int q = 0; q < BK_BATCH; q++)
        if (i0 + q < last) point_offsets[i0 + q] = tt[q];
    }
  }
  if (!staged) return;
  __syncthreads();
  // every tile's run: staged at [cursor of the tile before, cursor of the tile), to memory from s_next on
  for (uint32_t t = threadIdx.x; t < T; t += BK_THREADS) {
    const uint32_t lo = t > 0u ? s_cursor[t - 1u] : 0u, hi = s_cursor[t];
    TileRecord* dst = records + s_next[t];
    for (uint32_t k = lo; k < hi; k++) dst[k - lo] = make_uint4(stage_g[k], stage_e[k], stage_z[k], 0u);
  }
}

// 2. Per-tile sort, register variant: one workgroup of W waves per tile (4 for lists of up to 256 records, 8 up
// to 2048).  A wave holds 64 E keys, key i = r * 64 + lane in register r of its lane, and the waves hold
// consecutive runs of 64 E, so a list of up to 64 E W records is sorted with E = 1 .. 4.  In the bitonic network
// a step pairs i with i ^ j:
//   j < 64        the partner sits in another lane, same register: one cross-lane read, keep the smaller or larger;
//   64 <= j < 64E the partner sits in another register of the same lane: no data moves at all;
//   j >= 64 E     the partner sits in another wave: one exchange through LDS (3 such steps in a whole sort with
//                 4 waves, 6 with 8).
// A tile takes as long as the instruction stream of one of its waves, and the kernel as long as its longest tiles:
// a long list is spread over more waves rather than more registers per lane (eight waves with four records per
// lane for 2048 records, not four with eight).
//
// The key is one 32-bit word: (depth bits - smallest depth bits of the list) >> shift in the high bits, the
// record's place in the unsorted segment in the low log2(64 E W) bits; shift is what it takes to fit the list's
// range of depth bits (0 when it fits as it is).  A step then costs three vector instructions per key (one move,
// one comparison, one select) where a 64-bit key cost five.  Keys whose depths agree in the bits kept end up next
// to each other in the order of their places; the last step (emit_list_entry) puts every such run into its true
// order, by all depth bits and then the emission index, exactly as it does for runs of equal depth bits.  Depths
// inside a tile are spread over the view's range, so with the 21 to 24 bits kept runs are as rare as before.

// Which element of a pair (a, b) each lane keeps is decided in scalar registers: keep_min is the lane mask of the
// elements that keep the smaller one, less the lane mask of a < b; a lane keeps a where the two agree.
__device__ __forceinline__ uint32_t keep_pair(uint32_t a, uint32_t b, uint64_t keep_min) {
  const uint64_t less = __builtin_amdgcn_ballot_w64(a < b);
  return __builtin_amdgcn_inverse_ballot_w64(~(less ^ keep_min)) ? a : b;
}

// Lanes whose bit J of the lane number is clear: the lower element of every pair at distance J.
template <int J>
__device__ __forceinline__ constexpr uint64_t lower_lanes() {
  uint64_t m = 0;
  for (int l = 0; l < 64; l++)
    if ((l & J) == 0) m |= 1ull << l;
  return m;
}

// x of lane (lane ^ J), J = 1, 2, 4 or 8, by DPP moves inside a 16-lane row (xor 4 = reverse the quads' lanes,
// then mirror the half rows).  Every lane has a source, so nothing is kept of the old value (with bound_ctrl set
// the destination needs no initialisation).  A variable-distance __shfl_xor is a ds_bpermute, whose latency
// every one of the sort's dependent steps would wait for.  All 64 lanes must be active.
template <int J>
__device__ __forceinline__ uint32_t xor_lane(uint32_t x) {
  static_assert(J == 1 || J == 2 || J == 4 || J == 8, "distance inside a 16-lane row");
  if constexpr (J == 1) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
  } else if constexpr (J == 2) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
  } else if constexpr (J == 4) {
    const int t = __builtin_amdgcn_update_dpp(0, (int)x, 0x1B, 0xF, 0xF, true);     // quad_perm [3,2,1,0]: lane ^ 3
    return (uint32_t)__builtin_amdgcn_update_dpp(0, t, 0x141, 0xF, 0xF, true);      // row_half_mirror: lane ^ 7
  } else {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x128, 0xF, 0xF, true);  // row_ror:8
  }
}

// One step of the network with the partner in lane ^ J.  ascending[r]: lane mask of the elements of register r
// that lie in an ascending run of this stage.
template <int E, int J>
__device__ __forceinline__ void lane_step(uint32_t (&v)[E], const uint64_t (&ascending)[E]) {
  constexpr uint64_t lower = lower_lanes<J>();
#pragma unroll
  for (int r = 0; r < E; r++) {
    const uint64_t keep_min = ~(lower ^ ascending[r]);  // the lower element of an ascending pair, the upper of a descending
    if constexpr (J < 16) {
      v[r] = keep_pair(v[r], xor_lane<J>(v[r]), keep_min);
    } else {
      // v_permlane16_swap / v_permlane32_swap exchange the odd rows (the upper half) of their first operand with
      // the even rows (the lower half) of the second: from two copies of x they leave the lower element of every
      // pair in all lanes of the first result and the upper element in the second, so both lanes of a pair
      // compare the same two values and each keeps its own.
      if constexpr (J == 16) {
        const auto p = __builtin_amdgcn_permlane16_swap(v[r], v[r], false, false);
        v[r] = keep_pair(p[0], p[1], keep_min);
      } else {
        const auto p = __builtin_amdgcn_permlane32_swap(v[r], v[r], false, false);
        v[r] = keep_pair(p[0], p[1], keep_min);
      }
    }
  }
}

template <int E, int W>
__device__ __forceinline__ void register_sort(uint32_t (&v)[E], uint32_t wave, uint32_t lane, uint32_t* s_x) {
  constexpr uint32_t M = 64u * E * W;
  const uint32_t row0 = wave * E;
  for (uint32_t k = 2; k <= M; k <<= 1) {
    // the direction of this stage's runs: element i = (row << 6 | lane) ascends where (i & k) == 0, which is a
    // property of the lane below k = 64 and of the register (and wave) from there on
    uint64_t ascending[E];
    {
      const uint64_t by_lane = __builtin_amdgcn_ballot_w64((lane & k) == 0u);
#pragma unroll
      for (int r = 0; r < E; r++) {
        const uint64_t m = k < 64u ? by_lane : ((((row0 + (uint32_t)r) << 6) & k) == 0u ? ~0ull : 0ull);
        // (wave-uniform: kept in scalar registers)
        ascending[r] = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(m >> 32)) << 32) |
                       (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)m);
      }
    }
    for (uint32_t j = k >> 1; j >= 64; j >>= 1) {
      if (j < 64u * E) {
        const uint32_t jr = j >> 6;
#pragma unroll
        for (int b = 1; b < E; b <<= 1) {
          if (jr != (uint32_t)b) continue;
#pragma unroll
          for (int r = 0; r < E; r++) {
            if (r & b) continue;
            // (both registers of a pair lie in the same run)
            const uint32_t x = v[r], y = v[r | b];
            const uint64_t less = __builtin_amdgcn_ballot_w64(x < y);
            const bool x_first = __builtin_amdgcn_inverse_ballot_w64(~(less ^ ascending[r]));
            v[r] = x_first ? x : y;
            v[r | b] = x_first ? y : x;
          }
        }
      } else {
        // partner wave = wave ^ jw: everybody posts, everybody reads the partner's post
        const uint32_t jw = j / (64u * E);
        __syncthreads();
#pragma unroll
        for (int r = 0; r < E; r++) s_x[((wave * E + r) << 6) | lane] = v[r];
        __syncthreads();
        const bool lower = (wave & jw) == 0;
#pragma unroll
        for (int r = 0; r < E; r++) {
          const uint32_t other = s_x[(((wave ^ jw) * E + r) << 6) | lane];
          v[r] = keep_pair(v[r], other, lower ? ascending[r] : ~ascending[r]);
        }
      }
    }
    // the steps with the partner in another lane: distances min(k / 2, 32) down to 1
    if (k >= 64) lane_step<E, 32>(v, ascending);
    if (k >= 32) lane_step<E, 16>(v, ascending);
    if (k >= 16) lane_step<E, 8>(v, ascending);
    if (k >= 8) lane_step<E, 4>(v, ascending);
    if (k >= 4) lane_step<E, 2>(v, ascending);
    lane_step<E, 1>(v, ascending);
  }
}

// Sorts the tile's one-word keys and hands every entry to emit_list_entry, which puts runs of keys with the same
// depth field into their order by all depth bits and then emission index.  s_x: at least 64 E W 8-byte words.
template <int E, int W>
__device__ __forceinline__ void register_sort_tile(uint32_t t, uint32_t start, uint32_t n,
                                                   const TileRecord* __restrict__ records,
                                                   uint64_t* __restrict__ keys, uint32_t* __restrict__ emission,
                                                   uint32_t* __restrict__ point_list, uint64_t* s_x) {
  constexpr uint32_t M = 64u * E * W;
  constexpr int PLACE_BITS = M == 256 ? 8 : M == 512 ? 9 : M == 1024 ? 10 : 11;
  static_assert(M == 1u << PLACE_BITS, "a list of 256 to 2048 places");
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t* s_words = reinterpret_cast<uint32_t*>(s_x);
  uint32_t v[E];
  uint32_t lo = 0xFFFFFFFFu, hi = 0u;
#pragma unroll
  for (int r = 0; r < E; r++) {
    const uint32_t i = ((wave * E + r) << 6) | lane;
    v[r] = i < n ? records[start + i].z : 0u;
    if (i < n) {
      lo = v[r] < lo ? v[r] : lo;
      hi = v[r] > hi ? v[r] : hi;
    }
  }
  // smallest and largest depth bits of the list: over the wave by a scan (its last lane holds the result), over
  // the waves through LDS
  lo = ~(uint32_t)__builtin_amdgcn_readlane((int)wave_scan_max(~lo), GS_WAVE - 1);
  hi = (uint32_t)__builtin_amdgcn_readlane((int)wave_scan_max(hi), GS_WAVE - 1);
  if (lane == 0) {
    s_words[wave] = lo;
    s_words[W + wave] = hi;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < W; w++) {
    const uint32_t a = s_words[w], b = s_words[W + w];
    lo = a < lo ? a : lo;
    hi = b > hi ? b : hi;
  }
  const uint32_t range = hi - lo;  // (n >= 1, so lo <= hi)
  const int range_bits = range != 0u ? 32 - __builtin_clz(range) : 0;
  const uint32_t shift = range_bits + PLACE_BITS > 32 ? (uint32_t)(range_bits + PLACE_BITS - 32) : 0u;
#pragma unroll
  for (int r = 0; r < E; r++) {
    const uint32_t i = ((wave * E + r) << 6) | lane;
    v[r] = i < n ? ((((v[r] - lo) >> shift) << PLACE_BITS) | i) : 0xFFFFFFFFu;
  }
  // (a real key is below the padding's: a key of all ones would be the list's last place, which is padding
  // unless the list fills all M places, and then there is none)
  register_sort<E, W>(v, wave, lane, s_words);  // (starts its first exchange behind a barrier: lo and hi are read)
  uint32_t gaussian[E];
  uint64_t entry[E];
#pragma unroll
  for (int r = 0; r < E; r++) {
    const uint32_t i = ((wave * E + r) << 6) | lane;
    gaussian[r] = 0u;
    entry[r] = 0ull;
    if (i < n) {
      const TileRecord rec = records[start + (v[r] & (M - 1u))];
      gaussian[r] = rec.x;
      entry[r] = ((uint64_t)rec.z << 32) | (uint64_t)rec.y;
    }
  }
  __syncthreads();  // (the sort's last exchange between waves has been read by everybody)
#pragma unroll
  for (int r = 0; r < E; r++) {
    const uint32_t i = ((wave * E + r) << 6) | lane;
    if (i < n) s_x[i] = entry[r];
  }
  __syncthreads();
  const uint64_t* sorted = s_x;
#pragma unroll
  for (int r = 0; r < E; r++) {
    const uint32_t i = ((wave * E + r) << 6) | lane;
    if (i < n)
      emit_list_entry(t, start, n, i, gaussian[r], [&](uint32_t q) { return sorted[q]; }, keys, emission, point_list,
                      lo, shift);
  }
}

// Dynamic LDS: 8 bytes per record of the longest list the kernel takes, rounded up to a power of two (at least
// 256 records).  Lists of more than max_n records are left to the radix sort's kernels.
#define GS_SORT_CASE(EE, WW) register_sort_tile<EE, WW>(t, start, n, records, keys, emission, point_list, s_exchange)
__global__ void __launch_bounds__(512)
tile_sort_registers_kernel(const uint32_t* __restrict__ ranges, const TileRecord* __restrict__ records,
                           uint64_t* __restrict__ keys, uint32_t* __restrict__ emission,
                           uint32_t* __restrict__ point_list, uint32_t max_n,
                           const uint32_t* __restrict__ fits_word) {
  extern __shared__ uint64_t s_exchange[];
  if (fits_word != nullptr && *fits_word == 0u) return;  // launched ahead of the host's decision: see the scatter
  const uint32_t t = blockIdx.x;
  const uint32_t start = ranges[2 * t];
  const uint32_t n = ranges[2 * t + 1] - start;
  if (n == 0 || n > (uint32_t)TILE_SORT_SMALL || n > max_n) return;
  if (n <= 256) {
    if (threadIdx.x >= 256) return;  // (half the workgroup is enough; a wave that has left is not waited for)
    GS_SORT_CASE(1, 4);
  } else if (n <= 512) GS_SORT_CASE(1, 8);
  else if (n <= 1024) GS_SORT_CASE(2, 8);
  else GS_SORT_CASE(4, 8);
}
#undef GS_SORT_CASE

}  // namespace

// Tiles the LDS histograms of the counting kernels can hold.
int bucket_max_tiles() { return 30000; }

// workgroup-by-tile counts, then the tile totals, then the tile lists of the radix sort's kernels (2 T + 2 words), then
// the workgroups' sums of tiles touched and the word that says whether the view fits the buffers of kernels
// launched ahead of the host
size_t bucket_table_bytes(int T) {
  return (((size_t)BK_MAX_BLOCKS + 3) * (size_t)T + 2 + BK_MAX_BLOCKS + 1) * sizeof(uint32_t);
}
static uint32_t* bucket_block_sums(void* table, uint32_t T) {
  return (uint32_t*)table + ((size_t)BK_MAX_BLOCKS + 3) * (size_t)T + 2;
}
const uint32_t* bucket_fits_word(const void* table, int T) {
  return (const uint32_t*)table + ((size_t)BK_MAX_BLOCKS + 3) * (size_t)T + 2 + BK_MAX_BLOCKS;
}

int launch_bucket_count(int P, int W, int H, const int* radii, const float* means2D, const uint8_t* compute_locally,
                        uint32_t* tiles_touched, void* table, uint32_t* ranges, uint32_t small_limit,
                        uint32_t block_limit, uint32_t* host_words, int* zero_per_gaussian, uint32_t cap_instances,
                        uint32_t cap_longest, uint32_t* clear_word, hipStream_t stream) {
  if (P <= 0) return 0;
  if (small_limit == 0 || small_limit > (uint32_t)TILE_SORT_SMALL) small_limit = TILE_SORT_SMALL;
  // the lists one workgroup of the radix sort's smaller kernel holds; longer ones go to the larger kernel
  uint32_t mid_limit = (uint32_t)tile_radix_mid_records();
  if (block_limit != 0 && block_limit < mid_limit) mid_limit = block_limit;
  if (mid_limit < small_limit) mid_limit = small_limit;
  // ... and the lists the larger kernel holds; longer ones are split first
  uint32_t split_limit = (uint32_t)tile_radix_block_records();
  if (block_limit != 0 && block_limit < split_limit) split_limit = block_limit;
  if (split_limit < mid_limit) split_limit = mid_limit;
  const uint32_t gx = (W + GS_TILE_X - 1) / GS_TILE_X, gy = (H + GS_TILE_Y - 1) / GS_TILE_Y;
  const uint32_t T = gx * gy;
  const size_t lds = (size_t)T * (sizeof(uint32_t) + 1);
  // more than 64 KB of dynamic LDS has to be asked for, once per kernel and device (two threads that both find
  // the bit clear both ask, which is harmless)
  static std::atomic<uint64_t> raised{0};
  int dev = 0;
  GS_HIP_TRY(hipGetDevice(&dev));
  const uint64_t dev_bit = 1ull << (dev & 63);
  if (lds > 64 * 1024 && (dev >= 64 || !(raised.load(std::memory_order_acquire) & dev_bit))) {
    GS_HIP_TRY(hipFuncSetAttribute((const void*)bucket_count_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   bucket_max_tiles() * (int)(sizeof(uint32_t) + 1)));
    GS_HIP_TRY(hipFuncSetAttribute((const void*)bucket_scatter_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   bucket_max_tiles() * (int)(sizeof(uint32_t) + 1)));
    raised.fetch_or(dev_bit, std::memory_order_release);
  }
  const int nb = bucket_blocks(P), per = bucket_per_block(P);
  uint32_t* tab = (uint32_t*)table;
  uint32_t* totals = tab + (size_t)BK_MAX_BLOCKS * T;
  hipLaunchKernelGGL(bucket_count_kernel, dim3(nb), dim3(BK_THREADS), lds, stream, P, per, gx, gy, radii,
                     (const float2*)means2D, compute_locally, tiles_touched, tab, bucket_block_sums(table, T),
                     zero_per_gaussian);
  hipLaunchKernelGGL(bucket_columns_kernel, dim3((T + COL_TILES - 1) / COL_TILES), dim3(COL_TILES * COL_RUNS), 0, stream, nb, T,
                     tab, totals);
  hipLaunchKernelGGL(bucket_ranges_kernel, dim3(1), dim3(1024), 0, stream, T, small_limit, mid_limit, split_limit,
                     totals, ranges, totals + T,
                     bucket_block_sums(table, T), nb, host_words, cap_instances, cap_longest,
                     const_cast<uint32_t*>(bucket_fits_word(table, (int)T)), clear_word);
  return 0;
}

int launch_bucket_scatter(int P, int W, int H, const float* means2D, const float* depths,
                          const uint32_t* tiles_touched, uint32_t* point_offsets, const int* radii,
                          const uint8_t* compute_locally, void* table, const uint32_t* ranges, void* records,
                          bool ahead_of_host, hipStream_t stream) {
  if (P <= 0) return 0;
  const uint32_t gx = (W + GS_TILE_X - 1) / GS_TILE_X, gy = (H + GS_TILE_Y - 1) / GS_TILE_Y;
  const size_t lds = (size_t)gx * gy * (sizeof(uint32_t) + 1);
  const int vector_loads = (((uintptr_t)means2D | (uintptr_t)depths | (uintptr_t)tiles_touched |
                             (uintptr_t)point_offsets | (uintptr_t)radii) & 15u) == 0u ? 1 : 0;
  // One round per workgroup and room in the LDS for its records: they are staged and leave tile by tile.
  const size_t tiles_bytes = (size_t)gx * gy * (2 * sizeof(uint32_t) + 1);
  const size_t lds_room = 150 * 1024;
  if (bucket_per_block(P) <= BK_BATCH * BK_THREADS && tiles_bytes + 12 * 4096 <= lds_room) {
    const uint32_t cap = (uint32_t)((lds_room - tiles_bytes) / 12) & ~63u;
    const uint32_t T = gx * gy;
    const uint32_t* tab = (const uint32_t*)table;
    static std::atomic<uint64_t> raised{0};
    int dev = 0;
    GS_HIP_TRY(hipGetDevice(&dev));
    const uint64_t dev_bit = 1ull << (dev & 63);
    if (dev >= 64 || !(raised.load(std::memory_order_acquire) & dev_bit)) {
      GS_HIP_TRY(hipFuncSetAttribute((const void*)bucket_scatter_staged_kernel,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_room));
      raised.fetch_or(dev_bit, std::memory_order_release);
    }
    hipLaunchKernelGGL(bucket_scatter_staged_kernel, dim3(bucket_blocks(P)), dim3(BK_THREADS),
                       tiles_bytes + (size_t)cap * 12, stream, P, bucket_per_block(P), bucket_blocks(P), gx, gy,
                       (const float2*)means2D, depths, tiles_touched, bucket_block_sums(table, T), point_offsets, radii,
                       compute_locally, tab, tab + (size_t)BK_MAX_BLOCKS * T, ranges, (TileRecord*)records,
                       ahead_of_host ? bucket_fits_word(table, (int)T) : nullptr, vector_loads, cap);
    return 0;
  }
  hipLaunchKernelGGL(bucket_scatter_kernel, dim3(bucket_blocks(P)), dim3(BK_THREADS), lds, stream, P,
                     bucket_per_block(P), gx, gy, (const float2*)means2D, depths, tiles_touched,
                     bucket_block_sums(table, gx * gy), point_offsets, radii, compute_locally, (const uint32_t*)table,
                     ranges, (TileRecord*)records,
                     ahead_of_host ? bucket_fits_word(table, (int)(gx * gy)) : nullptr, vector_loads);
  return 0;
}

// Sorts every tile's segment of `records`.  `longest` is the longest list the launch has to be ready for and
// `radix_tiles` what the ranges kernel reported (number of lists for the radix sort's larger kernel << 16 | number
// for its smaller one; a caller that does not know passes 0xFFFFFFFF): the kernels that have nothing to do are
// not launched.  small_limit (at most TILE_SORT_SMALL) and block_limit as given to launch_bucket_count; `scratch`
// holds 24 bytes for each of the `capacity` instances the binning arrays are laid out for.
int launch_tile_sort(int T, uint32_t longest, uint32_t radix_tiles, uint32_t small_limit, uint32_t block_limit,
                     const uint32_t* ranges, const void* table, const void* records, void* scratch, int64_t capacity,
                     uint64_t* keys, uint32_t* emission, uint32_t* point_list, bool ahead_of_host,
                     hipStream_t stream) {
  if (T <= 0 || longest == 0) return 0;
  const uint32_t* fits = ahead_of_host ? bucket_fits_word(table, T) : nullptr;
  if (small_limit == 0 || small_limit > (uint32_t)TILE_SORT_SMALL) small_limit = TILE_SORT_SMALL;
  const uint32_t whole = longest < small_limit ? longest : small_limit;  // the longest list sorted in registers
  uint32_t m = 256;
  while (m < whole) m <<= 1;
  hipLaunchKernelGGL(tile_sort_registers_kernel, dim3(T), dim3(512), (size_t)m * sizeof(uint64_t), stream, ranges,
                     (const TileRecord*)records, keys, emission, point_list, small_limit, fits);
  if (longest > small_limit) {
    const uint32_t* tile_lists = (const uint32_t*)table + ((size_t)BK_MAX_BLOCKS + 1) * (size_t)T;
    // scratch: `capacity` 16-byte records for the lists that are split first, then as many 8-byte words
    uint64_t* pong = (uint64_t*)((char*)scratch + (size_t)capacity * 16);
    if (launch_tile_radix_sort(T, (radix_tiles & 0xFFFFu) != 0u, (radix_tiles >> 16) != 0u, ranges, tile_lists,
                               tile_lists + T, block_limit, records, scratch, keys, pong, keys, emission, point_list,
                               fits, stream))
      return 1;
  }
  return 0;
}

}  // namespace gs
