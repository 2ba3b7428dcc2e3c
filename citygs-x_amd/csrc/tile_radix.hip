// Per-tile sort of the longer lists: a stable least-significant-digit radix sort on the depth bits, one workgroup
// per tile.  The counting sort by tile (tile_bucket.hip) has left every tile's instances in one segment of 16-byte
// records; what remains of the reference's sort of (tile << 32 | depth) keys
// (cuda_rasterizer/rasterizer_impl.cu:675-684) is the order by depth bits inside each segment, ties in emission
// order.
//
// A list that fits one block (THREADS x ITEMS records) never leaves the CU: the workgroup holds one-word keys (the
// leading 18 bits of depth bits minus the list's smallest, over the record's place in the segment) in registers,
// ranks the keys of a pass per wave (lanes that hold the same digit find each other through a 64-bit lane mask per
// digit in LDS, a running count per wave and digit makes the rank stable), turns the waves' digit counts into
// places by one scan, moves every key to its place through LDS and reads its next batch back: two passes on 9-bit
// digits.  A longer list is first split by its leading depth bits into parts that fit; a part that still does not
// is sorted block by block on 64-bit records (depth bits << 32 | place) with 8-bit digits against running digit
// bases, ping-ponging between two arrays in memory.  The last step looks Gaussian, emission index and depth bits of
// every sorted entry up in the segment (a gather inside the tile's own records, through LDS) and writes the three
// lists, putting runs of equal depth field into their order by depth bits and emission index (tile_lists.h).
#include <atomic>

#include "gs_common.h"
#include "gs_kernels.h"
#include "tile_lists.h"

namespace gs {
namespace {

constexpr int TR_DIGITS = 256;  // digit values of the passes that go through memory and of the split by leading bits
constexpr int TR_PASSES = 4;
// Lists that one workgroup holds are sorted on one-word keys: a depth field of TR_FIELD_BITS bits over the
// record's place in the unsorted list, in two passes (or one) on digits of TR_KEY_DIGIT_BITS bits.
constexpr int TR_PLACE_BITS = 14;
constexpr int TR_FIELD_BITS = 32 - TR_PLACE_BITS;
constexpr int TR_KEY_DIGIT_BITS = 9;
constexpr int TR_KEY_DIGITS = 1 << TR_KEY_DIGIT_BITS;
static_assert(2 * TR_KEY_DIGIT_BITS == TR_FIELD_BITS, "two passes cover the depth field");

// Pointers into LDS, typed as such: through a plain pointer the volatile accesses of the ranking come out as
// flat loads and stores, which are slower and wait on the memory counters as well.
typedef __attribute__((address_space(3))) uint64_t lds_u64;
typedef __attribute__((address_space(3))) uint32_t lds_u32;
typedef __attribute__((address_space(3))) unsigned long long lds_mask;

__device__ __forceinline__ uint32_t tr_wave_inclusive_scan(uint32_t v, int lane) {
#pragma unroll
  for (int d = 1; d < GS_WAVE; d <<= 1) {
    const uint32_t o = __shfl_up(v, d, GS_WAVE);
    if (lane >= d) v += o;
  }
  return v;
}

// What one pass works in: the regrouping buffer (whose head holds the lane masks [WAVES][digits] during the
// ranking), per wave and digit the running count and then the place of the wave's first such record, per digit
// the records of the block and the place of the first, and 16 words for the scan over the digits.
template <typename RecPtr>
struct PassLds {
  RecPtr rec;
  lds_mask* mask;
  lds_u32* count;
  lds_u32* total;
  lds_u32* first;
  lds_u32* scan;
};

// The workgroup's LDS, carved from one dynamic allocation.  Two views of the leading region: `rec`, BLOCK 8-byte
// words (the passes on 64-bit records that go through memory; the last step of every sort), and for the passes on
// one-word keys `key` (BLOCK words) under the lane masks [WAVES][512] with the counts [WAVES][512] behind them.
template <int WAVES, int ITEMS>
struct TileRadixLds {
  static constexpr int THREADS = WAVES * GS_WAVE;
  static constexpr int BLOCK = THREADS * ITEMS;
  static_assert(BLOCK >= WAVES * TR_DIGITS, "the lane masks of the ranking live in the regrouping buffer");
  static_assert(BLOCK <= WAVES * TR_KEY_DIGITS * 2, "the one-word keys are regrouped under their lane masks");
  static_assert(BLOCK <= 1 << TR_PLACE_BITS, "a record's place fits the key's low bits");
  static_assert(THREADS >= TR_KEY_DIGITS, "one thread per digit in the scan");
  static_assert(ITEMS % 4 == 0, "items are ranked four at a time");
  static constexpr size_t LEAD_BYTES =
      (size_t)BLOCK * 8 > (size_t)WAVES * TR_KEY_DIGITS * 12 ? (size_t)BLOCK * 8 : (size_t)WAVES * TR_KEY_DIGITS * 12;
  lds_u64* rec;        // [BLOCK]
  lds_u32* key;        // [BLOCK], the same memory
  lds_u32* key_count;  // [WAVES][512], behind the masks of the one-word passes
  lds_u32* count;      // [WAVES][256]
  lds_u32* total;      // [512]
  lds_u32* first;      // [512]
  lds_u32* base;       // [4][256] blocked sort: where the next record of a digit goes in the segment, per pass
  lds_u32* scan;       // [16]
  lds_u32* bins;       // [257] partitioned sort: first place of every leading-digit bin in the list, then its length
  __device__ explicit TileRadixLds(lds_u64* p) {
    rec = p;
    key = (lds_u32*)p;
    key_count = (lds_u32*)p + WAVES * TR_KEY_DIGITS * 2;
    count = (lds_u32*)p + LEAD_BYTES / 4;
    total = count + WAVES * TR_DIGITS;
    first = total + TR_KEY_DIGITS;
    base = first + TR_KEY_DIGITS;
    scan = base + TR_PASSES * TR_DIGITS;
    bins = scan + 16;
  }
  static constexpr size_t bytes() {
    return LEAD_BYTES +
           (size_t)(WAVES * TR_DIGITS + 2 * TR_KEY_DIGITS + TR_PASSES * TR_DIGITS + 16 + TR_DIGITS + 4) * 4;
  }
  __device__ PassLds<lds_u64*> wide() const { return {rec, (lds_mask*)rec, count, total, first, scan}; }
  __device__ PassLds<lds_u32*> narrow() const { return {key, (lds_mask*)rec, key_count, total, first, scan}; }
};

// One pass over one block: the `count` records (record k of a lane sits at place wave * 64 E + k * 64 + lane of
// the block, E records per lane) end up in L.rec ordered by the digit at `shift`, records of equal digit in their
// old order.  Every thread of the workgroup calls this; it starts by overwriting L.rec and ends behind a barrier.
template <int WAVES, int ITEMS, int DIGIT_BITS, typename Rec, typename RecPtr>
__device__ __forceinline__ void radix_block_pass(const Rec (&rec)[ITEMS], uint32_t E, uint32_t count, int shift,
                                                 const PassLds<RecPtr>& L) {
  constexpr int THREADS = WAVES * GS_WAVE;
  constexpr int DIGITS = 1 << DIGIT_BITS;
  static_assert(THREADS >= DIGITS, "one thread per digit in the scan");
  const int tid = threadIdx.x, lane = tid & (GS_WAVE - 1), wave = tid / GS_WAVE;
  lds_mask* s_mask = L.mask;
  for (int i = tid; i < WAVES * DIGITS; i += THREADS) {
    s_mask[i] = 0ull;
    L.count[i] = 0u;
  }
  __syncthreads();
  // LDS operations of one wave execute in program order, which the two steps rely on; none of them waits for an
  // earlier one's result, so the items of a batch are in flight together.
  volatile lds_mask* vmask = s_mask + wave * DIGITS;
  volatile lds_u32* vcount = L.count + wave * DIGITS;
  const unsigned long long lane_bit = 1ull << lane;
  const unsigned long long lt_mask = lane_bit - 1ull;
  const uint32_t wave_first = (uint32_t)wave * GS_WAVE * E;
  uint32_t match[ITEMS];  // rank among the wave's records of the same digit
  bool valid[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    valid[k] = (uint32_t)k < E && wave_first + (uint32_t)k * GS_WAVE + (uint32_t)lane < count;
    match[k] = 0u;
  }
  constexpr int BATCH = 4;
#pragma unroll
  for (int h = 0; h < ITEMS / BATCH; h++) {
    if ((uint32_t)(h * BATCH) >= E) continue;  // (uniform over the workgroup)
    unsigned long long same[BATCH];
    // Step 1: the lanes that hold the same digit find each other.  A digit that many lanes share (the leading
    // bits of depths inside one tile take few values) would serialise the LDS atomic below lane after lane, so
    // up to three such digits are taken out first with one ballot each; the other lanes OR their bit into the
    // mask of their digit, read the mask back and clear it.
#pragma unroll
    for (int j = 0; j < BATCH; j++) {
      const int k = h * BATCH + j;
      const uint32_t d = (uint32_t)(rec[k] >> shift) & (DIGITS - 1);
      uint64_t rest = gs_ballot(valid[k]);
      unsigned long long mine = 0ull;
      bool placed = !valid[k];
#pragma unroll
      for (int round = 0; round < 3; round++) {
        if (rest == 0ull) break;
        const uint32_t d0 = (uint32_t)__builtin_amdgcn_readlane((int)d, (int)__builtin_ctzll(rest));
        const uint64_t m = gs_ballot(valid[k] && d == d0);
        if (__popcll(m) < 8) break;
        if (valid[k] && d == d0) {
          mine = m;
          placed = true;
        }
        rest &= ~m;
      }
      same[j] = mine;
      if (rest != 0ull) {
        if (!placed) atomicOr((unsigned long long*)&s_mask[wave * DIGITS + d], lane_bit);
        __builtin_amdgcn_wave_barrier();
        if (!placed) same[j] = vmask[d];
        __builtin_amdgcn_wave_barrier();
        if (!placed) vmask[d] = 0ull;
        __builtin_amdgcn_wave_barrier();
      }
    }
    // Step 2: all matching lanes read the wave's running count of the digit, the lowest of them adds their number.
#pragma unroll
    for (int j = 0; j < BATCH; j++) {
      const int k = h * BATCH + j;
      const uint32_t d = (uint32_t)(rec[k] >> shift) & (DIGITS - 1);
      const unsigned long long lower = same[j] & lt_mask;
      const uint32_t before = valid[k] ? vcount[d] : 0u;
      __builtin_amdgcn_wave_barrier();
      if (valid[k] && lower == 0ull)
        atomicAdd((uint32_t*)&L.count[wave * DIGITS + d], (uint32_t)__popcll(same[j]));
      __builtin_amdgcn_wave_barrier();
      match[k] = before + (uint32_t)__popcll(lower);
    }
  }
  __syncthreads();
  // thread d < 256: the block's records of digit d, their first place, and every wave's first place
  uint32_t tot = 0, inc = 0;
  if (tid < DIGITS) {
#pragma unroll
    for (int w = 0; w < WAVES; w++) tot += L.count[w * DIGITS + tid];
    inc = tr_wave_inclusive_scan(tot, lane);
    if (lane == GS_WAVE - 1) L.scan[wave] = inc;
  }
  __syncthreads();
  if (tid < DIGITS) {
    uint32_t before = 0;
#pragma unroll
    for (int w = 0; w < DIGITS / GS_WAVE; w++)
      if (w < wave) before += L.scan[w];
    uint32_t run = before + inc - tot;
    L.total[tid] = tot;
    L.first[tid] = run;
#pragma unroll
    for (int w = 0; w < WAVES; w++) {
      const uint32_t c = L.count[w * DIGITS + tid];
      L.count[w * DIGITS + tid] = run;
      run += c;
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    if (!valid[k]) continue;
    const uint32_t d = (uint32_t)(rec[k] >> shift) & (DIGITS - 1);
    L.rec[L.count[wave * DIGITS + d] + match[k]] = rec[k];
  }
  __syncthreads();
}


// Smallest and largest of the threads' values over the workgroup (every thread calls this; `lo_words` and
// `hi_words` are 16 words of LDS each, free for the duration).
template <int WAVES>
__device__ __forceinline__ void workgroup_min_max(uint32_t& lo, uint32_t& hi, lds_u32* lo_words, lds_u32* hi_words) {
  const int lane = threadIdx.x & (GS_WAVE - 1), wave = threadIdx.x / GS_WAVE;
#pragma unroll
  for (int d = GS_WAVE / 2; d >= 1; d >>= 1) {
    const uint32_t a = __shfl_xor(lo, d, GS_WAVE), b = __shfl_xor(hi, d, GS_WAVE);
    lo = a < lo ? a : lo;
    hi = b > hi ? b : hi;
  }
  if (lane == 0) {
    lo_words[wave] = lo;
    hi_words[wave] = hi;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < WAVES; w++) {
    const uint32_t a = lo_words[w], b = hi_words[w];
    lo = a < lo ? a : lo;
    hi = b > hi ? b : hi;
  }
  __syncthreads();
}

// Passes a list whose depth bits span `range` (largest minus smallest) needs: the sort runs on depth bits minus
// the smallest, whose digits above the range are all zero.  At least one, so that the pass's output exists.
__device__ __forceinline__ int passes_for_range(uint32_t range) {
  int p = 1;
  while (p < TR_PASSES && (range >> (8 * p)) != 0u) p++;
  return p;
}

// A list of at most BLOCK records, sorted inside the CU on one-word keys: the leading TR_FIELD_BITS bits of (depth
// bits - smallest of the list) over the record's place in the unsorted list, so two passes on 9-bit digits (one, if
// the list's depth bits span 9 bits or fewer) order it by the depth field with equal fields in the order of their
// places.  Where depths agree in the bits kept, the last step (emit_list_entry) orders the run by all depth bits
// and the emission index, as it does for equal depth bits; with 18 bits kept over a list's own range such runs
// stay short.
template <int WAVES, int ITEMS>
__device__ __forceinline__ void sort_resident(uint32_t tile, uint32_t start, uint32_t n,
                                              const TileRecord* __restrict__ records, uint64_t* __restrict__ keys,
                                              uint32_t* __restrict__ emission, uint32_t* __restrict__ point_list,
                                              const TileRadixLds<WAVES, ITEMS>& L) {
  constexpr int THREADS = WAVES * GS_WAVE;
  constexpr uint32_t PLACE_MASK = (1u << TR_PLACE_BITS) - 1u;
  const int tid = threadIdx.x, lane = tid & (GS_WAVE - 1), wave = tid / GS_WAVE;
  const uint32_t E = (n + THREADS - 1) / THREADS;
  const uint32_t wave_first = (uint32_t)wave * GS_WAVE * E;
  uint32_t key[ITEMS];
  uint32_t dmin = 0xFFFFFFFFu, dmax = 0u;
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = wave_first + (uint32_t)k * GS_WAVE + (uint32_t)lane;
    key[k] = 0u;
    if ((uint32_t)k < E && i < n) {
      key[k] = records[start + i].z;
      dmin = key[k] < dmin ? key[k] : dmin;
      dmax = key[k] > dmax ? key[k] : dmax;
    }
  }
  workgroup_min_max<WAVES>(dmin, dmax, L.scan, L.total);
  const uint32_t range = dmax - dmin;
  const int bits = range != 0u ? 32 - __builtin_clz(range) : 0;
  const uint32_t drop = bits > TR_FIELD_BITS ? (uint32_t)(bits - TR_FIELD_BITS) : 0u;
  const int passes = bits > TR_KEY_DIGIT_BITS ? 2 : 1;
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = wave_first + (uint32_t)k * GS_WAVE + (uint32_t)lane;
    // (keys of records that do not exist are never looked at)
    key[k] = (((key[k] - dmin) >> drop) << TR_PLACE_BITS) | (i & PLACE_MASK);
  }
  const PassLds<lds_u32*> view = L.narrow();
#pragma unroll 1
  for (int p = 0; p < passes; p++) {
    radix_block_pass<WAVES, ITEMS, TR_KEY_DIGIT_BITS>(key, E, n, TR_PLACE_BITS + TR_KEY_DIGIT_BITS * p, view);
    if (p + 1 < passes) {
#pragma unroll
      for (int k = 0; k < ITEMS; k++) {
        const uint32_t i = wave_first + (uint32_t)k * GS_WAVE + (uint32_t)lane;
        if ((uint32_t)k < E && i < n) key[k] = L.key[i];
      }
      __syncthreads();
    }
  }
  // L.key: the keys in their final order but for runs of equal depth field.  Gaussian, emission index and depth
  // bits of every entry are looked up through LDS: the sorted keys wait in registers while the list's (Gaussian,
  // emission index) pairs, and then its depth bits, are read in order into the buffer (a gather from memory, even
  // from the L2, costs as much as the passes); then the buffer takes (depth bits << 32 | emission index) in sorted
  // order for the last step.
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = (uint32_t)k * THREADS + (uint32_t)tid;
    key[k] = i < n ? L.key[i] & PLACE_MASK : 0u;  // from here on: the entry's place in the unsorted list
  }
  __syncthreads();
  uint32_t depth[ITEMS];
#pragma unroll
  for (int k0 = 0; k0 < ITEMS; k0 += 4) {
    // (four loads in flight at a time: with all of them hoisted to the front the kernel spills)
    TileRecord r[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const uint32_t i = (uint32_t)(k0 + u) * THREADS + (uint32_t)tid;
      r[u] = i < n ? records[start + i] : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const uint32_t i = (uint32_t)(k0 + u) * THREADS + (uint32_t)tid;
      if (i < n) L.rec[i] = ((uint64_t)r[u].y << 32) | (uint64_t)r[u].x;
      depth[k0 + u] = r[u].z;
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  __syncthreads();
  uint32_t gaussian[ITEMS], index[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = (uint32_t)k * THREADS + (uint32_t)tid;
    gaussian[k] = 0u;
    index[k] = 0u;
    if (i < n) {
      const uint64_t ge = L.rec[key[k]];
      gaussian[k] = (uint32_t)ge;
      index[k] = (uint32_t)(ge >> 32);
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = (uint32_t)k * THREADS + (uint32_t)tid;
    if (i < n) L.key[i] = depth[k];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = (uint32_t)k * THREADS + (uint32_t)tid;
    if (i < n) depth[k] = L.key[key[k]];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = (uint32_t)k * THREADS + (uint32_t)tid;
    if (i < n) L.rec[i] = ((uint64_t)depth[k] << 32) | (uint64_t)index[k];
  }
  __syncthreads();
  const lds_u64* sorted = L.rec;
#pragma unroll 1
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = (uint32_t)k * THREADS + (uint32_t)tid;
    if (i < n)
      emit_list_entry(tile, start, n, i, gaussian[k], [&](uint32_t q) { return sorted[q]; }, keys, emission,
                      point_list, dmin, drop);
  }
}

// A list of more than `blk` records (blk <= BLOCK): up to four passes over its blocks, the first from the segment's
// records, then between ping and pong, ending in pong; the lists are written from pong.
template <int WAVES, int ITEMS>
__device__ __forceinline__ void sort_blocked(uint32_t tile, uint32_t start, uint32_t n, uint32_t blk,
                                             const TileRecord* __restrict__ records, uint64_t* ping, uint64_t* pong,
                                             uint64_t* __restrict__ keys, uint32_t* __restrict__ emission,
                                             uint32_t* __restrict__ point_list,
                                             const TileRadixLds<WAVES, ITEMS>& L) {
  constexpr int THREADS = WAVES * GS_WAVE;
  const int tid = threadIdx.x, lane = tid & (GS_WAVE - 1), wave = tid / GS_WAVE;
  // (one workgroup has few loads in flight: every sweep over the list keeps SWEEP of them per thread going)
  constexpr int SWEEP = 8;
  uint32_t dmin = 0xFFFFFFFFu, dmax = 0u;
  for (uint32_t i0 = 0; i0 < n; i0 += THREADS * SWEEP) {
    uint32_t depth_bits[SWEEP];
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      depth_bits[u] = i < n ? records[start + i].z : dmax;
    }
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      if (i < n) {
        dmin = depth_bits[u] < dmin ? depth_bits[u] : dmin;
        dmax = depth_bits[u] > dmax ? depth_bits[u] : dmax;
      }
    }
  }
  workgroup_min_max<WAVES>(dmin, dmax, L.scan, L.total);
  const int passes = passes_for_range(dmax - dmin);
  for (int i = tid; i < TR_PASSES * TR_DIGITS; i += THREADS) L.base[i] = 0u;
  __syncthreads();
  // the digit histograms of all passes from one more read of the depth bits
  for (uint32_t i0 = 0; i0 < n; i0 += THREADS * SWEEP) {
    uint32_t depth_bits[SWEEP];
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      depth_bits[u] = i < n ? records[start + i].z : dmin;
    }
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const bool valid = i0 + (uint32_t)u * THREADS + (uint32_t)tid < n;
      const uint32_t key = depth_bits[u] - dmin;
#pragma unroll
      for (int p = 0; p < TR_PASSES; p++) {
        if (p >= passes) break;
        const uint32_t d = (key >> (8 * p)) & (TR_DIGITS - 1);
        // a digit shared by the whole wave (leading bits) would serialise the LDS atomic 64 ways: one lane adds
        const uint64_t vm = gs_ballot(valid);
        const uint32_t d0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
        if (vm != 0ull && gs_ballot(valid && d == d0) == vm && (vm & 1ull)) {
          if (lane == 0) atomicAdd((uint32_t*)&L.base[p * TR_DIGITS + d0], (uint32_t)__popcll(vm));
        } else if (valid) {
          atomicAdd((uint32_t*)&L.base[p * TR_DIGITS + d], 1u);
        }
      }
    }
  }
  __syncthreads();
#pragma unroll 1
  for (int p = 0; p < passes; p++) {
    uint32_t v = 0, inc = 0;
    if (tid < TR_DIGITS) {
      v = L.base[p * TR_DIGITS + tid];
      inc = tr_wave_inclusive_scan(v, lane);
      if (lane == GS_WAVE - 1) L.scan[wave] = inc;
    }
    __syncthreads();
    if (tid < TR_DIGITS) {
      uint32_t before = 0;
#pragma unroll
      for (int w = 0; w < TR_DIGITS / GS_WAVE; w++)
        if (w < wave) before += L.scan[w];
      L.base[p * TR_DIGITS + tid] = before + inc - v;
    }
    __syncthreads();
  }
  const uint32_t nblocks = (n + blk - 1u) / blk;
#pragma unroll 1
  for (int p = 0; p < passes; p++) {
    // the last pass writes pong (the lists, one of which may be ping itself, are written from there)
    const bool to_pong = ((passes - 1 - p) & 1) == 0;
    const uint64_t* src = to_pong ? ping : pong;  // (pass 0 reads the segment's records instead)
    uint64_t* dst = to_pong ? pong : ping;
    const int shift = 32 + 8 * p;
#pragma unroll 1
    for (uint32_t b = 0; b < nblocks; b++) {
      const uint32_t b0 = b * blk;
      const uint32_t cnt = n - b0 < blk ? n - b0 : blk;
      const uint32_t E = (cnt + THREADS - 1) / THREADS;
      const uint32_t wave_first = (uint32_t)wave * GS_WAVE * E;
      uint64_t rec[ITEMS];
#pragma unroll
      for (int k = 0; k < ITEMS; k++) {
        const uint32_t i = wave_first + (uint32_t)k * GS_WAVE + (uint32_t)lane;
        rec[k] = ~0ull;
        if ((uint32_t)k < E && i < cnt)
          rec[k] = p == 0 ? ((uint64_t)(records[start + b0 + i].z - dmin) << 32) | (uint64_t)(b0 + i)
                          : src[start + b0 + i];
      }
      radix_block_pass<WAVES, ITEMS, 8>(rec, E, cnt, shift, L.wide());
#pragma unroll
      for (int k = 0; k < ITEMS; k++) {
        const uint32_t q = (uint32_t)k * THREADS + (uint32_t)tid;
        if (q < cnt) {
          const uint64_t r = L.rec[q];
          const uint32_t d = (uint32_t)(r >> shift) & (TR_DIGITS - 1);
          dst[start + L.base[p * TR_DIGITS + d] + (q - L.first[d])] = r;
        }
      }
      __syncthreads();
      if (tid < TR_DIGITS) L.base[p * TR_DIGITS + tid] += L.total[tid];
      // (the next block's pass begins with a barrier of its own before anything reads L.base again)
    }
    // What this workgroup has written is read back by other threads of it, and by nobody else before the kernel
    // ends: the barrier's workgroup-scope release and acquire is all that takes (the waves of a workgroup share
    // their CU's vector cache; a device-scope fence here would write the whole L2's dirty lines back every time).
    __syncthreads();
  }
  const uint64_t* sorted = pong + start;
  const TileRecord* seg = records + start;
  // (emission index of a sorted entry: through its place in the segment)
  auto entry = [&](uint32_t q) {
    const uint64_t r = sorted[q];
    return ((r & 0xFFFFFFFF00000000ull) + ((uint64_t)dmin << 32)) | (uint64_t)seg[(uint32_t)r].y;
  };
  for (uint32_t i0 = 0; i0 < n; i0 += THREADS * SWEEP) {
    // Depth bits of the neighbours decide whether an entry is part of a run; only then are emission indices of
    // other entries needed, so the neighbours are compared on the sorted array alone first.
    uint64_t r[SWEEP], before[SWEEP], after[SWEEP];
    uint2 ge[SWEEP];
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      r[u] = i < n ? sorted[i] : 0ull;
      before[u] = (i < n && i > 0u) ? sorted[i - 1u] : 0ull;
      after[u] = i + 1u < n ? sorted[i + 1u] : 0ull;
    }
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      ge[u] = i < n ? *reinterpret_cast<const uint2*>(seg + (uint32_t)r[u]) : make_uint2(0u, 0u);
    }
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      if (i >= n) continue;
      const uint32_t key = (uint32_t)(r[u] >> 32);
      const bool tie = (i > 0u && (uint32_t)(before[u] >> 32) == key) || (i + 1u < n && (uint32_t)(after[u] >> 32) == key);
      if (tie) {
        emit_list_entry(tile, start, n, i, ge[u].x, entry, keys, emission, point_list);
      } else {
        keys[start + i] = ((uint64_t)tile << 32) | (uint64_t)(key + dmin);
        emission[start + i] = ge[u].y;
        point_list[start + i] = ge[u].x;
      }
    }
  }
}

// A list of more than `blk` records: split by the leading eight bits of (depth bits - smallest) into bins, moved
// bin by bin into `parted` (any order inside a bin), and runs of consecutive bins that hold at most blk records
// together are sorted like short lists, inside the CU.  A single bin beyond blk records (many instances within
// 1/256 of the list's depth range) goes block by block through memory.  Runs of equal depth bits never straddle
// two bins, so the last step of the sorts still sees them whole.
template <int WAVES, int ITEMS>
__device__ __forceinline__ void sort_partitioned(uint32_t tile, uint32_t start, uint32_t n, uint32_t blk,
                                                 const TileRecord* __restrict__ records, TileRecord* parted,
                                                 uint64_t* ping, uint64_t* pong, uint64_t* keys, uint32_t* emission,
                                                 uint32_t* point_list, const TileRadixLds<WAVES, ITEMS>& L) {
  constexpr int THREADS = WAVES * GS_WAVE;
  constexpr int SWEEP = 8;  // loads a thread keeps in flight in every sweep over the list
  const int tid = threadIdx.x, lane = tid & (GS_WAVE - 1), wave = tid / GS_WAVE;
  uint32_t dmin = 0xFFFFFFFFu, dmax = 0u;
  for (uint32_t i0 = 0; i0 < n; i0 += THREADS * SWEEP) {
    uint32_t depth_bits[SWEEP];
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      depth_bits[u] = i < n ? records[start + i].z : dmax;
    }
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      if (i < n) {
        dmin = depth_bits[u] < dmin ? depth_bits[u] : dmin;
        dmax = depth_bits[u] > dmax ? depth_bits[u] : dmax;
      }
    }
  }
  workgroup_min_max<WAVES>(dmin, dmax, L.scan, L.total);
  const uint32_t range = dmax - dmin;
  const int bits = range != 0u ? 32 - __builtin_clz(range) : 0;
  const int shift = bits > 8 ? bits - 8 : 0;
  for (int i = tid; i <= TR_DIGITS; i += THREADS) L.bins[i] = 0u;
  __syncthreads();
  for (uint32_t i0 = 0; i0 < n; i0 += THREADS * SWEEP) {
    uint32_t depth_bits[SWEEP];
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      depth_bits[u] = i < n ? records[start + i].z : dmin;
    }
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const bool valid = i0 + (uint32_t)u * THREADS + (uint32_t)tid < n;
      const uint32_t d = (depth_bits[u] - dmin) >> shift;
      // a digit shared by the whole wave would serialise the LDS atomic 64 ways: one lane adds
      const uint64_t vm = gs_ballot(valid);
      const uint32_t d0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
      if (vm != 0ull && gs_ballot(valid && d == d0) == vm && (vm & 1ull)) {
        if (lane == 0) atomicAdd((uint32_t*)&L.bins[d0], (uint32_t)__popcll(vm));
      } else if (valid) {
        atomicAdd((uint32_t*)&L.bins[d], 1u);
      }
    }
  }
  __syncthreads();
  {
    uint32_t v = 0, inc = 0;
    if (tid < TR_DIGITS) {
      v = L.bins[tid];
      inc = tr_wave_inclusive_scan(v, lane);
      if (lane == GS_WAVE - 1) L.scan[wave] = inc;
    }
    __syncthreads();
    if (tid < TR_DIGITS) {
      uint32_t before = 0;
#pragma unroll
      for (int w = 0; w < TR_DIGITS / GS_WAVE; w++)
        if (w < wave) before += L.scan[w];
      L.bins[tid] = before + inc - v;
      L.first[tid] = before + inc - v;  // where the bin's next record goes
      if (tid == TR_DIGITS - 1) L.bins[TR_DIGITS] = before + inc;
    }
    __syncthreads();
  }
  for (uint32_t i0 = 0; i0 < n; i0 += THREADS * SWEEP) {
    TileRecord r[SWEEP];
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      r[u] = i < n ? records[start + i] : make_uint4(0u, 0u, dmin, 0u);
    }
#pragma unroll
    for (int u = 0; u < SWEEP; u++) {
      const uint32_t i = i0 + (uint32_t)u * THREADS + (uint32_t)tid;
      if (i < n) parted[start + atomicAdd((uint32_t*)&L.first[(r[u].z - dmin) >> shift], 1u)] = r[u];
    }
  }
  __syncthreads();  // (the moved records are read back by this workgroup only: see sort_blocked)
  uint32_t g0 = 0;
  while (g0 < (uint32_t)TR_DIGITS) {
    const uint32_t first = L.bins[g0];
    uint32_t g1 = g0 + 1u;
    while (g1 < (uint32_t)TR_DIGITS && L.bins[g1 + 1u] - first <= blk) g1++;
    const uint32_t cnt = (uint32_t)__builtin_amdgcn_readfirstlane((int)(L.bins[g1] - first));
    g0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)g1);
    if (cnt == 0u) continue;
    if (cnt <= blk)
      sort_resident<WAVES, ITEMS>(tile, start + first, cnt, parted, keys, emission, point_list, L);
    else
      sort_blocked<WAVES, ITEMS>(tile, start + first, cnt, blk, parted, ping, pong, keys, emission, point_list, L);
    __syncthreads();
  }
}

// tile_list[0 .. *list_count) (walked with `step` = +1 or -1 from `tile_list`): the tiles this kernel sorts.  The
// lists that are split before they are sorted (more than block_limit records; the larger kernel only) are also
// entered in a list of their own, list_count[1] tiles from list_count + 2.  Such a list takes several times as long
// as the others, a CU holds one workgroup, and workgroups start in the order of their numbers: while there are
// fewer of them than CUs, they are taken first, so that the long jobs start at once and the short ones fill the
// gaps behind them (a view with 54 such lists among 900: 292 -> 250 us).  With more of them than CUs the tiles'
// own order, a mix of both kinds, is kept: all long jobs first then sweep their lists at the same time, bound by
// memory in that phase and idle in the next (3 % slower), and any order that starts some of them late is worse.
template <int WAVES, int ITEMS>
__global__ void __launch_bounds__(WAVES * GS_WAVE)
tile_radix_sort_kernel(const uint32_t* __restrict__ ranges, const uint32_t* __restrict__ tile_list, int step,
                       const uint32_t* __restrict__ list_count, uint32_t count_shift, uint32_t block_limit,
                       const TileRecord* __restrict__ records, TileRecord* parted, uint64_t* ping, uint64_t* pong,
                       uint64_t* keys, uint32_t* emission, uint32_t* point_list,
                       const uint32_t* __restrict__ fits_word) {
  extern __shared__ uint64_t s_tile_radix[];
  if (fits_word != nullptr && *fits_word == 0u) return;  // launched ahead of the host's decision: see the scatter
  const TileRadixLds<WAVES, ITEMS> L((lds_u64*)s_tile_radix);
  const uint32_t split = (WAVES == 16 && list_count[1] <= 256u) ? list_count[1] : 0u;  // taken first
  const uint32_t count = ((*list_count >> count_shift) & 0xFFFFu) + split;
  uint32_t blk = block_limit < (uint32_t)TileRadixLds<WAVES, ITEMS>::BLOCK ? block_limit
                                                                           : (uint32_t)TileRadixLds<WAVES, ITEMS>::BLOCK;
  if (blk == 0u) blk = 1u;
  for (uint32_t li = blockIdx.x; li < count; li += gridDim.x) {
    const uint32_t t = li < split ? list_count[2u + li] : tile_list[(int)(li - split) * step];
    const uint32_t start = ranges[2 * t];
    const uint32_t n = ranges[2 * t + 1] - start;
    if (n == 0u || (li >= split && split != 0u && n > blk)) continue;  // (the latter: done as one of the first)
    if (n <= blk)
      sort_resident<WAVES, ITEMS>(t, start, n, records, keys, emission, point_list, L);
    else if constexpr (WAVES == 16)
      sort_partitioned<WAVES, ITEMS>(t, start, n, blk, records, parted, ping, pong, keys, emission, point_list, L);
    __syncthreads();  // the next tile overwrites the LDS the last step has been reading
  }
}

}  // namespace

int tile_radix_mid_records() { return TileRadixLds<8, 8>::BLOCK; }
int tile_radix_block_records() { return TileRadixLds<16, 16>::BLOCK; }

// Sorts the tiles of the two lists the ranges kernel of the counting sort made: `mid` lists (ascending from
// tile_lists[0], their number in the low half of *counts) by workgroups of 8 waves that hold up to 4096 records,
// `long` lists (descending from tile_lists[T - 1], their number in the high half) by workgroups of 16 waves that
// hold up to 16384 records; a longer list (or one beyond block_limit records, at most 16384) is first split by its
// leading depth bits into `parted` (16 bytes per instance), and a part that is still too long goes block by block
// through `ping` (which may be `keys`) and `pong` (8 bytes per instance each).
int launch_tile_radix_sort(int T, bool mid, bool lng, const uint32_t* ranges, const uint32_t* tile_lists,
                           const uint32_t* counts, uint32_t block_limit, const void* records, void* parted,
                           uint64_t* ping, uint64_t* pong, uint64_t* keys, uint32_t* emission, uint32_t* point_list,
                           const uint32_t* fits_word, hipStream_t stream) {
  if (T <= 0) return 0;
  // more than 64 KB of dynamic LDS has to be asked for, once per device
  static std::atomic<uint64_t> raised{0};
  int dev = 0;
  GS_HIP_TRY(hipGetDevice(&dev));
  const uint64_t dev_bit = 1ull << (dev & 63);
  if ((mid || lng) && (dev >= 64 || !(raised.load(std::memory_order_acquire) & dev_bit))) {
    GS_HIP_TRY(hipFuncSetAttribute((const void*)tile_radix_sort_kernel<8, 8>,
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)TileRadixLds<8, 8>::bytes()));
    GS_HIP_TRY(hipFuncSetAttribute((const void*)tile_radix_sort_kernel<16, 16>,
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)TileRadixLds<16, 16>::bytes()));
    raised.fetch_or(dev_bit, std::memory_order_release);
  }
  if (block_limit == 0u || block_limit > (uint32_t)TileRadixLds<16, 16>::BLOCK)
    block_limit = TileRadixLds<16, 16>::BLOCK;
  using Mid = TileRadixLds<8, 8>;
  using Long = TileRadixLds<16, 16>;
  const size_t mid_lds = Mid::bytes(), long_lds = Long::bytes();
  const uint32_t mid_block = Mid::BLOCK;
  if (mid)
    hipLaunchKernelGGL((tile_radix_sort_kernel<8, 8>), dim3(T < 2048 ? T : 2048), dim3(8 * GS_WAVE), mid_lds, stream,
                       ranges, tile_lists, 1, counts, 0u, mid_block, (const TileRecord*)records, (TileRecord*)parted,
                       ping, pong, keys, emission, point_list, fits_word);
  if (lng)
    hipLaunchKernelGGL((tile_radix_sort_kernel<16, 16>), dim3(T < 1024 ? T : 1024), dim3(16 * GS_WAVE), long_lds,
                       stream, ranges, tile_lists + (T - 1), -1, counts, 16u, block_limit, (const TileRecord*)records,
                       (TileRecord*)parted, ping, pong, keys, emission, point_list, fits_word);
  return 0;
}

}  // namespace gs
