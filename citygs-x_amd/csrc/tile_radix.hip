// Per-tile sort of the longer lists: a stable least-significant-digit radix sort on the 32 depth bits, one
// workgroup per tile, 8-bit digits, four passes.  The counting sort by tile (tile_bucket.hip) has left every
// tile's instances in one segment of 16-byte records; what remains of the reference's sort of (tile << 32 | depth)
// keys (cuda_rasterizer/rasterizer_impl.cu:675-684) is the order by depth bits inside each segment, ties in
// emission order.
//
// A list that fits one block (THREADS x ITEMS records) never leaves the CU: the workgroup holds (depth bits << 32 |
// place in the segment) in registers, ranks the records of a pass per wave (lanes that hold the same digit find
// each other through a 64-bit lane mask per digit in LDS, a running count per wave and digit makes the rank stable),
// turns the waves' digit counts into places by one scan, moves every record to its place through LDS and reads
// its next batch back.  A longer list is sorted block by block against running digit bases, ping-ponging between
// two arrays in memory (its segment stays in the L2 of the workgroup's XCD).  The last step looks the Gaussian and
// the emission index of every sorted record up in the segment (a gather inside the tile's own records, not over
// the view's) and writes the three lists, putting runs of equal depth bits into emission order (tile_lists.h).
#include <atomic>

#include "gs_common.h"
#include "gs_kernels.h"
#include "tile_lists.h"

namespace gs {
namespace {

constexpr int TR_DIGITS = 256;
constexpr int TR_PASSES = 4;

__device__ __forceinline__ uint32_t tr_wave_inclusive_scan(uint32_t v, int lane) {
#pragma unroll
  for (int d = 1; d < GS_WAVE; d <<= 1) {
    const uint32_t o = __shfl_up(v, d, GS_WAVE);
    if (lane >= d) v += o;
  }
  return v;
}

// The workgroup's LDS, carved from one dynamic allocation.
template <int WAVES, int ITEMS>
struct TileRadixLds {
  static constexpr int THREADS = WAVES * GS_WAVE;
  static constexpr int BLOCK = THREADS * ITEMS;
  static_assert(BLOCK >= WAVES * TR_DIGITS, "the lane masks of the ranking live in the regrouping buffer");
  static_assert(ITEMS % 4 == 0, "items are ranked four at a time");
  uint64_t* rec;    // [BLOCK] regrouping buffer; during the ranking its head holds the lane masks [WAVES][256]
  uint32_t* count;  // [WAVES][256] per wave and digit: running count, then place of the wave's first such record
  uint32_t* total;  // [256] records of the block per digit
  uint32_t* first;  // [256] place in the regrouped block of the first record of a digit
  uint32_t* base;   // [4][256] blocked sort: where the next record of a digit goes in the segment, per pass
  uint32_t* scan;   // [16]
  __device__ explicit TileRadixLds(uint64_t* p) {
    rec = p;
    count = reinterpret_cast<uint32_t*>(p + BLOCK);
    total = count + WAVES * TR_DIGITS;
    first = total + TR_DIGITS;
    base = first + TR_DIGITS;
    scan = base + TR_PASSES * TR_DIGITS;
  }
  static constexpr size_t bytes() {
    return (size_t)BLOCK * 8 + (size_t)(WAVES * TR_DIGITS + 2 * TR_DIGITS + TR_PASSES * TR_DIGITS + 16) * 4;
  }
};

// One pass over one block: the `count` records (record k of a lane sits at place wave * 64 E + k * 64 + lane of
// the block, E records per lane) end up in L.rec ordered by the digit at `shift`, records of equal digit in their
// old order.  Every thread of the workgroup calls this; it starts by overwriting L.rec and ends behind a barrier.
template <int WAVES, int ITEMS>
__device__ __forceinline__ void radix_block_pass(const uint64_t (&rec)[ITEMS], uint32_t E, uint32_t count, int shift,
                                                 const TileRadixLds<WAVES, ITEMS>& L) {
  constexpr int THREADS = WAVES * GS_WAVE;
  const int tid = threadIdx.x, lane = tid & (GS_WAVE - 1), wave = tid / GS_WAVE;
  unsigned long long* s_mask = reinterpret_cast<unsigned long long*>(L.rec);
  for (int i = tid; i < WAVES * TR_DIGITS; i += THREADS) {
    s_mask[i] = 0ull;
    L.count[i] = 0u;
  }
  __syncthreads();
  // LDS operations of one wave execute in program order, which the two steps rely on; none of them waits for an
  // earlier one's result, so the items of a batch are in flight together.
  volatile unsigned long long* vmask = s_mask + wave * TR_DIGITS;
  volatile uint32_t* vcount = L.count + wave * TR_DIGITS;
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
    // Step 1: every lane ORs its bit into the mask of its digit, reads the mask back and clears it.
#pragma unroll
    for (int j = 0; j < BATCH; j++) {
      const int k = h * BATCH + j;
      const uint32_t d = (uint32_t)(rec[k] >> shift) & (TR_DIGITS - 1);
      if (valid[k]) atomicOr(&s_mask[wave * TR_DIGITS + d], lane_bit);
      __builtin_amdgcn_wave_barrier();
      same[j] = valid[k] ? vmask[d] : 0ull;
      __builtin_amdgcn_wave_barrier();
      if (valid[k]) vmask[d] = 0ull;
      __builtin_amdgcn_wave_barrier();
    }
    // Step 2: all matching lanes read the wave's running count of the digit, the lowest of them adds their number.
#pragma unroll
    for (int j = 0; j < BATCH; j++) {
      const int k = h * BATCH + j;
      const uint32_t d = (uint32_t)(rec[k] >> shift) & (TR_DIGITS - 1);
      const unsigned long long lower = same[j] & lt_mask;
      const uint32_t before = valid[k] ? vcount[d] : 0u;
      __builtin_amdgcn_wave_barrier();
      if (valid[k] && lower == 0ull) atomicAdd(&L.count[wave * TR_DIGITS + d], (uint32_t)__popcll(same[j]));
      __builtin_amdgcn_wave_barrier();
      match[k] = before + (uint32_t)__popcll(lower);
    }
  }
  __syncthreads();
  // thread d < 256: the block's records of digit d, their first place, and every wave's first place
  uint32_t tot = 0, inc = 0;
  if (tid < TR_DIGITS) {
#pragma unroll
    for (int w = 0; w < WAVES; w++) tot += L.count[w * TR_DIGITS + tid];
    inc = tr_wave_inclusive_scan(tot, lane);
    if (lane == GS_WAVE - 1) L.scan[wave] = inc;
  }
  __syncthreads();
  if (tid < TR_DIGITS) {
    uint32_t before = 0;
#pragma unroll
    for (int w = 0; w < TR_DIGITS / GS_WAVE; w++)
      if (w < wave) before += L.scan[w];
    uint32_t run = before + inc - tot;
    L.total[tid] = tot;
    L.first[tid] = run;
#pragma unroll
    for (int w = 0; w < WAVES; w++) {
      const uint32_t c = L.count[w * TR_DIGITS + tid];
      L.count[w * TR_DIGITS + tid] = run;
      run += c;
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    if (!valid[k]) continue;
    const uint32_t d = (uint32_t)(rec[k] >> shift) & (TR_DIGITS - 1);
    L.rec[L.count[wave * TR_DIGITS + d] + match[k]] = rec[k];
  }
  __syncthreads();
}

// A list of at most BLOCK records.
template <int WAVES, int ITEMS>
__device__ __forceinline__ void sort_resident(uint32_t tile, uint32_t start, uint32_t n,
                                              const TileRecord* __restrict__ records, uint64_t* __restrict__ keys,
                                              uint32_t* __restrict__ emission, uint32_t* __restrict__ point_list,
                                              const TileRadixLds<WAVES, ITEMS>& L) {
  constexpr int THREADS = WAVES * GS_WAVE;
  const int tid = threadIdx.x, lane = tid & (GS_WAVE - 1), wave = tid / GS_WAVE;
  const uint32_t E = (n + THREADS - 1) / THREADS;
  const uint32_t wave_first = (uint32_t)wave * GS_WAVE * E;
  uint64_t rec[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = wave_first + (uint32_t)k * GS_WAVE + (uint32_t)lane;
    rec[k] = ((uint32_t)k < E && i < n) ? ((uint64_t)records[start + i].z << 32) | (uint64_t)i : ~0ull;
  }
#pragma unroll 1
  for (int p = 0; p < TR_PASSES; p++) {
    radix_block_pass<WAVES, ITEMS>(rec, E, n, 32 + 8 * p, L);
    if (p + 1 < TR_PASSES) {
#pragma unroll
      for (int k = 0; k < ITEMS; k++) {
        const uint32_t i = wave_first + (uint32_t)k * GS_WAVE + (uint32_t)lane;
        if ((uint32_t)k < E && i < n) rec[k] = L.rec[i];
      }
      __syncthreads();
    }
  }
  // L.rec: (depth bits << 32 | place in the segment) in the final order but for runs of equal depth bits.  Replace
  // the place by the emission index, keep the Gaussian, and write the lists.
  uint32_t gaussian[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = (uint32_t)k * THREADS + (uint32_t)tid;
    gaussian[k] = 0u;
    if (i < n) {
      const uint64_t r = L.rec[i];
      const uint2 ge = *reinterpret_cast<const uint2*>(records + start + (uint32_t)r);
      gaussian[k] = ge.x;
      rec[k] = (r & 0xFFFFFFFF00000000ull) | (uint64_t)ge.y;
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = (uint32_t)k * THREADS + (uint32_t)tid;
    if (i < n) L.rec[i] = rec[k];
  }
  __syncthreads();
  const uint64_t* sorted = L.rec;
#pragma unroll 1
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = (uint32_t)k * THREADS + (uint32_t)tid;
    if (i < n)
      emit_list_entry(tile, start, n, i, gaussian[k], [&](uint32_t q) { return sorted[q]; }, keys, emission,
                      point_list);
  }
}

// A list of more than `blk` records (blk <= BLOCK): four passes over its blocks, from the segment's records into
// `ping`, then ping -> pong -> ping -> pong; the lists are written from pong.
template <int WAVES, int ITEMS>
__device__ __forceinline__ void sort_blocked(uint32_t tile, uint32_t start, uint32_t n, uint32_t blk,
                                             const TileRecord* __restrict__ records, uint64_t* ping, uint64_t* pong,
                                             uint64_t* __restrict__ keys, uint32_t* __restrict__ emission,
                                             uint32_t* __restrict__ point_list,
                                             const TileRadixLds<WAVES, ITEMS>& L) {
  constexpr int THREADS = WAVES * GS_WAVE;
  const int tid = threadIdx.x, lane = tid & (GS_WAVE - 1), wave = tid / GS_WAVE;
  for (int i = tid; i < TR_PASSES * TR_DIGITS; i += THREADS) L.base[i] = 0u;
  __syncthreads();
  // the digit histograms of all four passes from one read of the depth bits
  for (uint32_t i0 = 0; i0 < n; i0 += THREADS) {
    const uint32_t i = i0 + (uint32_t)tid;
    const bool valid = i < n;
    const uint32_t depth_bits = valid ? records[start + i].z : 0u;
#pragma unroll
    for (int p = 0; p < TR_PASSES; p++) {
      const uint32_t d = (depth_bits >> (8 * p)) & (TR_DIGITS - 1);
      // a digit shared by the whole wave (exponent bits) would serialise the LDS atomic 64 ways: one lane adds
      const uint64_t vm = gs_ballot(valid);
      const uint32_t d0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
      if (vm != 0ull && gs_ballot(valid && d == d0) == vm && (vm & 1ull)) {
        if (lane == 0) atomicAdd(&L.base[p * TR_DIGITS + d0], (uint32_t)__popcll(vm));
      } else if (valid) {
        atomicAdd(&L.base[p * TR_DIGITS + d], 1u);
      }
    }
  }
  __syncthreads();
#pragma unroll 1
  for (int p = 0; p < TR_PASSES; p++) {
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
  for (int p = 0; p < TR_PASSES; p++) {
    const uint64_t* src = (p & 1) ? ping : pong;  // (pass 0 reads the segment's records instead)
    uint64_t* dst = (p & 1) ? pong : ping;
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
          rec[k] = p == 0 ? ((uint64_t)records[start + b0 + i].z << 32) | (uint64_t)(b0 + i) : src[start + b0 + i];
      }
      radix_block_pass<WAVES, ITEMS>(rec, E, cnt, shift, L);
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
    // what this workgroup has written is read back by other threads of it: stores complete, then barrier, then
    // drop whatever stale lines of the two arrays the CU's vector cache holds
    __threadfence();
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  const uint64_t* sorted = pong + start;
  const TileRecord* seg = records + start;
  for (uint32_t i0 = 0; i0 < n; i0 += THREADS) {
    const uint32_t i = i0 + (uint32_t)tid;
    if (i >= n) continue;
    // (emission index of a sorted entry: through its place in the segment)
    auto entry = [&](uint32_t q) {
      const uint64_t r = sorted[q];
      return (r & 0xFFFFFFFF00000000ull) | (uint64_t)seg[(uint32_t)r].y;
    };
    // Depth bits of the neighbours decide whether the entry is part of a run; only then are emission indices of
    // other entries needed, so the neighbours are compared on the sorted array alone first.
    const uint64_t r = sorted[i];
    const uint32_t depth_bits = (uint32_t)(r >> 32);
    const bool tie = (i > 0u && (uint32_t)(sorted[i - 1u] >> 32) == depth_bits) ||
                     (i + 1u < n && (uint32_t)(sorted[i + 1u] >> 32) == depth_bits);
    const uint2 ge = *reinterpret_cast<const uint2*>(seg + (uint32_t)r);
    if (tie) {
      emit_list_entry(tile, start, n, i, ge.x, entry, keys, emission, point_list);
    } else {
      keys[start + i] = ((uint64_t)tile << 32) | (uint64_t)depth_bits;
      emission[start + i] = ge.y;
      point_list[start + i] = ge.x;
    }
  }
}

// tile_list[0 .. *list_count) (walked with `step` = +1 or -1 from `tile_list`): the tiles this kernel sorts.
template <int WAVES, int ITEMS>
__global__ void __launch_bounds__(WAVES * GS_WAVE)
tile_radix_sort_kernel(const uint32_t* __restrict__ ranges, const uint32_t* __restrict__ tile_list, int step,
                       const uint32_t* __restrict__ list_count, uint32_t count_shift, uint32_t block_limit,
                       const TileRecord* __restrict__ records, uint64_t* ping, uint64_t* pong,
                       uint64_t* __restrict__ keys, uint32_t* __restrict__ emission,
                       uint32_t* __restrict__ point_list, const uint32_t* __restrict__ fits_word) {
  extern __shared__ uint64_t s_tile_radix[];
  if (fits_word != nullptr && *fits_word == 0u) return;  // launched ahead of the host's decision: see the scatter
  const TileRadixLds<WAVES, ITEMS> L(s_tile_radix);
  const uint32_t count = (*list_count >> count_shift) & 0xFFFFu;
  uint32_t blk = block_limit < (uint32_t)TileRadixLds<WAVES, ITEMS>::BLOCK ? block_limit
                                                                           : (uint32_t)TileRadixLds<WAVES, ITEMS>::BLOCK;
  if (blk == 0u) blk = 1u;
  for (uint32_t li = blockIdx.x; li < count; li += gridDim.x) {
    const uint32_t t = tile_list[(int)li * step];
    const uint32_t start = ranges[2 * t];
    const uint32_t n = ranges[2 * t + 1] - start;
    if (n == 0u) continue;
    if (n <= blk)
      sort_resident<WAVES, ITEMS>(t, start, n, records, keys, emission, point_list, L);
    else
      sort_blocked<WAVES, ITEMS>(t, start, n, blk, records, ping, pong, keys, emission, point_list, L);
    __syncthreads();  // the next tile overwrites the LDS the last step has been reading
  }
}

}  // namespace

int tile_radix_mid_records() { return TileRadixLds<8, 8>::BLOCK; }
int tile_radix_block_records() { return TileRadixLds<16, 16>::BLOCK; }

// Sorts the tiles of the two lists the ranges kernel of the counting sort made: `mid` lists (ascending from
// tile_lists[0], their number in the low half of *counts) by workgroups of 8 waves that hold up to 4096 records,
// `long` lists (descending from tile_lists[T - 1], their number in the high half) by workgroups of 16 waves that
// hold up to 16384 records and sort longer lists in blocks of block_limit (at most 16384) records through
// `ping` (which may be `keys`) and `pong` (at least as long as the longest such list's segment end).
int launch_tile_radix_sort(int T, bool mid, bool lng, const uint32_t* ranges, const uint32_t* tile_lists,
                           const uint32_t* counts, uint32_t block_limit, const void* records, uint64_t* ping,
                           uint64_t* pong, uint64_t* keys, uint32_t* emission, uint32_t* point_list,
                           const uint32_t* fits_word, hipStream_t stream) {
  if (T <= 0) return 0;
  // more than 64 KB of dynamic LDS has to be asked for, once per device
  static std::atomic<uint64_t> raised{0};
  int dev = 0;
  GS_HIP_TRY(hipGetDevice(&dev));
  const uint64_t dev_bit = 1ull << (dev & 63);
  if (lng && (dev >= 64 || !(raised.load(std::memory_order_acquire) & dev_bit))) {
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
                       ranges, tile_lists, 1, counts, 0u, mid_block, (const TileRecord*)records, ping, pong, keys,
                       emission, point_list, fits_word);
  if (lng)
    hipLaunchKernelGGL((tile_radix_sort_kernel<16, 16>), dim3(T < 1024 ? T : 1024), dim3(16 * GS_WAVE), long_lds,
                       stream, ranges, tile_lists + (T - 1), -1, counts, 16u, block_limit, (const TileRecord*)records,
                       ping, pong, keys, emission, point_list, fits_word);
  return 0;
}

}  // namespace gs
