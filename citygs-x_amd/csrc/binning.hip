// Tile binning: per-Gaussian tile counts, uint32 prefix sum, (tile|depth) key
// emission and per-tile range detection
// (cuda_rasterizer/rasterizer_impl.cu:74-144, :264-288, :633-697).
// All of it is integer / bit work and must match a CPU bit for bit.
#include <mutex>

#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

constexpr int SCAN_THREADS = 256;
constexpr int SCAN_ITEMS = 8;
constexpr int SCAN_TILE = SCAN_THREADS * SCAN_ITEMS;

__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
  const int lane = threadIdx.x & (GS_WAVE - 1);
#pragma unroll
  for (int d = 1; d < GS_WAVE; d <<= 1) {
    const uint32_t o = __shfl_up(v, d, GS_WAVE);
    if (lane >= d) v += o;
  }
  return v;
}

// Exclusive prefix of v across the block plus the block total.
template <int THREADS>
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* s_wave /*THREADS/64 + 1*/,
                                                         uint32_t& total) {
  constexpr int NW = THREADS / GS_WAVE;
  const int lane = threadIdx.x & (GS_WAVE - 1), wave = threadIdx.x / GS_WAVE;
  const uint32_t inc = wave_inclusive_scan(v);
  if (lane == GS_WAVE - 1) s_wave[wave] = inc;
  __syncthreads();
  uint32_t base = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < NW; w++) {
    const uint32_t s = s_wave[w];
    if (w < wave) base += s;
    tot += s;
  }
  __syncthreads();
  total = tot;
  return base + inc - v;
}

// cuda_rasterizer/rasterizer_impl.cu:264-288.
__global__ void __launch_bounds__(GS_BLOCK_1D)
tile_count_kernel(int P, uint32_t gx, uint32_t gy, const int* __restrict__ radii,
                  const float2* __restrict__ means2D, const uint8_t* __restrict__ compute_locally,
                  uint32_t* __restrict__ tiles_touched, uint32_t* __restrict__ zero_words, int64_t zero_count,
                  int* __restrict__ zero_per_gaussian) {
  const int i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  // optionally clears another array on the side (the tile ranges of the same call: saves a launch)
  for (int64_t j = i; j < zero_count; j += (int64_t)gridDim.x * GS_BLOCK_1D) zero_words[j] = 0u;
  // (no early return: the walk below is a wave-wide operation)
  const bool live = i < P && radii[i] > 0;
  Rect rc = {0u, 0u, 0u, 0u};
  if (live) {
    const float2 p = means2D[i];
    rc = get_rect(p.x, p.y, radii[i], gx, gy);
  }
  struct None { uint32_t unused; } none = {0u};
  const uint32_t cnt = walk_wave_rects(
      live, rc, gx, none, [&](uint32_t tile) { return compute_locally[tile] != 0; },
      [](const None&, uint32_t, uint32_t) {});
  if (i < P) {
    tiles_touched[i] = cnt;
    if (zero_per_gaussian != nullptr) zero_per_gaussian[i] = 0;
  }
}

template <typename T>
__global__ void __launch_bounds__(SCAN_THREADS)
scan_block_sums_kernel(int64_t n, const T* __restrict__ in, uint32_t* __restrict__ block_sums) {
  __shared__ uint32_t s_wave[SCAN_THREADS / GS_WAVE];
  const int64_t base = (int64_t)blockIdx.x * SCAN_TILE;
  uint32_t s = 0;
#pragma unroll
  for (int k = 0; k < SCAN_ITEMS; k++) {
    const int64_t idx = base + (int64_t)k * SCAN_THREADS + threadIdx.x;
    if (idx < n) s += in[idx];
  }
#pragma unroll
  for (int d = GS_WAVE / 2; d >= 1; d >>= 1) s += __shfl_xor(s, d, GS_WAVE);
  if ((threadIdx.x & (GS_WAVE - 1)) == 0) s_wave[threadIdx.x / GS_WAVE] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t t = 0;
    for (int w = 0; w < SCAN_THREADS / GS_WAVE; w++) t += s_wave[w];
    block_sums[blockIdx.x] = t;
  }
}

// One block turns the per-tile sums into exclusive prefixes in place.
// block_sums[nblocks] receives 1 if the exact grand total exceeds GS_MAX_INSTANCES (the 32-bit sums wrap
// around), else 0.  A block's own sum is taken as exact: it covers SCAN_TILE elements.
__global__ void __launch_bounds__(1024) scan_spine_kernel(int nblocks, uint32_t* __restrict__ block_sums) {
  __shared__ uint32_t s_wave[1024 / GS_WAVE];
  __shared__ double s_exact[1024 / GS_WAVE];
  uint32_t carry = 0;
  double exact = 0.0;
  for (int start = 0; start < nblocks; start += 1024) {
    const int idx = start + threadIdx.x;
    const uint32_t v = idx < nblocks ? block_sums[idx] : 0u;
    exact += (double)v;
    uint32_t total;
    const uint32_t ex = block_exclusive_scan<1024>(v, s_wave, total);
    if (idx < nblocks) block_sums[idx] = carry + ex;
    carry += total;
  }
#pragma unroll
  for (int d = GS_WAVE / 2; d >= 1; d >>= 1) exact += __shfl_xor(exact, d, GS_WAVE);
  if ((threadIdx.x & (GS_WAVE - 1)) == 0) s_exact[threadIdx.x / GS_WAVE] = exact;
  __syncthreads();
  if (threadIdx.x == 0) {
    double all = 0.0;
    for (int w = 0; w < 1024 / GS_WAVE; w++) all += s_exact[w];
    block_sums[nblocks] = all > (double)GS_MAX_INSTANCES ? 1u : 0u;
  }
}

template <bool EXCLUSIVE, typename T>
__global__ void __launch_bounds__(SCAN_THREADS)
scan_apply_kernel(int64_t n, const T* in, const uint32_t* __restrict__ block_prefix, uint32_t* out,
                  uint32_t* total_out) {
  // in and out may be the same array: each thread reads its items before it writes them.
  __shared__ uint32_t s_wave[SCAN_THREADS / GS_WAVE];
  // Blocked arrangement: thread t owns SCAN_ITEMS consecutive elements.
  const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
  uint32_t v[SCAN_ITEMS];
  uint32_t s = 0;
#pragma unroll
  for (int k = 0; k < SCAN_ITEMS; k++) {
    v[k] = (base + k < n) ? in[base + k] : 0u;
    s += v[k];
  }
  uint32_t total;
  uint32_t run = block_prefix[blockIdx.x] + block_exclusive_scan<SCAN_THREADS>(s, s_wave, total);
#pragma unroll
  for (int k = 0; k < SCAN_ITEMS; k++) {
    if (EXCLUSIVE) {
      if (base + k < n) out[base + k] = run;
      run += v[k];
    } else {
      run += v[k];
      if (base + k < n) out[base + k] = run;
    }
  }
  // The owner of the last element also hands the grand total to the host, which may be polling this word
  // (host-visible memory), so the store is made visible system wide.
  if (total_out != nullptr && n - 1 >= base && n - 1 < base + SCAN_ITEMS)
    __hip_atomic_store(total_out, block_prefix[gridDim.x] != 0u ? GS_TOO_MANY_INSTANCES : run, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
}

// cuda_rasterizer/rasterizer_impl.cu:74-117.
__global__ void __launch_bounds__(GS_BLOCK_1D)
duplicate_with_keys_kernel(int P, uint32_t gx, uint32_t gy, const float2* __restrict__ means2D,
                           const float* __restrict__ depths, const uint32_t* __restrict__ offsets,
                           const int* __restrict__ radii, const uint8_t* __restrict__ compute_locally,
                           uint64_t* __restrict__ keys, uint32_t* __restrict__ values,
                           uint32_t* __restrict__ emission) {
  const int i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  const bool live = i < P && radii[i] > 0;
  Rect rc = {0u, 0u, 0u, 0u};
  struct Owner { uint32_t first, depth_bits, id; } mine = {0u, 0u, (uint32_t)i};
  if (live) {
    mine.first = (i == 0) ? 0u : offsets[i - 1];
    const float2 p = means2D[i];
    rc = get_rect(p.x, p.y, radii[i], gx, gy);
    mine.depth_bits = __float_as_uint(depths[i]);
  }
  walk_wave_rects(
      live, rc, gx, mine, [&](uint32_t tile) { return compute_locally[tile] != 0; },
      [&](const Owner& o, uint32_t tile, uint32_t rank) {
        const uint32_t e = o.first + rank;
        keys[e] = ((uint64_t)tile << 32) | (uint64_t)o.depth_bits;
        values[e] = o.id;
        if (emission) emission[e] = e;  // position in emission order, carried through the sort
      });
}

// point_list[k] = Gaussian of the instance that the sort moved to position k.
__global__ void __launch_bounds__(GS_BLOCK_1D)
gather_u32_kernel(int64_t n, const uint32_t* __restrict__ index, const uint32_t* __restrict__ table,
                  uint32_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (i < n) out[i] = table[index[i]];
}

// One thread per Gaussian; only visible Gaussians (radius > 0) are read and written: no tile lists the others.  A
// wave whose 64 Gaussians are all visible passes its records (4 KB, contiguous) through LDS so that every store
// instruction writes one contiguous kilobyte: lane l stores 16-byte word (l & 3) of record 16 k + (l >> 2) in
// round k.  (In LDS a record's four words sit 1040 bytes apart, so that neither the writes, record-major, nor the
// reads, word-minor, pile up on a few banks.)  In any other wave a visible lane stores its own record, four
// 16-byte stores that fill one 64-byte line.
__global__ void __launch_bounds__(GS_BLOCK_1D)
pack_blend_operands_kernel(int P, const int* __restrict__ radii, const float2* __restrict__ means2D,
                           const float4* __restrict__ conic_opacity, const float* __restrict__ rgb,
                           const float* __restrict__ all_map, const float* __restrict__ depths,
                           float4* __restrict__ packed, uint32_t* __restrict__ valid_word) {
  if (valid_word != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *valid_word = 1u;
  constexpr int WORD_STRIDE = GS_WAVE + 1;  // in 16-byte units
  __shared__ float4 s_rec[GS_BLOCK_1D / GS_WAVE][4 * WORD_STRIDE];
  const int lane = threadIdx.x & (GS_WAVE - 1), wave = threadIdx.x / GS_WAVE;
  const int i = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  const bool live = i < P && radii[i] > 0;
  const uint64_t live_m = gs_ballot(live);
  if (live_m == 0ull) return;
  float4 w0 = make_float4(0.f, 0.f, 0.f, 0.f), w1 = w0, w2 = w0, w3 = w0;
  if (live) {
    const float2 xy = means2D[i];
    const float4 co = conic_opacity[i];
    const float c0 = rgb[3 * (size_t)i], c1 = rgb[3 * (size_t)i + 1], c2 = rgb[3 * (size_t)i + 2];
    float m[5] = {0.f, 0.f, 0.f, 0.f, 0.f};
    if (all_map != nullptr) {
#pragma unroll
      for (int ch = 0; ch < 5; ch++) m[ch] = all_map[5 * (size_t)i + ch];
    }
    const float d = depths != nullptr ? depths[i] : 0.f;
    w0 = make_float4(xy.x, xy.y, co.x, co.y);
    w1 = make_float4(co.z, co.w, c0, c1);
    w2 = make_float4(c2, m[0], m[1], m[2]);
    w3 = make_float4(m[3], m[4], d, 0.f);
  }
  // (a wave with a few invisible Gaussians still takes the contiguous route: their records are zeros)
  if (__popcll(live_m) < 48) {
    if (live) {
      float4* rec = packed + 4 * (size_t)i;
      rec[0] = w0; rec[1] = w1; rec[2] = w2; rec[3] = w3;
    }
    return;
  }
  float4* mine = &s_rec[wave][0];
  mine[0 * WORD_STRIDE + lane] = w0;
  mine[1 * WORD_STRIDE + lane] = w1;
  mine[2 * WORD_STRIDE + lane] = w2;
  mine[3 * WORD_STRIDE + lane] = w3;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  float4* out = packed + 4 * (size_t)(blockIdx.x * GS_BLOCK_1D + wave * GS_WAVE);  // the wave's first record
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const int rec = 16 * k + (lane >> 2);
    if (blockIdx.x * GS_BLOCK_1D + wave * GS_WAVE + rec < P) out[64 * k + lane] = mine[(lane & 3) * WORD_STRIDE + rec];
  }
}

__global__ void fill_u32_kernel(int64_t n, uint32_t v, uint32_t* __restrict__ p) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// cuda_rasterizer/rasterizer_impl.cu:122-144.
__global__ void __launch_bounds__(GS_BLOCK_1D)
tile_ranges_kernel(int64_t L, const uint64_t* __restrict__ keys, uint32_t* __restrict__ ranges,
                   const uint32_t* __restrict__ gather_index, const uint32_t* __restrict__ gather_table,
                   uint32_t* __restrict__ gather_out, const uint32_t* __restrict__ sort_error,
                   uint32_t* __restrict__ fault_word) {
  const int64_t i = (int64_t)blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (i >= L) return;
  // a sort that gave up waiting for an earlier tile's counts left its error word set: tell the host (sticky word
  // in host-visible memory), which looks at it at its next call
  if (i == 0 && sort_error != nullptr && fault_word != nullptr && *sort_error != 0u)
    __hip_atomic_store(fault_word, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  // optionally also: gather_out[i] = gather_table[gather_index[i]] (the sorted list of Gaussian ids)
  if (gather_out != nullptr) gather_out[i] = gather_table[gather_index[i]];
  const uint32_t cur = (uint32_t)(keys[i] >> 32);
  if (i == 0)
    ranges[2 * cur] = 0;
  else {
    const uint32_t prev = (uint32_t)(keys[i - 1] >> 32);
    if (cur != prev) {
      ranges[2 * prev + 1] = (uint32_t)i;
      ranges[2 * cur] = (uint32_t)i;
    }
  }
  if (i == L - 1) ranges[2 * cur + 1] = (uint32_t)L;
}

}  // namespace

int launch_tile_count(int P, int W, int H, const int* radii, const float* means2D, const uint8_t* compute_locally,
                      uint32_t* tiles_touched, hipStream_t stream, uint32_t* zero_words, int64_t zero_count,
                      int* zero_per_gaussian) {
  if (P <= 0) return 0;
  const uint32_t gx = (W + GS_TILE_X - 1) / GS_TILE_X, gy = (H + GS_TILE_Y - 1) / GS_TILE_Y;
  hipLaunchKernelGGL(tile_count_kernel, dim3((P + GS_BLOCK_1D - 1) / GS_BLOCK_1D), dim3(GS_BLOCK_1D), 0, stream, P,
                     gx, gy, radii, (const float2*)means2D, compute_locally, tiles_touched, zero_words,
                     zero_words ? zero_count : 0, zero_per_gaussian);
  return 0;
}

size_t scan_temp_bytes(int64_t n) {
  const int64_t nb = (n + SCAN_TILE - 1) / SCAN_TILE;
  return align_up((size_t)((nb > 0 ? nb : 1) + 1) * sizeof(uint32_t), 256);  // block sums and the overflow word
}

const uint32_t* scan_overflow_word(const void* temp, int64_t n) {
  const int64_t nb = (n + SCAN_TILE - 1) / SCAN_TILE;
  return (const uint32_t*)temp + (nb > 0 ? nb : 1);
}

template <typename T>
static int scan_impl(int64_t n, const T* in, uint32_t* out, void* temp, bool exclusive, uint32_t* total_out,
                     hipStream_t stream) {
  if (n <= 0) return 0;
  const int nb = (int)((n + SCAN_TILE - 1) / SCAN_TILE);
  uint32_t* sums = (uint32_t*)temp;
  hipLaunchKernelGGL(scan_block_sums_kernel<T>, dim3(nb), dim3(SCAN_THREADS), 0, stream, n, in, sums);
  hipLaunchKernelGGL(scan_spine_kernel, dim3(1), dim3(1024), 0, stream, nb, sums);
  if (exclusive)
    hipLaunchKernelGGL((scan_apply_kernel<true, T>), dim3(nb), dim3(SCAN_THREADS), 0, stream, n, in, sums, out, total_out);
  else
    hipLaunchKernelGGL((scan_apply_kernel<false, T>), dim3(nb), dim3(SCAN_THREADS), 0, stream, n, in, sums, out, total_out);
  return 0;
}

// in and out may alias.
int launch_inclusive_sum(int64_t n, const uint32_t* in, uint32_t* out, void* temp, hipStream_t stream,
                         uint32_t* total_out) {
  return scan_impl(n, in, out, temp, false, total_out, stream);
}

int launch_exclusive_sum(int64_t n, const uint32_t* in, uint32_t* out, void* temp, hipStream_t stream) {
  return scan_impl(n, in, out, temp, true, nullptr, stream);
}

// ---- inclusive sum whose spine lives in a static device array (for callers that must not allocate) ----
// The array is part of the code object: every GPU the library runs on holds its own copy, at its own address,
// until the process ends.  Host code never passes the array's name to a kernel (there it is a host-side
// stand-in, not a device address): the device address is looked up once per device with hipGetSymbolAddress
// and kept in g_static_spine[device].
constexpr int64_t STATIC_SCAN_MAX = (int64_t)1 << 27;  // elements
constexpr size_t STATIC_SPINE_WORDS = (size_t)(STATIC_SCAN_MAX / SCAN_TILE) + 1;  // block sums + overflow word
static __device__ __align__(256) uint32_t scratch[STATIC_SPINE_WORDS];

namespace {
constexpr int STATIC_MAX_DEVICES = 64;
std::mutex g_static_mutex;
uint32_t* g_static_spine[STATIC_MAX_DEVICES] = {};
}  // namespace

int64_t static_scan_max_elements() { return STATIC_SCAN_MAX; }

// Device address of the current device's copy of the array (looked up on the first call per device).
static int static_spine(uint32_t** out) {
  int dev = -1;
  GS_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= STATIC_MAX_DEVICES) {
    set_error("gs_inclusive_sum_static: device ordinal %d outside the supported range [0, %d)", dev,
              STATIC_MAX_DEVICES);
    return 1;
  }
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (g_static_spine[dev] == nullptr) {
    uint32_t* p = nullptr;
    GS_HIP_TRY(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
    if (p == nullptr) {
      set_error("gs_inclusive_sum_static: hipGetSymbolAddress returned a null address");
      return 1;
    }
    g_static_spine[dev] = p;
  }
  *out = g_static_spine[dev];
  return 0;
}

// The scan of launch_inclusive_sum with the spine in the static array.  Every word of the spine that a call
// reads is written by the same call first (block sums by the first kernel, the overflow word by the second),
// so nothing has to be cleared; calls that overlap on one GPU race on the array.
int launch_inclusive_sum_static(int64_t n, const uint32_t* in, uint32_t* out, hipStream_t stream) {
  if (n <= 0) return 0;
  if (n > STATIC_SCAN_MAX) {
    set_error("gs_inclusive_sum_static: n = %lld exceeds the static scratch array's capacity of %lld elements",
              (long long)n, (long long)STATIC_SCAN_MAX);
    return 1;
  }
  uint32_t* spine = nullptr;
  if (static_spine(&spine)) return 1;
  return scan_impl(n, in, out, spine, false, nullptr, stream);
}

// exclusive prefix sums of small counts (a 0/1 mask gives the ranks of its set bytes)
int launch_exclusive_sum_u8(int64_t n, const uint8_t* in, uint32_t* out, void* temp, hipStream_t stream,
                            uint32_t* total_out) {
  return scan_impl(n, in, out, temp, true, total_out, stream);
}

int launch_duplicate_with_keys(int P, int W, int H, const float* means2D, const float* depths,
                               const uint32_t* offsets, const int* radii, const uint8_t* compute_locally,
                               uint64_t* keys, uint32_t* values, uint32_t* emission, hipStream_t stream) {
  if (P <= 0) return 0;
  const uint32_t gx = (W + GS_TILE_X - 1) / GS_TILE_X, gy = (H + GS_TILE_Y - 1) / GS_TILE_Y;
  hipLaunchKernelGGL(duplicate_with_keys_kernel, dim3((P + GS_BLOCK_1D - 1) / GS_BLOCK_1D), dim3(GS_BLOCK_1D), 0,
                     stream, P, gx, gy, (const float2*)means2D, depths, offsets, radii, compute_locally, keys, values,
                     emission);
  return 0;
}

int launch_pack_blend_operands(int P, const int* radii, const float* means2D, const float* conic_opacity,
                               const float* rgb, const float* all_map, const float* depths, float* packed,
                               uint32_t* valid_word, hipStream_t stream) {
  if (P <= 0) return 0;
  hipLaunchKernelGGL(pack_blend_operands_kernel, dim3((P + GS_BLOCK_1D - 1) / GS_BLOCK_1D), dim3(GS_BLOCK_1D), 0,
                     stream, P, radii, (const float2*)means2D, (const float4*)conic_opacity, rgb, all_map, depths,
                     (float4*)packed, valid_word);
  return 0;
}

int launch_fill_u32(int64_t n, uint32_t value, uint32_t* p, hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, n, value, p);
  return 0;
}

int launch_gather_u32(int64_t n, const uint32_t* index, const uint32_t* table, uint32_t* out, hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(gather_u32_kernel, dim3((unsigned)((n + GS_BLOCK_1D - 1) / GS_BLOCK_1D)), dim3(GS_BLOCK_1D), 0,
                     stream, n, index, table, out);
  return 0;
}

int launch_tile_ranges(int64_t L, const uint64_t* keys_sorted, int T, uint32_t* ranges, hipStream_t stream,
                       bool already_zero, const uint32_t* gather_index, const uint32_t* gather_table,
                       uint32_t* gather_out, const uint32_t* sort_error, uint32_t* fault_word) {
  if (T > 0 && !already_zero)
    hipLaunchKernelGGL(fill_u32_kernel, dim3((2 * T + 255) / 256), dim3(256), 0, stream, (int64_t)2 * T, 0u, ranges);
  if (L > 0)
    hipLaunchKernelGGL(tile_ranges_kernel, dim3((unsigned)((L + GS_BLOCK_1D - 1) / GS_BLOCK_1D)), dim3(GS_BLOCK_1D), 0,
                       stream, L, keys_sorted, ranges, gather_index, gather_table, gather_out, sort_error, fault_word);
  return 0;
}

}  // namespace gs
