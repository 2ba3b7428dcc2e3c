// C ABI of libgsrast.so (declarations and contracts: include/gsrast.h).
// Host-side orchestration only; kernels live in the other translation units.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <map>
#include <string>
#include <vector>

#include "../../include/gsrast.h"
#include "gs_common.h"
#include "gs_kernels.h"

#include <atomic>
#include <mutex>

namespace gs {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what, hipStream_t stream, bool sync) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess && sync) {
    e = hipStreamSynchronize(stream);
    if (e == hipSuccess) e = hipGetLastError();
  }
  if (e != hipSuccess) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return 1;
  }
  return 0;
}

// Optional per-stage GPU timing (the role of MyTimerOnGPU,
// cuda_rasterizer/timers.cu:11-79): when enabled, every stage of the composite
// entry points is bracketed by an event pair on its stream; pairs are resolved
// only when the caller collects them, so enabling it adds no synchronisation.
// Process-wide but safe to use from several threads: a stage's pair is filed,
// under the mutex, only once both events have been recorded.
struct StageClock {
  struct Rec {
    const char* name;
    hipEvent_t a, b;
  };
  std::atomic<bool> enabled{false};
  std::mutex mutex;
  std::vector<hipEvent_t> pool;
  std::vector<Rec> done;
  hipEvent_t take() {
    {
      std::lock_guard<std::mutex> lock(mutex);
      if (!pool.empty()) {
        hipEvent_t e = pool.back();
        pool.pop_back();
        return e;
      }
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    return e;
  }
  void give_back(hipEvent_t e) {
    if (e == nullptr) return;
    std::lock_guard<std::mutex> lock(mutex);
    pool.push_back(e);
  }
  void file(const Rec& r) {
    std::lock_guard<std::mutex> lock(mutex);
    done.push_back(r);
  }
};
static StageClock g_clock;

StageScope::StageScope(const char* stage, hipStream_t stream) : s(stream), name(stage) {
  if (!g_clock.enabled.load(std::memory_order_relaxed)) return;
  a = g_clock.take();
  b = g_clock.take();
  if (!a || !b || hipEventRecord(a, s) != hipSuccess) {
    g_clock.give_back(a);
    g_clock.give_back(b);
    a = b = nullptr;
  }
}

StageScope::~StageScope() {
  if (!a) return;
  if (hipEventRecord(b, s) == hipSuccess) {
    g_clock.file(StageClock::Rec{name, a, b});
  } else {
    g_clock.give_back(a);
    g_clock.give_back(b);
  }
}

namespace {

inline char* align_ptr(const char* p, size_t a) {
  return (char*)(((uintptr_t)p + a - 1) / a * a);
}

inline void tile_grid(int W, int H, int& gx, int& gy) {
  gx = (W + GS_TILE_X - 1) / GS_TILE_X;
  gy = (H + GS_TILE_Y - 1) / GS_TILE_Y;
}

struct ImageLayout {
  size_t accum_alpha, n_contrib, n_contrib2loss, ranges, bucket_table, total;
};
ImageLayout image_layout(int W, int H) {
  ImageLayout L;
  const size_t N = (size_t)W * H;
  int gx, gy;
  tile_grid(W, H, gx, gy);
  size_t off = 0;
  auto take = [&](size_t b) { size_t o = off; off += align_up(b, 256); return o; };
  L.accum_alpha = take(N * 4);
  L.n_contrib = take(N * 4);
  L.n_contrib2loss = take(N * 4);
  L.ranges = take((size_t)gx * gy * 8);
  // workgroup-by-tile counts of the counting sort by tile (nothing when the grid is too large for it)
  L.bucket_table = take(gx * gy <= bucket_max_tiles() ? bucket_table_bytes(gx * gy) : 0);
  L.total = off + 256;
  return L;
}

struct GeometryLayout {
  size_t tiles_touched, point_offsets, scan_temp, packed_valid, total;
};
GeometryLayout geometry_layout(int P) {
  GeometryLayout L;
  const size_t n = (size_t)(P > 0 ? P : 1);
  size_t off = 0;
  auto take = [&](size_t b) { size_t o = off; off += align_up(b, 256); return o; };
  L.tiles_touched = take(n * 4);
  L.point_offsets = take(n * 4);
  L.scan_temp = take(scan_temp_bytes((int64_t)n));
  L.packed_valid = take(4);  // one word: whether the forward call packed operand records (binning buffer)
  L.total = off + 256;
  return L;
}

struct BinningLayout {
  size_t point_list, keys, point_list_unsorted, keys_unsorted, emission, emission_other, sort_temp, block_hits,
      radix_scratch, packed, total;
};
// n = the number of instances the arrays are laid out for; packed_gaussians: the Gaussians the forward call packs
// operand records for (0 when it packs none, or when only the offsets are asked for)
BinningLayout binning_layout(int64_t R, int64_t packed_gaussians = 0) {
  BinningLayout L;
  const size_t n = (size_t)(R > 0 ? R : 1);
  size_t off = 0;
  auto take = [&](size_t b) { size_t o = off; off += align_up(b, 256); return o; };
  L.point_list = take(n * 4);
  L.keys = take(n * 8);
  // The next three lie back to back: on the per-tile route they are one array of 16-byte records (16 n bytes from
  // keys_unsorted on), on the radix route the unsorted keys, the Gaussian of every emission index and the sort's
  // second payload array.
  L.keys_unsorted = take(n * 8);
  L.point_list_unsorted = take(n * 4);
  L.emission_other = take(n * 4);
  L.emission = take(n * 4);
  L.sort_temp = take(sort_temp_bytes((int64_t)n));
  L.block_hits = take(n * 2);  // what the forward blend leaves for the backward blend, per sorted instance
  L.radix_scratch = take(n * 24);  // per-tile radix sort: lists beyond one block, split (16 B) and in blocks (8 B)
  // the blend kernels' operands, one 64-byte record per Gaussian, if the forward call packs them (last, so that
  // no other offset depends on whether it does)
  L.packed = take(packed_gaussians > 0 ? (size_t)packed_gaussians * 64 : 0);
  L.total = off + 256;
  return L;
}

int sort_end_bit(int W, int H) {
  int gx, gy;
  tile_grid(W, H, gx, gy);
  return 32 + (int)gs_higher_msb((uint32_t)(gx * gy));
}

struct EventTimer {
  hipEvent_t a = nullptr, b = nullptr;
  bool on = false;
  int begin(bool enable, hipStream_t s) {
    on = enable;
    if (!on) return 0;
    GS_HIP_TRY(hipEventCreate(&a));
    GS_HIP_TRY(hipEventCreate(&b));
    GS_HIP_TRY(hipEventRecord(a, s));
    return 0;
  }
  int end(hipStream_t s, float* ms) {
    if (!on) return 0;
    GS_HIP_TRY(hipEventRecord(b, s));
    GS_HIP_TRY(hipEventSynchronize(b));
    GS_HIP_TRY(hipEventElapsedTime(ms, a, b));
    return 0;
  }
  ~EventTimer() {
    if (a) (void)hipEventDestroy(a);
    if (b) (void)hipEventDestroy(b);
  }
};

#define GS_REQUIRE(cond, msg)        \
  do {                               \
    if (!(cond)) {                   \
      gs::set_error("%s", msg);      \
      return 1;                      \
    }                                \
  } while (0)

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

const char* gs_last_error(void) { return g_err; }

int gs_get_block_xy(int* bx, int* by, int* one_dim) {
  GS_REQUIRE(bx && by && one_dim, "gs_get_block_xy: null output");
  *bx = GS_TILE_X;
  *by = GS_TILE_Y;
  *one_dim = GS_BLOCK_1D;
  return 0;
}

uint32_t gs_higher_msb(uint32_t n) {
  // Smallest b with n < 2^b found by bisection from 16, as the reference's
  // host helper does; equals bit_length(n) for n >= 1 and 1 for n == 0.
  uint32_t msb = sizeof(n) * 4;
  uint32_t step = msb;
  while (step > 1) {
    step /= 2;
    if (n >> msb)
      msb += step;
    else
      msb -= step;
  }
  if (n >> msb) msb++;
  return msb;
}

int gs_mark_visible(int P, const float* means3D, const float* viewmatrix, const float* projmatrix, uint8_t* present,
                    gs_stream_t stream) {
  (void)projmatrix;
  GS_REQUIRE(P >= 0, "gs_mark_visible: negative P");
  if (P == 0) return 0;
  GS_REQUIRE(means3D && viewmatrix && present, "gs_mark_visible: null pointer");
  launch_mark_visible(P, means3D, viewmatrix, present, (hipStream_t)stream);
  return check_launch("mark_visible", (hipStream_t)stream, false);
}

int gs_visible_filter(int P, int M, int width, int height, const float* means3D, const float* scales,
                      float scale_modifier, const float* rotations, const float* cov3D_precomp,
                      const float* viewmatrix, const float* projmatrix, float tan_fovx, float tan_fovy,
                      int prefiltered, int* radii, int debug, gs_stream_t stream) {
  (void)M;
  (void)prefiltered;
  GS_REQUIRE(P >= 0 && width > 0 && height > 0, "gs_visible_filter: bad sizes");
  if (P == 0) return 0;
  GS_REQUIRE(means3D && viewmatrix && projmatrix && radii, "gs_visible_filter: null pointer");
  GS_REQUIRE(cov3D_precomp || (scales && rotations),
             "gs_visible_filter: need scales+rotations or a precomputed 3D covariance");
  {
    StageScope _t("visible_filter", (hipStream_t)stream);
    launch_visible_filter(P, means3D, scales, scale_modifier, rotations, cov3D_precomp, viewmatrix, projmatrix, width,
                        height, tan_fovx, tan_fovy, radii, (hipStream_t)stream);
  }
  return check_launch("visible_filter", (hipStream_t)stream, debug != 0);
}

int gs_preprocess_forward(float* means2D, float* depths, int* radii, float* cov3D, float* conic_opacity, float* rgb,
                          uint8_t* clamped, uint32_t* tiles_touched, int P, int D, int M, int width, int height,
                          const float* means3D, const float* scales, const float* rotations, const float* shs,
                          const float* opacities, float scale_modifier, const float* viewmatrix,
                          const float* projmatrix, const float* cam_pos, float tan_fovx, float tan_fovy,
                          int prefiltered, int debug, float* dcolor_ddir, float* blend_records,
                          gs_stream_t stream) {
  (void)prefiltered;
  GS_REQUIRE(P >= 0 && width > 0 && height > 0, "gs_preprocess_forward: bad sizes");
  GS_REQUIRE(((uintptr_t)blend_records & 15u) == 0u, "gs_preprocess_forward: blend_records must be 16-byte aligned");
  GS_REQUIRE(blend_records == nullptr || cam_pos != nullptr, "gs_preprocess_forward: blend_records needs cam_pos");
  if (P == 0) return 0;
  GS_REQUIRE(means2D && depths && radii && conic_opacity && rgb && clamped, "gs_preprocess_forward: null output");
  GS_REQUIRE(means3D && scales && rotations && opacities && viewmatrix && projmatrix,
             "gs_preprocess_forward: null input");
  const bool sh_mode = shs != nullptr && M > 0;
  GS_REQUIRE(!sh_mode || (cam_pos != nullptr && D >= 0 && D <= 3 && M >= (D + 1) * (D + 1) && M <= 16),
             "gs_preprocess_forward: SH mode needs cam_pos, 0<=D<=3 and (D+1)^2 <= M <= 16");
  PreprocessFwdArgs a;
  a.P = P; a.D = D; a.M = sh_mode ? M : 0; a.W = width; a.H = height;
  a.means3D = means3D; a.scales = scales; a.rotations = rotations; a.opacities = opacities;
  a.shs = sh_mode ? shs : nullptr;
  a.scale_modifier = scale_modifier;
  a.viewmatrix = viewmatrix; a.projmatrix = projmatrix; a.campos = cam_pos;
  a.tanx = tan_fovx; a.tany = tan_fovy;
  a.radii = radii; a.means2D = means2D; a.depths = depths; a.cov3D = cov3D; a.conic_opacity = conic_opacity;
  a.rgb = rgb; a.clamped = clamped; a.tiles_touched = tiles_touched;
  a.dcolor_ddir = sh_mode ? dcolor_ddir : nullptr;
  a.blend_records = blend_records;
  {
    StageScope _t("preprocess_fwd", (hipStream_t)stream);
    launch_preprocess_fwd(a, (hipStream_t)stream);
  }
  return check_launch("preprocess_forward", (hipStream_t)stream, debug != 0);
}

int gs_preprocess_backward(const int* radii, const float* cov3D, const uint8_t* clamped, int P, int D, int M,
                           int width, int height, const float* means3D, const float* scales, const float* rotations,
                           const float* shs, float scale_modifier, const float* viewmatrix, const float* projmatrix,
                           const float* campos, float tan_fovx, float tan_fovy, const float* dL_dmean2D,
                           int mean2D_stride, const float* dL_dconic_opacity, const float* dL_dcolor,
                           float* dL_dmean3D, float* dL_dcov3D, float* dL_dscale, float* dL_drot, float* dL_dsh,
                           float* dL_dopacity, int debug, const float* dcolor_ddir, gs_stream_t stream) {
  GS_REQUIRE(P >= 0 && width > 0 && height > 0, "gs_preprocess_backward: bad sizes");
  if (P == 0) return 0;
  GS_REQUIRE(radii && means3D && viewmatrix && projmatrix && dL_dmean2D && dL_dconic_opacity && dL_dmean3D,
             "gs_preprocess_backward: null pointer");
  GS_REQUIRE(cov3D || (scales && rotations), "gs_preprocess_backward: without cov3D, scales and rotations are needed");
  GS_REQUIRE(mean2D_stride == 2 || mean2D_stride == 3, "gs_preprocess_backward: mean2D_stride must be 2 or 3");
  GS_REQUIRE((scales == nullptr) == (rotations == nullptr), "gs_preprocess_backward: scales and rotations go together");
  GS_REQUIRE(!scales || (dL_dscale && dL_drot), "gs_preprocess_backward: null scale/rotation gradient");
  const bool sh_mode = (shs != nullptr || dcolor_ddir != nullptr) && M > 0 && dL_dsh != nullptr;
  GS_REQUIRE(!sh_mode || (campos && clamped && dL_dcolor && D >= 0 && D <= 3 && M >= (D + 1) * (D + 1) && M <= 16),
             "gs_preprocess_backward: SH mode needs campos, clamped, dL_dcolor and (D+1)^2 <= M <= 16");
  PreprocessBwdArgs a;
  a.P = P; a.D = D; a.M = sh_mode ? M : 0; a.W = width; a.H = height;
  a.means3D = means3D; a.radii = radii; a.shs = sh_mode ? shs : nullptr; a.clamped = clamped;
  a.dcolor_ddir = sh_mode ? dcolor_ddir : nullptr;
  a.scales = scales; a.rotations = rotations; a.scale_modifier = scale_modifier;
  a.cov3D = cov3D; a.viewmatrix = viewmatrix; a.projmatrix = projmatrix; a.campos = campos;
  a.tanx = tan_fovx; a.tany = tan_fovy;
  a.dL_dmean2D = dL_dmean2D; a.mean2D_stride = mean2D_stride; a.dL_dconic_opacity = dL_dconic_opacity;
  a.dL_dcolor = dL_dcolor;
  a.dL_dmean3D = dL_dmean3D; a.dL_dcov3D = dL_dcov3D; a.dL_dsh = sh_mode ? dL_dsh : nullptr;
  a.dL_dscale = dL_dscale; a.dL_drot = dL_drot; a.dL_dopacity = dL_dopacity;
  {
    StageScope _t("preprocess_bwd", (hipStream_t)stream);
    launch_preprocess_bwd(a, (hipStream_t)stream);
  }
  return check_launch("preprocess_backward", (hipStream_t)stream, debug != 0);
}

// Host-visible words through which the scan hands the instance count to the waiting host thread.  Pinned
// memory is allocated once per process; calls take the words in turn, so calls on different streams or
// threads do not share one unless more than TOTAL_SLOTS of them are inside gs_render_forward together.
namespace {
constexpr uint32_t TOTAL_PENDING = 0xFFFFFFFFu;  // never a valid count (counts stay below 2^31)
constexpr int TOTAL_SLOTS = 64;
std::atomic<uint32_t*> g_total_slots{nullptr};
std::atomic<unsigned> g_total_next{0};
std::mutex g_total_mutex;

uint32_t* pinned_words() {
  uint32_t* base = g_total_slots.load(std::memory_order_acquire);
  if (base == nullptr) {
    std::lock_guard<std::mutex> lock(g_total_mutex);
    base = g_total_slots.load(std::memory_order_acquire);
    if (base == nullptr) {
      void* p = nullptr;
      // 64-byte spacing keeps the words on separate lines; one more line holds the fault word (below)
      if (hipHostMalloc(&p, (TOTAL_SLOTS + 1) * 64, hipHostMallocDefault) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;  // the caller falls back to a copy and a stream wait
      }
      base = (uint32_t*)p;
      base[16 * TOTAL_SLOTS] = 0u;
      g_total_slots.store(base, std::memory_order_release);
    }
  }
  return base;
}

uint32_t* acquire_total_slot() {
  uint32_t* base = pinned_words();
  if (base == nullptr) return nullptr;
  uint32_t* slot = base + 16 * (g_total_next.fetch_add(1, std::memory_order_relaxed) % TOTAL_SLOTS);
  slot[1] = 0u;  // second and third word of the slot: the longest tile list and the numbers of lists for the
  slot[2] = 0u;  // per-tile radix sort's two kernels, both written before the total
  __atomic_store_n(slot, TOTAL_PENDING, __ATOMIC_RELEASE);
  return slot;
}

// Polls the word; looks at the stream now and then so that a failed launch ends the wait with its error.
int wait_for_total(uint32_t* slot, hipStream_t stream, uint32_t* out) {
  for (unsigned spins = 0;; spins++) {
    const uint32_t v = __atomic_load_n(slot, __ATOMIC_ACQUIRE);
    if (v != TOTAL_PENDING) {
      *out = v;
      return 0;
    }
    if ((spins & 0x3FFFu) == 0x3FFFu) {
      const hipError_t q = hipStreamQuery(stream);
      if (q == hipSuccess) {
        const uint32_t w = __atomic_load_n(slot, __ATOMIC_ACQUIRE);
        if (w != TOTAL_PENDING) {
          *out = w;
          return 0;
        }
        set_error("gs_render_forward: the stream drained without the scan reporting its total");
        return 1;
      }
      if (q != hipErrorNotReady) {
        set_error("gs_render_forward: waiting for the instance count: %s", hipGetErrorString(q));
        return 1;
      }
    }
  }
}
}  // namespace

namespace {
// A kernel that runs after a radix sort sets this host-visible word when the sort's bounded look-back wait ran
// out (its output is then not sorted).  The word is sticky: the entry points look at it when they are called,
// without waiting for anything, so the failure of a sort surfaces at the next call after its kernels have run
// (and at once in debug mode or when a call times itself, both of which wait for the stream).
uint32_t* fault_word() {
  uint32_t* base = pinned_words();
  return base ? base + 16 * TOTAL_SLOTS : nullptr;
}

int pending_fault(const char* who) {
  uint32_t* w = g_total_slots.load(std::memory_order_acquire);
  if (w == nullptr) return 0;
  w += 16 * TOTAL_SLOTS;
  if (__atomic_load_n(w, __ATOMIC_ACQUIRE) == 0u) return 0;
  __atomic_store_n(w, 0u, __ATOMIC_RELEASE);
  set_error("%s: an earlier radix sort on this process ran out of its bounded look-back wait; the per-tile lists "
            "(or neighbour distances) computed from it, and everything derived from them, are not to be trusted",
            who);
  return 1;
}

struct TileSortLimits {
  int small, block;
};
// The defaults, or what the caller's options ask for: the list length up to which a list is sorted in registers
// (0: the view takes the radix sort over all its keys), and the number of records the per-tile radix sort holds
// in one block (longer lists are sorted block by block through memory).
TileSortLimits tile_sort_limits(const gs_render_options* o) {
  TileSortLimits L = {TILE_SORT_SMALL, tile_radix_block_records()};
  if (o == nullptr || o->struct_bytes < 3 * sizeof(uint32_t)) return L;
  if (o->tile_sort_small_limit >= 0) L.small = o->tile_sort_small_limit < TILE_SORT_SMALL ? o->tile_sort_small_limit : TILE_SORT_SMALL;
  if (o->tile_sort_block_records > 0 && o->tile_sort_block_records < L.block) L.block = o->tile_sort_block_records;
  return L;
}
}  // namespace

int gs_pending_fault(void) { return pending_fault("gs_pending_fault"); }

int gs_render_forward(gs_resize_fn geometryBuffer, void* geometry_user, gs_resize_fn binningBuffer,
                      void* binning_user, gs_resize_fn imageBuffer, void* image_user, int P, const float* background,
                      int width, int height, float focal_x, float focal_y, float cx, float cy,
                      const float* viewmatrix, const float* cam_pos, const float* all_map, const float* means2D,
                      const float* depths, const int* radii, const float* conic_opacity, const float* rgb,
                      const uint8_t* compute_locally, float* out_color, int* n_render, int* n_consider,
                      int* n_contrib, int* out_observe, float* out_all_map, float* out_plane_depth,
                      float* out_max_weight_depth, int render_geo, int debug, int* num_rendered, float* elapsed_ms,
                      const gs_render_options* options, gs_render_result* result, gs_stream_t stream_) {
  (void)viewmatrix;
  (void)cam_pos;
  hipStream_t stream = (hipStream_t)stream_;
  if (pending_fault("gs_render_forward")) return 1;
  const TileSortLimits limits = tile_sort_limits(options);
  GS_REQUIRE(P > 0 && width > 0 && height > 0, "gs_render_forward: P, width and height must be positive");
  GS_REQUIRE(geometryBuffer && binningBuffer && imageBuffer, "gs_render_forward: null resize callback");
  GS_REQUIRE(background && means2D && depths && radii && conic_opacity && rgb && compute_locally,
             "gs_render_forward: null input");
  GS_REQUIRE(out_color && n_render && n_consider && n_contrib && out_observe && num_rendered,
             "gs_render_forward: null output");
  GS_REQUIRE(!render_geo || (all_map && out_all_map && out_plane_depth),
             "gs_render_forward: render_geo needs all_map, out_all_map and out_plane_depth");
  const bool dbg = debug != 0;
  int gx, gy;
  tile_grid(width, height, gx, gy);
  const int T = gx * gy;

  // The blend kernels' operand records: the caller's (complete: gs_preprocess_forward and gs_all_map_forward wrote
  // their parts), or packed here for a view with enough instances per Gaussian.
  const float* caller_records =
      (options != nullptr && options->struct_bytes >= sizeof(gs_render_options)) ? options->blend_records : nullptr;
  GS_REQUIRE(((uintptr_t)caller_records & 15u) == 0u, "gs_render_forward: blend_records must be 16-byte aligned");
  const GeometryLayout GL = geometry_layout(P);
  char* gbase = geometryBuffer(GL.total, geometry_user);
  GS_REQUIRE(gbase, "gs_render_forward: geometry buffer callback returned NULL");
  gbase = align_ptr(gbase, 256);
  uint32_t* tiles_touched = (uint32_t*)(gbase + GL.tiles_touched);
  uint32_t* point_offsets = (uint32_t*)(gbase + GL.point_offsets);
  void* scan_temp = gbase + GL.scan_temp;
  uint32_t* packed_valid = (uint32_t*)(gbase + GL.packed_valid);

  const ImageLayout IL = image_layout(width, height);
  char* ibase = imageBuffer(IL.total, image_user);
  GS_REQUIRE(ibase, "gs_render_forward: image buffer callback returned NULL");
  ibase = align_ptr(ibase, 256);
  float* accum_alpha = (float*)(ibase + IL.accum_alpha);
  uint32_t* n_contrib_px = (uint32_t*)(ibase + IL.n_contrib);
  uint32_t* n_contrib2loss_px = (uint32_t*)(ibase + IL.n_contrib2loss);
  uint32_t* ranges = (uint32_t*)(ibase + IL.ranges);

  // Two ways to the sorted per-tile lists.  The default buckets the instances by tile (counting sort) and sorts
  // every tile's list on its own; it needs the tile histogram to fit in LDS.  Otherwise: emit (tile | depth) keys,
  // radix-sort all of them, find the tile boundaries.
  uint32_t* total_slot = acquire_total_slot();
  void* bucket_table = ibase + IL.bucket_table;
  const uint32_t sort_limit = (uint32_t)limits.small;
  const bool bucketed = T <= bucket_max_tiles() && total_slot != nullptr && sort_limit > 0;

  // The instance count decides the size of the binning buffer, and the host learns it only after the counting
  // kernels have run: a round trip during which the GPU would idle.  A caller that says how many instances and
  // how long a list it expects (the previous view's figures with a margin) gets the list kernels and the blend
  // launched right behind the counting kernels, on buffers of the expected size; a device word tells them whether
  // the view fits (they do nothing otherwise), and the host, which meanwhile has received the counts, either
  // returns or builds the lists again the ordinary way.
  int64_t cap_n = 0;
  uint32_t cap_longest = 0;
  if (bucketed && !dbg && result != nullptr && result->struct_bytes >= sizeof(gs_render_result) &&
      options != nullptr && options->struct_bytes >= sizeof(gs_render_options) && options->expected_instances > 0) {
    cap_n = options->expected_instances < (int64_t)GS_MAX_INSTANCES ? options->expected_instances
                                                                     : (int64_t)GS_MAX_INSTANCES;
    // (0: any length; the sort kernels launched and their LDS depend on it)
    cap_longest = options->expected_longest_list > 0 ? (uint32_t)options->expected_longest_list : GS_MAX_INSTANCES;
  }
  const bool ahead = cap_n > 0;

  if (bucketed) {
    StageScope _t("tile_count", stream);
    // the histogram's grand total is the instance count: the host gets it from here
    if (launch_bucket_count(P, width, height, radii, means2D, compute_locally, tiles_touched, bucket_table, ranges,
                            sort_limit, (uint32_t)limits.block, total_slot, out_observe, (uint32_t)cap_n, cap_longest,
                            packed_valid, stream))
      return 1;
  } else {
    StageScope _t("tile_count", stream);
    // also clears the tile ranges (cudaMemset of CR/rasterizer_impl.cu:687), which nothing reads before
    // identify_tile_ranges fills them
    launch_tile_count(P, width, height, radii, means2D, compute_locally, tiles_touched, stream, ranges,
                      (int64_t)2 * T, out_observe);
  }
  if (check_launch("tile_count", stream, dbg)) return 1;
  if (!bucketed) {
    StageScope _t("inclusive_sum", stream);
    launch_inclusive_sum(P, tiles_touched, point_offsets, scan_temp, stream, total_slot);
  }
  if (check_launch("inclusive_sum", stream, dbg)) return 1;
  // The blend kernels (this call's and the backward call's) can fetch a Gaussian's operands as one 64-byte record
  // instead of gathering parts of five lines of memory.  Packing the records costs about 20 us per million
  // Gaussians and saves about 25 us per million instances: done for a view with enough instances per Gaussian.
  // The library's own records live at the end of the binning buffer, which is sized once the decision is made.
  bool use_packed = false, pack_decided = false;
  auto decide_packing = [&](int64_t instances) {
    if (pack_decided) return;
    pack_decided = true;
    use_packed = caller_records != nullptr || instances * 5 > (int64_t)P * 4;
  };

  EventTimer timer;
  struct Arrays {
    uint32_t *point_list, *gauss_of_emission, *emission, *emission_other;
    uint64_t *keys, *keys_other;
    void *sort_temp, *radix_scratch;
    int64_t capacity;
    uint16_t* block_hits;
    float* packed;
  };
  auto carve = [&](int64_t n, Arrays& A) -> int {
    const BinningLayout BL = binning_layout(n, (use_packed && caller_records == nullptr) ? (int64_t)P : 0);
    char* bbase = binningBuffer(BL.total, binning_user);
    GS_REQUIRE(bbase, "gs_render_forward: binning buffer callback returned NULL");
    bbase = align_ptr(bbase, 256);
    A.point_list = (uint32_t*)(bbase + BL.point_list);
    A.keys = (uint64_t*)(bbase + BL.keys);
    A.gauss_of_emission = (uint32_t*)(bbase + BL.point_list_unsorted);
    A.keys_other = (uint64_t*)(bbase + BL.keys_unsorted);
    A.emission = (uint32_t*)(bbase + BL.emission);
    A.emission_other = (uint32_t*)(bbase + BL.emission_other);
    A.sort_temp = bbase + BL.sort_temp;
    A.block_hits = (uint16_t*)(bbase + BL.block_hits);
    A.radix_scratch = bbase + BL.radix_scratch;
    A.packed = (float*)(bbase + BL.packed);
    A.capacity = n > 0 ? n : 1;
    return 0;
  };
  // Packs the library's own records into the arrays just carved.  With the caller's records, or none, the word
  // beside them must say "none" (a backward call that is not handed the caller's records again then gathers the
  // operands from the arrays): the counting kernels of the per-tile route have cleared it on their way.
  auto pack_records = [&](const Arrays& A) -> int {
    if (caller_records != nullptr || !use_packed) {
      if (bucketed) return 0;
      launch_fill_u32(1, 0u, packed_valid, stream);
      return check_launch("pack_operands", stream, dbg);
    }
    StageScope _t("pack_operands", stream);
    launch_pack_blend_operands(P, radii, means2D, conic_opacity, rgb, render_geo ? all_map : nullptr, depths,
                               A.packed, packed_valid, stream);
    return check_launch("pack_operands", stream, dbg);
  };
  auto blend = [&](const Arrays& A, bool ahead_of_host) -> int {
    RenderFwdArgs a;
    a.P = P; a.W = width; a.H = height;
    a.fx = focal_x; a.fy = focal_y; a.cx = cx; a.cy = cy;
    a.ranges = ranges; a.point_list = A.point_list;
    a.means2D = means2D; a.rgb = rgb; a.all_map = all_map; a.conic_opacity = conic_opacity;
    a.compute_locally = compute_locally; a.bg = background; a.render_geo = render_geo;
    a.final_T = accum_alpha; a.n_contrib_px = n_contrib_px; a.n_contrib2loss_px = n_contrib2loss_px;
    a.out_color = out_color; a.out_observe = out_observe; a.out_all_map = out_all_map;
    a.out_plane_depth = out_plane_depth;
    a.depths = depths; a.out_max_weight_depth = out_max_weight_depth;
    a.n_render = n_render; a.n_consider = n_consider; a.n_contrib_tile = n_contrib;
    a.fits_word = ahead_of_host ? bucket_fits_word(bucket_table, T) : nullptr;
    a.block_hits = A.block_hits;
    a.packed = use_packed ? (caller_records != nullptr ? caller_records : A.packed) : nullptr;
    {
      StageScope _t("render_fwd", stream);
      launch_render_fwd(a, stream);
    }
    return check_launch("render_forward", stream, dbg);
  };
  auto lists_by_tile = [&](const Arrays& A, uint32_t longest_for_launch, uint32_t radix_tiles,
                           bool ahead_of_host) -> int {
    {
      StageScope _t("bucket_scatter", stream);
      // (also finishes the prefix sum over the Gaussians: point_offsets; the 16-byte records take the place of
      // the three unsorted arrays of the other route)
      launch_bucket_scatter(P, width, height, means2D, depths, tiles_touched, point_offsets, radii, compute_locally,
                            bucket_table, ranges, A.keys_other, ahead_of_host, stream);
    }
    if (check_launch("bucket_scatter", stream, dbg)) return 1;
    {
      StageScope _t("tile_sort", stream);
      if (launch_tile_sort(T, longest_for_launch, radix_tiles, sort_limit, (uint32_t)limits.block, ranges,
                           bucket_table, A.keys_other, A.radix_scratch, A.capacity, A.keys, A.emission,
                           A.point_list, ahead_of_host, stream))
        return 1;
    }
    return check_launch("tile_sort", stream, dbg);
  };

  Arrays A;
  if (ahead) {
    // (on the expected count less a fifth: the caller's expectation carries a margin of a quarter)
    decide_packing(cap_n - cap_n / 5);
    if (carve(cap_n, A)) return 1;
    if (timer.begin(elapsed_ms != nullptr, stream)) return 1;
    if (pack_records(A)) return 1;
    if (lists_by_tile(A, cap_longest, 0xFFFFFFFFu, true)) return 1;
    if (blend(A, true)) return 1;
  }

  // The host needs the instance count: it sizes the binning buffer (unless that was done ahead), and the caller
  // gets it back.  The counting kernels write it straight into pinned host memory and the host polls that word:
  // no copy, and no sleeping wait.  On the bucketed route the longest tile list and the numbers of lists that go
  // to the per-tile radix sort's two kernels arrive in the words beside it.
  uint32_t R_u = 0, longest = 0, radix_tiles = 0;
  if (total_slot != nullptr) {
    if (wait_for_total(total_slot, stream, &R_u)) return 1;
    longest = __atomic_load_n(total_slot + 1, __ATOMIC_ACQUIRE);
    radix_tiles = __atomic_load_n(total_slot + 2, __ATOMIC_ACQUIRE);
  } else {
    uint32_t wrapped = 0;
    GS_HIP_TRY(hipMemcpyAsync(&R_u, point_offsets + (P - 1), sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
    GS_HIP_TRY(hipMemcpyAsync(&wrapped, scan_overflow_word(scan_temp, P), sizeof(uint32_t), hipMemcpyDeviceToHost,
                              stream));
    GS_HIP_TRY(hipStreamSynchronize(stream));
    if (wrapped != 0u) R_u = GS_TOO_MANY_INSTANCES;
  }
  if (R_u > GS_MAX_INSTANCES) {
    set_error("gs_render_forward: more than 2^31-2 (Gaussian, tile) instances in one view");
    return 1;
  }
  const int64_t R = (int64_t)R_u;
  *num_rendered = (int)R;
  if (result != nullptr && result->struct_bytes >= sizeof(gs_render_result)) {
    result->longest_list = bucketed ? (int32_t)longest : 0;
    result->binning_capacity = R;
    result->launched_ahead = 0;
  }

  // (the same test the ranges kernel made on the device)
  if (ahead && R <= cap_n && longest <= cap_longest) {
    result->binning_capacity = cap_n;
    result->launched_ahead = 1;
    if (timer.end(stream, elapsed_ms)) return 1;
    return 0;
  }

  // The ordinary way (also after kernels launched ahead found that the view does not fit and did nothing).
  // (after kernels launched ahead: the records are packed again, the buffer may be another one)
  decide_packing(R);
  if (carve(R, A)) return 1;
  if (!ahead && timer.begin(elapsed_ms != nullptr, stream)) return 1;
  if (pack_records(A)) return 1;

  if (bucketed) {
    if (lists_by_tile(A, longest, radix_tiles, false)) return 1;
  } else {
    if (R > sort_max_pairs()) {
      set_error("gs_render_forward: %lld instances in a view that takes the radix sort over all keys, which takes "
                "at most 2^30-2", (long long)R);
      return 1;
    }
    const int end_bit = sort_end_bit(width, height);
    // The sort carries each instance's index in emission order as its payload (the backward pass files
    // per-instance gradients under it); the Gaussian ids of the sorted list are gathered afterwards.
    // It ping-pongs, so start from the array pair that makes it finish in (keys, emission).
    const bool odd = sort_result_in_b(end_bit);
    uint64_t* k_start = odd ? A.keys_other : A.keys;
    uint32_t* e_start = odd ? A.emission_other : A.emission;
    uint64_t* k_partner = odd ? A.keys : A.keys_other;
    uint32_t* e_partner = odd ? A.emission : A.emission_other;
    if (R > 0) {
      {
        StageScope _t("duplicate_with_keys", stream);
        launch_duplicate_with_keys(P, width, height, means2D, depths, point_offsets, radii, compute_locally, k_start,
                                   A.gauss_of_emission, e_start, stream);
      }
      if (check_launch("duplicate_with_keys", stream, dbg)) return 1;
      {
        StageScope _t("sort_pairs", stream);
        if (launch_sort_pairs_u64(R, k_start, k_partner, e_start, e_partner, end_bit, A.sort_temp, stream)) return 1;
      }
      if (check_launch("sort_pairs", stream, dbg)) return 1;
      if (dbg) {  // (sort_temp is 256-byte aligned already)
        uint32_t word = 0;
        GS_HIP_TRY(hipMemcpyAsync(&word, sort_error_word(A.sort_temp), sizeof(uint32_t), hipMemcpyDeviceToHost,
                                  stream));
        GS_HIP_TRY(hipStreamSynchronize(stream));
        GS_REQUIRE(word == 0u, "gs_render_forward: the radix sort's bounded look-back wait ran out");
      }
    }
    {
      StageScope _t("identify_tile_ranges", stream);
      // ... and gathers the Gaussian ids of the sorted instances on the way (point_list).  The ranges were
      // cleared by the counting kernel of this path, or hold the other path's table and are cleared here.
      // It also looks at the sort's error word and raises the sticky fault word if the sort gave up.
      launch_tile_ranges(R, A.keys, T, ranges, stream, true, A.emission, A.gauss_of_emission,
                         A.point_list, R > 0 ? sort_error_word(A.sort_temp) : nullptr, fault_word());
    }
    if (check_launch("identify_tile_ranges", stream, dbg)) return 1;
  }

  if (blend(A, false)) return 1;
  if (timer.end(stream, elapsed_ms)) return 1;
  // (debug mode and the timer have waited for the stream: a sort that gave up in this call is known by now)
  if ((dbg || elapsed_ms != nullptr) && pending_fault("gs_render_forward")) return 1;
  return 0;
}

int gs_render_backward(int P, int R, const float* background, int width, int height, float tan_fovx, float tan_fovy,
                       const char* geom_buffer, const char* binning_buffer, const char* img_buffer,
                       const uint8_t* compute_locally, const float* dL_dpix, const float* dL_dout_all_map,
                       const float* dL_dout_plane_depth, float* dL_dmean2D, float* dL_dmean2D_abs,
                       float* dL_dconic_opacity, float* dL_dcolor, float* dL_dall_map, const float* means2D,
                       const float* conic_opacity, const float* rgb, const float* all_maps,
                       const float* all_map_pixels, int render_geo, int debug, float* instance_grads,
                       size_t instance_grads_bytes, float* elapsed_ms, int64_t binning_capacity,
                       const float* blend_records, gs_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (pending_fault("gs_render_backward")) return 1;
  GS_REQUIRE(binning_capacity <= 0 || binning_capacity >= R, "gs_render_backward: binning_capacity below R");
  GS_REQUIRE(P > 0 && R >= 0 && width > 0 && height > 0, "gs_render_backward: bad sizes");
  GS_REQUIRE(geom_buffer && binning_buffer && img_buffer && compute_locally && background,
             "gs_render_backward: null buffer");
  GS_REQUIRE(instance_grads && instance_grads_bytes >= gs_render_backward_workspace_bytes(R),
             "gs_render_backward: instance_grads workspace missing or too small");
  GS_REQUIRE(dL_dpix && dL_dmean2D && dL_dmean2D_abs && dL_dconic_opacity && dL_dcolor && means2D &&
                 conic_opacity && rgb,
             "gs_render_backward: null pointer");
  GS_REQUIRE(!render_geo || (dL_dout_all_map && dL_dout_plane_depth && dL_dall_map && all_maps && all_map_pixels),
             "gs_render_backward: render_geo needs the geometry-map tensors");
  const BinningLayout BL = binning_layout(binning_capacity > 0 ? binning_capacity : (int64_t)R);
  const ImageLayout IL = image_layout(width, height);
  const GeometryLayout GL = geometry_layout(P);
  const char* gbase = align_ptr(geom_buffer, 256);
  const char* bbase = align_ptr(binning_buffer, 256);
  const char* ibase = align_ptr(img_buffer, 256);
  RenderBwdArgs a;
  a.emission_sorted = (const uint32_t*)(bbase + BL.emission);
  a.block_hits = (const uint16_t*)(bbase + BL.block_hits);
  a.point_offsets = (const uint32_t*)(gbase + GL.point_offsets);
  // (records of the arrays the forward call was given: the caller's own, or what the forward call packed)
  GS_REQUIRE(((uintptr_t)blend_records & 15u) == 0u, "gs_render_backward: blend_records must be 16-byte aligned");
  a.packed = blend_records != nullptr ? blend_records : (const float*)(bbase + BL.packed);
  a.packed_valid = blend_records != nullptr ? nullptr : (const uint32_t*)(gbase + GL.packed_valid);
  a.instance_grads = (float*)align_ptr((const char*)instance_grads, 256);
  a.P = P; a.W = width; a.H = height;
  a.fy = height / (2.0f * tan_fovy);  // cuda_rasterizer/rasterizer_impl.cu:885-886
  a.fx = width / (2.0f * tan_fovx);
  a.bg = background;
  a.ranges = (const uint32_t*)(ibase + IL.ranges);
  a.point_list = (const uint32_t*)(bbase + BL.point_list);
  a.means2D = means2D; a.conic_opacity = conic_opacity; a.rgb = rgb; a.all_map = all_maps;
  a.all_map_pixels = all_map_pixels;
  a.final_T = (const float*)(ibase + IL.accum_alpha);
  a.n_contrib_px = (const uint32_t*)(ibase + IL.n_contrib);
  a.compute_locally = compute_locally;
  a.dL_dpix = dL_dpix; a.dL_dout_all_map = dL_dout_all_map; a.dL_dout_plane_depth = dL_dout_plane_depth;
  a.render_geo = render_geo;
  a.dL_dmean2D = dL_dmean2D; a.dL_dmean2D_abs = dL_dmean2D_abs; a.dL_dconic_opacity = dL_dconic_opacity;
  a.dL_dcolors = dL_dcolor; a.dL_dall_map = dL_dall_map;
  EventTimer timer;
  if (timer.begin(elapsed_ms != nullptr, stream)) return 1;
  {
    StageScope _t("render_bwd", stream);
    launch_render_bwd(a, stream);
  }
  if (check_launch("render_backward", stream, debug != 0)) return 1;
  if (timer.end(stream, elapsed_ms)) return 1;
  return 0;
}

size_t gs_render_backward_workspace_bytes(int R) { return (size_t)(R > 0 ? R : 1) * 16 * sizeof(float) + 256; }

size_t gs_knn_workspace_bytes(int P) { return knn_temp_bytes(P) + 256; }

int gs_ssim_l1_forward(int channels, int height, int width, const float* img1, const float* img2,
                       const uint8_t* pixel_mask, float* l1_map, float* ssim_map, float* d_mu, float* d_xx,
                       float* d_xy, gs_stream_t stream) {
  GS_REQUIRE(channels >= 0 && height >= 0 && width >= 0, "gs_ssim_l1_forward: negative size");
  if (channels == 0 || height == 0 || width == 0) return 0;
  GS_REQUIRE(channels <= 65535, "gs_ssim_l1_forward: too many channels");
  GS_REQUIRE(img1 && img2 && l1_map && ssim_map, "gs_ssim_l1_forward: null pointer");
  GS_REQUIRE((d_mu && d_xx && d_xy) || (!d_mu && !d_xx && !d_xy),
             "gs_ssim_l1_forward: pass all three derivative maps or none");
  {
    StageScope _t("ssim_l1_fwd", (hipStream_t)stream);
    launch_ssim_l1_fwd(channels, height, width, img1, img2, pixel_mask, l1_map, ssim_map, d_mu, d_xx, d_xy,
                       (hipStream_t)stream);
  }
  return check_launch("ssim_l1_forward", (hipStream_t)stream, false);
}

int gs_ssim_l1_backward(int channels, int height, int width, const float* img1, const float* img2,
                        const uint8_t* pixel_mask, const float* dL_dl1_map, const float* dL_dssim_map,
                        const float* d_mu, const float* d_xx, const float* d_xy, float* dL_dimg1,
                        gs_stream_t stream) {
  GS_REQUIRE(channels >= 0 && height >= 0 && width >= 0, "gs_ssim_l1_backward: negative size");
  if (channels == 0 || height == 0 || width == 0) return 0;
  GS_REQUIRE(channels <= 65535, "gs_ssim_l1_backward: too many channels");
  GS_REQUIRE(img1 && img2 && d_mu && d_xx && d_xy && dL_dimg1, "gs_ssim_l1_backward: null pointer");
  {
    StageScope _t("ssim_l1_bwd", (hipStream_t)stream);
    launch_ssim_l1_bwd(channels, height, width, img1, img2, pixel_mask, dL_dl1_map, dL_dssim_map, d_mu, d_xx, d_xy,
                       dL_dimg1, (hipStream_t)stream);
  }
  return check_launch("ssim_l1_backward", (hipStream_t)stream, false);
}

size_t gs_training_stats_workspace_bytes(int64_t num_anchors, int64_t num_candidates) {
  return train_stats_temp_bytes(num_anchors, num_candidates) + 256;
}

int gs_training_stats(int64_t num_anchors, int n_offsets, int64_t num_candidates, int64_t num_selected,
                      const uint8_t* anchor_visible_mask, const uint8_t* offset_selection_mask,
                      const uint8_t* update_filter, const float* viewspace_grad, int grad_stride,
                      const float* opacity, float* opacity_accum, float* anchor_demon,
                      float* offset_gradient_accum, float* offset_denom, void* workspace, size_t workspace_bytes,
                      gs_stream_t stream) {
  GS_REQUIRE(num_anchors >= 0 && n_offsets > 0 && num_candidates >= 0 && num_selected >= 0,
             "gs_training_stats: bad sizes");
  if (num_anchors == 0) return 0;
  GS_REQUIRE(num_anchors * (int64_t)n_offsets < 0x7FFFFFFFll * GS_BLOCK_1D, "gs_training_stats: too many slots");
  GS_REQUIRE(num_candidates < 0xFFFFFFFFll && num_anchors < 0xFFFFFFFFll, "gs_training_stats: ranks are 32-bit");
  GS_REQUIRE(anchor_visible_mask && opacity_accum && anchor_demon && offset_gradient_accum && offset_denom,
             "gs_training_stats: null pointer");
  GS_REQUIRE(num_candidates == 0 || (offset_selection_mask && opacity),
             "gs_training_stats: candidates without mask or opacity");
  GS_REQUIRE(num_selected == 0 || (update_filter && viewspace_grad && grad_stride >= 2),
             "gs_training_stats: selected Gaussians without filter or gradient (stride >= 2)");
  GS_REQUIRE(workspace && workspace_bytes >= gs_training_stats_workspace_bytes(num_anchors, num_candidates),
             "gs_training_stats: workspace missing or too small");
  {
    StageScope _t("training_stats", (hipStream_t)stream);
    launch_train_stats(num_anchors, n_offsets, num_candidates, num_selected, anchor_visible_mask,
                       offset_selection_mask, update_filter, viewspace_grad, grad_stride, opacity, opacity_accum,
                       anchor_demon, offset_gradient_accum, offset_denom, align_ptr((char*)workspace, 256),
                       (hipStream_t)stream);
  }
  return check_launch("training_stats", (hipStream_t)stream, false);
}

int gs_max_radii_update(int64_t n, const int* radii, const uint8_t* visibility_filter, float* max_radii2D,
                        gs_stream_t stream) {
  GS_REQUIRE(n >= 0, "gs_max_radii_update: negative n");
  if (n == 0) return 0;
  GS_REQUIRE(radii && visibility_filter && max_radii2D, "gs_max_radii_update: null pointer");
  launch_max_radii(n, radii, visibility_filter, max_radii2D, (hipStream_t)stream);
  return check_launch("max_radii_update", (hipStream_t)stream, false);
}

int gs_adam_step(int count, float* const* params, const float* const* grads, float* const* exp_avg,
                 float* const* exp_avg_sq, const long long* sizes, const double* lrs, const int* steps, double beta1,
                 double beta2, double eps, float grad_scale, gs_stream_t stream) {
  GS_REQUIRE(count >= 0, "gs_adam_step: negative count");
  if (count == 0) return 0;
  GS_REQUIRE(params && grads && exp_avg && exp_avg_sq && sizes && lrs && steps, "gs_adam_step: null table");
  for (int i = 0; i < count; i++) {
    if (sizes[i] <= 0) continue;
    GS_REQUIRE(params[i] && grads[i] && exp_avg[i] && exp_avg_sq[i], "gs_adam_step: null tensor pointer");
    GS_REQUIRE(steps[i] >= 1, "gs_adam_step: step numbers start at 1");
  }
  GS_REQUIRE(beta1 >= 0.0 && beta1 < 1.0 && beta2 >= 0.0 && beta2 < 1.0, "gs_adam_step: betas must lie in [0, 1)");
  {
    StageScope _t("adam_step", (hipStream_t)stream);
    launch_adam(count, params, grads, exp_avg, exp_avg_sq, sizes, lrs, steps, beta1, beta2, eps, grad_scale,
                (hipStream_t)stream);
  }
  return check_launch("adam_step", (hipStream_t)stream, false);
}

int gs_neural_supported(int n_offsets) { return neural_supported(n_offsets) ? 1 : 0; }

namespace {
struct NeuralWorkspace {
  size_t packed, counts, scan, total;
};
NeuralWorkspace neural_workspace(int64_t N, int k) {
  NeuralWorkspace L;
  size_t off = 0;
  L.packed = off; off += align_up(neural_packed_floats(k) * sizeof(float), 256);
  L.counts = off; off += align_up((size_t)(N > 0 ? N : 1), 256);
  L.scan = off; off += scan_temp_bytes(N);
  L.total = off;
  return L;
}
}  // namespace

size_t gs_neural_workspace_bytes(int64_t num_anchors, int n_offsets) {
  return neural_workspace(num_anchors, n_offsets).total + 256;
}

int gs_neural_opacity_forward(int64_t N, int k, const float* anchor, const float* feat, const float* campos,
                              const float* const* mlp_params, const float* opacity_scale, const float* level,
                              int input_flags, float* neural_opacity, float* opacity_tanh, uint8_t* mask,
                              uint32_t* first, void* workspace, size_t workspace_bytes, int64_t* num_selected,
                              gs_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  GS_REQUIRE(N >= 0, "gs_neural_opacity_forward: negative anchor count");
  GS_REQUIRE(neural_supported(k), "gs_neural_opacity_forward: n_offsets not among the supported values");
  GS_REQUIRE(num_selected, "gs_neural_opacity_forward: null num_selected");
  *num_selected = 0;
  GS_REQUIRE(N * (int64_t)k < 0x7FFFFFFFll, "gs_neural_opacity_forward: anchors x offsets exceed 2^31-1");
  GS_REQUIRE(mlp_params && campos, "gs_neural_opacity_forward: null pointer");
  GS_REQUIRE(input_flags >= 0 && input_flags < 16, "gs_neural_opacity_forward: input_flags has four bits");
  GS_REQUIRE(!(input_flags & 8) || level || N == 0, "gs_neural_opacity_forward: input_flags asks for the level");
  GS_REQUIRE(!opacity_scale || opacity_tanh || N == 0, "gs_neural_opacity_forward: opacity_scale needs opacity_tanh");
  for (int i = 0; i < 12; i++) GS_REQUIRE(mlp_params[i], "gs_neural_opacity_forward: null MLP parameter");
  GS_REQUIRE(workspace && workspace_bytes >= gs_neural_workspace_bytes(N, k),
             "gs_neural_opacity_forward: workspace missing or too small");
  char* base = align_ptr((char*)workspace, 256);
  const NeuralWorkspace L = neural_workspace(N, k);
  float* packed = (float*)(base + L.packed);
  {
    StageScope _t("neural_pack", stream);
    launch_neural_pack(k, mlp_params, input_flags, packed, stream);
  }
  if (check_launch("neural_pack", stream, false)) return 1;
  if (N == 0) return 0;
  GS_REQUIRE(anchor && feat && neural_opacity && mask && first, "gs_neural_opacity_forward: null pointer");
  uint8_t* counts = (uint8_t*)(base + L.counts);
  {
    StageScope _t("neural_opacity", stream);
    launch_neural_opacity(N, k, anchor, feat, (input_flags & 8) ? level : nullptr, campos, packed, opacity_scale,
                          neural_opacity, opacity_scale ? opacity_tanh : nullptr, mask, counts, stream);
  }
  if (check_launch("neural_opacity", stream, false)) return 1;
  uint32_t* total_slot = acquire_total_slot();
  {
    StageScope _t("neural_scan", stream);
    launch_exclusive_sum_u8(N, counts, first, base + L.scan, stream, total_slot);
  }
  if (check_launch("neural_scan", stream, false)) return 1;
  uint32_t total = 0;
  if (total_slot != nullptr) {
    if (wait_for_total(total_slot, stream, &total)) return 1;
  } else {
    uint32_t last_first = 0;
    uint8_t last_count = 0;
    GS_HIP_TRY(hipMemcpyAsync(&last_first, first + (N - 1), sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
    GS_HIP_TRY(hipMemcpyAsync(&last_count, counts + (N - 1), 1, hipMemcpyDeviceToHost, stream));
    GS_HIP_TRY(hipStreamSynchronize(stream));
    total = last_first + last_count;
  }
  *num_selected = (int64_t)total;
  return 0;
}

int gs_neural_gaussians_forward(int64_t N, int k, int64_t S, const float* anchor, const float* feat,
                                const float* offsets, const float* scaling, const float* campos, const float* level,
                                const float* neural_opacity, const uint32_t* first, const void* workspace,
                                size_t workspace_bytes, float* xyz, float* color, float* opacity, float* scaling_out,
                                float* rot, float* aux, gs_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  GS_REQUIRE(N >= 0 && S >= 0, "gs_neural_gaussians_forward: negative size");
  GS_REQUIRE(neural_supported(k), "gs_neural_gaussians_forward: n_offsets not among the supported values");
  if (N == 0 || S == 0) return 0;
  GS_REQUIRE(S <= N * (int64_t)k, "gs_neural_gaussians_forward: more selected Gaussians than offsets");
  GS_REQUIRE(anchor && feat && offsets && scaling && campos && neural_opacity && first,
             "gs_neural_gaussians_forward: null input");
  GS_REQUIRE(xyz && color && opacity && scaling_out && rot && aux, "gs_neural_gaussians_forward: null output");
  GS_REQUIRE(((uintptr_t)rot & 15) == 0 && ((uintptr_t)aux & 15) == 0 && ((uintptr_t)feat & 15) == 0,
             "gs_neural_gaussians_forward: feat, rot and aux must be 16-byte aligned");
  GS_REQUIRE(workspace && workspace_bytes >= gs_neural_workspace_bytes(N, k),
             "gs_neural_gaussians_forward: workspace missing or too small");
  const float* packed = (const float*)(align_ptr((const char*)workspace, 256) + neural_workspace(N, k).packed);
  {
    StageScope _t("neural_gaussians", stream);
    launch_neural_gaussians(N, k, anchor, feat, level, offsets, scaling, campos, packed, neural_opacity, first, xyz,
                            color, opacity, scaling_out, rot, aux, stream);
  }
  return check_launch("neural_gaussians", stream, false);
}

size_t gs_neural_backward_workspace_bytes(int64_t num_anchors, int n_offsets) {
  const int64_t n = num_anchors > 0 ? num_anchors : 1;
  return align_up(neural_packed_floats(n_offsets) * sizeof(float), 256) +
         align_up(neural_slot_grad_floats(n_offsets, n) * sizeof(float), 256) +
         align_up(neural_partial_floats(n_offsets, n) * sizeof(float), 256) + 256;
}

int gs_neural_backward(int64_t N, int k, int64_t S, const float* anchor, const float* feat, const float* offsets,
                       const float* scaling, const float* campos, const float* const* mlp_params,
                       const float* opacity_scale, const float* level, int input_flags,
                       const float* neural_opacity, const float* opacity_tanh, const uint32_t* first,
                       const float* color, const float* rot,
                       const float* aux, const float* dL_dxyz, const float* dL_dcolor, const float* dL_dopacity,
                       const float* dL_dscaling, const float* dL_drot, float* d_anchor, float* d_feat,
                       float* d_offsets, float* d_scaling, float* const* d_mlp_params, void* workspace,
                       size_t workspace_bytes, gs_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  GS_REQUIRE(N >= 0 && S >= 0, "gs_neural_backward: negative size");
  GS_REQUIRE(neural_supported(k), "gs_neural_backward: n_offsets not among the supported values");
  GS_REQUIRE(mlp_params && d_mlp_params && campos, "gs_neural_backward: null pointer");
  GS_REQUIRE(input_flags >= 0 && input_flags < 16, "gs_neural_backward: input_flags has four bits");
  GS_REQUIRE(!(input_flags & 8) || level || N == 0, "gs_neural_backward: input_flags asks for the level");
  GS_REQUIRE(!opacity_scale || opacity_tanh || N == 0, "gs_neural_backward: opacity_scale needs opacity_tanh");
  for (int i = 0; i < 12; i++)
    GS_REQUIRE(mlp_params[i] && d_mlp_params[i], "gs_neural_backward: null MLP parameter or gradient");
  if (N == 0) {
    // no anchors: the weight gradients are zero
    for (int i = 0; i < 12; i++) {
      const int m = i / 4;
      const size_t sizes[4] = {(size_t)32 * (35 + ((input_flags >> m) & 1) + ((input_flags >> 3) & 1)), 32, 0, 0};
      const int out = (m == 0 ? 1 : m == 1 ? 3 : 7) * k;
      const size_t n = i % 4 == 2 ? (size_t)out * 32 : i % 4 == 3 ? (size_t)out : sizes[i % 4];
      GS_HIP_TRY(hipMemsetAsync(d_mlp_params[i], 0, n * sizeof(float), stream));
    }
    return 0;
  }
  GS_REQUIRE(S <= N * (int64_t)k, "gs_neural_backward: more selected Gaussians than offsets");
  GS_REQUIRE(anchor && feat && offsets && scaling && neural_opacity && first, "gs_neural_backward: null input");
  GS_REQUIRE(S == 0 || (color && rot && aux && dL_dxyz && dL_dcolor && dL_dopacity && dL_dscaling && dL_drot),
             "gs_neural_backward: null saved output or upstream gradient");
  GS_REQUIRE(d_anchor && d_feat && d_offsets && d_scaling, "gs_neural_backward: null gradient output");
  GS_REQUIRE(((uintptr_t)rot & 15) == 0 && ((uintptr_t)aux & 15) == 0 && ((uintptr_t)feat & 15) == 0 &&
                 ((uintptr_t)dL_drot & 15) == 0 && ((uintptr_t)d_feat & 15) == 0,
             "gs_neural_backward: feat, rot, aux, dL_drot and d_feat must be 16-byte aligned");
  GS_REQUIRE(workspace && workspace_bytes >= gs_neural_backward_workspace_bytes(N, k),
             "gs_neural_backward: workspace missing or too small");
  char* base = align_ptr((char*)workspace, 256);
  float* packed = (float*)base;
  float* slot_grads = (float*)(base + align_up(neural_packed_floats(k) * sizeof(float), 256));
  float* partials = (float*)((char*)slot_grads + align_up(neural_slot_grad_floats(k, N) * sizeof(float), 256));
  {
    StageScope _t("neural_pack", stream);
    launch_neural_pack(k, mlp_params, input_flags, packed, stream);
  }
  if (check_launch("neural_pack", stream, false)) return 1;
  {
    StageScope _t("neural_backward", stream);
    launch_neural_backward(N, k, anchor, feat, (input_flags & 8) ? level : nullptr, input_flags, offsets, scaling,
                           campos, packed, neural_opacity, opacity_scale, opacity_tanh, first, color, rot, aux, dL_dxyz, dL_dcolor,
                           dL_dopacity, dL_dscaling, dL_drot, d_anchor, d_feat, d_offsets, d_scaling, d_mlp_params,
                           slot_grads, partials, stream);
  }
  return check_launch("neural_backward", stream, false);
}

int gs_all_map_forward(int P, const float* means3D, const float* scales, const float* rotations,
                       const float* viewmatrix, const float* campos, float* all_map, gs_stream_t stream) {
  GS_REQUIRE(P >= 0, "gs_all_map_forward: negative P");
  if (P == 0) return 0;
  GS_REQUIRE(means3D && scales && rotations && viewmatrix && campos && all_map, "gs_all_map_forward: null pointer");
  {
    StageScope _t("all_map_fwd", (hipStream_t)stream);
    launch_all_map_fwd(P, means3D, scales, rotations, viewmatrix, campos, all_map, (hipStream_t)stream);
  }
  return check_launch("all_map_forward", (hipStream_t)stream, false);
}

int gs_all_map_backward(int P, const float* means3D, const float* scales, const float* rotations,
                        const float* viewmatrix, const float* campos, const float* dL_dall_map,
                        float* dL_dmeans3D, float* dL_drotations, gs_stream_t stream) {
  GS_REQUIRE(P >= 0, "gs_all_map_backward: negative P");
  if (P == 0) return 0;
  GS_REQUIRE(means3D && scales && rotations && viewmatrix && campos && dL_dall_map && dL_dmeans3D && dL_drotations,
             "gs_all_map_backward: null pointer");
  {
    StageScope _t("all_map_bwd", (hipStream_t)stream);
    launch_all_map_bwd(P, means3D, scales, rotations, viewmatrix, campos, dL_dall_map, dL_dmeans3D, dL_drotations,
                       (hipStream_t)stream);
  }
  return check_launch("all_map_backward", (hipStream_t)stream, false);
}

int gs_knn_dist2(int P, const float* points, float* mean_dists, void* workspace, size_t workspace_bytes,
                 gs_stream_t stream) {
  GS_REQUIRE(P >= 0, "gs_knn_dist2: negative P");
  if (pending_fault("gs_knn_dist2")) return 1;
  if (P == 0) return 0;
  GS_REQUIRE(points && mean_dists && workspace, "gs_knn_dist2: null pointer");
  GS_REQUIRE(workspace_bytes >= gs_knn_workspace_bytes(P), "gs_knn_dist2: workspace too small");
  {
    StageScope _t("knn_dist2", (hipStream_t)stream);
    if (launch_knn_dist2(P, points, mean_dists, align_ptr((char*)workspace, 256), fault_word(), (hipStream_t)stream))
      return 1;
  }
  return check_launch("knn_dist2", (hipStream_t)stream, false);
}

// ------------------------------------------------------------ stage level --

int gs_tile_count(int P, int width, int height, const int* radii, const float* means2D,
                  const uint8_t* compute_locally, uint32_t* tiles_touched, gs_stream_t stream) {
  GS_REQUIRE(P >= 0 && width > 0 && height > 0, "gs_tile_count: bad sizes");
  if (P == 0) return 0;
  GS_REQUIRE(radii && means2D && compute_locally && tiles_touched, "gs_tile_count: null pointer");
  launch_tile_count(P, width, height, radii, means2D, compute_locally, tiles_touched, (hipStream_t)stream);
  return check_launch("tile_count", (hipStream_t)stream, false);
}

size_t gs_scan_workspace_bytes(int64_t n) { return scan_temp_bytes(n) + 256; }

int gs_inclusive_sum(int64_t n, const uint32_t* in, uint32_t* out, void* workspace, size_t workspace_bytes,
                     gs_stream_t stream) {
  GS_REQUIRE(n >= 0, "gs_inclusive_sum: negative n");
  if (n == 0) return 0;
  GS_REQUIRE(in && out && workspace, "gs_inclusive_sum: null pointer");
  GS_REQUIRE(workspace_bytes >= gs_scan_workspace_bytes(n), "gs_inclusive_sum: workspace too small");
  launch_inclusive_sum(n, in, out, align_ptr((char*)workspace, 256), (hipStream_t)stream);
  return check_launch("inclusive_sum", (hipStream_t)stream, false);
}

int64_t gs_inclusive_sum_static_max(void) { return static_scan_max_elements(); }

int gs_inclusive_sum_static(int64_t n, const uint32_t* in, uint32_t* out, gs_stream_t stream) {
  GS_REQUIRE(n >= 0, "gs_inclusive_sum_static: negative n");
  if (n == 0) return 0;
  GS_REQUIRE(in && out, "gs_inclusive_sum_static: null pointer");
  if (launch_inclusive_sum_static(n, in, out, (hipStream_t)stream)) return 1;
  return check_launch("inclusive_sum_static", (hipStream_t)stream, false);
}

int gs_duplicate_with_keys(int P, int width, int height, const float* means2D, const float* depths,
                           const uint32_t* offsets, const int* radii, const uint8_t* compute_locally, uint64_t* keys,
                           uint32_t* values, gs_stream_t stream) {
  GS_REQUIRE(P >= 0 && width > 0 && height > 0, "gs_duplicate_with_keys: bad sizes");
  if (P == 0) return 0;
  GS_REQUIRE(means2D && depths && offsets && radii && compute_locally && keys && values,
             "gs_duplicate_with_keys: null pointer");
  launch_duplicate_with_keys(P, width, height, means2D, depths, offsets, radii, compute_locally, keys, values, nullptr,
                             (hipStream_t)stream);
  return check_launch("duplicate_with_keys", (hipStream_t)stream, false);
}

size_t gs_sort_workspace_bytes(int64_t n) { return sort_temp_bytes(n) + 256; }

int64_t gs_sort_max_pairs(void) { return sort_max_pairs(); }

int gs_sort_pairs_u64(int64_t n, uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out,
                      int end_bit, void* workspace, size_t workspace_bytes, gs_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  GS_REQUIRE(n >= 0 && end_bit >= 1 && end_bit <= 64, "gs_sort_pairs_u64: bad n or end_bit");
  GS_REQUIRE(n <= sort_max_pairs(), "gs_sort_pairs_u64: more than 2^30-2 pairs");
  if (n == 0) return 0;
  GS_REQUIRE(keys_in && keys_out && vals_in && vals_out && workspace, "gs_sort_pairs_u64: null pointer");
  GS_REQUIRE(workspace_bytes >= gs_sort_workspace_bytes(n), "gs_sort_pairs_u64: workspace too small");
  void* temp = align_ptr((char*)workspace, 256);
  StageScope _t("sort_pairs", stream);
  if (sort_result_in_b(end_bit)) {
    if (launch_sort_pairs_u64(n, keys_in, keys_out, vals_in, vals_out, end_bit, temp, stream)) return 1;
  } else {
    GS_HIP_TRY(hipMemcpyAsync(keys_out, keys_in, (size_t)n * 8, hipMemcpyDeviceToDevice, stream));
    GS_HIP_TRY(hipMemcpyAsync(vals_out, vals_in, (size_t)n * 4, hipMemcpyDeviceToDevice, stream));
    if (launch_sort_pairs_u64(n, keys_out, keys_in, vals_out, vals_in, end_bit, temp, stream)) return 1;
  }
  return check_launch("sort_pairs_u64", stream, false);
}

int gs_sort_status(const void* workspace, gs_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  GS_REQUIRE(workspace, "gs_sort_status: null workspace");
  const void* temp = align_ptr((const char*)workspace, 256);
  uint32_t word = 0;
  GS_HIP_TRY(hipMemcpyAsync(&word, sort_error_word(temp), sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
  GS_HIP_TRY(hipStreamSynchronize(stream));
  if (word != 0u) {
    set_error("radix sort: a bounded wait on an earlier tile's digit counts ran out; the output is not sorted");
    return 1;
  }
  return 0;
}

size_t gs_sort_workspace_error_offset(void) { return sort_error_word_offset(); }

int gs_sort_check_async(const void* workspace, gs_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  GS_REQUIRE(workspace, "gs_sort_check_async: null workspace");
  uint32_t* fw = fault_word();
  GS_REQUIRE(fw, "gs_sort_check_async: no pinned host memory for the fault word");
  launch_sort_fault_report(sort_error_word(align_ptr((const char*)workspace, 256)), fw, stream);
  return check_launch("sort_check_async", stream, false);
}

int gs_sort_pairs_u32(int64_t n, uint32_t* keys_in, uint32_t* keys_out, uint32_t* vals_in, uint32_t* vals_out,
                      int end_bit, void* workspace, size_t workspace_bytes, gs_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  GS_REQUIRE(n >= 0 && end_bit >= 1 && end_bit <= 32, "gs_sort_pairs_u32: bad n or end_bit");
  GS_REQUIRE(n <= sort_max_pairs(), "gs_sort_pairs_u32: more than 2^30-2 pairs");
  if (n == 0) return 0;
  GS_REQUIRE(keys_in && keys_out && vals_in && vals_out && workspace, "gs_sort_pairs_u32: null pointer");
  GS_REQUIRE(workspace_bytes >= gs_sort_workspace_bytes(n), "gs_sort_pairs_u32: workspace too small");
  void* temp = align_ptr((char*)workspace, 256);
  if (sort_result_in_b(end_bit)) {
    if (launch_sort_pairs_u32(n, keys_in, keys_out, vals_in, vals_out, end_bit, temp, stream)) return 1;
  } else {
    GS_HIP_TRY(hipMemcpyAsync(keys_out, keys_in, (size_t)n * 4, hipMemcpyDeviceToDevice, stream));
    GS_HIP_TRY(hipMemcpyAsync(vals_out, vals_in, (size_t)n * 4, hipMemcpyDeviceToDevice, stream));
    if (launch_sort_pairs_u32(n, keys_out, keys_in, vals_out, vals_in, end_bit, temp, stream)) return 1;
  }
  return check_launch("sort_pairs_u32", stream, false);
}

int gs_identify_tile_ranges(int64_t L, const uint64_t* keys_sorted, int tiles, uint32_t* ranges, gs_stream_t stream) {
  GS_REQUIRE(L >= 0 && tiles > 0 && ranges && (L == 0 || keys_sorted), "gs_identify_tile_ranges: bad arguments");
  launch_tile_ranges(L, keys_sorted, tiles, ranges, (hipStream_t)stream);
  return check_launch("identify_tile_ranges", (hipStream_t)stream, false);
}

int gs_render_tiles_forward(int P, int width, int height, float focal_x, float focal_y, float cx, float cy,
                            const uint32_t* ranges, const uint32_t* point_list, const float* means2D,
                            const float* rgb, const float* all_map, const float* conic_opacity,
                            const uint8_t* compute_locally, const float* background, int render_geo, float* final_T,
                            uint32_t* n_contrib_px, uint32_t* n_contrib2loss_px, float* out_color, int* out_observe,
                            float* out_all_map, float* out_plane_depth, int* n_render, int* n_consider,
                            int* n_contrib, gs_stream_t stream) {
  GS_REQUIRE(P > 0 && width > 0 && height > 0, "gs_render_tiles_forward: bad sizes");
  GS_REQUIRE(ranges && point_list && means2D && rgb && conic_opacity && compute_locally && background && final_T &&
                 n_contrib_px && n_contrib2loss_px && out_color && out_observe && n_render && n_consider && n_contrib,
             "gs_render_tiles_forward: null pointer");
  GS_REQUIRE(!render_geo || (all_map && out_all_map && out_plane_depth),
             "gs_render_tiles_forward: render_geo needs all_map, out_all_map and out_plane_depth");
  RenderFwdArgs a;
  a.P = P; a.W = width; a.H = height;
  a.fx = focal_x; a.fy = focal_y; a.cx = cx; a.cy = cy;
  a.ranges = ranges; a.point_list = point_list;
  a.means2D = means2D; a.rgb = rgb; a.all_map = all_map; a.conic_opacity = conic_opacity;
  a.compute_locally = compute_locally; a.bg = background; a.render_geo = render_geo;
  a.final_T = final_T; a.n_contrib_px = n_contrib_px; a.n_contrib2loss_px = n_contrib2loss_px;
  a.out_color = out_color; a.out_observe = out_observe; a.out_all_map = out_all_map;
  a.out_plane_depth = out_plane_depth;
  a.n_render = n_render; a.n_consider = n_consider; a.n_contrib_tile = n_contrib;
  launch_render_fwd(a, (hipStream_t)stream);
  return check_launch("render_tiles_forward", (hipStream_t)stream, false);
}

int gs_render_tiles_backward(int P, int width, int height, float tan_fovx, float tan_fovy, const float* background,
                             const uint32_t* ranges, const uint32_t* point_list, const float* means2D,
                             const float* conic_opacity, const float* rgb, const float* all_maps,
                             const float* all_map_pixels, const float* final_T, const uint32_t* n_contrib_px,
                             const uint8_t* compute_locally, const float* dL_dpix, const float* dL_dout_all_map,
                             const float* dL_dout_plane_depth, int render_geo, const uint32_t* emission_sorted,
                             const uint32_t* point_offsets, float* instance_grads, float* dL_dmean2D,
                             float* dL_dmean2D_abs, float* dL_dconic_opacity, float* dL_dcolor, float* dL_dall_map,
                             gs_stream_t stream) {
  GS_REQUIRE(P > 0 && width > 0 && height > 0, "gs_render_tiles_backward: bad sizes");
  GS_REQUIRE(background && ranges && point_list && means2D && conic_opacity && rgb && final_T && n_contrib_px &&
                 compute_locally && dL_dpix && dL_dmean2D && dL_dmean2D_abs && dL_dconic_opacity && dL_dcolor &&
                 emission_sorted && point_offsets && instance_grads,
             "gs_render_tiles_backward: null pointer");
  GS_REQUIRE(!render_geo || (dL_dout_all_map && dL_dout_plane_depth && dL_dall_map && all_maps && all_map_pixels),
             "gs_render_tiles_backward: render_geo needs the geometry-map tensors");
  RenderBwdArgs a;
  a.P = P; a.W = width; a.H = height;
  a.fy = height / (2.0f * tan_fovy);
  a.fx = width / (2.0f * tan_fovx);
  a.bg = background; a.ranges = ranges; a.point_list = point_list;
  a.means2D = means2D; a.conic_opacity = conic_opacity; a.rgb = rgb; a.all_map = all_maps;
  a.all_map_pixels = all_map_pixels; a.final_T = final_T; a.n_contrib_px = n_contrib_px;
  a.compute_locally = compute_locally;
  a.dL_dpix = dL_dpix; a.dL_dout_all_map = dL_dout_all_map; a.dL_dout_plane_depth = dL_dout_plane_depth;
  a.render_geo = render_geo;
  a.emission_sorted = emission_sorted; a.point_offsets = point_offsets; a.instance_grads = instance_grads;
  a.dL_dmean2D = dL_dmean2D; a.dL_dmean2D_abs = dL_dmean2D_abs; a.dL_dconic_opacity = dL_dconic_opacity;
  a.dL_dcolors = dL_dcolor; a.dL_dall_map = dL_dall_map;
  launch_render_bwd(a, (hipStream_t)stream);
  return check_launch("render_tiles_backward", (hipStream_t)stream, false);
}

int gs_selftest_reductions(const float* in, float* out_wave, float* out_rows, gs_stream_t stream) {
  GS_REQUIRE(in && out_wave && out_rows, "gs_selftest_reductions: null pointer");
  launch_reduce_selftest(in, out_wave, out_rows, (hipStream_t)stream);
  return check_launch("selftest_reductions", (hipStream_t)stream, true);
}

int gs_stage_timing_enable(int enable) {
  g_clock.enabled.store(enable != 0);
  return 0;
}

int gs_stage_timing_collect(char* report, size_t report_bytes) {
  GS_REQUIRE(report && report_bytes > 0, "gs_stage_timing_collect: null report buffer");
  std::vector<StageClock::Rec> recs;
  {
    std::lock_guard<std::mutex> lock(g_clock.mutex);
    recs.swap(g_clock.done);
  }
  std::map<std::string, std::pair<double, long>> acc;
  std::vector<std::string> order;
  int failed = 0;
  for (auto& r : recs) {
    float ms = 0.f;
    if (hipEventSynchronize(r.b) == hipSuccess && hipEventElapsedTime(&ms, r.a, r.b) == hipSuccess) {
      if (!acc.count(r.name)) order.push_back(r.name);
      acc[r.name].first += ms;
      acc[r.name].second += 1;
    } else {
      (void)hipGetLastError();
      failed++;
    }
    g_clock.give_back(r.a);
    g_clock.give_back(r.b);
  }
  size_t used = 0;
  report[0] = 0;
  for (auto& name : order) {
    const int w = snprintf(report + used, report_bytes - used, "%s %.6f %ld\n", name.c_str(), acc[name].first,
                           acc[name].second);
    if (w < 0 || (size_t)w >= report_bytes - used) break;
    used += (size_t)w;
  }
  if (failed) {
    set_error("gs_stage_timing_collect: %d event pairs could not be read", failed);
    return 1;
  }
  return 0;
}

int gs_image_state_layout(int width, int height, size_t* accum_alpha, size_t* n_contrib, size_t* n_contrib2loss,
                          size_t* ranges, size_t* total_bytes) {
  GS_REQUIRE(width > 0 && height > 0, "gs_image_state_layout: bad sizes");
  const ImageLayout L = image_layout(width, height);
  if (accum_alpha) *accum_alpha = L.accum_alpha;
  if (n_contrib) *n_contrib = L.n_contrib;
  if (n_contrib2loss) *n_contrib2loss = L.n_contrib2loss;
  if (ranges) *ranges = L.ranges;
  if (total_bytes) *total_bytes = L.total;
  return 0;
}

int gs_binning_state_layout(int64_t R, int width, int height, size_t* point_list, size_t* point_list_keys,
                            size_t* point_list_unsorted, size_t* point_list_keys_unsorted, size_t* total_bytes) {
  (void)width;
  (void)height;
  GS_REQUIRE(R >= 0, "gs_binning_state_layout: negative R");
  const BinningLayout L = binning_layout(R);
  if (point_list) *point_list = L.point_list;
  if (point_list_keys) *point_list_keys = L.keys;
  if (point_list_unsorted) *point_list_unsorted = L.point_list_unsorted;
  if (point_list_keys_unsorted) *point_list_keys_unsorted = L.keys_unsorted;
  if (total_bytes) *total_bytes = L.total;
  return 0;
}

int gs_geometry_state_layout(int P, size_t* tiles_touched, size_t* point_offsets, size_t* total_bytes) {
  GS_REQUIRE(P >= 0, "gs_geometry_state_layout: negative P");
  const GeometryLayout L = geometry_layout(P);
  if (tiles_touched) *tiles_touched = L.tiles_touched;
  if (point_offsets) *point_offsets = L.point_offsets;
  if (total_bytes) *total_bytes = L.total;
  return 0;
}

}  // extern "C"
