// C ABI of the MXFP6 GEMM library (declared in include/mxfp6_gemm.h): argument validation and
// kernel selection.  Nothing here synchronises the device.  Allocations, all from the stream-ordered allocator on the
// caller's stream and all kept per (device, stream) until mxfp6_release_workspaces(): the workspace of the re-layout
// pre-pass (relayout_then_tiled; mxfp6_set_relayout(0) switches it off), the fp32 workspace of mxfp6_gemm_fused_fp6
// on shapes the tiled kernel does not run, the partial sums of the tiled and the block kernel's K split (plan_ksplit,
// plan_block_ksplit: one workspace, shared), and the K-split workspace of the skinny kernel (gemm_skinny.hip).  mxfp6_gemm_noalloc allocates nothing.
#include "../../include/mxfp6_gemm.h"
#ifdef MXFP6_PROBES
#include "../../include/mxfp6_probes.h"
#endif

#include <map>
#include <mutex>
#include <tuple>
#include <utility>

#include "kernels.hpp"

namespace {

// Overrides for measurement and tests: per thread, so that a thread that forces a kernel does not change what
// other threads' calls run.
thread_local int g_force = 0;
thread_local int g_relayout = 1;
thread_local int g_allow_e3m2_pair = 0;  // mxfp6_allow_e3m2_pair
thread_local int g_ksplit = 0;  // mxfp6_set_k_split: 0 = where it pays, -1 = wherever possible, 1 = never, n = n shares per output tile
#ifdef MXFP6_PROBES  // the measurement build (libmxfp6_probes.so, include/mxfp6_probes.h)
thread_local uint32_t* g_clock_stamps = nullptr;  // mxfp6_probe_tiled_clock
thread_local int g_raster_group_m = 0, g_raster_no_xcd = 0;  // mxfp6_probe_raster
thread_local int g_ablation = 0;                              // mxfp6_probe_tiled_ablation
thread_local int g_block = 1;                                 // mxfp6_probe_block: 0 keeps the block kernel out of the automatic choice
#else
constexpr int g_block = 1;
#endif

// Workspaces kept per (device, stream, kind): launches on one stream are ordered, so they can share one; it grows on
// demand (old one returned to the allocator in stream order) and lives until mxfp6_release_workspaces().
// A workspace that was handed out while its stream was being captured is recorded in a graph: it is `pinned`, and a
// pinned block is never freed again -- when it must grow, or at mxfp6_release_workspaces(), it is retired (kept
// allocated until the process ends), so that replays of the graph never write into memory somebody else owns.
struct StreamWs {
  uint8_t* p = nullptr;
  size_t bytes = 0;
  bool pinned = false;
  uint64_t used = 0;  // g_sws_clock at the last use (least recently used entries make room when the table is full)
};
std::mutex g_sws_mutex;
// Held while a call enqueues the kernels that write and then read a stream's workspace (pre-pass + GEMM, GEMM + quantiser):
// two threads that launch into the same stream must not interleave those, or one's GEMM would read the other's copies.
std::recursive_mutex g_sws_launch_mutex;
std::map<std::tuple<int, hipStream_t, int>, StreamWs> g_sws;
uint64_t g_sws_clock = 0;
constexpr size_t kStreamWsMax = 128;

bool stream_is_capturing(hipStream_t s) {
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &cap) != hipSuccess) {
    (void)hipGetLastError();
    return true;  // unknown: behave as if it were
  }
  return cap != hipStreamCaptureStatusNone;
}

// kind 0: pre-pass copies, kind 1: fp32 result of mxfp6_gemm_fused_fp6, kind 2: partial sums of a K split, kind 3: arrival
// counters of the ring kernel's K split (zeroed when allocated; the kernels leave them zero).
// nullptr: no workspace (capture without one, table full of pinned entries, out of memory).
uint8_t* stream_workspace(hipStream_t s, int kind, size_t bytes, bool zeroed = false) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(g_sws_mutex);
  const bool capturing = stream_is_capturing(s);
  auto it = g_sws.find({dev, s, kind});
  if (it != g_sws.end() && it->second.bytes >= bytes) {
    it->second.used = ++g_sws_clock;
    if (capturing) it->second.pinned = true;  // a graph now holds this pointer
    return it->second.p;
  }
  // never allocate into a stream that is being captured: the caller replays the graph with its own memory plan
  if (capturing) return nullptr;
  if (it == g_sws.end() && g_sws.size() >= kStreamWsMax) {
    // full: the least recently used workspace that no graph holds goes back to the allocator, in its own stream's order
    auto victim = g_sws.end();
    for (auto j = g_sws.begin(); j != g_sws.end(); ++j)
      if (!j->second.pinned && (victim == g_sws.end() || j->second.used < victim->second.used)) victim = j;
    if (victim == g_sws.end()) return nullptr;
    int cur = dev;
    (void)hipSetDevice(std::get<0>(victim->first));
    if (hipFreeAsync(victim->second.p, std::get<1>(victim->first)) != hipSuccess) (void)hipGetLastError();  // a destroyed stream: the block is lost to the pool
    (void)hipSetDevice(cur);
    g_sws.erase(victim);
  }
  uint8_t* p = nullptr;
  const size_t want = (bytes + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
  if (hipMallocAsync((void**)&p, want, s) != hipSuccess || !p) {
    (void)hipGetLastError();
    return nullptr;
  }
  if (zeroed && mxfp6::launch_fill_zero(p, want, s) != hipSuccess) {
    (void)hipFreeAsync(p, s);
    return nullptr;
  }
  if (it != g_sws.end()) {
    if (!it->second.pinned) (void)hipFreeAsync(it->second.p, s);  // a pinned block stays allocated: a graph may replay into it
    it->second = {p, want, false, ++g_sws_clock};
  } else {
    g_sws[{dev, s, kind}] = {p, want, false, ++g_sws_clock};
  }
  return p;
}

// Candidate sets of the kernel choice (bits of mxfp6::Candidate)
constexpr unsigned kTiledUnsplit = 1u << mxfp6::kCandTiled256 | 1u << mxfp6::kCandTiled128x256 | 1u << mxfp6::kCandTiled128x128;
constexpr unsigned kTiledSplits = 1u << mxfp6::kCandTiledSplit256 | 1u << mxfp6::kCandTiledSplit128;
constexpr unsigned kTiledFamily = kTiledUnsplit | kTiledSplits;
constexpr unsigned kBlockFamily = 1u << mxfp6::kCandBlock | 1u << mxfp6::kCandBlockSplit;
constexpr unsigned kBlockAll = kBlockFamily | 1u << mxfp6::kCandBlockWide;
constexpr unsigned kNeedsWorkspace = kTiledSplits | 1u << mxfp6::kCandBlockSplit;

// Codes mxfp6_kernel_choice reports (those of mxfp6_set_kernel; 25 / 27: the tiled / the block kernel with its K split)
constexpr int kChoiceGeneric = 1, kChoiceTiled = 2, kChoiceSkinny = 3, kChoiceBlock = 22, kChoiceTiledKsplit = 25, kChoiceBlockWide = 26, kChoiceBlockKsplit = 27, kChoiceRing = 28;
int choice_code(const mxfp6::KernelChoice& c) {
  switch (c.cand) {
    case mxfp6::kCandTiled256: case mxfp6::kCandTiled128x256: case mxfp6::kCandTiled128x128: return kChoiceTiled;
    case mxfp6::kCandBlock: return kChoiceBlock;
    case mxfp6::kCandBlockWide: return kChoiceBlockWide;
    case mxfp6::kCandSkinny: return kChoiceSkinny;
    case mxfp6::kCandTiledSplit256: case mxfp6::kCandTiledSplit128: return kChoiceTiledKsplit;
    case mxfp6::kCandBlockSplit: return kChoiceBlockKsplit;
    case mxfp6::kCandRing: return kChoiceRing;
    default: return kChoiceGeneric;
  }
}

// What the automatic path may choose from for a call.  force_split: the entry point that allocates nothing fixes the skinny
// kernel's split (1 = never split): no kernel that needs a workspace, and the skinny kernel whenever a split is asked for.
unsigned auto_mask(const mxfp6::GemmArgs& g, int force_split) {
  unsigned mask = ~0u;
  if (!g_block || force_split) mask &= ~kBlockAll;
  if (force_split || g.no_alloc) mask &= ~(kNeedsWorkspace | 1u << mxfp6::kCandRing);
  if (force_split > 1 && mxfp6::gemm_skinny_supports(g)) mask = 1u << mxfp6::kCandSkinny;
  return mask;
}

// The choice for a call: by the time model and the calibration table (dispatch.hip).  allow_split = false: what it is when a
// K split's workspace is not to be had (a stream that is being captured, the allocator's refusal).
mxfp6::KernelChoice auto_choice(const mxfp6::GemmArgs& g, int force_split, bool allow_split) {
  if (g.K == 0) return {-1, 1, 0, 0.0};  // act(bias) everywhere: the generic kernel's K loop runs zero times
  return mxfp6::choose_kernel(g, g_ksplit, allow_split, auto_mask(g, force_split));
}

// Sets a call up as the choice says: tile shape, K split and its workspace.  false: the split's workspace is not to be had.
bool apply_choice(mxfp6::GemmArgs& g, const mxfp6::KernelChoice& c, hipStream_t s) {
  switch (c.cand) {
    case mxfp6::kCandTiled256: g.tile_rows = 256, g.tile_cols = 256; return true;
    case mxfp6::kCandTiled128x256: g.tile_rows = 128, g.tile_cols = 256; return true;
    case mxfp6::kCandTiled128x128: g.tile_rows = 128, g.tile_cols = 128; return true;
    case mxfp6::kCandBlockWide: g.tile_cols = 256; return true;
    case mxfp6::kCandTiledSplit256: case mxfp6::kCandTiledSplit128: case mxfp6::kCandBlockSplit: {
      uint8_t* pp = stream_workspace(s, 2, (size_t)c.shares * g.M * g.N * sizeof(float));
      if (!pp) return false;
      g.ksplit = c.shares, g.ks_part = reinterpret_cast<float*>(pp);
      if (c.cand != mxfp6::kCandBlockSplit) g.tile_rows = c.rows, g.tile_cols = 256;
      return true;
    }
    case mxfp6::kCandRing: {
      if (c.shares <= 1) return true;
      size_t part = 0, counters = 0;
      if (mxfp6::ring_ksplit_plan(g, c.shares, &part, &counters) != c.shares) return false;
      uint8_t* pp = stream_workspace(s, 2, part);
      uint8_t* pc = pp ? stream_workspace(s, 3, counters * sizeof(int), true) : nullptr;
      if (!pc) return false;
      g.ksplit = c.shares, g.ks_part = reinterpret_cast<float*>(pp), g.ks_counters = reinterpret_cast<int*>(pc);
      return true;
    }
    default: return true;
  }
}

// A forced kernel family with this thread's K-split setting: 0 = the family's split where the model prefers it to the
// family's unsplit form, -1 / n = the split wherever the shape has one, 1 = never.  The tile shape of a forced tiled kernel
// without one (mxfp6_set_kernel 2) is the model's choice as well.
mxfp6::KernelChoice family_choice(const mxfp6::GemmArgs& g, unsigned unsplit, unsigned splits) {
  mxfp6::KernelChoice c = mxfp6::choose_kernel(g, g_ksplit, true, unsplit | (g_ksplit != 1 ? splits : 0u));
  if (g_ksplit != 0 && g_ksplit != 1 && !(splits >> c.cand & 1)) {  // the split is wanted wherever possible
    const mxfp6::KernelChoice forced = mxfp6::choose_kernel(g, g_ksplit, true, splits);
    if (forced.cand >= 0) c = forced;
  }
  return c;
}

hipError_t release_stream_workspaces() {
  std::lock_guard<std::recursive_mutex> launch_lock(g_sws_launch_mutex);
  std::lock_guard<std::mutex> lock(g_sws_mutex);
  if (g_sws.empty()) return hipSuccess;
  int cur = 0;
  (void)hipGetDevice(&cur);
  hipError_t first = hipSuccess;
  for (auto& kv : g_sws) {
    if (kv.second.pinned) continue;  // recorded in a graph: stays allocated until the process ends
    (void)hipSetDevice(std::get<0>(kv.first));
    const hipError_t e = hipFreeAsync(kv.second.p, std::get<1>(kv.first));
    if (e != hipSuccess && first == hipSuccess) first = e;
  }
  g_sws.clear();
  (void)hipSetDevice(cur);
  return first;
}

int check_device() {
  // cached per process: the library only carries gfx950 code objects
  static int cached = [] {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MXFP6_ENODEVICE;
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, dev) != hipSuccess) return MXFP6_ENODEVICE;
    return __builtin_strncmp(p.gcnArchName, "gfx950", 6) == 0 ? MXFP6_OK : MXFP6_ENODEVICE;
  }();
  return cached;
}

// Large row-major problems on the tiled kernel are bound by L2 request throughput: a 96-byte row piece straddles
// 128-byte lines and every row's scales are a request of their own (896 requests per K-tile and workgroup against
// 648 with one operand tile-major and 400 with both).  Re-laying an operand out tile-major first costs two passes
// over it at HBM speed (measured 23 us for 8192 x 8192) and shortens the GEMM by about 15 % (first operand) and
// 11 % (second): from about 8192^3 on that pays for both, for a tall or wide problem only for the operand with
// fewer rows.  The workspace is this stream's (stream_workspace: allocated once, kept).  Returns false when no
// pre-pass pays or it cannot run (then the caller launches the row-major path).
bool relayout_then_tiled(const mxfp6::GemmArgs& g, hipStream_t s, hipError_t& e) {
  if (!g_relayout || g.no_alloc || (g.layout_a && g.layout_b) || g.K % 128) return false;
  const double tiles = (double)((g.M + 255) / 256) * ((g.N + 255) / 256);
  const double t_gemm_us = (tiles > 256 ? tiles / 256 : 1.0) * (g.K / 128) * 1.5;            // row-major tiled kernel
  auto cost_us = [&](int rows) { return (double)rows * g.K * 0.78125 * 2 / 4.9e6; };         // read + write at 4.9 TB/s
  // the operand with fewer rows first (it is the cheaper one to convert; the gain is the same)
  const bool a_first = g.M <= g.N;
  const int rows1 = a_first ? g.M : g.N, rows2 = a_first ? g.N : g.M;
  bool conv1, conv2;
  if (g.layout_a || g.layout_b) {
    // one operand is tile-major already (prepared weights): the other one's copy is the second conversion of the two,
    // worth about 11 % of the row-major GEMM, for one launch in front of it
    const bool first_is_row = a_first ? !g.layout_a : !g.layout_b;
    const int rows = first_is_row ? rows1 : rows2;
    const bool conv = rows % 32 == 0 && 0.11 * t_gemm_us > 6 + cost_us(rows);
    conv1 = first_is_row && conv, conv2 = !first_is_row && conv;
  } else {
    // fixed costs: the dependent launch in front of the GEMM (about 10 us measured on a 33 us GEMM), a second operand about 3 us
    conv1 = rows1 % 32 == 0 && 0.15 * t_gemm_us > 10 + 1.5 * cost_us(rows1);
    conv2 = rows2 % 32 == 0 && (conv1 ? 0.11 * t_gemm_us > 3 + 1.5 * cost_us(rows2) : 0.15 * t_gemm_us > 10 + 1.5 * cost_us(rows2));
  }
  if (!conv1 && !conv2) return false;
  const bool conv_a = a_first ? conv1 : conv2, conv_b = a_first ? conv2 : conv1;
  auto bytes_of = [&](int rows) { return (((size_t)rows * (g.K / 4 * 3) + 255) & ~(size_t)255) + (((size_t)rows * ((g.K + 511) / 512) * 16 + 255) & ~(size_t)255); };
  const size_t bytes_a = conv_a ? bytes_of(g.M) : 0, bytes_b = conv_b ? bytes_of(g.N) : 0;
  std::lock_guard<std::recursive_mutex> launch_lock(g_sws_launch_mutex);
  uint8_t* ws = stream_workspace(s, 0, bytes_a + bytes_b);
  if (!ws) return false;
  mxfp6::GemmArgs t = g;
  uint8_t* pa = ws;
  uint8_t* sa = pa + (((size_t)g.M * (g.K / 4 * 3) + 255) & ~(size_t)255);
  uint8_t* pb = ws + bytes_a;
  uint8_t* sb = pb + (((size_t)g.N * (g.K / 4 * 3) + 255) & ~(size_t)255);
  if (conv_a && conv_b) {
    e = mxfp6::launch_tile_both(g.A, pa, g.As, sa, g.M, g.B, pb, g.Bs, sb, g.N, g.K, s);
  } else if (conv_a) {
    e = mxfp6::launch_tile_both(g.A, pa, g.As, sa, g.M, nullptr, nullptr, nullptr, nullptr, 0, g.K, s);
  } else {
    e = mxfp6::launch_tile_both(g.B, pb, g.Bs, sb, g.N, nullptr, nullptr, nullptr, nullptr, 0, g.K, s);
  }
  if (conv_a) { t.A = pa; t.As = sa; t.layout_a = 1; }
  if (conv_b) { t.B = pb; t.Bs = sb; t.layout_b = 1; }
  if (e == hipSuccess) e = mxfp6::launch_gemm_tiled(t, s);
  return true;
}

// The argument checks shared by the gemm entry points (c_align: alignment mask of C).  *empty: nothing to compute.
int check_gemm_args(const void* A, const void* B, const void* As, const void* Bs, const void* C, int M, int N, int K, int fmt_a, int fmt_b,
                    uintptr_t c_align, int layout_a, int layout_b, const mxfp6::Epilogue& ep, bool* empty) {
  *empty = false;
  if (M < 0 || N < 0 || K < 0 || K % 32 != 0) return MXFP6_EINVAL_SHAPE;
  if ((fmt_a != MXFP6_FMT_E2M3 && fmt_a != MXFP6_FMT_E3M2) || (fmt_b != MXFP6_FMT_E2M3 && fmt_b != MXFP6_FMT_E3M2))
    return MXFP6_EINVAL_FMT;
  // e3m2 on both sides is the one pair whose accumulators can miss the library's accuracy bar (the MFMA's own sum is
  // inexact there): only for callers that have said they accept that
  if (fmt_a == MXFP6_FMT_E3M2 && fmt_b == MXFP6_FMT_E3M2 && !g_allow_e3m2_pair) return MXFP6_EACCURACY;
  if ((layout_a != MXFP6_LAYOUT_ROW && layout_a != MXFP6_LAYOUT_TILE) || (layout_b != MXFP6_LAYOUT_ROW && layout_b != MXFP6_LAYOUT_TILE))
    return MXFP6_EINVAL_LAYOUT;
  if ((layout_a == MXFP6_LAYOUT_TILE && (M % 32 || K % 128)) || (layout_b == MXFP6_LAYOUT_TILE && (N % 32 || K % 128)))
    return MXFP6_EINVAL_SHAPE;
  if (M == 0 || N == 0) {
    *empty = true;
    return MXFP6_OK;
  }
  if (!C) return MXFP6_EINVAL_PTR;
  if (K > 0 && (!A || !B || !As || !Bs)) return MXFP6_EINVAL_PTR;
  if (((uintptr_t)A & 3) || ((uintptr_t)B & 3) || ((uintptr_t)C & c_align)) return MXFP6_EINVAL_ALIGN;
  // the tiled kernel reads four floats (or four bf16) of the per-column vectors at a time
  if (((uintptr_t)ep.col_scale & 15) || ((uintptr_t)ep.row_scale & 3) || ((uintptr_t)ep.bias & (ep.bias_bf16 ? 7 : 15))) return MXFP6_EINVAL_ALIGN;
  if (ep.act < 0 || ep.act > 3) return MXFP6_EINVAL_EPILOGUE;
  if ((long)M * N >= (1L << 40) || (long)K / 4 * 3 * 256 >= (1L << 31)) return MXFP6_EINVAL_SHAPE;
  return MXFP6_OK;
}

int gemm_common(const void* A, const void* B, const void* As, const void* Bs, void* C, int M, int N, int K, int fmt_a,
                int fmt_b, bool f32out, int layout_a, int layout_b, void* stream, const mxfp6::Epilogue& ep = mxfp6::Epilogue(),
                int no_alloc = 0, int force_split = 0) {
  bool empty;
  int rc = check_gemm_args(A, B, As, Bs, C, M, N, K, fmt_a, fmt_b, f32out ? 3 : 1, layout_a, layout_b, ep, &empty);
  if (rc || empty) return rc;
  rc = check_device();
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (K == 0 && !mxfp6::epilogue_any(ep)) {
    hipError_t e = mxfp6::launch_fill_zero(C, (size_t)M * N * (f32out ? 4 : 2), s);
    return e == hipSuccess ? MXFP6_OK : (int)e;
  }
  mxfp6::GemmArgs g{(const uint8_t*)A, (const uint8_t*)B, (const uint8_t*)As, (const uint8_t*)Bs, C, M, N, K, fmt_a, fmt_b, f32out, layout_a, layout_b};
  g.ep = ep;
  g.no_alloc = no_alloc, g.force_split = force_split;
#ifdef MXFP6_PROBES
  g.clock_stamps = g_clock_stamps;
  g.raster_group_m = g_raster_group_m, g.raster_no_xcd_remap = g_raster_no_xcd;
  g.ablation = g_ablation;
#endif
  const int force = no_alloc ? 0 : g_force;  // the entry point that allocates nothing takes no override
  hipError_t e;
  if (no_alloc && force_split > 1 && !(M <= 32 && mxfp6::gemm_skinny_supports(g))) return MXFP6_EINVAL_SHAPE;
  if (no_alloc && mxfp6::gemm_skinny_supports(g) && (force_split || auto_choice(g, force_split, false).cand == mxfp6::kCandSkinny) && !mxfp6::gemm_skinny_scratch_fits(g)) return MXFP6_ESCRATCH;
  std::lock_guard<std::recursive_mutex> launch_lock(g_sws_launch_mutex);  // a K split writes and then reads this stream's workspace
  if (K != 0 && force == 1) {
    e = mxfp6::launch_gemm_generic(g, s);
  } else if (K != 0 && (force == 2 || force == 5 || force == 6 || force == 17)) {
    if (!mxfp6::gemm_tiled_supports(g)) return MXFP6_EINVAL_SHAPE;
    g.tile_rows = force == 5 || force == 17 ? 128 : force == 6 ? 256 : 0, g.tile_cols = force == 17 ? 128 : 0;
    const unsigned shapes = force == 2 ? kTiledUnsplit : 1u << (force == 6 ? mxfp6::kCandTiled256 : force == 5 ? mxfp6::kCandTiled128x256 : mxfp6::kCandTiled128x128);
    mxfp6::KernelChoice c = family_choice(g, shapes, kTiledSplits);
    if (!apply_choice(g, c, s)) apply_choice(g, mxfp6::choose_kernel(g, 1, false, shapes), s);
    if (g.ksplit > 1 || !relayout_then_tiled(g, s, e)) e = mxfp6::launch_gemm_tiled(g, s);
  } else if (K != 0 && (force == 3 || (force >= 7 && force <= 16) || (force >= 19 && force <= 21))) {
    if (!mxfp6::gemm_skinny_supports(g)) return MXFP6_EINVAL_SHAPE;
    g.skinny_geometry = force == 3 ? 0 : force >= 19 ? force - 8 : force - 6;
    e = mxfp6::launch_gemm_skinny(g, s);
  } else if (K != 0 && force == 4) {
    if (!mxfp6::gemm_mid_supports(g)) return MXFP6_EINVAL_SHAPE;
    e = mxfp6::launch_gemm_mid(g, s);
  } else if (K != 0 && force == 18) {
    if (!mxfp6::gemm_tiled4_supports(g)) return MXFP6_EINVAL_SHAPE;
    e = mxfp6::launch_gemm_tiled4(g, s);
  } else if (K != 0 && force == 28) {
    if (!mxfp6::gemm_ring_supports(g)) return MXFP6_EINVAL_SHAPE;
    (void)apply_choice(g, mxfp6::choose_kernel(g, g_ksplit, true, 1u << mxfp6::kCandRing), s);  // without a workspace: unsplit
    e = mxfp6::launch_gemm_ring(g, s);
  } else if (K != 0 && ((force >= 22 && force <= 24) || force == 26)) {
    if (!mxfp6::gemm_block_supports(g)) return MXFP6_EINVAL_SHAPE;
    if (force != 26) (void)apply_choice(g, family_choice(g, 1u << mxfp6::kCandBlock, 1u << mxfp6::kCandBlockSplit), s);  // without a workspace: unsplit
    g.tile_rows = force == 23 ? 3 : force == 24 ? 6 : 0, g.tile_cols = force == 26 ? 256 : 0;
    e = mxfp6::launch_gemm_block(g, s);
  } else {
    mxfp6::KernelChoice c = auto_choice(g, force_split, true);
    // a split needs this stream's workspace: without it, what the shape gets otherwise
    if (!apply_choice(g, c, s)) {
      c = auto_choice(g, force_split, false);
      (void)apply_choice(g, c, s);
    }
    switch (c.cand) {
      case mxfp6::kCandTiled256: case mxfp6::kCandTiled128x256: case mxfp6::kCandTiled128x128:
        if (!relayout_then_tiled(g, s, e)) e = mxfp6::launch_gemm_tiled(g, s);
        break;
      case mxfp6::kCandTiledSplit256: case mxfp6::kCandTiledSplit128: e = mxfp6::launch_gemm_tiled(g, s); break;
      case mxfp6::kCandBlock: case mxfp6::kCandBlockWide: case mxfp6::kCandBlockSplit: e = mxfp6::launch_gemm_block(g, s); break;
      case mxfp6::kCandSkinny: e = mxfp6::launch_gemm_skinny(g, s); break;
      case mxfp6::kCandRing: e = mxfp6::launch_gemm_ring(g, s); break;
      default: e = mxfp6::launch_gemm_generic(g, s); break;
    }
  }
  return e == hipSuccess ? MXFP6_OK : (int)e;
}

}  // namespace

extern "C" {
#pragma GCC visibility push(default)

int mxfp6_gemm(const void* A, const void* B, const void* As, const void* Bs, void* C, int M, int N, int K, int fmt_a,
               int fmt_b, void* stream) {
  return gemm_common(A, B, As, Bs, C, M, N, K, fmt_a, fmt_b, false, 0, 0, stream);
}

int mxfp6_gemm_f32out(const void* A, const void* B, const void* As, const void* Bs, float* C, int M, int N, int K,
                      int fmt_a, int fmt_b, void* stream) {
  return gemm_common(A, B, As, Bs, C, M, N, K, fmt_a, fmt_b, true, 0, 0, stream);
}

int mxfp6_gemm_ex(const void* A, const void* B, const void* As, const void* Bs, void* C, int M, int N, int K, int fmt_a,
                  int fmt_b, int layout_a, int layout_b, int out_f32, void* stream) {
  return gemm_common(A, B, As, Bs, C, M, N, K, fmt_a, fmt_b, out_f32 != 0, layout_a, layout_b, stream);
}

int mxfp6_gemm_fused(const void* A, const void* B, const void* As, const void* Bs, void* C, int M, int N, int K, int fmt_a,
                     int fmt_b, int layout_a, int layout_b, int out_f32, const void* bias, int bias_bf16, const float* row_scale,
                     const float* col_scale, int activation, void* stream) {
  mxfp6::Epilogue ep;
  ep.bias = bias, ep.bias_bf16 = bias_bf16 != 0, ep.row_scale = row_scale, ep.col_scale = col_scale, ep.act = activation;
  return gemm_common(A, B, As, Bs, C, M, N, K, fmt_a, fmt_b, out_f32 != 0, layout_a, layout_b, stream, ep);
}

int mxfp6_gemm_fused_fp6(const void* A, const void* B, const void* As, const void* Bs, void* C_packed, void* C_scale, int M, int N,
                         int K, int fmt_a, int fmt_b, int layout_a, int layout_b, int fmt_c, const void* bias, int bias_bf16,
                         const float* row_scale, const float* col_scale, int activation, void* stream) {
  if (fmt_c != MXFP6_FMT_E2M3 && fmt_c != MXFP6_FMT_E3M2) return MXFP6_EINVAL_FMT;
  if (N < 0 || N % 32 != 0) return MXFP6_EINVAL_SHAPE;
  mxfp6::Epilogue ep;
  ep.bias = bias, ep.bias_bf16 = bias_bf16 != 0, ep.row_scale = row_scale, ep.col_scale = col_scale, ep.act = activation;
  bool empty;
  int rc = check_gemm_args(A, B, As, Bs, C_packed, M, N, K, fmt_a, fmt_b, 7, layout_a, layout_b, ep, &empty);
  if (rc || empty) return rc;
  if (!C_scale) return MXFP6_EINVAL_PTR;
  rc = check_device();
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  // the tiled kernel quantises its accumulators itself; where another kernel is the better one (few rows of A: C is
  // small there) the product goes to an fp32 workspace of the stream-ordered allocator and through the quantiser
  mxfp6::GemmArgs g{(const uint8_t*)A, (const uint8_t*)B, (const uint8_t*)As, (const uint8_t*)Bs, C_packed, M, N, K, fmt_a, fmt_b, false, layout_a, layout_b};
  const int force = g_force;
  // the tiled kernel's own fp6 epilogue only where the automatic choice is that kernel (unsplit); any other choice runs as
  // it would for an fp32 output, into the workspace, and the quantiser follows
  const bool tiled = K > 0 && mxfp6::gemm_tiled_supports(g) &&
                     (force == 2 || force == 5 || force == 6 || force == 17 || (force == 0 && choice_code(auto_choice(g, 0, true)) == kChoiceTiled));
  if (tiled) {
    g.ep = ep, g.C_scale = (uint8_t*)C_scale, g.fmt_c = fmt_c;
    g.tile_rows = force == 5 || force == 17 ? 128 : force == 6 ? 256 : 0, g.tile_cols = force == 17 ? 128 : 0;
    if (force == 0 || force == 2) (void)apply_choice(g, mxfp6::choose_kernel(g, 1, false, kTiledUnsplit), s);  // the tile height (the fp6 epilogue needs 256 columns)
    hipError_t e;
    if (force != 0 || !relayout_then_tiled(g, s, e)) e = mxfp6::launch_gemm_tiled(g, s);
    return e == hipSuccess ? MXFP6_OK : (int)e;
  }
  std::lock_guard<std::recursive_mutex> launch_lock(g_sws_launch_mutex);
  float* tmp = reinterpret_cast<float*>(stream_workspace(s, 1, (size_t)M * N * 4));
  if (!tmp) return stream_is_capturing(s) ? (int)hipErrorStreamCaptureUnsupported : MXFP6_EWORKSPACE;
  rc = gemm_common(A, B, As, Bs, tmp, M, N, K, fmt_a, fmt_b, true, layout_a, layout_b, stream, ep);
  if (rc == MXFP6_OK) {
    const hipError_t e = mxfp6::launch_quantize(tmp, 0, (uint8_t*)C_packed, (uint8_t*)C_scale, M, N, fmt_c, MXFP6_LAYOUT_ROW, s);
    rc = e == hipSuccess ? MXFP6_OK : (int)e;
  }
  return rc;
}

int mxfp6_tile_operand(const void* src, void* dst, int rows, int K, int tile, void* stream) {
  if (rows < 0 || K < 0 || rows % 32 || K % 128) return MXFP6_EINVAL_SHAPE;
  if (rows == 0 || K == 0) return MXFP6_OK;
  if (!src || !dst) return MXFP6_EINVAL_PTR;
  if (((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return MXFP6_EINVAL_ALIGN;
  int rc = check_device();
  if (rc) return rc;
  hipError_t e = mxfp6::launch_tile_operand((const uint8_t*)src, (uint8_t*)dst, rows, K, tile, (hipStream_t)stream);
  return e == hipSuccess ? MXFP6_OK : (int)e;
}

int mxfp6_tile_scales(const void* src, void* dst, int rows, int K, int tile, void* stream) {
  if (rows < 0 || K < 0 || rows % 32 || K % 128) return MXFP6_EINVAL_SHAPE;
  if (rows == 0 || K == 0) return MXFP6_OK;
  if (!src || !dst) return MXFP6_EINVAL_PTR;
  if (((uintptr_t)src & 3) || ((uintptr_t)dst & 3)) return MXFP6_EINVAL_ALIGN;
  int rc = check_device();
  if (rc) return rc;
  hipError_t e = mxfp6::launch_tile_scales((const uint8_t*)src, (uint8_t*)dst, rows, K, tile, (hipStream_t)stream);
  return e == hipSuccess ? MXFP6_OK : (int)e;
}

int mxfp6_set_relayout(int on) {
  const int prev = g_relayout;
  g_relayout = on ? 1 : 0;
  return prev;
}

int mxfp6_set_kernel(int which) {
  if (which < 0 || which > 28 || which == 25 || which == 27) return MXFP6_EINVAL_KERNEL;
  const int prev = g_force;
  g_force = which;
  return prev;
}

int mxfp6_gemm_noalloc(const void* A, const void* B, const void* As, const void* Bs, void* C, int M, int N, int K, int fmt_a,
                       int fmt_b, int nsplit, void* stream) {
  if (nsplit != 0 && nsplit != 1 && nsplit != 2 && nsplit != 4 && nsplit != 8) return MXFP6_EINVAL_SHAPE;
  return gemm_common(A, B, As, Bs, C, M, N, K, fmt_a, fmt_b, false, 0, 0, stream, mxfp6::Epilogue(), 1, nsplit);
}

// ---- serialised tile-major operand ("blob"): 16-byte header, tile-major packed bytes, tile-major scales
namespace {
constexpr uint32_t kBlobMagic = 0x5436584du;  // "MX6T"
constexpr uint8_t kBlobVersion = 1;
__global__ void blob_header_kernel(uint32_t* dst, uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3) {
  dst[0] = w0, dst[1] = w1, dst[2] = w2, dst[3] = w3;
}
bool blob_shape_ok(int rows, int K) { return rows > 0 && K > 0 && rows % 32 == 0 && K % 128 == 0 && (size_t)rows * (K / 4 * 3) < ((size_t)1 << 40); }
void blob_words(int rows, int K, int fmt, uint32_t w[4]) {
  w[0] = kBlobMagic;
  w[1] = (uint32_t)kBlobVersion | (uint32_t)fmt << 8 | (uint32_t)MXFP6_LAYOUT_TILE << 16;  // byte 7 reserved (0)
  w[2] = (uint32_t)rows;
  w[3] = (uint32_t)K;
}
}  // namespace

size_t mxfp6_blob_bytes(int rows, int K) {
  if (!blob_shape_ok(rows, K)) return 0;
  return 16 + (size_t)rows * (K / 4 * 3) + (size_t)rows * ((K + 511) / 512) * 16;
}

int mxfp6_blob_header_write(void* header16, int rows, int K, int fmt) {
  if (!header16) return MXFP6_EINVAL_PTR;
  if (!blob_shape_ok(rows, K)) return MXFP6_EINVAL_SHAPE;
  if (fmt != MXFP6_FMT_E2M3 && fmt != MXFP6_FMT_E3M2) return MXFP6_EINVAL_FMT;
  uint32_t w[4];
  blob_words(rows, K, fmt, w);
  uint8_t* h = static_cast<uint8_t*>(header16);
  for (int i = 0; i < 4; i++)
    for (int b = 0; b < 4; b++) h[4 * i + b] = (uint8_t)(w[i] >> (8 * b));  // little endian whatever the host is
  return MXFP6_OK;
}

int mxfp6_blob_header_read(const void* header16, int* rows, int* K, int* fmt) {
  if (!header16 || !rows || !K || !fmt) return MXFP6_EINVAL_PTR;
  const uint8_t* h = static_cast<const uint8_t*>(header16);
  uint32_t w[4];
  for (int i = 0; i < 4; i++) w[i] = (uint32_t)h[4 * i] | (uint32_t)h[4 * i + 1] << 8 | (uint32_t)h[4 * i + 2] << 16 | (uint32_t)h[4 * i + 3] << 24;
  if (w[0] != kBlobMagic) return MXFP6_EBLOB;
  if ((w[1] & 0xff) != kBlobVersion || ((w[1] >> 16) & 0xff) != MXFP6_LAYOUT_TILE || (w[1] >> 24) != 0) return MXFP6_EBLOB;
  const int f = (int)((w[1] >> 8) & 0xff);
  if (f != MXFP6_FMT_E2M3 && f != MXFP6_FMT_E3M2) return MXFP6_EBLOB;
  if (w[2] > 0x7fffffffu || w[3] > 0x7fffffffu || !blob_shape_ok((int)w[2], (int)w[3])) return MXFP6_EBLOB;
  *rows = (int)w[2], *K = (int)w[3], *fmt = f;
  return MXFP6_OK;
}

int mxfp6_blob_pack(const void* packed, const void* scales, void* blob, int rows, int K, int fmt, void* stream) {
  if (!blob_shape_ok(rows, K)) return MXFP6_EINVAL_SHAPE;
  if (fmt != MXFP6_FMT_E2M3 && fmt != MXFP6_FMT_E3M2) return MXFP6_EINVAL_FMT;
  if (!packed || !scales || !blob) return MXFP6_EINVAL_PTR;
  if (((uintptr_t)packed & 15) || ((uintptr_t)blob & 15) || ((uintptr_t)scales & 3)) return MXFP6_EINVAL_ALIGN;
  int rc = check_device();
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  uint32_t w[4];
  blob_words(rows, K, fmt, w);
  blob_header_kernel<<<1, 1, 0, s>>>(static_cast<uint32_t*>(blob), w[0], w[1], w[2], w[3]);
  hipError_t e = hipGetLastError();
  uint8_t* body = static_cast<uint8_t*>(blob) + 16;
  if (e == hipSuccess) e = mxfp6::launch_tile_operand((const uint8_t*)packed, body, rows, K, 1, s);
  if (e == hipSuccess) e = mxfp6::launch_tile_scales((const uint8_t*)scales, body + (size_t)rows * (K / 4 * 3), rows, K, 1, s);
  return e == hipSuccess ? MXFP6_OK : (int)e;
}

int mxfp6_blob_unpack(const void* blob, void* packed, void* scales, int rows, int K, void* stream) {
  if (!blob_shape_ok(rows, K)) return MXFP6_EINVAL_SHAPE;
  if (!packed || !scales || !blob) return MXFP6_EINVAL_PTR;
  if (((uintptr_t)packed & 15) || ((uintptr_t)blob & 15) || ((uintptr_t)scales & 3)) return MXFP6_EINVAL_ALIGN;
  int rc = check_device();
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  const uint8_t* body = static_cast<const uint8_t*>(blob) + 16;
  hipError_t e = mxfp6::launch_tile_operand(body, (uint8_t*)packed, rows, K, 0, s);
  if (e == hipSuccess) e = mxfp6::launch_tile_scales(body + (size_t)rows * (K / 4 * 3), (uint8_t*)scales, rows, K, 0, s);
  return e == hipSuccess ? MXFP6_OK : (int)e;
}

int mxfp6_allow_e3m2_pair(int allow) {
  const int prev = g_allow_e3m2_pair;
  g_allow_e3m2_pair = allow ? 1 : 0;
  return prev;
}

int mxfp6_set_k_split(int shares) {
  if (shares < -1 || shares > 64) return MXFP6_EINVAL_SHAPE;
  const int prev = g_ksplit;
  g_ksplit = shares;
  return prev;
}

int mxfp6_kernel_choice(int M, int N, int K, int layouts) {
  if (M <= 0 || N <= 0 || K < 0 || K % 32) return MXFP6_EINVAL_SHAPE;
  if (layouts < 0 || layouts > 3) return MXFP6_EINVAL_LAYOUT;
  const int layout_a = layouts & 1, layout_b = layouts >> 1;
  if ((layout_a && (M % 32 || K % 128)) || (layout_b && (N % 32 || K % 128))) return MXFP6_EINVAL_SHAPE;
  const int rc = check_device();
  if (rc) return rc;
  // aligned stand-ins for the pointers: the choice looks at their alignment only
  const uint8_t* p = reinterpret_cast<const uint8_t*>((uintptr_t)4096);
  mxfp6::GemmArgs g{p, p, p, p, const_cast<uint8_t*>(p), M, N, K, 2, 2, false, layout_a, layout_b};
  return choice_code(auto_choice(g, 0, true));
}

#ifdef MXFP6_PROBES  // ---- measurement entry points (include/mxfp6_probes.h)
int mxfp6_probe_tiled_ablation(int mask) {
  if (mask < 0 || (mask > 6 && mask != 8) || mask == 5) return MXFP6_EINVAL_SHAPE;
  g_ablation = mask;
  return MXFP6_OK;
}


int mxfp6_probe_ksplit_plan(int M, int N, int K, int layouts, int shares, int* tile_rows) {
  if (M <= 0 || N <= 0 || K <= 0 || shares < -1 || shares > 64) return MXFP6_EINVAL_SHAPE;
  if (layouts < 0 || layouts > 3) return MXFP6_EINVAL_LAYOUT;
  const int layout_a = layouts & 1, layout_b = layouts >> 1;
  if ((layout_a && M % 32) || (layout_b && N % 32)) return MXFP6_EINVAL_SHAPE;
  const int rc = check_device();
  if (rc) return rc;
  mxfp6::GemmArgs g{nullptr, nullptr, nullptr, nullptr, nullptr, M, N, K, 2, 2, false, layout_a, layout_b};
  int rows = 0, n = 1;
  // shares == 0: the split where the model prefers it to the tiled kernel's unsplit tiles; else the better of the two tile heights' splits
  const mxfp6::KernelChoice c = mxfp6::choose_kernel(g, shares, true, shares == 0 ? kTiledFamily : kTiledSplits);
  if (c.cand >= 0 && (kTiledSplits >> c.cand & 1)) n = c.shares, rows = c.rows;
  if (tile_rows) *tile_rows = n > 1 ? rows : 0;
  return n;
}

int mxfp6_probe_time_gemm(const void* A, const void* B, const void* As, const void* Bs, void* C, int M, int N, int K, int fmt_a, int fmt_b,
                          int layout_a, int layout_b, int out_f32, int b_sets, size_t b_stride, size_t bs_stride, int warmup, int reps, double* us,
                          void* stream) {
  if (!us || b_sets < 1 || warmup < 0 || reps < 1) return MXFP6_EINVAL_PTR;
  hipStream_t s = (hipStream_t)stream;
  auto launch = [&](int i) {
    const size_t set = (size_t)(i % b_sets);
    return gemm_common(A, (const uint8_t*)B + set * b_stride, As, (const uint8_t*)Bs + set * bs_stride, C, M, N, K, fmt_a, fmt_b, out_f32 != 0, layout_a, layout_b, stream);
  };
  for (int i = 0; i < warmup; i++) {
    const int rc = launch(i);
    if (rc) return rc;
  }
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return (int)hipErrorOutOfMemory;
  int rc = (int)hipEventRecord(e0, s);
  for (int i = 0; i < reps && !rc; i++) rc = launch(warmup + i);
  if (!rc) rc = (int)hipEventRecord(e1, s);
  if (!rc) rc = (int)hipEventSynchronize(e1);
  float ms = 0.f;
  if (!rc) rc = (int)hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0), (void)hipEventDestroy(e1);
  *us = ms * 1e3 / reps;
  return rc;
}

int mxfp6_probe_candidate(int M, int N, int K, int layouts, int candidate, int cus, double* model_us, double* calibrated_us, int* shares) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 32 || candidate < 0 || candidate >= mxfp6::kNumCandidates || cus < 0) return MXFP6_EINVAL_SHAPE;
  if (layouts < 0 || layouts > 3) return MXFP6_EINVAL_LAYOUT;
  if (!model_us || !calibrated_us || !shares) return MXFP6_EINVAL_PTR;
  const uint8_t* p = reinterpret_cast<const uint8_t*>((uintptr_t)4096);  // aligned stand-ins: the candidates look at the alignment only
  mxfp6::GemmArgs g{p, p, p, p, const_cast<uint8_t*>(p), M, N, K, 2, 2, false, layouts & 1, layouts >> 1};
  int rows = 0;
  *model_us = mxfp6::candidate_model_us(g, candidate, g_ksplit, cus ? cus : mxfp6::device_cus(), shares, &rows);
  const mxfp6::KernelChoice c = mxfp6::choose_kernel(g, g_ksplit, true, 1u << candidate);
  *calibrated_us = c.cand == candidate ? c.us : -1.0;
  return MXFP6_OK;
}

int mxfp6_probe_block(int enable) {
  const int prev = g_block;
  g_block = enable ? 1 : 0;
  return prev;
}


int mxfp6_probe_raster(int group_m, int xcd_remap) {
  if (group_m < 0 || group_m > 4096) return MXFP6_EINVAL_SHAPE;
  g_raster_group_m = group_m, g_raster_no_xcd = xcd_remap == 2 ? 2 : xcd_remap ? 0 : 1;
  return MXFP6_OK;
}

int mxfp6_tile_order(int tiles_m, int tiles_n, int group_m, int xcd_remap, int* order) {
  if (tiles_m < 1 || tiles_n < 1 || tiles_m > 65535 || tiles_n > 32767 || group_m < 1 || (long)tiles_m * tiles_n >= (1L << 31)) return MXFP6_EINVAL_SHAPE;
  if (!order) return MXFP6_EINVAL_PTR;
  const int nb = tiles_m * tiles_n;
  for (int b = 0; b < nb; b++) order[b] = mxfp6::tile_order(b, tiles_m, tiles_n, group_m, xcd_remap);
  return mxfp6::tile_order(nb, tiles_m, tiles_n, group_m, xcd_remap) == -1 ? MXFP6_OK : MXFP6_EINVAL_SHAPE;
}

int mxfp6_probe_tiled_clock(uint32_t* stamps) {
  g_clock_stamps = stamps;
  return MXFP6_OK;
}

int mxfp6_probe_mfma(const void* A, const void* B, const void* As, const void* Bs, int rows_a, int rows_b, int K, int fmt_a, int fmt_b, int iters,
                     float* sink, uint32_t* stats, void* stream) {
  if (rows_a < 32 || rows_b < 32 || K < 64 || K % 32 || iters < 1) return MXFP6_EINVAL_SHAPE;
  if ((fmt_a != MXFP6_FMT_E2M3 && fmt_a != MXFP6_FMT_E3M2) || (fmt_b != MXFP6_FMT_E2M3 && fmt_b != MXFP6_FMT_E3M2)) return MXFP6_EINVAL_FMT;
  if (!A || !B || !As || !Bs || !sink || !stats) return MXFP6_EINVAL_PTR;
  if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)sink | (uintptr_t)stats) & 3) return MXFP6_EINVAL_ALIGN;
  int rc = check_device();
  if (rc) return rc;
  // two workgroups of four waves per compute unit: two waves per SIMD, as in the tiled kernel
  int cus = 0, dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return MXFP6_ENODEVICE;
  const hipError_t e = mxfp6::launch_mfma_probe((const uint8_t*)A, (const uint8_t*)B, (const uint8_t*)As, (const uint8_t*)Bs, rows_a, rows_b, K, fmt_a, fmt_b,
                                                iters, 2 * cus, sink, stats, (hipStream_t)stream);
  return e == hipSuccess ? 2 * cus * 4 : -(int)e - 1000;  // waves launched (each issues 4 * iters MFMAs of 131072 flop)
}

int mxfp6_probe_stream(const void* buf, size_t bytes, int workgroups, int waves, uint32_t* stats, void* stream) {
  if (!buf || !stats) return MXFP6_EINVAL_PTR;
  if (((uintptr_t)buf & 15) || ((uintptr_t)stats & 3)) return MXFP6_EINVAL_ALIGN;
  if (workgroups < 1 || (waves != 4 && waves != 8) || bytes == 0 || bytes % ((size_t)workgroups * waves * 8192) != 0) return MXFP6_EINVAL_SHAPE;
  int rc = check_device();
  if (rc) return rc;
  const hipError_t e = mxfp6::launch_stream_probe((const uint8_t*)buf, bytes, workgroups, waves, stats, (hipStream_t)stream);
  return e == hipSuccess ? MXFP6_OK : (int)e;
}

#endif  // MXFP6_PROBES

int mxfp6_release_workspaces(void) {
  const hipError_t a = release_stream_workspaces();
  const hipError_t b = mxfp6::release_split_workspaces();
  return a != hipSuccess ? (int)a : (b == hipSuccess ? MXFP6_OK : (int)b);
}

int mxfp6_quantize(const float* X, void* packed, void* scales, int rows, int K, int fmt, void* stream) {
  return mxfp6_quantize_ex(X, packed, scales, rows, K, fmt, MXFP6_LAYOUT_ROW, stream);
}

static int quantize_common(const void* X, int x_bf16, void* packed, void* scales, int rows, int K, int fmt, int layout, void* stream) {
  if (rows < 0 || K < 0 || K % 32 != 0) return MXFP6_EINVAL_SHAPE;
  if (layout != MXFP6_LAYOUT_ROW && layout != MXFP6_LAYOUT_TILE) return MXFP6_EINVAL_LAYOUT;
  if (layout == MXFP6_LAYOUT_TILE && (rows % 32 || K % 128)) return MXFP6_EINVAL_SHAPE;
  if (fmt != MXFP6_FMT_E2M3 && fmt != MXFP6_FMT_E3M2) return MXFP6_EINVAL_FMT;
  if (rows == 0 || K == 0) return MXFP6_OK;
  if (!X || !packed || !scales) return MXFP6_EINVAL_PTR;
  if (((uintptr_t)X & 15) || ((uintptr_t)packed & 3)) return MXFP6_EINVAL_ALIGN;
  int rc = check_device();
  if (rc) return rc;
  hipError_t e = mxfp6::launch_quantize(X, x_bf16, (uint8_t*)packed, (uint8_t*)scales, rows, K, fmt, layout, (hipStream_t)stream);
  return e == hipSuccess ? MXFP6_OK : (int)e;
}

int mxfp6_quantize_ex(const float* X, void* packed, void* scales, int rows, int K, int fmt, int layout, void* stream) {
  return quantize_common(X, 0, packed, scales, rows, K, fmt, layout, stream);
}

int mxfp6_quantize_bf16(const void* X, void* packed, void* scales, int rows, int K, int fmt, int layout, void* stream) {
  return quantize_common(X, 1, packed, scales, rows, K, fmt, layout, stream);
}

const char* mxfp6_strerror(int code) {
  switch (code) {
    case MXFP6_OK: return "success";
    case MXFP6_EINVAL_PTR: return "mxfp6: a required pointer is NULL";
    case MXFP6_EINVAL_SHAPE: return "mxfp6: bad shape (M, N, K >= 0 and K % 32 == 0 required; a forced kernel may need more, and 16-byte aligned operands and scales)";
    case MXFP6_EINVAL_FMT: return "mxfp6: format must be 2 (e2m3) or 3 (e3m2)";
    case MXFP6_EINVAL_ALIGN: return "mxfp6: pointer alignment (packed operands 4 bytes, C its element size, fp32 / bf16 input and vectors of the fused epilogue 16 bytes)";
    case MXFP6_ENODEVICE: return "mxfp6: the current device is not gfx950 (MI355X)";
    case MXFP6_EINVAL_LAYOUT: return "mxfp6: layout must be 0 (row-major) or 1 (tile-major)";
    case MXFP6_EINVAL_EPILOGUE: return "mxfp6: activation must be 0 (none), 1 (relu), 2 (gelu) or 3 (silu)";
    case MXFP6_ESCRATCH: return "mxfp6: the K split of this call needs more than the static scratch memory holds (256 partial tiles: rows of C tiles times nsplit)";
    case MXFP6_EINVAL_KERNEL: return "mxfp6: unknown kernel code";
    case MXFP6_EWORKSPACE: return "mxfp6: no workspace for this call (the allocator refused, or every workspace slot is held by a captured graph)";
    case MXFP6_EACCURACY: return "mxfp6: e3m2 x e3m2 can exceed the 2e-3 accuracy bar (up to 1e-4 of sum |a||b| per output); call mxfp6_allow_e3m2_pair(1) to accept that";
    case MXFP6_EBLOB: return "mxfp6: not a tile-major operand blob this library reads (magic, version, format, layout or shape)";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "mxfp6: unknown error code";
}

int mxfp6_abi_version(void) { return MXFP6_ABI_VERSION; }

#pragma GCC visibility pop
}  // extern "C"
