// C ABI of the library: argument validation, route selection, launches.  No torch types, no
// allocation, no synchronisation; see include/glowq_w4a16.h for the contract of each entry point.
#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "common.hpp"
#include "side_stream.hpp"
#include "tiled.hpp"

namespace glowq {
// gemv.hip
hipError_t launch_wave_dot(GroupDev& g, int rows_per_task, int num_cus, hipStream_t stream);
hipError_t launch_generic(GroupDev& g, int num_cus, hipStream_t stream);
int wave_dot_rows(long total_rows);
int wave_dot_rows_single(long total_rows);
bool wave_dot_supported(int M, int K, int rank, bool has_r);
// gemv_stream.hip
bool stream_supported(const GroupDev& g);
hipError_t launch_stream(GroupDev& g, int num_cus, hipStream_t stream);
bool chain_combination_supported(int pro, int epi);
hipError_t launch_stream_chained(GroupDev& g, const streamk::ChainDev& ch, int pro, int epi, hipStream_t stream);
// gemv_quad.hip
int quad_capacity(int M, int K, int rank, bool has_r);
hipError_t launch_quad(GroupDev& g, int num_cus, hipStream_t stream);
bool qstream_supported(const GroupDev& g);
hipError_t launch_qstream(GroupDev& g, int num_cus, hipStream_t stream);
// misc.hip
hipError_t launch_dequant(const int32_t*, const half_t*, const int32_t*, half_t*, int, int, int, int, int, int, int,
                          hipStream_t);
hipError_t launch_unpack(const int32_t*, uint8_t*, int, int, int, int, hipStream_t);
hipError_t launch_shared_proj_small(const half_t*, const half_t*, half_t*, int, int, int, hipStream_t);
hipError_t launch_pack_side(const half_t*, const int32_t*, const half_t*, void*, int, int, int, int, int, int, int, hipStream_t);
// skinny.hip / gemm.hip
bool skinny_supported(const GroupDev& g);
bool skinny_group_form(const GroupDev& g);
bool skinny_raw_form(const GroupDev& g);
hipError_t launch_skinny(GroupDev& g, int num_cus, hipStream_t stream, bool raw);
bool gemm_supported(const GroupDev& g);
hipError_t launch_gemm(GroupDev& g, int num_cus, hipStream_t stream);
// misc.hip
hipError_t launch_probe_read(const void* src, size_t bytes, void* sink, int grid, int block, hipStream_t stream);
hipError_t launch_probe_empty(int grid, int block, hipStream_t stream);
size_t skinny_split_workspace_bytes(int M, int num_cus);  // skinny.hip
// skinny_tiled.hip
size_t tiled_split_workspace_bytes(int M, int num_cus);
bool skinny_tiled_supported(const GroupDev& g);
hipError_t launch_skinny_tiled(GroupDev& g, int num_cus, hipStream_t stream);
hipError_t launch_pack_tiled(const int32_t*, const half_t*, const int32_t*, void*, int, int, int, int, int, int, int, hipStream_t);
hipError_t launch_pack_tiled_left(const half_t*, void*, int, int, int, hipStream_t);
hipError_t launch_shared_proj_mfma(const half_t*, const half_t*, half_t*, int, int, int, int, hipStream_t, void* ws,
                                   size_t ws_bytes);
size_t proj_workspace_bytes(int M, int K, int rank, int num_cus);
}  // namespace glowq

using namespace glowq;

namespace {

thread_local char g_err[512] = "";

}  // namespace

// Scratch of glowq_w4a16_group_forward_fused_static: the workspace of the many-row projection and of the skinny kernel's
// split of K for callers that cannot bring one.  One copy per GPU the library runs on, held until the process ends.
constexpr size_t kStaticScratchBytes = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

// Device address of `scratch` on the current device.  The array's name is a host-side stand-in; the address each GPU
// keeps its copy at comes from hipGetSymbolAddress, asked once per device with that device current.
std::atomic<void*> g_scratch_ptr[64] = {};

void* static_scratch(bool lookup_allowed = true) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p != nullptr || !lookup_allowed) return p;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return nullptr;
  g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing host threads store the same address
  return p;
}

}  // namespace

namespace {
struct LaunchNote {
  char kernel[160];
  int grid_x, grid_y, block;
};
thread_local LaunchNote g_note = {};
}  // namespace

namespace glowq {
void note_launch(int grid_x, int grid_y, int block, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_note.kernel, sizeof(g_note.kernel), fmt, ap);
  va_end(ap);
  g_note.grid_x = grid_x;
  g_note.grid_y = grid_y;
  g_note.block = block;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// r = x R^T on the kernel with one workgroup per row (or two rows) of R and chunk of four token rows, or on the MFMA
// projection with its sum over K slices: the first up to 16 rows always, and up to 64 rows while M K rank stays below
// 90 M multiply-adds (timings of both next to proj_block_shape, misc.hip).
bool proj_on_small_kernel(int M, int K, int rank) {
  static const int force = getenv("GLOWQ_PROJ_SMALL") ? atoi(getenv("GLOWQ_PROJ_SMALL")) : -1;
  if (force >= 0) return force != 0 && M <= 64;
  return M <= 16 || (M <= 64 && (long)M * K * rank <= 90L * 1000 * 1000);
}

int num_cus() {
  // one value per device; the current device is the one the caller's tensors live on
  static std::atomic<int> cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}
}  // namespace glowq

namespace {

constexpr int kRouteWaveDot = 0, kRouteSkinny = 1, kRouteGemm = 2, kRouteGeneric = 3, kRouteQuad = 4, kRouteStream = 5, kRouteQStream = 6, kRouteSkinnyRaw = 7,
              kRouteSkinnyTiled = 8;
constexpr int kWaveDotMaxM = 4;  // row capacity of the wave-dot kernel

// Route limits, settable at run time (glowq_set_tuning) and initialised from the environment:
//   wave_dot_max_m  rows up to which the wave-dot GEMV is preferred over the skinny MFMA kernel (GLOWQ_WAVEDOT_M)
//   quad_max_m      rows up to which the 4x4x4 matrix-core GEMV is used; 0 switches it off (GLOWQ_QUAD_M).  Above it
//                   the skinny MFMA kernel takes over; where only that kernel's first form applies (K % 256 != 0 or
//                   small groups) the 4x4x4 GEMV still serves up to 16 rows
//   quad_min_m      rows from which it is used (GLOWQ_QUAD_MIN_M; a single row is faster on the wave-dot kernel)
int env_or(const char* name, int fallback) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : fallback;
}
int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }
std::atomic<int> g_wave_dot_max_m{clampi(env_or("GLOWQ_WAVEDOT_M", kWaveDotMaxM), 0, kWaveDotMaxM)};
std::atomic<int> g_quad_max_m{clampi(env_or("GLOWQ_QUAD_M", 4), 0, 16)};
std::atomic<int> g_quad_min_m{clampi(env_or("GLOWQ_QUAD_MIN_M", 2), 1, 16)};
//   skinny_max_m    rows up to which the skinny MFMA kernel is preferred over the tiled GEMM (GLOWQ_SKINNY_M)
std::atomic<int> g_skinny_max_m{clampi(env_or("GLOWQ_SKINNY_M", 64), 0, 64)};
//   small_group_mb  3..4 rows: groups whose int4 weights are smaller than this many MB go to the skinny MFMA kernel (or
//                   stay on the wave-dot GEMV), which start up faster than the 4x4x4 GEMV; at two rows they stay on the
//                   wave-dot GEMV and the limit is 40/17 of it (GLOWQ_SMALL_GROUP_MB; default 17; 0 switches the rule off).  8B-shape layers at two rows: q|k|v 8.9 -> 7.8 us, o_proj 7.2 -> 5.6,
//                   down_proj (29 MB) 13.1 -> 11.2, while gate|up (59 MB) is 1.6 us faster on the 4x4x4 kernel
std::atomic<int> g_small_group_mb{clampi(env_or("GLOWQ_SMALL_GROUP_MB", 17), 0, 4096)};
bool small_group_prefers_wave_dot(const GroupDev& g) {
  if (g.M < 2 || g.M > 4) return false;
  const size_t mb = (size_t)g_small_group_mb.load(std::memory_order_relaxed);
  const size_t limit = (g.M == 2 ? mb * 40 / 17 : mb) << 20;
  size_t bytes = 0;
  for (int i = 0; i < g.n_members; ++i) bytes += (size_t)g.mem[i].N * (size_t)(g.K >> 1);
  return bytes < limit;
}
int wave_dot_pref_m() { return g_wave_dot_max_m.load(std::memory_order_relaxed); }
bool quad_wanted(int M) {
  return M >= g_quad_min_m.load(std::memory_order_relaxed) && M <= g_quad_max_m.load(std::memory_order_relaxed);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

// The fast routes read weights in 16-byte units of 32 codes: a unit must not straddle a
// quantisation group and every row must start 16-byte aligned.
bool fast_layout(const GroupDev& g) {
  if ((g.K & 31) != 0 || (g.group_size & 31) != 0) return false;
  if (((g.group_size >> 5) & ((g.group_size >> 5) - 1)) != 0) return false;  // units per group: a power of two
  if (!aligned16(g.x)) return false;
  for (int i = 0; i < g.n_members; ++i) {
    const MemberDev& m = g.mem[i];
    if (!aligned16(m.qweight) || (m.ldw & 3) != 0) return false;
    if (m.L && !aligned4(m.L)) return false;
  }
  if ((g.r || g.R) && (g.rank & 1) != 0) return false;  // the L rows are read two halves at a time
  if (g.R && (!aligned16(g.R) || (g.K & 7) != 0)) return false;
  return true;
}

int check_common(const void* x, int M, int K, int group_size) {
  if (x == nullptr) return fail(GLOWQ_EINVAL, "inputs must be a device pointer (got NULL)");
  if (M <= 0 || K <= 0) return fail(GLOWQ_EINVAL, "inputs must be [M, IC] with M > 0 and IC > 0 (got M=%d, IC=%d)", M, K);
  if (group_size <= 0) return fail(GLOWQ_EINVAL, "group_size must be > 0");
  if (group_size % 8 != 0) return fail(GLOWQ_EINVAL, "group_size must be a multiple of 8");
  return GLOWQ_OK;
}

int check_member(const glowq_member_t& m, int K, int group_size, int idx) {
  const int groups = (K + group_size - 1) / group_size;
  const int packed_iters = (K + 7) / 8;
  if (m.qweight == nullptr || m.scales == nullptr || m.qzeros == nullptr || m.y == nullptr)
    return fail(GLOWQ_EINVAL, "member %d: qweight, scales, qzeros and y must be device pointers", idx);
  if (m.N <= 0) return fail(GLOWQ_EINVAL, "member %d: OC must be > 0", idx);
  if (m.lds < groups) return fail(GLOWQ_ESHAPE, "member %d: scales groups mismatch (%d < %d)", idx, m.lds, groups);
  if (m.ldw_i32 < packed_iters)
    return fail(GLOWQ_ESHAPE, "member %d: qweight packed cols too small (%d < %d)", idx, m.ldw_i32, packed_iters);
  if (m.ldz_i32 < (groups + 7) / 8)
    return fail(GLOWQ_ESHAPE, "member %d: qzeros packed cols too small (%d < %d)", idx, m.ldz_i32, (groups + 7) / 8);
  if (m.ldy < m.N) return fail(GLOWQ_ESHAPE, "member %d: output row stride %d < OC %d", idx, m.ldy, m.N);
  return GLOWQ_OK;
}

void to_dev(const glowq_member_t& s, MemberDev& d) {
  d.qweight = s.qweight;
  d.scales = static_cast<const half_t*>(s.scales);
  d.qzeros = s.qzeros;
  d.L = static_cast<const half_t*>(s.L);
  d.bias = static_cast<const half_t*>(s.bias);
  d.y = static_cast<half_t*>(s.y);
  d.side = aligned16(s.side) ? static_cast<const unsigned char*>(s.side) : nullptr;
  d.side_rank = s.side_rank;
  d.tiled = s.tiled;
  d.tiled_L = s.tiled_L;
  d.tiled_rank = s.tiled_rank;
  d.N = s.N;
  d.ldw = s.ldw_i32;
  d.lds = s.lds;
  d.ldz = s.ldz_i32;
  d.ldy = s.ldy;
}

//   stream_max_m    token rows up to which the stream GEMV (every request of a wave in flight up front) is used where it
//                   applies; 0 switches it off (GLOWQ_STREAM_M)
std::atomic<int> g_stream_max_m{clampi(env_or("GLOWQ_STREAM_M", 4), 0, 4)};
//   stream_shape_rule  1: with more than one token row the stream GEMV is used only for the shapes it was measured
//                   faster on (its dot products repeat per token row on the vector ALUs, the 4x4x4 kernel's do not);
//                   0: for every shape up to stream_max_m rows (GLOWQ_STREAM_SHAPE_RULE)
std::atomic<int> g_stream_shape_rule{clampi(env_or("GLOWQ_STREAM_SHAPE_RULE", 1), 0, 1)};

// 8B-shape groups, group launch alone, us (stream / others): two rows q|k|v 5.9 / 7.6, o_proj 4.9 / 5.4, gate|up 15.5 /
// 16.7, down_proj (K = 14336) 11.1 / 10.5; three rows 7.1 / 7.6, 5.6 / 7.4, 19.9 / 19.0, 13.4 / 14.3; four rows 8.1 / 7.7,
// 6.6 / 7.4, 24.2 / 18.8, 15.7 / 14.6.
bool stream_pays(const GroupDev& g) {
  if (g.M <= 1 || g_stream_shape_rule.load(std::memory_order_relaxed) == 0) return true;
  long rows = 0;
  for (int i = 0; i < g.n_members; ++i) rows += g.mem[i].N;
  const bool short_k = g.K <= 4 * 2048;
  if (g.M == 2) return short_k;
  if (g.M == 3) return (short_k && rows <= 8192) || (!short_k && rows <= 4096);
  return short_k && rows <= 4096;
}

//   qstream_max_m   token rows (2..4) up to which the stream-scheduled 4x4x4 matrix-core GEMV is used where it applies;
//                   0 switches it off (GLOWQ_QSTREAM_M).  (A form for five to eight rows, two sets of sums per row
//                   block, ran level with the skinny MFMA kernel and was taken out.)
//   qstream_shape_rule  1: only for the shapes it was measured faster on; 0: for every shape it can take
//                   (GLOWQ_QSTREAM_SHAPE_RULE)
std::atomic<int> g_qstream_max_m{clampi(env_or("GLOWQ_QSTREAM_M", 4), 0, 4)};
std::atomic<int> g_qstream_shape_rule{clampi(env_or("GLOWQ_QSTREAM_SHAPE_RULE", 1), 0, 1)};

// Group launch alone, us, this kernel / the route taken without it (6 to 32 layers of distinct weights back to back):
//   four rows   4096 x 4096: 4.7 / 6.9   6144 x 4096 (q|k|v): 6.7 / 7.6   28672 x 4096: 15.8 / 19.2   4096 x 14336: 11.7 / 14.5
//               4096 x 11008: 9.4 / 13.4   8192 x 8192: 10.9 / 14.2   10240 x 8192: 13.5 / 19.7   37888 x 3584: 18.9 / 23.6
//               7168 x 5120: 9.6 / 12.2   5120 x 5120: 8.2 / 9.3   34816 x 5120: 27.7 / 31.7   28672 x 6144: 24.0 / 25.6
//   two rows    4096 x 4096: 4.6 / 5.1   6144 x 4096: 6.2 / 6.1   28672 x 4096: 14.1 / 16.2   4096 x 14336: 10.5 / 10.7
//               5120 x 5120: 7.5 / 7.3   7168 x 5120: 8.5 / 8.4   34816 x 5120: 25.9 / 27.2   10240 x 8192: 12.9 / 13.2
// At two rows a last slice that is mostly empty (K = 5120: 2.5 slices of 2048 columns) is enough to fall behind the
// stream GEMV on groups of few rows.
bool qstream_pays(const GroupDev& g) {
  if (g_qstream_shape_rule.load(std::memory_order_relaxed) == 0) return true;
  long rows = 0;
  for (int i = 0; i < g.n_members; ++i) rows += g.mem[i].N;
  const int padded = (g.K + 2047) / 2048 * 2048;
  if (g.M == 2 && rows < 16384 && (padded - g.K) * 100 > 15 * g.K) return false;
  return true;
}

//   skinny_codes_max_m  token rows up to which the skinny MFMA kernel takes the codes as they are (unrounded
//                   arithmetic, reported as a route of its own) where its second form applies to groups of 128 columns;
//                   above, and with 0 everywhere, it dequantises to fp16 first (GLOWQ_SKINNY_CODES_M).
// Group launch alone, 8B shapes, us, codes as they are / dequantised first: 8 rows q|k|v 7.9 / 7.8, o_proj 7.5 / 7.5,
// gate|up 20.0 / 22.3, down_proj 14.3 / 15.4; 16 rows 9.2 / 8.7, 8.8 / 8.3, 22.7 / 23.5, 17.1 / 17.1; 32 rows 12.2 / 10.5,
// 11.8 / 10.0, 28.2 / 27.0, 22.9 / 21.0; 64 rows 23.9 / 17.4, 23.5 / 16.9, 53.3 / 51.2, 43.5 / 33.0: applying scale and
// zero-point to the sums costs two instructions per accumulator register and group, which grows with the rows, while
// what it saves on the codes does not.
std::atomic<int> g_skinny_codes_max_m{clampi(env_or("GLOWQ_SKINNY_CODES_M", 8), 0, 64)};

int pick_route_rounded(const GroupDev& g, int force);

//   tiled_min_m / tiled_max_m  token rows served by the matrix-core kernel that reads the tiled copy of the weights, where
//                   every member of the group brings one (GLOWQ_TILED_MIN_M, GLOWQ_TILED_MAX_M; max 0 switches it off)
std::atomic<int> g_tiled_min_m{clampi(env_or("GLOWQ_TILED_MIN_M", 2), 1, 64)};
std::atomic<int> g_tiled_max_m{clampi(env_or("GLOWQ_TILED_MAX_M", 64), 0, 64)};
//   tiled_shape_rule  1: up to 32 rows only groups whose stream is long enough to pay for the kernel's start-up take the
//                   tiled route, the others stay on the skinny kernel (GLOWQ_TILED_SHAPE_RULE; 0: every group that can).
//                   Group launch with the projection in front, us, tiled / skinny.  8B shapes: q|k|v (13 MB of codes) 8 rows
//                   14.9 / 11.3, 32 rows 17.8 / 15.2, 64 rows 24.6 / 24.5; o_proj (8 MB) 13.8 / 10.7, 16.4 / 14.8, 22.6 /
//                   23.9; gate|up (59 MB) 22.4 / 24.1, 26.3 / 31.1, 37.4 / 56.0; down_proj (29 MB) 21.3 / 19.5, 16 rows
//                   22.3 / 21.5, 32 rows 25.5 / 28.2, 64 rows 32.2 / 41.2.  14B shapes: gate|up (89 MB) 33.2 / 40.8,
//                   41.7 / 52.3, 62.7 / 93.9; down_proj (45 MB) 27.7 / 28.5, 32.0 / 40.2, 42.6 / 63.0.
std::atomic<int> g_tiled_shape_rule{clampi(env_or("GLOWQ_TILED_SHAPE_RULE", 1), 0, 1)};
bool tiled_pays(const GroupDev& g) {
  if (g.M > 32 || g_tiled_shape_rule.load(std::memory_order_relaxed) == 0) return true;
  long rows = 0;
  for (int i = 0; i < g.n_members; ++i) rows += g.mem[i].N;
  const long code_bytes = rows * (long)g.K / 2;
  // two to four rows: only the longest streams (gate|up of a 14B layer, 89 MB: 24.0 to 24.2 us against 26.1 to 27.6 on the
  // 4x4x4 stream kernel with r given, 25.0 against 30.1 with the projection, which the launch then takes along; gate|up of
  // an 8B layer, 59 MB: 17.5 against 14.8 to 15.8 with r given)
  if (g.M < 5) return code_bytes >= 80L * 1000 * 1000;
  return code_bytes >= 40L * 1000 * 1000 || (g.M > 16 && code_bytes >= 24L * 1000 * 1000);
}

//   proj_in_launch  1: a single token on the stream GEMV computes r = R x inside the group launch when the call brings a
//                   workspace for the hand-over (8 bytes per entry of r); 0: always the projection launch in front
//                   (GLOWQ_PROJ_IN_LAUNCH); 2, for tests: as 1, but the producing waves do not hand their entries over, so
//                   that every reader runs into the limit below and computes its entry itself
//   proj_spin_limit polls a reader spends on an entry of r that is not there yet before it computes the entry itself
//                   (GLOWQ_PROJ_SPIN_LIMIT; 0: never waits)
std::atomic<int> g_proj_in_launch{clampi(env_or("GLOWQ_PROJ_IN_LAUNCH", 1), 0, 2)};
std::atomic<int> g_proj_spin_limit{clampi(env_or("GLOWQ_PROJ_SPIN_LIMIT", 16384), 0, 1 << 24)};
//   small_rows_in_launch  1: a fused call with three or four token rows and a workspace goes to the skinny kernel where its
//                   launch computes r itself (GLOWQ_SMALL_ROWS_IN_LAUNCH; 0: always the 2..4-row kernels behind a
//                   projection launch)
std::atomic<int> g_small_rows_in_launch{clampi(env_or("GLOWQ_SMALL_ROWS_IN_LAUNCH", 1), 0, 1)};
// the block the readers look at and, 4096 bytes behind it, the staging words, each with room for rank 256
// (stream_kernel.hpp)
constexpr size_t kProjHandoverBytes = 4096 + 256 * 8;
bool proj_in_launch(const GroupDev& g) {
  if (g.M != 1 || g_proj_in_launch.load(std::memory_order_relaxed) == 0) return false;
  if (g.ws == nullptr || (reinterpret_cast<uintptr_t>(g.ws) & 7u) != 0 || g.ws_bytes < kProjHandoverBytes) return false;
  if (g.rank > 256 || !proj_on_small_kernel(g.M, g.K, g.rank) || !aligned16(g.x) || !aligned16(g.R)) return false;
  bool any_left = false;
  for (int i = 0; i < g.n_members; ++i) any_left = any_left || g.mem[i].L != nullptr;
  return any_left;  // (the launcher still turns down a grid that is not on the chip all at once)
}

// The same for the skinny kernel at 5..32 token rows (skinny.hip): the head of the workspace takes the hand-over words,
// and the producers in front compute r in the arithmetic of the small projection kernels.
constexpr size_t kSkinnyHandoverBytes = (size_t)(512 + 512) * 8;
bool skinny_proj_in_launch(const GroupDev& g) {
  if (g.M < 2 || g.M > 32 || g_proj_in_launch.load(std::memory_order_relaxed) == 0) return false;
  if (g.ws == nullptr || (reinterpret_cast<uintptr_t>(g.ws) & 15u) != 0 || g.ws_bytes < kSkinnyHandoverBytes) return false;
  if (!proj_on_small_kernel(g.M, g.K, g.rank) || (g.K & 255) != 0 || (g.rank & 7) != 0 || !aligned16(g.x) || !aligned16(g.R)) return false;
  if ((reinterpret_cast<uintptr_t>(g.r_out) & 15u) != 0) return false;
  bool any_left = false;
  for (int i = 0; i < g.n_members; ++i) any_left = any_left || g.mem[i].L != nullptr;
  return any_left;  // (the launcher still turns down shapes and grids it does not take)
}

int pick_route(const GroupDev& g, int force) {
  if (force < 0 && g.M >= g_tiled_min_m.load(std::memory_order_relaxed) && g.M <= g_tiled_max_m.load(std::memory_order_relaxed) &&
      skinny_tiled_supported(g) && tiled_pays(g))
    return kRouteSkinnyTiled;
  const int route = pick_route_rounded(g, force);
  if (route == kRouteSkinny && force < 0 && g.M <= g_skinny_codes_max_m.load(std::memory_order_relaxed) && skinny_raw_form(g)) return kRouteSkinnyRaw;
  return route;
}

int pick_route_rounded(const GroupDev& g, int force) {
  if (!fast_layout(g)) return kRouteGeneric;
  if (force == kRouteGemm) return gemm_supported(g) ? kRouteGemm : kRouteGeneric;
  if (force < 0 && g.M >= 2 && g.M <= g_qstream_max_m.load(std::memory_order_relaxed) && qstream_supported(g) && qstream_pays(g))
    return kRouteQStream;
  if (force < 0 && g.M <= g_stream_max_m.load(std::memory_order_relaxed) && stream_supported(g) && stream_pays(g))
    return kRouteStream;
  const bool quad_rows = quad_wanted(g.M) ||
                         (g.M > 1 && g.M <= 16 && g_quad_max_m.load(std::memory_order_relaxed) > 0 && !(skinny_supported(g) && skinny_group_form(g)));
  if (force < 0 && small_group_prefers_wave_dot(g)) {
    // two rows: the wave-dot GEMV; three and four: the skinny MFMA kernel where its super-block form applies
    // (8B-shape q|k|v at four rows: 10.5 us on the 4x4x4 GEMV, 10.0 on the wave-dot GEMV, 8.0 on the skinny kernel)
    if (g.M > 2 && skinny_supported(g) && skinny_group_form(g)) return kRouteSkinny;
    if (g.M <= wave_dot_pref_m() && wave_dot_supported(g.M, g.K, g.rank, g.r != nullptr || g.R != nullptr))
      return kRouteWaveDot;
  }
  if (quad_rows && force != kRouteSkinny && quad_capacity(g.M, g.K, g.rank, g.r != nullptr || g.R != nullptr) > 0) {
    bool ok = true;
    for (int i = 0; i < g.n_members; ++i)  // 16-byte L rows; 32-bit byte offsets inside every buffer of a member
      ok = ok && (g.mem[i].L == nullptr || aligned16(g.mem[i].L)) && (long)g.mem[i].N * g.mem[i].ldw * 4 < (1L << 31);
    if (ok) return kRouteQuad;
  }
  if (g.M <= wave_dot_pref_m() && force != kRouteSkinny && wave_dot_supported(g.M, g.K, g.rank, g.r != nullptr || g.R != nullptr))
    return kRouteWaveDot;
  const bool skinny_ok = skinny_supported(g);
  if (skinny_ok && (g.M <= g_skinny_max_m.load(std::memory_order_relaxed) || force == kRouteSkinny || !gemm_supported(g)))
    return kRouteSkinny;
  if (gemm_supported(g)) return kRouteGemm;
  return kRouteGeneric;
}

// Runs one group through the chosen route.  Routes with a row capacity smaller than M walk the
// token rows in chunks (weights are re-read once per chunk).
int run_group(GroupDev g, int route, hipStream_t stream) {
  const int cus = num_cus();
  hipError_t e = hipSuccess;
  g.pub = nullptr;
  // r = x R^T ahead of the group as a launch of its own.  (Having every workgroup of the group kernel compute r for
  // itself was measured: the R -> r -> L.r dependency chain then stalls the weight stream for longer than the extra
  // launch costs.)
  const auto launch_projection = [&]() -> hipError_t {
    hipError_t pe;
    if (!proj_on_small_kernel(g.M, g.K, g.rank) && (g.K & 63) == 0 && aligned16(g.x) && aligned16(g.R))
      pe = launch_shared_proj_mfma(g.x, g.R, g.r_out, g.M, g.K, g.rank, cus, stream, g.ws, g.ws_bytes);
    else
      pe = launch_shared_proj_small(g.x, g.R, g.r_out, g.M, g.K, g.rank, stream);
    g.r = g.r_out;
    g.R = nullptr;
    g.pub = nullptr;
    return pe;
  };
  // Three and four token rows of a fused call with a workspace: the skinny kernel in its raw-code form where its launch
  // takes r along (one launch instead of the projection launch and the launch of the 2..4-row kernels); where it turns
  // the shape down (gate|up: no compute units left for the producers of r), the route chosen above.  Group call, us, this /
  // the route above, at 4 rows: 8B shapes q|k|v 8.6 / 10.0, o_proj 8.2 / 8.1, down_proj 15.9 / 15.8 (16.4 / 15.7 at three
  // rows: the stream-scheduled kernel keeps a long K); 14B shapes (rank 256) q|k|v 12.2 / 13.1, o_proj 9.6 / 11.4,
  // down_proj (on the 4x4x4 kernel) 20.7 / 26.7.
  if (g.R != nullptr && g.M >= 3 && g.M <= 4 && g_small_rows_in_launch.load(std::memory_order_relaxed) != 0 &&
      (route == kRouteQuad || route == kRouteStream || route == kRouteWaveDot || (route == kRouteQStream && g.K <= 8192)) && skinny_supported(g) &&
      skinny_raw_form(g) && skinny_proj_in_launch(g)) {
    g.pub = static_cast<unsigned long long*>(g.ws);
    g.pub_spin = (unsigned)g_proj_spin_limit.load(std::memory_order_relaxed);
    g.pub_mute = g_proj_in_launch.load(std::memory_order_relaxed) == 2;
    note_launch(0, 0, 0, "%s", "skinny_codes_mfma");
    e = launch_skinny(g, cus, stream, true);
    if (e == hipSuccess) return GLOWQ_OK;
    if (e != hipErrorNotReady) return fail(GLOWQ_ELAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    e = hipSuccess;
    g.pub = nullptr;
  }
  const bool skinny_route = route == kRouteSkinny || route == kRouteSkinnyRaw;
  if (g.R != nullptr && ((route == kRouteStream && proj_in_launch(g)) || ((skinny_route || route == kRouteSkinnyTiled) && skinny_proj_in_launch(g)))) {
    // single token on the stream GEMV, a handful of rows on the skinny kernel: workgroups in front of the group launch
    // produce r and hand it to the others through the workspace (stream_kernel.hpp, skinny.hip), no launch in front
    g.pub = static_cast<unsigned long long*>(g.ws);
    g.pub_spin = (unsigned)g_proj_spin_limit.load(std::memory_order_relaxed);
    g.pub_mute = g_proj_in_launch.load(std::memory_order_relaxed) == 2;
  } else if (g.R != nullptr) {
    e = launch_projection();
    if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "shared_proj launch failed: %s", hipGetErrorString(e));
  }
  // side streams are used only where every member brings one packed for the rank this launch applies
  bool packed = true;
  for (int i = 0; i < g.n_members; ++i) packed = packed && g.mem[i].side != nullptr && g.mem[i].side_rank == ((g.r || g.pub) ? g.rank : 0);
  if (!packed)
    for (int i = 0; i < g.n_members; ++i) g.mem[i].side = nullptr;
  static const char* const kRouteNames[] = {"wave_dot_gemv", "skinny_mfma", "tiled_mfma_gemm", "generic", "quad_mfma_gemv",
                                            "stream_gemv", "quad_stream_gemv", "skinny_codes_mfma", "skinny_tiled_mfma"};
  note_launch(0, 0, 0, "%s", (route >= 0 && route <= kRouteSkinnyTiled) ? kRouteNames[route] : "?");  // launchers that know more overwrite it
  if (route == kRouteStream) {
    e = launch_stream(g, cus, stream);
    if (e == hipErrorNotReady && g.pub != nullptr) {
      // the grid with the producers of r in front does not fit the chip in one go: the projection launch after all
      e = launch_projection();
      if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "shared_proj launch failed: %s", hipGetErrorString(e));
      e = launch_stream(g, cus, stream);
    }
  } else if (route == kRouteQStream) {
    e = launch_qstream(g, cus, stream);
  } else if (route == kRouteGemm) {
    e = launch_gemm(g, cus, stream);
  } else if (route == kRouteSkinnyTiled) {
    e = launch_skinny_tiled(g, cus, stream);
    if (e == hipErrorNotReady && g.pub != nullptr) {
      e = launch_projection();
      if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "shared_proj launch failed: %s", hipGetErrorString(e));
      e = launch_skinny_tiled(g, cus, stream);
    }
  } else if (skinny_route) {
    e = launch_skinny(g, cus, stream, route == kRouteSkinnyRaw);
    if (e == hipErrorNotReady && g.pub != nullptr) {
      e = launch_projection();
      if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "shared_proj launch failed: %s", hipGetErrorString(e));
      e = launch_skinny(g, cus, stream, route == kRouteSkinnyRaw);
    }
  } else {
    const int cap = (route == kRouteWaveDot) ? kWaveDotMaxM
                    : (route == kRouteQuad) ? quad_capacity(g.M, g.K, g.rank, g.r != nullptr) : 65535;
    long rows = 0;
    for (int i = 0; i < g.n_members; ++i) rows += g.mem[i].N;
    const int M = g.M;
    const half_t* x0 = g.x;
    const half_t* r0 = g.r;
    half_t* y0[GLOWQ_MAX_MEMBERS];
    for (int i = 0; i < g.n_members; ++i) y0[i] = g.mem[i].y;
    for (int m0 = 0; m0 < M && e == hipSuccess; m0 += cap) {
      g.M = (M - m0 < cap) ? M - m0 : cap;
      g.x = x0 + (size_t)m0 * g.K;
      g.r = r0 ? r0 + (size_t)m0 * g.rank : nullptr;
      for (int i = 0; i < g.n_members; ++i) g.mem[i].y = y0[i] + (size_t)m0 * g.mem[i].ldy;
      e = (route == kRouteWaveDot) ? launch_wave_dot(g, g.M == 1 ? wave_dot_rows_single(rows) : wave_dot_rows(rows), cus, stream)
          : (route == kRouteQuad)  ? launch_quad(g, cus, stream)
                                   : launch_generic(g, cus, stream);
    }
  }
  if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
  return GLOWQ_OK;
}

int forward_single(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros, void* y, int M,
                   int K, int N, int group_size, int ldw, int lds, int ldz, int force, void* stream) {
  int rc = check_common(x, M, K, group_size);
  if (rc) return rc;
  glowq_member_t mem;
  memset(&mem, 0, sizeof(mem));
  mem.qweight = qweight;
  mem.scales = scales;
  mem.qzeros = qzeros;
  mem.y = y;
  mem.N = N;
  mem.ldw_i32 = ldw;
  mem.lds = lds;
  mem.ldz_i32 = ldz;
  mem.ldy = N;
  rc = check_member(mem, K, group_size, 0);
  if (rc) return rc;
  GroupDev g;
  memset(&g, 0, sizeof(g));
  g.x = static_cast<const half_t*>(x);
  g.n_members = 1;
  g.M = M;
  g.K = K;
  g.group_size = group_size;
  to_dev(mem, g.mem[0]);
  return run_group(g, pick_route(g, force), static_cast<hipStream_t>(stream));
}

}  // namespace

extern "C" {

int glowq_version(void) { return 102; }

const char* glowq_last_error(void) { return g_err; }

int glowq_w4a16_gemv_forward(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                             void* y, int M, int K, int N, int group_size, int ldw_i32, int lds, int ldz_i32,
                             void* stream) {
  return forward_single(x, qweight, scales, qzeros, y, M, K, N, group_size, ldw_i32, lds, ldz_i32, -1, stream);
}

int glowq_w4a16_gemm_forward(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                             void* y, int M, int K, int N, int group_size, int split_k_iters, int ldw_i32, int lds,
                             int ldz_i32, void* stream) {
  (void)split_k_iters;
  return forward_single(x, qweight, scales, qzeros, y, M, K, N, group_size, ldw_i32, lds, ldz_i32, kRouteGemm, stream);
}

int glowq_w4a16_dequant(const int32_t* qweight, const void* scales, const int32_t* qzeros, void* out, int N, int K,
                        int group_size, int ldw_i32, int lds, int ldz_i32, void* stream) {
  if (!qweight || !scales || !qzeros || !out) return fail(GLOWQ_EINVAL, "dequant: NULL pointer");
  if (N <= 0 || K <= 0) return fail(GLOWQ_EINVAL, "dequant: N and K must be > 0");
  if (group_size <= 0 || group_size % 8 != 0) return fail(GLOWQ_EINVAL, "group_size must be a multiple of 8");
  const int groups = (K + group_size - 1) / group_size;
  if (lds < groups) return fail(GLOWQ_ESHAPE, "scales groups mismatch");
  if (ldw_i32 < (K + 7) / 8) return fail(GLOWQ_ESHAPE, "qweight packed cols too small");
  if (ldz_i32 < (groups + 7) / 8) return fail(GLOWQ_ESHAPE, "qzeros packed cols too small");
  hipError_t e = launch_dequant(qweight, static_cast<const half_t*>(scales), qzeros, static_cast<half_t*>(out), N, K,
                                group_size, ldw_i32, lds, ldz_i32, num_cus(), static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "dequant launch failed: %s", hipGetErrorString(e));
  return GLOWQ_OK;
}

int glowq_w4a16_group_forward_chained(const void* x, const void* r, const glowq_member_t* members, int n_members, int K,
                                      int group_size, int rank, float alpha, const glowq_chain_t* chain, void* stream) {
  int rc = check_common(x, 1, K, group_size);
  if (rc) return rc;
  if (chain == nullptr || members == nullptr) return fail(GLOWQ_EINVAL, "chained: members and chain must not be NULL");
  if (n_members < 1 || n_members > GLOWQ_MAX_MEMBERS) return fail(GLOWQ_EINVAL, "n_members must be 1..%d", GLOWQ_MAX_MEMBERS);
  const int pro = chain->prologue, epi = chain->epilogue;
  if (!chain_combination_supported(pro, epi))
    return fail(GLOWQ_EUNSUPPORTED, "chained: prologue %d with epilogue %d is not served", pro, epi);
  if (rank <= 0) return fail(GLOWQ_EUNSUPPORTED, "chained: needs a correction (rank > 0)");
  if (pro == GLOWQ_CHAIN_PRO_PLAIN && r == nullptr) return fail(GLOWQ_EINVAL, "chained: the plain prologue needs r");
  if (pro != GLOWQ_CHAIN_PRO_PLAIN && (chain->acc_in == nullptr || (reinterpret_cast<uintptr_t>(chain->acc_in) & 7u)))
    return fail(GLOWQ_EINVAL, "chained: acc_in must be an 8-byte aligned device pointer");
  if (pro == GLOWQ_CHAIN_PRO_NORM_ACC && (chain->norm_weight == nullptr || !aligned16(chain->norm_weight)))
    return fail(GLOWQ_EINVAL, "chained: norm_weight must be a 16-byte aligned device pointer");
  if (epi == GLOWQ_CHAIN_EPI_RESIDUAL && (n_members != 1 || chain->resid == nullptr || !aligned4(chain->resid)))
    return fail(GLOWQ_EINVAL, "chained: the residual epilogue takes one member and a 4-byte aligned resid");
  if (epi == GLOWQ_CHAIN_EPI_SWIGLU && (n_members != 2 || members[0].N != members[1].N || chain->act == nullptr))
    return fail(GLOWQ_EINVAL, "chained: the SwiGLU epilogue takes two members of equal N and act");
  if (chain->next_Rt != nullptr && (chain->acc_out == nullptr || (reinterpret_cast<uintptr_t>(chain->acc_out) & 7u) || !aligned4(chain->next_Rt)))
    return fail(GLOWQ_EINVAL, "chained: next_Rt needs an 8-byte aligned acc_out and 4-byte alignment itself");
  GroupDev g;
  memset(&g, 0, sizeof(g));
  g.x = static_cast<const half_t*>(x);
  g.r = static_cast<const half_t*>(r);
  g.n_members = n_members;
  g.M = 1;
  g.K = K;
  g.group_size = group_size;
  g.rank = rank;
  g.alpha = alpha;
  for (int i = 0; i < n_members; ++i) {
    glowq_member_t m = members[i];
    const bool y_optional = epi != GLOWQ_CHAIN_EPI_NONE && m.y == nullptr;
    if (y_optional) m.y = const_cast<void*>(x);  // (passes the pointer check; restored below)
    if (m.ldy == 0) m.ldy = m.N;
    rc = check_member(m, K, group_size, i);
    if (rc) return rc;
    if (m.L == nullptr) return fail(GLOWQ_EUNSUPPORTED, "chained: member %d has no L", i);
    if (y_optional) m.y = nullptr;
    to_dev(m, g.mem[i]);
    g.mem[i].side = nullptr;
  }
  if (g.r == nullptr) g.r = g.x;  // (the layout check wants an r for a corrected group; chained prologues do not read it)
  const bool ok = fast_layout(g) && stream_supported(g);
  if (pro != GLOWQ_CHAIN_PRO_PLAIN) g.r = nullptr;
  if (!ok) return fail(GLOWQ_EUNSUPPORTED, "chained: shape outside the stream GEMV (K=%d, group_size=%d, rank=%d)", K, group_size, rank);
  streamk::ChainDev ch;
  memset(&ch, 0, sizeof(ch));
  ch.norm_w = static_cast<const half_t*>(chain->norm_weight);
  ch.acc_in = static_cast<const long long*>(chain->acc_in);
  ch.resid = static_cast<half_t*>(chain->resid);
  ch.next_w = static_cast<const half_t*>(chain->next_norm_weight);
  ch.next_rt = static_cast<const half_t*>(chain->next_Rt);
  ch.acc_out = static_cast<long long*>(chain->acc_out);
  ch.act = static_cast<half_t*>(chain->act);
  ch.eps = chain->eps;
  hipError_t e = launch_stream_chained(g, ch, pro, epi, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "chained launch failed: %s", hipGetErrorString(e));
  return GLOWQ_OK;
}

size_t glowq_side_bytes(int N, int K, int group_size, int rank) {
  SideLayout lay;
  if (N <= 0 || !side_layout(K, group_size, rank, lay)) return 0;
  return (size_t)((N + 1) >> 1) * side_block_bytes(lay);
}

int glowq_pack_side(const void* scales, const int32_t* qzeros, const void* L, void* side, int N, int K, int group_size,
                    int rank, int lds, int ldz_i32, void* stream) {
  if (!scales || !qzeros || !side) return fail(GLOWQ_EINVAL, "pack_side: NULL pointer");
  if (glowq_side_bytes(N, K, group_size, rank) == 0)
    return fail(GLOWQ_EUNSUPPORTED, "pack_side: no side stream for N=%d K=%d group_size=%d rank=%d", N, K, group_size, rank);
  const int groups = (K + group_size - 1) / group_size;
  if (lds < groups || ldz_i32 < (groups + 7) / 8) return fail(GLOWQ_ESHAPE, "pack_side: scales / qzeros rows too short");
  if (L != nullptr && (rank <= 0 || !aligned4(L))) return fail(GLOWQ_EINVAL, "pack_side: L needs a positive rank and 4-byte alignment");
  if (!aligned16(side)) return fail(GLOWQ_EINVAL, "pack_side: side must be 16-byte aligned");
  hipError_t e = launch_pack_side(static_cast<const half_t*>(scales), qzeros, static_cast<const half_t*>(L), side, N, K,
                                  group_size, rank, lds, ldz_i32, num_cus(), static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "pack_side launch failed: %s", hipGetErrorString(e));
  return GLOWQ_OK;
}

size_t glowq_tiled_bytes(int N, int K, int group_size) {
  return (N > 0 && tiled::applies(K, group_size)) ? tiled::weight_bytes(N, K) : 0;
}

int glowq_pack_tiled(const int32_t* qweight, const void* scales, const int32_t* qzeros, void* out, int N, int K, int group_size,
                     int ldw_i32, int lds, int ldz_i32, void* stream) {
  if (!qweight || !scales || !qzeros || !out) return fail(GLOWQ_EINVAL, "pack_tiled: NULL pointer");
  if (glowq_tiled_bytes(N, K, group_size) == 0)
    return fail(GLOWQ_EUNSUPPORTED, "pack_tiled: no tiled layout for N=%d K=%d group_size=%d", N, K, group_size);
  const int groups = K / group_size;
  if (ldw_i32 < K / 8 || lds < groups || ldz_i32 < (groups + 7) / 8) return fail(GLOWQ_ESHAPE, "pack_tiled: qweight / scales / qzeros rows too short");
  if (!aligned16(out)) return fail(GLOWQ_EINVAL, "pack_tiled: the output must be 16-byte aligned");
  hipError_t e = launch_pack_tiled(qweight, static_cast<const half_t*>(scales), qzeros, out, N, K, group_size, ldw_i32, lds, ldz_i32,
                                   num_cus(), static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "pack_tiled launch failed: %s", hipGetErrorString(e));
  return GLOWQ_OK;
}

size_t glowq_tiled_left_bytes(int N, int rank) { return (N > 0 && rank >= 8 && (rank & 7) == 0) ? tiled::left_bytes(N, rank) : 0; }

int glowq_pack_tiled_left(const void* L, void* out, int N, int rank, void* stream) {
  if (!L || !out) return fail(GLOWQ_EINVAL, "pack_tiled_left: NULL pointer");
  if (glowq_tiled_left_bytes(N, rank) == 0) return fail(GLOWQ_EUNSUPPORTED, "pack_tiled_left: no tiled layout for N=%d rank=%d", N, rank);
  if (!aligned16(out)) return fail(GLOWQ_EINVAL, "pack_tiled_left: the output must be 16-byte aligned");
  hipError_t e = launch_pack_tiled_left(static_cast<const half_t*>(L), out, N, rank, num_cus(), static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "pack_tiled_left launch failed: %s", hipGetErrorString(e));
  return GLOWQ_OK;
}

int glowq_unpack_int4(const int32_t* packed, uint8_t* codes, int rows, int total_vals, int ld_i32, void* stream) {
  if (!packed || !codes) return fail(GLOWQ_EINVAL, "unpack: NULL pointer");
  if (rows <= 0 || total_vals <= 0) return fail(GLOWQ_EINVAL, "unpack: rows and total_vals must be > 0");
  if (ld_i32 < (total_vals + 7) / 8) return fail(GLOWQ_ESHAPE, "unpack: packed cols too small");
  hipError_t e = launch_unpack(packed, codes, rows, total_vals, ld_i32, num_cus(), static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "unpack launch failed: %s", hipGetErrorString(e));
  return GLOWQ_OK;
}

static int shared_proj_impl(const void* x, const void* R, void* r, int M, int K, int rank, void* ws, size_t ws_bytes,
                            void* stream) {
  if (!x || !R || !r) return fail(GLOWQ_EINVAL, "shared_proj: NULL pointer");
  if (M <= 0 || K <= 0 || rank <= 0) return fail(GLOWQ_EINVAL, "shared_proj: M, K and rank must be > 0");
  const half_t* xp = static_cast<const half_t*>(x);
  const half_t* Rp = static_cast<const half_t*>(R);
  half_t* rp = static_cast<half_t*>(r);
  hipError_t e;
  if (!proj_on_small_kernel(M, K, rank) && (K & 63) == 0 && aligned16(x) && aligned16(R)) {
    e = launch_shared_proj_mfma(xp, Rp, rp, M, K, rank, num_cus(), static_cast<hipStream_t>(stream), ws, ws_bytes);
  } else {
    if ((K & 7) == 0 && (!aligned16(x) || !aligned16(R)))
      return fail(GLOWQ_EUNSUPPORTED, "shared_proj: x and R must be 16-byte aligned");
    e = launch_shared_proj_small(xp, Rp, rp, M, K, rank, static_cast<hipStream_t>(stream));
  }
  if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "shared_proj launch failed: %s", hipGetErrorString(e));
  return GLOWQ_OK;
}

int glowq_shared_proj(const void* x, const void* R, void* r, int M, int K, int rank, void* stream) {
  return shared_proj_impl(x, R, r, M, K, rank, nullptr, 0, stream);
}

int glowq_shared_proj_ws(const void* x, const void* R, void* r, int M, int K, int rank, void* workspace,
                         size_t workspace_bytes, void* stream) {
  return shared_proj_impl(x, R, r, M, K, rank, workspace, workspace_bytes, stream);
}

size_t glowq_proj_workspace_bytes(int M, int K, int rank) { return proj_workspace_bytes(M, K, rank, num_cus()); }

static int group_forward_impl(const void* x, const void* r, const glowq_member_t* members, int n_members, int M, int K,
                              int group_size, int rank, float alpha, void* ws, size_t ws_bytes, void* stream) {
  int rc = check_common(x, M, K, group_size);
  if (rc) return rc;
  if (members == nullptr || n_members < 1 || n_members > GLOWQ_MAX_MEMBERS)
    return fail(GLOWQ_EINVAL, "group_forward: n_members must be 1..%d", GLOWQ_MAX_MEMBERS);
  GroupDev g;
  memset(&g, 0, sizeof(g));
  bool any_L = false;
  for (int i = 0; i < n_members; ++i) {
    rc = check_member(members[i], K, group_size, i);
    if (rc) return rc;
    to_dev(members[i], g.mem[i]);
    any_L = any_L || members[i].L != nullptr;
  }
  if (any_L && alpha != 0.0f) {
    if (r == nullptr) return fail(GLOWQ_EINVAL, "group_forward: a member has L but r is NULL");
    if (rank <= 0) return fail(GLOWQ_EINVAL, "group_forward: rank must be > 0 when a correction is applied");
    g.r = static_cast<const half_t*>(r);
    g.rank = rank;
    g.alpha = alpha;
  } else {
    for (int i = 0; i < n_members; ++i) g.mem[i].L = nullptr;  // alpha == 0: the reference returns z untouched
  }
  g.x = static_cast<const half_t*>(x);
  g.ws = ws;
  g.ws_bytes = ws_bytes;
  g.n_members = n_members;
  g.M = M;
  g.K = K;
  g.group_size = group_size;
  return run_group(g, pick_route(g, -1), static_cast<hipStream_t>(stream));
}

int glowq_w4a16_group_forward(const void* x, const void* r, const glowq_member_t* members, int n_members, int M,
                              int K, int group_size, int rank, float alpha, void* stream) {
  return group_forward_impl(x, r, members, n_members, M, K, group_size, rank, alpha, nullptr, 0, stream);
}

int glowq_w4a16_group_forward_ws(const void* x, const void* r, const glowq_member_t* members, int n_members, int M,
                                 int K, int group_size, int rank, float alpha, void* workspace, size_t workspace_bytes,
                                 void* stream) {
  return group_forward_impl(x, r, members, n_members, M, K, group_size, rank, alpha, workspace, workspace_bytes, stream);
}

static int group_forward_fused_impl(const void* x, const void* R, void* r_out, const glowq_member_t* members,
                                    int n_members, int M, int K, int group_size, int rank, float alpha, void* ws,
                                    size_t ws_bytes, void* stream) {
  int rc = check_common(x, M, K, group_size);
  if (rc) return rc;
  if (members == nullptr || n_members < 1 || n_members > GLOWQ_MAX_MEMBERS)
    return fail(GLOWQ_EINVAL, "group_forward_fused: n_members must be 1..%d", GLOWQ_MAX_MEMBERS);
  if (R == nullptr || r_out == nullptr || rank <= 0)
    return fail(GLOWQ_EINVAL, "group_forward_fused: R, r_out and a positive rank are required");
  if ((K & 7) == 0 && (!aligned16(x) || !aligned16(R)))
    return fail(GLOWQ_EUNSUPPORTED, "group_forward_fused: x and R must be 16-byte aligned");
  GroupDev g;
  memset(&g, 0, sizeof(g));
  for (int i = 0; i < n_members; ++i) {
    rc = check_member(members[i], K, group_size, i);
    if (rc) return rc;
    to_dev(members[i], g.mem[i]);
  }
  g.x = static_cast<const half_t*>(x);
  g.R = static_cast<const half_t*>(R);
  g.r_out = static_cast<half_t*>(r_out);
  g.ws = ws;
  g.ws_bytes = ws_bytes;
  g.rank = rank;
  g.alpha = alpha;
  g.n_members = n_members;
  g.M = M;
  g.K = K;
  g.group_size = group_size;
  if (alpha == 0.0f)
    for (int i = 0; i < n_members; ++i) g.mem[i].L = nullptr;  // r is still produced: callers cache it
  return run_group(g, pick_route(g, -1), static_cast<hipStream_t>(stream));
}

int glowq_w4a16_group_forward_fused(const void* x, const void* R, void* r_out, const glowq_member_t* members,
                                    int n_members, int M, int K, int group_size, int rank, float alpha, void* stream) {
  return group_forward_fused_impl(x, R, r_out, members, n_members, M, K, group_size, rank, alpha, nullptr, 0, stream);
}

int glowq_w4a16_group_forward_fused_ws(const void* x, const void* R, void* r_out, const glowq_member_t* members,
                                       int n_members, int M, int K, int group_size, int rank, float alpha,
                                       void* workspace, size_t workspace_bytes, void* stream) {
  return group_forward_fused_impl(x, R, r_out, members, n_members, M, K, group_size, rank, alpha, workspace,
                                  workspace_bytes, stream);
}

int glowq_w4a16_group_forward_fused_static(const void* x, const void* R, void* r_out, const glowq_member_t* members,
                                           int n_members, int M, int K, int group_size, int rank, float alpha,
                                           void* stream) {
  if (M > GLOWQ_STATIC_MAX_ROWS)
    return fail(GLOWQ_EUNSUPPORTED, "group_forward_fused_static: %d token rows, the static scratch serves at most %d", M,
                GLOWQ_STATIC_MAX_ROWS);
  // what the users of the workspace ask for at this shape: the projection's split of K, the skinny kernel's and that of
  // the kernel that streams the tiled copy (each states its own bound next to its split rule)
  size_t need = (M > 0 && K > 0 && rank > 0) ? proj_workspace_bytes(M, K, rank, num_cus()) : 0;
  // (the skinny kernel that computes r itself keeps its hand-over words in front of the partial tiles)
  need = std::max(need, glowq::skinny_split_workspace_bytes(M, num_cus()) + (M >= 2 && M <= 32 ? kSkinnyHandoverBytes : 0));
  bool any_tiled = false;
  for (int i = 0; members != nullptr && i < n_members && i < GLOWQ_MAX_MEMBERS; ++i) any_tiled = any_tiled || members[i].tiled != nullptr;
  if (any_tiled) need = std::max(need, glowq::tiled_split_workspace_bytes(M, num_cus()));
  if (M == 1 && rank > 0) need = std::max(need, kProjHandoverBytes);  // hand-over words of the projection inside the launch
  if (need > kStaticScratchBytes)
    return fail(GLOWQ_EUNSUPPORTED, "group_forward_fused_static: this shape wants %zu bytes of scratch, the static buffer holds %zu",
                need, kStaticScratchBytes);
  void* ws = static_scratch(false);
  if (ws == nullptr) {
    // first use on this device: the lookup must not run under a stream capture
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      return fail(GLOWQ_EUNSUPPORTED, "group_forward_fused_static: call glowq_static_scratch_prepare() on this device before capturing");
    ws = static_scratch();
  }
  if (ws == nullptr) return fail(GLOWQ_ELAUNCH, "group_forward_fused_static: the address of the static scratch is not available");
  return group_forward_fused_impl(x, R, r_out, members, n_members, M, K, group_size, rank, alpha, ws, kStaticScratchBytes,
                                  stream);
}

size_t glowq_static_scratch_bytes(void) { return kStaticScratchBytes; }

int glowq_static_scratch_prepare(void) {
  if (static_scratch() == nullptr) return fail(GLOWQ_ELAUNCH, "static_scratch_prepare: the address of the static scratch is not available");
  return GLOWQ_OK;
}

static int route_query(int M, int K, int N, int group_size, int ldw_i32, bool with_tiled) {
  GroupDev g;
  memset(&g, 0, sizeof(g));
  g.n_members = 1;
  g.M = M;
  g.K = K;
  g.group_size = group_size;
  g.mem[0].N = N;
  g.mem[0].ldw = ldw_i32;
  if (with_tiled && tiled::applies(K, group_size)) g.mem[0].tiled = reinterpret_cast<const void*>(uintptr_t{16});  // never read
  return pick_route(g, -1);
}

int glowq_w4a16_route(int M, int K, int N, int group_size, int ldw_i32) { return route_query(M, K, N, group_size, ldw_i32, false); }

int glowq_w4a16_route_tiled(int M, int K, int N, int group_size, int ldw_i32) { return route_query(M, K, N, group_size, ldw_i32, true); }


int glowq_last_launch(char* kernel, size_t bytes, int* grid_x, int* grid_y, int* block) {
  if (kernel != nullptr && bytes > 0) snprintf(kernel, bytes, "%s", g_note.kernel);
  if (grid_x) *grid_x = g_note.grid_x;
  if (grid_y) *grid_y = g_note.grid_y;
  if (block) *block = g_note.block;
  return GLOWQ_OK;
}

int glowq_probe_stream_read(const void* src, size_t bytes, void* sink, int grid, int block, void* stream) {
  if (!src || !sink || grid <= 0 || block <= 0 || block > 1024 || (block & 63) != 0 || !aligned16(src) || (bytes & 15) != 0)
    return fail(GLOWQ_EINVAL, "probe_stream_read: 16-byte aligned source, whole 16-byte units, a grid and a workgroup of whole waves");
  hipError_t e = launch_probe_read(src, bytes, sink, grid, block, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "probe_stream_read launch failed: %s", hipGetErrorString(e));
  return GLOWQ_OK;
}

int glowq_probe_empty_launch(int grid, int block, void* stream) {
  if (grid <= 0 || block <= 0 || block > 1024) return fail(GLOWQ_EINVAL, "probe_empty_launch: a grid and a workgroup size");
  hipError_t e = launch_probe_empty(grid, block, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(GLOWQ_ELAUNCH, "probe_empty_launch launch failed: %s", hipGetErrorString(e));
  return GLOWQ_OK;
}

int glowq_set_tuning(const char* key, int value) {
  if (key == nullptr) return fail(GLOWQ_EINVAL, "tuning key must not be NULL");
  std::atomic<int>* slot = nullptr;
  int lo = 0, hi = 16;
  if (strcmp(key, "wave_dot_max_m") == 0) { slot = &g_wave_dot_max_m; hi = kWaveDotMaxM; }
  else if (strcmp(key, "quad_max_m") == 0) { slot = &g_quad_max_m; }
  else if (strcmp(key, "quad_min_m") == 0) { slot = &g_quad_min_m; lo = 1; }
  else if (strcmp(key, "skinny_max_m") == 0) { slot = &g_skinny_max_m; hi = 64; }
  else if (strcmp(key, "small_group_mb") == 0) { slot = &g_small_group_mb; hi = 4096; }
  else if (strcmp(key, "stream_max_m") == 0) { slot = &g_stream_max_m; hi = 4; }
  else if (strcmp(key, "qstream_max_m") == 0) { slot = &g_qstream_max_m; hi = 4; }
  else if (strcmp(key, "qstream_shape_rule") == 0) { slot = &g_qstream_shape_rule; hi = 1; }
  else if (strcmp(key, "skinny_codes_max_m") == 0) { slot = &g_skinny_codes_max_m; hi = 64; }
  else if (strcmp(key, "stream_shape_rule") == 0) { slot = &g_stream_shape_rule; hi = 1; }
  else if (strcmp(key, "tiled_min_m") == 0) { slot = &g_tiled_min_m; lo = 1; hi = 64; }
  else if (strcmp(key, "tiled_max_m") == 0) { slot = &g_tiled_max_m; hi = 64; }
  else if (strcmp(key, "tiled_shape_rule") == 0) { slot = &g_tiled_shape_rule; hi = 1; }
  else if (strcmp(key, "proj_in_launch") == 0) { slot = &g_proj_in_launch; hi = 2; }
  else if (strcmp(key, "proj_spin_limit") == 0) { slot = &g_proj_spin_limit; hi = 1 << 24; }
  else if (strcmp(key, "small_rows_in_launch") == 0) { slot = &g_small_rows_in_launch; hi = 1; }
  if (slot == nullptr) return fail(GLOWQ_EINVAL, "unknown tuning key '%s'", key);
  if (value < lo || value > hi) return fail(GLOWQ_EINVAL, "tuning key '%s': value %d outside [%d, %d]", key, value, lo, hi);
  return slot->exchange(value);
}
}  // extern "C"
