// Host side of the C ABI declared in include/pplx_a2a.h: world / rank-handle
// lifecycle, argument checks, table binding and kernel sequencing.
//
// Takes the place of the reference's host classes
// (csrc/all_to_all/all_to_all.cpp:8-40, csrc/all_to_all/intranode.cpp:11-162) and
// of the argument checks in csrc/bindings/all_to_all_ops.cpp:122-196,238-311 that
// do not depend on torch types.  Failures are reported as status codes plus a
// thread-local message; nothing here exits or traps.
#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "a2a_device.h"
#include "pplx_a2a.h"

// Profiler ranges around the launch sequences, like the reference's nvtxRangePush("dispatch") /
// ("combine") (csrc/all_to_all/intranode_dispatch.cu:354,389, intranode_combine.cu:245,265).
// The build links the roctx library when its header is installed.
#ifdef PPLX_A2A_ROCTX
#include <rocprofiler-sdk-roctx/roctx.h>
#endif

using namespace pplx_amd;

namespace {

thread_local std::string g_last_error;

int fail(int status, const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return status;
}

#define HIP_TRY(expr)                                                                        \
  do {                                                                                       \
    hipError_t err_ = (expr);                                                                \
    if (err_ != hipSuccess)                                                                  \
      return fail(PPLX_A2A_HIP_ERROR, "%s failed: %s", #expr, hipGetErrorString(err_));      \
  } while (0)

#define LAUNCH_TRY(expr)                                                                     \
  do {                                                                                       \
    int err_ = (expr);                                                                       \
    if (err_ != 0)                                                                           \
      return fail(PPLX_A2A_HIP_ERROR, "%s failed: %s", #expr,                                \
                  hipGetErrorString((hipError_t)err_));                                      \
  } while (0)

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

class ProfilerRange {
 public:
  explicit ProfilerRange(const char *name) {
#ifdef PPLX_A2A_ROCTX
    roctxRangePushA(name);
#else
    (void)name;
#endif
  }
  ~ProfilerRange() {
#ifdef PPLX_A2A_ROCTX
    roctxRangePop();
#endif
  }
  ProfilerRange(const ProfilerRange &) = delete;
  ProfilerRange &operator=(const ProfilerRange &) = delete;
};

// Restores the caller's current device on scope exit.
class DeviceScope {
 public:
  explicit DeviceScope(int device) {
    ok_ = hipGetDevice(&prev_) == hipSuccess;
    if (ok_ && prev_ != device) ok_ = hipSetDevice(device) == hipSuccess;
    switched_ = ok_ && prev_ != device;
  }
  ~DeviceScope() {
    if (switched_) (void)hipSetDevice(prev_);
  }
  bool ok() const { return ok_; }

 private:
  int prev_ = 0;
  bool ok_ = false;
  bool switched_ = false;
};

}  // namespace

struct pplx_a2a_world {
  pplx_a2a_config_t cfg;
  int device = 0;
  WorldDev dev{};
  std::mutex mu;
  int attached = 0;

  // Arguments recorded for the step being assembled, and which ranks have called.
  std::vector<DispatchRank> pend_dispatch;
  std::vector<CombineRank> pend_combine;
  std::vector<uint8_t> arrived_dispatch, arrived_combine;
  uint32_t n_arrived_dispatch = 0, n_arrived_combine = 0;
  int combine_in_dtype = -1, combine_out_dtype = -1;

  // What the device tables currently hold; trusted only while no stream capture
  // has recorded a bind (a replayed graph rewrites the tables behind our back).
  std::vector<DispatchRank> bound_dispatch;
  std::vector<CombineRank> bound_combine;
  bool bound_dispatch_valid = false, bound_combine_valid = false;
  bool captured_once = false;
  // Capture session that recorded the last bind of each table (0 = an eager bind).
  unsigned long long bind_capture_dispatch = 0, bind_capture_combine = 0;

  // Streams the ranks of the step being assembled called on (per-rank calls), and the events
  // that order them against the stream of the last caller, which gets the kernels.
  std::vector<void *> stream_dispatch, stream_combine;
  std::vector<hipEvent_t> rank_events;  // [R]
  hipEvent_t done_event = nullptr;

  // Split send / recv mode: staging is allocated by pplx_a2a_world_reserve_split; the masks
  // record which ranks have made which call of the step in flight.
  SplitDev split{};
  bool split_ready = false;
  std::vector<uint8_t> dsend, drecv, csend, crecv;
  uint32_t n_dsend = 0, n_drecv = 0, n_csend = 0, n_crecv = 0;
  int split_in_dtype = -1, split_out_dtype = -1;  // dtypes of the combine SEND phase in flight
};

struct pplx_a2a {
  pplx_a2a_world *world;
  uint32_t rank;
};

struct pplx_a2a_graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

namespace {

int check_config(const pplx_a2a_config_t &c) {
  if (c.world_size == 0 || c.dp_size == 0)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "world_size and dp_size must be positive");
  if (c.world_size % c.dp_size != 0)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "world_size must be a multiple of dp_size");
  if (c.num_experts == 0 || c.num_experts % c.world_size != 0)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "num_experts must be a positive multiple of world_size");
  if (c.experts_per_token == 0 || c.experts_per_token > kWave || c.experts_per_token > c.num_experts)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "experts_per_token must be in [1, min(64, num_experts)]");
  if (c.max_num_tokens == 0)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "max_num_tokens must be positive");
  // csrc/all_to_all/all_to_all.cpp:32-39
  if (c.hidden_dim_bytes == 0 || c.hidden_dim_bytes % 16 != 0)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "invalid hidden dim bytes");
  if (c.hidden_dim_scale_bytes % 16 != 0)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "invalid hidden dim scale bytes");
  if (c.hidden_dim_scale_bytes > c.hidden_dim_bytes)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "invalid hidden dim bytes");
  if (c.hidden_dim == 0)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "hidden_dim must be positive");
  const uint64_t groups = c.world_size / c.dp_size;
  if (groups * c.max_num_tokens > (1ull << 30) ||
      groups * c.max_num_tokens * c.experts_per_token > (1ull << 31) ||
      c.hidden_dim_bytes > (1ull << 30) || c.num_experts > 5461 ||
      // one wave per (rank, token, 512-element segment) / per (token, pick share): 32-bit grids
      (uint64_t)c.world_size * c.max_num_tokens * ((c.hidden_dim + 511) / 512) > (1ull << 32) ||
      groups * c.max_num_tokens * 64 > (1ull << 32))
    return fail(PPLX_A2A_UNSUPPORTED, "geometry exceeds the limits of this build");
  return PPLX_A2A_OK;
}

// LDS bytes per CU of `device` (0 when the runtime will not say), looked up once per device.
uint32_t lds_per_cu_of(int device) {
  static std::mutex mu;
  static int cached[64];
  static bool known[64];
  if (device < 0 || device >= 64) return 0;
  std::lock_guard<std::mutex> lock(mu);
  if (!known[device]) {
    int bytes = 0;
    if (hipDeviceGetAttribute(&bytes, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, device) != hipSuccess)
      bytes = 0;
    cached[device] = bytes > 0 ? bytes : 0;
    known[device] = true;
  }
  return (uint32_t)cached[device];
}

// The geometry part of a WorldDev (everything but the pointers) for a checked configuration.
void fill_geometry(const pplx_a2a_config_t &cfg, WorldDev &d) {
  d.R = cfg.world_size;
  d.dp = cfg.dp_size;
  d.G = d.R / d.dp;
  d.M = (uint32_t)cfg.max_num_tokens;
  d.E = (uint32_t)cfg.num_experts;
  d.L = d.E / d.R;
  d.K = (uint32_t)cfg.experts_per_token;
  d.H = (uint32_t)cfg.hidden_dim;
  d.Hb = (uint32_t)cfg.hidden_dim_bytes;
  d.S = (uint32_t)(cfg.hidden_dim_scale_bytes / 4);
  d.by_M = make_fast_div(d.M);
  d.by_dp = make_fast_div(d.dp);
  d.by_L = make_fast_div(d.L);
  d.by_K = make_fast_div(d.K);
  // Routing tiles of a whole step: small enough that a step has a few hundred of them (a tile
  // is one workgroup, and routing is a chain of short launches that only parallelism shortens),
  // at most 16 chunks of 64 tokens, and such that the LDS tables fit 64 KiB.
  const uint64_t step_chunks = ((uint64_t)d.G * d.M + kWave - 1) / kWave;
  // A step of up to 1024 tokens is a single tile (one launch instead of three).
  d.tile_chunks = 1;
  if (step_chunks <= 16) {
    while (d.tile_chunks < step_chunks) d.tile_chunks *= 2;
  } else {
    while (d.tile_chunks < 16 && step_chunks / d.tile_chunks > 256) d.tile_chunks *= 2;
  }
  while (d.tile_chunks > 1 && route_lds_bytes(d.E, d.tile_chunks) > 65536u) d.tile_chunks /= 2;
  const uint64_t tile_tokens = (uint64_t)d.tile_chunks * kWave;
  d.num_tiles = (uint32_t)(((uint64_t)d.G * d.M + tile_tokens - 1) / tile_tokens);
}

int convert_dispatch(const WorldDev &geo, uint32_t rank, const pplx_a2a_dispatch_args_t &a,
                     DispatchRank *out) {
  const uint32_t S = geo.S;
  if (!a.out_expert_num_tokens)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: out_expert_num_tokens is NULL", rank);
  if (!a.out_expert_x) return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: out_expert_x is NULL", rank);
  if (a.m > 0 && (!a.dp_x || !a.indices))
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: dp_x / indices is NULL with m > 0", rank);
  if (S > 0 && !a.out_expert_x_scale)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: out_expert_x_scale is NULL but scales are configured", rank);
  if (S > 0 && a.m > 0 && !a.dp_x_scale)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: dp_x_scale is NULL but scales are configured", rank);
  if (!aligned16(a.out_expert_x) || a.out_expert_x_stride_row % 16 || a.out_expert_x_stride_expert % 16)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: out_expert_x must be 16-byte aligned with 16-byte strides", rank);
  if (!aligned16(a.dp_x) || a.dp_x_stride_row % 16)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: dp_x must be 16-byte aligned with a 16-byte row stride", rank);
  if (a.out_expert_x_rows < 0)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: out_expert_x_rows is negative", rank);
  // csrc/all_to_all/intranode_dispatch.cu:65 asserts numSendTokens <= maxNumTokens; a device-side
  // bound_m beyond the limit is clamped and reported through the fault word instead.
  if (!a.bound_m && a.m > geo.M)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: %u tokens exceed max_num_tokens %u", rank, a.m, geo.M);
  const uint64_t rows = a.out_expert_x_rows ? (uint64_t)a.out_expert_x_rows : (uint64_t)geo.M * geo.G;
  DispatchRank d{};
  d.out_num_tokens = a.out_expert_num_tokens;
  d.out_num_tokens_stride = a.out_expert_num_tokens_stride;
  d.expert_x = static_cast<uint8_t *>(a.out_expert_x);
  d.x_stride_row = a.out_expert_x_stride_row;
  d.x_stride_expert = a.out_expert_x_stride_expert;
  d.expert_xs = S ? a.out_expert_x_scale : nullptr;
  d.xs_stride_elem = a.out_expert_x_scale_stride_elem;
  d.xs_stride_row = a.out_expert_x_scale_stride_row;
  d.xs_stride_expert = a.out_expert_x_scale_stride_expert;
  d.dp_x = static_cast<const uint8_t *>(a.dp_x);
  d.dp_x_stride_row = a.dp_x_stride_row;
  d.dp_xs = S ? a.dp_x_scale : nullptr;
  d.dp_xs_stride_elem = a.dp_x_scale_stride_elem;
  d.dp_xs_stride_row = a.dp_x_scale_stride_row;
  d.indices = a.indices;
  d.bound_m = a.bound_m;
  d.m = a.m;
  d.x_rows = rows > 0xfffffffeull ? 0xfffffffeu : (uint32_t)rows;
  *out = d;
  return PPLX_A2A_OK;
}

size_t dtype_size(int dt) { return dt == PPLX_A2A_F32 ? 4 : 2; }

int convert_combine(const WorldDev &geo, uint32_t rank, const pplx_a2a_combine_args_t &a,
                    CombineRank *out) {
  // csrc/bindings/all_to_all_ops.cpp:265-310
  if (a.in_dtype != PPLX_A2A_F32 && a.in_dtype != PPLX_A2A_BF16 && a.in_dtype != PPLX_A2A_F16)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "Unsupported dtype for expertY");
  if (a.out_dtype != PPLX_A2A_BF16 && a.out_dtype != PPLX_A2A_F16)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "Unsupported dtype for outTokens");
  if (geo.H % 8 != 0)
    return fail(PPLX_A2A_UNSUPPORTED, "combine needs hidden_dim to be a multiple of 8");
  if (!a.expert_y) return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: expert_y is NULL", rank);
  if (a.m > 0 && (!a.out_tokens || !a.indices || !a.weights))
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: out_tokens / indices / weights is NULL with m > 0", rank);
  const size_t in_sz = dtype_size(a.in_dtype), out_sz = dtype_size(a.out_dtype);
  if (!aligned16(a.expert_y) || (a.expert_y_stride_row * (int64_t)in_sz) % 16 ||
      (a.expert_y_stride_expert * (int64_t)in_sz) % 16)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: expert_y must be 16-byte aligned with 16-byte strides", rank);
  if (!aligned16(a.out_tokens) || (a.out_tokens_stride_row * (int64_t)out_sz) % 16)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: out_tokens must be 16-byte aligned with a 16-byte row stride", rank);
  if (a.expert_y_rows < 0)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: expert_y_rows is negative", rank);
  if (!a.bound_m && a.m > geo.M)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u: %u tokens exceed max_num_tokens %u", rank, a.m, geo.M);
  const uint64_t rows = a.expert_y_rows ? (uint64_t)a.expert_y_rows : (uint64_t)geo.M * geo.G;
  CombineRank c{};
  c.out_tokens = a.out_tokens;
  c.out_stride_row = a.out_tokens_stride_row;
  c.indices = a.indices;
  c.weights = a.weights;
  c.w_stride_row = a.weights_stride_row;
  c.expert_y = a.expert_y;
  c.y_stride_row = a.expert_y_stride_row;
  c.y_stride_expert = a.expert_y_stride_expert;
  c.bound_m = a.bound_m;
  c.m = a.m;
  c.y_rows = rows > 0xfffffffeull ? 0xfffffffeu : (uint32_t)rows;
  *out = c;
  return PPLX_A2A_OK;
}

// Capture session of `stream` (0 when it is not capturing).
int capture_session(void *stream, unsigned long long *out) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  unsigned long long id = 0;
  HIP_TRY(hipStreamGetCaptureInfo((hipStream_t)stream, &st, &id));
  *out = st == hipStreamCaptureStatusNone ? 0ull : (id ? id : ~0ull);
  return PPLX_A2A_OK;
}

// Decides whether the host mirror of a device table may be trusted for this call.
// Inside a capture only binds recorded earlier in the same capture count; in eager
// mode the mirror is void once any graph exists, because a replay rewrites the table.
void settle_mirror(pplx_a2a_world &w, unsigned long long session, unsigned long long &last_session,
                   bool &bound_valid) {
  if (session != 0) {
    w.captured_once = true;
    if (last_session != session) bound_valid = false;
  } else if (w.captured_once) {
    bound_valid = false;
  }
  last_session = session;
}

// Makes the device tables equal to `rows`, batch by batch, skipping batches the
// tables are known to hold already.
template <typename Row, typename Batch, typename Launch>
int flush_table(pplx_a2a_world &w, const std::vector<Row> &rows, std::vector<Row> &bound,
                bool &bound_valid, bool force, Launch launch, void *stream) {
  const uint32_t R = w.dev.R;
  for (uint32_t first = 0; first < R; first += kBindBatch) {
    const uint32_t count = (R - first < kBindBatch) ? R - first : kBindBatch;
    bool dirty = force || !bound_valid;
    if (!dirty) dirty = memcmp(&rows[first], &bound[first], sizeof(Row) * count) != 0;
    if (!dirty) continue;
    Batch b;
    memset(static_cast<void *>(&b), 0, sizeof(b));
    b.first = first;
    b.count = count;
    memcpy(static_cast<void *>(b.rows), &rows[first], sizeof(Row) * count);
    LAUNCH_TRY(launch(w.dev, b, stream));
  }
  bound = rows;
  bound_valid = true;
  return PPLX_A2A_OK;
}

// Widest load (in expert ids) that suits a row of K picks starting at `indices`.
uint32_t pick_vector_for(uint32_t K, const uint32_t *indices, uint32_t at_most = 4) {
  uint32_t pv = K % 4 == 0 ? 4 : K % 2 == 0 ? 2 : 1;
  if (pv > at_most) pv = at_most;
  const uintptr_t p = reinterpret_cast<uintptr_t>(indices);
  while (pv > 1 && p % (4 * pv) != 0) pv /= 2;
  return pv;
}

// ... that suits the indices of every rank of the pending step.
uint32_t pick_vector_of(const WorldDev &d, const DispatchRank *rows) {
  uint32_t pv = 4;
  for (uint32_t r = 0; r < d.R; ++r) pv = pick_vector_for(d.K, rows[r].indices, pv);
  return pv;
}
uint32_t pick_vector_of(const pplx_a2a_world &w) { return pick_vector_of(w.dev, w.pend_dispatch.data()); }

// The members of a DP group hold the same tokens (csrc/all_to_all/intranode_dispatch.cu:97
// strides one token list over them), so they must agree on how many rows there are: the
// kernels take the count from the group's first member and read every member's rows.
int check_groups(const WorldDev &d, const DispatchRank *rows) {
  const uint32_t dp = d.dp;
  if (dp == 1) return PPLX_A2A_OK;
  for (uint32_t g = 0; g < d.G; ++g) {
    const DispatchRank &head = rows[g * dp];
    for (uint32_t i = 1; i < dp; ++i) {
      const DispatchRank &member = rows[g * dp + i];
      if (member.m != head.m || (member.bound_m == nullptr) != (head.bound_m == nullptr))
        return fail(PPLX_A2A_INVALID_ARGUMENT,
                    "ranks %u and %u share a DP group but pass %u and %u tokens (or only one of them a bound_m)",
                    g * dp, g * dp + i, head.m, member.m);
    }
  }
  return PPLX_A2A_OK;
}

// Per-rank calls of one step may arrive on different streams (the reference runs each rank's op
// on that rank's current stream, csrc/bindings/all_to_all_ops.cpp:163,194).  The kernels go to
// the stream of the last caller: before them it waits for what the other streams hold so far,
// and afterwards those streams wait for the kernels, so that work enqueued on any of them after
// the step's last call sees the outputs.
template <typename Run>
int run_ordered(pplx_a2a_world &w, const std::vector<void *> &streams, void *launch, Run run) {
  bool mixed = false;
  for (void *s : streams) mixed = mixed || s != launch;
  if (!mixed) return run();
  DeviceScope scope(w.device);
  if (!scope.ok()) return fail(PPLX_A2A_HIP_ERROR, "cannot select device %d", w.device);
  const uint32_t R = w.dev.R;
  auto first_use = [&](uint32_t r) {
    if (streams[r] == launch) return false;
    for (uint32_t q = 0; q < r; ++q)
      if (streams[q] == streams[r]) return false;
    return true;
  };
  for (uint32_t r = 0; r <= R; ++r) {
    unsigned long long session = 0;
    int st = capture_session(r == R ? launch : streams[r], &session);
    if (st) return st;
    if (session != 0)
      return fail(PPLX_A2A_INVALID_STATE, "the ranks of a captured step must call on one stream");
  }
  for (uint32_t r = 0; r < R; ++r) {
    if (!first_use(r)) continue;
    HIP_TRY(hipEventRecord(w.rank_events[r], (hipStream_t)streams[r]));
    HIP_TRY(hipStreamWaitEvent((hipStream_t)launch, w.rank_events[r], 0));
  }
  int st = run();
  if (st) return st;
  HIP_TRY(hipEventRecord(w.done_event, (hipStream_t)launch));
  for (uint32_t r = 0; r < R; ++r) {
    if (first_use(r)) HIP_TRY(hipStreamWaitEvent((hipStream_t)streams[r], w.done_event, 0));
  }
  return PPLX_A2A_OK;
}

int run_dispatch(pplx_a2a_world &w, void *stream) {
  int st = check_groups(w.dev, w.pend_dispatch.data());
  if (st) return st;
  DeviceScope scope(w.device);
  if (!scope.ok()) return fail(PPLX_A2A_HIP_ERROR, "cannot select device %d", w.device);
  unsigned long long session = 0;
  st = capture_session(stream, &session);
  if (st) return st;
  settle_mirror(w, session, w.bind_capture_dispatch, w.bound_dispatch_valid);
  ProfilerRange range("dispatch");
  if (w.dev.R <= kInlineRanks) {
    LAUNCH_TRY(launch_dispatch(w.dev, w.pend_dispatch.data(), pick_vector_of(w), stream));
    return PPLX_A2A_OK;
  }
  st = flush_table<DispatchRank, BindDispatchBatch>(w, w.pend_dispatch, w.bound_dispatch,
                                                    w.bound_dispatch_valid, false,
                                                    launch_bind_dispatch, stream);
  if (st) return st;
  LAUNCH_TRY(launch_dispatch(w.dev, nullptr, pick_vector_of(w), stream));
  return PPLX_A2A_OK;
}

int run_combine(pplx_a2a_world &w, void *stream) {
  DeviceScope scope(w.device);
  if (!scope.ok()) return fail(PPLX_A2A_HIP_ERROR, "cannot select device %d", w.device);
  unsigned long long session = 0;
  int st = capture_session(stream, &session);
  if (st) return st;
  settle_mirror(w, session, w.bind_capture_combine, w.bound_combine_valid);
  ProfilerRange range("combine");
  if (w.dev.R <= kInlineRanks) {
    LAUNCH_TRY(launch_combine(w.dev, w.pend_combine.data(), w.combine_in_dtype, w.combine_out_dtype,
                              stream));
    return PPLX_A2A_OK;
  }
  st = flush_table<CombineRank, BindCombineBatch>(w, w.pend_combine, w.bound_combine,
                                                  w.bound_combine_valid, false,
                                                  launch_bind_combine, stream);
  if (st) return st;
  LAUNCH_TRY(launch_combine(w.dev, nullptr, w.combine_in_dtype, w.combine_out_dtype, stream));
  return PPLX_A2A_OK;
}

void free_split(pplx_a2a_world &w) {
  SplitDev &sp = w.split;
  (void)hipFree(sp.stage_x);  // the picks and the groups' counts live behind the rows
  (void)hipFree(sp.stage_y);
  sp = SplitDev{};
  w.split_ready = false;
}

// Allocates the staging of split mode: the tokens' area on the first call, the combined rows'
// area on the first call that asks for it.  Never part of a dispatch / combine call; nothing
// that has been allocated moves or is freed before the world goes.
int reserve_split(pplx_a2a_world &w, uint32_t y_elem_bytes) {
  if (y_elem_bytes != 0 && y_elem_bytes != 2 && y_elem_bytes != 4)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "expert_y_elem_bytes must be 0, 2 or 4");
  DeviceScope scope(w.device);
  if (!scope.ok()) return fail(PPLX_A2A_HIP_ERROR, "cannot select device %d", w.device);
  const WorldDev &d = w.dev;
  SplitDev &sp = w.split;
  if (!w.split_ready) {
    if (w.n_arrived_dispatch != 0 || w.n_arrived_combine != 0)
      return fail(PPLX_A2A_INVALID_STATE, "a step is being assembled");
    const StageLayout lay = stage_layout(d.Hb, d.S, (uint64_t)d.G * d.M, d.K, d.G);
    hipError_t err = hipMalloc(reinterpret_cast<void **>(&sp.stage_x), lay.bytes);
    if (err == hipSuccess) err = hipMemset(sp.stage_x, 0, lay.bytes);
    if (err != hipSuccess) {
      free_split(w);
      return fail(PPLX_A2A_HIP_ERROR, "allocating %zu bytes of split-mode staging failed: %s", (size_t)lay.bytes,
                  hipGetErrorString(err));
    }
    sp.token_stride = lay.token_stride;
    sp.stage_idx = reinterpret_cast<uint32_t *>(sp.stage_x + lay.idx_offset);
    sp.stage_n = reinterpret_cast<uint32_t *>(sp.stage_x + lay.n_offset);
    w.dsend.assign(d.R, 0);
    w.drecv.assign(d.R, 0);
    w.csend.assign(d.R, 0);
    w.crecv.assign(d.R, 0);
    w.split_ready = true;
  }
  if (y_elem_bytes != 0 && sp.stage_y == nullptr) {
    // one combined row per (rank, token); out_tokens has 2-byte elements whatever expert_y has
    const size_t bytes = (size_t)d.R * d.M * d.H * 2u;
    hipError_t err = hipMalloc(reinterpret_cast<void **>(&sp.stage_y), bytes);
    if (err != hipSuccess) {
      sp.stage_y = nullptr;
      return fail(PPLX_A2A_HIP_ERROR, "allocating %zu bytes of combine staging failed: %s", bytes,
                  hipGetErrorString(err));
    }
  }
  return PPLX_A2A_OK;
}

int need_split(const pplx_a2a_world &w, bool combine) {
  if (!w.split_ready || (combine && w.split.stage_y == nullptr))
    return fail(PPLX_A2A_INVALID_STATE,
                "send / recv calls need staging%s: call pplx_a2a_world_reserve_split first (dispatch and "
                "combine never allocate)", combine ? " for combine (a non-zero expert_y_elem_bytes)" : "");
  return PPLX_A2A_OK;
}

// Split mode is collective phase by phase: the calls of a phase are recorded and the last
// rank's call enqueues the phase for all ranks (on its stream, ordered against the streams the
// other ranks called on).  SEND reads the inputs recorded by the SEND calls, RECV writes the
// outputs named by the RECV calls.
int run_split_dispatch(pplx_a2a_world &w, int mode, void *stream) {
  DeviceScope scope(w.device);
  if (!scope.ok()) return fail(PPLX_A2A_HIP_ERROR, "cannot select device %d", w.device);
  unsigned long long session = 0;
  int st = capture_session(stream, &session);
  if (st) return st;
  settle_mirror(w, session, w.bind_capture_dispatch, w.bound_dispatch_valid);
  const WorldDev &d = w.dev;
  if (mode == PPLX_A2A_SPLIT_SEND) {
    st = check_groups(d, w.pend_dispatch.data());
    if (st) return st;
  } else {
    // RECV is the one-call dispatch on what SEND staged: every rank's inputs are its DP
    // group's part of the staging area, its outputs those of its RECV call.
    const SplitDev &sp = w.split;
    for (uint32_t r = 0; r < d.R; ++r) {
      const uint32_t g = r / d.dp;
      DispatchRank &row = w.pend_dispatch[r];
      const uint8_t *rows = sp.stage_x + (uint64_t)g * d.M * sp.token_stride;
      row.dp_x = rows;
      row.dp_x_stride_row = sp.token_stride;
      row.dp_xs = d.S ? reinterpret_cast<const float *>(rows + d.Hb) : nullptr;
      row.dp_xs_stride_elem = 1;
      row.dp_xs_stride_row = sp.token_stride / 4;
      row.indices = sp.stage_idx + (uint64_t)g * d.M * d.K;
      row.bound_m = sp.stage_n + g;
      row.m = d.M;
    }
  }
  const DispatchRank *inline_rows = d.R <= kInlineRanks ? w.pend_dispatch.data() : nullptr;
  if (!inline_rows) {
    st = flush_table<DispatchRank, BindDispatchBatch>(w, w.pend_dispatch, w.bound_dispatch,
                                                      w.bound_dispatch_valid, false, launch_bind_dispatch, stream);
    if (st) return st;
  }
  if (mode == PPLX_A2A_SPLIT_SEND) {
    ProfilerRange range("dispatch send");
    LAUNCH_TRY(launch_split_stage_tokens(d, w.split, inline_rows, stream));
  } else {
    ProfilerRange range("dispatch recv");
    LAUNCH_TRY(launch_dispatch(d, inline_rows, pick_vector_of(w), stream));
  }
  return PPLX_A2A_OK;
}

int split_dispatch(pplx_a2a_world &w, uint32_t rank, const DispatchRank &row, int mode, void *stream) {
  if (w.n_arrived_dispatch != 0)
    return fail(PPLX_A2A_INVALID_STATE, "a send+recv dispatch step is still being assembled");
  int st = need_split(w, false);
  if (st) return st;
  const uint32_t R = w.dev.R;
  if (mode == PPLX_A2A_SPLIT_SEND) {
    if (w.n_drecv != 0 || w.n_dsend == R)
      return fail(PPLX_A2A_INVALID_STATE,
                  "rank %u: dispatch SEND of the next step before every rank's RECV of this one", rank);
    if (w.dsend[rank]) return fail(PPLX_A2A_INVALID_STATE, "rank %u called dispatch SEND twice", rank);
    w.pend_dispatch[rank] = row;
    w.stream_dispatch[rank] = stream;
    w.dsend[rank] = 1;
    if (++w.n_dsend < R) return PPLX_A2A_OK;
    st = run_ordered(w, w.stream_dispatch, stream, [&] { return run_split_dispatch(w, mode, stream); });
    if (st) {  // nothing was sent: the step starts over
      std::fill(w.dsend.begin(), w.dsend.end(), 0);
      w.n_dsend = 0;
    }
    return st;
  }
  if (w.n_dsend != R)
    return fail(PPLX_A2A_INVALID_STATE,
                "rank %u: dispatch RECV before every rank's SEND (%u of %u sent); in a loopback "
                "world all SENDs must be enqueued first", rank, w.n_dsend, R);
  if (w.drecv[rank]) return fail(PPLX_A2A_INVALID_STATE, "rank %u called dispatch RECV twice", rank);
  w.pend_dispatch[rank] = row;
  w.stream_dispatch[rank] = stream;
  w.drecv[rank] = 1;
  if (++w.n_drecv < R) return PPLX_A2A_OK;
  std::fill(w.dsend.begin(), w.dsend.end(), 0);
  std::fill(w.drecv.begin(), w.drecv.end(), 0);
  w.n_dsend = w.n_drecv = 0;
  return run_ordered(w, w.stream_dispatch, stream, [&] { return run_split_dispatch(w, mode, stream); });
}

int run_split_combine(pplx_a2a_world &w, int mode, int in_dtype, int out_dtype, void *stream) {
  DeviceScope scope(w.device);
  if (!scope.ok()) return fail(PPLX_A2A_HIP_ERROR, "cannot select device %d", w.device);
  unsigned long long session = 0;
  int st = capture_session(stream, &session);
  if (st) return st;
  settle_mirror(w, session, w.bind_capture_combine, w.bound_combine_valid);
  const WorldDev &d = w.dev;
  if (mode == PPLX_A2A_SPLIT_SEND) {
    // SEND is the one-call combine with every rank's output rows in the staging area.
    for (uint32_t r = 0; r < d.R; ++r) {
      CombineRank &row = w.pend_combine[r];
      row.out_tokens = w.split.stage_y + (uint64_t)r * d.M * d.H * 2u;
      row.out_stride_row = d.H;
    }
  }
  const CombineRank *inline_rows = d.R <= kInlineRanks ? w.pend_combine.data() : nullptr;
  if (!inline_rows) {
    st = flush_table<CombineRank, BindCombineBatch>(w, w.pend_combine, w.bound_combine, w.bound_combine_valid,
                                                    false, launch_bind_combine, stream);
    if (st) return st;
  }
  if (mode == PPLX_A2A_SPLIT_SEND) {
    ProfilerRange range("combine send");
    LAUNCH_TRY(launch_combine(d, inline_rows, in_dtype, out_dtype, stream));
  } else {
    ProfilerRange range("combine recv");
    LAUNCH_TRY(launch_split_deliver(d, w.split, inline_rows, stream));
  }
  return PPLX_A2A_OK;
}

int split_combine(pplx_a2a_world &w, uint32_t rank, const CombineRank &row, int in_dtype, int out_dtype,
                  int mode, void *stream) {
  if (w.n_arrived_combine != 0)
    return fail(PPLX_A2A_INVALID_STATE, "a send+recv combine step is still being assembled");
  int st = need_split(w, true);
  if (st) return st;
  const uint32_t R = w.dev.R;
  if (mode == PPLX_A2A_SPLIT_SEND) {
    if (w.n_crecv != 0 || w.n_csend == R)
      return fail(PPLX_A2A_INVALID_STATE,
                  "rank %u: combine SEND of the next step before every rank's RECV of this one", rank);
    if (w.csend[rank]) return fail(PPLX_A2A_INVALID_STATE, "rank %u called combine SEND twice", rank);
    if (w.n_csend != 0 && (w.split_in_dtype != in_dtype || w.split_out_dtype != out_dtype))
      return fail(PPLX_A2A_UNSUPPORTED, "all ranks of a step must combine with the same dtypes");
    w.split_in_dtype = in_dtype;
    w.split_out_dtype = out_dtype;
    w.pend_combine[rank] = row;
    w.stream_combine[rank] = stream;
    w.csend[rank] = 1;
    if (++w.n_csend < R) return PPLX_A2A_OK;
    st = run_ordered(w, w.stream_combine, stream,
                     [&] { return run_split_combine(w, mode, in_dtype, out_dtype, stream); });
    if (st) {
      std::fill(w.csend.begin(), w.csend.end(), 0);
      w.n_csend = 0;
    }
    return st;
  }
  if (w.n_csend != R)
    return fail(PPLX_A2A_INVALID_STATE,
                "rank %u: combine RECV before every rank's SEND (%u of %u sent); in a loopback "
                "world all SENDs must be enqueued first", rank, w.n_csend, R);
  if (w.crecv[rank]) return fail(PPLX_A2A_INVALID_STATE, "rank %u called combine RECV twice", rank);
  // (the rows were combined, and converted to the out_tokens dtype, by the SEND phase)
  if (w.split_in_dtype != in_dtype || w.split_out_dtype != out_dtype)
    return fail(PPLX_A2A_UNSUPPORTED, "combine RECV must use the dtypes of the SEND phase");
  w.pend_combine[rank] = row;
  w.stream_combine[rank] = stream;
  w.crecv[rank] = 1;
  if (++w.n_crecv < R) return PPLX_A2A_OK;
  std::fill(w.csend.begin(), w.csend.end(), 0);
  std::fill(w.crecv.begin(), w.crecv.end(), 0);
  w.n_csend = w.n_crecv = 0;
  return run_ordered(w, w.stream_combine, stream,
                     [&] { return run_split_combine(w, mode, in_dtype, out_dtype, stream); });
}

void reset_dispatch_arrivals(pplx_a2a_world &w) {
  std::fill(w.arrived_dispatch.begin(), w.arrived_dispatch.end(), 0);
  w.n_arrived_dispatch = 0;
}

void reset_combine_arrivals(pplx_a2a_world &w) {
  std::fill(w.arrived_combine.begin(), w.arrived_combine.end(), 0);
  w.n_arrived_combine = 0;
  w.combine_in_dtype = w.combine_out_dtype = -1;
}

}  // namespace

extern "C" {

const char *pplx_a2a_last_error(void) { return g_last_error.c_str(); }

const char *pplx_a2a_version(void) { return "0.3.0"; }

#ifndef PPLX_A2A_SOURCE_ID
#define PPLX_A2A_SOURCE_ID "unknown"
#endif
const char *pplx_a2a_build_id(void) { return PPLX_A2A_SOURCE_ID; }

int pplx_a2a_world_create(const pplx_a2a_config_t *cfg, int device, pplx_a2a_world_t **out) {
  if (!cfg || !out) return fail(PPLX_A2A_INVALID_ARGUMENT, "cfg / out is NULL");
  *out = nullptr;
  int st = check_config(*cfg);
  if (st) return st;
  int n_dev = 0;
  HIP_TRY(hipGetDeviceCount(&n_dev));
  if (device < 0 || device >= n_dev)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "device %d out of range (%d visible)", device, n_dev);
  DeviceScope scope(device);
  if (!scope.ok()) return fail(PPLX_A2A_HIP_ERROR, "cannot select device %d", device);

  {
    // The first world on a device also looks up that device's copy of the library's static
    // scratch array, so that pplx_a2a_static_step finds it ready.
    // (a world does not need the array: a failed lookup is left for that entry point to report)
    void *unused = nullptr;
    (void)static_scratch_address(device, &unused);
  }
  pplx_a2a_world *w = new (std::nothrow) pplx_a2a_world();
  if (!w) return fail(PPLX_A2A_HIP_ERROR, "out of host memory");
  w->cfg = *cfg;
  w->device = device;
  WorldDev &d = w->dev;
  fill_geometry(*cfg, d);
  d.lds_per_cu = lds_per_cu_of(device);

  auto cleanup = [&]() {
    for (hipEvent_t ev : w->rank_events) (void)hipEventDestroy(ev);
    if (w->done_event) (void)hipEventDestroy(w->done_event);
    (void)hipFree(d.drank);
    (void)hipFree(d.crank);
    (void)hipFree(d.tile_cnt);
    (void)hipFree(d.slot_map);
    (void)hipFree(d.faults);
    delete w;
  };
  struct Alloc {
    void **ptr;
    size_t bytes;
  } allocs[] = {
      {reinterpret_cast<void **>(&d.drank), sizeof(DispatchRank) * d.R},
      {reinterpret_cast<void **>(&d.crank), sizeof(CombineRank) * d.R},
      {reinterpret_cast<void **>(&d.tile_cnt), (size_t)route_tables(d.num_tiles, d.tile_chunks, d.E).bytes},
      {reinterpret_cast<void **>(&d.slot_map), sizeof(uint32_t) * (size_t)d.G * d.M * d.K},
      {reinterpret_cast<void **>(&d.faults), 256},
  };
  for (const Alloc &a : allocs) {
    hipError_t err = hipMalloc(a.ptr, a.bytes);
    if (err == hipSuccess) err = hipMemset(*a.ptr, 0, a.bytes);
    if (err != hipSuccess) {
      cleanup();
      return fail(PPLX_A2A_HIP_ERROR, "allocating %zu bytes of world state failed: %s", a.bytes,
                  hipGetErrorString(err));
    }
  }
  // Events that order per-rank calls made on different streams (no timing: they only fence).
  for (uint32_t r = 0; r <= d.R; ++r) {
    hipEvent_t ev = nullptr;
    const hipError_t err = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
    if (err != hipSuccess) {
      cleanup();
      return fail(PPLX_A2A_HIP_ERROR, "hipEventCreateWithFlags failed: %s", hipGetErrorString(err));
    }
    if (r < d.R) w->rank_events.push_back(ev); else w->done_event = ev;
  }
  w->stream_dispatch.assign(d.R, nullptr);
  w->stream_combine.assign(d.R, nullptr);
  w->pend_dispatch.assign(d.R, DispatchRank{});
  w->pend_combine.assign(d.R, CombineRank{});
  w->bound_dispatch.assign(d.R, DispatchRank{});
  w->bound_combine.assign(d.R, CombineRank{});
  w->arrived_dispatch.assign(d.R, 0);
  w->arrived_combine.assign(d.R, 0);
  *out = w;
  return PPLX_A2A_OK;
}

int pplx_a2a_world_destroy(pplx_a2a_world_t *w) {
  if (!w) return PPLX_A2A_OK;
  if (w->attached != 0)
    return fail(PPLX_A2A_INVALID_STATE, "%d rank handle(s) still attached to the world", w->attached);
  DeviceScope scope(w->device);
  (void)hipDeviceSynchronize();
  for (hipEvent_t ev : w->rank_events) (void)hipEventDestroy(ev);
  if (w->done_event) (void)hipEventDestroy(w->done_event);
  (void)hipFree(w->dev.drank);
  (void)hipFree(w->dev.crank);
  (void)hipFree(w->dev.tile_cnt);
  (void)hipFree(w->dev.slot_map);
  (void)hipFree(w->dev.faults);
  free_split(*w);
  delete w;
  return PPLX_A2A_OK;
}

int pplx_a2a_create(pplx_a2a_world_t *w, uint32_t rank, pplx_a2a_t **out) {
  if (!w || !out) return fail(PPLX_A2A_INVALID_ARGUMENT, "world / out is NULL");
  *out = nullptr;
  if (rank >= w->dev.R)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "rank %u out of range for world_size %u", rank, w->dev.R);
  pplx_a2a *h = new (std::nothrow) pplx_a2a{w, rank};
  if (!h) return fail(PPLX_A2A_HIP_ERROR, "out of host memory");
  std::lock_guard<std::mutex> lock(w->mu);
  ++w->attached;
  *out = h;
  return PPLX_A2A_OK;
}

int pplx_a2a_destroy(pplx_a2a_t *h) {
  if (!h) return PPLX_A2A_OK;
  {
    pplx_a2a_world &w = *h->world;
    std::lock_guard<std::mutex> lock(w.mu);
    --w.attached;
    // A rank that leaves in the middle of a step takes its half-made call with it, so that the
    // handle which replaces it can call again.
    if (w.arrived_dispatch[h->rank]) {
      w.arrived_dispatch[h->rank] = 0;
      --w.n_arrived_dispatch;
    }
    if (w.arrived_combine[h->rank]) {
      w.arrived_combine[h->rank] = 0;
      --w.n_arrived_combine;
    }
    // ... and the same for a phase of split mode that has not been launched yet
    if (w.split_ready) {
      auto forget = [&](std::vector<uint8_t> &made, uint32_t &count) {
        if (count < w.dev.R && made[h->rank]) {
          made[h->rank] = 0;
          --count;
        }
      };
      forget(w.dsend, w.n_dsend);
      forget(w.drecv, w.n_drecv);
      forget(w.csend, w.n_csend);
      forget(w.crecv, w.n_crecv);
    }
  }
  delete h;
  return PPLX_A2A_OK;
}

uint64_t pplx_a2a_num_experts_per_token(const pplx_a2a_t *h) { return h ? h->world->dev.K : 0; }

uint32_t pplx_a2a_rank(const pplx_a2a_t *h) { return h ? h->rank : 0; }

pplx_a2a_world_t *pplx_a2a_world_of(const pplx_a2a_t *h) { return h ? h->world : nullptr; }

int pplx_a2a_dispatch(pplx_a2a_t *h, const pplx_a2a_dispatch_args_t *args, int split_mode,
                      void *stream) {
  if (!h || !args) return fail(PPLX_A2A_INVALID_ARGUMENT, "handle / args is NULL");
  pplx_a2a_world &w = *h->world;
  if (split_mode != PPLX_A2A_SPLIT_NONE && split_mode != PPLX_A2A_SPLIT_SEND &&
      split_mode != PPLX_A2A_SPLIT_RECV)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "Invalid split mode");
  DispatchRank row;
  int st = convert_dispatch(w.dev, h->rank, *args, &row);
  if (st) return st;
  std::lock_guard<std::mutex> lock(w.mu);
  if (split_mode != PPLX_A2A_SPLIT_NONE) return split_dispatch(w, h->rank, row, split_mode, stream);
  if (w.n_dsend != 0 || w.n_drecv != 0)
    return fail(PPLX_A2A_INVALID_STATE, "a split dispatch step is still in flight");
  if (w.arrived_dispatch[h->rank])
    return fail(PPLX_A2A_INVALID_STATE,
                "rank %u called dispatch twice before the other ranks of the step", h->rank);
  w.pend_dispatch[h->rank] = row;
  w.stream_dispatch[h->rank] = stream;
  w.arrived_dispatch[h->rank] = 1;
  if (++w.n_arrived_dispatch < w.dev.R) return PPLX_A2A_OK;
  reset_dispatch_arrivals(w);
  return run_ordered(w, w.stream_dispatch, stream, [&] { return run_dispatch(w, stream); });
}

int pplx_a2a_combine(pplx_a2a_t *h, const pplx_a2a_combine_args_t *args, int split_mode,
                     void *stream) {
  if (!h || !args) return fail(PPLX_A2A_INVALID_ARGUMENT, "handle / args is NULL");
  pplx_a2a_world &w = *h->world;
  if (split_mode != PPLX_A2A_SPLIT_NONE && split_mode != PPLX_A2A_SPLIT_SEND &&
      split_mode != PPLX_A2A_SPLIT_RECV)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "Invalid split mode");
  CombineRank row;
  int st = convert_combine(w.dev, h->rank, *args, &row);
  if (st) return st;
  std::lock_guard<std::mutex> lock(w.mu);
  if (split_mode != PPLX_A2A_SPLIT_NONE)
    return split_combine(w, h->rank, row, args->in_dtype, args->out_dtype, split_mode, stream);
  if (w.n_csend != 0 || w.n_crecv != 0)
    return fail(PPLX_A2A_INVALID_STATE, "a split combine step is still in flight");
  if (w.arrived_combine[h->rank])
    return fail(PPLX_A2A_INVALID_STATE,
                "rank %u called combine twice before the other ranks of the step", h->rank);
  if (w.n_arrived_combine > 0 &&
      (w.combine_in_dtype != args->in_dtype || w.combine_out_dtype != args->out_dtype))
    return fail(PPLX_A2A_UNSUPPORTED, "all ranks of a step must combine with the same dtypes");
  w.combine_in_dtype = args->in_dtype;
  w.combine_out_dtype = args->out_dtype;
  w.pend_combine[h->rank] = row;
  w.stream_combine[h->rank] = stream;
  w.arrived_combine[h->rank] = 1;
  if (++w.n_arrived_combine < w.dev.R) return PPLX_A2A_OK;
  const int in_dt = w.combine_in_dtype, out_dt = w.combine_out_dtype;
  reset_combine_arrivals(w);
  w.combine_in_dtype = in_dt;
  w.combine_out_dtype = out_dt;
  return run_ordered(w, w.stream_combine, stream, [&] { return run_combine(w, stream); });
}

int pplx_a2a_world_dispatch(pplx_a2a_world_t *w, const pplx_a2a_dispatch_args_t *per_rank,
                            void *stream) {
  if (!w || !per_rank) return fail(PPLX_A2A_INVALID_ARGUMENT, "world / per_rank is NULL");
  std::lock_guard<std::mutex> lock(w->mu);
  if (w->n_arrived_dispatch != 0 || w->n_dsend != 0 || w->n_drecv != 0)
    return fail(PPLX_A2A_INVALID_STATE, "a per-rank dispatch step is still being assembled");
  for (uint32_t r = 0; r < w->dev.R; ++r) {
    int st = convert_dispatch(w->dev, r, per_rank[r], &w->pend_dispatch[r]);
    if (st) return st;
  }
  return run_dispatch(*w, stream);
}

int pplx_a2a_world_combine(pplx_a2a_world_t *w, const pplx_a2a_combine_args_t *per_rank,
                           void *stream) {
  if (!w || !per_rank) return fail(PPLX_A2A_INVALID_ARGUMENT, "world / per_rank is NULL");
  std::lock_guard<std::mutex> lock(w->mu);
  if (w->n_arrived_combine != 0 || w->n_csend != 0 || w->n_crecv != 0)
    return fail(PPLX_A2A_INVALID_STATE, "a per-rank combine step is still being assembled");
  for (uint32_t r = 0; r < w->dev.R; ++r) {
    if (per_rank[r].in_dtype != per_rank[0].in_dtype || per_rank[r].out_dtype != per_rank[0].out_dtype)
      return fail(PPLX_A2A_UNSUPPORTED, "all ranks of a step must combine with the same dtypes");
    int st = convert_combine(w->dev, r, per_rank[r], &w->pend_combine[r]);
    if (st) return st;
  }
  w->combine_in_dtype = per_rank[0].in_dtype;
  w->combine_out_dtype = per_rank[0].out_dtype;
  return run_combine(*w, stream);
}

int pplx_a2a_world_recorded_calls(pplx_a2a_world_t *w, int op, int split_mode, uint32_t *out) {
  if (!w || !out) return fail(PPLX_A2A_INVALID_ARGUMENT, "world / out is NULL");
  if ((op != 0 && op != 1) || split_mode < PPLX_A2A_SPLIT_NONE || split_mode > PPLX_A2A_SPLIT_RECV)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "op must be 0 (dispatch) or 1 (combine), split_mode a pplx_a2a_split_mode");
  std::lock_guard<std::mutex> lock(w->mu);
  const uint32_t R = w->dev.R;
  // (a phase whose count has reached world_size has been launched: nothing of it is pending)
  auto pending = [R](uint32_t count) { return count < R ? count : 0u; };
  if (split_mode == PPLX_A2A_SPLIT_NONE) {
    *out = op == 0 ? w->n_arrived_dispatch : w->n_arrived_combine;
  } else if (split_mode == PPLX_A2A_SPLIT_SEND) {
    *out = pending(op == 0 ? w->n_dsend : w->n_csend);
  } else {
    *out = pending(op == 0 ? w->n_drecv : w->n_crecv);
  }
  return PPLX_A2A_OK;
}

int pplx_a2a_world_abandon_step(pplx_a2a_world_t *w, uint32_t which, uint32_t *dropped_calls) {
  if (!w) return fail(PPLX_A2A_INVALID_ARGUMENT, "world is NULL");
  if (which == 0 || (which & ~(uint32_t)(PPLX_A2A_ABANDON_DISPATCH | PPLX_A2A_ABANDON_COMBINE)) != 0)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "which must be PPLX_A2A_ABANDON_DISPATCH, _COMBINE or both");
  std::lock_guard<std::mutex> lock(w->mu);
  uint32_t dropped = 0;
  // Recorded calls are host state only: nothing of a step reaches the GPU before its last rank
  // has called.  A split step whose SEND phase has been launched loses what it staged (the next
  // SEND overwrites it).
  auto forget = [&](std::vector<uint8_t> &made, uint32_t &count) {
    if (count < w->dev.R) dropped += count;  // a complete phase has been launched, not recorded
    std::fill(made.begin(), made.end(), 0);
    count = 0;
  };
  if (which & PPLX_A2A_ABANDON_DISPATCH) {
    dropped += w->n_arrived_dispatch;
    reset_dispatch_arrivals(*w);
    if (w->split_ready) {
      forget(w->dsend, w->n_dsend);
      forget(w->drecv, w->n_drecv);
    }
  }
  if (which & PPLX_A2A_ABANDON_COMBINE) {
    dropped += w->n_arrived_combine;
    reset_combine_arrivals(*w);
    if (w->split_ready) {
      forget(w->csend, w->n_csend);
      forget(w->crecv, w->n_crecv);
    }
  }
  if (dropped_calls) *dropped_calls = dropped;
  return PPLX_A2A_OK;
}

int pplx_a2a_world_reserve_split(pplx_a2a_world_t *w, uint32_t expert_y_elem_bytes) {
  if (!w) return fail(PPLX_A2A_INVALID_ARGUMENT, "world is NULL");
  std::lock_guard<std::mutex> lock(w->mu);
  return reserve_split(*w, expert_y_elem_bytes);
}

int pplx_a2a_static_step(const pplx_a2a_config_t *cfg, int device,
                         const pplx_a2a_dispatch_args_t *dispatch_per_rank,
                         const pplx_a2a_combine_args_t *combine_per_rank, uint32_t *fault_bits,
                         void *stream) {
  if (!cfg) return fail(PPLX_A2A_INVALID_ARGUMENT, "cfg is NULL");
  if (!dispatch_per_rank && !combine_per_rank)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "neither a dispatch nor a combine to run");
  int st = check_config(*cfg);
  if (st) return st;
  if (cfg->world_size > kInlineRanks)
    return fail(PPLX_A2A_UNSUPPORTED, "the static step serves worlds of up to %u ranks, not %u", kInlineRanks,
                cfg->world_size);
  WorldDev d{};
  fill_geometry(*cfg, d);
  // Scratch layout: the fault word, the slot map (the hand-off from dispatch to combine, kept
  // from one call to the next), the routing tiles' counts and masks.
  const size_t slot_bytes = sizeof(uint32_t) * (size_t)d.G * d.M * d.K;
  const size_t tile_bytes = (size_t)route_tables(d.num_tiles, d.tile_chunks, d.E).bytes;
  const size_t slot_at = 256, tile_at = slot_at + (slot_bytes + 255) / 256 * 256;
  const size_t needed = tile_at + tile_bytes;
  if (needed > kStaticScratchBytes)
    return fail(PPLX_A2A_INVALID_ARGUMENT,
                "the geometry needs %zu bytes of scratch, the library's static array holds %zu: "
                "use a world (pplx_a2a_world_create) for it", needed, (size_t)kStaticScratchBytes);
  int n_dev = 0;
  HIP_TRY(hipGetDeviceCount(&n_dev));
  if (device < 0 || device >= n_dev)
    return fail(PPLX_A2A_INVALID_ARGUMENT, "device %d out of range (%d visible)", device, n_dev);
  DeviceScope scope(device);
  if (!scope.ok()) return fail(PPLX_A2A_HIP_ERROR, "cannot select device %d", device);
  // The first call on a device looks the array up (which may load the code object) and asks the
  // device for its LDS size: neither belongs into a stream capture.
  if (!static_scratch_known(device)) {
    unsigned long long session = 0;
    st = capture_session(stream, &session);
    if (st) return st;
    if (session != 0)
      return fail(PPLX_A2A_INVALID_STATE,
                  "the first pplx_a2a_static_step on a device sets the library up and cannot be captured: make "
                  "one call outside the capture (or create a world on the device) first");
  }
  d.lds_per_cu = lds_per_cu_of(device);
  void *base = nullptr;
  LAUNCH_TRY(static_scratch_address(device, &base));
  uint8_t *scratch = static_cast<uint8_t *>(base);
  d.faults = fault_bits ? fault_bits : reinterpret_cast<uint32_t *>(scratch);
  d.slot_map = reinterpret_cast<uint32_t *>(scratch + slot_at);
  d.tile_cnt = reinterpret_cast<uint32_t *>(scratch + tile_at);

  if (dispatch_per_rank) {
    DispatchRank rows[kInlineRanks];
    for (uint32_t r = 0; r < d.R; ++r) {
      st = convert_dispatch(d, r, dispatch_per_rank[r], &rows[r]);
      if (st) return st;
    }
    st = check_groups(d, rows);
    if (st) return st;
    ProfilerRange range("dispatch");
    LAUNCH_TRY(launch_dispatch(d, rows, pick_vector_of(d, rows), stream));
  }
  if (combine_per_rank) {
    CombineRank rows[kInlineRanks];
    for (uint32_t r = 0; r < d.R; ++r) {
      if (combine_per_rank[r].in_dtype != combine_per_rank[0].in_dtype ||
          combine_per_rank[r].out_dtype != combine_per_rank[0].out_dtype)
        return fail(PPLX_A2A_UNSUPPORTED, "all ranks of a step must combine with the same dtypes");
      st = convert_combine(d, r, combine_per_rank[r], &rows[r]);
      if (st) return st;
    }
    ProfilerRange range("combine");
    LAUNCH_TRY(launch_combine(d, rows, combine_per_rank[0].in_dtype, combine_per_rank[0].out_dtype, stream));
  }
  return PPLX_A2A_OK;
}

int pplx_a2a_world_faults(pplx_a2a_world_t *w, void *stream, uint32_t *out_bits) {
  if (!w || !out_bits) return fail(PPLX_A2A_INVALID_ARGUMENT, "world / out_bits is NULL");
  DeviceScope scope(w->device);
  if (!scope.ok()) return fail(PPLX_A2A_HIP_ERROR, "cannot select device %d", w->device);
  HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  uint32_t bits = 0;
  HIP_TRY(hipMemcpy(&bits, w->dev.faults, sizeof(bits), hipMemcpyDeviceToHost));
  if (bits) HIP_TRY(hipMemset(w->dev.faults, 0, sizeof(bits)));
  *out_bits = bits;
  return PPLX_A2A_OK;
}

int pplx_a2a_graph_begin_capture(void *stream) {
  HIP_TRY(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
  return PPLX_A2A_OK;
}

int pplx_a2a_graph_end_capture(void *stream, pplx_a2a_graph_t **out) {
  if (!out) return fail(PPLX_A2A_INVALID_ARGUMENT, "out is NULL");
  *out = nullptr;
  pplx_a2a_graph *g = new (std::nothrow) pplx_a2a_graph();
  if (!g) return fail(PPLX_A2A_HIP_ERROR, "out of host memory");
  hipError_t err = hipStreamEndCapture((hipStream_t)stream, &g->graph);
  if (err == hipSuccess) err = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
  if (err != hipSuccess) {
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
    return fail(PPLX_A2A_HIP_ERROR, "graph capture failed: %s", hipGetErrorString(err));
  }
  *out = g;
  return PPLX_A2A_OK;
}

int pplx_a2a_graph_launch(pplx_a2a_graph_t *g, void *stream) {
  if (!g) return fail(PPLX_A2A_INVALID_ARGUMENT, "graph is NULL");
  HIP_TRY(hipGraphLaunch(g->exec, (hipStream_t)stream));
  return PPLX_A2A_OK;
}

int pplx_a2a_graph_destroy(pplx_a2a_graph_t *g) {
  if (!g) return PPLX_A2A_OK;
  if (g->exec) (void)hipGraphExecDestroy(g->exec);
  if (g->graph) (void)hipGraphDestroy(g->graph);
  delete g;
  return PPLX_A2A_OK;
}

}  // extern "C"
