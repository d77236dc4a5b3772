// gfx950 kernels of split send / recv mode: two hops through world-owned staging in the
// reference's wire format (row | scales | source token, 16-byte padded).
//
// The reference lets a rank send, compute, then receive (csrc/all_to_all/all_to_all.h:9-13,
// csrc/all_to_all/bench_all_to_all.cpp:183-203).  In the loopback every phase is collective:
// the ranks' calls of a phase are recorded, and the call of the last rank enqueues ONE launch
// sequence for all of them, as in send+recv mode.
//   dispatch SEND   routes the whole step (slot map, rows per expert, expert of every pair) and
//                   leaves one copy of the row per (token, pick) in the staging area, in the
//                   order of the picks: small steps in the one launch of the one-call form
//                   (dispatch_fused with its rows pointed at the staging area, a2a_dispatch.hip),
//                   larger ones as the routing launches followed by split_pack
//   dispatch RECV   moves every staged row to its slot in the owning rank's outputs
//   combine SEND    copies the expert_y row of every (token, pick) into the pair's staging row
//                   (the reference copies it into the source rank's inbox,
//                   csrc/all_to_all/intranode_combine.cu:77-111)
//   combine RECV    is combine_gather reading the staged rows (a2a_combine.hip)
#include "a2a_route.h"
#include "a2a_rows.h"

namespace pplx_amd {
namespace {

__device__ __forceinline__ uint8_t *stage_row(const SplitDev &sp, uint64_t pair) {
  return sp.stage_x + pair * sp.token_stride;
}

// dispatch SEND, second half: one wave per token packs row | scales | source token for each of
// its picks.  Lane k resolves pick k.
template <int NV, bool EXACT, class DT>
__global__ __launch_bounds__(256) void split_pack(WorldDev w, DT tab, SplitDev sp, uint32_t write_through) {
  const uint32_t lane = lane_id();
  const uint32_t v = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave);
  const uint32_t g = group_of(w, v);
  const uint32_t t = v - g * w.M;
  if (g >= w.G) return;
  if (t >= dispatch_group_tokens(w, tab, g)) return;
  const DispatchRank &src = tab.at(sender_of(w, g, t));
  const uint32_t nvec = w.Hb / 16;
  const PPLX_GLOBAL u32x4 *row =
      as_global(reinterpret_cast<const u32x4 *>(src.dp_x + (int64_t)t * src.dp_x_stride_row));
  u32x4 x[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    uint32_t j = lane + i * kWave;
    if (!EXACT) j = j < nvec ? j : nvec - 1;
    x[i] = row[j];
  }
  const uint32_t S = w.S;
  // scale `lane` of the row; rows of more than 64 scales take the loop below
  float sc = 0.f;
  const PPLX_GLOBAL float *srow = as_global(src.dp_xs) + (int64_t)t * src.dp_xs_stride_row;
  if (S) sc = srow[(int64_t)(lane < S ? lane : S - 1) * src.dp_xs_stride_elem];
  uint64_t dst = 0;
  if (lane < w.K) {
    const size_t pair = (size_t)v * w.K + lane;
    if (as_global(sp.gexp)[pair] < w.E) dst = reinterpret_cast<uint64_t>(stage_row(sp, pair));
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) settle(x[i]);
  settle(sc);
  settle(dst);
  // The staged rows are read back by the RECV phase next: while they fit the last-level cache
  // they are stored write-through so that they stay there.
  for (uint32_t k = 0; k < w.K; ++k) {
    const uint64_t p = read_lane64(dst, k);
    if (p == 0) continue;
    PPLX_GLOBAL u32x4 *out = global_ptr<u32x4>(p);
    if (write_through) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const uint32_t j = lane + i * kWave;
        if (EXACT || j < nvec) row_store<RowStore::kKeep>(x[i], out + j);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const uint32_t j = lane + i * kWave;
        if (EXACT || j < nvec) row_store<RowStore::kStreamThrough>(x[i], out + j);
      }
    }
    PPLX_GLOBAL float *sout = global_ptr<float>(p + w.Hb);
    if (lane < S) row_store<RowStore::kKeep>(sc, sout + lane);
    for (uint32_t j = lane + kWave; j < S; j += kWave) sout[j] = srow[(int64_t)j * src.dp_xs_stride_elem];
    if (lane == 0) *global_ptr<uint32_t>(p + w.Hb + 4ull * S) = t;
  }
}

// Rows beyond the register variants: plain streaming loops, one workgroup per token.
template <class DT>
__global__ __launch_bounds__(256) void split_pack_long(WorldDev w, DT tab, SplitDev sp) {
  const uint32_t v = blockIdx.x;
  const uint32_t g = group_of(w, v);
  const uint32_t t = v - g * w.M;
  if (g >= w.G) return;
  if (t >= dispatch_group_tokens(w, tab, g)) return;
  const DispatchRank &src = tab.at(sender_of(w, g, t));
  const uint32_t nvec = w.Hb / 16;
  const PPLX_GLOBAL u32x4 *row =
      as_global(reinterpret_cast<const u32x4 *>(src.dp_x + (int64_t)t * src.dp_x_stride_row));
  const PPLX_GLOBAL float *srow = as_global(src.dp_xs) + (int64_t)t * src.dp_xs_stride_row;
  for (uint32_t k = 0; k < w.K; ++k) {
    const size_t pair = (size_t)v * w.K + k;
    if (as_global(sp.gexp)[pair] >= w.E) continue;
    uint8_t *p = stage_row(sp, pair);
    PPLX_GLOBAL u32x4 *out = as_global(reinterpret_cast<u32x4 *>(p));
    for (uint32_t j = threadIdx.x; j < nvec; j += blockDim.x) out[j] = row[j];
    PPLX_GLOBAL float *sout = as_global(reinterpret_cast<float *>(p + w.Hb));
    for (uint32_t j = threadIdx.x; j < w.S; j += blockDim.x) sout[j] = srow[(int64_t)j * src.dp_xs_stride_elem];
    if (threadIdx.x == 0) *as_global(reinterpret_cast<uint32_t *>(p + w.Hb + 4ull * w.S)) = t;
  }
}

// The first workgroup of a RECV launch hands the rows per expert to the owning ranks.
template <class DT>
__device__ __forceinline__ void publish_counts(const WorldDev &w, const DT &tab, const SplitDev &sp) {
  if (blockIdx.x != 0) return;
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) {
    const DispatchRank &dst = tab.at(owner_of(w, e));
    as_global(dst.out_num_tokens)[(int64_t)local_of(w, e) * dst.out_num_tokens_stride] = (int32_t)as_global(sp.gcnt)[e];
  }
}

// dispatch RECV: one wave per (token, pick) moves the pair's staged row to its slot in
// out_expert_x / out_expert_x_scale of the rank that owns the expert.  `eager`: the row is
// fetched together with the pair's expert and slot instead of behind them (one trip to memory
// instead of two; pays while few pairs are empty).
template <int NV, bool EXACT, class DT>
__global__ __launch_bounds__(256) void split_unpack(WorldDev w, DT tab, SplitDev sp, uint32_t write_through,
                                                    uint32_t eager) {
  publish_counts(w, tab, sp);
  const uint32_t lane = lane_id();
  const uint64_t pair = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave);
  if (pair >= (uint64_t)w.G * w.M * w.K) return;
  const uint32_t e = as_global(sp.gexp)[pair];
  const uint32_t slot = as_global(w.slot_map)[pair];
  if (!eager && (e >= w.E || slot == kInvalidSlot)) return;
  const uint8_t *src = stage_row(sp, pair);
  const PPLX_GLOBAL u32x4 *row = as_global(reinterpret_cast<const u32x4 *>(src));
  const uint32_t nvec = w.Hb / 16;
  const uint32_t S = w.S;
  u32x4 x[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    uint32_t j = lane + v * kWave;
    if (!EXACT) j = j < nvec ? j : nvec - 1;
    x[v] = row[j];
  }
  float sc = 0.f;
  const PPLX_GLOBAL float *sin = as_global(reinterpret_cast<const float *>(src + w.Hb));
  if (S) sc = sin[lane < S ? lane : S - 1];
  // (pins the row loads in front of the branch below)
#pragma unroll
  for (int v = 0; v < NV; ++v) settle(x[v]);
  settle(sc);
  if (e >= w.E || slot == kInvalidSlot) return;
  const DispatchRank &dst = tab.at(owner_of(w, e));
  const uint32_t el = local_of(w, e);
  if (slot >= dst.x_rows) {
    if (lane == 0) atomicOr(w.faults, kFaultRowDropped);
    return;
  }
  PPLX_GLOBAL u32x4 *out = as_global(reinterpret_cast<u32x4 *>(
      dst.expert_x + (int64_t)el * dst.x_stride_expert + (int64_t)slot * dst.x_stride_row));
  PPLX_GLOBAL float *sout = as_global(dst.expert_xs) + (int64_t)el * dst.xs_stride_expert +
                            (int64_t)slot * dst.xs_stride_row;
  // same policy as the one-call dispatch: rows that fit the last-level cache stay there
  if (write_through) {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const uint32_t j = lane + v * kWave;
      if (EXACT || j < nvec) row_store<RowStore::kKeep>(x[v], out + j);
    }
  } else {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const uint32_t j = lane + v * kWave;
      if (EXACT || j < nvec) row_store<RowStore::kStreamThrough>(x[v], out + j);
    }
  }
  if (lane < S) row_store<RowStore::kKeep>(sc, sout + (int64_t)lane * dst.xs_stride_elem);
  for (uint32_t j = lane + kWave; j < S; j += kWave) sout[(int64_t)j * dst.xs_stride_elem] = sin[j];
}

// Rows beyond the register variants: one workgroup per (token, pick).
template <class DT>
__global__ __launch_bounds__(256) void split_unpack_long(WorldDev w, DT tab, SplitDev sp) {
  publish_counts(w, tab, sp);
  const uint64_t pair = blockIdx.x;
  const uint32_t e = as_global(sp.gexp)[pair];
  const uint32_t slot = as_global(w.slot_map)[pair];
  if (e >= w.E || slot == kInvalidSlot) return;
  const DispatchRank &dst = tab.at(owner_of(w, e));
  const uint32_t el = local_of(w, e);
  if (slot >= dst.x_rows) {
    if (threadIdx.x == 0) atomicOr(w.faults, kFaultRowDropped);
    return;
  }
  const uint32_t nvec = w.Hb / 16;
  const uint8_t *src = stage_row(sp, pair);
  const PPLX_GLOBAL u32x4 *row = as_global(reinterpret_cast<const u32x4 *>(src));
  PPLX_GLOBAL u32x4 *out = as_global(reinterpret_cast<u32x4 *>(
      dst.expert_x + (int64_t)el * dst.x_stride_expert + (int64_t)slot * dst.x_stride_row));
  for (uint32_t j = threadIdx.x; j < nvec; j += blockDim.x) out[j] = row[j];
  const PPLX_GLOBAL float *sin = as_global(reinterpret_cast<const float *>(src + w.Hb));
  PPLX_GLOBAL float *sout = as_global(dst.expert_xs) + (int64_t)el * dst.xs_stride_expert +
                            (int64_t)slot * dst.xs_stride_row;
  for (uint32_t j = threadIdx.x; j < w.S; j += blockDim.x) sout[(int64_t)j * dst.xs_stride_elem] = sin[j];
}

// combine SEND: one wave per (token, pick) copies the expert_y row of the pick's expert into
// the pair's staging row, eight 16-byte vectors per lane in flight.
template <class CT>
__global__ __launch_bounds__(256) void split_combine_send(WorldDev w, CT tab, SplitDev sp, uint32_t elem_bytes) {
  const uint32_t lane = lane_id();
  const uint64_t pair = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave);
  if (pair >= (uint64_t)w.G * w.M * w.K) return;
  const uint32_t v = fast_div((uint32_t)pair, w.by_K);
  const uint32_t g = group_of(w, v);
  const uint32_t t = v - g * w.M;
  const CombineRank &head = tab.at(g * w.dp);
  if (t >= combine_rank_tokens(w, head)) return;
  // The pair's expert comes from this call's own indices, as in combine_gather: the routing
  // tables of split mode's dispatch SEND say nothing about a step that was dispatched in one
  // call.  The slot map alone says whether the pair has a row (a repeated or unknown expert
  // has none), whichever form of dispatch wrote it.
  const uint32_t e = as_global(head.indices)[pair - (uint64_t)g * w.M * w.K];
  const uint32_t slot = as_global(w.slot_map)[pair];
  if (e >= w.E || slot == kInvalidSlot) return;
  const CombineRank &own = tab.at(owner_of(w, e));
  if (slot >= own.y_rows) {
    if (lane == 0) atomicOr(w.faults, kFaultBadSlot);
    return;
  }
  const uint8_t *src = reinterpret_cast<const uint8_t *>(own.expert_y) +
                       ((int64_t)local_of(w, e) * own.y_stride_expert + (int64_t)slot * own.y_stride_row) * elem_bytes;
  const PPLX_GLOBAL u32x4 *row = as_global(reinterpret_cast<const u32x4 *>(src));
  PPLX_GLOBAL u32x4 *out = as_global(reinterpret_cast<u32x4 *>(sp.stage_y + pair * sp.y_row_bytes));
  const uint32_t nvec = (uint32_t)(sp.y_row_bytes / 16);
  constexpr uint32_t kBatch = 8;
  for (uint32_t j0 = 0; j0 < nvec; j0 += kBatch * kWave) {
    u32x4 x[kBatch];
#pragma unroll
    for (uint32_t b = 0; b < kBatch; ++b) {
      uint32_t j = j0 + b * kWave + lane;
      j = j < nvec ? j : nvec - 1;
      x[b] = __builtin_nontemporal_load(row + j);
    }
    SettleAll<kBatch>::of(x);
#pragma unroll
    for (uint32_t b = 0; b < kBatch; ++b) {
      const uint32_t j = j0 + b * kWave + lane;
      if (j < nvec) row_store<RowStore::kKeep>(x[b], out + j);
    }
  }
}

template <class DT>
int launch_split_pack_t(const WorldDev &w, const SplitDev &sp, const DT &tab, hipStream_t s) {
  const uint32_t lds = 0;
  const uint32_t tokens = w.G * w.M;
  if (!row_has_register_variant(w)) {
    hipLaunchKernelGGL(split_pack_long<DT>, dim3(tokens), dim3(256), 0, s, w, tab, sp);
    return (int)hipGetLastError();
  }
  const uint64_t row_bytes = (uint64_t)tokens * w.K * sp.token_stride;
  const uint32_t write_through = row_bytes <= kWriteThroughMaxBytes ? 1u : 0u;
  const dim3 grid((tokens + 3) / 4), block(256);
#define PPLX_ROW_KERNEL_ARGS sp, write_through
#define PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL) return (int)hipErrorInvalidValue
  PPLX_DISPATCH_ROW_VARIANTS(split_pack);
#undef PPLX_LAUNCH_LARGE_ROW_VARIANT
#undef PPLX_ROW_KERNEL_ARGS
  return (int)hipGetLastError();
}

template <class DT>
int launch_split_dispatch_recv_t(const WorldDev &w, const SplitDev &sp, const DT &tab, hipStream_t s) {
  const uint32_t lds = 0;
  const uint64_t pairs = (uint64_t)w.G * w.M * w.K;
  if (!row_has_register_variant(w)) {
    hipLaunchKernelGGL(split_unpack_long<DT>, dim3((uint32_t)pairs), dim3(256), 0, s, w, tab, sp);
    return (int)hipGetLastError();
  }
  const uint64_t row_bytes = pairs * (w.Hb + 4ull * w.S);
  const uint32_t write_through = row_bytes <= kWriteThroughMaxBytes ? 1u : 0u;
  // Small steps are mostly full (decode batches); the reads of empty pairs of a large ragged
  // one would cost more than the trip saved.
  const uint32_t eager = (uint64_t)w.G * w.M <= kFusedMaxTokens ? 1u : 0u;
  const dim3 grid((uint32_t)((pairs + 3) / 4)), block(256);
#define PPLX_ROW_KERNEL_ARGS sp, write_through, eager
#define PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL) return (int)hipErrorInvalidValue
  PPLX_DISPATCH_ROW_VARIANTS(split_unpack);
#undef PPLX_LAUNCH_LARGE_ROW_VARIANT
#undef PPLX_ROW_KERNEL_ARGS
  return (int)hipGetLastError();
}

template <class CT>
int launch_split_combine_send_t(const WorldDev &w, const SplitDev &sp, const CT &tab, int in_dtype,
                                hipStream_t s) {
  const uint64_t pairs = (uint64_t)w.G * w.M * w.K;
  const uint32_t elem_bytes = in_dtype == 0 ? 4u : 2u;
  hipLaunchKernelGGL(split_combine_send<CT>, dim3((uint32_t)((pairs + 3) / 4)), dim3(256), 0, s, w, tab, sp,
                     elem_bytes);
  return (int)hipGetLastError();
}

}  // namespace

int launch_split_pack(const WorldDev &w, const SplitDev &sp, const DispatchRank *inline_rows, void *stream) {
  if (inline_rows) return launch_split_pack_t(w, sp, make_inline(w, inline_rows), (hipStream_t)stream);
  return launch_split_pack_t(w, sp, HbmDispatch{w.drank}, (hipStream_t)stream);
}

int launch_split_dispatch_recv(const WorldDev &w, const SplitDev &sp, const DispatchRank *inline_rows,
                               void *stream) {
  if (inline_rows) return launch_split_dispatch_recv_t(w, sp, make_inline(w, inline_rows), (hipStream_t)stream);
  return launch_split_dispatch_recv_t(w, sp, HbmDispatch{w.drank}, (hipStream_t)stream);
}

int launch_split_combine_send(const WorldDev &w, const SplitDev &sp, const CombineRank *inline_rows,
                              int in_dtype, void *stream) {
  if (inline_rows)
    return launch_split_combine_send_t(w, sp, make_inline(w, inline_rows), in_dtype, (hipStream_t)stream);
  return launch_split_combine_send_t(w, sp, HbmCombine{w.crank}, in_dtype, (hipStream_t)stream);
}

}  // namespace pplx_amd
