// gfx950 kernels of split send / recv mode: two hops through staging that the world owns.
//
// The reference lets a rank send, compute, then receive (csrc/all_to_all/all_to_all.h:9-13,
// csrc/all_to_all/bench_all_to_all.cpp:183-203).  In the loopback every phase is collective:
// the ranks' calls of a phase are recorded, and the call of the last rank enqueues ONE launch
// sequence for all of them, as in send+recv mode.  What a SEND has to do is take over
// everything its inputs hold, so that the caller may reuse them; what a RECV has to do is write
// the outputs.  With every rank in one HBM that splits the work like this:
//   dispatch SEND   split_stage_tokens: one copy of every present token (row | scales), its
//                   picks and the DP groups' token counts into the staging area
//   dispatch RECV   the one-call dispatch (a2a_dispatch.hip) on rank-table rows whose inputs
//                   point into the staging area and whose outputs are those of the RECV calls
//   combine SEND    the one-call combine (a2a_combine.hip) with its output rows pointed at the
//                   staging area: expert_y, indices, weights and bound_m are consumed here
//   combine RECV    split_deliver: every present token's combined row to the caller's out_tokens
// A step moves T + T rows more than the one-call form on dispatch (T tokens, against T + K T)
// and two rows per token more on combine.  The reference's SEND leaves one copy per pick,
// because each copy crosses a link to the expert's rank (csrc/all_to_all/intranode_dispatch.cu:
// 146-180), and reduces at RECV (csrc/all_to_all/intranode_combine.cu:127-169); here the staging
// area is the wire.
#include "a2a_rows.h"

namespace pplx_amd {
namespace {

// dispatch SEND: one wave per virtual token.  The wave of a group's token 0 also records how
// many tokens the group has this step (and reports a count beyond the limit).
template <int NV, bool EXACT, class DT>
__global__ __launch_bounds__(256) void split_stage_tokens(WorldDev w, DT tab, SplitDev sp, uint32_t write_through) {
  const uint32_t lane = lane_id();
  const uint32_t v = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave);
  const uint32_t g = group_of(w, v);
  const uint32_t t = v - g * w.M;
  if (g >= w.G) return;
  const uint32_t n = dispatch_group_tokens(w, tab, g);
  if (t == 0 && lane == 0) {
    as_global(sp.stage_n)[g] = n;
    if (dispatch_group_overflows(w, tab, g)) atomicOr(w.faults, kFaultTooManyTokens);
  }
  if (t >= n) return;
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
  uint32_t pick = 0;
  if (lane < w.K) pick = as_global(src.indices)[(size_t)t * w.K + lane];
  uint8_t *staged = sp.stage_x + (uint64_t)v * sp.token_stride;
  PPLX_GLOBAL u32x4 *out = as_global(reinterpret_cast<u32x4 *>(staged));
  // RECV reads the staged rows next: while they fit the last-level cache they are stored
  // write-through so that they stay there.
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
  PPLX_GLOBAL float *sout = as_global(reinterpret_cast<float *>(staged + w.Hb));
  if (lane < S) row_store<RowStore::kKeep>(sc, sout + lane);
  for (uint32_t j = lane + kWave; j < S; j += kWave) sout[j] = srow[(int64_t)j * src.dp_xs_stride_elem];
  if (lane < w.K) as_global(sp.stage_idx)[(size_t)v * w.K + lane] = pick;
}

// Rows beyond the register variants: plain streaming loops, one workgroup per token.
template <class DT>
__global__ __launch_bounds__(256) void split_stage_tokens_long(WorldDev w, DT tab, SplitDev sp) {
  const uint32_t v = blockIdx.x;
  const uint32_t g = group_of(w, v);
  const uint32_t t = v - g * w.M;
  if (g >= w.G) return;
  const uint32_t n = dispatch_group_tokens(w, tab, g);
  if (t == 0 && threadIdx.x == 0) {
    as_global(sp.stage_n)[g] = n;
    if (dispatch_group_overflows(w, tab, g)) atomicOr(w.faults, kFaultTooManyTokens);
  }
  if (t >= n) return;
  const DispatchRank &src = tab.at(sender_of(w, g, t));
  const uint32_t nvec = w.Hb / 16;
  const PPLX_GLOBAL u32x4 *row =
      as_global(reinterpret_cast<const u32x4 *>(src.dp_x + (int64_t)t * src.dp_x_stride_row));
  const PPLX_GLOBAL float *srow = as_global(src.dp_xs) + (int64_t)t * src.dp_xs_stride_row;
  uint8_t *staged = sp.stage_x + (uint64_t)v * sp.token_stride;
  PPLX_GLOBAL u32x4 *out = as_global(reinterpret_cast<u32x4 *>(staged));
  for (uint32_t j = threadIdx.x; j < nvec; j += blockDim.x) out[j] = row[j];
  PPLX_GLOBAL float *sout = as_global(reinterpret_cast<float *>(staged + w.Hb));
  for (uint32_t j = threadIdx.x; j < w.S; j += blockDim.x) sout[j] = srow[(int64_t)j * src.dp_xs_stride_elem];
  for (uint32_t k = threadIdx.x; k < w.K; k += blockDim.x) {
    as_global(sp.stage_idx)[(size_t)v * w.K + k] = as_global(src.indices)[(size_t)t * w.K + k];
  }
}

// combine RECV: one wave per 8 KiB of a combined row (2-byte elements) copies it from the
// staging area to the caller's out_tokens; rows from the rank's token count on are left alone.
template <class CT>
__global__ __launch_bounds__(256) void split_deliver(WorldDev w, CT tab, SplitDev sp, uint32_t segments,
                                                     FastDiv by_segments) {
  constexpr uint32_t kBatch = 8;
  const uint32_t lane = lane_id();
  const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave);
  const uint32_t token = fast_div(wave, by_segments);
  const uint32_t segment = wave - token * segments;
  const uint32_t r = group_of(w, token);  // (rank, token of the rank): R * M rows
  const uint32_t t = token - r * w.M;
  if (r >= w.R) return;
  const CombineRank &c = tab.at(r);
  if (t >= combine_rank_tokens(w, c)) return;
  const uint32_t nvec = w.H / 8;  // 16-byte vectors of a row of 2-byte elements
  const PPLX_GLOBAL u32x4 *row =
      as_global(reinterpret_cast<const u32x4 *>(sp.stage_y + (uint64_t)token * w.H * 2u));
  PPLX_GLOBAL u32x4 *out = as_global(reinterpret_cast<u32x4 *>(
      reinterpret_cast<uint8_t *>(c.out_tokens) + (int64_t)t * c.out_stride_row * 2));
  u32x4 x[kBatch];
#pragma unroll
  for (uint32_t b = 0; b < kBatch; ++b) {
    uint32_t j = (segment * kBatch + b) * kWave + lane;
    j = j < nvec ? j : nvec - 1;
    x[b] = __builtin_nontemporal_load(row + j);
  }
  SettleAll<kBatch>::of(x);
#pragma unroll
  for (uint32_t b = 0; b < kBatch; ++b) {
    const uint32_t j = (segment * kBatch + b) * kWave + lane;
    if (j < nvec) __builtin_nontemporal_store(x[b], out + j);
  }
}

template <class DT>
int launch_split_stage_tokens_t(const WorldDev &w, const SplitDev &sp, const DT &tab, hipStream_t s) {
  const uint32_t lds = 0;
  const uint32_t tokens = w.G * w.M;
  if (!row_has_register_variant(w)) {
    hipLaunchKernelGGL(split_stage_tokens_long<DT>, dim3(tokens), dim3(256), 0, s, w, tab, sp);
    return (int)hipGetLastError();
  }
  const uint64_t row_bytes = (uint64_t)tokens * sp.token_stride;
  const uint32_t write_through = row_bytes <= kWriteThroughMaxBytes ? 1u : 0u;
  const dim3 grid((tokens + 3) / 4), block(256);
#define PPLX_ROW_KERNEL_ARGS sp, write_through
#define PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL) return (int)hipErrorInvalidValue
  PPLX_DISPATCH_ROW_VARIANTS(split_stage_tokens);
#undef PPLX_LAUNCH_LARGE_ROW_VARIANT
#undef PPLX_ROW_KERNEL_ARGS
  return (int)hipGetLastError();
}

template <class CT>
int launch_split_deliver_t(const WorldDev &w, const SplitDev &sp, const CT &tab, hipStream_t s) {
  const uint32_t nvec = w.H / 8;
  const uint32_t segments = (nvec + 8 * kWave - 1) / (8 * kWave);
  const uint64_t waves = (uint64_t)w.R * w.M * segments;
  hipLaunchKernelGGL(split_deliver<CT>, dim3((uint32_t)((waves + 3) / 4)), dim3(256), 0, s, w, tab, sp, segments,
                     make_fast_div(segments));
  return (int)hipGetLastError();
}

}  // namespace

int launch_split_stage_tokens(const WorldDev &w, const SplitDev &sp, const DispatchRank *inline_rows,
                              void *stream) {
  if (inline_rows) return launch_split_stage_tokens_t(w, sp, make_inline(w, inline_rows), (hipStream_t)stream);
  return launch_split_stage_tokens_t(w, sp, HbmDispatch{w.drank}, (hipStream_t)stream);
}

int launch_split_deliver(const WorldDev &w, const SplitDev &sp, const CombineRank *inline_rows, void *stream) {
  if (inline_rows) return launch_split_deliver_t(w, sp, make_inline(w, inline_rows), (hipStream_t)stream);
  return launch_split_deliver_t(w, sp, HbmCombine{w.crank}, (hipStream_t)stream);
}

}  // namespace pplx_amd
