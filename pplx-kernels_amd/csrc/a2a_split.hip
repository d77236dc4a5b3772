// gfx950 kernels of split send / recv mode: two hops through world-owned staging in the
// reference's wire format (row | scales | source token, 16-byte padded).
#include "a2a_route.h"
#include "a2a_rows.h"

namespace pplx_amd {
namespace {

// ---------------------------------------------------------------------------
// Split send / recv mode (two hops through world-owned staging).
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint8_t *stage_row(const WorldDev &w, const SplitDev &sp, uint32_t g,
                                              uint32_t position) {
  return sp.stage_x + ((uint64_t)g * w.M * w.K + position) * sp.token_stride;
}

// dispatch SEND, second half: one wave per token of the calling rank's share packs
// row | scales | source token into the group's staging area, grouped by expert.
template <int NV, bool EXACT, class DT>
__global__ __launch_bounds__(256) void split_pack(WorldDev w, DT tab, uint32_t g, uint32_t member,
                                                  SplitDev sp) {
  const uint32_t lane = lane_id();
  const uint32_t t = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave);
  if (t >= w.M || t % w.dp != member || t >= sp.gntok[g]) return;
  const DispatchRank &src = tab.at(0);
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
    const size_t pair = ((size_t)g * w.M + t) * w.K + lane;
    const uint32_t e = as_global(sp.gexp)[pair];
    if (e < w.E) {
      dst = reinterpret_cast<uint64_t>(
          stage_row(w, sp, g, as_global(sp.goff)[(size_t)g * w.E + e] + as_global(sp.gslot)[pair]));
    }
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) settle(x[i]);
  settle(sc);
  settle(dst);
  // The staged rows are read back by the RECV phase next: they are stored write-through so
  // that they stay in the last-level cache when they fit there.
  for (uint32_t k = 0; k < w.K; ++k) {
    const uint64_t p = read_lane64(dst, k);
    if (p == 0) continue;
    PPLX_GLOBAL u32x4 *out = global_ptr<u32x4>(p);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const uint32_t j = lane + i * kWave;
      if (EXACT || j < nvec) row_store<RowStore::kKeep>(x[i], out + j);
    }
    PPLX_GLOBAL float *sout = global_ptr<float>(p + w.Hb);
    if (lane < S) row_store<RowStore::kKeep>(sc, sout + lane);
    for (uint32_t j = lane + kWave; j < S; j += kWave) sout[j] = srow[(int64_t)j * src.dp_xs_stride_elem];
    if (lane == 0) *global_ptr<uint32_t>(p + w.Hb + 4ull * S) = t;
  }
}

// First dispatch RECV of a step: rows of every expert that come from earlier groups.
__global__ __launch_bounds__(256) void split_bases(WorldDev w, SplitDev sp) {
  const uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= w.E) return;
  uint32_t running = 0;
  for (uint32_t g = 0; g < w.G; ++g) {
    sp.gbase[(size_t)g * w.E + e] = running;
    running += sp.gcnt[(size_t)g * w.E + e];
  }
}

// ... and the slot map that combine reads: slot = rows from earlier groups + slot in the group.
__global__ __launch_bounds__(256) void split_finalize(WorldDev w, SplitDev sp) {
  const uint64_t pair = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (pair >= (uint64_t)w.G * w.M * w.K) return;
  const uint32_t v = (uint32_t)(pair / w.K);
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  if (t >= sp.gntok[g]) return;
  const uint32_t e = sp.gexp[pair];
  w.slot_map[pair] = e < w.E ? sp.gbase[(size_t)g * w.E + e] + sp.gslot[pair] : kInvalidSlot;
}

// dispatch RECV of rank d: workgroup (local expert, group) copies that run of staged rows
// into out_expert_x / out_expert_x_scale; blockIdx.y spreads long runs.
template <int NV, bool EXACT, class DT>
__global__ __launch_bounds__(256) void split_unpack(WorldDev w, DT tab, uint32_t d, SplitDev sp,
                                                    uint32_t write_through) {
  const uint32_t lane = lane_id();
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const uint32_t el = blockIdx.x / w.G;
  const uint32_t g = blockIdx.x - el * w.G;
  const uint32_t e = d * w.L + el;
  const DispatchRank &dst = tab.at(0);
  const size_t ge = (size_t)g * w.E + e;
  const uint32_t count = as_global(sp.gcnt)[ge], offset = as_global(sp.goff)[ge], base = as_global(sp.gbase)[ge];
  if (g == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
    const size_t last = (size_t)(w.G - 1) * w.E + e;
    as_global(dst.out_num_tokens)[(int64_t)el * dst.out_num_tokens_stride] =
        (int32_t)(as_global(sp.gbase)[last] + as_global(sp.gcnt)[last]);
  }
  const uint32_t nvec = w.Hb / 16;
  const uint32_t S = w.S;
  for (uint32_t i = blockIdx.y * (blockDim.x / kWave) + wave; i < count; i += gridDim.y * (blockDim.x / kWave)) {
    const uint32_t slot = base + i;
    if (slot >= dst.x_rows) {
      if (lane == 0) atomicOr(w.faults, kFaultRowDropped);
      continue;
    }
    const uint8_t *src = stage_row(w, sp, g, offset + i);
    const PPLX_GLOBAL u32x4 *row = as_global(reinterpret_cast<const u32x4 *>(src));
    PPLX_GLOBAL u32x4 *out = as_global(reinterpret_cast<u32x4 *>(
        dst.expert_x + (int64_t)el * dst.x_stride_expert + (int64_t)slot * dst.x_stride_row));
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
#pragma unroll
    for (int v = 0; v < NV; ++v) settle(x[v]);
    settle(sc);
    PPLX_GLOBAL float *sout = as_global(dst.expert_xs) + (int64_t)el * dst.xs_stride_expert +
                              (int64_t)slot * dst.xs_stride_row;
    // same policy as the one-call dispatch: rows that fit the last-level cache stay there
    if (write_through) {
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const uint32_t j = lane + v * kWave;
        if (EXACT || j < nvec) row_store<RowStore::kKeep>(x[v], out + j);
      }
      if (lane < S) row_store<RowStore::kKeep>(sc, sout + (int64_t)lane * dst.xs_stride_elem);
    } else {
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const uint32_t j = lane + v * kWave;
        if (EXACT || j < nvec) row_store<RowStore::kStream>(x[v], out + j);
      }
      if (lane < S) row_store<RowStore::kStream>(sc, sout + (int64_t)lane * dst.xs_stride_elem);
    }
    for (uint32_t j = lane + kWave; j < S; j += kWave) sout[(int64_t)j * dst.xs_stride_elem] = sin[j];
  }
}

// Rows beyond the register variants: plain streaming loops, one workgroup per staged row.
template <class DT>
__global__ __launch_bounds__(256) void split_pack_long(WorldDev w, DT tab, uint32_t g, uint32_t member,
                                                       SplitDev sp) {
  const uint32_t t = blockIdx.x;
  if (t >= w.M || t % w.dp != member || t >= sp.gntok[g]) return;
  const DispatchRank &src = tab.at(0);
  const uint32_t nvec = w.Hb / 16;
  const u32x4 *row = reinterpret_cast<const u32x4 *>(src.dp_x + (int64_t)t * src.dp_x_stride_row);
  for (uint32_t k = 0; k < w.K; ++k) {
    const size_t pair = ((size_t)g * w.M + t) * w.K + k;
    const uint32_t e = sp.gexp[pair];
    if (e >= w.E) continue;
    uint8_t *p = stage_row(w, sp, g, sp.goff[(size_t)g * w.E + e] + sp.gslot[pair]);
    u32x4 *out = reinterpret_cast<u32x4 *>(p);
    for (uint32_t j = threadIdx.x; j < nvec; j += blockDim.x) out[j] = row[j];
    float *sout = reinterpret_cast<float *>(p + w.Hb);
    for (uint32_t j = threadIdx.x; j < w.S; j += blockDim.x) {
      sout[j] = src.dp_xs[(int64_t)t * src.dp_xs_stride_row + (int64_t)j * src.dp_xs_stride_elem];
    }
    if (threadIdx.x == 0) *reinterpret_cast<uint32_t *>(p + w.Hb + 4ull * w.S) = t;
  }
}

template <class DT>
__global__ __launch_bounds__(256) void split_unpack_long(WorldDev w, DT tab, uint32_t d, SplitDev sp) {
  const uint32_t el = blockIdx.x / w.G;
  const uint32_t g = blockIdx.x - el * w.G;
  const uint32_t e = d * w.L + el;
  const DispatchRank &dst = tab.at(0);
  const size_t ge = (size_t)g * w.E + e;
  const uint32_t count = sp.gcnt[ge], offset = sp.goff[ge], base = sp.gbase[ge];
  if (g == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
    const size_t last = (size_t)(w.G - 1) * w.E + e;
    dst.out_num_tokens[(int64_t)el * dst.out_num_tokens_stride] = (int32_t)(sp.gbase[last] + sp.gcnt[last]);
  }
  const uint32_t nvec = w.Hb / 16;
  for (uint32_t i = blockIdx.y; i < count; i += gridDim.y) {
    const uint32_t slot = base + i;
    if (slot >= dst.x_rows) {
      if (threadIdx.x == 0) atomicOr(w.faults, kFaultRowDropped);
      continue;
    }
    const uint8_t *src = stage_row(w, sp, g, offset + i);
    const u32x4 *row = reinterpret_cast<const u32x4 *>(src);
    u32x4 *out = reinterpret_cast<u32x4 *>(dst.expert_x + (int64_t)el * dst.x_stride_expert +
                                           (int64_t)slot * dst.x_stride_row);
    for (uint32_t j = threadIdx.x; j < nvec; j += blockDim.x) out[j] = row[j];
    const float *sin = reinterpret_cast<const float *>(src + w.Hb);
    float *sout = dst.expert_xs + (int64_t)el * dst.xs_stride_expert + (int64_t)slot * dst.xs_stride_row;
    for (uint32_t j = threadIdx.x; j < w.S; j += blockDim.x) sout[(int64_t)j * dst.xs_stride_elem] = sin[j];
  }
}

// combine SEND of rank d: one wave per (token, pick) whose expert d owns copies that
// expert_y row into the pair's staging row (the reference copies it into the source
// rank's inbox, csrc/all_to_all/intranode_combine.cu:77-111).
template <class CT>
__global__ __launch_bounds__(256) void split_combine_send(WorldDev w, CT tab, uint32_t d, SplitDev sp,
                                                          uint32_t elem_bytes) {
  const uint32_t lane = lane_id();
  const uint64_t pair = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave);
  if (pair >= (uint64_t)w.G * w.M * w.K) return;
  const uint32_t v = (uint32_t)(pair / w.K);
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  if (t >= sp.gntok[g]) return;
  const uint32_t e = sp.gexp[pair];
  if (e >= w.E || e / w.L != d) return;
  const uint32_t slot = w.slot_map[pair];
  const CombineRank &own = tab.at(0);
  if (slot >= own.y_rows) {
    if (lane == 0) atomicOr(w.faults, kFaultBadSlot);
    return;
  }
  const uint8_t *src = reinterpret_cast<const uint8_t *>(own.expert_y) +
                       ((int64_t)(e % w.L) * own.y_stride_expert + (int64_t)slot * own.y_stride_row) * elem_bytes;
  const u32x4 *row = reinterpret_cast<const u32x4 *>(src);
  u32x4 *out = reinterpret_cast<u32x4 *>(sp.stage_y + pair * sp.y_row_bytes);
  const uint32_t nvec = (uint32_t)(sp.y_row_bytes / 16);
  for (uint32_t j = lane; j < nvec; j += kWave) out[j] = __builtin_nontemporal_load(row + j);
}

}  // namespace

int launch_split_route(const WorldDev &w, const SplitDev &sp, const DispatchRank &row, uint32_t rank,
                       uint32_t pick_vector, void *stream) {
  typedef SingleDispatch DT;
  const DT tab{row};
  const uint32_t g = rank / w.dp;
  RouteSpan span{};
  span.v_begin = g * w.M;
  span.v_count = w.M;
  span.tile_chunks = sp.tile_chunks;
  span.pick_vector = pick_vector;
  span.tile_cnt = sp.gtile_cnt + (size_t)g * sp.tiles_per_group * w.E;
  span.slot_out = sp.gslot;
  span.expert_out = sp.gexp;
  span.counts_out = sp.gcnt + (size_t)g * w.E;
  span.offsets_out = sp.goff + (size_t)g * w.E;
  span.ntok_out = sp.gntok + g;
  return launch_route_t<DT, true>(w, tab, span, (hipStream_t)stream);
}

int launch_split_dispatch_send(const WorldDev &w, const SplitDev &sp, const DispatchRank &row,
                               uint32_t rank, void *stream) {
  typedef SingleDispatch DT;
  hipStream_t s = (hipStream_t)stream;
  const DT tab{row};
  const uint32_t g = rank / w.dp, member = rank % w.dp;
  const uint32_t lds = 0;
  if (!row_has_register_variant(w)) {
    hipLaunchKernelGGL(split_pack_long<DT>, dim3(w.M), dim3(256), 0, s, w, tab, g, member, sp);
    return (int)hipGetLastError();
  }
  const dim3 grid((w.M + 3) / 4), block(256);
#define PPLX_ROW_KERNEL_ARGS g, member, sp
#define PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL) return (int)hipErrorInvalidValue
  PPLX_DISPATCH_ROW_VARIANTS(split_pack);
#undef PPLX_LAUNCH_LARGE_ROW_VARIANT
#undef PPLX_ROW_KERNEL_ARGS
  return (int)hipGetLastError();
}

int launch_split_dispatch_recv(const WorldDev &w, const SplitDev &sp, const DispatchRank &row,
                               uint32_t rank, bool first_of_step, void *stream) {
  typedef SingleDispatch DT;
  hipStream_t s = (hipStream_t)stream;
  const DT tab{row};
  if (first_of_step) {
    hipLaunchKernelGGL(split_bases, dim3((w.E + 255) / 256), dim3(256), 0, s, w, sp);
    const uint64_t pairs = (uint64_t)w.G * w.M * w.K;
    hipLaunchKernelGGL(split_finalize, dim3((uint32_t)((pairs + 255) / 256)), dim3(256), 0, s, w, sp);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return (int)err;
  }
  const uint32_t lds = 0;
  // Row groups per (local expert, group) run: enough workgroups to cover the CUs even with few
  // experts per rank, and a hot expert's long run is shared; never more than the run can use.
  const uint32_t runs = w.L * w.G;
  uint32_t spread = (2048 + runs - 1) / runs;
  const uint32_t most = (w.M + 3) / 4;
  if (spread > most) spread = most;
  if (spread > 256) spread = 256;
  if (spread < 1) spread = 1;
  const dim3 grid(w.L * w.G, spread), block(256);
  if (!row_has_register_variant(w)) {
    hipLaunchKernelGGL(split_unpack_long<DT>, grid, block, 0, s, w, tab, rank, sp);
    return (int)hipGetLastError();
  }
  const uint64_t row_bytes = (uint64_t)w.G * w.M * w.K * (w.Hb + 4ull * w.S);
  const uint32_t write_through = row_bytes <= kWriteThroughMaxBytes ? 1u : 0u;
#define PPLX_ROW_KERNEL_ARGS rank, sp, write_through
#define PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL) return (int)hipErrorInvalidValue
  PPLX_DISPATCH_ROW_VARIANTS(split_unpack);
#undef PPLX_LAUNCH_LARGE_ROW_VARIANT
#undef PPLX_ROW_KERNEL_ARGS
  return (int)hipGetLastError();
}

int launch_split_combine_send(const WorldDev &w, const SplitDev &sp, const CombineRank &row,
                              uint32_t rank, int in_dtype, void *stream) {
  const SingleCombine tab{row};
  const uint64_t pairs = (uint64_t)w.G * w.M * w.K;
  const uint32_t elem_bytes = in_dtype == 0 ? 4u : 2u;
  hipLaunchKernelGGL(split_combine_send<SingleCombine>, dim3((uint32_t)((pairs + 3) / 4)), dim3(256), 0,
                     (hipStream_t)stream, w, tab, rank, sp, elem_bytes);
  return (int)hipGetLastError();
}

}  // namespace pplx_amd
