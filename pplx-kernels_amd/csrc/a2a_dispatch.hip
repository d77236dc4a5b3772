// gfx950 kernels of the MoE dispatch / combine path (single-GPU loopback).
//
// The reference moves every token through a per-peer inbox with atomically
// assigned slots and grid-wide syncs (csrc/all_to_all/intranode_dispatch.cu:15-284,
// csrc/all_to_all/intranode_combine.cu:16-187).  With all simulated ranks in one
// HBM the same results come from a count -> scan -> scatter pipeline whose
// placement is the canonical (expert, DP group, token) order that the
// reference's tests enumerate (tests/test_all_to_all.py:113-120):
//
//   route_count      per routing tile: histogram of expert ids        (only if > 1 tile)
//   route_slots      per routing tile: 64-token bitmasks per expert in LDS,
//                    prefix over chunks and earlier tiles -> slot_map, counts
//   dispatch_scatter one wave per token (or per share of its K picks): the row
//                    is read once into registers and stored K times, 16 B / lane
//   dispatch_fused   small steps: routing and scatter in one launch; every
//                    workgroup recounts the picks of the tokens before its own
//   combine_gather   one wave per 1 KiB of an output row: K rows gathered through
//                    the slot map, fp32 accumulate in pick order, 16 B stores
//
// No atomics on global memory (fault flags aside), no spin waits, no
// cooperative launch: phase boundaries are kernel boundaries on one stream, so a
// step captures into a hipGraph as is.  Wavefronts are 64 wide throughout.
//
// Rank tables reach the kernels either inline, as kernel arguments (worlds of
// up to kInlineRanks ranks: nothing to bind, nothing to go stale), or through
// the HBM tables written by bind_rows.
#include "a2a_route.h"
#include "a2a_rows.h"

namespace pplx_amd {
namespace {

// ---------------------------------------------------------------------------
// Table binding: rows arrive as kernel arguments and are stored with vector
// stores, so a captured graph carries its own pointers.
// ---------------------------------------------------------------------------
template <typename Batch, typename Row>
__global__ __launch_bounds__(256) void bind_rows(Row *table, Batch b) {
  constexpr uint32_t kWords = sizeof(Row) / 8;
  const uint64_t *src = reinterpret_cast<const uint64_t *>(b.rows);
  uint64_t *dst = reinterpret_cast<uint64_t *>(table + b.first);
  for (uint32_t i = threadIdx.x; i < b.count * kWords; i += blockDim.x) {
    dst[i] = src[i];
  }
}

template <int NV, bool EXACT, class DT>
__global__ __launch_bounds__(256) void dispatch_scatter(WorldDev w, DT tab, uint32_t ksplit, uint32_t kper) {
  const uint32_t lane = lane_id();
  const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) +
                                                       threadIdx.x / kWave);
  const uint32_t v = wave / ksplit;
  const uint32_t part = wave - v * ksplit;
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  if (g >= w.G) return;
  if (t >= dispatch_group_tokens(w, tab, g)) return;
  // The sender of token t inside its DP group (csrc/all_to_all/intranode_dispatch.cu:97).
  const DispatchRank &src = tab.at(g * w.dp + t % w.dp);
  RowRegs<NV> regs;
  load_row<NV, EXACT>(w, src, t, lane, regs);
  Destination dst;
  if (lane < w.K) {
    dst = resolve_destination(w, tab, src.indices[(size_t)t * w.K + lane], w.slot_map[(size_t)v * w.K + lane],
                              part == 0);
  }
  const uint32_t k0 = part * kper;
  const uint32_t k1 = (k0 + kper < w.K) ? k0 + kper : w.K;
  store_row<NV, EXACT>(w, src, t, lane, dst, k0, k1, regs);
}

// Small steps: one launch does routing and scatter.  A workgroup owns tokens_per_block
// consecutive virtual tokens and their tokens_per_block * K picks, one thread per pick.
//   1. every wave issues the loads of its token's row, every pick thread the load of its
//      expert id: nothing here depends on the routing, so it overlaps with it;
//   2. the workgroup counts, per expert, the picks of all tokens before its own (every
//      workgroup repeats this over the indices, which are a few KiB in L2);
//   3. the pick threads take their slots token by token out of the LDS counters, resolve the
//      destination rows once for the workgroup and leave them in LDS;
//   4. the waves fan their rows out.  The last workgroup has counted everything and writes
//      out_expert_num_tokens.
template <int NV, bool EXACT, class DT>
__global__ __launch_bounds__(1024) void dispatch_fused(WorldDev w, DT tab, uint32_t ksplit, uint32_t kper) {
  extern __shared__ unsigned long long lds_u64[];
  const uint32_t waves = blockDim.x / kWave;
  const uint32_t tokens_per_block = waves / ksplit;
  const uint32_t own_pairs = tokens_per_block * w.K;
  unsigned long long *dst_row = lds_u64;                         // [own_pairs]
  unsigned long long *dst_scale = dst_row + own_pairs;           // [own_pairs]
  long long *dst_step = reinterpret_cast<long long *>(dst_scale + own_pairs);  // [own_pairs]
  uint32_t *hist = reinterpret_cast<uint32_t *>(dst_step + own_pairs);         // [E]
  uint32_t *ntok = hist + w.E;                                                 // [G]

  const uint32_t total = w.G * w.M;
  const uint32_t v0 = blockIdx.x * tokens_per_block;

  // 1a. this wave's token and its row
  const uint32_t lane = lane_id();
  const uint32_t my_wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const uint32_t my_j = my_wave / ksplit;
  const uint32_t my_part = my_wave - my_j * ksplit;
  const uint32_t my_v = v0 + my_j;
  const uint32_t my_g = my_v / w.M;
  const uint32_t my_t = my_v - my_g * w.M;
  const bool my_in_range = my_j < tokens_per_block && my_v < total;
  const DispatchRank &my_src = tab.at(my_in_range ? my_g * w.dp + my_t % w.dp : 0);
  const bool my_row_exists = my_in_range && my_t < my_src.m;
  RowRegs<NV> regs;
  if (my_row_exists) load_row<NV, EXACT>(w, my_src, my_t, lane, regs);

  // 1b. this thread's pick (threads beyond own_pairs have none)
  const uint32_t pick_j = threadIdx.x / w.K;
  const uint32_t pick_k = threadIdx.x - pick_j * w.K;
  const uint32_t pick_v = v0 + pick_j;
  const uint32_t pick_g = pick_v / w.M;
  const uint32_t pick_t = pick_v - pick_g * w.M;
  bool pick_exists = threadIdx.x < own_pairs && pick_v < total;
  uint32_t pick_e = w.E;
  if (pick_exists) {
    const DispatchRank &src = tab.at(pick_g * w.dp + pick_t % w.dp);
    pick_exists = pick_t < src.m;
    if (pick_exists) pick_e = src.indices[(size_t)pick_t * w.K + pick_k];
  }

  // 2. picks of all earlier tokens
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) hist[e] = 0;
  for (uint32_t g = threadIdx.x; g < w.G; g += blockDim.x) ntok[g] = dispatch_group_tokens(w, tab, g);
  __syncthreads();
  for (uint32_t v = threadIdx.x; v < v0; v += blockDim.x) {
    const uint32_t g = v / w.M;
    const uint32_t t = v - g * w.M;
    if (t < ntok[g]) {
      const uint32_t *idx = tab.at(g * w.dp + t % w.dp).indices + (size_t)t * w.K;
      for (uint32_t k = 0; k < w.K; ++k) {
        const uint32_t e = idx[k];
        if (e < w.E) atomicAdd(&hist[e], 1u);
      }
    }
  }
  __syncthreads();

  // 3. own slots, token by token (the experts of one token are distinct: no two threads of a
  // round share a counter), then the destinations
  const bool pick_live = pick_exists && pick_t < ntok[pick_g];
  uint32_t pick_slot = kInvalidSlot;
  for (uint32_t j = 0; j < tokens_per_block; ++j) {
    if (pick_live && pick_j == j && pick_e < w.E) {
      pick_slot = hist[pick_e];
      hist[pick_e] = pick_slot + 1;
    }
    __syncthreads();
  }
  if (threadIdx.x < own_pairs) {
    Destination d;
    if (pick_live) {
      d = resolve_destination(w, tab, pick_e, pick_slot, true);
      w.slot_map[(size_t)pick_v * w.K + pick_k] = pick_slot;
      if (pick_e >= w.E) atomicOr(w.faults, kFaultBadExpert);
    }
    dst_row[threadIdx.x] = d.row;
    dst_scale[threadIdx.x] = d.scale;
    dst_step[threadIdx.x] = d.scale_step;
  }
  if (blockIdx.x == gridDim.x - 1) {
    for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) {
      const DispatchRank &owner = tab.at(e / w.L);
      owner.out_num_tokens[(int64_t)(e % w.L) * owner.out_num_tokens_stride] = (int32_t)hist[e];
    }
  }
  __syncthreads();

  // 4. fan out
  if (!my_row_exists || my_t >= ntok[my_g]) return;
  Destination dst;
  if (lane < w.K) {
    dst.row = dst_row[my_j * w.K + lane];
    dst.scale = dst_scale[my_j * w.K + lane];
    dst.scale_step = dst_step[my_j * w.K + lane];
  }
  const uint32_t k0 = my_part * kper;
  const uint32_t k1 = (k0 + kper < w.K) ? k0 + kper : w.K;
  store_row<NV, EXACT>(w, my_src, my_t, lane, dst, k0, k1, regs);
}

// Rows longer than the register variants cover: stream each vector K times.
template <class DT>
__global__ __launch_bounds__(256) void dispatch_scatter_long(WorldDev w, DT tab) {
  __shared__ uint64_t s_row[kWave];
  __shared__ uint64_t s_scale[kWave];
  __shared__ int64_t s_step[kWave];
  const uint32_t v = blockIdx.x;
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  if (g >= w.G) return;
  if (t >= dispatch_group_tokens(w, tab, g)) return;
  const DispatchRank &src = tab.at(g * w.dp + t % w.dp);
  if (threadIdx.x < w.K) {
    uint64_t dst_row = 0, dst_scale = 0;
    int64_t step = 0;
    const uint32_t e = src.indices[(size_t)t * w.K + threadIdx.x];
    const uint32_t slot = w.slot_map[(size_t)v * w.K + threadIdx.x];
    if (e < w.E && slot != kInvalidSlot) {
      const DispatchRank &dst = tab.at(e / w.L);
      const uint32_t el = e % w.L;
      if (slot < dst.x_rows) {
        dst_row = reinterpret_cast<uint64_t>(dst.expert_x + (int64_t)el * dst.x_stride_expert +
                                             (int64_t)slot * dst.x_stride_row);
        if (w.S) {
          dst_scale = reinterpret_cast<uint64_t>(dst.expert_xs + (int64_t)el * dst.xs_stride_expert +
                                                 (int64_t)slot * dst.xs_stride_row);
          step = dst.xs_stride_elem;
        }
      } else {
        atomicOr(w.faults, kFaultRowDropped);
      }
    }
    s_row[threadIdx.x] = dst_row;
    s_scale[threadIdx.x] = dst_scale;
    s_step[threadIdx.x] = step;
  }
  __syncthreads();
  const uint32_t nvec = w.Hb / 16;
  const u32x4 *row = reinterpret_cast<const u32x4 *>(src.dp_x + (int64_t)t * src.dp_x_stride_row);
  for (uint32_t j = threadIdx.x; j < nvec; j += blockDim.x) {
    const u32x4 x = row[j];
    for (uint32_t k = 0; k < w.K; ++k) {
      if (s_row[k]) reinterpret_cast<u32x4 *>(s_row[k])[j] = x;
    }
  }
  if (w.S) {
    const float *srow = src.dp_xs + (int64_t)t * src.dp_xs_stride_row;
    for (uint32_t j = threadIdx.x; j < w.S; j += blockDim.x) {
      const float sc = srow[(int64_t)j * src.dp_xs_stride_elem];
      for (uint32_t k = 0; k < w.K; ++k) {
        if (s_scale[k]) reinterpret_cast<float *>(s_scale[k])[(int64_t)j * s_step[k]] = sc;
      }
    }
  }
}

// Number of waves a row's K copies are spread over: few tokens -> more waves,
// so that the launch still covers the 256 CUs (the row re-reads hit L2).
uint32_t fused_lds_bytes(const WorldDev &w, uint32_t tokens_per_block) {
  return tokens_per_block * w.K * 24u + (w.E + w.G) * (uint32_t)sizeof(uint32_t);
}

uint32_t pick_ksplit(const WorldDev &w, uint32_t max_split) {
  const uint64_t tokens = (uint64_t)w.G * w.M;
  uint32_t ksplit = 1;
  while (ksplit < max_split && ksplit < w.K && tokens * ksplit < 4096) ksplit *= 2;
  return ksplit;
}

template <class DT>
int launch_scatter_t(const WorldDev &w, const DT &tab, hipStream_t s) {
  const uint32_t tokens = w.G * w.M;
  if ((w.Hb / 16 + kWave - 1) / kWave > 32) {
    hipLaunchKernelGGL(dispatch_scatter_long<DT>, dim3(tokens), dim3(256), 0, s, w, tab);
    return (int)hipGetLastError();
  }
  const uint32_t ksplit = pick_ksplit(w, kWave);
  const uint32_t kper = (w.K + ksplit - 1) / ksplit;
  const uint64_t waves = (uint64_t)tokens * ksplit;
  const dim3 grid((uint32_t)((waves + 3) / 4)), block(256);
  const uint32_t lds = 0;
#define PPLX_ROW_KERNEL_ARGS ksplit, kper
#define PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL)                                                    \
  do {                                                                                           \
    if (per_lane <= 16) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 16, false);                              \
    else PPLX_LAUNCH_ROW_VARIANT(KERNEL, 32, false);                                             \
  } while (0)
  PPLX_DISPATCH_ROW_VARIANTS(dispatch_scatter);
#undef PPLX_LAUNCH_LARGE_ROW_VARIANT
#undef PPLX_ROW_KERNEL_ARGS
  return (int)hipGetLastError();
}

template <class DT>
int launch_fused_t(const WorldDev &w, const DT &tab, hipStream_t s) {
  const uint32_t tokens = w.G * w.M;
  constexpr uint32_t kWaves = 16;  // 1024 threads: fewer, larger workgroups repeat less counting
  const uint32_t ksplit = pick_ksplit(w, kWaves);
  const uint32_t kper = (w.K + ksplit - 1) / ksplit;
  const uint32_t tokens_per_block = kWaves / ksplit;
  const dim3 grid((tokens + tokens_per_block - 1) / tokens_per_block), block(kWaves * kWave);
  const uint32_t lds = fused_lds_bytes(w, tokens_per_block);
#define PPLX_ROW_KERNEL_ARGS ksplit, kper
#define PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL) return (int)hipErrorInvalidValue
  PPLX_DISPATCH_ROW_VARIANTS(dispatch_fused);
#undef PPLX_LAUNCH_LARGE_ROW_VARIANT
#undef PPLX_ROW_KERNEL_ARGS
  return (int)hipGetLastError();
}

template <class DT>
int launch_dispatch_t(const WorldDev &w, const DT &tab, hipStream_t s) {
  if (dispatch_is_fused(w)) return launch_fused_t(w, tab, s);
  RouteSpan span{};
  span.v_begin = 0;
  span.v_count = w.G * w.M;
  span.tile_cnt = w.tile_cnt;
  span.slot_out = w.slot_map;
  int err = launch_route_t<DT, false>(w, tab, span, s);
  if (err) return err;
  return launch_scatter_t(w, tab, s);
}

}  // namespace

// ---------------------------------------------------------------------------
// Launchers
// ---------------------------------------------------------------------------
uint32_t route_lds_bytes(uint32_t num_experts, uint32_t tile_chunks) {
  const uint32_t tables = tile_chunks * num_experts * (uint32_t)(sizeof(unsigned long long) + sizeof(uint32_t));
  const uint32_t scan = tile_chunks * kWave * (uint32_t)sizeof(uint32_t);  // split mode's block scan
  return tables > scan ? tables : scan;
}

bool dispatch_is_fused(const WorldDev &w) {
  // Every workgroup recounts all earlier picks, so the one-launch form only pays
  // while the whole step's routing is a few tens of KiB.
  const uint64_t pairs = (uint64_t)w.G * w.M * w.K;
  const uint32_t per_lane = (w.Hb / 16 + kWave - 1) / kWave;
  const bool exact = (w.Hb / 16) % kWave == 0;
  const bool row_fits = per_lane <= 8 || (exact && (per_lane == 14 || per_lane == 16));
  return pairs <= kFusedMaxPairs && row_fits && 16 * w.K * 24 + (w.E + w.G) * 4 <= 48 * 1024;
}

int launch_bind_dispatch(const WorldDev &w, const BindDispatchBatch &b, void *stream) {
  hipLaunchKernelGGL((bind_rows<BindDispatchBatch, DispatchRank>), dim3(1), dim3(256), 0,
                     (hipStream_t)stream, w.drank, b);
  return (int)hipGetLastError();
}

int launch_bind_combine(const WorldDev &w, const BindCombineBatch &b, void *stream) {
  hipLaunchKernelGGL((bind_rows<BindCombineBatch, CombineRank>), dim3(1), dim3(256), 0,
                     (hipStream_t)stream, w.crank, b);
  return (int)hipGetLastError();
}

int launch_dispatch(const WorldDev &w, const DispatchRank *inline_rows, void *stream) {
  if (inline_rows) return launch_dispatch_t(w, make_inline(w, inline_rows), (hipStream_t)stream);
  return launch_dispatch_t(w, HbmDispatch{w.drank}, (hipStream_t)stream);
}

}  // namespace pplx_amd
