// Routing kernels: per-expert counts and the slot of every (token, pick) pair.
#pragma once
#include "a2a_common.h"

namespace pplx_amd {
namespace {

// ---------------------------------------------------------------------------
// Routing.  Virtual token v = g * M + t enumerates (DP group asc, token asc),
// the order in which the reference test appends to expert_token_from.  A tile
// is tile_chunks consecutive chunks of 64 virtual tokens.
// ---------------------------------------------------------------------------
// SPLIT = false: one launch routes every DP group and writes out_expert_num_tokens of the
// owning ranks.  SPLIT = true: the launch routes the span of one DP group from the calling
// rank's indices alone and leaves group-local results (slot inside (group, expert), expert of
// each pair, rows per expert and their exclusive prefix over experts) for the later phases.
template <class DT>
__global__ __launch_bounds__(1024) void route_count(WorldDev w, DT tab, RouteSpan span) {
  extern __shared__ uint32_t lds_hist[];
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) lds_hist[e] = 0;
  __syncthreads();

  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t v = span.v_begin + i;
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  if (i < span.v_count && g < w.G && t < dispatch_group_tokens(w, tab, g)) {
    const PPLX_GLOBAL uint32_t *idx = as_global(tab.at(g * w.dp + t % w.dp).indices) + (size_t)t * w.K;
    for (uint32_t k = 0; k < w.K; ++k) {
      const uint32_t e = idx[k];
      if (e < w.E) atomicAdd(&lds_hist[e], 1u);
    }
  }
  __syncthreads();
  uint32_t *out = span.tile_cnt + (size_t)blockIdx.x * w.E;
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) out[e] = lds_hist[e];
}

template <class DT, bool SPLIT>
__global__ __launch_bounds__(1024) void route_slots(WorldDev w, DT tab, RouteSpan span) {
  // LDS: mask[chunks][E] (one bit per token of the chunk routed to e),
  //      then base[chunks][E] (rows of e taken before the chunk starts).
  extern __shared__ unsigned long long lds_mask[];
  const uint32_t chunks = w.tile_chunks;
  uint32_t *lds_base = reinterpret_cast<uint32_t *>(lds_mask + (size_t)chunks * w.E);

  for (uint32_t i = threadIdx.x; i < chunks * w.E; i += blockDim.x) lds_mask[i] = 0ull;
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) lds_base[e] = 0;
  __syncthreads();

  // Rows taken by earlier tiles, summed per expert into lds_base[0][e] by the whole workgroup:
  // the counts are fetched kTileLoads at a time so that their latencies overlap each other and
  // the index loads below (one thread per expert walking the tiles would pay one L2 round trip
  // per tile).
  {
    constexpr uint32_t kTileLoads = 8;
    const uint32_t total = blockIdx.x * w.E;
    for (uint32_t first = threadIdx.x; first < total; first += blockDim.x * kTileLoads) {
      uint32_t rows[kTileLoads];
#pragma unroll
      for (uint32_t u = 0; u < kTileLoads; ++u) {
        const uint32_t j = first + u * blockDim.x;
        rows[u] = j < total ? span.tile_cnt[j] : 0u;
      }
#pragma unroll
      for (uint32_t u = 0; u < kTileLoads; ++u) {
        if (rows[u]) atomicAdd(&lds_base[(first + u * blockDim.x) % w.E], rows[u]);
      }
    }
  }

  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t chunk = threadIdx.x / kWave;
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t v = span.v_begin + i;
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  const bool in_span = i < span.v_count && g < w.G;
  const uint32_t n_group = in_span ? dispatch_group_tokens(w, tab, g) : 0;
  const bool live = in_span && t < n_group;
  const PPLX_GLOBAL uint32_t *idx = nullptr;
  bool bad_expert = false;
  if (live) {
    idx = as_global(tab.at(g * w.dp + t % w.dp).indices) + (size_t)t * w.K;
    for (uint32_t k = 0; k < w.K; ++k) {
      const uint32_t e = idx[k];
      if (e < w.E) {
        atomicOr(&lds_mask[(size_t)chunk * w.E + e], 1ull << lane);
      } else {
        bad_expert = true;
      }
    }
  }
  __syncthreads();

  // Per expert: running prefix over chunks, starting from the rows of earlier tiles.
  const bool last_tile = blockIdx.x == gridDim.x - 1;
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) {
    uint32_t running = lds_base[e];
    for (uint32_t c = 0; c < chunks; ++c) {
      lds_base[c * w.E + e] = running;
      running += __popcll(lds_mask[(size_t)c * w.E + e]);
    }
    if (last_tile) {
      if (SPLIT) {
        span.counts_out[e] = running;
      } else {
        // out_expert_num_tokens of the owning rank
        // (csrc/all_to_all/intranode_dispatch.cu:221 accumulates the same total).
        const DispatchRank &owner = tab.at(e / w.L);
        as_global(owner.out_num_tokens)[(int64_t)(e % w.L) * owner.out_num_tokens_stride] = (int32_t)running;
      }
    }
  }
  __syncthreads();

  if (live) {
    const unsigned long long below = (1ull << lane) - 1ull;
    uint32_t *out = span.slot_out + (size_t)v * w.K;
    for (uint32_t k = 0; k < w.K; ++k) {
      const uint32_t e = idx[k];
      uint32_t slot = kInvalidSlot;
      if (e < w.E) {
        slot = lds_base[chunk * w.E + e] + __popcll(lds_mask[(size_t)chunk * w.E + e] & below);
      }
      out[k] = slot;
      if (SPLIT) span.expert_out[(size_t)v * w.K + k] = e;
    }
    if (bad_expert) atomicOr(w.faults, kFaultBadExpert);
  }

  if (SPLIT && last_tile) {
    // Exclusive prefix of counts_out over experts: where each expert's rows start in the
    // group's compact staging area.  counts_out was written by this workgroup above.
    __syncthreads();
    uint32_t *scan = reinterpret_cast<uint32_t *>(lds_mask);  // blockDim entries, LDS is free now
    const uint32_t per_thread = (w.E + blockDim.x - 1) / blockDim.x;
    const uint32_t e0 = threadIdx.x * per_thread;
    uint32_t local = 0;
    for (uint32_t e = e0; e < e0 + per_thread && e < w.E; ++e) local += span.counts_out[e];
    scan[threadIdx.x] = local;
    __syncthreads();
    for (uint32_t step = 1; step < blockDim.x; step *= 2) {
      const uint32_t add = threadIdx.x >= step ? scan[threadIdx.x - step] : 0;
      __syncthreads();
      scan[threadIdx.x] += add;
      __syncthreads();
    }
    uint32_t running = scan[threadIdx.x] - local;
    for (uint32_t e = e0; e < e0 + per_thread && e < w.E; ++e) {
      span.offsets_out[e] = running;
      running += span.counts_out[e];
    }
    if (threadIdx.x == 0) *span.ntok_out = dispatch_group_tokens(w, tab, span.v_begin / w.M);
  }
}

template <class DT, bool SPLIT>
int launch_route_t(const WorldDev &w, const DT &tab, const RouteSpan &span, hipStream_t s) {
  const uint32_t block = w.tile_chunks * kWave;
  const uint32_t tiles = (span.v_count + block - 1) / block;
  if (tiles > 1) {
    hipLaunchKernelGGL(route_count<DT>, dim3(tiles), dim3(block), w.E * sizeof(uint32_t), s, w, tab, span);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return (int)err;
  }
  hipLaunchKernelGGL((route_slots<DT, SPLIT>), dim3(tiles), dim3(block),
                     route_lds_bytes(w.E, w.tile_chunks), s, w, tab, span);
  return (int)hipGetLastError();
}

}  // namespace
}  // namespace pplx_amd
