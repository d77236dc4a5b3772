// Routing kernels: per-expert counts and the slot of every (token, pick) pair.
#pragma once
#include "a2a_common.h"

namespace pplx_amd {
namespace {

// ---------------------------------------------------------------------------
// Routing.  Virtual token v = g * M + t enumerates (DP group asc, token asc),
// the order in which the reference test appends to expert_token_from
// (tests/test_all_to_all.py:113-120).  A chunk is 64 consecutive virtual tokens
// (one wavefront, one token per lane), a tile is span.tile_chunks chunks (one
// workgroup).  Per chunk and expert a 64-bit mask in LDS holds one bit per token
// routed to the expert (ds_or_b64); a token's row inside the expert is
//     rows of earlier tiles + rows of earlier chunks of the tile + popc(mask & lanes below).
// Three launches when a span has more than one tile, one otherwise:
//   route_count   per tile: rows per expert                      -> tile_cnt[tile][e]
//   route_scan    per expert: exclusive prefix over the tiles    -> tile_cnt[tile][e], totals
//   route_slots   per tile: the masks again, slots               -> slot map
// An expert id repeated inside one token sets its bit once: the repeat takes no row, is not
// counted, and is reported (kFaultDuplicateExpert).
// With span.tile_mask set, route_count also keeps the masks and reports the faults, and there
// is no route_slots launch: the scatter that follows works each token's slots out of the
// scanned counts and the masks by itself (slots_from_masks).
// ---------------------------------------------------------------------------

// The token of this thread: which group and sender, whether its row of picks exists, and the
// loads that decide whether it is live (issued together with the picks by the callers).
struct RouteToken {
  uint32_t v, g, t;
  bool in_span;
  bool row_exists;                 // t < m of the sender: its picks may be read
  uint32_t n_group;                // tokens present in the group
  const PPLX_GLOBAL uint32_t *idx; // its K picks
};

template <class DT>
__device__ __forceinline__ RouteToken route_token(const WorldDev &w, const DT &tab, const RouteSpan &span) {
  RouteToken r;
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  r.v = span.v_begin + i;
  r.g = group_of(w, r.v);
  r.t = r.v - r.g * w.M;
  r.in_span = i < span.v_count && r.g < w.G;
  const DispatchRank &src = tab.at(r.in_span ? sender_of(w, r.g, r.t) : 0);
  r.row_exists = r.in_span && r.t < src.m;
  r.n_group = r.in_span ? dispatch_group_tokens(w, tab, r.g) : 0;
  r.idx = as_global(src.indices) + (size_t)r.t * w.K;
  return r;
}

template <class DT, int PV>
__global__ __launch_bounds__(1024) void route_count(WorldDev w, DT tab, RouteSpan span) {
  extern __shared__ unsigned long long lds_mask[];
  const uint32_t chunks = span.tile_chunks;
  for (uint32_t i = threadIdx.x; i < chunks * w.E; i += blockDim.x) lds_mask[i] = 0ull;
  __syncthreads();

  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t chunk = threadIdx.x / kWave;
  const RouteToken tok = route_token(w, tab, span);
  // (the picks are fetched whenever their row exists, behind the group's token count and not
  // after it: one trip to memory instead of two)
  uint32_t codes = 0;
  if (tok.row_exists) {
    const bool live = tok.t < tok.n_group;
    codes = for_each_pick<PV>(tok.idx, w.K, [&](uint32_t, uint32_t e) __attribute__((always_inline)) {
      if (!live) return 0u;
      if (e >= w.E) return kFaultBadExpert;
      const unsigned long long bit = 1ull << lane;
      return (atomicOr(&lds_mask[(size_t)chunk * w.E + e], bit) & bit) ? kFaultDuplicateExpert : 0u;
    }).codes;
  }
  __syncthreads();
  uint32_t *out = span.tile_cnt + (size_t)blockIdx.x * w.E;
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) {
    uint32_t rows = 0;
    for (uint32_t c = 0; c < chunks; ++c) rows += __popcll(lds_mask[(size_t)c * w.E + e]);
    out[e] = rows;
  }
  if (span.tile_mask != nullptr) {
    unsigned long long *keep = span.tile_mask + (size_t)blockIdx.x * chunks * w.E;
    for (uint32_t i = threadIdx.x; i < chunks * w.E; i += blockDim.x) keep[i] = lds_mask[i];
    if (codes) atomicOr(w.faults, codes);
    if (tok.in_span && tok.t == 0 && dispatch_group_overflows(w, tab, tok.g)) {
      atomicOr(w.faults, kFaultTooManyTokens);
    }
  }
}

// What route_slots would have written for pick `lane` of virtual token v (wave-uniform), from
// the scanned counts and the masks that route_count kept: rows of earlier tiles + rows of
// earlier chunks of the tile + earlier tokens of the chunk.  A pick that repeats an earlier
// one of its token, or names no expert, has no row.
__device__ __forceinline__ uint32_t slots_from_masks(const WorldDev &w, uint32_t v, uint32_t lane, uint32_t e) {
  const uint32_t chunks = w.tile_chunks;
  const uint32_t chunk_abs = v / kWave;
  const uint32_t tile = chunk_abs >> __builtin_ctz(chunks);  // (a tile is a power of two of chunks)
  const uint32_t c = chunk_abs - tile * chunks;
  const unsigned long long below = (1ull << (v & (kWave - 1))) - 1ull;
  bool has_row = lane < w.K && e < w.E;
  for (uint32_t k = 0; k + 1 < w.K; ++k) {
    const uint32_t earlier = (uint32_t)__builtin_amdgcn_readlane((int)e, (int)k);
    if (lane > k && earlier == e) has_row = false;
  }
  if (!has_row) return kInvalidSlot;
  const PPLX_GLOBAL unsigned long long *mask =
      as_global(reinterpret_cast<const unsigned long long *>(
          reinterpret_cast<const uint8_t *>(w.tile_cnt) + route_tables(w.num_tiles, chunks, w.E).mask_offset)) +
      (size_t)tile * chunks * w.E + e;
  uint32_t slot = as_global(w.tile_cnt)[(size_t)tile * w.E + e];
  // four masks per trip (tiles of four chunks: one trip)
  for (uint32_t c0 = 0; c0 <= c; c0 += 4) {
    unsigned long long m[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) m[i] = mask[(size_t)(c0 + i <= c ? c0 + i : c) * w.E];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
      if (c0 + i < c) slot += __popcll(m[i]);
      if (c0 + i == c) slot += __popcll(m[i] & below);
    }
  }
  return slot;
}

// One wavefront per expert: tile_cnt[.][e] becomes its own exclusive prefix over the tiles, and
// the total goes to out_expert_num_tokens of the owning rank
// (csrc/all_to_all/intranode_dispatch.cu:221 accumulates the same total).  Up to 256 tiles are
// fetched per trip to memory.
template <class DT>
__global__ __launch_bounds__(256) void route_scan(WorldDev w, DT tab, RouteSpan span, uint32_t tiles) {
  const uint32_t lane = lane_id();
  const uint32_t e = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave);
  if (e >= w.E) return;
  constexpr uint32_t kBatch = 4;
  uint32_t carry = 0;
  for (uint32_t t0 = 0; t0 < tiles; t0 += kBatch * kWave) {
    uint32_t rows[kBatch];
#pragma unroll
    for (uint32_t b = 0; b < kBatch; ++b) {
      const uint32_t t = t0 + b * kWave + lane;
      rows[b] = t < tiles ? span.tile_cnt[(size_t)t * w.E + e] : 0u;
    }
#pragma unroll
    for (uint32_t b = 0; b < kBatch; ++b) {
      const uint32_t t = t0 + b * kWave + lane;
      uint32_t incl = rows[b];
#pragma unroll
      for (uint32_t d = 1; d < kWave; d *= 2) {
        const uint32_t up = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += up;
      }
      if (t < tiles) span.tile_cnt[(size_t)t * w.E + e] = carry + incl - rows[b];
      carry += __shfl(incl, kWave - 1, kWave);
    }
  }
  if (lane == 0) {
    const DispatchRank &owner = tab.at(owner_of(w, e));
    as_global(owner.out_num_tokens)[(int64_t)local_of(w, e) * owner.out_num_tokens_stride] = (int32_t)carry;
  }
}

// `scanned`: tile_cnt holds the rows of earlier tiles (route_scan has run); otherwise the span
// is a single tile and this launch also writes the totals.
template <class DT, int PV>
__global__ __launch_bounds__(1024) void route_slots(WorldDev w, DT tab, RouteSpan span, uint32_t scanned) {
  // LDS: mask[chunks][E] (one bit per token of the chunk routed to e),
  //      then base[chunks][E] (rows of e taken before the chunk starts).
  extern __shared__ unsigned long long lds_mask[];
  const uint32_t chunks = span.tile_chunks;
  uint32_t *lds_base = reinterpret_cast<uint32_t *>(lds_mask + (size_t)chunks * w.E);

  for (uint32_t i = threadIdx.x; i < chunks * w.E; i += blockDim.x) lds_mask[i] = 0ull;
  {
    const uint32_t *earlier = span.tile_cnt + (size_t)blockIdx.x * w.E;
    for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) lds_base[e] = scanned ? earlier[e] : 0u;
  }
  __syncthreads();

  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t chunk = threadIdx.x / kWave;
  const RouteToken tok = route_token(w, tab, span);
  const bool live = tok.row_exists && tok.t < tok.n_group;
  // Marked picks have no row: an expert id out of range, or a repeat of an earlier pick.
  PickMarks no_row{0ull, 0u};
  if (tok.row_exists) {
    no_row = for_each_pick<PV>(tok.idx, w.K, [&](uint32_t, uint32_t e) __attribute__((always_inline)) {
      if (!live) return 0u;
      if (e >= w.E) return kFaultBadExpert;
      const unsigned long long bit = 1ull << lane;
      return (atomicOr(&lds_mask[(size_t)chunk * w.E + e], bit) & bit) ? kFaultDuplicateExpert : 0u;
    });
  }
  __syncthreads();

  // Per expert: running prefix over chunks, starting from the rows of earlier tiles.
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) {
    uint32_t running = lds_base[e];
    for (uint32_t c = 0; c < chunks; ++c) {
      lds_base[c * w.E + e] = running;
      running += __popcll(lds_mask[(size_t)c * w.E + e]);
    }
    if (!scanned) {
      const DispatchRank &owner = tab.at(owner_of(w, e));
      as_global(owner.out_num_tokens)[(int64_t)local_of(w, e) * owner.out_num_tokens_stride] = (int32_t)running;
    }
  }
  __syncthreads();

  if (live) {
    const unsigned long long below = (1ull << lane) - 1ull;
    uint32_t *out = span.slot_out + (size_t)tok.v * w.K;
    for_each_pick<PV>(tok.idx, w.K, [&](uint32_t k, uint32_t e) __attribute__((always_inline)) {
      uint32_t slot = kInvalidSlot;
      if (!((no_row.marked >> k) & 1ull)) {
        slot = lds_base[chunk * w.E + e] + __popcll(lds_mask[(size_t)chunk * w.E + e] & below);
      }
      out[k] = slot;
      return 0u;
    });
    if (no_row.codes) atomicOr(w.faults, no_row.codes);
  }
  if (tok.in_span && tok.t == 0 && dispatch_group_overflows(w, tab, tok.g)) {
    atomicOr(w.faults, kFaultTooManyTokens);
  }
}

template <class DT, int PV>
int launch_route_pv(const WorldDev &w, const DT &tab, const RouteSpan &span, hipStream_t s) {
  const uint32_t block = span.tile_chunks * kWave;
  const uint32_t tiles = (span.v_count + block - 1) / block;
  const uint32_t lds = route_lds_bytes(w.E, span.tile_chunks);
  if (tiles > 1) {
    hipLaunchKernelGGL((route_count<DT, PV>), dim3(tiles), dim3(block),
                       span.tile_chunks * w.E * sizeof(unsigned long long), s, w, tab, span);
    hipLaunchKernelGGL((route_scan<DT>), dim3((w.E + 3) / 4), dim3(256), 0, s, w, tab, span, tiles);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return (int)err;
    if (span.tile_mask != nullptr) return 0;  // the scatter works the slots out
  }
  hipLaunchKernelGGL((route_slots<DT, PV>), dim3(tiles), dim3(block), lds, s, w, tab, span,
                     tiles > 1 ? 1u : 0u);
  return (int)hipGetLastError();
}

template <class DT>
int launch_route_t(const WorldDev &w, const DT &tab, const RouteSpan &span, hipStream_t s) {
  if (span.pick_vector == 4) return launch_route_pv<DT, 4>(w, tab, span, s);
  if (span.pick_vector == 2) return launch_route_pv<DT, 2>(w, tab, span, s);
  return launch_route_pv<DT, 1>(w, tab, span, s);
}

}  // namespace
}  // namespace pplx_amd
