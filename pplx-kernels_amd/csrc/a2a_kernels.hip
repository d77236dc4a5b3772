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
#include <hip/hip_runtime.h>

#include "a2a_device.h"

namespace pplx_amd {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

struct InlineDispatch {
  DispatchRank rows[kInlineRanks];
  __device__ __forceinline__ const DispatchRank &at(uint32_t i) const { return rows[i]; }
};
struct HbmDispatch {
  const DispatchRank *rows;
  __device__ __forceinline__ const DispatchRank &at(uint32_t i) const { return rows[i]; }
};
struct InlineCombine {
  static constexpr bool kStaged = false;
  CombineRank rows[kInlineRanks];
  __device__ __forceinline__ const CombineRank &at(uint32_t i) const { return rows[i]; }
};
struct HbmCombine {
  static constexpr bool kStaged = false;
  const CombineRank *rows;
  __device__ __forceinline__ const CombineRank &at(uint32_t i) const { return rows[i]; }
};

// Pointers rebuilt from integers would be "flat" to the compiler; these casts say
// that they are global memory, so that plain global_load / global_store are emitted.
#define PPLX_GLOBAL __attribute__((address_space(1)))
template <typename V>
__device__ __forceinline__ PPLX_GLOBAL V *global_ptr(uint64_t address) {
  return (PPLX_GLOBAL V *)address;
}
template <typename V>
__device__ __forceinline__ const PPLX_GLOBAL V *global_cptr(uint64_t address) {
  return (const PPLX_GLOBAL V *)address;
}

// Makes the compiler treat `v` as consumed here, so that it waits for the loads
// feeding it at this point and not inside a later loop, where such a wait would
// also drain the stores of the previous iteration.
template <typename V>
__device__ __forceinline__ void settle(V &v) {
  asm volatile("" : "+v"(v));
}

// settle() for N registers at once: every load feeding them has to be issued
// before this point, so the N loads go out back to back behind one wait.
template <int N> struct SettleAll;
template <> struct SettleAll<1> {
  template <typename V> static __device__ __forceinline__ void of(V *r) { asm volatile("" : "+v"(r[0])); }
};
template <> struct SettleAll<2> {
  template <typename V> static __device__ __forceinline__ void of(V *r) {
    asm volatile("" : "+v"(r[0]), "+v"(r[1]));
  }
};
template <> struct SettleAll<4> {
  template <typename V> static __device__ __forceinline__ void of(V *r) {
    asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]));
  }
};
template <> struct SettleAll<8> {
  template <typename V> static __device__ __forceinline__ void of(V *r) {
    asm volatile(""
                 : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]),
                   "+v"(r[7]));
  }
};
template <> struct SettleAll<16> {
  template <typename V> static __device__ __forceinline__ void of(V *r) {
    asm volatile(""
                 : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]),
                   "+v"(r[7]), "+v"(r[8]), "+v"(r[9]), "+v"(r[10]), "+v"(r[11]), "+v"(r[12]),
                   "+v"(r[13]), "+v"(r[14]), "+v"(r[15]));
  }
};

// Split mode: a launch sees only the calling rank's arguments (its peers may not
// have called yet), whatever rank index is asked for.
struct SingleDispatch {
  DispatchRank row;
  __device__ __forceinline__ const DispatchRank &at(uint32_t) const { return row; }
};
struct SingleCombine {
  static constexpr bool kStaged = true;  // rows come from the world's stage_y, not expert_y
  CombineRank row;
  __device__ __forceinline__ const CombineRank &at(uint32_t) const { return row; }
};

__device__ __forceinline__ uint32_t lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

__device__ __forceinline__ uint64_t read_lane64(uint64_t v, uint32_t src_lane) {
  return ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), (int)src_lane) << 32) |
         (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, (int)src_lane);
}

// Tokens present in DP group g this step: the reference's numSendTokens
// (csrc/all_to_all/intranode_dispatch.cu:64), clamped to the rows that exist.
template <class DT>
__device__ __forceinline__ uint32_t dispatch_group_tokens(const WorldDev &w, const DT &tab, uint32_t g) {
  const DispatchRank &r = tab.at(g * w.dp);
  uint32_t n = r.bound_m ? *r.bound_m : r.m;
  n = n < r.m ? n : r.m;
  return n < w.M ? n : w.M;
}

__device__ __forceinline__ uint32_t combine_rank_tokens(const WorldDev &w, const CombineRank &c) {
  uint32_t n = c.bound_m ? *c.bound_m : c.m;
  n = n < c.m ? n : c.m;
  return n < w.M ? n : w.M;
}

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
    const uint32_t *idx = tab.at(g * w.dp + t % w.dp).indices + (size_t)t * w.K;
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
  __syncthreads();

  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t chunk = threadIdx.x / kWave;
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t v = span.v_begin + i;
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  const bool in_span = i < span.v_count && g < w.G;
  const uint32_t n_group = in_span ? dispatch_group_tokens(w, tab, g) : 0;
  const bool live = in_span && t < n_group;
  const uint32_t *idx = nullptr;
  bool bad_expert = false;
  if (live) {
    idx = tab.at(g * w.dp + t % w.dp).indices + (size_t)t * w.K;
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

  // Per expert: rows taken by earlier tiles, then running prefix over chunks.
  const bool last_tile = blockIdx.x == gridDim.x - 1;
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) {
    uint32_t running = 0;
    for (uint32_t tile = 0; tile < blockIdx.x; ++tile) running += span.tile_cnt[(size_t)tile * w.E + e];
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
        owner.out_num_tokens[(int64_t)(e % w.L) * owner.out_num_tokens_stride] = (int32_t)running;
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

// ---------------------------------------------------------------------------
// Row fan-out shared by dispatch_scatter and dispatch_fused.  The calling wave
// owns one token; the row is read once into NV 16-byte registers per lane
// (load_row) and stored for picks [k0, k1) (store_row), lane k passing the slot of
// pick k.  EXACT: the row is exactly NV * 64 vectors, so nothing is predicated.
// ---------------------------------------------------------------------------
template <int NV>
struct RowRegs {
  u32x4 x[NV];   // the row, 16 bytes per lane per register
  float sc;      // scale `lane` of the row (lanes >= S hold a copy of the last one)
};

// First half: issues the loads of row t of `src`; needs t < src.m only.
template <int NV, bool EXACT>
__device__ __forceinline__ void load_row(const WorldDev &w, const DispatchRank &src, uint32_t t,
                                         uint32_t lane, RowRegs<NV> &regs) {
  const uint32_t nvec = w.Hb / 16;
  const u32x4 *row = reinterpret_cast<const u32x4 *>(src.dp_x + (int64_t)t * src.dp_x_stride_row);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    uint32_t j = lane + i * kWave;
    if (!EXACT) j = j < nvec ? j : nvec - 1;  // clamp: loads stay unconditional
    regs.x[i] = row[j];
  }
  regs.sc = 0.f;
  if (w.S) {
    const uint32_t j = lane < w.S ? lane : w.S - 1;
    regs.sc = src.dp_xs[(int64_t)t * src.dp_xs_stride_row + (int64_t)j * src.dp_xs_stride_elem];
  }
}

// Where pick (expert e, row `slot`) of a token lands: row address, scale-row address and the
// element stride of the scale row; all zero when the pick has no destination.
struct Destination {
  uint64_t row = 0, scale = 0;
  int64_t scale_step = 0;
};

template <class DT>
__device__ __forceinline__ Destination resolve_destination(const WorldDev &w, const DT &tab, uint32_t e,
                                                           uint32_t slot, bool report) {
  Destination d;
  if (e < w.E && slot != kInvalidSlot) {
    const DispatchRank &dst = tab.at(e / w.L);
    const uint32_t el = e % w.L;
    if (slot < dst.x_rows) {
      d.row = reinterpret_cast<uint64_t>(dst.expert_x + (int64_t)el * dst.x_stride_expert +
                                         (int64_t)slot * dst.x_stride_row);
      if (w.S) {
        d.scale = reinterpret_cast<uint64_t>(dst.expert_xs + (int64_t)el * dst.xs_stride_expert +
                                             (int64_t)slot * dst.xs_stride_row);
        d.scale_step = dst.xs_stride_elem;
      }
    } else if (report) {
      atomicOr(w.faults, kFaultRowDropped);
    }
  }
  return d;
}

// Second half: lane k holds the destination of pick k; the row is stored for picks [k0, k1).
template <int NV, bool EXACT>
__device__ __forceinline__ void store_row(const WorldDev &w, const DispatchRank &src, uint32_t t,
                                          uint32_t lane, Destination dst, uint32_t k0, uint32_t k1,
                                          RowRegs<NV> &regs) {
  const uint32_t nvec = w.Hb / 16;
  const uint32_t S = w.S;
#pragma unroll
  for (int i = 0; i < NV; ++i) settle(regs.x[i]);
  settle(regs.sc);
  settle(dst.row);
  settle(dst.scale);
  settle(dst.scale_step);

  for (uint32_t k = k0; k < k1; ++k) {
    const uint64_t p = read_lane64(dst.row, k);
    if (p == 0) continue;
    PPLX_GLOBAL u32x4 *out = global_ptr<u32x4>(p);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const uint32_t j = lane + i * kWave;
      if (EXACT || j < nvec) __builtin_nontemporal_store(regs.x[i], out + j);
    }
    if (S) {
      PPLX_GLOBAL float *sout = global_ptr<float>(read_lane64(dst.scale, k));
      const int64_t step = (int64_t)read_lane64((uint64_t)dst.scale_step, k);
      if (lane < S) __builtin_nontemporal_store(regs.sc, sout + (int64_t)lane * step);
      if (S > kWave) {
        const float *srow = src.dp_xs + (int64_t)t * src.dp_xs_stride_row;
        for (uint32_t j = lane + kWave; j < S; j += kWave) {
          sout[(int64_t)j * step] = srow[(int64_t)j * src.dp_xs_stride_elem];
        }
      }
    }
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

// ---------------------------------------------------------------------------
// Combine: out[t, :] = (U) sum_k w[t, k] * (float) expert_y[e_k][slot(t, k), :]
// with k ascending and fp32 accumulation
// (csrc/all_to_all/intranode_combine.cu:141-168).
// ---------------------------------------------------------------------------
template <typename T> struct Row8;
template <> struct Row8<float> {
  struct Raw {
    f32x4 a, b;
  };
  static __device__ __forceinline__ Raw load(uint64_t row, uint32_t vec) {
    const PPLX_GLOBAL f32x4 *p = global_cptr<f32x4>(row) + 2 * (size_t)vec;
    return Raw{__builtin_nontemporal_load(p), __builtin_nontemporal_load(p + 1)};
  }
  static __device__ __forceinline__ f32x8 widen(const Raw &r) {
    return __builtin_shufflevector(r.a, r.b, 0, 1, 2, 3, 4, 5, 6, 7);
  }
  // N rows held as 2 N registers of 16 bytes
  template <int N> static __device__ __forceinline__ void settle(Raw *raw) {
    SettleAll<2 * N>::of(reinterpret_cast<f32x4 *>(raw));
  }
};
template <> struct Row8<__bf16> {
  typedef u32x4 Raw;
  static __device__ __forceinline__ Raw load(uint64_t row, uint32_t vec) {
    return __builtin_nontemporal_load(global_cptr<u32x4>(row) + vec);
  }
  static __device__ __forceinline__ f32x8 widen(const Raw &raw) {
    f32x8 out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[2 * i] = __uint_as_float(raw[i] << 16);
      out[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
    }
    return out;
  }
  template <int N> static __device__ __forceinline__ void settle(Raw *raw) { SettleAll<N>::of(raw); }
};
template <> struct Row8<_Float16> {
  typedef f16x8 Raw;
  static __device__ __forceinline__ Raw load(uint64_t row, uint32_t vec) {
    return __builtin_nontemporal_load(global_cptr<f16x8>(row) + vec);
  }
  static __device__ __forceinline__ f32x8 widen(const Raw &raw) {
    return __builtin_convertvector(raw, f32x8);
  }
  template <int N> static __device__ __forceinline__ void settle(Raw *raw) { SettleAll<N>::of(raw); }
};

template <typename U> struct Store8;
template <> struct Store8<__bf16> {
  static __device__ __forceinline__ void at(void *row, uint32_t vec, const f32x8 &acc) {
    __builtin_nontemporal_store(__builtin_convertvector(acc, bf16x8), reinterpret_cast<bf16x8 *>(row) + vec);
  }
};
template <> struct Store8<_Float16> {
  static __device__ __forceinline__ void at(void *row, uint32_t vec, const f32x8 &acc) {
    __builtin_nontemporal_store(__builtin_convertvector(acc, f16x8), reinterpret_cast<f16x8 *>(row) + vec);
  }
};

// N picks starting at k: all N loads are issued before the first is used.
template <typename T, int N>
__device__ __forceinline__ void gather_group(f32x8 &acc, uint64_t row_of_lane, float weight_of_lane,
                                             uint32_t k, uint32_t vec) {
  typename Row8<T>::Raw raw[N];
#pragma unroll
  for (int i = 0; i < N; ++i) raw[i] = Row8<T>::load(read_lane64(row_of_lane, k + i), vec);
  Row8<T>::template settle<N>(raw);
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float wk = __builtin_bit_cast(
        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, weight_of_lane), (int)(k + i)));
    acc += wk * Row8<T>::widen(raw[i]);
  }
}

// One wave owns VPL * 64 consecutive 8-element vectors of one output row.  With
// KK == 0 (any K) it is one vector per lane and the picks go in groups of up to
// eight loads; with KK in {1, 2, 4} the wave takes VPL = 8 / KK vectors per lane so
// that eight row loads per lane are in flight for small top-k too.
template <typename T, typename U, class CT, int KK, int VPL>
__global__ __launch_bounds__(256) void combine_gather(WorldDev w, CT tab, uint32_t segments,
                                                      uint32_t first_rank, uint32_t rank_count,
                                                      const uint8_t *stage_y, uint64_t stage_row_bytes) {
  const uint32_t lane = lane_id();
  const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) +
                                                       threadIdx.x / kWave);
  const uint32_t token = wave / segments;
  const uint32_t segment = wave - token * segments;
  const uint32_t r_local = token / w.M;
  const uint32_t t = token - r_local * w.M;
  if (r_local >= rank_count) return;
  const uint32_t r = first_rank + r_local;
  const CombineRank &c = tab.at(r);
  if (t >= combine_rank_tokens(w, c)) return;

  // Lane k resolves pick k: no LDS, no barrier.
  uint64_t row = 0;
  float weight = 0.f;
  if (lane < w.K) {
    const uint32_t e = c.indices[(size_t)t * w.K + lane];
    const uint32_t slot = w.slot_map[((size_t)(r / w.dp) * w.M + t) * w.K + lane];
    weight = c.weights[(int64_t)t * c.w_stride_row + lane];
    if (CT::kStaged) {
      // combine SEND left the row of (token, pick) in the staging area.
      if (e < w.E && slot != kInvalidSlot) {
        row = reinterpret_cast<uint64_t>(stage_y) +
              (((uint64_t)(r / w.dp) * w.M + t) * w.K + lane) * stage_row_bytes;
      }
    } else if (e < w.E && slot != kInvalidSlot) {
      const CombineRank &owner = tab.at(e / w.L);
      if (slot < owner.y_rows) {
        row = reinterpret_cast<uint64_t>(reinterpret_cast<const T *>(owner.expert_y) +
                                         (int64_t)(e % w.L) * owner.y_stride_expert +
                                         (int64_t)slot * owner.y_stride_row);
      } else if (segment == 0) {
        atomicOr(w.faults, kFaultBadSlot);
      }
    }
  }
  const bool all_rows = __builtin_amdgcn_ballot_w64(lane < w.K && row == 0) == 0;

  U *out = reinterpret_cast<U *>(c.out_tokens) + (int64_t)t * c.out_stride_row;
  const uint32_t nvec = w.H / 8;
  const uint32_t K = w.K;
  if (!all_rows) {
    // A pick without a row (bad expert id or slot) contributes nothing.
    for (int v = 0; v < VPL; ++v) {
      const uint32_t vec = (segment * VPL + v) * kWave + lane;
      const uint32_t vec_ld = vec < nvec ? vec : nvec - 1;
      f32x8 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      for (uint32_t k = 0; k < K; ++k) {
        if (read_lane64(row, k) != 0) gather_group<T, 1>(acc, row, weight, k, vec_ld);
      }
      if (vec < nvec) Store8<U>::at(out, vec, acc);
    }
    return;
  }
  if (KK == 0) {
    const uint32_t vec = segment * kWave + lane;
    const uint32_t vec_ld = vec < nvec ? vec : nvec - 1;  // clamp: loads stay unconditional
    f32x8 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    uint32_t k = 0;
    for (; k + 8 <= K; k += 8) gather_group<T, 8>(acc, row, weight, k, vec_ld);
    if (K & 4) { gather_group<T, 4>(acc, row, weight, k, vec_ld); k += 4; }
    if (K & 2) { gather_group<T, 2>(acc, row, weight, k, vec_ld); k += 2; }
    if (K & 1) { gather_group<T, 1>(acc, row, weight, k, vec_ld); }
    if (vec < nvec) Store8<U>::at(out, vec, acc);
  } else {
    constexpr int N = KK == 0 ? 1 : KK;
    typename Row8<T>::Raw raw[VPL][N];
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      const uint32_t vec = (segment * VPL + v) * kWave + lane;
      const uint32_t vec_ld = vec < nvec ? vec : nvec - 1;
#pragma unroll
      for (int k = 0; k < N; ++k) raw[v][k] = Row8<T>::load(read_lane64(row, k), vec_ld);
    }
    Row8<T>::template settle<VPL * N>(&raw[0][0]);
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      const uint32_t vec = (segment * VPL + v) * kWave + lane;
      f32x8 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k = 0; k < N; ++k) {
        const float wk = __builtin_bit_cast(
            float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, weight), k));
        acc += wk * Row8<T>::widen(raw[v][k]);
      }
      if (vec < nvec) Store8<U>::at(out, vec, acc);
    }
  }
}

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
  const u32x4 *row = reinterpret_cast<const u32x4 *>(src.dp_x + (int64_t)t * src.dp_x_stride_row);
  u32x4 x[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    uint32_t j = lane + i * kWave;
    if (!EXACT) j = j < nvec ? j : nvec - 1;
    x[i] = row[j];
  }
  const uint32_t S = w.S;
  const float *srow = S ? src.dp_xs + (int64_t)t * src.dp_xs_stride_row : nullptr;
  uint64_t dst = 0;
  if (lane < w.K) {
    const size_t pair = ((size_t)g * w.M + t) * w.K + lane;
    const uint32_t e = sp.gexp[pair];
    if (e < w.E) dst = reinterpret_cast<uint64_t>(stage_row(w, sp, g, sp.goff[(size_t)g * w.E + e] + sp.gslot[pair]));
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) settle(x[i]);
  settle(dst);
  for (uint32_t k = 0; k < w.K; ++k) {
    const uint64_t p = read_lane64(dst, k);
    if (p == 0) continue;
    PPLX_GLOBAL u32x4 *out = global_ptr<u32x4>(p);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const uint32_t j = lane + i * kWave;
      if (EXACT || j < nvec) out[j] = x[i];
    }
    PPLX_GLOBAL float *sout = global_ptr<float>(p + w.Hb);
    for (uint32_t j = lane; j < S; j += kWave) sout[j] = srow[(int64_t)j * src.dp_xs_stride_elem];
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
__global__ __launch_bounds__(256) void split_unpack(WorldDev w, DT tab, uint32_t d, SplitDev sp) {
  const uint32_t lane = lane_id();
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
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
  const uint32_t S = w.S;
  for (uint32_t i = blockIdx.y * (blockDim.x / kWave) + wave; i < count; i += gridDim.y * (blockDim.x / kWave)) {
    const uint32_t slot = base + i;
    if (slot >= dst.x_rows) {
      if (lane == 0) atomicOr(w.faults, kFaultRowDropped);
      continue;
    }
    const uint8_t *src = stage_row(w, sp, g, offset + i);
    const u32x4 *row = reinterpret_cast<const u32x4 *>(src);
    u32x4 *out = reinterpret_cast<u32x4 *>(dst.expert_x + (int64_t)el * dst.x_stride_expert +
                                           (int64_t)slot * dst.x_stride_row);
    u32x4 x[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      uint32_t j = lane + v * kWave;
      if (!EXACT) j = j < nvec ? j : nvec - 1;
      x[v] = row[j];
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const uint32_t j = lane + v * kWave;
      if (EXACT || j < nvec) __builtin_nontemporal_store(x[v], out + j);
    }
    if (S) {
      const float *sin = reinterpret_cast<const float *>(src + w.Hb);
      float *sout = dst.expert_xs + (int64_t)el * dst.xs_stride_expert + (int64_t)slot * dst.xs_stride_row;
      for (uint32_t j = lane; j < S; j += kWave) sout[(int64_t)j * dst.xs_stride_elem] = sin[j];
    }
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

// ---------------------------------------------------------------------------
// Launch helpers
// ---------------------------------------------------------------------------
InlineDispatch make_inline(const WorldDev &w, const DispatchRank *rows) {
  InlineDispatch t{};
  for (uint32_t i = 0; i < w.R && i < kInlineRanks; ++i) t.rows[i] = rows[i];
  return t;
}

InlineCombine make_inline(const WorldDev &w, const CombineRank *rows) {
  InlineCombine t{};
  for (uint32_t i = 0; i < w.R && i < kInlineRanks; ++i) t.rows[i] = rows[i];
  return t;
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

// Picks the register variant for the row size and launches KERNEL<NV, EXACT, DT>.
// Rows beyond 8 KiB exist only for dispatch_scatter (PPLX_LAUNCH_LARGE_ROW_VARIANT).
#define PPLX_LAUNCH_ROW_VARIANT(KERNEL, NV, EXACT)                                               \
  hipLaunchKernelGGL((KERNEL<NV, EXACT, DT>), grid, block, lds, s, w, tab, PPLX_ROW_KERNEL_ARGS)

#define PPLX_DISPATCH_ROW_VARIANTS(KERNEL)                                                       \
  do {                                                                                           \
    const uint32_t nvec = w.Hb / 16;                                                             \
    const uint32_t per_lane = (nvec + kWave - 1) / kWave;                                        \
    const bool exact = nvec % kWave == 0;                                                        \
    if (exact && per_lane == 1) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 1, true);                        \
    else if (exact && per_lane == 2) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 2, true);                   \
    else if (exact && per_lane == 3) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 3, true);                   \
    else if (exact && per_lane == 4) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 4, true);                   \
    else if (exact && per_lane == 5) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 5, true);                   \
    else if (exact && per_lane == 6) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 6, true);                   \
    else if (exact && per_lane == 7) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 7, true);                   \
    else if (exact && per_lane == 8) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 8, true);                   \
    else if (exact && per_lane == 14) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 14, true);                 \
    else if (exact && per_lane == 16) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 16, true);                 \
    else if (per_lane <= 1) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 1, false);                           \
    else if (per_lane <= 2) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 2, false);                           \
    else if (per_lane <= 4) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 4, false);                           \
    else if (per_lane <= 8) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 8, false);                           \
    else PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL);                                                  \
  } while (0)

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

template <typename T, typename U, class CT>
int launch_combine_k(const WorldDev &w, const CT &tab, uint32_t first_rank, uint32_t rank_count,
                     const uint8_t *stage_y, uint64_t stage_row_bytes, hipStream_t s) {
  const uint32_t nvec_segments = (w.H / 8 + kWave - 1) / kWave;
  const uint32_t vpl = w.K == 1 ? 8 : w.K == 2 ? 4 : w.K == 4 ? 2 : 1;
  const uint32_t segments = (nvec_segments + vpl - 1) / vpl;
  const uint64_t waves = (uint64_t)rank_count * w.M * segments;
  const dim3 grid((uint32_t)((waves + 3) / 4)), block(256);
  switch (w.K) {
    case 1: hipLaunchKernelGGL((combine_gather<T, U, CT, 1, 8>), grid, block, 0, s, w, tab, segments, first_rank, rank_count, stage_y, stage_row_bytes); break;
    case 2: hipLaunchKernelGGL((combine_gather<T, U, CT, 2, 4>), grid, block, 0, s, w, tab, segments, first_rank, rank_count, stage_y, stage_row_bytes); break;
    case 4: hipLaunchKernelGGL((combine_gather<T, U, CT, 4, 2>), grid, block, 0, s, w, tab, segments, first_rank, rank_count, stage_y, stage_row_bytes); break;
    default: hipLaunchKernelGGL((combine_gather<T, U, CT, 0, 1>), grid, block, 0, s, w, tab, segments, first_rank, rank_count, stage_y, stage_row_bytes); break;
  }
  return (int)hipGetLastError();
}

template <class CT>
int launch_combine_t(const WorldDev &w, const CT &tab, int in_dtype, int out_dtype, hipStream_t s,
                     uint32_t first_rank, uint32_t rank_count, const uint8_t *stage_y = nullptr,
                     uint64_t stage_row_bytes = 0) {
  // dtype codes follow pplx_a2a_dtype: 0 = f32, 1 = bf16, 2 = f16.
  switch (in_dtype * 4 + out_dtype) {
    case 0 * 4 + 1: return launch_combine_k<float, __bf16>(w, tab, first_rank, rank_count, stage_y, stage_row_bytes, s);
    case 0 * 4 + 2: return launch_combine_k<float, _Float16>(w, tab, first_rank, rank_count, stage_y, stage_row_bytes, s);
    case 1 * 4 + 1: return launch_combine_k<__bf16, __bf16>(w, tab, first_rank, rank_count, stage_y, stage_row_bytes, s);
    case 1 * 4 + 2: return launch_combine_k<__bf16, _Float16>(w, tab, first_rank, rank_count, stage_y, stage_row_bytes, s);
    case 2 * 4 + 1: return launch_combine_k<_Float16, __bf16>(w, tab, first_rank, rank_count, stage_y, stage_row_bytes, s);
    case 2 * 4 + 2: return launch_combine_k<_Float16, _Float16>(w, tab, first_rank, rank_count, stage_y, stage_row_bytes, s);
    default: return (int)hipErrorInvalidValue;
  }
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

int launch_split_dispatch_send(const WorldDev &w, const SplitDev &sp, const DispatchRank &row,
                               uint32_t rank, void *stream) {
  typedef SingleDispatch DT;
  hipStream_t s = (hipStream_t)stream;
  const DT tab{row};
  const uint32_t g = rank / w.dp, member = rank % w.dp;
  RouteSpan span{};
  span.v_begin = g * w.M;
  span.v_count = w.M;
  span.tile_cnt = sp.gtile_cnt + (size_t)g * sp.tiles_per_group * w.E;
  span.slot_out = sp.gslot;
  span.expert_out = sp.gexp;
  span.counts_out = sp.gcnt + (size_t)g * w.E;
  span.offsets_out = sp.goff + (size_t)g * w.E;
  span.ntok_out = sp.gntok + g;
  int err = launch_route_t<DT, true>(w, tab, span, s);
  if (err) return err;
  const uint32_t lds = 0;
  const uint32_t per_lane_rows = (w.Hb / 16 + kWave - 1) / kWave;
  const bool exact_rows = (w.Hb / 16) % kWave == 0;
  if (per_lane_rows > 8 && !(exact_rows && (per_lane_rows == 14 || per_lane_rows == 16))) {
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
  const uint32_t per_lane_rows = (w.Hb / 16 + kWave - 1) / kWave;
  const bool exact_rows = (w.Hb / 16) % kWave == 0;
  if (per_lane_rows > 8 && !(exact_rows && (per_lane_rows == 14 || per_lane_rows == 16))) {
    hipLaunchKernelGGL(split_unpack_long<DT>, grid, block, 0, s, w, tab, rank, sp);
    return (int)hipGetLastError();
  }
#define PPLX_ROW_KERNEL_ARGS rank, sp
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

int launch_split_combine_recv(const WorldDev &w, const SplitDev &sp, const CombineRank &row,
                              uint32_t rank, int in_dtype, int out_dtype, void *stream) {
  return launch_combine_t(w, SingleCombine{row}, in_dtype, out_dtype, (hipStream_t)stream, rank, 1,
                          sp.stage_y, sp.y_row_bytes);
}

int launch_combine(const WorldDev &w, const CombineRank *inline_rows, int in_dtype, int out_dtype,
                   void *stream) {
  if (inline_rows)
    return launch_combine_t(w, make_inline(w, inline_rows), in_dtype, out_dtype, (hipStream_t)stream, 0, w.R);
  return launch_combine_t(w, HbmCombine{w.crank}, in_dtype, out_dtype, (hipStream_t)stream, 0, w.R);
}

}  // namespace pplx_amd
