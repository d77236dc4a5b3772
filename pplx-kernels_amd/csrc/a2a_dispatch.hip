// gfx950 kernels of the MoE dispatch / combine path (single-GPU loopback).
//
// The reference moves every token through a per-peer inbox with atomically
// assigned slots and grid-wide syncs (csrc/all_to_all/intranode_dispatch.cu:15-284,
// csrc/all_to_all/intranode_combine.cu:16-187).  With all simulated ranks in one
// HBM the same results come from a count -> scan -> scatter pipeline whose
// placement is the canonical (expert, DP group, token) order that the
// reference's tests enumerate (tests/test_all_to_all.py:113-120):
//
//   route_count      per routing tile: 64-token bitmasks per expert in LDS -> rows per
//                    expert of the tile, and the masks themselves          (only if > 1 tile)
//   route_scan       per expert: prefix of the tiles' rows, totals         (only if > 1 tile)
//   dispatch_scatter_slots  one wave per token (or per share of its K picks): the row is
//                    read once into registers, lane k works the slot of pick k out of the
//                    scanned rows and the masks, the row is stored K times, 16 B / lane
//   route_slots + dispatch_scatter  the same with the slots written by a launch of their
//                    own (single tile, rows beyond the register variants)
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

// Built with -DPPLX_A2A_TIMELINE (make TIMELINE=1), dispatch_fused records when thread 0 of every
// workgroup passes its phase boundaries (the GPU's 100 MHz wall clock) into a table that
// pplx_a2a_debug_timeline copies out; `bench.py --timeline` prints the summary.  The waits that
// the stamps need (for the row, for the stores) are not in the regular build.
#ifdef PPLX_A2A_TIMELINE
__device__ unsigned long long g_timeline[1024 * 16];
extern "C" int pplx_a2a_debug_timeline(unsigned long long *host, int words) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(g_timeline), sizeof(unsigned long long) * (size_t)words);
}
#endif

namespace pplx_amd {
namespace {

struct Timeline {
#ifdef PPLX_A2A_TIMELINE
  unsigned long long at[9];
  __device__ __forceinline__ void mark(int i) { at[i] = wall_clock64(); }
  __device__ __forceinline__ void wait_for_memory() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }
  __device__ __forceinline__ void flush() {
    if (threadIdx.x != 0 || blockIdx.x >= 1024) return;
    for (int i = 0; i < 9; ++i) g_timeline[blockIdx.x * 16 + i] = at[i];
    g_timeline[blockIdx.x * 16 + 9] = __builtin_amdgcn_s_getreg((20 << 0) | (0 << 6) | (3 << 11)) & 0xf;  // XCC id
  }
#else
  __device__ __forceinline__ void mark(int) {}
  __device__ __forceinline__ void wait_for_memory() {}
  __device__ __forceinline__ void flush() {}
#endif
};

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

// One wave per token (or per share of its picks).  ROUTED: the slot map was written by
// route_slots; otherwise the wave works its token's slots out of the routing tables
// (slots_from_masks) and writes the slot map itself.
template <int NV, bool EXACT, class DT, bool ROUTED>
__device__ __forceinline__ void scatter_token(const WorldDev &w, const DT &tab, uint32_t ksplit, uint32_t kper) {
  const uint32_t lane = lane_id();
  const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) +
                                                       threadIdx.x / kWave);
  const uint32_t v = wave >> __builtin_ctz(ksplit);  // (ksplit is a power of two)
  const uint32_t part = wave - v * ksplit;
  const uint32_t g = group_of(w, v);
  const uint32_t t = v - g * w.M;
  if (g >= w.G) return;
  if (t >= dispatch_group_tokens(w, tab, g)) return;
  const DispatchRank &src = tab.at(sender_of(w, g, t));
  RowRegs<NV> regs;
  load_row<NV, EXACT>(w, src, t, lane, regs);
  Destination dst;
  if constexpr (ROUTED) {
    if (lane < w.K) {
      dst = resolve_destination(w, tab, as_global(src.indices)[(size_t)t * w.K + lane],
                                as_global(w.slot_map)[(size_t)v * w.K + lane],
                                part == 0);
    }
  } else {
    const uint32_t e = lane < w.K ? as_global(src.indices)[(size_t)t * w.K + lane] : w.E;
    const uint32_t slot = slots_from_masks(w, v, lane, e);
    if (lane < w.K) {
      dst = resolve_destination(w, tab, e, slot, part == 0);
      if (part == 0) as_global(w.slot_map)[(size_t)v * w.K + lane] = slot;
    }
  }
  const uint32_t k0 = part * kper;
  const uint32_t k1 = (k0 + kper < w.K) ? k0 + kper : w.K;
  // Rows stream past the caches; the 4-byte-per-lane scale rows are written through into the
  // last-level cache instead, where the partial lines of neighbouring rows meet before they go
  // to HBM (3-4 % of the kernel's time at 224-byte scale rows).
  store_row<NV, EXACT, RowStore::kStreamThrough, RowStore::kKeep>(w, src, t, lane, dst, k0, k1, regs);
}

// Launched as one-wave workgroups whose dynamic LDS size caps how many of them a CU holds at a
// time (see launch_scatter_t); the kernels themselves do not touch LDS.
template <int NV, bool EXACT, class DT>
__global__ __launch_bounds__(256) void dispatch_scatter(WorldDev w, DT tab, uint32_t ksplit, uint32_t kper) {
  scatter_token<NV, EXACT, DT, true>(w, tab, ksplit, kper);
}

template <int NV, bool EXACT, class DT>
__global__ __launch_bounds__(256) void dispatch_scatter_slots(WorldDev w, DT tab, uint32_t ksplit, uint32_t kper) {
  scatter_token<NV, EXACT, DT, false>(w, tab, ksplit, kper);
}

// Threads of a dispatch_fused workgroup: 16 waves (fewer, larger workgroups repeat less
// counting) while the row fits 8 registers of 16 bytes per lane, 8 waves for the 14- and
// 16-register rows, which would spill under the 128-register limit of a 1024-thread workgroup.
// A compile-time size also keeps the kernel's first loads free of any wait.
constexpr uint32_t fused_threads(int nv) { return nv > 8 ? 512u : 1024u; }

// A rank table that dispatch_fused has copied into LDS.
struct LdsDispatch {
  const DispatchRank *rows;
  __device__ __forceinline__ const DispatchRank &at(uint32_t i) const { return rows[i]; }
};

// Counts, per expert, the tokens before virtual token v_end that are routed to it, into the LDS
// histogram `hist`: one thread per token and pass, PV picks per load (K % PV == 0 and every
// indices pointer aligned to the vector: the host checks both).  Every expert a token names
// counts once (a repeat inside the token takes no row).
//
// The loads of a token (its group's token count and its first two vectors of picks) are
// unconditional, from a harmless address when the thread has no token, and sit in
// straight-line code: they are issued together and cost one trip to memory, and the count is
// applied afterwards.  The loads of the next pass are issued before the picks of this one are
// counted, so a step of several passes pays one trip, not one per pass.
template <int PV, uint32_t THREADS, class Table>
__device__ __forceinline__ void count_earlier_picks(const WorldDev &w, const Table &rows, uint32_t v_end,
                                                    uint32_t *hist) {
  typedef PickVector<PV> Vec;
  typedef typename Vec::type vec_t;
  const uint32_t vectors = w.K / PV;
  struct Fetch {
    vec_t a, b;           // vectors 0 and 1 of the token's picks (b repeats a when there is one)
    uint32_t n;           // tokens present in the group
    uint32_t t;           // token inside its group
    const PPLX_GLOBAL vec_t *idx;
    bool valid;
  };
  auto issue = [&](uint32_t v) {
    Fetch f;
    const bool in_range = v < v_end;
    const uint32_t g = in_range ? group_of(w, v) : 0;
    f.t = in_range ? v - g * w.M : 0;
    const DispatchRank &head = rows.at(g * w.dp);
    const DispatchRank &src = w.dp == 1 ? head : rows.at(sender_of(w, g, f.t));
    f.valid = in_range && f.t < src.m && f.t < head.m;
    const bool bounded = f.valid && head.bound_m != nullptr;
    const uint32_t loaded_n = *as_global(bounded ? head.bound_m : w.faults);
    f.idx = as_global(reinterpret_cast<const vec_t *>(f.valid ? src.indices + (size_t)f.t * w.K : w.slot_map));
    f.a = f.idx[0];
    f.b = f.idx[vectors > 1 ? 1 : 0];
    f.n = bounded ? loaded_n : head.m;
    return f;
  };
  auto place = [&](uint32_t j, vec_t a, vec_t b, const Fetch &f) {
    const bool second = j + 1 < vectors;
    // The picks of this call are compared in registers; those of earlier calls for the same
    // token (top-k beyond two vectors) are read again.
    uint32_t e[2 * PV];
#pragma unroll
    for (int u = 0; u < PV; ++u) {
      e[u] = Vec::at(a, u);
      e[PV + u] = second ? Vec::at(b, u) : w.E;
    }
#pragma unroll
    for (int u = 0; u < 2 * PV; ++u) {
      bool counts = e[u] < w.E;
#pragma unroll
      for (int p = 0; p < u; ++p) counts = counts && e[p] != e[u];
      if (counts && j != 0) {
        const PPLX_GLOBAL uint32_t *before = reinterpret_cast<const PPLX_GLOBAL uint32_t *>(f.idx);
        for (uint32_t p = 0; p < j * PV; ++p) counts = counts && before[p] != e[u];
      }
      if (counts) atomicAdd(&hist[e[u]], 1u);
    }
  };
  auto consume = [&](const Fetch &f) {
    if (!f.valid || f.t >= f.n) return;
    place(0, f.a, f.b, f);
    for (uint32_t j = 2; j < vectors; j += 2) place(j, f.idx[j], f.idx[j + 1 < vectors ? j + 1 : j], f);
  };

  Fetch current = issue(threadIdx.x);
  for (uint32_t v = threadIdx.x + THREADS; v < v_end; v += THREADS) {
    const Fetch next = issue(v);
    consume(current);
    current = next;
  }
  consume(current);
}

// Small steps: one launch does routing and scatter.  A workgroup owns tokens_per_block
// consecutive virtual tokens; each of them belongs to one wave (or to ksplit waves that share
// its picks), and lane k of such a row wave is the token's pick k.
//   0. the rank table (world_size rows of it) is copied from the kernel arguments into LDS with
//      loads that depend on nothing, so every later lookup is an LDS read and not another trip
//      to memory behind the one that fetches the geometry;
//   1. one batch of small loads: every thread fetches the picks of one token before the
//      workgroup's own (and its group's token count), the row waves their own picks;
//   2. the picks of the earlier tokens are counted per expert in an LDS histogram (every
//      workgroup repeats this over the indices, which are a few KiB in L2); the row waves mark
//      their token in a per-expert bit mask of the workgroup's own tokens and issue the loads of
//      their rows (where exactly the row loads go -- with the picks' loads, behind their
//      arrival, or behind the counting as written here -- changes nothing that can be measured:
//      8 x 128 DSv3 tokens take 13.5-13.7 us and 64 x 1 tokens 5.6-6.3 us in every order, the
//      first bound by the rate of their stores, the second by the chain of cold trips);
//   3. behind one barrier a pick's slot is the histogram's count plus the own tokens before
//      its own that go to the same expert (a popcount of the mask below the token's bit); the
//      lane resolves its destination row and keeps it in registers;
//   4. the waves fan their rows out.  The last workgroup has counted everything and writes
//      out_expert_num_tokens.
template <int NV, bool EXACT, class DT>
__global__ __launch_bounds__(fused_threads(NV)) void dispatch_fused(WorldDev w, DT tab, uint32_t ksplit,
                                                                  uint32_t kper, uint32_t tokens_per_block,
                                                                  uint32_t pick_vector, uint32_t write_through) {
  constexpr uint32_t kFusedThreads = fused_threads(NV);
  extern __shared__ unsigned long long lds_u64[];
  Timeline timeline;
  timeline.mark(0);
  constexpr bool kStaged = DT::kInline;
  constexpr uint32_t kRowWords = sizeof(DispatchRank) / 8;
  const uint32_t table_words = kStaged ? w.R * kRowWords : 0;
  if constexpr (kStaged) {
    const unsigned long long *args = reinterpret_cast<const unsigned long long *>(&tab);
    for (uint32_t i = threadIdx.x; i < table_words; i += kFusedThreads) lds_u64[i] = args[i];
  }
  uint32_t *hist = reinterpret_cast<uint32_t *>(lds_u64 + table_words);  // [E] tokens before the workgroup's own
  uint32_t *own_mask = hist + w.E;                                       // [E] bit j: own token j goes to e
  for (uint32_t e = threadIdx.x; e < 2 * w.E; e += kFusedThreads) hist[e] = 0;
  // Orders the zeroing (and the staged table) before the first counter update of any wave.
  __syncthreads();
  timeline.mark(1);
  const LdsDispatch staged{reinterpret_cast<const DispatchRank *>(lds_u64)};
  auto rows = [&]() -> decltype(auto) {
    if constexpr (kStaged) return (staged); else return (tab);
  };

  const uint32_t total = w.G * w.M;
  const uint32_t v0 = blockIdx.x * tokens_per_block;

  // 1. this wave's token; lane k is its pick k
  const uint32_t lane = lane_id();
  const uint32_t my_wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const uint32_t my_j = my_wave >> __builtin_ctz(ksplit);  // (ksplit is a power of two)
  const uint32_t my_part = my_wave - my_j * ksplit;
  const uint32_t my_v = v0 + my_j;
  const bool my_in_range = my_j < tokens_per_block && my_v < total;
  const uint32_t my_g = my_in_range ? group_of(w, my_v) : 0;
  const uint32_t my_t = my_in_range ? my_v - my_g * w.M : 0;
  const DispatchRank &my_head = rows().at(my_g * w.dp);
  const DispatchRank &my_src = w.dp == 1 ? my_head : rows().at(sender_of(w, my_g, my_t));
  const bool my_row_exists = my_in_range && my_t < my_src.m && my_t < my_head.m;
  const bool my_bounded = my_row_exists && my_head.bound_m != nullptr;
  const uint32_t my_loaded_n = *as_global(my_bounded ? my_head.bound_m : w.faults);
  const bool has_pick = my_row_exists && lane < w.K;
  const uint32_t my_loaded_e = *as_global(has_pick ? my_src.indices + (size_t)my_t * w.K + lane : w.faults);

  // 2. picks of all earlier tokens
  if (pick_vector == 4) {
    count_earlier_picks<4, kFusedThreads>(w, rows(), v0, hist);
  } else if (pick_vector == 2) {
    count_earlier_picks<2, kFusedThreads>(w, rows(), v0, hist);
  } else {
    count_earlier_picks<1, kFusedThreads>(w, rows(), v0, hist);
  }
  timeline.mark(2);
  // ... and the workgroup's own: a pick that names no expert, or repeats an earlier pick of its
  // token, has no row.
  uint32_t my_n = my_bounded ? my_loaded_n : my_head.m;
  my_n = my_n < w.M ? my_n : w.M;
  const bool my_live = my_row_exists && my_t < my_n;
  const uint32_t my_e = has_pick ? my_loaded_e : w.E;
  bool my_repeats = false;
  for (uint32_t k = 0; k + 1 < w.K; ++k) {
    const uint32_t earlier = (uint32_t)__builtin_amdgcn_readlane((int)my_e, (int)k);
    if (lane > k && earlier == my_e) my_repeats = true;
  }
  const bool my_pick_has_row = my_live && my_e < w.E && !my_repeats;
  if (my_pick_has_row && my_part == 0) atomicOr(&own_mask[my_e], 1u << my_j);
  timeline.mark(3);
  RowRegs<NV> regs;
  if (my_live) load_row<NV, EXACT>(w, my_src, my_t, lane, regs);
  __syncthreads();
  timeline.mark(4);

  // 3. own slots and destinations
  uint32_t my_slot = kInvalidSlot;
  if (my_pick_has_row) my_slot = hist[my_e] + __popc(own_mask[my_e] & ((1u << my_j) - 1u));
  Destination dst;
  if (my_in_range && lane < w.K) {
    const size_t pair = (size_t)my_v * w.K + lane;
    if (my_live) dst = resolve_destination(w, rows(), my_e, my_slot, my_part == 0);
    if (my_live && my_part == 0) {
      as_global(w.slot_map)[pair] = my_slot;
      if (my_e >= w.E) {
        atomicOr(w.faults, kFaultBadExpert);
      } else if (my_repeats) {
        atomicOr(w.faults, kFaultDuplicateExpert);
      }
    }
  }
  if (blockIdx.x == gridDim.x - 1) {
    for (uint32_t e = threadIdx.x; e < w.E; e += kFusedThreads) {
      const uint32_t rows_of_e = hist[e] + __popc(own_mask[e]);
      const DispatchRank &owner = rows().at(owner_of(w, e));
      as_global(owner.out_num_tokens)[(int64_t)local_of(w, e) * owner.out_num_tokens_stride] = (int32_t)rows_of_e;
    }
  }

  timeline.mark(5);
  // 4. fan out
  if (my_live) {
    timeline.wait_for_memory();
    timeline.mark(6);
    const uint32_t k0 = my_part * kper;
    const uint32_t k1 = (k0 + kper < w.K) ? k0 + kper : w.K;
    if (write_through) {
      store_row<NV, EXACT, RowStore::kKeep>(w, my_src, my_t, lane, dst, k0, k1, regs);
    } else {
      store_row<NV, EXACT, RowStore::kStream>(w, my_src, my_t, lane, dst, k0, k1, regs);
    }
  }
  timeline.mark(7);
  timeline.wait_for_memory();
  timeline.mark(8);
  timeline.flush();
  // A bound_m beyond the limit is reported once, behind the stores (it costs a trip to memory).
  if (blockIdx.x == 0) {
    for (uint32_t g = threadIdx.x; g < w.G; g += kFusedThreads) {
      if (dispatch_group_overflows(w, rows(), g)) atomicOr(w.faults, kFaultTooManyTokens);
    }
  }
}

// Rows longer than the register variants cover: stream each vector K times.
template <class DT>
__global__ __launch_bounds__(256) void dispatch_scatter_long(WorldDev w, DT tab) {
  __shared__ uint64_t s_row[kWave];
  __shared__ uint64_t s_scale[kWave];
  __shared__ int64_t s_step[kWave];
  const uint32_t v = blockIdx.x;
  const uint32_t g = group_of(w, v);
  const uint32_t t = v - g * w.M;
  if (g >= w.G) return;
  if (t >= dispatch_group_tokens(w, tab, g)) return;
  const DispatchRank &src = tab.at(sender_of(w, g, t));
  if (threadIdx.x < w.K) {
    uint64_t dst_row = 0, dst_scale = 0;
    int64_t step = 0;
    const uint32_t e = as_global(src.indices)[(size_t)t * w.K + threadIdx.x];
    const uint32_t slot = as_global(w.slot_map)[(size_t)v * w.K + threadIdx.x];
    if (e < w.E && slot != kInvalidSlot) {
      const DispatchRank &dst = tab.at(owner_of(w, e));
      const uint32_t el = local_of(w, e);
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
  const PPLX_GLOBAL u32x4 *row =
      as_global(reinterpret_cast<const u32x4 *>(src.dp_x + (int64_t)t * src.dp_x_stride_row));
  for (uint32_t j = threadIdx.x; j < nvec; j += blockDim.x) {
    const u32x4 x = row[j];
    for (uint32_t k = 0; k < w.K; ++k) {
      if (s_row[k]) global_ptr<u32x4>(s_row[k])[j] = x;
    }
  }
  if (w.S) {
    const PPLX_GLOBAL float *srow = as_global(src.dp_xs) + (int64_t)t * src.dp_xs_stride_row;
    for (uint32_t j = threadIdx.x; j < w.S; j += blockDim.x) {
      const float sc = srow[(int64_t)j * src.dp_xs_stride_elem];
      for (uint32_t k = 0; k < w.K; ++k) {
        if (s_scale[k]) global_ptr<float>(s_scale[k])[(int64_t)j * s_step[k]] = sc;
      }
    }
  }
}

// LDS of a dispatch_fused workgroup: the rank table (when it came inline), the histogram and
// the mask of the workgroup's own tokens.
uint32_t fused_lds_bytes(const WorldDev &w, bool inline_table) {
  const uint32_t table = inline_table ? w.R * (uint32_t)sizeof(DispatchRank) : 0u;
  return table + 2u * w.E * (uint32_t)sizeof(uint32_t);
}

// Number of waves a row's K copies are spread over: few tokens -> more waves,
// so that the launch still covers the 256 CUs (the row re-reads hit L2).
uint32_t pick_ksplit(const WorldDev &w, uint32_t max_split) {
  const uint64_t tokens = (uint64_t)w.G * w.M;
  uint32_t ksplit = 1;
  while (ksplit < max_split && ksplit < w.K && tokens * ksplit < 4096) ksplit *= 2;
  return ksplit;
}

// Scatter waves a CU should hold at a time (0 = as many as fit).
// Measured on 8 x 4096 tokens with the slots worked out by the scatter's waves
// (us at 3 / 4 / 6 / 8 / 12 / 16 waves per CU / full occupancy):
//   112 KiB stored per wave (14 KiB rows, top-8)      847 / 844 / 851 / 855 / 860 / 858 / 857
//   59 KiB (DSv3 fp8 rows, top-8)                     404 / 421 / 437 / 437 / 427 / 432 / 433
//   32 KiB (4 KiB rows, top-8)                        206 / 211 / 215 / 216 / 217 / 220 / 221
//   16 KiB (8 KiB rows, top-2)                        164 / 152 / 155 / 160 / 163 / 165 / 167
//   17 KiB (2 KiB fp8 rows with scales, top-8)        163 / 133 / 106 / 104 / 109 / 110 / 111
//   14 KiB (DSv3 fp8 rows, top-2)                     181 / 155 / 140 / 141 / 146 / 149 / 148
//    8 KiB (1 KiB rows, top-8)                        122 / 100 /  77 /  64 /  57 /  60 /  60
//    4 KiB (2 KiB rows, top-2)                        103 /  84 /  66 /  57 /  50 /  46 /  44
// and on the Mixtral prefill (8 x 4096 tokens of 8 KiB, top-2, skewed routing) 147.5 us at 4
// against 145.8 at 6.  A wave's launch, its loads and its slot arithmetic are dead time for the
// stores, so the less a wave stores the more of them it takes to keep the CU's stores going.
uint32_t scatter_waves_per_cu(const WorldDev &w, uint32_t picks_per_wave) {
  if (w.lds_per_cu == 0) return 0;
  const uint64_t row = w.Hb + 4ull * w.S;
  const uint64_t stored = (uint64_t)picks_per_wave * row;
  if (stored >= 24 * 1024) return 3;
  if (stored >= 12 * 1024) return row >= 4096 ? 6 : 8;
  if (stored >= 6 * 1024) return 12;
  return 0;
}

// Rows that dispatch_scatter holds in registers (longer ones stream through dispatch_scatter_long).
bool scatter_has_register_rows(const WorldDev &w) { return (w.Hb / 16 + kWave - 1) / kWave <= 32; }

template <class DT>
int launch_scatter_t(const WorldDev &w, const DT &tab, bool routed, hipStream_t s) {
  const uint32_t tokens = w.G * w.M;
  if (!scatter_has_register_rows(w)) {
    hipLaunchKernelGGL(dispatch_scatter_long<DT>, dim3(tokens), dim3(256), 0, s, w, tab);
    return (int)hipGetLastError();
  }
  const uint32_t ksplit = pick_ksplit(w, kWave);
  const uint32_t kper = (w.K + ksplit - 1) / ksplit;
  const uint64_t waves = (uint64_t)tokens * ksplit;
  // One wave per workgroup, and few of them per CU at a time.  A wave reads one row and then
  // has up to K rows of stores to issue; HBM takes those stores best when a CU sends the rows of
  // three or four waves at a time rather than those of thirty-two interleaved (figures at
  // scatter_waves_per_cu).  The hardware has no such knob, so each workgroup asks for a share of
  // the CU's LDS that only that many fit into.
  const uint32_t waves_per_cu = scatter_waves_per_cu(w, kper);
  // (LDS is handed out in blocks: a share that is not a multiple of 4 KiB can round up past
  // what the intended number of workgroups leaves room for)
  uint32_t lds = waves_per_cu ? (w.lds_per_cu / waves_per_cu) & ~4095u : 0u;
  if (lds > 65536u) lds = 65536u;
  const dim3 grid((uint32_t)waves), block(kWave);
#define PPLX_ROW_KERNEL_ARGS ksplit, kper
#define PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL)                                                    \
  do {                                                                                           \
    if (per_lane <= 16) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 16, false);                              \
    else PPLX_LAUNCH_ROW_VARIANT(KERNEL, 32, false);                                             \
  } while (0)
  if (routed) {
    PPLX_DISPATCH_ROW_VARIANTS(dispatch_scatter);
  }
#undef PPLX_LAUNCH_LARGE_ROW_VARIANT
  // (rows beyond 16 KiB leave no registers for the slot arithmetic: slots_in_scatter() sends
  // them through route_slots and the kernel above)
#define PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL)                                                    \
  do {                                                                                           \
    if (per_lane <= 16) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 16, false);                              \
    else return (int)hipErrorInvalidValue;                                                       \
  } while (0)
  if (!routed) {
    PPLX_DISPATCH_ROW_VARIANTS(dispatch_scatter_slots);
  }
#undef PPLX_LAUNCH_LARGE_ROW_VARIANT
#undef PPLX_ROW_KERNEL_ARGS
  return (int)hipGetLastError();
}

template <class DT>
int launch_fused_t(const WorldDev &w, const DT &tab, uint32_t pick_vector, hipStream_t s) {
  const uint32_t tokens = w.G * w.M;
  const uint32_t kWaves = fused_threads((int)((w.Hb / 16 + kWave - 1) / kWave)) / kWave;
  // Tokens per workgroup: as few as still give every CU a workgroup (all of a workgroup's waves
  // help with the counting; only the waves that own a token, or a share of one, load and store
  // rows, and few storing waves per CU suit the memory system better than sixteen: 8 x 128 DSv3
  // tokens take 14.7 us with 4 row waves per workgroup against 15.1 us with 16).  Steps of fewer
  // than 1024 tokens spread each token's picks over several waves instead.
  uint32_t tokens_per_block = (tokens + 255) / 256;
  if (tokens_per_block > kWaves) tokens_per_block = kWaves;
  if (tokens_per_block < 1) tokens_per_block = 1;
  uint32_t ksplit = 1;
  while (ksplit * 2 <= w.K && tokens_per_block * ksplit * 2 <= kWaves && (uint64_t)tokens * ksplit < 1024) ksplit *= 2;
  const uint32_t kper = (w.K + ksplit - 1) / ksplit;
  const dim3 grid((tokens + tokens_per_block - 1) / tokens_per_block), block(kWaves * kWave);
  const uint32_t lds = fused_lds_bytes(w, DT::kInline && w.R <= kInlineRanks);
  // Rows that fit the last-level cache with room to spare are written through into it.
  const uint64_t row_bytes = (uint64_t)tokens * w.K * (w.Hb + 4ull * w.S);
  const uint32_t write_through = row_bytes <= kWriteThroughMaxBytes ? 1u : 0u;
#define PPLX_ROW_KERNEL_ARGS ksplit, kper, tokens_per_block, pick_vector, write_through
#define PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL) return (int)hipErrorInvalidValue
  PPLX_DISPATCH_ROW_VARIANTS(dispatch_fused);
#undef PPLX_LAUNCH_LARGE_ROW_VARIANT
#undef PPLX_ROW_KERNEL_ARGS
  return (int)hipGetLastError();
}

template <class DT>
int launch_dispatch_t(const WorldDev &w, const DT &tab, uint32_t pick_vector, hipStream_t s) {
  if (dispatch_is_fused(w)) return launch_fused_t(w, tab, pick_vector, s);
  RouteSpan span{};
  span.v_begin = 0;
  span.v_count = w.G * w.M;
  span.tile_chunks = w.tile_chunks;
  span.pick_vector = pick_vector;
  span.tile_cnt = w.tile_cnt;
  span.slot_out = w.slot_map;
  // Steps of several tiles leave the last routing launch out: the scatter's waves work their
  // own slots out of the tiles' tables.
  const bool slots_in_scatter = w.num_tiles > 1 && (w.Hb / 16 + kWave - 1) / kWave <= 16;
  if (slots_in_scatter) {
    span.tile_mask = reinterpret_cast<unsigned long long *>(
        reinterpret_cast<uint8_t *>(w.tile_cnt) + route_tables(w.num_tiles, w.tile_chunks, w.E).mask_offset);
  }
  int err = launch_route_t(w, tab, span, s);
  if (err) return err;
  return launch_scatter_t(w, tab, !slots_in_scatter, s);
}

}  // namespace

// ---------------------------------------------------------------------------
// Launchers
// ---------------------------------------------------------------------------
uint32_t route_lds_bytes(uint32_t num_experts, uint32_t tile_chunks) {
  return tile_chunks * num_experts * (uint32_t)(sizeof(unsigned long long) + sizeof(uint32_t));
}

bool dispatch_is_fused(const WorldDev &w) {
  // Every workgroup recounts all earlier tokens (work that grows with the square of the token
  // count) and all of a workgroup's row waves store at once, while the scatter behind the two
  // routing launches keeps few storing waves per CU.  Measured on 8 ranks (us, one launch /
  // routing + scatter) at 2048, 3072, 4096, 6144 tokens: 7 KiB fp8 rows, top-8 of 256:
  // 24 / 37, 45 / 48, 61 / 56, 86 / 79; 8 KiB rows, top-2 of 8: 15 / 21, 20 / 25, 26 / 27,
  // 40 / 35; 4 KiB rows, top-8 of 64: 19 / 25, 26 / 32, 34 / 36, 49 / 49.  The one-launch form pays
  // while the routing launches (about 10 us of latency) weigh more than the scatter's better rate.
  const uint64_t tokens = (uint64_t)w.G * w.M;
  return tokens <= kFusedMaxTokens && row_has_register_variant(w) && fused_lds_bytes(w, true) <= 60 * 1024;
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

int launch_dispatch(const WorldDev &w, const DispatchRank *inline_rows, uint32_t pick_vector, void *stream) {
  if (pick_vector != 4 && pick_vector != 2) pick_vector = 1;
  if (inline_rows) return launch_dispatch_t(w, make_inline(w, inline_rows), pick_vector, (hipStream_t)stream);
  return launch_dispatch_t(w, HbmDispatch{w.drank}, pick_vector, (hipStream_t)stream);
}

}  // namespace pplx_amd
