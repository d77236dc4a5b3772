// Device-visible records shared by the host layer and the kernels.
//
// One DispatchRank / CombineRank row per simulated EP rank lives in a table in
// HBM; kernels index it by rank.  They carry what the reference passes as
// Strided1D/2D/3D views (csrc/core/buffer.h:116-161) in the kernel argument
// lists of csrc/all_to_all/intranode_dispatch.cu:15-53 and
// csrc/all_to_all/intranode_combine.cu:16-47.
#pragma once

#include <cstddef>
#include <cstdint>

namespace pplx_amd {

constexpr uint32_t kWave = 64;            // gfx950 wavefront
constexpr uint32_t kInvalidSlot = 0xffffffffu;

constexpr uint32_t kFaultRowDropped = 1u;   // slot >= out_expert_x rows
constexpr uint32_t kFaultBadExpert = 2u;    // index >= num_experts
constexpr uint32_t kFaultBadSlot = 4u;      // combine slot >= expert_y rows
constexpr uint32_t kFaultDuplicateExpert = 8u;   // an expert id repeated inside one token was dropped
constexpr uint32_t kFaultTooManyTokens = 16u;    // bound_m > max_num_tokens (or > rows) was clamped

// Division by a number that is fixed for a launch (tokens per group, experts per rank ...):
// a multiply-high, a subtract, an add and two shifts instead of the thirty-odd instructions of
// a 32-bit hardware-less division (Granlund & Montgomery, "Division by invariant integers using
// multiplication", figure 4.1, N = 32).  Exact for every 32-bit numerator and divisor >= 1.
struct FastDiv {
  uint32_t mul;
  uint32_t shifts;  // sh1 (0 or 1) in bit 0, sh2 from bit 8 up: q = (t + ((n - t) >> sh1)) >> sh2
};
inline FastDiv make_fast_div(uint32_t d) {
  FastDiv f{1u, 0u};
  if (d <= 1) return f;  // l = 0: q = n
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;  // ceil(log2 d)
  f.mul = (uint32_t)((((1ull << l) - d) << 32) / d + 1);
  f.shifts = 1u | ((l - 1) << 8);
  return f;
}
#ifdef __HIPCC__
__host__ __device__
#endif
inline uint32_t fast_div(uint32_t n, const FastDiv &f) {
  const uint32_t t = (uint32_t)(((uint64_t)f.mul * n) >> 32);
  return (t + ((n - t) >> (f.shifts & 1u))) >> (f.shifts >> 8);
}

struct alignas(16) DispatchRank {
  int32_t *out_num_tokens;
  int64_t out_num_tokens_stride;
  uint8_t *expert_x;
  int64_t x_stride_row;     // bytes
  int64_t x_stride_expert;  // bytes
  float *expert_xs;
  int64_t xs_stride_elem;   // floats
  int64_t xs_stride_row;
  int64_t xs_stride_expert;
  const uint8_t *dp_x;
  int64_t dp_x_stride_row;  // bytes
  const float *dp_xs;
  int64_t dp_xs_stride_elem;
  int64_t dp_xs_stride_row;
  const uint32_t *indices;
  const uint32_t *bound_m;
  uint32_t m;
  uint32_t x_rows;
  uint64_t pad_;
};
static_assert(sizeof(DispatchRank) == 144, "DispatchRank layout");

struct alignas(16) CombineRank {
  void *out_tokens;
  int64_t out_stride_row;   // elements
  const uint32_t *indices;
  const float *weights;
  int64_t w_stride_row;
  const void *expert_y;
  int64_t y_stride_row;     // elements
  int64_t y_stride_expert;
  const uint32_t *bound_m;
  uint32_t m;
  uint32_t y_rows;
};
static_assert(sizeof(CombineRank) == 80, "CombineRank layout");

// Geometry + scratch of a world; passed to every kernel by value.
struct WorldDev {
  uint32_t R;        // simulated ranks
  uint32_t dp;       // ranks per DP group
  uint32_t G;        // DP groups = R / dp
  uint32_t M;        // max tokens per DP group
  uint32_t E;        // experts
  uint32_t L;        // experts per rank
  uint32_t K;        // experts per token
  uint32_t H;        // elements per row
  uint32_t Hb;       // bytes per dispatched row
  uint32_t S;        // fp32 scales per row
  uint32_t tile_chunks;  // 64-token chunks per routing tile of a whole-step dispatch
  uint32_t num_tiles;    // ceil(G * M / (64 * tile_chunks))
  uint32_t lds_per_cu;   // bytes of LDS a CU has (0 = unknown): launches use it to cap residency
  FastDiv by_M, by_dp, by_L, by_K;  // fast_div(n, by_X) == n / X
  DispatchRank *drank;   // [R]
  CombineRank *crank;    // [R]
  uint32_t *tile_cnt;    // [num_tiles][E] tokens routed to e inside a tile; after route_scan the
                         // tokens routed to e in all earlier tiles.  Behind it (route_tables):
                         // [num_tiles * tile_chunks][E] 64-bit masks, one bit per token of a chunk
  uint32_t *slot_map;    // [G * M][K] row of (token, pick) inside its expert
  uint32_t *faults;      // [1] sticky fault bits
};

// The routing scratch of a world is one block: the tiles' counts, then the chunks' masks.
struct RouteTables {
  uint64_t mask_offset, bytes;
};
#ifdef __HIPCC__
__host__ __device__
#endif
inline RouteTables route_tables(uint32_t num_tiles, uint32_t tile_chunks, uint32_t experts) {
  RouteTables t;
  t.mask_offset = ((uint64_t)num_tiles * experts * 4u + 7u) & ~7ull;
  t.bytes = t.mask_offset + (uint64_t)num_tiles * tile_chunks * experts * 8u;
  return t;
}

// Which virtual tokens a routing launch covers and where its results go.
struct RouteSpan {
  uint32_t v_begin;       // first virtual token (tiles are counted from here)
  uint32_t v_count;       // virtual tokens covered
  uint32_t tile_chunks;   // 64-token chunks per tile (one workgroup)
  uint32_t pick_vector;   // expert ids one load may fetch (4, 2 or 1)
  uint32_t *tile_cnt;     // [tiles][E]
  unsigned long long *tile_mask;  // [tiles * tile_chunks][E] route_count keeps the chunks' masks
                                  // here (and reports the faults) when set: the scatter that
                                  // follows works the slots out by itself
  uint32_t *slot_out;     // [G * M][K], indexed by absolute virtual token
};

// Device state of split send / recv mode: two hops through staging that the world owns.
// The reference's SEND puts one copy of a row per pick into the inbox of the rank that owns the
// pick's expert, because that copy has to cross a link (csrc/all_to_all/intranode_dispatch.cu:
// 146-180); with every rank in one HBM the staging area is the wire, and one copy per TOKEN is
// all SEND has to leave behind:
//   dispatch SEND   copies what the call may not keep -- every present token's row, scales and
//                   picks, and the number of tokens present in each DP group -- into stage_x /
//                   stage_idx / stage_n (row | fp32 scales, padded to 16 bytes: the reference's
//                   wire row, csrc/all_to_all/intranode.cpp:41-47, without the source-token tag,
//                   which the position in the staging area stands for)
//   dispatch RECV   is the one-call dispatch reading the staged copies and writing the outputs
//                   named by the RECV calls
//   combine SEND    is the one-call combine writing into stage_y, one row per (rank, token)
//   combine RECV    copies each present token's combined row to the caller's out_tokens
struct SplitDev {
  uint8_t *stage_x;        // [G * M][token_stride]
  uint32_t token_stride;   // round_up(Hb + 4 S, 16)
  uint32_t pad_;
  uint32_t *stage_idx;     // [G * M][K] the staged tokens' picks
  uint32_t *stage_n;       // [G] tokens present in each DP group at SEND
  uint8_t *stage_y;        // [R * M][H] combined rows, 2-byte elements
};

// stage_x, stage_idx and stage_n are one allocation, in this order.
struct StageLayout {
  uint32_t token_stride;
  uint64_t idx_offset, n_offset, bytes;
};
#ifdef __HIPCC__
__host__ __device__
#endif
inline StageLayout stage_layout(uint32_t row_bytes, uint32_t scales, uint64_t tokens, uint32_t picks,
                                uint32_t groups) {
  StageLayout l;
  l.token_stride = (row_bytes + 4u * scales + 15u) & ~15u;
  l.idx_offset = tokens * l.token_stride;
  l.n_offset = (l.idx_offset + tokens * picks * 4u + 15u) & ~15ull;
  l.bytes = l.n_offset + ((4ull * groups + 15u) & ~15ull);
  return l;
}

// Worlds of up to kInlineRanks ranks pass their rank tables to the kernels as
// kernel arguments (9 KiB for dispatch, 5 KiB for combine; HIP on gfx950 takes kernel
// arguments well beyond 4 KiB, eagerly and as graph nodes); larger worlds go through the
// HBM tables (drank / crank), written by bind kernels that take up to kBindBatch rows as
// arguments each.
constexpr uint32_t kInlineRanks = 64;
constexpr uint32_t kBindBatch = 64;
// Steps of at most this many virtual tokens (DP groups x max_num_tokens) dispatch in one fused
// launch.
constexpr uint32_t kFusedMaxTokens = 3072;
// A fused launch whose rows (all picks of all tokens) stay within this many bytes stores them
// write-through into the 256 MB last-level cache instead of streaming them past it.
constexpr uint64_t kWriteThroughMaxBytes = 192ull << 20;

// Device memory that pplx_a2a_static_step works in instead of a world's allocations: a fixed
// array inside the library's code object (a2a_static.hip), one copy per GPU.
constexpr size_t kStaticScratchBytes = 8u << 20;
// Address of the calling thread's current device's copy (looked up once per device).
int static_scratch_address(int device, void **out);
// True once static_scratch_address has succeeded for `device`.
bool static_scratch_known(int device);

struct BindDispatchBatch {
  uint32_t first, count;
  uint64_t pad_;
  DispatchRank rows[kBindBatch];
};
struct BindCombineBatch {
  uint32_t first, count;
  uint64_t pad_;
  CombineRank rows[kBindBatch];
};

// Launchers implemented in a2a_dispatch.hip, a2a_combine.hip and a2a_split.hip; they return a
// hipError_t as int.
// `inline_rows` (world_size rows, host memory) selects the inline-table kernels;
// NULL selects the HBM tables, which must have been bound.
int launch_bind_dispatch(const WorldDev &w, const BindDispatchBatch &b, void *stream);
int launch_bind_combine(const WorldDev &w, const BindCombineBatch &b, void *stream);
// pick_vector: how many expert ids one load may fetch from any rank's indices (4, 2 or 1):
// K must be a multiple of it and every indices pointer aligned to 4 * pick_vector bytes.
int launch_dispatch(const WorldDev &w, const DispatchRank *inline_rows, uint32_t pick_vector,
                    void *stream);
int launch_combine(const WorldDev &w, const CombineRank *inline_rows, int in_dtype, int out_dtype,
                   void *stream);
// Split mode's own launches, each for all ranks at once (`inline_rows` as above): dispatch SEND
// stages the tokens, combine RECV delivers the combined rows (`elem_bytes` of out_tokens).
// dispatch RECV and combine SEND are launch_dispatch / launch_combine on rows that point into
// the staging area.
int launch_split_stage_tokens(const WorldDev &w, const SplitDev &sp, const DispatchRank *inline_rows,
                              void *stream);
int launch_split_deliver(const WorldDev &w, const SplitDev &sp, const CombineRank *inline_rows, void *stream);
// True when dispatch runs as the single fused launch for this geometry.
bool dispatch_is_fused(const WorldDev &w);
// LDS bytes the routing kernels need for a given geometry.
uint32_t route_lds_bytes(uint32_t num_experts, uint32_t tile_chunks);

}  // namespace pplx_amd
