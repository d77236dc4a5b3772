// Device-side helpers shared by the kernel sources of the dispatch / combine path:
// vector types, the rank-table flavours a kernel can be instantiated for, address-space
// casts, scheduling barriers and wave utilities.  Included only by the .hip sources; every
// definition sits in an unnamed namespace of the including translation unit.
#pragma once
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
  static constexpr bool kInline = true;  // the table itself is the kernel argument
  DispatchRank rows[kInlineRanks];
  __device__ __forceinline__ const DispatchRank &at(uint32_t i) const { return rows[i]; }
};
struct HbmDispatch {
  static constexpr bool kInline = false;
  const DispatchRank *rows;
  __device__ __forceinline__ const DispatchRank &at(uint32_t i) const { return rows[i]; }
};
struct InlineCombine {
  CombineRank rows[kInlineRanks];
  __device__ __forceinline__ const CombineRank &at(uint32_t i) const { return rows[i]; }
};
struct HbmCombine {
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
// The same for a pointer that was read back from a table (out of LDS or HBM, where the
// compiler cannot see what it points to): a flat load would also tie up the LDS counter and
// make every later wait a wait for everything.
template <typename V>
__device__ __forceinline__ const PPLX_GLOBAL V *as_global(const V *p) {
  return (const PPLX_GLOBAL V *)p;
}
template <typename V>
__device__ __forceinline__ PPLX_GLOBAL V *as_global(V *p) {
  return (PPLX_GLOBAL V *)p;
}

// Cache policy of a row store.
//   kStream        non-temporal: the data streams past the caches to HBM, which suits a step
//                  that writes more than the 256 MB last-level cache holds;
//   kStreamThrough non-temporal and written through at agent scope ("sc1 nt"): 1.5-2 % faster
//                  than kStream in the scatter of steps of 32768 tokens and more, 1-2 % slower
//                  in the one-launch dispatch of 8192-token steps;
//   kKeep          written through at agent scope ("sc1"): the data stays in the last-level
//                  cache, where the experts' GEMMs will look for it next, and a step whose rows
//                  fit there no longer waits for HBM to take them (dispatch of 8 x 128 DSv3
//                  tokens: 18.9 instead of 22.6 us; from about 240 MB per step on it is the
//                  slowest of the three).
// The compiler offers no builtin for the scoped forms, hence the asm; they are plain vector stores.
enum class RowStore { kStream, kStreamThrough, kKeep, kPlain };

template <RowStore POLICY, typename V>
__device__ __forceinline__ void row_store(V v, PPLX_GLOBAL V *p) {
  static_assert(sizeof(V) == 16 || sizeof(V) == 4, "row_store: 4- or 16-byte values");
  if constexpr (POLICY == RowStore::kPlain) {
    *p = v;
  } else if constexpr (POLICY == RowStore::kStream) {
    __builtin_nontemporal_store(v, p);
  } else if constexpr (POLICY == RowStore::kStreamThrough) {
    if constexpr (sizeof(V) == 16) {
      asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" ::"v"(p), "v"(v) : "memory");
    } else {
      asm volatile("global_store_dword %0, %1, off sc1 nt" ::"v"(p), "v"(v) : "memory");
    }
  } else {
    if constexpr (sizeof(V) == 16) {
      asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
    } else {
      asm volatile("global_store_dword %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
    }
  }
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
template <int N> struct SettleAll {
  // other counts: in pieces of 8, 4, 2, 1 (the common counts below are one statement each)
  template <typename V> static __device__ __forceinline__ void of(V *r) {
    constexpr int kHead = N >= 8 ? 8 : N >= 4 ? 4 : N >= 2 ? 2 : 1;
    SettleAll<kHead>::of(r);
    if constexpr (N > kHead) SettleAll<N - kHead>::of(r + kHead);
  }
};
template <> struct SettleAll<1> {
  template <typename V> static __device__ __forceinline__ void of(V *r) {
    asm volatile("" : "+v"(r[0]));
  }
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
template <> struct SettleAll<7> {
  template <typename V> static __device__ __forceinline__ void of(V *r) {
    asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]));
  }
};
template <> struct SettleAll<8> {
  template <typename V> static __device__ __forceinline__ void of(V *r) {
    asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
  }
};
template <> struct SettleAll<14> {
  template <typename V> static __device__ __forceinline__ void of(V *r) {
    asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]), "+v"(r[8]), "+v"(r[9]), "+v"(r[10]), "+v"(r[11]), "+v"(r[12]), "+v"(r[13]));
  }
};
template <> struct SettleAll<16> {
  template <typename V> static __device__ __forceinline__ void of(V *r) {
    asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]), "+v"(r[8]), "+v"(r[9]), "+v"(r[10]), "+v"(r[11]), "+v"(r[12]), "+v"(r[13]), "+v"(r[14]), "+v"(r[15]));
  }
};

__device__ __forceinline__ uint32_t lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

__device__ __forceinline__ uint64_t read_lane64(uint64_t v, uint32_t src_lane) {
  return ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), (int)src_lane) << 32) |
         (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, (int)src_lane);
}

// Virtual token v = g * M + t.
__device__ __forceinline__ uint32_t group_of(const WorldDev &w, uint32_t v) { return fast_div(v, w.by_M); }
// The member of DP group g that sends token t (csrc/all_to_all/intranode_dispatch.cu:97): g * dp + t % dp.
__device__ __forceinline__ uint32_t sender_of(const WorldDev &w, uint32_t g, uint32_t t) {
  return g * w.dp + (t - fast_div(t, w.by_dp) * w.dp);
}
// Expert e lives on rank e / L as local expert e % L (csrc/all_to_all/intranode_dispatch.cu:133-134).
__device__ __forceinline__ uint32_t owner_of(const WorldDev &w, uint32_t e) { return fast_div(e, w.by_L); }
__device__ __forceinline__ uint32_t local_of(const WorldDev &w, uint32_t e) { return e - fast_div(e, w.by_L) * w.L; }

// Tokens present in DP group g this step: the reference's numSendTokens
// (csrc/all_to_all/intranode_dispatch.cu:64), clamped to the rows that exist.
template <class DT>
__device__ __forceinline__ uint32_t dispatch_group_tokens(const WorldDev &w, const DT &tab, uint32_t g) {
  const DispatchRank &r = tab.at(g * w.dp);
  uint32_t n = r.bound_m ? *as_global(r.bound_m) : r.m;
  n = n < r.m ? n : r.m;
  return n < w.M ? n : w.M;
}

// True when the group's bound_m asks for more tokens than dispatch_group_tokens() lets through
// (the reference asserts numSendTokens <= maxNumTokens, csrc/all_to_all/intranode_dispatch.cu:65).
template <class DT>
__device__ __forceinline__ bool dispatch_group_overflows(const WorldDev &w, const DT &tab, uint32_t g) {
  const DispatchRank &r = tab.at(g * w.dp);
  if (!r.bound_m) return r.m > w.M;
  const uint32_t n = *as_global(r.bound_m);
  return n > r.m || n > w.M;
}

// PV consecutive expert ids as one register value (PV = 1, 2 or 4).
template <int PV> struct PickVector;
template <> struct PickVector<1> {
  typedef uint32_t type;
  static __device__ __forceinline__ uint32_t at(type x, int) { return x; }
};
template <> struct PickVector<2> {
  typedef uint32_t type __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ uint32_t at(type x, int u) { return x[u]; }
};
template <> struct PickVector<4> {
  typedef u32x4 type;
  static __device__ __forceinline__ uint32_t at(type x, int u) { return x[u]; }
};

// What a pass over the picks of one token found: bit k of `marked` is set when fn returned a
// non-zero code for pick k, `codes` is the OR of all codes.
struct PickMarks {
  unsigned long long marked;
  uint32_t codes;
};

// Calls fn(k, expert) for the K picks at `idx` in order and collects the codes it returns.  The
// picks are fetched PV at a time (K % PV == 0, idx aligned to the vector) and up to four vectors
// are in flight at once, so a top-8 row of picks costs one trip to memory instead of eight.
template <int PV, class Fn>
__device__ __forceinline__ PickMarks for_each_pick(const PPLX_GLOBAL uint32_t *idx, uint32_t K, Fn &&fn) {
  typedef PickVector<PV> Vec;
  typedef typename Vec::type vec_t;
  const PPLX_GLOBAL vec_t *p = reinterpret_cast<const PPLX_GLOBAL vec_t *>(idx);
  const uint32_t vectors = K / PV;
  PickMarks marks{0ull, 0u};
  auto visit = [&](uint32_t j, vec_t x) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < PV; ++u) {
      const uint32_t code = fn(j * PV + u, Vec::at(x, u));
      marks.codes |= code;
      marks.marked |= (unsigned long long)(code != 0) << (j * PV + u);
    }
  };
  uint32_t j = 0;
  for (; j + 4 <= vectors; j += 4) {
    const vec_t a = p[j], b = p[j + 1], c = p[j + 2], d = p[j + 3];
    visit(j, a);
    visit(j + 1, b);
    visit(j + 2, c);
    visit(j + 3, d);
  }
  if (vectors - j >= 2) {
    const vec_t a = p[j], b = p[j + 1];
    visit(j, a);
    visit(j + 1, b);
    j += 2;
  }
  if (j < vectors) visit(j, p[j]);
  return marks;
}

__device__ __forceinline__ uint32_t combine_rank_tokens(const WorldDev &w, const CombineRank &c) {
  uint32_t n = c.bound_m ? *as_global(c.bound_m) : c.m;
  n = n < c.m ? n : c.m;
  return n < w.M ? n : w.M;
}

inline InlineDispatch make_inline(const WorldDev &w, const DispatchRank *rows) {
  InlineDispatch t{};
  for (uint32_t i = 0; i < w.R && i < kInlineRanks; ++i) t.rows[i] = rows[i];
  return t;
}

inline InlineCombine make_inline(const WorldDev &w, const CombineRank *rows) {
  InlineCombine t{};
  for (uint32_t i = 0; i < w.R && i < kInlineRanks; ++i) t.rows[i] = rows[i];
  return t;
}

}  // namespace
}  // namespace pplx_amd
