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
//   combine_gather   one workgroup per token: K rows gathered through the slot
//                    map, fp32 accumulate in pick order, 16 B stores
//
// No atomics on global memory, no spin waits, no cooperative launch: phase
// boundaries are kernel boundaries on one stream, so a step captures into a
// hipGraph as is.  Wavefronts are 64 wide throughout.
#include <hip/hip_runtime.h>

#include "a2a_device.h"

namespace pplx_amd {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ uint32_t lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// Tokens present in DP group g this step: the reference's numSendTokens
// (csrc/all_to_all/intranode_dispatch.cu:64), clamped to the rows that exist.
__device__ __forceinline__ uint32_t dispatch_group_tokens(const WorldDev &w, uint32_t g) {
  const DispatchRank &r = w.drank[g * w.dp];
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
__global__ __launch_bounds__(1024) void route_count(WorldDev w) {
  extern __shared__ uint32_t lds_hist[];
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) lds_hist[e] = 0;
  __syncthreads();

  const uint32_t v = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  if (g < w.G && t < dispatch_group_tokens(w, g)) {
    const uint32_t *idx = w.drank[g * w.dp + t % w.dp].indices + (size_t)t * w.K;
    for (uint32_t k = 0; k < w.K; ++k) {
      const uint32_t e = idx[k];
      if (e < w.E) atomicAdd(&lds_hist[e], 1u);
    }
  }
  __syncthreads();
  uint32_t *out = w.tile_cnt + (size_t)blockIdx.x * w.E;
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) out[e] = lds_hist[e];
}

__global__ __launch_bounds__(1024) void route_slots(WorldDev w) {
  // LDS: mask[chunks][E] (one bit per token of the chunk routed to e),
  //      then base[chunks][E] (rows of e taken before the chunk starts).
  extern __shared__ unsigned long long lds_mask[];
  const uint32_t chunks = w.tile_chunks;
  uint32_t *lds_base = reinterpret_cast<uint32_t *>(lds_mask + (size_t)chunks * w.E);

  for (uint32_t i = threadIdx.x; i < chunks * w.E; i += blockDim.x) lds_mask[i] = 0ull;
  __syncthreads();

  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t chunk = threadIdx.x / kWave;
  const uint32_t v = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  const bool live = g < w.G && t < dispatch_group_tokens(w, g);
  const uint32_t *idx = nullptr;
  bool bad_expert = false;
  if (live) {
    idx = w.drank[g * w.dp + t % w.dp].indices + (size_t)t * w.K;
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
  for (uint32_t e = threadIdx.x; e < w.E; e += blockDim.x) {
    uint32_t running = 0;
    for (uint32_t tile = 0; tile < blockIdx.x; ++tile) running += w.tile_cnt[(size_t)tile * w.E + e];
    for (uint32_t c = 0; c < chunks; ++c) {
      lds_base[c * w.E + e] = running;
      running += __popcll(lds_mask[(size_t)c * w.E + e]);
    }
    if (blockIdx.x == gridDim.x - 1) {
      // out_expert_num_tokens of the owning rank
      // (csrc/all_to_all/intranode_dispatch.cu:221 accumulates the same total).
      const DispatchRank &owner = w.drank[e / w.L];
      owner.out_num_tokens[(int64_t)(e % w.L) * owner.out_num_tokens_stride] = (int32_t)running;
    }
  }
  __syncthreads();

  if (live) {
    const unsigned long long below = (1ull << lane) - 1ull;
    uint32_t *out = w.slot_map + (size_t)v * w.K;
    for (uint32_t k = 0; k < w.K; ++k) {
      const uint32_t e = idx[k];
      uint32_t slot = kInvalidSlot;
      if (e < w.E) {
        slot = lds_base[chunk * w.E + e] + __popcll(lds_mask[(size_t)chunk * w.E + e] & below);
      }
      out[k] = slot;
    }
    if (bad_expert) atomicOr(w.faults, kFaultBadExpert);
  }
}

// ---------------------------------------------------------------------------
// Dispatch scatter.  A wave owns one token and picks [k0, k1) of it.  NV is the
// number of 16-byte vectors each lane keeps in registers (row <= NV * 1 KiB).
// ---------------------------------------------------------------------------
template <int NV>
__global__ __launch_bounds__(256) void dispatch_scatter(WorldDev w, uint32_t ksplit, uint32_t kper) {
  const uint32_t lane = lane_id();
  const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) +
                                                       threadIdx.x / kWave);
  const uint32_t v = wave / ksplit;
  const uint32_t part = wave - v * ksplit;
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  if (g >= w.G) return;
  if (t >= dispatch_group_tokens(w, g)) return;

  // The sender of token t inside its DP group (csrc/all_to_all/intranode_dispatch.cu:97).
  const DispatchRank &src = w.drank[g * w.dp + t % w.dp];
  const uint32_t nvec = w.Hb / 16;
  const u32x4 *row = reinterpret_cast<const u32x4 *>(src.dp_x + (int64_t)t * src.dp_x_stride_row);

  u32x4 x[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t j = lane + i * kWave;
    if (j < nvec) x[i] = row[j];
  }
  const uint32_t S = w.S;
  const float *srow = nullptr;
  float sc = 0.f;
  if (S) {
    srow = src.dp_xs + (int64_t)t * src.dp_xs_stride_row;
    if (lane < S) sc = srow[(int64_t)lane * src.dp_xs_stride_elem];
  }

  // Lane k resolves the destination of pick k.
  uint64_t dst_row = 0, dst_scale = 0;
  int64_t dst_scale_step = 0;
  if (lane < w.K) {
    const uint32_t e = src.indices[(size_t)t * w.K + lane];
    const uint32_t slot = w.slot_map[(size_t)v * w.K + lane];
    if (e < w.E && slot != kInvalidSlot) {
      const DispatchRank &dst = w.drank[e / w.L];
      const uint32_t el = e % w.L;
      if (slot < dst.x_rows) {
        dst_row = reinterpret_cast<uint64_t>(dst.expert_x + (int64_t)el * dst.x_stride_expert +
                                             (int64_t)slot * dst.x_stride_row);
        if (S) {
          dst_scale = reinterpret_cast<uint64_t>(dst.expert_xs + (int64_t)el * dst.xs_stride_expert +
                                                 (int64_t)slot * dst.xs_stride_row);
          dst_scale_step = dst.xs_stride_elem;
        }
      } else if (part == 0) {
        atomicOr(w.faults, kFaultRowDropped);
      }
    }
  }

  const uint32_t k0 = part * kper;
  const uint32_t k1 = (k0 + kper < w.K) ? k0 + kper : w.K;
  for (uint32_t k = k0; k < k1; ++k) {
    const uint64_t p = ((uint64_t)__builtin_amdgcn_readlane((uint32_t)(dst_row >> 32), k) << 32) |
                       (uint32_t)__builtin_amdgcn_readlane((uint32_t)dst_row, k);
    if (p == 0) continue;
    u32x4 *out = reinterpret_cast<u32x4 *>(p);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const uint32_t j = lane + i * kWave;
      if (j < nvec) __builtin_nontemporal_store(x[i], out + j);
    }
    if (S) {
      const uint64_t q = ((uint64_t)__builtin_amdgcn_readlane((uint32_t)(dst_scale >> 32), k) << 32) |
                         (uint32_t)__builtin_amdgcn_readlane((uint32_t)dst_scale, k);
      const uint64_t step64 =
          ((uint64_t)__builtin_amdgcn_readlane((uint32_t)((uint64_t)dst_scale_step >> 32), k) << 32) |
          (uint32_t)__builtin_amdgcn_readlane((uint32_t)dst_scale_step, k);
      float *sout = reinterpret_cast<float *>(q);
      const int64_t step = (int64_t)step64;
      if (lane < S) sout[(int64_t)lane * step] = sc;
      for (uint32_t j = lane + kWave; j < S; j += kWave) {
        sout[(int64_t)j * step] = srow[(int64_t)j * src.dp_xs_stride_elem];
      }
    }
  }
}

// Rows longer than the register variants cover: stream each vector K times.
__global__ __launch_bounds__(256) void dispatch_scatter_long(WorldDev w) {
  __shared__ uint64_t s_row[kWave];
  __shared__ uint64_t s_scale[kWave];
  __shared__ int64_t s_step[kWave];
  const uint32_t v = blockIdx.x;
  const uint32_t g = v / w.M;
  const uint32_t t = v - g * w.M;
  if (g >= w.G) return;
  if (t >= dispatch_group_tokens(w, g)) return;
  const DispatchRank &src = w.drank[g * w.dp + t % w.dp];
  if (threadIdx.x < w.K) {
    uint64_t dst_row = 0, dst_scale = 0;
    int64_t step = 0;
    const uint32_t e = src.indices[(size_t)t * w.K + threadIdx.x];
    const uint32_t slot = w.slot_map[(size_t)v * w.K + threadIdx.x];
    if (e < w.E && slot != kInvalidSlot) {
      const DispatchRank &dst = w.drank[e / w.L];
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
template <typename T> struct Load8;
template <> struct Load8<float> {
  static __device__ __forceinline__ f32x8 at(const void *row, uint32_t vec) {
    const f32x4 *p = reinterpret_cast<const f32x4 *>(row) + 2 * (size_t)vec;
    const f32x4 a = __builtin_nontemporal_load(p);
    const f32x4 b = __builtin_nontemporal_load(p + 1);
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
  }
};
template <> struct Load8<__bf16> {
  static __device__ __forceinline__ f32x8 at(const void *row, uint32_t vec) {
    const u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(row) + vec);
    f32x8 out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[2 * i] = __uint_as_float(raw[i] << 16);
      out[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
    }
    return out;
  }
};
template <> struct Load8<_Float16> {
  static __device__ __forceinline__ f32x8 at(const void *row, uint32_t vec) {
    const f16x8 raw = __builtin_nontemporal_load(reinterpret_cast<const f16x8 *>(row) + vec);
    return __builtin_convertvector(raw, f32x8);
  }
};

template <typename U> struct Store8;
template <> struct Store8<__bf16> {
  static __device__ __forceinline__ void at(void *row, uint32_t vec, const f32x8 &acc) {
    reinterpret_cast<bf16x8 *>(row)[vec] = __builtin_convertvector(acc, bf16x8);
  }
};
template <> struct Store8<_Float16> {
  static __device__ __forceinline__ void at(void *row, uint32_t vec, const f32x8 &acc) {
    reinterpret_cast<f16x8 *>(row)[vec] = __builtin_convertvector(acc, f16x8);
  }
};

template <typename T, typename U>
__global__ __launch_bounds__(256) void combine_gather(WorldDev w) {
  __shared__ uint64_t s_row[kWave];
  __shared__ float s_weight[kWave];

  const uint32_t r = blockIdx.x / w.M;
  const uint32_t t = blockIdx.x - r * w.M;
  const CombineRank &c = w.crank[r];
  if (t >= combine_rank_tokens(w, c)) return;

  if (threadIdx.x < w.K) {
    const uint32_t k = threadIdx.x;
    const uint32_t e = c.indices[(size_t)t * w.K + k];
    const uint32_t slot = w.slot_map[((size_t)(r / w.dp) * w.M + t) * w.K + k];
    uint64_t p = 0;
    if (e < w.E && slot != kInvalidSlot) {
      const CombineRank &owner = w.crank[e / w.L];
      if (slot < owner.y_rows) {
        p = reinterpret_cast<uint64_t>(reinterpret_cast<const T *>(owner.expert_y) +
                                       (int64_t)(e % w.L) * owner.y_stride_expert +
                                       (int64_t)slot * owner.y_stride_row);
      } else {
        atomicOr(w.faults, kFaultBadSlot);
      }
    }
    s_row[k] = p;
    s_weight[k] = c.weights[(int64_t)t * c.w_stride_row + k];
  }
  __syncthreads();

  U *out = reinterpret_cast<U *>(c.out_tokens) + (int64_t)t * c.out_stride_row;
  const uint32_t nvec = w.H / 8;
  for (uint32_t vec = threadIdx.x; vec < nvec; vec += blockDim.x) {
    f32x8 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
    for (uint32_t k = 0; k < w.K; ++k) {
      const uint64_t p = s_row[k];
      if (p == 0) continue;
      const float wk = s_weight[k];
      const f32x8 y = Load8<T>::at(reinterpret_cast<const void *>(p), vec);
      acc += wk * y;
    }
    Store8<U>::at(out, vec, acc);
  }
}

}  // namespace

// ---------------------------------------------------------------------------
// Launchers
// ---------------------------------------------------------------------------
uint32_t route_lds_bytes(uint32_t num_experts, uint32_t tile_chunks) {
  return tile_chunks * num_experts * (uint32_t)(sizeof(unsigned long long) + sizeof(uint32_t));
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

int launch_route(const WorldDev &w, void *stream) {
  const uint32_t block = w.tile_chunks * kWave;
  if (w.num_tiles > 1) {
    hipLaunchKernelGGL(route_count, dim3(w.num_tiles), dim3(block), w.E * sizeof(uint32_t),
                       (hipStream_t)stream, w);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return (int)err;
  }
  hipLaunchKernelGGL(route_slots, dim3(w.num_tiles), dim3(block),
                     route_lds_bytes(w.E, w.tile_chunks), (hipStream_t)stream, w);
  return (int)hipGetLastError();
}

int launch_dispatch_scatter(const WorldDev &w, void *stream) {
  const uint32_t tokens = w.G * w.M;
  const uint32_t per_lane = (w.Hb / 16 + kWave - 1) / kWave;
  if (per_lane > 32) {
    hipLaunchKernelGGL(dispatch_scatter_long, dim3(tokens), dim3(256), 0, (hipStream_t)stream, w);
    return (int)hipGetLastError();
  }
  // Few tokens: spread the K copies of a row over several waves so the launch
  // still covers the 256 CUs; the row re-reads hit L2.
  uint32_t ksplit = 1;
  while (ksplit < w.K && (uint64_t)tokens * ksplit < 16384) ksplit *= 2;
  if (ksplit > w.K) ksplit = w.K;
  const uint32_t kper = (w.K + ksplit - 1) / ksplit;
  const uint64_t waves = (uint64_t)tokens * ksplit;
  const dim3 grid((uint32_t)((waves + 3) / 4)), block(256);
  hipStream_t s = (hipStream_t)stream;
  if (per_lane <= 1) {
    hipLaunchKernelGGL(dispatch_scatter<1>, grid, block, 0, s, w, ksplit, kper);
  } else if (per_lane <= 2) {
    hipLaunchKernelGGL(dispatch_scatter<2>, grid, block, 0, s, w, ksplit, kper);
  } else if (per_lane <= 4) {
    hipLaunchKernelGGL(dispatch_scatter<4>, grid, block, 0, s, w, ksplit, kper);
  } else if (per_lane <= 8) {
    hipLaunchKernelGGL(dispatch_scatter<8>, grid, block, 0, s, w, ksplit, kper);
  } else if (per_lane <= 16) {
    hipLaunchKernelGGL(dispatch_scatter<16>, grid, block, 0, s, w, ksplit, kper);
  } else {
    hipLaunchKernelGGL(dispatch_scatter<32>, grid, block, 0, s, w, ksplit, kper);
  }
  return (int)hipGetLastError();
}

int launch_combine_gather(const WorldDev &w, int in_dtype, int out_dtype, void *stream) {
  const dim3 grid(w.R * w.M), block(256);
  hipStream_t s = (hipStream_t)stream;
  // dtype codes follow pplx_a2a_dtype: 0 = f32, 1 = bf16, 2 = f16.
  switch (in_dtype * 4 + out_dtype) {
    case 0 * 4 + 1: hipLaunchKernelGGL((combine_gather<float, __bf16>), grid, block, 0, s, w); break;
    case 0 * 4 + 2: hipLaunchKernelGGL((combine_gather<float, _Float16>), grid, block, 0, s, w); break;
    case 1 * 4 + 1: hipLaunchKernelGGL((combine_gather<__bf16, __bf16>), grid, block, 0, s, w); break;
    case 1 * 4 + 2: hipLaunchKernelGGL((combine_gather<__bf16, _Float16>), grid, block, 0, s, w); break;
    case 2 * 4 + 1: hipLaunchKernelGGL((combine_gather<_Float16, __bf16>), grid, block, 0, s, w); break;
    case 2 * 4 + 2: hipLaunchKernelGGL((combine_gather<_Float16, _Float16>), grid, block, 0, s, w); break;
    default: return (int)hipErrorInvalidValue;
  }
  return (int)hipGetLastError();
}

}  // namespace pplx_amd
