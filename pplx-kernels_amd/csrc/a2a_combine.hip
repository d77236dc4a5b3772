// gfx950 combine kernel of the MoE dispatch / combine path: the top-k weighted
// gather-reduce (also the SEND phase of a split combine, with its output rows in the staging area).
#include "a2a_common.h"

namespace pplx_amd {
namespace {

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
    __builtin_nontemporal_store(__builtin_convertvector(acc, bf16x8),
                                as_global(reinterpret_cast<bf16x8 *>(row)) + vec);
  }
};
template <> struct Store8<_Float16> {
  static __device__ __forceinline__ void at(void *row, uint32_t vec, const f32x8 &acc) {
    __builtin_nontemporal_store(__builtin_convertvector(acc, f16x8),
                                as_global(reinterpret_cast<f16x8 *>(row)) + vec);
  }
};

// N picks starting at k, VPL vectors of each: all N * VPL loads are issued before the first is used.
template <typename T, int N, int VPL>
__device__ __forceinline__ void gather_group(f32x8 (&acc)[VPL], uint64_t row_of_lane, float weight_of_lane,
                                             uint32_t k, const uint32_t (&vec)[VPL]) {
  typename Row8<T>::Raw raw[VPL][N];
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
#pragma unroll
    for (int i = 0; i < N; ++i) raw[v][i] = Row8<T>::load(read_lane64(row_of_lane, k + i), vec[v]);
  }
  Row8<T>::template settle<VPL * N>(&raw[0][0]);
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float wk = __builtin_bit_cast(
        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, weight_of_lane), (int)(k + i)));
#pragma unroll
    for (int v = 0; v < VPL; ++v) acc[v] += wk * Row8<T>::widen(raw[v][i]);
  }
}

// One wave owns VPL * 64 consecutive 8-element vectors of one output row (VPL KiB of a bf16
// row) and takes the picks KB at a time, so KB * VPL row loads per lane are in flight: few
// picks read long pieces of their rows, many picks shorter ones.
template <typename T, typename U, class CT, int KB, int VPL>
__global__ __launch_bounds__(256) void combine_gather(WorldDev w, CT tab, uint32_t segments, FastDiv by_segments,
                                                      uint32_t first_rank, uint32_t rank_count) {
  const uint32_t lane = lane_id();
  const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x / kWave) +
                                                       threadIdx.x / kWave);
  const uint32_t token = fast_div(wave, by_segments);
  const uint32_t segment = wave - token * segments;
  const uint32_t r_local = group_of(w, token);
  const uint32_t t = token - r_local * w.M;
  if (r_local >= rank_count) return;
  const uint32_t r = first_rank + r_local;
  const CombineRank &c = tab.at(r);
  if (t >= combine_rank_tokens(w, c)) return;

  // Lane k resolves pick k: no LDS, no barrier.
  uint64_t row = 0;
  float weight = 0.f;
  if (lane < w.K) {
    const uint32_t e = as_global(c.indices)[(size_t)t * w.K + lane];
    const uint32_t slot = as_global(w.slot_map)[((size_t)fast_div(r, w.by_dp) * w.M + t) * w.K + lane];
    weight = as_global(c.weights)[(int64_t)t * c.w_stride_row + lane];
    if (e < w.E && slot != kInvalidSlot) {
      const CombineRank &owner = tab.at(owner_of(w, e));
      if (slot < owner.y_rows) {
        row = reinterpret_cast<uint64_t>(reinterpret_cast<const T *>(owner.expert_y) +
                                         (int64_t)local_of(w, e) * owner.y_stride_expert +
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
      const uint32_t one[1] = {vec < nvec ? vec : nvec - 1};
      f32x8 acc[1] = {{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}};
      for (uint32_t k = 0; k < K; ++k) {
        if (read_lane64(row, k) != 0) gather_group<T, 1, 1>(acc, row, weight, k, one);
      }
      if (vec < nvec) Store8<U>::at(out, vec, acc[0]);
    }
    return;
  }
  uint32_t vec_ld[VPL];
  f32x8 acc[VPL];
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const uint32_t vec = (segment * VPL + v) * kWave + lane;
    vec_ld[v] = vec < nvec ? vec : nvec - 1;  // clamp: loads stay unconditional
    acc[v] = f32x8{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  }
  uint32_t k = 0;
  for (; k + KB <= K; k += KB) gather_group<T, KB, VPL>(acc, row, weight, k, vec_ld);
  if constexpr (KB > 4) {
    if ((K - k) & 4) { gather_group<T, 4, VPL>(acc, row, weight, k, vec_ld); k += 4; }
  }
  if constexpr (KB > 2) {
    if ((K - k) & 2) { gather_group<T, 2, VPL>(acc, row, weight, k, vec_ld); k += 2; }
  }
  if constexpr (KB > 1) {
    if ((K - k) & 1) { gather_group<T, 1, VPL>(acc, row, weight, k, vec_ld); }
  }
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const uint32_t vec = (segment * VPL + v) * kWave + lane;
    if (vec < nvec) Store8<U>::at(out, vec, acc[v]);
  }
}

template <typename T, typename U, class CT, int KB, int VPL>
int launch_combine_v(const WorldDev &w, const CT &tab, uint32_t first_rank, uint32_t rank_count, hipStream_t s) {
  const uint32_t nvec_segments = (w.H / 8 + kWave - 1) / kWave;
  const uint32_t segments = (nvec_segments + VPL - 1) / VPL;
  const uint64_t waves = (uint64_t)rank_count * w.M * segments;
  const dim3 grid((uint32_t)((waves + 3) / 4)), block(256);
  hipLaunchKernelGGL((combine_gather<T, U, CT, KB, VPL>), grid, block, 0, s, w, tab, segments,
                     make_fast_div(segments), first_rank, rank_count);
  return (int)hipGetLastError();
}

template <typename T, typename U, class CT>
int launch_combine_k(const WorldDev &w, const CT &tab, uint32_t first_rank, uint32_t rank_count, hipStream_t s) {
#define PPLX_COMBINE(KB, VPL) \
  return launch_combine_v<T, U, CT, KB, VPL>(w, tab, first_rank, rank_count, s)
  // Few picks: long pieces of each row, all picks at once.  Many picks: all of them at once,
  // 1 KiB of each (eight loads per lane in flight either way) -- except for steps of a few
  // hundred to two thousand tokens, whose waves are all resident at the same moment: there the
  // picks are better taken one after the other in 7 or 8 KiB pieces by a quarter as many waves
  // (8 x 128 DSv3 tokens, top-8: 23.4 us against 25.3 us; 8 x 256: 45.8 against 46.8; from
  // 8 x 512 on the wide form wins, 88.7 against 91.5 us, and below 8 x 64 too).
  const uint32_t nvec_segments = (w.H / 8 + kWave - 1) / kWave;
  const uint64_t tokens = (uint64_t)rank_count * w.M;
  if (w.K > 4 && tokens > 384 && tokens <= 2048 && nvec_segments >= 7) {
    if (nvec_segments % 7 == 0) PPLX_COMBINE(1, 7);
    PPLX_COMBINE(1, 8);
  }
  switch (w.K) {
    case 1: PPLX_COMBINE(1, 8);
    case 2: PPLX_COMBINE(2, 4);
    case 4: PPLX_COMBINE(4, 2);
    default: PPLX_COMBINE(8, 1);
  }
#undef PPLX_COMBINE
}

template <class CT>
int launch_combine_t(const WorldDev &w, const CT &tab, int in_dtype, int out_dtype, hipStream_t s,
                     uint32_t first_rank, uint32_t rank_count) {
  // dtype codes follow pplx_a2a_dtype: 0 = f32, 1 = bf16, 2 = f16.
  switch (in_dtype * 4 + out_dtype) {
    case 0 * 4 + 1: return launch_combine_k<float, __bf16>(w, tab, first_rank, rank_count, s);
    case 0 * 4 + 2: return launch_combine_k<float, _Float16>(w, tab, first_rank, rank_count, s);
    case 1 * 4 + 1: return launch_combine_k<__bf16, __bf16>(w, tab, first_rank, rank_count, s);
    case 1 * 4 + 2: return launch_combine_k<__bf16, _Float16>(w, tab, first_rank, rank_count, s);
    case 2 * 4 + 1: return launch_combine_k<_Float16, __bf16>(w, tab, first_rank, rank_count, s);
    case 2 * 4 + 2: return launch_combine_k<_Float16, _Float16>(w, tab, first_rank, rank_count, s);
    default: return (int)hipErrorInvalidValue;
  }
}

}  // namespace

int launch_combine(const WorldDev &w, const CombineRank *inline_rows, int in_dtype, int out_dtype,
                   void *stream) {
  if (inline_rows)
    return launch_combine_t(w, make_inline(w, inline_rows), in_dtype, out_dtype, (hipStream_t)stream, 0, w.R);
  return launch_combine_t(w, HbmCombine{w.crank}, in_dtype, out_dtype, (hipStream_t)stream, 0, w.R);
}

}  // namespace pplx_amd
