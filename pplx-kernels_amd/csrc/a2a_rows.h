// Row fan-out in registers, shared by the dispatch kernels, and the macro that picks the register variant for a row size.
#pragma once
#include "a2a_common.h"

namespace pplx_amd {
namespace {

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
  const PPLX_GLOBAL u32x4 *row =
      as_global(reinterpret_cast<const u32x4 *>(src.dp_x + (int64_t)t * src.dp_x_stride_row));
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    uint32_t j = lane + i * kWave;
    if (!EXACT) j = j < nvec ? j : nvec - 1;  // clamp: loads stay unconditional
    regs.x[i] = row[j];
  }
  regs.sc = 0.f;
  if (w.S) {
    const uint32_t j = lane < w.S ? lane : w.S - 1;
    regs.sc = as_global(src.dp_xs)[(int64_t)t * src.dp_xs_stride_row + (int64_t)j * src.dp_xs_stride_elem];
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
    const DispatchRank &dst = tab.at(owner_of(w, e));
    const uint32_t el = local_of(w, e);
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
template <int NV, bool EXACT, RowStore POLICY = RowStore::kStream, RowStore SCALE_POLICY = POLICY>
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
      if (EXACT || j < nvec) row_store<POLICY>(regs.x[i], out + j);
    }
    if (S) {
      PPLX_GLOBAL float *sout = global_ptr<float>(read_lane64(dst.scale, k));
      const int64_t step = (int64_t)read_lane64((uint64_t)dst.scale_step, k);
      if (lane < S) row_store<SCALE_POLICY>(regs.sc, sout + (int64_t)lane * step);
      if (S > kWave) {
        const PPLX_GLOBAL float *srow = as_global(src.dp_xs) + (int64_t)t * src.dp_xs_stride_row;
        for (uint32_t j = lane + kWave; j < S; j += kWave) {
          sout[(int64_t)j * step] = srow[(int64_t)j * src.dp_xs_stride_elem];
        }
      }
    }
  }
}

}  // namespace
}  // namespace pplx_amd

namespace pplx_amd {
namespace {
// Rows of up to 8 KiB and rows of exactly 10, 12, 14 or 16 KiB (5120-, 6144-, 7168- and 8192-wide
// bf16) have a register variant in every row kernel; other sizes beyond 8 KiB take
// dispatch_scatter's padded variants or the streaming kernels.
inline bool row_has_register_variant(const WorldDev &w) {
  const uint32_t nvec = w.Hb / 16;
  const uint32_t per_lane = (nvec + kWave - 1) / kWave;
  const bool exact = nvec % kWave == 0;
  return per_lane <= 8 || (exact && (per_lane == 10 || per_lane == 12 || per_lane == 14 || per_lane == 16));
}
}  // namespace
}  // namespace pplx_amd

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
    else if (exact && per_lane == 10) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 10, true);                 \
    else if (exact && per_lane == 12) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 12, true);                 \
    else if (exact && per_lane == 14) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 14, true);                 \
    else if (exact && per_lane == 16) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 16, true);                 \
    else if (per_lane <= 1) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 1, false);                           \
    else if (per_lane <= 2) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 2, false);                           \
    else if (per_lane <= 4) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 4, false);                           \
    else if (per_lane <= 8) PPLX_LAUNCH_ROW_VARIANT(KERNEL, 8, false);                           \
    else PPLX_LAUNCH_LARGE_ROW_VARIANT(KERNEL);                                                  \
  } while (0)
