/*
 * a2a_oracle.c -- CPU restatement of the reference's MoE dispatch / combine.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the HIP path is
 * compared against; nothing in the product (the pplx_kernels package and its
 * libpplx_kernels.so) links, loads or calls it.  It may be used by tests/, by
 * __graft_entry__.smoke() and by bench.py's cpu_baseline leg.
 *
 * What it restates (paths relative to the reference tree):
 *   oracle_dispatch  routing order and outputs as enumerated by the reference's
 *                    own torch check, tests/test_all_to_all.py:113-120 (append
 *                    (dp_rank, token) per expert, dp_rank ascending then token
 *                    ascending), with owner/local-expert split of
 *                    csrc/all_to_all/intranode_dispatch.cu:133-134, the
 *                    bound_m rule of csrc/all_to_all/intranode_dispatch.cu:64,
 *                    and row + scale copies of :252-275.
 *   oracle_combine   csrc/all_to_all/intranode_combine.cu:141-168: fp32
 *                    accumulation, picks in ascending k, float -> out dtype by
 *                    round-to-nearest-even on the final store.
 *
 * The reference's native code is CUDA + NVSHMEM and cannot be built in this
 * image, so there is no oracle/_ref; this restatement is pinned by
 * tests/test_oracle.py (closed forms, a literal Python loop, committed golden
 * vectors, special cases) instead.
 *
 * Layout: all simulated ranks' expert-major buffers are one array indexed by
 * GLOBAL expert, [E][cap][...]; rank r owns experts r*L .. r*L+L-1.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

enum { ORACLE_F32 = 0, ORACLE_BF16 = 1, ORACLE_F16 = 2 };

static float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

static float bf16_to_float(uint16_t h) { return bits_to_float((uint32_t)h << 16); }

/* IEEE binary32 -> bfloat16, round to nearest even, NaN stays quiet NaN. */
static uint16_t float_to_bf16(float f) {
  uint32_t u = float_to_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static float f16_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_to_float(sign);
    /* subnormal: normalise */
    exp = 1;
    while (!(man & 0x400u)) {
      man <<= 1;
      exp--;
    }
    man &= 0x3ffu;
    return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
  }
  if (exp == 31) return bits_to_float(sign | 0x7f800000u | (man << 13));
  return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

/* IEEE binary32 -> binary16, round to nearest even. */
static uint16_t float_to_f16(float f) {
  const uint32_t u = float_to_bits(f);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t abs = u & 0x7fffffffu;
  if (abs > 0x7f800000u) return (uint16_t)(sign | 0x7e00u); /* NaN */
  if (abs >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* overflow -> inf (also inf) */
  if (abs < 0x33000000u) return sign;                       /* < 2^-25 -> 0 */
  int32_t exp = (int32_t)(abs >> 23) - 127;
  uint32_t man = (abs & 0x7fffffu) | 0x800000u;
  uint32_t shift;
  uint32_t half_exp;
  if (exp < -14) { /* subnormal result */
    shift = (uint32_t)(13 + (-14 - exp));
    half_exp = 0;
  } else {
    shift = 13;
    half_exp = (uint32_t)(exp + 15);
  }
  uint32_t q = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1u);
  const uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) q++;
  uint32_t out;
  if (half_exp == 0) {
    out = q; /* may carry into exponent 1: still the right encoding */
  } else {
    out = ((half_exp - 1) << 10) + q; /* q carries the implicit one at bit 10 */
  }
  if (out >= 0x7c00u) out = 0x7c00u;
  return (uint16_t)(sign | out);
}

/*
 * Dispatch for every DP group at once.
 *   G groups, each with n_tokens[g] live tokens (already min(bound_m, m)).
 *   dp_x[g]      row t at dp_x[g] + t * dp_x_stride[g] bytes, Hb bytes per row
 *   dp_xs[g]     row t at dp_xs[g] + t * S floats (NULL when S == 0)
 *   indices[g]   [m_g][K] expert ids
 * Outputs
 *   counts[E]            tokens per global expert
 *   expert_x [E][cap][Hb], expert_xs [E][cap][S]   rows beyond counts[e] untouched
 *   slot_map [G][M][K]   row of (g, t, k) inside its expert; untouched for t >= n
 * Returns 0, or 1 if an expert id is out of range, or 2 if a row did not fit cap.
 */
int oracle_dispatch(uint32_t G, uint32_t M, uint32_t E, uint32_t K, uint64_t Hb, uint32_t S,
                    const uint8_t *const *dp_x, const int64_t *dp_x_stride,
                    const float *const *dp_xs, const uint32_t *const *indices,
                    const uint32_t *n_tokens, int32_t *counts, uint8_t *expert_x,
                    float *expert_xs, int64_t cap, uint32_t *slot_map) {
  for (uint32_t e = 0; e < E; ++e) counts[e] = 0;
  for (uint32_t g = 0; g < G; ++g) {
    for (uint32_t t = 0; t < n_tokens[g]; ++t) {
      for (uint32_t k = 0; k < K; ++k) {
        const uint32_t e = indices[g][(size_t)t * K + k];
        if (e >= E) return 1;
        const int64_t slot = counts[e]++;
        if (slot >= cap) return 2;
        memcpy(expert_x + ((size_t)e * cap + slot) * Hb, dp_x[g] + (int64_t)t * dp_x_stride[g], Hb);
        if (S) {
          memcpy(expert_xs + ((size_t)e * cap + slot) * S, dp_xs[g] + (size_t)t * S,
                 (size_t)S * sizeof(float));
        }
        slot_map[((size_t)g * M + t) * K + k] = (uint32_t)slot;
      }
    }
  }
  return 0;
}

static float load_as_float(const void *base, size_t i, int dtype) {
  switch (dtype) {
    case ORACLE_F32: return ((const float *)base)[i];
    case ORACLE_BF16: return bf16_to_float(((const uint16_t *)base)[i]);
    default: return f16_to_float(((const uint16_t *)base)[i]);
  }
}

/*
 * Combine for every DP group at once.
 *   expert_y [E][cap][H] of in_dtype; out_tokens[g] is [>= n_tokens[g]][H] of
 *   out_dtype (contiguous rows); rows >= n_tokens[g] are not touched.
 * Compile with -ffp-contract=off: the sum is a separate multiply and add per
 * pick, in ascending k.
 */
int oracle_combine(uint32_t G, uint32_t M, uint32_t E, uint32_t K, uint32_t H, int in_dtype,
                   int out_dtype, const void *expert_y, int64_t cap,
                   const uint32_t *const *indices, const float *const *weights,
                   const uint32_t *n_tokens, const uint32_t *slot_map, void *const *out_tokens) {
  if (out_dtype != ORACLE_BF16 && out_dtype != ORACLE_F16) return 3;
  for (uint32_t g = 0; g < G; ++g) {
    for (uint32_t t = 0; t < n_tokens[g]; ++t) {
      uint16_t *out = (uint16_t *)out_tokens[g] + (size_t)t * H;
      for (uint32_t j = 0; j < H; ++j) {
        float sum = 0.0f;
        for (uint32_t k = 0; k < K; ++k) {
          const uint32_t e = indices[g][(size_t)t * K + k];
          if (e >= E) return 1;
          const uint32_t slot = slot_map[((size_t)g * M + t) * K + k];
          if ((int64_t)slot >= cap) return 2;
          const float w = weights[g][(size_t)t * K + k];
          const float y = load_as_float(expert_y, ((size_t)e * cap + slot) * H + j, in_dtype);
          sum += w * y;
        }
        out[j] = out_dtype == ORACLE_BF16 ? float_to_bf16(sum) : float_to_f16(sum);
      }
    }
  }
  return 0;
}

/* Exposed so the conversions themselves can be pinned against a library. */
uint16_t oracle_float_to_bf16(float f) { return float_to_bf16(f); }
uint16_t oracle_float_to_f16(float f) { return float_to_f16(f); }
float oracle_f16_to_float(uint16_t h) { return f16_to_float(h); }
float oracle_bf16_to_float(uint16_t h) { return bf16_to_float(h); }
