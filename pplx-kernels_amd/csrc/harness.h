// Shared pieces of the torch-free C++ test and benchmark binaries.  They use nothing but
// include/pplx_a2a.h and the HIP runtime, the way a native caller of the library would.
// All simulated ranks live in this one process (the reference's harness launches one MPI
// process per GPU: csrc/all_to_all/test_all_to_all.cpp:338-394).
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "pplx_a2a.h"

#define HIP_OK(expr)                                                                      \
  do {                                                                                    \
    hipError_t err_ = (expr);                                                             \
    if (err_ != hipSuccess) {                                                             \
      fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(err_)); \
      exit(2);                                                                            \
    }                                                                                     \
  } while (0)

#define A2A_OK(expr)                                                                      \
  do {                                                                                    \
    int st_ = (expr);                                                                     \
    if (st_ != PPLX_A2A_OK) {                                                             \
      fprintf(stderr, "%s:%d %s -> %d: %s\n", __FILE__, __LINE__, #expr, st_, pplx_a2a_last_error()); \
      exit(2);                                                                            \
    }                                                                                     \
  } while (0)

namespace harness {

inline uint16_t float_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

inline float bf16_to_float(uint16_t h) {
  const uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

template <typename T>
T *device_alloc(size_t count) {
  T *p = nullptr;
  HIP_OK(hipMalloc(reinterpret_cast<void **>(&p), count * sizeof(T) + 16));
  HIP_OK(hipMemset(p, 0, count * sizeof(T) + 16));
  return p;
}

template <typename T>
T *device_copy(const std::vector<T> &host) {
  T *p = device_alloc<T>(host.size());
  if (!host.empty()) HIP_OK(hipMemcpy(p, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
  return p;
}

template <typename T>
std::vector<T> host_copy(const T *dev, size_t count) {
  std::vector<T> out(count);
  if (count) HIP_OK(hipMemcpy(out.data(), dev, count * sizeof(T), hipMemcpyDeviceToHost));
  return out;
}

// One DP group's inputs: m tokens, K distinct experts each, weights in [0, 1), row bytes of
// `elem` bytes per element and `scale_dim` fp32 scales per token.
struct GroupData {
  uint32_t m = 0;
  std::vector<uint32_t> indices;  // [m][K]
  std::vector<float> weights;     // [m][K]
  std::vector<float> x;           // [m][H] values (exactly representable in bf16)
  std::vector<float> x_scale;     // [m][scale_dim]
};

inline GroupData make_group(std::mt19937 &gen, uint32_t min_tokens, uint32_t max_tokens, uint32_t E,
                            uint32_t K, uint32_t H, uint32_t scale_dim) {
  GroupData g;
  g.m = min_tokens + gen() % (max_tokens - min_tokens + 1);
  std::vector<uint32_t> perm(E);
  std::uniform_real_distribution<float> unit(0.f, 1.f);
  for (uint32_t t = 0; t < g.m; ++t) {
    for (uint32_t e = 0; e < E; ++e) perm[e] = e;
    for (uint32_t k = 0; k < K; ++k) {  // partial Fisher-Yates: K distinct experts
      const uint32_t j = k + gen() % (E - k);
      std::swap(perm[k], perm[j]);
      g.indices.push_back(perm[k]);
      g.weights.push_back(unit(gen));
    }
    for (uint32_t h = 0; h < H; ++h) g.x.push_back(bf16_to_float(float_to_bf16(unit(gen) * 4.f - 2.f)));
    for (uint32_t s = 0; s < scale_dim; ++s) g.x_scale.push_back(unit(gen));
  }
  return g;
}

}  // namespace harness
