// Torch-free correctness test of the C ABI: every simulated rank in this process, checks
// against an expectation computed on the host.
//
// Counterpart of the reference's csrc/all_to_all/test_all_to_all.cpp:46-336, whose first
// geometry (8 experts, top-3, hidden 16, 5..10 tokens, block size 2, T in {float, bf16},
// 4 ranks in 2 DP groups) is case 1 here.  The checks are the reference's (expected count per
// expert :248-256, every routed row present with its scales :258-305, combine result within
// 0.5 of sum_k w_k * x :309-327) made stricter: rows must sit at their canonical position
// (DP group ascending, then token) and the combine must also be within rtol 1e-2 / atol 1e-2.
#include <algorithm>
#include <cmath>
#include <string>

#include "a2a_device.h"
#include "harness.h"

using namespace harness;

namespace {

enum Mode { PER_RANK, WORLD, SPLIT };
const char *mode_name(Mode m) { return m == PER_RANK ? "per-rank" : m == WORLD ? "world" : "split send/recv"; }

struct Geometry {
  const char *name;
  uint32_t R, dp, E, K, H, M, min_tokens;
  uint32_t elem;       // bytes per element of the dispatched row: 4 float, 2 bf16, 1 opaque bytes
  uint32_t scale_dim;  // fp32 scales per token (0 = none)
  bool use_bound_m;
};

struct RankBuffers {
  int32_t *counts;
  uint8_t *expert_x;
  float *expert_xs;
  uint16_t *expert_y;  // bf16 rows handed to combine when the dispatched rows are opaque bytes
  uint8_t *dp_x;
  float *dp_xs;
  uint32_t *indices;
  float *weights;
  uint32_t *bound_m;
  uint16_t *out_tokens;
};

std::vector<uint8_t> encode_rows(const GroupData &g, uint32_t H, uint32_t elem, uint32_t rows) {
  std::vector<uint8_t> bytes((size_t)rows * H * elem, 0);
  for (size_t i = 0; i < (size_t)g.m * H; ++i) {
    if (elem == 4) {
      memcpy(&bytes[i * 4], &g.x[i], 4);
    } else if (elem == 2) {
      const uint16_t b = float_to_bf16(g.x[i]);
      memcpy(&bytes[i * 2], &b, 2);
    } else {
      uint32_t u;
      memcpy(&u, &g.x[i], 4);
      bytes[i] = (uint8_t)((u >> 13) ^ (u >> 21) ^ i);  // opaque payload byte
    }
  }
  return bytes;
}

bool run_case(const Geometry &geo, Mode mode, hipStream_t stream) {
  const uint32_t G = geo.R / geo.dp, L = geo.E / geo.R, cap = geo.M * G;
  const size_t Hb = (size_t)geo.H * geo.elem;
  std::mt19937 gen(0xdeadbeef);
  std::vector<GroupData> groups;
  for (uint32_t g = 0; g < G; ++g)
    groups.push_back(make_group(gen, geo.min_tokens, geo.M, geo.E, geo.K, geo.H, geo.scale_dim));

  // Expected placement: expert e receives (g, t) in group-then-token order.
  std::vector<std::vector<std::pair<uint32_t, uint32_t>>> expected(geo.E);
  for (uint32_t g = 0; g < G; ++g)
    for (uint32_t t = 0; t < groups[g].m; ++t)
      for (uint32_t k = 0; k < geo.K; ++k) expected[groups[g].indices[(size_t)t * geo.K + k]].push_back({g, t});

  pplx_a2a_config_t cfg{};
  cfg.max_num_tokens = geo.M;
  cfg.num_experts = geo.E;
  cfg.experts_per_token = geo.K;
  cfg.world_size = geo.R;
  cfg.dp_size = geo.dp;
  cfg.hidden_dim = geo.H;
  cfg.hidden_dim_bytes = Hb;
  cfg.hidden_dim_scale_bytes = geo.scale_dim * 4;
  pplx_a2a_world_t *world = nullptr;
  A2A_OK(pplx_a2a_world_create(&cfg, 0, &world));
  std::vector<pplx_a2a_t *> ranks(geo.R);
  for (uint32_t r = 0; r < geo.R; ++r) A2A_OK(pplx_a2a_create(world, r, &ranks[r]));

  const bool separate_y = geo.elem == 1;  // opaque rows cannot feed combine; use bf16 rows
  const int y_dtype = geo.elem == 4 ? PPLX_A2A_F32 : PPLX_A2A_BF16;
  std::vector<RankBuffers> buf(geo.R);
  std::vector<std::vector<uint8_t>> rows_of_group(G);
  for (uint32_t g = 0; g < G; ++g) rows_of_group[g] = encode_rows(groups[g], geo.H, geo.elem, geo.M);
  for (uint32_t r = 0; r < geo.R; ++r) {
    const GroupData &g = groups[r / geo.dp];
    RankBuffers &b = buf[r];
    b.counts = device_alloc<int32_t>(L);
    b.expert_x = device_alloc<uint8_t>((size_t)L * cap * Hb);
    b.expert_xs = geo.scale_dim ? device_alloc<float>((size_t)L * cap * geo.scale_dim) : nullptr;
    b.expert_y = separate_y ? device_alloc<uint16_t>((size_t)L * cap * geo.H) : nullptr;
    b.dp_x = device_copy(rows_of_group[r / geo.dp]);
    std::vector<float> xs((size_t)geo.M * geo.scale_dim, 0.f);
    std::copy(g.x_scale.begin(), g.x_scale.end(), xs.begin());
    b.dp_xs = geo.scale_dim ? device_copy(xs) : nullptr;
    std::vector<uint32_t> idx((size_t)geo.M * geo.K, 0);
    std::copy(g.indices.begin(), g.indices.end(), idx.begin());
    b.indices = device_copy(idx);
    std::vector<float> wts((size_t)geo.M * geo.K, 0.f);
    std::copy(g.weights.begin(), g.weights.end(), wts.begin());
    b.weights = device_copy(wts);
    b.bound_m = geo.use_bound_m ? device_copy(std::vector<uint32_t>{g.m}) : nullptr;
    b.out_tokens = device_copy(std::vector<uint16_t>((size_t)geo.M * geo.H, 0x7fc0));  // bf16 NaN
  }

  auto dispatch_args = [&](uint32_t r) {
    const RankBuffers &b = buf[r];
    pplx_a2a_dispatch_args_t a{};
    a.out_expert_num_tokens = b.counts;
    a.out_expert_num_tokens_stride = 1;
    a.out_expert_x = b.expert_x;
    a.out_expert_x_stride_row = (int64_t)Hb;
    a.out_expert_x_stride_expert = (int64_t)Hb * cap;
    a.out_expert_x_rows = cap;
    a.out_expert_x_scale = b.expert_xs;
    a.out_expert_x_scale_stride_elem = 1;
    a.out_expert_x_scale_stride_row = geo.scale_dim;
    a.out_expert_x_scale_stride_expert = (int64_t)geo.scale_dim * cap;
    a.dp_x = b.dp_x;
    a.dp_x_stride_row = (int64_t)Hb;
    a.dp_x_scale = b.dp_xs;
    a.dp_x_scale_stride_elem = 1;
    a.dp_x_scale_stride_row = geo.scale_dim;
    a.indices = b.indices;
    a.m = geo.use_bound_m ? geo.M : groups[r / geo.dp].m;
    a.bound_m = b.bound_m;
    return a;
  };
  auto combine_args = [&](uint32_t r) {
    const RankBuffers &b = buf[r];
    pplx_a2a_combine_args_t a{};
    a.out_tokens = b.out_tokens;
    a.out_tokens_stride_row = geo.H;
    a.out_dtype = PPLX_A2A_BF16;
    a.indices = b.indices;
    a.weights = b.weights;
    a.weights_stride_row = geo.K;
    a.expert_y = separate_y ? (const void *)b.expert_y : (const void *)b.expert_x;
    a.expert_y_stride_row = geo.H;
    a.expert_y_stride_expert = (int64_t)geo.H * cap;
    a.expert_y_rows = cap;
    a.in_dtype = y_dtype;
    a.m = geo.use_bound_m ? geo.M : groups[r / geo.dp].m;
    a.bound_m = b.bound_m;
    return a;
  };

  // ---- dispatch
  if (mode == WORLD) {
    std::vector<pplx_a2a_dispatch_args_t> all;
    for (uint32_t r = 0; r < geo.R; ++r) all.push_back(dispatch_args(r));
    A2A_OK(pplx_a2a_world_dispatch(world, all.data(), stream));
  } else if (mode == PER_RANK) {
    // A step that stops half way (all ranks but the last have called) is given up: the world is
    // idle again, nothing ran, and the whole step is made from the first rank on.
    {
      uint32_t recorded = 0, dropped = 0;
      for (uint32_t r = 0; r + 1 < geo.R; ++r) {
        auto a = dispatch_args(r);
        A2A_OK(pplx_a2a_dispatch(ranks[r], &a, PPLX_A2A_SPLIT_NONE, stream));
      }
      A2A_OK(pplx_a2a_world_recorded_calls(world, 0, PPLX_A2A_SPLIT_NONE, &recorded));
      auto again = dispatch_args(0);
      const int twice = pplx_a2a_dispatch(ranks[0], &again, PPLX_A2A_SPLIT_NONE, stream);
      A2A_OK(pplx_a2a_world_abandon_step(world, PPLX_A2A_ABANDON_DISPATCH | PPLX_A2A_ABANDON_COMBINE, &dropped));
      uint32_t after = ~0u;
      A2A_OK(pplx_a2a_world_recorded_calls(world, 0, PPLX_A2A_SPLIT_NONE, &after));
      if (recorded != geo.R - 1 || twice != PPLX_A2A_INVALID_STATE || dropped != geo.R - 1 || after != 0 ||
          pplx_a2a_world_abandon_step(world, 0, nullptr) != PPLX_A2A_INVALID_ARGUMENT) {
        printf("  FAIL %s [%s]: abandon: recorded %u, second call %d, dropped %u, left %u\n", geo.name,
               mode_name(mode), recorded, twice, dropped, after);
        return false;
      }
    }
    for (uint32_t r = 0; r < geo.R; ++r) {
      auto a = dispatch_args(r);
      A2A_OK(pplx_a2a_dispatch(ranks[r], &a, PPLX_A2A_SPLIT_NONE, stream));
    }
  } else {
    // dispatch / combine never allocate: a split call on a world without staging is refused
    {
      auto a = dispatch_args(0);
      if (pplx_a2a_dispatch(ranks[0], &a, PPLX_A2A_SPLIT_SEND, stream) != PPLX_A2A_INVALID_STATE) {
        printf("  FAIL %s [%s]: split call accepted without reserved staging\n", geo.name, mode_name(mode));
        return false;
      }
      A2A_OK(pplx_a2a_world_reserve_split(world, y_dtype == PPLX_A2A_F32 ? 4 : 2));
    }
    for (uint32_t r = 0; r < geo.R; ++r) {
      auto a = dispatch_args(r);
      A2A_OK(pplx_a2a_dispatch(ranks[r], &a, PPLX_A2A_SPLIT_SEND, stream));
    }
    for (uint32_t r = 0; r < geo.R; ++r) {
      auto a = dispatch_args(r);
      A2A_OK(pplx_a2a_dispatch(ranks[r], &a, PPLX_A2A_SPLIT_RECV, stream));
    }
  }
  HIP_OK(hipStreamSynchronize(stream));

  bool ok = true;
  auto fail = [&](const std::string &what) {
    if (ok) fprintf(stderr, "  FAIL [%s, %s]: %s\n", geo.name, mode_name(mode), what.c_str());
    ok = false;
  };
  for (uint32_t r = 0; r < geo.R && ok; ++r) {
    const auto counts = host_copy(buf[r].counts, L);
    const auto ex = host_copy(buf[r].expert_x, (size_t)L * cap * Hb);
    const auto exs = geo.scale_dim ? host_copy(buf[r].expert_xs, (size_t)L * cap * geo.scale_dim) : std::vector<float>();
    std::vector<uint16_t> y(separate_y ? (size_t)L * cap * geo.H : 0, 0);
    for (uint32_t el = 0; el < L; ++el) {
      const uint32_t e = r * L + el;
      if (counts[el] != (int32_t)expected[e].size()) {
        fail("expert " + std::to_string(e) + ": count " + std::to_string(counts[el]) + " != " +
             std::to_string(expected[e].size()));
        break;
      }
      for (size_t s = 0; s < expected[e].size(); ++s) {
        const auto [g, t] = expected[e][s];
        if (memcmp(&ex[((size_t)el * cap + s) * Hb], &rows_of_group[g][(size_t)t * Hb], Hb) != 0)
          fail("expert " + std::to_string(e) + " row " + std::to_string(s) + " is not token (" +
               std::to_string(g) + "," + std::to_string(t) + ")");
        if (geo.scale_dim &&
            memcmp(&exs[((size_t)el * cap + s) * geo.scale_dim], &groups[g].x_scale[(size_t)t * geo.scale_dim],
                   geo.scale_dim * 4) != 0)
          fail("expert " + std::to_string(e) + " row " + std::to_string(s) + ": scales differ");
        if (separate_y)
          for (uint32_t h = 0; h < geo.H; ++h)
            y[((size_t)el * cap + s) * geo.H + h] = float_to_bf16(groups[g].x[(size_t)t * geo.H + h]);
      }
    }
    if (separate_y) HIP_OK(hipMemcpy(buf[r].expert_y, y.data(), y.size() * 2, hipMemcpyHostToDevice));
  }

  // ---- combine: expert outputs = the dispatched rows themselves, as in the reference test
  if (ok) {
    if (mode == WORLD) {
      std::vector<pplx_a2a_combine_args_t> all;
      for (uint32_t r = 0; r < geo.R; ++r) all.push_back(combine_args(r));
      A2A_OK(pplx_a2a_world_combine(world, all.data(), stream));
    } else if (mode == PER_RANK) {
      for (uint32_t r = 0; r < geo.R; ++r) {
        auto a = combine_args(r);
        A2A_OK(pplx_a2a_combine(ranks[r], &a, PPLX_A2A_SPLIT_NONE, stream));
      }
    } else {
      for (uint32_t r = 0; r < geo.R; ++r) {
        auto a = combine_args(r);
        A2A_OK(pplx_a2a_combine(ranks[r], &a, PPLX_A2A_SPLIT_SEND, stream));
      }
      for (uint32_t r = 0; r < geo.R; ++r) {
        auto a = combine_args(r);
        A2A_OK(pplx_a2a_combine(ranks[r], &a, PPLX_A2A_SPLIT_RECV, stream));
      }
    }
    HIP_OK(hipStreamSynchronize(stream));
    for (uint32_t r = 0; r < geo.R && ok; ++r) {
      const GroupData &g = groups[r / geo.dp];
      const auto out = host_copy(buf[r].out_tokens, (size_t)geo.M * geo.H);
      for (uint32_t t = 0; t < geo.M && ok; ++t) {
        for (uint32_t h = 0; h < geo.H; ++h) {
          const uint16_t bits = out[(size_t)t * geo.H + h];
          if (t >= g.m) {
            if (bits != 0x7fc0) fail("rank " + std::to_string(r) + ": row " + std::to_string(t) + " beyond the token count was written");
            continue;
          }
          float sum = 0.f;
          for (uint32_t k = 0; k < geo.K; ++k) sum += g.weights[(size_t)t * geo.K + k] * g.x[(size_t)t * geo.H + h];
          const float got = bf16_to_float(bits);
          if (!(std::fabs(got - sum) <= 0.5f) || !(std::fabs(got - sum) <= 1e-2f + 1e-2f * std::fabs(sum)))
            fail("rank " + std::to_string(r) + " token " + std::to_string(t) + " col " + std::to_string(h) +
                 ": " + std::to_string(got) + " != " + std::to_string(sum));
        }
      }
    }
  }
  uint32_t faults = 0;
  A2A_OK(pplx_a2a_world_faults(world, stream, &faults));
  if (faults) fail("device fault bits " + std::to_string(faults));

  for (uint32_t r = 0; r < geo.R; ++r) {
    A2A_OK(pplx_a2a_destroy(ranks[r]));
    RankBuffers &b = buf[r];
    void *ptrs[] = {b.counts, b.expert_x, b.expert_xs, b.expert_y, b.dp_x, b.dp_xs, b.indices, b.weights, b.bound_m, b.out_tokens};
    for (void *p : ptrs)
      if (p) HIP_OK(hipFree(p));
  }
  A2A_OK(pplx_a2a_world_destroy(world));
  printf("  %s [%s, %s]\n", ok ? "pass" : "FAIL", geo.name, mode_name(mode));
  return ok;
}

// The division helper of the kernels (a2a_device.h) against the hardware's own, on the host:
// every divisor a geometry can produce in the small range, large ones in strides, numerators
// around every multiple's edge and across the 32-bit range.
bool check_fast_div() {
  uint64_t checked = 0;
  auto check = [&](uint32_t n, uint32_t d, const pplx_amd::FastDiv &f) {
    ++checked;
    if (pplx_amd::fast_div(n, f) == n / d) return true;
    printf("  FAIL fast_div(%u, %u) = %u, expected %u\n", n, d, pplx_amd::fast_div(n, f), n / d);
    return false;
  };
  std::vector<uint32_t> divisors;
  for (uint32_t d = 1; d <= 8200; ++d) divisors.push_back(d);
  for (uint64_t d = 8209; d < (1ull << 32); d = d * 3 / 2 + 7) divisors.push_back((uint32_t)d);
  for (uint32_t d : {0x3fffffffu, 0x40000000u, 0x40000001u, 0x7fffffffu, 0x80000000u, 0x80000001u, 0xfffffffeu, 0xffffffffu})
    divisors.push_back(d);
  for (uint32_t d : divisors) {
    const pplx_amd::FastDiv f = pplx_amd::make_fast_div(d);
    for (uint32_t n = 0; n < 300; ++n)
      if (!check(n, d, f)) return false;
    for (uint64_t q = 1; q * d < (1ull << 32) && q < 40; ++q)
      for (int64_t delta = -2; delta <= 2; ++delta) {
        const int64_t n = (int64_t)(q * d) + delta;
        if (n >= 0 && n < (1ll << 32) && !check((uint32_t)n, d, f)) return false;
      }
    uint32_t x = d * 2654435761u + 12345u;
    for (int i = 0; i < 200; ++i) {
      x = x * 1664525u + 1013904223u;
      if (!check(x, d, f) || !check(x >> (i % 31), d, f)) return false;
    }
    for (uint32_t n : {0xffffffffu, 0xfffffffeu, 0x80000000u, 0x7fffffffu})
      if (!check(n, d, f)) return false;
  }
  printf("  pass [fast_div: %llu quotients against the hardware's]\n", (unsigned long long)checked);
  return true;
}

}  // namespace

int main(int argc, char **argv) {
  if (!check_fast_div()) return 1;
  if (argc > 1 && std::string(argv[1]) == "--host-only") return 0;
  int n_dev = 0;
  if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev == 0) {
    fprintf(stderr, "test_a2a: no GPU visible\n");
    return 2;
  }
  HIP_OK(hipSetDevice(0));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  const Geometry cases[] = {
      {"reference test, float rows", 4, 2, 8, 3, 16, 10, 5, 4, 8, false},
      {"reference test, bf16 rows", 4, 2, 8, 3, 16, 10, 5, 2, 8, false},
      {"DSv3 row, 8 ranks x 16 tokens", 8, 1, 256, 8, 7168, 16, 1, 1, 56, true},
      {"72 ranks (tables in HBM)", 72, 1, 72, 2, 64, 3, 1, 2, 0, true},
      {"1300 tokens (one launch, several counting passes)", 2, 1, 8, 2, 64, 1300, 900, 2, 0, true},
      {"9000 tokens per rank (routing tiles + scatter)", 2, 1, 8, 2, 64, 9000, 7000, 2, 0, true},
  };
  bool ok = true;
  printf("libpplx_kernels %s\n", pplx_a2a_version());
  for (const Geometry &geo : cases)
    for (Mode mode : {PER_RANK, WORLD, SPLIT}) ok &= run_case(geo, mode, stream);
  HIP_OK(hipStreamDestroy(stream));
  printf("%s\n", ok ? "ALL PASSED" : "FAILED");
  return ok ? 0 : 1;
}
