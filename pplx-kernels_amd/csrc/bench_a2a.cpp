// Torch-free latency benchmark over the C ABI, in the layout of the reference's
// csrc/all_to_all/bench_all_to_all.cpp:116-283: per configuration the time of dispatch and
// combine as one call (send+recv) and split into send and recv, HIP events on the stream,
// 10 samples per repeat after warm-up, mean and standard deviation, and the payload
// bandwidth by the reference's formula (tokens * K * bytes per token, :266-275) summed over
// the simulated ranks.  The phases run in the reference's order (:183-203)
//     dispatch, combine, dispatch SEND, gap, dispatch RECV, combine SEND, gap, combine RECV
// where the gap is a kernel that sleeps for 100 us in place of the experts' compute.  A last
// section runs a SEND phase on one stream while the gap kernel occupies another, to show that
// a split phase overlaps with independent work.  All ranks run in this process on one GPU.
//
//   bench_a2a [ranks=8] [repeats=10] [quick]
#include <hip/hip_runtime.h>

#include <cmath>
#include <string>

#include "harness.h"

using namespace harness;

namespace {

struct Config {
  uint32_t tokens, experts, k, hidden;
};

// Stands in for the experts' compute between the phases (the reference's sleepOnStream over
// csrc/core/kernels.cu:8-12): one wavefront that naps until `us` microseconds of the 100 MHz
// wall clock have passed, in at most `max_naps` naps, so that it ends whatever the clock does.
__global__ void gap_kernel(uint32_t us, uint32_t max_naps) {
  const uint64_t start = wall_clock64();
  for (uint32_t i = 0; i < max_naps; ++i) {
    if (wall_clock64() - start >= (uint64_t)us * 100u) break;
    __builtin_amdgcn_s_sleep(32);
  }
}

constexpr uint32_t kGapUs = 100;

void gap(hipStream_t stream) {
  hipLaunchKernelGGL(gap_kernel, dim3(1), dim3(64), 0, stream, kGapUs, 4 * kGapUs);
  HIP_OK(hipGetLastError());
}

struct Stat {
  double mean, stddev;
};

Stat stat_of(const std::vector<float> &us) {
  double s = 0, s2 = 0;
  for (float v : us) {
    s += v;
    s2 += (double)v * v;
  }
  const double mean = s / us.size();
  return {mean, std::sqrt(std::max(0.0, s2 / us.size() - mean * mean))};
}

struct World {
  uint32_t R, L, cap, H, K, scale_dim;
  size_t Hb;
  pplx_a2a_world_t *world;
  std::vector<pplx_a2a_t *> ranks;
  std::vector<pplx_a2a_dispatch_args_t> d;
  std::vector<pplx_a2a_combine_args_t> c;
  std::vector<void *> allocations;
};

World make_world(const Config &cfg, uint32_t R, bool fp8) {
  World w{};
  w.R = R;
  w.L = cfg.experts / R;
  w.cap = cfg.tokens * R;
  w.H = cfg.hidden;
  w.K = cfg.k;
  w.scale_dim = fp8 ? (cfg.hidden + 127) / 128 : 0;
  w.Hb = (size_t)cfg.hidden * (fp8 ? 1 : 2);
  pplx_a2a_config_t c{};
  c.max_num_tokens = cfg.tokens;
  c.num_experts = cfg.experts;
  c.experts_per_token = cfg.k;
  c.world_size = R;
  c.dp_size = 1;
  c.hidden_dim = cfg.hidden;
  c.hidden_dim_bytes = w.Hb;
  c.hidden_dim_scale_bytes = w.scale_dim * 4;
  A2A_OK(pplx_a2a_world_create(&c, 0, &w.world));
  A2A_OK(pplx_a2a_world_reserve_split(w.world, 2));  // bf16 expert_y
  w.ranks.resize(R);
  std::mt19937 gen(1234);
  for (uint32_t r = 0; r < R; ++r) {
    A2A_OK(pplx_a2a_create(w.world, r, &w.ranks[r]));
    GroupData g = make_group(gen, cfg.tokens, cfg.tokens, cfg.experts, cfg.k, 8, w.scale_dim);
    auto keep = [&](auto *p) {
      w.allocations.push_back((void *)p);
      return p;
    };
    pplx_a2a_dispatch_args_t a{};
    a.out_expert_num_tokens = keep(device_alloc<int32_t>(w.L));
    a.out_expert_num_tokens_stride = 1;
    a.out_expert_x = keep(device_alloc<uint8_t>((size_t)w.L * w.cap * w.Hb));
    a.out_expert_x_stride_row = (int64_t)w.Hb;
    a.out_expert_x_stride_expert = (int64_t)w.Hb * w.cap;
    a.out_expert_x_rows = w.cap;
    if (w.scale_dim) {
      a.out_expert_x_scale = keep(device_alloc<float>((size_t)w.L * w.cap * w.scale_dim));
      a.out_expert_x_scale_stride_elem = 1;
      a.out_expert_x_scale_stride_row = w.scale_dim;
      a.out_expert_x_scale_stride_expert = (int64_t)w.scale_dim * w.cap;
      a.dp_x_scale = keep(device_copy(g.x_scale));
      a.dp_x_scale_stride_elem = 1;
      a.dp_x_scale_stride_row = w.scale_dim;
    }
    uint8_t *x = keep(device_alloc<uint8_t>((size_t)cfg.tokens * w.Hb));
    HIP_OK(hipMemset(x, 0x3c, (size_t)cfg.tokens * w.Hb));
    a.dp_x = x;
    a.dp_x_stride_row = (int64_t)w.Hb;
    a.indices = keep(device_copy(g.indices));
    a.m = cfg.tokens;
    w.d.push_back(a);
    pplx_a2a_combine_args_t b{};
    b.out_tokens = keep(device_alloc<uint16_t>((size_t)cfg.tokens * w.H));
    b.out_tokens_stride_row = w.H;
    b.out_dtype = PPLX_A2A_BF16;
    b.indices = a.indices;
    b.weights = keep(device_copy(g.weights));
    b.weights_stride_row = w.K;
    b.expert_y = keep(device_alloc<uint16_t>((size_t)w.L * w.cap * w.H));
    b.expert_y_stride_row = w.H;
    b.expert_y_stride_expert = (int64_t)w.H * w.cap;
    b.expert_y_rows = w.cap;
    b.in_dtype = PPLX_A2A_BF16;
    b.m = cfg.tokens;
    w.c.push_back(b);
  }
  return w;
}

void free_world(World &w) {
  for (auto *r : w.ranks) A2A_OK(pplx_a2a_destroy(r));
  A2A_OK(pplx_a2a_world_destroy(w.world));
  for (void *p : w.allocations) HIP_OK(hipFree(p));
}

void bench_config(const Config &cfg, uint32_t R, bool fp8, unsigned repeats, hipStream_t stream) {
  World w = make_world(cfg, R, fp8);
  constexpr int kSamples = 10, kPhases = 6;
  hipEvent_t ev[kSamples][kPhases * 2];
  for (auto &row : ev)
    for (auto &e : row) HIP_OK(hipEventCreate(&e));
  std::vector<float> times[kPhases];

  auto dispatch = [&](int mode) {
    for (uint32_t r = 0; r < R; ++r) A2A_OK(pplx_a2a_dispatch(w.ranks[r], &w.d[r], mode, stream));
  };
  auto combine = [&](int mode) {
    for (uint32_t r = 0; r < R; ++r) A2A_OK(pplx_a2a_combine(w.ranks[r], &w.c[r], mode, stream));
  };
  auto run = [&](bool record) {
    for (int i = 0; i < kSamples; ++i) {
      int p = 0;
      auto timed = [&](auto fn) {
        HIP_OK(hipEventRecord(ev[i][p++], stream));
        fn();
        HIP_OK(hipEventRecord(ev[i][p++], stream));
      };
      timed([&] { dispatch(PPLX_A2A_SPLIT_NONE); });
      timed([&] { combine(PPLX_A2A_SPLIT_NONE); });
      timed([&] { dispatch(PPLX_A2A_SPLIT_SEND); });
      gap(stream);
      timed([&] { dispatch(PPLX_A2A_SPLIT_RECV); });
      timed([&] { combine(PPLX_A2A_SPLIT_SEND); });
      gap(stream);
      timed([&] { combine(PPLX_A2A_SPLIT_RECV); });
    }
    HIP_OK(hipStreamSynchronize(stream));
    if (!record) return;
    for (int i = 0; i < kSamples; ++i)
      for (int p = 0; p < kPhases; ++p) {
        float ms = 0;
        HIP_OK(hipEventElapsedTime(&ms, ev[i][2 * p], ev[i][2 * p + 1]));
        times[p].push_back(ms * 1e3f);
      }
  };
  for (int i = 0; i < 3; ++i) run(false);
  for (unsigned i = 0; i < repeats; ++i) run(true);

  const double bytes_per_token = (double)w.Hb + 4.0 * w.scale_dim;
  const double pairs = (double)cfg.tokens * cfg.k * R;
  Stat s[kPhases];
  for (int p = 0; p < kPhases; ++p) s[p] = stat_of(times[p]);
  printf("%4u %4u %2u %5u | %7.1f ± %4.1f %7.1f ± %4.1f %7.1f ± %4.1f %6.0f GB/s | %7.1f ± %4.1f %7.1f ± %4.1f %7.1f ± %4.1f %6.0f GB/s\n",
         cfg.tokens, cfg.experts, cfg.k, cfg.hidden, s[0].mean, s[0].stddev, s[2].mean, s[2].stddev,
         s[3].mean, s[3].stddev, pairs * bytes_per_token / s[0].mean * 1e-3, s[1].mean, s[1].stddev,
         s[4].mean, s[4].stddev, s[5].mean, s[5].stddev, pairs * w.H * 2.0 / s[1].mean * 1e-3);
  fflush(stdout);
  if (cfg.tokens == 128 && cfg.experts == 256) {
    printf("     send+recv against one call: dispatch %.2fx, combine %.2fx\n",
           (s[2].mean + s[3].mean) / s[0].mean, (s[4].mean + s[5].mean) / s[1].mean);
  }
  for (auto &row : ev)
    for (auto &e : row) HIP_OK(hipEventDestroy(e));
  free_world(w);
}

// dispatch SEND on one stream while the gap kernel (the "experts") runs on another: the pair
// takes about as long as the longer of the two when the phases overlap, their sum when not.
void bench_overlap(const Config &cfg, uint32_t R, hipStream_t comm) {
  World w = make_world(cfg, R, true);
  hipStream_t compute;
  HIP_OK(hipStreamCreate(&compute));
  hipEvent_t begin, end, fork, join;
  for (hipEvent_t *e : {&begin, &end, &fork, &join}) HIP_OK(hipEventCreate(e));
  auto send = [&] {
    for (uint32_t r = 0; r < R; ++r) A2A_OK(pplx_a2a_dispatch(w.ranks[r], &w.d[r], PPLX_A2A_SPLIT_SEND, comm));
  };
  auto recv = [&] {
    for (uint32_t r = 0; r < R; ++r) A2A_OK(pplx_a2a_dispatch(w.ranks[r], &w.d[r], PPLX_A2A_SPLIT_RECV, comm));
  };
  auto measure = [&](bool with_send, bool with_gap) {
    double total = 0;
    const int reps = 20;
    for (int i = -3; i < reps; ++i) {
      HIP_OK(hipEventRecord(begin, comm));
      if (with_gap) {
        HIP_OK(hipEventRecord(fork, comm));
        HIP_OK(hipStreamWaitEvent(compute, fork, 0));
        gap(compute);
        HIP_OK(hipEventRecord(join, compute));
      }
      if (with_send) send();
      if (with_gap) HIP_OK(hipStreamWaitEvent(comm, join, 0));
      HIP_OK(hipEventRecord(end, comm));
      if (with_send) recv();  // completes the step
      HIP_OK(hipStreamSynchronize(comm));
      float ms = 0;
      HIP_OK(hipEventElapsedTime(&ms, begin, end));
      if (i >= 0) total += ms * 1e3;
    }
    return total / reps;
  };
  const double t_send = measure(true, false), t_gap = measure(false, true), t_both = measure(true, true);
  printf("overlap, %u tok x %u ranks: dispatch SEND alone %.1f us, gap kernel alone %.1f us, "
         "SEND on one stream with the gap kernel on another %.1f us (sum %.1f)\n",
         cfg.tokens, R, t_send, t_gap, t_both, t_send + t_gap);
  for (hipEvent_t e : {begin, end, fork, join}) HIP_OK(hipEventDestroy(e));
  HIP_OK(hipStreamDestroy(compute));
  free_world(w);
}

}  // namespace

int main(int argc, char **argv) {
  const uint32_t R = argc > 1 ? (uint32_t)atoi(argv[1]) : 8;
  const unsigned repeats = argc > 2 ? (unsigned)atoi(argv[2]) : 10;
  const bool quick = argc > 3 && std::string(argv[3]) == "quick";
  int n_dev = 0;
  if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev == 0) {
    fprintf(stderr, "bench_a2a: no GPU visible\n");
    return 2;
  }
  HIP_OK(hipSetDevice(0));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  std::vector<Config> configs = {{1, 8, 4, 128}, {4, 8, 6, 2048}};
  for (uint32_t experts : {8u, 16u, 64u, 256u})
    for (uint32_t tokens : {1u, 4u, 16u, 64u, 128u}) configs.push_back({tokens, experts, 8, 7168});
  if (quick) configs = {{4, 8, 6, 2048}, {128, 256, 8, 7168}};
  for (bool fp8 : {true, false}) {
    printf("%s rows, %u simulated ranks on one GPU, times in us (host-launched, per-rank calls)\n",
           fp8 ? "FP8 + block scales" : "BF16", R);
    printf(" tok  exp  k   dim | dispatch         send           recv            payload | combine          send           recv            payload\n");
    for (const Config &cfg : configs) {
      if (cfg.experts % R != 0 || cfg.k > cfg.experts) continue;
      if (fp8 && ((cfg.hidden + 127) / 128 * 4) % 16 != 0) continue;  // scale row must be 16-byte sized
      bench_config(cfg, R, fp8, repeats, stream);
    }
  }
  if (256 % R == 0) bench_overlap({128, 256, 8, 7168}, R, stream);
  HIP_OK(hipStreamDestroy(stream));
  return 0;
}
