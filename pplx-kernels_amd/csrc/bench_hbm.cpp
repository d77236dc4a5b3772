// What this GPU's memory gives to plain streaming kernels with the read : write mix of the
// dispatch and combine kernels, without any of their indirection: the yardstick beside the
// published 8 TB/s that their achieved rates are read against.
//
//   fill       write only                        (the scatter's stores alone)
//   read       read only
//   copy       1 read : 1 write                  (split mode's RECV)
//   fan-out    1 read : 8 writes, 7 KiB rows     (a top-8 dispatch)
//   gather     8 reads : 1 write, 14 KiB rows    (a top-8 combine of bf16 rows)
//   streams    the same 2 GiB written (read) in 4 KiB pieces that go round-robin to S regions of
//              the buffer: S = 256 is what a dispatch into 256 experts' buffers does to the
//              memory, S = 8 what a dispatch into 8 experts' buffers does
//   rows       2 GiB written as rows of 4, 7 or 8 KiB, one wavefront (a workgroup of its own) per
//              row, the rows in address order or scattered over the buffer one by one: what the
//              shape of the scatter (one wave, one row, 16 bytes per lane and store) gets from
//              the memory whatever it is asked to route
//
// Every kernel moves 16 bytes per lane and access, eight accesses in flight per lane, with
// non-temporal stores; buffers are 2 GiB, far beyond the 256 MB last-level cache.  Times are
// HIP events around `repeats` back-to-back launches.
//
//   bench_hbm [repeats=10]
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

#define HIP_OK(expr)                                                                      \
  do {                                                                                    \
    hipError_t err_ = (expr);                                                             \
    if (err_ != hipSuccess) {                                                             \
      fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(err_)); \
      exit(2);                                                                            \
    }                                                                                     \
  } while (0)

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr uint32_t kBatch = 8;
constexpr uint32_t kThreads = 256;

// Vector `i` of a launch: consecutive lanes take consecutive vectors, a workgroup takes
// kBatch * kThreads of them at a time.
__device__ __forceinline__ uint64_t first_vector() {
  return (uint64_t)blockIdx.x * kBatch * kThreads + threadIdx.x;
}
__device__ __forceinline__ uint64_t grid_vectors() { return (uint64_t)gridDim.x * kBatch * kThreads; }

__global__ __launch_bounds__(kThreads) void fill_kernel(u32x4 *dst, uint64_t n) {
  const u32x4 v = {threadIdx.x, blockIdx.x, 3u, 4u};
  for (uint64_t i0 = first_vector(); i0 < n; i0 += grid_vectors()) {
#pragma unroll
    for (uint32_t b = 0; b < kBatch; ++b) {
      const uint64_t i = i0 + (uint64_t)b * kThreads;
      if (i < n) __builtin_nontemporal_store(v, dst + i);
    }
  }
}

__global__ __launch_bounds__(kThreads) void read_kernel(const u32x4 *src, uint64_t n, u32x4 *sink) {
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (uint64_t i0 = first_vector(); i0 < n; i0 += grid_vectors()) {
    u32x4 x[kBatch];
#pragma unroll
    for (uint32_t b = 0; b < kBatch; ++b) {
      const uint64_t i = i0 + (uint64_t)b * kThreads;
      x[b] = __builtin_nontemporal_load(src + (i < n ? i : n - 1));
    }
#pragma unroll
    for (uint32_t b = 0; b < kBatch; ++b) acc ^= x[b];
  }
  // never true for the data of this program: keeps the loads alive without a store per lane
  if (acc[0] == 0xdeadbeefu && acc[1] == 0x12345678u) *sink = acc;
}

__global__ __launch_bounds__(kThreads) void copy_kernel(const u32x4 *src, u32x4 *dst, uint64_t n) {
  for (uint64_t i0 = first_vector(); i0 < n; i0 += grid_vectors()) {
    u32x4 x[kBatch];
#pragma unroll
    for (uint32_t b = 0; b < kBatch; ++b) {
      const uint64_t i = i0 + (uint64_t)b * kThreads;
      x[b] = __builtin_nontemporal_load(src + (i < n ? i : n - 1));
    }
#pragma unroll
    for (uint32_t b = 0; b < kBatch; ++b) {
      const uint64_t i = i0 + (uint64_t)b * kThreads;
      if (i < n) __builtin_nontemporal_store(x[b], dst + i);
    }
  }
}

// One wavefront per row of `row_vectors` 16-byte vectors (at most 8 per lane): the row is read
// once and written to the same row of `copies` destination planes of `rows` rows each.
__global__ __launch_bounds__(kThreads) void fan_out_kernel(const u32x4 *src, u32x4 *dst, uint64_t rows,
                                                           uint32_t row_vectors, uint32_t copies) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint64_t row = (uint64_t)blockIdx.x * (kThreads / 64) + threadIdx.x / 64;
  if (row >= rows) return;
  u32x4 x[kBatch];
#pragma unroll
  for (uint32_t b = 0; b < kBatch; ++b) {
    const uint32_t j = lane + b * 64u;
    x[b] = __builtin_nontemporal_load(src + row * row_vectors + (j < row_vectors ? j : row_vectors - 1));
  }
  for (uint32_t c = 0; c < copies; ++c) {
    u32x4 *out = dst + ((uint64_t)c * rows + row) * row_vectors;
#pragma unroll
    for (uint32_t b = 0; b < kBatch; ++b) {
      const uint32_t j = lane + b * 64u;
      if (j < row_vectors) __builtin_nontemporal_store(x[b], out + j);
    }
  }
}

// One wavefront per 64 vectors of an output row: the same vectors of `terms` source planes are
// read and added up.
__global__ __launch_bounds__(kThreads) void gather_kernel(const u32x4 *src, u32x4 *dst, uint64_t vectors,
                                                          uint32_t terms) {
  const uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= vectors) return;
  u32x4 x[kBatch];
#pragma unroll
  for (uint32_t b = 0; b < kBatch; ++b) {
    x[b] = __builtin_nontemporal_load(src + (uint64_t)(b < terms ? b : terms - 1) * vectors + i);
  }
  u32x4 acc = {0u, 0u, 0u, 0u};
#pragma unroll
  for (uint32_t b = 0; b < kBatch; ++b) {
    if (b < terms) acc += x[b];
  }
  __builtin_nontemporal_store(acc, dst + i);
}

// Piece c (256 vectors, one workgroup, one access per thread) belongs to region c % streams and
// is that region's piece number c / streams; a region is `spacing` pieces long.
__device__ __forceinline__ uint64_t piece_vector(uint32_t streams, uint32_t spacing) {
  const uint32_t c = blockIdx.x;
  return ((uint64_t)(c % streams) * spacing + c / streams) * kThreads + threadIdx.x;
}

__global__ __launch_bounds__(kThreads) void write_streams_kernel(u32x4 *dst, uint32_t streams, uint32_t spacing) {
  const u32x4 v = {threadIdx.x, blockIdx.x, 3u, 4u};
  __builtin_nontemporal_store(v, dst + piece_vector(streams, spacing));
}

__global__ __launch_bounds__(kThreads) void read_streams_kernel(const u32x4 *src, uint32_t streams, uint32_t spacing,
                                                                u32x4 *sink) {
  const u32x4 x = __builtin_nontemporal_load(src + piece_vector(streams, spacing));
  if (x[0] == 0xdeadbeefu && x[1] == 0x12345678u) *sink = x;
}

// One wavefront per row of `row_vectors` 16-byte vectors (NV per lane); row r goes to position
// (r * mult) % rows: mult = 1 writes in address order, a mult coprime to `rows` scatters.
template <int NV>
__global__ __launch_bounds__(64) void write_rows_kernel(u32x4 *dst, uint32_t rows, uint32_t row_vectors, uint32_t mult) {
  const uint32_t lane = threadIdx.x;
  const uint32_t row = blockIdx.x;
  if (row >= rows) return;
  const uint32_t place = (uint32_t)(((uint64_t)row * mult) % rows);
  u32x4 *out = dst + (uint64_t)place * row_vectors;
  const u32x4 v = {lane, row, 3u, 4u};
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (lane + i * 64u < row_vectors) __builtin_nontemporal_store(v, out + lane + i * 64u);
  }
}

uint32_t gcd(uint32_t a, uint32_t b) {
  while (b) {
    const uint32_t t = a % b;
    a = b;
    b = t;
  }
  return a;
}

template <class Launch>
void measure(const char *name, double bytes, unsigned repeats, hipStream_t stream, Launch &&launch) {
  hipEvent_t a, b;
  HIP_OK(hipEventCreate(&a));
  HIP_OK(hipEventCreate(&b));
  for (int i = 0; i < 2; ++i) launch();
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipEventRecord(a, stream));
  for (unsigned i = 0; i < repeats; ++i) launch();
  HIP_OK(hipEventRecord(b, stream));
  HIP_OK(hipEventSynchronize(b));
  HIP_OK(hipGetLastError());
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, a, b));
  const double us = ms * 1e3 / repeats;
  printf("%-44s %8.1f MB  %9.1f us  %6.2f TB/s  %5.1f %% of 8 TB/s\n", name, bytes / 1e6, us, bytes / us / 1e6,
         bytes / us / 1e6 / 8.0 * 100.0);
  HIP_OK(hipEventDestroy(a));
  HIP_OK(hipEventDestroy(b));
}

}  // namespace

int main(int argc, char **argv) {
  const unsigned repeats = argc > 1 ? (unsigned)atoi(argv[1]) : 10;
  int n_dev = 0;
  if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev == 0) {
    fprintf(stderr, "bench_hbm: no GPU visible\n");
    return 2;
  }
  HIP_OK(hipSetDevice(0));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  const uint64_t big = 2ull << 30, big_vectors = big / 16;
  u32x4 *a = nullptr, *b = nullptr, *sink = nullptr;
  HIP_OK(hipMalloc(reinterpret_cast<void **>(&a), big));
  HIP_OK(hipMalloc(reinterpret_cast<void **>(&b), big));
  HIP_OK(hipMalloc(reinterpret_cast<void **>(&sink), 256));
  HIP_OK(hipMemsetAsync(a, 1, big, stream));
  HIP_OK(hipMemsetAsync(b, 2, big, stream));
  const dim3 block(kThreads);
  const uint32_t stream_grid = 256 * 16;  // sixteen workgroups per CU, each looping over the buffer

  printf("plain streaming kernels, 16 B per lane, %u launches each (HIP events)\n", repeats);
  measure("fill: 2 GiB written", (double)big, repeats, stream, [&] {
    hipLaunchKernelGGL(fill_kernel, dim3(stream_grid), block, 0, stream, b, big_vectors);
  });
  measure("read: 2 GiB read", (double)big, repeats, stream, [&] {
    hipLaunchKernelGGL(read_kernel, dim3(stream_grid), block, 0, stream, a, big_vectors, sink);
  });
  measure("copy: 1 GiB read, 1 GiB written", (double)big, repeats, stream, [&] {
    hipLaunchKernelGGL(copy_kernel, dim3(stream_grid), block, 0, stream, a, b, big_vectors / 2);
  });
  {
    // 7 KiB rows (448 vectors), eight copies each: 1 : 8 like a top-8 dispatch of fp8 rows
    const uint32_t row_vectors = 448, copies = 8;
    const uint64_t rows = big_vectors / ((uint64_t)row_vectors * copies);
    const double bytes = (double)rows * row_vectors * 16.0 * (1 + copies);
    measure("fan-out: 7 KiB rows read once, written 8x", bytes, repeats, stream, [&] {
      hipLaunchKernelGGL(fan_out_kernel, dim3((uint32_t)((rows + 3) / 4)), block, 0, stream, a, b, rows, row_vectors,
                         copies);
    });
  }
  {
    // eight planes summed into one: 8 : 1 like a top-8 combine
    const uint32_t terms = 8;
    const uint64_t vectors = big_vectors / terms;
    const double bytes = (double)vectors * 16.0 * (terms + 1);
    measure("gather: 8 planes read, their sum written", bytes, repeats, stream, [&] {
      hipLaunchKernelGGL(gather_kernel, dim3((uint32_t)((vectors + kThreads - 1) / kThreads)), block, 0, stream, a, b,
                         vectors, terms);
    });
  }
  {
    const uint32_t pieces = (uint32_t)(big_vectors / kThreads);
    char name[96];
    for (uint32_t streams : {1u, 8u, 32u, 64u, 256u}) {
      const uint32_t spacing = pieces / streams;
      snprintf(name, sizeof name, "write: 4 KiB pieces into %u regions in turn", streams);
      measure(name, (double)big, repeats, stream, [&] {
        hipLaunchKernelGGL(write_streams_kernel, dim3(pieces), block, 0, stream, b, streams, spacing);
      });
    }
    for (uint32_t streams : {1u, 8u, 32u, 64u, 256u}) {
      const uint32_t spacing = pieces / streams;
      snprintf(name, sizeof name, "read: 4 KiB pieces out of %u regions in turn", streams);
      measure(name, (double)big, repeats, stream, [&] {
        hipLaunchKernelGGL(read_streams_kernel, dim3(pieces), block, 0, stream, a, streams, spacing, sink);
      });
    }
  }
  for (uint32_t row_vectors : {256u, 448u, 512u}) {
    const uint32_t rows = (uint32_t)(big_vectors / row_vectors);
    for (bool scattered : {false, true}) {
      uint32_t mult = 1;
      if (scattered) {
        mult = (uint32_t)(rows * 0.6180339887) | 1u;
        while (gcd(mult, rows) != 1) mult += 2;
      }
      char name[96];
      snprintf(name, sizeof name, "rows: %u KiB rows, one wave each, %s", row_vectors / 64,
               scattered ? "scattered" : "in address order");
      measure(name, (double)rows * row_vectors * 16.0, repeats, stream, [&] {
        hipLaunchKernelGGL(write_rows_kernel<8>, dim3(rows), dim3(64), 0, stream, b, rows, row_vectors, mult);
      });
    }
  }
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipFree(a));
  HIP_OK(hipFree(b));
  HIP_OK(hipFree(sink));
  HIP_OK(hipStreamDestroy(stream));
  return 0;
}
