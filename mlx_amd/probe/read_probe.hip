// read_probe.hip -- how fast can one kernel launch read N bytes of HBM on this
// GPU, with nothing else to do?  The decode kernel (qmv) reads its 33 MB of
// packed weights once per launch, so this is the floor its duration is judged
// against: the same bytes, the same launch protocol as bench.py (a HIP graph of
// back-to-back launches over a ring of buffers larger than the 256 MB Infinity
// Cache, timed with HIP events on the launching stream), but a kernel body
// that only loads.  Three bodies are timed:
//   stream<U>   every wave issues U wave-contiguous 1 KiB loads, then exits
//   rolling<D>  a persistent grid (4 workgroups per CU); each wave keeps D
//               1 KiB loads in flight and walks the buffer with a grid stride
//   empty       a grid of the same size whose waves exit at once (launch cost)
// Built by mlx_amd/_build.py (build_read_probe) into mlx_amd/lib/read_probe.
// Without arguments it prints the whole table; with --floor it times only the
// 33 MB read, the same read from the cache and the empty grid, 1800 launches per
// timed region like bench.py, and prints one JSON line -- bench.py runs it that
// way in a child process and reports the figures beside the decode kernel's.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#define HIP_OK(expr)                                                          \
  do {                                                                        \
    hipError_t e__ = (expr);                                                  \
    if (e__ != hipSuccess) {                                                  \
      std::fprintf(stderr, "%s failed: %s\n", #expr, hipGetErrorString(e__)); \
      std::exit(1);                                                           \
    }                                                                         \
  } while (0)

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned fold(u32x4 v) {
  return v.x ^ v.y ^ v.z ^ v.w;
}

template <int U>
__global__ __launch_bounds__(256) void stream_kernel(
    const u32x4* __restrict__ p, size_t n_vec, unsigned* sink) {
  const size_t wave = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) >> 6;
  const int lane = threadIdx.x & 63;
  u32x4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t idx = (wave * U + u) * 64 + lane;
    v[u] = idx < n_vec ? __builtin_nontemporal_load(p + idx) : u32x4{0, 0, 0, 0};
  }
  unsigned acc = 0;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    acc ^= fold(v[u]);
  }
  if (acc == 0x12345678u) { // never true for the fill pattern: keeps the loads
    sink[0] = acc;
  }
}

template <int D>
__global__ __launch_bounds__(256) void rolling_kernel(
    const u32x4* __restrict__ p, size_t n_vec, unsigned* sink) {
  const size_t waves = (static_cast<size_t>(gridDim.x) * 256) >> 6;
  const size_t wave = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) >> 6;
  const int lane = threadIdx.x & 63;
  const size_t n_kib = n_vec / 64;
  u32x4 v[D];
  unsigned acc = 0;
  size_t k = wave;
#pragma unroll
  for (int d = 0; d < D; ++d) {
    const size_t at = k + d * waves;
    v[d] = at < n_kib ? __builtin_nontemporal_load(p + at * 64 + lane) : u32x4{0, 0, 0, 0};
  }
  for (; k < n_kib; k += D * waves) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      acc ^= fold(v[d]);
      const size_t at = k + (D + d) * waves;
      v[d] = at < n_kib ? __builtin_nontemporal_load(p + at * 64 + lane) : u32x4{0, 0, 0, 0};
    }
  }
  if (acc == 0x12345678u) {
    sink[0] = acc;
  }
}

__global__ __launch_bounds__(256) void empty_kernel(unsigned* sink, int never) {
  if (never) {
    sink[0] = 1;
  }
}

struct Probe {
  hipStream_t stream;
  hipEvent_t start, stop;
  Probe() {
    HIP_OK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    HIP_OK(hipEventCreate(&start));
    HIP_OK(hipEventCreate(&stop));
  }
  // Median over 7 repeats of `replays` graph replays of `period` launches each,
  // in microseconds per launch.
  template <typename F>
  float time(int period, int replays, F launch) {
    hipGraph_t graph;
    hipGraphExec_t exec;
    HIP_OK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    for (int i = 0; i < period; ++i) {
      launch(i, stream);
    }
    HIP_OK(hipStreamEndCapture(stream, &graph));
    HIP_OK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    for (int r = 0; r < 3; ++r) {
      HIP_OK(hipGraphLaunch(exec, stream));
    }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<float> samples;
    for (int rep = 0; rep < 7; ++rep) {
      HIP_OK(hipEventRecord(start, stream));
      for (int r = 0; r < replays; ++r) {
        HIP_OK(hipGraphLaunch(exec, stream));
      }
      HIP_OK(hipEventRecord(stop, stream));
      HIP_OK(hipEventSynchronize(stop));
      float ms = 0;
      HIP_OK(hipEventElapsedTime(&ms, start, stop));
      samples.push_back(ms * 1000.0f / (replays * period));
    }
    std::sort(samples.begin(), samples.end());
    HIP_OK(hipGraphExecDestroy(exec));
    HIP_OK(hipGraphDestroy(graph));
    return samples[3];
  }
};

int main(int argc, char** argv) {
  const bool floor_only = argc > 1 && std::string(argv[1]) == "--floor";
  // W + scales + biases of the 4096 x 14336, 4-bit, group-64 decode weight,
  // rounded to whole KiB.
  const size_t unit = (static_cast<size_t>(4096) * 14336 / 2 + 2 * 2 * 4096 * 14336 / 64) / 1024 * 1024;
  const int ring = 18; // 18 x 33 MB = 595 MB
  std::vector<u32x4*> bufs(ring);
  for (auto& b : bufs) {
    HIP_OK(hipMalloc(&b, unit * 4));
    HIP_OK(hipMemset(b, 1, unit * 4));
  }
  unsigned* sink = nullptr;
  HIP_OK(hipMalloc(&sink, 4));
  HIP_OK(hipDeviceSynchronize());
  Probe probe;
  hipDeviceProp_t prop;
  HIP_OK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount;
  if (floor_only) {
    const size_t n_vec = unit / 16;
    const unsigned grid = static_cast<unsigned>((n_vec / 64 / 4 + 3) / 4);
    const float cold = probe.time(ring, 100, [&](int i, hipStream_t s) {
      stream_kernel<4><<<grid, 256, 0, s>>>(bufs[i % ring], n_vec, sink);
    });
    const float hot = probe.time(ring, 100, [&](int, hipStream_t s) {
      stream_kernel<4><<<grid, 256, 0, s>>>(bufs[0], n_vec, sink);
    });
    const float empty = probe.time(ring, 100, [&](int, hipStream_t s) {
      empty_kernel<<<1792, 256, 0, s>>>(sink, 0);
    });
    std::printf(
        "{\"bytes\": %zu, \"read_only_floor_us\": %.3f, \"read_only_cache_resident_us\": %.3f, "
        "\"empty_launch_us\": %.3f, \"launches_per_region\": %d, \"repeats\": 7}\n",
        unit, cold, hot, empty, ring * 100);
    return 0;
  }
  std::printf("device: %s, %d CUs; unit = %zu bytes\n", prop.name, cus, unit);
  std::printf("%-28s %8s %10s %10s\n", "kernel", "MB", "us/launch", "GB/s");
  auto row = [](const char* name, size_t bytes, float us) {
    std::printf("%-28s %8.1f %10.2f %10.1f\n", name, bytes / 1e6, us, bytes / us / 1e3);
    std::fflush(stdout);
  };
  for (int mul : {1, 2, 4}) {
    const size_t bytes = unit * mul;
    const size_t n_vec = bytes / 16;
    const int period = mul == 4 ? 9 : ring; // 9 x 132 MB still exceeds the cache
    {
      const unsigned grid = static_cast<unsigned>((n_vec / 64 / 4 + 3) / 4);
      row("stream<4> cold", bytes, probe.time(period, 20, [&](int i, hipStream_t s) {
        stream_kernel<4><<<grid, 256, 0, s>>>(bufs[i % ring], n_vec, sink);
      }));
    }
    {
      const unsigned grid = static_cast<unsigned>((n_vec / 64 / 8 + 3) / 4);
      row("stream<8> cold", bytes, probe.time(period, 20, [&](int i, hipStream_t s) {
        stream_kernel<8><<<grid, 256, 0, s>>>(bufs[i % ring], n_vec, sink);
      }));
    }
    row("rolling<4> cold, 4 WG/CU", bytes, probe.time(period, 20, [&](int i, hipStream_t s) {
      rolling_kernel<4><<<cus * 4, 256, 0, s>>>(bufs[i % ring], n_vec, sink);
    }));
    row("rolling<8> cold, 4 WG/CU", bytes, probe.time(period, 20, [&](int i, hipStream_t s) {
      rolling_kernel<8><<<cus * 4, 256, 0, s>>>(bufs[i % ring], n_vec, sink);
    }));
  }
  {
    const size_t n_vec = unit / 16;
    const unsigned grid = static_cast<unsigned>((n_vec / 64 / 4 + 3) / 4);
    row("stream<4> same buffer (hot)", unit, probe.time(ring, 20, [&](int, hipStream_t s) {
      stream_kernel<4><<<grid, 256, 0, s>>>(bufs[0], n_vec, sink);
    }));
  }
  {
    const float us = probe.time(ring, 20, [&](int, hipStream_t s) {
      empty_kernel<<<1792, 256, 0, s>>>(sink, 0);
    });
    std::printf("%-28s %8s %10.2f\n", "empty, 1792 workgroups", "-", us);
    const float us2 = probe.time(ring, 20, [&](int, hipStream_t s) {
      empty_kernel<<<cus, 256, 0, s>>>(sink, 0);
    });
    std::printf("%-28s %8s %10.2f\n", "empty, 1 workgroup per CU", "-", us2);
  }
  return 0;
}
