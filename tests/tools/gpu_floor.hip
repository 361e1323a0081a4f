// Two measurements of the machine that bound what ONE short kernel launch can
// reach, whatever the kernel (measurement tool, not part of the library):
//
//   gpu_floor launch
//       an empty kernel as 200 dependent launches of a replayed HIP graph:
//       microseconds from launch to launch, for several grids, workgroup
//       sizes and LDS sizes.  That much of every per-launch figure of a
//       replayed graph is not the kernel's own time.
//
//   gpu_floor clock [workgroups ...]
//       the shader clock the chip holds with `workgroups` CUs (one workgroup
//       of 8 waves each, two on every SIMD) busy on back-to-back
//       v_mfma_f32_16x16x32_f16 over pseudo-random fp16 data: stamp cycles
//       (s_memtime) over wall-clock time (s_memrealtime, 100 MHz) inside the
//       kernel, after 0.3 s of the same load, and the TFLOP/s that loop
//       sustains.  The MFMA peak of 2.5 PFLOP/s is 256 CUs x 4096 flop/clk at
//       2.4 GHz: clock / 2400 MHz x busy CUs / 256 is the share of it any
//       schedule on that many CUs can reach.
//
//   gpu_floor stream
//       what a kernel that does nothing but stream reaches at the depthwise
//       benchmark layer's size and mix (77.1 MB read, 19.3 MB written per
//       launch): every thread loads four 16-byte vectors from four input
//       planes and stores one, consecutive threads consecutive vectors,
//       buffers rotated over four sets (385 MB, beyond the 256 MB Infinity
//       Cache), 200 launches in a replayed HIP graph as bench.py issues its
//       steps.  Variants: U outputs per thread, plain or non-temporal loads
//       and stores, the four loads of an output far apart or adjacent.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define CHECK(x)                                                               \
  do {                                                                         \
    hipError_t e_ = (x);                                                       \
    if (e_ != hipSuccess) {                                                    \
      std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));             \
      std::exit(1);                                                            \
    }                                                                          \
  } while (0)

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

__global__ void emptyKernel(int *never) {
  if (never && threadIdx.x == 0x7fffffff)
    *never = 0;
}

/// Replays a graph of `launches` dependent launches of the empty kernel;
/// microseconds per launch, median of `passes`.
double launchFloor(int grid, int block, int ldsBytes, int launches = 200,
                   int passes = 7) {
  hipStream_t stream;
  CHECK(hipStreamCreate(&stream));
  CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&emptyKernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024));
  hipGraph_t graph;
  hipGraphExec_t exec;
  CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal));
  for (int i = 0; i != launches; ++i)
    hipLaunchKernelGGL(emptyKernel, dim3(grid), dim3(block), ldsBytes, stream,
                       static_cast<int *>(nullptr));
  CHECK(hipStreamEndCapture(stream, &graph));
  CHECK(hipGraphInstantiateWithFlags(&exec, graph, 0));
  CHECK(hipGraphLaunch(exec, stream));
  CHECK(hipStreamSynchronize(stream));
  hipEvent_t start, stop;
  CHECK(hipEventCreate(&start));
  CHECK(hipEventCreate(&stop));
  std::vector<double> us;
  for (int p = 0; p != passes; ++p) {
    const int replays = 20;
    CHECK(hipEventRecord(start, stream));
    for (int r = 0; r != replays; ++r)
      CHECK(hipGraphLaunch(exec, stream));
    CHECK(hipEventRecord(stop, stream));
    CHECK(hipStreamSynchronize(stream));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, start, stop));
    us.push_back(double(ms) * 1e3 / (replays * launches));
  }
  std::sort(us.begin(), us.end());
  CHECK(hipGraphExecDestroy(exec));
  CHECK(hipGraphDestroy(graph));
  CHECK(hipEventDestroy(start));
  CHECK(hipEventDestroy(stop));
  CHECK(hipStreamDestroy(stream));
  return us[us.size() / 2];
}

/// `iters` x 64 MFMAs per wave on eight accumulators; wave 0 of every
/// workgroup records cycle and wall-clock stamps around its loop.
__global__ __launch_bounds__(512) void mfmaLoop(int iters, const uint32_t *seed,
                                                uint64_t *stamps,
                                                float *sink) {
  const int lane = threadIdx.x & 63;
  half8 a[4], b[2];
  // operands of mixed magnitude and sign, so that the multipliers toggle
  uint32_t x = seed[(blockIdx.x * 512 + threadIdx.x) & 4095];
  auto next = [&] {
    x = x * 1664525u + 1013904223u;
    return _Float16(float(int(x >> 9) % 2048 - 1024) * (1.0f / 512));
  };
  for (int i = 0; i != 4; ++i)
    for (int e = 0; e != 8; ++e)
      a[i][e] = next();
  for (int i = 0; i != 2; ++i)
    for (int e = 0; e != 8; ++e)
      b[i][e] = next() * _Float16(0.03f);
  floatx4 acc[8];
  for (int i = 0; i != 8; ++i)
    acc[i] = floatx4{0, 0, 0, 0};
  const uint64_t r0 = __builtin_amdgcn_s_memrealtime();
  const uint64_t t0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it != iters; ++it) {
#pragma unroll
    for (int m = 0; m != 64; ++m)
      acc[m & 7] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
          b[(m >> 2) & 1], a[m & 3], acc[m & 7], 0, 0, 0);
  }
  const uint64_t t1 = __builtin_amdgcn_s_memtime();
  const uint64_t r1 = __builtin_amdgcn_s_memrealtime();
  float s = 0;
  for (int i = 0; i != 8; ++i)
    s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  if (s == 12345.678f)
    sink[0] = s;
  if (threadIdx.x == 0) {
    stamps[blockIdx.x * 4 + 0] = t0, stamps[blockIdx.x * 4 + 1] = t1;
    stamps[blockIdx.x * 4 + 2] = r0, stamps[blockIdx.x * 4 + 3] = r1;
  }
  (void)lane;
}

typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

/// U outputs per thread; NT: non-temporal loads and stores; ADJ: the four
/// loads of an output are neighbours in memory instead of a plane apart.
template <int U, bool NT, bool ADJ>
__global__ __launch_bounds__(256) void streamMix(const uintx4 *__restrict__ in,
                                                 uintx4 *__restrict__ out,
                                                 size_t outVecs) {
  uintx4 v[U][4];
#pragma unroll
  for (int u = 0; u != U; ++u) {
    const size_t o = (size_t(blockIdx.x) * U + u) * 256 + threadIdx.x;
#pragma unroll
    for (int k = 0; k != 4; ++k) {
      const uintx4 *p = ADJ ? in + ((size_t(blockIdx.x) * U + u) * 4 + k) * 256 +
                                  threadIdx.x
                            : in + size_t(k) * outVecs + o;
      if (o < outVecs)
        v[u][k] = NT ? __builtin_nontemporal_load(p) : *p;
    }
  }
#pragma unroll
  for (int u = 0; u != U; ++u) {
    const size_t o = (size_t(blockIdx.x) * U + u) * 256 + threadIdx.x;
    if (o < outVecs) {
      const uintx4 sum = v[u][0] + v[u][1] + v[u][2] + v[u][3];
      if (NT)
        __builtin_nontemporal_store(sum, out + o);
      else
        out[o] = sum;
    }
  }
}

template <int U, bool NT, bool ADJ>
void streamCeiling(const char *name, const std::vector<uintx4 *> &ins,
                   const std::vector<uintx4 *> &outs, size_t outVecs,
                   double bytes) {
  const int sets = int(ins.size());
  const int blocks = int((outVecs + size_t(256) * U - 1) / (size_t(256) * U));
  hipStream_t stream;
  CHECK(hipStreamCreate(&stream));
  hipGraph_t graph;
  hipGraphExec_t exec;
  const int launches = 200;
  CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal));
  for (int i = 0; i != launches; ++i)
    hipLaunchKernelGGL((streamMix<U, NT, ADJ>), dim3(blocks), dim3(256), 0,
                       stream, ins[i % sets], outs[i % sets], outVecs);
  CHECK(hipStreamEndCapture(stream, &graph));
  CHECK(hipGraphInstantiateWithFlags(&exec, graph, 0));
  CHECK(hipGraphLaunch(exec, stream));
  CHECK(hipStreamSynchronize(stream));
  hipEvent_t start, stop;
  CHECK(hipEventCreate(&start));
  CHECK(hipEventCreate(&stop));
  std::vector<double> us;
  for (int p = 0; p != 7; ++p) {
    CHECK(hipEventRecord(start, stream));
    for (int r = 0; r != 2; ++r)
      CHECK(hipGraphLaunch(exec, stream));
    CHECK(hipEventRecord(stop, stream));
    CHECK(hipStreamSynchronize(stream));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, start, stop));
    us.push_back(double(ms) * 1e3 / (2 * launches));
  }
  std::sort(us.begin(), us.end());
  const double t = us[us.size() / 2];
  std::printf("| %s | %d | %s | %.2f | %.0f | %.1f %% |\n", name, U,
              NT ? "non-temporal" : "plain", t, bytes / t / 1e3,
              bytes / t / 1e3 / 80.0);
  CHECK(hipGraphExecDestroy(exec));
  CHECK(hipGraphDestroy(graph));
  CHECK(hipEventDestroy(start));
  CHECK(hipEventDestroy(stop));
  CHECK(hipStreamDestroy(stream));
}

void clockUnderLoad(int workgroups) {
  const int iters = 400; // x 64 MFMAs of 16 cycles: ~0.2 ms per launch
  uint32_t *seed;
  uint64_t *stamps;
  float *sink;
  CHECK(hipMalloc(&seed, 4096 * 4));
  CHECK(hipMalloc(&stamps, size_t(workgroups) * 32));
  CHECK(hipMalloc(&sink, 64));
  std::vector<uint32_t> host(4096);
  for (int i = 0; i != 4096; ++i)
    host[i] = 2654435761u * uint32_t(i + 1);
  CHECK(hipMemcpy(seed, host.data(), 4096 * 4, hipMemcpyHostToDevice));
  hipEvent_t start, stop;
  CHECK(hipEventCreate(&start));
  CHECK(hipEventCreate(&stop));
  // settle: ~0.3 s of the same load, then the measured launches
  for (int i = 0; i != 1500; ++i)
    hipLaunchKernelGGL(mfmaLoop, dim3(workgroups), dim3(512), 0, 0, iters, seed,
                       stamps, sink);
  CHECK(hipDeviceSynchronize());
  const int launches = 200;
  CHECK(hipEventRecord(start, 0));
  for (int i = 0; i != launches; ++i)
    hipLaunchKernelGGL(mfmaLoop, dim3(workgroups), dim3(512), 0, 0, iters, seed,
                       stamps, sink);
  CHECK(hipEventRecord(stop, 0));
  CHECK(hipDeviceSynchronize());
  float ms = 0;
  CHECK(hipEventElapsedTime(&ms, start, stop));
  std::vector<uint64_t> h(size_t(workgroups) * 4);
  CHECK(hipMemcpy(h.data(), stamps, h.size() * 8, hipMemcpyDeviceToHost));
  double mhzSum = 0, mhzMin = 1e9, mhzMax = 0, cyclesPerMfma = 0;
  for (int w = 0; w != workgroups; ++w) {
    const double cycles = double(h[w * 4 + 1] - h[w * 4 + 0]);
    const double ns = double(h[w * 4 + 3] - h[w * 4 + 2]) * 10.0;
    const double mhz = cycles / ns * 1e3;
    mhzSum += mhz, mhzMin = std::min(mhzMin, mhz), mhzMax = std::max(mhzMax, mhz);
    // two waves share a SIMD: per SIMD 2 x iters x 64 MFMAs in `cycles`
    cyclesPerMfma += cycles / (2.0 * iters * 64);
  }
  const double flops = double(workgroups) * 8 * iters * 64 * (16.0 * 16 * 32 * 2);
  const double tflops = flops * launches / (double(ms) * 1e-3) / 1e12;
  const double mhz = mhzSum / workgroups;
  std::printf("| %d | %.0f | %.0f | %.0f | %.2f | %.0f | %.1f %% | %.1f %% |\n",
              workgroups, mhz, mhzMin, mhzMax, cyclesPerMfma / workgroups,
              tflops, 100.0 * tflops / 2500.0,
              100.0 * (mhz / 2400.0) * (workgroups / 256.0));
  CHECK(hipFree(seed));
  CHECK(hipFree(stamps));
  CHECK(hipFree(sink));
}

int main(int argc, char **argv) {
  if (argc < 2 || (std::strcmp(argv[1], "launch") && std::strcmp(argv[1], "clock") &&
                   std::strcmp(argv[1], "stream"))) {
    std::fprintf(stderr, "usage: gpu_floor launch | gpu_floor clock "
                         "[workgroups ...] | gpu_floor stream\n");
    return 2;
  }
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  std::printf("device: %s, %d CUs, clockRate %d kHz\n\n", prop.gcnArchName,
              prop.multiProcessorCount, prop.clockRate);
  if (!std::strcmp(argv[1], "launch")) {
    std::printf("empty kernel, 200 dependent launches in a replayed HIP graph, "
                "median of 7 passes of 20 replays\n\n");
    std::printf("| grid (workgroups) | threads | LDS bytes | us per launch |\n");
    std::printf("|---|---|---|---|\n");
    const int shapes[][3] = {{1, 64, 0},      {1, 512, 0},       {224, 512, 0},
                             {224, 512, 163840}, {256, 512, 0},  {256, 640, 110592},
                             {256, 512, 163840}, {2048, 256, 0}, {2048, 512, 65536}};
    for (const auto &s : shapes)
      std::printf("| %d | %d | %d | %.2f |\n", s[0], s[1], s[2],
                  launchFloor(s[0], s[1], s[2]));
    return 0;
  }
  if (!std::strcmp(argv[1], "stream")) {
    const size_t outBytes = 19267584, inBytes = 4 * outBytes;
    const size_t outVecs = outBytes / 16;
    std::vector<uintx4 *> ins(4), outs(4);
    for (int i = 0; i != 4; ++i) {
      CHECK(hipMalloc(&ins[i], inBytes));
      CHECK(hipMemset(ins[i], i + 1, inBytes));
      CHECK(hipMalloc(&outs[i], outBytes));
    }
    const double bytes = double(inBytes + outBytes);
    std::printf("4 : 1 stream of %.0f bytes per launch (%zu read, %zu "
                "written), 4 buffer sets in turn, 200 launches in a replayed "
                "HIP graph, median of 7 passes\n\n",
                bytes, inBytes, outBytes);
    std::printf("| the four loads of an output | outputs per thread | loads "
                "and stores | us per launch | GB/s | of 8 TB/s |\n");
    std::printf("|---|---|---|---|---|---|\n");
    streamCeiling<1, false, false>("a plane apart", ins, outs, outVecs, bytes);
    streamCeiling<1, true, false>("a plane apart", ins, outs, outVecs, bytes);
    streamCeiling<2, true, false>("a plane apart", ins, outs, outVecs, bytes);
    streamCeiling<4, true, false>("a plane apart", ins, outs, outVecs, bytes);
    streamCeiling<1, false, true>("adjacent", ins, outs, outVecs, bytes);
    streamCeiling<1, true, true>("adjacent", ins, outs, outVecs, bytes);
    return 0;
  }
  std::printf("8 waves per workgroup (two per SIMD) of back-to-back "
              "v_mfma_f32_16x16x32_f16 (16 cycles each), one workgroup per "
              "CU, after 0.3 s of the same load\n\n");
  std::printf("| busy CUs | shader clock MHz (mean) | min | max | cycles per "
              "MFMA and SIMD | TFLOP/s sustained | of 2.5 PFLOP/s | clock / "
              "2400 x CUs / 256 |\n");
  std::printf("|---|---|---|---|---|---|---|---|\n");
  std::vector<int> counts;
  for (int i = 2; i < argc; ++i)
    counts.push_back(std::atoi(argv[i]));
  if (counts.empty())
    counts = {1, 64, 128, 192, 224, 256};
  for (int n : counts)
    clockUnderLoad(n);
  return 0;
}
