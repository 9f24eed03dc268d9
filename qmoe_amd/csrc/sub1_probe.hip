// Gather-rate probe: how many nanoseconds a compute unit needs per wavefront
// instruction that reads one random dword per lane, from LDS or from a small
// global table (L1 / L2 resident).  The decode kernels are bound by exactly
// this rate (one table read and three activation reads per codeword), so the
// probe states the bound on the machine at hand.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <vector>

#include "sub1_common.h"

namespace {

using sub1::fail;

constexpr int kThreads = 1024;   // 16 wavefronts: what the decode kernels run with

// Every lane walks its own pseudo-random sequence of indices below `words`
// (a power of two); kPerStep independent gathers per step keep several in
// flight, as the decode loop does.  Time runs from the barrier before the loop
// to the last wavefront's end (the hardware favours the oldest wavefront, so
// one wavefront's own time says little), on the constant 100 MHz counter.
template <bool kLds, int kPerStep>
__global__ __launch_bounds__(kThreads) void gather_probe_kernel(const uint32_t *table, int words,
                                                                int steps, uint32_t *sink,
                                                                unsigned long long *ticks) {
  extern __shared__ uint32_t lds[];
  if (kLds)
    for (int i = threadIdx.x; i < words; i += kThreads) lds[i] = table[i];
  __syncthreads();
  const uint32_t mask = static_cast<uint32_t>(words - 1);
  uint32_t r = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
  uint32_t idx[kPerStep], stride[kPerStep];
#pragma unroll
  for (int u = 0; u < kPerStep; u++) {
    r = r * 1664525u + 1013904223u;
    idx[u] = (r >> 8) & mask;
    stride[u] = ((r >> 4) | 1u) & mask;
  }
  uint32_t acc = 0;
  __syncthreads();
  const unsigned long long t0 = wall_clock64();
  for (int i = 0; i < steps; i++) {
#pragma unroll
    for (int u = 0; u < kPerStep; u++) {
      idx[u] = (idx[u] + stride[u]) & mask;
      acc += kLds ? lds[idx[u]] : table[idx[u]];
    }
  }
  sink[blockIdx.x * kThreads + threadIdx.x] = acc;
  __syncthreads();
  const unsigned long long t1 = wall_clock64();
  if (threadIdx.x == 0) ticks[blockIdx.x] = t1 - t0;
}

}  // namespace

extern "C" int sub1_probe_gather(int from_lds, int words, int steps, double *ns_per_gather,
                                 void *stream) {
  if (!ns_per_gather) return fail(SUB1_ERR_NULL, "sub1_probe_gather: NULL argument");
  if (words < 64 || (words & (words - 1)) || steps < 1 || steps > (1 << 24))
    return fail(SUB1_ERR_SHAPE, "sub1_probe_gather: words %d (a power of two >= 64), steps %d",
                words, steps);
  if (from_lds && words > 32768)
    return fail(SUB1_ERR_SHAPE, "sub1_probe_gather: at most 32768 words fit LDS");
  hipStream_t s = static_cast<hipStream_t>(stream);
  int device = 0, cus = 0;
  HIP_TRY(hipGetDevice(&device));
  HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  constexpr int kPerStep = 4;
  uint32_t *table = nullptr, *sink = nullptr;
  unsigned long long *cycles = nullptr;
  HIP_TRY(hipMalloc(&table, static_cast<size_t>(words) * 4));
  HIP_TRY(hipMalloc(&sink, static_cast<size_t>(cus) * kThreads * 4));
  HIP_TRY(hipMalloc(&cycles, static_cast<size_t>(cus) * 8));
  HIP_TRY(hipMemsetAsync(table, 0, static_cast<size_t>(words) * 4, s));
  const size_t lds = from_lds ? static_cast<size_t>(words) * 4 : 0;
  if (from_lds) {
    HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gather_probe_kernel<true, kPerStep>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    for (int rep = 0; rep < 2; rep++)   // the first run warms caches and clocks
      gather_probe_kernel<true, kPerStep><<<cus, kThreads, lds, s>>>(table, words, steps, sink, cycles);
  } else {
    for (int rep = 0; rep < 2; rep++)
      gather_probe_kernel<false, kPerStep><<<cus, kThreads, 0, s>>>(table, words, steps, sink, cycles);
  }
  HIP_TRY(hipGetLastError());
  std::vector<unsigned long long> host(cus);
  HIP_TRY(hipMemcpyAsync(host.data(), cycles, host.size() * 8, hipMemcpyDeviceToHost, s));
  HIP_TRY(hipStreamSynchronize(s));
  HIP_TRY(hipFree(table));
  HIP_TRY(hipFree(sink));
  HIP_TRY(hipFree(cycles));
  double sum = 0;
  for (unsigned long long c : host) sum += static_cast<double>(c);
  // 16 wavefronts share the compute unit: each issued steps * kPerStep gathers
  *ns_per_gather = 10.0 * sum / cus / (static_cast<double>(steps) * kPerStep * (kThreads / 64));
  return SUB1_OK;
}
