// libfusedmm_amd_probes.so: the benchmark's yardsticks (see fusedmm_probes.h).  A library
// of its own, so that the product libraries carry no measuring code.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "fusedmm_probes.h"

namespace {

constexpr int kBlockThreads = 256;

// Plain 16-byte copy of known size: the yardstick the traffic counters
// (FETCH_SIZE / WRITE_SIZE) of the product's kernels are scaled by.
__global__ __launch_bounds__(kBlockThreads) void copy_probe_kernel(float4 *dst, const float4 *src, int64_t n16)
{
   for (int64_t i = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x; i < n16; i += (int64_t)gridDim.x * kBlockThreads)
      dst[i] = src[i];
}


// Read-only stream of known size: every thread keeps U independent 16-byte loads
// in flight and folds what it read into one word, stored only if it is a value
// the data never produces, so the loads cannot be dropped and nothing is
// written.  The yardstick for what this GPU's memory system delivers to reads alone.
typedef unsigned int probe16_t __attribute__((ext_vector_type(4)));
template <int U, bool NT>
__global__ __launch_bounds__(kBlockThreads) void read_probe_kernel(const probe16_t *src, int64_t n16, unsigned int *sink)
{
   const int64_t stride = (int64_t)gridDim.x * kBlockThreads;
   unsigned int acc = 0u;
   int64_t i = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x;
   for (; i + (U - 1) * stride < n16; i += U * stride)
   {
      probe16_t v[U];
#pragma unroll
      for (int u = 0; u < U; u++)
         v[u] = NT ? __builtin_nontemporal_load(src + i + u * stride) : src[i + u * stride];
#pragma unroll
      for (int u = 0; u < U; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
   }
   for (; i < n16; i += stride)
   {
      const probe16_t v = src[i];
      acc ^= v.x ^ v.y ^ v.z ^ v.w;
   }
   if (acc == 0x9E3779B9u) *sink = acc;
}

// Read-only gather of whole rows: row ids[j] of `row16` 16-byte pieces each (a power of
// two up to 64 * R), for j < n_ids, in the order given; a wavefront takes 64 / L rows at
// a time on L = min(64, row16) lanes each and keeps U such steps in flight.  Nothing but
// the loads and an exclusive-or: the yardstick for what the memory system delivers to
// gathers of rows of this size, as read_probe_kernel is for a stream.
template <int U, int R, bool NT>
__global__ __launch_bounds__(kBlockThreads) void gather_probe_kernel(const probe16_t *src, int row16, const unsigned int *ids,
                                                                     int64_t n_ids, unsigned int *sink)
{
   const int lane = threadIdx.x & 63;
   const int L = row16 / R, S = 64 / L;
   const int sub = lane / L, sl = lane % L;
   const int64_t wave = ((int64_t)blockIdx.x * kBlockThreads + threadIdx.x) >> 6;
   const int64_t nwaves = (int64_t)gridDim.x * (kBlockThreads / 64);
   unsigned int acc = 0u;
   for (int64_t b = wave * S * U; b < n_ids; b += nwaves * S * U)
   {
      int64_t row[U];
#pragma unroll
      for (int u = 0; u < U; u++)
      {
         const int64_t j = b + u * S + sub;
         row[u] = j < n_ids ? (int64_t)ids[j] : -1;
      }
      probe16_t v[U][R];
#pragma unroll
      for (int u = 0; u < U; u++)
#pragma unroll
         for (int r = 0; r < R; r++)
         {
            const probe16_t *at = src + row[u] * row16 + r * L + sl;
            if (row[u] >= 0) v[u][r] = NT ? __builtin_nontemporal_load(at) : *at;
            else v[u][r] = probe16_t{0u, 0u, 0u, 0u};
         }
#pragma unroll
      for (int u = 0; u < U; u++)
#pragma unroll
         for (int r = 0; r < R; r++) acc ^= v[u][r].x ^ v[u][r].y ^ v[u][r].z ^ v[u][r].w;
   }
   if (acc == 0x9E3779B9u) *sink = acc;
}


bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

int launched(const char *what)
{
   const hipError_t e = hipGetLastError();
   if (e == hipSuccess) return 0;
   fprintf(stderr, "fusedmm_amd probes: %s failed: %s\n", what, hipGetErrorString(e));
   return 1;
}

int cu_count()
{
   int dev = 0, cus = 0;
   if (hipGetDevice(&dev) != hipSuccess) return 256;
   if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) return 256;
   return cus;
}

}  // namespace

extern "C" {

__attribute__((visibility("default")))
int fusedMM_amd_copy_probe(void *dst, const void *src, int64_t bytes, void *stream)
{
   if (!dst || !src || bytes < 16 || (bytes & 15) || !aligned16(dst) || !aligned16(src)) return 1;
   hipLaunchKernelGGL(copy_probe_kernel, dim3((unsigned int)(cu_count() * 8)), dim3(kBlockThreads), 0, (hipStream_t)stream,
                      (float4 *)dst, (const float4 *)src, bytes / 16);
   return launched("copy probe launch");
}

__attribute__((visibility("default")))
int fusedMM_amd_read_probe(const void *src, int64_t bytes, int blocks_per_cu, int in_flight, int nontemporal,
                           void *sink, void *stream)
{
   if (!src || !sink || bytes < 16 || (bytes & 15) || !aligned16(src)) return 1;
   if (blocks_per_cu < 1) blocks_per_cu = 8;
   const dim3 grid((unsigned int)(cu_count() * blocks_per_cu)), block(kBlockThreads);
   const probe16_t *s4 = (const probe16_t *)src;
   unsigned int *out = (unsigned int *)sink;
   const int64_t n16 = bytes / 16;
   hipStream_t hs = (hipStream_t)stream;
#define FMM_PROBE(U_)                                                                                     \
   if (nontemporal) hipLaunchKernelGGL((read_probe_kernel<U_, true>), grid, block, 0, hs, s4, n16, out);  \
   else hipLaunchKernelGGL((read_probe_kernel<U_, false>), grid, block, 0, hs, s4, n16, out)
   if (in_flight >= 16) { FMM_PROBE(16); }
   else if (in_flight >= 8) { FMM_PROBE(8); }
   else if (in_flight >= 4) { FMM_PROBE(4); }
   else { FMM_PROBE(2); }
#undef FMM_PROBE
   return launched("read probe launch");
}

__attribute__((visibility("default")))
int fusedMM_amd_gather_probe(const void *src, int row_bytes, const unsigned int *ids, int64_t n_ids, int blocks_per_cu,
                             int in_flight, int nontemporal, void *sink, void *stream)
{
   if (!src || !ids || !sink || n_ids < 1 || !aligned16(src)) return 1;
   if (row_bytes < 16 || row_bytes > 2048 || (row_bytes & (row_bytes - 1))) return 1;
   if (blocks_per_cu < 1) blocks_per_cu = 4;
   const dim3 grid((unsigned int)(cu_count() * blocks_per_cu)), block(kBlockThreads);
   const probe16_t *s4 = (const probe16_t *)src;
   unsigned int *out = (unsigned int *)sink;
   const int row16 = row_bytes / 16;
   hipStream_t hs = (hipStream_t)stream;
#define FMM_GPROBE(U_, R_)                                                                                              \
   if (nontemporal) hipLaunchKernelGGL((gather_probe_kernel<U_, R_, true>), grid, block, 0, hs, s4, row16, ids, n_ids, out); \
   else hipLaunchKernelGGL((gather_probe_kernel<U_, R_, false>), grid, block, 0, hs, s4, row16, ids, n_ids, out)
   if (row16 > 64)   // 2 KiB rows: two pieces per lane
   {
      if (in_flight >= 8) { FMM_GPROBE(8, 2); }
      else { FMM_GPROBE(4, 2); }
   }
   else if (in_flight >= 16) { FMM_GPROBE(16, 1); }
   else if (in_flight >= 8) { FMM_GPROBE(8, 1); }
   else { FMM_GPROBE(4, 1); }
#undef FMM_GPROBE
   return launched("gather probe launch");
}

}  // extern "C"
