// Ceiling of the operand stream of a tiled GEMM on one MI355X: direct-to-LDS loads of HBM-resident
// panels that `share` workgroups of one XCD read at the same time, with no arithmetic at all.
//
// A 256x256 GEMM tile streams two 2 MB operand panels (k = 4096, bf16); the m-tiles next to it share
// one, the n-tiles next to it the other. This program reproduces only that traffic: 2048 workgroups
// of 8 waves (8 per CU, one after the other), each streaming one 2 MB region in 1 KB wave loads
// (global_load_lds_dwordx4) with a bounded number outstanding; groups of `share` workgroups that run
// on the same XCD at the same time read the same region. `stagger` starts sharer i at load
// i * stagger of the region (wrapping), to see whether sharers that are not in lock step do better.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
typedef __attribute__((address_space(1))) const void gvoid;
typedef __attribute__((address_space(3))) void lvoid;

template <int INFLIGHT>
__global__ __launch_bounds__(512) void stream(const unsigned char* src, size_t region_bytes, int share, int stagger) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, wave = tid >> 6;
  // Workgroup b runs on XCD b % 8; `share` consecutive workgroups of one XCD take the same region.
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const unsigned char* base = src + (size_t)(xcd * 64 + (idx / share) % 64) * region_bytes;
  const size_t per_iter = 512 * 16;  // one 1 KB load per wave
  const size_t iters = region_bytes / per_iter;
  const size_t start = (size_t)(idx % share) * stagger % iters;
  for (size_t it0 = 0; it0 < iters; ++it0) {
    size_t it = it0 + start;
    if (it >= iters) it -= iters;
    __builtin_amdgcn_global_load_lds((gvoid*)(base + it * per_iter + tid * 16),
                                     (lvoid*)(smem + ((it % 8) * 8 + wave) * 1024), 16, 0, 0);
    // keep INFLIGHT loads outstanding per wave (vmcnt: bits 3:0 and 15:14; other counters: no wait)
    if (INFLIGHT == 4) __builtin_amdgcn_s_waitcnt(0x0f70 | 3);
    if (INFLIGHT == 8) __builtin_amdgcn_s_waitcnt(0x0f70 | 7);
    if (INFLIGHT == 16) __builtin_amdgcn_s_waitcnt(0x0f70 | 15);
  }
  __builtin_amdgcn_s_waitcnt(0);
}

int main() {
  const size_t region = 2 << 20;  // 512 regions of 2 MB = 1 GB, far beyond the caches
  unsigned char* src;
  CK(hipMalloc(&src, region * 512));
  CK(hipMemset(src, 1, region * 512));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  CK(hipFuncSetAttribute((const void*)stream<4>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  CK(hipFuncSetAttribute((const void*)stream<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  CK(hipFuncSetAttribute((const void*)stream<16>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  const int grid = 2048;
  auto run = [&](int share, int inflight, int stagger) {
    auto launch = [&]() {
      if (inflight == 4) stream<4><<<grid, 512, 65536>>>(src, region, share, stagger);
      if (inflight == 8) stream<8><<<grid, 512, 65536>>>(src, region, share, stagger);
      if (inflight == 16) stream<16><<<grid, 512, 65536>>>(src, region, share, stagger);
    };
    launch();
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    launch();
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    const double bytes = (double)grid * region;
    printf("share=%2d  in flight per wave=%2d KB  stagger=%2d loads: %.3f ms  into LDS %5.2f TB/s (%5.1f GB/s per CU)  distinct bytes %4.2f TB/s\n",
           share, inflight, stagger, ms, bytes / ms / 1e9, bytes / ms / 1e6 / 256, bytes / share / ms / 1e9);
  };
  for (int share : {1, 2, 4, 8, 32})
    for (int inflight : {4, 8, 16}) run(share, inflight, 0);
  for (int share : {4, 8})
    for (int stagger : {1, 2, 4, 8, 16}) run(share, 8, stagger);
  return 0;
}
