// Plain streaming kernels of known size: the yardstick for the decode kernels.
//   stream_read  reads `bytes` once the way the decode kernels read the caches: non-temporal 16-byte
//                loads from global memory straight into LDS, three 8 KB steps in flight per wavefront,
//                every wavefront a contiguous region
//   stream_copy  copies `bytes` (reads + writes them once)
// Their duration gives the HBM rate this GPU sustains for a working set of that size, and
// the hardware counters read for them calibrate FETCH_SIZE / WRITE_SIZE.
#include <atomic>

#include "common.cuh"
#include "launch.h"

namespace xllm_mi355 {

namespace {

constexpr int kStep = 8192;      // bytes a wavefront moves per step: 8 loads of 64 lanes x 16 bytes
constexpr int kRingSteps = 4;    // LDS ring per wavefront
constexpr int kReadLds = 4 * kRingSteps * kStep;

__global__ __launch_bounds__(256) void stream_read_kernel(const char* __restrict__ p, size_t bytes, u32* sink) {
  extern __shared__ __align__(16) char smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const u32 lds0 = static_cast<u32>(reinterpret_cast<uintptr_t>(smem)) + wave * kRingSteps * kStep;
  const size_t n_steps = bytes / kStep;
  const size_t workers = static_cast<size_t>(gridDim.x) * 4, w = static_cast<size_t>(blockIdx.x) * 4 + wave;
  const size_t s0 = w * n_steps / workers, s1 = (w + 1) * n_steps / workers;
  auto issue = [&](size_t s) {
    const char* g = p + s * kStep + lane * 16;
    const u32 base = __builtin_amdgcn_readfirstlane(lds0 + static_cast<u32>((s - s0) % kRingSteps) * kStep);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const u32 m0 = base + i * 1024;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(m0), "v"(g + i * 1024) : "memory");
    }
  };
  size_t ps = s0;
  for (int k = 0; k < kRingSteps - 1 && ps < s1; ++k, ++ps) issue(ps);
  u32 acc = 0;
  for (size_t s = s0; s < s1; ++s) {
    const size_t younger = ps - 1 - s;  // steps issued after s: at most kRingSteps - 2 here
    if (younger >= 2) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else if (younger == 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (ps < s1) issue(ps++);
    acc ^= *reinterpret_cast<volatile u32*>(smem + wave * kRingSteps * kStep + ((s - s0) % kRingSteps) * kStep + lane * 4);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // what is left of the last step
  if (blockIdx.x == 0)
    for (size_t i = n_steps * kStep + threadIdx.x * 16; i < bytes; i += 256 * 16) acc ^= ldg16_stream(p + i)[0];
  // never true for real data patterns; keeps the reads alive
  if (acc == 0x9e3779b9u && sink != nullptr) sink[0] = acc;
}

__global__ __launch_bounds__(256) void stream_copy_kernel(u32x4* __restrict__ dst,
                                                          const u32x4* __restrict__ src, size_t n_vec) {
  // every workgroup a contiguous share; a thread asks for eight vectors before it stores the first; bytes that are
  // read once and written once: non-temporal both ways
  const size_t per = (n_vec + gridDim.x - 1) / gridDim.x;
  const size_t lo = per * blockIdx.x;
  const size_t hi = lo + per < n_vec ? lo + per : n_vec;
  size_t i = lo + threadIdx.x;
  for (; i + 7 * 256 < hi; i += 8 * 256) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * 256);
#pragma unroll
    for (int u = 0; u < 8; ++u) __builtin_nontemporal_store(v[u], dst + i + u * 256);
  }
  for (; i < hi; i += 256) dst[i] = src[i];
}

}  // namespace

}  // namespace xllm_mi355

using namespace xllm_mi355;

extern "C" {

int xllm_mi355_stream_read(const void* src, size_t bytes, void* sink, void* stream) {
  if (src == nullptr || (reinterpret_cast<uintptr_t>(src) & 15) != 0 || bytes % 16 != 0) return XLLM_MI355_EALIGN;
  if (bytes == 0) return XLLM_MI355_OK;
  static std::atomic<uint64_t> configured{0};
  if (first_use_on_current_device(configured)) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(stream_read_kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, kReadLds);
    if (e != hipSuccess) return static_cast<int>(e);
  }
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  launch_timed(stream_read_kernel, dim3(cus > 0 ? cus : 256), dim3(256), kReadLds, static_cast<hipStream_t>(stream),
               static_cast<const char*>(src), bytes, static_cast<u32*>(sink));
  return static_cast<int>(hipGetLastError());
}

int xllm_mi355_stream_copy(void* dst, const void* src, size_t bytes, void* stream) {
  if (dst == nullptr || src == nullptr || ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) != 0 ||
      bytes % 16 != 0)
    return XLLM_MI355_EALIGN;
  if (bytes == 0) return XLLM_MI355_OK;
  launch_timed(stream_copy_kernel, dim3(2048), dim3(256), 0, static_cast<hipStream_t>(stream),
               static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), bytes / 16);
  return static_cast<int>(hipGetLastError());
}

}  // extern "C"
