// Pinned host memory with a NUMA preference, GPU -> NUMA node lookup, and the
// asynchronous copy primitive of the host<->device streaming path.
//
// Pinned memory comes from hipHostMalloc (page-locked at allocation, exact size
// rounded to 4 KiB pages, no power-of-two rounding).  A NUMA preference is
// applied by setting the calling thread's memory policy to MPOL_PREFERRED for
// the duration of the allocation and asking HIP to honour the thread policy
// (hipHostMallocNumaUser); MPOL_PREFERRED is soft, so a full node spills to
// other nodes instead of failing.
//
// Zero-fill runs on the GPU (hipMemset on the pinned pointer, a fill kernel
// writing across the host link at ~50 GB/s).  The mapping is a device-file
// mapping whose pages enter the CPU page table one 4 KiB fault at a time: the
// first CPU write pass over a fresh buffer runs at 2.8 GB/s however many threads
// share it (measured: 43.7 ms per 117 MiB with 1 or 16 threads; huge-page and
// populate advice do not apply to such a mapping), which made 45 GiB of
// optimizer state take 17 s to create.  The optimizer never touches its state
// buffers from the CPU, so those faults are simply not taken; code that does read
// a buffer on the CPU later faults in only what it reads.  The CPU fill remains
// as the fallback when the GPU fill is refused.

#include <errno.h>
#include <string.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <algorithm>
#include <cstdio>
#include <thread>
#include <vector>

#include "oa_common.hpp"

namespace {

constexpr size_t kPage = 4096;
constexpr int kMpolDefault = 0;
constexpr int kMpolPreferred = 1;

long set_mempolicy_raw(int mode, const unsigned long* mask, unsigned long maxnode) {
  return syscall(SYS_set_mempolicy, mode, mask, maxnode);
}

void parallel_zero(char* p, size_t bytes) {
  constexpr size_t kChunk = size_t(64) << 20;
  size_t want = bytes / kChunk;
  unsigned hw = std::thread::hardware_concurrency();
  size_t nthreads = std::min<size_t>(std::min<size_t>(want, hw ? hw : 1), 16);
  if (nthreads <= 1) {
    memset(p, 0, bytes);
    return;
  }
  std::vector<std::thread> pool;
  size_t per = ((bytes / nthreads) + kPage - 1) / kPage * kPage;
  for (size_t t = 0; t < nthreads; ++t) {
    size_t off = t * per;
    if (off >= bytes) break;
    size_t len = std::min(per, bytes - off);
    pool.emplace_back([p, off, len] { memset(p + off, 0, len); });
  }
  for (auto& th : pool) th.join();
}

}  // namespace

extern "C" int oa_pinned_alloc(size_t bytes, int numa_node, void** out, int* os_errno) {
  if (os_errno) *os_errno = 0;
  if (!out || numa_node < -1 || numa_node >= 1024) return OA_EINVAL;
  *out = nullptr;
  size_t size = (bytes + kPage - 1) / kPage * kPage;
  if (size == 0) size = kPage;

  unsigned int flags = hipHostMallocDefault;
  bool policy_set = false;
  if (numa_node >= 0) {
    unsigned long mask[16] = {0};
    mask[numa_node / (8 * sizeof(unsigned long))] |= 1UL << (numa_node % (8 * sizeof(unsigned long)));
    if (set_mempolicy_raw(kMpolPreferred, mask, 8 * sizeof(mask)) != 0) {
      if (os_errno) *os_errno = errno;
      return OA_EOS;
    }
    policy_set = true;
    flags |= hipHostMallocNumaUser;
  }
  void* p = nullptr;
  hipError_t err = hipHostMalloc(&p, size, flags);
  if (policy_set) set_mempolicy_raw(kMpolDefault, nullptr, 0);
  if (err != hipSuccess) {
    (void)hipGetLastError();
    return static_cast<int>(err);
  }
  if (hipMemset(p, 0, size) != hipSuccess) {  // synchronous: zeroed on return
    (void)hipGetLastError();
    parallel_zero(static_cast<char*>(p), size);
  }
  *out = p;
  return 0;
}

extern "C" int oa_pinned_probe(size_t bytes) {
  size_t size = (bytes + kPage - 1) / kPage * kPage;
  if (size == 0) size = kPage;
  void* p = nullptr;
  hipError_t err = hipHostMalloc(&p, size, hipHostMallocDefault);
  if (err != hipSuccess) {
    (void)hipGetLastError();
    return static_cast<int>(err);
  }
  return static_cast<int>(hipHostFree(p));
}

extern "C" int oa_pinned_free(void* ptr) {
  if (!ptr) return 0;
  return static_cast<int>(hipHostFree(ptr));
}

extern "C" int oa_gpu_numa_node(int device, int* node_out) {
  if (!node_out || device < 0) return OA_EINVAL;
  *node_out = -1;
  char bus[32] = {0};
  hipError_t err = hipDeviceGetPCIBusId(bus, sizeof(bus), device);
  if (err != hipSuccess) {
    (void)hipGetLastError();
    return static_cast<int>(err);
  }
  for (char* c = bus; *c; ++c)
    if (*c >= 'A' && *c <= 'F') *c = static_cast<char>(*c - 'A' + 'a');
  char path[128];
  snprintf(path, sizeof(path), "/sys/bus/pci/devices/%s/numa_node", bus);
  FILE* f = fopen(path, "r");
  if (!f) return 0;  // unknown: -1
  int node = -1;
  if (fscanf(f, "%d", &node) != 1) node = -1;
  fclose(f);
  *node_out = node;
  return 0;
}

namespace {

typedef unsigned int copy_u32x4 __attribute__((ext_vector_type(4)));

constexpr int kCopyThreads = 1024;
constexpr int kCopyUnroll = 4;

// Grid-stride copy with 128-bit accesses.  Either side may be page-locked host
// memory: the lanes then read or write it across the host link directly.
// The kernel lives as long as the transfer, and a compute unit that hosts one
// of its waves cannot take a workgroup of a GEMM that wants whole register
// files (measured: 64 workgroups of 256 lanes on 64 CUs slowed concurrent GEMMs
// by 1.6x).  So it uses FEW, FAT workgroups - 1024 lanes with 4 loads in flight
// each - which fill the link from a handful of CUs and leave the rest alone.
__global__ void __launch_bounds__(kCopyThreads)
link_copy_kernel(const copy_u32x4* __restrict__ src, copy_u32x4* __restrict__ dst, size_t n16,
                 const unsigned char* __restrict__ src_tail, unsigned char* __restrict__ dst_tail,
                 unsigned tail) {
  const size_t stride = (size_t)gridDim.x * kCopyThreads;
  size_t i = (size_t)blockIdx.x * kCopyThreads + threadIdx.x;
  for (; i + (kCopyUnroll - 1) * stride < n16; i += kCopyUnroll * stride) {
    copy_u32x4 v[kCopyUnroll];
#pragma unroll
    for (int k = 0; k < kCopyUnroll; ++k) v[k] = __builtin_nontemporal_load(src + i + k * stride);
#pragma unroll
    for (int k = 0; k < kCopyUnroll; ++k) __builtin_nontemporal_store(v[k], dst + i + k * stride);
  }
  for (; i < n16; i += stride)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
  if (blockIdx.x == 0 && threadIdx.x < tail) dst_tail[threadIdx.x] = src_tail[threadIdx.x];
}

}  // namespace

extern "C" int oa_copy_kernel_async(void* dst, const void* src, size_t bytes, int workgroups,
                                    void* stream) {
  if (bytes == 0) return 0;
  if (!dst || !src || workgroups < 1 || workgroups > 65535) return OA_EINVAL;
  if (!oa::aligned_to(dst, 16) || !oa::aligned_to(src, 16)) return OA_EALIGN;
  const size_t n16 = bytes / 16;
  const unsigned tail = (unsigned)(bytes % 16);
  const unsigned char* s8 = static_cast<const unsigned char*>(src) + n16 * 16;
  unsigned char* d8 = static_cast<unsigned char*>(dst) + n16 * 16;
  size_t need = (n16 + kCopyThreads - 1) / kCopyThreads;
  unsigned grid = (unsigned)(need < (size_t)workgroups ? (need ? need : 1) : (size_t)workgroups);
  hipLaunchKernelGGL(link_copy_kernel, dim3(grid), dim3(kCopyThreads), 0,
                     static_cast<hipStream_t>(stream),
                     static_cast<const copy_u32x4*>(src), static_cast<copy_u32x4*>(dst), n16, s8,
                     d8, tail);
  return oa::launch_status();
}

extern "C" int oa_memcpy_async(void* dst, const void* src, size_t bytes, int kind,
                               void* stream) {
  if (bytes == 0) return 0;
  if (!dst || !src) return OA_EINVAL;
  hipMemcpyKind k;
  switch (kind) {
    case OA_COPY_H2D: k = hipMemcpyHostToDevice; break;
    case OA_COPY_D2H: k = hipMemcpyDeviceToHost; break;
    case OA_COPY_D2D: k = hipMemcpyDeviceToDevice; break;
    default: return OA_EINVAL;
  }
  return static_cast<int>(hipMemcpyAsync(dst, src, bytes, k, static_cast<hipStream_t>(stream)));
}
