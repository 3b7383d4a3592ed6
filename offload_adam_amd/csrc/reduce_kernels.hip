// Gradient L2 norm (per parameter) and global clip coefficient for gfx950.
//
// Per-parameter norm: two launches.  The first streams the bf16 gradient with
// 128-bit non-temporal loads, one contiguous tile of 512 lanes x 4 loads per
// block, keeps fp32 partial sums, folds the lanes with a wave64 butterfly
// (__shfl_xor) and the waves of the block through LDS, and stores one partial
// per block.  The second, one block, folds the partials in index order
// (deterministic), takes the square root and writes the bf16 norm.  2 bytes of
// HBM traffic per element.
//
// A single launch in which the block that takes the last ticket of an atomic
// counter folds the partials was measured at 55 us for a 117 MB gradient
// against 25 us for the two launches: publishing a partial to another block
// needs an agent-scope release fence, which on this multi-die GPU writes the
// die's L2 back, and the tickets serialise on one address.
//
// Clip coefficient: one small block over the bf16 norms of all parameters.

#include <atomic>

#include "oa_common.hpp"

#pragma clang fp contract(off)

// Partial sums of oa_grad_norm_bf16_static: one copy of this array per GPU,
// held until the process ends.  In host code the name is only a handle for
// hipGetSymbolAddress; kernels are given the address that call returns.
static __device__ __align__(256) float scratch[OA_NORM_STATIC_PARTIALS];

namespace oa {
namespace {

#ifndef OA_NORM_THREADS
#define OA_NORM_THREADS 512
#endif
#ifndef OA_NORM_UNROLL
#define OA_NORM_UNROLL 4
#endif
constexpr int kThreads = OA_NORM_THREADS;   // partial kernel
constexpr int kFinalThreads = 1024;  // 4 partials per lane per trip: 16384 partials = 4 trips
constexpr int kClipThreads = 256;
constexpr int kUnroll = OA_NORM_UNROLL;  // 16-byte loads in flight per lane
constexpr int kMaxBlocks = 16384;
constexpr int64_t kTileGroups = (int64_t)kThreads * kUnroll;  // 8-element groups per tile

struct NormWorkspace {
  float partial[kMaxBlocks];
};

template <int T>
__device__ __forceinline__ float block_sum(float x, float* lds) {
  x = wave_sum(x);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) lds[wave] = x;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int w = 0; w < T / kWave; ++w) t += lds[w];
  __syncthreads();
  return t;
}

__device__ __forceinline__ float sq8(const u32x4 w, float acc) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float lo = bf16lo_to_f32(w[j]), hi = bf16hi_to_f32(w[j]);
    acc = fmaf(lo, lo, acc);
    acc = fmaf(hi, hi, acc);
  }
  return acc;
}

// Sum of squares of one block's share of a gradient, the same value in every lane.
// head = elements before the first 16-byte boundary, groups = aligned 8-element
// groups after it; head and tail elements are folded in by block 0.  Block b of
// `blocks` takes tiles b, b + blocks, ... (one tile each unless the tensor has
// more than kMaxBlocks tiles).
__device__ __forceinline__ float block_sumsq(const uint16_t* __restrict__ g, int64_t n, int head,
                                             int64_t groups, uint32_t block, uint32_t blocks,
                                             float* lds) {
  const u32x4* body = reinterpret_cast<const u32x4*>(g + head);
  const int64_t tiles = (groups + kTileGroups - 1) / kTileGroups;
  float acc = 0.0f;
  for (int64_t tile = block; tile < tiles; tile += blocks) {
    const int64_t base = tile * kTileGroups + threadIdx.x;
    u32x4 w[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int64_t i = base + (int64_t)k * kThreads;
      w[k] = i < groups ? __builtin_nontemporal_load(body + i) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) acc = sq8(w[k], acc);
  }

  if (block == 0) {
    const int64_t tail_start = head + groups * 8;
    const int64_t extra = head + (n - tail_start);  // < 16
    if (threadIdx.x < extra) {
      const int64_t t = threadIdx.x;
      const int64_t idx = t < head ? t : tail_start + (t - head);
      const float x = bf16_bits_to_f32(g[idx]);
      acc = fmaf(x, x, acc);
    }
  }
  return block_sum<kThreads>(acc, lds);
}

__global__ void __launch_bounds__(kThreads)
grad_norm_partial_kernel(const uint16_t* __restrict__ g, int64_t n, int head, int64_t groups,
                         float* __restrict__ partial, uint16_t* __restrict__ norm_direct,
                         float* __restrict__ sumsq_direct) {
  __shared__ float lds[kThreads / kWave];
  const float total = block_sumsq(g, n, head, groups, blockIdx.x, gridDim.x, lds);
  if (threadIdx.x == 0) {
    if (norm_direct) {
      // a one-block launch is its own final pass: the second launch would add this
      // one partial to zeros, which changes no bit
      if (sumsq_direct) *sumsq_direct = total;
      *norm_direct = (uint16_t)f32_to_bf16_1(sqrtf(total));
    } else {
      partial[blockIdx.x] = total;
    }
  }
}

// The fold of one tensor's partials, in index order, by one block of kFinalThreads lanes.
__device__ __forceinline__ void fold_partials(const float* __restrict__ partial, int blocks,
                                              uint16_t* __restrict__ norm_out,
                                              float* __restrict__ sumsq_out, float* lds) {
  float s = 0.0f;
  for (int b = threadIdx.x; b < blocks; b += 4 * kFinalThreads) {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int i = b + k * kFinalThreads;
      v[k] = i < blocks ? partial[i] : 0.0f;
    }
    s += (v[0] + v[1]) + (v[2] + v[3]);
  }
  s = block_sum<kFinalThreads>(s, lds);
  if (threadIdx.x == 0) {
    if (sumsq_out) *sumsq_out = s;
    *norm_out = (uint16_t)f32_to_bf16_1(sqrtf(s));
  }
}

__global__ void __launch_bounds__(kFinalThreads)
grad_norm_final_kernel(const float* __restrict__ partial, int blocks,
                       uint16_t* __restrict__ norm_out, float* __restrict__ sumsq_out) {
  __shared__ float lds[kFinalThreads / kWave];
  fold_partials(partial, blocks, norm_out, sumsq_out, lds);
}

// Multi-tensor form: one launch takes the partial sums of up to kNormMultiMax
// gradients (descriptors travel as kernel arguments), a second one folds every
// tensor's partials, one block per tensor.  Each tensor gets the block count, the
// tile -> block map and the fold order of its own two-launch norm, so the results
// are the same bits.  A gradient of a few thousand elements costs two launches
// when it is taken alone; here a whole model's worth of them shares two.
constexpr int kNormMultiMax = 36;

struct NormMultiArgs {
  const uint16_t* g[kNormMultiMax];
  int64_t n[kNormMultiMax];
  uint16_t* norm[kNormMultiMax];
  float* sumsq[kNormMultiMax];
  uint32_t block_start[kNormMultiMax + 1];  // first workgroup (= first partial) of each tensor
  int count;
};

__global__ void __launch_bounds__(kThreads)
grad_norm_multi_partial_kernel(const NormMultiArgs a, float* __restrict__ partial) {
  __shared__ float lds[kThreads / kWave];
  const uint32_t b = blockIdx.x;
  const int t = tensor_of_block(b, a.block_start, a.count);
  const uint16_t* g = a.g[t];
  const int64_t n = a.n[t];
  int64_t head = (int64_t)(((16 - (reinterpret_cast<uintptr_t>(g) & 15)) & 15) / 2);
  if (head > n) head = n;
  const int64_t groups = (n - head) / 8;
  const float total = block_sumsq(g, n, (int)head, groups, b - a.block_start[t],
                                  a.block_start[t + 1] - a.block_start[t], lds);
  if (threadIdx.x == 0) partial[b] = total;
}

__global__ void __launch_bounds__(kFinalThreads)
grad_norm_multi_final_kernel(const NormMultiArgs a, const float* __restrict__ partial) {
  __shared__ float lds[kFinalThreads / kWave];
  const int t = blockIdx.x;
  fold_partials(partial + a.block_start[t], (int)(a.block_start[t + 1] - a.block_start[t]),
                a.norm[t], a.sumsq[t], lds);
}

// total = bf16(sqrt(sum norms^2)); coef = min(bf16(bf16(1/bf16(total+1e-6)) * max_norm), 1)
// -- the bf16 0-dim tensor arithmetic of the reference's clip step, where
// `python_float / tensor` is evaluated as `tensor.reciprocal() * python_float`.
__global__ void __launch_bounds__(kClipThreads)
clip_coef_kernel(const uint16_t* __restrict__ norms, int64_t count, float max_norm,
                 uint16_t* __restrict__ total_out, uint16_t* __restrict__ coef_out) {
  __shared__ float lds[kClipThreads / kWave];
  float acc = 0.0f;
  for (int64_t i = threadIdx.x; i < count; i += kClipThreads) {
    const float x = bf16_bits_to_f32(norms[i]);
    acc = fmaf(x, x, acc);
  }
  const float s = block_sum<kClipThreads>(acc, lds);
  if (threadIdx.x == 0) {
    const uint32_t total = f32_to_bf16_1(sqrtf(s));
    const uint32_t t1 = f32_to_bf16_1(bf16_bits_to_f32(total) + 1e-6f);
    const uint32_t r = f32_to_bf16_1(1.0f / bf16_bits_to_f32(t1));
    const uint32_t c = f32_to_bf16_1(bf16_bits_to_f32(r) * max_norm);
    const float cf = bf16_bits_to_f32(c);
    if (total_out) *total_out = (uint16_t)total;
    *coef_out = (uint16_t)((cf > 1.0f) ? 0x3F80u : c);
  }
}

}  // namespace
}  // namespace oa

using namespace oa;

extern "C" size_t oa_norm_workspace_bytes(void) { return sizeof(NormWorkspace); }

namespace oa {
namespace {

// Workgroups (= partials) of the first launch for a gradient at `grad`: one per
// 32 KiB tile, at most kMaxBlocks; also yields the unaligned head and the number
// of aligned 8-element groups.
int64_t norm_blocks(const void* grad, int64_t n, int64_t* head_out, int64_t* groups_out) {
  const uintptr_t addr = reinterpret_cast<uintptr_t>(grad);
  int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / 2);
  if (head > n) head = n;
  const int64_t groups = (n - head) / 8;
  int64_t blocks = (groups + kTileGroups - 1) / kTileGroups;
  if (blocks < 1) blocks = 1;
  if (blocks > kMaxBlocks) blocks = kMaxBlocks;
  if (head_out) *head_out = head;
  if (groups_out) *groups_out = groups;
  return blocks;
}

// The two launches of a norm; `partial` holds at least kMaxBlocks floats.
int launch_grad_norm(const void* grad, int64_t n, void* norm_out, void* sumsq_out,
                     float* partial, hipStream_t s) {
  int64_t head = 0, groups = 0;
  const int64_t blocks = norm_blocks(grad, n, &head, &groups);
  const bool single = blocks == 1;  // tensors of up to 16384 elements: one launch, not two
  hipLaunchKernelGGL(grad_norm_partial_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, s,
                     static_cast<const uint16_t*>(grad), n, (int)head, groups, partial,
                     single ? static_cast<uint16_t*>(norm_out) : nullptr,
                     single ? static_cast<float*>(sumsq_out) : nullptr);
  int rc = launch_status();
  if (single) return rc;
  if (rc) return rc;
  hipLaunchKernelGGL(grad_norm_final_kernel, dim3(1), dim3(kFinalThreads), 0, s, partial,
                     (int)blocks, static_cast<uint16_t*>(norm_out),
                     static_cast<float*>(sumsq_out));
  return launch_status();
}

// Device address of `scratch` on each GPU (every GPU holds its own copy of the
// array at its own address), looked up once per device with that device current.
constexpr int kMaxDevices = 64;
std::atomic<float*> g_scratch_addr[kMaxDevices];

int static_scratch(float** out) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return static_cast<int>(err);
  if (dev < 0 || dev >= kMaxDevices) return OA_ERANGE;
  float* addr = g_scratch_addr[dev].load(std::memory_order_acquire);
  if (!addr) {
    void* sym = nullptr;
    err = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return static_cast<int>(err);
    if (!sym) return static_cast<int>(hipErrorInvalidSymbol);
    addr = static_cast<float*>(sym);
    g_scratch_addr[dev].store(addr, std::memory_order_release);  // same value from any thread
  }
  *out = addr;
  return 0;
}

}  // namespace
}  // namespace oa

static_assert(OA_NORM_STATIC_PARTIALS >= kMaxBlocks, "scratch must hold every block's partial");
static_assert(OA_NORM_STATIC_MAX_ELEMS > 0, "");

extern "C" int oa_grad_norm_bf16(const void* grad, int64_t n, void* norm_out,
                                 void* sumsq_out, void* workspace, void* stream) {
  if (n < 0 || !norm_out || !workspace || (n > 0 && !grad)) return OA_EINVAL;
  if (!aligned_to(grad, 2) || !aligned_to(norm_out, 2) || !aligned_to(workspace, 64) ||
      (sumsq_out && !aligned_to(sumsq_out, 4)))
    return OA_EALIGN;
  return launch_grad_norm(grad, n, norm_out, sumsq_out,
                          static_cast<NormWorkspace*>(workspace)->partial,
                          static_cast<hipStream_t>(stream));
}

extern "C" int oa_grad_norm_bf16_static(const void* grad, int64_t n, void* norm_out,
                                        void* sumsq_out, void* stream) {
  if (n < 0 || !norm_out || (n > 0 && !grad)) return OA_EINVAL;
  if (n > OA_NORM_STATIC_MAX_ELEMS) return OA_ERANGE;
  if (!aligned_to(grad, 2) || !aligned_to(norm_out, 2) ||
      (sumsq_out && !aligned_to(sumsq_out, 4)))
    return OA_EALIGN;
  float* partial = nullptr;
  int rc = static_scratch(&partial);
  if (rc) return rc;
  // Every partial the second launch reads is written by the first: nothing in
  // the array has to start at zero.
  return launch_grad_norm(grad, n, norm_out, sumsq_out, partial,
                          static_cast<hipStream_t>(stream));
}

extern "C" size_t oa_norm_multi_workspace_bytes(void) {
  return sizeof(float) * (size_t)kNormMultiMax * kMaxBlocks;
}

extern "C" int oa_grad_norm_multi(int count, const void* const* grads, const int64_t* numels,
                                  void* const* norm_outs, void* const* sumsq_outs,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  if (count < 0) return OA_EINVAL;
  if (count == 0) return 0;
  if (!grads || !numels || !norm_outs || !workspace) return OA_EINVAL;
  if (workspace_bytes < sizeof(NormWorkspace)) return OA_EINVAL;  // one tensor must always fit
  if (!aligned_to(workspace, 64)) return OA_EALIGN;
  // Validate everything before the first launch.
  for (int i = 0; i < count; ++i) {
    if (numels[i] < 0 || !norm_outs[i] || (numels[i] > 0 && !grads[i])) return OA_EINVAL;
    if (!aligned_to(grads[i], 2) || !aligned_to(norm_outs[i], 2) ||
        (sumsq_outs && sumsq_outs[i] && !aligned_to(sumsq_outs[i], 4)))
      return OA_EALIGN;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* partial = static_cast<float*>(workspace);
  const uint64_t capacity = workspace_bytes / sizeof(float);  // partials one launch may write

  NormMultiArgs a;
  a.count = 0;
  a.block_start[0] = 0;
  auto flush = [&]() -> int {
    if (a.count == 0) return 0;
    hipLaunchKernelGGL(grad_norm_multi_partial_kernel, dim3(a.block_start[a.count]),
                       dim3(kThreads), 0, s, a, partial);
    int rc = launch_status();
    if (rc) return rc;
    hipLaunchKernelGGL(grad_norm_multi_final_kernel, dim3((unsigned)a.count),
                       dim3(kFinalThreads), 0, s, a, partial);
    a.count = 0;
    return launch_status();
  };
  // Launches on one stream run in order: the next group's partials overwrite the
  // workspace only after this group's fold has read it.
  for (int i = 0; i < count; ++i) {
    const uint64_t blocks = (uint64_t)norm_blocks(grads[i], numels[i], nullptr, nullptr);
    if (a.count == kNormMultiMax || a.block_start[a.count] + blocks > capacity) {
      int rc = flush();
      if (rc) return rc;
    }
    const int j = a.count;
    a.g[j] = static_cast<const uint16_t*>(grads[i]);
    a.n[j] = numels[i];
    a.norm[j] = static_cast<uint16_t*>(norm_outs[i]);
    a.sumsq[j] = sumsq_outs ? static_cast<float*>(sumsq_outs[i]) : nullptr;
    a.block_start[j + 1] = a.block_start[j] + (uint32_t)blocks;
    a.count = j + 1;
  }
  return flush();
}

extern "C" int oa_clip_coef_bf16(const void* norms, int64_t count, float max_norm,
                                 void* total_out, void* coef_out, void* stream) {
  if (count < 0 || !coef_out || (count > 0 && !norms)) return OA_EINVAL;
  if (!aligned_to(norms, 2) || !aligned_to(coef_out, 2) ||
      (total_out && !aligned_to(total_out, 2)))
    return OA_EALIGN;
  hipLaunchKernelGGL(clip_coef_kernel, dim3(1), dim3(kClipThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(norms),
                     count, max_norm, static_cast<uint16_t*>(total_out),
                     static_cast<uint16_t*>(coef_out));
  return launch_status();
}
