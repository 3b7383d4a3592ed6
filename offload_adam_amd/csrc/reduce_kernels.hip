// Gradient L2 norm (per parameter) and global clip coefficient for gfx950.
//
// Per-parameter norm: one launch.  Lanes stream the bf16 gradient with 128-bit
// loads and keep fp32 partial sums; a wave64 butterfly (__shfl_xor) folds the
// lanes, LDS folds the waves of a block, each block stores one partial, and
// the block that takes the last ticket folds the partials in index order
// (deterministic), takes the square root and writes the bf16 norm.  2 bytes of
// HBM traffic per element.
//
// Clip coefficient: one small block over the bf16 norms of all parameters.

#include "oa_common.hpp"

#pragma clang fp contract(off)

namespace oa {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kMaxBlocks = 1024;
constexpr int kUnroll = 4;  // 16-byte loads in flight per lane

struct NormWorkspace {
  unsigned int ticket;  // blocks that have stored their partial; 0 between launches
  unsigned int pad[15];
  float partial[kMaxBlocks];
};

__device__ __forceinline__ float block_sum(float x, float* lds) {
  x = wave_sum(x);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) lds[wave] = x;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) t += lds[w];
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

// head = elements before the first 16-byte boundary, groups = aligned 8-element
// groups after it; head and tail elements are folded in by block 0.
__global__ void __launch_bounds__(kThreads)
grad_norm_kernel(const uint16_t* __restrict__ g, int64_t n, int head, int64_t groups,
                 uint16_t* __restrict__ norm_out, float* __restrict__ sumsq_out,
                 NormWorkspace* __restrict__ ws) {
  __shared__ float lds[kWaves];
  __shared__ bool is_last;

  const u32x4* body = reinterpret_cast<const u32x4*>(g + head);
  float acc = 0.0f;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  for (; i + (kUnroll - 1) * stride < groups; i += kUnroll * stride) {
    u32x4 w[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) w[k] = __builtin_nontemporal_load(body + i + k * stride);
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) acc = sq8(w[k], acc);
  }
  for (; i < groups; i += stride) acc = sq8(__builtin_nontemporal_load(body + i), acc);

  if (blockIdx.x == 0) {
    const int64_t tail_start = head + groups * 8;
    const int64_t extra = head + (n - tail_start);  // < 16
    if (threadIdx.x < extra) {
      const int64_t idx = threadIdx.x < head ? threadIdx.x : tail_start + (threadIdx.x - head);
      const float x = bf16_bits_to_f32(g[idx]);
      acc = fmaf(x, x, acc);
    }
  }

  const float total = block_sum(acc, lds);
  if (threadIdx.x == 0) {
    // Publish this block's partial, then take a ticket.  The fence orders the
    // store before the ticket for whichever block reads the partials.
    __hip_atomic_store(&ws->partial[blockIdx.x], total, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    __threadfence();
    const unsigned int t = atomicAdd(&ws->ticket, 1u);
    is_last = (t == gridDim.x - 1);
  }
  __syncthreads();
  if (!is_last) return;

  __threadfence();
  float s = 0.0f;
  for (unsigned int b = threadIdx.x; b < gridDim.x; b += kThreads)
    s += __hip_atomic_load(&ws->partial[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  s = block_sum(s, lds);
  if (threadIdx.x == 0) {
    if (sumsq_out) *sumsq_out = s;
    *norm_out = (uint16_t)f32_to_bf16_1(sqrtf(s));
    __hip_atomic_store(&ws->ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// total = bf16(sqrt(sum norms^2)); coef = min(bf16(bf16(1/bf16(total+1e-6)) * max_norm), 1)
// -- the bf16 0-dim tensor arithmetic of the reference's clip step, where
// `python_float / tensor` is evaluated as `tensor.reciprocal() * python_float`.
__global__ void __launch_bounds__(kThreads)
clip_coef_kernel(const uint16_t* __restrict__ norms, int64_t count, float max_norm,
                 uint16_t* __restrict__ total_out, uint16_t* __restrict__ coef_out) {
  __shared__ float lds[kWaves];
  float acc = 0.0f;
  for (int64_t i = threadIdx.x; i < count; i += kThreads) {
    const float x = bf16_bits_to_f32(norms[i]);
    acc = fmaf(x, x, acc);
  }
  const float s = block_sum(acc, lds);
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

extern "C" int oa_grad_norm_bf16(const void* grad, int64_t n, void* norm_out,
                                 void* sumsq_out, void* workspace, void* stream) {
  if (n < 0 || !norm_out || !workspace || (n > 0 && !grad)) return OA_EINVAL;
  if (!aligned_to(grad, 2) || !aligned_to(norm_out, 2) || !aligned_to(workspace, 64) ||
      (sumsq_out && !aligned_to(sumsq_out, 4)))
    return OA_EALIGN;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(grad);
  int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / 2);
  if (head > n) head = n;
  const int64_t groups = (n - head) / 8;
  int64_t blocks = (groups + (int64_t)kThreads * kUnroll - 1) / ((int64_t)kThreads * kUnroll);
  if (blocks < 1) blocks = 1;
  if (blocks > kMaxBlocks) blocks = kMaxBlocks;
  hipLaunchKernelGGL(grad_norm_kernel, dim3((unsigned)blocks), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(grad), n,
                     (int)head, groups, static_cast<uint16_t*>(norm_out),
                     static_cast<float*>(sumsq_out), static_cast<NormWorkspace*>(workspace));
  return launch_status();
}

extern "C" int oa_clip_coef_bf16(const void* norms, int64_t count, float max_norm,
                                 void* total_out, void* coef_out, void* stream) {
  if (count < 0 || !coef_out || (count > 0 && !norms)) return OA_EINVAL;
  if (!aligned_to(norms, 2) || !aligned_to(coef_out, 2) ||
      (total_out && !aligned_to(total_out, 2)))
    return OA_EALIGN;
  hipLaunchKernelGGL(clip_coef_kernel, dim3(1), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(norms),
                     count, max_norm, static_cast<uint16_t*>(total_out),
                     static_cast<uint16_t*>(coef_out));
  return launch_status();
}
