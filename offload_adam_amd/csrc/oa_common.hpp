// Shared device/host helpers of liboffload_adam_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "offload_adam_hip.h"

// Every floating-point expression in this library is evaluated exactly as
// written: one IEEE rounding per operation, never contracted into an FMA.
#pragma clang fp contract(off)

namespace oa {

typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef short i16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned char u8x16 __attribute__((ext_vector_type(16)));
typedef unsigned char u8x8 __attribute__((ext_vector_type(8)));
typedef unsigned char u8x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;  // CDNA wavefront width

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) {
  return __uint_as_float(h << 16);
}

// Two fp32 -> packed bf16x2 (lo in bits 0..15) through the gfx950 hardware
// convert (v_cvt_pk_bf16_f32): round to nearest even, NaN stays a quiet NaN.
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  f32x2 in = {lo, hi};
  bf16x2_t out = __builtin_convertvector(in, bf16x2_t);
  return __builtin_bit_cast(uint32_t, out);
}

// One fp32 -> bf16 bits (in the low 16 bits of the result).
__device__ __forceinline__ uint32_t f32_to_bf16_1(float f) {
  return f32x2_to_bf16x2_bits(f, 0.0f) & 0xFFFFu;
}

// Low / high bf16 half of a packed dword, widened to fp32.
__device__ __forceinline__ float bf16lo_to_f32(uint32_t w) {
  return __uint_as_float(w << 16);
}
__device__ __forceinline__ float bf16hi_to_f32(uint32_t w) {
  return __uint_as_float(w & 0xFFFF0000u);
}

// The AdamW update of one element on folded (bias-corrected) betas, as
// src/offload_adam/kernels/fp32_master.py:46-53 writes it: M is the fp32 value
// being optimised, m / v the moments, omb = 1 - beta_hat.  One rounding per
// operation; sqrt and divide are correctly rounded (compile flags).
// Measurement switch, never set in the shipped build: 1 replaces the correctly
// rounded square root and divide by the hardware's approximate v_sqrt_f32 and
// v_rcp_f32 (about 20 instructions fewer per element).  Results then differ
// from the reference's; it exists to show what the exact arithmetic costs.
#ifndef OA_ADAM_APPROX_DIV_SQRT
#define OA_ADAM_APPROX_DIV_SQRT 0
#endif
__device__ __forceinline__ void adam_core(float& M, float g, float& m, float& v, bool decoupled,
                                          float lr, float wd, float lr_wd, float omb1,
                                          float omb2, float eps) {
  if (decoupled) {
    M = M - lr_wd * M;
  } else {
    g = g + wd * M;
  }
  m = m + omb1 * (g - m);
  v = v + omb2 * (g * g - v);
#if OA_ADAM_APPROX_DIV_SQRT
  const float denom = __builtin_amdgcn_sqrtf(v) + eps;
  M = M - (lr * m) * __builtin_amdgcn_rcpf(denom);
#else
  const float denom = sqrtf(v) + eps;
  M = M - (lr * m) / denom;
#endif
}

// Philox4x32-10 (Salmon et al., SC'11): round multipliers 0xD2511F53 and
// 0xCD9E8D57, key increments 0x9E3779B9 and 0xBB67AE85.
#ifndef OA_PHILOX_XOR3
#define OA_PHILOX_XOR3 1
#endif
struct Philox {
  uint32_t c0, c1, c2, c3;
};

// a ^ b ^ c in one instruction (gfx950's three-input bit operation with the
// truth table of a three-way xor); the compiler leaves two v_xor_b32 otherwise,
// and with one Philox block per element the update is bound by instruction issue.
__device__ __forceinline__ uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) {
#if OA_PHILOX_XOR3
  return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
#else
  return a ^ b ^ c;
#endif
}

__device__ __forceinline__ Philox philox4x32_10(uint32_t c0, uint32_t c1,
                                                uint32_t c2, uint32_t c3,
                                                uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t pb = (uint64_t)0xCD9E8D57u * (uint64_t)c2;
    const uint64_t pa = (uint64_t)0xD2511F53u * (uint64_t)c0;
    // the first round sees the constant words of the counter: plain xors fold away
    const uint32_t n0 = r == 0 ? (uint32_t)(pb >> 32) ^ c1 ^ k0 : xor3((uint32_t)(pb >> 32), c1, k0);
    const uint32_t n2 = r == 0 ? (uint32_t)(pa >> 32) ^ c3 ^ k1 : xor3((uint32_t)(pa >> 32), c3, k1);
    c1 = (uint32_t)pb;
    c3 = (uint32_t)pa;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return Philox{c0, c1, c2, c3};
}

// Wave64 all-lane sum via butterfly shuffles (every lane ends with the total).
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) x += __shfl_xor(x, off, kWave);
  return x;
}

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1)
    x = fmaxf(x, __shfl_xor(x, off, kWave));
  return x;
}

// Workgroup -> tile.  The dispatcher deals consecutive workgroups to the 8 XCDs
// round-robin (workgroup b runs on XCD b % 8), each with its own L2.  With
// tile = b every XCD touches every 8th tile of every array; mapping so that an
// XCD owns runs of CHUNK consecutive tiles gives each L2 and the memory channels
// behind it longer sequential streams (measured on a 4-read / 3-write stream
// kernel of this shape: +3 % at 15 GB, +10 % at 0.8 GB per launch).  The map is
// a bijection on [0, round_up(tiles, 8 * CHUNK)); grids are padded to that size
// and surplus workgroups exit.  CHUNK is a compile-time constant of each kernel
// family (0 = identity): the AdamW kernels and the encoders that read their
// elements through an AdamW update have tiles of different sizes.
#ifndef OA_CODEC_XCD_CHUNK
#define OA_CODEC_XCD_CHUNK 64  // tiles of 2048 elements
#endif
constexpr uint32_t kXcds = 8;
constexpr uint32_t kCodecXcdChunk = OA_CODEC_XCD_CHUNK;

template <uint32_t CHUNK>
__device__ __forceinline__ uint32_t xcd_tile(uint32_t b) {
  if (CHUNK == 0) return b;
  const uint32_t x = b % kXcds, j = b / kXcds;
  const uint32_t c = j / CHUNK, r = j % CHUNK;
  return (c * kXcds + x) * CHUNK + r;
}
inline uint32_t xcd_grid(uint32_t tiles, uint32_t chunk) {
  if (chunk == 0) return tiles;
  const uint32_t q = kXcds * chunk;
  return (tiles + q - 1) / q * q;
}


// Multi-tensor launches: `start[0..count]` are the prefix sums of the tensors'
// workgroup counts (count < 64, every tensor has at least one workgroup) and b <
// start[count].  Returns the tensor workgroup b belongs to, the same value in every
// lane: lane j compares b with the end of tensor j and the wave counts the tensors
// that end at or before b - one load and one ballot instead of a scan whose loads
// depend on each other.
__device__ __forceinline__ int tensor_of_block(uint32_t b, const uint32_t* start, int count) {
  const int lane = threadIdx.x & (kWave - 1);
  const uint32_t end = lane < count ? start[lane + 1] : 0xFFFFFFFFu;
  return __popcll(__ballot(b >= end));
}

inline bool aligned_to(const void* p, uintptr_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

inline int launch_status() { return static_cast<int>(hipGetLastError()); }

}  // namespace oa
