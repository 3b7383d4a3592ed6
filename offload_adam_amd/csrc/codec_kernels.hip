// Weight-only quantisation codecs for gfx950: int8 per-row, int4 group-wise
// (GPTQ layout), NF4 block-wise (bitsandbytes layout), NVFP4 (e2m1 codes,
// float8_e4m3fn block scales, fp32 tensor scale).
//
// All kernels are HBM-bound byte shuffling: a lane owns an "octet" (8
// consecutive columns of one row), loaded and stored with one or two 128-bit
// accesses; group maxima are folded with wave64 sub-group shuffles; the int4
// layout, which is stored transposed, goes through an LDS tile so that both the
// row-major side and the column-major side are written in long runs.
//
// Arithmetic is fp32 with one rounding per operation (no FMA contraction,
// correctly rounded divide), which makes the codes bit-identical to the
// reference's pure-torch quantisers.
//
// Each codec has a fast path (cols % 8 == 0, 16-byte aligned rows, power-of-two
// group) and a generic path (one lane per group, any shape and alignment).

#include <type_traits>

#include "oa_common.hpp"

#pragma clang fp contract(off)

namespace oa {
namespace {

constexpr int kT = 256;  // 128 lanes: flat kernels within 2 %, int8 encoder 36 -> 56 us
constexpr float kEps = 1e-12f;

// ------------------------------------------------------------ element access

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  // The empty asm keeps the fp32 value as computed: without it the backend may
  // merge a preceding fp32 multiply with this convert into one mixed-precision
  // instruction that rounds the exact product straight to fp16 (one rounding
  // instead of two), which differs at fp32 ties.
  asm volatile("" : "+v"(f));
  return (uint32_t)__builtin_bit_cast(unsigned short, (_Float16)f);
}

template <int DT>
__device__ __forceinline__ float load1(const void* base, int64_t i) {
  if (DT != OA_F32 && DT != OA_BF16 && DT != OA_F16) return 0.0f;  // octet-only sources
  if (DT == OA_F32) return static_cast<const float*>(base)[i];
  const uint32_t h = static_cast<const uint16_t*>(base)[i];
  return DT == OA_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
}

// 8 consecutive elements starting at element i (16-byte aligned address).
template <int DT>
__device__ __forceinline__ void load8(const void* base, int64_t i, float (&x)[8]) {
  if (DT == OA_F32) {
    const f32x4* p = reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + i);
    const f32x4 a = __builtin_nontemporal_load(p), b = __builtin_nontemporal_load(p + 1);
#pragma unroll
    for (int k = 0; k < 4; ++k) { x[k] = a[k]; x[4 + k] = b[k]; }
  } else {
    const u32x4 w = __builtin_nontemporal_load(
        reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(base) + i));
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (DT == OA_BF16) {
        x[2 * k] = bf16lo_to_f32(w[k]);
        x[2 * k + 1] = bf16hi_to_f32(w[k]);
      } else {
        x[2 * k] = f16_bits_to_f32(w[k] & 0xFFFFu);
        x[2 * k + 1] = f16_bits_to_f32(w[k] >> 16);
      }
    }
  }
}

template <int DT>
__device__ __forceinline__ void store1(void* base, int64_t i, float v) {
  if (DT == OA_F32) static_cast<float*>(base)[i] = v;
  else if (DT == OA_BF16) static_cast<uint16_t*>(base)[i] = (uint16_t)f32_to_bf16_1(v);
  else static_cast<uint16_t*>(base)[i] = (uint16_t)f32_to_f16_bits(v);
}

// Streaming accesses are non-temporal where that measured faster on MI355X
// (4096 x 14336 weight): source loads and packed-code stores of every encoder,
// and the float stores of the int4 / NF4 / NVFP4 decoders (27.5 -> 22.6 us for
// NF4).  Loading the packed codes non-temporally in the decoders (22.6 -> 27.3 us)
// and storing non-temporally from the int8 decoder (31.6 -> 34.4 us) were slower,
// so those stay ordinary.
template <int DT, bool NT = true>
__device__ __forceinline__ void store8(void* base, int64_t i, const float (&x)[8]) {
  if (DT == OA_F32) {
    f32x4* p = reinterpret_cast<f32x4*>(static_cast<float*>(base) + i);
    if (NT) {
      __builtin_nontemporal_store(f32x4{x[0], x[1], x[2], x[3]}, p);
      __builtin_nontemporal_store(f32x4{x[4], x[5], x[6], x[7]}, p + 1);
    } else {
      p[0] = f32x4{x[0], x[1], x[2], x[3]};
      p[1] = f32x4{x[4], x[5], x[6], x[7]};
    }
  } else {
    u32x4 w;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (DT == OA_BF16) w[k] = f32x2_to_bf16x2_bits(x[2 * k], x[2 * k + 1]);
      else w[k] = f32_to_f16_bits(x[2 * k]) | (f32_to_f16_bits(x[2 * k + 1]) << 16);
    }
    u32x4* p = reinterpret_cast<u32x4*>(static_cast<uint16_t*>(base) + i);
    if (NT) __builtin_nontemporal_store(w, p);
    else *p = w;
  }
}

__device__ __forceinline__ float load_scale(const void* s, int dt, int64_t i) {
  if (dt == OA_F32) return load1<OA_F32>(s, i);
  if (dt == OA_BF16) return load1<OA_BF16>(s, i);
  return load1<OA_F16>(s, i);
}
__device__ __forceinline__ void store_scale(void* s, int dt, int64_t i, float v) {
  if (dt == OA_F32) store1<OA_F32>(s, i, v);
  else if (dt == OA_BF16) store1<OA_BF16>(s, i, v);
  else store1<OA_F16>(s, i, v);
}

// ---------------------------------------------------- fused AdamW source
// The encoders below read every element of their source exactly once.  With
// SRC = kSrcAdam that read *is* the fp32_master AdamW step of the element
// (src/offload_adam/kernels/fp32_master.py:19-59 without the bf16 copy of the
// master): gradient, moments and master are loaded, updated and stored back,
// and the new master values are what the encoder sees.  One pass over HBM then
// does what the reference does with a step kernel followed by
// `p.data.copy_(master)` (src/offload_adam/offload_adam.py:427-444), bit for bit.
// The four arrays are flat and contiguous, octet-aligned (cols % 8 == 0).
constexpr int kSrcAdam = 100;

struct AdamSrc {
  const uint16_t* g;     // bf16 gradient
  uint16_t* m;           // bf16 exp_avg
  uint16_t* v;           // bf16 exp_avg_sq
  float* master;         // fp32 master
  const uint16_t* clip;  // nullptr, or ONE bf16 clip coefficient on the device
  float lr, wd, lr_wd, omb1, omb2, eps;
  int decoupled;
};

// The loads of one octet, and the rest of its step.  Split so that a kernel with
// several octets per lane can issue all their loads before the first store
// (the compiler cannot move a later octet's loads above an earlier one's stores
// on its own: it has to assume they alias).
struct AdamRaw {
  u32x4 G, Mo, Vo;
  f32x4 A, B;
};

__device__ __forceinline__ void adam_load8(const AdamSrc& ad, int64_t i, AdamRaw& r) {
  r.G = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(ad.g + i));
  r.Mo = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(ad.m + i));
  r.Vo = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(ad.v + i));
  const f32x4* mp = reinterpret_cast<const f32x4*>(ad.master + i);
  r.A = mp[0];
  r.B = mp[1];
}

__device__ __forceinline__ void adam_finish8(const AdamSrc& ad, int64_t i, const AdamRaw& r,
                                             float (&x)[8]) {
  const float clip = ad.clip ? bf16_bits_to_f32(*ad.clip) : 1.0f;
  u32x4 Mn, Vn;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float m[2], v[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int e = 2 * j + h;
      float g = bf16_bits_to_f32((r.G[j] >> (16 * h)) & 0xFFFFu);
      if (ad.clip) g = bf16_bits_to_f32(f32_to_bf16_1(g * clip));
      m[h] = h ? bf16hi_to_f32(r.Mo[j]) : bf16lo_to_f32(r.Mo[j]);
      v[h] = h ? bf16hi_to_f32(r.Vo[j]) : bf16lo_to_f32(r.Vo[j]);
      float M = e < 4 ? r.A[e & 3] : r.B[e & 3];
      adam_core(M, g, m[h], v[h], ad.decoupled != 0, ad.lr, ad.wd, ad.lr_wd, ad.omb1, ad.omb2,
                ad.eps);
      x[e] = M;
    }
    Mn[j] = f32x2_to_bf16x2_bits(m[0], m[1]);
    Vn[j] = f32x2_to_bf16x2_bits(v[0], v[1]);
  }
  f32x4* mp = reinterpret_cast<f32x4*>(ad.master + i);
  __builtin_nontemporal_store(Mn, reinterpret_cast<u32x4*>(ad.m + i));
  __builtin_nontemporal_store(Vn, reinterpret_cast<u32x4*>(ad.v + i));
  __builtin_nontemporal_store(f32x4{x[0], x[1], x[2], x[3]}, mp);
  __builtin_nontemporal_store(f32x4{x[4], x[5], x[6], x[7]}, mp + 1);
}

__device__ __forceinline__ void adam_fetch8(const AdamSrc& ad, int64_t i, float (&x)[8]) {
  AdamRaw r;
  adam_load8(ad, i, r);
  adam_finish8(ad, i, r, x);
}

// First (and normally only) read of an octet by an encoder.
template <int SRC>
__device__ __forceinline__ void fetch8(const void* src, const AdamSrc& ad, int64_t i,
                                       float (&x)[8]) {
  if constexpr (SRC == kSrcAdam) adam_fetch8(ad, i, x);
  else load8<SRC>(src, i, x);
}
// The same in two phases: begin issues the loads, end leaves the values in x.
template <int SRC>
__device__ __forceinline__ void fetch8_begin(const void* src, const AdamSrc& ad, int64_t i,
                                             AdamRaw& r, float (&x)[8]) {
  if constexpr (SRC == kSrcAdam) adam_load8(ad, i, r);
  else load8<SRC>(src, i, x);
}
template <int SRC>
__device__ __forceinline__ void fetch8_end(const AdamSrc& ad, int64_t i, const AdamRaw& r,
                                           float (&x)[8]) {
  if constexpr (SRC == kSrcAdam) adam_finish8(ad, i, r, x);
}
// A second read of an octet this lane has fetched before: the stored master.
template <int SRC>
__device__ __forceinline__ void refetch8(const void* src, const AdamSrc& ad, int64_t i,
                                         float (&x)[8]) {
  if constexpr (SRC == kSrcAdam) load8<OA_F32>(ad.master, i, x);
  else load8<SRC>(src, i, x);
}

__device__ __forceinline__ float absmax8(const float (&x)[8]) {
  float a = 0.0f;
#pragma unroll
  for (int k = 0; k < 8; ++k) a = fmaxf(a, fabsf(x[k]));
  return a;
}

// max over aligned sub-groups of `width` lanes (power of two <= 64)
__device__ __forceinline__ float group_max(float a, int width) {
  for (int off = width >> 1; off > 0; off >>= 1) a = fmaxf(a, __shfl_xor(a, off, kWave));
  return a;
}

__device__ __forceinline__ float block_max(float x, float* lds) {
  x = wave_max(x);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = x;
  __syncthreads();
  float t = lds[0];
#pragma unroll
  for (int w = 1; w < kT / kWave; ++w) t = fmaxf(t, lds[w]);
  __syncthreads();
  return t;
}

// The flat kernels give every lane kOct octets, kT lanes apart, all loaded
// before the first is used.
constexpr int kOct = 4;

// How octet index o maps to an element offset: rows stored back to back need no
// row index at all; otherwise row = o / octets_per_row, in 32 bits when it fits.
enum { kFlat = 0, kDiv32 = 1, kDiv64 = 2 };

__device__ __forceinline__ int64_t octet_row(int64_t o, int64_t opr, int mode) {
  if (mode == kDiv64) return o / opr;
  return (int64_t)((uint32_t)o / (uint32_t)opr);
}
__device__ __forceinline__ int64_t octet_elem(int64_t o, int64_t opr, int64_t stride, int mode) {
  if (mode == kFlat) return o * 8;
  const int64_t row = octet_row(o, opr, mode);
  return row * stride + (o - row * opr) * 8;
}

// ---------------------------------------------------------------- quads
// Encoders of row-contiguous matrices give a lane a "quad": 32 consecutive
// elements (four octets).  Global loads stay coalesced - in trip k a wave reads
// octets 64k .. 64k+63 of its 256-octet chunk, 1 KiB per instruction - and the
// octets change hands through LDS: written where they were loaded, read back four
// in a row.  (Loading a lane's 64 contiguous bytes directly, 64 bytes apart from
// its neighbour's, measured 2.3x slower on the NF4 encoder.)  Slot
// (o & ~15) | ((o + (o >> 4)) & 15) of octet o keeps both the 16-byte writes and
// the 16-byte reads of eight consecutive lanes on distinct bank groups.
#ifndef OA_QUAD_T
#define OA_QUAD_T 64
#endif
constexpr int kQuadT = OA_QUAD_T;  // lanes of a quad-encoder workgroup
__device__ __forceinline__ int quad_slot(int o) { return (o & ~15) | ((o + (o >> 4)) & 15); }

template <int DT>
__device__ __forceinline__ void unpack16(const u32x4 w, float (&x)[8]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (DT == OA_BF16) {
      x[2 * k] = bf16lo_to_f32(w[k]);
      x[2 * k + 1] = bf16hi_to_f32(w[k]);
    } else {
      x[2 * k] = f16_bits_to_f32(w[k] & 0xFFFFu);
      x[2 * k + 1] = f16_bits_to_f32(w[k] >> 16);
    }
  }
}

// LDS a workgroup of kQuadT lanes needs: one 16-byte plane per octet for 16-bit
// sources, two for fp32.
template <int SRC>
constexpr int quad_lds_slots() { return (SRC == OA_F32 ? 2 : 1) * kQuadT * 4; }

// A workgroup can walk kQuadChunks consecutive chunks of kQuadT quads, loading
// chunk c + 1 before it encodes chunk c.  Measured on the 4096 x 14336 weight it
// does not pay: 1 / 2 / 4 / 8 chunks per one-wave workgroup give 26.0 / 27.2 /
// 29.1 / 28.6 us for NF4 - the finest grain the dispatcher can deal is the
// fastest, as for the AdamW kernels - so the default is one chunk.
#ifndef OA_QUAD_CHUNKS
#define OA_QUAD_CHUNKS 1
#endif
constexpr int kQuadChunks = OA_QUAD_CHUNKS;

template <int SRC>
struct QuadRaw {
  u32x4 v[4][SRC == OA_F32 ? 2 : 1];
};

// Issues the loads of the chunk whose first quad is q0 (a multiple of kQuadT):
// in trip k the lane takes octet 64 k + lane of its wave's 256.  `octets` =
// octets of the whole matrix; lanes beyond it get zeros.
template <int SRC>
__device__ __forceinline__ void quad_load(const void* __restrict__ src, int64_t q0,
                                          int64_t octets, QuadRaw<SRC>& r) {
  constexpr int P = SRC == OA_F32 ? 2 : 1;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t o0 = (q0 + wave * kWave) * 4;  // first octet of this wave's chunk
  const char* base = static_cast<const char*>(src) + (o0 + lane) * (16 * P);
  if ((q0 + kQuadT) * 4 <= octets) {
    // every lane of the workgroup is in range (a scalar branch): the loads carry no
    // guards, so all of them are in flight before the first is waited for
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int pl = 0; pl < P; ++pl)
        r.v[k][pl] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4*>(base + (int64_t)k * (64 * 16 * P)) + pl);
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool in = o0 + 64 * k + lane < octets;
      // the matrix's last chunk: out-of-range lanes re-read its first octet
      const u32x4* p = reinterpret_cast<const u32x4*>(
          in ? base + (int64_t)k * (64 * 16 * P) : static_cast<const char*>(src));
#pragma unroll
      for (int pl = 0; pl < P; ++pl) {
        const u32x4 v = __builtin_nontemporal_load(p + pl);
        r.v[k][pl] = in ? v : u32x4{0u, 0u, 0u, 0u};
      }
    }
  }
}

// Hands the loaded octets over: afterwards x holds the lane's own quad (first
// element 32 * (q0 + threadIdx.x)).  Two workgroup barriers: every lane of the
// workgroup calls it.
template <int SRC>
__device__ __forceinline__ void quad_exchange(const QuadRaw<SRC>& r, u32x4* lds,
                                              float (&x)[4][8]) {
  constexpr int P = SRC == OA_F32 ? 2 : 1;
  const int lane = threadIdx.x & (kWave - 1);
  u32x4* mine = lds + (threadIdx.x / kWave) * (P * 256);
  __syncthreads();  // the previous chunk has been read
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int pl = 0; pl < P; ++pl) mine[pl * 256 + quad_slot(64 * k + lane)] = r.v[k][pl];
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int slot = quad_slot(4 * lane + j);
    if (SRC == OA_F32) {
      const u32x4 a = mine[slot], b = mine[256 + slot];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        x[j][i] = __uint_as_float(a[i]);
        x[j][4 + i] = __uint_as_float(b[i]);
      }
    } else {
      unpack16<SRC>(mine[slot], x[j]);
    }
  }
}

// N trips of a row: lane t takes octets t, t + kT, ..., all loads issued before
// the first value is converted; trips N .. kRowCache-1 read as zero.
template <int SRC, int N, int R>
__device__ __forceinline__ void load_trips(const void* lane_base, float (&x)[R][8]) {
  constexpr int P = SRC == OA_F32 ? 2 : 1;
  u32x4 raw[N][P];
#pragma unroll
  for (int k = 0; k < N; ++k)
#pragma unroll
    for (int pl = 0; pl < P; ++pl)
      raw[k][pl] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4*>(static_cast<const char*>(lane_base) +
                                         (int64_t)k * kT * 16 * P) + pl);
#pragma unroll
  for (int k = 0; k < R; ++k) {
    if (k < N) {
      if constexpr (SRC == OA_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          x[k][i] = __uint_as_float(raw[k < N ? k : 0][0][i]);
          x[k][4 + i] = __uint_as_float(raw[k < N ? k : 0][P - 1][i]);
        }
      } else {
        unpack16<SRC>(raw[k < N ? k : 0][0], x[k]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) x[k][i] = 0.0f;
    }
  }
}

// ------------------------------------------------------------------- int8

__device__ __forceinline__ int32_t q_int8(float x, float inv) {
  float t = __builtin_rintf(x * inv);
  t = fminf(fmaxf(t, -128.0f), 127.0f);
  return (int32_t)t;
}
// Four codes of one packed dword: clamp(rint(x * inv), -128, 127) + 128 is an
// integer in [0, 255], exact in fp32; v_cvt_pk_u8_f32 converts it and places the
// byte, and flipping the top bit of every byte afterwards takes the 128 off again
// (two's complement).  A NaN clamps to -128, as in q_int8().
__device__ __forceinline__ uint32_t q_int8_word(float a, float b, float c, float d, float inv) {
  uint32_t w = 0;
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      __builtin_amdgcn_fmed3f(__builtin_rintf(a * inv), -128.0f, 127.0f) + 128.0f, 0, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      __builtin_amdgcn_fmed3f(__builtin_rintf(b * inv), -128.0f, 127.0f) + 128.0f, 1, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      __builtin_amdgcn_fmed3f(__builtin_rintf(c * inv), -128.0f, 127.0f) + 128.0f, 2, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      __builtin_amdgcn_fmed3f(__builtin_rintf(d * inv), -128.0f, 127.0f) + 128.0f, 3, w);
  return w ^ 0x80808080u;
}

constexpr int kRowCache = 8;  // octets a lane keeps in registers between the two passes
#ifndef OA_I8_BATCH
#define OA_I8_BATCH 4
#endif
constexpr int kI8Batch = OA_I8_BATCH;  // fused AdamW source: octets whose loads are issued together

// One block per row.  Pass 1 loads the row (all of a lane's octets in flight at
// once, kept in registers when the row has at most kT * kRowCache octets) and
// folds |x| into the row maximum; pass 2 encodes from the registers.  Longer rows
// are re-read in pass 2 (L2-resident: a row is tens of KiB).
template <int SRC>
__global__ void __launch_bounds__(kT)
quant_int8_kernel(const void* __restrict__ src, int64_t stride, int64_t cols,
                  int8_t* __restrict__ q, void* __restrict__ scales, int sdt, int vec,
                  const AdamSrc ad) {
  __shared__ float lds[kT / kWave];
  const int64_t row = blockIdx.x;
  const int64_t base = row * stride;
  const int64_t octets = vec ? cols >> 3 : 0;
  const bool cached = octets <= (int64_t)kT * kRowCache;
  float xc[kRowCache][8];
  float a = 0.0f;
  if (cached) {
    bool loaded = false;
    if constexpr (SRC != kSrcAdam) {
      // A row of whole trips (octets % kT == 0): one straight-line run of
      // unguarded loads per trip count, all in flight before the first convert.
      // (A guarded load - or one inside any branch that also converts it - is
      // waited for before the next is issued: one load in flight per wave.)
      if (octets % kT == 0) {
        loaded = true;
        const void* at = static_cast<const char*>(src) +
                         (base + (int64_t)threadIdx.x * 8) * (SRC == OA_F32 ? 4 : 2);
        switch ((int)(octets / kT)) {
          case 1: load_trips<SRC, 1>(at, xc); break;
          case 2: load_trips<SRC, 2>(at, xc); break;
          case 3: load_trips<SRC, 3>(at, xc); break;
          case 4: load_trips<SRC, 4>(at, xc); break;
          case 5: load_trips<SRC, 5>(at, xc); break;
          case 6: load_trips<SRC, 6>(at, xc); break;
          case 7: load_trips<SRC, 7>(at, xc); break;
          case 8: load_trips<SRC, 8>(at, xc); break;
          default: loaded = false; break;
        }
      }
    }
    if (!loaded) {
      // loads of kI8Batch octets at a time before their stores (fused source)
#pragma unroll
      for (int kb = 0; kb < kRowCache; kb += kI8Batch) {
        AdamRaw raw[kI8Batch];
#pragma unroll
        for (int k = kb; k < kb + kI8Batch; ++k) {
          const int64_t o = threadIdx.x + (int64_t)k * kT;
          if (o < octets) {
            fetch8_begin<SRC>(src, ad, base + o * 8, raw[k - kb], xc[k]);
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) xc[k][j] = 0.0f;
          }
        }
#pragma unroll
        for (int k = kb; k < kb + kI8Batch; ++k) {
          const int64_t o = threadIdx.x + (int64_t)k * kT;
          if (o < octets) fetch8_end<SRC>(ad, base + o * 8, raw[k - kb], xc[k]);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < kRowCache; ++k) a = fmaxf(a, absmax8(xc[k]));
  } else {
    for (int64_t o = threadIdx.x; o < octets; o += kT) {
      float x[8];
      fetch8<SRC>(src, ad, base + o * 8, x);
      a = fmaxf(a, absmax8(x));
    }
  }
  for (int64_t c = octets * 8 + threadIdx.x; c < cols; c += kT)
    a = fmaxf(a, fabsf(load1<SRC>(src, base + c)));
  const float absmax = block_max(a, lds);
  const float scale = absmax / 127.0f;
  const float inv = 1.0f / fmaxf(scale, kEps);
  if (threadIdx.x == 0) store_scale(scales, sdt, row, scale);

  int8_t* qr = q + row * cols;
  auto encode = [&](const float (&x)[8], int64_t o) {
    const uint32_t w0 = q_int8_word(x[0], x[1], x[2], x[3], inv);
    const uint32_t w1 = q_int8_word(x[4], x[5], x[6], x[7], inv);
    __builtin_nontemporal_store(u32x2{w0, w1}, reinterpret_cast<u32x2*>(qr + o * 8));
  };
  if (cached) {
#pragma unroll
    for (int k = 0; k < kRowCache; ++k) {
      const int64_t o = threadIdx.x + (int64_t)k * kT;
      if (o < octets) encode(xc[k], o);
    }
  } else {
    for (int64_t o = threadIdx.x; o < octets; o += kT) {
      float x[8];
      refetch8<SRC>(src, ad, base + o * 8, x);
      encode(x, o);
    }
  }
  for (int64_t c = octets * 8 + threadIdx.x; c < cols; c += kT)
    qr[c] = (int8_t)q_int8(load1<SRC>(src, base + c), inv);
}

template <int OUT>
__global__ void __launch_bounds__(kT)
dequant_int8_kernel(const int8_t* __restrict__ q, const void* __restrict__ scales, int sdt,
                    int64_t rows, int64_t cols, void* __restrict__ out, int64_t ostride,
                    int vec, int mode) {
  if (vec) {
    const int64_t opr = cols >> 3, total = rows * opr;
    const int64_t o0 = (int64_t)blockIdx.x * (kT * kOct) + threadIdx.x;
    u32x2 w[kOct];
    float s[kOct];
    int64_t at[kOct];
#pragma unroll
    for (int k = 0; k < kOct; ++k) {
      const int64_t o = o0 + (int64_t)k * kT;
      w[k] = u32x2{0u, 0u};
      s[k] = 0.0f;
      at[k] = 0;
      if (o < total) {
        const int64_t row = octet_row(o, opr, mode), c8 = o - row * opr;
        w[k] = *reinterpret_cast<const u32x2*>(q + row * cols + c8 * 8);
        s[k] = load_scale(scales, sdt, row);
        at[k] = row * ostride + c8 * 8;
      }
    }
#pragma unroll
    for (int k = 0; k < kOct; ++k) {
      if (o0 + (int64_t)k * kT >= total) continue;
      float y[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int32_t v = (int32_t)(int8_t)((w[k][j >> 2] >> (8 * (j & 3))) & 0xFFu);
        y[j] = (float)v * s[k];
      }
      store8<OUT, false>(out, at[k], y);
    }
  } else {
    const int64_t i = (int64_t)blockIdx.x * kT + threadIdx.x;
    if (i >= rows * cols) return;
    const int64_t row = i / cols, c = i - row * cols;
    store1<OUT>(out, row * ostride + c, (float)q[i] * load_scale(scales, sdt, row));
  }
}

// The decoder's fast path with everything that made a load wait taken out: a tile
// that lies wholly inside the matrix is a scalar condition (the last tile clamps
// its octet index instead of guarding the load), and the scale dtype is a
// template argument (a run-time switch puts each scale load and its convert into
// a branch of its own).  All 2 x kOct loads of a lane are issued before the first
// convert.  A lane owns octets, so that each store instruction of a wave covers
// one contiguous KiB (16 codes per lane would load in one piece but store two
// interleaved halves: measured 34 us against 31.6).
template <int OUT, int SDT>
__global__ void __launch_bounds__(kT)
dequant_int8_tile_kernel(const int8_t* __restrict__ q, const void* __restrict__ scales,
                         int64_t rows, int64_t cols, void* __restrict__ out, int64_t ostride,
                         int mode) {
  const int64_t opr = cols >> 3, total = rows * opr;
  const int64_t tile0 = (int64_t)blockIdx.x * (kT * kOct);
  const int64_t o0 = tile0 + threadIdx.x;
  u32x2 w[kOct];
  uint32_t sraw[kOct];
  int64_t at[kOct];
  const bool full = tile0 + kT * kOct <= total;
#pragma unroll
  for (int k = 0; k < kOct; ++k) {
    int64_t o = o0 + (int64_t)k * kT;
    if (!full && o >= total) o = total - 1;  // re-read the last octet; its store is skipped
    const int64_t row = octet_row(o, opr, mode);
    w[k] = *reinterpret_cast<const u32x2*>(q + o * 8);
    if (SDT == OA_F32) sraw[k] = static_cast<const uint32_t*>(scales)[row];
    else sraw[k] = static_cast<const uint16_t*>(scales)[row];
    at[k] = row * ostride + (o - row * opr) * 8;
  }
#pragma unroll
  for (int k = 0; k < kOct; ++k) {
    if (!full && o0 + (int64_t)k * kT >= total) continue;
    const float sc = SDT == OA_F32 ? __uint_as_float(sraw[k])
                     : SDT == OA_BF16 ? bf16_bits_to_f32(sraw[k]) : f16_bits_to_f32(sraw[k]);
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int32_t v = (int32_t)(int8_t)((w[k][j >> 2] >> (8 * (j & 3))) & 0xFFu);
      y[j] = (float)v * sc;
    }
    store8<OUT, false>(out, at[k], y);
  }
}

// ------------------------------------------------------------------- int4

// Eight codes of one packed word.  clamp(rint(x * inv), -8, 7) + 8 is formed in
// fp32 (every intermediate is a small integer, hence exact), two codes are joined
// into their byte lo + 16 hi with one multiply-add, and the byte is converted and
// placed by one v_cvt_pk_u8_f32: 4.5 VALU operations per code instead of 7.
__device__ __forceinline__ uint32_t q_int4_word(const float (&x)[8], float inv) {
  uint32_t word = 0;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float lo = __builtin_amdgcn_fmed3f(__builtin_rintf(x[2 * k] * inv), -8.0f, 7.0f);
    const float hi = __builtin_amdgcn_fmed3f(__builtin_rintf(x[2 * k + 1] * inv), -8.0f, 7.0f);
    const float byte = __builtin_fmaf(hi, 16.0f, lo) + 136.0f;  // (hi + 8) * 16 + (lo + 8)
    word = __builtin_amdgcn_cvt_pk_u8_f32(byte, k, word);
  }
  return word;
}

#ifndef OA_I4_ROWS_Q
#define OA_I4_ROWS_Q 64
#endif
constexpr int kI4RowsQ = OA_I4_ROWS_Q;   // rows of one LDS tile, encoder
constexpr int kI4PitchQ = kI4RowsQ + 4;  // words per LDS row of it: 16-byte aligned rows, and the
                               // writes of a wave (16 word columns x 4 rows) hit 64 banks
constexpr int kI4RowsD = 128;  // rows of one LDS tile, decoder
constexpr int kI4Chunk = 4;    // decoder: packed words a lane fetches per trip
// Consecutive workgroups walk along the row (group index fastest): the tiles in
// flight then touch neighbouring 256-byte segments of the same rows.  Against
// row-tile-fastest: decoder 26.7 -> 24.6 us, fused AdamW encoder 226 -> 209 us.
#ifndef OA_I4_GROUP_FASTEST
#define OA_I4_GROUP_FASTEST 1
#endif
inline bool i4_grid_ok(int64_t row_tiles, int64_t groups) {  // y and z extents stop at 65535
  return OA_I4_GROUP_FASTEST ? row_tiles <= 65535 && groups <= 0x7FFFFFFFll : groups <= 65535;
}
inline dim3 i4_grid(unsigned row_tiles, unsigned groups) {
  return OA_I4_GROUP_FASTEST ? dim3(groups, row_tiles) : dim3(row_tiles, groups);
}

// Block tile: 64 rows (encoder) or 128 rows (decoder) x one group.  WPR = group/8
// lanes share a (row, group): they fold the group maximum with shuffles and emit
// one packed word each into LDS; the tile is then written with lanes running
// along the row index, which is the contiguous direction of the transposed
// (cols/8, rows) storage.  (Issuing the encoder's four row passes together, or a
// 128-row encoder tile, measured 10-15 % slower than this plain loop.)
// WPR = words per (row, group) when it is known at compile time (the usual
// group sizes 128, 64 and 32): every index division below folds into shifts and
// the row passes unroll; 0 = take it from `group` at run time.
template <int SRC, int WPR>
__global__ void __launch_bounds__(kT)
quant_int4_kernel(const void* __restrict__ src, int64_t stride, int64_t rows, int group,
                  int32_t* __restrict__ qweight, void* __restrict__ scales, int sdt,
                  const AdamSrc ad) {
  extern __shared__ uint32_t i4_lds[];
  const int wpr = WPR ? WPR : (group >> 3);
  uint32_t* words = i4_lds;                                  // [wpr][kI4PitchQ]
  float* scale_s = reinterpret_cast<float*>(words + wpr * kI4PitchQ);
#if OA_I4_GROUP_FASTEST
  const int64_t r0 = (int64_t)blockIdx.y * kI4RowsQ;
  const int64_t gi = blockIdx.x;
#else
  const int64_t r0 = (int64_t)blockIdx.x * kI4RowsQ;
  const int64_t gi = blockIdx.y;
#endif
  const int rows_per_pass = kT / wpr;
  const int k = threadIdx.x % wpr;
  const int rsub = threadIdx.x / wpr;
  // A tile that lies wholly inside the matrix (a scalar condition) loads without
  // per-lane guards; a guarded load sits in a divergent branch and is waited for
  // before the next one is issued.
  const bool full = r0 + kI4RowsQ <= rows;
  auto encode_row = [&](const float (&x)[8], int rl) {
    const float absmax = group_max(absmax8(x), wpr);
    const float scale = absmax / 8.0f;
    const float inv = 1.0f / fmaxf(scale, kEps);
    if (rl < kI4RowsQ) {
      words[k * kI4PitchQ + rl] = q_int4_word(x, inv);
      if (k == 0) scale_s[rl] = scale;
    }
  };
  if constexpr (WPR != 0 && SRC != kSrcAdam) {
    // plain sources: the loads of every row pass are issued before the first is used
    constexpr int kPasses = kI4RowsQ / (kT / WPR);
    float x[kPasses][8];
    if (full) {
#pragma unroll
      for (int p = 0; p < kPasses; ++p)
        load8<SRC>(src, (r0 + p * (kT / WPR) + rsub) * stride + gi * group + k * 8, x[p]);
    } else {
#pragma unroll
      for (int p = 0; p < kPasses; ++p) {
        const int64_t row = r0 + p * (kT / WPR) + rsub;
#pragma unroll
        for (int i = 0; i < 8; ++i) x[p][i] = 0.0f;
        if (row < rows) load8<SRC>(src, row * stride + gi * group + k * 8, x[p]);
      }
    }
#pragma unroll
    for (int p = 0; p < kPasses; ++p) encode_row(x[p], p * (kT / WPR) + rsub);
  } else if (WPR != 0 && full) {
    // fused AdamW source, whole tile: the loads of row pass p + 1 are issued before
    // pass p is updated, stored and encoded (two passes of operands in registers)
    constexpr int kRpp = kT / (WPR ? WPR : 1);
    constexpr int kPasses = kI4RowsQ / kRpp;
    AdamRaw raw[2];
    float x[8];
    fetch8_begin<SRC>(src, ad, (r0 + rsub) * stride + gi * group + k * 8, raw[0], x);
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int64_t at = (r0 + p * kRpp + rsub) * stride + gi * group + k * 8;
      if (p + 1 < kPasses) {
        float unused[8];
        fetch8_begin<SRC>(src, ad, at + (int64_t)kRpp * stride, raw[(p + 1) & 1], unused);
      }
      fetch8_end<SRC>(ad, at, raw[p & 1], x);
      encode_row(x, p * kRpp + rsub);
    }
  } else {
    for (int pr = 0; pr < kI4RowsQ; pr += rows_per_pass) {
      const int rl = pr + rsub;
      const int64_t row = r0 + rl;
      float x[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      if (rl < kI4RowsQ && row < rows) fetch8<SRC>(src, ad, row * stride + gi * group + k * 8, x);
      encode_row(x, rl);
    }
  }
  __syncthreads();
  if (full && (rows & 3) == 0 && (reinterpret_cast<uintptr_t>(qweight) & 15) == 0) {
    // 16 bytes of the transposed payload per lane: four consecutive rows of one word column
    // (a payload that is only 4-byte aligned takes the word-wise stores below)
    for (int idx = threadIdx.x; idx < wpr * (kI4RowsQ / 4); idx += kT) {
      const int kk = idx / (kI4RowsQ / 4), r4 = idx % (kI4RowsQ / 4);
      const u32x4 w = *reinterpret_cast<const u32x4*>(words + kk * kI4PitchQ + 4 * r4);
      __builtin_nontemporal_store(
          w, reinterpret_cast<u32x4*>(qweight + (gi * wpr + kk) * rows + r0 + 4 * r4));
    }
  } else {
    for (int idx = threadIdx.x; idx < wpr * kI4RowsQ; idx += kT) {
      const int kk = idx / kI4RowsQ, rl = idx % kI4RowsQ;
      if (r0 + rl < rows)
        qweight[(gi * wpr + kk) * rows + r0 + rl] = (int32_t)words[kk * kI4PitchQ + rl];
    }
  }
  if (threadIdx.x < kI4RowsQ && r0 + threadIdx.x < rows)
    store_scale(scales, sdt, gi * rows + r0 + threadIdx.x, scale_s[threadIdx.x]);
}

template <int OUT, int WPR>
__global__ void __launch_bounds__(kT)
dequant_int4_kernel(const int32_t* __restrict__ qweight, const void* __restrict__ scales,
                    int sdt, int64_t rows, int group, void* __restrict__ out,
                    int64_t ostride) {
  extern __shared__ uint32_t i4_lds[];
  const int wpr = WPR ? WPR : (group >> 3);
  uint32_t* words = i4_lds;
  float* scale_s = reinterpret_cast<float*>(words + wpr * (kI4RowsD + 1));
#if OA_I4_GROUP_FASTEST
  const int64_t r0 = (int64_t)blockIdx.y * kI4RowsD;
  const int64_t gi = blockIdx.x;
#else
  const int64_t r0 = (int64_t)blockIdx.x * kI4RowsD;
  const int64_t gi = blockIdx.y;
#endif
  // the tile's words: wpr * kI4RowsD of them, kI4Chunk per lane per trip
  for (int idx0 = threadIdx.x; idx0 < wpr * kI4RowsD; idx0 += kI4Chunk * kT) {
    uint32_t w[kI4Chunk];
#pragma unroll
    for (int c = 0; c < kI4Chunk; ++c) {
      const int idx = idx0 + c * kT;
      const int kk = idx / kI4RowsD, rl = idx % kI4RowsD;
      w[c] = (idx < wpr * kI4RowsD && r0 + rl < rows)
                 ? (uint32_t)qweight[(gi * wpr + kk) * rows + r0 + rl] : 0u;
    }
#pragma unroll
    for (int c = 0; c < kI4Chunk; ++c) {
      const int idx = idx0 + c * kT;
      if (idx < wpr * kI4RowsD) words[(idx / kI4RowsD) * (kI4RowsD + 1) + idx % kI4RowsD] = w[c];
    }
  }
  if (threadIdx.x < kI4RowsD)
    scale_s[threadIdx.x] = (r0 + threadIdx.x < rows)
                               ? load_scale(scales, sdt, gi * rows + r0 + threadIdx.x)
                               : 0.0f;
  __syncthreads();
  const int rows_per_pass = kT / wpr;
  const int k = threadIdx.x % wpr;
  for (int pr = 0; pr < kI4RowsD; pr += rows_per_pass) {
    const int rl = pr + threadIdx.x / wpr;
    const int64_t row = r0 + rl;
    if (rl >= kI4RowsD || row >= rows) continue;
    const uint32_t w = words[k * (kI4RowsD + 1) + rl];
    const float s = scale_s[rl];
    float y[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = (float)((int32_t)((w >> (4 * i)) & 0xFu) - 8) * s;
    store8<OUT>(out, row * ostride + gi * group + k * 8, y);
  }
}

// One lane per (row, group): any group size, any alignment.
template <int SRC>
__global__ void __launch_bounds__(kT)
quant_int4_generic(const void* __restrict__ src, int64_t stride, int64_t rows, int64_t cols,
                   int64_t group, int32_t* __restrict__ qweight, void* __restrict__ scales,
                   int sdt) {
  const int64_t ng = cols / group;
  const int64_t t = (int64_t)blockIdx.x * kT + threadIdx.x;
  if (t >= rows * ng) return;
  const int64_t gi = t / rows, row = t - gi * rows;  // consecutive lanes -> consecutive rows
  const int64_t base = row * stride + gi * group;
  float a = 0.0f;
  for (int64_t c = 0; c < group; ++c) a = fmaxf(a, fabsf(load1<SRC>(src, base + c)));
  const float scale = a / 8.0f;
  const float inv = 1.0f / fmaxf(scale, kEps);
  store_scale(scales, sdt, gi * rows + row, scale);
  for (int64_t k = 0; k < group / 8; ++k) {
    float x[8];
    for (int i = 0; i < 8; ++i) x[i] = load1<SRC>(src, base + k * 8 + i);
    qweight[(gi * (group / 8) + k) * rows + row] = (int32_t)q_int4_word(x, inv);
  }
}

template <int OUT>
__global__ void __launch_bounds__(kT)
dequant_int4_generic(const int32_t* __restrict__ qweight, const void* __restrict__ scales,
                     int sdt, int64_t rows, int64_t cols, int64_t group,
                     void* __restrict__ out, int64_t ostride) {
  const int64_t t = (int64_t)blockIdx.x * kT + threadIdx.x;
  if (t >= rows * (cols / 8)) return;
  const int64_t kw = t / rows, row = t - kw * rows;
  const uint32_t w = (uint32_t)qweight[kw * rows + row];
  const float s = load_scale(scales, sdt, ((kw * 8) / group) * rows + row);
  for (int i = 0; i < 8; ++i)
    store1<OUT>(out, row * ostride + kw * 8 + i,
                (float)((int32_t)((w >> (4 * i)) & 0xFu) - 8) * s);
}

// -------------------------------------------------------------------- NF4

__constant__ float kNf4Lut[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f,
    0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,
    0.7229568362236023f, 1.0f};

// Decision thresholds of the nearest-codebook search: the code of a normalised
// value n is the number of thresholds t_i with n >= t_i.  t_i is the smallest
// fp32 for which fl(|n - L[i+1]|) < fl(|n - L[i]|), found by bisection over
// the fp32 bit patterns, so the count equals the first-minimum argmin over the
// fp32 distances for every input (the neighbours are the only candidates: the
// codebook spacing is >= 0.079, rounding error of a distance <= 6e-8).
constexpr uint32_t kNf4T[15] = {
    0xbf591cd8u, 0xbf1c5270u, 0xbeeb847fu, 0xbeadea76u, 0xbe703cecu,
    0xbe0d38bbu, 0xbd3a7870u, 0x3d22fb00u, 0x3df64863u, 0x3e5067e1u,
    0x3e9582d5u, 0x3ec753fau, 0x3f006d04u, 0x3f248db0u, 0x3f5c89dau};

// Counting thresholds without walking them.  With m = 16 * n:
// bucket(m) = trunc(m + 16) clamped to [0, 31] is monotone in n, and the
// thresholds are further apart (>= 0.0805) than a bucket is wide (0.0625), so
// every bucket holds at most one.  For n in bucket k the thresholds of lower
// buckets are below n and those of higher buckets above; the bucket's own
// threshold, if any, is compared directly:
//     code(n) = below[k] + (m >= 16 * own[k]),      own = +inf if none
// Scaling by 16 is exact in fp32, so x * (16 * inv) == 16 * fl(x * inv) and
// m >= 16 * t  <=>  n >= t: the kernel never forms n itself.  The table is built
// at compile time with the same fp32 addition the kernel uses, so bucket(16 t_i)
// here and bucket(m) on the GPU agree bit for bit.  The 32 entries of 8 bytes
// cover the 64 LDS banks exactly once: the lookup has no bank conflicts.
constexpr int nf4_bucket(float m) {  // m = 16 n
  const float f = m + 16.0f;
  if (!(f > 0.0f)) return 0;
  if (f >= 31.0f) return 31;
  return (int)f;
}
struct Nf4Buckets {
  uint32_t own16[32];  // fp32 bits of 16 * (threshold inside the bucket), +inf if none
  uint32_t below[32];  // thresholds in lower buckets
};
constexpr Nf4Buckets make_nf4_buckets() {
  Nf4Buckets t{};
  for (int k = 0; k < 32; ++k) {
    t.own16[k] = 0x7F800000u;
    t.below[k] = 0;
  }
  for (int i = 0; i < 15; ++i) {
    const float t16 = __builtin_bit_cast(float, kNf4T[i]) * 16.0f;
    const int b = nf4_bucket(t16);
    t.own16[b] = __builtin_bit_cast(uint32_t, t16);
    for (int k = b + 1; k < 32; ++k) t.below[k] += 1;
  }
  return t;
}
constexpr bool nf4_buckets_distinct() {
  int last = -1;
  for (int i = 0; i < 15; ++i) {
    const int b = nf4_bucket(__builtin_bit_cast(float, kNf4T[i]) * 16.0f);
    if (b <= last) return false;
    last = b;
  }
  return true;
}
static_assert(nf4_buckets_distinct(), "two NF4 thresholds share a bucket");
__device__ const Nf4Buckets kNf4Buckets = make_nf4_buckets();

__device__ __forceinline__ void nf4_buckets_to_lds(u32x2* lut) {
  if (threadIdx.x < 32)
    lut[threadIdx.x] = u32x2{kNf4Buckets.own16[threadIdx.x], kNf4Buckets.below[threadIdx.x]};
}

// m = 16 * (x / absmax); |m| <= 16 (1 + 2^-23) for finite input, so m + 16 lies in
// (-1, 33) and the conversion to int is exact truncation.
__device__ __forceinline__ uint32_t nf4_code16(float m, const u32x2* lut) {
  int k = (int)(m + 16.0f);
  k = k > 31 ? 31 : k;
  k = k < 0 ? 0 : k;  // NaN
  const u32x2 e = lut[k];
  return e[1] + (uint32_t)(m >= __uint_as_float(e[0]));
}

// The same count by a four-level decision tree (no table): used by the generic
// kernel, which has no block-wide prologue.
#define NF4_T(i) __uint_as_float(kNf4T[i])
__device__ __forceinline__ uint32_t nf4_code_tree(float n) {
  const bool b3 = n >= NF4_T(7);
  const bool b2 = n >= (b3 ? NF4_T(11) : NF4_T(3));
  const bool b1 = n >= (b3 ? (b2 ? NF4_T(13) : NF4_T(9)) : (b2 ? NF4_T(5) : NF4_T(1)));
  const float t0 = b3 ? (b2 ? (b1 ? NF4_T(14) : NF4_T(12)) : (b1 ? NF4_T(10) : NF4_T(8)))
                      : (b2 ? (b1 ? NF4_T(6) : NF4_T(4)) : (b1 ? NF4_T(2) : NF4_T(0)));
  const bool b0 = n >= t0;
  return ((uint32_t)b3 << 3) | ((uint32_t)b2 << 2) | ((uint32_t)b1 << 1) | (uint32_t)b0;
}
#undef NF4_T

// inv16 = 16 / absmax (the exact 16-fold of the reference's 1 / absmax)
__device__ __forceinline__ uint32_t nf4_pack8(const float (&x)[8], float inv16, const u32x2* lut) {
  uint32_t w = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t hi = nf4_code16(x[2 * j] * inv16, lut);
    const uint32_t lo = nf4_code16(x[2 * j + 1] * inv16, lut);
    w |= ((hi << 4) | lo) << (8 * j);
  }
  return w;
}

// The same count with one fp32 add in place of add, convert and two clamps: the
// low mantissa bits of m + (2^23 + 16) are round-half-even(m + 16), an integer in
// [0, 32] for every finite input (|m| <= 16 (1 + 2^-23)).  Buckets are again
// monotone in n and one unit of m wide, so each holds at most one threshold; 64
// entries, because a NaN leaves arbitrary low bits (entries above 32 give code 0,
// as bucket 0 does for the canonical NaN: the reference's argmin over NaN
// distances is 0 as well).
constexpr float kNf4Magic = 8388624.0f;  // 2^23 + 16
constexpr int nf4_rbucket(float m) {
  return (int)(__builtin_bit_cast(uint32_t, m + kNf4Magic) & 63u);
}
struct Nf4RBuckets {
  uint32_t own16[64];
  uint32_t below[64];
};
constexpr Nf4RBuckets make_nf4_rbuckets() {
  Nf4RBuckets t{};
  for (int k = 0; k < 64; ++k) {
    t.own16[k] = 0x7F800000u;
    t.below[k] = 0;
  }
  for (int i = 0; i < 15; ++i) {
    const float t16 = __builtin_bit_cast(float, kNf4T[i]) * 16.0f;
    const int b = nf4_rbucket(t16);
    t.own16[b] = __builtin_bit_cast(uint32_t, t16);
    for (int k = b + 1; k <= 32; ++k) t.below[k] += 1;
  }
  return t;
}
constexpr bool nf4_rbuckets_distinct() {
  int last = -1;
  for (int i = 0; i < 15; ++i) {
    const int b = nf4_rbucket(__builtin_bit_cast(float, kNf4T[i]) * 16.0f);
    if (b <= last || b > 32) return false;
    last = b;
  }
  return nf4_rbucket(-16.000002f) == 0 && nf4_rbucket(16.000002f) == 32;
}
static_assert(nf4_rbuckets_distinct(), "two NF4 thresholds share a rounded bucket");
__device__ const Nf4RBuckets kNf4RBuckets = make_nf4_rbuckets();

__device__ __forceinline__ uint32_t nf4_code16r(float m, const u32x2* lut) {
  const u32x2 e = lut[__float_as_uint(m + kNf4Magic) & 63u];
  return e[1] + (uint32_t)(m >= __uint_as_float(e[0]));
}

__device__ __forceinline__ uint32_t nf4_pack8r(const float (&x)[8], float inv16, const u32x2* lut) {
  uint32_t w = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t hi = nf4_code16r(x[2 * j] * inv16, lut);
    const uint32_t lo = nf4_code16r(x[2 * j + 1] * inv16, lut);
    w |= ((hi << 4) | lo) << (8 * j);
  }
  return w;
}

// Row-contiguous matrices whose blocks are whole "quads": a lane owns 32
// consecutive elements (four octets), LPB lanes share a block (block = 32 LPB).
// Against one octet per lane and trip: the block maximum needs log2(LPB) shuffle
// steps per 32 elements instead of three per octet, the correctly rounded
// reciprocal is taken once per 32 elements, and the codes leave as one 16-byte
// store per lane (1 KiB per wave instruction; the maxima as one run of floats).
// The quad arrives through quad_load() / quad_exchange().
template <int SRC, int LPB>
__global__ void __launch_bounds__(kQuadT)
quant_nf4_quad_kernel(const void* __restrict__ src, int64_t quads, int lpb_arg, int lpb_shift_arg,
                      u32x4* __restrict__ packed, float* __restrict__ absmax_out) {
  const int lpb = LPB ? LPB : lpb_arg;
  const int lpb_shift = LPB ? __builtin_ctz((unsigned)(LPB ? LPB : 1)) : lpb_shift_arg;
  __shared__ u32x2 lut[64];
  __shared__ u32x4 stage[quad_lds_slots<SRC>()];
  if (threadIdx.x < 64)
    lut[threadIdx.x] = u32x2{kNf4RBuckets.own16[threadIdx.x], kNf4RBuckets.below[threadIdx.x]};
  const int64_t qbase = (int64_t)blockIdx.x * (kQuadT * kQuadChunks);
  QuadRaw<SRC> cur, nxt;
  quad_load<SRC>(src, qbase, quads * 4, cur);
#pragma unroll
  for (int c = 0; c < kQuadChunks; ++c) {
    const int64_t q0 = qbase + (int64_t)c * kQuadT;
    if (q0 >= quads) break;
    const bool more = c + 1 < kQuadChunks && q0 + kQuadT < quads;
    if (more) quad_load<SRC>(src, q0 + kQuadT, quads * 4, nxt);
    float x[4][8];
    quad_exchange<SRC>(cur, stage, x);  // its barriers also cover the table
    float a = fmaxf(fmaxf(absmax8(x[0]), absmax8(x[1])), fmaxf(absmax8(x[2]), absmax8(x[3])));
    a = group_max(a, lpb);
    const float inv16 = (1.0f / fmaxf(a, kEps)) * 16.0f;
    u32x4 w;
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = nf4_pack8r(x[j], inv16, lut);
    const int64_t q = q0 + threadIdx.x;
    if (q < quads) {
      __builtin_nontemporal_store(w, packed + q);
      if ((threadIdx.x & (lpb - 1)) == 0) absmax_out[q >> lpb_shift] = a;
    }
    cur = nxt;
  }
}

// Flat over octets; lpg = block/8 lanes share a block (power of two <= 64).
// LPG != 0: that many lanes per block, known at compile time (8 = the usual
// 64-element block): the shuffle ladder of the block maximum unrolls.
template <int SRC, int LPG>
__global__ void __launch_bounds__(kT)
quant_nf4_kernel(const void* __restrict__ src, int64_t stride, int64_t rows, int64_t cols,
                 int lpg_arg, int lpg_shift_arg, uint32_t* __restrict__ packed,
                 float* __restrict__ absmax_out, int mode, const AdamSrc ad) {
  const int lpg = LPG ? LPG : lpg_arg;
  const int lpg_shift = LPG ? __builtin_ctz((unsigned)(LPG ? LPG : 1)) : lpg_shift_arg;
  // The fused AdamW source moves 18 bytes per element: one octet per lane and the
  // XCD-aware tile order of the step kernels suit it better than four in flight.
  constexpr int kOct = SRC == kSrcAdam ? 1 : oa::kOct;
  __shared__ u32x2 lut[32];
  nf4_buckets_to_lds(lut);
  const int64_t opr = cols >> 3, total = rows * opr;
  const int64_t tile = SRC == kSrcAdam ? xcd_tile<kCodecXcdChunk>(blockIdx.x) : blockIdx.x;
  const int64_t o0 = tile * (kT * kOct) + threadIdx.x;
  float x[kOct][8];
#pragma unroll
  for (int k = 0; k < kOct; ++k) {
    const int64_t o = o0 + (int64_t)k * kT;
    if (o < total) {
      fetch8<SRC>(src, ad, octet_elem(o, opr, stride, mode), x[k]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) x[k][j] = 0.0f;
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kOct; ++k) {
    const int64_t o = o0 + (int64_t)k * kT;
    const float absmax = group_max(absmax8(x[k]), lpg);
    const float inv16 = (1.0f / fmaxf(absmax, kEps)) * 16.0f;
    if (o < total) {
      __builtin_nontemporal_store(nf4_pack8(x[k], inv16, lut), packed + o);
      if ((threadIdx.x & (lpg - 1)) == 0) absmax_out[o >> lpg_shift] = absmax;
    }
  }
}

template <int OUT>
__global__ void __launch_bounds__(kT)
dequant_nf4_kernel(const uint32_t* __restrict__ packed, const float* __restrict__ absmax,
                   int64_t rows, int64_t cols, int lpg_shift, void* __restrict__ out,
                   int64_t ostride, int mode) {
  __shared__ float lut[16];
  if (threadIdx.x < 16) lut[threadIdx.x] = kNf4Lut[threadIdx.x];
  const int64_t opr = cols >> 3, total = rows * opr;
  const int64_t o0 = (int64_t)blockIdx.x * (kT * kOct) + threadIdx.x;
  uint32_t w[kOct];
  float s[kOct];
#pragma unroll
  for (int k = 0; k < kOct; ++k) {
    const int64_t o = o0 + (int64_t)k * kT;
    w[k] = o < total ? packed[o] : 0u;
    s[k] = o < total ? absmax[o >> lpg_shift] : 0.0f;
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kOct; ++k) {
    const int64_t o = o0 + (int64_t)k * kT;
    if (o >= total) continue;
    float y[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t b = (w[k] >> (8 * j)) & 0xFFu;
      y[2 * j] = lut[b >> 4] * s[k];
      y[2 * j + 1] = lut[b & 0xFu] * s[k];
    }
    store8<OUT>(out, octet_elem(o, opr, ostride, mode), y);
  }
}

template <int SRC>
__global__ void __launch_bounds__(kT)
quant_nf4_generic(const void* __restrict__ src, int64_t stride, int64_t rows, int64_t cols,
                  int64_t block, uint8_t* __restrict__ packed, float* __restrict__ absmax_out) {
  const int64_t ng = cols / block;
  const int64_t t = (int64_t)blockIdx.x * kT + threadIdx.x;
  if (t >= rows * ng) return;
  const int64_t row = t / ng, gi = t - row * ng;
  const int64_t base = row * stride + gi * block;
  float a = 0.0f;
  for (int64_t c = 0; c < block; ++c) a = fmaxf(a, fabsf(load1<SRC>(src, base + c)));
  const float inv = 1.0f / fmaxf(a, kEps);
  absmax_out[t] = a;
  for (int64_t c = 0; c < block; c += 2) {
    const uint32_t hi = nf4_code_tree(load1<SRC>(src, base + c) * inv);
    const uint32_t lo = nf4_code_tree(load1<SRC>(src, base + c + 1) * inv);
    packed[row * (cols / 2) + (gi * block + c) / 2] = (uint8_t)((hi << 4) | lo);
  }
}

template <int OUT>
__global__ void __launch_bounds__(kT)
dequant_nf4_generic(const uint8_t* __restrict__ packed, const float* __restrict__ absmax,
                    int64_t rows, int64_t cols, int64_t block, void* __restrict__ out,
                    int64_t ostride) {
  const int64_t t = (int64_t)blockIdx.x * kT + threadIdx.x;
  if (t >= rows * (cols / 2)) return;
  const int64_t row = t / (cols / 2), cb = t - row * (cols / 2);
  const uint32_t b = packed[t];
  const float s = absmax[row * (cols / block) + (cb * 2) / block];
  store1<OUT>(out, row * ostride + cb * 2, kNf4Lut[b >> 4] * s);
  store1<OUT>(out, row * ostride + cb * 2 + 1, kNf4Lut[b & 0xFu] * s);
}

// ------------------------------------------------------------------ NVFP4

// fp32 -> float8_e4m3fn bits: round to nearest even, subnormal step 2^-9,
// everything at or above 480 (and NaN) -> 0x7F.
__device__ __forceinline__ uint32_t f32_to_e4m3fn_bits(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint32_t sign = (u >> 24) & 0x80u;
  uint32_t a = u & 0x7FFFFFFFu;
  uint32_t r;
  if (a >= 0x43F00000u) {
    r = 0x7Fu;
  } else if (a < 0x3C800000u) {
    r = (uint32_t)__builtin_rintf(__uint_as_float(a) * 512.0f);
  } else {
    const uint32_t odd = (a >> 20) & 1u;
    a += ((uint32_t)(7 - 127) << 23) + 0x7FFFFu;
    a += odd;
    r = (a >> 20) & 0xFFu;
  }
  return sign | r;
}

__device__ __forceinline__ float e4m3fn_bits_to_f32(uint32_t b) {
  const uint32_t sign = (b & 0x80u) << 24;
  const uint32_t e = (b >> 3) & 0xFu, m = b & 7u;
  uint32_t mag;
  if (e == 0xFu && m == 7u) mag = 0x7FC00000u;
  else if (e == 0) mag = __float_as_uint((float)m * (1.0f / 512.0f));
  else mag = ((e + 120u) << 23) | (m << 20);
  return __uint_as_float(sign | mag);
}

// e2m1 code, round to nearest even on the magnitude grid {0,.5,1,1.5,2,3,4,6},
// saturating; bit 3 is the IEEE sign bit (so -0 encodes as 8).
__device__ __forceinline__ uint32_t e2m1_code(float x) {
  const float ax = fabsf(x);
  const uint32_t pos = (uint32_t)(ax > 0.25f) + (uint32_t)(ax >= 0.75f) +
                       (uint32_t)(ax > 1.25f) + (uint32_t)(ax >= 1.75f) +
                       (uint32_t)(ax > 2.5f) + (uint32_t)(ax >= 3.5f) +
                       (uint32_t)(ax > 5.0f);
  return pos | ((__float_as_uint(x) >> 31) << 3);
}

__device__ __forceinline__ float e2m1_value(uint32_t code) {
  const uint32_t pos = code & 7u;
  uint32_t mag = ((126u + (pos >> 1)) << 23) | ((pos & 1u) << 22);
  if (pos == 1u) mag = 126u << 23;  // 0.5: the only subnormal of the format
  if (pos == 0u) mag = 0u;
  return __uint_as_float(((code & 8u) << 28) | mag);
}

constexpr int kAmaxMaxBlocks = 16384;  // floats of the shared norm/amax workspace
#ifndef OA_AMAX_UNROLL
#define OA_AMAX_UNROLL 4
#endif
constexpr int kAmaxUnroll = OA_AMAX_UNROLL;  // octets in flight per lane

// Tensor-wide max |x|, first launch: one partial maximum per block.  Octets of a
// row-contiguous matrix are addressed flat (no per-octet division).
template <int SRC>
__global__ void __launch_bounds__(kT)
nvfp4_amax_partial_kernel(const void* __restrict__ src, int64_t stride, int64_t rows,
                          int64_t cols, int vec, float* __restrict__ partial,
                          const AdamSrc ad) {
  constexpr int kAmaxUnroll = SRC == kSrcAdam ? 1 : oa::kAmaxUnroll;  // as in quant_nf4_kernel
  __shared__ float lds[kT / kWave];
  float a = 0.0f;
  const int64_t step = (int64_t)gridDim.x * kT;
  if (vec) {
    const int64_t opr = cols >> 3, total = rows * opr;
    const bool flat = stride == cols;
    const int64_t tile = SRC == kSrcAdam ? xcd_tile<kCodecXcdChunk>(blockIdx.x) : blockIdx.x;
    int64_t ob = tile * kT * kAmaxUnroll;  // the trip's first octet (the same in every lane)
    for (; ob < total; ob += step * kAmaxUnroll) {
      const int64_t o = ob + threadIdx.x;
      float x[kAmaxUnroll][8];
      // every lane of every trip in range (a scalar condition): loads without guards,
      // all in flight together
      if (flat && SRC != kSrcAdam && ob + (int64_t)kAmaxUnroll * kT <= total) {
#pragma unroll
        for (int k = 0; k < kAmaxUnroll; ++k)
          fetch8<SRC>(src, ad, (o + (int64_t)k * kT) * 8, x[k]);
#pragma unroll
        for (int k = 0; k < kAmaxUnroll; ++k) a = fmaxf(a, absmax8(x[k]));
        continue;
      }
#pragma unroll
      for (int k = 0; k < kAmaxUnroll; ++k) {
        const int64_t ok = o + (int64_t)k * kT;
        if (ok < total) {
          int64_t at = ok * 8;
          if (!flat) {
            const int64_t row = ok / opr;
            at = row * stride + (ok - row * opr) * 8;
          }
          fetch8<SRC>(src, ad, at, x[k]);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) x[k][j] = 0.0f;
        }
      }
#pragma unroll
      for (int k = 0; k < kAmaxUnroll; ++k) a = fmaxf(a, absmax8(x[k]));
    }
  } else {
    const int64_t total = rows * cols;
    for (int64_t i = (int64_t)blockIdx.x * kT + threadIdx.x; i < total; i += step) {
      const int64_t row = i / cols, c = i - row * cols;
      a = fmaxf(a, fabsf(load1<SRC>(src, row * stride + c)));
    }
  }
  const float m = block_max(a, lds);
  if (threadIdx.x == 0) partial[blockIdx.x] = m;
}

// Second launch: global scale = max(amax, 1e-12) / (448 * 6).  One block of 1024
// lanes, 4 partials per lane per trip, so 16384 partials are 4 dependent trips.
constexpr int kScaleThreads = 1024;
__global__ void __launch_bounds__(kScaleThreads)
nvfp4_global_scale_kernel(const float* __restrict__ partial, int blocks,
                          float* __restrict__ gs_out) {
  __shared__ float lds[kScaleThreads / kWave];
  float t = 0.0f;
  for (int b = threadIdx.x; b < blocks; b += 4 * kScaleThreads) {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int i = b + k * kScaleThreads;
      v[k] = i < blocks ? partial[i] : 0.0f;
    }
    t = fmaxf(fmaxf(t, fmaxf(v[0], v[1])), fmaxf(v[2], v[3]));
  }
  t = wave_max(t);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = t;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = lds[0];
#pragma unroll
    for (int w = 1; w < kScaleThreads / kWave; ++w) m = fmaxf(m, lds[w]);
    *gs_out = fmaxf(m, kEps) / (448.0f * 6.0f);
  }
}

// Eight e2m1 codes, even element in the low nibble.  gfx950 converts a pair of
// fp32 values to packed FP4 in one instruction (v_cvt_scalef32_pk_fp4_f32 with a
// scale of 1: round to nearest even on the e2m1 grid, saturating at 6, the sign
// of zero kept) - bit for bit what e2m1_code() computes for every non-NaN input
// (checked on the GPU over every float within 64 ulps of each grid point and
// rounding boundary, a 1e-5 sweep of [-8, 8], denormals, infinities and
// FLT_MAX).  A NaN becomes +-6 here and +-0 in e2m1_code(); a tensor with a NaN
// has a NaN scale in the reference and is outside the codec's contract.
__device__ __forceinline__ uint32_t nvfp4_pack8(const float (&x)[8], float inv_eff) {
  uint32_t w = 0;
  w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[0] * inv_eff, x[1] * inv_eff, 1.0f, 0);
  w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[2] * inv_eff, x[3] * inv_eff, 1.0f, 1);
  w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[4] * inv_eff, x[5] * inv_eff, 1.0f, 2);
  w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[6] * inv_eff, x[7] * inv_eff, 1.0f, 3);
  return w;
}

// block scale of a 16-element block from its amax
__device__ __forceinline__ uint32_t nvfp4_block_scale(float amax, float inv_global) {
  const float bs32 = fmaxf(amax, kEps) / 6.0f;
  return f32_to_e4m3fn_bits(bs32 * inv_global);
}

// Flat over octets, two lanes per 16-element block.
template <int SRC>
__global__ void __launch_bounds__(kT)
quant_nvfp4_kernel(const void* __restrict__ src, int64_t stride, int64_t rows, int64_t cols,
                   uint32_t* __restrict__ packed, uint8_t* __restrict__ scale8,
                   const float* __restrict__ gs_ptr, int mode) {
  const int64_t opr = cols >> 3, total = rows * opr;
  const int64_t o0 = (int64_t)blockIdx.x * (kT * kOct) + threadIdx.x;
  float x[kOct][8];
#pragma unroll
  for (int k = 0; k < kOct; ++k) {
    const int64_t o = o0 + (int64_t)k * kT;
    if (o < total) {
      load8<SRC>(src, octet_elem(o, opr, stride, mode), x[k]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) x[k][j] = 0.0f;
    }
  }
  const float gs = *gs_ptr;
  const float inv_global = 1.0f / gs;
  const int lane = threadIdx.x & (kWave - 1), base = lane & ~7;
#pragma unroll
  for (int k = 0; k < kOct; ++k) {
    const int64_t o = o0 + (int64_t)k * kT;
    const float amax = group_max(absmax8(x[k]), 2);
    const uint32_t s8 = nvfp4_block_scale(amax, inv_global);
    const float eff = e4m3fn_bits_to_f32(s8) * gs;
    const float inv_eff = 1.0f / fmaxf(eff, kEps);
    // gather the scales of the 4 blocks covered by 8 consecutive lanes
    const uint32_t s4 = __shfl(s8, base, kWave) | (__shfl(s8, base + 2, kWave) << 8) |
                        (__shfl(s8, base + 4, kWave) << 16) | (__shfl(s8, base + 6, kWave) << 24);
    if (o >= total) continue;
    __builtin_nontemporal_store(nvfp4_pack8(x[k], inv_eff), packed + o);
    const int64_t o_base = o - (lane & 7);
    if (o_base + 8 <= total) {
      if ((lane & 7) == 0) *reinterpret_cast<uint32_t*>(scale8 + (o_base >> 1)) = s4;
    } else if ((lane & 1) == 0) {
      scale8[o >> 1] = (uint8_t)s8;
    }
  }
}

// Row-contiguous matrices, 32 consecutive elements (two 16-element blocks) per
// lane: block maxima need no shuffle, each block's scale arithmetic runs once
// (not once in each of the two lanes that share a block in the octet kernel), and
// the codes leave as one 16-byte store, the two scale bytes as one 2-byte store.
template <int SRC>
__global__ void __launch_bounds__(kQuadT)
quant_nvfp4_quad_kernel(const void* __restrict__ src, int64_t quads, u32x4* __restrict__ packed,
                        uint16_t* __restrict__ scale16, const float* __restrict__ gs_ptr) {
  __shared__ u32x4 stage[quad_lds_slots<SRC>()];
  const int64_t qbase = (int64_t)blockIdx.x * (kQuadT * kQuadChunks);
  QuadRaw<SRC> cur, nxt;
  quad_load<SRC>(src, qbase, quads * 4, cur);
  const float gs = *gs_ptr;
  const float inv_global = 1.0f / gs;
#pragma unroll
  for (int c = 0; c < kQuadChunks; ++c) {
    const int64_t q0 = qbase + (int64_t)c * kQuadT;
    if (q0 >= quads) break;
    const bool more = c + 1 < kQuadChunks && q0 + kQuadT < quads;
    if (more) quad_load<SRC>(src, q0 + kQuadT, quads * 4, nxt);
    float x[4][8];
    quad_exchange<SRC>(cur, stage, x);
    u32x4 w;
    uint32_t s2 = 0;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const float amax = fmaxf(absmax8(x[2 * b]), absmax8(x[2 * b + 1]));
      const uint32_t s8 = nvfp4_block_scale(amax, inv_global);
      const float eff = e4m3fn_bits_to_f32(s8) * gs;
      const float inv_eff = 1.0f / fmaxf(eff, kEps);
      w[2 * b] = nvfp4_pack8(x[2 * b], inv_eff);
      w[2 * b + 1] = nvfp4_pack8(x[2 * b + 1], inv_eff);
      s2 |= s8 << (8 * b);
    }
    const int64_t q = q0 + threadIdx.x;
    if (q < quads) {
      __builtin_nontemporal_store(w, packed + q);
      scale16[q] = (uint16_t)s2;
    }
    cur = nxt;
  }
}

template <int OUT>
__global__ void __launch_bounds__(kT)
dequant_nvfp4_kernel(const uint32_t* __restrict__ packed, const uint8_t* __restrict__ scale8,
                     const float* __restrict__ gs_ptr, int64_t rows, int64_t cols,
                     void* __restrict__ out, int64_t ostride, int mode) {
  const int64_t opr = cols >> 3, total = rows * opr;
  const int64_t o0 = (int64_t)blockIdx.x * (kT * kOct) + threadIdx.x;
  uint32_t w[kOct], sb[kOct];
#pragma unroll
  for (int k = 0; k < kOct; ++k) {
    const int64_t o = o0 + (int64_t)k * kT;
    w[k] = o < total ? packed[o] : 0u;
    sb[k] = o < total ? (uint32_t)scale8[o >> 1] : 0u;
  }
  const float gs = *gs_ptr;
#pragma unroll
  for (int k = 0; k < kOct; ++k) {
    const int64_t o = o0 + (int64_t)k * kT;
    if (o >= total) continue;
    const float eff = e4m3fn_bits_to_f32(sb[k]) * gs;
    // v_cvt_scalef32_pk_f32_fp4: the two e2m1 values of one byte, exact in fp32
    const f32x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[k], 1.0f, 0);
    const f32x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[k], 1.0f, 1);
    const f32x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[k], 1.0f, 2);
    const f32x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[k], 1.0f, 3);
    const float y[8] = {p0[0] * eff, p0[1] * eff, p1[0] * eff, p1[1] * eff,
                        p2[0] * eff, p2[1] * eff, p3[0] * eff, p3[1] * eff};
    store8<OUT>(out, octet_elem(o, opr, ostride, mode), y);
  }
}

// One lane per 16-element block: any alignment.
template <int SRC>
__global__ void __launch_bounds__(kT)
quant_nvfp4_generic(const void* __restrict__ src, int64_t stride, int64_t rows, int64_t cols,
                    uint8_t* __restrict__ packed, uint8_t* __restrict__ scale8,
                    const float* __restrict__ gs_ptr) {
  const int64_t ng = cols / 16;
  const int64_t t = (int64_t)blockIdx.x * kT + threadIdx.x;
  if (t >= rows * ng) return;
  const int64_t row = t / ng, gi = t - row * ng;
  const int64_t base = row * stride + gi * 16;
  const float gs = *gs_ptr;
  float a = 0.0f;
  for (int c = 0; c < 16; ++c) a = fmaxf(a, fabsf(load1<SRC>(src, base + c)));
  const uint32_t s8 = nvfp4_block_scale(a, 1.0f / gs);
  scale8[t] = (uint8_t)s8;
  const float inv_eff = 1.0f / fmaxf(e4m3fn_bits_to_f32(s8) * gs, kEps);
  for (int c = 0; c < 16; c += 2) {
    const uint32_t lo = e2m1_code(load1<SRC>(src, base + c) * inv_eff);
    const uint32_t hi = e2m1_code(load1<SRC>(src, base + c + 1) * inv_eff);
    packed[row * (cols / 2) + (gi * 16 + c) / 2] = (uint8_t)((hi << 4) | lo);
  }
}

template <int OUT>
__global__ void __launch_bounds__(kT)
dequant_nvfp4_generic(const uint8_t* __restrict__ packed, const uint8_t* __restrict__ scale8,
                      const float* __restrict__ gs_ptr, int64_t rows, int64_t cols,
                      void* __restrict__ out, int64_t ostride) {
  const int64_t t = (int64_t)blockIdx.x * kT + threadIdx.x;
  if (t >= rows * (cols / 2)) return;
  const int64_t row = t / (cols / 2), cb = t - row * (cols / 2);
  const uint32_t b = packed[t];
  const float eff = e4m3fn_bits_to_f32(scale8[row * (cols / 16) + cb / 8]) * (*gs_ptr);
  store1<OUT>(out, row * ostride + cb * 2, e2m1_value(b & 0xFu) * eff);
  store1<OUT>(out, row * ostride + cb * 2 + 1, e2m1_value(b >> 4) * eff);
}

// ------------------------------------------------------------ host helpers

inline bool valid_dt(int dt) { return dt == OA_F32 || dt == OA_BF16 || dt == OA_F16; }
inline int64_t esize(int dt) { return dt == OA_F32 ? 4 : 2; }
inline bool pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
inline unsigned blocks_for(int64_t work) { return (unsigned)((work + kT - 1) / kT); }
inline unsigned blocks_oct(int64_t octets) {
  return (unsigned)((octets + (int64_t)kT * kOct - 1) / ((int64_t)kT * kOct));
}
inline int addr_mode(int64_t rows, int64_t cols, int64_t stride) {
  if (stride == cols || rows <= 1) return kFlat;
  return rows * (cols / 8) < (int64_t(1) << 31) ? kDiv32 : kDiv64;
}
inline int div_mode(int64_t rows, int64_t cols) {  // when the row index itself is needed
  return rows * (cols / 8) < (int64_t(1) << 31) ? kDiv32 : kDiv64;
}
inline int log2i(int64_t v) {
  int s = 0;
  while ((int64_t(1) << s) < v) ++s;
  return s;
}

// fast path: rows of 8-element octets that all start on 16-byte boundaries
inline bool rows_vec(const void* p, int dt, int64_t stride, int64_t cols) {
  return cols % 8 == 0 && aligned_to(p, 16) && (stride * esize(dt)) % 16 == 0;
}

#define OA_DISPATCH_WPR(wpr, CALL)                    \
  switch (wpr) {                                      \
    case 16: { constexpr int W = 16; CALL; break; }   \
    case 8: { constexpr int W = 8; CALL; break; }     \
    case 4: { constexpr int W = 4; CALL; break; }     \
    default: { constexpr int W = 0; CALL; break; }    \
  }

#define OA_DISPATCH_DT(dt, CALL)                      \
  switch (dt) {                                       \
    case OA_F32: { constexpr int DT = OA_F32; CALL; break; }   \
    case OA_BF16: { constexpr int DT = OA_BF16; CALL; break; } \
    default: { constexpr int DT = OA_F16; CALL; break; }       \
  }

int check_matrix(const void* m, int dt, int64_t stride, int64_t rows, int64_t cols) {
  if (!valid_dt(dt) || rows < 0 || cols < 0 || stride < cols) return OA_EINVAL;
  if (rows * cols > 0 && !m) return OA_EINVAL;
  if (!aligned_to(m, (uintptr_t)esize(dt))) return OA_EALIGN;
  if (rows > 0x7FFFFFFFll || rows * cols / 8 / kT > 0x7FFFFFFFll) return OA_ERANGE;
  return 0;
}

}  // namespace
}  // namespace oa

using namespace oa;

extern "C" int oa_quant_int8(const void* src, int src_dtype, int64_t src_row_stride,
                             int64_t rows, int64_t cols, void* q, void* scales,
                             int scale_dtype, void* stream) {
  int rc = check_matrix(src, src_dtype, src_row_stride, rows, cols);
  if (rc) return rc;
  if (!valid_dt(scale_dtype)) return OA_EINVAL;
  if (rows == 0) return 0;
  if (!q && cols > 0) return OA_EINVAL;
  if (!scales) return OA_EINVAL;
  if (!aligned_to(scales, (uintptr_t)esize(scale_dtype))) return OA_EALIGN;
  const int vec = rows_vec(src, src_dtype, src_row_stride, cols) && aligned_to(q, 8);
  hipStream_t s = static_cast<hipStream_t>(stream);
  OA_DISPATCH_DT(src_dtype,
                 hipLaunchKernelGGL(quant_int8_kernel<DT>, dim3((unsigned)rows), dim3(kT), 0, s,
                                    src, src_row_stride, cols, static_cast<int8_t*>(q), scales,
                                    scale_dtype, vec, AdamSrc{}));
  return launch_status();
}

extern "C" int oa_dequant_int8(const void* q, const void* scales, int scale_dtype,
                               int64_t rows, int64_t cols, void* out, int out_dtype,
                               int64_t out_row_stride, void* stream) {
  int rc = check_matrix(out, out_dtype, out_row_stride, rows, cols);
  if (rc) return rc;
  if (!valid_dt(scale_dtype)) return OA_EINVAL;
  if (rows * cols == 0) return 0;
  if (!q || !scales) return OA_EINVAL;
  if (!aligned_to(scales, (uintptr_t)esize(scale_dtype))) return OA_EALIGN;
  const int vec = rows_vec(out, out_dtype, out_row_stride, cols) && aligned_to(q, 8);
  const unsigned blocks = vec ? blocks_oct(rows * (cols / 8)) : blocks_for(rows * cols);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (vec) {
    const int mode = div_mode(rows, cols);
#define OA_I8_HEX(SD)                                                                        \
  OA_DISPATCH_DT(out_dtype,                                                                  \
                 hipLaunchKernelGGL((dequant_int8_tile_kernel<DT, SD>), dim3(blocks), dim3(kT), \
                                    0, s, static_cast<const int8_t*>(q), scales, rows, cols,  \
                                    out, out_row_stride, mode))
    if (scale_dtype == OA_F32) {
      OA_I8_HEX(OA_F32);
    } else if (scale_dtype == OA_BF16) {
      OA_I8_HEX(OA_BF16);
    } else {
      OA_I8_HEX(OA_F16);
    }
#undef OA_I8_HEX
    return launch_status();
  }
  OA_DISPATCH_DT(out_dtype,
                 hipLaunchKernelGGL(dequant_int8_kernel<DT>, dim3(blocks), dim3(kT), 0,
                                    s, static_cast<const int8_t*>(q), scales, scale_dtype, rows,
                                    cols, out, out_row_stride, vec, div_mode(rows, cols)));
  return launch_status();
}

extern "C" int oa_quant_int4(const void* src, int src_dtype, int64_t src_row_stride,
                             int64_t rows, int64_t cols, int64_t group, void* qweight,
                             void* scales, int scale_dtype, void* stream) {
  int rc = check_matrix(src, src_dtype, src_row_stride, rows, cols);
  if (rc) return rc;
  if (!valid_dt(scale_dtype) || group <= 0 || group % 8 != 0 || cols % group != 0)
    return OA_EINVAL;
  if (rows * cols == 0) return 0;
  if (!qweight || !scales) return OA_EINVAL;
  if (!aligned_to(qweight, 4) || !aligned_to(scales, (uintptr_t)esize(scale_dtype)))
    return OA_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t ng = cols / group;
  const bool fast = rows_vec(src, src_dtype, src_row_stride, cols) && pow2(group) &&
                    group <= 512 && i4_grid_ok((rows + kI4RowsQ - 1) / kI4RowsQ, ng);
  if (fast) {
    const int wpr = (int)(group / 8);
    const size_t lds = (size_t)wpr * kI4PitchQ * 4 + kI4RowsQ * 4;
    const dim3 grid = i4_grid((unsigned)((rows + kI4RowsQ - 1) / kI4RowsQ), (unsigned)ng);
    OA_DISPATCH_DT(src_dtype, OA_DISPATCH_WPR(
        wpr, hipLaunchKernelGGL((quant_int4_kernel<DT, W>), grid, dim3(kT), lds, s, src,
                                src_row_stride, rows, (int)group,
                                static_cast<int32_t*>(qweight), scales, scale_dtype,
                                AdamSrc{})));
  } else {
    OA_DISPATCH_DT(src_dtype,
                   hipLaunchKernelGGL(quant_int4_generic<DT>, dim3(blocks_for(rows * ng)),
                                      dim3(kT), 0, s, src, src_row_stride, rows, cols, group,
                                      static_cast<int32_t*>(qweight), scales, scale_dtype));
  }
  return launch_status();
}

extern "C" int oa_dequant_int4(const void* qweight, const void* scales, int scale_dtype,
                               int64_t rows, int64_t cols, int64_t group, void* out,
                               int out_dtype, int64_t out_row_stride, void* stream) {
  int rc = check_matrix(out, out_dtype, out_row_stride, rows, cols);
  if (rc) return rc;
  if (!valid_dt(scale_dtype) || group <= 0 || group % 8 != 0 || cols % group != 0)
    return OA_EINVAL;
  if (rows * cols == 0) return 0;
  if (!qweight || !scales) return OA_EINVAL;
  if (!aligned_to(qweight, 4) || !aligned_to(scales, (uintptr_t)esize(scale_dtype)))
    return OA_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t ng = cols / group;
  const bool fast = rows_vec(out, out_dtype, out_row_stride, cols) && pow2(group) &&
                    group <= 512 && i4_grid_ok((rows + kI4RowsD - 1) / kI4RowsD, ng);
  if (fast) {
    const int wpr = (int)(group / 8);
    const size_t lds = (size_t)wpr * (kI4RowsD + 1) * 4 + kI4RowsD * 4;
    const dim3 grid = i4_grid((unsigned)((rows + kI4RowsD - 1) / kI4RowsD), (unsigned)ng);
    OA_DISPATCH_DT(out_dtype, OA_DISPATCH_WPR(
        wpr, hipLaunchKernelGGL((dequant_int4_kernel<DT, W>), grid, dim3(kT), lds, s,
                                static_cast<const int32_t*>(qweight), scales, scale_dtype,
                                rows, (int)group, out, out_row_stride)));
  } else {
    OA_DISPATCH_DT(out_dtype,
                   hipLaunchKernelGGL(dequant_int4_generic<DT>,
                                      dim3(blocks_for(rows * (cols / 8))), dim3(kT), 0, s,
                                      static_cast<const int32_t*>(qweight), scales, scale_dtype,
                                      rows, cols, group, out, out_row_stride));
  }
  return launch_status();
}

extern "C" int oa_quant_nf4(const void* src, int src_dtype, int64_t src_row_stride,
                            int64_t rows, int64_t cols, int64_t block, void* packed,
                            void* absmax, void* stream) {
  int rc = check_matrix(src, src_dtype, src_row_stride, rows, cols);
  if (rc) return rc;
  if (block <= 0 || block % 2 != 0 || cols % block != 0) return OA_EINVAL;
  if (rows * cols == 0) return 0;
  if (!packed || !absmax) return OA_EINVAL;
  if (!aligned_to(absmax, 4)) return OA_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool fast = rows_vec(src, src_dtype, src_row_stride, cols) && block % 8 == 0 &&
                    pow2(block / 8) && block <= 512 && aligned_to(packed, 4);
  // whole 32-element quads in one contiguous run, 16-byte aligned stores
  const bool quad = fast && (src_row_stride == cols || rows <= 1) && block % 32 == 0 &&
                    pow2(block / 32) && block <= 2048 && aligned_to(packed, 16);
  if (quad) {
    const int64_t quads = rows * cols / 32;
    const int lpb = (int)(block / 32);
    OA_DISPATCH_DT(src_dtype,
                   hipLaunchKernelGGL((block == 64 ? quant_nf4_quad_kernel<DT, 2>
                                                   : quant_nf4_quad_kernel<DT, 0>),
                                      dim3((unsigned)((quads + kQuadT * kQuadChunks - 1) / (kQuadT * kQuadChunks))),
                                      dim3(kQuadT), 0, s, src, quads, lpb, log2i(lpb),
                                      static_cast<u32x4*>(packed), static_cast<float*>(absmax)));
  } else if (fast) {
    OA_DISPATCH_DT(src_dtype,
                   hipLaunchKernelGGL((block == 64 ? quant_nf4_kernel<DT, 8> : quant_nf4_kernel<DT, 0>), dim3(blocks_oct(rows * (cols / 8))),
                                      dim3(kT), 0, s, src, src_row_stride, rows, cols,
                                      (int)(block / 8), log2i(block / 8),
                                      static_cast<uint32_t*>(packed), static_cast<float*>(absmax),
                                      addr_mode(rows, cols, src_row_stride), AdamSrc{}));
  } else {
    OA_DISPATCH_DT(src_dtype,
                   hipLaunchKernelGGL(quant_nf4_generic<DT>,
                                      dim3(blocks_for(rows * (cols / block))), dim3(kT), 0, s,
                                      src, src_row_stride, rows, cols, block,
                                      static_cast<uint8_t*>(packed), static_cast<float*>(absmax)));
  }
  return launch_status();
}

extern "C" int oa_dequant_nf4(const void* packed, const void* absmax, int64_t rows,
                              int64_t cols, int64_t block, void* out, int out_dtype,
                              int64_t out_row_stride, void* stream) {
  int rc = check_matrix(out, out_dtype, out_row_stride, rows, cols);
  if (rc) return rc;
  if (block <= 0 || block % 2 != 0 || cols % block != 0) return OA_EINVAL;
  if (rows * cols == 0) return 0;
  if (!packed || !absmax) return OA_EINVAL;
  if (!aligned_to(absmax, 4)) return OA_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool fast = rows_vec(out, out_dtype, out_row_stride, cols) && block % 8 == 0 &&
                    pow2(block / 8) && block <= 512 && aligned_to(packed, 4);
  if (fast) {
    OA_DISPATCH_DT(out_dtype,
                   hipLaunchKernelGGL(dequant_nf4_kernel<DT>, dim3(blocks_oct(rows * (cols / 8))),
                                      dim3(kT), 0, s, static_cast<const uint32_t*>(packed),
                                      static_cast<const float*>(absmax), rows, cols,
                                      log2i(block / 8), out, out_row_stride,
                                      addr_mode(rows, cols, out_row_stride)));
  } else {
    OA_DISPATCH_DT(out_dtype,
                   hipLaunchKernelGGL(dequant_nf4_generic<DT>,
                                      dim3(blocks_for(rows * (cols / 2))), dim3(kT), 0, s,
                                      static_cast<const uint8_t*>(packed),
                                      static_cast<const float*>(absmax), rows, cols, block, out,
                                      out_row_stride));
  }
  return launch_status();
}

extern "C" int oa_quant_nvfp4(const void* src, int src_dtype, int64_t src_row_stride,
                              int64_t rows, int64_t cols, void* packed, void* block_scale,
                              void* global_scale, void* workspace, void* stream) {
  int rc = check_matrix(src, src_dtype, src_row_stride, rows, cols);
  if (rc) return rc;
  if (cols % 16 != 0 || !global_scale || !workspace) return OA_EINVAL;
  if (!aligned_to(global_scale, 4) || !aligned_to(workspace, 64)) return OA_EALIGN;
  if (rows * cols > 0 && (!packed || !block_scale)) return OA_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int vec = rows_vec(src, src_dtype, src_row_stride, cols);
  const int64_t per_block = (int64_t)kT * (vec ? kAmaxUnroll : 8);
  const int64_t work = vec ? rows * (cols / 8) : rows * cols;
  int64_t rblocks = (work + per_block - 1) / per_block;
  if (rblocks < 1) rblocks = 1;
  if (rblocks > kAmaxMaxBlocks) rblocks = kAmaxMaxBlocks;
  float* partial = static_cast<float*>(workspace);
  OA_DISPATCH_DT(src_dtype,
                 hipLaunchKernelGGL(nvfp4_amax_partial_kernel<DT>, dim3((unsigned)rblocks),
                                    dim3(kT), 0, s, src, src_row_stride, rows, cols, vec,
                                    partial, AdamSrc{}));
  rc = launch_status();
  if (rc) return rc;
  hipLaunchKernelGGL(nvfp4_global_scale_kernel, dim3(1), dim3(kScaleThreads), 0, s, partial,
                     (int)rblocks,
                     static_cast<float*>(global_scale));
  rc = launch_status();
  if (rc || rows * cols == 0) return rc;
  if (vec && (src_row_stride == cols || rows <= 1) && (rows * cols) % 32 == 0 &&
      aligned_to(packed, 16) && aligned_to(block_scale, 2)) {
    const int64_t quads = rows * cols / 32;
    OA_DISPATCH_DT(src_dtype,
                   hipLaunchKernelGGL(quant_nvfp4_quad_kernel<DT>,
                                      dim3((unsigned)((quads + kQuadT * kQuadChunks - 1) / (kQuadT * kQuadChunks))),
                                      dim3(kQuadT), 0, s, src, quads, static_cast<u32x4*>(packed),
                                      static_cast<uint16_t*>(block_scale),
                                      static_cast<const float*>(global_scale)));
  } else if (vec && aligned_to(packed, 4) && aligned_to(block_scale, 4)) {
    OA_DISPATCH_DT(src_dtype,
                   hipLaunchKernelGGL(quant_nvfp4_kernel<DT>, dim3(blocks_oct(rows * (cols / 8))),
                                      dim3(kT), 0, s, src, src_row_stride, rows, cols,
                                      static_cast<uint32_t*>(packed),
                                      static_cast<uint8_t*>(block_scale),
                                      static_cast<const float*>(global_scale),
                                      addr_mode(rows, cols, src_row_stride)));
  } else {
    OA_DISPATCH_DT(src_dtype,
                   hipLaunchKernelGGL(quant_nvfp4_generic<DT>,
                                      dim3(blocks_for(rows * (cols / 16))), dim3(kT), 0, s, src,
                                      src_row_stride, rows, cols, static_cast<uint8_t*>(packed),
                                      static_cast<uint8_t*>(block_scale),
                                      static_cast<const float*>(global_scale)));
  }
  return launch_status();
}

extern "C" int oa_dequant_nvfp4(const void* packed, const void* block_scale,
                                const void* global_scale, int64_t rows, int64_t cols,
                                void* out, int out_dtype, int64_t out_row_stride,
                                void* stream) {
  int rc = check_matrix(out, out_dtype, out_row_stride, rows, cols);
  if (rc) return rc;
  if (cols % 16 != 0) return OA_EINVAL;
  if (rows * cols == 0) return 0;
  if (!packed || !block_scale || !global_scale) return OA_EINVAL;
  if (!aligned_to(global_scale, 4)) return OA_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (rows_vec(out, out_dtype, out_row_stride, cols) && aligned_to(packed, 4)) {
    OA_DISPATCH_DT(out_dtype,
                   hipLaunchKernelGGL(dequant_nvfp4_kernel<DT>,
                                      dim3(blocks_oct(rows * (cols / 8))), dim3(kT), 0, s,
                                      static_cast<const uint32_t*>(packed),
                                      static_cast<const uint8_t*>(block_scale),
                                      static_cast<const float*>(global_scale), rows, cols, out,
                                      out_row_stride, addr_mode(rows, cols, out_row_stride)));
  } else {
    OA_DISPATCH_DT(out_dtype,
                   hipLaunchKernelGGL(dequant_nvfp4_generic<DT>,
                                      dim3(blocks_for(rows * (cols / 2))), dim3(kT), 0, s,
                                      static_cast<const uint8_t*>(packed),
                                      static_cast<const uint8_t*>(block_scale),
                                      static_cast<const float*>(global_scale), rows, cols, out,
                                      out_row_stride));
  }
  return launch_status();
}

// ------------------------------------------- fp32_master AdamW + re-encode

namespace oa {
namespace {

// Checks of the operands the fused step shares; fills `ad`.  The fused kernels
// take whole octets only: cols % 8 == 0 and 16-byte aligned arrays.
int make_adam_src(const void* grad, void* exp_avg, void* exp_avg_sq, void* master, int64_t rows,
                  int64_t cols, float lr, float wd, float b1h, float b2h, float eps,
                  int decoupled, const void* clip, AdamSrc* ad) {
  if (rows < 0 || cols < 0) return OA_EINVAL;
  if (rows > 0x7FFFFFFFll || rows * cols / 8 / kT > 0x7FFFFFFFll) return OA_ERANGE;
  if (rows * cols == 0) return 0;
  if (!grad || !exp_avg || !exp_avg_sq || !master) return OA_EINVAL;
  if (cols % 8 != 0) return OA_EINVAL;
  if (!aligned_to(grad, 16) || !aligned_to(exp_avg, 16) || !aligned_to(exp_avg_sq, 16) ||
      !aligned_to(master, 16) || (clip && !aligned_to(clip, 2)))
    return OA_EALIGN;
  const void* w[3] = {exp_avg, exp_avg_sq, master};
  for (int i = 0; i < 3; ++i) {
    if (w[i] == grad) return OA_EOVERLAP;
    for (int j = i + 1; j < 3; ++j)
      if (w[i] == w[j]) return OA_EOVERLAP;
  }
  ad->g = static_cast<const uint16_t*>(grad);
  ad->m = static_cast<uint16_t*>(exp_avg);
  ad->v = static_cast<uint16_t*>(exp_avg_sq);
  ad->master = static_cast<float*>(master);
  ad->clip = static_cast<const uint16_t*>(clip);
  ad->lr = lr;
  ad->wd = wd;
  // single fp32 operations, the values the step kernels use
  volatile float lr_wd = lr * wd, omb1 = 1.0f - b1h, omb2 = 1.0f - b2h;
  ad->lr_wd = lr_wd;
  ad->omb1 = omb1;
  ad->omb2 = omb2;
  ad->eps = eps;
  ad->decoupled = decoupled != 0;
  return 0;
}

}  // namespace
}  // namespace oa

extern "C" int oa_adam_requant_int8(const void* grad, void* exp_avg, void* exp_avg_sq,
                                    void* master, int64_t rows, int64_t cols, float lr,
                                    float weight_decay, float beta1_hat, float beta2_hat,
                                    float eps, int decoupled, const void* clip_coef, void* q,
                                    void* scales, int scale_dtype, void* stream) {
  AdamSrc ad{};
  int rc = make_adam_src(grad, exp_avg, exp_avg_sq, master, rows, cols, lr, weight_decay,
                         beta1_hat, beta2_hat, eps, decoupled, clip_coef, &ad);
  if (rc || rows * cols == 0) return rc;
  if (!valid_dt(scale_dtype) || !q || !scales) return OA_EINVAL;
  if (!aligned_to(q, 8) || !aligned_to(scales, (uintptr_t)esize(scale_dtype))) return OA_EALIGN;
  hipLaunchKernelGGL(quant_int8_kernel<kSrcAdam>, dim3((unsigned)rows), dim3(kT), 0,
                     static_cast<hipStream_t>(stream), nullptr, cols, cols,
                     static_cast<int8_t*>(q), scales, scale_dtype, 1, ad);
  return launch_status();
}

extern "C" int oa_adam_requant_int4(const void* grad, void* exp_avg, void* exp_avg_sq,
                                    void* master, int64_t rows, int64_t cols, float lr,
                                    float weight_decay, float beta1_hat, float beta2_hat,
                                    float eps, int decoupled, const void* clip_coef,
                                    int64_t group, void* qweight, void* scales, int scale_dtype,
                                    void* stream) {
  AdamSrc ad{};
  int rc = make_adam_src(grad, exp_avg, exp_avg_sq, master, rows, cols, lr, weight_decay,
                         beta1_hat, beta2_hat, eps, decoupled, clip_coef, &ad);
  if (rc) return rc;
  if (!valid_dt(scale_dtype) || group <= 0 || group % 8 != 0 || cols % group != 0)
    return OA_EINVAL;
  if (rows * cols == 0) return 0;
  // the LDS-tile encoder only: power-of-two groups up to 512 columns
  if (!pow2(group) || group > 512 || !i4_grid_ok((rows + kI4RowsQ - 1) / kI4RowsQ, cols / group))
    return OA_EINVAL;
  if (!qweight || !scales) return OA_EINVAL;
  if (!aligned_to(qweight, 4) || !aligned_to(scales, (uintptr_t)esize(scale_dtype)))
    return OA_EALIGN;
  const int wpr = (int)(group / 8);
  const size_t lds = (size_t)wpr * kI4PitchQ * 4 + kI4RowsQ * 4;
  const dim3 grid = i4_grid((unsigned)((rows + kI4RowsQ - 1) / kI4RowsQ), (unsigned)(cols / group));
  OA_DISPATCH_WPR(wpr, hipLaunchKernelGGL((quant_int4_kernel<kSrcAdam, W>), grid, dim3(kT), lds,
                                          static_cast<hipStream_t>(stream), nullptr, cols, rows,
                                          (int)group, static_cast<int32_t*>(qweight), scales,
                                          scale_dtype, ad));
  return launch_status();
}

extern "C" int oa_adam_requant_nf4(const void* grad, void* exp_avg, void* exp_avg_sq,
                                   void* master, int64_t rows, int64_t cols, float lr,
                                   float weight_decay, float beta1_hat, float beta2_hat,
                                   float eps, int decoupled, const void* clip_coef,
                                   int64_t block, void* packed, void* absmax, void* stream) {
  AdamSrc ad{};
  int rc = make_adam_src(grad, exp_avg, exp_avg_sq, master, rows, cols, lr, weight_decay,
                         beta1_hat, beta2_hat, eps, decoupled, clip_coef, &ad);
  if (rc) return rc;
  if (block <= 0 || block % 8 != 0 || cols % block != 0) return OA_EINVAL;
  if (rows * cols == 0) return 0;
  if (!pow2(block / 8) || block > 512) return OA_EINVAL;
  if (!packed || !absmax) return OA_EINVAL;
  if (!aligned_to(packed, 4) || !aligned_to(absmax, 4)) return OA_EALIGN;
  hipLaunchKernelGGL((block == 64 ? quant_nf4_kernel<kSrcAdam, 8> : quant_nf4_kernel<kSrcAdam, 0>),
                     dim3(xcd_grid(blocks_for(rows * (cols / 8)), kCodecXcdChunk)),
                     dim3(kT), 0, static_cast<hipStream_t>(stream), nullptr, cols, rows, cols,
                     (int)(block / 8), log2i(block / 8), static_cast<uint32_t*>(packed),
                     static_cast<float*>(absmax), kFlat, ad);
  return launch_status();
}

extern "C" int oa_adam_requant_nvfp4(const void* grad, void* exp_avg, void* exp_avg_sq,
                                     void* master, int64_t rows, int64_t cols, float lr,
                                     float weight_decay, float beta1_hat, float beta2_hat,
                                     float eps, int decoupled, const void* clip_coef,
                                     void* packed, void* block_scale, void* global_scale,
                                     void* workspace, void* stream) {
  AdamSrc ad{};
  int rc = make_adam_src(grad, exp_avg, exp_avg_sq, master, rows, cols, lr, weight_decay,
                         beta1_hat, beta2_hat, eps, decoupled, clip_coef, &ad);
  if (rc) return rc;
  if (cols % 16 != 0 || !global_scale || !workspace) return OA_EINVAL;
  if (!aligned_to(global_scale, 4) || !aligned_to(workspace, 64)) return OA_EALIGN;
  if (rows * cols == 0) return 0;
  if (!packed || !block_scale) return OA_EINVAL;
  if (!aligned_to(packed, 4) || !aligned_to(block_scale, 4)) return OA_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t octets = rows * (cols / 8);
  // one octet per lane per trip; the grid is a whole number of XCD rounds
  // (kAmaxMaxBlocks is one), every block writes its partial maximum
  int64_t rblocks = (octets + kT - 1) / kT;
  if (rblocks > kAmaxMaxBlocks) rblocks = kAmaxMaxBlocks;
  rblocks = xcd_grid((uint32_t)rblocks, kCodecXcdChunk);
  static_assert(kAmaxMaxBlocks % (kXcds * kCodecXcdChunk) == 0, "padded grid must fit the workspace");
  float* partial = static_cast<float*>(workspace);
  // launch 1: the AdamW step, folding |new master| into per-block maxima
  hipLaunchKernelGGL(nvfp4_amax_partial_kernel<kSrcAdam>, dim3((unsigned)rblocks), dim3(kT), 0, s,
                     nullptr, cols, rows, cols, 1, partial, ad);
  rc = launch_status();
  if (rc) return rc;
  hipLaunchKernelGGL(nvfp4_global_scale_kernel, dim3(1), dim3(kScaleThreads), 0, s, partial,
                     (int)rblocks, static_cast<float*>(global_scale));
  rc = launch_status();
  if (rc) return rc;
  // launch 3: encode from the stored master
  if ((rows * cols) % 32 == 0 && aligned_to(packed, 16)) {
    const int64_t quads = rows * cols / 32;
    hipLaunchKernelGGL(quant_nvfp4_quad_kernel<OA_F32>,
                       dim3((unsigned)((quads + kQuadT * kQuadChunks - 1) / (kQuadT * kQuadChunks))),
                       dim3(kQuadT), 0, s, static_cast<const void*>(master), quads,
                       static_cast<u32x4*>(packed), static_cast<uint16_t*>(block_scale),
                       static_cast<const float*>(global_scale));
    return launch_status();
  }
  hipLaunchKernelGGL(quant_nvfp4_kernel<OA_F32>, dim3(blocks_oct(octets)), dim3(kT), 0, s,
                     static_cast<const void*>(master), cols, rows, cols,
                     static_cast<uint32_t*>(packed), static_cast<uint8_t*>(block_scale),
                     static_cast<const float*>(global_scale), kFlat);
  return launch_status();
}
