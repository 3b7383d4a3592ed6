// Fused AdamW update kernels for gfx950 (MI355X) and their C entry points.
//
// One launch per parameter, one pass over HBM: every lane moves 8 consecutive
// elements per array with 128-bit loads/stores (a wave reads 1 KiB contiguous
// per array), does the whole update in registers and writes the results back.
// No LDS, no matrix cores: the work is elementwise and HBM-bound
// (14-20 bytes per element).
//
// Arithmetic contract (what the reference's Triton kernels compute,
// src/offload_adam/kernels/*.py): fp32, one rounding per operation, correctly
// rounded sqrt and divide, denormals kept, bf16 stores round to nearest even.

#include "oa_common.hpp"

#pragma clang fp contract(off)

// One wave per workgroup, 8 elements per lane: tiles of 512 elements.  Measured
// against 256-lane workgroups (same bytes per XCD run): +2 % on a 1.1 B-element
// set of 4-12 M-element tensors, +6-8 % on an 8 B-element set of 17-59 M-element
// ones, in every mode; 128 lanes lie between.
#ifndef OA_ADAM_THREADS
#define OA_ADAM_THREADS 64
#endif
// Tiles an XCD takes in a row.  384 x 512 elements: within 0.5 % of the best run
// length for every mode and tensor size tried (256 is best for 4-12 M-element
// tensors, 384-2048 equal for larger ones, 4096 loses 4 % on the small ones).
#ifndef OA_ADAM_XCD_CHUNK
#define OA_ADAM_XCD_CHUNK 384
#endif
#ifndef OA_ADAM_UNROLL
#define OA_ADAM_UNROLL 1
#endif
#ifndef OA_ADAM_NT_LD
#define OA_ADAM_NT_LD 1
#endif
#ifndef OA_ADAM_NT_ST
#define OA_ADAM_NT_ST 1
#endif
// The fp32 master is read as two 16-byte halves per lane, so one wave
// instruction uses half of every 128-byte line it touches and the next one
// the other half: a temporal load lets the second hit in cache (+2.6 % on a
// 58.7 M-element tensor); the stores stay non-temporal (temporal: -4 %).
#ifndef OA_ADAM_MASTER_LD_NT
#define OA_ADAM_MASTER_LD_NT 0
#endif
#ifndef OA_ADAM_MASTER_ST_NT
#define OA_ADAM_MASTER_ST_NT 1
#endif

namespace oa {
namespace {

enum Mode : int { kFp32Master = 0, kStochastic = 1, kFp31 = 2, kCustom = 3 };

// Launch shape per mode.  A lane moves kDwords dwords of every 16-bit array per
// access (4 = eight elements, 2 = four); a workgroup has kThreads lanes; an XCD
// takes kChunk tiles in a row.  fp32_master reads and writes 4 bytes per element
// of master: with four elements per lane that is ONE 16-byte access per lane and a
// wave covers 1 KiB of consecutive master (with eight, two accesses that each use
// half of every line they touch); measured +3-4 % for that mode, while the other
// modes lose 3-15 % with four elements per lane (stochastic rounding would compute
// every Philox block in two lanes).
#ifndef OA_ADAM_FP32M_THREADS
#define OA_ADAM_FP32M_THREADS 128
#endif
#ifndef OA_ADAM_FP32M_XCD_CHUNK
#define OA_ADAM_FP32M_XCD_CHUNK 512
#endif
template <int MODE> struct Shape {
  static constexpr int kThreads = OA_ADAM_THREADS;
  static constexpr int kDwords = 4;
  static constexpr uint32_t kChunk = OA_ADAM_XCD_CHUNK;
};
template <> struct Shape<kFp32Master> {
  static constexpr int kThreads = OA_ADAM_FP32M_THREADS;
  static constexpr int kDwords = 2;
  static constexpr uint32_t kChunk = OA_ADAM_FP32M_XCD_CHUNK;
};
template <int MODE> constexpr int64_t tile_elems() {
  return (int64_t)Shape<MODE>::kThreads * OA_ADAM_UNROLL * Shape<MODE>::kDwords * 2;
}
template <int N> struct LaneVec;
template <> struct LaneVec<4> { using type = u32x4; };
template <> struct LaneVec<2> { using type = u32x2; };

struct AdamArgs {
  uint16_t* p;        // bf16 param (fp32_master: write-only sink)
  const uint16_t* g;  // bf16 grad, read-only
  uint16_t* m;        // bf16 exp_avg
  uint16_t* v;        // bf16 exp_avg_sq
  void* aux;          // f32 master | i16 rounding_error | nullptr
  const uint16_t* rand16;
  const uint16_t* clip;  // one bf16 scalar or nullptr
  int64_t n;
  float lr, wd, lr_wd, omb1, omb2, eps;
  uint32_t k0, k1;  // Philox key = (seed_lo, seed_hi)
};

template <typename T>
__device__ __forceinline__ T ld(const T* p) {
#if OA_ADAM_NT_LD
  return __builtin_nontemporal_load(p);
#else
  return *p;
#endif
}
template <typename T>
__device__ __forceinline__ void st(T* p, T x) {
#if OA_ADAM_NT_ST
  __builtin_nontemporal_store(x, p);
#else
  *p = x;
#endif
}

// The 16 random bits of element i under a Philox layout.
template <int RNG>
__device__ __forceinline__ uint32_t rand16_of(int64_t i, const AdamArgs& a) {
  if (RNG == OA_RNG_TRITON) {
    Philox r = philox4x32_10((uint32_t)i, (uint32_t)((uint64_t)i >> 32), 0u, 0u,
                             a.k0, a.k1);
    return r.c0 & 0xFFFFu;
  } else if (RNG == OA_RNG_X8) {
    const uint64_t j = (uint64_t)i >> 3;
    Philox r = philox4x32_10((uint32_t)j, (uint32_t)(j >> 32), 1u, 0u, a.k0, a.k1);
    const uint32_t e = (uint32_t)i & 7u;
    const uint32_t w = (e >> 1) == 0 ? r.c0 : (e >> 1) == 1 ? r.c1
                       : (e >> 1) == 2 ? r.c2 : r.c3;
    return (w >> ((e & 1u) * 16u)) & 0xFFFFu;
  } else {
    return a.rand16[i];
  }
}

// One element.  `pb` = bf16 bits of the param, `mb`/`vb` = bf16 bits of the
// moments, `aux` = fp32 master bits or the int16 rounding error (low 16 bits).
template <int MODE, bool DEC, bool CLIP>
__device__ __forceinline__ void adam_elem(uint32_t& pb, uint32_t gb, float& m,
                                          float& v, uint32_t& aux, uint32_t r16,
                                          float clip, const AdamArgs& a) {
  float g = bf16_bits_to_f32(gb);
  if (CLIP) g = bf16_bits_to_f32(f32_to_bf16_1(g * clip));

  float M;
  if (MODE == kFp32Master) {
    M = __uint_as_float(aux);
  } else if (MODE == kStochastic) {
    M = bf16_bits_to_f32(pb);
  } else if (MODE == kFp31) {
    const int32_t e = (int32_t)(int16_t)aux;
    M = __uint_as_float((pb << 16) + ((uint32_t)e << 1));
  } else {
    const int32_t e = (int32_t)(int16_t)aux;
    M = __uint_as_float((pb << 16) + (uint32_t)e);
  }

  adam_core(M, g, m, v, DEC, a.lr, a.wd, a.lr_wd, a.omb1, a.omb2, a.eps);

  const uint32_t x = __float_as_uint(M);
  if (MODE == kFp32Master) {
    aux = x;  // the caller stores bf16_rne(M) as the param
  } else if (MODE == kStochastic) {
    const uint32_t frac = x & 0xFFFFu;
    const uint32_t trunc = x & 0xFFFF0000u;
    pb = ((r16 < frac) ? trunc + 0x10000u : trunc) >> 16;
  } else if (MODE == kFp31) {
    // round to 31 bits, ties to even on bit 0 (arithmetic shifts)
    const int32_t xi = (int32_t)x;
    const int32_t up = xi & (xi >> 1) & 1;
    const uint32_t x31 = (uint32_t)((xi >> 1) + up) << 1;
    pb = f32_to_bf16_1(__uint_as_float(x31));
    const int32_t err = (int32_t)(x31 - (pb << 16));
    aux = (uint32_t)(err >> 1) & 0xFFFFu;
  } else {
    const int32_t xi = (int32_t)x;
    pb = (uint32_t)((xi + 0x8000) >> 16) & 0xFFFFu;
    aux = (x - (pb << 16)) & 0xFFFFu;
  }
}

// Scalar path: one element per lane per trip.  Used for buffers that are not
// 16-byte aligned and for the (n % 8) tail of the vector kernel.
template <int MODE, bool DEC, bool CLIP, int RNG>
__device__ __forceinline__ void adam_scalar(int64_t i, float clip,
                                            const AdamArgs& a) {
  uint32_t pb = (MODE == kFp32Master) ? 0u : a.p[i];
  const uint32_t gb = a.g[i];
  float m = bf16_bits_to_f32(a.m[i]);
  float v = bf16_bits_to_f32(a.v[i]);
  uint32_t aux = 0;
  if (MODE == kFp32Master) aux = reinterpret_cast<const uint32_t*>(a.aux)[i];
  if (MODE == kFp31 || MODE == kCustom)
    aux = reinterpret_cast<const uint16_t*>(a.aux)[i];
  uint32_t r16 = 0;
  if (MODE == kStochastic) r16 = rand16_of<RNG>(i, a);
  adam_elem<MODE, DEC, CLIP>(pb, gb, m, v, aux, r16, clip, a);
  if (MODE == kFp32Master) pb = f32_to_bf16_1(__uint_as_float(aux));
  if (MODE != kFp32Master || a.p) a.p[i] = (uint16_t)pb;  // fp32_master: the bf16 copy is optional
  a.m[i] = (uint16_t)f32_to_bf16_1(m);
  a.v[i] = (uint16_t)f32_to_bf16_1(v);
  if (MODE == kFp32Master) reinterpret_cast<uint32_t*>(a.aux)[i] = aux;
  if (MODE == kFp31 || MODE == kCustom)
    reinterpret_cast<uint16_t*>(a.aux)[i] = (uint16_t)aux;
}

template <int MODE, bool DEC, bool CLIP, int RNG>
__global__ void __launch_bounds__(OA_ADAM_THREADS)
adam_scalar_kernel(const AdamArgs a) {
  const float clip = CLIP ? bf16_bits_to_f32(*a.clip) : 1.0f;
  const int64_t stride = (int64_t)gridDim.x * OA_ADAM_THREADS;
  for (int64_t i = (int64_t)blockIdx.x * OA_ADAM_THREADS + threadIdx.x; i < a.n;
       i += stride)
    adam_scalar<MODE, DEC, CLIP, RNG>(i, clip, a);
}

// Vector path.  A "group" is the 8 (or 4) consecutive elements of one lane.  Block b owns groups
// [b*T*U, (b+1)*T*U); lane t takes groups b*T*U + k*T + t for k < U, so each
// wave touches 1 KiB of consecutive bytes per array per k.  All loads of the
// U groups are issued before any arithmetic to keep many bytes in flight.
// 16-bit arrays travel as four packed dwords (element 2j in the low half of
// dword j), which is also the layout the hardware bf16 convert produces.
template <int MODE, bool DEC, bool CLIP, int RNG>
__device__ __forceinline__ void adam_tile(const AdamArgs& a, int64_t tile, bool last_tile) {
  constexpr int T = Shape<MODE>::kThreads;
  constexpr int U = OA_ADAM_UNROLL;
  constexpr int W = Shape<MODE>::kDwords;   // dwords of a 16-bit array per lane
  constexpr int kShift = W == 4 ? 3 : 2;    // log2(elements per lane)
  constexpr int kQuads = W / 2;             // f32x4 accesses of the fp32 master per lane
  using uvec = typename LaneVec<W>::type;
  const int64_t n_groups = a.n >> kShift;
  const float clip = CLIP ? bf16_bits_to_f32(*a.clip) : 1.0f;
  const int64_t g0 = tile * (T * U) + threadIdx.x;

  uvec P[U], G[U], Mo[U], Vo[U], R[U], E[U];
  f32x4 Mq[U][kQuads];
  bool live[U];

#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t grp = g0 + (int64_t)k * T;
    live[k] = grp < n_groups;
    if (live[k]) {
      const int64_t e0 = grp << kShift;
      if (MODE != kFp32Master) P[k] = ld(reinterpret_cast<const uvec*>(a.p + e0));
      G[k] = ld(reinterpret_cast<const uvec*>(a.g + e0));
      Mo[k] = ld(reinterpret_cast<const uvec*>(a.m + e0));
      Vo[k] = ld(reinterpret_cast<const uvec*>(a.v + e0));
      if (MODE == kFp32Master) {
        const float* mp = reinterpret_cast<const float*>(a.aux) + e0;
#pragma unroll
        for (int q = 0; q < kQuads; ++q) {
#if OA_ADAM_MASTER_LD_NT
          Mq[k][q] = ld(reinterpret_cast<const f32x4*>(mp + 4 * q));
#else
          Mq[k][q] = *reinterpret_cast<const f32x4*>(mp + 4 * q);
#endif
        }
      }
      if (MODE == kFp31 || MODE == kCustom)
        E[k] = ld(reinterpret_cast<const uvec*>(
            reinterpret_cast<const uint16_t*>(a.aux) + e0));
      if (MODE == kStochastic && RNG == OA_RNG_BUFFER)
        R[k] = ld(reinterpret_cast<const uvec*>(a.rand16 + e0));
    }
  }

#pragma unroll
  for (int k = 0; k < U; ++k) {
    if (!live[k]) continue;
    const int64_t grp = g0 + (int64_t)k * T;
    const int64_t e0 = grp << kShift;

    uvec RW = {};
    if (MODE == kStochastic && RNG == OA_RNG_X8) {
      // one Philox block per eight elements, whatever a lane's share of them
      const uint64_t oct = (uint64_t)e0 >> 3;
      Philox r = philox4x32_10((uint32_t)oct, (uint32_t)(oct >> 32), 1u, 0u, a.k0, a.k1);
      const uint32_t words[4] = {r.c0, r.c1, r.c2, r.c3};
      const bool upper = W == 2 && (e0 & 4) != 0;  // second half of the block
#pragma unroll
      for (int j = 0; j < W; ++j) RW[j] = upper ? words[(j + 2) & 3] : words[j];
    }
    if (MODE == kStochastic && RNG == OA_RNG_BUFFER) RW = R[k];

    uvec Pn, Mn, Vn, En;
    f32x4 Mout[kQuads];
#pragma unroll
    for (int j = 0; j < W; ++j) {
      uint32_t pb[2], ax[2];
      float m[2], v[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int e = 2 * j + h;
        const uint32_t sh = h * 16;
        pb[h] = (MODE == kFp32Master) ? 0u : ((P[k][j] >> sh) & 0xFFFFu);
        const uint32_t gb = (G[k][j] >> sh) & 0xFFFFu;
        m[h] = h ? bf16hi_to_f32(Mo[k][j]) : bf16lo_to_f32(Mo[k][j]);
        v[h] = h ? bf16hi_to_f32(Vo[k][j]) : bf16lo_to_f32(Vo[k][j]);
        ax[h] = 0;
        if (MODE == kFp32Master)
          ax[h] = __float_as_uint(Mq[k][e >> 2][e & 3]);
        if (MODE == kFp31 || MODE == kCustom) ax[h] = (E[k][j] >> sh) & 0xFFFFu;
        uint32_t r16 = 0;
        if (MODE == kStochastic) {
          if (RNG == OA_RNG_TRITON) {
            const int64_t i = e0 + e;
            Philox r = philox4x32_10((uint32_t)i, (uint32_t)((uint64_t)i >> 32),
                                     0u, 0u, a.k0, a.k1);
            r16 = r.c0 & 0xFFFFu;
          } else {
            r16 = (RW[j] >> sh) & 0xFFFFu;
          }
        }
        adam_elem<MODE, DEC, CLIP>(pb[h], gb, m[h], v[h], ax[h], r16, clip, a);
      }
      Mn[j] = f32x2_to_bf16x2_bits(m[0], m[1]);
      Vn[j] = f32x2_to_bf16x2_bits(v[0], v[1]);
      if (MODE == kFp32Master) {
        const float M0 = __uint_as_float(ax[0]), M1 = __uint_as_float(ax[1]);
        Pn[j] = f32x2_to_bf16x2_bits(M0, M1);
        Mout[j >> 1][(2 * j) & 3] = M0;
        Mout[j >> 1][(2 * j + 1) & 3] = M1;
      } else {
        Pn[j] = pb[0] | (pb[1] << 16);
      }
      if (MODE == kFp31 || MODE == kCustom) En[j] = ax[0] | (ax[1] << 16);
    }

    st(reinterpret_cast<uvec*>(a.m + e0), Mn);
    st(reinterpret_cast<uvec*>(a.v + e0), Vn);
    if (MODE != kFp32Master || a.p) st(reinterpret_cast<uvec*>(a.p + e0), Pn);
    if (MODE == kFp32Master) {
      float* mp = reinterpret_cast<float*>(a.aux) + e0;
#pragma unroll
      for (int q = 0; q < kQuads; ++q) {
#if OA_ADAM_MASTER_ST_NT
        st(reinterpret_cast<f32x4*>(mp + 4 * q), Mout[q]);
#else
        *reinterpret_cast<f32x4*>(mp + 4 * q) = Mout[q];
#endif
      }
    }
    if (MODE == kFp31 || MODE == kCustom)
      st(reinterpret_cast<uvec*>(reinterpret_cast<uint16_t*>(a.aux) + e0), En);
  }

  // Tail: the elements after the last whole group, one lane each, in the tensor's last tile.
  if (last_tile) {
    const int64_t i = (n_groups << kShift) + threadIdx.x;
    if (i < a.n) adam_scalar<MODE, DEC, CLIP, RNG>(i, clip, a);
  }
}

template <int MODE, bool DEC, bool CLIP, int RNG>
__global__ void __launch_bounds__(Shape<MODE>::kThreads)
adam_vec_kernel(const AdamArgs a, uint32_t tiles) {
  const uint32_t tile = xcd_tile<Shape<MODE>::kChunk>(blockIdx.x);
  if (tile >= tiles) return;
  adam_tile<MODE, DEC, CLIP, RNG>(a, tile, tile == tiles - 1);
}

// Multi-tensor form: one launch covers up to kMultiMax parameters.  The
// per-tensor pointers and scalars travel in the kernel arguments (no device
// table, nothing to allocate); block b finds its tensor from the prefix sums of
// tiles with one load and one ballot, the same value in every lane.  Back-to-back tensors share
// one grid, so the ramp-up and drain of a launch are paid once per chunk
// instead of once per parameter.
constexpr int kMultiMax = 36;

struct MultiArgs {
  uint16_t* p[kMultiMax];
  const uint16_t* g[kMultiMax];
  uint16_t* m[kMultiMax];
  uint16_t* v[kMultiMax];
  void* aux[kMultiMax];
  int64_t n[kMultiMax];
  uint32_t tile_start[kMultiMax + 1];
  float omb1[kMultiMax], omb2[kMultiMax];
  uint32_t k0[kMultiMax], k1[kMultiMax];
  const uint16_t* clip;
  float lr, wd, lr_wd, eps;
  int count;
};

template <int MODE, bool DEC, bool CLIP, int RNG>
__global__ void __launch_bounds__(Shape<MODE>::kThreads)
adam_multi_kernel(const MultiArgs ma) {
  const uint32_t b = xcd_tile<Shape<MODE>::kChunk>(blockIdx.x);
  if (b >= ma.tile_start[ma.count]) return;
  const int t = tensor_of_block(b, ma.tile_start, ma.count);
  AdamArgs a;
  a.p = ma.p[t];
  a.g = ma.g[t];
  a.m = ma.m[t];
  a.v = ma.v[t];
  a.aux = ma.aux[t];
  a.rand16 = nullptr;
  a.clip = ma.clip;
  a.n = ma.n[t];
  a.lr = ma.lr;
  a.wd = ma.wd;
  a.lr_wd = ma.lr_wd;
  a.omb1 = ma.omb1[t];
  a.omb2 = ma.omb2[t];
  a.eps = ma.eps;
  a.k0 = ma.k0[t];
  a.k1 = ma.k1[t];
  const uint32_t tile = b - ma.tile_start[t];
  adam_tile<MODE, DEC, CLIP, RNG>(a, tile, b + 1 == ma.tile_start[t + 1]);
}

template <int MODE, bool DEC, bool CLIP, int RNG>
int launch(const AdamArgs& a, bool vec, hipStream_t s) {
  if (vec) {
    constexpr int64_t per_block = tile_elems<MODE>();
    int64_t blocks = (a.n + per_block - 1) / per_block;
    if (blocks > 0x7FFF0000ll) return OA_ERANGE;
    hipLaunchKernelGGL((adam_vec_kernel<MODE, DEC, CLIP, RNG>),
                       dim3(xcd_grid((uint32_t)blocks, Shape<MODE>::kChunk)),
                       dim3(Shape<MODE>::kThreads), 0, s, a, (uint32_t)blocks);
  } else {
    constexpr int T = OA_ADAM_THREADS;
    int64_t blocks = (a.n + T - 1) / T;
    if (blocks > 65536) blocks = 65536;  // grid-stride beyond this
    hipLaunchKernelGGL((adam_scalar_kernel<MODE, DEC, CLIP, RNG>),
                       dim3((unsigned)blocks), dim3(T), 0, s, a);
  }
  return launch_status();
}

template <int MODE, int RNG>
int dispatch_flags(const AdamArgs& a, bool dec, bool vec, hipStream_t s) {
  const bool clip = a.clip != nullptr;
  if (dec) {
    return clip ? launch<MODE, true, true, RNG>(a, vec, s)
                : launch<MODE, true, false, RNG>(a, vec, s);
  }
  return clip ? launch<MODE, false, true, RNG>(a, vec, s)
              : launch<MODE, false, false, RNG>(a, vec, s);
}

// Argument checks shared by the four entry points.  Returns 0, or an OA_E*.
int check_common(const void* p, const void* g, const void* m, const void* v,
                 const void* aux, bool has_aux, size_t aux_align, int64_t n,
                 const void* clip, bool p_may_alias_g, bool p_optional = false) {
  if (n < 0) return OA_EINVAL;
  if (n == 0) return 0;
  if ((!p && !p_optional) || !g || !m || !v || (has_aux && !aux)) return OA_EINVAL;
  if (!aligned_to(p, 2) || !aligned_to(g, 2) || !aligned_to(m, 2) ||
      !aligned_to(v, 2) || (has_aux && !aligned_to(aux, aux_align)) ||
      (clip && !aligned_to(clip, 2)))
    return OA_EALIGN;
  // Buffers that are written must be pairwise distinct, and distinct from grad.
  const void* w[4] = {p, m, v, has_aux ? aux : nullptr};
  for (int i = 0; i < 4; ++i) {
    if (!w[i]) continue;
    for (int j = i + 1; j < 4; ++j)
      if (w[j] && w[i] == w[j]) return OA_EOVERLAP;
    if (w[i] == g && !(i == 0 && p_may_alias_g)) return OA_EOVERLAP;
  }
  return 0;
}

AdamArgs make_args(void* p, const void* g, void* m, void* v, void* aux,
                   int64_t n, float lr, float wd, float b1h, float b2h, float eps,
                   const void* clip) {
  AdamArgs a;
  a.p = static_cast<uint16_t*>(p);
  a.g = static_cast<const uint16_t*>(g);
  a.m = static_cast<uint16_t*>(m);
  a.v = static_cast<uint16_t*>(v);
  a.aux = aux;
  a.rand16 = nullptr;
  a.clip = static_cast<const uint16_t*>(clip);
  a.n = n;
  a.lr = lr;
  a.wd = wd;
  // Scalar sub-expressions of the update, each a single fp32 operation: the
  // same values the kernel would compute per element.
  volatile float lr_wd = lr * wd;
  volatile float omb1 = 1.0f - b1h;
  volatile float omb2 = 1.0f - b2h;
  a.lr_wd = lr_wd;
  a.omb1 = omb1;
  a.omb2 = omb2;
  a.eps = eps;
  a.k0 = a.k1 = 0;
  return a;
}

bool all16(const void* p, const void* g, const void* m, const void* v,
           const void* aux, const void* r) {
  return aligned_to(p, 16) && aligned_to(g, 16) && aligned_to(m, 16) &&
         aligned_to(v, 16) && (!aux || aligned_to(aux, 16)) &&
         (!r || aligned_to(r, 16));
}

}  // namespace
}  // namespace oa

using namespace oa;

extern "C" int oa_adam_fp32_master(void* param_out, const void* grad, void* exp_avg,
                                   void* exp_avg_sq, void* master, int64_t n,
                                   float lr, float weight_decay, float beta1_hat,
                                   float beta2_hat, float eps, int decoupled,
                                   const void* clip_coef, void* stream) {
  int rc = check_common(param_out, grad, exp_avg, exp_avg_sq, master, true, 4, n,
                        clip_coef, /*p_may_alias_g=*/true, /*p_optional=*/true);
  if (rc != 0 || n == 0) return rc;
  AdamArgs a = make_args(param_out, grad, exp_avg, exp_avg_sq, master, n, lr,
                         weight_decay, beta1_hat, beta2_hat, eps, clip_coef);
  const bool vec = all16(param_out, grad, exp_avg, exp_avg_sq, master, nullptr);
  return dispatch_flags<kFp32Master, OA_RNG_TRITON>(a, decoupled != 0, vec,
                                                    static_cast<hipStream_t>(stream));
}

extern "C" int oa_adam_stochastic_rounding(void* param, const void* grad,
                                           void* exp_avg, void* exp_avg_sq,
                                           int64_t n, float lr, float weight_decay,
                                           float beta1_hat, float beta2_hat,
                                           float eps, int decoupled, uint64_t seed,
                                           int rng, const void* rand16,
                                           const void* clip_coef, void* stream) {
  if (rng != OA_RNG_TRITON && rng != OA_RNG_X8 && rng != OA_RNG_BUFFER)
    return OA_EINVAL;
  int rc = check_common(param, grad, exp_avg, exp_avg_sq, nullptr, false, 1, n,
                        clip_coef, false);
  if (rc != 0 || n == 0) return rc;
  if (rng == OA_RNG_BUFFER) {
    if (!rand16) return OA_EINVAL;
    if (!aligned_to(rand16, 2)) return OA_EALIGN;
  }
  AdamArgs a = make_args(param, grad, exp_avg, exp_avg_sq, nullptr, n, lr,
                         weight_decay, beta1_hat, beta2_hat, eps, clip_coef);
  a.k0 = (uint32_t)(seed & 0xFFFFFFFFull);
  a.k1 = (uint32_t)(seed >> 32);
  a.rand16 = static_cast<const uint16_t*>(rand16);
  const bool vec = all16(param, grad, exp_avg, exp_avg_sq, nullptr,
                         rng == OA_RNG_BUFFER ? rand16 : nullptr);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool dec = decoupled != 0;
  if (rng == OA_RNG_TRITON)
    return dispatch_flags<kStochastic, OA_RNG_TRITON>(a, dec, vec, s);
  if (rng == OA_RNG_X8) return dispatch_flags<kStochastic, OA_RNG_X8>(a, dec, vec, s);
  return dispatch_flags<kStochastic, OA_RNG_BUFFER>(a, dec, vec, s);
}

extern "C" int oa_adam_fp31_master(void* param, const void* grad, void* exp_avg,
                                   void* exp_avg_sq, void* rounding_error,
                                   int64_t n, float lr, float weight_decay,
                                   float beta1_hat, float beta2_hat, float eps,
                                   int decoupled, const void* clip_coef,
                                   void* stream) {
  int rc = check_common(param, grad, exp_avg, exp_avg_sq, rounding_error, true, 2,
                        n, clip_coef, false);
  if (rc != 0 || n == 0) return rc;
  AdamArgs a = make_args(param, grad, exp_avg, exp_avg_sq, rounding_error, n, lr,
                         weight_decay, beta1_hat, beta2_hat, eps, clip_coef);
  const bool vec = all16(param, grad, exp_avg, exp_avg_sq, rounding_error, nullptr);
  return dispatch_flags<kFp31, OA_RNG_TRITON>(a, decoupled != 0, vec,
                                              static_cast<hipStream_t>(stream));
}

extern "C" int oa_adam_fp32_master_custom_rounding(
    void* param, const void* grad, void* exp_avg, void* exp_avg_sq,
    void* rounding_error, int64_t n, float lr, float weight_decay, float beta1_hat,
    float beta2_hat, float eps, int decoupled, const void* clip_coef,
    void* stream) {
  int rc = check_common(param, grad, exp_avg, exp_avg_sq, rounding_error, true, 2,
                        n, clip_coef, false);
  if (rc != 0 || n == 0) return rc;
  AdamArgs a = make_args(param, grad, exp_avg, exp_avg_sq, rounding_error, n, lr,
                         weight_decay, beta1_hat, beta2_hat, eps, clip_coef);
  const bool vec = all16(param, grad, exp_avg, exp_avg_sq, rounding_error, nullptr);
  return dispatch_flags<kCustom, OA_RNG_TRITON>(a, decoupled != 0, vec,
                                                static_cast<hipStream_t>(stream));
}

// ------------------------------------------------------------ multi-tensor

namespace oa {
namespace {

template <int MODE, int RNG>
int launch_multi(const MultiArgs& ma, bool dec, unsigned tiles, hipStream_t s) {
  const bool clip = ma.clip != nullptr;
#define OA_LAUNCH_MULTI(D, C)                                                            \
  hipLaunchKernelGGL((adam_multi_kernel<MODE, D, C, RNG>),                               \
                     dim3(xcd_grid(tiles, Shape<MODE>::kChunk)),                         \
                     dim3(Shape<MODE>::kThreads), 0, s, ma)
  if (dec) {
    if (clip) OA_LAUNCH_MULTI(true, true); else OA_LAUNCH_MULTI(true, false);
  } else {
    if (clip) OA_LAUNCH_MULTI(false, true); else OA_LAUNCH_MULTI(false, false);
  }
#undef OA_LAUNCH_MULTI
  return launch_status();
}

int launch_multi_mode(int mode, int rng, const MultiArgs& ma, bool dec, unsigned tiles,
                      hipStream_t s) {
  switch (mode) {
    case OA_MODE_FP32_MASTER:
      return launch_multi<kFp32Master, OA_RNG_TRITON>(ma, dec, tiles, s);
    case OA_MODE_STOCHASTIC_ROUNDING:
      return rng == OA_RNG_X8 ? launch_multi<kStochastic, OA_RNG_X8>(ma, dec, tiles, s)
                              : launch_multi<kStochastic, OA_RNG_TRITON>(ma, dec, tiles, s);
    case OA_MODE_FP31_MASTER:
      return launch_multi<kFp31, OA_RNG_TRITON>(ma, dec, tiles, s);
    default:
      return launch_multi<kCustom, OA_RNG_TRITON>(ma, dec, tiles, s);
  }
}

}  // namespace
}  // namespace oa

extern "C" int oa_adam_multi(int mode, int count, void* const* params,
                             const void* const* grads, void* const* exp_avgs,
                             void* const* exp_avg_sqs, void* const* aux,
                             const int64_t* numels, const float* beta1_hats,
                             const float* beta2_hats, const uint64_t* seeds, float lr,
                             float weight_decay, float eps, int decoupled, int rng,
                             const void* clip_coef, void* stream) {
  if (mode < OA_MODE_FP32_MASTER || mode > OA_MODE_CUSTOM_ROUNDING || count < 0)
    return OA_EINVAL;
  if (count == 0) return 0;
  if (!params || !grads || !exp_avgs || !exp_avg_sqs || !numels || !beta1_hats || !beta2_hats)
    return OA_EINVAL;
  const bool has_aux = mode != OA_MODE_STOCHASTIC_ROUNDING;
  const bool is_sr = mode == OA_MODE_STOCHASTIC_ROUNDING;
  if (has_aux && !aux) return OA_EINVAL;
  if (is_sr && (!seeds || (rng != OA_RNG_TRITON && rng != OA_RNG_X8))) return OA_EINVAL;
  const size_t aux_align = mode == OA_MODE_FP32_MASTER ? 4 : 2;
  // Validate everything before the first launch.
  for (int i = 0; i < count; ++i) {
    int rc = check_common(params[i], grads[i], exp_avgs[i], exp_avg_sqs[i],
                          has_aux ? aux[i] : nullptr, has_aux, aux_align, numels[i],
                          clip_coef, mode == OA_MODE_FP32_MASTER);
    if (rc) return rc;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool dec = decoupled != 0;
  const int64_t kPerTile = mode == OA_MODE_FP32_MASTER ? tile_elems<kFp32Master>()
                                                       : tile_elems<kStochastic>();
  static_assert(tile_elems<kStochastic>() == tile_elems<kFp31>() &&
                tile_elems<kStochastic>() == tile_elems<kCustom>(), "one tile size for these");

  MultiArgs ma;
  ma.clip = static_cast<const uint16_t*>(clip_coef);
  ma.lr = lr;
  ma.wd = weight_decay;
  volatile float lr_wd = lr * weight_decay;
  ma.lr_wd = lr_wd;
  ma.eps = eps;
  ma.count = 0;
  ma.tile_start[0] = 0;
  uint64_t tiles = 0;

  auto flush = [&]() -> int {
    if (ma.count == 0) return 0;
    int rc = launch_multi_mode(mode, rng, ma, dec, (unsigned)tiles, s);
    ma.count = 0;
    tiles = 0;
    return rc;
  };

  for (int i = 0; i < count; ++i) {
    const int64_t n = numels[i];
    if (n == 0) continue;
    void* ax = has_aux ? aux[i] : nullptr;
    if (!all16(params[i], grads[i], exp_avgs[i], exp_avg_sqs[i], ax, nullptr)) {
      // not 16-byte aligned: single-tensor scalar path, in order
      int rc = flush();
      if (rc) return rc;
      AdamArgs a = make_args(params[i], grads[i], exp_avgs[i], exp_avg_sqs[i], ax, n, lr,
                             weight_decay, beta1_hats[i], beta2_hats[i], eps, clip_coef);
      if (is_sr) {
        a.k0 = (uint32_t)(seeds[i] & 0xFFFFFFFFull);
        a.k1 = (uint32_t)(seeds[i] >> 32);
      }
      switch (mode) {
        case OA_MODE_FP32_MASTER:
          rc = dispatch_flags<kFp32Master, OA_RNG_TRITON>(a, dec, false, s); break;
        case OA_MODE_STOCHASTIC_ROUNDING:
          rc = rng == OA_RNG_X8 ? dispatch_flags<kStochastic, OA_RNG_X8>(a, dec, false, s)
                                : dispatch_flags<kStochastic, OA_RNG_TRITON>(a, dec, false, s);
          break;
        case OA_MODE_FP31_MASTER:
          rc = dispatch_flags<kFp31, OA_RNG_TRITON>(a, dec, false, s); break;
        default:
          rc = dispatch_flags<kCustom, OA_RNG_TRITON>(a, dec, false, s); break;
      }
      if (rc) return rc;
      continue;
    }
    int64_t t_tiles = (n + kPerTile - 1) / kPerTile;
    if (t_tiles > 0x7FFF0000ll) return OA_ERANGE;
    if (ma.count == kMultiMax || tiles + (uint64_t)t_tiles > 0x7FFF0000ull) {
      int rc = flush();
      if (rc) return rc;
    }
    const int j = ma.count;
    ma.p[j] = static_cast<uint16_t*>(params[i]);
    ma.g[j] = static_cast<const uint16_t*>(grads[i]);
    ma.m[j] = static_cast<uint16_t*>(exp_avgs[i]);
    ma.v[j] = static_cast<uint16_t*>(exp_avg_sqs[i]);
    ma.aux[j] = ax;
    ma.n[j] = n;
    volatile float o1 = 1.0f - beta1_hats[i];
    volatile float o2 = 1.0f - beta2_hats[i];
    ma.omb1[j] = o1;
    ma.omb2[j] = o2;
    ma.k0[j] = is_sr ? (uint32_t)(seeds[i] & 0xFFFFFFFFull) : 0u;
    ma.k1[j] = is_sr ? (uint32_t)(seeds[i] >> 32) : 0u;
    tiles += (uint64_t)t_tiles;
    ma.tile_start[j + 1] = (uint32_t)tiles;
    ma.count = j + 1;
  }
  return flush();
}
