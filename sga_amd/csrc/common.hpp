// Shared device/host helpers for the gfx950 (CDNA4, wave64) kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/sga_hip.h"

namespace sga {

constexpr int kWave = 64;
constexpr int kBlock = 256;            // 4 waves per workgroup
constexpr int kVec = 4;                // 128-bit fp32 vectors
constexpr int kChunkIters = 4;         // vectors per lane per chunk
constexpr int kChunk = kWave * kVec * kChunkIters;   // 1024 elements / wave
constexpr int kChunksPerBlock = kBlock / kWave;      // 4
constexpr int kBlockSpan = kChunk * kChunksPerBlock; // 4096 elements / block

// Packed state: four fp32 arrays of one bucket interleaved in records of
// 4 x kPackRun floats ([a0 run | a1 run | a2 run | a3 run], 64 KiB), so the
// four streams of a workgroup always sit in different DRAM banks of one
// physical page.  Element i of array a lives at
// state[(i >> 12) * 16384 + a * 4096 + (i & 4095)]; with the array bases set
// to state + a * 4096 that is base[i + (i >> 12) * 12288].
constexpr int kPackRunLog = 12;
constexpr int64_t kPackRun = 1ll << kPackRunLog;
constexpr int64_t kPackExtra = 3 * kPackRun;
static_assert(kPackRun % kChunk == 0 && kChunk == 1024, "a chunk never straddles two runs");

void set_error(const char* fmt, ...);
int check_launch(const char* what);

// Optional timing observer.  The two symbols below are WEAK references: this library neither
// defines nor exports them.  A benchmark process that wants the dominant kernels bracketed by
// HIP events on their launch stream loads a library that defines them into the global scope
// first; everywhere else the references stay null and a timed launch costs one pointer test.
#ifndef SGA_BENCH_LIBRARY      // (the companion library defines them, strongly)
extern "C" __attribute__((weak)) void* sga_bench_prof_begin(int tag, void* stream);
extern "C" __attribute__((weak)) void sga_bench_prof_end(void* pair, void* stream);
struct ProfPair;
static inline ProfPair* prof_begin(int tag, hipStream_t s) {
  return sga_bench_prof_begin ? reinterpret_cast<ProfPair*>(sga_bench_prof_begin(tag, s)) : nullptr;
}
static inline void prof_end(ProfPair* pp, hipStream_t s) {
  if (pp && sga_bench_prof_end) sga_bench_prof_end(pp, s);
}
#endif
constexpr int SGA_PROF_FUSED_FINAL = 0;   // k_fused_final / k_fused_spec
constexpr int SGA_PROF_SELECT_SWEEP = 1;  // k_bracket_sweep (any key source)
constexpr int SGA_PROF_REPLAY_PASS3 = 2;  // k_replay_pass3
constexpr int SGA_PROF_REPLAY_PASS1 = 3;  // k_replay_pass1 launches of one step

__host__ __device__ static inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Grid for streaming kernels that loop grid-stride: enough workgroups to fill
// 256 CUs several times over, never more than the work needs.
static inline unsigned stream_grid(int64_t n_items, int64_t items_per_block,
                                   int64_t max_blocks = 256 * 16) {
  int64_t b = cdiv64(n_items, items_per_block);
  if (b < 1) b = 1;
  if (b > max_blocks) b = max_blocks;
  return (unsigned)b;
}

// Workgroup ids are dealt round-robin over the 8 XCDs.  For a grid that walks
// library-owned packed records this permutation of [0, nb) hands every XCD one
// contiguous eighth of the range instead (measured: 2.4 % faster on the final
// sweep's stream mix over 64 KiB records, 3 % slower on four flat arrays, so
// only the packed layouts use it).  The tail beyond a multiple of 8 keeps its id.
__device__ __forceinline__ unsigned xcd_contiguous_block(unsigned b, unsigned nb) {
  const unsigned per = nb >> 3;
  return b < (per << 3) ? (b & 7u) * per + (b >> 3) : b;
}

// True when p is aligned for 4-element vector access of `elem` bytes each.
__host__ __device__ static inline bool aligned4(const void* p, int elem) {
  return p == nullptr || (reinterpret_cast<uintptr_t>(p) % (4 * (size_t)elem)) == 0;
}

#ifdef __HIPCC__

__device__ __forceinline__ uint32_t f2u(float x) { return __float_as_uint(x); }
__device__ __forceinline__ float u2f(uint32_t x) { return __uint_as_float(x); }
__device__ __forceinline__ uint32_t abs_key(float x) {
  return __float_as_uint(x) & 0x7FFFFFFFu;
}

// bf16 <-> fp32, round-to-nearest-even, NaN -> quiet NaN (torch's rule).
__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return __uint_as_float(((uint32_t)h) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Offset (in floats) that moves an array's run base to the record holding
// element i of a packed state.  UNIFORM promises that every lane of the wave
// addresses the same run (chunk-structured sweeps), so the offset is formed
// once on the scalar unit.
template <bool UNIFORM>
__device__ __forceinline__ int64_t pack_shift(int64_t i, int64_t pack_extra) {
  if (UNIFORM) {
    const int run = __builtin_amdgcn_readfirstlane((int)(i >> kPackRunLog));
    return (int64_t)run * pack_extra;
  }
  return (i >> kPackRunLog) * pack_extra;
}
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }

// Correctly rounded fp32 square root.  The hardware root is within 1 ulp, so
// the answer is it or one of its neighbours: the exact residuals x - t*s of
// the two neighbours t (one FMA each) say which.  Inputs below 2^-96 are
// scaled by 2^32 first so the residuals stay normal.  (__fsqrt_rn compiles to
// the bare hardware instruction on this toolchain.)
__device__ __forceinline__ float sqrt_rn(float x) {
  const bool small = x < 0x1p-96f;
  const float xs = small ? x * 0x1p+32f : x;
  float s = __builtin_amdgcn_sqrtf(xs);
  const float sd = __uint_as_float(__float_as_uint(s) - 1u);
  const float su = __uint_as_float(__float_as_uint(s) + 1u);
  const float vd = __fmaf_rn(-sd, s, xs);
  const float vu = __fmaf_rn(-su, s, xs);
  s = vd <= 0.0f ? sd : s;
  s = vu > 0.0f ? su : s;
  s = small ? s * 0x1p-16f : s;
  return (xs == 0.0f || xs == __builtin_huge_valf()) ? xs : s;
}

// Values every lane of the wave holds alike, moved to the scalar unit: what is
// derived from them (addresses, hyper-parameters, branches) stays scalar too.
__device__ __forceinline__ int uniform_i32(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ float uniform_f32(float x) {
  return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(x)));
}
__device__ __forceinline__ int64_t uniform_i64(int64_t x) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)x);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)x >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Number of set bits of `mask` strictly below the calling lane.
__device__ __forceinline__ uint32_t lanes_below(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

__device__ __forceinline__ uint64_t ballot64(bool p) { return __ballot(p); }

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// Inclusive scan across the 64 lanes of a wave.
__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v) {
  const int l = lane_id();
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    uint32_t t = __shfl_up(v, o, kWave);
    if (l >= o) v += t;
  }
  return v;
}

struct alignas(16) F4 { float x, y, z, w; };
struct alignas(8) H4 { uint16_t x, y, z, w; };
struct alignas(16) U4 { uint32_t x, y, z, w; };
struct alignas(4) B4 { uint8_t x, y, z, w; };

typedef float f4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ F4 ld4(const float* p) {
  return *reinterpret_cast<const F4*>(p);
}
__device__ __forceinline__ void st4(float* p, const F4& v) {
  *reinterpret_cast<F4*>(p) = v;
}
// Streaming (non-temporal) 128-bit accesses for data touched once per sweep.
__device__ __forceinline__ F4 ld4_nt(const float* p) {
  const f4v t = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(p));
  return F4{t.x, t.y, t.z, t.w};
}
typedef unsigned short h4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ H4 ldh4_nt(const uint16_t* p) {
  const h4v t = __builtin_nontemporal_load(reinterpret_cast<const h4v*>(p));
  return H4{t.x, t.y, t.z, t.w};
}
__device__ __forceinline__ void st4_nt(float* p, const F4& v) {
  f4v t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<f4v*>(p));
}

// Load 4 consecutive elements starting at i (i % 4 == 0 relative to a
// 16-byte aligned base) with a scalar tail when fewer than 4 remain.
__device__ __forceinline__ void load4_f32(const float* base, int64_t i,
                                          int64_t n, float out[4],
                                          bool vec = true) {
  if (vec && i + 4 <= n) {
    F4 v = ld4(base + i);
    out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = (i + e < n) ? base[i + e] : 0.0f;
  }
}
__device__ __forceinline__ void load4_bf16(const uint16_t* base, int64_t i,
                                           int64_t n, float out[4],
                                           bool vec = true) {
  if (vec && i + 4 <= n) {
    H4 v = *reinterpret_cast<const H4*>(base + i);
    out[0] = bf16_to_f32(v.x); out[1] = bf16_to_f32(v.y);
    out[2] = bf16_to_f32(v.z); out[3] = bf16_to_f32(v.w);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      out[e] = (i + e < n) ? bf16_to_f32(base[i + e]) : 0.0f;
  }
}
__device__ __forceinline__ void load4_u8(const uint8_t* base, int64_t i,
                                         int64_t n, uint32_t out[4],
                                         bool vec = true) {
  if (vec && i + 4 <= n) {
    B4 v = *reinterpret_cast<const B4*>(base + i);
    out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = (i + e < n) ? base[i + e] : 0u;
  }
}
__device__ __forceinline__ void store4_f32(float* base, int64_t i, int64_t n,
                                           const float v[4], bool vec = true) {
  if (vec && i + 4 <= n) {
    F4 t{v[0], v[1], v[2], v[3]};
    st4(base + i, t);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (i + e < n) base[i + e] = v[e];
  }
}
__device__ __forceinline__ void store4_u8(uint8_t* base, int64_t i, int64_t n,
                                          const uint32_t v[4], bool vec = true) {
  if (vec && i + 4 <= n) {
    B4 t{(uint8_t)v[0], (uint8_t)v[1], (uint8_t)v[2], (uint8_t)v[3]};
    *reinterpret_cast<B4*>(base + i) = t;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (i + e < n) base[i + e] = (uint8_t)v[e];
  }
}

// FULL variants: when the caller has established (wave-uniformly) that the
// whole span is in range and vector-aligned, the access is a single
// unconditional 64/128-bit instruction -- no per-lane branch, so the compiler
// can keep many loads in flight before the first wait.
template <bool FULL>
__device__ __forceinline__ void ld_f32(const float* base, int64_t i, int64_t n, float out[4], bool vec) {
  if (FULL) {
    const F4 v = ld4_nt(base + i);
    out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
  } else {
    load4_f32(base, i, n, out, vec);
  }
}
template <bool FULL>
__device__ __forceinline__ void ld_bf16(const uint16_t* base, int64_t i, int64_t n, float out[4], bool vec) {
  if (FULL) {
    const H4 v = ldh4_nt(base + i);
    out[0] = bf16_to_f32(v.x); out[1] = bf16_to_f32(v.y);
    out[2] = bf16_to_f32(v.z); out[3] = bf16_to_f32(v.w);
  } else {
    load4_bf16(base, i, n, out, vec);
  }
}
// Loads kept as the raw vectors that arrive from memory: nothing depends on
// them until they are unpacked, so a sweep can issue the loads of several
// slabs before it waits for the first.
template <bool FULL>
__device__ __forceinline__ F4 ldraw_f32(const float* base, int64_t i, int64_t n, bool vec) {
  if (FULL) return ld4_nt(base + i);
  float t[4];
  load4_f32(base, i, n, t, vec);
  return F4{t[0], t[1], t[2], t[3]};
}
__device__ __forceinline__ void unpack_f32(const F4& r, float out[4]) {
  out[0] = r.x; out[1] = r.y; out[2] = r.z; out[3] = r.w;
}
struct RawG { H4 h; F4 f; };      // a gradient quad: bf16 bits (full vector path) or fp32
template <bool BF16G, bool FULL>
__device__ __forceinline__ void fetch_g(const void* g, int64_t i, int64_t n, bool vec, RawG& r) {
  if (BF16G && FULL) {
    r.h = ldh4_nt(reinterpret_cast<const uint16_t*>(g) + i);
  } else if (BF16G) {
    float t[4];
    load4_bf16(reinterpret_cast<const uint16_t*>(g), i, n, t, vec);
    r.f = F4{t[0], t[1], t[2], t[3]};
  } else {
    r.f = ldraw_f32<FULL>(reinterpret_cast<const float*>(g), i, n, vec);
  }
}
template <bool BF16G, bool FULL>
__device__ __forceinline__ void unpack_g(const RawG& r, float out[4]) {
  if (BF16G && FULL) {
    out[0] = bf16_to_f32(r.h.x); out[1] = bf16_to_f32(r.h.y);
    out[2] = bf16_to_f32(r.h.z); out[3] = bf16_to_f32(r.h.w);
  } else {
    unpack_f32(r.f, out);
  }
}
template <bool FULL>
__device__ __forceinline__ void ld_u8(const uint8_t* base, int64_t i, int64_t n, uint32_t out[4], bool vec) {
  if (FULL) {
    const B4 v = *reinterpret_cast<const B4*>(base + i);
    out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
  } else {
    load4_u8(base, i, n, out, vec);
  }
}
template <bool FULL>
__device__ __forceinline__ void st_f32(float* base, int64_t i, int64_t n, const float v[4], bool vec) {
  if (FULL) {
    F4 t{v[0], v[1], v[2], v[3]};
    st4_nt(base + i, t);
  } else {
    store4_f32(base, i, n, v, vec);
  }
}
template <bool FULL>
__device__ __forceinline__ void st_u8(uint8_t* base, int64_t i, int64_t n, const uint32_t v[4], bool vec) {
  if (FULL) {
    B4 t{(uint8_t)v[0], (uint8_t)v[1], (uint8_t)v[2], (uint8_t)v[3]};
    *reinterpret_cast<B4*>(base + i) = t;
  } else {
    store4_u8(base, i, n, v, vec);
  }
}

// Selection masks as bit planes: per 1024-element chunk c and 256-element
// slab `it`, eight words; word 2e + h of the slab holds, for the element e of
// each lane, the lanes [32h, 32h + 32) -- exactly four wave ballots.  Element
// i = c*1024 + it*256 + lane*4 + e is bit (lane & 31) of word
// planes[(i >> 8) * 8 + 2*e + (lane >> 5)].  i must be a multiple of 4.
constexpr int kPlaneWordsPerChunk = 32;
// For a wave whose lane l holds the quad at i = 256 * slab + 4 l (every
// workgroup-structured sweep here): words 2e and 2e + 1 of the slab are the
// 64-bit ballot of element e, so the flags are read back as lane masks with
// no per-lane bit arithmetic at all.
__device__ __forceinline__ void plane_wave_flags4(const uint32_t* __restrict__ planes, int64_t i,
                                                  bool out[4]) {
  const int64_t slab = uniform_i64(i >> 8);
  const uint64_t* w = reinterpret_cast<const uint64_t*>(planes) + slab * 4;
#pragma unroll
  for (int e = 0; e < 4; ++e) out[e] = __builtin_amdgcn_inverse_ballot_w64(w[e]);
}

// Four ballots of a slab -> the lane's word of the chunk's 32 (lane 8*it + 2e + h).
__device__ __forceinline__ void plane_collect(const uint32_t flag[4], int it, uint32_t& word) {
  const uint64_t b0 = ballot64(flag[0] != 0), b1 = ballot64(flag[1] != 0);
  const uint64_t b2 = ballot64(flag[2] != 0), b3 = ballot64(flag[3] != 0);
  const int l = lane_id();
  if ((l >> 3) == it) {
    const uint64_t bb = (l & 4) ? ((l & 2) ? b3 : b2) : ((l & 2) ? b1 : b0);
    word = (l & 1) ? (uint32_t)(bb >> 32) : (uint32_t)bb;
  }
}

#endif  // __HIPCC__

}  // namespace sga
