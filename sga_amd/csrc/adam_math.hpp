// Shared AdamW arithmetic.  Every operation is a separately rounded IEEE fp32
// op (translation units are built with -ffp-contract=off); FMAs appear only
// where written explicitly.
#pragma once
#include "common.hpp"

namespace sga {

struct Hyper {
  float lr, b1, om1, b2, om2, eps, wd, bc1, bc2;
};

struct Commit {
  float m_new, v_new, u, upd;
};

#ifdef __HIPCC__
__device__ __forceinline__ Hyper hyper_of(const sga_segment& s) {
  Hyper h;
  h.lr = s.lr; h.b1 = s.beta1; h.om1 = s.om1; h.b2 = s.beta2; h.om2 = s.om2;
  h.eps = s.eps; h.wd = s.wd; h.bc1 = s.bc1; h.bc2 = s.bc2;
  return h;
}

// Online commit chain (torch elementwise ops, one rounding each):
//   sa = m*b1 + g*(1-b1)          sb = v*b2 + (g*(1-b2))*g
//   m' = sa                        v' = sb
//   u  = (sa/bc1) / (sqrt(sb/bc2) + eps)      upd = wd*p + u
__device__ __forceinline__ Commit adamw_commit(float p, float g, float m, float v,
                                               const Hyper& h) {
  Commit c;
  const float sa = m * h.b1 + g * h.om1;
  const float sb = v * h.b2 + (g * h.om2) * g;
  c.m_new = sa;
  c.v_new = sb;
  const float mh = __fdiv_rn(sa, h.bc1);
  const float vh = __fdiv_rn(sb, h.bc2);
  const float den = sqrt_rn(vh) + h.eps;
  c.u = __fdiv_rn(mh, den);
  c.upd = h.wd * p + c.u;
  return c;
}

// U(0): the direction the same commit would take with a zero gradient.
__device__ __forceinline__ float coi_u0(float m, float v, const Hyper& h) {
  const float num = __fdiv_rn(m * h.b1, h.bc1);
  const float den = sqrt_rn(__fdiv_rn(v * h.b2, h.bc2)) + h.eps;
  return __fdiv_rn(num, den);
}

// Signed registry score.  SCORE: 0 update, 1 g, 2 m, 3 coi (already >= 0).
// The Adam-normalised scores are the commit's own exact chain: every kernel
// that ranks by them gets the same bits, the bits of the IEEE-754 evaluation.
template <int SCORE>
__device__ __forceinline__ float score_value(float q, float p, float m, float v, const Hyper& h) {
  if (SCORE == SGA_SCORE_ABS_G || SCORE == SGA_SCORE_ABS_G_BLIND) return fabsf(q);
  if (SCORE == SGA_SCORE_ABS_M) return fabsf(m);
  // |g + r| / sqrt(v + eps): no counterpart in the reference's registry (a benchmark score)
  if (SCORE == SGA_SCORE_GR_OVER_SQRT_V) return __fdiv_rn(fabsf(q), sqrt_rn(v + h.eps));
  const Commit c = adamw_commit(p, q, m, v, h);
  if (SCORE == SGA_SCORE_UPDATE) return c.upd;
  return fabsf(c.u - coi_u0(m, v, h));
}
template <int SCORE>
__device__ __forceinline__ uint32_t score_key(float q, float p, float m, float v, const Hyper& h) {
  return abs_key(score_value<SCORE>(q, p, m, v, h));
}

// Segment cursor: segments tile [0, n) in ascending order.  `dir` (optional)
// is a directory over blocks of 2^kSegDirLog coordinates: dir[b] = segment
// that holds coordinate b << kSegDirLog, from where a seek walks forward the
// few tensors that start inside the block instead of bisecting the table.
constexpr int kSegDirLog = 16;
constexpr int kSegDirEntries = 1 << (31 - kSegDirLog);     // covers n < 2^31
struct SegCursor {
  const sga_segment* segs;
  const int32_t* dir;
  int n_segs;
  int64_t lo, hi;
  int at;                               // index of the cached segment (uniform seeks only)
  Hyper h;
  __host__ __device__ __forceinline__ void init(const sga_segment* s, int ns,
                                                const int32_t* d = nullptr) {
    segs = s; dir = d; n_segs = ns; lo = 1; hi = 0; at = 0;
  }
  // last segment with start <= i
  __device__ __forceinline__ int find(int64_t i) const {
    if (dir) {
      int a = dir[i >> kSegDirLog];
      while (a + 1 < n_segs && segs[a + 1].start <= i) ++a;
      return a;
    }
    int a = 0, b = n_segs - 1;
    while (a < b) {
      const int mid = (a + b + 1) >> 1;
      if (segs[mid].start <= i) a = mid; else b = mid - 1;
    }
    return a;
  }
  __device__ __forceinline__ void seek(int64_t i) {
    if (i >= lo && i < hi) return;
    const int a = find(i);
    lo = segs[a].start;
    hi = lo + segs[a].n;
    h = hyper_of(segs[a]);
  }
  // The same for an index every lane of the wave holds alike: the cursor and
  // the hyper-parameters it caches live on the scalar unit.
  __device__ __forceinline__ void take_uniform(int a) {
    const sga_segment& s = segs[a];
    at = a;
    lo = uniform_i64(s.start);
    hi = lo + uniform_i64(s.n);
    h.lr = uniform_f32(s.lr); h.b1 = uniform_f32(s.beta1); h.om1 = uniform_f32(s.om1);
    h.b2 = uniform_f32(s.beta2); h.om2 = uniform_f32(s.om2); h.eps = uniform_f32(s.eps);
    h.wd = uniform_f32(s.wd); h.bc1 = uniform_f32(s.bc1); h.bc2 = uniform_f32(s.bc2);
  }
  __device__ __forceinline__ void seek_uniform(int64_t i) {
    if (i >= lo && i < hi) return;
    int a;
    if (dir) {
      a = uniform_i32(dir[i >> kSegDirLog]);
      while (a + 1 < n_segs && uniform_i64(segs[a + 1].start) <= i) ++a;
    } else {
      a = 0;
      int b = n_segs - 1;
      while (a < b) {
        const int mid = (a + b + 1) >> 1;
        if (uniform_i64(segs[mid].start) <= i) a = mid; else b = mid - 1;
      }
    }
    take_uniform(a);
  }
  // Steps to the segment that holds i, a little past the cached one (the
  // next tensor of a slab that straddles a boundary).
  __device__ __forceinline__ void advance_uniform(int64_t i) {
    int a = at;
    while (a + 1 < n_segs && uniform_i64(segs[a + 1].start) <= i) ++a;
    take_uniform(a);
  }
};

// Builds the directory of a segment table: dir[b] = last segment with start <= b << kSegDirLog.
__device__ __forceinline__ void seg_dir_body(const sga_segment* __restrict__ segs, int n_segs,
                                             int64_t n, int32_t* __restrict__ dir) {
  const int64_t nb = (n + (1ll << kSegDirLog) - 1) >> kSegDirLog;
  for (int64_t b = (int64_t)blockIdx.x * kBlock + threadIdx.x; b < nb; b += (int64_t)gridDim.x * kBlock) {
    const int64_t i = b << kSegDirLog;
    int lo = 0, hi = n_segs - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (segs[mid].start <= i) lo = mid; else hi = mid - 1;
    }
    dir[b] = lo;
  }
}
static __global__ __launch_bounds__(kBlock) void k_seg_dir(const sga_segment* __restrict__ segs,
                                                           int n_segs, int64_t n,
                                                           int32_t* __restrict__ dir) {
  seg_dir_body(segs, n_segs, n, dir);
}
// The directories of up to 8 tables in one launch (blockIdx.y = table).
struct SegDirJobs {
  struct { const sga_segment* segs; int32_t* dir; int64_t n; int n_segs; } j[8];
};
static __global__ __launch_bounds__(kBlock) void k_seg_dir_batch(SegDirJobs jobs) {
  const auto& J = jobs.j[blockIdx.y];
  seg_dir_body(J.segs, J.n_segs, J.n, J.dir);
}
static inline void launch_seg_dir(const sga_segment* segs, int n_segs, int64_t n, int32_t* dir,
                                  hipStream_t s) {
  const int64_t nb = (n + (1ll << kSegDirLog) - 1) >> kSegDirLog;
  hipLaunchKernelGGL(k_seg_dir, dim3(stream_grid(nb, kBlock, 128)), dim3(kBlock), 0, s, segs, n_segs, n, dir);
}

// Keys of one slab of a chunk-structured sweep: lane l holds the quad at
// i = s0 + 4 l of the 256-element slab [s0, s0 + 256).  Hyper-parameters
// change only at tensor boundaries, so the slab is scored once per segment
// that intersects it (one, but for the few slabs that hold a boundary) with
// that segment's hyper-parameters as scalar operands.  `sc` was placed on the
// slab's chunk with seek_uniform and is only ever moved by the uniform seeks.
// key[] comes in zeroed; quads past n stay zero.
template <int SCORE, bool FULL>
__device__ __forceinline__ void slab_score_keys(SegCursor& sc, int adams, int64_t i, int64_t n,
                                                const float q[4], const float p[4],
                                                const float m[4], const float v[4],
                                                uint32_t key[4]) {
  const int64_t s0 = uniform_i64(i);
  int64_t s1 = s0 + kWave * kVec;
  if (!FULL && s1 > n) s1 = n;
  if (s0 >= sc.hi) sc.advance_uniform(s0);   // slabs of a chunk ascend from its seek_uniform
  for (;;) {
    Hyper h = sc.h;
    if (adams) { h.bc1 = 1.0f; h.bc2 = 1.0f; }
    uint32_t k4[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) k4[e] = score_key<SCORE>(q[e], p[e], m[e], v[e], h);
    if (sc.lo <= s0 && sc.hi >= s1) {
#pragma unroll
      for (int e = 0; e < 4; ++e) key[e] = k4[e];
      break;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (i + e >= sc.lo && i + e < sc.hi) key[e] = k4[e];
    const int64_t pos = sc.hi;
    if (pos >= s1) break;
    sc.advance_uniform(pos);
    if (sc.hi <= pos) break;              // the table does not tile [0, n): stop
  }
}
#endif

static inline Hyper mk_hyper(float lr, float b1, float om1, float b2, float om2, float eps,
                             float wd, float bc1, float bc2) {
  Hyper h;
  h.lr = lr; h.b1 = b1; h.om1 = om1; h.b2 = b2; h.om2 = om2; h.eps = eps;
  h.wd = wd; h.bc1 = bc1; h.bc2 = bc2;
  return h;
}

}  // namespace sga
