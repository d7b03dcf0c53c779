// Fused offline-replay group step: G configurations (score x ratio x cycle
// length x optimizer x fold x dual-lr) advance over ONE recorded gradient;
// the gradient is read once per pass and shared by all G state sets.
//
//   pass 1  qn2[c]  = sum q_pre^2,  q_pre = gd + res_c (boundary) | gd * sel_c
//           coef[c] = min(1, clip / (sqrt(qn2[c]) + 1e-6))
//   pass 2  (boundary re-selection) score = |formula(w,m,v,(gd+res)*coef)|,
//           exact top-k -> new sel_c                       [select_impl.hpp]
//   pass 3  boundary: q = (gd+res)*coef, res = 0
//           else    : q = (gd*sel)*coef, res += gd*(1-sel)
//           in-place AdamW / AdamS commit (optional dual-lr split)
//
// gd = fp32(g) / coef_dense.  Algorithmic HBM bytes per config-step at G
// configs, bf16 g: non-boundary 34 + 4/G (sel 1 | sel 1 + res 8 + m,v,w 24),
// boundary 36 + 4/G.
#include "adam_math.hpp"
#include "select_impl.hpp"

namespace sga {

constexpr int kMaxCfg = 16;

struct RCfg {
  float* w;
  float* m;
  float* v;
  float* res;
  const uint32_t* sel;      // current mask, bit planes (common.hpp: plane_wave_flags4)
  const uint32_t* out_sel;  // outgoing mask for the dual-lr split (may equal sel)
  double lr_scale;          // dual-lr scale (lr_inactive = lr * lr_scale)
  int boundary;
  int adams;
  int split;
  int packed;
  int res_zero;             // res is known to be all zeros when the step starts
  int pad_;
};

struct RGroup {
  RCfg c[kMaxCfg];
  int G;
  int64_t pack_extra;       // 0, or kPackExtra when every config's w/m/v/res is one packed state
};

template <bool BF16G, bool FULL>
__device__ __forceinline__ void load_gd(const void* g, int64_t i, int64_t n, float inv_is_one,
                                        float coef_dense, float gd[4], bool vec) {
  if (BF16G) ld_bf16<FULL>(reinterpret_cast<const uint16_t*>(g), i, n, gd, vec);
  else ld_f32<FULL>(reinterpret_cast<const float*>(g), i, n, gd, vec);
  if (inv_is_one == 0.0f) {
#pragma unroll
    for (int e = 0; e < 4; ++e) gd[e] = __fdiv_rn(gd[e], coef_dense);
  }
}

// ------------------------------------------------------------------ pass 1
// One launch per step: the gradient is read once for all configurations.
// The configs at a cycle boundary with a live residual (q = gd + res) load
// their residual quads -- their number NB is a template argument so those
// loads are unrolled and in flight together; every other config is a masked
// sum of gd^2 (q = gd * sel, from the mask's bit planes on the scalar unit;
// no mask = every coordinate, which also serves the boundary configs whose
// residual is known to be zero).  Squares are fp32 like the reference's
// (q * q).sum(); a lane adds the four squares of its quad in fp32 and widens
// once per quad into its double accumulator (the reference sums whole chunks
// in fp32), then the usual fixed-order fold.
struct P1Alias {
  int src[kMaxCfg];           // partials slot that holds config c's sums
};

struct P1List {
  const float* res[kMaxCfg];       // boundary list: residual arrays
  int res_slot[kMaxCfg];
  const uint32_t* sel[kMaxCfg];    // masked list: bit planes, or null for "every coordinate"
  int sel_slot[kMaxCfg];
  int n_sel;
};

template <bool BF16G, int NB>
__global__ __launch_bounds__(kBlock) void k_replay_pass1(const void* __restrict__ g, int64_t n,
                                                         float coef_dense, P1List lst,
                                                         double* __restrict__ partials, bool vec,
                                                         int64_t pack_extra) {
  constexpr int NBA = NB > 0 ? NB : 1;
  __shared__ double s_w[kChunksPerBlock][2 * kMaxCfg];
  double accb[NBA], accm[kMaxCfg];
#pragma unroll
  for (int c = 0; c < NBA; ++c) accb[c] = 0.0;
#pragma unroll
  for (int c = 0; c < kMaxCfg; ++c) accm[c] = 0.0;
  const int n_sel = lst.n_sel;
  const float is_one = coef_dense == 1.0f ? 1.0f : 0.0f;
  // chunk-structured: a wave owns 1024-element chunks and has the gradient quads of a chunk's four
  // slabs in flight together (8 bytes per lane and load: one load at a time is bound by latency)
  const int64_t n_chunks = cdiv64(n, kChunk);
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  for (int64_t ch = (int64_t)blockIdx.x * kChunksPerBlock + wave_id(); ch < n_chunks; ch += wstride) {
    const bool full = vec && (ch + 1) * kChunk <= n;
    float gq[kChunkIters][4];
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i = ch * kChunk + it * (kWave * kVec) + lane_id() * kVec;
      gq[it][0] = gq[it][1] = gq[it][2] = gq[it][3] = 0.0f;
      if (full) load_gd<BF16G, true>(g, i, n, is_one, coef_dense, gq[it], true);
      else if (i < n) load_gd<BF16G, false>(g, i, n, is_one, coef_dense, gq[it], vec);
    }
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i = ch * kChunk + it * (kWave * kVec) + lane_id() * kVec;
      const float* gd = gq[it];
      if (NB > 0) {
        float rr[NBA][4];
#pragma unroll
        for (int c = 0; c < NB; ++c) {
          const float* rp = lst.res[c] + pack_shift<true>(ch * kChunk, pack_extra);
          rr[c][0] = rr[c][1] = rr[c][2] = rr[c][3] = 0.0f;
          if (full) ld_f32<true>(rp, i, n, rr[c], true);
          else if (i < n) load4_f32(rp, i, n, rr[c], vec);
        }
#pragma unroll
        for (int c = 0; c < NB; ++c) {
          float part = 0.0f;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float q = gd[e] + rr[c][e];
            part += (full || i + e < n) ? q * q : 0.0f;
          }
          accb[c] += (double)part;
        }
      }
    }
    // q = gd * {0, 1}: q * q is gd * gd or 0, squared once for all configs.  Config by config the
    // chunk's 32 plane words come in as ONE batch of scalar loads (a load per slab would leave the
    // wave waiting on the scalar cache 4 x n_sel times per chunk) and serve directly as lane masks;
    // the lane's 16 squares are added in fp32, in a fixed order, and widened once.
    float gd2[kChunkIters][4];
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i = ch * kChunk + it * (kWave * kVec) + lane_id() * kVec;
#pragma unroll
      for (int e = 0; e < 4; ++e) gd2[it][e] = (full || i + e < n) ? gq[it][e] * gq[it][e] : 0.0f;
    }
#pragma unroll
    for (int c = 0; c < kMaxCfg; ++c) {
      if (c < n_sel) {                            // uniform
        const uint32_t* sp = lst.sel[c];
        float part = 0.0f;
        if (!sp) {                                // no mask: every coordinate counts (q = gd)
#pragma unroll
          for (int it = 0; it < kChunkIters; ++it)
#pragma unroll
            for (int e = 0; e < 4; ++e) part += gd2[it][e];
        } else {
          const uint64_t* w = reinterpret_cast<const uint64_t*>(sp) + uniform_i64(ch) * (kChunkIters * 4);
          uint64_t mk[kChunkIters * 4];
#pragma unroll
          for (int j = 0; j < kChunkIters * 4; ++j) mk[j] = w[j];     // bits past n are zero
#pragma unroll
          for (int it = 0; it < kChunkIters; ++it)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              part += __builtin_amdgcn_inverse_ballot_w64(mk[it * 4 + e]) ? gd2[it][e] : 0.0f;
        }
        accm[c] += (double)part;
      }
    }
  }
#pragma unroll
  for (int c = 0; c < NB; ++c) {
    const double t = wave_sum(accb[c]);
    if (lane_id() == 0) s_w[wave_id()][c] = t;
  }
#pragma unroll
  for (int c = 0; c < kMaxCfg; ++c) {
    if (c < n_sel) {
      const double t = wave_sum(accm[c]);
      if (lane_id() == 0) s_w[wave_id()][kMaxCfg + c] = t;
    }
  }
  __syncthreads();
  const int t = threadIdx.x;
  if (t < NB)
    partials[(int64_t)blockIdx.x * kMaxCfg + lst.res_slot[t]] =
        s_w[0][t] + s_w[1][t] + s_w[2][t] + s_w[3][t];
  if (t >= kMaxCfg && t < kMaxCfg + n_sel) {
    const int c = t - kMaxCfg;
    partials[(int64_t)blockIdx.x * kMaxCfg + lst.sel_slot[c]] =
        s_w[0][t] + s_w[1][t] + s_w[2][t] + s_w[3][t];
  }
}

// One workgroup per config folds the workgroup partials in a fixed order and
// forms the clip coefficient in double (the host formula of the reference).
// (One WAVE per config in a single workgroup took 85 us per step for the 8192
// rows of the table: 128 loads per lane, one after the other.)
__global__ __launch_bounds__(kBlock) void k_replay_coef(const double* __restrict__ partials,
                                                        int n_blocks, int G, double clip,
                                                        double* __restrict__ qn2,
                                                        double* __restrict__ coef_d,
                                                        float* __restrict__ coef_f, P1Alias al) {
  __shared__ double s_w[kChunksPerBlock];
  const int c = blockIdx.x;
  if (c >= G) return;
  const int src = al.src[c];
  double a = 0.0;
  for (int b = threadIdx.x; b < n_blocks; b += kBlock) a += partials[(int64_t)b * kMaxCfg + src];
  a = wave_sum(a);
  if (lane_id() == 0) s_w[wave_id()] = a;
  __syncthreads();
  if (threadIdx.x == 0) {
    a = ((s_w[0] + s_w[1]) + s_w[2]) + s_w[3];
    double coef = 1.0;
    if (clip > 0.0) {
      coef = clip / (sqrt(a) + 1.0e-6);
      if (coef > 1.0) coef = 1.0;
    }
    qn2[c] = a;
    coef_d[c] = coef;
    coef_f[c] = (float)coef;
  }
}

// ------------------------------------------------------------------ pass 3
struct RSeg {          // sga_replay_segment, see the header
  int64_t start, n;
  double lr, wd;
  float b1, om1, b2, om2, eps, bc1, bc2, wdf;
};

struct RSegCursor {
  const RSeg* segs;
  int n_segs;
  int64_t lo, hi;
  RSeg s;
  float omlwd, neglr, lrf;
  __device__ __forceinline__ void init(const RSeg* p, int ns) { segs = p; n_segs = ns; lo = 1; hi = 0; }
  __device__ __forceinline__ void seek(int64_t i) {
    if (i >= lo && i < hi) return;
    int a = 0, b = n_segs - 1;
    while (a < b) {
      const int mid = (a + b + 1) >> 1;
      if (segs[mid].start <= i) a = mid; else b = mid - 1;
    }
    s = segs[a];
    lo = s.start;
    hi = lo + s.n;
    omlwd = (float)(1.0 - s.lr * s.wd);
    neglr = (float)(-s.lr);
    lrf = (float)s.lr;
  }
};

template <bool BF16G, bool FULL>
__device__ __forceinline__ void pass3_vec(const void* g, int64_t i, int64_t n, float is_one,
                                          float coef_dense, const RGroup& grp,
                                          const float* __restrict__ coef_f, RSegCursor& sc,
                                          bool vec) {
  float gd[4];
  load_gd<BF16G, FULL>(g, i, n, is_one, coef_dense, gd, vec);
  const int64_t sh = pack_shift<FULL>(i, grp.pack_extra);
#pragma unroll 1
  for (int c = 0; c < grp.G; ++c) {
    const RCfg& cf = grp.c[c];
    const float coef = coef_f[c];
    float* const RES = cf.res + sh;
    float* const MM = cf.m + sh;
    float* const VV = cf.v + sh;
    float* const WW = cf.w + sh;
    float rr[4], mm[4], vv[4] = {0, 0, 0, 0}, ww[4];
    bool sl[4] = {true, true, true, true}, so[4] = {true, true, true, true};
    if (cf.res_zero) rr[0] = rr[1] = rr[2] = rr[3] = 0.0f;
    else ld_f32<FULL>(RES, i, n, rr, vec);
    ld_f32<FULL>(MM, i, n, mm, vec);
    if (!cf.adams) ld_f32<FULL>(VV, i, n, vv, vec);
    ld_f32<FULL>(WW, i, n, ww, vec);
    if (!cf.boundary) plane_wave_flags4(cf.sel, i, sl);
    if (cf.split) plane_wave_flags4(cf.out_sel, i, so);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (!FULL && i + e >= n) continue;
      sc.seek(i + e);
      float q;
      if (cf.boundary) {
        q = (gd[e] + rr[e]) * coef;
        rr[e] = 0.0f;
      } else {
        const float on = sl[e] ? 1.0f : 0.0f;
        q = (gd[e] * on) * coef;
        rr[e] = rr[e] + gd[e] * (1.0f - on);
      }
      const float bc1 = cf.adams ? 1.0f : sc.s.bc1, bc2 = cf.adams ? 1.0f : sc.s.bc2;
      const float vb = cf.adams ? (mm[e] * mm[e]) * sc.s.b2 : vv[e] * sc.s.b2;
      const float vn = __fmaf_rn(q * sc.s.om2, q, vb);
      const float mn = __fmaf_rn(q, sc.s.om1, mm[e] * sc.s.b1);
      const float mh = __fdiv_rn(mn, bc1);
      const float vh = sqrt_rn(__fdiv_rn(vn, bc2));
      const float upd = __fdiv_rn(mh, vh + sc.s.eps);
      if (cf.split) {
        const float lri = (float)(sc.s.lr * cf.lr_scale);
        const float step = so[e] ? sc.lrf : lri;          // inactive = NOT in the outgoing mask
        const float full_u = ww[e] * sc.s.wdf + upd;
        ww[e] = __fmaf_rn(-full_u, step, ww[e]);
      } else {
        ww[e] = __fmaf_rn(upd, sc.neglr, ww[e] * sc.omlwd);
      }
      mm[e] = mn;
      vv[e] = vn;
    }
    if (!(cf.boundary && cf.res_zero)) st_f32<FULL>(RES, i, n, rr, vec);   // zero stays zero
    st_f32<FULL>(MM, i, n, mm, vec);
    st_f32<FULL>(VV, i, n, vv, vec);
    st_f32<FULL>(WW, i, n, ww, vec);
  }
}

template <bool BF16G>
__global__ __launch_bounds__(kBlock) void k_replay_pass3(const void* __restrict__ g, int64_t n,
                                                         float coef_dense, RGroup grp,
                                                         const float* __restrict__ coef_f,
                                                         const RSeg* __restrict__ segs, int n_segs,
                                                         bool vec) {
  const float is_one = coef_dense == 1.0f ? 1.0f : 0.0f;
  RSegCursor sc;
  sc.init(segs, n_segs);
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  const unsigned blk = grp.pack_extra != 0 ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
  for (int64_t base = (int64_t)blk * kBlock * kVec; base < n; base += stride) {
    const int64_t i = base + (int64_t)threadIdx.x * kVec;
    if (vec && base + kBlock * kVec <= n)
      pass3_vec<BF16G, true>(g, i, n, is_one, coef_dense, grp, coef_f, sc, true);
    else if (i < n)
      pass3_vec<BF16G, false>(g, i, n, is_one, coef_dense, grp, coef_f, sc, vec);
  }
}

// ------------------------------------------------------- dense reference step
// One commit of the recorded (post-clip) gradient on the dense trajectory,
// with the per-coordinate label lab += (lr*upd)^2 and sum(q^2) in double for
// the pre-clip reconstruction (the launcher divides the sum by coef_dense^2).
template <bool BF16G, bool FULL>
__device__ __forceinline__ double dense_vec(const void* g, int64_t i, int64_t n, float* w,
                                            float* m, float* v, float* lab, int adams,
                                            RSegCursor& sc, bool vec) {
  float q[4], mm[4], vv[4] = {0, 0, 0, 0}, ww[4], ll[4] = {0, 0, 0, 0};
  if (BF16G) ld_bf16<FULL>(reinterpret_cast<const uint16_t*>(g), i, n, q, vec);
  else ld_f32<FULL>(reinterpret_cast<const float*>(g), i, n, q, vec);
  ld_f32<FULL>(m, i, n, mm, vec);
  if (!adams) ld_f32<FULL>(v, i, n, vv, vec);
  ld_f32<FULL>(w, i, n, ww, vec);
  if (lab) ld_f32<FULL>(lab, i, n, ll, vec);
  double acc = 0.0;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (!FULL && i + e >= n) continue;
    sc.seek(i + e);
    const float bc1 = adams ? 1.0f : sc.s.bc1, bc2 = adams ? 1.0f : sc.s.bc2;
    const float vb = adams ? (mm[e] * mm[e]) * sc.s.b2 : vv[e] * sc.s.b2;
    const float vn = __fmaf_rn(q[e] * sc.s.om2, q[e], vb);
    const float mn = __fmaf_rn(q[e], sc.s.om1, mm[e] * sc.s.b1);
    const float mh = __fdiv_rn(mn, bc1);
    const float vh = sqrt_rn(__fdiv_rn(vn, bc2));
    const float upd = __fdiv_rn(mh, vh + sc.s.eps);
    ww[e] = __fmaf_rn(upd, sc.neglr, ww[e] * sc.omlwd);
    ll[e] = __fmaf_rn(upd * (float)(sc.s.lr * sc.s.lr), upd, ll[e]);
    mm[e] = mn;
    vv[e] = vn;
    const double qd = (double)q[e];
    acc += qd * qd;                       // exact product; the divisor is applied once, to the sum
  }
  st_f32<FULL>(m, i, n, mm, vec);
  st_f32<FULL>(v, i, n, vv, vec);
  st_f32<FULL>(w, i, n, ww, vec);
  if (lab) st_f32<FULL>(lab, i, n, ll, vec);
  return acc;
}

template <bool BF16G>
__global__ __launch_bounds__(kBlock) void k_dense_step(const void* __restrict__ g, int64_t n,
                                                       float* w, float* m, float* v, float* lab,
                                                       int adams,
                                                       const RSeg* __restrict__ segs, int n_segs,
                                                       double* __restrict__ partials, bool vec) {
  __shared__ double s_w[kChunksPerBlock];
  RSegCursor sc;
  sc.init(segs, n_segs);
  double acc = 0.0;
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  for (int64_t base = (int64_t)blockIdx.x * kBlock * kVec; base < n; base += stride) {
    const int64_t i = base + (int64_t)threadIdx.x * kVec;
    if (vec && base + kBlock * kVec <= n)
      acc += dense_vec<BF16G, true>(g, i, n, w, m, v, lab, adams, sc, true);
    else if (i < n)
      acc += dense_vec<BF16G, false>(g, i, n, w, m, v, lab, adams, sc, vec);
  }
  acc = wave_sum(acc);
  if (lane_id() == 0) s_w[wave_id()] = acc;
  __syncthreads();
  if (threadIdx.x == 0) partials[blockIdx.x] = s_w[0] + s_w[1] + s_w[2] + s_w[3];
}

// --------------------------------------------------- pass 2 score source
// key = |score| of q = (gd + res) * coef against one config's state; the
// residual-blind |g| takes q = gd * coef.  Arrays read: as for the fused step
// (abs_g: g res; abs_m: m; update: g res w m v; coi: g res m v;
// abs_g_blind: g; abs_gr_over_sqrt_v: g res v; AdamS: m in the place of v).
template <bool BF16G, int SCORE>
struct SrcReplay {
  const void* g;
  const float* res;
  const float* w;
  const float* m;
  const float* v;
  const float* coef_f;       // device scalar of this config
  float coef_dense;
  int adams;
  bool vec;
  SegCursor sc;              // b1, b2, eps, wd, bc1, bc2 per tensor (cached per thread)
  int64_t pack_extra;        // 0 or kPackExtra (res/w/m/v of one packed state)
  int res_zero;              // res is known to be all zeros: not read
  // Stepwise interface of the one-sweep select.
  struct Raw { RawG g; F4 r, w, m, v; };
  struct Chunk { int64_t sh; float coef; };
  static constexpr bool kHyper = SCORE == SGA_SCORE_UPDATE || SCORE == SGA_SCORE_COI ||
                                 SCORE == SGA_SCORE_GR_OVER_SQRT_V;
  static constexpr bool kNeedG = SCORE != SGA_SCORE_ABS_M;
  static constexpr bool kNeedR = kNeedG && SCORE != SGA_SCORE_ABS_G_BLIND;
  static constexpr bool kNeedW = SCORE == SGA_SCORE_UPDATE;
  static constexpr bool kNeedV = kHyper;
  __device__ __forceinline__ bool need_r() const { return kNeedR && !res_zero; }
  __device__ __forceinline__ bool need_m() const {
    return SCORE == SGA_SCORE_UPDATE || SCORE == SGA_SCORE_COI || SCORE == SGA_SCORE_ABS_M ||
           (kNeedV && adams);
  }
  // measured: |q| mostly reads the bf16 gradient alone and is bound by latency, four slabs ahead
  // is 25 % faster than one; the Adam-normalised scores fit two slabs in the register budget
  static constexpr int kAhead = kHyper ? 2 : kChunkIters;
  __device__ __forceinline__ Chunk chunk_begin(int64_t c) {
    const int64_t i0 = uniform_i64(c) * kChunk;
    return Chunk{(i0 >> kPackRunLog) * pack_extra, uniform_f32(coef_f[0])};
  }
  __device__ __forceinline__ void chunk_hyper(int64_t c) {
    if (kHyper) sc.seek_uniform(uniform_i64(c) * kChunk);
  }
  template <bool FULL>
  __device__ __forceinline__ void fetch(const Chunk& ck, int64_t i, int64_t n, Raw& t) {
    if (kNeedG) fetch_g<BF16G, FULL>(g, i, n, vec, t.g);
    if (need_r()) t.r = ldraw_f32<FULL>(res + ck.sh, i, n, vec);
    if (need_m()) t.m = ldraw_f32<FULL>(m + ck.sh, i, n, vec);
    if (kNeedW) t.w = ldraw_f32<FULL>(w + ck.sh, i, n, vec);
    if (kNeedV && !adams) t.v = ldraw_f32<FULL>(v + ck.sh, i, n, vec);
  }
  // q of the four coordinates from the raw gradient quad and residual
  __device__ __forceinline__ void form_q(float gd[4], const float rr[4], float coef, float q[4]) const {
    if (coef_dense != 1.0f) {
#pragma unroll
      for (int e = 0; e < 4; ++e) gd[e] = __fdiv_rn(gd[e], coef_dense);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) q[e] = (gd[e] + rr[e]) * coef;
  }
  template <bool FULL>
  __device__ __forceinline__ void keys(const Chunk& ck, int64_t i, int64_t n, const Raw& t,
                                       uint32_t key[4]) {
    float gd[4] = {0, 0, 0, 0}, rr[4] = {0, 0, 0, 0}, q[4] = {0, 0, 0, 0};
    float ww[4] = {0, 0, 0, 0}, mm[4] = {0, 0, 0, 0}, vv[4] = {0, 0, 0, 0};
    if (kNeedG) {
      unpack_g<BF16G, FULL>(t.g, gd);
      if (need_r()) unpack_f32(t.r, rr);
      form_q(gd, rr, ck.coef, q);
    }
    if (need_m()) unpack_f32(t.m, mm);
    if (!kHyper) {
#pragma unroll
      for (int e = 0; e < 4; ++e) key[e] = abs_key(SCORE == SGA_SCORE_ABS_M ? mm[e] : q[e]);
      return;
    }
    if (kNeedW) unpack_f32(t.w, ww);
    if (adams) {
#pragma unroll
      for (int e = 0; e < 4; ++e) vv[e] = mm[e] * mm[e];
    } else {
      unpack_f32(t.v, vv);
    }
    slab_score_keys<SCORE, FULL>(sc, adams, i, n, q, ww, mm, vv, key);
  }
  template <bool FULL = false>
  __device__ __forceinline__ void load(int64_t i, int64_t n, uint32_t key[4]) {
    const int64_t sh = pack_shift<FULL>(i, pack_extra);
    float gd[4] = {0, 0, 0, 0}, rr[4] = {0, 0, 0, 0}, q[4] = {0, 0, 0, 0};
    float ww[4] = {0, 0, 0, 0}, mm[4] = {0, 0, 0, 0}, vv[4] = {0, 0, 0, 0};
    if (kNeedG) {
      if (BF16G) ld_bf16<FULL>(reinterpret_cast<const uint16_t*>(g), i, n, gd, vec);
      else ld_f32<FULL>(reinterpret_cast<const float*>(g), i, n, gd, vec);
      if (need_r()) ld_f32<FULL>(res + sh, i, n, rr, vec);
      form_q(gd, rr, coef_f[0], q);
    }
    if (need_m()) ld_f32<FULL>(m + sh, i, n, mm, vec);
    if (!kHyper) {
#pragma unroll
      for (int e = 0; e < 4; ++e) key[e] = abs_key(SCORE == SGA_SCORE_ABS_M ? mm[e] : q[e]);
      return;
    }
    if (kNeedW) ld_f32<FULL>(w + sh, i, n, ww, vec);
    if (!adams) ld_f32<FULL>(v + sh, i, n, vv, vec);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (FULL || i + e < n) {
        sc.seek(i + e);
        Hyper h = sc.h;
        float ve = vv[e];
        if (adams) { ve = mm[e] * mm[e]; h.bc1 = 1.0f; h.bc2 = 1.0f; }
        key[e] = score_key<SCORE>(q[e], ww[e], mm[e], ve, h);
      } else {
        key[e] = 0u;
      }
    }
  }
};

__global__ __launch_bounds__(kBlock) void k_div_inplace(float* __restrict__ x, int64_t n, float d,
                                                        bool vec, int64_t pack_extra) {
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  for (int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * kVec; i < n; i += stride) {
    float* xs = x + (i >> kPackRunLog) * pack_extra;
    float v[4];
    load4_f32(xs, i, n, v, vec);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = __fdiv_rn(v[e], d);
    store4_f32(xs, i, n, v, vec);
  }
}

// sum (a - b)^2 in double, two-stage
__global__ __launch_bounds__(kBlock) void k_sqdist_stage1(const float* __restrict__ a,
                                                          const float* __restrict__ b, int64_t n,
                                                          double* __restrict__ partials, bool vec,
                                                          int64_t a_pack_extra) {
  __shared__ double s_w[kChunksPerBlock];
  double acc = 0.0;
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  for (int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * kVec; i < n; i += stride) {
    float x[4], y[4];
    load4_f32(a + (i >> kPackRunLog) * a_pack_extra, i, n, x, vec);
    load4_f32(b, i, n, y, vec);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const double d = (double)(x[e] - y[e]);
      acc += d * d;
    }
  }
  acc = wave_sum(acc);
  if (lane_id() == 0) s_w[wave_id()] = acc;
  __syncthreads();
  if (threadIdx.x == 0) partials[blockIdx.x] = s_w[0] + s_w[1] + s_w[2] + s_w[3];
}
// Fold of up to kReplayBlocks * kMaxCfg workgroup partials by one wide workgroup, fixed order:
// lane t adds partials t, t + 1024, ... in turn, then a tree over the lanes.
constexpr int kFoldThreads = 1024;
__global__ __launch_bounds__(kFoldThreads) void k_fold_partials(const double* __restrict__ partials,
                                                                int nb, double divisor,
                                                                double* __restrict__ out) {
  __shared__ double s_p[kFoldThreads];
  double a = 0.0;
  for (int b = threadIdx.x; b < nb; b += kFoldThreads) a += partials[b];
  s_p[threadIdx.x] = a;
  __syncthreads();
  for (int o = kFoldThreads / 2; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) s_p[threadIdx.x] += s_p[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[0] = s_p[0] / divisor;
}
__global__ __launch_bounds__(kWave) void k_sqdist_stage2(const double* __restrict__ partials, int nb,
                                                         double* __restrict__ out) {
  double a = 0.0;
  for (int b = lane_id(); b < nb; b += kWave) a += partials[b];
  a = wave_sum(a);
  if (lane_id() == 0) out[0] = a;
}

static bool fill_group(RGroup* grp, const sga_replay_cfg* cfgs, int G) {
  if (G < 1 || G > kMaxCfg || !cfgs) return false;
  grp->G = G;
  for (int c = 0; c < G; ++c) {
    const sga_replay_cfg& s = cfgs[c];
    if (!s.w || !s.m || !s.v || !s.res || !s.sel) return false;
    RCfg& d = grp->c[c];
    d.w = s.w; d.m = s.m; d.v = s.v; d.res = s.res; d.sel = s.sel;
    d.out_sel = s.out_sel ? s.out_sel : s.sel;
    d.lr_scale = s.lr_scale; d.boundary = s.boundary; d.adams = s.adams; d.split = s.split;
    d.packed = s.packed != 0;
    d.res_zero = s.res_zero != 0;
    d.pad_ = 0;
    if (d.packed != (cfgs[0].packed != 0)) return false;     // one layout per group
  }
  grp->pack_extra = cfgs[0].packed ? kPackExtra : 0;
  for (int c = G; c < kMaxCfg; ++c) grp->c[c] = grp->c[0];
  return true;
}

static bool group_aligned(const RGroup& grp) {
  for (int c = 0; c < grp.G; ++c) {
    const RCfg& d = grp.c[c];
    if (!aligned4(d.w, 4) || !aligned4(d.m, 4) || !aligned4(d.v, 4) || !aligned4(d.res, 4) ||
        !aligned4(d.sel, 1) || !aligned4(d.out_sel, 1))   // 4-byte words
      return false;
  }
  return true;
}

constexpr int kReplayBlocks = 8192;   // grid cap of the reducing sweeps = rows of the partials table

}  // namespace sga

using namespace sga;

static_assert(sizeof(RSeg) == sizeof(sga_replay_segment), "replay segment layout");

template <bool BF16G>
static void launch_pass1(int n_b, unsigned nb, hipStream_t s, const void* g, int64_t n,
                         float coef_dense, const P1List& lst, double* partials, bool vec,
                         int64_t pack_extra) {
#define SGA_P1(NB)                                                                              \
  case NB:                                                                                      \
    hipLaunchKernelGGL((k_replay_pass1<BF16G, NB>), dim3(nb), dim3(kBlock), 0, s, g, n,         \
                       coef_dense, lst, partials, vec, pack_extra);                             \
    break;
  switch (n_b) {
    SGA_P1(0) SGA_P1(1) SGA_P1(2) SGA_P1(3) SGA_P1(4) SGA_P1(5) SGA_P1(6) SGA_P1(7) SGA_P1(8)
    SGA_P1(9) SGA_P1(10) SGA_P1(11) SGA_P1(12) SGA_P1(13) SGA_P1(14) SGA_P1(15) SGA_P1(16)
    default: break;
  }
#undef SGA_P1
}

extern "C" int64_t sga_replay_partials(void) { return (int64_t)kReplayBlocks * kMaxCfg; }

extern "C" int sga_replay_pass1(const void* g, int g_dtype, int64_t n, float coef_dense, double clip,
                                const sga_replay_cfg* cfgs, int G, double* partials, double* qn2,
                                double* coef_d, float* coef_f, void* stream) {
  RGroup grp;
  if (!g || n < 1 || !partials || !qn2 || !coef_d || !coef_f || !fill_group(&grp, cfgs, G) ||
      (g_dtype != SGA_F32 && g_dtype != SGA_BF16)) {
    set_error("sga_replay_pass1: bad argument (1 <= G <= %d, all state pointers set)", kMaxCfg);
    return SGA_ERR_ARG;
  }
  const bool bg = g_dtype == SGA_BF16;
  const bool vec = aligned4(g, bg ? 2 : 4) && group_aligned(grp);
  const unsigned nb = stream_grid(cdiv64(n, kChunk), kChunksPerBlock, kReplayBlocks);
  hipStream_t s = (hipStream_t)stream;
  P1List lst = {};
  P1Alias al;
  int n_b = 0, n_m = 0, plain = -1;
  for (int c = 0; c < G; ++c) {
    al.src[c] = c;
    if (grp.c[c].boundary && grp.c[c].res_zero) {
      // q = gd + 0: one unmasked sum of squares serves every such config
      if (plain < 0) { plain = c; lst.sel[n_m] = nullptr; lst.sel_slot[n_m++] = c; }
      al.src[c] = plain;
    } else if (grp.c[c].boundary) {
      lst.res[n_b] = grp.c[c].res; lst.res_slot[n_b++] = c;
    } else {
      lst.sel[n_m] = grp.c[c].sel; lst.sel_slot[n_m++] = c;
    }
  }
  lst.n_sel = n_m;
  for (int c = G; c < kMaxCfg; ++c) al.src[c] = 0;
  ProfPair* pp = prof_begin(SGA_PROF_REPLAY_PASS1, s);
  if (bg) launch_pass1<true>(n_b, nb, s, g, n, coef_dense, lst, partials, vec, grp.pack_extra);
  else launch_pass1<false>(n_b, nb, s, g, n, coef_dense, lst, partials, vec, grp.pack_extra);
  prof_end(pp, s);
  hipLaunchKernelGGL(k_replay_coef, dim3((unsigned)G), dim3(kBlock), 0, s, partials, (int)nb, G, clip, qn2, coef_d, coef_f, al);
  return check_launch("sga_replay_pass1");
}

extern "C" int sga_replay_pass3(const void* g, int g_dtype, int64_t n, float coef_dense,
                                const sga_replay_cfg* cfgs, int G, const float* coef_f,
                                const sga_replay_segment* segs, int n_segs, void* stream) {
  RGroup grp;
  if (!g || n < 1 || !coef_f || !segs || n_segs < 1 || !fill_group(&grp, cfgs, G) ||
      (g_dtype != SGA_F32 && g_dtype != SGA_BF16)) {
    set_error("sga_replay_pass3: bad argument");
    return SGA_ERR_ARG;
  }
  const bool bg = g_dtype == SGA_BF16;
  const bool vec = aligned4(g, bg ? 2 : 4) && group_aligned(grp);
  const unsigned nb = stream_grid(n, (int64_t)kBlock * kVec, 1 << 22);   // one-shot: nothing to reduce
  hipStream_t s = (hipStream_t)stream;
  const RSeg* rs = reinterpret_cast<const RSeg*>(segs);
  ProfPair* pp = prof_begin(SGA_PROF_REPLAY_PASS3, s);
  if (bg) hipLaunchKernelGGL((k_replay_pass3<true>), dim3(nb), dim3(kBlock), 0, s, g, n, coef_dense, grp, coef_f, rs, n_segs, vec);
  else hipLaunchKernelGGL((k_replay_pass3<false>), dim3(nb), dim3(kBlock), 0, s, g, n, coef_dense, grp, coef_f, rs, n_segs, vec);
  prof_end(pp, s);
  return check_launch("sga_replay_pass3");
}

// One boundary configuration of a (possibly batched) re-selection.
struct ReselJob {
  const float* res;
  const float* w;
  const float* m;
  const float* v;
  int64_t k;
  const float* coef_f;
  int adams, res_zero;
  uint32_t* sel_out;
  sga_select_result* result;
  SelWorkspace ws;
};

// A runtime score id as a compile-time constant for the key source templates.
template <class F>
static void with_score(int score_id, F&& f) {
  switch (score_id) {
    case 0: f(std::integral_constant<int, 0>{}); break;
    case 1: f(std::integral_constant<int, 1>{}); break;
    case 2: f(std::integral_constant<int, 2>{}); break;
    case 3: f(std::integral_constant<int, 3>{}); break;
    case 4: f(std::integral_constant<int, 4>{}); break;
    default: f(std::integral_constant<int, 5>{}); break;
  }
}

// Exact top-k re-selection of up to kMaxJobs configurations over the same recorded gradient: the
// kernels of the select chain that do not form keys run once for all of them, the ones that do
// (sample, score sweeps, radix fallback, ordered plane pass) once per score among them.
// score[b]: score id of job b.  All jobs take the same path (sampled bracket or radix passes).
template <bool BF16G>
static int run_reselect(const void* g, int64_t n, const sga_segment* segs, int n_segs,
                        float coef_dense, int packed, const ReselJob* rj, const int* score,
                        int count, hipStream_t s, const char* who) {
  static_assert(kMaxJobs <= 8, "one directory launch per batch");
  SegDirJobs dj = {};
  SelBatch B;
  bool fast = true, any_hyper = false;
  for (int b = 0; b < count; ++b) {
    const ReselJob& r = rj[b];
    dj.j[b].segs = segs; dj.j[b].dir = r.ws.seg_dir; dj.j[b].n = n; dj.j[b].n_segs = n_segs;
    ChainJob& J = B.add(r.ws, n, r.k, 0);
    J.planes = r.sel_out;
    J.result = r.result;
    fast = fast && SelBatch::fast_ok(r.ws, n);
    any_hyper = any_hyper || score[b] == SGA_SCORE_UPDATE || score[b] == SGA_SCORE_COI ||
                score[b] == SGA_SCORE_GR_OVER_SQRT_V;
  }
  if (any_hyper) {                     // only the Adam-normalised scores ever look a tensor up
    const int64_t nb = (n + (1ll << kSegDirLog) - 1) >> kSegDirLog;
    hipLaunchKernelGGL(k_seg_dir_batch, B.grid(stream_grid(nb, kBlock, 128)), dim3(kBlock), 0, s, dj);
  }
  // the jobs of one score, as a sub-batch over the same workspaces, and their key sources
  auto per_score = [&](auto&& phase) {
    bool seen[SGA_SCORE_GR_OVER_SQRT_V + 1] = {};
    for (int a = 0; a < count; ++a) {
      if (seen[score[a]]) continue;
      seen[score[a]] = true;
      with_score(score[a], [&](auto tag) {
        constexpr int SC = decltype(tag)::value;
        using Src = SrcReplay<BF16G, SC>;
        SrcPack<Src> srcs = {};
        SelBatch sub;
        for (int b = a; b < count; ++b) {
          if (score[b] != score[a]) continue;
          const ReselJob& r = rj[b];
          const bool vec = aligned4(g, BF16G ? 2 : 4) && aligned4(r.res, 4) && aligned4(r.w, 4) &&
                           aligned4(r.m, 4) && aligned4(r.v, 4);
          Src& src = srcs.s[sub.count];
          src = Src{g, r.res, r.w, r.m, r.v, r.coef_f, coef_dense, r.adams, vec, {},
                    packed ? kPackExtra : 0, r.res_zero};
          src.sc.init(segs, n_segs, Src::kHyper ? r.ws.seg_dir : nullptr);
          ChainJob& J = sub.add(r.ws, n, r.k, 0);
          J = B.jobs.j[b];
        }
        phase(srcs, sub);
      });
    }
  };
  chain_begin(B, fast, s);
  if (fast) {
    per_score([&](auto& srcs, const SelBatch& sub) { chain_sample(srcs, sub, s); });
    chain_sample_levels(B, s);
    per_score([&](auto& srcs, const SelBatch& sub) { chain_sweeps(srcs, sub, 1, s); });
    chain_candidates(B, s);
  }
  per_score([&](auto& srcs, const SelBatch& sub) { chain_fallback(srcs, sub, s); });
  launch_tile_scan(B, s);
  if (fast) hipLaunchKernelGGL(k_cand_bits, B.grid(256), dim3(kBlock), 0, s, B.jobs);
  per_score([&](auto& srcs, const SelBatch& sub) {
    using Src = typename std::remove_reference<decltype(srcs.s[0])>::type;
    hipLaunchKernelGGL((k_write_bits<Src>), sub.grid(stream_grid(sub.max_tiles, kChunksPerBlock, 1 << 14)),
                       dim3(kBlock), 0, s, srcs, sub.jobs);
  });
  launch_result(B, s);
  return check_launch(who);
}

extern "C" int sga_replay_reselect_multi(const void* g, int g_dtype, int64_t n,
                                         const sga_segment* segs, int n_segs, float coef_dense,
                                         int packed, const sga_reselect_job* jobs, int n_jobs,
                                         void* stream) {
  const char* who = "sga_replay_reselect_multi";
  if (!g || !segs || !jobs || n < 1 || n >= (1ll << 31) || n_segs < 1 || n_jobs < 1 ||
      (g_dtype != SGA_F32 && g_dtype != SGA_BF16)) {
    set_error("%s: bad argument (n=%lld n_jobs=%d)", who, (long long)n, n_jobs);
    return SGA_ERR_ARG;
  }
  hipStream_t s = (hipStream_t)stream;
  bool done[64] = {};
  if (n_jobs > 64) { set_error("%s: at most 64 jobs per call", who); return SGA_ERR_ARG; }
  for (int a = 0; a < n_jobs; ++a) {
    const sga_reselect_job& u = jobs[a];
    if (!u.res || !u.w || !u.m || !u.v || !u.coef_f || !u.sel_out || u.k < 1 || u.k > n ||
        u.score_id < 0 || u.score_id > SGA_SCORE_GR_OVER_SQRT_V) {
      set_error("%s: job %d: bad argument (k=%lld score=%d)", who, a, (long long)u.k, u.score_id);
      return SGA_ERR_ARG;
    }
  }
  // batches of up to kMaxJobs jobs that take the same path (a workspace too small for the
  // sampled bracket sends its job through the radix passes)
  for (int a = 0; a < n_jobs; ++a) {
    if (done[a]) continue;
    ReselJob rj[kMaxJobs];
    int score[kMaxJobs];
    int cnt = 0;
    bool fast0 = false;
    for (int b = a; b < n_jobs && cnt < kMaxJobs; ++b) {
      if (done[b]) continue;
      const sga_reselect_job& u = jobs[b];
      SelWorkspace sw;
      if (!sel_ws_carve(u.ws, u.ws_bytes, cdiv64(n, kChunk), &sw)) {
        set_error("%s: job %d: workspace too small (sga_select_workspace_bytes(n))", who, b);
        return SGA_ERR_WORKSPACE;
      }
      for (int c = 0; c < cnt; ++c)
        if (rj[c].ws.st == sw.st) {
          set_error("%s: job %d shares its workspace with an earlier job of the call", who, b);
          return SGA_ERR_ARG;
        }
      const bool f = SelBatch::fast_ok(sw, n);
      if (cnt == 0) fast0 = f;
      else if (f != fast0) continue;
      score[cnt] = u.score_id;
      rj[cnt++] = ReselJob{u.res, u.w, u.m, u.v, u.k, u.coef_f, u.adams, u.res_zero, u.sel_out,
                           u.result, sw};
      done[b] = true;
    }
    const int rc = g_dtype == SGA_BF16
        ? run_reselect<true>(g, n, segs, n_segs, coef_dense, packed, rj, score, cnt, s, who)
        : run_reselect<false>(g, n, segs, n_segs, coef_dense, packed, rj, score, cnt, s, who);
    if (rc != SGA_OK) return rc;
  }
  return SGA_OK;
}

extern "C" int sga_replay_reselect(const void* g, int g_dtype, const float* res, const float* w,
                                   const float* m, const float* v, int64_t n, int64_t k,
                                   const sga_segment* segs, int n_segs, int score_id,
                                   const float* coef_f, float coef_dense, int adams, int packed,
                                   int res_zero, uint32_t* sel_out, sga_select_result* result, void* ws,
                                   size_t ws_bytes, void* stream) {
  if (!g || !res || !w || !m || !v || !segs || !coef_f || !sel_out || n < 1 || n >= (1ll << 31) ||
      k < 1 || k > n || n_segs < 1 || score_id < 0 || score_id > SGA_SCORE_GR_OVER_SQRT_V ||
      (g_dtype != SGA_F32 && g_dtype != SGA_BF16)) {
    set_error("sga_replay_reselect: bad argument (n=%lld k=%lld)", (long long)n, (long long)k);
    return SGA_ERR_ARG;
  }
  SelWorkspace sw;
  if (!sel_ws_carve(ws, ws_bytes, cdiv64(n, kChunk), &sw)) {
    set_error("sga_replay_reselect: workspace too small (sga_select_workspace_bytes(n))");
    return SGA_ERR_WORKSPACE;
  }
  const ReselJob rj{res, w, m, v, k, coef_f, adams, res_zero, sel_out, result, sw};
  hipStream_t s = (hipStream_t)stream;
  return g_dtype == SGA_BF16
      ? run_reselect<true>(g, n, segs, n_segs, coef_dense, packed, &rj, &score_id, 1, s, "sga_replay_reselect")
      : run_reselect<false>(g, n, segs, n_segs, coef_dense, packed, &rj, &score_id, 1, s, "sga_replay_reselect");
}

// ------------------------------------------- balanced-histogram re-selection
// The online engine's approximate tier at a replay boundary (replay_fused.py:405-489,
// _histogram.py:115-123, 203-216): histogram of the keys' top 16 bits over a stride-8
// subsample taken on every tensor's own grid (element j of a tensor is sampled when
// j = phase (mod 8), phase = (-p_off) mod 8), crossing bin b = first bin whose running
// count reaches the rank r, selection = every coordinate whose top 16 bits are >= b.
// Two sweeps form the score on the fly; it is never materialised.
namespace sga {

constexpr int kBalBins = 32768;            // (31-bit key) >> 16
constexpr int kBalShift = 16;
constexpr int kBalStride = 8;
constexpr int kBalWide = 1024;             // 16 waves share one 128 KiB LDS table
constexpr int kBalState = 64;              // words behind the bins: [0] b, [1] selected, [2] non-finite

// Walks one chunk through a key source's stepwise interface (loads of kAhead slabs in flight
// before the first key is formed) and hands every slab's keys to f(it, i, key).
template <class Src, bool FULL, class F>
__device__ __forceinline__ void chunk_keys(Src& src, int64_t n, int64_t c, F&& f) {
  constexpr int kAhead = FULL ? Src::kAhead : 1;
  src.chunk_hyper(c);
  const typename Src::Chunk ck = src.chunk_begin(c);
#pragma unroll 1
  for (int g0 = 0; g0 < kChunkIters; g0 += kAhead) {
    typename Src::Raw raw[kAhead];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int64_t i = c * kChunk + (g0 + u) * (kWave * kVec) + lane_id() * kVec;
      if (FULL || i < n) src.template fetch<FULL>(ck, i, n, raw[u]);
    }
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int64_t i = c * kChunk + (g0 + u) * (kWave * kVec) + lane_id() * kVec;
      uint32_t key[4] = {0u, 0u, 0u, 0u};
      if (FULL || i < n) src.template keys<FULL>(ck, i, n, raw[u], key);
      f(g0 + u, i, key);
    }
  }
}

static __global__ __launch_bounds__(kBlock) void k_bal_zero(uint32_t* __restrict__ hist) {
  for (int i = blockIdx.x * kBlock + threadIdx.x; i < kBalBins + kBalState; i += gridDim.x * kBlock)
    hist[i] = 0u;
}

template <class Src>
__global__ __launch_bounds__(kBalWide) void k_bal_hist(Src src, int64_t n,
                                                       const sga_segment* __restrict__ segs,
                                                       int n_segs, const int32_t* __restrict__ seg_dir,
                                                       const int32_t* __restrict__ seg_phase,
                                                       uint32_t* __restrict__ hist) {
  extern __shared__ uint32_t s_bal[];
  for (int b = threadIdx.x; b < kBalBins; b += kBalWide) s_bal[b] = 0u;
  __syncthreads();
  SegCursor pc;                              // per lane: which tensor a coordinate lies in
  pc.init(segs, n_segs, seg_dir);
  int64_t lo = 1, hi = 0;
  int ph = 0;
  const int64_t n_chunks = cdiv64(n, kChunk);
  const int64_t wstride = (int64_t)gridDim.x * (kBalWide / kWave);
  for (int64_t c = (int64_t)blockIdx.x * (kBalWide / kWave) + wave_id(); c < n_chunks; c += wstride) {
    auto slab = [&](int, int64_t i, const uint32_t key[4]) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int64_t idx = i + e;
        const bool valid = idx < n;
        if (valid && (idx < lo || idx >= hi)) {
          const int a = pc.find(idx);
          lo = segs[a].start;
          hi = lo + segs[a].n;
          ph = seg_phase ? seg_phase[a] : 0;
        }
        const bool sampled = valid && idx >= lo && idx < hi &&
                             (((idx - lo - (int64_t)ph) & (kBalStride - 1)) == 0);
        lds_hist_add(s_bal, key[e] >> kBalShift, sampled);
      }
    };
    if (src.vec && (c + 1) * kChunk <= n) chunk_keys<Src, true>(src, n, c, slab);
    else chunk_keys<Src, false>(src, n, c, slab);
  }
  __syncthreads();
  for (int b = threadIdx.x; b < kBalBins; b += kBalWide) {
    const uint32_t cnt = s_bal[b];
    if (cnt) atomicAdd(&hist[b], cnt);
  }
}

// b = number of bins whose inclusive running count stays below the rank
// (torch.searchsorted(cumsum(hist), r), left): one workgroup, 32 bins per lane.
static __global__ __launch_bounds__(kBalWide) void k_bal_bin(uint32_t* __restrict__ hist, uint64_t rank) {
  __shared__ uint64_t s_sum[kBalWide];
  __shared__ uint32_t s_below[kBalWide];
  constexpr int PER = kBalBins / kBalWide;
  uint32_t loc[PER];
  uint64_t mine = 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) { loc[j] = hist[threadIdx.x * PER + j]; mine += loc[j]; }
  s_sum[threadIdx.x] = mine;
  __syncthreads();
  for (int o = 1; o < kBalWide; o <<= 1) {                 // inclusive scan over the lanes
    const uint64_t add = (int)threadIdx.x >= o ? s_sum[threadIdx.x - o] : 0ull;
    __syncthreads();
    s_sum[threadIdx.x] += add;
    __syncthreads();
  }
  uint64_t run = s_sum[threadIdx.x] - mine;
  uint32_t below = 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) { run += loc[j]; below += run < rank; }
  s_below[threadIdx.x] = below;
  __syncthreads();
  for (int o = kBalWide / 2; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) s_below[threadIdx.x] += s_below[threadIdx.x + o];
    __syncthreads();
  }
  // a rank beyond the sample's size: every bin stays below it, and searchsorted on the
  // reference's table of 32769 bins (the last one is never hit by a 31-bit key) returns 32769
  if (threadIdx.x == 0) hist[kBalBins] = s_below[0] < (uint32_t)kBalBins ? s_below[0] : kBalBins + 1u;
}

template <class Src>
__global__ __launch_bounds__(kBlock) void k_bal_planes(Src src, int64_t n, uint32_t* __restrict__ hist,
                                                       uint32_t* __restrict__ planes) {
  __shared__ uint32_t s_planes[kChunksPerBlock][kPlaneWordsPerChunk];
  const uint32_t b = hist[kBalBins];
  const int64_t n_chunks = cdiv64(n, kChunk);
  const int64_t c = (int64_t)blockIdx.x * kChunksPerBlock + wave_id();
  if (c >= n_chunks) return;
  uint32_t n_sel = 0, n_nf = 0;
  uint32_t* const lp = s_planes[wave_id()];
  auto slab = [&](int it, int64_t i, const uint32_t key[4]) {
    Ballot4 on;
    uint64_t nf = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint64_t valid = ballot64(i + e < n);
      on.m[e] = ballot64((key[e] >> kBalShift) >= b) & valid;
      nf |= ballot64(key[e] >= 0x7F800000u) & valid;
    }
    n_sel += on.count();
    if (nf) {
#pragma unroll
      for (int e = 0; e < 4; ++e) n_nf += (uint32_t)__popcll(ballot64(key[e] >= 0x7F800000u && i + e < n));
    }
    plane_put(on, it, lp);
  };
  if (src.vec && (c + 1) * kChunk <= n) chunk_keys<Src, true>(src, n, c, slab);
  else chunk_keys<Src, false>(src, n, c, slab);
  __builtin_amdgcn_wave_barrier();
  if (lane_id() < kPlaneWordsPerChunk) planes[c * kPlaneWordsPerChunk + lane_id()] = lp[lane_id()];
  if (lane_id() == 0) {
    if (n_sel) atomicAdd(&hist[kBalBins + 1], n_sel);
    if (n_nf) atomicAdd(&hist[kBalBins + 2], n_nf);
  }
}

static __global__ void k_bal_result(const uint32_t* __restrict__ hist, sga_select_result* __restrict__ out) {
  const uint32_t b = hist[kBalBins];
  out->thresh_bits = (b << kBalShift) & 0x7FFFFFFFu;      // the bin's lower edge (_bin_edge_float)
  out->need = 0u;
  out->n_gt = hist[kBalBins + 1];
  out->n_eq = 0u;
  out->n_selected = hist[kBalBins + 1];
  out->nonfinite = hist[kBalBins + 2];
  out->status = 0u;
  out->path = 3u;
}

template <bool BF16G, int SCORE>
static int run_reselect_balanced(const void* g, const float* res, const float* w, const float* m,
                                 const float* v, int64_t n, uint64_t rank, const sga_segment* segs,
                                 int n_segs, const int32_t* seg_phase, const float* coef_f,
                                 float coef_dense, int adams, int packed, int res_zero,
                                 uint32_t* sel_out, sga_select_result* result, uint32_t* hist,
                                 const SelWorkspace& ws, hipStream_t s) {
  const bool vec = aligned4(g, BF16G ? 2 : 4) && aligned4(res, 4) && aligned4(w, 4) &&
                   aligned4(m, 4) && aligned4(v, 4);
  SrcReplay<BF16G, SCORE> src{g, res, w, m, v, coef_f, coef_dense, adams, vec, {},
                              packed ? kPackExtra : 0, res_zero};
  launch_seg_dir(segs, n_segs, n, ws.seg_dir, s);
  src.sc.init(segs, n_segs, ws.seg_dir);
  const int64_t n_chunks = cdiv64(n, kChunk);
  hipLaunchKernelGGL(k_bal_zero, dim3(32), dim3(kBlock), 0, s, hist);
  hipLaunchKernelGGL((k_bal_hist<SrcReplay<BF16G, SCORE>>),
                     dim3(stream_grid(n_chunks, kBalWide / kWave, 256)), dim3(kBalWide),
                     (size_t)kBalBins * 4, s, src, n, segs, n_segs, ws.seg_dir, seg_phase, hist);
  hipLaunchKernelGGL(k_bal_bin, dim3(1), dim3(kBalWide), 0, s, hist, rank);
  hipLaunchKernelGGL((k_bal_planes<SrcReplay<BF16G, SCORE>>), dim3((unsigned)cdiv64(n_chunks, kChunksPerBlock)),
                     dim3(kBlock), 0, s, src, n, hist, sel_out);
  if (result) hipLaunchKernelGGL(k_bal_result, dim3(1), dim3(1), 0, s, hist, result);
  return check_launch("sga_replay_reselect_balanced");
}

}  // namespace sga

extern "C" int64_t sga_balanced_hist_words(void) { return kBalBins + kBalState; }

extern "C" int sga_replay_reselect_balanced(const void* g, int g_dtype, const float* res,
                                            const float* w, const float* m, const float* v,
                                            int64_t n, int64_t rank, const sga_segment* segs,
                                            int n_segs, const int32_t* seg_phase, int score_id,
                                            const float* coef_f, float coef_dense, int adams,
                                            int packed, int res_zero, uint32_t* sel_out,
                                            sga_select_result* result, uint32_t* hist, void* ws,
                                            size_t ws_bytes, void* stream) {
  if (!g || !res || !w || !m || !v || !segs || !coef_f || !sel_out || !hist || n < 1 ||
      n >= (1ll << 31) || rank < 1 || n_segs < 1 || score_id < 0 ||
      score_id > SGA_SCORE_GR_OVER_SQRT_V || (g_dtype != SGA_F32 && g_dtype != SGA_BF16)) {
    set_error("sga_replay_reselect_balanced: bad argument (n=%lld rank=%lld)", (long long)n,
              (long long)rank);
    return SGA_ERR_ARG;
  }
  SelWorkspace sw;
  if (!sel_ws_carve(ws, ws_bytes, cdiv64(n, kChunk), &sw)) {
    set_error("sga_replay_reselect_balanced: workspace too small (sga_select_workspace_bytes(n))");
    return SGA_ERR_WORKSPACE;
  }
  hipStream_t s = (hipStream_t)stream;
#define SGA_RB(BG, SC) return run_reselect_balanced<BG, SC>(g, res, w, m, v, n, (uint64_t)rank, segs, n_segs, seg_phase, coef_f, coef_dense, adams, packed, res_zero, sel_out, result, hist, sw, s)
  if (g_dtype == SGA_BF16) {
    switch (score_id) { case 0: SGA_RB(true, 0); case 1: SGA_RB(true, 1); case 2: SGA_RB(true, 2);
                        case 3: SGA_RB(true, 3); case 4: SGA_RB(true, 4); default: SGA_RB(true, 5); }
  } else {
    switch (score_id) { case 0: SGA_RB(false, 0); case 1: SGA_RB(false, 1); case 2: SGA_RB(false, 2);
                        case 3: SGA_RB(false, 3); case 4: SGA_RB(false, 4); default: SGA_RB(false, 5); }
  }
#undef SGA_RB
}

extern "C" int sga_dense_replay_step(const void* g, int g_dtype, float* w, float* m, float* v,
                                     float* lab, int64_t n, const sga_replay_segment* segs,
                                     int n_segs, int adams, double coef_dense, double* partials,
                                     double* recon2, void* stream) {
  if (!g || !w || !m || !v || !segs || !partials || !recon2 || n < 1 || n_segs < 1 ||
      !(coef_dense > 0.0) || (g_dtype != SGA_F32 && g_dtype != SGA_BF16)) {
    set_error("sga_dense_replay_step: bad argument");
    return SGA_ERR_ARG;
  }
  const bool bg = g_dtype == SGA_BF16;
  const bool vec = aligned4(g, bg ? 2 : 4) && aligned4(w, 4) && aligned4(m, 4) && aligned4(v, 4) &&
                   aligned4(lab, 4);
  // as close to one 1024-element slab per workgroup as the partials workspace allows (a capped
  // grid-stride loop leaves a quarter of the bandwidth unused); the fold stays in a fixed order
  const unsigned nb = stream_grid(n, (int64_t)kBlock * kVec, kReplayBlocks * kMaxCfg);
  hipStream_t s = (hipStream_t)stream;
  const RSeg* rs = reinterpret_cast<const RSeg*>(segs);
  if (bg) hipLaunchKernelGGL((k_dense_step<true>), dim3(nb), dim3(kBlock), 0, s, g, n, w, m, v, lab, adams, rs, n_segs, partials, vec);
  else hipLaunchKernelGGL((k_dense_step<false>), dim3(nb), dim3(kBlock), 0, s, g, n, w, m, v, lab, adams, rs, n_segs, partials, vec);
  hipLaunchKernelGGL(k_fold_partials, dim3(1), dim3(kFoldThreads), 0, s, partials, (int)nb,
                     coef_dense * coef_dense, recon2);
  return check_launch("sga_dense_replay_step");
}

extern "C" int64_t sga_plane_words(int64_t n) {
  return n <= 0 ? 0 : cdiv64(n, kChunk) * kPlaneWordsPerChunk;
}

extern "C" int sga_mask_to_planes(const uint8_t* mask, int64_t n, uint32_t* planes, void* stream) {
  if (n == 0) return SGA_OK;
  if (!mask || !planes || n < 0) { set_error("sga_mask_to_planes: bad argument"); return SGA_ERR_ARG; }
  hipLaunchKernelGGL(k_mask_to_planes, dim3(stream_grid(cdiv64(n, kChunk), kChunksPerBlock, 1 << 22)),
                     dim3(kBlock), 0, (hipStream_t)stream, mask, n, planes, aligned4(mask, 1));
  return check_launch("sga_mask_to_planes");
}

extern "C" int sga_planes_to_mask(const uint32_t* planes, int64_t n, uint8_t* mask, void* stream) {
  if (n == 0) return SGA_OK;
  if (!mask || !planes || n < 0) { set_error("sga_planes_to_mask: bad argument"); return SGA_ERR_ARG; }
  hipLaunchKernelGGL(k_expand_mask, dim3(stream_grid(cdiv64(n, kChunk), kChunksPerBlock, 1 << 22)),
                     dim3(kBlock), 0, (hipStream_t)stream, (const SelState*)nullptr, planes, n, mask,
                     (reinterpret_cast<uintptr_t>(mask) & 15) == 0);
  return check_launch("sga_planes_to_mask");
}

extern "C" int sga_div_inplace(float* x, int64_t n, float d, int packed, void* stream) {
  if (n == 0) return SGA_OK;
  if (!x || n < 0) { set_error("sga_div_inplace: bad argument"); return SGA_ERR_ARG; }
  hipLaunchKernelGGL(k_div_inplace, dim3(stream_grid(n, (int64_t)kBlock * kVec, 1 << 22)), dim3(kBlock), 0,
                     (hipStream_t)stream, x, n, d, aligned4(x, 4), packed ? kPackExtra : 0);
  return check_launch("sga_div_inplace");
}

extern "C" int sga_sq_dist(const float* a, int a_packed, const float* b, int64_t n, double* partials,
                           double* out, void* stream) {
  if (!a || !b || !partials || !out || n < 1) { set_error("sga_sq_dist: bad argument"); return SGA_ERR_ARG; }
  const unsigned nb = stream_grid(n, (int64_t)kBlock * kVec, 1024);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(k_sqdist_stage1, dim3(nb), dim3(kBlock), 0, s, a, b, n, partials,
                     aligned4(a, 4) && aligned4(b, 4), a_packed ? kPackExtra : 0);
  hipLaunchKernelGGL(k_sqdist_stage2, dim3(1), dim3(kWave), 0, s, partials, (int)nb, out);
  return check_launch("sga_sq_dist");
}
