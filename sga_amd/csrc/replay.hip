// Replay-side kernels: registry score formulas as one pass, and the in-place
// AdamW / AdamS commit with optional dual-lr split and label accumulation.
//
// Commit recipe (the in-place torch chain m.mul_().add_(alpha=),
// v.mul_().addcmul_(), true divisions, sqrt, w.mul_().add_(alpha=)):
//   m' = fma(q, 1-b1, m*b1)
//   v' = fma(round(q*(1-b2)), q, v*b2)        [AdamS: v := (m*m)*b2 first]
//   upd = (m'/bc1) / (sqrt(v'/bc2) + eps)
//   w' = fma(upd, -lr, w*(1-lr*wd))           [split: fma(-(w*wd+upd), step, w)]
//   lab' = fma(round(upd*lr^2), upd, lab)
#include "adam_math.hpp"

namespace sga {

template <int SCORE, bool FULL>
__device__ __forceinline__ void score_vec(const float* __restrict__ w, const float* __restrict__ m,
                                          const float* __restrict__ v, const float* __restrict__ g,
                                          float* __restrict__ out, int64_t i, int64_t n,
                                          const Hyper& h, bool absolute, bool adams, bool no_wd,
                                          bool vec) {
  float ww[4] = {0, 0, 0, 0}, mm[4] = {0, 0, 0, 0}, vv[4] = {0, 0, 0, 0}, gg[4] = {0, 0, 0, 0};
  if (SCORE != SGA_SCORE_ABS_M) ld_f32<FULL>(g, i, n, gg, vec);
  if (SCORE != SGA_SCORE_ABS_G) ld_f32<FULL>(m, i, n, mm, vec);
  if (SCORE == SGA_SCORE_UPDATE || SCORE == SGA_SCORE_COI) {
    ld_f32<FULL>(w, i, n, ww, vec);
    if (!adams) ld_f32<FULL>(v, i, n, vv, vec);
  }
  float o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float ve = adams ? mm[e] * mm[e] : vv[e];
    float s;
    if (SCORE == SGA_SCORE_UPDATE && no_wd) s = adamw_commit(ww[e], gg[e], mm[e], ve, h).u;   // U(g) alone
    else s = score_value<SCORE>(gg[e], ww[e], mm[e], ve, h);
    o[e] = absolute ? fabsf(s) : s;
  }
  st_f32<FULL>(out, i, n, o, vec);
}

template <int SCORE>
__global__ __launch_bounds__(kBlock) void k_score_formula(
    const float* __restrict__ w, const float* __restrict__ m, const float* __restrict__ v,
    const float* __restrict__ g, float* __restrict__ out, int64_t n, Hyper h, bool absolute,
    bool adams, bool no_wd, bool vec) {
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  for (int64_t base = (int64_t)blockIdx.x * kBlock * kVec; base < n; base += stride) {
    const int64_t i = base + (int64_t)threadIdx.x * kVec;
    if (vec && base + kBlock * kVec <= n)
      score_vec<SCORE, true>(w, m, v, g, out, i, n, h, absolute, adams, no_wd, true);
    else if (i < n)
      score_vec<SCORE, false>(w, m, v, g, out, i, n, h, absolute, adams, no_wd, vec);
  }
}

// Branch-point score: the registry formula evaluated in double on fp32
// inputs, |.| rounded once to fp32 (the replay's front select ranks these).
struct BranchK {
  double b1, om1, b2, om2, eps, wd, bc1, bc2;
};

template <int SCORE>
__global__ __launch_bounds__(kBlock) void k_branch_score(
    const float* __restrict__ w, const float* __restrict__ m, const float* __restrict__ v,
    const float* __restrict__ g, float* __restrict__ out, int64_t n, BranchK c, bool adams,
    bool include_wd, bool vec) {
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  for (int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * kVec; i < n; i += stride) {
    float ww[4] = {0, 0, 0, 0}, mm[4] = {0, 0, 0, 0}, vv[4] = {0, 0, 0, 0}, gg[4] = {0, 0, 0, 0};
    if (SCORE != SGA_SCORE_ABS_M) load4_f32(g, i, n, gg, vec);
    if (SCORE != SGA_SCORE_ABS_G) load4_f32(m, i, n, mm, vec);
    if (SCORE == SGA_SCORE_UPDATE || SCORE == SGA_SCORE_COI) {
      load4_f32(w, i, n, ww, vec);
      if (!adams) load4_f32(v, i, n, vv, vec);
    }
    float o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const double gd = gg[e], md = mm[e], wd_ = ww[e];
      const double vd = adams ? md * md : (double)vv[e];
      double r;
      if (SCORE == SGA_SCORE_ABS_G) {
        r = gd;
      } else if (SCORE == SGA_SCORE_ABS_M) {
        r = md;
      } else {
        const double sa = __ddiv_rn(md * c.b1 + gd * c.om1, c.bc1);
        const double sb = __ddiv_rn(vd * c.b2 + (gd * c.om2) * gd, c.bc2);
        const double ug = __ddiv_rn(sa, __dsqrt_rn(sb) + c.eps);
        if (SCORE == SGA_SCORE_UPDATE) {
          r = include_wd ? c.wd * wd_ + ug : ug;
        } else {
          const double u0 = __ddiv_rn(__ddiv_rn(md * c.b1, c.bc1),
                                      __dsqrt_rn(__ddiv_rn(vd * c.b2, c.bc2)) + c.eps);
          r = ug - u0;
        }
      }
      o[e] = (float)fabs(r);
    }
    store4_f32(out, i, n, o, vec);
  }
}

struct StepK {
  float b1, om1, b2, om2, bc1, bc2, eps, omlwd, neglr, lr2, lr, lri, wd;
};

template <bool ADAMS, bool SPLIT, bool LAB, bool FULL>
__device__ __forceinline__ void opt_step_vec(const float* __restrict__ q, float* __restrict__ m,
                                             float* __restrict__ v, float* __restrict__ w,
                                             float* __restrict__ lab,
                                             const uint8_t* __restrict__ inactive, int64_t i,
                                             int64_t n, const StepK& c, bool vec) {
  float qq[4], mm[4], vv[4] = {0, 0, 0, 0}, ww[4], ll[4] = {0, 0, 0, 0};
  uint32_t ina[4] = {0, 0, 0, 0};
  ld_f32<FULL>(q, i, n, qq, vec);
  ld_f32<FULL>(m, i, n, mm, vec);
  if (!ADAMS) ld_f32<FULL>(v, i, n, vv, vec);
  ld_f32<FULL>(w, i, n, ww, vec);
  if (LAB) ld_f32<FULL>(lab, i, n, ll, vec);
  if (SPLIT) ld_u8<FULL>(inactive, i, n, ina, vec);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float vb = ADAMS ? (mm[e] * mm[e]) * c.b2 : vv[e] * c.b2;
    const float vn = __fmaf_rn(qq[e] * c.om2, qq[e], vb);
    const float mn = __fmaf_rn(qq[e], c.om1, mm[e] * c.b1);
    const float mh = __fdiv_rn(mn, c.bc1);
    const float vh = sqrt_rn(__fdiv_rn(vn, c.bc2));
    const float upd = __fdiv_rn(mh, vh + c.eps);
    if (SPLIT) {
      const float step = ina[e] ? c.lri : c.lr;
      const float full = ww[e] * c.wd + upd;
      ww[e] = __fmaf_rn(-full, step, ww[e]);
    } else {
      ww[e] = __fmaf_rn(upd, c.neglr, ww[e] * c.omlwd);
    }
    if (LAB) ll[e] = __fmaf_rn(upd * c.lr2, upd, ll[e]);
    mm[e] = mn;
    vv[e] = vn;
  }
  st_f32<FULL>(m, i, n, mm, vec);
  st_f32<FULL>(v, i, n, vv, vec);
  st_f32<FULL>(w, i, n, ww, vec);
  if (LAB) st_f32<FULL>(lab, i, n, ll, vec);
}

template <bool ADAMS, bool SPLIT, bool LAB>
__global__ __launch_bounds__(kBlock) void k_opt_step(
    const float* __restrict__ q, float* __restrict__ m, float* __restrict__ v,
    float* __restrict__ w, float* __restrict__ lab, const uint8_t* __restrict__ inactive,
    int64_t n, StepK c, bool vec) {
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  for (int64_t base = (int64_t)blockIdx.x * kBlock * kVec; base < n; base += stride) {
    const int64_t i = base + (int64_t)threadIdx.x * kVec;
    if (vec && base + kBlock * kVec <= n)
      opt_step_vec<ADAMS, SPLIT, LAB, true>(q, m, v, w, lab, inactive, i, n, c, true);
    else if (i < n)
      opt_step_vec<ADAMS, SPLIT, LAB, false>(q, m, v, w, lab, inactive, i, n, c, vec);
  }
}

}  // namespace sga

using namespace sga;

extern "C" int sga_score_formula(int score_id, const float* w, const float* m, const float* v,
                                 const float* g, float* out, int64_t n, float beta1, float om1,
                                 float beta2, float om2, float wd, float bc1, float bc2,
                                 float eps, int absolute, int flags, void* stream) {
  const int adams = flags & SGA_SF_ADAMS;
  const bool no_wd = (flags & SGA_SF_NO_WD) != 0;
  if (n == 0) return SGA_OK;
  if (!out || n < 0 || score_id < 0 || score_id > 3) {
    set_error("sga_score_formula: bad argument (score_id=%d)", score_id);
    return SGA_ERR_ARG;
  }
  const bool need_g = score_id != SGA_SCORE_ABS_M, need_m = score_id != SGA_SCORE_ABS_G;
  const bool need_wv = score_id == SGA_SCORE_UPDATE || score_id == SGA_SCORE_COI;
  if ((need_g && !g) || (need_m && !m) || (need_wv && (!w || (!adams && !v)))) {
    set_error("sga_score_formula: missing input tensor for score %d", score_id);
    return SGA_ERR_ARG;
  }
  if (adams) { bc1 = 1.0f; bc2 = 1.0f; }
  const Hyper h = mk_hyper(0.0f, beta1, om1, beta2, om2, eps, wd, bc1, bc2);
  const bool vec = aligned4(w, 4) && aligned4(m, 4) && aligned4(v, 4) && aligned4(g, 4) &&
                   aligned4(out, 4);
  dim3 grid(stream_grid(n, (int64_t)kBlock * kVec, 1 << 22)), block(kBlock);
  hipStream_t st = (hipStream_t)stream;
#define SGA_SF(S) hipLaunchKernelGGL((k_score_formula<S>), grid, block, 0, st, w, m, v, g, out, n, h, absolute != 0, adams != 0, no_wd, vec)
  switch (score_id) {
    case 0: SGA_SF(0); break;
    case 1: SGA_SF(1); break;
    case 2: SGA_SF(2); break;
    default: SGA_SF(3); break;
  }
#undef SGA_SF
  return check_launch("sga_score_formula");
}

extern "C" int sga_branch_score_f64(int score_id, const float* w, const float* m, const float* v,
                                    const float* g, float* out, int64_t n, double beta1,
                                    double beta2, double eps, double wd, double bc1, double bc2,
                                    int adams, int include_wd, void* stream) {
  if (n == 0) return SGA_OK;
  if (!out || n < 0 || score_id < 0 || score_id > 3) {
    set_error("sga_branch_score_f64: bad argument (score_id=%d)", score_id);
    return SGA_ERR_ARG;
  }
  const bool need_g = score_id != SGA_SCORE_ABS_M, need_m = score_id != SGA_SCORE_ABS_G;
  const bool need_wv = score_id == SGA_SCORE_UPDATE || score_id == SGA_SCORE_COI;
  if ((need_g && !g) || (need_m && !m) || (need_wv && (!w || (!adams && !v)))) {
    set_error("sga_branch_score_f64: missing input tensor for score %d", score_id);
    return SGA_ERR_ARG;
  }
  if (adams) { bc1 = 1.0; bc2 = 1.0; }
  const BranchK c{beta1, 1.0 - beta1, beta2, 1.0 - beta2, eps, wd, bc1, bc2};
  const bool vec = aligned4(w, 4) && aligned4(m, 4) && aligned4(v, 4) && aligned4(g, 4) &&
                   aligned4(out, 4);
  dim3 grid(stream_grid(n, (int64_t)kBlock * kVec, 1 << 22)), block(kBlock);
  hipStream_t st = (hipStream_t)stream;
#define SGA_BS(S) hipLaunchKernelGGL((k_branch_score<S>), grid, block, 0, st, w, m, v, g, out, n, c, adams != 0, include_wd != 0, vec)
  switch (score_id) {
    case 0: SGA_BS(0); break;
    case 1: SGA_BS(1); break;
    case 2: SGA_BS(2); break;
    default: SGA_BS(3); break;
  }
#undef SGA_BS
  return check_launch("sga_branch_score_f64");
}

extern "C" int sga_opt_step_inplace(const float* q, float* m, float* v, float* w, float* lab,
                                    const uint8_t* inactive, int64_t n, float beta1, float om1,
                                    float beta2, float om2, float bc1, float bc2, float eps,
                                    float omlwd, float neglr, float lr2, float lr,
                                    float lr_inactive, float wd, int flags, void* stream) {
  if (n == 0) return SGA_OK;
  const bool has_lab = flags & SGA_RP_HAS_LAB, adams = flags & SGA_RP_ADAMS,
             split = flags & SGA_RP_SPLIT;
  if (!q || !m || !v || !w || n < 0 || (has_lab && !lab) || (split && !inactive)) {
    set_error("sga_opt_step_inplace: bad argument");
    return SGA_ERR_ARG;
  }
  StepK c{beta1, om1, beta2, om2, bc1, bc2, eps, omlwd, neglr, lr2, lr, lr_inactive, wd};
  const bool vec = aligned4(q, 4) && aligned4(m, 4) && aligned4(v, 4) && aligned4(w, 4) &&
                   aligned4(lab, 4) && aligned4(inactive, 1);
  dim3 grid(stream_grid(n, (int64_t)kBlock * kVec, 1 << 22)), block(kBlock);
  hipStream_t st = (hipStream_t)stream;
#define SGA_OS(A, S, L) hipLaunchKernelGGL((k_opt_step<A, S, L>), grid, block, 0, st, q, m, v, w, lab, inactive, n, c, vec)
  const int sel = (adams ? 4 : 0) | (split ? 2 : 0) | (has_lab ? 1 : 0);
  switch (sel) {
    case 0: SGA_OS(false, false, false); break;
    case 1: SGA_OS(false, false, true); break;
    case 2: SGA_OS(false, true, false); break;
    case 3: SGA_OS(false, true, true); break;
    case 4: SGA_OS(true, false, false); break;
    case 5: SGA_OS(true, false, true); break;
    case 6: SGA_OS(true, true, false); break;
    default: SGA_OS(true, true, true); break;
  }
#undef SGA_OS
  return check_launch("sga_opt_step_inplace");
}
