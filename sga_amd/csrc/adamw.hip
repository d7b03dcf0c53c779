// Residual-aware AdamW commit: masked / full-step / compact (merge-join) forms.
//
// Arithmetic recipe: every multiply, add, divide and square root below is a
// separately rounded IEEE fp32 operation (the translation unit is compiled
// with -ffp-contract=off), in the order of the torch elementwise chain
//     sa = m*b1 + g*(1-b1)            sb = v*b2 + (g*(1-b2))*g
//     m' = sa                          v' = sb
//     upd = wd*p + (sa/bc1) / (sqrt(sb/bc2) + eps)
//     p'  = p - lr*upd
// so m'/v' are bit-identical to a correctly rounded host evaluation and p'
// differs only where the host library's sqrt is not correctly rounded.
#include "adam_math.hpp"

namespace sga {

// One 4-element vector of the masked / full-step commit.
// EMIT: -1 sparse step; 0 update, 1 |g|, 2 |m|, 3 coi -> written into g.
// FULL: the whole workgroup span is in range and every array vector-aligned,
// so all loads are unconditional and in flight together.
template <int EMIT, bool FULL>
__device__ __forceinline__ void gc_vec(float* __restrict__ p, float* __restrict__ g,
                                       float* __restrict__ m, float* __restrict__ v,
                                       const uint8_t* __restrict__ mask, int64_t i, int64_t n,
                                       const Hyper& h, float coeff, float interval,
                                       float lr_inactive, int flags, bool vec) {
  const bool has_mask = flags & SGA_GC_HAS_MASK;
  const bool apply_coeff = flags & SGA_GC_APPLY_COEFF;
  const bool clear = flags & SGA_GC_CLEAR;
  const bool fold = flags & SGA_GC_FOLD;
  const bool split = flags & SGA_GC_LR_SPLIT;
  const bool adams = flags & SGA_GC_ADAMS;   // v basis = pre-commit m*m, h.bc1 = h.bc2 = 1
  float pp[4], gg[4], mm[4], vv[4];
  uint32_t mk[4] = {1, 1, 1, 1};
  ld_f32<FULL>(p, i, n, pp, vec);
  ld_f32<FULL>(g, i, n, gg, vec);
  ld_f32<FULL>(m, i, n, mm, vec);
  if (!adams) ld_f32<FULL>(v, i, n, vv, vec);
  if (has_mask) ld_u8<FULL>(mask, i, n, mk, vec);
  if (adams) {
#pragma unroll
    for (int e = 0; e < 4; ++e) vv[e] = mm[e] * mm[e];
  }
  float gout[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const bool active = mk[e] != 0;
    const float raw = gg[e];
    float ge = raw;
    if (EMIT < 0 && has_mask && !active) ge = 0.0f;
    if (apply_coeff && active) ge = ge * coeff;
    const Commit c = adamw_commit(pp[e], ge, mm[e], vv[e], h);
    if (EMIT == 0) gout[e] = c.upd;
    else if (EMIT == 1) gout[e] = fabsf(ge);
    else if (EMIT == 2) gout[e] = fabsf(mm[e]);
    else if (EMIT == 3) gout[e] = fabsf(c.u - coi_u0(mm[e], vv[e], h));
    else {
      float t = (clear && active) ? 0.0f : raw;
      if (fold) t = __fdiv_rn(t, interval);
      gout[e] = t;
    }
    const float lr_a = (split && !active) ? lr_inactive : h.lr;
    pp[e] = pp[e] - lr_a * c.upd;
    mm[e] = c.m_new;
    vv[e] = c.v_new;
  }
  st_f32<FULL>(m, i, n, mm, vec);
  st_f32<FULL>(v, i, n, vv, vec);
  if (EMIT >= 0 || clear || fold) st_f32<FULL>(g, i, n, gout, vec);
  st_f32<FULL>(p, i, n, pp, vec);
}

template <int EMIT>
__global__ __launch_bounds__(kBlock) void k_grad_correct(
    float* __restrict__ p, float* __restrict__ g, float* __restrict__ m,
    float* __restrict__ v, const uint8_t* __restrict__ mask, int64_t n, Hyper h,
    float coeff, float interval, float lr_inactive, int flags, bool vec) {
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  for (int64_t base = (int64_t)blockIdx.x * kBlock * kVec; base < n; base += stride) {
    const int64_t i = base + (int64_t)threadIdx.x * kVec;
    if (vec && base + kBlock * kVec <= n)
      gc_vec<EMIT, true>(p, g, m, v, mask, i, n, h, coeff, interval, lr_inactive, flags, true);
    else if (i < n)
      gc_vec<EMIT, false>(p, g, m, v, mask, i, n, h, coeff, interval, lr_inactive, flags, vec);
  }
}

// The same commit over MANY records (one per parameter tensor) in one launch:
// a workgroup owns one kBlockSpan-element span of one record, found by a
// search over the records' first-span indices.
struct GcRecord {           // sga_gc_record, see the header
  float* p; float* g; float* m; float* v;
  const uint8_t* mask;
  int64_t n, first_span;
  float lr, b1, om1, b2, om2, eps, wd, bc1, bc2, lr_inactive;
  int flags, pad_;
};

template <int EMIT>
__global__ __launch_bounds__(kBlock) void k_grad_correct_multi(const GcRecord* __restrict__ recs,
                                                               int n_recs, float coeff,
                                                               float interval) {
  const int64_t span = blockIdx.x;
  int a = 0, b = n_recs - 1;
  while (a < b) {                       // last record whose first span is <= this one
    const int mid = (a + b + 1) >> 1;
    if (recs[mid].first_span <= span) a = mid; else b = mid - 1;
  }
  const GcRecord r = recs[a];
  Hyper h;
  h.lr = r.lr; h.b1 = r.b1; h.om1 = r.om1; h.b2 = r.b2; h.om2 = r.om2; h.eps = r.eps;
  h.wd = r.wd; h.bc1 = r.bc1; h.bc2 = r.bc2;
  const bool vec = aligned4(r.p, 4) && aligned4(r.g, 4) && aligned4(r.m, 4) && aligned4(r.v, 4) &&
                   aligned4(r.mask, 1);
  const int64_t base = (span - r.first_span) * kBlockSpan;
  const bool full = vec && base + kBlockSpan <= r.n;
#pragma unroll
  for (int it = 0; it < kBlockSpan / (kBlock * kVec); ++it) {
    const int64_t i = base + ((int64_t)it * kBlock + threadIdx.x) * kVec;
    if (full)
      gc_vec<EMIT, true>(r.p, r.g, r.m, r.v, r.mask, i, r.n, h, coeff, interval, r.lr_inactive,
                         r.flags, true);
    else if (i < r.n)
      gc_vec<EMIT, false>(r.p, r.g, r.m, r.v, r.mask, i, r.n, h, coeff, interval, r.lr_inactive,
                          r.flags, vec);
  }
}

// ---------------------------------------------------------------- compact
// A workgroup owns kBlockSpan consecutive coordinates of the record.  The
// slice [lo, hi) of the bucket's sorted idx that falls in the span is found
// with two 64-way cooperative searches (<= 6 rounds for k < 2^31, or <= 2
// rounds from a directory-table bracket), staged through LDS as a dense
// (value, found-bit) span, and consumed by the same commit arithmetic.
__device__ __forceinline__ int64_t coop_lower_bound(
    const int32_t* __restrict__ idx, int64_t lo, int64_t hi, int64_t key) {
  // all 64 lanes of the calling wave participate; returns the first
  // position in [lo, hi] whose entry is >= key (hi when none).
  while (hi - lo > 0) {
    const int64_t width = hi - lo;
    const int64_t step = (width + kWave - 1) / kWave;   // >= 1
    const int64_t probe = lo + (int64_t)lane_id() * step;
    bool less = false;
    if (probe < hi) less = (int64_t)idx[probe] < key;
    const uint64_t b = ballot64(less);
    // entries are sorted, so `less` lanes form a prefix
    const int cnt = __popcll(b);
    if (cnt == 0) { hi = lo; break; }
    const int64_t last_less = lo + (int64_t)(cnt - 1) * step;
    const int64_t nlo = last_less + 1;
    int64_t nhi = lo + (int64_t)cnt * step;
    if (nhi > hi) nhi = hi;
    lo = nlo;
    hi = nhi;
  }
  return lo;
}

// One kBlockSpan-element span of one record (all 256 threads of the workgroup).
template <bool BF16>
__device__ __forceinline__ void compact_span(
    float* __restrict__ p, float* __restrict__ g, float* __restrict__ m,
    float* __restrict__ v, const int32_t* __restrict__ idx,
    const void* __restrict__ values, int64_t rec_start, int64_t n,
    int64_t k_total, const Hyper& h, float coeff, float interval, int flags,
    const int32_t* __restrict__ table, int64_t n_table, bool vec, int64_t span,
    float* s_val, uint32_t* s_found, int64_t* s_bounds) {
  const bool apply_coeff = flags & SGA_GC_APPLY_COEFF;
  const bool fold = flags & SGA_GC_FOLD;
  const bool adams = flags & SGA_GC_ADAMS;
  const int64_t off0 = span * kBlockSpan;
  const int64_t c0 = rec_start + off0;
  int64_t c1 = c0 + kBlockSpan;
  if (c1 > rec_start + n) c1 = rec_start + n;
  for (int t = threadIdx.x; t < kBlockSpan; t += kBlock) s_val[t] = 0.0f;
  if (threadIdx.x < kBlockSpan / 32) s_found[threadIdx.x] = 0u;
  if (wave_id() < 2) {
    const int64_t key = wave_id() == 0 ? c0 : c1;
    int64_t lo = 0, hi = k_total;
    if (table) {
      const int64_t j = key >> 10;
      if (j < n_table) {
        lo = table[j];
        hi = lo + (key & 1023);
        if (hi > k_total) hi = k_total;
        if (lo > k_total) lo = k_total;
      }
    }
    const int64_t r = coop_lower_bound(idx, lo, hi, key);
    if (lane_id() == 0) s_bounds[wave_id()] = r;
  }
  __syncthreads();
  const int64_t lo = s_bounds[0], hi = s_bounds[1];
  for (int64_t j = lo + threadIdx.x; j < hi; j += kBlock) {
    const int64_t t = (int64_t)idx[j] - c0;
    if (t >= 0 && t < kBlockSpan) {
      float x = BF16 ? bf16_to_f32(reinterpret_cast<const uint16_t*>(values)[j])
                     : reinterpret_cast<const float*>(values)[j];
      s_val[t] = x;
      atomicOr(&s_found[t >> 5], 1u << (t & 31));
    }
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < kChunkIters; ++it) {
    const int t0 = it * (kBlock * kVec) + threadIdx.x * kVec;
    const int64_t i = off0 + t0;
    if (i < n) {
      float pp[4], mm[4], vv[4], raw[4] = {0, 0, 0, 0};
      load4_f32(p, i, n, pp, vec);
      load4_f32(m, i, n, mm, vec);
      if (adams) {
#pragma unroll
        for (int e = 0; e < 4; ++e) vv[e] = mm[e] * mm[e];
      } else {
        load4_f32(v, i, n, vv, vec);
      }
      if (fold) load4_f32(g, i, n, raw, vec);
      const uint32_t fw = s_found[t0 >> 5] >> (t0 & 31);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool found = (fw >> e) & 1u;
        float ge = s_val[t0 + e];
        if (apply_coeff && found) ge = ge * coeff;
        const Commit c = adamw_commit(pp[e], ge, mm[e], vv[e], h);
        pp[e] = pp[e] - h.lr * c.upd;
        mm[e] = c.m_new;
        vv[e] = c.v_new;
        if (fold && !found) raw[e] = __fdiv_rn(raw[e], interval);
      }
      store4_f32(m, i, n, mm, vec);
      store4_f32(v, i, n, vv, vec);
      if (fold) store4_f32(g, i, n, raw, vec);
      store4_f32(p, i, n, pp, vec);
    }
  }
  __syncthreads();
}

template <bool BF16>
__global__ __launch_bounds__(kBlock) void k_grad_correct_compact(
    float* __restrict__ p, float* __restrict__ g, float* __restrict__ m,
    float* __restrict__ v, const int32_t* __restrict__ idx,
    const void* __restrict__ values, int64_t rec_start, int64_t n,
    int64_t k_total, Hyper h, float coeff, float interval, int flags,
    const int32_t* __restrict__ table, int64_t n_table, bool vec) {
  __shared__ float s_val[kBlockSpan];
  __shared__ uint32_t s_found[kBlockSpan / 32];
  __shared__ int64_t s_bounds[2];
  const int64_t n_spans = cdiv64(n, kBlockSpan);
  for (int64_t span = blockIdx.x; span < n_spans; span += gridDim.x)
    compact_span<BF16>(p, g, m, v, idx, values, rec_start, n, k_total, h, coeff, interval, flags,
                       table, n_table, vec, span, s_val, s_found, s_bounds);
}

// The compact commit over many records in one launch (one span per workgroup).
struct GccRecord {          // sga_gcc_record, see the header
  float* p; float* g; float* m; float* v;
  const int32_t* idx; const void* values; const int32_t* table;
  int64_t rec_start, n, k_total, n_table, first_span;
  float lr, b1, om1, b2, om2, eps, wd, bc1, bc2;
  int flags;
};

template <bool BF16>
__global__ __launch_bounds__(kBlock) void k_grad_correct_compact_multi(
    const GccRecord* __restrict__ recs, int n_recs, float coeff, float interval) {
  __shared__ float s_val[kBlockSpan];
  __shared__ uint32_t s_found[kBlockSpan / 32];
  __shared__ int64_t s_bounds[2];
  const int64_t span = blockIdx.x;
  int a = 0, b = n_recs - 1;
  while (a < b) {
    const int mid = (a + b + 1) >> 1;
    if (recs[mid].first_span <= span) a = mid; else b = mid - 1;
  }
  const GccRecord r = recs[a];
  Hyper h;
  h.lr = r.lr; h.b1 = r.b1; h.om1 = r.om1; h.b2 = r.b2; h.om2 = r.om2; h.eps = r.eps;
  h.wd = r.wd; h.bc1 = r.bc1; h.bc2 = r.bc2;
  const bool vec = aligned4(r.p, 4) && aligned4(r.g, 4) && aligned4(r.m, 4) && aligned4(r.v, 4);
  compact_span<BF16>(r.p, r.g, r.m, r.v, r.idx, r.values, r.rec_start, r.n, r.k_total, h, coeff,
                     interval, r.flags, r.table, r.n_table, vec, span - r.first_span, s_val,
                     s_found, s_bounds);
}

__global__ __launch_bounds__(kBlock) void k_dir_table(
    const int32_t* __restrict__ idx, int64_t k, int32_t* __restrict__ table,
    int64_t n_table) {
  for (int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x; j < n_table;
       j += (int64_t)gridDim.x * kBlock) {
    const int64_t key = j * 1024;
    int64_t a = 0, b = k;
    while (a < b) {
      const int64_t mid = a + (b - a) / 2;
      if ((int64_t)idx[mid] < key) a = mid + 1; else b = mid;
    }
    table[j] = (int32_t)a;
  }
}

}  // namespace sga

using namespace sga;

extern "C" int sga_adamw_grad_correct(float* p, float* g, float* m, float* v,
                                      const uint8_t* mask, int64_t n, float lr,
                                      float beta1, float om1, float beta2,
                                      float om2, float eps, float wd, float bc1,
                                      float bc2, float coeff, float interval,
                                      float lr_inactive, int emit_mode,
                                      int flags, void* stream) {
  if (n == 0) return SGA_OK;
  if (!p || !g || !m || !v || n < 0 || emit_mode < -1 || emit_mode > 3) {
    set_error("sga_adamw_grad_correct: bad argument (n=%lld emit_mode=%d)",
              (long long)n, emit_mode);
    return SGA_ERR_ARG;
  }
  if ((flags & SGA_GC_HAS_MASK) && !mask) {
    set_error("sga_adamw_grad_correct: HAS_MASK without a mask pointer");
    return SGA_ERR_ARG;
  }
  if ((flags & (SGA_GC_APPLY_COEFF | SGA_GC_CLEAR | SGA_GC_FOLD)) &&
      (emit_mode >= 0 || !(flags & SGA_GC_HAS_MASK))) {
    set_error("sga_adamw_grad_correct: coeff/clear/fold need a sparse step with a mask");
    return SGA_ERR_ARG;
  }
  if ((flags & SGA_GC_LR_SPLIT) && (emit_mode < 0 || !(flags & SGA_GC_HAS_MASK))) {
    set_error("sga_adamw_grad_correct: LR_SPLIT needs a full step with a mask");
    return SGA_ERR_ARG;
  }
  if (flags & SGA_GC_ADAMS) { bc1 = 1.0f; bc2 = 1.0f; }
  const Hyper h = mk_hyper(lr, beta1, om1, beta2, om2, eps, wd, bc1, bc2);
  const bool vec = aligned4(p, 4) && aligned4(g, 4) && aligned4(m, 4) &&
                   aligned4(v, 4) && aligned4(mask, 1);
  dim3 grid(stream_grid(n, (int64_t)kBlock * kVec, 1 << 22)), block(kBlock);
  hipStream_t st = (hipStream_t)stream;
#define SGA_GC_LAUNCH(E)                                                       \
  hipLaunchKernelGGL((k_grad_correct<E>), grid, block, 0, st, p, g, m, v, mask, \
                     n, h, coeff, interval, lr_inactive, flags, vec)
  switch (emit_mode) {
    case -1: SGA_GC_LAUNCH(-1); break;
    case 0: SGA_GC_LAUNCH(0); break;
    case 1: SGA_GC_LAUNCH(1); break;
    case 2: SGA_GC_LAUNCH(2); break;
    default: SGA_GC_LAUNCH(3); break;
  }
#undef SGA_GC_LAUNCH
  return check_launch("sga_adamw_grad_correct");
}

static_assert(sizeof(GcRecord) == sizeof(sga_gc_record), "commit record layout");

extern "C" int sga_adamw_grad_correct_multi(const sga_gc_record* recs, int n_recs,
                                            int64_t total_spans, float coeff, float interval,
                                            int emit_mode, void* stream) {
  if (n_recs == 0 || total_spans == 0) return SGA_OK;
  if (!recs || n_recs < 0 || total_spans < 0 || total_spans >= (1ll << 31) || emit_mode < -1 ||
      emit_mode > 3) {
    set_error("sga_adamw_grad_correct_multi: bad argument (n_recs=%d spans=%lld emit_mode=%d)",
              n_recs, (long long)total_spans, emit_mode);
    return SGA_ERR_ARG;
  }
  const GcRecord* r = reinterpret_cast<const GcRecord*>(recs);
  dim3 grid((unsigned)total_spans), block(kBlock);
  hipStream_t st = (hipStream_t)stream;
#define SGA_GCM_LAUNCH(E) \
  hipLaunchKernelGGL((k_grad_correct_multi<E>), grid, block, 0, st, r, n_recs, coeff, interval)
  switch (emit_mode) {
    case -1: SGA_GCM_LAUNCH(-1); break;
    case 0: SGA_GCM_LAUNCH(0); break;
    case 1: SGA_GCM_LAUNCH(1); break;
    case 2: SGA_GCM_LAUNCH(2); break;
    default: SGA_GCM_LAUNCH(3); break;
  }
#undef SGA_GCM_LAUNCH
  return check_launch("sga_adamw_grad_correct_multi");
}

extern "C" int sga_adamw_grad_correct_compact(
    float* p, float* g, float* m, float* v, const int32_t* idx,
    const void* values, int values_dtype, int64_t rec_start, int64_t n,
    int64_t k_total, float lr, float beta1, float om1, float beta2, float om2,
    float eps, float wd, float bc1, float bc2, float coeff, float interval,
    int flags, const int32_t* dir_table, int64_t n_table, void* stream) {
  if (n == 0) return SGA_OK;
  if (!p || !m || !v || n < 0 || k_total < 0 || rec_start < 0 ||
      (k_total > 0 && (!idx || !values)) ||
      ((flags & SGA_GC_FOLD) && !g) ||
      (values_dtype != SGA_F32 && values_dtype != SGA_BF16)) {
    set_error("sga_adamw_grad_correct_compact: bad argument");
    return SGA_ERR_ARG;
  }
  if (k_total + 1024 >= (1ll << 31) || rec_start + n + 1024 >= (1ll << 31)) {
    set_error("sga_adamw_grad_correct_compact: offsets must stay < 2^31 (k_total=%lld, rec_start+n=%lld)",
              (long long)k_total, (long long)(rec_start + n));
    return SGA_ERR_ARG;
  }
  if (dir_table && n_table < ((rec_start + n - 1) >> 10) + 2) {
    set_error("sga_adamw_grad_correct_compact: dir_table has %lld entries, needs >= %lld",
              (long long)n_table, (long long)(((rec_start + n - 1) >> 10) + 2));
    return SGA_ERR_ARG;
  }
  if (flags & SGA_GC_ADAMS) { bc1 = 1.0f; bc2 = 1.0f; }
  const Hyper h = mk_hyper(lr, beta1, om1, beta2, om2, eps, wd, bc1, bc2);
  const bool vec = aligned4(p, 4) && aligned4(g, 4) && aligned4(m, 4) && aligned4(v, 4);
  dim3 grid(stream_grid(n, kBlockSpan, 1 << 22)), block(kBlock);
  hipStream_t st = (hipStream_t)stream;
  if (values_dtype == SGA_BF16)
    hipLaunchKernelGGL((k_grad_correct_compact<true>), grid, block, 0, st, p, g, m, v, idx, values, rec_start, n, k_total, h, coeff, interval, flags, dir_table, n_table, vec);
  else
    hipLaunchKernelGGL((k_grad_correct_compact<false>), grid, block, 0, st, p, g, m, v, idx, values, rec_start, n, k_total, h, coeff, interval, flags, dir_table, n_table, vec);
  return check_launch("sga_adamw_grad_correct_compact");
}

static_assert(sizeof(GccRecord) == sizeof(sga_gcc_record), "compact commit record layout");

extern "C" int sga_adamw_grad_correct_compact_multi(const sga_gcc_record* recs, int n_recs,
                                                    int64_t total_spans, int values_dtype,
                                                    float coeff, float interval, void* stream) {
  if (n_recs == 0 || total_spans == 0) return SGA_OK;
  if (!recs || n_recs < 0 || total_spans < 0 || total_spans >= (1ll << 31) ||
      (values_dtype != SGA_F32 && values_dtype != SGA_BF16)) {
    set_error("sga_adamw_grad_correct_compact_multi: bad argument (n_recs=%d spans=%lld)", n_recs,
              (long long)total_spans);
    return SGA_ERR_ARG;
  }
  const GccRecord* r = reinterpret_cast<const GccRecord*>(recs);
  dim3 grid((unsigned)total_spans), block(kBlock);
  hipStream_t st = (hipStream_t)stream;
  if (values_dtype == SGA_BF16)
    hipLaunchKernelGGL((k_grad_correct_compact_multi<true>), grid, block, 0, st, r, n_recs, coeff, interval);
  else
    hipLaunchKernelGGL((k_grad_correct_compact_multi<false>), grid, block, 0, st, r, n_recs, coeff, interval);
  return check_launch("sga_adamw_grad_correct_compact_multi");
}

extern "C" int sga_build_dir_table(const int32_t* idx, int64_t k, int32_t* table,
                                   int64_t n_table, void* stream) {
  if (n_table == 0) return SGA_OK;
  if (!table || n_table < 0 || k < 0 || (k > 0 && !idx) ||
      (n_table - 1) * 1024 >= (1ll << 31)) {
    set_error("sga_build_dir_table: bad argument ((n_table-1)*1024 must stay < 2^31)");
    return SGA_ERR_ARG;
  }
  hipLaunchKernelGGL(k_dir_table, dim3(stream_grid(n_table, kBlock)),
                     dim3(kBlock), 0, (hipStream_t)stream, idx, k, table, n_table);
  return check_launch("sga_build_dir_table");
}
