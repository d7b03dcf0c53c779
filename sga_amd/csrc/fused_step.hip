// Fused per-rank sparse step over a flat bucket:
//   q = resid + g ; score(q) ; exact top-k (lowest-index ties) ;
//   idx/values pack ; resid <- q with selected coordinates zeroed ;
//   sparse AdamW commit on p/m/v with per-segment hyper-parameters.
//
// HBM traffic per element (bf16 g): the select sweeps read g and resid only
// (6 B each); the final sweep reads g, resid, p, m, v (18 B) and writes
// resid, p, m, v (16 B) plus the rho*(4+2) B pack.
#include "adam_math.hpp"
#include "select_impl.hpp"

namespace sga {

template <bool BF16G>
__device__ __forceinline__ void load_g(const void* g, int64_t i, int64_t n, float out[4], bool vec) {
  if (BF16G) load4_bf16(reinterpret_cast<const uint16_t*>(g), i, n, out, vec);
  else load4_f32(reinterpret_cast<const float*>(g), i, n, out, vec);
}

// Key source for the select sweeps.
template <bool BF16G, int SCORE>
struct SrcFused {
  const void* g;
  const float* r;
  const float* p;
  const float* m;
  const float* v;
  const sga_segment* segs;
  int n_segs;
  bool vec;
  __device__ __forceinline__ void load(int64_t i, int64_t n, uint32_t key[4]) const {
    float gg[4], rr[4];
    load_g<BF16G>(g, i, n, gg, vec);
    load4_f32(r, i, n, rr, vec);
    if (SCORE == SGA_SCORE_ABS_G) {
#pragma unroll
      for (int e = 0; e < 4; ++e) key[e] = abs_key(rr[e] + gg[e]);
      return;
    }
    float pp[4] = {0, 0, 0, 0}, mm[4], vv[4] = {0, 0, 0, 0};
    load4_f32(m, i, n, mm, vec);
    if (SCORE != SGA_SCORE_ABS_M) {
      load4_f32(p, i, n, pp, vec);
      load4_f32(v, i, n, vv, vec);
    }
    SegCursor sc;
    sc.init(segs, n_segs);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (i + e < n) {
        sc.seek(i + e);
        key[e] = score_key<SCORE>(rr[e] + gg[e], pp[e], mm[e], vv[e], sc.h);
      } else {
        key[e] = 0u;
      }
    }
  }
};

// Final sweep: select flags in index order, pack, residual, commit.
template <bool BF16G, bool BF16V, int SCORE>
__global__ __launch_bounds__(kBlock) void k_fused_final(
    const void* __restrict__ g, float* __restrict__ r, float* __restrict__ p,
    float* __restrict__ m, float* __restrict__ v, int64_t n, int64_t k,
    const sga_segment* __restrict__ segs, int n_segs,
    const SelState* __restrict__ st, const uint32_t* __restrict__ tile_sel,
    const uint32_t* __restrict__ tile_eq, int32_t* __restrict__ idx_out,
    void* __restrict__ values_out, uint8_t* __restrict__ mask_out, float factor,
    float coeff, bool vec, bool mvec) {
  const uint32_t T = st->thresh_bits;
  const uint32_t need = st->need;
  const bool scale = factor != 1.0f;
  const bool apply_coeff = coeff != 1.0f;
  const int64_t n_chunks = cdiv64(n, kChunk);
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  SegCursor sc;
  sc.init(segs, n_segs);
  for (int64_t c = (int64_t)blockIdx.x * kChunksPerBlock + wave_id(); c < n_chunks;
       c += wstride) {
    ChunkCursor cur;
    cur.sel_run = tile_sel[c];
    cur.eq_run = tile_eq[c];
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
      float gg[4] = {0, 0, 0, 0}, rr[4] = {0, 0, 0, 0}, pp[4] = {0, 0, 0, 0},
            mm[4] = {0, 0, 0, 0}, vv[4] = {0, 0, 0, 0};
      if (i < n) {
        load_g<BF16G>(g, i, n, gg, vec);
        load4_f32(r, i, n, rr, vec);
        load4_f32(p, i, n, pp, vec);
        load4_f32(m, i, n, mm, vec);
        load4_f32(v, i, n, vv, vec);
      }
      float q[4];
      uint32_t key[4];
      bool valid[4], sel[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        valid[e] = i + e < n;
        q[e] = rr[e] + gg[e];
        if (valid[e]) sc.seek(i + e);
        key[e] = valid[e] ? score_key<SCORE>(q[e], pp[e], mm[e], vv[e], sc.h) : 0u;
      }
      uint32_t pos;
      slab_select(key, valid, T, need, cur, sel, pos);
      if (i < n) {
        uint32_t mk[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          mk[e] = sel[e];
          if (!valid[e]) continue;
          sc.seek(i + e);
          float ge = 0.0f;
          if (sel[e]) {
            float val = q[e];
            if (scale) val = val * factor;
            if (BF16V) {
              const uint16_t hb = f32_to_bf16(val);
              if ((int64_t)pos < k) {
                idx_out[pos] = (int32_t)(i + e);
                reinterpret_cast<uint16_t*>(values_out)[pos] = hb;
              }
              ge = bf16_to_f32(hb);
            } else {
              if ((int64_t)pos < k) {
                idx_out[pos] = (int32_t)(i + e);
                reinterpret_cast<float*>(values_out)[pos] = val;
              }
              ge = val;
            }
            ++pos;
            if (apply_coeff) ge = ge * coeff;
          }
          const Commit cm = adamw_commit(pp[e], ge, mm[e], vv[e], sc.h);
          pp[e] = pp[e] - sc.h.lr * cm.upd;
          mm[e] = cm.m_new;
          vv[e] = cm.v_new;
          rr[e] = sel[e] ? 0.0f : q[e];
        }
        store4_f32(r, i, n, rr, vec);
        store4_f32(m, i, n, mm, vec);
        store4_f32(v, i, n, vv, vec);
        store4_f32(p, i, n, pp, vec);
        if (mask_out) store4_u8(mask_out, i, n, mk, mvec);
      }
    }
  }
}

// Optional live timing of the final sweep (HIP events on the launch stream),
// switched on by sga_prof_enable; read back with sga_prof_read after a sync.
struct ProfPair { hipEvent_t a, b; };
static bool g_prof_on = false;
static ProfPair g_prof[512];
static int g_prof_made = 0, g_prof_used = 0;

static ProfPair* prof_next() {
  if (!g_prof_on || g_prof_used >= 512) return nullptr;
  if (g_prof_used >= g_prof_made) {
    if (hipEventCreate(&g_prof[g_prof_made].a) != hipSuccess) return nullptr;
    if (hipEventCreate(&g_prof[g_prof_made].b) != hipSuccess) return nullptr;
    ++g_prof_made;
  }
  return &g_prof[g_prof_used++];
}

template <bool BF16G, bool BF16V, int SCORE>
static int run_fused(const void* g, float* resid, float* p, float* m, float* v, int64_t n,
                     int64_t k, const sga_segment* segs, int n_segs, int32_t* idx_out,
                     void* values_out, uint8_t* mask_out, float factor, float coeff, int fast,
                     sga_select_result* result, const SelWorkspace& w, hipStream_t s) {
  const bool vec = aligned4(g, BF16G ? 2 : 4) && aligned4(resid, 4) && aligned4(p, 4) &&
                   aligned4(m, 4) && aligned4(v, 4);
  SrcFused<BF16G, SCORE> src{g, resid, p, m, v, segs, n_segs, vec};
  run_select(src, n, k, 0, fast != 0, w, s);
  const int64_t n_tiles = cdiv64(n, kChunk);
  ProfPair* pp = prof_next();
  if (pp) (void)hipEventRecord(pp->a, s);
  hipLaunchKernelGGL((k_fused_final<BF16G, BF16V, SCORE>),
                     dim3(stream_grid(n_tiles, kChunksPerBlock, 1 << 20)), dim3(kBlock), 0, s, g,
                     resid, p, m, v, n, k, segs, n_segs, w.st, w.tile_gt, w.tile_eq, idx_out,
                     values_out, mask_out, factor, coeff, vec, aligned4(mask_out, 1));
  if (pp) (void)hipEventRecord(pp->b, s);
  if (result) hipLaunchKernelGGL(k_sel_result, dim3(1), dim3(1), 0, s, w.st, result);
  return check_launch("sga_fused_sparse_step");
}

}  // namespace sga

using namespace sga;

extern "C" int sga_prof_enable(int on) {
  g_prof_on = on != 0;
  g_prof_used = 0;
  return SGA_OK;
}

extern "C" int sga_prof_read(double* total_ms, int* launches) {
  if (!total_ms || !launches) { set_error("sga_prof_read: null output"); return SGA_ERR_ARG; }
  double tot = 0.0;
  int cnt = 0;
  for (int i = 0; i < g_prof_used; ++i) {
    float ms = 0.0f;
    if (hipEventSynchronize(g_prof[i].b) != hipSuccess ||
        hipEventElapsedTime(&ms, g_prof[i].a, g_prof[i].b) != hipSuccess) {
      set_error("sga_prof_read: event %d not ready", i);
      return SGA_ERR_LAUNCH;
    }
    tot += ms;
    ++cnt;
  }
  *total_ms = tot;
  *launches = cnt;
  return SGA_OK;
}

extern "C" size_t sga_fused_workspace_bytes(int64_t n) { return sel_ws_bytes(n < 0 ? 0 : n); }

extern "C" int sga_fused_sparse_step(const void* g, int g_dtype, float* resid, float* p, float* m,
                                     float* v, int64_t n, int64_t k, const sga_segment* segs,
                                     int n_segs, int score_id, int32_t* idx_out, void* values_out,
                                     int values_dtype, uint8_t* mask_out, float factor,
                                     float coeff, int fast, sga_select_result* result, void* ws,
                                     size_t ws_bytes, void* stream) {
  if (!g || !resid || !p || !m || !v || !segs || !idx_out || !values_out || n < 1 ||
      n >= (1ll << 31) || k < 1 || k > n || n_segs < 1 ||
      (g_dtype != SGA_F32 && g_dtype != SGA_BF16) ||
      (values_dtype != SGA_F32 && values_dtype != SGA_BF16) || score_id < 0 || score_id > 3) {
    set_error("sga_fused_sparse_step: bad argument (n=%lld k=%lld n_segs=%d score=%d; need "
              "1 <= k <= n < 2^31)", (long long)n, (long long)k, n_segs, score_id);
    return SGA_ERR_ARG;
  }
  SelWorkspace w;
  if (!sel_ws_carve(ws, ws_bytes, cdiv64(n, kChunk), &w)) {
    set_error("sga_fused_sparse_step: workspace missing, misaligned or smaller than "
              "sga_fused_workspace_bytes(n)=%zu", sel_ws_bytes(n));
    return SGA_ERR_WORKSPACE;
  }
  hipStream_t s = (hipStream_t)stream;
  const bool bg = g_dtype == SGA_BF16, bv = values_dtype == SGA_BF16;
#define SGA_RUN(BG, BV, SC)                                                                   \
  return run_fused<BG, BV, SC>(g, resid, p, m, v, n, k, segs, n_segs, idx_out, values_out,   \
                               mask_out, factor, coeff, fast, result, w, s)
#define SGA_RUN_SC(BG, BV)                    \
  switch (score_id) {                         \
    case 0: SGA_RUN(BG, BV, 0);               \
    case 1: SGA_RUN(BG, BV, 1);               \
    case 2: SGA_RUN(BG, BV, 2);               \
    default: SGA_RUN(BG, BV, 3);              \
  }
  if (bg && bv) { SGA_RUN_SC(true, true) }
  else if (bg) { SGA_RUN_SC(true, false) }
  else if (bv) { SGA_RUN_SC(false, true) }
  else { SGA_RUN_SC(false, false) }
#undef SGA_RUN_SC
#undef SGA_RUN
}
