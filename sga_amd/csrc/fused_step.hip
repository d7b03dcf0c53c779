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

template <bool BF16G, bool FULL = false>
__device__ __forceinline__ void load_g(const void* g, int64_t i, int64_t n, float out[4], bool vec) {
  if (BF16G) ld_bf16<FULL>(reinterpret_cast<const uint16_t*>(g), i, n, out, vec);
  else ld_f32<FULL>(reinterpret_cast<const float*>(g), i, n, out, vec);
}

// Key source for the select sweeps.  Which arrays a score reads:
//   abs_g  g r          abs_m  m              update  g r p m v      coi  g r m v
//   abs_g_blind  g      abs_gr_over_sqrt_v  g r v   (AdamS: m stands in for v = m*m)
template <bool BF16G, int SCORE>
struct SrcFused {
  const void* g;
  const float* r;
  const float* p;
  const float* m;
  const float* v;
  bool vec;
  SegCursor sc;        // per-thread cache of the current segment's hyper-parameters
  int64_t pack_extra;  // 0: separate arrays; else extra floats per kPackRun elements (packed state)
  int adams;           // AdamS: the second moment is rebuilt from m (v := m*m), no bias corrections
  // Stepwise interface of the one-sweep select.
  struct Raw { RawG g; F4 r, p, m, v; };
  struct Chunk { int64_t sh; };
  // scores that need the tensor's hyper-parameters
  static constexpr bool kHyper = SCORE == SGA_SCORE_UPDATE || SCORE == SGA_SCORE_COI ||
                                 SCORE == SGA_SCORE_GR_OVER_SQRT_V;
  static constexpr bool kNeedG = SCORE != SGA_SCORE_ABS_M;
  // g == nullptr (fp32 instantiations only): the caller's buffer `r` already holds g + r, the
  // reference's own contract (backward accumulates into the buffer that keeps the residual)
  __device__ __forceinline__ bool has_g() const { return BF16G || g != nullptr; }
  static constexpr bool kNeedR = kNeedG && SCORE != SGA_SCORE_ABS_G_BLIND;
  static constexpr bool kNeedP = SCORE == SGA_SCORE_UPDATE;
  static constexpr bool kNeedV = kHyper;                       // v, or m in its place under AdamS
  __device__ __forceinline__ bool need_m() const {
    return SCORE == SGA_SCORE_UPDATE || SCORE == SGA_SCORE_COI || SCORE == SGA_SCORE_ABS_M ||
           (kNeedV && adams);
  }
  // measured: look-ahead makes no difference beyond one slab for |g + r| and two for the chains
  static constexpr int kAhead = kHyper ? 2 : 1;
  __device__ __forceinline__ Chunk chunk_begin(int64_t c) {
    const int64_t i0 = uniform_i64(c) * kChunk;
    return Chunk{(i0 >> kPackRunLog) * pack_extra};
  }
  // The tensor of the chunk's first element (a walk from the segment directory).
  __device__ __forceinline__ void chunk_hyper(int64_t c) {
    if (kHyper) sc.seek_uniform(uniform_i64(c) * kChunk);
  }
  template <bool FULL>
  __device__ __forceinline__ void fetch(const Chunk& ck, int64_t i, int64_t n, Raw& w) {
    if (kNeedG && has_g()) fetch_g<BF16G, FULL>(g, i, n, vec, w.g);
    if (kNeedR) w.r = ldraw_f32<FULL>(r + ck.sh, i, n, vec);
    if (need_m()) w.m = ldraw_f32<FULL>(m + ck.sh, i, n, vec);
    if (kNeedP) w.p = ldraw_f32<FULL>(p + ck.sh, i, n, vec);
    if (kNeedV && !adams) w.v = ldraw_f32<FULL>(v + ck.sh, i, n, vec);
  }
  template <bool FULL>
  __device__ __forceinline__ void keys(const Chunk& ck, int64_t i, int64_t n, const Raw& w,
                                       uint32_t key[4]) {
    float q[4] = {0, 0, 0, 0}, rr[4] = {0, 0, 0, 0};
    float pp[4] = {0, 0, 0, 0}, mm[4] = {0, 0, 0, 0}, vv[4] = {0, 0, 0, 0};
    if (kNeedG && has_g()) unpack_g<BF16G, FULL>(w.g, q);
    if (kNeedR) {
      unpack_f32(w.r, rr);
#pragma unroll
      for (int e = 0; e < 4; ++e) q[e] = has_g() ? rr[e] + q[e] : rr[e];
    }
    if (need_m()) unpack_f32(w.m, mm);
    if (!kHyper) {
#pragma unroll
      for (int e = 0; e < 4; ++e) key[e] = abs_key(SCORE == SGA_SCORE_ABS_M ? mm[e] : q[e]);
      return;
    }
    if (kNeedP) unpack_f32(w.p, pp);
    if (adams) {
#pragma unroll
      for (int e = 0; e < 4; ++e) vv[e] = mm[e] * mm[e];
    } else {
      unpack_f32(w.v, vv);
    }
    slab_score_keys<SCORE, FULL>(sc, adams, i, n, q, pp, mm, vv, key);
  }
  template <bool FULL = false>
  __device__ __forceinline__ void load(int64_t i, int64_t n, uint32_t key[4]) {
    const int64_t sh = pack_shift<FULL>(i, pack_extra);
    float q[4] = {0, 0, 0, 0}, rr[4] = {0, 0, 0, 0};
    float pp[4] = {0, 0, 0, 0}, mm[4] = {0, 0, 0, 0}, vv[4] = {0, 0, 0, 0};
    if (kNeedG && has_g()) load_g<BF16G, FULL>(g, i, n, q, vec);
    if (kNeedR) {
      ld_f32<FULL>(r + sh, i, n, rr, vec);
#pragma unroll
      for (int e = 0; e < 4; ++e) q[e] = has_g() ? rr[e] + q[e] : rr[e];
    }
    if (need_m()) ld_f32<FULL>(m + sh, i, n, mm, vec);
    if (!kHyper) {
#pragma unroll
      for (int e = 0; e < 4; ++e) key[e] = abs_key(SCORE == SGA_SCORE_ABS_M ? mm[e] : q[e]);
      return;
    }
    if (kNeedP) ld_f32<FULL>(p + sh, i, n, pp, vec);
    if (!adams) ld_f32<FULL>(v + sh, i, n, vv, vec);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (FULL || i + e < n) {
        sc.seek(i + e);
        Hyper h = sc.h;
        float ve = vv[e];
        if (adams) { ve = mm[e] * mm[e]; h.bc1 = 1.0f; h.bc2 = 1.0f; }
        key[e] = score_key<SCORE>(q[e], pp[e], mm[e], ve, h);
      } else {
        key[e] = 0u;
      }
    }
  }
};

// Everything the final sweep needs besides the chunk index.
struct FinalArgs {
  const void* g;
  float* r;                 // state as the step reads it ...
  float* p;
  float* m;
  float* v;
  float* ro;                // ... and where it writes the new state (the same arrays for the
  float* po;                // in-place entry points, other ones for the out-of-place step)
  float* mo;
  float* vo;
  int64_t n, k;
  int32_t* idx_out;
  void* values_out;
  uint8_t* mask_out;
  float factor, coeff;
  uint32_t T, need;
  bool vec, mvec, scale, apply_coeff;
  bool adams, fold;         // AdamS commit (adams.py:87-213); residual-mean fold of the new residual
  float interval;           // fold divisor (true division, as adamw_torch.py does)
  int64_t pack_extra;
  const uint32_t* planes;   // the settled selection as bit planes (PLANES mode), else unused
};

// One 1024-element chunk of the final sweep, owned by one wave.  FULL: the
// chunk is entirely in range and every array is vector-aligned, so all 20
// loads are unconditional and issued before the first use.
// IT0 / NIT: the slabs [IT0, IT0+NIT) of the chunk are handled by this call;
// `cur` carries the running selected / tie counts across calls.
// PLANES: the selection was already settled as bit planes (bracket sweep +
// candidates): the slab's four 64-bit ballots are read on the scalar unit and
// the keys are not formed again; SCORE is then irrelevant.
template <bool BF16G, bool BF16V, int SCORE, bool FULL, int IT0, int NIT, bool PLANES>
__device__ __forceinline__ void final_chunk(const FinalArgs& a, int64_t c, ChunkCursor& cur,
                                            SegCursor& sc, SegCursor& lc) {
  const int64_t n = a.n;
  const int64_t sh = pack_shift<true>(c << 10, a.pack_extra);     // c is wave-uniform
  const float* const R = a.r + sh;
  const float* const P = a.p + sh;
  const float* const M = a.m + sh;
  const float* const V = a.v + sh;
  float* const RO = a.ro + sh;
  float* const PO = a.po + sh;
  float* const MO = a.mo + sh;
  float* const VO = a.vo + sh;
  float gg[kChunkIters][4], rr[kChunkIters][4], pp[kChunkIters][4], mm[kChunkIters][4],
      vv[kChunkIters][4];
  const bool has_g = BF16G || a.g != nullptr;     // no g: the buffer `r` already holds g + r
  if (FULL) {
    // raw loads first (bf16 kept packed), a scheduling fence, then unpacking:
    // the wave has all 20 loads of its chunk in flight before the first wait
    H4 graw_h[kChunkIters];
    F4 graw_f[kChunkIters], rraw[kChunkIters], praw[kChunkIters], mraw[kChunkIters],
        vraw[kChunkIters];
#pragma unroll
    for (int it = IT0; it < IT0 + NIT; ++it) {
      const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
      if (BF16G) graw_h[it] = ldh4_nt(reinterpret_cast<const uint16_t*>(a.g) + i);
      else if (has_g) graw_f[it] = ld4_nt(reinterpret_cast<const float*>(a.g) + i);
      else graw_f[it] = F4{0.0f, 0.0f, 0.0f, 0.0f};
      rraw[it] = ld4_nt(R + i);
      praw[it] = ld4_nt(P + i);
      mraw[it] = ld4_nt(M + i);
      vraw[it] = ld4_nt(V + i);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int it = IT0; it < IT0 + NIT; ++it) {
      if (BF16G) {
        gg[it][0] = bf16_to_f32(graw_h[it].x); gg[it][1] = bf16_to_f32(graw_h[it].y);
        gg[it][2] = bf16_to_f32(graw_h[it].z); gg[it][3] = bf16_to_f32(graw_h[it].w);
      } else {
        gg[it][0] = graw_f[it].x; gg[it][1] = graw_f[it].y; gg[it][2] = graw_f[it].z; gg[it][3] = graw_f[it].w;
      }
      rr[it][0] = rraw[it].x; rr[it][1] = rraw[it].y; rr[it][2] = rraw[it].z; rr[it][3] = rraw[it].w;
      pp[it][0] = praw[it].x; pp[it][1] = praw[it].y; pp[it][2] = praw[it].z; pp[it][3] = praw[it].w;
      mm[it][0] = mraw[it].x; mm[it][1] = mraw[it].y; mm[it][2] = mraw[it].z; mm[it][3] = mraw[it].w;
      vv[it][0] = vraw[it].x; vv[it][1] = vraw[it].y; vv[it][2] = vraw[it].z; vv[it][3] = vraw[it].w;
    }
  } else {
#pragma unroll
    for (int it = IT0; it < IT0 + NIT; ++it) {
      const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
#pragma unroll
      for (int e = 0; e < 4; ++e) gg[it][e] = rr[it][e] = pp[it][e] = mm[it][e] = vv[it][e] = 0.0f;
      if (i < n) {
        if (has_g) load_g<BF16G, false>(a.g, i, n, gg[it], a.vec);
        load4_f32(R, i, n, rr[it], a.vec);
        load4_f32(P, i, n, pp[it], a.vec);
        load4_f32(M, i, n, mm[it], a.vec);
        load4_f32(V, i, n, vv[it], a.vec);
      }
    }
  }
#pragma unroll
  for (int it = IT0; it < IT0 + NIT; ++it) {
    const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
    float q[4];
    bool valid[4], sel[4];
    uint32_t pos;
    if (PLANES) {
      // words 2e, 2e + 1 of the slab are the ballot of element e over the 64 lanes; lanes are in
      // index order, so the selected coordinates before (lane, e) are the mask bits below the
      // lane over all four ballots plus the lane's own earlier elements
      const uint64_t* pw = reinterpret_cast<const uint64_t*>(a.planes) + (uniform_i64(c) * kChunkIters + it) * 4;
      uint32_t below = 0, total = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint64_t mk = pw[e];
        valid[e] = FULL || i + e < n;
        q[e] = has_g ? rr[it][e] + gg[it][e] : rr[it][e];
        sel[e] = __builtin_amdgcn_inverse_ballot_w64(mk);
        below += lanes_below(mk);
        total += (uint32_t)__popcll(mk);
      }
      pos = cur.sel_run + below;
      cur.sel_run += total;
    } else {
      uint32_t key[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        valid[e] = FULL || i + e < n;
        q[e] = has_g ? rr[it][e] + gg[it][e] : rr[it][e];
        if (SCORE == SGA_SCORE_ABS_G) key[e] = abs_key(q[e]);
        else if (SCORE == SGA_SCORE_ABS_G_BLIND) key[e] = abs_key(gg[it][e]);
        else if (SCORE == SGA_SCORE_ABS_M) key[e] = abs_key(mm[it][e]);
        else {
          // only when the one-sweep select is off or failed: a per-lane cursor
          if (valid[e]) lc.seek(i + e);
          Hyper hk = lc.h;
          float ve = vv[it][e];
          if (a.adams) { ve = mm[it][e] * mm[it][e]; hk.bc1 = 1.0f; hk.bc2 = 1.0f; }
          key[e] = valid[e] ? score_key<SCORE>(q[e], pp[it][e], mm[it][e], ve, hk) : 0u;
        }
      }
      slab_select(key, valid, a.T, a.need, cur, sel, pos);
    }
    if (FULL || i < n) {
      uint32_t mk[4];
      float ge[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        mk[e] = sel[e];
        ge[e] = 0.0f;
        if (!valid[e] || !sel[e]) continue;
        float val = q[e];
        if (a.scale) val = val * a.factor;
        if (BF16V) {
          const uint16_t hb = f32_to_bf16(val);
          if ((int64_t)pos < a.k) {
            a.idx_out[pos] = (int32_t)(i + e);
            reinterpret_cast<uint16_t*>(a.values_out)[pos] = hb;
          }
          ge[e] = bf16_to_f32(hb);
        } else {
          if ((int64_t)pos < a.k) {
            a.idx_out[pos] = (int32_t)(i + e);
            reinterpret_cast<float*>(a.values_out)[pos] = val;
          }
          ge[e] = val;
        }
        ++pos;
        if (a.apply_coeff) ge[e] = ge[e] * a.coeff;
      }
      // The commit takes its hyper-parameters from the scalar unit: the slab lies inside one
      // tensor but for the few that hold a boundary, which are committed once per tensor piece.
      const int64_t s0 = uniform_i64(c) * kChunk + it * (kWave * kVec);
      int64_t s1 = s0 + kWave * kVec;
      if (!FULL && s1 > n) s1 = n;
      if (s0 < sc.lo || s0 >= sc.hi) sc.seek_uniform(s0);
      // a coordinate no tensor of the table covers keeps its p / m / v
      float pn[4] = {pp[it][0], pp[it][1], pp[it][2], pp[it][3]};
      float mn[4] = {mm[it][0], mm[it][1], mm[it][2], mm[it][3]};
      float vn[4] = {vv[it][0], vv[it][1], vv[it][2], vv[it][3]};
      for (;;) {
        const bool whole = sc.lo <= s0 && sc.hi >= s1;
        Hyper h = sc.h;
        if (a.adams) { h.bc1 = 1.0f; h.bc2 = 1.0f; }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float ve = a.adams ? mm[it][e] * mm[it][e] : vv[it][e];
          const Commit cm = adamw_commit(pp[it][e], ge[e], mm[it][e], ve, h);
          const float pe = pp[it][e] - h.lr * cm.upd;
          if (whole || (i + e >= sc.lo && i + e < sc.hi)) { pn[e] = pe; mn[e] = cm.m_new; vn[e] = cm.v_new; }
        }
        const int64_t nxt = sc.hi;
        if (whole || nxt >= s1) break;
        sc.advance_uniform(nxt);
        if (sc.hi <= nxt) break;              // the table does not tile [0, n): stop
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (!valid[e]) continue;
        pp[it][e] = pn[e]; mm[it][e] = mn[e]; vv[it][e] = vn[e];
        rr[it][e] = sel[e] ? 0.0f : q[e];
        if (a.fold) rr[it][e] = __fdiv_rn(rr[it][e], a.interval);
      }
      st_f32<FULL>(RO, i, n, rr[it], a.vec);
      st_f32<FULL>(MO, i, n, mm[it], a.vec);
      st_f32<FULL>(VO, i, n, vv[it], a.vec);
      st_f32<FULL>(PO, i, n, pp[it], a.vec);
      if (a.mask_out) st_u8<FULL>(a.mask_out, i, n, mk, a.mvec);
    }
  }
}

// Final sweep: select flags in index order, pack, residual, commit.
// `when`: 0 run always; 1 only if the sampled bracket held (the planes are
// settled); 2 only if it failed (the radix passes fixed the threshold and the
// keys are formed again here); 3 like 2, and only if the single-sweep step
// stood back before it touched anything.
// (five waves per SIMD wherever the key is not an Adam-normalised chain formed in this kernel)
template <bool BF16G, bool BF16V, int SCORE, bool PLANES>
__global__ __launch_bounds__(kBlock, (PLANES || SCORE == SGA_SCORE_ABS_G || SCORE == SGA_SCORE_ABS_M ||
                                      SCORE == SGA_SCORE_ABS_G_BLIND) ? 5 : 1)
void k_fused_final(
    FinalArgs a, const sga_segment* __restrict__ segs, int n_segs,
    const SelState* __restrict__ st, const uint32_t* __restrict__ tile_sel,
    const uint32_t* __restrict__ tile_eq, int when, const int32_t* __restrict__ seg_dir) {
  if (when == 3) { if (st->bracket_ok != 0 || st->spec != 0) return; }
  else if (when != 0 && (st->bracket_ok != 0) != (when == 1)) return;
  a.T = st->thresh_bits;
  a.need = st->need;
  const int64_t n_chunks = cdiv64(a.n, kChunk);
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  SegCursor sc, lc;              // sc: wave-uniform (scalar unit); lc: per lane, key forming only
  sc.init(segs, n_segs, seg_dir);
  lc.init(segs, n_segs, seg_dir);
  const bool can_full = a.vec && (a.mask_out == nullptr || a.mvec);
  const unsigned blk = a.pack_extra != 0 ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
  for (int64_t c = (int64_t)blk * kChunksPerBlock + wave_id(); c < n_chunks;
       c += wstride) {
    ChunkCursor cur;
    cur.sel_run = tile_sel[c];
    cur.eq_run = PLANES ? 0u : tile_eq[c];
    if (can_full && (c + 1) * kChunk <= a.n) {
      // one 256-element slab at a time (5 loads in flight per lane): measured
      // as fast as batching all four slabs, at twice the occupancy
      final_chunk<BF16G, BF16V, SCORE, true, 0, 1, PLANES>(a, c, cur, sc, lc);
      final_chunk<BF16G, BF16V, SCORE, true, 1, 1, PLANES>(a, c, cur, sc, lc);
      final_chunk<BF16G, BF16V, SCORE, true, 2, 1, PLANES>(a, c, cur, sc, lc);
      final_chunk<BF16G, BF16V, SCORE, true, 3, 1, PLANES>(a, c, cur, sc, lc);
    } else {
      // the ragged path too: holding four slabs at once would set the register count (and so
      // the occupancy) of the whole kernel
      final_chunk<BF16G, BF16V, SCORE, false, 0, 1, PLANES>(a, c, cur, sc, lc);
      final_chunk<BF16G, BF16V, SCORE, false, 1, 1, PLANES>(a, c, cur, sc, lc);
      final_chunk<BF16G, BF16V, SCORE, false, 2, 1, PLANES>(a, c, cur, sc, lc);
      final_chunk<BF16G, BF16V, SCORE, false, 3, 1, PLANES>(a, c, cur, sc, lc);
    }
  }
}

// One bucket of a (possibly batched) fused step.
struct FusedJob {
  const void* g;
  float* resid;
  float* p;
  float* m;
  float* v;
  int64_t n, k;
  const sga_segment* segs;
  int n_segs;
  int32_t* idx_out;
  void* values_out;
  uint8_t* mask_out;
  sga_select_result* result;
  SelWorkspace w;
  float* out[4];            // resid / p / m / v of the new state; all null: in place
};

// The two-sweep step for up to kMaxJobs buckets that share dtypes, score and knobs: the short
// kernels of the buckets' selects run as one batched chain, the sweeps are launched per bucket.
template <bool BF16G, bool BF16V, int SCORE>
static int run_fused(const FusedJob* fj, int count, float factor, float coeff, int fast, int flags,
                     float interval, hipStream_t s, int64_t pack_extra, const char* who) {
  using Src = SrcFused<BF16G, SCORE>;
  const int adams = (flags & SGA_GC_ADAMS) ? 1 : 0;
  static_assert(kSelDirEntries == kSegDirEntries, "the workspace holds one directory");
  SrcPack<Src> srcs = {};
  SegDirJobs dj = {};
  SelBatch B;
  bool vec[kMaxJobs];
  int64_t max_dir = 0;
  // Adam-normalised scores with the one-sweep select armed: the sweep leaves the selection as bit
  // planes (settled by the candidates) and the final sweep reads one bit per coordinate instead of
  // evaluating the score chain a second time; if the bracket fails on the device, the key-forming
  // final sweep runs instead.  For |g + r| and |m| the key is one instruction and re-forming it is
  // cheaper than writing and reading the planes (measured: 0.3 ms per step at 1.2e9 elements).
  bool use_fast = fast != 0;
  for (int b = 0; b < count; ++b) use_fast = use_fast && SelBatch::fast_ok(fj[b].w, fj[b].n);
  const bool planes = Src::kHyper && use_fast;
  for (int b = 0; b < count; ++b) {
    const FusedJob& f = fj[b];
    vec[b] = aligned4(f.g, BF16G ? 2 : 4) && aligned4(f.resid, 4) && aligned4(f.p, 4) &&
             aligned4(f.m, 4) && aligned4(f.v, 4) && aligned4(f.out[0], 4) &&
             aligned4(f.out[1], 4) && aligned4(f.out[2], 4) && aligned4(f.out[3], 4);
    srcs.s[b] = Src{f.g, f.resid, f.p, f.m, f.v, vec[b], {}, pack_extra, adams};
    srcs.s[b].sc.init(f.segs, f.n_segs, f.w.seg_dir);
    dj.j[b].segs = f.segs; dj.j[b].dir = f.w.seg_dir; dj.j[b].n = f.n; dj.j[b].n_segs = f.n_segs;
    const int64_t nb = (f.n + (1ll << kSegDirLog) - 1) >> kSegDirLog;
    if (nb > max_dir) max_dir = nb;
    ChainJob& J = B.add(f.w, f.n, f.k, 0);
    J.planes = planes ? f.w.pbits : nullptr;
    J.result = f.result;
  }
  hipLaunchKernelGGL(k_seg_dir_batch, B.grid(stream_grid(max_dir, kBlock, 128)), dim3(kBlock), 0, s, dj);
  run_select_batch(srcs, B, use_fast, planes ? 1 : 0, s);
  if (planes) hipLaunchKernelGGL(k_cand_bits, B.grid(256), dim3(kBlock), 0, s, B.jobs);
  for (int b = 0; b < count; ++b) {
    const FusedJob& f = fj[b];
    const SelWorkspace& w = f.w;
    const int64_t n_tiles = cdiv64(f.n, kChunk);
    ProfPair* pp = prof_begin(SGA_PROF_FUSED_FINAL, s);
    FinalArgs fa;
    fa.g = f.g; fa.r = f.resid; fa.p = f.p; fa.m = f.m; fa.v = f.v; fa.n = f.n; fa.k = f.k;
    fa.ro = f.out[0] ? f.out[0] : f.resid; fa.po = f.out[0] ? f.out[1] : f.p;
    fa.mo = f.out[0] ? f.out[2] : f.m; fa.vo = f.out[0] ? f.out[3] : f.v;
    fa.idx_out = f.idx_out; fa.values_out = f.values_out; fa.mask_out = f.mask_out;
    fa.factor = factor; fa.coeff = coeff; fa.T = 0; fa.need = 0;
    fa.vec = vec[b]; fa.mvec = aligned4(f.mask_out, 1);
    fa.scale = factor != 1.0f; fa.apply_coeff = coeff != 1.0f;
    fa.pack_extra = pack_extra;
    fa.adams = adams != 0; fa.fold = (flags & SGA_GC_FOLD) != 0; fa.interval = interval;
    fa.planes = w.pbits;
    const dim3 one_shot(stream_grid(n_tiles, kChunksPerBlock, 1 << 20));
    if (planes) {
      hipLaunchKernelGGL((k_fused_final<BF16G, BF16V, SGA_SCORE_ABS_G, true>), one_shot, dim3(kBlock), 0, s,
                         fa, f.segs, f.n_segs, w.st, w.tile_gt, w.tile_eq, 1, w.seg_dir);
      // the rare other outcome: a small grid that strides over the chunks (returns at once otherwise)
      hipLaunchKernelGGL((k_fused_final<BF16G, BF16V, SCORE, false>),
                         dim3(stream_grid(n_tiles, kChunksPerBlock, 2048)), dim3(kBlock), 0, s, fa,
                         f.segs, f.n_segs, w.st, w.tile_gt, w.tile_eq, 2, w.seg_dir);
    } else {
      hipLaunchKernelGGL((k_fused_final<BF16G, BF16V, SCORE, false>), one_shot, dim3(kBlock), 0, s, fa,
                         f.segs, f.n_segs, w.st, w.tile_gt, w.tile_eq, 0, w.seg_dir);
    }
    prof_end(pp, s);
  }
  launch_result(B, s);
  return check_launch(who);
}


// ====================================================== single-sweep step
// The step above reads the score inputs twice because the threshold is global.
// The sampled bracket [T_LO, T_HI) is known BEFORE any sweep, though, and it
// decides all but a few coordinates: a key at or above T_HI is selected, a key
// below T_LO is not, whatever the exact threshold turns out to be.  The
// single-sweep step therefore reads g, resid, p, m, v ONCE and commits every
// coordinate on the spot.  A coordinate inside the bracket is committed on a
// guess -- selected if its key is at or above the bracket's midpoint T_MID --
// and recorded with its key and the four inputs of its commit.  The candidate
// descent over the recorded keys then fixes the exact threshold; the guesses
// that turn out wrong (keys between the midpoint and the threshold: a few per
// cent of the records) are committed again from their records, and the pack
// is written in index order from two bit planes: S (what the sweep took as
// selected: it parked those pack values in a chunk-strided staging array) and
// F (the exact selection: S patched by the settlement).
//
// Exactness: whenever the bracket holds the k-th key and the record lists have
// room, every output is the two-sweep step's, bit for bit.  What cannot be
// undone is a commit on a bracket that MISSED: the margins are 12 sigma of the
// sample rank (6 sigma if the four neighbours of every sampled quad were
// perfectly correlated), the offsets move with a caller-provided seed, and a
// miss is reported as status 3 (the step is then invalid).  The kernel stands
// back, before touching anything, when the sample says the bracket holds more
// keys than the lists (plateaus of equal keys) or the bracket is open below:
// the radix passes and the key-forming final sweep then do the step exactly.
struct SpecArgs {
  uint32_t* splane;       // S: keys at or above T_MID (128 B per chunk), as the sweep committed
  uint32_t* fplane;       // F: starts as S, patched by the settlement into the exact selection
  void* stage;            // pack values of the S coordinates, chunk c at [c * 1024, ...)
  uint32_t* seg_idx;
  uint32_t* seg_key;
  F4* seg_rec;            // (q, p, m, v) of each recorded coordinate
  uint32_t* seg_cnt;
  uint32_t* seg_fail;     // per segment: 0, or ~base of the first reservation that did not fit
  uint32_t seg_cap;
  uint32_t* tile_gt;
  uint32_t* tile_eq;
  uint32_t* hi_part;
  uint32_t* nf_part;
  uint32_t* ovf_idx;      // shared overflow list: chunks whose segment is full, and what a
  uint32_t* ovf_key;      // chunk records beyond a wave's LDS buffer
  F4* ovf_rec;
  uint32_t* ovf_cnt;
  uint32_t ovf_cap;
  double n_over_ns;       // population / sample size
  double est_limit;       // stand back when the sample predicts more bracket keys than this
};

constexpr int kSpecCandCap = 256;          // records a chunk gathers in LDS before it spills

struct SpecLds {
  uint32_t idx[kSpecCandCap];
  uint32_t key[kSpecCandCap];
  F4 rec[kSpecCandCap];
  uint32_t splane[kPlaneWordsPerChunk];
};

// Midpoint of the bracket in key space: the guess for the coordinates inside it.
__device__ __forceinline__ uint32_t spec_mid(uint32_t t_lo, uint32_t t_hi) {
  return t_hi > 0x7FFFFFFFu ? t_hi : t_lo + ((t_hi - t_lo) >> 1);   // open above: guess "not selected"
}

// Pack value and commit gradient of a selected coordinate (the same chain as the final sweep).
template <bool BF16V>
__device__ __forceinline__ float spec_value(const FinalArgs& a, float q, uint16_t& hb, float& val) {
  val = q;
  if (a.scale) val = val * a.factor;
  float ge;
  if (BF16V) { hb = f32_to_bf16(val); ge = bf16_to_f32(hb); }
  else { hb = 0; ge = val; }
  if (a.apply_coeff) ge = ge * a.coeff;
  return ge;
}

// One 256-element slab of the single sweep.  chi: keys at or above T_HI so far
// in the chunk; s_run: S coordinates so far; mycnt: records so far.
template <bool BF16G, bool BF16V, int SCORE, bool FULL>
__device__ __forceinline__ void spec_slab(const FinalArgs& a, const SpecArgs& sa, SelState* st,
                                          int64_t c, int it, uint32_t T_LO, uint32_t T_MID,
                                          uint32_t T_HI, SegCursor& sc, uint32_t& chi,
                                          uint32_t& s_run, uint32_t& tot_nf, uint32_t& mycnt,
                                          SpecLds& lds, const float* R, const float* P,
                                          const float* M, const float* V, int64_t sh) {
  constexpr bool kHyper = SCORE == SGA_SCORE_UPDATE || SCORE == SGA_SCORE_COI ||
                          SCORE == SGA_SCORE_GR_OVER_SQRT_V;
  const int64_t n = a.n;
  const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
  float gg[4] = {0, 0, 0, 0}, rr[4] = {0, 0, 0, 0}, pp[4] = {0, 0, 0, 0}, mm[4] = {0, 0, 0, 0},
        vv[4] = {0, 0, 0, 0};
  const bool has_g = BF16G || a.g != nullptr;     // no g: the buffer `r` already holds g + r
  if (FULL) {
    H4 gh; F4 gf;
    if (BF16G) gh = ldh4_nt(reinterpret_cast<const uint16_t*>(a.g) + i);
    else if (has_g) gf = ld4_nt(reinterpret_cast<const float*>(a.g) + i);
    else gf = F4{0.0f, 0.0f, 0.0f, 0.0f};
    const F4 r4 = ld4_nt(R + i), p4 = ld4_nt(P + i), m4 = ld4_nt(M + i), v4 = ld4_nt(V + i);
    __builtin_amdgcn_sched_barrier(0);
    if (BF16G) { gg[0] = bf16_to_f32(gh.x); gg[1] = bf16_to_f32(gh.y); gg[2] = bf16_to_f32(gh.z); gg[3] = bf16_to_f32(gh.w); }
    else { gg[0] = gf.x; gg[1] = gf.y; gg[2] = gf.z; gg[3] = gf.w; }
    unpack_f32(r4, rr); unpack_f32(p4, pp); unpack_f32(m4, mm); unpack_f32(v4, vv);
  } else if (i < n) {
    if (has_g) load_g<BF16G, false>(a.g, i, n, gg, a.vec);
    load4_f32(R, i, n, rr, a.vec);
    load4_f32(P, i, n, pp, a.vec);
    load4_f32(M, i, n, mm, a.vec);
    load4_f32(V, i, n, vv, a.vec);
  }
  float q[4];
  uint32_t key[4] = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < 4; ++e) q[e] = has_g ? rr[e] + gg[e] : rr[e];
  if (!kHyper) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      key[e] = abs_key(SCORE == SGA_SCORE_ABS_M ? mm[e] : SCORE == SGA_SCORE_ABS_G_BLIND ? gg[e] : q[e]);
  } else if (FULL || uniform_i64(i) < n) {
    float vk[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) vk[e] = a.adams ? mm[e] * mm[e] : vv[e];
    slab_score_keys<SCORE, FULL>(sc, a.adams ? 1 : 0, i, n, q, pp, mm, vk, key);
  }
  Ballot4 above, cand, S;
  uint64_t nf = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint64_t valid = FULL ? ~0ull : ballot64(i + e < n);
    above.m[e] = ballot64(key[e] >= T_HI) & valid;
    cand.m[e] = ballot64(key[e] >= T_LO) & valid & ~above.m[e];
    S.m[e] = ballot64(key[e] >= T_MID) & valid;
    nf |= ballot64(key[e] >= 0x7F800000u) & valid;
  }
  chi += above.count();
  if (nf) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      tot_nf += (uint32_t)__popcll(ballot64(key[e] >= 0x7F800000u && (FULL || i + e < n)));
  }
  // records of the bracket's coordinates: the wave's LDS buffer, and past its end straight to
  // the overflow list (a reservation per slab; nothing downstream needs a chunk's records in
  // one piece)
  if (cand.any()) {                                      // scalar branch
    const uint32_t cnt = cand.count();
    const uint32_t room = mycnt < (uint32_t)kSpecCandCap ? (uint32_t)kSpecCandCap - mycnt : 0u;
    uint32_t obase = 0;
    bool fits = true;
    if (cnt > room) {
      if (lane_id() == 0) obase = atomicAdd(sa.ovf_cnt, cnt - room);
      obase = __shfl(obase, 0, kWave);
      fits = obase + (cnt - room) <= sa.ovf_cap;         // a list over its capacity is seen by the check
    }
    uint32_t pos = cand.below_lane();                    // position among the slab's records
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (!cand.mine(e)) continue;
      const F4 rec{q[e], pp[e], mm[e], vv[e]};
      if (pos < room) {
        lds.idx[mycnt + pos] = (uint32_t)(i + e); lds.key[mycnt + pos] = key[e]; lds.rec[mycnt + pos] = rec;
      } else if (fits) {
        const uint32_t o = obase + (pos - room);
        sa.ovf_idx[o] = (uint32_t)(i + e); sa.ovf_key[o] = key[e]; sa.ovf_rec[o] = rec;
      }
      ++pos;
    }
    mycnt += cnt < room ? cnt : room;
  }
  plane_put(S, it, lds.splane);
  const uint32_t s_before = s_run;
  s_run += S.count();
  if (!FULL && i >= n) return;
  bool sel[4], valid[4];
  float ge[4];
  uint32_t spos = s_before + S.below_lane();
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    valid[e] = FULL || i + e < n;
    sel[e] = S.mine(e);
    ge[e] = 0.0f;
    if (!sel[e]) continue;
    uint16_t hb; float val;
    ge[e] = spec_value<BF16V>(a, q[e], hb, val);
    if (BF16V) reinterpret_cast<uint16_t*>(sa.stage)[c * kChunk + spos] = hb;
    else reinterpret_cast<float*>(sa.stage)[c * kChunk + spos] = val;
    ++spos;
  }
  const int64_t s0 = uniform_i64(c) * kChunk + it * (kWave * kVec);
  int64_t s1 = s0 + kWave * kVec;
  if (!FULL && s1 > n) s1 = n;
  if (s0 < sc.lo || s0 >= sc.hi) sc.seek_uniform(s0);
  // a coordinate no tensor of the table covers keeps its p / m / v
  float pn[4] = {pp[0], pp[1], pp[2], pp[3]}, mn[4] = {mm[0], mm[1], mm[2], mm[3]},
        vn[4] = {vv[0], vv[1], vv[2], vv[3]};
  for (;;) {
    const bool whole = sc.lo <= s0 && sc.hi >= s1;
    Hyper h = sc.h;
    if (a.adams) { h.bc1 = 1.0f; h.bc2 = 1.0f; }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float ve = a.adams ? mm[e] * mm[e] : vv[e];
      const Commit cm = adamw_commit(pp[e], ge[e], mm[e], ve, h);
      const float pe = pp[e] - h.lr * cm.upd;
      if (whole || (i + e >= sc.lo && i + e < sc.hi)) { pn[e] = pe; mn[e] = cm.m_new; vn[e] = cm.v_new; }
    }
    const int64_t nxt = sc.hi;
    if (whole || nxt >= s1) break;
    sc.advance_uniform(nxt);
    if (sc.hi <= nxt) break;              // the table does not tile [0, n): stop
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (!valid[e]) continue;
    pp[e] = pn[e]; mm[e] = mn[e]; vv[e] = vn[e];
    rr[e] = sel[e] ? 0.0f : q[e];
    if (a.fold) rr[e] = __fdiv_rn(rr[e], a.interval);
  }
  st_f32<FULL>(a.ro + sh, i, n, rr, a.vec);
  st_f32<FULL>(a.mo + sh, i, n, mm, a.vec);
  st_f32<FULL>(a.vo + sh, i, n, vv, a.vec);
  st_f32<FULL>(a.po + sh, i, n, pp, a.vec);
}

template <bool BF16G, bool BF16V, int SCORE>
__global__ __launch_bounds__(kBlock) void k_fused_spec(
    FinalArgs a, SpecArgs sa, const sga_segment* __restrict__ segs, int n_segs,
    SelState* __restrict__ st, const SelState* __restrict__ aux,
    const int32_t* __restrict__ seg_dir) {
  __shared__ uint32_t s_hi[kChunksPerBlock], s_nf[kChunksPerBlock];
  __shared__ SpecLds s_lds[kChunksPerBlock];
  // the sample's own count of keys inside the bracket predicts the records
  const SelState hi = aux[0], lo = aux[1];
  if (lo.skip) return;                                   // open below: nothing bounds the records
  const double in_bracket = (double)(lo.k - lo.need + lo.n_eq) - (hi.skip ? 0.0 : (double)(hi.k - hi.need));
  if (in_bracket * sa.n_over_ns > sa.est_limit) return;  // plateau inside the bracket: stand back
  const uint32_t T_HI = hi.skip ? 0x80000000u : hi.thresh_bits + 1u;
  const uint32_t T_LO = lo.thresh_bits;
  const uint32_t T_MID = spec_mid(T_LO, T_HI);
  if (blockIdx.x == 0 && threadIdx.x == 0) { st->t_lo = T_LO; st->t_hi = T_HI; st->spec = 1u; }
  const int64_t n_chunks = cdiv64(a.n, kChunk);
  const unsigned blk = a.pack_extra != 0 ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
  const int64_t c = (int64_t)blk * kChunksPerBlock + wave_id();
  uint32_t chi = 0, tot_nf = 0;
  if (c < n_chunks) {
    uint32_t mycnt = 0, s_run = 0;
    SpecLds& lds = s_lds[wave_id()];
    SegCursor sc;
    sc.init(segs, n_segs, seg_dir);
    const int64_t sh = pack_shift<true>(c << 10, a.pack_extra);
    const float* const R = a.r + sh;
    const float* const P = a.p + sh;
    const float* const M = a.m + sh;
    const float* const V = a.v + sh;
    sc.seek_uniform(uniform_i64(c) * kChunk);
#define SGA_SPEC_SLAB(FULLP, IT) \
    spec_slab<BF16G, BF16V, SCORE, FULLP>(a, sa, st, c, IT, T_LO, T_MID, T_HI, sc, chi, s_run, tot_nf, mycnt, lds, R, P, M, V, sh)
    if (a.vec && (c + 1) * kChunk <= a.n) {
      SGA_SPEC_SLAB(true, 0); SGA_SPEC_SLAB(true, 1); SGA_SPEC_SLAB(true, 2); SGA_SPEC_SLAB(true, 3);
    } else {
      SGA_SPEC_SLAB(false, 0); SGA_SPEC_SLAB(false, 1); SGA_SPEC_SLAB(false, 2); SGA_SPEC_SLAB(false, 3);
    }
#undef SGA_SPEC_SLAB
    __builtin_amdgcn_wave_barrier();
    if (lane_id() < kPlaneWordsPerChunk) {
      sa.splane[c * kPlaneWordsPerChunk + lane_id()] = lds.splane[lane_id()];
      sa.fplane[c * kPlaneWordsPerChunk + lane_id()] = lds.splane[lane_id()];
    }
    if (lane_id() == 0) { sa.tile_gt[c] = chi; sa.tile_eq[c] = 0u; }
    if (mycnt) {                                        // wave-uniform
      // The chunk's LDS records go, in one piece, to the segment its chunk index hashes to
      // (neighbouring waves, which run at the same time, hit different counters: with one
      // segment per range of consecutive chunks the sweep was 0.25 ms slower); when they do not
      // fit there, to the shared overflow list.  A reservation is never taken back: the counter
      // only grows, so once one reservation has failed every later one fails as well, and the
      // records of the segment are exactly [0, base of the first failure) -- which the failing
      // wave leaves in seg_fail (the smallest failing base wins) for the check to clamp the
      // segment to.  (Taking the reservation back instead let a third wave slip into the gap
      // between two failed ones and left unwritten slots inside the counted range.)
      const uint32_t seg = (uint32_t)c & (uint32_t)(kSegWaves - 1);
      uint32_t base = 0;
      if (lane_id() == 0) {
        base = atomicAdd(&sa.seg_cnt[seg], mycnt);
        if (base + mycnt > sa.seg_cap) {
          if (base <= sa.seg_cap) atomicMax(&sa.seg_fail[seg], 0xFFFFFFFFu - base);
          base = 0xFFFFFFFFu;
        }
      }
      base = __shfl(base, 0, kWave);
      uint32_t* g_idx = sa.seg_idx + (int64_t)seg * sa.seg_cap;
      uint32_t* g_key = sa.seg_key + (int64_t)seg * sa.seg_cap;
      F4* g_rec = sa.seg_rec + (int64_t)seg * sa.seg_cap;
      bool room = true;
      if (base == 0xFFFFFFFFu) {
        if (lane_id() == 0) base = atomicAdd(sa.ovf_cnt, mycnt);
        base = __shfl(base, 0, kWave);
        room = base + mycnt <= sa.ovf_cap;
        g_idx = sa.ovf_idx; g_key = sa.ovf_key; g_rec = sa.ovf_rec;
      }
      if (room)
        for (uint32_t j = lane_id(); j < mycnt; j += kWave) {
          g_idx[base + j] = lds.idx[j]; g_key[base + j] = lds.key[j]; g_rec[base + j] = lds.rec[j];
        }
    }
  }
  if (lane_id() == 0) { s_hi[wave_id()] = chi; s_nf[wave_id()] = tot_nf; }
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t h = s_hi[0] + s_hi[1] + s_hi[2] + s_hi[3];
    const uint32_t f = s_nf[0] + s_nf[1] + s_nf[2] + s_nf[3];
    if (h) atomicAdd(&sa.hi_part[blockIdx.x & (kSweepParts - 1)], h);
    if (f) atomicAdd(&sa.nf_part[blockIdx.x & (kSweepParts - 1)], f);
  }
}

// Ties at the threshold are granted in index order.  After the tile scan
// tile_eq[c] counts the ties before chunk c, so only the one chunk where the
// quota runs out has to rank its ties: this pass gathers that chunk's ties
// (at most 1024) so the settlement can rank them wherever their records lie.
constexpr int kSpecTieCap = 1024;
static __global__ __launch_bounds__(kBlock) void k_spec_ties(
    const SelState* __restrict__ st, const uint32_t* __restrict__ cand_idx,
    const uint32_t* __restrict__ cand_key, const uint32_t* __restrict__ tile_eq,
    int64_t n_tiles, uint32_t* __restrict__ tie_cnt, uint32_t* __restrict__ tie_idx) {
  if (!st->bracket_ok || !st->spec) return;
  const uint32_t T = st->thresh_bits, nc = st->cand_count, n_eq = st->n_eq, need = st->need;
  if (need >= n_eq) return;                              // every tie is taken
  for (uint32_t j = blockIdx.x * kBlock + threadIdx.x; j < nc; j += gridDim.x * kBlock) {
    if (cand_key[j] != T) continue;
    const uint32_t idx = cand_idx[j], c = idx >> 10;
    const uint32_t before = tile_eq[c];
    const uint32_t upto = (int64_t)c + 1 < n_tiles ? tile_eq[c + 1] : n_eq;
    if (before < need && upto > need) {
      const uint32_t at = atomicAdd(tie_cnt, 1u);
      if (at < (uint32_t)kSpecTieCap) tie_idx[at] = idx;
    }
  }
}

// Settlement: the exact selection of every recorded coordinate against the
// sweep's guess; where they differ the F plane is patched.
static __global__ __launch_bounds__(kBlock) void k_spec_settle(
    const SelState* __restrict__ st, const uint32_t* __restrict__ cand_idx,
    const uint32_t* __restrict__ cand_key, const uint32_t* __restrict__ tile_eq,
    int64_t n_tiles, const uint32_t* __restrict__ tie_cnt, const uint32_t* __restrict__ tie_idx,
    uint32_t* __restrict__ fplane) {
  if (!st->bracket_ok || !st->spec) return;
  const uint32_t T = st->thresh_bits, nc = st->cand_count, n_eq = st->n_eq, need = st->need;
  const uint32_t T_MID = spec_mid(st->t_lo, st->t_hi);
  for (uint32_t j = blockIdx.x * kBlock + threadIdx.x; j < nc; j += gridDim.x * kBlock) {
    const uint32_t key = cand_key[j];
    const uint32_t idx = cand_idx[j];
    bool on = key >= T;
    if (key == T && need < n_eq) {
      const uint32_t c = idx >> 10;
      const uint32_t before = tile_eq[c];
      const uint32_t upto = (int64_t)c + 1 < n_tiles ? tile_eq[c + 1] : n_eq;
      if (before >= need) {
        on = false;
      } else if (upto > need) {            // the quota ends inside this chunk
        uint32_t rank = before;
        const uint32_t nt = *tie_cnt < (uint32_t)kSpecTieCap ? *tie_cnt : (uint32_t)kSpecTieCap;
        for (uint32_t t = 0; t < nt; ++t) rank += tie_idx[t] < idx;
        on = rank < need;
      }
    }
    if (on != (key >= T_MID)) {
      const uint32_t lane = (idx >> 2) & 63u, e = idx & 3u;
      uint32_t* w = &fplane[(idx >> 8) * 8 + 2 * e + (lane >> 5)];
      if (on) atomicOr(w, 1u << (lane & 31));
      else atomicAnd(w, ~(1u << (lane & 31)));
    }
  }
}

// Selected coordinates before element `idx` inside its 256-element slab of a
// bit plane: the lanes below its lane over the four ballots, plus its lane's
// earlier elements.
__device__ __forceinline__ uint32_t slab_rank_before(const uint32_t* __restrict__ plane, uint32_t idx) {
  const uint32_t lane0 = (idx >> 2) & 63u, e0 = idx & 3u;
  const U4* wp = reinterpret_cast<const U4*>(plane + (int64_t)(idx >> 8) * 8);
  const U4 x0 = wp[0], x1 = wp[1];
  const uint32_t w[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
  const uint64_t below = lane0 ? (~0ull >> (64 - lane0)) : 0ull;
  uint32_t rank = 0;
#pragma unroll
  for (uint32_t e = 0; e < 4; ++e) {
    const uint64_t m = ((uint64_t)w[2 * e + 1] << 32) | (uint64_t)w[2 * e];
    rank += (uint32_t)__popcll(m & below);
    if (e < e0) rank += (uint32_t)((m >> lane0) & 1ull);
  }
  return rank;
}

// Pack entries of the coordinates the sweep took as selected and the exact
// selection keeps (S & F), from the staging array.  One LANE per 256-element
// slab (a wave per slab spends a whole wave's ballot arithmetic on the two or
// three entries a slab holds at 1 %), one wave per workgroup: the lane reads
// its slab's 8 + 8 plane words, takes its starts inside the chunk from its
// three neighbours (a chunk is four consecutive lanes), then walks its set
// bits in index order.  The 64 slabs of a wave fill ONE contiguous run of the
// pack, so the entries go through LDS, a window of kPackWindow positions at a
// time, and leave as whole coalesced lines (a lane writing its own few entries
// straight to memory leaves every line half written when it is evicted: 4 ms
// instead of 0.3 at 10 %).  Positions of coordinates the repair pass adds
// (F without S) stay untouched: the window is pre-filled with a sentinel.
// slab_pos[slab] = pack position of the slab's first selected coordinate.
constexpr int kPackWindow = 512;
constexpr int kPackDenseCut = 32;         // k above n / this: a lane per quarter slab
constexpr int kPackAhead = 8;             // staged values a lane requests before it walks its bits
template <bool BF16V, int SUB>
__global__ __launch_bounds__(kBlock) void k_spec_pack(
    FinalArgs a, const SelState* __restrict__ st, const void* __restrict__ stage,
    const uint32_t* __restrict__ splane, const uint32_t* __restrict__ fplane,
    const uint32_t* __restrict__ tile_sel, uint32_t* __restrict__ slab_pos) {
  // Four independent waves per workgroup, each with LDS of its own and no workgroup barrier.
  // What the kernel costs is memory: both planes (n / 4 bytes), one line per chunk of the
  // chunk-strided staging array, the pack -- 0.54 GB at 1 % of 1.2e9 elements for 0.16 ms;
  // a third fewer vector instructions (single-bit extracts on 32-bit halves, staged values
  // picked from LDS by their running number) and a quarter of the workgroup launches left
  // that time where it was.
  __shared__ uint32_t s_idx[kChunksPerBlock][kPackWindow + 4];
  __shared__ uint32_t s_val[kChunksPerBlock][kPackWindow + 4];
  __shared__ uint32_t s_ahead[kChunksPerBlock][kPackAhead * kWave];
  if (!st->bracket_ok || !st->spec) return;
  uint32_t* const l_idx = s_idx[wave_id()];
  uint32_t* const l_val = s_val[wave_id()];
  uint32_t* const l_ahead = s_ahead[wave_id()];
  const int64_t n_slabs = cdiv64(a.n, kChunk) * kChunkIters;
  const int64_t part = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t slab = part / SUB;
  const bool live = slab < n_slabs;
  uint64_t S[4] = {0, 0, 0, 0}, F[4] = {0, 0, 0, 0};
  uint32_t base = 0;
  if (live) {
    const U4* ws = reinterpret_cast<const U4*>(splane + slab * 8);
    const U4* wf = reinterpret_cast<const U4*>(fplane + slab * 8);
    const U4 x0 = ws[0], x1 = ws[1], y0 = wf[0], y1 = wf[1];
    base = tile_sel[slab >> 2];
    S[0] = ((uint64_t)x0.y << 32) | x0.x; S[1] = ((uint64_t)x0.w << 32) | x0.z;
    S[2] = ((uint64_t)x1.y << 32) | x1.x; S[3] = ((uint64_t)x1.w << 32) | x1.z;
    F[0] = ((uint64_t)y0.y << 32) | y0.x; F[1] = ((uint64_t)y0.w << 32) | y0.z;
    F[2] = ((uint64_t)y1.y << 32) | y1.x; F[3] = ((uint64_t)y1.w << 32) | y1.z;
    if (SUB > 1) {                             // this lane's run of lane positions of the slab
      constexpr int kBits = kWave / SUB;
      const uint64_t own = (~0ull >> (64 - kBits)) << ((uint32_t)(part % SUB) * kBits);
#pragma unroll
      for (int e = 0; e < 4; ++e) { S[e] &= own; F[e] &= own; }
    }
  }
  const uint32_t cntS = (uint32_t)(__popcll(S[0]) + __popcll(S[1]) + __popcll(S[2]) + __popcll(S[3]));
  const uint32_t cntF = (uint32_t)(__popcll(F[0]) + __popcll(F[1]) + __popcll(F[2]) + __popcll(F[3]));
  // counts of the chunk's earlier lanes (a chunk is kChunkIters * SUB consecutive lanes)
  constexpr int kGroup = kChunkIters * SUB;
  uint32_t ps = cntS, pf = cntF;
#pragma unroll
  for (int o = 1; o < kGroup; o <<= 1) {
    const uint32_t ts = __shfl_up(ps, o, kWave), tf = __shfl_up(pf, o, kWave);
    if ((lane_id() & (kGroup - 1)) >= o) { ps += ts; pf += tf; }
  }
  ps -= cntS;
  pf -= cntF;
  const uint32_t f_start = base + pf;
  if (live && part % SUB == 0) slab_pos[slab] = f_start;
  // the wave's run of the pack: [F0, F0 + len)
  const uint32_t F0 = __shfl(f_start, 0, kWave);
  uint32_t end = live ? f_start + cntF : 0u;
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) { const uint32_t t = __shfl_xor(end, o, kWave); end = t > end ? t : end; }
  const uint32_t len = end - F0;
  const int64_t c = slab >> 2;
  // every lane position that holds a coordinate of either plane is visited, in index order, so
  // the positions in the staged run (S) and in the pack (F) are running counts
  uint64_t U = S[0] | S[1] | S[2] | S[3] | F[0] | F[1] | F[2] | F[3];
  uint32_t sr = 0, fr = f_start;
  // the lane's first staged values, all requested before the first is used (its run of the
  // staging array is contiguous) and parked in LDS, where the walk below picks them up by
  // their running number; a slab with more entries loads the rest as it goes
  {
    uint32_t ahead[kPackAhead];
#pragma unroll
    for (int t = 0; t < kPackAhead; ++t) {
      ahead[t] = 0u;
      if ((uint32_t)t < cntS) {
        if (BF16V) ahead[t] = reinterpret_cast<const uint16_t*>(stage)[c * kChunk + ps + t];
        else ahead[t] = reinterpret_cast<const uint32_t*>(stage)[c * kChunk + ps + t];
      }
    }
#pragma unroll
    for (int t = 0; t < kPackAhead; ++t) l_ahead[t * kWave + lane_id()] = ahead[t];
  }
  // the planes as 32-bit halves: a lane position's four S bits and four F bits are then eight
  // single-bit field extracts (lane positions differ from lane to lane, so 64-bit shifts by a
  // per-lane amount would run on the vector unit, two instructions each)
  const uint32_t s_lo[4] = {(uint32_t)S[0], (uint32_t)S[1], (uint32_t)S[2], (uint32_t)S[3]};
  const uint32_t s_hi[4] = {(uint32_t)(S[0] >> 32), (uint32_t)(S[1] >> 32), (uint32_t)(S[2] >> 32),
                            (uint32_t)(S[3] >> 32)};
  const uint32_t f_lo[4] = {(uint32_t)F[0], (uint32_t)F[1], (uint32_t)F[2], (uint32_t)F[3]};
  const uint32_t f_hi[4] = {(uint32_t)(F[0] >> 32), (uint32_t)(F[1] >> 32), (uint32_t)(F[2] >> 32),
                            (uint32_t)(F[3] >> 32)};
  for (uint32_t w0 = 0; w0 < len; w0 += kPackWindow) {
    const uint32_t wlen = len - w0 < (uint32_t)kPackWindow + 3u ? len - w0 : (uint32_t)kPackWindow + 3u;
    for (uint32_t t = lane_id(); t < wlen; t += kWave) l_idx[t] = 0xFFFFFFFFu;
    __builtin_amdgcn_wave_barrier();       // the wave's own LDS: its accesses stay in order
    while (U) {
      const int L = __ffsll((unsigned long long)U) - 1;
      if (fr - F0 >= w0 + (uint32_t)kPackWindow) break;     // belongs to a later window
      U &= U - 1;
      const bool upper = L >= 32;
      const uint32_t l = (uint32_t)L & 31u;
      uint32_t ns = 0, nf = 0;                              // the position's S and F bits, bit e = element e
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ns |= (((upper ? s_hi[e] : s_lo[e]) >> l) & 1u) << e;
        nf |= (((upper ? f_hi[e] : f_lo[e]) >> l) & 1u) << e;
      }
      uint32_t both = ns & nf;
      while (both) {
        const uint32_t e = (uint32_t)__ffs((int)both) - 1u;
        both &= both - 1u;
        const uint32_t lower = (1u << e) - 1u;
        const uint32_t srq = sr + (uint32_t)__popc(ns & lower);
        const uint32_t t = fr + (uint32_t)__popc(nf & lower) - F0 - w0;
        l_idx[t] = (uint32_t)(slab * (kWave * kVec) + L * kVec) + e;
        uint32_t val;
        if (srq < (uint32_t)kPackAhead) val = l_ahead[srq * kWave + lane_id()];
        else if (BF16V) val = reinterpret_cast<const uint16_t*>(stage)[c * kChunk + ps + srq];
        else val = reinterpret_cast<const uint32_t*>(stage)[c * kChunk + ps + srq];
        l_val[t] = val;
      }
      sr += (uint32_t)__popc(ns);
      fr += (uint32_t)__popc(nf);
    }
    __builtin_amdgcn_wave_barrier();       // the wave's own LDS: its accesses stay in order
    for (uint32_t t = lane_id(); t < wlen; t += kWave) {
      const uint32_t ix = l_idx[t];
      const int64_t pos = (int64_t)F0 + w0 + t;
      if (ix != 0xFFFFFFFFu && pos < a.k) {
        a.idx_out[pos] = (int32_t)ix;
        if (BF16V) reinterpret_cast<uint16_t*>(a.values_out)[pos] = (uint16_t)l_val[t];
        else reinterpret_cast<uint32_t*>(a.values_out)[pos] = l_val[t];
      }
    }
    __builtin_amdgcn_wave_barrier();       // the wave's own LDS: its accesses stay in order
  }
}

// Repair: the recorded coordinates whose guess was wrong are committed again,
// from their records, the way the exact selection says; the newly selected
// ones also get their pack entry.
template <bool BF16V>
__global__ __launch_bounds__(kBlock) void k_spec_repair(
    FinalArgs a, const sga_segment* __restrict__ segs, int n_segs,
    const int32_t* __restrict__ seg_dir, const SelState* __restrict__ st,
    const uint32_t* __restrict__ cand_idx, const uint32_t* __restrict__ cand_key,
    const F4* __restrict__ cand_rec, const uint32_t* __restrict__ fplane,
    const uint32_t* __restrict__ slab_pos) {
  if (!st->bracket_ok || !st->spec) return;
  const uint32_t nc = st->cand_count;
  const uint32_t T_MID = spec_mid(st->t_lo, st->t_hi);
  SegCursor lc;
  lc.init(segs, n_segs, seg_dir);
  for (uint32_t j = blockIdx.x * kBlock + threadIdx.x; j < nc; j += gridDim.x * kBlock) {
    const uint32_t idx = cand_idx[j];
    const uint32_t lane = (idx >> 2) & 63u, e = idx & 3u;
    const bool on = (fplane[(idx >> 8) * 8 + 2 * e + (lane >> 5)] >> (lane & 31)) & 1u;
    if (on == (cand_key[j] >= T_MID)) continue;          // the sweep's commit stands
    const F4 rec = cand_rec[j];
    lc.seek((int64_t)idx);
    Hyper h = lc.h;
    if (a.adams) { h.bc1 = 1.0f; h.bc2 = 1.0f; }
    float ge = 0.0f, val = 0.0f;
    uint16_t hb = 0;
    if (on) ge = spec_value<BF16V>(a, rec.x, hb, val);
    const float ve = a.adams ? rec.z * rec.z : rec.w;
    const Commit cm = adamw_commit(rec.y, ge, rec.z, ve, h);
    const float pe = rec.y - h.lr * cm.upd;
    float rn = on ? 0.0f : rec.x;
    if (a.fold) rn = __fdiv_rn(rn, a.interval);
    const int64_t at = (int64_t)idx + pack_shift<false>((int64_t)idx, a.pack_extra);
    a.ro[at] = rn;
    a.po[at] = pe;
    a.mo[at] = cm.m_new;
    a.vo[at] = cm.v_new;
    if (on) {
      const uint32_t pos = slab_pos[idx >> 8] + slab_rank_before(fplane, idx);
      if ((int64_t)pos < a.k) {
        a.idx_out[pos] = (int32_t)idx;
        if (BF16V) reinterpret_cast<uint16_t*>(a.values_out)[pos] = hb;
        else reinterpret_cast<float*>(a.values_out)[pos] = val;
      }
    }
  }
}

// Overflow list -> tail of the dense candidate list (behind the segments' records).
static __global__ __launch_bounds__(kBlock) void k_spec_ovf_compact(
    const SelState* __restrict__ aux, const uint32_t* __restrict__ seg_off,
    const uint32_t* __restrict__ ovf_idx, const uint32_t* __restrict__ ovf_key,
    const F4* __restrict__ ovf_rec, uint32_t ovf_cap, uint32_t* __restrict__ cand_idx,
    uint32_t* __restrict__ cand_key, F4* __restrict__ cand_rec, uint32_t* __restrict__ tie_cnt) {
  if (blockIdx.x == 0 && threadIdx.x == 0) *tie_cnt = 0u;     // the tie list of this step starts empty
  if (aux->skip) return;
  const uint32_t off = seg_off[kSegWaves];
  uint32_t cnt = seg_off[kSegWaves + 1];
  if (cnt > ovf_cap) cnt = ovf_cap;
  for (uint32_t j = blockIdx.x * kBlock + threadIdx.x; j < cnt; j += gridDim.x * kBlock) {
    cand_idx[off + j] = ovf_idx[j];
    cand_key[off + j] = ovf_key[j];
    cand_rec[off + j] = ovf_rec[j];
  }
}

// Extra workspace of the single-sweep step: [dplane: 128 B per chunk | records: 16 B per
// candidate slot | staging: one pack value per coordinate, chunk-strided].
struct SpecWorkspace {
  uint32_t* dplane;
  uint32_t* slab_pos;
  F4* seg_rec;
  F4* cand_rec;
  uint32_t* ovf_idx;
  uint32_t* ovf_key;
  F4* ovf_rec;
  int64_t ovf_cap;
  uint32_t* tie_cnt;      // [0]: ties gathered; tie_idx follows
  uint32_t* tie_idx;
  uint32_t* seg_fail;     // kSegWaves words
  void* stage;
};
static inline size_t spec_ws_bytes(int64_t n, int val_bytes) {
  const int64_t nt = cdiv64(n, kChunk) + 8;
  // records of the segments (16 B), dense records (16 B), overflow list (24 B, half the capacity)
  size_t b = (size_t)nt * (128 + 16) + (size_t)kSegWaves * fast_seg_cap(nt * kChunk) * (16 * 2 + 12) +
             (size_t)nt * kChunk * val_bytes + 4096 + 8192 + (size_t)kSegWaves * 4;
  return (b + 255) & ~(size_t)255;
}
static inline bool spec_ws_carve(void* ws, size_t bytes, int64_t n, int val_bytes, int64_t seg_cap,
                                 SpecWorkspace* out) {
  if (!ws || (reinterpret_cast<uintptr_t>(ws) & 255) || bytes < spec_ws_bytes(n, val_bytes)) return false;
  const int64_t nt = cdiv64(n, kChunk) + 8;
  char* p = reinterpret_cast<char*>(ws);
  out->dplane = reinterpret_cast<uint32_t*>(p);
  p += (size_t)nt * 128;
  out->slab_pos = reinterpret_cast<uint32_t*>(p);
  p += (size_t)nt * 16;
  p = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(p) + 255) & ~(uintptr_t)255);
  out->seg_rec = reinterpret_cast<F4*>(p);
  p += (size_t)kSegWaves * seg_cap * 16;
  p = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(p) + 255) & ~(uintptr_t)255);
  out->cand_rec = reinterpret_cast<F4*>(p);
  p += (size_t)kSegWaves * seg_cap * 16;
  p = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(p) + 255) & ~(uintptr_t)255);
  out->ovf_cap = (int64_t)kSegWaves * seg_cap / 2;
  out->ovf_rec = reinterpret_cast<F4*>(p);
  p += (size_t)out->ovf_cap * 16;
  out->ovf_idx = reinterpret_cast<uint32_t*>(p);
  p += (size_t)out->ovf_cap * 4;
  out->ovf_key = reinterpret_cast<uint32_t*>(p);
  p += (size_t)out->ovf_cap * 4;
  p = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(p) + 255) & ~(uintptr_t)255);
  out->tie_cnt = reinterpret_cast<uint32_t*>(p);
  out->tie_idx = out->tie_cnt + 64;
  p += 256 + (size_t)kSpecTieCap * 4;
  p = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(p) + 255) & ~(uintptr_t)255);
  out->seg_fail = reinterpret_cast<uint32_t*>(p);
  p += (size_t)kSegWaves * 4;
  out->stage = p;
  return true;
}

// Margin of the single-sweep bracket, in standard deviations of the sample rank.
constexpr double kSpecSigmas = 12.0;
// Out of place a missed bracket costs a redo (three more sweeps), not the state: the margin only
// has to make that rare, and it is the margin of the two-sweep step, which can fall back as
// well.  Measured on row-sparse gradients (whole rows of 2 K to 16 K coordinates active or
// zero, so that the four keys of a sampled quad are one draw), 2400 sample seeds per margin:
// no miss at 3, 4, 5 or 6 sigma, 22 at 2 sigma, each redone to the exact step (the strata of the
// sample make its rank tighter than the binomial the margin is computed for).  The sweep records
// 1.25 M coordinates at 1 % of 1.2e9 instead of the 3 M of the in-place step's 12 sigma, and
// the kernels behind it take 0.59 instead of 0.69 ms.
constexpr double kSpecSigmasOut = 5.0;

template <bool BF16G, bool BF16V, int SCORE>
static int run_fused_spec(const void* g, float* resid, float* p, float* m, float* v, int64_t n,
                          int64_t k, const sga_segment* segs, int n_segs, int32_t* idx_out,
                          void* values_out, uint8_t* mask_out, float factor, float coeff,
                          int flags, float interval, uint32_t seed, sga_select_result* result,
                          const SelWorkspace& w, const SpecWorkspace& x, hipStream_t s,
                          int64_t pack_extra, float* const* out = nullptr) {
  // out: resid / p / m / v of the NEW state when the step runs out of place (the inputs stay
  // untouched, so a bracket that missed is redone by the radix passes and the key-forming final
  // sweep like a sweep that stood back); null: in place
  const bool vec = aligned4(g, BF16G ? 2 : 4) && aligned4(resid, 4) && aligned4(p, 4) &&
                   aligned4(m, 4) && aligned4(v, 4) &&
                   (!out || (aligned4(out[0], 4) && aligned4(out[1], 4) && aligned4(out[2], 4) &&
                             aligned4(out[3], 4)));
  const int adams = (flags & SGA_GC_ADAMS) ? 1 : 0;
  SrcFused<BF16G, SCORE> src{g, resid, p, m, v, vec, {}, pack_extra, adams};
  launch_seg_dir(segs, n_segs, n, w.seg_dir, s);
  src.sc.init(segs, n_segs, w.seg_dir);
  const int64_t n_tiles = cdiv64(n, kChunk);
  FinalArgs fa;
  fa.g = g; fa.r = resid; fa.p = p; fa.m = m; fa.v = v; fa.n = n; fa.k = k;
  fa.ro = out ? out[0] : resid; fa.po = out ? out[1] : p;
  fa.mo = out ? out[2] : m; fa.vo = out ? out[3] : v;
  fa.idx_out = idx_out; fa.values_out = values_out; fa.mask_out = mask_out;
  fa.factor = factor; fa.coeff = coeff; fa.T = 0; fa.need = 0;
  fa.vec = vec; fa.mvec = aligned4(mask_out, 1);
  fa.scale = factor != 1.0f; fa.apply_coeff = coeff != 1.0f;
  fa.pack_extra = pack_extra;
  fa.adams = adams != 0; fa.fold = (flags & SGA_GC_FOLD) != 0; fa.interval = interval;
  fa.planes = w.pbits;
  // sample -> bracket with the wide margins (the chain kernels as a batch of one)
  SrcPack<SrcFused<BF16G, SCORE>> srcs = {};
  srcs.s[0] = src;
  SelBatch B;
  ChainJob& J = B.add(w, n, k, 0);
  J.seed = seed; J.spec = out ? 2 : 1; J.ovf_cap = (uint32_t)x.ovf_cap; J.seg_fail = x.seg_fail;
  J.seg_rec = x.seg_rec; J.cand_rec = x.cand_rec; J.result = result;
  const int64_t ns = J.n_sv * 4;
  hipLaunchKernelGGL(k_chain_begin, B.grid(1), dim3(kBlock), 0, s, B.jobs, 1,
                     out ? kSpecSigmasOut : kSpecSigmas);
  hipLaunchKernelGGL((k_sample<SrcFused<BF16G, SCORE>>), B.grid(stream_grid(B.max_nsv, kBlock)),
                     dim3(kBlock), 0, s, srcs, B.jobs);
  for (int level = 0; level < 3; ++level) launch_level_raw<false>(B, level, s, kRawKeyBlocks);
  // the sweep
  SpecArgs sa;
  sa.splane = w.pbits; sa.fplane = x.dplane; sa.stage = x.stage;
  sa.seg_idx = w.seg_idx; sa.seg_key = w.seg_key; sa.seg_rec = x.seg_rec; sa.seg_cnt = w.seg_cnt;
  sa.seg_fail = x.seg_fail;
  sa.seg_cap = (uint32_t)w.seg_cap;
  sa.tile_gt = w.tile_gt; sa.tile_eq = w.tile_eq; sa.hi_part = w.blk_gt; sa.nf_part = w.blk_eq;
  sa.ovf_idx = x.ovf_idx; sa.ovf_key = x.ovf_key; sa.ovf_rec = x.ovf_rec;
  sa.ovf_cnt = w.seg_cnt + kSegWaves + 1; sa.ovf_cap = (uint32_t)x.ovf_cap;
  sa.n_over_ns = (double)n / (double)ns;
  sa.est_limit = 0.5 * (double)kSegWaves * (double)w.seg_cap;
  const dim3 one_shot((unsigned)cdiv64(n_tiles, kChunksPerBlock));
  ProfPair* pp = prof_begin(SGA_PROF_FUSED_FINAL, s);
  hipLaunchKernelGGL((k_fused_spec<BF16G, BF16V, SCORE>), one_shot, dim3(kBlock), 0, s, fa, sa, segs,
                     n_segs, w.st, w.aux, w.seg_dir);
  prof_end(pp, s);
  hipLaunchKernelGGL(k_bracket_check, B.grid(1), dim3(kBlock), 0, s, B.jobs);
  hipLaunchKernelGGL(k_cand_compact, B.grid(kSegWaves / kChunksPerBlock), dim3(kBlock), 0, s, B.jobs);
  hipLaunchKernelGGL(k_spec_ovf_compact, dim3(64), dim3(kBlock), 0, s, w.aux, w.seg_cnt, x.ovf_idx,
                     x.ovf_key, x.ovf_rec, (uint32_t)x.ovf_cap, w.cand_idx, w.cand_key, x.cand_rec,
                     x.tie_cnt);
  for (int level = 0; level < 3; ++level) launch_level_raw<true>(B, level, s, 3 * kRawKeyBlocks);
  hipLaunchKernelGGL(k_cand_tiles, B.grid(512), dim3(kBlock), 0, s, B.jobs);
  // only when the sweep stood back: the radix passes over the untouched data
  for (int level = 0; level < 3; ++level)
    launch_level_data<SrcFused<BF16G, SCORE>, true>(srcs, B, level, s);
  launch_tile_count(srcs, B, 0, s);
  launch_tile_scan(B, s);
  hipLaunchKernelGGL(k_spec_ties, dim3(512), dim3(kBlock), 0, s, w.st, w.cand_idx, w.cand_key,
                     w.tile_eq, n_tiles, x.tie_cnt, x.tie_idx);
  hipLaunchKernelGGL(k_spec_settle, dim3(512), dim3(kBlock), 0, s, w.st, w.cand_idx, w.cand_key,
                     w.tile_eq, n_tiles, x.tie_cnt, x.tie_idx, x.dplane);
  // a lane per slab, or per quarter of one where a slab holds more entries than a lane has
  // staged values in flight
  if (k > n / kPackDenseCut)
    hipLaunchKernelGGL((k_spec_pack<BF16V, 4>), dim3((unsigned)cdiv64(n_tiles * kChunkIters * 4, kBlock)),
                       dim3(kBlock), 0, s, fa, w.st, x.stage, w.pbits, x.dplane, w.tile_gt, x.slab_pos);
  else
    hipLaunchKernelGGL((k_spec_pack<BF16V, 1>), dim3((unsigned)cdiv64(n_tiles * kChunkIters, kBlock)),
                       dim3(kBlock), 0, s, fa, w.st, x.stage, w.pbits, x.dplane, w.tile_gt, x.slab_pos);
  hipLaunchKernelGGL((k_spec_repair<BF16V>), dim3(1024), dim3(kBlock), 0, s, fa, segs, n_segs,
                     w.seg_dir, w.st, w.cand_idx, w.cand_key, x.cand_rec, x.dplane, x.slab_pos);
  if (mask_out)
    hipLaunchKernelGGL(k_expand_mask, dim3(stream_grid(n_tiles, kChunksPerBlock, 1 << 22)), dim3(kBlock),
                       0, s, w.st, x.dplane, n, mask_out, (reinterpret_cast<uintptr_t>(mask_out) & 15) == 0);
  // the sweep stood back: the key-forming final sweep does the step (a small grid that strides
  // over the chunks; it returns at once otherwise)
  hipLaunchKernelGGL((k_fused_final<BF16G, BF16V, SCORE, false>),
                     dim3(stream_grid(n_tiles, kChunksPerBlock, 2048)), dim3(kBlock), 0, s, fa,
                     segs, n_segs, w.st, w.tile_gt, w.tile_eq, 3, w.seg_dir);
  launch_result(B, s);
  return check_launch("sga_fused_sparse_step_single_sweep");
}

}  // namespace sga

using namespace sga;

extern "C" size_t sga_fused_workspace_bytes(int64_t n) { return sel_ws_bytes(n < 0 ? 0 : n); }

static int fused_entry(const char* who, const void* g, int g_dtype, float* resid, float* p,
                       float* m, float* v, int64_t pack_extra, int64_t n, int64_t k,
                       const sga_segment* segs, int n_segs, int score_id, int32_t* idx_out,
                       void* values_out, int values_dtype, uint8_t* mask_out, float factor,
                       float coeff, int fast, int flags, float interval, sga_select_result* result,
                       void* ws, size_t ws_bytes, void* stream, bool single = false,
                       void* ws2 = nullptr, size_t ws2_bytes = 0, uint32_t seed = 0u,
                       float* const* out = nullptr) {
  if ((flags & ~(SGA_GC_ADAMS | SGA_GC_FOLD)) != 0) {
    // the dual-lr split belongs to full steps (adamw.py:570-580); HAS_MASK / CLEAR / APPLY_COEFF
    // are what this step does anyway (coeff != 1 applies the coefficient)
    set_error("%s: flags may carry SGA_GC_ADAMS and SGA_GC_FOLD only (got %d); the boundary "
              "dual-lr split requires a full step", who, flags);
    return SGA_ERR_ARG;
  }
  if ((flags & SGA_GC_FOLD) && !(interval > 0.0f)) {
    set_error("%s: SGA_GC_FOLD needs interval > 0 (got %g)", who, (double)interval);
    return SGA_ERR_ARG;
  }
  if (!g && (g_dtype != SGA_F32 || score_id == SGA_SCORE_ABS_G_BLIND)) {
    // no separate gradient: resid already holds g + r (the reference's own buffer contract)
    set_error("%s: g may be NULL only with g_dtype SGA_F32 (resid then holds g + r already), and "
              "not for the residual-blind score, which ranks the step's own gradient", who);
    return SGA_ERR_ARG;
  }
  if (!resid || !p || !m || !v || !segs || !idx_out || !values_out || n < 1 ||
      n >= (1ll << 31) || k < 1 || k > n || n_segs < 1 ||
      (g_dtype != SGA_F32 && g_dtype != SGA_BF16) ||
      (values_dtype != SGA_F32 && values_dtype != SGA_BF16) || score_id < 0 ||
      score_id > SGA_SCORE_GR_OVER_SQRT_V) {
    set_error("%s: bad argument (n=%lld k=%lld n_segs=%d score=%d; need 1 <= k <= n < 2^31)", who,
              (long long)n, (long long)k, n_segs, score_id);
    return SGA_ERR_ARG;
  }
  SelWorkspace w;
  if (!sel_ws_carve(ws, ws_bytes, cdiv64(n, kChunk), &w)) {
    set_error("%s: workspace missing, misaligned or smaller than "
              "sga_fused_workspace_bytes(n)=%zu", who, sel_ws_bytes(n));
    return SGA_ERR_WORKSPACE;
  }
  hipStream_t s = (hipStream_t)stream;
  const bool bg = g_dtype == SGA_BF16, bv = values_dtype == SGA_BF16;
  SpecWorkspace x = {};
  if (single) {
    if (!spec_ws_carve(ws2, ws2_bytes, n, bv ? 2 : 4, fast_seg_cap((cdiv64(n, kChunk) + 8) * kChunk), &x)) {
      set_error("%s: second workspace missing, not 256-byte aligned or smaller than "
                "sga_fused_single_sweep_workspace_bytes(n, values_dtype)=%zu", who,
                spec_ws_bytes(n, bv ? 2 : 4));
      return SGA_ERR_WORKSPACE;
    }
    // Shapes the single sweep does not take (the two-sweep step does them, same outputs): buckets
    // too small for the sampled bracket, a bracket that would be open below, or one whose
    // expected candidates do not fit the buffers.
    bool take = n >= kFastMinN && w.sample != nullptr && w.pbits != nullptr &&
                w.seg_cap == fast_seg_cap((cdiv64(n, kChunk) + 8) * kChunk);
    if (take) {
      int64_t n_sv = w.sample_cap / 4;
      if (n_sv > n / 4) n_sv = n / 4;
      const double ns = (double)n_sv * 4.0, frac = (double)k / (double)n, r = frac * ns;
      const double d = (out ? kSpecSigmasOut : kSpecSigmas) * sqrt(r * (1.0 - frac) + 1.0) + 8.0;
      if (r + d > ns) take = false;
      if ((2.0 * d + 2.0) * ((double)n / ns) > 0.25 * (double)kSegWaves * (double)w.seg_cap) take = false;
    }
    if (!take) { single = false; fast = 1; }
  }
  const FusedJob job{g, resid, p, m, v, n, k, segs, n_segs, idx_out, values_out, mask_out, result, w,
                     {out ? out[0] : nullptr, out ? out[1] : nullptr, out ? out[2] : nullptr,
                      out ? out[3] : nullptr}};
#define SGA_RUN(BG, BV, SC)                                                                   \
  if (single)                                                                                 \
    return run_fused_spec<BG, BV, SC>(g, resid, p, m, v, n, k, segs, n_segs, idx_out,        \
                                      values_out, mask_out, factor, coeff, flags, interval,   \
                                      seed, result, w, x, s, pack_extra, out);                \
  return run_fused<BG, BV, SC>(&job, 1, factor, coeff, fast, flags, interval, s, pack_extra, who)
#define SGA_RUN_SC(BG, BV)                    \
  switch (score_id) {                         \
    case 0: SGA_RUN(BG, BV, 0);               \
    case 1: SGA_RUN(BG, BV, 1);               \
    case 2: SGA_RUN(BG, BV, 2);               \
    case 3: SGA_RUN(BG, BV, 3);               \
    case 4: SGA_RUN(BG, BV, 4);               \
    default: SGA_RUN(BG, BV, 5);              \
  }
  if (bg && bv) { SGA_RUN_SC(true, true) }
  else if (bg) { SGA_RUN_SC(true, false) }
  else if (bv) { SGA_RUN_SC(false, true) }
  else { SGA_RUN_SC(false, false) }
#undef SGA_RUN_SC
#undef SGA_RUN
}

extern "C" int sga_fused_sparse_step(const void* g, int g_dtype, float* resid, float* p, float* m,
                                     float* v, int64_t n, int64_t k, const sga_segment* segs,
                                     int n_segs, int score_id, int32_t* idx_out, void* values_out,
                                     int values_dtype, uint8_t* mask_out, float factor,
                                     float coeff, int fast, int flags, float interval,
                                     sga_select_result* result, void* ws, size_t ws_bytes,
                                     void* stream) {
  return fused_entry("sga_fused_sparse_step", g, g_dtype, resid, p, m, v, 0, n, k, segs, n_segs,
                     score_id, idx_out, values_out, values_dtype, mask_out, factor, coeff, fast,
                     flags, interval, result, ws, ws_bytes, stream);
}

extern "C" int sga_fused_sparse_step_multi(const sga_fused_bucket* buckets, int n_buckets,
                                           int g_dtype, int score_id, int values_dtype,
                                           float factor, float coeff, int fast, int flags,
                                           float interval, void* stream) {
  const char* who = "sga_fused_sparse_step_multi";
  if ((flags & ~(SGA_GC_ADAMS | SGA_GC_FOLD)) != 0) {
    set_error("%s: flags may carry SGA_GC_ADAMS and SGA_GC_FOLD only (got %d)", who, flags);
    return SGA_ERR_ARG;
  }
  if ((flags & SGA_GC_FOLD) && !(interval > 0.0f)) {
    set_error("%s: SGA_GC_FOLD needs interval > 0 (got %g)", who, (double)interval);
    return SGA_ERR_ARG;
  }
  if (!buckets || n_buckets < 1 || (g_dtype != SGA_F32 && g_dtype != SGA_BF16) ||
      (values_dtype != SGA_F32 && values_dtype != SGA_BF16) || score_id < 0 ||
      score_id > SGA_SCORE_GR_OVER_SQRT_V) {
    set_error("%s: bad argument (n_buckets=%d score=%d)", who, n_buckets, score_id);
    return SGA_ERR_ARG;
  }
  hipStream_t s = (hipStream_t)stream;
  const bool bg = g_dtype == SGA_BF16, bv = values_dtype == SGA_BF16;
  // buckets that take the sampled-bracket path and buckets too small for it go through the
  // chain in separate batches of up to kMaxJobs
  for (int pass = 0; pass < 2; ++pass) {
    FusedJob jobs[kMaxJobs];
    int cnt = 0;
    for (int b = 0; b <= n_buckets; ++b) {
      if (b < n_buckets) {
        const sga_fused_bucket& u = buckets[b];
        if ((!u.g && (g_dtype != SGA_F32 || score_id == SGA_SCORE_ABS_G_BLIND)) || !u.resid ||
            !u.p || !u.m || !u.v || !u.segs || !u.idx_out || !u.values_out || u.n < 1 || u.n >= (1ll << 31) || u.k < 1 || u.k > u.n || u.n_segs < 1) {
          set_error("%s: bucket %d: bad argument (n=%lld k=%lld n_segs=%d; need 1 <= k <= n < 2^31)",
                    who, b, (long long)u.n, (long long)u.k, u.n_segs);
          return SGA_ERR_ARG;
        }
        SelWorkspace w;
        if (!sel_ws_carve(u.ws, u.ws_bytes, cdiv64(u.n, kChunk), &w)) {
          set_error("%s: bucket %d: workspace missing, misaligned or smaller than "
                    "sga_fused_workspace_bytes(n)=%zu", who, b, sel_ws_bytes(u.n));
          return SGA_ERR_WORKSPACE;
        }
        const bool is_fast = fast != 0 && SelBatch::fast_ok(w, u.n);
        if (is_fast != (pass == 0)) continue;
        jobs[cnt++] = FusedJob{u.g, u.resid, u.p, u.m, u.v, u.n, u.k, u.segs, u.n_segs, u.idx_out,
                               u.values_out, u.mask_out, u.result, w, {nullptr, nullptr, nullptr, nullptr}};
      }
      if (cnt == kMaxJobs || (b == n_buckets && cnt > 0)) {
        int rc;
#define SGA_RUNM(BG, BV, SC) rc = run_fused<BG, BV, SC>(jobs, cnt, factor, coeff, pass == 0, flags, interval, s, 0, who); break
#define SGA_RUNM_SC(BG, BV)                    \
        switch (score_id) {                    \
          case 0: SGA_RUNM(BG, BV, 0);         \
          case 1: SGA_RUNM(BG, BV, 1);         \
          case 2: SGA_RUNM(BG, BV, 2);         \
          case 3: SGA_RUNM(BG, BV, 3);         \
          case 4: SGA_RUNM(BG, BV, 4);         \
          default: SGA_RUNM(BG, BV, 5);        \
        }
        if (bg && bv) { SGA_RUNM_SC(true, true) }
        else if (bg) { SGA_RUNM_SC(true, false) }
        else if (bv) { SGA_RUNM_SC(false, true) }
        else { SGA_RUNM_SC(false, false) }
#undef SGA_RUNM_SC
#undef SGA_RUNM
        if (rc != SGA_OK) return rc;
        cnt = 0;
      }
    }
  }
  return SGA_OK;
}

extern "C" size_t sga_fused_single_sweep_workspace_bytes(int64_t n, int values_dtype) {
  return spec_ws_bytes(n < 0 ? 0 : n, values_dtype == SGA_BF16 ? 2 : 4);
}

extern "C" int sga_fused_sparse_step_single_sweep(
    const void* g, int g_dtype, float* resid, float* p, float* m, float* v, int64_t n, int64_t k,
    const sga_segment* segs, int n_segs, int score_id, int32_t* idx_out, void* values_out,
    int values_dtype, uint8_t* mask_out, float factor, float coeff, int flags, float interval,
    uint32_t seed, sga_select_result* result, void* ws, size_t ws_bytes, void* ws2,
    size_t ws2_bytes, void* stream) {
  return fused_entry("sga_fused_sparse_step_single_sweep", g, g_dtype, resid, p, m, v, 0, n, k,
                     segs, n_segs, score_id, idx_out, values_out, values_dtype, mask_out, factor,
                     coeff, 1, flags, interval, result, ws, ws_bytes, stream, true, ws2, ws2_bytes,
                     seed);
}

extern "C" int sga_fused_sparse_step_single_sweep_packed(
    const void* g, int g_dtype, float* state, int64_t n, int64_t k, const sga_segment* segs,
    int n_segs, int score_id, int32_t* idx_out, void* values_out, int values_dtype,
    uint8_t* mask_out, float factor, float coeff, int flags, float interval, uint32_t seed,
    sga_select_result* result, void* ws, size_t ws_bytes, void* ws2, size_t ws2_bytes,
    void* stream) {
  if (state && (reinterpret_cast<uintptr_t>(state) & 15)) {
    set_error("sga_fused_sparse_step_single_sweep_packed: state must be 16-byte aligned");
    return SGA_ERR_ARG;
  }
  return fused_entry("sga_fused_sparse_step_single_sweep_packed", g, g_dtype, state,
                     state ? state + kPackRun : nullptr, state ? state + 2 * kPackRun : nullptr,
                     state ? state + 3 * kPackRun : nullptr, kPackExtra, n, k, segs, n_segs,
                     score_id, idx_out, values_out, values_dtype, mask_out, factor, coeff, 1,
                     flags, interval, result, ws, ws_bytes, stream, true, ws2, ws2_bytes, seed);
}

// true when [a, a + a_bytes) and [b, b + b_bytes) overlap
static bool ranges_overlap(const void* a, size_t a_bytes, const void* b, size_t b_bytes) {
  const uintptr_t x = reinterpret_cast<uintptr_t>(a), y = reinterpret_cast<uintptr_t>(b);
  return x < y + b_bytes && y < x + a_bytes;
}

extern "C" int sga_fused_sparse_step_single_sweep_out(
    const void* g, int g_dtype, const float* resid, const float* p, const float* m, const float* v,
    float* resid_out, float* p_out, float* m_out, float* v_out, int64_t n, int64_t k,
    const sga_segment* segs, int n_segs, int score_id, int32_t* idx_out, void* values_out,
    int values_dtype, uint8_t* mask_out, float factor, float coeff, int flags, float interval,
    uint32_t seed, sga_select_result* result, void* ws, size_t ws_bytes, void* ws2,
    size_t ws2_bytes, void* stream) {
  const char* who = "sga_fused_sparse_step_single_sweep_out";
  float* out[4] = {resid_out, p_out, m_out, v_out};
  const float* in[4] = {resid, p, m, v};
  if (!resid_out || !p_out || !m_out || !v_out) {
    set_error("%s: the four output arrays are required", who);
    return SGA_ERR_ARG;
  }
  if (n > 0) {
    const size_t bytes = (size_t)n * 4, g_bytes = (size_t)n * (g_dtype == SGA_BF16 ? 2 : 4);
    for (int a = 0; a < 4; ++a) {
      bool bad = g && ranges_overlap(out[a], bytes, g, g_bytes);
      for (int b = 0; b < 4; ++b)
        bad = bad || (in[b] && ranges_overlap(out[a], bytes, in[b], bytes)) ||
              (b != a && ranges_overlap(out[a], bytes, out[b], bytes));
      if (bad) {
        set_error("%s: an output array overlaps an input or another output (the step reads "
                  "the old state while it writes the new one)", who);
        return SGA_ERR_ARG;
      }
    }
  }
  return fused_entry(who, g, g_dtype, const_cast<float*>(resid), const_cast<float*>(p),
                     const_cast<float*>(m), const_cast<float*>(v), 0, n, k, segs, n_segs, score_id,
                     idx_out, values_out, values_dtype, mask_out, factor, coeff, 1, flags, interval,
                     result, ws, ws_bytes, stream, true, ws2, ws2_bytes, seed, out);
}

extern "C" int sga_fused_sparse_step_single_sweep_packed_out(
    const void* g, int g_dtype, const float* state, float* state_out, int64_t n, int64_t k,
    const sga_segment* segs, int n_segs, int score_id, int32_t* idx_out, void* values_out,
    int values_dtype, uint8_t* mask_out, float factor, float coeff, int flags, float interval,
    uint32_t seed, sga_select_result* result, void* ws, size_t ws_bytes, void* ws2,
    size_t ws2_bytes, void* stream) {
  const char* who = "sga_fused_sparse_step_single_sweep_packed_out";
  if (!state || !state_out || (reinterpret_cast<uintptr_t>(state) & 15) ||
      (reinterpret_cast<uintptr_t>(state_out) & 15)) {
    set_error("%s: both packed states are required, 16-byte aligned", who);
    return SGA_ERR_ARG;
  }
  const size_t bytes = (size_t)(n <= 0 ? 0 : cdiv64(n, kPackRun) * 4 * kPackRun) * 4;
  const size_t g_bytes = (size_t)(n <= 0 ? 0 : n) * (g_dtype == SGA_BF16 ? 2 : 4);
  if (ranges_overlap(state, bytes, state_out, bytes) ||
      (g && ranges_overlap(state_out, bytes, g, g_bytes))) {
    set_error("%s: the output state overlaps the input state or the gradient", who);
    return SGA_ERR_ARG;
  }
  float* out[4] = {state_out, state_out + kPackRun, state_out + 2 * kPackRun, state_out + 3 * kPackRun};
  float* in = const_cast<float*>(state);
  return fused_entry(who, g, g_dtype, in, in + kPackRun, in + 2 * kPackRun, in + 3 * kPackRun,
                     kPackExtra, n, k, segs, n_segs, score_id, idx_out, values_out, values_dtype,
                     mask_out, factor, coeff, 1, flags, interval, result, ws, ws_bytes, stream, true,
                     ws2, ws2_bytes, seed, out);
}

extern "C" int64_t sga_packed_state_elems(int64_t n) {
  return n <= 0 ? 0 : cdiv64(n, kPackRun) * 4 * kPackRun;
}

extern "C" int sga_fused_sparse_step_packed(const void* g, int g_dtype, float* state, int64_t n,
                                            int64_t k, const sga_segment* segs, int n_segs,
                                            int score_id, int32_t* idx_out, void* values_out,
                                            int values_dtype, uint8_t* mask_out, float factor,
                                            float coeff, int fast, int flags, float interval,
                                            sga_select_result* result, void* ws, size_t ws_bytes,
                                            void* stream) {
  if (state && (reinterpret_cast<uintptr_t>(state) & 15)) {
    set_error("sga_fused_sparse_step_packed: state must be 16-byte aligned");
    return SGA_ERR_ARG;
  }
  return fused_entry("sga_fused_sparse_step_packed", g, g_dtype, state,
                     state ? state + kPackRun : nullptr, state ? state + 2 * kPackRun : nullptr,
                     state ? state + 3 * kPackRun : nullptr, kPackExtra, n, k, segs, n_segs,
                     score_id, idx_out, values_out, values_dtype, mask_out, factor, coeff, fast,
                     flags, interval, result, ws, ws_bytes, stream);
}

// resid/p/m/v <-> packed state (dir 0: pack, 1: unpack); a null array is skipped.
static __global__ __launch_bounds__(kBlock) void k_state_repack(float* __restrict__ r,
                                                                float* __restrict__ p,
                                                                float* __restrict__ m,
                                                                float* __restrict__ v,
                                                                float* __restrict__ state,
                                                                int64_t n, int dir) {
  float* arr[4] = {r, p, m, v};
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * kBlock) {
    const int64_t j = i + (i >> kPackRunLog) * kPackExtra;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      if (!arr[a]) continue;
      if (dir == 0) state[j + a * kPackRun] = arr[a][i];
      else arr[a][i] = state[j + a * kPackRun];
    }
  }
}

extern "C" int sga_state_repack(float* resid, float* p, float* m, float* v, float* state,
                                int64_t n, int unpack, void* stream) {
  if (n == 0) return SGA_OK;
  if (!state || n < 0) { set_error("sga_state_repack: bad argument"); return SGA_ERR_ARG; }
  hipLaunchKernelGGL(k_state_repack, dim3(stream_grid(n, kBlock, 1 << 16)), dim3(kBlock), 0,
                     (hipStream_t)stream, resid, p, m, v, state, n, unpack ? 1 : 0);
  return check_launch("sga_state_repack");
}
