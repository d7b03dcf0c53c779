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
    if (kNeedG) fetch_g<BF16G, FULL>(g, i, n, vec, w.g);
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
    if (kNeedG) unpack_g<BF16G, FULL>(w.g, q);
    if (kNeedR) {
      unpack_f32(w.r, rr);
#pragma unroll
      for (int e = 0; e < 4; ++e) q[e] = rr[e] + q[e];
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
    if (kNeedG) load_g<BF16G, FULL>(g, i, n, q, vec);
    if (kNeedR) {
      ld_f32<FULL>(r + sh, i, n, rr, vec);
#pragma unroll
      for (int e = 0; e < 4; ++e) q[e] = rr[e] + q[e];
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
  float* r;
  float* p;
  float* m;
  float* v;
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
  float* const R = a.r + sh;
  float* const P = a.p + sh;
  float* const M = a.m + sh;
  float* const V = a.v + sh;
  float gg[kChunkIters][4], rr[kChunkIters][4], pp[kChunkIters][4], mm[kChunkIters][4],
      vv[kChunkIters][4];
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
      else graw_f[it] = ld4_nt(reinterpret_cast<const float*>(a.g) + i);
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
        load_g<BF16G, false>(a.g, i, n, gg[it], a.vec);
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
        q[e] = rr[it][e] + gg[it][e];
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
        q[e] = rr[it][e] + gg[it][e];
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
      float pn[4], mn[4], vn[4];
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
      st_f32<FULL>(R, i, n, rr[it], a.vec);
      st_f32<FULL>(M, i, n, mm[it], a.vec);
      st_f32<FULL>(V, i, n, vv[it], a.vec);
      st_f32<FULL>(P, i, n, pp[it], a.vec);
      if (a.mask_out) st_u8<FULL>(a.mask_out, i, n, mk, a.mvec);
    }
  }
}

// Final sweep: select flags in index order, pack, residual, commit.
// `when`: 0 run always; 1 only if the sampled bracket held (the planes are
// settled); 2 only if it failed (the radix passes fixed the threshold and the
// keys are formed again here).
// (five waves per SIMD wherever the key is not an Adam-normalised chain formed in this kernel)
template <bool BF16G, bool BF16V, int SCORE, bool PLANES>
__global__ __launch_bounds__(kBlock, (PLANES || SCORE == SGA_SCORE_ABS_G || SCORE == SGA_SCORE_ABS_M ||
                                      SCORE == SGA_SCORE_ABS_G_BLIND) ? 5 : 1)
void k_fused_final(
    FinalArgs a, const sga_segment* __restrict__ segs, int n_segs,
    const SelState* __restrict__ st, const uint32_t* __restrict__ tile_sel,
    const uint32_t* __restrict__ tile_eq, int when, const int32_t* __restrict__ seg_dir) {
  if (when != 0 && (st->bracket_ok != 0) != (when == 1)) return;
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

template <bool BF16G, bool BF16V, int SCORE>
static int run_fused(const void* g, float* resid, float* p, float* m, float* v, int64_t n,
                     int64_t k, const sga_segment* segs, int n_segs, int32_t* idx_out,
                     void* values_out, uint8_t* mask_out, float factor, float coeff, int fast,
                     int flags, float interval, sga_select_result* result, const SelWorkspace& w,
                     hipStream_t s, int64_t pack_extra) {
  const bool vec = aligned4(g, BF16G ? 2 : 4) && aligned4(resid, 4) && aligned4(p, 4) &&
                   aligned4(m, 4) && aligned4(v, 4);
  const int adams = (flags & SGA_GC_ADAMS) ? 1 : 0;
  SrcFused<BF16G, SCORE> src{g, resid, p, m, v, vec, {}, pack_extra, adams};
  static_assert(kSelDirEntries == kSegDirEntries, "the workspace holds one directory");
  launch_seg_dir(segs, n_segs, n, w.seg_dir, s);
  src.sc.init(segs, n_segs, w.seg_dir);
  // Adam-normalised scores with the one-sweep select armed: the sweep leaves the selection as bit
  // planes (settled by the candidates) and the final sweep reads one bit per coordinate instead of
  // evaluating the score chain a second time; if the bracket fails on the device, the key-forming
  // final sweep runs instead.  For |g + r| and |m| the key is one instruction and re-forming it is
  // cheaper than writing and reading the planes (measured: 0.3 ms per step at 1.2e9 elements).
  const bool planes = SrcFused<BF16G, SCORE>::kHyper && fast != 0 && n >= kFastMinN && w.pbits != nullptr;
  run_select(src, n, k, 0, fast != 0, w, s, planes ? w.pbits : nullptr);
  const int64_t n_tiles = cdiv64(n, kChunk);
  if (planes)
    hipLaunchKernelGGL(k_cand_bits, dim3(256), dim3(kBlock), 0, s, w.st, w.cand_idx, w.cand_key,
                       w.tile_eq, n_tiles, 0, w.pbits);
  ProfPair* pp = prof_begin(SGA_PROF_FUSED_FINAL, s);
  FinalArgs fa;
  fa.g = g; fa.r = resid; fa.p = p; fa.m = m; fa.v = v; fa.n = n; fa.k = k;
  fa.idx_out = idx_out; fa.values_out = values_out; fa.mask_out = mask_out;
  fa.factor = factor; fa.coeff = coeff; fa.T = 0; fa.need = 0;
  fa.vec = vec; fa.mvec = aligned4(mask_out, 1);
  fa.scale = factor != 1.0f; fa.apply_coeff = coeff != 1.0f;
  fa.pack_extra = pack_extra;
  fa.adams = adams != 0; fa.fold = (flags & SGA_GC_FOLD) != 0; fa.interval = interval;
  fa.planes = w.pbits;
  const dim3 one_shot(stream_grid(n_tiles, kChunksPerBlock, 1 << 20));
  if (planes) {
    hipLaunchKernelGGL((k_fused_final<BF16G, BF16V, SGA_SCORE_ABS_G, true>), one_shot, dim3(kBlock), 0, s,
                       fa, segs, n_segs, w.st, w.tile_gt, w.tile_eq, 1, w.seg_dir);
    // the rare other outcome: a small grid that strides over the chunks (returns at once otherwise)
    hipLaunchKernelGGL((k_fused_final<BF16G, BF16V, SCORE, false>),
                       dim3(stream_grid(n_tiles, kChunksPerBlock, 2048)), dim3(kBlock), 0, s, fa,
                       segs, n_segs, w.st, w.tile_gt, w.tile_eq, 2, w.seg_dir);
  } else {
    hipLaunchKernelGGL((k_fused_final<BF16G, BF16V, SCORE, false>), one_shot, dim3(kBlock), 0, s, fa,
                       segs, n_segs, w.st, w.tile_gt, w.tile_eq, 0, w.seg_dir);
  }
  prof_end(pp, s);
  if (result) hipLaunchKernelGGL(k_sel_result, dim3(1), dim3(1), 0, s, w.st, result);
  return check_launch("sga_fused_sparse_step");
}

}  // namespace sga

using namespace sga;

extern "C" size_t sga_fused_workspace_bytes(int64_t n) { return sel_ws_bytes(n < 0 ? 0 : n); }

static int fused_entry(const char* who, const void* g, int g_dtype, float* resid, float* p,
                       float* m, float* v, int64_t pack_extra, int64_t n, int64_t k,
                       const sga_segment* segs, int n_segs, int score_id, int32_t* idx_out,
                       void* values_out, int values_dtype, uint8_t* mask_out, float factor,
                       float coeff, int fast, int flags, float interval, sga_select_result* result,
                       void* ws, size_t ws_bytes, void* stream) {
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
  if (!g || !resid || !p || !m || !v || !segs || !idx_out || !values_out || n < 1 ||
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
#define SGA_RUN(BG, BV, SC)                                                                   \
  return run_fused<BG, BV, SC>(g, resid, p, m, v, n, k, segs, n_segs, idx_out, values_out,   \
                               mask_out, factor, coeff, fast, flags, interval, result, w, s,   \
                               pack_extra)
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
