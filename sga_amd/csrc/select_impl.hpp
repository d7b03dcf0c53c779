// Exact k-th-largest select over 31-bit magnitude keys, templated on where
// the keys come from (a score array, raw key buffers, or a fused g+residual
// expression).  Non-negative fp32 values order like their integer patterns,
// so the k-th largest key is found by a three-level radix descent
// (12 + 12 + 7 bits) over LDS-privatised histograms, followed by an ordered
// per-chunk count so that ties at the threshold can be granted in ascending
// index order without any float compare ambiguity.
#pragma once
#include <atomic>
#include <type_traits>
#include "common.hpp"

namespace sga {

constexpr int kL0Bits = 12, kL1Bits = 12, kL2Bits = 7;
constexpr int kL0Shift = 19, kL1Shift = 7;
constexpr int kBinsBig = 4096, kBinsSmall = 128;
constexpr int kTileScanPer = 16;
constexpr int kTileScanSpan = kBlock * kTileScanPer;  // 4096 tiles / workgroup
constexpr int kMaxTileBlocks = 1024;                  // covers n < 2^32

struct SelState {
  uint32_t k;
  uint32_t prefix;
  uint32_t krem;
  uint32_t thresh_bits;
  uint32_t need;
  uint32_t n_gt;
  uint32_t n_eq;
  uint32_t nonfinite;
  uint32_t status;
  uint32_t total;
  uint32_t n_selected;
  uint32_t path;
  // sampled-bracket path
  uint32_t t_lo;        // candidates are keys in [t_lo, t_hi)
  uint32_t t_hi;
  uint32_t n_hi;        // keys >= t_hi
  uint32_t cand_count;  // keys in the bracket (may exceed capacity)
  uint32_t cand_cap;
  uint32_t bracket_ok;  // 1: the sampled bracket holds the k-th key; radix passes skip
  uint32_t sample_n;
  uint32_t overflow;    // a candidate segment ran out of room
  uint32_t skip;        // 1: kernels driven by this state do nothing
  uint32_t done[3];     // per-level "workgroups finished" tickets (last one scans)
  uint32_t spec;        // 1: the single-sweep step committed on the sampled bracket (no way back)
  uint32_t negative;    // 1: an fp32 score array held a value below zero (magnitudes were ranked)
  uint32_t redone;      // 1: an out-of-place single-sweep step missed its bracket and was redone
  uint32_t pad_[5];
};
static_assert(sizeof(SelState) == 128, "SelState layout");

struct SelWorkspace {
  SelState* st;        // main state (result, bracket)
  SelState* aux;       // aux[0], aux[1]: states of the sample / candidate descents
  uint32_t* hist;      // 2 sets of 3 levels: [0,4096) [4096,8192) [8192,8320)
  uint32_t* tile_gt;   // n_tiles -> selected-count prefix
  uint32_t* tile_eq;   // n_tiles -> tie-count prefix
  uint32_t* blk_gt;    // kMaxTileBlocks
  uint32_t* blk_eq;    // kMaxTileBlocks
  int32_t* seg_dir;    // kSelDirEntries: tensor directory of segment-keyed sources (adam_math.hpp)
  int64_t n_tiles_cap;
  // sampled-bracket path (null / 0 when the workspace has no room for it)
  uint32_t* sample;    // sample_cap keys
  uint32_t* seg_cnt;   // kSegWaves (+1) counts -> offsets
  uint32_t* seg_idx;   // kSegWaves * seg_cap
  uint32_t* seg_key;
  uint32_t* cand_idx;  // dense candidates
  uint32_t* cand_key;
  uint32_t* pbits;     // 32 words per chunk: bit planes of "key above the bracket"
  int64_t sample_cap;
  int64_t seg_cap;     // per-wave candidate capacity
};

constexpr int kSegWaves = 8192;            // candidate segments the sweep's chunks hash to
constexpr int kSweepParts = 256;            // partial counters of the sweep's two totals
constexpr int64_t kFastMinN = 1 << 20;     // below this the radix passes are cheap enough

static inline int64_t fast_sample_vecs(int64_t n) {
  int64_t v = n / 1024;
  if (v < 16384) v = 16384;
  if (v > (1 << 18)) v = 1 << 18;
  return v;
}
static inline int64_t fast_seg_cap(int64_t n) {
  int64_t c = n / 32 / kSegWaves;
  if (c < 64) c = 64;
  if (c > 8192) c = 8192;
  return c;
}

// Batched chain: every short kernel around a select takes up to kMaxJobs
// independent select problems in one launch (blockIdx.y = job), so that a
// caller with several buckets (or several re-selections of one replay step)
// pays the chain of dependent launches once instead of once per problem.
// The operands travel by value in the kernel arguments.
constexpr int kMaxJobs = 8;
struct ChainJob {
  SelState* st;
  SelState* aux;
  uint32_t* hist;
  uint32_t* tile_gt;
  uint32_t* tile_eq;
  uint32_t* blk_gt;
  uint32_t* blk_eq;
  uint32_t* sample;
  uint32_t* seg_cnt;
  uint32_t* seg_idx;
  uint32_t* seg_key;
  uint32_t* cand_idx;
  uint32_t* cand_key;
  uint32_t* seg_fail;          // single-sweep step: per-segment first failed reservation
  const F4* seg_rec;           // single-sweep step: records beside the segments' keys
  F4* cand_rec;
  uint32_t* planes;            // where the settlement writes the selection (bit planes) ...
  uint8_t* mask;               // ... or mask bytes
  sga_select_result* result;
  int64_t n, n_tiles, n_sv, n_vec;
  uint32_t k, seg_cap, seed, ovf_cap;
  int tie_all, spec;
};
struct ChainJobs { ChainJob j[kMaxJobs]; };
template <class Src>
struct SrcPack { Src s[kMaxJobs]; };

// Workspace layout: [fixed: states | level histograms | tile-scan block sums]
// [tile_gt[nt] | tile_eq[nt]] [fast-path buffers sized from nt: sample keys,
// per-wave candidate segments, dense candidates, 128 B of bit planes per
// tile].  nt is derived from the byte size, so every entry point recovers
// the same carve from (ws, ws_bytes) alone.
constexpr int kHistEntries = 2 * kBinsBig + kBinsSmall;      // 8320
constexpr int kHistStride = kHistEntries + 64;               // per-state stride
constexpr int kSelDirEntries = 1 << 15;                        // n < 2^31 in blocks of 2^16
constexpr size_t kSelFixedBytes =
    512 + (size_t)kHistStride * 2 * 4 + (size_t)kMaxTileBlocks * 4 * 2 + (size_t)kSelDirEntries * 4;

static inline size_t fast_bytes_for_tiles(int64_t nt) {
  const int64_t n = nt * kChunk;
  if (n < kFastMinN) return 0;
  const int64_t sc = fast_seg_cap(n);
  return (size_t)fast_sample_vecs(n) * 16 + (size_t)(kSegWaves + 64) * 4 +
         (size_t)kSegWaves * sc * 4 * 4 + (size_t)nt * 128 + 256;
}

static inline size_t sel_ws_bytes(int64_t n) {
  const int64_t nt = cdiv64(n, kChunk) + 8;
  size_t b = kSelFixedBytes + (size_t)nt * 4 * 2 + fast_bytes_for_tiles(nt);
  return (b + 255) & ~(size_t)255;
}

static inline bool sel_ws_carve(void* ws, size_t bytes, int64_t n_tiles_needed,
                                SelWorkspace* out) {
  if (!ws || bytes < kSelFixedBytes || (reinterpret_cast<uintptr_t>(ws) & 15))
    return false;
  // largest nt whose full layout fits (layout size is monotone in nt)
  int64_t lo = 0, hi = (int64_t)((bytes - kSelFixedBytes) / 8);
  while (lo < hi) {
    const int64_t mid = lo + (hi - lo + 1) / 2;
    if (kSelFixedBytes + (size_t)mid * 8 + fast_bytes_for_tiles(mid) <= bytes) lo = mid;
    else hi = mid - 1;
  }
  const int64_t nt = lo;
  if (nt < n_tiles_needed) return false;
  char* p = reinterpret_cast<char*>(ws);
  out->st = reinterpret_cast<SelState*>(p);
  out->aux = reinterpret_cast<SelState*>(p + 128);
  p += 512;
  out->hist = reinterpret_cast<uint32_t*>(p);
  p += (size_t)kHistStride * 2 * 4;
  out->blk_gt = reinterpret_cast<uint32_t*>(p);
  p += (size_t)kMaxTileBlocks * 4;
  out->blk_eq = reinterpret_cast<uint32_t*>(p);
  p += (size_t)kMaxTileBlocks * 4;
  out->seg_dir = reinterpret_cast<int32_t*>(p);
  p += (size_t)kSelDirEntries * 4;
  out->tile_gt = reinterpret_cast<uint32_t*>(p);
  p += (size_t)nt * 4;
  out->tile_eq = reinterpret_cast<uint32_t*>(p);
  p += (size_t)nt * 4;
  out->n_tiles_cap = nt;
  out->sample = nullptr;
  out->seg_cnt = out->seg_idx = out->seg_key = out->cand_idx = out->cand_key = nullptr;
  out->pbits = nullptr;
  out->sample_cap = 0;
  out->seg_cap = 0;
  if (fast_bytes_for_tiles(nt) > 0) {
    const int64_t n = nt * kChunk;
    p = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(p) + 255) & ~(uintptr_t)255);
    out->sample_cap = fast_sample_vecs(n) * 4;
    out->seg_cap = fast_seg_cap(n);
    out->sample = reinterpret_cast<uint32_t*>(p);
    p += (size_t)out->sample_cap * 4;
    out->seg_cnt = reinterpret_cast<uint32_t*>(p);
    p += (size_t)(kSegWaves + 64) * 4;
    const size_t seg_bytes = (size_t)kSegWaves * out->seg_cap * 4;
    out->seg_idx = reinterpret_cast<uint32_t*>(p); p += seg_bytes;
    out->seg_key = reinterpret_cast<uint32_t*>(p); p += seg_bytes;
    out->cand_idx = reinterpret_cast<uint32_t*>(p); p += seg_bytes;
    out->cand_key = reinterpret_cast<uint32_t*>(p); p += seg_bytes;
    out->pbits = reinterpret_cast<uint32_t*>(p);
  }
  return true;
}

#ifdef __HIPCC__

// ------------------------------------------------------------ key sources
// A key source yields the 31-bit magnitude keys of 4 consecutive elements.
// load<FULL>: FULL promises i + 4 <= n and vector alignment (see ld_f32).
// The one-sweep select drives a source in three steps instead, so that the
// loads of kAhead slabs of a chunk are in flight before the first key is
// formed: chunk_begin (what is common to the chunk's 1024 elements, held on
// the scalar unit), fetch (loads only), keys (arithmetic only).
struct NoChunk {};
struct SrcF32 {                 // |x| of an fp32 score array
  const float* x;
  bool vec;
  uint32_t neg;                 // this lane has seen a value below zero (callers that promise
                                // non-negative scores are told, without a pass of their own)
  using Raw = F4;
  using Chunk = NoChunk;
  static constexpr int kAhead = kChunkIters;
  __device__ __forceinline__ Chunk chunk_begin(int64_t) { return Chunk{}; }
  __device__ __forceinline__ void chunk_hyper(int64_t) {}
  template <bool FULL>
  __device__ __forceinline__ void fetch(const Chunk&, int64_t i, int64_t n, Raw& r) {
    r = ldraw_f32<FULL>(x, i, n, vec);
  }
  template <bool FULL>
  __device__ __forceinline__ void keys(const Chunk&, int64_t, int64_t, const Raw& r, uint32_t key[4]) {
    key[0] = abs_key(r.x); key[1] = abs_key(r.y); key[2] = abs_key(r.z); key[3] = abs_key(r.w);
    neg |= (uint32_t)((r.x < 0.0f) | (r.y < 0.0f) | (r.z < 0.0f) | (r.w < 0.0f));
  }
  template <bool FULL = false>
  __device__ __forceinline__ void load(int64_t i, int64_t n, uint32_t key[4]) {
    float v[4];
    ld_f32<FULL>(x, i, n, v, vec);
#pragma unroll
    for (int e = 0; e < 4; ++e) { key[e] = abs_key(v[e]); neg |= (uint32_t)(v[e] < 0.0f); }
  }
};
// What a key source knows about the sign of its inputs (only fp32 score arrays keep track).
template <class Src>
__device__ __forceinline__ uint32_t src_negative(const Src&) { return 0u; }
__device__ __forceinline__ uint32_t src_negative(const SrcF32& s) { return s.neg; }
template <class Src>
__device__ __forceinline__ void note_negative(const Src& src, SelState* st) {
  if (ballot64(src_negative(src) != 0u) != 0ull && lane_id() == 0) atomicOr(&st->negative, 1u);
}

struct SrcU32 {                 // raw keys (sample / candidate buffers)
  const uint32_t* x;
  static constexpr bool vec = true;
  template <bool FULL = false>
  __device__ __forceinline__ void load(int64_t i, int64_t n, uint32_t key[4]) {
    if (FULL || i + 4 <= n) {
      U4 v = *reinterpret_cast<const U4*>(x + i);
      key[0] = v.x; key[1] = v.y; key[2] = v.z; key[3] = v.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) key[e] = (i + e < n) ? x[i + e] : 0u;
    }
  }
};

// ------------------------------------------------------------- LDS histogram
// One increment per participating lane; when many lanes of the wave hit the
// bin of the first participating lane (zero-heavy or plateau data) they are
// folded into a single add so same-address LDS atomics do not serialise.
__device__ __forceinline__ void lds_hist_add(uint32_t* s_h, uint32_t bin, bool part) {
  uint64_t act = ballot64(part);
  if (act == 0) return;
  const int leader = __ffsll((unsigned long long)act) - 1;
  const uint32_t lead_bin = __shfl(bin, leader, kWave);
  const uint64_t same = ballot64(part && bin == lead_bin);
  const int ns = __popcll(same);
  if (ns >= 8) {
    if (lane_id() == leader) atomicAdd(&s_h[lead_bin], (uint32_t)ns);
    part = part && bin != lead_bin;
  }
  if (part) atomicAdd(&s_h[bin], 1u);
}

template <int LEVEL>
__device__ __forceinline__ void level_bin(uint32_t key, uint32_t prefix, bool valid,
                                          uint32_t& bin, bool& part) {
  if (LEVEL == 0) { bin = key >> kL0Shift; part = valid; }
  else if (LEVEL == 1) { bin = (key >> kL1Shift) & (kBinsBig - 1); part = valid && (key >> kL0Shift) == prefix; }
  else { bin = key & (kBinsSmall - 1); part = valid && (key >> kL1Shift) == prefix; }
}

// One level of the descent for one state, run by a single workgroup: find
// the bin where the descending cumulative count crosses the remaining rank.
template <int LEVEL>
__device__ __forceinline__ void level_scan_body(SelState* __restrict__ st,
                                                const uint32_t* __restrict__ hist,
                                                uint32_t* s_suf /* kBlock + 1 */) {
  constexpr int NB = LEVEL == 2 ? kBinsSmall : kBinsBig;
  constexpr int PER = NB >= kBlock ? NB / kBlock : 1;
  constexpr int BITS = LEVEL == 2 ? kL2Bits : 12;
  const int t = threadIdx.x;
  // read the incoming rank before any barrier: the one thread that descends
  // overwrites st->krem after the barriers below
  const uint32_t krem = (LEVEL == 0) ? st->k : st->krem;
  const uint32_t pre_in = (LEVEL == 0) ? 0u : st->prefix;
  uint32_t loc[PER];
  uint32_t mine = 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int b = t * PER + j;
    loc[j] = (b < NB) ? __atomic_load_n(&hist[b], __ATOMIC_RELAXED) : 0u;
    mine += loc[j];
  }
  __syncthreads();
  s_suf[t] = mine;                       // suffix sums over threads
  if (t == 0) s_suf[kBlock] = 0u;
  __syncthreads();
  for (int o = 1; o < kBlock; o <<= 1) {
    uint32_t add = (t + o < kBlock) ? s_suf[t + o] : 0u;
    __syncthreads();
    s_suf[t] += add;
    __syncthreads();
  }
  const uint32_t total = s_suf[0];
  if (LEVEL == 0 && t == 0) {
    st->total = total;
    if (krem < 1 || krem > total) st->status = 1;
  }
  // exponent 255 (Inf / NaN) is bins 0xFF0..0xFFF: exactly the last thread's bins
  static_assert(kBinsBig / kBlock == 16 && (kBlock - 1) * 16 == 0xFF0, "non-finite bins = last thread");
  if (LEVEL == 0 && t == kBlock - 1) st->nonfinite = mine;
  const uint32_t above_me = s_suf[t + 1];
  if (krem >= 1 && above_me < krem && krem <= above_me + mine) {
    uint32_t above = above_me;
#pragma unroll
    for (int j = PER - 1; j >= 0; --j) {
      const int b = t * PER + j;
      if (b < NB) {
        if (above < krem && krem <= above + loc[j]) {
          const uint32_t np = (pre_in << BITS) | (uint32_t)b;
          st->prefix = np;
          st->krem = krem - above;
          if (LEVEL == 2) {
            st->thresh_bits = np;
            st->need = krem - above;
            st->n_eq = loc[j];
            st->n_gt = st->k - (krem - above);
          }
        }
        above += loc[j];
      }
    }
  }
  __syncthreads();
}

template <int LEVEL>
__device__ __forceinline__ uint32_t* level_hist_of(uint32_t* hist_set) {
  return hist_set + (LEVEL == 0 ? 0 : LEVEL == 1 ? kBinsBig : 2 * kBinsBig);
}

// Histogram sweep of one radix level for NS states at once (NS = 2 lets the
// two ends of the sample bracket descend together).  n_dev (optional) caps n
// with a count produced on the device; a state whose `skip` flag is set does
// not take part.  MERGE: the last workgroup to finish also runs the level's
// scan, so hist + scan is one launch.
template <class Src, int LEVEL, int NS, bool MERGE>
__device__ __forceinline__ void level_hist_body(Src& src, int64_t n,
                                                const uint32_t* __restrict__ n_dev,
                                                SelState* __restrict__ st,
                                                uint32_t* __restrict__ hist) {
  constexpr int NB = LEVEL == 2 ? kBinsSmall : kBinsBig;
  // Level 0 has no prefix: every state sees the same histogram of all keys, so it is built and
  // flushed once (set 0) and every state's scan reads that one.
  constexpr int NH = LEVEL == 0 ? 1 : NS;
  __shared__ uint32_t s_h[NH][NB];
  __shared__ uint32_t s_suf[kBlock + 1];
  __shared__ uint32_t s_last;
  bool on[NS];
  uint32_t prefix[NS];
  bool any = false;
#pragma unroll
  for (int q = 0; q < NS; ++q) {
    on[q] = st[q].skip == 0;
    prefix[q] = st[q].prefix;
    any = any || on[q];
  }
  if (!any) return;
  if (n_dev && (int64_t)*n_dev < n) n = (int64_t)*n_dev;
#pragma unroll
  for (int q = 0; q < NH; ++q)
    for (int b = threadIdx.x; b < NB; b += kBlock) s_h[q][b] = 0u;
  __syncthreads();
  // Raw key buffers (sample, candidates) are short and sit in L2: what their passes cost is load
  // latency, so each lane keeps kQuads 16-byte loads in flight per trip.  Key sources that compute
  // (the radix passes over the data itself) go one quad at a time.
  constexpr int kQuads = std::is_same<Src, SrcU32>::value ? 4 : 1;
  constexpr int64_t kSlabKeys = (int64_t)kBlock * kVec;
  const int64_t stride = (int64_t)gridDim.x * kSlabKeys * kQuads;
  // uniform trip count so the wave-level ballots inside lds_hist_add are safe
  const int64_t first = (int64_t)blockIdx.x * kSlabKeys * kQuads;
  for (int64_t base = first; base < n; base += stride) {
    uint32_t key[kQuads][4];
    bool full[kQuads];
#pragma unroll
    for (int u = 0; u < kQuads; ++u) {
      const int64_t bu = base + u * kSlabKeys;
      const int64_t i = bu + (int64_t)threadIdx.x * kVec;
      key[u][0] = key[u][1] = key[u][2] = key[u][3] = 0u;
      full[u] = src.vec && bu + kSlabKeys <= n;   // whole workgroup span in range
      if (full[u]) src.template load<true>(i, n, key[u]);
      else if (i < n) src.template load<false>(i, n, key[u]);
    }
#pragma unroll
    for (int u = 0; u < kQuads; ++u) {
      const int64_t i = base + u * kSlabKeys + (int64_t)threadIdx.x * kVec;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
#pragma unroll
        for (int q = 0; q < NH; ++q) {
          uint32_t bin; bool part;
          level_bin<LEVEL>(key[u][e], prefix[q], full[u] || i + e < n, bin, part);
          const bool live = NH == NS ? on[q] : any;
          // Raw key buffers are at most a few million keys for 64 workgroups of one wave per
          // SIMD: what a pass costs there is the latency of each key's chain, and the folding of
          // equal bins (two ballots, a cross-lane read and two scalar branches per key) is most of
          // it.  A plain LDS atomic per lane is shorter; on a plateau (every lane on one bin) it
          // serialises 64-fold, which for these few keys is a couple of microseconds.
          if (std::is_same<Src, SrcU32>::value) {
            if (part && live) atomicAdd(&s_h[q][bin], 1u);
          } else {
            lds_hist_add(s_h[q], bin, part && live);
          }
        }
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < NH; ++q) {
    if (NH == NS && !on[q]) continue;
    uint32_t* gh = level_hist_of<LEVEL>(hist + q * kHistStride);
    for (int b = threadIdx.x; b < NB; b += kBlock) {
      const uint32_t c = s_h[q][b];
      if (c) atomicAdd(&gh[b], c);
    }
  }
  if (!MERGE) return;
  __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t ticket = atomicAdd(&st[0].done[LEVEL], 1u);
    s_last = (ticket == gridDim.x - 1) ? 1u : 0u;
  }
  __syncthreads();
  if (!s_last) return;
  __threadfence();
#pragma unroll
  for (int q = 0; q < NS; ++q)
    if (on[q])
      level_scan_body<LEVEL>(&st[q], level_hist_of<LEVEL>(hist + (NH == NS ? q : 0) * kHistStride), s_suf);
  if (threadIdx.x == 0) st[0].done[LEVEL] = 0u;
}
// over the data itself (a key source per job): the radix passes, state = st
template <class Src, int LEVEL, bool MERGE>
__global__ __launch_bounds__(kBlock) void k_level_hist(SrcPack<Src> srcs, ChainJobs jobs) {
  const ChainJob& J = jobs.j[blockIdx.y];
  Src src = srcs.s[blockIdx.y];
  level_hist_body<Src, LEVEL, 1, MERGE>(src, J.n, nullptr, J.st, J.hist);
}
// over a raw key buffer of the job: the sample (both bracket ends descend together, states
// aux[0], aux[1]) or the candidates (their count lives on the device; state aux[0])
template <int LEVEL, bool CAND>
__global__ __launch_bounds__(kBlock) void k_level_hist_raw(ChainJobs jobs) {
  const ChainJob& J = jobs.j[blockIdx.y];
  SrcU32 src{CAND ? J.cand_key : J.sample};
  if (CAND)
    level_hist_body<SrcU32, LEVEL, 1, true>(src, (int64_t)kSegWaves * J.seg_cap, &J.st->cand_count,
                                            J.aux, J.hist);
  else
    level_hist_body<SrcU32, LEVEL, 2, true>(src, J.n_sv * 4, nullptr, J.aux, J.hist);
}

// Stand-alone scan (used when one level's histogram is built by several
// launches, one per view).
template <int LEVEL>
__global__ __launch_bounds__(kBlock) void k_level_scan(ChainJobs jobs) {
  __shared__ uint32_t s_suf[kBlock + 1];
  const ChainJob& J = jobs.j[blockIdx.y];
  if (J.st->skip) return;
  level_scan_body<LEVEL>(J.st, level_hist_of<LEVEL>(J.hist), s_suf);
}

// Per-chunk (1024 elements, one wave) counts of keys above / equal to the
// threshold.
template <class Src>
__global__ __launch_bounds__(kBlock) void k_tile_count(SrcPack<Src> srcs, ChainJobs jobs,
                                                       int64_t tile_base) {
  const ChainJob& J = jobs.j[blockIdx.y];
  SelState* __restrict__ st = J.st;
  if (st->skip) return;
  Src src = srcs.s[blockIdx.y];
  const int64_t n = J.n;
  uint32_t* __restrict__ tile_gt = J.tile_gt;
  uint32_t* __restrict__ tile_eq = J.tile_eq;
  const uint32_t T = st->thresh_bits;
  const int64_t n_chunks = cdiv64(n, kChunk);
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  for (int64_t c = (int64_t)blockIdx.x * kChunksPerBlock + wave_id(); c < n_chunks;
       c += wstride) {
    uint32_t cg = 0, ce = 0;
    if (src.vec && (c + 1) * kChunk <= n) {
      uint32_t key[kChunkIters][4];
#pragma unroll
      for (int it = 0; it < kChunkIters; ++it)
        src.template load<true>(c * kChunk + it * (kWave * kVec) + lane_id() * kVec, n, key[it]);
#pragma unroll
      for (int it = 0; it < kChunkIters; ++it)
#pragma unroll
        for (int e = 0; e < 4; ++e) { cg += key[it][e] > T; ce += key[it][e] == T; }
    } else {
#pragma unroll
      for (int it = 0; it < kChunkIters; ++it) {
        const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
        uint32_t key[4] = {0, 0, 0, 0};
        if (i < n) src.template load<false>(i, n, key);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const bool valid = i + e < n;
          cg += (valid && key[e] > T);
          ce += (valid && key[e] == T);
        }
      }
    }
    cg = wave_sum(cg);
    ce = wave_sum(ce);
    if (lane_id() == 0) {
      tile_gt[tile_base + c] = cg;
      tile_eq[tile_base + c] = ce;
    }
  }
  note_negative(src, st);
}

// Tile scan, kernel 1: per-workgroup totals of (gt, eq).
static __global__ __launch_bounds__(kBlock) void k_tile_sums(ChainJobs jobs) {
  __shared__ uint32_t s_g[kChunksPerBlock], s_e[kChunksPerBlock];
  const ChainJob& J = jobs.j[blockIdx.y];
  const int64_t n_tiles = J.n_tiles;
  if ((int64_t)blockIdx.x * kTileScanSpan >= n_tiles) return;     // a job with fewer tiles
  const uint32_t* __restrict__ tile_gt = J.tile_gt;
  const uint32_t* __restrict__ tile_eq = J.tile_eq;
  uint32_t* __restrict__ blk_gt = J.blk_gt;
  uint32_t* __restrict__ blk_eq = J.blk_eq;
  const int64_t base = (int64_t)blockIdx.x * kTileScanSpan + (int64_t)threadIdx.x * kTileScanPer;
  uint32_t g = 0, e = 0;
#pragma unroll
  for (int j = 0; j < kTileScanPer; ++j)
    if (base + j < n_tiles) { g += tile_gt[base + j]; e += tile_eq[base + j]; }
  g = wave_sum(g);
  e = wave_sum(e);
  if (lane_id() == 0) { s_g[wave_id()] = g; s_e[wave_id()] = e; }
  __syncthreads();
  if (threadIdx.x == 0) {
    blk_gt[blockIdx.x] = s_g[0] + s_g[1] + s_g[2] + s_g[3];
    blk_eq[blockIdx.x] = s_e[0] + s_e[1] + s_e[2] + s_e[3];
  }
}

__device__ __forceinline__ uint32_t ties_taken(uint32_t need, uint32_t eq_before, uint32_t eq_here) {
  if (need <= eq_before) return 0u;
  const uint32_t left = need - eq_before;
  return left < eq_here ? left : eq_here;
}

// Block-wide exclusive scan of one uint32 per thread (kBlock threads).
__device__ __forceinline__ uint32_t block_excl_scan(uint32_t v, uint32_t* s_w4, uint32_t& block_total) {
  const uint32_t incl = wave_incl_scan(v);
  __syncthreads();
  if (lane_id() == kWave - 1) s_w4[wave_id()] = incl;
  __syncthreads();
  uint32_t pre = 0;
  for (int w = 0; w < wave_id(); ++w) pre += s_w4[w];
  block_total = s_w4[0] + s_w4[1] + s_w4[2] + s_w4[3];
  return pre + incl - v;
}

// Tile scan, kernel 2: tile_eq[i] <- ties before tile i; tile_gt[i] <- selected
// coordinates before tile i (ties granted in ascending order until `need`
// is used up; all of them when tie_all).
static __global__ __launch_bounds__(kBlock) void k_tile_apply(ChainJobs jobs) {
  __shared__ uint32_t s_w4[kChunksPerBlock];
  const ChainJob& J = jobs.j[blockIdx.y];
  const int64_t n_tiles = J.n_tiles;
  const int n_blocks = (int)cdiv64(n_tiles, kTileScanSpan);
  if ((int)blockIdx.x >= n_blocks) return;                        // a job with fewer tiles
  uint32_t* __restrict__ tile_gt = J.tile_gt;
  uint32_t* __restrict__ tile_eq = J.tile_eq;
  const uint32_t* __restrict__ blk_gt = J.blk_gt;
  const uint32_t* __restrict__ blk_eq = J.blk_eq;
  const int tie_all = J.tie_all;
  SelState* __restrict__ st = J.st;
  const uint32_t need = tie_all ? 0xFFFFFFFFu : st->need;
  // prefixes of the workgroups before this one (n_blocks <= 1024 -> 4 each)
  uint32_t be[4], bg[4];
  uint32_t mine_e = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int b = threadIdx.x * 4 + j;
    be[j] = (b < n_blocks) ? blk_eq[b] : 0u;
    bg[j] = (b < n_blocks) ? blk_gt[b] : 0u;
    mine_e += be[j];
  }
  uint32_t tot_e;
  uint32_t e_run = block_excl_scan(mine_e, s_w4, tot_e);
  uint32_t sel_before = 0, eq_before = 0;   // contributions of blocks < blockIdx.x
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int b = threadIdx.x * 4 + j;
    if (b < (int)blockIdx.x) {
      sel_before += bg[j] + ties_taken(need, e_run, be[j]);
      eq_before += be[j];
    }
    e_run += be[j];
  }
  uint32_t dummy;
  __syncthreads();
  // reduce sel_before / eq_before across the workgroup via scans' totals
  block_excl_scan(sel_before, s_w4, dummy);
  const uint32_t S0 = dummy;
  __syncthreads();
  block_excl_scan(eq_before, s_w4, dummy);
  const uint32_t E0 = dummy;
  __syncthreads();

  const int64_t base = (int64_t)blockIdx.x * kTileScanSpan + (int64_t)threadIdx.x * kTileScanPer;
  uint32_t g[kTileScanPer], e[kTileScanPer];
  uint32_t my_e = 0;
#pragma unroll
  for (int j = 0; j < kTileScanPer; ++j) {
    const bool ok = base + j < n_tiles;
    g[j] = ok ? tile_gt[base + j] : 0u;
    e[j] = ok ? tile_eq[base + j] : 0u;
    my_e += e[j];
  }
  uint32_t blk_tot_e;
  uint32_t er = E0 + block_excl_scan(my_e, s_w4, blk_tot_e);
  uint32_t my_s = 0;
  uint32_t ebase[kTileScanPer], scount[kTileScanPer];
#pragma unroll
  for (int j = 0; j < kTileScanPer; ++j) {
    ebase[j] = er;
    scount[j] = g[j] + ties_taken(need, er, e[j]);
    my_s += scount[j];
    er += e[j];
  }
  __syncthreads();
  uint32_t blk_tot_s;
  uint32_t sr = S0 + block_excl_scan(my_s, s_w4, blk_tot_s);
#pragma unroll
  for (int j = 0; j < kTileScanPer; ++j) {
    if (base + j < n_tiles) {
      tile_gt[base + j] = sr;
      tile_eq[base + j] = ebase[j];
    }
    sr += scount[j];
  }
  if ((int)blockIdx.x == n_blocks - 1 && threadIdx.x == 0) st->n_selected = S0 + blk_tot_s;
}

// Ordered flags for one 256-element slab of a wave's chunk: `sel[e]` says
// whether element e of this lane is selected; `pos` is the number of selected
// elements before this lane's first element (within the whole array).
struct ChunkCursor {
  uint32_t sel_run;   // selected before the current slab
  uint32_t eq_run;    // ties before the current slab
};

__device__ __forceinline__ void slab_select(const uint32_t key[4], const bool valid[4],
                                            uint32_t T, uint32_t need, ChunkCursor& cur,
                                            bool sel[4], uint32_t& pos) {
  uint32_t my_eq = 0;
  bool eq[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    eq[e] = valid[e] && key[e] == T;
    my_eq += eq[e];
  }
  uint32_t eq_rank = cur.eq_run;
  const uint64_t any_eq = ballot64(my_eq != 0);
  if (any_eq) {
    const uint32_t incl = wave_incl_scan(my_eq);
    eq_rank += incl - my_eq;
    cur.eq_run += __shfl(incl, kWave - 1, kWave);
  }
  uint32_t my_sel = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    bool s = valid[e] && key[e] > T;
    if (eq[e]) { s = eq_rank < need; ++eq_rank; }
    sel[e] = s;
    my_sel += s;
  }
  const uint32_t incl = wave_incl_scan(my_sel);
  pos = cur.sel_run + incl - my_sel;
  cur.sel_run += __shfl(incl, kWave - 1, kWave);
}

template <class Src>
__global__ __launch_bounds__(kBlock) void k_write_mask(SrcPack<Src> srcs, ChainJobs jobs,
                                                       int64_t tile_base, int unless_settled,
                                                       uint8_t* __restrict__ mask_override) {
  const ChainJob& J = jobs.j[blockIdx.y];
  const SelState* __restrict__ st = J.st;
  if (unless_settled && st->bracket_ok) return;
  Src src = srcs.s[blockIdx.y];
  const int64_t n = J.n;
  const int tie_all = J.tie_all;
  const uint32_t* __restrict__ tile_sel = J.tile_gt;
  const uint32_t* __restrict__ tile_eq = J.tile_eq;
  uint8_t* __restrict__ mask = mask_override ? mask_override : J.mask;
  const bool mvec = aligned4(mask, 1);
  const uint32_t T = st->thresh_bits;
  const uint32_t need = tie_all ? 0xFFFFFFFFu : st->need;
  const int64_t n_chunks = cdiv64(n, kChunk);
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  for (int64_t c = (int64_t)blockIdx.x * kChunksPerBlock + wave_id(); c < n_chunks;
       c += wstride) {
    ChunkCursor cur;
    cur.sel_run = tile_sel[tile_base + c];
    cur.eq_run = tile_eq[tile_base + c];
    const bool full = src.vec && mvec && (c + 1) * kChunk <= n;
    uint32_t key[kChunkIters][4];
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
#pragma unroll
      for (int e = 0; e < 4; ++e) key[it][e] = 0u;
      if (full) src.template load<true>(i, n, key[it]);
      else if (i < n) src.template load<false>(i, n, key[it]);
    }
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
      bool valid[4], sel[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) valid[e] = full || i + e < n;
      uint32_t pos;
      slab_select(key[it], valid, T, need, cur, sel, pos);
      uint32_t mk[4] = {sel[0], sel[1], sel[2], sel[3]};
      if (full) st_u8<true>(mask, i, n, mk, true);
      else if (i < n) store4_u8(mask, i, n, mk, mvec);
    }
  }
}

static __global__ void k_sel_result(ChainJobs jobs) {
  const SelState* st = jobs.j[blockIdx.y].st;
  sga_select_result* out = jobs.j[blockIdx.y].result;
  if (!out) return;
  out->thresh_bits = st->thresh_bits;
  out->need = st->need;
  out->n_gt = st->n_gt;
  out->n_eq = st->n_eq;
  out->n_selected = st->n_selected;
  out->nonfinite = st->nonfinite;
  out->status = st->status;
  out->path = st->path | (st->negative ? 0x100u : 0u) | (st->redone ? 0x200u : 0u);
}

// -------------------------------------------------------------- host drivers
// Grid of the histogram passes over raw key buffers (<= 1M sample keys, ~1e6 candidates whose
// count lives on the device).  What a workgroup costs there is fixed (zeroing and flushing its
// LDS bins, the device-scope fence and ticket of the merged scan): measured, 256 or 1024
// workgroups are 5 and 40 us slower per pass than 64.
constexpr unsigned kRawKeyBlocks = 64;
static inline dim3 hist_grid(int64_t n) {
  return dim3(stream_grid(n, (int64_t)kBlock * kVec * 4, 256 * 8));
}

// Host side of a batched chain: up to kMaxJobs select problems that go through every short
// kernel together.  A single select is a batch of one.
struct SelBatch {
  int count = 0;
  ChainJobs jobs;
  SelWorkspace w[kMaxJobs];
  int64_t max_n = 0, max_tiles = 0, max_nsv = 0;
  // true when the job takes the sampled-bracket path (all jobs of one batch must agree)
  static bool fast_ok(const SelWorkspace& ws, int64_t n) {
    return n >= kFastMinN && ws.sample != nullptr && n < (1ll << 32);
  }
  ChainJob& add(const SelWorkspace& ws, int64_t n, int64_t k, int tie_all) {
    ChainJob& J = jobs.j[count];
    w[count++] = ws;
    J = ChainJob{};
    J.st = ws.st; J.aux = ws.aux; J.hist = ws.hist;
    J.tile_gt = ws.tile_gt; J.tile_eq = ws.tile_eq; J.blk_gt = ws.blk_gt; J.blk_eq = ws.blk_eq;
    J.sample = ws.sample; J.seg_cnt = ws.seg_cnt; J.seg_idx = ws.seg_idx; J.seg_key = ws.seg_key;
    J.cand_idx = ws.cand_idx; J.cand_key = ws.cand_key;
    J.n = n; J.n_tiles = cdiv64(n, kChunk);
    J.n_vec = n / 4;
    J.n_sv = ws.sample_cap / 4 < J.n_vec ? ws.sample_cap / 4 : J.n_vec;
    J.k = (uint32_t)k; J.seg_cap = (uint32_t)ws.seg_cap; J.tie_all = tie_all;
    if (n > max_n) max_n = n;
    if (J.n_tiles > max_tiles) max_tiles = J.n_tiles;
    if (J.n_sv > max_nsv) max_nsv = J.n_sv;
    return J;
  }
  dim3 grid(unsigned gx) const { return dim3(gx, (unsigned)count); }
};

// hist (+ merged scan) of one radix level over the data, for every job of the batch
template <class Src, bool MERGE>
static inline void launch_level_data(const SrcPack<Src>& srcs, const SelBatch& B, int level,
                                     hipStream_t s) {
  const dim3 grid = B.grid(hist_grid(B.max_n).x), block(kBlock);
  if (level == 0) hipLaunchKernelGGL((k_level_hist<Src, 0, MERGE>), grid, block, 0, s, srcs, B.jobs);
  else if (level == 1) hipLaunchKernelGGL((k_level_hist<Src, 1, MERGE>), grid, block, 0, s, srcs, B.jobs);
  else hipLaunchKernelGGL((k_level_hist<Src, 2, MERGE>), grid, block, 0, s, srcs, B.jobs);
}
// the same over the jobs' sample keys (CAND false) or candidate keys (CAND true)
template <bool CAND>
static inline void launch_level_raw(const SelBatch& B, int level, hipStream_t s, unsigned blocks) {
  // the fixed cost per workgroup is paid by every job of the batch at once: with 8 jobs, 16
  // workgroups per job take 86 us for the sample's three levels where 64 take 141
  if (B.count > 1) {
    blocks /= (unsigned)B.count;
    if (blocks < 16) blocks = 16;
  }
  const dim3 grid = B.grid(blocks), block(kBlock);
  if (level == 0) hipLaunchKernelGGL((k_level_hist_raw<0, CAND>), grid, block, 0, s, B.jobs);
  else if (level == 1) hipLaunchKernelGGL((k_level_hist_raw<1, CAND>), grid, block, 0, s, B.jobs);
  else hipLaunchKernelGGL((k_level_hist_raw<2, CAND>), grid, block, 0, s, B.jobs);
}
static inline void launch_level_scan(int level, const SelBatch& B, hipStream_t s) {
  if (level == 0) hipLaunchKernelGGL((k_level_scan<0>), B.grid(1), dim3(kBlock), 0, s, B.jobs);
  else if (level == 1) hipLaunchKernelGGL((k_level_scan<1>), B.grid(1), dim3(kBlock), 0, s, B.jobs);
  else hipLaunchKernelGGL((k_level_scan<2>), B.grid(1), dim3(kBlock), 0, s, B.jobs);
}

template <class Src>
static inline void launch_tile_count(const SrcPack<Src>& srcs, const SelBatch& B, int64_t tile_base,
                                     hipStream_t s) {
  hipLaunchKernelGGL((k_tile_count<Src>), B.grid(stream_grid(B.max_tiles, kChunksPerBlock)),
                     dim3(kBlock), 0, s, srcs, B.jobs, tile_base);
}

static inline void launch_tile_scan(const SelBatch& B, hipStream_t s) {
  const unsigned nb = (unsigned)cdiv64(B.max_tiles, kTileScanSpan);
  hipLaunchKernelGGL(k_tile_sums, B.grid(nb), dim3(kBlock), 0, s, B.jobs);
  hipLaunchKernelGGL(k_tile_apply, B.grid(nb), dim3(kBlock), 0, s, B.jobs);
}

static inline void launch_result(const SelBatch& B, hipStream_t s) {
  hipLaunchKernelGGL(k_sel_result, B.grid(1), dim3(1), 0, s, B.jobs);
}

// ===================================================== sampled-bracket path
// The k-th largest key is bracketed from a small deterministic sample, so
// the full data needs ONE sweep instead of four: that sweep counts, per
// chunk, the keys above the bracket and collects the few keys inside it;
// the exact threshold is then selected among those candidates only.  The
// result is exact for any sample; if the bracket misses the k-th key (or the
// candidate buffers overflow, e.g. on tie-heavy data) a flag routes the work
// to the radix passes, all on the device.

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16; x *= 0x7FEB352Du; x ^= x >> 15; x *= 0x846CA68Bu; x ^= x >> 16;
  return x;
}

// One 4-element vector per window, at a hashed offset; the n_sv windows tile
// ALL n_vec vectors (window j = [j n_vec / n_sv, (j + 1) n_vec / n_sv)): a tail
// that no window covered would bias the sample whenever the last tensors score
// differently from the rest.  `seed` moves the offsets (0: the fixed pattern);
// the select is exact for any of them.
template <class Src>
__global__ __launch_bounds__(kBlock) void k_sample(SrcPack<Src> srcs, ChainJobs jobs) {
  const ChainJob& J = jobs.j[blockIdx.y];
  Src src = srcs.s[blockIdx.y];
  const int64_t n = J.n, n_sv = J.n_sv, n_vec = J.n_vec;
  uint32_t* __restrict__ keys = J.sample;
  const uint32_t seed = J.seed;
  for (int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x; j < n_sv;
       j += (int64_t)gridDim.x * kBlock) {
    const int64_t w0 = j * n_vec / n_sv, w1 = (j + 1) * n_vec / n_sv;
    const int64_t vec = w0 + (int64_t)(mix32((uint32_t)j + seed * 0x9E3779B9u) % (uint32_t)(w1 - w0));
    uint32_t key[4];
    src.template load<false>(vec * 4, n, key);
    U4 o{key[0], key[1], key[2], key[3]};
    *reinterpret_cast<U4*>(keys + j * 4) = o;
  }
}

// First kernel of a select, one workgroup per job: zeroes both histogram sets and the sweep's
// counters, resets the main state to rank k and, on the sampled-bracket path (`fast`), places
// the two ends of the bracket inside the sample at ranks r = k*ns/n -/+ (sigmas * sigma + 8):
// aux[0] descends to the upper end (smaller rank = larger key), aux[1] to the lower end.
static __global__ __launch_bounds__(kBlock) void k_chain_begin(ChainJobs jobs, int fast, double sigmas) {
  const ChainJob& J = jobs.j[blockIdx.y];
  for (int i = threadIdx.x; i < kHistStride * 2; i += blockDim.x) J.hist[i] = 0u;
  if (fast) {
    for (int i = threadIdx.x; i <= kSegWaves + 1; i += blockDim.x) J.seg_cnt[i] = 0u;   // + overflow count
    for (int i = threadIdx.x; i < kSweepParts; i += blockDim.x) { J.blk_gt[i] = 0u; J.blk_eq[i] = 0u; }
    if (J.seg_fail)
      for (int i = threadIdx.x; i < kSegWaves; i += blockDim.x) J.seg_fail[i] = 0u;
  }
  if (threadIdx.x != 0) return;
  SelState z = {};
  z.k = J.k;
  *J.st = z;
  if (!fast) return;
  const double n = (double)J.n, ns = (double)(J.n_sv * 4);
  const double frac = (double)J.k / n;
  const double r = frac * ns;
  const double d = sigmas * sqrt(r * (1.0 - frac) + 1.0) + 8.0;
  SelState hi = {}, lo = {};
  const double rh = floor(r - d), rl = ceil(r + d);
  if (rh < 1.0) hi.skip = 1; else hi.k = (uint32_t)rh;
  if (rl > ns) lo.skip = 1; else lo.k = (uint32_t)rl;
  J.aux[0] = hi;
  J.aux[1] = lo;
}

// The one sweep over the data: a one-shot grid, one 1024-element chunk per
// wave (a capped grid that strides over the chunks reads 15 % slower).  The
// keys inside the bracket are first gathered, in index order, in the wave's
// LDS buffer; at the end of the chunk the wave reserves room for all of them
// with ONE atomic add on the counter of the candidate segment its chunk
// hashes to (kSegWaves counters, so neighbouring waves hit different
// addresses) and copies them there.  A chunk's candidates therefore stay
// contiguous and index-ordered in the list; the order of the chunks inside a
// segment is arbitrary and nothing downstream depends on it.
constexpr int kWaveCandCap = 256;          // candidates one chunk can hold before the sweep gives up

// LDS of one wave of the sweep.
struct SweepLds {
  uint32_t idx[kWaveCandCap];              // the chunk's candidates, index order
  uint32_t key[kWaveCandCap];
  uint32_t planes[kPlaneWordsPerChunk];    // the chunk's 32 plane words ("key above the bracket")
  uint32_t mbytes[kChunk / 4];             // the chunk's mask bytes in element order (mask-byte sweeps)
};

// The flags of a slab live as four wave ballots (element e of every lane), i.e.
// on the scalar unit: counts are popcounts, "any" is a scalar test, and the
// index-ordered position of a flagged element is the number of mask bits
// below its lane over the four ballots plus the lane's own earlier elements.
struct Ballot4 {
  uint64_t m[4];
  __device__ __forceinline__ uint64_t any() const { return m[0] | m[1] | m[2] | m[3]; }
  __device__ __forceinline__ uint32_t count() const {
    return (uint32_t)(__popcll(m[0]) + __popcll(m[1]) + __popcll(m[2]) + __popcll(m[3]));
  }
  __device__ __forceinline__ uint32_t below_lane() const {
    return lanes_below(m[0]) + lanes_below(m[1]) + lanes_below(m[2]) + lanes_below(m[3]);
  }
  __device__ __forceinline__ bool mine(int e) const { return (m[e] >> lane_id()) & 1ull; }
};

// Appends the flagged elements of one slab in index order: put(pos, e).
template <class F>
__device__ __forceinline__ void ballot_append(const Ballot4& f, uint32_t& count, F&& put) {
  if (f.any() == 0) return;                      // scalar branch
  uint32_t pos = count + f.below_lane();
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (f.mine(e)) { put(pos, e); ++pos; }
  count += f.count();
}

// The slab's four "above" ballots are eight of the chunk's 32 plane words
// (words 8 it + 2 e + h): one lane parks them in the wave's LDS planes, from
// where the chunk's 128 bytes are stored in one piece.
__device__ __forceinline__ void plane_put(const Ballot4& a, int it, uint32_t* lds_planes) {
  if (lane_id() == 0) {
    uint64_t* w = reinterpret_cast<uint64_t*>(lds_planes) + it * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = a.m[e];
  }
}

// One chunk of the sweep.  chi / tot_nf / mycnt are wave totals (scalar).
// PM: 0 counts only; 1 the provisional selection (keys above the bracket) also goes out as bit
// planes; 2 as mask bytes, straight into the caller's mask (a mask-only select then needs no
// expansion pass: the candidates are settled in the bytes).
template <class Src, bool FULL, int PM>
__device__ __forceinline__ void bracket_chunk(Src& src, const typename Src::Chunk& ck, int64_t n,
                                              int64_t c, uint32_t T_LO,
                                              uint32_t T_HI, uint32_t& chi, uint32_t& tot_nf,
                                              uint32_t& mycnt, SweepLds& lds,
                                              uint32_t* __restrict__ pbits,
                                              uint8_t* __restrict__ mask_bytes = nullptr,
                                              bool mvec = false, bool m16 = false) {
  // The loads of kAhead slabs (256 elements each) are issued together, then
  // their keys are formed slab by slab: expensive key sources (Adam-normalised
  // scores) look fewer slabs ahead to stay within their register budget.  The
  // ragged path (last chunk, unaligned views) goes one slab at a time through
  // a rolled loop: it only has to be small.
  constexpr int kAhead = FULL ? Src::kAhead : 1;
  static_assert(kChunkIters % kAhead == 0, "look-ahead divides the slabs of a chunk");
  constexpr int kGroupUnroll = kAhead == kChunkIters ? kChunkIters : 1;
  src.chunk_hyper(c);        // measured: looking the tensor up behind the first loads instead is slower
#pragma unroll kGroupUnroll
  for (int g0 = 0; g0 < kChunkIters; g0 += kAhead) {
    typename Src::Raw raw[kAhead];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int64_t i = c * kChunk + (g0 + u) * (kWave * kVec) + lane_id() * kVec;
      if (FULL || i < n) src.template fetch<FULL>(ck, i, n, raw[u]);
    }
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int it = g0 + u;
      const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
      uint32_t key[4] = {0u, 0u, 0u, 0u};
      if (FULL || i < n) src.template keys<FULL>(ck, i, n, raw[u], key);
      Ballot4 above, cand;
      uint64_t nf = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint64_t valid = FULL ? ~0ull : ballot64(i + e < n);
        above.m[e] = ballot64(key[e] >= T_HI) & valid;
        cand.m[e] = ballot64(key[e] >= T_LO) & valid & ~above.m[e];
        nf |= ballot64(key[e] >= 0x7F800000u) & valid;
      }
      chi += above.count();
      if (nf) {                                  // rare: count them properly
#pragma unroll
        for (int e = 0; e < 4; ++e)
          tot_nf += (uint32_t)__popcll(ballot64(key[e] >= 0x7F800000u && (FULL || i + e < n)));
      }
      ballot_append(cand, mycnt, [&](uint32_t pos, int e) {
        if (pos < (uint32_t)kWaveCandCap) { lds.idx[pos] = (uint32_t)(i + e); lds.key[pos] = key[e]; }
      });
      // provisional mask as bit planes: everything above the bracket is
      // certainly selected; the few keys inside it are settled after the
      // candidate descent.  One 128-byte store per chunk.
      if (PM == 1) plane_put(above, it, lds.planes);
      if (PM == 2 && (FULL || i < n)) {
        const uint32_t mk[4] = {above.mine(0), above.mine(1), above.mine(2), above.mine(3)};
        // a lane's four bytes per slab are parked in LDS in element order, and the chunk's 1024
        // bytes leave as one 16-byte store per lane (four 4-byte stores per lane otherwise)
        if (FULL && m16) lds.mbytes[it * kWave + lane_id()] = mk[0] | (mk[1] << 8) | (mk[2] << 16) | (mk[3] << 24);
        else if (FULL && mvec) st_u8<true>(mask_bytes, i, n, mk, true);
        else store4_u8(mask_bytes, i, n, mk, mvec);
      }
    }
  }
  if (PM == 1) {
    __builtin_amdgcn_wave_barrier();
    if (lane_id() < kPlaneWordsPerChunk) pbits[c * kPlaneWordsPerChunk + lane_id()] = lds.planes[lane_id()];
  }
  if (PM == 2 && FULL && m16) {
    __builtin_amdgcn_wave_barrier();
    const U4 v = reinterpret_cast<const U4*>(lds.mbytes)[lane_id()];
    *reinterpret_cast<U4*>(mask_bytes + c * kChunk + lane_id() * 16) = v;
  }
}

template <class Src, int PM>
__global__ __launch_bounds__(kBlock) void k_bracket_sweep(
    Src src, int64_t n, SelState* __restrict__ st, const SelState* __restrict__ aux,
    uint32_t* __restrict__ tile_gt, uint32_t* __restrict__ tile_eq, uint32_t* __restrict__ seg_idx,
    uint32_t* __restrict__ seg_key, uint32_t* __restrict__ seg_cnt, uint32_t seg_cap,
    uint32_t* __restrict__ pbits, uint32_t* __restrict__ hi_part, uint32_t* __restrict__ nf_part,
    uint8_t* __restrict__ mask_bytes = nullptr, bool mvec = false) {
  const bool m16 = PM == 2 && (reinterpret_cast<uintptr_t>(mask_bytes) & 15) == 0;
  __shared__ uint32_t s_hi[kChunksPerBlock], s_nf[kChunksPerBlock];
  __shared__ SweepLds s_lds[kChunksPerBlock];
  // keys equal to the upper sample key stay candidates; a skipped end means
  // the bracket is open on that side
  const uint32_t T_HI = aux[0].skip ? 0x80000000u : aux[0].thresh_bits + 1u;
  const uint32_t T_LO = aux[1].skip ? 0u : aux[1].thresh_bits;
  if (blockIdx.x == 0 && threadIdx.x == 0) { st->t_lo = T_LO; st->t_hi = T_HI; }
  const int64_t n_chunks = cdiv64(n, kChunk);
  const int64_t c = (int64_t)blockIdx.x * kChunksPerBlock + wave_id();
  uint32_t chi = 0, tot_nf = 0;
  if (c < n_chunks) {
    uint32_t mycnt = 0;
    SweepLds& lds = s_lds[wave_id()];
    uint32_t* const my_idx = lds.idx;
    uint32_t* const my_key = lds.key;
    const typename Src::Chunk ck = src.chunk_begin(c);
    if (src.vec && (c + 1) * kChunk <= n)
      bracket_chunk<Src, true, PM>(src, ck, n, c, T_LO, T_HI, chi, tot_nf, mycnt, lds, pbits, mask_bytes, mvec, m16);
    else
      bracket_chunk<Src, false, PM>(src, ck, n, c, T_LO, T_HI, chi, tot_nf, mycnt, lds, pbits, mask_bytes, mvec);
    if (lane_id() == 0) { tile_gt[c] = chi; tile_eq[c] = 0u; }     // chi / tot_nf are wave totals
    if (mycnt) {                                        // wave-uniform
      const uint32_t seg = (uint32_t)c & (uint32_t)(kSegWaves - 1);
      uint32_t base = 0;
      if (lane_id() == 0) base = atomicAdd(&seg_cnt[seg], mycnt);   // a segment over its capacity is seen by the check
      base = __shfl(base, 0, kWave);
      if (mycnt > (uint32_t)kWaveCandCap) {
        if (lane_id() == 0) atomicOr(&st->overflow, 1u);
      } else {
        __builtin_amdgcn_wave_barrier();                // the wave's LDS stores above are read below
        uint32_t* const g_idx = seg_idx + (int64_t)seg * seg_cap;
        uint32_t* const g_key = seg_key + (int64_t)seg * seg_cap;
        for (uint32_t j = lane_id(); j < mycnt; j += kWave)
          if (base + j < seg_cap) { g_idx[base + j] = my_idx[j]; g_key[base + j] = my_key[j]; }
      }
    }
  }
  note_negative(src, st);
  if (lane_id() == 0) { s_hi[wave_id()] = chi; s_nf[wave_id()] = tot_nf; }
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t h = s_hi[0] + s_hi[1] + s_hi[2] + s_hi[3];
    const uint32_t f = s_nf[0] + s_nf[1] + s_nf[2] + s_nf[3];
    if (h) atomicAdd(&hi_part[blockIdx.x & (kSweepParts - 1)], h);
    if (f) atomicAdd(&nf_part[blockIdx.x & (kSweepParts - 1)], f);
  }
}

// Single workgroup: segment counts -> offsets, validate the bracket, arm the
// candidate descent (aux) or the radix passes (st->skip == 0).
static __global__ __launch_bounds__(kBlock) void k_bracket_check(ChainJobs jobs) {
  __shared__ uint32_t s_w4[kChunksPerBlock];
  const ChainJob& J = jobs.j[blockIdx.y];
  SelState* __restrict__ st = J.st;
  SelState* __restrict__ aux = J.aux;
  uint32_t* __restrict__ seg_cnt = J.seg_cnt;
  uint32_t* __restrict__ hist = J.hist;
  constexpr int nhist = kHistStride * 2;
  const uint32_t seg_cap = J.seg_cap;
  const uint32_t* __restrict__ hi_part = J.blk_gt;
  const uint32_t* __restrict__ nf_part = J.blk_eq;
  const int spec = J.spec;
  const uint32_t ovf_cap = J.ovf_cap;
  const uint32_t* __restrict__ seg_fail = J.seg_fail;
  constexpr int PER = kSegWaves / kBlock;   // 32
  uint32_t v[PER], mine = 0, over = 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    uint32_t cnt = seg_cnt[threadIdx.x * PER + j];
    if (seg_fail && cnt > seg_cap) {
      // single-sweep step: reservations are never taken back, the segment's records end where
      // the first reservation that did not fit began (the later ones went to the overflow list)
      cnt = 0xFFFFFFFFu - seg_fail[threadIdx.x * PER + j];
    }
    over |= cnt > seg_cap;                    // the sweep reserved more than the segment holds
    v[j] = cnt < seg_cap ? cnt : seg_cap;
    mine += v[j];
  }
  uint32_t total;
  uint32_t run = block_excl_scan(mine, s_w4, total);
#pragma unroll
  for (int j = 0; j < PER; ++j) { seg_cnt[threadIdx.x * PER + j] = run; run += v[j]; }
  for (int i = threadIdx.x; i < nhist; i += kBlock) hist[i] = 0u;
  static_assert(kSweepParts == kBlock, "one partial counter per thread");
  uint32_t dummy;
  __syncthreads();
  block_excl_scan(hi_part[threadIdx.x], s_w4, dummy);
  const uint32_t n_hi = dummy;
  __syncthreads();
  block_excl_scan(nf_part[threadIdx.x], s_w4, dummy);
  const uint32_t n_nf = dummy;
  __syncthreads();
  block_excl_scan(over, s_w4, dummy);
  const bool any_over = dummy != 0;
  if (threadIdx.x == 0) {
    seg_cnt[kSegWaves] = total;       // where the overflow list's records go in the dense list
    bool ovf_over = false;
    if (ovf_cap) {                    // single-sweep step: records of the shared overflow list
      const uint32_t oc = seg_cnt[kSegWaves + 1];
      ovf_over = oc > ovf_cap || (uint64_t)total + oc > (uint64_t)kSegWaves * seg_cap;
      total += oc < ovf_cap ? oc : ovf_cap;
    }
    const uint32_t k = st->k;
    const bool ok = !st->overflow && !any_over && !ovf_over && n_hi < k && k <= n_hi + total;
    st->n_hi = n_hi;
    st->cand_count = total;
    // A single-sweep step that went ahead IN PLACE has already committed on the bracket: a miss
    // cannot be repaired by the radix passes, it is reported (status 3) and nothing further
    // runs.  Out of place (spec == 2) the inputs are untouched: the miss is an ordinary failed
    // bracket, the radix passes and the key-forming final sweep redo the step over what the
    // sweep wrote, and `redone` says so.
    const bool missed = spec && st->spec && !ok;
    const bool lost = missed && spec != 2;
    if (missed && spec == 2) { st->spec = 0u; st->redone = 1u; }
    st->bracket_ok = ok ? 1u : 0u;
    st->skip = (ok || lost) ? 1u : 0u;   // the radix passes run only when the bracket failed
    st->path = ok ? (spec ? 2u : 1u) : 0u;
    st->nonfinite = ok ? n_nf : 0u;   // recounted by the radix passes otherwise
    if (!ok) st->status = lost ? 3u : 0u;
    SelState z = {};
    z.k = ok ? k - n_hi : 0u;
    z.skip = ok ? 0u : 1u;
    aux[0] = z;                       // the candidate descent runs on aux[0]
  }
}

// Dense candidate list from the per-wave segments (order: wave, then index).
static __global__ __launch_bounds__(kBlock) void k_cand_compact(ChainJobs jobs) {
  const ChainJob& J = jobs.j[blockIdx.y];
  if (J.aux->skip) return;
  const uint32_t* __restrict__ seg_off = J.seg_cnt;
  const uint32_t* __restrict__ seg_idx = J.seg_idx;
  const uint32_t* __restrict__ seg_key = J.seg_key;
  const uint32_t seg_cap = J.seg_cap;
  uint32_t* __restrict__ cand_idx = J.cand_idx;
  uint32_t* __restrict__ cand_key = J.cand_key;
  const F4* __restrict__ seg_rec = J.seg_rec;
  F4* __restrict__ cand_rec = J.cand_rec;
  for (int w = blockIdx.x * kChunksPerBlock + wave_id(); w < kSegWaves;
       w += gridDim.x * kChunksPerBlock) {
    const uint32_t off = seg_off[w], cnt = seg_off[w + 1] - off;
    for (uint32_t j = lane_id(); j < cnt; j += kWave) {
      cand_idx[off + j] = seg_idx[(int64_t)w * seg_cap + j];
      cand_key[off + j] = seg_key[(int64_t)w * seg_cap + j];
      if (seg_rec) cand_rec[off + j] = seg_rec[(int64_t)w * seg_cap + j];
    }
  }
}

// After the candidate descent: publish the exact threshold and fold each
// candidate into its chunk's (above, equal) counts.
static __global__ __launch_bounds__(kBlock) void k_cand_tiles(ChainJobs jobs) {
  const ChainJob& J = jobs.j[blockIdx.y];
  SelState* __restrict__ st = J.st;
  const SelState* __restrict__ aux = J.aux;
  if (aux->skip) return;
  const uint32_t* __restrict__ cand_idx = J.cand_idx;
  const uint32_t* __restrict__ cand_key = J.cand_key;
  uint32_t* __restrict__ tile_gt = J.tile_gt;
  uint32_t* __restrict__ tile_eq = J.tile_eq;
  const uint32_t T = aux->thresh_bits;
  const uint32_t nc = st->cand_count;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    st->thresh_bits = T;
    st->need = aux->need;
    st->n_eq = aux->n_eq;
    st->n_gt = st->k - aux->need;
    st->status = aux->status;
  }
  for (uint32_t j = blockIdx.x * kBlock + threadIdx.x; j < nc; j += gridDim.x * kBlock) {
    const uint32_t key = cand_key[j];
    if (key > T) atomicAdd(&tile_gt[cand_idx[j] >> 10], 1u);
    else if (key == T) atomicAdd(&tile_eq[cand_idx[j] >> 10], 1u);
  }
}
static_assert(kChunk == 1024, "candidate -> chunk mapping uses idx >> 10");

// Bit planes of the bracket sweep -> mask bytes (keys above the bracket).
// Each lane expands 16 consecutive bytes: 4 lanes x 4 elements of one slab.
static __global__ __launch_bounds__(kBlock) void k_expand_mask(
    const SelState* __restrict__ st, const uint32_t* __restrict__ pbits, int64_t n,
    uint8_t* __restrict__ mask, bool mvec, const uint32_t* __restrict__ pbits2 = nullptr) {
  if (st && !st->bracket_ok) return;
  const int64_t n_chunks = cdiv64(n, kChunk);
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  const int l = lane_id();
  const int it = l >> 4, sl0 = (l & 15) * 4;        // slab, first slab-lane
  for (int64_t c = (int64_t)blockIdx.x * kChunksPerBlock + wave_id(); c < n_chunks; c += wstride) {
    const U4* pw = reinterpret_cast<const U4*>(pbits + c * 32 + it * 8);
    U4 lo = pw[0], hi = pw[1];
    if (pbits2) {                                   // union of two planes
      const U4* qw = reinterpret_cast<const U4*>(pbits2 + c * 32 + it * 8);
      const U4 l2 = qw[0], h2 = qw[1];
      lo = U4{lo.x | l2.x, lo.y | l2.y, lo.z | l2.z, lo.w | l2.w};
      hi = U4{hi.x | h2.x, hi.y | h2.y, hi.z | h2.z, hi.w | h2.w};
    }
    const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    uint32_t out[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {                   // slab-lane sl0 + j -> 4 bytes
      const int sl = sl0 + j;
      uint32_t v = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        v |= (((sl < 32 ? w[2 * e] : w[2 * e + 1]) >> (sl & 31)) & 1u) << (8 * e);
      out[j] = v;
    }
    const int64_t i = c * kChunk + (int64_t)l * 16;
    if (mvec && i + 16 <= n) {
      *reinterpret_cast<U4*>(mask + i) = U4{out[0], out[1], out[2], out[3]};
    } else {
      for (int b = 0; b < 16; ++b)
        if (i + b < n) mask[i + b] = (uint8_t)((out[b >> 2] >> (8 * (b & 3))) & 1u);
    }
  }
}

// Settles the bracket's candidates in the expanded mask: keys above the
// threshold are selected; of the ties, the first `need` by index.  After the
// tile scan tile_eq[c] counts the ties before chunk c, so only the one chunk
// where the quota runs out has to rank its ties (a chunk's candidates are
// contiguous and index-ordered in the list).
static __global__ __launch_bounds__(kBlock) void k_cand_mask(ChainJobs jobs) {
  const ChainJob& J = jobs.j[blockIdx.y];
  const SelState* __restrict__ st = J.st;
  if (!st->bracket_ok) return;
  const uint32_t* __restrict__ cand_idx = J.cand_idx;
  const uint32_t* __restrict__ cand_key = J.cand_key;
  const uint32_t* __restrict__ tile_eq = J.tile_eq;
  const int64_t n_tiles = J.n_tiles;
  const int tie_all = J.tie_all;
  uint8_t* __restrict__ mask = J.mask;
  const uint32_t T = st->thresh_bits, nc = st->cand_count, n_eq = st->n_eq;
  const uint32_t need = tie_all ? 0xFFFFFFFFu : st->need;
  for (uint32_t j = blockIdx.x * kBlock + threadIdx.x; j < nc; j += gridDim.x * kBlock) {
    const uint32_t key = cand_key[j];
    if (key < T) continue;
    const uint32_t idx = cand_idx[j];
    bool on = true;
    if (key == T && need < n_eq) {
      const uint32_t c = idx >> 10;
      const uint32_t before = tile_eq[c];
      const uint32_t upto = (int64_t)c + 1 < n_tiles ? tile_eq[c + 1] : n_eq;
      if (before >= need) {
        on = false;
      } else if (upto > need) {            // the quota ends inside this chunk
        uint32_t rank = before;
        for (uint32_t q = j; q > 0 && (cand_idx[q - 1] >> 10) == c; --q)
          rank += cand_key[q - 1] == T;
        on = rank < need;
      }
    }
    if (on) mask[idx] = 1;
  }
}

// The same settlement when the mask itself is kept as bit planes.
static __global__ __launch_bounds__(kBlock) void k_cand_bits(ChainJobs jobs) {
  const ChainJob& J = jobs.j[blockIdx.y];
  const SelState* __restrict__ st = J.st;
  if (!st->bracket_ok) return;
  const uint32_t* __restrict__ cand_idx = J.cand_idx;
  const uint32_t* __restrict__ cand_key = J.cand_key;
  const uint32_t* __restrict__ tile_eq = J.tile_eq;
  const int64_t n_tiles = J.n_tiles;
  const int tie_all = J.tie_all;
  uint32_t* __restrict__ planes = J.planes;
  const uint32_t T = st->thresh_bits, nc = st->cand_count, n_eq = st->n_eq;
  const uint32_t need = tie_all ? 0xFFFFFFFFu : st->need;
  for (uint32_t j = blockIdx.x * kBlock + threadIdx.x; j < nc; j += gridDim.x * kBlock) {
    const uint32_t key = cand_key[j];
    if (key < T) continue;
    const uint32_t idx = cand_idx[j];
    bool on = true;
    if (key == T && need < n_eq) {
      const uint32_t c = idx >> 10;
      const uint32_t before = tile_eq[c];
      const uint32_t upto = (int64_t)c + 1 < n_tiles ? tile_eq[c + 1] : n_eq;
      if (before >= need) {
        on = false;
      } else if (upto > need) {
        uint32_t rank = before;
        for (uint32_t q = j; q > 0 && (cand_idx[q - 1] >> 10) == c; --q)
          rank += cand_key[q - 1] == T;
        on = rank < need;
      }
    }
    if (on) {
      const uint32_t lane = (idx >> 2) & 63u, e = idx & 3u;
      atomicOr(&planes[(idx >> 8) * 8 + 2 * e + (lane >> 5)], 1u << (lane & 31));
    }
  }
}

// Ordered full pass that writes the mask as bit planes (the fallback of
// k_cand_bits when the sampled bracket failed or was never tried).
template <class Src>
__global__ __launch_bounds__(kBlock) void k_write_bits(SrcPack<Src> srcs, ChainJobs jobs) {
  const ChainJob& J = jobs.j[blockIdx.y];
  const SelState* __restrict__ st = J.st;
  if (st->bracket_ok) return;
  Src src = srcs.s[blockIdx.y];
  const int64_t n = J.n;
  const int tie_all = J.tie_all;
  const uint32_t* __restrict__ tile_sel = J.tile_gt;
  const uint32_t* __restrict__ tile_eq = J.tile_eq;
  uint32_t* __restrict__ planes = J.planes;
  const uint32_t T = st->thresh_bits;
  const uint32_t need = tie_all ? 0xFFFFFFFFu : st->need;
  const int64_t n_chunks = cdiv64(n, kChunk);
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  for (int64_t c = (int64_t)blockIdx.x * kChunksPerBlock + wave_id(); c < n_chunks; c += wstride) {
    ChunkCursor cur;
    cur.sel_run = tile_sel[c];
    cur.eq_run = tile_eq[c];
    const bool full = src.vec && (c + 1) * kChunk <= n;
    uint32_t word = 0u;
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
      uint32_t key[4] = {0u, 0u, 0u, 0u};
      if (full) src.template load<true>(i, n, key);
      else if (i < n) src.template load<false>(i, n, key);
      bool valid[4], sel[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) valid[e] = full || i + e < n;
      uint32_t pos;
      slab_select(key, valid, T, need, cur, sel, pos);
      const uint32_t flag[4] = {sel[0], sel[1], sel[2], sel[3]};
      plane_collect(flag, it, word);
    }
    if (lane_id() < 32) planes[c * kPlaneWordsPerChunk + lane_id()] = word;
  }
}

// Byte mask -> bit planes (chunk-structured, planes sized for cdiv(n, 1024) chunks).
static __global__ __launch_bounds__(kBlock) void k_mask_to_planes(const uint8_t* __restrict__ mask,
                                                                  int64_t n,
                                                                  uint32_t* __restrict__ planes,
                                                                  bool mvec) {
  const int64_t n_chunks = cdiv64(n, kChunk);
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  for (int64_t c = (int64_t)blockIdx.x * kChunksPerBlock + wave_id(); c < n_chunks; c += wstride) {
    uint32_t word = 0u;
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
      uint32_t mk[4] = {0u, 0u, 0u, 0u};
      if (i < n) load4_u8(mask, i, n, mk, mvec);
      plane_collect(mk, it, word);
    }
    if (lane_id() < 32) planes[c * kPlaneWordsPerChunk + lane_id()] = word;
  }
}

// The select of every job of a batch: begin -> (sampled-bracket path: sample, dual-rank descent,
// ONE data sweep per job, check, candidate compaction and descent, per-chunk counts) -> the radix
// passes (no-ops unless a job's bracket failed) -> chunk scan.  The short kernels run once for
// the whole batch; only the data sweeps are launched per job.
// PM: what the sweep leaves behind for a mask-only caller -- 0 nothing, 1 the keys above the
// bracket as bit planes (job.planes), 2 as mask bytes (job.mask) -- to be finished by
// finish_planes / finish_mask from those bits and the candidates instead of re-reading the data.
// All jobs of a batch take the same path (`fast`: SelBatch::fast_ok for every one of them).
//
// The chain comes in phases so that a batch whose jobs form their keys differently (the
// re-selections of a replay step rank by different scores) still shares every kernel that does
// not form keys: chain_begin, chain_sample_levels, chain_candidates, launch_tile_scan (and the
// settlement) take the whole batch; chain_sample, chain_sweeps and chain_fallback are templates
// of the key source and take the jobs of one kind (a sub-batch over the same workspaces).
static inline void chain_begin(const SelBatch& B, bool fast, hipStream_t s, double sigmas = 5.0) {
  hipLaunchKernelGGL(k_chain_begin, B.grid(1), dim3(kBlock), 0, s, B.jobs, fast ? 1 : 0, sigmas);
}
template <class Src>
static inline void chain_sample(const SrcPack<Src>& srcs, const SelBatch& B, hipStream_t s) {
  static_assert(sizeof(ChainJobs) + sizeof(SrcPack<Src>) + 64 <= 4096,
                "the operands of a batched chain kernel travel in its 4 KiB of kernel arguments");
  hipLaunchKernelGGL((k_sample<Src>), B.grid(stream_grid(B.max_nsv, kBlock)), dim3(kBlock), 0, s,
                     srcs, B.jobs);
}
static inline void chain_sample_levels(const SelBatch& B, hipStream_t s) {
  for (int level = 0; level < 3; ++level) launch_level_raw<false>(B, level, s, kRawKeyBlocks);
}
template <class Src>
static inline void chain_sweeps(const SrcPack<Src>& srcs, const SelBatch& B, int pm, hipStream_t s) {
  for (int b = 0; b < B.count; ++b) {
    const ChainJob& J = B.jobs.j[b];
    const SelWorkspace& w = B.w[b];
    const unsigned sweep_blocks = (unsigned)cdiv64(J.n_tiles, kChunksPerBlock);
    ProfPair* pp = prof_begin(SGA_PROF_SELECT_SWEEP, s);
    // the sweep's two totals go through 256 partial counters (blk_gt / blk_eq are free until
    // the tile scan, which runs after the check has read them)
    if (pm == 2)
      hipLaunchKernelGGL((k_bracket_sweep<Src, 2>), dim3(sweep_blocks), dim3(kBlock), 0, s,
                         srcs.s[b], J.n, w.st, w.aux, w.tile_gt, w.tile_eq, w.seg_idx, w.seg_key,
                         w.seg_cnt, (uint32_t)w.seg_cap, (uint32_t*)nullptr, w.blk_gt, w.blk_eq,
                         J.mask, (reinterpret_cast<uintptr_t>(J.mask) & 3) == 0);
    else if (pm == 1)
      hipLaunchKernelGGL((k_bracket_sweep<Src, 1>), dim3(sweep_blocks), dim3(kBlock), 0, s,
                         srcs.s[b], J.n, w.st, w.aux, w.tile_gt, w.tile_eq, w.seg_idx, w.seg_key,
                         w.seg_cnt, (uint32_t)w.seg_cap, J.planes, w.blk_gt, w.blk_eq);
    else
      hipLaunchKernelGGL((k_bracket_sweep<Src, 0>), dim3(sweep_blocks), dim3(kBlock), 0, s,
                         srcs.s[b], J.n, w.st, w.aux, w.tile_gt, w.tile_eq, w.seg_idx, w.seg_key,
                         w.seg_cnt, (uint32_t)w.seg_cap, (uint32_t*)nullptr, w.blk_gt, w.blk_eq);
    prof_end(pp, s);
  }
}
static inline void chain_candidates(const SelBatch& B, hipStream_t s) {
  hipLaunchKernelGGL(k_bracket_check, B.grid(1), dim3(kBlock), 0, s, B.jobs);
  hipLaunchKernelGGL(k_cand_compact, B.grid(256), dim3(kBlock), 0, s, B.jobs);
  // a batch's candidate lists are as long as a single select's (millions of keys each at large
  // sizes and ratios): 256 workgroups for the batch, where the sample's short passes take 64
  // (four re-selections of the 596 M-element replay set: 97 us for the three levels, 203 with 64)
  for (int level = 0; level < 3; ++level)
    launch_level_raw<true>(B, level, s, B.count > 1 ? 4 * kRawKeyBlocks : kRawKeyBlocks);
  hipLaunchKernelGGL(k_cand_tiles, B.grid(256), dim3(kBlock), 0, s, B.jobs);
}
// The radix passes and the per-chunk counts over the data: no-ops unless a job's bracket failed
// (st->skip == 0; k_bracket_check left the histograms zeroed for them) or was never tried.
template <class Src>
static inline void chain_fallback(const SrcPack<Src>& srcs, const SelBatch& B, hipStream_t s) {
  for (int level = 0; level < 3; ++level) launch_level_data<Src, true>(srcs, B, level, s);
  launch_tile_count(srcs, B, 0, s);
}

template <class Src>
static inline void run_select_batch(const SrcPack<Src>& srcs, const SelBatch& B, bool fast, int pm,
                                    hipStream_t s, double sigmas = 5.0) {
  chain_begin(B, fast, s, sigmas);
  if (fast) {
    chain_sample(srcs, B, s);
    chain_sample_levels(B, s);
    chain_sweeps(srcs, B, pm, s);
    chain_candidates(B, s);
  }
  chain_fallback(srcs, B, s);
  launch_tile_scan(B, s);
}

// Bit-plane masks of the selections after run_select_batch(..., pm = 1): the candidates settle
// the sweep's planes when the bracket held, else the ordered full pass writes them.
template <class Src>
static inline void finish_planes_batch(const SrcPack<Src>& srcs, const SelBatch& B, bool fast,
                                       hipStream_t s) {
  if (fast) hipLaunchKernelGGL(k_cand_bits, B.grid(256), dim3(kBlock), 0, s, B.jobs);
  hipLaunchKernelGGL((k_write_bits<Src>), B.grid(stream_grid(B.max_tiles, kChunksPerBlock, 1 << 14)),
                     dim3(kBlock), 0, s, srcs, B.jobs);
}

// Byte masks after run_select_batch(..., pm = 2) (the sweep wrote the provisional selection
// straight into the caller's mask): the candidates settle it when the bracket held, else the
// ordered full pass writes it.
template <class Src>
static inline void finish_mask_batch(const SrcPack<Src>& srcs, const SelBatch& B, bool fast,
                                     hipStream_t s) {
  if (fast) hipLaunchKernelGGL(k_cand_mask, B.grid(256), dim3(kBlock), 0, s, B.jobs);
  hipLaunchKernelGGL((k_write_mask<Src>), B.grid(stream_grid(B.max_tiles, kChunksPerBlock, 1 << 14)),
                     dim3(kBlock), 0, s, srcs, B.jobs, (int64_t)0, fast ? 1 : 0, (uint8_t*)nullptr);
}

#endif  // __HIPCC__
}  // namespace sga
