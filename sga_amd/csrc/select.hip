// Exact top-k selection entry points over fp32 score arrays, plus the
// histogram / candidate / compare building blocks of the replay select.
#include "select_impl.hpp"

namespace sga {
int exclusive_scan_u32(uint32_t* data, int64_t n, int64_t* total, hipStream_t st);
int64_t scan_scratch_entries(int64_t n);

// int64 histogram of (|x| bits >> shift) over a strided subsample; bins in
// LDS when they fit (4097 coarse bins), otherwise straight to global.
__global__ __launch_bounds__(kBlock) void k_hist_topbits(
    const float* __restrict__ x, int64_t n, int shift, int stride, int phase,
    unsigned long long* __restrict__ hist, int nbins, uint32_t* __restrict__ nonfinite) {
  extern __shared__ uint32_t s_h[];
  for (int b = threadIdx.x; b < nbins; b += kBlock) s_h[b] = 0u;
  __syncthreads();
  const int64_t n_s = n <= phase ? 0 : (n - phase + stride - 1) / stride;
  uint32_t nf = 0;
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t base = (int64_t)blockIdx.x * kBlock; base < n_s; base += step) {
    const int64_t j = base + threadIdx.x;
    const bool ok = j < n_s;
    uint32_t key = 0;
    if (ok) key = abs_key(x[phase + j * stride]);
    nf += (ok && key >= 0x7F800000u);
    uint32_t bin = key >> shift;
    if (bin >= (uint32_t)nbins) bin = nbins - 1;
    lds_hist_add(s_h, bin, ok);
  }
  __syncthreads();
  for (int b = threadIdx.x; b < nbins; b += kBlock) {
    const uint32_t c = s_h[b];
    if (c) atomicAdd(&hist[b], (unsigned long long)c);
  }
  nf = wave_sum(nf);
  if (lane_id() == 0 && nf && nonfinite) atomicAdd(nonfinite, nf);
}

// Same histogram over every element of a 16-byte aligned array: 1024 lanes share one LDS table (the
// 128 KiB of 32769 bins leave room for one workgroup per CU, so the workgroup is made as wide as it
// can be), and each lane keeps two 16-byte loads in flight per trip.
constexpr int kHistWide = 1024;
__global__ __launch_bounds__(kHistWide) void k_hist_topbits_dense(
    const float* __restrict__ x, int64_t n, int shift, unsigned long long* __restrict__ hist,
    int nbins, uint32_t* __restrict__ nonfinite) {
  extern __shared__ uint32_t s_h[];
  for (int b = threadIdx.x; b < nbins; b += kHistWide) s_h[b] = 0u;
  __syncthreads();
  uint32_t nf = 0;
  constexpr int64_t kSlab = (int64_t)kHistWide * kVec;
  const int64_t step = (int64_t)gridDim.x * kSlab * 2;
  // trip count is uniform over the workgroup: the ballots inside lds_hist_add need whole waves
  for (int64_t base = (int64_t)blockIdx.x * kSlab * 2; base < n; base += step) {
    float v[2][4];
    const int64_t i0 = base + (int64_t)threadIdx.x * kVec;
#pragma unroll
    for (int u = 0; u < 2; ++u) load4_f32(x, i0 + u * kSlab, n, v[u], true);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool ok = i0 + u * kSlab + e < n;
        const uint32_t key = ok ? abs_key(v[u][e]) : 0u;
        nf += (ok && key >= 0x7F800000u);
        uint32_t bin = key >> shift;
        if (bin >= (uint32_t)nbins) bin = nbins - 1;
        lds_hist_add(s_h, bin, ok);
      }
    }
  }
  __syncthreads();
  for (int b = threadIdx.x; b < nbins; b += kHistWide) {
    const uint32_t c = s_h[b];
    if (c) atomicAdd(&hist[b], (unsigned long long)c);
  }
  nf = wave_sum(nf);
  if (lane_id() == 0 && nf && nonfinite) atomicAdd(nonfinite, nf);
}

__global__ __launch_bounds__(kBlock) void k_mask_topbits_ge(
    const float* __restrict__ x, int64_t n, int shift, uint32_t bin,
    uint8_t* __restrict__ mask, bool vec) {
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  for (int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * kVec; i < n; i += stride) {
    float v[4];
    load4_f32(x, i, n, v, vec);
    uint32_t mk[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) mk[e] = (abs_key(v[e]) >> shift) >= bin;
    store4_u8(mask, i, n, mk, vec);
  }
}

// Candidates of one top-16 bin, in ascending index order (two sweeps).
__global__ __launch_bounds__(kBlock) void k_cand_count(
    const float* __restrict__ x, int64_t n, uint32_t bin, uint32_t* __restrict__ counts,
    int64_t n_chunks, bool vec) {
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  for (int64_t c = (int64_t)blockIdx.x * kChunksPerBlock + wave_id(); c < n_chunks; c += wstride) {
    uint32_t cnt = 0;
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
      float v[4] = {0, 0, 0, 0};
      if (i < n) load4_f32(x, i, n, v, vec);
#pragma unroll
      for (int e = 0; e < 4; ++e) cnt += (i + e < n && (abs_key(v[e]) >> 16) == bin);
    }
    cnt = wave_sum(cnt);
    if (lane_id() == 0) counts[c] = cnt;
  }
}

__global__ __launch_bounds__(kBlock) void k_cand_fill(
    const float* __restrict__ x, int64_t n, uint32_t bin, const uint32_t* __restrict__ offsets,
    float* __restrict__ cand, int64_t cap, int64_t n_chunks, bool vec) {
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  for (int64_t c = (int64_t)blockIdx.x * kChunksPerBlock + wave_id(); c < n_chunks; c += wstride) {
    uint32_t run = offsets[c];
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i = c * kChunk + it * (kWave * kVec) + lane_id() * kVec;
      float v[4] = {0, 0, 0, 0};
      if (i < n) load4_f32(x, i, n, v, vec);
      bool hit[4];
      uint32_t mine = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        hit[e] = i + e < n && (abs_key(v[e]) >> 16) == bin;
        mine += hit[e];
      }
      const uint32_t incl = wave_incl_scan(mine);
      uint32_t pos = run + incl - mine;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (hit[e]) {
          if ((int64_t)pos < cap) cand[pos] = v[e];
          ++pos;
        }
      run += __shfl(incl, kWave - 1, kWave);
    }
  }
}

__global__ __launch_bounds__(kBlock) void k_gt_eq(
    const float* __restrict__ x, int64_t n, float thresh, uint8_t* __restrict__ gt,
    uint8_t* __restrict__ eq, int32_t* __restrict__ counts, bool vec) {
  uint32_t cg = 0, ce = 0;
  // Capped grid (few count atomics), four independent loads per lane and trip.
  constexpr int kUnroll = 4;
  constexpr int64_t kSlab = (int64_t)kBlock * kVec;
  const int64_t stride = (int64_t)gridDim.x * kSlab * kUnroll;
  for (int64_t b = (int64_t)blockIdx.x * kSlab * kUnroll + (int64_t)threadIdx.x * kVec; b < n;
       b += stride) {
    float v[kUnroll][4];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) load4_f32(x, b + u * kSlab, n, v[u], vec);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = b + u * kSlab;
      if (i >= n) break;
      uint32_t g4[4], e4[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool ok = i + e < n;
        g4[e] = ok && v[u][e] > thresh;
        e4[e] = ok && v[u][e] == thresh;
        cg += g4[e];
        ce += e4[e];
      }
      store4_u8(gt, i, n, g4, vec);
      store4_u8(eq, i, n, e4, vec);
    }
  }
  __shared__ uint32_t s_g[kChunksPerBlock], s_e[kChunksPerBlock];
  cg = wave_sum(cg);
  ce = wave_sum(ce);
  if (lane_id() == 0) { s_g[wave_id()] = cg; s_e[wave_id()] = ce; }
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t tg = s_g[0] + s_g[1] + s_g[2] + s_g[3];
    const uint32_t te = s_e[0] + s_e[1] + s_e[2] + s_e[3];
    if (tg) atomicAdd(&counts[0], (int32_t)tg);
    if (te) atomicAdd(&counts[1], (int32_t)te);
  }
}

// mask = |x| >= tau (float compare, NaN -> 0), count accumulated (u64 atomic
// per workgroup: order-free)
__global__ __launch_bounds__(kBlock) void k_mask_abs_ge(const float* __restrict__ x, int64_t n,
                                                        float tau, uint8_t* __restrict__ mask,
                                                        unsigned long long* __restrict__ count,
                                                        bool vec) {
  __shared__ uint32_t s_w[kChunksPerBlock];
  uint32_t c = 0;
  // Four independent 16-byte loads per lane and trip keep enough bytes in flight for a grid small
  // enough that its one count atomic per block does not queue up on the single counter.
  constexpr int kUnroll = 4;
  constexpr int64_t kSlab = (int64_t)kBlock * kVec;
  const int64_t stride = (int64_t)gridDim.x * kSlab * kUnroll;
  for (int64_t b = (int64_t)blockIdx.x * kSlab * kUnroll + (int64_t)threadIdx.x * kVec; b < n;
       b += stride) {
    float v[kUnroll][4];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) load4_f32(x, b + u * kSlab, n, v[u], vec);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = b + u * kSlab;
      if (i >= n) break;
      uint32_t mk[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        mk[e] = (i + e < n) && fabsf(v[u][e]) >= tau;
        c += mk[e];
      }
      store4_u8(mask, i, n, mk, vec);
    }
  }
  c = wave_sum(c);
  if (lane_id() == 0) s_w[wave_id()] = c;
  __syncthreads();
  if (threadIdx.x == 0 && count) {
    const uint32_t t = s_w[0] + s_w[1] + s_w[2] + s_w[3];
    if (t) atomicAdd(count, (unsigned long long)t);
  }
}

__global__ void k_zero_i32(int32_t* p, int n) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) p[i] = 0;
}

}  // namespace sga

using namespace sga;

extern "C" size_t sga_select_workspace_bytes(int64_t n) { return sel_ws_bytes(n < 0 ? 0 : n); }

static int carve(void* ws, size_t bytes, int64_t tiles, SelWorkspace* w, const char* who) {
  if (!sel_ws_carve(ws, bytes, tiles, w)) {
    set_error("%s: workspace missing, misaligned (16 B) or too small for %lld chunks "
              "(size it with sga_select_workspace_bytes)", who, (long long)tiles);
    return SGA_ERR_WORKSPACE;
  }
  return SGA_OK;
}

extern "C" int sga_sel_begin(int64_t k, void* ws, size_t ws_bytes, void* stream) {
  SelWorkspace w;
  if (int rc = carve(ws, ws_bytes, 0, &w, "sga_sel_begin")) return rc;
  if (k < 1 || k >= (1ll << 31)) {
    set_error("sga_sel_begin: k=%lld out of range", (long long)k);
    return SGA_ERR_ARG;
  }
  SelBatch B;
  B.add(w, 1, k, 0);
  hipLaunchKernelGGL(k_chain_begin, B.grid(1), dim3(kBlock), 0, (hipStream_t)stream, B.jobs, 0, 0.0);
  return check_launch("sga_sel_begin");
}

extern "C" int sga_sel_hist(const float* score, int64_t n, int level, void* ws,
                            size_t ws_bytes, void* stream) {
  if (n == 0) return SGA_OK;
  SelWorkspace w;
  if (int rc = carve(ws, ws_bytes, 0, &w, "sga_sel_hist")) return rc;
  if (!score || n < 0 || n >= (1ll << 31) || level < 0 || level > 2) {
    set_error("sga_sel_hist: bad argument");
    return SGA_ERR_ARG;
  }
  // histogram only: several views feed one level before its scan
  SrcPack<SrcF32> srcs = {};
  srcs.s[0] = SrcF32{score, aligned4(score, 4)};
  SelBatch B;
  B.add(w, n, 1, 0);
  launch_level_data<SrcF32, false>(srcs, B, level, (hipStream_t)stream);
  return check_launch("sga_sel_hist");
}

extern "C" int sga_sel_scan(int level, void* ws, size_t ws_bytes, void* stream) {
  SelWorkspace w;
  if (int rc = carve(ws, ws_bytes, 0, &w, "sga_sel_scan")) return rc;
  if (level < 0 || level > 2) { set_error("sga_sel_scan: bad level"); return SGA_ERR_ARG; }
  SelBatch B;
  B.add(w, 1, 1, 0);
  launch_level_scan(level, B, (hipStream_t)stream);
  return check_launch("sga_sel_scan");
}

extern "C" int sga_sel_count(const float* score, int64_t n, int64_t tile_base, void* ws,
                             size_t ws_bytes, void* stream) {
  if (n == 0) return SGA_OK;
  SelWorkspace w;
  if (int rc = carve(ws, ws_bytes, tile_base + cdiv64(n, kChunk), &w, "sga_sel_count")) return rc;
  if (!score || n < 0 || tile_base < 0) { set_error("sga_sel_count: bad argument"); return SGA_ERR_ARG; }
  SrcPack<SrcF32> srcs = {};
  srcs.s[0] = SrcF32{score, aligned4(score, 4)};
  SelBatch B;
  B.add(w, n, 1, 0);
  launch_tile_count(srcs, B, tile_base, (hipStream_t)stream);
  return check_launch("sga_sel_count");
}

extern "C" int sga_sel_tile_scan(int64_t n_tiles, int tie_mode, void* ws, size_t ws_bytes,
                                 void* stream) {
  SelWorkspace w;
  if (int rc = carve(ws, ws_bytes, n_tiles, &w, "sga_sel_tile_scan")) return rc;
  if (n_tiles < 1 || cdiv64(n_tiles, kTileScanSpan) > kMaxTileBlocks) {
    set_error("sga_sel_tile_scan: n_tiles=%lld out of range", (long long)n_tiles);
    return SGA_ERR_ARG;
  }
  SelBatch B;
  B.add(w, n_tiles * kChunk, 1, tie_mode == SGA_TIE_ALL);
  launch_tile_scan(B, (hipStream_t)stream);
  return check_launch("sga_sel_tile_scan");
}

extern "C" int sga_sel_mask(const float* score, int64_t n, int64_t tile_base, int tie_mode,
                            uint8_t* mask_out, void* ws, size_t ws_bytes, void* stream) {
  if (n == 0) return SGA_OK;
  SelWorkspace w;
  if (int rc = carve(ws, ws_bytes, tile_base + cdiv64(n, kChunk), &w, "sga_sel_mask")) return rc;
  if (!score || !mask_out || n < 0 || tile_base < 0) { set_error("sga_sel_mask: bad argument"); return SGA_ERR_ARG; }
  SrcPack<SrcF32> srcs = {};
  srcs.s[0] = SrcF32{score, aligned4(score, 4)};
  SelBatch B;
  B.add(w, n, 1, tie_mode == SGA_TIE_ALL).mask = mask_out;
  hipLaunchKernelGGL((k_write_mask<SrcF32>), B.grid(stream_grid(B.max_tiles, kChunksPerBlock, 1 << 22)),
                     dim3(kBlock), 0, (hipStream_t)stream, srcs, B.jobs, tile_base, 0,
                     (uint8_t*)nullptr);
  return check_launch("sga_sel_mask");
}

extern "C" int sga_sel_result(sga_select_result* result, void* ws, size_t ws_bytes, void* stream) {
  SelWorkspace w;
  if (int rc = carve(ws, ws_bytes, 0, &w, "sga_sel_result")) return rc;
  if (!result) { set_error("sga_sel_result: null result"); return SGA_ERR_ARG; }
  SelBatch B;
  B.add(w, 1, 1, 0).result = result;
  launch_result(B, (hipStream_t)stream);
  return check_launch("sga_sel_result");
}

extern "C" int sga_select_topk(const float* score, int64_t n, int64_t k, int tie_mode,
                               uint8_t* mask_out, sga_select_result* result, void* ws,
                               size_t ws_bytes, void* stream) {
  if (!score || !mask_out || n < 1 || n >= (1ll << 31) || k < 1 || k > n) {
    set_error("sga_select_topk: bad argument (n=%lld k=%lld; need 1 <= k <= n < 2^31)",
              (long long)n, (long long)k);
    return SGA_ERR_ARG;
  }
  SelWorkspace w;
  if (int rc = carve(ws, ws_bytes, cdiv64(n, kChunk), &w, "sga_select_topk")) return rc;
  hipStream_t s = (hipStream_t)stream;
  SrcPack<SrcF32> srcs = {};
  srcs.s[0] = SrcF32{score, aligned4(score, 4)};
  SelBatch B;
  ChainJob& J = B.add(w, n, k, tie_mode == SGA_TIE_ALL);
  J.mask = mask_out;
  J.result = result;
  const bool fast = SelBatch::fast_ok(w, n);
  // the select sweep writes the keys above the bracket straight into mask_out
  run_select_batch(srcs, B, fast, 2, s);
  finish_mask_batch(srcs, B, fast, s);
  launch_result(B, s);
  return check_launch("sga_select_topk");
}

extern "C" int sga_hist_topbits(const float* score, int64_t n, int shift, int stride, int phase,
                                int64_t* hist, int nbins, uint32_t* nonfinite, void* stream) {
  if (n == 0) return SGA_OK;
  if (!score || !hist || n < 0 || shift < 1 || shift > 30 || stride < 1 || phase < 0 ||
      phase >= stride || nbins < 1 || nbins > 32769 || nbins < (int)((0x7FFFFFFFu >> shift) + 1)) {
    set_error("sga_hist_topbits: bad argument (shift=%d stride=%d phase=%d nbins=%d)", shift,
              stride, phase, nbins);
    return SGA_ERR_ARG;
  }
  const int64_t n_s = n <= phase ? 0 : (n - phase + stride - 1) / stride;
  if (n_s == 0) return SGA_OK;
  if (stride == 1 && aligned4(score, 4)) {
    hipLaunchKernelGGL(k_hist_topbits_dense, dim3(stream_grid(n, (int64_t)kHistWide * kVec * 2, 256)),
                       dim3(kHistWide), (size_t)nbins * 4, (hipStream_t)stream, score, n, shift,
                       reinterpret_cast<unsigned long long*>(hist), nbins, nonfinite);
    return check_launch("sga_hist_topbits");
  }
  hipLaunchKernelGGL(k_hist_topbits, dim3(stream_grid(n_s, (int64_t)kBlock * 16, 256 * 2)),
                     dim3(kBlock), (size_t)nbins * 4, (hipStream_t)stream, score, n, shift, stride,
                     phase, reinterpret_cast<unsigned long long*>(hist), nbins, nonfinite);
  return check_launch("sga_hist_topbits");
}

extern "C" int sga_mask_topbits_ge(const float* score, int64_t n, int shift, int32_t bin,
                                   uint8_t* mask_out, void* stream) {
  if (n == 0) return SGA_OK;
  if (!score || !mask_out || n < 0 || shift < 1 || shift > 30 || bin < 0) {
    set_error("sga_mask_topbits_ge: bad argument");
    return SGA_ERR_ARG;
  }
  hipLaunchKernelGGL(k_mask_topbits_ge, dim3(stream_grid(n, (int64_t)kBlock * kVec, 1 << 22)), dim3(kBlock),
                     0, (hipStream_t)stream, score, n, shift, (uint32_t)bin, mask_out,
                     aligned4(score, 4) && aligned4(mask_out, 1));
  return check_launch("sga_mask_topbits_ge");
}

extern "C" int sga_mask_abs_ge(const float* score, int64_t n, float tau, uint8_t* mask_out,
                               int64_t* count, void* stream) {
  if (n == 0) return SGA_OK;
  if (!score || !mask_out || n < 0) { set_error("sga_mask_abs_ge: bad argument"); return SGA_ERR_ARG; }
  hipLaunchKernelGGL(k_mask_abs_ge, dim3(stream_grid(n, (int64_t)kBlock * kVec * 4, 256 * 16)),
                     dim3(kBlock), 0, (hipStream_t)stream, score, n, tau, mask_out,
                     reinterpret_cast<unsigned long long*>(count),
                     aligned4(score, 4) && aligned4(mask_out, 1));
  return check_launch("sga_mask_abs_ge");
}

extern "C" int sga_cand_extract_count(const float* score, int64_t n, int32_t bin,
                                      uint32_t* chunk_counts, int64_t* total, void* stream) {
  if (!total || n < 0 || n >= (1ll << 31) || bin < 0 || (n > 0 && (!score || !chunk_counts))) {
    set_error("sga_cand_extract_count: bad argument");
    return SGA_ERR_ARG;
  }
  const int64_t nc = cdiv64(n, kChunk);
  hipStream_t st = (hipStream_t)stream;
  if (nc > 0)
    hipLaunchKernelGGL(k_cand_count, dim3(stream_grid(nc, kChunksPerBlock, 1 << 22)), dim3(kBlock), 0, st,
                       score, n, (uint32_t)bin, chunk_counts, nc, aligned4(score, 4));
  if (int rc = exclusive_scan_u32(chunk_counts, nc, total, st)) return rc;
  return check_launch("sga_cand_extract_count");
}

extern "C" int sga_cand_extract_fill(const float* score, int64_t n, int32_t bin,
                                     const uint32_t* chunk_offsets, float* cand,
                                     int64_t cand_capacity, void* stream) {
  if (n == 0 || cand_capacity == 0) return SGA_OK;
  if (!score || !chunk_offsets || !cand || n < 0 || bin < 0) {
    set_error("sga_cand_extract_fill: bad argument");
    return SGA_ERR_ARG;
  }
  const int64_t nc = cdiv64(n, kChunk);
  hipLaunchKernelGGL(k_cand_fill, dim3(stream_grid(nc, kChunksPerBlock, 1 << 22)), dim3(kBlock), 0,
                     (hipStream_t)stream, score, n, (uint32_t)bin, chunk_offsets, cand,
                     cand_capacity, nc, aligned4(score, 4));
  return check_launch("sga_cand_extract_fill");
}

extern "C" int sga_gt_eq(const float* score, int64_t n, float thresh, uint8_t* gt, uint8_t* eq,
                         int32_t* counts2, void* stream) {
  if (!counts2 || n < 0 || (n > 0 && (!score || !gt || !eq))) {
    set_error("sga_gt_eq: bad argument");
    return SGA_ERR_ARG;
  }
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(k_zero_i32, dim3(1), dim3(64), 0, st, counts2, 2);
  if (n > 0)
    hipLaunchKernelGGL(k_gt_eq, dim3(stream_grid(n, (int64_t)kBlock * kVec * 4, 256 * 16)),
                       dim3(kBlock), 0, st, score, n, thresh, gt, eq, counts2,
                       aligned4(score, 4) && aligned4(gt, 1) && aligned4(eq, 1));
  return check_launch("sga_gt_eq");
}
