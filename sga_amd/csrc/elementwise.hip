// Scheme-agnostic masked ops: pack / scatter / norms / block gather-scatter /
// mask compaction.  All are HBM-bound byte movers; nothing here is a
// contraction.
#include <mutex>

#include "common.hpp"

namespace sga {

// ---------------------------------------------------------------- scatter
__global__ __launch_bounds__(kBlock) void k_scatter(float* __restrict__ dst,
                                                    const int32_t* __restrict__ idx,
                                                    const float* __restrict__ src,
                                                    int64_t k, int64_t n_dst) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < k;
       i += (int64_t)gridDim.x * kBlock) {
    const int64_t j = idx[i];
    if (j >= 0 && j < n_dst) dst[j] = src[i];
  }
}

// ------------------------------------------------------------------- pack
template <bool BF16, bool SCALE>
__global__ __launch_bounds__(kBlock) void k_pack(float* __restrict__ grad,
                                                 const int32_t* __restrict__ idx,
                                                 void* __restrict__ values,
                                                 float factor, int64_t k,
                                                 int64_t n_grad) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < k;
       i += (int64_t)gridDim.x * kBlock) {
    const int64_t j = idx[i];
    if (j < 0 || j >= n_grad) continue;
    float x = grad[j];
    if (SCALE) x = x * factor;
    if (BF16)
      reinterpret_cast<uint16_t*>(values)[i] = f32_to_bf16(x);
    else
      reinterpret_cast<float*>(values)[i] = x;
    grad[j] = 0.0f;
  }
}

// ------------------------------------------------------------------ norms
// Stage 1: one fp32 partial per workgroup (fixed order: lane-strided sums,
// wave tree, then 4 waves) -- run-to-run deterministic for a given n.
template <bool MASKED>
__global__ __launch_bounds__(kBlock) void k_norm_stage1(
    const float* __restrict__ x, const uint8_t* __restrict__ mask, int64_t n,
    float* __restrict__ partials, bool vec) {
  __shared__ float s_w[kChunksPerBlock];
  float acc = 0.0f;
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  for (int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * kVec; i < n;
       i += stride) {
    float v[4];
    load4_f32(x, i, n, v, vec);
    if (MASKED) {
      uint32_t mk[4];
      load4_u8(mask, i, n, mk, vec);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = mk[e] ? v[e] : 0.0f;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) acc += v[e] * v[e];
  }
  acc = wave_sum(acc);
  if (lane_id() == 0) s_w[wave_id()] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.0f;
    for (int w = 0; w < kChunksPerBlock; ++w) t += s_w[w];
    partials[blockIdx.x] = t;
  }
}

// Stage 2: single workgroup folds the partials in index order.
__global__ __launch_bounds__(kBlock) void k_norm_stage2(
    const float* __restrict__ partials, int64_t np, float* __restrict__ total) {
  __shared__ float s_w[kChunksPerBlock];
  float acc = 0.0f;
  for (int64_t i = threadIdx.x; i < np; i += kBlock) acc += partials[i];
  acc = wave_sum(acc);
  if (lane_id() == 0) s_w[wave_id()] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.0f;
    for (int w = 0; w < kChunksPerBlock; ++w) t += s_w[w];
    total[0] += t;
  }
}

// --------------------------------------------------------- block gather
template <bool SCALE>
__global__ __launch_bounds__(kBlock) void k_gather_blocks(
    const float* __restrict__ grad, const uint8_t* __restrict__ mask,
    const int32_t* __restrict__ bidx, float* __restrict__ values, int64_t total,
    int xlog, float factor, int64_t n) {
  for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < total;
       t += (int64_t)gridDim.x * kBlock) {
    const int64_t j = t >> xlog;
    const int64_t pos = (int64_t)bidx[j] + (t & ((1 << xlog) - 1));
    float out = 0.0f;
    if (pos >= 0 && pos < n && mask[pos] != 0) {
      out = grad[pos];
      if (SCALE) out = out * factor;
    }
    values[t] = out;
  }
}

__global__ __launch_bounds__(kBlock) void k_scatter_blocks(
    float* __restrict__ dst, const uint8_t* __restrict__ mask,
    const int32_t* __restrict__ bidx, const float* __restrict__ src,
    int64_t total, int xlog, int64_t n) {
  for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < total;
       t += (int64_t)gridDim.x * kBlock) {
    const int64_t j = t >> xlog;
    const int64_t pos = (int64_t)bidx[j] + (t & ((1 << xlog) - 1));
    if (pos >= 0 && pos < n && mask[pos] != 0) dst[pos] = src[t];
  }
}

// ------------------------------------------------ block-granular helpers
// A group of L = min(x, 64) lanes cooperates on one x-element block of a
// view (the tail block of a view is short and reduces over its real length).
// MODE 0: mean of |g|, 1: max of |g|  -> float out[block]
template <int MODE>
__global__ __launch_bounds__(kBlock) void k_block_reduce(const float* __restrict__ g, int64_t n,
                                                         int x, int lanes, float* __restrict__ out,
                                                         int64_t n_blocks) {
  const int per_wave = kWave / lanes;
  const int sub = lane_id() / lanes, l = lane_id() % lanes;
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock * per_wave;
  for (int64_t b0 = ((int64_t)blockIdx.x * kChunksPerBlock + wave_id()) * per_wave; b0 < n_blocks;
       b0 += wstride) {
    const int64_t b = b0 + sub;
    float acc = 0.0f;
    int64_t len = 0;
    if (b < n_blocks) {
      const int64_t lo = b * x;
      len = n - lo < x ? n - lo : x;
      for (int64_t j = l; j < len; j += lanes) {
        const float a = fabsf(g[lo + j]);
        acc = MODE == 0 ? acc + a : fmaxf(acc, a);
      }
    }
    for (int o = lanes / 2; o > 0; o >>= 1) {
      const float t = __shfl_xor(acc, o, kWave);
      acc = MODE == 0 ? acc + t : fmaxf(acc, t);
    }
    if (b < n_blocks && l == 0) out[b] = MODE == 0 ? __fdiv_rn(acc, (float)len) : acc;
  }
}

// any_out[b] = 1 when block b of the span has a set byte
__global__ __launch_bounds__(kBlock) void k_block_any(const uint8_t* __restrict__ mask, int64_t n,
                                                      int x, int lanes, uint8_t* __restrict__ any_out,
                                                      int64_t n_blocks) {
  const int per_wave = kWave / lanes;
  const int sub = lane_id() / lanes, l = lane_id() % lanes;
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock * per_wave;
  for (int64_t b0 = ((int64_t)blockIdx.x * kChunksPerBlock + wave_id()) * per_wave; b0 < n_blocks;
       b0 += wstride) {
    const int64_t b = b0 + sub;
    uint32_t acc = 0;
    if (b < n_blocks) {
      const int64_t lo = b * x;
      const int64_t len = n - lo < x ? n - lo : x;
      for (int64_t j = l; j < len; j += lanes) acc |= mask[lo + j];
    }
    for (int o = lanes / 2; o > 0; o >>= 1) acc |= __shfl_xor(acc, o, kWave);
    if (b < n_blocks && l == 0) any_out[b] = acc ? 1 : 0;
  }
}

// out[i] = bmask[i / x]  (repeat_interleave(x)[:n])
__global__ __launch_bounds__(kBlock) void k_expand_blocks(const uint8_t* __restrict__ bmask, int xlog,
                                                          int64_t n, uint8_t* __restrict__ out) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * kBlock)
    out[i] = bmask[i >> xlog];
}

// ------------------------------------------------------- mask compaction
// Chunk = 1024 consecutive bytes owned by one wave (4 x 4 bytes per lane).
// Phase 1 counts the non-zero bytes of each chunk; a two-level exclusive scan
// turns counts into offsets; phase 2 rewrites positions in ascending order
// using wave ballots -- the output equals nonzero() for any launch geometry.
__global__ __launch_bounds__(kBlock) void k_mask_count(
    const uint8_t* __restrict__ mask, int64_t n, uint32_t* __restrict__ counts,
    int64_t n_chunks, bool vec) {
  const int64_t wave0 = (int64_t)blockIdx.x * kChunksPerBlock + wave_id();
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  for (int64_t c = wave0; c < n_chunks; c += wstride) {
    const int64_t base = c * kChunk;
    uint32_t cnt = 0;
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      uint32_t mk[4];
      load4_u8(mask, base + it * (kWave * kVec) + lane_id() * kVec, n, mk, vec);
#pragma unroll
      for (int e = 0; e < 4; ++e) cnt += (mk[e] != 0);
    }
    cnt = wave_sum(cnt);
    if (lane_id() == 0) counts[c] = cnt;
  }
}

__global__ __launch_bounds__(kBlock) void k_mask_fill(
    const uint8_t* __restrict__ mask, int64_t n,
    const uint32_t* __restrict__ offsets, int32_t* __restrict__ idx_out,
    int64_t cap, int64_t n_chunks, bool vec) {
  const int64_t wave0 = (int64_t)blockIdx.x * kChunksPerBlock + wave_id();
  const int64_t wstride = (int64_t)gridDim.x * kChunksPerBlock;
  for (int64_t c = wave0; c < n_chunks; c += wstride) {
    const int64_t base = c * kChunk;
    uint32_t run = offsets[c];
#pragma unroll
    for (int it = 0; it < kChunkIters; ++it) {
      const int64_t i0 = base + it * (kWave * kVec) + lane_id() * kVec;
      uint32_t mk[4];
      load4_u8(mask, i0, n, mk, vec);
      uint32_t mine = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) mine += (mk[e] != 0);
      const uint32_t incl = wave_incl_scan(mine);
      uint32_t pos = run + incl - mine;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (mk[e] != 0) {
          if ((int64_t)pos < cap) idx_out[pos] = (int32_t)(i0 + e);
          ++pos;
        }
      }
      run += __shfl(incl, kWave - 1, kWave);
    }
  }
}

}  // namespace sga

using namespace sga;

// Exclusive scan of uint32 counts in place (+ int64 total), shared by the
// compaction-style entry points.  Implemented in scan.hip.
namespace sga {
int exclusive_scan_u32(uint32_t* data, int64_t n, int64_t* total,
                       hipStream_t st);
int64_t scan_scratch_entries(int64_t n);
}

extern "C" int sga_scatter_selected(float* dst, const int32_t* idx,
                                    const float* src, int64_t k, int64_t n_dst,
                                    void* stream) {
  if (k == 0) return SGA_OK;
  if (!dst || !idx || !src || k < 0 || n_dst >= (1ll << 31)) {
    set_error("sga_scatter_selected: bad argument (k=%lld n_dst=%lld, needs < 2^31)",
              (long long)k, (long long)n_dst);
    return SGA_ERR_ARG;
  }
  hipLaunchKernelGGL(k_scatter, dim3(stream_grid(k, kBlock)), dim3(kBlock), 0,
                     (hipStream_t)stream, dst, idx, src, k, n_dst);
  return check_launch("sga_scatter_selected");
}

extern "C" int sga_pack_selected(float* grad, const int32_t* idx, void* values,
                                 int values_dtype, float factor, int64_t k,
                                 int64_t n_grad, void* stream) {
  if (k == 0) return SGA_OK;
  if (!grad || !idx || !values || k < 0 || n_grad >= (1ll << 31) ||
      (values_dtype != SGA_F32 && values_dtype != SGA_BF16)) {
    set_error("sga_pack_selected: bad argument (k=%lld n_grad=%lld dtype=%d, needs < 2^31)",
              (long long)k, (long long)n_grad, values_dtype);
    return SGA_ERR_ARG;
  }
  dim3 grid(stream_grid(k, kBlock)), block(kBlock);
  hipStream_t st = (hipStream_t)stream;
  const bool scale = factor != 1.0f;
  if (values_dtype == SGA_BF16) {
    if (scale) hipLaunchKernelGGL((k_pack<true, true>), grid, block, 0, st, grad, idx, values, factor, k, n_grad);
    else hipLaunchKernelGGL((k_pack<true, false>), grid, block, 0, st, grad, idx, values, factor, k, n_grad);
  } else {
    if (scale) hipLaunchKernelGGL((k_pack<false, true>), grid, block, 0, st, grad, idx, values, factor, k, n_grad);
    else hipLaunchKernelGGL((k_pack<false, false>), grid, block, 0, st, grad, idx, values, factor, k, n_grad);
  }
  return check_launch("sga_pack_selected");
}

static const int64_t kNormMaxBlocks = 2048;
// largest k of the allocation-free norm: the int32 index domain of a bucket (kernels.py:154)
static const int64_t kNoAllocNormMaxK = SGA_NOALLOC_NORM_MAX_K;

static int xlog_of(int x);

extern "C" int sga_block_reduce(const float* g, int64_t n, int x, int mode, float* out,
                                void* stream) {
  if (n == 0) return SGA_OK;
  if (!g || !out || n < 0 || xlog_of(x) < 0 || (mode != 0 && mode != 1)) {
    set_error("sga_block_reduce: bad argument (x=%d mode=%d)", x, mode);
    return SGA_ERR_ARG;
  }
  const int64_t nb = cdiv64(n, x);
  const int lanes = x < kWave ? x : kWave;
  dim3 grid(stream_grid(nb, kChunksPerBlock * (kWave / lanes))), block(kBlock);
  if (mode == 0) hipLaunchKernelGGL((k_block_reduce<0>), grid, block, 0, (hipStream_t)stream, g, n, x, lanes, out, nb);
  else hipLaunchKernelGGL((k_block_reduce<1>), grid, block, 0, (hipStream_t)stream, g, n, x, lanes, out, nb);
  return check_launch("sga_block_reduce");
}

extern "C" int sga_block_any(const uint8_t* mask, int64_t n, int x, uint8_t* any_out, void* stream) {
  if (n == 0) return SGA_OK;
  if (!mask || !any_out || n < 0 || xlog_of(x) < 0) {
    set_error("sga_block_any: bad argument (x=%d)", x);
    return SGA_ERR_ARG;
  }
  const int64_t nb = cdiv64(n, x);
  const int lanes = x < kWave ? x : kWave;
  hipLaunchKernelGGL(k_block_any, dim3(stream_grid(nb, kChunksPerBlock * (kWave / lanes))),
                     dim3(kBlock), 0, (hipStream_t)stream, mask, n, x, lanes, any_out, nb);
  return check_launch("sga_block_any");
}

extern "C" int sga_expand_blocks(const uint8_t* bmask, int x, int64_t n, uint8_t* out, void* stream) {
  if (n == 0) return SGA_OK;
  const int xl = xlog_of(x);
  if (!bmask || !out || n < 0 || xl < 0) {
    set_error("sga_expand_blocks: bad argument (x=%d)", x);
    return SGA_ERR_ARG;
  }
  hipLaunchKernelGGL(k_expand_blocks, dim3(stream_grid(n, kBlock)), dim3(kBlock), 0,
                     (hipStream_t)stream, bmask, xl, n, out);
  return check_launch("sga_expand_blocks");
}

extern "C" int64_t sga_norm_partials(int64_t n) {
  return stream_grid(n, (int64_t)kBlock * kVec, kNormMaxBlocks);
}

extern "C" int sga_compact_norm_sq(const float* values, int64_t k,
                                   float* partials, float* total, void* stream) {
  if (k == 0) return SGA_OK;
  if (!values || !partials || !total || k < 0) {
    set_error("sga_compact_norm_sq: bad argument");
    return SGA_ERR_ARG;
  }
  const unsigned nb = (unsigned)sga_norm_partials(k);
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL((k_norm_stage1<false>), dim3(nb), dim3(kBlock), 0, st,
                     values, (const uint8_t*)nullptr, k, partials,
                     aligned4(values, 4));
  hipLaunchKernelGGL(k_norm_stage2, dim3(1), dim3(kBlock), 0, st, partials,
                     (int64_t)nb, total);
  return check_launch("sga_compact_norm_sq");
}

// The stage-1 partials of the allocation-free norm: one array per device,
// held by every GPU the library runs on until the process ends (8 KiB).  In
// host code the array's name is only a stand-in for the symbol; the device
// address is resolved once per device and kept in g_norm_scratch_ptr.
static __device__ __align__(256) float scratch[kNormMaxBlocks];

static const int kNoAllocMaxDevices = 64;
static std::mutex g_norm_scratch_mu;
static float* g_norm_scratch_ptr[kNoAllocMaxDevices] = {};

// Device address of `scratch` on the current device, or null with the error
// text set.  The first call on a device resolves the symbol (no allocation).
static float* norm_scratch_of_current_device(const char* who) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kNoAllocMaxDevices) {
    set_error("%s: cannot name the current device (%s, device %d, at most %d supported)", who,
              hipGetErrorString(e), dev, kNoAllocMaxDevices);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_norm_scratch_mu);
  if (!g_norm_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev,
                hipGetErrorString(e));
      return nullptr;
    }
    g_norm_scratch_ptr[dev] = static_cast<float*>(ptr);
  }
  return g_norm_scratch_ptr[dev];
}

extern "C" int sga_compact_norm_sq_noalloc(const float* values, int64_t k, float* total,
                                           void* stream) {
  if (k == 0) return SGA_OK;
  if (!values || !total || k < 0) {
    set_error("sga_compact_norm_sq_noalloc: bad argument");
    return SGA_ERR_ARG;
  }
  if (k > kNoAllocNormMaxK) {
    set_error("sga_compact_norm_sq_noalloc: k=%lld exceeds the supported maximum %lld "
              "(use sga_compact_norm_sq with a caller workspace)",
              (long long)k, (long long)kNoAllocNormMaxK);
    return SGA_ERR_ARG;
  }
  float* partials = norm_scratch_of_current_device("sga_compact_norm_sq_noalloc");
  if (!partials) return SGA_ERR_LAUNCH;
  // same two kernels, same grid as sga_compact_norm_sq: the result has the same bits.  Stage 1
  // overwrites the nb slots stage 2 reads, so nothing in the array has to start at zero.
  const unsigned nb = (unsigned)sga_norm_partials(k);
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL((k_norm_stage1<false>), dim3(nb), dim3(kBlock), 0, st, values,
                     (const uint8_t*)nullptr, k, partials, aligned4(values, 4));
  hipLaunchKernelGGL(k_norm_stage2, dim3(1), dim3(kBlock), 0, st, partials, (int64_t)nb, total);
  return check_launch("sga_compact_norm_sq_noalloc");
}

extern "C" int sga_masked_norm_sq(const float* grad, const uint8_t* mask,
                                  int64_t n, float* partials, float* total,
                                  void* stream) {
  if (n == 0) return SGA_OK;
  if (!grad || !mask || !partials || !total || n < 0) {
    set_error("sga_masked_norm_sq: bad argument");
    return SGA_ERR_ARG;
  }
  const unsigned nb = (unsigned)sga_norm_partials(n);
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL((k_norm_stage1<true>), dim3(nb), dim3(kBlock), 0, st, grad,
                     mask, n, partials, aligned4(grad, 4) && aligned4(mask, 1));
  hipLaunchKernelGGL(k_norm_stage2, dim3(1), dim3(kBlock), 0, st, partials,
                     (int64_t)nb, total);
  return check_launch("sga_masked_norm_sq");
}

// g[i] *= coeff where mask[i] (every i when mask is null): the explicit clip
// scale, one fp32 multiply per touched coordinate.
template <bool MASKED>
__global__ __launch_bounds__(kBlock) void k_scale_masked(float* __restrict__ g,
                                                         const uint8_t* __restrict__ mask,
                                                         int64_t n, float coeff, bool vec) {
  const int64_t stride = (int64_t)gridDim.x * kBlock * kVec;
  for (int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * kVec; i < n; i += stride) {
    uint32_t mk[4] = {1u, 1u, 1u, 1u};
    if (MASKED) {
      load4_u8(mask, i, n, mk, vec);
      if (!(mk[0] | mk[1] | mk[2] | mk[3])) continue;   // untouched lanes move no gradient bytes
    }
    float v[4];
    load4_f32(g, i, n, v, vec);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = mk[e] ? v[e] * coeff : v[e];
    store4_f32(g, i, n, v, vec);
  }
}

extern "C" int sga_scale_masked(float* grad, const uint8_t* mask, int64_t n, float coeff,
                                void* stream) {
  if (n == 0) return SGA_OK;
  if (!grad || n < 0) { set_error("sga_scale_masked: bad argument"); return SGA_ERR_ARG; }
  dim3 grid(stream_grid(n, (int64_t)kBlock * kVec, 1 << 22)), block(kBlock);
  const bool vec = aligned4(grad, 4) && aligned4(mask, 1);
  if (mask)
    hipLaunchKernelGGL((k_scale_masked<true>), grid, block, 0, (hipStream_t)stream, grad, mask, n, coeff, vec);
  else
    hipLaunchKernelGGL((k_scale_masked<false>), grid, block, 0, (hipStream_t)stream, grad, mask, n, coeff, vec);
  return check_launch("sga_scale_masked");
}

static int xlog_of(int x) {
  if (x < 1 || x > 1024 || (x & (x - 1))) return -1;
  int l = 0;
  while ((1 << l) < x) ++l;
  return l;
}

extern "C" int sga_gather_selected_blocks(const float* grad, const uint8_t* mask,
                                          const int32_t* block_idx,
                                          float* values, int64_t kb, int x,
                                          float factor, int64_t n_grad,
                                          void* stream) {
  if (kb == 0) return SGA_OK;
  const int xl = xlog_of(x);
  if (!grad || !mask || !block_idx || !values || kb < 0 || xl < 0 ||
      n_grad >= (1ll << 31)) {
    set_error("sga_gather_selected_blocks: bad argument (x=%d must be a power of two in [1,1024]; n < 2^31)", x);
    return SGA_ERR_ARG;
  }
  const int64_t total = kb * x;
  dim3 grid(stream_grid(total, kBlock)), block(kBlock);
  if (factor != 1.0f)
    hipLaunchKernelGGL((k_gather_blocks<true>), grid, block, 0, (hipStream_t)stream, grad, mask, block_idx, values, total, xl, factor, n_grad);
  else
    hipLaunchKernelGGL((k_gather_blocks<false>), grid, block, 0, (hipStream_t)stream, grad, mask, block_idx, values, total, xl, factor, n_grad);
  return check_launch("sga_gather_selected_blocks");
}

extern "C" int sga_scatter_selected_blocks(float* dst, const uint8_t* mask,
                                           const int32_t* block_idx,
                                           const float* src, int64_t kb, int x,
                                           int64_t n_dst, void* stream) {
  if (kb == 0) return SGA_OK;
  const int xl = xlog_of(x);
  if (!dst || !mask || !block_idx || !src || kb < 0 || xl < 0 ||
      n_dst >= (1ll << 31)) {
    set_error("sga_scatter_selected_blocks: bad argument (x=%d)", x);
    return SGA_ERR_ARG;
  }
  const int64_t total = kb * x;
  hipLaunchKernelGGL(k_scatter_blocks, dim3(stream_grid(total, kBlock)),
                     dim3(kBlock), 0, (hipStream_t)stream, dst, mask, block_idx,
                     src, total, xl, n_dst);
  return check_launch("sga_scatter_selected_blocks");
}

// Entries the caller must provide for chunk_counts: one per 1024-byte chunk
// plus the scan's workgroup-sum scratch.
extern "C" int64_t sga_mask_chunks(int64_t n) {
  const int64_t nc = cdiv64(n, kChunk);
  return nc + scan_scratch_entries(nc);
}
static inline int64_t n_chunks_of(int64_t n) { return cdiv64(n, kChunk); }

extern "C" int sga_mask_count(const uint8_t* mask, int64_t n,
                              uint32_t* chunk_counts, int64_t* total,
                              void* stream) {
  if (!total || n < 0 || n >= (1ll << 31) || (n > 0 && (!mask || !chunk_counts))) {
    set_error("sga_mask_count: bad argument (n=%lld, int32 indices need n < 2^31)", (long long)n);
    return SGA_ERR_ARG;
  }
  hipStream_t st = (hipStream_t)stream;
  const int64_t nc = n_chunks_of(n);
  if (nc > 0)
    hipLaunchKernelGGL(k_mask_count, dim3(stream_grid(nc, kChunksPerBlock, 1 << 22)),
                       dim3(kBlock), 0, st, mask, n, chunk_counts, nc,
                       aligned4(mask, 1));
  int rc = exclusive_scan_u32(chunk_counts, nc, total, st);
  if (rc) return rc;
  return check_launch("sga_mask_count");
}

extern "C" int sga_mask_fill(const uint8_t* mask, int64_t n,
                             const uint32_t* chunk_offsets, int32_t* idx_out,
                             int64_t idx_capacity, void* stream) {
  if (n == 0) return SGA_OK;
  if (!mask || !chunk_offsets || (!idx_out && idx_capacity > 0) || n < 0 ||
      n >= (1ll << 31)) {
    set_error("sga_mask_fill: bad argument");
    return SGA_ERR_ARG;
  }
  const int64_t nc = n_chunks_of(n);
  hipLaunchKernelGGL(k_mask_fill, dim3(stream_grid(nc, kChunksPerBlock, 1 << 22)),
                     dim3(kBlock), 0, (hipStream_t)stream, mask, n,
                     chunk_offsets, idx_out, idx_capacity, nc,
                     aligned4(mask, 1));
  return check_launch("sga_mask_fill");
}
