// Two-kernel exclusive scan of uint32 counts (in place) for the
// compaction-style entry points.  data[] must be followed by
// scan_scratch_entries(n) spare uint32 slots (workgroup sums).
#include "common.hpp"

namespace sga {

constexpr int kScanPer = 16;
constexpr int kScanSpan = kBlock * kScanPer;  // 4096 entries per workgroup

int64_t scan_scratch_entries(int64_t n) { return cdiv64(n, kScanSpan) + 8; }

__global__ __launch_bounds__(kBlock) void k_scan_sums(
    const uint32_t* __restrict__ data, int64_t n, uint32_t* __restrict__ sums) {
  __shared__ uint32_t s_w[kChunksPerBlock];
  const int64_t base = (int64_t)blockIdx.x * kScanSpan + (int64_t)threadIdx.x * kScanPer;
  uint32_t acc = 0;
#pragma unroll
  for (int e = 0; e < kScanPer; ++e)
    if (base + e < n) acc += data[base + e];
  acc = wave_sum(acc);
  if (lane_id() == 0) s_w[wave_id()] = acc;
  __syncthreads();
  if (threadIdx.x == 0) sums[blockIdx.x] = s_w[0] + s_w[1] + s_w[2] + s_w[3];
}

__global__ __launch_bounds__(kBlock) void k_scan_apply(
    uint32_t* __restrict__ data, int64_t n, const uint32_t* __restrict__ sums,
    int64_t* __restrict__ total) {
  __shared__ unsigned long long s_w[kChunksPerBlock];
  __shared__ uint32_t s_x[kChunksPerBlock];
  // prefix of the workgroups before this one
  unsigned long long pre = 0;
  for (int64_t b = threadIdx.x; b < (int64_t)blockIdx.x; b += kBlock) pre += sums[b];
  pre = wave_sum(pre);
  if (lane_id() == 0) s_w[wave_id()] = pre;
  __syncthreads();
  const unsigned long long block_pre = s_w[0] + s_w[1] + s_w[2] + s_w[3];

  const int64_t base = (int64_t)blockIdx.x * kScanSpan + (int64_t)threadIdx.x * kScanPer;
  uint32_t v[kScanPer];
  uint32_t mine = 0;
#pragma unroll
  for (int e = 0; e < kScanPer; ++e) {
    v[e] = (base + e < n) ? data[base + e] : 0u;
    mine += v[e];
  }
  const uint32_t incl = wave_incl_scan(mine);
  if (lane_id() == kWave - 1) s_x[wave_id()] = incl;
  __syncthreads();
  uint32_t wpre = 0;
  for (int w = 0; w < wave_id(); ++w) wpre += s_x[w];
  uint32_t run = (uint32_t)block_pre + wpre + incl - mine;
#pragma unroll
  for (int e = 0; e < kScanPer; ++e) {
    if (base + e < n) data[base + e] = run;
    run += v[e];
  }
  if (total && blockIdx.x == gridDim.x - 1 && threadIdx.x == kBlock - 1)
    total[0] = (int64_t)(block_pre + s_x[0] + s_x[1] + s_x[2] + s_x[3]);
}

__global__ void k_zero_total(int64_t* total) { total[0] = 0; }

// data: n counts followed by scan_scratch_entries(n) scratch slots.
int exclusive_scan_u32(uint32_t* data, int64_t n, int64_t* total,
                       hipStream_t st) {
  if (n <= 0) {
    if (total) hipLaunchKernelGGL(k_zero_total, dim3(1), dim3(1), 0, st, total);
    return SGA_OK;
  }
  const unsigned nb = (unsigned)cdiv64(n, kScanSpan);
  uint32_t* sums = data + n;
  hipLaunchKernelGGL(k_scan_sums, dim3(nb), dim3(kBlock), 0, st, data, n, sums);
  hipLaunchKernelGGL(k_scan_apply, dim3(nb), dim3(kBlock), 0, st, data, n, sums, total);
  return SGA_OK;
}

}  // namespace sga
