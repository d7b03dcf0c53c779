// libsga_hip_bench.so: benchmark-only companion of libsga_hip.so (declared in
// include/sga_hip_bench.h, not part of the drop-in boundary).  It defines the
// two timing-observer symbols that libsga_hip.so references weakly -- so it
// has to be loaded, into the global symbol scope, BEFORE libsga_hip.so -- and
// two calibration kernels of known HBM traffic.  It links against nothing of
// the product library.
#include <atomic>
#include <mutex>
#include <stdarg.h>
#include <stdio.h>

#define SGA_BENCH_LIBRARY 1
#include "common.hpp"
#include "../../include/sga_hip_bench.h"

namespace {

struct Pair { hipEvent_t a, b; int tag; int closed; };
constexpr int kProfSlots = 4096;
std::atomic<int> g_prof_on{0};
std::mutex g_prof_mu;
Pair g_prof[kProfSlots];
int g_prof_made = 0, g_prof_used = 0;
thread_local char g_err[256] = "";

void bench_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int bench_check(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return SGA_OK;
  bench_error("%s: %s", what, hipGetErrorString(e));
  return SGA_ERR_LAUNCH;
}

}  // namespace

extern "C" const char* sga_bench_last_error(void) { return g_err; }

extern "C" void* sga_bench_prof_begin(int tag, void* stream) {
  if (!g_prof_on.load(std::memory_order_relaxed)) return nullptr;
  Pair* pp = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_prof_mu);
    if (!g_prof_on.load(std::memory_order_relaxed) || g_prof_used >= kProfSlots) return nullptr;
    if (g_prof_used >= g_prof_made) {
      if (hipEventCreate(&g_prof[g_prof_made].a) != hipSuccess) return nullptr;
      if (hipEventCreate(&g_prof[g_prof_made].b) != hipSuccess) {
        (void)hipEventDestroy(g_prof[g_prof_made].a);
        return nullptr;
      }
      ++g_prof_made;
    }
    pp = &g_prof[g_prof_used++];
    pp->tag = tag;
    pp->closed = 0;
  }
  (void)hipEventRecord(pp->a, (hipStream_t)stream);
  return pp;
}

extern "C" void sga_bench_prof_end(void* pair, void* stream) {
  Pair* pp = reinterpret_cast<Pair*>(pair);
  if (!pp) return;
  (void)hipEventRecord(pp->b, (hipStream_t)stream);
  std::lock_guard<std::mutex> lock(g_prof_mu);
  pp->closed = 1;
}

namespace sga {

// Plain 128-bit copy of known size: the yardstick the HBM traffic counters
// and the achievable streaming bandwidth are calibrated against.
__global__ __launch_bounds__(kBlock) void k_calib_copy(float* __restrict__ dst,
                                                       const float* __restrict__ src,
                                                       int64_t n4) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n4;
       i += (int64_t)gridDim.x * kBlock)
    reinterpret_cast<F4*>(dst)[i] = reinterpret_cast<const F4*>(src)[i];
}

// Math-free stand-in with the final sweep's stream structure (reads bf16 g
// and fp32 r, p, m, v; writes r, p, m, v; 34 B per element): what this mix of
// five read and four write streams can reach, as opposed to a plain copy.
__global__ __launch_bounds__(kBlock) void k_calib_streams(const uint16_t* __restrict__ g,
                                                          float* __restrict__ r,
                                                          float* __restrict__ p,
                                                          float* __restrict__ m,
                                                          float* __restrict__ v, int64_t n) {
  const int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * kVec;
  if (i + kVec > n) return;
  const H4 gh = ldh4_nt(g + i);
  F4 rr = ld4_nt(r + i), pp = ld4_nt(p + i), mm = ld4_nt(m + i), vv = ld4_nt(v + i);
  const float gf[4] = {bf16_to_f32(gh.x), bf16_to_f32(gh.y), bf16_to_f32(gh.z), bf16_to_f32(gh.w)};
  float* rp = &rr.x; float* ppp = &pp.x; float* mp = &mm.x; float* vp = &vv.x;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    rp[e] += gf[e];
    mp[e] = mp[e] * 0.5f + rp[e];
    vp[e] = vp[e] * 0.5f + rp[e] * rp[e];
    ppp[e] -= mp[e] * 0.5f;
  }
  st4_nt(r + i, rr);
  st4_nt(p + i, pp);
  st4_nt(m + i, mm);
  st4_nt(v + i, vv);
}

}  // namespace sga

using namespace sga;

extern "C" int sga_prof_enable(int on) {
  std::lock_guard<std::mutex> lock(g_prof_mu);
  // pairs still in flight from an earlier window are waited for before their slots are reused
  for (int i = 0; i < g_prof_used; ++i)
    if (g_prof[i].closed) (void)hipEventSynchronize(g_prof[i].b);
  g_prof_used = 0;
  g_prof_on.store(on != 0 ? 1 : 0, std::memory_order_relaxed);
  return SGA_OK;
}

extern "C" int sga_prof_read(int tag, double* total_ms, int* launches) {
  if (!total_ms || !launches) { bench_error("sga_prof_read: null output"); return SGA_ERR_ARG; }
  std::lock_guard<std::mutex> lock(g_prof_mu);
  double tot = 0.0;
  int cnt = 0;
  for (int i = 0; i < g_prof_used; ++i) {
    if (g_prof[i].tag != tag || !g_prof[i].closed) continue;
    float ms = 0.0f;
    if (hipEventSynchronize(g_prof[i].b) != hipSuccess ||
        hipEventElapsedTime(&ms, g_prof[i].a, g_prof[i].b) != hipSuccess) {
      bench_error("sga_prof_read: event %d not ready", i);
      return SGA_ERR_LAUNCH;
    }
    tot += ms;
    ++cnt;
  }
  *total_ms = tot;
  *launches = cnt;
  return SGA_OK;
}

extern "C" int sga_calib_copy(float* dst, const float* src, int64_t n, void* stream) {
  if (!dst || !src || n < 0 || (n & 3) || !aligned4(dst, 4) || !aligned4(src, 4)) {
    bench_error("sga_calib_copy: needs 16-byte aligned buffers and n %% 4 == 0");
    return SGA_ERR_ARG;
  }
  if (n == 0) return SGA_OK;
  hipLaunchKernelGGL(k_calib_copy, dim3(stream_grid(n / 4, kBlock, 1 << 20)), dim3(kBlock), 0,
                     (hipStream_t)stream, dst, src, n / 4);
  return bench_check("sga_calib_copy");
}

extern "C" int sga_calib_streams(const void* g_bf16, float* r, float* p, float* m, float* v,
                                 int64_t n, void* stream) {
  if (!g_bf16 || !r || !p || !m || !v || n < 0 || (n & 3) || !aligned4(g_bf16, 2) ||
      !aligned4(r, 4) || !aligned4(p, 4) || !aligned4(m, 4) || !aligned4(v, 4)) {
    bench_error("sga_calib_streams: needs aligned buffers and n a multiple of 4");
    return SGA_ERR_ARG;
  }
  if (n == 0) return SGA_OK;
  hipLaunchKernelGGL(k_calib_streams, dim3((unsigned)cdiv64(n, (int64_t)kBlock * kVec)),
                     dim3(kBlock), 0, (hipStream_t)stream,
                     reinterpret_cast<const uint16_t*>(g_bf16), r, p, m, v, n);
  return bench_check("sga_calib_streams");
}
