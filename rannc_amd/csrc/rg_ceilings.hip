// Yardstick kernels of libranncgrad: what the access patterns of the library's passes reach on
// this GPU when nothing else is in the way - flat arrays, no work table, no tensor boundaries,
// no reductions - written with the same load / store helpers and launch shapes as the passes
// themselves.  rg_ceiling_kernel runs one of them; bench.py reports them next to the passes
// so that "per cent of what the pattern allows" can be recomputed from one run.
#include "rg_device.h"
#include "rg_host.h"
#include "rg_internal.h"

namespace rg {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 as_f32x4(u32x4 v) { return __builtin_bit_cast(f32x4, v); }
__device__ __forceinline__ u32x4 as_u32x4(f32x4 v) { return __builtin_bit_cast(u32x4, v); }

// Streaming store as the passes that write one stream per launch issue it (buffer store, nt sc1).
__device__ __forceinline__ void st16_stream(char* p, u32x4 v) { st16_aux<2 | 16>(p, v); }

// Read only: the read-only pass's shape.  256 threads, eight 16-byte nontemporal loads in flight per
// lane (32 KiB per block), launched with the same unused dynamic LDS that caps the resident blocks.
__global__ __launch_bounds__(256) void ceiling_read_kernel(const char* src, int64_t nvec, float* sink) {
  const int64_t base = (int64_t)blockIdx.x * 2048 + threadIdx.x;
  u32x4 v[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    int64_t i = base + u * 256;
    if (i >= nvec) i = nvec - 1;
    v[u] = ld16_a4<true>(src + i * 16);
  }
  float acc = 0.0f;
#pragma unroll
  for (int u = 0; u < 8; ++u) acc += as_f32x4(v[u]).x + as_f32x4(v[u]).w;
  if (acc == 1.2345e-30f) *sink = acc;   // keeps the loads alive; never true for the bench's data
}

// The writing passes' shape: 128 threads, two steps per block, 16 bytes per lane and step on the
// wider side (one 4 KiB page of fp32 per block).
// kind 1: fill (write only, XCDs filling runs of 64 tiles)   2: fp32 copy   3: bf16 -> fp32 widening copy   4: four fp32 streams
// read, three of them written in place (Adam's pattern)   5: fp32 copy with plain `nt` stores
// 6: kind 4 plus the bf16 model copy as an eighth stream (the optimizer step under mixed precision)
// 8: kind 1 with every wavefront held for `delay_ticks` of the wall clock before its stores (rg_fill_zero's pacing)
template <int KIND>
__global__ __launch_bounds__(128) void ceiling_write_kernel(char* a0, char* a1, char* a2, char* a3, char* a4, int64_t nvec, int delay_ticks) {
  unsigned bid = blockIdx.x;
  if constexpr (KIND == 1) {
    // a write-only kernel is fastest when each XCD fills runs of consecutive tiles (rg_zero's order: runs of 64)
    const unsigned nb = gridDim.x, x = bid & 7u, q = bid >> 3, R = (unsigned)kZeroXcdRun, group = 8u * R;
    const unsigned g = bid / group;
    if ((g + 1) * group <= nb) bid = g * group + x * R + (q % R);
    if (delay_ticks > 0) {   // kind 8: the flat fill's pacing
      const uint64_t t_end = wall_clock64() + (uint64_t)delay_ticks;
      while (wall_clock64() < t_end) __builtin_amdgcn_s_sleep(1);
    }
  }
  const int64_t base = (int64_t)bid * 256 + threadIdx.x;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int64_t i = base + u * 128;
    if (i >= nvec) return;
    if constexpr (KIND == 1) {
      const u32x4 z = {0x3f800000u, 0x3f800000u, 0x3f800000u, 0x3f800000u};
      st16_stream(a0 + i * 16, z);
    } else if constexpr (KIND == 2) {
      const f32x4 x = as_f32x4(ld16_a4<true>(a0 + i * 16));
      st16_stream(a1 + i * 16, as_u32x4(x * 1.5f));
    } else if constexpr (KIND == 5) {
      const f32x4 x = as_f32x4(ld16_a4<true>(a0 + i * 16));
      st16<true>(a1 + i * 16, as_u32x4(x * 1.5f));
    } else if constexpr (KIND == 3) {
      const u32x2 h = ld8_a2<true>(a0 + i * 8);
      f32x4 x;
      x.x = __uint_as_float(h.x << 16);
      x.y = __uint_as_float(h.x & 0xffff0000u);
      x.z = __uint_as_float(h.y << 16);
      x.w = __uint_as_float(h.y & 0xffff0000u);
      st16_stream(a1 + i * 16, as_u32x4(x * 0.5f));
    } else {   // 4 and 6
      const f32x4 p = as_f32x4(ld16_a4<true>(a0 + i * 16));
      const f32x4 g = as_f32x4(ld16_a4<true>(a1 + i * 16));
      const f32x4 m = as_f32x4(ld16_a4<true>(a2 + i * 16));
      const f32x4 v = as_f32x4(ld16_a4<true>(a3 + i * 16));
      const f32x4 m2 = m + 0.1f * (g - m);
      const f32x4 v2 = v * 0.999f + 0.001f * g * g;
      const f32x4 p2 = p - 0.001f * m2;
      st16<true>(a0 + i * 16, as_u32x4(p2));
      st16<true>(a2 + i * 16, as_u32x4(m2));
      st16<true>(a3 + i * 16, as_u32x4(v2));
      if constexpr (KIND == 6) {
        const u32x2 h = {f32x2_to_bf16x2_bits(p2.x, p2.y), f32x2_to_bf16x2_bits(p2.z, p2.w)};
        st8<true>(a4 + i * 8, h);
      }
    }
  }
}

// Kind 7: the streams of kind 6 in the optimizer step's own launch shape - 256 threads over 4096 elements, the
// four vectors of every array in flight together - still over flat arrays.
__global__ __launch_bounds__(256) void ceiling_adam_shape_kernel(char* a0, char* a1, char* a2, char* a3, char* a4, int64_t nvec) {
  const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
  u32x4 p[4], g[4], m[4], v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    int64_t i = base + u * 256;
    if (i >= nvec) i = nvec - 1;
    p[u] = ld16_a4<true>(a0 + i * 16);
    g[u] = ld16_a4<true>(a1 + i * 16);
    m[u] = ld16_a4<true>(a2 + i * 16);
    v[u] = ld16_a4<true>(a3 + i * 16);
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int64_t i = base + u * 256;
    if (i >= nvec) return;
    const f32x4 m2 = as_f32x4(m[u]) + 0.1f * (as_f32x4(g[u]) - as_f32x4(m[u]));
    const f32x4 v2 = as_f32x4(v[u]) * 0.999f + 0.001f * as_f32x4(g[u]) * as_f32x4(g[u]);
    const f32x4 p2 = as_f32x4(p[u]) - 0.001f * m2;
    st16<true>(a0 + i * 16, as_u32x4(p2));
    st16<true>(a2 + i * 16, as_u32x4(m2));
    st16<true>(a3 + i * 16, as_u32x4(v2));
    const u32x2 h = {f32x2_to_bf16x2_bits(p2.x, p2.y), f32x2_to_bf16x2_bits(p2.z, p2.w)};
    st8<true>(a4 + i * 8, h);
  }
}

}  // namespace
}  // namespace rg

using namespace rg;

RG_API int rg_ceiling_kernel(int kind, void* const* arrays_dev, int n_arrays, int64_t nbytes, int device, void* stream) {
  static const int need[9] = {2, 1, 2, 2, 4, 2, 5, 5, 1};
  if (kind < 0 || kind > 8 || arrays_dev == nullptr || n_arrays < need[kind] || nbytes < 16 || nbytes % 16 != 0) {
    set_error("rg_ceiling_kernel: bad arguments (kind %d, %d arrays, %lld bytes)", kind, n_arrays, (long long)nbytes);
    return RG_EINVAL;
  }
  for (int i = 0; i < need[kind]; ++i) {
    if (arrays_dev[i] == nullptr || (reinterpret_cast<uintptr_t>(arrays_dev[i]) & 15u) != 0) {
      set_error("rg_ceiling_kernel: array %d is null or not 16-byte aligned", i);
      return RG_EINVAL;
    }
  }
  const int64_t nvec = nbytes / 16;   // 16-byte vectors of the widest stream
  char* a[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
  for (int i = 0; i < need[kind] && i < 5; ++i) a[i] = static_cast<char*>(arrays_dev[i]);
  DeviceGuard guard(device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (kind == 0) {
    const int64_t blocks = (nvec + 2047) / 2048;
    if (blocks > 0x7fffffffLL) {
      set_error("rg_ceiling_kernel: too large for one launch");
      return RG_EINVAL;
    }
    hipLaunchKernelGGL(ceiling_read_kernel, dim3((unsigned)blocks), dim3(256), kReducePassLdsBytes, s, a[0], nvec,
                       reinterpret_cast<float*>(a[1]));
    RG_HIP(hipGetLastError());
    return RG_OK;
  }
  if (kind == 7) {
    const int64_t blocks = (nvec + 1023) / 1024;
    if (blocks > 0x7fffffffLL) {
      set_error("rg_ceiling_kernel: too large for one launch");
      return RG_EINVAL;
    }
    hipLaunchKernelGGL(ceiling_adam_shape_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a[0], a[1], a[2], a[3], a[4], nvec);
    RG_HIP(hipGetLastError());
    return RG_OK;
  }
  const int64_t blocks = (nvec + 255) / 256;
  if (blocks > 0x7fffffffLL) {
    set_error("rg_ceiling_kernel: too large for one launch");
    return RG_EINVAL;
  }
  const dim3 grid((unsigned)blocks), block(128);
  switch (kind) {
    case 1: hipLaunchKernelGGL(ceiling_write_kernel<1>, grid, block, 0, s, a[0], a[1], a[2], a[3], a[4], nvec, 0); break;
    case 8: hipLaunchKernelGGL(ceiling_write_kernel<1>, grid, block, 0, s, a[0], a[1], a[2], a[3], a[4], nvec, fill_delay_ticks()); break;
    case 2: hipLaunchKernelGGL(ceiling_write_kernel<2>, grid, block, 0, s, a[0], a[1], a[2], a[3], a[4], nvec, 0); break;
    case 3: hipLaunchKernelGGL(ceiling_write_kernel<3>, grid, block, 0, s, a[0], a[1], a[2], a[3], a[4], nvec, 0); break;
    case 4: hipLaunchKernelGGL(ceiling_write_kernel<4>, grid, block, 0, s, a[0], a[1], a[2], a[3], a[4], nvec, 0); break;
    case 6: hipLaunchKernelGGL(ceiling_write_kernel<6>, grid, block, 0, s, a[0], a[1], a[2], a[3], a[4], nvec, 0); break;
    default: hipLaunchKernelGGL(ceiling_write_kernel<5>, grid, block, 0, s, a[0], a[1], a[2], a[3], a[4], nvec, 0); break;
  }
  RG_HIP(hipGetLastError());
  return RG_OK;
}
