// gfx950 kernels of libranncgrad.
//
// One "pass" kernel serves every per-step operation.  The grid is the plan's chunk list:
// block b looks up (tensor, chunk-of-tensor) in the device-side table, so a launch covers
// thousands of tensors of any size mix.  A chunk is a contiguous run of at most
// chunk_elems elements of one tensor; inside it a thread moves 8 elements per step with
// 128-bit accesses.  The side that is written (or, for a read-only pass, the side that is
// read) is peeled to a 16-byte boundary per chunk; the other side is accessed at its
// natural element alignment, which gfx950 serves with the same 128-bit instruction.
//
// The pass is purely bandwidth bound (a few ALU ops per element), so there is no LDS
// staging and no MFMA: LDS is used only for the 4-wavefront combine of the partial sums.
#include "rg_internal.h"

namespace rg {
namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// 16-byte vectors at element alignment (2 or 4 bytes).
struct __attribute__((packed, aligned(2))) V16A2 { u32x4 v; };
struct __attribute__((packed, aligned(4))) V16A4 { u32x4 v; };

template <int DT> struct ElemSize { static constexpr int value = 2; };
template <> struct ElemSize<RG_F32> { static constexpr int value = 4; };

// Eight elements in their memory representation.
template <int DT> struct Raw { u32x4 a; };
template <> struct Raw<RG_F32> { u32x4 a, b; };

template <int DT> __device__ __forceinline__ Raw<DT> load_raw(const char* p) {
  Raw<DT> r;
  r.a = reinterpret_cast<const V16A2*>(p)->v;
  return r;
}
template <> __device__ __forceinline__ Raw<RG_F32> load_raw<RG_F32>(const char* p) {
  Raw<RG_F32> r;
  r.a = reinterpret_cast<const V16A4*>(p)->v;
  r.b = reinterpret_cast<const V16A4*>(p + 16)->v;
  return r;
}

// Stores are always 16-byte aligned (the chunk head is peeled for that).
template <int DT> __device__ __forceinline__ void store_raw(char* p, const Raw<DT>& r) {
  *reinterpret_cast<u32x4*>(p) = r.a;
}
template <> __device__ __forceinline__ void store_raw<RG_F32>(char* p, const Raw<RG_F32>& r) {
  *reinterpret_cast<u32x4*>(p) = r.a;
  *reinterpret_cast<u32x4*>(p + 16) = r.b;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// Round-to-nearest-even narrowing; NaN becomes the canonical quiet NaN.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  return ((u & 0x7fffffffu) > 0x7f800000u) ? 0x7fc0u : r;
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(unsigned short, (_Float16)f);
}

template <int DT> __device__ __forceinline__ void unpack(const Raw<DT>& r, float (&f)[8]);
template <> __device__ __forceinline__ void unpack<RG_F32>(const Raw<RG_F32>& r, float (&f)[8]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[j] = __uint_as_float(r.a[j]);
    f[4 + j] = __uint_as_float(r.b[j]);
  }
}
template <> __device__ __forceinline__ void unpack<RG_F16>(const Raw<RG_F16>& r, float (&f)[8]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const unsigned int w = r.a[j];  // bit_cast must see a scalar, not a vector-element lvalue
    const f16x2 h = __builtin_bit_cast(f16x2, w);
    f[2 * j] = (float)h.x;
    f[2 * j + 1] = (float)h.y;
  }
}
template <> __device__ __forceinline__ void unpack<RG_BF16>(const Raw<RG_BF16>& r, float (&f)[8]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = __uint_as_float(r.a[j] << 16);
    f[2 * j + 1] = __uint_as_float(r.a[j] & 0xffff0000u);
  }
}

template <int DT> __device__ __forceinline__ Raw<DT> pack(const float (&f)[8]);
template <> __device__ __forceinline__ Raw<RG_F32> pack<RG_F32>(const float (&f)[8]) {
  Raw<RG_F32> r;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    r.a[j] = __float_as_uint(f[j]);
    r.b[j] = __float_as_uint(f[4 + j]);
  }
  return r;
}
template <> __device__ __forceinline__ Raw<RG_F16> pack<RG_F16>(const float (&f)[8]) {
  Raw<RG_F16> r;
#pragma unroll
  for (int j = 0; j < 4; ++j) r.a[j] = f32_to_f16_bits(f[2 * j]) | (f32_to_f16_bits(f[2 * j + 1]) << 16);
  return r;
}
template <> __device__ __forceinline__ Raw<RG_BF16> pack<RG_BF16>(const float (&f)[8]) {
  Raw<RG_BF16> r;
#pragma unroll
  for (int j = 0; j < 4; ++j) r.a[j] = f32_to_bf16_bits(f[2 * j]) | (f32_to_bf16_bits(f[2 * j + 1]) << 16);
  return r;
}

// The value as it reads back from a destination of type DT.
template <int DT> __device__ __forceinline__ float round_dst(float v) { return v; }
template <> __device__ __forceinline__ float round_dst<RG_F16>(float v) { return (float)(_Float16)v; }
template <> __device__ __forceinline__ float round_dst<RG_BF16>(float v) {
  return bf16_bits_to_f32(f32_to_bf16_bits(v));
}

template <int DT> __device__ __forceinline__ float load1(const char* p) {
  return *reinterpret_cast<const float*>(p);
}
template <> __device__ __forceinline__ float load1<RG_F16>(const char* p) {
  return (float)*reinterpret_cast<const _Float16*>(p);
}
template <> __device__ __forceinline__ float load1<RG_BF16>(const char* p) {
  return bf16_bits_to_f32(*reinterpret_cast<const unsigned short*>(p));
}
template <int DT> __device__ __forceinline__ void store1(char* p, float v) {
  *reinterpret_cast<float*>(p) = v;
}
template <> __device__ __forceinline__ void store1<RG_F16>(char* p, float v) {
  *reinterpret_cast<_Float16*>(p) = (_Float16)v;
}
template <> __device__ __forceinline__ void store1<RG_BF16>(char* p, float v) {
  *reinterpret_cast<unsigned short*>(p) = (unsigned short)f32_to_bf16_bits(v);
}

template <int DT> __device__ __forceinline__ bool nonfinite_at(const char* p) {
  return (*reinterpret_cast<const uint32_t*>(p) & 0x7f800000u) == 0x7f800000u;
}
template <> __device__ __forceinline__ bool nonfinite_at<RG_F16>(const char* p) {
  return (*reinterpret_cast<const unsigned short*>(p) & 0x7c00u) == 0x7c00u;
}
template <> __device__ __forceinline__ bool nonfinite_at<RG_BF16>(const char* p) {
  return (*reinterpret_cast<const unsigned short*>(p) & 0x7f80u) == 0x7f80u;
}

// v = round_dst(x * scale); sum += v^2; out = round_dst(v * coef).
// coef is 1 when nothing is clipped: v * 1 is v bit for bit, so no branch is needed.
// Two separate multiplies, never fused or reassociated (the file is built with
// -ffp-contract=off), so the result matches `x.float() * inv_scale` then `mul_(coef)`.
template <int S, int D, int MODE>
__device__ __forceinline__ void compute8(const Raw<S>& in, Raw<D>& out, float (&acc)[8], float scale,
                                         float coef) {
  float f[8];
  unpack<S>(in, f);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float v = round_dst<D>(f[j] * scale);
    if (MODE & kModeReduce) acc[j] = __builtin_fmaf(v, v, acc[j]);
    if (MODE & kModeWrite) f[j] = round_dst<D>(v * coef);
  }
  if (MODE & kModeWrite) out = pack<D>(f);
}

template <int S, int D, int MODE>
__device__ __forceinline__ void process_chunk(const char* sp, char* dp, int64_t len, float scale,
                                              float coef, bool raw_copy, float (&acc)[8]) {
  constexpr int SS = ElemSize<S>::value;
  constexpr int DS = ElemSize<D>::value;
  constexpr bool kWrite = (MODE & kModeWrite) != 0;
  constexpr int AS = kWrite ? DS : SS;
  const uintptr_t a = kWrite ? reinterpret_cast<uintptr_t>(dp) : reinterpret_cast<uintptr_t>(sp);
  int64_t head = (int64_t)(((16u - (unsigned)(a & 15u)) & 15u) / (unsigned)AS);
  if (head > len) head = len;
  const int64_t nvec = (len - head) / kVecElems;
  const int64_t tail0 = head + nvec * kVecElems;
  const int tid = threadIdx.x;

  // Unaligned head (< 8 elements) and ragged tail (< 8 elements): one element per thread.
  const int nscalar = (int)(head + (len - tail0));
  if (tid < nscalar) {
    const int64_t i = tid < head ? (int64_t)tid : tail0 + (tid - head);
    if (S == D && raw_copy) {
      if (SS == 4) *reinterpret_cast<uint32_t*>(dp + i * 4) = *reinterpret_cast<const uint32_t*>(sp + i * 4);
      else *reinterpret_cast<unsigned short*>(dp + i * 2) = *reinterpret_cast<const unsigned short*>(sp + i * 2);
    } else {
      const float v = round_dst<D>(load1<S>(sp + i * SS) * scale);
      if (MODE & kModeReduce) acc[0] = __builtin_fmaf(v, v, acc[0]);
      if (kWrite) store1<D>(dp + i * DS, v * coef);
    }
  }

  const char* sb = sp + head * SS;
  char* db = dp + head * DS;
  constexpr int64_t kStep = (int64_t)kBlockThreads * kUnroll;
  int64_t v0 = 0;
  for (; v0 + kStep <= nvec; v0 += kStep) {
    Raw<S> in[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      in[u] = load_raw<S>(sb + (v0 + u * kBlockThreads + tid) * (kVecElems * SS));
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t v = v0 + u * kBlockThreads + tid;
      if (S == D && raw_copy) {
        Raw<D> out;
        __builtin_memcpy(&out, &in[u], sizeof(out));
        store_raw<D>(db + v * (kVecElems * DS), out);
      } else {
        Raw<D> out;
        compute8<S, D, MODE>(in[u], out, acc, scale, coef);
        if (kWrite) store_raw<D>(db + v * (kVecElems * DS), out);
      }
    }
  }
  if (v0 < nvec) {
    Raw<S> in[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t v = v0 + u * kBlockThreads + tid;
      if (v < nvec) in[u] = load_raw<S>(sb + v * (kVecElems * SS));
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t v = v0 + u * kBlockThreads + tid;
      if (v < nvec) {
        if (S == D && raw_copy) {
          Raw<D> out;
          __builtin_memcpy(&out, &in[u], sizeof(out));
          store_raw<D>(db + v * (kVecElems * DS), out);
        } else {
          Raw<D> out;
          compute8<S, D, MODE>(in[u], out, acc, scale, coef);
          if (kWrite) store_raw<D>(db + v * (kVecElems * DS), out);
        }
      }
    }
  }
}

// Zero `nbytes` bytes at p (p and nbytes are multiples of 2).
__device__ __forceinline__ void zero_range(char* p, int64_t nbytes) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  int64_t head = (int64_t)((16u - (unsigned)(a & 15u)) & 15u);
  if (head > nbytes) head = nbytes;
  const int64_t nvec = (nbytes - head) / 16;
  const int64_t tail0 = head + nvec * 16;
  const int tid = threadIdx.x;
  const int nscalar = (int)((head + (nbytes - tail0)) / 2);
  if (tid < nscalar) {
    const int64_t off = tid < head / 2 ? (int64_t)tid * 2 : tail0 + ((int64_t)tid - head / 2) * 2;
    *reinterpret_cast<unsigned short*>(p + off) = 0;
  }
  const u32x4 z = {0u, 0u, 0u, 0u};
  for (int64_t v = tid; v < nvec; v += kBlockThreads) *reinterpret_cast<u32x4*>(p + head + v * 16) = z;
}

template <int S>
__device__ __forceinline__ int rescan_nonfinite(const char* sp, int64_t len) {
  int bad = 0;
  for (int64_t i = threadIdx.x; i < len; i += kBlockThreads)
    bad |= nonfinite_at<S>(sp + i * ElemSize<S>::value) ? 1 : 0;
  return bad;
}

template <int MODE>
__global__ __launch_bounds__(kBlockThreads) void pass_kernel(PassArgs a) {
  int64_t c = blockIdx.x;
  if (a.reverse) c = a.n_chunks - 1 - c;

  float coef = 1.0f;
  if (a.result != nullptr) {
    // Values produced by the finalize kernel earlier on the same stream.
    if (a.result->skipped != 0 && a.write_on_overflow == 0) return;
    coef = a.result->coef;
  }

  const TensorDesc t = a.tensors[a.chunk_tensor[c]];
  const int64_t start = (int64_t)a.chunk_index[c] * a.chunk_elems;
  int64_t len = t.numel - start;
  if (len > a.chunk_elems) len = a.chunk_elems;

  const int ss = t.src_dtype == RG_F32 ? 4 : 2;
  const int ds = t.dst_dtype == RG_F32 ? 4 : 2;
  const char* sp = reinterpret_cast<const char*>(t.src) + start * ss;
  char* dp = reinterpret_cast<char*>(t.dst) + start * ds;
  const bool raw_copy = (MODE == kModeWrite) && a.result == nullptr && a.scale == 1.0f;

  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int dst_kind = a.norm_of_source ? t.src_dtype : t.dst_dtype;
  if (t.src == nullptr || a.zero_fill) {
    if (MODE & kModeWrite) zero_range(dp, len * ds);
  } else {
    switch (t.src_dtype * 3 + dst_kind) {
      case RG_F32 * 3 + RG_F32: process_chunk<RG_F32, RG_F32, MODE>(sp, dp, len, a.scale, coef, raw_copy, acc); break;
      case RG_F32 * 3 + RG_F16: process_chunk<RG_F32, RG_F16, MODE>(sp, dp, len, a.scale, coef, raw_copy, acc); break;
      case RG_F32 * 3 + RG_BF16: process_chunk<RG_F32, RG_BF16, MODE>(sp, dp, len, a.scale, coef, raw_copy, acc); break;
      case RG_F16 * 3 + RG_F32: process_chunk<RG_F16, RG_F32, MODE>(sp, dp, len, a.scale, coef, raw_copy, acc); break;
      case RG_F16 * 3 + RG_F16: process_chunk<RG_F16, RG_F16, MODE>(sp, dp, len, a.scale, coef, raw_copy, acc); break;
      case RG_F16 * 3 + RG_BF16: process_chunk<RG_F16, RG_BF16, MODE>(sp, dp, len, a.scale, coef, raw_copy, acc); break;
      case RG_BF16 * 3 + RG_F32: process_chunk<RG_BF16, RG_F32, MODE>(sp, dp, len, a.scale, coef, raw_copy, acc); break;
      case RG_BF16 * 3 + RG_F16: process_chunk<RG_BF16, RG_F16, MODE>(sp, dp, len, a.scale, coef, raw_copy, acc); break;
      default: process_chunk<RG_BF16, RG_BF16, MODE>(sp, dp, len, a.scale, coef, raw_copy, acc); break;
    }
  }

  if (MODE & kModeReduce) {
    // Fixed-order combine: 8 lanes of the thread, 64 lanes of the wavefront by shuffle,
    // 4 wavefronts through LDS.  Everything past the per-thread fp32 sums is double.
    double s = (((double)acc[0] + (double)acc[1]) + ((double)acc[2] + (double)acc[3])) +
               (((double)acc[4] + (double)acc[5]) + ((double)acc[6] + (double)acc[7]));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off);
    __shared__ double wave_sum[kBlockThreads / 64];
    if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = s;
    __syncthreads();
    const double total = (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]);
    // A non-finite input makes its square, and so the chunk's sum, non-finite; a finite sum
    // therefore proves every input was finite.  Only chunks whose sum is not finite are
    // looked at again element by element (the sum can also overflow from finite inputs).
    int bad = 0;
    if (!(fabs(total) <= 1.79769313486231570e308)) {
      int mine = 0;
      if (t.src != nullptr) {
        if (t.src_dtype == RG_F32) mine = rescan_nonfinite<RG_F32>(sp, len);
        else if (t.src_dtype == RG_F16) mine = rescan_nonfinite<RG_F16>(sp, len);
        else mine = rescan_nonfinite<RG_BF16>(sp, len);
      }
      bad = __syncthreads_or(mine);
    }
    if (threadIdx.x == 0) {
      a.chunk_sumsq[c] = total;
      a.chunk_bad[c] = bad;
    }
  }
}

// Wavefront w of the grid reduces tensor w's chunk sums (lane-strided, then a fixed
// shuffle tree) to n_t = float(sqrt(sum)).  The last block to finish then adds
// double(n_t)^2 over all tensors in a fixed order and derives the clip decision.
__global__ __launch_bounds__(kBlockThreads) void finalize_kernel(FinalizeArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int t = blockIdx.x * (kBlockThreads / 64) + wave;
  if (t < a.n_tensors) {
    double s = 0.0;
    int bad = 0;
    const int64_t end = a.tensor_chunk_begin[t + 1];
    for (int64_t c = a.tensor_chunk_begin[t] + lane; c < end; c += 64) {
      s += a.chunk_sumsq[c];
      bad |= a.chunk_bad[c];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      s += __shfl_down(s, off);
      bad |= __shfl_down(bad, off);
    }
    if (lane == 0) {
      const float n = (float)sqrt(s);
      a.tensor_norm[t] = n;
      a.tensor_sq[t] = (double)n * (double)n;
      a.tensor_bad[t] = bad;
    }
  }

  __shared__ int is_last;
  __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned prev = atomicAdd(a.ticket, 1u);
    is_last = (prev == gridDim.x - 1) ? 1 : 0;
  }
  __syncthreads();
  if (!is_last) return;
  __threadfence();

  double s = 0.0;
  int bad = 0;
  for (int i = threadIdx.x; i < a.n_tensors; i += kBlockThreads) {
    s += a.tensor_sq[i];
    bad |= a.tensor_bad[i];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    s += __shfl_down(s, off);
    bad |= __shfl_down(bad, off);
  }
  __shared__ double wave_sum[kBlockThreads / 64];
  __shared__ int wave_bad[kBlockThreads / 64];
  if (lane == 0) {
    wave_sum[wave] = s;
    wave_bad[wave] = bad;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const double total = (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]);
    const int overflow = (wave_bad[0] | wave_bad[1] | wave_bad[2] | wave_bad[3]) != 0 ? 1 : 0;
    const double norm = sqrt(total);
    const double g = norm + 1e-6;
    const bool gate = overflow != 0 && a.ignore_overflow == 0;
    const bool clip = a.max_norm > 0.0f && !gate && (g > (double)a.max_norm);
    a.result->norm = norm;
    a.result->coef = clip ? (float)((double)a.max_norm / g) : 1.0f;
    a.result->overflow = overflow;
    a.result->clipped = clip ? 1 : 0;
    a.result->skipped = gate ? 1 : 0;
    *a.ticket = 0u;
  }
}

__global__ __launch_bounds__(kBlockThreads) void fill_zero_kernel(char* p, int64_t nbytes) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  int64_t head = (int64_t)((16u - (unsigned)(a & 15u)) & 15u);
  if (head > nbytes) head = nbytes;
  const int64_t nvec = (nbytes - head) / 16;
  const int64_t tail0 = head + nvec * 16;
  const int64_t gtid = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * kBlockThreads;
  const int64_t nscalar = head + (nbytes - tail0);
  if (gtid < nscalar) p[gtid < head ? gtid : tail0 + (gtid - head)] = 0;
  const u32x4 z = {0u, 0u, 0u, 0u};
  for (int64_t v = gtid; v < nvec; v += nthreads) *reinterpret_cast<u32x4*>(p + head + v * 16) = z;
}

}  // namespace

hipError_t launch_pass(int mode, const PassArgs& a, hipStream_t stream) {
  if (a.n_chunks <= 0) return hipSuccess;
  const dim3 grid((unsigned)a.n_chunks), block(kBlockThreads);
  switch (mode) {
    case kModeReduce: hipLaunchKernelGGL(pass_kernel<kModeReduce>, grid, block, 0, stream, a); break;
    case kModeWrite: hipLaunchKernelGGL(pass_kernel<kModeWrite>, grid, block, 0, stream, a); break;
    default: hipLaunchKernelGGL(pass_kernel<kModeReduce | kModeWrite>, grid, block, 0, stream, a); break;
  }
  return hipGetLastError();
}

hipError_t launch_finalize(const FinalizeArgs& a, hipStream_t stream) {
  const int waves_per_block = kBlockThreads / 64;
  int blocks = (a.n_tensors + waves_per_block - 1) / waves_per_block;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(finalize_kernel, dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_fill_zero(void* dst, int64_t nbytes, hipStream_t stream) {
  if (nbytes <= 0) return hipSuccess;
  int64_t blocks = (nbytes / 16 + (int64_t)kBlockThreads * 4 - 1) / ((int64_t)kBlockThreads * 4);
  if (blocks < 1) blocks = 1;
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream,
                     reinterpret_cast<char*>(dst), nbytes);
  return hipGetLastError();
}

}  // namespace rg
