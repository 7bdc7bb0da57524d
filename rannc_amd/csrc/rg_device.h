// Device-side helpers shared by the kernels of libranncgrad: element-aligned vector memory
// access, dtype conversion, packing of E elements per lane.
#pragma once

#include "rg_internal.h"

namespace rg {
namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// Vector types whose alignment is only that of one element (2 or 4 bytes).
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
typedef u32x2 u32x2_a2 __attribute__((aligned(2)));

template <int DT> struct ElemSize { static constexpr int value = 2; };
template <> struct ElemSize<RG_F32> { static constexpr int value = 4; };

// E elements of type DT as they sit in memory: 8 or 16 bytes.
template <int DT, int E> struct Raw;
template <> struct Raw<RG_F32, 4> { u32x4 v; };
template <> struct Raw<RG_F16, 4> { u32x2 v; };
template <> struct Raw<RG_BF16, 4> { u32x2 v; };
template <> struct Raw<RG_F16, 8> { u32x4 v; };
template <> struct Raw<RG_BF16, 8> { u32x4 v; };

// Every pointer these helpers see addresses device (global) memory; pointers read from a
// table in memory are "generic" to the compiler, which would then emit flat_* instructions
// (slower to issue, and they tie up the LDS counter).  The casts below state the address
// space, so the accesses compile to global_* whatever the compiler could infer.
#define RG_GLOBAL __attribute__((address_space(1)))

// Loads at element alignment.
template <bool NT> __device__ __forceinline__ u32x4 ld16_a4(const char* p) {
  const RG_GLOBAL u32x4_a4* g = (const RG_GLOBAL u32x4_a4*)p;
  return NT ? __builtin_nontemporal_load(g) : *g;
}
template <bool NT> __device__ __forceinline__ u32x4 ld16_a2(const char* p) {
  const RG_GLOBAL u32x4_a2* g = (const RG_GLOBAL u32x4_a2*)p;
  return NT ? __builtin_nontemporal_load(g) : *g;
}
template <bool NT> __device__ __forceinline__ u32x2 ld8_a2(const char* p) {
  const RG_GLOBAL u32x2_a2* g = (const RG_GLOBAL u32x2_a2*)p;
  return NT ? __builtin_nontemporal_load(g) : *g;
}
// Stores: the pointer type promises element alignment only (what the peel guarantees beyond
// that is a performance matter, not a correctness one).
// Streaming (NT) stores come in two forms.  The default is the compiler's nontemporal store
// (`nt`).  A translation unit that defines RG_STREAM_STORE_BITS before including this header
// gets its streaming stores issued with exactly those cache-policy bits instead: measured on
// MI355X, "sc1 nt" (agent-scope write-through, streaming) is 1.5-3 % faster than plain `nt`
// for the passes that write one stream per launch and slower for the optimizer step's three.
#ifndef RG_NT_STORES
#define RG_NT_STORES 1
#endif
// gfx940-family hazard: a VALU instruction that overwrites the data registers of a store of more than 64 bits
// within two wait states of it changes what is stored.  The compiler spaces its own stores accordingly, but it
// does not know that an asm statement is a store, so every 128-bit store issued through asm brings its own two
// wait states (the 64-bit ones are not affected).
#define RG_STORE_HAZARD_NOP "\n\ts_nop 1"
template <bool NT> __device__ __forceinline__ void st16(char* p, u32x4 v) {
  RG_GLOBAL u32x4_a2* g = (RG_GLOBAL u32x4_a2*)p;
#ifdef RG_STREAM_STORE_BITS
  if (NT) {
    asm volatile("global_store_dwordx4 %0, %1, off " RG_STREAM_STORE_BITS RG_STORE_HAZARD_NOP : : "v"(g), "v"(v));
    return;
  }
#endif
  if (NT && RG_NT_STORES) __builtin_nontemporal_store(v, g);
  else *g = v;
}
template <bool NT> __device__ __forceinline__ void st8(char* p, u32x2 v) {
  RG_GLOBAL u32x2_a2* g = (RG_GLOBAL u32x2_a2*)p;
#ifdef RG_STREAM_STORE_BITS
  if (NT) {
    asm volatile("global_store_dwordx2 %0, %1, off " RG_STREAM_STORE_BITS : : "v"(g), "v"(v));
    return;
  }
#endif
  if (NT && RG_NT_STORES) __builtin_nontemporal_store(v, g);
  else *g = v;
}

// Stores whose order in the instruction stream is fixed (volatile asm statements keep their relative order):
// st16_ordered is a plain 16-byte store, st16_last / st8_last are the stores above issued after it.
__device__ __forceinline__ void st16_ordered(char* p, u32x4 v) {
  RG_GLOBAL u32x4_a2* g = (RG_GLOBAL u32x4_a2*)p;
  asm volatile("global_store_dwordx4 %0, %1, off" RG_STORE_HAZARD_NOP : : "v"(g), "v"(v));
}
template <bool NT> __device__ __forceinline__ void st16_last(char* p, u32x4 v) {
  RG_GLOBAL u32x4_a2* g = (RG_GLOBAL u32x4_a2*)p;
#ifdef RG_STREAM_STORE_BITS
  if (NT) asm volatile("global_store_dwordx4 %0, %1, off " RG_STREAM_STORE_BITS RG_STORE_HAZARD_NOP : : "v"(g), "v"(v));
  else asm volatile("global_store_dwordx4 %0, %1, off" RG_STORE_HAZARD_NOP : : "v"(g), "v"(v));
#else
  if (NT) asm volatile("global_store_dwordx4 %0, %1, off nt" RG_STORE_HAZARD_NOP : : "v"(g), "v"(v));
  else asm volatile("global_store_dwordx4 %0, %1, off" RG_STORE_HAZARD_NOP : : "v"(g), "v"(v));
#endif
}
template <bool NT> __device__ __forceinline__ void st8_last(char* p, u32x2 v) {
  RG_GLOBAL u32x2_a2* g = (RG_GLOBAL u32x2_a2*)p;
#ifdef RG_STREAM_STORE_BITS
  if (NT) asm volatile("global_store_dwordx2 %0, %1, off " RG_STREAM_STORE_BITS : : "v"(g), "v"(v));
  else asm volatile("global_store_dwordx2 %0, %1, off" : : "v"(g), "v"(v));
#else
  if (NT) asm volatile("global_store_dwordx2 %0, %1, off nt" : : "v"(g), "v"(v));
  else asm volatile("global_store_dwordx2 %0, %1, off" : : "v"(g), "v"(v));
#endif
}

template <int DT, int E, bool NT> struct Mem;
template <bool NT> struct Mem<RG_F32, 4, NT> {
  static __device__ __forceinline__ Raw<RG_F32, 4> load(const char* p) { return {ld16_a4<NT>(p)}; }
  static __device__ __forceinline__ void store(char* p, const Raw<RG_F32, 4>& r) { st16<NT>(p, r.v); }
};
template <int DT, bool NT> struct Mem<DT, 4, NT> {   // 16-bit types, 4 elements = 8 bytes
  static __device__ __forceinline__ Raw<DT, 4> load(const char* p) { return {ld8_a2<NT>(p)}; }
  static __device__ __forceinline__ void store(char* p, const Raw<DT, 4>& r) { st8<NT>(p, r.v); }
};
template <int DT, bool NT> struct Mem<DT, 8, NT> {   // 16-bit types, 8 elements = 16 bytes
  static __device__ __forceinline__ Raw<DT, 8> load(const char* p) { return {ld16_a2<NT>(p)}; }
  static __device__ __forceinline__ void store(char* p, const Raw<DT, 8>& r) { st16<NT>(p, r.v); }
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// fp16 <-> fp32 conversions are kept apart from the neighbouring multiplies: left alone the
// compiler folds `(_Float16)(x * s)` into a mixed-precision fma with a +0 addend, which
// turns a -0 product into +0.  The empty asm makes the fp32 value opaque at that point.
__device__ __forceinline__ float opaque(float f) {
  asm("" : "+v"(f));
  return f;
}
__device__ __forceinline__ _Float16 f32_to_f16(float f) { return (_Float16)opaque(f); }
__device__ __forceinline__ float f16_to_f32(_Float16 h) { return opaque((float)h); }

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(unsigned short, f32_to_f16(f));
}

// fp32 -> bf16, round to nearest even, two elements per v_cvt_pk_bf16_f32 (the integer
// formulation costs eight ALU operations per element, which shows in a 6-byte-per-element
// copy).  A NaN stays a NaN; its payload bits are not specified.
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  const f32x2 v = {opaque(lo), opaque(hi)};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return f32x2_to_bf16x2_bits(f, 0.0f) & 0xffffu; }

template <int DT> __device__ __forceinline__ void unpack_word(uint32_t w, float& lo, float& hi);
template <> __device__ __forceinline__ void unpack_word<RG_F16>(uint32_t w, float& lo, float& hi) {
  const f16x2 h = __builtin_bit_cast(f16x2, w);   // bit_cast needs a scalar, not a vector-element lvalue
  lo = f16_to_f32(h.x);
  hi = f16_to_f32(h.y);
}
template <> __device__ __forceinline__ void unpack_word<RG_BF16>(uint32_t w, float& lo, float& hi) {
  lo = __uint_as_float(w << 16);
  hi = __uint_as_float(w & 0xffff0000u);
}
template <int DT> __device__ __forceinline__ uint32_t pack_word(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack_word<RG_F16>(float lo, float hi) {
  return f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);
}
template <> __device__ __forceinline__ uint32_t pack_word<RG_BF16>(float lo, float hi) {
  return f32x2_to_bf16x2_bits(lo, hi);
}

template <int DT, int E> struct Codec {   // 16-bit types
  static __device__ __forceinline__ void unpack(const Raw<DT, E>& r, float (&f)[E]) {
#pragma unroll
    for (int j = 0; j < E / 2; ++j) {
      const uint32_t w = r.v[j];
      unpack_word<DT>(w, f[2 * j], f[2 * j + 1]);
    }
  }
  static __device__ __forceinline__ Raw<DT, E> pack(const float (&f)[E]) {
    Raw<DT, E> r;
#pragma unroll
    for (int j = 0; j < E / 2; ++j) r.v[j] = pack_word<DT>(f[2 * j], f[2 * j + 1]);
    return r;
  }
};
template <> struct Codec<RG_F32, 4> {
  static __device__ __forceinline__ void unpack(const Raw<RG_F32, 4>& r, float (&f)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) f[j] = __uint_as_float(r.v[j]);
  }
  static __device__ __forceinline__ Raw<RG_F32, 4> pack(const float (&f)[4]) {
    Raw<RG_F32, 4> r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r.v[j] = __float_as_uint(f[j]);
    return r;
  }
};

// The value as it reads back from a destination of type DT.
template <int DT> __device__ __forceinline__ float round_dst(float v) { return v; }
template <> __device__ __forceinline__ float round_dst<RG_F16>(float v) { return f16_to_f32(f32_to_f16(v)); }
template <> __device__ __forceinline__ float round_dst<RG_BF16>(float v) {
  return bf16_bits_to_f32(f32_to_bf16_bits(v));
}

template <int DT> __device__ __forceinline__ void store1(char* p, float v) {
  *reinterpret_cast<float*>(p) = v;
}
template <> __device__ __forceinline__ void store1<RG_F16>(char* p, float v) {
  *reinterpret_cast<_Float16*>(p) = f32_to_f16(v);
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

// Sum of one double per lane over the 64-lane wavefront, the same value returned to every
// lane.  An inclusive scan inside each row of 16 lanes with DPP row shifts (lanes without a
// source add zero), then the four row totals - read from lanes 15, 31, 47, 63 - are added
// in a fixed order.  About a tenth of the latency of six 64-bit shuffles through the LDS
// crossbar, which matters in passes whose blocks only live for a few microseconds.
// All 64 lanes must be active.
template <int N> __device__ __forceinline__ double dpp_row_shr(double x) {
  int lo = __double2loint(x), hi = __double2hiint(x);
  lo = __builtin_amdgcn_update_dpp(0, lo, 0x110 + N, 0xf, 0xf, false);
  hi = __builtin_amdgcn_update_dpp(0, hi, 0x110 + N, 0xf, 0xf, false);
  return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double read_lane(double x, int lane) {
  const int lo = __builtin_amdgcn_readlane(__double2loint(x), lane);
  const int hi = __builtin_amdgcn_readlane(__double2hiint(x), lane);
  return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double wave_total(double x) {
  x += dpp_row_shr<1>(x);
  x += dpp_row_shr<2>(x);
  x += dpp_row_shr<4>(x);
  x += dpp_row_shr<8>(x);
  return (read_lane(x, 15) + read_lane(x, 31)) + (read_lane(x, 47) + read_lane(x, 63));
}

// Sum of one float per lane over the wavefront in six DPP additions (two butterflies inside each quad, two row
// shifts, two row broadcasts: ((r3 + r2) + (r1 + r0)) of the row sums ends up in lane 63), returned to every lane.
// All 64 lanes must be active.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ float dpp_f32(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_total_f32(float x) {
  x += dpp_f32<0xb1, 0xf>(x);    // quad_perm:[1,0,3,2]
  x += dpp_f32<0x4e, 0xf>(x);    // quad_perm:[2,3,0,1]
  x += dpp_f32<0x114, 0xf>(x);   // row_shr:4
  x += dpp_f32<0x118, 0xf>(x);   // row_shr:8
  x += dpp_f32<0x142, 0xa>(x);   // row_bcast:15 into rows 1 and 3
  x += dpp_f32<0x143, 0xc>(x);   // row_bcast:31 into rows 2 and 3
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 63));
}

}  // namespace
}  // namespace rg
