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
//
// Streaming (NT) stores come in three forms.  The default is the compiler's nontemporal store (`nt`).  A
// translation unit that defines RG_STREAM_STORE_AUX before including this header gets them issued as raw buffer
// stores with those cache-policy bits (1 = sc0, 2 = nt, 16 = sc1): measured on MI355X, "sc1 nt" (agent-scope
// write-through, streaming) is 1.5-3 % faster than plain `nt` for the passes that write one stream per launch and
// slower for the optimizer step's three.  Buffer instructions because they take the bits as an operand and - unlike
// a global store spelled out in an asm statement, which RG_STREAM_STORE_BITS still offers for comparison - are
// known to the compiler's wait-count bookkeeping: with an invisible store in flight the compiler believes the load
// it waits for is the only outstanding operation and drains the whole counter (vmcnt(0)), store included, where
// vmcnt(1) would do.  That over-wait, not the store, was what a pass paid for whenever it had work left after its
// last store (the pass that sums while it writes: 4-5 %).
//
// The descriptor's base is the address of the wavefront's first active lane, the lane's distance from it the
// offset: lanes ascend in address in every kernel of this library.
#ifndef RG_NT_STORES
#define RG_NT_STORES 1
#endif
__device__ __forceinline__ __amdgpu_buffer_rsrc_t wave_window(char* p, uint32_t& off) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  const uint64_t base = ((uint64_t)hi << 32) | lo;
  off = (uint32_t)(a - base);
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(base), 0, -1, 0x00020000);   // raw, unbounded
}
template <int AUX> __device__ __forceinline__ void st16_aux(char* p, u32x4 v) {
  uint32_t off;
  const __amdgpu_buffer_rsrc_t r = wave_window(p, off);
  __builtin_amdgcn_raw_buffer_store_b128(v, r, off, 0, AUX);
}
template <int AUX> __device__ __forceinline__ void st8_aux(char* p, u32x2 v) {
  uint32_t off;
  const __amdgpu_buffer_rsrc_t r = wave_window(p, off);
  __builtin_amdgcn_raw_buffer_store_b64(v, r, off, 0, AUX);
}
// gfx940-family hazard: a VALU instruction that overwrites the data registers of a store of more than 64 bits
// within two wait states of it changes what is stored.  The compiler spaces its own stores accordingly, but it
// does not know that an asm statement is a store, so every 128-bit store issued through asm brings its own two
// wait states (the 64-bit ones are not affected).
#define RG_STORE_HAZARD_NOP "\n\ts_nop 1"
template <bool NT> __device__ __forceinline__ void st16(char* p, u32x4 v) {
  RG_GLOBAL u32x4_a2* g = (RG_GLOBAL u32x4_a2*)p;
#if defined(RG_STREAM_STORE_AUX)
  if (NT) {
    st16_aux<RG_STREAM_STORE_AUX>(p, v);
    return;
  }
#elif defined(RG_STREAM_STORE_BITS)
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
#if defined(RG_STREAM_STORE_AUX)
  if (NT) {
    st8_aux<RG_STREAM_STORE_AUX>(p, v);
    return;
  }
#elif defined(RG_STREAM_STORE_BITS)
  if (NT) {
    asm volatile("global_store_dwordx2 %0, %1, off " RG_STREAM_STORE_BITS : : "v"(g), "v"(v));
    return;
  }
#endif
  if (NT && RG_NT_STORES) __builtin_nontemporal_store(v, g);
  else *g = v;
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

// One element at a time (unaligned heads, ragged tails, the re-scan after a non-finite sum).  Through pointers of
// the global address space, like the vector accesses: a generic pointer compiles to FLAT instructions, which count
// on two of the wave's counters at once, and the compiler then waits for both to drain (vmcnt(0) lgkmcnt(0)) before
// it reuses one of their registers - a wait that also covers every vector store still in flight.
template <int DT> __device__ __forceinline__ void store1(char* p, float v) {
  *(RG_GLOBAL float*)p = v;
}
template <> __device__ __forceinline__ void store1<RG_F16>(char* p, float v) {
  *(RG_GLOBAL _Float16*)p = f32_to_f16(v);
}
template <> __device__ __forceinline__ void store1<RG_BF16>(char* p, float v) {
  *(RG_GLOBAL unsigned short*)p = (unsigned short)f32_to_bf16_bits(v);
}
__device__ __forceinline__ uint32_t load_u32(const char* p) { return *(const RG_GLOBAL uint32_t*)p; }
__device__ __forceinline__ uint32_t load_u16(const char* p) { return (uint32_t)*(const RG_GLOBAL unsigned short*)p; }
__device__ __forceinline__ void store_u32(char* p, uint32_t v) { *(RG_GLOBAL uint32_t*)p = v; }
__device__ __forceinline__ void store_u16(char* p, uint32_t v) { *(RG_GLOBAL unsigned short*)p = (unsigned short)v; }
__device__ __forceinline__ void store_u8(char* p, uint32_t v) { *(RG_GLOBAL unsigned char*)p = (unsigned char)v; }

template <int DT> __device__ __forceinline__ bool nonfinite_at(const char* p) {
  return (load_u32(p) & 0x7f800000u) == 0x7f800000u;
}
template <> __device__ __forceinline__ bool nonfinite_at<RG_F16>(const char* p) {
  return (load_u16(p) & 0x7c00u) == 0x7c00u;
}
template <> __device__ __forceinline__ bool nonfinite_at<RG_BF16>(const char* p) {
  return (load_u16(p) & 0x7f80u) == 0x7f80u;
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

}  // namespace
}  // namespace rg
