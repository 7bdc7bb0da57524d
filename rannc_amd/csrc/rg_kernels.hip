// gfx950 kernels of libranncgrad.
//
// One "pass" kernel serves every per-step operation.  The grid is the plan's chunk list:
// block b reads one 32-byte chunk record (source pointer, destination pointer, length,
// element types) and streams that chunk, so a launch covers thousands of tensors of any
// size mix and a block needs a single table lookup before its first data load.
//
// Inside a chunk every load and store instruction is contiguous across the wavefront: a
// lane moves E consecutive elements per instruction, E = 4 when either side is fp32 and 8
// otherwise, so the wider side always moves 16 bytes per lane (1 KiB per wavefront
// instruction) and the narrower side 8.  Accesses only need element alignment: gfx950
// executes 2-byte-aligned 64/128-bit loads and stores.  Alignment is a performance matter:
// chunk boundaries sit on 128-byte boundaries of the written side, one head per tensor is
// peeled, and the read-only pass peels its source per chunk (see rg_internal.h).
//
// Plans whose data is far larger than the caches use nontemporal loads and stores: measured
// on MI355X that lifts a read-only pass from 6.3 to 7.1 TB/s, and nontemporal stores keep
// dirty lines from lingering in L2 / Infinity Cache where their write-back would slow the
// next kernel's reads.  Small plans use plain accesses so the second pass hits in cache.
//
// The work is purely bandwidth bound (a few ALU ops per element): no LDS staging and no
// MFMA.  LDS is used only for the 4-wavefront combine of the partial sums.
#include <atomic>
#include <cstdlib>
#include <type_traits>

// the passes of this file write one stream per launch: see the notes on streaming stores in rg_device.h
#if !defined(RG_STREAM_STORE_AUX) && !defined(RG_STREAM_STORE_BITS) && !defined(RG_STREAM_STORE_COMPILER_NT)
#define RG_STREAM_STORE_AUX (2 | 16)   // nt sc1
#endif
#include "rg_device.h"
#include "rg_internal.h"

// steps of a writing pass whose loads are issued together (see process_chunk)
#ifndef RG_WRITE_STEPS_IN_FLIGHT
#define RG_WRITE_STEPS_IN_FLIGHT 1
#endif
#ifndef RG_WRITE_STEPS_IN_FLIGHT_F32
#define RG_WRITE_STEPS_IN_FLIGHT_F32 1
#endif
#ifndef RG_SUM_WRITE_STEPS_IN_FLIGHT
#define RG_SUM_WRITE_STEPS_IN_FLIGHT 2
#endif
#ifndef RG_ACC_STEPS_IN_FLIGHT
#define RG_ACC_STEPS_IN_FLIGHT 1
#endif

namespace rg {
namespace {

// Block size of a pass: passes that write use smaller blocks than the read-only one.
template <int MODE> struct PassThreads { static constexpr int value = (MODE & kModeWrite) ? kWriteThreads : kBlockThreads; };

// One chunk.  v = round_dst(x * scale); sum += v^2; out = round_dst(v * coef).
// coef is 1 when nothing is clipped: v * 1 is v bit for bit, so no branch is needed.
// The two multiplies are never fused or reassociated (the file is built with
// -ffp-contract=off), so the result matches `x.float() * inv_scale` then `mul_(coef)`.
template <int S, int D, int MODE, bool NT, int T = PassThreads<MODE>::value, bool HEAD = true>
__device__ __forceinline__ void process_chunk(const char* sp, char* dp, int len, float scale, float coef,
                                              bool raw_copy, float (&acc)[8]) {
  constexpr int SS = ElemSize<S>::value;
  constexpr int DS = ElemSize<D>::value;
  constexpr bool kWrite = (MODE & kModeWrite) != 0;
  constexpr bool kReduce = (MODE & kModeReduce) != 0;
  constexpr bool kAcc = (MODE & kModeAccumulate) != 0;   // dst = round_dst(float(dst) + x * scale)
  constexpr int E = (SS == 4 || (kWrite && DS == 4)) ? 4 : 8;   // elements per lane per instruction
  // a read-only pass keeps 128 bytes of source in flight per lane (eight 16-byte loads) whatever the element size
  // A writing pass moves one vector per lane and step.  The pass that also sums issues the loads of both its steps
  // before the first store (measured with stores the compiler can account for: +1.5-3 points on every workload,
  // where the plain write pass loses 0.5-1.5 with 16-bit sources and the accumulating passes lose 1-2).
  constexpr int kSteps = kAcc ? RG_ACC_STEPS_IN_FLIGHT : ((kReduce && kWrite) ? RG_SUM_WRITE_STEPS_IN_FLIGHT : (SS == 4 ? RG_WRITE_STEPS_IN_FLIGHT_F32 : RG_WRITE_STEPS_IN_FLIGHT));
  constexpr int kPerThread = kReduceElemsPerThread * (4 / SS);   // read-only pass
  constexpr int U = kWrite ? kSteps * (kWriteElemsPerThread / 4) : (kPerThread >= E ? kPerThread / E : 1);   // instructions in flight per lane
  constexpr int AS = kWrite ? DS : SS;
  constexpr unsigned kPeel = kWrite ? kWriteAlignBytes : kAlignBytes;
  const uintptr_t a = kWrite ? reinterpret_cast<uintptr_t>(dp) : reinterpret_cast<uintptr_t>(sp);
  // HEAD == false: the caller has checked that the peeled side starts on a boundary.
  int head = HEAD ? (int)(((kPeel - (unsigned)(a & (kPeel - 1))) & (kPeel - 1)) / (unsigned)AS) : 0;
  if (head > len) head = len;
  const int nbody = (len - head) / E * E;
  const int tail0 = head + nbody;
  const int tid = threadIdx.x;

  // Unaligned head (read-only pass: < 128 bytes) and ragged tail (< E elements): one element per thread, after the
  // vector loop (a load issued up here, to overlap its latency with the vector loads, leaves the compiler with a
  // register it believes in flight on the path around that loop, and the wait it then places behind the loop - for
  // every block, with or without scalar elements - also waits for the vector stores: see the end of this function).
  const int nscalar = head + (len - tail0);
  auto scalar_index = [&](int k) { return k < head ? k : tail0 + (k - head); };
  auto scalar_load = [&](int i) -> uint32_t {
    return SS == 4 ? load_u32(sp + (size_t)i * 4) : load_u16(sp + (size_t)i * 2);
  };
  auto scalar_finish = [&](uint32_t raw, int i) {
    if (S == D && raw_copy) {
      if (SS == 4) store_u32(dp + (size_t)i * 4, raw);
      else store_u16(dp + (size_t)i * 2, raw);
    } else {
      float x;
      if (S == RG_F32) x = __uint_as_float(raw);
      else if (S == RG_F16) x = f16_to_f32(__builtin_bit_cast(_Float16, (unsigned short)raw));
      else x = bf16_bits_to_f32(raw);
      float t = x * scale;
      if (kAcc) {
        float old;
        if (D == RG_F32) old = __uint_as_float(load_u32(dp + (size_t)i * 4));
        else if (D == RG_F16) old = f16_to_f32(__builtin_bit_cast(_Float16, (unsigned short)load_u16(dp + (size_t)i * 2)));
        else old = bf16_bits_to_f32(load_u16(dp + (size_t)i * 2));
        t = opaque(t) + old;
      }
      const float v = round_dst<D>(t);
      if (kReduce) acc[0] = __builtin_fmaf(v, v, acc[0]);
      if (kWrite) store1<D>(dp + (size_t)i * DS, v * coef);
    }
  };

  const char* sb = sp + (size_t)head * SS;
  char* db = dp + (size_t)head * DS;
  constexpr int kIter = T * E * U;   // elements per block iteration

  // All U loads of an iteration are issued back to back with no branch between them, so
  // they are all in flight together.  `valid` only guards what is accumulated and stored.
  // previous destination values, only when accumulating (the type does not exist otherwise)
  struct Nothing {};
  using Old = std::conditional_t<kAcc, Raw<kAcc ? D : S, E>, Nothing>;
  auto consume = [&](const Raw<S, E>& in, const Old* old, int e, bool valid) {
    bool copied = false;
    if constexpr (S == D && kWrite) {
      if (raw_copy) {
        if (valid) Mem<D, E, NT>::store(db + (size_t)e * DS, in);
        copied = true;
      }
    }
    if (!copied) {
      float f[E];
      Codec<S, E>::unpack(in, f);
      float o[E];
      if constexpr (kAcc) Codec<D, E>::unpack(*old, o);
#pragma unroll
      for (int j = 0; j < E; ++j) {
        float t = f[j] * scale;
        if constexpr (kAcc) t = opaque(t) + o[j];   // product rounded first, then the sum
        float v = round_dst<D>(t);
        if (kReduce) {
          const float q = valid ? v : 0.0f;
          acc[j & 7] = __builtin_fmaf(q, q, acc[j & 7]);
        }
        if (kWrite) f[j] = round_dst<D>(v * coef);
      }
      if constexpr (kWrite) {
        if (valid) Mem<D, E, NT>::store(db + (size_t)e * DS, Codec<D, E>::pack(f));
      }
    }
  };

  int base = 0;
  for (; base + kIter <= nbody; base += kIter) {
    Raw<S, E> in[U];
    Old old[kAcc ? U : 1];
#pragma unroll
    for (int u = 0; u < U; ++u) in[u] = Mem<S, E, NT>::load(sb + (size_t)(base + (u * T + tid) * E) * SS);
    if constexpr (kAcc) {
#pragma unroll
      for (int u = 0; u < U; ++u) old[u] = Mem<D, E, NT>::load(db + (size_t)(base + (u * T + tid) * E) * DS);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) consume(in[u], &old[kAcc ? u : 0], base + (u * T + tid) * E, true);
  }
  if (base < nbody) {
    // Last, partial iteration: lanes past the end re-read the final vector (an address that
    // is certainly valid) so the loads stay unconditional, and are masked afterwards.
    Raw<S, E> in[U];
    Old old[kAcc ? U : 1];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int e = base + (u * T + tid) * E;
      in[u] = Mem<S, E, NT>::load(sb + (size_t)(e < nbody ? e : nbody - E) * SS);
      if constexpr (kAcc) old[u] = Mem<D, E, NT>::load(db + (size_t)(e < nbody ? e : nbody - E) * DS);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int e = base + (u * T + tid) * E;
      consume(in[u], &old[kAcc ? u : 0], e, e < nbody);
    }
  }

  // Block-uniform: most tiles have neither head nor tail.  The scalar stores in here are the only memory operations
  // the compiler knows to be in flight (the streaming vector stores are asm statements), and it waits for them -
  // with vmcnt(0), which covers those vector stores as well - before the first later instruction that reuses one of
  // their registers.  Left to the compiler that wait lands behind the join, in the path of every wavefront: a pass
  // that goes on to reduce and store a record then sits there until its last vector store has been acknowledged,
  // one more trip to memory in a block that lives for two (measured: 4-5 % of the pass).  Waiting inside the
  // branch keeps the common path free of it.
  if (nscalar > 0) {
    for (int k = tid; k < nscalar; k += T) {
      const int i = scalar_index(k);
      scalar_finish(scalar_load(i), i);
    }
#ifndef RG_NO_TAIL_WAIT
    __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0), expcnt untouched
#endif
  }
}

// Zero `nbytes` bytes at p (p and nbytes are multiples of 2).
template <bool NT, int T, bool PEEL>
__device__ __forceinline__ void zero_range(char* p, int nbytes) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  int head = PEEL ? (int)((kWriteAlignBytes - (unsigned)(a & (kWriteAlignBytes - 1))) & (kWriteAlignBytes - 1)) : 0;
  if (head > nbytes) head = nbytes;
  const int nvec = (nbytes - head) / 16;
  const int tail0 = head + nvec * 16;
  const int tid = threadIdx.x;
  const int nscalar = (head + (nbytes - tail0)) / 2;
  for (int k = tid; k < nscalar; k += T) {
    const int off = k < head / 2 ? k * 2 : tail0 + (k - head / 2) * 2;
    store_u16(p + off, 0u);
  }
  const u32x4 z = {0u, 0u, 0u, 0u};
  for (int v = tid; v < nvec; v += T) st16<NT>(p + head + (size_t)v * 16, z);
}

template <int S, int T>
__device__ __forceinline__ int rescan_nonfinite(const char* sp, int len) {
  int bad = 0;
  for (int i = threadIdx.x; i < len; i += T)
    bad |= nonfinite_at<S>(sp + (size_t)i * ElemSize<S>::value) ? 1 : 0;
  return bad;
}

// What one block does with block index `bid` of a pass (after any block -> XCD remapping):
// tile (bid % tiles_per_chunk) of chunk (bid / tiles_per_chunk).
// PEEL (writing passes only): some tensor's destination starts off a 128-byte boundary, so
// blocks look for an unaligned head.  Plans whose destinations are all aligned run the
// variant compiled without that logic (about 1 % faster on BERT-large).
template <int MODE, bool NT, bool PEEL>
__device__ __forceinline__ void pass_block(const PassArgs& a, unsigned bid, float coef) {
  constexpr int T = PassThreads<MODE>::value;
  const int64_t c = (int64_t)(bid / (unsigned)a.tiles_per_chunk);
  const int tile = (int)(bid % (unsigned)a.tiles_per_chunk);
  ChunkRec rec;
  if (a.chunks != nullptr) {
    rec = a.chunks[c];
  } else {
    // plan-free launch over one tensor: chunk c is a fixed-size slice of it
    rec = a.single;
    int64_t first = c == 0 ? 0 : a.single_head + c * a.single_chunk_elems;
    int64_t last = a.single_head + (c + 1) * a.single_chunk_elems;
    if (first > a.single_numel) first = a.single_numel;
    if (last > a.single_numel) last = a.single_numel;
    rec.len = (int32_t)(last - first);
    if (rec.src) rec.src = reinterpret_cast<const char*>(rec.src) + first * (rec.src_dtype == RG_F32 ? 4 : 2);
    rec.dst = reinterpret_cast<char*>(rec.dst) + first * (rec.dst_dtype == RG_F32 ? 4 : 2);
  }
  // Tiles are laid out from the first aligned boundary of the chunk's written side, so only
  // tile 0 of a chunk can have an unaligned head; the last tile takes whatever remains.
  int chunk_head = 0;
  if (PEEL && a.tiles_per_chunk > 1) {
    chunk_head = head_elems(reinterpret_cast<uintptr_t>(rec.dst), kWriteAlignBytes, rec.dst_dtype == RG_F32 ? 4u : 2u);
    if (chunk_head > rec.len) chunk_head = rec.len;
  }
  const size_t slot_id = bid;   // of this block's partial sums
  const int start = tile == 0 ? 0 : chunk_head + tile * a.tile_elems;
  int end = tile == a.tiles_per_chunk - 1 ? rec.len : chunk_head + (tile + 1) * a.tile_elems;
  if (end > rec.len) end = rec.len;
  // A pass that reduces and writes leaves one partial per tile, a read-only pass one per chunk.  (Per-wavefront
  // partials, without the barrier, were the faster form only while every wavefront also sat out a full drain of its
  // memory counter after its last store; since that wait is gone, one record per tile is 0.5 points faster and
  // halves what the reduction has to read.)
  constexpr bool kWavePartials = (MODE & kModeReduce) != 0 && (MODE & kModeWrite) != 0;
  constexpr int kSlots = kWavePartials ? kWaveSlotsPerTile : 1;
  if (start >= end) {
    if constexpr ((MODE & kModeReduce) != 0) {
      if (threadIdx.x < kSlots) a.partials[slot_id * kSlots + threadIdx.x] = Partial{0.0, 0, 0};
    }
    return;
  }
  const int len = end - start;
  if (a.src_is_dst) {
    rec.src = rec.dst;
    rec.src_dtype = rec.dst_dtype;
  }
  const char* sp = rec.src ? reinterpret_cast<const char*>(rec.src) + (size_t)start * (rec.src_dtype == RG_F32 ? 4 : 2) : nullptr;
  char* dp = reinterpret_cast<char*>(rec.dst) + (size_t)start * (rec.dst_dtype == RG_F32 ? 4 : 2);
  const int src_kind = rec.src_dtype;
  const int dst_kind = a.norm_of_source ? rec.src_dtype : rec.dst_dtype;
  const float scale = a.scale_dev != nullptr ? *a.scale_dev : a.scale;   // a scale kept on the device (a loss scaler's state)
  const bool raw_copy = (MODE == kModeWrite) && a.result == nullptr && a.scale_dev == nullptr && a.scale == 1.0f;   // never when accumulating

  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (sp == nullptr || a.zero_fill) {
    if constexpr ((MODE & kModeAccumulate) != 0) {
      // Nothing to add: the destination keeps its values, which still count towards the norm.
      if constexpr ((MODE & kModeReduce) != 0) {
        if (dst_kind == RG_F32) process_chunk<RG_F32, RG_F32, kModeReduce, NT, T>(dp, dp, len, 1.0f, 1.0f, false, acc);
        else if (dst_kind == RG_F16) process_chunk<RG_F16, RG_F16, kModeReduce, NT, T>(dp, dp, len, 1.0f, 1.0f, false, acc);
        else process_chunk<RG_BF16, RG_BF16, kModeReduce, NT, T>(dp, dp, len, 1.0f, 1.0f, false, acc);
      }
    } else if (MODE & kModeWrite) {
      if (NT && a.zero_delay_ticks > 0) {   // see rg_zero
        const uint64_t t_end = wall_clock64() + (uint64_t)a.zero_delay_ticks;
        while (wall_clock64() < t_end) __builtin_amdgcn_s_sleep(1);
      }
      zero_range<NT, T, PEEL>(dp, len * (rec.dst_dtype == RG_F32 ? 4 : 2));
    }
  } else {
    // Blocks that start on a boundary of the peeled side (all but one per tensor, when the
    // other passes' chunks are aligned too) take the variant without head handling.
    const unsigned peel = (MODE & kModeWrite) ? kWriteAlignBytes : kAlignBytes;
    const uintptr_t peeled = (MODE & kModeWrite) ? reinterpret_cast<uintptr_t>(dp) : reinterpret_cast<uintptr_t>(sp);
    const bool has_head = ((MODE & kModeWrite) == 0 || PEEL) && (peeled & (peel - 1)) != 0;
#define RG_PAIR(S, D)                                                                         \
  case S * 3 + D:                                                                             \
    if (has_head) process_chunk<S, D, MODE, NT, T, true>(sp, dp, len, scale, coef, raw_copy, acc);  \
    else process_chunk<S, D, MODE, NT, T, false>(sp, dp, len, scale, coef, raw_copy, acc);  \
    break;
    switch (src_kind * 3 + dst_kind) {
      RG_PAIR(RG_F32, RG_F32)
      RG_PAIR(RG_F32, RG_F16)
      RG_PAIR(RG_F32, RG_BF16)
      RG_PAIR(RG_F16, RG_F32)
      RG_PAIR(RG_F16, RG_F16)
      RG_PAIR(RG_F16, RG_BF16)
      RG_PAIR(RG_BF16, RG_F32)
      RG_PAIR(RG_BF16, RG_F16)
      default:
        if (has_head) process_chunk<RG_BF16, RG_BF16, MODE, NT, T, true>(sp, dp, len, scale, coef, raw_copy, acc);
        else process_chunk<RG_BF16, RG_BF16, MODE, NT, T, false>(sp, dp, len, scale, coef, raw_copy, acc);
        break;
    }
#undef RG_PAIR
  }

  if (MODE & kModeReduce) {
    // Fixed-order combine.  A non-finite input makes its square, and so the sum, non-finite; a finite sum
    // therefore proves every input was finite.  Only when a sum is not finite are the elements looked at again
    // one by one (the sum can also overflow from finite inputs).
    constexpr int kWaves = T / 64;
    if constexpr (kWavePartials) {
      // Each wavefront reduces its own lanes; a wavefront whose sum is not finite looks at every element of the
      // tile again (its own elements are strided through it), 64 at a time.  Sum and flag of the tile leave in
      // one 16-byte store.
      auto rescan = [&]() -> int {
        int mine = 0;
        if (sp != nullptr) {
          const int lane = threadIdx.x & 63;
          const int es = src_kind == RG_F32 ? 4 : 2;
          for (int i = lane; i < len; i += 64) {
            const char* q = sp + (size_t)i * es;
            mine |= (src_kind == RG_F32 ? nonfinite_at<RG_F32>(q) : src_kind == RG_F16 ? nonfinite_at<RG_F16>(q)
                                                                                        : nonfinite_at<RG_BF16>(q)) ? 1 : 0;
          }
        }
        return __any(mine) ? 1 : 0;
      };
      double s = (((double)acc[0] + (double)acc[1]) + ((double)acc[2] + (double)acc[3])) +
                 (((double)acc[4] + (double)acc[5]) + ((double)acc[6] + (double)acc[7]));
      s = wave_total(s);
      const int bad = !(fabs(s) <= 1.79769313486231570e308) ? rescan() : 0;
      // the wavefronts of the tile meet in LDS: one record per tile, added in wavefront order
      __shared__ double wave_sum[kWaves];
      __shared__ int wave_bad[kWaves];
      if ((threadIdx.x & 63) == 0) {
        wave_sum[threadIdx.x >> 6] = s;
        wave_bad[threadIdx.x >> 6] = bad;
      }
      __syncthreads();
      if (threadIdx.x == 0) {
        double total = wave_sum[0];
        int any = wave_bad[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) {
          total += wave_sum[w];
          any |= wave_bad[w];
        }
        a.partials[slot_id] = Partial{total, any, 0};
      }
    } else {
      // One partial per block: the 8 sums of the thread, the 64 lanes of the wavefront by DPP row scans, the
      // wavefronts through LDS in index order.  Everything past the per-thread fp32 sums is double.
      double s = (((double)acc[0] + (double)acc[1]) + ((double)acc[2] + (double)acc[3])) +
                 (((double)acc[4] + (double)acc[5]) + ((double)acc[6] + (double)acc[7]));
      s = wave_total(s);
      __shared__ double wave_sum[kWaves];
      if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = s;
      __syncthreads();
      double total = wave_sum[0];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) total += wave_sum[w];
      int bad = 0;
      if (!(fabs(total) <= 1.79769313486231570e308)) {
        int mine = 0;
        if (sp != nullptr) {
          if (src_kind == RG_F32) mine = rescan_nonfinite<RG_F32, T>(sp, len);
          else if (src_kind == RG_F16) mine = rescan_nonfinite<RG_F16, T>(sp, len);
          else mine = rescan_nonfinite<RG_BF16, T>(sp, len);
        }
        bad = __syncthreads_or(mine);
      }
      if (threadIdx.x == 0) a.partials[slot_id] = Partial{total, bad, 0};
    }
  }
}

template <int MODE, bool NT, bool PEEL>
__global__ __launch_bounds__(PassThreads<MODE>::value) void pass_kernel(PassArgs a) {
  // Block -> (chunk, tile of the chunk); its partial sum, if any, goes to the slot of that index.
  unsigned bid = blockIdx.x;
  if (a.xcd_run != 0) {
    // Workgroups go to the 8 XCDs round-robin.  xcd_run < 0: each XCD gets one contiguous
    // eighth of the blocks; xcd_run = R > 0: each XCD gets runs of R consecutive blocks.
    const unsigned nb = gridDim.x, x = bid & 7u, q = bid >> 3;
    if (a.xcd_run < 0) {
      bid = x * (nb >> 3) + (x < (nb & 7u) ? x : (nb & 7u)) + q;
    } else {
      const unsigned R = (unsigned)a.xcd_run, group = 8u * R;
      const unsigned g = bid / group;
      if ((g + 1) * group <= nb) bid = g * group + x * R + (q % R);   // the ragged last group keeps its order
    }
  }
  float coef = 1.0f;
  if (a.result != nullptr) {
    // Values produced by the finalize kernel earlier on the same stream.
    if (a.only_if_clipped != 0) {
      if (a.result->clipped == 0) return;
    } else if (a.result->skipped != 0 && a.write_on_overflow == 0) {
      return;
    }
    coef = a.result->coef;
  }

  pass_block<MODE, NT, PEEL>(a, bid, coef);
}

// A write pass that is expected to find nothing to do (an in-place multiply that only runs when the step
// clipped): each block takes `chunks_per_block` consecutive chunks, so that the launch has few blocks to
// retire when the decision says "not clipped".  When it does run it is slower than the tiled pass.
template <bool NT, bool PEEL>
__global__ __launch_bounds__(PassThreads<kModeWrite>::value) void gated_pass_kernel(PassArgs a) {
  if (a.result->clipped == 0) return;
  const float coef = a.result->coef;
  const int64_t first = (int64_t)blockIdx.x * a.chunks_per_block;
  int64_t last = first + a.chunks_per_block;
  if (last > a.n_chunks) last = a.n_chunks;
  for (int64_t c = first; c < last; ++c) pass_block<kModeWrite, NT, PEEL>(a, (unsigned)c, coef);
}

// Fixed-order sum of one value per thread over a block of W wavefronts: DPP row scans inside each
// wavefront, then the wavefront totals through LDS in index order.  Every thread returns the total.
template <int W>
__device__ __forceinline__ void block_sum_or(double& s, int& bad, double* lds_sum, int* lds_bad) {
  s = wave_total(s);
  bad = __any(bad) ? 1 : 0;
  if ((threadIdx.x & 63) == 0) {
    lds_sum[threadIdx.x >> 6] = s;
    lds_bad[threadIdx.x >> 6] = bad;
  }
  __syncthreads();
  double total = 0.0;
  int any = 0;
#pragma unroll
  for (int w = 0; w < W; w += 4) {
    total += (lds_sum[w] + lds_sum[w + 1]) + (lds_sum[w + 2] + lds_sum[w + 3]);
    any |= lds_bad[w] | lds_bad[w + 1] | lds_bad[w + 2] | lds_bad[w + 3];
  }
  s = total;
  bad = any;
  __syncthreads();
}

// Chunks [c0, c1) of segment `seg`.
__device__ __forceinline__ void segment_chunks(const ReduceArgs& a, int seg, int64_t& c0, int64_t& c1) {
  if (a.seg_chunk_begin != nullptr) {
    c0 = a.seg_chunk_begin[seg];
    c1 = a.seg_chunk_begin[seg + 1];
  } else {
    c0 = (int64_t)seg * a.single_seg_chunks;
    c1 = c0 + a.single_seg_chunks;
    if (c1 > a.single_chunks) c1 = a.single_chunks;
  }
}

// Stage 1: block b adds the partials of segment b (thread-strided with eight independent loads in
// flight, then a fixed tree).
template <int THREADS>
__global__ __launch_bounds__(THREADS) void reduce_segments_kernel(ReduceArgs a) {
  __shared__ double lds_sum[THREADS / 64];
  __shared__ int lds_bad[THREADS / 64];
  int64_t c0, c1;
  segment_chunks(a, (int)blockIdx.x, c0, c1);
  const int64_t end = c1 * a.partials_per_chunk;
  int64_t i = c0 * a.partials_per_chunk + threadIdx.x;
  double s[8] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
  int bad = 0;
  for (; i < end; i += 8 * THREADS) {
    Partial w[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int64_t j = i + (int64_t)k * THREADS;
      w[k] = a.partials[j < end ? j : end - 1];
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (i + (int64_t)k * THREADS < end) {
        s[k] += w[k].sumsq;
        bad |= w[k].bad;
      }
    }
  }
  double total = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
  block_sum_or<THREADS / 64>(total, bad, lds_sum, lds_bad);
  if (threadIdx.x == 0) a.seg_sums[blockIdx.x] = Partial{total, bad, 0};
}

// Stage 2, one block: thread t adds the segment sums of tensor t in order (eight loads in flight) and rounds
// to n_t = float(sqrt(sum)), the reference's rounding point; then double(n_t)^2 is added over all tensors in a
// fixed order and the clip decision derived.  `seg` is the segment sums, in device memory or in LDS.
template <typename SegPtr>
__device__ __forceinline__ void decide_body(const ReduceArgs& a, SegPtr seg, double* lds_sum, int* lds_bad) {
  double sq = 0.0;
  int bad = 0;
  for (int t = threadIdx.x; t < a.n_tensors; t += kDecideThreads) {
    const int b = a.tensor_seg_begin ? a.tensor_seg_begin[t] : 0;
    const int e = a.tensor_seg_begin ? a.tensor_seg_begin[t + 1] : a.n_segments;
    double sum = 0.0;
    for (int i = b; i < e; i += 8) {
      Partial w[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) w[k] = seg[i + k < e ? i + k : e - 1];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (i + k < e) {
          sum += w[k].sumsq;
          bad |= w[k].bad;
        }
      }
    }
    const float n = (float)sqrt(sum);
    a.tensor_norm[t] = n;
    sq += (double)n * (double)n;
  }
  block_sum_or<kDecideThreads / 64>(sq, bad, lds_sum, lds_bad);
  if (threadIdx.x == 0) {
    const int overflow = bad != 0 ? 1 : 0;
    const double norm = sqrt(sq);
    const double g = norm + 1e-6;
    const bool gate = overflow != 0 && a.ignore_overflow == 0;
    const bool clip = a.max_norm > 0.0f && !gate && (g > (double)a.max_norm);
    const float coef = clip ? (float)((double)a.max_norm / g) : 1.0f;
    a.result->norm = norm;
    a.result->coef = coef;
    a.result->overflow = overflow;
    a.result->clipped = clip ? 1 : 0;
    a.result->skipped = gate ? 1 : 0;
    if (a.result_copy != nullptr) {
      a.result_copy->norm = norm;
      a.result_copy->coef = coef;
      a.result_copy->overflow = overflow;
      a.result_copy->clipped = clip ? 1 : 0;
      a.result_copy->skipped = gate ? 1 : 0;
    }
  }
}

__global__ __launch_bounds__(kDecideThreads) void decide_kernel(ReduceArgs a) {
  __shared__ double lds_sum[kDecideThreads / 64];
  __shared__ int lds_bad[kDecideThreads / 64];
  decide_body(a, a.seg_sums, lds_sum, lds_bad);
}

// Both stages in one block, for plans with few segments and partials: wavefront w adds segments
// w, w + 16, ... (lane-strided, four loads in flight), the sums meet in LDS, and the block goes on
// as decide_kernel does.  The segment sums are stored as well, for a later launch_decide.
__global__ __launch_bounds__(kDecideThreads) void reduce_small_kernel(ReduceArgs a) {
  __shared__ double lds_sum[kDecideThreads / 64];
  __shared__ int lds_bad[kDecideThreads / 64];
  __shared__ Partial seg_lds[kSmallReduceSegments];
  const int lane = threadIdx.x & 63;
  for (int seg = threadIdx.x >> 6; seg < a.n_segments; seg += kDecideThreads / 64) {
    int64_t c0, c1;
    segment_chunks(a, seg, c0, c1);
    const int64_t end = c1 * a.partials_per_chunk;
    int64_t i = c0 * a.partials_per_chunk + lane;
    double s4[4] = {0.0, 0.0, 0.0, 0.0};
    int bad = 0;
    for (; i < end; i += 256) {
      Partial w[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) w[k] = a.partials[i + 64 * k < end ? i + 64 * k : end - 1];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (i + 64 * k < end) {
          s4[k] += w[k].sumsq;
          bad |= w[k].bad;
        }
      }
    }
    const double s = wave_total((s4[0] + s4[1]) + (s4[2] + s4[3]));
    bad = __any(bad) ? 1 : 0;
    if (lane == 0) {
      seg_lds[seg] = Partial{s, bad, 0};
      a.seg_sums[seg] = Partial{s, bad, 0};
    }
  }
  __syncthreads();
  decide_body(a, &seg_lds[0], lds_sum, lds_bad);
}

// Flat zero fill in rg_zero's shape: 128-thread blocks over 4 KiB tiles laid out from the first 128-byte boundary
// (two 16-byte stores per lane), each XCD filling runs of kZeroXcdRun consecutive tiles; the bytes before that
// boundary and behind the last whole 16 are written one at a time by block 0.  (A grid-stride loop over the same
// bytes ran at 63-65 % of peak where this runs at 90 % and more.)
//
// Pacing.  A wavefront of this kernel has nothing to wait for - it issues its two stores and ends - so the compute
// units hand stores to the memory system as fast as wavefronts can be launched, faster than HBM retires them, and
// the fill then runs at 85-88 % of peak.  Holding every wavefront for `delay_ticks` of the constant-rate wall clock
// before its stores makes the 32 wavefront slots of a compute unit a rate limiter (64 KiB per wavefront lifetime);
// measured on MI355X over 1-4 GiB, by delay: none 85-88 %, 1.25 us 89 %, 1.4-1.5 us 95-97 %, 1.55 us 94 %, 1.7 us
// 88 %, and falling in proportion from there (the limiter then sits below what HBM takes).  The wall clock, not
// s_sleep's shader cycles, measures the delay so that the rate does not move with the shader clock.  Passes that
// load before they store are paced by their loads and only lose from such a delay.
constexpr int kFillTileVecs = 4096 / 16;
template <bool NT>
__global__ __launch_bounds__(kWriteThreads) void fill_zero_kernel(char* p, int64_t nbytes, int64_t head, int delay_ticks) {
  unsigned bid = blockIdx.x;
  {
    const unsigned nb = gridDim.x, x = bid & 7u, q = bid >> 3;
    const unsigned R = (unsigned)kZeroXcdRun, group = 8u * R;
    const unsigned g = bid / group;
    if ((g + 1) * group <= nb) bid = g * group + x * R + (q % R);   // the ragged last group keeps its order
  }
  if (delay_ticks > 0) {
    const uint64_t t_end = wall_clock64() + (uint64_t)delay_ticks;
    while (wall_clock64() < t_end) __builtin_amdgcn_s_sleep(1);
  }
  const int64_t nvec = (nbytes - head) / 16;
  const int64_t tail0 = head + nvec * 16;
  const u32x4 z = {0u, 0u, 0u, 0u};
  const int64_t v0 = (int64_t)bid * kFillTileVecs + threadIdx.x;
#pragma unroll
  for (int u = 0; u < kFillTileVecs / kWriteThreads; ++u) {
    const int64_t v = v0 + u * kWriteThreads;
    if (v < nvec) st16<NT>(p + head + v * 16, z);
  }
  if (bid == 0) {
    const int64_t nscalar = head + (nbytes - tail0);   // < 128 + 16
    for (int64_t k = threadIdx.x; k < nscalar; k += kWriteThreads) store_u8(p + (k < head ? k : tail0 + (k - head)), 0u);
  }
}

template <int MODE>
void launch_mode(const PassArgs& a, bool streaming, hipStream_t stream) {
  const dim3 grid((unsigned)(a.n_chunks * a.tiles_per_chunk)), block(PassThreads<MODE>::value);
  const bool peel = (MODE & kModeWrite) == 0 || a.peel_heads != 0;
  // Unused dynamic LDS caps the blocks resident per compute unit (160 KiB each).  Measured on MI355X: the
  // streaming read-only pass is fastest with 4-5 blocks of 256 threads per unit instead of the 8 that fit
  // (7.1 -> 7.4 TB/s on 2.5e9 fp16 elements); every writing pass wants all the blocks it can get.
  unsigned lds = (MODE == kModeReduce && streaming) ? kReducePassLdsBytes : 0u;
  if ((MODE & kModeAccumulate) != 0 && streaming && a.dynamic_lds != 0) lds = a.dynamic_lds;
#ifdef RG_TUNING_ENV   // experiment builds only
  if (const char* env = getenv((MODE & kModeWrite) ? "RG_LDS_WRITE" : "RG_LDS_REDUCE")) lds = (unsigned)atoi(env);
#endif
  if (streaming) {
    if (peel) hipLaunchKernelGGL((pass_kernel<MODE, true, true>), grid, block, lds, stream, a);
    else hipLaunchKernelGGL((pass_kernel<MODE, true, false>), grid, block, lds, stream, a);
  } else {
    if (peel) hipLaunchKernelGGL((pass_kernel<MODE, false, true>), grid, block, lds, stream, a);
    else hipLaunchKernelGGL((pass_kernel<MODE, false, false>), grid, block, lds, stream, a);
  }
}

}  // namespace

hipError_t launch_pass(int mode, const PassArgs& a, bool streaming, hipStream_t stream) {
  if (a.n_chunks <= 0) return hipSuccess;
  switch (mode) {
    case kModeReduce: launch_mode<kModeReduce>(a, streaming, stream); break;
    case kModeWrite: launch_mode<kModeWrite>(a, streaming, stream); break;
    case kModeReduce | kModeWrite: launch_mode<kModeReduce | kModeWrite>(a, streaming, stream); break;
    case kModeWrite | kModeAccumulate: launch_mode<kModeWrite | kModeAccumulate>(a, streaming, stream); break;
    case kModeReduce | kModeWrite | kModeAccumulate:
      launch_mode<kModeReduce | kModeWrite | kModeAccumulate>(a, streaming, stream);
      break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_gated_pass(const PassArgs& a, bool streaming, hipStream_t stream) {
  if (a.n_chunks <= 0) return hipSuccess;
  if (a.result == nullptr || a.chunks_per_block < 1 || a.tiles_per_chunk != 1) return hipErrorInvalidValue;
  const dim3 grid((unsigned)((a.n_chunks + a.chunks_per_block - 1) / a.chunks_per_block)), block(PassThreads<kModeWrite>::value);
  const bool peel = a.peel_heads != 0;
  if (streaming) {
    if (peel) hipLaunchKernelGGL((gated_pass_kernel<true, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((gated_pass_kernel<true, false>), grid, block, 0, stream, a);
  } else {
    if (peel) hipLaunchKernelGGL((gated_pass_kernel<false, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((gated_pass_kernel<false, false>), grid, block, 0, stream, a);
  }
  return hipGetLastError();
}

hipError_t launch_reduce(const ReduceArgs& a, int64_t n_chunks, hipStream_t stream) {
  if (a.n_segments <= kSmallReduceSegments && n_chunks * a.partials_per_chunk <= kSmallReducePartials) {
    hipLaunchKernelGGL(reduce_small_kernel, dim3(1), dim3(kDecideThreads), 0, stream, a);
    return hipGetLastError();
  }
  hipLaunchKernelGGL(reduce_segments_kernel<256>, dim3((unsigned)a.n_segments), dim3(256), 0, stream, a);
  hipLaunchKernelGGL(decide_kernel, dim3(1), dim3(kDecideThreads), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_decide(const ReduceArgs& a, hipStream_t stream) {
  hipLaunchKernelGGL(decide_kernel, dim3(1), dim3(kDecideThreads), 0, stream, a);
  return hipGetLastError();
}

// kFillDelayNs in ticks of the current device's wall clock (0 when its rate cannot be read: the fill then runs unpaced).
#ifndef RG_FILL_DELAY_NS
#define RG_FILL_DELAY_NS 1450
#endif
constexpr int kFillDelayNs = RG_FILL_DELAY_NS;
constexpr int kMaxDevices = 64;
int fill_delay_ticks(int ns) {
  const int t = fill_delay_ticks();
  return t > 0 ? (int)(((int64_t)t * ns + kFillDelayNs / 2) / kFillDelayNs) : 0;
}

int fill_delay_ticks() {
  static std::atomic<int> cached[kMaxDevices];   // 0: not asked yet; -1: unknown rate
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  int t = cached[dev].load(std::memory_order_relaxed);
  if (t == 0) {
    int khz = 0;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || khz <= 0) {
      (void)hipGetLastError();
      t = -1;
    } else {
      t = (int)(((int64_t)khz * kFillDelayNs + 500000) / 1000000);
      if (t < 1) t = -1;
    }
    cached[dev].store(t, std::memory_order_relaxed);
  }
  return t > 0 ? t : 0;
}

hipError_t launch_fill_zero(void* dst, int64_t nbytes, hipStream_t stream) {
  if (nbytes <= 0) return hipSuccess;
  char* p = reinterpret_cast<char*>(dst);
  int64_t head = (int64_t)((kWriteAlignBytes - (unsigned)(reinterpret_cast<uintptr_t>(p) & (kWriteAlignBytes - 1))) & (kWriteAlignBytes - 1));
  if (head > nbytes) head = nbytes;
  const int64_t nvec = (nbytes - head) / 16;
  int64_t blocks = (nvec + kFillTileVecs - 1) / kFillTileVecs;
  if (blocks < 1) blocks = 1;   // block 0 writes the bytes outside the vectors
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  // Paced only where the stores go through to HBM: up to the 256 MiB of the memory-side cache the unpaced fill
  // is the faster one (192 MiB: 98 % of HBM's peak rate unpaced, 90 % paced), and a small fill would just start late.
  const bool streaming = nbytes > ((int64_t)256 << 20);
  const int delay = streaming ? fill_delay_ticks() : 0;
  if (streaming) hipLaunchKernelGGL(fill_zero_kernel<true>, dim3((unsigned)blocks), dim3(kWriteThreads), 0, stream, p, nbytes, head, delay);
  else hipLaunchKernelGGL(fill_zero_kernel<false>, dim3((unsigned)blocks), dim3(kWriteThreads), 0, stream, p, nbytes, head, delay);
  return hipGetLastError();
}

}  // namespace rg
