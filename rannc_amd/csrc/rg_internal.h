// Internal declarations shared by the kernel and host translation units of libranncgrad.
#ifndef RG_INTERNAL_H
#define RG_INTERNAL_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ranncgrad.h"

#define RG_API extern "C" __attribute__((visibility("default")))

namespace rg {

// One tensor pair as the caller described it (host side only).
struct TensorDesc {
  const void* src;
  void* dst;
  int64_t numel;
  int32_t src_dtype;
  int32_t dst_dtype;
};

// One row of the device-side work table: a contiguous run of one tensor (32 bytes, so a
// block fetches its whole work description with a single 32-byte load).
struct ChunkRec {
  const void* src;  // first source element of the chunk; null = the tensor has no gradient
  void* dst;        // first destination element of the chunk
  int32_t len;      // elements in the chunk
  int32_t tensor;   // row of the tensor in the plan
  int16_t src_dtype;
  int16_t dst_dtype;
  int32_t pad;
};
static_assert(sizeof(ChunkRec) == 32, "chunk record must stay 32 bytes");

// Device mirror of rg_step_result, padded to 32 bytes.
struct StepResult {
  double norm;
  float coef;
  int32_t overflow;
  int32_t clipped;
  int32_t skipped;
  int64_t pad;
};
static_assert(sizeof(StepResult) == 32, "result block must stay 32 bytes");

// Tunables (overridable at build time for experiments).
#ifndef RG_REDUCE_ELEMS_PER_THREAD
#define RG_REDUCE_ELEMS_PER_THREAD 32
#endif
#ifndef RG_WRITE_ELEMS_PER_THREAD
#define RG_WRITE_ELEMS_PER_THREAD 4
#endif
#ifndef RG_WRITE_THREADS
#define RG_WRITE_THREADS 128
#endif
#ifndef RG_WRITE_TILE_ELEMS
#define RG_WRITE_TILE_ELEMS 1024
#endif
#ifndef RG_ALIGN_BYTES
#define RG_ALIGN_BYTES 128
#endif
#ifndef RG_WRITE_ALIGN_BYTES
#define RG_WRITE_ALIGN_BYTES 128
#endif
#ifndef RG_DEFAULT_CHUNK_ELEMS
#define RG_DEFAULT_CHUNK_ELEMS 16384
#endif
constexpr int kBlockThreads = 256;                               // 4 wavefronts of 64
// Elements a thread has in flight per loop iteration.  Measured on MI355X: a read-only pass
// is fastest with deep unrolling over 8-16K-element chunks, a pass that also writes with
// shallow unrolling over small tiles.
constexpr int kReduceElemsPerThread = RG_REDUCE_ELEMS_PER_THREAD;   // of fp32; twice as many 16-bit elements (same bytes in flight)
constexpr int kWriteElemsPerThread = RG_WRITE_ELEMS_PER_THREAD;
constexpr int kWriteThreads = RG_WRITE_THREADS;                  // block size of write-only passes
constexpr int kWriteTileElems = RG_WRITE_TILE_ELEMS;             // writing passes cut each chunk into tiles of this size
// Alignment.  Measured on MI355X, a pass whose 128-bit stores are not 64-byte aligned loses
// 9 % (partial-line writes), one whose loads are not 128-byte aligned 3-6 %.  So the side a
// pass writes decides: chunk boundaries inside a tensor are placed on 128-byte boundaries of
// its destination (of its source when there is none), which leaves one unaligned head per
// tensor - not per chunk - to be peeled with scalar accesses; the loads absorb whatever
// relative misalignment remains.  Read-only passes peel their source per chunk.
// RG_WRITE_ALIGN_BYTES <= 4 switches the destination peel off (element-aligned vector stores).
constexpr unsigned kAlignBytes = RG_ALIGN_BYTES;
constexpr unsigned kWriteAlignBytes = RG_WRITE_ALIGN_BYTES;

// Elements from `addr` to the next `align`-byte boundary (align: power of two; 0 when
// alignment handling is off).
__host__ __device__ inline int head_elems(uintptr_t addr, unsigned align, unsigned elem_bytes) {
  if (align <= 4) return 0;
  return (int)(((align - (unsigned)(addr & (align - 1))) & (align - 1)) / elem_bytes);
}
constexpr int64_t kChunkQuantum = 2048;    // chunk sizes are multiples of this many elements
constexpr int64_t kMaxChunkElems = 1 << 20;
constexpr unsigned kReducePassLdsBytes = 32768;   // dynamic LDS of the streaming read-only pass: 5 resident blocks per compute unit
// rg_accumulate's pass reads more than it writes (source and old destination in, destination out) and, like the
// read-only pass, runs faster with fewer blocks resident per compute unit (measured on MI355X, streaming sizes):
// with 16 bytes loaded from each side per lane and step (both sides equally wide) ten blocks of 128 threads instead
// of sixteen gain 2-5 %, with 8 + 16 bytes (a 16-bit side and an fp32 side) twelve blocks gain 3-4 %; BERT-large's
// bf16 gradients into fp32: 79.6 -> 83.8 % of peak, the ResNet's fp32 into fp32: 79.3 -> 81.7 %.  The pass that also
// sums (rg_unscale_accumulate) holds twelve blocks by its register count already (ten gain on flat same-width data
// but lose on the ResNet's many small tensors); plain writing passes lose from the first block taken away.
constexpr int kZeroXcdRun = 64;                      // rg_zero: tiles of a run one XCD fills (see rg_zero)
constexpr int kZeroDelayNs = 100;                    // rg_zero through the table, large plans: wall-clock hold before a tile's stores
constexpr int64_t kZeroDelayMinBytes = (int64_t)1536 << 20;
constexpr unsigned kAccSameWidthLdsBytes = 16384;   // 10 resident blocks
constexpr unsigned kAccMixedWidthLdsBytes = 13600;  // 12 resident blocks
constexpr int64_t kMinWriteTileElems = 256;    // bounds the per-tile partial storage of a plan

// Pass selection for the chunk kernel.
enum : int { kModeReduce = 1, kModeWrite = 2, kModeAccumulate = 4 };  // accumulate: dst = round(dst + x * scale)

// A partial sum of squares with the inf/NaN flag of the elements it covers: what a block of the read-only pass
// and every wavefront of a pass that sums while it writes leave behind, in one 16-byte store.
struct alignas(16) Partial {
  double sumsq;
  int32_t bad;
  int32_t pad;
};
constexpr int kWaveSlotsPerTile = 1;   // partials one tile of a pass that sums while it writes leaves (its wavefronts meet in LDS)

// From partials to the decision in two launches.  The partials of a tensor are cut into segments of whole chunks
// (kSegmentChunks each; more for a tensor that would otherwise have over kMaxSegmentsPerTensor of them): one block
// per segment adds its partials in a fixed order, then a single block adds each tensor's segment sums (one thread
// per tensor), rounds to n_t = float(sqrt(sum)), adds double(n_t)^2 over the tensors and takes the clip decision.
// Plans with few segments and partials run both stages in that single block: one launch.
constexpr int64_t kSegmentChunks = 64;
constexpr int kMaxSegmentsPerTensor = 64;
constexpr int kDecideThreads = 1024;
constexpr int kSmallReduceSegments = 64;        // the one-launch form: at most this many segments ...
constexpr int64_t kSmallReducePartials = 16384; // ... and this many partials

struct PassArgs {
  const ChunkRec* chunks;        // [n_chunks]; null = one tensor described by `single`
  ChunkRec single;               // whole-tensor pointers and types (len unused)
  int64_t single_numel;
  int64_t single_chunk_elems;
  int64_t single_head;           // elements before the first aligned chunk boundary
  int32_t xcd_run;               // block -> XCD mapping, see pass_kernel
  int32_t peel_heads;            // writing passes: some destination starts off a boundary
  Partial* partials;             // read-only pass: [n_chunks]; pass that sums while it writes: one per tile
  const StepResult* result;      // non-null: take coef / overflow gate from the device
  int64_t n_chunks;
  int32_t tile_elems;            // elements one block handles (== chunk_elems unless the pass splits chunks)
  int32_t tiles_per_chunk;       // blocks per chunk record
  float scale;
  const float* scale_dev;        // non-null: the kernels read the scale from device memory instead of `scale`
  int32_t write_on_overflow;
  int32_t zero_fill;             // write pass: ignore the sources, store zeros
  int32_t zero_delay_ticks;      // ... after holding each wavefront for this many ticks of the wall clock (0: none)
  int32_t norm_of_source;        // reduce pass: measure the source as stored (no rounding to dst)
  int32_t only_if_clipped;       // with `result`: the whole launch does nothing unless result->clipped is set
  int32_t src_is_dst;            // read the destination instead of the record's source (in-place rescale)
  int32_t chunks_per_block;      // launch_gated_pass only: consecutive chunks one block walks through
  uint32_t dynamic_lds;          // host side only: unused dynamic LDS that caps the resident blocks (0: the mode's default)
};

struct ReduceArgs {
  const Partial* partials;            // chunk-major: chunk c owns [c * partials_per_chunk, (c + 1) * partials_per_chunk)
  const int64_t* seg_chunk_begin;     // [n_segments + 1]; null = one tensor cut into segments of single_seg_chunks chunks
  const int32_t* tensor_seg_begin;    // [n_tensors + 1]; null = one tensor that owns every segment
  int64_t single_chunks;
  int64_t single_seg_chunks;
  Partial* seg_sums;                  // [n_segments]
  float* tensor_norm;                 // [n_tensors]
  StepResult* result;
  rg_step_result* result_copy;        // optional second place the decision is written to (caller's memory)
  int32_t n_tensors;
  int32_t n_segments;
  int32_t partials_per_chunk;         // 1 after the read-only pass, else tiles per chunk (* kWaveSlotsPerTile)
  float max_norm;
  int32_t ignore_overflow;            // overflow is reported but neither gates the clip nor the write
};

// streaming: nontemporal loads/stores (data far larger than the caches).
hipError_t launch_pass(int mode, const PassArgs& a, bool streaming, hipStream_t stream);
// A whole-chunk write pass that runs only if result->clipped is set, launched with few blocks.
hipError_t launch_gated_pass(const PassArgs& a, bool streaming, hipStream_t stream);
// partials -> segment sums -> per-tensor norms -> decision (n_chunks: chunks the partials cover)
hipError_t launch_reduce(const ReduceArgs& a, int64_t n_chunks, hipStream_t stream);
// segment sums (left by an earlier launch_reduce) -> per-tensor norms -> decision for a.max_norm
hipError_t launch_decide(const ReduceArgs& a, hipStream_t stream);
hipError_t launch_fill_zero(void* dst, int64_t nbytes, hipStream_t stream);
// Ticks of the current device's wall clock that a wavefront of a large flat fill waits before it stores (0: unknown rate).
int fill_delay_ticks();
int fill_delay_ticks(int ns);   // the same clock, another delay

void set_error(const char* fmt, ...);

}  // namespace rg
#endif
