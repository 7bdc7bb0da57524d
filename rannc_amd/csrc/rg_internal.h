// Internal declarations shared by the kernel and host translation units of libranncgrad.
#ifndef RG_INTERNAL_H
#define RG_INTERNAL_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ranncgrad.h"

#define RG_API extern "C" __attribute__((visibility("default")))

namespace rg {

// One row of the device-side descriptor table (32 bytes).
struct TensorDesc {
  const void* src;
  void* dst;
  int64_t numel;
  int32_t src_dtype;
  int32_t dst_dtype;
};
static_assert(sizeof(TensorDesc) == 32, "descriptor row must stay 32 bytes");

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

constexpr int kBlockThreads = 256;   // 4 wavefronts of 64
constexpr int kVecElems = 8;         // elements one thread handles per vector step
constexpr int kUnroll = 4;           // vector steps in flight per thread
constexpr int64_t kChunkQuantum = (int64_t)kBlockThreads * kVecElems;  // 2048 elements

// Pass selection for the chunk kernel.
enum : int { kModeReduce = 1, kModeWrite = 2 };

struct PassArgs {
  const TensorDesc* tensors;
  const int32_t* chunk_tensor;   // [n_chunks] row of the descriptor table
  const int32_t* chunk_index;    // [n_chunks] which chunk of that tensor
  double* chunk_sumsq;           // [n_chunks] written when reducing
  int32_t* chunk_bad;            // [n_chunks] written when reducing
  const StepResult* result;      // non-null: take coef / overflow gate from the device
  int64_t chunk_elems;
  int64_t n_chunks;
  float scale;
  int32_t write_on_overflow;
  int32_t reverse;               // visit chunks last to first
  int32_t zero_fill;             // write pass: ignore the sources, store zeros
  int32_t norm_of_source;        // reduce pass: measure the source as stored (no rounding to dst)
};

struct FinalizeArgs {
  const int64_t* tensor_chunk_begin;  // [n_tensors + 1]
  const double* chunk_sumsq;
  const int32_t* chunk_bad;
  float* tensor_norm;                 // [n_tensors]
  double* tensor_sq;                  // [n_tensors]
  int32_t* tensor_bad;                // [n_tensors]
  unsigned int* ticket;
  StepResult* result;
  int32_t n_tensors;
  float max_norm;
  int32_t ignore_overflow;  // overflow is reported but neither gates the clip nor the write
};

hipError_t launch_pass(int mode, const PassArgs& a, hipStream_t stream);
hipError_t launch_finalize(const FinalizeArgs& a, hipStream_t stream);
hipError_t launch_fill_zero(void* dst, int64_t nbytes, hipStream_t stream);

void set_error(const char* fmt, ...);

}  // namespace rg
#endif
