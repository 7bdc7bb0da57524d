#include <cstdlib>
// Multi-tensor optimizer step (Adam / AdamW / SGD) with the fp32 -> fp16/bf16 model copy
// folded in.  Same launch shape as the writing passes of the gradient path: a device-
// resident table of chunk records, blocks of 128 threads over 1024-element tiles, four
// elements per lane per instruction, every access contiguous across the wavefront.
// Purely HBM-bound: Adam moves 16 bytes in and 12 (+2) out per element.
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <new>
#include <vector>

#include "rg_device.h"
#include "rg_host.h"
#include "rg_internal.h"

namespace rg {
namespace {

// One row of the optimizer's work table: a contiguous run of one parameter.
struct OptChunkRec {
  void* param;
  const void* grad;
  void* state1;
  void* state2;
  void* copy;
  int32_t len;
  int16_t grad_dtype;
  int16_t copy_dtype;
  int64_t pad[2];
};
static_assert(sizeof(OptChunkRec) == 64, "optimizer chunk record must stay 64 bytes");

enum : int { kAdam = 0, kSgd = 1 };

// Scalar factors, rounded once from double on the host.
struct OptConst {
  float grad_scale;
  float weight_decay;      // L2 form: g += wd * p (0 = off)
  float param_mul;         // decoupled form: p *= 1 - lr * wd (1 = off)
  float lerp_coeff;        // Adam: (1 - beta1) when that is < 0.5, else (1 - beta1) - 1
  float beta2, one_minus_beta2, neg_step_size, bias2_sqrt, eps;
  float neg_lr, momentum, one_minus_dampening;   // SGD
  int32_t lerp_from_end;   // Adam: weight >= 0.5, interpolate back from the gradient
  int32_t maximize, nesterov, first_step, has_momentum;
};

struct OptArgs {
  const OptChunkRec* chunks;
  const StepResult* gate;
  const rg_adam_clock* clock;   // Adam only, optional: the step-dependent factors live on the device
  const float* grad_scale_dev;  // optional: the gradient scale lives on the device (a loss scaler's 1 / scale)
  int32_t tile_elems;
  int32_t tiles_per_chunk;
  OptConst c;
};

// Launch shape per algorithm, measured on MI355X over BERT-large's tensors: SGD (3-4 streams)
// is fastest in the shape of the gradient path's writing passes; Adam (8 streams) gains 1-2 %
// from larger blocks over larger tiles with four vectors per array in flight.
template <int ALGO> struct OptShape;
template <> struct OptShape<kAdam> {
#if defined(RG_OPT_THREADS)
  static constexpr int kThreads = RG_OPT_THREADS, kTileElems = RG_OPT_TILE_ELEMS, kUnroll = RG_OPT_UNROLL;
#else
  static constexpr int kThreads = 256, kTileElems = 4096, kUnroll = 4;
#endif
};
template <> struct OptShape<kSgd> {
#if defined(RG_OPT_THREADS)
  static constexpr int kThreads = RG_OPT_THREADS, kTileElems = RG_OPT_TILE_ELEMS, kUnroll = RG_OPT_UNROLL;
#else
  static constexpr int kThreads = 128, kTileElems = 1024, kUnroll = 1;
#endif
};
constexpr int kOptMinTileElems = 1024;   // smallest tile of any shape (bounds the grid size of a table)
constexpr int kOptE = 4;    // elements per lane per instruction
#ifndef RG_OPT_NT_LOAD
#define RG_OPT_NT_LOAD 1
#endif
#ifndef RG_OPT_NT_STORE
#define RG_OPT_NT_STORE 1
#endif

template <int ALGO>
__device__ __forceinline__ void update_one(float& p, float g, float& s1, float& s2, const OptConst& c, float coef) {
  // two multiplies, each rounded: the value a pass that wrote the unscaled, clipped gradient
  // would have stored (x * 1 is x, so neither needs a branch)
  g = g * c.grad_scale;
  g = g * coef;
  if (c.maximize) g = -g;
  if (ALGO == kAdam) {
    p = p * c.param_mul;                                          // x * 1 is x: no branch needed
    if (c.weight_decay != 0.0f) g = __builtin_fmaf(c.weight_decay, p, g);
    // exp_avg.lerp_(g, 1 - beta1), ATen's two-sided form
    s1 = __builtin_fmaf(c.lerp_coeff, g - s1, c.lerp_from_end ? g : s1);
    // exp_avg_sq.mul_(beta2).addcmul_(g, g, value = 1 - beta2)
    s2 = __builtin_fmaf(c.one_minus_beta2 * g, g, s2 * c.beta2);
    const float denom = sqrtf(s2) / c.bias2_sqrt + c.eps;          // correctly rounded sqrt and divisions
    p = p + (c.neg_step_size * s1) / denom;
  } else {
    if (c.weight_decay != 0.0f) g = __builtin_fmaf(c.weight_decay, p, g);
    if (c.has_momentum) {
      s1 = c.first_step ? g : __builtin_fmaf(c.one_minus_dampening, g, s1 * c.momentum);
      g = c.nesterov ? __builtin_fmaf(c.momentum, s1, g) : s1;
    }
    p = __builtin_fmaf(c.neg_lr, g, p);
  }
}

template <int DT> __device__ __forceinline__ float load1(const char* p) { return __uint_as_float(load_u32(p)); }
template <> __device__ __forceinline__ float load1<RG_F16>(const char* p) {
  return f16_to_f32(__builtin_bit_cast(_Float16, (unsigned short)load_u16(p)));
}
template <> __device__ __forceinline__ float load1<RG_BF16>(const char* p) {
  return bf16_bits_to_f32(load_u16(p));
}

// One tile of one chunk.  G: gradient dtype; C: model-copy dtype, or -1 for none.
template <int ALGO, int G, int C, bool NT>
__device__ __forceinline__ void optim_tile(const OptChunkRec& r, int start, int len, const OptConst& c, float coef) {
  constexpr int T = OptShape<ALGO>::kThreads;
  constexpr int E = kOptE;
  constexpr bool NTL = NT && RG_OPT_NT_LOAD, NTS = NT && RG_OPT_NT_STORE;
  constexpr int GS = ElemSize<G>::value;
  constexpr bool kCopy = C >= 0;
  constexpr int CD = kCopy ? C : RG_F32;
  constexpr int CS = ElemSize<CD>::value;
  constexpr bool kS1 = true;                 // presence is decided at run time for SGD
  (void)kS1;
  char* pp = reinterpret_cast<char*>(r.param) + (size_t)start * 4;
  const char* gp = reinterpret_cast<const char*>(r.grad) + (size_t)start * GS;
  char* s1p = r.state1 ? reinterpret_cast<char*>(r.state1) + (size_t)start * 4 : nullptr;
  char* s2p = r.state2 ? reinterpret_cast<char*>(r.state2) + (size_t)start * 4 : nullptr;
  char* cp = kCopy ? reinterpret_cast<char*>(r.copy) + (size_t)start * CS : nullptr;
  const bool use_s1 = ALGO == kAdam || (c.has_momentum != 0 && s1p != nullptr);
  const int tid = threadIdx.x;

  // Unaligned head of the parameter (at most one per tensor: chunk and tile boundaries sit
  // on 128-byte boundaries of the parameter) and ragged tail: one element per thread.
  int head = head_elems(reinterpret_cast<uintptr_t>(pp), kWriteAlignBytes, 4u);
  if (head > len) head = len;
  const int nbody = (len - head) / E * E;
  const int tail0 = head + nbody;
  const int nscalar = head + (len - tail0);
  for (int k = tid; k < nscalar; k += T) {
    const int i = k < head ? k : tail0 + (k - head);
    float p = __uint_as_float(load_u32(pp + (size_t)i * 4));
    const float g = load1<G>(gp + (size_t)i * GS);
    float s1 = use_s1 ? __uint_as_float(load_u32(s1p + (size_t)i * 4)) : 0.0f;
    float s2 = ALGO == kAdam ? __uint_as_float(load_u32(s2p + (size_t)i * 4)) : 0.0f;
    update_one<ALGO>(p, g, s1, s2, c, coef);
    store_u32(pp + (size_t)i * 4, __float_as_uint(p));
    if (use_s1) store_u32(s1p + (size_t)i * 4, __float_as_uint(s1));
    if (ALGO == kAdam) store_u32(s2p + (size_t)i * 4, __float_as_uint(s2));
    if (kCopy) store1<CD>(cp + (size_t)i * CS, p);
  }

  auto vec = [&](int e, Raw<RG_F32, E>& rp, Raw<G, E>& rg, Raw<RG_F32, E>& r1, Raw<RG_F32, E>& r2) {
    rp = Mem<RG_F32, E, NTL>::load(pp + (size_t)e * 4);
    rg = Mem<G, E, NTL>::load(gp + (size_t)e * GS);
    r1 = rp;
    r2 = rp;
    if (use_s1) r1 = Mem<RG_F32, E, NTL>::load(s1p + (size_t)e * 4);
    if (ALGO == kAdam) r2 = Mem<RG_F32, E, NTL>::load(s2p + (size_t)e * 4);
  };
  auto finish = [&](int e, const Raw<RG_F32, E>& rp, const Raw<G, E>& rg, const Raw<RG_F32, E>& r1, const Raw<RG_F32, E>& r2) {
    float p[E], g[E], s1[E], s2[E];
    Codec<RG_F32, E>::unpack(rp, p);
    Codec<G, E>::unpack(rg, g);
    Codec<RG_F32, E>::unpack(r1, s1);
    Codec<RG_F32, E>::unpack(r2, s2);
#pragma unroll
    for (int j = 0; j < E; ++j) update_one<ALGO>(p[j], g[j], s1[j], s2[j], c, coef);
    Mem<RG_F32, E, NTS>::store(pp + (size_t)e * 4, Codec<RG_F32, E>::pack(p));
    if (use_s1) Mem<RG_F32, E, NTS>::store(s1p + (size_t)e * 4, Codec<RG_F32, E>::pack(s1));
    if (ALGO == kAdam) Mem<RG_F32, E, NTS>::store(s2p + (size_t)e * 4, Codec<RG_F32, E>::pack(s2));
    if constexpr (kCopy) Mem<CD, E, NTS>::store(cp + (size_t)e * CS, Codec<CD, E>::pack(p));
  };
  constexpr int U = OptShape<ALGO>::kUnroll;
  constexpr int kIter = T * E * U;
  int base = head;
  for (; base + kIter <= tail0; base += kIter) {     // all loads of U steps in flight together
    Raw<RG_F32, E> rp[U], r1[U], r2[U];
    Raw<G, E> rg[U];
#pragma unroll
    for (int u = 0; u < U; ++u) vec(base + (u * T + tid) * E, rp[u], rg[u], r1[u], r2[u]);
#pragma unroll
    for (int u = 0; u < U; ++u) finish(base + (u * T + tid) * E, rp[u], rg[u], r1[u], r2[u]);
  }
  for (int e = base + tid * E; e < tail0; e += T * E) {
    Raw<RG_F32, E> rp, r1, r2;
    Raw<G, E> rg;
    vec(e, rp, rg, r1, r2);
    finish(e, rp, rg, r1, r2);
  }
}

template <int ALGO, bool NT>
__global__ __launch_bounds__(OptShape<ALGO>::kThreads) void optim_kernel(OptArgs a) {
  float coef = 1.0f;
  if (a.gate != nullptr) {
    if (a.gate->skipped != 0) return;
    coef = a.gate->coef;
  }
  if (a.grad_scale_dev != nullptr) a.c.grad_scale = *a.grad_scale_dev;
  if (ALGO == kAdam && a.clock != nullptr) {
    // written by adam_clock_kernel earlier on the same stream
    a.c.neg_step_size = a.clock->neg_step_size;
    a.c.bias2_sqrt = a.clock->bias2_sqrt;
  }
  const unsigned bid = blockIdx.x;
  const OptChunkRec r = a.chunks[bid / (unsigned)a.tiles_per_chunk];
  const int tile = (int)(bid % (unsigned)a.tiles_per_chunk);
  int chunk_head = head_elems(reinterpret_cast<uintptr_t>(r.param), kWriteAlignBytes, 4u);
  if (chunk_head > r.len) chunk_head = r.len;
  const int start = tile == 0 ? 0 : chunk_head + tile * a.tile_elems;
  int end = tile == a.tiles_per_chunk - 1 ? r.len : chunk_head + (tile + 1) * a.tile_elems;
  if (end > r.len) end = r.len;
  if (start >= end) return;
  const int len = end - start;
  const int copy_kind = r.copy ? r.copy_dtype : -1;
#define RG_OPT(G, C)                                                       \
  if (r.grad_dtype == G && copy_kind == C) {                               \
    optim_tile<ALGO, G, C, NT>(r, start, len, a.c, coef);                \
    return;                                                                \
  }
  RG_OPT(RG_F32, -1)
  RG_OPT(RG_F32, RG_BF16)
  RG_OPT(RG_F32, RG_F16)
  RG_OPT(RG_F32, RG_F32)
  RG_OPT(RG_BF16, -1)
  RG_OPT(RG_BF16, RG_BF16)
  RG_OPT(RG_F16, -1)
  RG_OPT(RG_F16, RG_F16)
  RG_OPT(RG_F16, RG_BF16)
  RG_OPT(RG_BF16, RG_F16)
  RG_OPT(RG_F16, RG_F32)
  RG_OPT(RG_BF16, RG_F32)
#undef RG_OPT
}

// One thread: the next step of a device-resident Adam step count and the two factors that depend on it,
// computed as the host path computes them (in double).  A step the gate says was skipped does not count.
__global__ void adam_clock_kernel(rg_adam_clock* clock, double lr, double beta1, double beta2, const StepResult* gate) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  if (gate != nullptr && gate->skipped != 0) return;
  const int64_t step = clock->step + 1;
  const double bias1 = 1.0 - pow(beta1, (double)step);
  const double bias2 = 1.0 - pow(beta2, (double)step);
  clock->step = step;
  clock->neg_step_size = (float)(-(lr / bias1));
  clock->bias2_sqrt = (float)sqrt(bias2);
  clock->step_f32 = (float)step;
}

// One thread: the loss-scale schedule (see rg_scaler_update in ranncgrad.h).
__global__ void scaler_init_kernel(rg_scaler_state* st, rg_scaler_state v) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  v.inv_scale = (float)(1.0 / (double)v.loss_scale);
  *st = v;
}

__global__ void scaler_update_kernel(rg_scaler_state* st, const StepResult* result, int flags) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  const bool dynamic = (flags & RG_SCALER_DYNAMIC) != 0;
  float scale = st->loss_scale;
  int unskipped = st->unskipped;
  if (result->overflow != 0 && dynamic) {
    scale = scale / 2.0f;
    if (st->min_loss_scale > 0.0f && scale < st->min_loss_scale) scale = st->min_loss_scale;
    if ((flags & RG_SCALER_TRUNCATE) != 0) scale = (float)(int)scale;
    unskipped = 0;
    st->skipped_steps = st->skipped_steps + 1;
  } else {
    unskipped += 1;
  }
  if (unskipped == st->scale_window && dynamic) {
    scale = scale * st->scale_factor;
    if (scale > st->max_loss_scale) scale = st->max_loss_scale;
    unskipped = 0;
  }
  st->loss_scale = scale;
  st->inv_scale = (float)(1.0 / (double)scale);
  st->unskipped = unskipped;
}

}  // namespace
}  // namespace rg

using namespace rg;

struct rg_optim {
  int device = 0;
  int n_tensors = 0;
  int64_t n_chunks = 0;
  int64_t chunk_elems = RG_DEFAULT_CHUNK_ELEMS;
  int64_t total_numel = 0;
  bool has_state1 = false, has_state2 = false, any_copy = false;
  const float* grad_scale_dev = nullptr;   // rg_optim_set_grad_scale_source
  struct Row {
    void* param;
    const void* grad;
    void* state1;
    void* state2;
    void* copy;
    int64_t numel;
    int32_t grad_dtype, copy_dtype;
  };
  std::vector<Row> rows;
  std::vector<int64_t> chunk_begin;
  OptChunkRec* d_chunks = nullptr;
  OptChunkRec* stage[2] = {nullptr, nullptr};   // pinned
  hipEvent_t stage_done[2] = {nullptr, nullptr};
  bool stage_used[2] = {false, false};
  int next_stage = 0;
};

static void fill_opt_records(const rg_optim* o, OptChunkRec* out) {
  for (int i = 0; i < o->n_tensors; ++i) {
    const rg_optim::Row& t = o->rows[(size_t)i];
    const int gs = elem_size(t.grad_dtype), cs = elem_size(t.copy_dtype);
    const int64_t head = head_elems(reinterpret_cast<uintptr_t>(t.param), kWriteAlignBytes, 4u);
    for (int64_t c = o->chunk_begin[(size_t)i]; c < o->chunk_begin[(size_t)i + 1]; ++c) {
      const int64_t j = c - o->chunk_begin[(size_t)i];
      const int64_t start = j == 0 ? 0 : std::min(t.numel, head + j * o->chunk_elems);
      const int64_t end = std::min(t.numel, head + (j + 1) * o->chunk_elems);
      OptChunkRec& r = out[c];
      memset(&r, 0, sizeof(r));
      r.param = static_cast<char*>(t.param) + start * 4;
      r.grad = static_cast<const char*>(t.grad) + start * gs;
      r.state1 = t.state1 ? static_cast<char*>(t.state1) + start * 4 : nullptr;
      r.state2 = t.state2 ? static_cast<char*>(t.state2) + start * 4 : nullptr;
      r.copy = t.copy ? static_cast<char*>(t.copy) + start * cs : nullptr;
      r.len = (int32_t)(end - start);
      r.grad_dtype = (int16_t)t.grad_dtype;
      r.copy_dtype = (int16_t)t.copy_dtype;
    }
  }
}

static int check_rows(const rg_optim* o, const char* op) {
  for (int i = 0; i < o->n_tensors; ++i) {
    const rg_optim::Row& t = o->rows[(size_t)i];
    if (t.numel == 0) continue;
    if (t.param == nullptr || t.grad == nullptr) {
      set_error("%s: tensor %d lacks a parameter or gradient pointer", op, i);
      return RG_EINVAL;
    }
    if ((o->has_state1 && t.state1 == nullptr) || (o->has_state2 && t.state2 == nullptr)) {
      set_error("%s: tensor %d lacks a state pointer", op, i);
      return RG_EINVAL;
    }
    int rc = check_pointer(t.param, 4, "param", i);
    if (rc == RG_OK) rc = check_pointer(t.grad, elem_size(t.grad_dtype), "grad", i);
    if (rc == RG_OK) rc = check_pointer(t.state1, 4, "state1", i);
    if (rc == RG_OK) rc = check_pointer(t.state2, 4, "state2", i);
    if (rc == RG_OK) rc = check_pointer(t.copy, elem_size(t.copy_dtype), "model_copy", i);
    if (rc != RG_OK) return rc;
  }
  return RG_OK;
}

RG_API int rg_optim_create(rg_optim** out, int device, int n, void* const* param, const void* const* grad,
                           void* const* state1, void* const* state2, void* const* model_copy, const int64_t* numel,
                           const int* grad_dtype, const int* copy_dtype) {
  if (out == nullptr || n < 0 || (n > 0 && (param == nullptr || grad == nullptr || numel == nullptr || grad_dtype == nullptr))) {
    set_error("rg_optim_create: bad arguments");
    return RG_EINVAL;
  }
  *out = nullptr;
  rg_optim* o = new (std::nothrow) rg_optim;
  if (o == nullptr) {
    set_error("rg_optim_create: out of host memory");
    return RG_ENOMEM;
  }
  o->device = device;
  o->n_tensors = n;
  o->has_state1 = state1 != nullptr;
  o->has_state2 = state2 != nullptr;
  o->rows.resize((size_t)n);
  o->chunk_begin.assign((size_t)n + 1, 0);
  for (int i = 0; i < n; ++i) {
    rg_optim::Row& t = o->rows[(size_t)i];
    t.param = param[i];
    t.grad = grad[i];
    t.state1 = state1 ? state1[i] : nullptr;
    t.state2 = state2 ? state2[i] : nullptr;
    t.copy = model_copy ? model_copy[i] : nullptr;
    t.numel = numel[i];
    t.grad_dtype = grad_dtype[i];
    t.copy_dtype = (model_copy && model_copy[i] && copy_dtype) ? copy_dtype[i] : RG_F32;
    if (t.copy) o->any_copy = true;
    if (t.numel < 0 || elem_size(t.grad_dtype) < 0 || elem_size(t.copy_dtype) < 0) {
      set_error("rg_optim_create: tensor %d has a bad size or dtype", i);
      delete o;
      return RG_EINVAL;
    }
    o->total_numel += t.numel;
    o->chunk_begin[(size_t)i + 1] = o->chunk_begin[(size_t)i] + (t.numel + o->chunk_elems - 1) / o->chunk_elems;
  }
  o->n_chunks = o->chunk_begin[(size_t)n];
  int rc = check_rows(o, "rg_optim_create");
  const int64_t tiles = (o->chunk_elems + kOptMinTileElems - 1) / kOptMinTileElems;
  if (rc == RG_OK && o->n_chunks * tiles > 0x7fffffffLL) {
    set_error("rg_optim_create: %lld elements exceed one launch", (long long)o->total_numel);
    rc = RG_EINVAL;
  }
  if (rc != RG_OK) {
    delete o;
    return rc;
  }
  if (o->n_chunks > 0) {
    DeviceGuard guard(device);
    const size_t bytes = (size_t)o->n_chunks * sizeof(OptChunkRec);
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&o->d_chunks), bytes);
    for (int k = 0; k < 2 && e == hipSuccess; ++k) {
      e = hipHostMalloc(reinterpret_cast<void**>(&o->stage[k]), bytes, hipHostMallocDefault);
      if (e == hipSuccess) e = hipEventCreateWithFlags(&o->stage_done[k], hipEventDisableTiming);
    }
    if (e == hipSuccess) {
      fill_opt_records(o, o->stage[0]);
      e = hipMemcpy(o->d_chunks, o->stage[0], bytes, hipMemcpyHostToDevice);
    }
    if (e != hipSuccess) {
      const int code = hip_fail(e, "rg_optim_create");
      (void)rg_optim_destroy(o);
      return e == hipErrorOutOfMemory ? RG_ENOMEM : code;
    }
  }
  *out = o;
  return RG_OK;
}

RG_API int rg_optim_destroy(rg_optim* o) {
  if (o == nullptr) return RG_OK;
  DeviceGuard guard(o->device);
  for (int k = 0; k < 2; ++k) {
    if (o->stage_done[k]) {
      if (o->stage_used[k]) (void)hipEventSynchronize(o->stage_done[k]);
      (void)hipEventDestroy(o->stage_done[k]);
    }
    if (o->stage[k]) (void)hipHostFree(o->stage[k]);
  }
  if (o->d_chunks) (void)hipFree(o->d_chunks);
  delete o;
  return RG_OK;
}

RG_API int rg_optim_update_pointers(rg_optim* o, void* const* param, const void* const* grad, void* const* state1,
                                    void* const* state2, void* const* model_copy, void* stream) {
  if (o == nullptr) {
    set_error("rg_optim_update_pointers: null table");
    return RG_EINVAL;
  }
  if ((state1 != nullptr && !o->has_state1) || (state2 != nullptr && !o->has_state2)) {
    set_error("rg_optim_update_pointers: the table was created without these state arrays");
    return RG_EINVAL;
  }
  std::vector<rg_optim::Row> saved = o->rows;
  for (int i = 0; i < o->n_tensors; ++i) {
    rg_optim::Row& t = o->rows[(size_t)i];
    if (param) t.param = param[i];
    if (grad) t.grad = grad[i];
    if (state1) t.state1 = state1[i];
    if (state2) t.state2 = state2[i];
    if (model_copy && (model_copy[i] != nullptr) != (t.copy != nullptr)) {
      o->rows = saved;
      set_error("rg_optim_update_pointers: tensor %d gains or loses its model copy", i);
      return RG_EINVAL;
    }
    if (model_copy) t.copy = model_copy[i];
  }
  const int rc = check_rows(o, "rg_optim_update_pointers");
  if (rc != RG_OK) {
    o->rows = saved;
    return rc;
  }
  if (o->n_chunks == 0) return RG_OK;
  DeviceGuard guard(o->device);
  const int k = o->next_stage;
  o->next_stage ^= 1;
  if (o->stage_used[k]) RG_HIP(hipEventSynchronize(o->stage_done[k]));
  fill_opt_records(o, o->stage[k]);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  RG_HIP(hipMemcpyAsync(o->d_chunks, o->stage[k], (size_t)o->n_chunks * sizeof(OptChunkRec), hipMemcpyHostToDevice, s));
  RG_HIP(hipEventRecord(o->stage_done[k], s));
  o->stage_used[k] = true;
  return RG_OK;
}

template <int ALGO>
static int launch_optim(const rg_optim* o, const OptConst& c, const rg_step_result* gate, int64_t bytes_per_elem,
                        void* stream, const rg_adam_clock* clock = nullptr) {
  if (o->n_chunks == 0) return RG_OK;
  DeviceGuard guard(o->device);
  OptArgs a;
  memset(&a, 0, sizeof(a));
  a.chunks = o->d_chunks;
  a.gate = reinterpret_cast<const StepResult*>(gate);
  a.clock = clock;
  a.grad_scale_dev = o->grad_scale_dev;
  a.tile_elems = OptShape<ALGO>::kTileElems;
  a.tiles_per_chunk = (int32_t)((o->chunk_elems + OptShape<ALGO>::kTileElems - 1) / OptShape<ALGO>::kTileElems);
  a.c = c;
  const dim3 grid((unsigned)(o->n_chunks * a.tiles_per_chunk)), block(OptShape<ALGO>::kThreads);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  unsigned lds = 0;
#ifdef RG_TUNING_ENV   // experiment builds only: unused dynamic LDS caps the blocks resident per compute unit
  if (const char* env = getenv("RG_LDS_OPTIM")) lds = (unsigned)atoi(env);
#endif
  if (o->total_numel * bytes_per_elem > ((int64_t)256 << 20)) hipLaunchKernelGGL((optim_kernel<ALGO, true>), grid, block, lds, s, a);
  else hipLaunchKernelGGL((optim_kernel<ALGO, false>), grid, block, lds, s, a);
  RG_HIP(hipGetLastError());
  return RG_OK;
}

static int adam_step(rg_optim* o, const rg_adam_args* g, const rg_adam_clock* clock, void* stream, const char* op) {
  if (o == nullptr || g == nullptr) {
    set_error("%s: null argument", op);
    return RG_EINVAL;
  }
  if (!o->has_state1 || !o->has_state2) {
    set_error("%s: the table has no exp_avg / exp_avg_sq pointers", op);
    return RG_EINVAL;
  }
  const int64_t step = clock != nullptr ? 1 : g->step;      // with a clock the count lives on the device
  if (step < 1 || !(g->lr >= 0.0) || !(g->eps >= 0.0) || !(g->beta1 >= 0.0 && g->beta1 < 1.0) ||
      !(g->beta2 >= 0.0 && g->beta2 < 1.0) || !(g->weight_decay >= 0.0)) {
    set_error("%s: bad hyper-parameters (lr %g betas %g %g eps %g wd %g step %lld)", op, g->lr, g->beta1, g->beta2,
              g->eps, g->weight_decay, (long long)g->step);
    return RG_EINVAL;
  }
  // The scalar factors as torch/optim/adam.py computes them: in double, from Python floats.
  const double bias1 = 1.0 - pow(g->beta1, (double)step);
  const double bias2 = 1.0 - pow(g->beta2, (double)step);
  const double weight = 1.0 - g->beta1;
  OptConst c;
  memset(&c, 0, sizeof(c));
  c.grad_scale = g->grad_scale;
  c.maximize = g->maximize;
  c.weight_decay = g->decoupled_weight_decay ? 0.0f : (float)g->weight_decay;
  c.param_mul = g->decoupled_weight_decay ? (float)(1.0 - g->lr * g->weight_decay) : 1.0f;
  c.lerp_from_end = ((float)weight < 0.5f) ? 0 : 1;
  c.lerp_coeff = c.lerp_from_end ? (float)weight - 1.0f : (float)weight;
  c.beta2 = (float)g->beta2;
  c.one_minus_beta2 = (float)(1.0 - g->beta2);
  c.neg_step_size = (float)(-(g->lr / bias1));
  c.bias2_sqrt = (float)sqrt(bias2);
  c.eps = (float)g->eps;
  return launch_optim<kAdam>(o, c, g->gate, 30, stream, clock);
}

RG_API int rg_optim_set_grad_scale_source(rg_optim* o, const float* grad_scale_dev) {
  if (o == nullptr || (reinterpret_cast<uintptr_t>(grad_scale_dev) & 3u) != 0) {
    set_error("rg_optim_set_grad_scale_source: null table or a pointer that is not 4-byte aligned");
    return RG_EINVAL;
  }
  o->grad_scale_dev = grad_scale_dev;
  return RG_OK;
}

RG_API int rg_adam_step(rg_optim* o, const rg_adam_args* g, void* stream) {
  return adam_step(o, g, nullptr, stream, "rg_adam_step");
}

RG_API int rg_adam_step_clocked(rg_optim* o, const rg_adam_args* g, const rg_adam_clock* clock_dev, void* stream) {
  if (clock_dev == nullptr) {
    set_error("rg_adam_step_clocked: null clock");
    return RG_EINVAL;
  }
  return adam_step(o, g, clock_dev, stream, "rg_adam_step_clocked");
}

RG_API int rg_adam_clock_advance(rg_adam_clock* clock_dev, double lr, double beta1, double beta2, const rg_step_result* gate,
                                 int device, void* stream) {
  if (clock_dev == nullptr || (reinterpret_cast<uintptr_t>(clock_dev) & 7u) != 0) {
    set_error("rg_adam_clock_advance: the clock must be an 8-byte aligned device pointer");
    return RG_EINVAL;
  }
  if (!(lr >= 0.0) || !(beta1 >= 0.0 && beta1 < 1.0) || !(beta2 >= 0.0 && beta2 < 1.0)) {
    set_error("rg_adam_clock_advance: bad hyper-parameters (lr %g betas %g %g)", lr, beta1, beta2);
    return RG_EINVAL;
  }
  DeviceGuard guard(device);
  hipLaunchKernelGGL(adam_clock_kernel, dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(stream), clock_dev, lr, beta1, beta2,
                     reinterpret_cast<const StepResult*>(gate));
  RG_HIP(hipGetLastError());
  return RG_OK;
}

RG_API int rg_sgd_step(rg_optim* o, const rg_sgd_args* g, void* stream) {
  if (o == nullptr || g == nullptr) {
    set_error("rg_sgd_step: null argument");
    return RG_EINVAL;
  }
  if (!(g->lr >= 0.0) || !(g->momentum >= 0.0) || !(g->weight_decay >= 0.0) ||
      (g->nesterov && (g->momentum <= 0.0 || g->dampening != 0.0))) {
    set_error("rg_sgd_step: bad hyper-parameters (lr %g momentum %g dampening %g wd %g nesterov %d)", g->lr, g->momentum,
              g->dampening, g->weight_decay, g->nesterov);
    return RG_EINVAL;
  }
  if (g->momentum != 0.0 && !o->has_state1) {
    set_error("rg_sgd_step: momentum needs the state1 (momentum buffer) pointers");
    return RG_EINVAL;
  }
  OptConst c;
  memset(&c, 0, sizeof(c));
  c.grad_scale = g->grad_scale;
  c.maximize = g->maximize;
  c.weight_decay = (float)g->weight_decay;
  c.param_mul = 1.0f;
  c.neg_lr = (float)(-g->lr);
  c.momentum = (float)g->momentum;
  c.one_minus_dampening = (float)(1.0 - g->dampening);
  c.nesterov = g->nesterov;
  c.first_step = g->first_step;
  c.has_momentum = g->momentum != 0.0 ? 1 : 0;
  return launch_optim<kSgd>(o, c, g->gate, c.has_momentum ? 22 : 14, stream);
}

RG_API int rg_scaler_init(rg_scaler_state* state_dev, const rg_scaler_state* init_host, int device, void* stream) {
  if (state_dev == nullptr || init_host == nullptr || (reinterpret_cast<uintptr_t>(state_dev) & 3u) != 0) {
    set_error("rg_scaler_init: null argument or a state that is not 4-byte aligned");
    return RG_EINVAL;
  }
  if (!(init_host->loss_scale > 0.0f) || !(init_host->max_loss_scale > 0.0f) || !(init_host->min_loss_scale >= 0.0f) ||
      init_host->scale_window < 1 || !(init_host->scale_factor > 1.0f)) {
    set_error("rg_scaler_init: bad schedule (scale %g min %g max %g window %d factor %g)", init_host->loss_scale,
              init_host->min_loss_scale, init_host->max_loss_scale, init_host->scale_window, init_host->scale_factor);
    return RG_EINVAL;
  }
  DeviceGuard guard(device);
  hipLaunchKernelGGL(scaler_init_kernel, dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(stream), state_dev, *init_host);
  RG_HIP(hipGetLastError());
  return RG_OK;
}

RG_API int rg_scaler_update(rg_scaler_state* state_dev, const rg_step_result* result_dev, int flags, int device, void* stream) {
  if (state_dev == nullptr || result_dev == nullptr || (reinterpret_cast<uintptr_t>(state_dev) & 3u) != 0) {
    set_error("rg_scaler_update: null argument or a state that is not 4-byte aligned");
    return RG_EINVAL;
  }
  if ((flags & ~(RG_SCALER_DYNAMIC | RG_SCALER_TRUNCATE)) != 0) {
    set_error("rg_scaler_update: unknown flags %d", flags);
    return RG_EINVAL;
  }
  DeviceGuard guard(device);
  hipLaunchKernelGGL(scaler_update_kernel, dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(stream), state_dev,
                     reinterpret_cast<const StepResult*>(result_dev), flags);
  RG_HIP(hipGetLastError());
  return RG_OK;
}
