// Host side of libranncgrad: layout arithmetic, plans (the chunk table resident on the
// device) and the extern "C" entry points declared in include/ranncgrad.h.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <mutex>
#include <new>
#include <vector>

#include "rg_host.h"
#include "rg_internal.h"

namespace rg {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

}  // namespace rg

using namespace rg;

// Block order of the read-only pass (PassArgs::xcd_run).  Measured on MI355X: round robin loses 6 % on 2.5e9 elements;
// runs of 16 to 1024 chunks per XCD and one contiguous eighth per XCD are within 1 % of each other, the eighths
// ahead by 0.5-1 % on all three workloads tried.
#ifndef RG_XCD_REDUCE_RUN
#define RG_XCD_REDUCE_RUN (-1)
#endif
struct rg_plan {
  int device = 0;
  int n_tensors = 0;
  int64_t total_numel = 0;
  int64_t total_bytes = 0;  // source + destination bytes one full pass touches
  int64_t chunk_elems = 0;
  int64_t n_chunks = 0;
  bool streaming = false;   // nontemporal accesses: the data is far larger than the caches
  int64_t write_tile_elems = kWriteTileElems;
  unsigned accumulate_lds = 0;   // unused dynamic LDS of rg_accumulate's pass (resident-block cap)
  int xcd_reduce = RG_XCD_REDUCE_RUN;               // block -> XCD mapping of read-only / writing passes (PassArgs::xcd_run)
  int xcd_write = 0;                 //   ... when every source sits on the line grid of its destination
  int xcd_write_offgrid = 256;       //   ... when some source does not (see fill_chunk_records)
  float begun_inv_scale = 0.0f;  // inv_scale of the last rg_step_begin, 0 = none pending
  const float* begun_scale_dev = nullptr;   // ... or where the kernels read it from (rg_step_begin_scaled)
  bool sums_describe_dst = false;   // the per-tensor sums on the device are those of the destinations as last written
  std::vector<TensorDesc> host_tensors;
  std::vector<int64_t> chunk_begin;  // [n_tensors + 1]
  bool dst_heads = false;            // some destination starts off a 128-byte boundary
  bool offgrid = false;              // some source is off the 128-byte grid of its destination
  bool all_in_place = false;         // every tensor with elements has dst == src (and so one dtype)
  char* dst_range = nullptr;         // the destinations, in plan order, lie back to back: one range of dst_range_bytes
  int64_t dst_range_bytes = 0;       //   (a gradient bucket's views); null when they do not
  int64_t dst_bytes = 0;             // bytes of all destinations

  // one device allocation, carved up
  char* dev_base = nullptr;
  size_t dev_bytes = 0;
  ChunkRec* d_chunks = nullptr;
  Partial* d_partials = nullptr;            // [n_chunks * max tiles per chunk * wavefronts per tile]: what the reducing passes leave
  int64_t* d_seg_chunk_begin = nullptr;     // [n_segments + 1]
  int32_t* d_tensor_seg_begin = nullptr;    // [n_tensors + 1]
  Partial* d_seg_sums = nullptr;            // [n_segments]
  float* d_tensor_norm = nullptr;
  StepResult* d_result = nullptr;
  int n_segments = 0;

  // pinned host memory: two chunk-table staging buffers (pointer updates stay stream
  // ordered without a host wait in the common case) and a read-back area
  char* pinned = nullptr;
  ChunkRec* stage[2] = {nullptr, nullptr};
  hipEvent_t stage_done[2] = {nullptr, nullptr};
  bool stage_used[2] = {false, false};
  int next_stage = 0;
  StepResult* h_result = nullptr;
  float* h_norms = nullptr;

  // optional ring of event quadruples around the kernels of rg_fused_step
  std::vector<hipEvent_t> timing_events;
  int timing_slots = 0;
  int64_t timing_count = 0;   // steps bracketed so far
  int64_t timing_steps = 0;   // steps seen so far
  int timing_stride = 1;      // every stride-th step is bracketed
  bool timing_all = true;  // false: only the write pass is bracketed (two records per step)
};

// Elements of a tensor before the first 128-byte boundary of the side its passes write
// (the destination; the source of a plan without destinations).
static int64_t tensor_head(const void* src, const void* dst, int ss, int ds) {
  if (dst != nullptr) return head_elems(reinterpret_cast<uintptr_t>(dst), kWriteAlignBytes, (unsigned)ds);
  return head_elems(reinterpret_cast<uintptr_t>(src), kAlignBytes, (unsigned)ss);
}

// Writes the chunk records of every tensor into `out` ([n_chunks]).  Chunk j of a tensor
// covers elements [j ? head + j*C : 0, head + (j+1)*C), clipped to the tensor: every chunk but
// the first starts on an aligned address, the first is up to `head` elements longer, and
// the number of chunks stays ceil(numel / C) whatever the addresses are (trailing chunks may be empty).
static void fill_chunk_records(rg_plan* p, ChunkRec* out) {
  p->dst_heads = false;
  p->offgrid = false;
  p->all_in_place = true;
  p->dst_range = nullptr;
  p->dst_range_bytes = 0;
  p->dst_bytes = 0;
  bool back_to_back = true;
  for (int i = 0; i < p->n_tensors; ++i) {
    const TensorDesc& t = p->host_tensors[(size_t)i];
    if (t.numel > 0 && (t.dst == nullptr || t.dst != t.src)) p->all_in_place = false;
    const int ss = elem_size(t.src_dtype), ds = elem_size(t.dst_dtype);
    if (t.dst != nullptr) p->dst_bytes += t.numel * ds;
    if (t.numel > 0 && back_to_back) {
      char* d = static_cast<char*>(t.dst);
      if (d == nullptr || (p->dst_range != nullptr && d != p->dst_range + p->dst_range_bytes)) {
        back_to_back = false;
        p->dst_range = nullptr;
        p->dst_range_bytes = 0;
      } else {
        if (p->dst_range == nullptr) p->dst_range = d;
        p->dst_range_bytes += t.numel * ds;
      }
    }
    const int64_t head = tensor_head(t.src, t.dst, ss, ds);
    if (t.dst != nullptr && t.numel > 0 && head != 0) p->dst_heads = true;
    // Write tiles start on destination lines; where the matching source address is not on a
    // line too, the line at every tile boundary is read by two blocks.  Such plans give each
    // XCD runs of consecutive tiles, so that the second read hits that XCD's L2.
    if (t.dst != nullptr && t.src != nullptr && t.numel > head &&
        ((reinterpret_cast<uintptr_t>(t.src) + (uintptr_t)(head * ss)) & (kAlignBytes - 1)) != 0)
      p->offgrid = true;
    for (int64_t c = p->chunk_begin[(size_t)i]; c < p->chunk_begin[(size_t)i + 1]; ++c) {
      const int64_t j = c - p->chunk_begin[(size_t)i];
      const int64_t start = j == 0 ? 0 : std::min(t.numel, head + j * p->chunk_elems);
      const int64_t end = std::min(t.numel, head + (j + 1) * p->chunk_elems);
      ChunkRec& r = out[c];
      r.src = t.src ? static_cast<const char*>(t.src) + start * ss : nullptr;
      r.dst = t.dst ? static_cast<char*>(t.dst) + start * ds : nullptr;
      r.len = (int32_t)(end - start);
      r.tensor = i;
      r.src_dtype = (int16_t)t.src_dtype;
      r.dst_dtype = (int16_t)t.dst_dtype;
      r.pad = 0;
    }
  }
}

// ---------------------------------------------------------------------------- misc

RG_API const char* rg_last_error(void) { return g_error; }
RG_API int rg_version(void) { return RG_VERSION; }
RG_API int rg_elem_size(int dtype) { return elem_size(dtype); }

// ---------------------------------------------------------------------------- layout

RG_API int64_t rg_aligned_numel(int64_t numel, int esz, int split_num) {
  if (numel < 0 || split_num < 1 || esz < 1 || 16 % esz != 0) {
    set_error("rg_aligned_numel: bad arguments (numel=%lld elem_size=%d split=%d)", (long long)numel, esz, split_num);
    return -1;
  }
  const int64_t unit = (int64_t)(16 / esz) * split_num;
  return round_up(numel, unit);
}

RG_API int rg_segment_layout(int64_t numel, int esz, int nranks, int64_t* aligned_size, int64_t* segment_size,
                             int64_t* offsets, int64_t* src_sizes) {
  const int64_t aligned = rg_aligned_numel(numel, esz, nranks);
  if (aligned < 0 || offsets == nullptr || src_sizes == nullptr) {
    if (aligned >= 0) set_error("rg_segment_layout: null output array");
    return RG_EINVAL;
  }
  const int64_t seg = aligned / nranks;
  int64_t off = 0;
  for (int i = 0; i < nranks; ++i) {
    offsets[i] = off;
    const int64_t rest = numel - off;
    src_sizes[i] = rest < seg ? rest : seg;
    off += src_sizes[i];
  }
  if (aligned_size) *aligned_size = aligned;
  if (segment_size) *segment_size = seg;
  return RG_OK;
}

RG_API int rg_bucket_layout(int n, const int64_t* numels, const int* dtypes, int64_t* offsets,
                            int64_t bucket_lengths[3]) {
  if (n < 0 || (n > 0 && (numels == nullptr || dtypes == nullptr || offsets == nullptr)) || bucket_lengths == nullptr) {
    set_error("rg_bucket_layout: bad arguments");
    return RG_EINVAL;
  }
  int64_t running[3] = {0, 0, 0};
  for (int i = 0; i < n; ++i) {
    if (elem_size(dtypes[i]) < 0 || numels[i] < 0) {
      set_error("rg_bucket_layout: tensor %d has dtype %d / numel %lld", i, dtypes[i], (long long)numels[i]);
      return RG_EINVAL;
    }
    offsets[i] = running[dtypes[i]];
    running[dtypes[i]] += numels[i];
  }
  for (int k = 0; k < 3; ++k) bucket_lengths[k] = running[k];
  return RG_OK;
}

// ---------------------------------------------------------------------------- plans

static int64_t default_chunk_elems(int64_t total, int widest_src_bytes = 2) {
  // Enough chunks to keep 256 compute units busy several times over, but never so small
  // that the per-chunk record fetch and reduction epilogue show.  Measured on plans of 1 M to
  // 50 M elements: about 2000 chunks is where the step is fastest (4000 costs 2-6 %).
  // The upper bound is 32 KiB of source per chunk - what one block of the read-only pass
  // streams: 16384 elements of a 16-bit type, 8192 of fp32 (measured on 2.4e8 fp32 elements in
  // 934 tensors: read-only pass 4 % faster than with 16384, the whole step 1.4 %).
  const int64_t kMax = widest_src_bytes >= 4 ? RG_DEFAULT_CHUNK_ELEMS / 2 : RG_DEFAULT_CHUNK_ELEMS;
  const int64_t kMin = kChunkQuantum, kTargetChunks = 2048;
  int64_t c = round_up(total / kTargetChunks + 1, kChunkQuantum);
  if (c < kMin) c = kMin;
  if (c > kMax) c = kMax;
  return c;
}

RG_API int rg_plan_create(rg_plan** out, int device, int n, const void* const* src, void* const* dst,
                          const int64_t* numel, const int* src_dtype, const int* dst_dtype, int64_t chunk_elems) {
  if (out == nullptr || n < 0 || (n > 0 && (numel == nullptr || src_dtype == nullptr || dst_dtype == nullptr))) {
    set_error("rg_plan_create: bad arguments");
    return RG_EINVAL;
  }
  *out = nullptr;
  if (chunk_elems < 0 || chunk_elems % kChunkQuantum != 0 || chunk_elems > kMaxChunkElems) {
    set_error("rg_plan_create: chunk_elems %lld is not a multiple of %lld in [0, %lld]", (long long)chunk_elems,
              (long long)kChunkQuantum, (long long)kMaxChunkElems);
    return RG_EINVAL;
  }
  rg_plan* p = new (std::nothrow) rg_plan();
  if (p == nullptr) return RG_ENOMEM;
  p->device = device;
  p->n_tensors = n;
  p->host_tensors.resize((size_t)n);
  int64_t total = 0, bytes = 0, same_width_bytes = 0, mixed_width_bytes = 0;
  int widest_src = 2, widest_any = 2;
  for (int i = 0; i < n; ++i) {
    const int ss = elem_size(src_dtype[i]), ds = elem_size(dst_dtype[i]);
    if (ss > widest_src && numel[i] > 0) widest_src = ss;
    if (numel[i] > 0) widest_any = std::max(widest_any, std::max(ss, ds));
    if (ss < 0 || ds < 0 || numel[i] < 0) {
      set_error("rg_plan_create: tensor %d has dtypes %d->%d / numel %lld", i, src_dtype[i], dst_dtype[i], (long long)numel[i]);
      delete p;
      return RG_EINVAL;
    }
    TensorDesc& t = p->host_tensors[(size_t)i];
    t.src = src ? src[i] : nullptr;
    t.dst = dst ? dst[i] : nullptr;
    t.numel = numel[i];
    t.src_dtype = src_dtype[i];
    t.dst_dtype = dst_dtype[i];
    int rc = check_pointer(t.src, ss, "src", i);
    if (rc == RG_OK) rc = check_pointer(t.dst, ds, "dst", i);
    if (rc != RG_OK) {
      delete p;
      return rc;
    }
    total += numel[i];
    bytes += numel[i] * (ss + ds);
    (ss == ds ? same_width_bytes : mixed_width_bytes) += numel[i] * (ss + ds);
  }
  // resident-block cap of rg_accumulate's pass (rg_internal.h), by what most of the plan's bytes look like
  p->accumulate_lds = same_width_bytes >= mixed_width_bytes ? kAccSameWidthLdsBytes : kAccMixedWidthLdsBytes;
  p->total_numel = total;
  p->total_bytes = bytes;
  // The Infinity Cache holds 256 MiB: below that a second pass can still hit in cache.
  p->streaming = bytes > (int64_t)256 << 20;
  p->chunk_elems = chunk_elems > 0 ? chunk_elems : default_chunk_elems(total, widest_src);
  // A block of a writing pass works best over 4 KiB of the wider side in two steps (measured on MI355X): 1024
  // elements when either side is fp32, 2048 when every tensor is 16 bits wide on both sides (a lane then moves
  // eight elements per instruction; one step over 1024 of them costs such a copy 3-10 %).
  if (widest_any == 2) p->write_tile_elems = 2 * kWriteTileElems;
  p->chunk_begin.assign((size_t)n + 1, 0);
  for (int i = 0; i < n; ++i)
    p->chunk_begin[(size_t)i + 1] = p->chunk_begin[(size_t)i] + (numel[i] + p->chunk_elems - 1) / p->chunk_elems;
  p->n_chunks = p->chunk_begin[(size_t)n];
  if (p->n_chunks > 0x7fffffffLL) {
    set_error("rg_plan_create: %lld chunks exceed the grid limit; raise chunk_elems", (long long)p->n_chunks);
    delete p;
    return RG_EINVAL;
  }

  // Segments: the units the partial sums of a tensor are added in (see rg_internal.h).  They depend on the chunk
  // counts only, so they are laid out once.
  std::vector<int64_t> seg_chunk_begin;
  std::vector<int32_t> tensor_seg_begin((size_t)n + 1, 0);
  for (int i = 0; i < n; ++i) {
    const int64_t first = p->chunk_begin[(size_t)i], count = p->chunk_begin[(size_t)i + 1] - first;
    const int64_t per = std::max<int64_t>(kSegmentChunks, (count + kMaxSegmentsPerTensor - 1) / kMaxSegmentsPerTensor);
    for (int64_t c = 0; c < count; c += per) seg_chunk_begin.push_back(first + c);
    tensor_seg_begin[(size_t)i + 1] = (int32_t)seg_chunk_begin.size();
  }
  p->n_segments = (int)seg_chunk_begin.size();
  seg_chunk_begin.push_back(p->n_chunks);

  // carve one device allocation
  size_t off = 0;
  auto carve = [&off](size_t nbytes) {
    const size_t at = off;
    off += (nbytes + 255) / 256 * 256;
    return at;
  };
  const size_t nt = (size_t)(n > 0 ? n : 1), nc = (size_t)(p->n_chunks > 0 ? p->n_chunks : 1);
  const size_t ns = (size_t)(p->n_segments > 0 ? p->n_segments : 1);
  const size_t o_chunks = carve(nc * sizeof(ChunkRec));
  // a pass that sums while it writes leaves one partial per tile
  if (p->write_tile_elems < kMinWriteTileElems) p->write_tile_elems = kMinWriteTileElems;
  const size_t max_tiles = (size_t)((p->chunk_elems + p->write_tile_elems - 1) / p->write_tile_elems);
  const size_t o_partials = carve(nc * max_tiles * (size_t)kWaveSlotsPerTile * sizeof(Partial));
  const size_t o_seg_begin = carve((ns + 1) * sizeof(int64_t));
  const size_t o_tensor_seg = carve((nt + 1) * sizeof(int32_t));
  const size_t o_seg_sums = carve(ns * sizeof(Partial));
  const size_t o_tnorm = carve(nt * sizeof(float));
  const size_t o_result = carve(sizeof(StepResult));
  p->dev_bytes = off;

  DeviceGuard guard(device);
  (void)fill_delay_ticks();   // ask the device for its wall-clock rate here, not on the first large rg_zero (which a caller may be capturing)
  hipError_t e = hipMalloc(reinterpret_cast<void**>(&p->dev_base), p->dev_bytes);
  if (e != hipSuccess) {
    delete p;
    return hip_fail(e, "hipMalloc(plan tables)");
  }
  char* b = p->dev_base;
  p->d_chunks = reinterpret_cast<ChunkRec*>(b + o_chunks);
  p->d_partials = reinterpret_cast<Partial*>(b + o_partials);
  p->d_seg_chunk_begin = reinterpret_cast<int64_t*>(b + o_seg_begin);
  p->d_tensor_seg_begin = reinterpret_cast<int32_t*>(b + o_tensor_seg);
  p->d_seg_sums = reinterpret_cast<Partial*>(b + o_seg_sums);
  p->d_tensor_norm = reinterpret_cast<float*>(b + o_tnorm);
  p->d_result = reinterpret_cast<StepResult*>(b + o_result);

  const size_t stage_bytes = (nc * sizeof(ChunkRec) + 255) / 256 * 256;
  const size_t norms_bytes = (nt * sizeof(float) + 255) / 256 * 256;
  e = hipHostMalloc(reinterpret_cast<void**>(&p->pinned), 2 * stage_bytes + 256 + norms_bytes, hipHostMallocDefault);
  if (e != hipSuccess) {
    (void)hipFree(p->dev_base);
    delete p;
    return hip_fail(e, "hipHostMalloc(plan staging)");
  }
  p->stage[0] = reinterpret_cast<ChunkRec*>(p->pinned);
  p->stage[1] = reinterpret_cast<ChunkRec*>(p->pinned + stage_bytes);
  p->h_result = reinterpret_cast<StepResult*>(p->pinned + 2 * stage_bytes);
  p->h_norms = reinterpret_cast<float*>(p->pinned + 2 * stage_bytes + 256);

  fill_chunk_records(p, p->stage[0]);
  bool ok = hipMemset(p->dev_base, 0, p->dev_bytes) == hipSuccess;
  if (ok && p->n_chunks > 0)
    ok = hipMemcpy(p->d_chunks, p->stage[0], (size_t)p->n_chunks * sizeof(ChunkRec), hipMemcpyHostToDevice) == hipSuccess;
  if (ok)
    ok = hipMemcpy(p->d_seg_chunk_begin, seg_chunk_begin.data(), seg_chunk_begin.size() * sizeof(int64_t),
                   hipMemcpyHostToDevice) == hipSuccess;
  if (ok)
    ok = hipMemcpy(p->d_tensor_seg_begin, tensor_seg_begin.data(), tensor_seg_begin.size() * sizeof(int32_t),
                   hipMemcpyHostToDevice) == hipSuccess;
  for (int k = 0; ok && k < 2; ++k) ok = hipEventCreateWithFlags(&p->stage_done[k], hipEventDisableTiming) == hipSuccess;
  if (!ok) {
    const hipError_t last = hipGetLastError();
    rg_plan_destroy(p);
    return hip_fail(last, "rg_plan_create: uploading the tables");
  }
  *out = p;
  return RG_OK;
}

RG_API int rg_plan_destroy(rg_plan* p) {
  if (p == nullptr) return RG_OK;
  DeviceGuard guard(p->device);
  (void)hipDeviceSynchronize();
  for (int k = 0; k < 2; ++k)
    if (p->stage_done[k]) (void)hipEventDestroy(p->stage_done[k]);
  for (hipEvent_t e : p->timing_events) (void)hipEventDestroy(e);
  if (p->pinned) (void)hipHostFree(p->pinned);
  if (p->dev_base) (void)hipFree(p->dev_base);
  delete p;
  return RG_OK;
}

RG_API int rg_plan_update_pointers(rg_plan* p, const void* const* src, void* const* dst, void* stream) {
  if (p == nullptr) {
    set_error("rg_plan_update_pointers: null plan");
    return RG_EINVAL;
  }
  const int n = p->n_tensors;
  for (int i = 0; i < n; ++i) {
    const TensorDesc& t = p->host_tensors[(size_t)i];
    int rc = RG_OK;
    if (src) rc = check_pointer(src[i], elem_size(t.src_dtype), "src", i);
    if (rc == RG_OK && dst) rc = check_pointer(dst[i], elem_size(t.dst_dtype), "dst", i);
    if (rc != RG_OK) return rc;
  }
  for (int i = 0; i < n; ++i) {
    if (src) p->host_tensors[(size_t)i].src = src[i];
    if (dst) p->host_tensors[(size_t)i].dst = dst[i];
  }
  if (dst) p->sums_describe_dst = false;
  if (p->n_chunks == 0) return RG_OK;
  DeviceGuard guard(p->device);
  const int k = p->next_stage;
  p->next_stage ^= 1;
  if (p->stage_used[k]) RG_HIP(hipEventSynchronize(p->stage_done[k]));
  fill_chunk_records(p, p->stage[k]);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  RG_HIP(hipMemcpyAsync(p->d_chunks, p->stage[k], (size_t)p->n_chunks * sizeof(ChunkRec), hipMemcpyHostToDevice, s));
  RG_HIP(hipEventRecord(p->stage_done[k], s));
  p->stage_used[k] = true;
  return RG_OK;
}

RG_API int rg_plan_num_tensors(const rg_plan* p) { return p ? p->n_tensors : -1; }
RG_API int64_t rg_plan_num_chunks(const rg_plan* p) { return p ? p->n_chunks : -1; }
RG_API int64_t rg_plan_chunk_elems(const rg_plan* p) { return p ? p->chunk_elems : -1; }
RG_API int64_t rg_plan_total_numel(const rg_plan* p) { return p ? p->total_numel : -1; }

RG_API int rg_plan_set_streaming(rg_plan* p, int mode) {
  if (p == nullptr || mode < -1 || mode > 1) {
    set_error("rg_plan_set_streaming: bad arguments");
    return RG_EINVAL;
  }
  p->streaming = mode < 0 ? p->total_bytes > ((int64_t)256 << 20) : mode != 0;
  return RG_OK;
}

// ---------------------------------------------------------------------------- operations

static PassArgs pass_args(const rg_plan* p, float scale) {
  PassArgs a;
  memset(&a, 0, sizeof(a));
  a.chunks = p->d_chunks;
  a.partials = p->d_partials;
  a.result = nullptr;
  a.n_chunks = p->n_chunks;
  a.tile_elems = (int32_t)p->chunk_elems;
  a.tiles_per_chunk = 1;
  a.peel_heads = p->dst_heads ? 1 : 0;
  a.xcd_run = p->offgrid ? p->xcd_write_offgrid : p->xcd_write;
  a.scale = scale;
  a.write_on_overflow = 0;
  a.zero_fill = 0;
  a.norm_of_source = 0;
  return a;
}

static ReduceArgs reduce_args(const rg_plan* p, float max_norm, int ignore_overflow, int partials_per_chunk = 1) {
  ReduceArgs r;
  memset(&r, 0, sizeof(r));
  r.partials = p->d_partials;
  r.seg_chunk_begin = p->d_seg_chunk_begin;
  r.tensor_seg_begin = p->d_tensor_seg_begin;
  r.seg_sums = p->d_seg_sums;
  r.tensor_norm = p->d_tensor_norm;
  r.result = p->d_result;
  r.n_tensors = p->n_tensors;
  r.n_segments = p->n_segments;
  r.partials_per_chunk = partials_per_chunk;
  r.max_norm = max_norm;
  r.ignore_overflow = ignore_overflow;
  return r;
}

// Write-only passes cut every chunk into tiles so that more, smaller blocks are in flight.
static void split_for_write(const rg_plan* p, PassArgs& a) {
  int64_t tile = p->write_tile_elems;
  if (tile > 0 && tile < kMinWriteTileElems) tile = kMinWriteTileElems;
  if (tile > 0 && tile < p->chunk_elems && p->n_chunks * ((p->chunk_elems + tile - 1) / tile) <= 0x7fffffffLL) {
    a.tile_elems = (int32_t)tile;
    a.tiles_per_chunk = (int32_t)((p->chunk_elems + tile - 1) / tile);
  }
}

// The in-place multiply behind a one-pass write: does nothing unless the decision on the device says
// "clipped".  Its blocks walk several chunks each so that an idle launch retires about 16 K blocks at most
// (an empty block costs 0.2 ns of dispatch: one per chunk was 32 us on 2.5e9 elements).
static hipError_t launch_scale_if_clipped(const rg_plan* p, hipStream_t s) {
  PassArgs b = pass_args(p, 1.0f);
  b.result = p->d_result;
  b.only_if_clipped = 1;
  b.src_is_dst = 1;
  b.chunks_per_block = (int32_t)((p->n_chunks + 16383) / 16384);
  if (b.chunks_per_block < 1) b.chunks_per_block = 1;
  return launch_gated_pass(b, p->streaming, s);
}

// One pass that both reduces and writes, over tiles of each chunk: every tile leaves its own partial sum; two
// small launches (one for small plans) turn them into the per-tensor norms and the decision.
static int tiled_reduce_write(rg_plan* p, PassArgs& a, int mode, hipStream_t s, float max_norm = 0.0f,
                              int ignore_overflow = 0, hipEvent_t after_pass = nullptr) {
  split_for_write(p, a);
  RG_HIP(launch_pass(mode, a, p->streaming, s));
  if (after_pass) RG_HIP(hipEventRecord(after_pass, s));
  RG_HIP(launch_reduce(reduce_args(p, max_norm, ignore_overflow, a.tiles_per_chunk * kWaveSlotsPerTile), p->n_chunks, s));
  return RG_OK;
}

// Which pointers an operation dereferences.
enum { kNeedSrc = 1, kNeedDst = 2 };

static int check_plan(const rg_plan* p, int need, const char* op) {
  if (p == nullptr) {
    set_error("%s: null plan", op);
    return RG_EINVAL;
  }
  for (int i = 0; i < p->n_tensors; ++i) {
    const TensorDesc& t = p->host_tensors[(size_t)i];
    if (t.numel == 0) continue;
    if ((need & kNeedDst) && t.dst == nullptr) {
      set_error("%s: tensor %d has no destination pointer", op, i);
      return RG_EINVAL;
    }
    if ((need & kNeedDst) && t.dst == t.src && t.src_dtype != t.dst_dtype) {
      set_error("%s: tensor %d is in place but changes dtype", op, i);
      return RG_EINVAL;
    }
  }
  return RG_OK;
}

RG_API int rg_fused_step(rg_plan* p, float inv_scale, float max_norm, int flags, void* stream) {
  const int rc = check_plan(p, kNeedSrc | kNeedDst, "rg_fused_step");
  if (rc != RG_OK) return rc;
  p->sums_describe_dst = false;
  if (!(inv_scale == inv_scale) || inv_scale == 0.0f) {
    set_error("rg_fused_step: inv_scale must be a non-zero number");
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  hipEvent_t* ev = nullptr;
  if (p->timing_slots > 0 && p->timing_steps++ % p->timing_stride == 0)
    ev = &p->timing_events[(size_t)(p->timing_count++ % p->timing_slots) * 4];
  PassArgs a = pass_args(p, inv_scale);
  const bool all = ev != nullptr && p->timing_all;
  // In place with inv_scale == 1 a step that does not clip leaves every value as it is: the
  // second pass then has nothing to write and is gated on the decision.
  const bool identity_unless_clipped = p->all_in_place && inv_scale == 1.0f;
  if ((flags & RG_STEP_EXPECT_NO_CLIP) && !identity_unless_clipped) {
    // One pass writes the unscaled values while it sums them; only if the decision then says
    // "clip" does a second kernel scale the destination in place.  That kernel's blocks cover
    // several whole chunks each, so finding that there is nothing to do costs a few microseconds.
    if (all) RG_HIP(hipEventRecord(ev[0], s));
    const int rc1 = tiled_reduce_write(p, a, kModeReduce | kModeWrite, s, max_norm,
                                       (flags & RG_STEP_IGNORE_OVERFLOW) ? 1 : 0, all ? ev[1] : nullptr);
    if (rc1 != RG_OK) return rc1;
    if (ev) RG_HIP(hipEventRecord(ev[2], s));
    RG_HIP(launch_scale_if_clipped(p, s));
    if (ev) RG_HIP(hipEventRecord(ev[3], s));
    return RG_OK;
  }
  if (all) RG_HIP(hipEventRecord(ev[0], s));
  a.xcd_run = p->xcd_reduce;
  RG_HIP(launch_pass(kModeReduce, a, p->streaming, s));
  if (all) RG_HIP(hipEventRecord(ev[1], s));
  RG_HIP(launch_reduce(reduce_args(p, max_norm, (flags & RG_STEP_IGNORE_OVERFLOW) ? 1 : 0), p->n_chunks, s));
  if (ev) RG_HIP(hipEventRecord(ev[2], s));
  a.result = p->d_result;
  a.write_on_overflow = (flags & RG_STEP_WRITE_ON_OVERFLOW) ? 1 : 0;
  a.only_if_clipped = identity_unless_clipped ? 1 : 0;
  a.xcd_run = p->offgrid ? p->xcd_write_offgrid : p->xcd_write;
  if (identity_unless_clipped && (flags & RG_STEP_EXPECT_NO_CLIP)) {
    // a launch that will most likely find nothing to do: few blocks to retire
    a.chunks_per_block = (int32_t)((p->n_chunks + 16383) / 16384);
    RG_HIP(launch_gated_pass(a, p->streaming, s));
  } else {
    split_for_write(p, a);
    RG_HIP(launch_pass(kModeWrite, a, p->streaming, s));
  }
  if (ev) RG_HIP(hipEventRecord(ev[3], s));
  return RG_OK;
}

RG_API int rg_step_begin(rg_plan* p, float inv_scale, void* stream) {
  const int rc = check_plan(p, kNeedSrc | kNeedDst, "rg_step_begin");
  if (rc != RG_OK) return rc;
  p->sums_describe_dst = false;
  if (!(inv_scale == inv_scale) || inv_scale == 0.0f) {
    set_error("rg_step_begin: inv_scale must be a non-zero number");
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  PassArgs a = pass_args(p, inv_scale);
  a.xcd_run = p->xcd_reduce;
  RG_HIP(launch_pass(kModeReduce, a, p->streaming, s));
  RG_HIP(launch_reduce(reduce_args(p, 0.0f, 0), p->n_chunks, s));
  p->begun_inv_scale = inv_scale;
  p->begun_scale_dev = nullptr;
  return RG_OK;
}

RG_API int rg_step_begin_scaled(rg_plan* p, const float* inv_scale_dev, void* stream) {
  const int rc = check_plan(p, kNeedSrc | kNeedDst, "rg_step_begin_scaled");
  if (rc != RG_OK) return rc;
  p->sums_describe_dst = false;
  if (inv_scale_dev == nullptr || (reinterpret_cast<uintptr_t>(inv_scale_dev) & 3u) != 0) {
    set_error("rg_step_begin_scaled: inv_scale_dev must be a 4-byte aligned device pointer");
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  PassArgs a = pass_args(p, 1.0f);
  a.scale_dev = inv_scale_dev;
  a.xcd_run = p->xcd_reduce;
  RG_HIP(launch_pass(kModeReduce, a, p->streaming, s));
  RG_HIP(launch_reduce(reduce_args(p, 0.0f, 0), p->n_chunks, s));
  p->begun_inv_scale = 1.0f;           // pending; the value itself is read on the device
  p->begun_scale_dev = inv_scale_dev;
  return RG_OK;
}

RG_API int rg_step_finish(rg_plan* p, float max_norm, int flags, void* stream) {
  const int rc = check_plan(p, kNeedSrc | kNeedDst, "rg_step_finish");
  if (rc != RG_OK) return rc;
  if (p->begun_inv_scale == 0.0f) {
    set_error("rg_step_finish: no rg_step_begin is pending on this plan");
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  RG_HIP(launch_decide(reduce_args(p, max_norm, (flags & RG_STEP_IGNORE_OVERFLOW) ? 1 : 0), s));
  PassArgs a = pass_args(p, p->begun_inv_scale);
  a.scale_dev = p->begun_scale_dev;
  a.result = p->d_result;
  a.write_on_overflow = (flags & RG_STEP_WRITE_ON_OVERFLOW) ? 1 : 0;
  split_for_write(p, a);
  RG_HIP(launch_pass(kModeWrite, a, p->streaming, s));
  p->begun_inv_scale = 0.0f;
  p->begun_scale_dev = nullptr;
  return RG_OK;
}

RG_API int rg_step_decide(rg_plan* p, float max_norm, int flags, void* stream) {
  const int rc = check_plan(p, kNeedSrc, "rg_step_decide");
  if (rc != RG_OK) return rc;
  if (p->begun_inv_scale == 0.0f) {
    set_error("rg_step_decide: no rg_step_begin is pending on this plan");
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  RG_HIP(launch_decide(reduce_args(p, max_norm, (flags & RG_STEP_IGNORE_OVERFLOW) ? 1 : 0),
                       reinterpret_cast<hipStream_t>(stream)));
  return RG_OK;   // the begin stays pending: rg_step_finish may still write the gradients
}

RG_API int rg_unscale_pack(rg_plan* p, float inv_scale, void* stream) {
  const int rc = check_plan(p, kNeedSrc | kNeedDst, "rg_unscale_pack");
  if (rc != RG_OK) return rc;
  if (!(inv_scale == inv_scale) || inv_scale == 0.0f) {
    set_error("rg_unscale_pack: inv_scale must be a non-zero number");
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  PassArgs a = pass_args(p, inv_scale);
  const int rc2 = tiled_reduce_write(p, a, kModeReduce | kModeWrite, s);
  p->sums_describe_dst = rc2 == RG_OK;
  return rc2;
}

RG_API int rg_step_apply_clip(rg_plan* p, float max_norm, int flags, void* stream) {
  const int rc = check_plan(p, kNeedDst, "rg_step_apply_clip");
  if (rc != RG_OK) return rc;
  if (!p->sums_describe_dst) {
    set_error("rg_step_apply_clip: the last operation on this plan was not rg_unscale_pack / rg_unscale_accumulate");
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  RG_HIP(launch_decide(reduce_args(p, max_norm, (flags & RG_STEP_IGNORE_OVERFLOW) ? 1 : 0), s));
  RG_HIP(launch_scale_if_clipped(p, s));
  p->sums_describe_dst = false;                          // the destinations are about to change
  return RG_OK;
}

static int check_not_in_place(const rg_plan* p, const char* op) {
  for (int i = 0; i < p->n_tensors; ++i) {
    const TensorDesc& t = p->host_tensors[(size_t)i];
    if (t.numel > 0 && t.src != nullptr && t.src == t.dst) {
      set_error("%s: tensor %d accumulates into itself", op, i);
      return RG_EINVAL;
    }
  }
  return RG_OK;
}

RG_API int rg_accumulate(rg_plan* p, float scale, void* stream) {
  int rc = check_plan(p, kNeedSrc | kNeedDst, "rg_accumulate");
  if (rc == RG_OK) rc = check_not_in_place(p, "rg_accumulate");
  if (rc != RG_OK) return rc;
  p->sums_describe_dst = false;
  DeviceGuard guard(p->device);
  PassArgs a = pass_args(p, scale);
  split_for_write(p, a);
  a.dynamic_lds = p->accumulate_lds;
  RG_HIP(launch_pass(kModeWrite | kModeAccumulate, a, p->streaming, reinterpret_cast<hipStream_t>(stream)));
  return RG_OK;
}

RG_API int rg_unscale_accumulate(rg_plan* p, float inv_scale, void* stream) {
  int rc = check_plan(p, kNeedSrc | kNeedDst, "rg_unscale_accumulate");
  if (rc == RG_OK) rc = check_not_in_place(p, "rg_unscale_accumulate");
  if (rc != RG_OK) return rc;
  if (!(inv_scale == inv_scale) || inv_scale == 0.0f) {
    set_error("rg_unscale_accumulate: inv_scale must be a non-zero number");
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  PassArgs a = pass_args(p, inv_scale);
  // Twelve resident blocks: what this kernel's register count (76) allows anyway, and what measures best for it.
  // Said here so that the pass does not speed up or slow down with the compiler's register allocation.
  a.dynamic_lds = kAccMixedWidthLdsBytes;
  const int rc2 = tiled_reduce_write(p, a, kModeReduce | kModeWrite | kModeAccumulate, s);
  p->sums_describe_dst = rc2 == RG_OK;
  return rc2;
}

RG_API int rg_grad_norm(rg_plan* p, void* stream) {
  const int rc = check_plan(p, kNeedSrc, "rg_grad_norm");
  if (rc != RG_OK) return rc;
  p->sums_describe_dst = false;
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  PassArgs a = pass_args(p, 1.0f);
  a.norm_of_source = 1;
  a.xcd_run = p->xcd_reduce;
  RG_HIP(launch_pass(kModeReduce, a, p->streaming, s));
  RG_HIP(launch_reduce(reduce_args(p, 0.0f, 1), p->n_chunks, s));
  return RG_OK;
}

RG_API int rg_scale_cast(rg_plan* p, float scale, void* stream) {
  const int rc = check_plan(p, kNeedSrc | kNeedDst, "rg_scale_cast");
  if (rc != RG_OK) return rc;
  p->sums_describe_dst = false;
  DeviceGuard guard(p->device);
  PassArgs a = pass_args(p, scale);
  split_for_write(p, a);
  RG_HIP(launch_pass(kModeWrite, a, p->streaming, reinterpret_cast<hipStream_t>(stream)));
  return RG_OK;
}

RG_API int rg_plan_tune(rg_plan* p, void* stream) {
  const int rc = check_plan(p, kNeedSrc | kNeedDst, "rg_plan_tune");
  if (rc != RG_OK) return rc;
  if (p->all_in_place || p->n_chunks == 0) return RG_OK;   // nothing that could be run without changing the data
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  hipEvent_t e0 = nullptr, e1 = nullptr;
  RG_HIP(hipEventCreate(&e0));
  if (hipEventCreate(&e1) != hipSuccess) {
    (void)hipEventDestroy(e0);
    return hip_fail(hipGetLastError(), "hipEventCreate");
  }
  // Which order suits a plan depends on how its tensors lie in memory (packed into one bucket or scattered,
  // on or off each other's line grid) in ways no simple rule captured: measured, the best order differed by up
  // to 4 % of a pass between plans of the same sizes.
  // Candidates are timed in turn, three rounds, and each keeps its fastest round, so that a clock ramp or a
  // neighbour's burst does not pick the winner; the order in use is only given up for a gain above 1 %.
  const int current = p->offgrid ? p->xcd_write_offgrid : p->xcd_write;
  int candidates[5] = {current, 0, 64, 256, -1};
  float fastest[5] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
  hipError_t err = hipSuccess;
  for (int round = 0; round < 3 && err == hipSuccess; ++round) {
    for (int k = 0; k < 5 && err == hipSuccess; ++k) {
      if (k > 0 && candidates[k] == current) continue;
      PassArgs a = pass_args(p, 1.0f);
      a.xcd_run = candidates[k];
      split_for_write(p, a);
      err = launch_pass(kModeWrite, a, p->streaming, s);           // warm-up
      if (err == hipSuccess) err = hipEventRecord(e0, s);
      for (int rep = 0; rep < 2 && err == hipSuccess; ++rep) err = launch_pass(kModeWrite, a, p->streaming, s);
      if (err == hipSuccess) err = hipEventRecord(e1, s);
      if (err == hipSuccess) err = hipEventSynchronize(e1);
      float ms = 0.0f;
      if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
      if (err == hipSuccess && (fastest[k] == 0.0f || ms < fastest[k])) fastest[k] = ms;
    }
  }
  int best = current;
  float best_ms = fastest[0] * 0.99f;
  for (int k = 1; k < 5 && err == hipSuccess; ++k) {
    if (fastest[k] > 0.0f && fastest[k] < best_ms) {
      best_ms = fastest[k];
      best = candidates[k];
    }
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (err != hipSuccess) return hip_fail(err, "rg_plan_tune");
  p->xcd_write = p->xcd_write_offgrid = best;
  p->sums_describe_dst = false;
  return RG_OK;
}

RG_API int rg_plan_write_order(const rg_plan* p) {
  return p == nullptr ? 0 : (p->offgrid ? p->xcd_write_offgrid : p->xcd_write);
}

RG_API int rg_plan_set_write_order(rg_plan* p, int order) {
  if (p == nullptr || order < -1 || order > 65536) {
    set_error("rg_plan_set_write_order: bad arguments (order %d)", order);
    return RG_EINVAL;
  }
  p->xcd_write = p->xcd_write_offgrid = order;
  return RG_OK;
}

RG_API int rg_scale_cast_single(const void* src_dev, void* dst_dev, int64_t numel, int src_dtype, int dst_dtype,
                                float scale, int device, void* stream) {
  const int ss = elem_size(src_dtype), ds = elem_size(dst_dtype);
  if (ss < 0 || ds < 0 || numel < 0 || (numel > 0 && dst_dev == nullptr)) {
    set_error("rg_scale_cast_single: bad arguments (dtypes %d->%d, numel %lld)", src_dtype, dst_dtype, (long long)numel);
    return RG_EINVAL;
  }
  int rc = check_pointer(src_dev, ss, "src", 0);
  if (rc == RG_OK) rc = check_pointer(dst_dev, ds, "dst", 0);
  if (rc != RG_OK) return rc;
  if (src_dev == dst_dev && src_dtype != dst_dtype) {
    set_error("rg_scale_cast_single: in place but changes dtype");
    return RG_EINVAL;
  }
  if (numel == 0) return RG_OK;
  const int64_t chunk = RG_DEFAULT_CHUNK_ELEMS;
  const int64_t n_chunks = (numel + chunk - 1) / chunk;
  const int64_t tiles = (chunk + kWriteTileElems - 1) / kWriteTileElems;
  if (n_chunks * tiles > 0x7fffffffLL) {
    set_error("rg_scale_cast_single: %lld elements exceed one launch", (long long)numel);
    return RG_EINVAL;
  }
  PassArgs a;
  memset(&a, 0, sizeof(a));
  a.single.src = src_dev;
  a.single.dst = dst_dev;
  a.single.src_dtype = (int16_t)src_dtype;
  a.single.dst_dtype = (int16_t)dst_dtype;
  a.single_numel = numel;
  a.single_chunk_elems = chunk;
  a.single_head = tensor_head(src_dev, dst_dev, ss, ds);
  a.peel_heads = a.single_head != 0 ? 1 : 0;
  if (src_dev != nullptr && numel > a.single_head &&
      ((reinterpret_cast<uintptr_t>(src_dev) + (uintptr_t)(a.single_head * ss)) & (kAlignBytes - 1)) != 0)
    a.xcd_run = 256;   // source off the destination's line grid: consecutive tiles share an XCD's L2
  a.n_chunks = n_chunks;
  a.tile_elems = kWriteTileElems;
  a.tiles_per_chunk = (int32_t)tiles;
  a.scale = scale;
  a.zero_fill = src_dev == nullptr ? 1 : 0;
  DeviceGuard guard(device);
  const bool streaming = numel * (ss + ds) > ((int64_t)256 << 20);
  RG_HIP(launch_pass(kModeWrite, a, streaming, reinterpret_cast<hipStream_t>(stream)));
  return RG_OK;
}

// ---------------------------------------------------------------------------- allocation-free fused step

// Working memory of rg_fused_step_static: what a plan keeps in its own allocation (result
// block, per-tensor norm, segment sums, one partial per chunk), for one tensor pair of at most
// RG_STATIC_MAX_SRC_BYTES of source.  Every GPU the library runs on holds its own copy of this
// array until the process ends; host code only ever uses the per-device address looked up below.
constexpr int64_t kStaticMaxChunks = RG_STATIC_MAX_SRC_BYTES / (2 * RG_DEFAULT_CHUNK_ELEMS);   // 32 KiB of source per chunk
constexpr size_t kStaticResultOff = 0;        // StepResult
constexpr size_t kStaticTensorOff = 256;      // float norm
constexpr size_t kStaticSegOff = 512;         // Partial[kMaxSegmentsPerTensor]
constexpr size_t kStaticPartialsOff = kStaticSegOff + (size_t)kMaxSegmentsPerTensor * sizeof(Partial);
constexpr size_t kStaticScratchBytes = kStaticPartialsOff + (size_t)kStaticMaxChunks * sizeof(Partial);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static char* g_scratch_ptr[kMaxDevices] = {};   // device address of `scratch` on each GPU, looked up once

// The address of this GPU's copy of `scratch` (the caller has made `device` current).
static int static_scratch(int device, char** out) {
  if (device < 0 || device >= kMaxDevices) {
    set_error("rg_fused_step_static: device %d is outside [0, %d)", device, kMaxDevices);
    return RG_EINVAL;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    void* ptr = nullptr;
    RG_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    g_scratch_ptr[device] = static_cast<char*>(ptr);
  }
  *out = g_scratch_ptr[device];
  return RG_OK;
}

RG_API int rg_fused_step_static(const void* src_dev, void* dst_dev, int64_t numel, int src_dtype, int dst_dtype,
                                float inv_scale, float max_norm, int flags, rg_step_result* result_dev, int device,
                                void* stream) {
  const int ss = elem_size(src_dtype), ds = elem_size(dst_dtype);
  if (ss < 0 || ds < 0 || numel < 0 || (numel > 0 && (src_dev == nullptr || dst_dev == nullptr))) {
    set_error("rg_fused_step_static: bad arguments (dtypes %d->%d, numel %lld)", src_dtype, dst_dtype, (long long)numel);
    return RG_EINVAL;
  }
  if (numel > (int64_t)RG_STATIC_MAX_SRC_BYTES / ss) {
    set_error("rg_fused_step_static: %lld elements of %d bytes exceed the limit of %lld source bytes; use a plan (rg_fused_step)",
              (long long)numel, ss, (long long)RG_STATIC_MAX_SRC_BYTES);
    return RG_EINVAL;
  }
  if (!(inv_scale == inv_scale) || inv_scale == 0.0f) {
    set_error("rg_fused_step_static: inv_scale must be a non-zero number");
    return RG_EINVAL;
  }
  int rc = check_pointer(src_dev, ss, "src", 0);
  if (rc == RG_OK) rc = check_pointer(dst_dev, ds, "dst", 0);
  if (rc == RG_OK) rc = check_pointer(result_dev, 8, "result", 0);
  if (rc != RG_OK) return rc;
  if (src_dev == dst_dev && src_dtype != dst_dtype) {
    set_error("rg_fused_step_static: in place but changes dtype");
    return RG_EINVAL;
  }
  DeviceGuard guard(device);
  char* base = nullptr;
  rc = static_scratch(device, &base);
  if (rc != RG_OK) return rc;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);

  // the launch shapes of a one-tensor plan, so that both give the same bits
  const int64_t chunk = default_chunk_elems(numel, ss);
  const int64_t n_chunks = (numel + chunk - 1) / chunk;
  if (n_chunks > kStaticMaxChunks) {      // cannot happen below the size limit; the array's bound is checked all the same
    set_error("rg_fused_step_static: %lld chunks exceed the working memory", (long long)n_chunks);
    return RG_EINVAL;
  }
  const bool streaming = numel * (ss + ds) > ((int64_t)256 << 20);
  const int64_t head = numel > 0 ? tensor_head(src_dev, dst_dev, ss, ds) : 0;
  const bool offgrid = numel > head &&
      ((reinterpret_cast<uintptr_t>(src_dev) + (uintptr_t)(head * ss)) & (kAlignBytes - 1)) != 0;

  PassArgs a;
  memset(&a, 0, sizeof(a));
  a.single.src = src_dev;
  a.single.dst = dst_dev;
  a.single.src_dtype = (int16_t)src_dtype;
  a.single.dst_dtype = (int16_t)dst_dtype;
  a.single_numel = numel;
  a.single_chunk_elems = chunk;
  a.single_head = head;
  a.peel_heads = head != 0 ? 1 : 0;
  a.partials = reinterpret_cast<Partial*>(base + kStaticPartialsOff);
  a.n_chunks = n_chunks;
  a.tile_elems = (int32_t)chunk;
  a.tiles_per_chunk = 1;
  a.scale = inv_scale;
  a.xcd_run = RG_XCD_REDUCE_RUN;
  RG_HIP(launch_pass(kModeReduce, a, streaming, s));

  ReduceArgs f;
  memset(&f, 0, sizeof(f));
  f.partials = a.partials;
  f.single_chunks = n_chunks;
  f.single_seg_chunks = std::max<int64_t>(kSegmentChunks, (n_chunks + kMaxSegmentsPerTensor - 1) / kMaxSegmentsPerTensor);
  f.n_segments = (int)((n_chunks + f.single_seg_chunks - 1) / f.single_seg_chunks);
  f.seg_sums = reinterpret_cast<Partial*>(base + kStaticSegOff);
  f.tensor_norm = reinterpret_cast<float*>(base + kStaticTensorOff);
  f.result = reinterpret_cast<StepResult*>(base + kStaticResultOff);
  f.result_copy = result_dev;
  f.n_tensors = 1;
  f.partials_per_chunk = 1;
  f.max_norm = max_norm;
  f.ignore_overflow = (flags & RG_STEP_IGNORE_OVERFLOW) ? 1 : 0;
  RG_HIP(launch_reduce(f, n_chunks, s));

  a.result = f.result;
  a.write_on_overflow = (flags & RG_STEP_WRITE_ON_OVERFLOW) ? 1 : 0;
  a.xcd_run = offgrid ? 256 : 0;
  if (kWriteTileElems < chunk) {
    a.tile_elems = kWriteTileElems;
    a.tiles_per_chunk = (int32_t)((chunk + kWriteTileElems - 1) / kWriteTileElems);
  }
  RG_HIP(launch_pass(kModeWrite, a, streaming, s));
  return RG_OK;
}

RG_API int rg_zero(rg_plan* p, void* stream) {
  const int rc = check_plan(p, kNeedDst, "rg_zero");
  if (rc != RG_OK) return rc;
  p->sums_describe_dst = false;
  DeviceGuard guard(p->device);
  if (p->dst_range != nullptr) {
    // The destinations are the views of one bucket: a flat fill needs no table and, above the size of the
    // memory-side cache, is paced (BERT-large's bucket: 94 % of peak against 89 % through the table).
    RG_HIP(launch_fill_zero(p->dst_range, p->dst_range_bytes, reinterpret_cast<hipStream_t>(stream)));
    return RG_OK;
  }
  PassArgs a = pass_args(p, 1.0f);
  a.zero_fill = 1;
  split_for_write(p, a);
  // A write-only pass wants each XCD to fill runs of consecutive tiles, whatever order the plan's copies prefer
  // (measured on MI355X: BERT-large's bucket 83 % of peak round robin, 91.5 % with runs of 64 tiles, 90.6 % with
  // runs of 256, 86 % with contiguous eighths; the ResNet's 83.7 / 87.2 / 87.8 / 82.5 %).
  a.xcd_run = kZeroXcdRun;
  // Scattered destinations of streaming size: the flat fill's pacing in small.  A wavefront here first fetches its
  // chunk record, which spaces the stores already; holding it another 0.1 us pays from about 1.5 GiB (64 MiB
  // tensors, % of peak without / with: 1 GiB 93.8 / 92.9, 1.5 GiB 91.8 / 92.8, 2 GiB 91.4 / 93.2, 4 GiB 89.6 / 92.6,
  // 8 GiB 89.7 / 92.5; the 775 fp16 gradients of a 2.5e9-parameter stage 88.9 -> 92.9 %) and costs 2-4 points
  // below 1 GiB.
  if (p->streaming && p->dst_bytes >= kZeroDelayMinBytes) a.zero_delay_ticks = fill_delay_ticks(kZeroDelayNs);
  RG_HIP(launch_pass(kModeWrite, a, p->streaming, reinterpret_cast<hipStream_t>(stream)));
  return RG_OK;
}

RG_API int rg_fill_zero(void* dst_dev, int64_t nbytes, int device, void* stream) {
  if (nbytes < 0 || (nbytes > 0 && dst_dev == nullptr)) {
    set_error("rg_fill_zero: bad arguments");
    return RG_EINVAL;
  }
  DeviceGuard guard(device);
  RG_HIP(launch_fill_zero(dst_dev, nbytes, reinterpret_cast<hipStream_t>(stream)));
  return RG_OK;
}

RG_API int rg_result_device_ptr(const rg_plan* p, const rg_step_result** out_dev) {
  if (p == nullptr || out_dev == nullptr) {
    set_error("rg_result_device_ptr: null argument");
    return RG_EINVAL;
  }
  *out_dev = reinterpret_cast<const rg_step_result*>(p->d_result);
  return RG_OK;
}

RG_API int rg_tensor_norms_device_ptr(const rg_plan* p, const float** out_dev) {
  if (p == nullptr || out_dev == nullptr) {
    set_error("rg_tensor_norms_device_ptr: null argument");
    return RG_EINVAL;
  }
  *out_dev = p->d_tensor_norm;
  return RG_OK;
}

RG_API int rg_read_result(rg_plan* p, rg_step_result* out_host, void* stream) {
  if (p == nullptr || out_host == nullptr) {
    set_error("rg_read_result: null argument");
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  RG_HIP(hipMemcpyAsync(p->h_result, p->d_result, sizeof(StepResult), hipMemcpyDeviceToHost, s));
  RG_HIP(hipStreamSynchronize(s));
  out_host->norm = p->h_result->norm;
  out_host->coef = p->h_result->coef;
  out_host->overflow = p->h_result->overflow;
  out_host->clipped = p->h_result->clipped;
  out_host->skipped = p->h_result->skipped;
  return RG_OK;
}

RG_API int rg_read_tensor_norms(rg_plan* p, float* out_host, void* stream) {
  if (p == nullptr || (p->n_tensors > 0 && out_host == nullptr)) {
    set_error("rg_read_tensor_norms: null argument");
    return RG_EINVAL;
  }
  if (p->n_tensors == 0) return RG_OK;
  DeviceGuard guard(p->device);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  RG_HIP(hipMemcpyAsync(p->h_norms, p->d_tensor_norm, (size_t)p->n_tensors * sizeof(float), hipMemcpyDeviceToHost, s));
  RG_HIP(hipStreamSynchronize(s));
  memcpy(out_host, p->h_norms, (size_t)p->n_tensors * sizeof(float));
  return RG_OK;
}

// ---------------------------------------------------------------------------- timing

RG_API int rg_plan_enable_timing(rg_plan* p, int slots) {
  // slots < 0: bracket only the write pass (the dominant kernel) in |slots| slots
  const bool all = slots >= 0;
  if (slots < 0) slots = -slots;
  if (p != nullptr) p->timing_all = all;
  if (p == nullptr || slots < 0 || slots > 65536) {
    set_error("rg_plan_enable_timing: bad arguments");
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  for (hipEvent_t e : p->timing_events) (void)hipEventDestroy(e);
  p->timing_events.clear();
  p->timing_slots = 0;
  p->timing_count = 0;
  p->timing_steps = 0;
  p->timing_events.reserve((size_t)slots * 4);
  for (int i = 0; i < slots * 4; ++i) {
    hipEvent_t e;
    RG_HIP(hipEventCreate(&e));
    p->timing_events.push_back(e);
  }
  p->timing_slots = slots;
  return RG_OK;
}

RG_API int rg_plan_timing_stride(rg_plan* p, int stride) {
  if (p == nullptr || stride < 1) {
    set_error("rg_plan_timing_stride: bad arguments");
    return RG_EINVAL;
  }
  p->timing_stride = stride;
  p->timing_steps = 0;
  return RG_OK;
}

RG_API int rg_plan_read_timing(rg_plan* p, int slot, float ms[4]) {
  if (p == nullptr || ms == nullptr || slot < 0 || slot >= p->timing_slots || (int64_t)slot >= p->timing_count) {
    set_error("rg_plan_read_timing: no timing recorded in slot %d", slot);
    return RG_EINVAL;
  }
  DeviceGuard guard(p->device);
  hipEvent_t* ev = &p->timing_events[(size_t)slot * 4];
  RG_HIP(hipEventSynchronize(ev[3]));
  ms[0] = ms[1] = ms[3] = -1.0f;
  if (p->timing_all) {
    RG_HIP(hipEventElapsedTime(&ms[0], ev[0], ev[1]));
    RG_HIP(hipEventElapsedTime(&ms[1], ev[1], ev[2]));
    RG_HIP(hipEventElapsedTime(&ms[3], ev[0], ev[3]));
  }
  RG_HIP(hipEventElapsedTime(&ms[2], ev[2], ev[3]));
  return RG_OK;
}
