/*
 * libranncgrad -- C ABI of the MI355X (gfx950) kernel library for the per-step
 * parameter/gradient path of RaNNC: pack gradients into buckets, loss-scale
 * unscale with an inf/NaN flag, global L2 norm + clip-by-norm, master-parameter
 * casts, and flat-buffer <-> segment copies.
 *
 * Conventions
 *  - every entry point returns an int status (RG_OK == 0); none throws;
 *    rg_last_error() gives the message of the calling thread's last failure;
 *  - pointers named *_dev / src / dst are device pointers owned by the caller and
 *    borrowed for the duration of the call (plans keep them until updated);
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *    all device work is enqueued on it and nothing synchronises with the host
 *    except rg_plan_create / rg_plan_destroy / rg_read_* ;
 *  - after rg_plan_create no entry point allocates device memory.
 *
 * The reference has no GPU kernels for this path: it issues one ATen op per
 * tensor from C++ loops.  Each declaration cites the reference code it replaces
 * (paths relative to the reference tree).
 */
#ifndef RANNCGRAD_H
#define RANNCGRAD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RG_VERSION 1

/* status codes */
enum {
  RG_OK = 0,
  RG_EINVAL = 1, /* bad argument (reference: std::invalid_argument -> ValueError) */
  RG_EALIGN = 2, /* pointer not aligned to its element size */
  RG_EHIP = 3,   /* a HIP runtime call failed (reference: std::runtime_error)  */
  RG_ENOMEM = 4
};

/* element types; the reference admits exactly these three
 * (assert at src/comp/ParamStorage.cpp:51-53) */
enum { RG_F32 = 0, RG_F16 = 1, RG_BF16 = 2 };

/* flags for rg_fused_step */
enum {
  RG_STEP_DEFAULT = 0,
  /* On overflow still write the unscaled (unclipped) values, as Apex's
   * multi_tensor_scale does; by default the write pass is skipped because the
   * step is skipped and the gradients are discarded. */
  RG_STEP_WRITE_ON_OVERFLOW = 1,
  /* Report the flag but let it gate nothing: a non-finite norm then behaves exactly as in
   * ParamStorage::clipGradNorm (inf -> coef 0, NaN -> no clip; src/comp/ParamStorage.cpp:723-742).
   * This is what RaNNCModule.clip_grad_norm on existing gradients uses. */
  RG_STEP_IGNORE_OVERFLOW = 2,
  /* The caller expects that this step will not clip (its last one did not).  The step then
   * runs as ONE pass that writes the unscaled values while it sums them - (s + d) bytes per
   * element instead of (2s + d) - followed by the decision; only if the decision is "clip"
   * after all does a second kernel multiply the destination in place by the coefficient
   * ((s + 3d) bytes in that case).  Norm, flag, coefficient and every written bit are those
   * of the default strategy (the norm to rounding: its partial sums are taken per tile); on
   * overflow the destination holds the unscaled values (as with RG_STEP_WRITE_ON_OVERFLOW).
   * In place with inv_scale == 1 (clip_grad_norm on existing gradients) a step that does not
   * clip writes nothing under either strategy; the flag then only makes the gated second
   * kernel cheaper to find idle. */
  RG_STEP_EXPECT_NO_CLIP = 4
};

const char* rg_last_error(void);
int rg_version(void);
int rg_elem_size(int dtype); /* 4, 2, 2; -1 for an unknown dtype */

/* ---------------------------------------------------------------- layout (host only) */

/* calcAlignedNumElems, src/torch/TorchUtil.cpp:1579-1591: numel rounded up to a
 * multiple of (16 / elem_size) * split_num.  Returns -1 on bad arguments. */
int64_t rg_aligned_numel(int64_t numel, int elem_size, int split_num);

/* DistributedParamLocatorBase::doRegister, src/comp/DistributedParamLocatorBase.cpp:14-27.
 * offsets/src_sizes receive nranks entries each. */
int rg_segment_layout(int64_t numel, int elem_size, int nranks, int64_t* aligned_size,
                      int64_t* segment_size, int64_t* offsets, int64_t* src_sizes);

/* GradConsolidation constructor, src/comp/ParamStorage.cpp:48-57: element offset of
 * each tensor inside the bucket of its dtype (running sum, no padding).
 * bucket_lengths[3] is indexed by RG_F32 / RG_F16 / RG_BF16. */
int rg_bucket_layout(int n, const int64_t* numels, const int* dtypes, int64_t* offsets,
                     int64_t bucket_lengths[3]);

/* ---------------------------------------------------------------- plans */

/* A plan is a device-resident descriptor table: n tensors, each with a source
 * pointer, a destination pointer, an element count and the two element types,
 * cut into fixed-size chunks so that one launch covers all of them.  It replaces
 * the reference's host loops over parameters (`for (long pid : param_ids_)`,
 * src/comp/ParamStorage.cpp:135, 470, 726, 755).
 *
 * src[i] == NULL means "tensor i has no gradient": it reads as zeros
 * (src/comp/ParamStorage.cpp:169-175).  dst[i] may be NULL only for plans that
 * are used with rg_grad_norm alone.  dst[i] == src[i] (same dtype) is allowed:
 * every op is then in place. */
typedef struct rg_plan rg_plan;

/* chunk_elems: elements per work chunk (multiple of 2048, at most 2^20), 0 = choose from the
 * total size. */
int rg_plan_create(rg_plan** out, int device, int n, const void* const* src, void* const* dst,
                   const int64_t* numel, const int* src_dtype, const int* dst_dtype,
                   int64_t chunk_elems);
/* Replace the pointers (either array may be NULL = keep); stream ordered. */
int rg_plan_update_pointers(rg_plan* plan, const void* const* src, void* const* dst, void* stream);
int rg_plan_destroy(rg_plan* plan);
int rg_plan_num_tensors(const rg_plan* plan);
int64_t rg_plan_num_chunks(const rg_plan* plan);
int64_t rg_plan_chunk_elems(const rg_plan* plan);
int64_t rg_plan_total_numel(const rg_plan* plan);
/* Cache policy of the plan's kernels: 1 = nontemporal loads and stores (the data is streamed
 * once and is far larger than the caches), 0 = plain accesses (the second pass of a small
 * plan then hits in cache), -1 = decide from the plan's size (the default). */
int rg_plan_set_streaming(rg_plan* plan, int mode);

/* Optional: choose the order in which the plan's writing passes hand their tiles to the GPU's eight XCDs by
 * measuring it.  Runs the pass `dst = round_dst(float(src))` (what rg_scale_cast(plan, 1.0) writes) a few times
 * under each order the library knows (three interleaved rounds), on the plan's own tensors and on `stream`, waits
 * for them, and keeps the fastest for every later writing pass of this plan - the order in use is only given up
 * for one that is more than 1 % faster.  The destinations are overwritten, so call it where their
 * contents do not matter yet (right after creating the plan); in-place plans are left alone.  Results never
 * depend on the order - only the time does.  No counterpart in the reference (it has no kernels to tune).
 * rg_plan_write_order returns the order in use (0 = round robin, n > 0 = runs of n tiles per XCD, -1 = one
 * contiguous eighth per XCD). */
int rg_plan_tune(rg_plan* plan, void* stream);
int rg_plan_write_order(const rg_plan* plan);
/* Set that order directly (same encoding; RG_EINVAL outside [-1, 65536]): for a caller that has measured it on an
 * earlier plan of the same layout and must not have this plan's destinations overwritten by another measurement. */
int rg_plan_set_write_order(rg_plan* plan, int order);

/* ---------------------------------------------------------------- per-step operations */

typedef struct rg_step_result {
  double norm;      /* global L2 norm, as calc_grad_norm returns it (double) */
  float coef;       /* float(max_norm / (norm + 1e-6)) when clipped, else 1 */
  int32_t overflow; /* 1 iff any source element was +-inf or NaN */
  int32_t clipped;  /* 1 iff the clip multiply was applied */
  int32_t skipped;  /* 1 iff overflow gated the step (no clip; write pass skipped unless
                       RG_STEP_WRITE_ON_OVERFLOW) */
} rg_step_result;

/* The fused step, all on the stream, no host round trip:
 *   pass 1  read src: v = round_dst(float(x) * inv_scale); per-tensor sum v^2; inf/NaN flag
 *   final   n_t = float(sqrt(sum_t)); norm = sqrt(sum_t double(n_t)^2) in table order;
 *           g = norm + 1e-6; clipped = (g > max_norm) && !skipped; coef = float(max_norm / g)
 *   pass 2  re-read src, write dst = clipped ? round_dst(v * coef) : v
 * Replaces: Apex multi_tensor_scale (unscale + overflow flag; caller test/common.py:98-101),
 * GradConsolidation::consolidate copy_ (src/comp/ParamStorage.cpp:159-167),
 * ParamStorage::calcGradGlobalL2Norm (:747-819) and ParamStorage::clipGradNorm (:721-745).
 * With dst == src and inv_scale == 1 it is exactly clip_grad_norm on existing gradients
 * (RaNNCModule.clip_grad_norm, src/main.cpp:339-342).
 * max_norm <= 0 disables clipping (dst = v). */
int rg_fused_step(rg_plan* plan, float inv_scale, float max_norm, int flags, void* stream);

/* The same step in two calls, for callers that must look at the overflow flag in between
 * (the amp context exit updates the loss scale before the user asks for clipping:
 * pyrannc/amp/__init__.py:44-65 runs at scale_loss exit, RaNNCModule.clip_grad_norm later).
 * rg_step_begin  = pass 1 + norm/flag (result.coef = 1, clipped = 0);
 * rg_step_finish = clip decision for max_norm from the sums pass 1 left on the device, then
 *                  pass 2 with the inv_scale given to rg_step_begin.
 * Together they move exactly the bytes of rg_fused_step. */
int rg_step_begin(rg_plan* plan, float inv_scale, void* stream);
int rg_step_finish(rg_plan* plan, float max_norm, int flags, void* stream);
/* The clip decision alone: from the sums rg_step_begin left on the device, fills coef /
 * clipped / skipped of the result block for max_norm and launches no pass over the
 * gradients.  For callers whose next kernel consumes the decision on the device - the
 * optimizer step below with `gate`, reading the still-scaled gradients with grad_scale =
 * inv_scale - so that the unscaled, clipped gradients are never written to memory at all.
 * The begin stays pending: rg_step_finish may still be called to write them. */
int rg_step_decide(rg_plan* plan, float max_norm, int flags, void* stream);

/* One pass: dst = round_dst(float(x) * inv_scale), overflow flag and norm as above, no
 * clip.  Apex multi_tensor_scale semantics (LossScaler.unscale). */
int rg_unscale_pack(rg_plan* plan, float inv_scale, void* stream);

/* Clip after the fact: from the sums the last rg_unscale_pack / rg_unscale_accumulate on this plan left on
 * the device, the clip decision for max_norm (as rg_fused_step takes it), and - only if it says "clip" - an
 * in-place multiply of the destinations by the coefficient.  rg_unscale_pack + rg_step_apply_clip write the
 * bits of rg_fused_step and move (s + d) bytes per element when the step does not clip, (s + 3d) when it
 * does; the multiply's blocks cover whole chunks, so a launch that finds nothing to do costs microseconds.
 * ParamStorage::clipGradNorm (src/comp/ParamStorage.cpp:721-745) on gradients whose norm is already known.
 * RG_EINVAL unless the plan's last operation was one of the two named above. */
int rg_step_apply_clip(rg_plan* plan, float max_norm, int flags, void* stream);

/* Accumulating forms, for gradient accumulation over several backward passes:
 *   rg_accumulate:          dst = round_dst(float(dst) + float(src) * scale)
 *   rg_unscale_accumulate:  the same with scale = inv_scale, plus the inf/NaN flag of the sources
 *                           and the norm of the RESULT, as rg_unscale_pack reports them.
 * The product is rounded to fp32 before the sum (two roundings, `master.add_(model.float() *
 * inv_scale)`).  This is Apex's unscale_with_stashed / multi_tensor_axpby (external to the
 * reference; whether Apex's kernel contracts the two operations into one fma is not visible
 * from the reference tree, so bit parity with Apex is not claimed for this entry point).
 * Missing sources (NULL) add nothing.  dst must differ from src. */
int rg_accumulate(rg_plan* plan, float scale, void* stream);
int rg_unscale_accumulate(rg_plan* plan, float inv_scale, void* stream);

/* Read-only: per-tensor and global L2 norm of the SOURCE tensors and their inf/NaN flag.
 * ParamStorage::calcGradGlobalL2Norm, src/comp/ParamStorage.cpp:747-819
 * (RaNNCModule.calc_grad_norm, src/main.cpp:344-345). */
int rg_grad_norm(rg_plan* plan, void* stream);

/* dst = round_dst(float(src) * scale).  scale == 1 with equal dtypes is a raw copy.
 * Replaces per-tensor copy_/to/mul_: src/comp/ParamStorage.cpp:165, 493, 424-426, 609-611,
 * src/comp/DistributedParamLocator.cpp:33-34, 62-65, 76,
 * src/comp/DistributedGradLocator.cpp:59, DistributedParamLocatorBase.cpp:130-131,
 * and Apex's master<->model copies. */
int rg_scale_cast(rg_plan* plan, float scale, void* stream);

/* The same for ONE tensor, without a plan and without any allocation (src_dev == NULL
 * stores zeros): the one-off copies of DistributedParamLocator::store / set / setScalarType
 * (src/comp/DistributedParamLocator.cpp:14-83) and of gather's padded send buffer
 * (src/comp/DistributedParamLocatorBase.cpp:124-131). */
int rg_scale_cast_single(const void* src_dev, void* dst_dev, int64_t numel, int src_dtype, int dst_dtype,
                         float scale, int device, void* stream);

/* dst = 0 for every tensor.  ParamStorage::clearParamGrads, src/comp/ParamStorage.cpp:540-557.
 * Destinations that follow each other back to back in plan order (the views of a bucket) are cleared as one flat range,
 * as rg_fill_zero would; scattered ones through the plan's table. */
int rg_zero(rg_plan* plan, void* stream);

/* Fill `nbytes` bytes at dst_dev with zero (bucket / staging clears:
 * torch::zeros at src/torch/TorchUtil.cpp:1474, src/comp/ParamStorage.cpp:59-75). */
int rg_fill_zero(void* dst_dev, int64_t nbytes, int device, void* stream);

/* Results of the last rg_fused_step / rg_unscale_pack / rg_grad_norm on this plan. */
int rg_result_device_ptr(const rg_plan* plan, const rg_step_result** out_dev);
int rg_tensor_norms_device_ptr(const rg_plan* plan, const float** out_dev);
/* These two wait for the stream, then copy to host memory. */
int rg_read_result(rg_plan* plan, rg_step_result* out_host, void* stream);
int rg_read_tensor_norms(rg_plan* plan, float* out_host, void* stream);

/* The fused step of rg_fused_step for ONE tensor pair, without a plan and without allocating
 * anything.  It has no counterpart in the reference; it is for callers that cannot call
 * hipMalloc or rg_plan_create: code under HIP graph capture, tight serving loops, harnesses
 * that forbid allocation.  The working memory a plan would own (result block, per-chunk
 * partial sums) is a fixed array of about 4 MiB in the library's device image, one copy per
 * GPU, held until the process ends.  Limit: RG_STATIC_MAX_SRC_BYTES of source, i.e. 2^32
 * elements of fp16 / bf16 or 2^31 of fp32 (a chunk is 32 KiB of source whatever the type);
 * more is rejected with RG_EINVAL.  The kernels overwrite every slot they later read, so
 * nothing needs clearing between calls; calls that overlap on one GPU (two streams, two
 * threads) race on that array and must be serialised by the caller.  Same arithmetic, same
 * chunking and launch shapes and therefore the same bits as rg_fused_step on a one-tensor
 * plan; `result_dev` (device memory of the caller, 8-byte aligned, may be NULL) receives the
 * rg_step_result on the stream. */
#define RG_STATIC_MAX_SRC_BYTES 8589934592LL /* 2^33 */
#define RG_STATIC_MAX_NUMEL 4294967296LL     /* 2^32 elements of a 16-bit source type */
int rg_fused_step_static(const void* src_dev, void* dst_dev, int64_t numel, int src_dtype, int dst_dtype,
                         float inv_scale, float max_norm, int flags, rg_step_result* result_dev, int device,
                         void* stream);

/* ---------------------------------------------------------------- optimizer step */

/* Multi-tensor optimizer step on fp32 parameters, the step that follows the clip: the
 * reference leaves it to torch.optim (Adam at test/common.py:142,165, SGD at
 * examples/tutorial.py:28) on the parameters pyrannc/opt.py:205-312 hands it, and under amp
 * Apex then copies every fp32 master back into its fp16 model parameter
 * (pyrannc/amp/__init__.py:10-18 keeps the pairing).  One launch updates every tensor of
 * the table and, where `model_copy[i]` is given, writes round(param) there in the copy's
 * dtype - the master -> model copy-back without a second pass.
 *
 * Table: param, state1, state2 are fp32 and updated in place; grad has dtype grad_dtype[i]
 * (RG_F32 for master gradients); model_copy[i] may be NULL.  All tensors of a table share
 * the hyper-parameters and the step count of a call; a parameter without a gradient is
 * left out of the table (torch.optim skips it).  Adam: state1 = exp_avg, state2 =
 * exp_avg_sq.  SGD: state1 = momentum buffer (NULL array when momentum == 0), state2 unused. */
typedef struct rg_optim rg_optim;
int rg_optim_create(rg_optim** out, int device, int n_tensors, void* const* param, const void* const* grad,
                    void* const* state1, void* const* state2, void* const* model_copy, const int64_t* numel,
                    const int* grad_dtype, const int* copy_dtype);
/* New addresses, same sizes and dtypes; a NULL array keeps the current pointers. */
int rg_optim_update_pointers(rg_optim* opt, void* const* param, const void* const* grad, void* const* state1,
                             void* const* state2, void* const* model_copy, void* stream);
int rg_optim_destroy(rg_optim* opt);

/* Arithmetic of torch.optim.Adam / AdamW (single-tensor form, amsgrad off), in fp32 with
 * the scalar factors computed in double and rounded once, as ATen does with Python scalars:
 *   g  = grad * grad_scale            (then * gate->coef, a second multiply, exactly what rg_step_finish
 *                                      would have stored; the whole step is skipped when gate->skipped)
 *   g  = -g                           if maximize
 *   p  = p * (1 - lr * wd)            if decoupled_weight_decay (AdamW), else g = g + wd * p
 *   m  = m + (1 - beta1) * (g - m)
 *   v  = v * beta2 + (1 - beta2) * g * g
 *   p  = p + (-lr / (1 - beta1^step)) * m / (sqrt(v) / sqrt(1 - beta2^step) + eps)
 * `step` counts from 1.  `gate` (optional, device pointer from rg_result_device_ptr) lets the
 * clip coefficient and the overflow skip of a preceding rg_unscale_pack / rg_step_begin be
 * consumed on the device.  Results agree with torch.optim to rounding (ATen's own CPU and GPU
 * kernels differ from each other in the last bit); the model copy is bit-exact round-to-
 * nearest-even of the updated fp32 parameter. */
typedef struct rg_adam_args {
  double lr, beta1, beta2, eps, weight_decay;
  int64_t step;
  int32_t decoupled_weight_decay;
  int32_t maximize;
  float grad_scale;
  const rg_step_result* gate;
} rg_adam_args;
int rg_adam_step(rg_optim* opt, const rg_adam_args* args, void* stream);

/* The same step with its step count on the device, for callers that record the optimizer phase in a HIP graph
 * (a count passed by value would be frozen into the graph).  No counterpart in the reference, whose optimizer is
 * torch.optim's; torch's own graph-capturable Adam keeps `step` on the device in the same way.
 * An rg_adam_clock is 32 bytes of device memory owned by the caller (one per parameter group), zeroed before
 * the first step.  rg_adam_clock_advance launches one thread that adds 1 to `step` and stores the two factors
 * that depend on it, -lr / (1 - beta1^step) and sqrt(1 - beta2^step), computed in double as rg_adam_step
 * computes them on the host - unless `gate` (optional) says the step was skipped, in which case nothing
 * changes.  rg_adam_step_clocked is rg_adam_step reading those factors from the clock; args->step is ignored.
 * Call order on one stream: [rg_fused_step | rg_step_begin ...] -> rg_adam_clock_advance -> rg_adam_step_clocked. */
typedef struct rg_adam_clock {
  int64_t step;        /* steps taken so far */
  float neg_step_size; /* -lr / (1 - beta1^step) */
  float bias2_sqrt;    /* sqrt(1 - beta2^step) */
  float step_f32;      /* `step` again as a float (the form torch keeps state["step"] in) */
  int32_t pad[3];
} rg_adam_clock;
int rg_adam_clock_advance(rg_adam_clock* clock_dev, double lr, double beta1, double beta2, const rg_step_result* gate,
                          int device, void* stream);
int rg_adam_step_clocked(rg_optim* opt, const rg_adam_args* args, const rg_adam_clock* clock_dev, void* stream);

/* Arithmetic of torch.optim.SGD:
 *   g = grad * grad_scale; g = -g if maximize; g = g + wd * p if wd != 0
 *   momentum != 0:  buf = g on the first step of a buffer (first_step), else
 *                   buf = momentum * buf + (1 - dampening) * g;
 *                   g = g + momentum * buf if nesterov, else g = buf
 *   p = p - lr * g */
typedef struct rg_sgd_args {
  double lr, momentum, dampening, weight_decay;
  int32_t nesterov;
  int32_t maximize;
  int32_t first_step;
  float grad_scale;
  const rg_step_result* gate;
} rg_sgd_args;
int rg_sgd_step(rg_optim* opt, const rg_sgd_args* args, void* stream);

/* ---------------------------------------------------------------- loss scale on the device */

/* The dynamic loss-scale schedule as a one-thread kernel, so that a mixed-precision step needs no host read:
 * the reference reads the overflow flag back every step and updates the scale on the host
 * (pyrannc/amp/__init__.py:44-65 around Apex's LossScaler.update_scale; Apex is pinned at
 * docker/ubuntu/runtime/Dockerfile:13).  An rg_scaler_state is 32 bytes of device memory owned by the caller.
 * rg_scaler_update applies, to the `overflow` flag of a plan's result block:
 *   overflow and RG_SCALER_DYNAMIC:  loss_scale /= 2, floored at min_loss_scale when that is > 0, then truncated
 *                                    to an integer under RG_SCALER_TRUNCATE (what the reference's all-reduce of
 *                                    int(loss_scale) leaves, :57-61); unskipped = 0; skipped_steps += 1
 *   otherwise:                       unskipped += 1
 *   unskipped == scale_window and RG_SCALER_DYNAMIC:  loss_scale = min(max_loss_scale, loss_scale * scale_factor);
 *                                    unskipped = 0
 * and stores inv_scale = float(1 / double(loss_scale)).  A static scale (no RG_SCALER_DYNAMIC) only counts.
 * rg_step_begin_scaled is rg_step_begin with inv_scale read from device memory (normally &state->inv_scale) by
 * the kernels; rg_step_finish / rg_step_decide follow it as they follow rg_step_begin.
 * rg_optim_set_grad_scale_source makes every later step of an optimizer table multiply the gradients by the float
 * at `grad_scale_dev` instead of args->grad_scale (NULL: back to the argument).
 * Order on one stream: rg_step_begin_scaled -> rg_step_decide / rg_step_finish -> [optimizer step, gated] ->
 * rg_scaler_update; the next rg_step_begin_scaled then reads the new inv_scale.  All of it can be recorded in
 * a HIP graph. */
typedef struct rg_scaler_state {
  float loss_scale;
  float inv_scale;        /* 1 / loss_scale, what the next unscale multiplies by */
  int32_t unskipped;      /* clean steps since the scale last changed */
  int32_t skipped_steps;  /* steps skipped so far */
  float min_loss_scale;   /* 0: no floor */
  float max_loss_scale;
  int32_t scale_window;
  float scale_factor;
} rg_scaler_state;
enum { RG_SCALER_DYNAMIC = 1, RG_SCALER_TRUNCATE = 2 };
/* Writes *init_host (inv_scale recomputed) into state_dev with a kernel on `stream`. */
int rg_scaler_init(rg_scaler_state* state_dev, const rg_scaler_state* init_host, int device, void* stream);
int rg_scaler_update(rg_scaler_state* state_dev, const rg_step_result* result_dev, int flags, int device, void* stream);
int rg_step_begin_scaled(rg_plan* plan, const float* inv_scale_dev, void* stream);
int rg_optim_set_grad_scale_source(rg_optim* opt, const float* grad_scale_dev);

/* ---------------------------------------------------------------- per-kernel timing */

/* Optional profiling aid (no counterpart in the reference, which times with its own
 * TimeCounter around whole calls, src/comp/TimeCounter.cpp:10-27).  With `slots` > 0 every
 * rg_fused_step records HIP events on its stream around its three kernels into the next
 * slot of a ring; slots == 0 switches it off.  rg_plan_read_timing waits for that slot and
 * returns milliseconds: ms[0] reduce pass, ms[1] reduce + decide (the partial sums, the decision), ms[2] write pass, ms[3] whole step.
 * slot counts fused steps since timing was enabled, modulo `slots`.
 * A negative `slots` brackets only the write pass (two records per step instead of four, for
 * measurements where the records' own cost matters); ms[0], ms[1], ms[3] then read -1.
 * rg_plan_timing_stride(plan, k) brackets only every k-th step (slot = bracketed steps modulo
 * `slots`): each event record costs a few microseconds of stream time, so sampling keeps a
 * measurement loop close to the untimed one. */
int rg_plan_enable_timing(rg_plan* plan, int slots);
int rg_plan_timing_stride(rg_plan* plan, int stride);
int rg_plan_read_timing(rg_plan* plan, int slot, float ms[4]);

/* Yardstick kernels (no counterpart in the reference): the access patterns of the passes above over flat arrays -
 * no work table, no tensor boundaries, no sums - with the library's own load / store helpers and launch shapes, so
 * that a pass can be compared with what its pattern reaches on the same GPU in the same run.  One launch on `stream`.
 * `nbytes` (a multiple of 16) is the size of the widest stream; every array must be 16-byte aligned.
 *   kind 0  read only             arrays: src[nbytes], sink[>= 4 bytes, never written in practice]
 *   kind 1  fill (write only)     arrays: dst[nbytes]
 *   kind 2  fp32 copy * 1.5       arrays: src[nbytes], dst[nbytes]
 *   kind 3  bf16 -> fp32 * 0.5    arrays: src[nbytes / 2], dst[nbytes]
 *   kind 4  Adam's streams        arrays: p, g, m, v [nbytes each]; p, m, v rewritten in place
 *   kind 5  kind 2 with the compiler's plain nontemporal stores instead of the write passes' cache policy
 *   kind 6  kind 4 + a bf16 copy  arrays: p, g, m, v [nbytes each], copy[nbytes / 2] written (the step under mixed precision)
 *   kind 7  kind 6 in the optimizer step's launch shape (256 threads over 4096 elements, four vectors per array in flight)
 *   kind 8  kind 1 paced as rg_fill_zero paces a fill above 256 MiB (every wavefront waits 1.45 us before it stores) */
int rg_ceiling_kernel(int kind, void* const* arrays_dev, int n_arrays, int64_t nbytes, int device, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RANNCGRAD_H */
