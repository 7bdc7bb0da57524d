/* The C ABI of libranncgrad driven from plain C99, with nothing but the HIP runtime for device memory:
 * the way a caller that is not Python (the reference's C++ ParamStorage, or any other host) would use it.
 *
 * Built by rannc_amd/build.py into tests/abi_driver; tests/test_gpu_c_abi.py runs it on the GPU and checks
 * that it prints "abi_driver: OK".  Expected values are computed here on the host from first principles:
 * bf16 inputs that are exact multiples of 1/8, a power-of-two loss scale (the unscale is exact), the norm
 * summed in double, and the clipped value as one fp32 multiply by the coefficient the library reports.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "ranncgrad.h"

#define CHECK_HIP(x)                                                                     \
  do {                                                                                   \
    hipError_t e_ = (x);                                                                 \
    if (e_ != hipSuccess) {                                                              \
      printf("abi_driver: HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);  \
      return 2;                                                                          \
    }                                                                                    \
  } while (0)
#define CHECK_RG(x)                                                                      \
  do {                                                                                   \
    int rc_ = (x);                                                                       \
    if (rc_ != RG_OK) {                                                                  \
      printf("abi_driver: %s -> %d (%s) at line %d\n", #x, rc_, rg_last_error(), __LINE__); \
      return 3;                                                                          \
    }                                                                                    \
  } while (0)
#define EXPECT(cond)                                                                     \
  do {                                                                                   \
    if (!(cond)) {                                                                       \
      printf("abi_driver: expectation failed at line %d: %s\n", __LINE__, #cond);        \
      return 4;                                                                          \
    }                                                                                    \
  } while (0)

static uint16_t bf16_bits(float f) { /* exact for the values used here (low 16 bits are zero) */
  uint32_t u;
  memcpy(&u, &f, 4);
  return (uint16_t)(u >> 16);
}

static float value_at(int64_t tensor, int64_t i) { /* multiples of 1/8 in [-15.875, 15.875] */
  return (float)((int)((i * 37 + tensor * 11) % 255) - 127) * 0.125f;
}

static int same_bits(const float* a, const float* b, int64_t n) {
  return memcmp(a, b, (size_t)n * sizeof(float)) == 0;
}

int main(void) {
  enum { kTensors = 3 };
  const int64_t numel[kTensors] = {100003, 1, 40960};
  const float scale = 64.0f, inv_scale = 1.0f / 64.0f, max_norm = 1.0f;
  int64_t total = 0, t, i;
  int device = 0;

  EXPECT(rg_version() >= 1);
  for (t = 0; t < kTensors; ++t) total += numel[t];

  /* host data: scaled bf16 gradients, the fp32 bucket they are packed into */
  uint16_t* h_src = (uint16_t*)malloc((size_t)total * 2);
  float* h_want = (float*)malloc((size_t)total * 4);
  float* h_got = (float*)malloc((size_t)total * 4);
  EXPECT(h_src && h_want && h_got);
  double sumsq_total = 0.0;
  {
    int64_t off = 0;
    for (t = 0; t < kTensors; ++t) {
      double s = 0.0;
      for (i = 0; i < numel[t]; ++i) {
        const float x = value_at(t, i) * scale; /* exact */
        h_src[off + i] = bf16_bits(x);
        const float v = x * inv_scale; /* exact */
        h_want[off + i] = v;
        s += (double)v * (double)v;
      }
      /* the reference rounds every tensor's norm to float before squaring it again (ParamStorage.cpp:769-770, 809-817) */
      const float n_t = (float)sqrt(s);
      sumsq_total += (double)n_t * (double)n_t;
      off += numel[t];
    }
  }
  const double norm = sqrt(sumsq_total);
  const double g = norm + 1e-6;
  EXPECT(g > (double)max_norm);

  CHECK_HIP(hipSetDevice(device));
  char *d_src = NULL, *d_dst = NULL;
  CHECK_HIP(hipMalloc((void**)&d_src, (size_t)total * 2));
  CHECK_HIP(hipMalloc((void**)&d_dst, (size_t)total * 4));
  CHECK_HIP(hipMemcpy(d_src, h_src, (size_t)total * 2, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemset(d_dst, 0x7f, (size_t)total * 4));

  /* ---- a plan over the three tensors, the fused step, the decision read back */
  const void* src[kTensors];
  void* dst[kTensors];
  int sdt[kTensors], ddt[kTensors];
  {
    int64_t off = 0;
    for (t = 0; t < kTensors; ++t) {
      src[t] = d_src + off * 2;
      dst[t] = d_dst + off * 4;
      sdt[t] = RG_BF16;
      ddt[t] = RG_F32;
      off += numel[t];
    }
  }
  rg_plan* plan = NULL;
  CHECK_RG(rg_plan_create(&plan, device, kTensors, src, dst, numel, sdt, ddt, 0));
  EXPECT(rg_plan_num_tensors(plan) == kTensors && rg_plan_total_numel(plan) == total);
  CHECK_RG(rg_fused_step(plan, inv_scale, max_norm, RG_STEP_DEFAULT, NULL));
  rg_step_result res;
  CHECK_RG(rg_read_result(plan, &res, NULL));
  EXPECT(res.overflow == 0 && res.skipped == 0 && res.clipped == 1);
  EXPECT(fabs(res.norm - norm) <= 1e-6 * norm);
  EXPECT(fabs((double)res.coef - (double)max_norm / g) <= 1e-6 * ((double)max_norm / g));
  CHECK_HIP(hipMemcpy(h_got, d_dst, (size_t)total * 4, hipMemcpyDeviceToHost));
  {
    volatile float coef = res.coef; /* one rounding per element, no contraction with the multiply above */
    for (i = 0; i < total; ++i) h_want[i] = h_want[i] * coef;
  }
  EXPECT(same_bits(h_got, h_want, total));

  /* ---- the allocation-free entry point on the largest tensor: same bits as a one-tensor plan */
  {
    rg_plan* one = NULL;
    const void* s1[1] = {src[0]};
    void* d1[1] = {dst[0]};
    rg_step_result r_plan, r_static, *d_res = NULL;
    float* h_a = (float*)malloc((size_t)numel[0] * 4);
    float* h_b = (float*)malloc((size_t)numel[0] * 4);
    EXPECT(h_a && h_b);
    CHECK_RG(rg_plan_create(&one, device, 1, s1, d1, numel, sdt, ddt, 0));
    CHECK_RG(rg_fused_step(one, inv_scale, max_norm, RG_STEP_DEFAULT, NULL));
    CHECK_RG(rg_read_result(one, &r_plan, NULL));
    CHECK_HIP(hipMemcpy(h_a, dst[0], (size_t)numel[0] * 4, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemset(dst[0], 0, (size_t)numel[0] * 4));
    CHECK_HIP(hipMalloc((void**)&d_res, sizeof(rg_step_result)));
    CHECK_RG(rg_fused_step_static(src[0], dst[0], numel[0], RG_BF16, RG_F32, inv_scale, max_norm, RG_STEP_DEFAULT, d_res,
                                  device, NULL));
    CHECK_HIP(hipDeviceSynchronize());
    CHECK_HIP(hipMemcpy(&r_static, d_res, sizeof(r_static), hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(h_b, dst[0], (size_t)numel[0] * 4, hipMemcpyDeviceToHost));
    EXPECT(r_static.norm == r_plan.norm && r_static.coef == r_plan.coef && r_static.clipped == r_plan.clipped &&
           r_static.overflow == 0);
    EXPECT(same_bits(h_a, h_b, numel[0]));
    CHECK_RG(rg_plan_destroy(one));
    CHECK_HIP(hipFree(d_res));
    free(h_a);
    free(h_b);
  }

  /* ---- an inf in the gradients: flagged, the step skipped, the bucket left as it was */
  {
    const uint16_t inf_bits = 0x7f80;
    CHECK_HIP(hipMemcpy(d_src + 2 * 77777, &inf_bits, 2, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemset(d_dst, 0x11, (size_t)total * 4));
    CHECK_RG(rg_fused_step(plan, inv_scale, max_norm, RG_STEP_DEFAULT, NULL));
    CHECK_RG(rg_read_result(plan, &res, NULL));
    EXPECT(res.overflow == 1 && res.skipped == 1 && res.clipped == 0);
    CHECK_HIP(hipMemcpy(h_got, d_dst, (size_t)total * 4, hipMemcpyDeviceToHost));
    for (i = 0; i < total; ++i) {
      uint32_t u;
      memcpy(&u, &h_got[i], 4);
      EXPECT(u == 0x11111111u);
    }
    CHECK_HIP(hipMemcpy(d_src + 2 * 77777, &h_src[77777], 2, hipMemcpyHostToDevice));
  }

  /* ---- the loss scale on the device: the unscale reads 1/scale from the scaler's state, the schedule follows the
   *      result block - a clean step counts (window 2: the second one doubles the scale), an overflow halves it */
  {
    rg_scaler_state init, st, *d_state = NULL;
    const rg_step_result* d_result = NULL;
    memset(&init, 0, sizeof(init));
    init.loss_scale = scale; /* 64: the gradients above carry exactly this scale */
    init.max_loss_scale = 256.0f;
    init.scale_window = 2;
    init.scale_factor = 2.0f;
    CHECK_HIP(hipMalloc((void**)&d_state, sizeof(rg_scaler_state)));
    CHECK_RG(rg_scaler_init(d_state, &init, device, NULL));
    CHECK_RG(rg_result_device_ptr(plan, &d_result));
    CHECK_HIP(hipMemset(d_dst, 0x22, (size_t)total * 4));
    CHECK_RG(rg_step_begin_scaled(plan, &d_state->inv_scale, NULL));
    CHECK_RG(rg_step_finish(plan, max_norm, RG_STEP_DEFAULT, NULL));
    CHECK_RG(rg_scaler_update(d_state, d_result, RG_SCALER_DYNAMIC | RG_SCALER_TRUNCATE, device, NULL));
    CHECK_RG(rg_read_result(plan, &res, NULL));
    EXPECT(res.overflow == 0 && res.clipped == 1 && fabs(res.norm - norm) <= 1e-6 * norm);
    CHECK_HIP(hipMemcpy(h_got, d_dst, (size_t)total * 4, hipMemcpyDeviceToHost));
    EXPECT(same_bits(h_got, h_want, total)); /* the same bits as with the scale passed by value */
    CHECK_HIP(hipMemcpy(&st, d_state, sizeof(st), hipMemcpyDeviceToHost));
    EXPECT(st.loss_scale == 64.0f && st.inv_scale == 1.0f / 64.0f && st.unskipped == 1 && st.skipped_steps == 0);
    /* second clean step: the window is reached, the scale doubles */
    CHECK_RG(rg_step_begin_scaled(plan, &d_state->inv_scale, NULL));
    CHECK_RG(rg_step_decide(plan, max_norm, RG_STEP_DEFAULT, NULL));
    CHECK_RG(rg_scaler_update(d_state, d_result, RG_SCALER_DYNAMIC | RG_SCALER_TRUNCATE, device, NULL));
    CHECK_HIP(hipDeviceSynchronize());
    CHECK_HIP(hipMemcpy(&st, d_state, sizeof(st), hipMemcpyDeviceToHost));
    EXPECT(st.loss_scale == 128.0f && st.inv_scale == 1.0f / 128.0f && st.unskipped == 0);
    /* an inf: flagged with the new scale in use, the step skipped, the scale halved */
    {
      const uint16_t inf_bits = 0xff80; /* -inf */
      CHECK_HIP(hipMemcpy(d_src + 2 * 5, &inf_bits, 2, hipMemcpyHostToDevice));
      CHECK_RG(rg_step_begin_scaled(plan, &d_state->inv_scale, NULL));
      CHECK_RG(rg_step_decide(plan, max_norm, RG_STEP_DEFAULT, NULL));
      CHECK_RG(rg_scaler_update(d_state, d_result, RG_SCALER_DYNAMIC | RG_SCALER_TRUNCATE, device, NULL));
      CHECK_RG(rg_read_result(plan, &res, NULL));
      EXPECT(res.overflow == 1 && res.skipped == 1);
      CHECK_HIP(hipMemcpy(&st, d_state, sizeof(st), hipMemcpyDeviceToHost));
      EXPECT(st.loss_scale == 64.0f && st.unskipped == 0 && st.skipped_steps == 1);
      CHECK_HIP(hipMemcpy(d_src + 2 * 5, &h_src[5], 2, hipMemcpyHostToDevice));
    }
    EXPECT(rg_scaler_update(d_state, NULL, RG_SCALER_DYNAMIC, device, NULL) == RG_EINVAL);
    EXPECT(rg_scaler_update(d_state, d_result, 64, device, NULL) == RG_EINVAL);
    CHECK_HIP(hipFree(d_state));
  }

  /* ---- segment layout and a cast copy (the ZeRO unflatten), then errors as status codes */
  {
    EXPECT(rg_aligned_numel(1000, 2, 8) == 1024);
    CHECK_RG(rg_scale_cast_single(d_src, d_dst, numel[0], RG_BF16, RG_F32, 1.0f, device, NULL));
    CHECK_HIP(hipDeviceSynchronize());
    CHECK_HIP(hipMemcpy(h_got, d_dst, (size_t)numel[0] * 4, hipMemcpyDeviceToHost));
    for (i = 0; i < numel[0]; ++i) EXPECT(h_got[i] == value_at(0, i) * scale);
    EXPECT(rg_fused_step(NULL, inv_scale, max_norm, RG_STEP_DEFAULT, NULL) == RG_EINVAL);
    EXPECT(strlen(rg_last_error()) > 0);
    EXPECT(rg_scale_cast_single(d_src + 1, d_dst, 8, RG_BF16, RG_F32, 1.0f, device, NULL) == RG_EALIGN);
  }

  CHECK_RG(rg_plan_destroy(plan));
  CHECK_HIP(hipFree(d_src));
  CHECK_HIP(hipFree(d_dst));
  free(h_src);
  free(h_want);
  free(h_got);
  printf("abi_driver: OK\n");
  return 0;
}
