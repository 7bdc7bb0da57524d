// Shared by the translation units of the pybind11 module rannc_amd._ranncgrad: status codes to
// Python exceptions, tensor -> (pointer, element count, dtype code), the current stream, and
// PairPlan - a device table over explicit (source, destination) tensor pairs that is rebuilt
// only when the pairs change shape and re-pointed when they only move.
#pragma once

#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <stdexcept>
#include <string>
#include <vector>

#include "ranncgrad.h"

namespace py = pybind11;

namespace rgbind {

inline void check(int rc) {
  if (rc == RG_OK) return;
  const std::string msg = rg_last_error();
  if (rc == RG_EINVAL || rc == RG_EALIGN) throw std::invalid_argument(msg);
  if (rc == RG_ENOMEM) throw std::bad_alloc();
  throw std::runtime_error(msg);
}

// The reference admits float, half and bfloat16 only (assert at src/comp/ParamStorage.cpp:51-53).
inline int dtype_code(const at::Tensor& t) {
  switch (t.scalar_type()) {
    case at::kFloat: return RG_F32;
    case at::kHalf: return RG_F16;
    case at::kBFloat16: return RG_BF16;
    default:
      throw std::invalid_argument(std::string("unsupported dtype ") + c10::toString(t.scalar_type()) +
                                  ": expected float32, float16 or bfloat16");
  }
}

// hipStream_t of PyTorch's current stream on `device`, asked of PyTorch's own stream registry (what
// torch.cuda.current_stream(device).cuda_stream reads, without the trip through Python).
inline void* current_stream(int device) {
  return reinterpret_cast<void*>(c10::hip::getCurrentHIPStream((c10::DeviceIndex)device).stream());
}

inline void require_gpu_contiguous(const at::Tensor& t, const char* what, size_t i) {
  if (!t.is_cuda()) throw std::invalid_argument(std::string(what) + "[" + std::to_string(i) + "] is not on a GPU");
  if (!t.is_contiguous()) throw std::invalid_argument(std::string(what) + "[" + std::to_string(i) + "] is not contiguous");
}

// A tensor from a Python object; None gives an undefined tensor.
inline at::Tensor tensor_or_undefined(const py::handle& o, const char* what) {
  if (o.is_none()) return at::Tensor();
  if (!THPVariable_Check(o.ptr())) throw std::invalid_argument(std::string(what) + " expects tensors");
  return THPVariable_Unpack(o.ptr());
}

inline std::vector<at::Tensor> tensor_vector(const py::handle& seq, const char* what) {
  std::vector<at::Tensor> out;
  if (seq.is_none()) return out;
  for (const py::handle& o : py::reinterpret_borrow<py::iterable>(seq)) out.push_back(tensor_or_undefined(o, what));
  return out;
}

// Device table over tensor pairs.  src[i] undefined = "no gradient" (reads as zeros); dst[i] undefined only for
// norm-only use.  bind() points the table at the pairs given: it is rebuilt when a size, dtype or the set of
// defined tensors differs from the last call, re-pointed (one stream-ordered upload) when only addresses moved.
class PairPlan {
 public:
  PairPlan() = default;
  ~PairPlan() { close(); }
  PairPlan(const PairPlan&) = delete;
  PairPlan& operator=(const PairPlan&) = delete;

  void close() {
    if (plan_ != nullptr) {
      rg_plan_destroy(plan_);
      plan_ = nullptr;
    }
  }
  bool open() const { return plan_ != nullptr; }
  int device() const { return device_; }
  int size() const { return (int)numel_.size(); }
  void* stream() const { return current_stream(device_); }
  rg_plan* get() {
    if (plan_ == nullptr) throw std::runtime_error("the plan is closed");
    return plan_;
  }

  // Returns true when the table had to be built anew.
  bool bind(const std::vector<at::Tensor>& srcs, const std::vector<at::Tensor>& dsts, int64_t chunk_elems = 0) {
    const size_t n = srcs.size();
    const bool has_dsts = !dsts.empty() || n == 0;
    if (has_dsts && dsts.size() != n) throw std::invalid_argument("srcs and dsts differ in length");
    std::vector<const void*> src(n, nullptr);
    std::vector<void*> dst(n, nullptr);
    std::vector<int64_t> numel(n, 0);
    std::vector<int> sdt(n, 0), ddt(n, 0);
    std::vector<char> defined(n, 0);
    int device = -1;
    for (size_t i = 0; i < n; ++i) {
      const at::Tensor& s = srcs[i];
      const at::Tensor d = has_dsts ? dsts[i] : at::Tensor();
      if (!s.defined() && !d.defined()) throw std::invalid_argument("pair " + std::to_string(i) + " has neither source nor destination");
      if (s.defined()) require_gpu_contiguous(s, "src", i);
      if (d.defined()) require_gpu_contiguous(d, "dst", i);
      if (s.defined() && d.defined() && s.numel() != d.numel())
        throw std::invalid_argument("pair " + std::to_string(i) + ": source and destination differ in element count");
      const at::Tensor& any = s.defined() ? s : d;
      if (device < 0) device = any.get_device();
      if ((s.defined() && s.get_device() != device) || (d.defined() && d.get_device() != device))
        throw std::invalid_argument("pair " + std::to_string(i) + " is on another device");
      numel[i] = any.numel();
      sdt[i] = dtype_code(s.defined() ? s : d);
      ddt[i] = dtype_code(d.defined() ? d : s);
      src[i] = s.defined() && numel[i] ? s.data_ptr() : nullptr;
      dst[i] = d.defined() && numel[i] ? d.data_ptr() : nullptr;
      defined[i] = (char)((s.defined() ? 1 : 0) | (d.defined() ? 2 : 0));
    }
    if (device < 0) device = 0;
    const bool same_shape = plan_ != nullptr && device == device_ && numel == numel_ && sdt == sdt_ && ddt == ddt_ &&
                            defined == defined_ && chunk_elems == chunk_elems_;
    if (same_shape) {
      const bool src_moved = src != src_, dst_moved = dst != dst_;
      if (src_moved || dst_moved) {
        check(rg_plan_update_pointers(plan_, src_moved ? src.data() : nullptr, dst_moved ? dst.data() : nullptr,
                                      current_stream(device_)));
        src_.swap(src);
        dst_.swap(dst);
      }
      return false;
    }
    close();
    device_ = device;
    check(rg_plan_create(&plan_, device_, (int)n, src.data(), dst.data(), numel.data(), sdt.data(), ddt.data(), chunk_elems));
    numel_.swap(numel);
    sdt_.swap(sdt);
    ddt_.swap(ddt);
    defined_.swap(defined);
    src_.swap(src);
    dst_.swap(dst);
    chunk_elems_ = chunk_elems;
    return true;
  }

  rg_step_result result() {
    rg_step_result r;
    check(rg_read_result(get(), &r, stream()));
    return r;
  }

 private:
  rg_plan* plan_ = nullptr;
  int device_ = 0;
  int64_t chunk_elems_ = 0;
  std::vector<int64_t> numel_;
  std::vector<int> sdt_, ddt_;
  std::vector<char> defined_;
  std::vector<const void*> src_;
  std::vector<void*> dst_;
};

inline py::dict result_dict(const rg_step_result& r) {
  py::dict d;
  d["norm"] = r.norm;
  d["coef"] = r.coef;
  d["overflow"] = r.overflow;
  d["clipped"] = r.clipped;
  d["skipped"] = r.skipped;
  return d;
}

}  // namespace rgbind

// defined in rg_registry.cpp: ParamStorage, RaNNCModule, TensorList and GradPlan of the module
void bind_registry(py::module_& m);
// a fresh, empty registry (what the module's clear() does besides forgetting the distributed parameters)
void reset_registry();
