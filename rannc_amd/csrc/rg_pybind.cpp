// pybind11 entry points over the C ABI of libranncgrad that accept PyTorch-ROCm tensors
// directly (module rannc_amd._ranncgrad).  The reference's boundary for this path is a
// pybind11 module too (PYBIND11_MODULE(_pyrannc), src/main.cpp:30); like it, this layer only
// converts arguments (tensor -> pointer, element count, dtype code, current stream) and
// translates status codes into Python exceptions: std::invalid_argument -> ValueError,
// std::runtime_error -> RuntimeError.  This file holds the table classes (Plan, Optim), the
// plan-free copy and the reference's free functions; rg_registry.cpp adds the native registry
// (TensorList, GradPlan, ParamStorage, RaNNCModule).
#include <pybind11/stl.h>

#include <unordered_map>

#include "rg_bind.h"

using rgbind::check;

namespace {

int dtype_code(const py::handle& tensor) {
  const std::string name = py::str(tensor.attr("dtype"));
  if (name == "torch.float32") return RG_F32;
  if (name == "torch.float16") return RG_F16;
  if (name == "torch.bfloat16") return RG_BF16;
  throw std::invalid_argument("unsupported dtype " + name + ": expected float32, float16 or bfloat16");
}

struct Ref {
  void* ptr = nullptr;
  int64_t numel = 0;
  int dtype = -1;
  int device = -1;
  bool defined = false;
};

Ref tensor_ref(const py::handle& t, const char* what, size_t i) {
  Ref r;
  if (t.is_none()) return r;
  if (!t.attr("is_cuda").cast<bool>())
    throw std::invalid_argument(std::string(what) + "[" + std::to_string(i) + "] is not on a GPU");
  if (!t.attr("is_contiguous")().cast<bool>())
    throw std::invalid_argument(std::string(what) + "[" + std::to_string(i) + "] is not contiguous");
  r.defined = true;
  r.numel = t.attr("numel")().cast<int64_t>();
  r.dtype = dtype_code(t);
  r.device = t.attr("device").attr("index").cast<int>();
  r.ptr = r.numel ? reinterpret_cast<void*>(t.attr("data_ptr")().cast<uintptr_t>()) : nullptr;
  return r;
}

using rgbind::current_stream;

struct Tables {
  std::vector<const void*> src;
  std::vector<void*> dst;
  std::vector<int64_t> numel;
  std::vector<int> sdt, ddt;
  int device = -1;
};

Tables make_tables(const py::sequence& srcs, const py::object& dsts_obj) {
  Tables t;
  const size_t n = py::len(srcs);
  const bool has_dst = !dsts_obj.is_none();
  py::sequence dsts = has_dst ? dsts_obj.cast<py::sequence>() : py::sequence(py::list());
  if (has_dst && py::len(dsts) != n) throw std::invalid_argument("srcs and dsts differ in length");
  for (size_t i = 0; i < n; ++i) {
    const Ref s = tensor_ref(srcs[i], "src", i);
    const Ref d = has_dst ? tensor_ref(dsts[i], "dst", i) : Ref();
    if (!s.defined && !d.defined) throw std::invalid_argument("pair " + std::to_string(i) + " has neither source nor destination");
    if (s.defined && d.defined && s.numel != d.numel)
      throw std::invalid_argument("pair " + std::to_string(i) + ": source and destination differ in element count");
    const Ref& any = s.defined ? s : d;
    if (t.device < 0) t.device = any.device;
    if ((s.defined && s.device != t.device) || (d.defined && d.device != t.device))
      throw std::invalid_argument("pair " + std::to_string(i) + " is on another device");
    t.src.push_back(s.ptr);
    t.dst.push_back(d.ptr);
    t.numel.push_back(any.numel);
    t.sdt.push_back(s.defined ? s.dtype : d.dtype);
    t.ddt.push_back(d.defined ? d.dtype : s.dtype);
  }
  if (t.device < 0) t.device = 0;
  return t;
}

class Plan {
 public:
  Plan(const py::sequence& srcs, const py::object& dsts, int64_t chunk_elems) : keep_src_(srcs), keep_dst_(dsts) {
    const Tables t = make_tables(srcs, dsts);
    device_ = t.device;
    n_ = (int)t.numel.size();
    check(rg_plan_create(&plan_, device_, n_, t.src.data(), t.dst.data(), t.numel.data(), t.sdt.data(), t.ddt.data(),
                         chunk_elems));
  }
  ~Plan() { close(); }
  Plan(const Plan&) = delete;
  Plan& operator=(const Plan&) = delete;

  void close() {
    if (plan_ != nullptr) {
      rg_plan_destroy(plan_);
      plan_ = nullptr;
    }
  }
  void update(const py::sequence& srcs, const py::object& dsts) {
    const Tables t = make_tables(srcs, dsts);
    if ((int)t.numel.size() != n_) throw std::invalid_argument("update: the number of tensors changed");
    check(rg_plan_update_pointers(handle(), t.src.data(), dsts.is_none() ? nullptr : t.dst.data(), current_stream(device_)));
    keep_src_ = srcs;
    if (!dsts.is_none()) keep_dst_ = dsts;
  }
  void fused_step(float inv_scale, float max_norm, int flags) { check(rg_fused_step(handle(), inv_scale, max_norm, flags, current_stream(device_))); }
  void step_begin(float inv_scale) { check(rg_step_begin(handle(), inv_scale, current_stream(device_))); }
  void step_finish(float max_norm, int flags) { check(rg_step_finish(handle(), max_norm, flags, current_stream(device_))); }
  void step_decide(float max_norm, int flags) { check(rg_step_decide(handle(), max_norm, flags, current_stream(device_))); }
  uintptr_t result_device_ptr() {
    const rg_step_result* r = nullptr;
    check(rg_result_device_ptr(handle(), &r));
    return reinterpret_cast<uintptr_t>(r);
  }
  void unscale_pack(float inv_scale) { check(rg_unscale_pack(handle(), inv_scale, current_stream(device_))); }
  void step_apply_clip(float max_norm, int flags) { check(rg_step_apply_clip(handle(), max_norm, flags, current_stream(device_))); }
  void accumulate(float scale) { check(rg_accumulate(handle(), scale, current_stream(device_))); }
  void unscale_accumulate(float inv_scale) {
    check(rg_unscale_accumulate(handle(), inv_scale, current_stream(device_)));
  }
  void grad_norm() { check(rg_grad_norm(handle(), current_stream(device_))); }
  void scale_cast(float scale) { check(rg_scale_cast(handle(), scale, current_stream(device_))); }
  void zero() { check(rg_zero(handle(), current_stream(device_))); }
  py::dict result() {
    rg_step_result r;
    check(rg_read_result(handle(), &r, current_stream(device_)));
    py::dict d;
    d["norm"] = r.norm;
    d["coef"] = r.coef;
    d["overflow"] = r.overflow;
    d["clipped"] = r.clipped;
    d["skipped"] = r.skipped;
    return d;
  }
  std::vector<float> tensor_norms() {
    std::vector<float> out((size_t)(n_ > 0 ? n_ : 1));
    check(rg_read_tensor_norms(handle(), out.data(), current_stream(device_)));
    out.resize((size_t)n_);
    return out;
  }
  int64_t num_chunks() const { return rg_plan_num_chunks(plan_); }
  int64_t chunk_elems() const { return rg_plan_chunk_elems(plan_); }
  int64_t total_numel() const { return rg_plan_total_numel(plan_); }
  int num_tensors() const { return n_; }

 private:
  rg_plan* handle() {
    if (plan_ == nullptr) throw std::runtime_error("the plan is closed");
    return plan_;
  }
  rg_plan* plan_ = nullptr;
  int device_ = 0;
  int n_ = 0;
  py::object keep_src_, keep_dst_;  // the table points into these tensors
};

// Table of an optimizer launch: fp32 parameters, their gradients, one or two fp32 state
// tensors per parameter and (optionally) the low-precision model copies written by the step.
class Optim {
 public:
  Optim(const py::sequence& params, const py::sequence& grads, const py::object& state1, const py::object& state2,
        const py::object& copies)
      : keep_(py::make_tuple(params, grads, state1, state2, copies)) {
    const size_t n = py::len(params);
    if (py::len(grads) != n) throw std::invalid_argument("params and grads differ in length");
    std::vector<void*> p, s1, s2, c;
    std::vector<const void*> g;
    std::vector<int64_t> numel;
    std::vector<int> gdt, cdt;
    auto column = [&](const py::object& o, const char* what, std::vector<void*>& out, std::vector<int>* dtypes, bool need_f32) {
      if (o.is_none()) return;
      py::sequence seq = o.cast<py::sequence>();
      if (py::len(seq) != n) throw std::invalid_argument(std::string(what) + " differs in length from params");
      for (size_t i = 0; i < n; ++i) {
        const Ref r = tensor_ref(seq[i], what, i);
        if (r.defined && (r.numel != numel[i] || r.device != device_))
          throw std::invalid_argument(std::string(what) + "[" + std::to_string(i) + "] differs in size or device from its parameter");
        if (r.defined && need_f32 && r.dtype != RG_F32)
          throw std::invalid_argument(std::string(what) + "[" + std::to_string(i) + "] must be float32");
        out.push_back(r.ptr);
        if (dtypes) dtypes->push_back(r.defined ? r.dtype : (int)RG_F32);
      }
    };
    for (size_t i = 0; i < n; ++i) {
      const Ref r = tensor_ref(params[i], "param", i);
      if (!r.defined || r.dtype != RG_F32) throw std::invalid_argument("param[" + std::to_string(i) + "] must be a float32 tensor");
      if (i == 0) device_ = r.device;
      if (r.device != device_) throw std::invalid_argument("param[" + std::to_string(i) + "] is on another device");
      p.push_back(r.ptr);
      numel.push_back(r.numel);
    }
    for (size_t i = 0; i < n; ++i) {
      const Ref r = tensor_ref(grads[i], "grad", i);
      if (!r.defined || r.numel != numel[i] || r.device != device_)
        throw std::invalid_argument("grad[" + std::to_string(i) + "] must be a tensor of its parameter's size and device");
      g.push_back(r.ptr);
      gdt.push_back(r.dtype);
    }
    column(state1, "state1", s1, nullptr, true);
    column(state2, "state2", s2, nullptr, true);
    column(copies, "model_copy", c, &cdt, false);
    check(rg_optim_create(&opt_, device_, (int)n, p.data(), g.data(), s1.empty() && state1.is_none() ? nullptr : s1.data(),
                          s2.empty() && state2.is_none() ? nullptr : s2.data(), copies.is_none() ? nullptr : c.data(),
                          numel.data(), gdt.data(), copies.is_none() ? nullptr : cdt.data()));
  }
  ~Optim() { close(); }
  Optim(const Optim&) = delete;
  Optim& operator=(const Optim&) = delete;
  void close() {
    if (opt_ != nullptr) {
      rg_optim_destroy(opt_);
      opt_ = nullptr;
    }
  }
  void adam_step(double lr, double beta1, double beta2, double eps, double weight_decay, int64_t step, bool decoupled,
                 bool maximize, float grad_scale, uintptr_t gate) {
    rg_adam_args a{lr, beta1, beta2, eps, weight_decay, step, decoupled ? 1 : 0, maximize ? 1 : 0, grad_scale,
                   reinterpret_cast<const rg_step_result*>(gate)};
    check(rg_adam_step(handle(), &a, current_stream(device_)));
  }
  // `clock`: a float32 tensor of 8 elements on the device (an rg_adam_clock); advanced, then read by the step
  void adam_step_clocked(const py::object& clock, double lr, double beta1, double beta2, double eps, double weight_decay,
                         bool decoupled, bool maximize, float grad_scale, uintptr_t gate) {
    if (clock.attr("numel")().cast<int64_t>() * clock.attr("element_size")().cast<int64_t>() < (int64_t)sizeof(rg_adam_clock))
      throw std::invalid_argument("the clock tensor must hold at least 32 bytes");
    auto* c = reinterpret_cast<rg_adam_clock*>(clock.attr("data_ptr")().cast<uintptr_t>());
    const auto* g = reinterpret_cast<const rg_step_result*>(gate);
    check(rg_adam_clock_advance(c, lr, beta1, beta2, g, device_, current_stream(device_)));
    rg_adam_args a{lr, beta1, beta2, eps, weight_decay, 0, decoupled ? 1 : 0, maximize ? 1 : 0, grad_scale, g};
    check(rg_adam_step_clocked(handle(), &a, c, current_stream(device_)));
  }
  void sgd_step(double lr, double momentum, double dampening, double weight_decay, bool nesterov, bool maximize,
                bool first_step, float grad_scale, uintptr_t gate) {
    rg_sgd_args a{lr, momentum, dampening, weight_decay, nesterov ? 1 : 0, maximize ? 1 : 0, first_step ? 1 : 0, grad_scale,
                  reinterpret_cast<const rg_step_result*>(gate)};
    check(rg_sgd_step(handle(), &a, current_stream(device_)));
  }

 private:
  rg_optim* handle() {
    if (opt_ == nullptr) throw std::runtime_error("the optimizer table is closed");
    return opt_;
  }
  rg_optim* opt_ = nullptr;
  int device_ = 0;
  py::object keep_;  // the table points into these tensors
};

void copy_cast(const py::handle& dst, const py::handle& src, float scale) {
  const Ref d = tensor_ref(dst, "dst", 0);
  const Ref s = tensor_ref(src, "src", 0);
  if (!d.defined) throw std::invalid_argument("copy_cast needs a destination");
  if (s.defined && (s.numel != d.numel || s.device != d.device))
    throw std::invalid_argument("copy_cast: source and destination differ in element count or device");
  check(rg_scale_cast_single(s.ptr, d.ptr, d.numel, s.defined ? s.dtype : d.dtype, d.dtype, scale, d.device,
                             current_stream(d.device)));
}

// ---------------------------------------------------------------------------------------------
// The free functions of the reference's extension module that sit on this path, under their own
// names and with their argument meaning (src/main.cpp:55-59, 78-136, 191-245), for one process:
// a maintainer can register this module's functions as `_pyrannc`'s.  Tensors are identified by
// the Python id() of the object (src/bind/PybindUtil.cpp:8-12); the registries hold the tensors.

long object_id(const py::handle& o) { return (long)reinterpret_cast<intptr_t>(o.ptr()); }

py::object torch_empty(int64_t n, const py::object& dtype, const py::object& device) {
  return py::module_::import("torch").attr("empty")(n, py::arg("dtype") = dtype, py::arg("device") = device);
}

// DistributedParamLocator (src/comp/DistributedParamLocator.cpp:14-83) + gather
// (src/comp/DistributedParamLocatorBase.cpp:96-153) for a world of one rank.
class DistParamRegistry {
 public:
  struct Entry {
    int64_t numel = 0, aligned = 0, segment = 0, offset = 0, src_size = 0;
    py::object shape;       // torch.Size of the full tensor
    bool requires_grad = false;
    py::object part;        // this rank's segment
  };

  py::object store(const py::object& param) {
    const long pid = object_id(param);
    Entry e;
    e.numel = param.attr("numel")().cast<int64_t>();
    const int esz = param.attr("element_size")().cast<int>();
    dtype_code(param);                                            // float32 / float16 / bfloat16 only
    check(rg_segment_layout(e.numel, esz, 1, &e.aligned, &e.segment, &e.offset, &e.src_size));
    e.shape = param.attr("shape");
    e.requires_grad = param.attr("requires_grad").cast<bool>();
    py::object flat = param.attr("detach")().attr("contiguous")().attr("view")(-1).attr("narrow")(0, e.offset, e.src_size);
    if (param.attr("is_cuda").cast<bool>()) {
      e.part = torch_empty(e.src_size, param.attr("dtype"), param.attr("device"));
      if (e.src_size > 0) copy_cast(e.part, flat, 1.0f);
    } else {
      // built on the host: the slice is uploaded (a transfer, no arithmetic); the segment lives on the GPU
      e.part = flat.attr("to")("cuda");
    }
    e.part.attr("requires_grad_")(e.requires_grad);
    entries_[pid] = e;
    return e.part;
  }
  Entry& at(long pid) {
    auto it = entries_.find(pid);
    if (it == entries_.end()) throw std::invalid_argument("Parameter is not registered: " + std::to_string(pid));
    return it->second;
  }
  py::object load(long pid) {
    Entry& e = at(pid);
    py::object buf = torch_empty(e.segment, e.part.attr("dtype"), e.part.attr("device"));
    const int64_t n = e.part.attr("numel")().cast<int64_t>();
    if (n > 0) copy_cast(buf.attr("narrow")(0, 0, n), e.part.attr("detach")(), 1.0f);
    if (e.segment > n) copy_cast(buf.attr("narrow")(0, n, e.segment - n), py::none(), 1.0f);      // zero padding
    py::object out = buf.attr("narrow")(0, 0, e.numel).attr("view")(e.shape).attr("cpu")().attr("detach")();
    out.attr("requires_grad_")(e.requires_grad);
    return out;
  }
  void set(long pid, const py::object& full) {
    Entry& e = at(pid);
    if (e.src_size == 0) return;
    py::object src = full.attr("detach")().attr("to")(e.part.attr("device")).attr("contiguous")().attr("view")(-1)
                         .attr("narrow")(0, e.offset, e.src_size);
    copy_cast(e.part.attr("detach")(), src, 1.0f);
  }
  void set_dtype(long pid, const py::object& dtype) {
    Entry& e = at(pid);
    if (py::object(e.part.attr("dtype")).equal(dtype)) return;
    py::object fresh = torch_empty(e.part.attr("numel")().cast<int64_t>(), dtype, e.part.attr("device"));
    dtype_code(fresh);
    copy_cast(fresh, e.part.attr("detach")(), 1.0f);
    fresh.attr("requires_grad_")(e.requires_grad);
    e.part = fresh;
  }
  bool registered(long pid) const { return entries_.count(pid) != 0; }
  void remove(long pid) { entries_.erase(pid); }
  void clear() { entries_.clear(); }

 private:
  std::unordered_map<long, Entry> entries_;
};

DistParamRegistry& dist_params() {
  static DistParamRegistry* r = new DistParamRegistry();   // never destroyed: it holds Python objects
  return *r;
}

}  // namespace

PYBIND11_MODULE(_ranncgrad, m) {
  m.doc() = "pybind11 entry points of libranncgrad (per-step parameter/gradient path, MI355X)";
  m.attr("RG_F32") = (int)RG_F32;
  m.attr("RG_F16") = (int)RG_F16;
  m.attr("RG_BF16") = (int)RG_BF16;
  m.attr("STEP_DEFAULT") = (int)RG_STEP_DEFAULT;
  m.attr("STEP_WRITE_ON_OVERFLOW") = (int)RG_STEP_WRITE_ON_OVERFLOW;
  m.attr("STEP_IGNORE_OVERFLOW") = (int)RG_STEP_IGNORE_OVERFLOW;
  m.attr("STEP_EXPECT_NO_CLIP") = (int)RG_STEP_EXPECT_NO_CLIP;
  m.def("version", &rg_version);
  m.def("current_stream", [](int device) { return reinterpret_cast<uintptr_t>(current_stream(device)); }, py::arg("device"),
        "the hipStream_t PyTorch currently launches on for this device, as an integer (c10::hip::getCurrentHIPStream)");
  m.def("aligned_numel", [](int64_t numel, int elem_size, int split) {
    const int64_t r = rg_aligned_numel(numel, elem_size, split);
    if (r < 0) throw std::invalid_argument(rg_last_error());
    return r;
  });
  m.def("segment_layout", [](int64_t numel, int elem_size, int nranks) {
    if (nranks < 1) throw std::invalid_argument("nranks must be >= 1");
    int64_t aligned = 0, seg = 0;
    std::vector<int64_t> offs((size_t)nranks), srcs((size_t)nranks);
    check(rg_segment_layout(numel, elem_size, nranks, &aligned, &seg, offs.data(), srcs.data()));
    return py::make_tuple(aligned, seg, offs, srcs);
  });
  m.def("copy_cast", &copy_cast, py::arg("dst"), py::arg("src"), py::arg("scale") = 1.0f,
        "dst.copy_(src) with dtype conversion and optional scale for one pair of tensors; src=None stores zeros");
  // -- the reference's names (one process, one GPU)
  m.def("get_rank", [] { return 0; });
  m.def("get_world_size", [] { return 1; });
  m.def("barrier", [] {});
  m.def("allreduce_tensor", [](const py::object& tensor, bool sum) {
    (void)sum;                                       // a sum or a minimum over one rank leaves the tensor as it is
    if (!py::hasattr(tensor, "data_ptr")) throw std::invalid_argument("allreduce_tensor expects a tensor");
  }, py::arg("tensor"), py::arg("sum"));
  m.def("bcast_tensor", [](const py::object& tensor, int root) {
    if (root != 0) throw std::invalid_argument("root " + std::to_string(root) + " is not a rank of this world (size 1)");
    return tensor.attr("cuda")();
  });
  m.def("all_gather", [](const py::object& ten, const py::object& buf) {
    if (buf.attr("numel")().cast<int64_t>() != ten.attr("numel")().cast<int64_t>())
      throw std::invalid_argument("all_gather: receive buffer must hold world_size * numel elements");
    copy_cast(buf.attr("view")(-1), ten.attr("contiguous")().attr("view")(-1), 1.0f);
  });
  m.def("store_dist_param", [](const py::object& param) { return dist_params().store(param); });
  m.def("load_dist_param", [](long pid) { return dist_params().load(pid); });
  m.def("set_dist_param", [](long pid, const py::object& full) { dist_params().set(pid, full); });
  m.def("get_dist_param_segment", [](long pid) { return dist_params().at(pid).part; });
  m.def("set_dist_param_dtype", [](long pid, const py::object& dtype) { dist_params().set_dtype(pid, dtype); });
  m.def("get_dist_param_range", [](long pid) {
    const auto& e = dist_params().at(pid);
    return py::make_tuple(e.offset, e.offset + e.src_size);
  });
  m.def("remove_dist_param", [](long pid) { dist_params().remove(pid); });
  m.def("dist_param_registered", [](long pid) { return dist_params().registered(pid); });
  m.def("clear", [] {
    dist_params().clear();
    reset_registry();
  });
  bind_registry(m);
  py::class_<Plan>(m, "Plan")
      .def(py::init<const py::sequence&, const py::object&, int64_t>(), py::arg("srcs"), py::arg("dsts") = py::none(),
           py::arg("chunk_elems") = 0)
      .def("update", &Plan::update, py::arg("srcs"), py::arg("dsts") = py::none())
      .def("fused_step", &Plan::fused_step, py::arg("inv_scale"), py::arg("max_norm"), py::arg("flags") = 0)
      .def("step_begin", &Plan::step_begin)
      .def("step_finish", &Plan::step_finish, py::arg("max_norm"), py::arg("flags") = 0)
      .def("step_decide", &Plan::step_decide, py::arg("max_norm"), py::arg("flags") = 0)
      .def("result_device_ptr", &Plan::result_device_ptr)
      .def("unscale_pack", &Plan::unscale_pack)
      .def("step_apply_clip", &Plan::step_apply_clip, py::arg("max_norm"), py::arg("flags") = 0)
      .def("accumulate", &Plan::accumulate, py::arg("scale") = 1.0f)
      .def("unscale_accumulate", &Plan::unscale_accumulate)
      .def("grad_norm", &Plan::grad_norm)
      .def("scale_cast", &Plan::scale_cast, py::arg("scale") = 1.0f)
      .def("zero", &Plan::zero)
      .def("result", &Plan::result)
      .def("tensor_norms", &Plan::tensor_norms)
      .def("close", &Plan::close)
      .def_property_readonly("num_chunks", &Plan::num_chunks)
      .def_property_readonly("chunk_elems", &Plan::chunk_elems)
      .def_property_readonly("total_numel", &Plan::total_numel)
      .def_property_readonly("num_tensors", &Plan::num_tensors);
  py::class_<Optim>(m, "Optim")
      .def(py::init<const py::sequence&, const py::sequence&, const py::object&, const py::object&, const py::object&>(),
           py::arg("params"), py::arg("grads"), py::arg("state1") = py::none(), py::arg("state2") = py::none(),
           py::arg("model_copies") = py::none())
      .def("adam_step", &Optim::adam_step, py::arg("lr"), py::arg("beta1"), py::arg("beta2"), py::arg("eps"),
           py::arg("weight_decay"), py::arg("step"), py::arg("decoupled") = false, py::arg("maximize") = false,
           py::arg("grad_scale") = 1.0f, py::arg("gate") = (uintptr_t)0)
      .def("adam_step_clocked", &Optim::adam_step_clocked, py::arg("clock"), py::arg("lr"), py::arg("beta1"), py::arg("beta2"),
           py::arg("eps"), py::arg("weight_decay"), py::arg("decoupled") = false, py::arg("maximize") = false,
           py::arg("grad_scale") = 1.0f, py::arg("gate") = (uintptr_t)0)
      .def("sgd_step", &Optim::sgd_step, py::arg("lr"), py::arg("momentum") = 0.0, py::arg("dampening") = 0.0,
           py::arg("weight_decay") = 0.0, py::arg("nesterov") = false, py::arg("maximize") = false,
           py::arg("first_step") = false, py::arg("grad_scale") = 1.0f, py::arg("gate") = (uintptr_t)0)
      .def("close", &Optim::close);
}
