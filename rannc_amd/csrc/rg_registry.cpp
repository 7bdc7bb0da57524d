// Native registry of the per-step path (part of the pybind11 module rannc_amd._ranncgrad):
//
//   TensorList    a fixed list of tensors whose .grad fields are read, set and cleared in C++ loops
//   GradPlan      a device table that follows the gradients of such a list (in place, or into fixed
//                 destinations) - what the amp context exit, clip_grad_norm and zero_grad run on
//   ParamStorage  pid -> tensor, amp masters, name-sorted ids per graph, ZeRO layouts for one rank and the
//                 per-step operations of src/comp/ParamStorage.cpp (registry layout: src/comp/ParamStorage.h:155-168)
//   RaNNCModule   the methods of the reference's bound class that sit on this path (src/main.cpp:333-380)
//
// The reference walks its parameters in C++ and issues one ATen op per tensor; here the walk only collects
// addresses, and every loop over parameters is one launch of libranncgrad over a device table.
#include <algorithm>
#include <map>
#include <memory>
#include <unordered_map>

#include "rg_bind.h"

using namespace rgbind;

namespace {

// ------------------------------------------------------------------------------------------------ TensorList

class TensorList {
 public:
  explicit TensorList(const py::object& tensors) : t_(tensor_vector(tensors, "TensorList")) {}
  explicit TensorList(std::vector<at::Tensor> tensors) : t_(std::move(tensors)) {}
  size_t size() const { return t_.size(); }
  const std::vector<at::Tensor>& tensors() const { return t_; }

  int count_grads() const {
    int n = 0;
    for (const at::Tensor& t : t_) n += (t.defined() && t.grad().defined()) ? 1 : 0;
    return n;
  }
  py::list grads() const {
    py::list out;
    for (const at::Tensor& t : t_) {
      if (t.defined() && t.grad().defined()) out.append(t.grad());
      else out.append(py::none());
    }
    return out;
  }
  // t[i].grad = views[i] for every i (both lists are in the same order)
  void set_grads(const TensorList& views) {
    if (views.size() != t_.size()) throw std::invalid_argument("set_grads: the lists differ in length");
    for (size_t i = 0; i < t_.size(); ++i) t_[i].mutable_grad() = views.t_[i];
  }
  void clear_grads() {
    for (at::Tensor& t : t_)
      if (t.defined()) t.mutable_grad() = at::Tensor();
  }
  // How many tensors hold a gradient, and - in `each_usable` - whether every one of them can be a row of a device
  // table as it is (on the GPU, contiguous, of dtype `dtype`): what the steady state of a training loop looks like.
  int count_usable_grads(at::ScalarType dtype, bool* each_usable) const {
    int n = 0;
    bool ok = true;
    for (const at::Tensor& t : t_) {
      if (!t.defined()) continue;
      const at::Tensor& g = t.grad();
      if (!g.defined()) continue;
      ++n;
      ok = ok && g.is_cuda() && g.is_contiguous() && g.scalar_type() == dtype && g.numel() == t.numel();
    }
    *each_usable = ok;
    return n;
  }

 private:
  std::vector<at::Tensor> t_;
};

// ------------------------------------------------------------------------------------------------ GradPlan

// The gradients of `owners` as sources, written in place (no destinations) or into `dsts`.  bind() looks at
// the gradients that exist now; owners without one are left out of an in-place table and make a table with
// destinations unusable (the caller then takes its general path).
class GradPlan {
 public:
  GradPlan(std::shared_ptr<TensorList> owners, std::shared_ptr<TensorList> dsts) : owners_(std::move(owners)), dsts_(std::move(dsts)) {
    if (dsts_ && dsts_->size() != owners_->size()) throw std::invalid_argument("owners and destinations differ in length");
  }

  // Number of gradients the table now covers; -1 when destinations are given and some owner has no gradient.
  int bind() {
    const auto& owners = owners_->tensors();
    std::vector<at::Tensor> srcs, dsts;
    srcs.reserve(owners.size());
    for (size_t i = 0; i < owners.size(); ++i) {
      const at::Tensor& g = owners[i].grad();
      if (!g.defined()) {
        if (dsts_) return -1;
        continue;
      }
      srcs.push_back(g);
      if (dsts_) dsts.push_back(dsts_->tensors()[i]);
    }
    if (srcs.empty()) return 0;
    rebuilt_ = plan_.bind(srcs, dsts_ ? dsts : srcs);
    held_.swap(srcs);
    bound_ = (int)held_.size();
    return bound_;
  }
  bool rebuilt() const { return rebuilt_; }
  // bind() for the steady state of a mixed-precision loop, in one walk: every owner (half parameter) has a usable
  // gradient - on the GPU, contiguous, of `dtype`, of its size - and no master has one yet; then each master's
  // gradient becomes its destination view and the table is bound.  -1, with nothing changed, otherwise.
  int bind_steady(TensorList& masters, at::ScalarType dtype) {
    if (!dsts_ || masters.size() != owners_->size()) throw std::invalid_argument("bind_steady: one master and one view per owner");
    const auto& owners = owners_->tensors();
    const auto& ms = masters.tensors();
    for (size_t i = 0; i < owners.size(); ++i) {
      const at::Tensor& g = owners[i].grad();
      if (!g.defined() || !g.is_cuda() || !g.is_contiguous() || g.scalar_type() != dtype || g.numel() != owners[i].numel()) return -1;
      if (ms[i].grad().defined()) return -1;
    }
    masters.set_grads(*dsts_);
    return bind();
  }
  // The gradient addresses the table reads, handed to an optimizer table (an rg_optim made by any binding of the
  // library) whose rows [0, count) are the owners [offset, offset + count) of this plan: one stream-ordered
  // upload, and none when that table already points there.
  bool push_sources_to_optim(uintptr_t optim_handle, int offset, int count) {
    if (offset < 0 || count < 0 || (size_t)offset + (size_t)count > held_.size())
      throw std::invalid_argument("push_sources_to_optim: the rows are not covered by the gradients the plan holds");
    std::vector<const void*> ptrs((size_t)count);
    for (int i = 0; i < count; ++i) {
      const at::Tensor& g = held_[(size_t)(offset + i)];
      ptrs[(size_t)i] = g.numel() ? g.data_ptr() : nullptr;
    }
    std::vector<const void*>& last = pushed_[optim_handle];
    if (last == ptrs) return false;
    check(rg_optim_update_pointers(reinterpret_cast<rg_optim*>(optim_handle), nullptr, ptrs.data(), nullptr, nullptr, nullptr,
                                   plan_.stream()));
    last.swap(ptrs);
    return true;
  }
  void forget_optim(uintptr_t optim_handle) { pushed_.erase(optim_handle); }
  int held() const { return (int)held_.size(); }
  // dtype code of the gradients the table reads (-1: none held, or they differ)
  int source_dtype() const {
    if (held_.empty()) return -1;
    const int code = dtype_code(held_[0]);
    for (const at::Tensor& g : held_)
      if (dtype_code(g) != code) return -1;
    return code;
  }
  // the table keeps raw addresses: the gradients it reads stay alive here until every kernel reading them is queued
  void drop_sources() { held_.clear(); }
  py::list sources() const {
    py::list out;
    for (const at::Tensor& t : held_) out.append(t);
    return out;
  }

  void fused_step(float inv_scale, float max_norm, int flags) { check(rg_fused_step(plan_.get(), inv_scale, max_norm, flags, plan_.stream())); }
  void step_begin(float inv_scale) { check(rg_step_begin(plan_.get(), inv_scale, plan_.stream())); }
  void step_begin_scaled(uintptr_t inv_scale_dev) { check(rg_step_begin_scaled(plan_.get(), reinterpret_cast<const float*>(inv_scale_dev), plan_.stream())); }
  void step_finish(float max_norm, int flags) { check(rg_step_finish(plan_.get(), max_norm, flags, plan_.stream())); }
  void step_decide(float max_norm, int flags) { check(rg_step_decide(plan_.get(), max_norm, flags, plan_.stream())); }
  void unscale_pack(float inv_scale) { check(rg_unscale_pack(plan_.get(), inv_scale, plan_.stream())); }
  void step_apply_clip(float max_norm, int flags) { check(rg_step_apply_clip(plan_.get(), max_norm, flags, plan_.stream())); }
  void unscale_accumulate(float inv_scale) { check(rg_unscale_accumulate(plan_.get(), inv_scale, plan_.stream())); }
  void grad_norm() { check(rg_grad_norm(plan_.get(), plan_.stream())); }
  void scale_cast(float scale) { check(rg_scale_cast(plan_.get(), scale, plan_.stream())); }
  void zero() { check(rg_zero(plan_.get(), plan_.stream())); }
  int tune() {
    check(rg_plan_tune(plan_.get(), plan_.stream()));
    return rg_plan_write_order(plan_.get());
  }
  int write_order() { return rg_plan_write_order(plan_.get()); }
  void set_write_order(int order) { check(rg_plan_set_write_order(plan_.get(), order)); }
  py::dict result() { return result_dict(plan_.result()); }
  rg_step_result raw_result() { return plan_.result(); }
  uintptr_t result_device_ptr() {
    const rg_step_result* r = nullptr;
    check(rg_result_device_ptr(plan_.get(), &r));
    return reinterpret_cast<uintptr_t>(r);
  }
  bool is_open() const { return plan_.open(); }
  void close() {
    plan_.close();
    held_.clear();
  }
  int64_t num_chunks() { return rg_plan_num_chunks(plan_.get()); }
  uintptr_t handle() { return reinterpret_cast<uintptr_t>(plan_.get()); }   // the rg_plan*, for telling tables apart

 private:
  std::shared_ptr<TensorList> owners_, dsts_;
  PairPlan plan_;
  std::vector<at::Tensor> held_;
  std::unordered_map<uintptr_t, std::vector<const void*>> pushed_;
  int bound_ = 0;
  bool rebuilt_ = false;
};

// ------------------------------------------------------------------------------------------------ GradBuckets

// The per-step half of GradConsolidation (src/comp/ParamStorage.cpp:154-176) for parameters whose gradients live in
// their own buckets: `views[i]` is parameter i's slice of its dtype's bucket.  consolidate() makes every .grad that
// view - a gradient that lives elsewhere is copied in, a missing one starts from zeros - with one copy launch and
// one zero launch for all parameters, instead of the reference's copy_ / zero_ per parameter.
class GradBuckets {
 public:
  GradBuckets(std::shared_ptr<TensorList> params, std::shared_ptr<TensorList> views) : params_(std::move(params)), views_(std::move(views)) {
    if (params_->size() != views_->size()) throw std::invalid_argument("one bucket view per parameter");
  }
  // returns (gradients copied in, views zeroed)
  std::pair<int, int> consolidate() {
    const auto& views = views_->tensors();
    std::vector<at::Tensor> copy_src, copy_dst, zero_src, zero_dst;
    auto& params = const_cast<std::vector<at::Tensor>&>(params_->tensors());
    for (size_t i = 0; i < params.size(); ++i) {
      at::Tensor& p = params[i];
      const at::Tensor& view = views[i];
      const at::Tensor& g = p.grad();
      if (g.defined()) {
        if (g.data_ptr() == view.data_ptr()) continue;                       // :158-160
        copy_src.push_back(g.is_contiguous() ? g : g.contiguous());
        copy_dst.push_back(view);
        p.mutable_grad() = view;                                             // :163-166
      } else {
        p.mutable_grad() = view;                                             // :169-175
        zero_src.emplace_back();
        zero_dst.push_back(view);
      }
    }
    if (!copy_src.empty()) {
      copy_plan_.bind(copy_src, copy_dst);
      check(rg_scale_cast(copy_plan_.get(), 1.0f, copy_plan_.stream()));
    }
    if (!zero_dst.empty()) {
      zero_plan_.bind(zero_src, zero_dst);
      check(rg_zero(zero_plan_.get(), zero_plan_.stream()));
    }
    return {(int)copy_src.size(), (int)zero_dst.size()};
  }

 private:
  std::shared_ptr<TensorList> params_, views_;
  PairPlan copy_plan_, zero_plan_;
};

// ------------------------------------------------------------------------------------------------ ParamStorage

struct SegmentLayout {
  int64_t aligned = 0, segment = 0, offset = 0, src_size = 0;   // one rank: offset 0, src_size = numel
};

class ParamStorage {
 public:
  // ---- registry (src/comp/ParamStorage.cpp:195-205, 269-273, 648-650, 715-719)
  void register_param(long pid, const at::Tensor& t) {
    params_[pid] = t;
    ++generation_;
  }
  const at::Tensor& get_param_tensor(long pid) const {
    auto it = params_.find(pid);
    if (it == params_.end()) throw std::invalid_argument("Parameter not found: " + std::to_string(pid));
    return it->second;
  }
  bool has_param(long pid) const { return params_.count(pid) != 0; }
  void register_amp_master_param(long model_pid, long master_pid, const at::Tensor& t) {
    amp_masters_[model_pid] = t;
    amp_param_id_map_[master_pid] = model_pid;
    ++generation_;
  }
  bool has_amp_master_param(long pid) const { return amp_masters_.count(pid) != 0; }
  const at::Tensor& get_amp_master_param_tensor(long pid) const {
    auto it = amp_masters_.find(pid);
    if (it == amp_masters_.end()) throw std::invalid_argument("Amp master parameter not found: " + std::to_string(pid));
    return it->second;
  }

  // ---- deployment: the slice of ParamStorage::deploy (src/comp/ParamStorage.cpp:827-1022) the per-step path needs
  void deploy(const std::string& gid, const std::map<std::string, long>& name_to_pid, bool enable_zero, bool consolidate,
              bool use_amp_master, bool allreduce_amp_master) {
    graphs_.erase(gid);
    Graph& g = graphs_[gid];
    g.name_to_pid = name_to_pid;
    for (const auto& kv : name_to_pid) g.sorted.push_back(kv.second);       // std::map iterates in name order (:23-31)
    g.zero = enable_zero;
    g.consolidate = consolidate;
    g.use_amp_master = use_amp_master;
    allreduce_amp_master_ = allreduce_amp_master;
    if (enable_zero) {
      for (long pid : g.sorted) {
        const at::Tensor& p = get_param_tensor(pid);
        SegmentLayout l;
        check(rg_segment_layout(p.numel(), (int)p.element_size(), 1, &l.aligned, &l.segment, &l.offset, &l.src_size));
        g.layouts[pid] = l;
      }
    }
    ++generation_;
  }
  void undeploy(const std::string& gid) { graphs_.erase(gid); }
  bool deployed(const std::string& gid) const { return graphs_.count(gid) != 0; }
  std::vector<long> sorted_param_ids(const std::string& gid) { return graph(gid).sorted; }
  bool zero_enabled(const std::string& gid) { return graph(gid).zero; }
  // buckets the gradients of this graph are views of (GradConsolidation); clear_param_grads then clears those
  void set_consolidated_grads(const std::string& gid, const std::vector<at::Tensor>& buckets) {
    for (size_t i = 0; i < buckets.size(); ++i) require_gpu_contiguous(buckets[i], "bucket", i);
    graph(gid).buckets = buckets;
  }

  // ---- per-step operations
  // calcGradGlobalL2Norm (src/comp/ParamStorage.cpp:747-819): one read-only launch over all gradients in name
  // order, one read-back instead of one .item() per parameter.
  double calc_grad_global_l2_norm(const std::string& gid, bool use_amp_master) {
    GradPlan& plan = selected_plan(gid, use_amp_master);
    if (plan.bind() <= 0) return 0.0;
    plan.grad_norm();
    plan.drop_sources();   // queued: PyTorch's allocator is stream-ordered, so the gradients may be freed from here on
    return plan.raw_result().norm;
  }
  // clipGradNorm (:721-745): decided and applied on the device without a host round trip.
  void clip_grad_norm(const std::string& gid, float max_grad_norm, bool use_amp_master) {
    GradPlan& plan = selected_plan(gid, use_amp_master);
    if (plan.bind() <= 0) return;
    plan.fused_step(1.0f, max_grad_norm, RG_STEP_IGNORE_OVERFLOW);
    plan.drop_sources();
  }
  // doScaleGrads (:598-615): grad *= 1/world or grad *= world
  void do_scale_grads(const std::string& gid, bool unscale, bool amp_master_grads, int world_size) {
    Graph& g = graph(gid);
    std::unique_ptr<GradPlan>& slot = g.scale_plan[amp_master_grads ? 1 : 0];
    if (!slot || g.scale_generation != generation_) {
      std::vector<at::Tensor> owners;
      for (long pid : g.sorted)
        owners.push_back(amp_master_grads && has_amp_master_param(pid) ? get_amp_master_param_tensor(pid) : get_param_tensor(pid));
      slot.reset(new GradPlan(std::make_shared<TensorList>(std::move(owners)), nullptr));
      g.scale_generation = generation_;
    }
    if (slot->bind() <= 0) return;
    const float ratio = 1.0f / (float)world_size;
    slot->scale_cast(unscale ? 1.0f / ratio : ratio);
    slot->drop_sources();
  }
  // clearParamGrads (:540-557)
  void clear_param_grads(const std::string& gid) {
    Graph& g = graph(gid);
    if (g.consolidate && !g.buckets.empty()) {
      for (const at::Tensor& b : g.buckets)
        if (b.numel() > 0)
          check(rg_fill_zero(b.data_ptr(), (int64_t)b.numel() * (int64_t)b.element_size(), b.get_device(), current_stream(b.get_device())));
      return;
    }
    if (!g.zero_plan || g.zero_generation != generation_) {
      std::vector<at::Tensor> owners;
      for (long pid : g.sorted) owners.push_back(get_param_tensor(pid));
      g.zero_plan.reset(new GradPlan(std::make_shared<TensorList>(std::move(owners)), nullptr));
      g.zero_generation = generation_;
    }
    if (g.zero_plan->bind() <= 0) return;
    g.zero_plan->zero();
    g.zero_plan->drop_sources();
  }

  // allReduceParamGradsZero (:440-520) for a group of one: every defined gradient is packed (cast to fp32 for
  // half parameters when masters are reduced) into a zero-padded staging buffer of the aligned size; the
  // reduce-scatter over one rank returns the buffer itself, and the first numel elements are copied back over
  // the gradient (:419-427).  Two launches for all parameters; the buffers persist (BufferTensorCache).
  std::vector<at::Tensor> allreduce_param_grads_zero(const std::string& gid) {
    Graph& g = graph(gid);
    // The steady state - the same parameters hold gradients at the same addresses as last time - is two launches
    // over the tables of last time; anything else walks the parameters and rebinds them.
    if (g.stage_valid && g.stage_generation == generation_) {
      size_t k = 0;
      bool same = true;
      for (long pid : g.sorted) {
        const at::Tensor& param = get_param_tensor(pid);
        const at::Tensor& grad = param.grad();
        if (!param.requires_grad() || !grad.defined()) continue;
        if (k >= g.stage_grad_ptrs.size() || grad.data_ptr() != g.stage_grad_ptrs[k] || grad.numel() != g.stage_grad_numel[k] ||
            !grad.is_contiguous()) {
          same = false;
          break;
        }
        ++k;
      }
      if (same && k == g.stage_grad_ptrs.size()) {
        if (k > 0) {
          check(rg_scale_cast(g.stage_pack.get(), 1.0f, g.stage_pack.stream()));
          check(rg_scale_cast(g.stage_back.get(), 1.0f, g.stage_back.stream()));
        }
        return g.stage_bufs;
      }
    }
    g.stage_valid = false;
    g.stage_grad_ptrs.clear();
    g.stage_grad_numel.clear();
    std::vector<at::Tensor> srcs, dsts, back_src, back_dst, bufs;
    for (long pid : g.sorted) {
      const at::Tensor& param = get_param_tensor(pid);
      if (!param.requires_grad() || !param.grad().defined()) continue;         // :471-478
      const at::Tensor grad = param.grad();
      if (!grad.is_contiguous()) throw std::invalid_argument("gradients must be contiguous");
      const int64_t n = grad.numel();
      const int64_t aligned = rg_aligned_numel(n, (int)grad.element_size(), 1);
      const at::ScalarType bdt = (allreduce_amp_master_ && param.scalar_type() == at::kHalf) ? at::kFloat : param.scalar_type();
      at::Tensor& buf = g.staging[pid];
      if (!buf.defined() || buf.numel() != aligned || buf.scalar_type() != bdt || buf.device() != grad.device())
        buf = at::empty({aligned}, grad.options().dtype(bdt));
      const at::Tensor flat = grad.view({-1});
      srcs.push_back(flat);
      dsts.push_back(buf.narrow(0, 0, n));
      if (aligned > n) {
        srcs.push_back(at::Tensor());
        dsts.push_back(buf.narrow(0, n, aligned - n));
      }
      back_src.push_back(buf.narrow(0, 0, n));
      back_dst.push_back(flat);
      bufs.push_back(buf);
      g.stage_grad_ptrs.push_back(grad.data_ptr());
      g.stage_grad_numel.push_back(n);
    }
    if (!srcs.empty()) {
      g.stage_pack.bind(srcs, dsts);
      check(rg_scale_cast(g.stage_pack.get(), 1.0f, g.stage_pack.stream()));
      g.stage_back.bind(back_src, back_dst);
      check(rg_scale_cast(g.stage_back.get(), 1.0f, g.stage_back.stream()));
    }
    g.stage_bufs = bufs;
    g.stage_valid = true;
    g.stage_generation = generation_;
    return bufs;
  }

  // ---- ZeRO views for one rank (src/comp/DistributedGradLocator.cpp:17-86)
  const SegmentLayout& layout(const std::string& gid, long pid) {
    Graph& g = graph(gid);
    auto it = g.layouts.find(pid);
    if (it == g.layouts.end()) throw std::invalid_argument("Parameter is not registered: " + std::to_string(pid));
    return it->second;
  }
  std::pair<int64_t, int64_t> get_local_param_range(const std::string& gid, long pid) {
    const SegmentLayout& l = layout(gid, pid);
    return {l.offset, l.offset + l.src_size};
  }
  at::Tensor get_local_param_segment(const std::string& gid, long pid) {
    Graph& g = graph(gid);
    auto it = g.local_segments.find(pid);
    if (it != g.local_segments.end()) return it->second;
    const SegmentLayout& l = layout(gid, pid);
    const at::Tensor& param = get_param_tensor(pid);
    at::Tensor seg = param.view({-1}).narrow(0, l.offset, l.src_size).detach();      // :17-26
    seg.set_requires_grad(param.requires_grad());
    g.local_segments[pid] = seg;
    ++generation_;
    return seg;
  }
  void set_grad_to_local_param_segment(const std::string& gid) {
    Graph& g = graph(gid);
    if (!g.zero) return;                                                             // :522-529
    for (long pid : g.sorted) {
      const at::Tensor& param = get_param_tensor(pid);
      if (!param.grad().defined()) continue;
      at::Tensor seg = get_local_param_segment(gid, pid);
      if (!seg.requires_grad()) continue;
      const SegmentLayout& l = g.layouts[pid];
      seg.mutable_grad() = param.grad().view({-1}).narrow(0, l.offset, l.src_size);  // :28-34
    }
  }
  // alignBuffer for every parameter (:50-63, ParamStorage.cpp:531-538): re-homed into zero-padded buffers of the
  // aligned size, values preserved; all copies and pad fills in one launch
  void align_buffer_zero(const std::string& gid) {
    Graph& g = graph(gid);
    if (!g.zero) return;
    std::vector<at::Tensor> srcs, dsts;
    std::vector<std::pair<long, at::Tensor>> rehome;
    for (long pid : g.sorted) {
      at::Tensor param = get_param_tensor(pid);
      const SegmentLayout& l = g.layouts[pid];
      const int64_t n = param.numel();
      at::Tensor buf = at::empty({l.aligned}, param.options().requires_grad(false));
      srcs.push_back(param.detach().contiguous().view({-1}));
      dsts.push_back(buf.narrow(0, 0, n));
      if (l.aligned > n) {
        srcs.push_back(at::Tensor());
        dsts.push_back(buf.narrow(0, n, l.aligned - n));
      }
      g.buf_tensors[pid] = buf;
      rehome.emplace_back(pid, buf.narrow(0, 0, n).view(param.sizes()));
    }
    if (!srcs.empty()) {
      PairPlan plan;
      plan.bind(srcs, dsts);
      check(rg_scale_cast(plan.get(), 1.0f, plan.stream()));
    }
    for (auto& kv : rehome) {
      at::Tensor param = get_param_tensor(kv.first);
      param.set_data(kv.second);
      g.local_segments.erase(kv.first);
    }
    ++generation_;
  }
  at::Tensor get_buffer(const std::string& gid, long pid) {
    Graph& g = graph(gid);
    auto it = g.buf_tensors.find(pid);
    if (it == g.buf_tensors.end()) throw std::invalid_argument("Parameter has no aligned buffer: " + std::to_string(pid));
    return it->second;
  }
  at::Tensor get_buffer_segment(const std::string& gid, long pid, int index) {
    const SegmentLayout& l = layout(gid, pid);                                       // :73-86
    return get_buffer(gid, pid).view({-1}).narrow(0, l.segment * index, l.segment);
  }
  // gatherTensorZero (src/comp/ParamStorage.cpp:670-685) with one rank
  at::Tensor gather_tensor_zero(const at::Tensor& ten, long pid) {
    for (auto& kv : graphs_) {
      Graph& g = kv.second;
      if (!g.zero || g.layouts.count(pid) == 0) continue;
      const at::Tensor& param = get_param_tensor(pid);
      if (ten.numel() != param.numel())
        throw std::invalid_argument("tensor has " + std::to_string(ten.numel()) + " elements, parameter " + std::to_string(pid) +
                                    " has " + std::to_string(param.numel()));
      return ten.detach().reshape(param.sizes());
    }
    throw std::invalid_argument("Param is not registered for zero: " + std::to_string(pid));
  }

  // The tensor whose gradient counts for a parameter: its amp master, its local ZeRO segment, or the parameter
  // itself (src/comp/ParamStorage.cpp:726-738, 755-766).
  std::vector<at::Tensor> selected(const std::string& gid, bool use_amp_master) {
    Graph& g = graph(gid);
    std::vector<at::Tensor> out;
    for (long pid : g.sorted) {
      if (use_amp_master && has_amp_master_param(pid)) out.push_back(get_amp_master_param_tensor(pid));
      else if (g.zero) out.push_back(get_local_param_segment(gid, pid));
      else out.push_back(get_param_tensor(pid));
    }
    return out;
  }

  void clear() {
    graphs_.clear();
    params_.clear();
    amp_masters_.clear();
    amp_param_id_map_.clear();
    ++generation_;
  }

 private:
  struct Graph {
    std::map<std::string, long> name_to_pid;
    std::vector<long> sorted;
    bool zero = false, consolidate = false, use_amp_master = false;
    std::unordered_map<long, SegmentLayout> layouts;
    std::unordered_map<long, at::Tensor> buf_tensors, local_segments, staging;
    std::vector<at::Tensor> buckets;
    std::unique_ptr<GradPlan> selected_plan[2], scale_plan[2], zero_plan;
    uint64_t selected_generation[2] = {0, 0}, scale_generation = 0, zero_generation = 0;
    PairPlan stage_pack, stage_back;
    // what the last allreduce_param_grads_zero bound: the gradients' addresses and sizes, the staging buffers
    std::vector<const void*> stage_grad_ptrs;
    std::vector<int64_t> stage_grad_numel;
    std::vector<at::Tensor> stage_bufs;
    bool stage_valid = false;
    uint64_t stage_generation = 0;
  };

  Graph& graph(const std::string& gid) {
    auto it = graphs_.find(gid);
    if (it == graphs_.end()) throw std::invalid_argument("Graph is not deployed: " + gid);
    return it->second;
  }
  // the plan over the selected tensors' gradients; the selection is taken again whenever the registry changed
  GradPlan& selected_plan(const std::string& gid, bool use_amp_master) {
    Graph& g = graph(gid);
    const int k = use_amp_master ? 1 : 0;
    if (!g.selected_plan[k] || g.selected_generation[k] != generation_) {
      std::vector<at::Tensor> sel = selected(gid, use_amp_master);       // may create segments (bumps the generation)
      g.selected_plan[k].reset(new GradPlan(std::make_shared<TensorList>(std::move(sel)), nullptr));
      g.selected_generation[k] = generation_;
    }
    return *g.selected_plan[k];
  }

  std::unordered_map<long, at::Tensor> params_, amp_masters_;
  std::unordered_map<long, long> amp_param_id_map_;
  std::map<std::string, Graph> graphs_;
  bool allreduce_amp_master_ = false;
  uint64_t generation_ = 1;
};

std::shared_ptr<ParamStorage>& global_storage() {
  static auto* s = new std::shared_ptr<ParamStorage>(std::make_shared<ParamStorage>());   // never destroyed: it holds tensors
  return *s;
}

long object_id(const py::handle& o) { return (long)reinterpret_cast<intptr_t>(o.ptr()); }

// ------------------------------------------------------------------------------------------------ RaNNCModule

// The bound class of the reference (src/main.cpp:257-450), per-step methods only.  `init` registers the
// parameters of the whole model under one graph id; there is no tracing, profiling or partitioning.
class RaNNCModule {
 public:
  RaNNCModule(bool use_amp_master_params, bool allreduce_amp_master_params, bool enable_zero, bool check_unused_values,
              bool offload_params)
      : storage_(global_storage()), use_amp_master_(use_amp_master_params), allreduce_amp_master_(allreduce_amp_master_params),
        enable_zero_(enable_zero) {
    (void)check_unused_values;
    (void)offload_params;
    static int next_id = 0;
    graph_id_ = "native_graph_" + std::to_string(next_id++);
  }
  std::map<std::string, long> init(const py::dict& named_params, bool consolidate_grads) {
    std::map<std::string, long> ids;
    for (auto kv : named_params) {
      const std::string name = py::cast<std::string>(kv.first);
      const at::Tensor t = tensor_or_undefined(kv.second, "init");
      if (!t.defined()) throw std::invalid_argument("parameter " + name + " is None");
      const long pid = object_id(kv.second);
      storage_->register_param(pid, t);
      ids[name] = pid;
    }
    storage_->deploy(graph_id_, ids, enable_zero_, consolidate_grads, use_amp_master_, allreduce_amp_master_);
    deployed_ = true;
    return ids;
  }
  void require() const {
    if (!deployed_) throw std::runtime_error("RaNNCModule is not initialised");
  }
  const std::string& graph_id() const { return graph_id_; }
  void allreduce_grads() { require(); }                      // a sum over one process, pre-multiplied by 1/1
  void allreduce_grads_zero() {
    require();
    staging_ = storage_->allreduce_param_grads_zero(graph_id_);
  }
  void clip_grad_norm(float max_grad_norm) {
    require();
    storage_->clip_grad_norm(graph_id_, max_grad_norm, use_amp_master_);
  }
  double calc_grad_norm() {
    require();
    return storage_->calc_grad_global_l2_norm(graph_id_, use_amp_master_);
  }
  void zero_grad() {
    require();
    storage_->clear_param_grads(graph_id_);
  }
  bool use_amp_master_params() const { return use_amp_master_; }
  void align_params() {
    require();
    storage_->align_buffer_zero(graph_id_);
  }
  void sync_param_zero(bool grad) {                          // the all-gather of one segment into its own buffer
    (void)grad;
    require();
  }
  void set_grad_to_local_param_segment() {
    require();
    storage_->set_grad_to_local_param_segment(graph_id_);
  }
  std::pair<int64_t, int64_t> get_local_param_range(long pid) {
    require();
    return storage_->get_local_param_range(graph_id_, pid);
  }
  at::Tensor get_local_param_segment(long pid) {
    require();
    return storage_->get_local_param_segment(graph_id_, pid);
  }
  at::Tensor owned(long pid, bool amp_master) const {
    if (amp_master && storage_->has_amp_master_param(pid)) return storage_->get_amp_master_param_tensor(pid);
    return storage_->get_param_tensor(pid);
  }
  // Under ZeRO the tensor this process steps on is a flat local segment; callers get it in the parameter's shape
  // (ParamStorage::doGatherParam -> gatherTensorZero, src/comp/ParamStorage.cpp:1201-1232, 670-685).
  at::Tensor in_param_shape(const at::Tensor& ten, long pid) const {
    const at::Tensor& p = storage_->get_param_tensor(pid);
    if (ten.sizes() != p.sizes() && ten.numel() == p.numel()) return ten.detach().view(p.sizes());
    return ten;
  }
  at::Tensor get_param(long pid, bool amp_master) {
    require();
    return in_param_shape(owned(pid, amp_master), pid);
  }
  at::Tensor get_param_grad(long pid, bool amp_master) {     // gatherParamGrad (src/comp/ParamStorage.cpp:1197-1213)
    require();
    const at::Tensor o = owned(pid, amp_master);
    if (o.grad().defined()) return in_param_shape(o.grad(), pid);
    if (!o.is_cuda()) return in_param_shape(at::zeros_like(o.detach()), pid);   // a host tensor never reaches a kernel
    at::Tensor z = at::empty_like(o.detach());
    if (z.numel() > 0)
      check(rg_fill_zero(z.data_ptr(), (int64_t)z.numel() * (int64_t)z.element_size(), z.get_device(), current_stream(z.get_device())));
    return in_param_shape(z, pid);
  }
  // doSyncParam + bcastParam (src/comp/ParamStorage.cpp:1079-1133) at one rank: the root's copy on the host
  py::object sync(long pid, bool grad) {
    require();
    if (!storage_->has_param(pid)) return py::none();
    const at::Tensor& p = storage_->get_param_tensor(pid);
    if (grad && !p.grad().defined()) return py::cast(at::zeros(p.sizes(), p.options().device(at::kCPU).requires_grad(false)));
    return py::cast((grad ? p.grad() : p).detach().clone().cpu());
  }
  void undeploy() {
    if (deployed_) {
      storage_->undeploy(graph_id_);
      deployed_ = false;
      staging_.clear();
    }
  }

 private:
  std::shared_ptr<ParamStorage> storage_;
  bool use_amp_master_, allreduce_amp_master_, enable_zero_;
  bool deployed_ = false;
  std::string graph_id_;
  std::vector<at::Tensor> staging_;
};

}  // namespace

void reset_registry() {
  global_storage()->clear();
  global_storage() = std::make_shared<ParamStorage>();
}

void bind_registry(py::module_& m) {
  // amp masters (src/main.cpp:191-200): the master is registered under the id of the model parameter it belongs to
  m.def("register_amp_master_param", [](long model_param_id, const py::object& param) {
    const at::Tensor t = tensor_or_undefined(param, "register_amp_master_param");
    if (!t.defined()) throw std::invalid_argument("register_amp_master_param expects a tensor");
    global_storage()->register_amp_master_param(model_param_id, object_id(param), t);
  });
  m.def("get_amp_master_param", [](long model_param_id) { return global_storage()->get_amp_master_param_tensor(model_param_id); });

  py::class_<TensorList, std::shared_ptr<TensorList>>(m, "TensorList")
      .def(py::init<const py::object&>(), py::arg("tensors"))
      .def("__len__", &TensorList::size)
      .def("tensors", [](const TensorList& l) { return l.tensors(); })
      .def("count_grads", &TensorList::count_grads)
      .def("steady_grads", [](const TensorList& l, const py::object& dtype) {
             bool ok = false;
             const int n = l.count_usable_grads(torch::python::detail::py_object_to_dtype(dtype), &ok);
             return ok ? n : -1;
           }, "number of tensors with a gradient; -1 unless each of those gradients is a contiguous GPU tensor of `dtype` and of its owner's size")
      .def("grads", &TensorList::grads)
      .def("set_grads", &TensorList::set_grads)
      .def("clear_grads", &TensorList::clear_grads);

  py::class_<GradPlan>(m, "GradPlan")
      .def(py::init<std::shared_ptr<TensorList>, std::shared_ptr<TensorList>>(), py::arg("owners"), py::arg("dsts") = nullptr)
      .def("bind", &GradPlan::bind)
      .def("rebuilt", &GradPlan::rebuilt)
      .def("bind_steady", [](GradPlan& p, TensorList& masters, const py::object& dtype) {
             return p.bind_steady(masters, torch::python::detail::py_object_to_dtype(dtype));
           })
      .def("push_sources_to_optim", &GradPlan::push_sources_to_optim, py::arg("optim_handle"), py::arg("offset"), py::arg("count"))
      .def("forget_optim", &GradPlan::forget_optim)
      .def("held", &GradPlan::held)
      .def("source_dtype", &GradPlan::source_dtype)
      .def("drop_sources", &GradPlan::drop_sources)
      .def("sources", &GradPlan::sources)
      .def("fused_step", &GradPlan::fused_step, py::arg("inv_scale"), py::arg("max_norm"), py::arg("flags") = 0)
      .def("step_begin", &GradPlan::step_begin)
      .def("step_begin_scaled", &GradPlan::step_begin_scaled, py::arg("inv_scale_device_ptr"))
      .def("step_finish", &GradPlan::step_finish, py::arg("max_norm"), py::arg("flags") = 0)
      .def("step_decide", &GradPlan::step_decide, py::arg("max_norm"), py::arg("flags") = 0)
      .def("unscale_pack", &GradPlan::unscale_pack)
      .def("step_apply_clip", &GradPlan::step_apply_clip, py::arg("max_norm"), py::arg("flags") = 0)
      .def("unscale_accumulate", &GradPlan::unscale_accumulate)
      .def("grad_norm", &GradPlan::grad_norm)
      .def("scale_cast", &GradPlan::scale_cast, py::arg("scale") = 1.0f)
      .def("zero", &GradPlan::zero)
      .def("tune", &GradPlan::tune)
      .def("write_order", &GradPlan::write_order)
      .def("set_write_order", &GradPlan::set_write_order)
      .def("result", &GradPlan::result)
      .def("result_device_ptr", &GradPlan::result_device_ptr)
      .def("is_open", &GradPlan::is_open)
      .def("close", &GradPlan::close)
      .def_property_readonly("num_chunks", &GradPlan::num_chunks)
      .def_property_readonly("handle", &GradPlan::handle);

  py::class_<GradBuckets>(m, "GradBuckets")
      .def(py::init<std::shared_ptr<TensorList>, std::shared_ptr<TensorList>>(), py::arg("params"), py::arg("views"))
      .def("consolidate", &GradBuckets::consolidate);

  py::class_<ParamStorage, std::shared_ptr<ParamStorage>>(m, "ParamStorage")
      .def(py::init<>())
      .def("register_param", &ParamStorage::register_param)
      .def("get_param_tensor", &ParamStorage::get_param_tensor)
      .def("has_param", &ParamStorage::has_param)
      .def("register_amp_master_param", &ParamStorage::register_amp_master_param)
      .def("has_amp_master_param", &ParamStorage::has_amp_master_param)
      .def("get_amp_master_param_tensor", &ParamStorage::get_amp_master_param_tensor)
      .def("deploy", &ParamStorage::deploy, py::arg("graph_id"), py::arg("graph_params"), py::arg("enable_zero") = false,
           py::arg("consolidate") = false, py::arg("use_amp_master_params") = false, py::arg("allreduce_amp_master_params") = false)
      .def("undeploy", &ParamStorage::undeploy)
      .def("deployed", &ParamStorage::deployed)
      .def("sorted_param_ids", &ParamStorage::sorted_param_ids)
      .def("zero_enabled", &ParamStorage::zero_enabled)
      .def("set_consolidated_grads", &ParamStorage::set_consolidated_grads)
      .def("calc_grad_global_l2_norm", &ParamStorage::calc_grad_global_l2_norm)
      .def("clip_grad_norm", &ParamStorage::clip_grad_norm)
      .def("do_scale_grads", &ParamStorage::do_scale_grads)
      .def("clear_param_grads", &ParamStorage::clear_param_grads)
      .def("allreduce_param_grads_zero", &ParamStorage::allreduce_param_grads_zero)
      .def("get_local_param_range", &ParamStorage::get_local_param_range)
      .def("get_local_param_segment", &ParamStorage::get_local_param_segment)
      .def("set_grad_to_local_param_segment", &ParamStorage::set_grad_to_local_param_segment)
      .def("align_buffer_zero", &ParamStorage::align_buffer_zero)
      .def("get_buffer", &ParamStorage::get_buffer)
      .def("get_buffer_segment", &ParamStorage::get_buffer_segment)
      .def("gather_tensor_zero", &ParamStorage::gather_tensor_zero)
      .def("selected", &ParamStorage::selected)
      .def("clear", &ParamStorage::clear);
  m.def("get_param_storage", [] { return global_storage(); },
        "the registry the RaNNCModule objects and register_amp_master_param of this module work on");
  m.def("reset_param_storage", &reset_registry);

  py::class_<RaNNCModule>(m, "RaNNCModule")
      .def(py::init<bool, bool, bool, bool, bool>(), py::arg("use_amp_master_params") = false,
           py::arg("allreduce_amp_master_params") = false, py::arg("enable_zero") = false, py::arg("check_unused_values") = true,
           py::arg("offload_params") = false)
      .def("init", &RaNNCModule::init, py::arg("named_params"), py::arg("consolidate_grads") = false)
      .def_property_readonly("native_graph_id", &RaNNCModule::graph_id)
      .def("allreduce_grads", &RaNNCModule::allreduce_grads)
      .def("allreduce_grads_zero", &RaNNCModule::allreduce_grads_zero)
      .def("clip_grad_norm", &RaNNCModule::clip_grad_norm)
      .def("calc_grad_norm", &RaNNCModule::calc_grad_norm)
      .def("zero_grad", &RaNNCModule::zero_grad)
      .def("use_amp_master_params", &RaNNCModule::use_amp_master_params)
      .def("undeploy", &RaNNCModule::undeploy)
      .def("align_params", &RaNNCModule::align_params)
      .def("sync_param", [](RaNNCModule& self, long pid) { return self.sync(pid, false); })
      .def("sync_param_grad", [](RaNNCModule& self, long pid) { return self.sync(pid, true); })
      .def("sync_param_zero", &RaNNCModule::sync_param_zero)
      .def("set_grad_to_local_param_segment", &RaNNCModule::set_grad_to_local_param_segment)
      .def("get_local_param_range", &RaNNCModule::get_local_param_range)
      .def("get_local_param_segment", &RaNNCModule::get_local_param_segment)
      .def("get_param", &RaNNCModule::get_param)
      .def("get_param_grad", &RaNNCModule::get_param_grad);
}
