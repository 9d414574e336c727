// torchopt_amd._C -- the PyTorch-ROCm extension module in front of libtoa_adam.so.
//
// Counterpart of the reference's pybind11 module: PYBIND11_MODULE(_C) with one
// submodule, `adam_op` (/root/reference/src/extension.cpp:20,
// /root/reference/src/adam_op/adam_op.cpp:155-215).  Same seven functions, same
// keyword names (including backward_nu's fourth keyword being registered as
// "b1", adam_op.cpp:203), same conversions (double for floats, size_t for
// `count`, so a 0-dim integer tensor is accepted through __index__), same
// return conventions (std::array -> list; forward_ hands back its inputs), same
// exception classes.  It is thin on purpose: checks, empty_like, device and
// stream, then one call into the C ABI (include/toa_adam.h).  No arithmetic
// happens here and no torch type crosses the ABI.
//
// Deliberate differences from the reference dispatcher (adam_op.cpp:32-153):
//   * only GPU tensors are served; every other device raises
//     std::runtime_error("Not implemented"), the reference's own error for a
//     device it has no kernel for (adam_op.cpp:47-49);
//   * kernels go to PyTorch's current stream of the tensors' device instead of
//     the null stream (adam_op_impl_cuda.cu:83);
//   * element counts, dtypes, devices and memory layouts are checked instead of
//     assumed;
//   * additive list entry points (forward_multi_, ...) and the fused optimizer
//     step (fused_step_, fused_step_multi_).
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>
#include <pybind11/stl.h>
#include <ATen/FuncTorchTLS.h>
#include <torch/csrc/autograd/function.h>
#include <torch/csrc/autograd/functions/utils.h>
#include <torch/csrc/autograd/saved_variable.h>
#include <torch/extension.h>

#include <array>
#include <stdexcept>
#include <string>
#include <vector>

#include "toa_adam.h"

namespace py = pybind11;

namespace {

using at::Tensor;
using TensorList = std::vector<Tensor>;

int dtypeCode(const Tensor &t, const char *name) {
    switch (t.scalar_type()) {
        case at::kFloat: return TOA_F32;
        case at::kDouble: return TOA_F64;
        case at::kHalf: return TOA_F16;
        case at::kBFloat16: return TOA_BF16;
        default:
            // wording of ATen's dispatch failure, which is what the reference raises
            TORCH_CHECK(false, "\"", name, "\" not implemented for '", t.scalar_type(), "'");
    }
}

void check(int rc, const char *name) {
    TORCH_CHECK(rc == 0, name, ": ", toa_adam_error_string(rc), " (code ", rc, ")");
}

// Device, dtype and size agreement; returns the dtype code and sets n.
int gate(const char *name, const Tensor &lead, std::initializer_list<const Tensor *> others,
         size_t *n) {
    if (!lead.is_cuda()) throw std::runtime_error("Not implemented");
    const int code = dtypeCode(lead, name);
    *n = (size_t)lead.numel();
    for (const Tensor *t : others) {
        TORCH_CHECK(t->device() == lead.device(), name, ": expected all tensors on ",
                    lead.device(), ", got one on ", t->device());
        TORCH_CHECK(t->scalar_type() == lead.scalar_type(), name, ": expected scalar type ",
                    lead.scalar_type(), " but found ", t->scalar_type());
        TORCH_CHECK((size_t)t->numel() == *n, name, ": size mismatch, ", *n, " vs ", t->numel(),
                    " elements");
    }
    return code;
}

void requireDense(const char *name, const char *what, const Tensor &t) {
    TORCH_CHECK(t.is_non_overlapping_and_dense(), name, ": `", what,
                "` must be contiguous (non-overlapping and dense), got sizes ", t.sizes(),
                " strides ", t.strides());
}

bool sameLayout(const Tensor &a, const Tensor &b) {
    return a.numel() <= 1 || a.strides() == b.strides();
}

// A read-only operand in the memory order of `donor`, copying only if it is not already.
// (The reference makes incoming gradients .contiguous(), adam_op.cpp:107,123,143.)
Tensor asLayoutOf(const Tensor &x, const Tensor &donor) {
    if (x.numel() <= 1 || (x.is_contiguous() && donor.is_contiguous())) return x;
    // a wrong device or dtype is the gate's to report, not to be papered over by a copy
    if (x.device() != donor.device() || x.scalar_type() != donor.scalar_type()) return x;
    if (x.sizes() == donor.sizes())
        return x.strides() == donor.strides() ? x : at::empty_like(donor).copy_(x);
    TORCH_CHECK(donor.is_contiguous(), "operands of different shapes must be contiguous");
    return x.contiguous();
}

// Makes the tensors' device current for the launch (the C ABI uses the current device) and
// hands out PyTorch's current stream on it.
class OnDeviceOf {
  public:
    explicit OnDeviceOf(const Tensor &t) : index_((int)t.get_device()) {
        if (hipGetDevice(&prev_) != hipSuccess) prev_ = index_;
        if (prev_ != index_) TORCH_CHECK(hipSetDevice(index_) == hipSuccess, "hipSetDevice failed");
    }
    ~OnDeviceOf() {
        if (prev_ != index_) (void)hipSetDevice(prev_);
    }
    void *stream() const {
        return (void *)c10::hip::getCurrentHIPStream((c10::DeviceIndex)index_).stream();
    }

  private:
    int index_;
    int prev_ = 0;
};

// ---- single tensor -------------------------------------------------------------------------

std::array<Tensor, 3> forwardInplace(const Tensor &updates, const Tensor &mu, const Tensor &nu,
                                     double b1, double b2, double eps, double eps_root,
                                     size_t count) {
    const char *name = "adamForwardInplace";
    size_t n;
    const int code = gate(name, updates, {&mu, &nu}, &n);
    if (n) {
        requireDense(name, "updates", updates);
        requireDense(name, "mu", mu);
        requireDense(name, "nu", nu);
        TORCH_CHECK(sameLayout(updates, mu) && sameLayout(updates, nu), name,
                    ": updates, mu and nu must share one memory layout");
        const OnDeviceOf dev(updates);
        check(toa_adam_forward_inplace(code, updates.data_ptr(), mu.data_ptr(), nu.data_ptr(), n,
                                       b1, b2, eps, eps_root, count, dev.stream()),
              name);
    }
    return {updates, mu, nu};
}

Tensor forwardMu(const Tensor &updates_in, const Tensor &mu, double b1) {
    const char *name = "adamForwardMu";
    size_t n;
    const int code = gate(name, updates_in, {&mu}, &n);
    requireDense(name, "mu", mu);
    Tensor mu_out = at::empty_like(mu);
    if (n) {
        const Tensor updates = asLayoutOf(updates_in, mu);
        const OnDeviceOf dev(mu);
        check(toa_adam_forward_mu(code, updates.data_ptr(), mu.data_ptr(), n, b1,
                                  mu_out.data_ptr(), dev.stream()),
              name);
    }
    return mu_out;
}

Tensor forwardNu(const Tensor &updates_in, const Tensor &nu, double b2) {
    const char *name = "adamForwardNu";
    size_t n;
    const int code = gate(name, updates_in, {&nu}, &n);
    requireDense(name, "nu", nu);
    Tensor nu_out = at::empty_like(nu);
    if (n) {
        const Tensor updates = asLayoutOf(updates_in, nu);
        const OnDeviceOf dev(nu);
        check(toa_adam_forward_nu(code, updates.data_ptr(), nu.data_ptr(), n, b2,
                                  nu_out.data_ptr(), dev.stream()),
              name);
    }
    return nu_out;
}

Tensor forwardUpdates(const Tensor &new_mu, const Tensor &new_nu_in, double b1, double b2,
                      double eps, double eps_root, size_t count) {
    const char *name = "adamForwardUpdates";
    size_t n;
    const int code = gate(name, new_mu, {&new_nu_in}, &n);
    requireDense(name, "new_mu", new_mu);
    Tensor updates_out = at::empty_like(new_mu);
    if (n) {
        const Tensor new_nu = asLayoutOf(new_nu_in, new_mu);
        const OnDeviceOf dev(new_mu);
        check(toa_adam_forward_updates(code, new_mu.data_ptr(), new_nu.data_ptr(), n, b1, b2, eps,
                                       eps_root, count, updates_out.data_ptr(), dev.stream()),
              name);
    }
    return updates_out;
}

std::array<Tensor, 2> backwardMu(const Tensor &dmu_in, const Tensor &updates, const Tensor &mu,
                                 double b1) {
    const char *name = "adamBackwardMu";
    size_t n;
    const int code = gate(name, dmu_in, {&updates, &mu}, &n);
    requireDense(name, "updates", updates);
    requireDense(name, "mu", mu);
    Tensor dupdates_out = at::empty_like(updates);
    Tensor dmu_out = at::empty_like(mu);
    if (n) {
        TORCH_CHECK(sameLayout(dupdates_out, dmu_out), name,
                    ": updates and mu must share one memory layout");
        const Tensor dmu = asLayoutOf(dmu_in, dmu_out);
        const OnDeviceOf dev(dmu);
        check(toa_adam_backward_mu(code, dmu.data_ptr(), n, b1, dupdates_out.data_ptr(),
                                   dmu_out.data_ptr(), dev.stream()),
              name);
    }
    return {dupdates_out, dmu_out};
}

std::array<Tensor, 2> backwardNu(const Tensor &dnu_in, const Tensor &updates, const Tensor &nu,
                                 double b2) {
    const char *name = "adamBackwardNu";
    size_t n;
    const int code = gate(name, dnu_in, {&updates, &nu}, &n);
    requireDense(name, "updates", updates);
    requireDense(name, "nu", nu);
    Tensor dupdates_out = at::empty_like(updates);
    Tensor dnu_out = at::empty_like(nu);
    if (n) {
        TORCH_CHECK(sameLayout(dupdates_out, dnu_out), name,
                    ": updates and nu must share one memory layout");
        const Tensor dnu = asLayoutOf(dnu_in, dnu_out);
        const OnDeviceOf dev(dnu);
        check(toa_adam_backward_nu(code, dnu.data_ptr(), updates.data_ptr(), n, b2,
                                   dupdates_out.data_ptr(), dnu_out.data_ptr(), dev.stream()),
              name);
    }
    return {dupdates_out, dnu_out};
}

std::array<Tensor, 2> backwardUpdates(const Tensor &dupdates_in, const Tensor &updates_in,
                                      const Tensor &new_mu, const Tensor &new_nu, double b1,
                                      double b2, double eps_root, size_t count) {
    const char *name = "adamBackwardUpdates";
    size_t n;
    const int code = gate(name, dupdates_in, {&updates_in, &new_mu, &new_nu}, &n);
    requireDense(name, "new_mu", new_mu);
    requireDense(name, "new_nu", new_nu);
    Tensor dmu_out = at::empty_like(new_mu);
    Tensor dnu_out = at::empty_like(new_nu);
    if (n) {
        TORCH_CHECK(sameLayout(dmu_out, dnu_out), name,
                    ": new_mu and new_nu must share one memory layout");
        const Tensor dupdates = asLayoutOf(dupdates_in, dmu_out);
        const Tensor updates = asLayoutOf(updates_in, dmu_out);
        const OnDeviceOf dev(dupdates);
        check(toa_adam_backward_updates(code, dupdates.data_ptr(), updates.data_ptr(),
                                        new_mu.data_ptr(), n, b1, b2, eps_root, count,
                                        dmu_out.data_ptr(), dnu_out.data_ptr(), dev.stream()),
              name);
    }
    return {dmu_out, dnu_out};
}

// The differentiable step in one pass per direction (no single counterpart in the reference;
// results equal forward_mu / forward_nu / forward_updates and the backward chain bit for bit).
std::array<Tensor, 3> forwardAll(const Tensor &updates_in, const Tensor &mu, const Tensor &nu_in,
                                 double b1, double b2, double eps, double eps_root,
                                 size_t count) {
    const char *name = "adamForwardAll";
    size_t n;
    const int code = gate(name, updates_in, {&mu, &nu_in}, &n);
    requireDense(name, "mu", mu);
    Tensor new_mu = at::empty_like(mu), new_nu = at::empty_like(mu), new_updates = at::empty_like(mu);
    if (n) {
        const Tensor updates = asLayoutOf(updates_in, mu);
        const Tensor nu = asLayoutOf(nu_in, mu);
        const OnDeviceOf dev(mu);
        check(toa_adam_forward_all(code, updates.data_ptr(), mu.data_ptr(), nu.data_ptr(), n, b1,
                                   b2, eps, eps_root, count, new_mu.data_ptr(), new_nu.data_ptr(),
                                   new_updates.data_ptr(), dev.stream()),
              name);
    }
    return {new_mu, new_nu, new_updates};
}

// dnew_mu / dnew_nu: gradients reaching new_mu / new_nu from outside the step, or None.
std::array<Tensor, 3> backwardAll(const Tensor &dnew_updates_in,
                                  const c10::optional<Tensor> &dnew_mu_in,
                                  const c10::optional<Tensor> &dnew_nu_in,
                                  const Tensor &new_updates_in, const Tensor &new_mu,
                                  const Tensor &updates_in, double b1, double b2, double eps_root,
                                  size_t count) {
    const char *name = "adamBackwardAll";
    size_t n;
    const int code = gate(name, dnew_updates_in, {&new_updates_in, &new_mu, &updates_in}, &n);
    requireDense(name, "new_mu", new_mu);
    Tensor dupdates = at::empty_like(new_mu), dmu = at::empty_like(new_mu),
           dnu = at::empty_like(new_mu);
    if (n) {
        const Tensor du = asLayoutOf(dnew_updates_in, new_mu);
        const Tensor nu_ = asLayoutOf(new_updates_in, new_mu);
        const Tensor up = asLayoutOf(updates_in, new_mu);
        Tensor dm, dv;
        for (auto pair : {std::make_pair(&dnew_mu_in, &dm), std::make_pair(&dnew_nu_in, &dv)}) {
            if (!pair.first->has_value()) continue;
            const Tensor &t = pair.first->value();
            TORCH_CHECK(t.device() == new_mu.device() && t.scalar_type() == new_mu.scalar_type() &&
                            (size_t)t.numel() == n,
                        name, ": outside gradient does not match new_mu");
            *pair.second = asLayoutOf(t, new_mu);
        }
        const OnDeviceOf dev(new_mu);
        check(toa_adam_backward_all(code, du.data_ptr(), nu_.data_ptr(), new_mu.data_ptr(),
                                    up.data_ptr(), dm.defined() ? dm.data_ptr() : nullptr,
                                    dv.defined() ? dv.data_ptr() : nullptr, n, b1, b2, eps_root,
                                    count, dupdates.data_ptr(), dmu.data_ptr(), dnu.data_ptr(),
                                    dev.stream()),
              name);
    }
    return {dupdates, dmu, dnu};
}

std::array<Tensor, 4> fusedStep(const Tensor &params, const Tensor &updates_in, const Tensor &mu,
                                const Tensor &nu, double b1, double b2, double eps,
                                double eps_root, size_t count, double lr, bool maximize,
                                bool write_updates, double weight_decay, bool decoupled) {
    const char *name = "adamFusedStep";
    size_t n;
    const int code = gate(name, params, {&mu, &nu, &updates_in}, &n);
    // a gradient that is only read may come in any layout
    const Tensor updates = (n && !write_updates && params.is_non_overlapping_and_dense())
                               ? asLayoutOf(updates_in, params) : updates_in;
    if (n) {
        requireDense(name, "params", params);
        requireDense(name, "updates", updates);
        requireDense(name, "mu", mu);
        requireDense(name, "nu", nu);
        TORCH_CHECK(sameLayout(params, updates) && sameLayout(params, mu) && sameLayout(params, nu),
                    name, ": params, updates, mu and nu must share one memory layout");
        const OnDeviceOf dev(params);
        check(toa_adam_fused_step(code, params.data_ptr(), updates.data_ptr(), mu.data_ptr(),
                                  nu.data_ptr(), n, b1, b2, eps, eps_root, count, lr,
                                  weight_decay, (int)decoupled, (int)maximize,
                                  (int)write_updates, dev.stream()),
              name);
    }
    return {params, updates_in, mu, nu};
}

// ---- lists of tensors ----------------------------------------------------------------------

struct Lists {
    int code = TOA_F32;
    size_t num = 0;
    std::vector<size_t> n;
    std::vector<std::vector<void *>> ptr;  // one vector per operand list
};

// Checks for a list call: equal lengths, one device and dtype, per-tensor size agreement and a
// shared dense layout.  Collects sizes and data pointers on the way.
Lists gateLists(const char *name, std::initializer_list<const TensorList *> lists) {
    Lists out;
    const TensorList &first = **lists.begin();
    out.num = first.size();
    for (const TensorList *l : lists)
        TORCH_CHECK(l->size() == out.num, name, ": tensor lists differ in length");
    if (out.num == 0) return out;
    const Tensor &lead = first[0];
    if (!lead.is_cuda()) throw std::runtime_error("Not implemented");
    out.code = dtypeCode(lead, name);
    out.n.resize(out.num);
    for (size_t k = 0; k < out.num; ++k) out.n[k] = (size_t)first[k].numel();
    for (const TensorList *l : lists) {
        std::vector<void *> p(out.num);
        for (size_t k = 0; k < out.num; ++k) {
            const Tensor &t = (*l)[k];
            TORCH_CHECK(t.device() == lead.device(), name,
                        ": all tensors of one call must be on ", lead.device());
            TORCH_CHECK(t.scalar_type() == lead.scalar_type(), name, ": expected scalar type ",
                        lead.scalar_type(), " but found ", t.scalar_type());
            TORCH_CHECK((size_t)t.numel() == out.n[k], name, ": size mismatch in tensor ", k);
            if (out.n[k] > 1)
                TORCH_CHECK(t.is_non_overlapping_and_dense() && t.strides() == first[k].strides(),
                            name, ": tensor ", k, " operands must share one dense layout");
            p[k] = out.n[k] ? t.data_ptr() : nullptr;
        }
        out.ptr.push_back(std::move(p));
    }
    return out;
}

struct Counts {
    std::vector<uint64_t> each;  // empty when one value serves all
    uint64_t all = 0;
    const uint64_t *data() const { return each.empty() ? nullptr : each.data(); }
};

uint64_t toCount(const py::handle &h) {
    // what pybind11 does for a size_t parameter: __index__, non-negative
    py::object idx = py::reinterpret_steal<py::object>(PyNumber_Index(h.ptr()));
    if (!idx) throw py::error_already_set();
    if (PyObject_RichCompareBool(idx.ptr(), py::int_(0).ptr(), Py_LT) == 1)
        throw py::type_error("count must be a non-negative integer");
    return idx.cast<uint64_t>();
}

// `counts`: one step number for all tensors, or a list/tuple with one per tensor (ints or
// 0-dim integer tensors; a list of device tensors is read back with one transfer).
Counts parseCounts(const py::object &counts, size_t num) {
    Counts out;
    if (!py::isinstance<py::list>(counts) && !py::isinstance<py::tuple>(counts)) {
        out.all = toCount(counts);
        return out;
    }
    const py::sequence seq = py::reinterpret_borrow<py::sequence>(counts);
    TORCH_CHECK((size_t)py::len(seq) == num, "expected ", num, " counts, got ", py::len(seq));
    std::vector<uint64_t> values(num);
    bool all_tensors = num > 0;
    for (const py::handle &h : seq) all_tensors = all_tensors && THPVariable_Check(h.ptr());
    if (all_tensors) {
        TensorList ts;
        ts.reserve(num);
        for (const py::handle &h : seq) ts.push_back(THPVariable_Unpack(h.ptr()).reshape({}));
        const Tensor host = at::stack(ts).to(at::kLong).cpu();
        const int64_t *v = host.data_ptr<int64_t>();
        for (size_t k = 0; k < num; ++k) {
            if (v[k] < 0) throw py::type_error("counts must be non-negative integers");
            values[k] = (uint64_t)v[k];
        }
    } else {
        size_t k = 0;
        for (const py::handle &h : seq) values[k++] = toCount(h);
    }
    bool uniform = true;
    for (size_t k = 1; k < num; ++k) uniform = uniform && values[k] == values[0];
    if (uniform)
        out.all = num ? values[0] : 0;
    else
        out.each = std::move(values);
    return out;
}

// `sets` lists of outputs shaped like `donors` (dtype, device, sizes and strides as
// at::empty_like gives them).  Leaves below 1 MiB share ONE allocation per call, each starting on
// a 256-byte boundary: a tree of small leaves -- where the step is bound by host time, not
// bandwidth -- then costs one trip to the allocator instead of one per leaf and list (2-3 us
// each).  The leaves do not overlap; what they share is the storage's lifetime (it lives as long
// as any of them) and torch.save of a single leaf writing the whole storage.  Larger leaves get
// an allocation each, and so do the leaves that would take the shared allocation beyond 64 MiB:
// what one surviving leaf can keep alive stays bounded, and past that size the step is no longer
// bound by host time.
constexpr size_t kPooledLeafBytes = (size_t)1 << 20;
constexpr size_t kPoolMaxBytes = (size_t)64 << 20;

std::vector<TensorList> emptyLikeSets(const TensorList &donors, size_t sets) {
    std::vector<TensorList> out(sets, TensorList(donors.size()));
    std::vector<size_t> at(donors.size());
    size_t pooled = 0, bytes = 0, first = 0;
    for (size_t k = 0; k < donors.size(); ++k) {
        const Tensor &d = donors[k];
        const size_t need = (size_t)d.numel() * d.element_size();
        at[k] = SIZE_MAX;
        if (!d.is_cuda() || need == 0 || need >= kPooledLeafBytes ||
            !d.is_non_overlapping_and_dense() || d.layout() != at::kStrided)
            continue;
        if (pooled != 0 && d.device() != donors[first].device()) continue;
        const size_t padded = (need + 255) / 256 * 256;
        if ((bytes + padded) * sets > kPoolMaxBytes) continue;
        if (pooled++ == 0) first = k;
        at[k] = bytes;
        bytes += padded;
    }
    if (pooled * sets >= 2) {
        const Tensor pool =
            at::empty({(int64_t)(bytes * sets)}, donors[first].options().dtype(at::kByte));
        const c10::Storage &storage = pool.storage();
        for (size_t j = 0; j < sets; ++j)
            for (size_t k = 0; k < donors.size(); ++k) {
                if (at[k] == SIZE_MAX) continue;
                const Tensor &d = donors[k];
                Tensor t = at::detail::make_tensor<c10::TensorImpl>(c10::Storage(storage),
                                                                     pool.key_set(), d.dtype());
                c10::TensorImpl *impl = t.unsafeGetTensorImpl();
                impl->set_storage_offset((int64_t)((j * bytes + at[k]) / d.element_size()));
                impl->set_sizes_and_strides(d.sizes(), d.strides());
                out[j][k] = std::move(t);
            }
    }
    for (size_t j = 0; j < sets; ++j)
        for (size_t k = 0; k < donors.size(); ++k)
            if (!out[j][k].defined()) out[j][k] = at::empty_like(donors[k]);
    return out;
}

TensorList emptyLike(const TensorList &donors) { return std::move(emptyLikeSets(donors, 1)[0]); }

TensorList asLayoutOfEach(const TensorList &xs, const TensorList &donors, const char *name) {
    TORCH_CHECK(xs.size() == donors.size(), name, ": tensor lists differ in length");
    TensorList out;
    out.reserve(xs.size());
    for (size_t k = 0; k < xs.size(); ++k) out.push_back(asLayoutOf(xs[k], donors[k]));
    return out;
}

// Any member names the device of a list call (gateLists has checked they agree).
const Tensor &deviceDonor(const TensorList &l) { return l[0]; }

// A Python list or tuple of tensors -> TensorList without the generic sequence caster (which
// costs ~40 ns per element; long lists of small tensors are bound by exactly this).
TensorList toTensorList(const py::object &o, const char *what) {
    PyObject *seq = o.ptr();
    const bool is_list = PyList_Check(seq);
    if (!is_list && !PyTuple_Check(seq)) return o.cast<TensorList>();
    const Py_ssize_t num = is_list ? PyList_GET_SIZE(seq) : PyTuple_GET_SIZE(seq);
    TensorList out;
    out.reserve((size_t)num);
    for (Py_ssize_t k = 0; k < num; ++k) {
        PyObject *item = is_list ? PyList_GET_ITEM(seq, k) : PyTuple_GET_ITEM(seq, k);
        if (!THPVariable_Check(item))
            throw py::type_error(std::string(what) + ": expected a list of tensors");
        out.push_back(THPVariable_Unpack(item));
    }
    return out;
}

// True when `o` is a non-empty list or tuple whose members are all tensors of one device and one
// dtype: what a caller must know before it hands a whole tree to one list call, asked in C
// instead of a Python loop over the leaves.
bool oneKind(const py::object &o) {
    PyObject *seq = o.ptr();
    const bool is_list = PyList_Check(seq);
    if (!is_list && !PyTuple_Check(seq)) return false;
    const Py_ssize_t num = is_list ? PyList_GET_SIZE(seq) : PyTuple_GET_SIZE(seq);
    if (num == 0) return false;
    const Tensor *first = nullptr;
    for (Py_ssize_t k = 0; k < num; ++k) {
        PyObject *item = is_list ? PyList_GET_ITEM(seq, k) : PyTuple_GET_ITEM(seq, k);
        if (!THPVariable_Check(item)) return false;
        const Tensor &t = THPVariable_Unpack(item);
        if (!t.defined()) return false;
        if (first == nullptr)
            first = &t;
        else if (t.scalar_type() != first->scalar_type() || t.device() != first->device())
            return false;
    }
    return true;
}

py::tuple forwardMultiInplace(const py::object &updates_o, const py::object &mu_o,
                              const py::object &nu_o, double b1, double b2, double eps,
                              double eps_root, const py::object &counts) {
    const char *name = "adamForwardInplaceMulti";
    const auto updates = toTensorList(updates_o, "updates");
    const auto mu = toTensorList(mu_o, "mu");
    const auto nu = toTensorList(nu_o, "nu");
    Lists l = gateLists(name, {&updates, &mu, &nu});
    if (l.num) {
        const Counts c = parseCounts(counts, l.num);
        const OnDeviceOf dev(deviceDonor(updates));
        check(toa_adam_forward_inplace_multi(l.code, l.num, l.ptr[0].data(), l.ptr[1].data(),
                                             l.ptr[2].data(), l.n.data(), b1, b2, eps, eps_root,
                                             c.data(), c.all, dev.stream()),
              name);
    }
    return py::make_tuple(updates_o, mu_o, nu_o);  // the caller's own lists, mutated in place
}

TensorList forwardMuMulti(const TensorList &updates_in, const TensorList &mu, double b1) {
    const char *name = "adamForwardMuMulti";
    TensorList out = emptyLike(mu);
    const TensorList updates = asLayoutOfEach(updates_in, mu, name);
    Lists l = gateLists(name, {&mu, &updates, &out});
    if (l.num) {
        const OnDeviceOf dev(deviceDonor(mu));
        check(toa_adam_forward_mu_multi(l.code, l.num, l.ptr[1].data(), l.ptr[0].data(),
                                        l.n.data(), b1, l.ptr[2].data(), dev.stream()),
              name);
    }
    return out;
}

TensorList forwardNuMulti(const TensorList &updates_in, const TensorList &nu, double b2) {
    const char *name = "adamForwardNuMulti";
    TensorList out = emptyLike(nu);
    const TensorList updates = asLayoutOfEach(updates_in, nu, name);
    Lists l = gateLists(name, {&nu, &updates, &out});
    if (l.num) {
        const OnDeviceOf dev(deviceDonor(nu));
        check(toa_adam_forward_nu_multi(l.code, l.num, l.ptr[1].data(), l.ptr[0].data(),
                                        l.n.data(), b2, l.ptr[2].data(), dev.stream()),
              name);
    }
    return out;
}

TensorList forwardUpdatesMulti(const TensorList &new_mu, const TensorList &new_nu_in, double b1,
                               double b2, double eps, double eps_root, const py::object &counts) {
    const char *name = "adamForwardUpdatesMulti";
    TensorList out = emptyLike(new_mu);
    const TensorList new_nu = asLayoutOfEach(new_nu_in, new_mu, name);
    Lists l = gateLists(name, {&new_mu, &new_nu, &out});
    if (l.num) {
        const Counts c = parseCounts(counts, l.num);
        const OnDeviceOf dev(deviceDonor(new_mu));
        check(toa_adam_forward_updates_multi(l.code, l.num, l.ptr[0].data(), l.ptr[1].data(),
                                             l.n.data(), b1, b2, eps, eps_root, c.data(), c.all,
                                             l.ptr[2].data(), dev.stream()),
              name);
    }
    return out;
}

std::tuple<TensorList, TensorList> backwardMuMulti(const TensorList &dmu_in,
                                                   const TensorList &updates,
                                                   const TensorList &mu, double b1) {
    const char *name = "adamBackwardMuMulti";
    TORCH_CHECK(updates.size() == mu.size(), name, ": tensor lists differ in length");
    std::vector<TensorList> fresh = emptyLikeSets(mu, 2);
    TensorList &dupdates_out = fresh[0], &dmu_out = fresh[1];
    const TensorList dmu = asLayoutOfEach(dmu_in, dmu_out, name);
    Lists l = gateLists(name, {&dmu_out, &dmu, &dupdates_out});
    if (l.num) {
        const OnDeviceOf dev(deviceDonor(dmu));
        check(toa_adam_backward_mu_multi(l.code, l.num, l.ptr[1].data(), l.n.data(), b1,
                                         l.ptr[2].data(), l.ptr[0].data(), dev.stream()),
              name);
    }
    return {std::move(dupdates_out), std::move(dmu_out)};
}

std::tuple<TensorList, TensorList> backwardNuMulti(const TensorList &dnu_in,
                                                   const TensorList &updates_in,
                                                   const TensorList &nu, double b2) {
    const char *name = "adamBackwardNuMulti";
    std::vector<TensorList> fresh = emptyLikeSets(nu, 2);
    TensorList &dupdates_out = fresh[0], &dnu_out = fresh[1];
    const TensorList dnu = asLayoutOfEach(dnu_in, dnu_out, name);
    const TensorList updates = asLayoutOfEach(updates_in, nu, name);
    Lists l = gateLists(name, {&dnu, &updates, &dupdates_out, &dnu_out});
    if (l.num) {
        const OnDeviceOf dev(deviceDonor(dnu));
        check(toa_adam_backward_nu_multi(l.code, l.num, l.ptr[0].data(), l.ptr[1].data(),
                                         l.n.data(), b2, l.ptr[2].data(), l.ptr[3].data(),
                                         dev.stream()),
              name);
    }
    return {std::move(dupdates_out), std::move(dnu_out)};
}

std::tuple<TensorList, TensorList> backwardUpdatesMulti(
    const TensorList &dupdates_in, const TensorList &updates_in, const TensorList &new_mu,
    const TensorList &new_nu, double b1, double b2, double eps_root, const py::object &counts) {
    const char *name = "adamBackwardUpdatesMulti";
    TORCH_CHECK(new_nu.size() == new_mu.size(), name, ": tensor lists differ in length");
    std::vector<TensorList> fresh = emptyLikeSets(new_mu, 2);
    TensorList &dmu_out = fresh[0], &dnu_out = fresh[1];
    const TensorList dupdates = asLayoutOfEach(dupdates_in, dmu_out, name);
    const TensorList updates = asLayoutOfEach(updates_in, new_mu, name);
    Lists l = gateLists(name, {&dupdates, &updates, &new_mu, &dmu_out, &dnu_out});
    if (l.num) {
        const Counts c = parseCounts(counts, l.num);
        const OnDeviceOf dev(deviceDonor(dupdates));
        check(toa_adam_backward_updates_multi(l.code, l.num, l.ptr[0].data(), l.ptr[1].data(),
                                              l.ptr[2].data(), l.n.data(), b1, b2, eps_root,
                                              c.data(), c.all, l.ptr[3].data(), l.ptr[4].data(),
                                              dev.stream()),
              name);
    }
    return {std::move(dmu_out), std::move(dnu_out)};
}

std::tuple<TensorList, TensorList, TensorList> forwardAllMultiImpl(
    const TensorList &updates_in, const TensorList &mu, const TensorList &nu_in, double b1,
    double b2, double eps, double eps_root, const Counts &c) {
    const char *name = "adamForwardAllMulti";
    std::vector<TensorList> fresh = emptyLikeSets(mu, 3);
    TensorList &new_mu = fresh[0], &new_nu = fresh[1], &new_updates = fresh[2];
    // gradients may arrive expanded or in another memory order: bring them to mu's
    const TensorList updates = asLayoutOfEach(updates_in, mu, name);
    const TensorList nu = asLayoutOfEach(nu_in, mu, name);
    Lists l = gateLists(name, {&updates, &mu, &nu, &new_mu, &new_nu, &new_updates});
    if (l.num) {
        TORCH_CHECK(c.each.empty() || c.each.size() == l.num, name, ": expected ", l.num,
                    " counts, got ", c.each.size());
        const OnDeviceOf dev(deviceDonor(mu));
        check(toa_adam_forward_all_multi(l.code, l.num, l.ptr[0].data(), l.ptr[1].data(),
                                         l.ptr[2].data(), l.n.data(), b1, b2, eps, eps_root,
                                         c.data(), c.all, l.ptr[3].data(), l.ptr[4].data(),
                                         l.ptr[5].data(), dev.stream()),
              name);
    }
    return {std::move(new_mu), std::move(new_nu), std::move(new_updates)};
}

std::tuple<TensorList, TensorList, TensorList> forwardAllMulti(
    const TensorList &updates_in, const TensorList &mu, const TensorList &nu_in, double b1,
    double b2, double eps, double eps_root, const py::object &counts) {
    return forwardAllMultiImpl(updates_in, mu, nu_in, b1, b2, eps, eps_root,
                               parseCounts(counts, mu.size()));
}

// dnew_mu / dnew_nu: a list of outside gradients, or None when there are none at all (a list
// may not mix tensors and None: the caller substitutes -0.0 for the missing members).
std::tuple<TensorList, TensorList, TensorList> backwardAllMultiImpl(
    const TensorList &dnew_updates_in, const c10::optional<TensorList> &dnew_mu_in,
    const c10::optional<TensorList> &dnew_nu_in, const TensorList &new_updates_in,
    const TensorList &new_mu, const TensorList &updates_in, double b1, double b2,
    double eps_root, const Counts &c) {
    const char *name = "adamBackwardAllMulti";
    std::vector<TensorList> fresh = emptyLikeSets(new_mu, 3);
    TensorList &dupdates = fresh[0], &dmu = fresh[1], &dnu = fresh[2];
    const TensorList du = asLayoutOfEach(dnew_updates_in, new_mu, name);
    const TensorList new_updates = asLayoutOfEach(new_updates_in, new_mu, name);
    const TensorList updates = asLayoutOfEach(updates_in, new_mu, name);
    Lists l = gateLists(name, {&du, &new_updates, &new_mu, &updates, &dupdates, &dmu, &dnu});
    // outside gradients, brought to new_mu's layout; the (possibly copied) tensors live until
    // the launch below has been enqueued
    TensorList ext_m, ext_v;
    std::vector<void *> pm, pv;
    auto collect = [&](const c10::optional<TensorList> &in, TensorList *ext,
                       std::vector<void *> *ptrs) {
        if (!in.has_value()) return;
        *ext = asLayoutOfEach(in.value(), new_mu, name);
        Lists e = gateLists(name, {&new_mu, ext});
        *ptrs = e.num ? e.ptr[1] : std::vector<void *>();
    };
    collect(dnew_mu_in, &ext_m, &pm);
    collect(dnew_nu_in, &ext_v, &pv);
    if (l.num) {
        TORCH_CHECK(c.each.empty() || c.each.size() == l.num, name, ": expected ", l.num,
                    " counts, got ", c.each.size());
        const OnDeviceOf dev(deviceDonor(new_mu));
        check(toa_adam_backward_all_multi(
                  l.code, l.num, l.ptr[0].data(), l.ptr[1].data(), l.ptr[2].data(),
                  l.ptr[3].data(), dnew_mu_in.has_value() ? pm.data() : nullptr,
                  dnew_nu_in.has_value() ? pv.data() : nullptr, l.n.data(), b1, b2, eps_root,
                  c.data(), c.all, l.ptr[4].data(), l.ptr[5].data(), l.ptr[6].data(),
                  dev.stream()),
              name);
    }
    return {std::move(dupdates), std::move(dmu), std::move(dnu)};
}

std::tuple<TensorList, TensorList, TensorList> backwardAllMulti(
    const TensorList &dnew_updates_in, const c10::optional<TensorList> &dnew_mu_in,
    const c10::optional<TensorList> &dnew_nu_in, const TensorList &new_updates_in,
    const TensorList &new_mu, const TensorList &updates_in, double b1, double b2,
    double eps_root, const py::object &counts) {
    return backwardAllMultiImpl(dnew_updates_in, dnew_mu_in, dnew_nu_in, new_updates_in, new_mu,
                                updates_in, b1, b2, eps_root, parseCounts(counts, new_mu.size()));
}

// ---- the differentiable step of a whole tree as ONE autograd node ----------------------------
//
// (updates, mu, nu) -> (new_mu, new_nu, new_updates) for every leaf: forward_all_multi forward,
// backward_all_multi backward, one pass each.  Per leaf the values and gradients are those of the
// reference's three Functions (/root/reference/torchopt/accelerated_op/adam_op.py:36-121):
//   * saved for backward: new_updates, new_mu, updates (:44, :70, :104 between them);
//   * a gradient for new_updates runs backward_updates, whose results join the gradients that
//     reach new_mu / new_nu from outside (autograd's sums), then backward_mu and backward_nu, and
//     the two contributions to d(updates) are added -- all inside backward_all, rounding for
//     rounding;
//   * a leaf whose new_updates received NO gradient never runs backward_updates in the per-leaf
//     chain, so nothing of new_updates / new_mu (which may hold infinities) may enter: only the
//     outside gradients flow on, through backward_mu / backward_nu, and a leaf with neither gets
//     no gradient at all (undefined, not zeros: materialize_grads is off);
//   * the hyper-parameters and the step numbers get no gradient.
// Living in C++ it costs the host no Python between autograd's engine and the launch: the
// same node written in Python spends 0.2 ms per step on a ten-leaf tree (list slicing, per-leaf
// pybind conversions), twenty times what its two launches take on the device.
//
// The node derives from torch::autograd::Node itself, as PyTorch's own derivative nodes do,
// not from torch::autograd::Function: that wrapper's per-call work (an input record and an
// output record per tensor, sets of dirty and non-differentiable tensors, conversions of the
// argument pack and of the result) costs more host time on thirty inputs and thirty outputs
// than the node's own forward.  What Function would have provided is done here by hand: the
// edges to the inputs' gradient functions, the outputs' history, saved variables (so version
// checks and saved-tensor hooks behave as for any node), the lock around apply and the release
// of the saved tensors after a backward without retain_graph.  Compiled autograd does not know
// the node (no compiled_args); torch.compile traces the Python twin instead.
struct AdamStepBackward : public torch::autograd::Node {
    using variable_list = torch::autograd::variable_list;

    size_t k = 0;
    // new_updates, new_mu (outputs of this node) and updates (an input), k of each
    std::vector<torch::autograd::SavedVariable> saved;
    bool released = false;
    double b1 = 0, b2 = 0, eps_root = 0;
    std::vector<int64_t> counts;

    std::string name() const override { return "AdamStepBackward"; }

    void release_variables() override {
        std::lock_guard<std::mutex> lock(mutex_);
        saved.clear();
        released = true;
    }

    static Counts countsOf(const std::vector<int64_t> &values, size_t num) {
        Counts c;
        if (values.size() == 1) {
            c.all = (uint64_t)values[0];
        } else {
            TORCH_CHECK(values.size() == num, "adamStep: expected ", num, " counts, got ",
                        values.size());
            c.each.assign(values.begin(), values.end());
        }
        return c;
    }

    // grads: for new_mu, new_nu, new_updates of every leaf (undefined where none arrived: the
    // engine does not materialize zeros for a plain Node).  Returns d(updates), d(mu), d(nu).
    variable_list apply(variable_list &&grads) override {
        std::lock_guard<std::mutex> lock(mutex_);
        TORCH_CHECK(!released, torch::autograd::ERR_BACKWARD_TWICE);
        TORCH_CHECK(grads.size() == 3 * k, "adamStep: expected ", 3 * k, " gradients, got ",
                    grads.size());
        const std::shared_ptr<Node> self = shared_from_this();
        TensorList new_updates, new_mu, updates;
        new_updates.reserve(k);
        new_mu.reserve(k);
        updates.reserve(k);
        for (size_t i = 0; i < k; ++i) new_updates.push_back(saved[i].unpack(self));
        for (size_t i = 0; i < k; ++i) new_mu.push_back(saved[k + i].unpack(self));
        for (size_t i = 0; i < k; ++i) updates.push_back(saved[2 * k + i].unpack());
        const Tensor *g_mu = grads.data(), *g_nu = grads.data() + k, *g_u = grads.data() + 2 * k;

        variable_list result(3 * k);
        Tensor *dupdates = result.data(), *dmu = result.data() + k, *dnu = result.data() + 2 * k;

        std::vector<size_t> live, via_mu, via_nu;
        for (size_t i = 0; i < k; ++i) {
            if (g_u[i].defined()) {
                live.push_back(i);
            } else {
                if (g_mu[i].defined()) via_mu.push_back(i);
                if (g_nu[i].defined()) via_nu.push_back(i);
            }
        }
        auto pick = [this](const Tensor *from, const std::vector<size_t> &idx) {
            TensorList out;
            out.reserve(idx.size());
            for (size_t i : idx) out.push_back(from[i]);
            return out;
        };
        auto pick_list = [this, &pick](const TensorList &from, const std::vector<size_t> &idx) {
            return idx.size() == k ? from : pick(from.data(), idx);
        };
        auto counts_of = [&](const std::vector<size_t> &idx) {
            if (counts.size() <= 1 || idx.size() == k) return countsOf(counts, k);
            std::vector<int64_t> some;
            some.reserve(idx.size());
            for (size_t i : idx) some.push_back(counts[i]);
            return countsOf(some, idx.size());
        };
        if (!live.empty()) {
            // Gradients reaching new_mu / new_nu from outside the step.  None at all: the kernel
            // skips the addition, as autograd would.  Some: members without one get -0.0, the
            // exact identity of IEEE addition (x + -0.0 is x for every x, signed zeros
            // included), so they too come out as if nothing had been added.
            auto outside = [&](const Tensor *gs) -> c10::optional<TensorList> {
                bool any = false;
                for (size_t i : live) any = any || gs[i].defined();
                if (!any) return c10::nullopt;
                TensorList out;
                out.reserve(live.size());
                for (size_t i : live)
                    out.push_back(gs[i].defined() ? gs[i] : at::full_like(new_mu[i], -0.0));
                return out;
            };
            auto [du, dm, dn] = backwardAllMultiImpl(
                pick(g_u, live), outside(g_mu), outside(g_nu), pick_list(new_updates, live),
                pick_list(new_mu, live), pick_list(updates, live), b1, b2, eps_root,
                counts_of(live));
            for (size_t j = 0; j < live.size(); ++j) {
                dupdates[live[j]] = std::move(du[j]);
                dmu[live[j]] = std::move(dm[j]);
                dnu[live[j]] = std::move(dn[j]);
            }
        }
        if (!via_mu.empty()) {
            const TensorList donors = pick_list(updates, via_mu);
            auto [du, dm] = backwardMuMulti(pick(g_mu, via_mu), donors, donors, b1);
            for (size_t j = 0; j < via_mu.size(); ++j) {
                dupdates[via_mu[j]] = std::move(du[j]);
                dmu[via_mu[j]] = std::move(dm[j]);
            }
        }
        if (!via_nu.empty()) {
            const TensorList donors = pick_list(updates, via_nu);
            auto [du, dn] = backwardNuMulti(pick(g_nu, via_nu), donors, donors, b2);
            for (size_t j = 0; j < via_nu.size(); ++j) {
                const size_t i = via_nu[j];
                // autograd adds the two contributions to d(updates) where both exist
                dupdates[i] = dupdates[i].defined() ? dupdates[i] + du[j] : std::move(du[j]);
                dnu[i] = std::move(dn[j]);
            }
        }
        // Gradients nobody asked for (torch.autograd.grad with `inputs`, leaves that do not
        // require grad) are dropped here rather than checked and routed by the engine.
        for (size_t i = 0; i < 3 * k; ++i)
            if (result[i].defined() && !task_should_compute_output(i)) result[i] = Tensor();
        return result;
    }
};

// The forward of the node: new_mu, new_nu, new_updates of every leaf, in that order, with their
// history set when any input requires a gradient (and gradients are being recorded).
torch::autograd::variable_list adamStep(const TensorList &updates, const TensorList &mu,
                                        const TensorList &nu, double b1, double b2, double eps,
                                        double eps_root, std::vector<int64_t> counts) {
    const auto &functorch_tls = at::functorch::functorchTLSAccessor();
    // functorch transforms wrap custom nodes in Python; this one they would see through
    if (functorch_tls) functorch_tls->checkSupportsCppAutogradFunction();
    const size_t k = mu.size();
    std::shared_ptr<AdamStepBackward> node;
    if (torch::autograd::compute_requires_grad(updates, mu, nu)) {
        node = std::shared_ptr<AdamStepBackward>(new AdamStepBackward(),
                                                 torch::autograd::deleteNode);
        node->set_next_edges(torch::autograd::collect_next_edges(updates, mu, nu));
    }
    std::tuple<TensorList, TensorList, TensorList> fresh;
    {
        // layout conversions of the inputs in there must not be recorded: the gradients this
        // node returns are for the inputs as they came
        at::AutoGradMode no_grad(false);
        fresh = forwardAllMultiImpl(updates, mu, nu, b1, b2, eps, eps_root,
                                    AdamStepBackward::countsOf(counts, k));
    }
    auto &[new_mu, new_nu, new_updates] = fresh;
    torch::autograd::variable_list out;
    out.reserve(3 * k);
    for (TensorList *l : {&new_mu, &new_nu, &new_updates})
        for (Tensor &t : *l) out.push_back(std::move(t));
    if (node) {
        for (const Tensor &t : out) torch::autograd::set_history(t, node);
        node->k = k;
        node->b1 = b1;
        node->b2 = b2;
        node->eps_root = eps_root;
        node->counts = std::move(counts);
        node->saved.reserve(3 * k);
        for (size_t i = 0; i < k; ++i) node->saved.emplace_back(out[2 * k + i], /*is_output=*/true);
        for (size_t i = 0; i < k; ++i) node->saved.emplace_back(out[i], /*is_output=*/true);
        for (size_t i = 0; i < k; ++i) node->saved.emplace_back(updates[i], /*is_output=*/false);
    }
    return out;
}

// (new_mu, new_nu, new_updates) as lists, differentiable with respect to every tensor of the
// three input lists.  `counts` as for the other list functions.
py::tuple stepMulti(const py::object &updates_o, const py::object &mu_o, const py::object &nu_o,
                    double b1, double b2, double eps, double eps_root, const py::object &counts) {
    const TensorList updates = toTensorList(updates_o, "updates");
    const TensorList mu = toTensorList(mu_o, "mu");
    const TensorList nu = toTensorList(nu_o, "nu");
    const size_t k = mu.size();
    TORCH_CHECK(updates.size() == k && nu.size() == k, "adamStep: tensor lists differ in length");
    const Counts c = parseCounts(counts, k);
    std::vector<int64_t> values;
    if (c.each.empty())
        values.push_back((int64_t)c.all);
    else
        values.assign(c.each.begin(), c.each.end());
    for (int64_t v : values)
        if (v < 0) throw py::type_error("counts beyond INT64_MAX are not served here");
    const auto out = adamStep(updates, mu, nu, b1, b2, eps, eps_root, std::move(values));
    py::list lists[3];
    for (int j = 0; j < 3; ++j)
        for (size_t i = 0; i < k; ++i) lists[j].append(py::cast(out[j * k + i]));
    return py::make_tuple(lists[0], lists[1], lists[2]);
}

py::tuple fusedStepMulti(const py::object &params_o, const py::object &updates_o,
                         const py::object &mu_o, const py::object &nu_o, double b1, double b2,
                         double eps, double eps_root, const py::object &counts, double lr,
                         bool maximize, bool write_updates, double weight_decay,
                         bool decoupled) {
    const char *name = "adamFusedStepMulti";
    const auto params = toTensorList(params_o, "params");
    auto updates = toTensorList(updates_o, "updates");
    const auto mu = toTensorList(mu_o, "mu");
    const auto nu = toTensorList(nu_o, "nu");
    // gradients that are only read may come in any layout (channels-last, expanded, sliced)
    if (!write_updates) updates = asLayoutOfEach(updates, params, name);
    Lists l = gateLists(name, {&params, &mu, &nu, &updates});
    if (l.num) {
        const Counts c = parseCounts(counts, l.num);
        const OnDeviceOf dev(deviceDonor(params));
        check(toa_adam_fused_step_multi(l.code, l.num, l.ptr[0].data(), l.ptr[3].data(),
                                        l.ptr[1].data(), l.ptr[2].data(), l.n.data(), b1, b2, eps,
                                        eps_root, c.data(), c.all, lr, weight_decay,
                                        (int)decoupled, (int)maximize, (int)write_updates,
                                        dev.stream()),
              name);
    }
    return py::make_tuple(params_o, updates_o, mu_o, nu_o);
}

// ---- step number on the device ------------------------------------------------------------

// `rows` x 4 tensor on the CPU of element type `dtype`: the bias corrections of step numbers
// first_count, first_count + 1, ... as the launchers round them.
Tensor biasRows(const py::object &dtype_o, double b1, double b2, double eps_root,
                uint64_t first_count, size_t rows) {
    const at::ScalarType st = torch::python::detail::py_object_to_dtype(dtype_o);
    Tensor out = at::empty({(int64_t)rows, 4}, at::TensorOptions().dtype(st).device(at::kCPU));
    check(toa_adam_bias_rows(dtypeCode(out, "adamBiasRows"), b1, b2, eps_root, first_count, rows,
                             out.data_ptr()),
          "adamBiasRows");
    return out;
}

size_t biasRowsNeeded(double b1, double b2, uint64_t first_count, size_t limit) {
    return toa_adam_bias_rows_needed(b1, b2, first_count, limit);
}

// What the device-count entry points need beside the tensors: the table and the step number, on
// the tensors' device.
struct DeviceStep {
    const void *rows;
    size_t num_rows;
    const int64_t *count;
};
DeviceStep gateStep(const char *name, const Tensor &lead, const Tensor &bias_rows,
                    const Tensor &count) {
    TORCH_CHECK(bias_rows.device() == lead.device() && count.device() == lead.device(), name,
                ": bias_rows and count must live on ", lead.device());
    TORCH_CHECK(bias_rows.scalar_type() == lead.scalar_type(), name,
                ": bias_rows must have the tensors' scalar type ", lead.scalar_type());
    TORCH_CHECK(bias_rows.dim() == 2 && bias_rows.size(1) == 4 && bias_rows.size(0) >= 1 &&
                    bias_rows.is_contiguous(),
                name, ": bias_rows must be a contiguous (rows, 4) tensor");
    TORCH_CHECK(count.scalar_type() == at::kLong && count.numel() == 1, name,
                ": count must be a one-element int64 tensor");
    return {bias_rows.data_ptr(), (size_t)bias_rows.size(0), count.data_ptr<int64_t>()};
}

Tensor countAdvance(const Tensor &count) {
    if (!count.is_cuda()) throw std::runtime_error("Not implemented");
    TORCH_CHECK(count.scalar_type() == at::kLong && count.numel() == 1,
                "adamCountAdvance: count must be a one-element int64 tensor");
    const OnDeviceOf dev(count);
    check(toa_adam_count_advance(count.data_ptr<int64_t>(), dev.stream()), "adamCountAdvance");
    return count;
}

std::array<Tensor, 3> forwardInplaceDevCount(const Tensor &updates, const Tensor &mu,
                                             const Tensor &nu, double b1, double b2, double eps,
                                             double eps_root, const Tensor &bias_rows,
                                             uint64_t first_count, const Tensor &count) {
    const char *name = "adamForwardInplaceDevCount";
    size_t n;
    const int code = gate(name, updates, {&mu, &nu}, &n);
    const DeviceStep step = gateStep(name, updates, bias_rows, count);
    if (n) {
        requireDense(name, "updates", updates);
        requireDense(name, "mu", mu);
        requireDense(name, "nu", nu);
        TORCH_CHECK(sameLayout(updates, mu) && sameLayout(updates, nu), name,
                    ": updates, mu and nu must share one memory layout");
        const OnDeviceOf dev(updates);
        check(toa_adam_forward_inplace_devcount(code, updates.data_ptr(), mu.data_ptr(),
                                                nu.data_ptr(), n, b1, b2, eps, eps_root, step.rows,
                                                first_count, step.num_rows, step.count,
                                                dev.stream()),
              name);
    }
    return {updates, mu, nu};
}

py::tuple forwardMultiInplaceDevCount(const py::object &updates_o, const py::object &mu_o,
                                      const py::object &nu_o, double b1, double b2, double eps,
                                      double eps_root, const Tensor &bias_rows,
                                      uint64_t first_count, const Tensor &count) {
    const char *name = "adamForwardInplaceMultiDevCount";
    const auto updates = toTensorList(updates_o, "updates");
    const auto mu = toTensorList(mu_o, "mu");
    const auto nu = toTensorList(nu_o, "nu");
    Lists l = gateLists(name, {&updates, &mu, &nu});
    if (l.num) {
        const DeviceStep step = gateStep(name, deviceDonor(updates), bias_rows, count);
        const OnDeviceOf dev(deviceDonor(updates));
        check(toa_adam_forward_inplace_multi_devcount(
                  l.code, l.num, l.ptr[0].data(), l.ptr[1].data(), l.ptr[2].data(), l.n.data(), b1,
                  b2, eps, eps_root, step.rows, first_count, step.num_rows, step.count,
                  dev.stream()),
              name);
    }
    return py::make_tuple(updates_o, mu_o, nu_o);
}

py::tuple fusedStepMultiDevCount(const py::object &params_o, const py::object &updates_o,
                                 const py::object &mu_o, const py::object &nu_o, double b1,
                                 double b2, double eps, double eps_root, const Tensor &bias_rows,
                                 uint64_t first_count, const Tensor &count, double lr,
                                 bool maximize, bool write_updates, double weight_decay,
                                 bool decoupled) {
    const char *name = "adamFusedStepMultiDevCount";
    const auto params = toTensorList(params_o, "params");
    auto updates = toTensorList(updates_o, "updates");
    const auto mu = toTensorList(mu_o, "mu");
    const auto nu = toTensorList(nu_o, "nu");
    if (!write_updates) updates = asLayoutOfEach(updates, params, name);
    Lists l = gateLists(name, {&params, &mu, &nu, &updates});
    if (l.num) {
        const DeviceStep step = gateStep(name, deviceDonor(params), bias_rows, count);
        const OnDeviceOf dev(deviceDonor(params));
        check(toa_adam_fused_step_multi_devcount(
                  l.code, l.num, l.ptr[0].data(), l.ptr[3].data(), l.ptr[1].data(),
                  l.ptr[2].data(), l.n.data(), b1, b2, eps, eps_root, step.rows, first_count,
                  step.num_rows, step.count, lr, weight_decay, (int)decoupled, (int)maximize,
                  (int)write_updates, dev.stream()),
              name);
    }
    return py::make_tuple(params_o, updates_o, mu_o, nu_o);
}

}  // namespace

PYBIND11_MODULE(_C, mod) {
    mod.doc() = "MI355X-native counterpart of torchopt._C";
    py::module m = mod.def_submodule("adam_op", "Adam Ops");
    using namespace py::literals;

    // the reference's seven (names and keywords as in adam_op.cpp:157-214)
    m.def("forward_", &forwardInplace, "Adam forward inplace", "updates"_a, "mu"_a, "nu"_a, "b1"_a,
          "b2"_a, "eps"_a, "eps_root"_a, "count"_a);
    m.def("forward_mu", &forwardMu, "Adam forward mu", "updates"_a, "mu"_a, "b1"_a);
    m.def("forward_nu", &forwardNu, "Adam forward nu", "updates"_a, "nu"_a, "b2"_a);
    m.def("forward_updates", &forwardUpdates, "Adam forward updates", "new_mu"_a, "new_nu"_a,
          "b1"_a, "b2"_a, "eps"_a, "eps_root"_a, "count"_a);
    m.def("backward_mu", &backwardMu, "Adam backward mu", "dmu"_a, "updates"_a, "mu"_a, "b1"_a);
    m.def("backward_nu", &backwardNu, "Adam backward nu", "dnu"_a, "updates"_a, "nu"_a,
          "b1"_a);  // the decay is b2; the reference registers the keyword as b1
    m.def("backward_updates", &backwardUpdates, "Adam backward updates", "dupdates"_a, "updates"_a,
          "new_mu"_a, "new_nu"_a, "b1"_a, "b2"_a, "eps_root"_a, "count"_a);

    // lists of tensors: one launch per hundred-odd tensors
    m.def("forward_multi_", &forwardMultiInplace,
          "forward_ over lists; mutates and returns (updates, mu, nu)", "updates"_a, "mu"_a,
          "nu"_a, "b1"_a, "b2"_a, "eps"_a, "eps_root"_a, "counts"_a);
    m.def("forward_mu_multi", &forwardMuMulti, "forward_mu over lists", "updates"_a, "mu"_a,
          "b1"_a);
    m.def("forward_nu_multi", &forwardNuMulti, "forward_nu over lists", "updates"_a, "nu"_a,
          "b2"_a);
    m.def("forward_updates_multi", &forwardUpdatesMulti, "forward_updates over lists", "new_mu"_a,
          "new_nu"_a, "b1"_a, "b2"_a, "eps"_a, "eps_root"_a, "counts"_a);
    m.def("backward_mu_multi", &backwardMuMulti, "backward_mu over lists -> (dupdates, dmu)",
          "dmu"_a, "updates"_a, "mu"_a, "b1"_a);
    m.def("backward_nu_multi", &backwardNuMulti, "backward_nu over lists -> (dupdates, dnu)",
          "dnu"_a, "updates"_a, "nu"_a, "b2"_a);
    m.def("backward_updates_multi", &backwardUpdatesMulti,
          "backward_updates over lists -> (dnew_mu, dnew_nu)", "dupdates"_a, "updates"_a,
          "new_mu"_a, "new_nu"_a, "b1"_a, "b2"_a, "eps_root"_a, "counts"_a);

    // the differentiable step, one pass per direction
    m.def("forward_all", &forwardAll,
          "forward_mu, forward_nu and forward_updates in one pass -> [new_mu, new_nu, new_updates]",
          "updates"_a, "mu"_a, "nu"_a, "b1"_a, "b2"_a, "eps"_a, "eps_root"_a, "count"_a);
    m.def("backward_all", &backwardAll,
          "backward of forward_all in one pass -> [dupdates, dmu, dnu]", "dnew_updates"_a,
          "dnew_mu"_a, "dnew_nu"_a, "new_updates"_a, "new_mu"_a, "updates"_a, "b1"_a, "b2"_a,
          "eps_root"_a, "count"_a);
    m.def("forward_all_multi", &forwardAllMulti, "forward_all over lists", "updates"_a, "mu"_a,
          "nu"_a, "b1"_a, "b2"_a, "eps"_a, "eps_root"_a, "counts"_a);
    m.def("backward_all_multi", &backwardAllMulti, "backward_all over lists", "dnew_updates"_a,
          "dnew_mu"_a, "dnew_nu"_a, "new_updates"_a, "new_mu"_a, "updates"_a, "b1"_a, "b2"_a,
          "eps_root"_a, "counts"_a);

    m.def("one_kind", &oneKind,
          "whether a list or tuple holds only tensors, all of one device and one dtype",
          "tensors"_a);

    m.def("step_multi", &stepMulti,
          "the differentiable step of a whole list as one autograd node -> "
          "(new_mu, new_nu, new_updates)",
          "updates"_a, "mu"_a, "nu"_a, "b1"_a, "b2"_a, "eps"_a, "eps_root"_a, "counts"_a);

    // the classic in-place optimizer step in one pass
    m.def("fused_step_", &fusedStep,
          "Adam + scale(-lr) + apply in one pass; returns [params, updates, mu, nu]", "params"_a,
          "updates"_a, "mu"_a, "nu"_a, "b1"_a, "b2"_a, "eps"_a, "eps_root"_a, "count"_a, "lr"_a,
          py::kw_only(), "maximize"_a = false, "write_updates"_a = false,
          "weight_decay"_a = 0.0, "decoupled"_a = false);
    m.def("fused_step_multi_", &fusedStepMulti, "fused_step_ over lists", "params"_a, "updates"_a,
          "mu"_a, "nu"_a, "b1"_a, "b2"_a, "eps"_a, "eps_root"_a, "counts"_a, "lr"_a,
          py::kw_only(), "maximize"_a = false, "write_updates"_a = false,
          "weight_decay"_a = 0.0, "decoupled"_a = false);

    // the step number on the device: one captured graph serves a whole training loop
    m.def("bias_rows", &biasRows,
          "(rows, 4) CPU tensor of bias corrections for steps first_count, first_count + 1, ...",
          "dtype"_a, "b1"_a, "b2"_a, "eps_root"_a, "first_count"_a, "rows"_a);
    m.def("bias_rows_needed", &biasRowsNeeded,
          "rows from first_count on that make a table exact for every later step (0: > limit)",
          "b1"_a, "b2"_a, "first_count"_a, "limit"_a);
    m.def("count_advance_", &countAdvance, "count += (count != INT64_MAX), on the device",
          "count"_a);
    m.def("forward_devcount_", &forwardInplaceDevCount,
          "forward_ with the step number read on the device", "updates"_a, "mu"_a, "nu"_a, "b1"_a,
          "b2"_a, "eps"_a, "eps_root"_a, "bias_rows"_a, "first_count"_a, "count"_a);
    m.def("forward_multi_devcount_", &forwardMultiInplaceDevCount,
          "forward_multi_ with the step number read on the device", "updates"_a, "mu"_a, "nu"_a,
          "b1"_a, "b2"_a, "eps"_a, "eps_root"_a, "bias_rows"_a, "first_count"_a, "count"_a);
    m.def("fused_step_multi_devcount_", &fusedStepMultiDevCount,
          "fused_step_multi_ with the step number read on the device", "params"_a, "updates"_a,
          "mu"_a, "nu"_a, "b1"_a, "b2"_a, "eps"_a, "eps_root"_a, "bias_rows"_a, "first_count"_a,
          "count"_a, "lr"_a, py::kw_only(), "maximize"_a = false, "write_updates"_a = false,
          "weight_decay"_a = 0.0, "decoupled"_a = false);
}
