// Bodies for the reference's seven device launchers on top of libtoa_adam.so.
//
// This file belongs inside the reference's own C++ extension, in the place of
// /root/reference/src/adam_op/adam_op_impl_cuda.cu: it defines the functions that
// /root/reference/include/adam_op/adam_op_impl_cuda.cuh:26-68 declares and that the dispatcher
// in /root/reference/src/adam_op/adam_op.cpp:32-153 calls for `is_cuda()` tensors when it is
// compiled with __USE_CUDA__ (on PyTorch-ROCm an AMD GPU tensor answers is_cuda() with true).
// The dispatcher, the pybind11 module and everything above them stay as they are.  It is not
// part of this package's own build (it needs the reference's headers on the include path);
// `make -C oracle dropin` compiles the reference's extension with it to show that the boundary
// holds, and tests/test_dropin_gpu.py runs that module.
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include "include/adam_op/adam_op_impl_cuda.cuh"
#include "include/utils.h"
#include "toa_adam.h"

namespace torchopt {
namespace adam_op {
namespace {

int toaDtype(const torch::Tensor &t, const char *name) {
  switch (t.scalar_type()) {
    case at::kFloat: return TOA_F32;
    case at::kDouble: return TOA_F64;
    case at::kHalf: return TOA_F16;
    case at::kBFloat16: return TOA_BF16;
    default: TORCH_CHECK(false, "\"", name, "\" not implemented for '", t.scalar_type(), "'");
  }
}

void toaCheck(int rc, const char *name) {
  TORCH_CHECK(rc == 0, name, ": ", toa_adam_error_string(rc));
}

// Current device -> the tensor's device for the duration of a launch; PyTorch's current
// stream on that device.
class Launch {
 public:
  explicit Launch(const torch::Tensor &t) : index_(static_cast<int>(t.get_device())) {
    if (hipGetDevice(&prev_) != hipSuccess) prev_ = index_;
    if (prev_ != index_) TORCH_CHECK(hipSetDevice(index_) == hipSuccess, "hipSetDevice failed");
  }
  ~Launch() {
    if (prev_ != index_) (void)hipSetDevice(prev_);
  }
  void *stream() const {
    return c10::hip::getCurrentHIPStream(static_cast<c10::DeviceIndex>(index_)).stream();
  }

 private:
  int index_;
  int prev_ = 0;
};

}  // namespace

TensorArray<3> adamForwardInplaceCUDA(const torch::Tensor &updates, const torch::Tensor &mu,
                                      const torch::Tensor &nu, const pyfloat_t b1,
                                      const pyfloat_t b2, const pyfloat_t eps,
                                      const pyfloat_t eps_root, const pyuint_t count) {
  const char *name = "adamForwardInplaceCUDA";
  const Launch on(updates);
  toaCheck(toa_adam_forward_inplace(toaDtype(updates, name), updates.data_ptr(), mu.data_ptr(),
                                    nu.data_ptr(), getTensorPlainSize(updates), b1, b2, eps,
                                    eps_root, count, on.stream()),
           name);
  return TensorArray<3>{updates, mu, nu};
}

torch::Tensor adamForwardMuCUDA(const torch::Tensor &updates, const torch::Tensor &mu,
                                const pyfloat_t b1) {
  const char *name = "adamForwardMuCUDA";
  auto mu_out = torch::empty_like(mu);
  const Launch on(updates);
  toaCheck(toa_adam_forward_mu(toaDtype(updates, name), updates.data_ptr(), mu.data_ptr(),
                               getTensorPlainSize(updates), b1, mu_out.data_ptr(), on.stream()),
           name);
  return mu_out;
}

torch::Tensor adamForwardNuCUDA(const torch::Tensor &updates, const torch::Tensor &nu,
                                const pyfloat_t b2) {
  const char *name = "adamForwardNuCUDA";
  auto nu_out = torch::empty_like(nu);
  const Launch on(updates);
  toaCheck(toa_adam_forward_nu(toaDtype(updates, name), updates.data_ptr(), nu.data_ptr(),
                               getTensorPlainSize(updates), b2, nu_out.data_ptr(), on.stream()),
           name);
  return nu_out;
}

torch::Tensor adamForwardUpdatesCUDA(const torch::Tensor &new_mu, const torch::Tensor &new_nu,
                                     const pyfloat_t b1, const pyfloat_t b2, const pyfloat_t eps,
                                     const pyfloat_t eps_root, const pyuint_t count) {
  const char *name = "adamForwardUpdatesCUDA";
  auto updates_out = torch::empty_like(new_mu);
  const Launch on(new_mu);
  toaCheck(toa_adam_forward_updates(toaDtype(new_mu, name), new_mu.data_ptr(), new_nu.data_ptr(),
                                    getTensorPlainSize(new_mu), b1, b2, eps, eps_root, count,
                                    updates_out.data_ptr(), on.stream()),
           name);
  return updates_out;
}

TensorArray<2> adamBackwardMuCUDA(const torch::Tensor &dmu, const torch::Tensor &updates,
                                  const torch::Tensor &mu, const pyfloat_t b1) {
  const char *name = "adamBackwardMuCUDA";
  auto dupdates_out = torch::empty_like(updates);
  auto dmu_out = torch::empty_like(mu);
  const Launch on(dmu);
  toaCheck(toa_adam_backward_mu(toaDtype(dmu, name), dmu.data_ptr(), getTensorPlainSize(dmu), b1,
                                dupdates_out.data_ptr(), dmu_out.data_ptr(), on.stream()),
           name);
  return TensorArray<2>{std::move(dupdates_out), std::move(dmu_out)};
}

TensorArray<2> adamBackwardNuCUDA(const torch::Tensor &dnu, const torch::Tensor &updates,
                                  const torch::Tensor &nu, const pyfloat_t b2) {
  const char *name = "adamBackwardNuCUDA";
  auto dupdates_out = torch::empty_like(updates);
  auto dnu_out = torch::empty_like(nu);
  const Launch on(dnu);
  toaCheck(toa_adam_backward_nu(toaDtype(dnu, name), dnu.data_ptr(), updates.data_ptr(),
                                getTensorPlainSize(dnu), b2, dupdates_out.data_ptr(),
                                dnu_out.data_ptr(), on.stream()),
           name);
  return TensorArray<2>{std::move(dupdates_out), std::move(dnu_out)};
}

TensorArray<2> adamBackwardUpdatesCUDA(const torch::Tensor &dupdates, const torch::Tensor &updates,
                                       const torch::Tensor &new_mu, const torch::Tensor &new_nu,
                                       const pyfloat_t b1, const pyfloat_t b2,
                                       const pyfloat_t eps_root, const pyuint_t count) {
  const char *name = "adamBackwardUpdatesCUDA";
  auto dmu_out = torch::empty_like(new_mu);
  auto dnu_out = torch::empty_like(new_nu);
  const Launch on(dupdates);
  toaCheck(toa_adam_backward_updates(toaDtype(dupdates, name), dupdates.data_ptr(),
                                     updates.data_ptr(), new_mu.data_ptr(),
                                     getTensorPlainSize(dupdates), b1, b2, eps_root, count,
                                     dmu_out.data_ptr(), dnu_out.data_ptr(), on.stream()),
           name);
  return TensorArray<2>{std::move(dmu_out), std::move(dnu_out)};
}

}  // namespace adam_op
}  // namespace torchopt
