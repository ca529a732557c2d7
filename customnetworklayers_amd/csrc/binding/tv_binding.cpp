// Compiled PyTorch binding of the TV inpainting layer over the C ABI in include/tvinpaint.h: the functions of the
// reference's pybind module tvInpaint_cuda_ext (cudaTV/TVInpaintFista_cuda.cpp:47-150 of the reference) with the two
// static calls (lines 75-78 and 129-134 there) replaced by tvinpaint_forward / tvinpaint_backward.  No kernels here:
// this file is host C++ and links libinpaint_hip.so.  Differences from the reference binding, all at its edges:
// batches n >= 1 are accepted (TVInpaintFista_cuda.cpp:61-65 refuses them), failures throw instead of printing and
// returning an empty list (80-87), outputs are allocated uninitialised (the callee overwrites them), and the work is
// enqueued on PyTorch's current stream.
#include <torch/extension.h>

// PyTorch on ROCm presents its HIP devices under the device type "cuda"; these are the guard and stream of that view
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPCachingAllocator.h>

#include <string>
#include <vector>

#include "tvinpaint.h"

namespace {

void check_input(const at::Tensor& x, const char* name) {  // CHECK_INPUT, TVInpaintFista_cuda.cpp:24-26, and the type test of 68
  TORCH_CHECK(x.is_cuda(), name, " must be a CUDA tensor");
  TORCH_CHECK(x.is_contiguous(), name, " must be contiguous");
  TORCH_CHECK(x.scalar_type() == at::kFloat, "Input/Output type to the operator must be single/float (", name, ")");
}

void check_shapes(const at::Tensor& d_x, const at::Tensor& d_y, const at::Tensor& d_c, const at::Tensor& d_b,
                  const at::Tensor& other, const char* other_name) {
  TORCH_CHECK(d_b.dim() == 4, "d_b must be (n, c, h, w)");
  const auto n = d_b.size(0), h = d_b.size(2), w = d_b.size(3);
  for (const at::Tensor* t : {&d_x, &d_y, &d_c})
    TORCH_CHECK(t->dim() == 4 && t->size(0) == n && t->size(1) == 1 && t->size(2) == h && t->size(3) == w,
                "d_x, d_y, d_c must have shape (n, 1, h, w) of d_b");
  TORCH_CHECK(other.sizes() == d_b.sizes(), other_name, " must have the shape of d_b");
  for (const at::Tensor* t : {&d_x, &d_y, &d_c, &other})
    TORCH_CHECK(t->device() == d_b.device(), "all tensors must live on one device");
}

void* current_stream(const at::Tensor& t) { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream(); }

// The per-id device blocks out of PyTorch's caching allocator (tvinpaint_set_allocator): the reference callocs and frees
// its checkpoints on the host in every forward; here one block per id and shape lives in the pool PyTorch can see.
void* torch_alloc(unsigned long long bytes, int /*device: the current one*/, void* stream, void* /*user*/) {
  try {
    return c10::hip::HIPCachingAllocator::raw_alloc_with_stream((size_t)bytes, (hipStream_t)stream);
  } catch (const std::exception&) {  // out of memory: the library falls back to fewer kept rows or reports the failure
    return nullptr;
  }
}
void torch_release(void* ptr, void* /*user*/) { c10::hip::HIPCachingAllocator::raw_delete(ptr); }

}  // namespace

std::vector<at::Tensor> tvInpaint_dummy() {
  std::cout << "Input: not present just dummy:\n";
  return {};
}

void tvInpaint_dummy_only() { std::cout << "Dummy call:\n"; }

std::vector<at::Tensor> tvInpaint_forward(at::Tensor d_x, at::Tensor d_y, at::Tensor d_c, at::Tensor d_b, at::Tensor d_i,
                                          int its, int id) {
  check_input(d_x, "d_x"); check_input(d_y, "d_y"); check_input(d_c, "d_c"); check_input(d_b, "d_b"); check_input(d_i, "d_i");
  check_shapes(d_x, d_y, d_c, d_b, d_i, "d_i");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(d_b.device());
  at::Tensor solution = at::empty_like(d_b);
  const int rc = tvinpaint_forward(d_x.data_ptr<float>(), d_y.data_ptr<float>(), d_c.data_ptr<float>(), d_b.data_ptr<float>(),
                                   d_i.data_ptr<float>(), solution.data_ptr<float>(), (int)d_b.size(0), (int)d_b.size(1),
                                   (int)d_b.size(2), (int)d_b.size(3), its, id, current_stream(d_b));
  TORCH_CHECK(rc == 0, "TVInpaint::forward failed: ", tvinpaint_last_error());
  return {solution};
}

std::vector<at::Tensor> tvInpaint_backward(at::Tensor d_iGf, at::Tensor d_x, at::Tensor d_y, at::Tensor d_c, at::Tensor d_b,
                                           int its, int id) {
  check_input(d_x, "d_x"); check_input(d_y, "d_y"); check_input(d_c, "d_c"); check_input(d_b, "d_b"); check_input(d_iGf, "d_iGf");
  check_shapes(d_x, d_y, d_c, d_b, d_iGf, "d_iGf");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(d_b.device());
  at::Tensor d_oGx = at::empty_like(d_x), d_oGy = at::empty_like(d_y), d_oGc = at::empty_like(d_c);
  at::Tensor d_oGb = at::empty_like(d_b), d_oGi = at::empty_like(d_b);
  const int rc = tvinpaint_backward(d_x.data_ptr<float>(), d_y.data_ptr<float>(), d_c.data_ptr<float>(), d_b.data_ptr<float>(),
                                    d_iGf.data_ptr<float>(),  // non-finite entries are zeroed in place, as in the reference
                                    d_oGx.data_ptr<float>(), d_oGy.data_ptr<float>(), d_oGc.data_ptr<float>(),
                                    d_oGb.data_ptr<float>(), d_oGi.data_ptr<float>(), (int)d_b.size(0), (int)d_b.size(1),
                                    (int)d_b.size(2), (int)d_b.size(3), its, id, current_stream(d_b));
  TORCH_CHECK(rc == 0, "TVInpaint::backward failed: ", tvinpaint_last_error());
  return {d_oGx, d_oGy, d_oGc, d_oGb, d_oGi};
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  tvinpaint_set_allocator(torch_alloc, torch_release, nullptr);
  m.def("use_torch_allocator", [](bool enable) {
    TORCH_CHECK(tvinpaint_set_allocator(enable ? torch_alloc : nullptr, enable ? torch_release : nullptr, nullptr) == 0, tvinpaint_last_error());
  }, "take the ids' device blocks from PyTorch's caching allocator (default) or from hipMalloc");
  m.def("forward", &tvInpaint_forward, "tvInpaint forward (HIP)");
  m.def("backward", &tvInpaint_backward, "tvInpaint backward (HIP)");
  m.def("dummy", &tvInpaint_dummy, "tvInpaint dummy");
  m.def("dummy_only", &tvInpaint_dummy_only, "tvInpaint dummy2");
  m.def("reset_id", [](int id) { TORCH_CHECK(tvinpaint_reset_id(id) == 0, tvinpaint_last_error()); }, "free the id's state");
}
