// Host-side helper of the cached-plan optimizer step (heavyball_amd/optim.py, FirstOrder._fast_step): the per-parameter part of a
// step - read every gradient, check that it can go to the kernel as it is, note its address, drop it - as one C++ loop over the
// tensors instead of five Python calls per tensor.  No device work happens here and nothing is computed: the kernels stay
// behind the C ABI of libhbstep.so; this module only looks at tensor metadata through torch's C++ API.
//
// The checks are those of the Python loop it replaces (same order of precedence):
//   every parameter has a gradient; the gradient is a dense, contiguous tensor of the expected dtype whose address is a multiple
//   of 16; the parameter's own data still sits where the slab put it.
#include <torch/extension.h>

#include <cstdint>

namespace {

// Reasons a step cannot be replayed from its plan; 0 means every tensor passed.
enum : int { kOk = 0, kNoGrad = 1, kDtype = 2, kLayout = 3, kAlign = 4, kMoved = 5, kArgs = 6 };

// params: list of tensors (the bucket's parameters in slab order); home: int64 CPU tensor with the address each parameter's data
// must have; out: int64 CPU tensor that receives the gradients' addresses; dtype: the gradients' expected dtype.
int collect(const py::list& params, const at::Tensor& home, at::Tensor& out, const py::object& dtype) {
  const int64_t n = (int64_t)params.size();
  if (home.numel() != n || out.numel() != n || home.scalar_type() != at::kLong || out.scalar_type() != at::kLong || !home.is_contiguous() ||
      !out.is_contiguous() || home.is_cuda() || out.is_cuda())
    return kArgs;
  const at::ScalarType want = torch::python::detail::py_object_to_dtype(dtype);
  const int64_t* h = home.data_ptr<int64_t>();
  int64_t* o = out.data_ptr<int64_t>();
  for (int64_t i = 0; i < n; ++i) {
    PyObject* obj = PyList_GET_ITEM(params.ptr(), i);
    if (!THPVariable_Check(obj)) return kArgs;
    const at::Tensor& p = THPVariable_Unpack(obj);
    const at::Tensor& g = p.grad();
    if (!g.defined()) return kNoGrad;
    if (g.scalar_type() != want) return kDtype;
    if (g.layout() != at::kStrided || !g.is_contiguous()) return kLayout;
    const auto addr = reinterpret_cast<uintptr_t>(g.data_ptr());
    if (addr & 15u) return kAlign;
    if (reinterpret_cast<int64_t>(p.data_ptr()) != h[i]) return kMoved;
    o[i] = (int64_t)addr;
  }
  return kOk;
}

// p.grad = None for every parameter of the list
void drop_grads(const py::list& params) {
  const int64_t n = (int64_t)params.size();
  for (int64_t i = 0; i < n; ++i) {
    PyObject* obj = PyList_GET_ITEM(params.ptr(), i);
    if (!THPVariable_Check(obj)) continue;
    const at::Tensor& p = THPVariable_Unpack(obj);
    if (p.grad().defined()) p.mutable_grad() = at::Tensor();
  }
}

}  // namespace

PYBIND11_MODULE(_hostloop, m) {
  m.doc() = "per-parameter host loop of the cached-plan optimizer step";
  m.def("collect", &collect, "check the gradients of a bucket and write their addresses; returns 0 or the reason the plan does not fit");
  m.def("drop_grads", &drop_grads, "set the gradient of every parameter of the list to None");
  m.attr("OK") = (int)kOk;
}
