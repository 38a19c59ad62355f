// The torch operators' device implementations in C++: libsphericart_amd_torch.so, loaded with
// torch.ops.load_library. Host code only (no kernel): it defines the schemas of the `sphericart_amd` namespace and
// implements them for tensors on the GPU by calling the C entry points of libsphericart_amd.so on the tensor's
// current stream, as the reference's extension does with its calculators
// (sphericart-torch/src/torch.cpp:237-294 _compute_raw_cuda, :367-385 TORCH_LIBRARY). Autograd, fake-tensor and vmap
// rules stay in Python (sphericart_amd/torch/ops.py), as they do in the reference
// (sphericart-torch/python/sphericart/torch/register.py:60-185). A call through these costs the host the
// dispatcher, the allocation of its outputs and one C call; the same operators implemented in Python over ctypes,
// which ops.py registers when this library has not been built, cost about twice that.
#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <ATen/core/dispatch/Dispatcher.h>

#include <memory>
#include <string>
#include <tuple>

#include "../../include/sphx_launch.h"

namespace {

using at::Tensor;

void check(int status) {
    TORCH_CHECK(status == SPHX_OK, sphx_last_error());
}

bool is_double(const Tensor& tensor, const char* what) {
    TORCH_CHECK_TYPE(tensor.scalar_type() == at::kFloat || tensor.scalar_type() == at::kDouble, what,
                     " are implemented for float32 and float64, not ", tensor.scalar_type());
    return tensor.scalar_type() == at::kDouble;
}

// an empty tensor's pointer may be anything: the library takes null for "no array"
template <typename T> T* pointer(const Tensor& tensor) {
    return tensor.defined() && tensor.numel() > 0 ? tensor.data_ptr<T>() : nullptr;
}

void* stream_of(const Tensor& tensor) {
    return c10::hip::getCurrentHIPStream(tensor.device().index()).stream();
}

// compute_raw / _compute_raw_cuda (sphericart-torch/src/torch.cpp:126-146, 238-294)
std::tuple<Tensor, Tensor, Tensor> forward(const Tensor& xyz_in, int64_t l_max, bool normalized, int mode) {
    TORCH_CHECK_VALUE(xyz_in.dim() == 2 && xyz_in.size(1) == 3,
                      "xyz tensor must be a 2D array with shape `n_samples x 3`");
    TORCH_CHECK_VALUE(l_max >= 0, "l_max must be non-negative");
    const bool f64 = is_double(xyz_in, "spherical harmonics");
    const Tensor xyz = xyz_in.detach().contiguous();
    const int64_t n = xyz.size(0), ny = (l_max + 1) * (l_max + 1);
    const auto options = xyz.options();
    Tensor sph = at::empty({n, ny}, options), dsph, ddsph;
    if (mode >= 1) dsph = at::empty({n, 3, ny}, options);
    if (mode >= 2) ddsph = at::empty({n, 3, 3, ny}, options);
    const c10::DeviceGuard guard(xyz.device());
    if (f64) {
        check(sphx_forward_f64(pointer<double>(xyz), static_cast<size_t>(n), static_cast<int>(l_max), normalized, mode,
                               pointer<double>(sph), pointer<double>(dsph), pointer<double>(ddsph), stream_of(xyz)));
    } else {
        check(sphx_forward_f32(pointer<float>(xyz), static_cast<size_t>(n), static_cast<int>(l_max), normalized, mode,
                               pointer<float>(sph), pointer<float>(dsph), pointer<float>(ddsph), stream_of(xyz)));
    }
    return {sph, dsph, ddsph};
}

template <bool NORMALIZED> Tensor values(const Tensor& xyz, int64_t l_max) {
    return std::get<0>(forward(xyz, l_max, NORMALIZED, SPHX_VALUES));
}
template <bool NORMALIZED> std::tuple<Tensor, Tensor> with_gradients(const Tensor& xyz, int64_t l_max) {
    auto all = forward(xyz, l_max, NORMALIZED, SPHX_GRADIENTS);
    return {std::get<0>(all), std::get<1>(all)};
}
template <bool NORMALIZED> std::tuple<Tensor, Tensor, Tensor> with_hessians(const Tensor& xyz, int64_t l_max) {
    return forward(xyz, l_max, NORMALIZED, 2);
}

// the product of the gradients with sph_grad without the gradient array (sphx_vjp_*)
template <bool NORMALIZED> Tensor vjp(const Tensor& xyz_in, const Tensor& sph_grad_in, int64_t l_max) {
    const bool f64 = is_double(xyz_in, "spherical harmonics");
    TORCH_CHECK_VALUE(sph_grad_in.scalar_type() == xyz_in.scalar_type() && sph_grad_in.device() == xyz_in.device(),
                      "xyz and sph_grad must share dtype and device");
    const int64_t ny = (l_max + 1) * (l_max + 1);
    TORCH_CHECK_VALUE(xyz_in.dim() == 2 && sph_grad_in.dim() == 2 && sph_grad_in.size(0) == xyz_in.size(0) &&
                          sph_grad_in.size(1) == ny,
                      "sph_grad must have shape (", xyz_in.dim() == 2 ? xyz_in.size(0) : 0, ", ", ny, ")");
    const Tensor xyz = xyz_in.detach().contiguous(), sph_grad = sph_grad_in.detach().contiguous();
    Tensor out = at::empty_like(xyz);
    const c10::DeviceGuard guard(xyz.device());
    if (f64) {
        check(sphx_vjp_f64(pointer<double>(xyz), pointer<double>(sph_grad), static_cast<size_t>(xyz.size(0)),
                           static_cast<int>(l_max), NORMALIZED, pointer<double>(out), 0, stream_of(xyz)));
    } else {
        check(sphx_vjp_f32(pointer<float>(xyz), pointer<float>(sph_grad), static_cast<size_t>(xyz.size(0)),
                           static_cast<int>(l_max), NORMALIZED, pointer<float>(out), 0, stream_of(xyz)));
    }
    return out;
}

// xyz_grad = sum_k derivatives * upstream over the last axis (and, one order up, over the axis before the
// last but one as well): sphx_backward_* / sphx_backward_second_*
template <bool SECOND> Tensor contract(const Tensor& derivatives_in, const Tensor& upstream_in) {
    const bool f64 = is_double(derivatives_in, "contractions");
    TORCH_CHECK_VALUE(upstream_in.scalar_type() == derivatives_in.scalar_type() &&
                          upstream_in.device() == derivatives_in.device(),
                      "the two tensors of a contraction must share dtype and device");
    // dsph [n, 3, k] with sph_grad [n, k]; ddsph [n, 3, 3, k] with dsph_grad [n, 3, k]
    bool fit = derivatives_in.dim() == (SECOND ? 4 : 3) && upstream_in.dim() == derivatives_in.dim() - 1 &&
               derivatives_in.size(1) == 3;
    for (int64_t axis = 0; fit && axis < upstream_in.dim(); ++axis) {
        fit = upstream_in.size(axis) == derivatives_in.size(axis == 0 ? 0 : axis + 1);
    }
    TORCH_CHECK_VALUE(fit, "shapes ", derivatives_in.sizes(), " and ", upstream_in.sizes(), " do not contract");
    const Tensor derivatives = derivatives_in.detach().contiguous(), upstream = upstream_in.detach().contiguous();
    const int64_t n = derivatives.size(0), n_total = derivatives.size(-1);
    Tensor out = at::empty({n, 3}, derivatives.options());
    const c10::DeviceGuard guard(derivatives.device());
    void* stream = stream_of(derivatives);
    int status;
    if (f64) {
        auto* entry = SECOND ? sphx_backward_second_f64 : sphx_backward_f64;
        status = entry(pointer<double>(derivatives), pointer<double>(upstream), static_cast<size_t>(n),
                       static_cast<int>(n_total), pointer<double>(out), 0, stream);
    } else {
        auto* entry = SECOND ? sphx_backward_second_f32 : sphx_backward_f32;
        status = entry(pointer<float>(derivatives), pointer<float>(upstream), static_cast<size_t>(n),
                       static_cast<int>(n_total), pointer<float>(out), 0, stream);
    }
    check(status);
    return out;
}

[[noreturn]] void no_cpu() {
    TORCH_CHECK(false, "sphericart_amd evaluates on AMD GPUs only: move the tensor to the device "
                       "(there is no CPU implementation behind these operators)");
}
Tensor cpu_values(const Tensor&, int64_t) { no_cpu(); }
std::tuple<Tensor, Tensor> cpu_with_gradients(const Tensor&, int64_t) { no_cpu(); }
std::tuple<Tensor, Tensor, Tensor> cpu_with_hessians(const Tensor&, int64_t) { no_cpu(); }
Tensor cpu_vjp(const Tensor&, const Tensor&, int64_t) { no_cpu(); }
Tensor cpu_contract(const Tensor&, const Tensor&) { no_cpu(); }

} // namespace

// the reference's six schemas (torch.cpp:367-374) and, without counterpart there, the fused products
TORCH_LIBRARY(sphericart_amd, m) {
    for (const char* prefix : {"spherical_harmonics", "solid_harmonics"}) {
        const std::string name(prefix);
        m.def((name + "(Tensor xyz, int l_max) -> Tensor").c_str());
        m.def((name + "_with_gradients(Tensor xyz, int l_max) -> (Tensor, Tensor)").c_str());
        m.def((name + "_with_hessians(Tensor xyz, int l_max) -> (Tensor, Tensor, Tensor)").c_str());
        m.def((name + "_vjp(Tensor xyz, Tensor sph_grad, int l_max) -> Tensor").c_str());
    }
    m.def("contract_gradients(Tensor dsph, Tensor sph_grad) -> Tensor");
    m.def("contract_hessians(Tensor ddsph, Tensor dsph_grad) -> Tensor");
    m.def("owns_reference_namespace() -> bool");
}

// (the key of GPU tensors in a ROCm build of torch is CUDA)
TORCH_LIBRARY_IMPL(sphericart_amd, CUDA, m) {
    m.impl("spherical_harmonics", &values<true>);
    m.impl("spherical_harmonics_with_gradients", &with_gradients<true>);
    m.impl("spherical_harmonics_with_hessians", &with_hessians<true>);
    m.impl("spherical_harmonics_vjp", &vjp<true>);
    m.impl("solid_harmonics", &values<false>);
    m.impl("solid_harmonics_with_gradients", &with_gradients<false>);
    m.impl("solid_harmonics_with_hessians", &with_hessians<false>);
    m.impl("solid_harmonics_vjp", &vjp<false>);
    m.impl("contract_gradients", &contract<false>);
    m.impl("contract_hessians", &contract<true>);
}

TORCH_LIBRARY_IMPL(sphericart_amd, CPU, m) {
    for (const char* prefix : {"spherical_harmonics", "solid_harmonics"}) {
        const std::string name(prefix);
        m.impl(name.c_str(), &cpu_values);
        m.impl((name + "_with_gradients").c_str(), &cpu_with_gradients);
        m.impl((name + "_with_hessians").c_str(), &cpu_with_hessians);
        m.impl((name + "_vjp").c_str(), &cpu_vjp);
    }
    m.impl("contract_gradients", &cpu_contract);
    m.impl("contract_hessians", &cpu_contract);
}

// ---- the reference's namespace (sphericart-torch/src/torch.cpp:367-385) -------------------------------------
//
// `sphericart_torch` with the reference's eight schemas, so that code written against torch.ops.sphericart_torch.*,
// saved TorchScript modules included, resolves against this library alone. Every operator forwards to its twin
// above through the dispatcher (a composite implementation: whatever autograd, fake-tensor and vmap rules the twin
// has apply unchanged); the two *_omp_num_threads operators report 1, there being no host evaluator and no OpenMP
// team behind these operators. Defined when this library is loaded unless the namespace is taken already (the
// reference's own extension is loaded): then nothing is defined and owns_reference_namespace() says so.
namespace {

template <typename Signature> c10::TypedOperatorHandle<Signature> twin(const std::string& name) {
    return c10::Dispatcher::singleton().findSchemaOrThrow(("sphericart_amd::" + name).c_str(), "").typed<Signature>();
}

template <bool NORMALIZED> const char* prefix_of() {
    return NORMALIZED ? "spherical_harmonics" : "solid_harmonics";
}
template <bool NORMALIZED> Tensor reference_values(const Tensor& xyz, int64_t l_max) {
    static const auto op = twin<Tensor(const Tensor&, int64_t)>(prefix_of<NORMALIZED>());
    return op.call(xyz, l_max);
}
template <bool NORMALIZED> std::tuple<Tensor, Tensor> reference_with_gradients(const Tensor& xyz, int64_t l_max) {
    static const auto op =
        twin<std::tuple<Tensor, Tensor>(const Tensor&, int64_t)>(std::string(prefix_of<NORMALIZED>()) + "_with_gradients");
    return op.call(xyz, l_max);
}
template <bool NORMALIZED>
std::tuple<Tensor, Tensor, Tensor> reference_with_hessians(const Tensor& xyz, int64_t l_max) {
    static const auto op = twin<std::tuple<Tensor, Tensor, Tensor>(const Tensor&, int64_t)>(
        std::string(prefix_of<NORMALIZED>()) + "_with_hessians");
    return op.call(xyz, l_max);
}
int64_t one_thread(int64_t) { return 1; }

std::unique_ptr<torch::Library> define_reference_namespace() {
    try {
        auto m = std::make_unique<torch::Library>(torch::Library::DEF, "sphericart_torch", c10::nullopt, __FILE__,
                                                  __LINE__);
        for (const char* prefix : {"spherical_harmonics", "solid_harmonics"}) {
            const std::string name(prefix);
            m->def((name + "(Tensor xyz, int l_max) -> Tensor").c_str());
            m->def((name + "_with_gradients(Tensor xyz, int l_max) -> (Tensor, Tensor)").c_str());
            m->def((name + "_with_hessians(Tensor xyz, int l_max) -> (Tensor, Tensor, Tensor)").c_str());
            m->def((name + "_omp_num_threads(int l_max) -> int").c_str());
            m->impl((name + "_omp_num_threads").c_str(), c10::DispatchKey::CompositeExplicitAutograd, &one_thread);
        }
        const auto composite = c10::DispatchKey::CompositeImplicitAutograd;
        m->impl("spherical_harmonics", composite, &reference_values<true>);
        m->impl("spherical_harmonics_with_gradients", composite, &reference_with_gradients<true>);
        m->impl("spherical_harmonics_with_hessians", composite, &reference_with_hessians<true>);
        m->impl("solid_harmonics", composite, &reference_values<false>);
        m->impl("solid_harmonics_with_gradients", composite, &reference_with_gradients<false>);
        m->impl("solid_harmonics_with_hessians", composite, &reference_with_hessians<false>);
        return m;
    } catch (const c10::Error&) {
        return nullptr; // another library owns the namespace
    }
}

const std::unique_ptr<torch::Library> reference_namespace = define_reference_namespace();

bool owns_reference_namespace() { return reference_namespace != nullptr; }

} // namespace

TORCH_LIBRARY_IMPL(sphericart_amd, CompositeExplicitAutograd, m) {
    m.impl("owns_reference_namespace", &owns_reference_namespace);
}
