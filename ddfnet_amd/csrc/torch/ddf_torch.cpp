// PyTorch front end of libddf_hip.so as a C++ extension: the `ddf` operator as a
// C++ autograd function.  Host-side mirror of DDFFunction / ddf of the reference
// (ddf/ddf.py:27-122): same arguments, same assertion messages.  This file holds
// no device code; every kernel is behind the C ABI of include/ddf_hip.h, and
// torch is used for tensors, the caching allocator and the current stream.
//
// What it saves over the Python autograd.Function in functional.py is host time
// per call: argument checks, dtype promotion, output allocation and the two
// library calls happen without the interpreter.
#include <torch/extension.h>

#include <ATen/autocast_mode.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <sstream>
#include <string>

#include "ddf_hip.h"

namespace {

namespace py = pybind11;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

// `assert cond, msg` of the Python front end.
// (Also reached from the autograd engine's threads, which do not hold the GIL.)
[[noreturn]] void assertion_error(const std::string &msg) {
    py::gil_scoped_acquire gil;
    PyErr_SetString(PyExc_AssertionError, msg.c_str());
    throw py::error_already_set();
}

// A failed library call, raised as ddfnet_amd._lib.DDFHipError.
void check_status(int status) {
    if (status == DDF_OK) return;
    const std::string msg = std::string(ddf_hip_status_string(status)) + ": " + ddf_hip_last_error();
    py::gil_scoped_acquire gil;
    py::object cls = py::module_::import("ddfnet_amd._lib").attr("DDFHipError");
    PyErr_SetString(cls.ptr(), msg.c_str());
    throw py::error_already_set();
}

int dtype_code(at::ScalarType t) {
    switch (t) {
        case at::kHalf: return DDF_F16;
        case at::kFloat: return DDF_F32;
        case at::kDouble: return DDF_F64;
        default: return -1;
    }
}

std::string size_string(const at::Tensor &t) {
    // as torch.Size prints: torch.Size([2, 3, 4, 5])
    std::ostringstream os;
    os << "torch.Size([";
    for (int64_t i = 0; i < t.dim(); ++i) os << (i ? ", " : "") << t.size(i);
    os << "])";
    return os.str();
}

hipStream_t current_stream(const at::Tensor &t) {
    return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

class DDFAutograd : public torch::autograd::Function<DDFAutograd> {
public:
    // Operands are contiguous device tensors of one supported dtype with matching
    // shapes (ddf() below has seen to that).
    static at::Tensor forward(AutogradContext *ctx, const at::Tensor &features,
                              const at::Tensor &channel_filter, const at::Tensor &spatial_filter,
                              int64_t k, int64_t d, int64_t s, int64_t combine, int64_t variant) {
        const int64_t b = features.size(0), c = features.size(1), h = features.size(2),
                      w = features.size(3);
        // the kernels write every element, so no zero fill
        at::Tensor out = at::empty({b, c, h / s, w / s}, features.options());
        {
            c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(features.device());
            check_status(ddf_hip_forward(features.data_ptr(), channel_filter.data_ptr(),
                                         spatial_filter.data_ptr(), out.data_ptr(), b, c, h, w,
                                         (int)k, (int)d, (int)s, (int)combine,
                                         dtype_code(features.scalar_type()), (int)variant,
                                         current_stream(features)));
        }
        if (features.requires_grad() || channel_filter.requires_grad() || spatial_filter.requires_grad())
            ctx->save_for_backward({features, channel_filter, spatial_filter});
        ctx->saved_data["k"] = k;
        ctx->saved_data["d"] = d;
        ctx->saved_data["s"] = s;
        ctx->saved_data["combine"] = combine;
        ctx->saved_data["variant"] = variant;
        return out;
    }

    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const at::Tensor &features = saved[0], &channel_filter = saved[1], &spatial_filter = saved[2];
        const int k = (int)ctx->saved_data["k"].toInt(), d = (int)ctx->saved_data["d"].toInt(),
                  s = (int)ctx->saved_data["s"].toInt(),
                  combine = (int)ctx->saved_data["combine"].toInt();
        // 'f' forces the tiled kernels in the forward pass only (the reference's
        // faster modules export no backward)
        const int variant = ctx->saved_data["variant"].toInt() == DDF_VARIANT_GENERIC
                                ? DDF_VARIANT_GENERIC : DDF_VARIANT_AUTO;
        if (!grads[0].is_cuda()) assertion_error("");
        const at::Tensor go = grads[0].to(features.scalar_type()).contiguous();

        // only the gradients autograd asks for are computed
        unsigned need = 0;
        at::Tensor dx, dcf, dsf;
        if (ctx->needs_input_grad(0)) { need |= DDF_NEED_DX; dx = at::empty_like(features); }
        if (ctx->needs_input_grad(1)) { need |= DDF_NEED_DCF; dcf = at::empty_like(channel_filter); }
        if (ctx->needs_input_grad(2)) { need |= DDF_NEED_DSF; dsf = at::empty_like(spatial_filter); }
        if (need) {
            const int64_t b = features.size(0), c = features.size(1), h = features.size(2),
                          w = features.size(3);
            const int dt = dtype_code(features.scalar_type());
            c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(features.device());
            const size_t bytes = ddf_hip_backward_workspace_bytes(b, c, h, w, k, d, s, combine, dt,
                                                                  need, variant);
            at::Tensor ws;
            if (bytes) ws = at::empty({(int64_t)bytes}, features.options().dtype(at::kByte));
            check_status(ddf_hip_backward(
                go.data_ptr(), features.data_ptr(), channel_filter.data_ptr(),
                spatial_filter.data_ptr(), dx.defined() ? dx.data_ptr() : nullptr,
                dcf.defined() ? dcf.data_ptr() : nullptr, dsf.defined() ? dsf.data_ptr() : nullptr,
                bytes ? ws.data_ptr() : nullptr, bytes, b, c, h, w, k, d, s, combine, dt, need,
                variant, current_stream(features)));
        }
        return {dx, dcf, dsf, at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor()};
    }
};

// ddf(features, channel_filter, spatial_filter, kernel_size=3, dilation=1, stride=1,
//     kernel_combine='mul', version=''): checks in the order and with the messages of
// DDFFunction.forward in functional.py (ddf/ddf.py:29-62 of the reference).
at::Tensor ddf(at::Tensor features, at::Tensor channel_filter, at::Tensor spatial_filter,
               int64_t kernel_size, int64_t dilation, int64_t stride,
               const std::string &kernel_combine, const std::string &version) {
    if (!features.is_cuda()) assertion_error("input feature must be a CUDA tensor.");
    if (!channel_filter.is_cuda()) assertion_error("channel_filter must be a CUDA tensor.");
    if (!spatial_filter.is_cuda()) assertion_error("spatial_filter must be a CUDA tensor.");

    // One working dtype for the three operands.  Under autocast to fp16 that is
    // fp16 (the kernels accumulate in fp32); bf16 is not a storage type of the
    // library, so autocast to bf16 leaves the operands as they are.
    at::ScalarType dtype = at::promote_types(
        at::promote_types(features.scalar_type(), channel_filter.scalar_type()),
        spatial_filter.scalar_type());
    if (at::autocast::is_autocast_enabled(at::kCUDA) &&
        at::autocast::get_autocast_dtype(at::kCUDA) == at::kHalf && dtype == at::kFloat)
        dtype = at::kHalf;
    if (dtype_code(dtype) < 0) {
        std::ostringstream os;
        os << "unsupported dtype " << dtype;
        assertion_error(os.str());
    }
    if (features.dim() != 4 || channel_filter.dim() != 4 || spatial_filter.dim() != 4)
        assertion_error("features, channel_filter and spatial_filter must be 4-dimensional");
    if (stride < 1) assertion_error("");
    features = features.to(dtype).contiguous();
    channel_filter = channel_filter.to(dtype).contiguous();
    spatial_filter = spatial_filter.to(dtype).contiguous();

    const int64_t b = features.size(0), c = features.size(1), h = features.size(2), w = features.size(3);
    const int64_t out_h = h / stride, out_w = w / stride;
    if (channel_filter.size(0) != b || channel_filter.size(1) != c)
        assertion_error("channel_filter size " + size_string(channel_filter) +
                        " does not match feature size " + size_string(features));
    if (channel_filter.size(2) != kernel_size || channel_filter.size(3) != kernel_size)
        assertion_error("channel_filter size " + size_string(channel_filter) +
                        " does not match kernel size " + std::to_string(kernel_size));
    if (spatial_filter.size(0) != b || spatial_filter.size(2) != out_h || spatial_filter.size(3) != out_w)
        assertion_error("spatial_filter size " + size_string(spatial_filter) +
                        " does not match feature size " + size_string(features) + " with stride " +
                        std::to_string(stride));
    if (spatial_filter.size(1) != kernel_size * kernel_size)
        assertion_error("spatial_filter size " + size_string(spatial_filter) +
                        " does not match kernel size " + std::to_string(kernel_size));
    if ((kernel_size - 1) % 2 != 0 || kernel_size < 1 || dilation < 1) assertion_error("");
    int combine;
    if (kernel_combine == "mul") combine = DDF_MUL;
    else if (kernel_combine == "add") combine = DDF_ADD;
    else assertion_error("only support mul or add combination, instead of " + kernel_combine);
    int variant;
    if (version.empty()) variant = DDF_VARIANT_AUTO;
    else if (version == "o") variant = DDF_VARIANT_GENERIC;
    else if (version == "f") variant = DDF_VARIANT_TILED;
    else assertion_error("version must be '', 'o' or 'f', instead of " + version);

    return DDFAutograd::apply(features, channel_filter, spatial_filter, kernel_size, dilation, stride,
                              (int64_t)combine, (int64_t)variant);
}

// Up-sampling DDF (DDFUpPack.forward, ddf/ddf.py:264-272 of the reference: one
// ddf call per sub-pixel branch, torch.stack, F.pixel_shuffle) as one operator:
// one library call forward, one backward.  `filters` holds the scale*scale
// channel filters followed by the scale*scale spatial filters.
class DDFUpAutograd : public torch::autograd::Function<DDFUpAutograd> {
public:
    // (filters as a TensorList: that is the list type whose elements autograd tracks)
    static at::Tensor forward(AutogradContext *ctx, const at::Tensor &features, at::TensorList filters,
                              int64_t k, int64_t d, int64_t scale, int64_t combine) {
        const int64_t branches = scale * scale;
        const int64_t b = features.size(0), c = features.size(1), h = features.size(2),
                      w = features.size(3);
        const void *cf[DDF_UP_MAX_BRANCHES], *sf[DDF_UP_MAX_BRANCHES];
        for (int64_t i = 0; i < branches; ++i) {
            cf[i] = filters[i].data_ptr();
            sf[i] = filters[branches + i].data_ptr();
        }
        at::Tensor out = at::empty({b, c, h * scale, w * scale}, features.options());
        {
            c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(features.device());
            check_status(ddf_hip_up_forward(features.data_ptr(), cf, sf, out.data_ptr(), b, c, h, w,
                                            (int)k, (int)d, (int)scale, (int)combine,
                                            dtype_code(features.scalar_type()),
                                            current_stream(features)));
        }
        bool any = features.requires_grad();
        for (const auto &t : filters) any = any || t.requires_grad();
        if (any) {
            variable_list saved;
            saved.reserve(1 + filters.size());
            saved.push_back(features);
            for (const auto &t : filters) saved.push_back(t);
            ctx->save_for_backward(saved);
        }
        ctx->saved_data["k"] = k;
        ctx->saved_data["d"] = d;
        ctx->saved_data["scale"] = scale;
        ctx->saved_data["combine"] = combine;
        return out;
    }

    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const at::Tensor &features = saved[0];
        const int k = (int)ctx->saved_data["k"].toInt(), d = (int)ctx->saved_data["d"].toInt(),
                  scale = (int)ctx->saved_data["scale"].toInt(),
                  combine = (int)ctx->saved_data["combine"].toInt();
        const int branches = scale * scale;
        const at::Tensor go = grads[0].to(features.scalar_type()).contiguous();
        variable_list result(1 + 2 * branches + 4);
        unsigned need = 0;
        const void *cf[DDF_UP_MAX_BRANCHES], *sf[DDF_UP_MAX_BRANCHES];
        void *dcf[DDF_UP_MAX_BRANCHES], *dsf[DDF_UP_MAX_BRANCHES];
        if (ctx->needs_input_grad(0)) {
            need |= DDF_NEED_DX;
            result[0] = at::empty_like(features);
        }
        for (int i = 0; i < branches; ++i) {
            cf[i] = saved[1 + i].data_ptr();
            sf[i] = saved[1 + branches + i].data_ptr();
            dcf[i] = dsf[i] = nullptr;
            if (ctx->needs_input_grad(1 + i)) {
                need |= DDF_NEED_DCF;
                result[1 + i] = at::empty_like(saved[1 + i]);
                dcf[i] = result[1 + i].data_ptr();
            }
            if (ctx->needs_input_grad(1 + branches + i)) {
                need |= DDF_NEED_DSF;
                result[1 + branches + i] = at::empty_like(saved[1 + branches + i]);
                dsf[i] = result[1 + branches + i].data_ptr();
            }
        }
        if (need) {
            const int64_t b = features.size(0), c = features.size(1), h = features.size(2),
                          w = features.size(3);
            const int dt = dtype_code(features.scalar_type());
            c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(features.device());
            const size_t bytes = ddf_hip_up_backward_workspace_bytes(b, c, h, w, k, d, scale, combine,
                                                                     dt, need);
            at::Tensor ws = at::empty({(int64_t)std::max<size_t>(bytes, 1)},
                                      features.options().dtype(at::kByte));
            check_status(ddf_hip_up_backward(
                go.data_ptr(), features.data_ptr(), cf, sf,
                result[0].defined() ? result[0].data_ptr() : nullptr, dcf, dsf, ws.data_ptr(), bytes,
                b, c, h, w, k, d, scale, combine, dt, need, current_stream(features)));
        }
        return result;
    }
};

// ddf_up(features, channel_filters, spatial_filters, kernel_size, dilation, scale_factor,
// kernel_combine): the checks of DDFUpFunction.forward in functional.py.  The caller has
// asked ddf_hip_up_forward's coverage (functional.ddf_up falls back to the composition).
at::Tensor ddf_up(at::Tensor features, std::vector<at::Tensor> channel_filters,
                  std::vector<at::Tensor> spatial_filters, int64_t kernel_size, int64_t dilation,
                  int64_t scale, const std::string &kernel_combine) {
    const int64_t branches = scale * scale;
    if (scale < 2 || branches > DDF_UP_MAX_BRANCHES ||
        (int64_t)channel_filters.size() != branches || (int64_t)spatial_filters.size() != branches)
        assertion_error("expected " + std::to_string(branches) + " channel filters followed by " +
                        std::to_string(branches) + " spatial filters");
    if (!features.is_cuda()) assertion_error("input feature must be a CUDA tensor.");
    int combine;
    if (kernel_combine == "mul") combine = DDF_MUL;
    else if (kernel_combine == "add") combine = DDF_ADD;
    else assertion_error("only support mul or add combination, instead of " + kernel_combine);
    if ((kernel_size - 1) % 2 != 0 || kernel_size < 1 || dilation < 1) assertion_error("");
    at::ScalarType dtype = features.scalar_type();
    for (const auto *list : {&channel_filters, &spatial_filters})
        for (const auto &t : *list) {
            if (!t.is_cuda()) assertion_error("filters must be CUDA tensors.");
            dtype = at::promote_types(dtype, t.scalar_type());
        }
    if (at::autocast::is_autocast_enabled(at::kCUDA) &&
        at::autocast::get_autocast_dtype(at::kCUDA) == at::kHalf && dtype == at::kFloat)
        dtype = at::kHalf;
    if (dtype_code(dtype) < 0) {
        std::ostringstream os;
        os << "unsupported dtype " << dtype;
        assertion_error(os.str());
    }
    if (features.dim() != 4) assertion_error("features must be 4-dimensional");
    features = features.to(dtype).contiguous();
    const int64_t b = features.size(0), c = features.size(1), h = features.size(2), w = features.size(3);
    variable_list filters;
    filters.reserve(2 * branches);
    for (auto &t : channel_filters) {
        t = t.to(dtype).contiguous();
        if (t.dim() != 4 || t.size(0) != b || t.size(1) != c || t.size(2) != kernel_size ||
            t.size(3) != kernel_size)
            assertion_error("channel_filter size " + size_string(t) + " does not match feature size " +
                            size_string(features));
        filters.push_back(t);
    }
    for (auto &t : spatial_filters) {
        t = t.to(dtype).contiguous();
        if (t.dim() != 4 || t.size(0) != b || t.size(1) != kernel_size * kernel_size ||
            t.size(2) != h || t.size(3) != w)
            assertion_error("spatial_filter size " + size_string(t) + " does not match feature size " +
                            size_string(features));
        filters.push_back(t);
    }
    return DDFUpAutograd::apply(features, at::TensorList(filters), kernel_size, dilation, scale,
                                (int64_t)combine);
}

const void *ptr_or_null(const c10::optional<at::Tensor> &t) {
    return t.has_value() && t->defined() ? t->data_ptr() : nullptr;
}

// DDFPack.forward without gradients (ddf/ddf.py:195-222 of the reference), four
// launches: global average pool (torch), channel branch, spatial branch, operator.
// The caller (DDFPack._inference_forward in modules.py) has checked that the
// branches are the stock ones and that every tensor is a device tensor of the
// features' dtype; weights are the 1x1 convolutions' (out, in, 1, 1) tensors.
at::Tensor ddf_pack_forward(const at::Tensor &features, const at::Tensor &conv_weight,
                            const c10::optional<at::Tensor> &conv_bias, double spatial_gain,
                            const c10::optional<at::Tensor> &spatial_gain_vec,
                            const c10::optional<at::Tensor> &spatial_offset_vec,
                            const at::Tensor &fc1_weight, const c10::optional<at::Tensor> &fc1_bias,
                            const at::Tensor &fc2_weight, const c10::optional<at::Tensor> &fc2_bias,
                            double channel_gain, const c10::optional<at::Tensor> &channel_gain_vec,
                            const c10::optional<at::Tensor> &channel_offset_vec,
                            int64_t kernel_size, int64_t dilation, int64_t stride, int64_t head,
                            const std::string &kernel_combine, bool fuse_pool) {
    TORCH_CHECK(features.is_cuda() && features.dim() == 4, "features must be a 4-d device tensor");
    const int dt = dtype_code(features.scalar_type());
    TORCH_CHECK(dt == DDF_F16 || dt == DDF_F32, "ddf_pack_forward covers fp16 and fp32");
    int combine;
    if (kernel_combine == "mul") combine = DDF_MUL;
    else if (kernel_combine == "add") combine = DDF_ADD;
    else assertion_error("only support mul or add combination, instead of " + kernel_combine);
    const at::Tensor x = features.contiguous();
    const int64_t b = x.size(0), c = x.size(1), h = x.size(2), w = x.size(3);
    const int64_t ho = h / stride, wo = w / stride, kk = kernel_size * kernel_size;
    TORCH_CHECK(head >= 1 && c % head == 0, "channels must divide into heads");
    TORCH_CHECK(conv_weight.is_contiguous() && fc1_weight.is_contiguous() && fc2_weight.is_contiguous(),
                "weights must be contiguous");
    TORCH_CHECK(conv_weight.size(0) == head * kk && conv_weight.size(1) == c &&
                fc1_weight.size(1) == c && fc2_weight.size(0) == c * kk &&
                fc2_weight.size(1) == fc1_weight.size(0), "branch weights do not fit the features");
    const int64_t mid = fc1_weight.size(0);

    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(x.device());
    hipStream_t st = current_stream(x);
    at::Tensor cf = at::empty({b, c, kernel_size, kernel_size}, x.options());
    at::Tensor sf = at::empty({b, head * kk, ho, wo}, x.options());
    // The spatial branch reads every feature plane anyway: where its kernel can, it leaves
    // the planes' partial sums and the channel branch pools from those (one launch and
    // one read of the feature map fewer); else pool first.
    bool pooled_on_the_way = false;
    if (fuse_pool && b * c * ho * wo > 0) {
        const int64_t cap = b * c * ((ho * wo + 63) / 64) * 4;
        at::Tensor parts = at::empty({cap}, x.options().dtype(at::kFloat));
        int n_parts = 0;
        const int rc = ddf_hip_spatial_branch_pool(
            x.data_ptr(), conv_weight.data_ptr(), ptr_or_null(conv_bias), sf.data_ptr(),
            parts.data_ptr<float>(), cap, &n_parts, b, c, h, w, (int)head, (int)kernel_size, (int)stride,
            spatial_gain, ptr_or_null(spatial_gain_vec), ptr_or_null(spatial_offset_vec), dt, st);
        if (rc != DDF_ERR_UNSUPPORTED) {
            check_status(rc);
            check_status(ddf_hip_channel_branch_parts(
                parts.data_ptr<float>(), n_parts, 1.0 / (double)(h * w), fc1_weight.data_ptr(),
                ptr_or_null(fc1_bias), fc2_weight.data_ptr(), ptr_or_null(fc2_bias), cf.data_ptr(), b, c, mid,
                (int)kernel_size, channel_gain, ptr_or_null(channel_gain_vec),
                ptr_or_null(channel_offset_vec), dt, st));
            pooled_on_the_way = true;
        }
    }
    if (!pooled_on_the_way) {
        const at::Tensor pooled = at::mean(x, {2, 3});
        check_status(ddf_hip_channel_branch(
            pooled.data_ptr(), fc1_weight.data_ptr(), ptr_or_null(fc1_bias), fc2_weight.data_ptr(),
            ptr_or_null(fc2_bias), cf.data_ptr(), b, c, mid, (int)kernel_size, channel_gain,
            ptr_or_null(channel_gain_vec), ptr_or_null(channel_offset_vec), dt, st));
        check_status(ddf_hip_spatial_branch(
            x.data_ptr(), conv_weight.data_ptr(), ptr_or_null(conv_bias), sf.data_ptr(), b, c, h, w,
            (int)head, (int)kernel_size, (int)stride, spatial_gain, ptr_or_null(spatial_gain_vec),
            ptr_or_null(spatial_offset_vec), dt, st));
    }
    at::Tensor out = at::empty({b, c, ho, wo}, x.options());
    // heads are folded into the batch: (b * head, c / head, h, w)
    check_status(ddf_hip_forward(x.data_ptr(), cf.data_ptr(), sf.data_ptr(), out.data_ptr(), b * head,
                                 c / head, h, w, (int)kernel_size, (int)dilation, (int)stride, combine,
                                 dt, DDF_VARIANT_AUTO, st));
    return out;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "ddf operator of libddf_hip.so as a C++ autograd function";
    m.def("ddf", &ddf, py::arg("features"), py::arg("channel_filter"), py::arg("spatial_filter"),
          py::arg("kernel_size") = 3, py::arg("dilation") = 1, py::arg("stride") = 1,
          py::arg("kernel_combine") = "mul", py::arg("version") = "");
    m.def("ddf_up", &ddf_up, py::arg("features"), py::arg("channel_filters"),
          py::arg("spatial_filters"), py::arg("kernel_size") = 3, py::arg("dilation") = 1,
          py::arg("scale_factor") = 2, py::arg("kernel_combine") = "mul");
    m.def("ddf_pack_forward", &ddf_pack_forward,
          "DDFPack.forward without gradients: spatial branch (pooling on the way where it can), "
          "channel branch, operator");
    m.def("library_version", []() { return ddf_hip_version(); });
}
