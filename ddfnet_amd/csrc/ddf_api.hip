// C ABI of the DDF HIP library: argument validation and kernel-family choice.
// Declarations and the reference entry points each call replaces are in
// include/ddf_hip.h.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "ddf_common.h"

// Scratch of ddf_hip_backward_static: device memory that belongs to the library's
// code object, so that entry point never allocates.  Every GPU the library runs on
// holds its own copy at its own address until the process ends.  (In host code
// the name below is only a handle for hipGetSymbolAddress, not a device address.)
static __device__ __align__(256) unsigned char scratch[DDF_HIP_STATIC_SCRATCH_BYTES];

namespace {

thread_local char g_last_error[512] = "";

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return status;
}

int fail_hip(hipError_t err, const char *what) {
    return fail(DDF_ERR_HIP, "%s: %s", what, hipGetErrorString(err));
}

// Checks shared by forward and backward.  Mirrors the argument contract of
// DDFFunction.forward (ddf/ddf.py:45-65 of the reference): odd k >= 1,
// d >= 1, s >= 1, known combine; sizes must be non-negative.
int check_problem(int64_t N, int64_t C, int64_t H, int64_t W, int k, int d, int s,
                  int combine, int dtype, int variant) {
    if (N < 0 || C < 0 || H < 0 || W < 0)
        return fail(DDF_ERR_BAD_ARG, "negative tensor size (N=%lld C=%lld H=%lld W=%lld)",
                    (long long)N, (long long)C, (long long)H, (long long)W);
    if (k < 1 || (k - 1) % 2 != 0 || d < 1 || s < 1)
        return fail(DDF_ERR_BAD_ARG,
                    "kernel_size must be odd and >= 1, dilation and stride >= 1 "
                    "(got k=%d d=%d s=%d)", k, d, s);
    if (combine != DDF_MUL && combine != DDF_ADD)
        return fail(DDF_ERR_BAD_ARG, "combine must be DDF_MUL or DDF_ADD (got %d)", combine);
    if (dtype != DDF_F16 && dtype != DDF_F32 && dtype != DDF_F64)
        return fail(DDF_ERR_BAD_ARG, "unknown dtype %d", dtype);
    if (variant != DDF_VARIANT_AUTO && variant != DDF_VARIANT_GENERIC &&
        variant != DDF_VARIANT_TILED)
        return fail(DDF_ERR_BAD_ARG, "unknown variant %d", variant);
    // Index arithmetic inside the kernels is 64-bit, but a single (n, c) plane
    // and the tap window must fit 32-bit offsets.
    if (H > (1 << 24) || W > (1 << 24) || (int64_t)k * d > (1 << 20))
        return fail(DDF_ERR_UNSUPPORTED, "plane or window too large");
    return DDF_OK;
}

template <typename T>
int forward_typed(const ddf::Problem &p, const void *x, const void *cf, const void *sf,
                  void *out, int dtype, int variant, hipStream_t stream) {
    const bool tiled_ok = ddf::tiled_forward_supported(p, dtype);
    if (variant == DDF_VARIANT_TILED && !tiled_ok)
        return fail(DDF_ERR_UNSUPPORTED,
                    "tiled forward does not cover k=%d d=%d s=%d H=%lld W=%lld", p.k, p.d,
                    p.s, (long long)p.H, (long long)p.W);
    hipError_t err;
    if (tiled_ok && variant != DDF_VARIANT_GENERIC)
        err = ddf::tiled_forward<T>(p, (const T *)x, (const T *)cf, (const T *)sf, (T *)out,
                                    stream);
    else
        err = ddf::generic_forward<T>(p, (const T *)x, (const T *)cf, (const T *)sf,
                                      (T *)out, stream);
    return err == hipSuccess ? DDF_OK : fail_hip(err, "ddf_hip_forward launch");
}

template <typename T>
int backward_typed(const ddf::Problem &p, const void *go, const void *x, const void *cf,
                   const void *sf, void *dx, void *dcf, void *dsf, void *ws,
                   size_t ws_bytes, int dtype, unsigned need, int variant,
                   hipStream_t stream) {
    const bool tiled_ok = ddf::tiled_backward_supported(p, dtype);
    if (variant == DDF_VARIANT_TILED && !tiled_ok)
        return fail(DDF_ERR_UNSUPPORTED,
                    "tiled backward does not cover k=%d d=%d s=%d H=%lld W=%lld", p.k, p.d,
                    p.s, (long long)p.H, (long long)p.W);
    hipError_t err;
    if (tiled_ok && variant != DDF_VARIANT_GENERIC) {
        const size_t want = ddf::tiled_backward_workspace(p, dtype, need);
        if (want > 0 && (ws == nullptr || ws_bytes < want))
            return fail(DDF_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", want,
                        ws == nullptr ? (size_t)0 : ws_bytes);
        if (want > 0 && ((uintptr_t)ws & 255u) != 0)
            return fail(DDF_ERR_WORKSPACE, "workspace must be 256-byte aligned");
        err = ddf::tiled_backward<T>(p, (const T *)go, (const T *)x, (const T *)cf,
                                     (const T *)sf, (T *)dx, (T *)dcf, (T *)dsf, ws, need,
                                     stream);
    } else {
        err = ddf::generic_backward<T>(p, (const T *)go, (const T *)x, (const T *)cf,
                                       (const T *)sf, (T *)dx, (T *)dcf, (T *)dsf, need,
                                       stream);
    }
    return err == hipSuccess ? DDF_OK : fail_hip(err, "ddf_hip_backward launch");
}

size_t align256(size_t v) { return (v + 255) / 256 * 256; }

// ddf_hip_backward with the spatial filter normalisation behind dSF.  The
// workspace starts with room for a complete dSF (storage type); the rest is the
// backward pass's own.
template <typename T>
int backward_norm_typed(const ddf::Problem &p, const void *go, const void *x, const void *cf,
                        const void *sf, const void *raw, void *dx, void *dcf, void *d_raw,
                        void *terms, void *ws, size_t ws_bytes, int dtype, unsigned need,
                        int groups, double gain, const void *gain_vec, int variant,
                        hipStream_t stream) {
    const size_t n_sf = (size_t)(p.N * p.kk * p.Ho * p.Wo);
    const size_t tmp_bytes = (need & DDF_NEED_DSF) ? align256(n_sf * sizeof(T)) : 0;
    const bool tiled = variant != DDF_VARIANT_GENERIC && ddf::tiled_backward_supported(p, dtype);
    const size_t inner = tiled ? ddf::tiled_backward_workspace(p, dtype, need) : 0;
    if (tmp_bytes + inner > 0 && (ws == nullptr || ws_bytes < tmp_bytes + inner))
        return fail(DDF_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", tmp_bytes + inner,
                    ws == nullptr ? (size_t)0 : ws_bytes);
    if (tmp_bytes + inner > 0 && ((uintptr_t)ws & 255u) != 0)
        return fail(DDF_ERR_WORKSPACE, "workspace must be 256-byte aligned");
    T *tmp = tmp_bytes ? static_cast<T *>(ws) : nullptr;
    void *rest = inner ? static_cast<unsigned char *>(ws) + tmp_bytes : nullptr;
    ddf::NormTail<T> tail{(const T *)raw, (T *)d_raw, (T *)terms, (const T *)gain_vec, groups, gain,
                          false};
    hipError_t err;
    if (tiled)
        err = ddf::tiled_backward<T>(p, (const T *)go, (const T *)x, (const T *)cf, (const T *)sf,
                                     (T *)dx, (T *)dcf, tmp, rest, need, stream,
                                     (need & DDF_NEED_DSF) ? &tail : nullptr);
    else
        err = ddf::generic_backward<T>(p, (const T *)go, (const T *)x, (const T *)cf, (const T *)sf,
                                       (T *)dx, (T *)dcf, tmp, need, stream);
    if (err != hipSuccess) return fail_hip(err, "ddf_hip_backward_spatial_norm launch");
    if ((need & DDF_NEED_DSF) && !tail.applied) {
        // (no pass over dSF to ride on: the normalisation's gradient as a launch of its own)
        err = ddf::filter_norm_backward<T>(tmp, (const T *)raw, (T *)d_raw, (T *)terms,
                                           p.N / groups, groups, p.kk, p.Ho * p.Wo, gain,
                                           (const T *)gain_vec, stream);
        if (err != hipSuccess) return fail_hip(err, "ddf_hip_backward_spatial_norm norm launch");
    }
    return DDF_OK;
}

// Address of `scratch` on the current device, looked up once per device (with
// that device current) and kept.
constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

int scratch_of_current_device(void **out) {
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return fail_hip(err, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices)
        return fail(DDF_ERR_UNSUPPORTED, "device index %d beyond the %d this entry point keeps scratch for",
                    dev, kMaxDevices);
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        p = g_scratch_ptr[dev].load(std::memory_order_acquire);
        if (p == nullptr) {
            err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (err != hipSuccess || p == nullptr)
                return fail_hip(err, "hipGetSymbolAddress(scratch)");
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return DDF_OK;
}

// Workspace of the up-sampling backward: the lattices of dO, the per-branch
// feature gradients (when dX is wanted) and one branch's own workspace.
struct UpWorkspace {
    size_t lattices, dx_parts, branch, total;
    // all branches as one batch on the row-register kernels (batched = false: not covered)
    bool batched;
    size_t cf_all, sf_all, dcf_all, dsf_all, batch_ws;
};

UpWorkspace up_workspace(const ddf::Problem &p, int scale, int dtype, unsigned need) {
    const size_t esz = dtype == DDF_F16 ? 2 : dtype == DDF_F32 ? 4 : 8;
    const size_t n_x = (size_t)(p.N * p.C * p.H * p.W);
    const size_t branches = (size_t)scale * scale;
    UpWorkspace w{};
    w.lattices = align256(n_x * esz * branches);
    w.dx_parts = (need & DDF_NEED_DX) ? align256(n_x * esz * branches) : 0;
    w.branch = ddf::tiled_backward_supported(p, dtype)
                   ? align256(ddf::tiled_backward_workspace(p, dtype, need))
                   : 0;
    w.total = w.lattices + w.dx_parts + w.branch;
    // The batch of scale*scale * N samples: the branches' filters and filter
    // gradients back to back, and the kernels' own workspace for that batch.
    const ddf::Problem pb = ddf::make_problem(p.N * (int64_t)branches, p.C, p.H, p.W, p.k, p.d, 1,
                                              p.mul ? DDF_MUL : DDF_ADD);
    w.batched = dtype != DDF_F64 && p.N * (int64_t)branches <= (1 << 24) &&
                ddf::rows_cover_backward(pb, dtype);
    if (w.batched) {
        const size_t n_cf = (size_t)(p.N * p.C * p.kk), n_sf = (size_t)(p.N * p.kk * p.H * p.W);
        w.cf_all = align256(n_cf * esz * branches);
        w.sf_all = align256(n_sf * esz * branches);
        w.dcf_all = (need & DDF_NEED_DCF) ? w.cf_all : 0;
        w.dsf_all = (need & DDF_NEED_DSF) ? w.sf_all : 0;
        w.batch_ws = align256(ddf::rows_filters_workspace(pb, dtype, need));
        const size_t total = w.lattices + w.dx_parts + w.cf_all + w.sf_all + w.dcf_all + w.dsf_all +
                             w.batch_ws;
        w.total = std::max(w.total, total);   // (room for the branch-by-branch route as well)
    }
    return w;
}

template <typename T>
int up_backward_typed(const ddf::Problem &p, int scale, const void *go, const void *x,
                      const void *const *cfs, const void *const *sfs, void *dx, void *const *dcfs,
                      void *const *dsfs, void *ws, int dtype, unsigned need, hipStream_t stream) {
    const UpWorkspace w = up_workspace(p, scale, dtype, need);
    unsigned char *base = static_cast<unsigned char *>(ws);
    T *lat = reinterpret_cast<T *>(base);
    T *parts = reinterpret_cast<T *>(base + w.lattices);
    const int64_t n_x = p.N * p.C * p.H * p.W;
    const int branches = scale * scale;
    hipError_t err = ddf::up_split_lattices<T>((const T *)go, lat, p.N * p.C, p.H, p.W, scale, stream);
    if (err != hipSuccess) return fail_hip(err, "ddf_hip_up_backward split launch");

    // All branches as one batch of scale*scale * N samples that share the features:
    // a handful of launches that fill the machine, instead of three or four small
    // ones per branch.
    if constexpr (sizeof(T) != 8) if (w.batched) {
        unsigned char *q = base + w.lattices + w.dx_parts;
        T *cf_all = reinterpret_cast<T *>(q); q += w.cf_all;
        T *sf_all = reinterpret_cast<T *>(q); q += w.sf_all;
        T *dcf_all = w.dcf_all ? reinterpret_cast<T *>(q) : nullptr; q += w.dcf_all;
        T *dsf_all = w.dsf_all ? reinterpret_cast<T *>(q) : nullptr; q += w.dsf_all;
        const int64_t n_cf = p.N * p.C * p.kk, n_sf = p.N * p.kk * p.H * p.W;
        err = ddf::up_gather_filters<T>(cfs, sfs, cf_all, sf_all, n_cf, n_sf, branches, stream);
        if (err != hipSuccess) return fail_hip(err, "ddf_hip_up_backward gather launch");
        const ddf::Problem pb = ddf::make_problem(p.N * branches, p.C, p.H, p.W, p.k, p.d, 1,
                                                  p.mul ? DDF_MUL : DDF_ADD);
        err = ddf::rows_backward_shared_features<T>(
            pb, (int)p.N, lat, (const T *)x, cf_all, sf_all, (need & DDF_NEED_DX) ? parts : nullptr,
            dcf_all, dsf_all, w.batch_ws ? q : nullptr, need, stream);
        if (err == hipSuccess) {
            err = ddf::up_finish<T>((need & DDF_NEED_DX) ? parts : nullptr, (T *)dx, n_x, branches,
                                    dcf_all, dsf_all, dcfs, dsfs, n_cf, n_sf, stream);
            if (err != hipSuccess) return fail_hip(err, "ddf_hip_up_backward finish launch");
            return DDF_OK;
        }
        // (e.g. features not 16-byte aligned: nothing was launched, take the other route)
        if (err != hipErrorNotSupported) return fail_hip(err, "ddf_hip_up_backward batch launch");
    }

    void *branch_ws = w.branch ? base + w.lattices + w.dx_parts : nullptr;
    for (int b = 0; b < branches; ++b) {
        unsigned bneed = need & DDF_NEED_DX;
        if ((need & DDF_NEED_DCF) && dcfs && dcfs[b]) bneed |= DDF_NEED_DCF;
        if ((need & DDF_NEED_DSF) && dsfs && dsfs[b]) bneed |= DDF_NEED_DSF;
        if (bneed == 0) continue;
        const int rc = backward_typed<T>(p, lat + b * n_x, x, cfs[b], sfs[b],
                                         (need & DDF_NEED_DX) ? parts + b * n_x : nullptr,
                                         dcfs ? dcfs[b] : nullptr, dsfs ? dsfs[b] : nullptr,
                                         branch_ws, w.branch, dtype, bneed, DDF_VARIANT_AUTO,
                                         stream);
        if (rc != DDF_OK) return rc;
    }
    if (need & DDF_NEED_DX) {
        err = ddf::up_sum_parts<T>(parts, (T *)dx, n_x, branches, stream);
        if (err != hipSuccess) return fail_hip(err, "ddf_hip_up_backward sum launch");
    }
    return DDF_OK;
}

}  // namespace

extern "C" {

int ddf_hip_version(void) { return 100; }

const char *ddf_hip_status_string(int status) {
    switch (status) {
        case DDF_OK: return "ok";
        case DDF_ERR_BAD_ARG: return "bad argument";
        case DDF_ERR_UNSUPPORTED: return "unsupported configuration";
        case DDF_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case DDF_ERR_HIP: return "hip runtime error";
        default: return "unknown status";
    }
}

const char *ddf_hip_last_error(void) { return g_last_error; }

int ddf_hip_describe(int64_t N, int64_t C, int64_t H, int64_t W, int kernel_size, int dilation,
                     int stride, int combine, int dtype, unsigned need_mask, int variant,
                     char *buffer, int buffer_len) {
    if (!buffer || buffer_len <= 0) return fail(DDF_ERR_BAD_ARG, "no buffer for the description");
    buffer[0] = 0;
    int rc = check_problem(N, C, H, W, kernel_size, dilation, stride, combine, dtype, variant);
    if (rc != DDF_OK) return rc;
    const ddf::Problem p = ddf::make_problem(N, C, H, W, kernel_size, dilation, stride, combine);
    if (N * C * p.Ho * p.Wo == 0) { snprintf(buffer, buffer_len, "nothing"); return DDF_OK; }
    const unsigned need = need_mask & DDF_NEED_ALL;
    const bool norm = (need_mask & DDF_DESCRIBE_SPATIAL_NORM) && (need & DDF_NEED_DSF);
    if (need == 0) {
        if (variant == DDF_VARIANT_GENERIC || !ddf::tiled_forward_supported(p, dtype))
            snprintf(buffer, buffer_len, "generic_forward");
        else
            ddf::describe_forward(p, dtype, buffer, buffer_len);
    } else {
        if (variant == DDF_VARIANT_GENERIC || !ddf::tiled_backward_supported(p, dtype))
            snprintf(buffer, buffer_len, norm ? "generic_backward + k_filter_norm_backward" : "generic_backward");
        else
            ddf::describe_backward(p, dtype, need | (norm ? DDF_DESCRIBE_SPATIAL_NORM : 0u), buffer,
                                   buffer_len);
    }
    return DDF_OK;
}

int ddf_hip_forward(const void *features, const void *channel_filter,
                    const void *spatial_filter, void *output, int64_t N, int64_t C,
                    int64_t H, int64_t W, int kernel_size, int dilation, int stride,
                    int combine, int dtype, int variant, void *stream) {
    int rc = check_problem(N, C, H, W, kernel_size, dilation, stride, combine, dtype, variant);
    if (rc != DDF_OK) return rc;
    const ddf::Problem p = ddf::make_problem(N, C, H, W, kernel_size, dilation, stride, combine);
    if (N * C * p.Ho * p.Wo == 0) return DDF_OK;  // nothing to write
    if (!features || !channel_filter || !spatial_filter || !output)
        return fail(DDF_ERR_BAD_ARG, "null tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case DDF_F16:
            return forward_typed<__half>(p, features, channel_filter, spatial_filter, output,
                                         dtype, variant, st);
        case DDF_F32:
            return forward_typed<float>(p, features, channel_filter, spatial_filter, output,
                                        dtype, variant, st);
        default:
            return forward_typed<double>(p, features, channel_filter, spatial_filter, output,
                                         dtype, variant, st);
    }
}

size_t ddf_hip_backward_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W,
                                        int kernel_size, int dilation, int stride,
                                        int combine, int dtype, unsigned need_mask,
                                        int variant) {
    if (check_problem(N, C, H, W, kernel_size, dilation, stride, combine, dtype, variant) !=
        DDF_OK)
        return 0;
    if (variant == DDF_VARIANT_GENERIC) return 0;
    const ddf::Problem p = ddf::make_problem(N, C, H, W, kernel_size, dilation, stride, combine);
    if (!ddf::tiled_backward_supported(p, dtype)) return 0;
    return ddf::tiled_backward_workspace(p, dtype, need_mask & DDF_NEED_ALL);
}

int ddf_hip_backward(const void *grad_output, const void *features,
                     const void *channel_filter, const void *spatial_filter,
                     void *grad_features, void *grad_channel_filter,
                     void *grad_spatial_filter, void *workspace, size_t workspace_bytes,
                     int64_t N, int64_t C, int64_t H, int64_t W, int kernel_size,
                     int dilation, int stride, int combine, int dtype, unsigned need_mask,
                     int variant, void *stream) {
    int rc = check_problem(N, C, H, W, kernel_size, dilation, stride, combine, dtype, variant);
    if (rc != DDF_OK) return rc;
    const unsigned need = need_mask & DDF_NEED_ALL;
    if (need == 0) return DDF_OK;
    const ddf::Problem p = ddf::make_problem(N, C, H, W, kernel_size, dilation, stride, combine);
    if (N == 0) return DDF_OK;  // every gradient is empty
    // A pointer is only dereferenced when its tensor has elements.
    const int64_t n_x = N * C * H * W, n_o = N * C * p.Ho * p.Wo;
    const int64_t n_cf = N * C * p.kk, n_sf = N * p.kk * p.Ho * p.Wo;
    if ((!grad_output && n_o) || (!features && n_x) || (!channel_filter && n_cf) ||
        (!spatial_filter && n_sf))
        return fail(DDF_ERR_BAD_ARG, "null input tensor pointer");
    if (((need & DDF_NEED_DX) && !grad_features && n_x) ||
        ((need & DDF_NEED_DCF) && !grad_channel_filter && n_cf) ||
        ((need & DDF_NEED_DSF) && !grad_spatial_filter && n_sf))
        return fail(DDF_ERR_BAD_ARG, "null pointer for a requested gradient");
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case DDF_F16:
            return backward_typed<__half>(p, grad_output, features, channel_filter,
                                          spatial_filter, grad_features, grad_channel_filter,
                                          grad_spatial_filter, workspace, workspace_bytes,
                                          dtype, need, variant, st);
        case DDF_F32:
            return backward_typed<float>(p, grad_output, features, channel_filter,
                                         spatial_filter, grad_features, grad_channel_filter,
                                         grad_spatial_filter, workspace, workspace_bytes,
                                         dtype, need, variant, st);
        default:
            return backward_typed<double>(p, grad_output, features, channel_filter,
                                          spatial_filter, grad_features, grad_channel_filter,
                                          grad_spatial_filter, workspace, workspace_bytes,
                                          dtype, need, variant, st);
    }
}

size_t ddf_hip_backward_spatial_norm_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W,
                                                     int kernel_size, int dilation, int stride,
                                                     int combine, int dtype, unsigned need_mask,
                                                     int variant) {
    if (check_problem(N, C, H, W, kernel_size, dilation, stride, combine, dtype, variant) != DDF_OK)
        return 0;
    const ddf::Problem p = ddf::make_problem(N, C, H, W, kernel_size, dilation, stride, combine);
    const size_t esz = dtype == DDF_F16 ? 2 : dtype == DDF_F32 ? 4 : 8;
    const size_t tmp = (need_mask & DDF_NEED_DSF) ? align256((size_t)(N * p.kk * p.Ho * p.Wo) * esz) : 0;
    return tmp + ddf_hip_backward_workspace_bytes(N, C, H, W, kernel_size, dilation, stride, combine,
                                                  dtype, need_mask, variant);
}

int ddf_hip_backward_spatial_norm(const void *grad_output, const void *features,
                                  const void *channel_filter, const void *spatial_filter,
                                  const void *raw_spatial_filter, void *grad_features,
                                  void *grad_channel_filter, void *grad_raw_spatial_filter,
                                  void *gain_terms, void *workspace, size_t workspace_bytes,
                                  int64_t N, int64_t C, int64_t H, int64_t W, int kernel_size,
                                  int dilation, int stride, int combine, int dtype,
                                  unsigned need_mask, int groups, double gain, const void *gain_vec,
                                  int variant, void *stream) {
    int rc = check_problem(N, C, H, W, kernel_size, dilation, stride, combine, dtype, variant);
    if (rc != DDF_OK) return rc;
    const unsigned need = need_mask & DDF_NEED_ALL;
    if (need == 0 || N == 0) return DDF_OK;
    if (groups < 1 || N % groups != 0)
        return fail(DDF_ERR_BAD_ARG, "groups must be >= 1 and divide N (got %d, N=%lld)", groups,
                    (long long)N);
    const ddf::Problem p = ddf::make_problem(N, C, H, W, kernel_size, dilation, stride, combine);
    const int64_t n_x = N * C * H * W, n_o = N * C * p.Ho * p.Wo;
    const int64_t n_cf = N * C * p.kk, n_sf = N * p.kk * p.Ho * p.Wo;
    if ((!grad_output && n_o) || (!features && n_x) || (!channel_filter && n_cf) ||
        (!spatial_filter && n_sf))
        return fail(DDF_ERR_BAD_ARG, "null input tensor pointer");
    if ((need & DDF_NEED_DSF) && n_sf && (!raw_spatial_filter || !grad_raw_spatial_filter))
        return fail(DDF_ERR_BAD_ARG, "null pointer for the raw spatial filter or its gradient");
    if (((need & DDF_NEED_DX) && !grad_features && n_x) ||
        ((need & DDF_NEED_DCF) && !grad_channel_filter && n_cf))
        return fail(DDF_ERR_BAD_ARG, "null pointer for a requested gradient");
    hipStream_t st = (hipStream_t)stream;
#define DDF_NORM_CASE(T_)                                                                          \
    return backward_norm_typed<T_>(p, grad_output, features, channel_filter, spatial_filter,       \
                                   raw_spatial_filter, grad_features, grad_channel_filter,         \
                                   grad_raw_spatial_filter, gain_terms, workspace, workspace_bytes, \
                                   dtype, need, groups, gain, gain_vec, variant, st)
    switch (dtype) {
        case DDF_F16: DDF_NORM_CASE(__half);
        case DDF_F32: DDF_NORM_CASE(float);
        default: DDF_NORM_CASE(double);
    }
#undef DDF_NORM_CASE
}

int ddf_hip_backward_static(const void *grad_output, const void *features,
                            const void *channel_filter, const void *spatial_filter,
                            void *grad_features, void *grad_channel_filter,
                            void *grad_spatial_filter, int64_t N, int64_t C, int64_t H, int64_t W,
                            int kernel_size, int dilation, int stride, int combine, int dtype,
                            unsigned need_mask, int variant, void *stream) {
    // the device's copy of the scratch array (first call on a device: looked up, no allocation)
    void *ws = nullptr;
    int rc = scratch_of_current_device(&ws);
    if (rc != DDF_OK) return rc;
    rc = check_problem(N, C, H, W, kernel_size, dilation, stride, combine, dtype, variant);
    if (rc != DDF_OK) return rc;
    const size_t want = ddf_hip_backward_workspace_bytes(N, C, H, W, kernel_size, dilation, stride,
                                                         combine, dtype, need_mask, variant);
    if (want > (size_t)DDF_HIP_STATIC_SCRATCH_BYTES)
        return fail(DDF_ERR_WORKSPACE,
                    "this problem needs %zu bytes of scratch; ddf_hip_backward_static holds %zu "
                    "(use ddf_hip_backward with a workspace of your own)",
                    want, (size_t)DDF_HIP_STATIC_SCRATCH_BYTES);
    // Every partial sum the kernels read back from the scratch they have written in
    // the same call, so what an earlier call left there needs no clearing.
    return ddf_hip_backward(grad_output, features, channel_filter, spatial_filter, grad_features,
                            grad_channel_filter, grad_spatial_filter, ws,
                            (size_t)DDF_HIP_STATIC_SCRATCH_BYTES, N, C, H, W, kernel_size, dilation,
                            stride, combine, dtype, need_mask, variant, stream);
}

int ddf_hip_filter_norm(const void *x, void *y, int64_t outer, int64_t groups, int taps,
                        int64_t inner, double gain, const void *gain_vec, const void *offset_vec,
                        int dtype, void *stream) {
    if (outer < 0 || groups < 0 || taps < 0 || inner < 0)
        return fail(DDF_ERR_BAD_ARG, "negative tensor size");
    if (dtype != DDF_F16 && dtype != DDF_F32 && dtype != DDF_F64)
        return fail(DDF_ERR_BAD_ARG, "unknown dtype %d", dtype);
    if (outer * groups * taps * inner == 0) return DDF_OK;
    if (!x || !y) return fail(DDF_ERR_BAD_ARG, "null tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    hipError_t err;
    switch (dtype) {
        case DDF_F16:
            err = ddf::filter_norm<__half>((const __half *)x, (__half *)y, outer, groups, taps,
                                           inner, gain, (const __half *)gain_vec,
                                           (const __half *)offset_vec, st);
            break;
        case DDF_F32:
            err = ddf::filter_norm<float>((const float *)x, (float *)y, outer, groups, taps, inner,
                                          gain, (const float *)gain_vec,
                                          (const float *)offset_vec, st);
            break;
        default:
            err = ddf::filter_norm<double>((const double *)x, (double *)y, outer, groups, taps,
                                           inner, gain, (const double *)gain_vec,
                                           (const double *)offset_vec, st);
    }
    return err == hipSuccess ? DDF_OK : fail_hip(err, "ddf_hip_filter_norm launch");
}

int ddf_hip_filter_norm_backward(const void *grad_y, const void *x, void *grad_x,
                                 void *gain_terms, int64_t outer, int64_t groups, int taps,
                                 int64_t inner, double gain, const void *gain_vec, int dtype,
                                 void *stream) {
    if (outer < 0 || groups < 0 || taps < 0 || inner < 0)
        return fail(DDF_ERR_BAD_ARG, "negative tensor size");
    if (dtype != DDF_F16 && dtype != DDF_F32 && dtype != DDF_F64)
        return fail(DDF_ERR_BAD_ARG, "unknown dtype %d", dtype);
    if (outer * groups * taps * inner == 0) return DDF_OK;
    if (!grad_y || !x || !grad_x) return fail(DDF_ERR_BAD_ARG, "null tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    hipError_t err;
    switch (dtype) {
        case DDF_F16:
            err = ddf::filter_norm_backward<__half>(
                (const __half *)grad_y, (const __half *)x, (__half *)grad_x, (__half *)gain_terms,
                outer, groups, taps, inner, gain, (const __half *)gain_vec, st);
            break;
        case DDF_F32:
            err = ddf::filter_norm_backward<float>(
                (const float *)grad_y, (const float *)x, (float *)grad_x, (float *)gain_terms,
                outer, groups, taps, inner, gain, (const float *)gain_vec, st);
            break;
        default:
            err = ddf::filter_norm_backward<double>(
                (const double *)grad_y, (const double *)x, (double *)grad_x, (double *)gain_terms,
                outer, groups, taps, inner, gain, (const double *)gain_vec, st);
    }
    return err == hipSuccess ? DDF_OK : fail_hip(err, "ddf_hip_filter_norm_backward launch");
}

namespace {
int spatial_branch_impl(const void *features, const void *weight, const void *bias,
                        void *spatial_filter, float *pool_parts, int64_t pool_capacity, int *n_parts,
                        int64_t N, int64_t C, int64_t H, int64_t W,
                        int head, int kernel_size, int stride, double gain,
                        const void *gain_vec, const void *offset_vec, int dtype, void *stream) {
    if (N < 0 || C < 0 || H < 0 || W < 0 || head < 0) return fail(DDF_ERR_BAD_ARG, "negative tensor size");
    if (stride < 1) return fail(DDF_ERR_BAD_ARG, "stride must be >= 1 (got %d)", stride);
    if (dtype != DDF_F16 && dtype != DDF_F32)
        return fail(DDF_ERR_UNSUPPORTED, "the branch kernels cover fp16 and fp32 (dtype %d)", dtype);
    if (!ddf::branch_kernel_size_built(kernel_size))
        return fail(DDF_ERR_UNSUPPORTED, "the branch kernels cover kernel sizes 3 and 5 (got %d)", kernel_size);
    if (N * C * (H / stride) * (W / stride) * head == 0) return DDF_OK;
    if (!features || !weight || !spatial_filter) return fail(DDF_ERR_BAD_ARG, "null tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    const hipError_t err =
        dtype == DDF_F16
            ? ddf::spatial_branch<__half>((const __half *)features, (const __half *)weight,
                                          (const __half *)bias, (__half *)spatial_filter, N, C, H, W,
                                          head, kernel_size, stride, gain, (const __half *)gain_vec,
                                          (const __half *)offset_vec, st, pool_parts, pool_capacity, n_parts)
            : ddf::spatial_branch<float>((const float *)features, (const float *)weight,
                                         (const float *)bias, (float *)spatial_filter, N, C, H, W, head,
                                         kernel_size, stride, gain, (const float *)gain_vec,
                                         (const float *)offset_vec, st, pool_parts, pool_capacity, n_parts);
    if (err == hipErrorNotSupported) return fail(DDF_ERR_UNSUPPORTED, "spatial branch: sizes not covered");
    if (err == hipErrorInvalidValue && pool_parts)
        return fail(DDF_ERR_WORKSPACE, "spatial branch: the buffer of partial sums is too small");
    return err == hipSuccess ? DDF_OK : fail_hip(err, "ddf_hip_spatial_branch launch");
}
}  // namespace

int ddf_hip_spatial_branch(const void *features, const void *weight, const void *bias,
                           void *spatial_filter, int64_t N, int64_t C, int64_t H, int64_t W,
                           int head, int kernel_size, int stride, double gain,
                           const void *gain_vec, const void *offset_vec, int dtype, void *stream) {
    return spatial_branch_impl(features, weight, bias, spatial_filter, nullptr, 0, nullptr, N, C, H, W, head,
                               kernel_size, stride, gain, gain_vec, offset_vec, dtype, stream);
}

int ddf_hip_spatial_branch_pool(const void *features, const void *weight, const void *bias,
                                void *spatial_filter, float *pool_parts, int64_t pool_capacity,
                                int *n_parts, int64_t N, int64_t C, int64_t H, int64_t W, int head,
                                int kernel_size, int stride, double gain, const void *gain_vec,
                                const void *offset_vec, int dtype, void *stream) {
    if (!pool_parts || !n_parts || pool_capacity < 0)
        return fail(DDF_ERR_BAD_ARG, "ddf_hip_spatial_branch_pool: null buffer of partial sums");
    *n_parts = 0;
    if (N > 0 && C > 0 && head > 0 && stride >= 1 && (H / stride) * (W / stride) == 0)
        return fail(DDF_ERR_UNSUPPORTED, "spatial branch: nothing to pool into");
    return spatial_branch_impl(features, weight, bias, spatial_filter, pool_parts, pool_capacity, n_parts, N, C,
                               H, W, head, kernel_size, stride, gain, gain_vec, offset_vec, dtype, stream);
}

namespace {
int channel_branch_impl(const void *pooled, const float *parts, int n_parts, double scale,
                        const void *weight1, const void *bias1,
                        const void *weight2, const void *bias2, void *channel_filter, int64_t N,
                        int64_t C, int64_t mid, int kernel_size, double gain,
                        const void *gain_vec, const void *offset_vec, int dtype, void *stream) {
    if (N < 0 || C < 0 || mid < 0) return fail(DDF_ERR_BAD_ARG, "negative tensor size");
    if (dtype != DDF_F16 && dtype != DDF_F32)
        return fail(DDF_ERR_UNSUPPORTED, "the branch kernels cover fp16 and fp32 (dtype %d)", dtype);
    if (!ddf::branch_kernel_size_built(kernel_size))
        return fail(DDF_ERR_UNSUPPORTED, "the branch kernels cover kernel sizes 3 and 5 (got %d)", kernel_size);
    if (N * C == 0) return DDF_OK;
    if ((!pooled && !parts) || !weight1 || !weight2 || !channel_filter) return fail(DDF_ERR_BAD_ARG, "null tensor pointer");
    if (parts && n_parts < 1) return fail(DDF_ERR_BAD_ARG, "n_parts must be >= 1 (got %d)", n_parts);
    hipStream_t st = (hipStream_t)stream;
    const hipError_t err =
        dtype == DDF_F16
            ? ddf::channel_branch<__half>((const __half *)pooled, (const __half *)weight1,
                                          (const __half *)bias1, (const __half *)weight2,
                                          (const __half *)bias2, (__half *)channel_filter, N, C, mid,
                                          kernel_size, gain, (const __half *)gain_vec,
                                          (const __half *)offset_vec, st, parts, n_parts, scale)
            : ddf::channel_branch<float>((const float *)pooled, (const float *)weight1,
                                         (const float *)bias1, (const float *)weight2,
                                         (const float *)bias2, (float *)channel_filter, N, C, mid,
                                         kernel_size, gain, (const float *)gain_vec,
                                         (const float *)offset_vec, st, parts, n_parts, scale);
    if (err == hipErrorNotSupported) return fail(DDF_ERR_UNSUPPORTED, "channel branch: sizes not covered");
    return err == hipSuccess ? DDF_OK : fail_hip(err, "ddf_hip_channel_branch launch");
}
}  // namespace

int ddf_hip_channel_branch(const void *pooled, const void *weight1, const void *bias1,
                           const void *weight2, const void *bias2, void *channel_filter, int64_t N,
                           int64_t C, int64_t mid, int kernel_size, double gain,
                           const void *gain_vec, const void *offset_vec, int dtype, void *stream) {
    return channel_branch_impl(pooled, nullptr, 0, 1.0, weight1, bias1, weight2, bias2, channel_filter, N, C,
                               mid, kernel_size, gain, gain_vec, offset_vec, dtype, stream);
}

int ddf_hip_channel_branch_parts(const float *pool_parts, int n_parts, double scale,
                                 const void *weight1, const void *bias1, const void *weight2,
                                 const void *bias2, void *channel_filter, int64_t N, int64_t C,
                                 int64_t mid, int kernel_size, double gain, const void *gain_vec,
                                 const void *offset_vec, int dtype, void *stream) {
    if (!pool_parts) return fail(DDF_ERR_BAD_ARG, "ddf_hip_channel_branch_parts: null partial sums");
    return channel_branch_impl(nullptr, pool_parts, n_parts, scale, weight1, bias1, weight2, bias2,
                               channel_filter, N, C, mid, kernel_size, gain, gain_vec, offset_vec, dtype, stream);
}

int ddf_hip_up_forward(const void *features, const void *const *channel_filters,
                       const void *const *spatial_filters, void *output, int64_t N, int64_t C,
                       int64_t H, int64_t W, int kernel_size, int dilation, int scale,
                       int combine, int dtype, void *stream) {
    int rc = check_problem(N, C, H, W, kernel_size, dilation, 1, combine, dtype, DDF_VARIANT_AUTO);
    if (rc != DDF_OK) return rc;
    if (scale < 2 || scale * scale > DDF_UP_MAX_BRANCHES)
        return fail(DDF_ERR_BAD_ARG, "scale must be 2..4 (got %d)", scale);
    if (!ddf::up_forward_supported(H, W, kernel_size, dilation, scale))
        return fail(DDF_ERR_UNSUPPORTED,
                    "fused up-sampling forward does not cover k=%d scale=%d H=%lld W=%lld",
                    kernel_size, scale, (long long)H, (long long)W);
    if (N * C * H * W == 0) return DDF_OK;
    if (!features || !output || !channel_filters || !spatial_filters)
        return fail(DDF_ERR_BAD_ARG, "null tensor pointer");
    for (int b = 0; b < scale * scale; ++b)
        if (!channel_filters[b] || !spatial_filters[b])
            return fail(DDF_ERR_BAD_ARG, "null filter pointer for branch %d", b);
    hipStream_t st = (hipStream_t)stream;
    const bool mul = combine == DDF_MUL;
    hipError_t err;
    switch (dtype) {
        case DDF_F16:
            err = ddf::up_forward<__half>(N, C, H, W, kernel_size, dilation, scale, mul,
                                          (const __half *)features, channel_filters,
                                          spatial_filters, (__half *)output, st);
            break;
        case DDF_F32:
            err = ddf::up_forward<float>(N, C, H, W, kernel_size, dilation, scale, mul,
                                         (const float *)features, channel_filters,
                                         spatial_filters, (float *)output, st);
            break;
        default:
            err = ddf::up_forward<double>(N, C, H, W, kernel_size, dilation, scale, mul,
                                          (const double *)features, channel_filters,
                                          spatial_filters, (double *)output, st);
    }
    return err == hipSuccess ? DDF_OK : fail_hip(err, "ddf_hip_up_forward launch");
}

size_t ddf_hip_up_backward_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W,
                                           int kernel_size, int dilation, int scale, int combine,
                                           int dtype, unsigned need_mask) {
    if (check_problem(N, C, H, W, kernel_size, dilation, 1, combine, dtype, DDF_VARIANT_AUTO) !=
            DDF_OK || scale < 2 || scale * scale > DDF_UP_MAX_BRANCHES)
        return 0;
    const ddf::Problem p = ddf::make_problem(N, C, H, W, kernel_size, dilation, 1, combine);
    return up_workspace(p, scale, dtype, need_mask & DDF_NEED_ALL).total;
}

int ddf_hip_up_backward(const void *grad_output, const void *features,
                        const void *const *channel_filters, const void *const *spatial_filters,
                        void *grad_features, void *const *grad_channel_filters,
                        void *const *grad_spatial_filters, void *workspace, size_t workspace_bytes,
                        int64_t N, int64_t C, int64_t H, int64_t W, int kernel_size, int dilation,
                        int scale, int combine, int dtype, unsigned need_mask, void *stream) {
    int rc = check_problem(N, C, H, W, kernel_size, dilation, 1, combine, dtype, DDF_VARIANT_AUTO);
    if (rc != DDF_OK) return rc;
    if (scale < 2 || scale * scale > DDF_UP_MAX_BRANCHES)
        return fail(DDF_ERR_BAD_ARG, "scale must be 2..4 (got %d)", scale);
    const unsigned need = need_mask & DDF_NEED_ALL;
    if (need == 0 || N * C * H * W == 0) return DDF_OK;
    if (!grad_output || !features || !channel_filters || !spatial_filters)
        return fail(DDF_ERR_BAD_ARG, "null input tensor pointer");
    for (int b = 0; b < scale * scale; ++b)
        if (!channel_filters[b] || !spatial_filters[b])
            return fail(DDF_ERR_BAD_ARG, "null filter pointer for branch %d", b);
    if ((need & DDF_NEED_DX) && !grad_features)
        return fail(DDF_ERR_BAD_ARG, "null pointer for a requested gradient");
    const ddf::Problem p = ddf::make_problem(N, C, H, W, kernel_size, dilation, 1, combine);
    const size_t want = up_workspace(p, scale, dtype, need).total;
    if (!workspace || workspace_bytes < want)
        return fail(DDF_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", want,
                    workspace ? workspace_bytes : (size_t)0);
    if (((uintptr_t)workspace & 255u) != 0)
        return fail(DDF_ERR_WORKSPACE, "workspace must be 256-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case DDF_F16:
            return up_backward_typed<__half>(p, scale, grad_output, features, channel_filters,
                                             spatial_filters, grad_features, grad_channel_filters,
                                             grad_spatial_filters, workspace, dtype, need, st);
        case DDF_F32:
            return up_backward_typed<float>(p, scale, grad_output, features, channel_filters,
                                            spatial_filters, grad_features, grad_channel_filters,
                                            grad_spatial_filters, workspace, dtype, need, st);
        default:
            return up_backward_typed<double>(p, scale, grad_output, features, channel_filters,
                                             spatial_filters, grad_features, grad_channel_filters,
                                             grad_spatial_filters, workspace, dtype, need, st);
    }
}

}  // extern "C"
