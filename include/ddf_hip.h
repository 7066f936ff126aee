/*
 * ddf_hip.h - C ABI of the Decoupled Dynamic Filter (DDF) operator for gfx950.
 *
 * The library (libddf_hip.so) holds hand-written HIP kernels for the DDF
 * forward pass and its three gradients.  Every entry point takes plain device
 * pointers, sizes and enums; nothing here depends on torch.  All tensors are
 * dense NCHW ("contiguous") and live on the device that is current when the
 * call is made.  Calls are asynchronous: they enqueue kernels on `stream`
 * (a hipStream_t passed as void*, NULL = the default stream) and return
 * without synchronising.  The caller owns every buffer and the entry points
 * are re-entrant; the only state the library keeps is the per-device scratch
 * array of ddf_hip_backward_static (calls of that one entry point share it)
 * and a thread-local text of the last error.
 *
 * Operator (r = (k-1)/2, Ho = H / s, Wo = W / s with floor division,
 * t = i*k + j, comb(a,b) = a*b for DDF_MUL and a+b for DDF_ADD; a term whose
 * feature index falls outside the image is zero):
 *
 *   out[n,c,y,x] = sum_{i,j} X[n,c, y*s+(i-r)*d, x*s+(j-r)*d]
 *                            * comb(CF[n,c,i,j], SF[n,t,y,x])
 *
 * Shapes: X (N,C,H,W); CF (N,C,k,k); SF (N,k*k,Ho,Wo); out (N,C,Ho,Wo).
 *
 * Reference interface replaced (theFoxofSky/ddfnet):
 *   ddf/src/ddf_mul_ext.cpp:21-34, :36-55   forward / backward, 'mul'
 *   ddf/src/ddf_add_ext.cpp:21-34, :36-55   forward / backward, 'add'
 *   ddf/src/ddf_mul_faster_ext.cpp:13-26    tiled forward, 'mul'
 *   ddf/src/ddf_add_faster_ext.cpp:13-26    tiled forward, 'add'
 * The four pybind modules collapse into the two calls below; `combine`
 * selects mul/add and `variant` selects the generic or the tiled kernels.
 */
#ifndef DDF_HIP_H
#define DDF_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element type of every tensor of one call (no mixed types).  DDF_F16 reads
 * and writes IEEE half and accumulates in fp32. */
typedef enum { DDF_F16 = 0, DDF_F32 = 1, DDF_F64 = 2 } ddf_dtype_t;

/* How the channel filter and the spatial filter are combined per tap. */
typedef enum { DDF_MUL = 0, DDF_ADD = 1 } ddf_combine_t;

/* Kernel family.  DDF_VARIANT_AUTO picks the tiled kernels when the shape is
 * supported by them and the generic kernels otherwise.  DDF_VARIANT_GENERIC
 * corresponds to the reference's version 'o', DDF_VARIANT_TILED to 'f'
 * (ddf/ddf.py:77-84); asking for the tiled family on a shape it does not
 * cover returns DDF_ERR_UNSUPPORTED. */
typedef enum {
    DDF_VARIANT_AUTO = 0,
    DDF_VARIANT_GENERIC = 1,
    DDF_VARIANT_TILED = 2
} ddf_variant_t;

/* Return codes.  0 is success; hip runtime failures are reported as
 * DDF_ERR_HIP and the text is available from ddf_hip_last_error(). */
typedef enum {
    DDF_OK = 0,
    DDF_ERR_BAD_ARG = 1,      /* null pointer, non-positive size, even k ... */
    DDF_ERR_UNSUPPORTED = 2,  /* valid request no kernel here covers          */
    DDF_ERR_WORKSPACE = 3,    /* workspace missing or too small               */
    DDF_ERR_HIP = 4           /* hip runtime error at launch                  */
} ddf_status_t;

/* Bits of `need_mask` for ddf_hip_backward. */
#define DDF_NEED_DX  1u
#define DDF_NEED_DCF 2u
#define DDF_NEED_DSF 4u
#define DDF_NEED_ALL 7u
/* ddf_hip_describe only: name the launches of ddf_hip_backward_spatial_norm */
#define DDF_DESCRIBE_SPATIAL_NORM 8u

/* Library version: major*10000 + minor*100 + patch. */
int ddf_hip_version(void);

/* Text for a status code (static storage). */
const char *ddf_hip_status_string(int status);

/* Text of the last failure on the calling thread (thread-local storage). */
const char *ddf_hip_last_error(void);

/*
 * Names of the kernels a call with these arguments launches, as text in
 * `buffer` (diagnostics for benchmarks and profiles; no counterpart in the
 * reference).  need_mask 0 describes ddf_hip_forward, anything else
 * ddf_hip_backward with that mask (with DDF_DESCRIBE_SPATIAL_NORM added:
 * ddf_hip_backward_spatial_norm).  Pointer alignment, which can send a call
 * to the scalar-access kernels, is assumed to be 16 bytes.
 */
int ddf_hip_describe(int64_t N, int64_t C, int64_t H, int64_t W,
                     int kernel_size, int dilation, int stride, int combine,
                     int dtype, unsigned need_mask, int variant, char *buffer,
                     int buffer_len);

/*
 * Forward pass.  Replaces `forward(features, channel_filter, spatial_filter,
 * kernel_size, dilation, stride, output)` of ddf_{mul,add}{,_faster}_ext
 * (ddf/src/ddf_mul_ext.cpp:21-34, ddf/src/ddf_mul_faster_ext.cpp:13-26).
 * `output` is written in full, so it need not be zeroed.
 */
int ddf_hip_forward(const void *features, const void *channel_filter,
                    const void *spatial_filter, void *output,
                    int64_t N, int64_t C, int64_t H, int64_t W,
                    int kernel_size, int dilation, int stride,
                    int combine, int dtype, int variant, void *stream);

/*
 * Bytes of device scratch ddf_hip_backward needs for this problem (0 when
 * none).  Same arguments as the backward call.
 */
size_t ddf_hip_backward_workspace_bytes(int64_t N, int64_t C, int64_t H,
                                        int64_t W, int kernel_size,
                                        int dilation, int stride, int combine,
                                        int dtype, unsigned need_mask,
                                        int variant);

/*
 * Backward pass: gradients with respect to features, channel_filter and
 * spatial_filter.  Replaces `backward(top_grad, features, channel_filter,
 * spatial_filter, kernel_size, dilation, stride, rtop_grad, rbottom_grad,
 * rspatial_filter_grad, bottom_grad, channel_filter_grad,
 * spatial_filter_grad)` of ddf_{mul,add}_ext
 * (ddf/src/ddf_mul_ext.cpp:36-55).  The three NHWC scratch tensors of the
 * reference have no counterpart: gradients are produced directly in NCHW.
 * A gradient whose bit is clear in `need_mask` is not computed and its pointer
 * may be NULL.  Requested gradients are written in full (no zeroing needed).
 * `workspace` must hold at least ddf_hip_backward_workspace_bytes(...) bytes,
 * 256-byte aligned; it may be NULL when that size is 0.
 */
int ddf_hip_backward(const void *grad_output, const void *features,
                     const void *channel_filter, const void *spatial_filter,
                     void *grad_features, void *grad_channel_filter,
                     void *grad_spatial_filter, void *workspace,
                     size_t workspace_bytes, int64_t N, int64_t C, int64_t H,
                     int64_t W, int kernel_size, int dilation, int stride,
                     int combine, int dtype, unsigned need_mask, int variant,
                     void *stream);

/*
 * ddf_hip_backward for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It
 * has no counterpart in the reference (whose backward takes caller-allocated
 * scratch tensors, ddf/src/ddf_mul_ext.cpp:36-42).  Same arguments as
 * ddf_hip_backward without the workspace: the partial sums go to a buffer of
 * DDF_HIP_STATIC_SCRATCH_BYTES bytes that is part of the library's device
 * image (every GPU the library runs on holds it until the process ends), and
 * the call allocates and frees nothing.  A problem whose
 * ddf_hip_backward_workspace_bytes() exceeds that size is rejected with
 * DDF_ERR_WORKSPACE.  All calls on one GPU share the buffer: calls that
 * overlap in time on the same GPU (different streams, different threads) race
 * and must be serialised by the caller.  The first call on a device looks the
 * buffer's address up (no allocation); make it outside a graph capture.
 */
#define DDF_HIP_STATIC_SCRATCH_BYTES (16u * 1024u * 1024u)
int ddf_hip_backward_static(const void *grad_output, const void *features,
                            const void *channel_filter,
                            const void *spatial_filter, void *grad_features,
                            void *grad_channel_filter,
                            void *grad_spatial_filter, int64_t N, int64_t C,
                            int64_t H, int64_t W, int kernel_size,
                            int dilation, int stride, int combine, int dtype,
                            unsigned need_mask, int variant, void *stream);

/*
 * Filter normalisation of the two filter branches, one launch.  Restates
 * FilterNorm.forward of the reference (ddf/ddf.py:145-173), which is a chain
 * of elementwise and reduction ops there.  `x` and `y` are dense
 * (outer, groups, taps, inner) tensors; every filter, i.e. the `taps` values
 * at fixed (outer, group, inner), is standardised with its own mean and
 * unbiased standard deviation (+1e-10 in the denominator), multiplied by
 * `gain_vec[group*taps + tap]` (or by the scalar `gain` when gain_vec is
 * NULL) and shifted by `offset_vec[group*taps + tap]` (unless NULL).
 * Spatial branch: (b, head, k*k, h*w).  Channel branch: (b, c, k*k, 1).
 * `y` may alias `x` (not when ddf_hip_filter_norm_backward is to follow: it
 * needs the original `x`).
 */
int ddf_hip_filter_norm(const void *x, void *y, int64_t outer, int64_t groups,
                        int taps, int64_t inner, double gain,
                        const void *gain_vec, const void *offset_vec,
                        int dtype, void *stream);

/*
 * Gradient of ddf_hip_filter_norm with respect to `x` (what autograd derives
 * from the op chain of FilterNorm.forward, ddf/ddf.py:145-173, in the
 * reference).  `grad_y` and `x` are the (outer, groups, taps, inner) tensors of
 * the forward call, `gain` / `gain_vec` the same gains; mean and deviation are
 * recomputed from `x`.  `grad_x` is written in full.  `gain_terms`, unless
 * NULL, receives grad_y * standardised(x) element by element: its sum over
 * (outer, inner) is the gradient of `gain_vec`; the gradient of `offset_vec`
 * is the same sum of `grad_y` itself.  `grad_x` may alias `grad_y`.
 */
int ddf_hip_filter_norm_backward(const void *grad_y, const void *x,
                                 void *grad_x, void *gain_terms, int64_t outer,
                                 int64_t groups, int taps, int64_t inner,
                                 double gain, const void *gain_vec, int dtype,
                                 void *stream);

/*
 * ddf_hip_backward with the spatial branch's filter normalisation behind it:
 * what autograd runs, in the reference, for `ddf(x, cf, FilterNorm(raw), ...)`
 * (DDFPack.forward, ddf/ddf.py:217-221, with FilterNorm 'spatial',
 * ddf/ddf.py:146-157) - the operator's backward (ddf/src/ddf_mul_ext.cpp:36-55)
 * followed by the gradient of the normalisation's op chain.
 * `spatial_filter` is the normalised filter the forward pass used,
 * `raw_spatial_filter` the (N, k*k, Ho, Wo) tensor it was normalised from with
 * ddf_hip_filter_norm(raw, sf, N / groups, groups, k*k, Ho*Wo, gain, gain_vec,
 * ...): sample n belongs to group n % groups.  DDF_NEED_DSF asks for
 * `grad_raw_spatial_filter` (the gradient with respect to the raw filter; the
 * gradient of the normalised one is not written anywhere the caller sees) and,
 * unless `gain_terms` is NULL, for the per-element terms of the gain_vec
 * gradient as in ddf_hip_filter_norm_backward.  Where the backward pass ends
 * with a launch that adds up dSF or dCF partial sums, that launch applies the
 * normalisation's Jacobian: one launch fewer than the two calls, and dSF makes
 * no round trip through memory.  Workspace:
 * ddf_hip_backward_spatial_norm_workspace_bytes(...), 256-byte aligned.
 */
size_t ddf_hip_backward_spatial_norm_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W,
                                                     int kernel_size, int dilation, int stride,
                                                     int combine, int dtype, unsigned need_mask,
                                                     int variant);
int ddf_hip_backward_spatial_norm(const void *grad_output, const void *features,
                                  const void *channel_filter, const void *spatial_filter,
                                  const void *raw_spatial_filter, void *grad_features,
                                  void *grad_channel_filter, void *grad_raw_spatial_filter,
                                  void *gain_terms, void *workspace, size_t workspace_bytes,
                                  int64_t N, int64_t C, int64_t H, int64_t W, int kernel_size,
                                  int dilation, int stride, int combine, int dtype,
                                  unsigned need_mask, int groups, double gain, const void *gain_vec,
                                  int variant, void *stream);

/*
 * Spatial filter branch of DDFPack in one launch (build_spatial_branch,
 * ddf/ddf.py:176-180: a 1x1 convolution with the operator's stride to
 * head * k*k taps per pixel, then FilterNorm 'spatial', ddf/ddf.py:145-157).
 * `features` is (N, C, H, W), `weight` the convolution weight (head * k*k, C)
 * (its trailing 1x1 dimensions dropped), `bias` (head * k*k) or NULL;
 * `spatial_filter` receives the normalised (N, head * k*k, H/stride, W/stride)
 * taps, which is the (N * head, k*k, Ho, Wo) operand of the operator.  gain /
 * gain_vec / offset_vec as in ddf_hip_filter_norm with groups = head.
 * Inference path: there is no gradient counterpart; training runs the
 * convolution and ddf_hip_filter_norm / _backward separately.
 * DDF_ERR_UNSUPPORTED: kernel size other than 3 or 5, or fp64.
 */
int ddf_hip_spatial_branch(const void *features, const void *weight,
                           const void *bias, void *spatial_filter, int64_t N,
                           int64_t C, int64_t H, int64_t W, int head,
                           int kernel_size, int stride, double gain,
                           const void *gain_vec, const void *offset_vec,
                           int dtype, void *stream);

/*
 * Channel filter branch of DDFPack after its global average pool, in one
 * launch (build_channel_branch, ddf/ddf.py:183-192: 1x1 convolution C -> mid,
 * ReLU, 1x1 convolution mid -> C * k*k, then FilterNorm 'channel',
 * ddf/ddf.py:158-170).  `pooled` is the (N, C) mean of the features over H x W,
 * `weight1` (mid, C), `bias1` (mid) or NULL, `weight2` (C * k*k, mid), `bias2`
 * (C * k*k) or NULL; `channel_filter` receives the normalised (N, C, k, k)
 * filters.  gain / gain_vec / offset_vec as in ddf_hip_filter_norm with
 * groups = C.  Inference path, as above.  DDF_ERR_UNSUPPORTED: kernel size
 * other than 3 or 5, fp64, or C + mid beyond what one workgroup's LDS holds.
 * fp16 with mid >= 32 and C a multiple of 32 runs on the matrix cores (operands
 * aligned for vector loads: weight1 to 16 bytes, pooled, bias2, gain_vec,
 * offset_vec and channel_filter to 8; anything else takes the vector-ALU
 * kernel): sums in fp32, the pooled and hidden vectors rounded to fp16 as the
 * reference's half-precision modules round them.
 */
int ddf_hip_channel_branch(const void *pooled, const void *weight1,
                           const void *bias1, const void *weight2,
                           const void *bias2, void *channel_filter, int64_t N,
                           int64_t C, int64_t mid, int kernel_size,
                           double gain, const void *gain_vec,
                           const void *offset_vec, int dtype, void *stream);

/*
 * The two branches with the global average pool between them folded in
 * (DDFPack.forward computes the channel filter from the pooled features,
 * ddf/ddf.py:183-185 and :213-219; no counterpart as a function in the reference).
 * ddf_hip_spatial_branch_pool is ddf_hip_spatial_branch that also leaves, from
 * the feature values it has in registers anyway, partial sums of every feature
 * plane: pool_parts[(n * *n_parts + p) * C + c], fp32, is the sum of
 * features[n, c] over the pixels of part p.  The caller provides room for
 * pool_capacity floats (N * C * 4 * ceil((H/stride) * (W/stride) / 64) is always
 * enough) and gets the number of parts back in *n_parts.
 * ddf_hip_channel_branch_parts is ddf_hip_channel_branch with the pooled
 * vector given as scale * (sum of n_parts such partial sums), scale = 1 / (H*W).
 * One launch and one full read of the feature map fewer per layer than
 * pooling first.  DDF_ERR_UNSUPPORTED (then pool and call the plain entry
 * points): kernel size other than 3, odd H or W under stride 2, or a shape the
 * streaming kernel turns down; DDF_ERR_WORKSPACE: pool_capacity too small.
 */
int ddf_hip_spatial_branch_pool(const void *features, const void *weight,
                                const void *bias, void *spatial_filter,
                                float *pool_parts, int64_t pool_capacity,
                                int *n_parts, int64_t N, int64_t C, int64_t H,
                                int64_t W, int head, int kernel_size, int stride,
                                double gain, const void *gain_vec,
                                const void *offset_vec, int dtype, void *stream);
int ddf_hip_channel_branch_parts(const float *pool_parts, int n_parts,
                                 double scale, const void *weight1,
                                 const void *bias1, const void *weight2,
                                 const void *bias2, void *channel_filter,
                                 int64_t N, int64_t C, int64_t mid,
                                 int kernel_size, double gain,
                                 const void *gain_vec, const void *offset_vec,
                                 int dtype, void *stream);

/*
 * Up-sampling DDF forward (DDFUpPack.forward, ddf/ddf.py:257-272): the
 * reference calls `ddf` once per sub-pixel branch b = 0 .. scale*scale-1 on
 * the same features with that branch's filters (ddf.py:264-269), stacks the
 * results and pixel-shuffles them (ddf.py:270-272).  This entry point does all
 * of it in one launch:
 *   output[n, c, y*scale + i, x*scale + j] =
 *       ddf(features, channel_filters[i*scale + j], spatial_filters[i*scale + j],
 *           kernel_size, dilation, stride 1, combine)[n, c, y, x]
 * `channel_filters` and `spatial_filters` are host arrays of scale*scale device
 * pointers, each a dense (N, C, k, k) resp. (N, k*k, H, W) tensor; `output`
 * is dense (N, C, H*scale, W*scale).  Covered: k = 1 or 3 with scale 2..4 and
 * k = 5 with scale 2; anything else returns DDF_ERR_UNSUPPORTED and the caller
 * composes the result from ddf_hip_forward.
 */
#define DDF_UP_MAX_BRANCHES 16
int ddf_hip_up_forward(const void *features,
                       const void *const *channel_filters,
                       const void *const *spatial_filters, void *output,
                       int64_t N, int64_t C, int64_t H, int64_t W,
                       int kernel_size, int dilation, int scale, int combine,
                       int dtype, void *stream);

/*
 * Backward of ddf_hip_up_forward: what autograd derives in the reference from
 * F.pixel_shuffle, torch.stack and the scale*scale `ddf` calls of
 * DDFUpPack.forward (ddf/ddf.py:264-272), done inside the library: the
 * gradient is split into its sub-pixel lattices (one launch), every branch
 * runs the kernels of ddf_hip_backward on its lattice, and the branches'
 * feature gradients are summed (one launch).  `grad_output` is dense
 * (N, C, H*scale, W*scale); `grad_channel_filters` / `grad_spatial_filters`
 * are host arrays of scale*scale device pointers (an array, or single
 * entries of it, may be NULL: that gradient is not computed); `need_mask` as
 * in ddf_hip_backward.  Any odd kernel_size; scale 2..4.  `workspace` must
 * hold ddf_hip_up_backward_workspace_bytes(...) bytes, 256-byte aligned.
 */
size_t ddf_hip_up_backward_workspace_bytes(int64_t N, int64_t C, int64_t H,
                                           int64_t W, int kernel_size,
                                           int dilation, int scale,
                                           int combine, int dtype,
                                           unsigned need_mask);
int ddf_hip_up_backward(const void *grad_output, const void *features,
                        const void *const *channel_filters,
                        const void *const *spatial_filters,
                        void *grad_features,
                        void *const *grad_channel_filters,
                        void *const *grad_spatial_filters, void *workspace,
                        size_t workspace_bytes, int64_t N, int64_t C,
                        int64_t H, int64_t W, int kernel_size, int dilation,
                        int scale, int combine, int dtype, unsigned need_mask,
                        void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DDF_HIP_H */
