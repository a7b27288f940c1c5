/*
 * dcn_amd.h -- C ABI of the MI355X (gfx950) deformable-convolution library, libdcn_amd.so.
 *
 * Drop-in boundary for the three native entry points each operator package of
 * lshiwjx/deform_conv3d_pytorch_op binds through cffi:
 *
 *   deform_conv_forward_cuda                 deform3d/lib/deform_conv3d_cuda.h:12-18
 *                                            deform2d_double/lib/deform_conv2d_cuda.h:12-18
 *                                            deform2d/lib/deform_conv2d_cuda.h:12-17
 *   deform_conv_backward_input_offset_cuda   deform3d/lib/deform_conv3d_cuda.h:20-26
 *                                            deform2d_double/lib/deform_conv2d_cuda.h:20-26
 *                                            deform2d/lib/deform_conv2d_cuda.h:19-24
 *   deform_conv_backward_weight_cuda         deform3d/lib/deform_conv3d_cuda.h:28-34
 *                                            deform2d_double/lib/deform_conv2d_cuda.h:28-34
 *                                            deform2d/lib/deform_conv2d_cuda.h:26-31
 *
 * The reference passes THCudaTensor handles; here every tensor is a raw device pointer to a
 * contiguous row-major buffer and every extent is an explicit int, in the reference's argument
 * order (pad, stride, dilation triples, channel_per_deformable_group, group).  Layouts:
 *
 *   input        [batch][input_c][input_l][input_h][input_w]              (no input_l in 2-D)
 *   weight       [output_c][input_c / group][kernel_l][kernel_h][kernel_w]
 *   offset       [batch][input_c / channel_per_deformable_group][kernel volume][nd][output volume]
 *                axis order (l, h, w) in 3-D and (h, w) in 2-D
 *   output       [batch][output_c][output_l][output_h][output_w]
 *
 * Differences from the reference ABI, all on purpose:
 *   - there is no `columns` argument: the sampled column buffer never exists in device memory;
 *   - `workspace` is caller-owned scratch of at least dcn_workspace_bytes(...) bytes, 256-byte
 *     aligned; the library never allocates device memory;
 *   - `stream` is the hipStream_t to enqueue on (NULL = the null stream); calls are asynchronous;
 *   - the return value is 0 on success and a negative DCN_E_* code on failure, with the text
 *     from dcn_last_error() (thread-local).  The reference returns 1 and raises through THError.
 *   - the caller's weight tensor is never reshaped in place (the reference does that).
 *
 * Caller obligations kept from the reference: `output` and `grad_offset` are fully overwritten;
 * `grad_input` and `grad_weight` are ACCUMULATED into and must be zero-filled by the caller when
 * a plain gradient is wanted (deform3d/deform_conv3d_functions/deform_conv3d_function.py:53,64).
 * Output extents must satisfy the reference formula out = (in + 2*pad - kernel) / stride + 1
 * (integer division, dilation not included; deform3d/lib/deform_conv3d_cuda.cpp:15-17,81-86).
 * The dilation-aware size (in + 2*pad - dilation*(kernel-1) - 1) / stride + 1 is accepted as
 * well: it is the same layer cropped to the leading positions of each axis (no counterpart in
 * the reference, which always uses the first formula).
 */
#ifndef DCN_AMD_H
#define DCN_AMD_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DCN_OK            0
#define DCN_E_ARGUMENT   -1   /* inconsistent extents, null pointer, unsupported size */
#define DCN_E_WORKSPACE  -2   /* workspace missing or too small */
#define DCN_E_LAUNCH     -3   /* HIP reported an error when launching */
#define DCN_E_DEVICE     -4   /* no current HIP device, a query of it failed, or it is not a gfx950 GPU */

int dcn_version(void);              /* ABI version, currently 1 */
const char *dcn_arch(void);         /* the code-object target the kernels were built for: "gfx950" */
const char *dcn_last_error(void);   /* message of the last failing call on this thread ("" if none) */

/* Scratch bytes any of the three calls below needs for this layer (elem_size 4 = f32, 8 = f64; the
 * 16-bit formats, elem_size 2, are served by dcn_workspace_bytes_for only and get 0 here;
 * input_volume = input_l * input_h * input_w, output_volume likewise, kernel_volume =
 * kernel_l * kernel_h * kernel_w).  The workspace holds a re-laid-out copy of the weight and, for
 * the backward calls, channels-last copies of the input batch, its gradient and grad_output, and
 * one word in which the device records which of the planned LDS halo sizes it chose for the call
 * from the offsets (so two calls that overlap in time need a workspace each; the forward calls
 * keep it as a 32-bit index, 0 = the narrowest halo, at byte offset (workspace_bytes - 256) rounded
 * down to a multiple of 256, the backward_input_offset calls 64 bytes further; there the value 3
 * means that the device took the path without LDS tiling, which it does for a 3-D layer when most
 * samples would leave even the widest halo). */
size_t dcn_workspace_bytes(int elem_size, int batch, int input_c, int output_c, size_t input_volume,
                           size_t output_volume, int kernel_volume, int group);
/* The same for a known number of channels per deformable group (the reference's
 * `channel_per_group`, deform3d/lib/deform_conv3d_cuda.cpp:66): never larger than the figure
 * above, and much smaller for wide layers, whose per-chunk weight slabs the first query has to
 * size for one-channel deformable groups.  0 for an inconsistent geometry. */
size_t dcn_workspace_bytes_for(int elem_size, int batch, int input_c, int output_c, size_t input_volume,
                               size_t output_volume, int kernel_volume, int group,
                               int channel_per_deformable_group);

/* ---- 3-D, trilinear ------------------------------------------------------------------------
 * replaces deform3d/lib/deform_conv3d_cuda.cpp:90-165 (forward), :168-262 (backward_input_offset)
 * and :265-336 (backward_weight).  The reference instantiates float only; f64 is the same
 * arithmetic in double.  `bias` ([output_c] or NULL) is added in the epilogue; the reference adds
 * it from Python (deform_conv3d_function.py:41-42). */
#define DCN3D_GEOMETRY                                                                           \
    int batch, int input_c, int output_c, int input_l, int input_h, int input_w, int output_l,   \
    int output_h, int output_w, int kernel_l, int kernel_h, int kernel_w, int pad_l, int pad_h,  \
    int pad_w, int stride_l, int stride_h, int stride_w, int dilation_l, int dilation_h,         \
    int dilation_w, int channel_per_deformable_group, int group

int dcn3d_forward_f32(const float *input, const float *weight, const float *offset, const float *bias,
                      float *output, DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn3d_forward_f64(const double *input, const double *weight, const double *offset, const double *bias,
                      double *output, DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);

int dcn3d_backward_input_offset_f32(const float *input, const float *weight, const float *offset,
                                    const float *grad_output, float *grad_input, float *grad_offset,
                                    DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn3d_backward_input_offset_f64(const double *input, const double *weight, const double *offset,
                                    const double *grad_output, double *grad_input, double *grad_offset,
                                    DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);

/* Forward pass that allocates nothing and takes no workspace.  No counterpart in the reference: it
 * is for callers that cannot allocate device memory around the call (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  Same arguments, results and kernels as
 * dcn3d_forward_f32 without the workspace pair; the re-laid-out weight (and, for a layer of few
 * positions, as many partial outputs as still fit; in the last 256 bytes the halo size chosen for
 * the call) goes into a fixed device array
 * of DCN_NOALLOC_SCRATCH_BYTES inside the library, which every GPU the library runs on holds until
 * the process ends.  A layer whose re-laid-out weight is larger (roughly: 4 * kernel volume *
 * output_c rounded up to 256 * (input_c / group + 4) bytes) is rejected with DCN_E_WORKSPACE.  All
 * calls on one GPU share that array: calls that overlap there (two streams, two threads) race on it
 * and must be serialised by the caller; calls on different GPUs are independent. */
#define DCN_NOALLOC_SCRATCH_BYTES (8u << 20)
int dcn3d_forward_noalloc_f32(const float *input, const float *weight, const float *offset, const float *bias,
                              float *output, DCN3D_GEOMETRY, void *stream);

/* The same call with option flags.  No counterpart in the reference, whose 3-D col2im_offset kernel
 * always adds +-|grad column| to grad_offset for a sample that lies outside the input
 * (deform3d/lib/deform_conv3d_cuda_kernel.cu:470-481), although such a sample contributes nothing to
 * the output: with DCN_FLAG_OOB_OFFSET_GRAD_ZERO that term is left out and grad_offset is the
 * derivative of the forward pass everywhere.  flags = 0 is dcn3d_backward_input_offset_*; other
 * bits are rejected.  (The reference's 2-D kernels have no such term.) */
#define DCN_FLAG_OOB_OFFSET_GRAD_ZERO 1u
int dcn3d_backward_input_offset_flags_f32(const float *input, const float *weight, const float *offset,
                                          const float *grad_output, float *grad_input, float *grad_offset,
                                          DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes,
                                          void *stream, unsigned flags);
int dcn3d_backward_input_offset_flags_f64(const double *input, const double *weight, const double *offset,
                                          const double *grad_output, double *grad_input, double *grad_offset,
                                          DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes,
                                          void *stream, unsigned flags);

int dcn3d_backward_weight_f32(const float *input, const float *offset, const float *grad_output,
                              float *grad_weight, DCN3D_GEOMETRY, void *workspace,
                              size_t workspace_bytes, void *stream);
int dcn3d_backward_weight_f64(const double *input, const double *offset, const double *grad_output,
                              double *grad_weight, DCN3D_GEOMETRY, void *workspace,
                              size_t workspace_bytes, void *stream);

/* ---- 2-D, bilinear -------------------------------------------------------------------------
 * replaces deform2d_double/lib/deform_conv2d_cuda.cpp:82-155, :158-249, :252-325 (double, with
 * dilation and groups) and deform2d/lib/deform_conv2d_cuda.cpp:82-128, :131-190, :193-235
 * (float; its ABI has no dilation/group arguments: pass dilation 1, group 1). */
#define DCN2D_GEOMETRY                                                                           \
    int batch, int input_c, int output_c, int input_h, int input_w, int output_h, int output_w,  \
    int kernel_h, int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w,                \
    int dilation_h, int dilation_w, int channel_per_deformable_group, int group

int dcn2d_forward_f32(const float *input, const float *weight, const float *offset, const float *bias,
                      float *output, DCN2D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn2d_forward_f64(const double *input, const double *weight, const double *offset, const double *bias,
                      double *output, DCN2D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);

int dcn2d_backward_input_offset_f32(const float *input, const float *weight, const float *offset,
                                    const float *grad_output, float *grad_input, float *grad_offset,
                                    DCN2D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn2d_backward_input_offset_f64(const double *input, const double *weight, const double *offset,
                                    const double *grad_output, double *grad_input, double *grad_offset,
                                    DCN2D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);

int dcn2d_backward_weight_f32(const float *input, const float *offset, const float *grad_output,
                              float *grad_weight, DCN2D_GEOMETRY, void *workspace,
                              size_t workspace_bytes, void *stream);
int dcn2d_backward_weight_f64(const double *input, const double *offset, const double *grad_output,
                              double *grad_weight, DCN2D_GEOMETRY, void *workspace,
                              size_t workspace_bytes, void *stream);

/* ---- plain 2-D convolution -------------------------------------------------------------------
 * replaces the three symbols of the reference's conv2d package, conv2d/lib/conv2d_cuda.h:17-39
 * (conv_forward_cuda, conv_backward_input_cuda, conv_backward_weight_cuda; host loops
 * conv2d/lib/conv2d_cuda.cpp:77-290).  The reference's `columns` argument does not exist here.  The
 * output extents follow the dilation-aware formula of conv2d/lib/conv2d_cuda.cpp:20-22,
 * (input + 2 pad - dilation (kernel - 1) - 1) / stride + 1.  `bias` ([output_c] or NULL) is added in
 * the epilogue (the reference adds it from Python, conv2d/conv2d_functions/conv2d_function.py:34-35);
 * grad_input and grad_weight are accumulated into (the caller zero-fills them, as the reference's
 * Function does).  backward_input is not given the input, like the reference's.  The layer runs as the
 * 2-D deformable layer with every offset zero; the workspace (conv2d_workspace_bytes) holds that zero
 * offset tensor in front of the deformable layer's own workspace. */
#define CONV2D_GEOMETRY                                                                          \
    int batch, int input_c, int output_c, int input_h, int input_w, int output_h, int output_w,  \
    int kernel_h, int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w,                \
    int dilation_h, int dilation_w, int group
size_t conv2d_workspace_bytes(int elem_size, int batch, int input_c, int output_c, size_t input_volume,
                              size_t output_volume, int kernel_volume, int group);
int conv2d_forward_f32(const float *input, const float *weight, const float *bias, float *output, CONV2D_GEOMETRY,
                       void *workspace, size_t workspace_bytes, void *stream);
int conv2d_forward_f64(const double *input, const double *weight, const double *bias, double *output, CONV2D_GEOMETRY,
                       void *workspace, size_t workspace_bytes, void *stream);
int conv2d_backward_input_f32(const float *weight, const float *grad_output, float *grad_input, CONV2D_GEOMETRY,
                              void *workspace, size_t workspace_bytes, void *stream);
int conv2d_backward_input_f64(const double *weight, const double *grad_output, double *grad_input, CONV2D_GEOMETRY,
                              void *workspace, size_t workspace_bytes, void *stream);
int conv2d_backward_weight_f32(const float *input, const float *grad_output, float *grad_weight, CONV2D_GEOMETRY,
                               void *workspace, size_t workspace_bytes, void *stream);
int conv2d_backward_weight_f64(const double *input, const double *grad_output, double *grad_weight, CONV2D_GEOMETRY,
                               void *workspace, size_t workspace_bytes, void *stream);

/* ---- 16-bit storage, float32 accumulation ----------------------------------------------------
 * No counterpart in the reference, which instantiates float only
 * (deform3d/lib/deform_conv3d_cuda_kernel.cu:162-172).  Every tensor (input, weight, offset, bias,
 * grad_output and the results) is stored as bfloat16 (_bf16) or IEEE binary16 (_f16).
 * forward: coordinates and interpolation in float32; the sampled columns are rounded to the storage
 * format and multiplied with the weights by 16-bit matrix instructions that accumulate in float32;
 * bias added in float32, one rounding per output element.  (Layers that the LDS-halo kernel cannot
 * serve are widened to float32 and computed there.)
 * backward_input_offset: the fused kernel reads the 16-bit tensors itself and forms the grad columns
 * with 16-bit matrix instructions (products of 16-bit values are exact in float32; float32 sums);
 * coordinates, interpolation, the scatter and the coordinate gradient are float32.
 * backward_weight: like forward, the sampled columns are rounded to the storage format and multiplied
 * with grad_output by 16-bit matrix instructions that accumulate in float32.
 * Each result element is rounded once, to nearest even.  Layers that these kernels do not serve (more
 * output channels than the fused kernel keeps in registers, odd channel counts, ...) are widened exactly
 * into float32 copies and computed by the float32 kernels, with the same single rounding at the end.
 * Same argument meaning and accumulate / overwrite contract as the _f32 calls (grad_input and
 * grad_weight: rounded sum of their previous content and the gradient).  The workspace must come
 * from dcn_workspace_bytes_for(2, ...): it also holds float copies of the tensors.  Offsets in 16
 * bits limit the sampling positions to that format's grid (bfloat16: 1/128 voxel between 1 and 2,
 * coarser above). */
int dcn3d_forward_bf16(const void *input, const void *weight, const void *offset, const void *bias,
                       void *output, DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn3d_backward_input_offset_bf16(const void *input, const void *weight, const void *offset,
                                     const void *grad_output, void *grad_input, void *grad_offset,
                                     DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn3d_backward_weight_bf16(const void *input, const void *offset, const void *grad_output,
                               void *grad_weight, DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes,
                               void *stream);

int dcn2d_forward_bf16(const void *input, const void *weight, const void *offset, const void *bias,
                       void *output, DCN2D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn2d_backward_input_offset_bf16(const void *input, const void *weight, const void *offset,
                                     const void *grad_output, void *grad_input, void *grad_offset,
                                     DCN2D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn2d_backward_weight_bf16(const void *input, const void *offset, const void *grad_output,
                               void *grad_weight, DCN2D_GEOMETRY, void *workspace, size_t workspace_bytes,
                               void *stream);

int dcn3d_forward_f16(const void *input, const void *weight, const void *offset, const void *bias,
                       void *output, DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn3d_backward_input_offset_f16(const void *input, const void *weight, const void *offset,
                                     const void *grad_output, void *grad_input, void *grad_offset,
                                     DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn3d_backward_weight_f16(const void *input, const void *offset, const void *grad_output,
                               void *grad_weight, DCN3D_GEOMETRY, void *workspace, size_t workspace_bytes,
                               void *stream);

int dcn2d_forward_f16(const void *input, const void *weight, const void *offset, const void *bias,
                       void *output, DCN2D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn2d_backward_input_offset_f16(const void *input, const void *weight, const void *offset,
                                     const void *grad_output, void *grad_input, void *grad_offset,
                                     DCN2D_GEOMETRY, void *workspace, size_t workspace_bytes, void *stream);
int dcn2d_backward_weight_f16(const void *input, const void *offset, const void *grad_output,
                               void *grad_weight, DCN2D_GEOMETRY, void *workspace, size_t workspace_bytes,
                               void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DCN_AMD_H */
