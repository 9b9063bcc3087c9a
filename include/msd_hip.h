/*
 * C ABI of libmsd_hip.so: dilated 3x3 (2D) / 3x3x3 (3D) convolution with
 * symmetric ("reflection") padding, optional fused ReLU, forward and backward,
 * on AMD gfx950 (MI355X).
 *
 * One entry point per operator that the reference exports from its pybind11
 * module `msd_custom_convolutions` (msd_custom_convolutions.cpp:343-369); the
 * 2D/3D and float/double variants that the reference selects by tensor rank
 * and AT_DISPATCH_FLOATING_TYPES (torch_cuda_dispatch.cu:95-441) are selected
 * here by the `ndim` and `dtype` arguments.
 *
 * Conventions
 *   - every data pointer is DEVICE memory on the current HIP device;
 *   - a tensor view is a base pointer plus `ndim + 2` ELEMENT strides in the
 *     order {batch, channel, [z,] y, x}; views may be channel slices of a larger
 *     allocation (the dense block's growing stack, msd_block.py:30-46).
 *     Strides must be non-negative and no two elements of an output view may alias;
 *   - `spatial` holds `ndim` extents, {H, W} or {D, H, W};
 *   - weights are contiguous (c_out, c_in, 3, 3[, 3]); bias is contiguous (c_out);
 *   - 0 < dilation <= every spatial extent (msd_custom_convolutions.cpp:39-52),
 *     so a single fold of the index suffices;
 *   - `stream` is a hipStream_t (NULL = the default stream); calls are
 *     asynchronous and never synchronise the host;
 *   - return value 0 = success; otherwise an MSD_ERR_* code, and
 *     msd_last_error() returns a message for the calling thread.
 *   - the caller owns every buffer; `output` is overwritten; `grad_input`,
 *     `grad_kernel` and `grad_bias` are ACCUMULATED into
 *     (conv2d_backward_x.cu:103,205; conv2d_backward_k.cu:52,105;
 *     conv2d_backward_bias.cu:46).
 *   - results are deterministic: weight and bias gradients are reduced in a
 *     fixed order through `workspace` (the reference uses float atomics).
 */
#ifndef MSD_HIP_H
#define MSD_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MSD_F32 0
#define MSD_F64 1

#define MSD_OK 0
#define MSD_ERR_INVALID 1   /* bad argument; nothing was launched */
#define MSD_ERR_HIP 2       /* the HIP runtime reported an error */
#define MSD_ERR_WORKSPACE 3 /* workspace missing or too small */

/* Message describing the last failure on the calling thread ("" if none). */
const char *msd_last_error(void);

/* ABI version of this header: bumped on any incompatible change. */
int msd_abi_version(void);

/*
 * Test hook: 0 (default) lets the library pick the specialised gfx950 kernels
 * where they apply, 1 forces the shape-generic kernels for every call.  Both
 * paths compute the same operators; the parity tests run each against the other.
 * Process-wide; not meant to be switched while calls are in flight on other threads.
 */
int msd_set_kernel_path(int path);

/*
 * Tuning hook used by the operator benchmark (the counterpart of the
 * reference's per-call block_size argument, conv3d.py:8-37): overrides one
 * launch-shape parameter of the specialised kernels, e.g. "bwdx.vec3d" (voxels
 * per lane) or "bwdx.unroll3d" (channels in flight).  value < 0 restores the
 * library default; values a kernel was not built for fall back to the default.
 * Results do not depend on these settings beyond floating-point summation order.
 * Keys: "bwdx.vec2d", "bwdx.vec3d", "bwdk.vec2d", "bwdk.vec3d", "fwd.vec2d", "fwd.vec3d"
 * (voxels per lane), "bwdx.unroll2d", "bwdx.unroll3d" (channels in flight),
 * "bwdx.min_blocks", "bwdk.blocks" (workgroups per launch), "fwd.split" (channel groups
 * per workgroup), "fwd.rows2d" (rows per forward tile), "xcd_remap" (0/1: workgroup order
 * by XCD), "bwdk.rows" (0/1: row-team weight-gradient kernel), "bwdk.interleave" (0/1:
 * workgroups take every n-th row group), "block.fuse" (0/1: fused backward in the block),
 * "block.defer" (0/1: one reduction launch for many layers), "block.snake" (0/1: alternate
 * layers walk the channels in opposite directions), "fwd.class3d" (0/1: 3D forward tiles
 * numbered by residue class), "fwd.lattice3d" (24, 33 or 44: rows z x y of a 3D forward tile;
 * 0: chosen by the library), "block.pair" (0/1: the backward pass of a 2D block of one-channel
 * layers takes its layers two or three at a time), "block.triple" (0: never three at a time,
 * n > 0: three where the layers share at least n channels; 32 by default), "final.tiled" (0/1:
 * msd_final_forward_loss reads the stack once, through LDS tiles, where it can: fp32, up to 128
 * input and 4 output channels), "block.split3d" (the backward pass of a 3D block of one-channel
 * layers; 1: a chain of backward_x launches on the caller's stream and the weight gradients, two
 * layers per pass, on a second stream that is forked from and joined to the caller's inside the
 * call; 2: the same launches on the caller's stream alone; 0: one fused launch per layer),
 * "block.chainpair" (0/1: that chain takes two layers per read-modify-write pass over
 * grad_input where it can; 0: one launch per layer), "bwdk.fused3d" (0/1: the weight gradient of
 * a 3D layer of one or two output channels runs on the weight-gradient-only form of the fused
 * backward kernel where that takes the shape; 0: on the separate weight-gradient kernels),
 * "bwdx.lean1" (0/1: a 3D backward_x over one input and one output channel runs on a kernel
 * of its own; 0: on the general one).
 * Unknown keys return MSD_ERR_INVALID.
 */
int msd_set_tuning(const char *key, int value);

/*
 * Bytes of device scratch that msd_conv_backward_k, msd_conv_relu_backward_k,
 * msd_conv_relu_backward_kb and msd_conv_relu_backward_bias need for this
 * problem (partial sums of the fixed-order reduction).  Returns < 0 on
 * invalid arguments.
 */
int64_t msd_workspace_bytes(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                            const int64_t *spatial);

/* y = bias + conv(x).  Replaces conv_forward, msd_custom_convolutions.cpp:85-117
 * (kernels conv2d_forward.cu:22-93, conv3d_forward.cu:22-108). */
int msd_conv_forward(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                     const int64_t *spatial, int dilation,
                     const void *input, const int64_t *input_strides,
                     const void *kernel, const void *bias,
                     void *output, const int64_t *output_strides, void *stream);

/* y = max(0, bias + conv(x)).  Replaces conv_relu_forward,
 * msd_custom_convolutions.cpp:213-245 (kernels conv2d_forward.cu:95-174,
 * conv3d_forward.cu:110-196). */
int msd_conv_relu_forward(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                          const int64_t *spatial, int dilation,
                          const void *input, const int64_t *input_strides,
                          const void *kernel, const void *bias,
                          void *output, const int64_t *output_strides, void *stream);

/* grad_input += conv^T(grad_output).  Replaces conv_backward_x,
 * msd_custom_convolutions.cpp:119-148 (kernels conv2d_backward_x.cu:13-106,
 * conv3d_backward_x.cu:13-123). */
int msd_conv_backward_x(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                        const int64_t *spatial, int dilation,
                        const void *grad_output, const int64_t *grad_output_strides,
                        const void *kernel,
                        void *grad_input, const int64_t *grad_input_strides, void *stream);

/* grad_input += conv^T(grad_output * [0 < output]).  Replaces conv_relu_backward_x,
 * msd_custom_convolutions.cpp:247-281 (kernels conv2d_backward_x.cu:109-208,
 * conv3d_backward_x.cu:125-241). */
int msd_conv_relu_backward_x(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                             const int64_t *spatial, int dilation,
                             const void *output, const int64_t *output_strides,
                             const void *grad_output, const int64_t *grad_output_strides,
                             const void *kernel,
                             void *grad_input, const int64_t *grad_input_strides, void *stream);

/* grad_kernel += d/dk.  Replaces conv_backward_k, msd_custom_convolutions.cpp:150-178
 * (kernels conv2d_backward_k.cu:12-59, conv3d_backward_k.cu:11-64). */
int msd_conv_backward_k(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                        const int64_t *spatial, int dilation,
                        const void *grad_output, const int64_t *grad_output_strides,
                        const void *input, const int64_t *input_strides,
                        void *grad_kernel,
                        void *workspace, int64_t workspace_bytes, void *stream);

/* grad_kernel += d/dk with the ReLU mask.  Replaces conv_relu_backward_k,
 * msd_custom_convolutions.cpp:283-316 (kernels conv2d_backward_k.cu:61-112,
 * conv3d_backward_k.cu:66-122). */
int msd_conv_relu_backward_k(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                             const int64_t *spatial, int dilation,
                             const void *output, const int64_t *output_strides,
                             const void *grad_output, const int64_t *grad_output_strides,
                             const void *input, const int64_t *input_strides,
                             void *grad_kernel,
                             void *workspace, int64_t workspace_bytes, void *stream);

/* grad_bias += sum over batch and voxels of grad_output.  Replaces conv_backward_bias,
 * msd_custom_convolutions.cpp:180-211 (a torch sum in the reference). */
int msd_conv_backward_bias(int dtype, int ndim, int64_t batch, int64_t c_out,
                           const int64_t *spatial,
                           const void *grad_output, const int64_t *grad_output_strides,
                           void *grad_bias,
                           void *workspace, int64_t workspace_bytes, void *stream);

/* grad_bias += sum of grad_output where 0 < output.  Replaces conv_relu_backward_bias,
 * msd_custom_convolutions.cpp:318-338 (kernels conv2d_backward_bias.cu:12-49,
 * conv3d_backward_bias.cu:12-51). */
int msd_conv_relu_backward_bias(int dtype, int ndim, int64_t batch, int64_t c_out,
                                const int64_t *spatial,
                                const void *output, const int64_t *output_strides,
                                const void *grad_output, const int64_t *grad_output_strides,
                                void *grad_bias,
                                void *workspace, int64_t workspace_bytes, void *stream);

/* msd_conv_relu_backward_k and msd_conv_relu_backward_bias in one pass over the
 * data: the two calls the dense block makes back to back for every layer
 * (msd_block.py:113-126) share their reads of output and grad_output.
 * grad_bias may be NULL. */
int msd_conv_relu_backward_kb(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                              const int64_t *spatial, int dilation,
                              const void *output, const int64_t *output_strides,
                              const void *grad_output, const int64_t *grad_output_strides,
                              const void *input, const int64_t *input_strides,
                              void *grad_kernel, void *grad_bias,
                              void *workspace, int64_t workspace_bytes, void *stream);

/* msd_conv_relu_backward_kb without a workspace argument and without any allocation.
 * No counterpart in the reference.  It is for callers that cannot allocate device memory:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * The partial sums of the fixed-order reduction go through a buffer of
 * MSD_STATIC_SCRATCH_BYTES = 32 MiB that is part of the library's device image (each GPU
 * the library runs on holds it until the process ends); a problem whose msd_workspace_bytes
 * exceeds it is rejected with MSD_ERR_WORKSPACE and nothing is launched.  Same kernels and
 * the same bits as msd_conv_relu_backward_kb.  All calls on one GPU share the buffer: calls
 * that overlap on one GPU (different streams or threads) race.  The first call on a device
 * looks the buffer's address up (hipGetSymbolAddress) and so must not be made under stream
 * capture; later calls only launch kernels. */
#define MSD_STATIC_SCRATCH_BYTES (32 * 1024 * 1024)
int msd_conv_relu_backward_kb_static(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                                     const int64_t *spatial, int dilation,
                                     const void *output, const int64_t *output_strides,
                                     const void *grad_output, const int64_t *grad_output_strides,
                                     const void *input, const int64_t *input_strides,
                                     void *grad_kernel, void *grad_bias, void *stream);

/* msd_conv_backward_k and msd_conv_backward_bias in one pass (no ReLU mask).
 * grad_bias may be NULL.  No counterpart in the reference. */
int msd_conv_backward_kb(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                         const int64_t *spatial, int dilation,
                         const void *grad_output, const int64_t *grad_output_strides,
                         const void *input, const int64_t *input_strides,
                         void *grad_kernel, void *grad_bias,
                         void *workspace, int64_t workspace_bytes, void *stream);

/* The three plain backward operators of one layer in one call:
 *   grad_input += backward_x(grad_output, kernel), grad_kernel += backward_k(grad_output, input),
 *   grad_bias += backward_bias(grad_output)   (grad_bias may be NULL)
 * i.e. msd_block.py:107-126 for a grad_output that is already masked (msd_relu_mask_gradient).
 * fp32 problems with one output channel, unit x-strides and rows of whole 4-voxel groups run
 * as ONE pass over the input channels (the gather of grad_output is shared, input and
 * grad_input are read once, grad_input written once); everything else runs the two
 * operators one after the other.  grad_input must not alias input or grad_output.
 * No counterpart in the reference. */
int msd_conv_backward_xkb(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                          const int64_t *spatial, int dilation,
                          const void *grad_output, const int64_t *grad_output_strides,
                          const void *input, const int64_t *input_strides,
                          const void *kernel,
                          void *grad_input, const int64_t *grad_input_strides,
                          void *grad_kernel, void *grad_bias,
                          void *workspace, int64_t workspace_bytes, void *stream);

/* grad_output = grad_output * [0 < output], in place: the ReLU mask that the three
 * conv_relu_backward_* operators of one layer (msd_block.py:107-126) each apply on
 * the fly, applied once.  After it the plain backward operators give the layer's
 * gradients.  Only valid when the caller owns grad_output and no longer needs the
 * unmasked values, as in the dense block's private gradient stack (msd_block.py:83). */
int msd_relu_mask_gradient(int dtype, int ndim, int64_t batch, int64_t c_out, const int64_t *spatial,
                           const void *output, const int64_t *output_strides,
                           void *grad_output, const int64_t *grad_output_strides, void *stream);

/*
 * Dense block (MSDBlockFunction, msd_block.py:8-134) as one call per direction.
 * `stack` is the (batch, c_in + sum(widths), spatial) channel stack; layer i reads
 * channels [0, C_i) and writes [C_i, C_i + widths[i]), C_i = c_in + widths[0..i).
 * `weights[i]` is the contiguous (widths[i], C_i, 3, 3[, 3]) kernel of layer i
 * (host array of device pointers), `bias` the flat bias of sum(widths) entries.
 *
 * msd_block_forward: channels [0, c_in) of `stack` hold the input on entry; the
 * remaining channels are computed (the loop of msd_block.py:40-58).
 *
 * msd_block_backward: `grads` holds dL/dstack on entry and is MODIFIED IN PLACE (it
 * is the private working copy of msd_block.py:83); on return channels [0, c_in) hold
 * dL/dinput (if need_input_grad).  grad_weights[i] (zero-filled by the caller, NULL to
 * skip a layer) and grad_bias (zero-filled, NULL to skip) are accumulated into.
 * Replaces the loop of msd_block.py:89-130.  Workspace: msd_block_workspace_bytes,
 * which is the largest msd_workspace_bytes of the layers plus room (at most 1 GiB) for
 * the partial weight-gradient sums of many layers at once, so that one launch can
 * reduce up to 16 layers; the largest msd_workspace_bytes of the layers alone is
 * accepted too (every layer then reduces its sums right away; same results).
 */
int64_t msd_block_workspace_bytes(int dtype, int ndim, int64_t batch, int64_t c_in, int depth,
                                  const int64_t *widths, const int64_t *spatial);

int msd_block_forward(int dtype, int ndim, int64_t batch, int64_t c_in, int depth, const int64_t *widths,
                      const int64_t *spatial, const int64_t *dilations,
                      void *stack, const int64_t *stack_strides,
                      const void *const *weights, const void *bias, void *stream);

int msd_block_backward(int dtype, int ndim, int64_t batch, int64_t c_in, int depth, const int64_t *widths,
                       const int64_t *spatial, const int64_t *dilations,
                       const void *stack, const int64_t *stack_strides,
                       void *grads, const int64_t *grads_strides,
                       const void *const *weights, void *const *grad_weights, void *grad_bias,
                       int need_input_grad,
                       void *workspace, int64_t workspace_bytes, void *stream);

/*
 * Final layer of the network: out[b][o][n] = bias[o] + sum_c weight[o][c] * input[b][c][n],
 * the Conv1d(c_in, c_out, 1) over the flattened voxels of MSDFinalLayer
 * (msd_module.py:60-88), which the reference leaves to torch.  `nvox` voxels per channel
 * are contiguous; batch and channel strides are in elements, so `input` can be the dense
 * block's stack as it is.  weight is contiguous (c_out, c_in), bias (c_out) or NULL.
 * msd_final_backward OVERWRITES grad_input (same layout rules; NULL to skip),
 * grad_weight and grad_bias (either may be NULL); the sums over voxels are reduced in a
 * fixed order through `workspace` (msd_final_workspace_bytes); with grad_weight and
 * grad_bias both NULL (a frozen layer) the input is not read (it may be NULL) and no
 * workspace is needed.
 */
int64_t msd_final_workspace_bytes(int dtype, int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox);
int msd_final_forward(int dtype, int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox,
                      const void *input, int64_t input_batch_stride, int64_t input_channel_stride,
                      const void *weight, const void *bias,
                      void *output, int64_t output_batch_stride, int64_t output_channel_stride, void *stream);
int msd_final_backward(int dtype, int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox,
                       const void *input, int64_t input_batch_stride, int64_t input_channel_stride,
                       const void *grad_output, int64_t grad_output_batch_stride, int64_t grad_output_channel_stride,
                       const void *weight,
                       void *grad_input, int64_t grad_input_batch_stride, int64_t grad_input_channel_stride,
                       void *grad_weight, void *grad_bias,
                       void *workspace, int64_t workspace_bytes, void *stream);

/*
 * Final layer, loss and the gradient of the loss in one pass over the stack: what the
 * reference's models run as Conv1d [+ the 1x1 output scaling, folded into weight and bias by
 * the caller] [+ LogSoftmax] + MSELoss / L1Loss / NLLLoss (msd_module.py:60-88,
 * msd_model.py:220-223, msd_regression_model.py:5, msd_segmentation_model.py:61-68), all with
 * the default 'mean' reduction.  c_out <= 8.
 *   output       MSE, L1: bias + weight . input;  NLL: its log-softmax over the output channels
 *   loss         one element of `dtype` in device memory
 *   grad_output  d loss / d (bias + weight . input), same shape as output: handing it to
 *                msd_final_backward (input, grad_weight, grad_bias NULL) gives the gradient of
 *                the stack without reading the stack again
 *   grad_weight, grad_bias   OVERWRITTEN with the layer's parameter gradients (both NULL: skipped)
 * target: MSE, L1: values laid out like output (element strides given); NLL: int64 labels in
 * [0, c_out), one per voxel, target_batch_stride in labels, target_channel_stride ignored.
 * Workspace: msd_final_workspace_bytes.  Sums are reduced in a fixed order.
 */
#define MSD_LOSS_MSE 0
#define MSD_LOSS_L1 1
#define MSD_LOSS_NLL 2
int msd_final_forward_loss(int dtype, int loss_kind, int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox,
                           const void *input, int64_t input_batch_stride, int64_t input_channel_stride,
                           const void *weight, const void *bias,
                           const void *target, int64_t target_batch_stride, int64_t target_channel_stride,
                           void *output, int64_t output_batch_stride, int64_t output_channel_stride,
                           void *grad_output, int64_t grad_output_batch_stride, int64_t grad_output_channel_stride,
                           void *grad_weight, void *grad_bias, void *loss,
                           void *workspace, int64_t workspace_bytes, void *stream);

/*
 * Kernel timing for benchmarks.  While enabled, every operator call is bracketed by
 * HIP events recorded on its launch stream; inside the block calls consecutive launches
 * of one class share one pair of events (a pair per launch would add its own few
 * microseconds of idle stream to every launch).
 * msd_profile_read waits for the recorded events and returns, per class
 * {0 forward, 1 backward_x incl. the mask, 2 backward_k/bias, 3 fused backward_x +
 * backward_k/bias of the block backward pass}, the summed elapsed milliseconds and the
 * number of calls since msd_profile_enable(1); ms and calls hold
 * MSD_PROFILE_CLASSES entries.  Not thread-safe; no counterpart in the reference.
 */
#define MSD_PROFILE_CLASSES 4
int msd_profile_enable(int on);
int msd_profile_read(double *ms, int64_t *calls);

#ifdef __cplusplus
}
#endif
#endif /* MSD_HIP_H */
