/*
 * wtconv_hip.h -- C ABI of libwtconv_hip.so: the WTConv layer (wavelet convolution,
 * Haar/db1) forward and backward as hand-written gfx950 HIP kernels.
 *
 * Conventions (all entry points):
 *   - every pointer except the parameter/gradient tables is DEVICE memory owned by the
 *     caller; the library never allocates, frees or synchronises, and launches on the
 *     HIP stream handed in (`stream`, a hipStream_t passed as void*; NULL = default);
 *   - activations are contiguous NCHW (2-D) / NCL (1-D) in `dtype`; parameters are
 *     contiguous in `param_dtype`; parameter gradients are always written as float.
 *     The three element types are those the reference's fused twin dispatches
 *     (fast_wtconv/cuda_haar/haar_common.cuh:55-77): float, bfloat16 and IEEE half;
 *   - return value 0 on success, a negative WTCONV_E_* code otherwise, with a message
 *     retrievable from wtconv_last_error() on the calling thread;
 *   - `workspace` must hold at least wtconv*_workspace_bytes(...) bytes, 256-byte aligned.
 *
 * This boundary takes the place of the reference's pybind11 extension module
 * (fast_wtconv/cuda_haar/haar.cpp:5-39), whose six functions are likewise
 * caller-allocates / out-parameter style and launch on the current stream.
 */
#ifndef WTCONV_HIP_H
#define WTCONV_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WTCONV_MAX_LEVELS 5
#define WTCONV_ABI_VERSION 5

enum { WTCONV_F32 = 0, WTCONV_BF16 = 1, WTCONV_F16 = 2 };

enum {
  WTCONV_OK = 0,
  WTCONV_E_ARG = -1,        /* bad shape / dtype / null pointer / alignment          */
  WTCONV_E_UNSUPPORTED = -2,/* kernel size or tensor extent beyond the built kernels    */
  WTCONV_E_WORKSPACE = -3,  /* workspace too small                                   */
  WTCONV_E_LAUNCH = -4      /* HIP reported a launch error                           */
};

enum {
  WTCONV_PASS_FORWARD = 0, WTCONV_PASS_BACKWARD_INPUT = 1, WTCONV_PASS_BACKWARD_PARAMS = 2,
  WTCONV_PASS_BACKWARD = 3   /* wtconv*_backward: input and parameter gradients in one call */
};

/* Device pointers to the layer's parameters, in the reference module's own tensor
 * layouts (wtconv/wtconv2d.py:23-31, wtconv/wtconv1d.py:23-31):
 *   base_weight (C,1,K,K) | (C,1,K);  base_bias (C) or NULL;  base_scale C values;
 *   wt_weight[l] (S*C,1,K,K) | (S*C,1,K) and wt_scale[l] S*C values, S = 4 (2-D) or 2 (1-D);
 *   channel S*c+s of level l holds sub-band s (LL,LH,HL,HH | lo,hi) of input channel c
 *   (fast_wtconv/cuda_haar/haar_cuda.py:13). */
typedef struct wtconv_params {
  const void* base_weight;
  const void* base_bias;
  const void* base_scale;
  const void* wt_weight[WTCONV_MAX_LEVELS];
  const void* wt_scale[WTCONV_MAX_LEVELS];
} wtconv_params;

/* Device pointers receiving the parameter gradients (float, same shapes as above).
 * base_bias may be NULL when the layer has no bias. */
typedef struct wtconv_param_grads {
  float* base_weight;
  float* base_bias;
  float* base_scale;
  float* wt_weight[WTCONV_MAX_LEVELS];
  float* wt_scale[WTCONV_MAX_LEVELS];
} wtconv_param_grads;

/* ABI version of the loaded library (== WTCONV_ABI_VERSION). */
int wtconv_abi_version(void);

/* Message of the last failure on this thread ("" if none). */
const char* wtconv_last_error(void);

/* Largest odd kernel size the built kernels cover (cf. HAAR_MAX_K,
 * fast_wtconv/cuda_haar/haar_common.cuh:32-49). */
int wtconv_max_kernel_size(void);

/* ------------------------------------------------------------------ 2-D layer
 * Replaces, as one call each, what the reference composes from
 * wavelet_2d_transform / wavelet_convs / wavelet_scale / inverse_2d_wavelet_transform /
 * base_conv / base_scale (wtconv/wtconv2d.py:38-82) and, in the fast twin,
 * fused_haar_conv_forward + ihaar_cascade + the cuDNN base conv
 * (fast_wtconv/cuda_haar/haar_cuda.py:321-357,635-647).  Stride is not part of the
 * kernels: the caller sub-samples the stride-1 result (wtconv2d.py:84-85). */
size_t wtconv2d_workspace_bytes(int B, int C, int H, int W, int K, int levels, int pass);

int wtconv2d_forward(const void* x, void* out, const wtconv_params* params,
                     int B, int C, int H, int W, int K, int levels,
                     int dtype, int param_dtype,
                     void* workspace, size_t workspace_bytes, void* stream);

/* wtconv2d_forward without a workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  The scratch that wtconv2d_forward
 * takes from `workspace` (folded parameters) lives in a static device array of
 * wtconv_static_scratch_bytes() = 4 MiB that each GPU the library runs on holds until the
 * process ends; shapes whose forward pass needs more (planes too large for LDS, which stage
 * a pyramid in the workspace) are rejected with WTCONV_E_UNSUPPORTED.  The call allocates and
 * frees nothing.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU
 * (two streams, two threads) race; calls on one stream are ordered and safe.  The result is
 * bit-identical to wtconv2d_forward.  The first call on a GPU looks up the address of that GPU's
 * array (hipGetDevice + hipGetSymbolAddress, under a mutex) and must therefore happen outside a
 * stream capture; every later call on that GPU only launches kernels and may be captured. */
size_t wtconv_static_scratch_bytes(void);

int wtconv2d_forward_static(const void* x, void* out, const wtconv_params* params,
                            int B, int C, int H, int W, int K, int levels,
                            int dtype, int param_dtype, void* stream);

/* grad_x from grad_out: replaces autograd through wtconv2d.py:38-82 and
 * WaveletBranchFunction.backward + conv2d_input (haar_cuda.py:359-413,650-656). */
int wtconv2d_backward_input(const void* grad_out, void* grad_x, const wtconv_params* params,
                            int B, int C, int H, int W, int K, int levels,
                            int dtype, int param_dtype,
                            void* workspace, size_t workspace_bytes, void* stream);

/* Gradients of every trainable parameter (deterministic two-stage reduction; no
 * atomics): replaces fused_haar_grad_weight + depthwise_grad_weight and the host
 * algebra around them (haar_cuda.py:168-197,415-421,657-676). */
int wtconv2d_backward_params(const void* x, const void* grad_out, const wtconv_params* params,
                             const wtconv_param_grads* grads,
                             int B, int C, int H, int W, int K, int levels,
                             int dtype, int param_dtype,
                             void* workspace, size_t workspace_bytes, void* stream);

/* The whole backward pass in one call: grad_x and every parameter gradient, as
 * WaveletBranchFunction.backward + ScaledDepthwiseConvFunction.backward produce them in one
 * autograd node each (haar_cuda.py:359-424,650-676).  Same as wtconv2d_backward_input followed
 * by wtconv2d_backward_params on `stream`, sharing `workspace`
 * (wtconv2d_workspace_bytes(..., WTCONV_PASS_BACKWARD) bytes). */
int wtconv2d_backward(const void* x, const void* grad_out, void* grad_x, const wtconv_params* params,
                      const wtconv_param_grads* grads,
                      int B, int C, int H, int W, int K, int levels,
                      int dtype, int param_dtype,
                      void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ 1-D layer
 * Same three calls for wtconv/wtconv1d.py:38-82 (two sub-bands, 1/sqrt(2) butterflies). */
size_t wtconv1d_workspace_bytes(int B, int C, int N, int K, int levels, int pass);

int wtconv1d_forward(const void* x, void* out, const wtconv_params* params,
                     int B, int C, int N, int K, int levels,
                     int dtype, int param_dtype,
                     void* workspace, size_t workspace_bytes, void* stream);

int wtconv1d_backward_input(const void* grad_out, void* grad_x, const wtconv_params* params,
                            int B, int C, int N, int K, int levels,
                            int dtype, int param_dtype,
                            void* workspace, size_t workspace_bytes, void* stream);

int wtconv1d_backward_params(const void* x, const void* grad_out, const wtconv_params* params,
                             const wtconv_param_grads* grads,
                             int B, int C, int N, int K, int levels,
                             int dtype, int param_dtype,
                             void* workspace, size_t workspace_bytes, void* stream);

int wtconv1d_backward(const void* x, const void* grad_out, void* grad_x, const wtconv_params* params,
                      const wtconv_param_grads* grads,
                      int B, int C, int N, int K, int levels,
                      int dtype, int param_dtype,
                      void* workspace, size_t workspace_bytes, void* stream);

/* ---- the passes of a WTConvNeXt block around its WTConv layer, each as one kernel that transposes through LDS.
 * Activations in `dtype` (float or bfloat16), weight / bias / gamma in `param_dtype`; C must be even.
 *
 * wtconv_channel_norm: LayerNorm over the channels of every pixel of x (B, C, HW), biased variance, `eps` inside
 * the square root.  out_nhwc != 0 writes (B, HW, C): the permute to NHWC followed by nn.LayerNorm that the block
 * does after conv_dw (wtconvnext/wtconvnext.py:132-133).  out_nhwc == 0 writes (B, C, HW): the LayerNorm2d of the
 * stem and of the downsample layers (wtconvnext/wtconvnext.py:171, 296).  x and out must not overlap. */
int wtconv_channel_norm(const void* x, void* out, const void* weight, const void* bias, int B, int C, int HW,
                        float eps, int dtype, int param_dtype, int out_nhwc, void* stream);

/* wtconv_block_residual: out (B, C, HW) = shortcut (B, C, HW) + gamma[c] * y, with y (B, HW, C) the NHWC output
 * of the block's MLP: the permute back to NCHW, the layer scale and the residual add of
 * wtconvnext/wtconvnext.py:135-140 (drop_path is the identity at inference).  gamma may be NULL (no layer
 * scale).  out may be the shortcut itself. */
int wtconv_block_residual(const void* y, const void* shortcut, const void* gamma, void* out, int B, int C, int HW,
                          int dtype, int param_dtype, void* stream);

/* ---- the same two passes under autograd (training keeps the block's structure,
 * wtconvnext/wtconvnext.py:125-140; in the reference these gradients come from autograd through
 * permute / nn.LayerNorm / mul / add).  Parameter gradients are written as float; the workspace
 * (wtconv_block_workspace_bytes(...) bytes, 4-byte aligned) takes per-workgroup partial sums that a
 * second small kernel adds up in a fixed order (no atomics). */
size_t wtconv_block_workspace_bytes(int B, int C, int HW, int dtype);

/* Backward of wtconv_channel_norm: x (B, C, HW) is the forward input, dy the gradient of the forward
 * output ((B, HW, C) if dy_nhwc != 0, else (B, C, HW)); writes dx (B, C, HW), dweight (C), dbias (C). */
int wtconv_channel_norm_backward(const void* x, const void* dy, const void* weight, void* dx, float* dweight,
                                 float* dbias, int B, int C, int HW, float eps, int dtype, int param_dtype,
                                 int dy_nhwc, void* workspace, size_t workspace_bytes, void* stream);

/* Backward of wtconv_block_residual with a layer scale: dout (B, C, HW) is the gradient of the block's
 * output (the shortcut's gradient is dout itself), y (B, HW, C) the forward's NHWC input; writes
 * dy (B, HW, C) = gamma[c] * dout and dgamma (C) = sum dout * y. */
int wtconv_block_residual_backward(const void* dout, const void* y, const void* gamma, void* dy, float* dgamma,
                                   int B, int C, int HW, int dtype, int param_dtype, void* workspace,
                                   size_t workspace_bytes, void* stream);

/* ---- single-level Haar (db1) transforms as operators of their own: wavelet_2d_transform /
 * inverse_2d_wavelet_transform and their 1-D twins with the db1 bank (wtconv/util/wavelet.py:46-75; the fast
 * twin's haar2d / ihaar2d utilities, fast_wtconv/cuda_haar/__init__.py:52-55).  Even extents only (the reference
 * pads before it calls them, wtconv2d.py:49-51).
 *   wtconv_haar2d, inverse == 0: x (planes, H, W) -> out (planes, 4, H/2, W/2), sub-bands LL, LH, HL, HH;
 *                  inverse != 0: x (planes, 4, H/2, W/2) -> out (planes, H, W).
 *   wtconv_haar1d, inverse == 0: x (rows, N) -> out (rows, 2, N/2), lo then hi; inverse != 0 the other way. */
int wtconv_haar2d(const void* x, void* out, long long planes, int H, int W, int dtype, int inverse, void* stream);
int wtconv_haar1d(const void* x, void* out, long long rows, int N, int dtype, int inverse, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* WTCONV_HIP_H */
