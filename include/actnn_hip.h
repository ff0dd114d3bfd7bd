/*
 * actnn_hip.h - C ABI of the MI355X (gfx950) activation-compression kernels.
 *
 * Every entry point is `extern "C"`, takes plain pointers and sizes, launches on the HIP
 * stream it is given (`stream` is a hipStream_t passed as void*; NULL = the null stream)
 * and returns 0 on success, a negative ACTNN_E* code for a rejected argument, or a
 * positive hipError_t when a launch failed.  Nothing throws and nothing allocates: all
 * outputs are caller-allocated device buffers.  Unless noted, pointers are device
 * pointers, tensors are contiguous, and `dtype` is one of ACTNN_F32 / ACTNN_F16 /
 * ACTNN_BF16 (bf16 is an extension: the reference accepts f32 and f16 only,
 * actnn/actnn/cpp_extension/ext_common.h:15-19).
 *
 * Each declaration cites the reference interface it replaces (paths relative to the
 * reference tree, actnn/actnn/cpp_extension/).
 */
#ifndef ACTNN_HIP_H_
#define ACTNN_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ACTNN_F32 = 0, ACTNN_F16 = 1, ACTNN_BF16 = 2 };

enum {
  ACTNN_OK = 0,
  ACTNN_EINVAL = -1,   /* bad size / null pointer / unsupported combination */
  ACTNN_EDTYPE = -2,   /* unknown dtype */
  ACTNN_EBITS = -3,    /* bit width outside what the operator supports */
  ACTNN_EALIGN = -4,   /* pointer not aligned as the kernel requires (16 bytes) */
  ACTNN_ETOOBIG = -5   /* problem needs more scratch memory than the library's fixed buffer holds */
};

/* Human-readable text for a return code of this library (static storage). */
const char* actnn_strerror(int code);

/* Version string of the library (static storage). */
const char* actnn_version(void);

/* ---------------------------------------------------------------------------------
 * minimax: per-row minimum and maximum of data[M, D] -> mn[M], mx[M] (same dtype).
 * Replaces minimax(Tensor) -> (min, max): minimax.cc:7-11, minimax_cuda_kernel.cu:70-89.
 * Any D >= 1 is accepted (the reference requires D % 32 == 0 && D > 32).
 * ------------------------------------------------------------------------------- */
int actnn_minimax(const void* data, void* mn, void* mx, int64_t M, int64_t D, int dtype,
                  void* stream);

/* ---------------------------------------------------------------------------------
 * Per-sample sensitivity of the bit allocation from the group ranges:
 *   out[n] = factor * mult * sum_g (mx[n, g] - mn[n, g])^2        (out: fp32[N], device)
 * mult: NULL, one fp32 device scalar (mult_per_sample == 0) or fp32[N] (mult_per_sample != 0).
 * Replaces the chain of tensor ops behind Range_sqr and C in QScheme.compute_quantization_bits,
 * actnn/actnn/qscheme.py:80-82 (norm over the groups of a sample, squared, scaled by
 * group_size / num_pixels, by num_locations / 4 / depthwise_groups and by the gradient scale);
 * the squared norm is accumulated directly in fp32.
 * ------------------------------------------------------------------------------- */
int actnn_range_sqr(const void* mn, const void* mx, float* out, int64_t N, int64_t G, float factor,
                    const float* mult, int mult_per_sample, int dtype, void* stream);

/* Exclusive prefix sum of the per-sample bit widths: prefix[0] = 0,
 * prefix[n] = bits[0] + ... + bits[n-1], prefix has N + 1 entries.
 * Replaces the torch::cumsum calls at quantization_cuda_kernel.cu:97 and :182. */
int actnn_bits_prefix(const int32_t* bits, int32_t* prefix, int64_t N, void* stream);

/* ---------------------------------------------------------------------------------
 * pack_mixed_precision: quantise data[N, G, gs] with bits[n] in 1..8 bits per sample and
 * write the int32 bit stream `packed` (ceil(sum(bits) * G * gs / 32) words, reference
 * layout) and scale[N, G, 1] (dtype of data).
 * Replaces pack_mixed_precision(data, min, max, bits, stochastic) -> (packed, scale):
 * quantization.cc:46-57, quantization_cuda_kernel.cu:83-142.
 *   noise == NULL: in-kernel Philox4x32-10 stochastic rounding keyed by (seed, offset),
 *                  arithmetic of the reference's CUDA kernel (:32, :65).
 *   noise != NULL: deterministic mode. noise[N, G, gs] (dtype of data) holds U(-0.5, 0.5)
 *                  values; codes and scale are bit-identical to the reference's
 *                  config.simulate quantiser (actnn/actnn/ops.py:23-41) fed the same noise.
 * gs must be a multiple of 32 and at most 1024.  prefix comes from actnn_bits_prefix.
 * ------------------------------------------------------------------------------- */
int actnn_pack_mixed(const void* data, const void* mn, const void* mx, const int32_t* bits,
                     const int32_t* prefix, void* scale, int32_t* packed, const void* noise,
                     uint64_t seed, uint64_t offset, int64_t N, int64_t G, int64_t gs,
                     int dtype, void* stream);

/* unpack_mixed_precision: out[N, G, gs] = code / scale + min (dtype = dtype of scale).
 * Replaces unpack_mixed_precision(data, bits, scale, min, N, num_groups, group_size):
 * quantization.cc:59-73, quantization_cuda_kernel.cu:145-205. */
int actnn_unpack_mixed(const int32_t* packed, const int32_t* bits, const int32_t* prefix,
                       const void* scale, const void* mn, void* out, int64_t N, int64_t G,
                       int64_t gs, int dtype, void* stream);

/* ---------------------------------------------------------------------------------
 * pack_single_precision: one bit width (1, 2, 4 or 8) for the whole tensor; 8/bits
 * consecutive samples share a byte.  packed has (bits * N_round * G * gs + 8) / 8 bytes,
 * N_round = N rounded up to a multiple of 8/bits.
 * Replaces pack_single_precision(data, min, max, bits, stochastic) -> (packed, scale):
 * quantization.cc:77-87, quantization_cuda_kernel.cu:261-330.  noise as above.
 * ------------------------------------------------------------------------------- */
int actnn_pack_single(const void* data, const void* mn, const void* mx, int bits, void* scale,
                      int8_t* packed, const void* noise, uint64_t seed, uint64_t offset,
                      int64_t N, int64_t G, int64_t gs, int dtype, void* stream);

/* Replaces unpack_single_precision(data, bits, scale, min, N, num_groups, group_size):
 * quantization.cc:89-102, quantization_cuda_kernel.cu:364-405. */
int actnn_unpack_single(const int8_t* packed, int bits, const void* scale, const void* mn,
                        void* out, int64_t N, int64_t G, int64_t gs, int dtype, void* stream);

/* ---------------------------------------------------------------------------------
 * ReLU with a 1-bit mask.  mask holds 16 int32 words per block of 512 elements,
 * i.e. ceil(n / 512) * 16 words (equal to the reference's ceil(n / 32) whenever
 * n % 512 == 0; the reference's tail block writes past its shorter allocation).
 * Replaces act_quantized_relu_forward_cuda / _backward_cuda:
 * quantization_cuda_kernel.cu:446-467, :490-508 (quantization.cc:106-124).
 * ------------------------------------------------------------------------------- */
int actnn_relu_forward(const void* x, void* y, int32_t* mask, int64_t n, int dtype, void* stream);
/* ReLU forward that also writes the per-group minimum and maximum of its OUTPUT (groups of 256
 * consecutive elements; mn/mx[n / 256] in `dtype`) - what actnn_minimax returns for y viewed as
 * rows of 256 - so that a layer which quantises y next need not read it again.  16-bit dtypes,
 * n a multiple of 2048. */
int actnn_relu_forward_minmax(const void* x, void* y, int32_t* mask, void* mn, void* mx, int64_t n,
                              int dtype, void* stream);
/* y = relu(x + residual) in one pass over the two operands, with the same mask: the sum is
 * rounded to `dtype` as the tensor addition rounds it, so y and mask equal those of the addition
 * followed by actnn_relu_forward.  For the closing `out += identity; out = relu(out)` of a residual
 * block of the model the reference benchmarks (torchvision's resnet50,
 * mem_speed_benchmark/train.py:203-206; the ReLU is quantization.cc:106-124).  mn / mx: both
 * null, or as in actnn_relu_forward_minmax (16-bit dtypes, n a multiple of 2048).  The gradient of
 * both operands is actnn_relu_backward's. */
int actnn_relu_add_forward(const void* x, const void* residual, void* y, int32_t* mask, void* mn,
                           void* mx, int64_t n, int dtype, void* stream);
int actnn_relu_backward(const void* grad_out, const int32_t* mask, void* grad_in, int64_t n,
                        int dtype, void* stream);
/* grad_in = other + actnn_relu_backward(grad_out, mask), in one pass: the sum rounded to `dtype` as
 * the tensor addition of the two rounds it.  For the input of a residual block, whose gradient is
 * the one from the block's first convolution plus the masked gradient that arrives over the skip
 * connection (autograd's accumulation after quantization.cc:117-119 in the reference). */
int actnn_relu_backward_add(const void* grad_out, const int32_t* mask, const void* other, void* grad_in,
                            int64_t n, int dtype, void* stream);

/* Dropout with a 1-bit keep mask (same mask layout as ReLU); y = keep ? x / (1 - p) : 0.
 * keep is drawn from the Philox stream (seed, offset) with probability 1 - p (16-bit
 * resolution).  Replaces act_quantized_dropout_forward_cuda / _backward_cuda:
 * quantization_cuda_kernel.cu:555-585, :609-627 (quantization.cc:128-148). */
int actnn_dropout_forward(const void* x, void* y, int32_t* mask, int64_t n, float p,
                          uint64_t seed, uint64_t offset, int dtype, void* stream);
int actnn_dropout_backward(const void* grad_out, const int32_t* mask, void* grad_in, int64_t n,
                           float p, int dtype, void* stream);

/* ---------------------------------------------------------------------------------
 * MaxPool2d keeping the arg-max position inside the window as one int8 per output
 * element (kh * KW + kw relative to the unclipped window origin; first strict maximum).
 * KH * KW must be < 16.  Dilation only enters through Ho/Wo, which the caller computes
 * (quantization_cuda_kernel.cu:679-680); the window itself is undilated, as in the
 * reference (:649-654).  The backward is a deterministic gather (the reference scatters
 * with atomicAdd into a zeroed tensor, :723).
 * Replaces act_quantized_max_pool2d_forward_cuda / _backward_cuda:
 * quantization_cuda_kernel.cu:672-700, :727-754 (quantization.cc:152-196).
 * ------------------------------------------------------------------------------- */
int actnn_max_pool2d_forward(const void* x, void* y, int8_t* idx, int64_t N, int64_t C,
                             int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH, int KW,
                             int SH, int SW, int PH, int PW, int dtype, void* stream);
int actnn_max_pool2d_backward(const void* grad_out, const int8_t* idx, void* grad_in, int64_t N,
                              int64_t C, int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH,
                              int KW, int SH, int SW, int PH, int PW, int dtype, void* stream);
/* The same two operators on channels-last tensors: x, y, idx and the gradients are laid out
 * [N, H, W, C] / [N, Ho, Wo, C] (C a multiple of 4 for f32, 8 for 16-bit types; x, y and the
 * gradients 16-byte aligned; idx aligned to the indices of one 16-byte chunk of channels: 4 bytes
 * for f32, 8 bytes for 16-bit types - half of that for the two-per-byte format below;
 * ACTNN_EALIGN otherwise).  Values and indices equal those of the default-layout operators on the
 * transposed tensors. */
int actnn_max_pool2d_forward_cl(const void* x, void* y, int8_t* idx, int64_t N, int64_t C,
                                int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH, int KW,
                                int SH, int SW, int PH, int PW, int dtype, void* stream);
int actnn_max_pool2d_backward_cl(const void* grad_out, const int8_t* idx, void* grad_in, int64_t N,
                                 int64_t C, int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH,
                                 int KW, int SH, int SW, int PH, int PW, int dtype, void* stream);
/* The same four operators with the indices kept two per byte.  No counterpart in the reference,
 * which keeps one int8 per output although it already requires KH * KW < 16
 * (quantization.cc:162): output o of the flat order of y (default layout: [N, C, Ho, Wo];
 * channels-last: [N, Ho, Wo, C]) is stored in bits 4 * (o & 1) .. 4 * (o & 1) + 3 of byte
 * o / 2; idx holds (N * C * Ho * Wo + 1) / 2 bytes and the unused half of the last byte of an
 * odd count is written as 0.  Values, indices and gradients equal those of the int8 operators.
 * Default layout: idx needs no alignment (16-byte aligned pointers take the faster kernels);
 * channels-last: 2 bytes for f32, 4 bytes for 16-bit types. */
int actnn_max_pool2d_forward_nibble(const void* x, void* y, uint8_t* idx, int64_t N, int64_t C,
                                    int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH, int KW,
                                    int SH, int SW, int PH, int PW, int dtype, void* stream);
int actnn_max_pool2d_backward_nibble(const void* grad_out, const uint8_t* idx, void* grad_in, int64_t N,
                                     int64_t C, int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH,
                                     int KW, int SH, int SW, int PH, int PW, int dtype, void* stream);
int actnn_max_pool2d_forward_cl_nibble(const void* x, void* y, uint8_t* idx, int64_t N, int64_t C,
                                       int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH, int KW,
                                       int SH, int SW, int PH, int PW, int dtype, void* stream);
int actnn_max_pool2d_backward_cl_nibble(const void* grad_out, const uint8_t* idx, void* grad_in, int64_t N,
                                        int64_t C, int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH,
                                        int KW, int SH, int SW, int PH, int PW, int dtype, void* stream);

/* ---------------------------------------------------------------------------------
 * calc_precision (HOST pointers): greedy bit allocation, mutates b in place.
 * Replaces calc_precision(b, C, w, target): calc_precision.cc:9-50.
 * ------------------------------------------------------------------------------- */
int actnn_calc_precision(int32_t* b, const float* C, const int32_t* w, int64_t N, double target);

/* calc_precision_dp (HOST pointers): widths b_i in 1..max_b and keep probabilities p_i in
 * {1/states..1} minimising sum (1-p_i)/p_i*A_i + C_i/(p_i*(2^b_i-1)^2) with
 * sum b_i*p_i*states == target*N*states, by dynamic programming; b_out, p_out: fp32[N].
 * ACTNN_EINVAL when no assignment meets the budget (the reference raises "DP Failed").
 * Replaces calc_precision_dp(A, C, max_b, target, states): calc_precision.cc:58-125. */
int actnn_calc_precision_dp(const float* A, const float* C, int64_t N, int max_b, int target,
                            int states, float* b_out, float* p_out);

/* Squared L2 norm per sample of x[N, F] (the per-sample gradient statistic of the bit allocation,
 * qscheme.py:47-55, where the reference chains square / sum over a full-size temporary):
 * part[n * slices + b] = sum of squares of slice b of row n (fp32, fixed order); the caller adds the
 * `slices` values of a row.  F a multiple of 4 (f32) or 8 (16-bit types), N <= 65535, x 16-byte aligned. */
int actnn_sample_sqnorm(const void* x, float* part, int64_t N, int64_t F, int slices, int dtype,
                        void* stream);

/* Same allocation on the DEVICE for the case every layer uses at every step: all N items start
 * at initial_bits (1..8) with weight 1 and `target` is the bit budget, so exactly
 * N * initial_bits - target widths are taken away (clamped to [0, N * (initial_bits - 1)]).
 * C: fp32[N] device, bits: int32[N] device (output).  Bit-identical to actnn_calc_precision on
 * the same inputs; N * (initial_bits - 1) <= 8192, otherwise ACTNN_EINVAL (use the host routine).
 * Replaces the device -> host -> device round trip of qscheme.py:83-94. */
int actnn_calc_precision_device(const float* C, int32_t* bits, int64_t N, int initial_bits,
                                int64_t target, void* stream);

/* actnn_range_sqr, actnn_calc_precision_device and actnn_bits_prefix back to back on `stream`, for
 * the per-layer allocation of qscheme.py:76-94 in one call: sensitivity[N] (fp32), bits[N],
 * prefix[N + 1].  Arguments and limits as for the three calls. */
int actnn_allocate_bits_device(const void* mn, const void* mx, float factor, const float* mult,
                               int mult_per_sample, float* sensitivity, int32_t* bits,
                               int32_t* prefix, int64_t N, int64_t G, int initial_bits,
                               int64_t target, int dtype, void* stream);

/* actnn_batch_norm_forward_apply (with bits) with the ReLU that follows the batch norm folded into
 * the pass: y = relu(bn(x)), relu_mask and relu_mn / relu_mx[N * C * HW / 256] are what
 * actnn_relu_forward_minmax makes of the stored bn(x) (the normalised value is rounded to `dtype`
 * before the rule is applied), bn(x) itself is never written; scale and the packed copy of x as in
 * _apply.  One pass over x instead of a pass over x and a pass over bn(x) (torchvision's
 * `relu(bn(conv(x)))`, mem_speed_benchmark/train.py:203-206; ops.py:436-470 and
 * quantization.cc:106-124 in the reference).  Channels-last 16-bit tensors with C a divisor of 256
 * or a multiple of 512 and N * HW a multiple of 2048 / min(C, 256) (a wave's 64 chunks are then one
 * 512-element block of the mask, or the same half of two); everything else is ACTNN_EINVAL /
 * ACTNN_EDTYPE.  `residual` (null, or a tensor laid out like x): y = relu(bn(x) + residual), the
 * closing step of a residual block - bn(x) rounded to `dtype` as its store would round it, the sum
 * rounded as the tensor addition rounds it, so y and the mask equal those of the three separate
 * operators. */
int actnn_batch_norm_forward_apply_relu(const void* x, void* y, const void* workspace,
                                        int64_t workspace_bytes, const int32_t* bits,
                                        const int32_t* prefix, const void* mn, const void* mx, void* scale,
                                        int32_t* packed, uint64_t seed, uint64_t offset, int32_t* relu_mask,
                                        void* relu_mn, void* relu_mx, const void* residual, int64_t N,
                                        int64_t C, int64_t HW, int dtype, int channels_last, void* stream);

/* A layer's forward-side sequence in one call (the host layer's glue between the steps - Python
 * here, the Function bodies of actnn/actnn/ops.py:99-118 and :436-470 in the reference - costs more
 * than the kernels at small batch sizes).  Same kernels, same results, arguments as in the calls
 * they stand for:
 *   actnn_batch_norm_forward_quantize = actnn_batch_norm_forward_stats (with mn / mx)
 *       -> actnn_allocate_bits_device (G = C * HW / 256) -> actnn_batch_norm_forward_apply (with bits),
 *       or, with relu_mask / relu_mn / relu_mx given (all three; `residual` optional),
 *       -> actnn_batch_norm_forward_apply_relu;
 *   actnn_quantize_activation = [actnn_minimax of data as rows of 256 unless minmax_known]
 *       -> actnn_allocate_bits_device -> actnn_pack_mixed (gs = 256, in-kernel Philox mode).
 * Every output pointer is required. */
int actnn_batch_norm_forward_quantize(
    const void* x, const float* weight, const float* bias, float* running_mean, float* running_var, void* y,
    float* save_mean, float* save_invstd, void* mn, void* mx, void* workspace, int64_t workspace_bytes,
    float factor, const float* mult, int mult_per_sample, float* sensitivity, int32_t* bits, int32_t* prefix,
    int initial_bits, int64_t target, void* scale, int32_t* packed, uint64_t seed, uint64_t offset,
    int32_t* relu_mask, void* relu_mn, void* relu_mx, const void* residual, int64_t N, int64_t C, int64_t HW,
    double momentum, double eps, int dtype, int channels_last, void* stream);
int actnn_quantize_activation(const void* data, void* mn, void* mx, int minmax_known, float factor,
                              const float* mult, int mult_per_sample, float* sensitivity, int32_t* bits,
                              int32_t* prefix, int initial_bits, int64_t target, void* scale, int32_t* packed,
                              uint64_t seed, uint64_t offset, int64_t N, int64_t G, int dtype, void* stream);

/* ---------------------------------------------------------------------------------
 * Fused QLinear weight gradient: grad_w[O, I] = grad_out[M, O]^T @ dequant(x)[M, I] where x is
 * held as a stream of this library with scale/min[M, I/256, 1] (groups of 256 along a row):
 *   bits == NULL: the fixed-width stream of actnn_pack_single at `fixed_bits` (1, 2, 4 or 8);
 *   bits != NULL: the mixed-width stream of actnn_pack_mixed with bits[M] and prefix[M + 1]
 *                 (fixed_bits ignored) - what QScheme hands linear.backward at the default level.
 * The tile is unpacked and dequantised (code / scale + min, rounded as the unpack kernels round)
 * to the 16-bit format of grad_out inside the LDS loader of an MFMA GEMM (fp32 accumulation); the
 * full-precision input is never written to memory.  Replaces dequantize_activation +
 * grad_output.t().mm(input) in linear.backward, actnn/actnn/ops.py:407-421.
 * grad_out dtype: f16 or bf16; scale/min dtype = sm_dtype; grad_w dtype = out_dtype
 * (f32, f16 or bf16).  I % 256 == 0, O % 8 == 0; grad_out and grad_w 16-byte, packed 8-byte,
 * scale and min 4-byte aligned.  The 2-bit fixed-width stream takes the fast loader.
 * actnn_linear_grad_weight_q2 is the 2-bit fixed-width case with M % 4 == 0.
 * ------------------------------------------------------------------------------- */
int actnn_linear_grad_weight(const void* grad_out, const void* packed, const int32_t* bits,
                             const int32_t* prefix, int fixed_bits, const void* scale, const void* mn,
                             void* grad_w, int64_t M, int64_t O, int64_t I, int go_dtype,
                             int sm_dtype, int out_dtype, void* stream);
/* The same with a workspace for shapes whose few output tiles (256 x 256) would leave most of the
 * chip idle: the sum over the M samples is then split over several blocks per tile, their fp32
 * partial tiles go to `workspace` and a second kernel adds them in a fixed order (reproducible).
 * actnn_linear_grad_weight_workspace_bytes says how much such a shape needs (0: the plain kernel
 * is used and `workspace` may be null); with less than that the call runs unsplit, as
 * actnn_linear_grad_weight always does.  workspace 16-byte aligned.  The reference's cuBLAS mm
 * (ops.py:421) picks its own split the same way. */
int64_t actnn_linear_grad_weight_workspace_bytes(int64_t M, int64_t O, int64_t I);
int actnn_linear_grad_weight_ws(const void* grad_out, const void* packed, const int32_t* bits,
                                const int32_t* prefix, int fixed_bits, const void* scale,
                                const void* mn, void* grad_w, int64_t M, int64_t O, int64_t I,
                                int go_dtype, int sm_dtype, int out_dtype, void* workspace,
                                int64_t workspace_bytes, void* stream);
int actnn_linear_grad_weight_q2(const void* grad_out, const int8_t* packed, const void* scale,
                                const void* mn, void* grad_w, int64_t M, int64_t O, int64_t I,
                                int go_dtype, int sm_dtype, int out_dtype, void* stream);

/* ---------------------------------------------------------------------------------
 * Training-mode batch normalisation over a dense tensor of N samples, C channels and HW
 * positions, laid out [N, C, HW] (channels_last = 0) or [N, HW, C] (channels_last = 1, the
 * layout of this GPU's convolution kernels).
 * Replaces the two cuDNN calls the reference re-exports, at::cudnn_batch_norm and
 * at::cudnn_batch_norm_backward (cpp_extension/backward_func.cc:87-88; callers ops.py:448-449
 * and ops.py:479-481).  weight/bias (may be null = 1/0), running_* (may be null), save_* and
 * the gradients of weight/bias are fp32[C]; x, y, dy, dx are `dtype`.
 * forward: batch mean and biased variance per channel, y = (x - mean) * invstd * weight + bias,
 * running_mean/var updated in place with `momentum` (variance unbiased), save_mean/save_invstd
 * written.  When mn/mx are given (both or neither; needs C*HW % 256 == 0, and for channels_last
 * C % 256 == 0 or 256 % C == 0) the per-group minimum
 * and maximum of x over groups of 256 consecutive elements of a sample - what actnn_minimax
 * returns for x viewed as [N*C*HW/256, 256] - are written as well, from the same read of x.
 * backward: dx, dweight, dbias from x, dy and the saved statistics (dx may be null).
 * `workspace`: device scratch of actnn_batch_norm_workspace_bytes(...) bytes (16-byte aligned;
 * -1 = shape not supported), contents undefined before and after.
 * Shapes: every dense [N, C, HW] / [N, HW, C] tensor is taken.  Rows of whole 16-byte chunks
 * (C*HW a multiple of 4 for f32, 8 for 16-bit types, HW at least that; channels_last: C such a
 * multiple) take the streaming kernels; [N, C] inputs (HW = 1) are the channels-last layout
 * with one pixel per sample and take its kernels whatever `channels_last` says; anything else
 * goes element by element (correct, a fraction of the speed, no group min/max, no sumsq).
 * actnn_batch_norm_groups_align: 1 when the quantiser's groups of 256 coincide with runs of
 * threads of the streaming kernels, i.e. when mn/mx, the packed copy of _forward_apply and
 * _backward_packed are available for the shape.
 * ------------------------------------------------------------------------------- */
int64_t actnn_batch_norm_workspace_bytes(int64_t N, int64_t C, int64_t HW, int dtype,
                                         int channels_last);
int actnn_batch_norm_groups_align(int64_t N, int64_t C, int64_t HW, int dtype, int channels_last);
/* Evaluation mode (training = false in the reference's batch_norm Function, ops.py:458-461 and
 * :495-499, which calls at::native_batch_norm / _backward there, backward_func.cc:89-90): the
 * running estimates are the statistics.  forward_eval: y = (x - running_mean) / sqrt(running_var +
 * eps) * weight + bias; save_mean / save_invstd (may be null) receive running_mean and
 * 1 / sqrt(running_var + eps) for the backward call.  backward_eval: dx = dy * weight * invstd
 * (dx may be null), dweight = sum(dy * (x - mean) * invstd), dbias = sum(dy). */
int actnn_batch_norm_forward_eval(const void* x, const float* weight, const float* bias,
                                  const float* running_mean, const float* running_var, void* y,
                                  float* save_mean, float* save_invstd, void* workspace,
                                  int64_t workspace_bytes, int64_t N, int64_t C, int64_t HW, double eps,
                                  int dtype, int channels_last, void* stream);
int actnn_batch_norm_backward_eval(const void* x, const void* dy, const float* weight,
                                   const float* mean, const float* invstd, void* dx, float* dweight,
                                   float* dbias, void* workspace, int64_t workspace_bytes, int64_t N,
                                   int64_t C, int64_t HW, int dtype, int channels_last, void* stream);
int actnn_batch_norm_forward(const void* x, const float* weight, const float* bias,
                             float* running_mean, float* running_var, void* y, float* save_mean,
                             float* save_invstd, void* mn, void* mx, void* workspace,
                             int64_t workspace_bytes, int64_t N, int64_t C, int64_t HW,
                             double momentum, double eps, int dtype, int channels_last,
                             void* stream);
int actnn_batch_norm_backward(const void* x, const void* dy, const float* weight,
                              const float* save_mean, const float* save_invstd, void* dx,
                              float* dweight, float* dbias, void* workspace,
                              int64_t workspace_bytes, float* sumsq, int64_t sumsq_entries,
                              int64_t N, int64_t C, int64_t HW, int dtype, int channels_last,
                              void* stream);
/* `sumsq` (may be null) of the two backward entry points: a table of
 * actnn_batch_norm_backward_sumsq_entries(...) floats that receives partial sums of dx^2 (the values
 * as stored in dx); their total is the squared norm of the gradient the preceding layer receives -
 * the statistic of qscheme.py:47-55 - without another pass over dx. */
int64_t actnn_batch_norm_backward_sumsq_entries(int64_t N, int64_t C, int64_t HW, int dtype,
                                                int channels_last);

/* actnn_batch_norm_forward without the workspace arguments, for callers that cannot allocate
 * device memory and have no workspace to pass: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  The partial sums and
 * coefficients live in a fixed device array inside the library (one copy per GPU, held until the
 * process ends) of actnn_batch_norm_forward_static_limit() bytes (16 MiB: ResNet-50's batch norms up
 * to batch 1024 in either layout need at most 8.4 MB); a shape whose
 * actnn_batch_norm_workspace_bytes exceeds it is rejected with ACTNN_ETOOBIG.  Calls no hipMalloc,
 * hipFree or other allocating routine.  Results are bit-identical to actnn_batch_norm_forward.
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different
 * streams or threads) race; calls on one stream are ordered and safe.  `stream` must belong to the
 * current device (ACTNN_EINVAL otherwise: the array is looked up on the current device).
 * actnn_batch_norm_forward_static_limit() doubles as the set-up call: it resolves the array's
 * address on the current device (hipGetSymbolAddress, once per device); call it once per GPU, with
 * that GPU current, before the first forward call that runs under graph capture - a forward call on
 * a device that was not set up resolves the address itself, outside capture only. */
int64_t actnn_batch_norm_forward_static_limit(void);
int actnn_batch_norm_forward_static(const void* x, const float* weight, const float* bias,
                                    float* running_mean, float* running_var, void* y,
                                    float* save_mean, float* save_invstd, void* mn, void* mx,
                                    int64_t N, int64_t C, int64_t HW, double momentum, double eps,
                                    int dtype, int channels_last, void* stream);

/* The forward pass in two steps, for callers that want the quantiser's output from the same read
 * of x: _stats runs the statistics pass (save_mean/save_invstd, running estimates, optional group
 * min/max) and leaves the per-channel coefficients in `workspace`; the caller may then derive the
 * per-sample bit widths from mn/mx; _apply writes y from x and the same workspace and, when `bits`
 * is given (any dtype, the alignment conditions of mn/mx), also scale[N*G] and the packed
 * stream - bit for bit what actnn_pack_mixed(x, mn, mx, bits, prefix, ..., seed, offset) writes in
 * its in-kernel Philox mode.  actnn_batch_norm_forward is _stats followed by _apply without bits. */
int actnn_batch_norm_forward_stats(const void* x, const float* weight, const float* bias,
                                   float* running_mean, float* running_var, float* save_mean,
                                   float* save_invstd, void* mn, void* mx, void* workspace,
                                   int64_t workspace_bytes, int64_t N, int64_t C, int64_t HW,
                                   double momentum, double eps, int dtype, int channels_last,
                                   void* stream);
int actnn_batch_norm_forward_apply(const void* x, void* y, const void* workspace,
                                   int64_t workspace_bytes, const int32_t* bits,
                                   const int32_t* prefix, const void* mn, const void* mx, void* scale,
                                   int32_t* packed, uint64_t seed, uint64_t offset, int64_t N,
                                   int64_t C, int64_t HW, int dtype, int channels_last, void* stream);

/* The same backward pass with x held as the mixed-precision stream of actnn_pack_mixed (group
 * size 256 over the sample in memory order, the conditions of mn/mx above, any dtype with scale / mn
 * in that dtype; bits / prefix / scale / mn as for actnn_unpack_mixed):
 * both passes rebuild x in registers, bit for bit what actnn_unpack_mixed would write, so the
 * full-precision copy of x that ops.py:478 (dequantize_activation before
 * cudnn_batch_norm_backward) materialises never exists. */
int actnn_batch_norm_backward_packed(const int32_t* packed, const int32_t* bits,
                                     const int32_t* prefix, const void* scale, const void* mn,
                                     const void* dy, const float* weight, const float* save_mean,
                                     const float* save_invstd, void* dx, float* dweight,
                                     float* dbias, void* workspace, int64_t workspace_bytes,
                                     float* sumsq, int64_t sumsq_entries, int64_t N, int64_t C,
                                     int64_t HW, int dtype, int channels_last, void* stream);
/* The same for a batch norm whose output went through a ReLU (actnn_batch_norm_forward_apply_relu):
 * grad_out is the gradient of the ReLU's output and relu_mask the ReLU's mask; both passes zero what
 * actnn_relu_backward would have zeroed as they read, so the masked gradient is never written and
 * the results equal actnn_relu_backward followed by actnn_batch_norm_backward_packed bit for bit.
 * Shapes as actnn_batch_norm_forward_apply_relu takes them (replaces the same reference lines as
 * the two calls: quantization.cc:106-124, ops.py:472-502). */
int actnn_batch_norm_backward_packed_relu(const int32_t* packed, const int32_t* bits, const int32_t* prefix,
                                          const void* scale, const void* mn, const void* grad_out,
                                          const int32_t* relu_mask, const float* weight,
                                          const float* save_mean, const float* save_invstd, void* dx,
                                          float* dweight, float* dbias, void* workspace,
                                          int64_t workspace_bytes, float* sumsq, int64_t sumsq_entries,
                                          int64_t N, int64_t C, int64_t HW, int dtype, int channels_last,
                                          void* stream);

/* Plain device-to-device streaming copy of `bytes` bytes (16-byte aligned pointers and
 * size); used by the benchmark to calibrate bandwidth counters.  No reference counterpart. */
int actnn_stream_copy(const void* src, void* dst, int64_t bytes, void* stream);

/* What the matrix pipes alone sustain on given operand data; used by the benchmark to price the
 * fused weight-gradient GEMM against the rate the part reaches with the same operand statistics.
 * `blocks` blocks of 256 threads (one wave per SIMD) each load 8 fragments of 16 bytes per thread
 * from operands[blocks][8][256] (16 bytes each, bf16 values) and issue 16 * kblocks
 * v_mfma_f32_32x32x16_bf16 per wave on them (2 * 32 * 32 * 16 flop each); out[blocks * 256]
 * receives a checksum.  No reference counterpart. */
int actnn_matrix_pipe_probe(const void* operands, float* out, int blocks, int kblocks, void* stream);

#ifdef __cplusplus
}
#endif
#endif  /* ACTNN_HIP_H_ */
