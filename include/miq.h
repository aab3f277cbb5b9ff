/*
 * libmiq -- C ABI of the MI355X (gfx950) quantization-simulation kernels.
 *
 * Every entry point takes plain pointers and sizes (device pointers unless a parameter says "host"), an explicit
 * `void* stream` (a hipStream_t; NULL = the default stream) and returns an int status: MIQ_OK (0) or a negative
 * MIQ_ERR_* code, in which case miq_last_error() holds a message for the calling thread.  Nothing throws across
 * this boundary.  Kernels are enqueued asynchronously on `stream`; the caller owns every buffer and keeps it alive
 * until the stream has passed the call.  In-place operation (out == in) is allowed for every elementwise call.
 * Element counts are 64-bit.
 *
 * Each declaration names the reference interface it replaces (paths relative to the reference root;
 * DLQ = ModelOptimizations/DlQuantization, TSRC = TrainingExtensions/torch/src,
 * TORCH = TrainingExtensions/torch/src/python/aimet_torch).
 */
#ifndef MIQ_H
#define MIQ_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MIQ_OK 0
#define MIQ_ERR_INVALID_ARG (-1)
#define MIQ_ERR_HIP (-2)
#define MIQ_ERR_UNSUPPORTED (-3)

/* DLQ/include/DlQuantization/Quantization.hpp:145-149 (RoundingMode).
 * Stochastic: q = floor(t + u), u uniform in [0,1) (DLQ/src/trim_functions.cpp:155-158), accepted by the per-tensor
 * and per-channel quantize-dequantize entry points and by miq_quantize_per_tensor_f32.  The reference draws u from
 * libc rand() (CPU) or a clock-seeded generator per element (GPU); here u is a function of (seed, call, element index):
 *     key = splitmix64(seed + 0x9E3779B97F4A7C15 * (call + 1)), k0 = low word, k1 = high word
 *     r   = mix32((uint32) i + k0) ^ k1 ^ (uint32)(i >> 32),  u = (r >> 8) * 2^-24
 *     mix32(x): x ^= x >> 16; x *= 0x7feb352d; x ^= x >> 15; x *= 0x846ca68b; x ^= x >> 16
 * with `call` the number of stochastic launches on non-empty tensors since the seed was set. */
#define MIQ_ROUND_NEAREST 0
#define MIQ_ROUND_STOCHASTIC 1

/* Counterpart of srand() for the stochastic rounding mode: sets the seed (0 at load) and restarts the call count. */
int miq_set_stochastic_seed(uint64_t seed);
/* Current seed and number of stochastic launches since it was set. */
int miq_get_stochastic_state(uint64_t* seed /* host */, uint64_t* calls /* host */);

/* DLQ/include/DlQuantization/Quantization.hpp:83-105 (QuantizationMode) */
#define MIQ_QUANTIZATION_TF 0
#define MIQ_QUANTIZATION_TF_ENHANCED 1
#define MIQ_QUANTIZATION_PERCENTILE 2
#define MIQ_QUANTIZATION_MSE 3
#define MIQ_QUANTIZATION_ENTROPY 4

#define MIQ_PDF_SIZE 512 /* DLQ/src/math_functions.hpp:80 */

/* DLQ/include/DlQuantization/Quantization.hpp:113-120 (struct TfEncoding); same field order and types. */
typedef struct miq_encoding
{
    double min;
    double max;
    double delta;
    double offset;
    int bw;
} miq_encoding;

const char* miq_last_error(void);
/* Library/ABI version, bumped when a signature changes. */
int miq_version(void);
/* One-time, per-GPU set-up of the library for the current device (today: the device address of the static scratch
 * array behind miq_minmax_per_channel_static_f32).  Optional -- everything it prepares is also prepared on first use --
 * but callers that capture HIP graphs should call it before the first capture on each GPU.  Allocates nothing.
 * No counterpart in the reference. */
int miq_init(void);

/* ---------------------------------------------------------------------------------------------------------------
 * Host-side encoding arithmetic (double precision, no device work)
 * ------------------------------------------------------------------------------------------------------------- */

/* ITensorQuantizationSim<float>::fillEncodingInfo / generateScaleOffset
 * (DLQ/include/DlQuantization/ITensorQuantizationSim.h:102-105, DLQ/src/TensorQuantizationSim.cpp:62-92). */
int miq_fill_encoding_info(int bw, double enc_min, double enc_max, miq_encoding* out /* host */);

/* getComputedEncodings (DLQ/src/quantization_utils.cpp:58-143): (min, max) -> TF encoding. */
int miq_get_computed_encodings(int bw, double mn, double mx, int use_symmetric, int use_strict_symmetric,
                               int use_unsigned_symmetric, miq_encoding* out /* host */);

/* ---------------------------------------------------------------------------------------------------------------
 * v1 (DlQuantization) quantize-dequantize: clamp to [min,max], x/delta - offset, round half away from zero,
 * delta*(q+offset); all in float32
 * ------------------------------------------------------------------------------------------------------------- */

/* ITensorQuantizationSim<float>::quantizeDequantizeTensor(in, cnt, out, encMin, encMax, bw, roundMode, use_cuda, stream)
 * (ITensorQuantizationSim.h:49-55, DLQ/src/TensorQuantizationSim.cpp:104-114; kernel DLQ/src/trim_functions.cu:46-60).
 * As in the reference, delta/offset are re-derived from (enc_min, enc_max, bw). */
int miq_qdq_per_tensor_f32(const float* in, float* out, int64_t n, double enc_min, double enc_max, int bw,
                           int rounding_mode, void* stream);
/* Same arithmetic with bfloat16 storage (the reference's caller upcasts to float32 and casts the result back:
 * TORCH/v1/tensor_quantizer.py:1129-1138); the conversion passes are fused into the kernel. */
int miq_qdq_per_tensor_bf16(const uint16_t* in, uint16_t* out, int64_t n, double enc_min, double enc_max, int bw,
                            int rounding_mode, void* stream);

/* out = float(half(in)): quantize-dequantize of the float16 data type (QuantizationDataType.float, bitwidth 16), which
 * the reference forms as tensor.half().float() (TORCH/v1/tensor_quantizer.py:1104-1107), in one pass. */
int miq_fp16_round_trip_f32(const float* in, float* out, int64_t n, void* stream);

/* Quantize-dequantize of the 8-bit float data type (QuantizationDataType.float, bitwidth 8): quantize_to_fp8 /
 * fake_cast_to_ieee_float (TORCH/fp_quantization.py:133-209, called from TORCH/v1/tensor_quantizer.py:1108-1109).
 * Elements are laid out [outer][num_channels][inner]; channel c has the largest representable value maxval[c] and
 * bias[c] = 2^(7-M) - log2(maxval[c]) + log2(2 - 2^-M) - 1 (both device arrays of num_channels floats; per tensor:
 * num_channels = 1, inner = n).  Per element, in float32 and in this order: x_c = clamp(x, -maxval, maxval);
 * e = max(floor(log2|x_c| + bias), 1); step = 2^((e - M) - bias); out = rint(x_c / step) * step.  e is an integer in
 * [1, 2^(7-M)], so the caller passes the steps as a table: steps[c * T + e] = 2^((e - M) - bias[c]) for e = 0 .. T-1,
 * T = 2^(7-M) + 1 (a device array of num_channels * T floats). */
int miq_fp8_fake_cast_f32(const float* in, float* out, int64_t n, int64_t num_channels, int64_t inner,
                          const float* maxval, const float* bias, const float* steps, int mantissa_bits, void* stream);

/* The same for a float format of E exponent and M mantissa bits, E in [1, 8]: fake_cast_to_ieee_float as the v2 float
 * quantizer calls it (TORCH/v2/quantization/float/quantizer.py:302-322; TORCH/fp_quantization.py:171-209) with
 * bias[c] = 2^E - log2(maxval[c]) + log2(2 - 2^-M) - 1.  M enters only through the steps, so the entry point takes the
 * table and its length: steps[c * table + e] = 2^((e - M) - bias[c]) for e = 0 .. table - 1, table = 2^E + 1. */
int miq_float_fake_cast_f32(const float* in, float* out, int64_t n, int64_t num_channels, int64_t inner,
                            const float* maxval, const float* bias, const float* steps, int table, void* stream);

/* out = float(bfloat16(in)), round to nearest even, NaN stays NaN: the v2 float quantizer's bfloat16 case,
 * input.to(torch.bfloat16).to(input.dtype) (TORCH/v2/quantization/float/quantizer.py:309-314), in one pass. */
int miq_bf16_round_trip_f32(const float* in, float* out, int64_t n, void* stream);

/* ITensorQuantizationSim<float>::quantizeTensor(..., shiftToSigned) (ITensorQuantizationSim.h:57-59,
 * DLQ/src/TensorQuantizationSim.cpp:116-126; kernel DLQ/src/trim_functions.cu:62-76): float-valued grid indices. */
int miq_quantize_per_tensor_f32(const float* in, float* out, int64_t n, double enc_min, double enc_max, int bw,
                                int rounding_mode, int shift_to_signed, void* stream);

/* One pass that writes the dequantized tensor (out may be NULL) and the integer codes as bytes (bw <= 8):
 * uint8 grid index, or int8 (index - 2^(bw-1)) when shift_to_signed.  Fuses the two reference calls above. */
int miq_qdq_codes_per_tensor_f32(const float* in, float* out, uint8_t* codes, int64_t n, double enc_min,
                                 double enc_max, int bw, int shift_to_signed, void* stream);

/* Per-channel parameter recipe of AimetTensorQuantizer::quantizeDequantizePerChannel
 * (TSRC/AimetTensorQuantizer.cpp:209-227, 268-297): from per-channel (min,max) in float32, gate to include zero,
 * delta = (max-min)/num_steps, offset = round-half-even(min/delta).  enc_min/enc_max: device float[C] (raw encoding
 * values); the four outputs are device float[C].  num_steps = 2^bw - 1, minus 1 iff encodings[0].min == -encodings[0].max. */
int miq_per_channel_params_f32(const float* enc_min, const float* enc_max, int64_t num_channel, double num_steps,
                               float* out_min, float* out_max, float* out_delta, float* out_offset, void* stream);

/* The TF (min / max) encodings of all channels of a tensor, on the device: for channel c, TfEncodingAnalyzer::computeEncoding
 * (DLQ/src/TfEncodingAnalyzer.cpp:80-101) on the running (ch_min[c], ch_max[c]) and getComputedEncodings in double, as
 * miq_get_computed_encodings does on the host -- what StaticGridPerChannelQuantizer.compute_encoding
 * (TrainingExtensions/torch/src/python/aimet_torch/v1/tensor_quantizer.py:280-321) obtains from one analyzer object per
 * channel -- followed by miq_per_channel_params_f32 on the result.  enc: device double[num_channel][4] = (min, max,
 * delta, offset) of every channel's TfEncoding; out_*: the four kernel parameter vectors; raw_min / raw_max: float32 of
 * the encodings' min / max (the straight-through bounds).  All device float[num_channel].  Nothing waits: a wrapper in
 * training mode recomputes its parameter encodings in every forward (qc_quantize_op.py:769-777), and a caller that only
 * quantizes with them never needs them on the host. */
int miq_tf_encodings_per_channel_f32(const float* ch_min, const float* ch_max, int64_t num_channel, int bw,
                                     int use_symmetric, int use_strict_symmetric, int use_unsigned_symmetric,
                                     double* enc, float* out_min, float* out_max, float* out_delta, float* out_offset,
                                     float* raw_min, float* raw_max, void* stream);

/* ITensorQuantizationSim<float>::quantizeDequantizeTensorPerChannel(in, numChannel, numElement, numElementPerChannel,
 * out, encMin*, encMax*, encDelta*, encOffset*, roundMode, useCuda, stream) (ITensorQuantizationSim.h:107-118,
 * DLQ/src/TensorQuantizationSim.cpp:300-317; kernel DLQ/src/trim_functions.cu:78-92):
 * channel(i) = (i / num_element_per_channel) % num_channel. */
int miq_qdq_per_channel_f32(const float* in, float* out, int64_t num_channel, int64_t num_element,
                            int64_t num_element_per_channel, const float* enc_min, const float* enc_max,
                            const float* enc_delta, const float* enc_offset, int rounding_mode, void* stream);
int miq_qdq_per_channel_bf16(const uint16_t* in, uint16_t* out, int64_t num_channel, int64_t num_element,
                             int64_t num_element_per_channel, const float* enc_min, const float* enc_max,
                             const float* enc_delta, const float* enc_offset, int rounding_mode, void* stream);
/* As above, also writing the 8-bit grid indices (out may be NULL). */
int miq_qdq_codes_per_channel_f32(const float* in, float* out, uint8_t* codes, int64_t num_channel,
                                  int64_t num_element, int64_t num_element_per_channel, const float* enc_min,
                                  const float* enc_max, const float* enc_delta, const float* enc_offset,
                                  int shift_to_signed, int bw, void* stream);

/* quantizeDequantizeBroadcast<float> (DLQ/include/DlQuantization/Quantization.hpp:209-222, kernel
 * DLQ/src/trim_functions.cu:96-122).  input_strides / encoding_strides are HOST arrays of length num_dims
 * (num_dims <= 8); they travel as kernel arguments instead of device-resident arrays. */
int miq_qdq_broadcast_f32(const float* in, float* out, int64_t num_element, int64_t num_dims,
                          const int64_t* input_strides /* host */, const int64_t* encoding_strides /* host */,
                          const float* enc_min, const float* enc_max, const float* enc_delta,
                          const float* enc_offset, void* stream);

/* Straight-through backward of the v1 path, compute_dloss_by_dx
 * (TORCH/v1/quantsim_straight_through_grad.py:91-118): grad_in = grad_out * (min <= x && x <= max). */
int miq_ste_bwd_per_tensor_f32(const float* x, const float* grad_out, float* grad_in, int64_t n, float enc_min,
                               float enc_max, void* stream);
int miq_ste_bwd_per_tensor_bf16(const uint16_t* x, const uint16_t* grad_out, uint16_t* grad_in, int64_t n,
                                float enc_min, float enc_max, void* stream);
int miq_ste_bwd_per_channel_f32(const float* x, const float* grad_out, float* grad_in, int64_t num_channel,
                                int64_t num_element, int64_t num_element_per_channel, const float* enc_min,
                                const float* enc_max, void* stream);
int miq_ste_bwd_per_channel_bf16(const uint16_t* x, const uint16_t* grad_out, uint16_t* grad_in,
                                 int64_t num_channel, int64_t num_element, int64_t num_element_per_channel,
                                 const float* enc_min, const float* enc_max, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * Several tensors in one launch.  A simulation model quantizes every parameter tensor in every forward
 * (StaticGridQuantWrapper._quantize_dequantize_params, TORCH/v1/qc_quantize_op.py:705-763, one
 * quantizeDequantizePerChannel call per tensor); for the dozens of small tensors of a convolutional network the
 * launches' fixed cost exceeds their traffic.  One launch takes a table of segments instead; each segment is
 * miq_qdq_per_channel_* on its own tensor (nearest rounding), results identical.  No counterpart in the reference.
 * A per-tensor encoding is a segment with num_channel = 1 and one-element parameter vectors (the values
 * miq_fill_encoding_info gives, as float32).
 * ------------------------------------------------------------------------------------------------------------- */
typedef struct miq_qdq_segment
{
    const void* in;                    /* device: float32 or bfloat16 elements, 16-byte aligned */
    void* out;                         /* device, 16-byte aligned; may be `in` */
    int64_t num_element;               /* 1 .. 2^31 - 1 */
    int64_t num_channel;
    int64_t num_element_per_channel;   /* at least 8 (float32) / 16 (bfloat16) */
    const float* enc_min;              /* device float[num_channel]: as miq_qdq_per_channel_* takes them */
    const float* enc_max;
    const float* enc_delta;
    const float* enc_offset;
    uint32_t fd_magic, fd_shift;       /* filled by miq_qdq_multi_plan */
    int32_t first_tile;                /* filled by miq_qdq_multi_plan */
    int32_t reserved;
} miq_qdq_segment;
/* Host side, once per table: checks every segment, fills the fields marked above and returns the number of tiles of
 * the launch (-1 with miq_last_error() set when a segment cannot take part: the caller quantizes that one by itself).
 * segments: HOST array of 1 .. 256 records; the caller then copies it to device memory. */
int64_t miq_qdq_multi_plan(miq_qdq_segment* segments /* host, in/out */, int num_segments, int elem_bytes);
/* segments: the planned table in DEVICE memory; total_tiles: what miq_qdq_multi_plan returned for it. */
int miq_qdq_per_channel_multi_f32(const miq_qdq_segment* segments /* device */, int num_segments, int64_t total_tiles,
                                  void* stream);
int miq_qdq_per_channel_multi_bf16(const miq_qdq_segment* segments /* device */, int num_segments, int64_t total_tiles,
                                   void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * Straight-through estimator through a saved one-bit mask.
 * The reference's v2 QuantDequantFunc saves the mask of its backward as a bool tensor, one byte per element
 * (TORCH/v2/quantization/affine/backends/torch_builtins.py:303-327); its v1 QuantizeDequantize keeps the input alive
 * and recomputes the comparison (TORCH/v1/tensor_quantizer.py:1098-1212, quantsim_straight_through_grad.py:100-118).
 * Here the forward can write the mask with one BIT per element and the backward reads it instead of x: per float32
 * element 8.125 + 8.125 bytes instead of 8 + 12, and 1/8 byte kept between the passes instead of 4.
 * The miq_*_mask_* forwards compute exactly what their counterparts without "mask" compute, and mask bit = the factor
 * the matching backward would multiply the gradient with: (min <= x && x <= max) on the float32 casts of the stored
 * encoding's min / max for v1 (what miq_ste_bwd_per_*_* is given), qmin <= round(x / scale) - offset <= qmax for v2.
 * miq_ste_bwd_mask_* then gives grad_in = grad_out * bit, bit for bit what miq_ste_bwd_per_*_* / miq_v2_qdq_bwd_* give.
 * Mask layout (the same for every entry point of one storage type): with V = 4 (float32) or 8 (bfloat16) the elements
 * are taken in groups of 64 V; group g owns the 64-bit words g V .. g V + V - 1, and bit t of word j belongs to element
 * 64 V g + V t + j; the num_element % V elements after the last whole 16-byte vector have their bits in bits 0.. of
 * one more word after the last group.  mask: device memory of miq_ste_mask_bytes() bytes, 8-byte aligned.
 * Nearest rounding only (the stochastic mode keeps the recomputing backward).
 * ------------------------------------------------------------------------------------------------------------- */
/* Bytes of the mask for num_element elements stored in elem_bytes bytes each (4: float32, 2: bfloat16); -1 on
 * invalid arguments. */
int64_t miq_ste_mask_bytes(int64_t num_element, int elem_bytes);
/* miq_qdq_per_tensor_* + mask; mask_min / mask_max: the bounds the matching miq_ste_bwd_per_tensor_* call would be
 * given (the stored encoding's min / max as float32; for a bfloat16 tensor the reference's comparison casts them to
 * bfloat16, quantsim_straight_through_grad.py:115 with torch's promotion of a 0-dim tensor). */
int miq_qdq_mask_per_tensor_f32(const float* in, float* out, uint64_t* mask, int64_t n, double enc_min, double enc_max,
                                int bw, float mask_min, float mask_max, void* stream);
int miq_qdq_mask_per_tensor_bf16(const uint16_t* in, uint16_t* out, uint64_t* mask, int64_t n, double enc_min,
                                 double enc_max, int bw, float mask_min, float mask_max, void* stream);
/* miq_qdq_per_channel_* + mask; raw_min / raw_max: device float[num_channel], the stored encodings' min / max (the
 * vectors miq_ste_bwd_per_channel_* is given), as opposed to enc_min / enc_max, the gated ones of the forward. */
int miq_qdq_mask_per_channel_f32(const float* in, float* out, uint64_t* mask, int64_t num_channel, int64_t num_element,
                                 int64_t num_element_per_channel, const float* enc_min, const float* enc_max,
                                 const float* enc_delta, const float* enc_offset, const float* raw_min,
                                 const float* raw_max, void* stream);
int miq_qdq_mask_per_channel_bf16(const uint16_t* in, uint16_t* out, uint64_t* mask, int64_t num_channel,
                                  int64_t num_element, int64_t num_element_per_channel, const float* enc_min,
                                  const float* enc_max, const float* enc_delta, const float* enc_offset,
                                  const float* raw_min, const float* raw_max, void* stream);
/* miq_v2_qdq_* + mask */
int miq_v2_qdq_mask_f32(const float* in, float* out, uint64_t* mask, int64_t num_channel, int64_t num_element,
                        int64_t num_element_per_channel, const float* scale, const float* offset, int qmin, int qmax,
                        void* stream);
int miq_v2_qdq_mask_bf16(const uint16_t* in, uint16_t* out, uint64_t* mask, int64_t num_channel, int64_t num_element,
                         int64_t num_element_per_channel, const float* scale, const float* offset, int qmin, int qmax,
                         void* stream);
/* grad_in = grad_out * bit (grad_in may alias grad_out) */
int miq_ste_bwd_mask_f32(const uint64_t* mask, const float* grad_out, float* grad_in, int64_t n, void* stream);
int miq_ste_bwd_mask_bf16(const uint64_t* mask, const uint16_t* grad_out, uint16_t* grad_in, int64_t n, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * v2 quantize-dequantize (TORCH/v2/quantization/affine/backends/torch_builtins.py:290-344, QuantDequantFunc):
 * r = round-half-even(x/scale) - offset; mask = qmin <= r <= qmax; y = (clamp(r,qmin,qmax) + offset) * scale,
 * computed in float32.  scale/offset: device float[num_channel], channel(i) = (i / num_element_per_channel) %
 * num_channel (num_channel = 1 for per-tensor).  out and codes may each be NULL; codes are int32 grid values.
 * ------------------------------------------------------------------------------------------------------------- */
int miq_v2_qdq_f32(const float* in, float* out, int32_t* codes, int64_t num_channel, int64_t num_element,
                   int64_t num_element_per_channel, const float* scale, const float* offset, int qmin, int qmax,
                   void* stream);
int miq_v2_qdq_bf16(const uint16_t* in, uint16_t* out, int64_t num_channel, int64_t num_element,
                    int64_t num_element_per_channel, const float* scale, const float* offset, int qmin, int qmax,
                    void* stream);
/* Backward w.r.t. the input (torch_builtins.py:329-344, tensor_grad = grad * mask); the mask is recomputed from x. */
int miq_v2_qdq_bwd_f32(const float* x, const float* grad_out, float* grad_in, int64_t num_channel,
                       int64_t num_element, int64_t num_element_per_channel, const float* scale,
                       const float* offset, int qmin, int qmax, void* stream);
int miq_v2_qdq_bwd_bf16(const uint16_t* x, const uint16_t* grad_out, uint16_t* grad_in, int64_t num_channel,
                        int64_t num_element, int64_t num_element_per_channel, const float* scale,
                        const float* offset, int qmin, int qmax, void* stream);
/* Backward w.r.t. the input, scale and offset in one pass (torch_builtins.py:329-344):
 *   q = x / scale; r = round(q); mask = qmin <= r - offset <= qmax
 *   grad_in     = grad * mask                                                    (may be NULL: not written)
 *   scale_grad  = sum over the channel of grad * (clamp(r, offset+qmin, offset+qmax) - q * mask)
 *   offset_grad = sum over the channel of grad * (~mask * scale)
 * where the reference leaves the two sums to autograd's reduction to the parameter shape.  The tensor is laid out
 * [outer][num_channel][num_element_per_channel] (outer = num_element / (num_channel * num_element_per_channel)).
 * scale_grad / offset_grad: device float[num_channel], either may be NULL.  Element terms are float32; they are
 * added per workgroup in float32 and across workgroups in double, in a fixed order.  workspace: device memory of
 * miq_v2_qdq_bwd_params_workspace_bytes() bytes, overwritten by each call. */
int64_t miq_v2_qdq_bwd_params_workspace_bytes(int64_t num_channel, int64_t num_element,
                                              int64_t num_element_per_channel);
int miq_v2_qdq_bwd_params_f32(const float* x, const float* grad_out, float* grad_in, int64_t num_channel,
                              int64_t num_element, int64_t num_element_per_channel, const float* scale,
                              const float* offset, int qmin, int qmax, float* scale_grad, float* offset_grad,
                              void* workspace, void* stream);
int miq_v2_qdq_bwd_params_bf16(const uint16_t* x, const uint16_t* grad_out, uint16_t* grad_in, int64_t num_channel,
                               int64_t num_element, int64_t num_element_per_channel, const float* scale,
                               const float* offset, int qmin, int qmax, float* scale_grad, float* offset_grad,
                               void* workspace, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * Range learning: the quantization grid is a function of a learnable encoding min / max per channel, and the
 * gradients go back to that min / max.  The reference forms the grid and the encoding gradients with a dozen tensor
 * operations of parameter size per quantizer and step; here the grid is one small launch and the encoding gradients
 * leave the backward's reduction kernel directly.
 *
 * How (min, max) become (scale, offset), and (sum_s, sum_o) -- the two channel sums miq_v2_qdq_bwd_params_* returns
 * as scale_grad / offset_grad -- become (grad_min, grad_max).  steps = qmax - qmin; every operation is float32.
 *   MIQ_RANGE_V2_ASYMMETRIC (TORCH/v2/quantization/affine/quantizer.py:404-436, differentiated by autograd there;
 *   "/ steps" is the product with float32(1 / steps), which is how torch's device kernels divide a tensor by a number,
 *   so that the grid equals get_scale() / get_offset() of the same module to the bit)
 *     scale = (max - min) / steps, offset = round(min / scale) - qmin (round straight-through)
 *     s = sum_s - sum_o * ((min / scale) / scale); grad_max = s / steps; grad_min = sum_o / scale - s / steps
 *   MIQ_RANGE_V2_SYMMETRIC: scale as above, offset = 0; grad_max = sum_s / steps, grad_min = -grad_max
 *   MIQ_RANGE_V1_ASYMMETRIC (TORCH/v1/quantsim_straight_through_grad.py:121-162, :251-292; qmin must be 0; here and
 *   below every "/" is a division, the reference's operands being tensors)
 *     scale = (max - min) / steps, offset = -clamp(round(-min / scale), 0, steps)
 *     t1 = sum_s / steps, t2 = steps / (max - min)^2 * sum_o
 *     grad_min = -t1 + max * t2, grad_max = t1 - min * t2
 *   MIQ_RANGE_V1_SIGNED_SYMMETRIC (:143-146, :296-325): scale = max / floor(steps / 2), offset = -ceil(steps / 2)
 *     grad_max = sum_s / (steps div 2), grad_min = -grad_max
 *   MIQ_RANGE_V1_UNSIGNED_SYMMETRIC (:148-151): scale = (max - min) / steps, offset = min / scale; gradients as for
 *     the signed symmetric mode
 * ------------------------------------------------------------------------------------------------------------- */
#define MIQ_RANGE_V2_ASYMMETRIC 0
#define MIQ_RANGE_V2_SYMMETRIC 1
#define MIQ_RANGE_V1_ASYMMETRIC 2
#define MIQ_RANGE_V1_SIGNED_SYMMETRIC 3
#define MIQ_RANGE_V1_UNSIGNED_SYMMETRIC 4
/* grid: device float[4 * num_channel] = {scale_0.., offset_0.., min_0.., max_0..}, min / max being the values the grid
 * was made from.  gate != 0 first orders the range in place, in enc_min / enc_max themselves, as the v1 wrappers do
 * before every forward pass (TORCH/v1/tensor_quantizer.py:1347-1359): min = min(min, 0), max = max(max, 0),
 * max = max(max, min + 1e-5); NaN stays NaN. */
int miq_range_to_grid_f32(float* enc_min, float* enc_max, int64_t num_channel, int qmin, int qmax, int mode, int gate,
                          float* grid, void* stream);
/* miq_v2_qdq_bwd_params_* with the encoding gradients in place of the scale / offset gradients: `grid` as
 * miq_range_to_grid_f32 wrote it for the forward pass (scale and offset are read from it as well), grad_min /
 * grad_max: device float[num_channel].  Workspace: miq_v2_qdq_bwd_params_workspace_bytes(). */
int miq_qdq_bwd_range_f32(const float* x, const float* grad_out, float* grad_in, int64_t num_channel,
                          int64_t num_element, int64_t num_element_per_channel, const float* grid, int qmin, int qmax,
                          int mode, float* grad_min, float* grad_max, void* workspace, void* stream);
int miq_qdq_bwd_range_bf16(const uint16_t* x, const uint16_t* grad_out, uint16_t* grad_in, int64_t num_channel,
                           int64_t num_element, int64_t num_element_per_channel, const float* grid, int qmin,
                           int qmax, int mode, float* grad_min, float* grad_max, void* workspace, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * Calibration statistics
 * ------------------------------------------------------------------------------------------------------------- */

/* GetMin + GetMax (DLQ/src/math_functions.cpp:328-347; GPU twins math_functions.cu:52-64) fused into one pass.
 * out_min_max: device float[2] = {min, max}; NaN elements are ignored, an empty input yields {+inf, -inf}.
 * workspace: device memory of miq_minmax_workspace_bytes(1, n, n) bytes, or NULL.  With a workspace the partial
 * results of the workgroups are stored and folded by a second kernel; without one they meet in the output through
 * atomics, which is several times slower on large tensors. */
int64_t miq_minmax_workspace_bytes(int64_t num_channel, int64_t num_element, int64_t num_element_per_channel);
int miq_minmax_f32(const float* in, int64_t n, float* out_min_max, void* workspace, void* stream);
/* Per-channel form used for per-channel min/max (TF) encodings: out is device float[2*num_channel] laid out
 * {min_0..min_{C-1}, max_0..max_{C-1}}; channel(i) = (i / num_element_per_channel) % num_channel. */
int miq_minmax_per_channel_f32(const float* in, int64_t num_channel, int64_t num_element,
                               int64_t num_element_per_channel, float* out_min_max, void* workspace, void* stream);

/* miq_minmax_per_channel_f32 for callers that cannot allocate device memory (code under HIP graph capture, serving
 * loops, harnesses that forbid hipMalloc): the workgroups' partial results go to a 256 KiB array inside the loaded
 * library (one copy per GPU, held until the process ends) instead of a caller workspace, and the call allocates and
 * frees nothing.  No counterpart in the reference.  Same arguments and results as miq_minmax_per_channel_f32
 * (num_channel = 1, num_element_per_channel = num_element gives the per-tensor form).  Limit: tensors whose
 * miq_minmax_workspace_bytes() exceeds 256 KiB (32768 partial pairs: about 5.4e8 elements per tensor) are refused with
 * MIQ_ERR_INVALID_ARG.  All calls on one GPU share the array: calls that overlap in time on one GPU (two streams,
 * two threads) race and must be serialised by the caller.  The array's device address is looked up once per GPU
 * (hipGetSymbolAddress, under a mutex): by miq_init(), or else by the first call on that GPU -- call miq_init() with
 * the GPU current before a stream capture that contains this entry point, since the lookup is not a capturable
 * operation. */
int miq_minmax_per_channel_static_f32(const float* in, int64_t num_channel, int64_t num_element,
                                      int64_t num_element_per_channel, float* out_min_max, void* stream);

/* Encoding analyzer object = IQuantizationEncodingAnalyzer<float>
 * (DLQ/include/DlQuantization/IQuantizationEncodingAnalyzer.hpp:48-126) as instantiated by
 * getEncodingAnalyzerInstance<float>(mode) (DLQ/src/QuantizerFactory.cpp:74-97) for QUANTIZATION_TF
 * (TfEncodingAnalyzer, DLQ/src/TfEncodingAnalyzer.cpp:59-101) and QUANTIZATION_TF_ENHANCED
 * (TfEnhancedEncodingAnalyzer, DLQ/src/TfEnhancedEncodingAnalyzer.cpp:68-397) and QUANTIZATION_PERCENTILE
 * (PercentileEncodingAnalyzer, DLQ/src/PercentileEncodingAnalyzer.cpp:54-215: the same PDF, cut where its cumulative
 * sum reaches 100 - p and p percent) and QUANTIZATION_MSE (MseEncodingAnalyzer, DLQ/src/MseEncodingAnalyzer.cpp:54-262:
 * the same PDF; every pair of one bucket edge below zero and one above, zero included on either side, is a candidate
 * range, searched on the device for the least PDF-weighted squared quantization error of the bucket centres; this
 * analyzer holds 25 KB more device memory than the others, allocated by the library also when the state is the
 * caller's) and QUANTIZATION_ENTROPY (EntropyEncodingAnalyzer, DLQ/src/EntropyEncodingAnalyzer.cpp:54-436, over
 * updateTensorHistogram_cpu / rescaleHistogram, DLQ/src/math_functions.cpp:468-643: 512 counts over exactly the range
 * seen so far, moved into new bins whenever a batch widens it; for 8 bits the range is narrowed to the window whose
 * 255-level quantization has the least KL divergence from the histogram saturated into it, searched on the host over
 * the counts read back; this analyzer allocates its own device state and ignores a caller's; samples are taken to be
 * finite).  All statistics (running min/max,
 * the 512-bucket PDF, its range and iteration count) live in device memory owned by the object on the device that
 * was current at creation; update_stats enqueues work and never synchronises.  compute_encoding synchronises
 * `stream` once to read the result back.  An object must not be used from two threads at once. */
typedef struct miq_analyzer miq_analyzer;
int miq_analyzer_create(int quantization_mode, miq_analyzer** out);
/* The same with the object's device state in caller memory (miq_analyzer_state_bytes() bytes, 16-byte aligned, alive as
 * long as the object): the reference routes its scratch memory through the caller's allocator too (IAllocator,
 * DLQ/include/DlQuantization/Quantization.hpp:62-76, TrainingExtensions/torch/src/AimetTensorQuantizer.cpp:56-71).
 * Neither form queues or waits for device work. */
int64_t miq_analyzer_state_bytes(void);
int miq_analyzer_create_in(int quantization_mode, void* device_state, miq_analyzer** out);
int miq_analyzer_destroy(miq_analyzer* a);
/* setPercentileValue (IQuantizationEncodingAnalyzer.hpp:104-112; PercentileEncodingAnalyzer.cpp:203-207), 0..100,
 * default 100.  Stored by every analyzer, used by the percentile one. */
int miq_analyzer_set_percentile(miq_analyzer* a, float percentile);
/* resetEncodingStats (TSRC/AimetTensorQuantizer.cpp:85-92) */
int miq_analyzer_reset(miq_analyzer* a, void* stream);
/* updateStats(tensor, tensorSize, mode, allocator) (IQuantizationEncodingAnalyzer.hpp:59-69) */
int miq_analyzer_update_stats_f32(miq_analyzer* a, const float* data, int64_t n, void* stream);
/* computeEncoding(bw, useSymmetricEncodings, useStrictSymmetric, useUnsignedSymmetric)
 * (IQuantizationEncodingAnalyzer.hpp:71-93) + the validity flag of AimetTensorQuantizer::getEncoding
 * (TSRC/AimetTensorQuantizer.cpp:180-192): *is_valid = 0 when no statistics were ever supplied. */
int miq_analyzer_compute_encoding(miq_analyzer* a, int bw, int use_symmetric, int use_strict_symmetric,
                                  int use_unsigned_symmetric, miq_encoding* out /* host */, int* is_valid /* host */,
                                  void* stream);
/* The part of compute_encoding that needs no waiting, queued ahead: the pending batch is folded, the TF-Enhanced search
 * launched and the copy of its result requested on `stream`.  A compute_encoding call with the same arguments and
 * stream that follows with no other call on the object in between only waits for that copy, so a caller that owns many
 * analyzers (one per activation of a model: QuantizationSimModel.compute_encodings,
 * TrainingExtensions/torch/src/python/aimet_torch/v1/quantsim.py:435-470) queues all of them first and pays for one
 * round trip to the device instead of one per analyzer.  Any other call on the object drops the request, and
 * compute_encoding then does all of its work as usual; without statistics the call does nothing.  No counterpart in
 * the reference, whose analyzers compute on the host. */
int miq_analyzer_queue_encoding(miq_analyzer* a, int bw, int use_symmetric, int use_strict_symmetric,
                                int use_unsigned_symmetric, void* stream);
/* getStatsHistogram() (IQuantizationEncodingAnalyzer.hpp:95-102): 512 (xLeft, pdf) pairs into host arrays.
 * Returns MIQ_ERR_UNSUPPORTED for a TF analyzer (the reference asserts) and writes *num_buckets = 0 while the PDF
 * has not been initialised. */
int miq_analyzer_get_stats_histogram(miq_analyzer* a, double* x_left /* host[512] */, double* pdf /* host[512] */,
                                     int* num_buckets /* host */, void* stream);
/* The entropy analyzer's histogram as it stands (TensorProfilingParams, DLQ/src/math_functions.hpp:69-77): 512
 * counts, the range they span, whether a batch other than all zeros has been seen, and the number of batches counted.
 * MIQ_ERR_INVALID_ARG for any other analyzer.  (miq_analyzer_get_stats_histogram is MIQ_ERR_UNSUPPORTED for the
 * entropy analyzer: the reference's own getStatsHistogram for it has no defined result.) */
int miq_analyzer_entropy_histogram(miq_analyzer* a, double* counts /* host[512] */,
                                   double* range_min_max /* host[2] */, int* initialized /* host */,
                                   int* iterations /* host */, void* stream);
/* Test/inspection hooks: the integer bin counts of the most recent update_stats call (host uint32[512]) and the
 * TF-Enhanced candidate list with every candidate's cost from the most recent compute_encoding call
 * (host arrays of capacity `cap`; *count receives the number of candidates, *best_index the winner). */
int miq_analyzer_last_batch_counts(miq_analyzer* a, uint32_t* counts /* host[512] */, void* stream);
int miq_analyzer_last_search(miq_analyzer* a, float* deltas /* host */, int32_t* offsets /* host */,
                             double* costs /* host */, int cap, int* count /* host */, int* best_index /* host */,
                             void* stream);

/* Per-channel TF-Enhanced / percentile analyzer: C independent 512-bucket PDFs over the channels of one tensor,
 * channel(i) = (i / num_element_per_channel) % num_channel, updated by one launch sequence per batch and searched by
 * one launch.  It replaces the reference's list of per-channel analyzer objects fed slice by slice
 * (TrainingExtensions/torch/src/python/aimet_torch/v1/tensor_quantizer.py:535-570, each an
 * IQuantizationEncodingAnalyzer<float> behind TrainingExtensions/torch/src/AimetTensorQuantizer.cpp:85-126, 180-192):
 * channel c's PDF and encoding are those a miq_analyzer fed `tensor.select(axis, c).contiguous()` produces.
 * quantization_mode: MIQ_QUANTIZATION_TF_ENHANCED or MIQ_QUANTIZATION_PERCENTILE.
 * device_state: device memory of miq_channel_analyzer_state_bytes(num_channel) bytes, 16-byte aligned, owned by the
 * caller and alive as long as the object (so that it can come from the caller's own allocator), or NULL to let the
 * library allocate it.  workspace (update_stats): device memory of miq_channel_analyzer_workspace_bytes(...) bytes, or
 * NULL (slower min/max pass).  update_stats enqueues work and never synchronises; compute_encodings and
 * get_stats_histogram synchronise `stream` once.  out (compute_encodings): host miq_encoding[num_channel]. */
typedef struct miq_channel_analyzer miq_channel_analyzer;
int64_t miq_channel_analyzer_state_bytes(int64_t num_channel);
int64_t miq_channel_analyzer_workspace_bytes(int64_t num_channel, int64_t num_element,
                                             int64_t num_element_per_channel);
int miq_channel_analyzer_create(int quantization_mode, int64_t num_channel, void* device_state, void* stream,
                                miq_channel_analyzer** out);
int miq_channel_analyzer_destroy(miq_channel_analyzer* a);
int miq_channel_analyzer_reset(miq_channel_analyzer* a, void* stream);
int miq_channel_analyzer_set_percentile(miq_channel_analyzer* a, float percentile);
int miq_channel_analyzer_update_stats_f32(miq_channel_analyzer* a, const float* data, int64_t num_element,
                                          int64_t num_element_per_channel, void* workspace, void* stream);
int miq_channel_analyzer_compute_encodings(miq_channel_analyzer* a, int bw, int use_symmetric,
                                           int use_strict_symmetric, int use_unsigned_symmetric,
                                           miq_encoding* out /* host[num_channel] */, int* is_valid /* host */,
                                           void* stream);
/* The same search with the results left on the device, for a caller that only quantizes with them: enc receives
 * (min, max, delta, offset) of every channel's TfEncoding as device double[num_channel][4], the six device
 * float[num_channel] vectors the kernel parameters of miq_per_channel_params_f32 and float32(min), float32(max) (the
 * straight-through bounds).  Nothing waits.  *is_valid = 0 (and nothing is written) while no statistics were supplied.
 * MIQ_ERR_UNSUPPORTED for the percentile analyzer, whose encodings are host arithmetic.  No counterpart in the
 * reference. */
int miq_channel_analyzer_compute_encodings_device(miq_channel_analyzer* a, int bw, int use_symmetric,
                                                  int use_strict_symmetric, int use_unsigned_symmetric,
                                                  double* enc, float* out_min, float* out_max, float* out_delta,
                                                  float* out_offset, float* raw_min, float* raw_max,
                                                  int* is_valid /* host */, void* stream);
int miq_channel_analyzer_get_stats_histogram(miq_channel_analyzer* a, int64_t channel, double* x_left /* host[512] */,
                                             double* pdf /* host[512] */, int* num_buckets /* host */, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * AdaRound (ADA = TrainingExtensions/torch/src/python/aimet_torch/v1/adaround)
 *
 * All tensors are float32 in device memory; channel(i) = (i / num_element_per_channel) % num_channel selects the
 * entry of the device vectors delta / offset (one entry for a per-tensor encoding).  clip_min / clip_max are the
 * integer grid limits of AdaroundWrapper.apply_adaround (0 and 2^bw - 1, or -2^(bw-1) and 2^(bw-1) - 1 for the
 * signed-symmetric grid).  Tensors of at most 2^31 - 1 elements.
 * ------------------------------------------------------------------------------------------------------------- */

/* AdaroundWrapper.apply_adaround (ADA/adaround_wrapper.py:124-149):
 *   out = (clamp(floor(w / delta) + h(alpha) - offset, clip_min, clip_max) + offset) * delta
 * with h = clamp(sigmoid(alpha) * (zeta - gamma) + gamma, 0, 1) when use_soft_rounding != 0 and h = (alpha >= 0)
 * otherwise; zeta = 1.1, gamma = -0.1 (aimet_common/defs.py:302-306). */
int miq_adaround_soft_round_f32(const float* weight, const float* alpha, float* out, int64_t num_channel,
                                int64_t num_element, int64_t num_element_per_channel, const float* delta,
                                const float* offset, float clip_min, float clip_max, int use_soft_rounding,
                                void* stream);
/* weight_floor = floor(weight / delta) (ADA/adaround_wrapper.py:132), the part of apply_adaround that does not depend
 * on alpha; the fused Linear entry points below take it in place of the weight. */
int miq_adaround_floor_f32(const float* weight, float* weight_floor, int64_t num_channel, int64_t num_element,
                           int64_t num_element_per_channel, const float* delta, void* stream);
/* floor(weight / delta) saturated per channel to [offset + clip_min - 2, offset + clip_max + 1] and stored as int8.
 * h(alpha) lies in [0, 1], so outside that window clamp(floor + h - offset, clip_min, clip_max) and its gradient mask
 * no longer depend on the exact value: the fused Linear kernels give the same results from this form as from the
 * float32 one.  *unfit (device int32, zero on entry) is set to 1 when some channel's window leaves the int8 range
 * (grids wider than 7 bits, or offsets far from zero): the output is then unusable and the caller keeps float32. */
int miq_adaround_floor_i8(const float* weight, int8_t* weight_floor, int64_t num_channel, int64_t num_element,
                          int64_t num_element_per_channel, const float* delta, const float* offset, float clip_min,
                          float clip_max, int32_t* unfit, void* stream);
/* The same with int16 storage (grids of 8 to 14 bits). */
int miq_adaround_floor_i16(const float* weight, int16_t* weight_floor, int64_t num_channel, int64_t num_element,
                          int64_t num_element_per_channel, const float* delta, const float* offset, float clip_min,
                          float clip_max, int32_t* unfit, void* stream);
/* AdaroundWrapper._generate_alpha_parameter (ADA/adaround_wrapper.py:211-224):
 *   alpha = -log((zeta - gamma) / (w / delta - floor(w / delta) - gamma) - 1) */
int miq_adaround_init_alpha_f32(const float* weight, float* alpha, int64_t num_channel, int64_t num_element,
                                int64_t num_element_per_channel, const float* delta, void* stream);
/* One optimiser iteration's elementwise tail, fused (AdaroundOptimizer._optimize_rounding's loss.backward() +
 * optimizer.step(), ADA/adaround_optimizer.py:190-218, for the part below the layer's own backward):
 * given grad_weight = dLoss_recon/dW', computes dLoss/dalpha through apply_adaround's soft rounding (closed-interval
 * clamp gradients, as torch.clamp), adds the gradient of the rounding regulariser
 * reg_param * sum(1 - |2h - 1|^beta) (AdaroundLoss.compute_round_loss, ADA/adaround_loss.py:82-111) when beta >= 0
 * (beta < 0 = warm-start period, regulariser off), and applies torch.optim.Adam's update (no weight decay, no
 * amsgrad) to alpha with moments exp_avg / exp_avg_sq; `step` is the 1-based count of this update.
 * The hyper-parameters are doubles because the reference's are Python floats: 1 - beta1, 1 - beta2, the bias
 * corrections and lr / (1 - beta1^step) are formed in double and cast to float32 where torch's kernels cast them
 * (1 - float32(0.999) differs from float32(1 - 0.999) by 1.3e-5 of its value).  beta1 must exceed 0.5.
 * grad_alpha: optional (may be null) device tensor receiving dLoss/dalpha, what alpha.grad holds in the reference.
 * reg_partial: optional device float[miq_adaround_blocks(num_element)] receiving per-workgroup partial sums of
 * (1 - |2h - 1|^beta) evaluated at the alpha *before* the update (summed and scaled by reg_param by the caller). */
int miq_adaround_bwd_adam_f32(const float* weight, const float* grad_weight, float* alpha, float* exp_avg,
                              float* exp_avg_sq, float* grad_alpha, int64_t num_channel, int64_t num_element,
                              int64_t num_element_per_channel, const float* delta, const float* offset, float clip_min,
                              float clip_max, double reg_param, double beta, double lr, double beta1, double beta2,
                              double eps, int step, float* reg_partial, void* stream);
/* The gradient alone (autograd of apply_adaround + compute_round_loss w.r.t. alpha), nothing updated: for callers
 * that keep their own optimiser. */
int miq_adaround_bwd_f32(const float* weight, const float* grad_weight, const float* alpha, float* grad_alpha,
                         int64_t num_channel, int64_t num_element, int64_t num_element_per_channel,
                         const float* delta, const float* offset, float clip_min, float clip_max, double reg_param,
                         double beta, float* reg_partial, void* stream);
/* Number of workgroups (= partial sums) miq_adaround_bwd_adam_f32 / miq_adaround_bwd_f32 use for num_element elements. */
int miq_adaround_blocks(int64_t num_element);
/* dLoss/dout of the reconstruction loss (ADA/adaround_loss.py:71-80, after the activation of
 * ADA/adaround_optimizer.py:194-200) in one pass, where autograd runs relu twice, a subtraction, two products and a
 * comparison over the layer's output:
 *   grad_out[b][j] = (act(out[b][j]) - act(target[index[b]][j])) * scale [ * (act(out[b][j]) > 0) under ReLU ]
 * out / grad_out: [batch][per_sample]; target: the cached outputs of all num_cached samples, [num_cached][per_sample];
 * index: device int64[batch] sample numbers (NULL: sample b is row b); negative numbers count from the end, as in
 * torch's indexing, and a number outside [-num_cached, num_cached) turns its row of grad_out into NaN.  scale = 2 / (elements of `out` per channel), the factor the mean over all but dim 1 leaves.
 * activation: 0 none, 1 ReLU.  batch <= 65535. */
int miq_adaround_recon_grad_f32(const float* out, const float* target, const int64_t* index, int64_t batch,
                                int64_t num_cached, int64_t per_sample, int activation, float scale, float* grad_out,
                                void* stream);
/* The per-element terms exactly as the kernels above evaluate them, for accuracy measurements (no counterpart in the
 * reference, whose terms are separate torch ops: ADA/adaround_wrapper.py:136-139, ADA/adaround_loss.py:100-106).
 *   what = 0: in = alpha[n]; out = float[3 n]: sigmoid(alpha), h(alpha), dh/dalpha
 *   what = 1: in = h[n];     out = float[2 n]: 1 - |2h - 1|^beta, and its derivative with respect to h,
 *             -beta |2h - 1|^(beta - 1) sgn(2h - 1) 2, with the exponent float32(beta - 1) as torch's pow backward takes it */
int miq_adaround_eval_terms_f32(const float* in, float* out, int64_t num_element, int what, double beta, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * AdaRound iteration of a Linear layer, soft rounding fused into MFMA GEMMs (the adarounded weight and its gradient
 * never exist in memory).  One iteration of AdaroundOptimizer._optimize_rounding (ADA/adaround_optimizer.py:182-218)
 * for torch.nn.Linear with a batch of 32 rows (BATCH_SIZE, ADA/adaround_optimizer.py:58), or of 64, 128 or 256 rows
 * (a caller with another batch size; a 1x1 Conv2d over 2, 4 or 8 pixels, whose rows are the pixels of the 32 images
 * in channels-last order: ADA/adaround_optimizer.py:268-272 runs the same contraction as functional.conv2d):
 *   fwd:  out = linear(x[rows], apply_adaround(W), bias);  grad_out = d recon_loss(act(out), act(target[rows])) / d out
 *   bwd:  dLoss/dW' = grad_out^T x[rows]  ->  alpha gradient + regulariser + Adam, as miq_adaround_bwd_adam_f32
 * weight_floor (= floor(W / delta), from miq_adaround_floor_f32), alpha, moments: [out_features, in_features] float32
 * row-major.  x: rows of in_features floats, row r at
 * x + r * x_row_stride; target likewise with out_features floats.  batch: 32, 64, 128 or 256.  row_index: device
 * int32[batch] choosing the rows of x and target (NULL = rows 0..batch-1); num_rows: the number of rows x and target hold.  An index outside [0, num_rows) never
 * leaves the buffers: that row reads row 0 or num_rows - 1 and its grad_out / out entries are NaN, which the backward
 * spreads over alpha (the reference's indexing raises IndexError there; aimet_amd checks the indices on the host
 * before the first launch).  num_channel: 1 (per-tensor delta/offset) or out_features (per output channel).
 * Shapes: out_features % 32 == 0, in_features % 128 == 0, out_features * in_features < 2^31; other shapes return
 * MIQ_ERR_INVALID_ARG and the caller uses the elementwise entry points around its own GEMM.
 * activation: 0 none, 1 ReLU (the act_func the reference applies to both outputs, ADA/adaround_optimizer.py:192-194).
 * ------------------------------------------------------------------------------------------------------------- */

/* The same two entry points with weight_floor stored as int8 or int16 (miq_adaround_floor_i8 / _i16): a quarter or half of
 * the bytes of the one weight-shaped operand that never changes during the optimisation.  No counterpart in the reference; results are
 * identical to the float32 form, element for element. */

/* Bytes of device workspace the forward needs (partial products of the split K dimension). */
int64_t miq_adaround_linear_workspace_bytes(int64_t out_features, int64_t in_features, int64_t batch);
/* Number of regulariser partial sums miq_adaround_linear_bwd_adam_f32 writes. */
int miq_adaround_linear_blocks(int64_t out_features, int64_t in_features);
/* out (optional, may be NULL): device float[batch * out_features], the layer output before the activation.
 * grad_out: device float[batch * out_features] = 2 (act(out) - act(target)) act'(out) / batch, the gradient of
 * AdaroundLoss.compute_recon_loss (ADA/adaround_loss.py:70-80: squared error summed over dimension 1, mean over the
 * rest, which for rows that are pixels is the same number) w.r.t. out.
 * loss_partial (optional): device float[ceil(batch * out_features / 256)] partial sums of the reconstruction loss. */
int miq_adaround_linear_fwd_f32(const float* weight_floor, const float* alpha, const float* x, const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride,
                                const float* bias, int64_t out_features, int64_t in_features, int64_t num_channel,
                                const float* delta, const float* offset, float clip_min, float clip_max,
                                int activation, float* workspace, float* out, float* grad_out, float* loss_partial,
                                void* stream);
int miq_adaround_linear_bwd_adam_f32(const float* weight_floor, const float* grad_out, const float* x,
                                     const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg,
                                     float* exp_avg_sq, float* grad_alpha, int64_t out_features, int64_t in_features,
                                     int64_t num_channel, const float* delta, const float* offset, float clip_min,
                                     float clip_max, double reg_param, double beta, double lr, double beta1, double beta2,
                                     double eps, int step, float* reg_partial, void* stream);

int miq_adaround_linear_fwd_i8(const int8_t* weight_floor, const float* alpha, const float* x, const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride, const float* bias,
                               int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                               const float* offset, float clip_min, float clip_max, int activation, float* workspace,
                               float* out, float* grad_out, float* loss_partial, void* stream);
int miq_adaround_linear_bwd_adam_i8(const int8_t* weight_floor, const float* grad_out, const float* x,
                                    const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg,
                                    float* exp_avg_sq, float* grad_alpha, int64_t out_features, int64_t in_features,
                                    int64_t num_channel, const float* delta, const float* offset, float clip_min,
                                    float clip_max, double reg_param, double beta, double lr, double beta1, double beta2,
                                    double eps, int step, float* reg_partial, void* stream);
int miq_adaround_linear_fwd_i16(const int16_t* weight_floor, const float* alpha, const float* x, const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride, const float* bias,
                               int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                               const float* offset, float clip_min, float clip_max, int activation, float* workspace,
                               float* out, float* grad_out, float* loss_partial, void* stream);
int miq_adaround_linear_bwd_adam_i16(const int16_t* weight_floor, const float* grad_out, const float* x,
                                    const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg,
                                    float* exp_avg_sq, float* grad_alpha, int64_t out_features, int64_t in_features,
                                    int64_t num_channel, const float* delta, const float* offset, float clip_min,
                                    float clip_max, double reg_param, double beta, double lr, double beta1, double beta2,
                                    double eps, int step, float* reg_partial, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * v2 histogram observer + SQNR encoding analyzer
 * (EA = TORCH/v2/quantization/encoding_analyzer.py).  State lives in caller-owned device buffers:
 *   state_hist    float[num_hist * num_bins]   running histogram (integer-valued counts, as torch.histc returns)
 *   state_minmax  float[num_hist * 2]          running {min, max} of the finite values
 * Histogram h covers the contiguous slab data[h * n_per_hist, (h + 1) * n_per_hist) (per-tensor: num_hist = 1;
 * per-channel along axis 0: num_hist = C).
 * ------------------------------------------------------------------------------------------------------------- */

int64_t miq_v2_hist_workspace_bytes(int64_t num_hist, int64_t n_per_hist, int num_bins);
/* _HistogramObserver.collect_stats + merge_stats (EA:131-262) for one batch.  Writes the batch's own statistics
 * (what collect_stats returns) to batch_hist / batch_minmax and merges them into state_* (has_stats = 0: the state is
 * empty and becomes the batch's statistics).  bad_flag: device int32, set to 1 when a slab holds no finite value (the
 * reference raises ValueError there; the caller checks the flag when it next reads results).  workspace: device
 * buffer of miq_v2_hist_workspace_bytes, zero-filled by the caller before its first use and not written by anyone
 * else afterwards (it holds counters that every update leaves at zero); updates that share a workspace must not
 * overlap.  want_batch_hist = 0 skips the batch's own histogram (batch_hist may then be NULL; batch_minmax, optional,
 * is still written): only callers that quantize dynamically with the batch's statistics read it.
 * has_stats = 1, want_batch_hist = 0 (the calibration loop) enqueues two kernels and reads the batch once as long as
 * the batch stays inside the statistics' range (twice when it does not); the other modes enqueue three kernels and
 * read it twice.  Shapes that give every histogram to one workgroup (a thousand histograms or more, or slabs of up
 * to 6144 elements, at up to 2048 bins) take one kernel in every mode and leave the workspace untouched.
 * Never synchronises. */
int miq_v2_hist_update_f32(const float* data, int64_t num_hist, int64_t n_per_hist, int num_bins, int has_stats,
                           int want_batch_hist, float* state_hist, float* state_minmax, float* batch_hist,
                           float* batch_minmax, int32_t* bad_flag, void* workspace, void* stream);
/* Number of (delta, offset) candidates SqnrEncodingAnalyzer searches (EA:594-646); -1 on invalid arguments. */
int miq_v2_sqnr_num_candidates(double num_steps, int symmetric, int asym_deltas, int sym_deltas,
                               int offset_candidates);
/* SqnrEncodingAnalyzer.compute_encodings_from_stats (EA:566-592): candidate grid (EA:594-660), expected noise of every
 * candidate (EA:675-725, gamma-weighted clipping noise), first minimum wins; out_min / out_max: device float[num_hist].
 * noise: device double[num_hist * num_candidates] (scratch and inspection: the score of every candidate);
 * best_index (optional): device int32[num_hist]. */
int miq_v2_sqnr_search_f32(const float* hist, const float* minmax, int64_t num_hist, int num_bins, double num_steps,
                           int symmetric, double gamma, int asym_deltas, int sym_deltas, int offset_candidates,
                           float* out_min, float* out_max, double* noise, int32_t* best_index, void* stream);

/* Sequential MSE's loss (SequentialMse.compute_recon_loss, aimet_torch/v1/seq_mse.py:557-581; neg_sqnr :602-615; per
 * block of input channels in aimet_torch/v2/seq_mse.py:325-357): for two float32 tensors a, b of [blocks, rows, cols]
 * -- a layer's output with the candidate weight and with the float weight, one slab per block of input channels --
 * the error summed over rows, per block and column.  kind 0: (a - b)^2.  kind 1: |a - b|.  kind 2: two planes,
 * (b - a)^2 and b^2, from which the caller forms -10 log10(mean b^2 / (mean (b - a)^2 + eps)).
 * Rows are cut into `splits` pieces (miq_column_error_splits proposes a count that fills the device) whose sums land in
 * partial[splits][planes][blocks][cols]; the caller adds the pieces.  Each sum runs over its rows in order: the result
 * does not change from run to run. */
int64_t miq_column_error_splits(int64_t blocks, int64_t rows, int64_t cols);
int miq_column_error_f32(const float* a, const float* b, int64_t blocks, int64_t rows, int64_t cols, int kind,
                         int64_t splits, float* partial, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MIQ_H */
