/*
 * TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement, in plain C, of the arithmetic of the reference's quantization-simulation hot path
 * (the v1 / DlQuantization CPU loops and the v2 torch formulas).  It exists so that the HIP kernels can be
 * compared bit-for-bit with an independent, single-threaded statement of the same arithmetic.  Nothing in the
 * product package links, loads or calls this file: only tests/, the smoke check and the bench's CPU-baseline
 * leg do.
 *
 * Every function names the reference lines it follows.  Paths are relative to the reference root:
 *   DLQ   = ModelOptimizations/DlQuantization
 *   TSRC  = TrainingExtensions/torch/src
 *   TORCH = TrainingExtensions/torch/src/python/aimet_torch
 *
 * Build: gcc -O2 -std=c11 -ffp-contract=off -fno-fast-math (see oracle/Makefile).  The float/double/int type of
 * every intermediate below is deliberate: it is the type the reference's C++ expression has after the usual
 * arithmetic conversions with DTYPE = float.
 *
 * Pin status (what each function is checked against lives in tests/test_oracle_*.py):
 *   every function here is pinned by the reference's own golden vectors and/or by the compiled reference
 *   (oracle/_ref), except where its comment says "parity unpinned".
 */
#include <float.h>
#include <limits.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_PDF_SIZE 512 /* DLQ/src/math_functions.hpp:80 */

/* std::max(a, b) and std::min(a, b) exactly as libstdc++ evaluates them (this fixes which operand survives a NaN);
 * the arguments below are always written in the reference's order. */
#define STD_MAX(a, b) (((a) < (b)) ? (b) : (a))
#define STD_MIN(a, b) (((b) < (a)) ? (b) : (a))

typedef struct
{
    double min, max, delta, offset;
    int bw;
} orc_encoding; /* DLQ/include/DlQuantization/Quantization.hpp:113-120 */

typedef struct
{
    double xLeft[ORC_PDF_SIZE];
    double pdf[ORC_PDF_SIZE];
    int iterations;
    int initialized;   /* xLeft.size() != 0 in the reference */
    int stats_updated; /* _statsUpdated */
} orc_pdf;             /* DLQ/src/math_functions.hpp:59-67 + TfEnhancedEncodingAnalyzer.h:98-99 */

/* ------------------------------------------------------------------------------------------------------------
 * bf16 <-> f32 (round to nearest even), the conversion torch's .to(torch.bfloat16) performs
 * (TORCH/v1/tensor_quantizer.py:1129-1138 upcasts the input and casts the result back).
 * ---------------------------------------------------------------------------------------------------------- */
float orc_bf16_to_f32(uint16_t h)
{
    uint32_t u = ((uint32_t) h) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t orc_f32_to_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) /* NaN -> 0x7FC0, as c10::BFloat16's round_to_nearest_even does */
        return (uint16_t) 0x7fc0u;
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t) (u >> 16);
}

/* ------------------------------------------------------------------------------------------------------------
 * a2  encoding from (min, max, bw)
 * ---------------------------------------------------------------------------------------------------------- */

/* DLQ/src/quantization_utils.cpp:145-156, EPSILON = 1e-5 (quantization_utils.hpp:51) */
void orc_gate_min_max(double* mn, double* mx)
{
    *mn = fmin(*mn, 0.0);
    *mx = fmax(*mx, 0.0);
    *mx = fmax(*mx, *mn + 1e-5);
}

/* DLQ/src/TensorQuantizationSim.cpp:62-92 (generateScaleOffset + fillEncodingInfo),
 * DLQ/src/trim_functions.cpp:61-73 (computeDelta / computeOffset: C round(), half away from zero) */
void orc_fill_encoding_info(int bw, double mn, double mx, orc_encoding* e)
{
    orc_gate_min_max(&mn, &mx);
    double numSteps = pow(2, bw) - 1;
    if (mn == -mx)
        numSteps -= 1;
    double delta  = (mx - mn) / numSteps;
    double offset = round(mn / delta);
    e->bw         = bw;
    e->delta      = delta;
    e->offset     = offset;
    e->min        = offset * delta;
    e->max        = delta * numSteps + e->min;
}

/* ------------------------------------------------------------------------------------------------------------
 * a3  per-element quantize / dequantize, DTYPE = float
 * ---------------------------------------------------------------------------------------------------------- */

/* DLQ/src/trim_functions.cpp:141-165 with ROUND_NEAREST: clamp, scale, subtract offset, roundf */
static inline float orc_quantize_value(float x, float mn, float mx, float delta, float offset)
{
    float t = fmaxf(fminf(x, mx), mn);
    t       = t / delta - offset;
    return roundf(t);
}

/* DLQ/src/trim_functions.cpp:167-171 */
static inline float orc_dequantize_value(float q, float delta, float offset)
{
    return delta * (q + offset);
}

/* DLQ/src/TensorQuantizationSim.cpp:104-114 -> trim_functions.cpp:174-182 */
void orc_qdq_per_tensor_f32(const float* in, int64_t n, float* out, double encMin, double encMax, int bw)
{
    orc_encoding e;
    orc_fill_encoding_info(bw, encMin, encMax, &e);
    float mn = (float) e.min, mx = (float) e.max, d = (float) e.delta, o = (float) e.offset;
    for (int64_t i = 0; i < n; ++i)
        out[i] = orc_dequantize_value(orc_quantize_value(in[i], mn, mx, d, o), d, o);
}

/* DLQ/src/TensorQuantizationSim.cpp:116-126 -> trim_functions.cpp:203-218.
 * shift = 2^(bw-1) as unsigned int; out[i] -= shift is a float subtraction. */
void orc_quantize_per_tensor_f32(const float* in, int64_t n, float* out, double encMin, double encMax, int bw,
                                 int shiftToSigned)
{
    orc_encoding e;
    orc_fill_encoding_info(bw, encMin, encMax, &e);
    float mn = (float) e.min, mx = (float) e.max, d = (float) e.delta, o = (float) e.offset;
    unsigned int shift = 0;
    if (shiftToSigned)
        shift = (unsigned int) pow(2, bw - 1);
    for (int64_t i = 0; i < n; ++i)
    {
        float q = orc_quantize_value(in[i], mn, mx, d, o);
        q -= (float) shift;
        out[i] = q;
    }
}

/* Same arithmetic with bf16 storage: upcast, QDQ in float, round the result back to bf16
 * (TORCH/v1/tensor_quantizer.py:1129-1138). */
void orc_qdq_per_tensor_bf16(const uint16_t* in, int64_t n, uint16_t* out, double encMin, double encMax, int bw)
{
    orc_encoding e;
    orc_fill_encoding_info(bw, encMin, encMax, &e);
    float mn = (float) e.min, mx = (float) e.max, d = (float) e.delta, o = (float) e.offset;
    for (int64_t i = 0; i < n; ++i)
    {
        float x = orc_bf16_to_f32(in[i]);
        out[i]  = orc_f32_to_bf16(orc_dequantize_value(orc_quantize_value(x, mn, mx, d, o), d, o));
    }
}

/* ------------------------------------------------------------------------------------------------------------
 * a5  per-channel QDQ
 * ---------------------------------------------------------------------------------------------------------- */

/* TSRC/AimetTensorQuantizer.cpp:209-227, 268-297: the per-channel parameters are derived with float32 tensor ops:
 * minimum/maximum with 0, max >= min + 1e-5 (added in float), delta = (max - min) / numSteps,
 * offset = at::round(min / delta) which rounds half to even.  numSteps comes from encodings[0] only. */
void orc_per_channel_params_f32(const double* encMin, const double* encMax, int64_t numChannel, int bw, float* mn,
                                float* mx, float* delta, float* offset)
{
    double numSteps = pow(2, bw) - 1;
    if (encMin[0] == -encMax[0])
        numSteps -= 1;
    float numStepsF = (float) numSteps;
    for (int64_t c = 0; c < numChannel; ++c)
    {
        float lo  = (float) encMin[c];
        float hi  = (float) encMax[c];
        lo        = (lo < 0.0f) ? lo : 0.0f;
        hi        = (hi > 0.0f) ? hi : 0.0f;
        float eps = lo + 1e-5f;
        hi        = (hi > eps) ? hi : eps;
        float d   = (hi - lo) / numStepsF;
        mn[c]     = lo;
        mx[c]     = hi;
        delta[c]  = d;
        offset[c] = rintf(lo / d);
    }
}

/* DLQ/src/trim_functions.cpp:698-709 */
void orc_qdq_per_channel_f32(const float* in, int64_t numChannel, int64_t numElement, int64_t numElementPerChannel,
                             float* out, const float* mn, const float* mx, const float* delta, const float* offset)
{
    for (int64_t i = 0; i < numElement; ++i)
    {
        int64_t c = (i / numElementPerChannel) % numChannel;
        out[i] = orc_dequantize_value(orc_quantize_value(in[i], mn[c], mx[c], delta[c], offset[c]), delta[c], offset[c]);
    }
}

/* ------------------------------------------------------------------------------------------------------------
 * a3 with ROUND_STOCHASTIC (DLQ/src/trim_functions.cpp:141-166): *out = floor(*out + randUniformCpu()) -- the float
 * grid position is widened to double, the uniform number added, the floor stored back as float.  The uniform numbers
 * are an argument here so that the formula can be pinned against the reference fed from libc rand() and the product
 * kernel against its own documented generator (orc_stochastic_uniforms).
 * ---------------------------------------------------------------------------------------------------------- */
static inline float orc_quantize_value_stochastic(float x, float mn, float mx, float delta, float offset, double u)
{
    float t = fmaxf(fminf(x, mx), mn);
    t       = t / delta - offset;
    return (float) floor((double) t + u);
}

/* dequant != 0: quantize-dequantize; dequant == 0: grid index minus `shift` (quantizeToFxp, trim_functions.cpp:203-218).
 * numChannel == 1 with parameter vectors of length 1 is the per-tensor case. */
void orc_stochastic_f32(const float* in, int64_t numChannel, int64_t numElement, int64_t numElementPerChannel,
                        float* out, const float* mn, const float* mx, const float* delta, const float* offset,
                        const double* u, int dequant, float shift)
{
    for (int64_t i = 0; i < numElement; ++i)
    {
        int64_t c = (i / numElementPerChannel) % numChannel;
        float q   = orc_quantize_value_stochastic(in[i], mn[c], mx[c], delta[c], offset[c], u[i]);
        out[i]    = dequant ? orc_dequantize_value(q, delta[c], offset[c]) : q - shift;
    }
}

/* The product's generator (include/miq.h, MIQ_ROUND_STOCHASTIC): u is a function of (seed, call, element index). */
static inline uint32_t orc_mix32(uint32_t x)
{
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

void orc_stochastic_uniforms(uint64_t seed, uint64_t call, int64_t first, int64_t n, double* u)
{
    uint64_t z = seed + 0x9E3779B97F4A7C15ull * (call + 1);
    z          = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z          = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z          = z ^ (z >> 31);
    uint32_t k0 = (uint32_t) z, k1 = (uint32_t) (z >> 32);
    for (int64_t j = 0; j < n; ++j)
    {
        uint64_t i = (uint64_t) (first + j);
        uint32_t r = orc_mix32((uint32_t) i + k0) ^ k1 ^ (uint32_t) (i >> 32);
        u[j]       = (double) (r >> 8) * 0x1p-24;
    }
}

/* quantize only (the float-valued grid index), per channel; used to pin integer codes */
void orc_quantize_per_channel_f32(const float* in, int64_t numChannel, int64_t numElement,
                                  int64_t numElementPerChannel, float* out, const float* mn, const float* mx,
                                  const float* delta, const float* offset)
{
    for (int64_t i = 0; i < numElement; ++i)
    {
        int64_t c = (i / numElementPerChannel) % numChannel;
        out[i]    = orc_quantize_value(in[i], mn[c], mx[c], delta[c], offset[c]);
    }
}

void orc_qdq_per_channel_bf16(const uint16_t* in, int64_t numChannel, int64_t numElement,
                              int64_t numElementPerChannel, uint16_t* out, const float* mn, const float* mx,
                              const float* delta, const float* offset)
{
    for (int64_t i = 0; i < numElement; ++i)
    {
        int64_t c = (i / numElementPerChannel) % numChannel;
        float x   = orc_bf16_to_f32(in[i]);
        out[i]    = orc_f32_to_bf16(
            orc_dequantize_value(orc_quantize_value(x, mn[c], mx[c], delta[c], offset[c]), delta[c], offset[c]));
    }
}

/* DLQ/src/trim_functions.cpp:634-660: numpy-style broadcast of the encoding over the input.
 * The reference keeps the running remainder and the indices in `int`. */
void orc_qdq_broadcast_f32(const float* in, float* out, int64_t numElement, int64_t numDims,
                           const int64_t* inputStrides, const int64_t* encodingStrides, const float* mn,
                           const float* mx, const float* delta, const float* offset)
{
    for (int64_t i = 0; i < numElement; ++i)
    {
        int encIdx    = 0;
        int remainder = (int) i;
        for (int64_t dim = 0; dim < numDims; ++dim)
        {
            int dimIdx = (int) (remainder / inputStrides[dim]);
            remainder  = (int) (remainder - dimIdx * inputStrides[dim]);
            encIdx += (int) (encodingStrides[dim] * dimIdx);
        }
        out[i] = orc_dequantize_value(orc_quantize_value(in[i], mn[encIdx], mx[encIdx], delta[encIdx], offset[encIdx]),
                                      delta[encIdx], offset[encIdx]);
    }
}

/* ------------------------------------------------------------------------------------------------------------
 * a6  straight-through backward of the v1 path
 * TORCH/v1/quantsim_straight_through_grad.py:91-118: grad * ((min <= x) & (x <= max)), both ends inclusive,
 * min/max being the encoding's stored values converted to float32.
 * ---------------------------------------------------------------------------------------------------------- */
void orc_ste_bwd_per_tensor_f32(const float* x, const float* gout, float* gin, int64_t n, float mn, float mx)
{
    for (int64_t i = 0; i < n; ++i)
        gin[i] = gout[i] * (float) ((mn <= x[i]) && (x[i] <= mx));
}

void orc_ste_bwd_per_channel_f32(const float* x, const float* gout, float* gin, int64_t numChannel,
                                 int64_t numElement, int64_t numElementPerChannel, const float* mn, const float* mx)
{
    for (int64_t i = 0; i < numElement; ++i)
    {
        int64_t c = (i / numElementPerChannel) % numChannel;
        gin[i]    = gout[i] * (float) ((mn[c] <= x[i]) && (x[i] <= mx[c]));
    }
}

/* ------------------------------------------------------------------------------------------------------------
 * a9  min/max statistics and the TF (min/max) encoding
 * ---------------------------------------------------------------------------------------------------------- */

/* DLQ/src/math_functions.cpp:328-347: std::min/std::max against a running value that starts at -/+DBL_MAX cast
 * to float (= -/+inf); NaN inputs never replace the running value. */
void orc_minmax_f32(const float* in, int64_t n, float* mnOut, float* mxOut)
{
    float mx = -INFINITY, mn = INFINITY;
    for (int64_t i = 0; i < n; ++i)
    {
        mx = STD_MAX(mx, in[i]);
        mn = STD_MIN(mn, in[i]);
    }
    *mnOut = mn;
    *mxOut = mx;
}

/* DLQ/src/quantization_utils.cpp:58-143 */
void orc_get_computed_encodings(int bw, double mn, double mx, int sym, int strict, int unsignedSym, orc_encoding* e)
{
    double numSteps = pow(2, bw) - 1;
    if (sym && strict)
        numSteps -= 1;
    e->bw = bw;
    if (isinf(mn))
        mn = -(double) FLT_MAX;
    if (isinf(mx))
        mx = (double) FLT_MAX;

    if (sym && ((mn < 0.0) || !unsignedSym))
    {
        mx                       = fmax(fabs(mx), fabs(mn));
        unsigned int numPosSteps = (unsigned int) floor(numSteps / 2);
        e->delta                 = mx / numPosSteps;
        e->offset                = -ceil(numSteps / 2);
        e->min                   = fmax(e->offset * e->delta, -(double) FLT_MAX);
        e->max                   = fmin(e->delta * numPosSteps, (double) FLT_MAX);
        return;
    }
    e->delta = (mx - mn) / numSteps;
    if (mn < 0 && mx > 0)
    {
        double bZero = round(-mn / e->delta);
        bZero        = fmin(numSteps, fmax(0.0, bZero));
        e->offset    = -bZero;
    }
    else
    {
        e->offset = round(mn / e->delta);
        e->min    = mn;
        e->max    = mx;
        return;
    }
    double t = e->delta * e->offset;
    if (t >= -(double) FLT_MAX && t <= (double) FLT_MAX)
        e->min = t;
    else
        e->min = -(double) FLT_MAX;
    e->max = mx - mn + e->min;
    if (e->max > (double) FLT_MAX)
        e->max = (double) FLT_MAX;
}

/* DLQ/src/TfEncodingAnalyzer.cpp:80-101, MIN_RANGE = 0.01 (TfEncodingAnalyzer.h:81) */
void orc_tf_compute_encoding(double accMin, double accMax, int bw, int sym, int strict, int unsignedSym,
                             orc_encoding* e)
{
    double newMin = fmin(0.0, accMin);
    double newMax = fmax(0.0, accMax);
    newMax        = fmax(newMax, newMin + 0.01);
    orc_get_computed_encodings(bw, newMin, newMax, sym, strict, unsignedSym, e);
}

/* ------------------------------------------------------------------------------------------------------------
 * a10  512-bucket PDF accumulation (signed_vals = true, the only mode the TF-Enhanced analyzer uses)
 * ---------------------------------------------------------------------------------------------------------- */
void orc_pdf_reset(orc_pdf* p)
{
    memset(p, 0, sizeof(*p));
}

/* DLQ/src/math_functions.cpp:208-241 */
static void orc_initialize_pdf(orc_pdf* p, float minVal, float maxVal)
{
    if (minVal == maxVal)
    {
        float t = minVal + (float) 0.01;
        maxVal  = STD_MAX(maxVal, t);
    }
    float center = (maxVal + minVal) / 2;
    float lo     = center - 3 * (center - minVal);
    float hi     = center + 3 * (maxVal - center);
    minVal       = STD_MAX(-FLT_MAX, lo);
    maxVal       = STD_MIN(FLT_MAX, hi);
    double bucket = ((double) maxVal - (double) minVal) / ORC_PDF_SIZE;
    for (int i = 0; i < ORC_PDF_SIZE; ++i)
    {
        p->xLeft[i] = minVal + i * bucket;
        p->pdf[i]   = 0.0;
    }
    p->iterations  = 0;
    p->initialized = 1;
}

/* DLQ/src/math_functions.cpp:368-384.  The reference converts the rounded float straight to int, which for NaN and
 * for values beyond the int range is the x86 "integer indefinite" INT_MIN and is therefore dropped by the range
 * test; comparing in float before converting gives the same outcome without relying on that. */
void orc_histogram_f32(const float* data, int64_t n, uint32_t* hist, float bucket, float pdfOffset)
{
    for (int64_t i = 0; i < n; ++i)
    {
        float r = roundf(data[i] / bucket - pdfOffset);
        if (r >= 0.0f && r < (float) ORC_PDF_SIZE)
            hist[(int) r] += 1;
    }
}

/* DLQ/src/math_functions.cpp:244-288 + TfEnhancedEncodingAnalyzer.cpp:68-76.
 * histOut (may be NULL) receives this batch's 512 integer bin counts. */
void orc_pdf_update_f32(orc_pdf* p, const float* data, int64_t n, uint32_t* histOut)
{
    uint32_t hist[ORC_PDF_SIZE];
    memset(hist, 0, sizeof(hist));
    if (histOut)
        memset(histOut, 0, sizeof(hist));
    p->stats_updated = 1;
    if (!p->initialized)
    {
        float mn, mx;
        orc_minmax_f32(data, n, &mn, &mx);
        if (mn == 0 && mx == 0)
            return;
        orc_initialize_pdf(p, mn, mx);
    }
    float bucket    = (float) (p->xLeft[1] - p->xLeft[0]);
    float minVal    = (float) p->xLeft[0];
    float pdfOffset = minVal / bucket;
    orc_histogram_f32(data, n, hist, bucket, pdfOffset);
    int cnt = (int) n;
    for (int i = 0; i < ORC_PDF_SIZE; ++i)
    {
        double prob = (double) hist[i] / (double) cnt;
        p->pdf[i]   = (p->pdf[i] * p->iterations + prob) / (p->iterations + 1);
    }
    p->iterations++;
    if (histOut)
        memcpy(histOut, hist, sizeof(hist));
}

/* ------------------------------------------------------------------------------------------------------------
 * a11  TF-Enhanced (SQNR) candidate search
 * ---------------------------------------------------------------------------------------------------------- */

/* DLQ/src/TfEnhancedEncodingAnalyzer.cpp:255-291, MIN_RANGE = 0.01 (.h:105) */
void orc_tfe_find_range(const orc_pdf* p, float* minOut, float* maxOut)
{
    float minVal = (float) p->xLeft[0];
    float maxVal = (float) p->xLeft[ORC_PDF_SIZE - 1];
    for (int i = 0; i < ORC_PDF_SIZE; ++i)
        if (p->pdf[i] > 0)
        {
            minVal = (float) p->xLeft[i];
            break;
        }
    for (int i = ORC_PDF_SIZE - 1; i > 0; --i)
        if (p->pdf[i] > 0)
        {
            maxVal = (float) p->xLeft[i];
            break;
        }
    minVal  = STD_MIN(minVal, 0.0f);
    maxVal  = STD_MAX(maxVal, 0.0f);
    float t = minVal + (float) 0.01;
    maxVal  = STD_MAX(maxVal, t);
    *minOut = minVal;
    *maxOut = maxVal;
}

/* DLQ/src/TfEnhancedEncodingAnalyzer.cpp:149-175 */
static int orc_tfe_clamp_to_observed(float obsMin, float obsMax, float numSteps, float* testDelta, int* testOffset)
{
    float tMin = *testDelta * (float) *testOffset;
    tMin       = STD_MAX(tMin, -FLT_MAX);
    float tMax = *testDelta * ((float) *testOffset + numSteps);
    tMax       = STD_MIN(tMax, FLT_MAX);
    if ((tMin < obsMin) && (tMax > obsMax))
        return 0;
    tMin = STD_MAX(obsMin, tMin);
    tMax = STD_MIN(obsMax, tMax);
    if (tMin == tMax)
        return 0;
    *testDelta  = (float) (((double) tMax - tMin) / numSteps);
    *testOffset = (int) roundf(tMin / *testDelta);
    return 1;
}

/* DLQ/src/TfEnhancedEncodingAnalyzer.cpp:177-214.  The delta factor f is a float that is advanced by adding the
 * double 1/16 and rounding back to float; the loop bound is compared in double. */
static int orc_tfe_pick_asymmetric(float obsMin, float obsMax, float numSteps, float* deltas, int* offsets, int maxOut)
{
    int n          = 0;
    float obsDelta = (float) (((double) obsMax - (double) obsMin) / numSteps);
    int obsOffset  = (int) roundf(obsMin / obsDelta);
    float t        = obsDelta * (float) obsOffset;
    obsMin         = STD_MAX(t, -FLT_MAX);
    t              = obsDelta * ((float) obsOffset + numSteps);
    obsMax         = STD_MIN(t, FLT_MAX);
    float deltaMax = obsDelta;
    for (float f = (float) (1.0 / 16); (double) f <= 1 + 1.0 / 16; f = (float) ((double) f + 1.0 / 16))
    {
        for (int i = 0; i <= 20; ++i)
        {
            float testDelta = f * deltaMax;
            int testOffset  = (int) ((double) (-numSteps) + (double) numSteps / 20.0 * i);
            if (!orc_tfe_clamp_to_observed(obsMin, obsMax, numSteps, &testDelta, &testOffset))
                continue;
            if (n < maxOut)
            {
                deltas[n]  = testDelta;
                offsets[n] = testOffset;
            }
            ++n;
        }
    }
    if (n < maxOut)
    {
        deltas[n]  = obsDelta;
        offsets[n] = obsOffset;
    }
    ++n;
    return n;
}

/* DLQ/src/TfEnhancedEncodingAnalyzer.cpp:216-253 */
static int orc_tfe_pick_symmetric(float minVal, float maxVal, float numSteps, int unsignedSym, float* deltas,
                                  int* offsets, int maxOut)
{
    int n = 0;
    float deltaMax;
    int testOffset;
    if ((minVal == 0.0) && unsignedSym)
    {
        deltaMax   = maxVal / numSteps;
        testOffset = 0;
    }
    else
    {
        float a    = fabsf(maxVal), b = fabsf(minVal);
        float absM = STD_MAX(a, b);
        deltaMax   = (float) (absM / (numSteps / 2.0));
        testOffset = (int) floorf(-numSteps / 2);
    }
    for (float f = (float) (1.0 / 100); (double) f <= 1 + 1.0 / 100; f = (float) ((double) f + 1.0 / 100))
    {
        if (n < maxOut)
        {
            deltas[n]  = f * deltaMax;
            offsets[n] = testOffset;
        }
        ++n;
    }
    return n;
}

/* Candidate list exactly as DLQ/src/TfEnhancedEncodingAnalyzer.cpp:357-381 builds it; returns the count. */
int orc_tfe_candidates(const orc_pdf* p, int bw, int sym, int strict, int unsignedSym, float* deltas, int* offsets,
                       int maxOut)
{
    float minVal, maxVal;
    orc_tfe_find_range(p, &minVal, &maxVal);
    float numSteps = (float) (pow(2, bw) - 1);
    if (sym)
    {
        if (strict)
            numSteps -= 1;
        return orc_tfe_pick_symmetric(minVal, maxVal, numSteps, unsignedSym, deltas, offsets, maxOut);
    }
    return orc_tfe_pick_asymmetric(minVal, maxVal, numSteps, deltas, offsets, maxOut);
}

/* DLQ/src/TfEnhancedEncodingAnalyzer.cpp:293-355, GAMMA = 3.0 (.h:102).  pow(v, 2) of the reference is v*v. */
/* The reference casts with (int); outside the int range that is undefined in C++, and its x86-64 build (cvttsd2si /
 * cvttss2si) yields INT_MIN, which then clamps to bucket 0.  Written out so that the restatement does not depend on
 * what this compiler makes of the undefined cast. */
static inline int orc_cvtt_x86(double v)
{
    return (v >= -2147483648.0 && v < 2147483648.0) ? (int) v : INT_MIN;
}

double orc_tfe_cost(const orc_pdf* p, int bw, float delta, int offset)
{
    float minVal   = delta * (float) offset;
    float stepSize = (float) (pow(2, bw) - 1);
    float maxVal   = delta * ((float) offset + stepSize);
    float pdfStart = (float) p->xLeft[0];
    double pdfStep = p->xLeft[1] - p->xLeft[0];
    int minInd     = orc_cvtt_x86(floor((minVal - pdfStart) / pdfStep));
    minInd         = (minInd < 0) ? 0 : minInd;
    minInd         = (minInd > ORC_PDF_SIZE - 1) ? ORC_PDF_SIZE - 1 : minInd;
    int maxInd     = orc_cvtt_x86(floor((maxVal - pdfStart) / pdfStep));
    maxInd         = (maxInd < 0) ? 0 : maxInd;
    maxInd         = (maxInd > ORC_PDF_SIZE - 1) ? ORC_PDF_SIZE - 1 : maxInd;

    double satBottom = 0;
    float minMid     = (float) (pdfStart + (minInd * pdfStep) + pdfStep / 2);
    for (int i = 0; i < minInd; ++i)
    {
        double mid = pdfStart + i * pdfStep + pdfStep / 2;
        double d   = mid - minMid;
        satBottom += p->pdf[i] * (d * d);
    }
    double satTop = 0;
    float maxMid  = (float) (pdfStart + (maxInd * pdfStep) + pdfStep / 2);
    for (int i = maxInd; i < ORC_PDF_SIZE; ++i)
    {
        double mid = pdfStart + i * pdfStep + pdfStep / 2;
        double d   = mid - maxMid;
        satTop += p->pdf[i] * (d * d);
    }
    double quant = 0;
    for (int i = minInd; i < maxInd; ++i)
    {
        float fv    = (float) (pdfStart + i * pdfStep + pdfStep / 2);
        int q       = orc_cvtt_x86((double) roundf(fv / delta - (float) offset));
        float dq    = delta * (float) (q + offset);
        double diff = (double) (fv - dq);
        quant += p->pdf[i] * (diff * diff);
    }
    double sqnr = 3.0 * (satBottom + satTop) + quant;
    return (sqnr < DBL_MAX) ? sqnr : DBL_MAX;
}

/* DLQ/src/TfEnhancedEncodingAnalyzer.cpp:78-147, 357-397.
 * costsOut / bestIdxOut are optional (NULL) and report every candidate's cost and the winner's position. */
void orc_tfe_compute_encoding(const orc_pdf* p, int bw, int sym, int strict, int unsignedSym, orc_encoding* e,
                              double* costsOut, int* bestIdxOut)
{
    memset(e, 0, sizeof(*e));
    float numSteps = (float) (pow(2, bw) - 1);
    if (bestIdxOut)
        *bestIdxOut = -1;
    if (!p->initialized)
    {
        if (p->stats_updated)
        {
            e->min    = -1;
            e->max    = 1;
            e->delta  = (e->max - e->min) / (int) numSteps;
            e->offset = floor(e->min / e->delta);
            e->min    = e->offset * e->delta;
            e->max    = e->min + (int) numSteps * e->delta;
            e->bw     = bw;
        }
        return;
    }
    enum { MAXC = 512 };
    float deltas[MAXC];
    int offsets[MAXC];
    int n = orc_tfe_candidates(p, bw, sym, strict, unsignedSym, deltas, offsets, MAXC);
    if (sym && strict)
        numSteps -= 1;
    float bestDelta = -1;
    int bestOffset  = -1;
    double bestCost = DBL_MAX;
    for (int i = 0; i < n; ++i)
    {
        double cost = orc_tfe_cost(p, bw, deltas[i], offsets[i]);
        if (costsOut)
            costsOut[i] = cost;
        if (cost < bestCost)
        {
            bestCost   = cost;
            bestDelta  = deltas[i];
            bestOffset = offsets[i];
            if (bestIdxOut)
                *bestIdxOut = i;
        }
    }
    float bMin = bestDelta * (float) bestOffset;
    bMin       = STD_MAX(bMin, -FLT_MAX);
    float bMax = bestDelta * ((float) bestOffset + numSteps);
    bMax       = STD_MIN(bMax, FLT_MAX);
    e->delta   = bestDelta;
    e->offset  = bestOffset;
    e->bw      = bw;
    e->min     = bMin;
    e->max     = bMax;
}

/* ------------------------------------------------------------------------------------------------------------
 * Percentile calibration on the same 512-bucket PDF (PercentileEncodingAnalyzer<float>;
 * DLQ/src/PercentileEncodingAnalyzer.cpp:78-198).  Statistics are gathered by UpdatePdf with signed_vals = true,
 * i.e. by orc_pdf_update_f32 above.
 * ---------------------------------------------------------------------------------------------------------- */

/* _computePercentileRange, :133-198 */
void orc_percentile_range(const orc_pdf* p, float percentile, float* minOut, float* maxOut)
{
    float minVal, maxVal;
    orc_tfe_find_range(p, &minVal, &maxVal); /* findOriginalRange<float>: the same steps (math_functions.cpp:400-433) */
    if (percentile == 100.0f)
    {
        *minOut = minVal;
        *maxOut = maxVal;
        return;
    }
    const float histBinWidth = (float) (p->xLeft[1] - p->xLeft[0]);
    float histMin            = (float) p->xLeft[0];
    float histMax            = (float) (p->xLeft[ORC_PDF_SIZE - 1] + histBinWidth);
    float percentileMin      = histMin;
    float percentileMax      = histMax;
    double cdf[ORC_PDF_SIZE];
    cdf[0] = p->pdf[0];
    for (int i = 1; i < ORC_PDF_SIZE; ++i)
        cdf[i] = p->pdf[i] + cdf[i - 1];
    float leftPercentile = 1 - percentile / 100;
    for (int i = 0; i < ORC_PDF_SIZE; ++i)
        if (cdf[i] >= leftPercentile)
        {
            percentileMin = (float) p->xLeft[i];
            break;
        }
    float rightPercentile = percentile / 100;
    for (int i = ORC_PDF_SIZE - 1; i >= 0; --i)
        if (cdf[i] < rightPercentile && p->xLeft[i] < maxVal)
        {
            percentileMax = (float) (p->xLeft[i] + histBinWidth);
            break;
        }
    if (percentileMin == percentileMax)
        percentileMax += histBinWidth;
    *minOut = percentileMin;
    *maxOut = percentileMax;
}

/* computeEncoding, :78-130 */
void orc_percentile_compute_encoding(const orc_pdf* p, float percentile, int bw, int sym, int strict, int unsignedSym,
                                     orc_encoding* e)
{
    memset(e, 0, sizeof(*e));
    float numSteps = (float) (pow(2, bw) - 1);
    if (sym && strict)
        numSteps -= 1;
    if (!p->initialized)
    {
        if (p->stats_updated)
        {
            e->min    = -1;
            e->max    = 1;
            e->delta  = (e->max - e->min) / (int) numSteps;
            e->offset = floor(e->min / e->delta);
            e->min    = e->offset * e->delta;
            e->max    = e->min + (int) numSteps * e->delta;
            e->bw     = bw;
        }
        return;
    }
    float aMin, aMax;
    orc_percentile_range(p, percentile, &aMin, &aMax);
    aMin = STD_MIN(aMin, 0.0f);
    aMax = STD_MAX(aMax, 0.0f);
    orc_get_computed_encodings(bw, aMin, aMax, sym, strict, unsignedSym, e);
}

/* ------------------------------------------------------------------------------------------------------------
 * MSE calibration on the same 512-bucket PDF (MseEncodingAnalyzer<float>; DLQ/src/MseEncodingAnalyzer.cpp:78-262).
 * Statistics are gathered by UpdatePdf with signed_vals = true, i.e. by orc_pdf_update_f32 above.  Every (min, max)
 * pair made of one bucket edge below zero (or zero) and one above zero (or zero) is a candidate; its cost is the
 * PDF-weighted squared error of quantize-dequantizing the bucket centres on the candidate's grid; the first candidate
 * of least cost wins.
 *
 * The reference walks the edges with `for (float i = histMin; i <= histMax; i += histBinWidth)`, which does not end
 * when the bucket width is below half a unit in the last place of the edges.  This restatement (and the library)
 * stops the walk after ORC_MSE_MAX_WALK steps: a PDF laid out by UpdatePdf needs 512 to 514.
 * ---------------------------------------------------------------------------------------------------------- */
#define ORC_MSE_MAX_WALK 1025
#define ORC_MSE_MAX_EDGES (ORC_MSE_MAX_WALK + 1)

/* (int) of a double the way x86-64 converts (the reference runs there): values outside int are INT_MIN */
static int orc_double_to_int(double v)
{
    if (!(v > -2147483649.0 && v < 2147483648.0))
        return INT_MIN;
    return (int) v;
}

/* _computeMSECost, :236-262 */
float orc_mse_cost(int bw, const float* centers, const float* pdfAtCenter, int numCenters, float candMin,
                   float candMax, int sym, int strict, int unsignedSym)
{
    orc_encoding e;
    orc_get_computed_encodings(bw, candMin, candMax, sym, strict, unsignedSym, &e);
    float weightedSquareErr = 0;
    for (int i = 0; i < numCenters; ++i)
    {
        float floatVal = centers[i];
        float inner    = STD_MIN(floatVal, candMax);
        float clamped  = STD_MAX(candMin, inner);
        int quantized  = orc_double_to_int(round(clamped / e.delta - e.offset));
        float dequant  = (float) (e.delta * (quantized + e.offset));
        float diff     = floatVal - dequant;
        /* std::pow(float, int) is pow in double; the square of a float is exact there */
        weightedSquareErr = (float) (weightedSquareErr + pdfAtCenter[i] * ((double) diff * (double) diff));
    }
    return weightedSquareErr;
}

/* _minimizeMSE + _pickMinMaxCandidatesMSECalib, :139-234.  Optional outputs: the candidate lists and bucket centres
 * (arrays of ORC_MSE_MAX_EDGES + 1 floats) and their counts in counts[3] = {numMin, numMax, numCenters}. */
void orc_mse_minimize(const orc_pdf* p, int bw, int sym, int strict, int unsignedSym, float* bestMin, float* bestMax,
                      float* minCandOut, float* maxCandOut, float* centersOut, int* counts)
{
    const float histBinWidth = (float) (p->xLeft[1] - p->xLeft[0]);
    float histMin            = (float) p->xLeft[0];
    float histMax            = (float) (p->xLeft[ORC_PDF_SIZE - 1] + histBinWidth);
    float minVal, maxVal;
    orc_tfe_find_range(p, &minVal, &maxVal); /* findOriginalRange<float> (math_functions.cpp:400-433) */
    maxVal = maxVal + histBinWidth;

    float edges[ORC_MSE_MAX_EDGES];
    float minCand[ORC_MSE_MAX_EDGES + 1], maxCand[ORC_MSE_MAX_EDGES + 1];
    float centers[ORC_MSE_MAX_EDGES], pdfAt[ORC_MSE_MAX_EDGES];
    int numEdges = 0;
    edges[numEdges++] = minVal;
    int walked        = 0;
    for (float i = histMin; i <= histMax && walked < ORC_MSE_MAX_WALK; i += histBinWidth, ++walked)
        if (i >= minVal && i <= maxVal)
            edges[numEdges++] = i;

    int numMin = 0, numMax = 0;
    for (int k = 0; k < numEdges; ++k)
    {
        if (edges[k] < 0)
            minCand[numMin++] = edges[k];
        else if (edges[k] > 0)
            maxCand[numMax++] = edges[k];
    }
    minCand[numMin++] = 0;
    maxCand[numMax++] = 0;

    float pdfStart          = (float) p->xLeft[0];
    float pdfStep           = (float) (p->xLeft[1] - p->xLeft[0]);
    const int numBinCenters = numEdges - 1;
    for (int i = 0; i < numBinCenters; ++i)
    {
        centers[i] = (i == 0) ? minVal + histBinWidth / 2 : centers[i - 1] + histBinWidth;
        int ind    = orc_double_to_int(floorf((centers[i] - pdfStart) / pdfStep));
        ind        = STD_MIN(STD_MAX(0, ind), ORC_PDF_SIZE - 1);
        pdfAt[i]   = (float) p->pdf[ind];
    }

    float mseMin = FLT_MAX;
    *bestMin     = minVal;
    *bestMax     = maxVal;
    for (int i = 0; i < numMin; ++i)
        for (int j = 0; j < numMax; ++j)
        {
            if (i == numMin - 1 && j == numMax - 1)
                break; /* {0, 0} is no candidate */
            float mse = orc_mse_cost(bw, centers, pdfAt, numBinCenters, minCand[i], maxCand[j], sym, strict,
                                     unsignedSym);
            if (mse < mseMin)
            {
                mseMin   = mse;
                *bestMin = minCand[i];
                *bestMax = maxCand[j];
            }
        }
    if (counts)
    {
        counts[0] = numMin;
        counts[1] = numMax;
        counts[2] = numBinCenters;
    }
    if (minCandOut)
        memcpy(minCandOut, minCand, sizeof(float) * (size_t) numMin);
    if (maxCandOut)
        memcpy(maxCandOut, maxCand, sizeof(float) * (size_t) numMax);
    if (centersOut)
        memcpy(centersOut, centers, sizeof(float) * (size_t) (numBinCenters > 0 ? numBinCenters : 0));
}

/* computeEncoding, :78-130 */
void orc_mse_compute_encoding(const orc_pdf* p, int bw, int sym, int strict, int unsignedSym, orc_encoding* e)
{
    memset(e, 0, sizeof(*e));
    float numSteps = (float) (pow(2, bw) - 1);
    if (sym && strict)
        numSteps -= 1;
    if (!p->initialized)
    {
        if (p->stats_updated)
        {
            e->min    = -1;
            e->max    = 1;
            e->delta  = (e->max - e->min) / (int) numSteps;
            e->offset = floor(e->min / e->delta);
            e->min    = e->offset * e->delta;
            e->max    = e->min + (int) numSteps * e->delta;
            e->bw     = bw;
        }
        return;
    }
    float aMin, aMax;
    orc_mse_minimize(p, bw, sym, strict, unsignedSym, &aMin, &aMax, NULL, NULL, NULL, NULL);
    aMin = STD_MIN(aMin, 0.0f);
    aMax = STD_MAX(aMax, 0.0f);
    orc_get_computed_encodings(bw, aMin, aMax, sym, strict, unsignedSym, e);
}

/* ------------------------------------------------------------------------------------------------------------
 * Entropy (KL divergence) calibration: EntropyEncodingAnalyzer<float> (DLQ/src/EntropyEncodingAnalyzer.cpp:54-436)
 * over the rescaling 512-bin histogram of updateTensorHistogram_cpu / rescaleHistogram
 * (DLQ/src/math_functions.cpp:468-643).  The histogram spans exactly the range seen so far and is redistributed
 * when a batch widens it; only for 8 bits is the range then narrowed, window by window, to the one whose 255-level
 * quantization has the least KL divergence from the saturated histogram.
 * Data are taken to be finite (the reference's bin index of a NaN or infinite sample is whatever the conversion of an
 * out-of-range float to size_t yields).
 * ---------------------------------------------------------------------------------------------------------- */
typedef struct
{
    double min, max;
    double histogram[ORC_PDF_SIZE];
    int iterations;
    int initialized;   /* histogram.size() != 0 in the reference */
    int stats_updated; /* _statsUpdated */
} orc_tensor_profile;  /* TensorProfilingParams, DLQ/src/math_functions.hpp:69-77 + EntropyEncodingAnalyzer.h */

void orc_profile_reset(orc_tensor_profile* t)
{
    memset(t, 0, sizeof(*t));
}

/* getBin, math_functions.cpp:468-474: float arithmetic, the quotient truncated to size_t and capped at the last bin */
static size_t orc_get_bin(size_t nBins, float binWidth, float minValue, float value)
{
    if (binWidth == 0)
        return 0;
    float q = (value - minValue) / binWidth;
    if (!(q < (float) nBins) || q <= -1.0f)
        return nBins - 1;
    return (size_t) q;
}

/* std::accumulate(first, last, 0.f): the accumulator has the type of the initial value, float */
static double orc_accumulate_in_float(const double* v, size_t n)
{
    float acc = 0.f;
    for (size_t i = 0; i < n; ++i)
        acc = (float) (acc + v[i]);
    return acc;
}

/* updateTensorHistogram_cpu, math_functions.cpp:476-560 */
void orc_profile_update_f32(orc_tensor_profile* t, const float* data, int64_t n)
{
    t->stats_updated = 1;
    float mnf, mxf;
    orc_minmax_f32(data, n, &mnf, &mxf);
    double minInput = mnf, maxInput = mxf;
    if (minInput == 0 && maxInput == 0)
        return;
    if (minInput == maxInput)
    {
        double widened = minInput + (float) 0.01;
        maxInput       = STD_MAX(maxInput, widened);
    }
    if (!t->initialized)
    {
        memset(t->histogram, 0, sizeof(t->histogram));
        t->min         = minInput;
        t->max         = maxInput;
        t->initialized = 1;
    }
    if (minInput < t->min || maxInput > t->max)
    {
        double newMin       = STD_MIN(minInput, t->min);
        double newMax       = STD_MAX(maxInput, t->max);
        double destBinWidth = (newMax - newMin) / ORC_PDF_SIZE;
        double srcBinWidth  = (t->max - t->min) / ORC_PDF_SIZE;
        double scaled[ORC_PDF_SIZE];
        memset(scaled, 0, sizeof(scaled));
        for (size_t i = 0; i < ORC_PDF_SIZE; ++i)
        {
            if (t->histogram[i] == 0)
                continue;
            double srcBinBegin = t->min + srcBinWidth * i;
            size_t destBin     = (size_t) ((srcBinBegin - newMin) / destBinWidth);
            double destBinEnd  = newMin + destBinWidth * (destBin + 1);
            double share       = round((destBinEnd - srcBinBegin) / srcBinWidth * t->histogram[i]);
            double dstBinCnt   = STD_MIN(share, t->histogram[i]);
            size_t newBin      = orc_get_bin(ORC_PDF_SIZE, (float) destBinWidth, (float) newMin, (float) srcBinBegin);
            scaled[newBin] += dstBinCnt;
            if (dstBinCnt < t->histogram[i])
            {
                newBin = orc_get_bin(ORC_PDF_SIZE, (float) destBinWidth, (float) newMin,
                                     (float) (srcBinBegin + destBinWidth));
                scaled[newBin] += t->histogram[i] - dstBinCnt;
            }
        }
        memcpy(t->histogram, scaled, sizeof(scaled));
        t->min = newMin;
        t->max = newMax;
    }
    float binWidth = (float) ((t->max - t->min) / ORC_PDF_SIZE);
    for (int64_t i = 0; i < n; ++i)
        t->histogram[orc_get_bin(ORC_PDF_SIZE, binWidth, (float) t->min, data[i])] += 1;
    t->iterations++;
}

/* rescaleHistogram, math_functions.cpp:562-643 */
static void orc_rescale_histogram(const double* srcHist, double srcHistMin, double srcHistMax, double destHistMin,
                                  double destHistMax, double* destHist)
{
    const size_t numBins = ORC_PDF_SIZE;
    if (srcHistMin == destHistMin && srcHistMax == destHistMax)
    {
        memcpy(destHist, srcHist, sizeof(double) * numBins);
        return;
    }
    const double srcBinWidth  = (srcHistMax - srcHistMin) / numBins;
    const double destBinWidth = (destHistMax - destHistMin) / numBins;
    memset(destHist, 0, sizeof(double) * numBins);
    for (size_t srcBinIdx = 0; srcBinIdx < numBins; srcBinIdx++)
    {
        double srcBinVal = srcHist[srcBinIdx];
        if (srcBinVal == 0)
            continue;
        double srcBinStart     = srcHistMin + srcBinIdx * srcBinWidth;
        double srcBinStop      = srcHistMin + (srcBinIdx + 1) * srcBinWidth;
        double dstBinIdxStartF = floor((srcBinStart - destHistMin) / destBinWidth);
        double dstBinIdxStopF  = ceil((srcBinStop - destHistMin) / destBinWidth);
        size_t dstBinIdxStart  = (size_t) STD_MAX(dstBinIdxStartF, 0.0);
        size_t dstBinIdxStop   = (size_t) STD_MAX(dstBinIdxStopF, 0.0);
        if (dstBinIdxStart >= numBins)
            dstBinIdxStart = numBins - 1;
        if (dstBinIdxStop >= numBins)
            dstBinIdxStop = numBins - 1;
        double srcBinRem = srcBinVal;
        for (size_t destBinIdx = dstBinIdxStart; destBinIdx <= dstBinIdxStop; destBinIdx++)
        {
            double destBinStart = destHistMin + destBinIdx * destBinWidth;
            double destBinStop  = destHistMin + (destBinIdx + 1) * destBinWidth;
            double overlapStart = STD_MAX(srcBinStart, destBinStart);
            double overlapStop  = STD_MIN(srcBinStop, destBinStop);
            double overlapRatio = (overlapStop - overlapStart) / srcBinWidth;
            overlapRatio        = overlapRatio >= 0.0f ? overlapRatio : 0.0f;
            overlapRatio        = overlapRatio <= 1.0f ? overlapRatio : 1.0f;
            double distVal      = round(overlapRatio * srcBinVal);
            distVal             = distVal <= srcBinRem ? distVal : srcBinRem;
            destHist[destBinIdx] += distVal;
            srcBinRem -= distVal;
        }
    }
}

/* _conditionHistogram, EntropyEncodingAnalyzer.cpp:153-200 */
static void orc_condition_histogram(double* hist, size_t length)
{
    const double epsZero = 0.0001;
    if (length == 0)
        return;
    size_t numZeros = 0;
    for (size_t i = 0; i < length; ++i)
        numZeros += (hist[i] == 0.f);
    if (numZeros == length)
        return;
    size_t numNonZeros = length - numZeros;
    double epsNonZero  = epsZero * (double) numZeros / (double) numNonZeros;
    if (epsNonZero >= 1.0)
        return;
    for (size_t i = 0; i < length; ++i)
    {
        int isZero = (hist[i] == 0.f);
        hist[i] += epsZero * isZero;
        hist[i] -= epsNonZero * (1 - isZero);
    }
}

/* _computeKL, :202-228 (P and Q are normalised in place) */
static double orc_compute_kl(double* P, double* Q, size_t length)
{
    double sumP       = orc_accumulate_in_float(P, length);
    double sumQ       = orc_accumulate_in_float(Q, length);
    double divergence = 0;
    for (size_t i = 0; i < length; ++i)
    {
        P[i] /= sumP;
        Q[i] /= sumQ;
        if (P[i] > 0 && Q[i] > 0)
            divergence += P[i] * log(P[i] / Q[i]);
    }
    return divergence;
}

/* _optimizeKL, :230-431.  divergences (optional, ORC_PDF_SIZE doubles) receives the divergence of every window
 * tried, in order; *numWindows their count. */
void orc_entropy_optimize_kl(const orc_tensor_profile* t, int bw, int sym, int strict, int unsignedSym, float* minOut,
                             float* maxOut, double* divergences, int* numWindows)
{
    double histMin = t->min, histMax = t->max;
    double hist[ORC_PDF_SIZE];
    if (numWindows)
        *numWindows = 0;
    if (sym && (histMin < 0.0 || !unsignedSym))
    {
        double absHi      = fabs(histMax), absLo = fabs(histMin);
        float absoluteMax = (float) STD_MAX(absHi, absLo);
        float absoluteMin = -absoluteMax;
        orc_rescale_histogram(t->histogram, histMin, histMax, absoluteMin, absoluteMax, hist);
        histMin = absoluteMin;
        histMax = absoluteMax;
    }
    else
        memcpy(hist, t->histogram, sizeof(hist));

    const size_t numBins          = ORC_PDF_SIZE;
    const size_t numQuantizedBins = 255;
    if (bw != 8)
    {
        *minOut = (float) histMin;
        *maxOut = (float) histMax;
        return;
    }
    const double histBinWidth = (histMax - histMin) / (double) numBins;
    double divergenceOpt      = INFINITY;
    double thresholdMinOpt = histMin, thresholdMaxOpt = histMax;
    size_t start = 0, stop = numBins - 1;
    double P[ORC_PDF_SIZE], Q[ORC_PDF_SIZE];
    while ((stop - start + 1) >= numQuantizedBins)
    {
        const size_t winSize = stop - start + 1;
        const double* win    = hist + start;
        memset(P, 0, sizeof(double) * winSize);
        double leftSum = 0;
        for (size_t i = 0; i <= start; i++)
            leftSum += hist[i];
        P[0] += leftSum;
        for (size_t i = start + 1; i < stop; i++)
            P[i - start] = hist[i];
        double rightSum = 0;
        for (size_t i = stop; i < numBins; i++)
            rightSum += hist[i];
        P[winSize - 1] += rightSum;

        const double numMergedBins = (double) winSize / (double) numQuantizedBins;
        memset(Q, 0, sizeof(double) * winSize);
        for (size_t q = 0; q < numQuantizedBins; q++)
        {
            const size_t idxStart = (size_t) ceil(q * numMergedBins);
            const size_t idxStop  = (q < numQuantizedBins - 1) ? (size_t) ceil((q + 1) * numMergedBins) : winSize;
            double sum = 0, norm = 0;
            for (size_t i = idxStart; i < idxStop; i++)
            {
                sum += win[i];
                norm += (win[i] != 0);
            }
            if (norm != 0)
                for (size_t i = idxStart; i < idxStop; i++)
                    if (win[i])
                        Q[i] = sum / norm;
        }
        double sumP = orc_accumulate_in_float(P, winSize);
        double sumQ = orc_accumulate_in_float(Q, winSize);
        if (sumP == 0 || sumQ == 0)
            break;
        orc_condition_histogram(P, winSize);
        orc_condition_histogram(Q, winSize);
        double divergence = orc_compute_kl(P, Q, winSize);
        if (divergences && numWindows && *numWindows < ORC_PDF_SIZE)
            divergences[(*numWindows)++] = divergence;
        if (divergence < divergenceOpt)
        {
            divergenceOpt   = divergence;
            thresholdMinOpt = histMin + start * histBinWidth;
            thresholdMaxOpt = histMin + (stop + 1) * histBinWidth;
        }
        if (sym || strict)
        {
            start++;
            stop--;
        }
        else
        {
            double loss[3] = {hist[start] + hist[stop], hist[start] + hist[start + 1], hist[stop] + hist[stop - 1]};
            int lossMinIdx = 0; /* std::min_element: the first of equal minima */
            for (int k = 1; k < 3; ++k)
                if (loss[k] < loss[lossMinIdx])
                    lossMinIdx = k;
            if ((lossMinIdx == 0 && (histMin + (start + 1) * histBinWidth) > 0) ||
                (lossMinIdx == 1 && (histMin + (start + 2) * histBinWidth) > 0))
                lossMinIdx = 2;
            else if ((lossMinIdx == 0 && (histMin + stop * histBinWidth) < 0) ||
                     (lossMinIdx == 2 && (histMin + (stop - 1) * histBinWidth) < 0))
                lossMinIdx = 1;
            if (lossMinIdx == 0)
            {
                start++;
                stop--;
            }
            else if (lossMinIdx == 1)
                start += 2;
            else
                stop -= 2;
        }
    }
    *minOut = (float) thresholdMinOpt;
    *maxOut = (float) thresholdMaxOpt;
}

/* computeEncoding, :97-146 */
void orc_entropy_compute_encoding(const orc_tensor_profile* t, int bw, int sym, int strict, int unsignedSym,
                                  orc_encoding* e)
{
    memset(e, 0, sizeof(*e));
    float numSteps = (float) (pow(2, bw) - 1);
    if (sym && strict)
        numSteps -= 1;
    if (!t->initialized)
    {
        if (t->stats_updated)
        {
            e->min    = -1;
            e->max    = 1;
            e->delta  = (e->max - e->min) / (int) numSteps;
            e->offset = floor(e->min / e->delta);
            e->min    = e->offset * e->delta;
            e->max    = e->min + (int) numSteps * e->delta;
            e->bw     = bw;
        }
        return;
    }
    float aMin, aMax;
    orc_entropy_optimize_kl(t, bw, sym, strict, unsignedSym, &aMin, &aMax, NULL, NULL);
    aMin = STD_MIN(aMin, 0.0f);
    aMax = STD_MAX(aMax, 0.0f);
    orc_get_computed_encodings(bw, aMin, aMax, sym, strict, unsignedSym, e);
}

/* ------------------------------------------------------------------------------------------------------------
 * a7  v2 quantize-dequantize (TORCH/v2/quantization/affine/backends/torch_builtins.py:303-344), float32 internal
 * dtype.  scale/offset are per "channel" with channel = (i / numElementPerChannel) % numChannel, which covers the
 * per-tensor ([1]) and per-output-channel ([C,1,...]) broadcast shapes.  torch.round is half-to-even (rintf under
 * the default rounding mode).  maskOut (optional) receives 1 where qmin <= round(x/s) - o <= qmax.
 * ---------------------------------------------------------------------------------------------------------- */
void orc_v2_qdq_f32(const float* in, int64_t numChannel, int64_t numElement, int64_t numElementPerChannel,
                    float* out, float* codesOut, uint8_t* maskOut, const float* scale, const float* offset, int qmin,
                    int qmax)
{
    for (int64_t i = 0; i < numElement; ++i)
    {
        int64_t c  = (i / numElementPerChannel) % numChannel;
        float r    = rintf(in[i] / scale[c]) - offset[c];
        int inside = ((float) qmin <= r) && (r <= (float) qmax);
        float q    = r;
        if (q < (float) qmin)
            q = (float) qmin;
        if (q > (float) qmax)
            q = (float) qmax;
        if (codesOut)
            codesOut[i] = q;
        if (maskOut)
            maskOut[i] = (uint8_t) inside;
        if (out)
            out[i] = (q + offset[c]) * scale[c];
    }
}

void orc_v2_qdq_bf16(const uint16_t* in, int64_t numChannel, int64_t numElement, int64_t numElementPerChannel,
                     uint16_t* out, uint8_t* maskOut, const float* scale, const float* offset, int qmin, int qmax)
{
    for (int64_t i = 0; i < numElement; ++i)
    {
        int64_t c  = (i / numElementPerChannel) % numChannel;
        float r    = rintf(orc_bf16_to_f32(in[i]) / scale[c]) - offset[c];
        int inside = ((float) qmin <= r) && (r <= (float) qmax);
        float q    = r;
        if (q < (float) qmin)
            q = (float) qmin;
        if (q > (float) qmax)
            q = (float) qmax;
        if (maskOut)
            maskOut[i] = (uint8_t) inside;
        out[i] = orc_f32_to_bf16((q + offset[c]) * scale[c]);
    }
}

/* torch_builtins.py:329-344: tensor_grad = grad * mask */
void orc_v2_qdq_bwd_f32(const float* in, const float* gout, int64_t numChannel, int64_t numElement,
                        int64_t numElementPerChannel, float* gin, const float* scale, const float* offset, int qmin,
                        int qmax)
{
    for (int64_t i = 0; i < numElement; ++i)
    {
        int64_t c  = (i / numElementPerChannel) % numChannel;
        float r    = rintf(in[i] / scale[c]) - offset[c];
        int inside = ((float) qmin <= r) && (r <= (float) qmax);
        gin[i]     = gout[i] * (float) inside;
    }
}

/* torch_builtins.py:329-344, all three gradients of QuantDequantFunc:
 *   scale_grad  = grad * (clamp(round(x/s), o+qmin, o+qmax) - (x/s) * mask)
 *   offset_grad = grad * (~mask * s)
 * each element term in float32 as the reference forms it; the reduction to the parameter shape, which the reference
 * leaves to autograd's float32 sum (order unspecified), is done here in double.  gin may be NULL. */
void orc_v2_qdq_bwd_params_f32(const float* in, const float* gout, int64_t numChannel, int64_t numElement,
                               int64_t numElementPerChannel, float* gin, const float* scale, const float* offset,
                               int qmin, int qmax, double* scaleGrad, double* offsetGrad)
{
    for (int64_t c = 0; c < numChannel; ++c)
        scaleGrad[c] = offsetGrad[c] = 0.0;
    for (int64_t i = 0; i < numElement; ++i)
    {
        int64_t c  = (i / numElementPerChannel) % numChannel;
        float q    = in[i] / scale[c];
        float r    = rintf(q);
        float rm   = r - offset[c];
        int inside = ((float) qmin <= rm) && (rm <= (float) qmax);
        float lo   = offset[c] + (float) qmin;
        float hi   = offset[c] + (float) qmax;
        float cl   = r;
        if (cl < lo)
            cl = lo;
        if (cl > hi)
            cl = hi;
        float masked = q * (float) inside;
        float ts     = gout[i] * (cl - masked);
        float notm   = (float) (!inside) * scale[c];
        float to     = gout[i] * notm;
        scaleGrad[c] += (double) ts;
        offsetGrad[c] += (double) to;
        if (gin)
            gin[i] = gout[i] * (float) inside;
    }
}
