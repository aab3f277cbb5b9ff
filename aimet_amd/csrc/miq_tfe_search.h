// TF-Enhanced (SQNR) delta/offset candidate search over a 512-bucket PDF: the pieces one wavefront runs for one
// candidate, shared by the single-tensor analyzer and the per-channel (batched) one.
//
// Reference arithmetic (DLQ = ModelOptimizations/DlQuantization): DLQ/src/TfEnhancedEncodingAnalyzer.cpp:78-397, with
// DTYPE = float; every float / double / int conversion below is the reference's.
#ifndef MIQ_TFE_SEARCH_H
#define MIQ_TFE_SEARCH_H

#include <hip/hip_runtime.h>

#include <cfloat>
#include <climits>
#include <cmath>

#include "../../include/miq.h"
#include "miq_fastmath.h"

namespace miq
{
namespace tfe
{
constexpr int kBuckets = MIQ_PDF_SIZE;

// (int) of a floating-point value as the reference's x86-64 build performs it (cvttsd2si / cvttss2si): truncation
// inside the int range, INT_MIN for everything else, NaN included.  The C++ cast is undefined there and this GPU's
// conversion saturates instead; the difference decides a cost when a candidate range is more than 2^31 PDF buckets wide
// (data spanning less than about 1e-12 against the 1e-5 minimum encoding range).
__device__ __forceinline__ int cvtt_x86(double v)
{
    return (v >= -2147483648.0 && v < 2147483648.0) ? (int) v : INT_MIN;
}

struct SearchArgs
{
    int bw;
    int sym, strict, uns;
    float num_steps_cand;   // 2^bw - 1, minus 1 for strict symmetric (candidate generation and final min/max)
    float step_size_cost;   // 2^bw - 1 (the cost function never reduces it)
    int n_cand;             // grid size: 17*21 + 1 asymmetric, number of float steps of 0.01 symmetric
    int n_delta;            // 17 or the symmetric count
};

// Host: the candidate grid of a search.
inline SearchArgs make_search_args(int bw, int use_symmetric, int use_strict_symmetric, int use_unsigned_symmetric)
{
    SearchArgs sa{};
    sa.bw             = bw;
    sa.sym            = use_symmetric ? 1 : 0;
    sa.strict         = use_strict_symmetric ? 1 : 0;
    sa.uns            = use_unsigned_symmetric ? 1 : 0;
    sa.step_size_cost = (float) (std::pow(2, bw) - 1);
    sa.num_steps_cand = sa.step_size_cost;
    if (sa.sym && sa.strict)
        sa.num_steps_cand -= 1;
    int cnt = 0;
    if (sa.sym)
    {
        // the delta factor advances by adding the double 0.01 to a float; how many steps fit below 1.01 is decided
        // by that float arithmetic (DLQ/src/TfEnhancedEncodingAnalyzer.cpp:248)
        for (float f = (float) (1.0 / 100); (double) f <= 1 + 1.0 / 100; f = (float) ((double) f + 1.0 / 100))
            ++cnt;
        sa.n_delta = cnt;
        sa.n_cand  = cnt;
    }
    else
    {
        for (float f = (float) (1.0 / 16); (double) f <= 1 + 1.0 / 16; f = (float) ((double) f + 1.0 / 16))
            ++cnt;
        sa.n_delta = cnt;
        sa.n_cand  = cnt * 21 + 1;
    }
    return sa;
}

__device__ __forceinline__ float std_max(float a, float b)
{
    return (a < b) ? b : a;   // std::max(a, b)
}
__device__ __forceinline__ float std_min(float a, float b)
{
    return (b < a) ? b : a;   // std::min(a, b)
}

// Sum of term[lo..hi) in ascending index order.  Eight loads are issued ahead of the eight dependent adds.
__device__ __forceinline__ double ordered_sum(const double* term, int lo, int hi)
{
    double acc = 0;
    int i      = lo;
    for (; i + 8 <= hi; i += 8)
    {
        double t[8];
#pragma unroll
        for (int k = 0; k < 8; ++k)
            t[k] = term[i + k];
#pragma unroll
        for (int k = 0; k < 8; ++k)
            acc += t[k];
    }
    for (; i < hi; ++i)
        acc += term[i];
    return acc;
}

// The PDF a search reads: 512 running values and the left edges x_left[i] = min_val + i * bucket (a float plus a
// double product, the expression InitializePdf stores: DLQ/src/math_functions.cpp:232-236).
struct PdfView
{
    const double* pdf;
    float min_val;
    double bucket;
    __device__ __forceinline__ double x_left(int i) const
    {
        return min_val + i * bucket;
    }
};

// Range of the aggregate stats, DLQ/src/TfEnhancedEncodingAnalyzer.cpp:255-291.  Wavefront-wide (64 lanes).
__device__ __forceinline__ void wave_range(const PdfView& v, int lane, float& minVal, float& maxVal)
{
    int first = -1, last = -1;
#pragma unroll
    for (int k = 0; k < kBuckets / 64; ++k)
    {
        const uint64_t m = __ballot(v.pdf[k * 64 + lane] > 0);
        if (m)
        {
            if (first < 0)
                first = k * 64 + __builtin_ctzll(m);
            const uint64_t m1 = (k == 0) ? (m & ~1ull) : m;   // the downward scan stops above bucket 0
            if (m1)
                last = k * 64 + 63 - __builtin_clzll(m1);
        }
    }
    minVal = (float) v.x_left(first < 0 ? 0 : first);
    maxVal = (float) v.x_left(last < 0 ? kBuckets - 1 : last);
    minVal = std_min(minVal, 0.0f);
    maxVal = std_max(maxVal, 0.0f);
    maxVal = std_max(maxVal, minVal + (float) 0.01);
}

// Candidate number `cand` of the grid; false when the reference would not have kept it.
__device__ __forceinline__ bool candidate(const SearchArgs& a, float minVal, float maxVal, int cand, float& delta,
                                          int& offset)
{
    delta      = 0.f;
    offset     = 0;
    bool valid = true;
    const float numSteps = a.num_steps_cand;
    if (a.sym)
    {
        // DLQ/src/TfEnhancedEncodingAnalyzer.cpp:216-253
        float deltaMax;
        if ((minVal == 0.0) && a.uns)
        {
            deltaMax = maxVal / numSteps;
            offset   = 0;
        }
        else
        {
            const float absMax = std_max(fabsf(maxVal), fabsf(minVal));
            deltaMax           = (float) (absMax / (numSteps / 2.0));
            offset             = (int) floorf(-numSteps / 2);
        }
        float f = (float) (1.0 / 100);
        for (int k = 0; k < cand; ++k)
            f = (float) ((double) f + 1.0 / 100);
        delta = f * deltaMax;
    }
    else
    {
        // DLQ/src/TfEnhancedEncodingAnalyzer.cpp:177-214
        const float obsDelta = (float) (((double) maxVal - (double) minVal) / numSteps);
        const int obsOffset  = (int) roundf(minVal / obsDelta);
        const float obsMin   = std_max(obsDelta * (float) obsOffset, -FLT_MAX);
        const float obsMax   = std_min(obsDelta * ((float) obsOffset + numSteps), FLT_MAX);
        if (cand == a.n_cand - 1)
        {
            delta  = obsDelta;
            offset = obsOffset;
        }
        else
        {
            const int fi = cand / 21, oi = cand % 21;
            float f = (float) (1.0 / 16);
            for (int k = 0; k < fi; ++k)
                f = (float) ((double) f + 1.0 / 16);
            delta  = f * obsDelta;
            offset = (int) ((double) (-numSteps) + (double) numSteps / 20.0 * oi);
            // clamp to the observed range: DLQ/src/TfEnhancedEncodingAnalyzer.cpp:149-175
            float tMin = std_max(delta * (float) offset, -FLT_MAX);
            float tMax = std_min(delta * ((float) offset + numSteps), FLT_MAX);
            if ((tMin < obsMin) && (tMax > obsMax))
                valid = false;
            else
            {
                tMin = std_max(obsMin, tMin);
                tMax = std_min(obsMax, tMax);
                if (tMin == tMax)
                    valid = false;
                else
                {
                    delta  = (float) (((double) tMax - tMin) / numSteps);
                    offset = (int) roundf(tMin / delta);
                }
            }
        }
    }
    return valid;
}

// Cost of one candidate, DLQ/src/TfEnhancedEncodingAnalyzer.cpp:293-355.  Wavefront-wide: lanes evaluate the per-bucket
// error terms in parallel into `term` (this wavefront's kBuckets doubles of LDS); the three sums are then accumulated
// in ascending bucket order, the order of the reference's loops, so that costs are bit-identical to the CPU result and
// ties between candidates resolve identically.  Every lane runs the same chain (uniform bounds, LDS broadcast reads).
__device__ __forceinline__ double wave_cost(const PdfView& v, const SearchArgs& a, float delta, int offset, int lane,
                                            double* term)
{
    const float cMin      = delta * (float) offset;
    const float stepSize  = a.step_size_cost;
    const float cMax      = delta * ((float) offset + stepSize);
    const float pdfStart  = (float) v.x_left(0);
    const double pdfStep  = v.x_left(1) - v.x_left(0);
    int minInd            = cvtt_x86(floor((cMin - pdfStart) / pdfStep));
    minInd                = minInd < 0 ? 0 : (minInd > kBuckets - 1 ? kBuckets - 1 : minInd);
    int maxInd            = cvtt_x86(floor((cMax - pdfStart) / pdfStep));
    maxInd                = maxInd < 0 ? 0 : (maxInd > kBuckets - 1 ? kBuckets - 1 : maxInd);
    const float minMid    = (float) (pdfStart + (minInd * pdfStep) + pdfStep / 2);
    const float maxMid    = (float) (pdfStart + (maxInd * pdfStep) + pdfStep / 2);
#pragma unroll
    for (int k = 0; k < kBuckets / 64; ++k)
    {
        const int i      = k * 64 + lane;
        const double p   = v.pdf[i];
        const double mid = pdfStart + i * pdfStep + pdfStep / 2;
        double t;
        if (i < minInd)
        {
            const double d = mid - minMid;
            t              = p * (d * d);
        }
        else if (i >= maxInd)
        {
            const double d = mid - maxMid;
            t              = p * (d * d);
        }
        else
        {
            const float fv   = (float) mid;
            const int q      = cvtt_x86((double) roundf(fv / delta - (float) offset));
            const float dq   = delta * (float) (q + offset);
            const double d   = (double) (fv - dq);
            t                = p * (d * d);
        }
        term[i] = t;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);   // LDS writes of this wavefront have landed (lgkmcnt = 0)
    const double satBottom = ordered_sum(term, 0, minInd);
    double satTop          = ordered_sum(term, maxInd, kBuckets);
    const double quant     = ordered_sum(term, minInd, maxInd);
    if (maxInd < minInd)
    {
        // Only after an index conversion left the int range (cvtt_x86).  The reference's three loops then
        // overlap: buckets [maxInd, minInd) are saturation at the bottom AND at the top, and no bucket is
        // quantization noise.  Redo the top sum with every bucket's distance to the top mid-point.
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int k = 0; k < kBuckets / 64; ++k)
        {
            const int i      = k * 64 + lane;
            const double mid = pdfStart + i * pdfStep + pdfStep / 2;
            const double d   = mid - maxMid;
            term[i]          = v.pdf[i] * (d * d);
        }
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0xc07f);
        satTop = ordered_sum(term, maxInd, kBuckets);
    }
    __builtin_amdgcn_wave_barrier();   // the next candidate of this wavefront overwrites `term`
    double cost = 3.0 * (satBottom + satTop) + quant;
    return (cost < DBL_MAX) ? cost : DBL_MAX;   // std::min(sqnr, max())
}

// The same cost with one candidate per LANE: a lane walks the buckets in ascending order and keeps the three running
// sums itself, so a wavefront prices 64 candidates at once and nothing is exchanged between lanes.  Each sum receives
// the terms wave_cost() adds, in the same order, so the two functions agree bit for bit (wave_cost()'s overlap case
// included: a bucket below minInd and at or above maxInd enters both saturation sums, none enters the noise sum).
// The three sums are three loops, each over the buckets that at least one lane of the wavefront needs (the bounds are
// reduced over the wavefront, so they are uniform), with the lanes outside their own range masked off.
// pdf_s / mid_s / fmid_s: the PDF, the bucket mid-points and their binary32 values (stage_pdf()), read as LDS
// broadcasts.  Every lane of the wavefront must call lane_cost(); lanes without a candidate pass active = false.
//
// Three steps of the noise term have cheaper sequences with the same result: the division through
// div_by_invariant() where its contract holds (a quotient below its 2^-36 limit vanishes in the subtraction of the
// integer offset, or rounds to zero without one), roundf through round_half_away(), and the x86 conversion of the
// rounded value straight from binary32 (it is an integer, an infinity or NaN there, so the detour through double
// changes nothing; where |mid / delta| + |offset| stays below 2^30 for every bucket the range test is dropped too).
// A wavefront uses them when all its lanes can.
__device__ __forceinline__ void stage_pdf(const PdfView& v, double* pdf_s, double* mid_s, float* fmid_s, int tid,
                                          int nthreads)
{
    const float pdfStart = (float) v.x_left(0);
    const double pdfStep = v.x_left(1) - v.x_left(0);
    for (int i = tid; i < kBuckets; i += nthreads)
    {
        const double mid = pdfStart + i * pdfStep + pdfStep / 2;
        pdf_s[i]         = v.pdf[i];
        mid_s[i]         = mid;
        fmid_s[i]        = (float) mid;
    }
}
__device__ __forceinline__ int cvtt_x86_of_rounded(float r)
{
    return (r >= -2147483648.0f && r < 2147483648.0f) ? (int) r : INT_MIN;
}
__device__ __forceinline__ int wave_min_int(int v)
{
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
    {
        const int o = __shfl_xor(v, m);
        v           = o < v ? o : v;
    }
    return __builtin_amdgcn_readfirstlane(v);
}
// Sum of p * d^2 over the buckets [from, to) of this lane, d = mid - ref, inside the wavefront's loop [begin, end).
__device__ __forceinline__ double saturation_sum(const double* pdf_s, const double* mid_s, int begin, int end, int from,
                                                 int to, float ref)
{
    double acc = 0;
#pragma unroll 4
    for (int i = begin; i < end; ++i)
        if (i >= from && i < to)
        {
            const double d = mid_s[i] - ref;
            acc += pdf_s[i] * (d * d);
        }
    return acc;
}
template <bool SHORT>
__device__ __forceinline__ double noise_sum(const double* pdf_s, const float* fmid_s, int begin, int end, int from,
                                            int to, float delta, float rcp, int offset)
{
    const float foffset = (float) offset;
    double acc          = 0;
#pragma unroll 4
    for (int i = begin; i < end; ++i)
        if (i >= from && i < to)
        {
            const float fv = fmid_s[i];
            int q;
            if (SHORT)
                q = (int) round_half_away(div_by_invariant(fv, delta, rcp) - foffset);
            else
                q = cvtt_x86_of_rounded(round_half_away(fv / delta - foffset));
            const float dq = delta * (float) (q + offset);
            const double d = (double) (fv - dq);
            acc += pdf_s[i] * (d * d);
        }
    return acc;
}
__device__ __forceinline__ double lane_cost(const PdfView& v, const double* pdf_s, const double* mid_s,
                                            const float* fmid_s, const SearchArgs& a, bool active, float delta,
                                            int offset)
{
    const float foffset   = (float) offset;
    const float cMin      = delta * foffset;
    const float stepSize  = a.step_size_cost;
    const float cMax      = delta * (foffset + stepSize);
    const float pdfStart  = (float) v.x_left(0);
    const double pdfStep  = v.x_left(1) - v.x_left(0);
    int minInd            = cvtt_x86(floor((cMin - pdfStart) / pdfStep));
    minInd                = minInd < 0 ? 0 : (minInd > kBuckets - 1 ? kBuckets - 1 : minInd);
    int maxInd            = cvtt_x86(floor((cMax - pdfStart) / pdfStep));
    maxInd                = maxInd < 0 ? 0 : (maxInd > kBuckets - 1 ? kBuckets - 1 : maxInd);
    const float minMid    = (float) (pdfStart + (minInd * pdfStep) + pdfStep / 2);
    const float maxMid    = (float) (pdfStart + (maxInd * pdfStep) + pdfStep / 2);
    // this lane's three ranges (empty without a candidate) and the wavefront's
    const int bottom_to  = active ? minInd : 0;
    const int top_from   = active ? maxInd : kBuckets;
    const int noise_from = active ? minInd : kBuckets;
    const int noise_to   = active ? maxInd : 0;
    const int w_bottom_to  = -wave_min_int(-bottom_to);
    const int w_top_from   = wave_min_int(top_from);
    const int w_noise_from = wave_min_int(noise_from);
    const int w_noise_to   = -wave_min_int(-noise_to);
    // the mid-points grow with the bucket number: the end ones bound the dividends
    const float far      = fmaxf(fabsf(fmid_s[0]), fabsf(fmid_s[kBuckets - 1]));
    const bool can_short = fastdiv_divisor_ok(delta) && far <= kFastDivMaxDividend &&
                           far / delta + fabsf(foffset) < 1073741824.0f;
    const bool all_short = wave_min_int((can_short || !active) ? 1 : 0) != 0;
    const float rcp      = 1.0f / delta;

    const double satBottom = saturation_sum(pdf_s, mid_s, 0, w_bottom_to, 0, bottom_to, minMid);
    const double satTop    = saturation_sum(pdf_s, mid_s, w_top_from, kBuckets, top_from, kBuckets, maxMid);
    const double quant =
        all_short ? noise_sum<true>(pdf_s, fmid_s, w_noise_from, w_noise_to, noise_from, noise_to, delta, rcp, offset)
                  : noise_sum<false>(pdf_s, fmid_s, w_noise_from, w_noise_to, noise_from, noise_to, delta, rcp, offset);
    double cost = 3.0 * (satBottom + satTop) + quant;
    return (cost < DBL_MAX) ? cost : DBL_MAX;
}

// {min, max, delta, offset} of the winning candidate, DLQ/src/TfEnhancedEncodingAnalyzer.cpp:383-396
// (bestDelta = bestOffset = -1 when no candidate had a finite cost).
__device__ __forceinline__ void encoding_of(const SearchArgs& a, float bestDelta, int bestOffset, double enc[4])
{
    const float bMin = std_max(bestDelta * (float) bestOffset, -FLT_MAX);
    const float bMax = std_min(bestDelta * ((float) bestOffset + a.num_steps_cand), FLT_MAX);
    enc[0]           = bMin;
    enc[1]           = bMax;
    enc[2]           = bestDelta;
    enc[3]           = bestOffset;
}

// Only zeros were seen, DLQ/src/TfEnhancedEncodingAnalyzer.cpp:85-100.
__device__ __forceinline__ void encoding_of_zeros(const SearchArgs& a, double enc[4])
{
    const float ns = a.step_size_cost;
    double mn = -1, mx = 1;
    const double d = (mx - mn) / (int) ns;
    const double o = floor(mn / d);
    mn             = o * d;
    mx             = mn + (int) ns * d;
    enc[0] = mn, enc[1] = mx, enc[2] = d, enc[3] = o;
}
}   // namespace tfe
}   // namespace miq
#endif
