// TEST INFRASTRUCTURE ONLY -- never linked into, imported by or shipped with the product library.
//
// extern "C" shim over the reference's own DlQuantization CPU classes, so that the C restatement in
// oracle/miq_oracle.c can be checked bit-for-bit against the code it restates.  This file contains no
// reference source: it only calls the reference's classes, which are compiled from where they lie
// (see oracle/Makefile, target `ref`).  The resulting library lives in oracle/_ref/ and is git-ignored.
//
// Reference classes driven here:
//   TensorQuantizationSim<float>      ModelOptimizations/DlQuantization/src/TensorQuantizationSim.cpp:62-126, 300-317
//   TfEncodingAnalyzer<float>         ModelOptimizations/DlQuantization/src/TfEncodingAnalyzer.cpp:59-101
//   TfEnhancedEncodingAnalyzer<float> ModelOptimizations/DlQuantization/src/TfEnhancedEncodingAnalyzer.cpp:68-397
//   PercentileEncodingAnalyzer<float> ModelOptimizations/DlQuantization/src/PercentileEncodingAnalyzer.cpp:54-215
//   MseEncodingAnalyzer<float>        ModelOptimizations/DlQuantization/src/MseEncodingAnalyzer.cpp:54-262
//   EntropyEncodingAnalyzer<float>    ModelOptimizations/DlQuantization/src/EntropyEncodingAnalyzer.cpp:54-436
//   getComputedEncodings              ModelOptimizations/DlQuantization/src/quantization_utils.cpp:58-143
//   quantizeDequantizeBroadcastCpu    ModelOptimizations/DlQuantization/src/trim_functions.cpp:634-660

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

// The analyzer keeps its PDF and its candidate/cost helpers private; the checks need to see them.
#define private public
#include "TfEnhancedEncodingAnalyzer.h"
#include "MseEncodingAnalyzer.h"
#include "EntropyEncodingAnalyzer.h"
#undef private
#include "TensorQuantizationSim.h"
#include "PercentileEncodingAnalyzer.h"
#include "TfEncodingAnalyzer.h"
#include "quantization_utils.hpp"
#include "trim_functions.hpp"

using namespace DlQuantization;

namespace
{
void putEncoding(const TfEncoding& e, double* out5)
{
    out5[0] = e.min;
    out5[1] = e.max;
    out5[2] = e.delta;
    out5[3] = e.offset;
    out5[4] = (double) e.bw;
}
}   // namespace

extern "C"
{
// ---- TensorQuantizationSim<float> ---------------------------------------------------------------
void ref_fill_encoding_info(int bw, double encMin, double encMax, double* out5)
{
    TensorQuantizationSim<float> sim;
    TfEncoding e;
    sim.fillEncodingInfo(e, (uint8_t) bw, encMin, encMax);
    putEncoding(e, out5);
}

void ref_qdq_per_tensor(const float* in, int64_t n, float* out, double encMin, double encMax, int bw)
{
    TensorQuantizationSim<float> sim;
    sim.quantizeDequantizeTensor(in, (size_t) n, out, encMin, encMax, (uint8_t) bw, ROUND_NEAREST, false);
}

// ROUND_STOCHASTIC on the CPU path draws from libc rand() (trim_functions.cpp:56-59); srand(seed) first, and
// ref_libc_uniforms replays the same sequence: rand() / (RAND_MAX + 1.0).
void ref_qdq_per_tensor_stochastic(const float* in, int64_t n, float* out, double encMin, double encMax, int bw,
                                   unsigned int seed)
{
    TensorQuantizationSim<float> sim;
    srand(seed);
    sim.quantizeDequantizeTensor(in, (size_t) n, out, encMin, encMax, (uint8_t) bw, ROUND_STOCHASTIC, false);
}

void ref_quantize_per_tensor_stochastic(const float* in, int64_t n, float* out, double encMin, double encMax, int bw,
                                        int shiftToSigned, unsigned int seed)
{
    TensorQuantizationSim<float> sim;
    srand(seed);
    sim.quantizeTensor(in, (size_t) n, out, encMin, encMax, (uint8_t) bw, ROUND_STOCHASTIC, false,
                       shiftToSigned != 0);
}

void ref_qdq_per_channel_stochastic(const float* in, int64_t numChannel, int64_t numElement,
                                    int64_t numElementPerChannel, float* out, float* encMin, float* encMax,
                                    float* encDelta, float* encOffset, unsigned int seed)
{
    TensorQuantizationSim<float> sim;
    srand(seed);
    sim.quantizeDequantizeTensorPerChannel(in, (size_t) numChannel, (size_t) numElement,
                                           (size_t) numElementPerChannel, out, encMin, encMax, encDelta, encOffset,
                                           ROUND_STOCHASTIC, false);
}

void ref_libc_uniforms(unsigned int seed, int64_t n, double* u)
{
    srand(seed);
    for (int64_t i = 0; i < n; ++i)
        u[i] = rand() / (RAND_MAX + 1.0);
}

void ref_quantize_per_tensor(const float* in, int64_t n, float* out, double encMin, double encMax, int bw,
                             int shiftToSigned)
{
    TensorQuantizationSim<float> sim;
    sim.quantizeTensor(in, (size_t) n, out, encMin, encMax, (uint8_t) bw, ROUND_NEAREST, false,
                       shiftToSigned != 0);
}

void ref_qdq_per_channel(const float* in, int64_t numChannel, int64_t numElement, int64_t numElementPerChannel,
                         float* out, float* encMin, float* encMax, float* encDelta, float* encOffset)
{
    TensorQuantizationSim<float> sim;
    sim.quantizeDequantizeTensorPerChannel(in, (size_t) numChannel, (size_t) numElement,
                                           (size_t) numElementPerChannel, out, encMin, encMax, encDelta, encOffset,
                                           ROUND_NEAREST, false);
}

void ref_qdq_broadcast(const float* in, float* out, int64_t numElement, int64_t numDims, const int64_t* inputStrides,
                       const int64_t* encodingStrides, const float* encMin, const float* encMax,
                       const float* encDelta, const float* encOffset)
{
    quantizeDequantizeBroadcastCpu<float>(in, out, numElement, numDims, inputStrides, encodingStrides, encMin,
                                          encMax, encDelta, encOffset);
}

// ---- free function: min/max -> TF encoding ---------------------------------------------------------
void ref_get_computed_encodings(int bw, double mn, double mx, int sym, int strict, int unsignedSym, double* out5)
{
    TfEncoding e = getComputedEncodings((uint8_t) bw, mn, mx, sym != 0, strict != 0, unsignedSym != 0);
    putEncoding(e, out5);
}

// ---- TfEncodingAnalyzer<float> -------------------------------------------------------------------
void* ref_tf_create()
{
    return new TfEncodingAnalyzer<float>();
}
void ref_tf_destroy(void* h)
{
    delete static_cast<TfEncodingAnalyzer<float>*>(h);
}
void ref_tf_update(void* h, const float* data, int64_t n)
{
    static_cast<TfEncodingAnalyzer<float>*>(h)->updateStats(data, (size_t) n, COMP_MODE_CPU);
}
void ref_tf_compute(void* h, int bw, int sym, int strict, int unsignedSym, double* out5)
{
    TfEncoding e = static_cast<TfEncodingAnalyzer<float>*>(h)->computeEncoding((uint8_t) bw, sym != 0, strict != 0,
                                                                               unsignedSym != 0);
    putEncoding(e, out5);
}

// ---- TfEnhancedEncodingAnalyzer<float> -----------------------------------------------------------
void* ref_tfe_create()
{
    return new TfEnhancedEncodingAnalyzer<float>();
}
void ref_tfe_destroy(void* h)
{
    delete static_cast<TfEnhancedEncodingAnalyzer<float>*>(h);
}
void ref_tfe_update(void* h, const float* data, int64_t n)
{
    static_cast<TfEnhancedEncodingAnalyzer<float>*>(h)->updateStats(data, (size_t) n, COMP_MODE_CPU);
}
void ref_tfe_compute(void* h, int bw, int sym, int strict, int unsignedSym, double* out5)
{
    TfEncoding e = static_cast<TfEnhancedEncodingAnalyzer<float>*>(h)->computeEncoding(
        (uint8_t) bw, sym != 0, strict != 0, unsignedSym != 0);
    putEncoding(e, out5);
}
// Returns the number of buckets written (0 when the PDF has not been initialised yet).
int ref_tfe_get_pdf(void* h, double* xLeft, double* pdf, int* iterations)
{
    auto* a = static_cast<TfEnhancedEncodingAnalyzer<float>*>(h);
    int n   = (int) a->_stats.xLeft.size();
    for (int i = 0; i < n; ++i)
    {
        xLeft[i] = a->_stats.xLeft[i];
        pdf[i]   = a->_stats.pdf[i];
    }
    *iterations = a->_stats.iterations;
    return n;
}
// Candidate list in the reference's own order, with the cost of each; returns the candidate count.
int ref_tfe_candidates(void* h, int bw, int sym, int strict, int unsignedSym, int maxOut, float* deltas, int* offsets,
                       double* costs)
{
    auto* a = static_cast<TfEnhancedEncodingAnalyzer<float>*>(h);
    float minVal, maxVal;
    std::tie(minVal, maxVal) = a->_findRangeOfAggregateStats();
    float numSteps           = pow(2, bw) - 1;
    std::vector<std::tuple<float, int>> cands;
    if (sym)
    {
        if (strict)
            numSteps -= 1;
        a->_pickTestCandidatesSymmetric(minVal, maxVal, numSteps, cands, unsignedSym != 0);
    }
    else
    {
        a->_pickTestCandidatesAsymmetric(minVal, maxVal, numSteps, cands);
    }
    int n = (int) cands.size();
    for (int i = 0; i < n && i < maxOut; ++i)
    {
        deltas[i]  = std::get<0>(cands[i]);
        offsets[i] = std::get<1>(cands[i]);
        costs[i]   = a->_quantAndSatCost(a->_stats, bw, deltas[i], offsets[i]);
    }
    return n;
}
void ref_tfe_range(void* h, float* minVal, float* maxVal)
{
    auto* a                    = static_cast<TfEnhancedEncodingAnalyzer<float>*>(h);
    std::tie(*minVal, *maxVal) = a->_findRangeOfAggregateStats();
}
// ---- PercentileEncodingAnalyzer<float> -----------------------------------------------------------
void* ref_pct_create(float percentile)
{
    auto* a = new PercentileEncodingAnalyzer<float>();
    a->setPercentileValue(percentile);
    return a;
}
void ref_pct_destroy(void* h)
{
    delete static_cast<PercentileEncodingAnalyzer<float>*>(h);
}
void ref_pct_update(void* h, const float* data, int64_t n)
{
    static_cast<PercentileEncodingAnalyzer<float>*>(h)->updateStats(data, (size_t) n, COMP_MODE_CPU);
}
void ref_pct_compute(void* h, int bw, int sym, int strict, int unsignedSym, double* out5)
{
    TfEncoding e = static_cast<PercentileEncodingAnalyzer<float>*>(h)->computeEncoding((uint8_t) bw, sym != 0,
                                                                                       strict != 0, unsignedSym != 0);
    putEncoding(e, out5);
}
// ---- MseEncodingAnalyzer<float> ------------------------------------------------------------------
void* ref_mse_create()
{
    return new MseEncodingAnalyzer<float>();
}
void ref_mse_destroy(void* h)
{
    delete static_cast<MseEncodingAnalyzer<float>*>(h);
}
void ref_mse_update(void* h, const float* data, int64_t n)
{
    static_cast<MseEncodingAnalyzer<float>*>(h)->updateStats(data, (size_t) n, COMP_MODE_CPU);
}
void ref_mse_compute(void* h, int bw, int sym, int strict, int unsignedSym, double* out5)
{
    TfEncoding e = static_cast<MseEncodingAnalyzer<float>*>(h)->computeEncoding((uint8_t) bw, sym != 0, strict != 0,
                                                                                unsignedSym != 0);
    putEncoding(e, out5);
}
// the (min, max) pair the search settles on, before zero is gated in and the grid is formed
void ref_mse_minimize(void* h, int bw, int sym, int strict, int unsignedSym, float* bestMin, float* bestMax)
{
    auto* a                      = static_cast<MseEncodingAnalyzer<float>*>(h);
    std::tie(*bestMin, *bestMax) = a->_minimizeMSE((uint8_t) bw, sym != 0, strict != 0, unsignedSym != 0);
}
// the cost of one candidate on explicit bucket centres
float ref_mse_cost(void* h, int bw, const float* centers, const float* pdfAtCenter, int n, float candMin,
                   float candMax, int sym, int strict, int unsignedSym)
{
    auto* a = static_cast<MseEncodingAnalyzer<float>*>(h);
    std::vector<std::pair<float, float>> centersPdf((size_t) n);
    for (int i = 0; i < n; ++i)
        centersPdf[(size_t) i] = {centers[i], pdfAtCenter[i]};
    return a->_computeMSECost((uint8_t) bw, centersPdf, candMin, candMax, sym != 0, strict != 0, unsignedSym != 0);
}
// ---- EntropyEncodingAnalyzer<float> --------------------------------------------------------------
void* ref_entropy_create()
{
    return new EntropyEncodingAnalyzer<float>();
}
void ref_entropy_destroy(void* h)
{
    delete static_cast<EntropyEncodingAnalyzer<float>*>(h);
}
void ref_entropy_update(void* h, const float* data, int64_t n)
{
    static_cast<EntropyEncodingAnalyzer<float>*>(h)->updateStats(data, (size_t) n, COMP_MODE_CPU);
}
void ref_entropy_compute(void* h, int bw, int sym, int strict, int unsignedSym, double* out5)
{
    TfEncoding e = static_cast<EntropyEncodingAnalyzer<float>*>(h)->computeEncoding((uint8_t) bw, sym != 0,
                                                                                    strict != 0, unsignedSym != 0);
    putEncoding(e, out5);
}
// the rescaling histogram: returns the number of bins (0 before the first batch that is not all zeros)
int ref_entropy_get_histogram(void* h, double* hist512, double* minMax2, int* iterations)
{
    auto* a    = static_cast<EntropyEncodingAnalyzer<float>*>(h);
    auto& tpp  = a->_tensorProfilingParams;
    minMax2[0] = tpp.min;
    minMax2[1] = tpp.max;
    *iterations = tpp.iterations;
    for (size_t i = 0; i < tpp.histogram.size() && i < 512; ++i)
        hist512[i] = tpp.histogram[i];
    return (int) tpp.histogram.size();
}
// the range the window search settles on, before zero is gated in and the grid is formed
void ref_entropy_optimize(void* h, int bw, int sym, int strict, int unsignedSym, float* bestMin, float* bestMax)
{
    auto* a                      = static_cast<EntropyEncodingAnalyzer<float>*>(h);
    std::tie(*bestMin, *bestMax) = a->_optimizeKL((uint8_t) bw, sym != 0, strict != 0, unsignedSym != 0);
}
}   // extern "C"
