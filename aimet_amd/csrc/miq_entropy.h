// Entropy (KL divergence) encoding analyzer: the object behind miq_analyzer for MIQ_QUANTIZATION_ENTROPY.
// Internal to the library (miq_calib.hip dispatches to it); the C ABI is the miq_analyzer_* family.
#ifndef MIQ_ENTROPY_H
#define MIQ_ENTROPY_H

#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/miq.h"

namespace miq
{
struct EntropyAnalyzer;
int entropy_create(EntropyAnalyzer** out);
void entropy_destroy(EntropyAnalyzer* a);
int entropy_reset(EntropyAnalyzer* a, hipStream_t s);
int entropy_update(EntropyAnalyzer* a, const float* data, int64_t n, hipStream_t s);
// Reads the histogram back (synchronises `s`) and searches it on the host.
int entropy_compute(EntropyAnalyzer* a, int bw, int sym, int strict, int uns, miq_encoding* out, hipStream_t s);
// The histogram as it stands: 512 counts, its range, the number of batches counted (synchronises `s`).
int entropy_histogram(EntropyAnalyzer* a, double* counts, double* range_min_max, int* initialized, int* iterations,
                      hipStream_t s);
}   // namespace miq

#endif
