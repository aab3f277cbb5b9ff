// Launchers of the stochastic-rounding variants of the v1 kernels (miq_stochastic.hip).
#ifndef MIQ_STOCHASTIC_H
#define MIQ_STOCHASTIC_H

#include "miq_common.h"

namespace miq
{
template <typename IO>
int stochastic_qdq_per_tensor(const IO* in, IO* out, int64_t n, const miq_encoding& e, hipStream_t stream);

int stochastic_quantize_per_tensor(const float* in, float* out, int64_t n, const miq_encoding& e, float shift,
                                   hipStream_t stream);

template <typename IO>
int stochastic_qdq_per_channel(const IO* in, IO* out, int64_t num_channel, int64_t n, int64_t n_per_channel,
                               const float* mn, const float* mx, const float* delta, const float* offset,
                               hipStream_t stream);
}   // namespace miq

#endif
