// Sequential MSE's loss for gfx950: per output channel, the error between two layer outputs summed over rows
// (SequentialMse.compute_recon_loss, TrainingExtensions/torch/src/python/aimet_torch/v1/seq_mse.py:557-581, and
// neg_sqnr :602-615; per block of input channels in TrainingExtensions/torch/src/python/aimet_torch/v2/seq_mse.py
// :325-357).  Both outputs are read once; written as tensor operations the same loss is a subtraction, a square and a
// sum: six passes over tensors of [blocks, rows, channels].
#include "miq_common.h"

#include <algorithm>

namespace miq
{
namespace
{
constexpr int kColBlock = 256;

// kind 0: sum (a - b)^2      kind 1: sum |a - b|      kind 2: plane 0 = sum (b - a)^2, plane 1 = sum b^2
template <int KIND>
__global__ __launch_bounds__(kColBlock) void column_error_kernel(const float* __restrict__ a,
                                                                 const float* __restrict__ b, int64_t rows,
                                                                 int64_t cols, int64_t rows_per_split,
                                                                 float* __restrict__ partial)
{
    const int64_t col = (int64_t) blockIdx.x * kColBlock + threadIdx.x;
    if (col >= cols)
        return;
    const int64_t block = blockIdx.y, blocks = gridDim.y, split = blockIdx.z;
    const int64_t first = split * rows_per_split;
    const int64_t last  = first + rows_per_split < rows ? first + rows_per_split : rows;
    const float* pa     = a + (block * rows + first) * cols + col;
    const float* pb     = b + (block * rows + first) * cols + col;
    float sum = 0.f, sum_b = 0.f;
    int64_t r = first;
    constexpr int kInFlight = 4;   // rows requested before the first is used
    for (; r + kInFlight <= last; r += kInFlight)
    {
        float va[kInFlight], vb[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
        {
            va[u] = __builtin_nontemporal_load(pa + u * cols);
            vb[u] = __builtin_nontemporal_load(pb + u * cols);
        }
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
        {
            const float d = va[u] - vb[u];
            sum += (KIND == 1) ? fabsf(d) : d * d;
            if (KIND == 2)
                sum_b += vb[u] * vb[u];
        }
        pa += kInFlight * cols;
        pb += kInFlight * cols;
    }
    for (; r < last; ++r)
    {
        const float va = *pa, vb = *pb;
        const float d  = va - vb;
        sum += (KIND == 1) ? fabsf(d) : d * d;
        if (KIND == 2)
            sum_b += vb * vb;
        pa += cols;
        pb += cols;
    }
    const int64_t planes = (KIND == 2) ? 2 : 1;
    float* out           = partial + ((split * planes) * blocks + block) * cols + col;
    out[0]               = sum;
    if (KIND == 2)
        out[blocks * cols] = sum_b;
}
}   // namespace
}   // namespace miq

using namespace miq;

extern "C"
{
int64_t miq_column_error_splits(int64_t blocks, int64_t rows, int64_t cols)
{
    if (blocks <= 0 || rows <= 0 || cols <= 0)
        return 1;
    // enough workgroups to fill the device (1024), at least 32 rows each
    const int64_t groups = blocks * ((cols + kColBlock - 1) / kColBlock);
    const int64_t wanted = (1024 + groups - 1) / groups;
    return std::max<int64_t>(1, std::min<int64_t>(wanted, rows / 32));
}

int miq_column_error_f32(const float* a, const float* b, int64_t blocks, int64_t rows, int64_t cols, int kind,
                         int64_t splits, float* partial, void* stream)
{
    MIQ_CHECK_ARG(a && b && partial, "null pointer");
    MIQ_CHECK_ARG(blocks > 0 && rows > 0 && cols > 0, "blocks, rows and cols must be positive");
    MIQ_CHECK_ARG(kind >= 0 && kind <= 2, "kind must be 0 (squared), 1 (absolute) or 2 (squared error and signal)");
    MIQ_CHECK_ARG(splits >= 1 && splits <= rows && splits <= 65535 && blocks <= 65535,
                  "splits must be in [1, rows] and, like blocks, at most 65535");
    const int64_t rows_per_split = (rows + splits - 1) / splits;
    const dim3 grid((unsigned) ((cols + kColBlock - 1) / kColBlock), (unsigned) blocks, (unsigned) splits);
    hipStream_t s = (hipStream_t) stream;
    if (kind == 0)
        hipLaunchKernelGGL(column_error_kernel<0>, grid, dim3(kColBlock), 0, s, a, b, rows, cols, rows_per_split, partial);
    else if (kind == 1)
        hipLaunchKernelGGL(column_error_kernel<1>, grid, dim3(kColBlock), 0, s, a, b, rows, cols, rows_per_split, partial);
    else
        hipLaunchKernelGGL(column_error_kernel<2>, grid, dim3(kColBlock), 0, s, a, b, rows, cols, rows_per_split, partial);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}
}   // extern "C"
