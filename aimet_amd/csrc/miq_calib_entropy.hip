// Entropy (KL divergence) calibration for gfx950: EntropyEncodingAnalyzer<float>
// (ModelOptimizations/DlQuantization/src/EntropyEncodingAnalyzer.cpp:54-436) over the rescaling 512-bin histogram of
// updateTensorHistogram_cpu (ModelOptimizations/DlQuantization/src/math_functions.cpp:468-560).
//
// The reference copies every batch to the host and bins it there.  Here a batch costs three launches and no copy:
//   ent_minmax_kernel   one streaming pass, per-workgroup (min, max)
//   ent_range_kernel    one workgroup: the batch's range; an all-zero batch is dropped; the first other batch fixes the
//                       histogram's range; a batch outside it widens the range and moves the old counts into the new
//                       bins, each old bin split over at most two new ones
//   ent_bin_kernel      second streaming pass: float bin index per sample, counts in LDS, flushed to 64-bit counters
// The histogram holds whole counts at all times (the redistribution rounds the share it moves), so sums of them are
// exact in any order and the device's atomic adds give the reference's numbers.  compute_encoding reads the 512 counts
// back and runs the window search on the host: 129 windows of at most 512 bins.
// Samples are taken to be finite.
#include "miq_common.h"
#include "miq_encoding_math.h"
#include "miq_entropy.h"

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstring>
#include <new>
#include <vector>

namespace miq
{
namespace
{
constexpr int kBins     = MIQ_PDF_SIZE;
constexpr int kEntGrid  = 1024;   // workgroups of either streaming pass, at most
constexpr int kEntBlock = 256;
constexpr int kEntReplicas = 16;
typedef float v4f __attribute__((ext_vector_type(4)));

struct EntState
{
    double min, max;   // the histogram spans [min, max]
    int initialized;   // histogram.size() != 0 in the reference
    int iterations;    // batches counted (all-zero batches are not)
    int skip;          // the batch in flight is all zeros: nothing to count
    float bin_width_f, min_f;   // what getBin takes for the batch in flight
    unsigned long long hist[kBins];
    float2 partial[kEntGrid];
    // Counts of the batch binned last, not yet added to `hist`: workgroup b of the bin pass adds to replica
    // b % kEntReplicas.  Atomic adds of many workgroups to one address queue at about 15 ns each; with one set of 512
    // counters, 1024 workgroups spent 15 us of a 19 us launch there.  Folded into `hist` by the next range kernel and
    // before the histogram is read.
    unsigned long long replica[kEntReplicas][kBins];
};
constexpr size_t kEntReadBytes = offsetof(EntState, partial);

__device__ __forceinline__ float wave_lo(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v = fminf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_hi(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// getBin (math_functions.cpp:468-474): float arithmetic, truncated, capped at the last bin.  A quotient that is not
// below the bin count (or is NaN) lands in the last bin, as the reference's conversion to size_t makes it.
__host__ __device__ __forceinline__ int get_bin(float bin_width, float min_value, float value)
{
    if (bin_width == 0)
        return 0;
    const float q = (value - min_value) / bin_width;
    if (!(q < (float) kBins) || q <= -1.0f)
        return kBins - 1;
    return (int) q;
}

__global__ __launch_bounds__(kEntBlock) void ent_minmax_kernel(const float* __restrict__ data, int64_t n, EntState* st,
                                                                int vec)
{
    float lo = INFINITY, hi = -INFINITY;
    const int64_t stride = (int64_t) gridDim.x * blockDim.x;
    const int64_t first  = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    int64_t done         = 0;
    if (vec)
    {
        const v4f* d4    = reinterpret_cast<const v4f*>(data);
        const int64_t n4 = n / 4;
        for (int64_t k = first; k < n4; k += stride)
        {
            const v4f v = __builtin_nontemporal_load(d4 + k);   // read once: not kept in the caches
            lo             = fminf(fminf(lo, v.x), fminf(v.y, fminf(v.z, v.w)));
            hi             = fmaxf(fmaxf(hi, v.x), fmaxf(v.y, fmaxf(v.z, v.w)));
        }
        done = n4 * 4;
    }
    for (int64_t k = done + first; k < n; k += stride)
    {
        lo = fminf(lo, data[k]);
        hi = fmaxf(hi, data[k]);
    }
    __shared__ float s_lo[kEntBlock / 64], s_hi[kEntBlock / 64];
    lo = wave_lo(lo);
    hi = wave_hi(hi);
    if ((threadIdx.x & 63) == 0)
        s_lo[threadIdx.x >> 6] = lo, s_hi[threadIdx.x >> 6] = hi;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int w = 1; w < kEntBlock / 64; ++w)
            lo = fminf(lo, s_lo[w]), hi = fmaxf(hi, s_hi[w]);
        st->partial[blockIdx.x] = make_float2(lo, hi);
    }
}

enum
{
    kBatchZeros = 0,   // dropped
    kBatchInside,      // within the histogram's range
    kBatchFirst,       // fixes the range
    kBatchWidens       // widens it: the counts move
};

// hist[t] += the replicas' counts of bin t, which are cleared (thread t of a 512-thread workgroup)
__device__ __forceinline__ void fold_replicas(EntState* st, int t)
{
    // every load requested before the first is used: a dependent round trip to memory takes 1-2 us
    unsigned long long part[kEntReplicas];
#pragma unroll
    for (int r = 0; r < kEntReplicas; ++r)
        part[r] = st->replica[r][t];
    unsigned long long sum = st->hist[t];
#pragma unroll
    for (int r = 0; r < kEntReplicas; ++r)
    {
        sum += part[r];
        st->replica[r][t] = 0;
    }
    st->hist[t] = sum;
}

__global__ __launch_bounds__(kBins) void ent_fold_kernel(EntState* st)
{
    fold_replicas(st, threadIdx.x);
}

__global__ __launch_bounds__(kBins) void ent_range_kernel(EntState* st, int groups)
{
    __shared__ float s_lo[kBins / 64], s_hi[kBins / 64];
    __shared__ unsigned long long s_moved[kBins];
    __shared__ int s_kind;
    __shared__ double s_range[4];   // old min, old max, new min, new max
    const int t = threadIdx.x;
    fold_replicas(st, t);   // the batch before this one; thread t alone touches hist[t] until the barriers below
    float lo = INFINITY, hi = -INFINITY;
    for (int k = t; k < groups; k += kBins)
    {
        const float2 p = st->partial[k];
        lo             = fminf(lo, p.x);
        hi             = fmaxf(hi, p.y);
    }
    lo = wave_lo(lo);
    hi = wave_hi(hi);
    if ((t & 63) == 0)
        s_lo[t >> 6] = lo, s_hi[t >> 6] = hi;
    s_moved[t] = 0;
    __syncthreads();
    if (t == 0)
    {
        for (int w = 1; w < kBins / 64; ++w)
            lo = fminf(lo, s_lo[w]), hi = fmaxf(hi, s_hi[w]);
        double min_input = lo, max_input = hi;
        if (min_input == 0 && max_input == 0)
            s_kind = kBatchZeros;
        else
        {
            if (min_input == max_input)
                max_input = enc_max2(max_input, min_input + (float) 0.01);   // a range that is not empty
            if (!st->initialized)
            {
                s_kind     = kBatchFirst;
                s_range[2] = min_input, s_range[3] = max_input;
            }
            else if (min_input < st->min || max_input > st->max)
            {
                s_kind     = kBatchWidens;
                s_range[0] = st->min, s_range[1] = st->max;
                s_range[2] = enc_min2(min_input, st->min), s_range[3] = enc_max2(max_input, st->max);
            }
            else
            {
                s_kind     = kBatchInside;
                s_range[2] = st->min, s_range[3] = st->max;
            }
        }
    }
    __syncthreads();
    const int kind = s_kind;
    if (kind == kBatchZeros)
    {
        if (t == 0)
            st->skip = 1;
        return;
    }
    if (kind == kBatchFirst)
        st->hist[t] = 0;
    if (kind == kBatchWidens)
    {
        // math_functions.cpp:505-547: old bin t goes to the new bin its left edge falls into, and what does not fit
        // there (by the rounded share of its width) to the bin one new width further
        const double new_min = s_range[2], new_max = s_range[3];
        const double dest_width        = (new_max - new_min) / kBins;
        const double src_width         = (s_range[1] - s_range[0]) / kBins;
        const unsigned long long count = st->hist[t];
        if (count != 0)
        {
            const double held      = (double) count;
            const double src_begin = s_range[0] + src_width * t;
            const size_t dest_bin  = (size_t) ((src_begin - new_min) / dest_width);
            const double dest_end  = new_min + dest_width * (dest_bin + 1);
            const double share     = round((dest_end - src_begin) / src_width * held);
            const double stays     = enc_min2(share, held);
            atomicAdd(&s_moved[get_bin((float) dest_width, (float) new_min, (float) src_begin)],
                      (unsigned long long) (stays > 0 ? stays : 0.0));
            if (stays < held)
                atomicAdd(&s_moved[get_bin((float) dest_width, (float) new_min, (float) (src_begin + dest_width))],
                          (unsigned long long) (held - stays));
        }
        __syncthreads();
        st->hist[t] = s_moved[t];
    }
    if (t == 0)
    {
        st->min         = s_range[2];
        st->max         = s_range[3];
        st->initialized = 1;
        st->skip        = 0;
        st->iterations += 1;
        st->bin_width_f = (float) ((s_range[3] - s_range[2]) / kBins);
        st->min_f       = (float) s_range[2];
    }
}

// Activations pile up in a few bins (after a ReLU, half of them in one): eight copies of the counters in LDS, picked by
// lane, keep lanes of one wavefront from queueing on one address.
constexpr int kEntCopies = 8;
__global__ __launch_bounds__(kEntBlock) void ent_bin_kernel(const float* __restrict__ data, int64_t n, EntState* st,
                                                             int vec)
{
    if (st->skip)
        return;
    // the copies of one bin sit side by side, in different LDS banks: laid out copy after copy, all copies of a bin
    // share a bank and lanes on different copies still queue
    __shared__ unsigned int s_hist[kBins * kEntCopies];
    for (int k = threadIdx.x; k < kEntCopies * kBins; k += kEntBlock)
        s_hist[k] = 0;
    __syncthreads();
    unsigned int* mine = s_hist + (threadIdx.x & (kEntCopies - 1));
    const float width = st->bin_width_f, low = st->min_f;
    const int64_t stride = (int64_t) gridDim.x * blockDim.x;
    const int64_t first  = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    int64_t done         = 0;
    if (vec)
    {
        const v4f* d4    = reinterpret_cast<const v4f*>(data);
        const int64_t n4 = n / 4;
        // four loads per lane in flight before the first of them is counted: one load at a time leaves the launch
        // waiting on memory latency (12.8 us for 25.7 MB)
        constexpr int kInFlight = 4;
        for (int64_t k = first; k < n4; k += stride * kInFlight)
        {
            v4f v[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u)
                if (k + u * stride < n4)
                    v[u] = __builtin_nontemporal_load(d4 + k + u * stride);
#pragma unroll
            for (int u = 0; u < kInFlight; ++u)
                if (k + u * stride < n4)
                {
                    atomicAdd(&mine[get_bin(width, low, v[u].x) * kEntCopies], 1u);
                    atomicAdd(&mine[get_bin(width, low, v[u].y) * kEntCopies], 1u);
                    atomicAdd(&mine[get_bin(width, low, v[u].z) * kEntCopies], 1u);
                    atomicAdd(&mine[get_bin(width, low, v[u].w) * kEntCopies], 1u);
                }
        }
        done = n4 * 4;
    }
    for (int64_t k = done + first; k < n; k += stride)
        atomicAdd(&mine[get_bin(width, low, data[k]) * kEntCopies], 1u);
    __syncthreads();
    for (int k = threadIdx.x; k < kBins; k += kEntBlock)
    {
        unsigned int sum = 0;
#pragma unroll
        for (int c = 0; c < kEntCopies; ++c)
            sum += s_hist[k * kEntCopies + c];
        if (sum)
            atomicAdd(&st->replica[blockIdx.x % kEntReplicas][k], (unsigned long long) sum);
    }
}

__global__ void ent_reset_kernel(EntState* st)
{
    const int t = threadIdx.x;   // launched with kBins threads
    st->hist[t] = 0;
    for (int r = 0; r < kEntReplicas; ++r)
        st->replica[r][t] = 0;
    if (t == 0)
    {
        st->min = st->max = 0;
        st->initialized = st->iterations = st->skip = 0;
        st->bin_width_f = st->min_f = 0.f;
    }
}

// ---------------------------------------------------------------------------------------------- host: the search
// std::accumulate(first, last, 0.f) of the reference: the running sum has the type of its initial value, float.
double sum_in_float(const std::vector<double>& v)
{
    float running = 0.f;
    for (double x : v)
        running = (float) (running + x);
    return running;
}

// rescaleHistogram (math_functions.cpp:562-643): the counts laid over another range of as many bins, each source bin
// spread over the destination bins it overlaps in whole counts, never more than it holds.
std::vector<double> spread_over(const std::vector<double>& src, double src_min, double src_max, double dst_min,
                                double dst_max)
{
    if (src_min == dst_min && src_max == dst_max)
        return src;
    const size_t bins      = src.size();
    const double src_width = (src_max - src_min) / bins;
    const double dst_width = (dst_max - dst_min) / bins;
    std::vector<double> dst(bins, 0.0);
    for (size_t i = 0; i < bins; ++i)
    {
        const double held = src[i];
        if (held == 0)
            continue;
        const double begin = src_min + i * src_width;
        const double end   = src_min + (i + 1) * src_width;
        size_t from        = (size_t) enc_max2(std::floor((begin - dst_min) / dst_width), 0.0);
        size_t to          = (size_t) enc_max2(std::ceil((end - dst_min) / dst_width), 0.0);
        from               = std::min(from, bins - 1);
        to                 = std::min(to, bins - 1);
        double left        = held;
        for (size_t j = from; j <= to; ++j)
        {
            const double d_begin = dst_min + j * dst_width;
            const double d_end   = dst_min + (j + 1) * dst_width;
            double ratio         = (enc_min2(end, d_end) - enc_max2(begin, d_begin)) / src_width;
            ratio                = ratio >= 0.0f ? ratio : 0.0f;
            ratio                = ratio <= 1.0f ? ratio : 1.0f;
            double moved         = std::round(ratio * held);
            moved                = moved <= left ? moved : left;
            dst[j] += moved;
            left -= moved;
        }
    }
    return dst;
}

// _conditionHistogram (EntropyEncodingAnalyzer.cpp:153-200): 1e-4 into every empty bin, taken evenly from the others.
void smooth(std::vector<double>& h)
{
    const double eps_empty = 0.0001;
    size_t empty           = 0;
    for (double x : h)
        empty += (x == 0.f);
    if (h.empty() || empty == h.size())
        return;
    const double eps_other = eps_empty * (double) empty / (double) (h.size() - empty);
    if (eps_other >= 1.0)
        return;
    for (double& x : h)
    {
        const int is_empty = (x == 0.f);
        x += eps_empty * is_empty;
        x -= eps_other * (1 - is_empty);
    }
}

// _computeKL (:202-228)
double kl_divergence(std::vector<double>& p, std::vector<double>& q)
{
    const double sum_p = sum_in_float(p), sum_q = sum_in_float(q);
    double divergence = 0;
    for (size_t i = 0; i < p.size(); ++i)
    {
        p[i] /= sum_p;
        q[i] /= sum_q;
        if (p[i] > 0 && q[i] > 0)
            divergence += p[i] * std::log(p[i] / q[i]);
    }
    return divergence;
}

// _optimizeKL (:230-431): for 8 bits, the window [first, last] of the histogram whose 255-level quantization diverges
// least from the histogram saturated into it; windows shrink by two bins at a time.  Other bitwidths keep the range.
void narrowed_range(const double* counts, double hist_min, double hist_max, int bw, bool sym, bool strict, bool uns,
                    float* out_min, float* out_max)
{
    std::vector<double> hist(counts, counts + kBins);
    if (sym && (hist_min < 0.0 || !uns))
    {
        const float abs_max = (float) enc_max2(std::fabs(hist_max), std::fabs(hist_min));
        const float abs_min = -abs_max;
        hist                = spread_over(hist, hist_min, hist_max, abs_min, abs_max);
        hist_min            = abs_min;
        hist_max            = abs_max;
    }
    *out_min = (float) hist_min;
    *out_max = (float) hist_max;
    constexpr size_t kLevels = 255;
    if (bw != 8)
        return;
    const double width = (hist_max - hist_min) / (double) kBins;
    double least       = INFINITY;
    double best_min = hist_min, best_max = hist_max;
    size_t first = 0, last = kBins - 1;
    while (last - first + 1 >= kLevels)
    {
        const size_t span = last - first + 1;
        const double* win = hist.data() + first;
        // P: the histogram with everything outside the window piled onto the window's end bins
        std::vector<double> p(span, 0.0);
        double pile = 0;
        for (size_t i = 0; i <= first; ++i)
            pile += hist[i];
        p.front() += pile;
        for (size_t i = first + 1; i < last; ++i)
            p[i - first] = hist[i];
        pile = 0;
        for (size_t i = last; i < (size_t) kBins; ++i)
            pile += hist[i];
        p.back() += pile;
        // Q: 255 levels, each the mean of its non-empty bins, laid back over those bins
        const double per_level = (double) span / (double) kLevels;
        std::vector<double> q(span, 0.0);
        for (size_t level = 0; level < kLevels; ++level)
        {
            const size_t from = (size_t) std::ceil(level * per_level);
            const size_t to   = (level < kLevels - 1) ? (size_t) std::ceil((level + 1) * per_level) : span;
            double sum = 0, filled = 0;
            for (size_t i = from; i < to; ++i)
            {
                sum += win[i];
                filled += (win[i] != 0);
            }
            if (filled != 0)
                for (size_t i = from; i < to; ++i)
                    if (win[i])
                        q[i] = sum / filled;
        }
        if (sum_in_float(p) == 0 || sum_in_float(q) == 0)
            break;   // a one-sided distribution shrunk to nothing
        smooth(p);
        smooth(q);
        const double divergence = kl_divergence(p, q);
        if (divergence < least)
        {
            least    = divergence;
            best_min = hist_min + first * width;
            best_max = hist_min + (last + 1) * width;
        }
        if (sym || strict)
        {
            ++first;
            --last;
            continue;
        }
        // asymmetric: drop the two bins that lose least -- one at each end, two on the left or two on the right --
        // without letting the window leave zero behind
        const double loss[3] = {hist[first] + hist[last], hist[first] + hist[first + 1], hist[last] + hist[last - 1]};
        int pick             = (int) (std::min_element(loss, loss + 3) - loss);
        if ((pick == 0 && hist_min + (first + 1) * width > 0) || (pick == 1 && hist_min + (first + 2) * width > 0))
            pick = 2;
        else if ((pick == 0 && hist_min + last * width < 0) || (pick == 2 && hist_min + (last - 1) * width < 0))
            pick = 1;
        if (pick == 0)
            ++first, --last;
        else if (pick == 1)
            first += 2;
        else
            last -= 2;
    }
    *out_min = (float) best_min;
    *out_max = (float) best_max;
}
}   // namespace

struct EntropyAnalyzer
{
    EntState* st;
    void* pinned;
    bool needs_reset;
};

int entropy_create(EntropyAnalyzer** out)
{
    EntropyAnalyzer* a = new (std::nothrow) EntropyAnalyzer();
    MIQ_CHECK_ARG(a != nullptr, "out of host memory");
    a->st = nullptr, a->pinned = nullptr, a->needs_reset = true;
    hipError_t e = hipMalloc((void**) &a->st, sizeof(EntState));
    if (e == hipSuccess)
        e = hipHostMalloc(&a->pinned, kEntReadBytes, hipHostMallocDefault);
    if (e != hipSuccess)
    {
        set_error("entropy analyzer allocation failed: %s", hipGetErrorString(e));
        entropy_destroy(a);
        return MIQ_ERR_HIP;
    }
    *out = a;
    return MIQ_OK;
}

void entropy_destroy(EntropyAnalyzer* a)
{
    if (!a)
        return;
    if (a->st)
        (void) hipFree(a->st);
    if (a->pinned)
        (void) hipHostFree(a->pinned);
    delete a;
}

int entropy_reset(EntropyAnalyzer* a, hipStream_t s)
{
    hipLaunchKernelGGL(ent_reset_kernel, dim3(1), dim3(kBins), 0, s, a->st);
    MIQ_CHECK_LAUNCH();
    a->needs_reset = false;
    return MIQ_OK;
}

int entropy_update(EntropyAnalyzer* a, const float* data, int64_t n, hipStream_t s)
{
    if (a->needs_reset)
        if (int rc = entropy_reset(a, s))
            return rc;
    const int vec      = (reinterpret_cast<uintptr_t>(data) & 15u) == 0;
    const int64_t want = (n / 4 + kEntBlock * 4 - 1) / (kEntBlock * 4);   // four vectors per lane
    const int groups   = (int) std::max<int64_t>(1, std::min<int64_t>(kEntGrid, want));
    hipLaunchKernelGGL(ent_minmax_kernel, dim3(groups), dim3(kEntBlock), 0, s, data, n, a->st, vec);
    hipLaunchKernelGGL(ent_range_kernel, dim3(1), dim3(kBins), 0, s, a->st, groups);
    hipLaunchKernelGGL(ent_bin_kernel, dim3(groups), dim3(kEntBlock), 0, s, data, n, a->st, vec);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

static int read_back(EntropyAnalyzer* a, hipStream_t s)
{
    if (a->needs_reset)
        if (int rc = entropy_reset(a, s))
            return rc;
    hipLaunchKernelGGL(ent_fold_kernel, dim3(1), dim3(kBins), 0, s, a->st);
    MIQ_CHECK_LAUNCH();
    MIQ_CHECK_HIP(hipMemcpyAsync(a->pinned, a->st, kEntReadBytes, hipMemcpyDeviceToHost, s));
    MIQ_CHECK_HIP(hipStreamSynchronize(s));
    return MIQ_OK;
}

int entropy_histogram(EntropyAnalyzer* a, double* counts, double* range_min_max, int* initialized, int* iterations,
                      hipStream_t s)
{
    if (int rc = read_back(a, s))
        return rc;
    const EntState* h = static_cast<const EntState*>(a->pinned);
    for (int i = 0; i < kBins; ++i)
        counts[i] = (double) h->hist[i];
    range_min_max[0] = h->min, range_min_max[1] = h->max;
    *initialized = h->initialized, *iterations = h->iterations;
    return MIQ_OK;
}

// computeEncoding (:97-146); the caller has established that statistics were updated
int entropy_compute(EntropyAnalyzer* a, int bw, int sym, int strict, int uns, miq_encoding* out, hipStream_t s)
{
    if (int rc = read_back(a, s))
        return rc;
    const EntState* h = static_cast<const EntState*>(a->pinned);
    if (!h->initialized)
    {
        // only zeros were seen: an encoding that covers float 0
        float num_steps = (float) (std::pow(2, bw) - 1);
        if (sym && strict)
            num_steps -= 1;
        out->min    = -1;
        out->max    = 1;
        out->delta  = (out->max - out->min) / (int) num_steps;
        out->offset = std::floor(out->min / out->delta);
        out->min    = out->offset * out->delta;
        out->max    = out->min + (int) num_steps * out->delta;
        out->bw     = bw;
        return MIQ_OK;
    }
    double counts[kBins];
    for (int i = 0; i < kBins; ++i)
        counts[i] = (double) h->hist[i];
    float a_min, a_max;
    narrowed_range(counts, h->min, h->max, bw, sym != 0, strict != 0, uns != 0, &a_min, &a_max);
    a_min = std::min(a_min, 0.0f);
    a_max = std::max(a_max, 0.0f);
    return miq_get_computed_encodings(bw, a_min, a_max, sym, strict, uns, out);
}
}   // namespace miq
