// Per-channel TF-Enhanced / percentile calibration in one object: C independent 512-bucket PDFs over the channels of
// one tensor, fed by one launch sequence per update and searched by one launch, instead of C analyzer objects fed
// slice by slice.
//
// What it replaces in the reference: StaticGridPerChannelQuantizer.update_encoding_stats / compute_encoding
// (TrainingExtensions/torch/src/python/aimet_torch/v1/tensor_quantizer.py:535-570, 280-321), which keeps one
// AimetTensorQuantizer per channel and calls updateStats on `tensor.select(axis, c).contiguous()` and getEncoding
// once per channel (TrainingExtensions/torch/src/AimetTensorQuantizer.cpp:85-126, 180-192).  Channel c here sees
// exactly the samples that slice holds, every bucket index, PDF value, candidate cost and encoding is the one the
// single-tensor analyzer (miq_calib.hip) produces for that slice:
//   InitializePdf / UpdatePdf        DLQ/src/math_functions.cpp:208-288   (DLQ = ModelOptimizations/DlQuantization)
//   TfEnhancedEncodingAnalyzer       DLQ/src/TfEnhancedEncodingAnalyzer.cpp:78-397
//   PercentileEncodingAnalyzer       DLQ/src/PercentileEncodingAnalyzer.cpp:78-198
//
// Layout: channel(i) = (i / n_per_channel) % C, i.e. the tensor is [outer][C][n_per_channel]; a "row" is one run of
// n_per_channel consecutive elements.  State (device memory handed in by the caller, or allocated here): one head
// per channel, C x 512 running PDF values (double) and C x 512 counts of the batch in flight (uint32).
#include "miq_common.h"
#include "miq_encoding_math.h"
#include "miq_fastmath.h"
#include "miq_tfe_search.h"

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstring>
#include <new>
#include <vector>

namespace miq
{
int percentile_encoding_host(bool initialized, const double* x_left, const double* pdf, float percentile, int bw, int sym,
                             int strict, int uns, miq_encoding* out);

namespace
{
constexpr int kPdf      = MIQ_PDF_SIZE;
constexpr int kRows     = kPdf + 2;     // LDS rows: 1 + bucket; rows 0 and kPdf + 1 collect dropped samples
constexpr int kChCopies = 4;            // LDS copies per workgroup (weights spread over a third of the buckets)
constexpr int kRowChunk = 16384;        // elements of a row one workgroup streams
typedef float vf4 __attribute__((ext_vector_type(4)));

struct ChanHead
{
    int initialized;       // PDF range fixed
    int iterations;        // batches folded into the PDF
    int stats_updated;     // an update call has seen this channel
    int enc_bw;
    float bucket_f, offset_f;   // the two floats every bucket index is formed from
    float min_val;              // x_left[i] = min_val + i * bucket
    int pad;
    double bucket;
    double enc_min, enc_max, enc_delta, enc_offset;
};

struct ChanState
{
    ChanHead* head;     // [C]
    double* pdf;        // [C][512]
    uint32_t* counts;   // [C][512]   counts of the batch in flight (multi-workgroup channels only); zero when idle
    float* minmax;      // [2 C]      per-channel (min, max) of the batch in flight
    miq_encoding* enc;  // [C]        what the last search found, in the layout the caller's array has
};

size_t align_up(size_t v)
{
    return (v + 255) & ~(size_t) 255;
}
size_t state_bytes(int64_t c)
{
    return align_up(sizeof(ChanHead) * c) + align_up(sizeof(double) * kPdf * c) + align_up(sizeof(uint32_t) * kPdf * c) +
           align_up(sizeof(float) * 2 * c) + align_up(sizeof(miq_encoding) * c);
}
ChanState carve(void* base, int64_t c)
{
    char* p = static_cast<char*>(base);
    ChanState s;
    s.head = reinterpret_cast<ChanHead*>(p);
    p += align_up(sizeof(ChanHead) * c);
    s.pdf = reinterpret_cast<double*>(p);
    p += align_up(sizeof(double) * kPdf * c);
    s.counts = reinterpret_cast<uint32_t*>(p);
    p += align_up(sizeof(uint32_t) * kPdf * c);
    s.minmax = reinterpret_cast<float*>(p);
    p += align_up(sizeof(float) * 2 * c);
    s.enc = reinterpret_cast<miq_encoding*>(p);
    return s;
}

__global__ __launch_bounds__(256) void chan_reset_kernel(ChanState s, int64_t c)
{
    const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (i < c * kPdf)
    {
        s.pdf[i]    = 0.0;
        s.counts[i] = 0;
    }
    if (i < c)
    {
        ChanHead h{};
        s.head[i] = h;
    }
}

// Fixes the range of every channel that has none yet from the (min, max) of the batch in flight, with the
// reference's arithmetic: DLQ/src/math_functions.cpp:208-262 (signed_vals = true, DTYPE = float).
__global__ __launch_bounds__(256) void chan_init_kernel(ChanState s, int64_t c)
{
    const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (i >= c)
        return;
    ChanHead& h     = s.head[i];
    h.stats_updated = 1;
    if (h.initialized)
        return;
    float min_val = s.minmax[i], max_val = s.minmax[c + i];
    if (min_val == 0 && max_val == 0)
        return;   // an all-zero batch cannot fix a range; the PDF stays uninitialised and this batch is not counted
    if (min_val == max_val)
    {
        const float t = min_val + (float) 0.01;
        max_val       = (max_val < t) ? t : max_val;
    }
    const float center  = (max_val + min_val) / 2;
    const float lo      = center - 3 * (center - min_val);
    const float hi      = center + 3 * (max_val - center);
    min_val             = (-FLT_MAX < lo) ? lo : -FLT_MAX;
    max_val             = (hi < FLT_MAX) ? hi : FLT_MAX;
    const double bucket = ((double) max_val - (double) min_val) / kPdf;
    const double x0     = min_val + 0 * bucket;
    const double x1     = min_val + 1 * bucket;
    h.bucket_f          = (float) (x1 - x0);
    h.offset_f          = (float) x0 / h.bucket_f;
    h.min_val           = min_val;
    h.bucket            = bucket;
    h.iterations        = 0;
    h.initialized       = 1;
}

// One workgroup per (row, chunk of the row).  The bucket of a sample is the reference's for every sample
// (bucket_row, miq_fastmath.h).  `single`: each channel is covered by exactly one workgroup (one row per channel, one
// chunk per row -- the shape of a weight tensor), which then folds its counts into the channel's PDF itself
// (DLQ/src/math_functions.cpp:279-287); otherwise the counts meet in s.counts through atomics and chan_fold_kernel
// folds them.
template <bool VEC, bool SINGLE>
__global__ __launch_bounds__(256) void chan_hist_kernel(const float* __restrict__ in, ChanState s, int64_t num_channel,
                                                        int64_t n_per_channel, uint32_t chunks_per_row)
{
    const int64_t row   = blockIdx.x / chunks_per_row;
    const int64_t c     = row % num_channel;
    const int64_t begin = (int64_t) (blockIdx.x % chunks_per_row) * kRowChunk;
    const int64_t end   = (begin + kRowChunk < n_per_channel) ? begin + kRowChunk : n_per_channel;
    const float* p      = in + row * n_per_channel;
    const ChanHead h    = s.head[c];
    if (!h.initialized)
        return;   // only all-zero batches so far for this channel
    __shared__ uint32_t lds[kRows * kChCopies];
    for (int i = threadIdx.x; i < kRows * kChCopies; i += 256)
        lds[i] = 0;
    __syncthreads();
    const BucketMap map = make_bucket_map(h.bucket_f, h.offset_f, kPdf);
    const int copy      = threadIdx.x & (kChCopies - 1);
    if (VEC)
    {
        // row starts and chunk starts are multiples of four elements on this path
        const vf4* v      = reinterpret_cast<const vf4*>(p + begin);
        const int64_t cnt = (end - begin) / 4;
        for (int64_t i = threadIdx.x; i < cnt; i += 512)
        {
            const vf4 a = __builtin_nontemporal_load(v + i);
            vf4 b       = {NAN, NAN, NAN, NAN};   // dropped
            if (i + 256 < cnt)
                b = __builtin_nontemporal_load(v + i + 256);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                atomicAdd(&lds[bucket_row<kPdf>(a[e], map) * kChCopies + copy], 1u);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                atomicAdd(&lds[bucket_row<kPdf>(b[e], map) * kChCopies + copy], 1u);
        }
    }
    else
    {
        for (int64_t i = begin + threadIdx.x; i < end; i += 256)
            atomicAdd(&lds[bucket_row<kPdf>(p[i], map) * kChCopies + copy], 1u);
    }
    __syncthreads();
    for (int b = threadIdx.x; b < kPdf; b += 256)
    {
        uint32_t cnt = 0;
#pragma unroll
        for (int k = 0; k < kChCopies; ++k)
            cnt += lds[(b + 1) * kChCopies + k];
        if (SINGLE)
        {
            const double prob    = (double) cnt / (double) (int) n_per_channel;
            const int it         = h.iterations;
            s.pdf[c * kPdf + b]  = (s.pdf[c * kPdf + b] * it + prob) / (it + 1);
        }
        else if (cnt)
            atomicAdd(&s.counts[c * kPdf + b], cnt);
    }
    if (SINGLE && threadIdx.x == 0)
        s.head[c].iterations = h.iterations + 1;
}

// Folds the counts of the batch in flight into the PDFs (channels covered by several workgroups); one thread per
// (channel, bucket).  n_batch: samples of one channel in this batch.
__global__ __launch_bounds__(256) void chan_fold_kernel(ChanState s, int64_t c, int64_t n_batch)
{
    const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (i >= c * kPdf)
        return;
    const int64_t ch = i / kPdf;
    if (!s.head[ch].initialized)
        return;
    const int it      = s.head[ch].iterations;
    const double prob = (double) s.counts[i] / (double) (int) n_batch;
    s.pdf[i]          = (s.pdf[i] * it + prob) / (it + 1);
    s.counts[i]       = 0;
}
__global__ __launch_bounds__(256) void chan_count_batch_kernel(ChanState s, int64_t c)
{
    const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (i < c && s.head[i].initialized)
        s.head[i].iterations += 1;
}

// One workgroup per channel, one candidate of the grid per lane (tfe::lane_cost): every wavefront walks the channel's
// PDF once for its 64 candidates.  The lowest-numbered candidate among equal costs wins, as in the reference's single
// loop with its strict comparison.  Launched with 64 * ceil(n_cand / 64) threads (kSearchBlockMax at most; candidates
// beyond that take further walks).
constexpr int kSearchBlockMax = 512;
__global__ __launch_bounds__(kSearchBlockMax) void chan_search_kernel(ChanState s, tfe::SearchArgs a)
{
    constexpr int kWavesMax = kSearchBlockMax / 64;
    const int64_t c         = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int waves = (int) blockDim.x >> 6;
    __shared__ double pdf_s[kPdf];
    __shared__ double mid_s[kPdf];
    __shared__ float fmid_s[kPdf];
    __shared__ double best_cost[kWavesMax];
    __shared__ int best_index[kWavesMax];
    __shared__ float best_delta[kWavesMax];
    __shared__ int best_offset[kWavesMax];
    ChanHead& h = s.head[c];
    if (!h.initialized)
    {
        if (threadIdx.x == 0)
        {
            double enc[4] = {0, 0, 0, 0};
            if (h.stats_updated)
                tfe::encoding_of_zeros(a, enc);
            h.enc_min = enc[0], h.enc_max = enc[1], h.enc_delta = enc[2], h.enc_offset = enc[3];
            h.enc_bw = h.stats_updated ? a.bw : 0;
            s.enc[c] = miq_encoding{enc[0], enc[1], enc[2], enc[3], h.enc_bw};
        }
        return;
    }
    const tfe::PdfView view{s.pdf + c * kPdf, h.min_val, h.bucket};
    tfe::stage_pdf(view, pdf_s, mid_s, fmid_s, threadIdx.x, blockDim.x);
    float minVal, maxVal;
    tfe::wave_range(view, lane, minVal, maxVal);
    __syncthreads();
    double best = DBL_MAX;
    int bidx    = 0x7fffffff;
    float bdelta = -1;
    int boffset  = -1;
    for (int first = 0; first < a.n_cand; first += blockDim.x)
    {
        const int cand = first + threadIdx.x;
        float delta    = 1.f;
        int offset     = 0;
        const bool active = cand < a.n_cand && tfe::candidate(a, minVal, maxVal, cand, delta, offset);
        const double cost = tfe::lane_cost(view, pdf_s, mid_s, fmid_s, a, active, delta, offset);
        if (active && cost < best)
        {
            best = cost, bidx = cand, bdelta = delta, boffset = offset;
        }
    }
    // lowest (cost, candidate number) of the wavefront, then of the workgroup
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
    {
        const double oc = __shfl_xor(best, m);
        const int oi    = __shfl_xor(bidx, m);
        const float od  = __shfl_xor(bdelta, m);
        const int oo    = __shfl_xor(boffset, m);
        if (oc < best || (oc == best && oi < bidx))
        {
            best = oc, bidx = oi, bdelta = od, boffset = oo;
        }
    }
    if (lane == 0)
    {
        best_cost[wave]   = best;
        best_index[wave]  = bidx;
        best_delta[wave]  = bdelta;
        best_offset[wave] = boffset;
    }
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int w = 1; w < waves; ++w)
            if (best_cost[w] < best || (best_cost[w] == best && best_index[w] < bidx))
            {
                best = best_cost[w], bidx = best_index[w], bdelta = best_delta[w], boffset = best_offset[w];
            }
        if (!(bidx != 0x7fffffff && best < DBL_MAX))
        {
            bdelta  = -1;
            boffset = -1;
        }
        double enc[4];
        tfe::encoding_of(a, bdelta, boffset, enc);
        h.enc_min = enc[0], h.enc_max = enc[1], h.enc_delta = enc[2], h.enc_offset = enc[3];
        h.enc_bw = a.bw;
        s.enc[c] = miq_encoding{enc[0], enc[1], enc[2], enc[3], a.bw};
    }
}
}   // namespace
}   // namespace miq

using namespace miq;

struct miq_channel_analyzer
{
    int mode;
    int64_t num_channel;
    float percentile;
    int device;
    void* base;      // device state
    bool owns;       // allocated here (no caller memory given)
    ChanState st;
    bool stats_updated;
};

// Every channel's encoding as the search left it -> four doubles per channel for a later read-back, and the float32
// parameters of the per-channel kernels (the number of steps follows channel 0's encoding).
__global__ void chan_params_kernel(const miq_encoding* found, int64_t c, int bw, double* enc, float* omin, float* omax,
                                   float* odelta, float* ooffset, float* raw_min, float* raw_max)
{
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= c)
        return;
    const miq_encoding e = found[i];
    enc[4 * i + 0]       = e.min;
    enc[4 * i + 1]       = e.max;
    enc[4 * i + 2]       = e.delta;
    enc[4 * i + 3]       = e.offset;
    const ChannelKernelParams p = channel_kernel_params(e.min, e.max, found[0].min == -found[0].max, bw);
    omin[i]    = p.min;
    omax[i]    = p.max;
    odelta[i]  = p.delta;
    ooffset[i] = p.offset;
    raw_min[i] = p.raw_min;
    raw_max[i] = p.raw_max;
}

extern "C" {

int64_t miq_channel_analyzer_state_bytes(int64_t num_channel)
{
    return num_channel > 0 ? (int64_t) state_bytes(num_channel) : 0;
}

int64_t miq_channel_analyzer_workspace_bytes(int64_t num_channel, int64_t num_element, int64_t num_element_per_channel)
{
    return miq_minmax_workspace_bytes(num_channel, num_element, num_element_per_channel);
}

int miq_channel_analyzer_reset(miq_channel_analyzer* a, void* stream)
{
    MIQ_CHECK_ARG(a != nullptr, "null analyzer");
    const int64_t total = a->num_channel * kPdf;
    hipLaunchKernelGGL(chan_reset_kernel, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0, (hipStream_t) stream,
                       a->st, a->num_channel);
    MIQ_CHECK_LAUNCH();
    a->stats_updated = false;
    return MIQ_OK;
}

int miq_channel_analyzer_create(int quantization_mode, int64_t num_channel, void* device_state, void* stream,
                                miq_channel_analyzer** out)
{
    MIQ_CHECK_ARG(out != nullptr, "null output handle");
    MIQ_CHECK_ARG(num_channel > 0 && num_channel < (1ll << 22), "num_channel must be in [1, 2^22)");
    if (quantization_mode != MIQ_QUANTIZATION_TF_ENHANCED && quantization_mode != MIQ_QUANTIZATION_PERCENTILE)
    {
        set_error("quantization mode %d has no per-channel analyzer (TF_ENHANCED and PERCENTILE have; per-channel TF "
                  "statistics are miq_minmax_per_channel_f32)", quantization_mode);
        return MIQ_ERR_UNSUPPORTED;
    }
    MIQ_CHECK_ARG(device_state == nullptr || aligned16(device_state), "device_state must be 16-byte aligned");
    miq_channel_analyzer* a = new (std::nothrow) miq_channel_analyzer();
    MIQ_CHECK_ARG(a != nullptr, "out of host memory");
    a->mode          = quantization_mode;
    a->num_channel   = num_channel;
    a->percentile    = 100.0f;
    a->base          = device_state;
    a->owns          = false;
    a->stats_updated = false;
    hipError_t e     = hipGetDevice(&a->device);
    if (e == hipSuccess && !a->base)
    {
        e       = hipMalloc(&a->base, state_bytes(num_channel));
        a->owns = (e == hipSuccess);
    }
    if (e != hipSuccess)
    {
        set_error("channel analyzer allocation failed: %s", hipGetErrorString(e));
        delete a;
        return MIQ_ERR_HIP;
    }
    a->st = carve(a->base, num_channel);
    if (int rc = miq_channel_analyzer_reset(a, stream))
    {
        if (a->owns)
            (void) hipFree(a->base);
        delete a;
        return rc;
    }
    *out = a;
    return MIQ_OK;
}

int miq_channel_analyzer_destroy(miq_channel_analyzer* a)
{
    if (!a)
        return MIQ_OK;
    if (a->owns)
        (void) hipFree(a->base);
    delete a;
    return MIQ_OK;
}

int miq_channel_analyzer_set_percentile(miq_channel_analyzer* a, float percentile)
{
    MIQ_CHECK_ARG(a != nullptr, "null analyzer");
    MIQ_CHECK_ARG(percentile >= 0.0f && percentile <= 100.0f, "percentile must be in [0, 100] (got %g)",
                  (double) percentile);
    a->percentile = percentile;
    return MIQ_OK;
}

int miq_channel_analyzer_update_stats_f32(miq_channel_analyzer* a, const float* data, int64_t num_element,
                                          int64_t num_element_per_channel, void* workspace, void* stream)
{
    MIQ_CHECK_ARG(a != nullptr, "null analyzer");
    MIQ_CHECK_ARG(data && num_element > 0 && num_element_per_channel > 0, "update_stats needs a non-empty tensor");
    MIQ_CHECK_ARG(num_element % (a->num_channel * num_element_per_channel) == 0,
                  "num_element (%lld) must be a multiple of num_channel * num_element_per_channel (%lld x %lld)",
                  (long long) num_element, (long long) a->num_channel, (long long) num_element_per_channel);
    MIQ_CHECK_ARG(num_element_per_channel < (1ll << 31), "rows of 2^31 elements or more are not handled");
    // a channel's element count per batch is an int in the reference (UpdatePdf's `cnt`) and in the fold kernels
    MIQ_CHECK_ARG(num_element / a->num_channel < (1ll << 31),
                  "a channel holds %lld elements in this batch; the per-channel statistics take fewer than 2^31",
                  (long long) (num_element / a->num_channel));
    hipStream_t s      = (hipStream_t) stream;
    const int64_t c    = a->num_channel;
    const int64_t npc  = num_element_per_channel;
    const int64_t rows = num_element / npc;
    // 1. per-channel (min, max) of this batch, then the range of every channel that has none yet
    if (int rc = miq_minmax_per_channel_f32(data, c, num_element, npc, a->st.minmax, workspace, stream))
        return rc;
    hipLaunchKernelGGL(chan_init_kernel, dim3((unsigned) ((c + 255) / 256)), dim3(256), 0, s, a->st, c);
    // 2. counts
    const int64_t chunks = (npc + kRowChunk - 1) / kRowChunk;
    MIQ_CHECK_ARG(rows * chunks < (1ll << 31), "too many rows for one launch");
    const bool single = (rows == c && chunks == 1);
    const bool vec    = aligned16(data) && npc % 4 == 0;
    const dim3 grid((unsigned) (rows * chunks));
    if (single && vec)
        hipLaunchKernelGGL((chan_hist_kernel<true, true>), grid, dim3(256), 0, s, data, a->st, c, npc, (uint32_t) chunks);
    else if (single)
        hipLaunchKernelGGL((chan_hist_kernel<false, true>), grid, dim3(256), 0, s, data, a->st, c, npc, (uint32_t) chunks);
    else if (vec)
        hipLaunchKernelGGL((chan_hist_kernel<true, false>), grid, dim3(256), 0, s, data, a->st, c, npc, (uint32_t) chunks);
    else
        hipLaunchKernelGGL((chan_hist_kernel<false, false>), grid, dim3(256), 0, s, data, a->st, c, npc,
                           (uint32_t) chunks);
    if (!single)
    {
        // the element count of a channel's batch is an int in the reference (UpdatePdf's `cnt`)
        hipLaunchKernelGGL(chan_fold_kernel, dim3((unsigned) ((c * kPdf + 255) / 256)), dim3(256), 0, s, a->st, c,
                           (rows / c) * npc);
        hipLaunchKernelGGL(chan_count_batch_kernel, dim3((unsigned) ((c + 255) / 256)), dim3(256), 0, s, a->st, c);
    }
    MIQ_CHECK_LAUNCH();
    a->stats_updated = true;
    return MIQ_OK;
}

int miq_channel_analyzer_compute_encodings(miq_channel_analyzer* a, int bw, int use_symmetric, int use_strict_symmetric,
                                           int use_unsigned_symmetric, miq_encoding* out, int* is_valid, void* stream)
{
    MIQ_CHECK_ARG(a && out && is_valid, "null argument");
    MIQ_CHECK_ARG(bw >= 1 && bw <= 32, "bitwidth must be in [1, 32] (got %d)", bw);
    hipStream_t s   = (hipStream_t) stream;
    const int64_t c = a->num_channel;
    *is_valid = a->stats_updated ? 1 : 0;
    if (!a->stats_updated)
    {
        memset(out, 0, sizeof(miq_encoding) * c);
        return MIQ_OK;
    }
    if (a->mode == MIQ_QUANTIZATION_PERCENTILE)
    {
        memset(out, 0, sizeof(miq_encoding) * c);
        std::vector<ChanHead> heads(c);
        // PercentileEncodingAnalyzer::computeEncoding is 512 buckets of host arithmetic per channel: read the PDFs back
        std::vector<double> pdf((size_t) c * kPdf), x_left(kPdf);
        MIQ_CHECK_HIP(hipMemcpyAsync(heads.data(), a->st.head, sizeof(ChanHead) * c, hipMemcpyDeviceToHost, s));
        MIQ_CHECK_HIP(hipMemcpyAsync(pdf.data(), a->st.pdf, sizeof(double) * kPdf * c, hipMemcpyDeviceToHost, s));
        MIQ_CHECK_HIP(hipStreamSynchronize(s));
        for (int64_t ch = 0; ch < c; ++ch)
        {
            const ChanHead& h = heads[ch];
            for (int i = 0; i < kPdf; ++i)
                x_left[i] = h.min_val + i * h.bucket;
            if (int rc = percentile_encoding_host(h.initialized != 0, x_left.data(), pdf.data() + ch * kPdf,
                                                  a->percentile, bw, use_symmetric, use_strict_symmetric,
                                                  use_unsigned_symmetric, out + ch))
                return rc;
        }
        return MIQ_OK;
    }
    const tfe::SearchArgs sa =
        tfe::make_search_args(bw, use_symmetric, use_strict_symmetric, use_unsigned_symmetric);
    const int search_block = std::min(kSearchBlockMax, 64 * ((sa.n_cand + 63) / 64));
    hipLaunchKernelGGL(chan_search_kernel, dim3((unsigned) c), dim3(search_block), 0, s, a->st, sa);
    MIQ_CHECK_LAUNCH();
    // the kernel leaves the encodings in the caller's layout: one copy straight into `out`
    MIQ_CHECK_HIP(hipMemcpyAsync(out, a->st.enc, sizeof(miq_encoding) * c, hipMemcpyDeviceToHost, s));
    MIQ_CHECK_HIP(hipStreamSynchronize(s));
    return MIQ_OK;
}

int miq_channel_analyzer_compute_encodings_device(miq_channel_analyzer* a, int bw, int use_symmetric,
                                                  int use_strict_symmetric, int use_unsigned_symmetric, double* enc,
                                                  float* out_min, float* out_max, float* out_delta, float* out_offset,
                                                  float* raw_min, float* raw_max, int* is_valid, void* stream)
{
    MIQ_CHECK_ARG(a && enc && out_min && out_max && out_delta && out_offset && raw_min && raw_max && is_valid,
                  "null argument");
    MIQ_CHECK_ARG(bw >= 1 && bw <= 31, "bitwidth must be in [1, 31] (got %d)", bw);
    if (a->mode == MIQ_QUANTIZATION_PERCENTILE)
    {
        set_error("the percentile analyzer computes its encodings on the host: use miq_channel_analyzer_compute_encodings");
        return MIQ_ERR_UNSUPPORTED;
    }
    hipStream_t s   = (hipStream_t) stream;
    const int64_t c = a->num_channel;
    *is_valid       = a->stats_updated ? 1 : 0;
    if (!a->stats_updated)
        return MIQ_OK;
    const tfe::SearchArgs sa =
        tfe::make_search_args(bw, use_symmetric, use_strict_symmetric, use_unsigned_symmetric);
    const int search_block = std::min(kSearchBlockMax, 64 * ((sa.n_cand + 63) / 64));
    hipLaunchKernelGGL(chan_search_kernel, dim3((unsigned) c), dim3(search_block), 0, s, a->st, sa);
    MIQ_CHECK_LAUNCH();
    hipLaunchKernelGGL(chan_params_kernel, dim3((unsigned) ((c + 255) / 256)), dim3(256), 0, s, a->st.enc, c, bw, enc,
                       out_min, out_max, out_delta, out_offset, raw_min, raw_max);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_channel_analyzer_get_stats_histogram(miq_channel_analyzer* a, int64_t channel, double* x_left, double* pdf,
                                             int* num_buckets, void* stream)
{
    MIQ_CHECK_ARG(a && x_left && pdf && num_buckets, "null argument");
    MIQ_CHECK_ARG(channel >= 0 && channel < a->num_channel, "channel %lld out of range", (long long) channel);
    hipStream_t s = (hipStream_t) stream;
    ChanHead h;
    MIQ_CHECK_HIP(hipMemcpyAsync(&h, a->st.head + channel, sizeof(ChanHead), hipMemcpyDeviceToHost, s));
    MIQ_CHECK_HIP(hipMemcpyAsync(pdf, a->st.pdf + channel * kPdf, sizeof(double) * kPdf, hipMemcpyDeviceToHost, s));
    MIQ_CHECK_HIP(hipStreamSynchronize(s));
    *num_buckets = h.initialized ? kPdf : 0;
    for (int i = 0; i < kPdf; ++i)
        x_left[i] = h.min_val + i * h.bucket;
    return MIQ_OK;
}

}   // extern "C"
