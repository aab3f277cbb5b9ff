// Calibration kernels for gfx950: fused min/max reduction, 512-bucket histogram (PDF) accumulation and the
// TF-Enhanced (SQNR) delta/offset candidate search.
//
// Reference arithmetic followed here (paths relative to the reference root, DLQ = ModelOptimizations/DlQuantization):
//   GetMin/GetMax                    DLQ/src/math_functions.cpp:328-347
//   InitializePdf / UpdatePdf        DLQ/src/math_functions.cpp:208-288
//   GetHistogram_cpu                 DLQ/src/math_functions.cpp:368-384
//   TfEncodingAnalyzer               DLQ/src/TfEncodingAnalyzer.cpp:59-101
//   TfEnhancedEncodingAnalyzer       DLQ/src/TfEnhancedEncodingAnalyzer.cpp:78-397
//
// Design: every statistic lives in one device-resident state block per analyzer.  update_stats is one streaming
// kernel per batch in steady state (the first batch adds a min/max pass); each launch also folds the previous
// batch's integer bin counts into the running PDF, so nothing is copied to the host and nothing synchronises until
// an encoding is asked for.  Bin counts are integers, hence independent of the order in which lanes add them.
// The histogram is privatised in LDS: 8 interleaved copies of the 512 bins per workgroup, lane l using copy
// l mod 8, and merged into one of 32 global replicas per batch.
#include "miq_common.h"
#include "miq_agent.h"
#include "miq_fastmath.h"
#include "miq_tfe_search.h"
#include "miq_encoding_math.h"
#include "miq_entropy.h"

#include <algorithm>
#include <cfloat>
#include <climits>
#include <cstddef>
#include <cmath>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

namespace miq
{
namespace
{
constexpr int kPdf      = MIQ_PDF_SIZE;
constexpr int kMaxCand  = 512;
// LDS copies of the histogram per workgroup (lane l counts into copy l % kCopies) and the upper bound on streaming
// workgroups.  8 copies are 16 KB, so 8 workgroups fit a compute unit and 2048 are resident at once: the streaming
// workgroups plus the one that folds the previous batch must not exceed that, or the last one is dispatched only when
// another has retired and lengthens the launch (measured: 0.5 us of 7).  4 and 2 copies are faster on spread-out data but
// collapse when the values share a bucket (constant tensor: 8.8 / 14.0 us against 6.9 us with 8).
typedef float vf4 __attribute__((ext_vector_type(4)));
constexpr int kCopies   = 8;
constexpr int kMaxGrid  = 2048;
// The histogram launch: four 16-byte loads of a lane in flight and at most 1024 workgroups.  Every workgroup clears an
// LDS histogram and flushes it with up to 512 global atomics, so fewer, longer workgroups pay less of that (the flush
// alone is 0.8 us of a 7.5 us launch at 2048 workgroups); with two loads in flight 1024 workgroups keep too few bytes
// on their way.  Measured per [32,256,28,28] batch, back to back: 2 loads x 2048 workgroups 7.4 us, 4 x 1024 7.1 us,
// 4 x 1568 7.6 us, 4 x 512 9.2 us, 8 x 784 8.7 us.
constexpr int kHistUnroll  = 4;
constexpr int kHistMaxGrid = 1024;
constexpr int kReplicas = 32;     // global count replicas: workgroup b merges into replica b % kReplicas, so at most
                                  // kMaxGrid / kReplicas atomics ever meet on one address

// float <-> unsigned key whose integer order is the float order (for atomicMin/atomicMax)
__host__ __device__ inline uint32_t f2ord(float f)
{
    uint32_t u;
#ifdef __HIP_DEVICE_COMPILE__
    u = __float_as_uint(f);
#else
    memcpy(&u, &f, 4);
#endif
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__host__ __device__ inline float ord2f(uint32_t o)
{
    uint32_t u = (o & 0x80000000u) ? (o & 0x7fffffffu) : ~o;
#ifdef __HIP_DEVICE_COMPILE__
    return __uint_as_float(u);
#else
    float f;
    memcpy(&f, &u, 4);
    return f;
#endif
}
constexpr uint32_t kOrdPosInf = 0xff800000u;   // f2ord(+inf)
constexpr uint32_t kOrdNegInf = 0x007fffffu;   // f2ord(-inf)

// Layout: a small head that every read-back needs, then the inspection block (PDF, last counts, search scratch),
// then device-only accumulators.  Read-backs copy a prefix, never the accumulators.
struct DevState
{
    // ---- head
    uint32_t ticket_search;
    int stats_updated;   // _statsUpdated
    uint32_t minmax_seq; // number of the update call whose (min, max) partials wait in `partial`; 0 = none
    int initialized;     // PDF range fixed (xLeft.size() != 0 in the reference)
    int iterations;      // batches folded into the PDF so far (mirror of iters[] for inspection)
    float bucket_f, pdf_offset_f;
    float range_min;         // x_left[i] = range_min + i * range_bucket
    int n_cand;
    int best_index;
    int enc_bw;
    int iters[2];            // the same count, written alternately: the launch of update call k reads iters[(k - 1) & 1]
                             // and writes iters[k & 1], so that workgroups of one launch never read what it writes
    uint32_t batch_seq[2];   // update-call number whose counts sit in counts[i]; 0 = none pending
    int64_t batch_n[2];      // element count of that batch
    double range_bucket;
    double acc_min, acc_max; // TF analyzer: accumulated range in double (TfEncodingAnalyzer.h:84-90)
    double enc_min, enc_max, enc_delta, enc_offset;
    // ---- inspection block
    double xLeft[kPdf];
    double pdf[kPdf];
    uint32_t last_counts[kPdf];   // the last folded batch
    float cand_delta[kMaxCand];
    int cand_offset[kMaxCand];
    int cand_valid[kMaxCand];
    double cand_cost[kMaxCand];
    // ---- device-only accumulators
    uint32_t counts[2][kReplicas][kPdf];   // two batches in flight (filling / being folded), replicated; zero when idle
    float2 partial[kMaxGrid];              // per-workgroup (min, max) of the batch in flight
};
constexpr size_t kHeadBytes    = offsetof(DevState, xLeft);
constexpr size_t kInspectBytes = offsetof(DevState, counts);

__device__ __forceinline__ float wave_min(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v = fminf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// ---------------------------------------------------------------------------------------------------- min / max
// mode kMinMaxTf : TF analyzer   -> fold the batch range into acc_min / acc_max
// mode kMinMaxTfe: TF-Enhanced   -> if the PDF is not initialised yet, derive its range from this batch
enum
{
    kMinMaxTf  = 1,
    kMinMaxTfe = 2
};

// Range of the PDF from the extremes of the first batch that is not all zeros: DLQ/src/math_functions.cpp:208-241 with
// signed_vals = true, DTYPE = float.  bucket_f and offset_f are the two floats every later bucket index is formed from.
struct PdfRange
{
    float min_val;
    double bucket;
    float bucket_f, offset_f;
};
__device__ __forceinline__ PdfRange pdf_range(float min_val, float max_val)
{
    if (min_val == max_val)
    {
        const float t = min_val + (float) 0.01;
        max_val       = (max_val < t) ? t : max_val;
    }
    const float center = (max_val + min_val) / 2;
    const float lo     = center - 3 * (center - min_val);
    const float hi     = center + 3 * (max_val - center);
    min_val            = (-FLT_MAX < lo) ? lo : -FLT_MAX;
    max_val            = (hi < FLT_MAX) ? hi : FLT_MAX;
    PdfRange r;
    r.min_val = min_val;
    r.bucket  = ((double) max_val - (double) min_val) / kPdf;
    // x_left[1] - x_left[0] and x_left[0], rounded to float, drive the bucket index of every later batch
    const double x0 = min_val + 0 * r.bucket;
    const double x1 = min_val + 1 * r.bucket;
    r.bucket_f      = (float) (x1 - x0);
    r.offset_f      = (float) x0 / r.bucket_f;
    return r;
}

__device__ void initialize_pdf(DevState* st, const PdfRange& r)
{
    for (int i = threadIdx.x; i < kPdf; i += blockDim.x)
    {
        st->xLeft[i] = r.min_val + i * r.bucket;
        st->pdf[i]   = 0.0;
    }
    if (threadIdx.x == 0)
    {
        st->bucket_f     = r.bucket_f;
        st->pdf_offset_f = r.offset_f;
        st->range_min    = r.min_val;
        st->range_bucket = r.bucket;
        st->initialized  = 1;
    }
}

// Folds `count` per-workgroup (min, max) pairs; every thread of the workgroup (kBlock threads) gets the result.
__device__ __forceinline__ float2 fold_partials(const float2* partial, int count)
{
    float mn = INFINITY, mx = -INFINITY;
    for (int i = threadIdx.x; i < count; i += kBlock)
    {
        const float2 p = partial[i];
        mn             = fminf(mn, p.x);
        mx             = fmaxf(mx, p.y);
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    __shared__ float smn[kBlock / 64], smx[kBlock / 64];
    if ((threadIdx.x & 63) == 0)
    {
        smn[threadIdx.x >> 6] = mn;
        smx[threadIdx.x >> 6] = mx;
    }
    __syncthreads();
    float gmn = smn[0], gmx = smx[0];
    for (int w = 1; w < kBlock / 64; ++w)
    {
        gmn = fminf(gmn, smn[w]);
        gmx = fmaxf(gmx, smx[w]);
    }
    return make_float2(gmn, gmx);
}

// Pass 1: every workgroup reduces its share and stores one (min, max) pair -- plain stores, no atomics, because
// same-address device atomics from a thousand workgroups serialise at roughly 15 ns each on this part.  Wide workgroups
// (1024 lanes, four 16-byte loads in flight per lane, one workgroup per compute unit for a 25 MB batch) measured
// fastest for a read-only pass and leave few pairs for the consumer to fold.
constexpr int kMmBlock  = 1024;
constexpr int kMmUnroll = 4;
constexpr int kMmGrid   = 256;
template <bool VEC>
__global__ __launch_bounds__(kMmBlock) void minmax_kernel(const float* __restrict__ in, int64_t n, DevState* st, int mode,
                                                          uint32_t seq)
{
    if (mode == kMinMaxTfe && st->initialized)
        return;   // range already fixed: later batches need no min/max pass
    float mn = INFINITY, mx = -INFINITY;
    if (VEC)
    {
        const int64_t nvec   = n / 4;
        const vf4* v         = reinterpret_cast<const vf4*>(in);
        const int64_t stride = (int64_t) gridDim.x * kMmBlock * kMmUnroll;
        const vf4 nan4       = {NAN, NAN, NAN, NAN};   // fminf/fmaxf skip NaN
        for (int64_t base = (int64_t) blockIdx.x * kMmBlock * kMmUnroll; base < nvec; base += stride)
        {
            vf4 a[kMmUnroll];
#pragma unroll
            for (int u = 0; u < kMmUnroll; ++u)
            {
                const int64_t i = base + u * kMmBlock + threadIdx.x;
                a[u]            = nan4;
                if (i < nvec)
                    a[u] = __builtin_nontemporal_load(v + i);
            }
#pragma unroll
            for (int u = 0; u < kMmUnroll; ++u)
            {
                mn = fminf(fminf(mn, a[u][0]), fminf(a[u][1], fminf(a[u][2], a[u][3])));
                mx = fmaxf(fmaxf(mx, a[u][0]), fmaxf(a[u][1], fmaxf(a[u][2], a[u][3])));
            }
        }
        if (blockIdx.x == 0 && threadIdx.x < (uint32_t) (n - nvec * 4))
        {
            const float a = in[nvec * 4 + threadIdx.x];
            mn            = fminf(mn, a);
            mx            = fmaxf(mx, a);
        }
    }
    else
    {
        for (int64_t i = (int64_t) blockIdx.x * kMmBlock + threadIdx.x; i < n; i += (int64_t) gridDim.x * kMmBlock)
        {
            const float a = in[i];
            mn            = fminf(mn, a);
            mx            = fmaxf(mx, a);
        }
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    __shared__ float smn[kMmBlock / 64], smx[kMmBlock / 64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0)
    {
        smn[wave] = mn;
        smx[wave] = mx;
    }
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int w = 1; w < kMmBlock / 64; ++w)
        {
            mn = fminf(mn, smn[w]);
            mx = fmaxf(mx, smx[w]);
        }
        st->partial[blockIdx.x] = make_float2(mn, mx);
        if (blockIdx.x == 0)
            st->minmax_seq = seq;
    }
}

// Pass 2 of the TF (min/max) analyzer, one workgroup: fold the pairs into the accumulated range.  (The TF-Enhanced
// analyzer has no second launch: the histogram kernel of the same update call folds the pairs in its prologue.)
__global__ __launch_bounds__(kBlock) void minmax_finalize_kernel(DevState* st, int grid)
{
    if (st->minmax_seq == 0)
        return;
    const float2 g = fold_partials(st->partial, grid);
    if (threadIdx.x == 0)
    {
        st->minmax_seq    = 0;
        st->stats_updated = 1;
        // DLQ/src/TfEncodingAnalyzer.cpp:59-71
        const double cmn = (double) g.x, cmx = (double) g.y;
        st->acc_min = (cmn < st->acc_min) ? cmn : st->acc_min;
        st->acc_max = (st->acc_max < cmx) ? cmx : st->acc_max;
    }
}

// per-channel min/max: partial reductions meet in `keys` (uint32[2C], ordered keys) through atomics
__global__ void fill_keys_kernel(uint32_t* keys, int64_t c)
{
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < c)
    {
        keys[i]     = kOrdPosInf;
        keys[c + i] = kOrdNegInf;
    }
}
__global__ void decode_keys_kernel(uint32_t* keys, int64_t c2)
{
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < c2)
        reinterpret_cast<float*>(keys)[i] = ord2f(keys[i]);
}
// one workgroup per (row, chunk); row = outer * C + c, every row has n_per_channel contiguous elements
__global__ __launch_bounds__(kBlock) void minmax_rows_kernel(const float* __restrict__ in, int64_t num_channel,
                                                             int64_t n_per_channel, int64_t chunk,
                                                             uint32_t chunks_per_row, uint32_t* keys)
{
    const int64_t row   = blockIdx.x / chunks_per_row;
    const int64_t c     = row % num_channel;
    const int64_t begin = (int64_t) (blockIdx.x % chunks_per_row) * chunk;
    int64_t end         = begin + chunk;
    if (end > n_per_channel)
        end = n_per_channel;
    const float* p = in + row * n_per_channel;
    float mn = INFINITY, mx = -INFINITY;
    for (int64_t i = begin + threadIdx.x; i < end; i += kBlock)
    {
        const float a = p[i];
        mn            = fminf(mn, a);
        mx            = fmaxf(mx, a);
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    __shared__ float smn[kBlock / 64], smx[kBlock / 64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0)
    {
        smn[wave] = mn;
        smx[wave] = mx;
    }
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int w = 1; w < kBlock / 64; ++w)
        {
            mn = fminf(mn, smn[w]);
            mx = fmaxf(mx, smx[w]);
        }
        atomicMin(&keys[c], f2ord(mn));
        atomicMax(&keys[num_channel + c], f2ord(mx));
    }
}

// The same reduction without atomics: every (row, chunk) workgroup stores its pair, 16-byte loads where the row
// layout allows; a second kernel folds the pairs of a channel.  With one workgroup per channel (direct) the pair is
// the result.
template <bool VEC>
__global__ __launch_bounds__(kBlock) void minmax_rows_partial_kernel(const float* __restrict__ in,
                                                                     int64_t n_per_channel, int64_t chunk,
                                                                     uint32_t chunks_per_row, float2* partial,
                                                                     float* direct_out, int64_t num_channel)
{
    const int64_t row   = blockIdx.x / chunks_per_row;
    const int64_t begin = (int64_t) (blockIdx.x % chunks_per_row) * chunk;
    int64_t end         = begin + chunk;
    if (end > n_per_channel)
        end = n_per_channel;
    const float* p = in + row * n_per_channel;
    float mn = INFINITY, mx = -INFINITY;
    if (VEC)
    {
        // the base address and chunk are multiples of 16 bytes / 4 elements on this path, and so is the row
        // length unless there is only one row
        const float4* v   = reinterpret_cast<const float4*>(p + begin);
        const int64_t cnt = (end - begin) / 4;
        int64_t i         = threadIdx.x;
        for (; i + kBlock < cnt; i += 2 * kBlock)
        {
            const float4 a = v[i], b = v[i + kBlock];
            mn = fminf(fminf(fminf(mn, a.x), fminf(a.y, a.z)), fminf(fminf(a.w, b.x), fminf(b.y, fminf(b.z, b.w))));
            mx = fmaxf(fmaxf(fmaxf(mx, a.x), fmaxf(a.y, a.z)), fmaxf(fmaxf(a.w, b.x), fmaxf(b.y, fmaxf(b.z, b.w))));
        }
        if (i < cnt)
        {
            const float4 a = v[i];
            mn             = fminf(fminf(mn, a.x), fminf(fminf(a.y, a.z), a.w));
            mx             = fmaxf(fmaxf(mx, a.x), fmaxf(fmaxf(a.y, a.z), a.w));
        }
        // up to three trailing elements of a single row whose length is no multiple of 4
        const int64_t tail = begin + cnt * 4 + threadIdx.x;
        if (tail < end)
        {
            mn = fminf(mn, p[tail]);
            mx = fmaxf(mx, p[tail]);
        }
    }
    else
    {
        for (int64_t i = begin + threadIdx.x; i < end; i += kBlock)
        {
            const float a = p[i];
            mn            = fminf(mn, a);
            mx            = fmaxf(mx, a);
        }
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    __shared__ float smn[kBlock / 64], smx[kBlock / 64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0)
    {
        smn[wave] = mn;
        smx[wave] = mx;
    }
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int w = 1; w < kBlock / 64; ++w)
        {
            mn = fminf(mn, smn[w]);
            mx = fmaxf(mx, smx[w]);
        }
        if (direct_out)
        {
            direct_out[blockIdx.x]               = mn;
            direct_out[num_channel + blockIdx.x] = mx;
        }
        else
            partial[blockIdx.x] = make_float2(mn, mx);
    }
}

// LANES lanes per channel (a wavefront, or the workgroup when a channel has many pairs) fold its outer x chunks
// pairs.
template <int LANES>
__global__ __launch_bounds__(kBlock) void minmax_rows_fold_kernel(const float2* __restrict__ partial,
                                                                  int64_t num_channel, int64_t outer,
                                                                  uint32_t chunks_per_row, float* out)
{
    const int64_t c = (int64_t) blockIdx.x * (kBlock / LANES) + threadIdx.x / LANES;
    const int lane  = threadIdx.x % LANES;
    float mn = INFINITY, mx = -INFINITY;
    if (c < num_channel)
    {
        const int64_t items = outer * chunks_per_row;
        for (int64_t j = lane; j < items; j += LANES)
        {
            const int64_t o = j / chunks_per_row, k = j % chunks_per_row;
            const float2 v  = partial[(o * num_channel + c) * chunks_per_row + k];
            mn              = fminf(mn, v.x);
            mx              = fmaxf(mx, v.y);
        }
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    if (LANES > 64)
    {
        __shared__ float smn[kBlock / 64], smx[kBlock / 64];
        if ((threadIdx.x & 63) == 0)
        {
            smn[threadIdx.x >> 6] = mn;
            smx[threadIdx.x >> 6] = mx;
        }
        __syncthreads();
        for (int w = 0; w < kBlock / 64; ++w)
        {
            mn = fminf(mn, smn[w]);
            mx = fmaxf(mx, smx[w]);
        }
    }
    if (lane == 0 && c < num_channel)
    {
        out[c]               = mn;
        out[num_channel + c] = mx;
    }
}

// ---------------------------------------------------------------------------------------------------- histogram
// Adds one sample to the workgroup's LDS histogram: row 1 + bucket, rows 0 and kPdf + 1 collect dropped samples (out of
// range, NaN), so the add is unconditional.  bucket_row (miq_fastmath.h) decides most samples with one fused
// multiply-add and evaluates the reference's divide / subtract / round sequence (DLQ/src/math_functions.cpp:375-382)
// only within a hair of a bucket edge; the bucket is the reference's for every sample.
constexpr int kRows = kPdf + 2;
template <int COPIES>
__device__ __forceinline__ void hist_add(uint32_t* lds, float x, const BucketMap& m, int copy)
{
    atomicAdd(&lds[bucket_row<kPdf>(x, m) * COPIES + copy], 1u);
}

// Folds the counts of one finished batch into the running PDF (DLQ/src/math_functions.cpp:279-287; the element
// count is an int in the reference) and clears them.  The work is cut into kFoldSlices slices of kFoldBins buckets;
// a slice is folded by kFoldBins x kReplicas lanes, one replica count per lane (a single round trip to memory: load,
// clear, add up across the 32 lanes of a bucket, one lane updates the running value).  In a histogram launch the
// first kFoldSlices streaming workgroups fold one slice each while their first tile is on its way, so folding the
// previous batch adds no workgroup and no latency to the launch.
constexpr int kFoldBins   = kBlock / kReplicas;   // 8 buckets per slice
constexpr int kFoldSlices = kPdf / kFoldBins;     // 64 slices
static_assert(kReplicas == 32 && kFoldBins * kReplicas == kBlock && kFoldSlices * kFoldBins == kPdf, "fold layout");

// One slice in two steps so that a caller can keep the loads in flight under other work.
struct FoldLoad
{
    uint32_t count;   // this lane's replica count
    double running;   // leader lanes (replica 0): the bucket's running PDF value
    int it;           // leader lanes: batches folded so far.  A per-lane (vector) load on purpose: a scalar load shares
                      // its wait counter with the LDS operations and would hold up the histogram's LDS clear
};
// `lane_id` in [0, kBlock): lanes [32 j, 32 j + 32) share bucket slice * kFoldBins + j.
__device__ __forceinline__ FoldLoad fold_load(const DevState* st, int buf, int it_slot, int slice, int lane_id)
{
    const int b = slice * kFoldBins + lane_id / kReplicas;
    const int r = lane_id % kReplicas;
    FoldLoad f;
    f.running = 0.0;
    f.it      = 0;
    if (r == 0)
    {
        f.running = st->pdf[b];
        f.it      = st->iters[it_slot];
    }
    f.count = st->counts[buf][r][b];
    return f;
}
// Plain loads and stores, not an atomic exchange: an atomic in flight would have to complete before the workgroup's
// next barrier (its release fence), a load need not.
__device__ __forceinline__ void fold_store(DevState* st, int buf, int64_t batch_n, int slice, int lane_id, FoldLoad f)
{
    const int b           = slice * kFoldBins + lane_id / kReplicas;
    const int r           = lane_id % kReplicas;
    agent_store(&st->counts[buf][r][b], 0u);
    uint32_t c = f.count;
#pragma unroll
    for (int o = kReplicas / 2; o > 0; o >>= 1)
        c += __shfl_xor(c, o);   // stays inside the 32 lanes of this bucket
    if (r == 0)
    {
        agent_store(&st->last_counts[b], c);
        const double prob = (double) c / (double) (int) batch_n;
        agent_store(&st->pdf[b], (f.running * f.it + prob) / (f.it + 1));
    }
}

// One launch per batch, every workgroup streams its share of the tensor into counts[buf]; while the first tile is in
// flight kFoldSlices of the workgroups fold a slice each of the previous batch (counts[1 - buf], if that batch was
// accumulated) into the PDF, and the first of them keeps the books (iteration count, stamp of this batch): no second
// launch and no cross-workgroup hand-shake is needed.  (A dedicated folding workgroup was the longest-running one of
// the launch: with the memory system saturated every dependent round trip costs microseconds.)  `seq` numbers the update calls of this analyzer; a buffer is pending
// iff its stamp equals the sequence number of the call that filled it.
// Where the bucket width and offset come from:
//   KNOWN            kernel arguments (the host has learnt them; the steady state, compiled without the other two);
//   else, when the min/max pass of this same update call ran (st->minmax_seq == seq): every workgroup folds that pass's
//                    mm_grid (min, max) pairs itself and derives the range with the reference's arithmetic -- the first
//                    batch that is not all zeros costs two launches, not three -- and workgroup 0 writes the range into
//                    the state and, through `probe`, into host memory, so that the host can stop queuing min/max passes
//                    without ever waiting for the device;
//   else             the device state, which also says whether a range exists at all.
// prev_n (KNOWN only): element count of the previous update call when the host knows that call was counted, else 0
// (then the stamp decides).
// probe: device-visible pinned host words {generation, -, bucket_f, pdf_offset_f}; the generation word is written last.
template <bool VEC, bool KNOWN>
__global__ __launch_bounds__(kBlock) void hist_kernel(const float* __restrict__ in, int64_t n, DevState* st, int buf,
                                                      uint32_t seq, float bucket_arg, float off_arg, int mm_grid,
                                                      int* probe, int generation, int64_t prev_n, int fold_first)
{
    const int groups     = gridDim.x;
    const int group      = (int) blockIdx.x;
    const vf4* v         = reinterpret_cast<const vf4*>(in);
    const vf4 nan4       = {NAN, NAN, NAN, NAN};   // dropped by hist_add
    const int64_t nvec   = n / 4;
    const int64_t stride = (int64_t) groups * kBlock * kHistUnroll;
    int64_t base         = (int64_t) group * kBlock * kHistUnroll;
    // ---- the previous batch, step 1: kFoldSlices workgroups from fold_first on (the first of those with the smallest
    // share of the tensor: they retire earliest) request their slice of its counts before anything else, so that this
    // round trip runs under the first tile's
    int64_t pending_n = 0;
    const int slice   = group - fold_first;   // host: 0 <= fold_first <= groups - kFoldSlices
    const bool folds  = slice >= 0 && slice < kFoldSlices;
    FoldLoad fl{};
    if (folds)
    {
        pending_n = KNOWN ? prev_n : 0;
        if (pending_n == 0 && st->batch_seq[1 - buf] != 0 && st->batch_seq[1 - buf] == seq - 1)
            pending_n = st->batch_n[1 - buf];
        // (lane 0 of the last workgroup needs the iteration count even when nothing is pending: slice 0 loads it)
        if (pending_n > 0 || slice == 0)
            fl = fold_load(st, 1 - buf, 1 - buf, slice, threadIdx.x);
    }
    vf4 a[kHistUnroll];
    // first tile's loads go out next: they overlap the state reads, the fold and the LDS clear
    // (a tile that exists as a whole is requested without a condition per lane: the compiler then waits for each
    // vector where it is first used instead of for all four before the first)
    auto request = [&](vf4(&to)[kHistUnroll], int64_t at) {
        if (at + kHistUnroll * kBlock <= nvec)   // workgroup-uniform
        {
#pragma unroll
            for (int u = 0; u < kHistUnroll; ++u)
                to[u] = __builtin_nontemporal_load(v + at + u * kBlock + threadIdx.x);   // read once: not kept in the caches
        }
        else
        {
#pragma unroll
            for (int u = 0; u < kHistUnroll; ++u)
            {
                const int64_t i = at + u * kBlock + threadIdx.x;
                to[u]           = nan4;
                if (i < nvec)
                    to[u] = __builtin_nontemporal_load(v + i);
            }
        }
    };
    if (VEC)
        request(a, base);
    // ---- the range
    float bucket = bucket_arg, off = off_arg;
    bool have_range = true, fresh = false;
    PdfRange range{};
    if (!KNOWN)
    {
        fresh = (st->minmax_seq == seq);
        if (fresh)
        {
            const float2 g = fold_partials(st->partial, mm_grid);
            // DLQ/src/math_functions.cpp:248-262: an all-zero batch cannot fix a range; the PDF stays uninitialised and
            // this batch is not counted
            have_range = !(g.x == 0 && g.y == 0);
            range      = pdf_range(g.x, g.y);
            bucket     = range.bucket_f;
            off        = range.offset_f;
        }
        else
        {
            have_range = st->initialized != 0;
            bucket     = st->bucket_f;
            off        = st->pdf_offset_f;
        }
    }
    if (slice == 0)
    {
        if (fresh && have_range)
            initialize_pdf(st, range);
        if (threadIdx.x == 0)
        {
            if (fresh)
                st->stats_updated = 1;
            if (have_range)
            {
                agent_store(&st->batch_seq[buf], seq);
                agent_store(&st->batch_n[buf], n);
                if (!KNOWN && probe)
                {
                    probe[2] = __float_as_int(bucket);
                    probe[3] = __float_as_int(off);
                    __threadfence_system();
                    __hip_atomic_store(&probe[0], generation, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
                }
            }
        }
    }
    if (!have_range)
        return;   // only all-zero batches so far: the reference returns without touching the PDF (and nothing can be
                  // pending, both iteration slots are still 0: step 2 below has nothing to do)
    __shared__ uint32_t lds[kRows * kCopies];
    const BucketMap map = make_bucket_map(bucket, off, kPdf);
    for (int i = threadIdx.x; i < kRows * kCopies; i += kBlock)
        lds[i] = 0;
    __syncthreads();
    const int copy = threadIdx.x & (kCopies - 1);
    if (VEC)
    {
        while (true)
        {
#pragma unroll
            for (int u = 0; u < kHistUnroll; ++u)
            {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    hist_add<kCopies>(lds, a[u][e], map, copy);
            }
            base += stride;
            if (base >= nvec)
                break;
            request(a, base);   // (requested before the first tile is counted, into a second register set: 8.4 us per batch against 7.0)
        }
        if (group == 0 && threadIdx.x < (uint32_t) (n - nvec * 4))
            hist_add<kCopies>(lds, in[nvec * 4 + threadIdx.x], map, copy);
    }
    else
    {
        for (int64_t i = (int64_t) group * kBlock + threadIdx.x; i < n; i += (int64_t) groups * kBlock)
            hist_add<kCopies>(lds, in[i], map, copy);
    }
    __syncthreads();
    uint32_t* dst = st->counts[buf][group % kReplicas];
    for (int b = threadIdx.x; b < kPdf; b += kBlock)
    {
        uint32_t s = 0;
#pragma unroll
        for (int c = 0; c < kCopies; ++c)
            s += lds[(b + 1) * kCopies + c];
        if (s)
            atomicAdd(&dst[b], s);
    }
    // ---- the previous batch, step 2: fold the slice requested at the top (its loads landed long ago; doing this last
    // keeps every wait of the streaming part free of them); the workgroup of slice 0 keeps the books
    if (folds)
    {
        if (pending_n > 0)
            fold_store(st, 1 - buf, pending_n, slice, threadIdx.x, fl);
        if (slice == 0 && threadIdx.x == 0)
        {
            // (the stamp of the folded batch stays: the other folding workgroups may not have read it yet, and no
            // later launch can take it for pending because it compares with its own seq - 1)
            const int now = fl.it + (pending_n > 0 ? 1 : 0);
            agent_store(&st->iters[buf], now);
            agent_store(&st->iterations, now);
        }
    }
}

// Folds whichever batch is still pending (at most one).  Queued before anything reads the PDF.  kFoldSlices workgroups,
// a slice each, as in hist_kernel (one workgroup doing all of it took 28 us: its write-through stores go out one after
// the other).  Every workgroup reads the iteration count before it draws its ticket, so the workgroup that draws the
// last one may overwrite it.  (The ticket counter is the search kernel's: the two never run at the same time.)
__global__ __launch_bounds__(kBlock) void hist_flush_kernel(DevState* st, uint32_t seq)
{
    const int buf = (int) (seq & 1u);
    if (st->batch_seq[buf] == 0 || st->batch_seq[buf] != seq)
        return;
    const int64_t batch_n = st->batch_n[buf];
    const FoldLoad f      = fold_load(st, buf, buf, blockIdx.x, threadIdx.x);
    fold_store(st, buf, batch_n, blockIdx.x, threadIdx.x, f);
    __shared__ int it_seen;
    if (threadIdx.x == 0)
        it_seen = f.it;   // lane 0 leads a bucket: it has read the count
    __syncthreads();      // every leader of this workgroup has read iters[buf] and batch_seq[buf]
    if (threadIdx.x == 0 &&
        __hip_atomic_fetch_add(&st->ticket_search, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.x - 1)
    {
        st->ticket_search  = 0;
        st->iters[buf]     = it_seen + 1;   // what the next update call's launch reads
        st->iterations     = it_seen + 1;
        st->batch_seq[buf] = 0;
    }
}

// ------------------------------------------------------------------------------------------------ SQNR search
// One wavefront per candidate (miq_tfe_search.h); the workgroup that finishes last picks the winner.
using tfe::SearchArgs;
__global__ __launch_bounds__(kBlock) void tfe_search_kernel(DevState* st, SearchArgs a)
{
    constexpr int kWaves = kBlock / 64;
    const int wave       = threadIdx.x >> 6;
    const int cand       = blockIdx.x * kWaves + wave;   // one wavefront per candidate
    const int lane       = threadIdx.x & 63;
    __shared__ double term_all[kWaves][kPdf];
    __shared__ bool is_last;

    if (st->initialized && cand < a.n_cand)
    {
        // x_left[i] of the state is min_val + i * bucket with these two values (initialize_pdf)
        const tfe::PdfView view{st->pdf, st->range_min, st->range_bucket};
        float minVal, maxVal, delta;
        int offset;
        tfe::wave_range(view, lane, minVal, maxVal);
        const bool valid  = tfe::candidate(a, minVal, maxVal, cand, delta, offset);
        const double cost = valid ? tfe::wave_cost(view, a, delta, offset, lane, term_all[wave]) : 0.0;
        if (lane == 0)
        {
            // performed at the device's point of coherence: the workgroup that draws the last ticket reads them there
            agent_store(&st->cand_delta[cand], delta);
            agent_store(&st->cand_offset[cand], offset);
            agent_store(&st->cand_valid[cand], valid ? 1 : 0);
            agent_store(&st->cand_cost[cand], cost);
        }
    }
    // the ticket is drawn after every wavefront's stores have been acknowledged (miq_agent.h)
    publications_acknowledged();
    __syncthreads();
    if (threadIdx.x == 0)
    {
        const uint32_t t = __hip_atomic_fetch_add(&st->ticket_search, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last          = (t == gridDim.x - 1);
    }
    __syncthreads();
    if (!is_last || wave != 0)
        return;
    last_ticket_acquire();

    // ---- last wavefront: pick the winner (first strict minimum) and form the encoding
    if (lane == 0)
    {
        st->ticket_search = 0;
        st->n_cand        = st->initialized ? a.n_cand : 0;
    }
    double enc[4] = {0, 0, 0, 0};
    if (!st->initialized)
    {
        if (lane == 0)
        {
            st->best_index = -1;
            if (st->stats_updated)
                tfe::encoding_of_zeros(a, enc);
            st->enc_min = enc[0], st->enc_max = enc[1], st->enc_delta = enc[2], st->enc_offset = enc[3];
            st->enc_bw = st->stats_updated ? a.bw : 0;
        }
        return;
    }
    // every candidate's cost, validity, delta and offset are requested at once: a read at the device's point of
    // coherence takes 1-2 us, and six rounds of them plus the winner's two, with a release fence per wavefront before
    // the ticket, made the launch 20.1 us where it now takes 12.4
    constexpr int kPerLane = kMaxCand / 64;
    double cost[kPerLane];
    int valid[kPerLane], offs[kPerLane];
    float delt[kPerLane];
#pragma unroll
    for (int k = 0; k < kPerLane; ++k)
    {
        const int c = lane + 64 * k;
        valid[k]    = 0;
        if (c < a.n_cand)
        {
            cost[k]  = agent_load(&st->cand_cost[c]);
            valid[k] = agent_load(&st->cand_valid[c]);
            delt[k]  = agent_load(&st->cand_delta[c]);
            offs[k]  = agent_load(&st->cand_offset[c]);
        }
    }
    double best     = DBL_MAX;
    int bidx        = 0x7fffffff;
    float bestDelta = -1;
    int bestOffset  = -1;
#pragma unroll
    for (int k = 0; k < kPerLane; ++k)
        if (valid[k] && cost[k] < best)
        {
            best = cost[k], bidx = lane + 64 * k, bestDelta = delt[k], bestOffset = offs[k];
        }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        const double ob = __shfl_xor(best, o);
        const int oi    = __shfl_xor(bidx, o);
        const float od  = __shfl_xor(bestDelta, o);
        const int oo    = __shfl_xor(bestOffset, o);
        if (ob < best || (ob == best && oi < bidx))
        {
            best = ob, bidx = oi, bestDelta = od, bestOffset = oo;
        }
    }
    if (lane == 0)
    {
        if (!(bidx != 0x7fffffff && best < DBL_MAX))
        {
            bidx       = -1;
            bestDelta  = -1;
            bestOffset = -1;
        }
        tfe::encoding_of(a, bestDelta, bestOffset, enc);
        st->enc_min = enc[0], st->enc_max = enc[1], st->enc_delta = enc[2], st->enc_offset = enc[3];
        st->enc_bw     = a.bw;
        st->best_index = bidx;
    }
}

// ------------------------------------------------------------------------------------------------- MSE search
// MseEncodingAnalyzer<float>::computeEncoding on the PDF the TF-Enhanced analyzer keeps (DLQ/src/MseEncodingAnalyzer.cpp
// :78-262): every pair of one bucket edge below zero (or zero) and one above zero (or zero) inside the observed range
// is a candidate (min, max); a candidate's cost is the PDF-weighted squared error of quantize-dequantizing the bucket
// centres on its grid, accumulated bucket by bucket in the reference's types; the first candidate of least cost wins.
// Three launches on one stream: the edge walk (sequential float additions, one lane), one lane per candidate, the pick.
// The reference's edge walk `for (float i = histMin; i <= histMax; i += width)` has no end when `width` is below half
// a unit in the last place of the edges; here it stops after kMseMaxWalk steps (a PDF needs 512 to 514).
constexpr int kMseMaxWalk  = 1025;
constexpr int kMseMaxEdges = kMseMaxWalk + 1;
constexpr int kMseGrid     = 256;    // one workgroup per compute unit: 65536 candidates in one pass, more in strides
struct MseScratch
{
    int n_min, n_max, n_center, pad;
    float range_min, range_max;   // what the search returns when no candidate has a cost below FLT_MAX
    float min_cand[kMseMaxEdges + 1];
    float max_cand[kMseMaxEdges + 1];
    float center[kMseMaxEdges];
    float pdf_at[kMseMaxEdges];
    float part_cost[kMseGrid];
    int part_index[kMseGrid];
};

// (int) of a double or float the way x86-64 converts, where the reference runs: outside int -> INT_MIN
__device__ __forceinline__ int to_int_x86(double v)
{
    return (v > -2147483649.0 && v < 2147483648.0) ? (int) v : INT_MIN;
}

__global__ __launch_bounds__(kBlock) void mse_prepare_kernel(const DevState* st, MseScratch* m)
{
    __shared__ float s_range[2];
    __shared__ float s_walk[kMseMaxWalk];
    __shared__ float s_center[kMseMaxWalk];
    __shared__ int s_n_walk, s_n_center;
    if (!st->initialized)
    {
        if (threadIdx.x == 0)
            m->n_min = m->n_max = m->n_center = 0;
        return;
    }
    const tfe::PdfView view{st->pdf, st->range_min, st->range_bucket};
    const int lane = threadIdx.x;
    if (lane < 64)
    {
        float lo, hi;
        tfe::wave_range(view, lane, lo, hi);   // findOriginalRange<float>, DLQ/src/math_functions.cpp:400-433
        if (lane == 0)
            s_range[0] = lo, s_range[1] = hi;
    }
    __syncthreads();
    const float width    = (float) (view.x_left(1) - view.x_left(0));
    const float hist_min = (float) view.x_left(0);
    const float min_val  = s_range[0];
    const float max_val  = s_range[1] + width;
    // The two chains of float additions of _minimizeMSE: the walk over the bucket edges (:156-163) and the bucket
    // centres (:172-183; at most as many centres as edges are used).  The walk ends at the first value above hist_max,
    // normally the 513th to 515th: kMseFastWalk steps of both chains run without a test on one lane (additions and LDS
    // stores only), every lane then looks for the first value that ends the walk, and only a walk that has not ended
    // by then goes on step by step.
    constexpr int kMseFastWalk = 520;
    const float hist_max       = (float) (view.x_left(kPdf - 1) + width);
    if (lane == 0)
    {
        float i = hist_min, c = min_val + width / 2;
        for (int k = 0; k < kMseFastWalk; ++k)
        {
            s_walk[k]   = i;
            s_center[k] = c;
            i += width;
            c = c + width;
        }
        s_n_walk = kMseFastWalk;
    }
    __syncthreads();
    for (int k = lane; k < kMseFastWalk; k += blockDim.x)
        if (!(s_walk[k] <= hist_max))
            atomicMin(&s_n_walk, k);
    __syncthreads();
    if (lane == 0 && s_n_walk == kMseFastWalk)
    {
        int walked = kMseFastWalk;
        float c    = s_center[kMseFastWalk - 1] + width;
        for (float i = s_walk[kMseFastWalk - 1] + width; i <= hist_max && walked < kMseMaxWalk; i += width, ++walked)
        {
            s_walk[walked]   = i;
            s_center[walked] = c;
            c                = c + width;
        }
        s_n_walk = walked;
    }
    __syncthreads();
    if (lane < 64)
    {
        // Edges in the reference's order: the observed minimum, then every walked value inside [min_val, max_val];
        // those below zero are the min candidates, those above zero the max candidates, zero closes both lists
        // (_pickMinMaxCandidatesMSECalib :202-234).  One wavefront compacts 64 entries at a time, order kept.
        const int n_entries = s_n_walk + 1;
        int n_min = 0, n_max = 0, n_edges = 0;
        for (int base = 0; base < n_entries; base += 64)
        {
            const int j    = base + lane;
            const bool in  = j < n_entries;
            const float v  = !in ? 0.f : (j == 0 ? min_val : s_walk[j - 1]);
            const bool keep = in && (j == 0 || (v >= min_val && v <= max_val));
            const uint64_t below = __ballot(keep && v < 0);
            const uint64_t above = __ballot(keep && v > 0);
            const uint64_t before = (1ull << lane) - 1;
            if (keep && v < 0)
                m->min_cand[n_min + __popcll(below & before)] = v;
            if (keep && v > 0)
                m->max_cand[n_max + __popcll(above & before)] = v;
            n_min += __popcll(below);
            n_max += __popcll(above);
            n_edges += __popcll(__ballot(keep));
        }
        if (lane == 0)
        {
            m->min_cand[n_min] = 0.f;
            m->max_cand[n_max] = 0.f;
            m->n_min           = n_min + 1;
            m->n_max           = n_max + 1;
            m->n_center        = n_edges - 1;
            m->range_min       = min_val;
            m->range_max       = max_val;
            s_n_center         = n_edges - 1;
        }
    }
    __syncthreads();
    for (int k = lane; k < s_n_center; k += blockDim.x)
    {
        const float c = s_center[k];
        int ind       = to_int_x86(floorf((c - hist_min) / width));
        ind           = ind < 0 ? 0 : (ind > kPdf - 1 ? kPdf - 1 : ind);
        m->center[k]  = c;
        m->pdf_at[k]  = (float) st->pdf[ind];
    }
}

struct MseArgs
{
    int bw, sym, strict, uns;
    int int_steps;   // int(2^bw - 1), one less for strict symmetric, converted on the host
};

// _computeMSECost :236-262 for one candidate per lane; each workgroup keeps its first candidate of least cost.
__global__ __launch_bounds__(kBlock) void mse_cost_kernel(MseScratch* m, MseArgs a)
{
    __shared__ float s_center[kMseMaxEdges];
    __shared__ float s_pdf[kMseMaxEdges];
    __shared__ float s_cost[kBlock / 64];
    __shared__ int s_index[kBlock / 64];
    const int n_center = m->n_center, n_min = m->n_min, n_max = m->n_max;
    const int n_cand = n_min * n_max - 1;   // the last pair is {0, 0}: no candidate
    for (int k = threadIdx.x; k < n_center; k += blockDim.x)
    {
        s_center[k] = m->center[k];
        s_pdf[k]    = m->pdf_at[k];
    }
    __syncthreads();
    float best = FLT_MAX;
    int index  = INT_MAX;
    for (int cand = blockIdx.x * blockDim.x + threadIdx.x; cand < n_cand; cand += gridDim.x * blockDim.x)
    {
        const float c_min = m->min_cand[cand / n_max];
        const float c_max = m->max_cand[cand % n_max];
        const EncodingD e = computed_encodings(a.bw, c_min, c_max, a.sym != 0, a.strict != 0, a.uns != 0);
        float err         = 0.f;
        for (int k = 0; k < n_center; ++k)
        {
            const float v       = s_center[k];
            const float clamped = tfe::std_max(c_min, tfe::std_min(v, c_max));
            const int q         = to_int_x86(round(clamped / e.delta - e.offset));
            const float back    = (float) (e.delta * (q + e.offset));
            const double diff   = (double) (v - back);
            err                 = (float) (err + s_pdf[k] * (diff * diff));   // std::pow(float, 2) is exact in double
        }
        if (err < best)
            best = err, index = cand;
    }
    // lowest cost, lowest candidate number among equals
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        const float oc = __shfl_xor(best, o);
        const int oi   = __shfl_xor(index, o);
        if (oc < best || (oc == best && oi < index))
            best = oc, index = oi;
    }
    if ((threadIdx.x & 63) == 0)
        s_cost[threadIdx.x >> 6] = best, s_index[threadIdx.x >> 6] = index;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int w = 1; w < kBlock / 64; ++w)
            if (s_cost[w] < best || (s_cost[w] == best && s_index[w] < index))
                best = s_cost[w], index = s_index[w];
        m->part_cost[blockIdx.x]  = best;
        m->part_index[blockIdx.x] = index;
    }
}

// The winner among the workgroups' winners, zero gated into its range, the encoding of that range (computeEncoding
// :78-130) written where the host reads it.
__global__ __launch_bounds__(64) void mse_pick_kernel(DevState* st, const MseScratch* m, MseArgs a)
{
    const int lane = threadIdx.x;
    float best     = FLT_MAX;
    int index      = INT_MAX;
    if (st->initialized)
        for (int k = lane; k < kMseGrid; k += 64)
        {
            const float c = m->part_cost[k];
            const int i   = m->part_index[k];
            if (c < best || (c == best && i < index))
                best = c, index = i;
        }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        const float oc = __shfl_xor(best, o);
        const int oi   = __shfl_xor(index, o);
        if (oc < best || (oc == best && oi < index))
            best = oc, index = oi;
    }
    if (lane != 0)
        return;
    double enc[4] = {0, 0, 0, 0};
    if (!st->initialized)
    {
        if (st->stats_updated)
        {
            // only zeros were seen: an encoding that covers float 0 (:92-108)
            const double d = (1.0 - -1.0) / a.int_steps;
            const double o = floor(-1.0 / d);
            enc[0] = o * d, enc[1] = enc[0] + a.int_steps * d, enc[2] = d, enc[3] = o;
        }
        st->enc_min = enc[0], st->enc_max = enc[1], st->enc_delta = enc[2], st->enc_offset = enc[3];
        st->enc_bw     = st->stats_updated ? a.bw : 0;
        st->best_index = -1;
        st->n_cand     = 0;
        return;
    }
    float a_min = m->range_min, a_max = m->range_max;
    if (index != INT_MAX)
        a_min = m->min_cand[index / m->n_max], a_max = m->max_cand[index % m->n_max];
    a_min             = tfe::std_min(a_min, 0.f);
    a_max             = tfe::std_max(a_max, 0.f);
    const EncodingD e = computed_encodings(a.bw, a_min, a_max, a.sym != 0, a.strict != 0, a.uns != 0);
    st->enc_min = e.min, st->enc_max = e.max, st->enc_delta = e.delta, st->enc_offset = e.offset;
    st->enc_bw     = a.bw;
    st->best_index = (index == INT_MAX) ? -1 : index;
    st->n_cand     = 0;   // the candidate arrays of the state belong to the TF-Enhanced search and stay empty
}

__global__ void reset_state_kernel(DevState* st)
{
    const int i = threadIdx.x;   // launched with kPdf threads
    if (i == 0)
    {
        st->ticket_search = 0;
        st->stats_updated = 0;
        st->minmax_seq    = 0;
        st->acc_min       = DBL_MAX;
        st->acc_max       = -DBL_MAX;
        st->initialized = st->iterations = 0;
        st->iters[0] = st->iters[1] = 0;
        st->bucket_f = st->pdf_offset_f = st->range_min = 0.f;
        st->range_bucket                = 0;
        st->n_cand                      = 0;
        st->best_index                  = -1;
        st->enc_min = st->enc_max = st->enc_delta = st->enc_offset = 0;
        st->enc_bw                                                 = 0;
    }
    st->xLeft[i]       = 0;
    st->pdf[i]         = 0;
    for (int r = 0; r < kReplicas; ++r)
        st->counts[0][r][i] = st->counts[1][r][i] = 0;
    st->last_counts[i] = 0;
    if (i < 2)
    {
        st->batch_seq[i] = 0;
        st->batch_n[i]   = 0;
    }
}

// Partial (min, max) pairs of miq_minmax_per_channel_static_f32: device memory that belongs to the loaded library, one
// copy per GPU, held until the process ends.  In host code this name is only a handle for hipGetSymbolAddress; the
// address kernels receive is the one that call returns for the current device (static_scratch below).
constexpr int64_t kStaticPairs = 32768;   // 256 KiB
static __device__ __align__(256) float2 scratch[kStaticPairs];

constexpr int kMaxDevices = 64;
float2* g_scratch_ptr[kMaxDevices];   // per device: address of that GPU's copy of `scratch`; null until first use
std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch`, looked up once per device.
int static_scratch(float2** out)
{
    int dev = 0;
    MIQ_CHECK_HIP(hipGetDevice(&dev));
    MIQ_CHECK_ARG(dev >= 0 && dev < kMaxDevices, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev])
    {
        float2* ptr = nullptr;
        MIQ_CHECK_HIP(hipGetSymbolAddress((void**) &ptr, HIP_SYMBOL(scratch)));
        MIQ_CHECK_ARG(ptr != nullptr, "no device address for the library's scratch array");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return MIQ_OK;
}

int hist_grid(int64_t n)
{
    int64_t blocks = (n / 4 + (int64_t) kBlock * kHistUnroll - 1) / ((int64_t) kBlock * kHistUnroll);
    if (blocks < 1)
        blocks = 1;
    if (blocks > kHistMaxGrid)
        blocks = kHistMaxGrid;
    return (int) blocks;
}
}   // namespace

// PercentileEncodingAnalyzer<float>::computeEncoding on the PDF read back from the device
// (DLQ/src/PercentileEncodingAnalyzer.cpp:78-198; findOriginalRange: DLQ/src/math_functions.cpp:400-433).
// 512 buckets of host arithmetic, in the reference's types: float range values, double cdf.
int percentile_encoding_host(bool initialized, const double* x_left, const double* pdf, float percentile, int bw, int sym,
                             int strict, int uns, miq_encoding* out)
{
    float num_steps = (float) (std::pow(2, bw) - 1);
    if (sym && strict)
        num_steps -= 1;
    if (!initialized)
    {
        // only zeros were seen: an encoding that covers float 0
        out->min    = -1;
        out->max    = 1;
        out->delta  = (out->max - out->min) / (int) num_steps;
        out->offset = std::floor(out->min / out->delta);
        out->min    = out->offset * out->delta;
        out->max    = out->min + (int) num_steps * out->delta;
        out->bw     = bw;
        return MIQ_OK;
    }
    float min_val = (float) x_left[0], max_val = (float) x_left[kPdf - 1];
    for (int i = 0; i < kPdf; ++i)
        if (pdf[i] > 0)
        {
            min_val = (float) x_left[i];
            break;
        }
    for (int i = kPdf - 1; i > 0; --i)
        if (pdf[i] > 0)
        {
            max_val = (float) x_left[i];
            break;
        }
    min_val = std::min(min_val, 0.0f);
    max_val = std::max(max_val, 0.0f);
    max_val = std::max(max_val, min_val + (float) 0.01);
    float a_min = min_val, a_max = max_val;
    if (percentile != 100.0f)
    {
        const float width = (float) (x_left[1] - x_left[0]);
        a_min             = (float) x_left[0];
        a_max             = (float) (x_left[kPdf - 1] + width);
        std::vector<double> cdf(pdf, pdf + kPdf);
        for (int i = 1; i < kPdf; ++i)
            cdf[i] += cdf[i - 1];
        const float left = 1 - percentile / 100;
        for (int i = 0; i < kPdf; ++i)
            if (cdf[i] >= left)
            {
                a_min = (float) x_left[i];
                break;
            }
        const float right = percentile / 100;
        for (int i = kPdf - 1; i >= 0; --i)
            if (cdf[i] < right && x_left[i] < max_val)
            {
                a_max = (float) (x_left[i] + width);
                break;
            }
        if (a_min == a_max)
            a_max += width;
    }
    a_min = std::min(a_min, 0.0f);
    a_max = std::max(a_max, 0.0f);
    return miq_get_computed_encodings(bw, a_min, a_max, sym, strict, uns, out);
}

}   // namespace miq

using namespace miq;

struct miq_analyzer
{
    int mode;
    float percentile;    // percentile analyzer only
    MseScratch* mse;     // MSE analyzer only: candidate lists, bucket centres, per-workgroup winners (device)
    EntropyAnalyzer* entropy;   // entropy analyzer only: its own histogram and search; `st` is not used
    int device;
    DevState* st;        // device
    void* pinned;        // host staging (pinned) for read-backs
    bool owns_state;     // st was allocated here (no caller memory given)
    bool needs_reset;    // st has not been cleared yet: the first call that queues work does it
    bool stats_updated;  // host mirror of _isEncodingValid / _statsUpdated
    bool range_known;    // host knows the PDF range has been fixed, so no further min/max pass is queued
    int* probe_flag;     // pinned host words the histogram kernel writes once the range is fixed:
                         // {generation, -, bucket_f, pdf_offset_f}; the host only ever polls them
    int* probe_dev;      // the same words as the device addresses them
    int64_t counted_n;   // element count of the last update call if the range was already known to the host then, else 0
    int generation;      // bumped by reset, so that a launch queued before the reset cannot be believed after it
    float bucket_f, pdf_offset_f;   // valid once range_known
    uint32_t seq;        // number of TF-Enhanced update calls since the last reset
    int last_bw;
    // an encoding request queued ahead of its read-back (miq_analyzer_queue_encoding): valid while nothing else has
    // been asked of the object since
    bool queued;
    int queued_args[4];
    hipStream_t queued_stream;
};

extern "C" {

// chunk length and chunks per row of the workspace path: about 16 K elements per workgroup, shorter when that would
// leave compute units idle
static void minmax_geometry(int64_t rows, int64_t n_per_channel, int64_t& chunk, int64_t& bx)
{
    chunk = 16384;
    while (chunk > 2048 && rows * ((n_per_channel + chunk - 1) / chunk) < 2048)
        chunk /= 2;
    bx = (n_per_channel + chunk - 1) / chunk;
}

static int launch_minmax_rows(const float* in, int64_t num_channel, int64_t rows, int64_t n_per_channel,
                              uint32_t* keys, void* workspace, hipStream_t s)
{
    if (workspace && rows > 0)
    {
        int64_t chunk, bx;
        minmax_geometry(rows, n_per_channel, chunk, bx);
        MIQ_CHECK_ARG(rows * bx < (1ll << 31), "too many rows for one launch");
        float* out        = reinterpret_cast<float*>(keys);
        const bool direct = rows == num_channel && bx == 1;
        const bool vec    = (n_per_channel % 4 == 0 || rows == 1) && aligned16(in);
        float2* partial   = static_cast<float2*>(workspace);
        const dim3 grid((unsigned) (rows * bx));
        if (vec)
            hipLaunchKernelGGL(minmax_rows_partial_kernel<true>, grid, dim3(kBlock), 0, s, in, n_per_channel, chunk,
                               (uint32_t) bx, partial, direct ? out : nullptr, num_channel);
        else
            hipLaunchKernelGGL(minmax_rows_partial_kernel<false>, grid, dim3(kBlock), 0, s, in, n_per_channel, chunk,
                               (uint32_t) bx, partial, direct ? out : nullptr, num_channel);
        if (!direct && (rows / num_channel) * bx >= 1024)
            hipLaunchKernelGGL(minmax_rows_fold_kernel<kBlock>, dim3((unsigned) num_channel), dim3(kBlock), 0, s, partial,
                               num_channel, rows / num_channel, (uint32_t) bx, out);
        else if (!direct)
            hipLaunchKernelGGL(minmax_rows_fold_kernel<64>, dim3((unsigned) ((num_channel + 3) / 4)), dim3(kBlock), 0, s,
                               partial, num_channel, rows / num_channel, (uint32_t) bx, out);
        MIQ_CHECK_LAUNCH();
        return MIQ_OK;
    }
    // without a workspace: partial results meet in the output through atomics on order-preserving integer keys
    // keys: uint32[2C] ordered keys (min block then max block); decoded in place to float at the end
    hipLaunchKernelGGL(fill_keys_kernel, dim3((unsigned) ((num_channel + kBlock - 1) / kBlock)), dim3(kBlock), 0, s,
                       keys, num_channel);
    if (rows > 0)
    {
        int64_t chunk = (int64_t) kBlock * 16;
        int64_t bx    = (n_per_channel + chunk - 1) / chunk;
        if (rows * bx > (1ll << 20))
        {
            // keep the grid modest for very long rows: fewer, longer chunks
            bx    = ((1ll << 20) + rows - 1) / rows;
            chunk = (n_per_channel + bx - 1) / bx;
            bx    = (n_per_channel + chunk - 1) / chunk;
        }
        MIQ_CHECK_ARG(rows * bx < (1ll << 31), "too many rows for one launch");
        hipLaunchKernelGGL(minmax_rows_kernel, dim3((unsigned) (rows * bx)), dim3(kBlock), 0, s, in, num_channel,
                           n_per_channel, chunk, (uint32_t) bx, keys);
    }
    hipLaunchKernelGGL(decode_keys_kernel, dim3((unsigned) ((2 * num_channel + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       s, keys, 2 * num_channel);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int64_t miq_minmax_workspace_bytes(int64_t num_channel, int64_t num_element, int64_t num_element_per_channel)
{
    if (num_channel <= 0 || num_element_per_channel <= 0 || num_element <= 0)
        return 8;
    int64_t chunk, bx;
    const int64_t rows = num_element / num_element_per_channel;
    minmax_geometry(rows, num_element_per_channel, chunk, bx);
    return (int64_t) sizeof(float2) * std::max<int64_t>(rows * bx, 1);
}

int miq_minmax_f32(const float* in, int64_t n, float* out_min_max, void* workspace, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && out_min_max && (n == 0 || in), "null pointer or negative count");
    return launch_minmax_rows(in, 1, n > 0 ? 1 : 0, n > 0 ? n : 1, reinterpret_cast<uint32_t*>(out_min_max),
                              workspace, (hipStream_t) stream);
}

int miq_minmax_per_channel_f32(const float* in, int64_t num_channel, int64_t num_element,
                               int64_t num_element_per_channel, float* out_min_max, void* workspace, void* stream)
{
    MIQ_CHECK_ARG(num_channel > 0 && num_element_per_channel > 0 && num_element >= 0 && out_min_max,
                  "bad channel geometry or null output");
    MIQ_CHECK_ARG(num_element == 0 || in, "null input");
    MIQ_CHECK_ARG(num_element % num_element_per_channel == 0,
                  "num_element must be a multiple of num_element_per_channel");
    MIQ_CHECK_ARG((num_element / num_element_per_channel) % num_channel == 0,
                  "num_element must be a multiple of num_channel * num_element_per_channel");
    return launch_minmax_rows(in, num_channel, num_element / num_element_per_channel, num_element_per_channel,
                              reinterpret_cast<uint32_t*>(out_min_max), workspace, (hipStream_t) stream);
}

int miq_init(void)
{
    float2* unused = nullptr;
    return static_scratch(&unused);
}

int miq_minmax_per_channel_static_f32(const float* in, int64_t num_channel, int64_t num_element,
                                      int64_t num_element_per_channel, float* out_min_max, void* stream)
{
    MIQ_CHECK_ARG(num_channel > 0 && num_element_per_channel > 0 && num_element >= 0 && out_min_max,
                  "bad channel geometry or null output");
    MIQ_CHECK_ARG(num_element == 0 || in, "null input");
    MIQ_CHECK_ARG(num_element % num_element_per_channel == 0,
                  "num_element must be a multiple of num_element_per_channel");
    MIQ_CHECK_ARG((num_element / num_element_per_channel) % num_channel == 0,
                  "num_element must be a multiple of num_channel * num_element_per_channel");
    const int64_t need = miq_minmax_workspace_bytes(num_channel, num_element, num_element_per_channel);
    MIQ_CHECK_ARG(need <= kStaticPairs * (int64_t) sizeof(float2),
                  "tensor too large for the allocation-free min/max: it needs %lld bytes of partial results, the "
                  "library's static scratch holds %lld; use miq_minmax_per_channel_f32 with a workspace",
                  (long long) need, (long long) (kStaticPairs * (int64_t) sizeof(float2)));
    float2* ws = nullptr;
    if (int rc = static_scratch(&ws))
        return rc;
    // every partial pair the fold kernel reads is written by the kernel before it in this call: nothing to clear
    return launch_minmax_rows(in, num_channel, num_element / num_element_per_channel, num_element_per_channel,
                              reinterpret_cast<uint32_t*>(out_min_max), ws, (hipStream_t) stream);
}

static int percentile_encoding(const DevState* h, float percentile, int bw, int sym, int strict, int uns,
                               miq_encoding* out)
{
    return percentile_encoding_host(h->initialized != 0, h->xLeft, h->pdf, percentile, bw, sym, strict, uns, out);
}

int64_t miq_analyzer_state_bytes(void)
{
    return (int64_t) sizeof(DevState);
}

// The state is cleared by the first call that queues work (on that call's stream): creation itself queues nothing and
// waits for nothing.
static int ensure_reset(miq_analyzer* a, hipStream_t s)
{
    if (a->needs_reset)
    {
        hipLaunchKernelGGL(reset_state_kernel, dim3(1), dim3(kPdf), 0, s, a->st);
        MIQ_CHECK_LAUNCH();
        a->needs_reset = false;
    }
    return MIQ_OK;
}

int miq_analyzer_create(int quantization_mode, miq_analyzer** out)
{
    return miq_analyzer_create_in(quantization_mode, nullptr, out);
}

int miq_analyzer_create_in(int quantization_mode, void* device_state, miq_analyzer** out)
{
    MIQ_CHECK_ARG(out != nullptr, "null output handle");
    MIQ_CHECK_ARG(device_state == nullptr || aligned16(device_state), "device_state must be 16-byte aligned");
    if (quantization_mode != MIQ_QUANTIZATION_TF && quantization_mode != MIQ_QUANTIZATION_TF_ENHANCED &&
        quantization_mode != MIQ_QUANTIZATION_PERCENTILE && quantization_mode != MIQ_QUANTIZATION_MSE &&
        quantization_mode != MIQ_QUANTIZATION_ENTROPY)
    {
        set_error("quantization mode %d is not implemented (TF, TF_ENHANCED, PERCENTILE, MSE and ENTROPY are)",
                  quantization_mode);
        return MIQ_ERR_UNSUPPORTED;
    }
    miq_analyzer* a = new (std::nothrow) miq_analyzer();
    MIQ_CHECK_ARG(a != nullptr, "out of host memory");
    a->mode          = quantization_mode;
    a->percentile    = 100.0f;   // PercentileEncodingAnalyzer.h: the default clips nothing
    a->mse           = nullptr;
    a->entropy       = nullptr;
    a->st            = static_cast<DevState*>(device_state);
    a->owns_state    = (device_state == nullptr);
    a->needs_reset   = true;
    a->pinned        = nullptr;
    a->stats_updated = false;
    a->range_known   = false;
    a->probe_flag    = nullptr;
    a->probe_dev     = nullptr;
    a->generation    = 1;
    a->counted_n     = 0;
    a->bucket_f = a->pdf_offset_f = 0.f;
    a->seq           = 0;
    a->last_bw       = 0;
    hipError_t e     = hipGetDevice(&a->device);
    if (e == hipSuccess && quantization_mode == MIQ_QUANTIZATION_ENTROPY)
    {
        // the entropy analyzer keeps a histogram of its own kind in memory of its own; a caller's state is left alone
        a->owns_state = false;
        a->st         = nullptr;
        if (int rc = entropy_create(&a->entropy))
        {
            delete a;
            return rc;
        }
        *out = a;
        return MIQ_OK;
    }
    if (e == hipSuccess && a->owns_state)
        e = hipMalloc((void**) &a->st, sizeof(DevState));
    if (e == hipSuccess && quantization_mode == MIQ_QUANTIZATION_MSE)
        e = hipMalloc((void**) &a->mse, sizeof(MseScratch));   // every field is written before it is read
    if (e == hipSuccess)
        e = hipHostMalloc(&a->pinned, kInspectBytes + 64, hipHostMallocDefault);   // + 4 probe words
    if (e == hipSuccess)
    {
        a->probe_flag = reinterpret_cast<int*>(static_cast<char*>(a->pinned) + kInspectBytes);
        memset(a->probe_flag, 0, 4 * sizeof(int));
        e = hipHostGetDevicePointer(reinterpret_cast<void**>(&a->probe_dev), a->probe_flag, 0);
    }
    if (e != hipSuccess)
    {
        set_error("analyzer allocation failed: %s", hipGetErrorString(e));
        if (a->st && a->owns_state)
            (void) hipFree(a->st);
        if (a->mse)
            (void) hipFree(a->mse);
        if (a->pinned)
            (void) hipHostFree(a->pinned);
        delete a;
        return MIQ_ERR_HIP;
    }
    *out = a;
    return MIQ_OK;
}

int miq_analyzer_set_percentile(miq_analyzer* a, float percentile)
{
    MIQ_CHECK_ARG(a != nullptr, "null analyzer");
    MIQ_CHECK_ARG(percentile >= 0.0f && percentile <= 100.0f, "percentile must be in [0, 100] (got %g)",
                  (double) percentile);
    a->percentile = percentile;
    a->queued     = false;
    return MIQ_OK;
}

int miq_analyzer_destroy(miq_analyzer* a)
{
    if (!a)
        return MIQ_OK;
    if (a->owns_state)
        (void) hipFree(a->st);
    if (a->mse)
        (void) hipFree(a->mse);
    entropy_destroy(a->entropy);
    if (a->pinned)
        (void) hipHostFree(a->pinned);
    delete a;
    return MIQ_OK;
}

int miq_analyzer_reset(miq_analyzer* a, void* stream)
{
    MIQ_CHECK_ARG(a != nullptr, "null analyzer");
    if (a->entropy)
    {
        a->stats_updated = false;
        a->queued        = false;
        return entropy_reset(a->entropy, (hipStream_t) stream);
    }
    hipLaunchKernelGGL(reset_state_kernel, dim3(1), dim3(kPdf), 0, (hipStream_t) stream, a->st);
    MIQ_CHECK_LAUNCH();
    a->needs_reset = false;
    a->queued      = false;
    a->stats_updated = false;
    a->range_known   = false;
    a->seq           = 0;
    // a histogram launch queued before this reset may still publish its range: it carries the old generation
    a->generation = (a->generation == INT_MAX) ? 1 : a->generation + 1;
    a->counted_n  = 0;
    return MIQ_OK;
}

int miq_analyzer_update_stats_f32(miq_analyzer* a, const float* data, int64_t n, void* stream)
{
    MIQ_CHECK_ARG(a != nullptr, "null analyzer");
    MIQ_CHECK_ARG(n > 0 && data, "update_stats needs a non-empty tensor");
    hipStream_t s  = (hipStream_t) stream;
    const bool vec = aligned16(data);
    if (a->entropy)
    {
        a->stats_updated = true;
        a->queued        = false;
        return entropy_update(a->entropy, data, n, s);
    }
    if (int rc = ensure_reset(a, s))
        return rc;
    a->stats_updated = true;
    a->queued        = false;
    const int grid    = hist_grid(n);
    const int mm_grid = (int) std::max<int64_t>(
        1, std::min<int64_t>(kMmGrid, (n / 4 + (int64_t) kMmBlock * kMmUnroll - 1) / ((int64_t) kMmBlock * kMmUnroll)));
    if (a->mode == MIQ_QUANTIZATION_TF)
    {
        if (vec)
            hipLaunchKernelGGL(minmax_kernel<true>, dim3(mm_grid), dim3(kMmBlock), 0, s, data, n, a->st, kMinMaxTf, 1u);
        else
            hipLaunchKernelGGL(minmax_kernel<false>, dim3(mm_grid), dim3(kMmBlock), 0, s, data, n, a->st, kMinMaxTf, 1u);
        hipLaunchKernelGGL(minmax_finalize_kernel, dim3(1), dim3(kBlock), 0, s, a->st, mm_grid);
        MIQ_CHECK_LAUNCH();
        return MIQ_OK;
    }
    if (!a->range_known && __atomic_load_n(&a->probe_flag[0], __ATOMIC_ACQUIRE) == a->generation)
    {
        // a histogram launch of this generation has fixed the range and written it into these pinned words
        a->range_known = true;
        memcpy(&a->bucket_f, &a->probe_flag[2], sizeof(float));
        memcpy(&a->pdf_offset_f, &a->probe_flag[3], sizeof(float));
    }
    a->seq += 1;
    if (!a->range_known)
    {
        // The range is fixed by the first batch that is not all zeros.  Whether that has happened is device state:
        // the pass below returns at once when it has, and the host stops queuing it as soon as it sees the words a
        // histogram launch writes into pinned memory when it fixes the range.  Nothing here blocks or copies.
        if (vec)
            hipLaunchKernelGGL(minmax_kernel<true>, dim3(mm_grid), dim3(kMmBlock), 0, s, data, n, a->st, kMinMaxTfe,
                               a->seq);
        else
            hipLaunchKernelGGL(minmax_kernel<false>, dim3(mm_grid), dim3(kMmBlock), 0, s, data, n, a->st, kMinMaxTfe,
                               a->seq);
    }
    const int buf = (int) (a->seq & 1u);
    // at least one workgroup per fold slice (those beyond the data only fold)
    const int hist_groups = std::max(grid, kFoldSlices);
    const dim3 hgrid((unsigned) hist_groups), hblock(kBlock);
    // workgroups [rem, groups) stream one tile fewer than the others (none at all when there are fewer tiles than
    // workgroups): the previous batch is folded by the first kFoldSlices of them
    const int64_t tiles  = (n / 4 + (int64_t) kBlock * kHistUnroll - 1) / ((int64_t) kBlock * kHistUnroll);
    const int fold_first = (int) std::min<int64_t>(tiles % hist_groups, hist_groups - kFoldSlices);
    if (a->range_known)
    {
        if (vec)
            hipLaunchKernelGGL((hist_kernel<true, true>), hgrid, hblock, 0, s, data, n, a->st, buf, a->seq, a->bucket_f,
                               a->pdf_offset_f, mm_grid, a->probe_dev, a->generation, a->counted_n, fold_first);
        else
            hipLaunchKernelGGL((hist_kernel<false, true>), hgrid, hblock, 0, s, data, n, a->st, buf, a->seq, a->bucket_f,
                               a->pdf_offset_f, mm_grid, a->probe_dev, a->generation, a->counted_n, fold_first);
        a->counted_n = n;
    }
    else if (vec)
        hipLaunchKernelGGL((hist_kernel<true, false>), hgrid, hblock, 0, s, data, n, a->st, buf, a->seq, 0.f, 0.f, mm_grid,
                           a->probe_dev, a->generation, (int64_t) 0, fold_first);
    else
        hipLaunchKernelGGL((hist_kernel<false, false>), hgrid, hblock, 0, s, data, n, a->st, buf, a->seq, 0.f, 0.f,
                           mm_grid, a->probe_dev, a->generation, (int64_t) 0, fold_first);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

static int flush_pending(miq_analyzer* a, hipStream_t s)
{
    if (a->mode != MIQ_QUANTIZATION_TF && a->seq != 0)
    {
        hipLaunchKernelGGL(hist_flush_kernel, dim3(kFoldSlices), dim3(kBlock), 0, s, a->st, a->seq);
        MIQ_CHECK_LAUNCH();
        a->counted_n = 0;   // nothing is pending any more: the next launch must not fold on the host's word
    }
    return MIQ_OK;
}

static int finish_read(miq_analyzer* a, hipStream_t s);
static int read_state(miq_analyzer* a, hipStream_t s, size_t bytes = kInspectBytes, bool wait = true)
{
    a->queued = false;   // the staging buffer is about to be overwritten
    if (int rc = ensure_reset(a, s))
        return rc;
    MIQ_CHECK_HIP(hipMemcpyAsync(a->pinned, a->st, bytes, hipMemcpyDeviceToHost, s));
    if (!wait)
        return MIQ_OK;
    return finish_read(a, s);
}

static int finish_read(miq_analyzer* a, hipStream_t s)
{
    MIQ_CHECK_HIP(hipStreamSynchronize(s));
    const DevState* h = static_cast<const DevState*>(a->pinned);
    if (h->initialized)
    {
        a->range_known  = true;
        a->bucket_f     = h->bucket_f;
        a->pdf_offset_f = h->pdf_offset_f;
    }
    return MIQ_OK;
}

// Everything of compute_encoding that can be queued: the pending batch folded, the search launched, the copy of the
// results into the staging buffer requested.  Nothing waits.
static int queue_encoding(miq_analyzer* a, int bw, int use_symmetric, int use_strict_symmetric,
                          int use_unsigned_symmetric, hipStream_t s)
{
    if (a->mode == MIQ_QUANTIZATION_TF)
        return read_state(a, s, kHeadBytes, false);
    if (int rc = flush_pending(a, s))
        return rc;
    if (a->mode == MIQ_QUANTIZATION_PERCENTILE)
        return read_state(a, s, kInspectBytes, false);
    if (a->mode == MIQ_QUANTIZATION_MSE)
    {
        float num_steps = (float) (std::pow(2, bw) - 1);
        if (use_symmetric && use_strict_symmetric)
            num_steps -= 1;
        const MseArgs ma{bw, use_symmetric != 0, use_strict_symmetric != 0, use_unsigned_symmetric != 0,
                         (int) num_steps};
        hipLaunchKernelGGL(mse_prepare_kernel, dim3(1), dim3(kBlock), 0, s, a->st, a->mse);
        MIQ_CHECK_LAUNCH();
        hipLaunchKernelGGL(mse_cost_kernel, dim3(kMseGrid), dim3(kBlock), 0, s, a->mse, ma);
        MIQ_CHECK_LAUNCH();
        hipLaunchKernelGGL(mse_pick_kernel, dim3(1), dim3(64), 0, s, a->st, a->mse, ma);
        MIQ_CHECK_LAUNCH();
        return read_state(a, s, kHeadBytes, false);
    }
    const SearchArgs sa = tfe::make_search_args(bw, use_symmetric, use_strict_symmetric, use_unsigned_symmetric);
    MIQ_CHECK_ARG(sa.n_cand <= kMaxCand, "internal: candidate grid too large");
    hipLaunchKernelGGL(tfe_search_kernel, dim3((sa.n_cand + kBlock / 64 - 1) / (kBlock / 64)), dim3(kBlock), 0, s, a->st,
                       sa);
    MIQ_CHECK_LAUNCH();
    return read_state(a, s, kHeadBytes, false);
}

int miq_analyzer_queue_encoding(miq_analyzer* a, int bw, int use_symmetric, int use_strict_symmetric,
                                int use_unsigned_symmetric, void* stream)
{
    MIQ_CHECK_ARG(a != nullptr, "null argument");
    MIQ_CHECK_ARG(bw >= 1 && bw <= 32, "bitwidth must be in [1, 32] (got %d)", bw);
    if (!a->stats_updated || a->entropy)   // the entropy search runs on the host: nothing to queue ahead
        return MIQ_OK;
    if (int rc = queue_encoding(a, bw, use_symmetric, use_strict_symmetric, use_unsigned_symmetric, (hipStream_t) stream))
        return rc;
    a->queued         = true;
    a->queued_args[0] = bw;
    a->queued_args[1] = use_symmetric != 0;
    a->queued_args[2] = use_strict_symmetric != 0;
    a->queued_args[3] = use_unsigned_symmetric != 0;
    a->queued_stream  = (hipStream_t) stream;
    return MIQ_OK;
}

int miq_analyzer_compute_encoding(miq_analyzer* a, int bw, int use_symmetric, int use_strict_symmetric,
                                  int use_unsigned_symmetric, miq_encoding* out, int* is_valid, void* stream)
{
    MIQ_CHECK_ARG(a && out && is_valid, "null argument");
    MIQ_CHECK_ARG(bw >= 1 && bw <= 32, "bitwidth must be in [1, 32] (got %d)", bw);
    hipStream_t s = (hipStream_t) stream;
    memset(out, 0, sizeof(*out));
    *is_valid = a->stats_updated ? 1 : 0;
    if (!a->stats_updated)
        return MIQ_OK;   // AimetTensorQuantizer::getEncoding returns a default encoding and valid = false
    if (a->entropy)
        return entropy_compute(a->entropy, bw, use_symmetric, use_strict_symmetric, use_unsigned_symmetric, out, s);
    const bool ahead = a->queued && a->queued_stream == s && a->queued_args[0] == bw &&
                       a->queued_args[1] == (use_symmetric != 0) && a->queued_args[2] == (use_strict_symmetric != 0) &&
                       a->queued_args[3] == (use_unsigned_symmetric != 0);
    if (!ahead)
        if (int rc = queue_encoding(a, bw, use_symmetric, use_strict_symmetric, use_unsigned_symmetric, s))
            return rc;
    a->queued = false;
    if (int rc = finish_read(a, s))
        return rc;
    const DevState* h = static_cast<const DevState*>(a->pinned);
    if (a->mode == MIQ_QUANTIZATION_TF)
    {
        // DLQ/src/TfEncodingAnalyzer.cpp:80-101 (MIN_RANGE = 0.01)
        double lo = std::min(0.0, h->acc_min);
        double hi = std::max(0.0, h->acc_max);
        hi        = std::max(hi, lo + 0.01);
        return miq_get_computed_encodings(bw, lo, hi, use_symmetric, use_strict_symmetric, use_unsigned_symmetric, out);
    }
    if (a->mode == MIQ_QUANTIZATION_PERCENTILE)
        return percentile_encoding(h, a->percentile, bw, use_symmetric, use_strict_symmetric, use_unsigned_symmetric,
                                   out);
    out->min    = h->enc_min;
    out->max    = h->enc_max;
    out->delta  = h->enc_delta;
    out->offset = h->enc_offset;
    out->bw     = h->enc_bw;
    a->last_bw  = bw;
    return MIQ_OK;
}

int miq_analyzer_get_stats_histogram(miq_analyzer* a, double* x_left, double* pdf, int* num_buckets, void* stream)
{
    MIQ_CHECK_ARG(a && x_left && pdf && num_buckets, "null argument");
    if (a->mode == MIQ_QUANTIZATION_TF)
    {
        set_error("no histogram is kept by the TF (min/max) analyzer");
        return MIQ_ERR_UNSUPPORTED;
    }
    if (a->entropy)
    {
        // the reference's getStatsHistogram for this analyzer appends to vectors it has already sized
        // (DLQ/src/EntropyEncodingAnalyzer.cpp:54-78) and has no defined result; the counts themselves are read with
        // miq_analyzer_entropy_histogram
        set_error("the entropy analyzer keeps counts over a moving range, not a PDF: use miq_analyzer_entropy_histogram");
        return MIQ_ERR_UNSUPPORTED;
    }
    if (int rc = flush_pending(a, (hipStream_t) stream))
        return rc;
    if (int rc = read_state(a, (hipStream_t) stream))
        return rc;
    const DevState* h = static_cast<const DevState*>(a->pinned);
    *num_buckets      = h->initialized ? kPdf : 0;
    if (h->initialized)
    {
        memcpy(x_left, h->xLeft, sizeof(double) * kPdf);
        memcpy(pdf, h->pdf, sizeof(double) * kPdf);
    }
    return MIQ_OK;
}

int miq_analyzer_entropy_histogram(miq_analyzer* a, double* counts, double* range_min_max, int* initialized,
                                   int* iterations, void* stream)
{
    MIQ_CHECK_ARG(a && counts && range_min_max && initialized && iterations, "null argument");
    MIQ_CHECK_ARG(a->entropy != nullptr, "not an entropy analyzer");
    return entropy_histogram(a->entropy, counts, range_min_max, initialized, iterations, (hipStream_t) stream);
}

int miq_analyzer_last_batch_counts(miq_analyzer* a, uint32_t* counts, void* stream)
{
    MIQ_CHECK_ARG(a && counts, "null argument");
    if (a->entropy)
    {
        set_error("the entropy analyzer does not keep the last batch apart: use miq_analyzer_entropy_histogram");
        return MIQ_ERR_UNSUPPORTED;
    }
    if (int rc = flush_pending(a, (hipStream_t) stream))
        return rc;
    if (int rc = read_state(a, (hipStream_t) stream))
        return rc;
    memcpy(counts, static_cast<const DevState*>(a->pinned)->last_counts, sizeof(uint32_t) * kPdf);
    return MIQ_OK;
}

int miq_analyzer_last_search(miq_analyzer* a, float* deltas, int32_t* offsets, double* costs, int cap, int* count,
                             int* best_index, void* stream)
{
    MIQ_CHECK_ARG(a && deltas && offsets && costs && count && best_index && cap >= 0, "bad argument");
    if (a->entropy || a->mode == MIQ_QUANTIZATION_MSE)
    {
        set_error("only the TF-Enhanced analyzer keeps its candidate list");
        return MIQ_ERR_UNSUPPORTED;
    }
    if (int rc = read_state(a, (hipStream_t) stream))
        return rc;
    const DevState* h = static_cast<const DevState*>(a->pinned);
    // compact to the candidates the reference would have kept, in its order
    int n = 0, best = -1;
    for (int c = 0; c < h->n_cand; ++c)
    {
        if (!h->cand_valid[c])
            continue;
        if (c == h->best_index)
            best = n;
        if (n < cap)
        {
            deltas[n]  = h->cand_delta[c];
            offsets[n] = h->cand_offset[c];
            costs[n]   = h->cand_cost[c];
        }
        ++n;
    }
    *count      = n;
    *best_index = best;
    return MIQ_OK;
}

}   // extern "C"
