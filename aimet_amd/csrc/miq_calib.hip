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
// kernel per batch in steady state (the first batch adds a min/max pass); the workgroup that finishes last folds
// the batch's integer bin counts into the running PDF, so nothing is copied to the host and nothing synchronises
// until an encoding is asked for.  Bin counts are integers, hence independent of the order in which lanes add them.
// The histogram is privatised in LDS: 16 interleaved copies of the 512 bins per workgroup, lane l using copy
// l mod 16, so that even when every sample of a wavefront falls into one bin (post-ReLU data) at most two lanes
// meet on an address.
#include "miq_common.h"
#include "miq_fastmath.h"

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
// workgroups.  8 copies are 16 KB, so 8 workgroups fit a compute unit and 2048 run in a single round: 7.3 us for a 25.7 MB
// batch against 9.3 us with 16 copies / 1024 workgroups.  4 and 2 copies are faster still on spread-out data (6.9 / 6.7 us)
// but collapse when the values share a bucket (constant tensor: 8.8 / 14.0 us against 6.9 us here).
constexpr int kCopies   = 8;
constexpr int kMaxGrid  = 2048;
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
    int minmax_valid;    // the min/max pass of this batch ran (it returns at once when the PDF range is fixed)
    int initialized;     // PDF range fixed (xLeft.size() != 0 in the reference)
    int iterations;
    float bucket_f, pdf_offset_f;
    int n_cand;
    int best_index;
    int enc_bw;
    uint32_t batch_seq[2];   // update-call number whose counts sit in counts[i]; 0 = none pending
    int64_t batch_n[2];      // element count of that batch
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

// relaxed agent-scope loads: used by the workgroup that finishes last to read what the others published
template <typename T>
__device__ __forceinline__ T agent_load(const T* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

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

__device__ void initialize_pdf(DevState* st, float min_val, float max_val)
{
    // DLQ/src/math_functions.cpp:208-241 with signed_vals = true, DTYPE = float
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
    const double bucket = ((double) max_val - (double) min_val) / kPdf;
    for (int i = threadIdx.x; i < kPdf; i += blockDim.x)
    {
        st->xLeft[i] = min_val + i * bucket;
        st->pdf[i]   = 0.0;
    }
    if (threadIdx.x == 0)
    {
        // x_left[1] - x_left[0] and x_left[0], rounded to float, drive the bucket index of every later batch
        const double x0   = min_val + 0 * bucket;
        const double x1   = min_val + 1 * bucket;
        const float bf    = (float) (x1 - x0);
        st->bucket_f      = bf;
        st->pdf_offset_f  = (float) x0 / bf;
        st->iterations    = 0;
        st->initialized   = 1;
    }
}

// Pass 1: every workgroup reduces its share and stores one (min, max) pair -- plain stores, no atomics, because
// same-address device atomics from a thousand workgroups serialise at roughly 15 ns each on this part.
template <bool VEC>
__global__ __launch_bounds__(kBlock) void minmax_kernel(const float* __restrict__ in, int64_t n, DevState* st,
                                                        int mode)
{
    if (mode == kMinMaxTfe && st->initialized)
        return;   // range already fixed: later batches need no min/max pass
    float mn = INFINITY, mx = -INFINITY;
    if (VEC)
    {
        const int64_t nvec   = n / 4;
        const float4* v      = reinterpret_cast<const float4*>(in);
        const int64_t stride = (int64_t) gridDim.x * kBlock * kUnroll;
        for (int64_t base = (int64_t) blockIdx.x * kBlock * kUnroll; base < nvec; base += stride)
        {
            float4 a[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
            {
                const int64_t i = base + u * kBlock + threadIdx.x;
                a[u] = (i < nvec) ? v[i] : make_float4(NAN, NAN, NAN, NAN);   // fminf/fmaxf skip NaN
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
            {
                mn = fminf(fminf(mn, a[u].x), fminf(a[u].y, fminf(a[u].z, a[u].w)));
                mx = fmaxf(fmaxf(mx, a[u].x), fmaxf(a[u].y, fmaxf(a[u].z, a[u].w)));
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
        for (int64_t i = (int64_t) blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t) gridDim.x * kBlock)
        {
            const float a = in[i];
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
        st->partial[blockIdx.x] = make_float2(mn, mx);
        if (blockIdx.x == 0)
            st->minmax_valid = 1;
    }
}

// Pass 2 (one workgroup of kBlock lanes): fold the per-workgroup pairs and apply the analyzer's rule.
__global__ __launch_bounds__(kBlock) void minmax_finalize_kernel(DevState* st, int grid, int mode)
{
    if (!st->minmax_valid)
        return;
    float mn = INFINITY, mx = -INFINITY;
    for (int i = threadIdx.x; i < grid; i += kBlock)
    {
        const float2 p = st->partial[i];
        mn             = fminf(mn, p.x);
        mx             = fmaxf(mx, p.y);
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
    float gmn = smn[0], gmx = smx[0];
    for (int w = 1; w < kBlock / 64; ++w)
    {
        gmn = fminf(gmn, smn[w]);
        gmx = fmaxf(gmx, smx[w]);
    }
    if (threadIdx.x == 0)
    {
        st->minmax_valid  = 0;
        st->stats_updated = 1;
    }
    if (mode == kMinMaxTf)
    {
        if (threadIdx.x == 0)
        {
            // DLQ/src/TfEncodingAnalyzer.cpp:59-71
            const double cmn = (double) gmn, cmx = (double) gmx;
            st->acc_min = (cmn < st->acc_min) ? cmn : st->acc_min;
            st->acc_max = (st->acc_max < cmx) ? cmx : st->acc_max;
        }
        return;
    }
    // TF-Enhanced: DLQ/src/math_functions.cpp:248-262
    if (gmn == 0 && gmx == 0)
        return;   // an all-zero batch cannot fix a range; the PDF stays uninitialised and this batch is not counted
    initialize_pdf(st, gmn, gmx);
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
// Adds one sample to the workgroup's LDS histogram.  Row kPdf is a sink for dropped samples, so the add is
// unconditional (no divergent branch per element).
// `rcp` is the correctly rounded 1 / bucket when the five-operation exact division applies to this bucket width (else 0);
// it then gives the IEEE quotient bit for bit wherever the quotient can decide a bucket (miq_fastmath.h).
__device__ __forceinline__ void hist_add(uint32_t* lds, float x, float bucket, float rcp, float off, int copy)
{
    // DLQ/src/math_functions.cpp:375-382; the range test is done on the rounded float so that NaN and values
    // beyond the int range are dropped, as they are on the reference's CPU path
    const float q  = (rcp != 0.0f && fabsf(x) <= kFastDivMaxDividend) ? div_by_invariant(x, bucket, rcp) : x / bucket;
    const float r  = round_half_away(q - off);   // == roundf
    const bool ok  = (r >= 0.0f && r < (float) kPdf);
    const int row  = ok ? (int) r : kPdf;
    atomicAdd(&lds[row * kCopies + copy], 1u);
}

// Folds the counts of one finished batch into the running PDF (DLQ/src/math_functions.cpp:279-287; the element
// count is an int in the reference) and clears them.  Run by one workgroup.
__device__ void fold_batch(DevState* st, int buf)
{
    const int it     = st->iterations;
    const double cnt = (double) (int) st->batch_n[buf];
    for (int b = threadIdx.x; b < kPdf; b += blockDim.x)
    {
        // all replica loads in flight together, then the clears
        uint32_t t[kReplicas];
#pragma unroll
        for (int r = 0; r < kReplicas; ++r)
            t[r] = st->counts[buf][r][b];
        uint32_t c = 0;
#pragma unroll
        for (int r = 0; r < kReplicas; ++r)
        {
            c += t[r];
            st->counts[buf][r][b] = 0;
        }
        st->last_counts[b] = c;
        const double prob  = (double) c / cnt;
        st->pdf[b]         = (st->pdf[b] * it + prob) / (it + 1);
    }
    __syncthreads();
    if (threadIdx.x == 0)
    {
        st->iterations     = it + 1;
        st->batch_seq[buf] = 0;
    }
}

// One launch per batch.  Workgroups 0 .. gridDim.x-2 stream the tensor into counts[buf]; the extra last workgroup
// meanwhile folds the previous batch (counts[1-buf], if that batch was accumulated) into the PDF and stamps this
// batch as pending, so no second launch and no cross-workgroup hand-shake is needed.  `seq` numbers the update
// calls of this analyzer; a buffer is pending iff its stamp equals the sequence number of the call that filled it.
// With from_args the bucket width and offset arrive as kernel arguments (the host has learnt them); otherwise
// they are read from the device state, which also says whether a range exists at all.
template <bool VEC>
__global__ __launch_bounds__(kBlock) void hist_kernel(const float* __restrict__ in, int64_t n, DevState* st, int buf,
                                                      uint32_t seq, int from_args, float bucket_arg, float off_arg)
{
    // workgroup 0 folds: it is dispatched first and runs beside the data workgroups (as the last one it would start only
    // after a data workgroup had retired and would lengthen the launch by its own duration)
    const bool fold_group = (blockIdx.x == 0);
    const int data_groups = gridDim.x - 1;
    const int group       = (int) blockIdx.x - 1;
    if (fold_group)
    {
        if (st->batch_seq[1 - buf] != 0 && st->batch_seq[1 - buf] == seq - 1)
            fold_batch(st, 1 - buf);
        if (threadIdx.x == 0 && st->initialized)
        {
            st->batch_seq[buf] = seq;
            st->batch_n[buf]   = n;
        }
        return;
    }
    __shared__ uint32_t lds[(kPdf + 1) * kCopies];
    const int64_t nvec   = n / 4;
    const float4* v      = reinterpret_cast<const float4*>(in);
    const int64_t stride = (int64_t) data_groups * kBlock * kUnroll;
    int64_t base         = (int64_t) group * kBlock * kUnroll;
    float4 a[kUnroll];
    // first tile's loads go out before anything else: they overlap the state read and the LDS clear
    if (VEC)
    {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            const int64_t i = base + u * kBlock + threadIdx.x;
            a[u] = (i < nvec) ? v[i] : make_float4(NAN, NAN, NAN, NAN);   // NaN is dropped by hist_add
        }
    }
    float bucket = bucket_arg, off = off_arg;
    if (!from_args)
    {
        if (!st->initialized)
            return;   // only all-zero batches so far: the reference returns without touching the PDF
        bucket = st->bucket_f;
        off    = st->pdf_offset_f;
    }
    const float rcp = fastdiv_divisor_ok(bucket) ? 1.0f / bucket : 0.0f;
    for (int i = threadIdx.x; i < (kPdf + 1) * kCopies; i += kBlock)
        lds[i] = 0;
    __syncthreads();
    const int copy = threadIdx.x & (kCopies - 1);
    if (VEC)
    {
        while (true)
        {
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
            {
                hist_add(lds, a[u].x, bucket, rcp, off, copy);
                hist_add(lds, a[u].y, bucket, rcp, off, copy);
                hist_add(lds, a[u].z, bucket, rcp, off, copy);
                hist_add(lds, a[u].w, bucket, rcp, off, copy);
            }
            base += stride;
            if (base >= nvec)
                break;
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
            {
                const int64_t i = base + u * kBlock + threadIdx.x;
                a[u] = (i < nvec) ? v[i] : make_float4(NAN, NAN, NAN, NAN);
            }
        }
        if (group == 0 && threadIdx.x < (uint32_t) (n - nvec * 4))
            hist_add(lds, in[nvec * 4 + threadIdx.x], bucket, rcp, off, copy);
    }
    else
    {
        for (int64_t i = (int64_t) group * kBlock + threadIdx.x; i < n; i += (int64_t) data_groups * kBlock)
            hist_add(lds, in[i], bucket, rcp, off, copy);
    }
    __syncthreads();
    uint32_t* dst = st->counts[buf][group % kReplicas];
    for (int b = threadIdx.x; b < kPdf; b += kBlock)
    {
        uint32_t s = 0;
#pragma unroll
        for (int c = 0; c < kCopies; ++c)
            s += lds[b * kCopies + c];
        if (s)
            atomicAdd(&dst[b], s);
    }
}

// Folds whichever batch is still pending (at most one).  Queued before anything reads the PDF.
__global__ __launch_bounds__(kBlock) void hist_flush_kernel(DevState* st, uint32_t seq)
{
    for (int buf = 0; buf < 2; ++buf)
    {
        if (st->batch_seq[buf] != 0 && st->batch_seq[buf] == seq)
            fold_batch(st, buf);
        __syncthreads();
    }
}

// ------------------------------------------------------------------------------------------------ SQNR search
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

// One wavefront per candidate.  Lanes evaluate the per-bucket error terms in parallel; the three sums of the
// cost are then accumulated by one lane in bucket order, the order the reference's loops use, so that costs are
// bit-identical to the CPU result and ties between candidates resolve identically.
__global__ __launch_bounds__(kBlock) void tfe_search_kernel(DevState* st, SearchArgs a)
{
    constexpr int kWaves = kBlock / 64;
    const int wave       = threadIdx.x >> 6;
    const int cand       = blockIdx.x * kWaves + wave;   // one wavefront per candidate
    const int lane       = threadIdx.x & 63;
    __shared__ double term_all[kWaves][kPdf];
    __shared__ bool is_last;
    double* term = term_all[wave];

    if (st->initialized && cand < a.n_cand)
    {
        // ---- range of the aggregate stats: DLQ/src/TfEnhancedEncodingAnalyzer.cpp:255-291
        int first = -1, last = -1;
#pragma unroll
        for (int k = 0; k < kPdf / 64; ++k)
        {
            const uint64_t m = __ballot(st->pdf[k * 64 + lane] > 0);
            if (m)
            {
                if (first < 0)
                    first = k * 64 + __builtin_ctzll(m);
                const uint64_t m1 = (k == 0) ? (m & ~1ull) : m;   // the downward scan stops above bucket 0
                if (m1)
                    last = k * 64 + 63 - __builtin_clzll(m1);
            }
        }
        float minVal = (float) st->xLeft[first < 0 ? 0 : first];
        float maxVal = (float) st->xLeft[last < 0 ? kPdf - 1 : last];
        minVal       = std_min(minVal, 0.0f);
        maxVal       = std_max(maxVal, 0.0f);
        maxVal       = std_max(maxVal, minVal + (float) 0.01);

        // ---- this wavefront's candidate
        float delta = 0.f;
        int offset  = 0;
        bool valid  = true;
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

        // ---- cost: DLQ/src/TfEnhancedEncodingAnalyzer.cpp:293-355
        double cost = 0;
        if (valid)
        {
            const float cMin      = delta * (float) offset;
            const float stepSize  = a.step_size_cost;
            const float cMax      = delta * ((float) offset + stepSize);
            const float pdfStart  = (float) st->xLeft[0];
            const double pdfStep  = st->xLeft[1] - st->xLeft[0];
            int minInd            = cvtt_x86(floor((cMin - pdfStart) / pdfStep));
            minInd                = minInd < 0 ? 0 : (minInd > kPdf - 1 ? kPdf - 1 : minInd);
            int maxInd            = cvtt_x86(floor((cMax - pdfStart) / pdfStep));
            maxInd                = maxInd < 0 ? 0 : (maxInd > kPdf - 1 ? kPdf - 1 : maxInd);
            const float minMid    = (float) (pdfStart + (minInd * pdfStep) + pdfStep / 2);
            const float maxMid    = (float) (pdfStart + (maxInd * pdfStep) + pdfStep / 2);
#pragma unroll
            for (int k = 0; k < kPdf / 64; ++k)
            {
                const int i      = k * 64 + lane;
                const double p   = st->pdf[i];
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
            // The three sums are accumulated in ascending bucket order, the order of the reference's loops.  Every
            // lane runs the same chain (uniform bounds, LDS broadcast reads), so no cross-lane traffic is needed.
            const double satBottom = ordered_sum(term, 0, minInd);
            double satTop          = ordered_sum(term, maxInd, kPdf);
            const double quant     = ordered_sum(term, minInd, maxInd);
            if (maxInd < minInd)
            {
                // Only after an index conversion left the int range (cvtt_x86).  The reference's three loops then
                // overlap: buckets [maxInd, minInd) are saturation at the bottom AND at the top, and no bucket is
                // quantization noise.  Redo the top sum with every bucket's distance to the top mid-point.
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int k = 0; k < kPdf / 64; ++k)
                {
                    const int i      = k * 64 + lane;
                    const double mid = pdfStart + i * pdfStep + pdfStep / 2;
                    const double d   = mid - maxMid;
                    term[i]          = st->pdf[i] * (d * d);
                }
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_s_waitcnt(0xc07f);
                satTop = ordered_sum(term, maxInd, kPdf);
            }
            cost = 3.0 * (satBottom + satTop) + quant;
            cost                   = (cost < DBL_MAX) ? cost : DBL_MAX;   // std::min(sqnr, max())
        }
        if (lane == 0)
        {
            st->cand_delta[cand]  = delta;
            st->cand_offset[cand] = offset;
            st->cand_valid[cand]  = valid ? 1 : 0;
            st->cand_cost[cand]   = cost;
        }
    }
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0)
    {
        const uint32_t t = atomicAdd(&st->ticket_search, 1u);
        is_last          = (t == gridDim.x - 1);
    }
    __syncthreads();
    if (!is_last || wave != 0)
        return;
    __threadfence();

    // ---- last wavefront: pick the winner (first strict minimum) and form the encoding
    if (lane == 0)
    {
        st->ticket_search = 0;
        st->n_cand        = st->initialized ? a.n_cand : 0;
    }
    if (!st->initialized)
    {
        if (lane == 0)
        {
            st->best_index = -1;
            if (st->stats_updated)
            {
                // only zeros were seen: DLQ/src/TfEnhancedEncodingAnalyzer.cpp:85-100
                const float ns    = a.step_size_cost;
                double mn = -1, mx = 1;
                const double d = (mx - mn) / (int) ns;
                const double o = floor(mn / d);
                mn             = o * d;
                mx             = mn + (int) ns * d;
                st->enc_min = mn, st->enc_max = mx, st->enc_delta = d, st->enc_offset = o;
                st->enc_bw = a.bw;
            }
            else
            {
                st->enc_min = st->enc_max = st->enc_delta = st->enc_offset = 0;
                st->enc_bw                                                = 0;
            }
        }
        return;
    }
    double best = DBL_MAX;
    int bidx    = 0x7fffffff;
    for (int c = lane; c < a.n_cand; c += 64)
    {
        const double cost = agent_load(&st->cand_cost[c]);
        const int v       = agent_load(&st->cand_valid[c]);
        if (v && cost < best)
        {
            best = cost;
            bidx = c;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        const double ob = __shfl_xor(best, o);
        const int oi    = __shfl_xor(bidx, o);
        if (ob < best || (ob == best && oi < bidx))
        {
            best = ob;
            bidx = oi;
        }
    }
    if (lane == 0)
    {
        float bestDelta = -1;
        int bestOffset  = -1;
        if (bidx != 0x7fffffff && best < DBL_MAX)
        {
            bestDelta  = agent_load(&st->cand_delta[bidx]);
            bestOffset = agent_load(&st->cand_offset[bidx]);
        }
        else
            bidx = -1;
        // DLQ/src/TfEnhancedEncodingAnalyzer.cpp:383-396
        const float bMin = std_max(bestDelta * (float) bestOffset, -FLT_MAX);
        const float bMax = std_min(bestDelta * ((float) bestOffset + a.num_steps_cand), FLT_MAX);
        st->enc_delta    = bestDelta;
        st->enc_offset   = bestOffset;
        st->enc_bw       = a.bw;
        st->enc_min      = bMin;
        st->enc_max      = bMax;
        st->best_index   = bidx;
    }
}

__global__ void reset_state_kernel(DevState* st)
{
    const int i = threadIdx.x;   // launched with kPdf threads
    if (i == 0)
    {
        st->ticket_search = 0;
        st->stats_updated = 0;
        st->minmax_valid  = 0;
        st->acc_min       = DBL_MAX;
        st->acc_max       = -DBL_MAX;
        st->initialized = st->iterations = 0;
        st->bucket_f = st->pdf_offset_f = 0.f;
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

int stream_grid(int64_t n)
{
    int64_t blocks = (n / 4 + (int64_t) kBlock * kUnroll - 1) / ((int64_t) kBlock * kUnroll);
    if (blocks < 1)
        blocks = 1;
    if (blocks > kMaxGrid)
        blocks = kMaxGrid;
    return (int) blocks;
}
}   // namespace
}   // namespace miq

using namespace miq;

struct miq_analyzer
{
    int mode;
    float percentile;    // percentile analyzer only
    int device;
    DevState* st;        // device
    void* pinned;        // host staging (pinned) for read-backs
    bool stats_updated;  // host mirror of _isEncodingValid / _statsUpdated
    bool range_known;    // host knows the PDF range has been fixed, so no further min/max pass is queued
    hipEvent_t probe;    // marks the completion of an asynchronous read of DevState::initialized
    bool probe_pending;
    int* probe_flag;     // pinned host words receiving that read: {initialized, iterations, bucket_f, pdf_offset_f}
    float bucket_f, pdf_offset_f;   // valid once range_known
    uint32_t seq;        // number of TF-Enhanced update calls since the last reset
    int last_bw;
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

// PercentileEncodingAnalyzer<float>::computeEncoding on the PDF read back from the device
// (DLQ/src/PercentileEncodingAnalyzer.cpp:78-198; findOriginalRange: DLQ/src/math_functions.cpp:400-433).
// 512 buckets of host arithmetic, in the reference's types: float range values, double cdf.
static int percentile_encoding(const DevState* h, float percentile, int bw, int sym, int strict, int uns,
                               miq_encoding* out)
{
    float num_steps = (float) (std::pow(2, bw) - 1);
    if (sym && strict)
        num_steps -= 1;
    if (!h->initialized)
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
    float min_val = (float) h->xLeft[0], max_val = (float) h->xLeft[kPdf - 1];
    for (int i = 0; i < kPdf; ++i)
        if (h->pdf[i] > 0)
        {
            min_val = (float) h->xLeft[i];
            break;
        }
    for (int i = kPdf - 1; i > 0; --i)
        if (h->pdf[i] > 0)
        {
            max_val = (float) h->xLeft[i];
            break;
        }
    min_val = std::min(min_val, 0.0f);
    max_val = std::max(max_val, 0.0f);
    max_val = std::max(max_val, min_val + (float) 0.01);
    float a_min = min_val, a_max = max_val;
    if (percentile != 100.0f)
    {
        const float width = (float) (h->xLeft[1] - h->xLeft[0]);
        a_min             = (float) h->xLeft[0];
        a_max             = (float) (h->xLeft[kPdf - 1] + width);
        std::vector<double> cdf(h->pdf, h->pdf + kPdf);
        for (int i = 1; i < kPdf; ++i)
            cdf[i] += cdf[i - 1];
        const float left = 1 - percentile / 100;
        for (int i = 0; i < kPdf; ++i)
            if (cdf[i] >= left)
            {
                a_min = (float) h->xLeft[i];
                break;
            }
        const float right = percentile / 100;
        for (int i = kPdf - 1; i >= 0; --i)
            if (cdf[i] < right && h->xLeft[i] < max_val)
            {
                a_max = (float) (h->xLeft[i] + width);
                break;
            }
        if (a_min == a_max)
            a_max += width;
    }
    a_min = std::min(a_min, 0.0f);
    a_max = std::max(a_max, 0.0f);
    return miq_get_computed_encodings(bw, a_min, a_max, sym, strict, uns, out);
}

int miq_analyzer_create(int quantization_mode, miq_analyzer** out)
{
    MIQ_CHECK_ARG(out != nullptr, "null output handle");
    if (quantization_mode != MIQ_QUANTIZATION_TF && quantization_mode != MIQ_QUANTIZATION_TF_ENHANCED &&
        quantization_mode != MIQ_QUANTIZATION_PERCENTILE)
    {
        set_error("quantization mode %d is not implemented (TF, TF_ENHANCED and PERCENTILE are)", quantization_mode);
        return MIQ_ERR_UNSUPPORTED;
    }
    miq_analyzer* a = new (std::nothrow) miq_analyzer();
    MIQ_CHECK_ARG(a != nullptr, "out of host memory");
    a->mode          = quantization_mode;
    a->percentile    = 100.0f;   // PercentileEncodingAnalyzer.h: the default clips nothing
    a->st            = nullptr;
    a->pinned        = nullptr;
    a->stats_updated = false;
    a->range_known   = false;
    a->probe         = nullptr;
    a->probe_pending = false;
    a->probe_flag    = nullptr;
    a->bucket_f = a->pdf_offset_f = 0.f;
    a->seq           = 0;
    a->last_bw       = 0;
    hipError_t e     = hipGetDevice(&a->device);
    if (e == hipSuccess)
        e = hipMalloc((void**) &a->st, sizeof(DevState));
    if (e == hipSuccess)
        e = hipHostMalloc(&a->pinned, kInspectBytes + 64, hipHostMallocDefault);   // + 4 probe words
    if (e == hipSuccess)
        e = hipEventCreateWithFlags(&a->probe, hipEventDisableTiming);
    if (e != hipSuccess)
    {
        set_error("analyzer allocation failed: %s", hipGetErrorString(e));
        if (a->st)
            (void) hipFree(a->st);
        if (a->pinned)
            (void) hipHostFree(a->pinned);
        delete a;
        return MIQ_ERR_HIP;
    }
    a->probe_flag  = reinterpret_cast<int*>(static_cast<char*>(a->pinned) + kInspectBytes);
    *a->probe_flag = 0;
    hipLaunchKernelGGL(reset_state_kernel, dim3(1), dim3(kPdf), 0, (hipStream_t) nullptr, a->st);
    e = hipStreamSynchronize(nullptr);
    if (e != hipSuccess)
    {
        set_error("analyzer initialisation failed: %s", hipGetErrorString(e));
        (void) hipFree(a->st);
        (void) hipHostFree(a->pinned);
        (void) hipEventDestroy(a->probe);
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
    return MIQ_OK;
}

int miq_analyzer_destroy(miq_analyzer* a)
{
    if (!a)
        return MIQ_OK;
    if (a->probe_pending)
        (void) hipEventSynchronize(a->probe);
    (void) hipEventDestroy(a->probe);
    (void) hipFree(a->st);
    (void) hipHostFree(a->pinned);
    delete a;
    return MIQ_OK;
}

int miq_analyzer_reset(miq_analyzer* a, void* stream)
{
    MIQ_CHECK_ARG(a != nullptr, "null analyzer");
    hipLaunchKernelGGL(reset_state_kernel, dim3(1), dim3(kPdf), 0, (hipStream_t) stream, a->st);
    MIQ_CHECK_LAUNCH();
    a->stats_updated = false;
    a->range_known   = false;
    a->seq           = 0;
    if (a->probe_pending)
    {
        // a read of the pre-reset state may still be in flight; its answer must not be believed afterwards
        MIQ_CHECK_HIP(hipEventSynchronize(a->probe));
        a->probe_pending = false;
    }
    *a->probe_flag = 0;
    return MIQ_OK;
}

int miq_analyzer_update_stats_f32(miq_analyzer* a, const float* data, int64_t n, void* stream)
{
    MIQ_CHECK_ARG(a != nullptr, "null analyzer");
    MIQ_CHECK_ARG(n > 0 && data, "update_stats needs a non-empty tensor");
    hipStream_t s  = (hipStream_t) stream;
    const bool vec = aligned16(data);
    a->stats_updated = true;
    const int grid = stream_grid(n);
    if (a->mode == MIQ_QUANTIZATION_TF)
    {
        if (vec)
            hipLaunchKernelGGL(minmax_kernel<true>, dim3(grid), dim3(kBlock), 0, s, data, n, a->st, kMinMaxTf);
        else
            hipLaunchKernelGGL(minmax_kernel<false>, dim3(grid), dim3(kBlock), 0, s, data, n, a->st, kMinMaxTf);
        hipLaunchKernelGGL(minmax_finalize_kernel, dim3(1), dim3(kBlock), 0, s, a->st, grid, kMinMaxTf);
        MIQ_CHECK_LAUNCH();
        return MIQ_OK;
    }
    if (!a->range_known && a->probe_pending && hipEventQuery(a->probe) == hipSuccess)
    {
        a->probe_pending = false;
        if (a->probe_flag[0] != 0)
        {
            a->range_known = true;
            memcpy(&a->bucket_f, &a->probe_flag[2], sizeof(float));
            memcpy(&a->pdf_offset_f, &a->probe_flag[3], sizeof(float));
        }
    }
    if (!a->range_known)
    {
        // The range is fixed by the first batch that is not all zeros.  Whether that has happened is device state;
        // the pass below returns at once when it has, and the host stops queuing it once an asynchronous read of
        // that flag (queued after each batch until it answers yes) has landed.  Nothing here blocks.
        if (vec)
            hipLaunchKernelGGL(minmax_kernel<true>, dim3(grid), dim3(kBlock), 0, s, data, n, a->st, kMinMaxTfe);
        else
            hipLaunchKernelGGL(minmax_kernel<false>, dim3(grid), dim3(kBlock), 0, s, data, n, a->st, kMinMaxTfe);
        hipLaunchKernelGGL(minmax_finalize_kernel, dim3(1), dim3(kBlock), 0, s, a->st, grid, kMinMaxTfe);
    }
    a->seq += 1;
    const int buf       = (int) (a->seq & 1u);
    const int from_args = a->range_known ? 1 : 0;
    if (vec)
        hipLaunchKernelGGL(hist_kernel<true>, dim3(grid + 1), dim3(kBlock), 0, s, data, n, a->st, buf, a->seq, from_args,
                           a->bucket_f, a->pdf_offset_f);
    else
        hipLaunchKernelGGL(hist_kernel<false>, dim3(grid + 1), dim3(kBlock), 0, s, data, n, a->st, buf, a->seq,
                           from_args, a->bucket_f, a->pdf_offset_f);
    MIQ_CHECK_LAUNCH();
    if (!a->range_known && !a->probe_pending)
    {
        // {initialized, iterations, bucket_f, pdf_offset_f} are adjacent in DevState
        MIQ_CHECK_HIP(hipMemcpyAsync(a->probe_flag, &a->st->initialized, 4 * sizeof(int), hipMemcpyDeviceToHost, s));
        MIQ_CHECK_HIP(hipEventRecord(a->probe, s));
        a->probe_pending = true;
    }
    return MIQ_OK;
}

static int flush_pending(miq_analyzer* a, hipStream_t s)
{
    if (a->mode != MIQ_QUANTIZATION_TF && a->seq != 0)
    {
        hipLaunchKernelGGL(hist_flush_kernel, dim3(1), dim3(kBlock), 0, s, a->st, a->seq);
        MIQ_CHECK_LAUNCH();
    }
    return MIQ_OK;
}

static int read_state(miq_analyzer* a, hipStream_t s, size_t bytes = kInspectBytes)
{
    MIQ_CHECK_HIP(hipMemcpyAsync(a->pinned, a->st, bytes, hipMemcpyDeviceToHost, s));
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
    if (a->mode == MIQ_QUANTIZATION_TF)
    {
        if (int rc = read_state(a, s, kHeadBytes))
            return rc;
        const DevState* h = static_cast<const DevState*>(a->pinned);
        // DLQ/src/TfEncodingAnalyzer.cpp:80-101 (MIN_RANGE = 0.01)
        double lo = std::min(0.0, h->acc_min);
        double hi = std::max(0.0, h->acc_max);
        hi        = std::max(hi, lo + 0.01);
        return miq_get_computed_encodings(bw, lo, hi, use_symmetric, use_strict_symmetric, use_unsigned_symmetric, out);
    }
    if (a->mode == MIQ_QUANTIZATION_PERCENTILE)
    {
        if (int rc = flush_pending(a, s))
            return rc;
        if (int rc = read_state(a, s))
            return rc;
        return percentile_encoding(static_cast<const DevState*>(a->pinned), a->percentile, bw, use_symmetric,
                                   use_strict_symmetric, use_unsigned_symmetric, out);
    }
    SearchArgs sa{};
    sa.bw             = bw;
    sa.sym            = use_symmetric ? 1 : 0;
    sa.strict         = use_strict_symmetric ? 1 : 0;
    sa.uns            = use_unsigned_symmetric ? 1 : 0;
    sa.step_size_cost = (float) (std::pow(2, bw) - 1);
    sa.num_steps_cand = sa.step_size_cost;
    if (sa.sym && sa.strict)
        sa.num_steps_cand -= 1;
    if (sa.sym)
    {
        // the delta factor advances by adding the double 0.01 to a float; how many steps fit below 1.01 is decided
        // by that float arithmetic (DLQ/src/TfEnhancedEncodingAnalyzer.cpp:248)
        int cnt = 0;
        for (float f = (float) (1.0 / 100); (double) f <= 1 + 1.0 / 100; f = (float) ((double) f + 1.0 / 100))
            ++cnt;
        sa.n_delta = cnt;
        sa.n_cand  = cnt;
    }
    else
    {
        int cnt = 0;
        for (float f = (float) (1.0 / 16); (double) f <= 1 + 1.0 / 16; f = (float) ((double) f + 1.0 / 16))
            ++cnt;
        sa.n_delta = cnt;
        sa.n_cand  = cnt * 21 + 1;
    }
    MIQ_CHECK_ARG(sa.n_cand <= kMaxCand, "internal: candidate grid too large");
    if (int rc = flush_pending(a, s))
        return rc;
    hipLaunchKernelGGL(tfe_search_kernel, dim3((sa.n_cand + kBlock / 64 - 1) / (kBlock / 64)), dim3(kBlock), 0, s, a->st,
                       sa);
    MIQ_CHECK_LAUNCH();
    if (int rc = read_state(a, s, kHeadBytes))
        return rc;
    const DevState* h = static_cast<const DevState*>(a->pinned);
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

int miq_analyzer_last_batch_counts(miq_analyzer* a, uint32_t* counts, void* stream)
{
    MIQ_CHECK_ARG(a && counts, "null argument");
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
