// v2 histogram observer + SQNR encoding search on gfx950.
//
// Reference (EA = TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/encoding_analyzer.py):
//   _HistogramObserver.collect_stats / _handle_inputs / _create_bin_edges      EA:131-205
//   _HistogramObserver.merge_stats / _get_bin_num                              EA:207-262
//   SqnrEncodingAnalyzer._pick_test_candidates*, _clamp_delta_offset_values    EA:594-660
//   SqnrEncodingAnalyzer._estimate_clip_and_quant_noise, _select_best_candidates, compute_encodings_from_stats
//                                                                              EA:566-592, 662-725
// The reference's arithmetic is float32 torch ops (torch.histc for the binning); every float32 operation below is the
// same IEEE operation in the same order, so bin counts, candidate grids and per-bin noise terms are identical.  The
// only deliberate difference: the per-candidate sum over the bins is accumulated in double (torch.sum's float32
// blocked summation order is not reproduced), so scores agree to rounding (about 1e-6 relative), not bit for bit.
//
// An update of running statistics reads the batch once: one launch finds the batch's finite min / max and, in the same
// pass, bins the batch over the range the statistics already have; a second launch adds those counts to the running
// histogram if that range still holds (after the first batches it nearly always does: eight of its workgroups do the
// adding, the others leave at once), and otherwise bins the batch again over the new range and re-bins the running
// histogram.  The first batch, and updates that also want the batch's own
// histogram, read the batch twice (finite min/max, then one binning pass for both histograms).  The reference reads a
// batch about eight times (isfinite x4, histc x2, comparisons x4) and re-bins with per-element Python loops.
#include "miq_agent.h"
#include "miq_common.h"
#include "miq_fastmath.h"

#include <cmath>

namespace miq
{
namespace
{
constexpr int kMaxBins    = 4096;
constexpr int kHistBlock  = 256;
constexpr int kMaxReplicas = 32;   // global copies of a histogram's counts that the workgroups of one update add into
// Speculative update (measured on a 25.7 MB per-tensor batch, 2048 bins): 8 replicas (4 / 16 / 32: +1 / +2 / +7 us on
// the launch that adds them up), rows of 64 K elements or more go to workgroups of 1024 threads with 32 K elements each
// (8 K / 16 K / 50 K: +2.5 / +0.8 / +4 us), two 16-byte loads of a lane in flight (4 / 8: +0.8 / +1.1 us).
constexpr int kSpecReplicas     = 8;
constexpr int kSpecLoads        = 2;
constexpr int kSpecCopies       = 4;
constexpr int kCompactFrom      = 64;   // histograms per search from which empty bins are skipped
constexpr int64_t kSpecElems    = 32768;
constexpr int64_t kSpecWideFrom = 65536;
constexpr float kMinScale = 1.1920928955078125e-07f;   // torch.finfo(torch.float32).eps (EA:322)

typedef float v4f __attribute__((ext_vector_type(4)));

// Ticket counters of one launch: `last[h]` and, for grids of more than 32 workgroups per histogram, one counter per
// group of 32 workgroups, 128 bytes apart (tickets drawn from one address are served one after the other, about 25 ns
// each: 1024 workgroups that finish together would wait 25 us for theirs).
struct Tickets
{
    uint32_t* last;     // [H]
    uint32_t* group;    // [H][ceil(blocks / 32)][32 words], null for grids of up to 32 workgroups per histogram
};
constexpr int kTicketGroup  = 32;
constexpr int kTicketStride = 32;   // words

// Ticket of a workgroup that has finished its share of histogram h; true for the one that finishes last, which has
// then passed last_ticket_acquire() and reads what the others published (device-scope atomic adds and agent_store()s)
// with agent_load() -- the pattern and its invariant are stated in miq_agent.h.  All counters are back at zero
// afterwards.
__device__ __forceinline__ bool last_ticket(const Tickets& t, int h, int* s_flag)
{
    publications_acknowledged();
    __syncthreads();
    if (threadIdx.x == 0)
    {
        const uint32_t blocks = gridDim.x;
        bool last;
        if (t.group)
        {
            const uint32_t groups = (blocks + kTicketGroup - 1) / kTicketGroup;
            const uint32_t g      = blockIdx.x / kTicketGroup;
            const uint32_t size   = min((uint32_t) kTicketGroup, blocks - g * kTicketGroup);
            uint32_t* mine        = t.group + ((int64_t) h * groups + g) * kTicketStride;
            last = __hip_atomic_fetch_add(mine, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == size - 1;
            if (last)
            {
                agent_store(mine, 0u);
                last = __hip_atomic_fetch_add(&t.last[h], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == groups - 1;
            }
        }
        else
            last = __hip_atomic_fetch_add(&t.last[h], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == blocks - 1;
        if (last)
            agent_store(&t.last[h], 0u);
        *s_flag = last;
    }
    __syncthreads();
    const bool last = *s_flag != 0;
    if (last)
        last_ticket_acquire();
    return last;
}

// The last workgroup's reads are agent-scope loads that travel to the device's point of coherence (1-2 us each way):
// a whole batch of them is issued before the first use.

// Sum over the replicas of the counters at `slot` ([replica][slot_stride] words, num_bins of them per replica), which
// are left cleared, together with the counters `also_clear` words further on when that is not 0.  out(i, total) is
// called once per bin.  Up to 64 loads per lane are in flight at a time.
template <int BLOCK, typename Out>
__device__ void consume_counts(uint32_t* __restrict__ slot, int slot_stride, int replicas, int num_bins, int also_clear,
                               Out out)
{
    constexpr int kBinsAtOnce = BLOCK >= 1024 ? 2 : 8;
    for (int i0 = 0; i0 < num_bins; i0 += kBinsAtOnce * BLOCK)
    {
        uint32_t total[kBinsAtOnce];
#pragma unroll
        for (int j = 0; j < kBinsAtOnce; ++j)
            total[j] = 0;
        for (int k0 = 0; k0 < replicas; k0 += 8)
        {
            uint32_t t[8][kBinsAtOnce];
#pragma unroll
            for (int k = 0; k < 8; ++k)
#pragma unroll
                for (int j = 0; j < kBinsAtOnce; ++j)
                {
                    const int i = i0 + j * BLOCK + threadIdx.x;
                    t[k][j]     = (k0 + k < replicas && i < num_bins)
                                      ? agent_load(&slot[(int64_t) (k0 + k) * slot_stride + i])
                                      : 0u;
                }
#pragma unroll
            for (int k = 0; k < 8; ++k)
#pragma unroll
                for (int j = 0; j < kBinsAtOnce; ++j)
                    total[j] += t[k][j];
        }
        for (int k = 0; k < replicas; ++k)
#pragma unroll
            for (int j = 0; j < kBinsAtOnce; ++j)
            {
                const int i = i0 + j * BLOCK + threadIdx.x;
                if (i < num_bins)
                {
                    agent_store(&slot[(int64_t) k * slot_stride + i], 0u);
                    if (also_clear)
                        agent_store(&slot[(int64_t) k * slot_stride + also_clear + i], 0u);
                }
            }
#pragma unroll
        for (int j = 0; j < kBinsAtOnce; ++j)
        {
            const int i = i0 + j * BLOCK + threadIdx.x;
            if (i < num_bins)
                out(i, total[j]);
        }
    }
}

// ---- finite min / max per row --------------------------------------------------------------------------------
// partial[(h * blocks + b) * 2 + {0,1}]
__global__ __launch_bounds__(kHistBlock) void finite_minmax_kernel(const float* __restrict__ x, int64_t n_per_hist,
                                                                   float* __restrict__ partial,
                                                                   uint32_t* __restrict__ sums, int sums_per_hist,
                                                                   int vec)
{
    const int h = blockIdx.y;
    // this launch also clears the count replicas that the binning kernel of the same update accumulates into
    for (int i = blockIdx.x * kHistBlock + threadIdx.x; i < sums_per_hist; i += gridDim.x * kHistBlock)
        sums[(int64_t) h * sums_per_hist + i] = 0;
    const float* row = x + (int64_t) h * n_per_hist;
    float lo = INFINITY, hi = -INFINITY;
    auto take = [&](float v) {
        if (fabsf(v) < INFINITY)   // false for NaN and +-inf
        {
            lo = fminf(lo, v);
            hi = fmaxf(hi, v);
        }
    };
    if (vec)
    {
        // 16-byte loads, four in flight per lane
        const v4f* rv       = reinterpret_cast<const v4f*>(row);
        const int64_t nvec  = n_per_hist / 4;
        const int64_t stride = (int64_t) gridDim.x * kHistBlock * 4;
        for (int64_t base = (int64_t) blockIdx.x * kHistBlock * 4; base < nvec; base += stride)
        {
            v4f a[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                const int64_t i = base + u * kHistBlock + threadIdx.x;
                a[u]            = i < nvec ? __builtin_nontemporal_load(rv + i) : (v4f) {NAN, NAN, NAN, NAN};
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                take(a[u][0]);
                take(a[u][1]);
                take(a[u][2]);
                take(a[u][3]);
            }
        }
    }
    else
    {
        for (int64_t i = (int64_t) blockIdx.x * kHistBlock + threadIdx.x; i < n_per_hist;
             i += (int64_t) gridDim.x * kHistBlock)
            take(row[i]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        lo = fminf(lo, __shfl_xor(lo, o));
        hi = fmaxf(hi, __shfl_xor(hi, o));
    }
    __shared__ float s[2][kHistBlock / 64];
    if ((threadIdx.x & 63) == 0)
    {
        s[0][threadIdx.x >> 6] = lo;
        s[1][threadIdx.x >> 6] = hi;
    }
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int k = 1; k < kHistBlock / 64; ++k)
        {
            lo = fminf(lo, s[0][k]);
            hi = fmaxf(hi, s[1][k]);
        }
        float* p = partial + ((int64_t) h * gridDim.x + blockIdx.x) * 2;
        p[0]     = lo;
        p[1]     = hi;
    }
}

// Binning ranges of one update, per histogram (device resident so that nothing waits for the host).
struct Ranges
{
    float b_lo, b_hi;   // batch range = bin_edges[0], bin_edges[-1] of the batch's own histogram
    float m_lo, m_hi;   // range torch.histc uses for the merged histogram
    float new_min, new_max;   // merged (min, max) statistics
    float old_min, old_max;   // statistics before this update
    float batch_min, batch_max;   // finite (min, max) of the batch
    int   rebin;        // 1: the running histogram has to be re-binned into the merged range
    int   pad;
};

// The scalar work of _create_bin_edges and of merge_stats' range logic for one histogram, from the batch's finite
// (min, max); `ok` is false when the batch held no finite value (the reference raises ValueError there).
__device__ Ranges compute_ranges(float lo, float hi, int num_bins, int has_stats, const float* __restrict__ state_minmax,
                                 int h, bool& ok)
{
    ok = lo <= hi;
    if (!ok)
    {
        lo = 0.f;
        hi = 0.f;
    }
    Ranges r;
    r.batch_min = lo;
    r.batch_max = hi;
    // _create_bin_edges: equal min and max are widened by 0.5 each way; edges = arange(0, bins + 1) * step + min
    float e_lo = lo, e_hi = hi;
    if (e_hi == e_lo)
    {
        e_lo = e_lo - 0.5f;
        e_hi = e_hi + 0.5f;
    }
    const float step = (e_hi - e_lo) / (float) num_bins;
    r.b_lo           = 0.0f * step + e_lo;
    r.b_hi           = (float) num_bins * step + e_lo;
    r.old_min = r.old_max = 0.f;
    r.rebin               = 0;
    if (!has_stats)
    {
        r.new_min = lo;
        r.new_max = hi;
        r.m_lo    = r.b_lo;
        r.m_hi    = r.b_hi;
    }
    else
    {
        r.old_min = state_minmax[2 * h];
        r.old_max = state_minmax[2 * h + 1];
        r.new_min = fminf(lo, r.old_min);
        r.new_max = fmaxf(hi, r.old_max);
        r.rebin   = !(r.new_min == r.old_min && r.new_max == r.old_max);
        // torch.histc(min, max): equal bounds are widened by one each way
        r.m_lo = r.new_min;
        r.m_hi = r.new_max;
        if (r.m_lo == r.m_hi)
        {
            r.m_lo -= 1.0f;
            r.m_hi += 1.0f;
        }
    }
    return r;
}

// torch.histc's bin of x in [lo, hi] followed by the observer's rule for what lies outside: miq_fastmath.h
typedef HistcBinner Binner;

// grid (blocks, H).  Each workgroup first derives the binning ranges of histogram h from the (min, max) partials of the
// previous launch (every workgroup repeats this small reduction: cheaper than a launch of its own), then bins its
// share of row h into LDS -- the batch's own range and / or the merged range, in one pass over the data -- and adds
// its non-zero counts to one of `replicas` global copies (workgroup b -> copy b % replicas, so at most
// blocks / replicas atomics ever meet on one address; same-address device atomics cost about 15 ns each here).
// LDS: [kinds][num_bins][copies] uint32, copy = lane % copies (lanes of a wavefront that hit the same bin spread out).
// global layout: [h][replica][kinds][num_bins] uint32, cleared by the min/max kernel of the same update
__device__ void rebin_running_histogram(float* __restrict__ upd, const float* __restrict__ sh, const Ranges& r, int num_bins);

__global__ __launch_bounds__(kHistBlock) void hist_kernel(const float* __restrict__ x, int64_t n_per_hist, int num_bins,
                                                          int has_stats, int count_batch, int count_merged,
                                                          int copies, const float* __restrict__ mm_partial,
                                                          const float* __restrict__ state_minmax,
                                                          Ranges* __restrict__ ranges, float* __restrict__ batch_minmax,
                                                          int* __restrict__ bad_flag, uint32_t* __restrict__ partial,
                                                          int replicas, int vec)
{
    extern __shared__ uint32_t lds[];
    __shared__ float s_mm[2][kHistBlock / 64];
    const int h = blockIdx.y;
    const int kinds = count_batch + count_merged;
    // the first tile's loads go out before anything else: they are in flight while the ranges are derived
    const float* row     = x + (int64_t) h * n_per_hist;
    const v4f* rv        = reinterpret_cast<const v4f*>(row);
    const int64_t nvec   = n_per_hist / 4;
    const int64_t stride = (int64_t) gridDim.x * kHistBlock * 2;
    int64_t base         = (int64_t) blockIdx.x * kHistBlock * 2;
    v4f a[2];
    if (vec)
    {
#pragma unroll
        for (int u = 0; u < 2; ++u)
        {
            const int64_t i = base + u * kHistBlock + threadIdx.x;
            a[u]            = i < nvec ? __builtin_nontemporal_load(rv + i) : (v4f) {NAN, NAN, NAN, NAN};
        }
    }
    for (int i = threadIdx.x; i < kinds * num_bins * copies; i += kHistBlock)
        lds[i] = 0;
    float lo = INFINITY, hi = -INFINITY;
    for (int b = threadIdx.x; b < (int) gridDim.x; b += kHistBlock)
    {
        lo = fminf(lo, mm_partial[((int64_t) h * gridDim.x + b) * 2]);
        hi = fmaxf(hi, mm_partial[((int64_t) h * gridDim.x + b) * 2 + 1]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        lo = fminf(lo, __shfl_xor(lo, o));
        hi = fmaxf(hi, __shfl_xor(hi, o));
    }
    if ((threadIdx.x & 63) == 0)
    {
        s_mm[0][threadIdx.x >> 6] = lo;
        s_mm[1][threadIdx.x >> 6] = hi;
    }
    __syncthreads();
    for (int k = 0; k < kHistBlock / 64; ++k)
    {
        lo = fminf(lo, s_mm[0][k]);
        hi = fmaxf(hi, s_mm[1][k]);
    }
    bool ok;
    const Ranges r = compute_ranges(lo, hi, num_bins, has_stats, state_minmax, h, ok);
    if (blockIdx.x == 0 && threadIdx.x == 0)
    {
        ranges[h] = r;
        if (batch_minmax)
        {
            batch_minmax[2 * h]     = r.batch_min;
            batch_minmax[2 * h + 1] = r.batch_max;
        }
        if (!ok)
            atomicOr(bad_flag, 1);
    }
    Binner bb, mb;
    bb.init(r.b_lo, r.b_hi, num_bins);
    mb.init(r.m_lo, r.m_hi, num_bins);
    const int copy = threadIdx.x & (copies - 1);
    uint32_t* lb   = lds + copy;                                        // batch-range counts
    uint32_t* lm   = lds + (count_batch ? num_bins * copies : 0) + copy;   // merged-range counts
    auto count = [&](float v) {
        if (v != v)
            return;
        if (count_batch)
            atomicAdd(&lb[bb.bin(v) * copies], 1u);
        if (count_merged)
            atomicAdd(&lm[mb.bin(v) * copies], 1u);
    };
    if (vec)
    {
        while (base < nvec)
        {
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                count(a[u][0]);
                count(a[u][1]);
                count(a[u][2]);
                count(a[u][3]);
            }
            base += stride;
            if (base >= nvec)
                break;
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                const int64_t i = base + u * kHistBlock + threadIdx.x;
                a[u]            = i < nvec ? __builtin_nontemporal_load(rv + i) : (v4f) {NAN, NAN, NAN, NAN};
            }
        }
    }
    else
    {
        for (int64_t i = (int64_t) blockIdx.x * kHistBlock + threadIdx.x; i < n_per_hist;
             i += (int64_t) gridDim.x * kHistBlock)
            count(row[i]);
    }
    __syncthreads();
    uint32_t* dst = partial + ((int64_t) h * replicas + blockIdx.x % replicas) * kinds * num_bins;
    for (int i = threadIdx.x; i < kinds * num_bins; i += kHistBlock)
    {
        uint32_t sum = 0;
        for (int c = 0; c < copies; ++c)
            sum += lds[i * copies + c];
        if (sum)
            atomicAdd(&dst[i], sum);
    }
}

// merge_stats' re-binning of the running histogram `sh` (range old_min .. old_max) into upd (new_min .. new_max), by one
// workgroup (EA:222-251).  Ends with a barrier: upd is complete on return.
__device__ void rebin_running_histogram(float* __restrict__ upd, const float* __restrict__ sh, const Ranges& r, int num_bins)
{
    for (int i = threadIdx.x; i < num_bins; i += kHistBlock)
        upd[i] = 0.f;
    __syncthreads();
    const float nbf            = (float) num_bins;
    const float dest_bin_width = (r.new_max - r.new_min) / nbf;
    const float src_bin_width  = (r.old_max - r.old_min) / nbf;
    for (int i = threadIdx.x; i < num_bins; i += kHistBlock)
    {
        const float cur           = sh[i];
        const float src_bin_start = r.old_min + src_bin_width * (float) i;
        int dest                  = (int) ((src_bin_start - r.new_min) / dest_bin_width);
        dest                      = dest < num_bins - 1 ? dest : num_bins - 1;
        const float dest_bin_end  = r.new_min + dest_bin_width * (float) (dest + 1);
        const float split         = rintf(((dest_bin_end - src_bin_start) / src_bin_width) * cur);
        const float first         = fminf(split, cur);
        // counts are integer valued, so the order of these additions does not change the sums
        atomicAdd(&upd[dest], first);
        if (first < cur)
        {
            int other = (int) (((src_bin_start + dest_bin_width) - r.new_min) / dest_bin_width);
            other     = other < num_bins - 1 ? other : num_bins - 1;
            atomicAdd(&upd[other], cur - first);
        }
    }
    __syncthreads();
}

// ---- one workgroup per histogram ------------------------------------------------------------------------------
// grid (H), 256 threads.  When a row goes to a single workgroup (many histograms, or short rows: the weight of a layer
// with one histogram per output channel) the whole update is one launch and touches no workspace: the workgroup finds
// the row's finite min / max, derives the ranges, bins the row over the merged range into LDS, re-bins the running
// histogram if the range grew and writes the new running histogram.  Rows of up to 6144 elements stay in registers
// between the two passes; longer ones are read again (from the L2).  Serves the first batch (has_stats = 0) as well.
// BATCH: the batch's own histogram (over the batch's range) is written as well; with running statistics that is a
// second LDS histogram, counted in the same pass.
constexpr int kRowKeep    = 6;      // 16-byte groups a lane keeps
constexpr int kRowBinsMax = 2048;   // 16 KiB of counts + 8 KiB for re-binning per workgroup: six of them fit a compute unit
template <bool BATCH>
__global__ __launch_bounds__(kHistBlock) void row_update_kernel(const float* __restrict__ x, int64_t n_per_hist,
                                                                int num_bins, int has_stats,
                                                                float* __restrict__ state_hist,
                                                                float* __restrict__ state_minmax,
                                                                float* __restrict__ batch_hist,
                                                                float* __restrict__ batch_minmax,
                                                                int* __restrict__ bad_flag, int vec)
{
    // [kinds][num_bins][copies] words: 16 KiB at 2048 bins.  The workgroup's life is a chain of round trips, so what
    // counts is how many of them a compute unit holds: with twice the copies (three workgroups per unit instead of six)
    // the launch over [11008, 4096] took 94 us instead of 61.
    constexpr int kRowCopies = BATCH ? 1 : 2;
    extern __shared__ uint32_t lds[];
    __shared__ float upd[kRowBinsMax];
    __shared__ float s_mm[2][kHistBlock / 64];
    const int h        = blockIdx.x;
    const float* row   = x + (int64_t) h * n_per_hist;
    const v4f* rv      = reinterpret_cast<const v4f*>(row);
    const int64_t nvec = n_per_hist / 4;
    const bool kept    = vec && nvec <= (int64_t) kRowKeep * kHistBlock;
    v4f keep[kRowKeep];
    float lo = INFINITY, hi = -INFINITY;
    auto look = [&](float v) {
        if (fabsf(v) < INFINITY)   // false for NaN and +-inf
        {
            lo = fminf(lo, v);
            hi = fmaxf(hi, v);
        }
    };
    if (kept)
    {
#pragma unroll
        for (int u = 0; u < kRowKeep; ++u)
        {
            const int64_t i = u * kHistBlock + threadIdx.x;
            keep[u]         = i < nvec ? __builtin_nontemporal_load(rv + i) : (v4f) {NAN, NAN, NAN, NAN};
        }
    }
    // the running statistics are requested with the row: asked for where they are used, the range and the running
    // counts are two more round trips in a workgroup whose whole life is a handful of them
    float* sh = state_hist + (int64_t) h * num_bins;
    constexpr int kBinsPerLane = kRowBinsMax / kHistBlock;
    float old_mm[2]            = {0.f, 0.f};
    float old_count[kBinsPerLane];
    if (has_stats)
    {
        old_mm[0] = state_minmax[2 * h];
        old_mm[1] = state_minmax[2 * h + 1];
#pragma unroll
        for (int k = 0; k < kBinsPerLane; ++k)
        {
            const int i  = k * kHistBlock + threadIdx.x;
            old_count[k] = i < num_bins ? sh[i] : 0.f;
        }
    }
    const bool two = BATCH && has_stats;   // two histograms: batch range and merged range
    for (int i = threadIdx.x; i < (two ? 2 : 1) * num_bins * kRowCopies; i += kHistBlock)
        lds[i] = 0;
    if (kept)
    {
#pragma unroll
        for (int u = 0; u < kRowKeep; ++u)
        {
            look(keep[u][0]);
            look(keep[u][1]);
            look(keep[u][2]);
            look(keep[u][3]);
        }
    }
    else if (vec)
    {
        for (int64_t i = threadIdx.x; i < nvec; i += kHistBlock)
        {
            const v4f a = rv[i];
            look(a[0]);
            look(a[1]);
            look(a[2]);
            look(a[3]);
        }
    }
    else
    {
        for (int64_t i = threadIdx.x; i < n_per_hist; i += kHistBlock)
            look(row[i]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        lo = fminf(lo, __shfl_xor(lo, o));
        hi = fmaxf(hi, __shfl_xor(hi, o));
    }
    if ((threadIdx.x & 63) == 0)
    {
        s_mm[0][threadIdx.x >> 6] = lo;
        s_mm[1][threadIdx.x >> 6] = hi;
    }
    __syncthreads();   // also: the LDS histogram is clear
    for (int k = 0; k < kHistBlock / 64; ++k)
    {
        lo = fminf(lo, s_mm[0][k]);
        hi = fmaxf(hi, s_mm[1][k]);
    }
    bool ok;
    const Ranges r = compute_ranges(lo, hi, num_bins, has_stats, old_mm, 0, ok);
    if (threadIdx.x == 0)
    {
        if (batch_minmax)
        {
            batch_minmax[2 * h]     = r.batch_min;
            batch_minmax[2 * h + 1] = r.batch_max;
        }
        if (!ok)
            atomicOr(bad_flag, 1);
    }
    Binner mb, bb;
    mb.init(r.m_lo, r.m_hi, num_bins);
    bb.init(r.b_lo, r.b_hi, num_bins);
    uint32_t* lm = lds + (threadIdx.x & (kRowCopies - 1));   // merged range (= batch range without statistics)
    uint32_t* lb = lm + num_bins * kRowCopies;               // batch range, when both are counted
    auto count = [&](float v) {
        if (v == v)
        {
            atomicAdd(&lm[mb.bin(v) * kRowCopies], 1u);
            if (two)
                atomicAdd(&lb[bb.bin(v) * kRowCopies], 1u);
        }
    };
    if (kept)
    {
#pragma unroll
        for (int u = 0; u < kRowKeep; ++u)
        {
            count(keep[u][0]);
            count(keep[u][1]);
            count(keep[u][2]);
            count(keep[u][3]);
        }
    }
    else if (vec)
    {
        for (int64_t i = threadIdx.x; i < nvec; i += kHistBlock)
        {
            const v4f a = rv[i];
            count(a[0]);
            count(a[1]);
            count(a[2]);
            count(a[3]);
        }
    }
    else
    {
        for (int64_t i = threadIdx.x; i < n_per_hist; i += kHistBlock)
            count(row[i]);
    }
    __syncthreads();
    const bool rebins  = has_stats && r.rebin;
    if (rebins)
        rebin_running_histogram(upd, sh, r, num_bins);   // ends with a barrier
#pragma unroll
    for (int k = 0; k < kBinsPerLane; ++k)
    {
        const int i = k * kHistBlock + threadIdx.x;
        if (i >= num_bins)
            break;
        uint32_t total = 0;
#pragma unroll
        for (int c = 0; c < kRowCopies; ++c)
            total += lds[i * kRowCopies + c];
        const float before = !has_stats ? 0.0f : (rebins ? upd[i] : old_count[k]);
        sh[i]              = (float) total + before;
        if (BATCH)
        {
            uint32_t own = total;
            if (two)
            {
                own = 0;
#pragma unroll
                for (int c = 0; c < kRowCopies; ++c)
                    own += lds[(num_bins + i) * kRowCopies + c];
            }
            batch_hist[(int64_t) h * num_bins + i] = (float) own;
        }
    }
    if (threadIdx.x == 0)
    {
        state_minmax[2 * h]     = r.new_min;
        state_minmax[2 * h + 1] = r.new_max;
    }
}

// min / max of a number and a value that is a number or a quiet NaN: the number when the other is NaN.  One
// instruction each; fminf / fmaxf first pass both operands through a canonicalising max, which triples the count in
// a loop that is short on issue slots.
__device__ __forceinline__ float min_of_number_and_maybe_nan(float number, float other)
{
    float r;
    asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(number), "v"(other));
    return r;
}
__device__ __forceinline__ float max_of_number_and_maybe_nan(float number, float other)
{
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(number), "v"(other));
    return r;
}

// ---- speculative update (running statistics exist, the batch's own histogram is not wanted) -----------------
// First launch.  grid (blocks, H).  One pass over row h: finite min / max (one partial per workgroup, as
// finite_minmax_kernel writes them) and, in the same pass, the counts of the row over the range the running statistics
// have now -- which is the range merge_stats will use unless the batch reaches outside it (EA:216-221, 253-255).
// Counts go to LDS, then to the first slot of one of `replicas` global copies ([h][replica][2][num_bins] uint32, all
// zero between updates).  A workgroup clears and flushes a whole LDS histogram whatever its share of the row, so long
// rows go to few workgroups of 1024 threads.
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void spec_bin_kernel(const float* __restrict__ x, int64_t n_per_hist, int num_bins,
                                                         const float* __restrict__ state_minmax,
                                                         float* __restrict__ mm_partial, uint32_t* __restrict__ counts,
                                                         int replicas, int vec)
{
    constexpr int copies = kSpecCopies;   // LDS copies of the histogram, interleaved (a constant: the bin index is
                                          // scaled by it per element, and a 32-bit multiply runs at quarter rate)
    extern __shared__ uint32_t lds[];
    __shared__ float s_mm[2][BLOCK / 64];
    constexpr int kInFlight = kSpecLoads;   // 16-byte loads of a lane in flight
    const int h          = blockIdx.y;
    const float* row     = x + (int64_t) h * n_per_hist;
    const v4f* rv        = reinterpret_cast<const v4f*>(row);
    const int64_t nvec   = n_per_hist / 4;
    // workgroup b counts the 16-byte groups [b * share, (b + 1) * share) of the row: equal shares (a multiple of a
    // wavefront's 64 loads) whatever the grid, so that a grid of one workgroup per compute unit splits the row evenly
    const int64_t share  = (((nvec + gridDim.x - 1) / gridDim.x) + 63) & ~(int64_t) 63;
    const int64_t stride = (int64_t) BLOCK * kInFlight;
    int64_t base         = (int64_t) blockIdx.x * share;
    const int64_t end    = base + share < nvec ? base + share : nvec;
    v4f a[kInFlight];
    // A tile that lies inside the share as a whole is requested without a condition per lane.  With one, the loaded
    // value passes through a select, the compiler waits for it there, and a tile requested "ahead" is waited for
    // before the current one is counted.
    auto request = [&](v4f(&to)[kInFlight], int64_t at) {
        if (at + (int64_t) kInFlight * BLOCK <= end)   // workgroup-uniform
        {
#pragma unroll
            for (int u = 0; u < kInFlight; ++u)
                to[u] = __builtin_nontemporal_load(rv + at + u * BLOCK + threadIdx.x);
        }
        else
        {
#pragma unroll
            for (int u = 0; u < kInFlight; ++u)
            {
                const int64_t i = at + u * BLOCK + threadIdx.x;
                to[u]           = i < end ? __builtin_nontemporal_load(rv + i) : (v4f) {NAN, NAN, NAN, NAN};
            }
        }
    };
    if (vec)
        request(a, base);
    for (int i = threadIdx.x; i < num_bins * copies; i += BLOCK)
        lds[i] = 0;
    // torch.histc(min, max) over the statistics' range: equal bounds are widened by one each way
    float m_lo = state_minmax[2 * h], m_hi = state_minmax[2 * h + 1];
    if (m_lo == m_hi)
    {
        m_lo -= 1.0f;
        m_hi += 1.0f;
    }
    Binner mb;
    mb.init(m_lo, m_hi, num_bins);
    uint32_t* lm = lds + (threadIdx.x & (copies - 1));
    float lo = INFINITY, hi = -INFINITY;
    auto take = [&](float v) {
        if (v != v)
            return;
        // infinities enter the minimum and maximum as a quiet NaN, which the hardware's min / max drop
        const float finite = fabsf(v) < INFINITY ? v : NAN;
        lo                 = min_of_number_and_maybe_nan(lo, finite);
        hi                 = max_of_number_and_maybe_nan(hi, finite);
        atomicAdd(&lm[mb.bin(v) * copies], 1u);
    };
    __syncthreads();
    if (vec)
    {
        // the next tile is requested before this one is counted
        while (base < end)
        {
            const int64_t next = base + stride;
            v4f nx[kInFlight];
            if (next < end)
                request(nx, next);
#pragma unroll
            for (int u = 0; u < kInFlight; ++u)
            {
                take(a[u][0]);
                take(a[u][1]);
                take(a[u][2]);
                take(a[u][3]);
            }
            if (next >= end)
                break;
#pragma unroll
            for (int u = 0; u < kInFlight; ++u)
                a[u] = nx[u];
            base = next;
        }
    }
    else
    {
        for (int64_t i = (int64_t) blockIdx.x * BLOCK + threadIdx.x; i < n_per_hist; i += (int64_t) gridDim.x * BLOCK)
            take(row[i]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        lo = fminf(lo, __shfl_xor(lo, o));
        hi = fmaxf(hi, __shfl_xor(hi, o));
    }
    if ((threadIdx.x & 63) == 0)
    {
        s_mm[0][threadIdx.x >> 6] = lo;
        s_mm[1][threadIdx.x >> 6] = hi;
    }
    __syncthreads();   // also: every LDS count is in
    if (threadIdx.x == 0)
    {
        for (int k = 1; k < BLOCK / 64; ++k)
        {
            lo = fminf(lo, s_mm[0][k]);
            hi = fmaxf(hi, s_mm[1][k]);
        }
        float* p = mm_partial + ((int64_t) h * gridDim.x + blockIdx.x) * 2;
        p[0]     = lo;
        p[1]     = hi;
    }
    uint32_t* dst = counts + ((int64_t) h * replicas + blockIdx.x % replicas) * 2 * num_bins;
    for (int i = threadIdx.x; i < num_bins; i += BLOCK)
    {
        uint32_t sum = 0;
        for (int c = 0; c < copies; ++c)
            sum += lds[i * copies + c];
        if (sum)
            atomicAdd(&dst[i], sum);
    }
}

// Second launch.  grid (blocks, H), 256 threads.  Every workgroup derives the batch's range of histogram h from the
// first launch's partials (a small reduction, cheaper than a launch of its own, as in hist_kernel).
//  - The statistics' range holds (after the first batches, nearly always): the first launch's counts are the batch's
//    histogram over the merged range.  The first kSettlers workgroups add a slice of them each to the running
//    histogram and clear them; the others leave at once.
//  - The range grew: the workgroups bin the row again, over the new range, into the second slot of the replicas; the
//    one that draws the last ticket re-bins the running histogram (merge_stats, EA:222-251), adds the new counts and
//    clears both slots.
constexpr int kSettlers = 8;

__global__ __launch_bounds__(kHistBlock) void settle_kernel(const float* __restrict__ x, int64_t n_per_hist, int num_bins,
                                                            int copies, const float* __restrict__ mm_partial,
                                                            int num_partials, float* __restrict__ state_hist,
                                                            float* __restrict__ state_minmax,
                                                            Ranges* __restrict__ ranges, float* __restrict__ batch_minmax,
                                                            int* __restrict__ bad_flag, uint32_t* __restrict__ counts,
                                                            int replicas, Tickets tickets, int vec)
{
    extern __shared__ uint32_t lds[];
    __shared__ float s_mm[2][kHistBlock / 64];
    __shared__ int s_last;
    const int h = blockIdx.y;
    float* sh             = state_hist + (int64_t) h * num_bins;
    const int slot_stride = 2 * num_bins;
    uint32_t* rep         = counts + (int64_t) h * replicas * slot_stride;
    // The workgroups that would add the first launch's counts request their first bins' counts and running values
    // now, before it is known that they will be used: they arrive together with the partials.
    const int settlers = min((int) gridDim.x, kSettlers);
    const bool settler = (int) blockIdx.x < settlers;
    const int slice    = (num_bins + settlers - 1) / settlers;
    const int first = blockIdx.x * slice, last = min(num_bins, first + slice);
    constexpr int kEarly = 2;
    uint32_t early[kEarly][kSpecReplicas];
    float before[kEarly];
    if (settler)
    {
#pragma unroll
        for (int j = 0; j < kEarly; ++j)
        {
            const int i = first + j * kHistBlock + threadIdx.x;
#pragma unroll
            for (int k = 0; k < kSpecReplicas; ++k)
                early[j][k] = (i < last && k < replicas) ? rep[(int64_t) k * slot_stride + i] : 0u;
            before[j] = i < last ? sh[i] : 0.f;
        }
    }
    float lo = INFINITY, hi = -INFINITY;
    {
        const float* p = mm_partial + (int64_t) h * num_partials * 2;
        for (int b0 = 0; b0 < num_partials; b0 += 4 * kHistBlock)
        {
            float l[4], u[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                const int b = b0 + k * kHistBlock + threadIdx.x;
                l[k]        = b < num_partials ? p[2 * b] : INFINITY;
                u[k]        = b < num_partials ? p[2 * b + 1] : -INFINITY;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                lo = fminf(lo, l[k]);
                hi = fmaxf(hi, u[k]);
            }
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        lo = fminf(lo, __shfl_xor(lo, o));
        hi = fmaxf(hi, __shfl_xor(hi, o));
    }
    if ((threadIdx.x & 63) == 0)
    {
        s_mm[0][threadIdx.x >> 6] = lo;
        s_mm[1][threadIdx.x >> 6] = hi;
    }
    __syncthreads();
    for (int k = 0; k < kHistBlock / 64; ++k)
    {
        lo = fminf(lo, s_mm[0][k]);
        hi = fmaxf(hi, s_mm[1][k]);
    }
    bool ok;
    const Ranges r = compute_ranges(lo, hi, num_bins, 1, state_minmax, h, ok);
    auto publish = [&]() {
        ranges[h] = r;
        if (batch_minmax)
        {
            batch_minmax[2 * h]     = r.batch_min;
            batch_minmax[2 * h + 1] = r.batch_max;
        }
        if (!ok)
            atomicOr(bad_flag, 1);
    };
    if (!r.rebin)
    {
        if (!settler)
            return;
#pragma unroll
        for (int j = 0; j < kEarly; ++j)
        {
            const int i = first + j * kHistBlock + threadIdx.x;
            if (i < last)
            {
                uint32_t total = 0;
#pragma unroll
                for (int k = 0; k < kSpecReplicas; ++k)
                {
                    total += early[j][k];
                    if (k < replicas)
                        rep[(int64_t) k * slot_stride + i] = 0u;
                }
                sh[i] = (float) total + before[j];
            }
        }
        for (int i = first + kEarly * kHistBlock + threadIdx.x; i < last; i += kHistBlock)
        {
            // all loads of a bin are issued before the first addition: one round trip per bin, not one per replica
            uint32_t t[kSpecReplicas];
#pragma unroll
            for (int k = 0; k < kSpecReplicas; ++k)
                t[k] = k < replicas ? rep[(int64_t) k * slot_stride + i] : 0u;
            const float was = sh[i];
            uint32_t total  = 0;
#pragma unroll
            for (int k = 0; k < kSpecReplicas; ++k)
            {
                total += t[k];
                if (k < replicas)
                    rep[(int64_t) k * slot_stride + i] = 0u;
            }
            sh[i] = (float) total + was;
        }
        if (blockIdx.x == 0 && threadIdx.x == 0)
            publish();   // (state_minmax keeps its values)
        return;
    }

    // ---- the range grew
    Binner mb;
    mb.init(r.m_lo, r.m_hi, num_bins);
    for (int i = threadIdx.x; i < num_bins * copies; i += kHistBlock)
        lds[i] = 0;
    __syncthreads();
    uint32_t* lm = lds + (threadIdx.x & (copies - 1));
    auto count   = [&](float v) {
        if (v == v)
            atomicAdd(&lm[mb.bin(v) * copies], 1u);
    };
    if (vec)
    {
        const v4f* rv      = reinterpret_cast<const v4f*>(x + (int64_t) h * n_per_hist);
        const int64_t nvec = n_per_hist / 4;
        for (int64_t base = (int64_t) blockIdx.x * kHistBlock * 2; base < nvec; base += (int64_t) gridDim.x * kHistBlock * 2)
        {
            v4f a[2];
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                const int64_t i = base + u * kHistBlock + threadIdx.x;
                a[u]            = i < nvec ? __builtin_nontemporal_load(rv + i) : (v4f) {NAN, NAN, NAN, NAN};
            }
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                count(a[u][0]);
                count(a[u][1]);
                count(a[u][2]);
                count(a[u][3]);
            }
        }
    }
    else
    {
        const float* row = x + (int64_t) h * n_per_hist;
        for (int64_t i = (int64_t) blockIdx.x * kHistBlock + threadIdx.x; i < n_per_hist;
             i += (int64_t) gridDim.x * kHistBlock)
            count(row[i]);
    }
    __syncthreads();
    uint32_t* dst = rep + (int64_t) (blockIdx.x % replicas) * slot_stride + num_bins;
    for (int i = threadIdx.x; i < num_bins; i += kHistBlock)
    {
        uint32_t sum = 0;
        for (int c = 0; c < copies; ++c)
            sum += lds[i * copies + c];
        if (sum)
            atomicAdd(&dst[i], sum);
    }
    if (!last_ticket(tickets, h, &s_last))
        return;
    float* upd = reinterpret_cast<float*>(lds);   // num_bins floats fit where num_bins * copies counters were
    rebin_running_histogram(upd, sh, r, num_bins);
    // this launch's counts are in the second slot; the first launch's, over the old range, are cleared with them
    consume_counts<kHistBlock>(rep + num_bins, slot_stride, replicas, num_bins, -num_bins,
                               [&](int i, uint32_t total) { sh[i] = (float) total + upd[i]; });
    if (threadIdx.x == 0)
    {
        publish();
        state_minmax[2 * h]     = r.new_min;
        state_minmax[2 * h + 1] = r.new_max;
    }
}

// grid (H, ceil(bins / 256)), 256 threads: writes the batch histogram, re-bins the running histogram when the
// range grew (merge_stats, EA:222-251) and adds the batch's counts over the merged range.
__global__ __launch_bounds__(kHistBlock) void merge_kernel(uint32_t* __restrict__ sums, int replicas,
                                                           int num_bins, int has_stats, int count_batch,
                                                           int count_merged,
                                                           const Ranges* __restrict__ ranges,
                                                           float* __restrict__ state_hist,
                                                           float* __restrict__ state_minmax,
                                                           float* __restrict__ batch_hist)
{
    __shared__ float upd[kMaxBins];
    const int h    = blockIdx.x;
    const Ranges r = ranges[h];
    // gridDim.y workgroups share a histogram's bins when the running histogram keeps its range (the usual case: every
    // bin is then updated on its own).  Re-binning scatters every old bin into the new range, so one workgroup does
    // all of it and the others leave.
    const bool rebinning = has_stats && r.rebin;
    if (rebinning && blockIdx.y != 0)
        return;
    const int slice   = rebinning ? num_bins : (num_bins + (int) gridDim.y - 1) / (int) gridDim.y;
    const int bin_lo  = rebinning ? 0 : (int) blockIdx.y * slice;
    const int bin_hi  = min(num_bins, bin_lo + slice);
    float* sh      = state_hist + (int64_t) h * num_bins;
    float* bh      = batch_hist ? batch_hist + (int64_t) h * num_bins : nullptr;
    const int width      = (count_batch + count_merged) * num_bins;
    uint32_t* rep        = sums + (int64_t) h * replicas * width;
    const int merged_off = count_batch ? num_bins : 0;
    // counts of bin i over all replicas (integers: the order of the additions does not matter)
    // (all loads of a bin are issued before the first addition: one round trip per bin, not one per replica)
    // Every counter is read by exactly one thread of this launch, which leaves it cleared: between updates the count
    // replicas hold zeros (the speculative update relies on it).
    auto total = [&](int i) {
        uint32_t t[kMaxReplicas];
#pragma unroll
        for (int r = 0; r < kMaxReplicas; ++r)
            t[r] = r < replicas ? rep[(int64_t) r * width + i] : 0u;
        uint32_t sum = 0;
#pragma unroll
        for (int r = 0; r < kMaxReplicas; ++r)
        {
            sum += t[r];
            if (r < replicas)
                rep[(int64_t) r * width + i] = 0u;
        }
        return sum;
    };
    if (rebinning)
        rebin_running_histogram(upd, sh, r, num_bins);
    for (int i = bin_lo + threadIdx.x; i < bin_hi; i += kHistBlock)
    {
        if (count_batch && (batch_hist || !has_stats))
        {
            const float c = (float) total(i);
            if (batch_hist)
                bh[i] = c;
            if (!has_stats)
                sh[i] = c;
        }
        if (has_stats && count_merged)
            sh[i] = (float) total(merged_off + i) + (r.rebin ? upd[i] : sh[i]);
    }
    if (threadIdx.x == 0 && blockIdx.y == 0)
    {
        state_minmax[2 * h]     = r.new_min;
        state_minmax[2 * h + 1] = r.new_max;
    }
}

// ---- SQNR search ---------------------------------------------------------------------------------------------
struct SearchArgs
{
    int num_bins, num_hist;
    int symmetric;
    int n_delta;        // asymmetric: delta candidates; symmetric: delta candidates
    int n_offset;       // asymmetric: offsets from the arange + 1 observed; symmetric: 1
    int n_arange;       // asymmetric: number of arange offsets
    float num_steps;    // float32(num_steps)
    double num_steps_d;
    double offset_step; // num_steps / (num_offsets - 2)
    float sym_offset;   // (-num_steps) // 2
    float gamma;
    int use_gamma;      // gamma != 1.0
};

// candidate c of histogram with gated (min_v, max_v): (delta, offset) exactly as the reference's tensor ops give them
__device__ void candidate(const SearchArgs& a, float min_v, float max_v, int c, float& delta, float& offset)
{
    if (a.symmetric)
    {
        const float max_delta = 2.0f * fmaxf(max_v, -min_v) / a.num_steps;
        delta                 = fmaxf(max_delta * (float) (c + 1) / (float) (a.n_delta - 1), kMinScale);
        offset                = a.sym_offset;
        return;
    }
    const int di = c / a.n_offset, oi = c - di * a.n_offset;
    const float max_delta       = (max_v - min_v) / a.num_steps;
    const float observed_offset = rintf(min_v / max_delta);
    const float observed_min    = max_delta * observed_offset;
    const float observed_max    = observed_min + max_delta * a.num_steps;
    const float test_delta      = max_delta * (float) (di + 1) / (float) (a.n_delta - 1);
    const float test_offset =
        oi < a.n_arange ? rintf((float) (-a.num_steps_d + a.offset_step * (double) oi)) : observed_offset;
    float test_min = test_delta * test_offset;
    float test_max = test_min + test_delta * a.num_steps;
    test_min       = fmaxf(observed_min, test_min);
    test_max       = fminf(observed_max, test_max);
    delta          = fmaxf((test_max - test_min) / a.num_steps, kMinScale);
    offset         = rintf(test_min / delta);
}

__device__ __forceinline__ void gated_minmax(const float* minmax, int h, float num_steps, float eps_steps, float& mn,
                                             float& mx)
{
    mn = fminf(minmax[2 * h], 0.0f);
    mx = fmaxf(minmax[2 * h + 1], 0.0f);
    mx = fmaxf(mx, mn + eps_steps);
}

// grid (candidate groups, H), 256 threads = 4 wavefronts, one candidate per wavefront at a time
__global__ __launch_bounds__(256) void sqnr_noise_kernel(const float* __restrict__ hist,
                                                         const float* __restrict__ minmax, SearchArgs a,
                                                         float eps_steps, int cand_per_block,
                                                         double* __restrict__ noise)
{
    __shared__ float s_mid[kMaxBins];
    __shared__ float s_cnt[kMaxBins];
    const int h = blockIdx.y, nb = a.num_bins;
    // bin mid-points from the histogram's own edges: edges = arange * step + min (EA:197-205), mid-points EA:700-703
    float lo = minmax[2 * h], hi = minmax[2 * h + 1];
    if (hi == lo)
    {
        lo = lo - 0.5f;
        hi = hi + 0.5f;
    }
    const float step       = (hi - lo) / (float) nb;
    const float e0         = 0.0f * step + lo;
    const float e1         = 1.0f * step + lo;
    const float hist_delta = e1 - e0;
    const float base       = e0 + hist_delta / 2.0f;
    for (int i = threadIdx.x; i < nb; i += 256)
    {
        s_mid[i] = base + hist_delta * (float) i;
        s_cnt[i] = hist[(int64_t) h * nb + i];
    }
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // An empty bin adds an exact zero to every candidate's sum, so the bins that hold something are moved to the front
    // and only those are walked (a channel of a weight leaves a third or more of 2048 bins empty: 11008 channels of
    // 4096 samples search in 1.02 ms instead of 1.39 ms).  One wavefront does the moving, 5 us that a search over one
    // or a few histograms does not get back, so those walk all bins.  Nor is it done for ranges so wide that a squared
    // distance could overflow: there an empty bin contributes NaN, not zero, as in the tensor expression.
    __shared__ int s_used;
    if (a.num_hist < kCompactFrom)
    {
        if (threadIdx.x == 0)
            s_used = nb;
    }
    else if (wave == 0)
    {
        const bool keep_all = !(fmaxf(fabsf(lo), fabsf(hi)) < 1e18f);
        int used            = 0;
        for (int first = 0; first < nb; first += 64)
        {
            const int i      = first + lane;
            const float mid  = i < nb ? s_mid[i] : 0.0f;
            const float cnt  = i < nb ? s_cnt[i] : 0.0f;
            const bool keep  = i < nb && (keep_all || cnt != 0.0f);
            const uint64_t m = __ballot(keep);
            if (keep)
            {
                // (writes land at or below the lowest index this pass has read)
                const int at = used + __popcll(m & ((1ull << lane) - 1ull));
                s_mid[at]    = mid;
                s_cnt[at]    = cnt;
            }
            used += __popcll(m);
        }
        if (lane == 0)
            s_used = used;
    }
    __syncthreads();
    const int used = s_used;
    float mn, mx;
    gated_minmax(minmax, h, a.num_steps, eps_steps, mn, mx);
    const int ncand = a.n_delta * a.n_offset;
    const int c_end = min(ncand, (int) (blockIdx.x + 1) * cand_per_block);
    for (int c = blockIdx.x * cand_per_block + wave; c < c_end; c += 4)
    {
        float delta, offset;
        candidate(a, mn, mx, c, delta, offset);
        // mid / delta through div_by_invariant where its contract holds for every bin of this histogram (the end
        // mid-points bound the dividends; a quotient below its 2^-36 limit vanishes in the subtraction of the integer
        // offset, or rounds to zero without one); delta is the wavefront's, so the choice is uniform
        const bool short_div =
            __builtin_amdgcn_readfirstlane((int) (fastdiv_divisor_ok(delta) &&
                                                  fmaxf(fabsf(lo), fabsf(hi)) <= kFastDivMaxDividend)) != 0;
        const float rcp = 1.0f / delta;
        double acc      = 0.0;
        for (int i = lane; i < used; i += 64)
        {
            const float mid = s_mid[i];
            float q         = rintf((short_div ? div_by_invariant(mid, delta, rcp) : mid / delta) - offset);
            const bool clip = q < 0.0f || q > a.num_steps;
            q               = fminf(fmaxf(q, 0.0f), a.num_steps);
            const float d   = (q + offset) * delta - mid;
            float err       = d * d * s_cnt[i];
            if (a.use_gamma && clip)
                err = err * a.gamma;
            acc += (double) err;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1)
            acc += __shfl_xor(acc, o);
        if (lane == 0)
            noise[(int64_t) h * ncand + c] = acc;
    }
}

// grid H: first minimum in flattened (delta, offset) order, then min = offset * delta, max = min + num_steps * delta
__global__ __launch_bounds__(64) void sqnr_pick_kernel(const double* __restrict__ noise,
                                                       const float* __restrict__ minmax, SearchArgs a, float eps_steps,
                                                       float* __restrict__ out_min, float* __restrict__ out_max,
                                                       int* __restrict__ out_index)
{
    const int h = blockIdx.x, lane = threadIdx.x;
    const int ncand = a.n_delta * a.n_offset;
    double best = INFINITY;
    int best_c  = 0x7fffffff;
    for (int c = lane; c < ncand; c += 64)
    {
        const double v = noise[(int64_t) h * ncand + c];
        if (v < best || (v == best && c < best_c))
        {
            best   = v;
            best_c = c;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        const double ob = __shfl_xor(best, o);
        const int oc    = __shfl_xor(best_c, o);
        if (ob < best || (ob == best && oc < best_c))
        {
            best   = ob;
            best_c = oc;
        }
    }
    if (lane == 0)
    {
        if (best_c == 0x7fffffff)
            best_c = 0;   // every score NaN: torch.min returns the first NaN's index; candidate 0 stands in for it
        float mn, mx, delta, offset;
        gated_minmax(minmax, h, a.num_steps, eps_steps, mn, mx);
        candidate(a, mn, mx, best_c, delta, offset);
        const float emin = offset * delta;
        out_min[h]       = emin;
        out_max[h]       = emin + a.num_steps * delta;
        if (out_index)
            out_index[h] = best_c;
    }
}

int hist_blocks(int64_t num_hist, int64_t n_per_hist)
{
    // enough workgroups to fill 256 CUs three times over, at least ~8K elements each
    int64_t per_row = (n_per_hist + 6143) / 6144;
    int64_t want    = (1024 + num_hist - 1) / num_hist;
    int64_t b       = per_row < want ? per_row : want;
    return (int) (b < 1 ? 1 : b);
}

// workgroups of 1024 threads per row in a speculative update of long rows: about kSpecElems elements each, at most
// hist_blocks() of them (the workspace is sized for that many partials).  A compute unit runs one such workgroup after
// the other, so among the counts near that size the one is taken for which the busiest of the 256 compute units has
// the least to do: rounds * (elements of a workgroup + what clearing and flushing its LDS histogram is worth).
int spec_blocks(int64_t num_hist, int64_t n_per_hist)
{
    constexpr int64_t kComputeUnits = 256, kFixedCost = 6144;
    const int64_t cap  = hist_blocks(num_hist, n_per_hist);
    const int64_t near = (n_per_hist + kSpecElems - 1) / kSpecElems;
    int64_t best = 1, best_cost = INT64_MAX;
    int64_t first = near / 2 > 1 ? near / 2 : 1;
    first         = first < cap ? first : cap;
    for (int64_t b = first; b <= 2 * near && b <= cap; ++b)
    {
        const int64_t rounds = (b * num_hist + kComputeUnits - 1) / kComputeUnits;
        const int64_t cost   = rounds * ((n_per_hist + b - 1) / b + kFixedCost);
        if (cost < best_cost)
        {
            best_cost = cost;
            best      = b;
        }
    }
    return (int) best;
}

int make_search(SearchArgs& a, int64_t num_hist, int num_bins, double num_steps, int symmetric, double gamma,
                int asym_deltas, int sym_deltas, int offset_candidates)
{
    MIQ_CHECK_ARG(num_hist > 0 && num_hist < (1 << 30), "bad number of histograms");
    MIQ_CHECK_ARG(num_bins > 0 && num_bins <= kMaxBins, "num_bins must lie in 1..%d", kMaxBins);
    MIQ_CHECK_ARG(num_steps > 0, "The number of quantization bins cannot be less than or equal to 0.");
    MIQ_CHECK_ARG(asym_deltas >= 2 && sym_deltas >= 2 && offset_candidates >= 3, "too few search candidates");
    a.num_bins    = num_bins;
    a.num_hist    = (int) num_hist;
    a.symmetric   = symmetric != 0;
    a.num_steps   = (float) num_steps;
    a.num_steps_d = num_steps;
    a.gamma       = (float) gamma;
    a.use_gamma   = gamma != 1.0;
    a.sym_offset  = (float) std::floor(-num_steps / 2.0);
    a.offset_step = 0;
    a.n_arange    = 0;
    if (a.symmetric)
    {
        a.n_delta  = sym_deltas;
        a.n_offset = 1;
    }
    else
    {
        // num_offsets = min(num_steps + 2, offset_candidates); arange(-num_steps, step, step): ceil((end - start) / step)
        const double num_offsets = std::fmin(num_steps + 2.0, (double) offset_candidates);
        a.offset_step            = num_steps / (num_offsets - 2.0);
        a.n_arange               = (int) std::ceil((a.offset_step - (-num_steps)) / a.offset_step);
        a.n_delta                = asym_deltas;
        a.n_offset               = a.n_arange + 1;
    }
    return MIQ_OK;
}
}   // namespace
}   // namespace miq

using namespace miq;

extern "C" {

int64_t miq_v2_hist_workspace_bytes(int64_t num_hist, int64_t n_per_hist, int num_bins)
{
    if (num_hist <= 0 || n_per_hist <= 0 || num_bins <= 0)
        return 0;
    const int64_t blocks   = hist_blocks(num_hist, n_per_hist);
    const int64_t replicas = blocks < kMaxReplicas ? blocks : kMaxReplicas;
    // count replicas (two histograms each) + per-workgroup (min, max) + the per-histogram ranges + the ticket counters of
    // the speculative update's second launch
    const int64_t groups = (blocks + kTicketGroup - 1) / kTicketGroup;
    if (blocks == 1 && num_bins <= kRowBinsMax)   // a row per workgroup: nothing is kept outside LDS
        return 512;
    return num_hist * replicas * 2 * (int64_t) num_bins * 4 + num_hist * blocks * 2 * 4 +
           num_hist * (int64_t) sizeof(Ranges) + num_hist * 4 +
           (groups > 1 ? num_hist * groups * kTicketStride * 4 : 0) + 512;
}

int miq_v2_hist_update_f32(const float* data, int64_t num_hist, int64_t n_per_hist, int num_bins, int has_stats,
                           int want_batch_hist, float* state_hist, float* state_minmax, float* batch_hist,
                           float* batch_minmax, int32_t* bad_flag, void* workspace, void* stream)
{
    MIQ_CHECK_ARG(num_hist > 0 && n_per_hist > 0, "empty input");
    MIQ_CHECK_ARG(num_bins > 0 && num_bins <= kMaxBins, "num_bins must lie in 1..%d", kMaxBins);
    MIQ_CHECK_ARG(num_hist <= 65535, "at most 65535 histograms per call");
    MIQ_CHECK_ARG(data && state_hist && state_minmax && bad_flag && workspace, "null pointer");
    MIQ_CHECK_ARG(!want_batch_hist || batch_hist, "batch_hist is needed when want_batch_hist is set");
    // which histograms this pass fills: the batch's own range and / or the merged range
    const int count_batch  = !has_stats || want_batch_hist;
    const int count_merged = has_stats != 0;
    const int kinds        = count_batch + count_merged;
    const int copies       = kinds == 1 ? 4 : 2;   // LDS: kinds * bins * copies * 4 B <= 64 KiB at 4096 bins
    const int blocks   = hist_blocks(num_hist, n_per_hist);
    const int replicas = blocks < kMaxReplicas ? blocks : kMaxReplicas;
    char* ws           = (char*) workspace;
    uint32_t* counts   = (uint32_t*) ws;
    ws += num_hist * replicas * 2 * (int64_t) num_bins * 4;
    float* mm_part = (float*) ws;
    ws += num_hist * blocks * 2 * 4;
    ws             = (char*) (((uintptr_t) ws + 15) & ~(uintptr_t) 15);
    Ranges* ranges = (Ranges*) ws;
    hipStream_t s  = (hipStream_t) stream;
    const int vec  = (n_per_hist % 4 == 0) && aligned16(data);
    const int width = kinds * num_bins;
    ws += num_hist * (int64_t) sizeof(Ranges);
    // ticket counters of the speculative update's second launch
    uint32_t* words       = (uint32_t*) ws;
    const int64_t groups  = (blocks + kTicketGroup - 1) / kTicketGroup;
    uint32_t* group_words = (uint32_t*) (((uintptr_t) (words + num_hist) + 127) & ~(uintptr_t) 127);
    const Tickets tickets = {words, groups > 1 ? group_words : nullptr};
    if (blocks == 1 && num_bins <= kRowBinsMax)
    {
        // a row per workgroup: the whole update in one launch ([kinds][bins][copies] LDS words, kinds * copies = 2)
        const size_t lds_bytes = (size_t) num_bins * 2 * sizeof(uint32_t);   // row_update_kernel's [kinds][bins][copies]
        if (want_batch_hist)
            hipLaunchKernelGGL(row_update_kernel<true>, dim3((unsigned) num_hist), dim3(kHistBlock), lds_bytes, s, data,
                               n_per_hist, num_bins, has_stats, state_hist, state_minmax, batch_hist, batch_minmax,
                               bad_flag, vec);
        else
            hipLaunchKernelGGL(row_update_kernel<false>, dim3((unsigned) num_hist), dim3(kHistBlock), lds_bytes, s, data,
                               n_per_hist, num_bins, has_stats, state_hist, state_minmax, batch_hist, batch_minmax,
                               bad_flag, vec);
        MIQ_CHECK_LAUNCH();
        return MIQ_OK;
    }
    if (has_stats && !want_batch_hist)
    {
        // speculative update: one pass when the statistics' range holds
        const bool wide         = n_per_hist >= kSpecWideFrom;
        const int sblocks       = wide ? spec_blocks(num_hist, n_per_hist) : blocks;
        const int spec_replicas = sblocks < kSpecReplicas ? sblocks : kSpecReplicas;
        const size_t lds_bytes  = (size_t) num_bins * kSpecCopies * sizeof(uint32_t);
        if (wide)
            hipLaunchKernelGGL(spec_bin_kernel<1024>, dim3(sblocks, (unsigned) num_hist), dim3(1024), lds_bytes, s, data,
                               n_per_hist, num_bins, state_minmax, mm_part, counts, spec_replicas, vec);
        else
            hipLaunchKernelGGL(spec_bin_kernel<kHistBlock>, dim3(sblocks, (unsigned) num_hist), dim3(kHistBlock),
                               lds_bytes, s, data, n_per_hist, num_bins, state_minmax, mm_part, counts, spec_replicas,
                               vec);
        MIQ_CHECK_LAUNCH();
        // (a smaller grid for this launch -- all but eight workgroups per histogram leave at once -- measured the same)
        hipLaunchKernelGGL(settle_kernel, dim3(blocks, (unsigned) num_hist), dim3(kHistBlock), lds_bytes, s, data,
                           n_per_hist, num_bins, 4, mm_part, sblocks, state_hist, state_minmax, ranges, batch_minmax,
                           bad_flag, counts, spec_replicas, tickets, vec);
        MIQ_CHECK_LAUNCH();
        return MIQ_OK;
    }
    hipLaunchKernelGGL(finite_minmax_kernel, dim3(blocks, (unsigned) num_hist), dim3(kHistBlock), 0, s, data, n_per_hist,
                       mm_part, counts, replicas * width, vec);
    MIQ_CHECK_LAUNCH();
    hipLaunchKernelGGL(hist_kernel, dim3(blocks, (unsigned) num_hist), dim3(kHistBlock),
                       (size_t) width * copies * sizeof(uint32_t), s, data, n_per_hist, num_bins, has_stats, count_batch,
                       count_merged, copies, mm_part, state_minmax, ranges, batch_minmax, bad_flag, counts, replicas,
                       vec);
    MIQ_CHECK_LAUNCH();
    hipLaunchKernelGGL(merge_kernel, dim3((unsigned) num_hist, (unsigned) ((num_bins + kHistBlock - 1) / kHistBlock)),
                       dim3(kHistBlock), 0, s, counts, replicas, num_bins,
                       has_stats, count_batch, count_merged, ranges, state_hist, state_minmax,
                       want_batch_hist ? batch_hist : nullptr);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_v2_sqnr_num_candidates(double num_steps, int symmetric, int asym_deltas, int sym_deltas, int offset_candidates)
{
    SearchArgs a;
    if (make_search(a, 1, 1, num_steps, symmetric, 1.0, asym_deltas, sym_deltas, offset_candidates))
        return -1;
    return a.n_delta * a.n_offset;
}

int miq_v2_sqnr_search_f32(const float* hist, const float* minmax, int64_t num_hist, int num_bins, double num_steps,
                           int symmetric, double gamma, int asym_deltas, int sym_deltas, int offset_candidates,
                           float* out_min, float* out_max, double* noise, int32_t* best_index, void* stream)
{
    SearchArgs a;
    if (int rc = make_search(a, num_hist, num_bins, num_steps, symmetric, gamma, asym_deltas, sym_deltas,
                             offset_candidates))
        return rc;
    MIQ_CHECK_ARG(num_hist <= 65535, "at most 65535 histograms per call");
    MIQ_CHECK_ARG(hist && minmax && out_min && out_max && noise, "null pointer");
    const int ncand = a.n_delta * a.n_offset;
    // MINIMUM_SCALE * num_steps is a Python float product, cast to float32 when added to the tensor
    const float eps_steps = (float) ((double) kMinScale * num_steps);
    // few histograms: spread one histogram's candidates over many workgroups -- one candidate per wavefront while that
    // keeps the grid within about a thousand workgroups
    int64_t cand_per_block = (ncand * num_hist + 1023) / 1024;
    cand_per_block         = (cand_per_block + 3) / 4 * 4;
    cand_per_block         = cand_per_block > ncand ? ncand : cand_per_block;
    const int groups   = (int) ((ncand + cand_per_block - 1) / cand_per_block);
    hipStream_t s      = (hipStream_t) stream;
    hipLaunchKernelGGL(sqnr_noise_kernel, dim3(groups, (unsigned) num_hist), dim3(256), 0, s, hist, minmax, a, eps_steps,
                       (int) cand_per_block, noise);
    MIQ_CHECK_LAUNCH();
    hipLaunchKernelGGL(sqnr_pick_kernel, dim3((unsigned) num_hist), dim3(64), 0, s, noise, minmax, a, eps_steps, out_min,
                       out_max, best_index);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

}   // extern "C"
