// AdaRound iteration of a Linear layer with the soft rounding fused into MFMA GEMMs (gfx950).
//
// Reference (ADA = TrainingExtensions/torch/src/python/aimet_torch/v1/adaround), one iteration of
// AdaroundOptimizer._optimize_rounding (ADA/adaround_optimizer.py:182-218) for torch.nn.Linear:
//   W'   = apply_adaround(W)                                   ADA/adaround_wrapper.py:124-149
//   out  = functional.linear(x[batch], W', bias)               ADA/adaround_optimizer.py:276-277
//   loss = recon_loss(act(out), act(y[batch])) + round_loss    ADA/adaround_loss.py:70-111
//   loss.backward(); Adam step on alpha
//
// With 32 rows per iteration (the reference's BATCH_SIZE; 64, 128 and 256 rows are taken as 2, 4 and 8 blocks of 32, which
// is how a 1x1 convolution over a few pixels arrives here: its rows are the pixels of the 32 images) the GEMMs are
// bandwidth-bound on the weight-shaped operands, so the point of fusing is that W' and dLoss/dW' never exist in memory:
//   (W enters as F = floor(W / delta), computed once per layer: W and delta do not change during the optimisation)
//   lin_fwd_kernel   reads F and alpha once, forms W' in registers and feeds it to 16x16x4 fp32 MFMAs as the B
//                    operand; the K dimension is split over workgroups, partial [32, O] products go to a workspace
//   lin_loss_kernel  adds the partials in a fixed order (deterministic), bias, activation, and writes
//                    G = dLoss_recon/dout = 2 (act(out) - act(y)) act'(out) / batch
//   lin_bwd_kernel   forms dLoss/dW'[o][k] = sum_b G[b][o] x[b][k] as a rank-32 MFMA product in registers and runs
//                    the alpha-gradient + regulariser + Adam epilogue on it (reads W, alpha, m, v; writes alpha, m, v)
//
// MFMA operand layout used below (v_mfma_f32_16x16x4_f32, one wavefront): lane l supplies A[m = l % 16][k = l / 16]
// and B[k = l / 16][n = l % 16]; it receives D[m = 4 (l / 16) + i][n = l % 16] in element i of the accumulator.
#include "miq_adaround_math.h"

namespace miq
{
namespace
{
using namespace ada;

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kBatch  = 32;    // rows of a block: BATCH_SIZE of ADA/adaround_optimizer.py:58; an iteration has 1, 2, 4 or 8 blocks
constexpr int kMaxRowBlocks = 8;
constexpr int kTileO  = 32;    // output channels per workgroup
constexpr int kTileK  = 256;   // K extent of a tile: one 1 KiB row segment per wavefront-wide 16-byte access
constexpr int kFwdTileK = 128;        // k extent of a forward tile
constexpr int kFwdGroupsWanted = 512; // forward workgroups: two of them fit on each of the 256 CUs

struct LinGeom
{
    int out_features, in_features;
    int chan_stride;      // 1: delta/offset per output channel, 0: one entry for the whole tensor
    const float* delta;
    const float* offset;
    float clip_min, clip_max;
};

__device__ __forceinline__ v4f mfma16(float a, float b, v4f c)
{
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// Row of x / target for batch entry b.  An index outside [0, num_rows) is clamped so that the read stays inside the
// buffer; lin_loss_kernel marks such a row's results NaN.
__device__ __forceinline__ int64_t gather_row(const int* row_index, int b, int num_rows)
{
    const int r = row_index ? row_index[b] : b;
    return (int64_t) min(max(r, 0), num_rows - 1);
}

__device__ __forceinline__ v4f ldg4(const float* p)
{
    return *reinterpret_cast<const v4f*>(p);
}

__device__ __forceinline__ v4f ldg4_stream(const float* p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p));
}

// Four consecutive values of floor(W / delta), stored as float32 or, where every channel's window of useful values fits,
// as int8 or int16 (miq_adaround_floor_i8 / _i16): a quarter or half of the bytes of the operand that never changes
// during the optimisation.  `type` is the raw form in which they travel from memory (one register for int8): the
// forward kernel keeps them like that while the loads are in flight.
template <typename FT>
struct FloorRaw;
template <>
struct FloorRaw<float>
{
    typedef v4f type;
    static __device__ __forceinline__ type load(const float* p) { return ldg4_stream(p); }
    static __device__ __forceinline__ v4f widen(type w) { return w; }
};
template <>
struct FloorRaw<int8_t>
{
    typedef int32_t type;
    static __device__ __forceinline__ type load(const int8_t* p)
    {
        return __builtin_nontemporal_load(reinterpret_cast<const int32_t*>(p));
    }
    static __device__ __forceinline__ v4f widen(type w)
    {
        return (v4f) {(float) (int8_t) (w & 0xff), (float) (int8_t) ((w >> 8) & 0xff), (float) (int8_t) ((w >> 16) & 0xff),
                      (float) (w >> 24)};
    }
};
template <>
struct FloorRaw<int16_t>
{
    typedef int type __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ type load(const int16_t* p)
    {
        return __builtin_nontemporal_load(reinterpret_cast<const type*>(p));
    }
    static __device__ __forceinline__ v4f widen(type w)
    {
        return (v4f) {(float) (int16_t) (w[0] & 0xffff), (float) (w[0] >> 16), (float) (int16_t) (w[1] & 0xffff),
                      (float) (w[1] >> 16)};
    }
};

template <typename FT>
__device__ __forceinline__ v4f load_floor4(const FT* p)
{
    return FloorRaw<FT>::widen(FloorRaw<FT>::load(p));
}

constexpr int kLdsRow = kTileK + 4;   // floats per LDS tile row; the pad spreads the MFMA-layout accesses over banks

// Both kernels move [32 o] x [256 k] (backward) or [32 o] x [128 k] (forward) tiles of the weight-shaped tensors
// through LDS, so that global memory is always touched in the streaming layout (a lane owns 16 consecutive bytes of a
// row segment that its wavefront covers without gaps) while the MFMAs see their own operand / accumulator layout.
// (Measured alternative: wavefront-private [16 o] x [128 k] tiles without workgroup barriers were 10-20 % slower.)

// Workgroup barrier that waits for this wavefront's LDS traffic only.  __syncthreads() would also wait for every
// global load in flight, and the point of the loop below is to keep the next tile's loads in flight across it.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Forward tiles ([32 o] x [TK k]) are stored without a row pad, 16-byte chunk q of row r at chunk q ^ (r & 15): a
// wavefront's streaming store (consecutive chunks of a row) and its MFMA-layout load (16 rows x one chunk, four chunk
// columns) both touch every bank group once (SQ_LDS_BANK_CONFLICT reads 0).
template <int TK>
__device__ __forceinline__ int fwd_slot(int r, int chunk)
{
    return r * TK + 4 * (chunk ^ (r & 15));
}

// grid (ceil(K / TK / tiles_per_group), O / 32), 512 threads.  A workgroup owns 32 output channels and walks
// `tiles_per_group` consecutive TK-wide k tiles of them with its eight wavefronts in two roles:
//   wavefronts 4..7 (producers) stream floor(W / delta) and alpha, form W' and store it to one of two LDS tiles;
//   wavefronts 0..3 (consumers) multiply the other LDS tile with the 32 activation rows on the MFMA.
// One barrier per tile hands a finished tile over.  Every SIMD so holds wavefronts that issue the conversion's vector
// arithmetic and wavefronts that issue MFMAs -- the two run in different pipes -- and a producer requests its next tile
// as soon as it has converted one, before it waits at the barrier.
// Consumer w multiplies k in [TK/4 w, TK/4 (w + 1)) of every tile and keeps its [32 b] x [32 o] partial product in
// registers; the four are added once, at the end: K / TK / tiles_per_group partial products per output in the workspace.
// Consecutive workgroups walk along the rows, so the workgroups that run together cover contiguous memory.
//
// Measured on the [4096, 4096] layer with int8 floor values (84 MB moved; the same loads and barriers without the
// conversion and the MFMAs take 20 us):
//   one tile per 256-thread workgroup, every wavefront converts, then multiplies (2048 workgroups)       28.8 us
//   the same wavefronts walking 4 tiles with the next tile's loads in flight                              27.7 us
//   producer / consumer roles, TK 256, producers two tiles ahead                                          27.0 us
//   roles, TK 128: producers four / two / one tile ahead                                    26.0 / 23.4 / 22.9 us
//   roles, TK 64, one tile ahead, two / four workgroups per CU                                     25.3 / 24.3 us
//   roles, TK 128, two tiles ahead as straight-line code for exactly 8 tiles (the waits then count loads) 22.5 us,
//       and 2 us slower than one ahead with float32 floor values: not kept
// What a workgroup still has to compute when its last bytes arrive (a conversion, then a multiplication) is exposed at
// the end of the kernel, and loads requested further ahead arrive in larger bunches: small tiles, one tile ahead.
// Raising the producers' or the consumers' wavefront priority changed nothing or lost 1.5 us.
//
// R blocks of 32 rows: the consumers multiply every tile with each block in turn (the tile's W' is read from LDS once
// per tile, the blocks' activations come through the caches) and keep R partial products; more than two blocks need
// more registers than four wavefronts per SIMD leave.
template <typename FT, int TK, int R>
__global__ __launch_bounds__(512, (R <= 2 ? 4 : 2)) void lin_fwd_kernel(const FT* __restrict__ F,
                                                                       const float* __restrict__ alpha,
                                                                       const float* __restrict__ X,
                                                                       const int* __restrict__ row_index, int num_rows,
                                                                       int64_t x_row_stride, float* __restrict__ partial,
                                                                       LinGeom g, int tiles_per_group)
{
    static_assert(TK == 64 || TK == 128 || TK == 256, "a wavefront-wide 16-byte access covers one, two or four rows of a tile");
    constexpr int kLoads  = 8 * TK / 256;   // 16-byte accesses per lane and tile: 8 rows of TK floats per wavefront
    constexpr int kRowsPerLoad = 256 / TK;  // rows one wavefront-wide access covers
    constexpr int kSteps  = TK / 64;        // MFMA k steps of 16 per consumer and tile
    typedef FloorRaw<FT> Raw;
    __shared__ __attribute__((aligned(16))) float tile[2 * kTileO * TK];
    // the wavefront number as a scalar: the role branch below is then a scalar branch, and a wavefront executes the
    // barriers of its own role only
    const int wave = __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int w4   = wave & 3;
    const int o_blk   = blockIdx.y * kTileO;
    const int K       = g.in_features;
    const int t_first = blockIdx.x * tiles_per_group;
    const int T       = min(tiles_per_group, K / TK - t_first);   // tiles of this workgroup (>= 1)
    float* const buf0 = tile;
    float* const buf1 = tile + kTileO * TK;
    v4f* const red    = reinterpret_cast<v4f*>(tile);   // after the last tile: [4 consumers][4 blocks][64 lanes]
    static_assert(2 * kTileO * TK >= 4 * 4 * 64 * 4, "the partial products reuse the tiles' memory");
    v4f acc[R][2][2];   // consumers only

    if (wave >= 4)
    {
        // ---- producer: rows 8 w4 .. 8 w4 + 7 of every tile, streaming layout: access j of lane l is row
        // kRowsPerLoad j + l / (TK / 4), floats 4 (l % (TK / 4)) .. + 3
        const int sub_row = lane / (TK / 4), col4 = lane % (TK / 4);
        float dl[kLoads], of[kLoads];
#pragma unroll
        for (int j = 0; j < kLoads; ++j)
        {
            const int c = (o_blk + w4 * 8 + kRowsPerLoad * j + sub_row) * g.chan_stride;
            dl[j]       = g.delta[c];
            of[j]       = g.offset[c];
        }
        // everything but the lane's own offset is the same for the whole wavefront: scalar address arithmetic
        const int64_t w_base      = (int64_t) (o_blk + w4 * 8) * K + (int64_t) t_first * TK;
        const FT* const f_base    = F + w_base;
        const float* const a_base = alpha + w_base;
        const int64_t lane_off    = (int64_t) sub_row * K + 4 * col4;
        typename Raw::type f[kLoads];
        v4f al[kLoads];
        auto request = [&](int i) {
#pragma unroll
            for (int j = 0; j < kLoads; ++j)
            {
                const int64_t row = (int64_t) (kRowsPerLoad * j) * K + i * TK;
                f[j]  = Raw::load(f_base + row + lane_off);
                al[j] = ldg4_stream(a_base + row + lane_off);
            }
        };
        auto convert = [&](float* buf) {
#pragma unroll
            for (int j = 0; j < kLoads; ++j)
            {
                const v4f f4 = Raw::widen(f[j]);
                v4f wq;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    wq[i] = adarounded_f<true>(f4[i], al[j][i], dl[j], of[j], g.clip_min, g.clip_max);
                *reinterpret_cast<v4f*>(&buf[fwd_slot<TK>(w4 * 8 + kRowsPerLoad * j + sub_row, col4)]) = wq;
            }
        };
        request(0);
        convert(buf0);
        if (1 < T)
            request(1);
        lds_barrier();
        // phase i: tile i + 1 is converted while the consumers multiply tile i
        for (int i0 = 0; i0 < T; i0 += 2)
        {
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                const int i = i0 + u;
                if (i >= T)
                    break;
                if (i + 1 < T)
                {
                    convert(u == 0 ? buf1 : buf0);
                    if (i + 2 < T)
                        request(i + 2);
                }
                lds_barrier();
            }
        }
    }
    else
    {
        // ---- consumer: MFMA layout, lane (n, s) supplies rows n and 16 + n of a block, k = TK/4 w4 + 16 kk + 4 s + i
        const int n = lane & 15, s = lane >> 4;
        // the row numbers of a block in one load (lane l: entry l % 32), passed on by shuffles: a load per use is a
        // chain of round trips before the first activation can be requested
        int rows[R][2];
#pragma unroll
        for (int rb = 0; rb < R; ++rb)
        {
            const int row_of_lane = (int) gather_row(row_index, rb * kBatch + (lane & 31), num_rows);
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
                rows[rb][mt] = __shfl(row_of_lane, mt * 16 + n);
        }
        const float* const xcol = X + (int64_t) t_first * TK + w4 * (TK / 4) + 4 * s;
#pragma unroll
        for (int rb = 0; rb < R; ++rb)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int nt = 0; nt < 2; ++nt)
                    acc[rb][mt][nt] = (v4f) {0.f, 0.f, 0.f, 0.f};
        // the activations of (tile, block) units, requested two units ahead of their use
        v4f x[2][kSteps][2];
        auto request_x = [&](v4f(&xr)[kSteps][2], int i, const int(&row)[2]) {
#pragma unroll
            for (int kk = 0; kk < kSteps; ++kk)
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
                    xr[kk][mt] = ldg4(xcol + (int64_t) row[mt] * x_row_stride + i * TK + kk * 16);
        };
        v4f wq[kSteps][2];
        auto load_w = [&](const float* buf) {
#pragma unroll
            for (int kk = 0; kk < kSteps; ++kk)
#pragma unroll
                for (int nt = 0; nt < 2; ++nt)
                    wq[kk][nt] =
                        *reinterpret_cast<const v4f*>(&buf[fwd_slot<TK>(nt * 16 + n, w4 * (TK / 16) + kk * 4 + s)]);
        };
        auto multiply = [&](const v4f(&xr)[kSteps][2], v4f(&ac)[2][2]) {
#pragma unroll
            for (int kk = 0; kk < kSteps; ++kk)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
                        for (int mt = 0; mt < 2; ++mt)
                            ac[mt][nt] = mfma16(xr[kk][mt][i], wq[kk][nt][i], ac[mt][nt]);
        };
        request_x(x[0], 0, rows[0]);
        if constexpr (R > 1)
            request_x(x[1], 0, rows[R > 1 ? 1 : 0]);
        else if (1 < T)
            request_x(x[1], 1, rows[0]);
        lds_barrier();
        for (int i0 = 0; i0 < T; i0 += 2)
        {
#pragma unroll
            for (int u = 0; u < 2; ++u)
            {
                const int i = i0 + u;
                if (i >= T)
                    break;
                load_w(u == 0 ? buf0 : buf1);
#pragma unroll
                for (int rb = 0; rb < R; ++rb)
                {
                    constexpr int kAhead = 2;                      // units between a request and its use
                    const int b          = (u * R + rb) & 1;       // the unit's buffer (R is 1 or even)
                    multiply(x[b], acc[rb]);
                    const int next_rb = (rb + kAhead) % R, next_i = i + (rb + kAhead) / R;
                    if (next_i < T)
                        request_x(x[b], next_i, rows[next_rb]);
                }
                lds_barrier();
            }
        }
    }
    // Both roles have passed T + 1 barriers, the last of them after every consumer's last multiplication: the tiles'
    // memory is free.  Block by block, the four consumers' products are added in wavefront order: one partial [32, 32]
    // product per block and workgroup.
#pragma unroll
    for (int rb = 0; rb < R; ++rb)
    {
        if (rb > 0)
            __syncthreads();
        if (wave < 4)
        {
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int nt = 0; nt < 2; ++nt)
                    red[(wave * 4 + mt * 2 + nt) * 64 + lane] = acc[rb][mt][nt];
        }
        __syncthreads();
        if (wave < 4)
        {
            const int t4 = wave, ln = lane;   // block index, lane within the block
            const v4f sum = ((red[(0 * 4 + t4) * 64 + ln] + red[(1 * 4 + t4) * 64 + ln]) + red[(2 * 4 + t4) * 64 + ln]) +
                            red[(3 * 4 + t4) * 64 + ln];
            const int mt = t4 >> 1, nt = t4 & 1;
            const int o  = o_blk + nt * 16 + (ln & 15);
            const int b0 = rb * kBatch + mt * 16 + 4 * (ln >> 4);
            float* dst   = partial + ((int64_t) blockIdx.x * (R * kBatch) + b0) * g.out_features + o;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                dst[(int64_t) i * g.out_features] = sum[i];
        }
    }
}

// one thread per (b, o): out = sum_s partial[s][b][o] + bias[o]; G = 2 (act(out) - act(y)) act'(out) / batch
__global__ __launch_bounds__(256) void lin_loss_kernel(const float* __restrict__ partial, int num_split,
                                                       const float* __restrict__ bias, const float* __restrict__ Y,
                                                       const int* __restrict__ row_index, int num_rows,
                                                       int64_t y_row_stride, int out_features, int batch, int act,
                                                       float* __restrict__ out, float* __restrict__ G,
                                                       float* __restrict__ loss_partial)
{
    const int idx         = blockIdx.x * 256 + threadIdx.x;
    const float per_batch = 1.0f / (float) batch;   // a power of two: multiplying is dividing
    float sq              = 0.f;
    if (idx < batch * out_features)
    {
        const int b = idx / out_features, o = idx - b * out_features;
        // the row number and the bias are requested before the partial products, and the target as soon as the row
        // number is back: two dependent round trips in all (requested where they are used, the four kinds of load
        // form a chain of four)
        const int r         = row_index ? row_index[b] : b;
        const float bias_o  = bias ? bias[o] : 0.f;
        // the partial products are added in split order; four of them are requested at a time
        const float* p      = partial + (int64_t) b * out_features + o;
        const int64_t pitch = (int64_t) batch * out_features;
        float acc           = 0.f;
        int s               = 0;
        float first[4]      = {0.f, 0.f, 0.f, 0.f};
        if (num_split >= 4)
        {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                first[q] = p[q * pitch];
            s = 4;
        }
        float y = Y[(int64_t) min(max(r, 0), num_rows - 1) * y_row_stride + o];   // as gather_row
        if (num_split >= 4)
            acc = (((acc + first[0]) + first[1]) + first[2]) + first[3];
        for (; s + 4 <= num_split; s += 4)
        {
            const float p0 = p[s * pitch], p1 = p[(s + 1) * pitch], p2 = p[(s + 2) * pitch], p3 = p[(s + 3) * pitch];
            acc            = (((acc + p0) + p1) + p2) + p3;
        }
        for (; s < num_split; ++s)
            acc += p[s * pitch];
        if (bias)
            acc += bias_o;
        if (r < 0 || r >= num_rows)
            acc = NAN;   // no such row: poison everything derived from it
        if (out)
            out[idx] = acc;
        float pass = 1.f, ao = acc;
        if (act == 1)
        {
            pass = acc > 0.f ? 1.f : 0.f;
            ao   = fmaxf(acc, 0.f);
            y    = fmaxf(y, 0.f);
        }
        const float diff = ao - y;
        sq               = diff * diff;
        G[idx]           = (acc != acc) ? acc : 2.0f * diff * pass * per_batch;
    }
    if (loss_partial)
    {
        const float t = block_sum_256(sq);
        if (threadIdx.x == 0)
            loss_partial[blockIdx.x] = t * per_batch;
    }
}

// grid (K / 256, O / 32), 256 threads.  Phase 1: wavefront w forms dLoss/dW' for k in [64w, 64w + 64) as four 16-wide k
// tiles (the M dimension of the MFMA) by two 16-wide o tiles (N), the batch being the MFMA's K dimension (8 steps of
// 4), and parks it in the LDS tile.  Phase 2: the alpha-gradient + regulariser + Adam epilogue in the streaming layout.
//
// Measured on the [4096, 4096] layer with int8 floor values (432 MB moved): 78 us; without phase 1, 73.6 us; without
// phase 1 and with the epilogue's arithmetic replaced by additions, 70.9 us.  Phase 1 as a loop of "row number,
// activations, multiply" per step compiles into sixteen dependent round trips (a wait for every outstanding load
// before each of them, the epilogue's first rows included) and took 82.5 us: its operands are requested up front,
// ahead of the epilogue's rows, with the row numbers from one load.  Other ways of hiding phase 1 that were tried:
//   one 16-byte activation load per lane and step feeding four MFMAs (k interleaved instead of blocked)    no change
//   the register cap alone, eight registers spilled                                                         89 us
//   workgroups of two roles as in lin_fwd_kernel walking 4 tiles, two LDS tiles, two workgroups per CU:
//       4 epilogue + 4 MFMA wavefronts                                                                      86.5 us
//       4 epilogue + 1 MFMA wavefront, two or four rows ahead                                         125 / 121 us
// Eight streaming wavefronts per CU do not keep enough bytes in flight; sixteen with the multiplication in between do.
//
// More than 32 rows (MULTI): the rank-32 product is repeated for every block of 32 rows into the same accumulators, a
// block's operands being requested when the previous block's multiplications have been issued.
// in_features that are a multiple of 128 but not of 256: the last tile of a row has 128 columns.  Its workgroups read
// the first half twice (every address stays inside the row) and the lanes of the missing half store nothing.
template <int PF, typename FT, bool MULTI>
__global__ __launch_bounds__(256) void lin_bwd_kernel(const FT* __restrict__ F, const float* __restrict__ G,
                                                      const float* __restrict__ X, const int* __restrict__ row_index,
                                                      int num_rows, int64_t x_row_stride, float* __restrict__ alpha,
                                                      float* __restrict__ m, float* __restrict__ v,
                                                      float* __restrict__ grad_out, LinGeom g, AdamArgs a,
                                                      float* __restrict__ reg_partial, int row_blocks)
{
    __shared__ __attribute__((aligned(16))) float tile[kTileO * kLdsRow];
    __shared__ PowEntry tab[128];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n = lane & 15, s = lane >> 4;
    const int o_blk = blockIdx.y * kTileO;
    const int k_blk = blockIdx.x * kTileK;
    PowTableLoad tl;
    tl.request();
    const int K = g.in_features, O = g.out_features;
    const bool half_tile = k_blk + kTileK > K;          // the same for the whole workgroup
    const bool live      = k_blk + 4 * lane < K;        // this lane's four columns exist
    const int k_lane     = k_blk + 4 * lane - (live ? 0 : kTileK / 2);
    // the 64 columns whose products this wavefront forms: those of wavefront w - 2 again where there are none
    const int k_wave = k_blk + 64 * (half_tile && wave >= 2 ? wave - 2 : wave);

    // per-row delta / offset, requested here and not where they are used (see lin_fwd_kernel); a row belongs to one
    // wavefront, so with the wavefront number as a scalar these are scalar loads
    float dl[8], of[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
    {
        const int c = (o_blk + __builtin_amdgcn_readfirstlane(wave) * 8 + j) * g.chan_stride;
        dl[j]       = g.delta[c];
        of[j]       = g.offset[c];
    }

    // phase 1's operands are requested first: loads return in the order of their requests, so the multiplication
    // starts once these (cache hits) are back and does not wait for the epilogue's rows requested after them
    float xa[8][4], gb[8][2];
    // the 32 row numbers of a block in one load (lane l holds that of entry l % 32), handed to the lanes that need
    // them by shuffles: a load per step is a chain of eight round trips.  (Scalar loads of the 32 numbers measured
    // the same.)
    auto request_block = [&](int rb) {
        const int row_of_lane = (int) gather_row(row_index, rb * kBatch + (lane & 31), num_rows);
#pragma unroll
        for (int step = 0; step < 8; ++step)
        {
            const int b       = 4 * step + s;
            const float* xrow = X + (int64_t) __shfl(row_of_lane, b) * x_row_stride + k_wave + n;
            const float* grow = G + (int64_t) (rb * kBatch + b) * O + o_blk + n;
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
                xa[step][mt] = xrow[mt * 16];
#pragma unroll
            for (int nt = 0; nt < 2; ++nt)
                gb[step][nt] = grow[nt * 16];
        }
    };
    request_block(0);
    __builtin_amdgcn_sched_barrier(0);   // the requests above stay above: nothing below is scheduled between them
    // the epilogue's first rows: they arrive while phase 1 runs
    v4f fv[PF], av[PF], mv[PF], vv[PF];
#pragma unroll
    for (int j = 0; j < PF; ++j)
    {
        const int64_t e = (int64_t) (o_blk + wave * 8 + j) * K + k_lane;
        fv[j]           = load_floor4<FT>(F + e);
        av[j]           = ldg4(alpha + e);
        mv[j]           = ldg4(m + e);
        vv[j]           = ldg4(v + e);
    }

    __builtin_amdgcn_sched_barrier(0);   // the requests above stay above: nothing below is scheduled between them
    v4f acc[4][2];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
            acc[mt][nt] = (v4f) {0.f, 0.f, 0.f, 0.f};
    const int blocks = MULTI ? row_blocks : 1;
    for (int rb = 0; rb < blocks; ++rb)
    {
        if (MULTI && rb > 0)
            request_block(rb);
#pragma unroll
        for (int step = 0; step < 8; ++step)
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                for (int nt = 0; nt < 2; ++nt)
                    acc[mt][nt] = mfma16(xa[step][mt], gb[step][nt], acc[mt][nt]);
    }
    // lane holds dW'[o = 16 nt + n][k = 64 w + 16 mt + 4 s + i], i = 0..3
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
            *reinterpret_cast<v4f*>(&tile[(nt * 16 + n) * kLdsRow + wave * 64 + mt * 16 + 4 * s]) = acc[mt][nt];
    tl.store(tab);
    __syncthreads();

    float reg = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j)
    {
        const int r     = wave * 8 + j;
        const int slot  = j % PF;
        const int64_t e = (int64_t) (o_blk + r) * K + k_lane;
        const v4f f4 = fv[slot], a4 = av[slot], m4 = mv[slot], v4 = vv[slot];
        if (j + PF < 8)
        {
            const int64_t e2 = e + PF * (int64_t) K;
            fv[slot]         = load_floor4<FT>(F + e2);
            av[slot]         = ldg4(alpha + e2);
            mv[slot]         = ldg4(m + e2);
            vv[slot]         = ldg4(v + e2);
        }
        const float d = dl[j], off = of[j];
        const v4f gw  = *reinterpret_cast<const v4f*>(&tile[r * kLdsRow + 4 * lane]);
        float as[4] = {a4[0], a4[1], a4[2], a4[3]}, ms[4] = {m4[0], m4[1], m4[2], m4[3]};
        float vs[4] = {v4[0], v4[1], v4[2], v4[3]};
        v4f gr;
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            float rr;
            const float gi = alpha_grad_f(f4[i], gw[i], as[i], d, off, g.clip_min, g.clip_max, a, tab, rr);
            reg += live ? rr : 0.f;
            adam_update(gi, as[i], ms[i], vs[i], a);
            gr[i] = gi;
        }
        if (live)
        {
            *reinterpret_cast<v4f*>(alpha + e) = (v4f) {as[0], as[1], as[2], as[3]};
            *reinterpret_cast<v4f*>(m + e)     = (v4f) {ms[0], ms[1], ms[2], ms[3]};
            *reinterpret_cast<v4f*>(v + e)     = (v4f) {vs[0], vs[1], vs[2], vs[3]};
            if (grad_out)
                *reinterpret_cast<v4f*>(grad_out + e) = gr;
        }
    }
    if (reg_partial)
    {
        const float t = block_sum_256(reg);
        if (threadIdx.x == 0)
            reg_partial[blockIdx.y * gridDim.x + blockIdx.x] = t;
    }
}

// 1, 2, 4 or 8 blocks of 32 rows; 0 for a batch the fused path does not take
int row_blocks_of(int64_t batch)
{
    for (int r = 1; r <= kMaxRowBlocks; r *= 2)
        if (batch == (int64_t) r * kBatch)
            return r;
    return 0;
}

int make_lin_geom(LinGeom& g, int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                  const float* offset, float clip_min, float clip_max)
{
    MIQ_CHECK_ARG(out_features > 0 && in_features > 0, "bad layer shape");
    MIQ_CHECK_ARG(out_features % kTileO == 0 && in_features % kFwdTileK == 0,
                  "the fused Linear path takes out_features that are a multiple of 32 and in_features that are a "
                  "multiple of 128 (got %lld x %lld)", (long long) out_features, (long long) in_features);
    MIQ_CHECK_ARG(out_features * in_features < (1ll << 31), "layer too large for the fused Linear path");
    MIQ_CHECK_ARG(num_channel == 1 || num_channel == out_features,
                  "delta/offset must have one entry, or one per output channel");
    MIQ_CHECK_ARG(delta && offset, "null delta/offset");
    MIQ_CHECK_ARG(clip_min <= clip_max, "clip_min must not exceed clip_max");
    g.out_features = (int) out_features;
    g.in_features  = (int) in_features;
    g.chan_stride  = num_channel == 1 ? 0 : 1;
    g.delta        = delta;
    g.offset       = offset;
    g.clip_min     = clip_min;
    g.clip_max     = clip_max;
    return MIQ_OK;
}
}   // namespace
}   // namespace miq

using namespace miq;

// Consecutive k tiles per forward workgroup: as many as still leave one workgroup for each of the 512 places the chip
// has for this kernel (two per CU, 256 CUs), at most 16.
static int fwd_tiles_per_group(int64_t out_features, int64_t in_features)
{
    const int64_t along = in_features / kFwdTileK;
    const int64_t tiles = (out_features / kTileO) * along;
    int64_t per_group   = tiles / kFwdGroupsWanted;
    per_group           = per_group < 1 ? 1 : (per_group > 16 ? 16 : per_group);
    return (int) (per_group > along ? along : per_group);
}

template <typename FT, int R>
static void launch_lin_fwd(dim3 grid, hipStream_t s, const FT* weight_floor, const float* alpha, const float* x,
                           const int32_t* row_index, int num_rows, int64_t x_row_stride, float* workspace,
                           const LinGeom& g, int tiles_per_group)
{
    hipLaunchKernelGGL((lin_fwd_kernel<FT, kFwdTileK, R>), grid, dim3(512), 0, s, weight_floor, alpha, x, row_index,
                       num_rows, x_row_stride, workspace, g, tiles_per_group);
}

template <typename FT>
static int linear_fwd(const FT* weight_floor, const float* alpha, const float* x, const int32_t* row_index,
                      int64_t batch, int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride, const float* bias,
                      int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                      const float* offset, float clip_min, float clip_max, int activation, float* workspace, float* out,
                      float* grad_out, float* loss_partial, void* stream)
{
    LinGeom g;
    if (int rc = make_lin_geom(g, out_features, in_features, num_channel, delta, offset, clip_min, clip_max))
        return rc;
    MIQ_CHECK_ARG(weight_floor && alpha && x && target && workspace && grad_out, "null tensor pointer");
    MIQ_CHECK_ARG(aligned16(weight_floor) && aligned16(alpha) && aligned16(x) && (x_row_stride % 4) == 0,
                  "weight_floor, alpha and the rows of x must be 16-byte aligned");
    MIQ_CHECK_ARG(x_row_stride >= in_features && target_row_stride >= out_features, "row stride shorter than a row");
    MIQ_CHECK_ARG(activation == 0 || activation == 1, "activation must be 0 (none) or 1 (ReLU)");
    const int row_blocks = row_blocks_of(batch);
    MIQ_CHECK_ARG(row_blocks != 0, "the fused Linear path takes 32, 64, 128 or 256 rows per iteration (got %lld)",
                  (long long) batch);
    MIQ_CHECK_ARG(num_rows >= 1 && num_rows < (1ll << 31) && (row_index || num_rows >= batch),
                  "num_rows (%lld) must be positive, and at least the batch without a row index", (long long) num_rows);
    const int tiles_per_group = fwd_tiles_per_group(out_features, in_features);
    const int splits          = (int) ((in_features / kFwdTileK + tiles_per_group - 1) / tiles_per_group);
    const dim3 grid((unsigned) splits, (unsigned) (out_features / kTileO));
    hipStream_t s = (hipStream_t) stream;
    switch (row_blocks)
    {
    case 1: launch_lin_fwd<FT, 1>(grid, s, weight_floor, alpha, x, row_index, (int) num_rows, x_row_stride, workspace, g, tiles_per_group); break;
    case 2: launch_lin_fwd<FT, 2>(grid, s, weight_floor, alpha, x, row_index, (int) num_rows, x_row_stride, workspace, g, tiles_per_group); break;
    case 4: launch_lin_fwd<FT, 4>(grid, s, weight_floor, alpha, x, row_index, (int) num_rows, x_row_stride, workspace, g, tiles_per_group); break;
    default: launch_lin_fwd<FT, 8>(grid, s, weight_floor, alpha, x, row_index, (int) num_rows, x_row_stride, workspace, g, tiles_per_group); break;
    }
    MIQ_CHECK_LAUNCH();
    const unsigned blocks = (unsigned) ((batch * out_features + 255) / 256);
    hipLaunchKernelGGL(lin_loss_kernel, dim3(blocks), dim3(256), 0, s, workspace, splits, bias, target, row_index,
                       (int) num_rows, target_row_stride, (int) out_features, (int) batch, activation, out, grad_out,
                       loss_partial);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

template <typename FT>
static int linear_bwd_adam(const FT* weight_floor, const float* grad_out, const float* x, const int32_t* row_index,
                           int64_t batch, int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg, float* exp_avg_sq, float* grad_alpha,
                           int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                           const float* offset, float clip_min, float clip_max, double reg_param, double beta, double lr,
                           double beta1, double beta2, double eps, int step, float* reg_partial, void* stream)
{
    LinGeom g;
    if (int rc = make_lin_geom(g, out_features, in_features, num_channel, delta, offset, clip_min, clip_max))
        return rc;
    MIQ_CHECK_ARG(weight_floor && grad_out && x && alpha && exp_avg && exp_avg_sq, "null tensor pointer");
    MIQ_CHECK_ARG(aligned16(weight_floor) && aligned16(alpha) && aligned16(exp_avg) && aligned16(exp_avg_sq) &&
                      aligned16(grad_alpha),
                  "tensors must be 16-byte aligned");
    MIQ_CHECK_ARG(x_row_stride >= in_features, "row stride shorter than a row");
    const int row_blocks = row_blocks_of(batch);
    MIQ_CHECK_ARG(row_blocks != 0, "the fused Linear path takes 32, 64, 128 or 256 rows per iteration (got %lld)",
                  (long long) batch);
    MIQ_CHECK_ARG(num_rows >= 1 && num_rows < (1ll << 31) && (row_index || num_rows >= batch),
                  "num_rows (%lld) must be positive, and at least the batch without a row index", (long long) num_rows);
    MIQ_CHECK_ARG(step >= 1, "Adam step count starts at 1");
    AdamArgs a;
    if (int rc = make_adam(a, reg_param, beta, lr, beta1, beta2, eps, step))
        return rc;
    // two rows of the epilogue in flight per lane: deeper prefetch (3, 4) costs registers and measured no faster
    const dim3 grid((unsigned) ((in_features + kTileK - 1) / kTileK), (unsigned) (out_features / kTileO));
    if (row_blocks == 1)
        hipLaunchKernelGGL((lin_bwd_kernel<2, FT, false>), grid, dim3(256), 0, (hipStream_t) stream, weight_floor, grad_out,
                           x, row_index, (int) num_rows, x_row_stride, alpha, exp_avg, exp_avg_sq, grad_alpha, g, a,
                           reg_partial, 1);
    else
        hipLaunchKernelGGL((lin_bwd_kernel<2, FT, true>), grid, dim3(256), 0, (hipStream_t) stream, weight_floor, grad_out,
                           x, row_index, (int) num_rows, x_row_stride, alpha, exp_avg, exp_avg_sq, grad_alpha, g, a,
                           reg_partial, row_blocks);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

extern "C" {

int64_t miq_adaround_linear_workspace_bytes(int64_t out_features, int64_t in_features, int64_t batch)
{
    if (out_features <= 0 || in_features <= 0)
        return 0;
    if (out_features % kTileO != 0 || in_features % kFwdTileK != 0 || row_blocks_of(batch) == 0)
        return 0;   // not a shape the fused path takes
    const int64_t along  = in_features / kFwdTileK;
    const int64_t per    = fwd_tiles_per_group(out_features, in_features);
    const int64_t splits = (along + per - 1) / per;
    return splits * batch * out_features * (int64_t) sizeof(float);
}

int miq_adaround_linear_blocks(int64_t out_features, int64_t in_features)
{
    return (int) ((out_features / kTileO) * ((in_features + kTileK - 1) / kTileK));
}

int miq_adaround_linear_fwd_f32(const float* weight_floor, const float* alpha, const float* x, const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride,
                                const float* bias, int64_t out_features, int64_t in_features, int64_t num_channel,
                                const float* delta, const float* offset, float clip_min, float clip_max,
                                int activation, float* workspace, float* out, float* grad_out, float* loss_partial,
                                void* stream)
{
    return linear_fwd<float>(weight_floor, alpha, x, row_index, batch, num_rows, x_row_stride, target, target_row_stride, bias,
                             out_features, in_features, num_channel, delta, offset, clip_min, clip_max, activation,
                             workspace, out, grad_out, loss_partial, stream);
}

int miq_adaround_linear_fwd_i8(const int8_t* weight_floor, const float* alpha, const float* x, const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride, const float* bias,
                               int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                               const float* offset, float clip_min, float clip_max, int activation, float* workspace,
                               float* out, float* grad_out, float* loss_partial, void* stream)
{
    return linear_fwd<int8_t>(weight_floor, alpha, x, row_index, batch, num_rows, x_row_stride, target, target_row_stride, bias,
                              out_features, in_features, num_channel, delta, offset, clip_min, clip_max, activation,
                              workspace, out, grad_out, loss_partial, stream);
}

int miq_adaround_linear_bwd_adam_f32(const float* weight_floor, const float* grad_out, const float* x,
                                     const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg,
                                     float* exp_avg_sq, float* grad_alpha, int64_t out_features, int64_t in_features,
                                     int64_t num_channel, const float* delta, const float* offset, float clip_min,
                                     float clip_max, double reg_param, double beta, double lr, double beta1, double beta2,
                                     double eps, int step, float* reg_partial, void* stream)
{
    return linear_bwd_adam<float>(weight_floor, grad_out, x, row_index, batch, num_rows, x_row_stride, alpha, exp_avg, exp_avg_sq,
                                  grad_alpha, out_features, in_features, num_channel, delta, offset, clip_min, clip_max,
                                  reg_param, beta, lr, beta1, beta2, eps, step, reg_partial, stream);
}

int miq_adaround_linear_bwd_adam_i8(const int8_t* weight_floor, const float* grad_out, const float* x,
                                    const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg,
                                    float* exp_avg_sq, float* grad_alpha, int64_t out_features, int64_t in_features,
                                    int64_t num_channel, const float* delta, const float* offset, float clip_min,
                                    float clip_max, double reg_param, double beta, double lr, double beta1, double beta2,
                                    double eps, int step, float* reg_partial, void* stream)
{
    return linear_bwd_adam<int8_t>(weight_floor, grad_out, x, row_index, batch, num_rows, x_row_stride, alpha, exp_avg, exp_avg_sq,
                                   grad_alpha, out_features, in_features, num_channel, delta, offset, clip_min,
                                   clip_max, reg_param, beta, lr, beta1, beta2, eps, step, reg_partial, stream);
}

int miq_adaround_linear_fwd_i16(const int16_t* weight_floor, const float* alpha, const float* x, const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride, const float* bias,
                               int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                               const float* offset, float clip_min, float clip_max, int activation, float* workspace,
                               float* out, float* grad_out, float* loss_partial, void* stream)
{
    return linear_fwd<int16_t>(weight_floor, alpha, x, row_index, batch, num_rows, x_row_stride, target, target_row_stride, bias,
                              out_features, in_features, num_channel, delta, offset, clip_min, clip_max, activation,
                              workspace, out, grad_out, loss_partial, stream);
}

int miq_adaround_linear_bwd_adam_i16(const int16_t* weight_floor, const float* grad_out, const float* x,
                                    const int32_t* row_index, int64_t batch,
        int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg,
                                    float* exp_avg_sq, float* grad_alpha, int64_t out_features, int64_t in_features,
                                    int64_t num_channel, const float* delta, const float* offset, float clip_min,
                                    float clip_max, double reg_param, double beta, double lr, double beta1, double beta2,
                                    double eps, int step, float* reg_partial, void* stream)
{
    return linear_bwd_adam<int16_t>(weight_floor, grad_out, x, row_index, batch, num_rows, x_row_stride, alpha, exp_avg, exp_avg_sq,
                                   grad_alpha, out_features, in_features, num_channel, delta, offset, clip_min,
                                   clip_max, reg_param, beta, lr, beta1, beta2, eps, step, reg_partial, stream);
}

}   // extern "C"
