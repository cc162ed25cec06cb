// Row-wise compositions of the piecewise-affine primitives as single kernels for gfx950:
// softmax (forward and backward), logsumexp / log_softmax, layer_norm and the row mean.
//
// Each is, element for element, the chain of primitive calls that the reference's op
// library makes (pam/pam_ops.py:288-378) with its autograd formulas
// (pam/cuda_bindings.py:27-57, 66-97, 210-239); what is fused away is the traffic: the
// unfused chain moves every intermediate through HBM (68 B per element for softmax),
// here a row is read once from HBM (again from cache for the second sweep) and written
// once.  One wavefront owns a row: lane l takes the elements l, l + 64, l + 128, ...;
// rows of 4097 ... 16384 values are owned by a work-group of 1024 threads instead
// (thread t takes t, t + 1024, ...), which holds the row in registers too.
//
// The reference leaves the order of its row sums to torch.sum.  Here the order is fixed:
// lane l adds its elements in ascending order starting from +0, then the 64 partial sums
// are combined by a butterfly, p[l] = p[l] + p[l ^ s] for s = 32, 16, 8, 4, 2, 1; a
// work-group's 16 wavefront sums are then added in ascending order.
// All kernels are HBM-bound streams: 12 B/element for softmax forward (4 for the global
// maximum sweep, 4 in, 4 out), 12 for its backward, 8 for layer_norm and log_softmax.
//
// This file is compiled twice (pam_rowops_plain.hip, pam_rowops_offset.hip): PAM_ROW_OFFSETS says whether the unchecked
// first attempt of every kernel carries the code for an offset, PAM_ROW_FN(name) names the variant's host functions;
// pam_rowops.hip holds the entry points, which choose the variant by the call's offset.
#include <math.h>

#include <atomic>
#include <type_traits>

#include "pam_common.h"
#include "pam_device.h"
#include "pam_rowops.h"

#if !defined(PAM_ROW_OFFSETS) || !defined(PAM_ROW_FN)
#error "include from pam_rowops_plain.hip or pam_rowops_offset.hip"
#endif

using namespace pamdev;

namespace {

// Wavefronts per SIMD the row kernels are compiled for (a cap of 128 registers per lane); the
// gradient kernels for the longest register-resident rows take 2 (they would spill otherwise).
#ifndef PAM_ROW_WAVES
#define PAM_ROW_WAVES 4
#endif
#ifndef PAM_ROW_WAVES_SHORT
#define PAM_ROW_WAVES_SHORT 8
#endif
// rows of up to 256 values need few registers: more wavefronts in flight hide the load latency of the short rows
#define PAM_ROW_OCC(CH) (((CH) > 0 && (CH) <= 4) ? PAM_ROW_WAVES_SHORT : PAM_ROW_WAVES)
#define PAM_ROW_OCC_GRAD(CH) ((CH) >= 16 ? 2 : PAM_ROW_OCC(CH))
constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kMaxPartials = pamrows::kMaxPartials;
constexpr float kLog2E = (float)1.4426950408889634;      // math.log2(math.e) rounded to fp32 (pam/pam_ops.py:311)
constexpr float kLn2 = (float)0.6931471805599453;        // math.log(2.0) rounded to fp32 (pam/cuda_bindings.py:235-236)

struct Offset { float off; bool has; };

// The butterfly over a wavefront, lanes 32, 16, 8, 4, 2, 1 apart in that order, without a trip through LDS per step:
// the two halves and then the rows of 16 lanes are exchanged by the swap instructions, and within a row lane l takes
// the value 8, 4, 2, 1 lanes around the row from it (a DPP operand of the add).  After the step at distance 2d the
// values repeat every 2d lanes, so the lane d around the row holds what the lane d apart (l ^ d) holds, and every lane
// ends with the same bits as with exchanges between l and l ^ d.
template <class F>
__device__ __forceinline__ float wave_fold(float p, F f)
{
    typedef uint32_t Pair2 __attribute__((ext_vector_type(2)));
    Pair2 r = __builtin_amdgcn_permlane32_swap(f2u(p), f2u(p), false, false);
    p = f(u2f(r[0]), u2f(r[1]));
    r = __builtin_amdgcn_permlane16_swap(f2u(p), f2u(p), false, false);
    p = f(u2f(r[0]), u2f(r[1]));
    p = f(p, u2f(__builtin_amdgcn_update_dpp(0u, f2u(p), 0x128, 0xf, 0xf, false)));       // row_ror:8
    p = f(p, u2f(__builtin_amdgcn_update_dpp(0u, f2u(p), 0x124, 0xf, 0xf, false)));       // row_ror:4
    p = f(p, u2f(__builtin_amdgcn_update_dpp(0u, f2u(p), 0x122, 0xf, 0xf, false)));       // row_ror:2
    p = f(p, u2f(__builtin_amdgcn_update_dpp(0u, f2u(p), 0x121, 0xf, 0xf, false)));       // row_ror:1
    return p;
}
__device__ __forceinline__ float wave_sum(float p)
{
    return wave_fold(p, [](float a, float b) { return a + b; });
}

// Who holds which element of a row and how partial sums over the row are combined.
// WaveRow: one wavefront per row, lane l holds the elements l, l + 64, ...
// BlockRow: a work-group of 1024 threads per row (rows of 4097 ... 16384 values), thread t holds t, t + 1024, ...;
// its sums: every wavefront folds its 64 partial sums by the butterfly, then the 16 wavefront sums are added in
// ascending order, ((w0 + w1) + w2) + ... + w15, by every thread itself.  Two slots of LDS alternate, so one
// barrier per sum is enough (a thread can be at most one sum ahead of the slowest).
constexpr int kBlockThreads = 1024, kBlockWaves = kBlockThreads / 64;
constexpr long kBlockRowMin = 4096, kBlockRowMax = 16L * kBlockThreads;       // the block kernels take kBlockRowMin < n <= kBlockRowMax
struct WaveRow {
    static constexpr int kStride = 64;
    int id;
    __device__ __forceinline__ long index(int c) const { return id + 64L * c; }
    __device__ __forceinline__ float sum(float p) { return wave_sum(p); }
    __device__ __forceinline__ bool all(bool ok) { return __ballot(!ok) == 0ull; }
};
struct BlockRow {
    static constexpr int kStride = kBlockThreads;
    int id; float (*slots)[kBlockWaves]; int turn;
    __device__ __forceinline__ long index(int c) const { return id + (long)kBlockThreads * c; }
    __device__ __forceinline__ float sum(float p)
    {
        p = wave_sum(p);
        float* slot = slots[turn];
        turn ^= 1;
        if (id % 64 == 0) slot[id / 64] = p;
        __syncthreads();
        float t = slot[0];
#pragma unroll
        for (int w = 1; w < kBlockWaves; ++w) t = t + slot[w];
        return t;
    }
    __device__ __forceinline__ bool all(bool ok) { return __syncthreads_and(ok ? 1 : 0) != 0; }
};

// maximum that propagates NaN, as torch.max does
struct MaxNan {
    float mx = u2f(0xff800000u); bool nan = false;
    __device__ __forceinline__ void take(float v) { if (v != v) nan = true; else mx = fmaxf(mx, v); }
    __device__ __forceinline__ void merge_wave()
    {
        mx = wave_fold(mx, [](float a, float b) { return fmaxf(a, b); });
        nan = __ballot(nan) != 0ull;
    }
    __device__ __forceinline__ float value() const { return nan ? u2f(kQNaN) : mx; }
};

// x log2(e) as a PAM product; -inf (attention masks) stays -inf (pam/pam_ops.py:312-317)
__device__ __forceinline__ float scaled(float x, Offset o, bool mask_inf)
{
    if (mask_inf && f2u(x) == 0xff800000u) return x;
    return pam_mul_off(x, kLog2E, o.off, o.has);
}

// exp2 through the kernel entry point of that name: pa_exp2(t (*) log2(2)) (pam/cuda_bindings.py:246)
__device__ __forceinline__ float exp2_op(float t, Offset o) { return exp2_entry(t, o.off, o.has); }

// ---------------------------------------------------------------- global maximum of the scaled input
typedef float v4f __attribute__((ext_vector_type(4)));

// 128-bit loads, four in flight per lane; the maximum does not depend on the order
__global__ __launch_bounds__(kThreads) void scaled_max_kernel(const float* __restrict__ x, size_t n, size_t nvec, Offset o,
                                                             int mask_inf, float* __restrict__ partial)
{
    MaxNan m;
    const bool mask = mask_inf != 0;
    const v4f* xv = reinterpret_cast<const v4f*>(x);
    const size_t step = (size_t)gridDim.x * (kThreads * 4);
    for (size_t base = (size_t)blockIdx.x * (kThreads * 4) + threadIdx.x; base < nvec; base += step) {
        v4f q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) { size_t i = base + (size_t)u * kThreads; if (i < nvec) q[u] = xv[i]; }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (base + (size_t)u * kThreads < nvec) {
                m.take(scaled(q[u].x, o, mask)); m.take(scaled(q[u].y, o, mask));
                m.take(scaled(q[u].z, o, mask)); m.take(scaled(q[u].w, o, mask));
            }
        }
    }
    for (size_t i = nvec * 4 + (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kThreads)
        m.take(scaled(x[i], o, mask));
    m.merge_wave();
    __shared__ float smx[kWaves]; __shared__ int snan[kWaves];
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    if (lane == 0) { smx[wave] = m.mx; snan[wave] = m.nan; }
    __syncthreads();
    if (threadIdx.x == 0) {
        MaxNan t;
        for (int w = 0; w < kWaves; ++w) { t.mx = fmaxf(t.mx, smx[w]); t.nan |= snan[w] != 0; }
        partial[blockIdx.x] = t.value();
    }
}

// The work-group folds the per-block maxima together (at most 4 KiB, cache resident), each wavefront a share of
// them, and exchanges the results through LDS: floor(max).  The maximum does not depend on the order.
template <int WAVES>
__device__ __forceinline__ float fold_shift(const float* __restrict__ partial, int count)
{
    __shared__ float fold_mx[WAVES];
    __shared__ int fold_nan[WAVES];
    MaxNan m;
    // (all of a thread's loads in flight together: one after the other, each waited for, they were four cache
    // latencies at the start of every work-group)
    constexpr int kPer = (kMaxPartials + WAVES * 64 - 1) / (WAVES * 64);
    float q[kPer];
#pragma unroll
    for (int u = 0; u < kPer; ++u) { const int i = (int)threadIdx.x + u * WAVES * 64; q[u] = i < count ? partial[i] : u2f(0xff800000u); }
#pragma unroll
    for (int u = 0; u < kPer; ++u) m.take(q[u]);
    m.merge_wave();
    if (threadIdx.x % 64 == 0) { fold_mx[threadIdx.x / 64] = m.mx; fold_nan[threadIdx.x / 64] = m.nan; }
    __syncthreads();
    MaxNan t;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) { t.mx = fmaxf(t.mx, fold_mx[w]); t.nan |= fold_nan[w] != 0; }
    return floorf(t.value());
}

// ---------------------------------------------------------------- row access
// CH > 0: the row fits CH values per lane and is held in registers (one read of x, all loads
// of a row in flight together); CH == 0: rows of any length, swept twice (the second sweep
// comes from cache), four loads in flight per lane.
constexpr float kNegInf = -__builtin_inff();

template <int CH>
__device__ __forceinline__ void load_row(float (&v)[CH], const float* __restrict__ p, long n, int lane, float fill)
{
#pragma unroll
    for (int c = 0; c < CH; ++c) { long i = lane + 64L * c; v[c] = i < n ? p[i] : fill; }
}
template <int CH, class L>
__device__ __forceinline__ void load_row(float (&v)[CH], const float* __restrict__ p, long n, const L& lay, float fill)
{
#pragma unroll
    for (int c = 0; c < CH; ++c) { const long i = lay.index(c); v[c] = i < n ? p[i] : fill; }
}
// Register-resident rows, one wavefront per row, in the forward kernels (one array of registers per row; kernels
// with two or three measured slower with it): the next row of the wavefront is fetched while the current one is computed.  Past the last row the fetch repeats the last row: a conditional fetch would tie the registers to their
// old contents and make the compiler wait for them at once.
// ON (a compile-time choice per kernel and row length, by measurement) = false: the row is simply loaded.
#define PAM_WAVE_FIRST_ROW(ON, AHEAD, X, FILL) \
    if constexpr (ON) load_row<CH>(AHEAD, X + (wave < rows ? wave : rows - 1) * n, n, lane, FILL)
#define PAM_WAVE_NEXT_ROW(ON, NOW, AHEAD, X, FILL)                                                       \
    if constexpr (ON) {                                                                                  \
        _Pragma("unroll") for (int c = 0; c < CH; ++c) NOW[c] = AHEAD[c];                                \
        load_row<CH>(AHEAD, X + (r + nwaves < rows ? r + nwaves : rows - 1) * n, n, lane, FILL);         \
    } else load_row<CH>(NOW, X + r * n, n, lane, FILL)

template <int CH, class L>
__device__ __forceinline__ void store_row(const float (&v)[CH], float* __restrict__ p, long n, const L& lay)
{
#pragma unroll
    for (int c = 0; c < CH; ++c) { const long i = lay.index(c); if (i < n) p[i] = v[c]; }
}

// p = p + f(x[i]) over the lane's elements in ascending order
template <class F>
__device__ __forceinline__ float stream_sum(const float* __restrict__ p, long n, int lane, F f)
{
    float acc = 0.0f;
    long i = lane;
    for (; i + 192 < n; i += 256) {
        float a = p[i], b = p[i + 64], c = p[i + 128], d = p[i + 192];
        acc = acc + f(i, a); acc = acc + f(i + 64, b); acc = acc + f(i + 128, c); acc = acc + f(i + 192, d);
    }
    // the ragged end: up to three more elements, their loads in flight together (one after the other, each waited
    // for, they were most of the time of a row of 197 values)
    const bool has_a = i < n, has_b = i + 64 < n, has_c = i + 128 < n;
    const float a = has_a ? p[i] : 0.0f, b = has_b ? p[i + 64] : 0.0f, c = has_c ? p[i + 128] : 0.0f;
    if (has_a) acc = acc + f(i, a);
    if (has_b) acc = acc + f(i + 64, b);
    if (has_c) acc = acc + f(i + 128, c);
    return acc;
}

// ---------------------------------------------------------------- checked and unchecked arithmetic
// A register-resident row is first computed with the unchecked forms of the primitives (no
// branches; they record whether every operand and result was a normal number).  If any lane of
// the wavefront saw anything else -- a zero, a subnormal, inf, NaN, an exponent out of range --
// the row is redone with the checked functions.  Both give the same bits whenever the first
// is valid, so which one ran never shows in the result.
struct Checked {
    Offset o;
    __device__ __forceinline__ float mul(float a, float b) { return pam_mul_off(a, b, o.off, o.has); }
    __device__ __forceinline__ float div(float a, float b) { return pad_div_off(a, b, o.off, o.has); }
    __device__ __forceinline__ float exp2(float t) { return exp2_entry(t, o.off, o.has); }
    __device__ __forceinline__ float log2(float v) { return log2_entry(v, o.off, o.has); }
    // log2 as logsumexp calls it: without the keyword arguments, hence never with the offset (pam/pam_ops.py:341)
    __device__ __forceinline__ float log2_plain(float v) { return log2_entry(v, 1.0f, false); }
    __device__ __forceinline__ float root(float v) { return pow_half(v, o.off, o.has); }
    // 0 (/) b for an element whose weight is exactly zero
    __device__ __forceinline__ float zero_over(float b) { return pad_div_off(0.0f, b, o.off, o.has); }
    __device__ __forceinline__ bool valid() const { return true; }
    // the places where the unchecked arithmetic has cheaper forms
    __device__ __forceinline__ float mul_const(float a, float k) { return mul(a, k); }
    __device__ __forceinline__ float mul_seen(float a, float b) { return mul(a, b); }
    __device__ __forceinline__ float square(float a) { return mul(a, a); }
    __device__ __forceinline__ float div_by_positive(float a, float b) { return div(a, b); }
    __device__ __forceinline__ void record(float) {}
};
// OFFSETS: whether the chain carries the code for an offset.  Without it the chains are shorter; a call with an offset
// (the entry points send none here) would fail every row's check and have its rows redone with the checked functions.
template <bool OFFSETS>
struct UncheckedT {
    Offset o; Span sp;
    __device__ __forceinline__ float mul(float a, float b) { return pam_unchecked_off(a, b, o.off, OFFSETS && o.has, sp); }
    __device__ __forceinline__ float div(float a, float b) { return pad_unchecked_off(a, b, o.off, OFFSETS && o.has, sp); }
    __device__ __forceinline__ float exp2(float t) { return exp2_entry_unchecked(t, o.off, OFFSETS && o.has, sp); }
    __device__ __forceinline__ float log2(float v) { return log2_entry_unchecked(v, o.off, OFFSETS && o.has, sp); }
    __device__ __forceinline__ float log2_plain(float v) { return log2_entry_unchecked(v, 1.0f, false, sp); }
    __device__ __forceinline__ float root(float v) { return pow_half_unchecked(v, o.off, OFFSETS && o.has, sp); }
    __device__ __forceinline__ float zero_over(float) { return 0.0f; }      // the divisor is a positive normal number when valid
    __device__ __forceinline__ bool usable() const { return OFFSETS || !o.has; }         // (the same for every lane of a launch)
    __device__ __forceinline__ bool valid() const { return usable() && sp.normal(); }
    // Cheaper forms (an offset takes the general ones).  mul_const: k is a positive normal constant; mul_seen and
    // div_by_positive: a was recorded earlier in the chain or is a result of exp2; div_by_positive: b is not negative
    // and was given to record().
    __device__ __forceinline__ float mul_const(float a, float k) { return OFFSETS && o.has ? mul(a, k) : pam_unchecked_const(a, k, sp); }
    __device__ __forceinline__ float mul_seen(float a, float b) { return OFFSETS && o.has ? mul(a, b) : pam_unchecked_seen(a, b, sp); }
    __device__ __forceinline__ float square(float a) { return OFFSETS && o.has ? mul(a, a) : pam_unchecked_square(a, sp); }
    __device__ __forceinline__ float div_by_positive(float a, float b) { return OFFSETS && o.has ? div(a, b) : pad_unchecked_by_positive(a, b, sp); }
    __device__ __forceinline__ void record(float v) { sp.see(f2u(v) & ~kSign); }
};
template <bool OFFSETS>
__device__ __forceinline__ bool wave_valid(const UncheckedT<OFFSETS>& u) { return __ballot(!u.valid()) == 0ull; }

// Which kernel instances carry the offset's code in their unchecked first attempt.  In the variant for calls without an
// offset: those where the shorter chains made the compiler keep more in registers than the instance may have and spill
// (by measurement over every instance: the others run 3-20 % faster without it).  BLOCK: a work-group per row.
enum RowKernel { kSoftmaxFwd, kSoftmaxBwd, kSoftmaxBwdExact, kLogsumexpFwd, kLogsumexpBwd, kLayerNormFwd, kLayerNormBwd };
template <RowKernel K, int CH, bool BLOCK>
constexpr bool fast_path_offsets()
{
    if (PAM_ROW_OFFSETS) return true;                                    // the variant for calls with an offset
    if (K == kSoftmaxBwd || K == kSoftmaxBwdExact) return true;
    if (K == kLayerNormBwd) return BLOCK ? CH >= 8 : CH == 12;
    if (K == kLogsumexpBwd) return BLOCK ? CH >= 8 : (CH == 4 || CH == 12);
    if (K == kLayerNormFwd) return !BLOCK && CH == 16;
    if (K == kSoftmaxFwd) return BLOCK && (CH == 10 || CH == 12);
    return false;                                                       // logsumexp forward
}
template <RowKernel K, int CH, bool BLOCK> using UncheckedFor = UncheckedT<fast_path_offsets<K, CH, BLOCK>()>;

// ---------------------------------------------------------------- softmax forward (pam/pam_ops.py:305-328)
__device__ __forceinline__ float softmax_weight(float x, float shift, Offset o)
{
    if (f2u(x) == 0xff800000u) return 0.0f;
    return exp2_op(scaled(x, o, false) - shift, o);
}

// one row held in registers: weights, their sum, the quotients; masked (-inf) elements weigh exactly zero
// The row is transformed in place (inputs, then weights, then quotients): one array of registers per row leaves
// room to fetch the next row meanwhile.  A weight is never negative, so -1 marks the masked elements in between.
constexpr uint32_t kMaskedMark = 0xbf800000u;
template <int CH, class M, class L>
__device__ __forceinline__ float softmax_row(float (&v)[CH], float shift, M& m, L& lay)
{
    float p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const bool masked = f2u(v[c]) == 0xff800000u;        // computed on stand-in values, then replaced
        const float t = m.mul_const(masked ? 1.0f : v[c], kLog2E) - shift;
        const float e = m.exp2(masked ? 0.5f : t);
        v[c] = masked ? u2f(kMaskedMark) : e;
        p = p + (masked ? 0.0f : e);
    }
    const float total = lay.sum(p);                  // a sum of weights from +0: never negative
    m.record(total);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const bool masked = f2u(v[c]) == kMaskedMark;
        const float q = m.div_by_positive(masked ? 1.0f : v[c], total);         // a weight is a result of exp2
        v[c] = masked ? m.zero_over(total) : q;
    }
    return total;
}

// Rows too long for registers are swept in blocks of 64 x kBlock values, a lane meeting its elements in the
// same ascending order as in the register variants (so the row sums are the same sums); the later sweeps find
// the row in cache.  The same two-step scheme applies: branch-free forms first, the checked ones if any value
// left the normal range.
constexpr int kBlock = 8;

template <class F>
__device__ __forceinline__ void for_blocks(const float* __restrict__ row, int n, int lane, float fill, F&& body)
{
    for (int base = 0; base < n; base += 64 * kBlock) {
        float v[kBlock];
#pragma unroll
        for (int c = 0; c < kBlock; ++c) { const int i = base + lane + 64 * c; v[c] = i < n ? row[i] : fill; }
#pragma unroll
        for (int c = 0; c < kBlock; ++c) { const int i = base + lane + 64 * c; body(i, i < n, v[c]); }
    }
}

// the same over two rows at once (all loads of a block are issued before its arithmetic)
template <class F>
__device__ __forceinline__ void for_blocks2(const float* __restrict__ row_a, const float* __restrict__ row_b, int n, int lane,
                                            float fill_a, float fill_b, F&& body)
{
    for (int base = 0; base < n; base += 64 * kBlock) {
        float a[kBlock], b[kBlock];
#pragma unroll
        for (int c = 0; c < kBlock; ++c) {
            const int i = base + lane + 64 * c;
            a[c] = i < n ? row_a[i] : fill_a; b[c] = i < n ? row_b[i] : fill_b;
        }
#pragma unroll
        for (int c = 0; c < kBlock; ++c) { const int i = base + lane + 64 * c; body(i, i < n, a[c], b[c]); }
    }
}

template <class M>
__device__ __forceinline__ float softmax_stream(const float* __restrict__ xr, float* __restrict__ yr, long n, int lane, float shift, M& m)
{
    auto weight = [&](float x, bool masked) { return m.exp2(masked ? 0.5f : m.mul_const(masked ? 1.0f : x, kLog2E) - shift); };
    float p = 0.0f;
    for_blocks(xr, (int)n, lane, kNegInf, [&](long, bool, float x) {
        const bool masked = f2u(x) == 0xff800000u;
        const float e = weight(x, masked);
        p = p + (masked ? 0.0f : e);
    });
    const float total = wave_sum(p);
    m.record(total);
    for_blocks(xr, (int)n, lane, kNegInf, [&](long i, bool inside, float x) {
        const bool masked = f2u(x) == 0xff800000u;
        const float q = m.div_by_positive(masked ? 1.0f : weight(x, masked), total);
        if (inside) yr[i] = masked ? m.zero_over(total) : q;
    });
    return total;
}

template <int CH>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(PAM_ROW_OCC(CH)))) void softmax_fwd_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                              float* __restrict__ row_sum, float* __restrict__ shift_out,
                                                              long rows, long n, Offset o,
                                                              const float* __restrict__ partial, int partials)
{
    const int lane = threadIdx.x % 64;
    const long wave = (long)blockIdx.x * kWaves + threadIdx.x / 64, nwaves = (long)gridDim.x * kWaves;
    float ahead[CH > 0 ? CH : 1];
    constexpr bool kAhead = CH >= 8;
    PAM_WAVE_FIRST_ROW(kAhead, ahead, x, kNegInf);                      // the fill has weight zero; in flight while the maxima are folded
    const float shift = fold_shift<kWaves>(partial, partials);
    if (wave == 0 && lane == 0) *shift_out = shift;
    for (long r = wave; r < rows; r += nwaves) {
        const float* xr = x + r * n; float* yr = y + r * n;
        float total;
        if constexpr (CH > 0) {
            float v[CH];
            PAM_WAVE_NEXT_ROW(kAhead, v, ahead, x, kNegInf);
            WaveRow lay{lane};
            UncheckedFor<kSoftmaxFwd, CH, false> u{o, Span()};
            total = softmax_row<CH>(v, shift, u, lay);
            if (!wave_valid(u)) {                              // the row is read again (from cache)
                load_row<CH>(v, xr, n, lane, kNegInf);
                Checked k{o}; total = softmax_row<CH>(v, shift, k, lay);
            }
            store_row<CH>(v, yr, n, lay);
        } else {
            UncheckedFor<kSoftmaxFwd, CH, false> u{o, Span()};
            total = softmax_stream(xr, yr, n, lane, shift, u);
            if (!wave_valid(u)) { Checked k{o}; total = softmax_stream(xr, yr, n, lane, shift, k); }
        }
        if (lane == 0) row_sum[r] = total;
    }
}

// ---------------------------------------------------------------- softmax backward
// The chain of pad, sum, where, exp2, subtract, where, mul gradients in the order autograd
// applies them (pam/cuda_bindings.py:78-97, 224-239, 43-57).
struct Approx { bool a, b, e; };
// all three gradients exact (the reference's default), as a type: the chain is then compiled without the choices
struct ExactAll { static constexpr bool a = false, b = false, e = false; };

template <class AP>
__device__ __forceinline__ float softmax_dsum_term(float e, float total, float g, Offset o, AP ap)
{
    if (ap.b) return -pam_mul_off(pad_div_off(pad_div_off(e, total, o.off, o.has), total, o.off, o.has), g, o.off, o.has);
    return pad_div_bwd(e, total, g, o.off, o.has);
}

template <class AP>
__device__ __forceinline__ float softmax_dx(float xv, float e, float g, float inv, float dtotal, float shift, Offset o, AP ap)
{
    const bool masked = f2u(xv) == 0xff800000u;
    float de = ap.a ? pam_mul_off(inv, g, o.off, o.has) : pam_mul_bwd(e, inv, g, 1.0f, false);
    de = de + dtotal;                                 // quotient's first operand + the broadcast of the sum's
    if (masked) de = 0.0f;                            // where(x == -inf, 0, exp2(..))
    const float t = scaled(xv, o, true) - shift;
    float dt;
    if (ap.e) dt = pam_mul_off(pam_mul_off(exp2_op(t, o), kLn2, o.off, o.has), de, o.off, o.has);
    else dt = pam_mul_bwd(t, 1.0f, pa_exp2_bwd(pam_mul_off(t, 1.0f, o.off, o.has), de), o.off, o.has);
    if (masked) dt = 0.0f;                            // where(x == -inf, -inf, mul(..))
    return ap.a ? pam_mul_off(dt, kLog2E, o.off, o.has) : pam_mul_bwd(xv, kLog2E, dt, o.off, o.has);
}

// The all-approximate gradient of one register-resident row with unchecked arithmetic.  Masked
// (-inf) elements and the lanes past the end of the row are computed on a stand-in value and
// replaced by the zeros the chain gives them.
template <int CH, class L, class U>
__device__ __forceinline__ void softmax_grad_row_approx(const float (&xv)[CH], const float (&g)[CH], float (&out)[CH],
                                                        float total, float shift, L& lay, long n, U& m)
{
    // kCheap: the cheaper forms of the primitives where an operand is a constant, the row's positive total -- recorded
    // here, once -- or a value the chain has recorded already: the same bits, fewer magnitudes to record.  For the
    // instances where that measured faster (5-10 %); with 12 and 16 values per lane (16 per thread) the shorter code
    // made the kernels 9-14 % slower (registers), and they keep the general forms.
    constexpr bool kCheap = L::kStride == 64 ? CH <= 6 : CH <= 12;
    auto by_const = [&](float a, float k) __attribute__((always_inline)) { return kCheap ? m.mul_const(a, k) : m.mul(a, k); };
    auto by_seen = [&](float a, float b) __attribute__((always_inline)) { return kCheap ? m.mul_seen(a, b) : m.mul(a, b); };
    auto by_total = [&](float a) __attribute__((always_inline)) { return kCheap ? m.div_by_positive(a, total) : m.div(a, total); };
    const float inv = m.div(1.0f, total);
    if (kCheap) m.record(total);
    float e[CH];
    float p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const bool masked = f2u(xv[c]) == 0xff800000u;
        const bool inside = lay.index(c) < n;
        const float t = by_const(masked ? 1.0f : xv[c], kLog2E) - shift;
        e[c] = m.exp2(masked ? 0.5f : t);                                  // exp2 of the shifted input, unmasked
        // -(((e (/) total) (/) total) (*) g); a masked element has e = 0 and the checked chain gives
        // -(0 (*) g), a zero for finite g (adding it changes nothing: the sum is never -0) and NaN otherwise
        const float term = -by_seen(by_total(by_total(e[c])), (inside && !masked) ? g[c] : 1.0f);
        if (masked && inside) m.sp.see(f2u(g[c]) & ~kSign);
        if (inside && !masked) p = p + term;
    }
    const float dtotal = lay.sum(p);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const bool masked = f2u(xv[c]) == 0xff800000u;
        const bool inside = lay.index(c) < n;
        const float de = by_seen(inv, (inside && !masked) ? g[c] : 1.0f) + dtotal;
        const float dt = by_seen(by_const(e[c], kLn2), de);
        const float dx = by_const(dt, kLog2E);
        out[c] = masked ? 0.0f : dx;
    }
}

// The all-exact gradient (the reference's default) without an offset, on unchecked arithmetic.  In the normal range
// the exact backward formulas are short (pam/cuda_kernels.cu:40-58, 85-97, 115-123): the gradient of a (*) b for a
// is g times 2^(exponent of b, plus one if the two fractions carry), i.e. the bits of b plus the fraction bits of a,
// masked to sign and exponent; the quotient's gradient for its divisor is -(2^e(a (/) b) / 2^e(b)) g, a difference of
// exponent fields; exp2's is 2^e(exp2 t) g.  The products with the upstream gradients are IEEE products in both
// forms, so those gradients need no recording; everything else is recorded as in the approximate chain.
template <int CH, class L, class U>
__device__ __forceinline__ void softmax_grad_row_exact(const float (&xv)[CH], const float (&g)[CH], float (&out)[CH],
                                                       float total, float shift, L& lay, long n, U& m)
{
    const uint32_t tot = f2u(total);
    m.record(total);                                                       // a sum of weights: never negative
    const uint32_t inv = kBias - tot + kBias;                              // 1 (/) total
    m.sp.see(inv); m.sp.see(inv + 0x00800000u);                            // normal, and below 2^127 (a carry fits)
    const uint32_t slope_c = f2u(kLog2E);
    float e[CH];
    float p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const bool masked = f2u(xv[c]) == 0xff800000u;
        const bool inside = lay.index(c) < n;
        const float t = m.mul_const(masked ? 1.0f : xv[c], kLog2E) - shift;
        e[c] = m.exp2(masked ? 0.5f : t);
        // gradient of e (/) total for total: -(2^e(e (/) total) / 2^e(total)) g
        const uint32_t quot = f2u(e[c]) - tot + kBias;                     // e (/) total, positive
        const uint32_t ratio = (quot & kExpo) - (tot & kExpo) + kBias;
        m.sp.see(quot); m.sp.see(ratio);
        const float term = -u2f(ratio) * ((inside && !masked) ? g[c] : 1.0f);
        // a masked element: e = 0, the quotient's gradient is -(0 / 2^e(total)) g, a zero for finite g and NaN otherwise
        if (masked && inside) m.sp.see(f2u(g[c]) & ~kSign);
        if (inside && !masked) p = p + term;
    }
    const float dtotal = lay.sum(p);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const bool masked = f2u(xv[c]) == 0xff800000u;
        const bool inside = lay.index(c) < n;
        const uint32_t ei = f2u(e[c]);
        // e (/) total = e (*) inv for e: g 2^(e(inv) + carry)
        const float de = ((inside && !masked) ? g[c] : 1.0f) * u2f((inv + (ei & kMant)) & ~kMant) + dtotal;
        // exp2: 2^e(exp2 t) de; the product t (*) 1 in front of it passes its gradient on unchanged
        const float dt = u2f(ei & ~kMant) * de;
        // x (*) log2(e) for x
        const float dx = dt * u2f((slope_c + (f2u(masked ? 1.0f : xv[c]) & kMant)) & ~kMant);
        out[c] = masked ? 0.0f : dx;
    }
}
// The same gradient with the checked primitives, for every combination of exact and approximate terms.
template <int CH, class L, class AP>
__device__ __forceinline__ void softmax_grad_row_checked_as(const float (&xv)[CH], const float (&g)[CH], float (&out)[CH],
                                                            float total, float inv, float shift, L& lay, long n, Offset o, AP ap)
{
    float e[CH];
    float p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        e[c] = softmax_weight(xv[c], shift, o);
        if (lay.index(c) < n) p = p + softmax_dsum_term(e[c], total, g[c], o, ap);
    }
    const float dtotal = lay.sum(p);
#pragma unroll
    for (int c = 0; c < CH; ++c) out[c] = softmax_dx(xv[c], e[c], g[c], inv, dtotal, shift, o, ap);
}
template <int CH, class L>
__device__ __forceinline__ void softmax_grad_row_checked(const float (&xv)[CH], const float (&g)[CH], float (&out)[CH],
                                                         float total, float inv, float shift, L& lay, long n, Offset o, Approx ap)
{
    if (!ap.a && !ap.b && !ap.e) softmax_grad_row_checked_as<CH>(xv, g, out, total, inv, shift, lay, n, o, ExactAll());
    else softmax_grad_row_checked_as<CH>(xv, g, out, total, inv, shift, lay, n, o, ap);
}

// EXACT: the unchecked first attempt is the all-exact chain (chosen by the host for exact gradients without an offset);
// otherwise it is the all-approximate one.  Every other combination goes to the checked functions directly.
template <int CH, bool EXACT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(PAM_ROW_OCC_GRAD(CH)))) void softmax_bwd_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                              const float* __restrict__ row_sum, const float* __restrict__ shift_in,
                                                              float* __restrict__ dx, long rows, long n, Offset o, Approx ap)
{
    const int lane = threadIdx.x % 64;
    const long wave = (long)blockIdx.x * kWaves + threadIdx.x / 64, nwaves = (long)gridDim.x * kWaves;
    const float shift = *shift_in;
    for (long r = wave; r < rows; r += nwaves) {
        const float* xr = x + r * n; const float* gr = dy + r * n; float* dr = dx + r * n;
        if constexpr (CH > 0) {
            float xv[CH], g[CH], out[CH];
            load_row<CH>(xv, xr, n, lane, kNegInf);
            load_row<CH>(g, gr, n, lane, 0.0f);
            // (the row's total after the row's loads, and its reciprocal only where it is used: computed up here, it
            // made every row wait for the total before its own loads were issued)
            const float total = row_sum[r];
            bool done = false;
            WaveRow lay{lane};
            if (EXACT) {                                  // host: all exact, no offset
                UncheckedFor<kSoftmaxBwdExact, CH, false> u{o, Span()};
                softmax_grad_row_exact<CH>(xv, g, out, total, shift, lay, n, u);
                done = wave_valid(u);
            } else if (ap.a && ap.b && ap.e) {            // the all-approximate gradient has an unchecked form
                UncheckedFor<kSoftmaxBwd, CH, false> u{o, Span()};
                softmax_grad_row_approx<CH>(xv, g, out, total, shift, lay, n, u);
                done = wave_valid(u);
            }
            if (!done) softmax_grad_row_checked<CH>(xv, g, out, total, pad_div_off(1.0f, total, o.off, o.has), shift, lay, n, o, ap);
#pragma unroll
            for (int c = 0; c < CH; ++c) { long i = lane + 64L * c; if (i < n) dr[i] = out[c]; }
        } else {
            const float total = row_sum[r];
            const float inv = pad_div_off(1.0f, total, o.off, o.has);
            bool done = false;
            if (EXACT) {                                  // the all-exact gradient as in softmax_grad_row_exact, in two sweeps
                UncheckedFor<kSoftmaxBwdExact, CH, false> m{o, Span()};
                const uint32_t tot = f2u(total), inv_b = kBias - tot + kBias, slope_c = f2u(kLog2E);
                m.record(total); m.sp.see(inv_b); m.sp.see(inv_b + 0x00800000u);
                auto weight = [&](float x, bool masked) { return m.exp2(masked ? 0.5f : m.mul_const(masked ? 1.0f : x, kLog2E) - shift); };
                float p = 0.0f;
                for_blocks2(xr, gr, (int)n, lane, kNegInf, 1.0f, [&](long, bool inside, float x, float gi) {
                    const bool masked = f2u(x) == 0xff800000u;
                    const uint32_t quot = f2u(weight(x, masked)) - tot + kBias;
                    const uint32_t ratio = (quot & kExpo) - (tot & kExpo) + kBias;
                    m.sp.see(quot); m.sp.see(ratio);
                    const float term = -u2f(ratio) * (masked ? 1.0f : gi);
                    if (masked && inside) m.sp.see(f2u(gi) & ~kSign);
                    if (inside && !masked) p = p + term;
                });
                const float dtotal = wave_sum(p);
                for_blocks2(xr, gr, (int)n, lane, kNegInf, 1.0f, [&](long i, bool inside, float x, float gi) {
                    const bool masked = f2u(x) == 0xff800000u;
                    const uint32_t ei = f2u(weight(x, masked));
                    const float de = (masked ? 1.0f : gi) * u2f((inv_b + (ei & kMant)) & ~kMant) + dtotal;
                    const float dt = u2f(ei & ~kMant) * de;
                    const float d = dt * u2f((slope_c + (f2u(masked ? 1.0f : x) & kMant)) & ~kMant);
                    if (inside) dr[i] = masked ? 0.0f : d;
                });
                done = wave_valid(m);
            } else if (ap.a && ap.b && ap.e) {            // the all-approximate gradient, branch-free forms first
                UncheckedFor<kSoftmaxBwd, CH, false> m{o, Span()};
                const float inv_u = m.div(1.0f, total);
                auto weight = [&](float x, bool masked) { return m.exp2(masked ? 0.5f : m.mul(masked ? 1.0f : x, kLog2E) - shift); };
                float p = 0.0f;
                for_blocks2(xr, gr, (int)n, lane, kNegInf, 1.0f, [&](long, bool inside, float x, float gi) {
                    const bool masked = f2u(x) == 0xff800000u;
                    const float e = weight(x, masked);
                    const float term = -m.mul(m.div(m.div(e, total), total), masked ? 1.0f : gi);
                    if (masked && inside) m.sp.see(f2u(gi) & ~kSign);         // -(0 (*) g) is a zero only for finite g
                    if (inside && !masked) p = p + term;
                });
                const float dtotal = wave_sum(p);
                for_blocks2(xr, gr, (int)n, lane, kNegInf, 1.0f, [&](long i, bool inside, float x, float gi) {
                    const bool masked = f2u(x) == 0xff800000u;
                    const float e = weight(x, masked);
                    const float de = m.mul(inv_u, masked ? 1.0f : gi) + dtotal;
                    const float d = m.mul(m.mul(m.mul(e, kLn2), de), kLog2E);
                    if (inside) dr[i] = masked ? 0.0f : d;
                });
                done = wave_valid(m);
            }
            if (!done) {
                const float dtotal = wave_sum(stream_sum(xr, n, lane, [&](long i, float v) {
                    return softmax_dsum_term(softmax_weight(v, shift, o), total, gr[i], o, ap); }));
                for (long i = lane; i < n; i += 64) {
                    const float v = xr[i];
                    dr[i] = softmax_dx(v, softmax_weight(v, shift, o), gr[i], inv, dtotal, shift, o, ap);
                }
            }
        }
    }
}

// ---------------------------------------------------------------- logsumexp and log_softmax (pam/pam_ops.py:331-347)
template <int CH, class M, class L>
__device__ __forceinline__ float logsumexp_row(const float (&xv)[CH], float shift, L& lay, long n, M& m)
{
    float p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const bool inside = lay.index(c) < n;                    // lanes past the end work on stand-in values
        const float t = m.mul_const(inside ? xv[c] : 1.0f, kLog2E) - shift;
        const float e = m.exp2(inside ? t : 0.5f);
        if (inside) p = p + e;
    }
    return m.div(shift + m.log2_plain(lay.sum(p)), kLog2E);
}

template <int CH>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(PAM_ROW_OCC(CH)))) void logsumexp_kernel(const float* __restrict__ x, float* __restrict__ lse,
                                                            float* __restrict__ y, float* __restrict__ shift_out, long rows, long n,
                                                            Offset o, const float* __restrict__ partial, int partials)
{
    const int lane = threadIdx.x % 64;
    const long wave = (long)blockIdx.x * kWaves + threadIdx.x / 64, nwaves = (long)gridDim.x * kWaves;
    float ahead[CH > 0 ? CH : 1];
    constexpr bool kAhead = CH > 0;
    PAM_WAVE_FIRST_ROW(kAhead, ahead, x, 0.0f);                          // in flight while the maxima are folded
    const float shift = fold_shift<kWaves>(partial, partials);
    if (shift_out && wave == 0 && lane == 0) *shift_out = shift;
    for (long r = wave; r < rows; r += nwaves) {
        const float* xr = x + r * n;
        if constexpr (CH > 0) {
            float xv[CH];
            PAM_WAVE_NEXT_ROW(kAhead, xv, ahead, x, 0.0f);
            WaveRow lay{lane};
            UncheckedFor<kLogsumexpFwd, CH, false> u{o, Span()};
            float out = logsumexp_row<CH>(xv, shift, lay, n, u);
            if (!wave_valid(u)) { Checked k{o}; out = logsumexp_row<CH>(xv, shift, lay, n, k); }
            if (lse && lane == 0) lse[r] = out;
            if (y) {
#pragma unroll
                for (int c = 0; c < CH; ++c) { long i = lane + 64L * c; if (i < n) y[r * n + i] = xv[c] - out; }
            }
        } else {
            auto sweep = [&](auto& m) {
                float p = 0.0f;
                for_blocks(xr, (int)n, lane, 0.0f, [&](long, bool inside, float v) {
                    const float e = m.exp2(inside ? m.mul_const(v, kLog2E) - shift : 0.5f);
                    if (inside) p = p + e;
                });
                return m.div(shift + m.log2_plain(wave_sum(p)), kLog2E);
            };
            UncheckedFor<kLogsumexpFwd, CH, false> u{o, Span()};
            float out = sweep(u);
            if (!wave_valid(u)) { Checked k{o}; out = sweep(k); }
            if (lse && lane == 0) lse[r] = out;
            if (y) for_blocks(xr, (int)n, lane, 0.0f, [&](long i, bool inside, float v) { if (inside) y[r * n + i] = v - out; });
        }
    }
}

// ---------------------------------------------------------------- row mean (pam/pam_ops.py:288-302)
__global__ __launch_bounds__(kThreads) void row_mean_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                           long rows, long n, Offset o)
{
    const int lane = threadIdx.x % 64;
    const long wave = (long)blockIdx.x * kWaves + threadIdx.x / 64, nwaves = (long)gridDim.x * kWaves;
    const float count = (float)n;
    for (long r = wave; r < rows; r += nwaves) {
        const float total = wave_sum(stream_sum(x + r * n, n, lane, [](long, float v) { return v; }));
        if (lane == 0) y[r] = pad_div_off(total, count, o.off, o.has);
    }
}

// ---------------------------------------------------------------- layer_norm forward (pam/pam_ops.py:350-378)
// The weight and bias elements of a lane are the same for every row it works on.  KEEP: they are read once and stay in
// registers (rows of few values per lane, where a read per row and element -- each waited for where it is used, in the
// middle of the row's chain -- was most of a row's time); else they are read per row, from cache.
template <int CH, bool KEEP>
struct RowParams {
    const float* __restrict__ weight; const float* __restrict__ bias;
    float w[KEEP ? CH : 1], b[KEEP ? CH : 1];
    template <class L>
    __device__ __forceinline__ void fetch(const L& lay, long n)
    {
        if constexpr (KEEP) {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const long i = lay.index(c);
                w[c] = (weight && i < n) ? weight[i] : 1.0f;
                b[c] = (bias && i < n) ? bias[i] : 0.0f;
            }
        }
    }
    __device__ __forceinline__ float weight_at(int c, long i, bool inside) const
    {
        if constexpr (KEEP) return w[c]; else return inside ? weight[i] : 1.0f;
    }
    __device__ __forceinline__ float bias_at(int c, long i, bool inside) const
    {
        if constexpr (KEEP) return b[c]; else return inside ? bias[i] : 0.0f;
    }
};
constexpr int kKeepForward = 16;       // values per lane up to which the forward kernels keep them (the gradient kernels have
                                       // no registers to spare: with them kept, rows of 197 values ran 40 % slower)

template <int CH, class M, class L, class P>
__device__ __forceinline__ void layer_norm_row(float (&v)[CH], const P& par, L& lay, long n, float count, float eps, M& m)
{
    // in place: inputs, then centred values, then results (one array of registers per row)
    float p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) p = p + v[c];                           // the fill adds +0
    const float mu = m.div(lay.sum(p), count);
    p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        v[c] = v[c] - mu;                                                // lanes past the end hold -mu, a stand-in
        const float sq = m.square(v[c]);
        if (lay.index(c) < n) p = p + sq;
    }
    const float denom = m.root(m.div(lay.sum(p), count) + eps);         // a result of exp2 (or the zero of the power): never negative
    m.record(denom);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const long i = lay.index(c); const bool inside = i < n;
        float r = m.div_by_positive(v[c], denom);                        // the centred value was recorded by square()
        if (par.weight) r = m.mul_seen(r, par.weight_at(c, i, inside));
        if (par.bias) r = r + par.bias_at(c, i, inside);
        v[c] = r;
    }
}

template <int CH>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(PAM_ROW_OCC(CH)))) void layer_norm_fwd_kernel(const float* __restrict__ x, const float* __restrict__ weight,
                                                                 const float* __restrict__ bias, float* __restrict__ y,
                                                                 long rows, long n, float eps, Offset o)
{
    const int lane = threadIdx.x % 64;
    const long wave = (long)blockIdx.x * kWaves + threadIdx.x / 64, nwaves = (long)gridDim.x * kWaves;
    const float count = (float)n;
    float ahead[CH > 0 ? CH : 1];
    constexpr bool kAhead = false;                         // measured slower with it
    PAM_WAVE_FIRST_ROW(kAhead, ahead, x, 0.0f);
    RowParams<(CH > 0 ? CH : 1), (CH > 0 && CH <= kKeepForward)> par{weight, bias};
    if constexpr (CH > 0) par.fetch(WaveRow{lane}, n);
    for (long r = wave; r < rows; r += nwaves) {
        const float* xr = x + r * n; float* yr = y + r * n;
        if constexpr (CH > 0) {
            float v[CH];
            PAM_WAVE_NEXT_ROW(kAhead, v, ahead, x, 0.0f);
            WaveRow lay{lane};
            UncheckedFor<kLayerNormFwd, CH, false> u{o, Span()};
            layer_norm_row<CH>(v, par, lay, n, count, eps, u);
            if (!wave_valid(u)) {                              // the row is read again (from cache)
                load_row<CH>(v, xr, n, lane, 0.0f);
                Checked k{o}; layer_norm_row<CH>(v, par, lay, n, count, eps, k);
            }
            store_row<CH>(v, yr, n, lay);
        } else {
            auto sweep = [&](auto& m) {
                float p = 0.0f;
                for_blocks(xr, (int)n, lane, 0.0f, [&](long, bool, float v) { p = p + v; });            // the fill adds +0
                const float mu = m.div(wave_sum(p), count);
                p = 0.0f;
                for_blocks(xr, (int)n, lane, 0.0f, [&](long, bool inside, float v) {
                    const float c = v - mu, sq = m.square(c);                                    // past the end: -mu, a stand-in
                    if (inside) p = p + sq;
                });
                const float denom = m.root(m.div(wave_sum(p), count) + eps);
                m.record(denom);
                for_blocks(xr, (int)n, lane, 0.0f, [&](long i, bool inside, float v) {
                    float r = m.div_by_positive(v - mu, denom);                                  // v - mu was recorded by square()
                    if (weight) r = m.mul_seen(r, inside ? weight[i] : 1.0f);
                    if (bias) r = r + (inside ? bias[i] : 0.0f);
                    if (inside) yr[i] = r;
                });
            };
            UncheckedFor<kLayerNormFwd, CH, false> u{o, Span()};
            sweep(u);
            if (!wave_valid(u)) { Checked k{o}; sweep(k); }
        }
    }
}

// ---------------------------------------------------------------- gradients of logsumexp / log_softmax and layer_norm
// Autograd's chain over the unfused ops, written out (pam/cuda_bindings.py:43-57, 78-97, 224-239,
// 262-276 for the formulas; pam/pam_ops.py:331-378 for the ops).  Rows of up to 1024 values stay in
// registers; longer rows are swept several times (the later sweeps find the row in cache).
// GradChecked serves every combination of exact and approximate gradients;
// GradUncheckedT is the all-approximate chain on the branch-free primitives, tried first and kept
// when every value it touched was a normal number.
struct GradChecked {
    static constexpr bool kOffsets = true, kApproxUnchecked = false;
    Offset o; Approx ap;
    __device__ __forceinline__ float mul(float a, float b) { return pam_mul_off(a, b, o.off, o.has); }
    __device__ __forceinline__ float div(float a, float b) { return pad_div_off(a, b, o.off, o.has); }
    __device__ __forceinline__ float exp2(float t) { return exp2_entry(t, o.off, o.has); }
    __device__ __forceinline__ float log2(float v) { return log2_entry(v, o.off, o.has); }
    // gradient for the first / second operand of c = a (*) b
    __device__ __forceinline__ float mul_da(float a, float b, float g) { return ap.a ? mul(g, b) : pam_mul_bwd(a, b, g, o.off, o.has); }
    __device__ __forceinline__ float mul_db(float a, float b, float g) { return ap.b ? mul(g, a) : pam_mul_bwd(b, a, g, o.off, o.has); }
    // gradient for the first / second operand of c = a (/) b
    __device__ __forceinline__ float div_da(float a, float b, float g)
    { const float inv = div(1.0f, b); return ap.a ? mul(inv, g) : pam_mul_bwd(a, inv, g, 1.0f, false); }
    __device__ __forceinline__ float div_db(float a, float b, float g)
    { return ap.b ? -mul(div(div(a, b), b), g) : pad_div_bwd(a, b, g, o.off, o.has); }
    __device__ __forceinline__ float exp2_dx(float x, float g)
    { return ap.e ? mul(mul(exp2(x), kLn2), g) : exp2_entry_bwd(x, g, o.off, o.has); }
    __device__ __forceinline__ float log2_dx(float x, float g)
    { return ap.e ? div(div(g, x), kLn2) : log2_entry_bwd(x, g, o.off, o.has); }
    // logsumexp's log2 of the row total: called without the keyword arguments (pam/pam_ops.py:341), so it takes no
    // offset and its gradient is the exact one whatever approx_bwd says
    __device__ __forceinline__ float log2_plain(float v) { return log2_entry(v, 1.0f, false); }
    __device__ __forceinline__ float log2_plain_dx(float x, float g) { return log2_entry_bwd(x, g, 1.0f, false); }
    __device__ __forceinline__ bool valid() const { return true; }
};
// the exact gradient of log2 without an offset in the normal range: 2^-e(x) g (pam/cuda_kernels.cu:132-136)
__device__ __forceinline__ float log2_exact_dx_unchecked(float x, float g, Span& sp)
{
    const uint32_t xi = f2u(x);                                            // positive (a sign bit reads as too large), below 2^127
    sp.see(xi); sp.see(xi + 0x00800000u);
    return u2f((254u << 23) - (xi & kExpo)) * g;
}
template <bool OFFSETS>
struct GradUncheckedT {
    static constexpr bool kOffsets = OFFSETS, kApproxUnchecked = true;
    Offset o; Span sp;
    __device__ __forceinline__ float mul(float a, float b) { return pam_unchecked_off(a, b, o.off, OFFSETS && o.has, sp); }
    __device__ __forceinline__ float div(float a, float b) { return pad_unchecked_off(a, b, o.off, OFFSETS && o.has, sp); }
    __device__ __forceinline__ float exp2(float t) { return exp2_entry_unchecked(t, o.off, OFFSETS && o.has, sp); }
    __device__ __forceinline__ float log2(float v) { return log2_entry_unchecked(v, o.off, OFFSETS && o.has, sp); }
    __device__ __forceinline__ float mul_da(float, float b, float g) { return mul(g, b); }
    __device__ __forceinline__ float mul_db(float a, float, float g) { return mul(g, a); }
    __device__ __forceinline__ float div_da(float, float b, float g) { return mul(div(1.0f, b), g); }
    __device__ __forceinline__ float div_db(float a, float b, float g) { return -mul(div(div(a, b), b), g); }
    __device__ __forceinline__ float exp2_dx(float x, float g) { return mul(mul(exp2(x), kLn2), g); }
    __device__ __forceinline__ float log2_dx(float x, float g) { return div(div(g, x), kLn2); }
    __device__ __forceinline__ float log2_plain(float v) { return log2_entry_unchecked(v, 1.0f, false, sp); }
    __device__ __forceinline__ float log2_plain_dx(float x, float g) { return log2_exact_dx_unchecked(x, g, sp); }
    __device__ __forceinline__ bool usable() const { return OFFSETS || !o.has; }         // (the same for every lane of a launch)
    __device__ __forceinline__ bool valid() const { return usable() && sp.normal(); }
};
template <RowKernel K, int CH, bool BLOCK> using GradUncheckedFor = GradUncheckedT<fast_path_offsets<K, CH, BLOCK>()>;

// The all-exact gradients (the reference's default) without an offset, on unchecked arithmetic.  In the normal range
// the exact backward formulas are short (pam/cuda_kernels.cu:40-58, 85-97, 115-123, 132-136): the gradient of a (*) b
// for a is g 2^(e(b) + carry of the two fractions) with b's sign, i.e. the bits of b plus the fraction bits of a masked
// to sign and exponent; of a (/) b for b, -(2^e(a (/) b) / 2^e(b)) g, a difference of exponent fields; of exp2,
// 2^e(exp2 x) g; of log2, 2^-e(x) g.  The products with the upstream gradients are IEEE products in the checked forms
// too, so the gradients need no recording; the other operands are recorded, with the extra headroom the carries need.
struct GradUncheckedExact {
    static constexpr bool kOffsets = false, kApproxUnchecked = false;
    Offset o; Span sp;                            // used without an offset only
    __device__ __forceinline__ float mul(float a, float b) { return pam_unchecked(a, b, sp); }
    __device__ __forceinline__ float div(float a, float b) { return pad_unchecked(a, b, sp); }
    __device__ __forceinline__ float exp2(float t) { return exp2_entry_unchecked(t, 1.0f, false, sp); }
    __device__ __forceinline__ float log2(float v) { return log2_entry_unchecked(v, 1.0f, false, sp); }
    __device__ __forceinline__ float mul_da(float a, float b, float g)
    {
        const uint32_t ai = f2u(a), bi = f2u(b), mb = bi & ~kSign;
        sp.see(ai & ~kSign); sp.see(mb); sp.see(mb + 0x00800000u);             // b below 2^127: the carry fits
        return g * u2f((bi + (ai & kMant)) & ~kMant);
    }
    __device__ __forceinline__ float mul_db(float a, float b, float g) { return mul_da(b, a, g); }
    __device__ __forceinline__ float div_da(float a, float b, float g) { return mul_da(a, div(1.0f, b), g); }
    __device__ __forceinline__ float div_db(float a, float b, float g)
    {
        const uint32_t oi = f2u(div(a, b));
        const uint32_t ratio = (oi & kExpo) - (f2u(b) & kExpo) + kBias;        // a wrap lands above the exponent mask and is caught
        sp.see(ratio);
        return -u2f(ratio | (oi & kSign)) * g;
    }
    __device__ __forceinline__ float exp2_dx(float x, float g) { return u2f(f2u(exp2(x)) & ~kMant) * g; }
    __device__ __forceinline__ float log2_dx(float x, float g) { return log2_exact_dx_unchecked(x, g, sp); }
    __device__ __forceinline__ float log2_plain(float v) { return log2(v); }
    __device__ __forceinline__ float log2_plain_dx(float x, float g) { return log2_dx(x, g); }
    __device__ __forceinline__ bool usable() const { return true; }
    __device__ __forceinline__ bool valid() const { return sp.normal(); }
};

// One row of the logsumexp / log_softmax gradient.  xv: the inputs (any fill past the end); gy: the
// per-element gradients (log_softmax) with 1.0 past the end; out: dx.  Lanes past the end of the
// row work on stand-in values that are never stored or summed.
template <int CH, class G, class L>
__device__ __forceinline__ void logsumexp_grad_row(const float (&xv)[CH], const float (&gy)[CH], float (&out)[CH], float g_row,
                                                   bool log_softmax, float shift, L& lay, long n, G& m)
{
    float p = 0.0f, q = 0.0f, t[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const bool inside = lay.index(c) < n;
        const float s = m.mul(inside ? xv[c] : 1.0f, kLog2E) - shift;
        t[c] = inside ? s : 0.5f;
        const float e = m.exp2(t[c]);
        if (inside) { p = p + e; q = q + gy[c]; }
    }
    const float total = lay.sum(p);
    const float g_out = log_softmax ? -lay.sum(q) : g_row;         // log_softmax is the same for every thread of a launch         // x - lse: the broadcast lse collects -sum(gy)
    const float u = shift + m.log2_plain(total);
    const float du = m.div_da(u, kLog2E, g_out);
    const float dtotal = m.log2_plain_dx(total, du);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const bool inside = lay.index(c) < n;
        const float d = m.mul_da(inside ? xv[c] : 1.0f, kLog2E, m.exp2_dx(t[c], dtotal));
        out[c] = log_softmax ? gy[c] + d : d;
    }
}

// dx of out = logsumexp(x) (per row, gradient g_out) or of y = x - logsumexp(x) (gradient gy per element)
template <int CH, bool EXACT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(PAM_ROW_OCC_GRAD(CH)))) void logsumexp_bwd_kernel(
    const float* __restrict__ x, const float* __restrict__ grad, const float* __restrict__ shift_in, float* __restrict__ dx,
    long rows, long n, int log_softmax, Offset o, Approx ap)
{
    const int lane = threadIdx.x % 64;
    const long wave = (long)blockIdx.x * kWaves + threadIdx.x / 64, nwaves = (long)gridDim.x * kWaves;
    const float shift = *shift_in;
    for (long r = wave; r < rows; r += nwaves) {
        float xv[CH], gy[CH], out[CH];
        load_row<CH>(xv, x + r * n, n, lane, 0.0f);
#pragma unroll
        for (int c = 0; c < CH; ++c) gy[c] = 1.0f;
        if (log_softmax) load_row<CH>(gy, grad + r * n, n, lane, 1.0f);
        const float g_row = log_softmax ? 0.0f : grad[r];
        bool done = false;
        WaveRow lay{lane};
        if (EXACT || (ap.a && ap.b && ap.e)) {         // EXACT: the host chose this instance for all-exact gradients without an offset
            typename std::conditional<EXACT, GradUncheckedExact, GradUncheckedFor<kLogsumexpBwd, CH, false>>::type u{o, Span()};
            logsumexp_grad_row<CH>(xv, gy, out, g_row, log_softmax != 0, shift, lay, n, u);
            done = __ballot(!u.valid()) == 0ull;
        }
        if (!done) { GradChecked k{o, ap}; logsumexp_grad_row<CH>(xv, gy, out, g_row, log_softmax != 0, shift, lay, n, k); }
#pragma unroll
        for (int c = 0; c < CH; ++c) { const long i = lane + 64L * c; if (i < n) dx[r * n + i] = out[c]; }
    }
}

// The same gradient for rows too long for registers: two sweeps over the row in blocks of 64 x U
// values (the second sweep finds the row in cache).  A lane meets its elements in the same ascending
// order as in the register variant, so the sums are the same sums.
template <class G>
__device__ __forceinline__ void logsumexp_grad_stream(const float* __restrict__ xr, const float* __restrict__ gr, float* __restrict__ dr,
                                                      float g_row, bool log_softmax, float shift, int lane, long rowlen, G& m)
{
    const int n = (int)rowlen;                    // at most 2^30: 32-bit index arithmetic
    constexpr int U = 8;
    float p = 0.0f, q = 0.0f;
    for (int base = 0; base < n; base += 64 * U) {
        float xv[U], gy[U];
#pragma unroll
        for (int c = 0; c < U; ++c) {
            const int i = base + lane + 64 * c; const bool inside = i < n;
            xv[c] = inside ? xr[i] : 1.0f;
            gy[c] = (inside && log_softmax) ? gr[i] : 0.0f;
        }
#pragma unroll
        for (int c = 0; c < U; ++c) {
            const bool inside = base + lane + 64 * c < n;
            const float sc = m.mul(xv[c], kLog2E) - shift;
            const float e = m.exp2(inside ? sc : 0.5f);
            if (inside) { p = p + e; q = q + gy[c]; }
        }
    }
    const float total = wave_sum(p);
    const float g_out = log_softmax ? -wave_sum(q) : g_row;
    const float u = shift + m.log2_plain(total);
    const float du = m.div_da(u, kLog2E, g_out);
    const float dtotal = m.log2_plain_dx(total, du);
    for (int base = 0; base < n; base += 64 * U) {
        float xv[U], gy[U];
#pragma unroll
        for (int c = 0; c < U; ++c) {
            const int i = base + lane + 64 * c; const bool inside = i < n;
            xv[c] = inside ? xr[i] : 1.0f;
            gy[c] = (inside && log_softmax) ? gr[i] : 0.0f;
        }
#pragma unroll
        for (int c = 0; c < U; ++c) {
            const int i = base + lane + 64 * c; const bool inside = i < n;
            const float sc = m.mul(xv[c], kLog2E) - shift;
            const float d = m.mul_da(xv[c], kLog2E, m.exp2_dx(inside ? sc : 0.5f, dtotal));
            if (inside) dr[i] = log_softmax ? gy[c] + d : d;
        }
    }
}

template <bool EXACT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(PAM_ROW_WAVES))) void logsumexp_bwd_stream_kernel(
    const float* __restrict__ x, const float* __restrict__ grad, const float* __restrict__ shift_in, float* __restrict__ dx,
    long rows, long n, int log_softmax, Offset o, Approx ap)
{
    const int lane = threadIdx.x % 64;
    const long wave = (long)blockIdx.x * kWaves + threadIdx.x / 64, nwaves = (long)gridDim.x * kWaves;
    const float shift = *shift_in;
    for (long r = wave; r < rows; r += nwaves) {
        const float* gr = log_softmax ? grad + r * n : nullptr;
        const float g_row = log_softmax ? 0.0f : grad[r];
        bool done = false;
        if (EXACT || (ap.a && ap.b && ap.e)) {         // EXACT: the host chose this instance for all-exact gradients without an offset
            typename std::conditional<EXACT, GradUncheckedExact, GradUncheckedFor<kLogsumexpBwd, 0, false>>::type u{o, Span()};
            logsumexp_grad_stream(x + r * n, gr, dx + r * n, g_row, log_softmax != 0, shift, lane, n, u);
            done = __ballot(!u.valid()) == 0ull;
        }
        if (!done) { GradChecked k{o, ap}; logsumexp_grad_stream(x + r * n, gr, dx + r * n, g_row, log_softmax != 0, shift, lane, n, k); }
    }
}

// Which instances of the layer_norm gradient take the cheaper forms (see layer_norm_grad_row): by measurement.
template <int CH, class L>
constexpr bool layer_norm_grad_cheap() { return true; }

// One row of the layer_norm gradient.  cen: x on entry, overwritten; g: dy on entry (1.0 past the
// end), dx on exit; terms: the per-element terms of the weight gradient (if weight).
template <int CH, class G, class L, class P>
__device__ __forceinline__ void layer_norm_grad_row(float (&cen)[CH], float (&g)[CH], float (&terms)[CH],
                                                    const P& par, L& lay, long n, float count, float eps, G& m)
{
    // The all-approximate chain without an offset, on the cheaper forms of the unchecked primitives where an operand is
    // the row's positive denominator (recorded once), a value the chain has recorded already, or the same product twice:
    // the same bits, fewer magnitudes to record and fewer products.  In the instances where that measured faster.
    if constexpr (G::kApproxUnchecked && !G::kOffsets && layer_norm_grad_cheap<CH, L>()) {
        float p = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; ++c) p = p + cen[c];
        const float s1 = lay.sum(p);
        const float mu = m.div(s1, count);
        p = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; ++c) { cen[c] = cen[c] - mu; const float sq = pam_unchecked_square(cen[c], m.sp); if (lay.index(c) < n) p = p + sq; }
        const float s2 = lay.sum(p);
        const float v = m.div(s2, count) + eps;
        const float lg = m.log2(v);
        const float half = m.mul(lg, 0.5f);
        const float root = m.exp2(half);
        const float denom = v == 0.0f ? 0.0f : root;
        m.sp.see(f2u(denom) & ~kSign);
        const float inv = m.div(1.0f, denom);
        p = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const long i = lay.index(c); const bool inside = i < n;
            const float xn = pad_unchecked_by_positive(cen[c], denom, m.sp);           // (the centred value was recorded by its square)
            if (par.weight) {
                const float wi = par.weight_at(c, i, inside);
                terms[c] = pam_unchecked_seen(xn, g[c], m.sp);
                g[c] = m.mul(g[c], wi);
            }
            const float d = -pam_unchecked_seen(pad_unchecked_by_positive(xn, denom, m.sp), g[c], m.sp);
            if (inside) p = p + d;
        }
        float d = lay.sum(p);
        if (v == 0.0f) d = 0.0f;
        d = m.exp2_dx(half, d);
        d = m.mul_da(lg, 0.5f, d);
        d = m.log2_dx(v, d);
        const float ds2 = m.div_da(s2, count, d);
        p = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            float dc = pam_unchecked_seen(inv, g[c], m.sp);
            const float t = pam_unchecked_seen(cen[c], ds2, m.sp);                      // both operands of c (*) c get this gradient
            dc = dc + t;
            dc = dc + t;
            g[c] = dc;
            if (lay.index(c) < n) p = p + dc;
        }
        const float ds1 = m.div_da(s1, count, -lay.sum(p));
#pragma unroll
        for (int c = 0; c < CH; ++c) g[c] = g[c] + ds1;
        return;
    }
    float p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) p = p + cen[c];                        // the fill adds +0
    const float s1 = lay.sum(p);
    const float mu = m.div(s1, count);
    p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) { cen[c] = cen[c] - mu; const float sq = m.mul(cen[c], cen[c]); if (lay.index(c) < n) p = p + sq; }
    const float s2 = lay.sum(p);
    const float v = m.div(s2, count) + eps;
    const float lg = m.log2(v);
    const float half = m.mul(lg, 0.5f);
    const float root = m.exp2(half);
    const float denom = v == 0.0f ? 0.0f : root;
    // through the weight product and the quotient; the row sum for the broadcast denominator
    p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const long i = lay.index(c); const bool inside = i < n;
        if (par.weight) {
            const float xn = m.div(cen[c], denom), wi = par.weight_at(c, i, inside);
            terms[c] = m.mul_db(xn, wi, g[c]);
            g[c] = m.mul_da(xn, wi, g[c]);
        }
        const float d = m.div_db(cen[c], denom, g[c]);
        if (inside) p = p + d;
    }
    float d = lay.sum(p);
    if (v == 0.0f) d = 0.0f;                                            // where(v == 0, 0, exp2(..))
    d = m.exp2_dx(half, d);
    d = m.mul_da(lg, 0.5f, d);
    d = m.log2_dx(v, d);                                                // = d var
    const float ds2 = m.div_da(s2, count, d);
    // gradients reaching the centred values: quotient, then the two operands of c (*) c
    p = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        float dc = m.div_da(cen[c], denom, g[c]);
        dc = dc + m.mul_da(cen[c], cen[c], ds2);
        dc = dc + m.mul_db(cen[c], cen[c], ds2);
        g[c] = dc;
        if (lay.index(c) < n) p = p + dc;
    }
    const float ds1 = m.div_da(s1, count, -lay.sum(p));                // mu is subtracted: it collects -sum(dc)
#pragma unroll
    for (int c = 0; c < CH; ++c) g[c] = g[c] + ds1;
}

// The same gradient for rows too long for registers: five sweeps over the row (sum, sum of squares, the
// denominator's gradient, the centred values' gradients and their sum, the final add); after the first sweep
// the row comes from cache.  A lane meets its elements in the same ascending order as in the register
// variant, so the three row sums are the same sums.  dx holds the centred values' gradients between the
// last two sweeps (each lane re-reads only what it wrote itself).
template <class G>
__device__ __forceinline__ void layer_norm_grad_stream(const float* __restrict__ xr, const float* __restrict__ gr,
                                                       const float* __restrict__ weight, float* __restrict__ dr,
                                                       float* __restrict__ tr, int lane, long rowlen, float count, float eps, G& m)
{
    const int n = (int)rowlen;                    // at most 2^30: 32-bit index arithmetic
    float p = 0.0f;
#pragma unroll 4
    for (int i = lane; i < n; i += 64) p = p + xr[i];
    const float s1 = wave_sum(p);
    const float mu = m.div(s1, count);
    p = 0.0f;
#pragma unroll 4
    for (int i = lane; i < n; i += 64) { const float c = xr[i] - mu; p = p + m.mul(c, c); }
    const float s2 = wave_sum(p);
    const float v = m.div(s2, count) + eps;
    const float lg = m.log2(v);
    const float half = m.mul(lg, 0.5f);
    const float root = m.exp2(half);
    const float denom = v == 0.0f ? 0.0f : root;
    // the upstream gradient behind the weight product (and that product's term for the weight gradient)
    auto behind_weight = [&](int i, float c, bool store_term) {
        float g = gr[i];
        if (weight) {
            const float xn = m.div(c, denom), wi = weight[i];
            if (store_term && tr) tr[i] = m.mul_db(xn, wi, g);
            g = m.mul_da(xn, wi, g);
        }
        return g;
    };
    p = 0.0f;
#pragma unroll 4
    for (int i = lane; i < n; i += 64) {
        const float c = xr[i] - mu;
        p = p + m.div_db(c, denom, behind_weight(i, c, true));
    }
    float d = wave_sum(p);
    if (v == 0.0f) d = 0.0f;
    d = m.exp2_dx(half, d);
    d = m.mul_da(lg, 0.5f, d);
    d = m.log2_dx(v, d);
    const float ds2 = m.div_da(s2, count, d);
    p = 0.0f;
#pragma unroll 4
    for (int i = lane; i < n; i += 64) {
        const float c = xr[i] - mu;
        float dc = m.div_da(c, denom, behind_weight(i, c, false));
        dc = dc + m.mul_da(c, c, ds2);
        dc = dc + m.mul_db(c, c, ds2);
        dr[i] = dc;
        p = p + dc;
    }
    const float ds1 = m.div_da(s1, count, -wave_sum(p));
#pragma unroll 4
    for (int i = lane; i < n; i += 64) dr[i] = dr[i] + ds1;
}

template <bool EXACT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(PAM_ROW_WAVES))) void layer_norm_bwd_stream_kernel(
    const float* __restrict__ x, const float* __restrict__ weight, const float* __restrict__ gy, float* __restrict__ dx,
    float* __restrict__ dw_terms, long rows, long n, float eps, Offset o, Approx ap)
{
    const int lane = threadIdx.x % 64;
    const long wave = (long)blockIdx.x * kWaves + threadIdx.x / 64, nwaves = (long)gridDim.x * kWaves;
    const float count = (float)n;
    for (long r = wave; r < rows; r += nwaves) {
        float* tr = (weight && dw_terms) ? dw_terms + r * n : nullptr;
        bool done = false;
        if (EXACT || (ap.a && ap.b && ap.e)) {         // EXACT: the host chose this instance for all-exact gradients without an offset
            typename std::conditional<EXACT, GradUncheckedExact, GradUncheckedFor<kLayerNormBwd, 0, false>>::type u{o, Span()};
            layer_norm_grad_stream(x + r * n, gy + r * n, weight, dx + r * n, tr, lane, n, count, eps, u);
            done = __ballot(!u.valid()) == 0ull;
        }
        if (!done) { GradChecked k{o, ap}; layer_norm_grad_stream(x + r * n, gy + r * n, weight, dx + r * n, tr, lane, n, count, eps, k); }
    }
}

// dx and the per-element weight-gradient terms of y = layer_norm(x) * weight + bias.  Rows of 1024 values (and of 768
// for the exact chain, by measurement): three wavefronts per SIMD (168 registers); left at two the compiler takes 181
// and a third fewer wavefronts fit.
template <int CH, bool EXACT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(((CH) >= 16 || ((CH) >= 12 && EXACT)) ? 3 : ((CH) <= 4 ? 6 : PAM_ROW_WAVES)))) void layer_norm_bwd_kernel(
    const float* __restrict__ x, const float* __restrict__ weight, const float* __restrict__ gy, float* __restrict__ dx,
    float* __restrict__ dw_terms, long rows, long n, float eps, Offset o, Approx ap)
{
    const int lane = threadIdx.x % 64;
    const long wave = (long)blockIdx.x * kWaves + threadIdx.x / 64, nwaves = (long)gridDim.x * kWaves;
    const float count = (float)n;
    RowParams<CH, false> par{weight, nullptr};
    for (long r = wave; r < rows; r += nwaves) {
        float cen[CH], g[CH], terms[CH];
        bool done = false;
        WaveRow lay{lane};
        if (EXACT || (ap.a && ap.b && ap.e)) {
            load_row<CH>(cen, x + r * n, n, lane, 0.0f);
            load_row<CH>(g, gy + r * n, n, lane, 1.0f);
            typename std::conditional<EXACT, GradUncheckedExact, GradUncheckedFor<kLayerNormBwd, CH, false>>::type u{o, Span()};
            layer_norm_grad_row<CH>(cen, g, terms, par, lay, n, count, eps, u);
            done = __ballot(!u.valid()) == 0ull;
        }
        if (!done) {                                    // the row is read again (from cache) rather than kept in registers
            load_row<CH>(cen, x + r * n, n, lane, 0.0f);
            load_row<CH>(g, gy + r * n, n, lane, 1.0f);
            GradChecked k{o, ap};
            layer_norm_grad_row<CH>(cen, g, terms, par, lay, n, count, eps, k);
        }
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const long i = lane + 64L * c;
            if (i < n) { dx[r * n + i] = g[c]; if (weight && dw_terms) dw_terms[r * n + i] = terms[c]; }
        }
    }
}

// ---------------------------------------------------------------- a work-group per row (rows of 4097 ... 16384 values)
// One row is held in the registers of 1024 threads (CH values each), read once and written once; the row functions
// are the ones above, with the work-group's sum in place of the wavefront's.  Whether the unchecked arithmetic
// was valid is decided for the whole row, so that every thread takes the same path to the next barrier.
#ifdef PAM_BLOCK_WAVES
#define PAM_BLOCK_ATTR __attribute__((amdgpu_waves_per_eu(PAM_BLOCK_WAVES)))
#else
#define PAM_BLOCK_ATTR
#endif
// The forward kernels, which hold one array of registers per row: the input row of the next iteration is fetched
// while the current one is computed (there is one work-group per compute unit, so nothing else would hide the
// latency; the gradient kernels have no registers to spare for it).  Past the last row the fetch repeats the last row:
// a conditional fetch would tie the registers to their old contents and make the compiler wait for them at once.
#define PAM_BLOCK_FIRST_ROW(ON, AHEAD, X, FILL) \
    if constexpr (ON) load_row<CH>(AHEAD, X + (blockIdx.x < rows ? (long)blockIdx.x : rows - 1) * n, n, lay, FILL)
#define PAM_BLOCK_NEXT_ROW(ON, NOW, AHEAD, X, FILL)                                                      \
    if constexpr (ON) {                                                                                  \
        _Pragma("unroll") for (int c = 0; c < CH; ++c) NOW[c] = AHEAD[c];                                \
        load_row<CH>(AHEAD, X + (r + gridDim.x < rows ? r + gridDim.x : rows - 1) * n, n, lay, FILL);    \
    } else load_row<CH>(NOW, X + r * n, n, lay, FILL)
#define PAM_BLOCK_ROW_SETUP                                                        \
    __shared__ float red_slots[2][kBlockWaves];                                    \
    BlockRow lay{(int)threadIdx.x, red_slots, 0};                                  \
    const int lane = threadIdx.x % 64;                                             \
    (void)lane

// Up to 12 values per thread the kernel fits 64 registers: two work-groups per compute unit.
template <int CH>
__global__ __launch_bounds__(kBlockThreads) __attribute__((amdgpu_waves_per_eu(CH <= 12 ? 8 : 4))) void softmax_fwd_block_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                         float* __restrict__ row_sum, float* __restrict__ shift_out,
                                                                         long rows, long n, Offset o,
                                                                         const float* __restrict__ partial, int partials)
{
    PAM_BLOCK_ROW_SETUP;
    float ahead[CH];
    constexpr bool kAhead = CH >= 16;
    PAM_BLOCK_FIRST_ROW(kAhead, ahead, x, kNegInf);
    const float shift = fold_shift<kBlockWaves>(partial, partials);
    if (blockIdx.x == 0 && threadIdx.x == 0) *shift_out = shift;
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        float v[CH];
        PAM_BLOCK_NEXT_ROW(kAhead, v, ahead, x, kNegInf);
        UncheckedFor<kSoftmaxFwd, CH, true> u{o, Span()};
        float total = softmax_row<CH>(v, shift, u, lay);
        if (!lay.all(u.valid())) {                             // the row is read again (from cache)
            load_row<CH>(v, x + r * n, n, lay, kNegInf);
            Checked k{o}; total = softmax_row<CH>(v, shift, k, lay);
        }
        store_row<CH>(v, y + r * n, n, lay);
        if (threadIdx.x == 0) row_sum[r] = total;
    }
}

template <int CH, bool EXACT>
__global__ __launch_bounds__(kBlockThreads) PAM_BLOCK_ATTR void softmax_bwd_block_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                                         const float* __restrict__ row_sum, const float* __restrict__ shift_in,
                                                                         float* __restrict__ dx, long rows, long n, Offset o, Approx ap)
{
    PAM_BLOCK_ROW_SETUP;
    const float shift = *shift_in;
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        const float total = row_sum[r];
        float xv[CH], g[CH], out[CH];
        load_row<CH>(xv, x + r * n, n, lay, kNegInf);
        load_row<CH>(g, dy + r * n, n, lay, 0.0f);
        bool done = false;
        if (EXACT) {
            UncheckedFor<kSoftmaxBwdExact, CH, true> u{o, Span()};
            softmax_grad_row_exact<CH>(xv, g, out, total, shift, lay, n, u);
            done = lay.all(u.valid());
        } else if (ap.a && ap.b && ap.e) {
            UncheckedFor<kSoftmaxBwd, CH, true> u{o, Span()};
            softmax_grad_row_approx<CH>(xv, g, out, total, shift, lay, n, u);
            done = lay.all(u.valid());
        }
        if (!done) softmax_grad_row_checked<CH>(xv, g, out, total, pad_div_off(1.0f, total, o.off, o.has), shift, lay, n, o, ap);
        store_row<CH>(out, dx + r * n, n, lay);
    }
}

template <int CH>
__global__ __launch_bounds__(kBlockThreads) PAM_BLOCK_ATTR void logsumexp_block_kernel(const float* __restrict__ x, float* __restrict__ lse,
                                                                       float* __restrict__ y, float* __restrict__ shift_out, long rows, long n,
                                                                       Offset o, const float* __restrict__ partial, int partials)
{
    PAM_BLOCK_ROW_SETUP;
    float ahead[CH];
    constexpr bool kAhead = CH < 16;                       // sixteen values per thread twice over would spill
    PAM_BLOCK_FIRST_ROW(kAhead, ahead, x, 0.0f);
    const float shift = fold_shift<kBlockWaves>(partial, partials);
    if (shift_out && blockIdx.x == 0 && threadIdx.x == 0) *shift_out = shift;
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        float xv[CH];
        PAM_BLOCK_NEXT_ROW(kAhead, xv, ahead, x, 0.0f);
        UncheckedFor<kLogsumexpFwd, CH, true> u{o, Span()};
        float out = logsumexp_row<CH>(xv, shift, lay, n, u);
        if (!lay.all(u.valid())) { Checked k{o}; out = logsumexp_row<CH>(xv, shift, lay, n, k); }
        if (lse && threadIdx.x == 0) lse[r] = out;
        if (y) {
#pragma unroll
            for (int c = 0; c < CH; ++c) { const long i = lay.index(c); if (i < n) y[r * n + i] = xv[c] - out; }
        }
    }
}

__global__ __launch_bounds__(kBlockThreads) PAM_BLOCK_ATTR void row_mean_block_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                      long rows, long n, Offset o)
{
    PAM_BLOCK_ROW_SETUP;
    const float count = (float)n;
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        const float* xr = x + r * n;
        float p = 0.0f;
#pragma unroll 4
        for (long i = threadIdx.x; i < n; i += kBlockThreads) p = p + xr[i];
        const float total = lay.sum(p);
        if (threadIdx.x == 0) y[r] = pad_div_off(total, count, o.off, o.has);
    }
}

template <int CH>
__global__ __launch_bounds__(kBlockThreads) PAM_BLOCK_ATTR void layer_norm_fwd_block_kernel(const float* __restrict__ x, const float* __restrict__ weight,
                                                                            const float* __restrict__ bias, float* __restrict__ y,
                                                                            long rows, long n, float eps, Offset o)
{
    PAM_BLOCK_ROW_SETUP;
    const float count = (float)n;
    float ahead[CH];
    constexpr bool kAhead = CH < 16;                       // (rows of 10000 values: 91 -> 83 us for 4096 of them)
    PAM_BLOCK_FIRST_ROW(kAhead, ahead, x, 0.0f);
    RowParams<CH, (CH <= kKeepForward)> par{weight, bias};
    par.fetch(lay, n);
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        float v[CH];
        PAM_BLOCK_NEXT_ROW(kAhead, v, ahead, x, 0.0f);
        UncheckedFor<kLayerNormFwd, CH, true> u{o, Span()};
        layer_norm_row<CH>(v, par, lay, n, count, eps, u);
        if (!lay.all(u.valid())) {                             // the row is read again (from cache)
            load_row<CH>(v, x + r * n, n, lay, 0.0f);
            Checked k{o}; layer_norm_row<CH>(v, par, lay, n, count, eps, k);
        }
        store_row<CH>(v, y + r * n, n, lay);
    }
}

template <int CH, bool EXACT>
__global__ __launch_bounds__(kBlockThreads) PAM_BLOCK_ATTR void logsumexp_bwd_block_kernel(
    const float* __restrict__ x, const float* __restrict__ grad, const float* __restrict__ shift_in, float* __restrict__ dx,
    long rows, long n, int log_softmax, Offset o, Approx ap)
{
    PAM_BLOCK_ROW_SETUP;
    const float shift = *shift_in;
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        float xv[CH], gy[CH], out[CH];
        load_row<CH>(xv, x + r * n, n, lay, 0.0f);
#pragma unroll
        for (int c = 0; c < CH; ++c) gy[c] = 1.0f;
        if (log_softmax) load_row<CH>(gy, grad + r * n, n, lay, 1.0f);
        const float g_row = log_softmax ? 0.0f : grad[r];
        bool done = false;
        if (EXACT || (ap.a && ap.b && ap.e)) {         // EXACT: the host chose this instance for all-exact gradients without an offset
            typename std::conditional<EXACT, GradUncheckedExact, GradUncheckedFor<kLogsumexpBwd, CH, true>>::type u{o, Span()};
            logsumexp_grad_row<CH>(xv, gy, out, g_row, log_softmax != 0, shift, lay, n, u);
            done = lay.all(u.valid());
        }
        if (!done) { GradChecked k{o, ap}; logsumexp_grad_row<CH>(xv, gy, out, g_row, log_softmax != 0, shift, lay, n, k); }
        store_row<CH>(out, dx + r * n, n, lay);
    }
}

template <int CH, bool EXACT>
__global__ __launch_bounds__(kBlockThreads) PAM_BLOCK_ATTR void layer_norm_bwd_block_kernel(
    const float* __restrict__ x, const float* __restrict__ weight, const float* __restrict__ gy, float* __restrict__ dx,
    float* __restrict__ dw_terms, long rows, long n, float eps, Offset o, Approx ap)
{
    PAM_BLOCK_ROW_SETUP;
    const float count = (float)n;
    RowParams<CH, false> par{weight, nullptr};
    for (long r = blockIdx.x; r < rows; r += gridDim.x) {
        float cen[CH], g[CH], terms[CH];
        bool done = false;
        if (EXACT || (ap.a && ap.b && ap.e)) {
            load_row<CH>(cen, x + r * n, n, lay, 0.0f);
            load_row<CH>(g, gy + r * n, n, lay, 1.0f);
            typename std::conditional<EXACT, GradUncheckedExact, GradUncheckedFor<kLayerNormBwd, CH, true>>::type u{o, Span()};
            layer_norm_grad_row<CH>(cen, g, terms, par, lay, n, count, eps, u);
            done = lay.all(u.valid());
        }
        if (!done) {                                    // the row is read again (from cache) rather than kept in registers
            load_row<CH>(cen, x + r * n, n, lay, 0.0f);
            load_row<CH>(g, gy + r * n, n, lay, 1.0f);
            GradChecked k{o, ap};
            layer_norm_grad_row<CH>(cen, g, terms, par, lay, n, count, eps, k);
        }
        store_row<CH>(g, dx + r * n, n, lay);
        if (weight && dw_terms) store_row<CH>(terms, dw_terms + r * n, n, lay);
    }
}

// values per thread of the block kernels for a row of n values
int block_chunks(long n)
{
    for (int ch : {6, 8, 10, 12}) if (n <= (long)kBlockThreads * ch) return ch;
    return 16;
}
bool block_rows(long n) { return n > kBlockRowMin && n <= kBlockRowMax; }

#define PAM_BLOCK_DISPATCH_FLAG(KERNEL, FLAG, n, grid, st, ...)                                                 \
    switch (block_chunks(n)) {                                                                                  \
    case 6: hipLaunchKernelGGL((KERNEL<6, FLAG>), grid, dim3(kBlockThreads), 0, st, __VA_ARGS__); break;        \
    case 8: hipLaunchKernelGGL((KERNEL<8, FLAG>), grid, dim3(kBlockThreads), 0, st, __VA_ARGS__); break;        \
    case 10: hipLaunchKernelGGL((KERNEL<10, FLAG>), grid, dim3(kBlockThreads), 0, st, __VA_ARGS__); break;      \
    case 12: hipLaunchKernelGGL((KERNEL<12, FLAG>), grid, dim3(kBlockThreads), 0, st, __VA_ARGS__); break;      \
    default: hipLaunchKernelGGL((KERNEL<16, FLAG>), grid, dim3(kBlockThreads), 0, st, __VA_ARGS__); break;      \
    }

#define PAM_BLOCK_DISPATCH(KERNEL, n, grid, st, ...)                                                            \
    switch (block_chunks(n)) {                                                                                  \
    case 6: hipLaunchKernelGGL(KERNEL<6>, grid, dim3(kBlockThreads), 0, st, __VA_ARGS__); break;                \
    case 8: hipLaunchKernelGGL(KERNEL<8>, grid, dim3(kBlockThreads), 0, st, __VA_ARGS__); break;                \
    case 10: hipLaunchKernelGGL(KERNEL<10>, grid, dim3(kBlockThreads), 0, st, __VA_ARGS__); break;              \
    case 12: hipLaunchKernelGGL(KERNEL<12>, grid, dim3(kBlockThreads), 0, st, __VA_ARGS__); break;              \
    default: hipLaunchKernelGGL(KERNEL<16>, grid, dim3(kBlockThreads), 0, st, __VA_ARGS__); break;              \
    }

// smallest register-resident variant that holds a row of n values, 0 for the streaming one
int row_chunks(long n)
{
    for (int ch : {1, 2, 3, 4, 6, 8, 12, 16}) if (n <= 64L * ch) return ch;          // 3, 6, 12: rows of 192, 384, 768 values
    return 0;
}

#define PAM_ROW_DISPATCH(KERNEL, n, grid, st, ...)                                                              \
    switch (row_chunks(n)) {                                                                                    \
    case 1: hipLaunchKernelGGL(KERNEL<1>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 2: hipLaunchKernelGGL(KERNEL<2>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 3: hipLaunchKernelGGL(KERNEL<3>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 4: hipLaunchKernelGGL(KERNEL<4>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 6: hipLaunchKernelGGL(KERNEL<6>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 8: hipLaunchKernelGGL(KERNEL<8>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 12: hipLaunchKernelGGL(KERNEL<12>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                   \
    case 16: hipLaunchKernelGGL(KERNEL<16>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                   \
    default: hipLaunchKernelGGL(KERNEL<0>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                    \
    }

#define PAM_ROW_DISPATCH_FLAG(KERNEL, FLAG, n, grid, st, ...)                                                   \
    switch (row_chunks(n)) {                                                                                    \
    case 1: hipLaunchKernelGGL((KERNEL<1, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 2: hipLaunchKernelGGL((KERNEL<2, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 3: hipLaunchKernelGGL((KERNEL<3, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 4: hipLaunchKernelGGL((KERNEL<4, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 6: hipLaunchKernelGGL((KERNEL<6, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 8: hipLaunchKernelGGL((KERNEL<8, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 12: hipLaunchKernelGGL((KERNEL<12, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 16: hipLaunchKernelGGL((KERNEL<16, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;           \
    default: hipLaunchKernelGGL((KERNEL<0, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;            \
    }

#define PAM_ROW_DISPATCH_REGS_FLAG(KERNEL, FLAG, n, grid, st, ...)                                              \
    switch (row_chunks(n)) {                                                                                    \
    case 1: hipLaunchKernelGGL((KERNEL<1, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 2: hipLaunchKernelGGL((KERNEL<2, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 3: hipLaunchKernelGGL((KERNEL<3, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 4: hipLaunchKernelGGL((KERNEL<4, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 6: hipLaunchKernelGGL((KERNEL<6, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 8: hipLaunchKernelGGL((KERNEL<8, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    case 12: hipLaunchKernelGGL((KERNEL<12, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;             \
    default: hipLaunchKernelGGL((KERNEL<16, FLAG>), grid, dim3(kThreads), 0, st, __VA_ARGS__); break;           \
    }

#define PAM_ROW_DISPATCH_REGS(KERNEL, n, grid, st, ...)                                                         \
    switch (row_chunks(n)) {                                                                                    \
    case 1: hipLaunchKernelGGL(KERNEL<1>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 2: hipLaunchKernelGGL(KERNEL<2>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 3: hipLaunchKernelGGL(KERNEL<3>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 4: hipLaunchKernelGGL(KERNEL<4>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 6: hipLaunchKernelGGL(KERNEL<6>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 8: hipLaunchKernelGGL(KERNEL<8>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                     \
    case 12: hipLaunchKernelGGL(KERNEL<12>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                   \
    default: hipLaunchKernelGGL(KERNEL<16>, grid, dim3(kThreads), 0, st, __VA_ARGS__); break;                   \
    }

// compute units of the current device (looked up once per device)
int cu_count()
{
    static std::atomic<int> table[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int cus = table[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
        hipDeviceProp_t prop;
        cus = (hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
        table[dev].store(cus, std::memory_order_relaxed);
    }
    return cus;
}

// a work-group per row, at most four per compute unit in the launch
unsigned block_grid(long rows)
{
    long cap = (long)cu_count() * 4;
    return (unsigned)(rows < cap ? (rows < 1 ? 1 : rows) : cap);
}

// one wavefront per row, at most `per_cu` work-groups per compute unit in the launch: 16 (four wavefronts per SIMD's
// worth of waiting work-groups) for most kernels, 8 (exactly what is resident) for the short-row forward kernels
// that start by folding the shift, so that each wavefront does so once for more rows
unsigned row_grid(long rows, int per_cu = 16)
{
    long blocks = (rows + kWaves - 1) / kWaves;
    long cap = (long)cu_count() * per_cu;
    return (unsigned)(blocks < cap ? (blocks < 1 ? 1 : blocks) : cap);
}

int check_rows(const char* what, long rows, long n)
{
    if (rows < 0 || n < 0) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: negative size", what);
    if (n > (1L << 30) || rows > (1L << 40)) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: size out of range", what);
    return PAM_HIP_OK;
}

int launch_max(const char* what, const float* x, long rows, long n, Offset o, int mask_inf, void* workspace,
               size_t workspace_bytes, hipStream_t st, int* partials)
{
    if (!workspace || workspace_bytes < (size_t)kMaxPartials * sizeof(float))
        return pamhost::fail(PAM_HIP_ERR_WORKSPACE, "%s: workspace of %zu bytes needed", what, (size_t)kMaxPartials * sizeof(float));
    size_t total = (size_t)rows * (size_t)n;
    size_t nvec = ((uintptr_t)x & 15u) ? 0 : total / 4;
    size_t blocks = (total + (size_t)kThreads * 16 - 1) / ((size_t)kThreads * 16);
    if (blocks > (size_t)kMaxPartials) blocks = kMaxPartials;
    if (blocks < 1) blocks = 1;
    *partials = (int)blocks;
    hipLaunchKernelGGL(scaled_max_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, st, x, total, nvec, o, mask_inf,
                       (float*)workspace);
    return pamhost::check_launch(what);
}

}  // namespace

// ---------------------------------------------------------------- the variant's host functions (arguments as the entry points')

int PAM_ROW_FN(softmax_fwd)(const float* x, float* y, float* row_sum, float* shift, long rows, long n, float offset,
                        void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = check_rows("softmax_fwd", rows, n);
    if (rc != PAM_HIP_OK) return rc;
    if (rows == 0 || n == 0) return PAM_HIP_OK;
    if (!x || !y || !row_sum || !shift) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "softmax_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream; Offset o{offset, offset != 1.0f}; int partials = 0;
    rc = launch_max("softmax_fwd", x, rows, n, o, 1, workspace, workspace_bytes, st, &partials);
    if (rc != PAM_HIP_OK) return rc;
    if (block_rows(n)) {
        PAM_BLOCK_DISPATCH(softmax_fwd_block_kernel, n, dim3(block_grid(rows)), st, x, y, row_sum, shift, rows, n, o,
                           (const float*)workspace, partials);
    } else {
        PAM_ROW_DISPATCH(softmax_fwd_kernel, n, dim3(row_grid(rows, n <= 256 ? 8 : 16)), st, x, y, row_sum, shift, rows, n, o,
                         (const float*)workspace, partials);
    }
    return pamhost::check_launch("softmax_fwd");
}

int PAM_ROW_FN(softmax_bwd)(const float* x, const float* dy, const float* row_sum, const float* shift, float* dx,
                        long rows, long n, float offset, int approx_a, int approx_b, int approx_exp, void* stream)
{
    int rc = check_rows("softmax_bwd", rows, n);
    if (rc != PAM_HIP_OK) return rc;
    if (rows == 0 || n == 0) return PAM_HIP_OK;
    if (!x || !dy || !row_sum || !shift || !dx) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "softmax_bwd: null pointer");
    Offset o{offset, offset != 1.0f}; Approx ap{approx_a != 0, approx_b != 0, approx_exp != 0};
    const bool exact_fast = !ap.a && !ap.b && !ap.e && !o.has;
    if (block_rows(n)) {
        if (exact_fast) { PAM_BLOCK_DISPATCH_FLAG(softmax_bwd_block_kernel, true, n, dim3(block_grid(rows)), (hipStream_t)stream, x, dy, row_sum, shift, dx, rows, n, o, ap); }
        else { PAM_BLOCK_DISPATCH_FLAG(softmax_bwd_block_kernel, false, n, dim3(block_grid(rows)), (hipStream_t)stream, x, dy, row_sum, shift, dx, rows, n, o, ap); }
    } else {
        if (exact_fast) { PAM_ROW_DISPATCH_FLAG(softmax_bwd_kernel, true, n, dim3(row_grid(rows)), (hipStream_t)stream, x, dy, row_sum, shift, dx, rows, n, o, ap); }
        else { PAM_ROW_DISPATCH_FLAG(softmax_bwd_kernel, false, n, dim3(row_grid(rows)), (hipStream_t)stream, x, dy, row_sum, shift, dx, rows, n, o, ap); }
    }
    return pamhost::check_launch("softmax_bwd");
}

int PAM_ROW_FN(logsumexp_fwd)(const float* x, float* lse, float* log_softmax, float* shift, long rows, long n, float offset,
                          void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = check_rows("logsumexp_fwd", rows, n);
    if (rc != PAM_HIP_OK) return rc;
    if (rows == 0 || n == 0) return PAM_HIP_OK;
    if (!x || (!lse && !log_softmax)) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "logsumexp_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream; Offset o{offset, offset != 1.0f}; int partials = 0;
    rc = launch_max("logsumexp_fwd", x, rows, n, o, 0, workspace, workspace_bytes, st, &partials);
    if (rc != PAM_HIP_OK) return rc;
    if (block_rows(n)) {
        PAM_BLOCK_DISPATCH(logsumexp_block_kernel, n, dim3(block_grid(rows)), st, x, lse, log_softmax, shift, rows, n, o,
                           (const float*)workspace, partials);
    } else {
        PAM_ROW_DISPATCH(logsumexp_kernel, n, dim3(row_grid(rows, n <= 256 ? 8 : 16)), st, x, lse, log_softmax, shift, rows, n, o,
                         (const float*)workspace, partials);
    }
    return pamhost::check_launch("logsumexp_fwd");
}

int PAM_ROW_FN(row_mean_fwd)(const float* x, float* y, long rows, long n, float offset, void* stream)
{
    int rc = check_rows("row_mean_fwd", rows, n);
    if (rc != PAM_HIP_OK) return rc;
    if (rows == 0) return PAM_HIP_OK;
    if (!y || (n > 0 && !x)) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "row_mean_fwd: null pointer");
    if (block_rows(n))
        hipLaunchKernelGGL(row_mean_block_kernel, dim3(block_grid(rows)), dim3(kBlockThreads), 0, (hipStream_t)stream, x, y, rows, n,
                           Offset{offset, offset != 1.0f});
    else
        hipLaunchKernelGGL(row_mean_kernel, dim3(row_grid(rows)), dim3(kThreads), 0, (hipStream_t)stream, x, y, rows, n,
                           Offset{offset, offset != 1.0f});
    return pamhost::check_launch("row_mean_fwd");
}

int PAM_ROW_FN(layer_norm_fwd)(const float* x, const float* weight, const float* bias, float* y, long rows, long n,
                           float eps, float offset, void* stream)
{
    int rc = check_rows("layer_norm_fwd", rows, n);
    if (rc != PAM_HIP_OK) return rc;
    if (rows == 0 || n == 0) return PAM_HIP_OK;
    if (!x || !y) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "layer_norm_fwd: null pointer");
    const Offset o{offset, offset != 1.0f};
    if (block_rows(n)) {
        PAM_BLOCK_DISPATCH(layer_norm_fwd_block_kernel, n, dim3(block_grid(rows)), (hipStream_t)stream, x, weight, bias, y, rows, n, eps, o);
    } else {
        PAM_ROW_DISPATCH(layer_norm_fwd_kernel, n, dim3(row_grid(rows)), (hipStream_t)stream, x, weight, bias, y, rows, n, eps, o);
    }
    return pamhost::check_launch("layer_norm_fwd");
}

int PAM_ROW_FN(logsumexp_bwd)(const float* x, const float* grad, const float* shift, float* dx, long rows, long n,
                          int log_softmax, float offset, int approx_a, int approx_b, int approx_exp, void* stream)
{
    int rc = check_rows("logsumexp_bwd", rows, n);
    if (rc != PAM_HIP_OK) return rc;
    if (rows == 0 || n == 0) return PAM_HIP_OK;
    if (!x || !grad || !shift || !dx) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "logsumexp_bwd: null pointer");
    Offset o{offset, offset != 1.0f}; Approx ap{approx_a != 0, approx_b != 0, approx_exp != 0};
    const bool exact_fast = !ap.a && !ap.b && !ap.e && !o.has;
#define PAM_LSE_BWD(FLAG)                                                                                                       \
    if (block_rows(n)) {                                                                                                        \
        PAM_BLOCK_DISPATCH_FLAG(logsumexp_bwd_block_kernel, FLAG, n, dim3(block_grid(rows)), (hipStream_t)stream, x, grad, shift, dx, rows, n, \
                                log_softmax, o, ap);                                                                            \
    } else if (n > 1024)                                                                                                        \
        hipLaunchKernelGGL(logsumexp_bwd_stream_kernel<FLAG>, dim3(row_grid(rows)), dim3(kThreads), 0, (hipStream_t)stream, x, grad, shift, dx, \
                           rows, n, log_softmax, o, ap);                                                                        \
    else {                                                                                                                      \
        PAM_ROW_DISPATCH_REGS_FLAG(logsumexp_bwd_kernel, FLAG, n, dim3(row_grid(rows)), (hipStream_t)stream, x, grad, shift, dx, rows, n, \
                                   log_softmax, o, ap);                                                                         \
    }
    if (exact_fast) { PAM_LSE_BWD(true) } else { PAM_LSE_BWD(false) }
#undef PAM_LSE_BWD
    return pamhost::check_launch("logsumexp_bwd");
}

int PAM_ROW_FN(layer_norm_bwd)(const float* x, const float* weight, const float* dy, float* dx, float* dw_terms, long rows, long n,
                           float eps, float offset, int approx_a, int approx_b, int approx_exp, void* stream)
{
    int rc = check_rows("layer_norm_bwd", rows, n);
    if (rc != PAM_HIP_OK) return rc;
    if (rows == 0 || n == 0) return PAM_HIP_OK;
    if (!x || !dy || !dx) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "layer_norm_bwd: null pointer");
    Offset o{offset, offset != 1.0f}; Approx ap{approx_a != 0, approx_b != 0, approx_exp != 0};
    const bool exact_fast = !ap.a && !ap.b && !ap.e && !o.has;
#define PAM_LN_BWD(FLAG)                                                                                                        \
    if (block_rows(n)) {                                                                                                        \
        PAM_BLOCK_DISPATCH_FLAG(layer_norm_bwd_block_kernel, FLAG, n, dim3(block_grid(rows)), (hipStream_t)stream, x, weight, dy, dx, dw_terms, \
                                rows, n, eps, o, ap);                                                                           \
    } else if (n > 1024)                                                                                                        \
        hipLaunchKernelGGL(layer_norm_bwd_stream_kernel<FLAG>, dim3(row_grid(rows)), dim3(kThreads), 0, (hipStream_t)stream, x, weight, dy, dx, \
                           dw_terms, rows, n, eps, o, ap);                                                                      \
    else {                                                                                                                      \
        PAM_ROW_DISPATCH_REGS_FLAG(layer_norm_bwd_kernel, FLAG, n, dim3(row_grid(rows)), (hipStream_t)stream, x, weight, dy, dx, dw_terms, \
                                   rows, n, eps, o, ap);                                                                        \
    }
    if (exact_fast) { PAM_LN_BWD(true) } else { PAM_LN_BWD(false) }
#undef PAM_LN_BWD
    return pamhost::check_launch("layer_norm_bwd");
}


