// PAM matrix products for gfx950, host side: the plan of a launch, the entry points of the C ABI for products and
// convolutions, and the scratch the library owns.  The kernel is in pam_gemm_kernel.h.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <mutex>
#include <random>

#include "pam_gemm_kernel.h"
#include "../../include/pam_hip_probe.h"

using namespace pamdev;
using namespace pamgemm;

namespace {

// compute units of the current device (looked up once per device)
int cu_count()
{
    constexpr int kDevices = 64;
    static std::atomic<int> cus[kDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kDevices) return 256;
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        hipDeviceProp_t prop;
        n = (hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
        cus[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// How a product is scheduled (see the kernel's comment on units).  bk: depth of a k-tile; kt: k-tiles per output
// tile; pieces, piece_kt: the k ranges a tile is cut into and their length in k-tiles; units = tiles x pieces.
struct Plan { int bk, kt, pieces, piece_kt; long units; };

// Tuning override for experiments, per calling thread (include/pam_hip_probe.h): bk 0 = automatic (16 or 32);
// pieces 0 = automatic, > 0 that many k ranges per tile (as far as k allows).
thread_local int g_force_bk = 0, g_force_pieces = 0;

constexpr long kMostCutTiles = 8192;            // tiles of a product that cuts them (its arrival words: 64 KB)
constexpr int kResidentPerCu = 4;               // work-groups of the kernel a compute unit holds (LDS and registers)
constexpr size_t kPartBytes = (size_t)pamgemm::kPartFloats * sizeof(float);

// Work-groups own 64 x 64 output tiles.  k of 128 and more in whole multiples of 32, and any k
// from 512, uses 32-deep k-tiles (fewer barriers and more bytes in flight per round, measured 3-5 %
// faster on 12608-row products); short or ragged k (attention: 64, 197) 16-deep ones.
// Shapes with few output tiles and long k (dX: 12608 x 192, k = 768; dW: 192 x 768, k = 12608) cut every tile's k
// range into equal pieces, each at least 128 deep in k: few pieces by the cost model below (the tile's last
// work-group adds them up), or, where that asks for more than a work-group should add up, about two resident rounds of
// piece-major units and a second kernel.
Plan make_plan(long batch, long M, long N, long K, bool with_workspace)
{
    const long resident = (long)kResidentPerCu * cu_count();
    const long tiles = batch * ((M + 63) / 64) * ((N + 63) / 64);
    Plan p;
    p.bk = (K >= 512 || (K >= 128 && K % 32 == 0)) ? 32 : 16;
    if (g_force_bk) p.bk = g_force_bk;
    p.kt = (int)((K + p.bk - 1) / p.bk);
    p.pieces = 1; p.piece_kt = p.kt;
    const long least = (128 + p.bk - 1) / p.bk;                       // k-tiles in 128 k
    const long most = p.kt / least;                                   // pieces a tile can be cut into
    long want = 1;
    if (g_force_pieces > 0) want = g_force_pieces;
    else if (tiles < (3 * resident) / 2 && tiles <= kMostCutTiles && with_workspace) {
        // Time of the product cut into w pieces, in k-tile times of a work-group alone on its compute unit; fitted to
        // measurements on the 12608 x 192 <-> 768 products.  A unit costs its k-tiles plus about one more (fetch of its
        // first k-tile, way out, arrival).  Up to one unit per compute unit they all run at that speed; four on a compute
        // unit each run about 1.5 times slower; beyond what is resident the rounds add up, a last round that is not
        // full costing a little more than its share.
        const long cus = resident / kResidentPerCu;
        double best = 0.0;
        for (long w = 1; w <= (most > 1 ? most : 1); ++w) {
            const long per = (p.kt + w - 1) / w, pieces = (p.kt + per - 1) / per;
            if (pieces != w) continue;                                // the same cut as a smaller w
            const long n = tiles * pieces;
            const double rounds = (double)n / (double)resident;
            const double crowd = n <= cus ? 1.0 : n <= resident ? 1.0 + 0.5 * (double)(n - cus) / (double)(resident - cus)
                                                                 : 1.5 * (rounds + 0.15 * (std::ceil(rounds) - rounds));
            const double time = (double)(per + 1) * crowd * (pieces > pamgemm::kFoldInKernel ? 1.03 : 1.0);
            if (best == 0.0 || time < best) { best = time; want = pieces; }
        }
        // More pieces than a tile's last work-group adds up itself (few tiles, very long k: the weight gradients): the
        // units are piece-major in launch order and a second kernel adds them.  Two work-groups on a compute unit issue
        // at nearly the rate of four, and a third adds little, so such a launch runs in rounds of two units per compute
        // unit: its time goes as (rounds + 0.4) x (k-tiles per piece + 1.25), the 0.4 for the skew with which a round's
        // units end, the 1.25 for a unit's start and way out.  Fitted on weight gradients of 9 ... 144 tiles with k =
        // 3152 ... 50432 (pieces of 224 k for the 192 x 768, k = 12608 one: 86 us dense, 102 us with the zeros of a
        // ReLU in the left operand; one resident round of 27 pieces, a range of them per XCD: 88 and 111 us).
        if (want > pamgemm::kFoldInKernel) {
            const long quantum = 2 * cus;
            double least_time = 0.0;
            for (long per = least;; ++per) {
                const long pieces = (p.kt + per - 1) / per;
                if (pieces <= pamgemm::kFoldInKernel) break;
                if (pieces > most) continue;
                const long n = tiles * pieces;
                long rounds = (n - n / 50 + quantum - 1) / quantum;               // (2 % over whole rounds still counts as those)
                if (rounds < 1) rounds = 1;
                const double time = ((double)rounds + 0.4) * ((double)per + 1.25);
                if (least_time == 0.0 || time < least_time) { least_time = time; want = pieces; }
            }
        }
    }
    if (want > (g_force_pieces > 0 ? (long)p.kt : most)) want = g_force_pieces > 0 ? (long)p.kt : most;
    if (with_workspace && want > 1 && tiles <= kMostCutTiles) {
        p.piece_kt = (int)((p.kt + want - 1) / want);
        p.pieces = (p.kt + p.piece_kt - 1) / p.piece_kt;
    }
    p.units = tiles * p.pieces;
    return p;
}

// workspace of a plan that cuts tiles: [arrival words, one per tile][one piece per unit].  The words' part has one size
// for every shape, so that products of different shapes that share a workspace never write pieces over each other's
// words (a word that does not carry the launch's tag costs its first arriver two more round trips).
constexpr size_t kArriveBytes = (size_t)kMostCutTiles * sizeof(unsigned long long);
struct Space { size_t partial, total; };
Space plan_space(const Plan& p)
{
    Space w{0, 0};
    if (p.pieces > 1) {
        w.partial = kArriveBytes;
        w.total = w.partial + (size_t)p.units * kPartBytes;
    }
    return w;
}

// Tags of the launches that cut tiles: a 40-bit counter that starts at a random value.
unsigned long long next_tag()
{
    static std::atomic<unsigned long long> counter{[] {
        std::random_device rd;
        return ((unsigned long long)rd() << 32) | rd();
    }()};
    return counter.fetch_add(1, std::memory_order_relaxed) & pamgemm::kTagMask;
}

// sums over nothing: +0, plus the bias
__global__ __launch_bounds__(256) void empty_k_kernel(float* __restrict__ y, long y_sb, long y_sr, long y_sc, long batch, int M, int N,
                                                     const float* __restrict__ bias)
{
    const long per = (long)M * N, idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= batch * per) return;
    const long b = idx / per, rem = idx % per;
    y[b * y_sb + (rem / N) * y_sr + (rem % N) * y_sc] = bias ? 0.0f + bias[rem % N] : 0.0f;
}

// Cut tiles of many pieces: the pieces of every tile added in ascending order from +0 by a kernel of its own, one
// lane per 128-bit row of the tile (work-groups of 128 lanes, eight per tile); eight pieces' loads in flight.
__global__ __launch_bounds__(128) void fold_kernel(pamgemm::GemmArgs g)
{
    using pamgemm::v4f;
    const int flat = blockIdx.x / 8, i = (blockIdx.x % 8) / 2, tid = (blockIdx.x % 2) * 128 + threadIdx.x;
    v4f total = {0.0f, 0.0f, 0.0f, 0.0f};
    const long first = (long)flat * g.pieces;
    int p = 0;
    for (; p + 8 <= g.pieces; p += 8) {
        v4f v[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) v[c] = *pamgemm::piece_row(g.partial, first + p + c, i, tid);
#pragma unroll
        for (int c = 0; c < 8; ++c) total += v[c];
    }
    for (; p < g.pieces; ++p) total += *pamgemm::piece_row(g.partial, first + p, i, tid);
    const int zb = flat / g.tiles, tile = flat - zb * g.tiles, tr = tile / g.ntn;
    const int row0 = tr * 64, col0 = (tile - tr * g.ntn) * 64;
    const pamgemm::LanePlace place = pamgemm::lane_place(tid, row0, col0, g.M, g.N);
    const int r = row0 + place.ty * 4 + i, c = col0 + place.tx * 4;
    if (r >= g.M) return;
    float* dst = g.Y + (long)zb * g.y_sb + (long)r * g.y_sr + (long)c * g.y_sc;
    const float sums[4] = {total.x, total.y, total.z, total.w};
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (c + j < g.N) dst[(long)j * g.y_sc] = g.bias ? sums[j] + g.bias[c + j] : sums[j];
}

int load_kind(long s_row, long s_k, long s_batch, const float* p, long rows, long K)
{
    bool aligned = ((reinterpret_cast<uintptr_t>(p) & 15u) == 0) && (s_batch % 4 == 0);
    if (s_k == 1 && aligned && s_row % 4 == 0 && K % 4 == 0 && K >= 4) return LOAD_KVEC;
    if (s_row == 1 && aligned && s_k % 4 == 0 && rows % 4 == 0 && rows >= 4) return LOAD_RVEC;
    return LOAD_ANY;
}

template <int MODE>
void launch_mode(const Plan& p, int lk, int rk, hipStream_t st, const GemmArgs& g)
{
    // One contiguous range of units per XCD (see the kernel), rounded up to whole work-groups per XCD.  Piece-major
    // launches keep the launch order: all XCDs then work on the same few k ranges at a time (each L2 fetches them,
    // from the memory-side cache), where ranges would have every L2 hold three or four k ranges of both operands at
    // once -- measured 3 % (dense) to 9 % (left operand with zeros) slower.
    GemmArgs ga = g;
    unsigned groups = (unsigned)p.units;
    if (p.units >= 64 && (p.pieces == 1 || g.fold_here)) {
        ga.xcd_chunk = (int)((p.units + XCDS - 1) / XCDS);
        groups = (unsigned)(ga.xcd_chunk * XCDS);
    }
    if (p.bk == 32) pamgemm::launch_gemm<32, MODE>(lk, rk, groups, st, ga);
    else pamgemm::launch_gemm<16, MODE>(lk, rk, groups, st, ga);
}

int gemm(const char* what, int mode, long batch, long M, long N, long K,
         const float* l, long l_sb, long l_sr, long l_sc, const float* r, long r_sb, long r_sr, long r_sc,
         const float* d, long d_sb, long d_sr, long d_sc, float* y, long y_sb, long y_sr, long y_sc,
         float offset, void* workspace, size_t workspace_bytes, void* stream, const ConvGeom* conv = nullptr,
         const float* bias = nullptr)
{
    if (batch < 0 || M < 0 || N < 0 || K < 0) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: negative size", what);
    if (batch == 0 || M == 0 || N == 0) return PAM_HIP_OK;
    // with K == 0 the operands are empty (and may be null): the sums over nothing are +0 (plus the bias)
    if (((!l || !r) && K > 0) || !y || (mode >= MODE_BWD_DL && !d)) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: null pointer", what);
    if (M > (1L << 30) || N > (1L << 30) || K > (1L << 30) || batch > (1L << 30) || batch * ((M + 63) / 64) * ((N + 63) / 64) > 0x7fffff00L)
        return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: dimension too large (sizes and batch <= 2^30, output tiles of all matrices < 2^31)", what);
    hipStream_t st = (hipStream_t)stream;

    if (K == 0) {                                  // (the operands are empty, and may be null)
        const long n = batch * M * N;
        hipLaunchKernelGGL(empty_k_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, y, y_sb, y_sr, y_sc, batch, (int)M, (int)N, bias);
        return pamhost::check_launch(what);
    }
    const bool usable = workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0;
    Plan p = make_plan(batch, M, N, K, usable);
    if (p.pieces > 1 && plan_space(p).total > workspace_bytes) p = make_plan(batch, M, N, K, false);       // whole tiles
    const Space sp = plan_space(p);

    GemmArgs g;
    g.L = Operand{l, l_sb, l_sr, l_sc};
    g.R = Operand{r, r_sb, r_sc, r_sr};            // R's "row" index is the output column
    g.D = d; g.d_sb = d_sb; g.d_sr = d_sr; g.d_sc = d_sc;
    g.Y = y; g.y_sb = y_sb; g.y_sr = y_sr; g.y_sc = y_sc;
    g.bias = bias;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.ntn = (int)((N + 63) / 64); g.tiles = (int)(((M + 63) / 64) * g.ntn);
    g.pieces = p.pieces; g.piece_kt = p.piece_kt; g.units = (int)p.units;
    g.xcd_chunk = 0;
    g.fold_here = p.pieces > 1 && p.pieces <= pamgemm::kFoldInKernel;
    g.arrive = p.pieces > 1 ? (unsigned long long*)workspace : nullptr;
    g.tag = g.fold_here ? next_tag() : 0;
    g.partial = p.pieces > 1 ? (float*)((char*)workspace + sp.partial) : nullptr;
    g.off = offset; g.off_add = 0; g.has_off = 0;
    if (mode != MODE_STD && offset != 1.0f) {
        uint32_t bits; memcpy(&bits, &offset, sizeof bits);
        g.has_off = std::isnormal(offset) ? 1 : 2;
        g.off_add = bits - kBias;
    }

    g.cv = conv ? *conv : ConvGeom{nullptr, nullptr, 0, 0, 0, 0, 0};

    int lk = load_kind(l_sr, l_sc, l_sb, l, M, K);
    int rk = conv ? LOAD_CONV : load_kind(r_sc, r_sr, r_sb, r, N, K);
    if (conv && conv->quads && !conv->transposed && mode == MODE_PAM && lk == LOAD_KVEC && K % 4 == 0 && (reinterpret_cast<uintptr_t>(r) & 15u) == 0 && r_sb % 4 == 0)
        rk = LOAD_CONVQ;
    else if (conv && conv->row_quads && !conv->transposed && mode != MODE_STD && lk == LOAD_KVEC && N % 4 == 0)
        rk = LOAD_CONVR;
    else if (conv && conv->row_quads && conv->transposed && mode != MODE_STD && lk == LOAD_KVEC && K % 4 == 0)
        rk = LOAD_CONVK;
    switch (mode) {
    case MODE_PAM: launch_mode<MODE_PAM>(p, lk, rk, st, g); break;
    case MODE_STD: launch_mode<MODE_STD>(p, lk, rk, st, g); break;
    case MODE_BWD_DL: launch_mode<MODE_BWD_DL>(p, lk, rk, st, g); break;
    default: launch_mode<MODE_BWD_DR>(p, lk, rk, st, g); break;
    }
    if (p.pieces > 1 && !g.fold_here)
        hipLaunchKernelGGL(fold_kernel, dim3((unsigned)(p.units / p.pieces * 8)), dim3(128), 0, st, g);
    return pamhost::check_launch(what);
}

// ---------------------------------------------------------------- convolution as a product with image patches
// groups: channels and filters fall into `g` groups that do not mix (weights [co][c / g][kh][kw]); K() is the
// length of one group's sums
struct ConvShape {
    long batch, c, h, w, co, kh, kw, sh, sw, ph, pw, ho, wo, g;
    long cg() const { return c / g; } long cog() const { return co / g; }
    long K() const { return cg() * kh * kw; } long L() const { return ho * wo; }
};

__global__ __launch_bounds__(256) void conv_tables_kernel(int2* __restrict__ ktab, int2* __restrict__ ltab, int K, int L,
                                                         int kh, int kw, int H, int W, int wo, int sh, int sw, int ph, int pw)
{
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx < K) {
        const int c = idx / (kh * kw), rem = idx % (kh * kw), i = rem / kw, j = rem % kw;
        ktab[idx] = make_int2(c * H * W + i * W + j, (i << 16) | j);
    }
    if (idx < L) {
        const int h0 = (idx / wo) * sh - ph, w0 = (idx % wo) * sw - pw;
        ltab[idx] = make_int2(h0 * W + w0, (int)(((unsigned)h0 << 16) | ((unsigned)w0 & 0xffffu)));
    }
}

// out = `copies` copies of in[0 .. n), each value (*) off if has_off
__global__ __launch_bounds__(256) void scale_kernel(const float* __restrict__ in, float* __restrict__ out, size_t n, size_t copies, float off,
                                                    int has_off)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n * copies; i += (size_t)gridDim.x * 256) {
        const float v = in[i % n];
        out[i] = has_off ? pam_mul(v, off) : v;
    }
}
void launch_scale(const float* in, float* out, size_t n, size_t copies, float off, bool has_off, hipStream_t st)
{
    size_t blocks = (n * copies + 1023) / 1024;
    if (blocks > (1u << 20)) blocks = 1u << 20;
    hipLaunchKernelGGL(scale_kernel, dim3((unsigned)blocks), dim3(256), 0, st, in, out, n, copies, off, has_off ? 1 : 0);
}

// wf[c][co][i][j] = w[co][c][kh-1-i][kw-1-j] (*) off: the weights of the convolution over the
// upstream gradient that yields the gradient of the input (stride 1)
// (with groups: c runs over all channels, co over the filters of c's group, and w is [filters][c per group][kh][kw])
// (`copies` of them one after the other: see kReplicateBytes)
__global__ __launch_bounds__(256) void flip_weights_kernel(const float* __restrict__ w, float* __restrict__ wf, int c, int cog, int cg, int kh, int kw,
                                                          float off, int has_off, int copies)
{
    const long at = (long)blockIdx.x * 256 + threadIdx.x, n = (long)c * cog * kh * kw;
    if (at >= n * copies) return;
    const int idx = (int)(at % n);
    const int j = idx % kw, i = (idx / kw) % kh, o = (idx / (kw * kh)) % cog, ci = idx / (kw * kh * cog);
    const int filter = (ci / cg) * cog + o;
    const float v = w[(((long)filter * cg + ci % cg) * kh + (kh - 1 - i)) * kw + (kw - 1 - j)];
    wf[at] = has_off ? pam_mul(v, off) : v;
}

size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

int conv_shape(const char* what, ConvShape& s)
{
    if (s.batch < 0 || s.c <= 0 || s.h <= 0 || s.w <= 0 || s.co <= 0 || s.kh <= 0 || s.kw <= 0 || s.sh <= 0 || s.sw <= 0 || s.ph < 0 || s.pw < 0)
        return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: bad geometry", what);
    if (s.g <= 0 || s.c % s.g != 0 || s.co % s.g != 0 || s.g > 65535)
        return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: groups must divide the channel and filter counts", what);
    s.ho = (s.h + 2 * s.ph - s.kh) / s.sh + 1;             // (in + 2 pad - (k - 1) - 1) / stride + 1 (pam/pam_ops.py:137-138)
    s.wo = (s.w + 2 * s.pw - s.kw) / s.sw + 1;
    if (s.h + 2 * s.ph < s.kh || s.w + 2 * s.pw < s.kw) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: kernel larger than the padded image", what);
    if (s.c * s.h * s.w >= (1L << 31) || s.h >= 32768 || s.w >= 32768 || s.kh >= 32768 || s.kw >= 32768 || s.ph >= 16384 || s.pw >= 16384)
        return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: image too large for the patch tables", what);
    return PAM_HIP_OK;
}

// A grouped convolution is one launch over (image, group) pairs: unit z = image * groups + group finds its rows of the
// image, of the upstream gradient and of the output at z times one group's size, since an image's groups lie one after
// the other.  Only the weights do not follow that pattern (every image uses all of them), so where a product reads them
// it gets one copy per image -- up to this many bytes of copies; beyond, the groups are launched one by one.
constexpr size_t kReplicateBytes = 32u << 20;
bool replicated(const ConvShape& s) { return s.g > 1 && (size_t)s.batch * s.co * s.K() * sizeof(float) <= kReplicateBytes; }

// workspace: [k table][l table][operand scaled by the offset, or the weights' copies, if any][split-k partial tiles]
// which: 0 forward, 1 weight gradient approximate, 2 weight gradient exact
struct ConvSpace { size_t tables, scaled, total; };
ConvSpace conv_space(const ConvShape& s, int which, bool has_off)
{
    ConvSpace w;
    w.tables = align256((size_t)(s.K() + s.L()) * sizeof(int2));
    const size_t copies = replicated(s) ? (size_t)s.batch : 1;
    size_t scaled_elems = 0;
    if (which == 0) scaled_elems = (has_off || copies > 1) ? copies * s.co * s.K() : 0;
    else if (which == 1) scaled_elems = has_off ? (size_t)s.batch * s.co * s.L() : 0;
    else scaled_elems = copies > 1 ? copies * s.co * s.K() : 0;
    w.scaled = align256(scaled_elems * sizeof(float));
    const long launches = s.g > 1 && (which == 1 || replicated(s)) ? s.batch * s.g : s.batch;
    size_t split = which != 0 ? pam_hip_gemm_workspace_bytes(launches, s.cog(), s.K(), s.L())
                              : pam_hip_gemm_workspace_bytes(launches, s.cog(), s.L(), s.K());
    w.total = w.tables + w.scaled + split;
    return w;
}

int conv_prepare(const char* what, const ConvShape& s, const ConvSpace& sp, void* workspace, size_t workspace_bytes,
                 hipStream_t st, ConvGeom& cv, bool transposed)
{
    if (!workspace || workspace_bytes < sp.total)
        return pamhost::fail(PAM_HIP_ERR_WORKSPACE, "%s: workspace of %zu bytes needed", what, sp.total);
    int2* ktab = (int2*)workspace; int2* ltab = ktab + s.K();
    const long n = s.K() > s.L() ? s.K() : s.L();
    hipLaunchKernelGGL(conv_tables_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, ktab, ltab, (int)s.K(), (int)s.L(),
                       (int)s.kh, (int)s.kw, (int)s.h, (int)s.w, (int)s.wo, (int)s.sh, (int)s.sw, (int)s.ph, (int)s.pw);
    const bool quads = s.ph == 0 && s.pw == 0 && s.kw % 4 == 0 && s.w % 4 == 0 && s.sw % 4 == 0;
    const bool row_quads = s.sw == 1 && s.wo % 4 == 0;
    cv = ConvGeom{ktab, ltab, (int)s.h, (int)s.w, transposed ? 1 : 0, quads ? 1 : 0, row_quads ? 1 : 0};
    return PAM_HIP_OK;
}

// The gradient of the input of a stride-1 convolution is itself a convolution: of the upstream
// gradient [co, ho, wo], padded by (k - 1 - pad), with the weights flipped and their two channel
// indices exchanged.  `t` is that convolution's geometry (its "image" is the upstream gradient).
int input_gradient_shape(const char* what, const ConvShape& s, ConvShape& t)
{
    if (s.sh != 1 || s.sw != 1) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: the input gradient in place needs stride 1", what);
    if (s.ph > s.kh - 1 || s.pw > s.kw - 1) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: padding larger than kernel - 1", what);
    t = ConvShape{s.batch, s.co, s.ho, s.wo, s.c, s.kh, s.kw, 1, 1, s.kh - 1 - s.ph, s.kw - 1 - s.pw, 0, 0, s.g};
    int rc = conv_shape(what, t);
    if (rc != PAM_HIP_OK) return rc;
    if (t.ho != s.h || t.wo != s.w) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: geometry does not invert", what);
    return PAM_HIP_OK;
}

// workspace: [k table][l table][flipped weights][split-k partial tiles]
ConvSpace input_gradient_space(const ConvShape& t)
{
    ConvSpace w;
    w.tables = align256((size_t)(t.K() + t.L()) * sizeof(int2));
    const bool copies = replicated(t);
    w.scaled = align256((copies ? (size_t)t.batch : 1) * t.co * t.K() * sizeof(float));
    w.total = w.tables + w.scaled + pam_hip_gemm_workspace_bytes(copies ? t.batch * t.g : t.batch, t.cog(), t.L(), t.K());
    return w;
}

// ---------------------------------------------------------------- convolutions with small groups (depthwise among them)
// A group of a few channels and filters is a handful of terms per output ((c / groups) kh kw of them) and fills a few rows
// of a matrix tile; these kernels compute such convolutions directly, in the order the matrix kernel would: terms in
// ascending k from +0, a padding position contributing the product with +0.
// gin / gout: channels of a group that a sum runs over / that it produces.
struct DirectGeom { int IC, H, W, ho, wo, kh, kw, sh, sw, ph, pw, gin, gout; };

// out[b][p][oh][ow], p = g gout + oc, = sum over q < gin and (i, j) of term(weight, img[b][g gin + q][oh sh - ph + i][ow sw - pw + j]).
// The weight: w[p][q][i][j], or with `transposed` w[g gin + q][oc][kh - 1 - i][kw - 1 - j] (the input gradient: img = the
// upstream gradient, the stride-1 geometry of that convolution, the sum over a group's filters).
// EXACT false: term = (weight (*) off) (*) v -- the forward and the approximate input gradient; EXACT true:
// term = pam_bwd(d, weight, v) with the offset on the weight, d = the output position's own forward input.
// SIDE: the kernel is SIDE x SIDE taps and the loops over them are unrolled (all of a channel's loads in flight
// together); 0: any kernel size.
template <bool EXACT, int SIDE>
__global__ __launch_bounds__(256) void direct_conv_kernel(const float* __restrict__ img, const float* __restrict__ w, const float* __restrict__ d,
                                                         float* __restrict__ out, long total, int planes, DirectGeom q, int transposed, float off,
                                                         int has_off)
{
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    int ow, oh, p; long b;                                                // idx = ((b planes + p) ho + oh) wo + ow
    if (total <= 0x7fffffffL) {                                           // (32-bit divisions where they do: the 64-bit ones are long)
        const int at = (int)idx, hw = q.wo * q.ho, plane = at / hw, l = at - plane * hw, b32 = plane / planes;
        oh = l / q.wo; ow = l - oh * q.wo; p = plane - b32 * planes; b = b32;
    } else {
        const long plane = idx / ((long)q.wo * q.ho);
        ow = (int)(idx % q.wo); oh = (int)((idx / q.wo) % q.ho); p = (int)(plane % planes); b = plane / planes;
    }
    const int kh = SIDE ? SIDE : q.kh, kw = SIDE ? SIDE : q.kw;
    const int g = p / q.gout, oc = p % q.gout, taps = kh * kw;
    const float dv = EXACT ? d[idx] : 0.0f;
    float acc = 0.0f;
    for (int c = 0; c < q.gin; ++c) {
        const float* base = img + (b * q.IC + g * q.gin + c) * (long)q.H * q.W;
        const float* wc = w + (transposed ? ((long)(g * q.gin + c) * q.gout + oc) : ((long)p * q.gin + c)) * taps;
#pragma unroll
        for (int i = 0; i < kh; ++i) {
            const int h = oh * q.sh - q.ph + i;
#pragma unroll
            for (int j = 0; j < kw; ++j) {
                const int x = ow * q.sw - q.pw + j, k = i * kw + j;
                const float wk = wc[transposed ? taps - 1 - k : k];
                const bool inside = (unsigned)h < (unsigned)q.H && (unsigned)x < (unsigned)q.W;
                const float v = inside ? base[(long)h * q.W + x] : 0.0f;
                // A padding position's term is a zero, and adding it changes nothing (the sum starts at +0 and never
                // becomes -0) -- unless the weight (or d) is inf or NaN, which makes the term NaN: only then is it
                // computed.  (Computed always, the zeros took the primitives' full definition in nearly every wavefront.)
                const float ws = has_off ? pam_mul(wk, off) : wk;              // (the weight as the product sees it)
                // (EXACT: the slope of a weight of 2^127 and more can be inf, and inf times the zero NaN)
                const bool finite = (f2u(ws) & 0x7fffffffu) < (EXACT ? 0x7f000000u : 0x7f800000u) && (!EXACT || (f2u(dv) & 0x7f800000u) != 0x7f800000u);
                if (inside || !finite)
                    acc = acc + (EXACT ? pam_mul_bwd(dv, wk, v, off, has_off != 0) : pam_mul(ws, v));
            }
        }
    }
    out[idx] = acc;
}

// dw[b][co][k], k = (c, i, j) of the filter's group, = sum over the output positions l of term(dy[b][co][l], x patch
// entry (k, l)), l ascending in chunks of `chunk` whose sums are added in ascending order from +0 (the order the matrix
// kernel's plan gives this sum).  EXACT false: term = (dy (*) off) (*) v; EXACT true: term = pam_bwd(w[co][k], v, dy)
// with the offset on v.
template <bool EXACT>
__global__ __launch_bounds__(256) void direct_conv_weight_kernel(const float* __restrict__ x, const float* __restrict__ dy, const float* __restrict__ w,
                                                                float* __restrict__ dw, long total, int filters, DirectGeom q, int chunk, float off,
                                                                int has_off)
{
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int taps = q.kh * q.kw, K = q.gin * taps;
    const long plane = total <= 0x7fffffffL ? (long)((int)idx / K) : idx / K;          // b * filters + co
    const int k = (int)(idx - plane * K), c = k / taps, i = (k % taps) / q.kw, j = k % q.kw;
    const int co = (int)(plane % filters), L = q.ho * q.wo;
    const long b = plane / filters;
    const float* base = x + (b * q.IC + (co / q.gout) * q.gin + c) * (long)q.H * q.W;
    const float* g = dy + plane * L;
    const float wk = EXACT ? w[(long)co * K + k] : 0.0f;
    float sum = 0.0f;
    for (int l0 = 0; l0 < L; l0 += chunk) {
        float part = 0.0f;
        const int end = min(L, l0 + chunk);
        // eight positions' loads in flight at a time (there are few lanes, each with a long chain of sums); the terms
        // are added one by one in ascending order all the same
        constexpr int kAhead = 8;
        for (int lb = l0; lb < end; lb += kAhead) {
            float v[kAhead], gv[kAhead]; bool in[kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const int l = min(lb + u, end - 1);
                const int h = (l / q.wo) * q.sh - q.ph + i, xx = (l % q.wo) * q.sw - q.pw + j;
                in[u] = (unsigned)h < (unsigned)q.H && (unsigned)xx < (unsigned)q.W;
                v[u] = in[u] ? base[(long)h * q.W + xx] : 0.0f; gv[u] = g[l];
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                if (lb + u >= end) break;
                const float gl = gv[u];
                // (a padding position's term is a zero unless the gradient -- or w -- is inf or NaN: see direct_conv_kernel)
                const float gs = !EXACT && has_off ? pam_mul(gl, off) : gl;     // (the gradient as the approximate product sees it)
                const bool finite = (f2u(gs) & 0x7f800000u) != 0x7f800000u && (!EXACT || (f2u(wk) & 0x7f800000u) != 0x7f800000u);
                if (in[u] || !finite)
                    part = part + (EXACT ? pam_mul_bwd(wk, v[u], gl, off, has_off != 0) : pam_mul(gs, v[u]));
            }
        }
        sum = chunk >= L ? part : sum + part;
    }
    dw[idx] = sum;
}

template <bool EXACT>
void launch_direct_conv(const float* img, const float* w, const float* d, float* out, long total, int planes, const DirectGeom& q,
                        int transposed, float off, hipStream_t st)
{
    const dim3 grid((unsigned)((total + 255) / 256));
    const int has_off = off != 1.0f ? 1 : 0, side = q.kh == q.kw ? q.kh : 0;
#define PAM_DIRECT_SIDE(S) hipLaunchKernelGGL((direct_conv_kernel<EXACT, S>), grid, dim3(256), 0, st, img, w, d, out, total, planes, q, transposed, off, has_off)
    if (side == 3) PAM_DIRECT_SIDE(3); else if (side == 5) PAM_DIRECT_SIDE(5); else if (side == 7) PAM_DIRECT_SIDE(7); else PAM_DIRECT_SIDE(0);
#undef PAM_DIRECT_SIDE
}

// Which grouped convolutions: groups of up to kDirectGroup channels and filters whose sums (either way round) are short
// enough to never be cut along k.  Depthwise only: with four channels and filters per group (32 images of 128 x 28 x 28,
// 3 x 3) the forward ran 116 us here against 125 us on the matrix kernel, but the weight gradient 295 against 117.
constexpr long kDirectGroup = 1;
bool direct_conv(const ConvShape& s)
{
    return s.g > 1 && s.cg() <= kDirectGroup && s.cog() <= kDirectGroup && s.K() < 128 && s.cog() * s.kh * s.kw < 128;
}
DirectGeom direct_geom(const ConvShape& s)
{
    return DirectGeom{(int)s.c, (int)s.h, (int)s.w, (int)s.ho, (int)s.wo, (int)s.kh, (int)s.kw, (int)s.sh, (int)s.sw, (int)s.ph, (int)s.pw,
                      (int)s.cg(), (int)s.cog()};
}

// ---------------------------------------------------------------- scratch that the library owns
// For callers that cannot allocate (code under graph capture, serving loops, harnesses that forbid hipMalloc):
// the split-k partial tiles of pam_hip_pam_matmul_fwd_noalloc go to this array instead of a workspace argument.
// Every GPU the library runs on holds its own copy, at its own address, until the process ends.
constexpr size_t kScratchBytes = (size_t)PAM_HIP_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// The array's address on the current device.  In host code `scratch` is only a stand-in for the symbol, never an
// address to hand to a kernel; the address is looked up once per device, with that device current.
int scratch_address(const char* what, void** ptr)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return pamhost::fail(PAM_HIP_ERR_LAUNCH, "%s: hipGetDevice: %s", what, hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: device %d beyond the %d this entry point keeps scratch for", what, dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return pamhost::fail(PAM_HIP_ERR_LAUNCH, "%s: hipGetSymbolAddress: %s", what, hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return PAM_HIP_OK;
}

}  // namespace

extern "C" {

size_t pam_hip_gemm_workspace_bytes(long batch, long m, long n, long k)
{
    if (batch <= 0 || m <= 0 || n <= 0 || k <= 0) return 0;
    return plan_space(make_plan(batch, m, n, k, true)).total;
}

void pam_hip_set_tuning(int bk, int pieces) { g_force_bk = bk; g_force_pieces = pieces; }

int pam_hip_gemm_plan(long batch, long m, long n, long k, int* k_chunk)
{
    if (batch <= 0 || m <= 0 || n <= 0 || k < 0) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "gemm_plan: bad shape");
    Plan p = make_plan(batch, m, n, k > 0 ? k : 1, true);
    if (k_chunk) *k_chunk = p.piece_kt * p.bk;
    return PAM_HIP_OK;
}

int pam_hip_pam_matmul_fwd(const float* a, long a_sr, long a_sc, const float* b, long b_sr, long b_sc,
                           float* y, long y_sr, long y_sc, long m, long n, long k, float offset,
                           void* workspace, size_t workspace_bytes, void* stream)
{
    return gemm("pam_matmul_fwd", MODE_PAM, 1, m, n, k, a, 0, a_sr, a_sc, b, 0, b_sr, b_sc, nullptr, 0, 0, 0,
                y, 0, y_sr, y_sc, offset, workspace, workspace_bytes, stream);
}

int pam_hip_pam_matmul_fwd_noalloc(const float* a, long a_sr, long a_sc, const float* b, long b_sr, long b_sc,
                                   float* y, long y_sr, long y_sc, long m, long n, long k, float offset, void* stream)
{
    const size_t need = pam_hip_gemm_workspace_bytes(1, m, n, k);
    if (need > kScratchBytes)
        return pamhost::fail(PAM_HIP_ERR_WORKSPACE, "pam_matmul_fwd_noalloc: this shape needs %zu bytes of scratch, the library holds %zu; "
                             "use pam_hip_pam_matmul_fwd with a workspace", need, kScratchBytes);
    void* ws = nullptr;
    if (need > 0) {
        const int rc = scratch_address("pam_matmul_fwd_noalloc", &ws);
        if (rc != PAM_HIP_OK) return rc;
    }
    return gemm("pam_matmul_fwd_noalloc", MODE_PAM, 1, m, n, k, a, 0, a_sr, a_sc, b, 0, b_sr, b_sc, nullptr, 0, 0, 0,
                y, 0, y_sr, y_sc, offset, ws, need, stream);
}

int pam_hip_pam_linear_fwd(const float* a, long a_sr, long a_sc, const float* b, long b_sr, long b_sc, const float* bias,
                           float* y, long y_sr, long y_sc, long m, long n, long k, float offset,
                           void* workspace, size_t workspace_bytes, void* stream)
{
    return gemm("pam_linear_fwd", MODE_PAM, 1, m, n, k, a, 0, a_sr, a_sc, b, 0, b_sr, b_sc, nullptr, 0, 0, 0,
                y, 0, y_sr, y_sc, offset, workspace, workspace_bytes, stream, nullptr, bias);
}

int pam_hip_pam_bmm_fwd(PAM_HIP_MAT(a), PAM_HIP_MAT(b), PAM_HIP_OUT(y), long batch, long m, long n, long k,
                        float offset, void* workspace, size_t workspace_bytes, void* stream)
{
    return gemm("pam_bmm_fwd", MODE_PAM, batch, m, n, k, a, a_sb, a_sr, a_sc, b, b_sb, b_sr, b_sc, nullptr, 0, 0, 0,
                y, y_sb, y_sr, y_sc, offset, workspace, workspace_bytes, stream);
}

int pam_hip_standard_matmul(const float* a, long a_sr, long a_sc, const float* b, long b_sr, long b_sc,
                            float* y, long y_sr, long y_sc, long m, long n, long k, float ignored,
                            void* workspace, size_t workspace_bytes, void* stream)
{
    (void)ignored;
    return gemm("standard_matmul", MODE_STD, 1, m, n, k, a, 0, a_sr, a_sc, b, 0, b_sr, b_sc, nullptr, 0, 0, 0,
                y, 0, y_sr, y_sc, 1.0f, workspace, workspace_bytes, stream);
}

int pam_hip_standard_bmm(PAM_HIP_MAT(a), PAM_HIP_MAT(b), PAM_HIP_OUT(y), long batch, long m, long n, long k,
                         float ignored, void* workspace, size_t workspace_bytes, void* stream)
{
    (void)ignored;
    return gemm("standard_bmm", MODE_STD, batch, m, n, k, a, a_sb, a_sr, a_sc, b, b_sb, b_sr, b_sc, nullptr, 0, 0, 0,
                y, y_sb, y_sr, y_sc, 1.0f, workspace, workspace_bytes, stream);
}

int pam_hip_pam_matmul_bwd(const float* l, long l_sr, long l_sc, const float* r, long r_sr, long r_sc,
                           const float* mo, long mo_sr, long mo_sc, float* dm, long dm_sr, long dm_sc,
                           long m, long n, long k, int delta_l, float offset,
                           void* workspace, size_t workspace_bytes, void* stream)
{
    return gemm("pam_matmul_bwd", delta_l ? MODE_BWD_DL : MODE_BWD_DR, 1, m, n, k, l, 0, l_sr, l_sc, r, 0, r_sr, r_sc,
                mo, 0, mo_sr, mo_sc, dm, 0, dm_sr, dm_sc, offset, workspace, workspace_bytes, stream);
}

int pam_hip_pam_bmm_bwd(PAM_HIP_MAT(l), PAM_HIP_MAT(r), PAM_HIP_MAT(mo), PAM_HIP_OUT(dm),
                        long batch, long m, long n, long k, int delta_l, float offset,
                        void* workspace, size_t workspace_bytes, void* stream)
{
    return gemm("pam_bmm_bwd", delta_l ? MODE_BWD_DL : MODE_BWD_DR, batch, m, n, k, l, l_sb, l_sr, l_sc, r, r_sb, r_sr, r_sc,
                mo, mo_sb, mo_sr, mo_sc, dm, dm_sb, dm_sr, dm_sc, offset, workspace, workspace_bytes, stream);
}

size_t pam_hip_conv2d_workspace_bytes(long batch, long c, long h, long w, long co, long kh, long kw,
                                      long stride_h, long stride_w, long pad_h, long pad_w, long groups, int which, float offset)
{
    ConvShape s{batch, c, h, w, co, kh, kw, stride_h, stride_w, pad_h, pad_w, 0, 0, groups};
    if (conv_shape("conv2d_workspace_bytes", s) != PAM_HIP_OK || batch == 0) return 0;
    if (which == 2) {
        ConvShape t;
        if (input_gradient_shape("conv2d_workspace_bytes", s, t) != PAM_HIP_OK) return 0;
        return input_gradient_space(t).total;
    }
    // (1: the larger of the two weight gradients' needs, whichever the caller then asks for)
    if (which == 1) return std::max(conv_space(s, 1, offset != 1.0f).total, conv_space(s, 2, false).total);
    return conv_space(s, 0, offset != 1.0f).total;
}

int pam_hip_conv2d_bwd_input(const float* dy, const float* w, const float* x, float* dx, long batch, long c, long h, long wd,
                             long co, long kh, long kw, long stride_h, long stride_w, long pad_h, long pad_w, long groups,
                             int exact, float offset, void* workspace, size_t workspace_bytes, void* stream)
{
    ConvShape s{batch, c, h, wd, co, kh, kw, stride_h, stride_w, pad_h, pad_w, 0, 0, groups};
    int rc = conv_shape("conv2d_bwd_input", s);
    if (rc != PAM_HIP_OK) return rc;
    ConvShape t;
    rc = input_gradient_shape("conv2d_bwd_input", s, t);
    if (rc != PAM_HIP_OK) return rc;
    if (batch == 0) return PAM_HIP_OK;
    if (!dy || !w || !dx || (exact && !x)) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "conv2d_bwd_input: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (direct_conv(s)) {                             // the convolution of dy with the flipped weights, directly
        const long total = batch * c * h * wd;
        if (total >= (1L << 31) * 256) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "conv2d_bwd_input: too many outputs");
        const DirectGeom q = direct_geom(t);          // (t: the image is dy, a group's sums run over its filters)
        if (exact) launch_direct_conv<true>(dy, w, x, dx, total, (int)c, q, 1, offset, st);
        else launch_direct_conv<false>(dy, w, nullptr, dx, total, (int)c, q, 1, offset, st);
        return pamhost::check_launch("conv2d_bwd_input");
    }
    ConvSpace sp = input_gradient_space(t);
    ConvGeom cv;
    rc = conv_prepare("conv2d_bwd_input", t, sp, workspace, workspace_bytes, st, cv, false);
    if (rc != PAM_HIP_OK) return rc;
    float* wf = (float*)((char*)workspace + sp.tables);
    const bool one_launch = replicated(t);
    const long copies = one_launch ? batch : 1;
    const long n = c * s.cog() * kh * kw * copies;
    // approximate: the offset goes into the flipped weights; exact: the product kernel applies it to its slope operand
    hipLaunchKernelGGL(flip_weights_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, w, wf, (int)c, (int)s.cog(), (int)s.cg(),
                       (int)kh, (int)kw, offset, (!exact && offset != 1.0f) ? 1 : 0, (int)copies);
    const long K = t.K(), L = t.L();                  // K = (co / groups) kh kw, L = h w
    void* rest = (char*)workspace + sp.tables + sp.scaled; size_t rest_bytes = workspace_bytes - sp.tables - sp.scaled;
    const long hw_out = s.ho * s.wo;
    if (one_launch) {                                 // unit z = image * groups + group (see kReplicateBytes)
        if (exact)
            return gemm("conv2d_bwd_input", MODE_BWD_DR, batch * groups, s.cg(), L, K, wf, s.cg() * K, K, 1, dy, s.cog() * hw_out, 0, 0,
                        x, s.cg() * L, L, 1, dx, s.cg() * L, L, 1, offset, rest, rest_bytes, stream, &cv);
        return gemm("conv2d_bwd_input", MODE_PAM, batch * groups, s.cg(), L, K, wf, s.cg() * K, K, 1, dy, s.cog() * hw_out, 0, 0,
                    nullptr, 0, 0, 0, dx, s.cg() * L, L, 1, 1.0f, rest, rest_bytes, stream, &cv);
    }
    for (long gi = 0; gi < groups; ++gi) {            // one product per group: its filters' gradient slices in, its channels out
        const float* wg = wf + gi * s.cg() * K;
        const float* dyg = dy + gi * s.cog() * hw_out;
        float* dxg = dx + gi * s.cg() * L;
        if (exact)    // dX[c, l] = sum_k pam_bwd(x[c, l], wf[c, k], dY patch[k, l]): x is the same for every term of an output
            rc = gemm("conv2d_bwd_input", MODE_BWD_DR, batch, s.cg(), L, K, wg, 0, K, 1, dyg, co * hw_out, 0, 0, x + gi * s.cg() * L, c * L, L, 1,
                      dxg, c * L, L, 1, offset, rest, rest_bytes, stream, &cv);
        else
            rc = gemm("conv2d_bwd_input", MODE_PAM, batch, s.cg(), L, K, wg, 0, K, 1, dyg, co * hw_out, 0, 0, nullptr, 0, 0, 0,
                      dxg, c * L, L, 1, 1.0f, rest, rest_bytes, stream, &cv);
        if (rc != PAM_HIP_OK) return rc;
    }
    return PAM_HIP_OK;
}

int pam_hip_conv2d_fwd(const float* x, const float* w, float* y, long batch, long c, long h, long wd, long co, long kh, long kw,
                       long stride_h, long stride_w, long pad_h, long pad_w, long groups, float offset,
                       void* workspace, size_t workspace_bytes, void* stream)
{
    ConvShape s{batch, c, h, wd, co, kh, kw, stride_h, stride_w, pad_h, pad_w, 0, 0, groups};
    int rc = conv_shape("conv2d_fwd", s);
    if (rc != PAM_HIP_OK) return rc;
    if (batch == 0) return PAM_HIP_OK;
    if (!x || !w || !y) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "conv2d_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const bool has_off = offset != 1.0f;
    if (direct_conv(s)) {
        const long total = batch * co * s.L();
        if (total >= (1L << 31) * 256) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "conv2d_fwd: too many outputs");
        launch_direct_conv<false>(x, w, nullptr, y, total, (int)co, direct_geom(s), 0, offset, st);
        return pamhost::check_launch("conv2d_fwd");
    }
    ConvSpace sp = conv_space(s, 0, has_off);
    ConvGeom cv;
    rc = conv_prepare("conv2d_fwd", s, sp, workspace, workspace_bytes, st, cv, false);
    if (rc != PAM_HIP_OK) return rc;
    // the reference folds the offset into the weights (the right operand of its product); here the
    // weights are the left operand, so they are scaled once up front
    const float* wl = w;
    const bool one_launch = replicated(s);
    if (has_off || one_launch) {
        float* scaled = (float*)((char*)workspace + sp.tables);
        launch_scale(w, scaled, (size_t)co * s.K(), one_launch ? (size_t)batch : 1, offset, has_off, st);
        wl = scaled;
    }
    const long K = s.K(), L = s.L();
    if (one_launch)                                   // unit z = image * groups + group (see kReplicateBytes)
        return gemm("conv2d_fwd", MODE_PAM, batch * groups, s.cog(), L, K, wl, s.cog() * K, K, 1, x, s.cg() * h * wd, 0, 0,
                    nullptr, 0, 0, 0, y, s.cog() * L, L, 1, 1.0f,
                    (char*)workspace + sp.tables + sp.scaled, workspace_bytes - sp.tables - sp.scaled, stream, &cv);
    // per image and group: Y[co, l] = sum_k W[co, k] (*) patches[k, l] over the group's channels
    for (long gi = 0; gi < groups; ++gi) {
        rc = gemm("conv2d_fwd", MODE_PAM, batch, s.cog(), L, K, wl + gi * s.cog() * K, 0, K, 1, x + gi * s.cg() * h * wd, c * h * wd, 0, 0,
                  nullptr, 0, 0, 0, y + gi * s.cog() * L, co * L, L, 1, 1.0f,
                  (char*)workspace + sp.tables + sp.scaled, workspace_bytes - sp.tables - sp.scaled, stream, &cv);
        if (rc != PAM_HIP_OK) return rc;
    }
    return PAM_HIP_OK;
}

int pam_hip_conv2d_bwd_weight(const float* x, const float* dy, const float* w, float* dw, long batch, long c, long h, long wd,
                              long co, long kh, long kw, long stride_h, long stride_w, long pad_h, long pad_w, long groups,
                              int exact, float offset, void* workspace, size_t workspace_bytes, void* stream)
{
    ConvShape s{batch, c, h, wd, co, kh, kw, stride_h, stride_w, pad_h, pad_w, 0, 0, groups};
    int rc = conv_shape("conv2d_bwd_weight", s);
    if (rc != PAM_HIP_OK) return rc;
    if (batch == 0) return PAM_HIP_OK;
    if (!x || !dy || !dw || (exact && !w)) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "conv2d_bwd_weight: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (direct_conv(s)) {
        // the sum over the output positions in the chunks the matrix kernel would cut it into (given its workspace)
        const Plan p = make_plan(batch * groups, s.cog(), s.K(), s.L(), true);
        const int chunk = p.pieces > 1 ? p.piece_kt * p.bk : (int)std::min<long>(s.L(), 1L << 30);
        const long total = batch * co * s.K();
        const dim3 grid((unsigned)((total + 255) / 256));
        if (exact) hipLaunchKernelGGL(direct_conv_weight_kernel<true>, grid, dim3(256), 0, st, x, dy, w, dw, total, (int)co, direct_geom(s), chunk, offset, offset != 1.0f ? 1 : 0);
        else hipLaunchKernelGGL(direct_conv_weight_kernel<false>, grid, dim3(256), 0, st, x, dy, (const float*)nullptr, dw, total, (int)co, direct_geom(s), chunk, offset, offset != 1.0f ? 1 : 0);
        return pamhost::check_launch("conv2d_bwd_weight");
    }
    const bool scale = offset != 1.0f && !exact;
    ConvSpace sp = conv_space(s, exact ? 2 : 1, scale);
    ConvGeom cv;
    rc = conv_prepare("conv2d_bwd_weight", s, sp, workspace, workspace_bytes, st, cv, true);
    if (rc != PAM_HIP_OK) return rc;
    const long K = s.K(), L = s.L();
    void* rest = (char*)workspace + sp.tables + sp.scaled; size_t rest_bytes = workspace_bytes - sp.tables - sp.scaled;
    // approximate: dW[co, k] = sum_l patches[k, l] (*) (dY[co, l] (*) offset), the gradient scaled once up front
    const float* dl = dy;
    if (scale) {
        float* scaled = (float*)((char*)workspace + sp.tables);
        launch_scale(dy, scaled, (size_t)batch * co * L, 1, offset, true, st);
        dl = scaled;
    }
    // grouped: unit z = image * groups + group (see kReplicateBytes); only the exact gradient reads the weights
    if (groups > 1 && !exact)
        return gemm("conv2d_bwd_weight", MODE_PAM, batch * groups, s.cog(), K, L, dl, s.cog() * L, L, 1, x, s.cg() * h * wd, 0, 0,
                    nullptr, 0, 0, 0, dw, s.cog() * K, K, 1, 1.0f, rest, rest_bytes, stream, &cv);
    if (groups > 1 && replicated(s)) {
        float* copies = (float*)((char*)workspace + sp.tables);
        launch_scale(w, copies, (size_t)co * K, (size_t)batch, 1.0f, false, st);
        return gemm("conv2d_bwd_weight", MODE_BWD_DL, batch * groups, s.cog(), K, L, dy, s.cog() * L, L, 1, x, s.cg() * h * wd, 0, 0,
                    copies, s.cog() * K, K, 1, dw, s.cog() * K, K, 1, offset, rest, rest_bytes, stream, &cv);
    }
    for (long gi = 0; gi < groups; ++gi) {
        const float* xg = x + gi * s.cg() * h * wd;
        float* dwg = dw + gi * s.cog() * K;
        if (exact)    // dW[co, k] = sum_l pam_bwd(W[co, k], patches[k, l], dY[co, l]); the offset goes with the patches
            rc = gemm("conv2d_bwd_weight", MODE_BWD_DL, batch, s.cog(), K, L, dy + gi * s.cog() * L, co * L, L, 1, xg, c * h * wd, 0, 0,
                      w + gi * s.cog() * K, 0, K, 1, dwg, co * K, K, 1, offset, rest, rest_bytes, stream, &cv);
        else
            rc = gemm("conv2d_bwd_weight", MODE_PAM, batch, s.cog(), K, L, dl + gi * s.cog() * L, co * L, L, 1, xg, c * h * wd, 0, 0,
                      nullptr, 0, 0, 0, dwg, co * K, K, 1, 1.0f, rest, rest_bytes, stream, &cv);
        if (rc != PAM_HIP_OK) return rc;
    }
    return PAM_HIP_OK;
}

}  // extern "C"
