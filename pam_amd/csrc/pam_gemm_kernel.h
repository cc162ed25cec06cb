// PAM matrix products for gfx950: Y[b,i,j] = sum_k mul(L[b,i,k], R[b,k,j]).
//
// A PAM product is an integer add of the two bit patterns (pam/cuda_kernels.cu:17-19),
// so the matrix cores do not apply; this is a VALU kernel whose inner loop is, per
// multiply-accumulate, one v_add_u32 and one v_add_f32.
//
//  * A work-group of four wavefronts owns a 64 x 64 tile of Y.  Each lane owns a 4 x 4
//    micro-tile in registers, each wavefront 16 x 64 outputs (lane_place below).  Measured on
//    MI355X, a SIMD retires a wave64 VALU instruction every two cycles but one wavefront
//    issues at most one every four, so several wavefronts per SIMD are needed (four are
//    resident: at most 128 registers, 35 KB of LDS per work-group with 32-deep k-tiles); larger
//    micro-tiles and more resident wavefronts were measured and gained nothing.  Thousands
//    of equal work-groups per product are what balances the 256 compute units.
//  * L and R tiles are staged through LDS k-major ([k][row], 4-word row pad), so a fragment
//    for one k is two ds_read_b128, contiguous (R) or broadcast (L) across the wavefront.
//    Operands whose contiguous dimension is k (row-major L, "column-major" R) are
//    transposed on the way in; operands contiguous along the row use 128-bit LDS writes;
//    anything else goes through a scalar loader.  In a 32-deep tile the lines k = 16 ... 31
//    keep their 8-row groups exchanged (row ^ 8, `swizzled`): the transposing writes of the
//    two k halves then fall into different banks (a third of the bank-conflict cycles of the
//    plain layout).  No transposed copies are made in global
//    memory, so the backward products run on the views the autograd layer hands over
//    (pam/cuda_bindings.py:147-164).
//  * Global loads for k-tile t+1 are issued before the arithmetic of tile t (register
//    double buffering), LDS is double buffered, one barrier per k-tile, and inside a k-tile
//    the fragments of step k+1 are read while step k is computed.  k-tiles are 32 deep for
//    long k and 16 deep for short k.
//  * The bias subtraction and the optional offset (R' = R (*) offset) are applied once per
//    element while staging R.
//  * Staging begins with a quick test, one shift-add per value folded by max: if all of a k-tile's L and R
//    values are normal numbers with magnitude in [2^-63, 2^64), no product in the tile can leave the normal
//    range and the two-instruction loop is exact; such a tile is stored as it is.  Only a tile that fails is
//    classified value by value.  Its full k-tiles that only add zeros to that (ReLU activations, padding,
//    pruned weights) keep two instructions per product and skip the products with a zero under the
//    execution mask (a PAM product with a zero is +0, and adding it changes nothing); anything else
//    (subnormals, inf, NaN, extreme exponents) makes its k-tile choose per k-step: the steps that hold such
//    a value evaluate the full definition per product on operands decomposed once per k-step, the others
//    take the plain form, or the zero-replacing one if the tile holds zeros too.  The choices are uniform per work-group.
//  * The products of a full in-range k-tile are written out in assembly, sixteen per k-step, and take the
//    LDS addresses as in-out operands: given the unrolled k-tile as one block, the compiler issues all of
//    its LDS reads first and spills.
//  * Rows beyond M / N are clamped to the last valid row when loading (their results are
//    never stored); the k tail runs a shorter loop, padding never enters the arithmetic.
//  * Shapes with few output tiles and long k (dX: 12608 x 192, k = 768; dW: 192 x 768,
//    k = 12608) cut every tile's k range into pieces, one work-group each; the last
//    work-group to finish a piece of a tile adds the pieces up and writes the tile ("the
//    units of a launch" below), a second kernel does where the pieces are many.
//  * The launch is one-dimensional over the units and every XCD (own L2)
//    takes one contiguous range of them, so each operand is fetched from memory about once.
//  * The right operand may be the patches of an image read in place (convolutions), and a
//    bias may be added to the finished sums (linear layers).
//  * Accumulation order: every output is summed by one lane per k chunk (piece), k ascending,
//    from +0, and the chunks' sums are added in ascending order from +0 -- with one chunk
//    this is the order of the reference kernel (pam/cuda_kernels.cu:601, 608-627);
//    pam_hip_gemm_plan reports the chunk length.
#pragma once
#include <cmath>
#include <cstring>
#include <type_traits>

#include "pam_common.h"
#include "pam_device.h"

namespace pamgemm {
using namespace pamdev;

enum { MODE_PAM = 0, MODE_STD = 1, MODE_BWD_DL = 2, MODE_BWD_DR = 3 };
enum { LOAD_KVEC = 0, LOAD_RVEC = 1, LOAD_ANY = 2, LOAD_CONV = 3, LOAD_CONVQ = 4, LOAD_CONVR = 5, LOAD_CONVK = 6 };   // k contiguous / row contiguous / any strides / image patches / ... in quads along k / ... in quads of output positions / the same, transposed

constexpr int KGRAN = 32;         // k ranges handed to work-groups are multiples of this
constexpr int PAD = 4;
// gfx950 parts (MI350X, MI355X) have eight XCDs, each with its own L2, and work-groups are dealt to them in turn.
// The unit mapping built on this is a bijection for any count, so only locality depends on it.
constexpr int XCDS = 8;

struct Operand { const float* p; long sb, sr, sk; };    // batch, row (the non-k index), k strides

// The right operand as the patches of an image, never materialised (the reference unfolds them
// into a [C kh kw, Ho Wo] matrix per image, pam/pam_ops.py:118-160): entry (k, l) of that matrix
// is x[c, h0(l) + di(k), w0(l) + dj(k)], zero outside the image.  Two small tables hold, per k
// and per l, the address part and the coordinates: {c H W + di W + dj, di << 16 | dj} and
// {h0 W + w0, h0 << 16 | (w0 & 0xffff)}.  `transposed` exchanges the roles of the operand's two
// indices (the matrix is then [Ho Wo, C kh kw]: the weight-gradient product).
// `quads`: no padding, and the kernel's width, the image's width and the horizontal stride are multiples of four (the
// patch embeddings of vision transformers: 16 x 16 patches at stride 16): four consecutive k of one patch are then four
// consecutive, 16-byte aligned values of an image row and always inside the image, and the loader fetches them as one.
// `row_quads`: horizontal stride 1 and an output width that is a multiple of four: four consecutive output positions are
// then four consecutive pixels of one image row under every k, and the loader works out one address and one row test per
// four values and hands the staging 128-bit vectors along the positions (padding allowed: the ends of a row are tested
// per value).
struct ConvGeom { const int2* ktab; const int2* ltab; int H, W; int transposed; int quads; int row_quads; };

struct GemmArgs {
    Operand L, R;
    ConvGeom cv;
    const float* D; long d_sb, d_sr, d_sc;
    float* Y; long y_sb, y_sr, y_sc;
    const float* bias;           // one value per output column, added once after the sum, or null
    int M, N, K;
    int tiles, ntn;              // output tiles per matrix; tiles per row of tiles (consecutive tiles share rows of L)
    int pieces, piece_kt;        // k ranges a tile is cut into (1: whole tiles) and their length in k-tiles
    int units;                   // tiles of all matrices x pieces: one work-group each
    int xcd_chunk;               // > 0: work-group x takes unit (x % XCDS) * xcd_chunk + x / XCDS, else unit x
    int fold_here;               // cut tiles are added up by the work-group that arrives last (else by a second kernel)
    unsigned long long* arrive;  // cut tiles: one arrival word per tile
    unsigned long long tag;      // cut tiles: this launch's tag in the arrival words (40 bits)
    float* partial;              // cut tiles: one piece (64 x 64 sums) per unit
    float off; int has_off;      // has_off: 0 none, 1 a normal number (off_add = its bit-pattern increment), 2 any other value
    uint32_t off_add;
};

// Classifies and transforms one staged value.  MODE_PAM: R carries the bias subtraction, and
// zeros are staged in one canonical pattern (their sign never shows in a sum that starts at +0).
// Backward modes: the "slope side" is the forward operand b of pam_bwd(a, b, delta).
constexpr uint32_t kZeroL = 0u;                 // canonical staged zero of L
constexpr uint32_t kZeroR = 0u - kBias;         // canonical staged zero of R (bias already subtracted)

template <int MODE, bool IS_R>
struct Stager {
    static constexpr bool kSlopeSide = (MODE == MODE_BWD_DL && IS_R) || (MODE == MODE_BWD_DR && !IS_R);
    static constexpr bool kDeltaSide = (MODE >= MODE_BWD_DL) && !kSlopeSide;
    static constexpr bool kTakesOffset = (MODE == MODE_PAM && IS_R) || kSlopeSide;
    bool bad = false, zero = false;
    ExponentRange seen;
    __device__ __forceinline__ uint32_t one(float v)
    {
        uint32_t u = f2u(v);
        if (MODE == MODE_STD) return u;
        if (MODE == MODE_PAM) {                    // zeros get their own, cheaper loop
            const bool z = (u & ~kSign) == 0;
            zero |= z;
            seen.see(u, z);
            return z ? (IS_R ? kZeroR : kZeroL) : (IS_R ? u - kBias : u);
        }
        bad |= needs_full_definition(u);
        // Backward modes.  The upstream gradient: zero is harmless.  The slope side: a zero needs no care either,
        // (0 + fraction) & ~mantissa is 0 and the fma then adds delta * 0 (delta is finite in the plain loop), which
        // is what the definition gives.
        return u;
    }
    // some staged value lies outside [2^-63, 2^64) or is not a normal number or zero
    __device__ __forceinline__ bool out_of_range() const { return bad || (MODE == MODE_PAM && seen.needs_full_definition()); }
};

// Staging when the quick test below has passed: every value of the k-tile is a normal number in
// [2^-63, 2^64), so the transformed value is an integer add (the bias subtraction and a normal offset).
template <bool ADDS>
struct PlainStager {
    uint32_t add;
    __device__ __forceinline__ uint32_t one(float v) const { return ADDS ? f2u(v) + add : f2u(v); }
};

// Quick test of a staged value: (bits << 1) - (64 << 24) is below 127 << 24 exactly for the normal numbers
// with biased exponent 64 ... 190, whatever the sign.  One shift-add per value, the results folded by max.
constexpr uint32_t kWindowBase = 0u - (64u << 24), kWindowSpan = 127u << 24;
__device__ __forceinline__ uint32_t window(uint32_t u) { return (u << 1) + kWindowBase; }
__device__ __forceinline__ uint32_t max3u(uint32_t a, uint32_t b, uint32_t c) { return max(max(a, b), c); }

// Verdict of a k-tile: bit 0 / bit 1 = the left / right operand holds zeros (all else in range),
// kGuarded = some value needs the full definition.  Verdicts of wavefronts combine by OR.
constexpr uint32_t kZerosL = 1u, kZerosR = 2u, kGuarded = 4u;
// A wavefront none of whose outputs exist (see lane_place) stages and synchronises with the others but computes nothing.
constexpr uint32_t kIdle = 8u;

// Stand-ins that keep the integer sum a finite number when one operand is zero: 2^-64 on the
// left, 2^64 (less the bias) on the right, just outside the range [2^-63, 2^64) that the other
// values of such a k-tile lie in.  The product is then multiplied by 0.
constexpr uint32_t kStandInL = 63u << 23;
constexpr uint32_t kStandInR = 64u << 23;

// Where row `row` of k-step `k` sits within the k-step's line of a staged tile.  A 32-deep tile's lines 16 ... 31 have
// their 8-row groups exchanged in pairs (row ^ 8): the transposing writes of an operand whose contiguous dimension is k
// put a wavefront's eight k-quads at line distances that are multiples of 16 x (64 + 4) words = 0 mod 64 banks, so quads
// q and q + 4 would meet in the same banks; with the exchange they do not, and groups of four rows stay together for the
// 128-bit reads.
template <int BK>
__device__ __forceinline__ int swizzled(int row, int k) { return BK == 32 ? row ^ ((k & 16) >> 1) : row; }

// One operand's tile: ROWS x BK values from global memory into registers, then into LDS.
template <int ROWS, int NT, int KIND, int BK>
struct TileLoader {
    static constexpr int kVecs = ROWS * BK / 4 / NT;      // float4 per lane (vector kinds)
    static constexpr int kElems = ROWS * BK / NT;         // scalars per lane (generic kind)
    static_assert(ROWS * BK % (4 * NT) == 0 && NT % ROWS == 0, "tile must divide over the work-group");
    static constexpr bool kKQuads = KIND == LOAD_KVEC || KIND == LOAD_CONVQ || KIND == LOAD_CONVK;      // 128-bit loads along k
    static constexpr bool kRQuads = KIND == LOAD_RVEC || KIND == LOAD_CONVR;      // ... along the rows
    float4 v[kVecs > 0 ? kVecs : 1];
    int2 fixed; bool have_fixed = false;          // LOAD_CONV: the lane's own table entry
    int patch_at[kVecs > 0 ? kVecs : 1];          // LOAD_CONVQ: where the patches of the lane's rows begin in the image
    int2 row_entry[KIND == LOAD_CONVK && kVecs > 0 ? kVecs : 1];      // LOAD_CONVK: the k table's entries of the lane's rows

    __device__ __forceinline__ void load(const Operand& op, const float* base, int row0, int nrows, int k0, int kend, int tid,
                                         const ConvGeom& cv)
    {
        if (KIND == LOAD_CONV) {
            float* s = reinterpret_cast<float*>(v);
            // Every element of a lane has the same row (NT is a multiple of ROWS): one table entry,
            // fetched once per work-group.  The k index is the same for a whole wavefront (ROWS is
            // the wavefront size), so its table entry comes through the scalar unit.
            if (!have_fixed) {
                const int row = min(row0 + tid % ROWS, nrows - 1);
                fixed = cv.transposed ? cv.ktab[row] : cv.ltab[row];
                have_fixed = true;
            }
            const int kwave = __builtin_amdgcn_readfirstlane(tid / ROWS);
            // the tables are written before the launch and only read here: constant address space
            typedef const __attribute__((address_space(4))) int* ConstTable;
            ConstTable mtab = (ConstTable)(cv.transposed ? cv.ltab : cv.ktab);
#pragma unroll
            for (int i = 0; i < kElems; ++i) {
                const int kk = min(k0 + kwave + i * (NT / ROWS), kend - 1);
                const int2 moving = make_int2(mtab[2 * kk], mtab[2 * kk + 1]);
                const int2 ke = cv.transposed ? fixed : moving, le = cv.transposed ? moving : fixed;
                const int h = (le.y >> 16) + (ke.y >> 16), w = (int)(short)(le.y & 0xffff) + (ke.y & 0xffff);
                const bool inside = (unsigned)h < (unsigned)cv.H && (unsigned)w < (unsigned)cv.W;
                s[i] = inside ? base[ke.x + le.x] : 0.0f;
            }
        } else if (KIND == LOAD_CONVR) {
            // as LOAD_RVEC: vector i holds rows rq * 4 ... + 3 (four output positions of one image row) under one k
            if (!have_fixed) {
                fixed = cv.ltab[min(row0 + (tid % (ROWS / 4)) * 4, nrows - 4)];          // (the same rows for every vector of the lane)
                have_fixed = true;
            }
            static_assert(NT % (ROWS / 4) == 0, "a lane's vectors must share their rows");
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                const int kk = min(k0 + (tid + i * NT) / (ROWS / 4), kend - 1);
                const int2 ke = cv.ktab[kk];
                const int h = (fixed.y >> 16) + (ke.y >> 16), w = (int)(short)(fixed.y & 0xffff) + (ke.y & 0xffff);
                const bool row_inside = (unsigned)h < (unsigned)cv.H;
                const float* at = base + (ke.x + fixed.x);
                v[i].x = row_inside && (unsigned)w < (unsigned)cv.W ? at[0] : 0.0f;
                v[i].y = row_inside && (unsigned)(w + 1) < (unsigned)cv.W ? at[1] : 0.0f;
                v[i].z = row_inside && (unsigned)(w + 2) < (unsigned)cv.W ? at[2] : 0.0f;
                v[i].w = row_inside && (unsigned)(w + 3) < (unsigned)cv.W ? at[3] : 0.0f;
            }
        } else if (KIND == LOAD_CONVK) {
            // the transposed patches of a `row_quads` convolution (its weight gradient): the rows are (c, i, j) and k runs
            // over the output positions, four consecutive ones per vector as in LOAD_CONVR, staged as LOAD_KVEC is
            if (!have_fixed) {
#pragma unroll
                for (int i = 0; i < kVecs; ++i) row_entry[i] = cv.ktab[min(row0 + (tid + i * NT) / (BK / 4), nrows - 1)];
                have_fixed = true;
            }
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                const int2 le = cv.ltab[min(k0 + ((tid + i * NT) % (BK / 4)) * 4, kend - 4)], ke = row_entry[i];
                const int h = (le.y >> 16) + (ke.y >> 16), w = (int)(short)(le.y & 0xffff) + (ke.y & 0xffff);
                const bool row_inside = (unsigned)h < (unsigned)cv.H;
                const float* at = base + (ke.x + le.x);
                v[i].x = row_inside && (unsigned)w < (unsigned)cv.W ? at[0] : 0.0f;
                v[i].y = row_inside && (unsigned)(w + 1) < (unsigned)cv.W ? at[1] : 0.0f;
                v[i].z = row_inside && (unsigned)(w + 2) < (unsigned)cv.W ? at[2] : 0.0f;
                v[i].w = row_inside && (unsigned)(w + 3) < (unsigned)cv.W ? at[3] : 0.0f;
            }
        } else if (KIND == LOAD_CONVQ) {
            // as LOAD_KVEC, the address from the two tables: the rows' entries once per work-group, k's per k-tile
            typedef const __attribute__((address_space(4))) int* ConstTable;
            if (!have_fixed) {
#pragma unroll
                for (int i = 0; i < kVecs; ++i) patch_at[i] = cv.ltab[min(row0 + (tid + i * NT) / (BK / 4), nrows - 1)].x;
                have_fixed = true;
            }
            ConstTable ktab = (ConstTable)cv.ktab;
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                const int k = min(k0 + ((tid + i * NT) % (BK / 4)) * 4, kend - 4);
                v[i] = *reinterpret_cast<const float4*>(base + patch_at[i] + ktab[2 * k]);
            }
        } else if (KIND == LOAD_KVEC) {
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                int id = tid + i * NT;
                int r = id / (BK / 4), kq = id % (BK / 4);
                int row = min(row0 + r, nrows - 1);
                int k = min(k0 + kq * 4, kend - 4);
                v[i] = *reinterpret_cast<const float4*>(base + (long)row * op.sr + k);
            }
        } else if (KIND == LOAD_RVEC) {
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                int id = tid + i * NT;
                int k = id / (ROWS / 4), rq = id % (ROWS / 4);
                int row = min(row0 + rq * 4, nrows - 4);
                int kk = min(k0 + k, kend - 1);
                v[i] = *reinterpret_cast<const float4*>(base + (long)kk * op.sk + row);
            }
        } else {
            float* s = reinterpret_cast<float*>(v);
#pragma unroll
            for (int i = 0; i < kElems; ++i) {
                int id = tid + i * NT;
                int k = id / ROWS, r = id % ROWS;
                int row = min(row0 + r, nrows - 1);
                int kk = min(k0 + k, kend - 1);
                s[i] = base[(long)row * op.sr + (long)kk * op.sk];
            }
        }
    }

    // max over the tile's values of window(bits), and of window(bits + add) too when `shifted`
    // (an operand that takes a normal offset must be in range before and after it)
    __device__ __forceinline__ uint32_t window_max(bool shifted, uint32_t add) const
    {
        constexpr int n = (kKQuads || kRQuads) ? 4 * kVecs : kElems;
        const float* s = reinterpret_cast<const float*>(v);
        uint32_t m = 0;
#pragma unroll
        for (int i = 0; i + 1 < n; i += 2) m = max3u(m, window(f2u(s[i])), window(f2u(s[i + 1])));
        if (n % 2) m = max(m, window(f2u(s[n - 1])));
        if (shifted) {
#pragma unroll
            for (int i = 0; i + 1 < n; i += 2) m = max3u(m, window(f2u(s[i]) + add), window(f2u(s[i + 1]) + add));
            if (n % 2) m = max(m, window(f2u(s[n - 1]) + add));
        }
        return m;
    }

    // R' = R (*) offset, once per element (uniform branch around the whole tile)
    __device__ __forceinline__ void apply_offset(float off)
    {
        // fully unrolled: a run-time index would push the register tile into scratch memory
#pragma unroll
        for (int i = 0; i < (kVecs > 0 ? kVecs : 1); ++i) {
            v[i].x = pam_mul(v[i].x, off); v[i].y = pam_mul(v[i].y, off);
            v[i].z = pam_mul(v[i].z, off); v[i].w = pam_mul(v[i].w, off);
        }
    }

    // For a k-tile that holds a value in need of the full definition (rare): under which k of the tile the lane's
    // values of that kind sit, bit k for k.  The same walk over the register tile as store().
    __device__ __forceinline__ void odd_by_k(int tid, uint32_t& odd) const
    {
        auto see = [&](float f, int k) __attribute__((always_inline)) { odd |= (uint32_t)needs_full_definition(f2u(f)) << k; };
        if (kKQuads) {
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                const int k = ((tid + i * NT) % (BK / 4)) * 4;
                see(v[i].x, k); see(v[i].y, k + 1); see(v[i].z, k + 2); see(v[i].w, k + 3);
            }
        } else if (kRQuads) {
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                const int k = (tid + i * NT) / (ROWS / 4);
                see(v[i].x, k); see(v[i].y, k); see(v[i].z, k); see(v[i].w, k);
            }
        } else {
            const float* s = reinterpret_cast<const float*>(v);
#pragma unroll
            for (int i = 0; i < kElems; ++i) see(s[i], (tid + i * NT) / ROWS);
        }
    }

    template <class S>
    __device__ __forceinline__ void store(uint32_t* lds, int tid, S& st)
    {
        constexpr int LD = ROWS + PAD;
        if (kKQuads) {
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                int id = tid + i * NT;
                uint32_t* d = lds + ((id % (BK / 4)) * 4) * LD + swizzled<BK>(id / (BK / 4), (id % (BK / 4)) * 4);
                d[0 * LD] = st.one(v[i].x); d[1 * LD] = st.one(v[i].y);
                d[2 * LD] = st.one(v[i].z); d[3 * LD] = st.one(v[i].w);
            }
        } else if (kRQuads) {
            // (vector i of a lane sits under k = i * kPer + tid / (ROWS / 4), the second term below kPer: which half of a
            // 32-deep tile that is depends on i alone, so the exchange of the row groups costs nothing per vector)
            constexpr int kPer = NT / (ROWS / 4);
            static_assert(16 % kPer == 0, "a lane's vectors must not straddle the tile's k halves");
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                uint4 w;
                w.x = st.one(v[i].x); w.y = st.one(v[i].y); w.z = st.one(v[i].z); w.w = st.one(v[i].w);
                *reinterpret_cast<uint4*>(lds + (i * kPer + tid / (ROWS / 4)) * LD + swizzled<BK>((tid % (ROWS / 4)) * 4, i * kPer)) = w;
            }
        } else {                                    // LOAD_ANY and LOAD_CONV: lane-consecutive rows
            const float* s = reinterpret_cast<const float*>(v);
            // (element i of a lane sits under k = i * (NT / ROWS) + tid / ROWS: its half of the tile depends on i alone too)
            static_assert(16 % (NT / ROWS) == 0, "a lane's elements must not straddle the tile's k halves");
            const int row = tid % ROWS, kwave = tid / ROWS;
#pragma unroll
            for (int i = 0; i < kElems; ++i)
                lds[(i * (NT / ROWS) + kwave) * LD + swizzled<BK>(row, i * (NT / ROWS))] = st.one(s[i]);
        }
    }
};

// Per-lane choice by a wavefront mask (as __ballot returns it): one v_cndmask, kept opaque so that the
// 0 / 1 factor of the zero-skipping loops stays a factor and is not turned back into a select per product.
__device__ __forceinline__ uint32_t pick(uint64_t mask, uint32_t if_clear, uint32_t if_set)
{
    uint32_t r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(if_clear), "v"(if_set), "s"(mask));
    return r;
}

// Exact-backward product from the normalised mantissa fraction of the forward operand
// whose gradient is wanted, the other forward operand b (offset already applied) and the
// upstream gradient (pam/cuda_kernels.cu:48-57, pam/native.py:74-77), all classes.
__device__ __noinline__ float bwd_product_general(uint32_t frac_a, uint32_t bi, float delta)
{
    uint32_t mb = bi & ~kSign;
    if (mb > kExpo) return u2f(kQNaN);
    float sgn, p;
    if (mb == 0) { sgn = 0.0f; p = 0.0f; }
    else if (mb == kExpo) { sgn = (bi & kSign) ? -1.0f : 1.0f; p = u2f(kExpo); }
    else {
        int eb; uint32_t fb; split_mag(mb, eb, fb);
        sgn = (bi & kSign) ? -1.0f : 1.0f;
        p = pow2_int(eb + (int)((frac_a + fb) >> 23));
    }
    float t = delta * sgn;
    return t * p;
}

__device__ __forceinline__ uint32_t normalised_fraction(float d)
{
    uint32_t mag = f2u(d) & ~kSign;
    if (mag == 0 || mag >= kExpo) return 0;       // zero; inf/NaN never carry (their fraction compares false)
    int e; uint32_t m; split_mag(mag, e, m);
    return m;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(3))) u32x4* LdsVec;

// 16 PAM products of a 4 x 4 micro-tile added to their accumulators: v_add_u32 + v_add_f32 each, the integer add
// of the next product issued ahead of the float add of the current one.  Written out because the compiler, given
// the unrolled k-tile as one block, moves all of its LDS reads to the top and spills; the LDS addresses pass
// through (unchanged) so that the reads of the step after next cannot be issued before this block.
#define PAM_ACC_OPERANDS                                                                                      \
    [c00] "+v"(acc[0][0]), [c01] "+v"(acc[0][1]), [c02] "+v"(acc[0][2]), [c03] "+v"(acc[0][3]),               \
    [c10] "+v"(acc[1][0]), [c11] "+v"(acc[1][1]), [c12] "+v"(acc[1][2]), [c13] "+v"(acc[1][3]),               \
    [c20] "+v"(acc[2][0]), [c21] "+v"(acc[2][1]), [c22] "+v"(acc[2][2]), [c23] "+v"(acc[2][3]),               \
    [c30] "+v"(acc[3][0]), [c31] "+v"(acc[3][1]), [c32] "+v"(acc[3][2]), [c33] "+v"(acc[3][3])
#define PAM_FRAGMENT_OPERANDS \
    [a0] "v"(a.x), [a1] "v"(a.y), [a2] "v"(a.z), [a3] "v"(a.w), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w)
#define PAM_MAC_ROW(I)                                              \
    "v_add_u32 %[t1], %[a" #I "], %[b1]\n v_add_f32 %[c" #I "0], %[c" #I "0], %[t0]\n" \
    "v_add_u32 %[t0], %[a" #I "], %[b2]\n v_add_f32 %[c" #I "1], %[c" #I "1], %[t1]\n" \
    "v_add_u32 %[t1], %[a" #I "], %[b3]\n v_add_f32 %[c" #I "2], %[c" #I "2], %[t0]\n"
#define PAM_MAC_BODY                                                                  \
    "v_add_u32 %[t0], %[a0], %[b0]\n"                                                 \
    PAM_MAC_ROW(0) "v_add_u32 %[t0], %[a1], %[b0]\n v_add_f32 %[c03], %[c03], %[t1]\n" \
    PAM_MAC_ROW(1) "v_add_u32 %[t0], %[a2], %[b0]\n v_add_f32 %[c13], %[c13], %[t1]\n" \
    PAM_MAC_ROW(2) "v_add_u32 %[t0], %[a3], %[b0]\n v_add_f32 %[c23], %[c23], %[t1]\n" \
    PAM_MAC_ROW(3) "v_add_f32 %[c33], %[c33], %[t1]\n"
__device__ __forceinline__ void pam_mac_4x4(float (&acc)[4][4], const u32x4& a, const u32x4& b, uint32_t& pl, uint32_t& pr)
{
    uint32_t t0, t1;
    asm volatile(PAM_MAC_BODY
                 : PAM_ACC_OPERANDS, [t0] "=&v"(t0), [t1] "=&v"(t1), [pl] "+v"(pl), [pr] "+v"(pr)
                 : PAM_FRAGMENT_OPERANDS);
}

// The same block under a wavefront-uniform lane mask `run` (all ones or zero): with zero the instructions issue and
// change nothing.  For a loop whose k-steps are of two kinds, so that the accumulators pass through the same
// statement in every step and keep their registers (a branch around the statement made the compiler copy all sixteen
// before and after it).
__device__ __forceinline__ void pam_mac_4x4_under(float (&acc)[4][4], const u32x4& a, const u32x4& b, uint32_t& pl, uint32_t& pr,
                                                  uint64_t run)
{
    uint32_t t0, t1;
    uint64_t all;
    asm volatile("s_mov_b64 %[all], exec\n s_and_b64 exec, exec, %[run]\n" PAM_MAC_BODY "s_mov_b64 exec, %[all]\n"
                 : PAM_ACC_OPERANDS, [t0] "=&v"(t0), [t1] "=&v"(t1), [all] "=&s"(all), [pl] "+v"(pl), [pr] "+v"(pr)
                 : PAM_FRAGMENT_OPERANDS, [run] "s"(run)
                 : "scc");
}
#undef PAM_MAC_BODY
#undef PAM_MAC_ROW

// The same sixteen products for a k-tile whose LEFT (else right) operand holds zeros next to in-range values.  A PAM
// product with a zero is +0 and adding it changes nothing (the sums start at +0 and never become -0), so those
// products are not executed: per value of the operand with zeros one compare narrows the execution mask to the lanes
// whose value is not the staged zero, the four products of that value run under it, and the mask is restored.  Two
// instructions per product as in the plain block plus one compare per four products.
template <bool LEFT>
__device__ __forceinline__ void pam_mac_4x4_skip(float (&acc)[4][4], const u32x4& a, const u32x4& b, uint32_t& pl, uint32_t& pr)
{
    uint32_t t0, t1, t2, t3;
    uint64_t all;
    if (LEFT) {
#define PAM_SKIP_ROW(I)                                                                         \
    "v_cmpx_ne_u32_e32 vcc, 0, %[a" #I "]\n"                                                     \
    "v_add_u32 %[t0], %[a" #I "], %[b0]\n v_add_u32 %[t1], %[a" #I "], %[b1]\n"                  \
    "v_add_u32 %[t2], %[a" #I "], %[b2]\n v_add_u32 %[t3], %[a" #I "], %[b3]\n"                  \
    "v_add_f32 %[c" #I "0], %[c" #I "0], %[t0]\n v_add_f32 %[c" #I "1], %[c" #I "1], %[t1]\n"    \
    "v_add_f32 %[c" #I "2], %[c" #I "2], %[t2]\n v_add_f32 %[c" #I "3], %[c" #I "3], %[t3]\n"    \
    "s_mov_b64 exec, %[all]\n"
        asm volatile(
            "s_mov_b64 %[all], exec\n" PAM_SKIP_ROW(0) PAM_SKIP_ROW(1) PAM_SKIP_ROW(2) PAM_SKIP_ROW(3)
            : [c00] "+v"(acc[0][0]), [c01] "+v"(acc[0][1]), [c02] "+v"(acc[0][2]), [c03] "+v"(acc[0][3]),
              [c10] "+v"(acc[1][0]), [c11] "+v"(acc[1][1]), [c12] "+v"(acc[1][2]), [c13] "+v"(acc[1][3]),
              [c20] "+v"(acc[2][0]), [c21] "+v"(acc[2][1]), [c22] "+v"(acc[2][2]), [c23] "+v"(acc[2][3]),
              [c30] "+v"(acc[3][0]), [c31] "+v"(acc[3][1]), [c32] "+v"(acc[3][2]), [c33] "+v"(acc[3][3]),
              [t0] "=&v"(t0), [t1] "=&v"(t1), [t2] "=&v"(t2), [t3] "=&v"(t3), [all] "=&s"(all), [pl] "+v"(pl), [pr] "+v"(pr)
            : [a0] "v"(a.x), [a1] "v"(a.y), [a2] "v"(a.z), [a3] "v"(a.w), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w)
            : "vcc");
#undef PAM_SKIP_ROW
    } else {
#define PAM_SKIP_COL(J)                                                                         \
    "v_cmpx_ne_u32_e32 vcc, %[zero], %[b" #J "]\n"                                               \
    "v_add_u32 %[t0], %[a0], %[b" #J "]\n v_add_u32 %[t1], %[a1], %[b" #J "]\n"                  \
    "v_add_u32 %[t2], %[a2], %[b" #J "]\n v_add_u32 %[t3], %[a3], %[b" #J "]\n"                  \
    "v_add_f32 %[c0" #J "], %[c0" #J "], %[t0]\n v_add_f32 %[c1" #J "], %[c1" #J "], %[t1]\n"    \
    "v_add_f32 %[c2" #J "], %[c2" #J "], %[t2]\n v_add_f32 %[c3" #J "], %[c3" #J "], %[t3]\n"    \
    "s_mov_b64 exec, %[all]\n"
        asm volatile(
            "s_mov_b64 %[all], exec\n" PAM_SKIP_COL(0) PAM_SKIP_COL(1) PAM_SKIP_COL(2) PAM_SKIP_COL(3)
            : [c00] "+v"(acc[0][0]), [c01] "+v"(acc[0][1]), [c02] "+v"(acc[0][2]), [c03] "+v"(acc[0][3]),
              [c10] "+v"(acc[1][0]), [c11] "+v"(acc[1][1]), [c12] "+v"(acc[1][2]), [c13] "+v"(acc[1][3]),
              [c20] "+v"(acc[2][0]), [c21] "+v"(acc[2][1]), [c22] "+v"(acc[2][2]), [c23] "+v"(acc[2][3]),
              [c30] "+v"(acc[3][0]), [c31] "+v"(acc[3][1]), [c32] "+v"(acc[3][2]), [c33] "+v"(acc[3][3]),
              [t0] "=&v"(t0), [t1] "=&v"(t1), [t2] "=&v"(t2), [t3] "=&v"(t3), [all] "=&s"(all), [pl] "+v"(pl), [pr] "+v"(pr)
            : [a0] "v"(a.x), [a1] "v"(a.y), [a2] "v"(a.z), [a3] "v"(a.w), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w),
              [zero] "s"(kZeroR)
            : "vcc");
#undef PAM_SKIP_COL
    }
}

// Zeros in both operands: a product runs in the lanes where neither value is the staged zero.  Eight compares give
// the masks of the four left and four right values, the integer sums of a row are formed in all lanes, and each
// float add runs under the AND of its two masks (formed on the scalar unit).
#define PAM_BOTH_ROW(I, LIVE)                                                                   \
    "s_mov_b64 exec, %[" LIVE "]\n"                                                             \
    "v_add_u32 %[t0], %[a" #I "], %[b0]\n v_add_u32 %[t1], %[a" #I "], %[b1]\n"                  \
    "v_add_u32 %[t2], %[a" #I "], %[b2]\n v_add_u32 %[t3], %[a" #I "], %[b3]\n"                  \
    "s_and_b64 exec, %[ma" #I "], %[mb0]\n v_add_f32 %[c" #I "0], %[c" #I "0], %[t0]\n"          \
    "s_and_b64 exec, %[ma" #I "], %[mb1]\n v_add_f32 %[c" #I "1], %[c" #I "1], %[t1]\n"          \
    "s_and_b64 exec, %[ma" #I "], %[mb2]\n v_add_f32 %[c" #I "2], %[c" #I "2], %[t2]\n"          \
    "s_and_b64 exec, %[ma" #I "], %[mb3]\n v_add_f32 %[c" #I "3], %[c" #I "3], %[t3]\n"
#define PAM_BOTH_MASKS                                                                          \
    "v_cmp_ne_u32_e64 %[ma0], 0, %[a0]\n v_cmp_ne_u32_e64 %[ma1], 0, %[a1]\n"                    \
    "v_cmp_ne_u32_e64 %[ma2], 0, %[a2]\n v_cmp_ne_u32_e64 %[ma3], 0, %[a3]\n"                    \
    "v_cmp_ne_u32_e64 %[mb0], %[zero], %[b0]\n v_cmp_ne_u32_e64 %[mb1], %[zero], %[b1]\n"        \
    "v_cmp_ne_u32_e64 %[mb2], %[zero], %[b2]\n v_cmp_ne_u32_e64 %[mb3], %[zero], %[b3]\n"
#define PAM_BOTH_MASK_OPERANDS                                                                  \
    [ma0] "=&s"(ma0), [ma1] "=&s"(ma1), [ma2] "=&s"(ma2), [ma3] "=&s"(ma3),                      \
    [mb0] "=&s"(mb0), [mb1] "=&s"(mb1), [mb2] "=&s"(mb2), [mb3] "=&s"(mb3)
__device__ __forceinline__ void pam_mac_4x4_skip_both(float (&acc)[4][4], const u32x4& a, const u32x4& b, uint32_t& pl, uint32_t& pr)
{
    uint32_t t0, t1, t2, t3;
    uint64_t all, ma0, ma1, ma2, ma3, mb0, mb1, mb2, mb3;
    asm volatile(
        "s_mov_b64 %[all], exec\n" PAM_BOTH_MASKS
        PAM_BOTH_ROW(0, "all") PAM_BOTH_ROW(1, "all") PAM_BOTH_ROW(2, "all") PAM_BOTH_ROW(3, "all")
        "s_mov_b64 exec, %[all]\n"
        : PAM_ACC_OPERANDS, [t0] "=&v"(t0), [t1] "=&v"(t1), [t2] "=&v"(t2), [t3] "=&v"(t3), [all] "=&s"(all),
          PAM_BOTH_MASK_OPERANDS, [pl] "+v"(pl), [pr] "+v"(pr)
        : PAM_FRAGMENT_OPERANDS, [zero] "s"(kZeroR)
        : "scc");
}

// ... and under a wavefront-uniform lane mask `run`, as pam_mac_4x4_under
__device__ __forceinline__ void pam_mac_4x4_skip_both_under(float (&acc)[4][4], const u32x4& a, const u32x4& b, uint32_t& pl, uint32_t& pr,
                                                            uint64_t run)
{
    uint32_t t0, t1, t2, t3;
    uint64_t all, live, ma0, ma1, ma2, ma3, mb0, mb1, mb2, mb3;
    asm volatile(
        "s_mov_b64 %[all], exec\n s_and_b64 %[live], exec, %[run]\n" PAM_BOTH_MASKS
        "s_and_b64 %[ma0], %[ma0], %[run]\n s_and_b64 %[ma1], %[ma1], %[run]\n"
        "s_and_b64 %[ma2], %[ma2], %[run]\n s_and_b64 %[ma3], %[ma3], %[run]\n"
        PAM_BOTH_ROW(0, "live") PAM_BOTH_ROW(1, "live") PAM_BOTH_ROW(2, "live") PAM_BOTH_ROW(3, "live")
        "s_mov_b64 exec, %[all]\n"
        : PAM_ACC_OPERANDS, [t0] "=&v"(t0), [t1] "=&v"(t1), [t2] "=&v"(t2), [t3] "=&v"(t3), [all] "=&s"(all), [live] "=&s"(live),
          PAM_BOTH_MASK_OPERANDS, [pl] "+v"(pl), [pr] "+v"(pr)
        : PAM_FRAGMENT_OPERANDS, [zero] "s"(kZeroR), [run] "s"(run)
        : "scc");
}
#undef PAM_BOTH_ROW
#undef PAM_BOTH_MASKS
#undef PAM_BOTH_MASK_OPERANDS

// The exact-backward products of a 4 x 4 micro-tile for one k (pam/cuda_kernels.cu:48-57): per product the slope
// operand's bits plus the kept fraction, masked to sign and exponent, times the upstream gradient, added by one
// fma.  DELTA_LEFT: the gradient is the left fragment (a) and the slope operand the right one (b); else the reverse.
// Two statements of eight products; the LDS addresses pass through as in pam_mac_4x4.
#define PAM_BWD_DL_LOW "v_add_u32 %[t0], %[b0], %[d00]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[b1], %[d01]\nv_fma_f32 %[c00], %[a0], %[t0], %[c00]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[b2], %[d02]\nv_fma_f32 %[c01], %[a0], %[t1], %[c01]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[b3], %[d03]\nv_fma_f32 %[c02], %[a0], %[t0], %[c02]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[b0], %[d10]\nv_fma_f32 %[c03], %[a0], %[t1], %[c03]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[b1], %[d11]\nv_fma_f32 %[c10], %[a1], %[t0], %[c10]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[b2], %[d12]\nv_fma_f32 %[c11], %[a1], %[t1], %[c11]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[b3], %[d13]\nv_fma_f32 %[c12], %[a1], %[t0], %[c12]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_fma_f32 %[c13], %[a1], %[t1], %[c13]\n"
#define PAM_BWD_DL_HIGH "v_add_u32 %[t0], %[b0], %[d20]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[b1], %[d21]\nv_fma_f32 %[c20], %[a2], %[t0], %[c20]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[b2], %[d22]\nv_fma_f32 %[c21], %[a2], %[t1], %[c21]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[b3], %[d23]\nv_fma_f32 %[c22], %[a2], %[t0], %[c22]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[b0], %[d30]\nv_fma_f32 %[c23], %[a2], %[t1], %[c23]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[b1], %[d31]\nv_fma_f32 %[c30], %[a3], %[t0], %[c30]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[b2], %[d32]\nv_fma_f32 %[c31], %[a3], %[t1], %[c31]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[b3], %[d33]\nv_fma_f32 %[c32], %[a3], %[t0], %[c32]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_fma_f32 %[c33], %[a3], %[t1], %[c33]\n"
#define PAM_BWD_DR_LOW "v_add_u32 %[t0], %[a0], %[d00]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[a0], %[d01]\nv_fma_f32 %[c00], %[b0], %[t0], %[c00]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[a0], %[d02]\nv_fma_f32 %[c01], %[b1], %[t1], %[c01]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[a0], %[d03]\nv_fma_f32 %[c02], %[b2], %[t0], %[c02]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[a1], %[d10]\nv_fma_f32 %[c03], %[b3], %[t1], %[c03]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[a1], %[d11]\nv_fma_f32 %[c10], %[b0], %[t0], %[c10]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[a1], %[d12]\nv_fma_f32 %[c11], %[b1], %[t1], %[c11]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[a1], %[d13]\nv_fma_f32 %[c12], %[b2], %[t0], %[c12]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_fma_f32 %[c13], %[b3], %[t1], %[c13]\n"
#define PAM_BWD_DR_HIGH "v_add_u32 %[t0], %[a2], %[d20]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[a2], %[d21]\nv_fma_f32 %[c20], %[b0], %[t0], %[c20]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[a2], %[d22]\nv_fma_f32 %[c21], %[b1], %[t1], %[c21]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[a2], %[d23]\nv_fma_f32 %[c22], %[b2], %[t0], %[c22]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[a3], %[d30]\nv_fma_f32 %[c23], %[b3], %[t1], %[c23]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[a3], %[d31]\nv_fma_f32 %[c30], %[b0], %[t0], %[c30]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_add_u32 %[t0], %[a3], %[d32]\nv_fma_f32 %[c31], %[b1], %[t1], %[c31]\nv_and_b32 %[t0], 0xff800000, %[t0]\nv_add_u32 %[t1], %[a3], %[d33]\nv_fma_f32 %[c32], %[b2], %[t0], %[c32]\nv_and_b32 %[t1], 0xff800000, %[t1]\nv_fma_f32 %[c33], %[b3], %[t1], %[c33]\n"
// UNDER: the statements run under the wavefront-uniform lane mask `run` (all ones or zero), as pam_mac_4x4_under.
template <bool DELTA_LEFT, bool UNDER = false>
__device__ __forceinline__ void pam_bwd_mac_4x4(float (&acc)[4][4], const uint32_t (&dfrac)[4][4], const u32x4& a, const u32x4& b,
                                                uint32_t& pl, uint32_t& pr, uint64_t run = 0)
{
    uint32_t t0, t1;
    uint64_t all;
    if (DELTA_LEFT) {
        if constexpr (UNDER) {
            asm volatile("s_mov_b64 %[all], exec\n s_and_b64 exec, exec, %[run]\n" PAM_BWD_DL_LOW "s_mov_b64 exec, %[all]\n"
                         : [c00] "+v"(acc[0][0]), [c01] "+v"(acc[0][1]), [c02] "+v"(acc[0][2]), [c03] "+v"(acc[0][3]), [c10] "+v"(acc[1][0]), [c11] "+v"(acc[1][1]), [c12] "+v"(acc[1][2]), [c13] "+v"(acc[1][3]), [t0] "=&v"(t0), [t1] "=&v"(t1), [p] "+v"(pl), [all] "=&s"(all)
                         : [d00] "v"(dfrac[0][0]), [d01] "v"(dfrac[0][1]), [d02] "v"(dfrac[0][2]), [d03] "v"(dfrac[0][3]), [d10] "v"(dfrac[1][0]), [d11] "v"(dfrac[1][1]), [d12] "v"(dfrac[1][2]), [d13] "v"(dfrac[1][3]), [a0] "v"(a.x), [a1] "v"(a.y), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w), [run] "s"(run)
                         : "scc");
            asm volatile("s_mov_b64 %[all], exec\n s_and_b64 exec, exec, %[run]\n" PAM_BWD_DL_HIGH "s_mov_b64 exec, %[all]\n"
                         : [c20] "+v"(acc[2][0]), [c21] "+v"(acc[2][1]), [c22] "+v"(acc[2][2]), [c23] "+v"(acc[2][3]), [c30] "+v"(acc[3][0]), [c31] "+v"(acc[3][1]), [c32] "+v"(acc[3][2]), [c33] "+v"(acc[3][3]), [t0] "=&v"(t0), [t1] "=&v"(t1), [p] "+v"(pr), [all] "=&s"(all)
                         : [d20] "v"(dfrac[2][0]), [d21] "v"(dfrac[2][1]), [d22] "v"(dfrac[2][2]), [d23] "v"(dfrac[2][3]), [d30] "v"(dfrac[3][0]), [d31] "v"(dfrac[3][1]), [d32] "v"(dfrac[3][2]), [d33] "v"(dfrac[3][3]), [a2] "v"(a.z), [a3] "v"(a.w), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w), [run] "s"(run)
                         : "scc");
        } else {
            asm volatile(PAM_BWD_DL_LOW
                         : [c00] "+v"(acc[0][0]), [c01] "+v"(acc[0][1]), [c02] "+v"(acc[0][2]), [c03] "+v"(acc[0][3]), [c10] "+v"(acc[1][0]), [c11] "+v"(acc[1][1]), [c12] "+v"(acc[1][2]), [c13] "+v"(acc[1][3]), [t0] "=&v"(t0), [t1] "=&v"(t1), [p] "+v"(pl)
                         : [d00] "v"(dfrac[0][0]), [d01] "v"(dfrac[0][1]), [d02] "v"(dfrac[0][2]), [d03] "v"(dfrac[0][3]), [d10] "v"(dfrac[1][0]), [d11] "v"(dfrac[1][1]), [d12] "v"(dfrac[1][2]), [d13] "v"(dfrac[1][3]), [a0] "v"(a.x), [a1] "v"(a.y), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w));
            asm volatile(PAM_BWD_DL_HIGH
                         : [c20] "+v"(acc[2][0]), [c21] "+v"(acc[2][1]), [c22] "+v"(acc[2][2]), [c23] "+v"(acc[2][3]), [c30] "+v"(acc[3][0]), [c31] "+v"(acc[3][1]), [c32] "+v"(acc[3][2]), [c33] "+v"(acc[3][3]), [t0] "=&v"(t0), [t1] "=&v"(t1), [p] "+v"(pr)
                         : [d20] "v"(dfrac[2][0]), [d21] "v"(dfrac[2][1]), [d22] "v"(dfrac[2][2]), [d23] "v"(dfrac[2][3]), [d30] "v"(dfrac[3][0]), [d31] "v"(dfrac[3][1]), [d32] "v"(dfrac[3][2]), [d33] "v"(dfrac[3][3]), [a2] "v"(a.z), [a3] "v"(a.w), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w));
        }
    } else {
        if constexpr (UNDER) {
            asm volatile("s_mov_b64 %[all], exec\n s_and_b64 exec, exec, %[run]\n" PAM_BWD_DR_LOW "s_mov_b64 exec, %[all]\n"
                         : [c00] "+v"(acc[0][0]), [c01] "+v"(acc[0][1]), [c02] "+v"(acc[0][2]), [c03] "+v"(acc[0][3]), [c10] "+v"(acc[1][0]), [c11] "+v"(acc[1][1]), [c12] "+v"(acc[1][2]), [c13] "+v"(acc[1][3]), [t0] "=&v"(t0), [t1] "=&v"(t1), [p] "+v"(pl), [all] "=&s"(all)
                         : [d00] "v"(dfrac[0][0]), [d01] "v"(dfrac[0][1]), [d02] "v"(dfrac[0][2]), [d03] "v"(dfrac[0][3]), [d10] "v"(dfrac[1][0]), [d11] "v"(dfrac[1][1]), [d12] "v"(dfrac[1][2]), [d13] "v"(dfrac[1][3]), [a0] "v"(a.x), [a1] "v"(a.y), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w), [run] "s"(run)
                         : "scc");
            asm volatile("s_mov_b64 %[all], exec\n s_and_b64 exec, exec, %[run]\n" PAM_BWD_DR_HIGH "s_mov_b64 exec, %[all]\n"
                         : [c20] "+v"(acc[2][0]), [c21] "+v"(acc[2][1]), [c22] "+v"(acc[2][2]), [c23] "+v"(acc[2][3]), [c30] "+v"(acc[3][0]), [c31] "+v"(acc[3][1]), [c32] "+v"(acc[3][2]), [c33] "+v"(acc[3][3]), [t0] "=&v"(t0), [t1] "=&v"(t1), [p] "+v"(pr), [all] "=&s"(all)
                         : [d20] "v"(dfrac[2][0]), [d21] "v"(dfrac[2][1]), [d22] "v"(dfrac[2][2]), [d23] "v"(dfrac[2][3]), [d30] "v"(dfrac[3][0]), [d31] "v"(dfrac[3][1]), [d32] "v"(dfrac[3][2]), [d33] "v"(dfrac[3][3]), [a2] "v"(a.z), [a3] "v"(a.w), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w), [run] "s"(run)
                         : "scc");
        } else {
            asm volatile(PAM_BWD_DR_LOW
                         : [c00] "+v"(acc[0][0]), [c01] "+v"(acc[0][1]), [c02] "+v"(acc[0][2]), [c03] "+v"(acc[0][3]), [c10] "+v"(acc[1][0]), [c11] "+v"(acc[1][1]), [c12] "+v"(acc[1][2]), [c13] "+v"(acc[1][3]), [t0] "=&v"(t0), [t1] "=&v"(t1), [p] "+v"(pl)
                         : [d00] "v"(dfrac[0][0]), [d01] "v"(dfrac[0][1]), [d02] "v"(dfrac[0][2]), [d03] "v"(dfrac[0][3]), [d10] "v"(dfrac[1][0]), [d11] "v"(dfrac[1][1]), [d12] "v"(dfrac[1][2]), [d13] "v"(dfrac[1][3]), [a0] "v"(a.x), [a1] "v"(a.y), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w));
            asm volatile(PAM_BWD_DR_HIGH
                         : [c20] "+v"(acc[2][0]), [c21] "+v"(acc[2][1]), [c22] "+v"(acc[2][2]), [c23] "+v"(acc[2][3]), [c30] "+v"(acc[3][0]), [c31] "+v"(acc[3][1]), [c32] "+v"(acc[3][2]), [c33] "+v"(acc[3][3]), [t0] "=&v"(t0), [t1] "=&v"(t1), [p] "+v"(pr)
                         : [d20] "v"(dfrac[2][0]), [d21] "v"(dfrac[2][1]), [d22] "v"(dfrac[2][2]), [d23] "v"(dfrac[2][3]), [d30] "v"(dfrac[3][0]), [d31] "v"(dfrac[3][1]), [d32] "v"(dfrac[3][2]), [d33] "v"(dfrac[3][3]), [a2] "v"(a.z), [a3] "v"(a.w), [b0] "v"(b.x), [b1] "v"(b.y), [b2] "v"(b.z), [b3] "v"(b.w));
        }
    }
}
#undef PAM_BWD_DL_LOW
#undef PAM_BWD_DL_HIGH
#undef PAM_BWD_DR_LOW
#undef PAM_BWD_DR_HIGH

// Four work-groups per compute unit are what the LDS allows; the register budget follows (128 per lane), so that no
// instance of the kernel falls to three wavefronts per SIMD.
#define PAM_GEMM_OCCUPANCY __attribute__((amdgpu_waves_per_eu(4)))

// ---------------------------------------------------------------- the units of a launch
// The work of a product is a list of units: every 64 x 64 output tile, in the order (matrix, row tile, column
// tile), cut into `pieces` consecutive k ranges of `piece_kt` k-tiles each (the last one shorter; pieces == 1:
// whole tiles).  One work-group computes one unit; the hardware hands them to the compute units as these become
// free.  (A launch of only as many work-groups as are resident, each with a fixed share of the units, measured
// slower: the wavefront scheduler favours the oldest work-group of a compute unit, so equal shares finish at very
// different times -- 43 to 81 us for the four work-groups of one compute unit -- and the last ones run alone at
// half the issue rate.  Drawing the units from queues in memory instead cost 15-25 us per work-group in atomic
// operations on the queue words.)
//
// A cut tile: each piece is summed from +0 on its own and written to its slot of the workspace; the work-group
// that arrives last at the tile's arrival word adds the pieces in ascending k order from +0 and writes the tile
// (few pieces), or a second kernel does that for all tiles (many pieces).  Nothing ever waits for another
// work-group.  The arrival word is a 64-bit (tag << 24 | arrivals so far), advanced by an atomic add.  The tag is
// the launch's number (a process-wide counter that starts at a random value): a word that carries another tag --
// whatever an earlier product of another shape, or the allocator, left there -- counts as zero arrivals, so a
// workspace needs no preparation; the work-group that completes a tile leaves its word at the next launch's tag
// with zero arrivals, so products that follow each other on one workspace find their words ready.
//
// Pieces and words pass between compute units (and XCDs, each with its own L2) without fences: the pieces are
// written and read with agent-scope accesses, which go past the non-coherent caches, a work-group waits for its
// stores to complete before it arrives, and the words are only touched by agent-scope atomics.  A release /
// acquire fence pair at agent scope would do the same for ordinary stores, but it writes back and invalidates the
// whole L2 of the XCD per work-group (measured: a 85 us product took 350 us).
constexpr int kTagShift = 24;                                       // a word: 40 bits of tag, 24 bits of arrivals
constexpr unsigned long long kTagMask = (1ull << 40) - 1;

// An arrival at a word that carries another tag (`seen`: what it held after this work-group's add): whoever exchanges
// it for one with this launch's tag first is arrival 0, the others (whose adds went to the old contents and are lost
// with them) arrive again.  Each round ends with some work-group's progress, and there are no more rounds than pieces.
__device__ __forceinline__ uint32_t arrive_untagged(unsigned long long* word, unsigned long long tag, unsigned long long seen)
{
    for (;;) {
        if ((seen >> kTagShift) == tag) {
            seen = __hip_atomic_fetch_add(word, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((seen >> kTagShift) == tag) return (uint32_t)(seen & ((1u << kTagShift) - 1));
            seen += 1ull;
        } else if (__hip_atomic_compare_exchange_strong(word, &seen, (tag << kTagShift) | 1ull, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
            return 0u;
        }                                         // (a failed exchange has put the word's present contents into `seen`)
    }
}

// Arrives at a tile's word: returns how many arrived before.
__device__ __forceinline__ uint32_t arrive_at(unsigned long long* word, unsigned long long tag)
{
    const unsigned long long seen = __hip_atomic_fetch_add(word, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __builtin_expect((seen >> kTagShift) == tag, 1) ? (uint32_t)(seen & ((1u << kTagShift) - 1)) : arrive_untagged(word, tag, seen + 1ull);
}

constexpr int kPartFloats = 64 * 64;            // one piece of a tile: sixteen sums per lane of the work-group
constexpr int kFoldInKernel = 8;                // tiles of up to this many pieces are added up by their last arriver

// Where a lane's 4 x 4 outputs sit in its work-group's 64 x 64 tile: rows ty * 4 ..., columns tx * 4 ....  A wavefront
// covers 16 rows x 64 columns -- or, in a tile that the matrix fills less in its columns than in its rows, 64 rows x
// 16 columns: a wavefront none of whose outputs exist (the last tiles of 197 rows or columns leave three of the four
// without one) stages and synchronises with the others but computes nothing.
struct LanePlace { int tx, ty; bool idle; };
__device__ __forceinline__ LanePlace lane_place(int tid, int row0, int col0, int M, int N)
{
    const int wave = tid / 64, lane = tid % 64;
    if (N - col0 < 64 && N - col0 < M - row0) return LanePlace{4 * wave + lane % 4, lane / 4, col0 + 16 * wave >= N};
    return LanePlace{tid % 16, tid / 16, row0 + 16 * wave >= M};
}

typedef float v4f __attribute__((ext_vector_type(4)));
// A piece of a cut tile in the workspace: the work-group's lanes' sixteen sums each as four 128-bit rows, row i of
// lane `tid` at [unit][i][tid] -- every access of the work-group is one contiguous 4 KB run.
__device__ __forceinline__ v4f* piece_row(float* partial, long unit, int i, int tid)
{
    return reinterpret_cast<v4f*>(partial) + ((unit * 4 + i) * 256 + tid);
}
// The same where the pieces are exchanged inside the launch, which takes agent-scope accesses of at most 64 bits: half
// rows, half h of row i of lane `tid` at [unit][i][h][tid], so that every access of a wavefront is one contiguous
// 512-byte run (as halves of the 128-bit rows above, each store filled half of every 32-byte sector it touched, and
// the write-through stores counted twice their bytes in memory traffic).
typedef unsigned long long Pair;
__device__ __forceinline__ Pair* piece_half(float* partial, long unit, int i, int h, int tid)
{
    return reinterpret_cast<Pair*>(partial) + ((unit * 8 + i * 2 + h) * 256 + tid);
}

// acc = the pieces [first, first + count) of a tile added in ascending order from +0, read at agent scope (their
// writers belong to the same launch).  Two pieces' loads are in flight at a time: more would take registers from the
// kernel this is called from.
__device__ __forceinline__ void fold_pieces(float* partial, long first, int count, int tid, float (&acc)[4][4])
{
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
#pragma unroll 1
    for (int p = 0; p < count; p += 2) {
        const int second = min(p + 1, count - 1);           // (an odd count: the last piece is loaded twice, added once)
        Pair v[2][4][2];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                v[0][i][h] = __hip_atomic_load(piece_half(partial, first + p, i, h, tid), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                v[1][i][h] = __hip_atomic_load(piece_half(partial, first + second, i, h, tid), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            if (c == 1 && p + 1 >= count) break;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    acc[i][2 * h] = acc[i][2 * h] + u2f((uint32_t)v[c][i][h]);
                    acc[i][2 * h + 1] = acc[i][2 * h + 1] + u2f((uint32_t)(v[c][i][h] >> 32));
                }
        }
    }
}

// What only the sums' way out needs of the arguments (where the output and the pieces are, the bias, the arrival words)
// is read there from the kernel's argument segment, through a pointer the compiler cannot see through: held in scalar
// registers from the kernel's start, as it otherwise arranges, they are eighteen registers too many during the loops,
// which then spill scalar values into vector lanes (the k-tiles with zeros, which live on execution masks, ran 14 %
// slower for it, and the image-patch instance spilled vector registers on top).
typedef const __attribute__((address_space(4))) GemmArgs* LateArgs;
__device__ __forceinline__ LateArgs late_args()
{
    LateArgs p = (LateArgs)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(p));
    return p;
}

// CUT: the launch cuts its tiles' k ranges into pieces (an instance of its own, so that the kernel for whole tiles
// carries none of the pieces' way out).
template <int BM, int BN, int TM, int TN, int BK, int MODE, int LKIND, int RKIND, bool CUT>
__global__ __launch_bounds__((BM / TM) * (BN / TN)) PAM_GEMM_OCCUPANCY void gemm_kernel(GemmArgs g)
{
    constexpr int TXN = BN / TN, TYN = BM / TM, NT = TXN * TYN, NW = NT / 64;
    constexpr int GM = TM / 4, GN = TN / 4;               // 4-wide groups per micro-tile side
    constexpr int LDL = BM + PAD, LDR = BN + PAD;
    static_assert(TM == 4 && TN == 4 && BM == 64 && BN == 64 && NT == 256, "a tile's piece is sixteen sums per lane of 256");

    __shared__ __attribute__((aligned(16))) uint32_t lds_l[2][BK * LDL];
    __shared__ __attribute__((aligned(16))) uint32_t lds_r[2][BK * LDR];
    __shared__ uint32_t lds_flag[2][NW];
    __shared__ uint32_t lds_odd_k[2][NW];         // bit k: some value under k of the tile needs the full definition
    __shared__ uint32_t lds_arrived;

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    // This work-group's unit.  Work-groups go to the eight XCDs in turn and every XCD has its own L2, so with units in
    // launch order the column tiles of one row tile land on all eight and each L2 fetches the whole left operand.
    // Work-group x therefore takes unit (x mod 8) * ceil(units / 8) + x div 8: one contiguous range of units per XCD.
    int unit = blockIdx.x;
    if (g.xcd_chunk > 0) {
        unit = (int)(blockIdx.x % XCDS) * g.xcd_chunk + (int)(blockIdx.x / XCDS);
        if (unit >= g.units) return;              // the ranges are rounded up: a few work-groups have nothing to do
    }
    // The unit's tile (of all matrices) and k range.  Tiles cut into few pieces: a tile's pieces are consecutive units, so
    // they finish at about the same time and the tile is added up early.  Many pieces (few tiles, the weight-gradient
    // shape): the tiles of one k range are consecutive units -- they run together and share its rows of both operands.
    int flat = unit, piece = 0;
    if (CUT) {
        if (g.fold_here) { flat = unit / g.pieces; piece = unit - flat * g.pieces; }
        else { const int all = g.units / g.pieces; piece = unit / all; flat = unit - piece * all; }
    }
    const int zb = flat / g.tiles, tile = flat - zb * g.tiles;
    const int row0 = (tile / g.ntn) * BM, col0 = (tile % g.ntn) * BN;       // consecutive tiles share L rows
    const int kbegin = CUT ? piece * g.piece_kt * BK : 0;
    const int kend = CUT ? min(g.K, kbegin + g.piece_kt * BK) : g.K;
    const int ktiles = (kend - kbegin + BK - 1) / BK;
    // The lane's 4 x 4 outputs within the tile, rows ty * 4 ..., columns tx * 4 ....
    const LanePlace place = lane_place(tid, row0, col0, g.M, g.N);
    const int tx = place.tx, ty = place.ty;
    const bool has_off = g.has_off != 0;

    const float* lbase = g.L.p + (long)zb * g.L.sb;
    const float* rbase = g.R.p + (long)zb * g.R.sb;

    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = 0.0f;

    // forward operand whose gradient is wanted (backward modes): only its fraction matters
    uint32_t dfrac[(MODE >= MODE_BWD_DL) ? TM : 1][(MODE >= MODE_BWD_DL) ? TN : 1];
    if (MODE >= MODE_BWD_DL) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                int r = row0 + (i / 4) * (BM / GM) + ty * 4 + (i % 4);
                int c = col0 + (j / 4) * (BN / GN) + tx * 4 + (j % 4);
                float d = (r < g.M && c < g.N) ? g.D[(long)zb * g.d_sb + (long)r * g.d_sr + (long)c * g.d_sc] : 0.0f;
                dfrac[i][j] = normalised_fraction(d);
            }
    }

    TileLoader<BM, NT, LKIND, BK> ll;
    TileLoader<BN, NT, RKIND, BK> rl;

    auto stage = [&](int buf) __attribute__((always_inline)) {
        PlainStager<false> same{0u};
        if (MODE == MODE_STD) {
            ll.store(lds_l[buf], tid, same);
            rl.store(lds_r[buf], tid, same);
            return;
        }
        // Quick test first: nearly every k-tile holds only normal numbers of moderate size, and then staging is
        // the shift-add and max per value below plus an integer add for the operand that carries the bias.
        constexpr bool kOffL = Stager<MODE, false>::kTakesOffset, kOffR = Stager<MODE, true>::kTakesOffset;
        const bool shifted = g.has_off == 1;
        // (per operand: the zeros of a ReLU or of an image's padding sit in one of them, and the other one's values then
        // need no look each)
        const bool quick_l = __ballot(ll.window_max(kOffL && shifted, g.off_add) >= kWindowSpan) == 0ull && !(kOffL && g.has_off == 2);
        const bool quick_r = __ballot(rl.window_max(kOffR && shifted, g.off_add) >= kWindowSpan) == 0ull && !(kOffR && g.has_off == 2);
        PlainStager<true> plus{(MODE == MODE_PAM ? 0u - kBias : 0u) + (shifted ? g.off_add : 0u)};
        if (quick_l) { if (kOffL && (MODE == MODE_PAM || shifted)) ll.store(lds_l[buf], tid, plus); else ll.store(lds_l[buf], tid, same); }
        if (quick_r) { if (kOffR && (MODE == MODE_PAM || shifted)) rl.store(lds_r[buf], tid, plus); else rl.store(lds_r[buf], tid, same); }
        if (__builtin_expect(quick_l && quick_r, 1)) {
            if (lane == 0) lds_flag[buf][wave] = 0u;      // (its k mask keeps an older value: readers go by the flag)
            return;
        }
        Stager<MODE, false> sl; Stager<MODE, true> sr;
        if (!quick_l) {
            if (has_off && Stager<MODE, false>::kTakesOffset) ll.apply_offset(g.off);
            ll.store(lds_l[buf], tid, sl);
        }
        if (!quick_r) {
            if (has_off && Stager<MODE, true>::kTakesOffset) rl.apply_offset(g.off);
            rl.store(lds_r[buf], tid, sr);
        }
        const uint32_t found = (__ballot(sl.out_of_range() || sr.out_of_range()) != 0ull ? kGuarded : 0u)
                             | (__ballot(sl.zero) != 0ull ? kZerosL : 0u) | (__ballot(sr.zero) != 0ull ? kZerosR : 0u);
        if (lane == 0) lds_flag[buf][wave] = found;
        // A wavefront that found such a value (rare) walks its register tile once more and records under which k
        // they sit: the loop for this tile chooses per k-step.  The other wavefronts have none to report.
        uint32_t odd = 0u;
        if (__builtin_expect(found >= kGuarded, 0)) {
            ll.odd_by_k(tid, odd);
            rl.odd_by_k(tid, odd);
#pragma unroll
            for (int s = 32; s >= 1; s >>= 1) odd |= __shfl_xor(odd, s, 64);
        }
        if (lane == 0) lds_odd_k[buf][wave] = odd;
    };

    if (ktiles > 0) {
        ll.load(g.L, lbase, row0, g.M, kbegin, kend, tid, g.cv);
        rl.load(g.R, rbase, col0, g.N, kbegin, kend, tid, g.cv);
        stage(0);
    }
    __syncthreads();

    // per k-tile: where its fragments are in LDS, how many k it holds, and what the staging found in it
    const uint32_t* sl = nullptr; const uint32_t* sr = nullptr;           // the lane's rows of k-steps 0 ... 15
    const uint32_t* slx = nullptr; const uint32_t* srx = nullptr;         // and of k-steps 16 ... 31 (see swizzled)
    int kcount = 0;
    const bool idle_wave = MODE != MODE_STD && __builtin_amdgcn_readfirstlane(place.idle ? 1 : 0) != 0;
    uint32_t verdict = 0;                         // 0 plain loop, kZerosL / kZerosR bits, >= kGuarded guarded
    auto begin_tile = [&](int t) __attribute__((always_inline)) {
        const int cur = t & 1;
        const int k0 = kbegin + t * BK;
        // The next tile is fetched unconditionally: past the end the clamped addresses re-read the last
        // tile and the values are dropped.  A conditional fetch would merge with the registers' old
        // contents and make the compiler wait for the data right here.
        ll.load(g.L, lbase, row0, g.M, k0 + BK, kend, tid, g.cv);
        rl.load(g.R, rbase, col0, g.N, k0 + BK, kend, tid, g.cv);
        kcount = min(BK, kend - k0);
        if (MODE != MODE_STD) {
            uint32_t f = 0;
#pragma unroll
            for (int w = 0; w < NW; ++w) f |= lds_flag[cur][w];
            verdict = idle_wave ? kIdle : __builtin_amdgcn_readfirstlane(f);
        }
        sl = lds_l[cur] + ty * 4; slx = lds_l[cur] + swizzled<BK>(ty * 4, 16);
        sr = lds_r[cur] + tx * 4; srx = lds_r[cur] + swizzled<BK>(tx * 4, 16);
    };
    auto end_tile = [&](int t) __attribute__((always_inline)) {
        if (t + 1 < ktiles) stage((t & 1) ^ 1);
        __syncthreads();
    };

    auto fragment = [&](int kk, uint32_t (&a)[TM], uint32_t (&b)[TN]) __attribute__((always_inline)) {
#pragma unroll
        for (int gi = 0; gi < GM; ++gi) {
            uint4 q = *reinterpret_cast<const uint4*>(((BK == 32 && (kk & 16)) ? slx : sl) + kk * LDL + gi * (BM / GM));
            a[gi * 4 + 0] = q.x; a[gi * 4 + 1] = q.y; a[gi * 4 + 2] = q.z; a[gi * 4 + 3] = q.w;
        }
#pragma unroll
        for (int gj = 0; gj < GN; ++gj) {
            uint4 q = *reinterpret_cast<const uint4*>(((BK == 32 && (kk & 16)) ? srx : sr) + kk * LDR + gj * (BN / GN));
            b[gj * 4 + 0] = q.x; b[gj * 4 + 1] = q.y; b[gj * 4 + 2] = q.z; b[gj * 4 + 3] = q.w;
        }
    };
    auto fast_step = [&](int kk) __attribute__((always_inline)) {
        uint32_t a[TM], b[TN];
        fragment(kk, a, b);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if (MODE == MODE_PAM) acc[i][j] += u2f(a[i] + b[j]);
                else if (MODE == MODE_STD) acc[i][j] = fmaf(u2f(a[i]), u2f(b[j]), acc[i][j]);
                else if (MODE == MODE_BWD_DL) acc[i][j] = fmaf(u2f(a[i]), u2f((b[j] + dfrac[i][j]) & ~kMant), acc[i][j]);
                else acc[i][j] = fmaf(u2f(b[j]), u2f((a[i] + dfrac[i][j]) & ~kMant), acc[i][j]);
            }
    };
    // k-tile with zeros but otherwise in range: the integer add of a zero is garbage, so those
    // products are replaced by +0 (one v_cndmask per product, masks combined on the scalar unit)
    auto zeros_step = [&](int kk) __attribute__((always_inline)) {
        uint32_t a[TM], b[TN];
        fragment(kk, a, b);
        bool za[TM], zb[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) za[i] = a[i] == kZeroL;
#pragma unroll
        for (int j = 0; j < TN; ++j) zb[j] = b[j] == kZeroR;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] += u2f((za[i] | zb[j]) ? 0u : a[i] + b[j]);
    };
    // zeros in one operand only: its zeros become a stand-in that keeps the integer sum finite, and
    // the product is multiplied by 0 or 1 in the accumulating fma (x * 1 + acc rounds like acc + x;
    // x * 0 + acc leaves acc, which is never -0) -- two instructions per product like the plain loop,
    // plus three per value of the operand with zeros
    auto zeros_left_step = [&](int kk) __attribute__((always_inline)) {
        uint32_t a[TM], b[TN];
        fragment(kk, a, b);
        float keep[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const uint64_t nonzero = __ballot(a[i] != kZeroL);
            keep[i] = u2f(pick(nonzero, 0u, 0x3f800000u));
            a[i] = max(a[i], kStandInL);          // every other value is larger, as an unsigned number
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_fmaf(u2f(a[i] + b[j]), keep[i], acc[i][j]);
    };
    auto zeros_right_step = [&](int kk) __attribute__((always_inline)) {
        uint32_t a[TM], b[TN];
        fragment(kk, a, b);
        float keep[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const uint64_t nonzero = __ballot(b[j] != kZeroR);
            keep[j] = u2f(pick(nonzero, 0u, 0x3f800000u));
            b[j] = pick(nonzero, kStandInR, b[j]);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_fmaf(u2f(a[i] + b[j]), keep[j], acc[i][j]);
    };
    // the products of one k-step by the full definition
    auto guarded_products = [&](const uint32_t (&a)[TM], const uint32_t (&b)[TN]) __attribute__((always_inline)) {
        if (MODE == MODE_PAM) {
            Split sa[TM], sb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) sa[i] = split_operand(a[i], 127);
#pragma unroll
            for (int j = 0; j < TN; ++j) sb[j] = split_operand(b[j] + kBias, 0);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] += pam_from_split(sa[i], sb[j]);
            return;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if (MODE == MODE_BWD_DL) acc[i][j] += bwd_product_general(dfrac[i][j], b[j], u2f(a[i]));
                else if (MODE == MODE_BWD_DR) acc[i][j] += bwd_product_general(dfrac[i][j], a[i], u2f(b[j]));
            }
    };
    auto guarded_step = [&](int kk) __attribute__((always_inline)) {
        uint32_t a[TM], b[TN];
        fragment(kk, a, b);
        guarded_products(a, b);
    };

    // a full k-tile of in-range values: fragments for step kk+1 are read from LDS while step kk is computed
    auto plain_tile = [&]() __attribute__((always_inline)) {
        if constexpr (MODE != MODE_STD && TM == 4 && TN == 4) {
            typedef const __attribute__((address_space(3))) uint32_t* LdsWord;
            uint32_t pl = (uint32_t)(uintptr_t)(LdsWord)sl, pr = (uint32_t)(uintptr_t)(LdsWord)sr;
            uint32_t plx = (uint32_t)(uintptr_t)(LdsWord)slx, prx = (uint32_t)(uintptr_t)(LdsWord)srx;
            u32x4 fa[2], fb[2];
            fa[0] = *reinterpret_cast<LdsVec>(pl); fb[0] = *reinterpret_cast<LdsVec>(pr);
#pragma unroll
            for (int kk = 0; kk < BK; ++kk) {
                if (kk + 1 < BK) {
                    fa[(kk + 1) & 1] = *reinterpret_cast<LdsVec>((kk + 1 < 16 ? pl : plx) + (kk + 1) * LDL * 4);
                    fb[(kk + 1) & 1] = *reinterpret_cast<LdsVec>((kk + 1 < 16 ? pr : prx) + (kk + 1) * LDR * 4);
                }
                asm volatile("" : "+v"(plx), "+v"(prx));         // (the blocks below hold the other two addresses the same way)
                if constexpr (MODE == MODE_PAM) pam_mac_4x4(acc, fa[kk & 1], fb[kk & 1], pl, pr);
                else pam_bwd_mac_4x4<MODE == MODE_BWD_DL>(acc, dfrac, fa[kk & 1], fb[kk & 1], pl, pr);
            }
        } else {
            // The other modes leave the instructions to the compiler but keep the k-steps apart: an empty asm
            // statement that the LDS addresses and the accumulators pass through, so that the reads of the step
            // after next cannot move above this step's products (all of them at the top cost 300 registers).
            static_assert(TM == 4 && TN == 4, "the step fence names sixteen accumulators");
            typedef const __attribute__((address_space(3))) uint32_t* LdsWord;
            uint32_t pl = (uint32_t)(uintptr_t)(LdsWord)sl, pr = (uint32_t)(uintptr_t)(LdsWord)sr;
            uint32_t plx = (uint32_t)(uintptr_t)(LdsWord)slx, prx = (uint32_t)(uintptr_t)(LdsWord)srx;
            u32x4 va[2], vb[2];
            va[0] = *reinterpret_cast<LdsVec>(pl); vb[0] = *reinterpret_cast<LdsVec>(pr);
#pragma unroll
            for (int kk = 0; kk < BK; ++kk) {
                if (kk + 1 < BK) {
                    va[(kk + 1) & 1] = *reinterpret_cast<LdsVec>((kk + 1 < 16 ? pl : plx) + (kk + 1) * LDL * 4);
                    vb[(kk + 1) & 1] = *reinterpret_cast<LdsVec>((kk + 1 < 16 ? pr : prx) + (kk + 1) * LDR * 4);
                }
                const uint32_t fa[4] = {va[kk & 1].x, va[kk & 1].y, va[kk & 1].z, va[kk & 1].w};
                const uint32_t fb[4] = {vb[kk & 1].x, vb[kk & 1].y, vb[kk & 1].z, vb[kk & 1].w};
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        if (MODE == MODE_PAM) acc[i][j] += u2f(fa[i] + fb[j]);
                        else if (MODE == MODE_STD) acc[i][j] = fmaf(u2f(fa[i]), u2f(fb[j]), acc[i][j]);
                        else if (MODE == MODE_BWD_DL) acc[i][j] = fmaf(u2f(fa[i]), u2f((fb[j] + dfrac[i][j]) & ~kMant), acc[i][j]);
                        else acc[i][j] = fmaf(u2f(fb[j]), u2f((fa[i] + dfrac[i][j]) & ~kMant), acc[i][j]);
                    }
                asm volatile("" : "+v"(pl), "+v"(pr), "+v"(plx), "+v"(prx),
                             "+v"(acc[0][0]), "+v"(acc[0][1]), "+v"(acc[0][2]), "+v"(acc[0][3]), "+v"(acc[1][0]), "+v"(acc[1][1]), "+v"(acc[1][2]), "+v"(acc[1][3]),
                             "+v"(acc[2][0]), "+v"(acc[2][1]), "+v"(acc[2][2]), "+v"(acc[2][3]), "+v"(acc[3][0]), "+v"(acc[3][1]), "+v"(acc[3][2]), "+v"(acc[3][3]));
            }
        }
    };

    // a full k-tile with zeros: the plain tile's schedule around the blocks that skip the zero products
    auto skip_tile = [&](auto which) __attribute__((always_inline)) {
        if constexpr (MODE == MODE_PAM && TM == 4 && TN == 4) {
            typedef const __attribute__((address_space(3))) uint32_t* LdsWord;
            uint32_t pl = (uint32_t)(uintptr_t)(LdsWord)sl, pr = (uint32_t)(uintptr_t)(LdsWord)sr;
            uint32_t plx = (uint32_t)(uintptr_t)(LdsWord)slx, prx = (uint32_t)(uintptr_t)(LdsWord)srx;
            u32x4 fa[2], fb[2];
            fa[0] = *reinterpret_cast<LdsVec>(pl); fb[0] = *reinterpret_cast<LdsVec>(pr);
#pragma unroll
            for (int kk = 0; kk < BK; ++kk) {
                if (kk + 1 < BK) {
                    fa[(kk + 1) & 1] = *reinterpret_cast<LdsVec>((kk + 1 < 16 ? pl : plx) + (kk + 1) * LDL * 4);
                    fb[(kk + 1) & 1] = *reinterpret_cast<LdsVec>((kk + 1 < 16 ? pr : prx) + (kk + 1) * LDR * 4);
                }
                asm volatile("" : "+v"(plx), "+v"(prx));         // (the blocks below hold the other two addresses the same way)
                constexpr uint32_t kWhich = decltype(which)::value;
                if constexpr (kWhich == (kZerosL | kZerosR)) pam_mac_4x4_skip_both(acc, fa[kk & 1], fb[kk & 1], pl, pr);
                else pam_mac_4x4_skip<kWhich == kZerosL>(acc, fa[kk & 1], fb[kk & 1], pl, pr);
            }
        }
    };
    constexpr bool kSkips = MODE == MODE_PAM && TM == 4 && TN == 4;

    // a full k-tile some of whose k-steps hold a value in need of the full definition (bit k of `odd`): a loop over
    // fours of k-steps in which every step passes through the plain block (the skipping one if the tile holds zeros
    // too, ZEROS) -- under an empty lane mask in the marked steps, whose products the full definition then adds.
    // The fragments of the step after are read while a step is computed, in two sets of registers that the steps
    // alternate (one step per round of the loop and no reading ahead spent 26 instructions around every block and
    // most of the tile's time waiting for LDS).
    auto mixed_tile = [&](uint32_t odd, auto holds_zeros) __attribute__((always_inline)) {
        if constexpr (MODE != MODE_STD && TM == 4 && TN == 4) {
            constexpr bool ZEROS = decltype(holds_zeros)::value;
            typedef const __attribute__((address_space(3))) uint32_t* LdsWord;
            uint32_t pl = (uint32_t)(uintptr_t)(LdsWord)sl, pr = (uint32_t)(uintptr_t)(LdsWord)sr;
            const uint32_t to_plx = (uint32_t)(uintptr_t)(LdsWord)slx - pl, to_prx = (uint32_t)(uintptr_t)(LdsWord)srx - pr;
            auto step = [&](int kk, u32x4& va, u32x4& vb) __attribute__((always_inline)) {
                // a marked step concerns the wavefronts whose lanes hold one of its odd values: 16 of a work-group's 256
                // lanes for a value of the left operand, 16 per wavefront for one of the right operand
                bool marked = ((odd >> kk) & 1u) != 0;
                uint32_t half = ~0u;                   // the step's lane mask, wavefront-uniform: all lanes, or none (kept in scalar registers)
                if (__builtin_expect(marked, 0)) {
                    constexpr uint32_t kUnstage = MODE == MODE_PAM ? kBias : 0u;      // the right operand is staged less the bias
                    const uint32_t ua[4] = {va.x, va.y, va.z, va.w}, ub[4] = {vb.x + kUnstage, vb.y + kUnstage, vb.z + kUnstage, vb.w + kUnstage};
                    bool oa[4], ob[4], mine = false;
                    // (a tile without zeros tells its odd values by the staging's window test, two instructions a value)
                    auto is_odd = [](uint32_t u) __attribute__((always_inline)) {
                        if constexpr (ZEROS || MODE != MODE_PAM) return needs_full_definition(u);
                        else return window(u) >= kWindowSpan;
                    };
#pragma unroll
                    for (int i = 0; i < 4; ++i) { oa[i] = is_odd(ua[i]); ob[i] = is_odd(ub[i]); mine |= oa[i] || ob[i]; }
                    marked = __ballot(mine) != 0ull;
                    if constexpr (MODE == MODE_PAM) {
                        // Tiny odd values (subnormal, or below 2^-63) mostly change nothing: |a (*) b| < 2^(Ea + Eb - 252)
                        // for biased exponent fields Ea, Eb (a subnormal number's is 0; a PAM product is no larger than the
                        // true one), and a sum whose field is at least Ea + Eb - 96 is left as it is by adding anything that
                        // small (below an eighth of its last place).  Such a value is replaced by 2^-63, the smallest the
                        // plain block takes: if every sum that one of its products goes to passes that test with 2^-63 in its
                        // place -- which covers the value itself, it is smaller -- the step runs the plain block on the
                        // replaced fragments and adds products that change nothing, as the true ones would.  Otherwise
                        // (small sums, or an odd value that is inf, NaN or huge) the step takes the full definition.
                        if (marked) {
                            constexpr uint32_t kLeast = kPlainExpMin << 23;
                            // (row by row and column by column, and only those that hold an odd value somewhere in the
                            // wavefront: mostly one of the eight)
                            bool fits = true;
                            auto pair_fits = [&](int i, int j) __attribute__((always_inline)) {
                                const uint32_t fa = (ua[i] >> 23) & 0xffu, fb = (ub[j] >> 23) & 0xffu;
                                const int ea = oa[i] ? (int)kPlainExpMin : (int)fa, eb = ob[j] ? (int)kPlainExpMin : (int)fb;
                                const int es = (int)((f2u(acc[i][j]) >> 23) & 0xffu);
                                const bool tiny = (!oa[i] || fa < kPlainExpMin) && (!ob[j] || fb < kPlainExpMin);
                                return tiny && es >= ea + eb - 96;
                            };
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                if (__ballot(oa[i]) != 0ull) {
#pragma unroll
                                    for (int j = 0; j < 4; ++j) fits &= !oa[i] || pair_fits(i, j);
                                }
#pragma unroll
                            for (int j = 0; j < 4; ++j)
                                if (__ballot(ob[j]) != 0ull) {
#pragma unroll
                                    for (int i = 0; i < 4; ++i) fits &= !ob[j] || pair_fits(i, j);
                                }
                            if (__ballot(!fits) == 0ull) {
                                va.x = oa[0] ? kLeast : va.x; va.y = oa[1] ? kLeast : va.y; va.z = oa[2] ? kLeast : va.z; va.w = oa[3] ? kLeast : va.w;
                                vb.x = ob[0] ? kLeast - kUnstage : vb.x; vb.y = ob[1] ? kLeast - kUnstage : vb.y;
                                vb.z = ob[2] ? kLeast - kUnstage : vb.z; vb.w = ob[3] ? kLeast - kUnstage : vb.w;
                                marked = false;
                            }
                        }
                    }
                    half = __builtin_amdgcn_readfirstlane(marked ? 0u : ~0u);
                }
                const uint64_t run = ((uint64_t)half << 32) | half;
                if constexpr (MODE == MODE_PAM) {
                    if constexpr (ZEROS) pam_mac_4x4_skip_both_under(acc, va, vb, pl, pr, run);
                    else pam_mac_4x4_under(acc, va, vb, pl, pr, run);
                } else {
                    pam_bwd_mac_4x4<MODE == MODE_BWD_DL, true>(acc, dfrac, va, vb, pl, pr, run);
                }
                if (__builtin_expect(marked, 0)) {
                    const uint32_t a[4] = {va.x, va.y, va.z, va.w}, b[4] = {vb.x, vb.y, vb.z, vb.w};
                    guarded_products(a, b);
                }
            };
            u32x4 fa0 = *reinterpret_cast<LdsVec>(pl), fb0 = *reinterpret_cast<LdsVec>(pr), fa1, fb1;
#pragma unroll 1
            for (int kk = 0; kk < BK; kk += 4) {
                // (the reads of a four at constant distances from one address: one address update per operand and four)
                fa1 = *reinterpret_cast<LdsVec>(pl + LDL * 4); fb1 = *reinterpret_cast<LdsVec>(pr + LDR * 4);
                step(kk, fa0, fb0);
                fa0 = *reinterpret_cast<LdsVec>(pl + 2 * LDL * 4); fb0 = *reinterpret_cast<LdsVec>(pr + 2 * LDR * 4);
                step(kk + 1, fa1, fb1);
                fa1 = *reinterpret_cast<LdsVec>(pl + 3 * LDL * 4); fb1 = *reinterpret_cast<LdsVec>(pr + 3 * LDR * 4);
                step(kk + 2, fa0, fb0);
                // (the last four read their own last step again: a read under a condition would make the wait before
                // the block below one for all reads, the two just issued included)
                pl += (kk + 4 < BK ? 4 : 3) * LDL * 4; pr += (kk + 4 < BK ? 4 : 3) * LDR * 4;
                if (BK == 32 && kk == 12) { pl += to_plx; pr += to_prx; }        // (see swizzled)
                fa0 = *reinterpret_cast<LdsVec>(pl); fb0 = *reinterpret_cast<LdsVec>(pr);
                step(kk + 3, fa1, fb1);
            }
        }
    };

    int t = 0;
    while (t < ktiles) {
        begin_tile(t);
        // Runs of full plain k-tiles -- nearly all of them -- are a loop of their own: the accumulators then stay
        // in the same registers from one k-tile to the next instead of being moved to where the other loops want them.
        while (verdict == 0 && kcount == BK) {
            plain_tile();
            end_tile(t);
            if (++t == ktiles) break;
            begin_tile(t);
        }
        if (t == ktiles) break;
        if (verdict == kIdle) { end_tile(t); ++t; continue; }
        // full k-tiles with zeros (activations after a ReLU, padding, pruned weights)
        if (kSkips && kcount == BK && verdict != 0 && verdict < kGuarded) {
            if (verdict == kZerosL) skip_tile(std::integral_constant<uint32_t, kZerosL>());
            else if (verdict == kZerosR) skip_tile(std::integral_constant<uint32_t, kZerosR>());
            else skip_tile(std::integral_constant<uint32_t, kZerosL | kZerosR>());
            end_tile(t);
            ++t;
            continue;
        }
        if (verdict == 0) {
#pragma unroll 1
            for (int kk = 0; kk < kcount; ++kk) fast_step(kk);
        } else if (verdict == kZerosL && MODE == MODE_PAM) {
#pragma unroll 1
            for (int kk = 0; kk < kcount; ++kk) zeros_left_step(kk);
        } else if (verdict == kZerosR && MODE == MODE_PAM) {
#pragma unroll 1
            for (int kk = 0; kk < kcount; ++kk) zeros_right_step(kk);
        } else if (verdict == (kZerosL | kZerosR) && MODE == MODE_PAM) {
#pragma unroll 2
            for (int kk = 0; kk < kcount; ++kk) zeros_step(kk);
        } else {
            // some value of the k-tile needs the full definition: only the k-steps that hold one pay for it
            uint32_t odd = 0u;
#pragma unroll
            for (int w = 0; w < NW; ++w) odd |= lds_flag[t & 1][w] >= kGuarded ? lds_odd_k[t & 1][w] : 0u;     // only those wavefronts wrote one
            odd = __builtin_amdgcn_readfirstlane(odd);
            const bool zeros = MODE == MODE_PAM && (verdict & (kZerosL | kZerosR)) != 0;    // somewhere in the tile
            if (MODE != MODE_STD && TM == 4 && TN == 4 && kcount == BK) {
                if (zeros) mixed_tile(odd, std::true_type()); else mixed_tile(odd, std::false_type());
                end_tile(t);
                ++t;
                continue;
            }
#pragma unroll 1
            for (int kk = 0; kk < kcount; ++kk) {
                if ((odd >> kk) & 1u) guarded_step(kk);
                else if (zeros) zeros_step(kk);
                else fast_step(kk);
            }
        }
        end_tile(t);
        ++t;
    }

    // ---- the sums' way out
    // A piece of a cut tile goes to its slot of the workspace.  If that completes the tile (and the launch folds its
    // tiles itself), the pieces are added in ascending k order from +0.
    const LateArgs e = late_args();
    if constexpr (CUT) {
        if (!e->fold_here) {                       // a second kernel adds the pieces: ordinary stores, the launch's end publishes them
#pragma unroll
            for (int i = 0; i < TM; ++i) *piece_row(e->partial, (long)flat * e->pieces + piece, i, tid) = v4f{acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
            return;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                __hip_atomic_store(piece_half(e->partial, unit, i, h, tid), ((Pair)f2u(acc[i][2 * h + 1]) << 32) | f2u(acc[i][2 * h]),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // the stores have completed (they are write-through at this scope) before any lane of the work-group arrives
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        unsigned long long* word = e->arrive + flat;
        if (tid == 0) lds_arrived = arrive_at(word, e->tag) + 1u;
        __syncthreads();
        if (__builtin_amdgcn_readfirstlane(lds_arrived) != (uint32_t)e->pieces) return;
        asm volatile("" ::: "memory");
        fold_pieces(e->partial, (long)flat * e->pieces, e->pieces, tid, acc);
        if (tid == 0) __hip_atomic_store(word, ((e->tag + 1) & kTagMask) << kTagShift, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);    // ready for the next launch
    }
    // the finished sums of the tile to Y (plus the bias, if any)
    float* out = e->Y + (long)zb * e->y_sb;
    const long o_sr = e->y_sr, o_sc = e->y_sc;
    if (e->bias) {
#pragma unroll
        for (int gj = 0; gj < GN; ++gj)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = col0 + gj * (BN / GN) + tx * 4 + j;
                const float bv = c < g.N ? e->bias[c] : 0.0f;
#pragma unroll
                for (int i = 0; i < TM; ++i) acc[i][gj * 4 + j] = acc[i][gj * 4 + j] + bv;
            }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        int r = row0 + (i / 4) * (BM / GM) + ty * 4 + (i % 4);
        if (r >= g.M) continue;
#pragma unroll
        for (int gj = 0; gj < GN; ++gj) {
            int c = col0 + gj * (BN / GN) + tx * 4;
            float* dst = out + (long)r * o_sr + (long)c * o_sc;
            if (o_sc == 1 && c + 3 < g.N && ((reinterpret_cast<uintptr_t>(dst) & 15u) == 0)) {
                *reinterpret_cast<float4*>(dst) = make_float4(acc[i][gj * 4], acc[i][gj * 4 + 1], acc[i][gj * 4 + 2], acc[i][gj * 4 + 3]);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (c + j < g.N) dst[(long)j * o_sc] = acc[i][gj * 4 + j];
            }
        }
    }
}

template <int BK, int MODE>
void launch_gemm(int lk, int rk, unsigned groups, hipStream_t st, const GemmArgs& g)
{
#define PAM_GEMM_CASE(LK, RK) \
    if (lk == LK && rk == RK) {                                                                                                   \
        if (g.pieces > 1) hipLaunchKernelGGL((gemm_kernel<64, 64, 4, 4, BK, MODE, LK, RK, true>), dim3(groups), dim3(256), 0, st, g);  \
        else hipLaunchKernelGGL((gemm_kernel<64, 64, 4, 4, BK, MODE, LK, RK, false>), dim3(groups), dim3(256), 0, st, g);            \
        return;                                                                                                                   \
    }
    PAM_GEMM_CASE(LOAD_KVEC, LOAD_KVEC) PAM_GEMM_CASE(LOAD_KVEC, LOAD_RVEC) PAM_GEMM_CASE(LOAD_RVEC, LOAD_RVEC)
    PAM_GEMM_CASE(LOAD_KVEC, LOAD_ANY)
    PAM_GEMM_CASE(LOAD_RVEC, LOAD_KVEC) PAM_GEMM_CASE(LOAD_RVEC, LOAD_ANY)
    PAM_GEMM_CASE(LOAD_ANY, LOAD_KVEC) PAM_GEMM_CASE(LOAD_ANY, LOAD_RVEC) PAM_GEMM_CASE(LOAD_ANY, LOAD_ANY)
    if constexpr (MODE != MODE_STD) {                                  // image patches as the right operand
        PAM_GEMM_CASE(LOAD_KVEC, LOAD_CONV) PAM_GEMM_CASE(LOAD_RVEC, LOAD_CONV) PAM_GEMM_CASE(LOAD_ANY, LOAD_CONV)
        if constexpr (MODE == MODE_PAM) { PAM_GEMM_CASE(LOAD_KVEC, LOAD_CONVQ) }      // (forward products of patch embeddings)
        PAM_GEMM_CASE(LOAD_KVEC, LOAD_CONVR)                                          // (convolutions of horizontal stride 1)
        PAM_GEMM_CASE(LOAD_KVEC, LOAD_CONVK)                                          // (... their weight gradients)
    }
#undef PAM_GEMM_CASE
}

// Each (k-tile depth, mode) pair is instantiated in a source file of its own (pam_gemm_inst_*.hip).
#define PAM_GEMM_EXTERN(BK, MODE) extern template void launch_gemm<BK, MODE>(int, int, unsigned, hipStream_t, const GemmArgs&);
PAM_GEMM_EXTERN(16, MODE_PAM) PAM_GEMM_EXTERN(32, MODE_PAM) PAM_GEMM_EXTERN(16, MODE_STD) PAM_GEMM_EXTERN(32, MODE_STD)
PAM_GEMM_EXTERN(16, MODE_BWD_DL) PAM_GEMM_EXTERN(32, MODE_BWD_DL) PAM_GEMM_EXTERN(16, MODE_BWD_DR) PAM_GEMM_EXTERN(32, MODE_BWD_DR)
#undef PAM_GEMM_EXTERN

}  // namespace pamgemm
