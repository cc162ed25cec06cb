// PAM matrix products for gfx950: Y[b,i,j] = sum_k mul(L[b,i,k], R[b,k,j]).
//
// A PAM product is an integer add of the two bit patterns (pam/cuda_kernels.cu:17-19),
// so the matrix cores do not apply; this is a VALU kernel whose inner loop is, per
// multiply-accumulate, one v_add_u32 and one v_add_f32.
//
//  * A work-group of four wavefronts owns a 64 x 64 tile of Y.  Each lane owns a 4 x 4
//    micro-tile in registers, each wavefront 32 x 32 outputs (lanes 8 x 8).  Measured on
//    MI355X, a SIMD retires a wave64 VALU instruction every two cycles but one wavefront
//    issues at most one every four, so several wavefronts per SIMD are needed (four are
//    resident: 104 registers, 35 KB of LDS per work-group with 32-deep k-tiles); larger
//    micro-tiles and more resident wavefronts were measured and gained nothing.  Thousands
//    of equal work-groups per product are what balances the 256 compute units.
//  * L and R tiles are staged through LDS k-major ([k][row], 4-word row pad), so a fragment
//    for one k is two ds_read_b128, contiguous (R) or broadcast (L) across the wavefront.
//    Operands whose contiguous dimension is k (row-major L, "column-major" R) are
//    transposed on the way in; operands contiguous along the row use 128-bit LDS writes;
//    anything else goes through a scalar loader.  No transposed copies are made in global
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
//    k = 12608) split k across work-groups; the partial tiles go through a scratch buffer
//    and are added in ascending order by a second kernel.
//  * The launch is one-dimensional over (matrix, k chunk, tile) units and every XCD (own L2)
//    takes one contiguous range of them, so each operand is fetched from memory about once.
//  * The right operand may be the patches of an image read in place (convolutions), and a
//    bias may be added to the finished sums (linear layers).
//  * Accumulation order: every output is summed by one lane per k chunk, k ascending, from
//    +0 -- with one chunk this is the order of the reference kernel
//    (pam/cuda_kernels.cu:601, 608-627); pam_hip_gemm_plan reports the chunking.
#include <cmath>
#include <cstring>
#include <mutex>
#include <type_traits>

#include <atomic>

#include "pam_common.h"
#include "../../include/pam_hip_probe.h"
#include "pam_device.h"

using namespace pamdev;

namespace {

enum { MODE_PAM = 0, MODE_STD = 1, MODE_BWD_DL = 2, MODE_BWD_DR = 3 };
enum { LOAD_KVEC = 0, LOAD_RVEC = 1, LOAD_ANY = 2, LOAD_CONV = 3 };   // k contiguous / row contiguous / any strides / image patches

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
struct ConvGeom { const int2* ktab; const int2* ltab; int H, W; int transposed; };

struct GemmArgs {
    Operand L, R;
    ConvGeom cv;
    const float* D; long d_sb, d_sr, d_sc;
    float* Y; long y_sb, y_sr, y_sc;
    const float* bias;           // one value per output column, added once after the sum, or null
    int M, N, K;
    int ksplit, kchunk;          // kchunk is a multiple of 32; ksplit == 1 means no split
    int tiles, batch;            // output tiles per matrix, matrices
    long xcd_chunk, units;       // xcd_chunk > 0: a 1-D launch, work-group x takes unit (x % XCDS) * xcd_chunk + x / XCDS (see the launch)
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
    uint32_t emin = 255u, emax = 0u;
    bool bad = false, zero = false;
    __device__ __forceinline__ uint32_t one(float v)
    {
        uint32_t u = f2u(v);
        if (MODE == MODE_STD) return u;
        if (kDeltaSide) {                          // the upstream gradient: zero is harmless
            bad |= !((((u >> 23) & 0xffu) - 64u < 127u) || (u & ~kSign) == 0);
            return u;
        }
        uint32_t e = (u >> 23) & 0xffu;
        if (MODE == MODE_PAM) {                    // zeros get their own, cheaper loop
            bool z = (u & ~kSign) == 0;
            zero |= z;
            e = z ? 127u : e;
            emin = min(emin, e); emax = max(emax, e);
            return z ? (IS_R ? kZeroR : kZeroL) : (IS_R ? u - kBias : u);
        }
        // slope side of a backward mode: a zero needs no care, (0 + fraction) & ~mantissa is 0 and the
        // fma then adds delta * 0 (delta is finite in the plain loop), which is what the definition gives
        if ((u & ~kSign) == 0) return u;
        emin = min(emin, e); emax = max(emax, e);
        return u;
    }
    // some staged value lies outside [2^-63, 2^64) or is not a normal number or zero
    __device__ __forceinline__ bool out_of_range() const { return bad || emin < 64u || emax > 190u; }
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
// A wavefront all of whose rows lie beyond M (the last row tile of a matrix whose height is not a multiple of the
// tile: 197 rows leave three of the four wavefronts of the fourth tile without a row) stages and synchronises with
// the others but computes nothing.
constexpr uint32_t kIdle = 8u;

// Stand-ins that keep the integer sum a finite number when one operand is zero: 2^-64 on the
// left, 2^64 (less the bias) on the right, just outside the range [2^-63, 2^64) that the other
// values of such a k-tile lie in.  The product is then multiplied by 0.
constexpr uint32_t kStandInL = 63u << 23;
constexpr uint32_t kStandInR = 64u << 23;

// One operand's tile: ROWS x BK values from global memory into registers, then into LDS.
template <int ROWS, int NT, int KIND, int BK>
struct TileLoader {
    static constexpr int kVecs = ROWS * BK / 4 / NT;      // float4 per lane (vector kinds)
    static constexpr int kElems = ROWS * BK / NT;         // scalars per lane (generic kind)
    static_assert(ROWS * BK % (4 * NT) == 0 && NT % ROWS == 0, "tile must divide over the work-group");
    float4 v[kVecs > 0 ? kVecs : 1];
    int2 fixed; bool have_fixed = false;          // LOAD_CONV: the lane's own table entry

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
        constexpr int n = (KIND == LOAD_KVEC || KIND == LOAD_RVEC) ? 4 * kVecs : kElems;
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
        auto see = [&](float f, int k) __attribute__((always_inline)) {
            const uint32_t u = f2u(f), e = (u >> 23) & 0xffu;
            odd |= (uint32_t)((u & ~kSign) != 0 && e - 64u > 126u) << k;
        };
        if (KIND == LOAD_KVEC) {
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                const int k = ((tid + i * NT) % (BK / 4)) * 4;
                see(v[i].x, k); see(v[i].y, k + 1); see(v[i].z, k + 2); see(v[i].w, k + 3);
            }
        } else if (KIND == LOAD_RVEC) {
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
        if (KIND == LOAD_KVEC) {
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                int id = tid + i * NT;
                uint32_t* d = lds + ((id % (BK / 4)) * 4) * LD + id / (BK / 4);
                d[0 * LD] = st.one(v[i].x); d[1 * LD] = st.one(v[i].y);
                d[2 * LD] = st.one(v[i].z); d[3 * LD] = st.one(v[i].w);
            }
        } else if (KIND == LOAD_RVEC) {
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                int id = tid + i * NT;
                uint4 w;
                w.x = st.one(v[i].x); w.y = st.one(v[i].y); w.z = st.one(v[i].z); w.w = st.one(v[i].w);
                *reinterpret_cast<uint4*>(lds + (id / (ROWS / 4)) * LD + (id % (ROWS / 4)) * 4) = w;
            }
        } else {                                    // LOAD_ANY and LOAD_CONV: lane-consecutive rows
            const float* s = reinterpret_cast<const float*>(v);
#pragma unroll
            for (int i = 0; i < kElems; ++i) {
                int id = tid + i * NT;
                lds[(id / ROWS) * LD + id % ROWS] = st.one(s[i]);
            }
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

template <int BM, int BN, int TM, int TN, int BK, int MODE, int LKIND, int RKIND>
__global__ __launch_bounds__((BM / TM) * (BN / TN)) PAM_GEMM_OCCUPANCY void gemm_kernel(GemmArgs g, float* __restrict__ partial)
{
    constexpr int TXN = BN / TN, TYN = BM / TM, NT = TXN * TYN, NW = NT / 64;
    constexpr int GM = TM / 4, GN = TN / 4;               // 4-wide groups per micro-tile side
    constexpr int LDL = BM + PAD, LDR = BN + PAD;
    static_assert(TM % 4 == 0 && TN % 4 == 0 && NT % 64 == 0, "micro-tile is built from 4-wide groups");

    __shared__ __attribute__((aligned(16))) uint32_t lds_l[2][BK * LDL];
    __shared__ __attribute__((aligned(16))) uint32_t lds_r[2][BK * LDR];
    __shared__ uint32_t lds_flag[2][NW];
    __shared__ uint32_t lds_odd_k[2][NW];         // bit k: some value under k of the tile needs the full definition

    const int tid = threadIdx.x, tx = tid % TXN, ty = tid / TXN;
    const int wave = tid / 64, lane = tid % 64;
    const int ntn = (g.N + BN - 1) / BN;                  // consecutive tiles share L rows
    int tile = blockIdx.x, zs = blockIdx.y, zb = blockIdx.z;
    if (g.xcd_chunk > 0) {                                // units (matrix, k chunk, tile), one contiguous range per XCD
        const long unit = (long)(blockIdx.x % XCDS) * g.xcd_chunk + (long)(blockIdx.x / XCDS);
        if (unit >= g.units) return;                      // the ranges are rounded up: a few work-groups have nothing to do
        tile = (int)(unit % g.tiles);
        const long rest = unit / g.tiles;
        zs = (int)(rest % g.ksplit); zb = (int)(rest / g.ksplit);
    }
    const int row0 = (tile / ntn) * BM, col0 = (tile % ntn) * BN;
    const int kbegin = zs * g.kchunk;
    const int kend = min(g.K, kbegin + g.kchunk);
    const int ktiles = (kend - kbegin + BK - 1) / BK;
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
        const uint32_t worst = max(ll.window_max(kOffL && shifted, g.off_add), rl.window_max(kOffR && shifted, g.off_add));
        if (__builtin_expect(__ballot(worst >= kWindowSpan) == 0ull && g.has_off != 2, 1)) {
            PlainStager<true> plus{(MODE == MODE_PAM ? 0u - kBias : 0u) + (shifted ? g.off_add : 0u)};
            if (kOffL && (MODE == MODE_PAM || shifted)) ll.store(lds_l[buf], tid, plus); else ll.store(lds_l[buf], tid, same);
            if (kOffR && (MODE == MODE_PAM || shifted)) rl.store(lds_r[buf], tid, plus); else rl.store(lds_r[buf], tid, same);
            if (lane == 0) lds_flag[buf][wave] = 0u;      // (its k mask keeps an older value: readers go by the flag)
            return;
        }
        Stager<MODE, false> sl; Stager<MODE, true> sr;
        if (has_off) {
            if (Stager<MODE, false>::kTakesOffset) ll.apply_offset(g.off);
            if (Stager<MODE, true>::kTakesOffset) rl.apply_offset(g.off);
        }
        ll.store(lds_l[buf], tid, sl);
        rl.store(lds_r[buf], tid, sr);
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
    const uint32_t* sl = nullptr; const uint32_t* sr = nullptr;
    int kcount = 0;
    const bool idle_wave = MODE != MODE_STD && __builtin_amdgcn_readfirstlane(row0 + (wave * 64 / TXN) * 4 >= g.M ? 1 : 0) != 0;
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
        sl = lds_l[cur] + ty * 4;
        sr = lds_r[cur] + tx * 4;
    };
    auto end_tile = [&](int t) __attribute__((always_inline)) {
        if (t + 1 < ktiles) stage((t & 1) ^ 1);
        __syncthreads();
    };

    auto fragment = [&](int kk, uint32_t (&a)[TM], uint32_t (&b)[TN]) __attribute__((always_inline)) {
#pragma unroll
        for (int gi = 0; gi < GM; ++gi) {
            uint4 q = *reinterpret_cast<const uint4*>(sl + kk * LDL + gi * (BM / GM));
            a[gi * 4 + 0] = q.x; a[gi * 4 + 1] = q.y; a[gi * 4 + 2] = q.z; a[gi * 4 + 3] = q.w;
        }
#pragma unroll
        for (int gj = 0; gj < GN; ++gj) {
            uint4 q = *reinterpret_cast<const uint4*>(sr + kk * LDR + gj * (BN / GN));
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
            u32x4 fa[2], fb[2];
            fa[0] = *reinterpret_cast<LdsVec>(pl); fb[0] = *reinterpret_cast<LdsVec>(pr);
#pragma unroll
            for (int kk = 0; kk < BK; ++kk) {
                if (kk + 1 < BK) {
                    fa[(kk + 1) & 1] = *reinterpret_cast<LdsVec>(pl + (kk + 1) * LDL * 4);
                    fb[(kk + 1) & 1] = *reinterpret_cast<LdsVec>(pr + (kk + 1) * LDR * 4);
                }
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
            u32x4 va[2], vb[2];
            va[0] = *reinterpret_cast<LdsVec>(pl); vb[0] = *reinterpret_cast<LdsVec>(pr);
#pragma unroll
            for (int kk = 0; kk < BK; ++kk) {
                if (kk + 1 < BK) {
                    va[(kk + 1) & 1] = *reinterpret_cast<LdsVec>(pl + (kk + 1) * LDL * 4);
                    vb[(kk + 1) & 1] = *reinterpret_cast<LdsVec>(pr + (kk + 1) * LDR * 4);
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
                asm volatile("" : "+v"(pl), "+v"(pr),
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
            u32x4 fa[2], fb[2];
            fa[0] = *reinterpret_cast<LdsVec>(pl); fb[0] = *reinterpret_cast<LdsVec>(pr);
#pragma unroll
            for (int kk = 0; kk < BK; ++kk) {
                if (kk + 1 < BK) {
                    fa[(kk + 1) & 1] = *reinterpret_cast<LdsVec>(pl + (kk + 1) * LDL * 4);
                    fb[(kk + 1) & 1] = *reinterpret_cast<LdsVec>(pr + (kk + 1) * LDR * 4);
                }
                constexpr uint32_t kWhich = decltype(which)::value;
                if constexpr (kWhich == (kZerosL | kZerosR)) pam_mac_4x4_skip_both(acc, fa[kk & 1], fb[kk & 1], pl, pr);
                else pam_mac_4x4_skip<kWhich == kZerosL>(acc, fa[kk & 1], fb[kk & 1], pl, pr);
            }
        }
    };
    constexpr bool kSkips = MODE == MODE_PAM && TM == 4 && TN == 4;

    // a full k-tile some of whose k-steps hold a value in need of the full definition (bit k of `odd`): a rolled loop
    // over the k-steps in which every step passes through the plain block (the skipping one if the tile holds zeros
    // too, ZEROS) -- under an empty lane mask in the marked steps, whose products the full definition then adds.
    auto mixed_tile = [&](uint32_t odd, auto holds_zeros) __attribute__((always_inline)) {
        if constexpr (MODE != MODE_STD && TM == 4 && TN == 4) {
            constexpr bool ZEROS = decltype(holds_zeros)::value;
            typedef const __attribute__((address_space(3))) uint32_t* LdsWord;
            uint32_t pl = (uint32_t)(uintptr_t)(LdsWord)sl, pr = (uint32_t)(uintptr_t)(LdsWord)sr;
#pragma unroll 1
            for (int kk = 0; kk < BK; ++kk) {
                const u32x4 va = *reinterpret_cast<LdsVec>(pl), vb = *reinterpret_cast<LdsVec>(pr);
                pl += LDL * 4; pr += LDR * 4;
                // a marked step concerns the wavefronts whose lanes hold one of its odd values: 16 of a work-group's 256
                // lanes for a value of the left operand, 16 per wavefront for one of the right operand
                bool marked = ((odd >> kk) & 1u) != 0;
                if (__builtin_expect(marked, 0)) {
                    constexpr uint32_t kUnstage = MODE == MODE_PAM ? kBias : 0u;      // the right operand is staged less the bias
                    auto is_odd = [](uint32_t u) { return (u & ~kSign) != 0 && ((u >> 23) & 0xffu) - 64u > 126u; };
                    const bool mine = is_odd(va.x) || is_odd(va.y) || is_odd(va.z) || is_odd(va.w) || is_odd(vb.x + kUnstage)
                                   || is_odd(vb.y + kUnstage) || is_odd(vb.z + kUnstage) || is_odd(vb.w + kUnstage);
                    marked = __ballot(mine) != 0ull;
                }
                const uint32_t half = __builtin_amdgcn_readfirstlane(marked ? 0u : ~0u);     // (keeps the mask in scalar registers)
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

    // epilogue: to Y, or to this chunk's slab of the split-K scratch ([chunk][batch][M][N])
    float* out; long o_sr, o_sc;
    if (g.ksplit > 1) {
        out = partial + ((long)zs * g.batch + zb) * (long)g.M * g.N; o_sr = g.N; o_sc = 1;
    } else {
        out = g.Y + (long)zb * g.y_sb; o_sr = g.y_sr; o_sc = g.y_sc;
    }
    if (g.bias && g.ksplit == 1) {           // with split-K the reduction adds it
#pragma unroll
        for (int gj = 0; gj < GN; ++gj)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = col0 + gj * (BN / GN) + tx * 4 + j;
                const float bv = c < g.N ? g.bias[c] : 0.0f;
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

// Split-K: Y = ((0 + chunk0) + chunk1) + ... in ascending chunk order.  Loads of several chunks are
// in flight together; the additions keep their order.
template <class T>
__device__ __forceinline__ T splitk_sum(const T* __restrict__ p, int chunks, long stride)
{
    T total = T{};
    int c = 0;
    for (; c + 8 <= chunks; c += 8) {
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = p[(long)(c + u) * stride];
#pragma unroll
        for (int u = 0; u < 8; ++u) total += v[u];
    }
    for (; c < chunks; ++c) total += p[(long)c * stride];
    return total;
}

__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int chunks, long slab,
                                                           float* __restrict__ y, long y_sb, long y_sr, long y_sc, int M, int N,
                                                           const float* __restrict__ bias)
{
    long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= slab) return;
    float total = splitk_sum(partial + idx, chunks, slab);
    long b = idx / ((long)M * N), rem = idx % ((long)M * N);
    if (bias) total = total + bias[rem % N];
    y[b * y_sb + (rem / N) * y_sr + (rem % N) * y_sc] = total;
}

typedef float v4f __attribute__((ext_vector_type(4)));

// contiguous output, slab a multiple of four: 128-bit accesses
__global__ __launch_bounds__(256) void splitk_reduce_vec_kernel(const v4f* __restrict__ partial, int chunks, long slab4,
                                                               v4f* __restrict__ y, const float* __restrict__ bias, int N)
{
    long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= slab4) return;
    v4f total = splitk_sum(partial + idx, chunks, slab4);
    if (bias) {                                   // N is a multiple of four here: the four lanes share a row
        const int c = (int)((idx * 4) % N);
        total.x = total.x + bias[c]; total.y = total.y + bias[c + 1]; total.z = total.z + bias[c + 2]; total.w = total.w + bias[c + 3];
    }
    y[idx] = total;
}

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

struct Plan { int bk; int ksplit; int kchunk; };

// Tuning override for experiments, per calling thread (include/pam_hip_probe.h): bk 0 = automatic (16 or 32),
// ksplit 0 = automatic.
thread_local int g_force_bk = 0, g_force_ksplit = 0;

// Work-groups own 64 x 64 output tiles.  k of 128 and more in whole multiples of 32, and any k
// from 512, uses 32-deep k-tiles (fewer barriers and more bytes in flight per round, measured 3-5 %
// faster on 12608-row products); short or ragged k (attention: 64, 197) 16-deep ones.  k is split
// across work-groups when the tiles alone do not give each compute unit several work-groups: the aim is about
// eight equal work-groups per unit, each at least 128 deep in k.
Plan make_plan(long batch, long M, long N, long K, bool allow_split)
{
    const long cus = cu_count();
    const long tiles = batch * ((M + 63) / 64) * ((N + 63) / 64);
    const long kunits = K > 0 ? (K + KGRAN - 1) / KGRAN : 1;
    Plan p{(K >= 512 || (K >= 128 && K % 32 == 0)) ? 32 : 16, 1, (int)(kunits * KGRAN)};
    if (g_force_bk) p.bk = g_force_bk;
    long want = 1;
    if (g_force_ksplit > 0) want = g_force_ksplit;
    else if (tiles < 6 * cus) want = (8 * cus + tiles - 1) / tiles;
    long maxsplit = kunits / 4;                                  // at least 128 k per work-group
    if (want > maxsplit) want = maxsplit;
    if (allow_split && want > 1) {
        // Work-groups are dealt to the compute units in rounds of one each, and a round that is nearly empty costs
        // almost a full one: of the split counts next to the wanted one, take the one whose last round is fullest
        // (each extra chunk also costs a little in the reduction).
        long best_per = 0; double best = 0.0;
        for (long w = want - 1; w <= want + 1; ++w) {
            if (w < 2 || w > maxsplit || (g_force_ksplit > 0 && w != want)) continue;
            const long per = (kunits + w - 1) / w, chunks = (kunits + per - 1) / per;
            const double rounds = (double)(tiles * chunks) / (double)cus;
            const double cost = std::ceil(rounds) / rounds * (1.0 + 0.015 * (double)chunks);
            if (best_per == 0 || cost < best) { best = cost; best_per = per; }
        }
        if (best_per == 0) best_per = (kunits + want - 1) / want;
        p.kchunk = (int)(best_per * KGRAN);
        p.ksplit = (int)((kunits + best_per - 1) / best_per);
    }
    return p;
}

int load_kind(long s_row, long s_k, long s_batch, const float* p, long rows, long K)
{
    bool aligned = ((reinterpret_cast<uintptr_t>(p) & 15u) == 0) && (s_batch % 4 == 0);
    if (s_k == 1 && aligned && s_row % 4 == 0 && K % 4 == 0 && K >= 4) return LOAD_KVEC;
    if (s_row == 1 && aligned && s_k % 4 == 0 && rows % 4 == 0 && rows >= 4) return LOAD_RVEC;
    return LOAD_ANY;
}

template <int BK, int MODE>
void launch_kinds(int lk, int rk, dim3 grid, hipStream_t st, const GemmArgs& g, float* partial)
{
#define PAM_GEMM_CASE(LK, RK) \
    if (lk == LK && rk == RK) { hipLaunchKernelGGL((gemm_kernel<64, 64, 4, 4, BK, MODE, LK, RK>), grid, dim3(256), 0, st, g, partial); return; }
    PAM_GEMM_CASE(LOAD_KVEC, LOAD_KVEC) PAM_GEMM_CASE(LOAD_KVEC, LOAD_RVEC) PAM_GEMM_CASE(LOAD_RVEC, LOAD_RVEC)
    PAM_GEMM_CASE(LOAD_KVEC, LOAD_ANY)
    PAM_GEMM_CASE(LOAD_RVEC, LOAD_KVEC) PAM_GEMM_CASE(LOAD_RVEC, LOAD_ANY)
    PAM_GEMM_CASE(LOAD_ANY, LOAD_KVEC) PAM_GEMM_CASE(LOAD_ANY, LOAD_RVEC) PAM_GEMM_CASE(LOAD_ANY, LOAD_ANY)
    if constexpr (MODE != MODE_STD) {                                  // image patches as the right operand
        PAM_GEMM_CASE(LOAD_KVEC, LOAD_CONV) PAM_GEMM_CASE(LOAD_RVEC, LOAD_CONV) PAM_GEMM_CASE(LOAD_ANY, LOAD_CONV)
    }
#undef PAM_GEMM_CASE
}

template <int MODE>
void launch_mode(const Plan& p, int lk, int rk, hipStream_t st, const GemmArgs& g, long batch, float* partial)
{
    dim3 grid((unsigned)(((g.N + 63) / 64) * (long)((g.M + 63) / 64)), (unsigned)p.ksplit, (unsigned)batch);
    // Work-groups go to the eight XCDs in turn, and every XCD has its own L2.  With tiles in launch order the
    // column tiles of one row tile land on all eight, and each L2 fetches the whole left operand.  So the launch
    // is one-dimensional over units (matrix, k chunk, tile) and each XCD is given a contiguous range of them:
    // it reads only its own rows, chunks and matrices.
    GemmArgs ga = g;
    ga.tiles = (int)grid.x; ga.batch = (int)batch;
    const long units = (long)grid.x * p.ksplit * batch;
    // (not for few tiles with many k chunks, the weight-gradient shape: measured 8 % slower that way)
    if (units >= 64 && units < (1L << 31) - 8 && (p.ksplit == 1 || (long)grid.x >= cu_count())) {
        ga.units = units;
        ga.xcd_chunk = (units + XCDS - 1) / XCDS;
        grid = dim3((unsigned)(XCDS * ga.xcd_chunk), 1, 1);
    }
    if (p.bk == 32) launch_kinds<32, MODE>(lk, rk, grid, st, ga, partial);
    else launch_kinds<16, MODE>(lk, rk, grid, st, ga, partial);
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
    if (M > (1L << 30) || N > (1L << 30) || K > (1L << 30) || batch > 65535 || ((M + 63) / 64) * ((N + 63) / 64) > 0x7fffffffL)
        return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "%s: dimension too large (sizes <= 2^30, batch <= 65535, output tiles < 2^31)", what);
    hipStream_t st = (hipStream_t)stream;

    Plan p = make_plan(batch, M, N, K, workspace != nullptr);
    if (p.ksplit > 1 && (size_t)p.ksplit * batch * M * N * sizeof(float) > workspace_bytes) {
        p.ksplit = 1; p.kchunk = (int)((K + KGRAN - 1) / KGRAN * KGRAN);
    }
    if (p.kchunk < KGRAN) p.kchunk = KGRAN;

    GemmArgs g;
    g.L = Operand{l, l_sb, l_sr, l_sc};
    g.R = Operand{r, r_sb, r_sc, r_sr};            // R's "row" index is the output column
    g.D = d; g.d_sb = d_sb; g.d_sr = d_sr; g.d_sc = d_sc;
    g.Y = y; g.y_sb = y_sb; g.y_sr = y_sr; g.y_sc = y_sc;
    g.bias = bias;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.ksplit = p.ksplit; g.kchunk = p.kchunk;
    g.xcd_chunk = 0; g.units = 0; g.tiles = 0; g.batch = (int)batch;
    g.off = offset; g.off_add = 0; g.has_off = 0;
    if (mode != MODE_STD && offset != 1.0f) {
        uint32_t bits; memcpy(&bits, &offset, sizeof bits);
        g.has_off = std::isnormal(offset) ? 1 : 2;
        g.off_add = bits - kBias;
    }

    g.cv = conv ? *conv : ConvGeom{nullptr, nullptr, 0, 0, 0};

    int lk = load_kind(l_sr, l_sc, l_sb, l, M, K);
    int rk = conv ? LOAD_CONV : load_kind(r_sc, r_sr, r_sb, r, N, K);
    float* partial = (float*)workspace;
    switch (mode) {
    case MODE_PAM: launch_mode<MODE_PAM>(p, lk, rk, st, g, batch, partial); break;
    case MODE_STD: launch_mode<MODE_STD>(p, lk, rk, st, g, batch, partial); break;
    case MODE_BWD_DL: launch_mode<MODE_BWD_DL>(p, lk, rk, st, g, batch, partial); break;
    default: launch_mode<MODE_BWD_DR>(p, lk, rk, st, g, batch, partial); break;
    }
    if (p.ksplit > 1) {
        long slab = batch * M * N;
        const bool dense = y_sc == 1 && y_sr == N && (batch == 1 || y_sb == M * N) && slab % 4 == 0 && (!bias || N % 4 == 0) &&
                           ((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(partial)) & 15u) == 0;
        if (dense && slab / 4 >= 64L * cu_count())         // enough 128-bit lanes to fill the machine
            hipLaunchKernelGGL(splitk_reduce_vec_kernel, dim3((unsigned)((slab / 4 + 255) / 256)), dim3(256), 0, st,
                               (const v4f*)partial, p.ksplit, slab / 4, (v4f*)y, bias, (int)N);
        else
            hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((slab + 255) / 256)), dim3(256), 0, st,
                               partial, p.ksplit, slab, y, y_sb, y_sr, y_sc, (int)M, (int)N, bias);
    }
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

__global__ __launch_bounds__(256) void scale_kernel(const float* __restrict__ in, float* __restrict__ out, size_t n, float off)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) out[i] = pam_mul(in[i], off);
}

// wf[c][co][i][j] = w[co][c][kh-1-i][kw-1-j] (*) off: the weights of the convolution over the
// upstream gradient that yields the gradient of the input (stride 1)
// (with groups: c runs over all channels, co over the filters of c's group, and w is [filters][c per group][kh][kw])
__global__ __launch_bounds__(256) void flip_weights_kernel(const float* __restrict__ w, float* __restrict__ wf, int c, int cog, int cg, int kh, int kw,
                                                          float off, int has_off)
{
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= c * cog * kh * kw) return;
    const int j = idx % kw, i = (idx / kw) % kh, o = (idx / (kw * kh)) % cog, ci = idx / (kw * kh * cog);
    const int filter = (ci / cg) * cog + o;
    const float v = w[(((long)filter * cg + ci % cg) * kh + (kh - 1 - i)) * kw + (kw - 1 - j)];
    wf[idx] = has_off ? pam_mul(v, off) : v;
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

// workspace: [k table][l table][operand scaled by the offset, if any][split-k partial tiles]
struct ConvSpace { size_t tables, scaled, total; };
ConvSpace conv_space(const ConvShape& s, bool weight_gradient, bool has_off)
{
    ConvSpace w;
    w.tables = align256((size_t)(s.K() + s.L()) * sizeof(int2));
    size_t scaled_elems = !has_off ? 0 : weight_gradient ? (size_t)s.batch * s.co * s.L() : (size_t)s.co * s.K();
    w.scaled = align256(scaled_elems * sizeof(float));
    size_t split = weight_gradient ? pam_hip_gemm_workspace_bytes(s.batch, s.cog(), s.K(), s.L())
                                   : pam_hip_gemm_workspace_bytes(s.batch, s.cog(), s.L(), s.K());
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
    cv = ConvGeom{ktab, ltab, (int)s.h, (int)s.w, transposed ? 1 : 0};
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
    w.scaled = align256((size_t)t.co * t.K() * sizeof(float));
    w.total = w.tables + w.scaled + pam_hip_gemm_workspace_bytes(t.batch, t.cog(), t.L(), t.K());
    return w;
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
    Plan p = make_plan(batch, m, n, k, true);
    return p.ksplit > 1 ? (size_t)p.ksplit * batch * m * n * sizeof(float) : 0;
}

void pam_hip_set_tuning(int bk, int ksplit) { g_force_bk = bk; g_force_ksplit = ksplit; }

int pam_hip_gemm_plan(long batch, long m, long n, long k, int* k_chunk, int* k_group)
{
    if (batch <= 0 || m <= 0 || n <= 0 || k < 0) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "gemm_plan: bad shape");
    Plan p = make_plan(batch, m, n, k, true);
    if (k_chunk) *k_chunk = p.kchunk;
    if (k_group) *k_group = 1;
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
    return conv_space(s, which != 0, offset != 1.0f).total;
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
    ConvSpace sp = input_gradient_space(t);
    ConvGeom cv;
    rc = conv_prepare("conv2d_bwd_input", t, sp, workspace, workspace_bytes, st, cv, false);
    if (rc != PAM_HIP_OK) return rc;
    float* wf = (float*)((char*)workspace + sp.tables);
    const long n = c * s.cog() * kh * kw;
    // approximate: the offset goes into the flipped weights; exact: the product kernel applies it to its slope operand
    hipLaunchKernelGGL(flip_weights_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, w, wf, (int)c, (int)s.cog(), (int)s.cg(),
                       (int)kh, (int)kw, offset, (!exact && offset != 1.0f) ? 1 : 0);
    const long K = t.K(), L = t.L();                  // K = (co / groups) kh kw, L = h w
    void* rest = (char*)workspace + sp.tables + sp.scaled; size_t rest_bytes = workspace_bytes - sp.tables - sp.scaled;
    const long hw_out = s.ho * s.wo;
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
    ConvSpace sp = conv_space(s, false, has_off);
    ConvGeom cv;
    rc = conv_prepare("conv2d_fwd", s, sp, workspace, workspace_bytes, st, cv, false);
    if (rc != PAM_HIP_OK) return rc;
    // the reference folds the offset into the weights (the right operand of its product); here the
    // weights are the left operand, so they are scaled once up front
    const float* wl = w;
    if (has_off) {
        float* scaled = (float*)((char*)workspace + sp.tables);
        size_t n = (size_t)co * s.K();
        hipLaunchKernelGGL(scale_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, st, w, scaled, n, offset);
        wl = scaled;
    }
    const long K = s.K(), L = s.L();
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
    const bool scale = offset != 1.0f && !exact;
    ConvSpace sp = conv_space(s, true, scale);
    ConvGeom cv;
    rc = conv_prepare("conv2d_bwd_weight", s, sp, workspace, workspace_bytes, st, cv, true);
    if (rc != PAM_HIP_OK) return rc;
    const long K = s.K(), L = s.L();
    void* rest = (char*)workspace + sp.tables + sp.scaled; size_t rest_bytes = workspace_bytes - sp.tables - sp.scaled;
    // approximate: dW[co, k] = sum_l patches[k, l] (*) (dY[co, l] (*) offset), the gradient scaled once up front
    const float* dl = dy;
    if (scale) {
        float* scaled = (float*)((char*)workspace + sp.tables);
        size_t n = (size_t)batch * co * L;
        size_t blocks = (n + 1023) / 1024; if (blocks > (1u << 20)) blocks = 1u << 20;
        hipLaunchKernelGGL(scale_kernel, dim3((unsigned)blocks), dim3(256), 0, st, dy, scaled, n, offset);
        dl = scaled;
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
