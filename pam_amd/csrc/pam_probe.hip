// Measurement probes of libpam_hip.so (include/pam_hip_probe.h): the matrix kernel's instruction mix on register
// operands and on operands read from LDS, for the vector issue rate that roofline figures are stated against.
// Not part of the drop-in interface; the benchmark uses them.
#include "pam_common.h"
#include "pam_device.h"
#include "../../include/pam_hip_probe.h"

using namespace pamdev;

namespace {

constexpr int kThreads = 256;

// Measures what the vector ALUs issue on the matrix kernel's instruction mix with nothing else in the way:
// per lane 4 x 8 accumulators, and per product one v_add_u32 and one v_add_f32 that depends on it, operands in
// registers, no memory traffic.  The empty asm statements keep the compiler from hoisting the integer adds.
__global__ __launch_bounds__(kThreads) void issue_probe_kernel(const uint32_t* __restrict__ seed, float* __restrict__ out, int iters)
{
    const int lane = threadIdx.x;
    float acc[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = 0.0f;
    uint32_t a[4], b[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = seed[(lane + i) & 1023];
#pragma unroll
    for (int j = 0; j < 8; ++j) b[j] = seed[(lane * 3 + j) & 1023];
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(a[i]));
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[i][j] += u2f(a[i] + b[j]);
        }
    }
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) total += acc[i][j];
    out[(size_t)blockIdx.x * kThreads + lane] = total;
}

// The same with the operands of every step read from LDS as the matrix kernel reads them (k-major tiles, TM / 4 and
// TN / 4 128-bit reads per step, the next step's reads issued before this step's arithmetic): what a TM x TN
// micro-tile can reach with no staging, global loads or barriers in the way.
template <int TM, int TN>
__global__ __launch_bounds__(kThreads) void issue_probe_lds_kernel(const uint32_t* __restrict__ seed, float* __restrict__ out, int iters)
{
    constexpr int BK = 32, LD = 16 * (TM > TN ? TM : TN) + 4;
    __shared__ __attribute__((aligned(16))) uint32_t tile_a[BK * LD];
    __shared__ __attribute__((aligned(16))) uint32_t tile_b[BK * LD];
    const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    for (int i = tid; i < BK * LD; i += kThreads) { tile_a[i] = seed[i & 1023]; tile_b[i] = seed[(i * 7) & 1023]; }
    __syncthreads();
    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = 0.0f;
    const uint32_t* sa = tile_a + ty * 4;
    const uint32_t* sb = tile_b + tx * 4;
    auto fragment = [&](int kk, uint32_t (&a)[TM], uint32_t (&b)[TN]) {
#pragma unroll
        for (int g = 0; g < TM / 4; ++g) {
            const uint4 q = *reinterpret_cast<const uint4*>(sa + kk * LD + g * 64);
            a[g * 4] = q.x; a[g * 4 + 1] = q.y; a[g * 4 + 2] = q.z; a[g * 4 + 3] = q.w;
        }
#pragma unroll
        for (int g = 0; g < TN / 4; ++g) {
            const uint4 q = *reinterpret_cast<const uint4*>(sb + kk * LD + g * 64);
            b[g * 4] = q.x; b[g * 4 + 1] = q.y; b[g * 4 + 2] = q.z; b[g * 4 + 3] = q.w;
        }
    };
    for (int it = 0; it < iters; ++it) {
        int again = 0;
        asm volatile("" : "+v"(again));           // keeps the reads inside the loop: the compiler cannot tell the addresses repeat
        sa += again; sb += again;
        uint32_t fa[2][TM], fb[2][TN];
        fragment(0, fa[0], fb[0]);
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            if (kk + 1 < BK) fragment(kk + 1, fa[(kk + 1) & 1], fb[(kk + 1) & 1]);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] += u2f(fa[kk & 1][i] + fb[kk & 1][j]);
        }
    }
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) total += acc[i][j];
    out[(size_t)blockIdx.x * kThreads + tid] = total;
}

}  // namespace

extern "C" {

// seed: 1024 words (any bit patterns of normal numbers), out: blocks * 256 floats; each lane executes
// iters * 4 * 32 product-accumulate pairs = iters * 256 VALU lane-operations
int pam_hip_issue_probe(const void* seed, float* out, int blocks, int iters, void* stream)
{
    if (!seed || !out || blocks <= 0 || iters < 0) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "issue_probe: bad argument");
    hipLaunchKernelGGL(issue_probe_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream, (const uint32_t*)seed, out, iters);
    return pamhost::check_launch("issue_probe");
}

// micro-tile tm x tn in {4x4, 8x4, 8x8}; each lane executes iters * 32 * tm * tn product-accumulate pairs
int pam_hip_issue_probe_lds(const void* seed, float* out, int blocks, int iters, int tm, int tn, void* stream)
{
    if (!seed || !out || blocks <= 0 || iters < 0) return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "issue_probe_lds: bad argument");
    hipStream_t st = (hipStream_t)stream; const uint32_t* sd = (const uint32_t*)seed;
    if (tm == 4 && tn == 4) hipLaunchKernelGGL((issue_probe_lds_kernel<4, 4>), dim3((unsigned)blocks), dim3(kThreads), 0, st, sd, out, iters);
    else if (tm == 8 && tn == 4) hipLaunchKernelGGL((issue_probe_lds_kernel<8, 4>), dim3((unsigned)blocks), dim3(kThreads), 0, st, sd, out, iters);
    else if (tm == 8 && tn == 8) hipLaunchKernelGGL((issue_probe_lds_kernel<8, 8>), dim3((unsigned)blocks), dim3(kThreads), 0, st, sd, out, iters);
    else return pamhost::fail(PAM_HIP_ERR_ARGUMENT, "issue_probe_lds: micro-tile must be 4x4, 8x4 or 8x8");
    return pamhost::check_launch("issue_probe_lds");
}

}  // extern "C"
