// out[m, n] = sum_k x[m, k] * w[n, k] + bias[n]: the linear layer y = x W^T + b with W stored [out, in]
// (/root/reference/src/ops.cpp:101-118).
//
// gemm_tiled: plain FMA tiles in float32 arithmetic for every element type.  It is the product
// path for float32 (true 32-bit: no reduced-precision matrix mode) and the fallback for sizes the
// MFMA kernels refuse.
#include "api.h"
#include "common.h"

namespace egpt {

constexpr int BM = 64, BN = 64, BK = 16;

template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const TIn* __restrict__ x, const TIn* __restrict__ w,
                                                         const TIn* __restrict__ bias, TOut* __restrict__ out,
                                                         int m, int n, int k) {
    __shared__ float xs[BK][BM + 4];
    __shared__ float ws[BK][BN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int ty = tid / 16, tx = tid % 16;  // 16 x 16 threads, 4 x 4 outputs each
    float acc[4][4] = {};
    for (int k0 = 0; k0 < k; k0 += BK) {
        // each thread loads 4 elements of each tile: tile row = idx / BK, column = idx % BK
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = tid + i * 256;
            const int r = idx / BK, c = idx % BK;
            const int gm = m0 + r, gn = n0 + r, gk = k0 + c;
            xs[c][r] = (gm < m && gk < k) ? to_float(x[static_cast<size_t>(gm) * k + gk]) : 0.f;
            ws[c][r] = (gn < n && gk < k) ? to_float(w[static_cast<size_t>(gn) * k + gk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + ty * 4 + i;
        if (gm >= m) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tx * 4 + j;
            if (gn >= n) continue;
            const float v = acc[i][j] + (bias ? to_float(bias[gn]) : 0.f);
            out[static_cast<size_t>(gm) * n + gn] = from_float<TOut>(v);
        }
    }
}

template <typename TIn, typename TOut>
int launch_tiled(const void* x, const void* w, const void* bias, void* out, int m, int n, int k, hipStream_t s) {
    dim3 grid((n + BN - 1) / BN, (m + BM - 1) / BM);
    gemm_tiled_kernel<TIn, TOut><<<grid, 256, 0, s>>>(static_cast<const TIn*>(x), static_cast<const TIn*>(w),
                                                      static_cast<const TIn*>(bias), static_cast<TOut*>(out), m, n,
                                                      k);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

// ----------------------------------------------------------------------------- float32 on the matrix cores
// The float32 product: v_mfma_f32_16x16x4_f32 takes float32 operands and accumulates in float32 (no reduced-precision
// matrix mode).  A wavefront owns 16 rows of w (16 columns of the result) and streams them once for up to 64 rows of
// x, which the workgroup's four wavefronts share through LDS; more rows are further groups of 64 (blockIdx.z), the k
// range may be split over workgroups (blockIdx.y) into partial sums out[split][m][n].  Every element of the result is
// the same sequence of operations whatever m is and wherever its row lies in x: a step of 64 after the other, within
// a step one instruction after the other, each adding the products of four values of k.  So a token's values do not
// depend on what else is in the batch, to the bit.
constexpr int kStepF = 64;            // values of k per step
constexpr int kLdsRowF = kStepF + 4;  // floats per staged row of x (16 bytes of padding)
typedef __attribute__((ext_vector_type(4))) float f32x4;

template <int MT>
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ bias, float* __restrict__ out,
                                                            int m, int n, int k, int steps_per_split) {
    __shared__ __attribute__((aligned(16))) float xs[2][MT * 16][kLdsRowF];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int li = lane % 16, lg = lane / 16;
    const int split = blockIdx.y;
    const int m0 = blockIdx.z * 64;                       // first row of this group
    const int n0 = (blockIdx.x * 4 + wave) * 16;
    const int total_steps = (k + kStepF - 1) / kStepF;
    const int step_begin = split * steps_per_split;
    const int step_end = min(total_steps, step_begin + steps_per_split);
    // lane (li, lg) of a load takes the lg-th 16 bytes of each 64 of row li: an instruction reads 64 contiguous bytes
    // of each of its 16 rows; the j-th of its four values goes into the j-th product instruction, x likewise
    const float* wp = w + static_cast<size_t>(min(n0 + li, n - 1)) * k + lg * 4;
    auto load_w = [&](f32x4* av, int step) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int k0 = step * kStepF + q * 16 + lg * 4;
            av[q] = k0 < k ? *reinterpret_cast<const f32x4*>(wp + static_cast<size_t>(step) * kStepF + q * 16)
                           : f32x4{0.f, 0.f, 0.f, 0.f};
        }
    };
    float4 xr[MT];
    auto x_load = [&](int step) {
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            const int c = tid + j * 256, r = m0 + c / 16, kc = step * kStepF + (c % 16) * 4;
            xr[j] = (r < m && kc < k) ? *reinterpret_cast<const float4*>(x + static_cast<size_t>(r) * k + kc)
                                      : float4{0.f, 0.f, 0.f, 0.f};
        }
    };
    auto x_store = [&](int buf) {
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            const int c = tid + j * 256;
            *reinterpret_cast<float4*>(&xs[buf][c / 16][(c % 16) * 4]) = xr[j];
        }
    };
    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    // w runs kAhead steps ahead of the products (16 KB per wavefront on their way: with few rows the kernel is a
    // stream of w, and a stream one step deep was a chain of round trips, 1.1 TB/s on a 17 MB matrix); the order of
    // the products, and so every bit of the result, is that of the steps
    constexpr int kAhead = 4;
    f32x4 a[kAhead][4];     // (a native vector type: arrays of it stay in registers across the loop's back edge)
#pragma unroll
    for (int u = 0; u < kAhead; ++u)
        if (step_begin + u < step_end) load_w(a[u], step_begin + u);
    if (step_begin < step_end) {
        x_load(step_begin);
        x_store(0);
        if (step_begin + 1 < step_end) x_load(step_begin + 1);
    }
    __syncthreads();
    for (int step0 = step_begin; step0 < step_end; step0 += kAhead) {
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int step = step0 + u;
            if (step >= step_end) break;
            const int buf = u & 1;                  // (step - step_begin) & 1: kAhead is even
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float av[4] = {a[u][q][0], a[u][q][1], a[u][q][2], a[u][q][3]};
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const float4 b4 = *reinterpret_cast<const float4*>(&xs[buf][t * 16 + li][q * 16 + lg * 4]);
                    const float bv[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], bv[j], acc[t], 0, 0, 0);
                }
            }
            if (step + kAhead < step_end) load_w(a[u], step + kAhead);
            if (step + 1 < step_end) x_store(buf ^ 1);
            if (step + 2 < step_end) x_load(step + 2);
            __syncthreads();
        }
    }
    // D layout: lane (li, lg) holds rows lg*4 + v of the 16 x 16 tile (an n index) at column li (an m index)
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int mm = m0 + t * 16 + li;
        if (mm >= m) continue;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int nn = n0 + lg * 4 + v;
            if (nn >= n) continue;
            float val = acc[t][v];
            if (bias) val += bias[nn];
            out[(static_cast<size_t>(split) * m + mm) * n + nn] = val;
        }
    }
}

}  // namespace egpt

using namespace egpt;

extern "C" int egpt_gemm_f32(const float* x, const float* w, const float* bias, float* out, int m, int n, int k,
                             int n_splits, void* stream) {
    if (!x || !w || !out || m < 0 || n <= 0 || k <= 0 || n_splits < 1) return EGPT_BAD_ARGUMENT;
    if (k % 4 != 0 || (bias && n_splits != 1)) return EGPT_UNSUPPORTED_SIZE;
    if (m == 0) return EGPT_OK;
    const int total_steps = (k + kStepF - 1) / kStepF;
    const int steps_per_split = (total_steps + n_splits - 1) / n_splits;
    if (n_splits > total_steps || (n_splits - 1) * steps_per_split >= total_steps) return EGPT_BAD_ARGUMENT;   // an empty split
    const long groups = (static_cast<long>(m) + 63) / 64;
    if (groups > 65535 || n_splits > 65535) return EGPT_UNSUPPORTED_SIZE;
    const dim3 grid(static_cast<unsigned>((n + 63) / 64), static_cast<unsigned>(n_splits), static_cast<unsigned>(groups));
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (m > 64 ? 4 : (m + 15) / 16) {
        case 1: gemm_f32_mfma_kernel<1><<<grid, 256, 0, s>>>(x, w, bias, out, m, n, k, steps_per_split); break;
        case 2: gemm_f32_mfma_kernel<2><<<grid, 256, 0, s>>>(x, w, bias, out, m, n, k, steps_per_split); break;
        case 3: gemm_f32_mfma_kernel<3><<<grid, 256, 0, s>>>(x, w, bias, out, m, n, k, steps_per_split); break;
        default: gemm_f32_mfma_kernel<4><<<grid, 256, 0, s>>>(x, w, bias, out, m, n, k, steps_per_split); break;
    }
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_linear(const void* x, const void* w, const void* bias, void* out, int m, int n, int k, int dtype,
                           int out_f32, void* stream) {
    if (!x || !w || !out || m < 0 || n <= 0 || k <= 0) return EGPT_BAD_ARGUMENT;
    if (m == 0) return EGPT_OK;
    if ((static_cast<long>(m) + BM - 1) / BM > 65535) return EGPT_UNSUPPORTED_SIZE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == 0) return launch_tiled<float, float>(x, w, bias, out, m, n, k, s);
    if (dtype == 1) {
        if (out_f32) return launch_tiled<bf16_t, float>(x, w, bias, out, m, n, k, s);
        return launch_tiled<bf16_t, bf16_t>(x, w, bias, out, m, n, k, s);
    }
    return EGPT_BAD_ARGUMENT;
}
