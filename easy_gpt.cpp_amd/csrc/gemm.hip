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

}  // namespace egpt

using namespace egpt;

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
