// Weight-streaming product for few rows: out[m, n] = sum_k x[m, k] * w[n, k], m <= 64, bfloat16 operands,
// float32 accumulation on the matrix cores (v_mfma_f32_16x16x32_bf16).
//
// The time of such a product is the time to read w once from HBM, so the kernel is built around that
// stream: a wavefront owns 16 rows of w and walks a range of k in steps of 128; every lane loads 64
// contiguous bytes of one row per step (four 16-byte loads, issued one step ahead), which are four MFMA
// A operands as they are.  The k index inside an MFMA is only a summation index, so any assignment of k
// to (lane group, element) is right as long as x uses the same one; x is staged through LDS once per
// workgroup (four wavefronts = 64 rows of w share it) in exactly that order.
//
// To fill 256 CUs when n is small the k range is split over `n_splits` workgroups, each writing its
// partial sums to out[split][m][n] in float32.  The kernels that consume the result (bias + rotary +
// cache store, SwiGLU, residual add + RMSNorm) add the partial sums up, in a fixed order, so the result
// does not depend on scheduling.
#include "api.h"
#include "common.h"

namespace egpt {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kStep = 128;          // k elements per step
constexpr int kRowsPerWave = 16;
constexpr int kWavesPerBlock = 4;
constexpr int kLdsRow = kStep + 8;  // bf16 elements per staged row of x (16 bytes of padding)

__device__ __forceinline__ uint4 load16(const bf16_t* p, bool ok) {
    return ok ? *reinterpret_cast<const uint4*>(p) : uint4{0u, 0u, 0u, 0u};
}

template <int MT>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                          const bf16_t* __restrict__ bias, float* __restrict__ out_f32,
                                                          bf16_t* __restrict__ out_bf16, int m, int n, int k,
                                                          int steps_per_split) {
    __shared__ __attribute__((aligned(16))) bf16_t xs[2][MT * 16][kLdsRow];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int li = lane % 16, lg = lane / 16;
    const int split = blockIdx.y;
    const int n0 = (blockIdx.x * kWavesPerBlock + wave) * kRowsPerWave;
    const int total_steps = (k + kStep - 1) / kStep;
    const int step_begin = split * steps_per_split;
    const int step_end = min(total_steps, step_begin + steps_per_split);
    const int w_row = min(n0 + li, n - 1);
    const bf16_t* wp = w + static_cast<size_t>(w_row) * k + lg * 32;

    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    // staging of x: MT*16 rows x 128 columns = MT*16*16 chunks of 16 bytes, 256 threads
    auto stage = [&](int buf, int step) {
        const int k0 = step * kStep;
#pragma unroll
        for (int c = tid; c < MT * 16 * 16; c += 256) {
            const int r = c / 16, col = (c % 16) * 8;
            const bool ok = r < m && k0 + col < k;
            const uint4 v = load16(x + static_cast<size_t>(r) * k + k0 + col, ok);
            *reinterpret_cast<uint4*>(&xs[buf][r][col]) = v;
        }
    };
    uint4 a_cur[4], a_next[4];
    auto load_w = [&](uint4* a, int step) {
        const int k0 = step * kStep + lg * 32;
#pragma unroll
        for (int q = 0; q < 4; ++q) a[q] = load16(wp + static_cast<size_t>(step) * kStep + q * 8, k0 + q * 8 < k);
    };

    if (step_begin < step_end) {
        load_w(a_cur, step_begin);
        stage(0, step_begin);
    }
    __syncthreads();
    for (int step = step_begin; step < step_end; ++step) {
        const int buf = (step - step_begin) & 1;
        if (step + 1 < step_end) {
            load_w(a_next, step + 1);
            stage(buf ^ 1, step + 1);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const bf16x8 a = __builtin_bit_cast(bf16x8, a_cur[q]);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const uint4 bv = *reinterpret_cast<const uint4*>(&xs[buf][t * 16 + li][lg * 32 + q * 8]);
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, bv), acc[t], 0, 0, 0);
            }
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 4; ++q) a_cur[q] = a_next[q];
    }
    // D layout: lane (li, lg) holds rows lg*4 + v of the 16 x 16 tile (an n index) at column li (an m index)
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int mm = t * 16 + li;
        if (mm >= m) continue;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int nn = n0 + lg * 4 + v;
            if (nn >= n) continue;
            float val = acc[t][v];
            if (out_bf16) {
                if (bias) val += to_float(bias[nn]);
                out_bf16[static_cast<size_t>(mm) * n + nn] = from_float<bf16_t>(val);
            } else {
                if (bias) val += to_float(bias[nn]);
                out_f32[(static_cast<size_t>(split) * m + mm) * n + nn] = val;
            }
        }
    }
}

}  // namespace egpt

using namespace egpt;

// out_f32 != null: float32 [n_splits][m][n] partial sums (bias only allowed with n_splits == 1).
// out_bf16 != null: bfloat16 [m][n], n_splits must be 1.
extern "C" int egpt_gemm_skinny(const void* x, const void* w, const void* bias, float* out_f32, void* out_bf16, int m,
                                int n, int k, int n_splits, void* stream) {
    if (!x || !w || (!out_f32 && !out_bf16) || (out_f32 && out_bf16) || m <= 0 || n <= 0 || k <= 0 || n_splits <= 0)
        return EGPT_BAD_ARGUMENT;
    if (m > 64 || (k % 8) != 0) return EGPT_UNSUPPORTED_SIZE;
    if (n_splits > 1 && (bias || out_bf16)) return EGPT_BAD_ARGUMENT;
    const int total_steps = (k + kStep - 1) / kStep;
    if (n_splits > total_steps) return EGPT_BAD_ARGUMENT;
    const int steps_per_split = (total_steps + n_splits - 1) / n_splits;
    if ((n_splits - 1) * steps_per_split >= total_steps) return EGPT_BAD_ARGUMENT;  // an empty split
    dim3 grid((n + kRowsPerWave * kWavesPerBlock - 1) / (kRowsPerWave * kWavesPerBlock), n_splits);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const bf16_t* wp = static_cast<const bf16_t*>(w);
    const bf16_t* bp = static_cast<const bf16_t*>(bias);
    bf16_t* ob = static_cast<bf16_t*>(out_bf16);
    const int mt = (m + 15) / 16;
    switch (mt) {
        case 1: gemm_skinny_kernel<1><<<grid, 256, 0, s>>>(xp, wp, bp, out_f32, ob, m, n, k, steps_per_split); break;
        case 2: gemm_skinny_kernel<2><<<grid, 256, 0, s>>>(xp, wp, bp, out_f32, ob, m, n, k, steps_per_split); break;
        case 3: gemm_skinny_kernel<3><<<grid, 256, 0, s>>>(xp, wp, bp, out_f32, ob, m, n, k, steps_per_split); break;
        default: gemm_skinny_kernel<4><<<grid, 256, 0, s>>>(xp, wp, bp, out_f32, ob, m, n, k, steps_per_split); break;
    }
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
