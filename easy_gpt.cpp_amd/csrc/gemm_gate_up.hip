// Gate/up product with SwiGLU for a few dozen rows (17 to 64), bfloat16:
//     out[m, j] = up[m, j] * silu(gate[m, j]),  [gate | up] = x w^T,  w = [gate rows ; up rows]  ([2 * inter, k])
// (/root/reference/src/cuda/ops/mlp.cu:152-162 for the activation).
//
// With this many rows the weights are still read once and the time is still theirs, but x is no longer small:
// a workgroup that kept all of x in LDS would be alone on its CU, and with one workgroup per 64 columns most CUs
// would have none.  Here a workgroup owns only 16 gate columns and the 16 up columns of the same indices, and its
// four wavefronts share the k range (a quarter each): a wavefront loads its part of the 32 weight rows and of
// all rows of x straight into matrix-core operands (x comes from L2, where every workgroup finds it), with all
// loads of up to KC chunks of 32 in flight before the first product.  The four partial results meet in LDS, are
// added in wavefront order, and leave as activated bfloat16: neither the float32 product nor a SwiGLU kernel
// of its own stands between the norm and the down product.
#include "api.h"
#include "common.h"

namespace egpt {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kGuWaves = 4;
constexpr int kGuCols = 16;       // gate columns (and as many up columns) per column group

__device__ __forceinline__ uint4 load16_if(const bf16_t* p, bool ok) {
    return ok ? *reinterpret_cast<const uint4*>(p) : uint4{0u, 0u, 0u, 0u};
}

// MT: tiles of 16 rows of x; KC: chunks of 32 k elements whose loads are in flight together
template <int MT, int KC, int NG>
__global__ __launch_bounds__(64 * kGuWaves) void gemm_gate_up_kernel(const bf16_t* __restrict__ x,
                                                                     const bf16_t* __restrict__ w,
                                                                     bf16_t* __restrict__ out, int m, int inter, int k) {
    __shared__ f32x4 part[kGuWaves][MT][NG][2][kWave];
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int li = lane % 16, lg = lane / 16;
    const int n0 = blockIdx.x * kGuCols * NG;
    const int n_chunks = (k + 31) / 32;
    const int per_wave = (n_chunks + kGuWaves - 1) / kGuWaves;
    const int c_begin = wave * per_wave, c_end = min(n_chunks, c_begin + per_wave);
    const bf16_t* wg[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) wg[g] = w + static_cast<size_t>(min(n0 + g * kGuCols + li, inter - 1)) * k + lg * 8;
    const size_t up = static_cast<size_t>(inter) * k;          // from a gate row to the up row of the same column
    // Workgroups run in step and all read the same x: each starts at a row tile and a chunk of its own (and goes
    // round), so that they do not all ask the same lines of L2 for it at the same moment.  The order in which a
    // column's sum runs over k thus depends on the column, never on the rows.
    const int rot_t = (blockIdx.x / 8) % MT;
    const bf16_t* xp[MT];
    bool row_ok[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int tt = (t + rot_t) % MT;
        row_ok[t] = tt * 16 + li < m;
        xp[t] = x + static_cast<size_t>(min(tt * 16 + li, m - 1)) * k + lg * 8;
    }
    f32x4 acc[MT][NG][2];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int g = 0; g < NG; ++g) acc[t][g][0] = acc[t][g][1] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int c0 = c_begin; c0 < c_end; c0 += KC) {
        const int n_valid = min(KC, c_end - c0);
        const int rot_c = blockIdx.x % n_valid;
        uint4 gv[NG][KC], uv[NG][KC], xv[MT][KC];
        int kk[KC];
        bool ok[KC];
#pragma unroll
        for (int c = 0; c < KC; ++c) {                        // the weights first: they come from farther away
            const int cc = c + rot_c < n_valid ? c + rot_c : c + rot_c - n_valid;
            kk[c] = (c0 + cc) * 32;
            ok[c] = c < n_valid && kk[c] + lg * 8 < k;
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                gv[g][c] = load16_if(wg[g] + kk[c], ok[c]);
                uv[g][c] = load16_if(wg[g] + up + kk[c], ok[c]);
            }
        }
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int c = 0; c < KC; ++c) xv[t][c] = load16_if(xp[t] + kk[c], row_ok[t] && ok[c]);
        // D[row of x = lg * 4 + v][column = li]: a lane's four values are four rows of one column
#pragma unroll
        for (int c = 0; c < KC; ++c) {
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                const bf16x8 gw = __builtin_bit_cast(bf16x8, gv[g][c]), uw = __builtin_bit_cast(bf16x8, uv[g][c]);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const bf16x8 xa = __builtin_bit_cast(bf16x8, xv[t][c]);
                    acc[t][g][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa, gw, acc[t][g][0], 0, 0, 0);
                    acc[t][g][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa, uw, acc[t][g][1], 0, 0, 0);
                }
            }
        }
    }
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            part[wave][t][g][0][lane] = acc[t][g][0];
            part[wave][t][g][1][lane] = acc[t][g][1];
        }
    __syncthreads();
    // the wavefronts share the (row tile, column group) pairs: sums in wavefront order, the activation, one rounding
    for (int job = wave; job < MT * NG; job += kGuWaves) {
        const int t = job / NG, cg = job % NG;
        f32x4 g = part[0][t][cg][0][lane], u = part[0][t][cg][1][lane];
#pragma unroll
        for (int s = 1; s < kGuWaves; ++s) {
            const f32x4 pg = part[s][t][cg][0][lane], pu = part[s][t][cg][1][lane];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                g[v] += pg[v];
                u[v] += pu[v];
            }
        }
        const int column = n0 + cg * kGuCols + li;
        if (column >= inter) continue;
        const int tt = (t + rot_t) % MT;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int row = tt * 16 + lg * 4 + v;
            if (row < m)
                out[static_cast<size_t>(row) * inter + column] = from_float<bf16_t>(u[v] * (g[v] / (1.0f + expf(-g[v]))));
        }
    }
}

template <int MT, int NG>
static void launch_gate_up(const bf16_t* x, const bf16_t* w, bf16_t* out, int m, int inter, int k, hipStream_t s) {
    const int blocks = (inter + kGuCols * NG - 1) / (kGuCols * NG);
    const int per_wave = ((k + 31) / 32 + kGuWaves - 1) / kGuWaves;
    [[maybe_unused]] const dim3 grid(blocks);
    // rounds of 7 or 8 chunks: the fewer rounds, and of those the fewer registers
    if ((per_wave + 7) / 8 < (per_wave + 6) / 7)
        gemm_gate_up_kernel<MT, 8, NG><<<blocks, 64 * kGuWaves, 0, s>>>(x, w, out, m, inter, k);
    else
        gemm_gate_up_kernel<MT, 7, NG><<<blocks, 64 * kGuWaves, 0, s>>>(x, w, out, m, inter, k);
}

}  // namespace egpt

using namespace egpt;

// out bfloat16 [m][inter] = SwiGLU of x w^T; x bfloat16 [m][k], w bfloat16 [2 * inter][k] (gate rows, then up rows);
// m <= 64, k % 8 == 0.
extern "C" int egpt_gemm_gate_up_swiglu(const void* x, const void* w, void* out, int m, int inter, int k, int groups,
                                        void* stream) {
    if (!x || !w || !out || m <= 0 || inter <= 0 || k <= 0) return EGPT_BAD_ARGUMENT;
    if (m > 64 || (k % 8) != 0 || (groups != 1 && groups != 2)) return EGPT_UNSUPPORTED_SIZE;
    const bf16_t* xb = static_cast<const bf16_t*>(x);
    const bf16_t* wb = static_cast<const bf16_t*>(w);
    bf16_t* ob = static_cast<bf16_t*>(out);
    hipStream_t s = static_cast<hipStream_t>(stream);
#define EGPT_GATE_UP(MT_)                                                        \
    do {                                                                         \
        if (groups == 1) launch_gate_up<MT_, 1>(xb, wb, ob, m, inter, k, s);     \
        else launch_gate_up<MT_, 2>(xb, wb, ob, m, inter, k, s);                 \
    } while (0)
    switch ((m + 15) / 16) {
        case 1: EGPT_GATE_UP(1); break;
        case 2: EGPT_GATE_UP(2); break;
        case 3: EGPT_GATE_UP(3); break;
        default: EGPT_GATE_UP(4); break;
    }
#undef EGPT_GATE_UP
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
