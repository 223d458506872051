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
// partial sums to out[split][m][n] in float32.  The kernels that consume the result add the partial sums
// up, in a fixed order, so the result does not depend on scheduling.
//
// A decode step is a chain of small dependent kernels, and each link costs a few microseconds whatever it
// computes.  So for m <= 16 the staging of x can also compute x from what the previous kernels left
// ("prologues"), which removes the separate norm, SwiGLU and attention-combine kernels from the chain:
//   NORM    x = (h + sum_s delta_s) * norm_weight, not yet divided by the row's RMS: that factor is the same
//           for the whole row, so it is applied to the product afterwards by the consumer.  Workgroups of
//           the first column also write h + delta (the new residual stream, into a second buffer) and the
//           row's sum of squares of their k range.
//   SWIGLU  x = silu(g) * u with [g | u] = inv_rms * sum_s gate_up_s (partial sums of a NORM product).
//   ATTN    x = sum_s wgt_s * o_s: the combination of the partial attention results over key splits.
#include "api.h"
#include "common.h"

namespace egpt {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kStep = 128;          // k elements per step
constexpr int kRowsPerWave = 16;
constexpr int kLdsRow = kStep + 8;  // bf16 elements per staged row of x (16 bytes of padding)
constexpr int kMaxLocalHeads = 8;   // ATTN prologue: heads that one workgroup's k range may touch
constexpr int kMaxAttnSplits = 64;

enum Prologue { kPlain = 0, kNorm = 1, kSwiglu = 2, kAttn = 3 };

struct SkinnyArgs {
    const bf16_t* w;
    const bf16_t* bias;
    float* out_f32;
    bf16_t* out_bf16;
    fixed_t* acc_fixed;        // [m][n] residual stream in fixed point that the product is added into, or null
    int m, n, k, steps_per_split;
    // kPlain
    const bf16_t* x;
    // kNorm
    const float* h_in;
    const fixed_t* h_in_fixed; // the residual stream in fixed point instead of h_in (then no delta, no h_out)
    float* h_out;
    const float* delta;        // [delta_splits][m][k] or null
    int delta_splits;
    const bf16_t* norm_w;      // [k]
    float* ss_out;             // [n_splits][m]
    // kSwiglu: x[m][k] from gate_up [gu_splits][m][2k]
    const float* gu;
    int gu_splits;
    const float* ss_in;        // [ss_splits][m] or null
    int ss_splits;
    float inv_hidden, eps;
    // kAttn: x[m][head*hd + d] from part_o [a_splits][m*nq][hd], part_ml [a_splits][m*nq][2]
    const float* part_o;
    const float* part_ml;
    int a_splits, nq, hd;
};

__device__ __forceinline__ uint4 load16(const bf16_t* p, bool ok) {
    return ok ? *reinterpret_cast<const uint4*>(p) : uint4{0u, 0u, 0u, 0u};
}

__device__ __forceinline__ uint4 pack8(const float* v) {
    uint4 r;
    r.x = f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16);
    r.y = f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16);
    r.z = f32_to_bf16_bits(v[4]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[5])) << 16);
    r.w = f32_to_bf16_bits(v[6]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[7])) << 16);
    return r;
}

__device__ __forceinline__ void load8f(const float* p, float* v) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
    v[0] = a[0]; v[1] = a[1]; v[2] = a[2]; v[3] = a[3];
    v[4] = b[0]; v[5] = b[1]; v[6] = b[2]; v[7] = b[3];
}

// Adding partial sums up.  What a dependent kernel chain pays for is round trips to L2, not bytes, so the
// loads of one batch of splits are issued together, as straight-line code: a split past the last one reads
// the last one again (a cached line) and counts with weight zero, instead of a branch that would end the
// batch.  More loads in flight cost registers and with them the co-residency of workgroups, hence the batch
// size is the caller's choice.  Additions are in split order.
template <int INF>
__device__ __forceinline__ void add_splits8(const float* p, int n_splits, size_t stride, float* v) {
    for (int s0 = 0; s0 < n_splits; s0 += INF) {
        float t[INF][8];
#pragma unroll
        for (int i = 0; i < INF; ++i) load8f(p + min(s0 + i, n_splits - 1) * stride, t[i]);
#pragma unroll
        for (int i = 0; i < INF; ++i) {
            const float on = s0 + i < n_splits ? 1.f : 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = fmaf(on, t[i][j], v[j]);
        }
    }
}

// sum over splits of p[s * stride], 16 loads in flight
__device__ __forceinline__ float sum_splits(const float* p, int n_splits, size_t stride) {
    float v = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += 16) {
        float t[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) t[i] = p[min(s0 + i, n_splits - 1) * stride];
#pragma unroll
        for (int i = 0; i < 16; ++i) v += s0 + i < n_splits ? t[i] : 0.f;
    }
    return v;
}

// INF: how many splits' loads of the prologue's input are in flight together (kNorm, kAttn)
// NW: wavefronts per workgroup (each 16 rows of w); they share the staged x, so a wide workgroup reads the
// prologue's inputs fewer times
template <int MT, int PRO, int INF, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_skinny_kernel(SkinnyArgs a) {
    constexpr int kThreads = 64 * NW;
    __shared__ __attribute__((aligned(16))) bf16_t xs[2][MT * 16][kLdsRow];
    __shared__ float ss_part[2][16];                                     // kNorm: sums of squares of a short range
    __shared__ float head_wgt[PRO == kAttn ? 16 * kMaxLocalHeads * kMaxAttnSplits : 1];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int li = lane % 16, lg = lane / 16;
    const int split = blockIdx.y;
    const int m = a.m, n = a.n, k = a.k;
    const int n0 = (blockIdx.x * NW + wave) * kRowsPerWave;
    const int total_steps = (k + kStep - 1) / kStep;
    const int step_begin = split * a.steps_per_split;
    const int step_end = min(total_steps, step_begin + a.steps_per_split);
    const int n_steps = step_end - step_begin;
    const int w_row = min(n0 + li, n - 1);
    // lane group lg takes the lg-th 16 bytes of each 64 of a row: the four groups of a load instruction read 64
    // contiguous bytes of each of its 16 rows (a memory request is 64 bytes wide; x is read from LDS the same way)
    const bf16_t* wp = a.w + static_cast<size_t>(w_row) * k + lg * 8;

    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    uint4 a_cur[4], a_next[4];
    auto load_w = [&](uint4* av, int step) {
        const int k0 = step * kStep + lg * 8;
#pragma unroll
        for (int q = 0; q < 4; ++q) av[q] = load16(wp + static_cast<size_t>(step) * kStep + q * 32, k0 + q * 32 < k);
    };
    // the stream of w starts before anything else
    if (n_steps > 0) load_w(a_cur, step_begin);
    if (n_steps > 1) load_w(a_next, step_begin + 1);

    // ---- kAttn with many key splits: the weights of the splits once per workgroup, through LDS
    int head_begin = 0;
    const bool attn_wide = PRO == kAttn && a.a_splits > INF;
    if constexpr (PRO == kAttn) {
        head_begin = (step_begin * kStep) / a.hd;
        if (attn_wide) {
            // weight of split s for (row r, head): exp(max_s - max) / sum_s exp(max_s - max) * l_s
            const int head_end = min(a.nq, (min(k, step_end * kStep) + a.hd - 1) / a.hd);
            const int n_local = head_end - head_begin;
            const int rows = m * a.nq;
            // 16 lanes per (row, head) pair, each lane four of the (at most 64) splits, so that all loads of a
            // pair are in flight together
            const int sub = tid % 16;
            for (int pair = tid / 16; pair < 16 * kMaxLocalHeads; pair += kThreads / 16) {
                const int r = pair / kMaxLocalHeads, hl = pair % kMaxLocalHeads;
                if (r >= m || hl >= n_local) continue;                 // the same for all 16 lanes of the pair
                const size_t row = static_cast<size_t>(r) * a.nq + head_begin + hl;
                float ms[4], ls[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int sp = sub + 16 * i;
                    const bool has = sp < a.a_splits;
                    const float* p = a.part_ml + (static_cast<size_t>(has ? sp : 0) * rows + row) * 2;
                    ms[i] = has ? p[0] : -INFINITY;
                    ls[i] = has ? p[1] : 0.f;
                }
                float mx = fmaxf(fmaxf(ms[0], ms[1]), fmaxf(ms[2], ms[3]));
                mx = fmaxf(mx, __shfl_xor(mx, 1, kWave));
                mx = fmaxf(mx, __shfl_xor(mx, 2, kWave));
                mx = fmaxf(mx, __shfl_xor(mx, 4, kWave));
                mx = fmaxf(mx, __shfl_xor(mx, 8, kWave));
                float wg[4], denom = 0.f;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    wg[i] = ms[i] == -INFINITY ? 0.f : __expf(ms[i] - mx);
                    denom += wg[i] * ls[i];
                }
                denom += __shfl_xor(denom, 1, kWave);
                denom += __shfl_xor(denom, 2, kWave);
                denom += __shfl_xor(denom, 4, kWave);
                denom += __shfl_xor(denom, 8, kWave);
                const float inv = 1.0f / denom;
#pragma unroll
                for (int i = 0; i < 4; ++i) head_wgt[pair * kMaxAttnSplits + sub + 16 * i] = wg[i] * inv;
            }
            __syncthreads();
        }
    }

    // ---- one chunk of x: the 8 values of row r at columns col.. of step `step`, computed by the prologue and
    // stored where the MFMA operand loads expect them.  Returns the chunk's sum of squares (kNorm).
    // Rows >= m are never written: an MFMA output column depends on its own column of x only, and the
    // columns of those rows are not stored.
    auto chunk = [&](int buf, int step, int r, int col) -> float {
        const int kc = step * kStep + col;
        uint4 v = uint4{0u, 0u, 0u, 0u};          // past k the operand is zero, as w's is
        float ssq = 0.f;
        if constexpr (PRO == kPlain) {
            v = load16(a.x + static_cast<size_t>(r) * k + kc, kc < k);
        } else if (kc < k) {
            float f[8];
            if constexpr (PRO == kNorm) {
                const size_t idx = static_cast<size_t>(r) * k + kc;
                const uint4 wv = *reinterpret_cast<const uint4*>(a.norm_w + kc);
                if (a.h_in_fixed) {
                    // the stream as the products before left it: nothing to add, nothing to write back
                    fixed_t hv[8];
                    const uint4* hp = reinterpret_cast<const uint4*>(a.h_in_fixed + idx);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint4 d = hp[q];
                        hv[2 * q] = static_cast<fixed_t>((static_cast<unsigned long long>(d.y) << 32) | d.x);
                        hv[2 * q + 1] = static_cast<fixed_t>((static_cast<unsigned long long>(d.w) << 32) | d.z);
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j) f[j] = fixed_to_float(hv[j]);
                } else {
                    load8f(a.h_in + idx, f);
                    if (a.delta) add_splits8<INF>(a.delta + idx, a.delta_splits, static_cast<size_t>(m) * k, f);
                    if (blockIdx.x == 0) {
                        *reinterpret_cast<f32x4*>(a.h_out + idx) = f32x4{f[0], f[1], f[2], f[3]};
                        *reinterpret_cast<f32x4*>(a.h_out + idx + 4) = f32x4{f[4], f[5], f[6], f[7]};
                    }
                }
                const uint32_t wb[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    ssq += f[j] * f[j];
                    const uint32_t bits = (j & 1) ? (wb[j / 2] & 0xffff0000u) : (wb[j / 2] << 16);
                    f[j] *= __uint_as_float(bits);
                }
            } else if constexpr (PRO == kSwiglu) {
                // gate, up and the row's sums of squares: every load is issued before the first is waited
                // for (the counter of outstanding loads is in order, so a wait for any of them is a wait for
                // the stream of w as well: one round trip in all)
                constexpr int GU = 4, SS = 8;     // splits per batch of loads
                const size_t idx = static_cast<size_t>(r) * 2 * k + kc;
                const size_t stride = static_cast<size_t>(m) * 2 * k;
                float tg[GU][8], tu[GU][8], sst[SS];
#pragma unroll
                for (int i = 0; i < GU; ++i) {
                    const float* p = a.gu + idx + min(i, a.gu_splits - 1) * stride;
                    load8f(p, tg[i]);
                    load8f(p + k, tu[i]);
                }
                const float* ssp = a.ss_in ? a.ss_in + r : a.gu;       // without a scale: any readable address
                const int ss_n = a.ss_in ? a.ss_splits : 1;
#pragma unroll
                for (int i = 0; i < SS; ++i) sst[i] = ssp[min(i, ss_n - 1) * m];
                float g[8] = {}, u[8] = {};
#pragma unroll
                for (int i = 0; i < GU; ++i) {
                    const float on = i < a.gu_splits ? 1.f : 0.f;
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        g[j] = fmaf(on, tg[i][j], g[j]);
                        u[j] = fmaf(on, tu[i][j], u[j]);
                    }
                }
                if (a.gu_splits > GU) {
                    add_splits8<GU>(a.gu + idx + GU * stride, a.gu_splits - GU, stride, g);
                    add_splits8<GU>(a.gu + idx + GU * stride + k, a.gu_splits - GU, stride, u);
                }
                float ss = 0.f;
#pragma unroll
                for (int i = 0; i < SS; ++i) ss += i < ss_n ? sst[i] : 0.f;
                if (ss_n > SS) ss += sum_splits(ssp + SS * m, ss_n - SS, m);
                const float inv = a.ss_in ? 1.0f / sqrtf(ss * a.inv_hidden + a.eps) : 1.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float gg = g[j] * inv;
                    f[j] = (u[j] * inv) * gg * __builtin_amdgcn_rcpf(1.0f + __expf(-gg));
                }
            } else {  // kAttn
                const int head = kc / a.hd, d = kc % a.hd;
                const size_t rows = static_cast<size_t>(m) * a.nq;
                const size_t row = static_cast<size_t>(r) * a.nq + head;
                const float* po = a.part_o + row * a.hd + d;
#pragma unroll
                for (int j = 0; j < 8; ++j) f[j] = 0.f;
                if (!attn_wide) {
                    // few splits: their (maximum, sum) pairs and outputs in one batch of loads, the weights
                    // computed by every thread for itself
                    float ms[INF], ls[INF], t[INF][8];
#pragma unroll
                    for (int i = 0; i < INF; ++i) {
                        const int sp = min(i, a.a_splits - 1);
                        const float* pm = a.part_ml + (sp * rows + row) * 2;
                        ms[i] = pm[0];
                        ls[i] = pm[1];
                        load8f(po + sp * rows * a.hd, t[i]);
                    }
                    float mx = -INFINITY;
#pragma unroll
                    for (int i = 0; i < INF; ++i) {
                        if (i >= a.a_splits) ms[i] = -INFINITY;
                        mx = fmaxf(mx, ms[i]);
                    }
                    float wg[INF], denom = 0.f;
#pragma unroll
                    for (int i = 0; i < INF; ++i) {
                        wg[i] = ms[i] == -INFINITY ? 0.f : __expf(ms[i] - mx);
                        denom += wg[i] * ls[i];
                    }
                    const float inv = 1.0f / denom;
#pragma unroll
                    for (int i = 0; i < INF; ++i) {
                        const float wt = wg[i] * inv;
#pragma unroll
                        for (int j = 0; j < 8; ++j) f[j] = fmaf(wt, t[i][j], f[j]);
                    }
                } else {
                    const float* wl = head_wgt + (r * kMaxLocalHeads + head - head_begin) * kMaxAttnSplits;
                    for (int s0 = 0; s0 < a.a_splits; s0 += INF) {
                        float t[INF][8];
#pragma unroll
                        for (int i = 0; i < INF; ++i) load8f(po + min(s0 + i, a.a_splits - 1) * rows * a.hd, t[i]);
#pragma unroll
                        for (int i = 0; i < INF; ++i) {
                            const float wt = s0 + i < a.a_splits ? wl[s0 + i] : 0.f;
#pragma unroll
                            for (int j = 0; j < 8; ++j) f[j] = fmaf(wt, t[i][j], f[j]);
                        }
                    }
                }
            }
            v = pack8(f);
        }
        *reinterpret_cast<uint4*>(&xs[buf][r][col]) = v;
        return ssq;
    };
    auto products = [&](int buf, const uint4* av4) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const bf16x8 av = __builtin_bit_cast(bf16x8, av4[q]);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const uint4 bv = *reinterpret_cast<const uint4*>(&xs[buf][t * 16 + li][q * 32 + lg * 8]);
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, __builtin_bit_cast(bf16x8, bv), acc[t], 0, 0, 0);
            }
        }
    };

    if (n_steps <= 2) {
        // A short range (the usual case when the k range is split): both steps are staged at once, the
        // chunks of the valid rows dealt out over all threads, so that the prologue is one round of loads.
        const int per_step = m * 16;
        for (int it = tid; it < n_steps * per_step; it += kThreads) {
            const int s = it / per_step, rem = it % per_step;
            const int r = rem / 16;
            float ssq = chunk(s, step_begin + s, r, (rem % 16) * 8);
            if constexpr (PRO == kNorm) {
                // the 16 threads of a (step, row) sit side by side in one wavefront
                ssq += __shfl_xor(ssq, 1, kWave);
                ssq += __shfl_xor(ssq, 2, kWave);
                ssq += __shfl_xor(ssq, 4, kWave);
                ssq += __shfl_xor(ssq, 8, kWave);
                if (rem % 16 == 0) ss_part[s][r] = ssq;
            }
        }
        __syncthreads();
        if (n_steps > 0) products(0, a_cur);
        if (n_steps > 1) products(1, a_next);
        if constexpr (PRO == kNorm) {
            if (blockIdx.x == 0 && tid < m)
                a.ss_out[split * m + tid] = (n_steps > 0 ? ss_part[0][tid] : 0.f) + (n_steps > 1 ? ss_part[1][tid] : 0.f);
        }
    } else if constexpr (PRO == kPlain) {
        // A long range of a given x: double-buffered in LDS, and on its way through registers a step before that:
        // the loads of step + 2 are issued when step + 1 has been written to LDS, so that a step does not wait for
        // its own x (with 64 rows that wait was a third of the kernel's time).
        constexpr int kChunks = (MT * 16 * 16 + kThreads - 1) / kThreads;
        uint4 xr[kChunks];
        auto x_load = [&](int step) {
#pragma unroll
            for (int j = 0; j < kChunks; ++j) {
                const int c = tid + j * kThreads, r = c / 16, kc = step * kStep + (c % 16) * 8;
                xr[j] = load16(a.x + static_cast<size_t>(min(r, m - 1)) * k + kc, r < m && kc < k);
            }
        };
        auto x_store = [&](int buf) {
#pragma unroll
            for (int j = 0; j < kChunks; ++j) {
                const int c = tid + j * kThreads;
                if (c < MT * 16 * 16) *reinterpret_cast<uint4*>(&xs[buf][c / 16][(c % 16) * 8]) = xr[j];
            }
        };
        x_load(step_begin);
        x_store(0);
        x_load(step_begin + 1);                   // n_steps > 2 here
        __syncthreads();
        for (int step = step_begin; step < step_end; ++step) {
            const int buf = (step - step_begin) & 1;
            if (step > step_begin && step + 1 < step_end) load_w(a_next, step + 1);
            products(buf, a_cur);
            if (step + 1 < step_end) x_store(buf ^ 1);
            if (step + 2 < step_end) x_load(step + 2);
            __syncthreads();
#pragma unroll
            for (int q = 0; q < 4; ++q) a_cur[q] = a_next[q];
        }
    } else {
        // A long range: x double-buffered in LDS, a thread keeps its (row, column) over the steps.
        float ss_acc = 0.f;
        auto stage = [&](int buf, int step) {
#pragma unroll
            for (int c = tid; c < MT * 16 * 16; c += kThreads) {
                const int r = c / 16;
                if (r < m) ss_acc += chunk(buf, step, r, (c % 16) * 8);
            }
        };
        stage(0, step_begin);
        __syncthreads();
        for (int step = step_begin; step < step_end; ++step) {
            const int buf = (step - step_begin) & 1;
            if (step > step_begin && step + 1 < step_end) load_w(a_next, step + 1);
            if (step + 1 < step_end) stage(buf ^ 1, step + 1);
            products(buf, a_cur);
            __syncthreads();
#pragma unroll
            for (int q = 0; q < 4; ++q) a_cur[q] = a_next[q];
        }
        if constexpr (PRO == kNorm) {
            if (blockIdx.x == 0) {
                float ss = ss_acc;
                ss += __shfl_xor(ss, 1, kWave);
                ss += __shfl_xor(ss, 2, kWave);
                ss += __shfl_xor(ss, 4, kWave);
                ss += __shfl_xor(ss, 8, kWave);
                const int r = tid / 16;
                if (tid % 16 == 0 && r < m) a.ss_out[split * m + r] = ss;
            }
        }
    }
    // D layout: lane (li, lg) holds rows lg*4 + v of the 16 x 16 tile (an n index) at column li (an m index)
    if (a.acc_fixed) {
        // Into the residual stream with atomics.  As the tiles lie in the registers, neighbouring lanes hold
        // neighbouring rows of x, far apart in memory, and an atomic instruction would touch a cache line per
        // lane; through LDS the workgroup's tile is turned so that neighbouring threads add to neighbouring
        // columns of one row (a quarter of the time for the down projection of the 0.5B sizes).
        if constexpr (MT == 1) {
            __shared__ float turned[16][NW * 16 + 1];
#pragma unroll
            for (int v = 0; v < 4; ++v) turned[li][wave * 16 + lg * 4 + v] = acc[0][v];
            __syncthreads();
            const int col0 = blockIdx.x * NW * 16;
            for (int idx = tid; idx < m * NW * 16; idx += kThreads) {
                const int r = idx / (NW * 16), c = idx % (NW * 16);
                if (col0 + c < n) fixed_add(a.acc_fixed + static_cast<size_t>(r) * n + col0 + c, turned[r][c]);
            }
        }
        return;
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int mm = t * 16 + li;
        if (mm >= m) continue;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int nn = n0 + lg * 4 + v;
            if (nn >= n) continue;
            float val = acc[t][v];
            if (a.bias) val += to_float(a.bias[nn]);
            if (a.out_bf16)
                a.out_bf16[static_cast<size_t>(mm) * n + nn] = from_float<bf16_t>(val);
            else
                a.out_f32[(static_cast<size_t>(split) * m + mm) * n + nn] = val;
        }
    }
}

// The product for 17 to 64 rows and many columns: x stays in LDS for the workgroup's whole k range (up to
// kResidentSteps steps of 128), staged once, and every load of w for that range is issued before the first
// product.  With that many rows the step-by-step kernel above pays for its barriers and for float32 partial
// sums that weigh as much as the weights; here a workgroup is one round of loads, its products and one store,
// and with a k range of the whole k the output needs no partial sums.
constexpr int kResidentSteps = 8;

template <int MT, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_resident_kernel(SkinnyArgs a) {
    constexpr int kThreads = 64 * NW;
    constexpr int kRow = kResidentSteps * kStep + 8;                       // bf16 elements per staged row
    __shared__ __attribute__((aligned(16))) bf16_t xs[MT * 16][kRow];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int li = lane % 16, lg = lane / 16;
    const int split = blockIdx.y;
    const int m = a.m, n = a.n, k = a.k;
    const int n0 = (blockIdx.x * NW + wave) * kRowsPerWave;
    const int total_steps = (k + kStep - 1) / kStep;
    const int step_begin = split * a.steps_per_split;
    const int n_steps = min(total_steps, step_begin + a.steps_per_split) - step_begin;       // <= kResidentSteps
    const int k_begin = step_begin * kStep;
    const int w_row = min(n0 + li, n - 1);
    const bf16_t* wp = a.w + static_cast<size_t>(w_row) * k + k_begin + lg * 8;

    // the whole stream of w for this workgroup
    uint4 av[kResidentSteps][4];
#pragma unroll
    for (int s = 0; s < kResidentSteps; ++s)
#pragma unroll
        for (int q = 0; q < 4; ++q)
            av[s][q] = load16(wp + s * kStep + q * 32, s < n_steps && k_begin + s * kStep + q * 32 + lg * 8 < k);
    // x: sixteen threads per row take its sixteen chunks of a step; a thread walks the steps of a row (all its
    // loads in flight together), then the next of its rows.  No division in any index: with a vector
    // instruction at four cycles, index arithmetic is what such a kernel would otherwise spend its time on.
    constexpr int kRowsPerPass = kThreads / 16;
    const int r16 = tid / 16, c16 = (tid % 16) * 8;
#pragma unroll
    for (int j = 0; j < (MT * 16 + kRowsPerPass - 1) / kRowsPerPass; ++j) {
        const int r = r16 + kRowsPerPass * j;
        if (r >= m) break;                     // rows past m are never read back
        const bf16_t* xp = a.x + static_cast<size_t>(r) * k + k_begin + c16;
        uint4 v[kResidentSteps];
#pragma unroll
        for (int st = 0; st < kResidentSteps; ++st)
            v[st] = load16(xp + st * kStep, st < n_steps && k_begin + st * kStep + c16 < k);
#pragma unroll
        for (int st = 0; st < kResidentSteps; ++st)
            if (st < n_steps) *reinterpret_cast<uint4*>(&xs[r][st * kStep + c16]) = v[st];
    }
    __syncthreads();

    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < kResidentSteps; ++s) {
        if (s >= n_steps) break;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const bf16x8 wv = __builtin_bit_cast(bf16x8, av[s][q]);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const uint4 bv = *reinterpret_cast<const uint4*>(&xs[t * 16 + li][s * kStep + q * 32 + lg * 8]);
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv, __builtin_bit_cast(bf16x8, bv), acc[t], 0, 0, 0);
            }
        }
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
            if (a.bias) val += to_float(a.bias[nn]);
            if (a.out_bf16)
                a.out_bf16[static_cast<size_t>(mm) * n + nn] = from_float<bf16_t>(val);
            else
                a.out_f32[(static_cast<size_t>(split) * m + mm) * n + nn] = val;
        }
    }
}

static int check_splits(int k, int n_splits, int* steps_per_split) {
    const int total_steps = (k + kStep - 1) / kStep;
    if (n_splits < 1 || n_splits > total_steps) return EGPT_BAD_ARGUMENT;
    *steps_per_split = (total_steps + n_splits - 1) / n_splits;
    if ((n_splits - 1) * *steps_per_split >= total_steps) return EGPT_BAD_ARGUMENT;  // an empty split
    return EGPT_OK;
}

static dim3 skinny_grid(int n, int n_splits, int waves) {
    return dim3((n + kRowsPerWave * waves - 1) / (kRowsPerWave * waves), n_splits);
}

// launches the instance for `waves` wavefronts per workgroup (4, 8 or 16)
#define EGPT_SKINNY(MT_, PRO_, INF_)                                                                         \
    do {                                                                                                     \
        const dim3 grid = skinny_grid(a.n, n_splits, waves);                                                 \
        hipStream_t s_ = static_cast<hipStream_t>(stream);                                                   \
        if (waves == 4) gemm_skinny_kernel<MT_, PRO_, INF_, 4><<<grid, 256, 0, s_>>>(a);                     \
        else if (waves == 8) gemm_skinny_kernel<MT_, PRO_, INF_, 8><<<grid, 512, 0, s_>>>(a);                \
        else gemm_skinny_kernel<MT_, PRO_, INF_, 16><<<grid, 1024, 0, s_>>>(a);                              \
    } while (0)

}  // namespace egpt

using namespace egpt;

// out_f32 != null: float32 [n_splits][m][n] partial sums (bias only allowed with n_splits == 1).
// out_bf16 != null: bfloat16 [m][n], n_splits must be 1.
extern "C" int egpt_gemm_skinny(const void* x, const void* w, const void* bias, float* out_f32, void* out_bf16,
                                void* acc_fixed, int m, int n, int k, int n_splits, int waves, void* stream) {
    const int n_outs = (out_f32 ? 1 : 0) + (out_bf16 ? 1 : 0) + (acc_fixed ? 1 : 0);
    if (!x || !w || n_outs != 1 || m <= 0 || n <= 0 || k <= 0 || n_splits <= 0 ||
        (waves != 4 && waves != 8 && waves != 16))
        return EGPT_BAD_ARGUMENT;
    if (m > 64 || (k % 8) != 0 || (acc_fixed && m > 16)) return EGPT_UNSUPPORTED_SIZE;
    if ((n_splits > 1 && (bias || out_bf16)) || (acc_fixed && bias)) return EGPT_BAD_ARGUMENT;
    SkinnyArgs a = {};
    if (int e = check_splits(k, n_splits, &a.steps_per_split)) return e;
    a.x = static_cast<const bf16_t*>(x);
    a.w = static_cast<const bf16_t*>(w);
    a.bias = static_cast<const bf16_t*>(bias);
    a.out_f32 = out_f32;
    a.out_bf16 = static_cast<bf16_t*>(out_bf16);
    a.acc_fixed = static_cast<fixed_t*>(acc_fixed);
    a.m = m; a.n = n; a.k = k;
    if (waves != 16 && m > 16 && a.steps_per_split <= kResidentSteps && n >= 4096 && !acc_fixed) {
        // many columns, more than one tile of rows, a k range that fits in LDS: x resident, one round of loads
        const dim3 grid = skinny_grid(n, n_splits, waves);
        hipStream_t s_ = static_cast<hipStream_t>(stream);
        const int mt = (m + 15) / 16;
        if (waves == 4) {
            if (mt == 2) gemm_resident_kernel<2, 4><<<grid, 256, 0, s_>>>(a);
            else if (mt == 3) gemm_resident_kernel<3, 4><<<grid, 256, 0, s_>>>(a);
            else gemm_resident_kernel<4, 4><<<grid, 256, 0, s_>>>(a);
        } else {
            if (mt == 2) gemm_resident_kernel<2, 8><<<grid, 512, 0, s_>>>(a);
            else if (mt == 3) gemm_resident_kernel<3, 8><<<grid, 512, 0, s_>>>(a);
            else gemm_resident_kernel<4, 8><<<grid, 512, 0, s_>>>(a);
        }
        EGPT_CHECK_LAUNCH();
        return EGPT_OK;
    }
    switch ((m + 15) / 16) {
        case 1: EGPT_SKINNY(1, kPlain, 8); break;
        case 2: EGPT_SKINNY(2, kPlain, 8); break;
        case 3: EGPT_SKINNY(3, kPlain, 8); break;
        default: EGPT_SKINNY(4, kPlain, 8); break;
    }
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

// out[split][m][n] = partial sums of ((h_in + sum delta) * norm_w) w^T; h_out = h_in + sum delta;
// ss_out[split][m] = sums of squares of h_out over the split's k range.  m <= 16, k % 8 == 0.
extern "C" int egpt_gemm_skinny_norm(const void* h_in, int h_fixed, float* h_out, const float* delta, int delta_splits,
                                     const void* norm_w, const void* w, float* out, float* ss_out, int m, int n, int k,
                                     int n_splits, int waves, void* stream) {
    if (!h_in || !norm_w || !w || !out || !ss_out || m <= 0 || n <= 0 || k <= 0 ||
        delta_splits < 0 || (delta && delta_splits == 0) || (waves != 4 && waves != 8 && waves != 16))
        return EGPT_BAD_ARGUMENT;
    if (h_fixed ? (delta != nullptr) : (!h_out || h_in == h_out)) return EGPT_BAD_ARGUMENT;
    if (m > 16 || (k % 8) != 0) return EGPT_UNSUPPORTED_SIZE;
    SkinnyArgs a = {};
    if (int e = check_splits(k, n_splits, &a.steps_per_split)) return e;
    a.w = static_cast<const bf16_t*>(w);
    a.out_f32 = out;
    a.m = m; a.n = n; a.k = k;
    if (h_fixed) a.h_in_fixed = static_cast<const fixed_t*>(h_in);
    else a.h_in = static_cast<const float*>(h_in);
    a.h_out = h_out; a.delta = delta; a.delta_splits = delta ? delta_splits : 0;
    a.norm_w = static_cast<const bf16_t*>(norm_w);
    a.ss_out = ss_out;
    // Many partial sums to add and few workgroups (which then need not share a CU): more loads in flight.
    // As many loads in flight as there are partial sums to add, if registers allow: few workgroups need not
    // share a CU.
    const dim3 g = skinny_grid(n, n_splits, waves);
    if (a.delta_splits <= 4)
        EGPT_SKINNY(1, kNorm, 4);
    else if (a.delta_splits > 8 && g.x * g.y <= 512 && waves == 4)
        EGPT_SKINNY(1, kNorm, 20);
    else
        EGPT_SKINNY(1, kNorm, 8);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

// out[split][m][n] = partial sums of swiglu(inv_rms * sum gate_up) w^T, gate_up [gu_splits][m][2k];
// inv_rms[m] = 1 / sqrt(sum_s ss_in[s][m] / hidden + eps), or 1 if ss_in is null.
extern "C" int egpt_gemm_skinny_swiglu(const float* gate_up, int gu_splits, const float* ss_in, int ss_splits,
                                       int hidden, float eps, const void* w, float* out, void* acc_fixed, int m, int n,
                                       int k, int n_splits, int waves, void* stream) {
    if (!gate_up || gu_splits < 1 || !w || (!out == !acc_fixed) || m <= 0 || n <= 0 || k <= 0 || (ss_in && (ss_splits < 1 || hidden < 1)) ||
        (waves != 4 && waves != 8 && waves != 16))
        return EGPT_BAD_ARGUMENT;
    if (m > 16 || (k % 8) != 0) return EGPT_UNSUPPORTED_SIZE;
    SkinnyArgs a = {};
    if (int e = check_splits(k, n_splits, &a.steps_per_split)) return e;
    a.w = static_cast<const bf16_t*>(w);
    a.out_f32 = out;
    a.acc_fixed = static_cast<fixed_t*>(acc_fixed);
    a.m = m; a.n = n; a.k = k;
    a.gu = gate_up; a.gu_splits = gu_splits; a.ss_in = ss_in; a.ss_splits = ss_splits;
    a.inv_hidden = ss_in ? 1.0f / static_cast<float>(hidden) : 0.f;
    a.eps = eps;
    EGPT_SKINNY(1, kSwiglu, 8);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

// out[split][m][n] = partial sums of (combined attention output) w^T; part_o [a_splits][m*nq][hd] unnormalised
// partial outputs, part_ml [a_splits][m*nq][2] their (maximum, sum); k = nq * hd.
extern "C" int egpt_gemm_skinny_attn(const float* part_o, const float* part_ml, int a_splits, int nq, int hd,
                                     const void* w, float* out, void* acc_fixed, int m, int n, int n_splits, int waves,
                                     void* stream) {
    if (!part_o || !part_ml || a_splits < 1 || nq < 1 || hd < 1 || !w || (!out == !acc_fixed) || m <= 0 || n <= 0 ||
        (waves != 4 && waves != 8 && waves != 16))
        return EGPT_BAD_ARGUMENT;
    const int k = nq * hd;
    if (m > 16 || (hd % 8) != 0 || a_splits > kMaxAttnSplits) return EGPT_UNSUPPORTED_SIZE;
    SkinnyArgs a = {};
    if (int e = check_splits(k, n_splits, &a.steps_per_split)) return e;
    if ((a.steps_per_split * kStep + hd - 1) / hd + 1 > kMaxLocalHeads) return EGPT_UNSUPPORTED_SIZE;
    a.w = static_cast<const bf16_t*>(w);
    a.out_f32 = out;
    a.acc_fixed = static_cast<fixed_t*>(acc_fixed);
    a.m = m; a.n = n; a.k = k;
    a.part_o = part_o; a.part_ml = part_ml; a.a_splits = a_splits; a.nq = nq; a.hd = hd;
    EGPT_SKINNY(1, kAttn, 8);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
