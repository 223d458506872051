// Sampling from float32 logits on the device: argmax, and temperature / top-k / top-p sampling.
//
// The reference samples from probabilities on the host (/root/reference/src/sampler.cpp:39-105):
// p^(1/T) (== softmax(logits / T) after normalisation), keep the k most likely, then the smallest
// set of most likely tokens whose normalised mass reaches top_p, then one uniform draw over the
// kept mass.  Here the kept set is found without sorting, by bisection on the weight threshold
// (32 passes over the row, which stays in cache), and the draw walks the kept weights in index order.
#include "api.h"
#include "common.h"

namespace egpt {

constexpr int kSampleThreads = 1024;

// lowest index among equal maxima (/root/reference/src/sampler.cpp:13-20: std::max_element)
__device__ __forceinline__ void argmax_combine(float& v, int& i, float ov, int oi) {
    if (ov > v || (ov == v && oi < i)) {
        v = ov;
        i = oi;
    }
}

__device__ int block_argmax(const float* __restrict__ row, int vocab, float* s_val, int* s_idx) {
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int j = threadIdx.x; j < vocab; j += blockDim.x) {
        const float v = row[j];
        if (v > best) {          // strictly greater keeps the lowest index of this thread's stride
            best = v;
            best_i = j;
        }
    }
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, kWave);
        const int oi = __shfl_xor(best_i, o, kWave);
        argmax_combine(best, best_i, ov, oi);
    }
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) {
        s_val[wave] = best;
        s_idx[wave] = best_i;
    }
    __syncthreads();
    const int n_waves = (blockDim.x + kWave - 1) / kWave;
    best = s_val[0];
    best_i = s_idx[0];
    for (int w = 1; w < n_waves; ++w) argmax_combine(best, best_i, s_val[w], s_idx[w]);
    return best_i == 0x7fffffff ? 0 : best_i;
}

__global__ __launch_bounds__(kSampleThreads) void argmax_kernel(const float* __restrict__ logits,
                                                                int32_t* __restrict__ out, int vocab) {
    __shared__ float s_val[16];
    __shared__ int s_idx[16];
    const int r = blockIdx.x;
    const int best = block_argmax(logits + static_cast<size_t>(r) * vocab, vocab, s_val, s_idx);
    if (threadIdx.x == 0) out[r] = best;
}

// Two stages for wide vocabularies: workgroup (row, c) finds the maximum of its piece of the row, then one
// workgroup per row picks among the pieces (lowest index among equal maxima in both stages).
constexpr int kArgmaxPieces = 32;

__global__ __launch_bounds__(256) void argmax_pieces_kernel(const float* __restrict__ logits,
                                                            float* __restrict__ piece_val,
                                                            int32_t* __restrict__ piece_idx, int vocab) {
    __shared__ float s_val[16];
    __shared__ int s_idx[16];
    const int r = blockIdx.x, c = blockIdx.y;
    const int piece = (vocab + kArgmaxPieces - 1) / kArgmaxPieces;
    const int begin = min(vocab, c * piece), n = min(vocab, begin + piece) - begin;
    int best = 0;
    float val = -INFINITY;
    if (n > 0) {
        const float* row = logits + static_cast<size_t>(r) * vocab + begin;
        best = block_argmax(row, n, s_val, s_idx);
        val = row[best];
    }
    if (threadIdx.x == 0) {
        piece_val[r * kArgmaxPieces + c] = val;
        piece_idx[r * kArgmaxPieces + c] = begin + best;
    }
}

__global__ __launch_bounds__(64) void argmax_pick_kernel(const float* __restrict__ piece_val,
                                                         const int32_t* __restrict__ piece_idx,
                                                         int32_t* __restrict__ out) {
    const int r = blockIdx.x, lane = threadIdx.x;
    float v = lane < kArgmaxPieces ? piece_val[r * kArgmaxPieces + lane] : -INFINITY;
    int i = lane < kArgmaxPieces ? piece_idx[r * kArgmaxPieces + lane] : 0x7fffffff;
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, kWave);
        const int oi = __shfl_xor(i, o, kWave);
        argmax_combine(v, i, ov, oi);
    }
    if (lane == 0) out[r] = i;
}

// weight of token j: exp((x_j - max) / T), in (0, 1]
__device__ __forceinline__ float weight_of(float x, float mx, float inv_t) { return expf((x - mx) * inv_t); }

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const float* __restrict__ uniform, int32_t* __restrict__ out, int vocab) {
    __shared__ float s_val[16];
    __shared__ int s_idx[16];
    __shared__ float s_scan[kSampleThreads];
    const int r = blockIdx.x;
    const float* row = logits + static_cast<size_t>(r) * vocab;
    const float temp = temperature[r];
    const int best = block_argmax(row, vocab, s_val, s_idx);
    if (!(temp > 0.f)) {  // greedy, as the reference for temperature <= 0 (sampler.cpp:46-49)
        if (threadIdx.x == 0) out[r] = best;
        return;
    }
    const float mx = row[best];
    const float inv_t = 1.0f / fmaxf(temp, 1e-6f);
    // kept set = { j : w_j >= threshold }; the threshold starts at 0 (everything)
    float threshold = 0.f;
    const int k = top_k[r];
    if (k > 0 && k < vocab) {
        // largest bit pattern tau with count(w >= tau) >= k; positive floats order like their bits
        uint32_t lo = 0u, hi = 0x3f800000u;  // w in (0, 1]
        while (lo < hi) {
            const uint32_t mid = lo + (hi - lo + 1) / 2;
            const float tau = __uint_as_float(mid);
            float cnt = 0.f;
            for (int j = threadIdx.x; j < vocab; j += blockDim.x) cnt += weight_of(row[j], mx, inv_t) >= tau ? 1.f : 0.f;
            cnt = block_sum(cnt, s_val);
            if (cnt >= static_cast<float>(k)) lo = mid; else hi = mid - 1;
        }
        threshold = __uint_as_float(lo);
    }
    float kept = 0.f;
    for (int j = threadIdx.x; j < vocab; j += blockDim.x) {
        const float w = weight_of(row[j], mx, inv_t);
        kept += w >= threshold ? w : 0.f;
    }
    kept = block_sum(kept, s_val);
    const float p = top_p[r];
    if (p > 0.f && p < 1.f) {
        // largest tau with mass(w >= tau) >= p * kept: the smallest set of most likely tokens reaching p
        uint32_t lo = __float_as_uint(threshold), hi = 0x3f800000u;
        const float need = p * kept;
        while (lo < hi) {
            const uint32_t mid = lo + (hi - lo + 1) / 2;
            const float tau = __uint_as_float(mid);
            float mass = 0.f;
            for (int j = threadIdx.x; j < vocab; j += blockDim.x) {
                const float w = weight_of(row[j], mx, inv_t);
                mass += w >= tau ? w : 0.f;
            }
            mass = block_sum(mass, s_val);
            if (mass >= need) lo = mid; else hi = mid - 1;
        }
        threshold = fmaxf(threshold, __uint_as_float(lo));
    }
    // inverse CDF in index order: every thread owns a contiguous piece of the row
    const int chunk = (vocab + blockDim.x - 1) / blockDim.x;
    const int begin = min(vocab, static_cast<int>(threadIdx.x) * chunk), end = min(vocab, begin + chunk);
    float mine = 0.f;
    for (int j = begin; j < end; ++j) {
        const float w = weight_of(row[j], mx, inv_t);
        mine += w >= threshold ? w : 0.f;
    }
    s_scan[threadIdx.x] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int i = 0; i < blockDim.x; ++i) total += s_scan[i];
        float u = uniform[r];
        u = fminf(fmaxf(u, 0.f), 0.99999994f);
        const float target = u * total;
        float cum = 0.f;
        int owner = -1;
        for (int i = 0; i < blockDim.x; ++i) {
            if (s_scan[i] > 0.f) {
                owner = i;                      // last piece with mass catches rounding at the end
                if (cum + s_scan[i] > target) break;
            }
            cum += s_scan[i];
        }
        int pick = best;
        if (owner >= 0) {
            // cum must be the mass before `owner`
            cum = 0.f;
            for (int i = 0; i < owner; ++i) cum += s_scan[i];
            const int b0 = min(vocab, owner * chunk), e0 = min(vocab, b0 + chunk);
            for (int j = b0; j < e0; ++j) {
                const float w = weight_of(row[j], mx, inv_t);
                if (w >= threshold) {
                    pick = j;
                    cum += w;
                    if (cum > target) break;
                }
            }
        }
        out[r] = pick;
    }
}

}  // namespace egpt

using namespace egpt;

// scratch: room for n_rows * 32 floats and n_rows * 32 int32 (used for wide vocabularies), or null.
extern "C" int egpt_argmax(const float* logits, int32_t* out, void* scratch, int n_rows, int vocab, void* stream) {
    if (!logits || !out || n_rows < 0 || vocab <= 0) return EGPT_BAD_ARGUMENT;
    if (n_rows == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (scratch && vocab >= 8192) {
        float* pv = static_cast<float*>(scratch);
        int32_t* pi = reinterpret_cast<int32_t*>(pv + static_cast<size_t>(n_rows) * kArgmaxPieces);
        argmax_pieces_kernel<<<dim3(n_rows, kArgmaxPieces), 256, 0, s>>>(logits, pv, pi, vocab);
        EGPT_CHECK_LAUNCH();
        argmax_pick_kernel<<<n_rows, kWave, 0, s>>>(pv, pi, out);
    } else {
        argmax_kernel<<<n_rows, kSampleThreads, 0, s>>>(logits, out, vocab);
    }
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_sample(const float* logits, const float* temperature, const int32_t* top_k, const float* top_p,
                           const float* uniform, int32_t* out, int n_rows, int vocab, void* stream) {
    if (!logits || !temperature || !top_k || !top_p || !uniform || !out || n_rows < 0 || vocab <= 0)
        return EGPT_BAD_ARGUMENT;
    if (n_rows == 0) return EGPT_OK;
    sample_kernel<<<n_rows, kSampleThreads, 0, static_cast<hipStream_t>(stream)>>>(logits, temperature, top_k,
                                                                                   top_p, uniform, out, vocab);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
