// Softmax attention over the paged cache for a ragged batch: prompt portions and single decoded
// tokens in one launch.
//
// Query i of request b stands at position p = kv_len[b] - q_len[b] + i and reads keys j <= p
// (causal key limit as /root/reference/src/cuda/ops/self_attn_detail.cuh:695-751), and j > p - window
// when a window is set.  score = (q . k) * scale, online softmax with float32 running maximum, sum and
// accumulator (/root/reference/src/cuda/ops/self_attn_detail.cuh:299-383); query head h reads kv head
// h / (nq / nkv) (:669).  Keys lie in pages [page][kv head][offset][hd], values in pages
// [page][kv head][hd][offset], and are found
// through the request's block table; nothing beyond kv_len is ever read, so pages need no clearing.
#include "api.h"
#include "common.h"

namespace egpt {

constexpr int kMaxHeadDim = 256;

__device__ __forceinline__ int find_request(const int32_t* q_start, int n_seqs, int t) {
    int lo = 0, hi = n_seqs - 1;  // last b with q_start[b] <= t
    while (lo < hi) {
        const int mid = (lo + hi + 1) / 2;
        if (q_start[mid] <= t) lo = mid; else hi = mid - 1;
    }
    return lo;
}

// One workgroup of kGenericWaves wavefronts per (token, query head).  Keys are taken 64 at a time, a chunk of 64
// by the wavefront whose number is the chunk's number modulo kGenericWaves: each lane scores one key, the wavefront
// agrees on the new maximum, then each lane owns head features lane, lane+64, ... of the output.  At the end the
// wavefronts' running (maximum, sum, output) are merged in the order of their numbers.  Which wavefront takes which
// keys depends on the keys' positions alone, so a token's result is the same bits however the work was cut into
// steps and whatever else is in the batch.
constexpr int kGenericWaves = 8;

__device__ __forceinline__ void load4f(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
__device__ __forceinline__ void load4f(const bf16_t* p, float* v) {
    const uint2 a = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
    v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
}
// the value that lane `from` (the same for all lanes) holds
__device__ __forceinline__ float from_lane(float v, int from) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), from));
}

template <typename T>
__global__ __launch_bounds__(64 * kGenericWaves) void paged_attention_generic_kernel(
    const T* __restrict__ qkv, T* __restrict__ out, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ kv_len, int n_seqs, int nq, int nkv, int hd,
    int page_size, float scale, int window) {
    constexpr int kMaxOwn = kMaxHeadDim / kWave;
    __shared__ __attribute__((aligned(16))) float q_s[kMaxHeadDim];
    __shared__ float part_ml[kGenericWaves][2];
    __shared__ float part_o[kGenericWaves][kMaxHeadDim];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int b = find_request(q_start, n_seqs, t);
    const int i = t - q_start[b];
    const int p = kv_len[b] - q_len[b] + i;
    const int hi = p + 1;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int kvh = h / (nq / nkv);
    const int row_width = (nq + 2 * nkv) * hd;
    const T* q = qkv + static_cast<size_t>(t) * row_width + h * hd;
    for (int d = threadIdx.x; d < hd; d += kWave * kGenericWaves) q_s[d] = to_float(q[d]);
    __syncthreads();
    const int32_t* table = block_table + static_cast<size_t>(b) * table_width;
    const bool vec4 = hd % 4 == 0 && page_size % 4 == 0;       // rows of keys and of values start at 16 (8) bytes
    float acc[kMaxOwn] = {};
    float m_run = -INFINITY, l_run = 0.f;
    for (int c = lo + wave * kWave; c < hi; c += kWave * kGenericWaves) {
        const int j = c + lane;
        float s = -INFINITY;
        if (j < hi) {
            const long page = table[j / page_size];
            const long head_base = (page * nkv + kvh) * page_size * hd;   // same for keys and values
            const T* kr = k_cache + head_base + (j % page_size) * hd;     // keys: [offset][feature]
            float dot = 0.f;
            if (vec4) {          // the same sum, its operands loaded four at a time
                for (int d = 0; d < hd; d += 4) {
                    float kv[4];
                    load4f(kr + d, kv);
                    const float4 qv = *reinterpret_cast<const float4*>(&q_s[d]);
                    dot = fmaf(qv.x, kv[0], dot);
                    dot = fmaf(qv.y, kv[1], dot);
                    dot = fmaf(qv.z, kv[2], dot);
                    dot = fmaf(qv.w, kv[3], dot);
                }
            } else {
                for (int d = 0; d < hd; ++d) dot = fmaf(q_s[d], to_float(kr[d]), dot);
            }
            s = dot * scale;
        }
        const float m_new = fmaxf(m_run, wave_max(s));   // finite: key c is always visible
        const float pj = j < hi ? expf(s - m_new) : 0.f;
        const float alpha = expf(m_run - m_new);          // exp(-inf) = 0 on the wavefront's first chunk
        l_run = l_run * alpha + wave_sum(pj);
        m_run = m_new;
        const int n_valid = min(kWave, hi - c);
#pragma unroll
        for (int r = 0; r < kMaxOwn; ++r) acc[r] *= alpha;
        // every lane needs every key's weight and place: taken from the lane that holds them.  Four keys that lie
        // side by side in a page are one load per feature (the sum goes on key by key as without it).
        int jj = 0;
        if (vec4 && c % 4 == 0) {
            for (; jj + 4 <= n_valid; jj += 4) {
                const long page = table[(c + jj) / page_size];
                const long vo = (page * nkv + kvh) * page_size * hd + (c + jj) % page_size;
                const float pw[4] = {from_lane(pj, jj), from_lane(pj, jj + 1), from_lane(pj, jj + 2), from_lane(pj, jj + 3)};
#pragma unroll
                for (int r = 0; r < kMaxOwn; ++r) {
                    const int d = lane + r * kWave;
                    if (d < hd) {
                        float vv[4];
                        load4f(v_cache + vo + static_cast<long>(d) * page_size, vv);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[r] = fmaf(pw[e], vv[e], acc[r]);
                    }
                }
            }
        }
        for (; jj < n_valid; ++jj) {
            const float pw = from_lane(pj, jj);
            const long page = table[(c + jj) / page_size];
            const long vo = (page * nkv + kvh) * page_size * hd + (c + jj) % page_size;
#pragma unroll
            for (int r = 0; r < kMaxOwn; ++r) {
                const int d = lane + r * kWave;
                if (d < hd) acc[r] = fmaf(pw, to_float(v_cache[vo + static_cast<long>(d) * page_size]), acc[r]);
            }
        }
    }
    // merge: wavefront 0 holds the first chunk, so the overall maximum is finite; a wavefront without keys has
    // maximum -inf and weight exp(-inf) = 0
    if (lane == 0) {
        part_ml[wave][0] = m_run;
        part_ml[wave][1] = l_run;
    }
#pragma unroll
    for (int r = 0; r < kMaxOwn; ++r) {
        const int d = lane + r * kWave;
        if (d < hd) part_o[wave][d] = acc[r];
    }
    __syncthreads();
    if (wave != 0) return;
    float m_all = -INFINITY;
    for (int w = 0; w < kGenericWaves; ++w) m_all = fmaxf(m_all, part_ml[w][0]);
    float l_all = 0.f;
    for (int w = 0; w < kGenericWaves; ++w) l_all = fmaf(part_ml[w][1], expf(part_ml[w][0] - m_all), l_all);
    const float inv_l = 1.0f / l_all;
    T* o = out + static_cast<size_t>(t) * nq * hd + h * hd;
#pragma unroll
    for (int r = 0; r < kMaxOwn; ++r) {
        const int d = lane + r * kWave;
        if (d < hd) {
            float a = 0.f;
            for (int w = 0; w < kGenericWaves; ++w) a = fmaf(part_o[w][d], expf(part_ml[w][0] - m_all), a);
            o[d] = from_float<T>(a * inv_l);
        }
    }
}

}  // namespace egpt

using namespace egpt;

extern "C" int egpt_paged_attention(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                                    const int32_t* block_table, int table_width, const int32_t* q_start,
                                    const int32_t* q_len, const int32_t* kv_len, int n_seqs, int n_tokens, int nq,
                                    int nkv, int hd, int page_size, float scale, int window, int dtype,
                                    void* stream) {
    if (!qkv || !out || !k_cache || !v_cache || !block_table || !q_start || !q_len || !kv_len)
        return EGPT_BAD_ARGUMENT;
    if (n_seqs <= 0 || n_tokens < 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || hd <= 0 || page_size <= 0 ||
        table_width <= 0 || window < 0)
        return EGPT_BAD_ARGUMENT;
    if (hd > kMaxHeadDim || nq > 65535) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(n_tokens, nq);
    if (dtype == 0)
        paged_attention_generic_kernel<float><<<grid, kWave * kGenericWaves, 0, s>>>(
            static_cast<const float*>(qkv), static_cast<float*>(out), static_cast<const float*>(k_cache),
            static_cast<const float*>(v_cache), block_table, table_width, q_start, q_len, kv_len, n_seqs, nq, nkv,
            hd, page_size, scale, window);
    else if (dtype == 1)
        paged_attention_generic_kernel<bf16_t><<<grid, kWave * kGenericWaves, 0, s>>>(
            static_cast<const bf16_t*>(qkv), static_cast<bf16_t*>(out), static_cast<const bf16_t*>(k_cache),
            static_cast<const bf16_t*>(v_cache), block_table, table_width, q_start, q_len, kv_len, n_seqs, nq, nkv,
            hd, page_size, scale, window);
    else
        return EGPT_BAD_ARGUMENT;
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
