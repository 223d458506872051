// Embedding gather, residual-add + RMSNorm, SwiGLU, and the QKV epilogue
// (bias + rotary position encoding + store of keys and values into cache pages).
#include "api.h"
#include "common.h"

namespace egpt {

// The output of a product arrives either as one tensor of the activation type, or as float32 partial
// sums [n_splits][rows][cols] of a split-k product, which are added here in split order.
template <typename T>
struct ProductView {
    const T* whole;          // used when n_splits == 0
    const float* partial;    // used when n_splits > 0
    int n_splits;
    size_t split_stride;     // rows * cols
    __device__ __forceinline__ bool present() const { return whole != nullptr || partial != nullptr; }
    __device__ __forceinline__ float at(size_t idx) const {
        if (n_splits == 0) return to_float(whole[idx]);
        // up to sixteen loads in flight at a time (a chain of dependent kernels pays for round trips, not
        // bytes); the order of the additions is fixed
        float v = 0.f;
        for (int s0 = 0; s0 < n_splits; s0 += 16) {
            float t[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) t[i] = s0 + i < n_splits ? partial[(s0 + i) * split_stride + idx] : 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) v += t[i];
        }
        return v;
    }
};

// ----------------------------------------------------------------------------- embedding
// x[t, :] = E[id_t, :]   (/root/reference/src/models/embedding.cpp:54-76); output: the residual stream, float32 or
// fixed point.
template <typename T, typename R>
__global__ void embed_kernel(const int32_t* __restrict__ ids, const T* __restrict__ table, R* __restrict__ out,
                             int hidden, int vocab) {
    const int t = blockIdx.x;
    int id = ids[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // ids are range-checked on the host; never read outside
    const T* row = table + static_cast<size_t>(id) * hidden;
    R* o = out + static_cast<size_t>(t) * hidden;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) residual_store(o + j, to_float(row[j]));
}

// ----------------------------------------------------------------------------- add + RMSNorm
// ss = sum x^2 (float32), inv = 1/sqrt(ss/H + eps), y = x * inv * w
// (/root/reference/src/models/norm.cpp:47-59, /root/reference/src/cuda/ops/self_attn_detail.cuh:385-418).
// The residual addition h += delta happens here too, in float32.
template <typename T, typename R, int KEEP>
__global__ void add_rmsnorm_kernel(R* __restrict__ h, ProductView<T> delta,
                                   const int32_t* __restrict__ rows, const T* __restrict__ weight, float eps,
                                   T* __restrict__ out, int hidden) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
    R* hrow = h + src * hidden;
    const bool has_delta = delta.present();
    const size_t dbase = src * hidden;
    const bool write_back = (rows == nullptr) && has_delta;
    // A row of up to KEEP (four or eight) values per thread stays in registers, with its norm weight: all of a
    // thread's loads are issued together, and the sum over the workgroup is the only wait between them and the
    // stores.  (A loop over the row instead waits for memory once per round: 10 us for a row of 3,584 values with 512
    // threads, 7.4 us for one of 5,120 with 1,024 against 6.2 from registers; eight where four are enough cost 0.3 to
    // 0.7 us.)
    if (hidden <= KEEP * static_cast<int>(blockDim.x)) {
        float v[KEEP], w[KEEP];
#pragma unroll
        for (int i = 0; i < KEEP; ++i) {
            const int j = threadIdx.x + i * blockDim.x;
            v[i] = 0.f;
            w[i] = 0.f;
            if (j < hidden) {
                v[i] = residual_load(hrow + j);
                w[i] = to_float(weight[j]);
            }
        }
        if (has_delta) {
#pragma unroll
            for (int i = 0; i < KEEP; ++i) {
                const int j = threadIdx.x + i * blockDim.x;
                if (j < hidden) v[i] += delta.at(dbase + j);
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < KEEP; ++i) {
            const int j = threadIdx.x + i * blockDim.x;
            if (write_back && j < hidden) residual_store(hrow + j, v[i]);
            ss += v[i] * v[i];
        }
        ss = block_sum(ss, scratch);
        const float inv = 1.0f / sqrtf(ss / static_cast<float>(hidden) + eps);
        T* orow = out + static_cast<size_t>(r) * hidden;
#pragma unroll
        for (int i = 0; i < KEEP; ++i) {
            const int j = threadIdx.x + i * blockDim.x;
            if (j < hidden) orow[j] = from_float<T>(v[i] * inv * w[i]);
        }
        return;
    }
    float ss = 0.f;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        float v = residual_load(hrow + j);
        if (has_delta) v += delta.at(dbase + j);
        if (write_back) residual_store(hrow + j, v);
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(hidden) + eps);
    T* orow = out + static_cast<size_t>(r) * hidden;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        float v = residual_load(hrow + j);       // already updated when written back
        if (has_delta && !write_back) v += delta.at(dbase + j);
        orow[j] = from_float<T>(v * inv * to_float(weight[j]));
    }
}

// eight consecutive values, stored as bfloat16 (one 16-byte load) or float32 (two), as floats
__device__ __forceinline__ void load8_as_float(const bf16_t* p, float* v) {
    const uint4 d = *reinterpret_cast<const uint4*>(p);
    v[0] = __uint_as_float(d.x << 16); v[1] = __uint_as_float(d.x & 0xffff0000u);
    v[2] = __uint_as_float(d.y << 16); v[3] = __uint_as_float(d.y & 0xffff0000u);
    v[4] = __uint_as_float(d.z << 16); v[5] = __uint_as_float(d.z & 0xffff0000u);
    v[6] = __uint_as_float(d.w << 16); v[7] = __uint_as_float(d.w & 0xffff0000u);
}
__device__ __forceinline__ void load8_as_float(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// The same for bfloat16 activations with eight features per thread and load (16-byte loads of the
// activations, 32 bytes of the residual stream): the form that prompt portions of many tokens take.
template <typename DT>   // delta as bfloat16, or as float32 (a product that was written out in float32)
__global__ __launch_bounds__(256) void add_rmsnorm_vec8_kernel(float* __restrict__ h, const DT* __restrict__ delta,
                                                               const int32_t* __restrict__ rows,
                                                               const bf16_t* __restrict__ weight, float eps,
                                                               bf16_t* __restrict__ out, int hidden) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
    float* hrow = h + src * hidden;
    const DT* drow = delta ? delta + src * hidden : nullptr;
    const bool write_back = (rows == nullptr) && (delta != nullptr);
    // a row that the workgroup covers in one pass stays in registers for the second pass (one round trip less)
    const bool one_pass = hidden <= static_cast<int>(blockDim.x) * 8;
    float kept[8] = {}, kept_w[8] = {};
    float ss = 0.f;
    for (int j = threadIdx.x * 8; j < hidden; j += blockDim.x * 8) {
        float v[8];
        load8_as_float(hrow + j, v);
        if (one_pass) load8_as_float(weight + j, kept_w);     // with the row's loads, not behind the workgroup's sum
        if (drow) {
            float d[8];
            load8_as_float(drow + j, d);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] += d[i];
            if (write_back) {
                *reinterpret_cast<float4*>(hrow + j) = float4{v[0], v[1], v[2], v[3]};
                *reinterpret_cast<float4*>(hrow + j + 4) = float4{v[4], v[5], v[6], v[7]};
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            ss += v[i] * v[i];
            kept[i] = v[i];
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(hidden) + eps);
    bf16_t* orow = out + static_cast<size_t>(r) * hidden;
    for (int j = threadIdx.x * 8; j < hidden; j += blockDim.x * 8) {
        float v[8], w[8];
        if (one_pass) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v[i] = kept[i];
                w[i] = kept_w[i];
            }
        } else {
            load8_as_float(hrow + j, v);
            if (drow && !write_back) {
                float d[8];
                load8_as_float(drow + j, d);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] += d[i];
            }
            load8_as_float(weight + j, w);
        }
        uint4 o;
        o.x = f32_to_bf16_bits(v[0] * inv * w[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1] * inv * w[1])) << 16);
        o.y = f32_to_bf16_bits(v[2] * inv * w[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3] * inv * w[3])) << 16);
        o.z = f32_to_bf16_bits(v[4] * inv * w[4]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[5] * inv * w[5])) << 16);
        o.w = f32_to_bf16_bits(v[6] * inv * w[6]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[7] * inv * w[7])) << 16);
        *reinterpret_cast<uint4*>(orow + j) = o;
    }
}

// ----------------------------------------------------------------------------- SwiGLU
// out = up * gate / (1 + exp(-gate))   (/root/reference/src/cuda/ops/mlp.cu:152-162); [gate | up] per row.
template <typename T>
__global__ void swiglu_kernel(ProductView<T> gate_up, T* __restrict__ out, int n_tokens, int inter) {
    const size_t total = static_cast<size_t>(n_tokens) * inter;
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
         i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const size_t t = i / inter, j = i % inter;
        const float g = gate_up.at(t * 2 * inter + j);
        const float u = gate_up.at(t * 2 * inter + inter + j);
        out[i] = from_float<T>(u * (g / (1.0f + expf(-g))));
    }
}

// The same from float32 partial sums of a product that still lacks each row's factor 1/rms (a norm folded into
// the product leaves the factor to its consumer): scale = 1/sqrt(sum_s row_ss[s][t] / hidden + eps) multiplies gate and
// up before the activation.  One row of workgroups per token.
template <typename T>
__global__ void swiglu_scaled_kernel(ProductView<float> gate_up, const float* __restrict__ row_ss, int ss_splits,
                                     float inv_hidden, float eps, T* __restrict__ out, int n_tokens, int inter) {
    const size_t t = blockIdx.y;
    float ss = 0.f;
    for (int s = 0; s < ss_splits; ++s) ss += row_ss[static_cast<size_t>(s) * n_tokens + t];
    const float scale = inv_rms(ss, inv_hidden, eps);
    for (int j = blockIdx.x * blockDim.x + threadIdx.x; j < inter; j += gridDim.x * blockDim.x) {
        const float g = scale_then_bias(gate_up.at(t * 2 * inter + j), scale, 0.f);
        const float u = scale_then_bias(gate_up.at(t * 2 * inter + inter + j), scale, 0.f);
        out[t * inter + j] = from_float<T>(u * (g / (1.0f + expf(-g))));
    }
}

// bfloat16, eight features per thread (inter % 8 == 0, one tensor, no partial sums)
template <typename GT>
__global__ __launch_bounds__(256) void swiglu_vec8_kernel(const GT* __restrict__ gate_up, bf16_t* __restrict__ out,
                                                          int n_tokens, int inter) {
    const size_t chunks_per_row = inter / 8;
    const size_t total = static_cast<size_t>(n_tokens) * chunks_per_row;
    for (size_t c = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; c < total;
         c += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const size_t t = c / chunks_per_row, j = (c % chunks_per_row) * 8;
        float g[8], u[8];
        load8_as_float(gate_up + t * 2 * inter + j, g);
        load8_as_float(gate_up + t * 2 * inter + inter + j, u);
        uint32_t ow[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float r0 = u[2 * i] * (g[2 * i] / (1.0f + expf(-g[2 * i])));
            const float r1 = u[2 * i + 1] * (g[2 * i + 1] / (1.0f + expf(-g[2 * i + 1])));
            ow[i] = f32_to_bf16_bits(r0) | (static_cast<uint32_t>(f32_to_bf16_bits(r1)) << 16);
        }
        *reinterpret_cast<uint4*>(out + t * inter + j) = uint4{ow[0], ow[1], ow[2], ow[3]};
    }
}

// ----------------------------------------------------------------------------- QKV epilogue
// For each token: add bias; rotate the first rotary_dim features of every query and key head, pairs
// (i, i + rotary_dim/2), angle = float(position) * inv_freq[i], cos/sin in float32
// (/root/reference/src/ops.cpp:404-420, /root/reference/src/cuda/ops/self_attn_detail.cuh:512-541);
// write the result back in place and store keys and values at their slot of the paged cache
// (keys [page][kv head][offset][hd], values [page][kv head][hd][offset]).
constexpr int kHeadsPerBlock = 2;   // heads of one token that a workgroup of the QKV epilogue handles

template <typename T>
__global__ void qkv_rope_store_kernel(ProductView<T> qkv_in, const float* __restrict__ row_ss, int ss_splits,
                                      float inv_hidden, float eps, T* __restrict__ qkv_out, const T* __restrict__ bias,
                                      const int32_t* __restrict__ positions, const float* __restrict__ inv_freq,
                                      const float* __restrict__ cos_sin, int rotary_dim,
                                      const int32_t* __restrict__ slots, T* __restrict__ k_cache,
                                      T* __restrict__ v_cache, int nq, int nkv, int hd, int page_size) {
    const int t = blockIdx.x;
    const int n_heads = nq + 2 * nkv;
    const int item_begin = blockIdx.y * kHeadsPerBlock * hd;
    const int item_end = min(n_heads * hd, item_begin + kHeadsPerBlock * hd);
    const size_t base = static_cast<size_t>(t) * n_heads * hd;
    T* row = qkv_out + base;
    const float pos = static_cast<float>(positions[t]);
    const int half = rotary_dim / 2;
    // the product may still lack its row's 1/rms factor (sum of squares of the row in row_ss, by split)
    float row_scale = 1.f;
    if (row_ss) {
        float ss = 0.f;
        for (int s0 = 0; s0 < ss_splits; s0 += 16) {
            float part[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) part[i] = s0 + i < ss_splits ? row_ss[(s0 + i) * gridDim.x + t] : 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) ss += part[i];
        }
        row_scale = inv_rms(ss, inv_hidden, eps);
    }
    long slot = slots ? slots[t] : -1;
    const long page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
    for (int item = item_begin + threadIdx.x; item < item_end; item += blockDim.x) {
        const int head = item / hd, d = item % hd;
        const bool rotated = head < nq + nkv && d < rotary_dim;
        if (rotated && d >= half) continue;  // done by its partner
        float a = scale_then_bias(qkv_in.at(base + item), row_scale, bias ? to_float(bias[item]) : 0.f);
        float b = 0.f;
        if (rotated) {
            b = scale_then_bias(qkv_in.at(base + item + half), row_scale, bias ? to_float(bias[item + half]) : 0.f);
            float s, c;
            if (cos_sin) {                       // the step's table of the same values
                c = cos_sin[(static_cast<size_t>(t) * half + d) * 2];
                s = cos_sin[(static_cast<size_t>(t) * half + d) * 2 + 1];
            } else {
                sincosf(pos * inv_freq[d], &s, &c);
            }
            float ra, rb;
            rotate_pair(a, b, c, s, ra, rb);
            a = ra;
            b = rb;
        }
        const T ta = from_float<T>(a), tb = from_float<T>(b);
        row[item] = ta;
        if (rotated) row[item + half] = tb;
        if (slot >= 0 && head >= nq) {
            const bool is_k = head < nq + nkv;
            const int kvh = is_k ? head - nq : head - nq - nkv;
            if (is_k) {   // keys: [page][kv head][offset][feature]
                T* dst = k_cache + ((page * nkv + kvh) * page_size + off) * hd;
                dst[d] = ta;
                if (rotated) dst[d + half] = tb;
            } else {      // values: [page][kv head][feature][offset]
                v_cache[((page * nkv + kvh) * hd + d) * page_size + off] = ta;
            }
        }
    }
}

// cos_sin[t][i] = (cos, sin)(float(positions[t]) * inv_freq[i]): the angles of a step are the same in every
// layer, so they are computed once per step and the layers' kernels read them.
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, const float* __restrict__ inv_freq,
                                  float* __restrict__ cos_sin, int n_tokens, int half) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_tokens * half) return;
    float sn, cs;
    sincosf(static_cast<float>(positions[idx / half]) * inv_freq[idx % half], &sn, &cs);
    cos_sin[2 * static_cast<size_t>(idx)] = cs;
    cos_sin[2 * static_cast<size_t>(idx) + 1] = sn;
}

__device__ __forceinline__ void load4_as_float(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
__device__ __forceinline__ void load4_as_float(const bf16_t* p, float* v) {
    const uint2 a = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
    v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
}

// The same for many tokens (prompt portions) in bfloat16, full rotation (rotary_dim == hd), one tensor in and
// out, angles from the step's table: a thread owns four neighbouring pairs (i, i + hd/2) of one (token, head).
template <typename IN>
__global__ __launch_bounds__(256) void qkv_rope_store_rows_kernel(const IN* __restrict__ qkv_in, bf16_t* __restrict__ qkv_out,
                                                                  const bf16_t* __restrict__ bias,
                                                                  const float* __restrict__ cos_sin,
                                                                  const int32_t* __restrict__ slots,
                                                                  bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
                                                                  int n_tokens, int nq, int nkv, int hd, int page_size) {
    const int half = hd / 2, chunks = half / 4;
    const int n_heads = nq + 2 * nkv;
    const long idx = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= static_cast<long>(n_tokens) * n_heads * chunks) return;
    const int i = static_cast<int>(idx % chunks) * 4;
    const int head = static_cast<int>((idx / chunks) % n_heads);
    const int t = static_cast<int>(idx / (static_cast<long>(chunks) * n_heads));
    const size_t lo = static_cast<size_t>(t) * n_heads * hd + head * hd + i, hi = lo + half;
    float a[4], b[4];
    load4_as_float(qkv_in + lo, a);
    load4_as_float(qkv_in + hi, b);
    if (bias) {
        float ba[4], bb[4];
        load4_as_float(bias + head * hd + i, ba);
        load4_as_float(bias + head * hd + i + half, bb);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a[j] = scale_then_bias(a[j], 1.f, ba[j]);
            b[j] = scale_then_bias(b[j], 1.f, bb[j]);
        }
    }
    const bool is_v = head >= nq + nkv;
    if (!is_v) {
        float cs[8];
        load4_as_float(cos_sin + (static_cast<size_t>(t) * half + i) * 2, cs);
        load4_as_float(cos_sin + (static_cast<size_t>(t) * half + i) * 2 + 4, cs + 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float ra, rb;
            rotate_pair(a[j], b[j], cs[2 * j], cs[2 * j + 1], ra, rb);
            a[j] = ra;
            b[j] = rb;
        }
    }
    uint2 pa, pb;
    pa.x = f32_to_bf16_bits(a[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(a[1])) << 16);
    pa.y = f32_to_bf16_bits(a[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(a[3])) << 16);
    pb.x = f32_to_bf16_bits(b[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(b[1])) << 16);
    pb.y = f32_to_bf16_bits(b[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(b[3])) << 16);
    *reinterpret_cast<uint2*>(qkv_out + lo) = pa;
    *reinterpret_cast<uint2*>(qkv_out + hi) = pb;
    const long slot = (slots && head >= nq) ? slots[t] : -1;
    if (slot >= 0) {
        const long page = slot / page_size, off = slot % page_size;
        if (!is_v) {      // keys: [page][kv head][offset][feature]
            bf16_t* dst = k_cache + ((page * nkv + (head - nq)) * page_size + off) * hd + i;
            *reinterpret_cast<uint2*>(dst) = pa;
            *reinterpret_cast<uint2*>(dst + half) = pb;
        } else {          // values: [page][kv head][feature][offset]
            bf16_t* dst = v_cache + ((page * nkv + (head - nq - nkv)) * hd + i) * page_size + off;
            const uint32_t wa[2] = {pa.x, pa.y}, wb[2] = {pb.x, pb.y};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                dst[static_cast<long>(j) * page_size].bits = static_cast<uint16_t>(wa[j / 2] >> (16 * (j & 1)));
                dst[static_cast<long>(j + half) * page_size].bits = static_cast<uint16_t>(wb[j / 2] >> (16 * (j & 1)));
            }
        }
    }
}

}  // namespace egpt

using namespace egpt;

extern "C" int egpt_embed(const int32_t* ids, const void* table, void* out, int fixed, int n_tokens, int hidden,
                          int vocab, int dtype, void* stream) {
    if (!ids || !table || !out || n_tokens < 0 || hidden <= 0 || vocab <= 0 || (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == 0 && !fixed)
        embed_kernel<<<n_tokens, 256, 0, s>>>(ids, static_cast<const float*>(table), static_cast<float*>(out), hidden, vocab);
    else if (dtype == 0)
        embed_kernel<<<n_tokens, 256, 0, s>>>(ids, static_cast<const float*>(table), static_cast<fixed_t*>(out), hidden, vocab);
    else if (!fixed)
        embed_kernel<<<n_tokens, 256, 0, s>>>(ids, static_cast<const bf16_t*>(table), static_cast<float*>(out), hidden, vocab);
    else
        embed_kernel<<<n_tokens, 256, 0, s>>>(ids, static_cast<const bf16_t*>(table), static_cast<fixed_t*>(out), hidden, vocab);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

template <typename T>
static ProductView<T> make_view(const void* p, int n_splits, size_t split_stride) {
    ProductView<T> v;
    v.whole = n_splits == 0 ? static_cast<const T*>(p) : nullptr;
    v.partial = n_splits > 0 ? static_cast<const float*>(p) : nullptr;
    v.n_splits = n_splits;
    v.split_stride = split_stride;
    return v;
}

extern "C" int egpt_add_rmsnorm(void* h, int fixed, const void* delta, int delta_splits, int delta_rows,
                                const int32_t* rows, const void* weight, float eps, void* out, int n_rows, int hidden,
                                int dtype, void* stream) {
    if (!h || !weight || !out || n_rows < 0 || hidden <= 0 || delta_splits < 0) return EGPT_BAD_ARGUMENT;
    if (delta && delta_rows <= 0) return EGPT_BAD_ARGUMENT;
    if (n_rows == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // few rows with many partial sums each: more threads, so that each has fewer dependent loads to wait for; and
    // enough threads for a row to stay in registers (four values a thread, eight for the widest rows)
    const int threads = (delta_splits > 1 || hidden > 2048) ? 1024 : (hidden > 1024 ? 512 : 256);
    const size_t stride = static_cast<size_t>(delta_rows) * hidden;
    if (dtype == 1 && delta_splits <= 1 && hidden % 8 == 0 && n_rows >= 32 && !fixed) {
        const int threads = hidden >= 2048 ? 256 : 128;
        float* hf = static_cast<float*>(h);
        if (delta_splits == 0)
            add_rmsnorm_vec8_kernel<bf16_t><<<n_rows, threads, 0, s>>>(
                hf, static_cast<const bf16_t*>(delta), rows, static_cast<const bf16_t*>(weight), eps,
                static_cast<bf16_t*>(out), hidden);
        else   // one float32 "partial sum": a product written out in float32
            add_rmsnorm_vec8_kernel<float><<<n_rows, threads, 0, s>>>(
                hf, static_cast<const float*>(delta), rows, static_cast<const bf16_t*>(weight), eps,
                static_cast<bf16_t*>(out), hidden);
        EGPT_CHECK_LAUNCH();
        return EGPT_OK;
    }
    if (dtype != 0 && dtype != 1) return EGPT_BAD_ARGUMENT;
#define EGPT_NORM_KEEP(T_, R_, KEEP_)                                                                      \
    add_rmsnorm_kernel<T_, R_, KEEP_><<<n_rows, threads, 0, s>>>(                                          \
        static_cast<R_*>(h), make_view<T_>(delta, delta_splits, stride), rows, static_cast<const T_*>(weight), eps, \
        static_cast<T_*>(out), hidden)
#define EGPT_NORM(T_, R_)                                        \
    do {                                                         \
        /* (a wide row behind partial sums is faster in the loop: 7.7 against 8.7 us at 64 rows of 5,120) */ \
        if (hidden <= 4 * threads || delta_splits > 1) EGPT_NORM_KEEP(T_, R_, 4);    \
        else EGPT_NORM_KEEP(T_, R_, 8);                          \
    } while (0)
    if (dtype == 0 && !fixed) EGPT_NORM(float, float);
    else if (dtype == 0) EGPT_NORM(float, fixed_t);
    else if (!fixed) EGPT_NORM(bf16_t, float);
    else EGPT_NORM(bf16_t, fixed_t);
#undef EGPT_NORM
#undef EGPT_NORM_KEEP
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_swiglu(const void* gate_up, int n_splits, const float* row_ss, int ss_splits, int hidden, float eps,
                           void* out, int n_tokens, int inter, int dtype, void* stream) {
    if (!gate_up || !out || n_tokens < 0 || inter <= 0 || n_splits < 0) return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t total = static_cast<size_t>(n_tokens) * inter;
    const int blocks = static_cast<int>(total / 256 + 1 > 8192 ? 8192 : total / 256 + 1);
    const size_t stride = total * 2;
    if (row_ss) {
        // float32 partial sums with a pending row factor
        if (n_splits < 1 || ss_splits < 1 || hidden <= 0 || n_tokens > 65535 || (dtype != 0 && dtype != 1))
            return EGPT_BAD_ARGUMENT;
        const dim3 grid(static_cast<unsigned>((inter + 255) / 256 > 64 ? 64 : (inter + 255) / 256),
                        static_cast<unsigned>(n_tokens));
        const ProductView<float> view = make_view<float>(gate_up, n_splits, stride);
        if (dtype == 0)
            swiglu_scaled_kernel<float><<<grid, 256, 0, s>>>(view, row_ss, ss_splits, 1.0f / hidden, eps,
                                                             static_cast<float*>(out), n_tokens, inter);
        else
            swiglu_scaled_kernel<bf16_t><<<grid, 256, 0, s>>>(view, row_ss, ss_splits, 1.0f / hidden, eps,
                                                              static_cast<bf16_t*>(out), n_tokens, inter);
        EGPT_CHECK_LAUNCH();
        return EGPT_OK;
    }
    if (dtype == 1 && n_splits <= 1 && inter % 8 == 0) {
        const size_t chunks = total / 8;
        const int vblocks = static_cast<int>(chunks / 256 + 1 > 16384 ? 16384 : chunks / 256 + 1);
        if (n_splits == 0)
            swiglu_vec8_kernel<bf16_t><<<vblocks, 256, 0, s>>>(static_cast<const bf16_t*>(gate_up),
                                                               static_cast<bf16_t*>(out), n_tokens, inter);
        else
            swiglu_vec8_kernel<float><<<vblocks, 256, 0, s>>>(static_cast<const float*>(gate_up),
                                                              static_cast<bf16_t*>(out), n_tokens, inter);
        EGPT_CHECK_LAUNCH();
        return EGPT_OK;
    }
    if (dtype == 0)
        swiglu_kernel<float><<<blocks, 256, 0, s>>>(make_view<float>(gate_up, n_splits, stride),
                                                    static_cast<float*>(out), n_tokens, inter);
    else if (dtype == 1)
        swiglu_kernel<bf16_t><<<blocks, 256, 0, s>>>(make_view<bf16_t>(gate_up, n_splits, stride),
                                                     static_cast<bf16_t*>(out), n_tokens, inter);
    else
        return EGPT_BAD_ARGUMENT;
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" int egpt_qkv_rope_store(const void* qkv_in, int n_splits, const float* row_ss, int ss_splits, int hidden,
                                   float eps, void* qkv_out, const void* bias,
                                   const int32_t* positions, const float* inv_freq, const float* cos_sin,
                                   int rotary_dim, const int32_t* slots, void* k_cache, void* v_cache, int n_tokens,
                                   int nq, int nkv, int hd, int page_size, int dtype, void* stream) {
    if (!qkv_in || !qkv_out || !positions || n_tokens < 0 || nq <= 0 || nkv <= 0 || hd <= 0 || page_size <= 0 ||
        n_splits < 0)
        return EGPT_BAD_ARGUMENT;
    if (rotary_dim < 0 || rotary_dim > hd || (rotary_dim % 2) != 0 || (rotary_dim > 0 && !inv_freq && !cos_sin))
        return EGPT_BAD_ARGUMENT;
    if (slots && (!k_cache || !v_cache)) return EGPT_BAD_ARGUMENT;
    if (row_ss && (ss_splits < 1 || hidden < 1)) return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const float inv_hidden = row_ss ? 1.0f / static_cast<float>(hidden) : 0.f;
    const size_t stride = static_cast<size_t>(n_tokens) * (nq + 2 * nkv) * hd;
    if (dtype == 1 && n_splits <= 1 && !row_ss && rotary_dim == hd && n_tokens >= 64 && hd % 8 == 0 && cos_sin) {
        // many tokens: one thread per four pairs of a (token, head).  (bfloat16 only: the float32 path keeps
        // one kernel per operation whatever the batch, so that its results do not depend on the batch in any
        // bit.)  The input is bfloat16, or one float32 "partial sum".
        const long items = static_cast<long>(n_tokens) * (nq + 2 * nkv) * (hd / 8);
        const unsigned blocks = static_cast<unsigned>((items + 255) / 256);
        if (n_splits == 0)
            qkv_rope_store_rows_kernel<bf16_t><<<blocks, 256, 0, s>>>(
                static_cast<const bf16_t*>(qkv_in), static_cast<bf16_t*>(qkv_out), static_cast<const bf16_t*>(bias),
                cos_sin, slots, static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), n_tokens, nq, nkv, hd,
                page_size);
        else
            qkv_rope_store_rows_kernel<float><<<blocks, 256, 0, s>>>(
                static_cast<const float*>(qkv_in), static_cast<bf16_t*>(qkv_out), static_cast<const bf16_t*>(bias),
                cos_sin, slots, static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), n_tokens, nq, nkv, hd,
                page_size);
        EGPT_CHECK_LAUNCH();
        return EGPT_OK;
    }
    const dim3 grid(n_tokens, (nq + 2 * nkv + kHeadsPerBlock - 1) / kHeadsPerBlock);
    const int block = kHeadsPerBlock * hd >= 256 ? 256 : (kHeadsPerBlock * hd >= 128 ? 128 : 64);
    if (dtype == 0)
        qkv_rope_store_kernel<float><<<grid, block, 0, s>>>(
            make_view<float>(qkv_in, n_splits, stride), row_ss, ss_splits, inv_hidden, eps,
            static_cast<float*>(qkv_out), static_cast<const float*>(bias),
            positions, inv_freq, cos_sin, rotary_dim, slots, static_cast<float*>(k_cache), static_cast<float*>(v_cache), nq,
            nkv, hd, page_size);
    else if (dtype == 1)
        qkv_rope_store_kernel<bf16_t><<<grid, block, 0, s>>>(
            make_view<bf16_t>(qkv_in, n_splits, stride), row_ss, ss_splits, inv_hidden, eps,
            static_cast<bf16_t*>(qkv_out), static_cast<const bf16_t*>(bias), positions, inv_freq, cos_sin, rotary_dim, slots,
            static_cast<bf16_t*>(k_cache),
            static_cast<bf16_t*>(v_cache), nq, nkv, hd, page_size);
    else
        return EGPT_BAD_ARGUMENT;
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

// cos_sin [n_tokens][half][2] = (cos, sin) of float(positions[t]) * inv_freq[i]
extern "C" int egpt_rope_table(const int32_t* positions, const float* inv_freq, float* cos_sin, int n_tokens, int half,
                               void* stream) {
    if (!positions || !inv_freq || !cos_sin || n_tokens < 0 || half <= 0) return EGPT_BAD_ARGUMENT;
    if (n_tokens == 0) return EGPT_OK;
    const long items = static_cast<long>(n_tokens) * half;
    rope_table_kernel<<<static_cast<unsigned>((items + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(
        positions, inv_freq, cos_sin, n_tokens, half);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

extern "C" const char* egpt_error_string(int code) {
    switch (code) {
        case EGPT_OK: return "ok";
        case EGPT_BAD_ARGUMENT: return "bad argument (null pointer, negative size or unknown dtype)";
        case EGPT_UNSUPPORTED_SIZE: return "size not supported by this kernel";
        case EGPT_LAUNCH_FAILED: return "kernel launch failed";
        case EGPT_STATIC_SCRATCH_TOO_SMALL:
            return "more rows than the library's static scratch buffer holds (egpt_argmax_static takes at most 1024 rows)";
        case EGPT_STATIC_SCRATCH_UNRESOLVED:
            return "the device address of the library's static scratch buffer could not be resolved on the current device";
        default: return "unknown error";
    }
}

extern "C" int egpt_abi_version(void) { return 16; }
