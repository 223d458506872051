// Shared device helpers for the gfx950 kernels: element types, conversions, reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace egpt {

constexpr int kWave = 64;  // CDNA wavefront width

// bfloat16 as raw bits; arithmetic is always done in float.
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(static_cast<uint32_t>(v.bits) << 16); }

// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return bf16_t{f32_to_bf16_bits(v)}; }

// The QKV epilogue's arithmetic, spelled out operation by operation: several kernels do it (one by one, four
// pairs at a time, inside the decode attention) and must leave the same bits, which they would not if the
// compiler were free to contract each one's multiplications and additions in its own way.
__device__ __forceinline__ float scale_then_bias(float x, float scale, float bias) { return __fmaf_rn(x, scale, bias); }
__device__ __forceinline__ float inv_rms(float ss, float inv_hidden, float eps) {
    return 1.0f / sqrtf(__fmaf_rn(ss, inv_hidden, eps));
}
__device__ __forceinline__ void rotate_pair(float a, float b, float c, float s, float& ra, float& rb) {
    ra = __fmaf_rn(a, c, -__fmul_rn(b, s));
    rb = __fmaf_rn(a, s, __fmul_rn(b, c));
}

// The residual stream of steps of few tokens in 64-bit fixed point (units of 2^-32).  Several workgroups that split
// a product's k range add their partial results straight into it with integer atomics: integer addition does not
// care for the order, so the sum is the same bits whatever the scheduling, and the kernels that read the stream
// read one small tensor instead of every workgroup's partial sums.  A float32 value times 2^32 is an integer for
// every magnitude of 2^-8 and above and is rounded to one below (an absolute error of at most 2^-33, whatever the
// other values of the stream are); the stream holds magnitudes below 2^31.  What does not fit is not hidden as
// a small number: a magnitude of 2^31 or more, an infinity or a NaN enters as the largest magnitude of its sign
// (NaN: the negative one), which the norm behind it turns into a row of zeros and one entry of +-sqrt(width) - a
// step of more than 16 rows, and the float32 path, keep such values in float32 and show them as they are.
typedef long long fixed_t;
constexpr float kFixedOne = 4294967296.0f;
constexpr float kFixedLimit = 2147483648.0f;          // 2^31
__device__ __forceinline__ fixed_t to_fixed(float v) {
    if (!(fabsf(v) < kFixedLimit)) return v > 0.f ? 0x7fffffffffffffffLL : -0x7fffffffffffffffLL - 1;
    return __float2ll_rn(v * kFixedOne);
}
__device__ __forceinline__ float fixed_to_float(fixed_t v) { return __ll2float_rn(v) * (1.0f / kFixedOne); }
__device__ __forceinline__ void fixed_add(fixed_t* p, float v) {
    atomicAdd(reinterpret_cast<unsigned long long*>(p), static_cast<unsigned long long>(to_fixed(v)));
}
// what a residual stream of either kind is read and written as
__device__ __forceinline__ float residual_load(const float* p) { return *p; }
__device__ __forceinline__ float residual_load(const fixed_t* p) { return fixed_to_float(*p); }
__device__ __forceinline__ void residual_store(float* p, float v) { *p = v; }
__device__ __forceinline__ void residual_store(fixed_t* p, float v) { *p = to_fixed(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `scratch` holds >= 16 floats.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int n_waves = (blockDim.x + kWave - 1) / kWave;
    v = wave_sum(v);
    __syncthreads();  // scratch may still be read from an earlier call
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < n_waves; ++w) total += scratch[w];
    return total;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int n_waves = (blockDim.x + kWave - 1) / kWave;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float m = scratch[0];
    for (int w = 1; w < n_waves; ++w) m = fmaxf(m, scratch[w]);
    return m;
}

}  // namespace egpt

// Error codes returned by every entry point (0 = launched).
#define EGPT_OK 0
#define EGPT_BAD_ARGUMENT 1
#define EGPT_UNSUPPORTED_SIZE 2
#define EGPT_LAUNCH_FAILED 3
#define EGPT_STATIC_SCRATCH_TOO_SMALL 4
#define EGPT_STATIC_SCRATCH_UNRESOLVED 5

#define EGPT_CHECK_LAUNCH()                                   \
    do {                                                      \
        hipError_t e_ = hipGetLastError();                    \
        if (e_ != hipSuccess) return EGPT_LAUNCH_FAILED;      \
    } while (0)
