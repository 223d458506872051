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
// every magnitude of 2^-8 and above and is rounded to one below; the stream holds magnitudes below 2^31.
typedef long long fixed_t;
constexpr float kFixedOne = 4294967296.0f;
__device__ __forceinline__ fixed_t to_fixed(float v) { return __float2ll_rn(v * kFixedOne); }
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

// Timestamps from inside kernels, for builds with -DEGPT_TRACE only (an ordinary build has none of this).
// EGPT_MARK(base, kernel, phase): the first thread of a workgroup stores the wall clock (units of 10 ns) of `phase`
// (0 to 3) into record `base + workgroup` of a buffer that the host attached with
// egpt_trace_attach_<file>(buffer, capacity); a launcher takes `base` for its grid from egpt_trace_take, so a
// captured graph's nodes keep their records over replays.  A decode step is a chain of short dependent kernels;
// what a link's time is made of (launch, the first load's way from memory, arithmetic, the tail) shows only
// from inside.  A record is five words: (kernel << 48 | workgroup), then the four phases' clocks.
#ifdef EGPT_TRACE
extern "C" unsigned egpt_trace_take(unsigned n_workgroups);
namespace egpt {
static __device__ unsigned long long* trace_buf = nullptr;
static __device__ unsigned int trace_cap = 0;
__device__ __forceinline__ void trace_mark(unsigned base, unsigned kernel, unsigned phase) {
    __builtin_amdgcn_sched_barrier(0);
    if (threadIdx.x == 0 && trace_buf) {
        const unsigned wg = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        if (base + wg < trace_cap) {
            unsigned long long* rec = trace_buf + static_cast<size_t>(base + wg) * 5;
            if (phase == 0) rec[0] = (static_cast<unsigned long long>(kernel) << 48) | wg;
            // low words of the wall clock (10 ns) and of the shader clock (cycles): the two together give the clock rate
            rec[1 + phase] = (wall_clock64() & 0xffffffffull) | (static_cast<unsigned long long>(clock64()) << 32);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
}
}  // namespace egpt
#define EGPT_MARK(base, kernel, phase) egpt::trace_mark(base, kernel, phase)
#define EGPT_TRACE_TAKE(grid) egpt_trace_take((grid).x * (grid).y * (grid).z)
#define EGPT_TRACE_ATTACH(file)                                                                          \
    extern "C" int egpt_trace_attach_##file(void* buf, unsigned cap) {                                   \
        if (hipMemcpyToSymbol(HIP_SYMBOL(egpt::trace_buf), &buf, sizeof(buf)) != hipSuccess) return 1;   \
        if (hipMemcpyToSymbol(HIP_SYMBOL(egpt::trace_cap), &cap, sizeof(cap)) != hipSuccess) return 1;   \
        return 0;                                                                                        \
    }
#else
#define EGPT_MARK(base, kernel, phase) do {} while (0)
#define EGPT_TRACE_TAKE(grid) 0u
#define EGPT_TRACE_ATTACH(file)
#endif

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
