// Sampling from float32 logits on the device: argmax, and temperature / top-k / top-p sampling.
//
// The reference samples from probabilities on the host (/root/reference/src/sampler.cpp:39-105):
// p^(1/T) (== softmax(logits / T) after normalisation), keep the k most likely, then the smallest
// set of most likely tokens whose normalised mass reaches top_p, then one uniform draw over the
// kept mass.  Here the kept set is found without sorting, by radix selection on the bit patterns of the
// weights (four passes of eight bits over the row, which stays in cache; masses are added in fixed point so
// that no decision depends on the order of additions), and the draw walks the kept weights in index order.
#include <mutex>

#include "api.h"
#include "common.h"

namespace egpt {

constexpr int kSampleThreads = 1024;

// Calls f(index, value) for every element of p[0..n) once, spread over the workgroup's threads (thread `tid` of
// `n_threads`).  The body reads 16 bytes per thread and keeps eight such loads in flight: a pass over a row is a
// chain of dependent loads otherwise, and its time is their latency, not the row's size.
template <typename F>
__device__ __forceinline__ void for_each_in_row(const float* __restrict__ p, int n, int tid, int n_threads, F f) {
    const int head = min(n, static_cast<int>((4u - ((reinterpret_cast<uintptr_t>(p) >> 2) & 3u)) & 3u));
    for (int j = tid; j < head; j += n_threads) f(j, p[j]);
    const float4* p4 = reinterpret_cast<const float4*>(p + head);
    const int n4 = (n - head) / 4;
    // eight loads issued before the first value is used (the compiler does not do this by itself across calls of f
    // that hold ballots or atomic additions)
    constexpr int kAhead = 8;
    int i = tid;
    for (; i + (kAhead - 1) * n_threads < n4; i += kAhead * n_threads) {
        float4 v[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) v[u] = p4[i + u * n_threads];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int j = head + 4 * (i + u * n_threads);
            f(j, v[u].x);
            f(j + 1, v[u].y);
            f(j + 2, v[u].z);
            f(j + 3, v[u].w);
        }
    }
    for (; i < n4; i += n_threads) {
        const float4 v = p4[i];
        const int j = head + 4 * i;
        f(j, v.x);
        f(j + 1, v.y);
        f(j + 2, v.z);
        f(j + 3, v.w);
    }
    for (int j = head + 4 * n4 + tid; j < n; j += n_threads) f(j, p[j]);
}

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
    for_each_in_row(row, vocab, threadIdx.x, blockDim.x, [&](int j, float v) {
        if (v > best || (v == best && j < best_i)) {
            best = v;
            best_i = j;
        }
    });
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

// weight of token j: exp((x_j - max) / T), in [0, 1]
__device__ __forceinline__ float weight_of(float x, float mx, float inv_t) { return expf((x - mx) * inv_t); }

// Fixed-point image of a weight in [0, 1] (40 fractional bits): sums of these are integers, so a sum over the
// row does not depend on the order in which threads add, and neither does any decision taken from it.
__device__ __forceinline__ unsigned long long fixed_of(float w) {
    return static_cast<unsigned long long>(static_cast<double>(w) * 1099511627776.0);
}

// The largest bit pattern tau with count(w >= tau) >= need (non-negative floats order like their bits): radix
// selection, eight bits a level, histogram in LDS.  The weights of a row crowd into a few exponents, so the
// lanes of a wavefront that hit the same bin first agree on one addition (a ballot and a population count).
__device__ uint32_t select_by_count(const float* __restrict__ w, int vocab, unsigned int need, unsigned int* hist,
                                    uint32_t* shared_prefix, unsigned int* shared_need) {
    uint32_t prefix = 0u, mask = 0u;
    const int lane = threadIdx.x % kWave;
    int first_level = 3;
    {
        // The highest digit of a weight's pattern is its exponent (two exponents a bin), and the k-th largest
        // weight is almost always within 2^-16 of the largest (1.0, digit 0x3f): count those eight bins in
        // registers.  If the k-th weight is smaller still, the general histogram below takes over.
        unsigned int c[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
        for_each_in_row(w, vocab, threadIdx.x, blockDim.x, [&](int, float wj) {
            const uint32_t bits = __float_as_uint(wj);
            if (bits >= 0x38000000u) {
                const uint32_t d = 0x3fu - (bits >> 24);
#pragma unroll
                for (int i = 0; i < 8; ++i) c[i] += d == static_cast<uint32_t>(i) ? 1u : 0u;
            }
        });
        for (int i = threadIdx.x; i < 8; i += blockDim.x) hist[i] = 0u;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            unsigned int v = c[i];
#pragma unroll
            for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
            if (lane == 0 && v) atomicAdd(&hist[i], v);          // integer sums: order does not matter
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned int cum = 0u;
            int found = -1;
            for (int i = 0; i < 8; ++i) {
                if (cum + hist[i] >= need) {
                    found = i;
                    break;
                }
                cum += hist[i];
            }
            *shared_prefix = found >= 0 ? (0x3fu - found) << 24 : 0xffffffffu;
            *shared_need = found >= 0 ? need - cum : need;
        }
        __syncthreads();
        if (*shared_prefix != 0xffffffffu) {
            prefix = *shared_prefix;
            need = *shared_need;
            mask = 255u << 24;
            first_level = 2;
        }
        __syncthreads();
    }
    for (int level = first_level; level >= 0; --level) {
        const int shift = 8 * level;
        for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0u;
        __syncthreads();
        for_each_in_row(w, vocab, threadIdx.x, blockDim.x, [&](int, float wj) {
            const uint32_t bits = __float_as_uint(wj);
            const uint32_t bin = (bits & mask) == prefix ? (bits >> shift) & 255u : 0xffffffffu;
            unsigned long long todo = __ballot(bin != 0xffffffffu);      // over the lanes that are here
            while (todo) {
                const int leader = __ffsll(static_cast<long long>(todo)) - 1;
                const uint32_t b0 = __shfl(bin, leader, kWave);
                const unsigned long long same = __ballot(bin == b0);
                if (lane == leader) atomicAdd(&hist[b0], static_cast<unsigned int>(__popcll(same)));
                todo &= ~same;
            }
        });
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned int cum = 0u;
            int bin = 255;
            for (; bin > 0; --bin) {
                if (cum + hist[bin] >= need) break;
                cum += hist[bin];
            }
            *shared_prefix = prefix | (static_cast<uint32_t>(bin) << shift);
            *shared_need = need - cum;
        }
        __syncthreads();
        prefix = *shared_prefix;
        need = *shared_need;
        mask |= 255u << shift;
        __syncthreads();
    }
    return prefix;
}

// Among the weights >= floor_bits, the largest bit pattern tau with mass(w >= tau) >= need: the smallest set of
// most likely tokens whose mass reaches need, ties at tau included whole.  Sixteen-way search on the bit
// pattern: each pass sums, per thread and then over the workgroup in a fixed order, the fixed-point mass at or
// above fifteen pivots; about eight passes.
__device__ uint32_t select_by_mass(const float* __restrict__ w, int vocab, uint32_t floor_bits, unsigned long long need,
                                   unsigned long long* wave_sums /* [16][15] */, uint32_t* shared_lo,
                                   uint32_t* shared_hi, unsigned long long* shared_above) {
    uint32_t lo = floor_bits, hi = 0x3f800001u;      // mass(w >= lo) >= need, mass(w >= hi) < need
    unsigned long long above = 0ull;                 // mass(w >= hi), known from the pass that set hi
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, n_waves = blockDim.x / kWave;
    while (hi - lo > 1u) {
        // the first pass puts its pivots on exponent boundaries near 1.0, where the mass is; later passes
        // divide [lo, hi) evenly
        const bool first = hi == 0x3f800001u && lo < 0x38000000u;
        const uint32_t step = first ? 0x01000000u : (hi - lo + 15u) / 16u;
        const uint32_t base = first ? 0x37000000u : lo;               // pivot i = base + (i + 1) * step
        unsigned long long acc[15];
#pragma unroll
        for (int i = 0; i < 15; ++i) acc[i] = 0ull;
        for_each_in_row(w, vocab, threadIdx.x, blockDim.x, [&](int, float wj) {
            const uint32_t bits = __float_as_uint(wj);
            if (bits > base && bits < hi && bits >= floor_bits) {     // only these can lie at or above a pivot
                const unsigned long long f = fixed_of(wj);
#pragma unroll
                for (int i = 0; i < 15; ++i) acc[i] += bits >= base + (i + 1) * step ? f : 0ull;
            }
        });
#pragma unroll
        for (int i = 0; i < 15; ++i) {
            unsigned long long v = acc[i];
#pragma unroll
            for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
            if (lane == 0) wave_sums[wave * 15 + i] = v;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            uint32_t new_lo = lo, new_hi = hi;
            unsigned long long new_above = above;
            for (int i = 0; i < 15; ++i) {
                const uint32_t pivot = base + (i + 1) * step;
                if (pivot >= hi) break;
                if (pivot <= lo) continue;
                unsigned long long mass = above;
                for (int wv = 0; wv < n_waves; ++wv) mass += wave_sums[wv * 15 + i];
                if (mass >= need) {
                    new_lo = pivot;
                } else {
                    new_hi = pivot;
                    new_above = mass;
                    break;
                }
            }
            *shared_lo = new_lo;
            *shared_hi = new_hi;
            *shared_above = new_above;
        }
        __syncthreads();
        lo = *shared_lo;
        hi = *shared_hi;
        above = *shared_above;
        __syncthreads();
    }
    return lo;
}

// ---- wide vocabularies: the row-wide work spread over many workgroups, the selection on what is left of the row
//
// The selection below walks its row a dozen times with one workgroup, which for 150,000 tokens is 300 us whatever the
// number of rows.  For a wide vocabulary three small kernels with kSamplePieces workgroups per row come first: they
// count the weights by exponent (those within 2^-16 of the largest, which hold the top-k tokens and the top-p mass of
// any distribution that is not nearly flat), decide below which exponent no token can be kept, and write the tokens at
// or above it, in index order, into a list of candidates.  The selection then runs on that list: one thread per
// candidate when they are at most kSampleThreads (the usual case), the row-walking selection otherwise.  A row for
// which neither cut is asked gets no list: the pieces' masses say in which piece the drawn point lies, and that
// piece alone is walked.
constexpr int kSamplePieces = 32;
constexpr int kTopBins = 16;            // exponents 127 (weight 1.0) down to 112, one bin each; bin kTopBins: the rest

__device__ __forceinline__ int top_bin_of(uint32_t bits) {           // bits of a weight in [0, 1]
    const int e = static_cast<int>(bits >> 23);
    return e >= 128 - kTopBins ? 127 - e : kTopBins;
}

// piece_count / piece_mass [rows][kSamplePieces][kTopBins + 1]: per piece of the row, how many weights each bin holds
// and their mass in fixed point
__global__ __launch_bounds__(256) void sample_hist_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                          const int32_t* __restrict__ best, unsigned int* __restrict__ piece_count,
                                                          unsigned long long* __restrict__ piece_mass, int vocab) {
    __shared__ unsigned int s_count[kTopBins + 1];
    __shared__ unsigned long long s_mass[kTopBins + 1];
    const int r = blockIdx.x, c = blockIdx.y;
    const float temp = temperature[r];
    if (!(temp > 0.f)) return;
    const float* row = logits + static_cast<size_t>(r) * vocab;
    const float mx = row[best[r]];
    const float inv_t = 1.0f / fmaxf(temp, 1e-6f);
    const int piece = (vocab + kSamplePieces - 1) / kSamplePieces;
    const int begin = min(vocab, c * piece), n = min(vocab, begin + piece) - begin;
    for (int i = threadIdx.x; i <= kTopBins; i += blockDim.x) {
        s_count[i] = 0u;
        s_mass[i] = 0ull;
    }
    __syncthreads();
    // Nearly every weight lies below the top bins and is summed in registers; the few above go to the bins in LDS
    // (integer additions: the order does not matter).
    unsigned int rest_count = 0u;
    unsigned long long rest_mass = 0ull;
    for_each_in_row(row + begin, n, threadIdx.x, blockDim.x, [&](int, float x) {
        const float w = weight_of(x, mx, inv_t);
        const int bin = top_bin_of(__float_as_uint(w));
        const unsigned long long f = fixed_of(w);
        if (bin == kTopBins) {
            rest_count += 1u;
            rest_mass += f;
        } else {
            atomicAdd(&s_count[bin], 1u);
            atomicAdd(&s_mass[bin], f);
        }
    });
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
        rest_count += __shfl_xor(rest_count, o, kWave);
        rest_mass += __shfl_xor(rest_mass, o, kWave);
    }
    if (threadIdx.x % kWave == 0 && rest_count) {
        atomicAdd(&s_count[kTopBins], rest_count);
        atomicAdd(&s_mass[kTopBins], rest_mass);
    }
    __syncthreads();
    const size_t base = (static_cast<size_t>(r) * kSamplePieces + c) * (kTopBins + 1);
    for (int i = threadIdx.x; i <= kTopBins; i += blockDim.x) {
        piece_count[base + i] = s_count[i];
        piece_mass[base + i] = s_mass[i];
    }
}

// cutoff[r]: bit pattern below which no weight of row r can be kept; offsets[r][0..kSamplePieces]: where each piece's
// candidates start in the row's list (the last entry is their number)
__global__ __launch_bounds__(64) void sample_plan_kernel(const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
                                                         const float* __restrict__ top_p,
                                                         const unsigned int* __restrict__ piece_count,
                                                         const unsigned long long* __restrict__ piece_mass,
                                                         uint32_t* __restrict__ cutoff, int32_t* __restrict__ offsets,
                                                         unsigned long long* __restrict__ row_mass,
                                                         const float* __restrict__ uniform, int32_t* __restrict__ direct_piece,
                                                         unsigned long long* __restrict__ direct_target, int vocab) {
    __shared__ unsigned int s_count[kTopBins + 1];
    __shared__ unsigned long long s_mass[kTopBins + 1];
    __shared__ int s_bin;
    const int r = blockIdx.x, t = threadIdx.x;
    if (!(temperature[r] > 0.f)) {
        if (t == 0) direct_piece[r] = -1;
        return;
    }
    const size_t base = static_cast<size_t>(r) * kSamplePieces * (kTopBins + 1);
    {
        // Neither cut is asked for: the draw needs no selection.  The pieces' masses are known, so the drawn point
        // (in fixed point, of the whole row's mass) names its piece and what is left of it inside that piece; the
        // last kernel walks that piece alone.  No list of candidates is made for such a row.
        const int k = top_k[r];
        const float p = top_p[r];
        if (!(k > 0 && k < vocab) && !(p > 0.f && p < 1.f)) {
            unsigned long long mine = 0ull;
            if (t < kSamplePieces)
                for (int i = 0; i <= kTopBins; ++i) mine += piece_mass[base + t * (kTopBins + 1) + i];
            unsigned long long incl = mine;
#pragma unroll
            for (int o = 1; o < kWave; o <<= 1) {
                const unsigned long long up = __shfl_up(incl, o, kWave);
                if (t >= o) incl += up;
            }
            const unsigned long long total = __shfl(incl, kSamplePieces - 1, kWave);
            const float u = fminf(fmaxf(uniform[r], 0.f), 0.99999994f);
            unsigned long long target = static_cast<unsigned long long>(static_cast<double>(u) * static_cast<double>(total));
            if (total > 0ull && target >= total) target = total - 1ull;
            const bool here = t < kSamplePieces && incl > target && incl - mine <= target;   // at most one piece
            const unsigned long long holders = __ballot(here);
            const int piece = holders ? __ffsll(static_cast<long long>(holders)) - 1 : 0;      // (an empty row: piece 0)
            const unsigned long long inside = __shfl(target - (incl - mine), piece, kWave);
            if (t < kSamplePieces) offsets[r * (kSamplePieces + 1) + t] = 0;
            if (t == 0) {
                direct_piece[r] = piece;
                direct_target[r] = holders ? inside : 0ull;
                offsets[r * (kSamplePieces + 1) + kSamplePieces] = 0;
                cutoff[r] = 0xffffffffu;
                row_mass[r] = total;
            }
            return;
        }
    }
    if (t <= kTopBins) {
        unsigned int cv = 0u;
        unsigned long long mv = 0ull;
        for (int c = 0; c < kSamplePieces; ++c) {
            cv += piece_count[base + c * (kTopBins + 1) + t];
            mv += piece_mass[base + c * (kTopBins + 1) + t];
        }
        s_count[t] = cv;
        s_mass[t] = mv;
    }
    __syncthreads();
    if (t == 0) {
        // the last bin whose tokens can be kept (kTopBins: every token can)
        const int k = top_k[r];
        const float p = top_p[r];
        int last = kTopBins;
        if (k > 0 && k < vocab) {                    // the k-th largest weight lies in this bin; top-p only removes more
            unsigned int cum = 0u;
            for (int i = 0; i <= kTopBins; ++i) {
                cum += s_count[i];
                if (cum >= static_cast<unsigned int>(k)) {
                    last = i;
                    break;
                }
            }
        } else if (p > 0.f && p < 1.f) {             // the mass p of the whole row is reached within this bin
            unsigned long long total = 0ull;
            for (int i = 0; i <= kTopBins; ++i) total += s_mass[i];
            unsigned long long need = static_cast<unsigned long long>(static_cast<double>(p) * static_cast<double>(total));
            if (need == 0ull) need = 1ull;
            unsigned long long cum = 0ull;
            for (int i = 0; i <= kTopBins; ++i) {
                cum += s_mass[i];
                if (cum >= need) {
                    last = i;
                    break;
                }
            }
        }
        s_bin = last;
        direct_piece[r] = -1;
        cutoff[r] = last >= kTopBins ? 0u : static_cast<uint32_t>(127 - last) << 23;
        unsigned long long all = 0ull;
        for (int i = 0; i <= kTopBins; ++i) all += s_mass[i];
        row_mass[r] = all;                           // the mass of the whole row: what top-p without top-k refers to
    }
    __syncthreads();
    // where each piece's candidates start: thread c counts piece c, a prefix sum over the wavefront does the rest
    const int last = s_bin;
    int mine = 0;
    if (t < kSamplePieces) {
        unsigned int v[kTopBins + 1];
#pragma unroll
        for (int i = 0; i <= kTopBins; ++i) v[i] = piece_count[base + t * (kTopBins + 1) + i];
#pragma unroll
        for (int i = 0; i <= kTopBins; ++i) mine += i <= last ? static_cast<int>(v[i]) : 0;
    }
    int incl = mine;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const int up = __shfl_up(incl, o, kWave);
        if (t >= o) incl += up;
    }
    if (t < kSamplePieces) offsets[r * (kSamplePieces + 1) + t] = incl - mine;
    if (t == kSamplePieces - 1) offsets[r * (kSamplePieces + 1) + kSamplePieces] = incl;
}

// the candidates of a piece, in index order: cand_w / cand_idx [rows][vocab]
__global__ __launch_bounds__(256) void sample_compact_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                             const int32_t* __restrict__ best, const uint32_t* __restrict__ cutoff,
                                                             const int32_t* __restrict__ offsets, float* __restrict__ cand_w,
                                                             int32_t* __restrict__ cand_idx,
                                                             const int32_t* __restrict__ direct_piece, int vocab) {
    __shared__ int s_wave[4];
    const int r = blockIdx.x, c = blockIdx.y;
    const float temp = temperature[r];
    if (!(temp > 0.f) || direct_piece[r] >= 0) return;
    const float* row = logits + static_cast<size_t>(r) * vocab;
    const float mx = row[best[r]];
    const float inv_t = 1.0f / fmaxf(temp, 1e-6f);
    const uint32_t cut = cutoff[r];
    const int piece = (vocab + kSamplePieces - 1) / kSamplePieces;
    const int begin = min(vocab, c * piece), end = min(vocab, begin + piece);
    float* ow = cand_w + static_cast<size_t>(r) * vocab;
    int32_t* oi = cand_idx + static_cast<size_t>(r) * vocab;
    int at = offsets[r * (kSamplePieces + 1) + c];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    // 256 tokens at a time, token j by thread j: the order of the list is the order of the tokens
    for (int j0 = begin; j0 < end; j0 += 256) {
        const int j = j0 + threadIdx.x;
        float w = 0.f;
        bool keep = false;
        if (j < end) {
            w = weight_of(row[j], mx, inv_t);
            keep = __float_as_uint(w) >= cut;
        }
        const unsigned long long mask = __ballot(keep);
        const int before = __popcll(mask & ((1ull << lane) - 1ull));
        if (lane == 0) s_wave[wave] = __popcll(mask);
        __syncthreads();
        int wave_base = 0, total = 0;
        for (int i = 0; i < 4; ++i) {
            wave_base += i < wave ? s_wave[i] : 0;
            total += s_wave[i];
        }
        if (keep) {
            ow[at + wave_base + before] = w;
            oi[at + wave_base + before] = j;
        }
        at += total;
        __syncthreads();
    }
}

// The selection and the draw for a list of at most kSampleThreads weights, one thread each (a list of candidates is
// usually a few dozen tokens, and the passes of the general selection cost their barriers, not their data).
// Token j is among the k most likely iff fewer than k weights are greater than its own, and within the mass `need`
// iff the mass of the greater weights is below it: the same sets as the thresholds of select_by_count and
// select_by_mass (ties whole).  Counts and fixed-point masses are integers, so nothing depends on an order; the
// draw walks the kept weights in index order.  Returns the picked position in the list or -1 (every thread).
__device__ int pick_from_short_list(const float* __restrict__ w, int n, bool cut_by_count, unsigned int k, float p,
                                    bool mass_of_row, unsigned long long row_mass, float u, float* s_list /* [kSampleThreads] */,
                                    unsigned long long* s_wave /* [16] */, float* s_piece /* [16] */, int* s_pick /* [2] */) {
    const int j = threadIdx.x, lane = j % kWave, wave = j / kWave, n_waves = blockDim.x / kWave;
    const float wj = j < n ? w[j] : 0.f;
    s_list[j] = wj;                                   // slots past n hold 0: never greater than a weight
    if (j < 2) s_pick[j] = j == 0 ? 0x7fffffff : -1;
    __syncthreads();
    unsigned int above = 0u;
    unsigned long long mass_above = 0ull;
    const int n4 = (n + 3) / 4;
    for (int i = 0; i < n4; ++i) {                    // every thread reads the same address: a broadcast
        const float4 v = reinterpret_cast<const float4*>(s_list)[i];
        above += (v.x > wj) + (v.y > wj) + (v.z > wj) + (v.w > wj);
        mass_above += (v.x > wj ? fixed_of(v.x) : 0ull) + (v.y > wj ? fixed_of(v.y) : 0ull) +
                      (v.z > wj ? fixed_of(v.z) : 0ull) + (v.w > wj ? fixed_of(v.w) : 0ull);
    }
    bool keep = j < n && (!cut_by_count || above < k);
    if (p > 0.f && p < 1.f) {
        unsigned long long mine = keep ? fixed_of(wj) : 0ull;
#pragma unroll
        for (int o = kWave / 2; o > 0; o >>= 1) mine += __shfl_xor(mine, o, kWave);
        if (lane == 0) s_wave[wave] = mine;
        __syncthreads();
        unsigned long long kept = 0ull;
        for (int i = 0; i < n_waves; ++i) kept += s_wave[i];
        if (mass_of_row) kept = row_mass;
        unsigned long long need = static_cast<unsigned long long>(static_cast<double>(p) * static_cast<double>(kept));
        if (need == 0ull) need = 1ull;
        keep = keep && mass_above < need;
    }
    // inverse CDF in index order: prefix sums inside the wavefronts, then over them
    const float mine = keep ? wj : 0.f;
    float incl = mine;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const float up = __shfl_up(incl, o, kWave);
        if (lane >= o) incl += up;
    }
    if (lane == kWave - 1) s_piece[wave] = incl;
    __syncthreads();
    float before = 0.f, total = 0.f;
    for (int i = 0; i < n_waves; ++i) {
        before += i < wave ? s_piece[i] : 0.f;
        total += s_piece[i];
    }
    const float target = fminf(fmaxf(u, 0.f), 0.99999994f) * total;
    if (keep && before + incl > target) atomicMin(&s_pick[0], j);
    if (keep) atomicMax(&s_pick[1], j);               // the last kept token catches rounding at the end
    __syncthreads();
    return s_pick[0] != 0x7fffffff ? s_pick[0] : s_pick[1];
}

// The draw inside one piece of a row (tokens [begin, begin + n)) for a row without cuts: `target` is the drawn point
// in the fixed-point mass of the piece.  Every thread takes a run of consecutive tokens, the runs' masses are summed
// up over the workgroup in index order, and the thread whose run holds the point finds the token.  The weights
// are computed as the counting kernel computed them, so the masses are the same integers.  Returns the token or
// -1 (every thread).
__device__ int pick_in_piece(const float* __restrict__ row, int begin, int n, float mx, float inv_t, unsigned long long target,
                             unsigned long long* s_wave /* [16] */, int* s_pick /* [1] */) {
    const int j = threadIdx.x, lane = j % kWave, wave = j / kWave, n_waves = blockDim.x / kWave;
    const int run = (n + static_cast<int>(blockDim.x) - 1) / static_cast<int>(blockDim.x);
    const int r_begin = min(n, j * run), r_end = min(n, r_begin + run);
    unsigned long long mine = 0ull;
    for (int i = r_begin; i < r_end; ++i) mine += fixed_of(weight_of(row[begin + i], mx, inv_t));
    unsigned long long incl = mine;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const unsigned long long up = __shfl_up(incl, o, kWave);
        if (lane >= o) incl += up;
    }
    if (lane == kWave - 1) s_wave[wave] = incl;
    if (j == 0) s_pick[0] = -1;
    __syncthreads();
    unsigned long long before = 0ull;
    for (int i = 0; i < wave; ++i) before += s_wave[i];
    const unsigned long long excl = before + incl - mine;
    if (mine > 0ull && excl <= target && target < excl + mine) {
        unsigned long long cum = excl;
        for (int i = r_begin; i < r_end; ++i) {
            cum += fixed_of(weight_of(row[begin + i], mx, inv_t));
            if (cum > target) {
                s_pick[0] = begin + i;
                break;
            }
        }
    }
    __syncthreads();
    return s_pick[0];
}

// One workgroup per row.  `weights` is scratch [rows][vocab] float32: the weights are computed once and the
// selection passes read them back (from cache).  With a list of candidates (cand_idx != null) `weights` holds the
// candidates' weights, cand_count[r * cand_stride] their number, and `best` the row's argmax.
__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const float* __restrict__ uniform, int32_t* __restrict__ out,
    float* __restrict__ weights, int vocab, const int32_t* __restrict__ cand_idx, const int32_t* __restrict__ cand_count,
    int cand_stride, const int32_t* __restrict__ best_in, const unsigned long long* __restrict__ row_mass,
    const int32_t* __restrict__ direct_piece, const unsigned long long* __restrict__ direct_target) {
    __shared__ float s_val[16];
    __shared__ int s_idx[16];
    __shared__ unsigned int hist[256];
    __shared__ unsigned long long s_wave[16 * 15];
    __shared__ unsigned int s_need;
    __shared__ uint32_t s_a, s_b;
    __shared__ unsigned long long s_above;
    __shared__ float s_piece[16];
    __shared__ int s_owner;
    __shared__ float s_before;
    __shared__ __attribute__((aligned(16))) float s_list[kSampleThreads];
    __shared__ int s_pick[2];
    const int r = blockIdx.x;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, n_waves = blockDim.x / kWave;
    const float* row = logits + static_cast<size_t>(r) * vocab;
    float* w = weights + static_cast<size_t>(r) * vocab;
    const int32_t* idx_of = cand_idx ? cand_idx + static_cast<size_t>(r) * vocab : nullptr;
    const float temp = temperature[r];
    const int best = cand_idx ? best_in[r] : block_argmax(row, vocab, s_val, s_idx);
    if (!(temp > 0.f)) {  // greedy, as the reference for temperature <= 0 (sampler.cpp:46-49)
        if (threadIdx.x == 0) out[r] = best;
        return;
    }
    const int full_vocab = vocab;
    if (cand_idx && direct_piece[r] >= 0) {          // no cuts: the drawn point's piece is known, walk it
        const int piece = (vocab + kSamplePieces - 1) / kSamplePieces;
        const int begin = min(vocab, direct_piece[r] * piece), n = min(vocab, begin + piece) - begin;
        const int at = pick_in_piece(row, begin, n, row[best], 1.0f / fmaxf(temp, 1e-6f), direct_target[r], s_wave, s_pick);
        if (threadIdx.x == 0) out[r] = at < 0 ? best : at;
        return;
    }
    if (cand_idx) {
        vocab = cand_count[r * cand_stride];         // from here on the row is the list of candidates
    } else {
        const float mx = row[best];
        const float inv_t = 1.0f / fmaxf(temp, 1e-6f);
        for_each_in_row(row, vocab, threadIdx.x, blockDim.x, [&](int j, float x) { w[j] = weight_of(x, mx, inv_t); });
        __syncthreads();   // each thread reads back what others wrote: same workgroup, so a barrier suffices
    }
    const int k = top_k[r];
    const bool k_active = k > 0 && k < full_vocab;
    if (vocab <= kSampleThreads) {                   // a short row or list: one thread per token
        const int at = pick_from_short_list(w, vocab, k_active && k < vocab, static_cast<unsigned int>(k), top_p[r],
                                            cand_idx && !k_active, cand_idx ? row_mass[r] : 0ull, uniform[r], s_list,
                                            s_wave, s_piece, s_pick);
        if (threadIdx.x == 0) out[r] = at < 0 ? best : (idx_of ? idx_of[at] : at);
        return;
    }
    // kept set = { j : w_j >= threshold }; the threshold starts at 0 (everything)
    uint32_t threshold = 0u;
    if (k_active && k < vocab)        // (a list of exactly k candidates is the top k)
        threshold = select_by_count(w, vocab, static_cast<unsigned int>(k), hist, &s_a, &s_need);
    const float p = top_p[r];
    if (p > 0.f && p < 1.f) {
        // mass of what top-k kept, in fixed point: per-thread sums, then over the wavefronts in order
        unsigned long long mine = 0ull;
        for_each_in_row(w, vocab, threadIdx.x, blockDim.x, [&](int, float wj) {
            if (__float_as_uint(wj) >= threshold) mine += fixed_of(wj);
        });
#pragma unroll
        for (int o = kWave / 2; o > 0; o >>= 1) mine += __shfl_xor(mine, o, kWave);
        if (lane == 0) s_wave[wave] = mine;
        __syncthreads();
        unsigned long long kept = 0ull;
        for (int i = 0; i < n_waves; ++i) kept += s_wave[i];
        __syncthreads();
        // (a list of candidates without top-k holds only the upper part of the row: the mass p refers to the whole row)
        if (cand_idx && !k_active) kept = row_mass[r];
        unsigned long long need = static_cast<unsigned long long>(static_cast<double>(p) * static_cast<double>(kept));
        if (need == 0ull) need = 1ull;
        threshold = select_by_mass(w, vocab, threshold, need, s_wave, &s_a, &s_b, &s_above);
    }
    // inverse CDF in index order.  Every wavefront owns a contiguous piece of the row; the piece that holds the
    // drawn point is then walked 64 tokens at a time with a prefix sum over the lanes.
    const int piece = ((vocab + n_waves - 1) / n_waves + kWave - 1) / kWave * kWave;
    const int p_begin = min(vocab, wave * piece), p_end = min(vocab, p_begin + piece);
    float mine = 0.f;
    for_each_in_row(w + p_begin, p_end - p_begin, lane, kWave, [&](int, float wj) {
        mine += __float_as_uint(wj) >= threshold ? wj : 0.f;
    });
    mine = wave_sum(mine);
    if (lane == 0) s_piece[wave] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int i = 0; i < n_waves; ++i) total += s_piece[i];
        const float u = fminf(fmaxf(uniform[r], 0.f), 0.99999994f);
        const float target = u * total;
        float cum = 0.f;
        int owner = -1;
        float before = 0.f;
        for (int i = 0; i < n_waves; ++i) {
            if (s_piece[i] > 0.f) {
                owner = i;                      // the last piece with mass catches rounding at the end
                before = cum;
                if (cum + s_piece[i] > target) break;
            }
            cum += s_piece[i];
        }
        s_owner = owner;
        s_before = target - before;             // what is left of the target inside the owner's piece
        if (owner < 0) out[r] = best;
    }
    __syncthreads();
    if (wave == s_owner) {
        const float target = s_before;
        float cum = 0.f;
        int pick = -1, last_kept = -1;
        for (int base = p_begin; base < p_end && pick < 0; base += kWave) {
            const int j = base + lane;
            float wj = 0.f;
            if (j < p_end) {
                const float v = w[j];
                wj = __float_as_uint(v) >= threshold ? v : 0.f;
            }
            float incl = wj;                     // inclusive prefix sum over the lanes
#pragma unroll
            for (int o = 1; o < kWave; o <<= 1) {
                const float up = __shfl_up(incl, o, kWave);
                if (lane >= o) incl += up;
            }
            const unsigned long long kept_mask = __ballot(wj > 0.f);
            const unsigned long long hit = __ballot(wj > 0.f && cum + incl > target);
            if (kept_mask) last_kept = base + 63 - __clzll(static_cast<long long>(kept_mask));
            if (hit) pick = base + __ffsll(static_cast<long long>(hit)) - 1;
            cum += __shfl(incl, kWave - 1, kWave);
        }
        if (lane == 0) {
            const int at = pick >= 0 ? pick : last_kept;
            out[r] = at < 0 ? best : (idx_of ? idx_of[at] : at);
        }
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

// ---- the same search without a workspace argument and without any allocation: the pieces live in the library's
// device image.  In host code `argmax_static_scratch` is only a stand-in for the symbol: the memory's address on
// a device comes from hipGetSymbolAddress with that device current, and every GPU has its own copy.
static __device__ __align__(256) unsigned char argmax_static_scratch[EGPT_ARGMAX_STATIC_MAX_ROWS * kArgmaxPieces * 8];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
void* g_static_ptr[kMaxDevices] = {};

// The buffer's address on the current device, resolved once per device; null on failure.
void* static_scratch_of_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_ptr[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(argmax_static_scratch)) != hipSuccess) return nullptr;
        g_static_ptr[dev] = ptr;
    }
    return g_static_ptr[dev];
}
}  // namespace

extern "C" int egpt_argmax_static_init(void) {
    return static_scratch_of_current_device() ? EGPT_OK : EGPT_STATIC_SCRATCH_UNRESOLVED;
}

extern "C" int egpt_argmax_static(const float* logits, int32_t* out, int n_rows, int vocab, void* stream) {
    if (!logits || !out || n_rows < 0 || vocab <= 0) return EGPT_BAD_ARGUMENT;
    if (n_rows > EGPT_ARGMAX_STATIC_MAX_ROWS) return EGPT_STATIC_SCRATCH_TOO_SMALL;
    if (n_rows == 0) return EGPT_OK;
    void* scratch = static_scratch_of_current_device();
    if (!scratch) return EGPT_STATIC_SCRATCH_UNRESOLVED;
    return egpt_argmax(logits, out, scratch, n_rows, vocab, stream);
}

// weights: scratch for n_rows * vocab floats.
extern "C" int egpt_sample(const float* logits, const float* temperature, const int32_t* top_k, const float* top_p,
                           const float* uniform, int32_t* out, float* weights, int n_rows, int vocab, void* stream) {
    if (!logits || !temperature || !top_k || !top_p || !uniform || !out || !weights || n_rows < 0 || vocab <= 0)
        return EGPT_BAD_ARGUMENT;
    if (n_rows == 0) return EGPT_OK;
    sample_kernel<<<n_rows, kSampleThreads, 0, static_cast<hipStream_t>(stream)>>>(
        logits, temperature, top_k, top_p, uniform, out, weights, vocab, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

// The same for wide vocabularies, in stages (argmax, counts by exponent, the plan, the list of candidates, the
// selection on the list).  workspace: egpt_sample_workspace(n_rows, vocab) bytes of device memory.
static size_t align256(size_t n) { return (n + 255) / 256 * 256; }

extern "C" size_t egpt_sample_workspace(int n_rows, int vocab) {
    const size_t r = static_cast<size_t>(n_rows > 0 ? n_rows : 0), v = static_cast<size_t>(vocab > 0 ? vocab : 0);
    return align256(r * v * 4) * 2                                         // candidates: weights, indices
           + align256(r * kSamplePieces * (kTopBins + 1) * 8)            // masses
           + align256(r * kSamplePieces * (kTopBins + 1) * 4)            // counts
           + align256(r * (kSamplePieces + 1) * 4) + align256(r * 4) * 2   // offsets, cutoff, best
           + align256(r * 8) * 2 + align256(r * 4)                         // mass of the row; the direct draw's point, piece
           + align256(r * kArgmaxPieces * 8);                              // argmax pieces
}

extern "C" int egpt_sample_wide(const float* logits, const float* temperature, const int32_t* top_k, const float* top_p,
                                const float* uniform, int32_t* out, void* workspace, int n_rows, int vocab, void* stream) {
    if (!logits || !temperature || !top_k || !top_p || !uniform || !out || !workspace || n_rows < 0 || vocab <= 0)
        return EGPT_BAD_ARGUMENT;
    if (n_rows == 0) return EGPT_OK;
    if (n_rows > 65535) return EGPT_UNSUPPORTED_SIZE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t r = static_cast<size_t>(n_rows), v = static_cast<size_t>(vocab);
    char* p = static_cast<char*>(workspace);
    float* cand_w = reinterpret_cast<float*>(p);                               p += align256(r * v * 4);
    int32_t* cand_idx = reinterpret_cast<int32_t*>(p);                         p += align256(r * v * 4);
    unsigned long long* piece_mass = reinterpret_cast<unsigned long long*>(p); p += align256(r * kSamplePieces * (kTopBins + 1) * 8);
    unsigned int* piece_count = reinterpret_cast<unsigned int*>(p);            p += align256(r * kSamplePieces * (kTopBins + 1) * 4);
    int32_t* offsets = reinterpret_cast<int32_t*>(p);                          p += align256(r * (kSamplePieces + 1) * 4);
    uint32_t* cutoff = reinterpret_cast<uint32_t*>(p);                         p += align256(r * 4);
    int32_t* best = reinterpret_cast<int32_t*>(p);                             p += align256(r * 4);
    unsigned long long* row_mass = reinterpret_cast<unsigned long long*>(p);   p += align256(r * 8);
    unsigned long long* direct_target = reinterpret_cast<unsigned long long*>(p); p += align256(r * 8);
    int32_t* direct_piece = reinterpret_cast<int32_t*>(p);                     p += align256(r * 4);
    float* pv = reinterpret_cast<float*>(p);
    int32_t* pi = reinterpret_cast<int32_t*>(pv + r * kArgmaxPieces);
    argmax_pieces_kernel<<<dim3(n_rows, kArgmaxPieces), 256, 0, s>>>(logits, pv, pi, vocab);
    EGPT_CHECK_LAUNCH();
    argmax_pick_kernel<<<n_rows, kWave, 0, s>>>(pv, pi, best);
    EGPT_CHECK_LAUNCH();
    sample_hist_kernel<<<dim3(n_rows, kSamplePieces), 256, 0, s>>>(logits, temperature, best, piece_count, piece_mass, vocab);
    EGPT_CHECK_LAUNCH();
    sample_plan_kernel<<<n_rows, 64, 0, s>>>(temperature, top_k, top_p, piece_count, piece_mass, cutoff, offsets, row_mass,
                                             uniform, direct_piece, direct_target, vocab);
    EGPT_CHECK_LAUNCH();
    sample_compact_kernel<<<dim3(n_rows, kSamplePieces), 256, 0, s>>>(logits, temperature, best, cutoff, offsets, cand_w,
                                                                      cand_idx, direct_piece, vocab);
    EGPT_CHECK_LAUNCH();
    sample_kernel<<<n_rows, kSampleThreads, 0, s>>>(logits, temperature, top_k, top_p, uniform, out, cand_w, vocab, cand_idx,
                                                    offsets + kSamplePieces, kSamplePieces + 1, best, row_mass,
                                                    direct_piece, direct_target);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
