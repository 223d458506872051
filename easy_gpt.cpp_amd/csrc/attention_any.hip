// Paged attention on the matrix cores for every head size that is a multiple of 16 (up to 256), in bfloat16 and in
// true float32: prompt portions and mixed batches (attention_any_tiled_kernel) and batches of single decoded tokens
// (attention_any_decode_kernel + attention_fold_kernel).  The kernels of attention_mfma.hip are tuned for bfloat16
// heads of 64 and 128; these take everything else that the configuration allows.
//
// As there, rows are (token, query head) pairs of one key/value head's group, 16 to a tile, and the scores are
// computed transposed, S^T[key, row] = K[key, :] . Q[row, :], so that a lane holds scores of one row, the row's
// statistics are per-lane scalars and the probabilities are the second product's operand as they lie in registers:
// O^T[feature, row] += V^T[feature, key] . P^T[key, row] (values are stored transposed within a page).
//   bfloat16: v_mfma_f32_16x16x32_bf16, a lane's 16 bytes of an operand are 8 features (or 8 keys);
//   float32:  v_mfma_f32_16x16x4_f32 (float32 operands and accumulation, no reduced precision anywhere), a lane's
//             16 bytes are 4 features (or 4 keys), one instruction each.  A sum over features or keys does not care
//             in which order the matrix cores take them, as long as both operands agree, so a lane's 16 bytes are
//             consecutive elements in memory in both types.
// Every head size has kernels of its own (the size is a template parameter): nothing in a kernel depends on a size
// known only at run time, so the products are straight-line code.  (A product skipped by a branch on the head size,
// right before the accumulators are read, gave results that lacked the last product's part: the wait between a matrix
// instruction and the read of its result was not kept across that branch.)  In bfloat16 a head size that is no
// multiple of 32 has a last piece of features that is half zeros.
//
// Softmax statistics and accumulators are float32 (/root/reference/src/cuda/ops/self_attn_detail.cuh:299-383:
// running maximum, sum and output, one rounding at the end); causal limit and window as in attention.hip.
//
// float32 results are the same bits however the work is cut: keys are taken in chunks of chunk_keys() keys and
// segments of kSegment keys at fixed positions of the sequence; a segment's chunks go through the online softmax in
// ascending order, starting from nothing, and the segments' results are folded into the row's result in ascending
// order by fold_weights / fold_value.  The prompt kernel does that in registers as it walks the keys; the decode
// kernel gives every segment to a wavefront of its own, writes the segments' results out, and the fold kernel folds
// them with the same operations.  A chunk or segment without visible keys changes nothing, exactly, so it does not
// matter whether a kernel walks it.  The same structure serves bfloat16, where only the prompt kernel skips the
// segments (one running result per row).
#include "api.h"
#include "common.h"

namespace egpt {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
// 16 and 8 bytes as native vectors: arrays of these stay in registers across a loop's back edge, which arrays of
// HIP's uint4 structs do not always
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

// keys per segment: a multiple of every chunk size.  Small, so that a batch of a few decoded tokens behind contexts of
// a few thousand keys is hundreds of wavefronts, each with one round of loads (256 keys a segment: 23 us for eight
// requests behind 2,048 float32 keys, four rounds of loads per wavefront)
constexpr int kSegment = 64;

// keys per chunk (one step of the online softmax, and one LDS tile of the prompt kernel): 64, or 32 where two
// stages of 64 keys and their values would not fit into LDS
template <typename T, int HD>
constexpr int chunk_keys() { return HD * sizeof(T) <= 512 ? 64 : 32; }

// acc += A . B for one 16-byte piece of each operand per lane (32 features or keys of bfloat16, 16 of float32)
template <typename T>
__device__ __forceinline__ f32x4 mma_piece(const u32x4& a, const u32x4& b, f32x4 acc) {
    if constexpr (sizeof(T) == 2) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc,
                                                       0, 0, 0);
    } else {
        const f32x4 av = __builtin_bit_cast(f32x4, a), bv = __builtin_bit_cast(f32x4, b);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], bv[i], acc, 0, 0, 0);
        return acc;
    }
}

// One chunk's step of the online softmax for the row of this lane.  acc: the lane's raw scores (q . k, masked ones
// -inf) of NKT tiles of 16 keys; they come back as probabilities exp2((s - m) * scale2).  m_run is in units of the raw
// scores; l_run is this lane's share of the row's sum (the four lanes of a row are added up at the end).  The
// accumulator is rescaled only when some row's maximum moved (a factor of exactly 1 otherwise).
template <int NKT, int DT>
__device__ __forceinline__ void softmax_chunk(f32x4 (&acc)[NKT], float& m_run, float& l_run, f32x4 (&o)[DT], float scale2) {
#pragma clang fp contract(off)
    float mx = fmaxf(fmaxf(acc[0][0], acc[0][1]), fmaxf(acc[0][2], acc[0][3]));
#pragma unroll
    for (int kt = 1; kt < NKT; ++kt)
        mx = fmaxf(mx, fmaxf(fmaxf(acc[kt][0], acc[kt][1]), fmaxf(acc[kt][2], acc[kt][3])));
    mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m_run, mx);
    // a row without any visible key so far keeps maximum -inf; a finite stand-in makes every exp below 0
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    if (__any(m_new != m_run)) {
        const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * scale2);
        l_run = l_run * alpha;
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            o[d][0] *= alpha; o[d][1] *= alpha; o[d][2] *= alpha; o[d][3] *= alpha;
        }
        m_run = m_new;
    }
    const float shift = -m_use * scale2;
    float sum = 0.f;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(acc[kt][v], scale2, shift));
            sum = sum + pv;
            acc[kt][v] = pv;
        }
    l_run = l_run + sum;
}

// The probabilities of a chunk as the second product's operand: 16-byte pieces of 8 keys (bfloat16, rounded here:
// keys kt * 16 + lg * 4 + v of two tiles kt) or of 4 keys (float32, as they are).
template <typename T, int NKT, int NP>
__device__ __forceinline__ void probabilities(const f32x4 (&acc)[NKT], u32x4 (&p)[NP]) {
    if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            bf16x8 pb;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                pb[v] = static_cast<__bf16>(acc[2 * j][v]);
                pb[4 + v] = static_cast<__bf16>(acc[2 * j + 1][v]);
            }
            p[j] = __builtin_bit_cast(u32x4, pb);
        }
    } else {
#pragma unroll
        for (int j = 0; j < NP; ++j) p[j] = __builtin_bit_cast(u32x4, acc[j]);
    }
}

// Folding a segment's result (m, l, o) into the row's running result (M, L, O): the weights of both sides, then
// value by value.  Starting from (M, L, O) = (-inf, 0, 0) the first segment with visible keys is taken as it is, and a
// segment without visible keys (m = -inf, l = 0, o = 0) changes nothing.
__device__ __forceinline__ void fold_weights(float M, float m, float scale2, float& M_new, float& a, float& b) {
#pragma clang fp contract(off)
    M_new = fmaxf(M, m);
    const float M_use = M_new == -INFINITY ? 0.f : M_new;
    a = __builtin_amdgcn_exp2f((M - M_use) * scale2);
    b = __builtin_amdgcn_exp2f((m - M_use) * scale2);
}
__device__ __forceinline__ float fold_value(float O, float o, float a, float b) {
#pragma clang fp contract(off)
    return __builtin_fmaf(o, b, O * a);
}
__device__ __forceinline__ float normalised(float O, float L) {
#pragma clang fp contract(off)
    return O * (1.0f / L);
}

// Before accumulators of the matrix cores are read on a path that may have skipped instructions: the compiler keeps
// the wait between a matrix instruction and a read of its result by counting the instructions that lie between them
// in the code, also those that a branch jumps over.  Sixteen idle cycles cover the longest of the instructions used here.
__device__ __forceinline__ void settle_matrix_results() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15");
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ int page_of(int key, int page_size, int page_shift) {
    return page_shift >= 0 ? key >> page_shift : key / page_size;
}
__device__ __forceinline__ int offset_in_page(int key, int page_size, int page_shift) {
    return page_shift >= 0 ? key & (page_size - 1) : key % page_size;
}

template <typename T>
__device__ __forceinline__ void store4(T* dst, float a, float b, float c, float d) {
    if constexpr (sizeof(T) == 2) {
        uint2 packed;
        packed.x = f32_to_bf16_bits(a) | (static_cast<uint32_t>(f32_to_bf16_bits(b)) << 16);
        packed.y = f32_to_bf16_bits(c) | (static_cast<uint32_t>(f32_to_bf16_bits(d)) << 16);
        *reinterpret_cast<uint2*>(dst) = packed;
    } else {
        *reinterpret_cast<float4*>(dst) = float4{a, b, c, d};
    }
}

// ---------------------------------------------------------------------------------------------- prompt portions
// A workgroup of RT wavefronts takes 16 * RT rows of one request and key/value head, a tile of 16 rows per
// wavefront, and walks the keys chunk by chunk; a chunk's keys and values are staged through LDS and shared by the
// wavefronts.  Loads run in three stages as in attention_tiled_kernel: page numbers two chunks ahead, keys and
// values into registers one chunk ahead, registers into the other LDS stage behind this chunk's products.
// LDS rows are padded by 16 bytes, which spreads the 16 rows that a quarter of a wavefront reads over all banks.
// In bfloat16 a value row's keys are stored in the order in which a lane takes them (within 32 keys: lg, tile, v),
// so that a lane's 8 keys are one 16-byte read.
template <typename T, int HD, int RT>
__global__ __launch_bounds__(64 * RT) void attention_any_tiled_kernel(
    const T* __restrict__ qkv, T* __restrict__ out, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ kv_len, int n_seqs, int nq, int nkv,
    int page_size, int page_shift, float scale, int window) {
    constexpr int hd = HD;
    constexpr int E = 16 / sizeof(T);             // elements in 16 bytes
    constexpr int KT = chunk_keys<T, HD>();
    constexpr int NKT = KT / 16;                  // tiles of 16 keys in a chunk
    constexpr int NQ = (HD + 4 * E - 1) / (4 * E);    // 16-byte pieces of a row's features that a lane holds
    constexpr int HDP = NQ * 4 * E;               // the head size rounded up to whole pieces (bfloat16: to 32)
    constexpr int NP = KT / (4 * E);              // 16-byte pieces of a chunk's keys that a lane holds
    constexpr int DT = HD / 16;                   // tiles of 16 output features
    constexpr bool SEGMENTS = sizeof(T) == 4;
    constexpr int TPS = kSegment / KT;            // chunks per segment
    constexpr int ROWS = 16 * RT, THREADS = 64 * RT;
    constexpr int KROW = HDP + E, VROW = KT + E;  // padded LDS rows (elements)
    constexpr int STAGE = KT * KROW + HD * VROW;
    constexpr int TPK = THREADS / KT;             // threads that share a key when a chunk is staged
    constexpr int NK = (HD / E + TPK - 1) / TPK;  // 16-byte pieces of its key per thread
    constexpr int VKP = KT / E;                   // 16-byte pieces of a value row (one feature, the chunk's keys)
    constexpr int VPP = THREADS / VKP;            // value rows per pass of all threads
    constexpr int NV = (HD + VPP - 1) / VPP;
    static_assert(THREADS % KT == 0 && THREADS % VKP == 0 && kSegment % KT == 0, "staging shapes");
    __shared__ __attribute__((aligned(16))) T smem[2 * STAGE];

    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int lj = lane % 16, lg = lane / 16;
    const int kh = blockIdx.y;
    const int group_size = nq / nkv;

    int b = 0, grp = blockIdx.x;
    for (; b < n_seqs; ++b) {
        const int groups = (q_len[b] * group_size + ROWS - 1) / ROWS;
        if (grp < groups) {
            grp = groups - 1 - grp;          // the last rows first: they have the most keys to walk
            break;
        }
        grp -= groups;
    }
    if (b >= n_seqs) return;
    const int n = q_len[b], kv = kv_len[b], qs = q_start[b];
    const int rows = n * group_size;
    const int width = (nq + 2 * nkv) * hd;
    const int32_t* table = block_table + static_cast<size_t>(b) * table_width;

    // the workgroup's rows and the keys they need
    const int blk_first = grp * ROWS, blk_last = min(rows, blk_first + ROWS) - 1;
    const int blk_p_hi = kv - n + blk_last / group_size;
    const int blk_first_pos = kv - n + blk_first / group_size;
    const int blk_lo = window > 0 ? max(0, blk_first_pos - window + 1) : 0;
    const int t_begin = blk_lo / KT, t_end = blk_p_hi / KT + 1;

    // this wavefront's tile of 16 rows, this lane's row
    const int row_base = blk_first + wave * 16;
    const int r = row_base + lj;
    const bool valid = r < rows;
    const int i_tok = valid ? r / group_size : 0;
    const int tok = qs + i_tok;
    const int head = kh * group_size + (valid ? r % group_size : 0);
    const int p_row = valid ? kv - n + i_tok : -1;
    const int lo_row = (window > 0 && valid) ? max(0, p_row - window + 1) : 0;
    const bool wave_any = row_base < rows;
    const int w_last = min(rows, row_base + 16) - 1;
    const int w_p_hi = wave_any ? kv - n + w_last / group_size : -1;       // largest causal limit in the tile
    const int w_p_min = wave_any ? kv - n + row_base / group_size : -1;    // smallest
    const int w_lo_first = (window > 0 && wave_any) ? max(0, w_p_min - window + 1) : 0;
    const int w_lo_max = (window > 0 && wave_any) ? max(0, w_p_hi - window + 1) : 0;

    // features beyond the head size stay zero in LDS: nothing below writes them
    if constexpr (HD < HDP) {
        u32x4* z = reinterpret_cast<u32x4*>(smem);
        for (int i = tid; i < 2 * STAGE / E; i += THREADS) z[i] = u32x4{0u, 0u, 0u, 0u};
        __syncthreads();
    }

    u32x4 q[NQ];
    {
        const T* qp = qkv + static_cast<size_t>(tok) * width + head * hd;
#pragma unroll
        for (int j = 0; j < NQ; ++j) {
            const int f = (j * 4 + lg) * E;
            q[j] = (valid && f < hd) ? *reinterpret_cast<const u32x4*>(qp + f) : u32x4{0u, 0u, 0u, 0u};
        }
    }
    const float scale2 = scale * 1.4426950408889634f;   // exp(x) = exp2(x * log2(e))

    f32x4 o[DT];
#pragma unroll
    for (int d = 0; d < DT; ++d) o[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    // float32: (m_run, l_run, o) belong to the segment being walked, (M, L, O) to the row
    [[maybe_unused]] f32x4 O[SEGMENTS ? DT : 1];
    [[maybe_unused]] float M = -INFINITY, L = 0.f;
    if constexpr (SEGMENTS) {
#pragma unroll
        for (int d = 0; d < DT; ++d) O[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    auto fold_segment = [&]() {
        if constexpr (SEGMENTS) {
            settle_matrix_results();
            float l = l_run;
            l += __shfl_xor(l, 16, kWave);
            l += __shfl_xor(l, 32, kWave);
            float M_new, wa, wb;
            fold_weights(M, m_run, scale2, M_new, wa, wb);
            L = fold_value(L, l, wa, wb);
#pragma unroll
            for (int d = 0; d < DT; ++d) {
#pragma unroll
                for (int v = 0; v < 4; ++v) O[d][v] = fold_value(O[d][v], o[d][v], wa, wb);
                o[d] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            M = M_new;
            m_run = -INFINITY;
            l_run = 0.f;
        }
    };

    // staging: a thread takes pieces of one key (all in one page) and of one run of E keys of several value rows
    const int k_row = tid / TPK, k_piece = tid % TPK;
    const int v_key = (tid % VKP) * E, v_row = tid / VKP;
    const int pieces = hd / E;
    u32x4 k_regs[NK], v_regs[NV];
    int k_page, v_page;                              // -1: nothing to read (zeros)
    auto lookup = [&](int tile) {
        const int kk = tile * KT + k_row, vk = tile * KT + v_key;
        k_page = (kk <= blk_p_hi && kk >= blk_lo) ? table[page_of(kk, page_size, page_shift)] : -1;
        v_page = (vk <= blk_p_hi && vk + E - 1 >= blk_lo) ? table[page_of(vk, page_size, page_shift)] : -1;
    };
    auto fetch = [&](int tile) {
        const int kk = tile * KT + k_row, vk = tile * KT + v_key;
        const T* ksrc = k_cache + ((static_cast<long>(max(k_page, 0)) * nkv + kh) * page_size +
                                   offset_in_page(kk, page_size, page_shift)) * hd;
#pragma unroll
        for (int u = 0; u < NK; ++u) {
            const int c = k_piece + u * TPK;
            k_regs[u] = (k_page >= 0 && c < pieces) ? *reinterpret_cast<const u32x4*>(ksrc + c * E) : u32x4{0u, 0u, 0u, 0u};
        }
        const T* vsrc = v_cache + (static_cast<long>(max(v_page, 0)) * nkv + kh) * hd * page_size +
                        offset_in_page(vk, page_size, page_shift);
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int f = v_row + u * VPP;
            v_regs[u] = (v_page >= 0 && f < hd) ? *reinterpret_cast<const u32x4*>(vsrc + static_cast<long>(f) * page_size)
                                                 : u32x4{0u, 0u, 0u, 0u};
        }
    };
    // where this thread's E keys of a value row go: as they are (float32), or in the lanes' order (bfloat16)
    const int v_pos = sizeof(T) == 4 ? v_key : (v_key / 32) * 32 + ((v_key % 16) / 4) * 8 + ((v_key % 32) / 16) * 4;
    auto stash = [&](int stage) {
        T* ks = smem + stage * STAGE + k_row * KROW;
#pragma unroll
        for (int u = 0; u < NK; ++u) {
            const int c = k_piece + u * TPK;
            if (c < pieces) *reinterpret_cast<u32x4*>(ks + c * E) = k_regs[u];
        }
        T* vs = smem + stage * STAGE + KT * KROW + v_pos;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int f = v_row + u * VPP;
            if (f < hd) {
                if constexpr (sizeof(T) == 4) {
                    *reinterpret_cast<u32x4*>(vs + f * VROW) = v_regs[u];
                } else {
                    *reinterpret_cast<u32x2*>(vs + f * VROW) = u32x2{v_regs[u].x, v_regs[u].y};
                    *reinterpret_cast<u32x2*>(vs + f * VROW + 8) = u32x2{v_regs[u].z, v_regs[u].w};
                }
            }
        }
    };

    lookup(t_begin);
    fetch(t_begin);
    lookup(t_begin + 1);
    stash(0);
    __syncthreads();
    for (int tile = t_begin; tile < t_end; ++tile) {
        const int stage = (tile - t_begin) & 1;
        fetch(tile + 1);           // past the last chunk every page number is -1: nothing is read
        lookup(tile + 2);
        const int key0 = tile * KT;
        if (wave_any && key0 <= w_p_hi && key0 + KT - 1 >= w_lo_first) {     // else nothing visible to these rows
            const T* ks = smem + stage * STAGE + lj * KROW + lg * E;
            const T* vs = smem + stage * STAGE + KT * KROW + lj * VROW + lg * E;
            f32x4 acc[NKT];
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) {
                acc[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < NQ; ++j) {
                    const u32x4 a = *reinterpret_cast<const u32x4*>(ks + kt * 16 * KROW + j * 4 * E);
                    acc[kt] = mma_piece<T>(a, q[j], acc[kt]);
                }
            }
            if (!(key0 + KT - 1 <= w_p_min && key0 >= w_lo_max)) {           // on the diagonal or the window's edge
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int key = key0 + kt * 16 + lg * 4 + v;
                        if (!(key <= p_row && key >= lo_row)) acc[kt][v] = -INFINITY;
                    }
            }
            softmax_chunk<NKT, DT>(acc, m_run, l_run, o, scale2);
            u32x4 p[NP];
            probabilities<T, NKT, NP>(acc, p);
#pragma unroll
            for (int d = 0; d < DT; ++d) {
#pragma unroll
                for (int j = 0; j < NP; ++j) {
                    const u32x4 a = *reinterpret_cast<const u32x4*>(vs + d * 16 * VROW + j * 4 * E);
                    o[d] = mma_piece<T>(a, p[j], o[d]);
                }
            }
        }
        if (SEGMENTS && (tile + 1) % TPS == 0) fold_segment();
        stash(stage ^ 1);
        __syncthreads();
    }
    float l;
    if constexpr (SEGMENTS) {
        fold_segment();                     // the segment that the last chunk left open (nothing, if it closed one)
        l = L;
    } else {
        settle_matrix_results();
        l = l_run;
        l += __shfl_xor(l, 16, kWave);
        l += __shfl_xor(l, 32, kWave);
    }
    if (valid) {
        T* op = out + (static_cast<size_t>(tok) * nq + head) * hd + lg * 4;
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            f32x4 v;
            if constexpr (SEGMENTS) v = O[d]; else v = o[d];
            store4<T>(op + d * 16, normalised(v[0], l), normalised(v[1], l), normalised(v[2], l), normalised(v[3], l));
        }
    }
}

// ---------------------------------------------------------------------------------------------- decoded tokens
// One query token per request.  A wavefront takes one segment of the keys of one (request, key/value head, tile of
// up to 16 of the group's heads), reads its keys and values straight into the operands of the matrix cores (nothing
// is shared, so nothing passes through LDS), the next chunk's loads in flight while this one is computed where the
// registers allow, and writes the segment's unnormalised result and its (maximum, sum) to part_o / part_ml, which
// attention_fold_kernel folds.
template <typename T, int HD>
__global__ __launch_bounds__(256) void attention_any_decode_kernel(
    const T* __restrict__ qkv, float* __restrict__ part_o, float* __restrict__ part_ml, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int32_t* __restrict__ block_table, int table_width,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ kv_len, int n_tokens, int nq, int nkv,
    int page_size, int page_shift, float scale, int window, int row_tiles) {
    constexpr int hd = HD;
    constexpr int E = 16 / sizeof(T);
    constexpr int KT = chunk_keys<T, HD>();
    constexpr int NKT = KT / 16, NQ = (HD + 4 * E - 1) / (4 * E), NP = KT / (4 * E), DT = HD / 16;
    constexpr int TPS = kSegment / KT;
    // 16-byte registers of a chunk's keys and values per lane; two chunks are held (one in flight) if that fits
    constexpr int CHUNK_REGS = NKT * NQ + DT * NP;
    constexpr bool AHEAD = CHUNK_REGS <= 32;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, n_waves = blockDim.x / kWave;
    const int lj = lane % 16, lg = lane / 16;
    const int b = blockIdx.x, kh = blockIdx.y / row_tiles, rt = blockIdx.y % row_tiles;
    const int seg = blockIdx.z * n_waves + wave;
    const int group_size = nq / nkv;
    const int kv = kv_len[b], tok = q_start[b];
    const int p = kv - 1;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    if (seg < lo / kSegment || seg > p / kSegment) return;       // (no barrier below)
    const int r = rt * 16 + lj;
    const bool valid = r < group_size;
    const int head = kh * group_size + (valid ? r : 0);
    const int width = (nq + 2 * nkv) * hd;
    const int32_t* table = block_table + static_cast<size_t>(b) * table_width;

    u32x4 q[NQ];
    {
        const T* qp = qkv + static_cast<size_t>(tok) * width + head * hd;
#pragma unroll
        for (int j = 0; j < NQ; ++j) {
            const int f = (j * 4 + lg) * E;
            q[j] = (valid && f < hd) ? *reinterpret_cast<const u32x4*>(qp + f) : u32x4{0u, 0u, 0u, 0u};
        }
    }
    const float scale2 = scale * 1.4426950408889634f;

    // a chunk's operands: keys [tile of 16 keys][piece of features], values [tile of 16 features][piece of keys]
    struct Chunk {
        u32x4 k[NKT][NQ];
        u32x4 v[DT][NP];
    };
    auto visible = [&](int c) {
        const int key0 = seg * kSegment + c * KT;
        return key0 <= p && key0 + KT - 1 >= lo;
    };
    // Every load is issued whatever it is for: a piece beyond the head size, or a tile without visible keys, reads a
    // neighbouring piece (or page 0) and is zeroed afterwards, so that nothing stands between the loads of a chunk.
    auto load_chunk = [&](Chunk& ch, int c) {
        const int key0 = seg * kSegment + c * KT;
        int pages[NKT];
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            const int k0 = key0 + kt * 16;
            // a tile is read only if one of its keys is visible: then it lies in a page that the request holds
            const bool live = k0 <= p && k0 + 15 >= lo;
            pages[kt] = table[live ? page_of(k0, page_size, page_shift) : 0];
            if (!live) pages[kt] = -1;
        }
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            const int k0 = key0 + kt * 16;
            const bool ok = pages[kt] >= 0;
            const long page = ok ? pages[kt] : 0;
            const int off = offset_in_page(k0, page_size, page_shift);
            const T* kp = k_cache + ((page * nkv + kh) * page_size + off + lj) * hd;
#pragma unroll
            for (int j = 0; j < NQ; ++j) {
                const int f = (j * 4 + lg) * E;
                const u32x4 piece = *reinterpret_cast<const u32x4*>(kp + min(f, hd - E));
                ch.k[kt][j] = (ok && f < hd) ? piece : u32x4{0u, 0u, 0u, 0u};
            }
            // values: feature d * 16 + lj, keys off + lg * 4 .. + 3 of this tile
            const T* vp = v_cache + ((page * nkv + kh) * hd + lj) * static_cast<long>(page_size) + off + lg * 4;
#pragma unroll
            for (int d = 0; d < DT; ++d) {
                const bool in = ok;
                const T* src = vp + static_cast<long>(d * 16) * page_size;
                if constexpr (sizeof(T) == 4) {
                    const u32x4 piece = *reinterpret_cast<const u32x4*>(src);
                    ch.v[d][kt] = in ? piece : u32x4{0u, 0u, 0u, 0u};
                } else {
                    u32x2 half = *reinterpret_cast<const u32x2*>(src);
                    if (!in) half = u32x2{0u, 0u};
                    if (kt % 2 == 0) {
                        ch.v[d][kt / 2].x = half.x;
                        ch.v[d][kt / 2].y = half.y;
                    } else {
                        ch.v[d][kt / 2].z = half.x;
                        ch.v[d][kt / 2].w = half.y;
                    }
                }
            }
        }
    };

    f32x4 o[DT];
#pragma unroll
    for (int d = 0; d < DT; ++d) o[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    auto compute_chunk = [&](const Chunk& ch, int c) {
        const int key0 = seg * kSegment + c * KT;
        f32x4 acc[NKT];
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            acc[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < NQ; ++j) acc[kt] = mma_piece<T>(ch.k[kt][j], q[j], acc[kt]);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int key = key0 + kt * 16 + lg * 4 + v;
                if (!(valid && key <= p && key >= lo)) acc[kt][v] = -INFINITY;
            }
        }
        softmax_chunk<NKT, DT>(acc, m_run, l_run, o, scale2);
        u32x4 pr[NP];
        probabilities<T, NKT, NP>(acc, pr);
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int j = 0; j < NP; ++j) o[d] = mma_piece<T>(ch.v[d][j], pr[j], o[d]);
    };

    if constexpr (AHEAD) {
        Chunk ch[2];
        if (visible(0)) load_chunk(ch[0], 0);
#pragma unroll
        for (int c = 0; c < TPS; ++c) {
            if (c + 1 < TPS && visible(c + 1)) load_chunk(ch[(c + 1) & 1], c + 1);
            if (visible(c)) compute_chunk(ch[c & 1], c);
        }
    } else {
        for (int c = 0; c < TPS; ++c) {
            if (!visible(c)) continue;
            Chunk ch;
            load_chunk(ch, c);
            compute_chunk(ch, c);
        }
    }
    settle_matrix_results();
    float l = l_run;
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (valid) {
        const size_t prow = (static_cast<size_t>(seg) * n_tokens + tok) * nq + head;
        float* pp = part_o + prow * hd + lg * 4;
#pragma unroll
        for (int d = 0; d < DT; ++d) *reinterpret_cast<f32x4*>(pp + d * 16) = o[d];
        if (lg == 0) {
            part_ml[prow * 2] = m_run;
            part_ml[prow * 2 + 1] = l;
        }
    }
}

// The row's result from its segments' results, folded in ascending order: one wavefront per (request, head).  The
// fold is a chain, but only its last link has to be walked one segment after the other: the running maximum before
// each segment is a prefix maximum (lane i takes segment i and a scan gives it), the two weights of each fold follow
// from it by fold_weights as they would in the chain, and what is left per segment is one fold_value per feature, a
// lane per feature (and R - 1 more, 64 features apart), with the segments' results loaded sixteen at a time.
template <typename T, int R>
__global__ __launch_bounds__(64) void attention_fold_kernel(const float* __restrict__ part_o,
                                                            const float* __restrict__ part_ml, T* __restrict__ out,
                                                            const int32_t* __restrict__ q_start,
                                                            const int32_t* __restrict__ kv_len, int n_tokens, int nq,
                                                            int hd, float scale, int window, int n_segments) {
    constexpr int BATCH = 16;
    const int b = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int tok = q_start[b], p = kv_len[b] - 1;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int s_lo = lo / kSegment, s_hi = min(p / kSegment, n_segments - 1);     // (the buffers hold n_segments)
    const float scale2 = scale * 1.4426950408889634f;
    const size_t seg_stride = static_cast<size_t>(n_tokens) * nq;
    const size_t row = static_cast<size_t>(tok) * nq + head;
    float M = -INFINITY, L = 0.f, O[R];
#pragma unroll
    for (int r = 0; r < R; ++r) O[r] = 0.f;
    for (int s0 = s_lo; s0 <= s_hi; s0 += kWave) {
        const int n = min(kWave, s_hi - s0 + 1);
        // lane i: the maximum and sum of segment s0 + i, the running maximum before it, and the fold's weights
        float m_i = -INFINITY, l_i = 0.f;
        if (lane < n) {
            const size_t prow = (s0 + lane) * seg_stride + row;
            m_i = part_ml[prow * 2];
            l_i = part_ml[prow * 2 + 1];
        }
        float run = m_i;                      // inclusive prefix maximum over the lanes
#pragma unroll
        for (int off = 1; off < kWave; off *= 2) {
            const float other = __shfl_up(run, off, kWave);
            if (lane >= off) run = fmaxf(run, other);
        }
        run = fmaxf(run, M);
        float before = __shfl_up(run, 1, kWave);
        if (lane == 0) before = M;
        float M_new, wa, wb;
        fold_weights(before, m_i, scale2, M_new, wa, wb);
        for (int i0 = 0; i0 < n; i0 += BATCH) {
            float o_i[BATCH][R];
#pragma unroll
            for (int i = 0; i < BATCH; ++i) {
                const size_t prow = (s0 + min(i0 + i, n - 1)) * seg_stride + row;
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const int d = lane + r * kWave;
                    o_i[i][r] = d < hd ? part_o[prow * hd + d] : 0.f;
                }
            }
#pragma unroll
            for (int i = 0; i < BATCH; ++i) {
                if (i0 + i >= n) break;
                const float a = __shfl(wa, i0 + i, kWave), bw = __shfl(wb, i0 + i, kWave);
                L = fold_value(L, __shfl(l_i, i0 + i, kWave), a, bw);
#pragma unroll
                for (int r = 0; r < R; ++r) O[r] = fold_value(O[r], o_i[i][r], a, bw);
            }
        }
        M = __shfl(run, n - 1, kWave);
    }
    T* op = out + (static_cast<size_t>(tok) * nq + head) * hd;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int d = lane + r * kWave;
        if (d < hd) op[d] = from_float<T>(normalised(O[r], L));
    }
}

template <typename T, int HD>
static int launch_any_tiled(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                            const int32_t* block_table, int table_width, const int32_t* q_start, const int32_t* q_len,
                            const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv, int page_size,
                            int page_shift, float scale, int window, hipStream_t s) {
    constexpr int RT = 4;
    const long groups = (static_cast<long>(n_tokens) * (nq / nkv)) / (16 * RT) + n_seqs;   // upper bound
    dim3 grid(static_cast<unsigned>(groups), nkv);
    attention_any_tiled_kernel<T, HD, RT><<<grid, 64 * RT, 0, s>>>(
        static_cast<const T*>(qkv), static_cast<T*>(out), static_cast<const T*>(k_cache), static_cast<const T*>(v_cache),
        block_table, table_width, q_start, q_len, kv_len, n_seqs, nq, nkv, page_size, page_shift, scale, window);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

template <typename T, int HD>
static int launch_any_decode(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                             const void* v_cache, const int32_t* block_table, int table_width, const int32_t* q_start,
                             const int32_t* kv_len, int n_seqs, int nq, int nkv, int page_size, int page_shift,
                             float scale, int window, int n_segments, hipStream_t s) {
    constexpr int hd = HD;
    const int row_tiles = (nq / nkv + 15) / 16;
    // a wavefront per workgroup while there are few of them: a CU has only so many bytes on their way, so a short
    // batch wants its wavefronts on as many CUs as it can get
    const long waves_in_all = static_cast<long>(n_seqs) * nkv * row_tiles * n_segments;
    const int n_waves = waves_in_all <= 2048 ? 1 : (n_segments < 4 ? n_segments : 4);
    dim3 grid(n_seqs, nkv * row_tiles, (n_segments + n_waves - 1) / n_waves);
    attention_any_decode_kernel<T, HD><<<grid, n_waves * kWave, 0, s>>>(
        static_cast<const T*>(qkv), part_o, part_ml, static_cast<const T*>(k_cache), static_cast<const T*>(v_cache),
        block_table, table_width, q_start, kv_len, n_seqs, nq, nkv, page_size, page_shift, scale, window, row_tiles);
    EGPT_CHECK_LAUNCH();
    constexpr int R = (HD + 63) / 64;
    attention_fold_kernel<T, R><<<dim3(n_seqs, nq), kWave, 0, s>>>(part_o, part_ml, static_cast<T*>(out), q_start, kv_len,
                                                                   n_seqs, nq, hd, scale, window, n_segments);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}

static int shift_of(int page_size) {
    if (page_size & (page_size - 1)) return -1;
    int shift = 0;
    while ((1 << shift) < page_size) ++shift;
    return shift;
}

}  // namespace egpt

using namespace egpt;

#define EGPT_ANY_BY_HEAD(CALL, T_)                        \
    switch (hd / 16) {                                    \
        case 1: return CALL(T_, 16);                      \
        case 2: return CALL(T_, 32);                      \
        case 3: return CALL(T_, 48);                      \
        case 4: return CALL(T_, 64);                      \
        case 5: return CALL(T_, 80);                      \
        case 6: return CALL(T_, 96);                      \
        case 7: return CALL(T_, 112);                     \
        case 8: return CALL(T_, 128);                     \
        case 9: return CALL(T_, 144);                     \
        case 10: return CALL(T_, 160);                    \
        case 11: return CALL(T_, 176);                    \
        case 12: return CALL(T_, 192);                    \
        case 13: return CALL(T_, 208);                    \
        case 14: return CALL(T_, 224);                    \
        case 15: return CALL(T_, 240);                    \
        default: return CALL(T_, 256);                    \
    }

// Prompt portions and mixed batches; same operands and meaning as egpt_paged_attention.  Head sizes that are
// multiples of 16 up to 256, page sizes that are multiples of 16; dtype 0 float32, 1 bfloat16.
extern "C" int egpt_attention_any_tiled(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                                        const int32_t* block_table, int table_width, const int32_t* q_start,
                                        const int32_t* q_len, const int32_t* kv_len, int n_seqs, int n_tokens, int nq,
                                        int nkv, int hd, int page_size, float scale, int window, int dtype,
                                        void* stream) {
    if (!qkv || !out || !k_cache || !v_cache || !block_table || !q_start || !q_len || !kv_len)
        return EGPT_BAD_ARGUMENT;
    if (n_seqs <= 0 || n_tokens < 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || table_width <= 0 || window < 0 ||
        (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (hd <= 0 || hd % 16 != 0 || hd > 256 || page_size <= 0 || page_size % 16 != 0 || nkv > 65535)
        return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int page_shift = shift_of(page_size);
#define EGPT_ANY_TILED(T_, HD_)                                                                                   \
    launch_any_tiled<T_, HD_>(qkv, out, k_cache, v_cache, block_table, table_width, q_start, q_len, kv_len, n_seqs, \
                              n_tokens, nq, nkv, page_size, page_shift, scale, window, s)
    if (dtype == 0) {
        EGPT_ANY_BY_HEAD(EGPT_ANY_TILED, float)
    }
    EGPT_ANY_BY_HEAD(EGPT_ANY_TILED, bf16_t)
#undef EGPT_ANY_TILED
}

// One decoded token per request (token q_start[b] belongs to request b; n_seqs tokens in all).  The keys of a
// request are cut into segments of 64; part_o [n_segments][n_seqs][nq][hd] and part_ml [n_segments][n_seqs][nq][2]
// (float32) take the segments' results, n_segments = ceil(max_kv_len / 64) for the longest context of the batch.
extern "C" int egpt_attention_any_decode(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                                         const void* v_cache, const int32_t* block_table, int table_width,
                                         const int32_t* q_start, const int32_t* kv_len, int n_seqs, int nq, int nkv,
                                         int hd, int page_size, float scale, int window, int n_segments, int dtype,
                                         void* stream) {
    if (!qkv || !out || !part_o || !part_ml || !k_cache || !v_cache || !block_table || !q_start || !kv_len)
        return EGPT_BAD_ARGUMENT;
    if (n_seqs <= 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || table_width <= 0 || window < 0 || n_segments < 1 ||
        (dtype != 0 && dtype != 1))
        return EGPT_BAD_ARGUMENT;
    if (hd <= 0 || hd % 16 != 0 || hd > 256 || page_size <= 0 || page_size % 16 != 0 || nq > 65535 ||
        n_segments > 65535 * 4)
        return EGPT_UNSUPPORTED_SIZE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int page_shift = shift_of(page_size);
#define EGPT_ANY_DECODE(T_, HD_)                                                                                    \
    launch_any_decode<T_, HD_>(qkv, out, part_o, part_ml, k_cache, v_cache, block_table, table_width, q_start, kv_len, \
                               n_seqs, nq, nkv, page_size, page_shift, scale, window, n_segments, s)
    if (dtype == 0) {
        EGPT_ANY_BY_HEAD(EGPT_ANY_DECODE, float)
    }
    EGPT_ANY_BY_HEAD(EGPT_ANY_DECODE, bf16_t)
#undef EGPT_ANY_DECODE
}
