// Paged attention on the matrix cores (bfloat16), for prompt portions and decoded tokens alike.
//
// A wavefront owns QT tiles of 16 query rows of one request and one key/value head.  A row is a
// (token, query head) pair of the head's group, token-major, so the 7 heads of a decoded token share one
// tile (and every load of its keys), and the rows of a prompt tile have nearly the same causal limit.
// Keys are walked 32 at a time.  The scores are computed transposed,
//     S^T[key, row] = K[key, :] . Q[row, :]        v_mfma_f32_16x16x32_bf16, A = K, B = Q
// so that a lane ends up with the scores of ONE row (its column) for four keys per tile: the row's
// running maximum and sum are per-lane scalars, and the probabilities are, as they lie in registers,
// the B operand of the second product
//     O^T[feature, row] += V^T[feature, key] . P^T[key, row]     A = V^T, B = P^T
// whose A operand is what a page of values looks like in memory (values are stored transposed within
// a page).  No operand passes through LDS.  Softmax statistics and the accumulator are float32
// (as /root/reference/src/cuda/ops/self_attn_detail.cuh:299-383); P is rounded to bfloat16 for the
// second product.  With n_splits > 1 each split of the key range writes an unnormalised partial result
// and its (maximum, sum), which attention_reduce_kernel combines.
#include <type_traits>
#include <utility>

#include "api.h"
#include "common.h"

namespace egpt {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

template <int HD, int QT>
__global__ __launch_bounds__(64) void attention_mfma_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ kv_len, int n_seqs, int n_tokens, int nq, int nkv,
    int page_size, float scale, int window, int n_splits) {
    constexpr int KD = HD / 32;  // score MFMAs per key tile (32 features each)
    constexpr int DT = HD / 16;  // output feature tiles
    const int lane = threadIdx.x, lj = lane % 16, lg = lane / 16;
    const int kh = blockIdx.y, split = blockIdx.z;
    const int group_size = nq / nkv;

    // which request, and which group of 16*QT rows of it; within a request the last rows come first: they
    // have the most keys to walk, and the launch is over when the longest wavefront is
    int b = 0, grp = blockIdx.x;
    for (; b < n_seqs; ++b) {
        const int groups = (q_len[b] * group_size + 16 * QT - 1) / (16 * QT);
        if (grp < groups) {
            grp = groups - 1 - grp;
            break;
        }
        grp -= groups;
    }
    if (b >= n_seqs) return;
    const int n = q_len[b], kv = kv_len[b], qs = q_start[b];
    const int rows = n * group_size;
    const int row_base = grp * 16 * QT;
    const int width = (nq + 2 * nkv) * HD;
    const int32_t* table = block_table + static_cast<size_t>(b) * table_width;

    // this lane's row in each tile
    bool valid[QT];
    int tok[QT], head[QT], p_row[QT], lo_row[QT];
    bf16x8 q[QT][KD];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        const int r = row_base + t * 16 + lj;
        valid[t] = r < rows;
        const int i = valid[t] ? r / group_size : 0;
        tok[t] = qs + i;
        head[t] = kh * group_size + (valid[t] ? r % group_size : 0);
        p_row[t] = valid[t] ? kv - n + i : -1;
        lo_row[t] = (window > 0 && valid[t]) ? max(0, p_row[t] - window + 1) : 0;
        const bf16_t* qp = qkv + static_cast<size_t>(tok[t]) * width + head[t] * HD + lg * 8;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            uint4 v = valid[t] ? *reinterpret_cast<const uint4*>(qp + kd * 32) : uint4{0u, 0u, 0u, 0u};
            q[t][kd] = __builtin_bit_cast(bf16x8, v);
        }
    }
    const float scale2 = scale * 1.4426950408889634f;   // scores are kept in units of log 2
    // the smallest causal limit and the largest window start among the valid rows of each tile
    int p_min[QT], lo_max[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        const int r_first = row_base + t * 16, r_last = min(rows, r_first + 16) - 1;
        const bool any = r_first < rows;
        p_min[t] = any ? kv - n + r_first / group_size : -1;
        const int p_last = any ? kv - n + r_last / group_size : -1;
        lo_max[t] = window > 0 ? max(0, p_last - window + 1) : 0;
    }
    // key blocks (32 keys) this wave needs, and this split's share of them
    const int last_row = min(rows, row_base + 16 * QT) - 1;
    const int p_hi = kv - n + last_row / group_size;
    const int first_pos = kv - n + row_base / group_size;
    const int lo_first = window > 0 ? max(0, first_pos - window + 1) : 0;
    const int kb_begin = lo_first / 32, kb_end = p_hi / 32 + 1;
    const int per_split = (kb_end - kb_begin + n_splits - 1) / n_splits;
    const int my_begin = kb_begin + split * per_split;
    const int my_end = min(kb_end, my_begin + per_split);

    f32x4 o[QT][DT];
    float m_run[QT], l_run[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        m_run[t] = -INFINITY;
        l_run[t] = 0.f;
#pragma unroll
        for (int d = 0; d < DT; ++d) o[t][d] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // Keys are walked in rounds of kRound blocks of 32; the loads of the next round are in flight while this
    // round computes (a wavefront is alone on its SIMD here, so nothing else hides the latency).
    constexpr int kRound = 2;
    uint4 k_cur[kRound][2][KD], k_nxt[kRound][2][KD];
    uint2 v_cur[kRound][2][DT], v_nxt[kRound][2][DT];
    auto load_round = [&](uint4 (*kk)[2][KD], uint2 (*vv)[2][DT], int kb0) {
        int pages[kRound][2];
        bool live[kRound][2];
#pragma unroll
        for (int i = 0; i < kRound; ++i)
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                const int key0 = (kb0 + i) * 32 + kt * 16;
                // a tile is read only if some row of this wave can see one of its keys: then it lies in a page the
                // request still holds (p_hi < kv; pages wholly behind the window may have been given back)
                live[i][kt] = kb0 + i < my_end && key0 <= p_hi && key0 + 15 >= lo_first;
                pages[i][kt] = table[live[i][kt] ? key0 / page_size : 0];
            }
#pragma unroll
        for (int i = 0; i < kRound; ++i)
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                const int key0 = (kb0 + i) * 32 + kt * 16;
                const bool ok = live[i][kt] && pages[i][kt] >= 0;
                const long page = ok ? pages[i][kt] : 0;
                const int off = ok ? key0 % page_size : 0;
                const bf16_t* kp = k_cache + ((page * nkv + kh) * page_size + off + lj) * HD + lg * 8;
                const bf16_t* vp = v_cache + ((page * nkv + kh) * HD + lj) * static_cast<long>(page_size) + off + lg * 4;
#pragma unroll
                for (int kd = 0; kd < KD; ++kd)
                    kk[i][kt][kd] = ok ? *reinterpret_cast<const uint4*>(kp + kd * 32) : uint4{0u, 0u, 0u, 0u};
#pragma unroll
                for (int d = 0; d < DT; ++d)
                    vv[i][kt][d] = ok ? *reinterpret_cast<const uint2*>(vp + static_cast<long>(d) * 16 * page_size)
                                      : uint2{0u, 0u};
            }
    };

    if (my_begin < my_end) load_round(k_cur, v_cur, my_begin);
    for (int kb0 = my_begin; kb0 < my_end; kb0 += kRound) {
        if (kb0 + kRound < my_end) load_round(k_nxt, v_nxt, kb0 + kRound);
#pragma unroll
        for (int i = 0; i < kRound; ++i) {
            const int kb = kb0 + i;
            if (kb >= my_end) break;
#pragma unroll
            for (int t = 0; t < QT; ++t) {
                // scores in units of log 2: s = (q . k) * scale * log2(e), so that exp is one v_exp_f32
                float s[2][4];
                float mx = -INFINITY;
                // most blocks lie wholly below the diagonal (and inside the window) for every row of the tile:
                // they need no masking
                const bool all_visible = kb * 32 + 31 <= p_min[t] && kb * 32 >= lo_max[t];
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int kd = 0; kd < KD; ++kd)
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, k_cur[i][kt][kd]),
                                                                      q[t][kd], acc, 0, 0, 0);
                    if (all_visible) {
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            s[kt][v] = acc[v] * scale2;
                            mx = fmaxf(mx, s[kt][v]);
                        }
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            const int key = kb * 32 + kt * 16 + lg * 4 + v;
                            const bool vis = key <= p_row[t] && key >= lo_row[t];
                            s[kt][v] = vis ? acc[v] * scale2 : -INFINITY;
                            mx = fmaxf(mx, s[kt][v]);
                        }
                    }
                }
                mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
                mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
                const float m_new = fmaxf(m_run[t], mx);
                // a row without any visible key so far keeps maximum -inf; subtracting a finite stand-in makes
                // every exp below 0 without a special case (exp2(-inf) = 0)
                const float m_use = m_new == -INFINITY ? 0.f : m_new;
                const float alpha = __builtin_amdgcn_exp2f(m_run[t] - m_use);
                float sum = 0.f;
                bf16x8 pb;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float pv = __builtin_amdgcn_exp2f(s[kt][v] - m_use);
                        sum += pv;
                        pb[kt * 4 + v] = static_cast<__bf16>(pv);
                    }
                l_run[t] = l_run[t] * alpha + sum;
                m_run[t] = m_new;
#pragma unroll
                for (int d = 0; d < DT; ++d) {
                    const uint4 a = uint4{v_cur[i][0][d].x, v_cur[i][0][d].y, v_cur[i][1][d].x, v_cur[i][1][d].y};
                    f32x4 acc = o[t][d];
                    acc[0] *= alpha; acc[1] *= alpha; acc[2] *= alpha; acc[3] *= alpha;
                    o[t][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), pb, acc, 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kRound; ++i)
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) k_cur[i][kt][kd] = k_nxt[i][kt][kd];
#pragma unroll
                for (int d = 0; d < DT; ++d) v_cur[i][kt][d] = v_nxt[i][kt][d];
            }
    }

#pragma unroll
    for (int t = 0; t < QT; ++t) {
        float l = l_run[t];
        l += __shfl_xor(l, 16, kWave);
        l += __shfl_xor(l, 32, kWave);
        if (!valid[t]) continue;
        const size_t row = static_cast<size_t>(tok[t]) * nq + head[t];
        if (n_splits == 1) {
            const float inv = 1.0f / l;
            bf16_t* op = out + row * HD + lg * 4;
#pragma unroll
            for (int d = 0; d < DT; ++d) {
                uint2 packed;
                packed.x = f32_to_bf16_bits(o[t][d][0] * inv) | (static_cast<uint32_t>(f32_to_bf16_bits(o[t][d][1] * inv)) << 16);
                packed.y = f32_to_bf16_bits(o[t][d][2] * inv) | (static_cast<uint32_t>(f32_to_bf16_bits(o[t][d][3] * inv)) << 16);
                *reinterpret_cast<uint2*>(op + d * 16) = packed;
            }
        } else {
            const size_t prow = static_cast<size_t>(split) * n_tokens * nq + row;
            float* pp = part_o + prow * HD + lg * 4;
#pragma unroll
            for (int d = 0; d < DT; ++d) *reinterpret_cast<f32x4*>(pp + d * 16) = o[t][d];
            if (lg == 0) {
                part_ml[prow * 2] = m_run[t] * 0.6931471805599453f;      // back to natural units for the combine
                part_ml[prow * 2 + 1] = l;
            }
        }
    }
}

// Prompt portions.  A workgroup takes RT tiles of 16 rows (of one request and kv head) and walks the keys in
// tiles of 64 * KS, which are staged through LDS and shared by its RT * KS wavefronts; wavefront (rt, ks)
// multiplies row tile rt with the ks-th 64 keys of each tile, and the KS partial results of a row tile are
// combined through LDS at the end.  The next tile's loads are in flight while this one is computed.
// Without the sharing every wavefront reads all of its keys from L2 itself (about 0.5 GB per layer for a
// 2,048-token prompt at these sizes).  A wavefront issues a vector instruction in four cycles, and a prompt
// of a few thousand tokens gives each SIMD only a few wavefronts, so what a tile costs is the vector
// instructions and the waits between them rather than the matrix cores: hence 64 keys per softmax step, the
// accumulator rescaled only when a row's maximum moved, and the split of the keys over wavefronts.
// The arithmetic is that of attention_mfma_kernel.
template <int HD, int RT, int KS>
__global__ __launch_bounds__(64 * RT * KS) void attention_tiled_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ out, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_table, int table_width,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ kv_len,
    int n_seqs, int nq, int nkv, int page_size, int page_shift, float scale, int window, int skip_single) {
    constexpr int KD = HD / 32, DT = HD / 16;
    constexpr int ROWS = 16 * RT;                // rows per workgroup
    constexpr int KT = 64 * KS;                  // keys per LDS tile
    constexpr int KROW = HD + 8, VROW = KT + 8;  // padded rows (bf16 elements)
    constexpr int THREADS = 64 * RT * KS;
    constexpr int CH = HD / (8 * RT);            // 16-byte chunks per thread and tile, of keys and of values
    constexpr int STAGE = KT * KROW + HD * VROW;  // bf16 elements per stage
    constexpr int COMBINE = (KS - 1) * RT * 64 * (DT * 4 + 2) * 2;    // the combination's floats, in bf16 elements
    static_assert(CH >= 1 && HD % (8 * RT) == 0, "a thread takes whole chunks");
    __shared__ __attribute__((aligned(16))) bf16_t smem[(2 * STAGE > COMBINE) ? 2 * STAGE : COMBINE];
    auto ks_at = [&](int stage, int key, int col) -> bf16_t* { return smem + stage * STAGE + key * KROW + col; };
    auto vs_at = [&](int stage, int d, int key) -> bf16_t* { return smem + stage * STAGE + KT * KROW + d * VROW + key; };
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int rt = wave % RT, ksi = wave / RT;
    const int lj = lane % 16, lg = lane / 16;
    const int kh = blockIdx.y;
    const int group_size = nq / nkv;

    int b = 0, grp = blockIdx.x;
    for (; b < n_seqs; ++b) {
        // (skip_single: requests of one token are the decode kernel's, which spreads their keys over wavefronts)
        const int groups = (skip_single && q_len[b] == 1) ? 0 : (q_len[b] * group_size + ROWS - 1) / ROWS;
        if (grp < groups) {
            grp = groups - 1 - grp;          // the last rows first: they have the most keys to walk
            break;
        }
        grp -= groups;
    }
    if (b >= n_seqs) return;
    const int n = q_len[b], kv = kv_len[b], qs = q_start[b];
    const int rows = n * group_size;
    const int width = (nq + 2 * nkv) * HD;
    const int32_t* table = block_table + static_cast<size_t>(b) * table_width;

    // the workgroup's rows and the keys they need
    const int blk_first = grp * ROWS, blk_last = min(rows, blk_first + ROWS) - 1;
    const int blk_p_hi = kv - n + blk_last / group_size;
    const int blk_first_pos = kv - n + blk_first / group_size;
    const int blk_lo = window > 0 ? max(0, blk_first_pos - window + 1) : 0;
    const int t_begin = blk_lo / KT, t_end = blk_p_hi / KT + 1;

    // this wavefront's tile of 16 rows, this lane's row
    const int row_base = blk_first + rt * 16;
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
    bf16x8 q[KD];
    {
        const bf16_t* qp = qkv + static_cast<size_t>(tok) * width + head * HD + lg * 8;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            const uint4 v = valid ? *reinterpret_cast<const uint4*>(qp + kd * 32) : uint4{0u, 0u, 0u, 0u};
            q[kd] = __builtin_bit_cast(bf16x8, v);
        }
    }
    const float scale2 = scale * 1.4426950408889634f;

    f32x4 o[DT];
#pragma unroll
    for (int d = 0; d < DT; ++d) o[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY;                  // the maximum in units of the raw scores
    // The rows' sums of probabilities are left to the matrix cores: one more tile of "values" whose first feature is
    // all ones (lanes lj == 0 hold it, the other features are zeros) gives sum_key P[key, row] as feature 0 of a
    // 17th output tile, in element 0 of the lanes lg == 0.  (Sixteen additions per step on the vector pipe, which is
    // what this kernel waits for, against two matrix instructions on a pipe that is idle seven eighths of the time.)
    f32x4 o_sum = f32x4{0.f, 0.f, 0.f, 0.f};
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = static_cast<__bf16>(lj == 0 ? 1.0f : 0.0f);

    // The loads of a tile go through three stages, each one iteration ahead of the next, so that no load
    // waits for another inside an iteration: page numbers (tile + 2), keys and values into registers
    // (tile + 1), registers into LDS after the products of this tile.  A thread's chunks of a tile lie in
    // one page (keys: CH chunks of one key; values: eight keys of CH features), so a tile costs it two
    // table entries and two addresses.
    const int page_mask = page_size - 1;             // page sizes here are powers of two
    const int k_row = tid / RT, k_col = (tid % RT) * CH * 8;                 // key within the tile, first feature
    const int v_key = (tid % (KT / 8)) * 8, v_row = tid / (KT / 8);          // first of eight keys, feature (+ 8 RT u)
    uint4 k_regs[CH], v_regs[CH];
    int k_page, v_page;                              // -1: nothing to read (zeros)
    auto lookup = [&](int tile) {
        const int kk = tile * KT + k_row, vk = tile * KT + v_key;
        k_page = (kk <= blk_p_hi && kk >= blk_lo) ? table[kk >> page_shift] : -1;
        v_page = (vk <= blk_p_hi && vk + 7 >= blk_lo) ? table[vk >> page_shift] : -1;
    };
    auto fetch = [&](int tile) {
        const int kk = tile * KT + k_row, vk = tile * KT + v_key;
        if (k_page >= 0) {
            const bf16_t* src = k_cache + ((static_cast<long>(k_page) * nkv + kh) * page_size + (kk & page_mask)) * HD + k_col;
#pragma unroll
            for (int u = 0; u < CH; ++u) k_regs[u] = *reinterpret_cast<const uint4*>(src + u * 8);
        } else {
#pragma unroll
            for (int u = 0; u < CH; ++u) k_regs[u] = uint4{0u, 0u, 0u, 0u};
        }
        if (v_page >= 0) {
            const bf16_t* src = v_cache + ((static_cast<long>(v_page) * nkv + kh) * HD + v_row) * page_size + (vk & page_mask);
#pragma unroll
            for (int u = 0; u < CH; ++u)
                v_regs[u] = *reinterpret_cast<const uint4*>(src + static_cast<long>(u) * (8 * RT) * page_size);
        } else {
#pragma unroll
            for (int u = 0; u < CH; ++u) v_regs[u] = uint4{0u, 0u, 0u, 0u};
        }
    };
    // Where this thread puts its chunks, and where this lane reads its operands, in either stage: the loop below is
    // unrolled over the two stages, so that every LDS access is one of these registers plus an immediate offset.
    bf16_t* const k_put[2] = {ks_at(0, k_row, k_col), ks_at(1, k_row, k_col)};
    bf16_t* const v_put[2] = {vs_at(0, v_row, v_key), vs_at(1, v_row, v_key)};
    const bf16_t* const k_get[2] = {ks_at(0, ksi * 64 + lj, lg * 8), ks_at(1, ksi * 64 + lj, lg * 8)};
    const bf16_t* const v_get[2] = {vs_at(0, lj, ksi * 64 + lg * 4), vs_at(1, lj, ksi * 64 + lg * 4)};
    auto stash = [&](auto stage_c) {
        constexpr int stage = decltype(stage_c)::value;
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            *reinterpret_cast<uint4*>(k_put[stage] + u * 8) = k_regs[u];
            *reinterpret_cast<uint4*>(v_put[stage] + u * 8 * RT * VROW) = v_regs[u];
        }
    };
    auto walk = [&](auto stage_c, int tile) {
        constexpr int stage = decltype(stage_c)::value;
        fetch(tile + 1);           // past the last tile every page number is -1: nothing is read
        lookup(tile + 2);
        const int key0 = tile * KT + ksi * 64;       // this wavefront's 64 keys
        if (wave_any && key0 <= w_p_hi && key0 + 63 >= w_lo_first) {     // else nothing visible to these rows
            // S^T = K Q^T: lane (lj, lg) holds keys kt*16 + lg*4 + v of row lj
            f32x4 acc[4];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                acc[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) {
                    const uint4 kk = *reinterpret_cast<const uint4*>(k_get[stage] + kt * 16 * KROW + kd * 32);
                    acc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kk), q[kd], acc[kt], 0, 0, 0);
                }
            }
            if (!(key0 + 63 <= w_p_min && key0 >= w_lo_max)) {           // on the diagonal or the window's edge
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int key = key0 + kt * 16 + lg * 4 + v;
                        if (!(key <= p_row && key >= lo_row)) acc[kt][v] = -INFINITY;
                    }
            }
            float mx = fmaxf(fmaxf(acc[0][0], acc[0][1]), fmaxf(acc[0][2], acc[0][3]));
#pragma unroll
            for (int kt = 1; kt < 4; ++kt) mx = fmaxf(mx, fmaxf(fmaxf(acc[kt][0], acc[kt][1]), fmaxf(acc[kt][2], acc[kt][3])));
            mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
            mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
            const float m_new = fmaxf(m_run, mx);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            if (__any(m_new != m_run)) {             // some row's maximum moved: rescale what is accumulated
                const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * scale2);
                o_sum[0] *= alpha;
#pragma unroll
                for (int d = 0; d < DT; ++d) {
                    o[d][0] *= alpha; o[d][1] *= alpha; o[d][2] *= alpha; o[d][3] *= alpha;
                }
                m_run = m_new;
            }
            const float shift = -m_use * scale2;
            bf16x8 pb[2];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    pb[kt / 2][(kt % 2) * 4 + v] = static_cast<__bf16>(__builtin_amdgcn_exp2f(fmaf(acc[kt][v], scale2, shift)));
            // O^T += V^T P^T, two products of 32 keys per 16 features, and the tile of ones for the rows' sums
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) o_sum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[kb], o_sum, 0, 0, 0);
#pragma unroll
            for (int d = 0; d < DT; ++d)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    const uint2 v0 = *reinterpret_cast<const uint2*>(v_get[stage] + d * 16 * VROW + kb * 32);
                    const uint2 v1 = *reinterpret_cast<const uint2*>(v_get[stage] + d * 16 * VROW + kb * 32 + 16);
                    const uint4 a = uint4{v0.x, v0.y, v1.x, v1.y};
                    o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), pb[kb], o[d], 0, 0, 0);
                }
        }
        stash(std::integral_constant<int, stage ^ 1>{});
        __syncthreads();
    };

    lookup(t_begin);
    fetch(t_begin);
    lookup(t_begin + 1);
    stash(std::integral_constant<int, 0>{});
    __syncthreads();
    for (int tile = t_begin; tile < t_end; tile += 2) {
        walk(std::integral_constant<int, 0>{}, tile);
        if (tile + 1 < t_end) walk(std::integral_constant<int, 1>{}, tile + 1);
    }
    // the row's sum: feature 0 of the tile of ones, which the lane lj of the first quarter holds
    float l = __shfl(o_sum[0], lj, kWave);
    if constexpr (KS > 1) {
        // The wavefronts of one row tile hold partial results over their keys: those with ks > 0 leave
        // theirs in LDS (the tiles are no longer read: the loop ended with a barrier), ks == 0 adds them up.
        constexpr int PER_LANE = DT * 4 + 2;
        float* comb = reinterpret_cast<float*>(smem);
        if (ksi > 0) {
            float* dst = comb + (static_cast<size_t>((ksi - 1) * RT + rt) * PER_LANE) * 64 + lane;
#pragma unroll
            for (int d = 0; d < DT; ++d)
#pragma unroll
                for (int v = 0; v < 4; ++v) dst[(d * 4 + v) * 64] = o[d][v];
            dst[(DT * 4) * 64] = m_run;
            dst[(DT * 4 + 1) * 64] = l;
        }
        __syncthreads();
        if (ksi > 0) return;
        float m_all = m_run;
#pragma unroll
        for (int j = 0; j < KS - 1; ++j)
            m_all = fmaxf(m_all, comb[(static_cast<size_t>(j * RT + rt) * PER_LANE + DT * 4) * 64 + lane]);
        const float m_ref = m_all == -INFINITY ? 0.f : m_all;
        const float w0 = __builtin_amdgcn_exp2f((m_run - m_ref) * scale2);
        l *= w0;
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            o[d][0] *= w0; o[d][1] *= w0; o[d][2] *= w0; o[d][3] *= w0;
        }
#pragma unroll
        for (int j = 0; j < KS - 1; ++j) {
            const float* src = comb + (static_cast<size_t>(j * RT + rt) * PER_LANE) * 64 + lane;
            const float wj = __builtin_amdgcn_exp2f((src[(DT * 4) * 64] - m_ref) * scale2);
            l += src[(DT * 4 + 1) * 64] * wj;
#pragma unroll
            for (int d = 0; d < DT; ++d)
#pragma unroll
                for (int v = 0; v < 4; ++v) o[d][v] += src[(d * 4 + v) * 64] * wj;
        }
    }
    if (valid) {
        const float inv = 1.0f / l;
        bf16_t* op = out + (static_cast<size_t>(tok) * nq + head) * HD + lg * 4;
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            uint2 packed;
            packed.x = f32_to_bf16_bits(o[d][0] * inv) | (static_cast<uint32_t>(f32_to_bf16_bits(o[d][1] * inv)) << 16);
            packed.y = f32_to_bf16_bits(o[d][2] * inv) | (static_cast<uint32_t>(f32_to_bf16_bits(o[d][3] * inv)) << 16);
            *reinterpret_cast<uint2*>(op + d * 16) = packed;
        }
    }
}

// Prompt portions, 32 rows to a wavefront.  The same arithmetic as attention_tiled_kernel with the 32 x 32 x 16 matrix
// instruction: a wavefront takes a block of 32 rows and 64 keys of each tile, S^T[32 keys, 32 rows] = K Q^T leaves a lane
// 16 scores of one row (row = lane % 32; the lane's half h = lane / 32 holds keys 8b + 4h + v of a block of 32, b and v
// in 0..3), and the probabilities are again the second product's operand as they lie: for its step over 16 keys a lane
// supplies eight of them, the same eight that it holds, so a page's values are staged into LDS in that order (within 16
// keys: [h][b % 2][v]).  Against the kernel of 16-row tiles, a score costs half the matrix instructions, half the LDS
// reads and half the staging and loop instructions; what is left per score is its exponential, a multiply-add, a
// maximum and half a conversion, and the kernel is bound by the issue of these vector instructions (an exponential
// takes a wavefront's issue slot for about 8.5 cycles, the others for 4.4, a matrix instruction for 8 of its 32: with
// 32 scores to a lane and tile that is about 1,000 cycles a wavefront and tile, against 640 of the matrix cores), so
// the loop below is built to keep the vector pipe issuing while the matrix cores work.  A workgroup takes RB blocks
// of rows; KS wavefronts per block split each tile of 64 * KS keys and are combined through LDS at the end.  The tiles
// of 64 keys must be whole pages (page sizes 16, 32, 64).
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;      // (native vectors: arrays of them stay in registers)
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// max(a, b, c) in one instruction.  (fmaxf quiets signalling NaNs first, which costs an instruction per operand that
// comes from the matrix cores; scores are never NaN here.)
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in this order
template <int... I, class F>
__device__ __forceinline__ void static_for_each(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_each(std::make_integer_sequence<int, N>{}, f);
}

template <int HD, int RB, int KS, bool SPLIT>
__global__ __launch_bounds__(64 * RB * KS) void attention_rows32_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ out, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_table, int table_width,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ kv_len,
    int n_seqs, int nq, int nkv, int page_size, int page_shift, float scale, int window, int skip_single,
    float* __restrict__ part_o, float* __restrict__ part_ml, int n_splits, int n_tokens) {
    constexpr int NQ = HD / 16;                  // steps of 16 features of the score product
    constexpr int FB = HD / 32;                  // blocks of 32 output features
    constexpr int ROWS = 32 * RB;
    constexpr int KT = 64 * KS;                  // keys per LDS tile
    constexpr int KROW = HD + 8, VROW = KT + 8;  // padded rows (bf16 elements)
    constexpr int THREADS = 64 * RB * KS;
    constexpr int CH = HD / (8 * RB);            // 16-byte chunks per thread and tile, of keys and of values
    constexpr int STAGE = KT * KROW + HD * VROW;
    constexpr int PER_LANE = FB * 16 + 2;        // floats a lane leaves for the combination
    constexpr int COMBINE = (KS - 1) * RB * 64 * PER_LANE * 2;    // in bf16 elements
    static_assert(CH >= 1 && HD % (8 * RB) == 0, "a thread takes whole chunks");
    __shared__ __attribute__((aligned(16))) bf16_t smem[(2 * STAGE > COMBINE) ? 2 * STAGE : COMBINE];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int rb = wave % RB, ksi = wave / RB;
    const int lr = lane % 32, lh = lane / 32;
    const int kh = blockIdx.y;
    const int group_size = nq / nkv;

    int b = 0, grp = blockIdx.x;
    for (; b < n_seqs; ++b) {
        // (skip_single: requests of one token are the decode kernel's, which spreads their keys over wavefronts)
        const int groups = (skip_single && q_len[b] == 1) ? 0 : (q_len[b] * group_size + ROWS - 1) / ROWS;
        if (grp < groups) {
            grp = groups - 1 - grp;          // the last rows first: they have the most keys to walk
            break;
        }
        grp -= groups;
    }
    if (b >= n_seqs) return;
    const int n = q_len[b], kv = kv_len[b], qs = q_start[b];
    const int rows = n * group_size;
    const int width = (nq + 2 * nkv) * HD;
    const int32_t* table = block_table + static_cast<size_t>(b) * table_width;

    // the workgroup's rows and the keys they need
    const int blk_first = grp * ROWS, blk_last = min(rows, blk_first + ROWS) - 1;
    const int blk_p_hi = kv - n + blk_last / group_size;
    const int blk_first_pos = kv - n + blk_first / group_size;
    const int blk_lo = window > 0 ? max(0, blk_first_pos - window + 1) : 0;
    // n_splits > 1: the tiles of keys are dealt over as many workgroups (blockIdx.z), each of which leaves its rows'
    // unnormalised result with its maximum and sum in part_o / part_ml for the kernel that combines them
    // (SPLIT is a parameter of the template so that the kernel without it is compiled as if this were not here; a
    // workgroup takes four tiles at least: fewer are not worth sharing)
    const int t_first = blk_lo / KT, t_last = blk_p_hi / KT + 1;
    const int t_per = SPLIT ? max((t_last - t_first + n_splits - 1) / n_splits, 4) : t_last - t_first;
    const int t_begin = SPLIT ? t_first + static_cast<int>(blockIdx.z) * t_per : t_first;
    const int t_end = SPLIT ? min(t_last, t_begin + t_per) : t_last;
    [[maybe_unused]] const size_t part_row0 = SPLIT ? static_cast<size_t>(blockIdx.z) * n_tokens * nq : 0;

    // this wavefront's block of 32 rows, this lane's row
    const int row_base = blk_first + rb * 32;
    const int r = row_base + lr;
    const bool valid = r < rows;
    const int i_tok = valid ? r / group_size : 0;
    const int tok = qs + i_tok;
    const int head = kh * group_size + (valid ? r % group_size : 0);
    const int p_row = valid ? kv - n + i_tok : -1;
    const int lo_row = (window > 0 && valid) ? max(0, p_row - window + 1) : 0;
    const bool wave_any = row_base < rows;
    const int w_last = min(rows, row_base + 32) - 1;
    const int w_p_hi = wave_any ? kv - n + w_last / group_size : -1;       // largest causal limit in the block
    const int w_p_min = wave_any ? kv - n + row_base / group_size : -1;    // smallest
    const int w_lo_first = (window > 0 && wave_any) ? max(0, w_p_min - window + 1) : 0;
    const int w_lo_max = (window > 0 && wave_any) ? max(0, w_p_hi - window + 1) : 0;
    bf16x8 q[NQ];
    {
        const bf16_t* qp = qkv + static_cast<size_t>(tok) * width + head * HD + lh * 8;
#pragma unroll
        for (int j = 0; j < NQ; ++j) {
            const uint4 v = valid ? *reinterpret_cast<const uint4*>(qp + j * 16) : uint4{0u, 0u, 0u, 0u};
            q[j] = __builtin_bit_cast(bf16x8, v);
        }
    }
    const float scale2 = scale * 1.4426950408889634f;
    if constexpr (SPLIT) {
        if (t_begin >= t_end) {              // no tile of keys is left for this workgroup
            if (valid && ksi == 0 && lh == 0) {
                float* ml = part_ml + (part_row0 + static_cast<size_t>(tok) * nq + head) * 2;
                ml[0] = -INFINITY;
                ml[1] = 0.f;
            }
            return;
        }
    }

    f32x16 o[FB];
#pragma unroll
    for (int f = 0; f < FB; ++f)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[f][e] = 0.f;
    float m_run = -INFINITY;                  // the maximum in units of the raw scores
    // the rows' sums of probabilities come from the matrix cores: a block of "values" whose first feature is all ones
    // (the lanes lane % 32 == 0 hold it) gives them as feature 0 of one more output block, element 0 of the lanes of
    // half 0 (32 additions per step on the vector pipe, which this kernel waits for, against four matrix instructions)
    f32x16 o_sum;
#pragma unroll
    for (int e = 0; e < 16; ++e) o_sum[e] = 0.f;
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = static_cast<__bf16>(lr == 0 ? 1.0f : 0.0f);
    f32x16 zero16;
#pragma unroll
    for (int e = 0; e < 16; ++e) zero16[e] = 0.f;

    // The loop is a pipeline of three stages over the tiles.  In the iteration of tile i a wavefront issues, as one
    // straight line of code, the score product of tile i + 1, the exponentials of tile i and the output product of tile
    // i - 1: the matrix instructions of the two products alternate with the vector instructions of the softmax between
    // them (in groups whose order scheduling fences keep), so that both pipes work at once.  (With a tile's products on
    // either side of its softmax, and the wavefronts of a workgroup in step from barrier to barrier, the pipes took
    // turns: at 8,192 tokens the SIMDs issued vector instructions half of the time and did nothing for much of the
    // rest.)  What does not fit into a straight
    // line is kept out of it: masking (tiles on the diagonal or a window's edge) comes before it, and the accumulated
    // output is rescaled after it, and only when a row's maximum has grown by more than 2^kSlack since the last time:
    // until then the exponentials are taken against the old maximum, so they may reach 2^kSlack instead of 1, which
    // float32 sums and bfloat16 probabilities (the same relative precision at any magnitude) do not mind.
    // LDS holds the keys of tiles i + 1 and i + 2 and the values of tiles i - 1 and i, two slots each; the keys of tile
    // i + 3 and the values of tile i + 1 are on their way from memory meanwhile.
    constexpr float kSlack = 8.0f;
    const int page_mask = page_size - 1;             // page sizes here are powers of two
    const int k_row = tid / RB, k_col = (tid % RB) * CH * 8;                 // key within the tile, first feature
    const int v_key = (tid % (KT / 8)) * 8, v_row = tid / (KT / 8);          // first of eight keys, feature (+ 8 RB u)
    // where a run of eight keys goes within its 16 keys of a value row: the first four to half 0, the others to half 1
    const int v_pos = (v_key / 16) * 16 + ((v_key % 16) / 8) * 4;
    // Loads without branches, so that they can stand in the straight line: a thread's key row and its run of eight
    // values lie at the same place of their page in every tile (a tile is whole pages), so a load's address is the
    // page's number times the pages' stride plus a constant of the thread.  The index into the block table is clamped
    // to the pages that hold the workgroup's keys, so every load reads memory of this request; what lies outside the
    // keys that the rows see is replaced by zeros when a tile at either end is put into LDS.
    u32x4 k_regs[CH], v_regs[CH];
    int k_page, v_page;
    const long page_stride = static_cast<long>(nkv) * page_size * HD;
    const bf16_t* const k_base = k_cache + (static_cast<long>(kh) * page_size + (k_row & page_mask)) * HD + k_col;
    const bf16_t* const v_base = v_cache + (static_cast<long>(kh) * HD + v_row) * page_size + (v_key & page_mask);
    const int idx_lo = blk_lo >> page_shift, idx_hi = blk_p_hi >> page_shift, idx_step = KT >> page_shift;
    const int k_sub = k_row >> page_shift, v_sub = v_key >> page_shift;
    auto clamped = [&](int idx) { return min(max(idx, idx_lo), idx_hi); };
    auto lookup_k = [&](int tile) { k_page = max(table[clamped(tile * idx_step + k_sub)], 0); };
    auto lookup_v = [&](int tile) { v_page = max(table[clamped(tile * idx_step + v_sub)], 0); };
    auto fetch_k = [&]() {
        const bf16_t* src = k_base + k_page * page_stride;
#pragma unroll
        for (int u = 0; u < CH; ++u) k_regs[u] = *reinterpret_cast<const u32x4*>(src + u * 8);
    };
    auto fetch_v = [&]() {
        const bf16_t* src = v_base + v_page * page_stride;
#pragma unroll
        for (int u = 0; u < CH; ++u)
            v_regs[u] = *reinterpret_cast<const u32x4*>(src + static_cast<long>(u) * (8 * RB) * page_size);
    };
    auto at_an_end = [&](int tile) { return tile * KT < blk_lo || tile * KT + KT - 1 > blk_p_hi; };
    auto trim_k = [&](int tile) {            // zeros for the keys of this tile that no row of the workgroup sees
        if (at_an_end(tile)) {
            const int kk = tile * KT + k_row;
            if (!(kk <= blk_p_hi && kk >= blk_lo)) {
#pragma unroll
                for (int u = 0; u < CH; ++u) k_regs[u] = u32x4{0u, 0u, 0u, 0u};
            }
        }
    };
    auto trim_v = [&](int tile) {
        if (at_an_end(tile)) {
            const int vk = tile * KT + v_key;
            if (!(vk <= blk_p_hi && vk + 7 >= blk_lo)) {
#pragma unroll
                for (int u = 0; u < CH; ++u) v_regs[u] = u32x4{0u, 0u, 0u, 0u};
            }
        }
    };
    // the slots: keys [2][KT][KROW], then values [2][HD][VROW]
    constexpr int KSLOT = KT * KROW, VSLOT = HD * VROW;
    static_assert(2 * (KSLOT + VSLOT) == 2 * STAGE, "the slots fill the two stages");
    bf16_t* const k_put[2] = {smem + k_row * KROW + k_col, smem + KSLOT + k_row * KROW + k_col};
    bf16_t* const v_put[2] = {smem + 2 * KSLOT + v_row * VROW + v_pos, smem + 2 * KSLOT + VSLOT + v_row * VROW + v_pos};
    const bf16_t* const k_get[2] = {smem + (ksi * 64 + lr) * KROW + lh * 8, smem + KSLOT + (ksi * 64 + lr) * KROW + lh * 8};
    const bf16_t* const v_get[2] = {smem + 2 * KSLOT + lr * VROW + ksi * 64 + lh * 8,
                                    smem + 2 * KSLOT + VSLOT + lr * VROW + ksi * 64 + lh * 8};
    auto stash_k = [&](auto slot_c) {
        constexpr int slot = decltype(slot_c)::value;
#pragma unroll
        for (int u = 0; u < CH; ++u) *reinterpret_cast<u32x4*>(k_put[slot] + u * 8) = k_regs[u];
    };
    auto stash_v = [&](auto slot_c) {
        constexpr int slot = decltype(slot_c)::value;
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            bf16_t* vp = v_put[slot] + u * 8 * RB * VROW;
            *reinterpret_cast<u32x2*>(vp) = u32x2{v_regs[u][0], v_regs[u][1]};
            *reinterpret_cast<u32x2*>(vp + 8) = u32x2{v_regs[u][2], v_regs[u][3]};
        }
    };
    // the scores of a tile from a key slot
    auto scores = [&](auto slot_c, f32x16 (&acc)[2]) {
        constexpr int slot = decltype(slot_c)::value;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int j = 0; j < NQ; ++j) {
                const u32x4 kk = *reinterpret_cast<const u32x4*>(k_get[slot] + kb * 32 * KROW + j * 16);
                acc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kk), q[j],
                                                                  j == 0 ? zero16 : acc[kb], 0, 0, 0);
            }
        }
    };
    // the output product of a tile from a value slot
    auto outputs = [&](auto slot_c, const bf16x8 (&pb)[4]) {
        constexpr int slot = decltype(slot_c)::value;
#pragma unroll
        for (int t = 0; t < 4; ++t) o_sum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[t], o_sum, 0, 0, 0);
#pragma unroll
        for (int f = 0; f < FB; ++f)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const u32x4 a = *reinterpret_cast<const u32x4*>(v_get[slot] + f * 32 * VROW + t * 16);
                o[f] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), pb[t], o[f], 0, 0, 0);
            }
    };
    const float slack = kSlack / scale2;
    // Iteration of tile i, whose parity relative to the first tile is PAR.  The keys of tile i + 1 lie in key slot
    // PAR ^ 1, the values of tile i - 1 in value slot PAR ^ 1; `cur` holds the scores of tile i, `nxt` takes those of
    // tile i + 1; `pb_prev` holds the probabilities of tile i - 1, `pb_new` takes those of tile i.
    auto iterate = [&](auto par_c, int tile, f32x16 (&cur)[2], f32x16 (&nxt)[2], const bf16x8 (&pb_prev)[4],
                       bf16x8 (&pb_new)[4]) {
        constexpr int par = decltype(par_c)::value;
        // what the iteration before has loaded goes into the slots that it has read for the last time (the barrier
        // at its end lies between); the loads of this iteration have all of it to arrive
        trim_k(tile + 2);
        stash_k(std::integral_constant<int, par>{});     // read from the next iteration on
        trim_v(tile);
        stash_v(std::integral_constant<int, par>{});
        const int key0 = tile * KT + ksi * 64;
        if (!(wave_any && key0 + 63 <= w_p_min && key0 >= w_lo_max)) {   // the diagonal, a window's edge, or nothing at all
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = key0 + kb * 32 + (e / 4) * 8 + lh * 4 + e % 4;
                    if (!(key <= p_row && key >= lo_row)) cur[kb][e] = -INFINITY;
                }
        }
        // The straight line, group by group: a matrix instruction, the LDS read of the operand that the matrix
        // instruction three groups on will take, and a share of the vector work; a scheduling fence after every group
        // keeps them in this order.  The matrix instructions: 2 NQ for the scores of tile i + 1, four that sum the rows
        // of tile i - 1, 4 FB for its output.  The vector work: the rows' maxima of tile i in the first four groups (with
        // the loads of the tiles to come, whose addresses are a few instructions), the new maximum and what follows
        // from it in the fifth, then the 32 exponentials of a lane dealt over the groups that are left.
        constexpr int N_QK = 2 * NQ, N_MATRIX = N_QK + 4 + 4 * FB, AHEAD = 3, MAX_GROUPS = 4;
        constexpr int EXP_GROUPS = N_MATRIX - MAX_GROUPS - 1;
        u32x4 operand[AHEAD + 1];
        // (consecutive matrix instructions go to different accumulators: one that adds to the result of the one before
        // it would wait for it)
        auto read_operand = [&](auto g_c) {
            constexpr int g = decltype(g_c)::value;
            if constexpr (g < N_QK) {
                operand[g % (AHEAD + 1)] =
                    *reinterpret_cast<const u32x4*>(k_get[par ^ 1] + (g % 2) * 32 * KROW + (g / 2) * 16);
            } else if constexpr (g < N_MATRIX && (g - N_QK) % (1 + FB) != 0) {
                constexpr int t = (g - N_QK) / (1 + FB), f = (g - N_QK) % (1 + FB) - 1;
                operand[g % (AHEAD + 1)] = *reinterpret_cast<const u32x4*>(v_get[par ^ 1] + f * 32 * VROW + t * 16);
            }
        };
        float mx = -INFINITY, mx1 = -INFINITY, alpha = 1.0f, shift = 0.0f;
        bool rescale = false;
        auto group = [&](auto g_c) {
            constexpr int g = decltype(g_c)::value;
            read_operand(std::integral_constant<int, g + AHEAD>{});
            const bf16x8 from_lds = __builtin_bit_cast(bf16x8, operand[g % (AHEAD + 1)]);
            if constexpr (g < N_QK) {
                nxt[g % 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(from_lds, q[g / 2], g / 2 == 0 ? zero16 : nxt[g % 2],
                                                                     0, 0, 0);
            } else if constexpr ((g - N_QK) % (1 + FB) == 0) {
                o_sum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb_prev[(g - N_QK) / (1 + FB)], o_sum, 0, 0, 0);
            } else {
                constexpr int t = (g - N_QK) / (1 + FB), f = (g - N_QK) % (1 + FB) - 1;
                o[f] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(from_lds, pb_prev[t], o[f], 0, 0, 0);
            }
            if constexpr (g < MAX_GROUPS) {
                // a quarter of the 32 scores of a lane: four of each of its two blocks
#pragma unroll
                for (int e = 4 * g; e < 4 * g + 4; e += 2) {
                    mx = max3(mx, cur[0][e], cur[0][e + 1]);
                    mx1 = max3(mx1, cur[1][e], cur[1][e + 1]);
                }
                if constexpr (g == 0) fetch_k();          // tile i + 3, whose page number the iteration before looked up
                if constexpr (g == 1) fetch_v();          // tile i + 1
                if constexpr (g == 2) lookup_k(tile + 4);
                if constexpr (g == 3) lookup_v(tile + 2);
            } else if constexpr (g == MAX_GROUPS) {
                mx = fmaxf(mx, mx1);
                mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
                // (without a branch, which would cut the straight line in two)
                rescale = __any(mx > m_run + slack);      // (-inf + slack is -inf: the first key a row sees counts)
                const float m_new = rescale ? fmaxf(m_run, mx) : m_run;
                const float m_use = m_new == -INFINITY ? 0.f : m_new;
                alpha = __builtin_amdgcn_exp2f((m_run - m_use) * scale2);
                m_run = m_new;
                shift = -m_use * scale2;
            } else {
                // the second product's steps of 16 keys: step t takes elements 8 (t % 2) .. + 7 of block t / 2 from a lane
                constexpr int eg = g - MAX_GROUPS - 1;
                constexpr int first = eg * 32 / EXP_GROUPS, last = (eg + 1) * 32 / EXP_GROUPS;
#pragma unroll
                for (int i = first; i < last; ++i) {
                    const int t = i / 8, e = i % 8;
                    pb_new[t][e] = static_cast<__bf16>(__builtin_amdgcn_exp2f(fmaf(cur[t / 2][(t % 2) * 8 + e], scale2, shift)));
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        static_for<AHEAD>(read_operand);
        __builtin_amdgcn_sched_barrier(0);
        static_for<N_MATRIX>(group);
        // (the probabilities are first used in the next iteration; this keeps the compiler from moving their
        // computation out of the straight line, behind the branch below)
#pragma unroll
        for (int t = 0; t < 4; ++t) asm volatile("" : "+v"(pb_new[t]));
        if (rescale) {               // what is accumulated, the product of tile i - 1 included, in units of the new maximum
            o_sum[0] *= alpha;
#pragma unroll
            for (int f = 0; f < FB; ++f)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[f][e] *= alpha;
        }
        __syncthreads();
    };

    f32x16 acc_a[2], acc_b[2];
    bf16x8 pb_a[4], pb_b[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int e = 0; e < 8; ++e) pb_b[t][e] = static_cast<__bf16>(0.0f);
    lookup_k(t_begin);
    fetch_k();
    lookup_k(t_begin + 1);
    trim_k(t_begin);
    stash_k(std::integral_constant<int, 0>{});
    fetch_k();
    lookup_k(t_begin + 2);
#pragma unroll
    for (int u = 0; u < CH; ++u) v_regs[u] = u32x4{0u, 0u, 0u, 0u};
    stash_v(std::integral_constant<int, 1>{});       // the first iteration multiplies this slot by probabilities of zero
    lookup_v(t_begin);
    fetch_v();
    lookup_v(t_begin + 1);
    trim_k(t_begin + 1);
    stash_k(std::integral_constant<int, 1>{});
    fetch_k();                                       // tile 2, for the first iteration to put into slot 0
    lookup_k(t_begin + 3);
    __syncthreads();
    scores(std::integral_constant<int, 0>{}, acc_a);
    __syncthreads();                 // every wavefront has read the first tile's keys before their slot is written again
    for (int tile = t_begin; tile < t_end; tile += 2) {
        iterate(std::integral_constant<int, 0>{}, tile, acc_a, acc_b, pb_b, pb_a);
        if (tile + 1 < t_end) iterate(std::integral_constant<int, 1>{}, tile + 1, acc_b, acc_a, pb_a, pb_b);
    }
    // the output product of the last tile
    if ((t_end - t_begin) & 1) outputs(std::integral_constant<int, 0>{}, pb_a);
    else outputs(std::integral_constant<int, 1>{}, pb_b);
    if constexpr (KS > 1) __syncthreads();           // the combination below writes over the tiles
    // the row's sum: feature 0 of the block of ones, which lane lr of half 0 holds
    float l = __shfl(o_sum[0], lr, kWave);
    [[maybe_unused]] float m_part = m_run;           // the maximum that o and l are in units of
    if constexpr (KS > 1) {
        // The wavefronts of one block of rows hold partial results over their keys: those with ks > 0 leave
        // theirs in LDS (the tiles are no longer read: the loop ended with a barrier), ks == 0 adds them up.
        float* comb = reinterpret_cast<float*>(smem);
        if (ksi > 0) {
            float* dst = comb + (static_cast<size_t>((ksi - 1) * RB + rb) * PER_LANE) * 64 + lane;
#pragma unroll
            for (int f = 0; f < FB; ++f)
#pragma unroll
                for (int e = 0; e < 16; ++e) dst[(f * 16 + e) * 64] = o[f][e];
            dst[(FB * 16) * 64] = m_run;
            dst[(FB * 16 + 1) * 64] = l;
        }
        __syncthreads();
        if (ksi > 0) return;
        float m_all = m_run;
#pragma unroll
        for (int j = 0; j < KS - 1; ++j)
            m_all = fmaxf(m_all, comb[(static_cast<size_t>(j * RB + rb) * PER_LANE + FB * 16) * 64 + lane]);
        if constexpr (SPLIT) m_part = m_all;
        const float m_ref = m_all == -INFINITY ? 0.f : m_all;
        const float w0 = __builtin_amdgcn_exp2f((m_run - m_ref) * scale2);
        l *= w0;
#pragma unroll
        for (int f = 0; f < FB; ++f)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[f][e] *= w0;
#pragma unroll
        for (int j = 0; j < KS - 1; ++j) {
            const float* src = comb + (static_cast<size_t>(j * RB + rb) * PER_LANE) * 64 + lane;
            const float wj = __builtin_amdgcn_exp2f((src[(FB * 16) * 64] - m_ref) * scale2);
            l += src[(FB * 16 + 1) * 64] * wj;
#pragma unroll
            for (int f = 0; f < FB; ++f)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[f][e] += src[(f * 16 + e) * 64] * wj;
        }
    }
    if constexpr (SPLIT) {
        // (element e of block f is feature f * 32 + (e / 4) * 8 + lh * 4 + e % 4: runs of four features; the maximum
        // goes out in units of the exponent's argument, as the combining kernel takes it; -inf: no key seen)
        if (valid) {
            const size_t prow = part_row0 + static_cast<size_t>(tok) * nq + head;
            float* po = part_o + prow * HD + lh * 4;
#pragma unroll
            for (int f = 0; f < FB; ++f)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    *reinterpret_cast<float4*>(po + f * 32 + g * 8) =
                        float4{o[f][g * 4], o[f][g * 4 + 1], o[f][g * 4 + 2], o[f][g * 4 + 3]};
            if (lh == 0) {
                part_ml[prow * 2] = m_part * scale;
                part_ml[prow * 2 + 1] = l;
            }
        }
        return;
    }
    if (valid) {
        // element e of block f is feature f * 32 + (e / 4) * 8 + lh * 4 + e % 4: runs of four features
        const float inv = 1.0f / l;
        bf16_t* op = out + (static_cast<size_t>(tok) * nq + head) * HD + lh * 4;
#pragma unroll
        for (int f = 0; f < FB; ++f)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint2 packed;
                packed.x = f32_to_bf16_bits(o[f][g * 4] * inv) | (static_cast<uint32_t>(f32_to_bf16_bits(o[f][g * 4 + 1] * inv)) << 16);
                packed.y = f32_to_bf16_bits(o[f][g * 4 + 2] * inv) | (static_cast<uint32_t>(f32_to_bf16_bits(o[f][g * 4 + 3] * inv)) << 16);
                *reinterpret_cast<uint2*>(op + f * 32 + g * 8) = packed;
            }
    }
}

// What the fused variant of the decode kernel computes its queries (and the new token's key and value) from:
// the QKV product as it comes out of the skinny product kernel, before bias, rotation and rounding.
struct FusedQkv {
    const float* prod;        // [in_splits][n_tokens][(nq + 2 nkv) * hd] float32 partial sums
    int in_splits;
    const float* row_ss;      // [ss_splits][n_tokens] sums of squares of the rows (1/rms still to apply), or null
    int ss_splits;
    float inv_hidden, eps;
    const bf16_t* bias;       // [(nq + 2 nkv) * hd] or null
    const float* cos_sin;     // [n_tokens][hd / 2][2]: (cos, sin) of the tokens' rotation angles (egpt_rope_table)
    const int32_t* slots;     // [n_tokens] page * page_size + offset of the token's key and value
    bf16_t* k_cache_w;        // the caches again, writable
    bf16_t* v_cache_w;
};

// Decoded tokens only (one query token per request, its heads of one kv group in one 16-row tile): a
// workgroup of NW wavefronts shares one (request, kv head, key split); each wavefront walks its share of
// the keys, PF blocks of 32 keys per round with all of the round's loads in flight together (the kernel is
// a chain of round trips to memory, not of arithmetic), and the wavefronts' results are combined through
// LDS.  With n_splits > 1 the combined, still unnormalised result goes to part_o / part_ml.
//
// FUSED: the kernel also does what the QKV epilogue kernel does for these tokens, which takes that kernel
// out of the chain of a decode step.  Every workgroup adds up the product's partial sums for its query
// heads, applies the rows' 1/rms, bias and rotation (same operations in the same order as
// qkv_rope_store_kernel, so the same bits) and keeps the queries in LDS.  The workgroup whose key range ends
// with the new token does the same for that token's key and value, writes them to the cache and, because
// its own loads of that cache line may have been issued before, puts them into its operands itself.
template <int HD, int PF, bool FUSED, bool MIXED = false>
__global__ __launch_bounds__(512) void attention_decode_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ kv_len, int n_tokens, int nq, int nkv, int page_size, float scale, int window,
    int n_splits, FusedQkv f, const int32_t* __restrict__ q_len) {
    constexpr int KD = HD / 32, DT = HD / 16;
    constexpr int kRow = HD + 2;
    // MIXED: a step that also holds portions of prompts; this kernel takes its requests of one token, parts are kept
    // by request (n_tokens is the number of requests then) and the rest is another kernel's.  (A parameter of the
    // template, so that the kernel of the decode step is compiled as if this were not here.)
    if constexpr (MIXED) {
        if (q_len[blockIdx.x] != 1) return;
    }
    extern __shared__ float wave_state[];          // [n_waves][16][HD + 2]: O, then maximum, then sum
    const int lane = threadIdx.x % kWave, n_waves = blockDim.x / kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // known to be the same for the wavefront
    const int lj = lane % 16, lg = lane / 16;
    const int b = blockIdx.x, kh = blockIdx.y, split = blockIdx.z;
    const int group_size = nq / nkv;
    const int kv = kv_len[b], tok = q_start[b];
    const int p = kv - 1;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const bool valid = lj < group_size;
    const int head = kh * group_size + (valid ? lj : 0);
    const int width = (nq + 2 * nkv) * HD;
    const int32_t* table = block_table + static_cast<size_t>(b) * table_width;

    const int kb_begin = lo / 32, kb_end = p / 32 + 1;
    const int per_split = (kb_end - kb_begin + n_splits - 1) / n_splits;
    const int s_begin = kb_begin + split * per_split, s_end = min(kb_end, s_begin + per_split);
    const int per_wave = (max(s_end - s_begin, 0) + n_waves - 1) / n_waves;
    const int w_begin = s_begin + wave * per_wave, w_end = min(s_end, w_begin + per_wave);
    // FUSED: does this workgroup's key range end with the new token?
    const bool writer = FUSED && split == (kb_end - 1 - kb_begin) / per_split;
    bf16_t* q_lds = reinterpret_cast<bf16_t*>(wave_state + n_waves * 16 * kRow);   // FUSED: [16][HD], then k, v [HD]
    bf16_t* k_lds = q_lds + 16 * HD;
    bf16_t* v_lds = k_lds + HD;

    // One round of loads: PF blocks of 32 keys and their values for this wavefront, first all page numbers
    // (one wait for all of them), then all key and value loads.  The first round is issued before anything
    // else, so that the queries (a round trip of their own, two in the fused variant) arrive meanwhile.
    uint4 kk[PF][2][KD];
    uint2 vv[PF][2][DT];
    auto load_round = [&](int kb0) {
        int pages[PF][2];
        bool live[PF][2];
#pragma unroll
        for (int i = 0; i < PF; ++i)
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                const int key0 = (kb0 + i) * 32 + kt * 16;
                live[i][kt] = kb0 + i < w_end && key0 <= p && key0 + 15 >= lo;
                pages[i][kt] = table[live[i][kt] ? key0 / page_size : 0];
            }
#pragma unroll
        for (int i = 0; i < PF; ++i)
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                const int key0 = (kb0 + i) * 32 + kt * 16;
                const bool ok = live[i][kt] && pages[i][kt] >= 0;
                const long page = ok ? pages[i][kt] : 0;
                const int off = ok ? key0 % page_size : 0;
                const bf16_t* kp = k_cache + ((page * nkv + kh) * page_size + off + lj) * HD + lg * 8;
                const bf16_t* vp = v_cache + ((page * nkv + kh) * HD + lj) * static_cast<long>(page_size) + off + lg * 4;
#pragma unroll
                for (int kd = 0; kd < KD; ++kd)
                    kk[i][kt][kd] = ok ? *reinterpret_cast<const uint4*>(kp + kd * 32) : uint4{0u, 0u, 0u, 0u};
#pragma unroll
                for (int d = 0; d < DT; ++d)
                    vv[i][kt][d] = ok ? *reinterpret_cast<const uint2*>(vp + static_cast<long>(d) * 16 * page_size)
                                      : uint2{0u, 0u};
            }
    };
    // The queries.  Their loads are issued here, ahead of the first round of keys and values, and used behind
    // it: loads are waited for in the order of their issue, so what the fused variant computes from its loads
    // (which come from L2) is done while the keys and values (from HBM) are still on their way.
    bf16x8 q[KD];
    constexpr int half = HD / 2, INF = 8;
    struct Item {
        float ta[INF], tb[INF], b0, b1, cs, sn;
    };
    [[maybe_unused]] Item first;
    [[maybe_unused]] float sst[16];
    [[maybe_unused]] int slot_page = 0, slot_off = 0;
    const int n_items = FUSED ? (group_size + (writer ? 2 : 0)) * half : 0;      // pairs (i, i + half) of a head
    const size_t stride = static_cast<size_t>(n_tokens) * width;
    auto item_col = [&](int it) {
        const int h = it / half, i = it % half;
        return (h < group_size ? kh * group_size + h : h == group_size ? nq + kh : nq + nkv + kh) * HD + i;
    };
    auto item_load = [&](int it, Item& r) {
        const int h = it / half, i = it % half, col = item_col(it);
        const float* src = f.prod + static_cast<size_t>(tok) * width + col;
#pragma unroll
        for (int j = 0; j < INF; ++j) {
            const float* pj = src + min(j, f.in_splits - 1) * stride;
            r.ta[j] = pj[0];
            r.tb[j] = pj[half];
        }
        r.b0 = f.bias ? to_float(f.bias[col]) : 0.f;
        r.b1 = f.bias ? to_float(f.bias[col + half]) : 0.f;
        r.cs = 1.f;
        r.sn = 0.f;
        if (h <= group_size) {                   // queries and the key are rotated, the value is not
            r.cs = f.cos_sin[(static_cast<size_t>(tok) * half + i) * 2];
            r.sn = f.cos_sin[(static_cast<size_t>(tok) * half + i) * 2 + 1];
        }
    };
    auto item_finish = [&](int it, const Item& r, float row_scale) {
        const int h = it / half, i = it % half, col = item_col(it);
        float x0 = 0.f, x1 = 0.f;
#pragma unroll
        for (int j = 0; j < INF; ++j) {
            if (j < f.in_splits) {
                x0 += r.ta[j];
                x1 += r.tb[j];
            }
        }
        const float* src = f.prod + static_cast<size_t>(tok) * width + col;
        for (int j = INF; j < f.in_splits; ++j) {          // more partial sums than one batch of loads: rare
            x0 += src[j * stride];
            x1 += src[j * stride + half];
        }
        x0 = scale_then_bias(x0, row_scale, r.b0);
        x1 = scale_then_bias(x1, row_scale, r.b1);
        if (h <= group_size) {
            float r0, r1;
            rotate_pair(x0, x1, r.cs, r.sn, r0, r1);
            x0 = r0;
            x1 = r1;
        }
        const bf16_t y0 = from_float<bf16_t>(x0), y1 = from_float<bf16_t>(x1);
        const long page = slot_page, off = slot_off;
        if (h < group_size) {
            q_lds[h * HD + i] = y0;
            q_lds[h * HD + i + half] = y1;
        } else if (h == group_size) {            // keys: [page][kv head][offset][feature]
            k_lds[i] = y0;
            k_lds[i + half] = y1;
            bf16_t* dst = f.k_cache_w + ((page * nkv + kh) * page_size + off) * HD;
            dst[i] = y0;
            dst[i + half] = y1;
        } else {                                 // values: [page][kv head][feature][offset]
            v_lds[i] = y0;
            v_lds[i + half] = y1;
            f.v_cache_w[((page * nkv + kh) * HD + i) * page_size + off] = y0;
            f.v_cache_w[((page * nkv + kh) * HD + i + half) * page_size + off] = y1;
        }
    };
    if constexpr (!FUSED) {
        const bf16_t* qp = qkv + static_cast<size_t>(tok) * width + head * HD + lg * 8;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            const uint4 v = valid ? *reinterpret_cast<const uint4*>(qp + kd * 32) : uint4{0u, 0u, 0u, 0u};
            q[kd] = __builtin_bit_cast(bf16x8, v);
        }
    } else {
        if (f.row_ss) {
#pragma unroll
            for (int i = 0; i < 16; ++i) sst[i] = f.row_ss[min(i, f.ss_splits - 1) * n_tokens + tok];
        }
        const int slot = f.slots[tok];
        slot_page = slot / page_size;
        slot_off = slot % page_size;
        if (static_cast<int>(threadIdx.x) < n_items) item_load(threadIdx.x, first);
    }
    auto make_q = [&]() {
        if constexpr (FUSED) {
            float row_scale = 1.f;
            if (f.row_ss) {
                float ss = 0.f;
#pragma unroll
                for (int i = 0; i < 16; ++i) ss += i < f.ss_splits ? sst[i] : 0.f;
                for (int s0 = 16; s0 < f.ss_splits; s0 += 16) {
                    float part[16];
#pragma unroll
                    for (int i = 0; i < 16; ++i) part[i] = f.row_ss[min(s0 + i, f.ss_splits - 1) * n_tokens + tok];
#pragma unroll
                    for (int i = 0; i < 16; ++i) ss += s0 + i < f.ss_splits ? part[i] : 0.f;
                }
                row_scale = inv_rms(ss, f.inv_hidden, f.eps);
            }
            if (static_cast<int>(threadIdx.x) < n_items) item_finish(threadIdx.x, first, row_scale);
            for (int it = threadIdx.x + blockDim.x; it < n_items; it += blockDim.x) {
                Item r;
                item_load(it, r);
                item_finish(it, r, row_scale);
            }
            __syncthreads();
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) {
                const uint4 v = valid ? *reinterpret_cast<const uint4*>(q_lds + lj * HD + kd * 32 + lg * 8)
                                      : uint4{0u, 0u, 0u, 0u};
                q[kd] = __builtin_bit_cast(bf16x8, v);
            }
        }
    };

    f32x4 o[DT];
#pragma unroll
    for (int d = 0; d < DT; ++d) o[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    // Every wavefront goes through the body at least once (one with no keys loads nothing and multiplies
    // nothing): the fused variant's queries are made there, behind the first round's loads, with a barrier.
    int kb0 = w_begin;
    do {
        load_round(kb0);
        if (kb0 == w_begin) {
            make_q();
        }
        if constexpr (FUSED) {
            // the new token's key and value come from LDS, not from the cache line that was just written
            if (writer && kb0 <= kb_end - 1 && kb_end - 1 < min(w_end, kb0 + PF)) {
                const int i_new = kb_end - 1 - kb0;
#pragma unroll
                for (int i = 0; i < PF; ++i) {
                    if (i != i_new) continue;
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt) {
                        const int key0 = (kb0 + i) * 32 + kt * 16;
                        if (key0 + lj == p) {
#pragma unroll
                            for (int kd = 0; kd < KD; ++kd)
                                kk[i][kt][kd] = *reinterpret_cast<const uint4*>(k_lds + kd * 32 + lg * 8);
                        }
                        const int e = p - (key0 + lg * 4);          // which of this lane's four keys, if any
                        if (e >= 0 && e < 4) {
#pragma unroll
                            for (int d = 0; d < DT; ++d) {
                                const uint32_t nv = v_lds[d * 16 + lj].bits;
                                uint32_t& word = (e < 2) ? vv[i][kt][d].x : vv[i][kt][d].y;
                                word = (e & 1) ? ((word & 0x0000ffffu) | (nv << 16)) : ((word & 0xffff0000u) | nv);
                            }
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < PF; ++i) {
            if (kb0 + i >= w_end) break;
            float s[2][4];
            float mx = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kd = 0; kd < KD; ++kd)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kk[i][kt][kd]), q[kd], acc,
                                                                  0, 0, 0);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int key = (kb0 + i) * 32 + kt * 16 + lg * 4 + v;
                    const bool vis = valid && key <= p && key >= lo;
                    s[kt][v] = vis ? acc[v] * scale : -INFINITY;
                    mx = fmaxf(mx, s[kt][v]);
                }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
            mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
            const float m_new = fmaxf(m_run, mx);
            const bool none = m_new == -INFINITY;
            const float alpha = none ? 1.f : __expf(m_run - m_new);
            float sum = 0.f;
            bf16x8 pb;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float pv = none ? 0.f : __expf(s[kt][v] - m_new);
                    sum += pv;
                    pb[kt * 4 + v] = static_cast<__bf16>(pv);
                }
            l_run = l_run * alpha + sum;
            m_run = m_new;
#pragma unroll
            for (int d = 0; d < DT; ++d) {
                const uint4 av = uint4{vv[i][0][d].x, vv[i][0][d].y, vv[i][1][d].x, vv[i][1][d].y};
                f32x4 acc = o[d];
                acc[0] *= alpha; acc[1] *= alpha; acc[2] *= alpha; acc[3] *= alpha;
                o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), pb, acc, 0, 0, 0);
            }
        }
        kb0 += PF;
    } while (kb0 < w_end);
    float l = l_run;
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);

    // every wavefront leaves its state in LDS; then all threads combine
    float* mine = wave_state + (wave * 16 + lj) * kRow;
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
        for (int v = 0; v < 4; ++v) mine[d * 16 + lg * 4 + v] = o[d][v];
    if (lg == 0) {
        mine[HD] = m_run;
        mine[HD + 1] = l;
    }
    __syncthreads();
    const size_t row0 = static_cast<size_t>(tok) * nq + kh * group_size;
    for (int idx = threadIdx.x; idx < group_size * HD; idx += blockDim.x) {
        const int r = idx / HD, d = idx % HD;
        float mx = -INFINITY;
        for (int w = 0; w < n_waves; ++w) mx = fmaxf(mx, wave_state[(w * 16 + r) * kRow + HD]);
        float num = 0.f, den = 0.f;
        for (int w = 0; w < n_waves; ++w) {
            const float* st = wave_state + (w * 16 + r) * kRow;
            const float wgt = st[HD] == -INFINITY ? 0.f : __expf(st[HD] - mx);
            num += wgt * st[d];
            den += wgt * st[HD + 1];
        }
        if (n_splits == 1) {
            out[(row0 + r) * HD + d] = from_float<bf16_t>(num / den);
        } else {
            const size_t prow = static_cast<size_t>(split) * n_tokens * nq +
                                (MIXED ? static_cast<size_t>(b) * nq + kh * group_size : row0) + r;
            part_o[prow * HD + d] = num;
            if (d == 0) {
                part_ml[prow * 2] = mx;
                part_ml[prow * 2 + 1] = den;
            }
        }
    }
}

// out[row, :] = sum_s exp(m_s - M) o_s / sum_s exp(m_s - M) l_s over the splits; one wavefront per row.
// Lane s first takes split s's (maximum, sum) so that the weights of up to 64 splits are known after one
// round of loads; the partial outputs are then read eight splits at a time.
__global__ __launch_bounds__(64) void attention_reduce_kernel(const float* __restrict__ part_o,
                                                              const float* __restrict__ part_ml,
                                                              bf16_t* __restrict__ out, int n_rows, int hd, int n_splits,
                                                              const int32_t* __restrict__ q_start = nullptr,
                                                              const int32_t* __restrict__ q_len = nullptr, int nq = 1) {
    const int row = blockIdx.x, lane = threadIdx.x;
    // q_start given: the parts are kept by request, of which only those of one token have any, and the result goes
    // to that token's row
    int out_row = row;
    if (q_start != nullptr) {
        const int seq = row / nq;
        if (q_len[seq] != 1) return;
        out_row = q_start[seq] * nq + row % nq;
    }
    // the first eight splits' parts are asked for together with their weights' inputs, not behind them (a part of a
    // split without visible keys may hold anything: it is read and then dropped)
    float first[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const size_t pr = static_cast<size_t>(min(i, n_splits - 1)) * n_rows + row;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int d = lane + r * kWave;
            first[i][r] = d < hd ? part_o[pr * hd + d] : 0.f;
        }
    }
    float m = -INFINITY, l = 0.f;
    if (lane < n_splits) {
        const size_t pr = static_cast<size_t>(lane) * n_rows + row;
        m = part_ml[pr * 2];
        l = part_ml[pr * 2 + 1];
    }
    const float m_max = wave_max(m);
    const float wgt = m == -INFINITY ? 0.f : __expf(m - m_max);    // a split without visible keys weighs nothing
    const float inv = 1.0f / wave_sum(wgt * l);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < n_splits; s0 += 8) {
        float v[8][4], w8[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int s = s0 + i;
            w8[i] = __shfl(wgt, s < n_splits ? s : 0, kWave);
            if (s >= n_splits) w8[i] = 0.f;
            const size_t pr = static_cast<size_t>(s < n_splits ? s : 0) * n_rows + row;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int d = lane + r * kWave;
                if (s0 == 0) v[i][r] = w8[i] != 0.f ? first[i][r] : 0.f;
                else v[i][r] = (d < hd && w8[i] != 0.f) ? part_o[pr * hd + d] : 0.f;
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] += w8[i] * v[i][r];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int d = lane + r * kWave;
        if (d < hd) out[static_cast<size_t>(out_row) * hd + d] = from_float<bf16_t>(acc[r] * inv);
    }
}

template <int HD, int QT>
static int launch_mfma(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                       const void* v_cache, const int32_t* block_table, int table_width, const int32_t* q_start,
                       const int32_t* q_len, const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv,
                       int page_size, float scale, int window, int n_splits, int combine, hipStream_t s) {
    const int group = nq / nkv;
    const long groups = (static_cast<long>(n_tokens) * group) / (16 * QT) + n_seqs;   // upper bound
    dim3 grid(static_cast<unsigned>(groups), nkv, n_splits);
    attention_mfma_kernel<HD, QT><<<grid, 64, 0, s>>>(
        static_cast<const bf16_t*>(qkv), static_cast<bf16_t*>(out), part_o, part_ml,
        static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache), block_table, table_width, q_start,
        q_len, kv_len, n_seqs, n_tokens, nq, nkv, page_size, scale, window, n_splits);
    EGPT_CHECK_LAUNCH();
    if (n_splits > 1 && combine) {
        attention_reduce_kernel<<<n_tokens * nq, 64, 0, s>>>(part_o, part_ml, static_cast<bf16_t*>(out), n_tokens * nq,
                                                             HD, n_splits);
        EGPT_CHECK_LAUNCH();
    }
    return EGPT_OK;
}

constexpr int kDecodeLdsMost = 96 * 1024;       // bytes of LDS a workgroup of the decode kernel may ask for

// PF: key blocks per round of loads of a wavefront.  More of them in flight is fewer round trips but more
// registers; when there are so many workgroups that they must share CUs, fewer registers are worth more.
template <int HD, int PF>
static int launch_decode(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                         const void* v_cache, const int32_t* block_table, int table_width, const int32_t* q_start,
                         const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv, int page_size, float scale,
                         int window, int n_splits, int n_waves, int combine, const FusedQkv* fused,
                         const int32_t* q_len, hipStream_t s) {
    dim3 grid(n_seqs, nkv, n_splits);
    size_t lds = static_cast<size_t>(n_waves) * 16 * (HD + 2) * sizeof(float);
    if (fused) lds += 18 * HD * sizeof(bf16_t);          // 16 query heads, the new key and value
    if (lds > kDecodeLdsMost) return EGPT_UNSUPPORTED_SIZE;
    if (lds > 64 * 1024) {
        // (eight wavefronts at head size 128: more than a kernel may take without being asked; once per instance)
        static bool raised_fused = false, raised_plain = false, raised_mixed = false;
        bool& raised = fused ? raised_fused : q_len ? raised_mixed : raised_plain;
        if (!raised) {
            const void* fn = fused   ? reinterpret_cast<const void*>(&attention_decode_kernel<HD, PF, true>)
                             : q_len ? reinterpret_cast<const void*>(&attention_decode_kernel<HD, PF, false, true>)
                                     : reinterpret_cast<const void*>(&attention_decode_kernel<HD, PF, false>);
            if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kDecodeLdsMost) != hipSuccess)
                return EGPT_UNSUPPORTED_SIZE;
            raised = true;
        }
    }
    FusedQkv fq = fused ? *fused : FusedQkv{};
    if (fused)
        attention_decode_kernel<HD, PF, true><<<grid, n_waves * kWave, lds, s>>>(
            nullptr, static_cast<bf16_t*>(out), part_o, part_ml, static_cast<const bf16_t*>(k_cache),
            static_cast<const bf16_t*>(v_cache), block_table, table_width, q_start, kv_len, n_tokens, nq, nkv,
            page_size, scale, window, n_splits, fq, nullptr);
    else if (q_len)
        attention_decode_kernel<HD, PF, false, true><<<grid, n_waves * kWave, lds, s>>>(
            static_cast<const bf16_t*>(qkv), static_cast<bf16_t*>(out), part_o, part_ml,
            static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache), block_table, table_width, q_start,
            kv_len, n_tokens, nq, nkv, page_size, scale, window, n_splits, fq, q_len);
    else
        attention_decode_kernel<HD, PF, false><<<grid, n_waves * kWave, lds, s>>>(
            static_cast<const bf16_t*>(qkv), static_cast<bf16_t*>(out), part_o, part_ml,
            static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache), block_table, table_width, q_start,
            kv_len, n_tokens, nq, nkv, page_size, scale, window, n_splits, fq, nullptr);
    EGPT_CHECK_LAUNCH();
    if (n_splits > 1 && combine) {
        attention_reduce_kernel<<<n_tokens * nq, 64, 0, s>>>(part_o, part_ml, static_cast<bf16_t*>(out), n_tokens * nq,
                                                             HD, n_splits, q_len ? q_start : nullptr, q_len, nq);
        EGPT_CHECK_LAUNCH();
    }
    return EGPT_OK;
}

static int dispatch_decode(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                           const void* v_cache, const int32_t* block_table, int table_width, const int32_t* q_start,
                           const int32_t* kv_len, int n_seqs, int nq, int nkv, int hd, int page_size, float scale,
                           int window, int n_splits, int n_waves, int combine, bool lean, const FusedQkv* fused,
                           const int32_t* q_len, hipStream_t s) {
    // lean: the variant with half the loads in flight and fewer registers (the caller's choice, see the wrapper)
#define EGPT_LAUNCH_DECODE(HD_, PF_)                                                                                \
    launch_decode<HD_, PF_>(qkv, out, part_o, part_ml, k_cache, v_cache, block_table, table_width, q_start, kv_len, \
                            n_seqs, n_seqs, nq, nkv, page_size, scale, window, n_splits, n_waves, combine, fused,   \
                            q_len, s)
    if (hd == 64) return lean ? EGPT_LAUNCH_DECODE(64, 2) : EGPT_LAUNCH_DECODE(64, 4);
    return lean ? EGPT_LAUNCH_DECODE(128, 1) : EGPT_LAUNCH_DECODE(128, 2);
#undef EGPT_LAUNCH_DECODE
}

}  // namespace egpt

using namespace egpt;

// Prompt portions (and mixed batches) with keys and values shared through LDS by the wavefronts of a
// workgroup.  Same operands and meaning as egpt_paged_attention_mfma with n_splits == 1; page sizes that are
// powers of two.  `shape` = 10 * (tiles of 16 rows per workgroup) + (wavefronts that split a tile's keys).
template <int HD, int RT, int KS>
static void launch_tiled(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                         const int32_t* block_table, int table_width, const int32_t* q_start, const int32_t* q_len,
                         const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv, int page_size,
                         int page_shift, float scale, int window, int skip_single, hipStream_t s) {
    const long groups = (static_cast<long>(n_tokens) * (nq / nkv)) / (16 * RT) + n_seqs;   // upper bound
    dim3 grid(static_cast<unsigned>(groups), nkv);
    attention_tiled_kernel<HD, RT, KS><<<grid, 64 * RT * KS, 0, s>>>(
        static_cast<const bf16_t*>(qkv), static_cast<bf16_t*>(out), static_cast<const bf16_t*>(k_cache),
        static_cast<const bf16_t*>(v_cache), block_table, table_width, q_start, q_len, kv_len, n_seqs, nq, nkv,
        page_size, page_shift, scale, window, skip_single);
}

template <int HD, int RB, int KS>
static void launch_rows32(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                          const int32_t* block_table, int table_width, const int32_t* q_start, const int32_t* q_len,
                          const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv, int page_size,
                          int page_shift, float scale, int window, int skip_single, float* part_o, float* part_ml,
                          int n_splits, hipStream_t s) {
    const long groups = (static_cast<long>(n_tokens) * (nq / nkv)) / (32 * RB) + n_seqs;   // upper bound
    dim3 grid(static_cast<unsigned>(groups), nkv, n_splits);
#define EGPT_ROWS32_ARGS                                                                                           \
    static_cast<const bf16_t*>(qkv), static_cast<bf16_t*>(out), static_cast<const bf16_t*>(k_cache),               \
        static_cast<const bf16_t*>(v_cache), block_table, table_width, q_start, q_len, kv_len, n_seqs, nq, nkv,    \
        page_size, page_shift, scale, window, skip_single, part_o, part_ml, n_splits, n_tokens
    if (n_splits > 1) attention_rows32_kernel<HD, RB, KS, true><<<grid, 64 * RB * KS, 0, s>>>(EGPT_ROWS32_ARGS);
    else attention_rows32_kernel<HD, RB, KS, false><<<grid, 64 * RB * KS, 0, s>>>(EGPT_ROWS32_ARGS);
#undef EGPT_ROWS32_ARGS
    // (the rows of requests that were left out have no parts: what is combined for them is written over by the
    // kernel that takes them, which runs behind this one)
    if (n_splits > 1)
        attention_reduce_kernel<<<n_tokens * nq, 64, 0, s>>>(part_o, part_ml, static_cast<bf16_t*>(out), n_tokens * nq,
                                                             HD, n_splits);
}

extern "C" int egpt_paged_attention_tiled(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                                          const int32_t* block_table, int table_width, const int32_t* q_start,
                                          const int32_t* q_len, const int32_t* kv_len, int n_seqs, int n_tokens,
                                          int nq, int nkv, int hd, int page_size, float scale, int window,
                                          int shape, int key_splits, float* part_o, float* part_ml,
                                          int single_splits, int single_waves, int single_lean, void* stream) {
    if (!qkv || !out || !k_cache || !v_cache || !block_table || !q_start || !q_len || !kv_len)
        return EGPT_BAD_ARGUMENT;
    if (n_seqs <= 0 || n_tokens < 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || table_width <= 0 || window < 0)
        return EGPT_BAD_ARGUMENT;
    if ((hd != 64 && hd != 128) || page_size < 16 || (page_size & (page_size - 1)) != 0 || nkv > 65535)
        return EGPT_UNSUPPORTED_SIZE;
    const int skip_single = single_waves != 0;
    if (skip_single) {
        if (single_waves < 0 || single_splits < 1 || (single_splits > 1 && (!part_o || !part_ml)))
            return EGPT_BAD_ARGUMENT;
        if (nq / nkv > 16 || single_splits > 64 || single_waves > 8) return EGPT_UNSUPPORTED_SIZE;
    }
    if (shape >= 100 && page_size > 64) return EGPT_UNSUPPORTED_SIZE;     // its tiles of 64 keys are whole pages
    if (key_splits < 1 || (key_splits > 1 && (!part_o || !part_ml))) return EGPT_BAD_ARGUMENT;
    if (key_splits > 64 || (key_splits > 1 && shape < 100)) return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    hipStream_t s = static_cast<hipStream_t>(stream);
#define EGPT_TILED(HD_, RT_, KS_)                                                                                  \
    launch_tiled<HD_, RT_, KS_>(qkv, out, k_cache, v_cache, block_table, table_width, q_start, q_len, kv_len,      \
                                n_seqs, n_tokens, nq, nkv, page_size, page_shift, scale, window, skip_single, s)
#define EGPT_ROWS32(HD_, RB_, KS_)                                                                                 \
    launch_rows32<HD_, RB_, KS_>(qkv, out, k_cache, v_cache, block_table, table_width, q_start, q_len, kv_len,     \
                                 n_seqs, n_tokens, nq, nkv, page_size, page_shift, scale, window, skip_single,     \
                                 part_o, part_ml, key_splits, s)
    // shape = 10 * row tiles + key splits of a workgroup; 100 + 10 * blocks of 32 rows + key splits: the kernel of
    // 32-row blocks
    if (hd == 64) {
        switch (shape) {
            case 121: EGPT_ROWS32(64, 2, 1); break;
            case 122: EGPT_ROWS32(64, 2, 2); break;
            case 124: EGPT_ROWS32(64, 2, 4); break;
            case 141: EGPT_ROWS32(64, 4, 1); break;
            case 142: EGPT_ROWS32(64, 4, 2); break;
            case 41: EGPT_TILED(64, 4, 1); break;
            case 42: EGPT_TILED(64, 4, 2); break;
            case 44: EGPT_TILED(64, 4, 4); break;
            case 22: EGPT_TILED(64, 2, 2); break;
            case 24: EGPT_TILED(64, 2, 4); break;
            default: return EGPT_BAD_ARGUMENT;
        }
    } else {
        switch (shape) {
            case 121: EGPT_ROWS32(128, 2, 1); break;
            case 122: EGPT_ROWS32(128, 2, 2); break;
            case 141: EGPT_ROWS32(128, 4, 1); break;
            case 41: EGPT_TILED(128, 4, 1); break;
            case 42: EGPT_TILED(128, 4, 2); break;
            case 22: EGPT_TILED(128, 2, 2); break;
            default: return EGPT_BAD_ARGUMENT;
        }
    }
#undef EGPT_TILED
#undef EGPT_ROWS32
    EGPT_CHECK_LAUNCH();
    if (skip_single)
        return dispatch_decode(qkv, out, part_o, part_ml, k_cache, v_cache, block_table, table_width, q_start, kv_len,
                               n_seqs, nq, nkv, hd, page_size, scale, window, single_splits, single_waves, 1,
                               single_lean != 0, nullptr, q_len, s);
    return EGPT_OK;
}

// One decoded token per request (n_tokens == n_seqs, q_len all 1), nq / nkv <= 16: workgroups of n_waves
// wavefronts (1..8) per (request, kv head, key split).  Same operands and meaning as egpt_paged_attention_mfma.
extern "C" int egpt_paged_attention_decode(const void* qkv, void* out, float* part_o, float* part_ml,
                                           const void* k_cache, const void* v_cache, const int32_t* block_table,
                                           int table_width, const int32_t* q_start, const int32_t* kv_len, int n_seqs,
                                           int nq, int nkv, int hd, int page_size, float scale, int window,
                                           int n_splits, int n_waves, int combine, int lean, void* stream) {
    if (!qkv || !out || !k_cache || !v_cache || !block_table || !q_start || !kv_len) return EGPT_BAD_ARGUMENT;
    if (n_seqs <= 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || table_width <= 0 || window < 0 || n_splits < 1 ||
        (n_splits > 1 && (!part_o || !part_ml)))
        return EGPT_BAD_ARGUMENT;
    if ((hd != 64 && hd != 128) || page_size % 16 != 0 || nq / nkv > 16 || nkv > 65535 || n_splits > 64 ||
        n_waves < 1 || n_waves > 8)
        return EGPT_UNSUPPORTED_SIZE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dispatch_decode(qkv, out, part_o, part_ml, k_cache, v_cache, block_table, table_width, q_start, kv_len,
                           n_seqs, nq, nkv, hd, page_size, scale, window, n_splits, n_waves, combine, lean != 0, nullptr, nullptr, s);
}

// The same with the QKV epilogue folded in: the queries, and the new token's key and value, are computed from
// the float32 QKV product (partial sums qkv_prod [in_splits][n_seqs][(nq + 2 nkv) * hd], the rows' sums of
// squares row_ss [ss_splits][n_seqs] or null, bias or null), rotated over the whole head by the angles whose
// cosines and sines are in cos_sin [n_seqs][hd / 2][2] (egpt_rope_table), and the key and value are stored at
// slots[t] of the caches.  Token t belongs to request t.
extern "C" int egpt_attention_decode_fused(const float* qkv_prod, int in_splits, const float* row_ss, int ss_splits,
                                           int hidden, float eps, const void* bias, const float* cos_sin,
                                           const int32_t* slots, void* out, float* part_o,
                                           float* part_ml, void* k_cache, void* v_cache, const int32_t* block_table,
                                           int table_width, const int32_t* q_start, const int32_t* kv_len, int n_seqs,
                                           int nq, int nkv, int hd, int page_size, float scale, int window,
                                           int n_splits, int n_waves, int combine, int lean, void* stream) {
    if (!qkv_prod || in_splits < 1 || !cos_sin || !slots || !out || !k_cache || !v_cache ||
        !block_table || !q_start || !kv_len || (row_ss && (ss_splits < 1 || hidden < 1)))
        return EGPT_BAD_ARGUMENT;
    if (n_seqs <= 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || table_width <= 0 || window < 0 || n_splits < 1 ||
        (n_splits > 1 && (!part_o || !part_ml)))
        return EGPT_BAD_ARGUMENT;
    if ((hd != 64 && hd != 128) || page_size % 16 != 0 || nq / nkv > 16 || nkv > 65535 || n_splits > 64 ||
        n_waves < 1 || n_waves > 8)
        return EGPT_UNSUPPORTED_SIZE;
    FusedQkv f = {};
    f.prod = qkv_prod; f.in_splits = in_splits;
    f.row_ss = row_ss; f.ss_splits = row_ss ? ss_splits : 0;
    f.inv_hidden = row_ss ? 1.0f / static_cast<float>(hidden) : 0.f;
    f.eps = eps;
    f.bias = static_cast<const bf16_t*>(bias);
    f.cos_sin = cos_sin; f.slots = slots;
    f.k_cache_w = static_cast<bf16_t*>(k_cache); f.v_cache_w = static_cast<bf16_t*>(v_cache);
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dispatch_decode(nullptr, out, part_o, part_ml, k_cache, v_cache, block_table, table_width, q_start, kv_len,
                           n_seqs, nq, nkv, hd, page_size, scale, window, n_splits, n_waves, combine, lean != 0, &f, nullptr, s);
}

// bfloat16 only; head size 64 or 128; page size a multiple of 16.  rows_per_wave: 16 (decoded tokens) or 32.
// part_o [n_splits][n_tokens][nq][hd] and part_ml [n_splits][n_tokens][nq][2] float32 are needed when n_splits > 1;
// with combine == 0 they are left for the caller to combine (the output projection does it while it stages x).
extern "C" int egpt_paged_attention_mfma(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                                         const void* v_cache, const int32_t* block_table, int table_width,
                                         const int32_t* q_start, const int32_t* q_len, const int32_t* kv_len,
                                         int n_seqs, int n_tokens, int nq, int nkv, int hd, int page_size, float scale,
                                         int window, int n_splits, int rows_per_wave, int combine, void* stream) {
    if (!qkv || !out || !k_cache || !v_cache || !block_table || !q_start || !q_len || !kv_len)
        return EGPT_BAD_ARGUMENT;
    if (n_seqs <= 0 || n_tokens < 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || table_width <= 0 || window < 0 ||
        n_splits < 1 || (n_splits > 1 && (!part_o || !part_ml)))
        return EGPT_BAD_ARGUMENT;
    if ((hd != 64 && hd != 128) || page_size % 16 != 0 || nkv > 65535 || n_splits > 64 ||
        (rows_per_wave != 16 && rows_per_wave != 32))
        return EGPT_UNSUPPORTED_SIZE;
    if (n_tokens == 0) return EGPT_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
#define EGPT_ATTN_ARGS                                                                                              \
    qkv, out, part_o, part_ml, k_cache, v_cache, block_table, table_width, q_start, q_len, kv_len, n_seqs, n_tokens, \
        nq, nkv, page_size, scale, window, n_splits, combine, s
    if (hd == 64) return rows_per_wave == 16 ? launch_mfma<64, 1>(EGPT_ATTN_ARGS) : launch_mfma<64, 2>(EGPT_ATTN_ARGS);
    return rows_per_wave == 16 ? launch_mfma<128, 1>(EGPT_ATTN_ARGS) : launch_mfma<128, 2>(EGPT_ATTN_ARGS);
#undef EGPT_ATTN_ARGS
}

// Combines the parts that egpt_paged_attention_mfma left with combine == 0: out [n_rows][hd] bfloat16.
extern "C" int egpt_attention_combine(const float* part_o, const float* part_ml, void* out, int n_rows, int hd,
                                      int n_splits, void* stream) {
    if (!part_o || !part_ml || !out || n_rows < 0 || hd <= 0 || n_splits < 1) return EGPT_BAD_ARGUMENT;
    if (n_splits > 64 || hd > 256) return EGPT_UNSUPPORTED_SIZE;
    if (n_rows == 0) return EGPT_OK;
    attention_reduce_kernel<<<n_rows, 64, 0, static_cast<hipStream_t>(stream)>>>(part_o, part_ml,
                                                                               static_cast<bf16_t*>(out), n_rows, hd,
                                                                               n_splits);
    EGPT_CHECK_LAUNCH();
    return EGPT_OK;
}
