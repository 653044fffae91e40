// Attention whose softmax weights are mixed across heads, over the paged cache, for any mix of query tokens
// (prompt portions and single decoded tokens alike), any head sizes up to 256 and both storage types.
//
//   q, k  RMS-normed over their WHOLE projection (all heads of a token at once), plain weights
//   score_h(i, j) = scale * q_h(i) . k_c(j) - r1_h * ln(1 + r2_h * (i - j)),   c = h / (heads / kv heads)
//   i sees j <= i when i - j < window (window 0: every key) or j < keep_first
//   p_h(i, j) = exp(score_h(i, j)) / (exp(sink_h) + sum_j' exp(score_h(i, j')))
//   p'_h = sum_g mix[h, g] p_g;  o_h(i) = sum_j p'_h(i, j) v_c(j);  out = o * sigmoid(gate)
//
// Keys and values have sizes of their own (d and dv).  Scores, softmax, the mixing and all sums are float32.
// Keys lie in the cache as [page][kv head][slot][d]; values transposed inside a page, [page][kv head][dv][slot]
// (the same bytes a page: the matrix-core form reads eight keys of one value column as sixteen contiguous bytes).
//
// Two kernels: `mixed_prepare_kernel` norms q and k of every token of a step, keeps q and writes k and v into
// their pages; `mixed_attention_kernel` (this file's plain form: one workgroup a token, the float32 path's kernel
// and the fallback of shapes the matrix-core forms refuse) walks the keys a token sees twice: once for every head's
// maximum and denominator, once more for the weights themselves, which are then final, so the heads can be mixed
// key tile by key tile before they meet the values.  Keys are taken in tiles of 64 aligned to the absolute key index
// (the kept first keys and the window as two runs), so a token's sequence of operations follows from its own
// position alone, never from what else is in the batch.
#include "common.h"
#include <math.h>

#define MIXED_THREADS 256
#define MIXED_WAVES (MIXED_THREADS / KIPP_WAVE)
#define MIXED_MAX_D 256
#define MIXED_MAX_HEADS 64
#define MIXED_HPW (MIXED_MAX_HEADS / MIXED_WAVES)      // heads a wave carries at most

// proj [n, stride] float32 holds a token's projections: q at column 0 (n_q * d), k at `k_at` (n_kv * d), v at `v_at`
// (n_kv * dv).  One workgroup a token.  Values are written transposed inside their page.
template <typename TQ, typename TC>
__global__ void __launch_bounds__(MIXED_THREADS) mixed_prepare_kernel(
    const float* __restrict__ proj, int parts, size_t part_stride, int stride, int k_at, int v_at,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    TQ* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks, int n_q, int n_kv, int d, int dv, int page, int write_kv) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const float* row = proj + (size_t)t * stride;
    const int q_dim = n_q * d, k_dim = n_kv * d, v_dim = n_kv * dv;
    float ss_q = 0.0f, ss_k = 0.0f;
    for (int e = threadIdx.x; e < q_dim; e += MIXED_THREADS) {
        float v = 0.0f;
        for (int p = 0; p < parts; ++p) v += row[p * part_stride + e];
        ss_q = fmaf(v, v, ss_q);
    }
    for (int e = threadIdx.x; e < k_dim; e += MIXED_THREADS) {
        float v = 0.0f;
        for (int p = 0; p < parts; ++p) v += row[p * part_stride + k_at + e];
        ss_k = fmaf(v, v, ss_k);
    }
    ss_q = block_sum(ss_q, scratch);
    ss_k = block_sum(ss_k, scratch);
    const float scale_q = 1.0f / sqrtf(ss_q / (float)q_dim + eps);
    const float scale_k = 1.0f / sqrtf(ss_k / (float)k_dim + eps);
    for (int e = threadIdx.x; e < q_dim; e += MIXED_THREADS) {
        float v = 0.0f;
        for (int p = 0; p < parts; ++p) v += row[p * part_stride + e];
        store_f(q_out, (size_t)t * q_dim + e, v * scale_q * q_weight[e]);
    }
    if (!write_kv) return;
    const int pos = positions[t];
    const int page_id = block_table[(size_t)seq_of_token[t] * max_blocks + pos / page];
    const int slot = pos % page;
    for (int e = threadIdx.x; e < k_dim; e += MIXED_THREADS) {
        float v = 0.0f;
        for (int p = 0; p < parts; ++p) v += row[p * part_stride + k_at + e];
        const int g = e / d, i = e - g * d;
        store_f(k_cache, (((size_t)page_id * n_kv + g) * page + slot) * d + i, v * scale_k * k_weight[e]);
    }
    for (int e = threadIdx.x; e < v_dim; e += MIXED_THREADS) {
        float v = 0.0f;
        for (int p = 0; p < parts; ++p) v += row[p * part_stride + v_at + e];
        const int g = e / dv, i = e - g * dv;
        store_f(v_cache, (((size_t)page_id * n_kv + g) * dv + i) * page + slot, v);      // transposed inside the page
    }
}

// The same with a token's sums staged in LDS (dynamic, n_q d + n_kv d + n_kv dv floats): the slabs are read once, four
// at a time, and every value is normed or written from LDS; few tokens get workgroups of 1,024 threads (the sums of
// squares then add up in another order: the float32 path, whose bits must not depend on the batch, stays at 256).
// The order of a token's additions follows from the sizes alone.
template <typename TQ, typename TC>
__global__ void __launch_bounds__(1024) mixed_prepare_lds_kernel(
    const float* __restrict__ proj, int parts, size_t part_stride, int stride, int k_at, int v_at,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    TQ* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks, int n_q, int n_kv, int d, int dv, int page, int write_kv) {
    extern __shared__ __attribute__((aligned(16))) float sums[];
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const float* row = proj + (size_t)t * stride;
    const int q_dim = n_q * d, k_dim = n_kv * d, v_dim = n_kv * dv;
    const int total = q_dim + k_dim + v_dim;
    float ss_q = 0.0f, ss_k = 0.0f;
    if (((q_dim | k_dim | v_dim | k_at | v_at | stride) & 3) == 0) {
        // four columns a lane and load (every run of columns begins at a multiple of four, so a group never straddles two)
        for (int e = 4 * threadIdx.x; e < total; e += 4 * blockDim.x) {
            const int col = e < q_dim ? e : (e < q_dim + k_dim ? k_at + e - q_dim : v_at + e - q_dim - k_dim);
            float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            for (int p0 = 0; p0 < parts; p0 += 4) {
                float4 part[4];
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    part[u] = p0 + u < parts ? *(const float4*)(row + (p0 + u) * part_stride + col) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    v.x += part[u].x;
                    v.y += part[u].y;
                    v.z += part[u].z;
                    v.w += part[u].w;
                }
            }
            *(float4*)(sums + e) = v;
            const float sq = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, v.w * v.w)));
            if (e < q_dim) ss_q += sq;
            else if (e < q_dim + k_dim) ss_k += sq;
        }
    } else {
        for (int e = threadIdx.x; e < total; e += blockDim.x) {
            const int col = e < q_dim ? e : (e < q_dim + k_dim ? k_at + e - q_dim : v_at + e - q_dim - k_dim);
            float v = 0.0f;
            for (int p0 = 0; p0 < parts; p0 += 4) {
                float part[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) part[u] = p0 + u < parts ? row[(p0 + u) * part_stride + col] : 0.0f;
#pragma unroll
                for (int u = 0; u < 4; ++u) v += part[u];
            }
            sums[e] = v;
            if (e < q_dim) ss_q = fmaf(v, v, ss_q);
            else if (e < q_dim + k_dim) ss_k = fmaf(v, v, ss_k);
        }
    }
    ss_q = block_sum(ss_q, scratch);
    ss_k = block_sum(ss_k, scratch);
    const float scale_q = 1.0f / sqrtf(ss_q / (float)q_dim + eps);
    const float scale_k = 1.0f / sqrtf(ss_k / (float)k_dim + eps);
    const int pos = positions[t];
    const int page_id = write_kv ? block_table[(size_t)seq_of_token[t] * max_blocks + pos / page] : 0;
    const int slot = pos % page;
    for (int e = threadIdx.x; e < (write_kv ? total : q_dim); e += blockDim.x) {
        const float v = sums[e];
        if (e < q_dim) {
            store_f(q_out, (size_t)t * q_dim + e, v * scale_q * q_weight[e]);
        } else if (e < q_dim + k_dim) {
            const int c = e - q_dim, g = c / d, i = c - g * d;
            store_f(k_cache, (((size_t)page_id * n_kv + g) * page + slot) * d + i, v * scale_k * k_weight[c]);
        } else {
            const int c = e - q_dim - k_dim, g = c / dv, i = c - g * dv;
            store_f(v_cache, (((size_t)page_id * n_kv + g) * dv + i) * page + slot, v);
        }
    }
}

// One workgroup a token, 4 waves; wave w carries heads w, w + 4, ...  LDS (dynamic): q of every head as float32
// [n_q][d], the tile's weights [n_q][64] before and after the heads are mixed, the tile's page offsets [64], and
// every head's maximum and denominator.
template <typename TQ, typename TC, typename TO>
__global__ void __launch_bounds__(MIXED_THREADS) mixed_attention_kernel(
    const TQ* __restrict__ q, const TC* __restrict__ k_cache, const TC* __restrict__ v_cache, TO* __restrict__ out,
    const float* __restrict__ gate, int gate_stride, int gate_parts, size_t gate_part_stride,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks,
    const float* __restrict__ r1, const float* __restrict__ r2, const float* __restrict__ sink, const float* __restrict__ mix,
    int n_q, int n_kv, int d, int dv, int page, float scale, int window, int keep_first) {
    extern __shared__ float lds[];
    float* q_s = lds;                                   // [n_q][d]
    float* p_s = q_s + (size_t)n_q * d;                 // [n_q][64]
    float* pm_s = p_s + (size_t)n_q * KIPP_WAVE;        // [n_q][64]: the weights after the heads are mixed
    float* m_s = pm_s + (size_t)n_q * KIPP_WAVE;        // [n_q]
    float* l_s = m_s + n_q;                             // [n_q]
    long long* page_s = (long long*)(l_s + n_q + ((n_q & 1) ? 1 : 0));   // [64]: page id * n_kv of the tile's keys
    int* slot_s = (int*)(page_s + KIPP_WAVE);                            // [64]: their slots in the page
    const int wave = threadIdx.x / KIPP_WAVE;
    const int lane = threadIdx.x & (KIPP_WAVE - 1);
    const int t = blockIdx.x;
    const int pos = positions[t];
    const int32_t* table = block_table + (size_t)seq_of_token[t] * max_blocks;
    const int group = n_q / n_kv;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int kept = window > 0 ? min(keep_first, lo) : 0;       // keys [0, kept) and [lo, pos]

    for (int e = threadIdx.x; e < n_q * d; e += MIXED_THREADS) q_s[e] = load_f(q, (size_t)t * n_q * d + e);
    __syncthreads();

    // -- every head's maximum and denominator; the sink is the first member of both
    for (int h = wave; h < n_q; h += MIXED_WAVES) {
        const int c = h / group;
        const float a = r1 != nullptr ? r1[h] : 0.0f, b = r2 != nullptr ? r2[h] : 0.0f;
        float m = sink != nullptr ? sink[h] : -INFINITY, l = sink != nullptr ? 1.0f : 0.0f;
        for (int run = 0; run < 2; ++run) {
            const int from = run == 0 ? 0 : lo, to = run == 0 ? kept - 1 : pos;      // inclusive
            for (int s0 = (from / KIPP_WAVE) * KIPP_WAVE; s0 <= to; s0 += KIPP_WAVE) {
                const int s = s0 + lane;
                float score = -INFINITY;
                if (s >= from && s <= to) {
                    const TC* k_row = k_cache + (((size_t)table[s / page] * n_kv + c) * page + s % page) * d;
                    float dot = 0.0f;
                    for (int e = 0; e < d; ++e) dot = fmaf(q_s[h * d + e], load_f(k_row, e), dot);
                    score = dot * scale - a * log1pf(b * (float)(pos - s));
                }
                const float m_new = fmaxf(m, wave_max(score));
                const float p = score == -INFINITY ? 0.0f : expf(score - m_new);
                l = l * expf(m - m_new) + wave_sum(p);
                m = m_new;
            }
        }
        if (lane == 0) {
            m_s[h] = m;
            l_s[h] = l;
        }
    }
    __syncthreads();

    float acc[MIXED_HPW][MIXED_MAX_D / KIPP_WAVE];
#pragma unroll
    for (int i = 0; i < MIXED_HPW; ++i)
#pragma unroll
        for (int c = 0; c < MIXED_MAX_D / KIPP_WAVE; ++c) acc[i][c] = 0.0f;

    // -- the weights themselves, tile by tile: all heads' weights of a tile, mixed, times the values
    for (int run = 0; run < 2; ++run) {
        const int from = run == 0 ? 0 : lo, to = run == 0 ? kept - 1 : pos;
        for (int s0 = (from / KIPP_WAVE) * KIPP_WAVE; s0 <= to; s0 += KIPP_WAVE) {
            const int s = s0 + lane;
            const bool valid = s >= from && s <= to;
            const long long at = valid ? (long long)table[s / page] * n_kv : 0;
            if (wave == 0) {
                page_s[lane] = at;
                slot_s[lane] = s % page;
            }
            for (int h = wave; h < n_q; h += MIXED_WAVES) {
                const int c = h / group;
                float p = 0.0f;
                if (valid) {
                    const TC* k_row = k_cache + (((size_t)at + c) * page + s % page) * d;
                    float dot = 0.0f;
                    for (int e = 0; e < d; ++e) dot = fmaf(q_s[h * d + e], load_f(k_row, e), dot);
                    const float a = r1 != nullptr ? r1[h] : 0.0f, b = r2 != nullptr ? r2[h] : 0.0f;
                    const float score = dot * scale - a * log1pf(b * (float)(pos - s));
                    p = expf(score - m_s[h]) / l_s[h];
                }
                p_s[h * KIPP_WAVE + lane] = p;
            }
            __syncthreads();
            if (mix != nullptr) {
                for (int h = wave; h < n_q; h += MIXED_WAVES) {
                    float pm = 0.0f;
                    for (int g = 0; g < n_q; ++g) pm = fmaf(mix[h * n_q + g], p_s[g * KIPP_WAVE + lane], pm);
                    pm_s[h * KIPP_WAVE + lane] = pm;
                }
                __syncthreads();
            }
            const float* w_s = mix != nullptr ? pm_s : p_s;
            const int j_lo = max(0, from - s0), j_hi = min(KIPP_WAVE, to - s0 + 1);
#pragma unroll
            for (int i = 0; i < MIXED_HPW; ++i) {
                const int h = wave + i * MIXED_WAVES;
                if (h < n_q) {
                    const int c = h / group;
#pragma unroll
                    for (int cc = 0; cc < MIXED_MAX_D / KIPP_WAVE; ++cc) {
                        const int e = lane + cc * KIPP_WAVE;
                        if (e < dv) {
                            float a = acc[i][cc];
                            for (int j = j_lo; j < j_hi; ++j)
                                a = fmaf(w_s[h * KIPP_WAVE + j], load_f(v_cache, (((size_t)page_s[j] + c) * dv + e) * page + slot_s[j]), a);
                            acc[i][cc] = a;
                        }
                    }
                }
            }
            __syncthreads();
        }
    }

#pragma unroll
    for (int i = 0; i < MIXED_HPW; ++i) {
        const int h = wave + i * MIXED_WAVES;
        if (h < n_q) {
#pragma unroll
            for (int cc = 0; cc < MIXED_MAX_D / KIPP_WAVE; ++cc) {
                const int e = lane + cc * KIPP_WAVE;
                if (e < dv) {
                    float o = acc[i][cc];
                    if (gate != nullptr) {
                        float z = 0.0f;
                        for (int p = 0; p < gate_parts; ++p) z += gate[p * gate_part_stride + (size_t)t * gate_stride + h * dv + e];
                        o *= 1.0f / (1.0f + expf(-z));
                    }
                    store_f(out, ((size_t)t * n_q + h) * dv + e, o);
                }
            }
        }
    }
}

extern "C" {

// proj: float32 [parts][n_tokens][stride] whose sum over parts holds q | k | v (and whatever follows) of every token.
int kipp_mixed_prepare(const float* proj, int parts, int stride, int k_at, int v_at, const float* q_weight, const float* k_weight,
                       float eps, void* q_out, int q_dtype, void* k_cache, void* v_cache, int cache_dtype,
                       const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
                       int n_tokens, int n_q, int n_kv, int d, int dv, int page, int write_kv, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (parts < 1 || n_q <= 0 || n_kv <= 0 || d <= 0 || dv <= 0 || page <= 0) return -1;
    const size_t part_stride = (size_t)n_tokens * stride;
    const size_t staged = ((size_t)n_q * d + (size_t)n_kv * d + (size_t)n_kv * dv) * sizeof(float);
#define KIPP_MP(TQ, TC)                                                                                                    \
    do {                                                                                                                   \
        if (staged <= 48 * 1024)                                                                                           \
            hipLaunchKernelGGL((mixed_prepare_lds_kernel<TQ, TC>), dim3(n_tokens), dim3(sizeof(TQ) == 2 && n_tokens <= 256 ? 1024 : 256), staged, stream, proj, \
                               parts, part_stride, stride, k_at, v_at, q_weight, k_weight, eps, (TQ*)q_out, (TC*)k_cache,    \
                               (TC*)v_cache, positions, seq_of_token, block_table, max_blocks, n_q, n_kv, d, dv, page,      \
                               write_kv);                                                                                   \
        else                                                                                                               \
            hipLaunchKernelGGL((mixed_prepare_kernel<TQ, TC>), dim3(n_tokens), dim3(MIXED_THREADS), 0, stream, proj, parts,  \
                               part_stride, stride, k_at, v_at, q_weight, k_weight, eps, (TQ*)q_out, (TC*)k_cache,          \
                               (TC*)v_cache, positions, seq_of_token, block_table, max_blocks, n_q, n_kv, d, dv, page,      \
                               write_kv);                                                                                   \
    } while (0)
    if (q_dtype == KIPP_F32 && cache_dtype == KIPP_F32) KIPP_MP(float, float);
    else if (q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16) KIPP_MP(bf16_t, bf16_t);
    else return -2;
#undef KIPP_MP
    return KIPP_LAUNCH_CHECK();
}

int kipp_mixed_attention_lds_bytes(int n_q, int d) {
    return (int)(((size_t)n_q * d + 2 * (size_t)n_q * KIPP_WAVE + 2 * n_q + (n_q & 1)) * 4 + KIPP_WAVE * 12);
}

int kipp_mixed_attention(const void* q, int q_dtype, const void* k_cache, const void* v_cache, int cache_dtype, void* out, int out_dtype,
                         const float* gate, int gate_stride, int gate_parts,
                         const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
                         const float* r1, const float* r2, const float* sink, const float* mix,
                         int n_tokens, int n_q, int n_kv, int d, int dv, int page, float scale, int window, int keep_first,
                         hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (d > MIXED_MAX_D || dv > MIXED_MAX_D || d <= 0 || dv <= 0 || n_kv <= 0 || n_q % n_kv || n_q > MIXED_MAX_HEADS) return -1;
    const int lds = kipp_mixed_attention_lds_bytes(n_q, d);
    if (lds > 64 * 1024) return -3;
    const size_t gate_part_stride = (size_t)n_tokens * gate_stride;
#define KIPP_MA(TQ, TC, TO)                                                                                                  \
    hipLaunchKernelGGL((mixed_attention_kernel<TQ, TC, TO>), dim3(n_tokens), dim3(MIXED_THREADS), lds, stream, (const TQ*)q,   \
                       (const TC*)k_cache, (const TC*)v_cache, (TO*)out, gate, gate_stride, gate_parts, gate_part_stride,      \
                       positions, seq_of_token, block_table, max_blocks, r1, r2, sink, mix, n_q, n_kv, d, dv, page, scale,     \
                       window, keep_first)
    if (q_dtype == KIPP_F32 && cache_dtype == KIPP_F32 && out_dtype == KIPP_F32) KIPP_MA(float, float, float);
    else if (q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16 && out_dtype == KIPP_BF16) KIPP_MA(bf16_t, bf16_t, bf16_t);
    else return -2;
#undef KIPP_MA
    return KIPP_LAUNCH_CHECK();
}

}  // extern "C"
