// Attention through a latent: the three kernels around the attention itself.
//
// A token keeps ONE row [c | kr] of rank + dr numbers in the paged cache: c, the RMS-normed latent from which
// every head's unrotated key W_uk_h c and value W_uv_h c would be made, and kr, the rotated key part that all
// heads share.  Nothing is expanded: since q_h . (W_uk_h c) = (W_uk_h^T q_h) . c, a head's query is carried
// into the latent's space, the attention runs over the cached rows as they lie (one key/value "head" of rank + dr
// numbers that every query head reads; a value is the first `rank` numbers of its key's row), and a head's
// result sum_j p_j c_j is carried back by W_uv_h.
//
//   prepare  from the input product [dq | dkv | gate] (float32, maybe in slabs): the query latent RMS-normed
//            with its weight (for the product W_uq that follows), c RMS-normed with its weight, kr rotated at
//            the token's position, [c | kr] written into the token's page
//   absorb   from q = W_uq cq [tokens][heads][d + dr] (float32, maybe in slabs):
//            out[t][h] = [ W_uk_h^T q_h[:d] | rot(q_h[d:]) ]  (rank + dr numbers)
//   expand   o[t][h][j] = sigmoid(gate[t][h]) * sum_r lat[t][h][r] * W_uv[h][j][r]
//
// Rotation: of the first `rot_dims` numbers of the rotated part, dimension 2i with dimension 2i + 1, by the
// angle float(position) * freq[i] (float32); cosine and sine are multiplied by `magnitude` (frequency
// scaling that comes with a factor on both).  All arithmetic is float32.
#include "common.h"
#include <math.h>

__device__ __forceinline__ void rotate_pair(float& a, float& b, int pos, float freq, float magnitude) {
    const float angle = (float)pos * freq;
    const float cs = cosf(angle) * magnitude, sn = sinf(angle) * magnitude;
    const float lo = a * cs - b * sn, hi = b * cs + a * sn;
    a = lo;
    b = hi;
}

// One workgroup a token.  LDS: 16 floats for the sums.
template <typename TO, typename TC>
__global__ void latent_prepare_kernel(
    const float* __restrict__ proj, int parts, size_t part_stride, int stride,
    const float* __restrict__ q_norm_w, const float* __restrict__ c_norm_w, float eps,
    TO* __restrict__ cq_out, TC* __restrict__ cache, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ block_table, int max_blocks,
    const float* __restrict__ freq, int rot_dims, float magnitude, int q_rank, int rank, int dr, int page, int write_kv) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const int pos = positions[t];
    const float* src = proj + (size_t)t * stride;
    // the query latent
    float ss = 0.0f;
    for (int e = threadIdx.x; e < q_rank; e += blockDim.x) {
        float v = 0.0f;
        for (int p = 0; p < parts; ++p) v += src[p * part_stride + e];
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    float scale = 1.0f / sqrtf(ss / (float)q_rank + eps);
    for (int e = threadIdx.x; e < q_rank; e += blockDim.x) {
        float v = 0.0f;
        for (int p = 0; p < parts; ++p) v += src[p * part_stride + e];
        store_f(cq_out + (size_t)t * q_rank, e, v * scale * q_norm_w[e]);
    }
    if (!write_kv) return;
    // the key/value latent and the shared rotated part
    src += q_rank;
    ss = 0.0f;
    for (int e = threadIdx.x; e < rank; e += blockDim.x) {
        float v = 0.0f;
        for (int p = 0; p < parts; ++p) v += src[p * part_stride + e];
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    scale = 1.0f / sqrtf(ss / (float)rank + eps);
    const int seq = seq_of_token[t];
    const int page_id = block_table[(size_t)seq * max_blocks + pos / page];
    TC* dst = cache + ((size_t)page_id * page + pos % page) * (rank + dr);
    for (int e = threadIdx.x; e < rank; e += blockDim.x) {
        float v = 0.0f;
        for (int p = 0; p < parts; ++p) v += src[p * part_stride + e];
        store_f(dst, e, v * scale * c_norm_w[e]);
    }
    src += rank;
    for (int i = threadIdx.x; 2 * i < dr; i += blockDim.x) {
        float a = 0.0f, b = 0.0f;
        for (int p = 0; p < parts; ++p) {
            a += src[p * part_stride + 2 * i];
            if (2 * i + 1 < dr) b += src[p * part_stride + 2 * i + 1];
        }
        if (2 * i + 1 < rot_dims) rotate_pair(a, b, pos, freq[i], magnitude);
        store_f(dst, rank + 2 * i, a);
        if (2 * i + 1 < dr) store_f(dst, rank + 2 * i + 1, b);
    }
}

#define TILE_TOKENS 8       // tokens of a workgroup of absorb and of expand: a weight is read once for all of them
#define TILE_COLS 64        // output columns of a workgroup (a lane a column, so that a wave reads a run of a weight row)
#define TILE_WAVES 4        // the contraction is shared out over the waves and summed through LDS

// acc[r] += sum over this wave's share of e of in_s[r][e] * w[e][c]: four weight rows asked for at a time.
template <typename TW>
__device__ __forceinline__ void tile_product(const float* in_s, int k, const TW* w, int n, int c, bool live, float (&acc)[TILE_TOKENS]) {
    const int wave = threadIdx.x / KIPP_WAVE;
    const int share = (k + TILE_WAVES - 1) / TILE_WAVES;
    const int e0 = wave * share, e1 = min(k, e0 + share);
#pragma unroll
    for (int r = 0; r < TILE_TOKENS; ++r) acc[r] = 0.0f;
    if (!live) return;
    int e = e0;
    for (; e + 4 <= e1; e += 4) {
        float wv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) wv[u] = load_f(w, (size_t)(e + u) * n + c);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int r = 0; r < TILE_TOKENS; ++r) acc[r] = fmaf(in_s[r * k + e + u], wv[u], acc[r]);
    }
    for (; e < e1; ++e) {
        const float wv = load_f(w, (size_t)e * n + c);
#pragma unroll
        for (int r = 0; r < TILE_TOKENS; ++r) acc[r] = fmaf(in_s[r * k + e], wv, acc[r]);
    }
}

// The waves' partial sums added in wave order; every thread of wave 0 gets its column's totals.  red: TILE_WAVES * TILE_TOKENS * TILE_COLS floats.
__device__ __forceinline__ void tile_reduce(float* red, float (&acc)[TILE_TOKENS]) {
    const int wave = threadIdx.x / KIPP_WAVE, lane = threadIdx.x & (KIPP_WAVE - 1);
#pragma unroll
    for (int r = 0; r < TILE_TOKENS; ++r) red[(wave * TILE_TOKENS + r) * TILE_COLS + lane] = acc[r];
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < TILE_TOKENS; ++r) {
            float total = 0.0f;
#pragma unroll
            for (int w = 0; w < TILE_WAVES; ++w) total += red[(w * TILE_TOKENS + r) * TILE_COLS + lane];
            acc[r] = total;
        }
    }
}

// One workgroup a (tile of tokens, head, 64 columns of the latent).  LDS: TILE_TOKENS * d floats, then the partial sums.
template <typename TW, typename TO>
__global__ void __launch_bounds__(TILE_WAVES * KIPP_WAVE) latent_absorb_kernel(
    const float* __restrict__ q, int parts, size_t part_stride, const TW* __restrict__ w_uk, TO* __restrict__ out,
    const int32_t* __restrict__ positions, const float* __restrict__ freq, int rot_dims, float magnitude,
    int n_tokens, int heads, int d, int dr, int rank) {
    extern __shared__ float lds[];
    float* q_s = lds;
    float* red = lds + TILE_TOKENS * d;
    const int t0 = blockIdx.x * TILE_TOKENS;
    const int head = blockIdx.y;
    const int rows = min(TILE_TOKENS, n_tokens - t0);
    const int q_row = heads * (d + dr);
    for (int i = threadIdx.x; i < TILE_TOKENS * d; i += blockDim.x) {
        const int r = i / d, e = i - r * d;
        float v = 0.0f;
        if (r < rows)
            for (int p = 0; p < parts; ++p) v += q[p * part_stride + (size_t)(t0 + r) * q_row + head * (d + dr) + e];
        q_s[i] = v;
    }
    __syncthreads();
    const int width = rank + dr;
    const int c = blockIdx.z * TILE_COLS + (threadIdx.x & (KIPP_WAVE - 1));
    float acc[TILE_TOKENS];
    tile_product(q_s, d, w_uk + (size_t)head * d * rank, rank, c, c < rank, acc);
    tile_reduce(red, acc);
    if (threadIdx.x < KIPP_WAVE && c < rank) {
#pragma unroll
        for (int r = 0; r < TILE_TOKENS; ++r)
            if (r < rows) store_f(out + ((size_t)(t0 + r) * heads + head) * width, c, acc[r]);
    }
    if (blockIdx.z != 0) return;
    // the rotated part
    for (int i = threadIdx.x; i < TILE_TOKENS * ((dr + 1) / 2); i += blockDim.x) {
        const int r = i / ((dr + 1) / 2), pair = i - r * ((dr + 1) / 2);
        if (r >= rows) continue;
        const size_t at = (size_t)(t0 + r) * q_row + head * (d + dr) + d + 2 * pair;
        float a = 0.0f, b = 0.0f;
        for (int p = 0; p < parts; ++p) {
            a += q[p * part_stride + at];
            if (2 * pair + 1 < dr) b += q[p * part_stride + at + 1];
        }
        if (2 * pair + 1 < rot_dims) rotate_pair(a, b, positions[t0 + r], freq[pair], magnitude);
        TO* dst = out + ((size_t)(t0 + r) * heads + head) * width + rank;
        store_f(dst, 2 * pair, a);
        if (2 * pair + 1 < dr) store_f(dst, 2 * pair + 1, b);
    }
}

// One workgroup a (tile of tokens, head, 64 value columns).  w_uv_t is [heads][rank][dv] (transposed at load, so that
// lanes read neighbouring numbers).  `lat` rows are `lat_row` wide, of which the first `rank` are read.
// LDS: TILE_TOKENS * rank floats, then the partial sums.
template <typename TI, typename TW, typename TO>
__global__ void __launch_bounds__(TILE_WAVES * KIPP_WAVE) latent_expand_kernel(
    const TI* __restrict__ lat, int lat_row, const TW* __restrict__ w_uv_t, const float* __restrict__ gate, int gate_parts,
    size_t gate_part_stride, int gate_stride, TO* __restrict__ out, int n_tokens, int heads, int rank, int dv) {
    extern __shared__ float lds[];
    float* l_s = lds;
    float* red = lds + TILE_TOKENS * rank;
    const int t0 = blockIdx.x * TILE_TOKENS;
    const int head = blockIdx.y;
    const int rows = min(TILE_TOKENS, n_tokens - t0);
    for (int i = threadIdx.x; i < TILE_TOKENS * rank; i += blockDim.x) {
        const int r = i / rank, e = i - r * rank;
        l_s[i] = r < rows ? load_f(lat, ((size_t)(t0 + r) * heads + head) * lat_row + e) : 0.0f;
    }
    __syncthreads();
    const int c = blockIdx.z * TILE_COLS + (threadIdx.x & (KIPP_WAVE - 1));
    float acc[TILE_TOKENS];
    tile_product(l_s, rank, w_uv_t + (size_t)head * rank * dv, dv, c, c < dv, acc);
    tile_reduce(red, acc);
    if (threadIdx.x >= KIPP_WAVE || c >= dv) return;
#pragma unroll
    for (int r = 0; r < TILE_TOKENS; ++r) {
        if (r >= rows) continue;
        float g = 1.0f;
        if (gate != nullptr) {
            float z = 0.0f;
            for (int p = 0; p < gate_parts; ++p) z += gate[p * gate_part_stride + (size_t)(t0 + r) * gate_stride + head];
            g = 1.0f / (1.0f + expf(-z));
        }
        store_f(out + ((size_t)(t0 + r) * heads + head) * dv, c, acc[r] * g);
    }
}

extern "C" {

int kipp_latent_prepare(const float* proj, int parts, int stride, const float* q_norm_w, const float* c_norm_w, float eps,
                        void* cq_out, int cq_dtype, void* cache, int cache_dtype, const int32_t* positions,
                        const int32_t* seq_of_token, const int32_t* block_table, int max_blocks, const float* freq, int rot_dims,
                        float magnitude, int n_tokens, int q_rank, int rank, int dr, int page, int write_kv, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (q_rank <= 0 || rank <= 0 || dr < 0 || rot_dims < 0 || rot_dims > dr || rot_dims % 2 || page <= 0 || stride < q_rank + rank + dr) return -1;
    const int most = q_rank > rank ? q_rank : rank;
    const int block = most >= 1024 ? 1024 : (most >= 512 ? 512 : 256);
    const size_t part_stride = (size_t)n_tokens * stride;
#define KIPP_LP(TO, TC)                                                                                                  \
    hipLaunchKernelGGL((latent_prepare_kernel<TO, TC>), dim3(n_tokens), dim3(block), 0, stream, proj, parts, part_stride, \
                       stride, q_norm_w, c_norm_w, eps, (TO*)cq_out, (TC*)cache, positions, seq_of_token, block_table,   \
                       max_blocks, freq, rot_dims, magnitude, q_rank, rank, dr, page, write_kv)
    if (cq_dtype == KIPP_F32 && cache_dtype == KIPP_F32) KIPP_LP(float, float);
    else if (cq_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16) KIPP_LP(bf16_t, bf16_t);
    else return -2;
#undef KIPP_LP
    return KIPP_LAUNCH_CHECK();
}

int kipp_latent_absorb(const float* q, int parts, const void* w_uk, int w_dtype, void* out, int out_dtype,
                       const int32_t* positions, const float* freq, int rot_dims, float magnitude, int n_tokens, int heads,
                       int d, int dr, int rank, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (heads <= 0 || d <= 0 || dr < 0 || rank <= 0 || rot_dims > dr || rot_dims % 2) return -1;
    const size_t lds = (size_t)(TILE_TOKENS * d + TILE_WAVES * TILE_TOKENS * TILE_COLS) * sizeof(float);
    if (lds > 64 * 1024) return -1;
    dim3 grid((n_tokens + TILE_TOKENS - 1) / TILE_TOKENS, heads, (rank + TILE_COLS - 1) / TILE_COLS), block(TILE_WAVES * KIPP_WAVE);
    const size_t part_stride = (size_t)n_tokens * heads * (d + dr);
#define KIPP_LA(TW, TO)                                                                                                 \
    hipLaunchKernelGGL((latent_absorb_kernel<TW, TO>), grid, block, lds, stream, q, parts, part_stride, (const TW*)w_uk, \
                       (TO*)out, positions, freq, rot_dims, magnitude, n_tokens, heads, d, dr, rank)
    if (w_dtype == KIPP_F32 && out_dtype == KIPP_F32) KIPP_LA(float, float);
    else if (w_dtype == KIPP_BF16 && out_dtype == KIPP_BF16) KIPP_LA(bf16_t, bf16_t);
    else return -2;
#undef KIPP_LA
    return KIPP_LAUNCH_CHECK();
}

int kipp_latent_expand(const void* lat, int lat_dtype, int lat_row, const void* w_uv_t, int w_dtype, const float* gate,
                       int gate_parts, int gate_stride, void* out, int out_dtype, int n_tokens, int heads, int rank, int dv,
                       hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (heads <= 0 || rank <= 0 || dv <= 0 || lat_row < rank) return -1;
    const size_t lds = (size_t)(TILE_TOKENS * rank + TILE_WAVES * TILE_TOKENS * TILE_COLS) * sizeof(float);
    if (lds > 64 * 1024) return -1;
    dim3 grid((n_tokens + TILE_TOKENS - 1) / TILE_TOKENS, heads, (dv + TILE_COLS - 1) / TILE_COLS), block(TILE_WAVES * KIPP_WAVE);
    const size_t gate_part_stride = (size_t)n_tokens * gate_stride;
#define KIPP_LE(TI, TW, TO)                                                                                             \
    hipLaunchKernelGGL((latent_expand_kernel<TI, TW, TO>), grid, block, lds, stream, (const TI*)lat, lat_row,            \
                       (const TW*)w_uv_t, gate, gate_parts, gate_part_stride, gate_stride, (TO*)out, n_tokens, heads, rank, dv)
    if (lat_dtype == KIPP_F32 && w_dtype == KIPP_F32 && out_dtype == KIPP_F32) KIPP_LE(float, float, float);
    else if (lat_dtype == KIPP_BF16 && w_dtype == KIPP_BF16 && out_dtype == KIPP_BF16) KIPP_LE(bf16_t, bf16_t, bf16_t);
    else return -2;
#undef KIPP_LE
    return KIPP_LAUNCH_CHECK();
}

}  // extern "C"
