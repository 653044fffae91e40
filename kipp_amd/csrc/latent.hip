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

#define ABSORB_TOKENS 8

// One workgroup a (tile of ABSORB_TOKENS tokens, head): a weight row is read once for the tile.
// LDS: ABSORB_TOKENS * d floats.
template <typename TW, typename TO>
__global__ void latent_absorb_kernel(
    const float* __restrict__ q, int parts, size_t part_stride, const TW* __restrict__ w_uk, TO* __restrict__ out,
    const int32_t* __restrict__ positions, const float* __restrict__ freq, int rot_dims, float magnitude,
    int n_tokens, int heads, int d, int dr, int rank) {
    extern __shared__ float q_s[];
    const int t0 = blockIdx.x * ABSORB_TOKENS;
    const int head = blockIdx.y;
    const int rows = min(ABSORB_TOKENS, n_tokens - t0);
    const int q_row = heads * (d + dr);
    for (int i = threadIdx.x; i < ABSORB_TOKENS * d; i += blockDim.x) {
        const int r = i / d, e = i - r * d;
        float v = 0.0f;
        if (r < rows)
            for (int p = 0; p < parts; ++p) v += q[p * part_stride + (size_t)(t0 + r) * q_row + head * (d + dr) + e];
        q_s[i] = v;
    }
    __syncthreads();
    const TW* w = w_uk + (size_t)head * d * rank;
    const int width = rank + dr;
    for (int c = threadIdx.x; c < rank; c += blockDim.x) {
        float acc[ABSORB_TOKENS];
#pragma unroll
        for (int r = 0; r < ABSORB_TOKENS; ++r) acc[r] = 0.0f;
        for (int e = 0; e < d; ++e) {
            const float wv = load_f(w, (size_t)e * rank + c);
#pragma unroll
            for (int r = 0; r < ABSORB_TOKENS; ++r) acc[r] = fmaf(q_s[r * d + e], wv, acc[r]);
        }
#pragma unroll
        for (int r = 0; r < ABSORB_TOKENS; ++r)
            if (r < rows) store_f(out + ((size_t)(t0 + r) * heads + head) * width, c, acc[r]);
    }
    // the rotated part
    for (int i = threadIdx.x; i < ABSORB_TOKENS * ((dr + 1) / 2); i += blockDim.x) {
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

#define EXPAND_TOKENS 8

// One workgroup a (tile of tokens, head).  w_uv_t is [heads][rank][dv] (transposed at load, so that lanes
// read neighbouring numbers).  `lat` rows are `lat_row` wide, of which the first `rank` are read.
// LDS: EXPAND_TOKENS * rank floats.
template <typename TI, typename TW, typename TO>
__global__ void latent_expand_kernel(
    const TI* __restrict__ lat, int lat_row, const TW* __restrict__ w_uv_t, const float* __restrict__ gate, int gate_parts,
    size_t gate_part_stride, int gate_stride, TO* __restrict__ out, int n_tokens, int heads, int rank, int dv) {
    extern __shared__ float l_s[];
    const int t0 = blockIdx.x * EXPAND_TOKENS;
    const int head = blockIdx.y;
    const int rows = min(EXPAND_TOKENS, n_tokens - t0);
    for (int i = threadIdx.x; i < EXPAND_TOKENS * rank; i += blockDim.x) {
        const int r = i / rank, e = i - r * rank;
        l_s[i] = r < rows ? load_f(lat, ((size_t)(t0 + r) * heads + head) * lat_row + e) : 0.0f;
    }
    __syncthreads();
    const TW* w = w_uv_t + (size_t)head * rank * dv;
    for (int c = threadIdx.x; c < dv; c += blockDim.x) {
        float acc[EXPAND_TOKENS];
#pragma unroll
        for (int r = 0; r < EXPAND_TOKENS; ++r) acc[r] = 0.0f;
        for (int e = 0; e < rank; ++e) {
            const float wv = load_f(w, (size_t)e * dv + c);
#pragma unroll
            for (int r = 0; r < EXPAND_TOKENS; ++r) acc[r] = fmaf(l_s[r * rank + e], wv, acc[r]);
        }
#pragma unroll
        for (int r = 0; r < EXPAND_TOKENS; ++r) {
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
    const size_t lds = (size_t)ABSORB_TOKENS * d * sizeof(float);
    if (lds > 64 * 1024) return -1;
    dim3 grid((n_tokens + ABSORB_TOKENS - 1) / ABSORB_TOKENS, heads), block(rank >= 256 ? 256 : (rank >= 128 ? 128 : 64));
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
    const size_t lds = (size_t)EXPAND_TOKENS * rank * sizeof(float);
    if (lds > 64 * 1024) return -1;
    dim3 grid((n_tokens + EXPAND_TOKENS - 1) / EXPAND_TOKENS, heads), block(dv >= 256 ? 256 : (dv >= 128 ? 128 : 64));
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
