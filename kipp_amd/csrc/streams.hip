// Several copies of the residual stream ("hyper-connections").
//
// Instead of one row x a token there are R rows X_1 .. X_R, kept as float32 [tokens][R][width].  A sublayer
// reads a weighted sum of them and its result y goes back into all of them at once:
//
//     read    u = sum_r a[r] X_r ;  h = u * rsqrt(mean(u^2) + eps) * w          (the sublayer's RMS norm)
//     write   X_t <- sum_r M[r][t] X_r + b[t] y       for every t, from the old rows
//
// A layer's write and the next sublayer's read are one pass over the token's rows (`kipp_streams_step` takes
// either half or both): the rows are read once, written once, and the normed row leaves in the type the next
// product reads.  y may come as slabs [parts][tokens][width] of a product whose contraction was split; they
// are added in order.  Everything is float32; a token is one workgroup's, and the sums of a token run in an
// order that its own row fixes.
//
//     open    X_r = table[token] for every r
//     close   out = sum_t (sum_r M[r][t] X_r + b[t] y), for all tokens or for the rows named by `rows`
//             (what the final norm reads; nothing is written back)
#include "common.h"

#define STREAMS_MAX 8

template <typename TT>
__global__ void streams_open_kernel(const TT* __restrict__ table, const int32_t* __restrict__ tokens, float* __restrict__ X,
                                    int R, int width) {
    const int t = blockIdx.x;
    const TT* src = table + (size_t)tokens[t] * width;
    float* dst = X + (size_t)t * R * width;
    for (int e = threadIdx.x; e < width; e += blockDim.x) {
        const float v = load_f(src, e);
        for (int r = 0; r < R; ++r) dst[(size_t)r * width + e] = v;
    }
}

// write (if mix != nullptr), then read and norm (if inw != nullptr).  R copies (a build constant where it is 1 to 4, so
// that the coefficients and a lane's rows stay in registers), VEC numbers a lane and load (4 where the width
// allows); the workgroup is sized so that a lane meets its numbers once where the width allows, with every load
// of a token asked for before the first is used.  LDS: width floats + 16.
template <int RMAX, int VEC, typename TO>
__global__ void streams_step_kernel(float* __restrict__ X, const float* __restrict__ delta, int parts, size_t part_stride,
                                    const float* __restrict__ mix, const float* __restrict__ outw,
                                    const float* __restrict__ inw, const float* __restrict__ norm_w, float eps,
                                    TO* __restrict__ h, int R, int width, const int32_t* __restrict__ which, int store) {
    extern __shared__ float lds[];
    float* u_s = lds + 16;
    const int t = which != nullptr ? which[blockIdx.x] : blockIdx.x;     // the token; the normed row leaves as row blockIdx.x
    float* rows = X + (size_t)t * R * width;
    float c_mix[RMAX][RMAX], c_out[RMAX], c_in[RMAX];
#pragma unroll
    for (int s = 0; s < RMAX; ++s) {
#pragma unroll
        for (int to = 0; to < RMAX; ++to) c_mix[s][to] = (mix != nullptr && s < R && to < R) ? mix[s * R + to] : 0.0f;
        c_out[s] = (outw != nullptr && s < R) ? outw[s] : 0.0f;
        c_in[s] = (inw != nullptr && s < R) ? inw[s] : 0.0f;
    }
    float ss = 0.0f;
    for (int e = threadIdx.x * VEC; e < width; e += blockDim.x * VEC) {
        float x[RMAX][VEC], y[VEC];
#pragma unroll
        for (int r = 0; r < RMAX; ++r) {
            if (r < R) {
                if (VEC == 4) *reinterpret_cast<float4*>(x[r]) = *reinterpret_cast<const float4*>(rows + (size_t)r * width + e);
                else x[r][0] = rows[(size_t)r * width + e];
            } else {
#pragma unroll
                for (int v = 0; v < VEC; ++v) x[r][v] = 0.0f;
            }
        }
        if (mix != nullptr) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) y[v] = 0.0f;
            for (int p = 0; p < parts; ++p) {
                float d4[VEC];
                if (VEC == 4) *reinterpret_cast<float4*>(d4) = *reinterpret_cast<const float4*>(delta + p * part_stride + (size_t)t * width + e);
                else d4[0] = delta[p * part_stride + (size_t)t * width + e];
#pragma unroll
                for (int v = 0; v < VEC; ++v) y[v] += d4[v];
            }
            float fresh[RMAX][VEC];
#pragma unroll
            for (int to = 0; to < RMAX; ++to) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    float acc = 0.0f;
#pragma unroll
                    for (int s = 0; s < RMAX; ++s) acc += c_mix[s][to] * x[s][v];
                    fresh[to][v] = acc + c_out[to] * y[v];
                }
                if (to < R && store) {
                    if (VEC == 4) *reinterpret_cast<float4*>(rows + (size_t)to * width + e) = *reinterpret_cast<float4*>(fresh[to]);
                    else rows[(size_t)to * width + e] = fresh[to][0];
                }
            }
#pragma unroll
            for (int r = 0; r < RMAX; ++r)
#pragma unroll
                for (int v = 0; v < VEC; ++v) x[r][v] = fresh[r][v];
        }
        if (inw != nullptr) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                float u = 0.0f;
#pragma unroll
                for (int r = 0; r < RMAX; ++r) u += c_in[r] * x[r][v];
                u_s[e + v] = u;
                ss = fmaf(u, u, ss);
            }
        }
    }
    if (inw == nullptr) return;
    ss = block_sum(ss, lds);
    const float scale = 1.0f / sqrtf(ss / (float)width + eps);
    TO* dst = h + (size_t)blockIdx.x * width;
    for (int e = threadIdx.x * VEC; e < width; e += blockDim.x * VEC)
#pragma unroll
        for (int v = 0; v < VEC; ++v) store_f(dst, e + v, u_s[e + v] * scale * norm_w[e + v]);
}

template <int RMAX>
__global__ void streams_close_kernel(const float* __restrict__ X, const float* __restrict__ delta, int parts, size_t part_stride,
                                     const float* __restrict__ mix, const float* __restrict__ outw,
                                     const int32_t* __restrict__ which, float* __restrict__ out, int R, int width) {
    const int i = blockIdx.x;
    const int t = which != nullptr ? which[i] : i;
    const float* rows = X + (size_t)t * R * width;
    float c_mix[RMAX][RMAX], c_out[RMAX];
#pragma unroll
    for (int s = 0; s < RMAX; ++s) {
#pragma unroll
        for (int to = 0; to < RMAX; ++to) c_mix[s][to] = (mix != nullptr && s < R && to < R) ? mix[s * R + to] : 0.0f;
        c_out[s] = (outw != nullptr && s < R) ? outw[s] : 0.0f;
    }
    for (int e = threadIdx.x; e < width; e += blockDim.x) {
        float x[RMAX];
#pragma unroll
        for (int r = 0; r < RMAX; ++r) x[r] = r < R ? rows[(size_t)r * width + e] : 0.0f;
        float total = 0.0f;
        if (mix != nullptr) {
            float y = 0.0f;
            for (int p = 0; p < parts; ++p) y += delta[p * part_stride + (size_t)t * width + e];
#pragma unroll
            for (int to = 0; to < RMAX; ++to) {
                float v = 0.0f;
#pragma unroll
                for (int s = 0; s < RMAX; ++s) v += c_mix[s][to] * x[s];
                if (to < R) total += v + c_out[to] * y;
            }
        } else {
#pragma unroll
            for (int r = 0; r < RMAX; ++r) total += x[r];
        }
        out[(size_t)i * width + e] = total;
    }
}

static int block_for(int width) { return width >= 2048 ? 1024 : (width >= 1024 ? 512 : (width >= 256 ? 256 : 64)); }

extern "C" {

int kipp_streams_open(const void* table, int table_dtype, const int32_t* tokens, float* X, int n, int R, int width,
                      hipStream_t stream) {
    if (n <= 0) return 0;
    if (R <= 0 || R > STREAMS_MAX || width <= 0) return -1;
    if (table_dtype == KIPP_BF16)
        hipLaunchKernelGGL(streams_open_kernel<bf16_t>, dim3(n), dim3(block_for(width)), 0, stream, (const bf16_t*)table, tokens, X, R, width);
    else
        hipLaunchKernelGGL(streams_open_kernel<float>, dim3(n), dim3(block_for(width)), 0, stream, (const float*)table, tokens, X, R, width);
    return KIPP_LAUNCH_CHECK();
}

// delta/mix/outw null: no write.  inw null: no read (h unused).  `which` (n_rows token numbers, or null: all n tokens in
// order): the tokens that are read; `store` 0: the written copies are not stored (the last read of a forward pass).
int kipp_streams_step(float* X, const float* delta, int parts, const float* mix, const float* outw, const float* inw,
                      const float* norm_w, float eps, void* h, int h_dtype, int n, int R, int width, const int32_t* which,
                      int n_rows, int store, hipStream_t stream) {
    if (which == nullptr) n_rows = n;
    if (n <= 0 || n_rows <= 0) return 0;
    if (which != nullptr && store) return -2;
    if (R <= 0 || R > STREAMS_MAX || width <= 0 || width > 32768) return -1;
    if ((mix == nullptr) != (delta == nullptr) || (mix != nullptr && outw == nullptr)) return -2;
    if (inw != nullptr && (norm_w == nullptr || h == nullptr)) return -2;
    const size_t lds = (size_t)(width + 16) * sizeof(float);
    const size_t stride = (size_t)n * width;
    const bool wide = width % 4 == 0 && (((uintptr_t)X | (uintptr_t)delta) & 15) == 0;
    const int lanes = wide ? width / 4 : width;
    const int threads = lanes >= 1024 ? 1024 : ((lanes + KIPP_WAVE - 1) / KIPP_WAVE) * KIPP_WAVE;
#define KIPP_SS(RMAX, VEC, TO)                                                                                                  \
    hipLaunchKernelGGL((streams_step_kernel<RMAX, VEC, TO>), dim3(n_rows), dim3(threads), lds, stream, X, delta, parts, stride, mix, \
                       outw, inw, norm_w, eps, (TO*)h, R, width, which, store)
#define KIPP_SS_R(VEC, TO)                   \
    do {                                     \
        if (R == 1) KIPP_SS(1, VEC, TO);     \
        else if (R == 2) KIPP_SS(2, VEC, TO); \
        else if (R <= 4) KIPP_SS(4, VEC, TO); \
        else KIPP_SS(STREAMS_MAX, VEC, TO);  \
    } while (0)
    if (h_dtype == KIPP_BF16) {
        if (wide) KIPP_SS_R(4, bf16_t); else KIPP_SS_R(1, bf16_t);
    } else {
        if (wide) KIPP_SS_R(4, float); else KIPP_SS_R(1, float);
    }
#undef KIPP_SS_R
#undef KIPP_SS
    return KIPP_LAUNCH_CHECK();
}

// `n` tokens in X and delta; `n_out` rows leave (`which` names them, or null: all n in order).
int kipp_streams_close(const float* X, const float* delta, int parts, const float* mix, const float* outw,
                       const int32_t* which, float* out, int n, int n_out, int R, int width, hipStream_t stream) {
    if (n_out <= 0) return 0;
    if (R <= 0 || R > STREAMS_MAX || width <= 0) return -1;
    if ((mix == nullptr) != (delta == nullptr) || (mix != nullptr && outw == nullptr)) return -2;
#define KIPP_SC(RMAX)                                                                                                     \
    hipLaunchKernelGGL(streams_close_kernel<RMAX>, dim3(n_out), dim3(block_for(width)), 0, stream, X, delta, parts,           \
                       (size_t)n * width, mix, outw, which, out, R, width)
    if (R <= 2) KIPP_SC(2);
    else if (R <= 4) KIPP_SC(4);
    else KIPP_SC(STREAMS_MAX);
#undef KIPP_SC
    return KIPP_LAUNCH_CHECK();
}

}  // extern "C"
