// The matrix memory of an mLSTM layer: the recurrence itself, for prompt portions and single tokens alike, and
// the step between it and the output projection.
//
// Per head, with a query q (already times d^(-1/2)), key k (d numbers), value v (dv numbers) and the two gate
// pre-activations zi, zf of a token:
//     li = cap * tanh((zi + bi) / cap)                   the log of the input gate
//     lf = logsigmoid(cap * tanh((zf + bf) / cap))       the log of the forget gate
//     m' = max(lf + m, li)
//     S' = exp(lf + m - m') S + exp(li - m') k v^T       (d x dv),   n' likewise with k alone
//     o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
// S, n and m live in the request's state slot as float32 [heads][d][dv] | [Z][heads][d] | [Z][heads], Z = ceil(dv / columns of a workgroup):
// every workgroup of a head keeps a copy of n and m of its own (all equal), so that none reads what another has
// already written for the next step.  A slot that was just claimed holds zeros, which is the recurrence's start.
// Everything here is float32.
//
// scan    a workgroup takes (entry of the batch, head, 64 columns of S) and walks the entry's tokens in order.
//         A column is shared by 4 lanes that stand side by side in a wave, each with every fourth row of it, so
//         the sum over rows ends in two lane exchanges and no wave waits for another: there is no barrier in
//         the walk.  (Keys of more than 256 numbers: 16 lanes a column, 16 columns a workgroup.)  Every lane also keeps its rows of n (the same arithmetic in every column, hence the same
//         bits), so the denominator needs no exchange between columns either.
// finish  every head of a token divided by its root mean square, times the norm's weight, times sigmoid(gate),
//         in the type the output projection reads.
//
// `proj` is the input product, float32 [tokens][stride], with the columns
//     [q: heads d | k: heads d | v: heads dv | gate: heads dv | zi: heads | zf: heads].
#include "common.h"
#include <math.h>

#define SCAN_THREADS 256

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.0f) - log1pf(expf(-fabsf(z))); }

template <int ROWS, int SCAN_PARTS>     // rows of a column that one lane holds: ceil(d / SCAN_PARTS) <= ROWS
__global__ void __launch_bounds__(SCAN_THREADS) mlstm_scan_kernel(
    const float* __restrict__ proj, int stride, const float* __restrict__ bias_i, const float* __restrict__ bias_f, float cap,
    float* __restrict__ state, size_t state_stride, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
    const int32_t* __restrict__ slots, float* __restrict__ o_raw, int heads, int d, int dv) {
    constexpr int SCAN_COLS = SCAN_THREADS / SCAN_PARTS;
    const int seq = blockIdx.x, head = blockIdx.y;
    const int part = threadIdx.x & (SCAN_PARTS - 1);
    const int col = blockIdx.z * SCAN_COLS + threadIdx.x / SCAN_PARTS;
    const bool live = col < dv;
    const int first = q_start[seq], count = q_len[seq];
    float* slot = state + (size_t)slots[seq] * state_stride;
    float* S_g = slot + (size_t)head * d * dv;
    float* n_g = slot + (size_t)heads * d * dv + ((size_t)blockIdx.z * heads + head) * d;
    float* m_g = slot + (size_t)heads * d * dv + (size_t)gridDim.z * heads * d + (size_t)blockIdx.z * heads + head;

    float S[ROWS], nv[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int row = part + r * SCAN_PARTS;
        S[r] = (live && row < d) ? S_g[(size_t)row * dv + col] : 0.0f;
        nv[r] = row < d ? n_g[row] : 0.0f;
    }
    float m = *m_g;
    const float q_scale = 1.0f / sqrtf((float)d);
    const float bi = bias_i[head], bf = bias_f[head];
    const int at_k = heads * d, at_v = 2 * heads * d, at_i = 2 * heads * d + 2 * heads * dv, at_f = at_i + heads;

    for (int t = first; t < first + count; ++t) {
        const float* row_p = proj + (size_t)t * stride;
        const float li = cap * tanhf((row_p[at_i + head] + bi) / cap);
        const float lf = log_sigmoid(cap * tanhf((row_p[at_f + head] + bf) / cap));
        const float m_new = fmaxf(lf + m, li);
        const float keep = expf(lf + m - m_new), take = expf(li - m_new);
        const float v = live ? row_p[at_v + head * dv + col] : 0.0f;
        float num = 0.0f, den = 0.0f;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int row = part + r * SCAN_PARTS;
            const float k = row < d ? row_p[at_k + head * d + row] : 0.0f;
            const float q = row < d ? row_p[head * d + row] * q_scale : 0.0f;
            const float tk = take * k;
            S[r] = fmaf(keep, S[r], tk * v);
            nv[r] = fmaf(keep, nv[r], tk);
            num = fmaf(S[r], q, num);
            den = fmaf(nv[r], q, den);
        }
#pragma unroll
        for (int off = 1; off < SCAN_PARTS; off <<= 1) {
            num += __shfl_xor(num, off, KIPP_WAVE);
            den += __shfl_xor(den, off, KIPP_WAVE);
        }
        m = m_new;
        if (live && part == 0)
            o_raw[((size_t)t * heads + head) * dv + col] = num / (fmaxf(fabsf(den), expf(-m)) + 1e-6f);
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int row = part + r * SCAN_PARTS;
        if (live && row < d) S_g[(size_t)row * dv + col] = S[r];
        if (threadIdx.x < SCAN_PARTS && row < d) n_g[row] = nv[r];
    }
    if (threadIdx.x == 0) *m_g = m;
}

#define FINISH_HEADS 4

template <typename TO>
__global__ void mlstm_finish_kernel(const float* __restrict__ o_raw, const float* __restrict__ proj, int stride, int gate_at,
                                    const float* __restrict__ norm_w, float eps, TO* __restrict__ out, int heads, int dv) {
    const int wave = threadIdx.x / KIPP_WAVE, lane = threadIdx.x & (KIPP_WAVE - 1);
    const int t = blockIdx.y, head = blockIdx.x * FINISH_HEADS + wave;
    if (head >= heads) return;
    const float* src = o_raw + ((size_t)t * heads + head) * dv;
    float ss = 0.0f;
    for (int e = lane; e < dv; e += KIPP_WAVE) ss = fmaf(src[e], src[e], ss);
    ss = wave_sum(ss);
    const float scale = 1.0f / sqrtf(ss / (float)dv + eps);
    const float* gate = proj + (size_t)t * stride + gate_at + head * dv;
    TO* dst = out + ((size_t)t * heads + head) * dv;
    for (int e = lane; e < dv; e += KIPP_WAVE)
        store_f(dst, e, src[e] * scale * norm_w[head * dv + e] * (1.0f / (1.0f + expf(-gate[e]))));
}

extern "C" {

int kipp_mlstm_scan(const float* proj, int stride, const float* bias_i, const float* bias_f, float cap, float* state,
                    size_t state_stride, const int32_t* q_start, const int32_t* q_len, const int32_t* slots, float* o_raw,
                    int n_seqs, int heads, int d, int dv, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (heads <= 0 || d <= 0 || d > 1024 || dv <= 0 || !(cap > 0.0f)) return -1;
    const int parts = d <= 256 ? 4 : 16;
    const int cols = SCAN_THREADS / parts;
    if (stride < 2 * heads * d + 2 * heads * dv + 2 * heads || state_stride < (size_t)heads * d * dv + (size_t)((dv + cols - 1) / cols) * (heads * d + heads)) return -1;
    dim3 grid(n_seqs, heads, (dv + cols - 1) / cols), block(SCAN_THREADS);
    const int rows = (d + parts - 1) / parts;
#define KIPP_SCAN(R, P)                                                                                                        \
    hipLaunchKernelGGL((mlstm_scan_kernel<R, P>), grid, block, 0, stream, proj, stride, bias_i, bias_f, cap, state, state_stride, \
                       q_start, q_len, slots, o_raw, heads, d, dv)
    if (parts == 16) KIPP_SCAN(64, 16);
    else if (rows <= 4) KIPP_SCAN(4, 4);
    else if (rows <= 8) KIPP_SCAN(8, 4);
    else if (rows <= 16) KIPP_SCAN(16, 4);
    else if (rows <= 32) KIPP_SCAN(32, 4);
    else KIPP_SCAN(64, 4);
#undef KIPP_SCAN
    return KIPP_LAUNCH_CHECK();
}

int kipp_mlstm_finish(const float* o_raw, const float* proj, int stride, int gate_at, const float* norm_w, float eps,
                      void* out, int out_dtype, int n_tokens, int heads, int dv, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (heads <= 0 || dv <= 0 || stride < gate_at + heads * dv) return -1;
    dim3 grid((heads + FINISH_HEADS - 1) / FINISH_HEADS, n_tokens), block(FINISH_HEADS * KIPP_WAVE);
    if (out_dtype == KIPP_BF16)
        hipLaunchKernelGGL(mlstm_finish_kernel<bf16_t>, grid, block, 0, stream, o_raw, proj, stride, gate_at, norm_w, eps, (bf16_t*)out, heads, dv);
    else
        hipLaunchKernelGGL(mlstm_finish_kernel<float>, grid, block, 0, stream, o_raw, proj, stride, gate_at, norm_w, eps, (float*)out, heads, dv);
    return KIPP_LAUNCH_CHECK();
}

}  // extern "C"
