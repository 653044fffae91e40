// Attention whose softmax weights are mixed across heads, on the matrix cores (bfloat16 storage, float32
// arithmetic around the products).  The formulas are those at the head of attention_mixed.hip; built for one key
// size HEAD_DIM (a multiple of 32), one value size V_DIM (a multiple of 16) and HPW heads a wave (up to 8 HPW heads);
// SHARED_KV says that a wave's heads all read one key/value head, whose keys and values it then loads once.
//
// Mixing the heads' weights needs every head's FINAL weight of a (query, key) pair in one place, so the softmax
// cannot be rescaled on the way as flash attention does.  The work is therefore cut into items (a tile of up to 16
// query rows of one entry, a run of its keys) and done in two walks over the keys:
//
//   mixed_stats_kernel    scores of all heads, each lane keeping a running maximum and sum of its own keys;
//                         an item leaves (maximum, sum) of every (head, row);
//   mixed_values_kernel   merges the items' statistics of its tile (the sink joins here), then, 32 keys at a time:
//                         1. scores again, weights p = exp(s - M) / L, final, into LDS as [row][key][head],
//                            split into two bfloat16 halves (hi + lo carries 16 bits of mantissa);
//                         2. p' = mix . p on the matrix cores, contraction over heads, into LDS as [head][row][key];
//                         3. O^T[dv][row] += V^T . p'^T, the values read as they lie in the cache: the cache keeps
//                            them transposed inside a page, [page][kv head][dv][slot], so eight keys of one value
//                            column are sixteen contiguous bytes.
//                         A tile whose keys are one run writes gate * O as bfloat16; otherwise float32 partial sums
//                         (weights are final, so runs simply add), which mixed_finish_kernel adds and gates.
//
// v_mfma_f32_16x16x32_bf16: A lane l holds row l % 16, k = 8 (l / 16) + j; B lane l holds column l % 16, same k;
// D lane l holds rows 4 (l / 16) + v of column l % 16.  Scores: A = 16 keys, B = 16 query rows.  Mixing: A = 16
// (row, key) pairs over heads, B = mix^T.  Values: A = V^T (16 value columns over 32 keys), B = p'.
//
// Everything a workgroup does follows from device-side lengths (ctx_len, q_len), so a recorded step whose item list
// was made for the longest context of its class still computes each sequence's own keys; an item whose run of keys
// is empty leaves neutral statistics and zeros.
#include "common.h"
#include <math.h>

#ifndef HEAD_DIM
#define HEAD_DIM 64
#endif
#ifndef V_DIM
#define V_DIM 64
#endif
#ifndef HPW
#define HPW 1
#endif
#ifndef SHARED_KV
#define SHARED_KV 1                     // the HPW heads of a wave read one key/value head (heads a kv head are a multiple of HPW)
#endif

#define MX_WAVES 8
#define MX_THREADS (MX_WAVES * KIPP_WAVE)
#define MX_ROWS 16
#define MX_KEYS 32
#define MX_HPAD 32                      // heads padded to one step of the mixing product
// LDS strides, in bfloat16 values, chosen so that the lanes of a wave fall into different banks: the weights as
// [row][key][head] with 40 values a key (32 heads and 8 unused) and 1,288 a row, which a lane writes two bytes at a
// time (16 rows x 4 keys of one head: 4 lanes a bank instead of 64 with the plain strides) and reads 16 bytes at a
// time (no conflict); the mixed weights as [head][row][key] with 40 values a row and 656 a head.
#define P_KEY 40
#define P_ROW 1288
#define M_ROW 40
#define M_HEAD 656
#define MX_LDS_BYTES ((2 * MX_ROWS * P_ROW + MX_HPAD * M_HEAD) * 2)
#define KSTEPS (HEAD_DIM / 32)
#ifndef V_SLICE
#define V_SLICE V_DIM                   // value columns a workgroup sums: V_DIM / V_SLICE workgroups share an item, each
#endif                                  // with its own columns (their sums then fit a wave's registers) and all of the weights
#define VBLOCKS (V_SLICE / 16)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// float32 -> bfloat16 by the hardware's conversion (round to nearest even, as f32_to_bf16 does for finite values)
__device__ __forceinline__ bf16_t to_bf16(float f) {
    const __bf16 b = (__bf16)f;
    return __builtin_bit_cast(bf16_t, b);
}

union Frag {
    u32x4 u;
    bf16x8 v;
    bf16_t h[8];
};

struct MixedGeometry {
    const int32_t* item_entry;      // [items] entry of the batch
    const int32_t* item_row0;       // [items] first row of the tile within its entry
    const int32_t* item_split;      // [items] which run of the tile's keys
    const int32_t* item_nsplits;    // [items] runs of the tile (its items are consecutive)
    const int32_t* q_start;         // [entries]
    const int32_t* q_len;           // [entries]
    const int32_t* ctx_len;         // [entries] tokens of the sequence after this step
    const int32_t* block_table;     // [entries][max_blocks]
    int max_blocks, page, n_q, n_kv, window, keep_first;
    float scale;
    const float *r1, *r2;           // [n_q] or null
};

struct Tile {
    int entry, first_row, rows, pos0, last;     // rows of the batch first_row .. + rows - 1 at positions pos0 ..; last = pos0 + rows - 1
    int kept_tiles, window_tile0;               // key tiles 0 .. kept_tiles - 1, then window_tile0 ..
    int begin, end;                             // this item's run of tile indices
    const int32_t* table;
};

__device__ __forceinline__ Tile tile_of(const MixedGeometry& g, int item) {
    Tile t;
    t.entry = g.item_entry[item];
    const int row0 = g.item_row0[item], q_len = g.q_len[t.entry];
    t.rows = max(0, min(MX_ROWS, q_len - row0));
    t.first_row = g.q_start[t.entry] + row0;
    t.pos0 = g.ctx_len[t.entry] - q_len + row0;
    t.last = t.pos0 + t.rows - 1;
    t.table = g.block_table + (size_t)t.entry * g.max_blocks;
    const int lo = g.window > 0 ? max(0, t.pos0 - g.window + 1) : 0;
    const int kept = g.window > 0 ? min(g.keep_first, lo) : 0;
    t.kept_tiles = kept > 0 ? (kept - 1) / MX_KEYS + 1 : 0;
    t.window_tile0 = max(lo / MX_KEYS, t.kept_tiles);
    const int total = t.rows > 0 ? t.kept_tiles + (t.last / MX_KEYS - t.window_tile0 + 1) : 0;
    const int nsplits = g.item_nsplits[item], split = g.item_split[item];
    const int chunk = (total + nsplits - 1) / nsplits;
    t.begin = min(total, split * chunk);
    t.end = min(total, t.begin + chunk);
    return t;
}

__device__ __forceinline__ int key_tile(const Tile& t, int index) {
    return index < t.kept_tiles ? index : t.window_tile0 + index - t.kept_tiles;
}

// The 16 keys from `key0` on of key/value head `c` as A operands: lane l holds key l % 16, columns 32 s + 8 (l / 16) ..
__device__ __forceinline__ void load_keys(const MixedGeometry& g, const Tile& t, const bf16_t* __restrict__ k_cache, int c, int key0,
                                          Frag* kf) {
    const int lane = threadIdx.x & (KIPP_WAVE - 1), l16 = lane & 15, quarter = lane >> 4;
    const int key = min(key0 + l16, t.last);            // rows beyond the context are masked later; their loads stay inside it
    const bf16_t* row = k_cache + (((size_t)t.table[key / g.page] * g.n_kv + c) * g.page + key % g.page) * HEAD_DIM + 8 * quarter;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) kf[s].u = *(const u32x4*)(row + 32 * s);
}

// S^T[key][row] of one head for the 16 keys from `key0` on: lane l gets keys key0 + 4 (l / 16) + v of row l % 16,
// already scaled, biased by distance and masked (-inf).  `kf`: the keys as A operands, `qf`: the head's query rows
// as B operands.
template <bool INSIDE>
__device__ __forceinline__ void scores16(const MixedGeometry& g, const Tile& t, int key0, const Frag* kf, const Frag* qf,
                                         float a, float b, float sc[4]) {
    const int lane = threadIdx.x & (KIPP_WAVE - 1), l16 = lane & 15, quarter = lane >> 4;
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[s].v, qf[s].v, acc, 0, 0, 0);
    const int i = t.pos0 + l16;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int j = key0 + 4 * quarter + v;
        // INSIDE: every row of the tile sees all 16 keys (rows that only fill the tile up compute unused numbers)
        const bool sees = INSIDE || (l16 < t.rows && j <= i && (g.window <= 0 || i - j < g.window || j < g.keep_first));
        sc[v] = sees ? acc[v] * g.scale - a * __logf(1.0f + b * (float)(i - j)) : -INFINITY;
    }
}

// Whether every row of the tile sees every key of the 32 from `key0` on: behind the first row, and inside the window of
// the last (or among the kept first keys).
__device__ __forceinline__ bool all_seen(const MixedGeometry& g, const Tile& t, int key0) {
    return key0 + MX_KEYS - 1 <= t.pos0 && (g.window <= 0 || t.pos0 + MX_ROWS - 1 - key0 < g.window || key0 + MX_KEYS <= g.keep_first);
}

// The query rows of head h as B operands: lane l holds row l % 16, columns 32 s + 8 (l / 16) ..
__device__ __forceinline__ void load_queries(const Tile& t, const bf16_t* __restrict__ q, int n_q, int h, Frag* qf) {
    const int lane = threadIdx.x & (KIPP_WAVE - 1), l16 = lane & 15, quarter = lane >> 4;
    const int row = t.first_row + min(l16, max(t.rows - 1, 0));
    const bf16_t* at = q + ((size_t)row * n_q + h) * HEAD_DIM + 8 * quarter;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) qf[s].u = *(const u32x4*)(at + 32 * s);
}

// stats [items][n_q][16][2]: (maximum, sum of exp(score - maximum)) over the item's keys, without the sink.
__global__ void __launch_bounds__(MX_THREADS) mixed_stats_kernel(MixedGeometry g, const bf16_t* __restrict__ q,
                                                                 const bf16_t* __restrict__ k_cache, float* __restrict__ stats) {
    const int item = blockIdx.x;
    const Tile t = tile_of(g, item);
    const int wave = threadIdx.x / KIPP_WAVE, lane = threadIdx.x & (KIPP_WAVE - 1);
    const int group = g.n_q / g.n_kv, h0 = wave * HPW;
    if (h0 >= g.n_q) return;
    constexpr bool shared = SHARED_KV != 0;                 // the wave's heads read one key/value head
    Frag qf[HPW][KSTEPS];
    float a[HPW], b[HPW], m[HPW], l[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        const int h = min(h0 + hh, g.n_q - 1);
        load_queries(t, q, g.n_q, h, qf[hh]);
        a[hh] = g.r1 != nullptr ? g.r1[h] : 0.0f;
        b[hh] = g.r2 != nullptr ? g.r2[h] : 0.0f;
        m[hh] = -INFINITY;
        l[hh] = 0.0f;
    }
    Frag kf[MX_KEYS / 16][KSTEPS], next[MX_KEYS / 16][KSTEPS];
    if (t.begin < t.end) {
#pragma unroll
        for (int kb = 0; kb < MX_KEYS / 16; ++kb) load_keys(g, t, k_cache, h0 / group, key_tile(t, t.begin) * MX_KEYS + 16 * kb, next[kb]);
    }
    for (int index = t.begin; index < t.end; ++index) {
        const int key0 = key_tile(t, index) * MX_KEYS;
#pragma unroll
        for (int kb = 0; kb < MX_KEYS / 16; ++kb)
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) kf[kb][s] = next[kb][s];
        const bool inside = all_seen(g, t, key0);
        if (index + 1 < t.end) {            // the next tile's keys are on their way while this one is scored
#pragma unroll
            for (int kb = 0; kb < MX_KEYS / 16; ++kb) load_keys(g, t, k_cache, h0 / group, key_tile(t, index + 1) * MX_KEYS + 16 * kb, next[kb]);
        }
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            if (h0 + hh >= g.n_q) break;
#pragma unroll
            for (int kb = 0; kb < MX_KEYS / 16; ++kb) {
                Frag own[KSTEPS];
                if (!shared && hh > 0) load_keys(g, t, k_cache, (h0 + hh) / group, key0 + 16 * kb, own);
                float sc[4];
                if (inside) scores16<true>(g, t, key0 + 16 * kb, (!shared && hh > 0) ? own : kf[kb], qf[hh], a[hh], b[hh], sc);
                else scores16<false>(g, t, key0 + 16 * kb, (!shared && hh > 0) ? own : kf[kb], qf[hh], a[hh], b[hh], sc);
                const float m_new = fmaxf(m[hh], fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])));
                if (m_new != -INFINITY) {
                    float sum = 0.0f;
#pragma unroll
                    for (int v = 0; v < 4; ++v) sum += __expf(sc[v] - m_new);       // exp(-inf) = 0
                    l[hh] = l[hh] * __expf(m[hh] - m_new) + sum;
                    m[hh] = m_new;
                }
            }
        }
    }
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        if (h0 + hh >= g.n_q) break;
        float mm = m[hh], ll = l[hh];
        // the four lanes that share a row
#pragma unroll
        for (int off = 16; off <= 32; off <<= 1) {
            const float m_o = __shfl_xor(mm, off, KIPP_WAVE), l_o = __shfl_xor(ll, off, KIPP_WAVE);
            const float m_new = fmaxf(mm, m_o);
            if (m_new != -INFINITY) ll = ll * __expf(mm - m_new) + l_o * __expf(m_o - m_new);
            mm = m_new;
        }
        if (lane < 16) {
            float* out = stats + (((size_t)item * g.n_q + h0 + hh) * MX_ROWS + lane) * 2;
            out[0] = mm;
            out[1] = ll;
        }
    }
}

// LDS: p_hi, p_lo [16 rows][32 keys][32 heads] bfloat16, then p' [32 heads][16 rows][32 keys] bfloat16, with the padded strides above.
__global__ void __launch_bounds__(MX_THREADS) mixed_values_kernel(
    MixedGeometry g, const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const float* __restrict__ stats, const float* __restrict__ sink, const float* __restrict__ mix,
    const float* __restrict__ gate, int gate_stride, int gate_parts, size_t gate_part_stride,
    bf16_t* __restrict__ out, float* __restrict__ partial, size_t partial_stride) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    bf16_t* p_hi = (bf16_t*)lds_raw;
    bf16_t* p_lo = p_hi + MX_ROWS * P_ROW;
    bf16_t* p_mixed = p_lo + MX_ROWS * P_ROW;
    const int item = blockIdx.x, v0 = blockIdx.y * V_SLICE;        // this workgroup's value columns v0 .. v0 + V_SLICE - 1 of every head
    const Tile t = tile_of(g, item);
    const int wave = threadIdx.x / KIPP_WAVE, lane = threadIdx.x & (KIPP_WAVE - 1), l16 = lane & 15, quarter = lane >> 4;
    const int nsplits = g.item_nsplits[item], split = g.item_split[item];
    const int n_q = g.n_q, group = g.n_q / g.n_kv;
    constexpr bool shared = SHARED_KV != 0;                 // the wave's heads read one key/value head

    // columns of heads that do not exist stay zero for the whole walk
    if (n_q < MX_HPAD)
        for (int e = threadIdx.x; e < 2 * MX_ROWS * P_ROW / 8; e += MX_THREADS) ((u32x4*)p_hi)[e] = (u32x4){0u, 0u, 0u, 0u};

    // mix^T as B operands: lane holds head (column) 16 nb + l % 16, contraction heads 8 (l / 16) ..
    Frag mf[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const int h = 16 * nb + l16;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int from = 8 * quarter + j;
            float w = 0.0f;
            if (h < n_q && from < n_q) w = mix != nullptr ? mix[h * n_q + from] : (h == from ? 1.0f : 0.0f);
            mf[nb].h[j] = f32_to_bf16(w);
        }
    }

    // this wave's heads: queries, bias numbers, and every row's maximum and 1 / denominator over ALL runs of the tile
    Frag qf[HPW][KSTEPS];
    float bias_a[HPW], bias_b[HPW], top[HPW], inv[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        const int h = wave * HPW + hh;
        top[hh] = 0.0f;
        inv[hh] = 0.0f;
        bias_a[hh] = bias_b[hh] = 0.0f;
        if (h < n_q) {
            load_queries(t, q, n_q, h, qf[hh]);
            bias_a[hh] = g.r1 != nullptr ? g.r1[h] : 0.0f;
            bias_b[hh] = g.r2 != nullptr ? g.r2[h] : 0.0f;
            // the runs' statistics: each quarter of the wave takes every fourth run (four asked for at once), the
            // quarters are then merged, the sink last; any order gives the same maximum, and the sums differ in rounding only
            float m = -INFINITY, l = 0.0f;
            for (int s0 = quarter; s0 < nsplits; s0 += 16) {
                float2 st[4];
#pragma unroll
                for (int s = 0; s < 4; ++s)
                    st[s] = s0 + 4 * s < nsplits ? *(const float2*)(stats + (((size_t)(item - split + s0 + 4 * s) * n_q + h) * MX_ROWS + l16) * 2)
                                                 : make_float2(-INFINITY, 0.0f);
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const float m_new = fmaxf(m, st[s].x);
                    if (m_new != -INFINITY) l = l * __expf(m - m_new) + st[s].y * __expf(st[s].x - m_new);
                    m = m_new;
                }
            }
#pragma unroll
            for (int off = 16; off <= 32; off <<= 1) {
                const float m_o = __shfl_xor(m, off, KIPP_WAVE), l_o = __shfl_xor(l, off, KIPP_WAVE);
                const float m_new = fmaxf(m, m_o);
                if (m_new != -INFINITY) l = l * __expf(m - m_new) + l_o * __expf(m_o - m_new);
                m = m_new;
            }
            if (sink != nullptr) {
                const float m_new = fmaxf(m, sink[h]);
                l = (m == -INFINITY ? 0.0f : l * __expf(m - m_new)) + __expf(sink[h] - m_new);
                m = m_new;
            }
            top[hh] = m;
            inv[hh] = l > 0.0f ? 1.0f / l : 0.0f;
        }
    }

    f32x4 acc[HPW][VBLOCKS];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
        for (int mb = 0; mb < VBLOCKS; ++mb) acc[hh][mb] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    __syncthreads();

    for (int index = t.begin; index < t.end; ++index) {
        const int key0 = key_tile(t, index) * MX_KEYS;
        const bool inside = all_seen(g, t, key0);
        // 1. the final weights of this wave's heads; 16 keys are loaded once for all heads that share them, and a lane
        //    writes the weights of its heads (they are neighbours in the [row][key][head] layout) with one store
#pragma unroll
        for (int kb = 0; kb < MX_KEYS / 16; ++kb) {
            if (wave * HPW < n_q) {
                Frag kf[KSTEPS];
                load_keys(g, t, k_cache, wave * HPW / group, key0 + 16 * kb, kf);
                float p[HPW][4];
#pragma unroll
                for (int hh = 0; hh < HPW; ++hh) {
                    const int h = wave * HPW + hh;
#pragma unroll
                    for (int v = 0; v < 4; ++v) p[hh][v] = 0.0f;
                    if (h < n_q) {
                        if (!shared && hh > 0) load_keys(g, t, k_cache, h / group, key0 + 16 * kb, kf);
                        float sc[4];
                        if (inside) scores16<true>(g, t, key0 + 16 * kb, kf, qf[hh], bias_a[hh], bias_b[hh], sc);
                        else scores16<false>(g, t, key0 + 16 * kb, kf, qf[hh], bias_a[hh], bias_b[hh], sc);
#pragma unroll
                        for (int v = 0; v < 4; ++v) p[hh][v] = sc[v] == -INFINITY ? 0.0f : __expf(sc[v] - top[hh]) * inv[hh];
                    }
                }
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int at = l16 * P_ROW + (16 * kb + 4 * quarter + v) * P_KEY + wave * HPW;
                    bf16_t hi[HPW], lo[HPW];
#pragma unroll
                    for (int hh = 0; hh < HPW; ++hh) {
                        hi[hh] = to_bf16(p[hh][v]);
                        lo[hh] = to_bf16(p[hh][v] - bf16_to_f32(hi[hh]));
                    }
                    if (HPW == 4) {
                        *(uint2*)(p_hi + at) = make_uint2((uint32_t)hi[0] | ((uint32_t)hi[1 % HPW] << 16), (uint32_t)hi[2 % HPW] | ((uint32_t)hi[3 % HPW] << 16));
                        *(uint2*)(p_lo + at) = make_uint2((uint32_t)lo[0] | ((uint32_t)lo[1 % HPW] << 16), (uint32_t)lo[2 % HPW] | ((uint32_t)lo[3 % HPW] << 16));
                    } else if (HPW == 2) {
                        *(uint32_t*)(p_hi + at) = (uint32_t)hi[0] | ((uint32_t)hi[1 % HPW] << 16);
                        *(uint32_t*)(p_lo + at) = (uint32_t)lo[0] | ((uint32_t)lo[1 % HPW] << 16);
                    } else {
#pragma unroll
                        for (int hh = 0; hh < HPW; ++hh) {
                            p_hi[at + hh] = hi[hh];
                            p_lo[at + hh] = lo[hh];
                        }
                    }
                }
            }
        }
        __syncthreads();
        // 2. the heads mixed: 32 blocks of 16 (row, key) pairs, four a wave
#pragma unroll
        for (int u = 0; u < (MX_ROWS * MX_KEYS / 16) / MX_WAVES; ++u) {
            const int block = wave + MX_WAVES * u;              // row = block / 2, keys 16 (block % 2) ..
            const int row = block >> 1, kb = block & 1;
            const int at = row * P_ROW + (16 * kb + l16) * P_KEY + 8 * quarter;
            Frag hi, lo;
            hi.u = *(const u32x4*)(p_hi + at);
            lo.u = *(const u32x4*)(p_lo + at);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                if (16 * nb < n_q) {
                    f32x4 d = {0.0f, 0.0f, 0.0f, 0.0f};
                    d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(lo.v, mf[nb].v, d, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi.v, mf[nb].v, d, 0, 0, 0);
                    const int h = 16 * nb + l16;        // d[v]: keys 16 kb + 4 quarter + v of `row`, head h
                    if (h < n_q) {
                        uint2 w;
                        w.x = (uint32_t)to_bf16(d[0]) | ((uint32_t)to_bf16(d[1]) << 16);
                        w.y = (uint32_t)to_bf16(d[2]) | ((uint32_t)to_bf16(d[3]) << 16);
                        *(uint2*)(p_mixed + (h * M_HEAD + row * M_ROW + 16 * kb + 4 * quarter)) = w;
                    }
                }
            }
        }
        __syncthreads();
        // 3. times the values
        const int chunk = min(key0 + 8 * quarter, t.last);          // eight keys of one page (a page holds a multiple of 8)
        const size_t v_page = (size_t)t.table[chunk / g.page] * g.n_kv;
        const int v_slot = (key0 + 8 * quarter) % g.page;
        if (shared) {
            if (wave * HPW < n_q) {
                const bf16_t* v_at = v_cache + ((v_page + wave * HPW / group) * V_DIM + v0 + l16) * g.page + v_slot;
                constexpr int VB = VBLOCKS < 4 ? VBLOCKS : 4;        // value blocks asked for together
#pragma unroll
                for (int m0 = 0; m0 < VBLOCKS; m0 += VB) {
                    Frag vf[VB];
#pragma unroll
                    for (int mb = 0; mb < VB; ++mb)
                        if (m0 + mb < VBLOCKS) vf[mb].u = *(const u32x4*)(v_at + (size_t)16 * (m0 + mb) * g.page);
#pragma unroll
                    for (int hh = 0; hh < HPW; ++hh) {
                        Frag pf;
                        pf.u = *(const u32x4*)(p_mixed + (min(wave * HPW + hh, n_q - 1) * M_HEAD + l16 * M_ROW + 8 * quarter));
#pragma unroll
                        for (int mb = 0; mb < VB; ++mb)
                            if (m0 + mb < VBLOCKS && wave * HPW + hh < n_q)
                                acc[hh][m0 + mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[mb].v, pf.v, acc[hh][m0 + mb], 0, 0, 0);
                    }
                }
            }
        } else {
#pragma unroll
            for (int hh = 0; hh < HPW; ++hh) {
                const int h = wave * HPW + hh;
                if (h < n_q) {
                    Frag pf;
                    pf.u = *(const u32x4*)(p_mixed + (h * M_HEAD + l16 * M_ROW + 8 * quarter));
                    const bf16_t* v_at = v_cache + ((v_page + h / group) * V_DIM + v0 + l16) * g.page + v_slot;
#pragma unroll
                    for (int mb = 0; mb < VBLOCKS; ++mb) {
                        Frag vf;
                        vf.u = *(const u32x4*)(v_at + (size_t)16 * mb * g.page);
                        acc[hh][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, acc[hh][mb], 0, 0, 0);
                    }
                }
            }
        }
        // the next tile's weights overwrite p only after every wave has passed the barrier behind step 2,
        // and p' only after the barrier behind the next step 1
    }

    // acc[hh][mb][v]: value column 16 mb + 4 quarter + v of row l16
    if (l16 >= t.rows) return;
    const size_t row = (size_t)t.first_row + l16;
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        const int h = wave * HPW + hh;
        if (h >= n_q) break;
#pragma unroll
        for (int mb = 0; mb < VBLOCKS; ++mb) {
            const int col = h * V_DIM + v0 + 16 * mb + 4 * quarter;
            if (nsplits > 1) {
                *(f32x4*)(partial + split * partial_stride + row * ((size_t)n_q * V_DIM) + col) = acc[hh][mb];
            } else {
                float o[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    o[v] = acc[hh][mb][v];
                    if (gate != nullptr) {
                        float z = 0.0f;
                        for (int p = 0; p < gate_parts; ++p) z += gate[p * gate_part_stride + row * gate_stride + col + v];
                        o[v] *= 1.0f / (1.0f + __expf(-z));
                    }
                }
                uint2 w;
                w.x = (uint32_t)f32_to_bf16(o[0]) | ((uint32_t)f32_to_bf16(o[1]) << 16);
                w.y = (uint32_t)f32_to_bf16(o[2]) | ((uint32_t)f32_to_bf16(o[3]) << 16);
                *(uint2*)(out + row * ((size_t)n_q * V_DIM) + col) = w;
            }
        }
    }
}

// Rows whose keys were cut into runs: out = gate * (sum of the runs' partial sums, in order).  A thread takes four
// columns of a row and asks for every run's sums before it adds the first.
__global__ void __launch_bounds__(256) mixed_finish_kernel(const float* __restrict__ partial, size_t partial_stride,
                                                           const int32_t* __restrict__ row_splits, const float* __restrict__ gate,
                                                           int gate_stride, int gate_parts, size_t gate_part_stride,
                                                           bf16_t* __restrict__ out, int width) {
    const size_t row = blockIdx.y;
    const int n = row_splits[row];
    const int e = 4 * (blockIdx.x * 256 + threadIdx.x);
    if (n <= 1 || e >= width) return;
    f32x4 o = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int s0 = 0; s0 < n; s0 += 8) {
        f32x4 part[8];
#pragma unroll
        for (int s = 0; s < 8; ++s)
            part[s] = s0 + s < n ? *(const f32x4*)(partial + (s0 + s) * partial_stride + row * width + e) : (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < 8; ++s) o += part[s];
    }
    float r[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        r[v] = o[v];
        if (gate != nullptr) {
            float z = 0.0f;
            for (int p = 0; p < gate_parts; ++p) z += gate[p * gate_part_stride + row * gate_stride + e + v];
            r[v] *= 1.0f / (1.0f + __expf(-z));
        }
    }
    uint2 w;
    w.x = (uint32_t)f32_to_bf16(r[0]) | ((uint32_t)f32_to_bf16(r[1]) << 16);
    w.y = (uint32_t)f32_to_bf16(r[2]) | ((uint32_t)f32_to_bf16(r[3]) << 16);
    *(uint2*)(out + row * width + e) = w;
}

extern "C" {

int kipp_mixed_mfma_sizes(int* head_dim, int* v_dim, int* heads_per_wave, int* lds_bytes) {
    *head_dim = HEAD_DIM;
    *v_dim = V_DIM;
    *heads_per_wave = HPW;
    *lds_bytes = MX_LDS_BYTES;
    return 0;
}

// stats: float32 [items][n_q][16][2]; partial: float32 [max_splits][n_rows][n_q V_DIM] (may be null when no tile is cut);
// row_splits: int32 [n_rows], the runs of each row's tile; out: bfloat16 [n_rows][n_q V_DIM].
int kipp_mixed_attention_mfma(const void* q, const void* k_cache, const void* v_cache, void* out,
                              const float* gate, int gate_stride, int gate_parts,
                              const int32_t* item_entry, const int32_t* item_row0, const int32_t* item_split,
                              const int32_t* item_nsplits, int n_items, const int32_t* row_splits, int max_splits,
                              const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                              const int32_t* block_table, int max_blocks,
                              const float* r1, const float* r2, const float* sink, const float* mix,
                              float* stats, float* partial,
                              int n_rows, int n_q, int n_kv, int d, int dv, int page, float scale, int window, int keep_first,
                              hipStream_t stream) {
    if (n_items <= 0 || n_rows <= 0) return 0;
    if (V_DIM % V_SLICE || V_SLICE % 16) return -5;
    if (d != HEAD_DIM || dv != V_DIM || n_kv <= 0 || n_q % n_kv || n_q > MX_WAVES * HPW || n_q > MX_HPAD) return -1;
    if (SHARED_KV && HPW > 1 && (n_q / n_kv) % HPW) return -4;
    if (page <= 0 || page % 16 || max_splits < 1 || (max_splits > 1 && (partial == nullptr || row_splits == nullptr))) return -2;
    MixedGeometry g;
    g.item_entry = item_entry; g.item_row0 = item_row0; g.item_split = item_split; g.item_nsplits = item_nsplits;
    g.q_start = q_start; g.q_len = q_len; g.ctx_len = ctx_len; g.block_table = block_table;
    g.max_blocks = max_blocks; g.page = page; g.n_q = n_q; g.n_kv = n_kv; g.window = window; g.keep_first = keep_first;
    g.scale = scale; g.r1 = r1; g.r2 = r2;
    const int lds = MX_LDS_BYTES;
    static bool raised = false;
    if (!raised) {
        if (hipFuncSetAttribute((const void*)mixed_values_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -3;
        raised = true;
    }
    const size_t gate_part_stride = (size_t)n_rows * gate_stride;
    const size_t partial_stride = (size_t)n_rows * n_q * V_DIM;
    hipLaunchKernelGGL(mixed_stats_kernel, dim3(n_items), dim3(MX_THREADS), 0, stream, g, (const bf16_t*)q, (const bf16_t*)k_cache, stats);
    hipLaunchKernelGGL(mixed_values_kernel, dim3(n_items, V_DIM / V_SLICE), dim3(MX_THREADS), lds, stream, g, (const bf16_t*)q,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, stats, sink, mix, gate, gate_stride, gate_parts,
                       gate_part_stride, (bf16_t*)out, partial, partial_stride);
    if (max_splits > 1)
        hipLaunchKernelGGL(mixed_finish_kernel, dim3((n_q * V_DIM / 4 + 255) / 256, n_rows), dim3(256), 0, stream, partial, partial_stride, row_splits, gate,
                           gate_stride, gate_parts, gate_part_stride, (bf16_t*)out, n_q * V_DIM);
    return KIPP_LAUNCH_CHECK();
}

}  // extern "C"
