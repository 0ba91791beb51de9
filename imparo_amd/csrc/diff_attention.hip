// Differential attention over the paged cache: every head holds two softmax maps over the same
// values, combined as a1 - lambda a2, brought to unit RMS per head, scaled, gated and stored.
//
// Cache layout: K [n_pages, 2 kv_heads, page_size, dim] (key head g's map m is row 2g + m), V
// [n_pages, kv_heads, page_size, vdim]. Queries [tokens, heads, 2, dim] arrive already multiplied by
// their position's temperature. Scores, softmax, the combination and the norm are float32.
//
// k_diff_qkv_store: from the fused projection's float32 rows [q | k | v | ...] the queries (times the
// temperature 1 + coef * ln(floor((pos + 1) / every) + 1)) and the new keys and values into their pages.
// k_diff_attention: one wave per (token, head, split of the keys). Keys are walked in chunks of 64 at
// absolute multiples of 64, one key a lane for the two scores, one value dimension a lane for the two
// weighted sums; both maps share every value load. With one split the wave finishes the head itself;
// with more, the splits (DA_SPLIT keys each, at absolute multiples) leave their running maxima, sums
// and weighted sums, and k_diff_merge finishes.
#include "common.h"
#include "api.h"

#define DA_WAVES 4
#define DA_MAX_DIM 256
#define DA_MAX_VDIM 512
#define DA_SPLIT 128

extern "C" int imparo_diff_attention_split(void) { return DA_SPLIT; }

template <typename T>
__global__ void k_diff_qkv_store(const float* __restrict__ rows_in, int ld, const int32_t* __restrict__ positions,
                                 const int32_t* __restrict__ row_of_token, const int32_t* __restrict__ block_table,
                                 int table_stride, int page_size, T* __restrict__ q_out, T* __restrict__ k_cache,
                                 T* __restrict__ v_cache, int write_kv, int heads, int kv_heads, int dim, int vdim,
                                 int n_pages, float temp_coef, int temp_every) {
    const int t = blockIdx.x;
    const int pos = positions[t];
    const float* row = rows_in + (size_t)t * ld;
    const int nq = heads * 2 * dim, nk = kv_heads * 2 * dim, nv = kv_heads * vdim;
    float temp = 1.0f;
    if (temp_every > 0) temp = 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
    for (int i = threadIdx.x; i < nq; i += blockDim.x) store_f32<T>(q_out, (size_t)t * nq + i, row[i] * temp);
    if (!write_kv) return;
    const int page = block_table[(size_t)row_of_token[t] * table_stride + pos / page_size];
    if (page < 0 || page >= n_pages) return;
    const int in_page = pos % page_size;
    for (int i = threadIdx.x; i < nk; i += blockDim.x) {
        const int kh = i / dim, d = i - kh * dim;
        store_f32<T>(k_cache, (((size_t)page * 2 * kv_heads + kh) * page_size + in_page) * dim + d, row[nq + i]);
    }
    for (int i = threadIdx.x; i < nv; i += blockDim.x) {
        const int g = i / vdim, d = i - g * vdim;
        store_f32<T>(v_cache, (((size_t)page * kv_heads + g) * page_size + in_page) * vdim + d, row[nq + nk + i]);
    }
}

template <typename T>
__device__ __forceinline__ float da_dot(const float* __restrict__ q, const T* __restrict__ k, int dim);

// 16 bytes a load where the rows allow it (every key row then starts at a multiple of 16 bytes)
template <>
__device__ __forceinline__ float da_dot<float>(const float* __restrict__ q, const float* __restrict__ k, int dim) {
    float s = 0.f;
    if ((dim & 3) == 0) {
        for (int i = 0; i < dim; i += 4) {
            const float4 kv = *reinterpret_cast<const float4*>(k + i);
            s += q[i] * kv.x;
            s += q[i + 1] * kv.y;
            s += q[i + 2] * kv.z;
            s += q[i + 3] * kv.w;
        }
    } else {
        for (int i = 0; i < dim; ++i) s += q[i] * k[i];
    }
    return s;
}

template <>
__device__ __forceinline__ float da_dot<bf16_t>(const float* __restrict__ q, const bf16_t* __restrict__ k, int dim) {
    float s = 0.f;
    if ((dim & 7) == 0) {
        for (int i = 0; i < dim; i += 8) {
            const uint4 kv = *reinterpret_cast<const uint4*>(k + i);
            const uint32_t w[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                s += q[i + 2 * j] * __uint_as_float(w[j] << 16);
                s += q[i + 2 * j + 1] * __uint_as_float(w[j] & 0xffff0000u);
            }
        }
    } else {
        for (int i = 0; i < dim; ++i) s += q[i] * bf16_to_f32(k[i]);
    }
    return s;
}

// What finishes a head: o = a1 - lambda a2 over the head's vdim values (lane d holds d, d + 64, ...), divided
// by its root mean square, times out_scale, times sigmoid(gate).
template <typename T, int VPL>
__device__ __forceinline__ void da_finish(const float (&a1)[VPL], const float (&a2)[VPL], float lambda, float eps,
                                          float out_scale, const float* __restrict__ gate, T* __restrict__ dst, int vdim,
                                          int lane) {
    float o[VPL];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        const int d = lane + j * WAVE;
        o[j] = d < vdim ? a1[j] - lambda * a2[j] : 0.f;
        ss += o[j] * o[j];
    }
    ss = wave_sum(ss);
    const float r = out_scale / sqrtf(ss / (float)vdim + eps);
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        const int d = lane + j * WAVE;
        if (d < vdim) {
            float y = o[j] * r;
            if (gate) y *= 1.0f / (1.0f + expf(-gate[d]));
            store_f32<T>(dst, d, y);
        }
    }
}

// VPL: value dimensions a lane holds (d = lane, lane + 64, ...): vdim <= 64 VPL.
template <typename T, int VPL>
__global__ void k_diff_attention(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                 const float* __restrict__ gate, int gate_ld, T* __restrict__ out,
                                 float* __restrict__ part, const int32_t* __restrict__ positions,
                                 const int32_t* __restrict__ row_of_token, const int32_t* __restrict__ block_table,
                                 int table_stride, int page_size, int n_tokens, int heads, int kv_heads, int dim,
                                 int vdim, int n_pages, float scale, int window, float lambda, float eps,
                                 float out_scale, int n_splits, const int32_t* __restrict__ seg_len, int below) {
    __shared__ float q_rows[DA_WAVES][2 * DA_MAX_DIM];
    __shared__ float probs[DA_WAVES][2][WAVE];
    __shared__ long long v_off[DA_WAVES][WAVE];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const long long id = (long long)blockIdx.x * DA_WAVES + wave;
    if (id >= (long long)n_tokens * heads * n_splits) return;
    const int split = (int)(id % n_splits);
    const long long th = id / n_splits;
    const int t = (int)(th / heads);
    const int h = (int)(th - (long long)t * heads);
    const int g = h / (heads / kv_heads);
    if (below > 0 && seg_len[row_of_token[t]] >= below) return;   // a longer row's tokens are another launch's
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
    int first = (lo / WAVE) * WAVE, last = pos;             // chunks from `first`, keys up to `last`
    if (n_splits > 1) {
        first = max(first, split * DA_SPLIT);
        last = min(pos, (split + 1) * DA_SPLIT - 1);
        if (first > last) return;                             // this split holds no key of the query (uniform over the wave)
    }
    const int32_t* table = block_table + (size_t)row_of_token[t] * table_stride;

    float* qr = q_rows[wave];
    const T* qsrc = q + ((size_t)t * heads + h) * 2 * dim;
    for (int i = lane; i < 2 * dim; i += WAVE) qr[i] = load_f32<T>(qsrc, i);
    wave_lds_sync();

    float a1[VPL], a2[VPL];
#pragma unroll
    for (int j = 0; j < VPL; ++j) a1[j] = a2[j] = 0.f;
    float m1 = -INFINITY, l1 = 0.f, m2 = -INFINITY, l2 = 0.f;

    for (int c = first; c <= last; c += WAVE) {
        const int p = c + lane;
        const bool valid = p >= lo && p <= last;
        float s1 = -INFINITY, s2 = -INFINITY;
        long long off = -1;
        if (valid) {
            const int page = table[p / page_size];
            if (page >= 0 && page < n_pages) {
                const long long k_off = (((long long)page * 2 * kv_heads + 2 * g) * page_size + (p % page_size)) * dim;
                s1 = da_dot<T>(qr, k_cache + k_off, dim) * scale;
                s2 = da_dot<T>(qr + dim, k_cache + k_off + (long long)page_size * dim, dim) * scale;
                off = (((long long)page * kv_heads + g) * page_size + (p % page_size)) * vdim;
            }
        }
        const float m1n = fmaxf(m1, wave_max(s1));
        const float m2n = fmaxf(m2, wave_max(s2));
        const float p1 = off >= 0 ? expf(s1 - m1n) : 0.f;
        const float p2 = off >= 0 ? expf(s2 - m2n) : 0.f;
        const float c1 = m1 == -INFINITY ? 0.f : expf(m1 - m1n);
        const float c2 = m2 == -INFINITY ? 0.f : expf(m2 - m2n);
        l1 = l1 * c1 + wave_sum(p1);
        l2 = l2 * c2 + wave_sum(p2);
        m1 = m1n;
        m2 = m2n;
        probs[wave][0][lane] = p1;
        probs[wave][1][lane] = p2;
        v_off[wave][lane] = off;
        wave_lds_sync();
        const int n_keys = min(WAVE, last - c + 1);
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            a1[j] *= c1;
            a2[j] *= c2;
        }
        // eight keys' values are asked for before any is used, from addresses that always lie in the cache
        // (a key that is not there reads row 0 and weighs nothing); the sums run in the order of the keys
        for (int kk0 = 0; kk0 < n_keys; kk0 += 8) {
            float vals[8][VPL], w1[8], w2[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int kk = min(kk0 + u, WAVE - 1);
                const long long vo = v_off[wave][kk];
                const bool on = kk0 + u < n_keys && vo >= 0;
                const T* vrow = v_cache + (on ? vo : 0);
                w1[u] = on ? probs[wave][0][kk] : 0.f;
                w2[u] = on ? probs[wave][1][kk] : 0.f;
#pragma unroll
                for (int j = 0; j < VPL; ++j) {
                    const int d = lane + j * WAVE;
                    const float v = load_f32<T>(vrow, min(d, vdim - 1));
                    vals[u][j] = on && d < vdim ? v : 0.f;
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
#pragma unroll
                for (int j = 0; j < VPL; ++j) {
                    a1[j] += w1[u] * vals[u][j];
                    a2[j] += w2[u] * vals[u][j];
                }
            }
        }
        wave_lds_sync();
    }
    if (n_splits > 1) {
        float* dst = part + ((size_t)th * n_splits + split) * (2 * vdim + 4);
        if (lane == 0) {
            dst[0] = m1;
            dst[1] = l1;
            dst[2] = m2;
            dst[3] = l2;
        }
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int d = lane + j * WAVE;
            if (d < vdim) {
                dst[4 + d] = a1[j];
                dst[4 + vdim + d] = a2[j];
            }
        }
        return;
    }
    const float i1 = l1 > 0.f ? 1.0f / l1 : 0.f, i2 = l2 > 0.f ? 1.0f / l2 : 0.f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        a1[j] *= i1;
        a2[j] *= i2;
    }
    da_finish<T, VPL>(a1, a2, lambda, eps, out_scale, gate ? gate + (size_t)t * gate_ld + (size_t)h * vdim : nullptr,
                 out + ((size_t)t * heads + h) * vdim, vdim, lane);
}

// One wave per (token, head): the splits that hold keys of the query, in order.
template <typename T, int VPL>
__global__ void k_diff_merge(const float* __restrict__ part, const float* __restrict__ gate, int gate_ld,
                             T* __restrict__ out, const int32_t* __restrict__ positions, int n_tokens, int heads,
                             int vdim, int window, float lambda, float eps, float out_scale, int n_splits,
                             const int32_t* __restrict__ row_of_token, const int32_t* __restrict__ seg_len, int below) {
    const int lane = threadIdx.x & (WAVE - 1);
    const long long th = (long long)blockIdx.x * DA_WAVES + threadIdx.x / WAVE;
    if (th >= (long long)n_tokens * heads) return;
    const int t = (int)(th / heads);
    if (below > 0 && seg_len[row_of_token[t]] >= below) return;
    const int h = (int)(th - (long long)t * heads);
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
    const int s_first = lo / DA_SPLIT, s_last = min(pos / DA_SPLIT, n_splits - 1);
    const float* base = part + (size_t)th * n_splits * (2 * vdim + 4);
    const int stride = 2 * vdim + 4;
    // the splits' maxima: a split a lane, 64 at a time
    float m1 = -INFINITY, m2 = -INFINITY;
    for (int s0 = s_first; s0 <= s_last; s0 += WAVE) {
        const int s = min(s0 + lane, s_last);
        m1 = fmaxf(m1, base[(size_t)s * stride]);
        m2 = fmaxf(m2, base[(size_t)s * stride + 2]);
    }
    m1 = wave_max(m1);
    m2 = wave_max(m2);
    float a1[VPL], a2[VPL];
#pragma unroll
    for (int j = 0; j < VPL; ++j) a1[j] = a2[j] = 0.f;
    float l1 = 0.f, l2 = 0.f;
    // the weighted sums in the order of the splits, four splits' rows asked for at once
    for (int s0 = s_first; s0 <= s_last; s0 += 4) {
        float w1[4], w2[4], r1[4][VPL], r2[4][VPL];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const bool on = s0 + u <= s_last;
            const float* p = base + (size_t)min(s0 + u, s_last) * stride;
            const float pm1 = p[0], pl1 = p[1], pm2 = p[2], pl2 = p[3];
            w1[u] = on && pm1 != -INFINITY ? expf(pm1 - m1) : 0.f;
            w2[u] = on && pm2 != -INFINITY ? expf(pm2 - m2) : 0.f;
            l1 += w1[u] * pl1;
            l2 += w2[u] * pl2;
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
                const int d = min(lane + j * WAVE, vdim - 1);
                r1[u][j] = p[4 + d];
                r2[u][j] = p[4 + vdim + d];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
                a1[j] += w1[u] * r1[u][j];
                a2[j] += w2[u] * r2[u][j];
            }
    }
    const float i1 = l1 > 0.f ? 1.0f / l1 : 0.f, i2 = l2 > 0.f ? 1.0f / l2 : 0.f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        a1[j] *= i1;
        a2[j] *= i2;
    }
    da_finish<T, VPL>(a1, a2, lambda, eps, out_scale, gate ? gate + (size_t)t * gate_ld + (size_t)h * vdim : nullptr,
                 out + ((size_t)t * heads + h) * vdim, vdim, lane);
}

// ---------------------------------------------------------------- matrix-core kernel for prompt portions
// bfloat16, pages of a multiple of 16 positions, dim and vdim multiples of 4 up to 128. A block is four
// waves of one head over 64 consecutive queries of one request's portion, a wave takes 16 of them. Keys
// are walked in tiles of 32 at absolute multiples of 32. Both products are taken transposed, S^T = K Q^T
// and O^T = V^T P^T (16x16x16 products): the scores a lane holds after the first product (four
// consecutive keys of one query) are exactly what the second wants from it as its right operand, so no
// value crosses lanes between the two; a query's maximum and sum meet over the four lanes that share its
// column. Each map keeps its own maximum, sum and O^T; both share every V^T operand.
typedef short da_s16x4 __attribute__((ext_vector_type(4)));
typedef float da_f32x4 __attribute__((ext_vector_type(4)));
#define DAM_TILE 64          // queries a block
#define DAM_MAX16 8          // 16-wide blocks of dim and of vdim that the registers hold

extern "C" int imparo_diff_attention_tile(void) { return DAM_TILE; }

__device__ __forceinline__ da_s16x4 da_pack4(float a, float b, float c, float d) {
    const uint32_t lo = f32x2_to_bf16x2(a, b), hi = f32x2_to_bf16x2(c, d);
    da_s16x4 r;
    r[0] = (short)(lo & 0xffff);
    r[1] = (short)(lo >> 16);
    r[2] = (short)(hi & 0xffff);
    r[3] = (short)(hi >> 16);
    return r;
}

// The operands of one tile of 32 keys: for each of its two blocks of 16 keys whether its page is there, and
// the K rows (both maps) as the first product's left operand.
template <int D16>
struct DaKeys {
    da_s16x4 k[2][2][D16];       // [map][block of 16 keys][16 dims]
    long long vbase[2];
    bool there[2];
};

template <int D16>
__device__ __forceinline__ void da_load_keys(DaKeys<D16>& t, const bf16_t* __restrict__ k_cache,
                                             const int32_t* __restrict__ table, int k0, int pos_last, int page_size,
                                             int n_pages, int kv_heads, int g, int dim, int vdim, int col, int quad) {
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
        const int key0 = k0 + mb * 16;                       // a block of 16 keys lies in one page
        const int page = key0 <= pos_last ? table[key0 / page_size] : -1;
        t.there[mb] = page >= 0 && page < n_pages;
        const long long pg = t.there[mb] ? page : 0;          // a block that is not there reads page 0 and counts for nothing
        const long long kbase = ((pg * 2 * kv_heads + 2 * g) * page_size + (key0 % page_size)) * dim;
        t.vbase[mb] = ((pg * kv_heads + g) * page_size + (key0 % page_size)) * (long long)vdim;
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int kk = 0; kk < D16; ++kk) {
                const int d = min(kk * 16 + quad * 4, dim - 4);          // dims past the head repeat its end; the query holds zeros there
                t.k[m][mb][kk] = *reinterpret_cast<const da_s16x4*>(k_cache + kbase + ((long long)m * page_size + col) * dim + d);
            }
    }
}

// D16, V16: blocks of 16 of dim and of vdim that the registers hold (4 or 8).
template <int D16, int V16>
__global__ __launch_bounds__(256) void k_diff_attention_tiles(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const float* __restrict__ gate, int gate_ld, bf16_t* __restrict__ out, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
    const int32_t* __restrict__ block_table, int table_stride, int page_size, int heads, int kv_heads, int dim,
    int vdim, int n_pages, float scale, int window, float lambda, float eps, float out_scale, int min_len) {
    const int r = blockIdx.x, h = blockIdx.z;
    const int len = seg_len[r];
    if (len < min_len) return;                                 // (uniform over the block) such rows are another launch's
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int q0 = blockIdx.y * DAM_TILE + wave * 16;          // this wave's first query within the portion
    if (q0 >= len) return;
    const int col = lane & 15, quad = lane >> 4;               // a lane's query column and its group of four rows
    const int t0 = seg_start[r];
    const int n_q = min(16, len - q0);
    const int qi = min(col, n_q - 1);                          // columns past the portion repeat its last query and store nothing
    const int t = t0 + q0 + qi;
    const int pos = positions[t];
    const int pos_first = positions[t0 + q0], pos_last = positions[t0 + q0 + n_q - 1];
    const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
    const int lo_first = window > 0 ? max(0, pos_first + 1 - window) : 0;
    const int lo_last = window > 0 ? max(0, pos_last + 1 - window) : 0;
    const int g = h / (heads / kv_heads);
    const int vd16 = (vdim + 15) >> 4;
    const int32_t* table = block_table + (size_t)r * table_stride;

    // Q^T operands: query `col`, dims 16 kk + 4 quad .. + 3, both maps; zeros past the head's dims
    da_s16x4 qf[2][D16];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int kk = 0; kk < D16; ++kk) {
            const int d = kk * 16 + quad * 4;
            const da_s16x4 v = *reinterpret_cast<const da_s16x4*>(q + (((size_t)t * heads + h) * 2 + m) * dim + min(d, dim - 4));
            qf[m][kk] = d < dim ? v : da_s16x4{0, 0, 0, 0};
        }
    da_f32x4 o[2][V16];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int vb = 0; vb < V16; ++vb) o[m][vb] = da_f32x4{0.f, 0.f, 0.f, 0.f};
    float mx[2] = {-INFINITY, -INFINITY}, sum[2] = {0.f, 0.f};

    DaKeys<D16> cur, nxt;
    int k0 = (lo_first / 32) * 32;
    da_load_keys<D16>(cur, k_cache, table, k0, pos_last, page_size, n_pages, kv_heads, g, dim, vdim, col, quad);
    for (; k0 <= pos_last; k0 += 32) {
        // this tile's values and the next tile's keys are asked for before this tile's products begin
        da_s16x4 vt[2][V16];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int vb = 0; vb < V16; ++vb) {
                if (vb >= vd16) continue;
                // keys 4 quad .. + 3 of the block, value dimension 16 vb + col: four rows of V, one value each
                const int d = min(vb * 16 + col, vdim - 1);
                const bf16_t* src = v_cache + cur.vbase[mb] + (long long)(quad * 4) * vdim + d;
                vt[mb][vb][0] = (short)src[0];
                vt[mb][vb][1] = (short)src[vdim];
                vt[mb][vb][2] = (short)src[2 * vdim];
                vt[mb][vb][3] = (short)src[3 * vdim];
            }
        da_load_keys<D16>(nxt, k_cache, table, k0 + 32, pos_last, page_size, n_pages, kv_heads, g, dim, vdim, col, quad);

        da_s16x4 pb[2][2];                                   // P^T operands: [map][block of 16 keys]
        float corr[2];
        // a tile that every query of the wave sees whole needs no look at single keys (uniform over the wave)
        const bool whole = cur.there[0] && cur.there[1] && k0 + 31 <= pos_first && k0 >= lo_last;
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            da_f32x4 sc[2] = {da_f32x4{0.f, 0.f, 0.f, 0.f}, da_f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int kk = 0; kk < D16; ++kk)
                    sc[mb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(cur.k[m][mb][kk], qf[m][kk], sc[mb], 0, 0, 0);
            // a lane holds keys k0 + 16 mb + 4 quad + i of query `col`
            float tile_max = -INFINITY;
            if (whole) {
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        sc[mb][i] *= scale;
                        tile_max = fmaxf(tile_max, sc[mb][i]);
                    }
            } else {
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int key = k0 + mb * 16 + quad * 4 + i;
                        const bool seen = cur.there[mb] && key <= pos && key >= lo;
                        sc[mb][i] = seen ? sc[mb][i] * scale : -INFINITY;
                        tile_max = fmaxf(tile_max, sc[mb][i]);
                    }
            }
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE));
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE));
            const float m_new = fmaxf(mx[m], tile_max);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            corr[m] = mx[m] == -INFINITY ? 0.f : __expf(mx[m] - m_use);
            float tile_sum = 0.f;
            float p[2][4];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    p[mb][i] = __expf(sc[mb][i] - m_use);       // exp(-inf) = 0 for keys that are not seen
                    tile_sum += p[mb][i];
                }
            tile_sum += __shfl_xor(tile_sum, 16, WAVE);
            tile_sum += __shfl_xor(tile_sum, 32, WAVE);
            sum[m] = sum[m] * corr[m] + tile_sum;
            mx[m] = m_new;
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) pb[m][mb] = da_pack4(p[mb][0], p[mb][1], p[mb][2], p[mb][3]);
        }
        // the old sums are rescaled only when some query's maximum moved (uniform over the wave)
        const bool rescale = __any(corr[0] != 1.0f || corr[1] != 1.0f);
#pragma unroll
        for (int vb = 0; vb < V16; ++vb) {
            if (vb < vd16) {
                if (rescale) {
#pragma unroll
                    for (int m = 0; m < 2; ++m) {
                        o[m][vb][0] *= corr[m];
                        o[m][vb][1] *= corr[m];
                        o[m][vb][2] *= corr[m];
                        o[m][vb][3] *= corr[m];
                    }
                }
                const bool on_d = vb * 16 + col < vdim;
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) {
                    da_s16x4 v = vt[mb][vb];
                    if (!whole) {
                        const int key = k0 + mb * 16 + quad * 4;     // what lies past the last query's position is not a value yet
                        if (key + 1 > pos_last) v[1] = 0;
                        if (key + 2 > pos_last) v[2] = 0;
                        if (key + 3 > pos_last) v[3] = 0;
                        if (!cur.there[mb] || key > pos_last) v = da_s16x4{0, 0, 0, 0};
                    }
                    if (!on_d) v = da_s16x4{0, 0, 0, 0};
                    o[0][vb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v, pb[0][mb], o[0][vb], 0, 0, 0);
                    o[1][vb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v, pb[1][mb], o[1][vb], 0, 0, 0);
                }
            }
        }
        cur = nxt;
    }
    // finish: a lane holds value dimensions 16 vb + 4 quad + i of query `col`
    const float i1 = sum[0] > 0.f ? 1.0f / sum[0] : 0.f, i2 = sum[1] > 0.f ? 1.0f / sum[1] : 0.f;
    float ss = 0.f;
#pragma unroll
    for (int vb = 0; vb < V16; ++vb)
        if (vb < vd16) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool on = vb * 16 + quad * 4 + i < vdim;
                const float v = on ? o[0][vb][i] * i1 - lambda * (o[1][vb][i] * i2) : 0.f;
                o[0][vb][i] = v;
                ss += v * v;
            }
        }
    ss += __shfl_xor(ss, 16, WAVE);
    ss += __shfl_xor(ss, 32, WAVE);
    const float rr = out_scale / sqrtf(ss / (float)vdim + eps);
    if (col < n_q) {
        const float* gt = gate ? gate + (size_t)t * gate_ld + (size_t)h * vdim : nullptr;
        bf16_t* dst = out + ((size_t)t * heads + h) * vdim;
#pragma unroll
        for (int vb = 0; vb < V16; ++vb)
            if (vb < vd16) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int d = vb * 16 + quad * 4 + i;
                    if (d < vdim) {
                        float y = o[0][vb][i] * rr;
                        if (gt) y *= 1.0f / (1.0f + __expf(-gt[d]));
                        dst[d] = f32_to_bf16(y);
                    }
                }
            }
    }
}

// The same walk with every tile staged once a block: the four waves of a block (64 consecutive queries
// of one head) walk the same keys, so each tile of 32 keys is brought into LDS by all 256 threads
// together, K rows as they lie (rows 8 bytes apart from a power of two, so that the operand reads of 16
// rows spread over the banks) and V transposed on the way in, [value dimension][key], so that the second
// product's operand, four consecutive keys of one value dimension, is one 8-byte read. The next tile's
// global loads are in flight in registers while this tile's products run. For dim and vdim multiples of 8.
#define DAS_KPAD 4           // bf16 elements between K rows in LDS beyond dim
#define DAS_VROW 36          // bf16 elements of a V^T row in LDS: 32 keys + 4

template <int D16, int V16>
__global__ __launch_bounds__(256, 2) void k_diff_attention_shared(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const float* __restrict__ gate, int gate_ld, bf16_t* __restrict__ out, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
    const int32_t* __restrict__ block_table, int table_stride, int page_size, int heads, int kv_heads, int dim,
    int vdim, int n_pages, float scale, int window, float lambda, float eps, float out_scale, int min_len) {
    __shared__ __attribute__((aligned(16))) bf16_t k_lds[2 * 32 * (16 * D16 + DAS_KPAD)];
    __shared__ __attribute__((aligned(16))) bf16_t v_lds[16 * V16 * DAS_VROW];
    const int r = blockIdx.x, h = blockIdx.z;
    const int len = seg_len[r];
    if (len < min_len) return;                                 // (uniform over the block)
    // the last queries walk the most keys: their blocks go first (blocks start in the order of their numbers)
    const int b0 = ((int)gridDim.y - 1 - (int)blockIdx.y) * DAM_TILE;     // the block's first query within the portion
    if (b0 >= len) return;                                     // (uniform over the block)
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int col = lane & 15, quad = lane >> 4;
    const int t0 = seg_start[r];
    const int q0 = b0 + wave * 16;
    const bool wave_on = q0 < len;                             // a wave past the portion helps to stage and computes nothing
    const int n_q = wave_on ? min(16, len - q0) : 1;
    const int qi = wave_on ? min(col, n_q - 1) : 0;
    const int t = t0 + (wave_on ? q0 + qi : b0);
    const int pos = positions[t];
    const int pos_first = positions[t0 + (wave_on ? q0 : b0)], pos_last = positions[t0 + (wave_on ? q0 + n_q - 1 : b0)];
    const int block_first = positions[t0 + b0], block_last = positions[t0 + min(b0 + DAM_TILE, len) - 1];
    const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
    const int lo_first = window > 0 ? max(0, pos_first + 1 - window) : 0;
    const int lo_last = window > 0 ? max(0, pos_last + 1 - window) : 0;
    const int lo_block = window > 0 ? max(0, block_first + 1 - window) : 0;
    const int g = h / (heads / kv_heads);
    const int vd16 = (vdim + 15) >> 4;
    const int krow = dim + DAS_KPAD;
    const int page_shift = __ffs(page_size) - 1, page_mask = page_size - 1;     // pages are a power of two
    const int32_t* table = block_table + (size_t)r * table_stride;

    da_s16x4 qf[2][D16];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int kk = 0; kk < D16; ++kk) {
            const int d = kk * 16 + quad * 4;
            const da_s16x4 v = *reinterpret_cast<const da_s16x4*>(q + (((size_t)t * heads + h) * 2 + m) * dim + min(d, dim - 4));
            qf[m][kk] = d < dim ? v : da_s16x4{0, 0, 0, 0};
        }
    da_f32x4 o[2][V16];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int vb = 0; vb < V16; ++vb) o[m][vb] = da_f32x4{0.f, 0.f, 0.f, 0.f};
    float mx[2] = {-INFINITY, -INFINITY}, sum[2] = {0.f, 0.f};

    // staging: a thread's 16-byte pieces of the K tile (64 rows: map, key) and of the V tile (32 rows: key)
    constexpr int KP = (2 * 32 * 2 * D16 + 255) / 256;         // pieces of 8 elements a thread, K: 64 rows x dim / 8
    constexpr int VP = (32 * 2 * V16 + 255) / 256;             // V: 32 rows x vdim / 8
    const int k_per_row = dim >> 3, v_per_row = vdim >> 3;
    uint4 kreg[KP], vreg[VP];
    // which piece of a tile a thread brings does not change from tile to tile
    int k_row[KP], k_part[KP], v_key[VP], v_part[VP];
    bool k_in[KP], v_in[VP];
#pragma unroll
    for (int i = 0; i < KP; ++i) {
        const int c = threadIdx.x + i * 256;
        k_in[i] = c < 64 * k_per_row;
        k_row[i] = min(c / k_per_row, 63);
        k_part[i] = c - (c / k_per_row) * k_per_row;
    }
#pragma unroll
    for (int i = 0; i < VP; ++i) {
        const int c = threadIdx.x + i * 256;
        v_in[i] = c < 32 * v_per_row;
        v_key[i] = min(c / v_per_row, 31);
        v_part[i] = c - (c / v_per_row) * v_per_row;
    }
    auto ask = [&](int k0) {
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            const int m = k_row[i] >> 5, key = k_row[i] & 31;
            const int key0 = k0 + (key & 16);
            const int page = key0 <= block_last ? table[key0 >> page_shift] : -1;
            const bool on = page >= 0 && page < n_pages && k_in[i];
            const long long pg = on ? page : 0;
            const uint4 v = *reinterpret_cast<const uint4*>(
                k_cache + ((pg * 2 * kv_heads + 2 * g + m) * page_size + ((k0 + key) & page_mask)) * dim + k_part[i] * 8);
            kreg[i] = on ? v : uint4{0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            const int key = v_key[i];
            const int key0 = k0 + (key & 16);
            const int page = key0 <= block_last ? table[key0 >> page_shift] : -1;
            // what lies past the block's last position is not a value yet: zeros, which weigh nothing
            const bool on = page >= 0 && page < n_pages && v_in[i] && k0 + key <= block_last;
            const long long pg = on ? page : 0;
            const uint4 v = *reinterpret_cast<const uint4*>(
                v_cache + ((pg * kv_heads + g) * page_size + ((k0 + key) & page_mask)) * (long long)vdim + v_part[i] * 8);
            vreg[i] = on ? v : uint4{0, 0, 0, 0};
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            if (k_in[i]) {
                // rows lie krow elements apart: 8 bytes past a multiple of 16, so a piece goes in two halves
                uint2* dst = reinterpret_cast<uint2*>(k_lds + k_row[i] * krow + k_part[i] * 8);
                dst[0] = uint2{kreg[i].x, kreg[i].y};
                dst[1] = uint2{kreg[i].z, kreg[i].w};
            }
        }
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            if (v_in[i]) {
                const uint32_t w[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
                bf16_t* dst = v_lds + (v_part[i] * 8) * DAS_VROW + v_key[i];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    dst[(2 * e) * DAS_VROW] = (bf16_t)(w[e] & 0xffff);
                    dst[(2 * e + 1) * DAS_VROW] = (bf16_t)(w[e] >> 16);
                }
            }
        }
    };

    int k0 = (lo_block / 32) * 32;
    ask(k0);
    stage();
    __syncthreads();
    for (; k0 <= block_last; k0 += 32) {
        if (k0 + 32 <= block_last) ask(k0 + 32);               // (uniform over the block)
        if (wave_on && k0 <= pos_last && k0 + 31 >= lo_first) {
            da_s16x4 pb[2][2];
            float corr[2];
            bool there[2];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
                const int key0 = k0 + mb * 16;
                const int page = key0 <= pos_last ? table[key0 >> page_shift] : -1;
                there[mb] = page >= 0 && page < n_pages;
            }
            const bool whole = there[0] && there[1] && k0 + 31 <= pos_first && k0 >= lo_last;
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                da_f32x4 sc[2] = {da_f32x4{0.f, 0.f, 0.f, 0.f}, da_f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                    for (int kk = 0; kk < D16; ++kk) {
                        const int d = min(kk * 16 + quad * 4, dim - 4);
                        const da_s16x4 kf = *reinterpret_cast<const da_s16x4*>(k_lds + (m * 32 + mb * 16 + col) * krow + d);
                        sc[mb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kf, qf[m][kk], sc[mb], 0, 0, 0);
                    }
                float tile_max = -INFINITY;
                if (whole) {
#pragma unroll
                    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            sc[mb][i] *= scale;
                            tile_max = fmaxf(tile_max, sc[mb][i]);
                        }
                } else {
#pragma unroll
                    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int key = k0 + mb * 16 + quad * 4 + i;
                            const bool seen = there[mb] && key <= pos && key >= lo;
                            sc[mb][i] = seen ? sc[mb][i] * scale : -INFINITY;
                            tile_max = fmaxf(tile_max, sc[mb][i]);
                        }
                }
                tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE));
                tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE));
                const float m_new = fmaxf(mx[m], tile_max);
                const float m_use = m_new == -INFINITY ? 0.f : m_new;
                corr[m] = mx[m] == -INFINITY ? 0.f : __expf(mx[m] - m_use);
                float tile_sum = 0.f;
                float p[2][4];
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        p[mb][i] = __expf(sc[mb][i] - m_use);
                        tile_sum += p[mb][i];
                    }
                tile_sum += __shfl_xor(tile_sum, 16, WAVE);
                tile_sum += __shfl_xor(tile_sum, 32, WAVE);
                sum[m] = sum[m] * corr[m] + tile_sum;
                mx[m] = m_new;
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) pb[m][mb] = da_pack4(p[mb][0], p[mb][1], p[mb][2], p[mb][3]);
            }
            const bool rescale = __any(corr[0] != 1.0f || corr[1] != 1.0f);
#pragma unroll
            for (int vb = 0; vb < V16; ++vb) {
                if (vb < vd16) {
                    if (rescale) {
#pragma unroll
                        for (int m = 0; m < 2; ++m) {
                            o[m][vb][0] *= corr[m];
                            o[m][vb][1] *= corr[m];
                            o[m][vb][2] *= corr[m];
                            o[m][vb][3] *= corr[m];
                        }
                    }
                    const int d = min(vb * 16 + col, vdim - 1);
                    const bool on_d = vb * 16 + col < vdim;
#pragma unroll
                    for (int mb = 0; mb < 2; ++mb) {
                        // keys 4 quad .. + 3 of the block, value dimension d: eight bytes of a V^T row. A key that this
                        // wave's queries do not see weighs nothing (its P is zero) and its value is finite or zero
                        da_s16x4 v = *reinterpret_cast<const da_s16x4*>(v_lds + d * DAS_VROW + mb * 16 + quad * 4);
                        if (!on_d) v = da_s16x4{0, 0, 0, 0};
                        o[0][vb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v, pb[0][mb], o[0][vb], 0, 0, 0);
                        o[1][vb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v, pb[1][mb], o[1][vb], 0, 0, 0);
                    }
                }
            }
        }
        __syncthreads();                                       // every wave has read this tile
        if (k0 + 32 <= block_last) stage();
        __syncthreads();
    }
    if (!wave_on) return;
    const float i1 = sum[0] > 0.f ? 1.0f / sum[0] : 0.f, i2 = sum[1] > 0.f ? 1.0f / sum[1] : 0.f;
    float ss = 0.f;
#pragma unroll
    for (int vb = 0; vb < V16; ++vb)
        if (vb < vd16) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool on = vb * 16 + quad * 4 + i < vdim;
                const float v = on ? o[0][vb][i] * i1 - lambda * (o[1][vb][i] * i2) : 0.f;
                o[0][vb][i] = v;
                ss += v * v;
            }
        }
    ss += __shfl_xor(ss, 16, WAVE);
    ss += __shfl_xor(ss, 32, WAVE);
    const float rr = out_scale / sqrtf(ss / (float)vdim + eps);
    if (col < n_q) {
        const float* gt = gate ? gate + (size_t)t * gate_ld + (size_t)h * vdim : nullptr;
        bf16_t* dst = out + ((size_t)t * heads + h) * vdim;
#pragma unroll
        for (int vb = 0; vb < V16; ++vb)
            if (vb < vd16) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int d = vb * 16 + quad * 4 + i;
                    if (d < vdim) {
                        float y = o[0][vb][i] * rr;
                        if (gt) y *= 1.0f / (1.0f + __expf(-gt[d]));
                        dst[d] = f32_to_bf16(y);
                    }
                }
            }
    }
}

// Whether the matrix-core kernel takes these sizes (bfloat16 only).
extern "C" int imparo_diff_attention_tiles_takes(int page_size, int dim, int vdim) {
    return page_size >= 16 && page_size % 16 == 0 && dim > 0 && vdim > 0 && dim % 4 == 0 && vdim % 4 == 0 &&
           dim <= 16 * DAM_MAX16 && vdim <= 16 * DAM_MAX16;
}

// Differential attention of whole portions: every token of every row (seg_start, seg_len) of at least min_len
// tokens, a row's tokens at consecutive positions. max_seg_len bounds every row's tokens. Sizes as imparo_diff_attention_tiles_takes says.
extern "C" int imparo_diff_attention_tiles(const void* q, const void* k_cache, const void* v_cache, const float* gate,
                                           int gate_ld, void* out, const int32_t* positions, const int32_t* seg_start,
                                           const int32_t* seg_len, const int32_t* block_table, int table_stride,
                                           int page_size, int n_rows, int max_seg_len, int heads, int kv_heads, int dim,
                                           int vdim, int n_pages, float scale, int window, float lambda, float eps,
                                           float out_scale, int min_len, imparo_stream stream) {
    if (!q || !k_cache || !v_cache || !out || !positions || !seg_start || !seg_len || !block_table) return IMPARO_BAD_ARGUMENT;
    if (n_rows < 0 || max_seg_len < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads) return IMPARO_BAD_ARGUMENT;
    if (!imparo_diff_attention_tiles_takes(page_size, dim, vdim)) return IMPARO_BAD_ARGUMENT;
    if (table_stride <= 0 || n_pages <= 0 || window < 0 || heads > 65535) return IMPARO_BAD_ARGUMENT;
    if (gate && gate_ld < heads * vdim) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0 || max_seg_len == 0) return IMPARO_OK;
    const int tiles = (max_seg_len + DAM_TILE - 1) / DAM_TILE;
    if (tiles > 65535) return IMPARO_BAD_ARGUMENT;
    dim3 grid(n_rows, tiles, heads);
#define DAM_LAUNCH(D16, V16)                                                                                             \
    k_diff_attention_tiles<D16, V16><<<grid, 256, 0, (hipStream_t)stream>>>(                                              \
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, gate, gate_ld, (bf16_t*)out, positions, seg_start, \
        seg_len, block_table, table_stride, page_size, heads, kv_heads, dim, vdim, n_pages, scale, window, lambda, eps,   \
        out_scale, min_len)
#define DAS_LAUNCH(D16, V16)                                                                                             \
    k_diff_attention_shared<D16, V16><<<grid, 256, 0, (hipStream_t)stream>>>(                                             \
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, gate, gate_ld, (bf16_t*)out, positions, seg_start, \
        seg_len, block_table, table_stride, page_size, heads, kv_heads, dim, vdim, n_pages, scale, window, lambda, eps,   \
        out_scale, min_len)
    if (dim % 8 == 0 && vdim % 8 == 0 && (page_size & (page_size - 1)) == 0) {          // every tile staged once a block in LDS
        if (dim <= 64 && vdim <= 64) DAS_LAUNCH(4, 4);
        else if (dim <= 64) DAS_LAUNCH(4, 8);
        else if (vdim <= 64) DAS_LAUNCH(8, 4);
        else DAS_LAUNCH(8, 8);
    } else if (dim <= 64 && vdim <= 64) DAM_LAUNCH(4, 4);
    else if (dim <= 64) DAM_LAUNCH(4, 8);
    else if (vdim <= 64) DAM_LAUNCH(8, 4);
    else DAM_LAUNCH(8, 8);
#undef DAS_LAUNCH
#undef DAM_LAUNCH
    return launch_status();
}

extern "C" int imparo_diff_qkv_store(const float* rows_in, int ld, const int32_t* positions, const int32_t* row_of_token,
                                     const int32_t* block_table, int table_stride, int page_size, void* q_out,
                                     void* k_cache, void* v_cache, int dtype, int write_kv, int n_tokens, int heads,
                                     int kv_heads, int dim, int vdim, int n_pages, float temp_coef, int temp_every,
                                     imparo_stream stream) {
    if (!rows_in || !positions || !row_of_token || !q_out) return IMPARO_BAD_ARGUMENT;
    if (write_kv && (!block_table || !k_cache || !v_cache || table_stride <= 0 || n_pages <= 0)) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || vdim <= 0 || page_size <= 0)
        return IMPARO_BAD_ARGUMENT;
    if (ld < (heads + kv_heads) * 2 * dim + kv_heads * vdim || temp_every < 0) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == IMPARO_F32)
        k_diff_qkv_store<float><<<n_tokens, 256, 0, s>>>(rows_in, ld, positions, row_of_token, block_table, table_stride,
                                                         page_size, (float*)q_out, (float*)k_cache, (float*)v_cache, write_kv,
                                                         heads, kv_heads, dim, vdim, n_pages, temp_coef, temp_every);
    else if (dtype == IMPARO_BF16)
        k_diff_qkv_store<bf16_t><<<n_tokens, 256, 0, s>>>(rows_in, ld, positions, row_of_token, block_table, table_stride,
                                                          page_size, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache,
                                                          write_kv, heads, kv_heads, dim, vdim, n_pages, temp_coef, temp_every);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// q [tokens, heads, 2, dim]; gate (may be null) float32 rows gate_ld apart, heads * vdim values a row, the
// gate's logits; out [tokens, heads * vdim]. n_splits 1: no partial results; more: part holds
// tokens * heads * n_splits * (2 vdim + 4) floats and n_splits covers every key (ceil(longest context / split)).
// below > 0: only the tokens of rows that bring fewer than `below` tokens (seg_len per row); the others' outputs
// are left as they are.
extern "C" int imparo_diff_attention(const void* q, const void* k_cache, const void* v_cache, const float* gate,
                                     int gate_ld, void* out, float* part, int dtype, const int32_t* positions,
                                     const int32_t* row_of_token, const int32_t* block_table, int table_stride,
                                     int page_size, int n_tokens, int heads, int kv_heads, int dim, int vdim,
                                     int n_pages, float scale, int window, float lambda, float eps, float out_scale,
                                     int n_splits, const int32_t* seg_len, int below, imparo_stream stream) {
    if (!q || !k_cache || !v_cache || !out || !positions || !row_of_token || !block_table) return IMPARO_BAD_ARGUMENT;
    if (below < 0 || (below > 0 && !seg_len)) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads) return IMPARO_BAD_ARGUMENT;
    if (dim <= 0 || dim > DA_MAX_DIM || vdim <= 0 || vdim > DA_MAX_VDIM) return IMPARO_BAD_ARGUMENT;
    if (page_size <= 0 || table_stride <= 0 || n_pages <= 0 || window < 0 || n_splits < 1) return IMPARO_BAD_ARGUMENT;
    if (n_splits > 1 && !part) return IMPARO_BAD_ARGUMENT;
    if (gate && gate_ld < heads * vdim) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    const long long total = (long long)n_tokens * heads * n_splits;
    const long long blocks = (total + DA_WAVES - 1) / DA_WAVES;
    if (blocks > 0x7fffffffLL) return IMPARO_BAD_ARGUMENT;
    hipStream_t s = (hipStream_t)stream;
    const unsigned merge_blocks = (unsigned)(((long long)n_tokens * heads + DA_WAVES - 1) / DA_WAVES);
    if (dtype != IMPARO_F32 && dtype != IMPARO_BF16) return IMPARO_BAD_ARGUMENT;
#define DA_LAUNCH(T, VPL)                                                                                              \
    do {                                                                                                               \
        k_diff_attention<T, VPL><<<(unsigned)blocks, DA_WAVES * WAVE, 0, s>>>(                                          \
            (const T*)q, (const T*)k_cache, (const T*)v_cache, gate, gate_ld, (T*)out, part, positions, row_of_token,  \
            block_table, table_stride, page_size, n_tokens, heads, kv_heads, dim, vdim, n_pages, scale, window, lambda, \
            eps, out_scale, n_splits, seg_len, below);                                                                 \
        if (n_splits > 1) {                                                                                            \
            if (launch_status()) return IMPARO_LAUNCH_FAILED;                                                          \
            k_diff_merge<T, VPL><<<merge_blocks, DA_WAVES * WAVE, 0, s>>>(part, gate, gate_ld, (T*)out, positions,      \
                                                                         n_tokens, heads, vdim, window, lambda, eps,  \
                                                                         out_scale, n_splits, row_of_token, seg_len,   \
                                                                         below);                                       \
        }                                                                                                              \
    } while (0)
#define DA_LAUNCH_T(T)                  \
    do {                                \
        if (vdim <= 64) DA_LAUNCH(T, 1);       \
        else if (vdim <= 128) DA_LAUNCH(T, 2); \
        else if (vdim <= 256) DA_LAUNCH(T, 4); \
        else DA_LAUNCH(T, 8);                  \
    } while (0)
    if (dtype == IMPARO_F32) DA_LAUNCH_T(float);
    else DA_LAUNCH_T(bf16_t);
#undef DA_LAUNCH_T
#undef DA_LAUNCH
    return launch_status();
}

int imparo_load_code_diff_attention() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_diff_attention<float, 1>)) == hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
