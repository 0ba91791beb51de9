// Row-wise kernels of layers that norm in groups, mix a token's input with the token before it, add a
// sinusoidal position vector to the embedding, or use a polynomial of unit-RMS powers as activation.
// Everything here sums and norms in float32; outputs go out in float32 or bfloat16.
#include "common.h"
#include "api.h"

// ---------------------------------------------------------------- embedding + sinusoidal position
// x[t, 2i] = table[id, 2i] + sin(pos * inv_freq[i]), x[t, 2i+1] = table[id, 2i+1] + cos(same angle).
template <typename T>
__global__ void k_embed_sinusoid(const T* __restrict__ table, const int32_t* __restrict__ ids,
                                 const int32_t* __restrict__ positions, const float* __restrict__ inv_freq,
                                 float* __restrict__ x, int width) {
    const int t = blockIdx.x;
    const size_t src = (size_t)ids[t] * width;
    const size_t dst = (size_t)t * width;
    const int pos = positions[t];
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float sn, cs;
        rotation_of(pos, inv_freq[i >> 1], sn, cs);
        x[dst + i] = load_f32<T>(table, src + i) + ((i & 1) ? cs : sn);
    }
}

extern "C" int imparo_embed_sinusoid(const void* table, int table_dtype, const int32_t* ids, const int32_t* positions,
                                     const float* inv_freq, float* x, int n_tokens, int width, int vocab,
                                     imparo_stream stream) {
    if (!table || !ids || !positions || !inv_freq || !x || n_tokens < 0 || width <= 0 || vocab <= 0)
        return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const int threads = width >= 1024 ? 256 : 64;
    if (table_dtype == IMPARO_F32)
        k_embed_sinusoid<float><<<n_tokens, threads, 0, s>>>((const float*)table, ids, positions, inv_freq, x, width);
    else if (table_dtype == IMPARO_BF16)
        k_embed_sinusoid<bf16_t><<<n_tokens, threads, 0, s>>>((const bf16_t*)table, ids, positions, inv_freq, x, width);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// ---------------------------------------------------------------- RMS norm in groups
// One block per output row, one wave per group at a time: the row is cut into `groups` equal
// consecutive parts and each is divided by its own sqrt(mean(part^2) + eps); the whole is multiplied by
// the weight. The residual add is fused as in the plain norm (delta slices added in order, write_back).
// With shift_mix (rows of one token each, row i in slot[i]): the normed row h is mixed with the row
// the request's last token left, out = h + (prev - h) * mix, and h becomes the new prev: the token
// shift of a decode step in the norm's launch.
// PER: values of a group a lane keeps in registers (a group of up to 64 PER values is read once, every
// load asked for before any is used; a wider group, PER 0, is walked twice).
template <typename TOut, int PER>
__global__ void k_group_rms_norm(float* __restrict__ x, const float* __restrict__ delta, int n_delta,
                                 size_t delta_stride, const int32_t* __restrict__ rows,
                                 const float* __restrict__ weight, TOut* __restrict__ out, int width, int groups,
                                 float eps, int write_back, const float* __restrict__ shift_mix,
                                 float* __restrict__ shift_state, const int32_t* __restrict__ slot) {
    const int i_out = blockIdx.x;
    const size_t src = (size_t)(rows ? rows[i_out] : i_out) * width;
    const size_t dst = (size_t)i_out * width;
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const int n_waves = blockDim.x / WAVE;
    const int gw = width / groups;
    float* st = shift_mix ? shift_state + (size_t)slot[i_out] * width : nullptr;
    for (int g = wave; g < groups; g += n_waves) {
        const int first = g * gw;
        if constexpr (PER > 0) {
            float v[PER], d[PER], w[PER], prev[PER], mix[PER];
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                const int i = first + min(lane + j * WAVE, gw - 1);   // lanes past the group repeat its end and store nothing
                v[j] = x[src + i];
                w[j] = weight[i];
                prev[j] = st ? st[i] : 0.f;
                mix[j] = shift_mix ? shift_mix[i] : 0.f;
                d[j] = 0.f;
            }
            for (int s = 0; s < n_delta; ++s) {            // the slices make up the delta first, then the delta joins x
                float p[PER];
#pragma unroll
                for (int j = 0; j < PER; ++j) p[j] = delta[s * delta_stride + src + first + min(lane + j * WAVE, gw - 1)];
#pragma unroll
                for (int j = 0; j < PER; ++j) d[j] += p[j];
            }
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                const bool in = lane + j * WAVE < gw;
                v[j] += d[j];
                if (write_back && in) x[src + first + lane + j * WAVE] = v[j];
                ss += in ? v[j] * v[j] : 0.f;
            }
            ss = wave_sum(ss);
            const float scale = 1.0f / sqrtf(ss / (float)gw + eps);
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                const int i = first + lane + j * WAVE;
                if (lane + j * WAVE < gw) {
                    float h = v[j] * scale * w[j];
                    if (shift_mix) {
                        st[i] = h;
                        h = h + (prev[j] - h) * mix[j];
                    }
                    store_f32<TOut>(out, dst + i, h);
                }
            }
        } else {
            float ss = 0.f;
            for (int i = lane; i < gw; i += WAVE) {
                float a = x[src + first + i];
                float d = 0.f;
                for (int s = 0; s < n_delta; ++s) d += delta[s * delta_stride + src + first + i];
                a += d;
                if (write_back) x[src + first + i] = a;
                ss += a * a;
            }
            ss = wave_sum(ss);
            const float scale = 1.0f / sqrtf(ss / (float)gw + eps);
            for (int i = lane; i < gw; i += WAVE) {
                float a = x[src + first + i];          // with write_back: what this lane stored above
                if (!write_back) {
                    float d = 0.f;
                    for (int s = 0; s < n_delta; ++s) d += delta[s * delta_stride + src + first + i];
                    a += d;
                }
                float h = a * scale * weight[first + i];
                if (shift_mix) {
                    const float prev = st[first + i];
                    st[first + i] = h;
                    h = h + (prev - h) * shift_mix[first + i];
                }
                store_f32<TOut>(out, dst + first + i, h);
            }
        }
    }
}

template <typename TOut>
static void launch_group_norm(int per, int n_rows, int threads, hipStream_t s, float* x, const float* delta, int n_delta,
                              size_t delta_stride, const int32_t* rows, const float* weight, void* out, int width,
                              int groups, float eps, int write_back, const float* shift_mix, float* shift_state,
                              const int32_t* slot) {
#define GN_LAUNCH(PER)                                                                                                    \
    k_group_rms_norm<TOut, PER><<<n_rows, threads, 0, s>>>(x, delta, n_delta, delta_stride, rows, weight, (TOut*)out, width, \
                                                           groups, eps, write_back, shift_mix, shift_state, slot)
    if (per <= 1) GN_LAUNCH(1);
    else if (per <= 2) GN_LAUNCH(2);
    else if (per <= 4) GN_LAUNCH(4);
    else if (per <= 8) GN_LAUNCH(8);
    else if (per <= 16) GN_LAUNCH(16);
    else GN_LAUNCH(0);
#undef GN_LAUNCH
}

extern "C" int imparo_group_rms_norm(float* x, const float* delta, int n_delta, int n_x_rows, const int32_t* rows,
                                     const float* weight, void* out, int out_dtype, int n_rows, int width, int groups,
                                     float eps, int write_back, const float* shift_mix, float* shift_state,
                                     const int32_t* slot, imparo_stream stream) {
    if (!x || !weight || !out || n_rows < 0 || width <= 0 || groups <= 0 || width % groups) return IMPARO_BAD_ARGUMENT;
    if (n_delta < 0 || n_delta > 64 || (n_delta > 0 && !delta) || n_x_rows < 0) return IMPARO_BAD_ARGUMENT;
    if (write_back && rows) return IMPARO_BAD_ARGUMENT;
    if (shift_mix && (!shift_state || !slot || rows)) return IMPARO_BAD_ARGUMENT;
    if (!delta) n_delta = 0;
    if (n_rows == 0) return IMPARO_OK;
    const size_t delta_stride = (size_t)n_x_rows * width;
    const int threads = WAVE * (groups < 16 ? groups : 16);      // a wave a group, up to sixteen at once
    hipStream_t s = (hipStream_t)stream;
    const int per = (width / groups + WAVE - 1) / WAVE;
    if (out_dtype == IMPARO_F32)
        launch_group_norm<float>(per, n_rows, threads, s, x, delta, n_delta, delta_stride, rows, weight, out, width, groups,
                                 eps, write_back, shift_mix, shift_state, slot);
    else if (out_dtype == IMPARO_BF16)
        launch_group_norm<bf16_t>(per, n_rows, threads, s, x, delta, n_delta, delta_stride, rows, weight, out, width, groups,
                                  eps, write_back, shift_mix, shift_state, slot);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// ---------------------------------------------------------------- token shift
// out[t] = h[t] + (prev - h[t]) * mix, prev = h[t - 1] inside a request's segment and the request's
// state (what its last token left; zeros for a new request) at the segment's first token. The state is
// read here and written by k_token_shift_state, a launch of its own behind this one: a segment's first
// token reads the state that its last token replaces.
template <typename TOut>
__global__ void k_token_shift(const float* __restrict__ h, const float* __restrict__ mix,
                              const float* __restrict__ state, const int32_t* __restrict__ row_of_token,
                              const int32_t* __restrict__ seg_start, const int32_t* __restrict__ slot,
                              TOut* __restrict__ out, int width) {
    const int t = blockIdx.x;
    const int r = row_of_token[t];
    const float* prev = t > seg_start[r] ? h + (size_t)(t - 1) * width : state + (size_t)slot[r] * width;
    const float* cur = h + (size_t)t * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float a = cur[i];
        store_f32<TOut>(out, (size_t)t * width + i, a + (prev[i] - a) * mix[i]);
    }
}

__global__ void k_token_shift_state(const float* __restrict__ h, float* __restrict__ state,
                                    const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
                                    const int32_t* __restrict__ slot, int width) {
    const int r = blockIdx.x;
    const int n = seg_len[r];
    if (n <= 0) return;
    const float* last = h + (size_t)(seg_start[r] + n - 1) * width;
    float* st = state + (size_t)slot[r] * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) st[i] = last[i];
}

extern "C" int imparo_token_shift(const float* h, const float* mix, float* state, const int32_t* row_of_token,
                                  const int32_t* seg_start, const int32_t* seg_len, const int32_t* slot, void* out,
                                  int out_dtype, int n_tokens, int n_rows, int width, imparo_stream stream) {
    if (!h || !mix || !state || !row_of_token || !seg_start || !seg_len || !slot || !out) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || n_rows < 0 || width <= 0) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0 || n_rows == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const int threads = width >= 1024 ? 256 : 64;
    if (out_dtype == IMPARO_F32)
        k_token_shift<float><<<n_tokens, threads, 0, s>>>(h, mix, state, row_of_token, seg_start, slot, (float*)out, width);
    else if (out_dtype == IMPARO_BF16)
        k_token_shift<bf16_t><<<n_tokens, threads, 0, s>>>(h, mix, state, row_of_token, seg_start, slot, (bf16_t*)out, width);
    else
        return IMPARO_BAD_ARGUMENT;
    if (launch_status()) return IMPARO_LAUNCH_FAILED;
    k_token_shift_state<<<n_rows, threads, 0, s>>>(h, state, seg_start, seg_len, slot, width);
    return launch_status();
}

// ---------------------------------------------------------------- polynomial activation of unit-RMS powers
// out = a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, N(v) = v / sqrt(mean(v^2) + eps)
// over the `width` values of a token. coef holds a, b, c, e. z rows lie z_ld apart, out rows out_ld;
// columns from width to out_ld of out are set to zero (room that a product's inner size was filled up to).
// PER: values a thread keeps in registers (rows of up to blockDim * PER values are read once).
template <typename TOut, int PER>
__global__ void k_poly_norm(const float* __restrict__ z, int z_ld, const float* __restrict__ coef,
                            TOut* __restrict__ out, int out_ld, int width, float eps) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const float* row = z + (size_t)t * z_ld;
    float v[PER];
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        v[j] = row[min(i, width - 1)];
        if (i >= width) v[j] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const float v2 = v[j] * v[j];
        const float v3 = v2 * v[j];
        s2 += v2;
        s4 += v2 * v2;
        s6 += v3 * v3;
    }
    for (int i = threadIdx.x + PER * blockDim.x; i < width; i += blockDim.x) {     // a row wider than the registers hold
        const float a = row[i];
        const float a2 = a * a;
        const float a3 = a2 * a;
        s2 += a2;
        s4 += a2 * a2;
        s6 += a3 * a3;
    }
    s2 = block_sum(s2, scratch);
    s4 = block_sum(s4, scratch);
    s6 = block_sum(s6, scratch);
    const float n = (float)width;
    const float r1 = coef[0] / sqrtf(s2 / n + eps);
    const float r2 = coef[1] / sqrtf(s4 / n + eps);
    const float r3 = coef[2] / sqrtf(s6 / n + eps);
    const float e = coef[3];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        if (i < out_ld) {
            const float v2 = v[j] * v[j];
            store_f32<TOut>(out, (size_t)t * out_ld + i, i < width ? r1 * v[j] + r2 * v2 + r3 * (v2 * v[j]) + e : 0.f);
        }
    }
    for (int i = threadIdx.x + PER * blockDim.x; i < out_ld; i += blockDim.x) {
        float y = 0.f;
        if (i < width) {
            const float a = row[i];
            const float a2 = a * a;
            y = r1 * a + r2 * a2 + r3 * (a2 * a) + e;
        }
        store_f32<TOut>(out, (size_t)t * out_ld + i, y);
    }
}

extern "C" int imparo_poly_norm(const float* z, int z_ld, const float* coef, void* out, int out_dtype, int out_ld,
                                int n_tokens, int width, float eps, imparo_stream stream) {
    if (!z || !coef || !out || n_tokens < 0 || width <= 0 || z_ld < width || out_ld < width) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    // few rows: many threads a row, so that a row's loads are all in flight at once; the sums' order depends on
    // the width only
    const int threads = width >= 8192 ? 1024 : width >= 2048 ? 512 : width >= 512 ? 256 : 64;
    if (out_dtype == IMPARO_F32)
        k_poly_norm<float, 8><<<n_tokens, threads, 0, s>>>(z, z_ld, coef, (float*)out, out_ld, width, eps);
    else if (out_dtype == IMPARO_BF16)
        k_poly_norm<bf16_t, 8><<<n_tokens, threads, 0, s>>>(z, z_ld, coef, (bf16_t*)out, out_ld, width, eps);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (a stream under capture cannot).
int imparo_load_code_row_ops() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_token_shift_state)) == hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
