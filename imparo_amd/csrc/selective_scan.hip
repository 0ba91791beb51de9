// Kernels of a selective state-space mixer: the causal per-channel convolution with its rolling
// history, and the selective scan with its float32 state per request.
//
// Convolution: y[t, c] = act(b[c] + sum_k w[c, k] u[t - (taps - 1) + k, c]), u the request's inputs with
// zeros before its start; the last taps - 1 inputs of a request are its history [slots, taps - 1, C].
// Scan, per channel c and state n:  S <- exp(dt A[c, n]) S + dt x B[n];  y = sum_n S C[n] + D x, then
// y * silu(z); dt = softplus(raw). The state lives in float32 [slots, C, N] and is carried from step to step.
#include "common.h"
#include "api.h"

#define SCAN_MAX_TAPS 64

__device__ __forceinline__ float silu_f32(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float softplus_f32(float v) { return v > 20.0f ? v : log1pf(expf(v)); }

// ---------------------------------------------------------------- causal convolution
// One thread per (token, channel). u rows lie u_ld floats apart (the x half of a wider projection).
template <typename TOut>
__global__ void k_causal_conv(const float* __restrict__ u, int u_ld, const float* __restrict__ weight,
                              const float* __restrict__ bias, const float* __restrict__ state,
                              const int32_t* __restrict__ row_of_token, const int32_t* __restrict__ seg_start,
                              const int32_t* __restrict__ slot, TOut* __restrict__ out, int channels, int taps,
                              int silu) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int t = blockIdx.x;
    if (c >= channels) return;
    const int r = row_of_token[t];
    const int t0 = seg_start[r];
    const int history = taps - 1;
    const float* st = state + (size_t)slot[r] * history * channels;
    float acc = bias ? bias[c] : 0.f;
    for (int k = 0; k < taps; ++k) {
        const int back = history - k;               // tap k looks `back` tokens back
        const int src = t - back;
        float v;
        if (src >= t0)
            v = u[(size_t)src * u_ld + c];
        else
            v = st[(size_t)(history - (t0 - src)) * channels + c];   // history row history-1 is the newest
        acc += weight[(size_t)c * taps + k] * v;
    }
    store_f32<TOut>(out, (size_t)t * channels + c, silu ? silu_f32(acc) : acc);
}

// One thread per (request, channel) owns that channel's whole history, so the update is race-free in
// place: it reads every value it needs before it writes. Works for segments shorter than the history.
__global__ void k_causal_conv_state(const float* __restrict__ u, int u_ld, float* __restrict__ state,
                                    const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
                                    const int32_t* __restrict__ slot, int channels, int taps) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int r = blockIdx.x;
    if (c >= channels) return;
    const int history = taps - 1;
    const int n = seg_len[r];
    const int t0 = seg_start[r];
    float* st = state + (size_t)slot[r] * history * channels;
    float next[SCAN_MAX_TAPS - 1];
    for (int s = 0; s < history; ++s) {
        const int e = n + s;                        // index into history ++ inputs
        next[s] = e < history ? st[(size_t)e * channels + c] : u[(size_t)(t0 + e - history) * u_ld + c];
    }
    for (int s = 0; s < history; ++s) st[(size_t)s * channels + c] = next[s];
}

// Rows of one token each: output and history shift in one launch, one thread per (row, channel).
template <typename TOut>
__global__ void k_causal_conv_single(const float* __restrict__ u, int u_ld, const float* __restrict__ weight,
                                     const float* __restrict__ bias, float* __restrict__ state,
                                     const int32_t* __restrict__ slot, TOut* __restrict__ out, int channels, int taps,
                                     int silu) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int r = blockIdx.x;
    if (c >= channels) return;
    const int history = taps - 1;
    float* st = state + (size_t)slot[r] * history * channels;
    const float now = u[(size_t)r * u_ld + c];
    float acc = bias ? bias[c] : 0.f;
    for (int k = 0; k < history; ++k) {
        const float v = st[(size_t)k * channels + c];
        acc += weight[(size_t)c * taps + k] * v;
        if (k > 0) st[(size_t)(k - 1) * channels + c] = v;
    }
    if (history > 0) st[(size_t)(history - 1) * channels + c] = now;
    acc += weight[(size_t)c * taps + history] * now;
    store_f32<TOut>(out, (size_t)r * channels + c, silu ? silu_f32(acc) : acc);
}

extern "C" int imparo_causal_conv(const float* u, int u_ld, const float* weight, const float* bias, float* state,
                                  const int32_t* row_of_token, const int32_t* seg_start, const int32_t* seg_len,
                                  const int32_t* slot, void* out, int out_dtype, int n_tokens, int n_rows, int channels,
                                  int taps, int silu, int single_tokens, imparo_stream stream) {
    if (!u || !weight || !row_of_token || !seg_start || !seg_len || !slot || !out) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || n_rows < 0 || channels <= 0 || taps < 1 || taps > SCAN_MAX_TAPS || u_ld < channels)
        return IMPARO_BAD_ARGUMENT;
    if (taps > 1 && !state) return IMPARO_BAD_ARGUMENT;
    if (single_tokens && n_tokens != n_rows) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0 || n_rows == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const int threads = channels >= 256 ? 256 : 64;
    const unsigned cb = (channels + threads - 1) / threads;
    if (cb > 65535) return IMPARO_BAD_ARGUMENT;
    if (out_dtype != IMPARO_F32 && out_dtype != IMPARO_BF16) return IMPARO_BAD_ARGUMENT;
    if (single_tokens) {
        dim3 grid(n_rows, cb);
        if (out_dtype == IMPARO_F32)
            k_causal_conv_single<float><<<grid, threads, 0, s>>>(u, u_ld, weight, bias, state, slot, (float*)out, channels, taps, silu);
        else
            k_causal_conv_single<bf16_t><<<grid, threads, 0, s>>>(u, u_ld, weight, bias, state, slot, (bf16_t*)out, channels, taps, silu);
        return launch_status();
    }
    dim3 grid(n_tokens, cb);
    if (out_dtype == IMPARO_F32)
        k_causal_conv<float><<<grid, threads, 0, s>>>(u, u_ld, weight, bias, state, row_of_token, seg_start, slot,
                                                      (float*)out, channels, taps, silu);
    else
        k_causal_conv<bf16_t><<<grid, threads, 0, s>>>(u, u_ld, weight, bias, state, row_of_token, seg_start, slot,
                                                       (bf16_t*)out, channels, taps, silu);
    if (launch_status()) return IMPARO_LAUNCH_FAILED;
    if (taps > 1) {
        dim3 rows_grid(n_rows, cb);
        k_causal_conv_state<<<rows_grid, threads, 0, s>>>(u, u_ld, state, seg_start, seg_len, slot, channels, taps);
    }
    return launch_status();
}

// ---------------------------------------------------------------- selective scan
// A block takes 256 / LP channels of one request; LP lanes (a power of two, at most 64) share a
// channel's states, SPL states a lane (n = lane + j * LP). The request's tokens are walked in order;
// a token's contribution sum_n S[n] C[n] is added up across the LP lanes by a butterfly, the same
// order whatever the batch.
template <typename TX, typename TOut, int SPL>
__global__ void k_selective_scan(const float* __restrict__ dt_raw, const TX* __restrict__ x,
                                 const float* __restrict__ bc, const float* __restrict__ z, int z_ld,
                                 const float* __restrict__ A, const float* __restrict__ D, float* __restrict__ state,
                                 const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
                                 const int32_t* __restrict__ slot, TOut* __restrict__ out, int channels, int n_state,
                                 int lp) {
    const int r = blockIdx.x;
    const int ln = threadIdx.x & (lp - 1);
    const int c = blockIdx.y * (blockDim.x / lp) + threadIdx.x / lp;
    const bool live = c < channels;
    const int cc = live ? c : channels - 1;            // lanes past the last channel repeat it and store nothing
    float S[SPL], a[SPL];
    float* st = state + ((size_t)slot[r] * channels + cc) * n_state;
#pragma unroll
    for (int j = 0; j < SPL; ++j) {
        const int n = ln + j * lp;
        const bool on = n < n_state;
        S[j] = on ? st[n] : 0.f;
        a[j] = on ? A[(size_t)cc * n_state + n] : 0.f;
    }
    const float d_skip = D[cc];
    const int t0 = seg_start[r];
    const int len = seg_len[r];
    for (int i = 0; i < len; ++i) {
        const size_t t = (size_t)(t0 + i);
        const float dt = softplus_f32(dt_raw[t * channels + cc]);
        const float xv = load_f32<TX>(x, t * channels + cc);
        const float dx = dt * xv;
        float y = 0.f;
#pragma unroll
        for (int j = 0; j < SPL; ++j) {
            const int n = ln + j * lp;
            const bool on = n < n_state;
            const int nn = on ? n : 0;
            const float b = bc[t * 2 * n_state + nn];
            const float cv = bc[t * 2 * n_state + n_state + nn];
            const float s_new = expf(dt * a[j]) * S[j] + dx * b;
            S[j] = on ? s_new : 0.f;
            y += on ? s_new * cv : 0.f;
        }
        for (int off = lp >> 1; off > 0; off >>= 1) y += __shfl_xor(y, off, WAVE);
        if (ln == 0 && live) {
            y += d_skip * xv;
            const float zv = z[t * z_ld + cc];
            store_f32<TOut>(out, t * channels + cc, y * silu_f32(zv));
        }
    }
    if (live) {
#pragma unroll
        for (int j = 0; j < SPL; ++j) {
            const int n = ln + j * lp;
            if (n < n_state) st[n] = S[j];
        }
    }
}

template <typename TX, typename TOut>
static int launch_scan(const float* dt_raw, const void* x, const float* bc, const float* z, int z_ld, const float* A,
                       const float* D, float* state, const int32_t* seg_start, const int32_t* seg_len,
                       const int32_t* slot, void* out, int n_rows, int channels, int n_state, hipStream_t s) {
    int lp = 1;
    while (lp < n_state && lp < WAVE) lp <<= 1;
    const int spl = (n_state + lp - 1) / lp;
    const int threads = 256;
    const int per_block = threads / lp;
    dim3 grid(n_rows, (channels + per_block - 1) / per_block);
    if (grid.y > 65535) return IMPARO_BAD_ARGUMENT;
#define SCAN_LAUNCH(N) \
    k_selective_scan<TX, TOut, N><<<grid, threads, 0, s>>>(dt_raw, (const TX*)x, bc, z, z_ld, A, D, state, seg_start, \
                                                           seg_len, slot, (TOut*)out, channels, n_state, lp)
    if (spl == 1) SCAN_LAUNCH(1);
    else if (spl == 2) SCAN_LAUNCH(2);
    else if (spl <= 4) SCAN_LAUNCH(4);
    else if (spl <= 8) SCAN_LAUNCH(8);
    else return IMPARO_BAD_ARGUMENT;
#undef SCAN_LAUNCH
    return launch_status();
}

// dt_raw [tokens, channels] float32 (the step projection with its bias, before softplus); x [tokens,
// channels] in `dtype`; bc [tokens, 2 n_state] float32 (B then C); z rows z_ld floats apart; A, D float32
// (A = -exp(A_log), [channels, n_state]); state [slots, channels, n_state] float32; out [tokens, channels]
// in `dtype`. n_state at most 512.
extern "C" int imparo_selective_scan(const float* dt_raw, const void* x, const float* bc, const float* z, int z_ld,
                                     const float* A, const float* D, float* state, const int32_t* seg_start,
                                     const int32_t* seg_len, const int32_t* slot, void* out, int dtype, int n_rows,
                                     int channels, int n_state, imparo_stream stream) {
    if (!dt_raw || !x || !bc || !z || !A || !D || !state || !seg_start || !seg_len || !slot || !out)
        return IMPARO_BAD_ARGUMENT;
    if (n_rows < 0 || channels <= 0 || n_state <= 0 || n_state > 512 || z_ld < channels) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == IMPARO_F32)
        return launch_scan<float, float>(dt_raw, x, bc, z, z_ld, A, D, state, seg_start, seg_len, slot, out, n_rows,
                                         channels, n_state, s);
    if (dtype == IMPARO_BF16)
        return launch_scan<bf16_t, bf16_t>(dt_raw, x, bc, z, z_ld, A, D, state, seg_start, seg_len, slot, out, n_rows,
                                           channels, n_state, s);
    return IMPARO_BAD_ARGUMENT;
}

int imparo_load_code_selective_scan() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_causal_conv_state)) == hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
