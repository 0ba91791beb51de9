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
// channel's states, SPL states a lane (n = lane + j * LP). Tokens are walked in order, UNR at a time:
// their inputs are asked for together, from clamped addresses, and a token past the end walks with a
// step of zero, which leaves the state as it is. A token's sum_n S[n] C[n] is added up across the LP
// lanes by a butterfly, the same order whatever the batch; lane u of the channel then gates and stores
// the batch's token u (UNR never passes LP).
//
// A long segment is cut into chunks of SCAN_CHUNK tokens that run side by side: k_scan_chunk_state walks
// every chunk but the last from a zero state and leaves its end state E_k and the sum of its steps (the
// chunk's decay is exp(A sum dt)); k_selective_scan then starts chunk k from I_k, with I_0 the request's
// state and I_{j+1} = exp(A sum_j) I_j + E_j, and walks it again, now with outputs. The request's state
// is copied aside first (chunk 0 of the first launch), since the last chunk replaces it while others read.
#define SCAN_CHUNK 64

extern "C" int imparo_selective_scan_chunk(void) { return SCAN_CHUNK; }

// dt <- softplus(dt) in place, once per (token, channel): the scan's lanes that share a channel would each
// take it again, in both of its launches.
__global__ void k_softplus_rows(float* __restrict__ dt, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dt[i] = softplus_f32(dt[i]);
}

// exp of a decay's exponent: the library's in float32, the hardware's exp2 where the engine rounds its
// activations to bfloat16 anyway
template <typename TX> __device__ __forceinline__ float decay_exp(float v);
template <> __device__ __forceinline__ float decay_exp<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ float decay_exp<bf16_t>(float v) { return __expf(v); }

template <typename TX, typename TOut, int SPL, int UNR, bool EMIT>
__device__ __forceinline__ float scan_walk(const float* __restrict__ dt_raw /* steps; raw == true: before softplus */, const TX* __restrict__ x,
                                           const float* __restrict__ bc, const float* __restrict__ z, int z_ld,
                                           TOut* __restrict__ out, float (&S)[SPL], const float (&a)[SPL], float d_skip,
                                           size_t t_first, int count, int channels, int cc, int n_state, int lp, int ln,
                                           bool live, bool raw = false) {
    float dt_sum = 0.f;
    for (int i = 0; i < count; i += UNR) {
        float dt[UNR], xv[UNR], b[UNR][SPL], cv[UNR][SPL];
        // lane u of a channel's lanes finishes token i + u of the batch: its gate is all it has to ask for
        const bool finisher = EMIT && ln < UNR && live && i + ln < count;
        const float z_mine = EMIT ? z[(t_first + (size_t)min(i + min(ln, UNR - 1), count - 1)) * z_ld + cc] : 0.f;
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const size_t t = t_first + (size_t)min(i + u, count - 1);
            dt[u] = dt_raw[t * channels + cc];
            xv[u] = load_f32<TX>(x, t * channels + cc);
#pragma unroll
            for (int j = 0; j < SPL; ++j) {
                const int nn = min(ln + j * lp, n_state - 1);
                b[u][j] = bc[t * 2 * n_state + nn];
                cv[u][j] = EMIT ? bc[t * 2 * n_state + n_state + nn] : 0.f;
            }
        }
        float y_mine = 0.f, x_mine = 0.f;
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const bool on = i + u < count;
            const float step = on ? (raw ? softplus_f32(dt[u]) : dt[u]) : 0.f;
            const float dx = step * xv[u];
            dt_sum += step;
            float y = 0.f;
#pragma unroll
            for (int j = 0; j < SPL; ++j) {
                const bool has = ln + j * lp < n_state;
                const float s_new = decay_exp<TX>(step * a[j]) * S[j] + dx * b[u][j];
                S[j] = has ? s_new : 0.f;
                y += has ? s_new * cv[u][j] : 0.f;
            }
            if (EMIT) {
                for (int off = lp >> 1; off > 0; off >>= 1) y += __shfl_xor(y, off, WAVE);   // every lane of the channel has the sum
                y_mine = ln == u ? y : y_mine;
                x_mine = ln == u ? xv[u] : x_mine;
            }
        }
        if (finisher) {
            const float gate = z_mine / (1.0f + decay_exp<TX>(-z_mine));
            store_f32<TOut>(out, (t_first + i + ln) * channels + cc, (y_mine + d_skip * x_mine) * gate);
        }
    }
    return dt_sum;
}

// scratch: [rows, n_chunks, channels, n_state] end states, then [rows, n_chunks, channels] step sums, then
// [rows, channels, n_state] the requests' states as they were.
template <typename TX, int SPL, int UNR>
__global__ void k_scan_chunk_state(const float* __restrict__ dt_raw, const TX* __restrict__ x,
                                   const float* __restrict__ bc, const float* __restrict__ A,
                                   const float* __restrict__ state, const int32_t* __restrict__ seg_start,
                                   const int32_t* __restrict__ seg_len, const int32_t* __restrict__ slot,
                                   float* __restrict__ scratch, int n_rows, int n_chunks, int channels, int n_state,
                                   int lp) {
    const int r = blockIdx.x, k = blockIdx.z;
    const int len = seg_len[r];
    const int chunks = (len + SCAN_CHUNK - 1) / SCAN_CHUNK;
    if (chunks < 2 || k >= chunks - 1) return;
    const int ln = threadIdx.x & (lp - 1);
    const int c = blockIdx.y * (blockDim.x / lp) + threadIdx.x / lp;
    const bool live = c < channels;
    const int cc = live ? c : channels - 1;
    float S[SPL], a[SPL];
#pragma unroll
    for (int j = 0; j < SPL; ++j) {
        const int n = min(ln + j * lp, n_state - 1);
        S[j] = 0.f;
        a[j] = A[(size_t)cc * n_state + n];
    }
    const float sum = scan_walk<TX, float, SPL, UNR, false>(dt_raw, x, bc, nullptr, 0, nullptr, S, a, 0.f,
                                                            (size_t)seg_start[r] + (size_t)k * SCAN_CHUNK, SCAN_CHUNK,
                                                            channels, cc, n_state, lp, ln, live);
    if (!live) return;
    float* ends = scratch + (((size_t)r * n_chunks + k) * channels + cc) * n_state;
    float* sums = scratch + (size_t)n_rows * n_chunks * channels * n_state + ((size_t)r * n_chunks + k) * channels;
    float* was = scratch + (size_t)n_rows * n_chunks * channels * (n_state + 1) + ((size_t)r * channels + cc) * n_state;
    const float* st = state + ((size_t)slot[r] * channels + cc) * n_state;
#pragma unroll
    for (int j = 0; j < SPL; ++j) {
        const int n = ln + j * lp;
        if (n < n_state) {
            ends[n] = S[j];
            if (k == 0) was[n] = st[n];
        }
    }
    if (ln == 0) sums[cc] = sum;
}

template <typename TX, typename TOut, int SPL, int UNR>
__global__ void k_selective_scan(const float* __restrict__ dt_raw, const TX* __restrict__ x,
                                 const float* __restrict__ bc, const float* __restrict__ z, int z_ld,
                                 const float* __restrict__ A, const float* __restrict__ D, float* __restrict__ state,
                                 const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
                                 const int32_t* __restrict__ slot, TOut* __restrict__ out,
                                 const float* __restrict__ scratch, int n_rows, int n_chunks, int channels, int n_state,
                                 int lp, int raw) {
    const int r = blockIdx.x, k = blockIdx.z;
    const int len = seg_len[r];
    const int chunks = n_chunks > 1 ? max(1, (len + SCAN_CHUNK - 1) / SCAN_CHUNK) : 1;
    if (k >= chunks) return;
    const int ln = threadIdx.x & (lp - 1);
    const int c = blockIdx.y * (blockDim.x / lp) + threadIdx.x / lp;
    const bool live = c < channels;
    const int cc = live ? c : channels - 1;            // lanes past the last channel repeat it and store nothing
    float S[SPL], a[SPL];
    float* st = state + ((size_t)slot[r] * channels + cc) * n_state;
    const float* from = st;
    if (chunks > 1)
        from = scratch + (size_t)n_rows * n_chunks * channels * (n_state + 1) + ((size_t)r * channels + cc) * n_state;
#pragma unroll
    for (int j = 0; j < SPL; ++j) {
        const int n = min(ln + j * lp, n_state - 1);
        S[j] = ln + j * lp < n_state ? from[n] : 0.f;
        a[j] = A[(size_t)cc * n_state + n];
    }
    for (int p = 0; p < k; ++p) {                       // the chunks before this one, in order
        const float* ends = scratch + (((size_t)r * n_chunks + p) * channels + cc) * n_state;
        const float sum = scratch[(size_t)n_rows * n_chunks * channels * n_state + ((size_t)r * n_chunks + p) * channels + cc];
#pragma unroll
        for (int j = 0; j < SPL; ++j) {
            const int n = min(ln + j * lp, n_state - 1);
            S[j] = ln + j * lp < n_state ? decay_exp<TX>(sum * a[j]) * S[j] + ends[n] : 0.f;
        }
    }
    const int first = chunks > 1 ? k * SCAN_CHUNK : 0;
    const int count = chunks > 1 ? min(SCAN_CHUNK, len - first) : len;
    scan_walk<TX, TOut, SPL, UNR, true>(dt_raw, x, bc, z, z_ld, out, S, a, D[cc], (size_t)seg_start[r] + first, count,
                                        channels, cc, n_state, lp, ln, live, raw != 0);
    if (live && k == chunks - 1 && len > 0) {
#pragma unroll
        for (int j = 0; j < SPL; ++j) {
            const int n = ln + j * lp;
            if (n < n_state) st[n] = S[j];
        }
    }
}

template <typename TX, typename TOut>
static int launch_scan(float* dt_raw, const void* x, const float* bc, const float* z, int z_ld, const float* A,
                       const float* D, float* state, const int32_t* seg_start, const int32_t* seg_len,
                       const int32_t* slot, void* out, float* scratch, int n_chunks, int n_tokens, int n_rows,
                       int channels, int n_state, hipStream_t s) {
    int lp = 1;
    while (lp < n_state && lp < WAVE) lp <<= 1;
    const int spl = (n_state + lp - 1) / lp;
    const int threads = 256;
    const int per_block = threads / lp;
    dim3 grid(n_rows, (channels + per_block - 1) / per_block, n_chunks);
    if (grid.y > 65535 || grid.z > 65535) return IMPARO_BAD_ARGUMENT;
    // one token a row (as many tokens as rows): softplus is taken inside the walk, a launch less for a decode step
    const int raw = n_chunks == 1 && n_tokens == n_rows;
    if (!raw) {
        const long long n_dt = (long long)n_tokens * channels;
        k_softplus_rows<<<(unsigned)((n_dt + 255) / 256), 256, 0, s>>>(dt_raw, n_dt);
        if (launch_status()) return IMPARO_LAUNCH_FAILED;
    }
#define SCAN_LAUNCH(N, U)                                                                                             \
    do {                                                                                                              \
        if (n_chunks > 1) {                                                                                           \
            k_scan_chunk_state<TX, N, U><<<grid, threads, 0, s>>>(dt_raw, (const TX*)x, bc, A, state, seg_start,      \
                                                                  seg_len, slot, scratch, n_rows, n_chunks, channels, \
                                                                  n_state, lp);                                       \
            if (launch_status()) return IMPARO_LAUNCH_FAILED;                                                         \
        }                                                                                                             \
        k_selective_scan<TX, TOut, N, U><<<grid, threads, 0, s>>>(dt_raw, (const TX*)x, bc, z, z_ld, A, D, state,     \
                                                                  seg_start, seg_len, slot, (TOut*)out, scratch,      \
                                                                  n_rows, n_chunks, channels, n_state, lp, raw);      \
    } while (0)
    if (spl == 1 && lp >= 8) SCAN_LAUNCH(1, 8);        // a batch of tokens is finished by as many lanes of the channel
    else if (spl == 1 && lp == 4) SCAN_LAUNCH(1, 4);
    else if (spl == 1 && lp == 2) SCAN_LAUNCH(1, 2);
    else if (spl == 1) SCAN_LAUNCH(1, 1);
    else if (spl == 2) SCAN_LAUNCH(2, 4);
    else if (spl <= 4) SCAN_LAUNCH(4, 2);
    else if (spl <= 8) SCAN_LAUNCH(8, 1);
    else return IMPARO_BAD_ARGUMENT;
#undef SCAN_LAUNCH
    return launch_status();
}

// dt_raw [tokens, channels] float32 (the step projection with its bias, before softplus; softplus is taken in
// place, so the array holds the steps afterwards, unless every row brings one token: then inside the walk); x [tokens,
// channels] in `dtype`; bc [tokens, 2 n_state] float32 (B then C); z rows z_ld floats apart; A, D float32
// (A = -exp(A_log), [channels, n_state]); state [slots, channels, n_state] float32; out [tokens, channels]
// in `dtype`. n_state at most 512. n_chunks 1: every segment is walked in one piece. More (at least
// ceil(longest segment / imparo_selective_scan_chunk())): segments are walked in chunks side by side through
// `scratch`, n_rows * (n_chunks * channels * (n_state + 1) + channels * n_state) floats.
extern "C" int imparo_selective_scan(float* dt_raw, const void* x, const float* bc, const float* z, int z_ld,
                                     const float* A, const float* D, float* state, const int32_t* seg_start,
                                     const int32_t* seg_len, const int32_t* slot, void* out, int dtype, float* scratch,
                                     int n_chunks, int n_tokens, int n_rows, int channels, int n_state,
                                     imparo_stream stream) {
    if (!dt_raw || !x || !bc || !z || !A || !D || !state || !seg_start || !seg_len || !slot || !out)
        return IMPARO_BAD_ARGUMENT;
    if (n_rows < 0 || n_tokens < 0 || channels <= 0 || n_state <= 0 || n_state > 512 || z_ld < channels) return IMPARO_BAD_ARGUMENT;
    if (n_chunks < 1 || (n_chunks > 1 && !scratch)) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0 || n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == IMPARO_F32)
        return launch_scan<float, float>(dt_raw, x, bc, z, z_ld, A, D, state, seg_start, seg_len, slot, out, scratch,
                                         n_chunks, n_tokens, n_rows, channels, n_state, s);
    if (dtype == IMPARO_BF16)
        return launch_scan<bf16_t, bf16_t>(dt_raw, x, bc, z, z_ld, A, D, state, seg_start, seg_len, slot, out, scratch,
                                           n_chunks, n_tokens, n_rows, channels, n_state, s);
    return IMPARO_BAD_ARGUMENT;
}

int imparo_load_code_selective_scan() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_causal_conv_state)) == hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
