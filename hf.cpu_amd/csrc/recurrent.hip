// Mixers with per-request state of fixed size: a short causal convolution whose last inputs are carried from step to
// step, and a linear recurrence over a matrix state per head (state-space layers, linear attention).
//
//   hfa_causal_conv   out[t, c] = act(bias[c] + sum_j taps[c, j] in[t - (K - 1) + j, c]) per channel, the K - 1 inputs
//                     before a request's first token of this step taken from its state row, which then receives the
//                     last K - 1 inputs of the step
//   hfa_linear_scan   S <- a_t S + k_t (b_t v_t)^T, y_t = S^T q_t + d v_t per (request, head), S in fp32 in the state row
//
// Both walk a request's tokens of the step in order from the state that the step before left, so a token's result
// does not depend on where a prompt was cut or on what else the step holds.
#include "api.h"
#include "common.h"

#define CONV_MAX_TAPS 8
#define CONV_SEG 64              // tokens that one thread walks

// One thread a (request, run of CONV_SEG tokens, channel). state row: [K - 1][C] inputs, oldest first.
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(const T* __restrict__ in, int ld_in, const float* __restrict__ taps,
                                                         const float* __restrict__ bias, int C, int K,
                                                         float* __restrict__ state, size_t state_ld,
                                                         const int* __restrict__ q_start, const int* __restrict__ seq_slot,
                                                         float* __restrict__ out, int ldo, int act) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, s = blockIdx.z;
    if (c >= C) return;
    const int q0 = q_start[s], n = q_start[s + 1] - q0, t0 = blockIdx.y * CONV_SEG;
    if (t0 >= n) return;
    float* st = state + (size_t)seq_slot[s] * state_ld;
    // the input at place i of the request's tokens of this step; i < 0 reaches into the state
    auto input = [&](int i) { return i >= 0 ? to_f32(in[(size_t)(q0 + i) * ld_in + c]) : st[(size_t)(K - 1 + i) * C + c]; };
    float w[CONV_MAX_TAPS], win[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; j++) {
        w[j] = j < K ? taps[(size_t)c * K + j] : 0.f;
        win[j] = j < K - 1 ? input(t0 - (K - 1) + j) : 0.f;
    }
    if (t0 == 0) {
        // The only thread that reads this channel's state is also the one that writes it: all reads come first.
        float next[CONV_MAX_TAPS];
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; j++) next[j] = j < K - 1 ? input(n - (K - 1) + j) : 0.f;
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; j++)
            if (j < K - 1) st[(size_t)j * C + c] = next[j];
    }
    const float b = bias ? bias[c] : 0.f;
    const int t1 = t0 + CONV_SEG < n ? t0 + CONV_SEG : n;
    for (int t = t0; t < t1; t++) {
        win[K - 1] = to_f32(in[(size_t)(q0 + t) * ld_in + c]);
        float acc = b;
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; j++)
            if (j < K) acc = fmaf(w[j], win[j], acc);
        out[(size_t)(q0 + t) * ldo + c] = act == HFA_ACT_SILU ? acc / (1.0f + expf(-acc)) : acc;
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS - 1; j++) win[j] = win[j + 1];
    }
}

extern "C" int hfa_causal_conv(const void* in, int dtype, int ld_in, const float* taps, const float* bias, int n_channels,
                               int n_taps, float* state, size_t state_ld, const int* q_start, const int* seq_slot, int n_seqs,
                               int max_q_len, float* out, int ldo, int act, hipStream_t stream) {
    HFA_REQUIRE(in && taps && (state || n_taps == 1) && q_start && seq_slot && out && n_channels > 0 && n_seqs > 0 && max_q_len > 0,
                "causal_conv: bad arguments");
    HFA_REQUIRE(n_taps >= 1 && n_taps <= CONV_MAX_TAPS, "causal_conv: %d taps (1 to %d)", n_taps, CONV_MAX_TAPS);
    HFA_REQUIRE(ld_in >= n_channels && ldo >= n_channels && state_ld >= (size_t)(n_taps - 1) * n_channels,
                "causal_conv: a row is shorter than its channels");
    HFA_REQUIRE(act == HFA_ACT_NONE || act == HFA_ACT_SILU, "causal_conv: the activation is silu or none");
    HFA_REQUIRE(dtype == HFA_F32 || dtype == HFA_BF16, "causal_conv: unknown dtype %d", dtype);
    HFA_REQUIRE(n_seqs <= 65535 && (max_q_len + CONV_SEG - 1) / CONV_SEG <= 65535, "causal_conv: the step exceeds the grid");
    dim3 grid((n_channels + 255) / 256, (max_q_len + CONV_SEG - 1) / CONV_SEG, n_seqs);
    if (dtype == HFA_F32)
        causal_conv_kernel<float><<<grid, 256, 0, stream>>>((const float*)in, ld_in, taps, bias, n_channels, n_taps, state, state_ld,
                                                            q_start, seq_slot, out, ldo, act);
    else
        causal_conv_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)in, ld_in, taps, bias, n_channels, n_taps, state, state_ld,
                                                           q_start, seq_slot, out, ldo, act);
    HFA_LAUNCH_CHECK("causal_conv");
    return 0;
}

// ---- the linear recurrence ------------------------------------------------------------------------------------
// One block a (request, head). The state S [N][P] of the head lives in registers for the whole walk: thread (p, ns)
// holds S[n][p] for the n of its slice (n = ns, ns + 4, ...: the four slices of a column sit in neighbouring lanes, and
// a token's output is their sum). The tokens' k, q, v, a and b are staged through LDS SCAN_TOKENS at a time.
//
// gate 0: a_t = decay[h], b_t = 1 (a fixed decay per head).
// gate 1: dt = softplus(step[t, h] + step_bias[h]), a_t = exp(-exp(a_log[h]) dt), b_t = dt (a step size per token).
#define SCAN_NS 4
#define SCAN_TOKENS 16
template <typename T, typename TS, int NPT>
__global__ __launch_bounds__(1024) void linear_scan_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, int heads_per_qk, int N, const T* __restrict__ v,
    int ldv, int P, int gate, const float* __restrict__ decay, const TS* __restrict__ step, int ld_step,
    const float* __restrict__ step_bias, const float* __restrict__ a_log, const float* __restrict__ skip,
    float* __restrict__ state, size_t state_ld, const int* __restrict__ q_start, const int* __restrict__ seq_slot,
    float* __restrict__ y, int ldy) {
    extern __shared__ float lds[];
    const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
    const int p = tid / SCAN_NS, ns = tid % SCAN_NS;
    const int q0 = q_start[s], n_tok = q_start[s + 1] - q0;
    if (n_tok <= 0) return;
    float* k_s = lds;                                   // [SCAN_TOKENS][N]
    float* q_s = k_s + SCAN_TOKENS * N;                 // [SCAN_TOKENS][N]
    float* v_s = q_s + SCAN_TOKENS * N;                 // [SCAN_TOKENS][P]
    float* a_s = v_s + SCAN_TOKENS * P;                 // [SCAN_TOKENS]
    float* b_s = a_s + SCAN_TOKENS;                     // [SCAN_TOKENS]
    const int g = h / heads_per_qk;
    float* S = state + (size_t)seq_slot[s] * state_ld + (size_t)h * N * P;
    const bool live = p < P;
    float st[NPT];
#pragma unroll
    for (int i = 0; i < NPT; i++) {
        const int n = ns + SCAN_NS * i;
        st[i] = live && n < N ? S[(size_t)n * P + p] : 0.f;
    }
    const float d = skip ? skip[h] : 0.f;
    const float head_decay = gate == 0 ? decay[h] : 0.f;
    const float neg_rate = gate == 1 ? -expf(a_log[h]) : 0.f, sb = gate == 1 ? step_bias[h] : 0.f;
    for (int c0 = 0; c0 < n_tok; c0 += SCAN_TOKENS) {
        const int nt = n_tok - c0 < SCAN_TOKENS ? n_tok - c0 : SCAN_TOKENS;
        __syncthreads();
        for (int i = tid; i < nt * N; i += blockDim.x) {
            const int t = i / N, n = i % N;
            k_s[i] = to_f32(k[(size_t)(q0 + c0 + t) * ldk + g * N + n]);
            q_s[i] = to_f32(q[(size_t)(q0 + c0 + t) * ldq + g * N + n]);
        }
        for (int i = tid; i < nt * P; i += blockDim.x) {
            const int t = i / P, pp = i % P;
            v_s[i] = to_f32(v[(size_t)(q0 + c0 + t) * ldv + h * P + pp]);
        }
        if (tid < nt) {
            if (gate == 1) {
                const float z = to_f32(step[(size_t)(q0 + c0 + tid) * ld_step + h]) + sb;
                const float dt = fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));          // softplus, exact for every z
                a_s[tid] = expf(neg_rate * dt);
                b_s[tid] = dt;
            } else {
                a_s[tid] = head_decay;
                b_s[tid] = 1.f;
            }
        }
        __syncthreads();
        if (!live) continue;
        for (int t = 0; t < nt; t++) {
            const float a = a_s[t], vt = v_s[t * P + p], bv = b_s[t] * vt;
            const float* kt = k_s + t * N;
            const float* qt = q_s + t * N;
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NPT; i++) {
                const int n = ns + SCAN_NS * i;
                if (n < N) {
                    st[i] = fmaf(a, st[i], kt[n] * bv);
                    acc = fmaf(st[i], qt[n], acc);
                }
            }
            acc += __shfl_xor(acc, 1, WAVE);
            acc += __shfl_xor(acc, 2, WAVE);
            if (ns == 0) y[(size_t)(q0 + c0 + t) * ldy + h * P + p] = fmaf(d, vt, acc);
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < NPT; i++) {
            const int n = ns + SCAN_NS * i;
            if (n < N) S[(size_t)n * P + p] = st[i];
        }
    }
}

extern "C" int hfa_linear_scan(const void* q, int ldq, const void* k, int ldk, int qk_heads, int qk_dim, const void* v,
                               int ldv, int n_heads, int v_dim, int dtype, int gate, const float* decay, const void* step,
                               int step_dtype, int ld_step, const float* step_bias, const float* a_log, const float* skip,
                               float* state, size_t state_ld, const int* q_start, const int* seq_slot, int n_seqs, float* y,
                               int ldy, hipStream_t stream) {
    HFA_REQUIRE(q && k && v && state && q_start && seq_slot && y && n_seqs > 0, "linear_scan: a null argument");
    HFA_REQUIRE(n_heads > 0 && qk_heads > 0 && n_heads % qk_heads == 0 && qk_dim > 0 && v_dim > 0,
                "linear_scan: %d heads over %d heads of keys", n_heads, qk_heads);
    HFA_REQUIRE(ldq >= qk_heads * qk_dim && ldk >= qk_heads * qk_dim && ldv >= n_heads * v_dim && ldy >= n_heads * v_dim &&
                    state_ld >= (size_t)n_heads * qk_dim * v_dim, "linear_scan: a row is shorter than its heads");
    HFA_REQUIRE(qk_dim <= SCAN_NS * 64 && v_dim <= 1024 / SCAN_NS, "linear_scan: a state of %d x %d a head is too large (at most %d x %d)",
                qk_dim, v_dim, SCAN_NS * 64, 1024 / SCAN_NS);
    HFA_REQUIRE(dtype == HFA_F32 || dtype == HFA_BF16, "linear_scan: unknown dtype %d", dtype);
    HFA_REQUIRE((gate == 0 && decay) || (gate == 1 && step && step_bias && a_log && ld_step >= n_heads &&
                                         (step_dtype == HFA_F32 || step_dtype == HFA_BF16)),
                "linear_scan: gate 0 needs a decay per head, gate 1 step sizes, their bias and the logarithm of the rate");
    HFA_REQUIRE(n_heads <= 65535 && n_seqs <= 65535, "linear_scan: the step exceeds the grid");
    const int threads = (v_dim * SCAN_NS + WAVE - 1) / WAVE * WAVE;
    const size_t smem = (size_t)(SCAN_TOKENS * (2 * qk_dim + v_dim + 2)) * sizeof(float);
    const int per = (qk_dim + SCAN_NS - 1) / SCAN_NS;
    dim3 grid(n_heads, n_seqs);
#define SCAN_GO(T, TS, NPT)                                                                                              \
    linear_scan_kernel<T, TS, NPT><<<grid, threads, smem, stream>>>(                                                     \
        (const T*)q, ldq, (const T*)k, ldk, n_heads / qk_heads, qk_dim, (const T*)v, ldv, v_dim, gate, decay, (const TS*)step, \
        ld_step, step_bias, a_log, skip, state, state_ld, q_start, seq_slot, y, ldy)
#define SCAN_SIZES(T, TS)                        \
    do {                                         \
        if (per <= 4) SCAN_GO(T, TS, 4);         \
        else if (per <= 8) SCAN_GO(T, TS, 8);    \
        else if (per <= 16) SCAN_GO(T, TS, 16);  \
        else if (per <= 32) SCAN_GO(T, TS, 32);  \
        else SCAN_GO(T, TS, 64);                 \
    } while (0)
    if (dtype == HFA_F32) { if (step_dtype == HFA_BF16 && gate == 1) SCAN_SIZES(float, bf16); else SCAN_SIZES(float, float); }
    else { if (step_dtype == HFA_F32 && gate == 1) SCAN_SIZES(bf16, float); else SCAN_SIZES(bf16, bf16); }
#undef SCAN_SIZES
#undef SCAN_GO
    HFA_LAUNCH_CHECK("linear_scan");
    return 0;
}
