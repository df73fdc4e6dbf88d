// Recurrent mixers: a short causal convolution with its carried inputs, and the gated delta
// rule with one decay per key channel, whose state is a [key channels, value channels] matrix per head.
//
// Everything that enters the recurrence is float32: the convolved q, k, v, the decays, the step
// sizes, the state.  A sequence's tokens lie next to each other in the batch: sequence s owns
// tokens [seq_starts[s], seq_starts[s + 1]); its state lives in slot slots[s] of the state slabs.
#include "common.h"

FX_DEFINE_LAST_ERROR()

// ---------------------------------------------------------------------------
// Short convolution over time per channel, then silu:
//   y[t, c] = silu(sum_j taps[c, n-1-j] * x[t-j, c]),   j < n
// where x[t-j] is a token of this step if it lies in the sequence's portion, else one of the n-1
// inputs carried from before the portion (state[slot, c, :], oldest first; zeros at a sequence's start).
// One thread per (token, channel).
// ---------------------------------------------------------------------------
#define CONV_MAX_TAPS 16
__global__ __launch_bounds__(256) void short_conv_kernel(const float* __restrict__ x, long ldx, float* __restrict__ y, long ldy,
                                                         const void* __restrict__ taps, int taps_dtype, int n_taps,
                                                         const float* __restrict__ state, const int* __restrict__ token_seq,
                                                         const int* __restrict__ seq_starts, const int* __restrict__ slots,
                                                         int C) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int s = token_seq[t];
    const int i = t - seq_starts[s];                 // place in the portion
    const float* carried = state + ((size_t)slots[s] * C + c) * (n_taps - 1);
    float acc = 0.f;
    for (int j = n_taps - 1; j >= 0; --j) {          // oldest input first
        const float xv = j <= i ? x[(size_t)(t - j) * ldx + c] : carried[n_taps - 1 + i - j];
        acc = fmaf(load_as_float(taps, taps_dtype, (size_t)c * n_taps + n_taps - 1 - j), xv, acc);
    }
    y[(size_t)t * ldy + c] = acc / (1.0f + expf(-acc));
}

// After the step: the last n-1 inputs of every sequence, oldest first.  One thread per (sequence, channel);
// it reads an entry that it is about to overwrite before it writes it (entries move toward the front).
__global__ __launch_bounds__(256) void conv_carry_kernel(const float* __restrict__ x, long ldx, float* __restrict__ state,
                                                         const int* __restrict__ seq_starts, const int* __restrict__ slots,
                                                         int C, int n_taps) {
    const int s = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int t0 = seq_starts[s], n = seq_starts[s + 1] - t0;
    if (n <= 0) return;
    float* carried = state + ((size_t)slots[s] * C + c) * (n_taps - 1);
    for (int j = 0; j < n_taps - 1; ++j) {
        const int i = n - (n_taps - 1) + j;          // place in the portion of the input that entry j holds afterwards
        carried[j] = i >= 0 ? x[(size_t)(t0 + i) * ldx + c] : carried[j + n];
    }
}

FX_API int fx_short_conv(void* stream, const float* x, long ldx, float* y, long ldy, const void* taps, int taps_dtype,
                         int n_taps, float* state, const int* token_seq, const int* seq_starts, const int* slots,
                         int T, int n_seqs, int C) {
    FX_REQUIRE(T >= 0 && n_seqs >= 0 && C > 0, "short_conv: bad sizes T=%d sequences=%d C=%d", T, n_seqs, C);
    FX_REQUIRE(n_taps >= 1 && n_taps <= CONV_MAX_TAPS, "short_conv: %d taps, this kernel takes 1..%d", n_taps, CONV_MAX_TAPS);
    FX_REQUIRE(ldx >= C && ldy >= C, "short_conv: rows of %ld and %ld hold fewer than %d channels", ldx, ldy, C);
    FX_REQUIRE(taps_dtype == FX_F32 || taps_dtype == FX_BF16, "short_conv: unknown dtype %d of the taps", taps_dtype);
    FX_REQUIRE(T <= 65535 && n_seqs <= 65535, "short_conv: %d tokens of %d sequences are more than a launch takes", T, n_seqs);
    FX_REQUIRE(x != y, "short_conv: the output must not be the input (carried inputs are read from it afterwards)");
    if (T == 0 || n_seqs == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    short_conv_kernel<<<dim3((C + 255) / 256, T), 256, 0, s>>>(x, ldx, y, ldy, taps, taps_dtype, n_taps, state, token_seq,
                                                               seq_starts, slots, C);
    if (n_taps > 1)
        conv_carry_kernel<<<dim3((C + 255) / 256, n_seqs), 256, 0, s>>>(x, ldx, state, seq_starts, slots, C, n_taps);
    FX_CHECK_LAUNCH("short_conv");
    return 0;
}

// ---------------------------------------------------------------------------
// What the delta rule's recurrence reads, made per token from the convolved q and k and from the
// projections of the gates (all float32):
//   qn = q / sqrt(sum(q^2) + 1e-6) * D^-1/2,  kn = k / sqrt(sum(k^2) + 1e-6)        per q/k head
//   decay[h, i] = exp(-exp(A_log[h]) * softplus(a[h, i] + dt_bias[h, i]))             per head and key channel
//   beta[h] = sigmoid(b[h])
// One block per token.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float softplus_f(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

__global__ __launch_bounds__(256) void delta_prepare_kernel(const float* __restrict__ q, long ldq, const float* __restrict__ k, long ldk,
                                                            const float* __restrict__ a, long lda, const float* __restrict__ b, long ldb,
                                                            const void* __restrict__ A_log, const void* __restrict__ dt_bias, int w_dtype,
                                                            float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ decay,
                                                            float* __restrict__ beta, int H, int G, int D) {
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int g = wave; g < 2 * G; g += 4) {          // a wave per head of q (g < G) or of k
        const bool is_q = g < G;
        const float* src = is_q ? q + (size_t)t * ldq + (size_t)g * D : k + (size_t)t * ldk + (size_t)(g - G) * D;
        float* dst = is_q ? qn + ((size_t)t * G + g) * D : kn + ((size_t)t * G + g - G) * D;
        float ss = 0.f;
        for (int i = lane; i < D; i += 64) ss = fmaf(src[i], src[i], ss);
        ss = wave_sum(ss);
        float scale = 1.0f / sqrtf(ss + 1e-6f);
        if (is_q) scale *= 1.0f / sqrtf((float)D);
        for (int i = lane; i < D; i += 64) dst[i] = src[i] * scale;
    }
    for (int idx = threadIdx.x; idx < H * D; idx += 256) {
        const int h = idx / D;
        const float rate = expf(load_as_float(A_log, w_dtype, h));
        const float step = softplus_f(a[(size_t)t * lda + idx] + load_as_float(dt_bias, w_dtype, idx));
        decay[(size_t)t * H * D + idx] = expf(-rate * step);
    }
    for (int h = threadIdx.x; h < H; h += 256) beta[(size_t)t * H + h] = 1.0f / (1.0f + expf(-b[(size_t)t * ldb + h]));
}

FX_API int fx_delta_prepare(void* stream, const float* q, long ldq, const float* k, long ldk, const float* a, long lda,
                            const float* b, long ldb, const void* A_log, const void* dt_bias, int w_dtype, float* qn,
                            float* kn, float* decay, float* beta, int T, int H, int G, int D) {
    FX_REQUIRE(T >= 0 && H > 0 && G > 0 && D > 0 && H % G == 0, "delta_prepare: bad sizes T=%d H=%d G=%d D=%d", T, H, G, D);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "delta_prepare: unknown dtype %d", w_dtype);
    if (T == 0) return 0;
    delta_prepare_kernel<<<T, 256, 0, (hipStream_t)stream>>>(q, ldq, k, ldk, a, lda, b, ldb, A_log, dt_bias, w_dtype, qn, kn,
                                                             decay, beta, H, G, D);
    FX_CHECK_LAUNCH("delta_prepare");
    return 0;
}

// ---------------------------------------------------------------------------
// The recurrence.  Per head, with S [D, V] carried from token to token:
//   S <- diag(decay_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
// Columns of S never meet, so a block of one wave owns 16 of them: lane (r, j), r = lane / 16, j = lane % 16,
// holds rows [r DR, (r + 1) DR) of column j in registers (DR = ceil(D / 4) rounded up to the template's size; rows
// past D stay zero).  Per token it forms, over its rows, the parts of (dS)^T k, (dS)^T q and k.q; the four lanes of
// a column add theirs with two lane-swapping moves; then u and o = (dS)^T q + u (k.q) follow, and S takes
// k u^T.  The token's k, q and decay go through LDS (written a token ahead by the wave itself), so every lane
// reads its rows as broadcasts.  Grid: (ceil(V / 16), heads, sequences).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float column_sum(float x) {      // over lanes j, j + 16, j + 32, j + 48, in each of them
    const unsigned u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const unsigned v = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

template <int DR>
__global__ __launch_bounds__(64) void channel_delta_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                                                           const float* __restrict__ decay, const float* __restrict__ beta,
                                                           const float* __restrict__ v, long ldv, float* __restrict__ out, long ldo,
                                                           float* __restrict__ state, const int* __restrict__ seq_starts,
                                                           const int* __restrict__ slots, int H, int G, int D, int V) {
    constexpr int DP = 4 * DR;                       // rows as the wave holds them
    __shared__ __attribute__((aligned(16))) float kqd[2][3][DP];      // two tokens x (k, q, decay)
    const int lane = threadIdx.x, r = lane >> 4, j = blockIdx.x * 16 + (lane & 15);
    const int h = blockIdx.y, s = blockIdx.z, g = h / (H / G);
    const int t0 = seq_starts[s], t1 = seq_starts[s + 1];
    if (t1 <= t0) return;
    const bool col = j < V;
    float* S_g = state + (((size_t)slots[s] * H + h) * D) * V + (col ? j : 0);
    float S[DR];
#pragma unroll
    for (int i = 0; i < DR; ++i) {
        const int row = r * DR + i;
        S[i] = (col && row < D) ? S_g[(size_t)row * V] : 0.f;
    }
    // the wave brings a token's k, q and decay into LDS: 3 DP floats, lane-strided; rows past D are zeros
    auto fetch = [&](int t, float (&buf)[3 * DP / 64 + 1]) {
#pragma unroll
        for (int n = 0; n < 3 * DP / 64 + 1; ++n) {
            const int e = n * 64 + lane, which = e / DP, row = e - which * DP;
            float x = 0.f;
            if (e < 3 * DP && row < D) {
                const float* src = which == 0 ? kn + ((size_t)t * G + g) * D : (which == 1 ? qn + ((size_t)t * G + g) * D
                                                                                             : decay + ((size_t)t * H + h) * D);
                x = src[row];
            }
            buf[n] = x;
        }
    };
    auto stage = [&](int slot, const float (&buf)[3 * DP / 64 + 1]) {
#pragma unroll
        for (int n = 0; n < 3 * DP / 64 + 1; ++n) {
            const int e = n * 64 + lane;
            if (e < 3 * DP) (&kqd[slot][0][0])[e] = buf[n];
        }
    };
    float next[3 * DP / 64 + 1];
    fetch(t0, next);
    stage(0, next);
    float v_next = col ? v[(size_t)t0 * ldv + (size_t)h * V + j] : 0.f, beta_next = beta[(size_t)t0 * H + h];
    for (int t = t0; t < t1; ++t) {
        const int cur = (t - t0) & 1;
        const float vt = v_next, bt = beta_next;
        if (t + 1 < t1) {                            // the next token's operands leave now and are staged after this token's work
            fetch(t + 1, next);
            v_next = col ? v[(size_t)(t + 1) * ldv + (size_t)h * V + j] : 0.f;
            beta_next = beta[(size_t)(t + 1) * H + h];
        }
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // what the wave staged a token ago is in LDS
        const float* kk = &kqd[cur][0][r * DR];
        const float* qq = &kqd[cur][1][r * DR];
        const float* dd = &kqd[cur][2][r * DR];
        float kv[DR];
        float sk = 0.f, sq = 0.f, kq = 0.f;
#pragma unroll
        for (int i = 0; i < DR; i += 4) {
            const float4 k4 = *(const float4*)(kk + i), q4 = *(const float4*)(qq + i), d4 = *(const float4*)(dd + i);
            const float ka[4] = {k4.x, k4.y, k4.z, k4.w}, qa[4] = {q4.x, q4.y, q4.z, q4.w}, da[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                S[i + e] *= da[e];
                sk = fmaf(S[i + e], ka[e], sk);
                sq = fmaf(S[i + e], qa[e], sq);
                kq = fmaf(ka[e], qa[e], kq);
                kv[i + e] = ka[e];
            }
        }
        sk = column_sum(sk);
        sq = column_sum(sq);
        kq = column_sum(kq);
        const float u = bt * (vt - sk);
        if (col && r == 0) out[(size_t)t * ldo + (size_t)h * V + j] = fmaf(u, kq, sq);
#pragma unroll
        for (int i = 0; i < DR; ++i) S[i] = fmaf(kv[i], u, S[i]);
        if (t + 1 < t1) stage(cur ^ 1, next);
    }
#pragma unroll
    for (int i = 0; i < DR; ++i) {
        const int row = r * DR + i;
        if (col && row < D) S_g[(size_t)row * V] = S[i];
    }
}

FX_API int fx_channel_delta(void* stream, const float* qn, const float* kn, const float* decay, const float* beta,
                            const float* v, long ldv, float* out, long ldo, float* state, const int* seq_starts,
                            const int* slots, int n_seqs, int H, int G, int D, int V) {
    FX_REQUIRE(n_seqs >= 0 && H > 0 && G > 0 && H % G == 0, "channel_delta: bad sizes sequences=%d H=%d G=%d", n_seqs, H, G);
    FX_REQUIRE(D >= 1 && D <= 256 && V >= 1, "channel_delta: key size %d (up to 256) and value size %d", D, V);
    FX_REQUIRE(ldv >= (long)H * V && ldo >= (long)H * V, "channel_delta: rows of %ld and %ld hold fewer than %d values", ldv, ldo, H * V);
    FX_REQUIRE(n_seqs <= 65535 && H <= 65535, "channel_delta: %d sequences of %d heads are more than a launch takes", n_seqs, H);
    if (n_seqs == 0) return 0;
    const dim3 grid((V + 15) / 16, H, n_seqs);
    hipStream_t s = (hipStream_t)stream;
    if (D <= 64) channel_delta_kernel<16><<<grid, 64, 0, s>>>(qn, kn, decay, beta, v, ldv, out, ldo, state, seq_starts, slots, H, G, D, V);
    else if (D <= 128) channel_delta_kernel<32><<<grid, 64, 0, s>>>(qn, kn, decay, beta, v, ldv, out, ldo, state, seq_starts, slots, H, G, D, V);
    else channel_delta_kernel<64><<<grid, 64, 0, s>>>(qn, kn, decay, beta, v, ldv, out, ldo, state, seq_starts, slots, H, G, D, V);
    FX_CHECK_LAUNCH("channel_delta");
    return 0;
}

// ---------------------------------------------------------------------------
// The read-out's way to the output projection: every head's o is divided by its root mean square over V
// (eps inside the root), times a weight shared by the heads, times sigmoid(gate[h, :]).  One wave per (token, head).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(const float* __restrict__ o, long ldo, const float* __restrict__ gate,
                                                              long ldg, const void* __restrict__ w, int w_dtype, T* __restrict__ y,
                                                              long ldy, int n_rows, int H, int V, float eps) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= n_rows) return;
    const int t = row / H, h = row - t * H;
    const float* src = o + (size_t)t * ldo + (size_t)h * V;
    float ss = 0.f;
    for (int i = lane; i < V; i += 64) ss = fmaf(src[i], src[i], ss);
    ss = wave_sum(ss);
    const float scale = 1.0f / sqrtf(ss / (float)V + eps);
    for (int i = lane; i < V; i += 64) {
        const float gt = 1.0f / (1.0f + expf(-gate[(size_t)t * ldg + (size_t)h * V + i]));
        from_float(y + (size_t)t * ldy + (size_t)h * V + i, src[i] * scale * load_as_float(w, w_dtype, i) * gt);
    }
}

FX_API int fx_gated_head_norm(void* stream, int out_dtype, const float* o, long ldo, const float* gate, long ldg,
                              const void* w, int w_dtype, void* y, long ldy, int T, int H, int V, float eps) {
    FX_REQUIRE(T >= 0 && H > 0 && V > 0, "gated_head_norm: bad sizes T=%d H=%d V=%d", T, H, V);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "gated_head_norm: unknown weight dtype %d", w_dtype);
    FX_REQUIRE((long)T * H < (1L << 31), "gated_head_norm: too many rows for one launch");
    if (T == 0) return 0;
    const int rows = T * H;
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == FX_F32)
        gated_head_norm_kernel<float><<<(rows + 3) / 4, 256, 0, s>>>(o, ldo, gate, ldg, w, w_dtype, (float*)y, ldy, rows, H, V, eps);
    else if (out_dtype == FX_BF16)
        gated_head_norm_kernel<bf16><<<(rows + 3) / 4, 256, 0, s>>>(o, ldo, gate, ldg, w, w_dtype, (bf16*)y, ldy, rows, H, V, eps);
    else
        return fx_fail("gated_head_norm: unknown output dtype %d", out_dtype);
    FX_CHECK_LAUNCH("gated_head_norm");
    return 0;
}
