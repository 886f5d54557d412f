// Recurrent mixers whose state is a matrix per head, S [d, dv] in float32 in the request's slot: a write k v^T per
// token, a read-out S^T q.  One block per (entry, head); thread j owns column j of S (the d values that belong to value
// channel j) in registers and walks the entry's tokens; the token's key and query go through LDS.  Everything behind
// the projections is float32; the result is rounded once, at its store.
//
//   mlstm:       S = a S + b k v^T, n = a n + b k with a = exp(f + m' - m), b = exp(i - m), m = max(f + m', i) (m starts at
//                0), i and f capped log gates; o = S^T q / (max(|n . q|, exp(-m)) + 1e-6); then o / rms(o) * w * sigmoid(g).
//   delta rule:  S = diag(g) S; u = beta (v - S^T k); S = S + k u^T; o = S^T q, g a decay per key channel, q and k unit
//                vectors; then o / rms(o) * w * sigmoid(gate).
//   causal_conv_silu: the short convolution over time that feeds the delta rule, with its last inputs kept per request.
#include "common.h"
#include <math.h>

__device__ __forceinline__ float mm_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float mm_logsigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// sums of two values over the block; red holds 2 * 16 floats
__device__ __forceinline__ void block_sum2(float& a, float& b, float* red) {
    a = wave_sum(a);
    b = wave_sum(b);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if (lane == 0) { red[w] = a; red[16 + w] = b; }
    __syncthreads();
    float x = 0.f, y = 0.f;
    for (int i = 0; i < nw; ++i) { x += red[i]; y += red[16 + i]; }
    a = x;
    b = y;
}

// ---- mLSTM ----------------------------------------------------------------------------------------------------------
// x: rows of the fused projection, xs values apart; q at column q_off (H heads of d), k at k_off, v at v_off (H heads of
// dv), the output gate's rows at g_off (H dv).  gates [T, 2 H] float32: the raw products of the input and the forget
// gate.  state [slots][H][d dv + d + 1]: S (row dd, column j at dd dv + j), n, m.
template <typename TA, typename TW, int DR, int BT>
__global__ __launch_bounds__(BT) void mlstm_kernel(
    TA* __restrict__ out, float* __restrict__ state, const TA* __restrict__ x, long long xs, int q_off, int k_off, int v_off,
    int g_off, const float* __restrict__ gates, const TW* __restrict__ bi, const TW* __restrict__ bf, float cap,
    const TW* __restrict__ norm_w, float eps, const int* __restrict__ cu_q, const int* __restrict__ slot_ids, int num_slots, int H,
    int d, int dv) {
    __shared__ float ks[DR], qs[DR], red[32];
    const int s = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
    const int slot = slot_ids[s];
    if (slot < 0 || slot >= num_slots) return;
    const size_t head_state = (size_t)d * dv + d + 1;
    float* st = state + ((size_t)slot * H + h) * head_state;
    float S[DR];
    const bool col = j < dv, row = j < d;
#pragma unroll
    for (int dd = 0; dd < DR; ++dd) S[dd] = (col && dd < d) ? st[(size_t)dd * dv + j] : 0.f;
    float n = row ? st[(size_t)d * dv + j] : 0.f;
    float m = st[(size_t)d * dv + d];
    const float b_i = to_f32<TW>(bi[h]), b_f = to_f32<TW>(bf[h]);
    const float wn = col ? to_f32<TW>(norm_w[(size_t)h * dv + j]) : 0.f;
    const float qscale = 1.0f / sqrtf((float)d);
    const int t1 = cu_q[s + 1];
    for (int t = cu_q[s]; t < t1; ++t) {
        const TA* xr = x + (size_t)t * xs;
        if (row) {
            ks[j] = to_f32<TA>(xr[k_off + (size_t)h * d + j]);
            qs[j] = to_f32<TA>(xr[q_off + (size_t)h * d + j]) * qscale;
        }
        const float vj = col ? to_f32<TA>(xr[v_off + (size_t)h * dv + j]) : 0.f;
        const float gj = col ? to_f32<TA>(xr[g_off + (size_t)h * dv + j]) : 0.f;
        const float ig = cap * tanhf((gates[(size_t)t * 2 * H + h] + b_i) / cap);
        const float fg = mm_logsigmoid(cap * tanhf((gates[(size_t)t * 2 * H + H + h] + b_f) / cap));
        const float m_new = fmaxf(fg + m, ig);
        const float a = expf(fg + m - m_new), b = expf(ig - m_new);
        m = m_new;
        __syncthreads();
        float acc = 0.f, nq = 0.f;
        const float bv = b * vj;
#pragma unroll
        for (int dd = 0; dd < DR; ++dd) {
            if (dd < d) {
                S[dd] = fmaf(a, S[dd], ks[dd] * bv);
                acc = fmaf(S[dd], qs[dd], acc);
            }
        }
        if (row) {
            n = fmaf(a, n, b * ks[j]);
            nq = n * qs[j];
        }
        float ss = col ? acc * acc : 0.f;
        block_sum2(nq, ss, red);
        const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
        if (col) {
            const float o = acc / den;
            const float r = 1.0f / sqrtf(ss / (den * den) / (float)dv + eps);
            out[(size_t)t * H * dv + (size_t)h * dv + j] = from_f32<TA>(((o * r) * wn) * mm_sigmoid(gj));
        }
    }
#pragma unroll
    for (int dd = 0; dd < DR; ++dd)
        if (col && dd < d) st[(size_t)dd * dv + j] = S[dd];
    if (row) st[(size_t)d * dv + j] = n;
    if (j == 0) st[(size_t)d * dv + d] = m;
}

#define MM_LAUNCH(KERNEL, ...)                                                                                  \
    do {                                                                                                        \
        const int need_ = d > dv ? d : dv;                                                                      \
        const int bt_ = need_ <= 64 ? 64 : (need_ <= 256 ? 256 : 1024);                                        \
        const int threads_ = (need_ + 63) / 64 * 64;                                                            \
        if (d <= 64) {                                                                                          \
            if (bt_ == 64) KERNEL<TA, TW, 64, 64><<<grid, threads_, 0, st>>>(__VA_ARGS__);                      \
            else if (bt_ == 256) KERNEL<TA, TW, 64, 256><<<grid, threads_, 0, st>>>(__VA_ARGS__);               \
            else KERNEL<TA, TW, 64, 1024><<<grid, threads_, 0, st>>>(__VA_ARGS__);                              \
        } else if (d <= 128) {                                                                                  \
            if (bt_ <= 256) KERNEL<TA, TW, 128, 256><<<grid, threads_, 0, st>>>(__VA_ARGS__);                   \
            else KERNEL<TA, TW, 128, 1024><<<grid, threads_, 0, st>>>(__VA_ARGS__);                             \
        } else {                                                                                                \
            if (bt_ <= 256) KERNEL<TA, TW, 256, 256><<<grid, threads_, 0, st>>>(__VA_ARGS__);                   \
            else KERNEL<TA, TW, 256, 1024><<<grid, threads_, 0, st>>>(__VA_ARGS__);                             \
        }                                                                                                       \
    } while (0)

extern "C" int spy_mlstm(void* out, float* state, const void* x, long long xs, int dtype, int q_off, int k_off, int v_off, int g_off,
                         const float* gates, const void* bi, const void* bf, int w_dtype, float cap, const void* norm_w, float eps,
                         const int* cu_q, const int* slot_ids, int num_slots, int S, int T, int H, int d, int dv, hipStream_t st) {
    SPY_REQUIRE(S > 0 && T > 0 && H > 0 && d > 0 && dv > 0 && num_slots > 0, "spy_mlstm: empty operand");
    SPY_REQUIRE(d <= 256 && dv <= 1024 && H <= 65535, "spy_mlstm: heads of %d x %d (key size up to 256, value size up to 1024)", d, dv);
    SPY_REQUIRE(cap > 0.f, "spy_mlstm: the gates' cap must be positive");
    const dim3 grid(S, H);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, MM_LAUNCH(mlstm_kernel, (TA*)out, state, (const TA*)x, xs, q_off, k_off, v_off,
        g_off, gates, (const TW*)bi, (const TW*)bf, cap, (const TW*)norm_w, eps, cu_q, slot_ids, num_slots, H, d, dv)));
    SPY_CHECK_LAUNCH("spy_mlstm");
    return 0;
}

// ---- short causal convolution + silu -----------------------------------------------------------------------------------
// y[t, c] = silu(sum_j taps[c, j] x[t - (n - 1) + j, c]); inputs before the entry's first token come from the request's
// kept inputs keep[slot][n - 1][C] (index n - 2 the newest), which are zero for a new request.
template <typename TA, typename TW>
__global__ void causal_conv_silu_kernel(TA* __restrict__ y, const TA* __restrict__ x, long long xs, const TW* __restrict__ taps,
                                        const float* __restrict__ keep, long long keep_stride, const int* __restrict__ token_entry,
                                        const int* __restrict__ cu_q, const int* __restrict__ slot_ids, int num_slots, int T, int C,
                                        int n) {
    const size_t total = (size_t)T * C;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int t = (int)(i / C), c = (int)(i - (size_t)t * C);
        const int e = token_entry[t];
        const int t0 = cu_q[e];
        const int slot = slot_ids[e];
        const bool ok = slot >= 0 && slot < num_slots;
        float acc = 0.f;
        for (int j = 0; j < n; ++j) {
            const int src = t - (n - 1) + j;
            float v;
            if (src >= t0) v = to_f32<TA>(x[(size_t)src * xs + c]);
            else v = ok ? keep[(size_t)slot * keep_stride + (size_t)((n - 1) + (src - t0)) * C + c] : 0.f;
            acc = fmaf(to_f32<TW>(taps[(size_t)c * n + j]), v, acc);
        }
        y[i] = from_f32<TA>(acc * mm_sigmoid(acc));
    }
}

// after the convolution has read them: the kept inputs move on by the entry's tokens
#define CONV_MAX_TAPS 8
template <typename TA>
__global__ void conv_keep_kernel(float* __restrict__ keep, long long keep_stride, const TA* __restrict__ x, long long xs,
                                 const int* __restrict__ cu_q, const int* __restrict__ slot_ids, int num_slots, int C, int n) {
    const int e = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int slot = slot_ids[e];
    if (slot < 0 || slot >= num_slots) return;
    const int t0 = cu_q[e], L = cu_q[e + 1] - t0;
    float* kp = keep + (size_t)slot * keep_stride;
    float v[CONV_MAX_TAPS];
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
        if (i < n - 1) {
            const int rel = L - (n - 1) + i;
            v[i] = rel >= 0 ? to_f32<TA>(x[(size_t)(t0 + rel) * xs + c]) : kp[(size_t)(i + L) * C + c];
        }
    }
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS - 1; ++i)
        if (i < n - 1) kp[(size_t)i * C + c] = v[i];
}

extern "C" int spy_causal_conv_silu(void* y, const void* x, long long xs, int dtype, const void* taps, int w_dtype, float* keep,
                                    long long keep_stride, const int* token_entry, const int* cu_q, const int* slot_ids,
                                    int num_slots, int S, int T, int C, int n, hipStream_t st) {
    SPY_REQUIRE(S > 0 && T > 0 && C > 0 && num_slots > 0 && xs >= C, "spy_causal_conv_silu: empty operand");
    SPY_REQUIRE(n >= 1 && n <= CONV_MAX_TAPS && keep_stride >= (long long)(n - 1) * C && S <= 65535, "spy_causal_conv_silu: %d taps (1..%d)", n, CONV_MAX_TAPS);
    const size_t total = (size_t)T * C;
    const unsigned blocks = (unsigned)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (causal_conv_silu_kernel<TA, TW><<<blocks, 256, 0, st>>>(
        (TA*)y, (const TA*)x, xs, (const TW*)taps, keep, keep_stride, token_entry, cu_q, slot_ids, num_slots, T, C, n))));
    SPY_CHECK_LAUNCH("spy_causal_conv_silu");
    if (n > 1) {
        const dim3 grid((C + 255) / 256, S);
        SPY_DISPATCH(dtype, TA, (conv_keep_kernel<TA><<<grid, 256, 0, st>>>(keep, keep_stride, (const TA*)x, xs, cu_q, slot_ids, num_slots, C, n)));
        SPY_CHECK_LAUNCH("spy_causal_conv_silu (kept inputs)");
    }
    return 0;
}

// ---- gated delta rule with a decay per key channel ----------------------------------------------------------------------
// qkv [T, 2 G d + H dv]: the convolved, activated q (G heads of d), k (G heads of d), v (H heads of dv).  beta_pre [T, H]
// and dec_pre [T, H d] float32: raw products.  gate: rows of H dv values, gs apart.  state [slots][stride]: S of head h at
// h d dv, row dd and column j at dd dv + j.
template <typename TA, typename TW, int DR, int BT>
__global__ __launch_bounds__(BT) void delta_rule_kernel(
    TA* __restrict__ out, float* __restrict__ state, long long state_stride, const TA* __restrict__ qkv, const float* __restrict__ beta_pre,
    const float* __restrict__ dec_pre, const TW* __restrict__ a_log, const TW* __restrict__ dt_bias, const TA* __restrict__ gate,
    long long gs, const TW* __restrict__ norm_w, float eps, const int* __restrict__ cu_q, const int* __restrict__ slot_ids, int num_slots,
    int H, int G, int d, int dv) {
    __shared__ float ks[DR], qs[DR], dec[DR], red1[32], red2[32];
    const int s = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
    const int slot = slot_ids[s];
    if (slot < 0 || slot >= num_slots) return;
    const int g = h / (H / G);
    float* st = state + (size_t)slot * state_stride + (size_t)h * d * dv;
    float S[DR];
    const bool col = j < dv, row = j < d;
#pragma unroll
    for (int dd = 0; dd < DR; ++dd) S[dd] = (col && dd < d) ? st[(size_t)dd * dv + j] : 0.f;
    const float rate = expf(to_f32<TW>(a_log[h]));
    const float dtb = row ? to_f32<TW>(dt_bias[(size_t)h * d + j]) : 0.f;
    const float wn = col ? to_f32<TW>(norm_w[j]) : 0.f;
    const float qscale = 1.0f / sqrtf((float)d);
    const int C = 2 * G * d + H * dv;
    const int t1 = cu_q[s + 1];
    for (int t = cu_q[s]; t < t1; ++t) {
        const TA* xr = qkv + (size_t)t * C;
        float qq = 0.f, kk = 0.f, dc = 1.f;
        if (row) {
            qq = to_f32<TA>(xr[(size_t)g * d + j]);
            kk = to_f32<TA>(xr[(size_t)(G + g) * d + j]);
            const float z = dec_pre[(size_t)t * H * d + (size_t)h * d + j] + dtb;
            dc = expf(-rate * softplus_f(z));
        }
        const float vj = col ? to_f32<TA>(xr[(size_t)2 * G * d + (size_t)h * dv + j]) : 0.f;
        const float gj = col ? to_f32<TA>(gate[(size_t)t * gs + (size_t)h * dv + j]) : 0.f;
        const float beta = mm_sigmoid(beta_pre[(size_t)t * H + h]);
        float sq = qq * qq, sk = kk * kk;
        block_sum2(sq, sk, red1);
        if (row) {
            qs[j] = qq / sqrtf(sq + 1e-6f) * qscale;
            ks[j] = kk / sqrtf(sk + 1e-6f);
            dec[j] = dc;
        }
        __syncthreads();
        float r = 0.f;
#pragma unroll
        for (int dd = 0; dd < DR; ++dd) {
            if (dd < d) {
                S[dd] *= dec[dd];
                r = fmaf(S[dd], ks[dd], r);
            }
        }
        const float u = beta * (vj - r);
        float acc = 0.f;
#pragma unroll
        for (int dd = 0; dd < DR; ++dd) {
            if (dd < d) {
                S[dd] = fmaf(ks[dd], u, S[dd]);
                acc = fmaf(S[dd], qs[dd], acc);
            }
        }
        float ss = col ? acc * acc : 0.f, unused = 0.f;
        block_sum2(ss, unused, red2);
        if (col) {
            const float rr = 1.0f / sqrtf(ss / (float)dv + eps);
            out[(size_t)t * H * dv + (size_t)h * dv + j] = from_f32<TA>(((acc * rr) * wn) * mm_sigmoid(gj));
        }
    }
#pragma unroll
    for (int dd = 0; dd < DR; ++dd)
        if (col && dd < d) st[(size_t)dd * dv + j] = S[dd];
}

extern "C" int spy_delta_rule(void* out, float* state, long long state_stride, const void* qkv, int dtype, const float* beta_pre,
                              const float* dec_pre, const void* a_log, const void* dt_bias, int w_dtype, const void* gate, long long gs,
                              const void* norm_w, float eps, const int* cu_q, const int* slot_ids, int num_slots, int S, int T, int H,
                              int G, int d, int dv, hipStream_t st) {
    SPY_REQUIRE(S > 0 && T > 0 && H > 0 && G > 0 && H % G == 0 && d > 0 && dv > 0 && num_slots > 0, "spy_delta_rule: empty operand");
    SPY_REQUIRE(d <= 256 && dv <= 1024 && H <= 65535, "spy_delta_rule: heads of %d x %d (key size up to 256, value size up to 1024)", d, dv);
    SPY_REQUIRE(state_stride >= (long long)H * d * dv && gs >= (long long)H * dv, "spy_delta_rule: the state or the gate rows are too short");
    const dim3 grid(S, H);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, MM_LAUNCH(delta_rule_kernel, (TA*)out, state, state_stride, (const TA*)qkv, beta_pre,
        dec_pre, (const TW*)a_log, (const TW*)dt_bias, (const TA*)gate, gs, (const TW*)norm_w, eps, cu_q, slot_ids, num_slots, H, G, d, dv)));
    SPY_CHECK_LAUNCH("spy_delta_rule");
    return 0;
}
