// Attention over a cache of latent vectors: per token the cache holds one row [c (R) | kr (DR)] shared by all heads,
// c a normed low-rank vector from which keys and values are expanded (k_h = Wuk_h c, v_h = Wuv_h c) and kr a rotated key
// part.  The expansion is never formed: with qa_h = Wuk_h^T q_h the score is (qa_h . c + qr_h . kr) * scale, and the
// head's output is Wuv_h (sum_j p_j c_j).  So the kernels here see one "key" row of R + DR values and one "value" row of
// R values (its first part) per token and H query rows per token against them.
//
//   spy_latent_prepare    c = rmsnorm(dkv[:R]) * w and kr = rotate(dkv[R:]) into the pages; the heads' rotated query parts
//                         into the absorbed query rows
//   spy_gemm_strided      batched product with element strides (the per-head products with Wuk and Wuv), float32 sums
//   spy_latent_attention  plain kernel, float32: one block per (token, head); softmax with a sink in the denominator
#include "common.h"
#include <math.h>

// ---------------------------------------------------------------------------------------------
// Rotation: pair (i, i + dims/2), i < dims/2, of the rotated part; angle = position * freq[i] in float32, cos and sin
// times `mag`.  Values beyond `dims` pass unchanged.
template <typename TA, typename TW>
__global__ void latent_prepare_kernel(float* __restrict__ qa, const TA* __restrict__ q, int ldq, const TA* __restrict__ dkv, int ldd,
                                      TA* __restrict__ cache, const int* __restrict__ slot_mapping, long long cache_rows,
                                      const TW* __restrict__ w_norm, float eps, const float* __restrict__ freq, float mag,
                                      int dims, const int* __restrict__ positions, int H, int DN, int DR, int R) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const float p = (float)positions[t];
    const int half = dims / 2;
    // the heads' rotated parts -> qa[t, h, R ..]
    for (int idx = threadIdx.x; idx < H * DR; idx += blockDim.x) {
        const int h = idx / DR, i = idx - h * DR;
        const TA* src = q + (size_t)t * ldq + (size_t)h * (DN + DR) + DN;
        float v = to_f32<TA>(src[i]);
        if (i < dims) {
            const int j = i < half ? i : i - half;
            const float ang = p * freq[j];
            const float c = cosf(ang) * mag, s = sinf(ang) * mag;
            const float a = to_f32<TA>(src[j]), b = to_f32<TA>(src[j + half]);
            v = i < half ? a * c - b * s : b * c + a * s;
        }
        qa[((size_t)t * H + h) * (R + DR) + R + i] = v;
    }
    if (!dkv) return;
    const long long slot = slot_mapping[t];
    const TA* d = dkv + (size_t)t * ldd;
    float ss = 0.f;
    for (int i = threadIdx.x; i < R; i += blockDim.x) { const float v = to_f32<TA>(d[i]); ss += v * v; }
    ss = block_sum(ss, red);
    if (slot < 0 || slot >= cache_rows) return;
    TA* row = cache + (size_t)slot * (R + DR);
    const float scale = 1.0f / sqrtf(ss / (float)R + eps);
    for (int i = threadIdx.x; i < R; i += blockDim.x) row[i] = from_f32<TA>((scale * to_f32<TA>(d[i])) * to_f32<TW>(w_norm[i]));
    for (int i = threadIdx.x; i < DR; i += blockDim.x) {
        float v = to_f32<TA>(d[R + i]);
        if (i < dims) {
            const int j = i < half ? i : i - half;
            const float ang = p * freq[j];
            const float c = cosf(ang) * mag, s = sinf(ang) * mag;
            const float a = to_f32<TA>(d[R + j]), b = to_f32<TA>(d[R + j + half]);
            v = i < half ? a * c - b * s : b * c + a * s;
        }
        row[R + i] = from_f32<TA>(v);
    }
}

extern "C" int spy_latent_prepare(float* qa, const void* q, int ldq, const void* dkv, int ldd, int dtype, void* cache,
                                  const int* slot_mapping, long long cache_rows, const void* w_norm, int w_dtype, float eps,
                                  const float* freq, float mag, int dims, const int* positions, int T, int H, int DN, int DR, int R,
                                  hipStream_t st) {
    SPY_REQUIRE(T > 0 && H > 0 && DN >= 0 && DR >= 0 && R > 0, "spy_latent_prepare: empty operand");
    SPY_REQUIRE(dims >= 0 && dims <= DR && dims % 2 == 0 && (dims == 0 || freq), "spy_latent_prepare: %d rotated dims of %d", dims, DR);
    SPY_REQUIRE(!dkv || (cache && slot_mapping && w_norm), "spy_latent_prepare: storing needs the cache, the tokens' slots and the norm weight");
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (latent_prepare_kernel<TA, TW><<<T, 256, 0, st>>>(
        qa, (const TA*)q, ldq, (const TA*)dkv, ldd, (TA*)cache, slot_mapping, cache_rows, (const TW*)w_norm, eps, freq, mag, dims,
        positions, H, DN, DR, R))));
    SPY_CHECK_LAUNCH("spy_latent_prepare");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// C[b][m][n] = sum_k A[b][m][k] * B[b][n][k], element strides for every index, float32 products and sums in ascending k.
// A 64 x 64 tile of C per block as in the plain product; blockIdx.z = b.
#define GS_T 64
#define GS_K 16
template <typename TA, typename TB, typename TC>
__global__ __launch_bounds__(256) void gemm_strided_kernel(const TA* __restrict__ A, long long ab, long long am, long long ak,
                                                           const TB* __restrict__ B, long long bb, long long bn, long long bk,
                                                           TC* __restrict__ C, long long cb, long long cm, long long cn, int M, int N, int K) {
    __shared__ float As[GS_K][GS_T + 4];
    __shared__ float Bs[GS_K][GS_T + 4];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * GS_T, n0 = blockIdx.x * GS_T;
    A += (size_t)blockIdx.z * ab; B += (size_t)blockIdx.z * bb; C += (size_t)blockIdx.z * cb;
    float acc[4][4] = {};
    // A's k is the fast index of its loads where ak == 1 (rows of 16 k values), B's n or k whichever has stride 1
    const int lr = threadIdx.x >> 2, lk = (threadIdx.x & 3) * 4;
    for (int k0 = 0; k0 < K; k0 += GS_K) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k = k0 + lk + e;
            const int m = m0 + lr, n = n0 + lr;
            As[lk + e][lr] = (m < M && k < K) ? to_f32<TA>(A[(size_t)m * am + (size_t)k * ak]) : 0.f;
            Bs[lk + e][lr] = (n < N && k < K) ? to_f32<TB>(B[(size_t)n * bn + (size_t)k * bk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GS_K; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[k][ty * 4 + i]; b[i] = Bs[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) C[(size_t)m * cm + (size_t)n * cn] = from_f32<TC>(acc[i][j]);
        }
    }
}

extern "C" int spy_gemm_strided(const void* A, int a_dtype, long long ab, long long am, long long ak, const void* B, int b_dtype,
                                long long bb, long long bn, long long bk, void* C, int c_dtype, long long cb, long long cm,
                                long long cn, int batch, int M, int N, int K, hipStream_t st) {
    SPY_REQUIRE(batch > 0 && M > 0 && N > 0 && K > 0, "spy_gemm_strided: empty operand");
    const dim3 grid((N + GS_T - 1) / GS_T, (M + GS_T - 1) / GS_T, batch);
    SPY_REQUIRE(grid.y <= 65535 && batch <= 65535, "spy_gemm_strided: M = %d or batch = %d is too large for this kernel", M, batch);
    SPY_DISPATCH(a_dtype, TA, SPY_DISPATCH(b_dtype, TB, SPY_DISPATCH(c_dtype, TC, (gemm_strided_kernel<TA, TB, TC><<<grid, 256, 0, st>>>(
        (const TA*)A, ab, am, ak, (const TB*)B, bb, bn, bk, (TC*)C, cb, cm, cn, M, N, K)))));
    SPY_CHECK_LAUNCH("spy_gemm_strided");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// Plain attention over latent rows: one block per (token, head).  qa [T, H, R + DR] float32; cache [pages, P, R + DR];
// out [T, H, R] = sum_j p_j c_j with p = softmax over the keys the token sees and one more term, exp(sink_h), that has no
// key and no value.  Position i sees j with 0 <= i - j < window (window <= 0: all j <= i).  Keys in chunks of
// LA_THREADS with a running maximum that starts at the sink (so the denominator starts at 1).
#define LA_THREADS 256
#define LA_MAX_D 1024
template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(LA_THREADS) void latent_attention_kernel(
    TO* __restrict__ out, const float* __restrict__ qa, const TA* __restrict__ cache, int P, int num_pages,
    const int* __restrict__ kv_len, const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_entry,
    const int* __restrict__ positions, const TW* __restrict__ sink, int H, int R, int DR, float scale, int window) {
    __shared__ float qs[LA_MAX_D];
    __shared__ float ps[LA_THREADS];
    __shared__ long long ro[LA_THREADS];
    __shared__ float red[4];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int D = R + DR;
    const int s = token_entry[t];
    const int p = positions[t];
    int hi = p;
    if (hi > kv_len[s] - 1) hi = kv_len[s] - 1;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const float* qv = qa + ((size_t)t * H + h) * D;
    for (int j = tid; j < D; j += LA_THREADS) qs[j] = qv[j];
    float acc[LA_MAX_D / LA_THREADS] = {};
    float m = sink ? to_f32<TW>(sink[h]) : -INFINITY;
    float l = sink ? 1.f : 0.f;
    const int* bt = block_table + (size_t)s * max_blocks;
    __syncthreads();
    for (int c0 = lo; c0 <= hi; c0 += LA_THREADS) {
        const int c = c0 + tid;
        float sc = -INFINITY;
        long long row = -1;
        if (c <= hi) {
            const int page = bt[c / P];
            if (page >= 0 && page < num_pages) {
                row = ((long long)page * P + c % P) * D;
                const TA* kr = cache + row;
                float dot = 0.f;
                for (int j = 0; j < D; ++j) dot = fmaf(qs[j], to_f32<TA>(kr[j]), dot);
                sc = dot * scale;
            }
        }
        const float cm = block_max(sc, red);
        const float m_new = fmaxf(m, cm);
        const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
        const float pr = (sc == -INFINITY) ? 0.f : expf(sc - m_new);
        ps[tid] = pr; ro[tid] = row;
        const float csum = block_sum(pr, red);      // has the barriers that publish ps and ro
        l = l * alpha + csum;
        m = m_new;
        const int nk = min(LA_THREADS, hi - c0 + 1);
#pragma unroll
        for (int r = 0; r < LA_MAX_D / LA_THREADS; ++r) {
            const int j = tid + r * LA_THREADS;
            if (j < R) {
                float a = acc[r] * alpha;
                for (int i = 0; i < nk; ++i)
                    if (ro[i] >= 0) a = fmaf(ps[i], to_f32<TA>(cache[ro[i] + j]), a);
                acc[r] = a;
            }
        }
        __syncthreads();
    }
    TO* o = out + ((size_t)t * H + h) * R;
#pragma unroll
    for (int r = 0; r < LA_MAX_D / LA_THREADS; ++r) {
        const int j = tid + r * LA_THREADS;
        if (j < R) o[j] = from_f32<TO>(l > 0.f ? acc[r] / l : 0.f);
    }
}

extern "C" int spy_latent_attention(void* out, int out_dtype, const float* qa, const void* cache, int dtype, int P, int num_pages,
                                    const int* kv_len, const int* block_table, int max_blocks, const int* token_entry,
                                    const int* positions, const void* sink, int sink_dtype, int S, int T, int H, int R, int DR,
                                    float scale, int window, hipStream_t st) {
    SPY_REQUIRE(T > 0 && S > 0 && H > 0 && R > 0 && DR >= 0 && P > 0 && num_pages > 0 && max_blocks > 0,
                "spy_latent_attention: empty operand");
    SPY_REQUIRE(R + DR <= LA_MAX_D, "spy_latent_attention: rows of %d values exceed the supported %d", R + DR, LA_MAX_D);
    SPY_REQUIRE(H <= 65535, "spy_latent_attention: too many heads");
    const dim3 grid(T, H);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(sink_dtype, TW, SPY_DISPATCH(out_dtype, TO, (latent_attention_kernel<TA, TW, TO><<<grid, LA_THREADS, 0, st>>>(
        (TO*)out, qa, (const TA*)cache, P, num_pages, kv_len, block_table, max_blocks, token_entry, positions, (const TW*)sink, H, R,
        DR, scale, window)))));
    SPY_CHECK_LAUNCH("spy_latent_attention");
    return 0;
}
