// Operations on the float32 residual stream for layers that norm a sublayer's OUTPUT and for models that mix the
// results of earlier layers: an embedding with a hashed pair table, stream + norm(y), a weighted sum of kept layer
// results, and the xIELU activation.  All arithmetic is float32; a bfloat16 value is rounded once, when it is written.
#include "common.h"
#include <math.h>

// ---------------------------------------------------------------------------------------------
// out[t] = table[id[t]] + pair[row(t)], row = (prev * mul_prev + id * mul_cur) mod buckets, the last row (number
// `buckets`) for a request's first token.  prev is the token before in the step, or for an entry's first token the one
// that the request's state slot holds (`last_token`, where the entry's last token is left for the next step).  copy
// (optional): the same values in
// the activation dtype, for the products that read the stream.
template <typename TW, typename TA>
__global__ void pair_embedding_kernel(float* __restrict__ out, TA* __restrict__ copy, const TW* __restrict__ table,
                                      const TW* __restrict__ pair, const int* __restrict__ ids, const int* __restrict__ positions,
                                      const int* __restrict__ token_entry, const int* __restrict__ cu_q,
                                      const int* __restrict__ slot_ids, int* last_token, int num_slots,
                                      int H, int V, int buckets, long long mul_prev, long long mul_cur) {
    const int t = blockIdx.x;
    const int id = ids[t];
    float* o = out + (size_t)t * H;
    TA* c = copy ? copy + (size_t)t * H : nullptr;
    if (id < 0 || id >= V) {
        for (int i = threadIdx.x; i < H; i += blockDim.x) { o[i] = 0.f; if (c) c[i] = from_f32<TA>(0.f); }
        return;
    }
    const TW* row = table + (size_t)id * H;
    const TW* prow = nullptr;
    if (pair) {
        // One thread finds the row of the pair table and hands it to the block.  Everything it reads is asked for whether
        // or not it is needed, so that the loads go out together: the token before, the entry with its first row and
        // slot, the slot's last token.  The block of an entry's FIRST token is the only one that reads the slot, so it is
        // also the one that leaves the entry's last token there: the same thread, after the barrier that its read's
        // result had to reach first (no other block touches the slot in this step).
        __shared__ int pair_row;
        int e = 0, first = 0, slot = -1;
        if (threadIdx.x == 0) {
            const int pos = positions[t], before = ids[t > 0 ? t - 1 : 0];
            e = token_entry[t];
            first = cu_q[e];
            slot = slot_ids[e];
            const int held = (slot >= 0 && slot < num_slots) ? last_token[slot] : 0;
            int r = buckets;
            if (pos > 0) {
                const int prev = t == first ? held : before;
                long long h = ((long long)prev * mul_prev + (long long)id * mul_cur) % (long long)buckets;
                if (h < 0) h += buckets;
                r = (int)h;
            }
            pair_row = r;
        }
        __syncthreads();
        prow = pair + (size_t)pair_row * H;
        if (threadIdx.x == 0 && t == first && slot >= 0 && slot < num_slots) last_token[slot] = ids[cu_q[e + 1] - 1];
    }
    if (sizeof(TW) == 2 && H % 8 == 0 && ((uintptr_t)row % 16) == 0 && (!prow || ((uintptr_t)prow % 16) == 0) && ((uintptr_t)o % 16) == 0 &&
        (!c || ((uintptr_t)c % 16) == 0)) {
        // bfloat16 tables: 8 values a thread and step, 16-byte loads of both rows asked for together
        typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
        typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f4_t;
#pragma unroll 2
        for (int i = threadIdx.x * 8; i < H; i += blockDim.x * 8) {
            const u32x4_t a = *reinterpret_cast<const u32x4_t*>(row + i);
            u32x4_t b = {0u, 0u, 0u, 0u};
            if (prow) b = *reinterpret_cast<const u32x4_t*>(prow + i);
            float v[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[2 * e] = __uint_as_float(a[e] << 16) + __uint_as_float(b[e] << 16);
                v[2 * e + 1] = __uint_as_float(a[e] & 0xffff0000u) + __uint_as_float(b[e] & 0xffff0000u);
            }
            *reinterpret_cast<f4_t*>(o + i) = f4_t{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<f4_t*>(o + i + 4) = f4_t{v[4], v[5], v[6], v[7]};
            if (c) {
                if (sizeof(TA) == 2) {
                    *reinterpret_cast<u32x4_t*>(c + i) = u32x4_t{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7])};
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) c[i + e] = from_f32<TA>(v[e]);
                }
            }
        }
        return;
    }
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float v = to_f32<TW>(row[i]);
        if (prow) v += to_f32<TW>(prow[i]);
        o[i] = v;
        if (c) c[i] = from_f32<TA>(v);
    }
}

extern "C" int spy_pair_embedding(float* out, void* copy, int copy_dtype, const void* table, const void* pair, int table_dtype,
                                  const int* ids, const int* positions, const int* token_entry, const int* cu_q,
                                  const int* slot_ids, int* last_token, int num_slots, int S, int T, int H, int V, int buckets,
                                  long long mul_prev, long long mul_cur, hipStream_t st) {
    SPY_REQUIRE(T > 0 && S > 0 && H > 0 && V > 0, "spy_pair_embedding: empty operand");
    SPY_REQUIRE(!pair || (buckets > 0 && last_token && num_slots > 0), "spy_pair_embedding: a pair table needs buckets and the slots' last tokens");
    const int threads = H >= 1024 ? 256 : 64;
    SPY_DISPATCH(table_dtype, TW, SPY_DISPATCH(copy_dtype, TA, (pair_embedding_kernel<TW, TA><<<T, threads, 0, st>>>(
        out, (TA*)copy, (const TW*)table, (const TW*)pair, ids, positions, token_entry, cu_q, slot_ids, last_token, num_slots, H, V,
        buckets, mul_prev, mul_cur))));
    SPY_CHECK_LAUNCH("spy_pair_embedding");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// out[t] = base[t] + y[t] / sqrt(mean(y[t]^2) + eps) * w;  copy[t] (optional) = the same in the activation dtype.
// out may be base (in place).  One block per row; y is read twice (the second read comes from the cache).
// With `mix` (n weights): out[t] is one of n kept layer results, kept[n - 1][t], and the kernel also writes
// mixed[t] = sum over j < n of mix[j] * kept[j][t] (added in ascending j, the new result last), whose copy `copy` then is:
// a layer's last sublayer and the weighted sum over all layer results that follows it, in one pass.
#define NR_PER 8      // values of a row that a thread keeps in registers between the two passes
template <typename TY, typename TW, typename TA, bool REG>
__global__ void norm_residual_kernel(float* out, TA* __restrict__ copy, const float* base,
                                     const TY* __restrict__ y, const TW* __restrict__ w, float eps, int H,
                                     float* __restrict__ mixed, const float* __restrict__ kept, size_t stride,
                                     const TW* __restrict__ mix, int n) {
    __shared__ float red[16];
    const size_t off = (size_t)blockIdx.x * H;
    const TY* yr = y + off;
    float ss = 0.f;
    if (REG) {
        // H <= NR_PER * blockDim.x: y is read once; what does not depend on the sum of squares (the stream's old values,
        // the norm weight, the other kept results) is asked for before the block's sum, so that one memory round trip
        // covers all of it
        float yv[NR_PER], bv[NR_PER], wv[NR_PER], sv[NR_PER];
#pragma unroll
        for (int e = 0; e < NR_PER; ++e) {
            const int i = threadIdx.x + e * blockDim.x;
            yv[e] = i < H ? to_f32<TY>(yr[i]) : 0.f;
            bv[e] = i < H ? base[off + i] : 0.f;
            wv[e] = i < H ? to_f32<TW>(w[i]) : 0.f;
            sv[e] = 0.f;
            ss += yv[e] * yv[e];
        }
        if (mixed) {
            for (int j = 0; j + 1 < n; ++j) {
                const float a = to_f32<TW>(mix[j]);
#pragma unroll
                for (int e = 0; e < NR_PER; ++e) {
                    const int i = threadIdx.x + e * blockDim.x;
                    if (i < H) sv[e] = fmaf(a, kept[(size_t)j * stride + off + i], sv[e]);
                }
            }
        }
        ss = block_sum(ss, red);
        const float scale = 1.0f / sqrtf(ss / (float)H + eps);
        const float a_last = mixed ? to_f32<TW>(mix[n - 1]) : 0.f;
#pragma unroll
        for (int e = 0; e < NR_PER; ++e) {
            const int i = threadIdx.x + e * blockDim.x;
            if (i < H) {
                float v = bv[e] + (scale * yv[e]) * wv[e];
                out[off + i] = v;
                if (mixed) { v = fmaf(a_last, v, sv[e]); mixed[off + i] = v; }
                if (copy) copy[off + i] = from_f32<TA>(v);
            }
        }
        return;
    }
    // Few rows: gridDim.y blocks share a row.  Each forms the whole row's sum of squares (the row is a few kilobytes, from
    // L2) and writes its slice of the outputs, so that a step of a handful of tokens still has blocks for many units.
    if (sizeof(TY) == 2 && H % 8 == 0 && ((uintptr_t)yr % 16) == 0) {
        // bfloat16 rows in 16-byte pieces, all of a thread's pieces asked for before the first is squared
        typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
        const u32x4_t* y8 = reinterpret_cast<const u32x4_t*>(yr);
#pragma unroll 4
        for (int i = threadIdx.x; i < H / 8; i += blockDim.x) {
            const u32x4_t v = y8[i];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float a = __uint_as_float(v[e] << 16), b = __uint_as_float(v[e] & 0xffff0000u);
                ss = fmaf(a, a, fmaf(b, b, ss));
            }
        }
    } else {
#pragma unroll 8
        for (int i = threadIdx.x; i < H; i += blockDim.x) { const float v = to_f32<TY>(yr[i]); ss += v * v; }
    }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)H + eps);
    const int lo = (int)((long long)H * blockIdx.y / gridDim.y), hi = (int)((long long)H * (blockIdx.y + 1) / gridDim.y);
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        float v = base[off + i] + (scale * to_f32<TY>(yr[i])) * to_f32<TW>(w[i]);
        out[off + i] = v;
        if (mixed) {
            float s = 0.f;
#pragma unroll 4
            for (int j = 0; j + 1 < n; ++j) s = fmaf(to_f32<TW>(mix[j]), kept[(size_t)j * stride + off + i], s);
            v = fmaf(to_f32<TW>(mix[n - 1]), v, s);
            mixed[off + i] = v;
        }
        if (copy) copy[off + i] = from_f32<TA>(v);
    }
}

extern "C" int spy_norm_residual(float* out, void* copy, int copy_dtype, const float* base, const void* y, int y_dtype,
                                 const void* w, int w_dtype, float eps, int T, int H, float* mixed, const float* kept,
                                 long long stride, const void* mix, int n, hipStream_t st) {
    SPY_REQUIRE(T > 0 && H > 0, "spy_norm_residual: empty operand");
    SPY_REQUIRE(!mixed || (kept && mix && n > 0 && stride >= (long long)T * H && out == kept + (size_t)(n - 1) * stride),
                "spy_norm_residual: the mix needs the kept results, whose last one is this result, and their weights");
    const int threads = H >= 2048 ? 512 : (H >= 512 ? 256 : 64);
    if (T <= 128 && H >= 1024) {
        // rows for fewer blocks than the device has units: several blocks per row
        const int per_row = T <= 32 ? 8 : (T <= 64 ? 4 : 2);
        const dim3 grid(T, per_row);
        SPY_DISPATCH(y_dtype, TY, SPY_DISPATCH(w_dtype, TW, SPY_DISPATCH(copy_dtype, TA, (norm_residual_kernel<TY, TW, TA, false><<<grid, 256, 0, st>>>(
            out, (TA*)copy, base, (const TY*)y, (const TW*)w, eps, H, mixed, kept, (size_t)stride, (const TW*)mix, n)))));
    } else if (H <= NR_PER * threads) {
        SPY_DISPATCH(y_dtype, TY, SPY_DISPATCH(w_dtype, TW, SPY_DISPATCH(copy_dtype, TA, (norm_residual_kernel<TY, TW, TA, true><<<T, threads, 0, st>>>(
            out, (TA*)copy, base, (const TY*)y, (const TW*)w, eps, H, mixed, kept, (size_t)stride, (const TW*)mix, n)))));
    } else {
        SPY_DISPATCH(y_dtype, TY, SPY_DISPATCH(w_dtype, TW, SPY_DISPATCH(copy_dtype, TA, (norm_residual_kernel<TY, TW, TA, false><<<T, threads, 0, st>>>(
            out, (TA*)copy, base, (const TY*)y, (const TW*)w, eps, H, mixed, kept, (size_t)stride, (const TW*)mix, n)))));
    }
    SPY_CHECK_LAUNCH("spy_norm_residual");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// out[i] = sum over j < n of a[j] * kept[j][i], added in ascending j; kept is [n or more][count] float32 with `stride`
// elements between layers.  copy (optional): the result in the activation dtype.
#define DEPTH_MAX 256
template <typename TW, typename TA>
__global__ void depth_mix_kernel(float* __restrict__ out, TA* __restrict__ copy, const float* __restrict__ kept, size_t stride,
                                 const TW* __restrict__ a, int n, size_t count) {
    __shared__ float as[DEPTH_MAX];
    for (int j = threadIdx.x; j < n; j += blockDim.x) as[j] = to_f32<TW>(a[j]);
    __syncthreads();
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
        float s = 0.f;
        for (int j = 0; j < n; ++j) s = fmaf(as[j], kept[(size_t)j * stride + i], s);
        out[i] = s;
        if (copy) copy[i] = from_f32<TA>(s);
    }
}

extern "C" int spy_depth_mix(float* out, void* copy, int copy_dtype, const float* kept, long long stride, const void* a, int a_dtype,
                             int n, long long count, hipStream_t st) {
    SPY_REQUIRE(n > 0 && n <= DEPTH_MAX && count > 0 && stride >= count, "spy_depth_mix: %d layers (1..%d allowed), %lld values", n, DEPTH_MAX, count);
    long long blocks = (count + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    SPY_DISPATCH(a_dtype, TW, SPY_DISPATCH(copy_dtype, TA, (depth_mix_kernel<TW, TA><<<(unsigned)blocks, 256, 0, st>>>(
        out, (TA*)copy, kept, (size_t)stride, (const TW*)a, n, (size_t)count))));
    SPY_CHECK_LAUNCH("spy_depth_mix");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// xIELU with the two learned numbers pq = (p, q):  z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2
// (softplus_f and xielu_f: common.h, shared with the decode product's store epilogue)

template <typename TA, typename TW>
__global__ void xielu_kernel(TA* __restrict__ out, const TA* __restrict__ in, const TW* __restrict__ pq, size_t count) {
    const float ap = softplus_f(to_f32<TW>(pq[0])), aq = 0.5f + softplus_f(to_f32<TW>(pq[1]));
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        out[i] = from_f32<TA>(xielu_f(to_f32<TA>(in[i]), ap, aq));
}

// the same, 8 bfloat16 values per thread and step with 16-byte loads and stores (count % 8 == 0, aligned)
template <typename TW>
__global__ void xielu_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ in, const TW* __restrict__ pq, size_t count8) {
    typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
    const float ap = softplus_f(to_f32<TW>(pq[0])), aq = 0.5f + softplus_f(to_f32<TW>(pq[1]));
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count8; i += (size_t)gridDim.x * blockDim.x) {
        const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(in) + i);
        u32x4_t y;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            y[e] = pack_bf16x2(xielu_f(__uint_as_float(v[e] << 16), ap, aq), xielu_f(__uint_as_float(v[e] & 0xffff0000u), ap, aq));
        reinterpret_cast<u32x4_t*>(out)[i] = y;
    }
}

extern "C" int spy_xielu(void* out, const void* in, int dtype, const void* pq, int pq_dtype, long long count, hipStream_t st) {
    SPY_REQUIRE(count > 0, "spy_xielu: empty operand");
    if (dtype == SPY_BF16 && count % 8 == 0 && ((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 16) == 0) {
        long long blocks = (count / 8 + 255) / 256;
        if (blocks > 16384) blocks = 16384;
        SPY_DISPATCH(pq_dtype, TW, (xielu_bf16x8_kernel<TW><<<(unsigned)blocks, 256, 0, st>>>((bf16_t*)out, (const bf16_t*)in, (const TW*)pq, (size_t)(count / 8))));
        SPY_CHECK_LAUNCH("spy_xielu");
        return 0;
    }
    long long blocks = (count + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(pq_dtype, TW, (xielu_kernel<TA, TW><<<(unsigned)blocks, 256, 0, st>>>(
        (TA*)out, (const TA*)in, (const TW*)pq, (size_t)count))));
    SPY_CHECK_LAUNCH("spy_xielu");
    return 0;
}
