// Gated linear recurrences whose gates read the current token only: S_t = (1 - z_t) S_(t-1) + z_t c_t per channel,
// the state float32 in a slot per request.  The projections come in as one row [z | x | g] per token.
//
// minGRU: z = sigmoid(zr + bz), u = xr + bx, c = u + 1/2 (u >= 0) or sigmoid(u) (u < 0), out = S_t * silu(g).
// Everything behind the projections is float32.
//
// A short entry (a decoded token, a small portion) is walked by one thread per channel.  A long one is cut into
// pieces of `piece` tokens: the recurrence is linear in the state, S_end = A S_start + B with A = prod(1 - z) and B the
// piece's walk from zero, so a first launch computes (A, B) of every piece, and the second launch folds the pieces
// before its own into its start state and walks its piece again with the outputs.
#include "common.h"
#include <math.h>

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ void mingru_gate(float zr, float xr, float bz, float bx, float& z, float& c) {
    z = sigmoid_f(zr + bz);
    const float u = xr + bx;
    c = u >= 0.f ? u + 0.5f : sigmoid_f(u);
}

// piece records: piece_entry[k], piece_t0[k], piece_t1[k] (token rows of the step), piece_first[k] = index of the
// entry's first piece.  AB [pieces][2][W] float32.
template <typename TA, typename TW>
__global__ void mingru_pieces_kernel(float* __restrict__ AB, const TA* __restrict__ zxg, const TW* __restrict__ bz,
                                     const TW* __restrict__ bx, const int* __restrict__ piece_t0, const int* __restrict__ piece_t1,
                                     int W) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= W) return;
    const int k = blockIdx.y;
    const float b_z = to_f32<TW>(bz[ch]), b_x = to_f32<TW>(bx[ch]);
    float A = 1.f, B = 0.f;
    const int t_end = piece_t1[k];
    // (unrolled: the loads do not depend on the recurrence and go out ahead of it)
#pragma unroll 8
    for (int t = piece_t0[k]; t < t_end; ++t) {
        const TA* row = zxg + (size_t)t * 3 * W;
        float z, c;
        mingru_gate(to_f32<TA>(row[ch]), to_f32<TA>(row[W + ch]), b_z, b_x, z, c);
        A *= (1.f - z);
        B = fmaf(1.f - z, B, z * c);
    }
    AB[((size_t)k * 2) * W + ch] = A;
    AB[((size_t)k * 2 + 1) * W + ch] = B;
}

template <typename TA, typename TW>
__global__ void mingru_scan_kernel(TA* __restrict__ out, float* __restrict__ state, const float* __restrict__ AB,
                                   const TA* __restrict__ zxg, const TW* __restrict__ bz, const TW* __restrict__ bx,
                                   const int* __restrict__ piece_entry, const int* __restrict__ piece_t0,
                                   const int* __restrict__ piece_t1, const int* __restrict__ piece_first,
                                   const int* __restrict__ slot_ids, int num_slots, int W) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= W) return;
    const int k = blockIdx.y;
    const int e = piece_entry[k];
    const int slot = slot_ids[e];
    if (slot < 0 || slot >= num_slots) return;
    const float b_z = to_f32<TW>(bz[ch]), b_x = to_f32<TW>(bx[ch]);
    float s = state[(size_t)slot * W + ch];
    for (int j = piece_first[k]; j < k; ++j) s = fmaf(AB[((size_t)j * 2) * W + ch], s, AB[((size_t)j * 2 + 1) * W + ch]);
    const int t1 = piece_t1[k];
#pragma unroll 8
    for (int t = piece_t0[k]; t < t1; ++t) {
        const TA* row = zxg + (size_t)t * 3 * W;
        float z, c;
        mingru_gate(to_f32<TA>(row[ch]), to_f32<TA>(row[W + ch]), b_z, b_x, z, c);
        s = fmaf(1.f - z, s, z * c);
        const float g = to_f32<TA>(row[2 * W + ch]);
        out[(size_t)t * W + ch] = from_f32<TA>(s * (g * sigmoid_f(g)));
    }
    // the entry's last piece leaves the state (the others read the old one: the write must wait for them, so it is a
    // launch of its own below when an entry has several pieces)
    if (piece_first[k] == k && (k + 1 == (int)gridDim.y || piece_first[k + 1] == k + 1)) state[(size_t)slot * W + ch] = s;
    else if (k + 1 == (int)gridDim.y || piece_first[k + 1] == k + 1) {
        // last of several pieces: park the state in this piece's A record, which nobody reads any more in this launch
        // (pieces after k belong to other entries)
        const_cast<float*>(AB)[((size_t)k * 2) * W + ch] = s;
    }
}

__global__ void mingru_keep_kernel(float* __restrict__ state, const float* __restrict__ AB, const int* __restrict__ piece_entry,
                                   const int* __restrict__ piece_first, const int* __restrict__ slot_ids, int num_slots, int W,
                                   int pieces) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= W) return;
    const int k = blockIdx.y;
    const bool last = k + 1 == pieces || piece_first[k + 1] == k + 1;
    if (!last || piece_first[k] == k) return;
    const int slot = slot_ids[piece_entry[k]];
    if (slot < 0 || slot >= num_slots) return;
    state[(size_t)slot * W + ch] = AB[((size_t)k * 2) * W + ch];
}

// The same two kernels for bfloat16 projections with an even number of channels: a thread owns two neighbouring channels,
// so that every load and store moves 4 bytes a lane (256 bytes a wave instead of 128: the walk is bound by the number
// of memory transactions, not by their bytes).
__device__ __forceinline__ float lo_bf16(uint32_t v) { return __uint_as_float(v << 16); }
__device__ __forceinline__ float hi_bf16(uint32_t v) { return __uint_as_float(v & 0xffff0000u); }

template <typename TW>
__global__ void mingru_pieces2_kernel(float* __restrict__ AB, const bf16_t* __restrict__ zxg, const TW* __restrict__ bz,
                                      const TW* __restrict__ bx, const int* __restrict__ piece_t0, const int* __restrict__ piece_t1,
                                      int W) {
    const int ch = 2 * (blockIdx.x * blockDim.x + threadIdx.x);
    if (ch >= W) return;
    const int k = blockIdx.y;
    const float bz0 = to_f32<TW>(bz[ch]), bz1 = to_f32<TW>(bz[ch + 1]), bx0 = to_f32<TW>(bx[ch]), bx1 = to_f32<TW>(bx[ch + 1]);
    float A0 = 1.f, B0 = 0.f, A1 = 1.f, B1 = 0.f;
    const int t_end = piece_t1[k];
#pragma unroll 8
    for (int t = piece_t0[k]; t < t_end; ++t) {
        const bf16_t* row = zxg + (size_t)t * 3 * W + ch;
        const uint32_t zr = *reinterpret_cast<const uint32_t*>(row), xr = *reinterpret_cast<const uint32_t*>(row + W);
        float z, c;
        mingru_gate(lo_bf16(zr), lo_bf16(xr), bz0, bx0, z, c);
        A0 *= (1.f - z); B0 = fmaf(1.f - z, B0, z * c);
        mingru_gate(hi_bf16(zr), hi_bf16(xr), bz1, bx1, z, c);
        A1 *= (1.f - z); B1 = fmaf(1.f - z, B1, z * c);
    }
    *reinterpret_cast<float2*>(AB + ((size_t)k * 2) * W + ch) = make_float2(A0, A1);
    *reinterpret_cast<float2*>(AB + ((size_t)k * 2 + 1) * W + ch) = make_float2(B0, B1);
}

template <typename TW>
__global__ void mingru_scan2_kernel(bf16_t* __restrict__ out, float* __restrict__ state, const float* __restrict__ AB,
                                    const bf16_t* __restrict__ zxg, const TW* __restrict__ bz, const TW* __restrict__ bx,
                                    const int* __restrict__ piece_entry, const int* __restrict__ piece_t0,
                                    const int* __restrict__ piece_t1, const int* __restrict__ piece_first,
                                    const int* __restrict__ slot_ids, int num_slots, int W) {
    const int ch = 2 * (blockIdx.x * blockDim.x + threadIdx.x);
    if (ch >= W) return;
    const int k = blockIdx.y;
    const int e = piece_entry[k];
    const int slot = slot_ids[e];
    if (slot < 0 || slot >= num_slots) return;
    const float bz0 = to_f32<TW>(bz[ch]), bz1 = to_f32<TW>(bz[ch + 1]), bx0 = to_f32<TW>(bx[ch]), bx1 = to_f32<TW>(bx[ch + 1]);
    float2 s = *reinterpret_cast<const float2*>(state + (size_t)slot * W + ch);
    for (int j = piece_first[k]; j < k; ++j) {
        const float2 a = *reinterpret_cast<const float2*>(AB + ((size_t)j * 2) * W + ch);
        const float2 b = *reinterpret_cast<const float2*>(AB + ((size_t)j * 2 + 1) * W + ch);
        s.x = fmaf(a.x, s.x, b.x);
        s.y = fmaf(a.y, s.y, b.y);
    }
    const int t1 = piece_t1[k];
#pragma unroll 8
    for (int t = piece_t0[k]; t < t1; ++t) {
        const bf16_t* row = zxg + (size_t)t * 3 * W + ch;
        const uint32_t zr = *reinterpret_cast<const uint32_t*>(row), xr = *reinterpret_cast<const uint32_t*>(row + W);
        const uint32_t gr = *reinterpret_cast<const uint32_t*>(row + 2 * W);
        float z, c;
        mingru_gate(lo_bf16(zr), lo_bf16(xr), bz0, bx0, z, c);
        s.x = fmaf(1.f - z, s.x, z * c);
        mingru_gate(hi_bf16(zr), hi_bf16(xr), bz1, bx1, z, c);
        s.y = fmaf(1.f - z, s.y, z * c);
        const float g0 = lo_bf16(gr), g1 = hi_bf16(gr);
        *reinterpret_cast<uint32_t*>(out + (size_t)t * W + ch) = pack_bf16x2(s.x * (g0 * sigmoid_f(g0)), s.y * (g1 * sigmoid_f(g1)));
    }
    const bool last = k + 1 == (int)gridDim.y || piece_first[k + 1] == k + 1;
    if (last && piece_first[k] == k) *reinterpret_cast<float2*>(state + (size_t)slot * W + ch) = s;
    else if (last) *reinterpret_cast<float2*>(const_cast<float*>(AB) + ((size_t)k * 2) * W + ch) = s;       // see mingru_scan_kernel
}

// pieces: int32 [4][n]: entry, t0, t1, first piece of the entry.  multi: some entry has more than one piece (then AB,
// float32 [n][2][W], is needed).
extern "C" int spy_mingru(void* out, float* state, float* AB, const void* zxg, int dtype, const void* bz, const void* bx,
                          int b_dtype, const int* pieces, int n_pieces, int multi, const int* slot_ids, int num_slots, int T,
                          int W, hipStream_t st) {
    SPY_REQUIRE(T > 0 && W > 0 && n_pieces > 0 && n_pieces <= 65535 && num_slots > 0, "spy_mingru: bad sizes (%d tokens, %d pieces)", T, n_pieces);
    SPY_REQUIRE(!multi || AB, "spy_mingru: entries in several pieces need the pieces' workspace");
    const int* pe = pieces;
    const int* p0 = pieces + n_pieces;
    const int* p1 = pieces + 2 * (size_t)n_pieces;
    const int* pf = pieces + 3 * (size_t)n_pieces;
    const int threads = W >= 256 ? 256 : 64;
    const dim3 grid((W + threads - 1) / threads, n_pieces);
    const bool two = dtype == SPY_BF16 && W % 2 == 0 && ((uintptr_t)zxg % 4) == 0 && ((uintptr_t)out % 4) == 0 &&
                     ((uintptr_t)state % 8) == 0 && ((uintptr_t)AB % 8) == 0;
    if (two) {
        const int th = W >= 512 ? 256 : 64;
        const dim3 grid2((W / 2 + th - 1) / th, n_pieces);
        if (multi) {
            SPY_DISPATCH(b_dtype, TW, (mingru_pieces2_kernel<TW><<<grid2, th, 0, st>>>(AB, (const bf16_t*)zxg, (const TW*)bz, (const TW*)bx, p0, p1, W)));
            SPY_CHECK_LAUNCH("spy_mingru (pieces)");
        }
        SPY_DISPATCH(b_dtype, TW, (mingru_scan2_kernel<TW><<<grid2, th, 0, st>>>(
            (bf16_t*)out, state, AB, (const bf16_t*)zxg, (const TW*)bz, (const TW*)bx, pe, p0, p1, pf, slot_ids, num_slots, W)));
        SPY_CHECK_LAUNCH("spy_mingru (scan)");
    } else {
        if (multi) {
            SPY_DISPATCH(dtype, TA, SPY_DISPATCH(b_dtype, TW, (mingru_pieces_kernel<TA, TW><<<grid, threads, 0, st>>>(
                AB, (const TA*)zxg, (const TW*)bz, (const TW*)bx, p0, p1, W))));
            SPY_CHECK_LAUNCH("spy_mingru (pieces)");
        }
        SPY_DISPATCH(dtype, TA, SPY_DISPATCH(b_dtype, TW, (mingru_scan_kernel<TA, TW><<<grid, threads, 0, st>>>(
            (TA*)out, state, AB, (const TA*)zxg, (const TW*)bz, (const TW*)bx, pe, p0, p1, pf, slot_ids, num_slots, W))));
        SPY_CHECK_LAUNCH("spy_mingru (scan)");
    }
    if (multi) {
        mingru_keep_kernel<<<grid, threads, 0, st>>>(state, AB, pe, pf, slot_ids, num_slots, W, n_pieces);
        SPY_CHECK_LAUNCH("spy_mingru (state)");
    }
    return 0;
}
