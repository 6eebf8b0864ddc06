// The experts' products on the matrix cores (bfloat16), and a product with few output features.
#include "common.h"
#include "api.h"
#include "recordable.h"

#define MT_TILE 64            // rows of a tile (fl_moe_route cuts the sorted pairs into tiles of this many)
#define MT_FEATURES 256       // output features per block: four waves of 64

// out[p][:] = (scale[p] * x[src[p]]) W_e^T over the tiles of fl_moe_route, as fl_moe_gemm computes it, with
// v_mfma_f32_16x16x32_bf16, K in steps of 32.  A wave takes 64 features (four A operands, read straight
// from the expert's rows, four steps ahead) against the tile's rows in groups of 16 (B operands).  The rows
// are gathered, scaled and rounded once per block and shared through LDS (two slots, one barrier a
// step; the 16-byte pieces of a row are exchanged by (row / 2) % 4 so that the reads of a group of
// rows meet in no bank).  Row groups a tile does not have are skipped, so a decode step (a row or two
// per expert) streams the weights once.
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(const bf16_t* __restrict__ x, const int* __restrict__ src_row,
                                                            const float* __restrict__ src_scale, const bf16_t* __restrict__ w,
                                                            float* __restrict__ out, const int* __restrict__ tiles, int N, int K) {
    __shared__ bf16x8 xs[2][MT_TILE * 4];
    const int e = tiles[4 * blockIdx.y + 0];
    if (e < 0) return;                                   // (the whole block: tiles are per block)
    const int p0 = tiles[4 * blockIdx.y + 1], M = tiles[4 * blockIdx.y + 2];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col = lane & 15, g = lane >> 4;
    const int f0 = blockIdx.x * MT_FEATURES + wave * 64;
    const bf16_t* we = w + (size_t)e * N * K;
    const bf16_t* wrow[4];
    bool wlive[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int f = f0 + 16 * a + col;
        wlive[a] = f < N;
        wrow[a] = we + (size_t)(wlive[a] ? f : 0) * K + 8 * g;
    }
    const int groups = (M + 15) >> 4;
    // this thread's share of the rows' staging: row threadIdx.x / 4, the 16-byte piece threadIdx.x % 4 of a step
    const int srow = threadIdx.x >> 2, spiece = threadIdx.x & 3;
    const bool slive = srow < M;
    const int sp = p0 + (slive ? srow : 0);
    const bf16_t* sx = x + (size_t)(src_row ? src_row[sp] : sp) * K + 8 * spiece;
    const float sscale = src_scale ? src_scale[sp] : 1.0f;
    const int sslot = srow * 4 + (spiece ^ ((srow >> 1) & 3));
    const bf16x8 zero = {(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};
    auto staged = [&](int k0) {
        bf16x8 v = slive ? *(const bf16x8*)(sx + k0) : zero;
        if (src_scale) {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = (bf16_t)((float)v[i] * sscale);
        }
        return v;
    };
    f32x4 acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[a][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // The weights and the rows' pieces of a step are asked for four steps before they are used (a ring of registers):
    // a trip to memory takes some thousand clocks, the products of a step a few hundred.
    const int steps = K >> 5;
    bf16x8 avq[4][4], xq[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        if (d < steps) {
#pragma unroll
            for (int a = 0; a < 4; ++a) avq[d][a] = wlive[a] ? *(const bf16x8*)(wrow[a] + 32 * d) : zero;
            xq[d] = staged(32 * d);
        }
    }
    xs[0][sslot] = xq[0];
    __syncthreads();
    for (int s0 = 0; s0 < steps; s0 += 4) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int s_now = s0 + j;
            if (s_now < steps) {                                   // (the same for every thread of the block)
                const int cur = j & 1;
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (t < groups) {
                        const int r = 16 * t + col;
                        const bf16x8 bv = xs[cur][r * 4 + (g ^ ((r >> 1) & 3))];
#pragma unroll
                        for (int a = 0; a < 4; ++a) acc[a][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(avq[j][a], bv, acc[a][t], 0, 0, 0);
                    }
                if (s_now + 1 < steps) xs[cur ^ 1][sslot] = xq[(j + 1) & 3];
                if (s_now + 4 < steps) {
#pragma unroll
                    for (int a = 0; a < 4; ++a) avq[j][a] = wlive[a] ? *(const bf16x8*)(wrow[a] + 32 * (s_now + 4)) : zero;
                    xq[j] = staged(32 * (s_now + 4));
                }
                __syncthreads();
            }
        }
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int r = 16 * t + col;
        if (r >= M) continue;
        float* dst = out + (size_t)(p0 + r) * N;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int f = f0 + 16 * a + 4 * g;
            if (f + 3 < N) {
                *(f32x4*)(dst + f) = acc[a][t];
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (f + q < N) dst[f + q] = acc[a][t][q];
            }
        }
    }
}

#define MT_STREAM_FEATURES 32        // output features per block of the streaming form
// The same for steps of few rows (decoding), where nearly every tile holds a row or two and all a block does is
// stream its expert's weights: a block takes 32 features and its four waves deal the steps of K out among them
// (wave w: steps w, w + 4, ...; together they read the rows end to end), so that even a step that touches four
// experts has some hundred blocks; their sums are added through LDS in a fixed order.  No barrier inside the loop.
__global__ __launch_bounds__(256) void moe_gemm_mfma_stream_kernel(const bf16_t* __restrict__ x, const int* __restrict__ src_row,
                                                                   const float* __restrict__ src_scale, const bf16_t* __restrict__ w,
                                                                   float* __restrict__ out, const int* __restrict__ tiles, int N, int K) {
    __shared__ f32x4 part[4][2][4][64];
    const int e = tiles[4 * blockIdx.y + 0];
    if (e < 0) return;
    const int p0 = tiles[4 * blockIdx.y + 1], M = tiles[4 * blockIdx.y + 2];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col = lane & 15, g = lane >> 4;
    const int f0 = blockIdx.x * MT_STREAM_FEATURES;
    const bf16_t* we = w + (size_t)e * N * K;
    const bf16_t* wrow[2];
    bool wlive[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const int f = f0 + 16 * a + col;
        wlive[a] = f < N;
        wrow[a] = we + (size_t)(wlive[a] ? f : 0) * K + 8 * g;
    }
    const int groups = (M + 15) >> 4;
    const bf16_t* xrow[4];
    float xs[4];
    bool xlive[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int r = 16 * t + col;
        xlive[t] = r < M;
        const int p = p0 + (xlive[t] ? r : 0);
        xrow[t] = x + (size_t)(src_row ? src_row[p] : p) * K + 8 * g;
        xs[t] = src_scale ? src_scale[p] : 1.0f;
    }
    f32x4 acc[2][4];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[a][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const bf16x8 zero = {(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};
#pragma unroll 4
    for (int k0 = 32 * wave; k0 < K; k0 += 128) {
        bf16x8 av[2], bv[4];
#pragma unroll
        for (int a = 0; a < 2; ++a) av[a] = wlive[a] ? *(const bf16x8*)(wrow[a] + k0) : zero;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (t < groups) {
                bv[t] = xlive[t] ? *(const bf16x8*)(xrow[t] + k0) : zero;
                if (src_scale) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) bv[t][i] = (bf16_t)((float)bv[t][i] * xs[t]);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
            if (t < groups) {
#pragma unroll
                for (int a = 0; a < 2; ++a) acc[a][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[a], bv[t], acc[a][t], 0, 0, 0);
            }
    }
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int t = 0; t < 4; ++t)
            if (t < groups) part[wave][a][t][lane] = acc[a][t];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (!xlive[t] || t >= groups) continue;
        float* dst = out + (size_t)(p0 + 16 * t + col) * N;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            const f32x4 sum = (part[0][a][t][lane] + part[1][a][t][lane]) + (part[2][a][t][lane] + part[3][a][t][lane]);
            const int f = f0 + 16 * a + 4 * g;
            if (f + 3 < N) {
                *(f32x4*)(dst + f) = sum;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (f + r < N) dst[f + r] = sum[r];
            }
        }
    }
}

extern "C" int fl_moe_gemm_mfma_takes(int N, int K) { return N > 0 && N % 4 == 0 && K > 0 && K % 32 == 0; }

extern "C" int fl_moe_gemm_mfma(const void* x, const int* src_row, const float* src_scale, const void* w, float* out,
                                const int* tiles, int max_tiles, int n_rows, int N, int K, hipStream_t stream) {
    FL_CHECK(max_tiles >= 0 && n_rows >= 0 && fl_moe_gemm_mfma_takes(N, K), "moe_gemm_mfma: %d features over %d values are not taken", N, K);
    FL_CHECK((uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)out % 16 == 0, "moe_gemm_mfma: operands must be 16-byte aligned");
    if (max_tiles == 0) return 0;
    FL_CHECK(max_tiles <= 65535, "moe_gemm_mfma: %d row tiles are more than one grid takes", max_tiles);
    if (n_rows <= 2 * MT_TILE) {
        dim3 grid(ceil_div(N, MT_STREAM_FEATURES), max_tiles);
        moe_gemm_mfma_stream_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)x, src_row, src_scale, (const bf16_t*)w, out, tiles, N, K);
    } else {
        dim3 grid(ceil_div(N, MT_FEATURES), max_tiles);
        moe_gemm_mfma_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)x, src_row, src_scale, (const bf16_t*)w, out, tiles, N, K);
    }
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_moe_gemm_mfma)

// ------------------------------------------------------------------ a product with few output features
// out[m][f] = sum_k x[m][k] w[f][k] for a handful of features (a router's scores, a gate's logit): one
// wave per output element, the lanes stride over k and add their parts in a fixed tree, so an element
// does not depend on how many rows the call has.  Products of stored values are exact in float; the
// sums are float.
template <typename T>
__global__ __launch_bounds__(256) void gemm_few_kernel(const T* __restrict__ x, const T* __restrict__ w, float* __restrict__ out,
                                                       long total, int N, int K) {
    const long unit = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= total) return;
    const int lane = threadIdx.x & 63;
    const long m = unit / N;
    const int f = (int)(unit - m * N);
    const T* xr = x + (size_t)m * K;
    const T* wr = w + (size_t)f * K;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int k = 4 * lane;
    if (K % 4 == 0) {
        for (; k + 3 < K; k += 256) {
            a0 = fmaf(to_f32(xr[k]), to_f32(wr[k]), a0);
            a1 = fmaf(to_f32(xr[k + 1]), to_f32(wr[k + 1]), a1);
            a2 = fmaf(to_f32(xr[k + 2]), to_f32(wr[k + 2]), a2);
            a3 = fmaf(to_f32(xr[k + 3]), to_f32(wr[k + 3]), a3);
        }
    } else {
        for (k = lane; k < K; k += 64) a0 = fmaf(to_f32(xr[k]), to_f32(wr[k]), a0);
    }
    const float s = wave_sum((a0 + a1) + (a2 + a3));
    if (lane == 0) out[unit] = s;
}

extern "C" int fl_gemm_few(const void* x, const void* w, float* out, int dtype, int M, int N, int K, hipStream_t stream) {
    FL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_few: bad sizes M=%d N=%d K=%d", M, N, K);
    if (M == 0) return 0;
    const long total = (long)M * N;
    const long blocks = (total + 3) / 4;
    FL_CHECK(blocks < (1L << 31), "gemm_few: too many outputs");
    if (dtype == FL_F32) gemm_few_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>((const float*)x, (const float*)w, out, total, N, K);
    else if (dtype == FL_BF16) gemm_few_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)w, out, total, N, K);
    else FL_CHECK(false, "gemm_few: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_gemm_few)
