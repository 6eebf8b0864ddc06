// Attention over one cached latent per token.
//
// A token keeps one normed row c [R] in the paged cache; every head's keys and values are linear in c
// (k = Wk_h c, v = Wv_h c), so the key expansion is folded into the query and the value expansion is
// applied after the weighted sum:
//     qa_h = Wk_h^T q_h                      (fl_heads_matmul, weights as they are)
//     s_j  = scale * qa_h . c_j,  p = softmax over j <= position
//     z_h  = sum_j p_j c_j                    (fl_latent_attention)
//     o_h  = sigmoid(gate_h) * Wv_h z_h       (fl_heads_matmul, weights transposed, gated)
// Scores, softmax, z and the two small products are 32-bit whatever the storage type of the cache.
#include "common.h"
#include "api.h"
#include "recordable.h"

// ------------------------------------------------------------------ norm of a slice of columns
// out[r, :] = v * w * rsqrt(mean(v^2) + eps), v = x[r, col0 : col0 + width] of float rows ld wide.
// With a block table the result goes to the page of the token's position, else to the dense
// out[n][width].  A page holds its rows twice, [n_pages][2][page_size * width]: row by row
// ([page_size][width]) and transposed ([width][page_size]); the matrix cores want the index that is
// summed over contiguous, the latent's dims for the scores and the keys for the weighted sum.
template <typename T>
__global__ __launch_bounds__(256) void norm_slice_kernel(const float* __restrict__ x, int ld, int col0, int width,
                                                         const float* __restrict__ w, float eps, T* __restrict__ out,
                                                         const int* __restrict__ positions, const int* __restrict__ tok_seq,
                                                         const int* __restrict__ block_table, int max_blocks,
                                                         int page_size, int n_pages) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float* xr = x + (size_t)r * ld + col0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += 256) ss += xr[i] * xr[i];
    const float total = block_sum<4>(ss, red);
    const float inv = 1.0f / sqrtf(total / (float)width + eps);
    if (block_table) {
        const int pos = positions[r];
        const int page = block_table[(size_t)tok_seq[r] * max_blocks + pos / page_size];
        if (page < 0 || page >= n_pages) return;          // rows that pad a batch of fixed shape
        const int row = pos % page_size;
        T* rows = out + (size_t)page * 2 * page_size * width;
        T* cols = rows + (size_t)page_size * width;
        for (int i = threadIdx.x; i < width; i += 256) {
            const T v = from_f32<T>(xr[i] * (w ? w[i] : 1.0f) * inv);
            rows[(size_t)row * width + i] = v;
            cols[(size_t)i * page_size + row] = v;
        }
        return;
    }
    T* dst = out + (size_t)r * width;
    for (int i = threadIdx.x; i < width; i += 256) dst[i] = from_f32<T>(xr[i] * (w ? w[i] : 1.0f) * inv);
}

extern "C" int fl_norm_slice(const float* x, int ld, int col0, int width, const float* w, float eps, void* out,
                             int out_dtype, int n, const int* positions, const int* tok_seq, const int* block_table,
                             int max_blocks, int page_size, int n_pages, hipStream_t stream) {
    FL_CHECK(n >= 0 && width > 0 && col0 >= 0 && ld >= col0 + width, "norm_slice: columns %d..%d of rows %d wide", col0, col0 + width, ld);
    FL_CHECK(!block_table || (positions && tok_seq && max_blocks > 0 && page_size > 0 && n_pages > 0), "norm_slice: a paged store needs positions, requests and the pool's sizes");
    if (n == 0) return 0;
    if (out_dtype == FL_F32)
        norm_slice_kernel<float><<<n, 256, 0, stream>>>(x, ld, col0, width, w, eps, (float*)out, positions, tok_seq, block_table, max_blocks, page_size, n_pages);
    else if (out_dtype == FL_BF16)
        norm_slice_kernel<bf16_t><<<n, 256, 0, stream>>>(x, ld, col0, width, w, eps, (bf16_t*)out, positions, tok_seq, block_table, max_blocks, page_size, n_pages);
    else
        FL_CHECK(false, "norm_slice: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_norm_slice)

// ------------------------------------------------------------------ one small product per head
// x [n][H][K] (float, rows ldx apart), one matrix per head taken from w [H * rows_per_head][cols]:
//   transposed = 0: w_h is [K][J] (rows_per_head = K, cols = J),   out[t][h][j] = sum_k x[t][h][k] w_h[k][j]
//   transposed = 1: w_h is [J][K] (rows_per_head = J, cols = K),   out[t][h][j] = sum_k x[t][h][k] w_h[j][k]
// gate (or null): float rows ldg apart, gate[t][gate_col0 + h] is a logit; the head's output is multiplied
// by its sigmoid.  A block takes HM_TOKENS tokens of one head; a thread owns output columns and keeps
// one sum per token, so every weight is read once per block.  Sums run over k in rising order.
#define HM_TOKENS 8
template <typename TW, typename TOut>
__global__ __launch_bounds__(256) void heads_matmul_kernel(const float* __restrict__ x, int ldx, const TW* __restrict__ w,
                                                           TOut* __restrict__ out, int n, int H, int K, int J, int transposed,
                                                           const float* __restrict__ gate, int ldg, int gate_col0) {
    extern __shared__ float xs[];                     // [HM_TOKENS][K]
    const int t0 = blockIdx.x * HM_TOKENS, h = blockIdx.y;
    const int nt = min(HM_TOKENS, n - t0);
    for (int e = threadIdx.x; e < HM_TOKENS * K; e += 256) {
        const int i = e / K, k = e - i * K;
        xs[e] = i < nt ? x[(size_t)(t0 + i) * ldx + (size_t)h * K + k] : 0.f;
    }
    __syncthreads();
    const TW* wh = w + (size_t)h * K * J;             // either form holds K * J values per head
    for (int j = threadIdx.x; j < J; j += 256) {
        float acc[HM_TOKENS];
#pragma unroll
        for (int i = 0; i < HM_TOKENS; ++i) acc[i] = 0.f;
        if (transposed) {
            const TW* row = wh + (size_t)j * K;
            for (int k = 0; k < K; ++k) {
                const float wv = to_f32(row[k]);
#pragma unroll
                for (int i = 0; i < HM_TOKENS; ++i) acc[i] = fmaf(xs[i * K + k], wv, acc[i]);
            }
        } else {
            for (int k = 0; k < K; ++k) {
                const float wv = to_f32(wh[(size_t)k * J + j]);
#pragma unroll
                for (int i = 0; i < HM_TOKENS; ++i) acc[i] = fmaf(xs[i * K + k], wv, acc[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < HM_TOKENS; ++i) {
            if (i >= nt) break;
            float v = acc[i];
            if (gate) v *= 1.0f / (1.0f + expf(-gate[(size_t)(t0 + i) * ldg + gate_col0 + h]));
            out[((size_t)(t0 + i) * H + h) * J + j] = from_f32<TOut>(v);
        }
    }
}

extern "C" int fl_heads_matmul(const float* x, int ldx, const void* w, int w_dtype, void* out, int out_dtype, int n,
                               int H, int K, int J, int transposed, const float* gate, int ldg, int gate_col0,
                               hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && K > 0 && J > 0 && ldx >= H * K, "heads_matmul: bad sizes n=%d H=%d K=%d J=%d ld=%d", n, H, K, J, ldx);
    const size_t lds = (size_t)HM_TOKENS * K * sizeof(float);
    FL_CHECK(lds <= 64 * 1024, "heads_matmul: %d values per head are more than a block keeps", K);
    FL_CHECK(!gate || ldg >= gate_col0 + H, "heads_matmul: gate columns %d..%d of rows %d wide", gate_col0, gate_col0 + H, ldg);
    if (n == 0) return 0;
    dim3 grid(ceil_div(n, HM_TOKENS), H);
#define FL_HM(TW, TO) heads_matmul_kernel<TW, TO><<<grid, 256, lds, stream>>>(x, ldx, (const TW*)w, (TO*)out, n, H, K, J, transposed, gate, ldg, gate_col0)
    if (w_dtype == FL_F32 && out_dtype == FL_F32) FL_HM(float, float);
    else if (w_dtype == FL_BF16 && out_dtype == FL_F32) FL_HM(bf16_t, float);
    else if (w_dtype == FL_BF16 && out_dtype == FL_BF16) FL_HM(bf16_t, bf16_t);
    else FL_CHECK(false, "heads_matmul: unsupported dtypes w=%d out=%d", w_dtype, out_dtype);
#undef FL_HM
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_heads_matmul)

// ------------------------------------------------------------------ attention over the latent rows
// One block per (token, group of heads); a wave takes LA_HPW heads one after the other.  Keys come in
// chunks of 64: a lane scores one key against the head's folded query (kept in LDS), the wave takes
// maximum and sum, then lanes own the latent's dims and add the chunk's weighted rows.  The query at
// position p sees keys 0..p of its own request (window > 0: the newest `window` of them), all read
// from the pages (this step's rows were stored before).  Rows beyond p are never loaded, so whatever
// an unused or reused page holds cannot reach a sum.
#define LA_WAVES 4
#define LA_MAX_DIMS 16        // latent dims per lane: R <= 64 * LA_MAX_DIMS
template <typename T, int VPL>
__global__ __launch_bounds__(64 * LA_WAVES) void latent_attention_kernel(
    const float* __restrict__ qa, float* __restrict__ z, const T* __restrict__ pool, const int* __restrict__ positions,
    const int* __restrict__ tok_seq, const int* __restrict__ block_table, int max_blocks, int H, int R, int page_size,
    int n_pages, float scale, int window, int heads_per_block) {
    extern __shared__ float lds[];                    // [heads_per_block][R] folded queries, then [LA_WAVES][64] weights
    const int token = blockIdx.x;
    const int h0 = blockIdx.y * heads_per_block;
    const int nh = min(heads_per_block, H - h0);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float* qs = lds;
    volatile float* ps = lds + (size_t)heads_per_block * R + wave * 64;   // written and read by this wave alone
    for (int e = threadIdx.x; e < nh * R; e += 64 * LA_WAVES) qs[e] = qa[((size_t)token * H + h0) * R + e] * scale;
    __syncthreads();
    const int p = positions[token];
    const int* table = block_table + (size_t)tok_seq[token] * max_blocks;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    for (int hh = wave; hh < nh; hh += LA_WAVES) {
        const float* qh = qs + (size_t)hh * R;
        float acc[VPL];
#pragma unroll
        for (int u = 0; u < VPL; ++u) acc[u] = 0.f;
        float m = -INFINITY, l = 0.f;
        for (int t0 = lo; t0 <= p; t0 += 64) {
            const int t = t0 + lane;
            float s = -INFINITY;
            if (t <= p) {
                const int page = table[t / page_size];
                const T* row = pool + ((size_t)page * 2 * page_size + t % page_size) * R;
                float a = 0.f;
                if (page >= 0 && page < n_pages)
                    for (int d = 0; d < R; ++d) a = fmaf(qh[d], to_f32(row[d]), a);
                s = a;
            }
            const float m_new = fmaxf(m, wave_max(s));
            const float corr = expf(m - m_new);       // 0 in the first chunk
            const float e = t <= p ? expf(s - m_new) : 0.f;
            l = l * corr + wave_sum(e);
            m = m_new;
            ps[lane] = e;
            __builtin_amdgcn_wave_barrier();
            const int cnt = min(64, p - t0 + 1);
#pragma unroll
            for (int u = 0; u < VPL; ++u) acc[u] *= corr;
            for (int j = 0; j < cnt; ++j) {
                const int tj = t0 + j;
                const int page = table[tj / page_size];
                if (page < 0 || page >= n_pages) continue;          // (rows that pad a batch of fixed shape have no pages)
                const T* row = pool + ((size_t)page * 2 * page_size + tj % page_size) * R;
                const float w = ps[j];
#pragma unroll
                for (int u = 0; u < VPL; ++u) {
                    const int d = lane + 64 * u;
                    if (d < R) acc[u] = fmaf(w, to_f32(row[d]), acc[u]);
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        float* zr = z + ((size_t)token * H + h0 + hh) * R;
#pragma unroll
        for (int u = 0; u < VPL; ++u) {
            const int d = lane + 64 * u;
            if (d < R) zr[d] = acc[u] * inv;
        }
    }
}

extern "C" int fl_latent_max_width(void) { return 64 * LA_MAX_DIMS; }

extern "C" int fl_latent_attention(const float* qa, float* z, const void* pool, int dtype, const int* positions,
                                   const int* tok_seq, const int* block_table, int max_blocks, int n, int H, int R,
                                   int page_size, int n_pages, float scale, int window, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && R > 0 && page_size > 0 && n_pages > 0 && max_blocks > 0, "latent_attention: bad sizes");
    FL_CHECK(R <= 64 * LA_MAX_DIMS, "latent_attention: a latent of %d values, at most %d", R, 64 * LA_MAX_DIMS);
    FL_CHECK(window >= 0, "latent_attention: negative window");
    if (n == 0) return 0;
    // as many heads per block as keep the folded queries within 32 KB; a wave walks its heads in turn
    int hpb = (int)((32 * 1024) / ((size_t)R * sizeof(float)));
    hpb = hpb < 1 ? 1 : (hpb > H ? H : hpb);
    if (hpb > 2 * LA_WAVES) hpb = 2 * LA_WAVES;
    const size_t lds = ((size_t)hpb * R + 64 * LA_WAVES) * sizeof(float);
    dim3 grid(n, ceil_div(H, hpb));
    const int vpl = ceil_div(R, 64);
#define FL_LA(TT, V)                                                                                                  \
    latent_attention_kernel<TT, V><<<grid, 64 * LA_WAVES, lds, stream>>>(qa, z, (const TT*)pool, positions, tok_seq, \
                                                                         block_table, max_blocks, H, R, page_size,   \
                                                                         n_pages, scale, window, hpb)
#define FL_LA_V(TT)                                  \
    do {                                             \
        if (vpl <= 1) FL_LA(TT, 1);                  \
        else if (vpl <= 2) FL_LA(TT, 2);             \
        else if (vpl <= 4) FL_LA(TT, 4);             \
        else if (vpl <= 8) FL_LA(TT, 8);             \
        else FL_LA(TT, LA_MAX_DIMS);                 \
    } while (0)
    if (dtype == FL_F32) FL_LA_V(float);
    else if (dtype == FL_BF16) FL_LA_V(bf16_t);
    else FL_CHECK(false, "latent_attention: unknown dtype %d", dtype);
#undef FL_LA_V
#undef FL_LA
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_latent_attention)
