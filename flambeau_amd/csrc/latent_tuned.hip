// Attention over cached latent rows on the matrix cores (bfloat16 pools), and the small products per
// head around it.
//
// A wave takes one token and up to 16 of its heads; every head of a token sees the same rows, so a
// loaded row serves all 16.  Everything is computed transposed, as in the other attention kernels of
// this library: S^T[key][head] = C[key][:] . Qa[head][:] (A = rows of the page, B = the folded queries,
// held in registers for the whole walk) and Z^T[dim][head] += C^T[dim][key] P^T[key][head] (A = the
// page's transposed copy, B = the weights, which are the lanes' own score accumulators: the rows of
// the score tiles are dealt out so that a lane's eight values of two tiles are eight keys in a row).
// A head is a lane column, so maxima, sums and rescaling need no broadcast.  Waves share nothing:
// rows of different requests may lie in one block.  Keys beyond the query's position are given weight
// zero and their values are set to zero before they are multiplied, so what an unused or reused page
// holds (a NaN too) never reaches a sum.
#include "common.h"
#include "api.h"
#include "recordable.h"

#define LT_WAVES 4
#define LT_CHUNK 64

__device__ __forceinline__ bf16x8 zero_keys_beyond(bf16x8 v, int first_key, int last_visible) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
        if (first_key + e > last_visible) v[e] = (bf16_t)0.f;
    return v;
}

// qa: bfloat16 [n][H][R]; z: float [n][H][R]; pool: [n_pages][2][page_size * R]; R = 32 * ns, ns <= NS.
// n_split > 1: the keys of every token are dealt out to that many waves, which leave their sums in
// part_o [n * groups * n_split * 16][R] and (maximum, sum of weights) in part_ml [...][2]; a second kernel adds them.
template <int NS>
__global__ __launch_bounds__(64 * LT_WAVES) void latent_attention_mfma_kernel(
    const bf16_t* __restrict__ qa, float* __restrict__ z, const bf16_t* __restrict__ pool,
    const int* __restrict__ positions, const int* __restrict__ tok_seq, const int* __restrict__ block_table,
    int max_blocks, int n, int H, int R, int page_size, int n_pages, float scale, int window, int groups_per_token,
    int n_split, float* __restrict__ part_o, float* __restrict__ part_ml) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int unit = blockIdx.x * LT_WAVES + wave;                 // (token, group of 16 heads, part of the keys)
    if (unit >= n * groups_per_token * n_split) return;
    const int split = unit % n_split, tg = unit / n_split;
    const int token = tg / groups_per_token, h0 = (tg - token * groups_per_token) * 16;
    const int col = lane & 15, g = lane >> 4;                      // col: head (B columns) or row of an A tile
    const int ns = R >> 5;
    const int p = positions[token];
    const int* table = block_table + (size_t)tok_seq[token] * max_blocks;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const size_t page_stride = (size_t)2 * page_size * R;
    const bool head_live = h0 + col < H;

    // the folded queries of this lane's head, scaled: B operand of every score product
    bf16x8 qreg[NS];
    {
        const bf16_t* qr = qa + ((size_t)token * H + h0 + (head_live ? col : 0)) * R;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            if (s < ns && head_live) {
                const bf16x8 v = *(const bf16x8*)(qr + 32 * s + 8 * g);
#pragma unroll
                for (int e = 0; e < 8; ++e) qreg[s][e] = (bf16_t)((float)v[e] * scale);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) qreg[s][e] = (bf16_t)0.f;
            }
        }
    }
    f32x4 o[2 * NS];                                               // Z^T tiles: dims 16 t + 4 g + r of head `col`
#pragma unroll
    for (int t = 0; t < 2 * NS; ++t) o[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    int first = lo & ~(LT_CHUNK - 1);                              // chunks are aligned, so a tile of 16 keys lies in one page
    int last = p;
    if (n_split > 1) {
        // this part's chunks: the token's chunks dealt out in equal runs (a short context leaves late parts empty)
        const int chunks = (p - first) / LT_CHUNK + 1, per = (chunks + n_split - 1) / n_split;
        last = min(p, first + (split + 1) * per * LT_CHUNK - 1);
        first += split * per * LT_CHUNK;
    }
    for (int t0 = first; t0 <= last; t0 += LT_CHUNK) {
        // ---- scores of 64 keys: four tiles of 16; tile 2 q + b, row i <-> key t0 + 32 q + 8 (i / 4) + 4 b + i % 4
        f32x4 sacc[4];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            sacc[a] = (f32x4){0.f, 0.f, 0.f, 0.f};
            const int key = t0 + 32 * (a >> 1) + 8 * (col >> 2) + 4 * (a & 1) + (col & 3);
            const int kc = min(key, p);                            // a key beyond p: any loadable row, masked below
            int page = table[kc / page_size];
            page = min(max(page, 0), n_pages - 1);
            const bf16_t* row = pool + (size_t)page * page_stride + (size_t)(kc % page_size) * R + 8 * g;
#pragma unroll
            for (int s = 0; s < NS; ++s)
                if (s < ns) sacc[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8*)(row + 32 * s), qreg[s], sacc[a], 0, 0, 0);
        }
        // lane (head col, g): sacc[2 q + b][e] is key t0 + 32 q + 8 g + 4 b + e
        float cmax = -INFINITY;
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int key = t0 + 32 * (a >> 1) + 8 * g + 4 * (a & 1) + e;
                if (key > p || key < lo) sacc[a][e] = -INFINITY;
                cmax = fmaxf(cmax, sacc[a][e]);
            }
        cmax = fmaxf(cmax, __shfl_xor(cmax, 16, FL_WAVE));
        cmax = fmaxf(cmax, __shfl_xor(cmax, 32, FL_WAVE));
        const float m_new = fmaxf(m, cmax);                        // finite: every chunk holds a visible key
        const float corr = expf(m - m_new);
        m = m_new;
        bf16x8 pb[2];
        float lsum = 0.f;
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bf16_t w = (bf16_t)expf(sacc[a][e] - m_new);
                pb[a >> 1][4 * (a & 1) + e] = w;
                lsum += (float)w;                                  // the sum of the weights as they are multiplied
            }
        lsum += __shfl_xor(lsum, 16, FL_WAVE);
        lsum += __shfl_xor(lsum, 32, FL_WAVE);
        l = l * corr + lsum;
        // ---- weighted sum: Z^T[dim][head] += C^T[dim][keys] P^T[keys][head], 32 keys a step
        const bool edge = t0 + LT_CHUNK - 1 > p || t0 < lo;
        const bf16_t* cols[2];
        int key0[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            key0[q] = t0 + 32 * q + 8 * g;
            const int kc = min(key0[q], p);
            int page = table[kc / page_size];
            page = min(max(page, 0), n_pages - 1);
            cols[q] = pool + (size_t)page * page_stride + (size_t)page_size * R + (key0[q] % page_size);
        }
#pragma unroll
        for (int t = 0; t < 2 * NS; ++t) {
            if (t < 2 * ns) {
                o[t] *= corr;
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    bf16x8 v = *(const bf16x8*)(cols[q] + (size_t)(16 * t + col) * page_size);
                    if (edge) {
                        v = zero_keys_beyond(v, key0[q], p);
                        if (key0[q] < lo) {
#pragma unroll
                            for (int e = 0; e < 8; ++e)
                                if (key0[q] + e < lo) v[e] = (bf16_t)0.f;
                        }
                    }
                    o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, pb[q], o[t], 0, 0, 0);
                }
            }
        }
    }
    if (n_split > 1) {
        // unnormalised sums relative to this part's own maximum; fl_latent_attention_mfma's second kernel adds the parts
        float* po = part_o + ((size_t)unit * 16 + col) * R;
#pragma unroll
        for (int t = 0; t < 2 * NS; ++t)
            if (t < 2 * ns) *(f32x4*)(po + 16 * t + 4 * g) = o[t];
        if (g == 0) {
            part_ml[((size_t)unit * 16 + col) * 2] = m;
            part_ml[((size_t)unit * 16 + col) * 2 + 1] = l;
        }
        return;
    }
    if (!head_live) return;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    float* zr = z + ((size_t)token * H + h0 + col) * R;
#pragma unroll
    for (int t = 0; t < 2 * NS; ++t)
        if (t < 2 * ns) *(f32x4*)(zr + 16 * t + 4 * g) = o[t] * inv;
}

// z[token][head][:] = sum_s o_s exp(m_s - M) / sum_s l_s exp(m_s - M), M = max_s m_s, over the parts of the keys
// (rising s; an empty part left zeros and has weight 0).  A block takes 256 dims of one (token, head): its
// first wave makes the parts' weights, then every thread adds its dim's parts, all loads independent.
__global__ __launch_bounds__(256) void latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                           float* __restrict__ z, int H, int R, int groups, int n_split) {
    __shared__ float ws[64];
    __shared__ float inv_l;
    const int unit = blockIdx.x, d = blockIdx.y * 256 + threadIdx.x;
    const int token = unit / H, h = unit - token * H;
    const size_t base = ((size_t)(token * groups + (h >> 4)) * n_split) * 16 + (h & 15);        // part 0; parts are 16 rows apart
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        const float ms = lane < n_split ? part_ml[(base + (size_t)lane * 16) * 2] : -INFINITY;
        const float ls = lane < n_split ? part_ml[(base + (size_t)lane * 16) * 2 + 1] : 0.f;
        const float M = wave_max(ms);
        const float w = ms > -INFINITY ? expf(ms - M) : 0.f;
        const float L = wave_sum(ls * w);
        ws[lane] = w;
        if (lane == 0) inv_l = L > 0.f ? 1.0f / L : 0.f;
    }
    __syncthreads();
    if (d >= R) return;
    float acc = 0.f;
#pragma unroll 8
    for (int s = 0; s < n_split; ++s) acc = fmaf(part_o[(base + (size_t)s * 16) * R + d], ws[s], acc);
    z[(size_t)unit * R + d] = acc * inv_l;
}

// Whether the kernel takes a pool's shape: rows of a multiple of 32 values up to 512, pages of a multiple of 16 rows.
extern "C" int fl_latent_attention_mfma_takes(int R, int page_size) {
    return R > 0 && R % 32 == 0 && R <= 512 && page_size > 0 && page_size % 16 == 0;
}

extern "C" int fl_latent_attention_mfma(const void* qa, float* z, const void* pool, const int* positions,
                                        const int* tok_seq, const int* block_table, int max_blocks, int n, int H, int R,
                                        int page_size, int n_pages, float scale, int window, int n_split, float* part_o,
                                        float* part_ml, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && n_pages > 0 && max_blocks > 0, "latent_attention_mfma: bad sizes");
    FL_CHECK(n_split >= 1 && n_split <= 64 && (n_split == 1 || (part_o && part_ml)), "latent_attention_mfma: %d parts of the keys (at most 64) need a workspace", n_split);
    FL_CHECK(fl_latent_attention_mfma_takes(R, page_size), "latent_attention_mfma: rows of %d values in pages of %d are not taken", R, page_size);
    FL_CHECK((uintptr_t)qa % 16 == 0 && (uintptr_t)pool % 16 == 0 && (uintptr_t)z % 16 == 0, "latent_attention_mfma: operands must be 16-byte aligned");
    FL_CHECK(window >= 0, "latent_attention_mfma: negative window");
    if (n == 0) return 0;
    const int groups = ceil_div(H, 16);
    const long units = (long)n * groups * n_split;
    FL_CHECK(units < (1L << 30), "latent_attention_mfma: too many rows");
    const int blocks = (int)((units + LT_WAVES - 1) / LT_WAVES);
    const int ns = R / 32;
#define FL_LT(NS)                                                                                                       \
    latent_attention_mfma_kernel<NS><<<blocks, 64 * LT_WAVES, 0, stream>>>((const bf16_t*)qa, z, (const bf16_t*)pool,  \
                                                                           positions, tok_seq, block_table, max_blocks, \
                                                                           n, H, R, page_size, n_pages, scale, window, groups, \
                                                                           n_split, part_o, part_ml)
    if (ns <= 2) FL_LT(2);
    else if (ns <= 4) FL_LT(4);
    else if (ns <= 8) FL_LT(8);
    else FL_LT(16);
#undef FL_LT
    FL_LAUNCH_CHECK();
    if (n_split > 1) {
        dim3 mgrid(n * H, ceil_div(R, 256));
        latent_merge_kernel<<<mgrid, 256, 0, stream>>>(part_o, part_ml, z, H, R, groups, n_split);
        FL_LAUNCH_CHECK();
    }
    return 0;
}
FL_RECORDABLE(fl_latent_attention_mfma)


// The same walk for prompt portions, four waves to a block that share their keys: a tile (from the host:
// first token, tokens, first group of 16 heads, groups; tokens x groups <= 4, all of one request) loads
// every chunk of 64 rows once into LDS, as it is and transposed, and its waves read their operands from
// there.  Without this every wave fetches every row itself and the kernel runs at the rate of the
// caches, 16 flops a byte.  Rows are padded by 16 bytes so that the 16 rows (or dims) of an operand
// start in different banks.  A wave whose token lies before a chunk sits the chunk out.
template <int NS>
__global__ __launch_bounds__(64 * LT_WAVES) void latent_attention_shared_kernel(
    const bf16_t* __restrict__ qa, float* __restrict__ z, const bf16_t* __restrict__ pool,
    const int* __restrict__ positions, const int* __restrict__ tok_seq, const int* __restrict__ block_table,
    int max_blocks, int H, int R, int page_size, int n_pages, float scale, int window, const int* __restrict__ tiles) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lt_smem[];
    const int stride_r = R + 8, stride_c = LT_CHUNK + 8;
    bf16_t* ks = (bf16_t*)lt_smem;                                  // [64 keys][R + 8]
    bf16_t* vs = ks + (size_t)LT_CHUNK * stride_r;                  // [R dims][64 + 8]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int t_first = tiles[4 * blockIdx.x], n_tok = tiles[4 * blockIdx.x + 1];
    const int g_first = tiles[4 * blockIdx.x + 2], n_grp = tiles[4 * blockIdx.x + 3];
    const int tw = wave / n_grp, gw = wave - tw * n_grp;
    const bool active = tw < n_tok;
    const int token = t_first + (active ? tw : 0), h0 = (g_first + gw) * 16;
    const int col = lane & 15, g = lane >> 4;
    const int ns = R >> 5;
    const int p = active ? positions[token] : -1;
    const int p_max = positions[t_first + n_tok - 1];              // a request's tokens of a step stand in rising order
    const int* table = block_table + (size_t)tok_seq[t_first] * max_blocks;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int lo_min = window > 0 ? max(0, positions[t_first] - window + 1) : 0;
    const size_t page_stride = (size_t)2 * page_size * R;
    const bool head_live = active && h0 + col < H;
    bf16x8 qreg[NS];
    {
        const bf16_t* qr = qa + ((size_t)token * H + (head_live ? h0 + col : 0)) * R;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            if (s < ns && head_live) {
                const bf16x8 v = *(const bf16x8*)(qr + 32 * s + 8 * g);
#pragma unroll
                for (int e = 0; e < 8; ++e) qreg[s][e] = (bf16_t)((float)v[e] * scale);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) qreg[s][e] = (bf16_t)0.f;
            }
        }
    }
    f32x4 o[2 * NS];
#pragma unroll
    for (int t = 0; t < 2 * NS; ++t) o[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const int pieces_r = R >> 3;                                    // 16-byte pieces of a row
    for (int t0 = lo_min & ~(LT_CHUNK - 1); t0 <= p_max; t0 += LT_CHUNK) {
        // ---- the chunk into LDS: rows as they are, and the pages' transposed copies dim by dim.  The pages of the
        // chunk's four runs of 16 keys are looked up first (pages hold a multiple of 16 rows), so that all copies
        // of a thread are in flight at once; a run beyond the newest token takes that token's page and is masked.
        const bf16_t* run_rows[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int kc = min(t0 + 16 * j, p_max & ~15);
            int page = table[kc / page_size];
            page = min(max(page, 0), n_pages - 1);
            run_rows[j] = pool + (size_t)page * page_stride + (size_t)(kc % page_size) * R;       // row kc of the page; its transposed copy lies page_size * R further, at column kc % page_size
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {                             // wave w copies rows w, w + 4, ...: row 4 i + w lies in run i / 4
            const int row = 4 * i + wave;
            const bf16_t* src = run_rows[i >> 2] + (size_t)(row & 15) * R;
            for (int c = lane; c < pieces_r; c += 64) *(bf16x8*)(ks + (size_t)row * stride_r + 8 * c) = *(const bf16x8*)(src + 8 * c);
        }
        {
            const int k8 = threadIdx.x & 7;                        // this thread's 8 keys of every dim: run k8 / 2, its first or second half
            const int kc = min(t0 + 16 * (k8 >> 1), p_max & ~15);
            const bf16_t* src = run_rows[0];
#pragma unroll
            for (int j = 1; j < 4; ++j) src = (k8 >> 1) == j ? run_rows[j] : src;
            src += (size_t)(page_size - (kc % page_size)) * R + (kc % page_size) + 8 * (k8 & 1);    // from row kc of the page to column kc (+ 8) of its transposed copy
            for (int dim = threadIdx.x >> 3; dim < R; dim += 32)
                *(bf16x8*)(vs + (size_t)dim * stride_c + 8 * k8) = *(const bf16x8*)(src + (size_t)dim * page_size);
        }
        __syncthreads();
        if (active && t0 <= p && t0 + LT_CHUNK - 1 >= lo) {
            f32x4 sacc[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                sacc[a] = (f32x4){0.f, 0.f, 0.f, 0.f};
                const bf16_t* row = ks + (size_t)(32 * (a >> 1) + 8 * (col >> 2) + 4 * (a & 1) + (col & 3)) * stride_r + 8 * g;
#pragma unroll
                for (int s = 0; s < NS; ++s)
                    if (s < ns) sacc[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8*)(row + 32 * s), qreg[s], sacc[a], 0, 0, 0);
            }
            float cmax = -INFINITY;
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int key = t0 + 32 * (a >> 1) + 8 * g + 4 * (a & 1) + e;
                    if (key > p || key < lo) sacc[a][e] = -INFINITY;
                    cmax = fmaxf(cmax, sacc[a][e]);
                }
            cmax = fmaxf(cmax, __shfl_xor(cmax, 16, FL_WAVE));
            cmax = fmaxf(cmax, __shfl_xor(cmax, 32, FL_WAVE));
            // The base of the exponents follows the maximum lazily: it moves only when a score exceeds it by more
            // than 8 (weights stay below e^8, exact enough in bfloat16 and float), so that in most chunks nothing
            // is rescaled and the sums can stay where the matrix cores accumulate them.
            const float m_new = (cmax > m + 8.0f) ? cmax : m;      // finite after the first chunk: it holds a key this wave sees
            const bool moved = __any(m_new != m);
            const float corr = expf(m - m_new);
            m = m_new;
            bf16x8 pb[2];
            float lsum = 0.f;
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const bf16_t w = (bf16_t)expf(sacc[a][e] - m_new);
                    pb[a >> 1][4 * (a & 1) + e] = w;
                    lsum += (float)w;
                }
            lsum += __shfl_xor(lsum, 16, FL_WAVE);
            lsum += __shfl_xor(lsum, 32, FL_WAVE);
            l = l * corr + lsum;
            if (moved) {
#pragma unroll
                for (int t = 0; t < 2 * NS; ++t)
                    if (t < 2 * ns) o[t] *= corr;
            }
            const bool edge = t0 + LT_CHUNK - 1 > p || t0 < lo;
#pragma unroll
            for (int t = 0; t < 2 * NS; ++t) {
                if (t < 2 * ns) {
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        const int key0 = t0 + 32 * q + 8 * g;
                        bf16x8 v = *(const bf16x8*)(vs + (size_t)(16 * t + col) * stride_c + 32 * q + 8 * g);
                        if (edge) {
#pragma unroll
                            for (int e = 0; e < 8; ++e)
                                if (key0 + e > p || key0 + e < lo) v[e] = (bf16_t)0.f;
                        }
                        o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, pb[q], o[t], 0, 0, 0);
                    }
                }
            }
        }
        __syncthreads();
    }
    if (!head_live) return;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    float* zr = z + ((size_t)token * H + h0 + col) * R;
#pragma unroll
    for (int t = 0; t < 2 * NS; ++t)
        if (t < 2 * ns) *(f32x4*)(zr + 16 * t + 4 * g) = o[t] * inv;
}

extern "C" long fl_latent_attention_shared_lds(int R) { return (long)LT_CHUNK * (R + 8) * 2 + (long)R * (LT_CHUNK + 8) * 2; }

// tiles [n_tiles][4] = (first token, tokens, first group of 16 heads, groups): tokens x groups <= 4, the tokens of one request
extern "C" int fl_latent_attention_shared(const void* qa, float* z, const void* pool, const int* positions,
                                          const int* tok_seq, const int* block_table, int max_blocks, int H, int R,
                                          int page_size, int n_pages, float scale, int window, const int* tiles, int n_tiles,
                                          hipStream_t stream) {
    FL_CHECK(n_tiles >= 0 && H > 0 && n_pages > 0 && max_blocks > 0, "latent_attention_shared: bad sizes");
    FL_CHECK(fl_latent_attention_mfma_takes(R, page_size), "latent_attention_shared: rows of %d values in pages of %d are not taken", R, page_size);
    FL_CHECK((uintptr_t)qa % 16 == 0 && (uintptr_t)pool % 16 == 0 && (uintptr_t)z % 16 == 0, "latent_attention_shared: operands must be 16-byte aligned");
    
    FL_CHECK(window >= 0, "latent_attention_shared: negative window");
    if (n_tiles == 0) return 0;
    const size_t lds = (size_t)fl_latent_attention_shared_lds(R);
    const int ns = R / 32;
#define FL_LTS(NS)                                                                                                     \
    do {                                                                                                               \
        static bool sized = false;                                                                                     \
        if (!sized) {                                                                                                  \
            hipError_t e_ = hipFuncSetAttribute((const void*)latent_attention_shared_kernel<NS>,                      \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);              \
            FL_CHECK(e_ == hipSuccess, "latent_attention_shared: %s", hipGetErrorString(e_));                          \
            sized = true;                                                                                              \
        }                                                                                                              \
        latent_attention_shared_kernel<NS><<<n_tiles, 64 * LT_WAVES, lds, stream>>>(                                  \
            (const bf16_t*)qa, z, (const bf16_t*)pool, positions, tok_seq, block_table, max_blocks, H, R, page_size,   \
            n_pages, scale, window, tiles);                                                                            \
    } while (0)
    if (ns <= 2) FL_LTS(2);
    else if (ns <= 4) FL_LTS(4);
    else if (ns <= 8) FL_LTS(8);
    else FL_LTS(16);
#undef FL_LTS
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_latent_attention_shared)


// The same walk for steps of few rows (decoding), where a wave that holds all of a latent's dims has no register
// left for reads in flight and waits for every operand: the four waves of a block take one (token, 16 heads, part
// of the keys) together and deal the latent's steps of 32 dims out among them (wave w: steps w, w + 4, ...).
// Each forms its share of the scores, the shares are added through LDS in a fixed order (every wave gets the
// same sums, hence the same maxima and weights), and each adds the weighted rows of its own dims.  A wave then
// holds a quarter of the accumulators and queries, and the reads of a chunk are all in flight at once.
template <int NSW>
__global__ __launch_bounds__(64 * LT_WAVES) void latent_attention_dealt_kernel(
    const bf16_t* __restrict__ qa, float* __restrict__ z, const bf16_t* __restrict__ pool,
    const int* __restrict__ positions, const int* __restrict__ tok_seq, const int* __restrict__ block_table,
    int max_blocks, int n, int H, int R, int page_size, int n_pages, float scale, int window, int groups_per_token,
    int n_split, float* __restrict__ part_o, float* __restrict__ part_ml) {
    __shared__ f32x4 sx[LT_WAVES][4][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int unit = blockIdx.x;                                   // (token, group of 16 heads, part of the keys)
    const int split = unit % n_split, tg = unit / n_split;
    const int token = tg / groups_per_token, h0 = (tg - token * groups_per_token) * 16;
    const int col = lane & 15, g = lane >> 4;
    const int ns = R >> 5;
    const int p = positions[token];
    const int* table = block_table + (size_t)tok_seq[token] * max_blocks;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const size_t page_stride = (size_t)2 * page_size * R;
    const bool head_live = h0 + col < H;
    bf16x8 qreg[NSW];
    {
        const bf16_t* qr = qa + ((size_t)token * H + h0 + (head_live ? col : 0)) * R;
#pragma unroll
        for (int i = 0; i < NSW; ++i) {
            const int s = wave + LT_WAVES * i;
            if (s < ns && head_live) {
                const bf16x8 v = *(const bf16x8*)(qr + 32 * s + 8 * g);
#pragma unroll
                for (int e = 0; e < 8; ++e) qreg[i][e] = (bf16_t)((float)v[e] * scale);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) qreg[i][e] = (bf16_t)0.f;
            }
        }
    }
    f32x4 o[2 * NSW];                                              // dims 32 s + 16 u + 4 g + r of the wave's steps s, u = 0, 1
#pragma unroll
    for (int t = 0; t < 2 * NSW; ++t) o[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    int first = lo & ~(LT_CHUNK - 1), last = p;
    if (n_split > 1) {
        const int chunks = (p - first) / LT_CHUNK + 1, per = (chunks + n_split - 1) / n_split;
        last = min(p, first + (split + 1) * per * LT_CHUNK - 1);
        first += split * per * LT_CHUNK;
    }
    for (int t0 = first; t0 <= last; t0 += LT_CHUNK) {
        f32x4 sacc[4];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            sacc[a] = (f32x4){0.f, 0.f, 0.f, 0.f};
            const int key = t0 + 32 * (a >> 1) + 8 * (col >> 2) + 4 * (a & 1) + (col & 3);
            const int kc = min(key, p);
            int page = table[kc / page_size];
            page = min(max(page, 0), n_pages - 1);
            const bf16_t* row = pool + (size_t)page * page_stride + (size_t)(kc % page_size) * R + 8 * g;
#pragma unroll
            for (int i = 0; i < NSW; ++i) {
                const int s = wave + LT_WAVES * i;
                if (s < ns) sacc[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8*)(row + 32 * s), qreg[i], sacc[a], 0, 0, 0);
            }
            sx[wave][a][lane] = sacc[a];
        }
        __syncthreads();
        float cmax = -INFINITY;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            sacc[a] = (sx[0][a][lane] + sx[1][a][lane]) + (sx[2][a][lane] + sx[3][a][lane]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int key = t0 + 32 * (a >> 1) + 8 * g + 4 * (a & 1) + e;
                if (key > p || key < lo) sacc[a][e] = -INFINITY;
                cmax = fmaxf(cmax, sacc[a][e]);
            }
        }
        __syncthreads();                                           // (the next chunk's shares overwrite sx)
        cmax = fmaxf(cmax, __shfl_xor(cmax, 16, FL_WAVE));
        cmax = fmaxf(cmax, __shfl_xor(cmax, 32, FL_WAVE));
        const float m_new = fmaxf(m, cmax);
        const float corr = expf(m - m_new);
        m = m_new;
        bf16x8 pb[2];
        float lsum = 0.f;
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bf16_t w = (bf16_t)expf(sacc[a][e] - m_new);
                pb[a >> 1][4 * (a & 1) + e] = w;
                lsum += (float)w;
            }
        lsum += __shfl_xor(lsum, 16, FL_WAVE);
        lsum += __shfl_xor(lsum, 32, FL_WAVE);
        l = l * corr + lsum;
        const bool edge = t0 + LT_CHUNK - 1 > p || t0 < lo;
        const bf16_t* cols[2];
        int key0[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            key0[q] = t0 + 32 * q + 8 * g;
            const int kc = min(key0[q], p);
            int page = table[kc / page_size];
            page = min(max(page, 0), n_pages - 1);
            cols[q] = pool + (size_t)page * page_stride + (size_t)page_size * R + (key0[q] % page_size);
        }
#pragma unroll
        for (int t = 0; t < 2 * NSW; ++t) {
            const int s = wave + LT_WAVES * (t >> 1);
            if (s < ns) {
                const int dim = 32 * s + 16 * (t & 1) + col;
                o[t] *= corr;
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    bf16x8 v = *(const bf16x8*)(cols[q] + (size_t)dim * page_size);
                    if (edge) {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (key0[q] + e > p || key0[q] + e < lo) v[e] = (bf16_t)0.f;
                    }
                    o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, pb[q], o[t], 0, 0, 0);
                }
            }
        }
    }
    if (n_split > 1) {
        float* po = part_o + ((size_t)unit * 16 + col) * R;
#pragma unroll
        for (int t = 0; t < 2 * NSW; ++t) {
            const int s = wave + LT_WAVES * (t >> 1);
            if (s < ns) *(f32x4*)(po + 32 * s + 16 * (t & 1) + 4 * g) = o[t];
        }
        if (wave == 0 && g == 0) {
            part_ml[((size_t)unit * 16 + col) * 2] = m;
            part_ml[((size_t)unit * 16 + col) * 2 + 1] = l;
        }
        return;
    }
    if (!head_live) return;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    float* zr = z + ((size_t)token * H + h0 + col) * R;
#pragma unroll
    for (int t = 0; t < 2 * NSW; ++t) {
        const int s = wave + LT_WAVES * (t >> 1);
        if (s < ns) *(f32x4*)(zr + 32 * s + 16 * (t & 1) + 4 * g) = o[t] * inv;
    }
}

// fl_latent_attention_mfma with a block of four waves per (token, 16 heads, part of the keys): for steps of few rows
extern "C" int fl_latent_attention_dealt(const void* qa, float* z, const void* pool, const int* positions,
                                         const int* tok_seq, const int* block_table, int max_blocks, int n, int H, int R,
                                         int page_size, int n_pages, float scale, int window, int n_split, float* part_o,
                                         float* part_ml, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && n_pages > 0 && max_blocks > 0, "latent_attention_dealt: bad sizes");
    FL_CHECK(n_split >= 1 && n_split <= 64 && (n_split == 1 || (part_o && part_ml)), "latent_attention_dealt: %d parts of the keys (at most 64) need a workspace", n_split);
    FL_CHECK(fl_latent_attention_mfma_takes(R, page_size), "latent_attention_dealt: rows of %d values in pages of %d are not taken", R, page_size);
    FL_CHECK((uintptr_t)qa % 16 == 0 && (uintptr_t)pool % 16 == 0 && (uintptr_t)z % 16 == 0, "latent_attention_dealt: operands must be 16-byte aligned");
    FL_CHECK(window >= 0, "latent_attention_dealt: negative window");
    if (n == 0) return 0;
    const int groups = ceil_div(H, 16);
    const long units = (long)n * groups * n_split;
    FL_CHECK(units < (1L << 30), "latent_attention_dealt: too many rows");
    const int nsw = ceil_div(R / 32, LT_WAVES);
#define FL_LTD(NSW)                                                                                                       \
    latent_attention_dealt_kernel<NSW><<<(unsigned)units, 64 * LT_WAVES, 0, stream>>>((const bf16_t*)qa, z, (const bf16_t*)pool, \
                                                                                      positions, tok_seq, block_table, max_blocks, \
                                                                                      n, H, R, page_size, n_pages, scale, window,  \
                                                                                      groups, n_split, part_o, part_ml)
    if (nsw <= 1) FL_LTD(1);
    else if (nsw <= 2) FL_LTD(2);
    else FL_LTD(4);
#undef FL_LTD
    FL_LAUNCH_CHECK();
    if (n_split > 1) {
        dim3 mgrid(n * H, ceil_div(R, 256));
        latent_merge_kernel<<<mgrid, 256, 0, stream>>>(part_o, part_ml, z, H, R, groups, n_split);
        FL_LAUNCH_CHECK();
    }
    return 0;
}
FL_RECORDABLE(fl_latent_attention_dealt)

// ------------------------------------------------------------------ one product per head on the matrix cores
// out[t][h][j] = sum_k x[t][h][k] w[h][j][k]   (x float or bfloat16 rows ldx apart, w bfloat16 [H][J][K], K a multiple
// of 32, J of 16), optionally times sigmoid(gate[t][gate_col0 + h]).  A wave takes 16 tokens of one head: its x is
// the B operand, held in registers for all of K; the weights are the A operand, so a lane ends with four
// consecutive outputs of one token.
template <typename TX, typename TOut, int NS>
__global__ __launch_bounds__(64 * LT_WAVES) void heads_matmul_mfma_kernel(
    const TX* __restrict__ x, int ldx, const bf16_t* __restrict__ w, TOut* __restrict__ out, int n, int H, int K, int J,
    const float* __restrict__ gate, int ldg, int gate_col0, int j_parts) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // a wave takes 16 tokens and every j_parts-th tile of 16 output columns (few tokens: many parts, so that
    // a decode step still fills the chip)
    const int unit = blockIdx.x * LT_WAVES + wave;
    const int t0 = (unit / j_parts) * 16, j_first = unit % j_parts, h = blockIdx.y;
    if (t0 >= n) return;
    const int col = lane & 15, g = lane >> 4;
    const int ns = K >> 5;
    const int token = t0 + col;
    const bool live = token < n;
    bf16x8 xreg[NS];
    {
        const TX* xr = x + (size_t)(live ? token : t0) * ldx + (size_t)h * K + 8 * g;
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) xreg[s][e] = (s < ns && live) ? (bf16_t)to_f32(xr[32 * s + e]) : (bf16_t)0.f;
    }
    const float gv = (gate && live) ? 1.0f / (1.0f + expf(-gate[(size_t)token * ldg + gate_col0 + h])) : 1.0f;
    const bf16_t* wh = w + (size_t)h * J * K;
#pragma unroll 4
    for (int jt = j_first; jt < J / 16; jt += j_parts) {
        f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
        const bf16_t* row = wh + (size_t)(16 * jt + col) * K + 8 * g;
#pragma unroll
        for (int s = 0; s < NS; ++s)
            if (s < ns) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8*)(row + 32 * s), xreg[s], acc, 0, 0, 0);
        if (live) {
            TOut* dst = out + ((size_t)token * H + h) * J + 16 * jt + 4 * g;
#pragma unroll
            for (int r = 0; r < 4; ++r) dst[r] = from_f32<TOut>(acc[r] * gv);
        }
    }
}

extern "C" int fl_heads_matmul_mfma_takes(int K, int J) { return K > 0 && K % 32 == 0 && K <= 512 && J > 0 && J % 16 == 0; }

extern "C" int fl_heads_matmul_mfma(const void* x, int x_dtype, int ldx, const void* w, void* out, int out_dtype, int n,
                                    int H, int K, int J, const float* gate, int ldg, int gate_col0, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && ldx >= H * K, "heads_matmul_mfma: bad sizes");
    FL_CHECK(fl_heads_matmul_mfma_takes(K, J), "heads_matmul_mfma: %d x %d per head is not taken", J, K);
    FL_CHECK((uintptr_t)w % 16 == 0, "heads_matmul_mfma: the weights must be 16-byte aligned");
    FL_CHECK(!gate || ldg >= gate_col0 + H, "heads_matmul_mfma: gate columns beyond rows %d wide", ldg);
    if (n == 0) return 0;
    FL_CHECK(H <= 65535, "heads_matmul_mfma: too many heads");
    // enough waves for four per compute unit, as far as the column tiles go
    const int groups = ceil_div(n, 16);
    int j_parts = (4 * fl_units()) / (groups * H);
    j_parts = j_parts < 1 ? 1 : (j_parts > J / 16 ? J / 16 : j_parts);
    dim3 grid(ceil_div(groups * j_parts, LT_WAVES), H);
    const int ns = K / 32;
#define FL_HMM(TX, TO, NS) heads_matmul_mfma_kernel<TX, TO, NS><<<grid, 64 * LT_WAVES, 0, stream>>>((const TX*)x, ldx, (const bf16_t*)w, (TO*)out, n, H, K, J, gate, ldg, gate_col0, j_parts)
#define FL_HMM_NS(TX, TO)                      \
    do {                                       \
        if (ns <= 2) FL_HMM(TX, TO, 2);        \
        else if (ns <= 4) FL_HMM(TX, TO, 4);   \
        else if (ns <= 8) FL_HMM(TX, TO, 8);   \
        else FL_HMM(TX, TO, 16);               \
    } while (0)
    if (x_dtype == FL_F32 && out_dtype == FL_BF16) FL_HMM_NS(float, bf16_t);
    else if (x_dtype == FL_F32 && out_dtype == FL_F32) FL_HMM_NS(float, float);
    else if (x_dtype == FL_BF16 && out_dtype == FL_BF16) FL_HMM_NS(bf16_t, bf16_t);
    else FL_CHECK(false, "heads_matmul_mfma: unsupported dtypes x=%d out=%d", x_dtype, out_dtype);
#undef FL_HMM_NS
#undef FL_HMM
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_heads_matmul_mfma)
