// Matrix memory with exponential gating (the mLSTM recurrence), token by token.
//
// Per request and head the state is the memory S [D][Dv], the normaliser n [D] and the running
// maximum m of the log gates, all float, kept in the request's slot between steps and zero when the
// slot is claimed (so m starts at 0).  For every token, with log gates i (input) and f (forget):
//     i = cap * tanh((zi + bi) / cap),   f = logsigmoid(cap * tanh((zf + bf) / cap))
//     m' = max(f + m, i);  a = exp(f + m - m');  b = exp(i - m')
//     S <- a S + b k v^T;  n <- a n + b k;  m <- m'
//     o = S^T q / (max(|n . q|, exp(-m)) + 1e-6)
// Two kernels: the gates and their running maximum for all tokens (only the maximum is a chain there), then the
// memory's walk with the factors exp(f + m - m'), exp(i - m'), exp(-m') ready.
// The walk is the recurrence itself, so a prompt cut anywhere leaves the same state and the same o.
#include "common.h"
#include "api.h"
#include "recordable.h"
#include "lanes.h"

#define ML_GROUP 16          // threads that share a column of S; they own the rows d = g, g + 16, ...
#define ML_COLS 16           // columns of S per block
#define ML_MAX_ROWS 32       // rows per thread: D <= ML_GROUP * ML_MAX_ROWS

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// The gates first, for all tokens of the step (fl_mlstm_scan's first kernel): per (request, head) a wave takes 64
// tokens at a time, forms i and f in parallel, walks the running maximum m through them (a max-plus chain,
// which is all that is sequential in the gates) and leaves for every token the three factors the memory's
// walk needs: a = exp(f + m' - m), b = exp(i - m), c = exp(-m) (m' the maximum before the token).  The
// head's m lives in the state behind S (the first float after it) and is read and written here alone.
__global__ __launch_bounds__(64) void mlstm_gates_kernel(const float* __restrict__ proj, int ld, int col_i, int col_f,
                                                         const float* __restrict__ bias_i, const float* __restrict__ bias_f, float cap,
                                                         float* __restrict__ state, size_t rec, size_t m_at,
                                                         const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
                                                         const int* __restrict__ seq_slots, float* __restrict__ factors, int H) {
    const int head = blockIdx.x, s = blockIdx.y, lane = threadIdx.x;
    const int start = seq_q_start[s], len = seq_q_len[s];
    float* mp = state + ((size_t)seq_slots[s] * H + head) * rec + m_at;
    float m = *mp;
    const float bi = bias_i ? bias_i[head] : 0.f, bf = bias_f ? bias_f[head] : 0.f;
    for (int t0 = 0; t0 < len; t0 += 64) {
        const int t = t0 + lane;
        const bool live = t < len;
        const float* row = proj + (size_t)(start + (live ? t : 0)) * ld;
        const float gi = cap * tanhf((row[col_i + head] + bi) / cap);
        const float gf = log_sigmoid(cap * tanhf((row[col_f + head] + bf) / cap));
        float m_before = m, m_mine = m;
        const int cnt = min(64, len - t0);
        for (int u = 0; u < cnt; ++u) {                            // every lane walks the same chain and keeps its own link
            const float mb = m;
            m = fmaxf(__shfl(gf, u, FL_WAVE) + m, __shfl(gi, u, FL_WAVE));
            if (u == lane) { m_before = mb; m_mine = m; }
        }
        if (live) {
            float* f3 = factors + ((size_t)(start + t) * H + head) * 3;
            f3[0] = expf(gf + m_before - m_mine);
            f3[1] = expf(gi - m_mine);
            f3[2] = expf(-m_mine);
        }
    }
    if (lane == 0) *mp = m;
}

// proj: float rows ld wide holding, per token, q [H][D] at col_q, k [H][D] at col_k, v [H][Dv] at col_v;
// factors [n][H][3] = (a, b, c) of mlstm_gates_kernel.
// Block = (columns j0 .. j0 + 15, head, request); thread (g, c) holds S[d][j0 + c] for its rows d.
// Every block walks n for itself and keeps a copy of its own in the state, since blocks of one head start
// and end at different times: state [slots][H][D * Dv + 1 + blocks * D], S first (column by column,
// S[d][j] at j * D + d, so that the threads of a column read neighbours), then m, then per block of
// columns n [D] (fl_mlstm_state_floats gives the record's size).
template <int RPT>
__global__ __launch_bounds__(ML_GROUP * ML_COLS) void mlstm_scan_kernel(
    const float* __restrict__ proj, int ld, int col_q, int col_k, int col_v, const float* __restrict__ factors, float q_scale,
    float* __restrict__ state, const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
    const int* __restrict__ seq_slots, float* __restrict__ out, int H, int D, int Dv, int run) {
    const int g = threadIdx.x & (ML_GROUP - 1), c = threadIdx.x / ML_GROUP;
    const int j = blockIdx.x * ML_COLS + c, head = blockIdx.y, s = blockIdx.z;
    const bool live = j < Dv;
    const int start = seq_q_start[s], len = seq_q_len[s];
    const size_t rec = (size_t)D * Dv + 1 + (size_t)gridDim.x * D;
    float* st = state + ((size_t)seq_slots[s] * H + head) * rec;
    float* mine = st + (size_t)D * Dv + 1 + (size_t)blockIdx.x * D;         // this block's n [D]
    float S[RPT], nn[RPT];
#pragma unroll
    for (int u = 0; u < RPT; ++u) {
        const int d = g + ML_GROUP * u;
        S[u] = (live && d < D) ? st[(size_t)j * D + d] : 0.f;
        nn[u] = d < D ? mine[d] : 0.f;
    }
    // The step's tokens come through LDS a run at a time (q and k of the head, the block's 16 values, the three
    // factors): one trip to memory per run instead of one per token, which is what the walk would wait for.
    extern __shared__ float ml_smem[];
    float* qs = ml_smem;                          // [run][D], scaled
    float* ks = qs + (size_t)run * D;             // [run][D]
    float* vs = ks + (size_t)run * D;             // [run][16]
    float* fs = vs + (size_t)run * ML_COLS;       // [run][3]
    for (int t0 = 0; t0 < len; t0 += run) {
        const int cnt = min(run, len - t0);
        __syncthreads();
        for (int e = threadIdx.x; e < cnt * D; e += ML_GROUP * ML_COLS) {
            const int tt = e / D, d = e - tt * D;
            const float* row = proj + (size_t)(start + t0 + tt) * ld;
            qs[e] = row[col_q + head * D + d] * q_scale;
            ks[e] = row[col_k + head * D + d];
        }
        for (int e = threadIdx.x; e < cnt * ML_COLS; e += ML_GROUP * ML_COLS) {
            const int tt = e / ML_COLS, jj = blockIdx.x * ML_COLS + (e - tt * ML_COLS);
            vs[e] = jj < Dv ? proj[(size_t)(start + t0 + tt) * ld + col_v + head * Dv + jj] : 0.f;
        }
        for (int e = threadIdx.x; e < cnt * 3; e += ML_GROUP * ML_COLS) {
            const int tt = e / 3;
            fs[e] = factors[((size_t)(start + t0 + tt) * H + head) * 3 + (e - tt * 3)];
        }
        __syncthreads();
        for (int tt = 0; tt < cnt; ++tt) {
            const float fa = fs[3 * tt], fb = fs[3 * tt + 1], fc = fs[3 * tt + 2];
            const float bv = fb * vs[tt * ML_COLS + c];
            float num = 0.f, den = 0.f;
#pragma unroll
            for (int u = 0; u < RPT; ++u) {
                const int d = g + ML_GROUP * u;
                const float qv = d < D ? qs[tt * D + d] : 0.f, kv = d < D ? ks[tt * D + d] : 0.f;
                S[u] = fa * S[u] + bv * kv;
                nn[u] = fa * nn[u] + fb * kv;
                num = fmaf(S[u], qv, num);
                den = fmaf(nn[u], qv, den);
            }
            num = row_sum16(num);                                  // the 16 threads of a column are a row of lanes
            den = row_sum16(den);
            if (live && g == 0) out[((size_t)(start + t0 + tt) * H + head) * Dv + j] = num / (fmaxf(fabsf(den), fc) + 1e-6f);
        }
    }
#pragma unroll
    for (int u = 0; u < RPT; ++u) {
        const int d = g + ML_GROUP * u;
        if (live && d < D) st[(size_t)j * D + d] = S[u];
        if (c == 0 && d < D) mine[d] = nn[u];
    }
}

extern "C" int fl_mlstm_max_dim(void) { return ML_GROUP * ML_MAX_ROWS; }
// floats of one head's record in the state
extern "C" long fl_mlstm_state_floats(int D, int Dv) { return (long)D * Dv + 1 + (long)ceil_div(Dv, ML_COLS) * D; }

extern "C" int fl_mlstm_scan(const float* proj, int ld, int col_q, int col_k, int col_v, int col_i, int col_f,
                             const float* bias_i, const float* bias_f, float cap, float q_scale, float* state,
                             const int* seq_q_start, const int* seq_q_len, const int* seq_slots, float* out, float* factors,
                             int n_seqs, int H, int D, int Dv, hipStream_t stream) {
    FL_CHECK(n_seqs >= 0 && H > 0 && D > 0 && Dv > 0, "mlstm_scan: bad sizes");
    FL_CHECK(D <= ML_GROUP * ML_MAX_ROWS, "mlstm_scan: %d key dims per head, at most %d", D, ML_GROUP * ML_MAX_ROWS);
    FL_CHECK(cap > 0.f, "mlstm_scan: the gates' cap must be positive");
    FL_CHECK(ld >= col_q + H * D && ld >= col_k + H * D && ld >= col_v + H * Dv && ld >= col_i + H && ld >= col_f + H,
             "mlstm_scan: columns beyond rows %d wide", ld);
    if (n_seqs == 0) return 0;
    FL_CHECK(n_seqs <= 65535 && H <= 65535, "mlstm_scan: %d requests of %d heads are more than one grid takes", n_seqs, H);
    FL_CHECK(factors, "mlstm_scan: no room for the gates' factors ([tokens][heads][3] floats)");
    dim3 ggrid(H, n_seqs);
    mlstm_gates_kernel<<<ggrid, 64, 0, stream>>>(proj, ld, col_i, col_f, bias_i, bias_f, cap, state, (size_t)fl_mlstm_state_floats(D, Dv),
                                                 (size_t)D * Dv, seq_q_start, seq_q_len, seq_slots, factors, H);
    FL_LAUNCH_CHECK();
    dim3 grid(ceil_div(Dv, ML_COLS), H, n_seqs);
    const int rpt = ceil_div(D, ML_GROUP);
    // tokens per run through LDS: up to 32, as many as 60 KB hold
    int run = (60 * 1024) / ((2 * D + ML_COLS + 3) * (int)sizeof(float));
    run = run > 32 ? 32 : (run < 1 ? 1 : run);
    const size_t lds = (size_t)run * (2 * D + ML_COLS + 3) * sizeof(float);
#define FL_ML(R)                                                                                                      \
    mlstm_scan_kernel<R><<<grid, ML_GROUP * ML_COLS, lds, stream>>>(proj, ld, col_q, col_k, col_v, factors, q_scale, state, \
                                                                    seq_q_start, seq_q_len, seq_slots, out, H, D, Dv, run)
    if (rpt <= 1) FL_ML(1);
    else if (rpt <= 2) FL_ML(2);
    else if (rpt <= 4) FL_ML(4);
    else if (rpt <= 8) FL_ML(8);
    else if (rpt <= 16) FL_ML(16);
    else FL_ML(ML_MAX_ROWS);
#undef FL_ML
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_mlstm_scan)

// ------------------------------------------------------------------ unit norm per head, gain, gate
// out[t][h][:] = o / sqrt(mean(o^2) + eps) * w[h][:] * g(gate[t][gate_col0 + h * Dv + :]),
// o = x[t][h][:] (float); g the sigmoid (gate_kind 1) or silu (2).  One wave per (token, head).
template <typename T>
__global__ __launch_bounds__(256) void headnorm_gate_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ gate, int ldg, int gate_col0,
                                                            T* __restrict__ out, int n_heads_total, int H, int Dv, float eps,
                                                            int gate_kind) {
    const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (unit >= n_heads_total) return;
    const int t = unit / H, h = unit - t * H;
    const float* xr = x + (size_t)unit * Dv;
    float ss = 0.f;
    for (int i = lane; i < Dv; i += 64) ss += xr[i] * xr[i];
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)Dv + eps);
    for (int i = lane; i < Dv; i += 64) {
        float v = xr[i] * inv * (w ? w[h * Dv + i] : 1.0f);
        if (gate) {
            const float z = gate[(size_t)t * ldg + gate_col0 + h * Dv + i];
            v *= (gate_kind == 2 ? z : 1.0f) / (1.0f + expf(-z));
        }
        out[(size_t)unit * Dv + i] = from_f32<T>(v);
    }
}

extern "C" int fl_headnorm_gate(const float* x, const float* w, const float* gate, int ldg, int gate_col0, void* out,
                                int out_dtype, int n, int H, int Dv, float eps, int gate_kind, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && Dv > 0, "headnorm_gate: bad sizes");
    FL_CHECK(gate_kind == 1 || gate_kind == 2, "headnorm_gate: gate %d (1 sigmoid, 2 silu)", gate_kind);
    FL_CHECK(!gate || ldg >= gate_col0 + H * Dv, "headnorm_gate: gate columns beyond rows %d wide", ldg);
    if (n == 0) return 0;
    const long units = (long)n * H;
    FL_CHECK(units < (1L << 31), "headnorm_gate: too many rows");
    const int blocks = (int)((units + 3) / 4);
    if (out_dtype == FL_F32)
        headnorm_gate_kernel<float><<<blocks, 256, 0, stream>>>(x, w, gate, ldg, gate_col0, (float*)out, (int)units, H, Dv, eps, gate_kind);
    else if (out_dtype == FL_BF16)
        headnorm_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, w, gate, ldg, gate_col0, (bf16_t*)out, (int)units, H, Dv, eps, gate_kind);
    else
        FL_CHECK(false, "headnorm_gate: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_headnorm_gate)
