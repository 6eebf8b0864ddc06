// Matrix memory with exponential gating (the mLSTM recurrence), token by token.
//
// Per request and head the state is the memory S [D][Dv], the normaliser n [D] and the running
// maximum m of the log gates, all float, kept in the request's slot between steps and zero when the
// slot is claimed (so m starts at 0).  For every token, with log gates i (input) and f (forget):
//     i = cap * tanh((zi + bi) / cap),   f = logsigmoid(cap * tanh((zf + bf) / cap))
//     m' = max(f + m, i);  a = exp(f + m - m');  b = exp(i - m')
//     S <- a S + b k v^T;  n <- a n + b k;  m <- m'
//     o = S^T q / (max(|n . q|, exp(-m)) + 1e-6)
// The walk is the recurrence itself, so a prompt cut anywhere leaves the same state and the same o.
#include "common.h"
#include "api.h"
#include "recordable.h"

#define ML_GROUP 16          // threads that share a column of S; they own the rows d = g, g + 16, ...
#define ML_COLS 16           // columns of S per block
#define ML_MAX_ROWS 32       // rows per thread: D <= ML_GROUP * ML_MAX_ROWS

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// proj: float rows ld wide holding, per token, q [H][D] at col_q, k [H][D] at col_k, v [H][Dv] at col_v and
// the gate pre-activations zi [H] at col_i, zf [H] at col_f.
// Block = (columns j0 .. j0 + 15, head, request); thread (g, c) holds S[d][j0 + c] for its rows d.
// Every block walks n and m for itself and keeps a copy of its own in the state, since blocks of one
// head start and end at different times: state [slots][H][D * Dv + blocks * (D + 1)], S first (column by
// column, S[d][j] at j * D + d, so that the threads of a column read neighbours), then per block of
// columns n [D] and m (fl_mlstm_state_floats gives the record's size).  A token's inputs are fetched
// while the token before it is worked on.
template <int RPT>
__global__ __launch_bounds__(ML_GROUP * ML_COLS) void mlstm_scan_kernel(
    const float* __restrict__ proj, int ld, int col_q, int col_k, int col_v, int col_i, int col_f,
    const float* __restrict__ bias_i, const float* __restrict__ bias_f, float cap, float q_scale,
    float* __restrict__ state, const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
    const int* __restrict__ seq_slots, float* __restrict__ out, int H, int D, int Dv) {
    const int g = threadIdx.x & (ML_GROUP - 1), c = threadIdx.x / ML_GROUP;
    const int j = blockIdx.x * ML_COLS + c, head = blockIdx.y, s = blockIdx.z;
    const bool live = j < Dv;
    const int start = seq_q_start[s], len = seq_q_len[s];
    const size_t rec = (size_t)D * Dv + (size_t)gridDim.x * (D + 1);
    float* st = state + ((size_t)seq_slots[s] * H + head) * rec;
    float* mine = st + (size_t)D * Dv + (size_t)blockIdx.x * (D + 1);       // this block's n [D] and m
    float S[RPT], nn[RPT];
#pragma unroll
    for (int u = 0; u < RPT; ++u) {
        const int d = g + ML_GROUP * u;
        S[u] = (live && d < D) ? st[(size_t)j * D + d] : 0.f;
        nn[u] = d < D ? mine[d] : 0.f;
    }
    float m = mine[D];
    const float bi = bias_i ? bias_i[head] : 0.f, bf = bias_f ? bias_f[head] : 0.f;
    float q[RPT], k[RPT], v = 0.f, zi = 0.f, zf = 0.f;
    auto fetch = [&](int t, float* qn, float* kn, float& vn, float& zin, float& zfn) {
        const float* row = proj + (size_t)(start + t) * ld;
#pragma unroll
        for (int u = 0; u < RPT; ++u) {
            const int d = g + ML_GROUP * u;
            qn[u] = d < D ? row[col_q + head * D + d] : 0.f;
            kn[u] = d < D ? row[col_k + head * D + d] : 0.f;
        }
        vn = live ? row[col_v + head * Dv + j] : 0.f;
        zin = row[col_i + head];
        zfn = row[col_f + head];
    };
    if (len > 0) fetch(0, q, k, v, zi, zf);
    for (int t = 0; t < len; ++t) {
        float qn[RPT], kn[RPT], vn = 0.f, zin = 0.f, zfn = 0.f;
        if (t + 1 < len) fetch(t + 1, qn, kn, vn, zin, zfn);
#pragma unroll
        for (int u = 0; u < RPT; ++u) q[u] *= q_scale;
        const float gi = cap * tanhf((zi + bi) / cap);
        const float gf = log_sigmoid(cap * tanhf((zf + bf) / cap));
        const float m_new = fmaxf(gf + m, gi);
        const float a = expf(gf + m - m_new), b = expf(gi - m_new);
        m = m_new;
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int u = 0; u < RPT; ++u) {
            S[u] = a * S[u] + b * k[u] * v;
            nn[u] = a * nn[u] + b * k[u];
            num = fmaf(S[u], q[u], num);
            den = fmaf(nn[u], q[u], den);
        }
#pragma unroll
        for (int off = ML_GROUP / 2; off > 0; off >>= 1) {
            num += __shfl_xor(num, off, FL_WAVE);
            den += __shfl_xor(den, off, FL_WAVE);
        }
        if (live && g == 0) out[((size_t)(start + t) * H + head) * Dv + j] = num / (fmaxf(fabsf(den), expf(-m)) + 1e-6f);
        if (t + 1 < len) {
#pragma unroll
            for (int u = 0; u < RPT; ++u) { q[u] = qn[u]; k[u] = kn[u]; }
            v = vn; zi = zin; zf = zfn;
        }
    }
#pragma unroll
    for (int u = 0; u < RPT; ++u) {
        const int d = g + ML_GROUP * u;
        if (live && d < D) st[(size_t)j * D + d] = S[u];
        if (c == 0 && d < D) mine[d] = nn[u];
    }
    if (threadIdx.x == 0) mine[D] = m;
}

extern "C" int fl_mlstm_max_dim(void) { return ML_GROUP * ML_MAX_ROWS; }
// floats of one head's record in the state
extern "C" long fl_mlstm_state_floats(int D, int Dv) { return (long)D * Dv + (long)ceil_div(Dv, ML_COLS) * (D + 1); }

extern "C" int fl_mlstm_scan(const float* proj, int ld, int col_q, int col_k, int col_v, int col_i, int col_f,
                             const float* bias_i, const float* bias_f, float cap, float q_scale, float* state,
                             const int* seq_q_start, const int* seq_q_len, const int* seq_slots, float* out,
                             int n_seqs, int H, int D, int Dv, hipStream_t stream) {
    FL_CHECK(n_seqs >= 0 && H > 0 && D > 0 && Dv > 0, "mlstm_scan: bad sizes");
    FL_CHECK(D <= ML_GROUP * ML_MAX_ROWS, "mlstm_scan: %d key dims per head, at most %d", D, ML_GROUP * ML_MAX_ROWS);
    FL_CHECK(cap > 0.f, "mlstm_scan: the gates' cap must be positive");
    FL_CHECK(ld >= col_q + H * D && ld >= col_k + H * D && ld >= col_v + H * Dv && ld >= col_i + H && ld >= col_f + H,
             "mlstm_scan: columns beyond rows %d wide", ld);
    if (n_seqs == 0) return 0;
    FL_CHECK(n_seqs <= 65535 && H <= 65535, "mlstm_scan: %d requests of %d heads are more than one grid takes", n_seqs, H);
    dim3 grid(ceil_div(Dv, ML_COLS), H, n_seqs);
    const int rpt = ceil_div(D, ML_GROUP);
#define FL_ML(R)                                                                                                      \
    mlstm_scan_kernel<R><<<grid, ML_GROUP * ML_COLS, 0, stream>>>(proj, ld, col_q, col_k, col_v, col_i, col_f, bias_i, \
                                                                  bias_f, cap, q_scale, state, seq_q_start, seq_q_len, \
                                                                  seq_slots, out, H, D, Dv)
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
// out[t][h][:] = o / sqrt(mean(o^2) + eps) * w[h][:] * sigmoid(gate[t][gate_col0 + h * Dv + :]),
// o = x[t][h][:] (float).  One wave per (token, head).
template <typename T>
__global__ __launch_bounds__(256) void headnorm_gate_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ gate, int ldg, int gate_col0,
                                                            T* __restrict__ out, int n_heads_total, int H, int Dv, float eps) {
    const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (unit >= n_heads_total) return;
    const int t = unit / H, h = unit - t * H;
    const float* xr = x + (size_t)unit * Dv;
    float ss = 0.f;
    for (int i = lane; i < Dv; i += 64) ss += xr[i] * xr[i];
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)Dv + eps);
    for (int i = lane; i < Dv; i += 64) {
        float v = xr[i] * inv * (w ? w[h * Dv + i] : 1.0f);
        if (gate) v *= 1.0f / (1.0f + expf(-gate[(size_t)t * ldg + gate_col0 + h * Dv + i]));
        out[(size_t)unit * Dv + i] = from_f32<T>(v);
    }
}

extern "C" int fl_headnorm_gate(const float* x, const float* w, const float* gate, int ldg, int gate_col0, void* out,
                                int out_dtype, int n, int H, int Dv, float eps, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && Dv > 0, "headnorm_gate: bad sizes");
    FL_CHECK(!gate || ldg >= gate_col0 + H * Dv, "headnorm_gate: gate columns beyond rows %d wide", ldg);
    if (n == 0) return 0;
    const long units = (long)n * H;
    FL_CHECK(units < (1L << 31), "headnorm_gate: too many rows");
    const int blocks = (int)((units + 3) / 4);
    if (out_dtype == FL_F32)
        headnorm_gate_kernel<float><<<blocks, 256, 0, stream>>>(x, w, gate, ldg, gate_col0, (float*)out, (int)units, H, Dv, eps);
    else if (out_dtype == FL_BF16)
        headnorm_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, w, gate, ldg, gate_col0, (bf16_t*)out, (int)units, H, Dv, eps);
    else
        FL_CHECK(false, "headnorm_gate: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_headnorm_gate)
