// Row-wise operations on the residual stream and on mixers' outputs that need no matrix product:
// the Dynamic Tanh norm, an embedding look-up with a factor, a gated activation of choice, the
// weighted sum of two normed rows, and a gate (with compaction) on heads side by side.
// All arithmetic is float; only the stores are in the storage type.
#include "common.h"
#include "api.h"
#include "recordable.h"

// ------------------------------------------------------------------ Dynamic Tanh
// out[r][i] = tanh(alpha * s) * w[i] + b[i], s = x[row][i] (+ delta[row][i]); with resid_out the sum is
// written back.  No mean, no variance: nothing crosses the elements of a row.
// A thread takes four neighbouring values of a row (one 16-byte load where the width allows it); a row is
// spread over as many blocks as it has thousands of values, so that a step of few rows still fills units.
template <typename TOut>
__global__ __launch_bounds__(256) void dyt_kernel(const float* __restrict__ x, const float* __restrict__ delta,
                                                  float* __restrict__ resid_out, const int* __restrict__ rows,
                                                  const float* __restrict__ alpha, const float* __restrict__ w,
                                                  const float* __restrict__ b, TOut* __restrict__ out, int H) {
    const int r = blockIdx.x;
    const size_t row = rows ? (size_t)rows[r] : (size_t)r;
    const float a = alpha[0];
    const int i0 = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (i0 >= H) return;
    float s[4];
    if ((H & 3) == 0) {
        const f32x4 v = *(const f32x4*)(x + row * H + i0);
        s[0] = v[0]; s[1] = v[1]; s[2] = v[2]; s[3] = v[3];
        if (delta) {
            const f32x4 d = *(const f32x4*)(delta + row * H + i0);
            s[0] += d[0]; s[1] += d[1]; s[2] += d[2]; s[3] += d[3];
        }
        if (resid_out) *(f32x4*)(resid_out + row * H + i0) = (f32x4){s[0], s[1], s[2], s[3]};
    } else {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = i0 + u;
            s[u] = i < H ? x[row * H + i] + (delta ? delta[row * H + i] : 0.f) : 0.f;
            if (resid_out && i < H) resid_out[row * H + i] = s[u];
        }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = i0 + u;
        if (i < H) out[(size_t)r * H + i] = from_f32<TOut>(tanhf(a * s[u]) * w[i] + (b ? b[i] : 0.f));
    }
}

extern "C" int fl_dyt(const float* x, const float* delta, float* resid_out, const int* rows, const float* alpha,
                      const float* w, const float* b, void* out, int out_dtype, int n_rows, int H, hipStream_t stream) {
    FL_CHECK(n_rows >= 0 && H > 0, "dyt: bad sizes");
    FL_CHECK(alpha && w, "dyt: needs alpha and a gain");
    FL_CHECK(!(rows && resid_out), "dyt: picked rows are not stored back");
    if (n_rows == 0) return 0;
    FL_CHECK(ceil_div(H, 1024) <= 65535, "dyt: rows of %d values are more than one grid takes", H);
    dim3 grid(n_rows, ceil_div(H, 1024));
    if (out_dtype == FL_F32)
        dyt_kernel<float><<<grid, 256, 0, stream>>>(x, delta, resid_out, rows, alpha, w, b, (float*)out, H);
    else if (out_dtype == FL_BF16)
        dyt_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, delta, resid_out, rows, alpha, w, b, (bf16_t*)out, H);
    else
        FL_CHECK(false, "dyt: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_dyt)

// ------------------------------------------------------------------ embedding with a factor
template <typename T>
__global__ __launch_bounds__(256) void embed_scaled_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                                                           float* __restrict__ out, int H, int V, float scale) {
    int tok = tokens[blockIdx.x];
    if (tok < 0 || tok >= V) tok = 0;  // the host rejects such ids before the launch
    const T* src = table + (size_t)tok * H;
    for (int i = threadIdx.x; i < H; i += 256) out[(size_t)blockIdx.x * H + i] = to_f32(src[i]) * scale;
}

extern "C" int fl_embed_scaled(const void* table, int dtype, const int* tokens, float* out, int n, int H, int V, float scale,
                               hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && V > 0, "embed_scaled: bad sizes");
    if (n == 0) return 0;
    if (dtype == FL_F32)
        embed_scaled_kernel<float><<<n, 256, 0, stream>>>((const float*)table, tokens, out, H, V, scale);
    else if (dtype == FL_BF16)
        embed_scaled_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)table, tokens, out, H, V, scale);
    else
        FL_CHECK(false, "embed_scaled: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_embed_scaled)

// ------------------------------------------------------------------ gated activation
// kinds as in fl_activation: 0 gelu (error function), 1 gelu (tanh form), 2 silu
__device__ __forceinline__ float activate(float z, int kind) {
    if (kind == 0) return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f));
    if (kind == 1) return 0.5f * z * (1.0f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
    return z / (1.0f + expf(-z));
}

// out[r][i] = act(gu[r][i]) * gu[r][I + i]
template <typename TOut>
__global__ __launch_bounds__(256) void gated_act_kernel(const float* __restrict__ gu, TOut* __restrict__ out, int I, int kind) {
    const float* row = gu + (size_t)blockIdx.x * 2 * I;
    const int i0 = (blockIdx.y * 256 + threadIdx.x) * 4;        // four neighbouring values per thread, a row over several blocks
    if (i0 >= I) return;
    if ((I & 3) == 0) {
        const f32x4 g = *(const f32x4*)(row + i0), u = *(const f32x4*)(row + I + i0);
#pragma unroll
        for (int e = 0; e < 4; ++e) out[(size_t)blockIdx.x * I + i0 + e] = from_f32<TOut>(activate(g[e], kind) * u[e]);
    } else {
        for (int i = i0; i < min(i0 + 4, I); ++i) out[(size_t)blockIdx.x * I + i] = from_f32<TOut>(activate(row[i], kind) * row[I + i]);
    }
}

extern "C" int fl_gated_act(const float* gu, void* out, int out_dtype, int n, int I, int kind, hipStream_t stream) {
    FL_CHECK(n >= 0 && I > 0, "gated_act: bad sizes");
    FL_CHECK(kind >= 0 && kind <= 2, "gated_act: unknown activation %d", kind);
    if (n == 0) return 0;
    FL_CHECK(ceil_div(I, 1024) <= 65535, "gated_act: rows of %d values are more than one grid takes", I);
    dim3 grid(n, ceil_div(I, 1024));
    if (out_dtype == FL_F32)
        gated_act_kernel<float><<<grid, 256, 0, stream>>>(gu, (float*)out, I, kind);
    else if (out_dtype == FL_BF16)
        gated_act_kernel<bf16_t><<<grid, 256, 0, stream>>>(gu, (bf16_t*)out, I, kind);
    else
        FL_CHECK(false, "gated_act: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_gated_act)

// ------------------------------------------------------------------ weighted sum of two normed rows
// out[t][i] = ca * a[t][i] / rms(a[t]) * wa[i] + cb * b[t][i] / rms(b[t]) * wb[i], rms with eps inside the root.
__global__ __launch_bounds__(256) void norm_mix_kernel(const float* __restrict__ a, const float* __restrict__ wa, float ca,
                                                       const float* __restrict__ b, const float* __restrict__ wb, float cb,
                                                       float* __restrict__ out, int H, float eps) {
    __shared__ float lds[8];
    const float* ar = a + (size_t)blockIdx.x * H;
    const float* br = b + (size_t)blockIdx.x * H;
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < H; i += 256) {
        sa = fmaf(ar[i], ar[i], sa);
        sb = fmaf(br[i], br[i], sb);
    }
    sa = block_sum<4>(sa, lds);
    sb = block_sum<4>(sb, lds + 4);
    const float ia = ca / sqrtf(sa / (float)H + eps), ib = cb / sqrtf(sb / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += 256) out[(size_t)blockIdx.x * H + i] = ar[i] * ia * wa[i] + br[i] * ib * wb[i];
}

extern "C" int fl_norm_mix(const float* a, const float* wa, float ca, const float* b, const float* wb, float cb, float* out,
                           int n, int H, float eps, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0, "norm_mix: bad sizes");
    if (n == 0) return 0;
    norm_mix_kernel<<<n, 256, 0, stream>>>(a, wa, ca, b, wb, cb, out, H, eps);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_norm_mix)

// ------------------------------------------------------------------ gate on heads side by side
// out[t][h * Dv + j] = x[t][h * ldh + j] * g(gate[t][gate_col0 + h * Dv + j]) for j < Dv: the heads of x may be
// wider than Dv (padded); g: 0 none, 1 sigmoid, 2 silu.
template <typename T>
__global__ __launch_bounds__(256) void heads_gate_kernel(const T* __restrict__ x, int ldh, const float* __restrict__ gate, int ldg,
                                                         int gate_col0, int kind, T* __restrict__ out, int H, int Dv) {
    const size_t t = blockIdx.x;
    for (int e = threadIdx.x; e < H * Dv; e += 256) {
        const int h = e / Dv, j = e - h * Dv;
        float v = to_f32(x[(t * H + h) * ldh + j]);
        if (kind) {
            const float z = gate[t * ldg + gate_col0 + e];
            v *= kind == 1 ? 1.0f / (1.0f + expf(-z)) : z / (1.0f + expf(-z));
        }
        out[t * H * Dv + e] = from_f32<T>(v);
    }
}

extern "C" int fl_heads_gate(const void* x, int dtype, int ldh, const float* gate, int ldg, int gate_col0, int kind, void* out,
                             int n, int H, int Dv, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && Dv > 0 && ldh >= Dv, "heads_gate: bad sizes");
    FL_CHECK(kind >= 0 && kind <= 2 && (kind == 0 || (gate && ldg >= gate_col0 + H * Dv)), "heads_gate: gate %d over rows %d wide", kind, ldg);
    if (n == 0) return 0;
    if (dtype == FL_F32)
        heads_gate_kernel<float><<<n, 256, 0, stream>>>((const float*)x, ldh, gate, ldg, gate_col0, kind, (float*)out, H, Dv);
    else if (dtype == FL_BF16)
        heads_gate_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)x, ldh, gate, ldg, gate_col0, kind, (bf16_t*)out, H, Dv);
    else
        FL_CHECK(false, "heads_gate: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_heads_gate)
