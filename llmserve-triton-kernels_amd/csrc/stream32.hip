// Kernels of a layer whose residual stream is kept in 32-bit whatever the model's dtype:
//   embed_scale      x[n] = table[ids[n]] * scale                                   (table T, x float)
//   rmsnorm32        y[r] = x[s] * rsqrt(mean(x[s]^2) + eps) * (offset + w), s = rows[r] or r   (x float, y T)
//   gated_add        x[n] += sum over branches b of g_b * y_b[n]                    (all float)
//                    g_b = sigmoid(z_b[n] + bias_b) where the branch has a gate, else 1
//   gated_add_norm   the same sum and, in the same kernel, the norm of the summed row for the next layer
//   streams_norm     a residual stream of S parallel copies (S = 1: the plain residual sum).  With the result y of
//                    the sublayer before and its coefficients, new_t = sum_s mix[s, t] x_s + out[t] y for all t at
//                    once; u = sum_t read[t] new_t; out = (u - mean) / sqrt(var + eps) * w (layer norm, no bias; the
//                    variance is the mean squared deviation).                       (x, y, coefficients float; out T)
//   normed_add_norm  a sublayer's result joins the stream through a norm of its own, and the next sublayer's input is
//                    formed in the same pass: x += y / sqrt(mean(y^2) + eps) * wb; out = x / sqrt(mean(x^2) + eps) * w
//   add_vector       x[n] += v for every row
// T is float or bfloat16.  One workgroup per row; every reduction has an order fixed by the sizes alone.
#include "common.h"

#define S32_THREADS 256

template <typename T>
__global__ __launch_bounds__(S32_THREADS) void embed_scale_kernel(float* __restrict__ out, const T* __restrict__ table,
                                                                  const int* __restrict__ ids, int hidden, int vocab,
                                                                  float scale) {
    const int n = blockIdx.x;
    int id = ids[n];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const T* row = table + (size_t)id * hidden;
    for (int c = threadIdx.x; c < hidden; c += S32_THREADS) out[(size_t)n * hidden + c] = to_f32(row[c]) * scale;
}

// Rows whose length is a multiple of 4: a thread brings up to S32_VEC float4 of its row at once (rows of up to
// 4 * S32_VEC * S32_THREADS), so a row costs one wait for memory and not one per 256 elements.
#define S32_VEC 8

template <typename T>
__global__ __launch_bounds__(S32_THREADS) void rmsnorm32_vec_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                                    const float* __restrict__ weight,
                                                                    const int* __restrict__ rows, int hidden, float eps,
                                                                    float offset) {
    __shared__ float lds[16];
    const int r = blockIdx.x;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)(rows ? rows[r] : r) * hidden);
    const float4* wr = reinterpret_cast<const float4*>(weight);
    const int n4 = hidden / 4;
    float4 v[S32_VEC], w[S32_VEC];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < S32_VEC; ++i) {
        const int c = threadIdx.x + i * S32_THREADS;
        v[i] = c < n4 ? xr[c] : make_float4(0.f, 0.f, 0.f, 0.f);
        w[i] = c < n4 ? wr[c] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < S32_VEC; ++i) ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    const float inv = 1.0f / sqrtf(block_sum(ss, lds) / (float)hidden + eps);
    T* orow = out + (size_t)r * hidden;
#pragma unroll
    for (int i = 0; i < S32_VEC; ++i) {
        const int c = threadIdx.x + i * S32_THREADS;
        if (c < n4) {
            orow[4 * c + 0] = from_f32<T>(v[i].x * inv * (offset + w[i].x));
            orow[4 * c + 1] = from_f32<T>(v[i].y * inv * (offset + w[i].y));
            orow[4 * c + 2] = from_f32<T>(v[i].z * inv * (offset + w[i].z));
            orow[4 * c + 3] = from_f32<T>(v[i].w * inv * (offset + w[i].w));
        }
    }
}

__device__ __forceinline__ float4 gate4(float4 z, float4 b) {
    return make_float4(1.f / (1.f + expf(-(z.x + b.x))), 1.f / (1.f + expf(-(z.y + b.y))), 1.f / (1.f + expf(-(z.z + b.z))),
                       1.f / (1.f + expf(-(z.w + b.w))));
}

// gated_add for rows of a multiple of 4 (and gate columns at multiples of 4): grid (rows, ceil(hidden / 4 / threads))
__global__ __launch_bounds__(S32_THREADS) void gated_add_vec_kernel(float* __restrict__ x, const float* __restrict__ z,
                                                                    int z_stride, int z_col0, int z_col1,
                                                                    const float* __restrict__ bias0,
                                                                    const float* __restrict__ bias1,
                                                                    const float* __restrict__ y0, int y0_stride,
                                                                    const float* __restrict__ y1, int y1_stride,
                                                                    int hidden) {
    const int n = blockIdx.x, c = 4 * (blockIdx.y * S32_THREADS + threadIdx.x);
    if (c >= hidden) return;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f), one = make_float4(1.f, 1.f, 1.f, 1.f);
    auto at = [](const float* p) { return *reinterpret_cast<const float4*>(p); };
    // every load is asked for before the first is used
    const float4 xv = at(x + (size_t)n * hidden + c);
    const float4 a0 = y0 ? at(y0 + (size_t)n * y0_stride + c) : zero;
    const float4 a1 = y1 ? at(y1 + (size_t)n * y1_stride + c) : zero;
    const float4 z0 = (y0 && z_col0 >= 0) ? at(z + (size_t)n * z_stride + z_col0 + c) : zero;
    const float4 z1 = (y1 && z_col1 >= 0) ? at(z + (size_t)n * z_stride + z_col1 + c) : zero;
    const float4 b0 = (y0 && z_col0 >= 0 && bias0) ? at(bias0 + c) : zero;
    const float4 b1 = (y1 && z_col1 >= 0 && bias1) ? at(bias1 + c) : zero;
    const float4 g0 = (y0 && z_col0 >= 0) ? gate4(z0, b0) : one;
    const float4 g1 = (y1 && z_col1 >= 0) ? gate4(z1, b1) : one;
    float4 r;
    r.x = xv.x + (g0.x * a0.x + g1.x * a1.x);
    r.y = xv.y + (g0.y * a0.y + g1.y * a1.y);
    r.z = xv.z + (g0.z * a0.z + g1.z * a1.z);
    r.w = xv.w + (g0.w * a0.w + g1.w * a1.w);
    *reinterpret_cast<float4*>(x + (size_t)n * hidden + c) = r;
}

// gated_add and the norm of the summed row in one kernel (what the next layer reads): x[n] is summed and stored as in
// gated_add_vec, out[n] = x[n] * rsqrt(mean(x[n]^2) + eps) * (offset + w).  One workgroup a row of up to
// 4 * S32_VEC * S32_THREADS.
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void gated_add_norm_vec_kernel(
    T* __restrict__ out, float* __restrict__ x, const float* __restrict__ z, int z_stride, int z_col0, int z_col1,
    const float* __restrict__ bias0, const float* __restrict__ bias1, const float* __restrict__ y0, int y0_stride,
    const float* __restrict__ y1, int y1_stride, const float* __restrict__ weight, int hidden, float eps, float offset) {
    __shared__ float lds[16];
    const int n = blockIdx.x, n4 = hidden / 4;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f), one = make_float4(1.f, 1.f, 1.f, 1.f);
    auto at = [](const float* p) { return *reinterpret_cast<const float4*>(p); };
    float4 r[S32_VEC];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < S32_VEC; ++i) {
        const int c = 4 * (threadIdx.x + i * S32_THREADS);
        r[i] = zero;
        if (c < hidden) {
            const float4 xv = at(x + (size_t)n * hidden + c);
            const float4 a0 = y0 ? at(y0 + (size_t)n * y0_stride + c) : zero;
            const float4 a1 = y1 ? at(y1 + (size_t)n * y1_stride + c) : zero;
            const float4 z0 = (y0 && z_col0 >= 0) ? at(z + (size_t)n * z_stride + z_col0 + c) : zero;
            const float4 z1 = (y1 && z_col1 >= 0) ? at(z + (size_t)n * z_stride + z_col1 + c) : zero;
            const float4 b0 = (y0 && z_col0 >= 0 && bias0) ? at(bias0 + c) : zero;
            const float4 b1 = (y1 && z_col1 >= 0 && bias1) ? at(bias1 + c) : zero;
            const float4 g0 = (y0 && z_col0 >= 0) ? gate4(z0, b0) : one;
            const float4 g1 = (y1 && z_col1 >= 0) ? gate4(z1, b1) : one;
            float4 s;
            s.x = xv.x + (g0.x * a0.x + g1.x * a1.x);
            s.y = xv.y + (g0.y * a0.y + g1.y * a1.y);
            s.z = xv.z + (g0.z * a0.z + g1.z * a1.z);
            s.w = xv.w + (g0.w * a0.w + g1.w * a1.w);
            *reinterpret_cast<float4*>(x + (size_t)n * hidden + c) = s;
            r[i] = s;
            ss += s.x * s.x + s.y * s.y + s.z * s.z + s.w * s.w;
        }
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, lds) / (float)hidden + eps);
    T* orow = out + (size_t)n * hidden;
#pragma unroll
    for (int i = 0; i < S32_VEC; ++i) {
        const int c = 4 * (threadIdx.x + i * S32_THREADS);
        if (c < hidden) {
            const float4 w = at(weight + c);
            orow[c + 0] = from_f32<T>(r[i].x * inv * (offset + w.x));
            orow[c + 1] = from_f32<T>(r[i].y * inv * (offset + w.y));
            orow[c + 2] = from_f32<T>(r[i].z * inv * (offset + w.z));
            orow[c + 3] = from_f32<T>(r[i].w * inv * (offset + w.w));
        }
    }
    (void)n4;
}

template <typename T>
__global__ __launch_bounds__(S32_THREADS) void rmsnorm32_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                                const float* __restrict__ weight,
                                                                const int* __restrict__ rows, int hidden, float eps,
                                                                float offset) {
    __shared__ float lds[16];
    const int r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : r) * hidden;
    float ss = 0.f;
    for (int c = threadIdx.x; c < hidden; c += S32_THREADS) {
        const float v = xr[c];
        ss = fmaf(v, v, ss);
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, lds) / (float)hidden + eps);
    for (int c = threadIdx.x; c < hidden; c += S32_THREADS)
        out[(size_t)r * hidden + c] = from_f32<T>(xr[c] * inv * (offset + weight[c]));
}

// z: [N, z_stride] raw gate products, branch b's at columns z_col[b] .. z_col[b] + hidden (z_col[b] < 0: no gate).
__global__ __launch_bounds__(S32_THREADS) void gated_add_kernel(float* __restrict__ x, const float* __restrict__ z,
                                                                int z_stride, int z_col0, int z_col1,
                                                                const float* __restrict__ bias0,
                                                                const float* __restrict__ bias1,
                                                                const float* __restrict__ y0, int y0_stride,
                                                                const float* __restrict__ y1, int y1_stride,
                                                                int hidden) {
    const int n = blockIdx.x;
    for (int c = threadIdx.x; c < hidden; c += S32_THREADS) {
        float sum = 0.f;
        if (y0) {
            float g = 1.f;
            if (z_col0 >= 0) g = 1.f / (1.f + expf(-(z[(size_t)n * z_stride + z_col0 + c] + (bias0 ? bias0[c] : 0.f))));
            sum = g * y0[(size_t)n * y0_stride + c];
        }
        if (y1) {
            float g = 1.f;
            if (z_col1 >= 0) g = 1.f / (1.f + expf(-(z[(size_t)n * z_stride + z_col1 + c] + (bias1 ? bias1[c] : 0.f))));
            sum += g * y1[(size_t)n * y1_stride + c];
        }
        x[(size_t)n * hidden + c] += sum;
    }
}

#define STREAMS_MAX 8

// One workgroup a row.  x_src is [N, S, hidden] (stream stride `hidden`) or, with src_broadcast, [N, hidden] read as
// S equal copies; x_dst (may be x_src itself: every thread reads all of a column's streams before it writes them) takes
// the new streams when `store`.  `y` null: nothing is added and the streams pass as they are.  `read` null: the plain
// sum of the streams.  `rows`: only these rows are worked out (out[r] from row rows[r]).  `center` 0: the mean is not
// taken off (an RMS norm: u / sqrt(mean(u^2) + eps) * w).  Dynamic LDS: hidden floats.
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void streams_norm_kernel(
    T* __restrict__ out, float* x_dst, const float* x_src, int src_broadcast, const float* __restrict__ y,
    const float* __restrict__ mix, const float* __restrict__ wout, const float* __restrict__ read,
    const float* __restrict__ weight, const int* __restrict__ rows, int streams, int hidden, float eps, int store,
    int center) {
    extern __shared__ float u_row[];
    __shared__ float red[16];
    __shared__ float coef[STREAMS_MAX * STREAMS_MAX + 2 * STREAMS_MAX];
    const int r = blockIdx.x, n = rows ? rows[r] : r, S = streams;
    for (int i = threadIdx.x; i < S * S + 2 * S; i += S32_THREADS) {
        float v;
        if (i < S * S) v = mix ? mix[i] : (i / S == i % S ? 1.f : 0.f);
        else if (i < S * S + S) v = wout ? wout[i - S * S] : 1.f;
        else v = read ? read[i - S * S - S] : 1.f;
        coef[i] = v;
    }
    __syncthreads();
    const float* cm = coef;
    const float* co = coef + S * S;
    const float* cr = co + S;
    const float* src = x_src + (size_t)n * hidden * (src_broadcast ? 1 : S);
    float* dst = x_dst + (size_t)n * hidden * S;
    float total = 0.f;
    for (int c = threadIdx.x; c < hidden; c += S32_THREADS) {
        float xs[STREAMS_MAX];
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s) xs[s] = s < S ? src[src_broadcast ? c : (size_t)s * hidden + c] : 0.f;
        const float yv = y ? y[(size_t)n * hidden + c] : 0.f;
        float u = 0.f;
#pragma unroll
        for (int t = 0; t < STREAMS_MAX; ++t) {
            if (t < S) {
                float v = xs[t];
                if (y) {
                    v = 0.f;
#pragma unroll
                    for (int s = 0; s < STREAMS_MAX; ++s)
                        if (s < S) v = fmaf(cm[s * S + t], xs[s], v);
                    v = fmaf(co[t], yv, v);
                }
                if (store) dst[(size_t)t * hidden + c] = v;
                u = fmaf(cr[t], v, u);
            }
        }
        u_row[c] = u;
        total += u;
    }
    const float mean = center ? block_sum(total, red) / (float)hidden : 0.f;
    float dev2 = 0.f;
    for (int c = threadIdx.x; c < hidden; c += S32_THREADS) {
        const float d = u_row[c] - mean;
        dev2 = fmaf(d, d, dev2);
    }
    const float inv = 1.0f / sqrtf(block_sum(dev2, red) / (float)hidden + eps);
    if (!out) return;
    T* orow = out + (size_t)r * hidden;
    for (int c = threadIdx.x; c < hidden; c += S32_THREADS) orow[c] = from_f32<T>((u_row[c] - mean) * inv * weight[c]);
}

// The same for rows of a multiple of 4: a thread takes two float4 columns at a time with every load of both asked for
// before the first is used, so a row of 2,048 costs one wait for memory.
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void streams_norm_vec_kernel(
    T* __restrict__ out, float* x_dst, const float* x_src, int src_broadcast, const float* __restrict__ y,
    const float* __restrict__ mix, const float* __restrict__ wout, const float* __restrict__ read,
    const float* __restrict__ weight, const int* __restrict__ rows, int streams, int hidden, float eps, int store,
    int center) {
    extern __shared__ float u_row[];
    __shared__ float red[16];
    __shared__ float coef[STREAMS_MAX * STREAMS_MAX + 2 * STREAMS_MAX];
    const int r = blockIdx.x, n = rows ? rows[r] : r, S = streams, n4 = hidden / 4;
    const float* src = x_src + (size_t)n * hidden * (src_broadcast ? 1 : S);
    float* dst = x_dst + (size_t)n * hidden * S;
    auto at = [](const float* p) { return *reinterpret_cast<const float4*>(p); };
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    // the first columns are asked for before the coefficients are waited for
    float4 xs[2][STREAMS_MAX], yv[2];
    auto ask = [&](int base) {
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            const int c4 = base + v * S32_THREADS + threadIdx.x;
#pragma unroll
            for (int s = 0; s < STREAMS_MAX; ++s)
                xs[v][s] = (s < S && c4 < n4) ? at(src + (src_broadcast ? 0 : (size_t)s * hidden) + 4 * c4) : zero;
            yv[v] = (y && c4 < n4) ? at(y + (size_t)n * hidden + 4 * c4) : zero;
        }
    };
    ask(0);
    for (int i = threadIdx.x; i < S * S + 2 * S; i += S32_THREADS) {
        float v;
        if (i < S * S) v = mix ? mix[i] : (i / S == i % S ? 1.f : 0.f);
        else if (i < S * S + S) v = wout ? wout[i - S * S] : 1.f;
        else v = read ? read[i - S * S - S] : 1.f;
        coef[i] = v;
    }
    __syncthreads();
    const float* cm = coef;
    const float* co = coef + S * S;
    const float* cr = co + S;
    float total = 0.f;
    for (int base = 0; base < n4; base += 2 * S32_THREADS) {
        if (base) ask(base);
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            const int c4 = base + v * S32_THREADS + threadIdx.x;
            if (c4 >= n4) continue;
            float4 u = zero;
#pragma unroll
            for (int t = 0; t < STREAMS_MAX; ++t) {
                if (t < S) {
                    float4 w4 = xs[v][t];
                    if (y) {
                        w4 = zero;
#pragma unroll
                        for (int s = 0; s < STREAMS_MAX; ++s)
                            if (s < S) {
                                const float k = cm[s * S + t];
                                w4.x = fmaf(k, xs[v][s].x, w4.x), w4.y = fmaf(k, xs[v][s].y, w4.y);
                                w4.z = fmaf(k, xs[v][s].z, w4.z), w4.w = fmaf(k, xs[v][s].w, w4.w);
                            }
                        const float k = co[t];
                        w4.x = fmaf(k, yv[v].x, w4.x), w4.y = fmaf(k, yv[v].y, w4.y);
                        w4.z = fmaf(k, yv[v].z, w4.z), w4.w = fmaf(k, yv[v].w, w4.w);
                    }
                    if (store) *reinterpret_cast<float4*>(dst + (size_t)t * hidden + 4 * c4) = w4;
                    const float k = cr[t];
                    u.x = fmaf(k, w4.x, u.x), u.y = fmaf(k, w4.y, u.y), u.z = fmaf(k, w4.z, u.z), u.w = fmaf(k, w4.w, u.w);
                }
            }
            *reinterpret_cast<float4*>(u_row + 4 * c4) = u;
            total += (u.x + u.y) + (u.z + u.w);
        }
    }
    const float mean = center ? block_sum(total, red) / (float)hidden : 0.f;
    float dev2 = 0.f;
    for (int c4 = threadIdx.x; c4 < n4; c4 += S32_THREADS) {
        const float4 u = *reinterpret_cast<const float4*>(u_row + 4 * c4);
        const float a = u.x - mean, b = u.y - mean, c = u.z - mean, d = u.w - mean;
        dev2 += (a * a + b * b) + (c * c + d * d);
    }
    const float inv = 1.0f / sqrtf(block_sum(dev2, red) / (float)hidden + eps);
    if (!out) return;
    T* orow = out + (size_t)r * hidden;
    for (int c4 = threadIdx.x; c4 < n4; c4 += S32_THREADS) {
        const float4 u = *reinterpret_cast<const float4*>(u_row + 4 * c4);
        const float4 w4 = at(weight + 4 * c4);
        const float a = (u.x - mean) * inv * w4.x, b = (u.y - mean) * inv * w4.y;
        const float c = (u.z - mean) * inv * w4.z, d = (u.w - mean) * inv * w4.w;
        if constexpr (sizeof(T) == 2) {  // (rows of a multiple of 4 at an aligned start: 8 bytes at once)
            *reinterpret_cast<uint2*>(orow + 4 * c4) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(c, d));
        } else {
            *reinterpret_cast<float4*>(orow + 4 * c4) = make_float4(a, b, c, d);
        }
    }
}

// One stream (S = 1) with rows of 256 V numbers, V up to 16: a wave takes a row and keeps it in registers (V float4 a
// lane), so the row costs one wait for memory, no LDS and no barrier; a workgroup is 4 rows.  The same arithmetic per
// element as above (new = mix x + write y, u = read new); the sums of a row are formed lane by lane and then across
// the wave, in an order that depends on the row's length alone.
template <typename T, int V>
__global__ __launch_bounds__(S32_THREADS) void streams_norm_wave_kernel(
    T* __restrict__ out, float* x_dst, const float* x_src, const float* __restrict__ y, const float* __restrict__ mix,
    const float* __restrict__ wout, const float* __restrict__ read, const float* __restrict__ weight,
    const int* __restrict__ rows, int n_out, int hidden, float eps, int store, int center) {
    const int lane = threadIdx.x % LLMS_WAVE, r = blockIdx.x * (S32_THREADS / LLMS_WAVE) + threadIdx.x / LLMS_WAVE;
    if (r >= n_out) return;
    const int n = rows ? rows[r] : r;
    const float4* src = reinterpret_cast<const float4*>(x_src + (size_t)n * hidden);
    const float4* ys = y ? reinterpret_cast<const float4*>(y + (size_t)n * hidden) : nullptr;
    float4 u[V], yv[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        u[v] = src[v * LLMS_WAVE + lane];
        yv[v] = ys ? ys[v * LLMS_WAVE + lane] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    const float cm = mix ? mix[0] : 1.f, co = wout ? wout[0] : 1.f, cr = read ? read[0] : 1.f;
    float total = 0.f;
#pragma unroll
    for (int v = 0; v < V; ++v) {
        float4 w4 = u[v];
        if (ys) {
            w4.x = fmaf(co, yv[v].x, cm * w4.x), w4.y = fmaf(co, yv[v].y, cm * w4.y);
            w4.z = fmaf(co, yv[v].z, cm * w4.z), w4.w = fmaf(co, yv[v].w, cm * w4.w);
        }
        if (store) reinterpret_cast<float4*>(x_dst + (size_t)n * hidden)[v * LLMS_WAVE + lane] = w4;
        u[v] = make_float4(cr * w4.x, cr * w4.y, cr * w4.z, cr * w4.w);
        total += (u[v].x + u[v].y) + (u[v].z + u[v].w);
    }
    if (!out) return;
    const float mean = center ? wave_sum(total) / (float)hidden : 0.f;
    float dev2 = 0.f;
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const float a = u[v].x - mean, b = u[v].y - mean, c = u[v].z - mean, d = u[v].w - mean;
        dev2 += (a * a + b * b) + (c * c + d * d);
    }
    const float inv = 1.0f / sqrtf(wave_sum(dev2) / (float)hidden + eps);
    T* orow = out + (size_t)r * hidden;
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const int c4 = v * LLMS_WAVE + lane;
        const float4 w4 = reinterpret_cast<const float4*>(weight)[c4];
        const float a = (u[v].x - mean) * inv * w4.x, b = (u[v].y - mean) * inv * w4.y;
        const float c = (u[v].z - mean) * inv * w4.z, d = (u[v].w - mean) * inv * w4.w;
        if constexpr (sizeof(T) == 2) {
            *reinterpret_cast<uint2*>(orow + 4 * c4) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(c, d));
        } else {
            *reinterpret_cast<float4*>(orow + 4 * c4) = make_float4(a, b, c, d);
        }
    }
}

// x <- cap * tanh(x / cap), in place on 32-bit numbers (logits)
__global__ void softcap_kernel(float* __restrict__ x, size_t total, float cap) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total) x[i] = cap * tanhf(x[i] / cap);
}

// out = sa * a + sb * b (out may be a or b: a thread reads both before it writes)
__global__ void weighted_sum_kernel(float* out, const float* a, const float* b, float sa, float sb, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total) out[i] = fmaf(sa, a[i], sb * b[i]);
}

// grid: rows.  Dynamic LDS: hidden floats (the summed row; rows of up to 4,096 numbers in 16-byte pieces stay in
// registers instead).  `y` null: nothing joins; `out` null: the sum alone.
#define NAN_VEC 4
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void normed_add_norm_kernel(T* __restrict__ out, float* __restrict__ x,
                                                                      const float* __restrict__ y, const float* __restrict__ wb,
                                                                      const float* __restrict__ w, const int* __restrict__ rows,
                                                                      int hidden, float eps_y, float eps, int store) {
    extern __shared__ float summed[];
    __shared__ float red[16];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* xr = x + src * hidden;
    const float* yr = y ? y + src * hidden : nullptr;
    const bool vec = hidden % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)wb % 16) == 0 &&
                     ((uintptr_t)w % 16) == 0 && ((uintptr_t)out % 16) == 0;
    if (vec && hidden <= 4 * NAN_VEC * S32_THREADS) {
        // the row, what joins it and that norm's weight in registers, all asked for at once: one trip to memory
        float4 xv[NAN_VEC], yv[NAN_VEC], bv[NAN_VEC];
#pragma unroll
        for (int i = 0; i < NAN_VEC; ++i) {
            const int c = 4 * (threadIdx.x + i * S32_THREADS);
            const bool in = c < hidden;
            xv[i] = in ? *reinterpret_cast<const float4*>(xr + c) : make_float4(0.f, 0.f, 0.f, 0.f);
            yv[i] = (in && yr) ? *reinterpret_cast<const float4*>(yr + c) : make_float4(0.f, 0.f, 0.f, 0.f);
            bv[i] = (in && yr) ? *reinterpret_cast<const float4*>(wb + c) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        if (yr) {
            float sy = 0.f;
#pragma unroll
            for (int i = 0; i < NAN_VEC; ++i)
                sy = fmaf(yv[i].x, yv[i].x, sy), sy = fmaf(yv[i].y, yv[i].y, sy), sy = fmaf(yv[i].z, yv[i].z, sy), sy = fmaf(yv[i].w, yv[i].w, sy);
            const float inv_y = 1.f / sqrtf(block_sum(sy, red) / (float)hidden + eps_y);
#pragma unroll
            for (int i = 0; i < NAN_VEC; ++i) {
                xv[i].x += yv[i].x * inv_y * bv[i].x, xv[i].y += yv[i].y * inv_y * bv[i].y;
                xv[i].z += yv[i].z * inv_y * bv[i].z, xv[i].w += yv[i].w * inv_y * bv[i].w;
                const int c = 4 * (threadIdx.x + i * S32_THREADS);
                if (store && c < hidden) *reinterpret_cast<float4*>(xr + c) = xv[i];
            }
        }
        if (!out) return;
        float sx = 0.f;
#pragma unroll
        for (int i = 0; i < NAN_VEC; ++i)
            sx = fmaf(xv[i].x, xv[i].x, sx), sx = fmaf(xv[i].y, xv[i].y, sx), sx = fmaf(xv[i].z, xv[i].z, sx), sx = fmaf(xv[i].w, xv[i].w, sx);
        const float inv = 1.f / sqrtf(block_sum(sx, red) / (float)hidden + eps);
        T* orow = out + (size_t)r * hidden;
#pragma unroll
        for (int i = 0; i < NAN_VEC; ++i) {
            const int c = 4 * (threadIdx.x + i * S32_THREADS);
            if (c >= hidden) continue;
            const float4 wv = *reinterpret_cast<const float4*>(w + c);
            const float a = xv[i].x * inv * wv.x, b = xv[i].y * inv * wv.y, cc = xv[i].z * inv * wv.z, d = xv[i].w * inv * wv.w;
            if constexpr (sizeof(T) == 2) {
                uint2 packed = make_uint2(pack_bf16x2(a, b), pack_bf16x2(cc, d));
                *reinterpret_cast<uint2*>(orow + c) = packed;
            } else {
                *reinterpret_cast<float4*>(orow + c) = make_float4(a, b, cc, d);
            }
        }
        return;
    }
    float inv_y = 0.f;
    if (yr) {
        float ss = 0.f;
        if (vec) {
            for (int c = 4 * threadIdx.x; c < hidden; c += 4 * S32_THREADS) {
                const float4 v = *reinterpret_cast<const float4*>(yr + c);
                ss = fmaf(v.x, v.x, ss), ss = fmaf(v.y, v.y, ss), ss = fmaf(v.z, v.z, ss), ss = fmaf(v.w, v.w, ss);
            }
        } else {
            for (int c = threadIdx.x; c < hidden; c += S32_THREADS) ss = fmaf(yr[c], yr[c], ss);
        }
        inv_y = 1.f / sqrtf(block_sum(ss, red) / (float)hidden + eps_y);
    }
    float ss = 0.f;
    if (vec) {
        for (int c = 4 * threadIdx.x; c < hidden; c += 4 * S32_THREADS) {
            float4 v = *reinterpret_cast<const float4*>(xr + c);
            if (yr) {
                const float4 a = *reinterpret_cast<const float4*>(yr + c);
                const float4 b = *reinterpret_cast<const float4*>(wb + c);
                v.x += a.x * inv_y * b.x, v.y += a.y * inv_y * b.y, v.z += a.z * inv_y * b.z, v.w += a.w * inv_y * b.w;
                if (store) *reinterpret_cast<float4*>(xr + c) = v;
            }
            *reinterpret_cast<float4*>(summed + c) = v;
            ss = fmaf(v.x, v.x, ss), ss = fmaf(v.y, v.y, ss), ss = fmaf(v.z, v.z, ss), ss = fmaf(v.w, v.w, ss);
        }
    } else {
        for (int c = threadIdx.x; c < hidden; c += S32_THREADS) {
            float v = xr[c];
            if (yr) {
                v += yr[c] * inv_y * wb[c];
                if (store) xr[c] = v;
            }
            summed[c] = v;
            ss = fmaf(v, v, ss);
        }
    }
    if (!out) return;
    const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)hidden + eps);
    T* orow = out + (size_t)r * hidden;
    for (int c = threadIdx.x; c < hidden; c += S32_THREADS) orow[c] = from_f32<T>(summed[c] * inv * w[c]);
}

__global__ __launch_bounds__(S32_THREADS) void add_vector_kernel(float* __restrict__ x, const float* __restrict__ v, int hidden) {
    float* xr = x + (size_t)blockIdx.x * hidden;
    for (int c = threadIdx.x; c < hidden; c += S32_THREADS) xr[c] += v[c];
}

extern "C" {

int llms_weighted_sum(float* out, const float* a, const float* b, float sa, float sb, size_t total, hipStream_t stream) {
    LLMS_REQUIRE(total > 0, "weighted_sum: a positive size");
    weighted_sum_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(out, a, b, sa, sb, total);
    LLMS_LAUNCH_CHECK();
}

int llms_softcap(float* x, size_t total, float cap, hipStream_t stream) {
    LLMS_REQUIRE(total > 0 && cap > 0.f, "softcap: a positive size and a positive cap");
    softcap_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(x, total, cap);
    LLMS_LAUNCH_CHECK();
}

int llms_embed_scale(int dtype, float* out, const void* table, const int* ids, int n, int hidden, int vocab, float scale,
                     hipStream_t stream) {
    LLMS_REQUIRE(n > 0 && hidden > 0 && vocab > 0, "embed_scale: sizes must be positive");
    if (dtype == 0)
        embed_scale_kernel<float><<<n, S32_THREADS, 0, stream>>>(out, (const float*)table, ids, hidden, vocab, scale);
    else if (dtype == 1)
        embed_scale_kernel<bf16><<<n, S32_THREADS, 0, stream>>>(out, (const bf16*)table, ids, hidden, vocab, scale);
    else
        LLMS_REQUIRE(false, "embed_scale: dtype must be 0 (float32) or 1 (bfloat16)");
    LLMS_LAUNCH_CHECK();
}

int llms_rmsnorm32(int dtype, void* out, const float* x, const float* weight, const int* rows, float eps, float offset,
                   int n_out, int hidden, hipStream_t stream) {
    LLMS_REQUIRE(n_out > 0 && hidden > 0, "rmsnorm32: sizes must be positive");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "rmsnorm32: dtype must be 0 (float32) or 1 (bfloat16)");
    if (hidden % 4 == 0 && hidden <= 4 * S32_VEC * S32_THREADS && ((uintptr_t)x % 16) == 0 && ((uintptr_t)weight % 16) == 0) {
        if (dtype == 0)
            rmsnorm32_vec_kernel<float><<<n_out, S32_THREADS, 0, stream>>>((float*)out, x, weight, rows, hidden, eps, offset);
        else
            rmsnorm32_vec_kernel<bf16><<<n_out, S32_THREADS, 0, stream>>>((bf16*)out, x, weight, rows, hidden, eps, offset);
        LLMS_LAUNCH_CHECK();
    }
    if (dtype == 0)
        rmsnorm32_kernel<float><<<n_out, S32_THREADS, 0, stream>>>((float*)out, x, weight, rows, hidden, eps, offset);
    else if (dtype == 1)
        rmsnorm32_kernel<bf16><<<n_out, S32_THREADS, 0, stream>>>((bf16*)out, x, weight, rows, hidden, eps, offset);
    else
        LLMS_REQUIRE(false, "rmsnorm32: dtype must be 0 (float32) or 1 (bfloat16)");
    LLMS_LAUNCH_CHECK();
}

int llms_gated_add(float* x, const float* z, int z_stride, int z_col0, int z_col1, const float* bias0,
                   const float* bias1, const float* y0, int y0_stride, const float* y1, int y1_stride, int n,
                   int hidden, hipStream_t stream) {
    LLMS_REQUIRE(n > 0 && hidden > 0, "gated_add: sizes must be positive");
    LLMS_REQUIRE(y0 || y1, "gated_add: no branch to add");
    LLMS_REQUIRE(z || (z_col0 < 0 && z_col1 < 0), "gated_add: gate columns named without gate products");
    auto aligned = [](const void* p) { return ((uintptr_t)p % 16) == 0; };
    const bool vec = hidden % 4 == 0 && z_stride % 4 == 0 && y0_stride % 4 == 0 && y1_stride % 4 == 0 &&
                     (z_col0 < 0 || z_col0 % 4 == 0) && (z_col1 < 0 || z_col1 % 4 == 0) && aligned(x) && aligned(z) &&
                     aligned(bias0) && aligned(bias1) && aligned(y0) && aligned(y1);
    if (vec) {
        dim3 grid(n, (hidden / 4 + S32_THREADS - 1) / S32_THREADS);
        gated_add_vec_kernel<<<grid, S32_THREADS, 0, stream>>>(x, z, z_stride, z_col0, z_col1, bias0, bias1, y0, y0_stride,
                                                               y1, y1_stride, hidden);
    } else {
        gated_add_kernel<<<n, S32_THREADS, 0, stream>>>(x, z, z_stride, z_col0, z_col1, bias0, bias1, y0, y0_stride, y1,
                                                        y1_stride, hidden);
    }
    LLMS_LAUNCH_CHECK();
}

// 0: launched; 3: the sizes are not what the fused kernel takes (the caller runs gated_add and rmsnorm32 instead)
int llms_gated_add_norm(int dtype, void* out, float* x, const float* z, int z_stride, int z_col0, int z_col1,
                        const float* bias0, const float* bias1, const float* y0, int y0_stride, const float* y1,
                        int y1_stride, const float* weight, float eps, float offset, int n, int hidden, hipStream_t stream) {
    LLMS_REQUIRE(n > 0 && hidden > 0, "gated_add_norm: sizes must be positive");
    LLMS_REQUIRE(y0 || y1, "gated_add_norm: no branch to add");
    LLMS_REQUIRE(z || (z_col0 < 0 && z_col1 < 0), "gated_add_norm: gate columns named without gate products");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "gated_add_norm: dtype must be 0 (float32) or 1 (bfloat16)");
    auto aligned = [](const void* p) { return ((uintptr_t)p % 16) == 0; };
    const bool vec = hidden % 4 == 0 && hidden <= 4 * S32_VEC * S32_THREADS && z_stride % 4 == 0 && y0_stride % 4 == 0 &&
                     y1_stride % 4 == 0 && (z_col0 < 0 || z_col0 % 4 == 0) && (z_col1 < 0 || z_col1 % 4 == 0) &&
                     aligned(x) && aligned(z) && aligned(bias0) && aligned(bias1) && aligned(y0) && aligned(y1) &&
                     aligned(weight);
    if (!vec) return 3;
    if (dtype == 0)
        gated_add_norm_vec_kernel<float><<<n, S32_THREADS, 0, stream>>>((float*)out, x, z, z_stride, z_col0, z_col1, bias0, bias1,
                                                                        y0, y0_stride, y1, y1_stride, weight, hidden, eps, offset);
    else
        gated_add_norm_vec_kernel<bf16><<<n, S32_THREADS, 0, stream>>>((bf16*)out, x, z, z_stride, z_col0, z_col1, bias0, bias1,
                                                                       y0, y0_stride, y1, y1_stride, weight, hidden, eps, offset);
    LLMS_LAUNCH_CHECK();
}

int llms_streams_norm(int dtype, void* out, float* x_dst, const float* x_src, int src_broadcast, const float* y,
                      const float* mix, const float* wout, const float* read, const float* weight, const int* rows,
                      int n_out, int streams, int hidden, float eps, int store, int center, hipStream_t stream) {
    LLMS_REQUIRE(n_out > 0 && hidden > 0, "streams_norm: sizes must be positive");
    LLMS_REQUIRE(streams >= 1 && streams <= STREAMS_MAX, "streams_norm: 1 to 8 streams");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "streams_norm: dtype must be 0 (float32) or 1 (bfloat16)");
    LLMS_REQUIRE(x_src && (x_dst || !store) && (weight || !out), "streams_norm: a needed operand is missing");
    LLMS_REQUIRE((size_t)hidden * 4 <= 96 * 1024, "streams_norm: a row of up to 24,576 elements");
    const size_t lds = (size_t)hidden * sizeof(float);
    auto aligned = [](const void* p) { return ((uintptr_t)p % 16) == 0; };
    const bool vec = hidden % 4 == 0 && aligned(x_dst) && aligned(x_src) && aligned(y) && aligned(weight) && aligned(out);
    // one stream with rows of 256, 512, 1,024, 2,048 or 4,096 numbers: a wave a row, the row in registers
    const int per_lane = hidden % (4 * LLMS_WAVE) == 0 ? hidden / (4 * LLMS_WAVE) : 0;
    if (vec && streams == 1 && (per_lane == 1 || per_lane == 2 || per_lane == 4 || per_lane == 8 || per_lane == 16)) {
        const int per_wg = S32_THREADS / LLMS_WAVE;
        const dim3 grid((n_out + per_wg - 1) / per_wg);
#define WAVE_GO(V)                                                                                                          \
    do {                                                                                                                    \
        if (dtype == 0)                                                                                                     \
            streams_norm_wave_kernel<float, V><<<grid, S32_THREADS, 0, stream>>>((float*)out, x_dst, x_src, y, mix, wout, read, \
                                                                                 weight, rows, n_out, hidden, eps, store, center); \
        else                                                                                                                \
            streams_norm_wave_kernel<bf16, V><<<grid, S32_THREADS, 0, stream>>>((bf16*)out, x_dst, x_src, y, mix, wout, read, \
                                                                                weight, rows, n_out, hidden, eps, store, center); \
    } while (0)
        if (per_lane == 1) WAVE_GO(1);
        else if (per_lane == 2) WAVE_GO(2);
        else if (per_lane == 4) WAVE_GO(4);
        else if (per_lane == 8) WAVE_GO(8);
        else WAVE_GO(16);
#undef WAVE_GO
        LLMS_LAUNCH_CHECK();
    }
#define STREAMS_GO(KERNEL, T)                                                                                               \
    do {                                                                                                                    \
        if (lds > 32 * 1024)                                                                                                \
            LLMS_HIP_CHECK(hipFuncSetAttribute((const void*)KERNEL<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        KERNEL<T><<<n_out, S32_THREADS, lds, stream>>>((T*)out, x_dst, x_src, src_broadcast, y, mix, wout, read, weight, rows, \
                                                       streams, hidden, eps, store, center);                                \
    } while (0)
    if (vec && dtype == 0) STREAMS_GO(streams_norm_vec_kernel, float);
    else if (vec) STREAMS_GO(streams_norm_vec_kernel, bf16);
    else if (dtype == 0) STREAMS_GO(streams_norm_kernel, float);
    else STREAMS_GO(streams_norm_kernel, bf16);
#undef STREAMS_GO
    LLMS_LAUNCH_CHECK();
}

int llms_normed_add_norm(int dtype, void* out, float* x, const float* y, const float* wb, const float* w, const int* rows,
                         int n_out, int hidden, float eps_y, float eps, int store, hipStream_t stream) {
    LLMS_REQUIRE(n_out > 0 && hidden > 0, "normed_add_norm: sizes must be positive");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "normed_add_norm: dtype must be 0 (float32) or 1 (bfloat16)");
    LLMS_REQUIRE(x && (!y || wb) && (!out || w), "normed_add_norm: a needed operand is missing");
    LLMS_REQUIRE((size_t)hidden * 4 <= 128 * 1024, "normed_add_norm: a row of up to 32,768 elements");
    const size_t lds = (size_t)hidden * sizeof(float);
#define NAN_GO(T)                                                                                                         \
    do {                                                                                                                  \
        if (lds > 32 * 1024)                                                                                              \
            LLMS_HIP_CHECK(hipFuncSetAttribute((const void*)normed_add_norm_kernel<T>,                                    \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                    \
        normed_add_norm_kernel<T><<<n_out, S32_THREADS, lds, stream>>>((T*)out, x, y, wb, w, rows, hidden, eps_y, eps, store); \
    } while (0)
    if (dtype == 0) NAN_GO(float);
    else NAN_GO(bf16);
#undef NAN_GO
    LLMS_LAUNCH_CHECK();
}

int llms_add_vector(float* x, const float* v, int n, int hidden, hipStream_t stream) {
    LLMS_REQUIRE(n > 0 && hidden > 0, "add_vector: sizes must be positive");
    add_vector_kernel<<<n, S32_THREADS, 0, stream>>>(x, v, hidden);
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
