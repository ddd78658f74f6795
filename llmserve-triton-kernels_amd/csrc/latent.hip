// Attention through a latent: a token keeps one row [c ; kr] of r + dr numbers for all heads (c the normed latent
// that keys and values are projected from, kr one rotated key part that all heads share).  With the keys' projection
// folded into the query, q'_h = [W_uk_h^T q_h ; qr_h], head h's score against key j is q'_h . [c_j ; kr_j] and its
// result the softmax-weighted sum of c_j, which the caller projects to values afterwards.
//
//   latent_prepare   from the 32-bit input products z of a step's tokens: cq = rms_unit(z_q) * wq (rounded once);
//                    c = rms_unit(z_c) * wc and kr = rotated z_kr stored at the token's cache row
//   latent_query     from the 32-bit queries [N, H, dn + dr]: the unrotated parts side by side [N, H, dn] and the
//                    rotated parts turned into q'[n, h, r ..]
//   attend_latent    out[n, h, :r] = sum_j softmax_j(q'[n, h] . row_j * scale) c_j over the keys the window allows
//
// Rotation: pairs (2i, 2i+1) of the first `dims` numbers of the rotated part (`half`: pairs (i, i + dims/2) instead),
// angle position * freq[i], the rest of the part passes.  Norms, angles, scores, softmax and sums are 32-bit; T (float or bfloat16) is what is stored.
#include "common.h"

#define LAT_THREADS 256

__device__ __forceinline__ float rotated_element(const float* __restrict__ part, int e, int dims, float position,
                                                 const float* __restrict__ freq, int half = 0) {
    if (e >= dims) return part[e];
    if (half) {  // dimension i turns together with dimension i + dims / 2
        const int h = dims >> 1, i = e < h ? e : e - h;
        const float2 sc = rotary_angle(position, freq[i]);
        const float2 turned = rotate_pair(part[i], part[i + h], sc.y, sc.x);
        return e < h ? turned.x : turned.y;
    }
    const int i = e >> 1;
    const float2 sc = rotary_angle(position, freq[i]);  // (sine, cosine)
    const float2 turned = rotate_pair(part[2 * i], part[2 * i + 1], sc.y, sc.x);
    return (e & 1) ? turned.y : turned.x;
}

// grid: tokens.  z [N, z_ld] float: columns col_q .. + q_rank are the query latent, col_c .. + r + dr the key/value
// latent and the rotated key part (col_c < 0: the layer keeps none).  pool [rows, r + dr] rows at slots[n] (< 0: none).
template <typename T>
__global__ __launch_bounds__(LAT_THREADS) void latent_prepare_kernel(
    T* __restrict__ cq, T* __restrict__ pool, const float* __restrict__ z, int z_ld, int col_q, int q_rank, int col_c,
    int r, int dr, const float* __restrict__ wq, const float* __restrict__ wc, const float* __restrict__ freq, int dims,
    const int* __restrict__ positions, const int* __restrict__ slots, float eps, int half) {
    __shared__ float red[16];
    const int n = blockIdx.x;
    const float* zr = z + (size_t)n * z_ld;
    if (q_rank > 0) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < q_rank; c += LAT_THREADS) ss = fmaf(zr[col_q + c], zr[col_q + c], ss);
        const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)q_rank + eps);
        for (int c = threadIdx.x; c < q_rank; c += LAT_THREADS)
            cq[(size_t)n * q_rank + c] = from_f32<T>(zr[col_q + c] * inv * wq[c]);
    }
    if (col_c < 0) return;
    float ss = 0.f;
    for (int c = threadIdx.x; c < r; c += LAT_THREADS) ss = fmaf(zr[col_c + c], zr[col_c + c], ss);
    const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)r + eps);
    const int slot = slots ? slots[n] : -1;
    if (slot < 0) return;
    T* row = pool + (size_t)slot * (r + dr);
    for (int c = threadIdx.x; c < r; c += LAT_THREADS) row[c] = from_f32<T>(zr[col_c + c] * inv * wc[c]);
    const float position = (float)positions[n];
    for (int e = threadIdx.x; e < dr; e += LAT_THREADS)
        row[r + e] = from_f32<T>(rotated_element(zr + col_c + r, e, dims, position, freq, half));
}

// grid: tokens.  q [N, H, dn + dr] float -> plain [N, H, dn] and folded[n, h, r + e] (row length H * (r + dr)).
template <typename T>
__global__ __launch_bounds__(LAT_THREADS) void latent_query_kernel(
    T* __restrict__ plain, T* __restrict__ folded, const float* __restrict__ q, int heads, int dn, int dr, int r,
    const float* __restrict__ freq, int dims, const int* __restrict__ positions, int half_pairs) {
    const int n = blockIdx.x, dq = dn + dr;
    const float position = (float)positions[n];
    const float* qr = q + (size_t)n * heads * dq;
    if (dn % 2 == 0 && dr % 2 == 0 && !half_pairs) {  // a thread takes two neighbours: a pair of the rotation has one sine and cosine
        const int half = dq / 2;
        for (int i = threadIdx.x; i < heads * half; i += LAT_THREADS) {
            const int h = i / half, e = 2 * (i - h * half);
            const float a = qr[h * dq + e], b = qr[h * dq + e + 1];
            if (e < dn) {
                T* dst = plain + ((size_t)n * heads + h) * dn + e;
                dst[0] = from_f32<T>(a), dst[1] = from_f32<T>(b);
            } else {
                T* dst = folded + ((size_t)n * heads + h) * (r + dr) + r + (e - dn);
                float2 turned = make_float2(a, b);
                if (e - dn < dims) {
                    const float2 sc = rotary_angle(position, freq[(e - dn) >> 1]);
                    turned = rotate_pair(a, b, sc.y, sc.x);
                }
                dst[0] = from_f32<T>(turned.x), dst[1] = from_f32<T>(turned.y);
            }
        }
        return;
    }
    for (int i = threadIdx.x; i < heads * dq; i += LAT_THREADS) {
        const int h = i / dq, e = i - h * dq;
        if (e < dn)
            plain[((size_t)n * heads + h) * dn + e] = from_f32<T>(qr[i]);
        else
            folded[((size_t)n * heads + h) * (r + dr) + r + (e - dn)] =
                from_f32<T>(rotated_element(qr + h * dq + dn, e - dn, dims, position, freq, half_pairs));
    }
}

// What a lane holds of a row of up to 64 * LAT_PER_LANE numbers: elements lane, lane + 64, ...
#define LAT_PER_LANE 16
#define LAT_WAVES (LAT_THREADS / LLMS_WAVE)

// grid (tokens, heads); the workgroup's 4 waves take the keys j with j % 4 == wave, each with a running softmax, and
// meet in LDS.  Which keys a wave takes, and in which order, depends on the token's position alone.
template <typename T>
__global__ __launch_bounds__(LAT_THREADS) void attend_latent_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ pool, const int* __restrict__ tables,
    int table_width, const int* __restrict__ table_rows, const int* __restrict__ token_seq,
    const int* __restrict__ positions, const int* __restrict__ context_lens, int heads, int r, int dr, int block_size,
    int window, float scale) {
    extern __shared__ float lds[];  // per wave: r sums, maximum, sum of weights
    const int n = blockIdx.x, h = blockIdx.y, dk = r + dr;
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    const int seq = token_seq[n], pos = positions[n];
    T* orow = out + ((size_t)n * heads + h) * r;
    if (context_lens[seq] <= pos) {  // (a padding row: a request without keys)
        for (int c = threadIdx.x; c < r; c += LAT_THREADS) orow[c] = from_f32<T>(0.f);
        return;
    }
    const int* table = tables + (size_t)(table_rows ? table_rows[seq] : seq) * table_width;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    float qv[LAT_PER_LANE], acc[LAT_PER_LANE];
    const T* qrow = q + ((size_t)n * heads + h) * dk;
#pragma unroll
    for (int i = 0; i < LAT_PER_LANE; ++i) {
        const int e = lane + i * LLMS_WAVE;
        qv[i] = e < dk ? to_f32(qrow[e]) : 0.f;
        acc[i] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    int j = lo + ((wave - lo) % LAT_WAVES + LAT_WAVES) % LAT_WAVES;  // the first key >= lo with j % 4 == wave
    for (; j <= pos; j += LAT_WAVES) {
        const int page = table[j / block_size];
        const T* krow = pool + ((size_t)page * block_size + j % block_size) * dk;
        float kv[LAT_PER_LANE];
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < LAT_PER_LANE; ++i) {
            const int e = lane + i * LLMS_WAVE;
            kv[i] = e < dk ? to_f32(krow[e]) : 0.f;
            dot = fmaf(qv[i], kv[i], dot);
        }
        const float s = wave_sum(dot) * scale;
        const float m_new = fmaxf(m, s);
        const float fix = expf(m - m_new), p = expf(s - m_new);
        l = l * fix + p;
#pragma unroll
        for (int i = 0; i < LAT_PER_LANE; ++i) acc[i] = fmaf(p, kv[i], acc[i] * fix);
        m = m_new;
    }
    float* mine = lds + (size_t)wave * (r + 2);
#pragma unroll
    for (int i = 0; i < LAT_PER_LANE; ++i) {
        const int e = lane + i * LLMS_WAVE;
        if (e < r) mine[e] = acc[i];
    }
    if (lane == 0) {
        mine[r] = m;
        mine[r + 1] = l;
    }
    __syncthreads();
    float top = -INFINITY;
#pragma unroll
    for (int w = 0; w < LAT_WAVES; ++w) top = fmaxf(top, lds[(size_t)w * (r + 2) + r]);
    float f[LAT_WAVES], total = 0.f;
#pragma unroll
    for (int w = 0; w < LAT_WAVES; ++w) {
        f[w] = expf(lds[(size_t)w * (r + 2) + r] - top);  // (a wave without keys: exp(-inf) = 0)
        total = fmaf(lds[(size_t)w * (r + 2) + r + 1], f[w], total);
    }
    const float inv = 1.0f / total;
    for (int c = threadIdx.x; c < r; c += LAT_THREADS) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < LAT_WAVES; ++w) v = fmaf(lds[(size_t)w * (r + 2) + c], f[w], v);
        orow[c] = from_f32<T>(v * inv);
    }
}

extern "C" {

int llms_latent_prepare(int dtype, void* cq, void* pool, const float* z, int z_ld, int col_q, int q_rank, int col_c, int r,
                        int dr, const float* wq, const float* wc, const float* freq, int dims, const int* positions,
                        const int* slots, float eps, int n, int half_pairs, hipStream_t stream) {
    LLMS_REQUIRE(n > 0 && r > 0 && dr >= 0 && q_rank >= 0, "latent_prepare: sizes must be positive");
    LLMS_REQUIRE(dims >= 0 && dims <= dr && dims % 2 == 0, "latent_prepare: an even number of turned dimensions within the part");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "latent_prepare: dtype must be 0 (float32) or 1 (bfloat16)");
    if (dtype == 0)
        latent_prepare_kernel<float><<<n, LAT_THREADS, 0, stream>>>((float*)cq, (float*)pool, z, z_ld, col_q, q_rank, col_c, r, dr,
                                                                    wq, wc, freq, dims, positions, slots, eps, half_pairs);
    else
        latent_prepare_kernel<bf16><<<n, LAT_THREADS, 0, stream>>>((bf16*)cq, (bf16*)pool, z, z_ld, col_q, q_rank, col_c, r, dr,
                                                                   wq, wc, freq, dims, positions, slots, eps, half_pairs);
    LLMS_LAUNCH_CHECK();
}

int llms_latent_query(int dtype, void* plain, void* folded, const float* q, int heads, int dn, int dr, int r,
                      const float* freq, int dims, const int* positions, int n, int half_pairs, hipStream_t stream) {
    LLMS_REQUIRE(n > 0 && heads > 0 && dn > 0 && dr >= 0 && r > 0, "latent_query: sizes must be positive");
    LLMS_REQUIRE(dims >= 0 && dims <= dr && dims % 2 == 0, "latent_query: an even number of turned dimensions within the part");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "latent_query: dtype must be 0 (float32) or 1 (bfloat16)");
    if (dtype == 0)
        latent_query_kernel<float><<<n, LAT_THREADS, 0, stream>>>((float*)plain, (float*)folded, q, heads, dn, dr, r, freq, dims,
                                                                  positions, half_pairs);
    else
        latent_query_kernel<bf16><<<n, LAT_THREADS, 0, stream>>>((bf16*)plain, (bf16*)folded, q, heads, dn, dr, r, freq, dims,
                                                                 positions, half_pairs);
    LLMS_LAUNCH_CHECK();
}

int llms_attend_latent(int dtype, void* out, const void* q, const void* pool, const int* tables, int table_width,
                       const int* table_rows, const int* token_seq, const int* positions, const int* context_lens, int n,
                       int heads, int r, int dr, int block_size, int window, float scale, hipStream_t stream) {
    LLMS_REQUIRE(n > 0 && heads > 0 && r > 0 && dr >= 0 && block_size > 0 && table_width > 0, "attend_latent: sizes must be positive");
    LLMS_REQUIRE(r + dr <= LLMS_WAVE * LAT_PER_LANE, "attend_latent: a cache row of up to 1,024 numbers");
    LLMS_REQUIRE(heads <= 65535, "attend_latent: too many heads for one launch");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "attend_latent: dtype must be 0 (float32) or 1 (bfloat16)");
    const size_t lds = (size_t)LAT_WAVES * (r + 2) * sizeof(float);
    dim3 grid(n, heads);
    if (dtype == 0)
        attend_latent_kernel<float><<<grid, LAT_THREADS, lds, stream>>>((float*)out, (const float*)q, (const float*)pool, tables,
                                                                        table_width, table_rows, token_seq, positions,
                                                                        context_lens, heads, r, dr, block_size, window, scale);
    else
        attend_latent_kernel<bf16><<<grid, LAT_THREADS, lds, stream>>>((bf16*)out, (const bf16*)q, (const bf16*)pool, tables,
                                                                       table_width, table_rows, token_seq, positions,
                                                                       context_lens, heads, r, dr, block_size, window, scale);
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
