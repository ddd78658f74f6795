// Attention over the paged cache whose ingredients are chosen by arguments, for float and bfloat16 storage:
//
//   conv_store    what the q, k, v projection of the new tokens gives (32-bit, [N, Cq + Ck + Cv]) goes through a short
//                 causal convolution per channel (from 2 taps on the request's last taps - 1 projected rows lie in its
//                 state, a ring indexed by position), is rounded once, and lands in the query rows and at the tokens'
//                 cache slots.  taps = 1: a factor per channel; taps = 0: rounding and store alone.
//   conv_state    the ring takes the last taps - 1 projected rows of every request of the step (a kernel of its own,
//                 because a token's write would race with its neighbours' reads; when every request brings one
//                 token, conv_store writes the ring itself).
//   norm_store    the same without a convolution, for queries and keys that are normed head by head: every head of q
//                 and of k is divided by its root mean square over its dk numbers (eps inside the root) and multiplied by a
//                 weight that all heads share (`unit_norm`: no weight); with `freq` the first rot_dims numbers of every
//                 head of q and k are turned by the token's position first (dimension i together with dimension
//                 i + rot_dims / 2, angle position * freq[i]); q is then multiplied by 1 + coef * ln(floor((p + 1) / every) + 1) at
//                 position p (every 0: no factor); all in 32-bit, rounded once, into the query rows and the cache slots.
//   attend        one workgroup per new token, all heads.  Score heads s = h * maps + m (maps = 2: two score maps
//                 per query head over the same values); s reads key head (h / (H / G)) * maps + m, values come from
//                 value head h / (H / G).  A query at position i sees the key j <= i if
//                     j >= chunk_start(i)  and  (i - j < window  or  j < keep_first)
//                 (window 0: no window; chunk 0: no chunks).  score = q . k * scale - slope_h * (i - j) + dist_bias[h, min(i - j,
//                 dist_reach)] (a table per head over the distance, which stays at its last entry beyond dist_reach); softmax over the
//                 visible keys in 32-bit, normalised before anything else happens to it; with `sink` the denominator holds one more term exp(0); optionally the heads' weights
//                 are mixed, w_h = sum_g talk[h, g] w_g; then the values.  maps = 2 ends with o = a_1 - lambda a_2;
//                 head_norm divides a head's result by its root mean square (eps inside the root) and multiplies
//                 by out_scale.  With gate products z (32-bit) the result is multiplied by sigmoid(z[n, h * dv + d]).
//
// Keys are [pages, key heads, block, dk], values [pages, value heads, dv, block] (transposed inside a page).
#include "common.h"

#define AC_THREADS 256
#define AC_WAVES (AC_THREADS / LLMS_WAVE)
#define AC_TILE LLMS_WAVE

// ------------------------------------------------------------------------------------------- conv + store
template <typename T>
__global__ __launch_bounds__(AC_THREADS) void conv_store_kernel(
    T* __restrict__ q_out, int q_stride, const float* __restrict__ proj, int proj_stride, const float* __restrict__ taps_w,
    int taps, const float* __restrict__ state, size_t state_slot_stride, const int* __restrict__ state_slots,
    const int* __restrict__ token_seq, const int* __restrict__ positions, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, T* __restrict__ k_pool, T* __restrict__ v_pool, int cq, int ck, int cv, int k_heads,
    int dk, int v_heads, int dv, int block_size, float* __restrict__ state_out, const int* __restrict__ context_lens) {
    const int n = blockIdx.x;
    const int c = blockIdx.y * AC_THREADS + threadIdx.x;
    const int channels = cq + ck + cv;
    if (c >= channels) return;
    float y;
    if (taps >= 1) {
        const int b = token_seq[n];
        const int p = positions[n];
        const int first_row = cu_seqlens[b];
        const int first_pos = p - (n - first_row);  // position of the portion's first token
        const float* ring = taps > 1 ? state + (size_t)state_slots[b] * state_slot_stride : nullptr;
        y = 0.f;
        for (int j = 0; j < taps; ++j) {
            const int pos = p - (taps - 1) + j;
            float u = 0.f;
            if (pos >= first_pos)
                u = proj[(size_t)(first_row + pos - first_pos) * proj_stride + c];
            else if (pos >= 0)
                u = ring[(size_t)(pos % (taps - 1)) * channels + c];
            y = fmaf(taps_w[(size_t)c * taps + j], u, y);
        }
        // every request brings one token: the ring takes the token's own row here (nobody else reads this request's
        // ring in this launch, and this thread has read the place it overwrites); a request of length 0 is padding
        if (state_out && taps > 1 && context_lens[b] > 0)
            state_out[(size_t)state_slots[b] * state_slot_stride + (size_t)(p % (taps - 1)) * channels + c] =
                proj[(size_t)n * proj_stride + c];
    } else {
        y = proj[(size_t)n * proj_stride + c];
    }
    const T r = from_f32<T>(y);
    if (c < cq) {
        q_out[(size_t)n * q_stride + c] = r;
        return;
    }
    if (!slots) return;
    const int slot = slots[n];
    if (slot < 0) return;
    const int page = slot / block_size, off = slot % block_size;
    if (c < cq + ck) {
        const int kc = c - cq, head = kc / dk, d = kc % dk;
        k_pool[(((size_t)page * k_heads + head) * block_size + off) * dk + d] = r;
    } else {
        const int vc = c - cq - ck, head = vc / dv, d = vc % dv;
        v_pool[(((size_t)page * v_heads + head) * dv + d) * block_size + off] = r;
    }
}

__global__ __launch_bounds__(AC_THREADS) void conv_state_kernel(
    float* __restrict__ state, size_t state_slot_stride, const int* __restrict__ state_slots,
    const float* __restrict__ proj, int proj_stride, const int* __restrict__ cu_seqlens,
    const int* __restrict__ context_lens, int taps, int channels) {
    const int b = blockIdx.x;
    const int c = blockIdx.y * AC_THREADS + threadIdx.x;
    if (c >= channels) return;
    const int first_row = cu_seqlens[b], count = cu_seqlens[b + 1] - first_row;
    const int end = context_lens[b];  // the request's length after this step (0: not a request)
    if (count <= 0 || end <= 0) return;
    const int first_pos = end - count;
    float* ring = state + (size_t)state_slots[b] * state_slot_stride;
    int pos = end - (taps - 1);
    if (pos < first_pos) pos = first_pos;
    for (; pos < end; ++pos)
        ring[(size_t)(pos % (taps - 1)) * channels + c] = proj[(size_t)(first_row + pos - first_pos) * proj_stride + c];
}

// element d of a head after the rotation of its first rot_dims numbers (pairs i, i + rot_dims / 2)
__device__ __forceinline__ float turned_element(const float* __restrict__ src, int d, int rot_dims, float position,
                                                const float* __restrict__ freq) {
    if (d >= rot_dims) return src[d];
    const int h = rot_dims >> 1, i = d < h ? d : d - h;
    const float2 sc = rotary_angle(position, freq[i]);  // (sine, cosine)
    const float2 turned = rotate_pair(src[i], src[i + h], sc.y, sc.x);
    return d < h ? turned.x : turned.y;
}

// grid: (tokens, query heads + key heads + value heads); one wave per head
template <typename T>
__global__ __launch_bounds__(LLMS_WAVE) void norm_store_kernel(
    T* __restrict__ q_out, int q_stride, const float* __restrict__ proj, int proj_stride, const float* __restrict__ q_norm,
    const float* __restrict__ k_norm, float eps, float temp_coef, int temp_every, const int* __restrict__ positions,
    const int* __restrict__ slots, T* __restrict__ k_pool, T* __restrict__ v_pool, int q_heads, int k_heads, int dk,
    int v_heads, int dv, int block_size, const float* __restrict__ freq, int rot_dims, int unit_norm) {
    const int n = blockIdx.x, lane = threadIdx.x;
    int head = blockIdx.y;
    const float* row = proj + (size_t)n * proj_stride;
    if (head < q_heads + k_heads) {
        const bool is_q = head < q_heads;
        const float* src = row + (size_t)head * dk;  // (keys follow the queries)
        const float* w = is_q ? q_norm : k_norm;
        float mul = 1.f;
        const float position = rot_dims > 0 ? (float)positions[n] : 0.f;
        if (w || unit_norm) {
            float ss = 0.f;
            for (int d = lane; d < dk; d += LLMS_WAVE) {
                const float x = rot_dims > 0 ? turned_element(src, d, rot_dims, position, freq) : src[d];
                ss = fmaf(x, x, ss);
            }
            mul = 1.f / sqrtf(wave_sum(ss) / (float)dk + eps);
        }
        float factor = 1.f;
        if (is_q && temp_every > 0) factor = 1.f + temp_coef * logf((float)((positions[n] + 1) / temp_every + 1));
        T* dst;
        if (is_q) {
            dst = q_out + (size_t)n * q_stride + (size_t)head * dk;
        } else {
            if (!slots) return;
            const int slot = slots[n];
            if (slot < 0) return;
            const int page = slot / block_size, off = slot % block_size;
            dst = k_pool + (((size_t)page * k_heads + (head - q_heads)) * block_size + off) * dk;
        }
        for (int d = lane; d < dk; d += LLMS_WAVE) {
            float x = (rot_dims > 0 ? turned_element(src, d, rot_dims, position, freq) : src[d]) * mul;
            if (w) x *= w[d];
            dst[d] = from_f32<T>(x * factor);
        }
        return;
    }
    head -= q_heads + k_heads;
    if (!slots) return;
    const int slot = slots[n];
    if (slot < 0) return;
    const int page = slot / block_size, off = slot % block_size;
    const float* src = row + (size_t)(q_heads + k_heads) * dk + (size_t)head * dv;
    for (int d = lane; d < dv; d += LLMS_WAVE)
        v_pool[(((size_t)page * v_heads + head) * dv + d) * block_size + off] = from_f32<T>(src[d]);
}

// ------------------------------------------------------------------------------------------- attention
struct ComposedArgs {
    int out_stride, q_stride, max_blocks;
    int heads, kv_heads, maps, dk, dv, block_size;
    int window, keep_first, chunk;
    float scale, lambda, eps, out_scale;
    int head_norm;
    const float* dist_bias;  // [heads, dist_reach + 1], or null
    int dist_reach;
    const float* gate;  // 32-bit products [N, gate_stride], or null
    int gate_stride;
    int sink;  // the softmax's denominator holds one more term, exp(0): a key of score zero that has no value
};

template <typename T>
__device__ __forceinline__ float dot_row(const float* __restrict__ q, const T* __restrict__ k, int dk) {
    float acc = 0.f;
    if (dk % 8 == 0) {
        for (int d = 0; d < dk; d += 8) {
            float kv[8];
            if constexpr (sizeof(T) == 2) {
                const uint4 raw = *reinterpret_cast<const uint4*>(k + d);
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    kv[2 * i] = __uint_as_float(w[i] << 16);
                    kv[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
                }
            } else {
                const float4 a = *reinterpret_cast<const float4*>(k + d);
                const float4 b = *reinterpret_cast<const float4*>(k + d + 4);
                kv[0] = a.x, kv[1] = a.y, kv[2] = a.z, kv[3] = a.w, kv[4] = b.x, kv[5] = b.y, kv[6] = b.z, kv[7] = b.w;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = fmaf(q[d + i], kv[i], acc);
        }
    } else {
        for (int d = 0; d < dk; ++d) acc = fmaf(q[d], to_f32(k[d]), acc);
    }
    return acc;
}

template <typename T>
__global__ __launch_bounds__(AC_THREADS) void attend_composed_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int* __restrict__ block_tables, const int* __restrict__ table_rows, const int* __restrict__ token_seq,
    const int* __restrict__ positions, const int* __restrict__ context_lens, const float* __restrict__ slopes,
    const float* __restrict__ talk, ComposedArgs a) {
    extern __shared__ float lds[];
    const int H = a.heads, G = a.kv_heads, S = H * a.maps, dk = a.dk, dv = a.dv, bs = a.block_size;
    float* qs = lds;                      // [S][dk], scaled
    float* stat_m = qs + S * dk;          // [S]
    float* stat_l = stat_m + S;           // [S]
    float* prob = stat_l + S;             // [S][AC_TILE]
    float* mixed = prob + S * AC_TILE;    // [H][AC_TILE] (only with talk)
    float* acc_o = mixed + (talk ? H * AC_TILE : 0);  // [S][dv]
    float* talk_s = acc_o + S * dv;       // [H][H] (only with talk)
    int* key_page = reinterpret_cast<int*>(talk_s + (talk ? H * H : 0));  // [AC_TILE]
    int* key_off = key_page + AC_TILE;    // [AC_TILE]

    const int n = blockIdx.x;
    const int tid = threadIdx.x, wave = tid / LLMS_WAVE, lane = tid % LLMS_WAVE;
    const int p = positions[n];
    const int seq = token_seq[n];
    if (context_lens && context_lens[seq] <= 0) {  // a row of padding: it belongs to no request and has no keys
        for (int i = tid; i < H * dv; i += AC_THREADS) out[(size_t)n * a.out_stride + i] = from_f32<T>(0.f);
        return;
    }
    const int* table = block_tables + (size_t)(table_rows ? table_rows[seq] : seq) * a.max_blocks;

    // the visible keys: [r1_lo, r1_lo + n1) (kept first keys that the window has passed) and [r2_lo, p]
    const int lo_chunk = a.chunk > 0 ? p / a.chunk * a.chunk : 0;
    const int lo_win = (a.window > 0 && p - a.window + 1 > 0) ? p - a.window + 1 : 0;
    const int r2_lo = lo_chunk > lo_win ? lo_chunk : lo_win;
    const int r1_lo = lo_chunk;
    int r1_hi = a.keep_first < lo_win ? a.keep_first : lo_win;
    const int n1 = r1_hi > r1_lo ? r1_hi - r1_lo : 0;
    const int n_vis = n1 + (p - r2_lo + 1);
    const int group = H / G;

    const T* qrow = q + (size_t)n * a.q_stride;
    for (int i = tid; i < S * dk; i += AC_THREADS) qs[i] = to_f32(qrow[i]) * a.scale;
    for (int i = tid; i < S * dv; i += AC_THREADS) acc_o[i] = 0.f;
    if (talk)
        for (int i = tid; i < H * H; i += AC_THREADS) talk_s[i] = talk[i];
    __syncthreads();

    // pass 1: every score head's maximum and sum over the visible keys
    for (int s = wave; s < S; s += AC_WAVES) {
        const int h = s / a.maps, kh = (h / group) * a.maps + s % a.maps;
        const float slope = slopes ? slopes[h] : 0.f;
        float m = -INFINITY, l = 0.f;
        for (int v0 = 0; v0 < n_vis; v0 += AC_TILE) {
            const int v = v0 + lane;
            float sc = -INFINITY;
            if (v < n_vis) {
                const int j = v < n1 ? r1_lo + v : r2_lo + (v - n1);
                const int page = table[j / bs], off = j % bs;
                const T* kr = k_pool + (((size_t)page * (G * a.maps) + kh) * bs + off) * dk;
                sc = dot_row<T>(qs + s * dk, kr, dk) - slope * (float)(p - j);
                if (a.dist_bias) sc += a.dist_bias[(size_t)h * (a.dist_reach + 1) + min(p - j, a.dist_reach)];
            }
            const float m_new = fmaxf(m, wave_max(sc));
            const float e = v < n_vis ? expf(sc - m_new) : 0.f;
            l = l * expf(m - m_new) + wave_sum(e);
            m = m_new;
        }
        if (a.sink) {
            const float m_new = fmaxf(m, 0.f);
            l = l * expf(m - m_new) + expf(-m_new);
            m = m_new;
        }
        if (lane == 0) {
            stat_m[s] = m;
            stat_l[s] = l;
        }
    }
    __syncthreads();

    // pass 2: normalised weights tile by tile, mixed over heads if asked for, then the values
    for (int v0 = 0; v0 < n_vis; v0 += AC_TILE) {
        const int v = v0 + lane;
        const int count = n_vis - v0 < AC_TILE ? n_vis - v0 : AC_TILE;
        int j = 0, page = 0, off = 0;
        if (v < n_vis) {
            j = v < n1 ? r1_lo + v : r2_lo + (v - n1);
            page = table[j / bs];
            off = j % bs;
        }
        if (wave == 0) {
            key_page[lane] = page;
            key_off[lane] = off;
        }
        for (int s = wave; s < S; s += AC_WAVES) {
            const int h = s / a.maps, kh = (h / group) * a.maps + s % a.maps;
            float w = 0.f;
            if (v < n_vis) {
                const float slope = slopes ? slopes[h] : 0.f;
                const T* kr = k_pool + (((size_t)page * (G * a.maps) + kh) * bs + off) * dk;
                float sc = dot_row<T>(qs + s * dk, kr, dk) - slope * (float)(p - j);
                if (a.dist_bias) sc += a.dist_bias[(size_t)h * (a.dist_reach + 1) + min(p - j, a.dist_reach)];
                w = expf(sc - stat_m[s]) / stat_l[s];
            }
            prob[s * AC_TILE + lane] = w;
        }
        __syncthreads();
        const float* weights = prob;
        if (talk) {
            for (int i = tid; i < H * AC_TILE; i += AC_THREADS) {
                const int h = i / AC_TILE, jj = i % AC_TILE;
                float t = 0.f;
                for (int g = 0; g < H; ++g) t = fmaf(talk_s[h * H + g], prob[g * AC_TILE + jj], t);
                mixed[i] = t;
            }
            __syncthreads();
            weights = mixed;
        }
        for (int s = wave; s < S; s += AC_WAVES) {
            const int vh = (s / a.maps) / group;
            for (int d = lane; d < dv; d += LLMS_WAVE) {
                float o = acc_o[s * dv + d];
                for (int jj = 0; jj < count; ++jj) {
                    const T* vr = v_pool + (((size_t)key_page[jj] * G + vh) * dv + d) * bs + key_off[jj];
                    o = fmaf(weights[s * AC_TILE + jj], to_f32(*vr), o);
                }
                acc_o[s * dv + d] = o;
            }
        }
        __syncthreads();
    }

    // what leaves: per query head, the two maps combined and the head normed where asked for
    T* orow = out + (size_t)n * a.out_stride;
    for (int h = wave; h < H; h += AC_WAVES) {
        float ss = 0.f;
        for (int d = lane; d < dv; d += LLMS_WAVE) {
            float o = acc_o[(h * a.maps) * dv + d];
            if (a.maps == 2) o -= a.lambda * acc_o[(h * 2 + 1) * dv + d];
            ss = fmaf(o, o, ss);
        }
        float mul = 1.f;
        if (a.head_norm) mul = a.out_scale / sqrtf(wave_sum(ss) / (float)dv + a.eps);
        for (int d = lane; d < dv; d += LLMS_WAVE) {
            float o = acc_o[(h * a.maps) * dv + d];
            if (a.maps == 2) o -= a.lambda * acc_o[(h * 2 + 1) * dv + d];
            o *= mul;
            if (a.gate) o /= 1.f + expf(-a.gate[(size_t)n * a.gate_stride + h * dv + d]);
            orow[h * dv + d] = from_f32<T>(o);
        }
    }
}

static size_t composed_lds_bytes(int heads, int maps, int dk, int dv, bool talk) {
    const size_t S = (size_t)heads * maps;
    size_t floats = S * dk + 2 * S + S * AC_TILE + S * dv;
    if (talk) floats += (size_t)heads * AC_TILE + (size_t)heads * heads;
    return floats * sizeof(float) + 2 * AC_TILE * sizeof(int);
}

extern "C" {

int llms_conv_store(int dtype, void* q_out, int q_stride, const float* proj, int proj_stride, const float* taps_w, int taps,
                    const float* state, size_t state_slot_stride, const int* state_slots, const int* token_seq,
                    const int* positions, const int* cu_seqlens, const int* slots, void* k_pool, void* v_pool, int n_tokens,
                    int cq, int ck, int cv, int k_heads, int dk, int v_heads, int dv, int block_size, float* state_out,
                    const int* context_lens, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && cq > 0 && ck >= 0 && cv >= 0, "conv_store: sizes must be positive");
    LLMS_REQUIRE(ck == k_heads * dk && cv == v_heads * dv, "conv_store: channels do not match heads times sizes");
    LLMS_REQUIRE(taps < 1 || (taps_w && token_seq && positions && cu_seqlens),
                 "conv_store: a convolution needs its taps and the batch's arrays");
    LLMS_REQUIRE(taps <= 1 || (state && state_slots), "conv_store: a convolution of two taps or more needs the state");
    LLMS_REQUIRE(!slots || (k_pool && v_pool && block_size > 0), "conv_store: slots given without pools");
    LLMS_REQUIRE(!state_out || (context_lens && state_out == state), "conv_store: the ring is updated in place, with the requests' lengths at hand");
    dim3 grid(n_tokens, (cq + ck + cv + AC_THREADS - 1) / AC_THREADS);
    if (dtype == 0)
        conv_store_kernel<float><<<grid, AC_THREADS, 0, stream>>>(
            (float*)q_out, q_stride, proj, proj_stride, taps_w, taps, state, state_slot_stride, state_slots, token_seq,
            positions, cu_seqlens, slots, (float*)k_pool, (float*)v_pool, cq, ck, cv, k_heads, dk, v_heads, dv, block_size,
            state_out, context_lens);
    else if (dtype == 1)
        conv_store_kernel<bf16><<<grid, AC_THREADS, 0, stream>>>(
            (bf16*)q_out, q_stride, proj, proj_stride, taps_w, taps, state, state_slot_stride, state_slots, token_seq,
            positions, cu_seqlens, slots, (bf16*)k_pool, (bf16*)v_pool, cq, ck, cv, k_heads, dk, v_heads, dv, block_size,
            state_out, context_lens);
    else
        LLMS_REQUIRE(false, "conv_store: dtype must be 0 (float32) or 1 (bfloat16)");
    LLMS_LAUNCH_CHECK();
}

int llms_norm_store(int dtype, void* q_out, int q_stride, const float* proj, int proj_stride, const float* q_norm,
                    const float* k_norm, float eps, float temp_coef, int temp_every, const int* positions, const int* slots,
                    void* k_pool, void* v_pool, int n_tokens, int q_heads, int k_heads, int dk, int v_heads, int dv,
                    int block_size, const float* freq, int rot_dims, int unit_norm, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && q_heads > 0 && k_heads >= 0 && v_heads >= 0 && dk > 0 && dv > 0, "norm_store: sizes must be positive");
    LLMS_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dk && (rot_dims == 0 || (freq && positions)),
                 "norm_store: an even number of turned dimensions within a head, with frequencies and positions");
    LLMS_REQUIRE(temp_every == 0 || positions, "norm_store: a factor by position needs the positions");
    LLMS_REQUIRE(!slots || (k_pool && v_pool && block_size > 0), "norm_store: slots given without pools");
    LLMS_REQUIRE(q_heads + k_heads + v_heads <= 65535, "norm_store: up to 65,535 heads in all");
    dim3 grid(n_tokens, q_heads + k_heads + v_heads);
    if (dtype == 0)
        norm_store_kernel<float><<<grid, LLMS_WAVE, 0, stream>>>((float*)q_out, q_stride, proj, proj_stride, q_norm, k_norm, eps,
                                                                 temp_coef, temp_every, positions, slots, (float*)k_pool,
                                                                 (float*)v_pool, q_heads, k_heads, dk, v_heads, dv, block_size,
                                                                 freq, rot_dims, unit_norm);
    else if (dtype == 1)
        norm_store_kernel<bf16><<<grid, LLMS_WAVE, 0, stream>>>((bf16*)q_out, q_stride, proj, proj_stride, q_norm, k_norm, eps,
                                                                temp_coef, temp_every, positions, slots, (bf16*)k_pool,
                                                                (bf16*)v_pool, q_heads, k_heads, dk, v_heads, dv, block_size,
                                                                freq, rot_dims, unit_norm);
    else
        LLMS_REQUIRE(false, "norm_store: dtype must be 0 (float32) or 1 (bfloat16)");
    LLMS_LAUNCH_CHECK();
}

int llms_conv_state(float* state, size_t state_slot_stride, const int* state_slots, const float* proj, int proj_stride,
                    const int* cu_seqlens, const int* context_lens, int n_seqs, int taps, int channels,
                    hipStream_t stream) {
    LLMS_REQUIRE(n_seqs > 0 && taps > 1 && channels > 0, "conv_state: sizes must be positive and taps at least 2");
    dim3 grid(n_seqs, (channels + AC_THREADS - 1) / AC_THREADS);
    conv_state_kernel<<<grid, AC_THREADS, 0, stream>>>(state, state_slot_stride, state_slots, proj, proj_stride, cu_seqlens,
                                                       context_lens, taps, channels);
    LLMS_LAUNCH_CHECK();
}

int llms_attend_composed(int dtype, void* out, int out_stride, const void* q, int q_stride, const void* k_pool,
                         const void* v_pool, const int* block_tables, const int* table_rows, int max_blocks,
                         const int* token_seq, const int* positions, const int* context_lens, int n_tokens, int heads,
                         int kv_heads, int maps,
                         int dk, int dv, int block_size, int window, int keep_first, int chunk, float scale,
                         const float* slopes, const float* talk, float lambda, int head_norm, float eps, float out_scale,
                         const float* dist_bias, int dist_reach, const float* gate, int gate_stride, int sink,
                         hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && heads > 0 && kv_heads > 0 && dk > 0 && dv > 0, "attend_composed: sizes must be positive");
    LLMS_REQUIRE(!dist_bias || dist_reach >= 0, "attend_composed: a distance table has at least one entry per head");
    LLMS_REQUIRE(heads % kv_heads == 0, "attend_composed: heads must be a multiple of kv_heads");
    LLMS_REQUIRE(maps == 1 || maps == 2, "attend_composed: one or two score maps");
    LLMS_REQUIRE(!(talk && maps != 1), "attend_composed: mixing heads' weights goes with one score map");
    LLMS_REQUIRE(block_size > 0 && max_blocks > 0, "attend_composed: block_size and max_blocks must be positive");
    LLMS_REQUIRE(window >= 0 && keep_first >= 0 && chunk >= 0, "attend_composed: window, keep_first and chunk are >= 0");
    const size_t lds = composed_lds_bytes(heads, maps, dk, dv, talk != nullptr);
    LLMS_REQUIRE(lds <= 160 * 1024, "attend_composed: heads times sizes do not fit the 160 KB of LDS");
    ComposedArgs a;
    a.out_stride = out_stride, a.q_stride = q_stride, a.max_blocks = max_blocks;
    a.heads = heads, a.kv_heads = kv_heads, a.maps = maps, a.dk = dk, a.dv = dv, a.block_size = block_size;
    a.window = window, a.keep_first = keep_first, a.chunk = chunk;
    a.scale = scale, a.lambda = lambda, a.eps = eps, a.out_scale = out_scale, a.head_norm = head_norm;
    a.dist_bias = dist_bias, a.dist_reach = dist_reach, a.gate = gate, a.gate_stride = gate_stride, a.sink = sink;
    if (dtype == 0) {
        auto kernel = attend_composed_kernel<float>;
        if (lds > 48 * 1024)
            LLMS_HIP_CHECK(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        kernel<<<n_tokens, AC_THREADS, lds, stream>>>((float*)out, (const float*)q, (const float*)k_pool,
                                                      (const float*)v_pool, block_tables, table_rows, token_seq, positions,
                                                      context_lens, slopes, talk, a);
    } else if (dtype == 1) {
        auto kernel = attend_composed_kernel<bf16>;
        if (lds > 48 * 1024)
            LLMS_HIP_CHECK(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        kernel<<<n_tokens, AC_THREADS, lds, stream>>>((bf16*)out, (const bf16*)q, (const bf16*)k_pool, (const bf16*)v_pool,
                                                      block_tables, table_rows, token_seq, positions, context_lens, slopes, talk,
                                                      a);
    } else {
        LLMS_REQUIRE(false, "attend_composed: dtype must be 0 (float32) or 1 (bfloat16)");
    }
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
