// Linear attention with a fixed decay per head and no softmax or denominator, over a state of fixed size per request:
//     S_t = decay_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t        (S is [dk, dv] per head, 32-bit, zero before position 0)
//
//   decay_prepare   the projection of the new tokens (32-bit, [N, columns] with q, k, v side by side, head by head) is made
//                   ready in place: an activation on q, k and v (SiLU or none), a rotation of q and k by position
//                   (dimension i < dims/2 of a head is turned together with dimension i + dims/2, by position * freq[i];
//                   the rest passes), a factor on k.
//   decay_scan      the recurrence token by token: a workgroup owns 64 columns of one head's state of one request, walks
//                   the request's new tokens from the stored state (from zero if the portion starts at position 0) and
//                   stores the state it ends with.  Any portion, down to one token; the decode kernel.
//   decay_chunks    the same for portions of many tokens, in three launches: every run of DA_CHUNK tokens first gathers
//                   its own sum_t decay^(C-1-t) k_t v_t^T, a scan over the runs turns those into the state before each run
//                   (and stores the request's last state), and every run then adds what its own tokens see of each other,
//                   (q_t . k_s) decay^(t-s) for s <= t, to decay^(t+1) S_before^T q_t.
//   decay_finish    what leaves a token: each head's o divided by its own root mean square (mode 0), or all heads together
//                   RMS-normed with a weight (mode 1); times sigmoid or SiLU of the gate's product; rounded once.
//
// Everything here is 32-bit; only what decay_finish stores is rounded to the model's number format.
#include "common.h"

#define DA_THREADS 256
#define DA_COLS 64  // columns of the state a workgroup of the scan owns
#define DA_ROWGROUPS (DA_THREADS / DA_COLS)

#define DA_ACT_NONE 0
#define DA_ACT_SILU 1
#define DA_ACT_SIGMOID 2

__device__ __forceinline__ float da_silu(float z) { return z / (1.f + expf(-z)); }

// grid: (tokens, heads)
__global__ __launch_bounds__(DA_THREADS) void decay_prepare_kernel(
    float* __restrict__ proj, int stride, int col_q, int col_k, int col_v, const int* __restrict__ positions,
    const float* __restrict__ freq, int rot_dims, int heads, int dk, int dv, int act, float key_scale) {
    const int n = blockIdx.x, h = blockIdx.y;
    float* row = proj + (size_t)n * stride;
    float* q = row + col_q + h * dk;
    float* k = row + col_k + h * dk;
    float* v = row + col_v + h * dv;
    const int half = rot_dims / 2;
    const float position = rot_dims > 0 ? (float)positions[n] : 0.f;  // (no rotation: no positions are handed over)
    // dimensions [0, half) carry their partner half places on; dimensions from rot_dims on stand alone
    for (int i = threadIdx.x; i < dk; i += DA_THREADS) {
        if (i >= half && i < rot_dims) continue;  // (done by its partner)
        const bool turned = i < half;
        float qa = q[i], ka = k[i], qb = 0.f, kb = 0.f;
        if (turned) qb = q[i + half], kb = k[i + half];
        if (act == DA_ACT_SILU) {
            qa = da_silu(qa), ka = da_silu(ka);
            if (turned) qb = da_silu(qb), kb = da_silu(kb);
        }
        if (turned) {
            const float2 sc = rotary_angle(position, freq[i]);  // (sine, cosine)
            const float2 qr = rotate_pair(qa, qb, sc.y, sc.x), kr = rotate_pair(ka, kb, sc.y, sc.x);
            q[i] = qr.x, q[i + half] = qr.y;
            k[i] = kr.x * key_scale, k[i + half] = kr.y * key_scale;
        } else {
            q[i] = qa;
            k[i] = ka * key_scale;
        }
    }
    if (act == DA_ACT_SILU)
        for (int i = threadIdx.x; i < dv; i += DA_THREADS) v[i] = da_silu(v[i]);
}

// grid: (ceil(dv / 64), heads, requests).  Thread (r, j): column 64 * slice + j, rows r, r + 4, ... (RPT of them).
template <int RPT>
__global__ __launch_bounds__(DA_THREADS) void decay_scan_kernel(
    float* __restrict__ out, int out_stride, const float* __restrict__ proj, int stride, int col_q, int col_k, int col_v,
    float* __restrict__ state, const int* __restrict__ state_slots, const int* __restrict__ cu_seqlens,
    const int* __restrict__ context_lens, const float* __restrict__ decay, int heads, int dk, int dv) {
    __shared__ float qk[2][4 * RPT * 2];
    __shared__ float part[2][DA_ROWGROUPS][DA_COLS];
    const int b = blockIdx.z, h = blockIdx.y;
    const int j = threadIdx.x % DA_COLS, r = threadIdx.x / DA_COLS;
    const int c = blockIdx.x * DA_COLS + j;
    const int row0 = cu_seqlens[b], count = cu_seqlens[b + 1] - row0, length = context_lens[b];
    if (length <= 0 || count <= 0) {  // padding: no request, no state; its rows (if any) leave zeros
        if (r == 0 && c < dv)
            for (int t = 0; t < count; ++t) out[(size_t)(row0 + t) * out_stride + h * dv + c] = 0.f;
        return;
    }
    const float d = decay[h];
    float* st = state + (((size_t)state_slots[b] * heads + h) * dk) * dv;
    float s[RPT];
#pragma unroll
    for (int u = 0; u < RPT; ++u) {
        const int i = r + DA_ROWGROUPS * u;
        s[u] = (length > count && i < dk && c < dv) ? st[(size_t)i * dv + c] : 0.f;  // (a portion from position 0 starts from zero)
    }
    for (int t = 0; t < count; ++t) {
        const float* row = proj + (size_t)(row0 + t) * stride;
        float* buf = qk[t & 1];
        for (int i = threadIdx.x; i < 2 * dk; i += DA_THREADS)
            buf[i] = i < dk ? row[col_q + h * dk + i] : row[col_k + h * dk + (i - dk)];
        const float v = c < dv ? row[col_v + h * dv + c] : 0.f;
        __syncthreads();
        // (the sums of the token before, left in the other buffer, are added up behind this barrier)
        if (t > 0 && r == 0 && c < dv) {
            const float(*p)[DA_COLS] = part[(t - 1) & 1];
            out[(size_t)(row0 + t - 1) * out_stride + h * dv + c] = (p[0][j] + p[1][j]) + (p[2][j] + p[3][j]);
        }
        float o = 0.f;
#pragma unroll
        for (int u = 0; u < RPT; ++u) {
            const int i = r + DA_ROWGROUPS * u;
            if (i < dk) {
                s[u] = fmaf(d, s[u], buf[dk + i] * v);
                o = fmaf(s[u], buf[i], o);
            }
        }
        part[t & 1][r][j] = o;
    }
    __syncthreads();
    if (r == 0 && c < dv) {
        const float(*p)[DA_COLS] = part[(count - 1) & 1];
        out[(size_t)(row0 + count - 1) * out_stride + h * dv + c] = (p[0][j] + p[1][j]) + (p[2][j] + p[3][j]);
    }
#pragma unroll
    for (int u = 0; u < RPT; ++u) {
        const int i = r + DA_ROWGROUPS * u;
        if (i < dk && c < dv) st[(size_t)i * dv + c] = s[u];
    }
}

// grid: tokens.  Dynamic LDS: heads * dv floats.
template <typename T>
__global__ __launch_bounds__(DA_THREADS) void decay_finish_kernel(
    T* __restrict__ out, int out_stride, const float* __restrict__ o, int o_stride, const float* __restrict__ gate,
    int gate_stride, const float* __restrict__ weight, int heads, int dv, int joint, int gate_act, float eps) {
    extern __shared__ float row[];
    __shared__ float red[16];
    __shared__ float inv_of[256];
    const int n = blockIdx.x, width = heads * dv;
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += DA_THREADS) {
        const float x = o[(size_t)n * o_stride + i];
        row[i] = x;
        ss = fmaf(x, x, ss);
    }
    float inv_all = 0.f;
    if (joint) {
        inv_all = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
    } else {
        __syncthreads();
        for (int h0 = 0; h0 < heads; h0 += 256) {
            for (int h = h0 + wave; h < min(heads, h0 + 256); h += DA_THREADS / LLMS_WAVE) {
                float a = 0.f;
                for (int i = lane; i < dv; i += LLMS_WAVE) a = fmaf(row[h * dv + i], row[h * dv + i], a);
                a = wave_sum(a);
                if (lane == 0) inv_of[h - h0] = 1.f / sqrtf(a / (float)dv + eps);
            }
            __syncthreads();
            for (int i = threadIdx.x + h0 * dv; i < min(heads, h0 + 256) * dv; i += DA_THREADS) row[i] *= inv_of[i / dv - h0];
            __syncthreads();
        }
    }
    for (int i = threadIdx.x; i < width; i += DA_THREADS) {
        float x = row[i];
        if (joint) x = x * inv_all * weight[i];
        if (gate_act != DA_ACT_NONE) {
            const float z = gate[(size_t)n * gate_stride + i];
            x *= gate_act == DA_ACT_SILU ? da_silu(z) : 1.f / (1.f + expf(-z));
        }
        out[(size_t)n * out_stride + i] = from_f32<T>(x);
    }
}

extern "C" {

int llms_decay_prepare(float* proj, int stride, int col_q, int col_k, int col_v, const int* positions, const float* freq,
                       int rot_dims, int n_tokens, int heads, int dk, int dv, int act, float key_scale, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && heads > 0 && dk > 0 && dv > 0, "decay_prepare: sizes must be positive");
    LLMS_REQUIRE(rot_dims >= 0 && rot_dims <= dk && rot_dims % 2 == 0, "decay_prepare: an even number of turned dimensions, up to dk");
    LLMS_REQUIRE(rot_dims == 0 || (freq && positions), "decay_prepare: a rotation needs frequencies and positions");
    LLMS_REQUIRE(act == DA_ACT_NONE || act == DA_ACT_SILU, "decay_prepare: activation 0 (none) or 1 (SiLU)");
    LLMS_REQUIRE(heads <= 65535, "decay_prepare: up to 65,535 heads");
    decay_prepare_kernel<<<dim3(n_tokens, heads), DA_THREADS, 0, stream>>>(proj, stride, col_q, col_k, col_v, positions, freq,
                                                                           rot_dims, heads, dk, dv, act, key_scale);
    LLMS_LAUNCH_CHECK();
}

int llms_decay_scan(float* out, int out_stride, const float* proj, int stride, int col_q, int col_k, int col_v, float* state,
                    const int* state_slots, const int* cu_seqlens, const int* context_lens, const float* decay, int n_seqs,
                    int heads, int dk, int dv, hipStream_t stream) {
    LLMS_REQUIRE(n_seqs > 0 && heads > 0 && dk > 0 && dv > 0, "decay_scan: sizes must be positive");
    LLMS_REQUIRE(dk <= 256, "decay_scan: keys of up to 256 numbers");
    LLMS_REQUIRE(heads <= 65535 && n_seqs <= 65535, "decay_scan: up to 65,535 heads and requests");
    dim3 grid((dv + DA_COLS - 1) / DA_COLS, heads, n_seqs);
#define DA_GO(RPT)                                                                                                     \
    decay_scan_kernel<RPT><<<grid, DA_THREADS, 0, stream>>>(out, out_stride, proj, stride, col_q, col_k, col_v, state,  \
                                                            state_slots, cu_seqlens, context_lens, decay, heads, dk, dv)
    if (dk <= 32) DA_GO(8);
    else if (dk <= 64) DA_GO(16);
    else if (dk <= 128) DA_GO(32);
    else DA_GO(64);
#undef DA_GO
    LLMS_LAUNCH_CHECK();
}

int llms_decay_finish(int dtype, void* out, int out_stride, const float* o, int o_stride, const float* gate, int gate_stride,
                      const float* weight, int n_tokens, int heads, int dv, int joint, int gate_act, float eps,
                      hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && heads > 0 && dv > 0, "decay_finish: sizes must be positive");
    LLMS_REQUIRE(!joint || weight, "decay_finish: the norm over all heads has a weight");
    LLMS_REQUIRE(gate_act == DA_ACT_NONE || gate, "decay_finish: a gate needs its products");
    LLMS_REQUIRE(gate_act >= 0 && gate_act <= 2, "decay_finish: gate 0 (none), 1 (SiLU) or 2 (sigmoid)");
    const size_t lds = (size_t)heads * dv * sizeof(float);
    LLMS_REQUIRE(lds <= 128 * 1024, "decay_finish: heads times value size up to 32,768");
#define DA_GO(T)                                                                                                          \
    do {                                                                                                                  \
        if (lds > 32 * 1024)                                                                                              \
            LLMS_HIP_CHECK(hipFuncSetAttribute((const void*)decay_finish_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                               (int)lds));                                                                \
        decay_finish_kernel<T><<<n_tokens, DA_THREADS, lds, stream>>>((T*)out, out_stride, o, o_stride, gate, gate_stride, \
                                                                      weight, heads, dv, joint, gate_act, eps);           \
    } while (0)
    if (dtype == 0) DA_GO(float);
    else if (dtype == 1) DA_GO(bf16);
    else LLMS_REQUIRE(false, "decay_finish: dtype must be 0 (float32) or 1 (bfloat16)");
#undef DA_GO
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
