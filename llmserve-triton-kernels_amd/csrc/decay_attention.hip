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
// PREP: q, k and v are taken as the projection left them, and what decay_prepare would do to them (activation, rotation
// by positions[row], the factor on k) is done on their way in, with the same arithmetic; proj is not written.
struct DecayPrep {
    const int* positions;
    const float* freq;
    int rot_dims, act;
    float key_scale;
};

// Dimension e of a head's q (or, `key`, k) of the token at row `row`, prepared; `src`: the head's numbers in that row.
template <bool PREP>
__device__ __forceinline__ float da_take(const float* __restrict__ src, int e, bool key, const DecayPrep& prep, int row) {
    float x = src[e];
    if constexpr (PREP) {
        if (prep.act == DA_ACT_SILU) x = da_silu(x);
        if (e < prep.rot_dims) {  // dimension e < half is turned together with dimension e + half
            const int half = prep.rot_dims / 2;
            const bool first = e < half;
            float y = src[first ? e + half : e - half];
            if (prep.act == DA_ACT_SILU) y = da_silu(y);
            const float2 sc = rotary_angle((float)prep.positions[row], prep.freq[first ? e : e - half]);
            const float2 turned = first ? rotate_pair(x, y, sc.y, sc.x) : rotate_pair(y, x, sc.y, sc.x);
            x = first ? turned.x : turned.y;
        }
        if (key) x *= prep.key_scale;
    }
    return x;
}

template <bool PREP>
__device__ __forceinline__ float da_take_value(float v, const DecayPrep& prep) {
    if constexpr (PREP)
        if (prep.act == DA_ACT_SILU) v = da_silu(v);
    return v;
}

template <int RPT, bool PREP>
__global__ __launch_bounds__(DA_THREADS) void decay_scan_kernel(
    float* __restrict__ out, int out_stride, const float* __restrict__ proj, int stride, int col_q, int col_k, int col_v,
    float* __restrict__ state, const int* __restrict__ state_slots, const int* __restrict__ cu_seqlens,
    const int* __restrict__ context_lens, const float* __restrict__ decay, int heads, int dk, int dv, const DecayPrep prep) {
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
        for (int i = threadIdx.x; i < 2 * dk; i += DA_THREADS) {
            const bool key = i >= dk;
            buf[i] = da_take<PREP>(row + (key ? col_k : col_q) + h * dk, key ? i - dk : i, key, prep, row0 + t);
        }
        const float v = c < dv ? da_take_value<PREP>(row[col_v + h * dv + c], prep) : 0.f;
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

// ---- portions of many tokens: runs of DA_CHUNK tokens on the 32-bit matrix instruction ------------------------------
//
// A run is DA_CHUNK (64) neighbouring new tokens of one request, counted from the start of its portion (any cut gives the
// same recurrence).  Its place in the workspace [runs, heads, dk, dv] is cu_seqlens[b] / 64 + b + j (run j of request b):
// the runs of different requests never meet, and N / 64 + requests places hold them all.
// All three kernels form products of 32 x 32 tiles with v_mfma_f32_32x32x2_f32 (true 32-bit operands and sums):
// lane l brings A[l % 32][l / 32] and B[l / 32][l % 32] of a step of 2, and holds the 16 numbers
// C[8 (i / 4) + 4 (l / 32) + i % 4][l % 32], i = 0 .. 15.  Operands lie in LDS, rows padded by one number.
#define DA_CHUNK 64
#define DA_SLAB 64  // columns of v (and of the state) that a workgroup takes

typedef __attribute__((ext_vector_type(16))) float f32x16;

// powers[n] = decay^n, n = 0 .. DA_CHUNK, by repeated multiplication (any decay, also 0 and negative ones)
__device__ __forceinline__ void da_powers(float* powers, float d) {
    if (threadIdx.x == 0) {
        double p = 1.0;
        for (int n = 0; n <= DA_CHUNK; ++n) powers[n] = (float)p, p *= (double)d;
    }
}

__device__ __forceinline__ int da_run_place(int row0, int b, int j) { return row0 / DA_CHUNK + b + j; }

// grid: (runs of the longest portion, heads, requests * slabs).  ws[run][h] = sum_t decay^(n - 1 - t) k_t v_t^T over the
// run's n tokens.
template <int DKP, bool PREP>
__global__ __launch_bounds__(DA_THREADS) void decay_chunk_sums_kernel(
    float* __restrict__ ws, const float* __restrict__ proj, int stride, int col_k, int col_v,
    const int* __restrict__ cu_seqlens, const int* __restrict__ context_lens, const float* __restrict__ decay, int heads,
    int dk, int dv, int slabs, const DecayPrep prep) {
    constexpr int LD = DKP + 1, LV = DA_SLAB + 1;
    __shared__ float ks[DA_CHUNK * LD];
    __shared__ float vs[DA_CHUNK * LV];
    __shared__ float powers[DA_CHUNK + 1];
    const int b = blockIdx.z / slabs, c0 = (blockIdx.z % slabs) * DA_SLAB, h = blockIdx.y, j = blockIdx.x;
    const int row0 = cu_seqlens[b], count = cu_seqlens[b + 1] - row0;
    if (context_lens[b] <= 0 || j * DA_CHUNK >= count) return;
    const int n = min(DA_CHUNK, count - j * DA_CHUNK);
    da_powers(powers, decay[h]);
    __syncthreads();
    const float* rows = proj + (size_t)(row0 + j * DA_CHUNK) * stride;
    for (int e = threadIdx.x; e < DA_CHUNK * DKP; e += DA_THREADS) {
        const int t = e / DKP, i = e % DKP;
        ks[t * LD + i] = (t < n && i < dk) ? da_take<PREP>(rows + (size_t)t * stride + col_k + h * dk, i, true, prep,
                                                           row0 + j * DA_CHUNK + t) * powers[n - 1 - t]
                                           : 0.f;
    }
    for (int e = threadIdx.x; e < DA_CHUNK * DA_SLAB; e += DA_THREADS) {
        const int t = e / DA_SLAB, c = e % DA_SLAB;
        vs[t * LV + c] = (t < n && c0 + c < dv) ? da_take_value<PREP>(rows[(size_t)t * stride + col_v + h * dv + c0 + c], prep) : 0.f;
    }
    __syncthreads();
    const int wave = threadIdx.x / LLMS_WAVE, lane = threadIdx.x % LLMS_WAVE, lo = lane % 32, hi = lane / 32;
    float* dst = ws + ((size_t)da_run_place(row0, b, j) * heads + h) * dk * dv;
    for (int tile = wave; tile < (DKP / 32) * (DA_SLAB / 32); tile += DA_THREADS / LLMS_WAVE) {
        const int ir = tile / (DA_SLAB / 32) * 32, tc = tile % (DA_SLAB / 32) * 32;
        f32x16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
        for (int t = 0; t < DA_CHUNK; t += 2)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ks[(t + hi) * LD + ir + lo], vs[(t + hi) * LV + tc + lo], acc, 0, 0, 0);
#pragma unroll
        for (int x = 0; x < 16; ++x) {
            const int i = ir + 8 * (x / 4) + 4 * hi + x % 4, c = c0 + tc + lo;
            if (i < dk && c < dv) dst[(size_t)i * dv + c] = acc[x];
        }
    }
}

// grid: (ceil(dk dv / 256), heads, requests).  Turns the runs' sums into the state before each run, in place, and stores
// the request's last state.
__global__ __launch_bounds__(DA_THREADS) void decay_chunk_scan_kernel(
    float* __restrict__ ws, float* __restrict__ state, const int* __restrict__ state_slots, const int* __restrict__ cu_seqlens,
    const int* __restrict__ context_lens, const float* __restrict__ decay, int heads, int dk, int dv) {
    const int b = blockIdx.z, h = blockIdx.y, e = blockIdx.x * DA_THREADS + threadIdx.x;
    const int row0 = cu_seqlens[b], count = cu_seqlens[b + 1] - row0, length = context_lens[b];
    if (length <= 0 || count <= 0 || e >= dk * dv) return;
    const float d = decay[h];
    double full = 1.0, rest = 1.0;
    const int runs = (count + DA_CHUNK - 1) / DA_CHUNK, last = count - (runs - 1) * DA_CHUNK;
    for (int n = 0; n < DA_CHUNK; ++n) {
        full *= (double)d;
        if (n < last) rest *= (double)d;
    }
    float* st = state + ((size_t)state_slots[b] * heads + h) * dk * dv + e;
    float s = length > count ? *st : 0.f;  // (a portion from position 0 starts from zero)
    float* at = ws + ((size_t)da_run_place(row0, b, 0) * heads + h) * dk * dv + e;
    const size_t step = (size_t)heads * dk * dv;
    for (int j0 = 0; j0 < runs; j0 += 8) {  // 8 runs' sums are asked for together, then replaced one after the other
        float sums[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) sums[u] = j0 + u < runs ? at[(size_t)u * step] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int j = j0 + u;
            if (j < runs) {
                at[(size_t)u * step] = s;
                s = fmaf(j + 1 < runs ? (float)full : (float)rest, s, sums[u]);
            }
        }
        at += 8 * step;
    }
    *st = s;
}

// grid: (runs of the longest portion, heads, requests * slabs).  o_t = decay^(t + 1) S^T q_t + sum_(s <= t) (q_t . k_s)
// decay^(t - s) v_s over the run's tokens, S being the state before the run (ws[run][h]).
template <int DKP, bool PREP>
__global__ __launch_bounds__(DA_THREADS) void decay_chunk_out_kernel(
    float* __restrict__ out, int out_stride, const float* __restrict__ ws, const float* __restrict__ proj, int stride, int col_q,
    int col_k, int col_v, const int* __restrict__ cu_seqlens, const int* __restrict__ context_lens,
    const float* __restrict__ decay, int heads, int dk, int dv, int slabs, const DecayPrep prep) {
    constexpr int LD = DKP + 1, LV = DA_SLAB + 1, LP = DA_CHUNK + 1;
    constexpr int KS = DA_CHUNK * LD > DKP * LV ? DA_CHUNK * LD : DKP * LV;  // the keys, and after them the state's columns
    extern __shared__ float lds[];
    float* qs = lds;                    // [64][LD]
    float* ks = qs + DA_CHUNK * LD;     // [64][LD], later ss [DKP][LV]
    float* ps = ks + KS;                // [64][LP]
    float* vs = ps + DA_CHUNK * LP;     // [64][LV]
    float* powers = vs + DA_CHUNK * LV; // [65]
    const int b = blockIdx.z / slabs, c0 = (blockIdx.z % slabs) * DA_SLAB, h = blockIdx.y, j = blockIdx.x;
    const int row0 = cu_seqlens[b], count = cu_seqlens[b + 1] - row0;
    if (j * DA_CHUNK >= count) return;
    const int n = min(DA_CHUNK, count - j * DA_CHUNK);
    if (context_lens[b] <= 0) {  // padding: no request, no state; its rows leave zeros
        for (int e = threadIdx.x; e < n * DA_SLAB; e += DA_THREADS)
            if (c0 + e % DA_SLAB < dv) out[(size_t)(row0 + j * DA_CHUNK + e / DA_SLAB) * out_stride + h * dv + c0 + e % DA_SLAB] = 0.f;
        return;
    }
    da_powers(powers, decay[h]);
    const float* rows = proj + (size_t)(row0 + j * DA_CHUNK) * stride;
    for (int e = threadIdx.x; e < DA_CHUNK * DKP; e += DA_THREADS) {
        const int t = e / DKP, i = e % DKP;
        const bool there = t < n && i < dk;
        const int row = row0 + j * DA_CHUNK + t;
        qs[t * LD + i] = there ? da_take<PREP>(rows + (size_t)t * stride + col_q + h * dk, i, false, prep, row) : 0.f;
        ks[t * LD + i] = there ? da_take<PREP>(rows + (size_t)t * stride + col_k + h * dk, i, true, prep, row) : 0.f;
    }
    for (int e = threadIdx.x; e < DA_CHUNK * DA_SLAB; e += DA_THREADS) {
        const int t = e / DA_SLAB, c = e % DA_SLAB;
        vs[t * LV + c] = (t < n && c0 + c < dv) ? da_take_value<PREP>(rows[(size_t)t * stride + col_v + h * dv + c0 + c], prep) : 0.f;
    }
    // the state before the run is asked for now and put into LDS (in the keys' place) once the scores are done with the keys
    constexpr int S_EACH = DKP * DA_SLAB / DA_THREADS;
    float s_before[S_EACH];
    const float* before = ws + ((size_t)da_run_place(row0, b, j) * heads + h) * dk * dv;
#pragma unroll
    for (int u = 0; u < S_EACH; ++u) {
        const int e = threadIdx.x + u * DA_THREADS, i = e / DA_SLAB, c = e % DA_SLAB;
        s_before[u] = (i < dk && c0 + c < dv) ? before[(size_t)i * dv + c0 + c] : 0.f;
    }
    __syncthreads();
    const int wave = threadIdx.x / LLMS_WAVE, lane = threadIdx.x % LLMS_WAVE, lo = lane % 32, hi = lane / 32;
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    {   // what the run's tokens see of each other: tiles (0,0), (1,0), (1,1) of q k^T, each weighted by the decay over the
        // distance; tile (0,1) lies ahead of its queries
        const int tr = wave == 0 ? 0 : 32, tc = wave == 2 ? 32 : 0;
        f32x16 acc = zero;
        if (wave < 3) {
#pragma unroll 8
            for (int i = 0; i < DKP; i += 2)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qs[(tr + lo) * LD + i + hi], ks[(tc + lo) * LD + i + hi], acc, 0, 0, 0);
        }
#pragma unroll
        for (int x = 0; x < 16; ++x) {
            const int t = (wave == 3 ? 0 : tr) + 8 * (x / 4) + 4 * hi + x % 4, s2 = (wave == 3 ? 32 : tc) + lo;
            ps[t * LP + s2] = (wave < 3 && s2 <= t) ? acc[x] * powers[t - s2] : 0.f;
        }
    }
    __syncthreads();  // (the keys are done with)
    float* ss = ks;
#pragma unroll
    for (int u = 0; u < S_EACH; ++u) {
        const int e = threadIdx.x + u * DA_THREADS;
        ss[(e / DA_SLAB) * LV + e % DA_SLAB] = s_before[u];
    }
    __syncthreads();
    const int tr = (wave % 2) * 32, tc = (wave / 2) * 32;
    f32x16 acc = zero;
#pragma unroll 8
    for (int i = 0; i < DKP; i += 2)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qs[(tr + lo) * LD + i + hi], ss[(i + hi) * LV + tc + lo], acc, 0, 0, 0);
#pragma unroll
    for (int x = 0; x < 16; ++x) acc[x] *= powers[tr + 8 * (x / 4) + 4 * hi + x % 4 + 1];
    const int keys = tr + 32;  // (the keys behind the tile's last query weigh nothing)
#pragma unroll 8
    for (int s2 = 0; s2 < keys; s2 += 2)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ps[(tr + lo) * LP + s2 + hi], vs[(s2 + hi) * LV + tc + lo], acc, 0, 0, 0);
#pragma unroll
    for (int x = 0; x < 16; ++x) {
        const int t = tr + 8 * (x / 4) + 4 * hi + x % 4, c = c0 + tc + lo;
        if (t < n && c < dv) out[(size_t)(row0 + j * DA_CHUNK + t) * out_stride + h * dv + c] = acc[x];
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

// The same for rows of heads * dv = 1,024 E numbers, E up to 8, in 16-byte pieces: a thread keeps its E pieces of o, of the
// gate's products and of the weight in registers, all asked for before anything is waited for, so a token costs one trip
// to memory (decoding is a chain of such trips).  The norm over all heads only (a head's own norm needs the row in LDS).
template <typename T, int E>
__global__ __launch_bounds__(DA_THREADS) void decay_finish_joint_kernel(
    T* __restrict__ out, int out_stride, const float* __restrict__ o, int o_stride, const float* __restrict__ gate,
    int gate_stride, const float* __restrict__ weight, int width, int gate_act, float eps) {
    __shared__ float red[16];
    const int n = blockIdx.x;
    float4 x[E], z[E], w[E];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < E; ++u) {
        const int c = 4 * (u * DA_THREADS + threadIdx.x);
        x[u] = *reinterpret_cast<const float4*>(o + (size_t)n * o_stride + c);
        w[u] = *reinterpret_cast<const float4*>(weight + c);
        z[u] = gate_act != DA_ACT_NONE ? *reinterpret_cast<const float4*>(gate + (size_t)n * gate_stride + c)
                                       : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < E; ++u) ss += (x[u].x * x[u].x + x[u].y * x[u].y) + (x[u].z * x[u].z + x[u].w * x[u].w);
    const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
    auto gated = [&](float v, float g) {
        if (gate_act == DA_ACT_NONE) return v;
        return v * (gate_act == DA_ACT_SILU ? da_silu(g) : 1.f / (1.f + expf(-g)));
    };
#pragma unroll
    for (int u = 0; u < E; ++u) {
        const int c = 4 * (u * DA_THREADS + threadIdx.x);
        const float a = gated(x[u].x * inv * w[u].x, z[u].x), b = gated(x[u].y * inv * w[u].y, z[u].y);
        const float cc = gated(x[u].z * inv * w[u].z, z[u].z), d = gated(x[u].w * inv * w[u].w, z[u].w);
        T* at = out + (size_t)n * out_stride + c;
        if constexpr (sizeof(T) == 2) {
            *reinterpret_cast<uint2*>(at) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(cc, d));
        } else {
            *reinterpret_cast<float4*>(at) = make_float4(a, b, cc, d);
        }
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

// `prepare` != 0: the rows of proj are as the projection left them, and positions, freq, rot_dims, act and key_scale say
// what llms_decay_prepare would have done to them (done here on their way in; proj is left as it is).
int llms_decay_scan(float* out, int out_stride, const float* proj, int stride, int col_q, int col_k, int col_v, float* state,
                    const int* state_slots, const int* cu_seqlens, const int* context_lens, const float* decay, int n_seqs,
                    int heads, int dk, int dv, int prepare, const int* positions, const float* freq, int rot_dims, int act,
                    float key_scale, hipStream_t stream) {
    LLMS_REQUIRE(n_seqs > 0 && heads > 0 && dk > 0 && dv > 0, "decay_scan: sizes must be positive");
    LLMS_REQUIRE(dk <= 256, "decay_scan: keys of up to 256 numbers");
    LLMS_REQUIRE(heads <= 65535 && n_seqs <= 65535, "decay_scan: up to 65,535 heads and requests");
    if (prepare) {
        LLMS_REQUIRE(rot_dims >= 0 && rot_dims <= dk && rot_dims % 2 == 0, "decay_scan: an even number of turned dimensions, up to dk");
        LLMS_REQUIRE(rot_dims == 0 || (freq && positions), "decay_scan: a rotation needs frequencies and positions");
        LLMS_REQUIRE(act == DA_ACT_NONE || act == DA_ACT_SILU, "decay_scan: activation 0 (none) or 1 (SiLU)");
    }
    const DecayPrep prep = {positions, freq, rot_dims, act, key_scale};
    dim3 grid((dv + DA_COLS - 1) / DA_COLS, heads, n_seqs);
#define DA_GO(RPT)                                                                                                          \
    do {                                                                                                                    \
        if (prepare)                                                                                                        \
            decay_scan_kernel<RPT, true><<<grid, DA_THREADS, 0, stream>>>(out, out_stride, proj, stride, col_q, col_k, col_v, \
                                                                          state, state_slots, cu_seqlens, context_lens,     \
                                                                          decay, heads, dk, dv, prep);                      \
        else                                                                                                                \
            decay_scan_kernel<RPT, false><<<grid, DA_THREADS, 0, stream>>>(out, out_stride, proj, stride, col_q, col_k,     \
                                                                           col_v, state, state_slots, cu_seqlens,           \
                                                                           context_lens, decay, heads, dk, dv, prep);       \
    } while (0)
    if (dk <= 32) DA_GO(8);
    else if (dk <= 64) DA_GO(16);
    else if (dk <= 128) DA_GO(32);
    else DA_GO(64);
#undef DA_GO
    LLMS_LAUNCH_CHECK();
}

// Floats of the workspace that `llms_decay_chunks` needs for n_tokens rows of n_seqs requests.
long long llms_decay_chunks_workspace(int n_tokens, int n_seqs, int heads, int dk, int dv) {
    return ((long long)n_tokens / DA_CHUNK + n_seqs + 1) * heads * dk * dv;
}

// The same recurrence as llms_decay_scan for portions of many tokens (`max_new`: the most one request brings).
int llms_decay_chunks(float* out, int out_stride, const float* proj, int stride, int col_q, int col_k, int col_v, float* state,
                      const int* state_slots, const int* cu_seqlens, const int* context_lens, const float* decay, float* ws,
                      int n_seqs, int max_new, int heads, int dk, int dv, int prepare, const int* positions, const float* freq,
                      int rot_dims, int act, float key_scale, hipStream_t stream) {
    LLMS_REQUIRE(n_seqs > 0 && max_new > 0 && heads > 0 && dk > 0 && dv > 0, "decay_chunks: sizes must be positive");
    LLMS_REQUIRE(dk <= 128, "decay_chunks: keys of up to 128 numbers");
    LLMS_REQUIRE(ws, "decay_chunks: a workspace");
    const int slabs = (dv + DA_SLAB - 1) / DA_SLAB, runs = (max_new + DA_CHUNK - 1) / DA_CHUNK;
    LLMS_REQUIRE(heads <= 65535 && (long long)n_seqs * slabs <= 65535, "decay_chunks: up to 65,535 heads, and requests times slabs");
    const dim3 grid(runs, heads, n_seqs * slabs);
    const int dkp = (dk + 31) / 32 * 32;
    if (prepare) {
        LLMS_REQUIRE(rot_dims >= 0 && rot_dims <= dk && rot_dims % 2 == 0, "decay_chunks: an even number of turned dimensions, up to dk");
        LLMS_REQUIRE(rot_dims == 0 || (freq && positions), "decay_chunks: a rotation needs frequencies and positions");
        LLMS_REQUIRE(act == DA_ACT_NONE || act == DA_ACT_SILU, "decay_chunks: activation 0 (none) or 1 (SiLU)");
    }
    const DecayPrep prep = {positions, freq, rot_dims, act, key_scale};
#define DA_GO(DKP)                                                                                                        \
    do {                                                                                                                  \
        if (prepare) DA_GO2(DKP, true);                                                                                   \
        else DA_GO2(DKP, false);                                                                                          \
    } while (0)
#define DA_GO2(DKP, PREP)                                                                                                        \
    do {                                                                                                                  \
        decay_chunk_sums_kernel<DKP, PREP><<<grid, DA_THREADS, 0, stream>>>(ws, proj, stride, col_k, col_v, cu_seqlens,    \
                                                                            context_lens, decay, heads, dk, dv, slabs, prep); \
        decay_chunk_scan_kernel<<<dim3((dk * dv + DA_THREADS - 1) / DA_THREADS, heads, n_seqs), DA_THREADS, 0, stream>>>(   \
            ws, state, state_slots, cu_seqlens, context_lens, decay, heads, dk, dv);                                      \
        constexpr int ks = DA_CHUNK * (DKP + 1) > DKP * (DA_SLAB + 1) ? DA_CHUNK * (DKP + 1) : DKP * (DA_SLAB + 1);       \
        const size_t lds = (size_t)(DA_CHUNK * (DKP + 1) + ks + DA_CHUNK * (DA_CHUNK + 1) + DA_CHUNK * (DA_SLAB + 1) +    \
                                    DA_CHUNK + 1) * sizeof(float);                                                        \
        if (lds > 48 * 1024)                                                                                              \
            LLMS_HIP_CHECK(hipFuncSetAttribute((const void*)decay_chunk_out_kernel<DKP, PREP>,                            \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                    \
        decay_chunk_out_kernel<DKP, PREP><<<grid, DA_THREADS, lds, stream>>>(out, out_stride, ws, proj, stride, col_q,     \
                                                                             col_k, col_v, cu_seqlens, context_lens,      \
                                                                             decay, heads, dk, dv, slabs, prep);          \
    } while (0)
    if (dkp == 32) DA_GO(32);
    else if (dkp == 64) DA_GO(64);
    else if (dkp == 96) DA_GO(96);
    else DA_GO(128);
#undef DA_GO
#undef DA_GO2
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
    const int width = heads * dv, each = width % (4 * DA_THREADS) == 0 ? width / (4 * DA_THREADS) : 0;
    auto aligned = [](const void* p, int stride) { return ((uintptr_t)p % 16) == 0 && stride % 4 == 0; };
    if (joint && (each == 1 || each == 2 || each == 4 || each == 8) && aligned(o, o_stride) && aligned(weight, 0) &&
        (gate_act == DA_ACT_NONE || aligned(gate, gate_stride)) && aligned(out, dtype == 0 ? out_stride : out_stride / 2) &&
        (dtype == 0 || out_stride % 4 == 0)) {
#define DA_JOINT(T, E)                                                                                                    \
    decay_finish_joint_kernel<T, E><<<n_tokens, DA_THREADS, 0, stream>>>((T*)out, out_stride, o, o_stride, gate, gate_stride, \
                                                                         weight, width, gate_act, eps)
#define DA_JOINT_T(T)                                                                                                     \
    do {                                                                                                                  \
        if (each == 1) DA_JOINT(T, 1);                                                                                    \
        else if (each == 2) DA_JOINT(T, 2);                                                                               \
        else if (each == 4) DA_JOINT(T, 4);                                                                               \
        else DA_JOINT(T, 8);                                                                                              \
    } while (0)
        if (dtype == 0) DA_JOINT_T(float);
        else if (dtype == 1) DA_JOINT_T(bf16);
        else LLMS_REQUIRE(false, "decay_finish: dtype must be 0 (float32) or 1 (bfloat16)");
#undef DA_JOINT_T
#undef DA_JOINT
        LLMS_LAUNCH_CHECK();
    }
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
