// Recurrent mixers over a state of fixed size per request, everything in 32-bit:
//
//   conv_act        a short causal convolution per channel over the 32-bit products of a step's tokens, plus a bias,
//                   then SiLU: y_t = act(b + sum_j w[c, j] u_(t - taps + 1 + j)), zeros before the sequence.  A request's
//                   last taps - 1 input rows are a ring in its state, indexed by position, so a portion of any length
//                   reads what it needs.  The result leaves as 32-bit and, where asked for, rounded to T as well.
//   conv_ring       the ring takes the last taps - 1 input rows of every request of the step (a launch of its own,
//                   because a token's write would race with its neighbours' reads; when every request brings one
//                   token, conv_act writes the ring itself).
//   selective_scan  per channel c and state n:  S <- exp(dt_c A[c, n]) S + dt_c x_c B_n,  y_c = sum_n S C_n + D_c x_c,
//                   dt from `step_sizes`, and y silu(z) leaves rounded once.  16 lanes share a channel's states.
//   conv_heads      conv_act and unit_heads in one launch, a wave a head: what the delta rule's layer runs.
//   unit_heads      every head of q and k is divided by sqrt(sum of squares + eps); q is multiplied by a factor; where
//                   a step brings many tokens it also turns the gates' products into decay and beta, and
//   step_sizes      forms the step sizes (their small product, the bias, softplus) and, for steps of many tokens, silu(z)
//                   of the selective scan, so that no logarithm and no exponential besides the recurrence's own stands
//                   in the chain from token to token.
//   delta_scan      the gated delta rule per head over a state S [dk, dv]:
//                   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q   (the read-out sees the token's write)
//                   with beta = sigmoid(zb) and g = exp(-exp(A_log) softplus(za + dt_bias)).  16 lanes share a column.
//   delta_finish    each head of o is divided by its root mean square (eps inside the root), multiplied by a weight
//                   that all heads share and by silu(gate), rounded once.
//
// A request of length 0 is padding: nothing of it is read or written.  The state of request b lies at
// state + state_slots[b] * slot_stride (+ an offset per kind of state); a portion starts from it and leaves it behind
// its last token, so any cut of a prompt gives the same recurrence.
#include "common.h"

#define RC_THREADS 256

__device__ __forceinline__ float rc_silu(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float rc_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }
// exp(x) for the inside of a recurrence, a handful of instructions: 2^(x log2 e) by the hardware's exponential, with the
// rounding of the product x log2 e put back as a factor (1 + error ln 2); within two units in the last place for x <= 0
__device__ __forceinline__ float rc_exp(float x) {
    const float t = x * 1.44269504f;
    const float err = fmaf(x, 1.92596299e-8f, fmaf(x, 1.44269504f, -t));
    const float e = __builtin_amdgcn_exp2f(t);
    return fmaf(e, err * 0.693147181f, e);
}

// sum over the 16 lanes of a row of the wave, the same value in all of them (no LDS: four lane exchanges inside the row)
__device__ __forceinline__ float row16_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // row_mirror
    return v;
}

// ------------------------------------------------------------------------------------------- convolution
// grid (tokens, channel blocks).  u [N, u_ld] columns u_col ..; ring [taps - 1, channels] at ring_off inside a slot.
struct ConvArgs {
    const float* u;  // [N, u_ld], columns u_col ..
    int u_ld, u_col;
    const float* taps_w;  // [channels, taps]
    const float* bias;    // [channels] or null
    int taps, channels;
    float* state;  // slots; the ring [taps - 1, channels] lies at ring_off inside a slot
    size_t slot_stride, ring_off;
    const int* state_slots;
    const int* token_seq;
    const int* positions;
    const int* cu_seqlens;
    const int* context_lens;
    int activation, update;
};

// channel c of token n after the convolution and the activation (the token belongs to a request that exists)
__device__ __forceinline__ float conv_channel(const ConvArgs& a, int n, int c) {
    const int b = a.token_seq[n];
    const int p = a.positions[n];
    const int first_row = a.cu_seqlens[b];
    const int first_pos = p - (n - first_row);
    float* ring = a.taps > 1 ? a.state + (size_t)a.state_slots[b] * a.slot_stride + a.ring_off : nullptr;
    float y = a.bias ? a.bias[c] : 0.f;
    for (int j = 0; j < a.taps; ++j) {
        const int pos = p - (a.taps - 1) + j;
        float v = 0.f;
        if (pos >= first_pos)
            v = a.u[(size_t)(first_row + pos - first_pos) * a.u_ld + a.u_col + c];
        else if (pos >= 0)
            v = ring[(size_t)(pos % (a.taps - 1)) * a.channels + c];
        y = fmaf(a.taps_w[(size_t)c * a.taps + j], v, y);
    }
    if (a.update && a.taps > 1)  // (every request brings one token: nobody else reads this ring, and this thread has read its place)
        ring[(size_t)(p % (a.taps - 1)) * a.channels + c] = a.u[(size_t)n * a.u_ld + a.u_col + c];
    return a.activation ? rc_silu(y) : y;
}

template <typename T>
__global__ __launch_bounds__(RC_THREADS) void conv_act_kernel(float* __restrict__ y32, int y32_ld, T* __restrict__ y16, int y16_ld,
                                                             const ConvArgs a) {
    const int n = blockIdx.x;
    const int c = blockIdx.y * RC_THREADS + threadIdx.x;
    if (c >= a.channels || a.context_lens[a.token_seq[n]] <= 0) return;
    const float y = conv_channel(a, n, c);
    if (y32) y32[(size_t)n * y32_ld + c] = y;
    if (y16) y16[(size_t)n * y16_ld + c] = from_f32<T>(y);
}

// The convolution where the first channels are heads of q and k that are made unit vectors behind it: grid (tokens, q heads
// + k heads + blocks of 64 other channels [+ 1 for the gates]), one wave each.  A head of dk numbers (up to 256; q heads
// first, k heads behind them, from channel 0) is divided by sqrt(sum of squares + eps), q also multiplied by q_factor; the
// last block (with `gates`) turns the gates' products into decay and beta, as `unit_heads` does.
#define CH_PER_LANE 4
__global__ __launch_bounds__(LLMS_WAVE) void conv_heads_kernel(float* __restrict__ y32, int y32_ld, const ConvArgs a, int q_heads,
                                                               int k_heads, int dk, float eps, float q_factor,
                                                               float* __restrict__ gates, int g_ld, int a_col, int b_col,
                                                               const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                                               int heads) {
    const int n = blockIdx.x, lane = threadIdx.x, role = blockIdx.y;
    if (a.context_lens[a.token_seq[n]] <= 0) return;
    const int first_other = (q_heads + k_heads) * dk;
    const int other_blocks = (a.channels - first_other + LLMS_WAVE - 1) / LLMS_WAVE;
    if (role < q_heads + k_heads) {
        float y[CH_PER_LANE];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < CH_PER_LANE; ++i) {
            const int d = lane + i * LLMS_WAVE;
            y[i] = d < dk ? conv_channel(a, n, role * dk + d) : 0.f;
            ss = fmaf(y[i], y[i], ss);
        }
        const float mul = (role < q_heads ? q_factor : 1.f) / sqrtf(wave_sum(ss) + eps);
#pragma unroll
        for (int i = 0; i < CH_PER_LANE; ++i) {
            const int d = lane + i * LLMS_WAVE;
            if (d < dk) y32[(size_t)n * y32_ld + role * dk + d] = y[i] * mul;
        }
    } else if (role < q_heads + k_heads + other_blocks) {
        const int c = first_other + (role - q_heads - k_heads) * LLMS_WAVE + lane;
        if (c < a.channels) y32[(size_t)n * y32_ld + c] = conv_channel(a, n, c);
    } else {
        float* g = gates + (size_t)n * g_ld;
        for (int h = lane; h < heads; h += LLMS_WAVE) {
            g[a_col + h] = expf(-expf(a_log[h]) * rc_softplus(g[a_col + h] + dt_bias[h]));
            g[b_col + h] = 1.f / (1.f + expf(-g[b_col + h]));
        }
    }
}

// grid (requests, channel blocks)
__global__ __launch_bounds__(RC_THREADS) void conv_ring_kernel(
    float* __restrict__ state, size_t slot_stride, size_t ring_off, const int* __restrict__ state_slots,
    const float* __restrict__ u, int u_ld, int u_col, const int* __restrict__ cu_seqlens,
    const int* __restrict__ context_lens, int taps, int channels) {
    const int b = blockIdx.x;
    const int c = blockIdx.y * RC_THREADS + threadIdx.x;
    if (c >= channels) return;
    const int first_row = cu_seqlens[b], count = cu_seqlens[b + 1] - first_row;
    const int end = context_lens[b];
    if (count <= 0 || end <= 0) return;
    const int first_pos = end - count;
    float* ring = state + (size_t)state_slots[b] * slot_stride + ring_off;
    int pos = end - (taps - 1);
    if (pos < first_pos) pos = first_pos;
    for (; pos < end; ++pos)
        ring[(size_t)(pos % (taps - 1)) * channels + c] = u[(size_t)(first_row + pos - first_pos) * u_ld + u_col + c];
}

// ------------------------------------------------------------------------------------------- selective scan
// grid (requests, channels / 16).  Thread (channel, lane of 16): states lane, lane + 16, ...  R = ceil(states / 16).
// x [N, x_ld] (after the convolution), z [N, z_ld] columns z_col .., low [N, low_ld]: B at b_col, C at c_col,
// dt_raw [N, dt_ld]; S [channels, states] at scan_off inside a slot.
// dt holds the step sizes (`step_sizes`).  PREP: z already holds silu(z) (the same launch), which keeps the exponential
// that does not belong to the recurrence out of its chain.
template <typename T, int R, bool PREP>
__global__ __launch_bounds__(RC_THREADS) void selective_scan_kernel(
    T* __restrict__ out, int out_ld, const float* __restrict__ x, int x_ld, const float* __restrict__ z, int z_ld, int z_col,
    const float* __restrict__ low, int low_ld, int b_col, int c_col, const float* __restrict__ dt_raw, int dt_ld,
    const float* __restrict__ dt_bias, const float* __restrict__ a_neg, const float* __restrict__ d_skip, int channels,
    int states, float* __restrict__ state, size_t slot_stride, size_t scan_off, const int* __restrict__ state_slots,
    const int* __restrict__ cu_seqlens, const int* __restrict__ context_lens) {
    const int b = blockIdx.x;
    const int lane = threadIdx.x & 15;
    const int c = blockIdx.y * (RC_THREADS / 16) + (threadIdx.x >> 4);
    const int first_row = cu_seqlens[b], count = cu_seqlens[b + 1] - first_row;
    if (count <= 0 || context_lens[b] <= 0) return;
    const bool live = c < channels;
    const int cc = live ? c : channels - 1;  // (lanes beyond the last channel compute along and store nothing)
    float* srow = state + (size_t)state_slots[b] * slot_stride + scan_off + (size_t)cc * states;
    float s[R], a[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int k = lane + 16 * r;
        s[r] = k < states ? srow[k] : 0.f;
        a[r] = k < states ? a_neg[(size_t)cc * states + k] : 0.f;
    }
    const float skip = d_skip[cc];
    // tokens in groups of U, two groups in registers: the next group is asked for before the present one is worked on, so
    // the chain from token to token never waits for memory
    constexpr int U = R <= 2 ? 8 : (R <= 4 ? 4 : 2);
    struct Group {
        float dtr[U], xs[U], zs[U], bn[U][R], cn[U][R];
    };
    auto fetch = [&](Group& g, int t0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int t = t0 + u < count ? t0 + u : count - 1;
            const size_t row = (size_t)(first_row + t);
            g.dtr[u] = dt_raw[row * dt_ld + cc];
            g.xs[u] = x[row * x_ld + cc];
            g.zs[u] = z[row * z_ld + z_col + cc];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int k = lane + 16 * r;
                g.bn[u][r] = k < states ? low[row * low_ld + b_col + k] : 0.f;
                g.cn[u][r] = k < states ? low[row * low_ld + c_col + k] : 0.f;
            }
        }
    };
    // (results wait in registers and leave four groups at a time: loads and stores share one counter of what is in
    // flight, and a wait for loads that has stores before it waits for everything, the next group's loads too)
    float held[4 * U];
    auto work = [&](const Group& g, int t0, int slot) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (t0 + u >= count) break;
            const float dt = g.dtr[u];
            const float dx = dt * g.xs[u];
            float y = 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                s[r] = fmaf(rc_exp(dt * a[r]), s[r], dx * g.bn[u][r]);
                y = fmaf(s[r], g.cn[u][r], y);
            }
            y = fmaf(skip, g.xs[u], row16_sum(y));
            held[slot * U + u] = y * (PREP ? g.zs[u] : rc_silu(g.zs[u]));
        }
    };
    auto leave = [&](int t0, int n) {
        if (lane == 0 && live) {
#pragma unroll
            for (int i = 0; i < 4 * U; ++i)
                if (i < n && t0 + i < count) out[(size_t)(first_row + t0 + i) * out_ld + c] = from_f32<T>(held[i]);
        }
    };
    Group ga;
    fetch(ga, 0);
    if (count <= U) {  // (decoding, short portions: one group and no more)
        work(ga, 0, 0);
        leave(0, U);
    } else {
        Group gb;
        for (int t0 = 0; t0 < count; t0 += 4 * U) {
            fetch(gb, t0 + U);  // (a group beyond the last reads the last token again: no branch stands around a load)
            work(ga, t0, 0);
            fetch(ga, t0 + 2 * U);
            work(gb, t0 + U, 1);
            fetch(gb, t0 + 3 * U);
            work(ga, t0 + 2 * U, 2);
            fetch(ga, t0 + 4 * U);
            work(gb, t0 + 3 * U, 3);
            leave(t0, 4 * U);
        }
    }
    if (live) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int k = lane + 16 * r;
            if (k < states) srow[k] = s[r];
        }
    }
}

// grid (blocks of SS_TOKENS tokens, blocks of 64 channels): dt[n, c] = softplus(sum_r low[n, low_col + r] w_t[r, c] + bias[c]),
// the step sizes' product (a weight of few columns, kept transposed so that neighbouring threads read neighbouring
// numbers; a number of the weight serves SS_TOKENS tokens) with what follows it; with `z`, z <- silu(z) in place as well
#define SS_TOKENS 8
__global__ __launch_bounds__(LLMS_WAVE) void step_sizes_kernel(float* __restrict__ dt, int dt_ld, const float* __restrict__ low,
                                                               int low_ld, int low_col, int rank, const float* __restrict__ w_t,
                                                               const float* __restrict__ dt_bias, float* __restrict__ z, int z_ld,
                                                               int z_col, int channels, int n_tokens) {
    extern __shared__ float lows[];  // [rank][SS_TOKENS]
    const int n0 = blockIdx.x * SS_TOKENS, c = blockIdx.y * LLMS_WAVE + threadIdx.x;
    for (int i = threadIdx.x; i < rank * SS_TOKENS; i += LLMS_WAVE) {
        const int t = i % SS_TOKENS, r = i / SS_TOKENS;
        lows[i] = n0 + t < n_tokens ? low[(size_t)(n0 + t) * low_ld + low_col + r] : 0.f;
    }
    __syncthreads();
    if (c >= channels) return;
    float acc[SS_TOKENS];
#pragma unroll
    for (int t = 0; t < SS_TOKENS; ++t) acc[t] = 0.f;
    int r = 0;
    for (; r + 16 <= rank; r += 16) {  // sixteen numbers of the weight asked for at once (few waves run when decoding)
        float w[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) w[k] = w_t[(size_t)(r + k) * channels + c];
#pragma unroll
        for (int k = 0; k < 16; ++k)
#pragma unroll
            for (int t = 0; t < SS_TOKENS; ++t) acc[t] = fmaf(lows[(r + k) * SS_TOKENS + t], w[k], acc[t]);
    }
    for (; r < rank; ++r) {
        const float w = w_t[(size_t)r * channels + c];
#pragma unroll
        for (int t = 0; t < SS_TOKENS; ++t) acc[t] = fmaf(lows[r * SS_TOKENS + t], w, acc[t]);
    }
    const float bias = dt_bias[c];
#pragma unroll
    for (int t = 0; t < SS_TOKENS; ++t) {
        if (n0 + t >= n_tokens) break;
        dt[(size_t)(n0 + t) * dt_ld + c] = rc_softplus(acc[t] + bias);
        if (z) {
            float* zp = z + (size_t)(n0 + t) * z_ld + z_col + c;
            *zp = rc_silu(*zp);
        }
    }
}

// ------------------------------------------------------------------------------------------- unit heads
// grid (tokens, heads of q + heads of k): one wave a head, in place on x [N, ld]: q heads at q_col, k heads behind them at k_col
// A last block per token (with `gates`): gates[n, a_col + h] <- exp(-exp(a_log[h]) softplus(. + dt_bias[h])) and
// gates[n, b_col + h] <- sigmoid(.), the decay and the step of the delta rule, in place.
__global__ __launch_bounds__(LLMS_WAVE) void unit_heads_kernel(float* __restrict__ x, int ld, int q_col, int k_col, int q_heads,
                                                               int k_heads, int dk, float eps, float q_factor,
                                                               float* __restrict__ gates, int g_ld, int a_col, int b_col,
                                                               const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                                               int heads) {
    const int n = blockIdx.x, lane = threadIdx.x;
    const int head = blockIdx.y;
    if (head >= q_heads + k_heads) {
        float* g = gates + (size_t)n * g_ld;
        for (int h = lane; h < heads; h += LLMS_WAVE) {
            g[a_col + h] = expf(-expf(a_log[h]) * rc_softplus(g[a_col + h] + dt_bias[h]));
            g[b_col + h] = 1.f / (1.f + expf(-g[b_col + h]));
        }
        return;
    }
    const bool is_q = head < q_heads;
    float* v = x + (size_t)n * ld + (is_q ? q_col + head * dk : k_col + (head - q_heads) * dk);
    float ss = 0.f;
    for (int d = lane; d < dk; d += LLMS_WAVE) ss = fmaf(v[d], v[d], ss);
    const float mul = (is_q ? q_factor : 1.f) / sqrtf(wave_sum(ss) + eps);
    for (int d = lane; d < dk; d += LLMS_WAVE) v[d] *= mul;
}

// ------------------------------------------------------------------------------------------- delta rule
// grid (requests, heads, columns / 16).  Thread (column j, lane of 16): rows lane, lane + 16, ... of column j of S.
// qkv [N, qkv_ld]: q heads at q_col (kv_heads * dk), k heads at k_col, v heads at v_col (heads * dv), prepared;
// gates [N, g_ld]: za at a_col + head, zb at b_col + head.  S at scan_off inside a slot, [heads][dv][dk] (a head's state
// column by column).
// PREP: the gates' columns already hold decay and beta (`unit_heads` with gates).  VEC: a lane's R rows (R lane .. R lane
// + R - 1, neighbours, so that k and q arrive in 16-byte pieces) are read four at a time.
template <int R, bool PREP, bool VEC>
__global__ __launch_bounds__(RC_THREADS) void delta_scan_kernel(
    float* __restrict__ o, int o_ld, const float* __restrict__ qkv, int qkv_ld, int q_col, int k_col, int v_col,
    const float* __restrict__ gates, int g_ld, int a_col, int b_col, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, int heads, int kv_heads, int dk, int dv, float* __restrict__ state, size_t slot_stride,
    size_t scan_off, const int* __restrict__ state_slots, const int* __restrict__ cu_seqlens,
    const int* __restrict__ context_lens) {
    const int b = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x & 15;
    const int j = blockIdx.z * (RC_THREADS / 16) + (threadIdx.x >> 4);
    const int first_row = cu_seqlens[b], count = cu_seqlens[b + 1] - first_row;
    if (count <= 0 || context_lens[b] <= 0) return;
    const bool live = j < dv;
    const int jj = live ? j : dv - 1;
    const int g = h / (heads / kv_heads);
    const int i0 = R * lane;  // this lane's first row
    // a head's state lies column by column ([dv][dk]): a lane's rows are neighbours in memory, a wave reads whole lines
    float* sh = state + (size_t)state_slots[b] * slot_stride + scan_off + (size_t)h * dk * dv;
    float* scol = sh + (size_t)jj * dk + i0;
    const bool svec = VEC && ((uintptr_t)sh % 16) == 0;  // (dk is a multiple of 4 with VEC)
    float s[R];
    if (svec) {
#pragma unroll
        for (int r = 0; r < R; r += 4) {
            const float4 v = i0 + r < dk ? *reinterpret_cast<const float4*>(scol + r) : make_float4(0.f, 0.f, 0.f, 0.f);
            s[r] = v.x, s[r + 1 < R ? r + 1 : r] = v.y, s[r + 2 < R ? r + 2 : r] = v.z, s[r + 3 < R ? r + 3 : r] = v.w;
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) s[r] = i0 + r < dk ? scol[r] : 0.f;
    }
    const float rate = expf(a_log[h]), bias = dt_bias[h];
    // tokens in groups of U, two groups in registers: the next group is asked for before the present one is worked on
    constexpr int U = R <= 4 ? 8 : (R <= 8 ? 4 : 2);
    struct Group {
        float kk[U][R], qq[U][R], vs[U], za[U], zb[U];
    };
    const float* q_at = qkv + (size_t)first_row * qkv_ld + q_col + g * dk + i0;
    const float* k_at = qkv + (size_t)first_row * qkv_ld + k_col + g * dk + i0;
    const float* v_at = qkv + (size_t)first_row * qkv_ld + v_col + h * dv + jj;
    const float* a_at = gates + (size_t)first_row * g_ld + a_col + h;
    const float* b_at = gates + (size_t)first_row * g_ld + b_col + h;
    auto fetch = [&](Group& gr, int t0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = t0 + u < count ? t0 + u : count - 1;
            const float* qr = q_at + (size_t)t * qkv_ld;
            const float* kr = k_at + (size_t)t * qkv_ld;
            if constexpr (VEC) {
#pragma unroll
                for (int r = 0; r < R; r += 4) {
                    const bool in = i0 + r < dk;  // (dk is a multiple of 4 here: four rows are inside or outside together)
                    const float4 kv = in ? *reinterpret_cast<const float4*>(kr + r) : make_float4(0.f, 0.f, 0.f, 0.f);
                    const float4 qv = in ? *reinterpret_cast<const float4*>(qr + r) : make_float4(0.f, 0.f, 0.f, 0.f);
                    gr.kk[u][r] = kv.x, gr.kk[u][r + 1] = kv.y, gr.kk[u][r + 2] = kv.z, gr.kk[u][r + 3] = kv.w;
                    gr.qq[u][r] = qv.x, gr.qq[u][r + 1] = qv.y, gr.qq[u][r + 2] = qv.z, gr.qq[u][r + 3] = qv.w;
                }
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    gr.kk[u][r] = i0 + r < dk ? kr[r] : 0.f;
                    gr.qq[u][r] = i0 + r < dk ? qr[r] : 0.f;
                }
            }
            gr.vs[u] = v_at[(size_t)t * qkv_ld];
            gr.za[u] = a_at[(size_t)t * g_ld];
            gr.zb[u] = b_at[(size_t)t * g_ld];
        }
    };
    float held[4 * U];  // (results wait in registers and leave up to four groups at a time)
    auto work = [&](const Group& gr, int t0, int slot) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (t0 + u >= count) break;
            const float decay = PREP ? gr.za[u] : expf(-rate * rc_softplus(gr.za[u] + bias));
            const float beta = PREP ? gr.zb[u] : 1.f / (1.f + expf(-gr.zb[u]));
            // with S' = decay S:  u = beta (v - S'^T k),  o = (S' + k u^T)^T q = S'^T q + (k . q) u
            float sk = 0.f, sq = 0.f, kq = 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                s[r] *= decay;
                sk = fmaf(s[r], gr.kk[u][r], sk);
                sq = fmaf(s[r], gr.qq[u][r], sq);
                kq = fmaf(gr.kk[u][r], gr.qq[u][r], kq);
            }
            sk = row16_sum(sk), sq = row16_sum(sq), kq = row16_sum(kq);
            const float w = beta * (gr.vs[u] - sk);
#pragma unroll
            for (int r = 0; r < R; ++r) s[r] = fmaf(gr.kk[u][r], w, s[r]);
            held[slot * U + u] = fmaf(kq, w, sq);
        }
    };
    auto leave = [&](int t0, int n) {
        if (lane == 0 && live) {
#pragma unroll
            for (int i = 0; i < 4 * U; ++i)
                if (i < n && t0 + i < count) o[(size_t)(first_row + t0 + i) * o_ld + h * dv + j] = held[i];
        }
    };
    Group ga;
    fetch(ga, 0);
    if (count <= U) {  // (decoding, short portions: one group and no more)
        work(ga, 0, 0);
        leave(0, U);
    } else {
        Group gb;
        for (int t0 = 0; t0 < count; t0 += 4 * U) {
            fetch(gb, t0 + U);  // (a group beyond the last reads the last token again: no branch stands around a load)
            work(ga, t0, 0);
            fetch(ga, t0 + 2 * U);
            work(gb, t0 + U, 1);
            fetch(gb, t0 + 3 * U);
            work(ga, t0 + 2 * U, 2);
            fetch(ga, t0 + 4 * U);
            work(gb, t0 + 3 * U, 3);
            leave(t0, 4 * U);
        }
    }
    if (live && svec) {
#pragma unroll
        for (int r = 0; r < R; r += 4)
            if (i0 + r < dk)
                *reinterpret_cast<float4*>(scol + r) = make_float4(s[r], s[r + 1 < R ? r + 1 : r], s[r + 2 < R ? r + 2 : r], s[r + 3 < R ? r + 3 : r]);
    } else if (live) {
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (i0 + r < dk) scol[r] = s[r];
    }
}

// grid (tokens, heads): one wave a head
template <typename T>
__global__ __launch_bounds__(LLMS_WAVE) void delta_finish_kernel(T* __restrict__ out, int out_ld, const float* __restrict__ o,
                                                                 int o_ld, const float* __restrict__ gate, int gate_ld,
                                                                 int gate_col, const float* __restrict__ weight, int dv,
                                                                 float eps) {
    const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* v = o + (size_t)n * o_ld + (size_t)h * dv;
    float ss = 0.f;
    for (int d = lane; d < dv; d += LLMS_WAVE) ss = fmaf(v[d], v[d], ss);
    const float mul = 1.f / sqrtf(wave_sum(ss) / (float)dv + eps);
    for (int d = lane; d < dv; d += LLMS_WAVE) {
        const float z = gate[(size_t)n * gate_ld + gate_col + h * dv + d];
        out[(size_t)n * out_ld + h * dv + d] = from_f32<T>(v[d] * mul * weight[d] * rc_silu(z));
    }
}

extern "C" {

static ConvArgs conv_args(const float* u, int u_ld, int u_col, const float* taps_w, const float* bias, int taps, int channels,
                          float* state, size_t slot_stride, size_t ring_off, const int* state_slots, const int* token_seq,
                          const int* positions, const int* cu_seqlens, const int* context_lens, int activation, int update) {
    ConvArgs a;
    a.u = u, a.u_ld = u_ld, a.u_col = u_col, a.taps_w = taps_w, a.bias = bias, a.taps = taps, a.channels = channels;
    a.state = state, a.slot_stride = slot_stride, a.ring_off = ring_off, a.state_slots = state_slots;
    a.token_seq = token_seq, a.positions = positions, a.cu_seqlens = cu_seqlens, a.context_lens = context_lens;
    a.activation = activation, a.update = update;
    return a;
}

int llms_conv_act(int dtype, float* y32, int y32_ld, void* y16, int y16_ld, const float* u, int u_ld, int u_col,
                  const float* taps_w, const float* bias, int taps, int channels, float* state, size_t slot_stride,
                  size_t ring_off, const int* state_slots, const int* token_seq, const int* positions, const int* cu_seqlens,
                  const int* context_lens, int n_tokens, int activation, int update, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && channels > 0 && taps >= 1, "conv_act: sizes must be positive");
    LLMS_REQUIRE(u && taps_w && token_seq && positions && cu_seqlens && context_lens, "conv_act: a needed operand is missing");
    LLMS_REQUIRE(taps == 1 || (state && state_slots), "conv_act: two taps or more need the state");
    LLMS_REQUIRE(y32 || y16, "conv_act: nothing to store");
    const ConvArgs a = conv_args(u, u_ld, u_col, taps_w, bias, taps, channels, state, slot_stride, ring_off, state_slots, token_seq,
                                 positions, cu_seqlens, context_lens, activation, update);
    dim3 grid(n_tokens, (channels + RC_THREADS - 1) / RC_THREADS);
    if (dtype == 0)
        conv_act_kernel<float><<<grid, RC_THREADS, 0, stream>>>(y32, y32_ld, (float*)y16, y16_ld, a);
    else if (dtype == 1)
        conv_act_kernel<bf16><<<grid, RC_THREADS, 0, stream>>>(y32, y32_ld, (bf16*)y16, y16_ld, a);
    else
        LLMS_REQUIRE(false, "conv_act: dtype must be 0 (float32) or 1 (bfloat16)");
    LLMS_LAUNCH_CHECK();
}

int llms_conv_heads(float* y32, int y32_ld, const float* u, int u_ld, int u_col, const float* taps_w, const float* bias, int taps,
                    int channels, float* state, size_t slot_stride, size_t ring_off, const int* state_slots, const int* token_seq,
                    const int* positions, const int* cu_seqlens, const int* context_lens, int n_tokens, int activation, int update,
                    int q_heads, int k_heads, int dk, float eps, float q_factor, float* gates, int g_ld, int a_col, int b_col,
                    const float* a_log, const float* dt_bias, int heads, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && channels > 0 && taps >= 1 && y32, "conv_heads: sizes must be positive");
    LLMS_REQUIRE(u && taps_w && token_seq && positions && cu_seqlens && context_lens, "conv_heads: a needed operand is missing");
    LLMS_REQUIRE(taps == 1 || (state && state_slots), "conv_heads: two taps or more need the state");
    LLMS_REQUIRE(q_heads >= 0 && k_heads >= 0 && dk > 0 && dk <= CH_PER_LANE * LLMS_WAVE && (q_heads + k_heads) * dk <= channels,
                 "conv_heads: heads of up to 256 numbers within the channels");
    LLMS_REQUIRE(!gates || (a_log && dt_bias && heads > 0), "conv_heads: gates need their rates and biases");
    const ConvArgs a = conv_args(u, u_ld, u_col, taps_w, bias, taps, channels, state, slot_stride, ring_off, state_slots, token_seq,
                                 positions, cu_seqlens, context_lens, activation, update);
    const int blocks = q_heads + k_heads + (channels - (q_heads + k_heads) * dk + LLMS_WAVE - 1) / LLMS_WAVE + (gates ? 1 : 0);
    LLMS_REQUIRE(blocks <= 65535, "conv_heads: too many heads and channels for one launch");
    dim3 grid(n_tokens, blocks);
    conv_heads_kernel<<<grid, LLMS_WAVE, 0, stream>>>(y32, y32_ld, a, q_heads, k_heads, dk, eps, q_factor, gates, g_ld, a_col, b_col,
                                                      a_log, dt_bias, heads);
    LLMS_LAUNCH_CHECK();
}

int llms_conv_ring(float* state, size_t slot_stride, size_t ring_off, const int* state_slots, const float* u, int u_ld,
                   int u_col, const int* cu_seqlens, const int* context_lens, int n_seqs, int taps, int channels,
                   hipStream_t stream) {
    LLMS_REQUIRE(n_seqs > 0 && taps > 1 && channels > 0, "conv_ring: sizes must be positive and taps at least 2");
    dim3 grid(n_seqs, (channels + RC_THREADS - 1) / RC_THREADS);
    conv_ring_kernel<<<grid, RC_THREADS, 0, stream>>>(state, slot_stride, ring_off, state_slots, u, u_ld, u_col, cu_seqlens,
                                                      context_lens, taps, channels);
    LLMS_LAUNCH_CHECK();
}

int llms_selective_scan(int dtype, void* out, int out_ld, const float* x, int x_ld, const float* z, int z_ld, int z_col,
                        const float* low, int low_ld, int b_col, int c_col, const float* dt_raw, int dt_ld,
                        const float* dt_bias, const float* a_neg, const float* d_skip, int channels, int states, float* state,
                        size_t slot_stride, size_t scan_off, const int* state_slots, const int* cu_seqlens,
                        const int* context_lens, int n_seqs, int prepared, hipStream_t stream) {
    LLMS_REQUIRE(n_seqs > 0 && channels > 0 && states > 0 && states <= 256, "selective_scan: 1 to 256 states per channel");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "selective_scan: dtype must be 0 (float32) or 1 (bfloat16)");
    dim3 grid(n_seqs, (channels + RC_THREADS / 16 - 1) / (RC_THREADS / 16));
    const int r = (states + 15) / 16;
#define SCAN_GO(T, R, P)                                                                                                  \
    selective_scan_kernel<T, R, P><<<grid, RC_THREADS, 0, stream>>>((T*)out, out_ld, x, x_ld, z, z_ld, z_col, low, low_ld,    \
                                                                    b_col, c_col, dt_raw, dt_ld, dt_bias, a_neg, d_skip,  \
                                                                    channels, states, state, slot_stride, scan_off,      \
                                                                    state_slots, cu_seqlens, context_lens)
#define SCAN_R(R)                                                                                                         \
    do {                                                                                                                  \
        if (dtype == 0 && prepared) SCAN_GO(float, R, true);                                                              \
        else if (dtype == 0) SCAN_GO(float, R, false);                                                                    \
        else if (prepared) SCAN_GO(bf16, R, true);                                                                        \
        else SCAN_GO(bf16, R, false);                                                                                     \
    } while (0)
    if (r <= 1) SCAN_R(1);
    else if (r <= 2) SCAN_R(2);
    else if (r <= 4) SCAN_R(4);
    else if (r <= 8) SCAN_R(8);
    else SCAN_R(16);
#undef SCAN_R
#undef SCAN_GO
    LLMS_LAUNCH_CHECK();
}

int llms_unit_heads(float* x, int ld, int q_col, int k_col, int q_heads, int k_heads, int dk, float eps, float q_factor,
                    int n_tokens, float* gates, int g_ld, int a_col, int b_col, const float* a_log, const float* dt_bias,
                    int heads, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && q_heads >= 0 && k_heads >= 0 && q_heads + k_heads > 0 && dk > 0, "unit_heads: sizes must be positive");
    LLMS_REQUIRE(q_heads + k_heads < 65535, "unit_heads: up to 65,534 heads in all");
    LLMS_REQUIRE(!gates || (a_log && dt_bias && heads > 0), "unit_heads: gates need their rates and biases");
    dim3 grid(n_tokens, q_heads + k_heads + (gates ? 1 : 0));
    unit_heads_kernel<<<grid, LLMS_WAVE, 0, stream>>>(x, ld, q_col, k_col, q_heads, k_heads, dk, eps, q_factor, gates, g_ld, a_col,
                                                      b_col, a_log, dt_bias, heads);
    LLMS_LAUNCH_CHECK();
}

int llms_step_sizes(float* dt, int dt_ld, const float* low, int low_ld, int low_col, int rank, const float* w_t,
                    const float* dt_bias, float* z, int z_ld, int z_col, int channels, int n_tokens, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && channels > 0 && rank > 0 && rank <= 1024, "step_sizes: sizes must be positive, up to 1,024 columns");
    LLMS_REQUIRE((channels + LLMS_WAVE - 1) / LLMS_WAVE <= 65535, "step_sizes: too many channels for one launch");
    dim3 grid((n_tokens + SS_TOKENS - 1) / SS_TOKENS, (channels + LLMS_WAVE - 1) / LLMS_WAVE);
    step_sizes_kernel<<<grid, LLMS_WAVE, (size_t)rank * SS_TOKENS * sizeof(float), stream>>>(dt, dt_ld, low, low_ld, low_col, rank, w_t,
                                                                                          dt_bias, z, z_ld, z_col, channels, n_tokens);
    LLMS_LAUNCH_CHECK();
}

int llms_delta_scan(float* o, int o_ld, const float* qkv, int qkv_ld, int q_col, int k_col, int v_col, const float* gates,
                    int g_ld, int a_col, int b_col, const float* a_log, const float* dt_bias, int heads, int kv_heads, int dk,
                    int dv, float* state, size_t slot_stride, size_t scan_off, const int* state_slots, const int* cu_seqlens,
                    const int* context_lens, int n_seqs, int prepared, hipStream_t stream) {
    LLMS_REQUIRE(n_seqs > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "delta_scan: heads must be a multiple of kv_heads");
    LLMS_REQUIRE(dk > 0 && dk <= 256 && dv > 0, "delta_scan: keys of 1 to 256 numbers");
    LLMS_REQUIRE(heads <= 65535, "delta_scan: up to 65,535 heads");
    dim3 grid(n_seqs, heads, (dv + RC_THREADS / 16 - 1) / (RC_THREADS / 16));
    const int r = (dk + 15) / 16;
    // rows in 16-byte pieces where a lane's rows come in fours and every piece is aligned
    const bool vec = r % 4 == 0 && dk % 4 == 0 && qkv_ld % 4 == 0 && q_col % 4 == 0 && k_col % 4 == 0 && ((uintptr_t)qkv % 16) == 0;
#define DELTA_P(R, P, V)                                                                                                  \
    delta_scan_kernel<R, P, V><<<grid, RC_THREADS, 0, stream>>>(o, o_ld, qkv, qkv_ld, q_col, k_col, v_col, gates, g_ld, a_col, \
                                                                b_col, a_log, dt_bias, heads, kv_heads, dk, dv, state,    \
                                                                slot_stride, scan_off, state_slots, cu_seqlens, context_lens)
#define DELTA_GO(R)                                                                                                       \
    do {                                                                                                                  \
        if (prepared && vec && R % 4 == 0) DELTA_P(R, true, (R % 4 == 0));                                                \
        else if (prepared) DELTA_P(R, true, false);                                                                       \
        else if (vec && R % 4 == 0) DELTA_P(R, false, (R % 4 == 0));                                                      \
        else DELTA_P(R, false, false);                                                                                    \
    } while (0)
    if (r <= 1) DELTA_GO(1);
    else if (r <= 2) DELTA_GO(2);
    else if (r <= 4) DELTA_GO(4);
    else if (r <= 8) DELTA_GO(8);
    else DELTA_GO(16);
#undef DELTA_GO
#undef DELTA_P
    LLMS_LAUNCH_CHECK();
}

int llms_delta_finish(int dtype, void* out, int out_ld, const float* o, int o_ld, const float* gate, int gate_ld, int gate_col,
                      const float* weight, int heads, int dv, float eps, int n_tokens, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && heads > 0 && heads <= 65535 && dv > 0, "delta_finish: sizes must be positive");
    dim3 grid(n_tokens, heads);
    if (dtype == 0)
        delta_finish_kernel<float><<<grid, LLMS_WAVE, 0, stream>>>((float*)out, out_ld, o, o_ld, gate, gate_ld, gate_col, weight, dv, eps);
    else if (dtype == 1)
        delta_finish_kernel<bf16><<<grid, LLMS_WAVE, 0, stream>>>((bf16*)out, out_ld, o, o_ld, gate, gate_ld, gate_col, weight, dv, eps);
    else
        LLMS_REQUIRE(false, "delta_finish: dtype must be 0 (float32) or 1 (bfloat16)");
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
