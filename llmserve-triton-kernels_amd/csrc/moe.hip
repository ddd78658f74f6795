// Routing for a feed-forward of many small experts, of which each token uses `top`.
//   moe_router    z = W_router h in 32-bit, s = sigmoid(z) or softmax(z) over all experts, the `top` largest (the lower expert
//                 wins a tie), in descending order; weight = score or score / (sum of the chosen scores + renorm_eps).
//                 With `groups` > 1 the experts form that many equal groups of neighbours, a group's score is its largest
//                 score, and only experts of the `keep` best groups (the lower group wins a tie) can be chosen.
//                 `bias` is added to z; `extra` rows of W_router behind the experts' give extra_out = their products
//   moe_rank      for expert e: how many (token, choice) pairs chose it, and each such pair's rank among them in the
//                 order of the pairs (so the sorted order is stable and the same whatever runs beside it)
//   moe_offsets   seg[e] = pairs of all experts before e, tile_start[e] = tiles of rows of all experts before e
//   moe_scatter   rows sorted by expert: xs[seg[e] + rank] = weight * h[token] (the weight multiplies the expert's
//                 input), rounded to T, or h[token] as it is where no weight is given; place[pair] = that row
//   moe_combine   y[n] = sum over the token's choices, in their order, of the experts' results rows, each times its
//                 weight where weights are given (32-bit; a row may arrive as partial sums over shares of the last
//                 product's K, added in the order of the shares)
// A pair is p = token * top + choice.
#include "common.h"

#define MOE_THREADS 256
#define MOE_MAX_TOP 16

template <typename T>
__global__ __launch_bounds__(MOE_THREADS) void moe_router_kernel(
    int* __restrict__ chosen, float* __restrict__ weight, const T* __restrict__ h, const T* __restrict__ w_router,
    int hidden, int experts, int top, int renormalize, int softmax, int groups, int keep, float renorm_eps,
    const float* __restrict__ bias, int extra, float* __restrict__ extra_out) {
    extern __shared__ float score[];  // experts, then groups
    const int n = blockIdx.x, lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    const T* row = h + (size_t)n * hidden;
    const bool vec = hidden % (16 / sizeof(T)) == 0 && ((uintptr_t)h % 16) == 0 && ((uintptr_t)w_router % 16) == 0;
    for (int e = wave; e < experts + extra; e += MOE_THREADS / LLMS_WAVE) {
        const T* wr = w_router + (size_t)e * hidden;
        float dot = 0.f;
        if (vec) {  // 16 bytes a lane and load, four loads in flight
            constexpr int PER = 16 / sizeof(T);
            typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
            for (int c0 = lane * PER; c0 < hidden; c0 += 4 * LLMS_WAVE * PER) {
                u32x4 hv[4], wv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int c = c0 + u * LLMS_WAVE * PER;
                    const bool in = c < hidden;
                    hv[u] = in ? *reinterpret_cast<const u32x4*>(row + c) : (u32x4){0, 0, 0, 0};
                    wv[u] = in ? *reinterpret_cast<const u32x4*>(wr + c) : (u32x4){0, 0, 0, 0};
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const T* hp = reinterpret_cast<const T*>(&hv[u]);
                    const T* wp = reinterpret_cast<const T*>(&wv[u]);
#pragma unroll
                    for (int k = 0; k < PER; ++k) dot = fmaf(to_f32(hp[k]), to_f32(wp[k]), dot);
                }
            }
        } else {
            for (int c = lane; c < hidden; c += LLMS_WAVE) dot = fmaf(to_f32(row[c]), to_f32(wr[c]), dot);
        }
        dot = wave_sum(dot);
        if (e >= experts) {  // rows of the weight behind the experts': their products leave as they are
            if (lane == 0) extra_out[(size_t)n * extra + (e - experts)] = dot;
            continue;
        }
        if (bias) dot += bias[e];
        // (a row that is not a number, as a padding row may be, gets a score like any other: every choice below must
        // name an expert that exists)
        if (lane == 0) score[e] = dot == dot ? (softmax ? dot : 1.f / (1.f + expf(-dot))) : 0.f;
    }
    __syncthreads();
    if (wave != 0) return;
    if (softmax) {  // over all experts, in 32-bit: exp(z - max) / sum
        float top_z = -INFINITY;
        for (int e = lane; e < experts; e += LLMS_WAVE) top_z = fmaxf(top_z, score[e]);
        top_z = wave_max(top_z);
        float total = 0.f;
        for (int e = lane; e < experts; e += LLMS_WAVE) {
            const float w = expf(score[e] - top_z);
            score[e] = w;
            total += w;
        }
        total = wave_sum(total);
        for (int e = lane; e < experts; e += LLMS_WAVE) score[e] = score[e] / total;
        __builtin_amdgcn_s_waitcnt(0);
        __builtin_amdgcn_wave_barrier();
    }
    if (groups > 1) {  // experts outside the `keep` best groups are marked taken
        float* best_of = score + experts;
        const int per = experts / groups;
        for (int g = lane; g < groups; g += LLMS_WAVE) {
            float b = -1.f;
            for (int e = g * per; e < (g + 1) * per; ++e) b = fmaxf(b, score[e]);
            best_of[g] = b;
        }
        __builtin_amdgcn_s_waitcnt(0);
        __builtin_amdgcn_wave_barrier();
        for (int k = 0; k < keep; ++k) {
            float best = -1.f;
            int at = 0x7fffffff;
            for (int g = lane; g < groups; g += LLMS_WAVE) {
                const float b = best_of[g];
                if (b > best) {
                    best = b;
                    at = g;
                }
            }
#pragma unroll
            for (int o = LLMS_WAVE / 2; o > 0; o >>= 1) {
                const float ob = __shfl_xor(best, o, LLMS_WAVE);
                const int oa = __shfl_xor(at, o, LLMS_WAVE);
                if (ob > best || (ob == best && oa < at)) {
                    best = ob;
                    at = oa;
                }
            }
            at = min(at, groups - 1);
            if (lane == 0) best_of[at] = -3.f;  // kept
            __builtin_amdgcn_s_waitcnt(0);
            __builtin_amdgcn_wave_barrier();
        }
        for (int e = lane; e < experts; e += LLMS_WAVE)
            if (best_of[e / per] != -3.f) score[e] = -2.f;
        __builtin_amdgcn_s_waitcnt(0);
        __builtin_amdgcn_wave_barrier();
    }
    float picked[MOE_MAX_TOP];
    int which[MOE_MAX_TOP];
    float sum = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = -1.f;  // (scores are in (0, 1); a taken expert is marked -2)
        int at = 0x7fffffff;
        for (int e = lane; e < experts; e += LLMS_WAVE) {
            const float s = score[e];
            if (s > best) {
                best = s;
                at = e;
            }
        }
#pragma unroll
        for (int o = LLMS_WAVE / 2; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, LLMS_WAVE);
            const int oa = __shfl_xor(at, o, LLMS_WAVE);
            if (ob > best || (ob == best && oa < at)) {
                best = ob;
                at = oa;
            }
        }
        at = min(at, experts - 1);
        picked[k] = best;
        which[k] = at;
        sum += best;
        if (lane == 0) score[at] = -2.f;
        __builtin_amdgcn_s_waitcnt(0);
        __builtin_amdgcn_wave_barrier();
    }
    if (lane == 0)
        for (int k = 0; k < top; ++k) {
            chosen[(size_t)n * top + k] = which[k];
            weight[(size_t)n * top + k] = renormalize ? picked[k] / (sum + renorm_eps) : picked[k];
        }
}

// grid: experts.  One workgroup walks all pairs in order, 256 at a time.
__global__ __launch_bounds__(MOE_THREADS) void moe_rank_kernel(int* __restrict__ count, int* __restrict__ rank,
                                                               const int* __restrict__ chosen, int pairs) {
    __shared__ int wave_total[MOE_THREADS / LLMS_WAVE];
    const int e = blockIdx.x, lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    int base = 0;
    for (int p0 = 0; p0 < pairs; p0 += MOE_THREADS) {
        const int p = p0 + threadIdx.x;
        const bool mine = p < pairs && chosen[p] == e;
        const unsigned long long votes = __ballot(mine);
        const int before = __popcll(votes & ((1ull << lane) - 1ull));
        if (lane == 0) wave_total[wave] = __popcll(votes);
        __syncthreads();
        int ahead = 0, all = 0;
#pragma unroll
        for (int w = 0; w < MOE_THREADS / LLMS_WAVE; ++w) {
            ahead += w < wave ? wave_total[w] : 0;
            all += wave_total[w];
        }
        if (mine) rank[p] = base + ahead + before;
        base += all;
        __syncthreads();
    }
    if (threadIdx.x == 0) count[e] = base;
}

// one workgroup of one thread's work: experts are few.  tile_start [2, experts + 1]: for tiles of `tile_a` and of
// `tile_b` rows (the two kernels that multiply segments of rows have tiles of different heights)
__global__ void moe_offsets_kernel(int* __restrict__ seg, int* __restrict__ tile_start, const int* __restrict__ count,
                                   int experts, int tile_a, int tile_b) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    int rows = 0, tiles_a = 0, tiles_b = 0;
    for (int e = 0; e < experts; ++e) {
        seg[e] = rows;
        tile_start[e] = tiles_a;
        tile_start[experts + 1 + e] = tiles_b;
        rows += count[e];
        tiles_a += (count[e] + tile_a - 1) / tile_a;
        tiles_b += (count[e] + tile_b - 1) / tile_b;
    }
    seg[experts] = rows;
    tile_start[experts] = tiles_a;
    tile_start[2 * experts + 1] = tiles_b;
}

// grid: pairs
template <typename T>
__global__ __launch_bounds__(MOE_THREADS) void moe_scatter_kernel(
    T* __restrict__ xs, int* __restrict__ place, const T* __restrict__ h, const int* __restrict__ chosen,
    const float* __restrict__ weight, const int* __restrict__ rank, const int* __restrict__ seg, int hidden, int top) {
    const int p = blockIdx.x, n = p / top;
    const int dest = seg[chosen[p]] + rank[p];
    if (threadIdx.x == 0) place[p] = dest;
    const T* src = h + (size_t)n * hidden;
    T* dst = xs + (size_t)dest * hidden;
    if (!weight) {
        for (int c = threadIdx.x; c < hidden; c += MOE_THREADS) dst[c] = src[c];
        return;
    }
    const float wgt = weight[p];
    for (int c = threadIdx.x; c < hidden; c += MOE_THREADS) dst[c] = from_f32<T>(wgt * to_f32(src[c]));
}

// Few pairs (decoding): the sort and the scatter in one launch.  grid: pairs; dynamic LDS: experts ints (used by the first
// workgroup).  Every workgroup reads all choices and counts, for its own pair p of expert e, the pairs of experts before e
// and the earlier pairs of e itself: their sum is the pair's row in the order sorted stably by expert, the same row as
// moe_rank, moe_offsets and moe_scatter give.  The first workgroup also counts every expert's pairs and leaves seg and
// tile_start.
template <typename T>
__global__ __launch_bounds__(MOE_THREADS) void moe_place_few_kernel(
    T* __restrict__ xs, int* __restrict__ place, int* __restrict__ seg, int* __restrict__ tile_start, const T* __restrict__ h,
    const int* __restrict__ chosen, const float* __restrict__ weight, int pairs, int hidden, int top, int experts, int tile_a,
    int tile_b) {
    extern __shared__ int hist[];
    __shared__ float red[16];
    const int p = blockIdx.x, n = p / top, e = chosen[p];
    int ahead = 0;
    for (int q = threadIdx.x; q < pairs; q += MOE_THREADS) {
        const int c = chosen[q];
        ahead += (c < e || (c == e && q < p)) ? 1 : 0;
    }
    const int dest = (int)block_sum((float)ahead, red);  // (whole numbers far below 2^24: exact)
    if (threadIdx.x == 0) place[p] = dest;
    const T* src = h + (size_t)n * hidden;
    T* dst = xs + (size_t)dest * hidden;
    if (!weight) {
        for (int c = threadIdx.x; c < hidden; c += MOE_THREADS) dst[c] = src[c];
    } else {
        const float wgt = weight[p];
        for (int c = threadIdx.x; c < hidden; c += MOE_THREADS) dst[c] = from_f32<T>(wgt * to_f32(src[c]));
    }
    if (p != 0) return;
    for (int i = threadIdx.x; i < experts; i += MOE_THREADS) hist[i] = 0;
    __syncthreads();
    for (int q = threadIdx.x; q < pairs; q += MOE_THREADS) atomicAdd(&hist[chosen[q]], 1);
    __syncthreads();
    if (threadIdx.x != 0) return;
    int rows = 0, tiles_a = 0, tiles_b = 0;
    for (int i = 0; i < experts; ++i) {
        seg[i] = rows;
        tile_start[i] = tiles_a;
        tile_start[experts + 1 + i] = tiles_b;
        rows += hist[i];
        tiles_a += (hist[i] + tile_a - 1) / tile_a;
        tiles_b += (hist[i] + tile_b - 1) / tile_b;
    }
    seg[experts] = rows;
    tile_start[experts] = tiles_a;
    tile_start[2 * experts + 1] = tiles_b;
}

// grid: tokens.  rows [parts, pairs, hidden]: a choice's result may arrive as several partial sums
__global__ __launch_bounds__(MOE_THREADS) void moe_combine_kernel(float* __restrict__ y, const float* __restrict__ rows,
                                                                  const int* __restrict__ place, int hidden, int top,
                                                                  int parts, long part_stride,
                                                                  const float* __restrict__ weight,
                                                                  const float* __restrict__ always,
                                                                  const float* __restrict__ always_gate) {
    const int n = blockIdx.x;
    float always_w = 0.f;  // what every token adds beside its choices: sigmoid(gate[n]) * always[n] (gate null: 1)
    if (always) always_w = always_gate ? 1.f / (1.f + expf(-always_gate[n])) : 1.f;
    if (hidden % 4 == 0 && part_stride % 4 == 0 && ((uintptr_t)rows % 16) == 0 && ((uintptr_t)y % 16) == 0 &&
        ((uintptr_t)always % 16) == 0) {
        // 16 bytes a thread and load, the loads of four summands in flight together
        for (int c = 4 * threadIdx.x; c < hidden; c += 4 * MOE_THREADS) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            const int terms = top * parts;
            for (int t0 = 0; t0 < terms; t0 += 4) {
                float4 part[4];
                float wk[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int t = t0 + u, k = t / parts, p = t - k * parts;
                    wk[u] = (weight && t < terms) ? weight[(size_t)n * top + k] : 1.f;
                    part[u] = t < terms ? *reinterpret_cast<const float4*>(rows + (size_t)place[(size_t)n * top + k] * hidden +
                                                                           (size_t)p * part_stride + c)
                                        : make_float4(0.f, 0.f, 0.f, 0.f);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (weight) {
                        v.x = fmaf(wk[u], part[u].x, v.x), v.y = fmaf(wk[u], part[u].y, v.y);
                        v.z = fmaf(wk[u], part[u].z, v.z), v.w = fmaf(wk[u], part[u].w, v.w);
                    } else {
                        v.x += part[u].x, v.y += part[u].y, v.z += part[u].z, v.w += part[u].w;
                    }
                }
            }
            if (always) {
                const float4 a = *reinterpret_cast<const float4*>(always + (size_t)n * hidden + c);
                v.x = fmaf(always_w, a.x, v.x), v.y = fmaf(always_w, a.y, v.y);
                v.z = fmaf(always_w, a.z, v.z), v.w = fmaf(always_w, a.w, v.w);
            }
            *reinterpret_cast<float4*>(y + (size_t)n * hidden + c) = v;
        }
        return;
    }
    for (int c = threadIdx.x; c < hidden; c += MOE_THREADS) {
        float v = 0.f;
        for (int k = 0; k < top; ++k) {
            const float* row = rows + (size_t)place[(size_t)n * top + k] * hidden + c;
            const float wk = weight ? weight[(size_t)n * top + k] : 1.f;
            for (int p = 0; p < parts; ++p) v = weight ? fmaf(wk, row[(size_t)p * part_stride], v) : v + row[(size_t)p * part_stride];
        }
        if (always) v = fmaf(always_w, always[(size_t)n * hidden + c], v);
        y[(size_t)n * hidden + c] = v;
    }
}

extern "C" {

int llms_moe_router(int dtype, int* chosen, float* weight, const void* h, const void* w_router, int n, int hidden, int experts,
                    int top, int renormalize, int softmax, int groups, int keep, float renorm_eps, const float* bias, int extra,
                    float* extra_out, hipStream_t stream) {
    LLMS_REQUIRE(n > 0 && hidden > 0 && experts > 0, "moe_router: sizes must be positive");
    LLMS_REQUIRE(extra >= 0 && (extra == 0 || extra_out), "moe_router: extra rows need a place for their products");
    LLMS_REQUIRE(top >= 1 && top <= MOE_MAX_TOP && top <= experts, "moe_router: 1 to 16 choices, no more than there are experts");
    LLMS_REQUIRE(experts <= 8192, "moe_router: up to 8,192 experts");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "moe_router: dtype must be 0 (float32) or 1 (bfloat16)");
    LLMS_REQUIRE(groups >= 1 && experts % groups == 0 && keep >= 1 && keep <= groups,
                 "moe_router: the groups must share the experts out equally, and 1 to all of them are kept");
    LLMS_REQUIRE(groups == 1 || top <= keep * (experts / groups), "moe_router: the kept groups hold fewer experts than are chosen");
    const size_t lds = (size_t)(experts + groups) * sizeof(float);
    if (dtype == 0)
        moe_router_kernel<float><<<n, MOE_THREADS, lds, stream>>>(chosen, weight, (const float*)h, (const float*)w_router, hidden,
                                                                  experts, top, renormalize, softmax, groups, keep, renorm_eps, bias, extra, extra_out);
    else
        moe_router_kernel<bf16><<<n, MOE_THREADS, lds, stream>>>(chosen, weight, (const bf16*)h, (const bf16*)w_router, hidden,
                                                                 experts, top, renormalize, softmax, groups, keep, renorm_eps, bias, extra, extra_out);
    LLMS_LAUNCH_CHECK();
}

// count [E], rank [pairs], seg [E + 1], tile_start [2, E + 1]
int llms_moe_sort(int* count, int* rank, int* seg, int* tile_start, const int* chosen, int pairs, int experts, int tile_a,
                  int tile_b, hipStream_t stream) {
    LLMS_REQUIRE(pairs > 0 && experts > 0 && tile_a > 0 && tile_b > 0, "moe_sort: sizes must be positive");
    moe_rank_kernel<<<experts, MOE_THREADS, 0, stream>>>(count, rank, chosen, pairs);
    moe_offsets_kernel<<<1, 64, 0, stream>>>(seg, tile_start, count, experts, tile_a, tile_b);
    LLMS_LAUNCH_CHECK();
}

int llms_moe_scatter(int dtype, void* xs, int* place, const void* h, const int* chosen, const float* weight, const int* rank,
                     const int* seg, int pairs, int hidden, int top, hipStream_t stream) {
    LLMS_REQUIRE(pairs > 0 && hidden > 0 && top > 0, "moe_scatter: sizes must be positive");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "moe_scatter: dtype must be 0 (float32) or 1 (bfloat16)");
    if (dtype == 0)
        moe_scatter_kernel<float><<<pairs, MOE_THREADS, 0, stream>>>((float*)xs, place, (const float*)h, chosen, weight, rank, seg,
                                                                     hidden, top);
    else
        moe_scatter_kernel<bf16><<<pairs, MOE_THREADS, 0, stream>>>((bf16*)xs, place, (const bf16*)h, chosen, weight, rank, seg,
                                                                    hidden, top);
    LLMS_LAUNCH_CHECK();
}

// seg [E + 1], tile_start [2, E + 1], place [pairs], xs [pairs, hidden]: llms_moe_sort and llms_moe_scatter in one launch,
// for up to 2,048 pairs.
int llms_moe_place_few(int dtype, void* xs, int* place, int* seg, int* tile_start, const void* h, const int* chosen,
                       const float* weight, int pairs, int hidden, int top, int experts, int tile_a, int tile_b,
                       hipStream_t stream) {
    LLMS_REQUIRE(pairs > 0 && pairs <= 2048 && hidden > 0 && top > 0, "moe_place_few: 1 to 2,048 pairs");
    LLMS_REQUIRE(experts > 0 && experts <= 8192 && tile_a > 0 && tile_b > 0, "moe_place_few: up to 8,192 experts");
    LLMS_REQUIRE(dtype == 0 || dtype == 1, "moe_place_few: dtype must be 0 (float32) or 1 (bfloat16)");
    const size_t lds = (size_t)experts * sizeof(int);
    if (dtype == 0)
        moe_place_few_kernel<float><<<pairs, MOE_THREADS, lds, stream>>>((float*)xs, place, seg, tile_start, (const float*)h,
                                                                         chosen, weight, pairs, hidden, top, experts, tile_a, tile_b);
    else
        moe_place_few_kernel<bf16><<<pairs, MOE_THREADS, lds, stream>>>((bf16*)xs, place, seg, tile_start, (const bf16*)h, chosen,
                                                                        weight, pairs, hidden, top, experts, tile_a, tile_b);
    LLMS_LAUNCH_CHECK();
}

int llms_moe_combine(float* y, const float* rows, const int* place, int n, int hidden, int top, int parts, long part_stride,
                     const float* weight, const float* always, const float* always_gate, hipStream_t stream) {
    LLMS_REQUIRE(n > 0 && hidden > 0 && top > 0 && parts > 0, "moe_combine: sizes must be positive");
    moe_combine_kernel<<<n, MOE_THREADS, 0, stream>>>(y, rows, place, hidden, top, parts, part_stride, weight, always, always_gate);
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
