// Products with a weight per group:  out[m, g_out + n] = sum_k x[m, g_x + k] * w[g][n][k]
//   groups as column blocks   every row meets every group; group g reads the columns g * x_gs .. + K of x and writes
//                             the columns g * out_gs .. of out (a product per head)
//   groups as row segments    rows seg[g] .. seg[g + 1] belong to group g (rows sorted by expert); a workgroup finds
//                             its group and tile from tile_start[g] = tiles of all groups before g
// Epilogues: plain; "paired" for a weight that stacks two projections a, b of a gated unit in blocks of 64 rows (32
// rows of a, then the 32 rows of b of the same units, so that a thread or lane holds both of a unit):
// out[m, u] = min(a, limit) * sigmoid(1.702 min(a, limit)) * (clamp(b, -limit, limit) + 1) for the `units` units
// (unit 0), or a * sigmoid(a) * b (unit 1);
// "gated": the result times sigmoid(z[m, g * z_gs + n]) with z in 32-bit.
// Two kernels: 32-bit multiply-add (any sizes, float or bfloat16 operands, 32-bit products and sums) and bfloat16 on
// the matrix cores (K and the strides of x in multiples of 8, 16-byte aligned operands).
#include "common.h"

#define GG_TM 64
#define GG_TN 64
#define GG_TK 16

#define GG_PLAIN 0
#define GG_PAIRED 1
#define GG_GATED 2

// which gated unit the paired epilogue forms
#define GG_UNIT_CLAMPED 0
#define GG_UNIT_SILU 1

// (the operands of the gated unit are rounded as a stored activation would be)
template <typename TOut>
__device__ __forceinline__ float gated_unit(float a_sum, float b_sum, float limit, int unit) {
    if (unit == GG_UNIT_SILU) {
        const float a = round_to<TOut>(a_sum), b = round_to<TOut>(b_sum);
        return a / (1.f + expf(-a)) * b;
    }
    const float a = fminf(round_to<TOut>(a_sum), limit);
    const float b = fminf(fmaxf(round_to<TOut>(b_sum), -limit), limit);
    return a / (1.f + expf(-1.702f * a)) * (b + 1.f);
}

template <typename TIn, typename TOut, int EPI>
__global__ __launch_bounds__(256) void grouped_fma_kernel(
    TOut* __restrict__ out, long out_ld, long out_gs, const TIn* __restrict__ x, long x_ld, long x_gs,
    const TIn* __restrict__ w, int M, int N, int K, int G, const int* __restrict__ seg, const int* __restrict__ tile_start,
    const float* __restrict__ z, long z_ld, long z_gs, float limit, int unit, int units) {
    __shared__ float As[GG_TK][GG_TM + 4];
    __shared__ float Ws[GG_TK][GG_TN + 4];
    const int tid = threadIdx.x;
    int g, row0, row_end;
    if (seg) {
        const int t = blockIdx.y;
        if (t >= tile_start[G]) return;
        g = 0;
        while (tile_start[g + 1] <= t) ++g;  // (uniform over the workgroup)
        row0 = seg[g] + (t - tile_start[g]) * GG_TM;
        row_end = seg[g + 1];
    } else {
        g = blockIdx.z;
        row0 = blockIdx.y * GG_TM;
        row_end = M;
    }
    const int n0 = blockIdx.x * GG_TN;
    const TIn* xg = x + (seg ? 0 : (size_t)g * x_gs);
    const TIn* wg = w + (size_t)g * N * K;
    // a thread's four columns: two neighbours in the first half of the tile and the same two in the second half
    const int tm = (tid / 16) * 4, tn = (tid % 16) * 2;
    auto column = [&](int j) { return tn + (j & 1) + 32 * (j >> 1); };
    const int lr = tid / 4, lk = (tid % 4) * 4;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += GG_TK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int am = row0 + lr, wn = n0 + lr;
            As[lk + i][lr] = (am < row_end && k < K) ? to_f32(xg[(size_t)am * x_ld + k]) : 0.f;
            Ws[lk + i][lr] = (wn < N && k < K) ? to_f32(wg[(size_t)wn * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GG_TK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][tm + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Ws[k][column(j)];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
    TOut* og = out + (seg ? 0 : (size_t)g * out_gs);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = row0 + tm + i;
        if (m >= row_end) continue;
        if (EPI == GG_PAIRED) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int u = n0 / 2 + tn + j;
                if (u >= units) continue;
                og[(size_t)m * out_ld + u] = from_f32<TOut>(gated_unit<TOut>(acc[i][j], acc[i][j + 2], limit, unit));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + column(j);
                if (n >= N) continue;
                float v = acc[i][j];
                if (EPI == GG_GATED) v = v / (1.f + expf(-z[(size_t)m * z_ld + (size_t)g * z_gs + n]));
                og[(size_t)m * out_ld + n] = from_f32<TOut>(v);
            }
        }
    }
}

template <typename TIn, typename TOut>
static int launch_fma(int epilogue, dim3 grid, hipStream_t stream, void* out, long out_ld, long out_gs, const void* x, long x_ld,
                      long x_gs, const void* w, int M, int N, int K, int G, const int* seg, const int* tile_start, const float* z,
                      long z_ld, long z_gs, float limit, int unit, int units) {
#define GG_GO(EPI)                                                                                                          \
    grouped_fma_kernel<TIn, TOut, EPI><<<grid, 256, 0, stream>>>((TOut*)out, out_ld, out_gs, (const TIn*)x, x_ld, x_gs,      \
                                                                 (const TIn*)w, M, N, K, G, seg, tile_start, z, z_ld, z_gs, limit, unit, units)
    if (epilogue == GG_PLAIN) GG_GO(GG_PLAIN);
    else if (epilogue == GG_PAIRED) GG_GO(GG_PAIRED);
    else GG_GO(GG_GATED);
#undef GG_GO
    LLMS_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ bfloat16 on the matrix cores
// 128 x 128 tiles, 64 of K at a time, through double-buffered LDS (72 KB: two workgroups a compute unit) with two more
// tiles of K in flight in registers, 4 waves of 64 x 64, v_mfma_f32_32x32x16_bf16: lane l holds
// A[i = l%32][k = 8*(l/32) .. +7] and B[k = same][j = l%32]; result D[i = 8*(r/4) + 4*(l/32) + r%4][j = l%32].
// Here i = row m and j = weight row n, so a wave's two column blocks of 32 are the a and b rows of the same 32 units
// of a paired weight (columns 0..31 and 32..63 of its 64), both in the same lane.
typedef __attribute__((ext_vector_type(8))) __bf16 gg_bf16x8;
typedef __attribute__((ext_vector_type(16))) float gg_f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t gg_u32x4;

#define GM_BM 128
#define GM_BN 128
#define GM_BK 64
#define GM_LD 72  // LDS row stride in elements: 64 + 8 of padding against bank conflicts
#define GM_PIECES (GM_BM * GM_BK / 8 / 256)  // 16-byte pieces of an operand tile per thread
#define GM_LDS_BYTES (2 * 2 * GM_BM * GM_LD * 2)  // two buffers of two operand tiles

template <typename TOut, int EPI>
__global__ __launch_bounds__(256) void grouped_mfma_kernel(
    TOut* __restrict__ out, long out_ld, long out_gs, const bf16* __restrict__ x, long x_ld, long x_gs,
    const bf16* __restrict__ w, int M, int N, int K, int G, const int* __restrict__ seg, const int* __restrict__ tile_start,
    const float* __restrict__ z, long z_ld, long z_gs, float limit, int unit, int units, int k_part, long part_stride) {
    extern __shared__ __attribute__((aligned(16))) uint16_t gm_lds[];
    uint16_t(*As)[GM_BM * GM_LD] = reinterpret_cast<uint16_t(*)[GM_BM * GM_LD]>(gm_lds);
    uint16_t(*Bs)[GM_BN * GM_LD] = reinterpret_cast<uint16_t(*)[GM_BN * GM_LD]>(gm_lds + 2 * GM_BM * GM_LD);
    int g, row0, row_end;
    if (seg) {
        const int t = blockIdx.y;
        if (t >= tile_start[G]) return;
        g = 0;
        while (tile_start[g + 1] <= t) ++g;  // (uniform over the workgroup)
        row0 = seg[g] + (t - tile_start[g]) * GM_BM;
        row_end = seg[g + 1];
    } else {
        g = blockIdx.z;
        row0 = blockIdx.y * GM_BM;
        row_end = M;
    }
    const int n0 = blockIdx.x * GM_BN;
    const bf16* xg = x + (seg ? 0 : (size_t)g * x_gs);
    const bf16* wg = w + (size_t)g * N * K;
    const int w_ld = K;
    const int tid = threadIdx.x, wave = tid / LLMS_WAVE, lane = tid % LLMS_WAVE;
    const int wm = (wave % 2) * 64, wn = (wave / 2) * 64;
    const int l32 = lane % 32, hi = lane / 32;
    const gg_u32x4 zero = {0, 0, 0, 0};
    gg_f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    // staging: 1,024 pieces of 8 elements per operand tile, four per thread.  Two tiles of K are in flight in two sets of
    // registers (set kt % 2 holds tile kt) beside the tile in LDS that is being multiplied: 64 KB a workgroup, which is what
    // lets few rows stream the weights near the memory's rate, and many rows hide a trip to memory behind two tiles' products.
    // A piece beyond the rows, the weight or K is not asked for and counts as zeros, so tiles past the last are fetched too.
    gg_u32x4 ra0[GM_PIECES], rb0[GM_PIECES], ra1[GM_PIECES], rb1[GM_PIECES];
    const int crow0 = tid / 8, ckc = (tid % 8) * 8;
    // (with segments the third grid dimension may share K out: part p takes k_part numbers from p * k_part on and
    // leaves its sums in an array of its own, for the caller to add up)
    const int k_begin = seg ? blockIdx.z * k_part : 0;
    const int k_end = seg ? min(K, k_begin + k_part) : K;
    const int ktiles = (k_end - k_begin + GM_BK - 1) / GM_BK;
    K = k_end;
#define GM_FETCH(RA, RB, K0)                                                                                               \
    _Pragma("unroll") for (int c = 0; c < GM_PIECES; ++c) {                                                                \
        const int k = (K0) + ckc;                                                                                          \
        const int am = row0 + crow0 + 32 * c, wr = n0 + crow0 + 32 * c;                                                    \
        RA[c] = (am < row_end && k < K) ? *reinterpret_cast<const gg_u32x4*>(xg + (size_t)am * x_ld + k) : zero;           \
        RB[c] = (wr < N && k < K) ? *reinterpret_cast<const gg_u32x4*>(wg + (size_t)wr * w_ld + k) : zero;                 \
    }
#define GM_STAGE(BUF, RA, RB)                                                                                              \
    _Pragma("unroll") for (int c = 0; c < GM_PIECES; ++c) {                                                                \
        *reinterpret_cast<gg_u32x4*>(&As[BUF][(crow0 + 32 * c) * GM_LD + ckc]) = RA[c];                                    \
        *reinterpret_cast<gg_u32x4*>(&Bs[BUF][(crow0 + 32 * c) * GM_LD + ckc]) = RB[c];                                    \
    }
#define GM_MULTIPLY(BUF)                                                                                                   \
    _Pragma("unroll") for (int s = 0; s < GM_BK / 16; ++s) {                                                               \
        gg_bf16x8 af[2], bfr[2];                                                                                           \
        _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                                                    \
            af[i] = __builtin_bit_cast(gg_bf16x8, *reinterpret_cast<const gg_u32x4*>(&As[BUF][(wm + i * 32 + l32) * GM_LD + s * 16 + hi * 8])); \
            bfr[i] = __builtin_bit_cast(gg_bf16x8, *reinterpret_cast<const gg_u32x4*>(&Bs[BUF][(wn + i * 32 + l32) * GM_LD + s * 16 + hi * 8])); \
        }                                                                                                                  \
        _Pragma("unroll") for (int i = 0; i < 2; ++i)                                                                      \
            _Pragma("unroll") for (int j = 0; j < 2; ++j)                                                                  \
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);                    \
    }
    GM_FETCH(ra0, rb0, k_begin);
    GM_FETCH(ra1, rb1, k_begin + GM_BK);
    GM_STAGE(0, ra0, rb0);
    __syncthreads();
    for (int kt = 0; kt < ktiles; kt += 2) {
        // LDS buffer 0 holds tile kt, set 1 tile kt + 1; set 0 is free for tile kt + 2
        GM_FETCH(ra0, rb0, k_begin + (kt + 2) * GM_BK);
        GM_MULTIPLY(0);
        GM_STAGE(1, ra1, rb1);
        __syncthreads();
        if (kt + 1 >= ktiles) break;
        // LDS buffer 1 holds tile kt + 1, set 0 tile kt + 2; set 1 is free for tile kt + 3
        GM_FETCH(ra1, rb1, k_begin + (kt + 3) * GM_BK);
        GM_MULTIPLY(1);
        GM_STAGE(0, ra0, rb0);
        __syncthreads();
    }
#undef GM_FETCH
#undef GM_STAGE
#undef GM_MULTIPLY
    TOut* og = out + (seg ? (size_t)blockIdx.z * part_stride : (size_t)g * out_gs);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = row0 + wm + i * 32 + 8 * (r / 4) + 4 * hi + (r % 4);
            if (m >= row_end) continue;
            if (EPI == GG_PAIRED) {
                const int u = (n0 + wn) / 2 + l32;
                if (u < units) og[(size_t)m * out_ld + u] = from_f32<TOut>(gated_unit<TOut>(acc[i][0][r], acc[i][1][r], limit, unit));
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int n = n0 + wn + j * 32 + l32;
                    if (n >= N) continue;
                    float v = acc[i][j][r];
                    if (EPI == GG_GATED) v = v / (1.f + expf(-z[(size_t)m * z_ld + (size_t)g * z_gs + n]));
                    og[(size_t)m * out_ld + n] = from_f32<TOut>(v);
                }
            }
        }
    }
}

template <typename TOut>
static int launch_mfma(int epilogue, dim3 grid, hipStream_t stream, void* out, long out_ld, long out_gs, const void* x, long x_ld,
                       long x_gs, const void* w, int M, int N, int K, int G, const int* seg, const int* tile_start, const float* z,
                       long z_ld, long z_gs, float limit, int unit, int units, int k_part, long part_stride) {
#define GM_GO(EPI)                                                                                                          \
    LLMS_HIP_CHECK(hipFuncSetAttribute((const void*)grouped_mfma_kernel<TOut, EPI>,                                         \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, GM_LDS_BYTES));                          \
    grouped_mfma_kernel<TOut, EPI><<<grid, 256, GM_LDS_BYTES, stream>>>((TOut*)out, out_ld, out_gs, (const bf16*)x, x_ld, x_gs, \
                                                             (const bf16*)w, M, N, K, G, seg, tile_start, z, z_ld, z_gs, limit, unit, units, \
                                                             k_part, part_stride)
    if (epilogue == GG_PLAIN) {
        GM_GO(GG_PLAIN);
    } else if (epilogue == GG_PAIRED) {
        GM_GO(GG_PAIRED);
    } else {
        GM_GO(GG_GATED);
    }
#undef GM_GO
    LLMS_LAUNCH_CHECK();
}

extern "C" {

// in_dtype / out_dtype: 0 = float32, 1 = bfloat16; (0,0), (1,1), (1,0).  `seg` null: groups as column blocks over all
// M rows; else groups as row segments and `max_tiles` workgroups in the grid's second dimension (at least
// tile_start[G], which the host bounds by ceil(M / 64) + G).
int llms_grouped_fma(int in_dtype, int out_dtype, int epilogue, void* out, long out_ld, long out_gs, const void* x, long x_ld,
                     long x_gs, const void* w, int M, int N, int K, int G, const int* seg, const int* tile_start,
                     int max_tiles, const float* z, long z_ld, long z_gs, float limit, int unit, int units, hipStream_t stream) {
    LLMS_REQUIRE(M > 0 && N > 0 && K > 0 && G > 0, "grouped_fma: sizes must be positive");
    LLMS_REQUIRE(epilogue >= 0 && epilogue <= 2, "grouped_fma: epilogue 0 (plain), 1 (paired) or 2 (gated)");
    LLMS_REQUIRE(epilogue != GG_PAIRED || (N % 64 == 0 && units > 0 && units <= N / 2),
                 "grouped_fma: a paired weight has blocks of 64 rows for 32 units each");
    LLMS_REQUIRE(epilogue != GG_GATED || z, "grouped_fma: the gated epilogue needs its gate products");
    LLMS_REQUIRE((seg == nullptr) == (tile_start == nullptr), "grouped_fma: segments come with their tile starts");
    dim3 grid((N + GG_TN - 1) / GG_TN, seg ? max_tiles : (M + GG_TM - 1) / GG_TM, seg ? 1 : G);
    LLMS_REQUIRE(grid.y > 0 && grid.y <= 65535 && grid.z <= 65535, "grouped_fma: too many rows or groups for one launch");
    if (in_dtype == 0 && out_dtype == 0)
        return launch_fma<float, float>(epilogue, grid, stream, out, out_ld, out_gs, x, x_ld, x_gs, w, M, N, K, G, seg, tile_start,
                                        z, z_ld, z_gs, limit, unit, units);
    if (in_dtype == 1 && out_dtype == 1)
        return launch_fma<bf16, bf16>(epilogue, grid, stream, out, out_ld, out_gs, x, x_ld, x_gs, w, M, N, K, G, seg, tile_start, z,
                                      z_ld, z_gs, limit, unit, units);
    if (in_dtype == 1 && out_dtype == 0)
        return launch_fma<bf16, float>(epilogue, grid, stream, out, out_ld, out_gs, x, x_ld, x_gs, w, M, N, K, G, seg, tile_start, z,
                                       z_ld, z_gs, limit, unit, units);
    LLMS_REQUIRE(false, "grouped_fma: unsupported dtype pair");
}

// The same on the matrix cores: bfloat16 operands, out_dtype 0 (float32) or 1 (bfloat16); tiles of 128 rows.
// `k_parts` > 1 (segments, plain epilogue, float32 result): K is shared out to that many sets of workgroups, set p
// leaving its sums at out + p * part_stride.
int llms_grouped_mfma(int out_dtype, int epilogue, void* out, long out_ld, long out_gs, const void* x, long x_ld, long x_gs,
                      const void* w, int M, int N, int K, int G, const int* seg, const int* tile_start, int max_tiles,
                      const float* z, long z_ld, long z_gs, float limit, int unit, int units, int k_parts, long part_stride,
                      hipStream_t stream) {
    LLMS_REQUIRE(M > 0 && N > 0 && K > 0 && G > 0, "grouped_mfma: sizes must be positive");
    LLMS_REQUIRE(epilogue >= 0 && epilogue <= 2, "grouped_mfma: epilogue 0 (plain), 1 (paired) or 2 (gated)");
    LLMS_REQUIRE(epilogue != GG_PAIRED || (N % 64 == 0 && units > 0 && units <= N / 2),
                 "grouped_mfma: a paired weight has blocks of 64 rows for 32 units each");
    LLMS_REQUIRE(epilogue != GG_GATED || z, "grouped_mfma: the gated epilogue needs its gate products");
    LLMS_REQUIRE((seg == nullptr) == (tile_start == nullptr), "grouped_mfma: segments come with their tile starts");
    LLMS_REQUIRE(K % 8 == 0 && x_ld % 8 == 0 && x_gs % 8 == 0, "grouped_mfma: K and the strides of x in multiples of 8");
    LLMS_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "grouped_mfma: x and w must be 16-byte aligned");
    LLMS_REQUIRE(k_parts >= 1 && k_parts <= 16, "grouped_mfma: 1 to 16 parts of K");
    LLMS_REQUIRE(k_parts == 1 || (seg && epilogue == GG_PLAIN && out_dtype == 0),
                 "grouped_mfma: K is shared out only with segments, the plain epilogue and a float32 result");
    const int k_part = k_parts == 1 ? K : ((K + k_parts - 1) / k_parts + GM_BK - 1) / GM_BK * GM_BK;
    dim3 grid((N + GM_BN - 1) / GM_BN, seg ? max_tiles : (M + GM_BM - 1) / GM_BM, seg ? k_parts : G);
    LLMS_REQUIRE(grid.y > 0 && grid.y <= 65535 && grid.z <= 65535, "grouped_mfma: too many rows or groups for one launch");
    if (out_dtype == 0)
        return launch_mfma<float>(epilogue, grid, stream, out, out_ld, out_gs, x, x_ld, x_gs, w, M, N, K, G, seg, tile_start, z, z_ld,
                                  z_gs, limit, unit, units, k_part, part_stride);
    if (out_dtype == 1)
        return launch_mfma<bf16>(epilogue, grid, stream, out, out_ld, out_gs, x, x_ld, x_gs, w, M, N, K, G, seg, tile_start, z, z_ld,
                                 z_gs, limit, unit, units, k_part, part_stride);
    LLMS_REQUIRE(false, "grouped_mfma: out_dtype must be 0 or 1");
}

}  // extern "C"
