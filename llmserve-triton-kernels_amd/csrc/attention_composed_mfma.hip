// The composed attention (see attention_composed.hip for its ingredients) on the matrix cores, bfloat16 storage.
//
// A *unit* is 16 columns that share a key/value head: `tpw` neighbouring tokens of one request times the `grp`
// query heads of that key/value head (grp <= 16; columns beyond tpw * grp are padding).  A wave owns one or two
// units.  Per tile of 16 keys it forms S^T = K Q^T with v_mfma_f32_16x16x16_bf16: the key rows are the A operand as
// they lie in a page, the queries the B operand, and the result holds, per lane, 4 keys of one column, which is
// exactly the B operand of O^T = V^T P^T; the values, transposed inside a page, are its A operand as they lie.
// Scores, softmax, the mixing of heads and the difference of two maps are 32-bit; the weights are rounded to
// bfloat16 only as the operand of the value product.
//
//   MAPS = 2   two score maps per query head over the same values, kept side by side in one wave (online
//              softmax each), o = a_1 - lambda a_2, optionally normed per head.  A workgroup is 4 units of one
//              key/value head; the grid runs over requests, blocks of tokens and key/value heads.
//   TALK       the heads' normalised weights are mixed before they meet the values, so a workgroup holds every head
//              of its tokens (up to 32 units in up to 16 waves) and walks the keys twice: once for every column's
//              maximum and sum, once more to form the normalised weights, which go through LDS ([token][head][key],
//              32-bit), are mixed per column by sum_g talk[h, g] w_g, and then multiply the values.
//   neither    plain softmax attention with the same masks and slopes.
//
// Keys are walked in groups of TG tiles: all of a group's key rows are asked for before the first product, all its
// values before the softmax arithmetic, so a wave waits for memory once per 16 TG keys.  When a workgroup holds no
// more tokens than one unit (decoding), the groups are dealt to `slices` waves per unit, which merge through LDS at
// the end (maxima, sums and partial results; with TALK the maxima and sums after the first walk, the partial
// results, already normalised, after the second).
//
// Masks: a column at position i sees j <= i with j >= its chunk's start and (i - j < window or j < keep_first).
// The tiles a workgroup walks are those its first token can reach up to its last token's position, and before
// them the tiles of the kept first keys; what a column does not see is masked by comparison.  Keys of pages that
// were given back (table entry < 0) and values behind the request's end are read as zeros.
#include "common.h"

#include <type_traits>

#define AM_PAGE_CACHE 1024  // page ids (4 bytes each) a workgroup keeps in LDS

#define LOG2E 1.4426950408889634f
#define NOTHING_YET (-1.0e30f)

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

struct MfmaArgs {
    bf16* out;
    const bf16* q;
    const bf16* k_pool;
    const bf16* v_pool;
    const int* block_tables;
    const int* table_rows;
    const int* cu_seqlens;
    const int* context_lens;
    const float* slopes;
    const float* talk;
    const float* dist_bias;  // [heads, dist_reach + 1]: a bias per head and distance, the last entry for everything beyond; or null
    const float* gate;       // 32-bit products [N, gate_stride]: the result is multiplied by their sigmoid; or null
    int dist_reach, gate_stride;
    int out_stride, q_stride, max_blocks;
    int seq_begin, n_seqs, blocks_per_seq;
    int heads, kv_heads, grp, dk, dv, block_size;
    int window, keep_first, chunk;
    int tok, tpw, upk, units, kv_per_wg, slices;
    unsigned bs_magic;  // ceil(2^32 / block_size): key / block_size is one multiply-high
    // a request's keys shared out to `shares` workgroups (grid z), with TALK: mode 1 leaves every column's maximum and
    // sum over its share in ws_stats [row][head][share][2] and ends; mode 2 takes them from there, walks its share once
    // more and leaves its part of the result, 32-bit, in ws_o [share][row][heads * dv]; a last kernel adds the parts up
    int shares, mode, ws_rows;
    float* ws_stats;
    float* ws_o;
    float scale, lambda, eps, out_scale;
    int head_norm;
    int sink;  // the softmax's denominator holds one more term, exp(0) (without mixed heads)
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }  // v_exp_f32; 0 for -inf

__device__ __forceinline__ s16x4 load4(const bf16* p) { return *reinterpret_cast<const s16x4*>(p); }

__device__ __forceinline__ s16x4 pack4(float a, float b, float c, float d) {
    typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
    const u32x2 v = {pack_bf16x2(a, b), pack_bf16x2(c, d)};
    return __builtin_bit_cast(s16x4, v);
}

__device__ __forceinline__ float column_max(float v) {  // over the 4 lanes that share a column
    v = fmaxf(v, __shfl_xor(v, 16, LLMS_WAVE));
    return fmaxf(v, __shfl_xor(v, 32, LLMS_WAVE));
}

__device__ __forceinline__ float column_sum(float v) {
    v += __shfl_xor(v, 16, LLMS_WAVE);
    return v + __shfl_xor(v, 32, LLMS_WAVE);
}

template <int MAPS, bool TALK, int MAXTK, int MAXTV, int MAXU, int TG, int THREADS>
__global__ __launch_bounds__(THREADS) void attend_mfma_kernel(const MfmaArgs a) {
    extern __shared__ float lds_all[];
    int* pages_s = reinterpret_cast<int*>(lds_all);  // the request's page ids over the keys this workgroup walks
    float* lds = lds_all + AM_PAGE_CACHE;
    const int wave = threadIdx.x / LLMS_WAVE, lane = threadIdx.x % LLMS_WAVE, nwaves = blockDim.x / LLMS_WAVE;
    const int col = lane % 16, q4 = lane / 16;
    const int NS = a.slices, slice = wave % NS, uw = wave / NS, n_uw = nwaves / NS;
    // blocks of tokens are handed out from every request's end: the last block sees the most keys and should not
    // be the last to start
    const int b = a.seq_begin + blockIdx.x % a.n_seqs, blk = a.blocks_per_seq - 1 - blockIdx.x / a.n_seqs;
    const int row0 = a.cu_seqlens[b], count = a.cu_seqlens[b + 1] - row0;
    const int end = a.context_lens[b];
    const int t0 = blk * a.tok;
    if (t0 >= count || end <= 0) return;  // (the same for every thread of the workgroup)
    const int ntok = count - t0 < a.tok ? count - t0 : a.tok;
    const int pos_lo = end - count + t0, pos_hi = pos_lo + ntok - 1;
    const int* table = a.block_tables + (size_t)(a.table_rows ? a.table_rows[b] : b) * a.max_blocks;
    const int kv_base = blockIdx.y * a.kv_per_wg;
    const int H = a.heads, G = a.kv_heads, dk = a.dk, dv = a.dv, bs = a.block_size;
    const int dkt = dk / 16, dvt = dv / 16;
    const int used_cols = a.tpw * a.grp;

    // the tiles of 16 keys to walk: those of kept first keys that the first token's window has passed, then from
    // the first key the first token reaches to the last token's own
    const int lo_chunk = a.chunk > 0 ? pos_lo / a.chunk * a.chunk : 0;
    const int lo_win = (a.window > 0 && pos_lo - a.window + 1 > 0) ? pos_lo - a.window + 1 : 0;
    const int main_begin = (lo_chunk > lo_win ? lo_chunk : lo_win) / 16, main_end = pos_hi / 16 + 1;
    int sink_begin = lo_chunk / 16, sink_end = (a.keep_first + 15) / 16;
    if (sink_end > main_begin) sink_end = main_begin;
    if (a.window <= 0 || sink_end < sink_begin) sink_end = sink_begin;
    const int n_sink = sink_end - sink_begin;
    const int n_tiles = n_sink + (main_end - main_begin);
    const int n_groups = (n_tiles + TG - 1) / TG;
    const int NSG = a.shares, share = blockIdx.z;
    const int n_rounds = (n_groups + NS * NSG - 1) / (NS * NSG);  // every slice walks this many groups (the last may be empty)
    // groups behind this one hold only tiles whose keys the first token reaches: their pages are all there
    const int first_plain = n_sink / TG + 1;
    // the pages of the walked keys (those from the first reachable key on; up to AM_PAGE_CACHE of them) are read once
    const int first_block = (int)__umulhi((unsigned)(main_begin * 16), a.bs_magic);
    int cached = (int)__umulhi((unsigned)end, a.bs_magic) + 1 - first_block;
    if (cached > AM_PAGE_CACHE) cached = AM_PAGE_CACHE;
    for (int i = threadIdx.x; i < cached; i += blockDim.x) pages_s[i] = first_block + i < a.max_blocks ? table[first_block + i] : -1;
    __syncthreads();
    // (one load through a pointer chosen between LDS and memory: no branch stands between the loads of a group)
    auto block_of = [&](int key) { return (int)__umulhi((unsigned)key, a.bs_magic); };
    auto page_at = [&](int block) {
        const int i = block - first_block;
        const int* at = (i >= 0 && i < cached) ? static_cast<const int*>(pages_s + i) : table + block;
        return *at;
    };
    // first key of tile i; tiles behind the last lie behind every token's position and hold nothing
    auto tile_start = [&](int i) { return 16 * (i < n_sink ? sink_begin + i : main_begin + (i - n_sink)); };

    // this wave's units and columns
    bool valid[MAXU], mine[MAXU];
    int u_kvh[MAXU], u_h[MAXU], u_tl[MAXU], u_pos[MAXU], u_chunk_lo[MAXU];
    float u_slope[MAXU], u_far[MAXU];
    const float* u_bias[MAXU];  // the column's head's row of the distance table
    int u_pmin[MAXU], u_pmax[MAXU];
    s16x4 qf[MAXU][MAPS][MAXTK];
#pragma unroll
    for (int uu = 0; uu < MAXU; ++uu) {
        const int u = uw + uu * n_uw;
        mine[uu] = u < a.units;
        const int kvh = kv_base + (mine[uu] ? u / a.upk : 0), sub = mine[uu] ? u % a.upk : 0;
        const int tl = sub * a.tpw + col / a.grp, h = kvh * a.grp + col % a.grp;
        valid[uu] = mine[uu] && col < used_cols && tl < ntok;
        u_kvh[uu] = kvh, u_h[uu] = h, u_tl[uu] = tl, u_pos[uu] = pos_lo + tl;
        u_chunk_lo[uu] = a.chunk > 0 ? u_pos[uu] / a.chunk * a.chunk : 0;
        u_slope[uu] = (a.slopes && valid[uu]) ? a.slopes[h] * LOG2E : 0.f;
        u_bias[uu] = a.dist_bias ? a.dist_bias + (size_t)(valid[uu] ? h : 0) * (a.dist_reach + 1) : nullptr;
        u_far[uu] = a.dist_bias ? u_bias[uu][a.dist_reach] * LOG2E : 0.f;
        // the unit's first and last position (the same for all its lanes): a tile that all of them see whole
        // needs no comparisons
        u_pmin[uu] = pos_lo + sub * a.tpw;
        u_pmax[uu] = u_pmin[uu] + a.tpw - 1 < pos_hi ? u_pmin[uu] + a.tpw - 1 : pos_hi;
        const bf16* qrow = a.q + (size_t)(row0 + t0 + tl) * a.q_stride + (size_t)h * MAPS * dk + 4 * q4;
#pragma unroll
        for (int m = 0; m < MAPS; ++m)
#pragma unroll
            for (int t = 0; t < MAXTK; ++t)
                qf[uu][m][t] = (valid[uu] && t < dkt) ? load4(qrow + m * dk + 16 * t) : s16x4{0, 0, 0, 0};  // (once; rows of padding are not read)
    }

    // scores of one group of tiles for one unit and map: per tile 4 keys (j0 + 4 q4 + r) of the lane's column,
    // masked to -inf.  Every lane takes part, also one whose column is padding: it still brings a key's row.
    // scores are kept in units of log 2 (scale and slopes carry the factor), so a weight is one subtraction and one
    // v_exp_f32; a maximum of -inf (nothing seen yet) is replaced by a large negative number, so that exp2(-inf - m) is 0
    const float scale2 = a.scale * LOG2E;
    const size_t k_page = (size_t)G * MAPS * bs * dk, v_page = (size_t)G * dv * bs;  // elements in a page
    // A group is *plain* when pages hold a multiple of 16 keys, keys and values are as wide as the kernel's tiles, and
    // all its keys are there, on pages whose ids are in LDS: then a tile's page and place are the same for every
    // lane, worked out by the scalar unit, and a lane adds only its own fixed offset.
    auto plain_group = [&](int group) {
        if constexpr (TALK) return false;  // (with mixed heads the second set of loops did not fit the 128 registers of 16 waves)
        const int last = tile_start(group * TG + TG - 1) + 15;
        return (bs & 15) == 0 && dkt == MAXTK && dvt == MAXTV && group > first_plain && group * TG + TG <= n_tiles &&
               last <= pos_hi && block_of(last) - first_block < cached;
    };
    const int lane_k = col * dk + 4 * q4, lane_v = col * bs + 4 * q4;
    const bool sloped = a.slopes != nullptr;
    auto scores = [&](auto plain_tag, int uu, int m, int group, float sc[TG][4]) {
        constexpr bool PLAIN = decltype(plain_tag)::value;
        s16x4 kf[TG][MAXTK];
        const bf16* kbase = a.k_pool + (size_t)(u_kvh[uu] * MAPS + m) * bs * dk + 4 * q4;
        if constexpr (PLAIN) {
            const int head = __builtin_amdgcn_readfirstlane(u_kvh[uu]) * MAPS + m;
#pragma unroll
            for (int tt = 0; tt < TG; ++tt) {
                const int j0 = tile_start(group * TG + tt), block = block_of(j0);
                const int page = __builtin_amdgcn_readfirstlane(pages_s[block - first_block]);
                const bf16* tile = a.k_pool + (size_t)page * k_page + ((size_t)head * bs + (j0 - block * bs)) * dk;
#pragma unroll
                for (int t = 0; t < MAXTK; ++t) kf[tt][t] = load4(tile + lane_k + 16 * t);
            }
        } else {
#pragma unroll
        for (int tt = 0; tt < TG; ++tt) {
            const int j = tile_start(group * TG + tt) + col;  // the key whose row this lane brings
            // every load is issued whatever it brings (a key that is not there reads the request's first row and is
            // replaced by zeros afterwards): a branch around a load would make the wave wait for all loads in flight
            const int jj = j <= pos_hi ? j : pos_lo;
            const int block = block_of(jj);
            const int got = page_at(block);
            const int page = j <= pos_hi ? got : -1;
            const bf16* krow = kbase + (size_t)(page < 0 ? 0 : page) * k_page + (jj - block * bs) * dk;
#pragma unroll
            for (int t = 0; t < MAXTK; ++t) {
                const s16x4 k = load4(krow + (t < dkt ? 16 * t : 0));
                kf[tt][t] = (page >= 0 && t < dkt) ? k : s16x4{0, 0, 0, 0};
            }
        }
        }
        const int pos = u_pos[uu];
#pragma unroll
        for (int tt = 0; tt < TG; ++tt) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < MAXTK; ++t)  // (tiles beyond the keys' size hold zeros)
                acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kf[tt][t], qf[uu][m][t], acc, 0, 0, 0);
            const int j0 = tile_start(group * TG + tt);
            const float dist0 = (float)(pos - j0 - 4 * q4);
            // all the unit's positions see all 16 keys (the same answer in every lane): no comparison per key; a
            // column of padding then holds numbers that nobody reads
            const bool whole = j0 + 15 <= u_pmin[uu] && (a.chunk <= 0 || j0 >= u_pmax[uu] / a.chunk * a.chunk) &&
                               (a.window <= 0 || u_pmax[uu] - j0 < a.window);
            if (whole && !sloped) {
#pragma unroll
                for (int r = 0; r < 4; ++r) sc[tt][r] = acc[r] * scale2;
            } else if (whole) {
#pragma unroll
                for (int r = 0; r < 4; ++r) sc[tt][r] = acc[r] * scale2 - u_slope[uu] * (dist0 - (float)r);
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = j0 + 4 * q4 + r;
                    const bool vis = valid[uu] && key <= pos && key >= u_chunk_lo[uu] &&
                                     (a.window <= 0 || pos - key < a.window || key < a.keep_first);
                    sc[tt][r] = vis ? acc[r] * scale2 - u_slope[uu] * (dist0 - (float)r) : -INFINITY;
                }
            }
            if (a.dist_bias) {  // the table's entry of every key's distance; a tile that lies beyond the table's reach for all has one
                const int d0 = pos - j0 - 4 * q4;
                if (__all(d0 - 3 >= a.dist_reach)) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) sc[tt][r] += u_far[uu];
                } else {
                    float bias[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {  // (a key that is not seen holds -inf already; its entry is read from a place that exists)
                        const int d = d0 - r;
                        bias[r] = u_bias[uu][d < 0 ? 0 : (d < a.dist_reach ? d : a.dist_reach)];
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) sc[tt][r] = fmaf(bias[r], LOG2E, sc[tt][r]);
                }
            }
        }
    };
    // the values of key/value head u_kvh for one group: per tile, keys j0 + 4 q4 .. + 3 of dimension 16 t + col
    auto load_values = [&](auto plain_tag, int uu, int group, s16x4 vf[TG][MAXTV]) {
        constexpr bool PLAIN = decltype(plain_tag)::value;
        if constexpr (PLAIN) {
            const int head = __builtin_amdgcn_readfirstlane(u_kvh[uu]);
#pragma unroll
            for (int tt = 0; tt < TG; ++tt) {
                const int j0 = tile_start(group * TG + tt), block = block_of(j0);
                const int page = __builtin_amdgcn_readfirstlane(pages_s[block - first_block]);
                const bf16* tile = a.v_pool + (size_t)page * v_page + (size_t)head * dv * bs + (j0 - block * bs);
#pragma unroll
                for (int t = 0; t < MAXTV; ++t) vf[tt][t] = load4(tile + lane_v + (size_t)16 * t * bs);
            }
            return;
        }
        const bf16* vbase = a.v_pool + ((size_t)u_kvh[uu] * dv + col) * bs;
#pragma unroll
        for (int tt = 0; tt < TG; ++tt) {
            const int key = tile_start(group * TG + tt) + 4 * q4;
            const int kk = key < end ? key : pos_lo / 4 * 4;
            const int block = block_of(kk);
            const int got = page_at(block);
            const int page = key < end ? got : -1;
            const int keep = end - key;  // keys behind the request's end hold nothing
            const bf16* vrow = vbase + (size_t)(page < 0 ? 0 : page) * v_page + (kk - block * bs);
#pragma unroll
            for (int t = 0; t < MAXTV; ++t) {
                const s16x4 got_v = load4(vrow + (t < dvt ? (size_t)16 * t * bs : 0));
                s16x4 v = (page >= 0 && t < dvt) ? got_v : s16x4{0, 0, 0, 0};
                v.y = keep < 2 ? (short)0 : v.y;
                v.z = keep < 3 ? (short)0 : v.z;
                v.w = keep < 4 ? (short)0 : v.w;
                vf[tt][t] = v;
            }
        }
    };
    auto times_values = [&](const s16x4 vf[TG][MAXTV], const s16x4 pf[TG], f32x4 o[MAXTV]) {
#pragma unroll
        for (int tt = 0; tt < TG; ++tt)
#pragma unroll
            for (int t = 0; t < MAXTV; ++t) o[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf[tt][t], pf[tt], o[t], 0, 0, 0);
    };

    f32x4 acc_o[MAXU][MAPS][MAXTV];
    float run_m[MAXU][MAPS], run_l[MAXU][MAPS];  // (a lane's share of its column's sum)
#pragma unroll
    for (int uu = 0; uu < MAXU; ++uu)
#pragma unroll
        for (int m = 0; m < MAPS; ++m) {
            run_m[uu][m] = NOTHING_YET, run_l[uu][m] = 0.f;
#pragma unroll
            for (int t = 0; t < MAXTV; ++t) acc_o[uu][m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    // a group's scores join a column's running maximum and sum; returns the factor for what was gathered before
    auto join = [&](const float sc[TG][4], float& m_run, float& l_run, float p[TG][4]) {
        float mx = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < TG; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) mx = fmaxf(mx, sc[tt][r]);
        const float m_new = fmaxf(fmaxf(m_run, column_max(mx)), NOTHING_YET);
        const float corr = fast_exp2(m_run - m_new);
        float sum = 0.f;
#pragma unroll
        for (int tt = 0; tt < TG; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                p[tt][r] = fast_exp2(sc[tt][r] - m_new);
                sum += p[tt][r];
            }
        l_run = l_run * corr + sum;
        m_run = m_new;
        return corr;
    };

    float col_l[MAXU][MAPS];  // a column's whole sum, once it is known
    float col_m[MAXU][MAPS];  // and the reference its weights were taken against (for the sink's term)
    if constexpr (!TALK) {
        for (int round = 0; round < n_rounds; ++round) {
            const int group = (round * NS + slice) * NSG + share;
            if (group >= n_groups) break;  // (nothing left for this slice)
            auto walk = [&](auto plain_tag) {
#pragma unroll
                for (int uu = 0; uu < MAXU; ++uu) {
                    if (!mine[uu]) continue;
                    s16x4 vf[TG][MAXTV];
#pragma unroll
                    for (int m = 0; m < MAPS; ++m) {
                        float sc[TG][4], p[TG][4];
                        if (m == 0) load_values(plain_tag, uu, group, vf);  // (asked for beside the keys; both maps use them)
                        scores(plain_tag, uu, m, group, sc);
                        const float corr = join(sc, run_m[uu][m], run_l[uu][m], p);
                        s16x4 pf[TG];
#pragma unroll
                        for (int tt = 0; tt < TG; ++tt) pf[tt] = pack4(p[tt][0], p[tt][1], p[tt][2], p[tt][3]);
                        if (__any(corr != 1.f)) {  // (no column's maximum moved: nothing to scale)
#pragma unroll
                            for (int t = 0; t < MAXTV; ++t) acc_o[uu][m][t] *= corr;
                        }
                        times_values(vf, pf, acc_o[uu][m]);
                    }
                }
            };
            if (plain_group(group)) walk(std::true_type{});
            else walk(std::false_type{});
        }
#pragma unroll
        for (int uu = 0; uu < MAXU; ++uu)
#pragma unroll
            for (int m = 0; m < MAPS; ++m) col_l[uu][m] = column_sum(run_l[uu][m]), col_m[uu][m] = run_m[uu][m];
        if (NS > 1) {  // the slices of a unit meet in LDS: [unit wave][slice][map]{m[16], l[16], o[dv][16]}
            const int per = 16 * (2 + dv);
#pragma unroll
            for (int uu = 0; uu < MAXU; ++uu)
#pragma unroll
                for (int m = 0; m < MAPS; ++m) {
                    float* mine_at = lds + (size_t)(((uw + uu * n_uw) * NS + slice) * MAPS + m) * per;
                    if (!mine[uu]) continue;
                    if (q4 == 0) mine_at[col] = run_m[uu][m], mine_at[16 + col] = col_l[uu][m];
#pragma unroll
                    for (int t = 0; t < MAXTV; ++t)
                        if (t < dvt)
#pragma unroll
                            for (int r = 0; r < 4; ++r) mine_at[32 + (16 * t + 4 * q4 + r) * 16 + col] = acc_o[uu][m][t][r];
                }
            __syncthreads();
            if (slice != 0) return;
#pragma unroll
            for (int uu = 0; uu < MAXU; ++uu)
#pragma unroll
                for (int m = 0; m < MAPS; ++m) {
                    if (!mine[uu]) continue;
                    const float* base = lds + (size_t)(((uw + uu * n_uw) * NS) * MAPS + m) * per;
                    float top = NOTHING_YET;
                    for (int s2 = 0; s2 < NS; ++s2) top = fmaxf(top, base[(size_t)s2 * MAPS * per + col]);
                    float total = 0.f;
#pragma unroll
                    for (int t = 0; t < MAXTV; ++t) acc_o[uu][m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
                    for (int s2 = 0; s2 < NS; ++s2) {
                        const float* at = base + (size_t)s2 * MAPS * per;
                        const float f = fast_exp2(at[col] - top);
                        total += f * at[16 + col];
#pragma unroll
                        for (int t = 0; t < MAXTV; ++t)
                            if (t < dvt)
#pragma unroll
                                for (int r = 0; r < 4; ++r) acc_o[uu][m][t][r] += f * at[32 + (16 * t + 4 * q4 + r) * 16 + col];
                    }
                    col_l[uu][m] = total;
                    col_m[uu][m] = top;
                }
        }
    } else {
        const int group_keys = 16 * TG;
        float* pbuf = lds + (size_t)slice * a.tok * H * group_keys;  // [slice][tok][H][16 TG]
        float* talk_s = lds + (size_t)NS * a.tok * H * group_keys;    // [g][h]
        float* stats = talk_s + H * H;                               // [unit][slice][2][16]
        for (int i = threadIdx.x; i < H * H; i += blockDim.x) talk_s[(i % H) * H + i / H] = a.talk[i];
        // first walk: every column's maximum and sum
        for (int round = 0; round < (a.mode == 2 ? 0 : n_rounds); ++round) {
            const int group = (round * NS + slice) * NSG + share;
            if (group >= n_groups) break;  // (nothing left for this slice)
            auto walk = [&](auto plain_tag) {
#pragma unroll
                for (int uu = 0; uu < MAXU; ++uu) {
                    if (!mine[uu]) continue;
                    float sc[TG][4], p[TG][4];
                    scores(plain_tag, uu, 0, group, sc);
                    join(sc, run_m[uu][0], run_l[uu][0], p);
                }
            };
            walk(std::false_type{});
        }
        float inv_l[MAXU];
#pragma unroll
        for (int uu = 0; uu < MAXU; ++uu) col_l[uu][0] = column_sum(run_l[uu][0]);
        if (NS > 1) {
#pragma unroll
            for (int uu = 0; uu < MAXU; ++uu)
                if (mine[uu] && q4 == 0) {
                    float* at = stats + (size_t)((uw + uu * n_uw) * NS + slice) * 32;
                    at[col] = run_m[uu][0], at[16 + col] = col_l[uu][0];
                }
            __syncthreads();
#pragma unroll
            for (int uu = 0; uu < MAXU; ++uu) {
                if (!mine[uu]) continue;
                const float* at = stats + (size_t)((uw + uu * n_uw) * NS) * 32;
                float top = NOTHING_YET, total = 0.f;
                for (int s2 = 0; s2 < NS; ++s2) top = fmaxf(top, at[s2 * 32 + col]);
                for (int s2 = 0; s2 < NS; ++s2) total += fast_exp2(at[s2 * 32 + col] - top) * at[s2 * 32 + 16 + col];
                run_m[uu][0] = top, col_l[uu][0] = total;
            }
        }
        if (a.mode == 1) {  // this share's maxima and sums go to memory; the second walk is another launch
#pragma unroll
            for (int uu = 0; uu < MAXU; ++uu)
                if (valid[uu] && q4 == 0 && slice == 0) {
                    float* at = a.ws_stats + (((size_t)(row0 + t0 + u_tl[uu]) * H + u_h[uu]) * NSG + share) * 2;
                    at[0] = run_m[uu][0], at[1] = col_l[uu][0];
                }
            return;
        }
        if (a.mode == 2) {
#pragma unroll
            for (int uu = 0; uu < MAXU; ++uu) {
                float top = NOTHING_YET, total = 0.f;
                if (valid[uu]) {
                    const float* at = a.ws_stats + ((size_t)(row0 + t0 + u_tl[uu]) * H + u_h[uu]) * NSG * 2;
                    for (int s2 = 0; s2 < NSG; ++s2) top = fmaxf(top, at[2 * s2]);
                    for (int s2 = 0; s2 < NSG; ++s2) total += fast_exp2(at[2 * s2] - top) * at[2 * s2 + 1];
                }
                run_m[uu][0] = top, col_l[uu][0] = total;
            }
        }
#pragma unroll
        for (int uu = 0; uu < MAXU; ++uu) inv_l[uu] = 1.f / col_l[uu][0];
        __syncthreads();  // (the mixing matrix is in LDS)
        // second walk: normalised weights through LDS, mixed, times the values
        for (int round = 0; round < n_rounds; ++round) {
            const int group = (round * NS + slice) * NSG + share;
            const bool some = group < n_groups;  // (a slice without keys at this turn of the loop only keeps the barriers' count)
            s16x4 vf[MAXU][TG][MAXTV];
            auto walk = [&](auto plain_tag) {
#pragma unroll
                for (int uu = 0; uu < MAXU; ++uu) {
                    if (!mine[uu]) continue;
                    float sc[TG][4];
                    load_values(plain_tag, uu, group, vf[uu]);
                    scores(plain_tag, uu, 0, group, sc);
#pragma unroll
                    for (int tt = 0; tt < TG; ++tt) {
                        f32x4 w;
#pragma unroll
                        for (int r = 0; r < 4; ++r) w[r] = fast_exp2(sc[tt][r] - run_m[uu][0]) * inv_l[uu];
                        if (col < used_cols)
                            *reinterpret_cast<f32x4*>(pbuf + ((size_t)u_tl[uu] * H + u_h[uu]) * group_keys + 16 * tt + 4 * q4) = w;
                    }
                }
            };
            if (some) walk(std::false_type{});
            __syncthreads();
#pragma unroll
            for (int uu = 0; uu < MAXU; ++uu) {
                if (!mine[uu] || !some) continue;
                f32x4 w[TG];
#pragma unroll
                for (int tt = 0; tt < TG; ++tt) w[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (col < used_cols) {
                    const float* prow = pbuf + (size_t)u_tl[uu] * H * group_keys + 4 * q4;
                    const float* trow = talk_s + u_h[uu];
                    for (int g = 0; g < H; ++g) {
                        const float tg = trow[g * H];
#pragma unroll
                        for (int tt = 0; tt < TG; ++tt) w[tt] += tg * *reinterpret_cast<const f32x4*>(prow + g * group_keys + 16 * tt);
                    }
                }
                s16x4 pf[TG];
#pragma unroll
                for (int tt = 0; tt < TG; ++tt) pf[tt] = pack4(w[tt][0], w[tt][1], w[tt][2], w[tt][3]);
                times_values(vf[uu], pf, acc_o[uu][0]);
            }
            __syncthreads();
        }
        if (NS > 1) {  // the slices' partial results, already normalised, add up: [unit][slice][dv][16] over the weights' place
            float* sums = lds;
            const int per = 16 * dv;
#pragma unroll
            for (int uu = 0; uu < MAXU; ++uu) {
                if (!mine[uu]) continue;
                float* at = sums + (size_t)((uw + uu * n_uw) * NS + slice) * per;
#pragma unroll
                for (int t = 0; t < MAXTV; ++t)
                    if (t < dvt)
#pragma unroll
                        for (int r = 0; r < 4; ++r) at[(16 * t + 4 * q4 + r) * 16 + col] = acc_o[uu][0][t][r];
            }
            __syncthreads();
            if (slice != 0) return;
#pragma unroll
            for (int uu = 0; uu < MAXU; ++uu) {
                if (!mine[uu]) continue;
                const float* at = sums + (size_t)((uw + uu * n_uw) * NS) * per;
                for (int s2 = 1; s2 < NS; ++s2)
#pragma unroll
                    for (int t = 0; t < MAXTV; ++t)
                        if (t < dvt)
#pragma unroll
                            for (int r = 0; r < 4; ++r) acc_o[uu][0][t][r] += at[(size_t)s2 * per + (16 * t + 4 * q4 + r) * 16 + col];
            }
        }
    }

    // what leaves: per column, 4 neighbouring dimensions per tile of 16
#pragma unroll
    for (int uu = 0; uu < MAXU; ++uu) {
        if (!mine[uu]) continue;
        float mul[MAPS];
#pragma unroll
        for (int m = 0; m < MAPS; ++m) {
            if constexpr (TALK) {
                mul[m] = 1.f;
            } else {  // (scores are in units of log2: the sink's score 0 stays 0)
                const float l = a.sink ? col_l[uu][m] + fast_exp2(-col_m[uu][m]) : col_l[uu][m];
                mul[m] = 1.f / l;
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int t = 0; t < MAXTV; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float o = acc_o[uu][0][t][r] * mul[0];
                if constexpr (MAPS == 2) o -= a.lambda * (acc_o[uu][1][t][r] * mul[1]);
                acc_o[uu][0][t][r] = o;
                if (t < dvt) ss = fmaf(o, o, ss);
            }
        float norm = 1.f;
        if (a.head_norm) norm = a.out_scale / sqrtf(column_sum(ss) / (float)dv + a.eps);
        if (!valid[uu]) continue;
        if (TALK && a.mode == 2) {  // this share's part, unrounded
            float* part = a.ws_o + ((size_t)share * a.ws_rows + row0 + t0 + u_tl[uu]) * ((size_t)H * dv) + (size_t)u_h[uu] * dv + 4 * q4;
#pragma unroll
            for (int t = 0; t < MAXTV; ++t)
                if (t < dvt) *reinterpret_cast<f32x4*>(part + 16 * t) = acc_o[uu][0][t];
            continue;
        }
        bf16* orow = a.out + (size_t)(row0 + t0 + u_tl[uu]) * a.out_stride + (size_t)u_h[uu] * dv + 4 * q4;
        const float* grow = a.gate ? a.gate + (size_t)(row0 + t0 + u_tl[uu]) * a.gate_stride + (size_t)u_h[uu] * dv + 4 * q4 : nullptr;
#pragma unroll
        for (int t = 0; t < MAXTV; ++t)
            if (t < dvt) {
                f32x4 o = acc_o[uu][0][t] * norm;
                if (grow) {
                    const f32x4 z = *reinterpret_cast<const f32x4*>(grow + 16 * t);
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[r] /= 1.f + expf(-z[r]);
                }
                *reinterpret_cast<s16x4*>(orow + 16 * t) = pack4(o[0], o[1], o[2], o[3]);
            }
    }
}

// out[row] = the sum of the shares' parts (up to 16), rounded once.  The workgroups (request, y, z) take the request's
// rows in turn (y) and 1,024 columns each (z); a thread asks for all shares of its 4 columns before it adds them up.
__global__ __launch_bounds__(256) void add_shares_kernel(bf16* __restrict__ out, int out_stride, const float* __restrict__ ws_o,
                                                         int ws_rows, int shares, int width, const int* __restrict__ cu_seqlens,
                                                         const int* __restrict__ context_lens, int seq_begin) {
    const int b = seq_begin + blockIdx.x;
    if (context_lens[b] <= 0) return;
    const int c = 4 * (blockIdx.z * 256 + threadIdx.x);
    if (c >= width) return;
    for (int row = cu_seqlens[b] + blockIdx.y; row < cu_seqlens[b + 1]; row += gridDim.y) {
        f32x4 part[16];
#pragma unroll
        for (int s2 = 0; s2 < 16; ++s2)  // (a share that does not exist reads the last one and counts for nothing)
            part[s2] = *reinterpret_cast<const f32x4*>(ws_o + ((size_t)(s2 < shares ? s2 : shares - 1) * ws_rows + row) * width + c);
        f32x4 sum = part[0];
#pragma unroll
        for (int s2 = 1; s2 < 16; ++s2) sum += s2 < shares ? part[s2] : f32x4{0.f, 0.f, 0.f, 0.f};
        *reinterpret_cast<s16x4*>(out + (size_t)row * out_stride + c) = pack4(sum[0], sum[1], sum[2], sum[3]);
    }
}

// tiles in a group: 4 (64 keys) up to sizes of 64; wider keys or values leave registers for 2
#define AM_TG 4
#define AM_TG_WIDE 2

template <int MAPS, bool TALK, int MAXU, int THREADS>
static int launch(const MfmaArgs& a, dim3 grid, int threads, size_t lds, hipStream_t stream) {
#define AM_LAUNCH(TK, TV)                                                                                              \
    do {                                                                                                               \
        auto kernel = attend_mfma_kernel<MAPS, TALK, TK, TV, MAXU, (TK > 4 || TV > 4) ? AM_TG_WIDE : AM_TG, THREADS>;  \
        if (lds > 48 * 1024)                                                                                           \
            LLMS_HIP_CHECK(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        kernel<<<grid, threads, lds, stream>>>(a);                                                                     \
    } while (0)
    if (a.dk <= 64 && a.dv <= 64) AM_LAUNCH(4, 4);
    else if (a.dk <= 64) AM_LAUNCH(4, 8);
    else if (a.dv <= 64) AM_LAUNCH(8, 4);
    else AM_LAUNCH(8, 8);
#undef AM_LAUNCH
    LLMS_LAUNCH_CHECK();
}

extern "C" {

// Tokens one workgroup takes when heads are mixed (what a caller needs to count the workgroups of a launch).
int llms_attend_composed_mfma_tokens(int heads, int kv_heads, int dk, int dv, int max_new) {
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || heads / kv_heads > 16 || kv_heads > 32) return 0;
    const int tpw = 16 / (heads / kv_heads);
    const int group_keys = 16 * ((dk > 64 || dv > 64) ? 2 : 4);
    int upk = 32 / kv_heads;
    while (upk > 1 && (size_t)upk * tpw * heads * group_keys * sizeof(float) > 64 * 1024) --upk;
    while (upk > 1 && (upk - 1) * tpw >= max_new) --upk;
    return upk * tpw;
}

// Rows [token rows of requests seq_begin .. seq_begin + n_seqs) of q and out; `max_new`: most tokens one of them brings.
int llms_attend_composed_mfma(void* out, int out_stride, const void* q, int q_stride, const void* k_pool,
                              const void* v_pool, const int* block_tables, const int* table_rows, int max_blocks,
                              const int* cu_seqlens, const int* context_lens, int seq_begin, int n_seqs, int max_new,
                              int heads, int kv_heads, int maps, int dk, int dv, int block_size, int window,
                              int keep_first, int chunk, float scale, const float* slopes, const float* talk, float lambda,
                              int head_norm, float eps, float out_scale, int shares, float* ws_stats, float* ws_o, int ws_rows,
                              const float* dist_bias, int dist_reach, const float* gate, int gate_stride, int sink,
                              hipStream_t stream) {
    LLMS_REQUIRE(n_seqs > 0 && max_new > 0 && heads > 0 && kv_heads > 0, "attend_composed_mfma: sizes must be positive");
    LLMS_REQUIRE(!(sink && talk), "attend_composed_mfma: no sink where heads are mixed");
    LLMS_REQUIRE(heads % kv_heads == 0 && heads / kv_heads <= 16, "attend_composed_mfma: up to 16 query heads per key/value head");
    LLMS_REQUIRE(maps == 1 || maps == 2, "attend_composed_mfma: one or two score maps");
    LLMS_REQUIRE(!(talk && maps != 1), "attend_composed_mfma: mixing heads' weights goes with one score map");
    LLMS_REQUIRE(dk % 16 == 0 && dv % 16 == 0 && dk <= 128 && dv <= 128 && dk > 0 && dv > 0,
                 "attend_composed_mfma: key and value sizes are multiples of 16 up to 128");
    LLMS_REQUIRE(block_size > 0 && block_size % 4 == 0 && max_blocks > 0, "attend_composed_mfma: pages of a multiple of 4 keys");
    LLMS_REQUIRE(q_stride % 4 == 0 && out_stride % 4 == 0, "attend_composed_mfma: rows must be 8-byte aligned");
    LLMS_REQUIRE(window >= 0 && keep_first >= 0 && chunk >= 0, "attend_composed_mfma: window, keep_first and chunk are >= 0");
    MfmaArgs a;
    a.out = (bf16*)out, a.q = (const bf16*)q, a.k_pool = (const bf16*)k_pool, a.v_pool = (const bf16*)v_pool;
    a.block_tables = block_tables, a.table_rows = table_rows, a.cu_seqlens = cu_seqlens, a.context_lens = context_lens;
    a.slopes = slopes, a.talk = talk;
    LLMS_REQUIRE(!dist_bias || dist_reach >= 0, "attend_composed_mfma: a distance table has at least one entry per head");
    LLMS_REQUIRE(!gate || (!talk && gate_stride % 4 == 0), "attend_composed_mfma: gate rows are 16-byte aligned, and no gate where heads are mixed");
    a.dist_bias = dist_bias, a.dist_reach = dist_reach, a.gate = gate, a.gate_stride = gate_stride;
    a.out_stride = out_stride, a.q_stride = q_stride, a.max_blocks = max_blocks, a.seq_begin = seq_begin, a.n_seqs = n_seqs;
    a.heads = heads, a.kv_heads = kv_heads, a.grp = heads / kv_heads, a.dk = dk, a.dv = dv, a.block_size = block_size;
    a.window = window, a.keep_first = keep_first, a.chunk = chunk;
    a.scale = scale, a.lambda = lambda, a.eps = eps, a.out_scale = out_scale, a.head_norm = head_norm, a.sink = sink;
    a.tpw = 16 / a.grp;
    a.shares = 1, a.mode = 0, a.ws_stats = ws_stats, a.ws_o = ws_o, a.ws_rows = ws_rows;
    a.bs_magic = (unsigned)((0x100000000ull + block_size - 1) / block_size);
    const int group_keys = 16 * ((dk > 64 || dv > 64) ? AM_TG_WIDE : AM_TG);
    if (talk) {
        LLMS_REQUIRE(kv_heads <= 32, "attend_composed_mfma: mixing heads takes up to 32 key/value heads");
        // every head of a block of tokens in one workgroup: up to 32 units in up to 16 waves, the normalised
        // weights of a group of keys in up to 64 KB of LDS (more only if a single unit per key/value head needs it)
        int upk = 32 / kv_heads;
        while (upk > 1 && (size_t)upk * a.tpw * heads * group_keys * sizeof(float) > 64 * 1024) --upk;
        while (upk > 1 && (upk - 1) * a.tpw >= max_new) --upk;  // (no more tokens than the longest portion has)
        a.upk = upk, a.tok = upk * a.tpw, a.kv_per_wg = kv_heads, a.units = kv_heads * upk;
        a.slices = 1;
        if (upk == 1 && shares <= 1)  // few tokens (decoding) in one workgroup: the groups of keys are dealt to several waves
            while (a.slices < 4 && a.units * a.slices * 2 <= 16) a.slices *= 2;  // per unit (with shares: to workgroups)
        const int unit_waves = a.units > 16 ? (a.units + 1) / 2 : a.units;
        const int waves = unit_waves * a.slices;
        a.blocks_per_seq = (max_new + a.tok - 1) / a.tok;
        size_t floats = (size_t)a.slices * a.tok * heads * group_keys + (size_t)heads * heads + (size_t)a.units * a.slices * 32;
        const size_t merge = a.slices > 1 ? (size_t)a.units * a.slices * 16 * dv : 0;
        if (merge > floats) floats = merge;
        const size_t lds = (floats + AM_PAGE_CACHE) * sizeof(float);
        LLMS_REQUIRE(lds <= 160 * 1024, "attend_composed_mfma: too many heads for the LDS");
        dim3 grid(n_seqs * a.blocks_per_seq, 1);
        if (shares > 1) {  // the keys of every block of tokens go to `shares` workgroups
            LLMS_REQUIRE(ws_stats && ws_o && ws_rows > 0, "attend_composed_mfma: shares need their workspaces");
            a.shares = shares;
            grid.z = shares;
            for (a.mode = 1; a.mode <= 2; ++a.mode) {
                const int rc = a.units > 16 ? launch<1, true, 2, 1024>(a, grid, waves * LLMS_WAVE, lds, stream)
                                            : launch<1, true, 1, 1024>(a, grid, waves * LLMS_WAVE, lds, stream);
                if (rc != LLMS_OK) return rc;
            }
            LLMS_REQUIRE(shares <= 16, "attend_composed_mfma: up to 16 shares");
            add_shares_kernel<<<dim3(n_seqs, max_new < 64 ? max_new : 64, (heads * dv + 1023) / 1024), 256, 0, stream>>>(
                a.out, out_stride, ws_o, ws_rows, shares, heads * dv, cu_seqlens, context_lens, seq_begin);
            LLMS_LAUNCH_CHECK();
        }
        if (a.units > 16) return launch<1, true, 2, 1024>(a, grid, waves * LLMS_WAVE, lds, stream);
        return launch<1, true, 1, 1024>(a, grid, waves * LLMS_WAVE, lds, stream);
    }
    int upk = 4;
    while (upk > 1 && (upk - 1) * a.tpw >= max_new) --upk;
    a.upk = upk, a.tok = upk * a.tpw, a.kv_per_wg = 1, a.units = upk;
    a.slices = 1;
    if (upk == 1)  // few tokens (decoding): the groups of keys go to 8 waves, or to 4 where 8 would not fit the LDS
        a.slices = ((size_t)8 * maps * 16 * (2 + dv) + AM_PAGE_CACHE) * sizeof(float) <= 96 * 1024 ? 8 : 4;
    a.blocks_per_seq = (max_new + a.tok - 1) / a.tok;
    const size_t lds = ((a.slices > 1 ? (size_t)a.units * a.slices * maps * 16 * (2 + dv) : 0) + AM_PAGE_CACHE) * sizeof(float);
    dim3 grid(n_seqs * a.blocks_per_seq, kv_heads);
    LLMS_REQUIRE(grid.y <= 65535, "attend_composed_mfma: too many key/value heads");
    if (maps == 2) return launch<2, false, 1, 512>(a, grid, upk * a.slices * LLMS_WAVE, lds, stream);
    return launch<1, false, 1, 512>(a, grid, upk * a.slices * LLMS_WAVE, lds, stream);
}

}  // extern "C"
