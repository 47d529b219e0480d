// Many small products at once on the matrix cores: y_g = x_g W_g^T for groups g that each have a
// weight of their own [N, K] (K contiguous) and some rows of x.  Two callers:
//
//   routed experts   a group is an expert; its rows are the step's (token, choice) pairs that the router gave
//                    it, cut into tiles listed on the device (moe.hip: tqk_moe_group); rows of x are gathered
//                    by token; gate and up weights lie one behind the other and the gate is applied in place
//   heads            a group is a head; every token has a row in every group, x and y are [tokens, heads, ...]
//                    (the two products around the attention over latents: the query into the latent's space
//                    and the attended latent into the head's values, times the head's output gate)
//
// v_mfma_f32_16x16x32_bf16, D[16x16] += A[16x32] B[32x16]: A = 16 rows of x, B = 16 rows of the weight, both
// read straight from memory, 16 contiguous bytes per lane (float32 x: 32 bytes, rounded to bfloat16); the lane
// then holds, for feature l%16, rows 4*(l/16)+i.  A wave keeps RT x CB such blocks (RT * 16 rows, CB * 16
// features) so that a loaded operand serves several products; the four waves of a block take neighbouring
// features and share their rows of x through the cache.  There is no shared memory and no barrier: tiles of one
// row (decoding) stream the weights, large tiles reuse them from the caches.
// A row's sums depend on its own values alone, never on its place in a tile.
#include "common.h"
#include "tq_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 grp_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float grp_floatx4_t;
union grp_pack8 {
    grp_bf16x8_t v;
    uint16_t u[8];
    uint4 q;
};

#define GRP_WAVES 4

struct GroupedArgs {
    const void* x;                  // rows of K values, bfloat16 or float32
    int x_f32;
    long long x_row_stride, x_group_stride;
    const int32_t* x_rows;          // row r of a tile reads x row x_rows[row0 + r] (null: row0 + r)
    const bf16_t* w;                // group g: w + g * w_group_stride, [N, K] (gated: [2 N, K], gate rows first)
    long long w_group_stride;
    void* y;                        // bfloat16 or float32
    int y_f32;
    long long y_row_stride, y_group_stride;
    const float* row_scale;         // y[row, group] is multiplied by row_scale[row * scale_row_stride + group] (or null)
    long long scale_row_stride;
    int N, K;
    int gate;
    float gate_limit, gate_alpha;
    int activated;                  // not gated: the gate's function of the product itself is applied (see act_value)
    // tiles from lists on the device (tile_group != null), or every group over all rows in tiles of tile_rows_max
    const int32_t *tile_group, *tile_row0, *tile_rows, *n_tiles;
    int n_groups, n_rows, tile_rows_max;
};

template <int RT, int CB, bool GATED>
__global__ __launch_bounds__(GRP_WAVES * TQK_WAVE)
void grouped_mfma_kernel(GroupedArgs p) {
    // tiles of more than 16 rows: the block brings a step's rows of x into LDS once (one 16-byte piece a thread), in the
    // order the lanes take them, two buffers in turn with one barrier a step; its waves read them from there
    constexpr bool STAGE = RT > 1;
    // tiles of up to 16 rows: the block's four waves take the same features and a quarter of K each (a wave alone would
    // walk all of K with one load under way after the other), and add their sums up through LDS in the waves' order
    constexpr bool SPLIT = RT == 1;
    constexpr int NBK = GATED ? 2 : 1;
    __shared__ uint4 x_lds[STAGE ? 2 : 1][4][STAGE ? 16 * RT : 1];
    __shared__ grp_floatx4_t sum_lds[SPLIT ? GRP_WAVES : 1][NBK][CB][SPLIT ? TQK_WAVE : 1];
    int group, row0, n_rows;
    if (p.tile_group) {
        const int tile = blockIdx.y;
        if (tile >= *p.n_tiles) return;
        group = p.tile_group[tile];
        row0 = p.tile_row0[tile];
        n_rows = p.tile_rows[tile];
    } else {
        group = blockIdx.y % p.n_groups;
        row0 = (blockIdx.y / p.n_groups) * p.tile_rows_max;
        n_rows = min(p.tile_rows_max, p.n_rows - row0);
    }
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int g = lane / 16, r16 = lane % 16;
    const int n0 = (SPLIT ? blockIdx.x : blockIdx.x * GRP_WAVES + wave) * CB * 16;
    const bool active = n0 < p.N;
    if (!STAGE && !SPLIT && !active) return;
    constexpr int NB = GATED ? 2 : 1;
    grp_floatx4_t acc[NB][RT][CB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) acc[b][rt][cb] = grp_floatx4_t{0.f, 0.f, 0.f, 0.f};
    // where the rows of x begin: the lane's own (no staging), or the one row whose pieces the thread stages
    auto row_offset = [&](int r) -> long long {
        return r < n_rows ? (long long)(p.x_rows ? p.x_rows[row0 + r] : row0 + r) * p.x_row_stride + (long long)group * p.x_group_stride : -1;
    };
    // (no branch on what is outside: such a lane reads a piece that exists and drops it, so that loads can be under way
    // over several steps)
    auto load_x = [&](long long off, int e0) -> uint4 {
        grp_pack8 a;
        const bool out = off < 0 || e0 + 8 > p.K;
        if (off < 0) off = (long long)group * p.x_group_stride + (p.x_rows ? (long long)p.x_rows[row0] * p.x_row_stride : (long long)row0 * p.x_row_stride);
        e0 = min(e0, p.K - 8);
        if (p.x_f32) {
            const float4* src = reinterpret_cast<const float4*>((const float*)p.x + off + e0);
            const float4 lo = src[0], hi = src[1];
            a.u[0] = float_to_bf16_bits(lo.x); a.u[1] = float_to_bf16_bits(lo.y);
            a.u[2] = float_to_bf16_bits(lo.z); a.u[3] = float_to_bf16_bits(lo.w);
            a.u[4] = float_to_bf16_bits(hi.x); a.u[5] = float_to_bf16_bits(hi.y);
            a.u[6] = float_to_bf16_bits(hi.z); a.u[7] = float_to_bf16_bits(hi.w);
        } else {
            a.q = *reinterpret_cast<const uint4*>((const bf16_t*)p.x + off + e0);
        }
        if (out) a.q = make_uint4(0, 0, 0, 0);
        return a.q;
    };
    long long xoff[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) xoff[rt] = STAGE ? -1 : row_offset(16 * rt + r16);
    const int stage_row = threadIdx.x / 4, stage_g = threadIdx.x % 4;
    const bool stages = STAGE && stage_row < 16 * RT;
    const long long stage_off = stages ? row_offset(stage_row) : -1;
    const bf16_t* wg = p.w + (size_t)group * p.w_group_stride;
    long long woff[CB];
    bool w_ok[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        w_ok[cb] = active && n0 + 16 * cb + r16 < p.N;
        woff[cb] = (long long)(w_ok[cb] ? n0 + 16 * cb + r16 : 0) * p.K;
    }
    const long long up = (long long)p.N * p.K;

    // what the next step needs is asked for before this step's products: the weights' pieces and, where the rows of x are
    // staged, the thread's piece of them
    auto load_w = [&](int k0, grp_pack8 (&b)[NB][CB]) {
        const int e0 = min(k0 + 8 * g, p.K - 8);
        const bool in = k0 + 8 * g + 8 <= p.K;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            const bool w_in = in && w_ok[cb];
            // tiles of up to 16 rows read a weight once: such loads say so
            const grp_bf16x8_t* w0 = reinterpret_cast<const grp_bf16x8_t*>(wg + woff[cb] + e0);
            const grp_bf16x8_t* w1 = reinterpret_cast<const grp_bf16x8_t*>(wg + up + woff[cb] + e0);
            b[0][cb].v = RT == 1 ? __builtin_nontemporal_load(w0) : *w0;
            if (!w_in) b[0][cb].q = make_uint4(0, 0, 0, 0);
            if (GATED) {
                b[NB - 1][cb].v = RT == 1 ? __builtin_nontemporal_load(w1) : *w1;
                if (!w_in) b[NB - 1][cb].q = make_uint4(0, 0, 0, 0);
            }
        }
    };
    grp_pack8 b_next[NB][CB];
    uint4 x_next = make_uint4(0, 0, 0, 0);
    load_w(min(SPLIT ? wave * (((p.K + 32 * GRP_WAVES - 1) / (32 * GRP_WAVES)) * 32) : 0, ((p.K - 1) / 32) * 32), b_next);
    if (STAGE) x_next = load_x(stage_off, 8 * stage_g);
    const int k_quarter = SPLIT ? ((p.K + 32 * GRP_WAVES - 1) / (32 * GRP_WAVES)) * 32 : p.K;
    const int k_begin = SPLIT ? wave * k_quarter : 0, k_end = SPLIT ? min(p.K, k_begin + k_quarter) : p.K;
    const int k_last = k_end > k_begin ? ((k_end - 1 - k_begin) / 32) * 32 + k_begin : k_begin;
    for (int k0 = k_begin, step = 0; k0 < k_end; k0 += 32, ++step) {
        grp_pack8 a[RT], b[NB][CB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) b[nb][cb] = b_next[nb][cb];
        if (STAGE) {
            if (stages) x_lds[step & 1][stage_g][stage_row] = x_next;
            __syncthreads();
        }
        // (after the last step this asks for the last step's again and drops it: no branch between the loads)
        load_w(min(k0 + 32, k_last), b_next);
        if (STAGE) x_next = load_x(stage_off, min(k0 + 32, k_last) + 8 * stage_g);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) a[rt].q = STAGE ? x_lds[step & 1][g][STAGE ? 16 * rt + r16 : 0] : load_x(xoff[rt], k0 + 8 * g);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
                    acc[nb][rt][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt].v, b[nb][cb].v, acc[nb][rt][cb], 0, 0, 0);
    }
    if (SPLIT) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) sum_lds[SPLIT ? wave : 0][nb][cb][SPLIT ? lane : 0] = acc[nb][0][cb];
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
                for (int w = 1; w < (SPLIT ? GRP_WAVES : 1); ++w) acc[nb][0][cb] += sum_lds[w][nb][cb][SPLIT ? lane : 0];
    }
    if (!active) return;
    // the lane holds, of each block, feature n0 + 16 cb + r16 of rows 16 rt + 4 g + i
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 16 * rt + 4 * g + i;
            if (r >= n_rows) continue;
            const long long row = row0 + r;
            const float scale = p.row_scale ? p.row_scale[row * p.scale_row_stride + group] : 1.f;
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const int n = n0 + 16 * cb + r16;
                if (n >= p.N) continue;
                float v = acc[0][rt][cb][i];
                if (GATED) {
                    // gate and up rounded as stored products would be, then the gate in float32
                    const float gv = to_float(from_float<bf16_t>(v)), uv = to_float(from_float<bf16_t>(acc[NB - 1][rt][cb][i]));
                    v = gate_value(p.gate, p.gate_limit, p.gate_alpha, gv, uv);
                } else if (p.activated) {
                    v = act_value(p.gate, p.gate_limit, p.gate_alpha, to_float(from_float<bf16_t>(v)));
                }
                v *= scale;
                const long long at = row * p.y_row_stride + (long long)group * p.y_group_stride + n;
                if (p.y_f32) ((float*)p.y)[at] = v;
                else ((bf16_t*)p.y)[at] = from_float<bf16_t>(v);
            }
        }
}

template <bool GATED>
static int launch_grouped(const GroupedArgs& a, int tiles, hipStream_t s) {
    // rows of a tile: up to 16, 32 or 64; features of a wave: 16 or 32 (32 where there are enough of them to fill the chip)
    // tiles of more than 16 rows share their rows of x through LDS and keep 32 (gated) or 64 features a wave, so that what is
    // loaded serves many products; tiles of up to 16 rows stream the weights, 16 features a wave, 32 where there are many
    const int rt = a.tile_rows_max > 32 ? 4 : a.tile_rows_max > 16 ? 2 : 1;
    const int cb = rt > 1 ? (GATED ? 2 : (a.N >= 256 ? 4 : 2)) : (((long long)a.N / 16) * tiles >= 4096 && !GATED ? 2 : 1);
    const int per_block = (rt == 1 ? 1 : GRP_WAVES) * cb * 16;       // tiles of up to 16 rows: the waves of a block share its features
    dim3 grid((a.N + per_block - 1) / per_block, tiles);
#define TQK_GRP(RT, CB) grouped_mfma_kernel<RT, CB, GATED><<<grid, GRP_WAVES * TQK_WAVE, 0, s>>>(a)
    if (rt == 4) { if (cb == 4) TQK_GRP(4, 4); else TQK_GRP(4, 2); }
    else if (rt == 2) { if (cb == 4) TQK_GRP(2, 4); else TQK_GRP(2, 2); }
    else { if (cb == 2) TQK_GRP(1, 2); else TQK_GRP(1, 1); }
#undef TQK_GRP
    return tqk_check_launch("tqk grouped product");
}

extern "C" int tqk_grouped_supported(int K) { return K % 8 == 0; }

/* The experts' products over tiles of up to tile_m rows (16, 32 or 64: what tqk_moe_group was given). */
extern "C" int tqk_moe_product_mfma(const void* x, const int32_t* x_rows, const void* w, long long expert_stride, void* y, int N, int K,
                                    int gated, int gate, float limit, float alpha, const int32_t* tile_expert, const int32_t* tile_row0,
                                    const int32_t* tile_rows, const int32_t* n_tiles, int max_tiles, int tile_m, void* stream) {
    TQK_REQUIRE(x && w && y && tile_expert && tile_row0 && tile_rows && n_tiles, "tqk_moe_product_mfma: null pointer");
    TQK_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && max_tiles >= 0 && max_tiles <= 65535, "tqk_moe_product_mfma: bad sizes (N %d, K %d, %d tiles)", N, K, max_tiles);
    TQK_REQUIRE(tile_m == 16 || tile_m == 32 || tile_m == 64, "tqk_moe_product_mfma: tiles of %d rows", tile_m);
    TQK_REQUIRE(gated >= 0 && gated <= 2, "tqk_moe_product_mfma: gated must be 0, 1 or 2, got %d", gated);
    TQK_REQUIRE(!gated || (gate >= 0 && gate < TQK_GATE_KINDS), "tqk_moe_product_mfma: unknown gate %d", gate);
    TQK_REQUIRE(expert_stride >= (long long)(gated == 1 ? 2 : 1) * N * K && expert_stride % 8 == 0, "tqk_moe_product_mfma: experts overlap or are not aligned");
    TQK_REQUIRE(((((uintptr_t)x) | ((uintptr_t)w)) & 15) == 0, "tqk_moe_product_mfma: x and w must be 16-byte aligned");
    if (max_tiles == 0) return 0;
    GroupedArgs a = {};
    a.x = x; a.x_row_stride = K; a.x_rows = x_rows;
    a.w = (const bf16_t*)w; a.w_group_stride = expert_stride;
    a.y = y; a.y_row_stride = N;
    a.N = N; a.K = K; a.gate = gate; a.gate_limit = limit; a.gate_alpha = alpha; a.activated = gated == 2;
    a.tile_group = tile_expert; a.tile_row0 = tile_row0; a.tile_rows = tile_rows; a.n_tiles = n_tiles; a.tile_rows_max = tile_m;
    return gated == 1 ? launch_grouped<true>(a, max_tiles, (hipStream_t)stream) : launch_grouped<false>(a, max_tiles, (hipStream_t)stream);
}

/* y[t, h, :N] = scale[t, h] * W_h x[t, h, :K] for every token t and head h.  x: [tokens, heads, x_head_stride...] rows of
 * x_row_stride values, bfloat16 or float32 (x_f32); w: [heads][N][K] bfloat16; y likewise with its own strides;
 * scale [tokens, heads] float32 or null. */
extern "C" int tqk_head_product(const void* x, int x_f32, long long x_row_stride, long long x_head_stride, const void* w, void* y, int y_f32,
                                long long y_row_stride, long long y_head_stride, const float* scale, int n_tokens, int n_heads, int N, int K,
                                void* stream) {
    TQK_REQUIRE(x && w && y, "tqk_head_product: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_heads > 0 && N > 0 && K > 0 && K % 8 == 0, "tqk_head_product: bad sizes (N %d, K %d)", N, K);
    TQK_REQUIRE(x_row_stride % 8 == 0 && x_head_stride % 8 == 0 && ((((uintptr_t)x) | ((uintptr_t)w)) & 15) == 0,
                "tqk_head_product: rows of x and w must begin at multiples of 16 bytes");
    if (n_tokens == 0) return 0;
    GroupedArgs a = {};
    a.x = x; a.x_f32 = x_f32; a.x_row_stride = x_row_stride; a.x_group_stride = x_head_stride;
    a.w = (const bf16_t*)w; a.w_group_stride = (long long)N * K;
    a.y = y; a.y_f32 = y_f32; a.y_row_stride = y_row_stride; a.y_group_stride = y_head_stride;
    a.row_scale = scale; a.scale_row_stride = n_heads;
    a.N = N; a.K = K;
    a.n_groups = n_heads; a.n_rows = n_tokens;
    a.tile_rows_max = n_tokens > 32 ? 64 : n_tokens > 16 ? 32 : 16;
    const long long tiles = (long long)n_heads * ((n_tokens + a.tile_rows_max - 1) / a.tile_rows_max);
    TQK_REQUIRE(tiles <= 65535, "tqk_head_product: %lld tiles are more than the grid takes", tiles);
    return launch_grouped<false>(a, (int)tiles, (hipStream_t)stream);
}
