// The attention of attention_masked.hip on the matrix cores (bfloat16 in, float32 softmax): keys of key_dim and
// values of value_dim per head, a cap on the scores, a window that keeps a sequence's first positions, a sink in
// the softmax's denominator.  One body serves two kinds of step.
//
// A wave computes 16 columns against a page of 64 keys at a time (v_mfma_f32_16x16x32_bf16, the mapping of
// attention_decode.hip: scores^T[key][column] = K . Q^T, out^T[element][column] = V^T . P^T with P staying in the
// lanes' registers, the cache's value pages being laid out for exactly that).  What a column is differs:
//   rows   (one token a sequence, or a few chosen rows): the columns are the query heads that share a kv head, for
//          one token; a row's pages are dealt out to n_parts blocks of W waves, merged through LDS and, with more
//          than one partition, by a second kernel (which also adds the sink);
//   tiles  (several tokens a sequence): the columns are up to 16 consecutive queries of one sequence, for one head;
//          a block's W waves take W heads next to each other, which share a kv head where the group is that large,
//          so a page is read from memory once and from the caches by the others.  Every column has its own
//          position, window and first visible key.
// Pages between the kept first positions and the window are passed over.  Sizes need not be those of a build:
// key_dim <= 32 KB (a multiple of 8), value_dim <= 16 DB; what lies beyond a head's sizes is not loaded.
#include "common.h"
#include "tq_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

namespace {

union pack8 {
    bf16x8_t v;
    uint16_t u[8];
    uint4 q;
};

struct MaskedArgs {
    const bf16_t *q, *keys, *values;
    const int32_t *tok_pos, *page_table;
    int table_width, window, keep_first;
    float scale, cap;
    const void* sink;               // [heads] or null
    int sink_f32;
    int n_parts, n_heads, n_kv_heads, q_blocks, dk, dv;
    const int32_t *tile_seq, *tile_tok0, *tile_count;      // tiles
    float *part_out, *part_ml;      // rows with more than one partition
    bf16_t* out;
};

#define LOG2E 1.4426950408889634f

__device__ __forceinline__ float sink_of(const MaskedArgs& a, int head) {
    return (a.sink_f32 ? ((const float*)a.sink)[head] : to_float(((const bf16_t*)a.sink)[head])) * LOG2E;
}

// tanh by one exponential: 1 - 2 / (e^(2x) + 1); exact at both ends (e^(2x) = inf gives 1, 0 gives -1)
__device__ __forceinline__ float tanh_fast(float x) {
    const float t = __builtin_amdgcn_exp2f(x * (2.f * LOG2E));
    return 1.f - 2.f / (t + 1.f);
}

template <int KB, int DB, int W, bool TILE>
__global__ __launch_bounds__(W * TQK_WAVE)
void attention_masked_mfma_kernel(const MaskedArgs a) {
    constexpr int ROW = DB * 4 + 2;         // floats a lane hands over: its out^T values, m, l
    __shared__ __attribute__((aligned(16))) float xch[(W > 1 && !TILE) ? (W - 1) * TQK_WAVE * ROW : 1];
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int col = lane % 16, g = lane / 16;
    const int n_rep = a.n_heads / a.n_kv_heads;
    const int dk = a.dk, dv = a.dv;

    // the lane's column: which query row, at which position, for which head
    int seq, head, kvh, pos_c, pos_first, pos_max, part = 0;
    bool live;
    size_t qrow;
    if (TILE) {
        head = blockIdx.y * W + wave;
        if (head >= a.n_heads) return;
        const int tile = blockIdx.x;
        seq = a.tile_seq[tile];
        const int tok0 = a.tile_tok0[tile], count = a.tile_count[tile];
        live = col < count;
        const int tok = tok0 + (live ? col : 0);
        pos_first = __builtin_amdgcn_readfirstlane(a.tok_pos[tok0]);
        pos_max = pos_first + count - 1;
        pos_c = pos_first + (live ? col : 0);
        kvh = head / n_rep;
        qrow = (size_t)tok * a.n_heads + head;
    } else {
        part = blockIdx.x;
        kvh = blockIdx.y / a.q_blocks;
        const int rep = (blockIdx.y % a.q_blocks) * 16 + col;
        seq = blockIdx.z;
        live = rep < n_rep;
        head = kvh * n_rep + (live ? rep : 0);
        pos_c = pos_first = pos_max = __builtin_amdgcn_readfirstlane(a.tok_pos[seq]);
        qrow = (size_t)seq * a.n_heads + head;
    }
    const int window = a.window;
    const int kept = window > 0 ? a.keep_first : 0;
    const int lo_c = window > 0 ? max(0, pos_c - window + 1) : 0;
    const int lo_min = window > 0 ? max(0, pos_first - window + 1) : 0;      // the first column's: the smallest
    const int lo_max = window > 0 ? max(0, pos_max - window + 1) : 0;
    const float scale = a.scale, cap = a.cap;
    const float scale2 = scale * LOG2E;
    const float cap2 = cap * LOG2E, scale_over_cap = cap > 0.f ? scale / cap : 0.f;

    // the pages this block visits: those of the kept first positions that lie before the window's, then the window's
    const int first_win_page = lo_min / TQK_PAGE, last_page = pos_max / TQK_PAGE;
    const int kept_pages = min((kept + TQK_PAGE - 1) / TQK_PAGE, first_win_page);
    const int n_visits = kept_pages + last_page - first_win_page + 1;
    const int visit0 = TILE ? 0 : part + wave * a.n_parts, visit_step = TILE ? 1 : W * a.n_parts;

    // tiles: the sink is a key of score sink_h without a value, and the running maximum and sum start from it; rows add it
    // when the partitions are merged
    float m = -INFINITY, l = 0.f;
    if (TILE && a.sink) { m = sink_of(a, head); l = (g == 0) ? 1.f : 0.f; }     // l is summed over the four lanes of a column at the end
    floatx4_t o[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i) o[i] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    if (visit0 < n_visits) {
        pack8 zero;
        zero.q = make_uint4(0, 0, 0, 0);
        bf16x8_t bq[KB];
        const bf16_t* qr = a.q + qrow * dk + g * 8;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) bq[kb] = (live && kb * 32 + g * 8 < dk) ? *reinterpret_cast<const bf16x8_t*>(qr + kb * 32) : zero.v;

        const int32_t* pages = a.page_table + (size_t)seq * a.table_width;
        const size_t k_stride = (size_t)a.n_kv_heads * TQK_PAGE * dk, v_stride = (size_t)a.n_kv_heads * TQK_PAGE * dv;
        for (int visit = visit0; visit < n_visits; visit += visit_step) {
            const int pg = visit < kept_pages ? visit : first_win_page + (visit - kept_pages);
            const int page = __builtin_amdgcn_readfirstlane(pages[pg]);
            if (page < 0) continue;                     // the host never lets this happen for a page that holds a visible key
            const bf16_t* kp = a.keys + (size_t)page * k_stride + (size_t)kvh * TQK_PAGE * dk;
            const bf16_t* vp = a.values + (size_t)page * v_stride + (size_t)kvh * TQK_PAGE * dv;
            const int key0 = pg * TQK_PAGE;
            // a page all of whose keys every column sees needs no mask
            const bool inside = key0 + TQK_PAGE - 1 <= pos_first && (key0 >= lo_max || key0 + TQK_PAGE <= kept);

            bf16x8_t ka[4][KB], va[DB][2];
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
                    ka[t][kb] = kb * 32 + g * 8 < dk ? *reinterpret_cast<const bf16x8_t*>(kp + (size_t)(t * 16 + col) * dk + kb * 32 + g * 8) : zero.v;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int pr = 0; pr < 2; ++pr)
                    va[db][pr] = db * 16 + col < dv ? *reinterpret_cast<const bf16x8_t*>(vp + (size_t)(db * 16 + col) * TQK_PAGE + pr * 32 + g * 8) : zero.v;

            floatx4_t s[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                s[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[t][kb], bq[kb], s[t], 0, 0, 0);
            }
            // scale, cap, mask, running maximum (the lane's keys are key0 + 16 t + 4 g + r)
            float mx = m;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int j = key0 + t * 16 + g * 4 + r;
                    float v = cap > 0.f ? cap2 * tanh_fast(s[t][r] * scale_over_cap) : s[t][r] * scale2;
                    if (!inside && !(j <= pos_c && (j >= lo_c || j < kept))) v = -INFINITY;
                    s[t][r] = v;
                    mx = fmaxf(mx, v);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, TQK_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, TQK_WAVE));
            // a column may not have met a key it sees yet: its maximum is still -inf, and nothing of it counts
            const float base = mx == -INFINITY ? 0.f : mx;
            const float alpha = __builtin_amdgcn_exp2f(m - base);
            m = mx;
            float psum = 0.f;
            pack8 pb[2];
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = __builtin_amdgcn_exp2f(s[t][r] - base);
                    const uint16_t pbits = float_to_bf16_bits(p);
                    psum += __uint_as_float(((uint32_t)pbits) << 16);
                    pb[t / 2].u[(t % 2) * 4 + r] = pbits;
                }
            l = l * alpha + psum;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                o[db][0] *= alpha; o[db][1] *= alpha; o[db][2] *= alpha; o[db][3] *= alpha;
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    pack8 av;
                    av.v = va[db][pr];
                    if (key0 + TQK_PAGE - 1 > pos_max) {
                        // beyond the last position of the step nothing has been written yet: whatever lies there must not meet a zero
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            const int j = key0 + (2 * pr + i / 4) * 16 + g * 4 + (i % 4);
                            if (j > pos_max) av.u[i] = 0;
                        }
                    }
                    o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av.v, pb[pr].v, o[db], 0, 0, 0);
                }
            }
        }
    }
    l += __shfl_xor(l, 16, TQK_WAVE);
    l += __shfl_xor(l, 32, TQK_WAVE);

    if (TILE) {
        if (!live) return;
        bf16_t* po = a.out + qrow * dv;
        const float inv = 1.f / l;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = db * 16 + g * 4 + r;
                if (e < dv) po[e] = from_float<bf16_t>(o[db][r] * inv);
            }
        return;
    }

    // rows: the waves' results into wave 0, in wave order
    if (W > 1) {
        if (wave > 0) {
            float* mine = xch + ((size_t)(wave - 1) * TQK_WAVE + lane) * ROW;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) mine[db * 4 + r] = o[db][r];
            mine[DB * 4] = m;
            mine[DB * 4 + 1] = l;
        }
        __syncthreads();
    }
    if (wave != 0) return;
    for (int w = 1; w < W; ++w) {
        const float* theirs = xch + ((size_t)(w - 1) * TQK_WAVE + lane) * ROW;
        const float m2 = theirs[DB * 4], l2 = theirs[DB * 4 + 1];
        if (m2 == -INFINITY) continue;
        const float mn = fmaxf(m, m2);
        const float a1 = __builtin_amdgcn_exp2f(m - mn), a2 = __builtin_amdgcn_exp2f(m2 - mn);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[db][r] = o[db][r] * a1 + theirs[db * 4 + r] * a2;
        l = l * a1 + l2 * a2;
        m = mn;
    }
    if (!live) return;
    const size_t row = ((size_t)seq * a.n_heads + head) * a.n_parts + part;
    if (a.n_parts == 1) {
        if (a.sink) {
            const float sk = sink_of(a, head), mn = fmaxf(m, sk);
            const float a1 = __builtin_amdgcn_exp2f(m - mn);
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[db][r] *= a1;
            l = l * a1 + __builtin_amdgcn_exp2f(sk - mn);
        }
        bf16_t* po = a.out + qrow * dv;
        const float inv = 1.f / l;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = db * 16 + g * 4 + r;
                if (e < dv) po[e] = from_float<bf16_t>(o[db][r] * inv);
            }
    } else {
        float* po = a.part_out + row * dv;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = db * 16 + g * 4 + r;
                if (e < dv) po[e] = o[db][r];
            }
        if (g == 0) { a.part_ml[row * 2] = m; a.part_ml[row * 2 + 1] = l; }
    }
}

// out[row, :] = sum_p 2^(m_p - M) o_p / (sum_p 2^(m_p - M) l_p + 2^(sink - M)), partitions in order
__global__ void attention_masked_merge_kernel(const float* __restrict__ part_out, const float* __restrict__ part_ml, int n_parts, int dv, int n_heads,
                                              const void* __restrict__ sink, int sink_f32, bf16_t* __restrict__ out) {
    const size_t row = blockIdx.x;                     // row * n_heads + head
    const float2* ml = reinterpret_cast<const float2*>(part_ml) + row * n_parts;
    float M = -INFINITY, sk = -INFINITY;
    if (sink) {
        const int head = (int)(row % n_heads);
        sk = (sink_f32 ? ((const float*)sink)[head] : to_float(((const bf16_t*)sink)[head])) * LOG2E;
        M = sk;
    }
#pragma unroll 8
    for (int p = 0; p < n_parts; ++p) M = fmaxf(M, ml[p].x);
    for (int c = threadIdx.x; c < dv; c += blockDim.x) {
        float acc = 0.f, denom = sink ? __builtin_amdgcn_exp2f(sk - M) : 0.f;
        const float* po = part_out + row * n_parts * dv + c;
#pragma unroll 8
        for (int p = 0; p < n_parts; ++p) {
            const float2 s = ml[p];
            const float v = po[(size_t)p * dv];
            const bool has = s.x != -INFINITY;
            const float wgt = has ? __builtin_amdgcn_exp2f(s.x - M) : 0.f;
            denom += wgt * s.y;
            acc += has ? wgt * v : 0.f;
        }
        out[row * dv + c] = from_float<bf16_t>(acc / denom);
    }
}

template <int KB, int DB>
int launch_masked(const MaskedArgs& a, bool tiles, int n_tiles, int n_rows, hipStream_t s) {
    if (tiles) {
        dim3 grid(n_tiles, (a.n_heads + 3) / 4);
        attention_masked_mfma_kernel<KB, DB, 4, true><<<grid, 4 * TQK_WAVE, 0, s>>>(a);
    } else {
        dim3 grid(a.n_parts, a.n_kv_heads * a.q_blocks, n_rows);
        // a partition per page of the table: a block has one page to read, and one wave does it
        if (a.n_parts > 1 && a.n_parts >= a.table_width) attention_masked_mfma_kernel<KB, DB, 1, false><<<grid, TQK_WAVE, 0, s>>>(a);
        else attention_masked_mfma_kernel<KB, DB, 4, false><<<grid, 4 * TQK_WAVE, 0, s>>>(a);
    }
    return tqk_check_launch("tqk_attention_masked_mfma");
}

template <int KB>
int launch_masked_dv(const MaskedArgs& a, bool tiles, int n_tiles, int n_rows, hipStream_t s) {
    if (a.dv <= 32) return launch_masked<KB, 2>(a, tiles, n_tiles, n_rows, s);
    if (a.dv <= 64) return launch_masked<KB, 4>(a, tiles, n_tiles, n_rows, s);
    if (a.dv <= 128) return launch_masked<KB, 8>(a, tiles, n_tiles, n_rows, s);
    return launch_masked<KB, 16>(a, tiles, n_tiles, n_rows, s);
}

}  // namespace

extern "C" int tqk_attention_masked_mfma_supported(int key_dim, int value_dim) {
    return key_dim > 0 && key_dim % 8 == 0 && key_dim <= 256 && value_dim > 0 && value_dim <= 256;
}
extern "C" int tqk_attention_masked_mfma_tile(void) { return 16; }

/* n_tiles > 0: tiles of up to 16 consecutive queries of one sequence (tile_seq, tile_tok0, tile_count on the device; tok_pos and q by
 * packed token, page_table by sequence of the step).  Else rows: row r is a token of its own at position tok_pos[r] whose pages are
 * page_table row r, in n_parts partitions (part_out float32 [rows, heads, n_parts, value_dim], part_ml [rows, heads, n_parts, 2]
 * where n_parts > 1). */
extern "C" int tqk_attention_masked_mfma(const void* q, const void* keys, const void* values, const int32_t* tok_pos, const int32_t* page_table,
                                         int table_width, int n_pages, int window, int keep_first, float scale, float cap, const void* sink,
                                         int sink_dtype, const int32_t* tile_seq, const int32_t* tile_tok0, const int32_t* tile_count, int n_tiles,
                                         int n_rows, int n_parts, void* part_out, void* part_ml, void* out, int n_heads, int n_kv_heads,
                                         int key_dim, int value_dim, void* stream) {
    TQK_REQUIRE(q && keys && values && tok_pos && page_table && out, "tqk_attention_masked_mfma: null pointer");
    TQK_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0, "tqk_attention_masked_mfma: %d heads and %d kv heads", n_heads, n_kv_heads);
    TQK_REQUIRE(tqk_attention_masked_mfma_supported(key_dim, value_dim), "tqk_attention_masked_mfma: head sizes %d and %d are not taken", key_dim, value_dim);
    TQK_REQUIRE(table_width > 0 && n_pages > 0, "tqk_attention_masked_mfma: empty page table");
    TQK_REQUIRE(window >= 0 && keep_first >= 0 && cap >= 0.f, "tqk_attention_masked_mfma: negative window, kept positions or cap");
    TQK_REQUIRE(!sink || sink_dtype == TQK_F32 || sink_dtype == TQK_BF16, "tqk_attention_masked_mfma: unknown dtype %d of the sink", sink_dtype);
    const bool tiles = n_tiles > 0;
    if (tiles) TQK_REQUIRE(tile_seq && tile_tok0 && tile_count && n_tiles <= 0x7fffffff, "tqk_attention_masked_mfma: tiles without their lists");
    else {
        TQK_REQUIRE(n_rows >= 0 && n_rows <= 65535, "tqk_attention_masked_mfma: %d rows", n_rows);
        TQK_REQUIRE(n_parts > 0 && n_parts <= 65535 && (n_parts == 1 || (part_out && part_ml)), "tqk_attention_masked_mfma: %d partitions, or no room for them", n_parts);
        if (n_rows == 0) return 0;
    }
    MaskedArgs a = {};
    a.q = (const bf16_t*)q; a.keys = (const bf16_t*)keys; a.values = (const bf16_t*)values;
    a.tok_pos = tok_pos; a.page_table = page_table; a.table_width = table_width;
    a.window = window; a.keep_first = keep_first; a.scale = scale; a.cap = cap;
    a.sink = sink; a.sink_f32 = sink_dtype == TQK_F32;
    a.n_parts = tiles ? 1 : n_parts; a.n_heads = n_heads; a.n_kv_heads = n_kv_heads;
    a.q_blocks = (n_heads / n_kv_heads + 15) / 16;
    TQK_REQUIRE((long long)n_kv_heads * a.q_blocks <= 65535 && (n_heads + 3) / 4 <= 65535, "tqk_attention_masked_mfma: grid too large");
    a.dk = key_dim; a.dv = value_dim;
    a.tile_seq = tile_seq; a.tile_tok0 = tile_tok0; a.tile_count = tile_count;
    a.part_out = (float*)part_out; a.part_ml = (float*)part_ml; a.out = (bf16_t*)out;
    hipStream_t s = (hipStream_t)stream;
    int status;
    if (key_dim <= 64) status = launch_masked_dv<2>(a, tiles, n_tiles, n_rows, s);
    else if (key_dim <= 128) status = launch_masked_dv<4>(a, tiles, n_tiles, n_rows, s);
    else status = launch_masked_dv<8>(a, tiles, n_tiles, n_rows, s);
    if (status || tiles || n_parts == 1) return status;
    attention_masked_merge_kernel<<<n_rows * n_heads, value_dim >= 128 ? 128 : 64, 0, s>>>((const float*)part_out, (const float*)part_ml, n_parts, value_dim,
                                                                                            n_heads, sink, a.sink_f32, (bf16_t*)out);
    return tqk_check_launch("tqk_attention_masked_mfma merge");
}
