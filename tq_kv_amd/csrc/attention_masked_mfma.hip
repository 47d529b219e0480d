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
#include <type_traits>

#include "common.h"
#include "tq_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

namespace {

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

// A 16-byte operand that lies beyond a head's size is zero.  The load itself is never under a condition (a branch around every load
// would let none of them be under way together): it reads a place that is there, and the value is dropped.
__device__ __forceinline__ bf16x8_t load_or_zero(const void* base, int offset_bytes, bool wanted) {
    const bf16x8_t v = *reinterpret_cast<const bf16x8_t*>((const unsigned char*)base + (wanted ? offset_bytes : 0));
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
    return wanted ? v : zero;
}

// Eight probabilities of a lane as the second product's operand: bfloat16, two a word, built in registers (element i of the operand is
// word i / 2, low half first).  The sum takes the rounded values.
__device__ __forceinline__ uint32_t two_probabilities(float s0, float s1, float base, float& sum) {
    const uint32_t b0 = float_to_bf16_bits(__builtin_amdgcn_exp2f(s0 - base)), b1 = float_to_bf16_bits(__builtin_amdgcn_exp2f(s1 - base));
    sum += __uint_as_float(b0 << 16) + __uint_as_float(b1 << 16);
    return b0 | (b1 << 16);
}
// the operand of values of a page's keys key0 + (2 pr + i / 4) 16 + 4 g + i % 4, those beyond `last` set to zero
__device__ __forceinline__ bf16x8_t values_up_to(bf16x8_t v, int key0, int pr, int g, int last) {
    u32x4_t w = __builtin_bit_cast(u32x4_t, v);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int j = key0 + (2 * pr + k / 2) * 16 + g * 4 + (k % 2) * 2;
        w[k] &= (j > last ? 0u : 0xffffu) | (j + 1 > last ? 0u : 0xffff0000u);
    }
    return __builtin_bit_cast(bf16x8_t, w);
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
        bf16x8_t bq[KB];
        const bf16_t* qr = a.q + qrow * dk;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) bq[kb] = load_or_zero(qr, (kb * 32 + g * 8) * 2, live && kb * 32 + g * 8 < dk);

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
                    ka[t][kb] = load_or_zero(kp + (size_t)(t * 16 + col) * dk, (kb * 32 + g * 8) * 2, kb * 32 + g * 8 < dk);
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int pr = 0; pr < 2; ++pr)
                    va[db][pr] = load_or_zero(vp, ((db * 16 + col) * TQK_PAGE + pr * 32 + g * 8) * 2, db * 16 + col < dv);

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
            u32x4_t pw[2];
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int h = 0; h < 2; ++h) pw[t / 2][(t % 2) * 2 + h] = two_probabilities(s[t][2 * h], s[t][2 * h + 1], base, psum);
            const bf16x8_t pb[2] = {__builtin_bit_cast(bf16x8_t, pw[0]), __builtin_bit_cast(bf16x8_t, pw[1])};
            l = l * alpha + psum;
            // beyond the last position of the step nothing has been written yet: whatever lies there must not meet a zero
            const bool beyond = key0 + TQK_PAGE - 1 > pos_max;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                o[db][0] *= alpha; o[db][1] *= alpha; o[db][2] *= alpha; o[db][3] *= alpha;
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    const bf16x8_t av = beyond ? values_up_to(va[db][pr], key0, pr, g, pos_max) : va[db][pr];
                    o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, pb[pr], o[db], 0, 0, 0);
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

// Tiles, with a page staged once for a block.  A block of W = 4 or 8 waves takes one kv head and a tile of consecutive queries
// of one sequence: its waves are min(4, heads of the group) query heads times W / that many sub-tiles of 16 CT queries
// (CT = 2; with four waves a group of one head: 128 queries a block; of two: 64; of four or more: 32, the further heads in
// further blocks; with eight waves twice that, for steps that give blocks enough).  A wave holds CT sets of 16 columns, so that what it reads of a page from LDS serves CT products.  Every
// thread brings its pieces of the next page's keys and values into registers while the block computes on the page that
// lies in LDS (two pages under way were measured no faster; rows padded by 16 bytes, so that the 16 rows a load of the matrix cores' operands touches fall on
// different banks); a wave passes over a page none of its queries sees.  Sizes up to 128 and 128.
template <int KB, int DB, int CT, int W>
__global__ __launch_bounds__(W * TQK_WAVE) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attention_masked_block_kernel(const MaskedArgs a) {
    constexpr int KS_MAX = KB * 64 + 16, VS = 2 * TQK_PAGE + 16;        // bytes of a key row and of a value row in LDS
    constexpr int THREADS = W * TQK_WAVE;
    constexpr int KJ = (KB * 256 + THREADS - 1) / THREADS, VJ = (DB * 128 + THREADS - 1) / THREADS;     // pieces of keys and of values a thread brings
    constexpr int SUB = 16 * CT;                                            // queries of a wave
    __shared__ __attribute__((aligned(16))) unsigned char lds_k[TQK_PAGE * KS_MAX];
    __shared__ __attribute__((aligned(16))) unsigned char lds_v[DB * 16 * VS];
    const int tid = threadIdx.x, wave = tid / TQK_WAVE, lane = tid % TQK_WAVE;
    const int col = lane % 16, g = lane / 16;
    const int n_rep = a.n_heads / a.n_kv_heads;
    const int dk = a.dk, dv = a.dv, ks = dk * 2 + 16;
    const int hpb = min(n_rep, 4), sph = W / hpb, chunks = (n_rep + hpb - 1) / hpb;
    const int kvh = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
    const int tile = blockIdx.x;
    const int seq = a.tile_seq[tile], tok0 = a.tile_tok0[tile], count = a.tile_count[tile];
    const int pos0 = __builtin_amdgcn_readfirstlane(a.tok_pos[tok0]);

    // the wave's head and sub-tile; a wave without either still brings pages in
    const int rep = chunk * hpb + wave % hpb, sub = wave / hpb;
    const bool active = rep < n_rep && sub < sph && sub * SUB < count;
    const int head = kvh * n_rep + (rep < n_rep ? rep : 0);
    const int w_first = pos0 + sub * SUB, w_max = min(pos0 + count - 1, w_first + SUB - 1);
    bool live[CT];
    int pos_c[CT], lo_c[CT];
    size_t qrow[CT];
    const int window = a.window;
    const int kept = window > 0 ? a.keep_first : 0;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
        const int i = sub * SUB + c * 16 + col;
        live[c] = active && i < count;
        pos_c[c] = live[c] ? pos0 + i : w_first;
        lo_c[c] = window > 0 ? max(0, pos_c[c] - window + 1) : 0;
        qrow[c] = (size_t)(tok0 + (live[c] ? i : 0)) * a.n_heads + head;
    }
    const int w_lo_min = window > 0 ? max(0, w_first - window + 1) : 0, w_lo_max = window > 0 ? max(0, w_max - window + 1) : 0;
    const int lo_min = window > 0 ? max(0, pos0 - window + 1) : 0;
    const int pos_max = pos0 + count - 1;
    const float scale = a.scale, cap = a.cap;
    const float scale2 = scale * LOG2E;
    const float cap2 = cap * LOG2E, scale_over_cap = cap > 0.f ? scale / cap : 0.f;

    const int first_win_page = lo_min / TQK_PAGE, last_page = pos_max / TQK_PAGE;
    const int kept_pages = min((kept + TQK_PAGE - 1) / TQK_PAGE, first_win_page);
    const int n_visits = kept_pages + last_page - first_win_page + 1;

    // where the thread's pieces of a page (16 bytes each) come from and go to
    int k_src[KJ], k_dst[KJ], v_src[VJ], v_dst[VJ];
    const int k_per_row = dk / 8;
#pragma unroll
    for (int j = 0; j < KJ; ++j) {
        const int p = tid + THREADS * j;
        const int pk = p < 8 * dk ? p : tid % (8 * dk);       // a piece beyond the page: one that is there, once more (the same bytes to the same place)
        k_src[j] = pk;
        k_dst[j] = (pk / k_per_row) * ks + (pk % k_per_row) * 16;
    }
#pragma unroll
    for (int j = 0; j < VJ; ++j) {
        const int p = tid + THREADS * j;
        const int pv = p < 8 * dv ? p : tid % (8 * dv);
        v_src[j] = pv;
        v_dst[j] = (pv / 8) * VS + (pv % 8) * 16;
    }

    float m[CT], l[CT];
    floatx4_t o[CT][DB];
    bf16x8_t bq[CT][KB];
#pragma unroll
    for (int c = 0; c < CT; ++c) {
        m[c] = -INFINITY;
        l[c] = 0.f;
        if (a.sink && active) { m[c] = sink_of(a, head); l[c] = (g == 0) ? 1.f : 0.f; }       // l is summed over a column's four lanes at the end
#pragma unroll
        for (int i = 0; i < DB; ++i) o[c][i] = floatx4_t{0.f, 0.f, 0.f, 0.f};
        const bf16_t* qr = a.q + qrow[c] * dk;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) bq[c][kb] = load_or_zero(qr, (kb * 32 + g * 8) * 2, live[c] && kb * 32 + g * 8 < dk);
    }

    const int32_t* pages = a.page_table + (size_t)seq * a.table_width;
    const size_t k_stride = (size_t)a.n_kv_heads * TQK_PAGE * dk, v_stride = (size_t)a.n_kv_heads * TQK_PAGE * dv;
    auto page_of = [&](int visit) { return visit < kept_pages ? visit : first_win_page + (visit - kept_pages); };
    uint4 k_reg[KJ], v_reg[VJ];
    auto fetch = [&](int visit) {
        const int page = __builtin_amdgcn_readfirstlane(pages[page_of(visit)]);
        if (page < 0) return;                           // nothing of it is visible to anyone: what LDS then holds is not looked at
        const uint4* kp = reinterpret_cast<const uint4*>(a.keys + (size_t)page * k_stride + (size_t)kvh * TQK_PAGE * dk);
        const uint4* vp = reinterpret_cast<const uint4*>(a.values + (size_t)page * v_stride + (size_t)kvh * TQK_PAGE * dv);
#pragma unroll
        for (int j = 0; j < KJ; ++j) k_reg[j] = kp[k_src[j]];
#pragma unroll
        for (int j = 0; j < VJ; ++j) v_reg[j] = vp[v_src[j]];
    };
    fetch(0);
    for (int visit = 0; visit < n_visits; ++visit) {
        const int pg = page_of(visit);
        const int page = __builtin_amdgcn_readfirstlane(pages[pg]);
        __syncthreads();                                // everyone has done with the page before
#pragma unroll
        for (int j = 0; j < KJ; ++j) *reinterpret_cast<uint4*>(lds_k + k_dst[j]) = k_reg[j];
#pragma unroll
        for (int j = 0; j < VJ; ++j) *reinterpret_cast<uint4*>(lds_v + v_dst[j]) = v_reg[j];
        __syncthreads();
        if (visit + 1 < n_visits) fetch(visit + 1);
        const int key0 = pg * TQK_PAGE;
        // does any of the wave's queries see any of the page's keys
        if (!active || page < 0 || key0 > w_max || !(key0 + TQK_PAGE > w_lo_min || key0 < kept)) continue;
        const bool inside = key0 + TQK_PAGE - 1 <= w_first && (key0 >= w_lo_max || key0 + TQK_PAGE <= kept);

        // scores^T for the page's four groups of 16 keys, a group's keys read once for all of the wave's columns
        floatx4_t s[CT][4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            bf16x8_t ka[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
                ka[kb] = load_or_zero(lds_k, (t * 16 + col) * ks + (kb * 32 + g * 8) * 2, kb * 32 + g * 8 < dk);
#pragma unroll
            for (int c = 0; c < CT; ++c) {
                s[c][t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s[c][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[kb], bq[c][kb], s[c][t], 0, 0, 0);
            }
        }
        bf16x8_t pb[CT][2];
        float alpha[CT];
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            float mx = m[c];
            // three shapes of the same loop, chosen by what holds for the whole wave: most pages of a prompt lie inside what every
            // column sees and carry no cap, and then a score costs a multiplication and a maximum
            if (cap > 0.f) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int j = key0 + t * 16 + g * 4 + r;
                        float v = cap2 * tanh_fast(s[c][t][r] * scale_over_cap);
                        if (!inside && !(j <= pos_c[c] && (j >= lo_c[c] || j < kept))) v = -INFINITY;
                        s[c][t][r] = v;
                        mx = fmaxf(mx, v);
                    }
            } else if (inside) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        s[c][t][r] *= scale2;
                        mx = fmaxf(mx, s[c][t][r]);
                    }
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int j = key0 + t * 16 + g * 4 + r;
                        const float v = (j <= pos_c[c] && (j >= lo_c[c] || j < kept)) ? s[c][t][r] * scale2 : -INFINITY;
                        s[c][t][r] = v;
                        mx = fmaxf(mx, v);
                    }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, TQK_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, TQK_WAVE));
            const float base = mx == -INFINITY ? 0.f : mx;      // a column that has met no key it sees yet
            alpha[c] = __builtin_amdgcn_exp2f(m[c] - base);
            m[c] = mx;
            float psum = 0.f;
            u32x4_t pw[2];
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int h = 0; h < 2; ++h) pw[t / 2][(t % 2) * 2 + h] = two_probabilities(s[c][t][2 * h], s[c][t][2 * h + 1], base, psum);
            pb[c][0] = __builtin_bit_cast(bf16x8_t, pw[0]);
            pb[c][1] = __builtin_bit_cast(bf16x8_t, pw[1]);
            l[c] = l[c] * alpha[c] + psum;
        }
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            bf16x8_t av[2];
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) {
                av[pr] = load_or_zero(lds_v, (db * 16 + col) * VS + (pr * 32 + g * 8) * 2, db * 16 + col < dv);
                // beyond the last position of the step nothing has been written yet: whatever lies there must not meet a zero
                if (key0 + TQK_PAGE - 1 > pos_max) av[pr] = values_up_to(av[pr], key0, pr, g, pos_max);
            }
#pragma unroll
            for (int c = 0; c < CT; ++c) {
                o[c][db][0] *= alpha[c]; o[c][db][1] *= alpha[c]; o[c][db][2] *= alpha[c]; o[c][db][3] *= alpha[c];
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) o[c][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[pr], pb[c][pr], o[c][db], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < CT; ++c) {
        float lc = l[c];
        lc += __shfl_xor(lc, 16, TQK_WAVE);
        lc += __shfl_xor(lc, 32, TQK_WAVE);
        if (!live[c]) continue;
        bf16_t* po = a.out + qrow[c] * dv;
        const float inv = 1.f / lc;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = db * 16 + g * 4 + r;
                if (e < dv) po[e] = from_float<bf16_t>(o[c][db][r] * inv);
            }
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
int launch_masked(const MaskedArgs& a, bool tiles, int n_tiles, int tile_queries, int n_rows, hipStream_t s) {
    if (tiles) {
        if constexpr (KB <= 4 && DB <= 8) {
            const int n_rep = a.n_heads / a.n_kv_heads, hpb = n_rep < 4 ? n_rep : 4;
            dim3 grid(n_tiles, a.n_kv_heads * ((n_rep + hpb - 1) / hpb));
            // eight waves a block where the tiles are that large: a page brought in then serves twice the queries
            if (tile_queries >= 32 * (8 / hpb)) attention_masked_block_kernel<KB, DB, 2, 8><<<grid, 8 * TQK_WAVE, 0, s>>>(a);
            else attention_masked_block_kernel<KB, DB, 2, 4><<<grid, 4 * TQK_WAVE, 0, s>>>(a);
        } else {
            dim3 grid(n_tiles, (a.n_heads + 3) / 4);
            attention_masked_mfma_kernel<KB, DB, 4, true><<<grid, 4 * TQK_WAVE, 0, s>>>(a);
        }
    } else {
        dim3 grid(a.n_parts, a.n_kv_heads * a.q_blocks, n_rows);
        // a partition per page of the table: a block has one page to read, and one wave does it
        if (a.n_parts > 1 && a.n_parts >= a.table_width) attention_masked_mfma_kernel<KB, DB, 1, false><<<grid, TQK_WAVE, 0, s>>>(a);
        else attention_masked_mfma_kernel<KB, DB, 4, false><<<grid, 4 * TQK_WAVE, 0, s>>>(a);
    }
    return tqk_check_launch("tqk_attention_masked_mfma");
}

template <int KB>
int launch_masked_dv(const MaskedArgs& a, bool tiles, int n_tiles, int tile_queries, int n_rows, hipStream_t s) {
    if (a.dv <= 32) return launch_masked<KB, 2>(a, tiles, n_tiles, tile_queries, n_rows, s);
    if (a.dv <= 64) return launch_masked<KB, 4>(a, tiles, n_tiles, tile_queries, n_rows, s);
    if (a.dv <= 128) return launch_masked<KB, 8>(a, tiles, n_tiles, tile_queries, n_rows, s);
    return launch_masked<KB, 16>(a, tiles, n_tiles, tile_queries, n_rows, s);
}

}  // namespace

extern "C" int tqk_attention_masked_mfma_supported(int key_dim, int value_dim) {
    return key_dim > 0 && key_dim % 8 == 0 && key_dim <= 256 && value_dim > 0 && value_dim <= 256;
}
/* queries per tile for steps of several tokens a sequence: 32 for each sub-tile a block's waves make of a tile */
extern "C" int tqk_attention_masked_mfma_tile(int n_tokens, int n_heads, int n_kv_heads, int key_dim, int value_dim) {
    if (key_dim > 128 || value_dim > 128 || n_kv_heads <= 0) return 16;
    const int n_rep = n_heads / n_kv_heads, hpb = n_rep < 4 ? (n_rep > 0 ? n_rep : 1) : 4;
    // blocks of four waves, or of eight (twice the queries for every page brought in) where that still leaves four blocks a compute unit
    const long long blocks8 = (long long)((n_tokens + 32 * (8 / hpb) - 1) / (32 * (8 / hpb))) * n_kv_heads * ((n_rep + hpb - 1) / hpb);
    return 32 * ((blocks8 >= 1024 ? 8 : 4) / hpb);
}

/* n_tiles > 0: tiles of up to 16 consecutive queries of one sequence (tile_seq, tile_tok0, tile_count on the device; tok_pos and q by
 * packed token, page_table by sequence of the step).  Else rows: row r is a token of its own at position tok_pos[r] whose pages are
 * page_table row r, in n_parts partitions (part_out float32 [rows, heads, n_parts, value_dim], part_ml [rows, heads, n_parts, 2]
 * where n_parts > 1). */
extern "C" int tqk_attention_masked_mfma(const void* q, const void* keys, const void* values, const int32_t* tok_pos, const int32_t* page_table,
                                         int table_width, int n_pages, int window, int keep_first, float scale, float cap, const void* sink,
                                         int sink_dtype, const int32_t* tile_seq, const int32_t* tile_tok0, const int32_t* tile_count, int n_tiles,
                                         int tile_queries, int n_rows, int n_parts, void* part_out, void* part_ml, void* out, int n_heads, int n_kv_heads,
                                         int key_dim, int value_dim, void* stream) {
    TQK_REQUIRE(q && keys && values && tok_pos && page_table && out, "tqk_attention_masked_mfma: null pointer");
    TQK_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0, "tqk_attention_masked_mfma: %d heads and %d kv heads", n_heads, n_kv_heads);
    TQK_REQUIRE(tqk_attention_masked_mfma_supported(key_dim, value_dim), "tqk_attention_masked_mfma: head sizes %d and %d are not taken", key_dim, value_dim);
    TQK_REQUIRE(table_width > 0 && n_pages > 0, "tqk_attention_masked_mfma: empty page table");
    TQK_REQUIRE(window >= 0 && keep_first >= 0 && cap >= 0.f, "tqk_attention_masked_mfma: negative window, kept positions or cap");
    TQK_REQUIRE(!sink || sink_dtype == TQK_F32 || sink_dtype == TQK_BF16, "tqk_attention_masked_mfma: unknown dtype %d of the sink", sink_dtype);
    const bool tiles = n_tiles > 0;
    if (tiles) TQK_REQUIRE(tile_seq && tile_tok0 && tile_count && tile_queries >= 16, "tqk_attention_masked_mfma: tiles without their lists or their size");
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
    TQK_REQUIRE((long long)n_kv_heads * a.q_blocks <= 65535 && n_heads <= 65535, "tqk_attention_masked_mfma: grid too large");
    a.dk = key_dim; a.dv = value_dim;
    a.tile_seq = tile_seq; a.tile_tok0 = tile_tok0; a.tile_count = tile_count;
    a.part_out = (float*)part_out; a.part_ml = (float*)part_ml; a.out = (bf16_t*)out;
    hipStream_t s = (hipStream_t)stream;
    int status;
    if (key_dim <= 64) status = launch_masked_dv<2>(a, tiles, n_tiles, tile_queries, n_rows, s);
    else if (key_dim <= 128) status = launch_masked_dv<4>(a, tiles, n_tiles, tile_queries, n_rows, s);
    else status = launch_masked_dv<8>(a, tiles, n_tiles, tile_queries, n_rows, s);
    if (status || tiles || n_parts == 1) return status;
    attention_masked_merge_kernel<<<n_rows * n_heads, value_dim >= 128 ? 128 : 64, 0, s>>>((const float*)part_out, (const float*)part_ml, n_parts, value_dim,
                                                                                            n_heads, sink, a.sink_f32, (bf16_t*)out);
    return tqk_check_launch("tqk_attention_masked_mfma merge");
}
