// Attention through a low-rank latent: the kernels around the cache of latents.
//
// Every position leaves one row in the cache, shared by all heads: the normed latent c [rk] and
// one rotated key part r [dr].  A head's key would be (W_uk,h c, r) and its value W_uv,h c; neither
// is ever formed.  Since q_h . (W_uk,h c) = (W_uk,h^T q_h) . c, the query is taken into the latent's
// space once per token ("absorbed"), attention runs with the cache row as the key and its first rk
// elements as the value, the same for every head, and W_uv,h is applied to the attended latent:
//
//   split      one row of the stacked first products [q latent | kv latent, rotated part | gate logits]:
//              RMS norm of the q latent -> cq; RMS norm of the kv latent and rotation of the rotated part
//              -> the cache row of the token's position; sigmoid of the gate logits -> gate [T, H]
//   absorb     q [T, H, dn + dr] -> qa [T, H, rk + dr]: qa[:rk] = W_uk,h^T q[:dn], qa[rk:] = rotated q[dn:]
//   attention  softmax((qa . row) * scale) over the window, times row[:rk] -> o [T, H, rk]
//   values     y[t, h, :] = gate[t, h] * W_uv,h o[t, h, :]
//
// Norms, angles, scores, softmax weights, gates and all sums are float32; qa and o stay float32
// between the kernels.  The order of a query's operations depends on its position alone.
// Cache pages: [position in page][rk + dr].
#include <algorithm>

#include "common.h"
#include "tq_kernels.h"

#define LAT_MAX_RK 512          // largest latent the attention kernel's accumulators hold
#define LAT_MAX_DK 640          // largest cache row (latent + rotated part)
#define LAT_TT 8                // tokens a block of the absorb and values kernels takes

// ---- split -----------------------------------------------------------------------------------
template <typename TA, typename TW>
__global__ __launch_bounds__(256)
void latent_split_kernel(const TA* __restrict__ proj, int row_stride, int q_rank, int kv_rank, int rot_dim, int n_gate,
                         const TW* __restrict__ q_norm_w, const TW* __restrict__ kv_norm_w, float eps,
                         const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot_dims, int max_positions,
                         const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                         const int32_t* __restrict__ page_table, int table_width, TA* __restrict__ cache, TA* __restrict__ turned,
                         int n_pages, TA* __restrict__ cq_out, float* __restrict__ gate_out) {
    __shared__ float scratch[8];
    const int t = blockIdx.x;
    const int kv_cols = kv_rank > 0 ? kv_rank + rot_dim : 0;
    const TA* row = proj + (size_t)t * row_stride;
    // the query's latent
    float ss = 0.f;
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) { const float v = to_float(row[i]); ss = fmaf(v, v, ss); }
    ss = block_sum(ss, scratch);
    const float inv_q = 1.f / sqrtf(ss / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
        cq_out[(size_t)t * q_rank + i] = from_float<TA>(to_float(row[i]) * inv_q * to_float(q_norm_w[i]));
    // the gates
    for (int i = threadIdx.x; i < n_gate; i += blockDim.x)
        gate_out[(size_t)t * n_gate + i] = 1.f / (1.f + expf(-to_float(row[q_rank + kv_cols + i])));
    if (kv_rank <= 0) return;
    // the cache row
    const TA* kv = row + q_rank;
    ss = 0.f;
    for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) { const float v = to_float(kv[i]); ss = fmaf(v, v, ss); }
    ss = block_sum(ss, scratch);
    const float inv_kv = 1.f / sqrtf(ss / (float)kv_rank + eps);
    const int pos = tok_pos[t];
    const int page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
    if (page < 0 || page >= n_pages) return;
    TA* dst = cache + ((size_t)page * TQK_PAGE + (size_t)(pos % TQK_PAGE)) * kv_cols;
    // the latent a second time, turned: [element][place of the position], for the matrix cores' second product
    TA* dst_t = turned ? turned + (size_t)page * kv_rank * TQK_PAGE + value_place(pos % TQK_PAGE) : nullptr;
    for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
        const TA v = from_float<TA>(to_float(kv[i]) * inv_kv * to_float(kv_norm_w[i]));
        dst[i] = v;
        if (dst_t) dst_t[(size_t)i * TQK_PAGE] = v;
    }
    const int half = rot_dims / 2;
    const int p = min(pos, max_positions - 1);
    for (int i = threadIdx.x; i < rot_dim; i += blockDim.x) {
        const float v = to_float(kv[kv_rank + i]);
        float r = v;
        if (i < rot_dims) {
            const int j = i < half ? i : i - half;
            const float c = cos_table[(size_t)p * half + j], s = sin_table[(size_t)p * half + j];
            const float other = to_float(kv[kv_rank + (i < half ? i + half : i - half)]);
            r = i < half ? v * c - other * s : v * c + other * s;
        }
        dst[kv_rank + i] = from_float<TA>(r);
    }
}

// ---- absorb ----------------------------------------------------------------------------------
// A block: LAT_TT tokens of one head.  Thread j takes latent columns j, j + 128, ...; the head's rows
// of W_uk are read along their columns, so a wave's loads are contiguous.
template <typename TA, typename TW>
__global__ __launch_bounds__(128)
void latent_absorb_kernel(const TA* __restrict__ q, const TW* __restrict__ w_uk, int n_heads, int dn, int dr, int rk,
                          const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot_dims, int max_positions,
                          const int32_t* __restrict__ tok_pos, float* __restrict__ qa, int n_tokens, int tail_only) {
    extern __shared__ float q_lds[];            // [LAT_TT][dn + dr]
    const int head = blockIdx.y, t0 = blockIdx.x * LAT_TT, d = dn + dr;
    const int n_t = min(LAT_TT, n_tokens - t0);
    for (int i = threadIdx.x; i < LAT_TT * d; i += blockDim.x) {
        const int tt = i / d, c = i % d;
        q_lds[i] = tt < n_t ? to_float(q[((size_t)(t0 + tt) * n_heads + head) * d + c]) : 0.f;
    }
    __syncthreads();
    const TW* w = w_uk + (size_t)head * dn * rk;
    for (int j = threadIdx.x; j < (tail_only ? 0 : rk); j += blockDim.x) {
        float acc[LAT_TT];
#pragma unroll
        for (int tt = 0; tt < LAT_TT; ++tt) acc[tt] = 0.f;
        for (int c = 0; c < dn; ++c) {
            const float wv = to_float(w[(size_t)c * rk + j]);
#pragma unroll
            for (int tt = 0; tt < LAT_TT; ++tt) acc[tt] = fmaf(q_lds[tt * d + c], wv, acc[tt]);
        }
#pragma unroll
        for (int tt = 0; tt < LAT_TT; ++tt)
            if (tt < n_t) qa[((size_t)(t0 + tt) * n_heads + head) * (rk + dr) + j] = acc[tt];
    }
    const int half = rot_dims / 2;
    for (int i = threadIdx.x; i < n_t * dr; i += blockDim.x) {
        const int tt = i / dr, c = i % dr;
        const float* qr = q_lds + tt * d + dn;
        float r = qr[c];
        if (c < rot_dims) {
            const int p = min(tok_pos[t0 + tt], max_positions - 1);
            const int j = c < half ? c : c - half;
            const float cs = cos_table[(size_t)p * half + j], sn = sin_table[(size_t)p * half + j];
            r = c < half ? qr[c] * cs - qr[c + half] * sn : qr[c] * cs + qr[c - half] * sn;
        }
        qa[((size_t)(t0 + tt) * n_heads + head) * (rk + dr) + rk + c] = r;
    }
}

// ---- attention -------------------------------------------------------------------------------
// One wave per (token, head).  Keys are taken a page at a time: lane j computes the score of the
// page's position j, the softmax runs online over pages, then lane c accumulates element c
// (+64, +128, ...) of the attended latent over the page's positions.
#define LAT_WAVES 4
template <typename TA>
__global__ __launch_bounds__(LAT_WAVES * TQK_WAVE)
void latent_attention_kernel(const float* __restrict__ qa, const TA* __restrict__ cache, const int32_t* __restrict__ tok_seq,
                             const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table, int table_width,
                             int window, float scale, float* __restrict__ out, int n_tokens, int n_heads, int rk, int dk) {
    __shared__ float q_lds[LAT_WAVES][LAT_MAX_DK];
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int t = blockIdx.x * LAT_WAVES + wave;
    const int head = blockIdx.y;
    const bool live = t < n_tokens;
    if (live) {
        const float* qv = qa + ((size_t)t * n_heads + head) * dk;
        for (int i = lane; i < dk; i += TQK_WAVE) q_lds[wave][i] = qv[i];
    }
    __syncthreads();
    if (!live) return;
    const int pos = tok_pos[t];
    const int32_t* pages = page_table + (size_t)tok_seq[t] * table_width;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const float* qf = q_lds[wave];
    constexpr int NACC = LAT_MAX_RK / TQK_WAVE;
    float acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.f;
    float m = -INFINITY, l = 0.f;
    for (int kb = (lo / TQK_PAGE) * TQK_PAGE; kb <= pos; kb += TQK_PAGE) {
        const int page = pages[kb / TQK_PAGE];
        const int j = kb + lane;
        const bool valid = j >= lo && j <= pos && page >= 0;
        const TA* base = cache + (size_t)(page < 0 ? 0 : page) * TQK_PAGE * dk;
        float s = -INFINITY;
        if (valid) {
            const TA* kr = base + (size_t)lane * dk;
            float dot = 0.f;
            for (int i = 0; i < dk; ++i) dot = fmaf(qf[i], to_float(kr[i]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float alpha = expf(m - m_new);
        l = l * alpha + wave_sum(p);
        m = m_new;
        const int n_keys = min(TQK_PAGE, pos - kb + 1);
        const int first_key = max(0, lo - kb);
#pragma unroll
        for (int a = 0; a < NACC; ++a) {
            const int c = lane + a * TQK_WAVE;
            float sum = acc[a] * alpha;
            if (a * TQK_WAVE < rk) {
                for (int jj = first_key; jj < n_keys; ++jj) {
                    const float pj = __shfl(p, jj, TQK_WAVE);
                    if (c < rk) sum = fmaf(pj, to_float(base[(size_t)jj * dk + c]), sum);
                }
            }
            acc[a] = sum;
        }
    }
    float* o = out + ((size_t)t * n_heads + head) * rk;
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
        const int c = lane + a * TQK_WAVE;
        if (c < rk) o[c] = acc[a] / l;
    }
}

// ---- attention on the matrix cores (bfloat16 cache) -------------------------------------------
// One wave per (token, 16 heads).  v_mfma_f32_16x16x32_bf16, D[16x16] += A[16x32] B[32x16]:
//   scores^T[key][head] = row[key][:] . qa^T[:][head]
//       A = 16 cache rows x 32 of their elements, 16 contiguous bytes per lane straight from the page; B = the heads'
//       absorbed queries, held in registers for the whole walk.  The lane then holds, for head l%16, keys 4*(l/16)+i.
//   out^T[element][head] = turned[element][key] . P^T[key][head]
//       B: the eight keys a lane holds of two groups of 16 are the product's eight k slots, so P never leaves its
//       registers; A: the turned copy of the latents keeps a page's positions in exactly that order (value_place),
//       16 contiguous bytes per lane.
// KS: 32-element steps of a cache row the kernel is built for; NCT: 16-element blocks of the latent.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 lat_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float lat_floatx4_t;
union lat_pack8 {
    lat_bf16x8_t v;
    uint16_t u[8];
    uint4 q;
};

// WAVES: waves of a block (each with a token's 16 heads of its own; the queries wait in LDS, 1 KB per step and wave).
// n_parts > 1: a token's pages are dealt out to that many waves, which leave their sums, maxima and weights for
// latent_merge_kernel (decoding steps, where the tokens alone are too few waves).
template <int KS, int NCT, int WAVES>
__global__ __launch_bounds__(WAVES * TQK_WAVE)
void latent_attention_mfma_kernel(const float* __restrict__ qa, const bf16_t* __restrict__ cache, const bf16_t* __restrict__ turned,
                                  const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                  const int32_t* __restrict__ page_table, int table_width, int window, float scale,
                                  float* __restrict__ out, int n_tokens, int n_heads, int n_chunks, int rk, int dk, int n_parts,
                                  float* __restrict__ part_o, float* __restrict__ part_ml) {
    __shared__ uint4 q_lds[WAVES][KS][TQK_WAVE];
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int item = blockIdx.x * WAVES + wave;
    if (item >= n_tokens * n_chunks * n_parts) return;
    const int part = item % n_parts;
    const int t = (item / n_parts) / n_chunks, head = ((item / n_parts) % n_chunks) * 16 + lane % 16;
    const int g = lane / 16, r16 = lane % 16;
    const int pos = tok_pos[t];
    const int32_t* pages = page_table + (size_t)tok_seq[t] * table_width;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int ks_used = (dk + 31) / 32, ct_used = (rk + 15) / 16;
    (void)ct_used;

#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int e0 = 32 * ks + 8 * g;
        lat_pack8 bq;
        bq.q = make_uint4(0, 0, 0, 0);
        if (ks < ks_used && head < n_heads && e0 + 8 <= dk) {
            const float4* src = reinterpret_cast<const float4*>(qa + ((size_t)t * n_heads + head) * dk + e0);
            const float4 a = src[0], b = src[1];
            bq.u[0] = float_to_bf16_bits(a.x); bq.u[1] = float_to_bf16_bits(a.y);
            bq.u[2] = float_to_bf16_bits(a.z); bq.u[3] = float_to_bf16_bits(a.w);
            bq.u[4] = float_to_bf16_bits(b.x); bq.u[5] = float_to_bf16_bits(b.y);
            bq.u[6] = float_to_bf16_bits(b.z); bq.u[7] = float_to_bf16_bits(b.w);
        }
        q_lds[wave][ks][lane] = bq.q;           // read back by the lane that wrote it: no barrier
    }
    lat_floatx4_t o[NCT];
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) o[ct] = lat_floatx4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    for (int kb = (lo / TQK_PAGE + part) * TQK_PAGE; kb <= pos; kb += TQK_PAGE * n_parts) {
        const int page = max(0, pages[kb / TQK_PAGE]);
        const bf16_t* kp = cache + (size_t)page * TQK_PAGE * dk;
        const bf16_t* vp = turned + (size_t)page * rk * TQK_PAGE;
        lat_floatx4_t s[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) s[j] = lat_floatx4_t{0.f, 0.f, 0.f, 0.f};
        // (no branch inside: a lane whose piece lies beyond the row reads the row's last piece instead and drops it, so
        // that the loads of many steps can be under way at once)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int e0 = 32 * ks + 8 * g;
            const bool in = e0 + 8 <= dk;
            const int e0c = in ? e0 : dk - 8;
            lat_pack8 bq;
            bq.q = q_lds[wave][ks][lane];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                lat_pack8 a;
                a.q = *reinterpret_cast<const uint4*>(kp + (size_t)(16 * j + r16) * dk + e0c);
                if (!in) a.q = make_uint4(0, 0, 0, 0);
                s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, bq.v, s[j], 0, 0, 0);
            }
        }
        // the lane's 16 scores belong to its head and keys kb + 16 j + 4 g + i
        float p[4][4];
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + 16 * j + 4 * g + i;
                const bool valid = key >= lo && key <= pos;
                p[j][i] = valid ? s[j][i] * scale : -INFINITY;
                mx = fmaxf(mx, p[j][i]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, TQK_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, TQK_WAVE));
        const float m_new = fmaxf(m, mx);               // finite: the page holds at least one visible key
        const float alpha = expf(m - m_new);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                p[j][i] = expf(p[j][i] - m_new);        // exp(-inf) = 0 for keys that are not seen
                sum += p[j][i];
            }
        sum += __shfl_xor(sum, 16, TQK_WAVE);
        sum += __shfl_xor(sum, 32, TQK_WAVE);
        l = l * alpha + sum;
        m = m_new;
        lat_pack8 pb[2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 8; ++e) pb[h].u[e] = float_to_bf16_bits(p[2 * h + e / 4][e % 4]);
        // what lies at places of keys that are not seen may be anything: it is replaced by zero
        const bool edge = kb < lo || kb + TQK_PAGE - 1 > pos;
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
            const int col = 16 * ct + r16;
            const int colc = min(col, rk - 1);
            o[ct] *= alpha;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                lat_pack8 a;
                a.q = *reinterpret_cast<const uint4*>(vp + (size_t)colc * TQK_PAGE + 32 * h + 8 * g);
                if (col >= rk) a.q = make_uint4(0, 0, 0, 0);
                if (edge) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int key = kb + value_position(32 * h + 8 * g + e);
                        if (key < lo || key > pos) a.u[e] = 0;
                    }
                }
                o[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pb[h].v, o[ct], 0, 0, 0);
            }
        }
    }
    if (head >= n_heads) return;
    float* dst = n_parts > 1 ? part_o + (((size_t)t * n_heads + head) * n_parts + part) * rk : out + ((size_t)t * n_heads + head) * rk;
    const float inv = n_parts > 1 ? 1.f : 1.f / l;
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
        if (ct < ct_used) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int col = 16 * ct + 4 * g + i;
                if (col < rk) dst[col] = o[ct][i] * inv;
            }
        }
    }
    if (n_parts > 1 && g == 0) {
        float* ml = part_ml + (((size_t)t * n_heads + head) * n_parts + part) * 2;
        ml[0] = m;                  // -inf and 0 where the part had no page
        ml[1] = l;
    }
}

// ---- attention on the matrix cores, a block per (token, 16 heads, part) (decoding) -------------------
// The same products as latent_attention_mfma_kernel, shared out over the four waves of a block so that no wave has a
// long chain of loads to wait for: wave j takes the scores of the page's keys 16 j .. 16 j + 15 (a quarter of the rows),
// the waves exchange their maxima, sums and probabilities through LDS, and wave w takes a quarter of the latent's
// elements in the second product.  The absorbed queries wait in LDS for all four.
template <int KS, int NCT>
__global__ __launch_bounds__(4 * TQK_WAVE)
void latent_attention_page_kernel(const float* __restrict__ qa, const bf16_t* __restrict__ cache, const bf16_t* __restrict__ turned,
                                  const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                  const int32_t* __restrict__ page_table, int table_width, int window, float scale,
                                  float* __restrict__ out, int n_heads, int n_chunks, int rk, int dk, int n_parts,
                                  float* __restrict__ part_o, float* __restrict__ part_ml) {
    constexpr int CT = NCT / 4;                         // 16-element blocks of the latent a wave takes
    __shared__ uint4 q_lds[KS][TQK_WAVE];
    __shared__ float mx_lds[4][16], sum_lds[4][16];
    __shared__ uint2 p_lds[4][TQK_WAVE];
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int g = lane / 16, r16 = lane % 16;
    const int item = blockIdx.x;
    const int part = item % n_parts;
    const int t = (item / n_parts) / n_chunks, chunk = (item / n_parts) % n_chunks;
    const int head = chunk * 16 + r16;
    const int pos = tok_pos[t];
    const int32_t* pages = page_table + (size_t)tok_seq[t] * table_width;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    for (int i = threadIdx.x; i < KS * TQK_WAVE; i += 4 * TQK_WAVE) {
        const int ks = i / TQK_WAVE, ln = i % TQK_WAVE;
        const int h = chunk * 16 + ln % 16, e0 = 32 * ks + 8 * (ln / 16);
        lat_pack8 bq;
        bq.q = make_uint4(0, 0, 0, 0);
        if (h < n_heads && e0 + 8 <= dk) {
            const float4* src = reinterpret_cast<const float4*>(qa + ((size_t)t * n_heads + h) * dk + e0);
            const float4 a = src[0], b = src[1];
            bq.u[0] = float_to_bf16_bits(a.x); bq.u[1] = float_to_bf16_bits(a.y);
            bq.u[2] = float_to_bf16_bits(a.z); bq.u[3] = float_to_bf16_bits(a.w);
            bq.u[4] = float_to_bf16_bits(b.x); bq.u[5] = float_to_bf16_bits(b.y);
            bq.u[6] = float_to_bf16_bits(b.z); bq.u[7] = float_to_bf16_bits(b.w);
        }
        q_lds[ks][ln] = bq.q;
    }
    __syncthreads();
    lat_floatx4_t o[CT];
#pragma unroll
    for (int c = 0; c < CT; ++c) o[c] = lat_floatx4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    for (int kb = (lo / TQK_PAGE + part) * TQK_PAGE; kb <= pos; kb += TQK_PAGE * n_parts) {
        const int page = max(0, pages[kb / TQK_PAGE]);
        const bf16_t* kp = cache + ((size_t)page * TQK_PAGE + 16 * wave + r16) * dk;
        const bf16_t* vp = turned + (size_t)page * rk * TQK_PAGE;
        lat_floatx4_t s = lat_floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int e0 = 32 * ks + 8 * g;
            const bool in = e0 + 8 <= dk;
            lat_pack8 a, bq;
            a.q = *reinterpret_cast<const uint4*>(kp + (in ? e0 : dk - 8));
            if (!in) a.q = make_uint4(0, 0, 0, 0);
            bq.q = q_lds[ks][lane];
            s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, bq.v, s, 0, 0, 0);
        }
        float p[4];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = kb + 16 * wave + 4 * g + i;
            p[i] = key >= lo && key <= pos ? s[i] * scale : -INFINITY;
            mx = fmaxf(mx, p[i]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, TQK_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, TQK_WAVE));
        if (g == 0) mx_lds[wave][r16] = mx;
        __syncthreads();
        const float m_new = fmaxf(fmaxf(m, fmaxf(mx_lds[0][r16], mx_lds[1][r16])), fmaxf(mx_lds[2][r16], mx_lds[3][r16]));   // finite
        const float alpha = expf(m - m_new);
        float sum = 0.f;
        lat_pack8 mine;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            p[i] = expf(p[i] - m_new);
            sum += p[i];
            mine.u[i] = float_to_bf16_bits(p[i]);
        }
        sum += __shfl_xor(sum, 16, TQK_WAVE);
        sum += __shfl_xor(sum, 32, TQK_WAVE);
        if (g == 0) sum_lds[wave][r16] = sum;
        p_lds[wave][lane] = make_uint2(mine.q.x, mine.q.y);
        __syncthreads();
        l = l * alpha + ((sum_lds[0][r16] + sum_lds[1][r16]) + (sum_lds[2][r16] + sum_lds[3][r16]));
        m = m_new;
        lat_pack8 pb[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint2 first = p_lds[2 * h][lane], second = p_lds[2 * h + 1][lane];
            pb[h].q = make_uint4(first.x, first.y, second.x, second.y);
        }
        const bool edge = kb < lo || kb + TQK_PAGE - 1 > pos;
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            const int col = 16 * (wave * CT + c) + r16;
            const int colc = min(col, rk - 1);
            o[c] *= alpha;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                lat_pack8 a;
                a.q = *reinterpret_cast<const uint4*>(vp + (size_t)colc * TQK_PAGE + 32 * h + 8 * g);
                if (col >= rk) a.q = make_uint4(0, 0, 0, 0);
                if (edge) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int key = kb + value_position(32 * h + 8 * g + e);
                        if (key < lo || key > pos) a.u[e] = 0;
                    }
                }
                o[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pb[h].v, o[c], 0, 0, 0);
            }
        }
        __syncthreads();                                // the next page writes the exchanged values again
    }
    if (head >= n_heads) return;
    float* dst = n_parts > 1 ? part_o + (((size_t)t * n_heads + head) * n_parts + part) * rk : out + ((size_t)t * n_heads + head) * rk;
    const float inv = n_parts > 1 ? 1.f : 1.f / l;
#pragma unroll
    for (int c = 0; c < CT; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int col = 16 * (wave * CT + c) + 4 * g + i;
            if (col < rk) dst[col] = o[c][i] * inv;
        }
    if (n_parts > 1 && wave == 0 && g == 0) {
        float* ml = part_ml + (((size_t)t * n_heads + head) * n_parts + part) * 2;
        ml[0] = m;
        ml[1] = l;
    }
}

// the parts of a (token, head) in their order: out = sum_p o_p e^(m_p - M) / sum_p l_p e^(m_p - M)
#define LAT_MAX_PARTS 128
__global__ __launch_bounds__(128)
void latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, int n_parts, int rk, float* __restrict__ out) {
    __shared__ float wgt[LAT_MAX_PARTS];
    __shared__ float total;
    const size_t row = blockIdx.x;
    const float* ml = part_ml + row * n_parts * 2;
    // the parts' maxima and weights once, side by side, instead of one load after the other in every thread
    const float mine = threadIdx.x < n_parts ? ml[2 * threadIdx.x] : -INFINITY;
    const float mine_l = threadIdx.x < n_parts ? ml[2 * threadIdx.x + 1] : 0.f;
    if (threadIdx.x < LAT_MAX_PARTS) wgt[threadIdx.x] = mine;
    __syncthreads();
    float M = -INFINITY;
    for (int p = 0; p < n_parts; ++p) M = fmaxf(M, wgt[p]);
    __syncthreads();
    if (threadIdx.x < LAT_MAX_PARTS) wgt[threadIdx.x] = threadIdx.x < n_parts ? expf(mine - M) : 0.f;
    __syncthreads();
    if (threadIdx.x == 0) {
        float L = 0.f;
        for (int p = 0; p < n_parts; ++p) L += part_ml[(row * n_parts + p) * 2 + 1] * wgt[p];
        total = L;
    }
    (void)mine_l;
    __syncthreads();
    const float inv = 1.f / total;
    for (int c = threadIdx.x; c < rk; c += blockDim.x) {
        float v = 0.f;
#pragma unroll 8
        for (int p = 0; p < n_parts; ++p) {
            const float x = part_o[(row * n_parts + p) * rk + c];
            v = fmaf(wgt[p] > 0.f ? x : 0.f, wgt[p], v);        // a part without a page left its memory as it was
        }
        out[row * rk + c] = v * inv;
    }
}

// ---- attention on the matrix cores, tiles of queries (prompts) -----------------------------------
// A block of four waves takes up to four consecutive tokens of one sequence, a wave a token's 16 heads.  The products
// are those of the kernel above; what differs is where the cache comes from: the block brings half a page (32
// positions) of rows and of turned latents into LDS in the order the lanes take them, once for all four tokens, so
// the cache is read a quarter as often.  A thread's pieces of the next half are asked for before the products on
// this one and written to LDS after the barrier that ends them.  The absorbed queries stay in registers.
template <int KS, int NCT>
__global__ __launch_bounds__(4 * TQK_WAVE)
void latent_attention_tile_kernel(const float* __restrict__ qa, const bf16_t* __restrict__ cache, const bf16_t* __restrict__ turned,
                                  const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table, int table_width,
                                  const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_tok0,
                                  const int32_t* __restrict__ tile_count, int window, float scale, float* __restrict__ out, int n_heads,
                                  int rk, int dk) {
    constexpr int KP = (128 * KS + 255) / 256;          // 16-byte pieces of half a page of rows a thread brings
    constexpr int VP = NCT / 4;                         // and of turned latents
    __shared__ uint4 lds_k[2 * KS * TQK_WAVE];          // (together up to 72 KB of the 160 KB a compute unit has)
    __shared__ uint4 lds_v[NCT * TQK_WAVE];
    const int tile = blockIdx.x;
    const int tok0 = tile_tok0[tile], count = min(4, tile_count[tile]);
    const int32_t* pages = page_table + (size_t)tile_seq[tile] * table_width;
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int g = lane / 16, r16 = lane % 16;
    const bool has = wave < count;
    const int t = tok0 + min(wave, count - 1);
    const int head = blockIdx.y * 16 + r16;
    const int pos = tok_pos[t];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int pos_max = tok_pos[tok0 + count - 1];
    const int lo_min = window > 0 ? max(0, tok_pos[tok0] - window + 1) : 0;

    lat_pack8 bq[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int e0 = 32 * ks + 8 * g;
        bq[ks].q = make_uint4(0, 0, 0, 0);
        if (has && head < n_heads && e0 + 8 <= dk) {
            const float4* src = reinterpret_cast<const float4*>(qa + ((size_t)t * n_heads + head) * dk + e0);
            const float4 a = src[0], b = src[1];
            bq[ks].u[0] = float_to_bf16_bits(a.x); bq[ks].u[1] = float_to_bf16_bits(a.y);
            bq[ks].u[2] = float_to_bf16_bits(a.z); bq[ks].u[3] = float_to_bf16_bits(a.w);
            bq[ks].u[4] = float_to_bf16_bits(b.x); bq[ks].u[5] = float_to_bf16_bits(b.y);
            bq[ks].u[6] = float_to_bf16_bits(b.z); bq[ks].u[7] = float_to_bf16_bits(b.w);
        }
    }
    lat_floatx4_t o[NCT];
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) o[ct] = lat_floatx4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    // A thread's pieces of half a page are those whose places in LDS follow one another from thread to thread (its
    // writes to LDS then meet no bank twice); in memory a wave's pieces are 64 contiguous bytes of each of 16 rows.
    uint4 k_regs[KP], v_regs[VP];
    auto fetch_rows = [&](int hp) {
        const int page = max(0, pages[hp / 2]);
        const bf16_t* kp = cache + ((size_t)page * TQK_PAGE + (size_t)(hp & 1) * 32) * dk;
#pragma unroll
        for (int n = 0; n < KP; ++n) {
            const int slot = min((int)threadIdx.x + n * 256, 2 * KS * TQK_WAVE - 1);
            const int j = slot / (KS * TQK_WAVE), ks = (slot / TQK_WAVE) % KS, ln = slot % TQK_WAVE;
            const int key = 16 * j + ln % 16, e0 = 32 * ks + 8 * (ln / 16);
            const bool in = e0 + 8 <= dk;
            k_regs[n] = *reinterpret_cast<const uint4*>(kp + (size_t)key * dk + (in ? e0 : 0));
            if (!in) k_regs[n] = make_uint4(0, 0, 0, 0);
        }
    };
    auto store_rows = [&]() {
#pragma unroll
        for (int n = 0; n < KP; ++n) {
            const int slot = threadIdx.x + n * 256;
            if (slot < 2 * KS * TQK_WAVE) lds_k[slot] = k_regs[n];
        }
    };
    // turned latents; what lies at places of positions beyond the tile's last token may be anything and is replaced by zero
    auto fetch_turned = [&](int hp) {
        const int page = max(0, pages[hp / 2]);
        const bf16_t* vp = turned + (size_t)page * rk * TQK_PAGE + (hp & 1) * 32;
        const bool edge = hp * 32 + 31 > pos_max;
#pragma unroll
        for (int n = 0; n < VP; ++n) {
            const int slot = threadIdx.x + n * 256;
            const int col = 16 * (slot / TQK_WAVE) + slot % 16, gq = (slot % TQK_WAVE) / 16;
            lat_pack8 a;
            a.q = *reinterpret_cast<const uint4*>(vp + (size_t)min(col, rk - 1) * TQK_PAGE + 8 * gq);
            if (col >= rk) a.q = make_uint4(0, 0, 0, 0);
            if (edge) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if ((hp / 2) * TQK_PAGE + value_position((hp & 1) * 32 + 8 * gq + e) > pos_max) a.u[e] = 0;
            }
            v_regs[n] = a.q;
        }
    };
    auto store_turned = [&]() {
#pragma unroll
        for (int n = 0; n < VP; ++n) lds_v[threadIdx.x + n * 256] = v_regs[n];
    };

    const int hp_first = lo_min / 32, hp_last = pos_max / 32;
    fetch_rows(hp_first);
    fetch_turned(hp_first);
    store_rows();
    store_turned();
    __syncthreads();
    for (int hp = hp_first; hp <= hp_last; ++hp) {
        const int kb = hp * 32;
        // the next half is asked for now and has this half's products to arrive
        if (hp < hp_last) {
            fetch_rows(hp + 1);
            fetch_turned(hp + 1);
        }
        const bool mine = has && kb <= pos && kb + 31 >= lo;          // the half holds a position this wave's token sees
        if (mine) {
            lat_floatx4_t s[2] = {lat_floatx4_t{0.f, 0.f, 0.f, 0.f}, lat_floatx4_t{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    lat_pack8 a;
                    a.q = lds_k[(j * KS + ks) * TQK_WAVE + lane];
                    s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, bq[ks].v, s[j], 0, 0, 0);
                }
            float p[2][4];
            float mx = -INFINITY;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = kb + 16 * j + 4 * g + i;
                    p[j][i] = key >= lo && key <= pos ? s[j][i] * scale : -INFINITY;
                    mx = fmaxf(mx, p[j][i]);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, TQK_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, TQK_WAVE));
            const float m_new = fmaxf(m, mx);               // finite: the half holds a visible position
            const float alpha = expf(m - m_new);
            float sum = 0.f;
            lat_pack8 pb;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    p[j][i] = expf(p[j][i] - m_new);
                    sum += p[j][i];
                    pb.u[4 * j + i] = float_to_bf16_bits(p[j][i]);
                }
            sum += __shfl_xor(sum, 16, TQK_WAVE);
            sum += __shfl_xor(sum, 32, TQK_WAVE);
            l = l * alpha + sum;
            m = m_new;
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) {
                lat_pack8 a;
                a.q = lds_v[ct * TQK_WAVE + lane];
                o[ct] *= alpha;
                o[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pb.v, o[ct], 0, 0, 0);
            }
        }
        __syncthreads();                                    // every wave is done with this half
        if (hp < hp_last) {
            store_rows();
            store_turned();
        }
        __syncthreads();
    }
    if (!has || head >= n_heads) return;
    float* dst = out + ((size_t)t * n_heads + head) * rk;
    const float inv = 1.f / l;
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int col = 16 * ct + 4 * g + i;
            if (col < rk) dst[col] = o[ct][i] * inv;
        }
}

// ---- values ----------------------------------------------------------------------------------
// A block: LAT_TT tokens of one head; a wave takes value columns in turn, its lanes share a row of
// W_uv (contiguous loads) and their partial sums are added up in a fixed order.
template <typename TA, typename TW>
__global__ __launch_bounds__(256)
void latent_values_kernel(const float* __restrict__ o, const TW* __restrict__ w_uv, const float* __restrict__ gate, int n_heads, int rk,
                          int dv, TA* __restrict__ y, int n_tokens) {
    extern __shared__ float o_lds[];            // [LAT_TT][rk]
    const int head = blockIdx.y, t0 = blockIdx.x * LAT_TT;
    const int n_t = min(LAT_TT, n_tokens - t0);
    for (int i = threadIdx.x; i < LAT_TT * rk; i += blockDim.x) {
        const int tt = i / rk, c = i % rk;
        o_lds[i] = tt < n_t ? o[((size_t)(t0 + tt) * n_heads + head) * rk + c] : 0.f;
    }
    __syncthreads();
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE, n_waves = blockDim.x / TQK_WAVE;
    for (int n = wave; n < dv; n += n_waves) {
        const TW* w = w_uv + ((size_t)head * dv + n) * rk;
        float acc[LAT_TT];
#pragma unroll
        for (int tt = 0; tt < LAT_TT; ++tt) acc[tt] = 0.f;
        for (int c = lane; c < rk; c += TQK_WAVE) {
            const float wv = to_float(w[c]);
#pragma unroll
            for (int tt = 0; tt < LAT_TT; ++tt) acc[tt] = fmaf(o_lds[tt * rk + c], wv, acc[tt]);
        }
#pragma unroll
        for (int tt = 0; tt < LAT_TT; ++tt) acc[tt] = wave_sum(acc[tt]);
        if (lane < n_t) {
            float v = 0.f;
#pragma unroll
            for (int tt = 0; tt < LAT_TT; ++tt) v = lane == tt ? acc[tt] : v;
            const int t = t0 + lane;
            const float g = gate ? gate[(size_t)t * n_heads + head] : 1.f;
            y[((size_t)t * n_heads + head) * dv + n] = from_float<TA>(v * g);
        }
    }
}

// ---- entry points ----------------------------------------------------------------------------
extern "C" int tqk_latent_max_rank(void) { return LAT_MAX_RK; }
extern "C" int tqk_latent_max_row(void) { return LAT_MAX_DK; }

extern "C" int tqk_latent_split(const void* proj, int act_dtype, int row_stride, int q_rank, int kv_rank, int rot_dim, int n_gate, const void* q_norm_w,
                                const void* kv_norm_w, int norm_dtype, float eps, const float* cos_table, const float* sin_table,
                                int rot_dims, int max_positions, const int32_t* tok_seq, const int32_t* tok_pos,
                                const int32_t* page_table, int table_width, void* cache, void* turned, int n_pages, void* cq_out,
                                float* gate_out, int n_tokens, void* stream) {
    TQK_REQUIRE(proj && q_norm_w && cq_out, "tqk_latent_split: null pointer");
    TQK_REQUIRE(q_rank > 0 && kv_rank >= 0 && rot_dim >= 0 && n_gate >= 0 && n_tokens >= 0, "tqk_latent_split: bad sizes");
    TQK_REQUIRE(n_gate == 0 || gate_out, "tqk_latent_split: no place for the gates");
    TQK_REQUIRE(row_stride >= q_rank + (kv_rank > 0 ? kv_rank + rot_dim : 0) + n_gate, "tqk_latent_split: rows of %d values are too short", row_stride);
    if (kv_rank > 0) {
        TQK_REQUIRE(kv_norm_w && cache && tok_seq && tok_pos && page_table && table_width > 0 && n_pages > 0, "tqk_latent_split: no cache to write");
        TQK_REQUIRE(rot_dims >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0, "tqk_latent_split: %d of %d elements rotate", rot_dims, rot_dim);
        TQK_REQUIRE(rot_dims == 0 || (cos_table && sin_table && max_positions > 0), "tqk_latent_split: no angle tables");
    }
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
#define TQK_SPLIT(TA, TW)                                                                                                              \
    latent_split_kernel<TA, TW><<<n_tokens, 256, 0, s>>>((const TA*)proj, row_stride, q_rank, kv_rank, rot_dim, n_gate, (const TW*)q_norm_w,       \
                                                         (const TW*)kv_norm_w, eps, cos_table, sin_table, rot_dims, max_positions,     \
                                                         tok_seq, tok_pos, page_table, table_width, (TA*)cache, (TA*)turned, n_pages,  \
                                                         (TA*)cq_out, gate_out)
    if (act_dtype == TQK_F32 && norm_dtype == TQK_F32) TQK_SPLIT(float, float);
    else if (act_dtype == TQK_F32 && norm_dtype == TQK_BF16) TQK_SPLIT(float, bf16_t);
    else if (act_dtype == TQK_BF16 && norm_dtype == TQK_F32) TQK_SPLIT(bf16_t, float);
    else if (act_dtype == TQK_BF16 && norm_dtype == TQK_BF16) TQK_SPLIT(bf16_t, bf16_t);
    else return tqk_fail("tqk_latent_split: unknown dtypes %d, %d", act_dtype, norm_dtype);
#undef TQK_SPLIT
    return tqk_check_launch("tqk_latent_split");
}

extern "C" int tqk_latent_absorb(const void* q, int act_dtype, const void* w_uk, int w_dtype, int n_heads, int dn, int dr, int rk,
                                 const float* cos_table, const float* sin_table, int rot_dims, int max_positions,
                                 const int32_t* tok_pos, float* qa, int n_tokens, int tail_only, void* stream) {
    TQK_REQUIRE(q && (w_uk || tail_only) && qa && tok_pos, "tqk_latent_absorb: null pointer");
    TQK_REQUIRE(n_heads > 0 && n_heads <= 65535 && dn > 0 && dr >= 0 && rk > 0 && n_tokens >= 0, "tqk_latent_absorb: bad sizes");
    TQK_REQUIRE(rot_dims >= 0 && rot_dims <= dr && rot_dims % 2 == 0, "tqk_latent_absorb: %d of %d elements rotate", rot_dims, dr);
    TQK_REQUIRE(rot_dims == 0 || (cos_table && sin_table && max_positions > 0), "tqk_latent_absorb: no angle tables");
    const size_t lds = (size_t)LAT_TT * (dn + dr) * sizeof(float);
    TQK_REQUIRE(lds <= 48 * 1024, "tqk_latent_absorb: a head of %d + %d elements is more than the kernel stages", dn, dr);
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((n_tokens + LAT_TT - 1) / LAT_TT, n_heads);
#define TQK_ABSORB(TA, TW)                                                                                                             \
    latent_absorb_kernel<TA, TW><<<grid, 128, lds, s>>>((const TA*)q, (const TW*)w_uk, n_heads, dn, dr, rk, cos_table, sin_table,      \
                                                        rot_dims, max_positions, tok_pos, qa, n_tokens, tail_only)
    if (act_dtype == TQK_F32 && w_dtype == TQK_F32) TQK_ABSORB(float, float);
    else if (act_dtype == TQK_F32 && w_dtype == TQK_BF16) TQK_ABSORB(float, bf16_t);
    else if (act_dtype == TQK_BF16 && w_dtype == TQK_F32) TQK_ABSORB(bf16_t, float);
    else if (act_dtype == TQK_BF16 && w_dtype == TQK_BF16) TQK_ABSORB(bf16_t, bf16_t);
    else return tqk_fail("tqk_latent_absorb: unknown dtypes %d, %d", act_dtype, w_dtype);
#undef TQK_ABSORB
    return tqk_check_launch("tqk_latent_absorb");
}

extern "C" int tqk_latent_attention_mfma_supported(int rk, int dr) { return (rk + dr) % 8 == 0 && rk <= LAT_MAX_RK && rk + dr <= LAT_MAX_DK; }

/* how many waves a token's pages are best dealt out to (1: none of it), and the scratch memory that takes */
extern "C" int tqk_latent_attention_parts(int n_tokens, int n_heads, int table_width, int window) {
    const long long items = (long long)n_tokens * ((n_heads + 15) / 16);
    const int pages = window > 0 ? std::min(table_width, (window + TQK_PAGE - 2) / TQK_PAGE + 1) : table_width;
    if (items >= 512 || pages <= 1) return 1;
    return (int)std::max(1LL, std::min(std::min((long long)pages, (long long)LAT_MAX_PARTS), 1024 / std::max(1LL, items)));
}

extern "C" int tqk_latent_attention_mfma(const float* qa, const void* cache, const void* turned, const int32_t* tok_seq, const int32_t* tok_pos,
                                         const int32_t* page_table, int table_width, int n_seqs, int n_pages, int window, float scale,
                                         float* out, int n_tokens, int n_heads, int rk, int dr, int n_parts, float* part_o, float* part_ml,
                                         void* stream) {
    TQK_REQUIRE(n_parts >= 1 && n_parts <= LAT_MAX_PARTS && (n_parts == 1 || (part_o && part_ml)),
                "tqk_latent_attention_mfma: %d parts (1 to %d, with memory for them)", n_parts, LAT_MAX_PARTS);
    TQK_REQUIRE(qa && cache && turned && tok_seq && tok_pos && page_table && out, "tqk_latent_attention_mfma: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_heads > 0 && rk > 0 && dr >= 0, "tqk_latent_attention_mfma: bad sizes");
    TQK_REQUIRE(tqk_latent_attention_mfma_supported(rk, dr), "tqk_latent_attention_mfma: a latent of %d + %d values is not taken", rk, dr);
    TQK_REQUIRE(table_width > 0 && n_pages > 0 && n_seqs > 0 && window >= 0, "tqk_latent_attention_mfma: empty page table or negative window");
    TQK_REQUIRE(((((uintptr_t)qa) | ((uintptr_t)cache) | ((uintptr_t)turned)) & 15) == 0, "tqk_latent_attention_mfma: operands must be 16-byte aligned");
    if (n_tokens == 0) return 0;
    const int dk = rk + dr, n_chunks = (n_heads + 15) / 16;
    const long long items = (long long)n_tokens * n_chunks * n_parts;
    TQK_REQUIRE(items <= 0x7fffffffLL, "tqk_latent_attention_mfma: too many rows");
    hipStream_t s = (hipStream_t)stream;
#define TQK_LAT_MFMA(KS, NCT, WAVES)                                                                                                  \
    latent_attention_mfma_kernel<KS, NCT, WAVES><<<(unsigned)((items + WAVES - 1) / WAVES), WAVES * TQK_WAVE, 0, s>>>(                  \
        qa, (const bf16_t*)cache, (const bf16_t*)turned, tok_seq, tok_pos, page_table, table_width, window, scale, out, n_tokens, n_heads, \
        n_chunks, rk, dk, n_parts, part_o, part_ml)
    // the smallest build that holds the row and the latent (steps and blocks beyond the sizes multiply zeros)
    // a block of four waves per (token, 16 heads, part) wherever that leaves the chip enough blocks; a wave each otherwise
#define TQK_LAT_PAGE(KS, NCT)                                                                                                          \
    latent_attention_page_kernel<KS, NCT><<<(unsigned)items, 4 * TQK_WAVE, 0, s>>>(qa, (const bf16_t*)cache, (const bf16_t*)turned, tok_seq, \
                                                                                   tok_pos, page_table, table_width, window, scale, out,    \
                                                                                   n_heads, n_chunks, rk, dk, n_parts, part_o, part_ml)
    const bool by_block = items <= 16384;
    if (rk <= 128 && dk <= 160) { if (by_block) TQK_LAT_PAGE(5, 8); else TQK_LAT_MFMA(5, 8, 4); }
    else if (rk <= 256 && dk <= 320) { if (by_block) TQK_LAT_PAGE(10, 16); else TQK_LAT_MFMA(10, 16, 4); }
    else if (dk <= 576) { if (by_block) TQK_LAT_PAGE(18, 32); else TQK_LAT_MFMA(18, 32, 2); }
    else { if (by_block) TQK_LAT_PAGE(20, 32); else TQK_LAT_MFMA(20, 32, 2); }
#undef TQK_LAT_PAGE
#undef TQK_LAT_MFMA
    if (tqk_check_launch("tqk_latent_attention_mfma")) return -1;
    if (n_parts > 1) {
        latent_merge_kernel<<<(unsigned)(n_tokens * n_heads), 128, 0, s>>>(part_o, part_ml, n_parts, rk, out);
        return tqk_check_launch("tqk_latent_attention_mfma merge");
    }
    return 0;
}

/* The same for steps that bring several tokens per sequence: tiles of up to 4 consecutive tokens of one sequence (tile i:
 * sequence tile_seq[i], first packed token tile_tok0[i], tile_count[i] tokens), a block a tile. */
extern "C" int tqk_latent_attention_tiles(const float* qa, const void* cache, const void* turned, const int32_t* tok_pos,
                                          const int32_t* page_table, int table_width, int n_seqs, int n_pages, const int32_t* tile_seq,
                                          const int32_t* tile_tok0, const int32_t* tile_count, int n_tiles, int window, float scale,
                                          float* out, int n_tokens, int n_heads, int rk, int dr, void* stream) {
    TQK_REQUIRE(qa && cache && turned && tok_pos && page_table && out && tile_seq && tile_tok0 && tile_count, "tqk_latent_attention_tiles: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_tiles >= 0 && n_heads > 0 && rk > 0 && dr >= 0, "tqk_latent_attention_tiles: bad sizes");
    TQK_REQUIRE(tqk_latent_attention_mfma_supported(rk, dr), "tqk_latent_attention_tiles: a latent of %d + %d values is not taken", rk, dr);
    TQK_REQUIRE(table_width > 0 && n_pages > 0 && n_seqs > 0 && window >= 0, "tqk_latent_attention_tiles: empty page table or negative window");
    TQK_REQUIRE(((((uintptr_t)qa) | ((uintptr_t)cache) | ((uintptr_t)turned)) & 15) == 0, "tqk_latent_attention_tiles: operands must be 16-byte aligned");
    if (n_tokens == 0 || n_tiles == 0) return 0;
    const int dk = rk + dr;
    dim3 grid(n_tiles, (n_heads + 15) / 16);
    TQK_REQUIRE(grid.y <= 65535, "tqk_latent_attention_tiles: too many heads for the grid");
    hipStream_t s = (hipStream_t)stream;
#define TQK_LAT_TILE(KS, NCT)                                                                                                           \
    latent_attention_tile_kernel<KS, NCT><<<grid, 4 * TQK_WAVE, 0, s>>>(qa, (const bf16_t*)cache, (const bf16_t*)turned, tok_pos, page_table, \
                                                                        table_width, tile_seq, tile_tok0, tile_count, window, scale, out,    \
                                                                        n_heads, rk, dk)
    if (rk <= 128 && dk <= 160) TQK_LAT_TILE(5, 8);
    else if (rk <= 256 && dk <= 320) TQK_LAT_TILE(10, 16);
    else if (dk <= 576) TQK_LAT_TILE(18, 32);
    else TQK_LAT_TILE(20, 32);
#undef TQK_LAT_TILE
    return tqk_check_launch("tqk_latent_attention_tiles");
}

extern "C" int tqk_latent_attention(const float* qa, const void* cache, int cache_dtype, const int32_t* tok_seq, const int32_t* tok_pos,
                                    const int32_t* page_table, int table_width, int n_seqs, int n_pages, int window, float scale,
                                    float* out, int n_tokens, int n_heads, int rk, int dr, void* stream) {
    TQK_REQUIRE(qa && cache && tok_seq && tok_pos && page_table && out, "tqk_latent_attention: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_heads <= 65535 && rk > 0 && dr >= 0, "tqk_latent_attention: bad sizes");
    TQK_REQUIRE(rk <= LAT_MAX_RK && rk + dr <= LAT_MAX_DK, "tqk_latent_attention: a latent of %d + %d is more than %d + %d", rk, dr, LAT_MAX_RK,
                LAT_MAX_DK - LAT_MAX_RK);
    TQK_REQUIRE(table_width > 0 && n_pages > 0 && n_seqs > 0 && window >= 0, "tqk_latent_attention: empty page table or negative window");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((n_tokens + LAT_WAVES - 1) / LAT_WAVES, n_heads);
    if (cache_dtype == TQK_F32)
        latent_attention_kernel<float><<<grid, LAT_WAVES * TQK_WAVE, 0, s>>>(qa, (const float*)cache, tok_seq, tok_pos, page_table, table_width,
                                                                             window, scale, out, n_tokens, n_heads, rk, rk + dr);
    else if (cache_dtype == TQK_BF16)
        latent_attention_kernel<bf16_t><<<grid, LAT_WAVES * TQK_WAVE, 0, s>>>(qa, (const bf16_t*)cache, tok_seq, tok_pos, page_table, table_width,
                                                                              window, scale, out, n_tokens, n_heads, rk, rk + dr);
    else return tqk_fail("tqk_latent_attention: unknown dtype %d", cache_dtype);
    return tqk_check_launch("tqk_latent_attention");
}

extern "C" int tqk_latent_values(const float* o, const void* w_uv, int w_dtype, const float* gate, int n_heads, int rk, int dv, void* y,
                                 int y_dtype, int n_tokens, void* stream) {
    TQK_REQUIRE(o && w_uv && y, "tqk_latent_values: null pointer");
    TQK_REQUIRE(n_heads > 0 && n_heads <= 65535 && rk > 0 && dv > 0 && n_tokens >= 0, "tqk_latent_values: bad sizes");
    const size_t lds = (size_t)LAT_TT * rk * sizeof(float);
    TQK_REQUIRE(lds <= 48 * 1024, "tqk_latent_values: a latent of %d elements is more than the kernel stages", rk);
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((n_tokens + LAT_TT - 1) / LAT_TT, n_heads);
#define TQK_VALUES(TA, TW) \
    latent_values_kernel<TA, TW><<<grid, 256, lds, s>>>(o, (const TW*)w_uv, gate, n_heads, rk, dv, (TA*)y, n_tokens)
    if (y_dtype == TQK_F32 && w_dtype == TQK_F32) TQK_VALUES(float, float);
    else if (y_dtype == TQK_F32 && w_dtype == TQK_BF16) TQK_VALUES(float, bf16_t);
    else if (y_dtype == TQK_BF16 && w_dtype == TQK_F32) TQK_VALUES(bf16_t, float);
    else if (y_dtype == TQK_BF16 && w_dtype == TQK_BF16) TQK_VALUES(bf16_t, bf16_t);
    else return tqk_fail("tqk_latent_values: unknown dtypes %d, %d", y_dtype, w_dtype);
#undef TQK_VALUES
    return tqk_check_launch("tqk_latent_values");
}
