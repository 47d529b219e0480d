// Small kernels on the residual stream and beside it: an embedding of hashed token pairs with
// the previous token kept per sequence, a norm on a part's output that is added to the stream,
// an activation of one product, and a per-token sigmoid gate.  float32 arithmetic throughout.
#include "common.h"
#include "tq_kernels.h"

// ---- hashed pairs ------------------------------------------------------------------------------
// h[t] += table[row], row = (prev * mul_prev + token * mul_cur) mod buckets, and the table's row
// `buckets` for a sequence's first token.  The previous token is the one before it in the step, or,
// for the first token a step brings of a sequence that has begun, what `last` holds for its slot.
template <typename TT>
__global__ __launch_bounds__(256)
void pair_embed_kernel(const TT* __restrict__ table, int buckets, long long mul_prev, long long mul_cur, const int32_t* __restrict__ tokens,
                       const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ seq_slot,
                       const int32_t* __restrict__ seq_start, int32_t* __restrict__ last, float* __restrict__ h, int hidden, int vocab,
                       bf16_t* __restrict__ copy, int remember) {
    const int t = blockIdx.x;
    const int pos = tok_pos[t], seq = tok_seq[t];
    const int tok = tokens[t];
    if (tok < 0 || tok >= vocab) return;
    long long row = buckets;
    if (pos > 0) {
        const long long prev = pos > seq_start[seq] ? tokens[t - 1] : last[seq_slot[seq]];
        row = (prev * mul_prev + (long long)tok * mul_cur) % buckets;
        if (row < 0) row += buckets;
    }
    // a step of one token a sequence: the token that read the slot's previous token is the one that replaces it
    __syncthreads();
    if (remember && threadIdx.x == 0) last[seq_slot[seq]] = tok;
    const TT* src = table + (size_t)row * hidden;
    float* dst = h + (size_t)t * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float v = dst[i] + to_float(src[i]);
        dst[i] = v;
        if (copy) copy[(size_t)t * hidden + i] = from_float<bf16_t>(v);
    }
}

// last[slot of sequence s] = the last token the step brings of s
__global__ void remember_tokens_kernel(const int32_t* __restrict__ tokens, const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_new,
                                       const int32_t* __restrict__ seq_slot, int32_t* __restrict__ last, int n_seqs) {
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= n_seqs || seq_new[s] <= 0) return;
    last[seq_slot[s]] = tokens[cu[s] + seq_new[s] - 1];
}

// ---- norm of an output, added to the stream ------------------------------------------------------
// h[t] += y[t] / sqrt(mean(y[t]^2) + eps) * w (w null: h[t] += y[t]); copy[t] = h[t] in the activation type.
template <typename TA, typename TW>
__global__ __launch_bounds__(256)
void norm_add_kernel(float* __restrict__ h, const TA* __restrict__ y, const TW* __restrict__ w, float eps, TA* __restrict__ copy, int hidden) {
    __shared__ float scratch[4];
    const int t = blockIdx.x;
    const TA* yr = y ? y + (size_t)t * hidden : nullptr;
    float* hr = h + (size_t)t * hidden;
    float inv = 1.f;
    if (yr && w) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) { const float v = to_float(yr[i]); ss = fmaf(v, v, ss); }
        ss = block_sum(ss, scratch);
        inv = 1.f / sqrtf(ss / (float)hidden + eps);
    }
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v = hr[i];
        if (yr) {
            v += w ? to_float(yr[i]) * inv * to_float(w[i]) : to_float(yr[i]);
            hr[i] = v;
        }
        if (copy) copy[(size_t)t * hidden + i] = from_float<TA>(v);
    }
}

// The same for bfloat16 rows whose length is a multiple of 8 and at most 2048 NCH: a thread takes 8 neighbouring elements at a time with
// 16-byte loads and keeps its part of y in registers between the sum of squares and the update, so a row is read once.
template <typename TW, int NCH>
__global__ __launch_bounds__(256)
void norm_add_vec_kernel(float* __restrict__ h, const bf16_t* __restrict__ y, const TW* __restrict__ w, float eps, bf16_t* __restrict__ copy, int hidden) {
    __shared__ float scratch[4];
    const int t = blockIdx.x;
    float yv[NCH][8];
    float ss = 0.f;
    if (y) {
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            const int i = (threadIdx.x + k * 256) * 8;
            if (i < hidden) {
                const uint4 raw = *reinterpret_cast<const uint4*>(y + (size_t)t * hidden + i);
                const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) { yv[k][2 * j] = __uint_as_float(u[j] << 16); yv[k][2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u); }
#pragma unroll
                for (int j = 0; j < 8; ++j) ss = fmaf(yv[k][j], yv[k][j], ss);
            }
        }
    }
    float inv = 1.f;
    if (y && w) inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)hidden + eps);
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int i = (threadIdx.x + k * 256) * 8;
        if (i >= hidden) continue;
        float* hr = h + (size_t)t * hidden + i;
        float4 a = *reinterpret_cast<const float4*>(hr), b = *reinterpret_cast<const float4*>(hr + 4);
        float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        if (y) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] += w ? yv[k][j] * inv * to_float(w[i + j]) : yv[k][j];
            *reinterpret_cast<float4*>(hr) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4*>(hr + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
        if (copy) {
            uint4 out;
            out.x = float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
            out.y = float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
            out.z = float_to_bf16_bits(v[4]) | ((uint32_t)float_to_bf16_bits(v[5]) << 16);
            out.w = float_to_bf16_bits(v[6]) | ((uint32_t)float_to_bf16_bits(v[7]) << 16);
            *reinterpret_cast<uint4*>(copy + (size_t)t * hidden + i) = out;
        }
    }
}

template <typename TA>
__global__ void unary_act_kernel(const TA* __restrict__ x, TA* __restrict__ out, long long n, int kind, float limit, float alpha) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = from_float<TA>(act_value(kind, limit, alpha, to_float(x[i])));
}

// out[t] = sigmoid(x[t] . w), a wave per token
template <typename TA, typename TW>
__global__ __launch_bounds__(256)
void row_gate_kernel(const TA* __restrict__ x, const TW* __restrict__ w, float* __restrict__ out, int n_tokens, int hidden) {
    const int t = blockIdx.x * 4 + threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    if (t >= n_tokens) return;
    const TA* xr = x + (size_t)t * hidden;
    float d = 0.f;
    for (int i = lane; i < hidden; i += TQK_WAVE) d = fmaf(to_float(xr[i]), to_float(w[i]), d);
    d = wave_sum(d);
    if (lane == 0) out[t] = 1.f / (1.f + expf(-d));
}

extern "C" int tqk_pair_embed(const void* table, int table_dtype, int buckets, long long mul_prev, long long mul_cur, const int32_t* tokens,
                              const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* seq_slot, const int32_t* seq_start,
                              int32_t* last, float* h, int n_tokens, int hidden, int vocab, void* copy_bf16, int remember, void* stream) {
    TQK_REQUIRE(table && tokens && tok_seq && tok_pos && seq_slot && seq_start && last && h, "tqk_pair_embed: null pointer");
    TQK_REQUIRE(buckets > 0 && hidden > 0 && n_tokens >= 0 && vocab > 0, "tqk_pair_embed: bad sizes");
    TQK_REQUIRE(mul_prev >= 0 && mul_cur >= 0 && mul_prev < (1LL << 31) && mul_cur < (1LL << 31), "tqk_pair_embed: multipliers out of range");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (table_dtype == TQK_F32)
        pair_embed_kernel<float><<<n_tokens, 256, 0, s>>>((const float*)table, buckets, mul_prev, mul_cur, tokens, tok_seq, tok_pos, seq_slot, seq_start, last, h, hidden, vocab, (bf16_t*)copy_bf16, remember);
    else if (table_dtype == TQK_BF16)
        pair_embed_kernel<bf16_t><<<n_tokens, 256, 0, s>>>((const bf16_t*)table, buckets, mul_prev, mul_cur, tokens, tok_seq, tok_pos, seq_slot, seq_start, last, h, hidden, vocab, (bf16_t*)copy_bf16, remember);
    else return tqk_fail("tqk_pair_embed: unknown dtype %d", table_dtype);
    return tqk_check_launch("tqk_pair_embed");
}

extern "C" int tqk_remember_tokens(const int32_t* tokens, const int32_t* cu, const int32_t* seq_new, const int32_t* seq_slot, int32_t* last,
                                   int n_seqs, void* stream) {
    TQK_REQUIRE(tokens && cu && seq_new && seq_slot && last, "tqk_remember_tokens: null pointer");
    if (n_seqs <= 0) return 0;
    remember_tokens_kernel<<<(n_seqs + 255) / 256, 256, 0, (hipStream_t)stream>>>(tokens, cu, seq_new, seq_slot, last, n_seqs);
    return tqk_check_launch("tqk_remember_tokens");
}

extern "C" int tqk_norm_add(float* h, const void* y, int act_dtype, const void* weight, int weight_dtype, float eps, void* copy, int n_tokens,
                            int hidden, void* stream) {
    TQK_REQUIRE(h && (y || copy), "tqk_norm_add: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && hidden > 0, "tqk_norm_add: bad sizes");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == TQK_BF16 && hidden % 8 == 0 && hidden <= 8192 && ((((uintptr_t)h) | ((uintptr_t)y) | ((uintptr_t)copy)) & 15) == 0) {
        // (the weight's type only matters where there is a weight)
#define TQK_NAV(TW, NCH) norm_add_vec_kernel<TW, NCH><<<n_tokens, 256, 0, s>>>(h, (const bf16_t*)y, (const TW*)weight, eps, (bf16_t*)copy, hidden)
        if (weight && weight_dtype == TQK_F32) { if (hidden <= 2048) TQK_NAV(float, 1); else if (hidden <= 4096) TQK_NAV(float, 2); else TQK_NAV(float, 4); }
        else { if (hidden <= 2048) TQK_NAV(bf16_t, 1); else if (hidden <= 4096) TQK_NAV(bf16_t, 2); else TQK_NAV(bf16_t, 4); }
#undef TQK_NAV
        return tqk_check_launch("tqk_norm_add");
    }
#define TQK_NA(TA, TW) norm_add_kernel<TA, TW><<<n_tokens, 256, 0, s>>>(h, (const TA*)y, (const TW*)weight, eps, (TA*)copy, hidden)
    if (act_dtype == TQK_F32 && weight_dtype == TQK_F32) TQK_NA(float, float);
    else if (act_dtype == TQK_F32 && weight_dtype == TQK_BF16) TQK_NA(float, bf16_t);
    else if (act_dtype == TQK_BF16 && weight_dtype == TQK_F32) TQK_NA(bf16_t, float);
    else if (act_dtype == TQK_BF16 && weight_dtype == TQK_BF16) TQK_NA(bf16_t, bf16_t);
    else return tqk_fail("tqk_norm_add: unknown dtypes %d, %d", act_dtype, weight_dtype);
#undef TQK_NA
    return tqk_check_launch("tqk_norm_add");
}

extern "C" int tqk_unary_act(const void* x, void* out, int act_dtype, long long n, int kind, float limit, float alpha, void* stream) {
    TQK_REQUIRE(x && out && n >= 0, "tqk_unary_act: null pointer");
    TQK_REQUIRE(kind >= 0 && kind < TQK_GATE_KINDS, "tqk_unary_act: unknown activation %d", kind);
    if (n == 0) return 0;
    const long long blocks = (n + 255) / 256;
    TQK_REQUIRE(blocks <= 0x7fffffff, "tqk_unary_act: too many elements");
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == TQK_F32) unary_act_kernel<float><<<(unsigned)blocks, 256, 0, s>>>((const float*)x, (float*)out, n, kind, limit, alpha);
    else if (act_dtype == TQK_BF16) unary_act_kernel<bf16_t><<<(unsigned)blocks, 256, 0, s>>>((const bf16_t*)x, (bf16_t*)out, n, kind, limit, alpha);
    else return tqk_fail("tqk_unary_act: unknown dtype %d", act_dtype);
    return tqk_check_launch("tqk_unary_act");
}

extern "C" int tqk_row_gate(const void* x, int act_dtype, const void* w, int w_dtype, float* out, int n_tokens, int hidden, void* stream) {
    TQK_REQUIRE(x && w && out, "tqk_row_gate: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && hidden > 0, "tqk_row_gate: bad sizes");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
#define TQK_RG(TA, TW) row_gate_kernel<TA, TW><<<(n_tokens + 3) / 4, 256, 0, s>>>((const TA*)x, (const TW*)w, out, n_tokens, hidden)
    if (act_dtype == TQK_F32 && w_dtype == TQK_F32) TQK_RG(float, float);
    else if (act_dtype == TQK_F32 && w_dtype == TQK_BF16) TQK_RG(float, bf16_t);
    else if (act_dtype == TQK_BF16 && w_dtype == TQK_F32) TQK_RG(bf16_t, float);
    else if (act_dtype == TQK_BF16 && w_dtype == TQK_BF16) TQK_RG(bf16_t, bf16_t);
    else return tqk_fail("tqk_row_gate: unknown dtypes %d, %d", act_dtype, w_dtype);
#undef TQK_RG
    return tqk_check_launch("tqk_row_gate");
}
