// Attention through low-rank latents, with a window, an output gate per head, and layers that read
// another layer's cache.
//
// h is the mixer's input [tokens, hidden].  Queries go through a latent: cq = norm(W_dq h) with a
// plain weight, q = W_uq cq, laid out head by head as [dim unrotated | rot_dim rotated].  Keys and
// values come from one latent per position: W_dkv h gives kv_rank values, normed with a plain
// weight, which are the latent c, and rot_dim more, which (rotated, not normed) are a key part
// that all heads share.  Head i's key is (W_uk,i c, shared part), its value W_uv,i c; the score is
// the dot product of query and key times `scale`, over the positions the window shows, with an
// ordinary softmax.  Head i's output is multiplied by sigmoid(W_g h)_i, and W_o is applied to the
// heads side by side.
//
// Only c and the rotated part are cached, one row per position for all heads.  The kernels never
// form a key or a value: the query is taken into the latent's space (W_uk,i^T q_i), attention runs
// on the cache rows, and W_uv,i is applied to the attended latent (latent.hip).  A layer without a
// projection of its own (own_kv false) reads the rows another run of the order left, with its own
// W_uk, W_uv, queries and window.
//
// params: hidden, n_heads, head_dim (unrotated), rot_dim, value_dim, q_rank, kv_rank, scale, eps,
// window (null: all earlier positions), cache_window (what the cache must keep: the largest window of
// the runs that read it; null: everything), own_kv, gate (the output gate, true unless given),
// position (a part spec whose tables turn the rotated parts).
// Tensors: dq, dq.norm, uq, [dkv, dkv.norm,] uk, uv, [g,] o.
#include <math.h>

#include "kernels.h"
#include "linear.h"
#include "parts.h"
#include "step.h"

namespace tq {
namespace {

OwnedPtr take(Loaded& tensors, const char* name) {
    auto it = tensors.find(name);
    if (it == tensors.end() || !it->second) raise(TQE_ERR_WEIGHTS, "a part was not given its tensor '%s'", name);
    return it->second;
}

class LatentAttention : public Mixer {
public:
    LatentAttention(const PartSpec& spec, BuildEnv& env) {
        KeyReader r(spec.params, "latent_attention", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        n_heads_ = (int)r.integer("n_heads", 1);
        dn_ = (int)r.integer("head_dim", 1);
        dr_ = (int)r.integer("rot_dim", 0);
        dv_ = (int)r.integer("value_dim", 1);
        q_rank_ = (int)r.integer("q_rank", 1);
        kv_rank_ = (int)r.integer("kv_rank", 1);
        scale_ = (float)r.number("scale");
        eps_ = (float)r.number("eps");
        window_ = r.has("window") ? (int)r.integer("window", 1) : 0;
        cache_window_ = r.has("cache_window") ? (int)r.integer("cache_window", 1) : 0;
        if (window_ == 0 && cache_window_ != 0) raise(TQE_ERR_ARGUMENT, "latent_attention: the cache keeps %d positions but the mixer sees all", cache_window_);
        if (cache_window_ != 0 && cache_window_ < window_)
            raise(TQE_ERR_ARGUMENT, "latent_attention: the cache keeps %d positions, fewer than the window of %d", cache_window_, window_);
        own_kv_ = r.boolean_or("own_kv", true);
        gated_ = r.boolean_or("gate", true);
        if (n_heads_ > 65535) raise(TQE_ERR_CONFIG, "latent_attention: %d heads are more than the kernels take (65535)", n_heads_);
        const int max_rk = K::latent_max_rank.raw(), max_row = K::latent_max_row.raw();
        if (kv_rank_ > max_rk || kv_rank_ + dr_ > max_row)
            raise(TQE_ERR_CONFIG, "latent_attention: a latent of %d + %d values is more than the kernels take (%d, %d with the rotated part)", kv_rank_,
                  dr_, max_rk, max_row);
        if ((int64_t)(dn_ + dr_) * 8 * 4 > 48 * 1024 || (int64_t)kv_rank_ * 8 * 4 > 48 * 1024)
            raise(TQE_ERR_CONFIG, "latent_attention: heads of %d + %d values are more than the kernels stage", dn_, dr_);
        if (dr_ > 0) {
            const PartSpec pos = PartSpec::from_json(spec.params["position"], "latent_attention: position");
            const std::string key = "position:" + pos.key();
            auto it = env.shared.find(key);
            if (it == env.shared.end()) it = env.shared.emplace(key, build_part("position", pos, env)).first;
            position_ = std::dynamic_pointer_cast<Position>(it->second);
            if (!position_ || position_->has_apply() || position_->acts_on_stream())
                raise(TQE_ERR_ARGUMENT, "latent_attention: position kind '%s' offers no tables", pos.kind.c_str());
            const Position::Tables tb = position_->tables();
            if (tb.style != STYLE_NONE && (tb.style != STYLE_HALVES || tb.rot_dim > dr_))
                raise(TQE_ERR_ARGUMENT, "latent_attention: the rotated part has %d values and turns in halves; the position part turns %d", dr_, tb.rot_dim);
        }
        graph_safe = true;
    }

    TensorSpecs tensors() const override {
        auto w = [](int64_t a, int64_t b) { TensorSpec t; t.shape = {a, b}; return t; };
        auto n = [](int64_t a) { TensorSpec t; t.shape = {a}; t.init = "one_plus_normal"; return t; };
        TensorSpecs t = {{"dq", w(q_rank_, hidden_)}, {"dq.norm", n(q_rank_)}, {"uq", w((int64_t)n_heads_ * (dn_ + dr_), q_rank_)}};
        if (own_kv_) { t.push_back({"dkv", w(kv_rank_ + dr_, hidden_)}); t.push_back({"dkv.norm", n(kv_rank_)}); }
        t.push_back({"uk", w((int64_t)n_heads_ * dn_, kv_rank_)});
        t.push_back({"uv", w((int64_t)n_heads_ * dv_, kv_rank_)});
        if (gated_) t.push_back({"g", w(n_heads_, hidden_)});
        t.push_back({"o", w(hidden_, (int64_t)n_heads_ * dv_)});
        return t;
    }

    void load(Loaded& t, hipStream_t stream) override {
        // the products that read h are one: [q latent | kv latent and rotated part | gate logits], rows padded to 16
        std::vector<OwnedPtr> first = {take(t, "dq")};
        if (own_kv_) first.push_back(take(t, "dkv"));
        if (gated_) first.push_back(take(t, "g"));
        OwnedPtr in = stack_rows(first, stream, 16);
        in_cols_ = in->t.shape[0];
        w_in_ = make_weight(in, 1, false, stream);
        q_norm_ = take(t, "dq.norm");
        if (own_kv_) kv_norm_ = take(t, "dkv.norm");
        if (kv_norm_ && kv_norm_->t.dtype != q_norm_->t.dtype) raise(TQE_ERR_WEIGHTS, "latent_attention: the two latents' norm weights differ in type");
        w_uq_ = make_weight(take(t, "uq"), 1, false, stream);
        uk_ = take(t, "uk");
        uv_ = take(t, "uv");
        // For the matrix cores a head's W_uk is wanted with the latent's elements as its rows, [heads][kv_rank][head_dim]:
        // turned once, on the host.
        if (uk_->t.dtype == BF16 && uv_->t.dtype == BF16 && dn_ % 8 == 0 && (dn_ + dr_) % 8 == 0 && kv_rank_ % 8 == 0) {
            std::vector<uint16_t> rows((size_t)uk_->t.numel()), turned(rows.size());
            copy_to_host(rows.data(), uk_->t.data, uk_->t.bytes(), stream);
            for (int h = 0; h < n_heads_; ++h)
                for (int d = 0; d < dn_; ++d)
                    for (int j = 0; j < kv_rank_; ++j)
                        turned[((size_t)h * kv_rank_ + j) * dn_ + d] = rows[((size_t)h * dn_ + d) * kv_rank_ + j];
            uk_turned_ = make_owned(BF16, {n_heads_, kv_rank_, dn_});
            copy_to_device(uk_turned_->t.data, turned.data(), turned.size() * 2, stream);
            stream_synchronize(stream);
        }
        w_o_ = make_weight(take(t, "o"), 1, false, stream);
    }
    OwnedPtr held(const std::string& name) const override {
        if (name == "in.weight") return w_in_.rows;
        if (name == "uq") return w_uq_.rows;
        if (name == "uk") return uk_;
        if (name == "uk.turned") return uk_turned_;
        if (name == "uv") return uv_;
        if (name == "o") return w_o_.rows;
        if (name == "dq.norm") return q_norm_;
        if (name == "dkv.norm") return kv_norm_;
        return nullptr;
    }
    const char* trace_name() const override { return "attn"; }
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        out.push_back({in_cols_ ? in_cols_ : q_rank_ + kv_rank_ + dr_ + n_heads_, hidden_});
        out.push_back({(int64_t)n_heads_ * (dn_ + dr_), q_rank_});
        out.push_back({hidden_, (int64_t)n_heads_ * dv_});
    }

    CacheNeed cache_need() const override {
        CacheNeed n;
        n.kind = CacheNeed::Pages;
        n.key_page = {TQE_PAGE, kv_rank_ + dr_};
        n.value_page = {kv_rank_, TQE_PAGE};    // the latents a second time, turned, for the matrix cores (bfloat16 runs)
        n.window = cache_window_;
        return n;
    }
    bool adds_to_stream(const StepContext& c) const override { return fusable(c.n_tokens, w_o_, true) || leaves_sums(c.n_tokens, w_o_); }

    Tensor forward(StepContext& c, const Activation& x, const CacheEntry& entry, Stream* stream, bool) override {
        if (entry.kind != CacheNeed::Pages) raise(TQE_ERR_STATE, "latent_attention was given no pages of the cache");
        if (x.lazy) raise(TQE_ERR_STATE, "latent_attention takes no folded norm");
        if (entry.writes != own_kv_)
            raise(TQE_ERR_STATE, own_kv_ ? "latent_attention: a layer with a key-value projection of its own was told to read another run's cache"
                                         : "latent_attention: a layer without a key-value projection has no run to read the cache of");
        const int64_t n = x.x.shape[0];
        const int dtype = x.x.dtype;
        const StepContext::Table& table = c.tables.at((size_t)entry.group);
        const int n_pages = (int)entry.keys.shape[0];
        Position::Tables tb;
        if (position_) tb = position_->tables();
        const bool turns = tb.style != STYLE_NONE;
        const float* cos = turns ? (const float*)tb.cos.data : nullptr;
        const float* sin = turns ? (const float*)tb.sin.data : nullptr;
        const int rot_dims = turns ? tb.rot_dim : 0, max_pos = turns ? (int)tb.cos.shape[0] : 0;

        // a bfloat16 cache is read by the matrix cores, which want the latents a second time, turned
        const bool on_cores = entry.keys.dtype == BF16 && policy().prefill_mfma && policy().decode_mfma &&
                              K::latent_attention_mfma_supported.raw(kv_rank_, dr_) != 0;
        Tensor first = linear(c, x.x, w_in_, nullptr, dtype).t;                 // [n, in_cols_]
        Tensor cq = c.alloc(dtype, {n, q_rank_});
        Tensor gate = gated_ ? c.alloc(F32, {n, n_heads_}) : Tensor();
        K::latent_split(first.data, dtype, (int)in_cols_, q_rank_, own_kv_ ? kv_rank_ : 0, dr_, gated_ ? n_heads_ : 0, q_norm_->t.data,
                        kv_norm_ ? kv_norm_->t.data : nullptr, q_norm_->t.dtype, eps_, cos, sin, rot_dims, max_pos, c.dev.tok_seq, c.dev.tok_pos,
                        table.dev, table.width, own_kv_ ? entry.keys.data : nullptr, own_kv_ && on_cores ? entry.values.data : nullptr, n_pages, cq.data,
                        (float*)gate.data, (int)n, c.stream);
        Tensor q = linear(c, cq, w_uq_, nullptr, dtype).t;                        // [n, heads, dn + dr]
        Tensor qa = c.alloc(F32, {n, n_heads_, kv_rank_ + dr_});
        // the two products per head: bfloat16 on the matrix cores where the sizes allow, else in the latent kernels themselves
        const bool heads_on_cores = dtype == BF16 && uk_turned_ && policy().skinny;
        if (heads_on_cores)
            K::head_product(q.data, 0, (long long)n_heads_ * (dn_ + dr_), (long long)(dn_ + dr_), uk_turned_->t.data, qa.data, 1,
                            (long long)n_heads_ * (kv_rank_ + dr_), (long long)(kv_rank_ + dr_), nullptr, (int)n, n_heads_, kv_rank_, dn_, c.stream);
        K::latent_absorb(q.data, dtype, uk_->t.data, uk_->t.dtype, n_heads_, dn_, dr_, kv_rank_, cos, sin, rot_dims, max_pos, c.dev.tok_pos,
                         (float*)qa.data, (int)n, heads_on_cores ? 1 : 0, c.stream);
        Tensor o = c.alloc(F32, {n, n_heads_, kv_rank_});
        if (on_cores && !c.all_decode && !c.capturing) {
            // several tokens per sequence: tiles of four consecutive tokens share what they read of the cache
            const Tiles tl = c.query_tiles(4);
            K::latent_attention_tiles((const float*)qa.data, entry.keys.data, entry.values.data, c.dev.tok_pos, table.dev, table.width, c.n_seqs,
                                      n_pages, tl.seq, tl.tok0, tl.count, tl.n, window_, scale_, (float*)o.data, (int)n, n_heads_, kv_rank_, dr_,
                                      c.stream);
        } else if (on_cores) {
            // few tokens (decoding): a token's pages go to several waves, whose results a second kernel merges
            const int n_parts = K::latent_attention_parts.raw((int)n, n_heads_, table.width, window_);
            Tensor part_o, part_ml;
            if (n_parts > 1) {
                part_o = c.alloc(F32, {n, n_heads_, n_parts, kv_rank_});
                part_ml = c.alloc(F32, {n, n_heads_, n_parts, 2});
            }
            K::latent_attention_mfma((const float*)qa.data, entry.keys.data, entry.values.data, c.dev.tok_seq, c.dev.tok_pos, table.dev, table.width,
                                     c.n_seqs, n_pages, window_, scale_, (float*)o.data, (int)n, n_heads_, kv_rank_, dr_, n_parts,
                                     (float*)part_o.data, (float*)part_ml.data, c.stream);
        } else
            K::latent_attention((const float*)qa.data, entry.keys.data, entry.keys.dtype, c.dev.tok_seq, c.dev.tok_pos, table.dev, table.width, c.n_seqs,
                                n_pages, window_, scale_, (float*)o.data, (int)n, n_heads_, kv_rank_, dr_, c.stream);
        Tensor y = c.alloc(dtype, {n, (int64_t)n_heads_ * dv_});
        if (heads_on_cores)
            K::head_product(o.data, 1, (long long)n_heads_ * kv_rank_, (long long)kv_rank_, uv_->t.data, y.data, 0, (long long)n_heads_ * dv_,
                            (long long)dv_, (const float*)gate.data, (int)n, n_heads_, dv_, kv_rank_, c.stream);
        else
            K::latent_values((const float*)o.data, uv_->t.data, uv_->t.dtype, (const float*)gate.data, n_heads_, kv_rank_, dv_, y.data, dtype, (int)n,
                             c.stream);
        if (stream) {
            add_product(c, *stream, y, w_o_);
            return Tensor();
        }
        return linear(c, y, w_o_, nullptr, dtype).t;
    }

private:
    int64_t hidden_, in_cols_ = 0;
    int n_heads_, dn_, dr_, dv_, q_rank_, kv_rank_, window_, cache_window_;
    float scale_, eps_;
    bool own_kv_, gated_;
    std::shared_ptr<Position> position_;
    Weight w_in_, w_uq_, w_o_;
    OwnedPtr q_norm_, kv_norm_, uk_, uv_, uk_turned_;
};

}  // namespace

void register_latent_parts() {
    register_kind("mixer", "latent_attention", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<LatentAttention>(s, e); });
}

}  // namespace tq
