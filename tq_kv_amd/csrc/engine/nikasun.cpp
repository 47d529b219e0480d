// Nikasun: a decoder whose layers are listed one by one in its configuration.  Every layer is
// pre-norm (RMS norms whose weights are stored around zero) around a mixer and an optional
// feed-forward; the mixer is attention through low-rank latents with a sliding window, an output
// gate per head and, in some layers, the cache of an earlier layer instead of a key-value
// projection of its own; the feed-forward is dense (ReLU gate) or a set of routed experts with a
// shared one (clamped gates).  The embedding is scaled and doubles as the head.
//
// This file holds what is particular to the architecture: which config.json keys it reads and how
// they become a ModelSpec with the checkpoint's tensor names.  Nothing here computes.
//
// config.json: architecture "Nikasun"; vocab, width; embedding.scale; norm.eps; layers: a list of
// {type, mixer, mlp}.  type "latent_attention": mixer {heads, dim, rot_dim, vdim, q_rank, kv_rank,
// scale, rot {base, dims}, mask {size}, kv_from (optional: the layer whose cache this one reads)}.
// mlp: null, {kind "dense", ff}, or {kind "moe", router {experts, top, scale}, expert {ff, limit},
// shared {ff, limit} (optional)}.  max_positions (optional): the longest sequence, 131072 unless given.
// Tensors: embed, final.norm, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*.
#include <algorithm>

#include "config.h"

namespace tq {
namespace {

const double EXPERT_GATE_ALPHA = 1.702;         // the slope inside the experts' sigmoid: fixed by the design
const long long DEFAULT_MAX_POSITIONS = 131072;

const Json& object_at(const Json& parent, const char* key, const std::string& where) {
    const Json& j = parent[key];
    if (!j.is_object()) raise(TQE_ERR_CONFIG, "%s: '%s' must be an object", where.c_str(), key);
    return j;
}

Json mixer_typed(const Json& raw, const std::string& where, long long layer, const std::vector<Json>& before) {
    KeyReader r(raw, where);
    Json m = Json::object();
    m.set("heads", r.integer("heads", 1));
    m.set("dim", r.integer("dim", 1));
    m.set("rot_dim", r.integer("rot_dim", 0));
    m.set("vdim", r.integer("vdim", 1));
    m.set("q_rank", r.integer("q_rank", 1));
    m.set("kv_rank", r.integer("kv_rank", 1));
    m.set("scale", r.number("scale", true));
    const long long rot_dim = m["rot_dim"].as_int();
    if (rot_dim > 0) {
        KeyReader rot(object_at(raw, "rot", where), where + ".rot");
        const long long dims = rot.integer("dims", 0);
        if (dims % 2 || dims > rot_dim) raise(TQE_ERR_CONFIG, "%s.rot: dims %lld must be even and at most rot_dim %lld", where.c_str(), dims, rot_dim);
        m.set("rot_base", rot.number("base", true));
        m.set("rot_dims", dims);
    } else {
        m.set("rot_base", 1.0);
        m.set("rot_dims", 0);
    }
    if (raw["mask"].is_null()) m.set("window", Json());
    else m.set("window", KeyReader(object_at(raw, "mask", where), where + ".mask").integer("size", 1));
    if (r.has("kv_from")) {
        const long long from = r.integer("kv_from", 0);
        if (from >= layer) raise(TQE_ERR_CONFIG, "%s: kv_from %lld is not an earlier layer", where.c_str(), from);
        const Json& src = before[(size_t)from]["mixer"];
        if (!src["kv_from"].is_null()) raise(TQE_ERR_CONFIG, "%s: kv_from %lld names a layer that keeps no cache of its own", where.c_str(), from);
        for (const char* key : {"kv_rank", "rot_dim", "rot_dims"})
            if (src[key].as_int() != m[key].as_int())
                raise(TQE_ERR_CONFIG, "%s: %s differs from that of layer %lld, whose cache it reads", where.c_str(), key, from);
        if (src["rot_base"].as_number() != m["rot_base"].as_number())
            raise(TQE_ERR_CONFIG, "%s: rot.base differs from that of layer %lld, whose cache it reads", where.c_str(), from);
        m.set("kv_from", from);
    } else {
        m.set("kv_from", Json());
    }
    return m;
}

Json expert_typed(const Json& raw, const std::string& where) {
    KeyReader r(raw, where);
    Json e = Json::object();
    e.set("ff", r.integer("ff", 1));
    e.set("limit", r.number("limit", true));
    return e;
}

Json mlp_typed(const Json& raw, const std::string& where) {
    if (raw.is_null()) return Json();
    if (!raw.is_object()) raise(TQE_ERR_CONFIG, "%s must be an object or null", where.c_str());
    KeyReader r(raw, where);
    const std::string kind = r.string("kind");
    Json m = Json::object();
    m.set("kind", kind);
    if (kind == "dense") {
        m.set("ff", r.integer("ff", 1));
    } else if (kind == "moe") {
        KeyReader router(object_at(raw, "router", where), where + ".router");
        const long long experts = router.integer("experts", 1), top = router.integer("top", 1);
        if (top > experts) raise(TQE_ERR_CONFIG, "%s.router: top %lld of %lld experts", where.c_str(), top, experts);
        m.set("experts", experts);
        m.set("top", top);
        m.set("router_scale", router.number_or("scale", 1.0));
        m.set("expert", expert_typed(object_at(raw, "expert", where), where + ".expert"));
        m.set("shared", raw["shared"].is_null() ? Json() : expert_typed(object_at(raw, "shared", where), where + ".shared"));
    } else {
        raise(TQE_ERR_CONFIG, "%s: unknown kind '%s' (known: dense, moe)", where.c_str(), kind.c_str());
    }
    return m;
}

Json nikasun_typed(const Json& raw, const std::string& where) {
    KeyReader r(raw, where);
    Json c = Json::object();
    c.set("vocab", r.integer("vocab", 1));
    c.set("width", r.integer("width", 1));
    c.set("embedding_scale", KeyReader(object_at(raw, "embedding", where), where + ": embedding").number("scale"));
    c.set("norm_eps", KeyReader(object_at(raw, "norm", where), where + ": norm").number("eps"));
    c.set("max_positions", r.integer_or("max_positions", DEFAULT_MAX_POSITIONS, 1));
    if (!raw["layers"].is_array() || raw["layers"].items().empty()) raise(TQE_ERR_CONFIG, "%s: 'layers' must be a list of at least one layer", where.c_str());
    std::vector<Json> layers;
    for (const Json& l : raw["layers"].items()) {
        const long long i = (long long)layers.size();
        const std::string at = format("%s: layers[%lld]", where.c_str(), i);
        if (!l.is_object()) raise(TQE_ERR_CONFIG, "%s must be an object", at.c_str());
        KeyReader lr(l, at);
        const std::string type = lr.string("type");
        if (type != "latent_attention") raise(TQE_ERR_CONFIG, "%s: unknown type '%s' (known: latent_attention)", at.c_str(), type.c_str());
        Json t = Json::object();
        t.set("type", type);
        t.set("mixer", mixer_typed(object_at(l, "mixer", at), at + ".mixer", i, layers));
        t.set("mlp", mlp_typed(l["mlp"], at + ".mlp"));
        layers.push_back(t);
    }
    Json list = Json::array();
    for (const Json& l : layers) list.push(l);
    c.set("layers", list);
    return c;
}

PartSpec part(const char* kind, std::initializer_list<std::pair<const char*, Json>> params) {
    PartSpec p;
    p.kind = kind;
    for (const auto& kv : params) p.params.set(kv.first, kv.second);
    return p;
}

PartSpec expert_part(long long width, const Json& e) {
    Json names = Json::object();
    names.set("gate", "gate");
    names.set("up", "up");
    names.set("down", "down");
    return part("gated", {{"hidden", width}, {"inter", e["ff"]}, {"gate", "clamped"}, {"limit", e["limit"]}, {"alpha", EXPERT_GATE_ALPHA}, {"names", names}});
}

ModelSpec nikasun_spec(const Json& c) {
    const long long width = c["width"].as_int();
    const std::vector<Json>& layers = c["layers"].items();
    const PartSpec norm = part("rms_norm", {{"size", width}, {"eps", c["norm_eps"]}, {"unit_offset", true}, {"tensor", ""}});
    // what a layer's cache must keep: the largest window of the layers that read it (none: everything)
    std::vector<long long> keep(layers.size(), 0);
    std::vector<bool> keep_all(layers.size(), false);
    for (size_t l = 0; l < layers.size(); ++l) {
        const Json& m = layers[l]["mixer"];
        const size_t owner = m["kv_from"].is_null() ? l : (size_t)m["kv_from"].as_int();
        if (m["window"].is_null()) keep_all[owner] = true;
        else keep[owner] = std::max(keep[owner], (long long)m["window"].as_int());
    }
    // Caches of equal row size and window are one group of the cache, and the cache's bookkeeping takes TQE_MAX_GROUPS of
    // them.  A model with more different windows than that keeps, in caches of equal row size, the largest of their
    // windows (what a layer sees is its own window still).
    auto row_of = [&](size_t l) { return std::make_pair(layers[l]["mixer"]["kv_rank"].as_int(), layers[l]["mixer"]["rot_dim"].as_int()); };
    std::vector<std::vector<long long>> distinct;
    for (size_t l = 0; l < layers.size(); ++l) {
        if (!layers[l]["mixer"]["kv_from"].is_null()) continue;
        const std::vector<long long> key = {row_of(l).first, row_of(l).second, keep_all[l] ? -1 : keep[l]};
        if (std::find(distinct.begin(), distinct.end(), key) == distinct.end()) distinct.push_back(key);
    }
    if ((int)distinct.size() > TQE_MAX_GROUPS)
        for (size_t l = 0; l < layers.size(); ++l)
            for (size_t o = 0; o < layers.size(); ++o)
                if (layers[l]["mixer"]["kv_from"].is_null() && layers[o]["mixer"]["kv_from"].is_null() && row_of(l) == row_of(o)) {
                    keep[l] = std::max(keep[l], keep[o]);
                    if (keep_all[o]) keep_all[l] = true;
                }
    ModelSpec s;
    s.architecture = "Nikasun";
    s.vocab_size = c["vocab"].as_int();
    s.hidden_size = width;
    s.max_positions = c["max_positions"].as_int();
    s.embedding_name = "embed";
    s.has_embedding_scale = true;
    s.embedding_scale = c["embedding_scale"].as_number();
    for (size_t l = 0; l < layers.size(); ++l) {
        const Json& m = layers[l]["mixer"];
        const Json& mlp = layers[l]["mlp"];
        const size_t owner = m["kv_from"].is_null() ? l : (size_t)m["kv_from"].as_int();
        const PartSpec position = m["rot_dims"].as_int() > 0
            ? part("rotary", {{"theta", m["rot_base"]}, {"rot_dim", m["rot_dims"]}, {"max_positions", c["max_positions"]}, {"style", "halves"}})
            : part("none", {{"max_positions", c["max_positions"]}});
        const PartSpec mixer = part("latent_attention", {{"hidden", width}, {"n_heads", m["heads"]}, {"head_dim", m["dim"]}, {"rot_dim", m["rot_dim"]},
                                                         {"value_dim", m["vdim"]}, {"q_rank", m["q_rank"]}, {"kv_rank", m["kv_rank"]}, {"scale", m["scale"]},
                                                         {"eps", c["norm_eps"]}, {"window", m["window"]},
                                                         {"cache_window", keep_all[owner] ? Json() : Json(keep[owner])},
                                                         {"own_kv", m["kv_from"].is_null()}, {"gate", true}, {"position", position.to_json()}});
        Json names = Json::object();
        names.set("mixer", "mix.");
        names.set("feed_forward", "mlp.");
        names.set("mixer_norm", "norm1");
        names.set("ff_norm", "norm2");
        Json ff;
        if (!mlp.is_null()) {
            if (mlp["kind"].as_string() == "dense") {
                Json dense_names = Json::object();
                dense_names.set("gate", "gate");
                dense_names.set("up", "up");
                dense_names.set("down", "down");
                ff = part("gated", {{"hidden", width}, {"inter", mlp["ff"]}, {"gate", "relu"}, {"names", dense_names}}).to_json();
            } else {
                const Json& e = mlp["expert"];
                ff = part("routed_experts", {{"hidden", width}, {"inter", e["ff"]}, {"n_experts", mlp["experts"]}, {"top", mlp["top"]},
                                             {"router_scale", mlp["router_scale"]}, {"gate", "clamped"}, {"limit", e["limit"]},
                                             {"alpha", EXPERT_GATE_ALPHA},
                                             {"shared", mlp["shared"].is_null() ? Json() : expert_part(width, mlp["shared"]).to_json()}}).to_json();
            }
        }
        LayerSpec layer;
        layer.prefix = format("l%zu.", l);
        layer.block = part("pre_norm", {{"mixer", mixer.to_json()}, {"feed_forward", ff}, {"mixer_norm", norm.to_json()},
                                        {"ff_norm", mlp.is_null() ? Json() : norm.to_json()}, {"names", names}});
        s.layers.push_back(layer);
        Run run;
        run.layer = (int)l;
        run.cache_of = m["kv_from"].is_null() ? -1 : (int)m["kv_from"].as_int();
        s.order.push_back(run);
    }
    s.final_norm = norm;
    s.final_norm_prefix = "final.norm";
    s.head_name = "";
    return s;
}

}  // namespace

void register_nikasun() {
    Architecture a;
    a.name = "Nikasun";
    a.model_types = {"nikasun"};
    a.typed_config = nikasun_typed;
    a.build_spec = nikasun_spec;
    register_architecture(a);
}

}  // namespace tq
