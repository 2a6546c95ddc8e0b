// lm_host.hpp — the host program's side of the layered-model tier (zg_lm_* of include/zgpt2.h): reads a checkpoint folder
// (config.json + model.safetensors), builds the library's layer descriptors from the configuration, loads the tensors by name
// and generates from token ids.  `zgpt2_main lm <dir> <tok,tok,...[;tok,...]> <n_new> [--dtype float32] [--temp T] [--seed S]`.
// A small JSON reader is enough for both files (the safetensors header is JSON too); nothing of a checkpoint is executed.
#pragma once
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <fstream>
#include <map>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/zgpt2.h"

namespace lmhost {

struct Json {
    enum Kind { Null, Bool, Num, Str, Arr, Obj } kind = Null;
    double num = 0;
    bool b = false;
    std::string str;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;
    const Json* get(const std::string& k) const {
        for (auto& kv : obj)
            if (kv.first == k) return &kv.second;
        return nullptr;
    }
    const Json& at(const std::string& k) const {
        const Json* j = get(k);
        if (!j) throw std::runtime_error("config: key '" + k + "' is missing");
        return *j;
    }
    bool truthy() const { return !(kind == Null || (kind == Bool && !b)); }
};

class JsonReader {
  public:
    explicit JsonReader(const std::string& s) : s_(s) {}
    Json parse() {
        Json j = value();
        ws();
        if (p_ != s_.size()) fail("trailing characters");
        return j;
    }

  private:
    const std::string& s_;
    size_t p_ = 0;
    [[noreturn]] void fail(const char* what) { throw std::runtime_error(std::string("JSON: ") + what + " at byte " + std::to_string(p_)); }
    void ws() {
        while (p_ < s_.size() && (s_[p_] == ' ' || s_[p_] == '\n' || s_[p_] == '\t' || s_[p_] == '\r')) ++p_;
    }
    bool eat(char c) {
        ws();
        if (p_ < s_.size() && s_[p_] == c) {
            ++p_;
            return true;
        }
        return false;
    }
    std::string string() {
        if (!eat('"')) fail("string expected");
        std::string out;
        while (p_ < s_.size() && s_[p_] != '"') {
            char c = s_[p_++];
            if (c == '\\' && p_ < s_.size()) {
                c = s_[p_++];
                if (c == 'n') c = '\n';
                else if (c == 't') c = '\t';
                else if (c == 'u') {  // tensor names and keys are ASCII: keep the escape's low byte
                    if (p_ + 4 > s_.size()) fail("short \\u escape");
                    c = (char)strtol(s_.substr(p_, 4).c_str(), nullptr, 16);
                    p_ += 4;
                }
            }
            out.push_back(c);
        }
        if (p_ >= s_.size()) fail("unterminated string");
        ++p_;
        return out;
    }
    Json value() {
        ws();
        if (p_ >= s_.size()) fail("value expected");
        Json j;
        const char c = s_[p_];
        if (c == '{') {
            ++p_;
            j.kind = Json::Obj;
            if (eat('}')) return j;
            do {
                std::string k = string();
                if (!eat(':')) fail("':' expected");
                j.obj.emplace_back(k, value());
            } while (eat(','));
            if (!eat('}')) fail("'}' expected");
        } else if (c == '[') {
            ++p_;
            j.kind = Json::Arr;
            if (eat(']')) return j;
            do j.arr.push_back(value());
            while (eat(','));
            if (!eat(']')) fail("']' expected");
        } else if (c == '"') {
            j.kind = Json::Str;
            j.str = string();
        } else if (s_.compare(p_, 4, "null") == 0) {
            p_ += 4;
        } else if (s_.compare(p_, 4, "true") == 0) {
            p_ += 4;
            j.kind = Json::Bool;
            j.b = true;
        } else if (s_.compare(p_, 5, "false") == 0) {
            p_ += 5;
            j.kind = Json::Bool;
        } else {
            char* end = nullptr;
            j.kind = Json::Num;
            j.num = strtod(s_.c_str() + p_, &end);
            if (end == s_.c_str() + p_) fail("value expected");
            p_ = (size_t)(end - s_.c_str());
        }
        return j;
    }
};

inline std::string slurp(const std::string& path, size_t max_bytes = (size_t)-1) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("cannot open " + path);
    std::ostringstream ss;
    ss << f.rdbuf();
    std::string s = ss.str();
    if (s.size() > max_bytes) s.resize(max_bytes);
    return s;
}

// the JSON header of a safetensors file (name -> dtype, shape, data_offsets)
inline Json safetensors_header(const std::string& path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("cannot open " + path);
    uint64_t n = 0;
    f.read(reinterpret_cast<char*>(&n), 8);
    if (!f || n > (1u << 28)) throw std::runtime_error(path + ": no safetensors header");
    std::string head((size_t)n, ' ');
    f.read(&head[0], (std::streamsize)n);
    if (!f) throw std::runtime_error(path + ": header length exceeds the file");
    return JsonReader(head).parse();
}

// config.json of a layered design -> layer descriptors (the keys zig_gpt2_amd/lm.py reads).  tensors: the checkpoint's
// safetensors header, for the sizes that only a tensor's shape gives (may be null when the configuration lists them).
// derived (may be null): tensors of the library that the configuration fills instead of the checkpoint (constants per head).
typedef std::vector<std::pair<std::string, std::vector<float>>> DerivedTensors;
inline void build_config(const Json& cfg, const Json* tensors, std::vector<zg_lm_layer>& layers, zg_lm_config& out, DerivedTensors* derived = nullptr) {
    const Json* arch = cfg.get("architecture");
    const std::string design = arch ? arch->str : std::string("?");
    if (design != "Tokosun" && design != "Gupizen" && design != "Sanazen" && design != "Vovalorn")
        throw std::runtime_error("config: architecture '" + design + "' is not served");
    const bool gup = design == "Gupizen", san = design == "Sanazen", vov = design == "Vovalorn";
    memset(&out, 0, sizeof(out));
    if (vov) {  // what the name fixes: norms without statistics, one of them behind the embedding
        out.flags |= ZG_LM_TANH_NORMS | ZG_LM_EMBED_NORM;
        out.residual_mult = 1.0f;
        if (const Json* v = cfg.get("residual_mult")) out.residual_mult = (float)v->num;
    }
    if (san) {  // what the name fixes: side-by-side sublayers with plain norms, sinusoid positions
        out.flags |= ZG_LM_SIDE_BY_SIDE | ZG_LM_SINUSOID_POSITIONS;
        out.embed_scale = 1.0f;
        if (const Json* e = cfg.get("embedding"))
            if (e->truthy())
                if (const Json* v = e->get("scale")) out.embed_scale = (float)v->num;
        if (const Json* v = cfg.get("logit_scale"))
            if (v->truthy()) out.logit_scale = (float)v->num;
        if (const Json* v = cfg.get("logit_softcap"))
            if (v->truthy()) out.logit_softcap = (float)v->num;
    }
    if (gup) {  // what the name fixes: tied head, the embedding output added again per repetition of the loop
        out.flags |= ZG_LM_TIED_HEAD | ZG_LM_LOOP_READD;
        out.embed_scale = 1.0f;
        if (const Json* e = cfg.get("embedding"))
            if (e->truthy())
                if (const Json* v = e->get("scale")) out.embed_scale = (float)v->num;
        if (const Json* c = cfg.get("canon"))
            if (c->truthy())
                if (const Json* v = c->get("taps")) out.canon_taps = (int)v->num;
    }
    size_t layer_index = 0;
    out.vocab = (size_t)cfg.at("vocab").num;
    out.width = (size_t)cfg.at("width").num;
    out.norm_eps = (float)cfg.at("norm").at("eps").num;
    out.loop_times = 1;
    if (const Json* loop = cfg.get("loop"))
        if (loop->truthy()) {
            out.loop_start = (int)loop->at("start").num;
            out.loop_stop = (int)loop->at("stop").num;
            out.loop_times = (int)loop->at("times").num;
        }
    const std::vector<Json>& entries = cfg.at("layers").arr;
    auto owner = [&](size_t i) {  // the layer whose tensors layer i runs
        for (size_t hops = 0; hops <= entries.size(); ++hops) {
            const Json* w = entries.at(i).get("weights_of");
            if (!w || w->kind != Json::Num) return i;
            if (w->num < 0 || (size_t)w->num >= entries.size()) break;
            i = (size_t)w->num;
        }
        throw std::runtime_error("config: a layer's weights_of names no layer with tensors");
    };
    for (const Json& e : entries) {
        zg_lm_layer d;
        memset(&d, 0, sizeof(d));
        const std::string& type = e.at("type").str;
        const Json& m = e.at("mixer");
        const size_t own = owner(layer_index);
        if (own != layer_index) d.weights_of = (int)own + 1;
        ++layer_index;
        const std::string prefix = "l" + std::to_string(own) + ".";
        const Json& sizes = ((gup || san) && type == "parallel") ? m.at("left") : m;
        d.heads = (int)sizes.at("heads").num;
        d.dim = (int)sizes.at("dim").num;
        d.vdim = sizes.get("vdim") ? (int)sizes.at("vdim").num : d.dim;
        if (gup) {
            d.ff_act = ZG_LM_ACT_GELU;
            d.router = ZG_LM_ROUTE_TOP_LOGITS;
            d.kv_heads = sizes.get("kv_heads") ? (int)sizes.at("kv_heads").num : d.heads;
        }
        if (san && type == "parallel") {
            d.mixer = ZG_LM_MIX_WINDOW_LINEAR;
            d.ff_act = ZG_LM_ACT_GLU_CLIPPED;
            d.router = ZG_LM_ROUTE_SIGMOID_INPUT;
            d.kv_heads = sizes.get("kv_heads") ? (int)sizes.at("kv_heads").num : d.heads;
            d.scale = (float)sizes.at("scale").num;
            if (const Json* mask = sizes.get("mask"))
                if (mask->truthy()) {
                    if (const Json* v = mask->get("size")) d.window = (int)v->num;
                    if (const Json* v = mask->get("keep_first")) d.keep_first = (int)v->num;
                }
            if (const Json* v = sizes.get("conv")) {
                d.conv = (int)v->num;
            } else if (const Json* t = tensors ? tensors->get(prefix + "mix.left.q.conv") : nullptr) {  // the taps from the checkpoint
                d.conv = (int)t->at("shape").arr.at(1).num;
            }
            d.left_scale = m.get("left_scale") ? (float)m.at("left_scale").num : 1.0f;
            d.right_scale = m.get("right_scale") ? (float)m.at("right_scale").num : 1.0f;
            const Json& r = m.at("right");
            d.lin_heads = (int)r.at("heads").num;
            d.lin_dim = (int)r.at("dim").num;
            d.lin_vdim = (int)r.at("vdim").num;
            std::vector<float> decay;
            for (const Json& v : r.at("decay").arr) decay.push_back((float)v.num);
            if ((int)decay.size() != d.lin_heads) throw std::runtime_error("config: " + prefix + "mix.right lists " + std::to_string(decay.size()) + " decays");
            if (derived) derived->push_back({prefix + "mix.right.decay", decay});
        } else if (san) {
            throw std::runtime_error("config: unknown mixer type '" + type + "'");
        } else if (gup && type == "parallel") {
            d.mixer = ZG_LM_MIX_PARALLEL;
            d.scale = (float)sizes.at("scale").num;
            if (const Json* mask = sizes.get("mask"))
                if (mask->truthy())
                    if (const Json* v = mask->get("size")) d.window = (int)v->num;
            d.rot_base = 10000.0f;
            if (const Json* rot = sizes.get("rot"))
                if (rot->truthy()) {
                    if (const Json* v = rot->get("dims")) d.rot_dims = (int)v->num;
                    if (const Json* v = rot->get("base")) d.rot_base = (float)v->num;
                    const Json* sc = rot->get("scaling");
                    if (sc && sc->truthy()) {  // wavelength bands: `high` / `low` travel in the fields of the blend's `fast` / `slow`
                        d.rot_scaled = ZG_LM_ROT_BANDS;
                        d.rot_factor = (float)sc->at("factor").num;
                        d.rot_original = (float)sc->at("original").num;
                        d.rot_fast = (float)sc->at("high").num;
                        d.rot_slow = (float)sc->at("low").num;
                    }
                }
            const Json& r = m.at("right");
            d.lru_width = (int)r.at("width").num;
            d.lru_blocks = (int)r.at("blocks").num;
            d.lru_conv = (int)r.at("conv").num;
        } else if (gup && type == "channel_delta") {
            d.mixer = ZG_LM_MIX_CHANNEL_DELTA;
            d.conv = (int)m.at("conv").num;
            auto inner = [&](const char* key, const char* tensor) -> int {
                if (const Json* v = m.get(key)) return (int)v->num;
                const Json* t = tensors ? tensors->get(prefix + tensor) : nullptr;
                if (!t) throw std::runtime_error("config: the inner size '" + std::string(key) + "' needs the shape of tensor " + prefix + tensor);
                return (int)t->at("shape").arr.at(0).num;
            };
            d.decay_rank = inner("decay_rank", "mix.a1");
            d.gate_rank = inner("gate_rank", "mix.g1");
        } else if (gup) {
            throw std::runtime_error("config: unknown mixer type '" + type + "'");
        } else if (vov && type == "gla") {
            d.mixer = ZG_LM_MIX_GLA;
            d.ff_act = ZG_LM_ACT_GLU_SILU;
            d.router = ZG_LM_ROUTE_SIGMOID_GROUPS;
            d.tau = (float)m.at("tau").num;
            if (const Json* v = m.get("decay_rank")) {
                d.decay_rank = (int)v->num;
            } else {
                const Json* t = tensors ? tensors->get(prefix + "mix.a1") : nullptr;
                if (!t) throw std::runtime_error("config: the inner size 'decay_rank' needs the shape of tensor " + prefix + "mix.a1");
                d.decay_rank = (int)t->at("shape").arr.at(0).num;
            }
        } else if (vov && type == "attention") {
            d.mixer = ZG_LM_MIX_ATTENTION;
            d.ff_act = ZG_LM_ACT_GLU_SILU;
            d.router = ZG_LM_ROUTE_SIGMOID_GROUPS;
            d.kv_heads = m.get("kv_heads") ? (int)m.at("kv_heads").num : d.heads;
            d.scale = (float)m.at("scale").num;
            if (const Json* v = m.get("softcap"))
                if (v->truthy()) d.softcap = (float)v->num;
            if (const Json* qt = m.get("q_temp"))
                if (qt->truthy()) {
                    d.qtemp_coef = (float)qt->at("coef").num;
                    d.qtemp_every = (int)qt->at("every").num;
                }
            d.dist_bias = 1;
            if (const Json* v = m.get("dist_bias")) d.dist_bias = v->truthy() ? 1 : 0;
        } else if (vov) {
            throw std::runtime_error("config: unknown mixer type '" + type + "'");
        } else if (type == "hgrn2") {
            d.mixer = ZG_LM_MIX_HGRN2;
        } else if (type == "latent_attention") {
            d.mixer = ZG_LM_MIX_LATENT_ATTENTION;
            d.rot_dim = (int)m.at("rot_dim").num;
            d.kv_rank = (int)m.at("kv_rank").num;
            d.q_rank = (int)m.at("q_rank").num;
            d.scale = (float)m.at("scale").num;
            d.rot_dims = d.rot_dim;
            d.rot_base = 10000.0f;
            if (const Json* rot = m.get("rot"))
                if (rot->truthy()) {
                    if (const Json* v = rot->get("dims")) d.rot_dims = (int)v->num;
                    if (const Json* v = rot->get("base")) d.rot_base = (float)v->num;
                    const Json* sc = rot->get("scaling");
                    if (sc && sc->truthy()) {
                        d.rot_scaled = 1;
                        d.rot_factor = (float)sc->at("factor").num;
                        d.rot_original = (float)sc->at("original").num;
                        d.rot_fast = (float)sc->at("fast").num;
                        d.rot_slow = (float)sc->at("slow").num;
                    }
                }
        } else {
            throw std::runtime_error("config: unknown mixer type '" + type + "'");
        }
        const Json* mlp = e.get("mlp");
        if (mlp && mlp->truthy()) {
            const std::string& kind = mlp->at("kind").str;
            if (kind == "dense") {
                d.ff = ZG_LM_FF_DENSE;
                d.ff_width = (int)mlp->at("ff").num;
            } else if (kind == "moe") {
                d.ff = ZG_LM_FF_MOE;
                d.ff_width = (int)mlp->at("expert").at("ff").num;
                d.experts = (int)mlp->at("router").at("experts").num;
                d.top = (int)mlp->at("router").at("top").num;
                if (san) {
                    d.ff_limit = (float)mlp->at("expert").at("limit").num;
                    const Json* sh = mlp->get("shared");
                    if (sh && sh->truthy()) {
                        d.shared_width = (int)sh->at("ff").num;
                        d.shared_limit = (float)sh->at("limit").num;
                    }
                }
                if (vov) {
                    const Json& r = mlp->at("router");
                    d.route_groups = d.route_keep = 1;
                    d.route_scale = r.get("scale") ? (float)r.at("scale").num : 1.0f;
                    if (const Json* gr = r.get("groups"))
                        if (gr->truthy()) {
                            d.route_groups = gr->get("count") ? (int)gr->at("count").num : 1;
                            d.route_keep = gr->get("keep") ? (int)gr->at("keep").num : d.route_groups;
                        }
                    const Json* sh = mlp->get("shared");
                    if (sh && sh->truthy()) d.shared_width = (int)sh->at("ff").num;
                }
            } else {
                throw std::runtime_error("config: unknown feed-forward kind '" + kind + "'");
            }
        }
        layers.push_back(d);
    }
    out.n_layers = layers.size();
    out.layers = layers.data();
}

// every tensor of a safetensors file -> zg_lm_load_tensor (BF16 / F32 / F16 values widened or kept as fp32; integer tables skipped)
inline void load_safetensors(zg_lm* g, const std::string& path) {
    const std::string file = slurp(path);
    if (file.size() < 8) throw std::runtime_error(path + ": too short");
    uint64_t n = 0;
    memcpy(&n, file.data(), 8);
    if (n > file.size() - 8) throw std::runtime_error(path + ": header length exceeds the file");
    const std::string head = file.substr(8, (size_t)n);
    const Json meta = JsonReader(head).parse();
    const char* data = file.data() + 8 + n;
    const size_t data_bytes = file.size() - 8 - (size_t)n;
    std::vector<float> buf;
    for (auto& kv : meta.obj) {
        if (kv.first == "__metadata__") continue;
        const std::string& dt = kv.second.at("dtype").str;
        const size_t lo = (size_t)kv.second.at("data_offsets").arr.at(0).num, hi = (size_t)kv.second.at("data_offsets").arr.at(1).num;
        size_t count = 1;
        for (const Json& d : kv.second.at("shape").arr) count *= (size_t)d.num;
        const size_t width = dt == "BF16" || dt == "F16" ? 2 : dt == "F32" ? 4 : 0;
        if (width == 0) continue;  // integer tables: nothing of this design reads them
        if (hi > data_bytes || hi - lo != count * width) throw std::runtime_error(path + ": tensor " + kv.first + " does not fit its shape");
        buf.resize(count);
        if (dt == "F32") {
            memcpy(buf.data(), data + lo, count * 4);
        } else if (dt == "BF16") {
            for (size_t i = 0; i < count; ++i) {
                uint16_t h;
                memcpy(&h, data + lo + 2 * i, 2);
                const uint32_t w = (uint32_t)h << 16;
                memcpy(&buf[i], &w, 4);
            }
        } else {
            for (size_t i = 0; i < count; ++i) {
                uint16_t h;
                memcpy(&h, data + lo + 2 * i, 2);
                const uint32_t s = (h >> 15) & 1u, e = (h >> 10) & 31u, f = h & 1023u;
                float v;
                if (e == 0) v = (float)f * 5.9604644775390625e-08f;
                else if (e == 31) v = f ? NAN : INFINITY;
                else {
                    const uint32_t w = ((e + 112u) << 23) | (f << 13);
                    memcpy(&v, &w, 4);
                }
                buf[i] = s ? -v : v;
            }
        }
        const int st = zg_lm_load_tensor(g, kv.first.c_str(), buf.data(), count);
        if (st == ZG_ERR_ARG && strstr(zg_last_error(), "has no tensor")) continue;  // not a tensor of this configuration: left alone
        if (st != ZG_OK) throw std::runtime_error(std::string("load: ") + zg_last_error());
    }
    size_t missing = 0;
    char names[512];
    zg_lm_missing_tensors(g, &missing, names, sizeof(names));
    if (missing) throw std::runtime_error(std::to_string(missing) + " tensors missing from the checkpoint: " + names);
}

inline int lm_main(int argc, char** argv) {
    if (argc < 5) {
        fprintf(stderr, "usage: %s lm <checkpoint dir> <tok,tok,...[;tok,...]> <n_new> [--dtype bfloat16|float32] [--temp T] [--seed S]\n", argv[0]);
        return 2;
    }
    try {
        const std::string dir = argv[2];
        std::vector<std::vector<int32_t>> prompts(1);
        for (const char* p = argv[3]; *p;) {
            if (*p == ';') {
                prompts.emplace_back();
                ++p;
            } else if (*p == ',') {
                ++p;
            } else {
                char* end = nullptr;
                const long v = strtol(p, &end, 10);
                if (end == p || v < 0) throw std::runtime_error(std::string("token list: '") + p + "'");
                prompts.back().push_back((int32_t)v);
                p = end;
            }
        }
        for (auto& pr : prompts)
            if (pr.empty()) throw std::runtime_error("empty prompt");
        const size_t n_new = strtoull(argv[4], nullptr, 10);
        float temp = 0.0f;
        uint64_t seed = 0;
        unsigned flags = 0;
        for (int i = 5; i < argc; ++i) {
            const std::string o = argv[i];
            if (o == "--temp" && i + 1 < argc) temp = (float)atof(argv[++i]);
            else if (o == "--seed" && i + 1 < argc) seed = strtoull(argv[++i], nullptr, 10);
            else if (o == "--dtype" && i + 1 < argc) {
                const std::string d = argv[++i];
                if (d == "float32") flags |= ZG_LM_F32;
                else if (d != "bfloat16") throw std::runtime_error("--dtype " + d + ": bfloat16 or float32");
            } else throw std::runtime_error("unknown or incomplete option '" + o + "'");
        }
        std::vector<zg_lm_layer> layers;
        zg_lm_config cfg;
        const Json tensors = safetensors_header(dir + "/model.safetensors");
        DerivedTensors derived;
        build_config(JsonReader(slurp(dir + "/config.json")).parse(), &tensors, layers, cfg, &derived);
        size_t longest = 0, stride = 0;
        for (auto& pr : prompts) longest = std::max(longest, pr.size() + n_new), stride = std::max(stride, pr.size());
        cfg.max_seqs = prompts.size();
        cfg.max_tokens = prompts.size() * (longest + 64);
        cfg.flags |= flags;
        zg_lm* g = nullptr;
        if (zg_lm_create(&g, &cfg, 0) != ZG_OK) throw std::runtime_error(std::string("create: ") + zg_last_error());
        for (auto& kv : derived)
            if (zg_lm_load_tensor(g, kv.first.c_str(), kv.second.data(), kv.second.size()) != ZG_OK)
                throw std::runtime_error(std::string("load: ") + zg_last_error());
        load_safetensors(g, dir + "/model.safetensors");
        std::vector<int32_t> mat(prompts.size() * stride, 0), out(prompts.size() * n_new);
        std::vector<size_t> lens(prompts.size());
        for (size_t b = 0; b < prompts.size(); ++b) {
            lens[b] = prompts[b].size();
            memcpy(&mat[b * stride], prompts[b].data(), lens[b] * sizeof(int32_t));
        }
        if (zg_lm_generate(g, mat.data(), stride, lens.data(), prompts.size(), n_new, temp, seed, out.data(), out.size()) != ZG_OK)
            throw std::runtime_error(std::string("generate: ") + zg_last_error());
        for (size_t b = 0; b < prompts.size(); ++b) {
            for (size_t i = 0; i < n_new; ++i) printf("%s%d", i ? " " : "", out[b * n_new + i]);
            printf("\n");
        }
        zg_lm_destroy(g);
        return 0;
    } catch (const std::exception& e) {
        fprintf(stderr, "zgpt2_main lm: %s\n", e.what());
        return 1;
    }
}

}  // namespace lmhost
