#include "executor/model.h"

#include <cstdio>
#include <cstring>
#include <memory>
#include <sstream>

#include "util/common.h"
#include "util/json.h"

namespace reef {
namespace executor {

using util::JsonValue;

Model* Model::from_json_text(const std::string& text, std::string* err) {
    std::string perr;
    std::unique_ptr<JsonValue> root = util::parse_json(text, &perr);
    auto bad = [&](const std::string& m) -> Model* {
        if (err) *err = m;
        return nullptr;
    };
    if (!root) return bad("json: " + perr);
    const JsonValue* st = root->get("storage");
    const JsonValue* ks = root->get("kernels");
    if (!st || st->type != JsonValue::List || !ks || ks->type != JsonValue::List)
        return bad("model json needs 'storage' and 'kernels' lists");

    std::unique_ptr<Model> m(new Model);
    for (const auto& s : st->lval) {
        const JsonValue *n = s->get("name"), *sz = s->get("size"), *ty = s->get("stype");
        if (!n || !sz || !ty) return bad("storage entry needs name/size/stype");
        m->storage.push_back(StorageInfo{n->sval, (size_t)sz->as_int(), ty->sval});
    }
    for (const auto& k : ks->lval) {
        const JsonValue *n = k->get("name"), *lp = k->get("launch_params"), *ar = k->get("args");
        if (!n || !lp || !ar) return bad("kernel entry needs name/launch_params/args");
        if (lp->lval.size() != 6) return bad("launch_params must have 6 entries: " + n->sval);
        KernelInfo ki;
        ki.name = n->sval;
        for (int i = 0; i < 6; ++i) ki.launch_params[i] = (uint32_t)lp->lval[i]->as_int();
        for (const auto& a : ar->lval) {
            const int64_t idx = a->as_int();
            if (idx < 0 || (size_t)idx >= m->storage.size())
                return bad("kernel arg out of range in " + n->sval);
            ki.args.push_back((size_t)idx);
        }
        if (const JsonValue* at = k->get("attrs"))
            for (const auto& a : at->lval) ki.attrs.push_back((int32_t)a->as_int());
        if (const JsonValue* ao = k->get("arg_offsets")) {
            if (ao->lval.size() != ki.args.size())
                return bad("arg_offsets must have one entry per arg in " + n->sval);
            for (size_t j = 0; j < ao->lval.size(); ++j) {
                const int64_t off = ao->lval[j]->as_int();
                const StorageInfo& st = m->storage[ki.args[j]];
                const size_t bytes = st.size * get_stype_size(st.stype);
                if (off < 0 || off % 16 != 0 || (off != 0 && (size_t)off >= bytes))
                    return bad("arg offset outside its storage or not a multiple of 16 in " + n->sval);
                ki.arg_offsets.push_back((size_t)off);
            }
        }
        m->kernels.push_back(std::move(ki));
    }
    if (const JsonValue* ga = root->get("args"))
        for (const auto& a : ga->lval) m->args.push_back((uint32_t)a->as_int());
    if (const JsonValue* sm = root->get("shared_memory"))
        for (const auto& kv : sm->mval) m->shared_memory[kv.first] = (size_t)kv.second->as_int();
    return m.release();
}

static bool read_file(const char* path, std::string& out) {
    FILE* fp = std::fopen(path, "rb");
    if (!fp) return false;
    std::fseek(fp, 0, SEEK_END);
    long n = std::ftell(fp);
    std::fseek(fp, 0, SEEK_SET);
    out.resize(n > 0 ? (size_t)n : 0);
    size_t got = n > 0 ? std::fread(&out[0], 1, (size_t)n, fp) : 0;
    std::fclose(fp);
    return got == out.size();
}

Model* Model::from_json(const char* json_file) {
    std::string text, err;
    if (!read_file(json_file, text)) {
        REEF_LOG_ERROR("cannot read %s", json_file);
        return nullptr;
    }
    Model* m = from_json_text(text, &err);
    if (!m) REEF_LOG_ERROR("%s: %s", json_file, err.c_str());
    return m;
}

size_t Model::get_stype_size(const std::string& stype) {
    if (stype == "float32") return 4;
    if (stype == "int64") return 8;
    if (stype == "byte") return 1;
    if (stype == "uint1") return 1;
    if (stype == "int32") return 4;
    REEF_LOG_ERROR("stype %s is undefined", stype.c_str());
    return 0;
}

ModelProfile* ModelProfile::from_json_text(const std::string& text, std::string* err) {
    std::string perr;
    std::unique_ptr<JsonValue> root = util::parse_json(text, &perr);
    if (!root) {
        if (err) *err = "json: " + perr;
        return nullptr;
    }
    const JsonValue* ml = root->get("model_latency");
    const JsonValue* kl = root->get("kernel_latency");
    if (!ml || !kl || kl->type != JsonValue::Dict) {
        if (err) *err = "profile json needs model_latency and kernel_latency";
        return nullptr;
    }
    std::unique_ptr<ModelProfile> p(new ModelProfile);
    p->model_latency = (int)ml->as_int();
    for (const auto& kv : kl->mval) {
        KernelProfile kp;
        if (const JsonValue* t = kv.second->get("total_latency")) kp.total_latency = (int)t->as_int();
        if (const JsonValue* l = kv.second->get("latency"))
            for (const auto& v : l->lval) kp.latency.push_back((int)v->as_int());
        const JsonValue* tn = kv.second->get("total_latency_ns");
        const JsonValue* ln = kv.second->get("latency_ns");
        if (tn && ln && ln->lval.size() == kp.latency.size()) {
            kp.has_ns = true;
            kp.total_latency_ns = (int)tn->as_int();
            for (const auto& v : ln->lval) kp.latency_ns.push_back((int)v->as_int());
        } else {
            kp.total_latency_ns = kp.total_latency * 1000;
            for (int v : kp.latency) kp.latency_ns.push_back(v * 1000);
        }
        p->kernel_latency.emplace(kv.first, std::move(kp));
    }
    return p.release();
}

ModelProfile* ModelProfile::from_json(const char* json_file) {
    std::string text, err;
    if (!read_file(json_file, text)) {
        REEF_LOG_ERROR("cannot read %s", json_file);
        return nullptr;
    }
    ModelProfile* p = from_json_text(text, &err);
    if (!p) REEF_LOG_ERROR("%s: %s", json_file, err.c_str());
    return p;
}

std::string ModelProfile::to_json() const {
    std::ostringstream ss;
    ss << "{\"model_latency\":" << model_latency << ",\"kernel_latency\":{";
    bool first = true;
    for (const auto& kv : kernel_latency) {
        if (!first) ss << ",";
        first = false;
        ss << "\"" << kv.first << "\":{\"total_latency\":" << kv.second.total_latency
           << ", \"latency\":[";
        for (size_t j = 0; j < kv.second.latency.size(); ++j) {
            if (j) ss << ",";
            ss << kv.second.latency[j];
        }
        ss << "]";
        if (kv.second.has_ns) {
            ss << ", \"total_latency_ns\":" << kv.second.total_latency_ns << ", \"latency_ns\":[";
            for (size_t j = 0; j < kv.second.latency_ns.size(); ++j) {
                if (j) ss << ",";
                ss << kv.second.latency_ns[j];
            }
            ss << "]";
        }
        ss << "}";
    }
    ss << "}}";
    return ss.str();
}

static const char kParamMagic[] = "TVM_MODEL_PARAMS";  // 17 bytes with the NUL

ModelParam* ModelParamParser::parse_from_file(const char* param_file) {
    FILE* fp = std::fopen(param_file, "rb");
    if (!fp) {
        REEF_LOG_ERROR("cannot open %s", param_file);
        return nullptr;
    }
    std::unique_ptr<ModelParam> params(new ModelParam);
    auto fail = [&](const char* why) -> ModelParam* {
        REEF_LOG_ERROR("%s: %s", param_file, why);
        std::fclose(fp);
        return nullptr;
    };
    char magic[sizeof(kParamMagic)];
    if (std::fread(magic, 1, sizeof(magic), fp) != sizeof(magic) ||
        std::memcmp(magic, kParamMagic, sizeof(magic)) != 0)
        return fail("bad magic");
    uint64_t n = 0;
    if (std::fread(&n, sizeof(n), 1, fp) != 1 || n == 0) return fail("bad tensor count");
    for (uint64_t i = 0; i < n; ++i) {
        std::string key;
        for (;;) {
            int c = std::fgetc(fp);
            if (c == EOF) return fail("truncated key");
            if (c == 0) break;
            key.push_back((char)c);
            if (key.size() > 255) return fail("key longer than 255 bytes");
        }
        uint64_t len = 0;
        if (std::fread(&len, sizeof(len), 1, fp) != 1 || len == 0) return fail("bad tensor length");
        std::vector<float> data(len);
        if (std::fread(data.data(), sizeof(float), len, fp) != len) return fail("truncated tensor");
        (*params)[key] = std::move(data);
    }
    std::fclose(fp);
    return params.release();
}

bool ModelParamParser::write_to_file(
    const char* param_file, const std::vector<std::pair<std::string, std::vector<float>>>& params) {
    FILE* fp = std::fopen(param_file, "wb");
    if (!fp) return false;
    std::fwrite(kParamMagic, 1, sizeof(kParamMagic), fp);
    uint64_t n = params.size();
    std::fwrite(&n, sizeof(n), 1, fp);
    for (const auto& kv : params) {
        std::fwrite(kv.first.c_str(), 1, kv.first.size() + 1, fp);
        uint64_t len = kv.second.size();
        std::fwrite(&len, sizeof(len), 1, fp);
        std::fwrite(kv.second.data(), sizeof(float), len, fp);
    }
    return std::fclose(fp) == 0;
}

}  // namespace executor
}  // namespace reef
