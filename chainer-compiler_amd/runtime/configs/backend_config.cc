#include "backend_config.h"

#include <iostream>

#include "../log.h"
#include "json.h"

namespace chainer_compiler {

namespace {

struct BuiltinConfig {
    const char* name;
    const char* text;
};

const BuiltinConfig kBuiltinConfigs[] = {
#include "../gen/config_jsons.inc"
};

Json LoadJSONFromString(const std::string& json_str);

Json LoadJSONFromName(const std::string& name) {
    return LoadJSONFromString(BuiltinConfigText(name));
}

Json LoadJSONFromString(const std::string& json_str) {
    Json j = Json::Parse(json_str);
    CHECK(j.is_object()) << json_str;
    if (const Json* base_name = j.find("base")) {
        CHECK(base_name->is_string()) << "`base` must be a string: " << json_str;
        Json base = LoadJSONFromName(base_name->string());
        base.merge_patch(j);
        j = base;
        j.erase("base");
    }
    return j;
}

class BackendConfigImpl : public BackendConfig {
public:
    BackendConfigImpl(const std::string& name, const Json& config) : name_(name) {
        CHECK(config.is_object()) << config.dump();
        for (const auto& el : config.items()) {
            if (el.first == "simplify_preproc") {
                ReadFlags("simplify", el.second, &simplify_preproc_);
            } else if (el.first == "simplify") {
                ReadFlags("simplify", el.second, &simplify_);
            } else if (el.first == "supported_ops") {
                ReadFlags("supported ops", el.second, &supported_ops_);
                has_supported_ops_ = true;
            } else if (el.first == "merge") {
                ReadFlags("merge", el.second, &merge_);
            } else if (el.first == "expanding_functions") {
                ReadFlags("expanding functions", el.second, &expanding_functions_);
            } else {
                std::cerr << "WARNING: Unknown backend config: " << el.first << std::endl;
            }
        }
        // every pre-processing rewrite also runs in the main simplification
        simplify_.insert(simplify_preproc_.begin(), simplify_preproc_.end());
    }

    const std::string& name() const override {
        return name_;
    }
    const std::set<std::string>& GetSimplifyPreproc() const override {
        return simplify_preproc_;
    }
    const std::set<std::string>& GetSimplify() const override {
        return simplify_;
    }
    const std::set<std::string>& GetMerge() const override {
        return merge_;
    }
    const std::set<std::string>& GetExpandingFunctions() const override {
        return expanding_functions_;
    }
    bool HasOp(const std::string& op) const override {
        return !has_supported_ops_ || supported_ops_.count(op) > 0;
    }

private:
    static void ReadFlags(const std::string& what, const Json& flags, std::set<std::string>* names) {
        CHECK(flags.is_object()) << what << " must be an object: " << flags.dump();
        for (const auto& el : flags.items()) {
            CHECK(el.second.is_boolean()) << what << " values must be bool: " << flags.dump();
            if (el.second.boolean()) names->insert(el.first);
        }
    }

    std::string name_;
    std::set<std::string> simplify_preproc_;
    std::set<std::string> simplify_;
    bool has_supported_ops_ = false;
    std::set<std::string> supported_ops_;
    std::set<std::string> merge_;
    std::set<std::string> expanding_functions_;
};

}  // namespace

const char* BuiltinConfigText(const std::string& name) {
    for (const BuiltinConfig& c : kBuiltinConfigs)
        if (name == c.name) return c.text;
    CHECK(false) << "Unknown backend config name: " << name;
    return nullptr;
}

std::unique_ptr<BackendConfig> BackendConfig::FromName(const std::string& name) {
    return std::make_unique<BackendConfigImpl>(name, LoadJSONFromName(name));
}

std::unique_ptr<BackendConfig> BackendConfig::FromJSON(const std::string& json_str) {
    return std::make_unique<BackendConfigImpl>("custom", LoadJSONFromString(json_str));
}

}  // namespace chainer_compiler
