// BackendConfig: which graph rewrites run and which ops a backend takes, read from a JSON
// document with an optional `base` it patches (configs/backend_config.h:9-24,
// configs/json_repository.cc:7-21 of the chainer-compiler tree).  The `hip` backend is
// {"base": "chxvm"}, the way `nvrtc` is in the reference.
#pragma once

#include <memory>
#include <set>
#include <string>

namespace chainer_compiler {

class BackendConfig {
public:
    static std::unique_ptr<BackendConfig> FromName(const std::string& name);
    static std::unique_ptr<BackendConfig> FromJSON(const std::string& json_str);

    virtual ~BackendConfig() = default;

    virtual const std::string& name() const = 0;

    virtual const std::set<std::string>& GetSimplifyPreproc() const = 0;
    virtual const std::set<std::string>& GetSimplify() const = 0;
    virtual bool HasOp(const std::string& name) const = 0;
    virtual const std::set<std::string>& GetMerge() const = 0;
    virtual const std::set<std::string>& GetExpandingFunctions() const = 0;
};

// The text of a built-in configuration; CHECK-fails on an unknown name.
const char* BuiltinConfigText(const std::string& name);

}  // namespace chainer_compiler
