#include "compiler_capi.h"

#include <cstdlib>
#include <cstring>
#include <string>

#include "../runtime/configs/json.h"
#include "../runtime/log.h"
#include "emitter.h"
#include "fusion.h"
#include "graph.h"
#include "quantize.h"

namespace chainer_compiler {
namespace runtime {
void SetLastError(const std::string& message);  // chxvm_capi.cc
}
}  // namespace chainer_compiler

using namespace chainer_compiler;

namespace {

template <class Fn>
int32_t Guard(Fn fn) {
    try {
        fn();
        return 0;
    } catch (const std::exception& e) {
        runtime::SetLastError(e.what());
        return 1;
    }
}

QuantizationParams ParamsFrom(const Json& j, const std::string& where) {
    QuantizationParams p;
    CHECK(j.is_object()) << where << " must be an object";
    if (const Json* s = j.find("scale")) p.scale = static_cast<float>(s->number());
    if (const Json* z = j.find("zero_point")) p.zero_point = static_cast<int64_t>(z->number());
    if (const Json* d = j.find("dtype")) {
        CHECK(d->is_string() && (d->string() == "uint8" || d->string() == "int8")) << where << ": dtype is 'uint8' or 'int8'";
        p.zero_point_dtype = d->string() == "int8" ? kInt8 : kUInt8;
    }
    return p;
}

struct Options {
    bool quantize = false;
    QuantizationOptions q;
    std::string fuse = "hip";
};

Options ParseOptions(const char* text) {
    Options o;
    if (!text || !*text) return o;
    const Json j = Json::Parse(text);
    CHECK(j.is_object()) << "options must be a JSON object";
    // Besides "fuse" and the "quantize" object, the compiler flags of the reference that concern this
    // path are accepted under their own names (scripts/generate_flags_code.py:4-173; use_hip is the
    // flag a hip back-end adds next to use_nvrtc): fuse_operations, use_hip, use_nvrtc, backend_name,
    // quantize as a bool (its default mode, compiler/passes.cc:121-125), disable_per_channel_quantize.
    static const char* const kKnown[] = {"quantize", "fuse", "fuse_operations", "use_hip", "use_nvrtc", "backend_name",
                                         "disable_per_channel_quantize"};
    for (const auto& kv : j.items()) {
        bool known = false;
        for (const char* k : kKnown) known = known || kv.first == k;
        CHECK(known) << "unknown option '" << kv.first << "'";
    }
    if (const Json* b = j.find("backend_name")) CHECK(b->is_string() && b->string() == "hip") << "backend_name is 'hip' here";
    if (const Json* f = j.find("fuse")) {
        CHECK(f->is_string() && (f->string() == "hip" || f->string() == "nvrtc" || f->string() == "none")) << "fuse is 'hip', 'nvrtc' or 'none'";
        o.fuse = f->string();
    } else if (j.find("fuse_operations") || j.find("use_hip") || j.find("use_nvrtc")) {
        auto flag = [&](const char* name) {
            const Json* v = j.find(name);
            return v && v->boolean();
        };
        // groups are formed when fuse_operations is on; which generator they are built for follows
        // the use_* flag (compiler/passes.cc:56-60, compiler/chxvm/emitter.cc:697-700)
        o.fuse = !flag("fuse_operations") ? "none" : flag("use_nvrtc") && !flag("use_hip") ? "nvrtc" : "hip";
    }
    const Json* quantize = j.find("quantize");
    if (quantize && !quantize->is_object()) {
        o.quantize = quantize->boolean();
        quantize = nullptr;
    }
    if (const Json* d = j.find("disable_per_channel_quantize")) o.q.per_channel = !d->boolean();
    if (const Json* q = quantize) {
        CHECK(q->is_object()) << "quantize must be an object";
        o.quantize = true;
        for (const auto& kv : q->items()) {
            const std::string& k = kv.first;
            const Json& v = kv.second;
            if (k == "mode") {
                CHECK(v.is_string() && (v.string() == "IntegerOps" || v.string() == "QLinearOps")) << "quantize.mode is 'IntegerOps' or 'QLinearOps'";
                o.q.mode = v.string() == "QLinearOps" ? QuantizationMode::QLinearOps : QuantizationMode::IntegerOps;
            } else if (k == "per_channel") {
                o.q.per_channel = v.boolean();
            } else if (k == "static") {
                o.q.is_static = v.boolean();
            } else if (k == "asymmetric_input_types") {
                o.q.asymmertic_input_types = v.boolean();
            } else if (k == "inputs" || k == "outputs") {
                CHECK(v.is_object()) << "quantize." << k << " must be an object";
                for (const auto& p : v.items())
                    (k == "inputs" ? o.q.input_quantization_params : o.q.output_quantization_params)[p.first] =
                            ParamsFrom(p.second, "quantize." + k + "." + p.first);
            } else {
                CHECK(false) << "unknown option 'quantize." << k << "'";
            }
        }
    }
    return o;
}

std::unique_ptr<Graph> Transform(const void* model, size_t size, const char* options, OnnxModel* xmodel) {
    CHECK(model != nullptr) << "null model";
    *xmodel = ParseOnnxModel(std::string(static_cast<const char*>(model), size));
    std::unique_ptr<Graph> graph = Graph::FromOnnx(xmodel->graph);
    const Options o = ParseOptions(options);
    ExpandDynamicQuantizeLinear(graph.get());
    if (o.quantize) Quantize(o.q, graph.get());
    InferDtypes(graph.get());
    if (o.fuse == "hip") FuseHipOperations(graph.get());
    else if (o.fuse == "nvrtc") FuseElementwiseOperations(graph.get());
    graph->CheckSanity("after the passes");
    return graph;
}

void* CopyOut(const std::string& s, size_t* size) {
    void* p = malloc(s.size() + 1);
    CHECK(p) << "out of memory";
    memcpy(p, s.data(), s.size());
    static_cast<char*>(p)[s.size()] = 0;
    if (size) *size = s.size();
    return p;
}

}  // namespace

extern "C" {

int32_t chxc_compile(const void* onnx_model, size_t size, const char* options_json, void** program, size_t* program_size) {
    return Guard([&] {
        CHECK(program && program_size) << "null output";
        OnnxModel xmodel;
        std::unique_ptr<Graph> graph = Transform(onnx_model, size, options_json, &xmodel);
        *program = CopyOut(EmitProgram(*graph).SerializeAsString(), program_size);
    });
}

int32_t chxc_transform(const void* onnx_model, size_t size, const char* options_json, void** out_model, size_t* out_size,
                       char** description) {
    return Guard([&] {
        OnnxModel xmodel;
        std::unique_ptr<Graph> graph = Transform(onnx_model, size, options_json, &xmodel);
        if (out_model) {
            xmodel.graph = graph->ToOnnx();
            *out_model = CopyOut(SerializeOnnxModel(xmodel), out_size);
        }
        if (description) *description = static_cast<char*>(CopyOut(graph->DebugString(), nullptr));
    });
}

int32_t chxc_fusion_program(const void* onnx_model, size_t size, const char* options_json, int32_t group, char** text) {
    return Guard([&] {
        CHECK(text) << "null output";
        OnnxModel xmodel;
        std::unique_ptr<Graph> graph = Transform(onnx_model, size, options_json, &xmodel);
        for (Node* n : graph->GetLiveNodes()) {
            if (n->op_type() != "ChainerFusionGroup" || n->chainer_fusion_group() != group) continue;
            std::vector<int> used;
            *text = static_cast<char*>(CopyOut(BuildHipProgram(*n, &used), nullptr));
            return;
        }
        CHECK(false) << "the graph has no fusion group " << group;
    });
}

int32_t chxc_quantize_data(const float* data, size_t n, int32_t qtype, float* scale, int64_t* zero_point, int32_t* codes) {
    return Guard([&] {
        CHECK(qtype == kUInt8 || qtype == kInt8) << "qtype is 6 (uint8) or 2 (int8)";
        const QuantizedData q = QuantizeData(std::vector<float>(data, data + n), static_cast<CDtype>(qtype));
        if (scale) *scale = q.scale;
        if (zero_point) *zero_point = q.zero_point;
        if (codes) memcpy(codes, q.data.data(), n * sizeof(int32_t));
    });
}

void chxc_free(void* p) {
    free(p);
}

}  // extern "C"
