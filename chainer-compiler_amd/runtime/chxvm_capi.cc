#include "chxvm_capi.h"

#include <cstdlib>
#include <cstring>
#include <string>

#include "chrome_tracing.h"
#include "chxvm.h"
#include "configs/backend_config.h"
#include "replay.h"

using chainer_compiler::BackendConfig;
using namespace chainer_compiler::runtime;

namespace {

thread_local std::string g_last_error;
// run options of chxvm_set_option, applied by every later chxvm_program_run
std::string g_chrome_tracing_path, g_dump_outputs_dir;
bool g_check_nans = false, g_check_infs = false, g_check_types = false;
bool g_onnx_int32_bias = false;  // the default of programs that have not been given their own (chxvm_program_set_option)
int g_dump_memory_usage = 0;

template <class Fn>
int32_t Guard(Fn fn) {
    try {
        fn();
        return 0;
    } catch (const std::exception& e) {
        g_last_error = e.what();
        return 1;
    }
}

}  // namespace

namespace chainer_compiler {
namespace runtime {
// for the other C faces of this library (compiler/compiler_capi.cc)
void SetLastError(const std::string& message) {
    g_last_error = message;
}
}  // namespace runtime
}  // namespace chainer_compiler

struct chxvm_program {
    std::unique_ptr<ChxVM> vm;
    int onnx_int32_bias = -1;  // -1: the process default at the time of a run
};

struct chxvm_outputs {
    std::vector<std::string> names;
    std::vector<chainerx::Array> arrays;
    InOuts keep_inputs;
};

struct chxvm_replay {
    std::shared_ptr<PoolAllocator> pool;
    void* stream = nullptr;
    chx_hip_graph* graph = nullptr;
    chxvm_outputs outputs;
    int32_t warm_runs = 0;
    std::vector<chx_hip_qconv_plan*> pinned_plans;  // whose memory the graph's kernels address

    ~chxvm_replay() {
        chx_hip_graph_destroy(graph);
        for (chx_hip_qconv_plan* plan : pinned_plans) (void)chx_hip_qconv_plan_pin(plan, -1);
        outputs.arrays.clear();
        outputs.keep_inputs.clear();
        if (stream) (void)chx_hip_stream_destroy(stream);
    }
};

namespace {

InOuts BorrowInputs(const char* const* input_names, const chx_hip_tensor* inputs, int32_t num_inputs) {
    InOuts in;
    for (int32_t i = 0; i < num_inputs; ++i) {
        const chx_hip_tensor& t = inputs[i];
        chainerx::Shape shape;
        chainerx::Strides strides;
        for (int d = 0; d < t.ndim; ++d) {
            shape.push_back(t.shape[d]);
            strides.push_back(t.strides[d]);
        }
        chainerx::Array a = chainerx::Array::MakeBorrowed(t.data, static_cast<chainerx::Dtype>(t.dtype), shape, strides);
        CHECK(in.emplace(input_names[i], std::make_shared<ChxVMVar>(a)).second) << "duplicate input " << input_names[i];
    }
    return in;
}

}  // namespace

extern "C" {

const char* chxvm_last_error(void) {
    return g_last_error.c_str();
}

int32_t chxvm_num_ops(void) {
    return NumOps();
}

const char* chxvm_op_name(int32_t op) {
    return OpName(op);
}

int32_t chxvm_op_number(const char* name) {
    return OpNumber(name);
}

int32_t chxvm_proto_roundtrip(const void* bytes, size_t size, void** out, size_t* out_size) {
    return Guard([&] {
        const ChxVMProgramProto program = ChxVMProgramProto::ParseFromString(std::string(static_cast<const char*>(bytes), size));
        const std::string again = program.SerializeAsString();
        *out = std::malloc(again.size() ? again.size() : 1);
        std::memcpy(*out, again.data(), again.size());
        *out_size = again.size();
    });
}

void chxvm_free(void* p) {
    std::free(p);
}

int32_t chxvm_program_create(const void* bytes, size_t size, chxvm_program** out) {
    return Guard([&] {
        const ChxVMProgramProto program = ChxVMProgramProto::ParseFromString(std::string(static_cast<const char*>(bytes), size));
        std::unique_ptr<chxvm_program> p(new chxvm_program());
        p->vm.reset(new ChxVM(program));
        *out = p.release();
    });
}

void chxvm_program_destroy(chxvm_program* program) {
    delete program;
}

int32_t chxvm_program_num_instructions(const chxvm_program* program) {
    return static_cast<int32_t>(program->vm->num_instructions());
}

int32_t chxvm_program_num_inputs(const chxvm_program* program) {
    return static_cast<int32_t>(program->vm->input_names().size());
}

const char* chxvm_program_input_name(const chxvm_program* program, int32_t i) {
    return program->vm->input_names()[static_cast<size_t>(i)].c_str();
}

int32_t chxvm_program_run(
        chxvm_program* program,
        const char* const* input_names,
        const chx_hip_tensor* inputs,
        int32_t num_inputs,
        int32_t trace_level,
        chxvm_outputs** out) {
    return Guard([&] {
        InOuts in = BorrowInputs(input_names, inputs, num_inputs);
        ChxVMOptions options;
        options.trace_level = trace_level;
        options.dump_outputs_dir = g_dump_outputs_dir;
        options.check_nans = g_check_nans;
        options.check_infs = g_check_infs;
        options.check_types = g_check_types;
        options.dump_memory_usage = g_dump_memory_usage;
        options.qlinearconv_onnx_int32_bias = program->onnx_int32_bias >= 0 ? program->onnx_int32_bias != 0 : g_onnx_int32_bias;
        std::unique_ptr<ChromeTracingEmitter> tracing;
        if (!g_chrome_tracing_path.empty()) {
            tracing.reset(new ChromeTracingEmitter());
            options.chrome_tracing = tracing.get();
        }
        InOuts result = program->vm->Run(in, options);
        if (tracing) tracing->Emit(g_chrome_tracing_path);
        std::unique_ptr<chxvm_outputs> o(new chxvm_outputs());
        for (const auto& p : result) {
            o->names.push_back(p.first);
            o->arrays.push_back(p.second->GetArray());
        }
        o->keep_inputs = in;
        CHXVM_HIP_CALL(chx_hip_stream_synchronize(nullptr));  // device sync at the end of a run (tools/run_onnx.cc:462)
        *out = o.release();
    });
}

int32_t chxvm_program_capture(
        chxvm_program* program, const char* const* input_names, const chx_hip_tensor* inputs, int32_t num_inputs, chxvm_replay** out) {
    return Guard([&] {
        CHECK(program != nullptr && out != nullptr) << "null argument";
        *out = nullptr;
        InOuts in = BorrowInputs(input_names, inputs, num_inputs);
        ChxVMOptions options;  // no tracing, checking or dumping: all of them read results back
        options.qlinearconv_onnx_int32_bias = program->onnx_int32_bias >= 0 ? program->onnx_int32_bias != 0 : g_onnx_int32_bias;
        std::unique_ptr<chxvm_replay> r(new chxvm_replay());
        r->pool = std::make_shared<PoolAllocator>();
        CHXVM_HIP_CALL(chx_hip_stream_create(&r->stream));
        // Eager runs on the stream until one of them finds every block it asks for in the pool: plans are
        // built, launch configurations measured, fused kernels compiled, and the pool reaches the state that
        // the recorded run starts from.
        for (;;) {
            const int64_t before = r->pool->blocks_created();
            {
                chainerx::DeviceContextScope scope(r->stream, r->pool.get());
                (void)program->vm->Run(in, options);
            }
            CHXVM_HIP_CALL(chx_hip_stream_synchronize(r->stream));
            ++r->warm_runs;
            if (r->pool->blocks_created() == before) break;
            CHECK_LT(r->warm_runs, 8) << "the runs of this program keep allocating new blocks";
        }
        r->pool->set_frozen(true);
        CHXVM_HIP_CALL(chx_hip_capture_begin(r->stream));
        InOuts result;
        try {
            chainerx::DeviceContextScope scope(r->stream, r->pool.get());
            ChxVMOptions recorded = options;
            recorded.pinned_plans = &r->pinned_plans;
            result = program->vm->Run(in, recorded);
        } catch (...) {
            chx_hip_graph* dropped = nullptr;
            (void)chx_hip_capture_end(r->stream, &dropped);
            chx_hip_graph_destroy(dropped);
            throw;
        }
        CHXVM_HIP_CALL(chx_hip_capture_end(r->stream, &r->graph));
        for (const auto& p : result) {
            r->outputs.names.push_back(p.first);
            r->outputs.arrays.push_back(p.second->GetArray());
        }
        r->outputs.keep_inputs = in;
        *out = r.release();
    });
}

int32_t chxvm_replay_launch(chxvm_replay* replay, void* stream) {
    return Guard([&] {
        CHECK(replay != nullptr && replay->graph != nullptr) << "null replay";
        CHXVM_HIP_CALL(chx_hip_graph_launch(replay->graph, stream ? stream : replay->stream));
    });
}

int32_t chxvm_replay_synchronize(chxvm_replay* replay) {
    return Guard([&] {
        CHECK(replay != nullptr) << "null replay";
        CHXVM_HIP_CALL(chx_hip_stream_synchronize(replay->stream));
    });
}

const chxvm_outputs* chxvm_replay_outputs(const chxvm_replay* replay) {
    return replay ? &replay->outputs : nullptr;
}

int64_t chxvm_replay_info(const chxvm_replay* replay, const char* name) {
    const std::string n = name ? name : "";
    if (!replay) return -1;
    if (n == "pool_bytes") return replay->pool->bytes_reserved();
    if (n == "pool_blocks") return replay->pool->blocks_created();
    if (n == "warm_runs") return replay->warm_runs;
    return -1;
}

void chxvm_replay_destroy(chxvm_replay* replay) {
    delete replay;
}

int32_t chxvm_outputs_count(const chxvm_outputs* outputs) {
    return static_cast<int32_t>(outputs->arrays.size());
}

const char* chxvm_outputs_name(const chxvm_outputs* outputs, int32_t i) {
    return outputs->names[static_cast<size_t>(i)].c_str();
}

int32_t chxvm_outputs_get(const chxvm_outputs* outputs, int32_t i, chx_hip_tensor* out) {
    return Guard([&] {
        CHECK_LT(static_cast<size_t>(i), outputs->arrays.size());
        *out = outputs->arrays[static_cast<size_t>(i)].hip();
    });
}

void chxvm_outputs_destroy(chxvm_outputs* outputs) {
    delete outputs;
}

int32_t chxvm_set_option(const char* name, const char* value) {
    return Guard([&] {
        const std::string n = name, v = value;
        if (n == "qlinearconv_bias") {
            CHECK(v == "reference" || v == "onnx_int32") << "qlinearconv_bias is 'reference' or 'onnx_int32', got " << v;
            g_onnx_int32_bias = v == "onnx_int32";
        } else if (n == "fuse_residual") {
            CHECK(v == "on" || v == "off") << "fuse_residual is 'on' or 'off', got " << v;
            SetFuseResidual(v == "on");
        } else if (n == "pair_convolutions") {
            CHECK(v == "on" || v == "off") << "pair_convolutions is 'on' or 'off', got " << v;
            SetPairConvolutions(v == "on");
        } else if (n == "store_minus_128") {
            CHECK(v == "on" || v == "off") << "store_minus_128 is 'on' or 'off', got " << v;
            SetStoreMinus128(v == "on");
        } else if (n == "chrome_tracing") {
            g_chrome_tracing_path = v;
        } else if (n == "dump_outputs_dir") {
            g_dump_outputs_dir = v;
        } else if (n == "check_nans" || n == "check_infs" || n == "check_types") {  // the flags of the same names of tools/run_onnx.cc
            CHECK(v == "on" || v == "off") << n << " is 'on' or 'off', got " << v;
            (n == "check_nans" ? g_check_nans : n == "check_infs" ? g_check_infs : g_check_types) = v == "on";
        } else if (n == "dump_memory_usage") {
            CHECK(v == "0" || v == "1" || v == "2") << "dump_memory_usage is 0, 1 or 2, got " << v;
            g_dump_memory_usage = v[0] - '0';
        } else {
            CHECK(false) << "unknown option " << n;
        }
    });
}

int32_t chxvm_program_set_option(chxvm_program* program, const char* name, const char* value) {
    return Guard([&] {
        CHECK(program != nullptr) << "null program";
        const std::string n = name, v = value;
        if (n == "qlinearconv_bias") {
            CHECK(v == "reference" || v == "onnx_int32" || v == "default") << "qlinearconv_bias is 'reference', 'onnx_int32' or 'default', got " << v;
            program->onnx_int32_bias = v == "default" ? -1 : v == "onnx_int32" ? 1 : 0;
        } else {
            CHECK(false) << "unknown program option " << n;
        }
    });
}

int64_t chxvm_program_counter(const chxvm_program* program, const char* name) {
    const std::string n = name ? name : "";
    if (program && n == "qlinearconv_residual_fusions") return program->vm->residual_fusions();
    if (program && n == "minus_128_variables") return program->vm->minus_128_variables();
    return -1;
}

int64_t chxvm_counter(const char* name) {
    const std::string n = name ? name : "";
    if (n == "qlinearconv_residual_fusions") return QLinearConvResidualFusions();
    if (n == "qlinearconv_pair_fusions") return QLinearConvPairFusions();
    if (n == "minus_128_stores") return Minus128Stores();
    return -1;
}

int32_t chxvm_backend_config_has(const char* config, int32_t is_json, const char* section, const char* key, int32_t* out) {
    return Guard([&] {
        std::unique_ptr<BackendConfig> c = is_json ? BackendConfig::FromJSON(config) : BackendConfig::FromName(config);
        const std::string s = section;
        if (s == "simplify_preproc") *out = static_cast<int32_t>(c->GetSimplifyPreproc().count(key));
        else if (s == "simplify") *out = static_cast<int32_t>(c->GetSimplify().count(key));
        else if (s == "merge") *out = static_cast<int32_t>(c->GetMerge().count(key));
        else if (s == "expanding_functions") *out = static_cast<int32_t>(c->GetExpandingFunctions().count(key));
        else if (s == "supported_ops") *out = c->HasOp(key) ? 1 : 0;
        else CHECK(false) << "unknown section " << s;
    });
}

int32_t chxvm_backend_config_name(const char* config, int32_t is_json, char* buf, size_t buf_size) {
    return Guard([&] {
        std::unique_ptr<BackendConfig> c = is_json ? BackendConfig::FromJSON(config) : BackendConfig::FromName(config);
        CHECK_LT(c->name().size(), buf_size);
        std::strcpy(buf, c->name().c_str());
    });
}

}  // extern "C"
