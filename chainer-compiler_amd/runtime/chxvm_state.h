// ChxVMState: the variable slots of one run, with the accessors the generated Run() glue uses
// (runtime/chxvm_state.h:21-106, runtime/chxvm_state.cc of the chainer-compiler tree).
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "chxvm_var.h"

namespace chainer_compiler {
namespace runtime {

typedef std::map<std::string, std::shared_ptr<ChxVMVar>> InOuts;

class ChromeTracingEmitter;
struct QLinearConvResidualRequest;

struct ChxVMOptions {
    int trace_level = 0;
    bool is_training = false;
    // inputs against the program's input_types before the run, every typed result against the
    // instruction's output_types after it (runtime/chxvm.cc:38-64,140-158)
    bool check_types = false;
    bool check_nans = false;
    bool check_infs = false;
    // 1: bytes held by the variable slots at their peak, printed after the run; 2: also after every
    // instruction (runtime/chxvm.cc:208-237; the allocator hooks of the reference have no counterpart)
    int dump_memory_usage = 0;
    // an event per executed instruction; the device is synchronized after each one so that an
    // event spans the instruction's kernels (runtime/chxvm.cc:180 times the host side only)
    ChromeTracingEmitter* chrome_tracing = nullptr;
    // every named array output of every instruction as <dir>/<5-digit instruction id>_<name>.npy
    // (runtime/chxvm.cc:70-92)
    std::string dump_outputs_dir;
    // QLinearConv bias: false = the reference's unscaled float bias added after the convolution
    // (runtime/ops/quantize.cc:93), true = the ONNX operator's int32 bias added to the accumulator
    bool qlinearconv_onnx_int32_bias = false;
    // set while a run is being recorded into a device graph: every convolution plan the run uses is pinned and listed
    // here, so that the recording can release them when it is destroyed (chx_hip_qconv_plan_pin)
    std::vector<struct chx_hip_qconv_plan*>* pinned_plans = nullptr;
};

class ChxVMState {
public:
    ChxVMState(const ChxVMOptions& options, int num_variables, const InOuts& inputs);

    int pc() const {
        return pc_;
    }
    void set_pc(int pc) {
        pc_ = pc;
    }

    chainerx::Array GetArray(int index);
    absl::optional<chainerx::Array> GetOptionalArray(int index);
    void SetArray(int index, const chainerx::Array& value);
    void FreeVar(int index);

    std::vector<chainerx::Array> GetArrayList(const std::vector<int>& index);
    void SetArrayList(const std::vector<int>& index, const std::vector<chainerx::Array>& vars);

    ChxVMVar* GetVar(int index);
    // the same without the check that the slot is set: null for a slot that holds nothing (never written, or freed)
    ChxVMVar* PeekVar(int index);
    void SetVar(int index, const ChxVMVar& var);

    const chainerx::Shape& GetShape(int index);
    void SetShape(int index, chainerx::Shape s);

    const StrictScalar& GetScalar(int index);
    absl::optional<StrictScalar> GetOptionalScalar(int index);
    void SetScalar(int index, StrictScalar s);

    std::string GetVarString(int index);
    std::string GetVarListString(const std::vector<int>& indices);

    void Input(const std::string& name, int index);
    void Output(const std::string& name, int index);

    // bytes of device memory the variable slots keep alive, shared buffers counted once
    // (runtime/chxvm_state.cc:274-290), and the per-slot list of runtime/chxvm_state.cc:265-272
    int64_t GetTotalVariableSize() const;
    void ShowVariableStatus() const;

    const InOuts& GetOutputs() const {
        return outputs_;
    }

    // Scans of an instruction's outputs for NaN / Inf elements (runtime/chxvm_state.cc:202-263): a hit
    // prints every operand and result of the instruction and fails the run.  float32 arrays are
    // scanned on the device; the 8-bit and int32 arrays of the quantized path hold neither.
    void CheckNans(const std::vector<int>& inputs, const std::vector<int>& outputs);
    void CheckInfs(const std::vector<int>& inputs, const std::vector<int>& outputs);

    int trace_level() const {
        return options_.trace_level;
    }
    bool is_training() const {
        return options_.is_training;
    }
    bool check_nans() const {
        return options_.check_nans;
    }
    bool check_infs() const {
        return options_.check_infs;
    }
    const ChxVMOptions& options() const {
        return options_;
    }

    // A residual sum that the next QLinearConvOp::RunImpl of this run may compute inside its kernel
    // (see QLinearConvResidualRequest in chxvm.h); null when none is pending.
    QLinearConvResidualRequest* residual_request() const {
        return residual_request_;
    }
    void set_residual_request(QLinearConvResidualRequest* request) {
        residual_request_ = request;
    }
    // residual sums computed inside a convolution during this run
    int64_t residual_fusions() const {
        return residual_fusions_;
    }
    void count_residual_fusion() {
        ++residual_fusions_;
    }

    // Whether the uint8 value of variable `slot` may be stored as code - 128 in an int8 array in this run (the
    // program's analysis found only readers that take that storage, and no option of the run looks at raw values);
    // an int8 array found in such a slot where the program's types say uint8 holds that storage.
    bool store_minus_128(int slot) const {
        return minus_128_slots_ && slot >= 0 && slot < static_cast<int>(minus_128_slots_->size()) && (*minus_128_slots_)[slot];
    }
    void set_minus_128_slots(const std::vector<bool>* slots) {
        minus_128_slots_ = slots;
    }

private:
    void CheckNonFinite(const std::vector<int>& inputs, const std::vector<int>& outputs, bool infinities);

    int pc_ = 0;
    std::vector<std::unique_ptr<ChxVMVar>> variables_;
    InOuts inputs_;
    InOuts outputs_;
    ChxVMOptions options_;
    QLinearConvResidualRequest* residual_request_ = nullptr;
    int64_t residual_fusions_ = 0;
    const std::vector<bool>* minus_128_slots_ = nullptr;
};

}  // namespace runtime
}  // namespace chainer_compiler
