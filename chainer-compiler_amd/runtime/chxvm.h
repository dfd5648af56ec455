// ChxVM: builds the instruction objects of a program and runs them in order
// (runtime/chxvm.h, runtime/chxvm.cc:104-236 of the chainer-compiler tree).
#pragma once

#include <memory>
#include <vector>

#include "chxvm_op.h"
#include "chxvm_state.h"

namespace chainer_compiler {
namespace runtime {

// QLinearConv bias: false (default) = the reference's unscaled float bias, true = the ONNX
// operator's int32 bias added to the accumulator.
void SetQLinearConvOnnxInt32Bias(bool on);

class ChxVM {
public:
    explicit ChxVM(const ChxVMProgramProto& program);
    ~ChxVM();

    // Runs the whole program; returns the values named by its Out instructions.
    InOuts Run(const InOuts& program_inputs, const ChxVMOptions& options);

    int num_variables() const {
        return num_variables_;
    }
    const std::vector<std::string>& input_names() const {
        return input_names_;
    }
    size_t num_instructions() const {
        return program_.size();
    }

private:
    std::vector<std::unique_ptr<ChxVMOp>> program_;
    std::vector<std::string> input_names_;
    int num_variables_ = 0;
};

}  // namespace runtime
}  // namespace chainer_compiler
