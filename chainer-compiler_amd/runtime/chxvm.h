// ChxVM: builds the instruction objects of a program and runs them in order
// (runtime/chxvm.h, runtime/chxvm.cc:104-236 of the chainer-compiler tree).
#pragma once

#include <memory>
#include <vector>

#include "chxvm_op.h"
#include "chxvm_state.h"

namespace chainer_compiler {
namespace runtime {

// A residual sum that the next QLinearConvOp::RunImpl of a run (ChxVMState::set_residual_request) may
// compute inside its kernel: out = QuantizeLinear(act(DequantizeLinear(y) + DequantizeLinear(r))) for its own result
// y.  The op takes the request when y's quantization is the one the group dequantizes with and the
// kernel accepts the operands; it then sets `done`, leaves the group's result in `out` and returns
// a null array for y.  Otherwise it runs as usual and the caller runs the group afterwards.
struct QLinearConvResidualRequest {
    chainerx::Array r;
    float y_scale = 0, r_scale = 0, out_scale = 0;
    int32_t y_zero_point = 0, r_zero_point = 0, out_zero_point = 0;
    chainerx::Dtype y_dtype = chainerx::Dtype::kUInt8, out_dtype = chainerx::Dtype::kUInt8;
    bool relu = false;
    int out_slot = -1;  // the variable the sum goes to (ChxVMState::store_minus_128 says how it may be stored)
    chainerx::Array out;
    bool done = false;
};
int64_t QLinearConvResidualFusions();  // requests taken so far, process-wide (a statistic; the runs count their own)
// Whether programs loaded from now on pair such convolutions and groups at all (default: yes).
void SetFuseResidual(bool on);

// Two QLinearConv instructions that read the same value with the same geometry (the main-path and the shortcut
// convolution of a down-sampling block), run as one launch where the second one's operands allow it
// (chx_hip_qconv_plan_run_pair) and one after the other otherwise; it stands at the place of the first and writes
// both results.
std::unique_ptr<ChxVMOp> MakeQLinearConvPairOp(const ChxVMInstructionProto& first, const ChxVMInstructionProto& second);
int64_t QLinearConvPairFusions();  // pairs run as one launch so far, process-wide
// Whether programs loaded from now on pair such convolutions at all (default: yes).
void SetPairConvolutions(bool on);

// Values that only convolutions read (as their input, or as the residual operand of a sum computed inside one) are
// stored as code - 128 in int8 arrays (CHX_HIP_STORE_MINUS_128 of the device library): the reading kernel then
// needs no sign flips in its inner loop.  Whether programs loaded from now on do so at all (default: yes).
void SetStoreMinus128(bool on);
int64_t Minus128Stores();  // results written in that storage so far, process-wide
// The plain uint8 array of a value held in that storage (chx_hip_codes_minus_128).
chainerx::Array PlainCodes(const chainerx::Array& minus_128);

class ChxVM {
public:
    explicit ChxVM(const ChxVMProgramProto& program);
    ~ChxVM();

    // Runs the whole program; returns the values named by its Out instructions.
    InOuts Run(const InOuts& program_inputs, const ChxVMOptions& options);
    // residual sums that convolutions of this program computed inside their kernels, over all runs
    int64_t residual_fusions() const {
        return residual_fusions_;
    }

    // variables of the program that its convolutions keep as code - 128 between them (ChxVMState::store_minus_128)
    int64_t minus_128_variables() const {
        int64_t n = 0;
        for (bool marked : minus_128_slots_) n += marked ? 1 : 0;
        return n;
    }

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
    std::vector<ChxVMTypeProto> input_types_;
    int num_variables_ = 0;
    int64_t residual_fusions_ = 0;
    std::vector<bool> minus_128_slots_;  // per variable: see ChxVMState::store_minus_128
};

}  // namespace runtime
}  // namespace chainer_compiler
