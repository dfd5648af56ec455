#include "chxvm.h"

#include <iostream>

namespace chainer_compiler {
namespace runtime {

namespace {

// DequantizeLinear(a), DequantizeLinear(b), MatMul, QuantizeLinear as one instruction: the
// quantized matrix product with the reference's float semantics (chx_hip_qlinear_matmul).
class FusedQLinearMatMulOp : public ChxVMOp {
public:
    FusedQLinearMatMulOp(const ChxVMInstructionProto& quantize, const ChxVMInstructionProto& dq_a,
                         const ChxVMInstructionProto& dq_b)
        : ChxVMOp(quantize),
          a_(dq_a.inputs[0].array), a_scale_(dq_a.inputs[1].scalar), a_zp_(dq_a.inputs[2].scalar),
          b_(dq_b.inputs[0].array), b_scale_(dq_b.inputs[1].scalar), b_zp_(dq_b.inputs[2].scalar),
          y_scale_(quantize.inputs[1].scalar), y_zp_(quantize.inputs[2].scalar), y_(quantize.outputs[0]) {
    }

    void Run(ChxVMState* st) override {
        if (st->trace_level()) std::cerr << "QLinearMatMul(fused) $" << a_ << " $" << b_ << " -> $" << y_ << std::endl;
        const chainerx::Array a = st->GetArray(a_), b = st->GetArray(b_);
        auto zp_of = [&](int slot) -> StrictScalar {
            absl::optional<StrictScalar> z = st->GetOptionalScalar(slot);
            return z.has_value() ? *z : StrictScalar(chainerx::Dtype::kUInt8, chainerx::Scalar(0u), false);
        };
        const StrictScalar az = zp_of(a_zp_), bz = zp_of(b_zp_), yz = zp_of(y_zp_);
        CHECK_LE(2, a.ndim());
        CHECK_EQ(a.ndim(), b.ndim());
        chainerx::Shape shape(a.shape().begin(), a.shape().end() - 1);
        shape.push_back(b.shape()[b.ndim() - 1]);
        chainerx::Array y = chainerx::Empty(shape, yz.dtype());
        chx_hip_tensor at = a.hip(), bt = b.hip(), yt = y.hip();
        CHXVM_HIP_CALL(chx_hip_qlinear_matmul(
                &at, static_cast<float>(st->GetScalar(a_scale_)), static_cast<int32_t>(static_cast<int64_t>(az)), &bt,
                static_cast<float>(st->GetScalar(b_scale_)), static_cast<int32_t>(static_cast<int64_t>(bz)),
                static_cast<float>(st->GetScalar(y_scale_)), static_cast<int32_t>(static_cast<int64_t>(yz)),
                nullptr, CHX_HIP_ROUND_REFERENCE, &yt, nullptr));
        st->SetArray(y_, y);
    }

private:
    int a_, a_scale_, a_zp_, b_, b_scale_, b_zp_, y_scale_, y_zp_, y_;
};

class NopOp : public ChxVMOp {
public:
    explicit NopOp(const ChxVMInstructionProto& inst) : ChxVMOp(inst) {
    }
    void Run(ChxVMState*) override {
    }
};

// Number of times a variable slot is read by the program.
int CountUses(const ChxVMProgramProto& program, int slot) {
    int n = 0;
    for (const ChxVMInstructionProto& inst : program.instructions)
        for (const ChxVMValueProto& v : inst.inputs) {
            if ((v.type == ChxVMValueProto::ARRAY || v.type == ChxVMValueProto::OPTIONAL_ARRAY) && v.array == slot) ++n;
            if (v.type == ChxVMValueProto::ARRAY_LIST)
                for (int id : v.array_list) n += id == slot;
        }
    return n;
}

}  // namespace

ChxVM::ChxVM(const ChxVMProgramProto& program) : input_names_(program.input_names) {
    // number of variable slots = highest id mentioned + 1 (runtime/chxvm.cc:104-140)
    int max_id = -1;
    for (const ChxVMInstructionProto& inst : program.instructions) {
        for (int o : inst.outputs) max_id = o > max_id ? o : max_id;
        for (const ChxVMValueProto& v : inst.inputs) {
            for (int id : {v.array, v.sequence, v.opaque, v.shape, v.scalar}) max_id = id > max_id ? id : max_id;
            for (int id : v.array_list) max_id = id > max_id ? id : max_id;
        }
    }
    num_variables_ = max_id + 1;
    // Find the QLinearMatMul sequences: QuantizeLinear <- MatMul <- two DequantizeLinear, every
    // intermediate read exactly once apart from its Free.
    const int n = static_cast<int>(program.instructions.size());
    const int kDequantize = OpNumber("DequantizeLinear"), kMatMul = OpNumber("MatMul"), kQuantize = OpNumber("QuantizeLinear"),
              kFree = OpNumber("Free");
    std::vector<int> producer(num_variables_ > 0 ? num_variables_ : 1, -1);
    for (int i = 0; i < n; ++i)
        for (int o : program.instructions[i].outputs)
            if (o >= 0) producer[o] = i;
    std::vector<int> role(n, 0);  // 0 plain, 1 dropped, 2 fused (at the QuantizeLinear)
    std::vector<std::pair<int, int>> fused_inputs(n);
    auto single_use = [&](int slot) {
        // one consumer plus at most one Free
        int frees = 0;
        for (const ChxVMInstructionProto& inst : program.instructions)
            if (inst.op == kFree && inst.inputs.size() == 1 && inst.inputs[0].array == slot) ++frees;
        return CountUses(program, slot) - frees == 1;
    };
    for (int q = 0; q < n; ++q) {
        const ChxVMInstructionProto& qi = program.instructions[q];
        if (qi.op != kQuantize || qi.inputs.size() != 3 || qi.inputs[0].array < 0) continue;
        const int m = producer[qi.inputs[0].array];
        if (m < 0 || program.instructions[m].op != kMatMul || !single_use(qi.inputs[0].array)) continue;
        const ChxVMInstructionProto& mi = program.instructions[m];
        const int da = producer[mi.inputs[0].array], db = producer[mi.inputs[1].array];
        if (da < 0 || db < 0 || da == db || program.instructions[da].op != kDequantize ||
            program.instructions[db].op != kDequantize)
            continue;
        if (!single_use(mi.inputs[0].array) || !single_use(mi.inputs[1].array)) continue;
        role[q] = 2;
        fused_inputs[q] = std::make_pair(da, db);
        role[m] = role[da] = role[db] = 1;
    }
    std::vector<bool> dead(num_variables_ > 0 ? num_variables_ : 1, false);
    for (int i = 0; i < n; ++i)
        if (role[i] == 1)
            for (int o : program.instructions[i].outputs)
                if (o >= 0) dead[o] = true;
    for (int i = 0; i < n; ++i) {
        const ChxVMInstructionProto& inst = program.instructions[i];
        const bool frees_dead = inst.op == kFree && inst.inputs.size() == 1 && inst.inputs[0].array >= 0 && dead[inst.inputs[0].array];
        if (role[i] == 1 || frees_dead) {
            program_.emplace_back(new NopOp(inst));
        } else if (role[i] == 2) {
            program_.emplace_back(new FusedQLinearMatMulOp(inst, program.instructions[fused_inputs[i].first],
                                                           program.instructions[fused_inputs[i].second]));
        } else {
            program_.emplace_back(MakeChxVMOp(inst));
        }
        program_.back()->InitImpl();
    }
}

ChxVM::~ChxVM() = default;

InOuts ChxVM::Run(const InOuts& program_inputs, const ChxVMOptions& options) {
    for (const std::string& name : input_names_)
        CHECK(program_inputs.count(name)) << "Input '" << name << "' not found";  // runtime/chxvm.cc:142-143
    ChxVMState state(options, num_variables_, program_inputs);
    while (state.pc() < static_cast<int>(program_.size())) {
        const int pc = state.pc();
        ChxVMOp* op = program_[pc].get();
        try {
            op->Run(&state);
        } catch (...) {
            std::cerr << "Exception in " << op->name() << " (pc " << pc << ") " << op->debug_info() << std::endl;
            throw;
        }
        state.set_pc(state.pc() + 1);  // jumps set pc - 1 themselves (runtime/ops/controlflow.cc:7-21)
    }
    return state.GetOutputs();
}

}  // namespace runtime
}  // namespace chainer_compiler
