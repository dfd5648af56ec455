#include "chxvm.h"

#include <iostream>

namespace chainer_compiler {
namespace runtime {

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
    for (const ChxVMInstructionProto& inst : program.instructions) {
        program_.emplace_back(MakeChxVMOp(inst));
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
