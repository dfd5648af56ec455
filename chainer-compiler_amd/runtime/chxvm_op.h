// ChxVMOp: base class of every instruction object (runtime/chxvm_op.h:13-50 of the
// chainer-compiler tree).
#pragma once

#include <cstdint>
#include <string>

#include "chxvm_proto.h"

namespace chainer_compiler {
namespace runtime {

class ChxVMState;

class ChxVMOp {
public:
    explicit ChxVMOp(const ChxVMInstructionProto& inst) : inst_(inst), id_(inst.id), op_(inst.op), name_(OpName(inst.op)) {
    }
    virtual ~ChxVMOp() = default;

    virtual void Run(ChxVMState* state) = 0;

    const ChxVMInstructionProto& instruction() const {
        return inst_;
    }
    int64_t id() const {
        return id_;
    }
    int op() const {
        return op_;
    }
    const std::string& name() const {
        return name_;
    }
    const std::string& debug_info() const {
        return inst_.debug_info;
    }
    virtual void InitImpl() {
    }

protected:
    ChxVMInstructionProto inst_;
    const int64_t id_;
    const int op_;
    const std::string name_;
};

ChxVMOp* MakeChxVMOp(const ChxVMInstructionProto& inst);

}  // namespace runtime
}  // namespace chainer_compiler
