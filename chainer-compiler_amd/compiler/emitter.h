// Graph -> ChxVMProgramProto for the hip backend: the part of compiler/chxvm/emitter.cc and
// compiler/chxvm/simple_node_emitter.cc of the chainer-compiler tree that the quantized-inference
// path and its element-wise groups need.  Instructions follow a topological order; every value is
// freed after its last reader (compiler/chxvm/emitter.cc EmitGraph).
#pragma once

#include <string>

#include "../runtime/chxvm_proto.h"
#include "graph.h"

namespace chainer_compiler {

// CHECK-fails on a node type the hip backend does not run.
runtime::ChxVMProgramProto EmitProgram(const Graph& graph);

}  // namespace chainer_compiler
