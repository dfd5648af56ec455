// Formation of fusion groups (compiler/fusion.cc:165-214, :90-163, compiler/fusion_elementwise.cc of
// the chainer-compiler tree) and the element-wise program text of a group for the hip backend (the
// role of compiler/nvrtc_builder.cc:91-206).
#pragma once

#include <functional>
#include <set>
#include <string>
#include <vector>

#include "graph.h"

namespace chainer_compiler {

// Grows a candidate set from every fusable node over fusable producers and users, drops what
// would make the group cyclic and constants nobody in the set reads, and turns sets with at
// least `min_fuse_ops` non-trivial nodes into ChainerFusionGroup nodes of type `name`.
// Returns the number of groups created.
// can_cross (optional, not in the reference): an edge producer -> user between two fusable nodes
// that a group may not grow across.
int FuseAllConnectedNodes(const char* name, Graph* graph, int min_fuse_ops, bool can_fuse_initializers,
                          const std::function<bool(const Node&)>& is_fusable,
                          const std::function<bool(const Node& producer, const Node& user)>& can_cross = nullptr);
void CreateFusionGroup(Graph* graph, const std::set<Node*>& nodes, const std::string& fusion_type, int fusion_group_id,
                       bool can_fuse_initializers);

// The reference's element-wise rule: Identity, Add, Sub, Mul, Tanh, Sigmoid, Exp on float (or
// not yet inferred) operands and one-element float Constants; groups of type "nvrtc".
int FuseElementwiseOperations(Graph* graph);
// The hip backend's rule: the same plus Div, Neg, Max, Min (two operands), Relu, Clip with
// constant bounds, and QuantizeLinear / DequantizeLinear whose scale and zero point are
// one-element constants; groups of type "hip".
int FuseHipOperations(Graph* graph);

// Program text of a "hip" (or "nvrtc") fusion group in the format that chx_hip_elementwise takes:
// one statement per node in dependency order, the traversal of BuildNvrtcProgram.  used_inputs
// receives the indices of the group's inputs that are operands of the kernel, in `in` order (scale,
// zero-point and bound parameters are written into the text instead).
std::string BuildHipProgram(const Node& fusion_group, std::vector<int>* used_inputs);

}  // namespace chainer_compiler
