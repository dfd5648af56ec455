// Graph IR of the compiler side: values, nodes, graphs and a builder, the parts of
// compiler/{graph,node,value,tensor,type,graph_builder}.h of the chainer-compiler tree that the
// quantizer, the fusion pass and the ChxVM emitter work on.  Op types are ONNX op names
// ("Conv", "QLinearConv", ...); a fusion group is a node "ChainerFusionGroup" with a subgraph.
#pragma once

#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "onnx_proto.h"

namespace chainer_compiler {

// element types as ChainerX numbers them (compiler/dtype.h:14-25); 0 = unknown
enum CDtype { kUnknown = 0, kBool = 1, kInt8 = 2, kInt16 = 3, kInt32 = 4, kInt64 = 5, kUInt8 = 6, kFloat16 = 7, kFloat32 = 8, kFloat64 = 9 };
CDtype DtypeFromOnnx(int onnx_dtype);
int DtypeToOnnx(CDtype dtype);
int DtypeSize(CDtype dtype);
bool DtypeIsFloat(CDtype dtype);
const char* DtypeName(CDtype dtype);

struct Type {
    CDtype dtype = kUnknown;
    std::vector<int64_t> dims;
    bool has_dims = false;
    Type() = default;
    Type(CDtype dt, std::vector<int64_t> d) : dtype(dt), dims(std::move(d)), has_dims(true) {}
};

// A constant tensor held by the compiler (host memory).
class Tensor {
public:
    Tensor(std::string name, CDtype dtype, std::vector<int64_t> dims, std::string raw);
    static Tensor FromOnnx(const OnnxTensor& t);
    OnnxTensor ToOnnx() const;
    template <class T>
    static Tensor FromVector(const std::string& name, CDtype dtype, std::vector<int64_t> dims, const std::vector<T>& data) {
        return Tensor(name, dtype, std::move(dims), std::string(reinterpret_cast<const char*>(data.data()), data.size() * sizeof(T)));
    }
    const std::string& name() const { return name_; }
    CDtype dtype() const { return dtype_; }
    const std::vector<int64_t>& dims() const { return dims_; }
    int64_t NumElements() const;
    const std::string& raw() const { return raw_; }
    double GetAsDouble(int64_t i) const;  // element i converted to double
    std::vector<float> AsFloats() const;  // every element converted to float

private:
    std::string name_;
    CDtype dtype_;
    std::vector<int64_t> dims_;
    std::string raw_;
};

class Node;
class Graph;

class Value {
public:
    enum Kind { kInput, kOutput, kTemp, kNull };
    Value(std::string name, Type type, Kind kind) : name_(std::move(name)), type_(std::move(type)), kind_(kind) {}
    const std::string& name() const { return name_; }
    const Type& type() const { return type_; }
    void set_type(const Type& t) { type_ = t; }
    Kind kind() const { return kind_; }
    bool IsInput() const { return kind_ == kInput; }
    bool IsOutput() const { return kind_ == kOutput; }
    bool IsNull() const { return kind_ == kNull; }
    const Tensor* initializer() const { return initializer_.get(); }
    void ResetInitializer(std::unique_ptr<Tensor> t) { initializer_ = std::move(t); }
    Node* producer() const { return producer_; }
    const std::vector<Node*>& users() const { return users_; }
    // the constant behind the value: its initializer, or the tensor of the Constant node producing it
    const Tensor* GetConstTensor() const;

private:
    friend class Node;
    friend class Graph;
    std::string name_;
    Type type_;
    Kind kind_;
    std::unique_ptr<Tensor> initializer_;
    Node* producer_ = nullptr;
    std::vector<Node*> users_;
};

class Node {
public:
    Node(std::string name, std::string op_type, std::vector<Value*> inputs, std::vector<Value*> outputs);
    const std::string& name() const { return name_; }
    const std::string& op_type() const { return op_type_; }
    const std::string& domain() const { return domain_; }
    void set_domain(const std::string& d) { domain_ = d; }
    const std::vector<Value*>& inputs() const { return inputs_; }
    const std::vector<Value*>& outputs() const { return outputs_; }
    Value* input(int i) const { return inputs_.at(i); }
    Value* output(int i) const { return outputs_.at(i); }
    void ReplaceInput(Value* from, Value* to);
    void ReplaceOutput(Value* from, Value* to);
    bool detached() const { return detached_; }
    int GetNumActualInputs() const;  // inputs that are not null values
    bool IsZeroCost() const { return op_type_ == "Identity" || op_type_ == "Constant"; }  // compiler/node.cc:146-153

    // attributes
    std::vector<OnnxAttr>& attrs() { return attrs_; }
    const std::vector<OnnxAttr>& attrs() const { return attrs_; }
    const OnnxAttr* FindAttr(const std::string& name) const;
    int64_t GetInt(const std::string& name, int64_t def) const;
    float GetFloat(const std::string& name, float def) const;
    std::string GetString(const std::string& name, const std::string& def) const;
    std::vector<int64_t> GetInts(const std::string& name) const;
    void SetInt(const std::string& name, int64_t v);
    void SetInts(const std::string& name, const std::vector<int64_t>& v);
    void SetString(const std::string& name, const std::string& v);
    void SetTensor(const std::string& name, const Tensor& t);
    void CopyAttrsFrom(const Node& other, const std::vector<std::string>& names);
    std::unique_ptr<Tensor> tensor_value() const;  // the "value" attribute of a Constant

    // fusion
    Graph* subgraph() const { return subgraph_.get(); }
    void set_subgraph(std::unique_ptr<Graph> g);
    const std::string& fusion_type() const { return fusion_type_; }
    void set_fusion_type(const std::string& t) { fusion_type_ = t; }
    int chainer_fusion_group() const { return fusion_group_; }
    void set_chainer_fusion_group(int id) { fusion_group_ = id; }

    std::string ToString() const;

private:
    friend class Graph;
    std::string name_, op_type_, domain_;
    std::vector<Value*> inputs_, outputs_;
    std::vector<OnnxAttr> attrs_;
    std::unique_ptr<Graph> subgraph_;
    std::string fusion_type_;
    int fusion_group_ = 0;
    bool detached_ = false;
};

class Graph {
public:
    explicit Graph(std::string name) : name_(std::move(name)) {}
    ~Graph();
    static std::unique_ptr<Graph> FromOnnx(const OnnxGraph& xgraph);
    OnnxGraph ToOnnx() const;  // fusion groups are expanded back into their nodes

    const std::string& name() const { return name_; }
    const std::vector<Value*>& input_values() const { return input_values_; }
    const std::vector<Value*>& output_values() const { return output_values_; }
    const std::vector<Node*>& nodes() const { return nodes_; }  // including detached ones, in creation order
    std::vector<Node*> GetLiveNodes() const;
    std::vector<Node*> GetTopologicallySortedNodes() const;  // live nodes; CHECK-fails on a cycle

    Value* AddValue(const std::string& name, const Type& type = Type(), Value::Kind kind = Value::kTemp);
    Value* AddInputValue(const std::string& name, const Type& type) { return AddValue(name, type, Value::kInput); }
    Value* AddOutputValue(const std::string& name, const Type& type) { return AddValue(name, type, Value::kOutput); }
    Value* AddNullValue() { return AddValue("", Type(), Value::kNull); }
    Node* AddNode(const std::string& op_type, const std::vector<Value*>& inputs, const std::vector<Value*>& outputs,
                  const std::string& base_name = "");
    void DetachNode(Node* node);
    // moves nodes and their temporary values into `to` (compiler/graph.cc MigrateNodes)
    void MigrateNodes(const std::vector<Node*>& nodes, const std::vector<Value*>& temps, Graph* to);
    std::string GenSym(const std::string& base);
    void CheckSanity(const std::string& where) const;
    std::string DebugString() const;

private:
    std::string name_;
    std::vector<std::unique_ptr<Value>> all_values_;
    std::vector<std::unique_ptr<Node>> all_nodes_;
    std::vector<Value*> input_values_, output_values_, temp_values_;
    std::vector<Node*> nodes_;
    std::map<std::string, int> ids_;
};

// compiler/graph_builder.h: adds nodes with generated value names next to a target value
class GraphBuilder {
public:
    GraphBuilder(Graph* graph, const std::string& category, Value* target);
    Value* Op(const std::string& op_type, const std::vector<Value*>& inputs, Value* output = nullptr);
    Node* MOp(const std::string& op_type, const std::vector<Value*>& inputs, const std::vector<Value*>& outputs);
    Value* Const(const Tensor& tensor);
    Value* Temp(const Type& type = Type());

private:
    Graph* graph_;
    std::string category_, target_name_;
};

// Element types of the values no ValueInfo speaks of, for the node types of this path: the 8-bit
// type of a quantizing op is that of its zero-point operand (uint8 without one), DequantizeLinear
// gives float32, the integer contractions int32, Cast its `to`, everything else its first operand's
// type; shapes where they follow from the operands alone (constants, reductions over everything,
// element-wise broadcasting).  The part of the reference's type inference
// (compiler/type_inference.cc) that the fusion rule and the program builder depend on.
void InferDtypes(Graph* graph);

// compiler/topology.cc:15-59
void ClassifyValues(const std::vector<Node*>& nodes, std::vector<Value*>* inputs, std::vector<Value*>* outputs, std::vector<Value*>* temps);

}  // namespace chainer_compiler
