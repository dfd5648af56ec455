// The ONNX messages the compiler side reads and writes (ModelProto / GraphProto / NodeProto /
// AttributeProto / TensorProto / ValueInfoProto, field numbers of onnx.proto), as plain structs with
// a reader and a writer of the protobuf wire format.  The reference links the onnx package for this
// (compiler/graph.cc, compiler/node.cc, compiler/tensor.cc of the chainer-compiler tree); no
// protobuf library is involved here.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace chainer_compiler {

// TensorProto.DataType
enum OnnxDtype { kOnnxFloat = 1, kOnnxUInt8 = 2, kOnnxInt8 = 3, kOnnxInt32 = 6, kOnnxInt64 = 7, kOnnxBool = 9, kOnnxDouble = 11 };

int OnnxElementSize(int dtype);  // 0 for unsupported types

struct OnnxTensor {
    std::string name;
    int dtype = kOnnxFloat;
    std::vector<int64_t> dims;
    std::string raw;  // little-endian elements of `dtype`, whatever field carried them
    int64_t NumElements() const;
};

struct OnnxAttr {
    enum Type { kFloat = 1, kInt = 2, kString = 3, kTensor = 4, kFloats = 6, kInts = 7 };
    std::string name;
    int type = 0;
    float f = 0;
    int64_t i = 0;
    std::string s;
    OnnxTensor t;
    std::vector<float> floats;
    std::vector<int64_t> ints;
};

struct OnnxNode {
    std::string op_type, name, domain;
    std::vector<std::string> inputs, outputs;
    std::vector<OnnxAttr> attrs;
};

struct OnnxValueInfo {
    std::string name;
    int elem_type = 0;          // 0: unknown
    std::vector<int64_t> dims;  // -1: symbolic or unknown
    bool has_shape = false;
};

struct OnnxGraph {
    std::string name;
    std::vector<OnnxNode> nodes;
    std::vector<OnnxTensor> initializers;
    std::vector<OnnxValueInfo> inputs, outputs, value_info;
};

struct OnnxModel {
    int64_t ir_version = 5;
    int64_t opset = 10;
    std::string producer;
    OnnxGraph graph;
};

OnnxModel ParseOnnxModel(const std::string& bytes);   // CHECK-fails on malformed input
std::string SerializeOnnxModel(const OnnxModel& model);
OnnxTensor ParseOnnxTensor(const std::string& bytes);
std::string SerializeOnnxTensor(const OnnxTensor& tensor);

}  // namespace chainer_compiler
