// ChxVMProgramProto and its parts as plain structs, with a reader and writer of the protobuf
// wire format for exactly the messages of runtime/chxvm.proto.tmpl:1-65 (proto2) of the
// chainer-compiler tree, so that a program serialized by the reference's compiler
// (compiler/chxvm/emitter.cc) loads here and vice versa.  No protoc / libprotobuf involved.
// The op enum values come from the generated table (gen/chxvm_op_table.inc).
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace chainer_compiler {
namespace runtime {

struct ChxVMValueProto {
    enum Type {
        ARRAY = 1,
        OPTIONAL_ARRAY = 2,
        ARRAY_LIST = 3,
        SEQUENCE = 4,
        OPAQUE = 5,
        INT = 6,
        FLOAT = 7,
        INTS = 8,
        STRING = 9,
        LONGS = 10,
        DOUBLES = 11,
        INT_VALUES = 12,
        SHAPE = 13,
        SCALAR = 14,
        OPTIONAL_SCALAR = 15,
        STRINGS = 16,
    };
    int type = 0;                     // field 1 (required)
    int32_t array = 0;                // 2
    int64_t i = 0;                    // 3
    double f = 0;                     // 4
    std::vector<int64_t> ints;        // 5
    std::string s;                    // 6
    std::vector<int32_t> array_list;  // 7
    int32_t sequence = 0;             // 8
    std::vector<double> doubles;      // 10
    int32_t opaque = 0;               // 11
    int32_t shape = 0;                // 12
    int32_t scalar = 0;               // 13
    std::vector<std::string> strings; // 14

    // proto2 field presence of the optional fields: bit n = field number n was read or set
    uint32_t present = 0;
    bool has(int field) const { return (present >> field) & 1u; }
    void set_array(int32_t v) { array = v; present |= 1u << 2; }
    void set_i(int64_t v) { i = v; present |= 1u << 3; }
    void set_f(double v) { f = v; present |= 1u << 4; }
    void set_s(const std::string& v) { s = v; present |= 1u << 6; }
    void set_sequence(int32_t v) { sequence = v; present |= 1u << 8; }
    void set_opaque(int32_t v) { opaque = v; present |= 1u << 11; }
    void set_shape(int32_t v) { shape = v; present |= 1u << 12; }
    void set_scalar(int32_t v) { scalar = v; present |= 1u << 13; }
};

struct ChxVMTypeProto {
    int32_t dtype = 0;           // 1
    std::vector<int32_t> shape;  // 2

    uint32_t present = 0;
    bool has(int field) const { return (present >> field) & 1u; }
    void set_dtype(int32_t v) { dtype = v; present |= 1u << 1; }
};

struct ChxVMInstructionProto {
    int op = 0;                                 // 1 (required) enum Op
    std::vector<ChxVMValueProto> inputs;        // 2
    std::vector<int32_t> outputs;               // 3
    std::string debug_info;                     // 4
    int64_t id = 0;                             // 5
    std::vector<ChxVMTypeProto> output_types;   // 6
    std::vector<std::string> output_names;      // 7
    int64_t flops = 0;                          // 8

    uint32_t present = 0;
    bool has(int field) const { return (present >> field) & 1u; }
    void set_op(int v) { op = v; present |= 1u << 1; }
    void set_debug_info(const std::string& v) { debug_info = v; present |= 1u << 4; }
    void set_id(int64_t v) { id = v; present |= 1u << 5; }
    void set_flops(int64_t v) { flops = v; present |= 1u << 8; }
};

struct ChxVMProgramProto {
    std::vector<ChxVMInstructionProto> instructions;  // 1
    std::vector<std::string> input_names;             // 2
    std::vector<ChxVMTypeProto> input_types;          // 3

    std::string SerializeAsString() const;
    // Throws chainer_compiler::CheckFailure on malformed input.
    static ChxVMProgramProto ParseFromString(const std::string& bytes);
};

// Name <-> number of the op enum (1-based position in the op table).
const char* OpName(int op);  // "?" when out of range
int OpNumber(const std::string& name);  // -1 when unknown
int NumOps();

}  // namespace runtime
}  // namespace chainer_compiler
