#include "chxvm_proto.h"

#include <cstring>

#include "log.h"

namespace chainer_compiler {
namespace runtime {

namespace {

const char* const kOpNames[] = {
#include "gen/chxvm_op_table.inc"
};
constexpr int kNumOps = sizeof(kOpNames) / sizeof(kOpNames[0]);

// ---- writer ----
void PutVarint(std::string* out, uint64_t v) {
    while (v >= 0x80) {
        out->push_back(static_cast<char>((v & 0x7f) | 0x80));
        v >>= 7;
    }
    out->push_back(static_cast<char>(v));
}
void PutTag(std::string* out, int field, int wire) {
    PutVarint(out, static_cast<uint64_t>(field) << 3 | wire);
}
void PutInt(std::string* out, int field, int64_t v) {  // int32/int64/enum: sign-extended varint
    PutTag(out, field, 0);
    PutVarint(out, static_cast<uint64_t>(v));
}
void PutDouble(std::string* out, int field, double v) {
    PutTag(out, field, 1);
    char b[8];
    memcpy(b, &v, 8);
    out->append(b, 8);
}
void PutBytes(std::string* out, int field, const std::string& s) {
    PutTag(out, field, 2);
    PutVarint(out, s.size());
    out->append(s);
}

std::string Encode(const ChxVMValueProto& v) {
    std::string o;
    PutInt(&o, 1, v.type);
    // proto2 optional fields are written exactly when they are present
    if (v.has(2)) PutInt(&o, 2, v.array);
    if (v.has(3)) PutInt(&o, 3, v.i);
    if (v.has(4)) PutDouble(&o, 4, v.f);
    if (v.has(6)) PutBytes(&o, 6, v.s);
    if (v.has(8)) PutInt(&o, 8, v.sequence);
    if (v.has(11)) PutInt(&o, 11, v.opaque);
    if (v.has(12)) PutInt(&o, 12, v.shape);
    if (v.has(13)) PutInt(&o, 13, v.scalar);
    for (int64_t x : v.ints) PutInt(&o, 5, x);  // proto2 repeated scalars are not packed
    for (int32_t x : v.array_list) PutInt(&o, 7, x);
    for (double x : v.doubles) PutDouble(&o, 10, x);
    for (const std::string& x : v.strings) PutBytes(&o, 14, x);
    return o;
}

std::string Encode(const ChxVMTypeProto& t) {
    std::string o;
    if (t.has(1)) PutInt(&o, 1, t.dtype);
    for (int32_t x : t.shape) PutInt(&o, 2, x);
    return o;
}

std::string Encode(const ChxVMInstructionProto& in) {
    std::string o;
    PutInt(&o, 1, in.op);
    for (const auto& v : in.inputs) PutBytes(&o, 2, Encode(v));
    for (int32_t x : in.outputs) PutInt(&o, 3, x);
    if (in.has(4)) PutBytes(&o, 4, in.debug_info);
    if (in.has(5)) PutInt(&o, 5, in.id);
    for (const auto& t : in.output_types) PutBytes(&o, 6, Encode(t));
    for (const auto& n : in.output_names) PutBytes(&o, 7, n);
    if (in.has(8)) PutInt(&o, 8, in.flops);
    return o;
}

// ---- reader ----
struct Reader {
    const unsigned char* p;
    const unsigned char* end;
    bool done() const {
        return p >= end;
    }
    uint64_t Varint() {
        uint64_t v = 0;
        for (int shift = 0; shift < 70; shift += 7) {
            CHECK(p < end) << "truncated varint in ChxVM program";
            const unsigned char b = *p++;
            v |= static_cast<uint64_t>(b & 0x7f) << shift;
            if (!(b & 0x80)) return v;
        }
        CHECK(false) << "varint too long in ChxVM program";
        return 0;
    }
    double Fixed64() {
        CHECK(end - p >= 8) << "truncated fixed64 in ChxVM program";
        double d;
        memcpy(&d, p, 8);
        p += 8;
        return d;
    }
    Reader Sub() {
        const uint64_t n = Varint();
        CHECK(static_cast<uint64_t>(end - p) >= n) << "truncated length-delimited field in ChxVM program";
        Reader r{p, p + n};
        p += n;
        return r;
    }
    std::string Bytes() {
        Reader r = Sub();
        return std::string(reinterpret_cast<const char*>(r.p), r.end - r.p);
    }
    void Skip(int wire) {
        switch (wire) {
            case 0: Varint(); break;
            case 1: Fixed64(); break;
            case 2: Sub(); break;
            case 5:
                CHECK(end - p >= 4) << "truncated fixed32 in ChxVM program";
                p += 4;
                break;
            default: CHECK(false) << "unsupported wire type " << wire << " in ChxVM program";
        }
    }
};

// repeated scalar: accepts both the unpacked (one tag per element) and the packed encoding
template <class T, class F>
void ReadRepeated(Reader* r, int wire, int elem_wire, std::vector<T>* out, F one) {
    if (wire == 2 && elem_wire != 2) {
        Reader sub = r->Sub();
        while (!sub.done()) out->push_back(one(&sub));
    } else {
        CHECK_EQ(elem_wire, wire) << "unexpected wire type for a repeated field";
        out->push_back(one(r));
    }
}

ChxVMValueProto DecodeValue(Reader r) {
    ChxVMValueProto v;
    auto i64 = [](Reader* x) { return static_cast<int64_t>(x->Varint()); };
    auto i32 = [](Reader* x) { return static_cast<int32_t>(x->Varint()); };
    auto f64 = [](Reader* x) { return x->Fixed64(); };
    while (!r.done()) {
        const uint64_t tag = r.Varint();
        const int field = static_cast<int>(tag >> 3), wire = static_cast<int>(tag & 7);
        if (field >= 1 && field < 32) v.present |= 1u << field;
        switch (field) {
            case 1: v.type = static_cast<int>(r.Varint()); break;
            case 2: v.array = static_cast<int32_t>(r.Varint()); break;
            case 3: v.i = static_cast<int64_t>(r.Varint()); break;
            case 4: v.f = r.Fixed64(); break;
            case 5: ReadRepeated(&r, wire, 0, &v.ints, i64); break;
            case 6: v.s = r.Bytes(); break;
            case 7: ReadRepeated(&r, wire, 0, &v.array_list, i32); break;
            case 8: v.sequence = static_cast<int32_t>(r.Varint()); break;
            case 10: ReadRepeated(&r, wire, 1, &v.doubles, f64); break;
            case 11: v.opaque = static_cast<int32_t>(r.Varint()); break;
            case 12: v.shape = static_cast<int32_t>(r.Varint()); break;
            case 13: v.scalar = static_cast<int32_t>(r.Varint()); break;
            case 14: v.strings.push_back(r.Bytes()); break;
            default: r.Skip(wire);
        }
    }
    CHECK(v.has(1) && v.type >= 1 && v.type <= 16) << "ChxVMValueProto without a valid type";
    return v;
}

ChxVMTypeProto DecodeType(Reader r) {
    ChxVMTypeProto t;
    auto i32 = [](Reader* x) { return static_cast<int32_t>(x->Varint()); };
    while (!r.done()) {
        const uint64_t tag = r.Varint();
        const int field = static_cast<int>(tag >> 3), wire = static_cast<int>(tag & 7);
        if (field >= 1 && field < 32) t.present |= 1u << field;
        switch (field) {
            case 1: t.dtype = static_cast<int32_t>(r.Varint()); break;
            case 2: ReadRepeated(&r, wire, 0, &t.shape, i32); break;
            default: r.Skip(wire);
        }
    }
    return t;
}

ChxVMInstructionProto DecodeInstruction(Reader r) {
    ChxVMInstructionProto in;
    auto i32 = [](Reader* x) { return static_cast<int32_t>(x->Varint()); };
    while (!r.done()) {
        const uint64_t tag = r.Varint();
        const int field = static_cast<int>(tag >> 3), wire = static_cast<int>(tag & 7);
        if (field >= 1 && field < 32) in.present |= 1u << field;
        switch (field) {
            case 1: in.op = static_cast<int>(r.Varint()); break;
            case 2: in.inputs.push_back(DecodeValue(r.Sub())); break;
            case 3: ReadRepeated(&r, wire, 0, &in.outputs, i32); break;
            case 4: in.debug_info = r.Bytes(); break;
            case 5: in.id = static_cast<int64_t>(r.Varint()); break;
            case 6: in.output_types.push_back(DecodeType(r.Sub())); break;
            case 7: in.output_names.push_back(r.Bytes()); break;
            case 8: in.flops = static_cast<int64_t>(r.Varint()); break;
            default: r.Skip(wire);
        }
    }
    CHECK(in.has(1)) << "instruction without the required field `op`";
    CHECK(in.op >= 1 && in.op <= kNumOps) << "instruction with unknown op number " << in.op;
    return in;
}

}  // namespace

std::string ChxVMProgramProto::SerializeAsString() const {
    std::string o;
    for (const auto& in : instructions) PutBytes(&o, 1, Encode(in));
    for (const auto& n : input_names) PutBytes(&o, 2, n);
    for (const auto& t : input_types) PutBytes(&o, 3, Encode(t));
    return o;
}

ChxVMProgramProto ChxVMProgramProto::ParseFromString(const std::string& bytes) {
    ChxVMProgramProto prog;
    Reader r{reinterpret_cast<const unsigned char*>(bytes.data()),
             reinterpret_cast<const unsigned char*>(bytes.data()) + bytes.size()};
    while (!r.done()) {
        const uint64_t tag = r.Varint();
        const int field = static_cast<int>(tag >> 3), wire = static_cast<int>(tag & 7);
        switch (field) {
            case 1: prog.instructions.push_back(DecodeInstruction(r.Sub())); break;
            case 2: prog.input_names.push_back(r.Bytes()); break;
            case 3: prog.input_types.push_back(DecodeType(r.Sub())); break;
            default: r.Skip(wire);
        }
    }
    return prog;
}

const char* OpName(int op) {
    return op >= 1 && op <= kNumOps ? kOpNames[op - 1] : "?";
}

int OpNumber(const std::string& name) {
    for (int i = 0; i < kNumOps; ++i)
        if (name == kOpNames[i]) return i + 1;
    return -1;
}

int NumOps() {
    return kNumOps;
}

}  // namespace runtime
}  // namespace chainer_compiler
