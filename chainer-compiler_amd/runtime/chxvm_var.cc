#include "chxvm_var.h"

#include <sstream>

namespace chainer_compiler {
namespace runtime {

ChxVMVar::ChxVMVar() : val_(NullType()) {
}
ChxVMVar::ChxVMVar(chainerx::Array array) : val_(std::move(array)) {
}
ChxVMVar::ChxVMVar(ChxVMOpaque* opaque) : val_(std::shared_ptr<ChxVMOpaque>(opaque)) {
}
ChxVMVar::ChxVMVar(std::shared_ptr<ChxVMSequence> seq) : val_(std::move(seq)) {
}
ChxVMVar::ChxVMVar(chainerx::Shape shape) : val_(shape) {
}
ChxVMVar::ChxVMVar(StrictScalar scalar) : val_(scalar) {
}
ChxVMVar::ChxVMVar(const std::vector<std::string>& str) : val_(str) {
}

const chainerx::Array& ChxVMVar::GetArray() const {
    if (kind() == Kind::kScalar) {
        if (!scalar_as_array_) {
            const StrictScalar& s = std::get<StrictScalar>(val_);
            unsigned char buf[8] = {0};
            switch (s.dtype()) {
                case chainerx::Dtype::kBool: buf[0] = static_cast<bool>(s); break;
                case chainerx::Dtype::kInt8: { int8_t v = static_cast<int8_t>(static_cast<int64_t>(s)); memcpy(buf, &v, 1); } break;
                case chainerx::Dtype::kUInt8: { uint8_t v = static_cast<uint8_t>(static_cast<int64_t>(s)); memcpy(buf, &v, 1); } break;
                case chainerx::Dtype::kInt16: { int16_t v = static_cast<int16_t>(static_cast<int64_t>(s)); memcpy(buf, &v, 2); } break;
                case chainerx::Dtype::kInt32: { int32_t v = static_cast<int32_t>(static_cast<int64_t>(s)); memcpy(buf, &v, 4); } break;
                case chainerx::Dtype::kInt64: { int64_t v = static_cast<int64_t>(s); memcpy(buf, &v, 8); } break;
                case chainerx::Dtype::kFloat32: { float v = static_cast<float>(s); memcpy(buf, &v, 4); } break;
                case chainerx::Dtype::kFloat64: { double v = static_cast<double>(s); memcpy(buf, &v, 8); } break;
                default: CHECK(false) << "scalar of dtype " << s.dtype() << " cannot become an array";
            }
            scalar_as_array_ = std::make_shared<chainerx::Array>(chainerx::FromHost(buf, chainerx::Shape{}, s.dtype()));
        }
        return *scalar_as_array_;
    }
    CHECK_EQ(static_cast<int>(Kind::kArray), static_cast<int>(kind())) << "slot is not an array: " << ToString();
    return std::get<chainerx::Array>(val_);
}

const StrictScalar& ChxVMVar::GetScalar() const {
    if (kind() == Kind::kArray) {
        if (!array_as_scalar_) {
            const chainerx::Array& a = std::get<chainerx::Array>(val_);
            array_as_scalar_ = std::make_shared<StrictScalar>(a.dtype(), chainerx::AsScalar(a), false);
        }
        return *array_as_scalar_;
    }
    CHECK_EQ(static_cast<int>(Kind::kScalar), static_cast<int>(kind())) << "slot is not a scalar: " << ToString();
    return std::get<StrictScalar>(val_);
}

const chainerx::Shape& ChxVMVar::GetShape() const {
    if (kind() == Kind::kArray) {
        // a 1-D integer array read back as a shape (runtime/chxvm_var.cc:78-83, ArrayToShape)
        if (!array_as_shape_) {
            const chainerx::Array& a = std::get<chainerx::Array>(val_);
            CHECK_GE(1, a.ndim()) << "a shape operand must be a vector";
            CHECK(a.dtype() == chainerx::Dtype::kInt64 && a.IsContiguous()) << "a shape operand must be a contiguous int64 vector";
            std::vector<int64_t> host(a.GetTotalSize());
            if (!host.empty()) chainerx::ToHost(a, host.data());
            chainerx::Shape shape;
            for (int64_t d : host) shape.push_back(d);
            array_as_shape_ = std::make_shared<chainerx::Shape>(shape);
        }
        return *array_as_shape_;
    }
    CHECK_EQ(static_cast<int>(Kind::kShape), static_cast<int>(kind()));
    return std::get<chainerx::Shape>(val_);
}

ChxVMSequence* ChxVMVar::GetSequence() const {
    CHECK_EQ(static_cast<int>(Kind::kSequence), static_cast<int>(kind()));
    return std::get<std::shared_ptr<ChxVMSequence>>(val_).get();
}

ChxVMOpaque* ChxVMVar::GetOpaque() const {
    CHECK_EQ(static_cast<int>(Kind::kOpaque), static_cast<int>(kind()));
    return std::get<std::shared_ptr<ChxVMOpaque>>(val_).get();
}

int64_t ChxVMVar::GetNBytes() const {
    return kind() == Kind::kArray ? std::get<chainerx::Array>(val_).GetNBytes() : 0;
}

char ChxVMVar::Sigil() const {
    switch (kind()) {
        case Kind::kSequence: return '@';
        case Kind::kOpaque: return '*';
        default: return '$';
    }
}

std::string ChxVMVar::ToString() const {
    std::ostringstream oss;
    switch (kind()) {
        case Kind::kArray: {
            const chainerx::Array& a = std::get<chainerx::Array>(val_);
            oss << a.dtype() << a.shape();
        } break;
        case Kind::kScalar: oss << "scalar(" << std::get<StrictScalar>(val_).dtype() << ")"; break;
        case Kind::kShape: oss << "shape" << std::get<chainerx::Shape>(val_); break;
        case Kind::kSequence: oss << "[sequence]"; break;
        case Kind::kOpaque: oss << "(opaque)"; break;
        case Kind::kString: oss << "(strings)"; break;
        case Kind::kNull: oss << "(null)"; break;
    }
    return oss.str();
}

}  // namespace runtime
}  // namespace chainer_compiler
