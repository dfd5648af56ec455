// In / Out / Identity / Free / NullConstant and the constant ops
// (runtime/ops/generic.cc:38-60, runtime/ops/creation.cc:11-57 of the chainer-compiler tree).
#include "../gen/gen_chxvm_ops.h"

namespace chainer_compiler {
namespace runtime {

void InOp::RunImpl(ChxVMState* st) {
    st->Input(name, v);
}

void OutOp::RunImpl(ChxVMState* st) {
    st->Output(name, v);
}

void IdentityOp::RunImpl(ChxVMState* st) {
    st->SetVar(y, *st->GetVar(x));
}

void FreeOp::RunImpl(ChxVMState* st) {
    st->FreeVar(v);
}

void NullConstantOp::RunImpl(ChxVMState* st) {
    st->SetVar(output, ChxVMVar());
}

StrictScalar IntScalarConstantOp::RunImpl(ChxVMState* st) {
    return StrictScalar(static_cast<chainerx::Dtype>(dtype), chainerx::Scalar(static_cast<int64_t>(value)), host);
}

StrictScalar FloatScalarConstantOp::RunImpl(ChxVMState* st) {
    return StrictScalar(static_cast<chainerx::Dtype>(dtype), chainerx::Scalar(static_cast<double>(value)), host);
}

namespace {

// int64 / double host values -> device array of `dtype` (MakeArray(...).AsType(dtype))
template <class Src>
chainerx::Array MakeConstant(const std::vector<Src>& values, chainerx::Dtype dtype, const chainerx::Shape& shape) {
    CHECK_EQ(static_cast<int64_t>(values.size()), shape.GetTotalSize());
    const int64_t n = shape.GetTotalSize();
    std::vector<unsigned char> buf(static_cast<size_t>(n * chainerx::GetItemSize(dtype) + 8));
    for (int64_t i = 0; i < n; ++i) {
        unsigned char* p = buf.data() + i * chainerx::GetItemSize(dtype);
        switch (dtype) {
            case chainerx::Dtype::kBool: { uint8_t v = values[i] != 0; memcpy(p, &v, 1); } break;
            case chainerx::Dtype::kInt8: { int8_t v = static_cast<int8_t>(values[i]); memcpy(p, &v, 1); } break;
            case chainerx::Dtype::kUInt8: { uint8_t v = static_cast<uint8_t>(values[i]); memcpy(p, &v, 1); } break;
            case chainerx::Dtype::kInt16: { int16_t v = static_cast<int16_t>(values[i]); memcpy(p, &v, 2); } break;
            case chainerx::Dtype::kInt32: { int32_t v = static_cast<int32_t>(values[i]); memcpy(p, &v, 4); } break;
            case chainerx::Dtype::kInt64: { int64_t v = static_cast<int64_t>(values[i]); memcpy(p, &v, 8); } break;
            case chainerx::Dtype::kFloat32: { float v = static_cast<float>(values[i]); memcpy(p, &v, 4); } break;
            case chainerx::Dtype::kFloat64: { double v = static_cast<double>(values[i]); memcpy(p, &v, 8); } break;
            default: CHECK(false) << "constant of unsupported dtype " << dtype;
        }
    }
    return chainerx::FromHost(buf.data(), shape, dtype);
}

}  // namespace

class IntConstantOp::IntConstantImpl {
public:
    chainerx::Array cache;
};

void IntConstantOp::InitImpl() {
    impl_ = new IntConstantImpl();
    impl_->cache = MakeConstant(value, static_cast<chainerx::Dtype>(dtype), chainerx::Shape(shape.begin(), shape.end()));
}

IntConstantOp::~IntConstantOp() {
    delete impl_;
}

chainerx::Array IntConstantOp::RunImpl(ChxVMState* st) {
    return impl_->cache;
}

class FloatConstantOp::FloatConstantImpl {
public:
    chainerx::Array cache;
};

void FloatConstantOp::InitImpl() {
    impl_ = new FloatConstantImpl();
    impl_->cache = MakeConstant(value, static_cast<chainerx::Dtype>(dtype), chainerx::Shape(shape.begin(), shape.end()));
}

FloatConstantOp::~FloatConstantOp() {
    delete impl_;
}

chainerx::Array FloatConstantOp::RunImpl(ChxVMState* st) {
    return impl_->cache;
}

}  // namespace runtime
}  // namespace chainer_compiler
