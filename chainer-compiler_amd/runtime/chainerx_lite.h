// The slice of ChainerX's C++ interface that the ChxVM op layer of the quantized-inference
// path touches, so that the RunImpl signatures compile as they are written in the reference
// (runtime/gen_chxvm.py:57-126): chainerx::Array / Shape / Strides / Dtype / Scalar /
// StackVector and absl::optional.  ChainerX itself is not part of the chainer-compiler tree.
//
// An Array is a ref-counted handle on device memory (copy = shared body, as in ChainerX) with a
// dtype, a shape and BYTE strides; views with arbitrary strides are ordinary arrays.  Device
// memory is obtained through the C ABI (chx_hip_malloc / chx_hip_free), never from HIP directly.
#pragma once

#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <memory>
#include <optional>
#include <ostream>
#include <vector>

#include <chx_hip.h>

#include "log.h"

namespace absl {
using std::nullopt;
using std::optional;
}  // namespace absl

namespace chainerx {

constexpr int8_t kMaxNdim = CHX_HIP_MAX_NDIM;

enum class Dtype : int {
    kBool = 1,
    kInt8,
    kInt16,
    kInt32,
    kInt64,
    kUInt8,
    kFloat16,
    kFloat32,
    kFloat64,
};

inline int64_t GetItemSize(Dtype dt) {
    switch (dt) {
        case Dtype::kBool:
        case Dtype::kInt8:
        case Dtype::kUInt8:
            return 1;
        case Dtype::kInt16:
        case Dtype::kFloat16:
            return 2;
        case Dtype::kInt32:
        case Dtype::kFloat32:
            return 4;
        case Dtype::kInt64:
        case Dtype::kFloat64:
            return 8;
    }
    CHECK(false) << "unknown dtype " << static_cast<int>(dt);
}

inline const char* GetDtypeName(Dtype dt) {
    static const char* names[] = {"?", "bool", "int8", "int16", "int32", "int64", "uint8", "float16", "float32", "float64"};
    const int i = static_cast<int>(dt);
    return i >= 1 && i <= 9 ? names[i] : "?";
}

inline std::ostream& operator<<(std::ostream& os, Dtype dt) {
    return os << GetDtypeName(dt);
}

enum class DtypeKind { kBool, kInt, kUInt, kFloat };

inline DtypeKind GetKind(Dtype dt) {
    switch (dt) {
        case Dtype::kBool:
            return DtypeKind::kBool;
        case Dtype::kUInt8:
            return DtypeKind::kUInt;
        case Dtype::kFloat16:
        case Dtype::kFloat32:
        case Dtype::kFloat64:
            return DtypeKind::kFloat;
        default:
            return DtypeKind::kInt;
    }
}

template <typename T, int8_t N>
class StackVector {
public:
    StackVector() = default;
    StackVector(std::initializer_list<T> l) {
        for (const T& v : l) push_back(v);
    }
    template <typename It>
    StackVector(It first, It last) {
        for (; first != last; ++first) push_back(static_cast<T>(*first));
    }
    void push_back(const T& v) {
        CHECK_LT(size_, N) << "StackVector overflow";
        d_[size_++] = v;
    }
    size_t size() const {
        return size_;
    }
    bool empty() const {
        return size_ == 0;
    }
    void resize(size_t n) {
        CHECK_LE(n, static_cast<size_t>(N));
        for (size_t i = size_; i < n; ++i) d_[i] = T();
        size_ = static_cast<int8_t>(n);
    }
    T& operator[](size_t i) {
        return d_[i];
    }
    const T& operator[](size_t i) const {
        return d_[i];
    }
    T* begin() {
        return d_;
    }
    T* end() {
        return d_ + size_;
    }
    const T* begin() const {
        return d_;
    }
    const T* end() const {
        return d_ + size_;
    }
    bool operator==(const StackVector& o) const {
        if (size_ != o.size_) return false;
        for (int i = 0; i < size_; ++i)
            if (!(d_[i] == o.d_[i])) return false;
        return true;
    }
    bool operator!=(const StackVector& o) const {
        return !(*this == o);
    }

private:
    T d_[N] = {};
    int8_t size_ = 0;
};

class Shape : public StackVector<int64_t, kMaxNdim> {
public:
    using StackVector::StackVector;
    int64_t GetTotalSize() const {
        int64_t n = 1;
        for (int64_t v : *this) n *= v;
        return n;
    }
    int8_t ndim() const {
        return static_cast<int8_t>(size());
    }
};

using Strides = StackVector<int64_t, kMaxNdim>;

inline std::ostream& operator<<(std::ostream& os, const Shape& s) {
    os << "(";
    for (size_t i = 0; i < s.size(); ++i) os << (i ? ", " : "") << s[i];
    return os << ")";
}

// chainerx::Scalar: a tagged host value.
class Scalar {
public:
    Scalar() : Scalar(int64_t(0)) {
    }
    Scalar(bool v) : kind_(DtypeKind::kBool), i_(v), f_(v) {
    }
    Scalar(int v) : Scalar(int64_t(v)) {
    }
    Scalar(unsigned v) : Scalar(int64_t(v)) {
    }
    Scalar(int64_t v) : kind_(DtypeKind::kInt), i_(v), f_(static_cast<double>(v)) {
    }
    Scalar(float v) : Scalar(double(v)) {
    }
    Scalar(double v) : kind_(DtypeKind::kFloat), i_(static_cast<int64_t>(v)), f_(v) {
    }
    DtypeKind kind() const {
        return kind_;
    }
    explicit operator bool() const {
        return kind_ == DtypeKind::kFloat ? f_ != 0 : i_ != 0;
    }
    explicit operator int64_t() const {
        return kind_ == DtypeKind::kFloat ? static_cast<int64_t>(f_) : i_;
    }
    explicit operator int() const {
        return static_cast<int>(static_cast<int64_t>(*this));
    }
    explicit operator double() const {
        return kind_ == DtypeKind::kFloat ? f_ : static_cast<double>(i_);
    }
    explicit operator float() const {
        return static_cast<float>(static_cast<double>(*this));
    }

private:
    DtypeKind kind_;
    int64_t i_;
    double f_;
};

class Array {
public:
    Array() = default;  // null handle

    bool IsNullHandle() const {
        return !body_;
    }
    Dtype dtype() const {
        return body_->dtype;
    }
    const Shape& shape() const {
        return body_->shape;
    }
    const Strides& strides() const {
        return body_->strides;
    }
    int8_t ndim() const {
        return body_->shape.ndim();
    }
    int64_t GetTotalSize() const {
        return body_->shape.GetTotalSize();
    }
    int64_t GetItemSize() const {
        return chainerx::GetItemSize(body_->dtype);
    }
    int64_t GetNBytes() const {
        return GetTotalSize() * GetItemSize();
    }
    void* raw_data() const {
        return body_->data.get();
    }
    int64_t offset() const {
        return body_->offset;
    }
    bool IsContiguous() const {
        int64_t expect = GetItemSize();
        for (int i = ndim() - 1; i >= 0; --i) {
            if (shape()[i] != 1 && strides()[i] != expect) return false;
            expect *= shape()[i];
        }
        return true;
    }
    // A view with permuted axes (no data movement), as chainerx::Array::Transpose.
    Array Transpose(std::initializer_list<int> perm) const {
        return Transpose(std::vector<int>(perm));
    }
    Array Transpose(const std::vector<int>& perm) const {
        Array r;
        r.body_ = std::make_shared<Body>(*body_);
        r.body_->shape = Shape();
        r.body_->strides = Strides();
        for (int ax : perm) {
            r.body_->shape.push_back(body_->shape[ax]);
            r.body_->strides.push_back(body_->strides[ax]);
        }
        return r;
    }

    // A view of `length` positions of one axis from `start` on (no data movement).
    Array Narrow(int axis, int64_t start, int64_t length) const {
        Array r;
        r.body_ = std::make_shared<Body>(*body_);
        r.body_->offset = body_->offset + start * body_->strides[axis];
        r.body_->shape[axis] = length;
        return r;
    }

    // A view of a contiguous array with another shape of the same size.
    Array Reshape(const Shape& to) const;

    // chx_hip_tensor of this array (ChainerX strides are bytes already).
    chx_hip_tensor hip() const {
        chx_hip_tensor t;
        memset(&t, 0, sizeof(t));
        t.data = static_cast<char*>(raw_data()) + offset();
        t.dtype = static_cast<int32_t>(dtype());
        t.ndim = ndim();
        for (int i = 0; i < ndim(); ++i) {
            t.shape[i] = shape()[i];
            t.strides[i] = strides()[i];
        }
        return t;
    }

    static Array MakeOwned(std::shared_ptr<void> data, Dtype dtype, const Shape& shape, const Strides& strides) {
        Array a;
        a.body_ = std::make_shared<Body>();
        a.body_->data = std::move(data);
        a.body_->dtype = dtype;
        a.body_->shape = shape;
        a.body_->strides = strides;
        return a;
    }

    // An array over memory that the caller of the runtime keeps alive and may rewrite or release between
    // runs.  Views of it (Transpose, Reshape) are borrowed as well.  Anything derived from its contents and
    // kept beyond the instruction that reads it would go stale.
    static Array MakeBorrowed(void* data, Dtype dtype, const Shape& shape, const Strides& strides) {
        Array a = MakeOwned(std::shared_ptr<void>(data, [](void*) {}), dtype, shape, strides);
        a.body_->borrowed = true;
        return a;
    }
    bool IsBorrowed() const {
        return body_->borrowed;
    }

private:
    struct Body {
        std::shared_ptr<void> data;
        int64_t offset = 0;
        bool borrowed = false;
        Dtype dtype = Dtype::kFloat32;
        Shape shape;
        Strides strides;
    };
    std::shared_ptr<Body> body_;
};

#define CHXVM_HIP_CALL(expr) CHECK_EQ(0, (expr)) << chx_hip_last_error()

inline Strides ContiguousStrides(const Shape& shape, int64_t item_size) {
    Strides s;
    s.resize(shape.size());
    int64_t acc = item_size;
    for (int i = static_cast<int>(shape.size()) - 1; i >= 0; --i) {
        s[i] = acc;
        acc *= shape[i];
    }
    return s;
}

// Where the arrays of the calling thread come from and which stream its kernels go to.  The default is the
// device runtime's allocator and the null stream, the counterpart of ChainerX's default device.  A run that is
// to be captured into a graph installs a pool of its own (no allocation by the device runtime may happen while
// a stream records) and the stream that records.
class DeviceAllocator {
public:
    virtual ~DeviceAllocator() = default;
    // memory of at least `bytes` bytes that stays valid until the returned handle is released
    virtual std::shared_ptr<void> Allocate(size_t bytes) = 0;
};

struct DeviceContext {
    void* stream = nullptr;
    DeviceAllocator* allocator = nullptr;
};

inline DeviceContext& CurrentDeviceContext() {
    thread_local DeviceContext context;
    return context;
}

inline void* CurrentStream() {
    return CurrentDeviceContext().stream;
}

// Installs a context for the lifetime of the object (one run of a program).
class DeviceContextScope {
public:
    DeviceContextScope(void* stream, DeviceAllocator* allocator) : saved_(CurrentDeviceContext()) {
        CurrentDeviceContext().stream = stream;
        CurrentDeviceContext().allocator = allocator;
    }
    ~DeviceContextScope() {
        CurrentDeviceContext() = saved_;
    }
    DeviceContextScope(const DeviceContextScope&) = delete;
    DeviceContextScope& operator=(const DeviceContextScope&) = delete;

private:
    DeviceContext saved_;
};

// chainerx::Empty on the HIP device: C-contiguous.
inline Array Empty(const Shape& shape, Dtype dtype) {
    const int64_t bytes = shape.GetTotalSize() * GetItemSize(dtype);
    const size_t want = static_cast<size_t>(bytes > 0 ? bytes : 1);
    std::shared_ptr<void> data;
    if (DeviceAllocator* allocator = CurrentDeviceContext().allocator) {
        data = allocator->Allocate(want);
    } else {
        void* p = nullptr;
        CHXVM_HIP_CALL(chx_hip_malloc(&p, want));
        data = std::shared_ptr<void>(p, [](void* q) { (void)chx_hip_free(q); });
    }
    return Array::MakeOwned(std::move(data), dtype, shape, ContiguousStrides(shape, GetItemSize(dtype)));
}

// [N,C,H,W]-shaped array over channels-last memory: the layout the convolution kernels
// read and write without a transposition.
inline Array EmptyChannelsLast(const Shape& nchw, Dtype dtype) {
    CHECK_EQ(4, nchw.size());
    Array nhwc = Empty(Shape{nchw[0], nchw[2], nchw[3], nchw[1]}, dtype);
    return nhwc.Transpose({0, 3, 1, 2});
}

// The same with the pixel pitch rounded up to 16 bytes (8-bit arrays): every pixel is then a whole
// number of aligned 16-byte vectors, which the convolution kernels need, also for C = 24.
inline Array EmptyChannelsLastPadded(const Shape& nchw, Dtype dtype) {
    CHECK_EQ(4, nchw.size());
    const int64_t es = GetItemSize(dtype);
    const int64_t pitch = (nchw[1] * es + 15) / 16 * 16;
    if (pitch == nchw[1] * es) return EmptyChannelsLast(nchw, dtype);
    Array flat = Empty(Shape{nchw[0] * nchw[2] * nchw[3] * pitch}, Dtype::kUInt8);
    std::shared_ptr<void> keep(flat.raw_data(), [flat](void*) {});  // shares the allocation
    return Array::MakeOwned(keep, dtype, nchw, Strides{nchw[2] * nchw[3] * pitch, es, nchw[3] * pitch, pitch});
}

inline Array FromHost(const void* src, const Shape& shape, Dtype dtype) {
    Array a = Empty(shape, dtype);
    CHXVM_HIP_CALL(chx_hip_memcpy_h2d(a.raw_data(), src, static_cast<size_t>(a.GetNBytes()), chainerx::CurrentStream()));
    return a;
}

// Synchronizing read of a contiguous array.
inline Array Array::Reshape(const Shape& to) const {
    CHECK(IsContiguous());
    Array r;
    r.body_ = std::make_shared<Body>(*body_);
    r.body_->shape = to;
    r.body_->strides = ContiguousStrides(to, GetItemSize());
    return r;
}

inline void ToHost(const Array& a, void* dst) {
    CHECK(a.IsContiguous()) << "ToHost needs a contiguous array";
    CHXVM_HIP_CALL(chx_hip_memcpy_d2h(dst, static_cast<char*>(a.raw_data()) + a.offset(), static_cast<size_t>(a.GetNBytes()), chainerx::CurrentStream()));
}

// chainerx::AsScalar: the single element of an array, read back to the host (a stream
// synchronization, as in the reference: runtime/chxvm_var.cc:70-76).
inline Scalar AsScalar(const Array& a) {
    CHECK_EQ(1, a.GetTotalSize()) << "AsScalar needs exactly one element";
    unsigned char buf[8] = {0};
    CHXVM_HIP_CALL(chx_hip_memcpy_d2h(buf, static_cast<char*>(a.raw_data()) + a.offset(), static_cast<size_t>(a.GetItemSize()), chainerx::CurrentStream()));
    switch (a.dtype()) {
        case Dtype::kBool: return Scalar(buf[0] != 0);
        case Dtype::kInt8: return Scalar(int64_t(*reinterpret_cast<int8_t*>(buf)));
        case Dtype::kUInt8: return Scalar(int64_t(buf[0]));
        case Dtype::kInt16: { int16_t v; memcpy(&v, buf, 2); return Scalar(int64_t(v)); }
        case Dtype::kInt32: { int32_t v; memcpy(&v, buf, 4); return Scalar(int64_t(v)); }
        case Dtype::kInt64: { int64_t v; memcpy(&v, buf, 8); return Scalar(v); }
        case Dtype::kFloat32: { float v; memcpy(&v, buf, 4); return Scalar(double(v)); }
        case Dtype::kFloat64: { double v; memcpy(&v, buf, 8); return Scalar(v); }
        default: CHECK(false) << "AsScalar: unsupported dtype " << a.dtype();
    }
    return Scalar();
}

namespace internal {
// numpy broadcasting of two shapes (chainerx::internal::BroadcastShapes)
inline Shape BroadcastShapes(const Shape& a, const Shape& b) {
    const size_t nd = a.size() > b.size() ? a.size() : b.size();
    Shape r;
    r.resize(nd);
    for (size_t i = 0; i < nd; ++i) {
        const int64_t da = i + a.size() >= nd ? a[i + a.size() - nd] : 1;
        const int64_t db = i + b.size() >= nd ? b[i + b.size() - nd] : 1;
        CHECK(da == db || da == 1 || db == 1) << "shapes " << a << " and " << b << " do not broadcast";
        r[i] = da == 1 ? db : da;
    }
    return r;
}
}  // namespace internal

}  // namespace chainerx
