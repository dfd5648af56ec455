// ChxVMVar: one variable slot of the VM (runtime/chxvm_var.h:38-95 of the chainer-compiler
// tree).  The kinds the quantized-inference path uses are implemented: array, scalar, shape,
// strings, null.  Sequence and opaque slots exist so that the op interface keeps its shape.
#pragma once

#include <memory>
#include <string>
#include <variant>
#include <vector>

#include "chainerx_lite.h"
#include "strict_scalar.h"

namespace chainer_compiler {
namespace runtime {

class ChxVMVar;
typedef std::vector<ChxVMVar> ChxVMSequence;

class ChxVMOpaque {
public:
    virtual ~ChxVMOpaque() = default;
    virtual std::string ToString() const {
        return "???";
    }
};

class ChxVMVar {
public:
    // Order matches the variant below (kind() is the variant index, as in the reference).
    enum class Kind { kArray, kSequence, kOpaque, kScalar, kShape, kString, kNull };

    ChxVMVar();
    explicit ChxVMVar(chainerx::Array array);
    explicit ChxVMVar(ChxVMOpaque* opaque);  // takes ownership
    explicit ChxVMVar(std::shared_ptr<ChxVMSequence> seq);
    explicit ChxVMVar(chainerx::Shape shape);
    explicit ChxVMVar(StrictScalar scalar);
    explicit ChxVMVar(const std::vector<std::string>& str);

    // A scalar slot is materialised as a 0-d device array on demand; an array slot of one
    // element is read back on demand (runtime/chxvm_var.cc:40-76).
    const chainerx::Array& GetArray() const;
    const StrictScalar& GetScalar() const;
    const chainerx::Shape& GetShape() const;
    ChxVMSequence* GetSequence() const;
    ChxVMOpaque* GetOpaque() const;

    Kind kind() const {
        return static_cast<Kind>(val_.index());
    }
    bool IsNull() const {
        return kind() == Kind::kNull;
    }
    bool IsArray() const {
        return kind() == Kind::kArray || kind() == Kind::kScalar;
    }
    int64_t GetNBytes() const;
    char Sigil() const;
    std::string ToString() const;
    std::string DebugString() const {
        return ToString();
    }

private:
    struct NullType {};
    using VarInternalType = std::variant<chainerx::Array, std::shared_ptr<ChxVMSequence>, std::shared_ptr<ChxVMOpaque>,
                                         StrictScalar, chainerx::Shape, std::vector<std::string>, NullType>;
    mutable VarInternalType val_;
    mutable std::shared_ptr<chainerx::Array> scalar_as_array_;
    mutable std::shared_ptr<StrictScalar> array_as_scalar_;
    mutable std::shared_ptr<chainerx::Shape> array_as_shape_;
};

}  // namespace runtime
}  // namespace chainer_compiler
