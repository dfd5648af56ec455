// CHECK / CHECK_EQ ... with the reference's streaming syntax (common/log.h:31-44 of the
// chainer-compiler tree).  The reference prints and aborts; here a failed check throws
// chainer_compiler::CheckFailure so that an embedding host (and the test harness) gets the
// message back; the ChxVM loop adds the op's debug_info and rethrows, as runtime/chxvm.cc:184-190.
#pragma once

#include <sstream>
#include <stdexcept>
#include <string>

namespace chainer_compiler {

class CheckFailure : public std::runtime_error {
public:
    explicit CheckFailure(const std::string& what) : std::runtime_error(what) {
    }
};

class FailMessageStream {
public:
    FailMessageStream(const char* msg, const char* file, int line) {
        oss_ << msg << " at " << file << ":" << line << ": ";
    }
    [[noreturn]] ~FailMessageStream() noexcept(false) {
        throw CheckFailure(oss_.str());
    }
    template <class T>
    FailMessageStream& operator<<(const T& v) {
        oss_ << v;
        return *this;
    }

private:
    std::ostringstream oss_;
};

#define CHECK(cond) \
    while (!(cond)) ::chainer_compiler::FailMessageStream("Check `" #cond "' failed!", __FILE__, __LINE__)

#define CHECK_CMP(a, b, op) \
    while (!((a)op(b)))     \
    ::chainer_compiler::FailMessageStream("Check `" #a "' " #op " `" #b "' failed!", __FILE__, __LINE__) << "(" << (a) << " vs. " << (b) << ") "

#define CHECK_EQ(a, b) CHECK_CMP(a, b, ==)
#define CHECK_NE(a, b) CHECK_CMP(a, b, !=)
#define CHECK_LT(a, b) CHECK_CMP(a, b, <)
#define CHECK_LE(a, b) CHECK_CMP(a, b, <=)
#define CHECK_GT(a, b) CHECK_CMP(a, b, >)
#define CHECK_GE(a, b) CHECK_CMP(a, b, >=)

}  // namespace chainer_compiler
