// Fused element-wise chains (the FusionGroup kernels).
//
// The reference lowers a FusionGroup on the GPU by generating CUDA source at compile
// time (compiler/nvrtc_builder.cc:91-206), compiling it with NVRTC on first use and
// launching one thread per element over inputs that were first broadcast and copied
// (runtime/ops/nvrtc.cc:90-161).  Here the FusionGroup travels as a small SSA program
// text; the HIP source is generated at run time, when the operand layouts are known,
// so that
//   - broadcast operands are read through their strides (a [1024] vector against a
//     [64,1024,1024] tensor costs 4 KiB of traffic, not 256 MiB),
//   - every full-size operand moves in 128-bit accesses,
//   - the arithmetic is the CPU path's: one IEEE operation per node in topological
//     order, no contraction, tanh/exp as the host C library computes them
//     (faithful_math.h), sigmoid as 1/(1+exp(-x)).
// Compiled code objects are cached by generated source text; loaded kernels by the
// same key (the reference's two-level cache, runtime/ops/nvrtc.cc:41-84, here under a
// mutex).
//
// Program text (one statement per line, '#' starts a comment):
//   chxhip-fusion 1
//   in  <name>:<dtype> ...            dtype: float32 | float16 | float64 | uint8 | int8
//   <name> = <Op> <operand> ...       operands are earlier names or, where noted, literals
//   out <name>:<dtype> ...
// Ops: Identity a | Neg a | Abs a | Floor a | Round a | Add a b | Sub a b | Mul a b | Div a b | Max a b | Min a b
//      Tanh a | Sigmoid a | Exp a | Relu a | Clip a <lo> <hi> | Const <value>
//      QuantizeLinear a <scale> <zero_point> <uint8|int8> [rne]   (float -> 8-bit code)
//      DequantizeLinear q <scale> <zero_point>                    (8-bit code -> float)
// Float literals are decimal or 0x######## (the bit pattern of the float32).
// The arithmetic type of a program is that of its floating-point ports (one type per program, as the reference's
// `typedef ... T`, compiler/nvrtc_builder.cc:118-127): float32; float16, where every node computes in float32 and
// rounds to float16 (what a half-precision operation is); or float64.  The 8-bit ops go with float32 only, and only
// float32 programs have the vector kernel; the other two types run on the general kernel.
//
// The CUDA C text that the reference's compiler emits for a group (BuildNvrtcProgram, nvrtc_builder.cc:91-206) is
// accepted as well and turned into the same internal program: `typedef half|float|double T;`, the kernel's
// parameters `T* i_<name>` / `T* o_<name>`, one `const T <name> = <expression>;` per node (a + b, a - b, a * b,
// a / b, tanh(a), exp(a), sigmoid(a), a, or a number) and `o_<name>[tid] = <name>;` per output.  Its sigmoid is the
// helper that text defines, tanh(x * 0.5) * 0.5 + 0.5, one rounding per operation.
#include <hip/hiprtc.h>

#include <cmath>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "chx_internal.h"

namespace chx {
namespace {

const char* kFaithfulMathText =
#include "faithful_math_text.inc"
        ;

struct Stmt {
    std::string out, op;
    std::vector<std::string> args;
};

struct Port {
    std::string name;
    int32_t dtype;
};

struct Program {
    std::vector<Port> inputs, outputs;
    std::vector<Stmt> stmts;
    int32_t arith = CHX_HIP_FLOAT32;  // type of the floating-point values: float32, float16 or float64
};

bool is_float_dtype(int32_t dt) {
    return dt == CHX_HIP_FLOAT32 || dt == CHX_HIP_FLOAT16 || dt == CHX_HIP_FLOAT64;
}

bool parse_dtype(const std::string& s, int32_t* dt) {
    if (s == "float32") *dt = CHX_HIP_FLOAT32;
    else if (s == "float16") *dt = CHX_HIP_FLOAT16;
    else if (s == "float64") *dt = CHX_HIP_FLOAT64;
    else if (s == "uint8") *dt = CHX_HIP_UINT8;
    else if (s == "int8") *dt = CHX_HIP_INT8;
    else return false;
    return true;
}

std::vector<std::string> split_ws(const std::string& line) {
    std::vector<std::string> out;
    std::istringstream iss(line);
    std::string tok;
    while (iss >> tok) out.push_back(tok);
    return out;
}

int parse_port(const std::string& tok, Port* p) {
    const size_t c = tok.find(':');
    CHX_REQUIRE(c != std::string::npos, "fusion program: expected name:dtype, got '%s'", tok.c_str());
    p->name = tok.substr(0, c);
    CHX_REQUIRE(parse_dtype(tok.substr(c + 1), &p->dtype), "fusion program: unsupported dtype in '%s'", tok.c_str());
    return CHX_HIP_OK;
}

int parse_nvrtc_source(const char* code, Program* prog);

// One floating-point type per program; 8-bit ports only beside float32.
int settle_arithmetic_type(Program* prog) {
    int32_t arith = 0;
    bool any8 = false;
    auto see = [&](const Port& p) -> int {
        if (!is_float_dtype(p.dtype)) {
            any8 = true;
            return CHX_HIP_OK;
        }
        CHX_REQUIRE(arith == 0 || arith == p.dtype, "fusion program: ports of two floating-point types (%s and %s)", dtype_name(arith),
                    dtype_name(p.dtype));
        arith = p.dtype;
        return CHX_HIP_OK;
    };
    for (const Port& p : prog->inputs) CHX_PROPAGATE(see(p));
    for (const Port& p : prog->outputs) CHX_PROPAGATE(see(p));
    prog->arith = arith ? arith : CHX_HIP_FLOAT32;
    CHX_REQUIRE(!any8 || prog->arith == CHX_HIP_FLOAT32, "fusion program: 8-bit ports go with float32 arithmetic, not %s", dtype_name(prog->arith));
    return CHX_HIP_OK;
}

int parse_program(const char* code, Program* prog) {
    CHX_REQUIRE(code != nullptr, "fusion program: null code");
    if (strstr(code, "__global__") != nullptr && strstr(code, "typedef") != nullptr) return parse_nvrtc_source(code, prog);
    std::istringstream iss(code);
    std::string line;
    bool header = false;
    while (std::getline(iss, line)) {
        const size_t hash = line.find('#');
        if (hash != std::string::npos) line.resize(hash);
        std::vector<std::string> t = split_ws(line);
        if (t.empty()) continue;
        if (!header) {
            CHX_REQUIRE(t.size() == 2 && t[0] == "chxhip-fusion" && t[1] == "1",
                        "fusion program: missing 'chxhip-fusion 1' header (is this NVRTC source?)");
            header = true;
            continue;
        }
        if (t[0] == "in" || t[0] == "out") {
            for (size_t i = 1; i < t.size(); ++i) {
                Port p;
                CHX_PROPAGATE(parse_port(t[i], &p));
                (t[0] == "in" ? prog->inputs : prog->outputs).push_back(p);
            }
            continue;
        }
        CHX_REQUIRE(t.size() >= 3 && t[1] == "=", "fusion program: cannot parse statement '%s'", line.c_str());
        Stmt s;
        s.out = t[0];
        s.op = t[2];
        s.args.assign(t.begin() + 3, t.end());
        prog->stmts.push_back(s);
    }
    CHX_REQUIRE(header, "fusion program: empty");
    CHX_REQUIRE(!prog->inputs.empty(), "fusion program: no inputs");
    CHX_REQUIRE(!prog->outputs.empty(), "fusion program: no outputs");
    return settle_arithmetic_type(prog);
}

std::string trimmed(const std::string& s) {
    size_t a = 0, b = s.size();
    while (a < b && isspace((unsigned char)s[a])) ++a;
    while (b > a && isspace((unsigned char)s[b - 1])) --b;
    return s.substr(a, b - a);
}

bool is_identifier(const std::string& s) {
    if (s.empty() || !(isalpha((unsigned char)s[0]) || s[0] == '_')) return false;
    for (char c : s)
        if (!(isalnum((unsigned char)c) || c == '_')) return false;
    return true;
}

// The CUDA C text of BuildNvrtcProgram (compiler/nvrtc_builder.cc:91-206).  Port names are the variables the kernel
// loads its inputs into / stores its outputs from; inputs and outputs keep the order of the kernel's parameters,
// which is the order the op hands its arrays over in (runtime/ops/nvrtc.cc:134-150).
int parse_nvrtc_source(const char* code, Program* prog) {
    std::vector<std::string> lines;
    {
        std::istringstream iss(code);
        std::string line;
        while (std::getline(iss, line)) {
            const size_t c = line.find("//");
            if (c != std::string::npos) line.resize(c);
            line = trimmed(line);
            if (!line.empty()) lines.push_back(line);
        }
    }
    int32_t arith = 0;
    size_t i = 0;
    for (; i < lines.size(); ++i) {
        if (lines[i].compare(0, 8, "typedef ") != 0) continue;
        const std::vector<std::string> t = split_ws(lines[i]);
        CHX_REQUIRE(t.size() == 3 && t[2] == "T;", "fusion source: expected 'typedef <type> T;', got '%s'", lines[i].c_str());
        if (t[1] == "half") arith = CHX_HIP_FLOAT16;
        else if (t[1] == "float") arith = CHX_HIP_FLOAT32;
        else if (t[1] == "double") arith = CHX_HIP_FLOAT64;
        else CHX_FAIL(CHX_HIP_EUNSUPPORTED, "fusion source: element type '%s' (half, float or double expected)", t[1].c_str());
        ++i;
        break;
    }
    CHX_REQUIRE(arith != 0, "fusion source: no 'typedef ... T;'");
    // the sigmoid helper, when the group has one
    if (i < lines.size() && lines[i].compare(0, 10, "__device__") == 0) {
        CHX_REQUIRE(lines[i].find("T sigmoid(T x)") != std::string::npos, "fusion source: unknown helper '%s'", lines[i].c_str());
        bool body = false;
        for (++i; i < lines.size() && lines[i] != "}"; ++i)
            if (lines[i].find("tanh(x * half) * half + half") != std::string::npos) body = true;
        CHX_REQUIRE(body && i < lines.size(), "fusion source: the sigmoid helper is not tanh(x * half) * half + half");
        ++i;
    }
    // extern "C" __global__ / void fusionN(size_t n, T* i_a, ..., T* o_y) {
    std::string sig;
    for (; i < lines.size(); ++i) {
        if (lines[i].compare(0, 5, "void ") == 0) {
            sig = lines[i++];
            break;
        }
        CHX_REQUIRE(lines[i].find("__global__") != std::string::npos, "fusion source: unexpected line '%s' in front of the kernel", lines[i].c_str());
    }
    const size_t lp = sig.find('('), rp = sig.rfind(')');
    CHX_REQUIRE(!sig.empty() && lp != std::string::npos && rp != std::string::npos && rp > lp, "fusion source: no kernel signature");
    std::vector<std::string> in_params, out_params;
    {
        std::istringstream ps(sig.substr(lp + 1, rp - lp - 1));
        std::string param;
        bool first = true;
        while (std::getline(ps, param, ',')) {
            param = trimmed(param);
            if (first) {
                CHX_REQUIRE(param == "size_t n", "fusion source: the first kernel parameter is '%s', not 'size_t n'", param.c_str());
                first = false;
                continue;
            }
            CHX_REQUIRE(param.compare(0, 3, "T* ") == 0, "fusion source: kernel parameter '%s' is not a T*", param.c_str());
            const std::string name = trimmed(param.substr(3));
            if (name.compare(0, 2, "i_") == 0) in_params.push_back(name);
            else if (name.compare(0, 2, "o_") == 0) out_params.push_back(name);
            else CHX_FAIL(CHX_HIP_EINVAL, "fusion source: kernel parameter '%s' is neither an input (i_) nor an output (o_)", name.c_str());
        }
    }
    CHX_REQUIRE(!in_params.empty() && !out_params.empty(), "fusion source: the kernel needs inputs and outputs");
    std::vector<std::string> in_var(in_params.size()), out_var(out_params.size());
    for (; i < lines.size(); ++i) {
        std::string line = lines[i];
        if (line == "}") break;
        if (line.compare(0, 11, "size_t tid ") == 0 || line.compare(0, 13, "if (tid >= n)") == 0) continue;
        CHX_REQUIRE(line.back() == ';', "fusion source: statement without ';': '%s'", line.c_str());
        line.resize(line.size() - 1);
        const size_t eq = line.find(" = ");
        CHX_REQUIRE(eq != std::string::npos, "fusion source: cannot parse '%s'", lines[i].c_str());
        const std::string lhs = trimmed(line.substr(0, eq)), rhs = trimmed(line.substr(eq + 3));
        if (lhs.compare(0, 8, "const T ") != 0) {
            // o_<name>[tid] = <name>
            const size_t br = lhs.find("[tid]");
            CHX_REQUIRE(br != std::string::npos && br + 5 == lhs.size(), "fusion source: cannot parse '%s'", lines[i].c_str());
            const std::string param = lhs.substr(0, br);
            size_t k = 0;
            while (k < out_params.size() && out_params[k] != param) ++k;
            CHX_REQUIRE(k < out_params.size() && is_identifier(rhs), "fusion source: '%s' stores to something that is not an output", lines[i].c_str());
            out_var[k] = rhs;
            continue;
        }
        const std::string out = trimmed(lhs.substr(8));
        CHX_REQUIRE(is_identifier(out), "fusion source: '%s' does not define a variable", lines[i].c_str());
        const size_t br = rhs.find("[tid]");
        if (br != std::string::npos) {
            // <name> = i_<name>[tid]
            const std::string param = rhs.substr(0, br);
            size_t k = 0;
            while (k < in_params.size() && in_params[k] != param) ++k;
            CHX_REQUIRE(k < in_params.size() && br + 5 == rhs.size(), "fusion source: '%s' loads from something that is not an input", lines[i].c_str());
            CHX_REQUIRE(in_var[k].empty(), "fusion source: input '%s' is loaded twice", param.c_str());
            in_var[k] = out;
            continue;
        }
        Stmt st;
        st.out = out;
        const std::vector<std::string> t = split_ws(rhs);
        const size_t call = rhs.find('(');
        if (t.size() == 3 && t[1].size() == 1 && strchr("+-*/", t[1][0]) && is_identifier(t[0]) && is_identifier(t[2])) {
            st.op = t[1] == "+" ? "Add" : t[1] == "-" ? "Sub" : t[1] == "*" ? "Mul" : "Div";
            st.args = {t[0], t[2]};
            prog->stmts.push_back(st);
        } else if (call != std::string::npos && rhs.back() == ')') {
            const std::string fn = rhs.substr(0, call), arg = trimmed(rhs.substr(call + 1, rhs.size() - call - 2));
            CHX_REQUIRE(is_identifier(arg), "fusion source: cannot parse the argument of '%s'", lines[i].c_str());
            if (fn == "tanh" || fn == "exp") {
                st.op = fn == "tanh" ? "Tanh" : "Exp";
                st.args = {arg};
                prog->stmts.push_back(st);
            } else if (fn == "sigmoid") {
                // the helper of this text, operation by operation: tanh(x * half) * half + half with half = 0.5
                const std::string h = out + "__half", a = out + "__arg", th = out + "__tanh", m = out + "__scaled";
                prog->stmts.push_back(Stmt{h, "Const", {"0.5"}});
                prog->stmts.push_back(Stmt{a, "Mul", {arg, h}});
                prog->stmts.push_back(Stmt{th, "Tanh", {a}});
                prog->stmts.push_back(Stmt{m, "Mul", {th, h}});
                prog->stmts.push_back(Stmt{out, "Add", {m, h}});
            } else {
                CHX_FAIL(CHX_HIP_EUNSUPPORTED, "fusion source: function '%s' is not one the reference's builder emits", fn.c_str());
            }
        } else if (t.size() == 1 && is_identifier(t[0])) {
            st.op = "Identity";
            st.args = {t[0]};
            prog->stmts.push_back(st);
        } else {
            char* end = nullptr;
            (void)strtod(rhs.c_str(), &end);
            CHX_REQUIRE(end && *end == 0 && end != rhs.c_str(), "fusion source: cannot parse the expression of '%s'", lines[i].c_str());
            st.op = "Const";
            st.args = {rhs};
            prog->stmts.push_back(st);
        }
    }
    CHX_REQUIRE(i < lines.size(), "fusion source: the kernel body does not end");
    for (size_t k = 0; k < in_params.size(); ++k) {
        // an input that the kernel never loads keeps its place in the argument list
        prog->inputs.push_back(Port{in_var[k].empty() ? in_params[k] + "__unused" : in_var[k], arith});
    }
    for (size_t k = 0; k < out_params.size(); ++k) {
        CHX_REQUIRE(!out_var[k].empty(), "fusion source: output '%s' is never stored", out_params[k].c_str());
        prog->outputs.push_back(Port{out_var[k], arith});
    }
    return settle_arithmetic_type(prog);
}

std::string ident(const std::string& s) {
    std::string o = "v_";
    for (char c : s) o += (isalnum((unsigned char)c) ? c : '_');
    return o;
}

int float_value(const std::string& tok, float* value);

// A literal of the program's arithmetic type, as source text that reproduces its bits: float32 and float64 by their
// bit patterns; float16 as the float32 that equals the literal rounded to float16.
int float_literal(const std::string& tok, std::string* out, int32_t arith = CHX_HIP_FLOAT32) {
    char buf[80];
    if (arith == CHX_HIP_FLOAT64 || arith == CHX_HIP_FLOAT16) {
        double d;
        if (tok.size() == 10 && tok[0] == '0' && (tok[1] == 'x' || tok[1] == 'X')) {
            float f;
            CHX_PROPAGATE(float_value(tok, &f));
            d = f;
        } else {
            char* end = nullptr;
            d = strtod(tok.c_str(), &end);
            CHX_REQUIRE(end && *end == 0 && end != tok.c_str(), "fusion program: bad float literal '%s'", tok.c_str());
        }
        if (arith == CHX_HIP_FLOAT64) {
            uint64_t bits;
            memcpy(&bits, &d, 8);
            snprintf(buf, sizeof(buf), "__builtin_bit_cast(double, 0x%016llxull)", (unsigned long long)bits);
        } else {
            const float f = (float)(_Float16)d;
            uint32_t bits;
            memcpy(&bits, &f, 4);
            snprintf(buf, sizeof(buf), "__builtin_bit_cast(float, 0x%08xu)", bits);
        }
        *out = buf;
        return CHX_HIP_OK;
    }
    float f;
    CHX_PROPAGATE(float_value(tok, &f));
    uint32_t bits;
    memcpy(&bits, &f, 4);
    snprintf(buf, sizeof(buf), "__builtin_bit_cast(float, 0x%08xu)", bits);
    *out = buf;
    return CHX_HIP_OK;
}

int float_value(const std::string& tok, float* value) {
    float f;
    if (tok.size() == 10 && tok[0] == '0' && (tok[1] == 'x' || tok[1] == 'X')) {
        char* end = nullptr;
        const unsigned long u = strtoul(tok.c_str(), &end, 16);
        CHX_REQUIRE(end && *end == 0, "fusion program: bad float bit pattern '%s'", tok.c_str());
        const uint32_t u32 = (uint32_t)u;
        memcpy(&f, &u32, 4);
    } else {
        char* end = nullptr;
        const double d = strtod(tok.c_str(), &end);
        CHX_REQUIRE(end && *end == 0 && end != tok.c_str(), "fusion program: bad float literal '%s'", tok.c_str());
        f = (float)d;
    }
    *value = f;
    return CHX_HIP_OK;
}

// Emits the per-element device function:  elem(in..., &out...).
// Value kinds: 'f' floating-point value, 'q' 8-bit code held in an int.  A floating-point value is held as TY:
// float for float32 and for float16 programs (in the latter every node's result goes through R(), the rounding
// to float16, so that it is a float16 value at all times), double for float64 programs.
int emit_elem(const Program& prog, bool use_fma, std::ostringstream& os, bool* uses_exp_table) {
    std::map<std::string, char> kind;
    const bool f64 = prog.arith == CHX_HIP_FLOAT64, f16 = prog.arith == CHX_HIP_FLOAT16;
    const std::string TY = f64 ? "double" : "float";
    const std::string decl = "  const " + TY + " ";
    const char* R0 = f16 ? "chx_round_f16(" : "(";
    const std::string zero = f64 ? "0.0" : "0.0f";
    // kFast: Exp and Sigmoid without their rare cases (arguments beyond +-88, quotients near the denormal range);
    // `rare` comes back set when an element met one, and the caller evaluates it again with kFast = false
    os << "template <bool kFast>\n__device__ __forceinline__ void elem(";
    bool first = true;
    for (const Port& p : prog.inputs) {
        CHX_REQUIRE(!kind.count(p.name), "fusion program: duplicate input '%s'", p.name.c_str());
        kind[p.name] = is_float_dtype(p.dtype) ? 'f' : 'q';
        os << (first ? "" : ", ") << (is_float_dtype(p.dtype) ? "const " + TY + " " : std::string("const int ")) << ident(p.name);
        first = false;
    }
    for (size_t i = 0; i < prog.outputs.size(); ++i)
        os << ", " << (is_float_dtype(prog.outputs[i].dtype) ? TY + "& " : std::string("int& ")) << "o_" << i;
    os << ", bool& rare) {\n";
    const char* fma = use_fma ? "true" : "false";
    for (const Stmt& s : prog.stmts) {
        CHX_REQUIRE(!kind.count(s.out), "fusion program: '%s' assigned twice", s.out.c_str());
        auto need = [&](size_t n) -> int {
            CHX_REQUIRE(s.args.size() == n, "fusion program: %s takes %zu operands, got %zu", s.op.c_str(), n,
                        s.args.size());
            return CHX_HIP_OK;
        };
        auto val = [&](size_t i, char k, std::string* out) -> int {
            auto it = kind.find(s.args[i]);
            CHX_REQUIRE(it != kind.end(), "fusion program: '%s' used before definition in '%s'", s.args[i].c_str(),
                        s.op.c_str());
            CHX_REQUIRE(it->second == k, "fusion program: operand '%s' of %s has the wrong kind (%s expected)",
                        s.args[i].c_str(), s.op.c_str(), k == 'f' ? "float" : "8-bit code");
            *out = ident(s.args[i]);
            return CHX_HIP_OK;
        };
        const std::string o = ident(s.out);
        std::string a, b, l0, l1;
        char out_kind = 'f';
        static const std::map<std::string, const char*> binops = {{"Add", "+"}, {"Sub", "-"}, {"Mul", "*"}, {"Div", "/"}};
        if (binops.count(s.op)) {
            CHX_PROPAGATE(need(2));
            CHX_PROPAGATE(val(0, 'f', &a));
            CHX_PROPAGATE(val(1, 'f', &b));
            os << decl << o << " = " << R0 << a << " " << binops.at(s.op) << " " << b << ");\n";
        } else if (s.op == "Max" || s.op == "Min") {
            CHX_PROPAGATE(need(2));
            CHX_PROPAGATE(val(0, 'f', &a));
            CHX_PROPAGATE(val(1, 'f', &b));
            if (s.op == "Max")
                os << decl << o << " = " << a << " < " << b << " ? " << b << " : " << a << ";\n";
            else
                os << decl << o << " = " << b << " < " << a << " ? " << b << " : " << a << ";\n";
        } else if (s.op == "Identity") {
            CHX_PROPAGATE(need(1));
            auto it = kind.find(s.args[0]);
            CHX_REQUIRE(it != kind.end(), "fusion program: '%s' used before definition", s.args[0].c_str());
            out_kind = it->second;
            os << "  const " << (out_kind == 'f' ? TY + " " : std::string("int ")) << o << " = " << ident(s.args[0]) << ";\n";
        } else if (s.op == "Neg") {
            CHX_PROPAGATE(need(1));
            CHX_PROPAGATE(val(0, 'f', &a));
            os << decl << o << " = -" << a << ";\n";
        } else if (s.op == "Abs") {
            CHX_PROPAGATE(need(1));
            CHX_PROPAGATE(val(0, 'f', &a));
            os << decl << o << " = " << (f64 ? "__builtin_fabs(" : "__builtin_fabsf(") << a << ");\n";
        } else if (s.op == "Floor") {
            CHX_PROPAGATE(need(1));
            CHX_PROPAGATE(val(0, 'f', &a));
            os << decl << o << " = " << (f64 ? "__builtin_floor(" : "__builtin_floorf(") << a << ");\n";
        } else if (s.op == "Round") {
            // to the nearest integer, ties to even (RoundOp, runtime/ops/quantize.cc:148-151)
            CHX_PROPAGATE(need(1));
            CHX_PROPAGATE(val(0, 'f', &a));
            os << decl << o << " = " << (f64 ? "__builtin_rint(" : "__builtin_rintf(") << a << ");\n";
        } else if (s.op == "Tanh") {
            CHX_PROPAGATE(need(1));
            CHX_PROPAGATE(val(0, 'f', &a));
            if (f64) os << decl << o << " = ::tanh(" << a << ");\n";
            else os << decl << o << " = " << R0 << "chx_fm::tanhf_faithful(" << a << "));\n";
        } else if (s.op == "Exp") {
            CHX_PROPAGATE(need(1));
            CHX_PROPAGATE(val(0, 'f', &a));
            if (f64) {
                os << decl << o << " = ::exp(" << a << ");\n";
            } else {
                os << decl << o << " = " << R0 << "kFast ? chx_fm::expf_unless_rare<" << fma << ">(" << a << ", rare) : chx_fm::expf_faithful<"
                   << fma << ">(" << a << "));\n";
                *uses_exp_table = true;
            }
        } else if (s.op == "Sigmoid") {
            CHX_PROPAGATE(need(1));
            CHX_PROPAGATE(val(0, 'f', &a));
            if (f64) {
                // 1 / (1 + exp(-x)), as the CPU path spells it
                os << decl << o << " = 1.0 / (1.0 + ::exp(-" << a << "));\n";
            } else if (f16) {
                // the same, every operation a float16 operation
                os << decl << o << "_e = chx_round_f16(chx_fm::expf_faithful<" << fma << ">(-" << a << "));\n";
                os << decl << o << "_d = chx_round_f16(1.0f + " << o << "_e);\n";
                os << decl << o << " = chx_round_f16(1.0f / " << o << "_d);\n";
                *uses_exp_table = true;
            } else {
                os << decl << o << " = kFast ? chx_fm::sigmoid_unless_rare<" << fma << ">(" << a
                   << ", rare) : chx_fm::sigmoid_faithful<" << fma << ">(" << a << ");\n";
                *uses_exp_table = true;
            }
        } else if (s.op == "Relu") {
            CHX_PROPAGATE(need(1));
            CHX_PROPAGATE(val(0, 'f', &a));
            os << decl << o << " = " << a << " < " << zero << " ? " << zero << " : " << a << ";\n";
        } else if (s.op == "Clip") {
            CHX_PROPAGATE(need(3));
            CHX_PROPAGATE(val(0, 'f', &a));
            CHX_PROPAGATE(float_literal(s.args[1], &l0, prog.arith));
            CHX_PROPAGATE(float_literal(s.args[2], &l1, prog.arith));
            os << decl << o << "_lo = " << a << " < " << l0 << " ? " << l0 << " : " << a << ";\n";
            os << decl << o << " = " << o << "_lo < " << l1 << " ? " << o << "_lo : " << l1 << ";\n";
        } else if (s.op == "Const") {
            CHX_PROPAGATE(need(1));
            CHX_PROPAGATE(float_literal(s.args[0], &l0, prog.arith));
            os << decl << o << " = " << l0 << ";\n";
        } else if (s.op == "QuantizeLinear") {
            CHX_REQUIRE(s.args.size() == 4 || (s.args.size() == 5 && s.args[4] == "rne"),
                        "fusion program: QuantizeLinear a scale zero_point dtype [rne]");
            CHX_REQUIRE(prog.arith == CHX_HIP_FLOAT32, "fusion program: QuantizeLinear inside a %s program", dtype_name(prog.arith));
            CHX_PROPAGATE(val(0, 'f', &a));
            CHX_PROPAGATE(float_literal(s.args[1], &l0));
            char* end = nullptr;
            const long zp = strtol(s.args[2].c_str(), &end, 10);
            CHX_REQUIRE(end && *end == 0, "fusion program: bad zero point '%s'", s.args[2].c_str());
            int32_t dt;
            CHX_REQUIRE(parse_dtype(s.args[3], &dt) && is_q8(dt), "fusion program: QuantizeLinear dtype must be uint8 or int8");
            const bool i8 = dt == CHX_HIP_INT8;
            CHX_REQUIRE(zp >= (i8 ? -128 : 0) && zp <= (i8 ? 127 : 255), "fusion program: zero point %ld out of range", zp);
            const char* lo = i8 ? "-128.0f" : "0.0f";
            const char* hi = i8 ? "127.0f" : "255.0f";
            // quantize_array, runtime/ops/quantize.cc:29-34.  The correctly rounded quotient comes from
            // three multiply-adds with the rounded reciprocal (q0 within an ulp, exact residual, one
            // correction) instead of the ten-instruction IEEE division.  The dividend is first limited
            // to +-2^40 * scale: beyond that both the true quotient and the limited one are far outside
            // the 8-bit range and saturate alike, and no intermediate can overflow.
            float scale_value;
            CHX_PROPAGATE(float_value(s.args[1], &scale_value));
            if (scale_value >= 0x1p-60f && scale_value <= 0x1p60f) {
                const float inv = 1.0f / scale_value, big = 0x1p40f * scale_value;
                uint32_t inv_bits, big_bits;
                memcpy(&inv_bits, &inv, 4);
                memcpy(&big_bits, &big, 4);
                char inv_lit[64], big_lit[64];
                snprintf(inv_lit, sizeof(inv_lit), "__builtin_bit_cast(float, 0x%08xu)", inv_bits);
                snprintf(big_lit, sizeof(big_lit), "__builtin_bit_cast(float, 0x%08xu)", big_bits);
                os << "  const float " << o << "_v = __builtin_amdgcn_fmed3f(" << a << ", -" << big_lit << ", " << big_lit << ");\n";
                os << "  const float " << o << "_q0 = " << o << "_v * " << inv_lit << ";\n";
                os << "  const float " << o << "_r = __builtin_fmaf(-" << o << "_q0, " << l0 << ", " << o << "_v);\n";
                os << "  float " << o << "_s = __builtin_fmaf(" << o << "_r, " << inv_lit << ", " << o << "_q0);\n";
            } else {
                os << "  float " << o << "_s = " << a << " / " << l0 << ";\n";
            }
            // the clamp is one median instruction: the same function as Maximum(lo, Minimum(s, hi))
            // for every value that is not a NaN
            if (s.args.size() == 5) {
                os << "  " << o << "_s = __builtin_rintf(" << o << "_s) + " << zp << ".0f;\n";
                os << "  " << o << "_s = __builtin_amdgcn_fmed3f(" << o << "_s, " << lo << ", " << hi << ");\n";
            } else {
                os << "  " << o << "_s = " << o << "_s + " << zp << ".0f;\n";
                os << "  " << o << "_s = __builtin_amdgcn_fmed3f(" << o << "_s, " << lo << ", " << hi << ");\n";
                os << "  " << o << "_s = " << o << "_s + 0.5f;\n";
            }
            os << "  const int " << o << " = (int)" << o << "_s;\n";
            out_kind = 'q';
        } else if (s.op == "DequantizeLinear") {
            CHX_PROPAGATE(need(3));
            CHX_REQUIRE(prog.arith == CHX_HIP_FLOAT32, "fusion program: DequantizeLinear inside a %s program", dtype_name(prog.arith));
            CHX_PROPAGATE(val(0, 'q', &a));
            CHX_PROPAGATE(float_literal(s.args[1], &l0));
            char* end = nullptr;
            const long zp = strtol(s.args[2].c_str(), &end, 10);
            CHX_REQUIRE(end && *end == 0, "fusion program: bad zero point '%s'", s.args[2].c_str());
            // dequantize_array, runtime/ops/quantize.cc:37-44
            os << "  const float " << o << "_f = (float)" << a << " - " << zp << ".0f;\n";
            os << "  const float " << o << " = " << o << "_f * " << l0 << ";\n";
        } else {
            CHX_FAIL(CHX_HIP_EUNSUPPORTED, "fusion program: op '%s' is not in the fusable set", s.op.c_str());
        }
        kind[s.out] = out_kind;
    }
    for (size_t i = 0; i < prog.outputs.size(); ++i) {
        auto it = kind.find(prog.outputs[i].name);
        CHX_REQUIRE(it != kind.end(), "fusion program: output '%s' is never defined", prog.outputs[i].name.c_str());
        const char want = is_float_dtype(prog.outputs[i].dtype) ? 'f' : 'q';
        CHX_REQUIRE(it->second == want, "fusion program: output '%s' is declared %s but computed as %s",
                    prog.outputs[i].name.c_str(), dtype_name(prog.outputs[i].dtype), it->second == 'f' ? "float" : "code");
        os << "  o_" << i << " = " << ident(prog.outputs[i].name) << ";\n";
    }
    os << "}\n";
    return CHX_HIP_OK;
}

enum Mode : char { kFull = 'F', kScalar = 'S', kPeriodic = 'P' };

const char* ctype_of(int32_t dt) {
    return dt == CHX_HIP_FLOAT32 ? "float" : dt == CHX_HIP_FLOAT16 ? "_Float16" : dt == CHX_HIP_FLOAT64 ? "double"
           : dt == CHX_HIP_INT8 ? "signed char" : "unsigned char";
}

// Source of both kernels for one (program, operand modes) combination.
//   <name>_vec : V elements per thread through 128-bit accesses; operands are full
//                (same flat index as the output), scalar, or periodic (index modulo a
//                period that is a multiple of V).
//   <name>_gen : one element per thread, operands addressed through per-axis strides.
int generate_source(
        const Program& prog, const std::string& name, const std::string& modes, const std::vector<uint32_t>& periods,
        int vec, bool use_fma, std::string* out) {
    std::ostringstream os;
    os << "#pragma clang fp contract(off)\n";
    os << "#define FM_FN __device__ __forceinline__\n";
    os << "#define FM_TABLE_QUALIFIER static __device__ const\n";
    os << "#define FM_DEVICE_DIV 1\n";
    os << "#define FM_ANY_LANE(c) (__builtin_amdgcn_ballot_w64(c) != 0ull)\n";
    std::ostringstream body;
    bool uses_table = false;
    CHX_PROPAGATE(emit_elem(prog, use_fma, body, &uses_table));
    os << kFaithfulMathText << "\n";
    os << "__device__ __forceinline__ float chx_round_f16(float x) { return (float)(_Float16)x; }\n";
    os << "typedef float v4f __attribute__((ext_vector_type(4)));\n";
    os << "typedef unsigned int v4u __attribute__((ext_vector_type(4)));\n";
    os << "namespace {\n" << body.str() << "}\n";
    const size_t nin = prog.inputs.size(), nout = prog.outputs.size();

    // ---- vector kernel ----
    // `vec` elements per lane and step: 4 when any full-size operand is float32 (float32
    // moves as one 128-bit access per lane, 8-bit codes as one 32-bit access), 16 when all
    // of them are 8-bit (one 128-bit access each).  kSteps steps per thread at a stride of
    // one block keep every access instruction of a wavefront on one contiguous span.
    const int steps = 2;
    const std::string VT = prog.arith == CHX_HIP_FLOAT64 ? "double" : "float";  // what elem() takes and gives
    if (prog.arith != CHX_HIP_FLOAT32) {
        // float16 and float64 programs run on the general kernel; this one is never launched
        os << "extern \"C\" __global__ void " << name << "_vec(unsigned int n_vec) {}\n";
    } else {
    os << "extern \"C\" __global__ __launch_bounds__(256) void " << name << "_vec(unsigned int n_vec";
    for (size_t i = 0; i < nin; ++i) os << ", const " << ctype_of(prog.inputs[i].dtype) << "* __restrict__ i" << i;
    for (size_t i = 0; i < nout; ++i) os << ", " << ctype_of(prog.outputs[i].dtype) << "* __restrict__ o" << i;
    os << ") {\n";
    os << "  const unsigned int vid0 = blockIdx.x * " << 256 * steps << "u + threadIdx.x;\n";
    os << "#pragma unroll\n  for (int st = 0; st < " << steps << "; ++st) {\n";
    os << "  const unsigned int vid = vid0 + st * 256u;\n";
    os << "  if (vid < n_vec) {\n";
    os << "  const unsigned int base = vid * " << vec << "u;  // fewer than 2^31 elements\n";
    for (size_t i = 0; i < nin; ++i) {
        const bool f32 = prog.inputs[i].dtype == CHX_HIP_FLOAT32;
        const bool sgn = prog.inputs[i].dtype == CHX_HIP_INT8;
        os << "  " << (f32 ? "float" : "int") << " x" << i << "[" << vec << "];\n";
        if (modes[i] == kScalar) {
            os << "  for (int e = 0; e < " << vec << "; ++e) x" << i << "[e] = i" << i << "[0];\n";
            continue;
        }
        std::string idx = "base";
        if (modes[i] == kPeriodic) idx = "(base % " + std::to_string(periods[i]) + "u)";
        const bool nt = modes[i] == kFull;
        const char* ld0 = nt ? "__builtin_nontemporal_load(" : "*(";
        if (f32) {
            os << "  { const v4f* src = (const v4f*)(i" << i << " + " << idx << ");\n";
            for (int j = 0; j < vec / 4; ++j) {
                os << "    const v4f t" << j << " = " << ld0 << "src + " << j << ");\n";
                for (int k = 0; k < 4; ++k) os << "    x" << i << "[" << (j * 4 + k) << "] = t" << j << "[" << k << "];\n";
            }
            os << "  }\n";
        } else {
            const int words = vec / 4;
            os << "  { unsigned int t[" << words << "];\n";
            if (words == 4) {
                os << "    const v4u tv = " << ld0 << "(const v4u*)(i" << i << " + " << idx << "));\n";
                os << "    t[0] = tv[0]; t[1] = tv[1]; t[2] = tv[2]; t[3] = tv[3];\n";
            } else {
                os << "    t[0] = " << ld0 << "(const unsigned int*)(i" << i << " + " << idx << "));\n";
            }
            for (int e = 0; e < vec; ++e) {
                os << "    x" << i << "[" << e << "] = ";
                if (sgn)
                    os << "(int)(signed char)((t[" << (e / 4) << "] >> " << (8 * (e % 4)) << ") & 0xffu);\n";
                else
                    os << "(int)((t[" << (e / 4) << "] >> " << (8 * (e % 4)) << ") & 0xffu);\n";
            }
            os << "  }\n";
        }
    }
    for (size_t i = 0; i < nout; ++i)
        os << "  " << (prog.outputs[i].dtype == CHX_HIP_FLOAT32 ? "float" : "int") << " y" << i << "[" << vec << "];\n";
    // all elements of the step without the rare cases first, one wavefront-wide test, and again in full if any lane
    // met one: a branch per element costs more than the rare cases' few instructions
    os << "  bool rare = false;\n";
    for (int fast = 1; fast >= 0; --fast) {
        if (!fast) os << "  if (__builtin_expect(FM_ANY_LANE(rare), 0)) {\n";
        os << "#pragma unroll\n  for (int e = 0; e < " << vec << "; ++e) elem<" << (fast ? "true" : "false") << ">(";
        for (size_t i = 0; i < nin; ++i) os << (i ? ", " : "") << "x" << i << "[e]";
        for (size_t i = 0; i < nout; ++i) os << ", y" << i << "[e]";
        os << ", rare);\n";
        if (!fast) os << "  }\n";
    }
    for (size_t i = 0; i < nout; ++i) {
        if (prog.outputs[i].dtype == CHX_HIP_FLOAT32) {
            os << "  { v4f* dst = (v4f*)(o" << i << " + base);\n";
            for (int j = 0; j < vec / 4; ++j) {
                os << "    v4f t" << j << ";\n";
                for (int k = 0; k < 4; ++k) os << "    t" << j << "[" << k << "] = y" << i << "[" << (j * 4 + k) << "];\n";
                os << "    __builtin_nontemporal_store(t" << j << ", dst + " << j << ");\n";
            }
            os << "  }\n";
        } else {
            const int words = vec / 4;
            os << "  { unsigned int t[" << words << "];\n";
            for (int w = 0; w < words; ++w) {
                os << "    t[" << w << "] = ";
                for (int k = 0; k < 4; ++k)
                    os << (k ? " | " : "") << "(((unsigned int)y" << i << "[" << (w * 4 + k) << "] & 0xffu) << " << (8 * k) << ")";
                os << ";\n";
            }
            if (words == 4) {
                os << "    v4u tv; tv[0] = t[0]; tv[1] = t[1]; tv[2] = t[2]; tv[3] = t[3];\n";
                os << "    __builtin_nontemporal_store(tv, (v4u*)(o" << i << " + base));\n  }\n";
            } else {
                os << "    __builtin_nontemporal_store(t[0], (unsigned int*)(o" << i << " + base));\n  }\n";
            }
        }
    }
    os << "  }\n  }\n}\n";
    }

    // ---- general kernel ----
    os << "struct GenDesc { int ndim; int pad; long long shape[" << CHX_HIP_MAX_NDIM << "]; long long istr[" << nin << "]["
       << CHX_HIP_MAX_NDIM << "]; };\n";
    os << "extern \"C\" __global__ __launch_bounds__(256) void " << name
       << "_gen(unsigned long long begin, unsigned long long n";
    for (size_t i = 0; i < nin; ++i) os << ", const " << ctype_of(prog.inputs[i].dtype) << "* __restrict__ i" << i;
    for (size_t i = 0; i < nout; ++i) os << ", " << ctype_of(prog.outputs[i].dtype) << "* __restrict__ o" << i;
    os << ", GenDesc d) {\n";
    os << "  const unsigned long long idx = begin + (unsigned long long)blockIdx.x * 256ull + threadIdx.x;\n";
    os << "  if (idx >= n) return;\n";
    os << "  long long off[" << nin << "];\n";
    os << "  for (int i = 0; i < " << nin << "; ++i) off[i] = 0;\n";
    os << "  unsigned long long rest = idx;\n";
    os << "  for (int a = d.ndim - 1; a >= 0; --a) {\n";
    os << "    const unsigned long long q = rest / (unsigned long long)d.shape[a];\n";
    os << "    const long long r = (long long)(rest - q * (unsigned long long)d.shape[a]);\n";
    os << "    for (int i = 0; i < " << nin << "; ++i) off[i] += r * d.istr[i][a];\n";
    os << "    rest = q;\n  }\n";
    for (size_t i = 0; i < nout; ++i)
        os << "  " << (is_float_dtype(prog.outputs[i].dtype) ? VT : std::string("int")) << " r" << i << ";\n";
    os << "  bool rare = false;\n  elem<false>(";
    for (size_t i = 0; i < nin; ++i)
        os << (i ? ", " : "") << "(" << (is_float_dtype(prog.inputs[i].dtype) ? VT : std::string("int")) << ")i" << i << "[off[" << i << "]]";
    for (size_t i = 0; i < nout; ++i) os << ", r" << i;
    os << ", rare);\n";
    for (size_t i = 0; i < nout; ++i) {
        os << "  o" << i << "[idx] = (" << ctype_of(prog.outputs[i].dtype) << ")r" << i << ";\n";
    }
    os << "}\n";
    *out = os.str();
    return CHX_HIP_OK;
}

struct CompiledKernels {
    std::vector<char> code;
    hipModule_t module = nullptr;  // loaded lazily, per process (one GPU)
    hipFunction_t vec = nullptr, gen = nullptr;
};

std::mutex g_cache_mutex;
std::map<std::string, std::shared_ptr<CompiledKernels>> g_cache;  // key: generated source

int compile_source(const std::string& src, const std::string& name, std::vector<char>* code) {
    hiprtcProgram p;
    if (hiprtcCreateProgram(&p, src.c_str(), (name + ".hip").c_str(), 0, nullptr, nullptr) != HIPRTC_SUCCESS)
        CHX_FAIL(CHX_HIP_ERUNTIME, "hiprtcCreateProgram failed for %s", name.c_str());
    const char* opts[] = {"--offload-arch=gfx950", "-O3", "-ffp-contract=off", "-Xclang", "-target-feature",
                          "-Xclang", "-packed-fp32-ops"};
    const hiprtcResult r = hiprtcCompileProgram(p, (int)(sizeof(opts) / sizeof(opts[0])), opts);
    if (r != HIPRTC_SUCCESS) {
        size_t ls = 0;
        hiprtcGetProgramLogSize(p, &ls);
        std::string log(ls, '\0');
        if (ls) hiprtcGetProgramLog(p, &log[0]);
        hiprtcDestroyProgram(&p);
        CHX_FAIL(CHX_HIP_ECOMPILE, "hiprtc could not compile %s: %s\n%s", name.c_str(), hiprtcGetErrorString(r),
                 log.c_str());
    }
    size_t cs = 0;
    hiprtcGetCodeSize(p, &cs);
    code->resize(cs);
    hiprtcGetCode(p, code->data());
    hiprtcDestroyProgram(&p);
    return CHX_HIP_OK;
}

struct Plan {
    std::string modes;             // per input
    bool vector_ok = false;
    int vec = 4;
    int64_t n = 0;
    int ndim = 0;
    int64_t shape[CHX_HIP_MAX_NDIM];
    std::vector<std::vector<int64_t>> istr;  // element strides per input, per collapsed axis
    std::vector<uint32_t> periods;
};

int make_plan(
        const Program& prog, const chx_hip_tensor* const* inputs, int32_t n_inputs, chx_hip_tensor* const* outputs,
        int32_t n_outputs, Plan* plan) {
    CHX_REQUIRE((size_t)n_inputs == prog.inputs.size(), "fusion: program declares %zu inputs, %d given",
                prog.inputs.size(), n_inputs);
    CHX_REQUIRE((size_t)n_outputs == prog.outputs.size(), "fusion: program declares %zu outputs, %d given",
                prog.outputs.size(), n_outputs);
    int nd = 0;
    for (int i = 0; i < n_inputs; ++i) {
        CHX_PROPAGATE(check_tensor(inputs[i], "fusion input"));
        CHX_REQUIRE(inputs[i]->dtype == prog.inputs[i].dtype, "fusion: input %d is %s, program says %s", i,
                    dtype_name(inputs[i]->dtype), dtype_name(prog.inputs[i].dtype));
        nd = inputs[i]->ndim > nd ? inputs[i]->ndim : nd;
    }
    // BroadcastShapes over all inputs, runtime/ops/nvrtc.cc:100-104
    int64_t shape[CHX_HIP_MAX_NDIM];
    for (int a = 0; a < nd; ++a) shape[a] = 1;
    for (int i = 0; i < n_inputs; ++i) {
        const chx_hip_tensor& t = *inputs[i];
        for (int a = 0; a < t.ndim; ++a) {
            const int oa = nd - t.ndim + a;
            if (t.shape[a] == 1) continue;
            CHX_REQUIRE(shape[oa] == 1 || shape[oa] == t.shape[a], "fusion: input %d does not broadcast (axis %d: %lld vs %lld)",
                        i, a, (long long)t.shape[a], (long long)shape[oa]);
            shape[oa] = t.shape[a];
        }
    }
    int64_t n = 1;
    for (int a = 0; a < nd; ++a) n *= shape[a];
    plan->n = n;
    for (int i = 0; i < n_outputs; ++i) {
        CHX_PROPAGATE(check_tensor(outputs[i], "fusion output"));
        const chx_hip_tensor& t = *outputs[i];
        CHX_REQUIRE(t.dtype == prog.outputs[i].dtype, "fusion: output %d is %s, program says %s", i, dtype_name(t.dtype),
                    dtype_name(prog.outputs[i].dtype));
        CHX_REQUIRE(t.ndim == nd, "fusion: output %d has ndim %d, the broadcast result has %d", i, t.ndim, nd);
        for (int a = 0; a < nd; ++a)
            CHX_REQUIRE(t.shape[a] == shape[a], "fusion: output %d has extent %lld on axis %d, expected %lld", i,
                        (long long)t.shape[a], a, (long long)shape[a]);
    }
    // Iteration order: axes of output 0 by decreasing stride; every output must be dense in
    // that order with the same element strides.
    int order[CHX_HIP_MAX_NDIM];
    int na = 0;
    const chx_hip_tensor& o0 = *outputs[0];
    const int64_t es0 = dtype_size(o0.dtype);
    for (int a = 0; a < nd; ++a)
        if (shape[a] != 1) order[na++] = a;
    for (int i = 0; i < na; ++i)
        for (int j = i + 1; j < na; ++j)
            if (o0.strides[order[j]] > o0.strides[order[i]]) {
                const int t = order[i];
                order[i] = order[j];
                order[j] = t;
            }
    {
        int64_t expect = 1;
        for (int i = na - 1; i >= 0; --i) {
            for (int k = 0; k < n_outputs; ++k) {
                const int64_t es = dtype_size(outputs[k]->dtype);
                CHX_REQUIRE(outputs[k]->strides[order[i]] == expect * es,
                            "fusion: output %d is not dense, or outputs differ in layout", k);
            }
            expect *= shape[order[i]];
        }
        (void)es0;
    }
    // Element strides of every input along the ordered axes (0 where it broadcasts).
    std::vector<std::vector<int64_t>> istr(n_inputs, std::vector<int64_t>(na, 0));
    for (int i = 0; i < n_inputs; ++i) {
        const chx_hip_tensor& t = *inputs[i];
        const int64_t es = dtype_size(t.dtype);
        for (int k = 0; k < na; ++k) {
            const int ia = order[k] - (nd - t.ndim);
            if (ia < 0 || t.shape[ia] == 1) continue;
            CHX_REQUIRE(t.strides[ia] % es == 0, "fusion: input %d has a stride that is not a multiple of its element size", i);
            istr[i][k] = t.strides[ia] / es;
        }
    }
    // Collapse neighbouring axes that every operand walks contiguously.
    std::vector<int64_t> cshape;
    std::vector<std::vector<int64_t>> cstr(n_inputs);
    for (int k = 0; k < na; ++k) {
        const int64_t ext = shape[order[k]];
        bool merge = !cshape.empty();
        if (merge)
            for (int i = 0; i < n_inputs; ++i)
                if (cstr[i].back() != istr[i][k] * ext) merge = false;
        if (merge) {
            cshape.back() *= ext;
            for (int i = 0; i < n_inputs; ++i) cstr[i].back() = istr[i][k];
        } else {
            cshape.push_back(ext);
            for (int i = 0; i < n_inputs; ++i) cstr[i].push_back(istr[i][k]);
        }
    }
    plan->ndim = (int)cshape.size();
    for (int a = 0; a < plan->ndim; ++a) plan->shape[a] = cshape[a];
    plan->istr = cstr;

    bool any32 = false;
    for (const Port& p : prog.inputs) any32 = any32 || p.dtype == CHX_HIP_FLOAT32;
    for (const Port& p : prog.outputs) any32 = any32 || p.dtype == CHX_HIP_FLOAT32;
    plan->vec = any32 ? 4 : 16;
    plan->modes.assign(n_inputs, kFull);
    plan->periods.assign(n_inputs, 0);
    bool ok = n < (int64_t(1) << 31);  // CHECK_GT(1 << 31, size), runtime/ops/nvrtc.cc:127
    // dense inner strides of the output in collapsed axes
    std::vector<int64_t> dense(plan->ndim, 1);
    for (int a = plan->ndim - 2; a >= 0; --a) dense[a] = dense[a + 1] * cshape[a + 1];
    for (int i = 0; i < n_inputs; ++i) {
        bool all_zero = true, full = true;
        for (int a = 0; a < plan->ndim; ++a) {
            if (cstr[i][a] != 0) all_zero = false;
            if (cstr[i][a] != dense[a]) full = false;
        }
        const int64_t es = dtype_size(inputs[i]->dtype);
        if (plan->ndim == 0 || all_zero) {
            plan->modes[i] = kScalar;
        } else if (full) {
            plan->modes[i] = kFull;
            if (!aligned(inputs[i]->data, 16)) ok = false;
        } else {
            // periodic: zero strides on the outer axes, dense strides on the inner ones
            int a = 0;
            while (a < plan->ndim && cstr[i][a] == 0) ++a;
            bool inner_dense = a > 0;
            for (int b = a; b < plan->ndim; ++b)
                if (cstr[i][b] != dense[b]) inner_dense = false;
            const int64_t period = a > 0 ? dense[a - 1] : 0;
            if (inner_dense && period % plan->vec == 0 && period < (int64_t(1) << 31) && aligned(inputs[i]->data, 16)) {
                plan->modes[i] = kPeriodic;
                plan->periods[i] = (uint32_t)period;
            } else {
                ok = false;
            }
        }
        (void)es;
    }
    for (int k = 0; k < n_outputs; ++k)
        if (!aligned(outputs[k]->data, 16)) ok = false;
    plan->vector_ok = ok && n >= plan->vec && prog.arith == CHX_HIP_FLOAT32;
    if (!plan->vector_ok) {
        // the general kernel ignores modes; use one canonical key
        plan->modes.assign(n_inputs, kFull);
        plan->periods.assign(n_inputs, 0);
    }
    return CHX_HIP_OK;
}

struct ArgPacker {
    std::vector<char> buf;
    template <typename T>
    void push(const T& v) {
        const size_t a = alignof(T);
        const size_t off = (buf.size() + a - 1) / a * a;
        buf.resize(off + sizeof(T));
        memcpy(buf.data() + off, &v, sizeof(T));
    }
    void push_bytes(const void* p, size_t n, size_t a) {
        const size_t off = (buf.size() + a - 1) / a * a;
        buf.resize(off + n);
        memcpy(buf.data() + off, p, n);
    }
};

int prepare(
        const char* code, int32_t fusion_id, const chx_hip_tensor* const* inputs, int32_t n_inputs,
        chx_hip_tensor* const* outputs, int32_t n_outputs, Program* prog, Plan* plan, std::string* name,
        std::string* src) {
    CHX_REQUIRE(inputs != nullptr && n_inputs > 0, "fusion: no inputs");  // CHECK(!inputs.empty()), nvrtc.cc:93
    CHX_REQUIRE(outputs != nullptr && n_outputs > 0, "fusion: no outputs");
    CHX_PROPAGATE(parse_program(code, prog));
    CHX_PROPAGATE(make_plan(*prog, inputs, n_inputs, outputs, n_outputs, plan));
    *name = "fusion" + std::to_string(fusion_id < 0 ? 0 : fusion_id);
    CHX_PROPAGATE(generate_source(*prog, *name, plan->modes, plan->periods, plan->vec, host_libm_uses_fma(), src));
    return CHX_HIP_OK;
}

int get_compiled(const std::string& src, const std::string& name, std::shared_ptr<CompiledKernels>* out) {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    auto it = g_cache.find(src);
    if (it != g_cache.end()) {
        *out = it->second;
        return CHX_HIP_OK;
    }
    auto ck = std::make_shared<CompiledKernels>();
    CHX_PROPAGATE(compile_source(src, name, &ck->code));
    g_cache.emplace(src, ck);
    *out = ck;
    return CHX_HIP_OK;
}

int load_kernels(CompiledKernels* ck, const std::string& name) {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    if (ck->module) return CHX_HIP_OK;
    hipModule_t m;
    CHX_HIP_CALL(hipModuleLoadData(&m, ck->code.data()));
    CHX_HIP_CALL(hipModuleGetFunction(&ck->vec, m, (name + "_vec").c_str()));
    CHX_HIP_CALL(hipModuleGetFunction(&ck->gen, m, (name + "_gen").c_str()));
    ck->module = m;
    return CHX_HIP_OK;
}

int launch(hipFunction_t f, unsigned grid, ArgPacker& args, hipStream_t s) {
    size_t size = args.buf.size();
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, args.buf.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size,
                     HIP_LAUNCH_PARAM_END};
    CHX_HIP_CALL(hipModuleLaunchKernel(f, grid, 1, 1, 256, 1, 1, 0, s, nullptr, extra));
    return CHX_HIP_OK;
}

}  // namespace
}  // namespace chx

using namespace chx;

extern "C" int chx_hip_elementwise_output_dtypes(const char* code, int32_t* dtypes, int32_t capacity, int32_t* count) {
    CHX_REQUIRE(count != nullptr && (dtypes != nullptr || capacity == 0), "elementwise_output_dtypes: null output");
    Program prog;
    CHX_PROPAGATE(parse_program(code, &prog));
    *count = (int32_t)prog.outputs.size();
    for (int32_t i = 0; i < *count && i < capacity; ++i) dtypes[i] = prog.outputs[(size_t)i].dtype;
    return CHX_HIP_OK;
}

extern "C" int chx_hip_elementwise_source(
        const char* code, int32_t fusion_id, const chx_hip_tensor* const* inputs, int32_t n_inputs,
        chx_hip_tensor* const* outputs, int32_t n_outputs, int32_t compile, char* buffer, size_t buffer_size,
        size_t* needed) {
    Program prog;
    Plan plan;
    std::string name, src;
    CHX_PROPAGATE(prepare(code, fusion_id, inputs, n_inputs, outputs, n_outputs, &prog, &plan, &name, &src));
    if (compile) {
        std::shared_ptr<CompiledKernels> ck;
        CHX_PROPAGATE(get_compiled(src, name, &ck));
    }
    std::string text = std::string("// modes=") + plan.modes + (plan.vector_ok ? " vector" : " general") + "\n" + src;
    if (needed) *needed = text.size() + 1;
    if (buffer && buffer_size) {
        const size_t n = text.size() < buffer_size - 1 ? text.size() : buffer_size - 1;
        memcpy(buffer, text.data(), n);
        buffer[n] = 0;
    }
    return CHX_HIP_OK;
}

extern "C" int chx_hip_elementwise(
        const char* code, int32_t fusion_id, const chx_hip_tensor* const* inputs, int32_t n_inputs,
        chx_hip_tensor* const* outputs, int32_t n_outputs, void* stream) {
    Program prog;
    Plan plan;
    std::string name, src;
    CHX_PROPAGATE(prepare(code, fusion_id, inputs, n_inputs, outputs, n_outputs, &prog, &plan, &name, &src));
    if (plan.n == 0) return CHX_HIP_OK;
    std::shared_ptr<CompiledKernels> ck;
    CHX_PROPAGATE(get_compiled(src, name, &ck));
    CHX_PROPAGATE(load_kernels(ck.get(), name));
    hipStream_t s = as_stream(stream);

    int64_t done = 0;
    if (plan.vector_ok) {
        const int64_t n_vec = plan.n / plan.vec;
        ArgPacker a;
        a.push((uint32_t)n_vec);
        for (int i = 0; i < n_inputs; ++i) a.push(inputs[i]->data);
        for (int i = 0; i < n_outputs; ++i) a.push(outputs[i]->data);
        CHX_PROPAGATE(launch(ck->vec, (unsigned)((n_vec + 511) / 512), a, s));
        done = n_vec * plan.vec;
    }
    if (done < plan.n) {
        CHX_REQUIRE(plan.n - done < (int64_t(1) << 39), "fusion: %lld elements is beyond what the general kernel covers",
                    (long long)(plan.n - done));
        ArgPacker a;
        a.push((unsigned long long)done);
        a.push((unsigned long long)plan.n);
        for (int i = 0; i < n_inputs; ++i) a.push(inputs[i]->data);
        for (int i = 0; i < n_outputs; ++i) a.push(outputs[i]->data);
        // GenDesc { int ndim; int pad; long long shape[MAX]; long long istr[nin][MAX]; }
        std::vector<long long> d(1 + CHX_HIP_MAX_NDIM + (size_t)n_inputs * CHX_HIP_MAX_NDIM, 0);
        int32_t head[2] = {plan.ndim, 0};
        memcpy(&d[0], head, 8);
        for (int k = 0; k < plan.ndim; ++k) d[1 + k] = plan.shape[k];
        for (int k = plan.ndim; k < CHX_HIP_MAX_NDIM; ++k) d[1 + k] = 1;
        for (int i = 0; i < n_inputs; ++i)
            for (int k = 0; k < plan.ndim; ++k) d[1 + CHX_HIP_MAX_NDIM + (size_t)i * CHX_HIP_MAX_NDIM + k] = plan.istr[i][k];
        a.push_bytes(d.data(), d.size() * sizeof(long long), 8);
        CHX_PROPAGATE(launch(ck->gen, (unsigned)((plan.n - done + 255) / 256), a, s));
    }
    return CHX_HIP_OK;
}

extern "C" int chx_hip_elementwise_match_residual_add(const char* code, int32_t* matches, chx_hip_residual_group* group) {
    using namespace chx;
    CHX_REQUIRE(matches != nullptr && group != nullptr, "match_residual_add: null output");
    *matches = 0;
    memset(group, 0, sizeof(*group));
    Program prog;
    CHX_PROPAGATE(parse_program(code, &prog));
    if (prog.inputs.size() != 2 || prog.outputs.size() != 1) return CHX_HIP_OK;
    if (!is_q8(prog.inputs[0].dtype) || !is_q8(prog.inputs[1].dtype) || !is_q8(prog.outputs[0].dtype)) return CHX_HIP_OK;
    if (prog.stmts.size() != 4 && prog.stmts.size() != 5) return CHX_HIP_OK;
    const bool relu = prog.stmts.size() == 5;
    std::string dq_name[2];
    for (int i = 0; i < 2; ++i) {
        // one DequantizeLinear per input, among the first two statements
        const Stmt* found = nullptr;
        for (int j = 0; j < 2; ++j)
            if (prog.stmts[j].op == "DequantizeLinear" && prog.stmts[j].args.size() == 3 && prog.stmts[j].args[0] == prog.inputs[i].name)
                found = found ? nullptr : &prog.stmts[j];
        if (!found || prog.inputs[0].name == prog.inputs[1].name) return CHX_HIP_OK;
        CHX_PROPAGATE(float_value(found->args[1], &group->in_scale[i]));
        char* end = nullptr;
        const long zp = strtol(found->args[2].c_str(), &end, 10);
        if (!end || *end != 0) return CHX_HIP_OK;
        group->in_zero_point[i] = (int32_t)zp;
        group->in_dtype[i] = prog.inputs[i].dtype;
        dq_name[i] = found->out;
    }
    const Stmt& add = prog.stmts[2];
    if (add.op != "Add" || add.args.size() != 2) return CHX_HIP_OK;
    if (!((add.args[0] == dq_name[0] && add.args[1] == dq_name[1]) || (add.args[0] == dq_name[1] && add.args[1] == dq_name[0])))
        return CHX_HIP_OK;
    std::string last = add.out;
    if (relu) {
        const Stmt& r = prog.stmts[3];
        if (r.op != "Relu" || r.args.size() != 1 || r.args[0] != last) return CHX_HIP_OK;
        last = r.out;
    }
    const Stmt& q = prog.stmts.back();
    if (q.op != "QuantizeLinear" || q.args.size() != 4 || q.args[0] != last || q.out != prog.outputs[0].name) return CHX_HIP_OK;
    CHX_PROPAGATE(float_value(q.args[1], &group->out_scale));
    char* end = nullptr;
    const long zp = strtol(q.args[2].c_str(), &end, 10);
    int32_t qdt = 0;
    if (!end || *end != 0 || !parse_dtype(q.args[3], &qdt) || qdt != prog.outputs[0].dtype) return CHX_HIP_OK;
    group->out_zero_point = (int32_t)zp;
    group->out_dtype = qdt;
    group->relu = relu ? 1 : 0;
    *matches = 1;
    return CHX_HIP_OK;
}
