#include "chxvm.h"

#include <algorithm>
#include <cstring>
#include <fstream>
#include <iomanip>
#include <map>
#include <sstream>

#include <set>

#include <iostream>

#include "chrome_tracing.h"

namespace chainer_compiler {
namespace runtime {

namespace {

// DequantizeLinear(a), DequantizeLinear(b), MatMul, QuantizeLinear as one instruction: the
// quantized matrix product with the reference's float semantics (chx_hip_qlinear_matmul).
class FusedQLinearMatMulOp : public ChxVMOp {
public:
    FusedQLinearMatMulOp(const ChxVMInstructionProto& quantize, const ChxVMInstructionProto& dq_a,
                         const ChxVMInstructionProto& dq_b)
        : ChxVMOp(quantize),
          a_(dq_a.inputs[0].array), a_scale_(dq_a.inputs[1].scalar), a_zp_(dq_a.inputs[2].scalar),
          b_(dq_b.inputs[0].array), b_scale_(dq_b.inputs[1].scalar), b_zp_(dq_b.inputs[2].scalar),
          y_scale_(quantize.inputs[1].scalar), y_zp_(quantize.inputs[2].scalar), y_(quantize.outputs[0]) {
    }

    void Run(ChxVMState* st) override {
        if (st->trace_level()) std::cerr << "QLinearMatMul(fused) $" << a_ << " $" << b_ << " -> $" << y_ << std::endl;
        const chainerx::Array a = st->GetArray(a_), b = st->GetArray(b_);
        auto zp_of = [&](int slot) -> StrictScalar {
            absl::optional<StrictScalar> z = st->GetOptionalScalar(slot);
            return z.has_value() ? *z : StrictScalar(chainerx::Dtype::kUInt8, chainerx::Scalar(0u), false);
        };
        const StrictScalar az = zp_of(a_zp_), bz = zp_of(b_zp_), yz = zp_of(y_zp_);
        CHECK_LE(2, a.ndim());
        CHECK_EQ(a.ndim(), b.ndim());
        chainerx::Shape shape(a.shape().begin(), a.shape().end() - 1);
        shape.push_back(b.shape()[b.ndim() - 1]);
        chainerx::Array y = chainerx::Empty(shape, yz.dtype());
        chx_hip_tensor at = a.hip(), bt = b.hip(), yt = y.hip();
        CHXVM_HIP_CALL(chx_hip_qlinear_matmul(
                &at, static_cast<float>(st->GetScalar(a_scale_)), static_cast<int32_t>(static_cast<int64_t>(az)), &bt,
                static_cast<float>(st->GetScalar(b_scale_)), static_cast<int32_t>(static_cast<int64_t>(bz)),
                static_cast<float>(st->GetScalar(y_scale_)), static_cast<int32_t>(static_cast<int64_t>(yz)),
                nullptr, CHX_HIP_ROUND_REFERENCE, &yt, chainerx::CurrentStream()));
        st->SetArray(y_, y);
    }

private:
    int a_, a_scale_, a_zp_, b_, b_scale_, b_zp_, y_scale_, y_zp_, y_;
};

// DequantizeLinear, MaxPool | AveragePool, QuantizeLinear as one instruction on the 8-bit codes
// (chx_hip_max_pool_q8 / chx_hip_average_pool_q8).  MaxPool operands: x, kernel_shape, strides,
// pads, cover_all, auto_pad; AveragePool: x, kernel_shape, strides, pads, count_include_pad
// (runtime/chxvm_defs.py:314-321 of the chainer-compiler tree).
class FusedQuantizedPoolOp : public ChxVMOp {
public:
    FusedQuantizedPoolOp(const ChxVMInstructionProto& quantize, const ChxVMInstructionProto& pool,
                         const ChxVMInstructionProto& dq, bool is_max)
        : ChxVMOp(quantize), is_max_(is_max),
          x_(dq.inputs[0].array), x_scale_(dq.inputs[1].scalar), x_zp_(dq.inputs[2].scalar),
          y_scale_(quantize.inputs[1].scalar), y_zp_(quantize.inputs[2].scalar), y_(quantize.outputs[0]),
          kernel_(pool.inputs[1].ints), strides_(pool.inputs[2].ints), pads_(pool.inputs[3].ints),
          flag_(static_cast<int>(pool.inputs[4].i)) {
        CHECK_EQ(2u, kernel_.size()) << "only 2-D pooling on the hip backend";
        if (is_max) CHECK(pool.inputs[5].s.empty() || pool.inputs[5].s == "NOTSET") << "auto_pad is not supported for a quantized MaxPool";
    }

    void Run(ChxVMState* st) override {
        if (st->trace_level()) std::cerr << (is_max_ ? "MaxPool" : "AveragePool") << "(quantized, fused) $" << x_ << " -> $" << y_ << std::endl;
        const chainerx::Array x = st->GetArray(x_);
        CHECK_EQ(4, x.ndim());
        auto scalar_or_zero = [&](int slot) -> StrictScalar {
            absl::optional<StrictScalar> z = st->GetOptionalScalar(slot);
            return z.has_value() ? *z : StrictScalar(chainerx::Dtype::kUInt8, chainerx::Scalar(0u), false);
        };
        const float xs = static_cast<float>(st->GetScalar(x_scale_)), ys = static_cast<float>(st->GetScalar(y_scale_));
        const StrictScalar xz = scalar_or_zero(x_zp_), yz = scalar_or_zero(y_zp_);
        const int kh = static_cast<int>(kernel_[0]), kw = static_cast<int>(kernel_[1]);
        const int sh = strides_.empty() ? 1 : static_cast<int>(strides_[0]), sw = strides_.empty() ? 1 : static_cast<int>(strides_[1]);
        int pb[2] = {0, 0}, pe[2] = {0, 0};
        if (pads_.size() == 2) { pb[0] = pe[0] = static_cast<int>(pads_[0]); pb[1] = pe[1] = static_cast<int>(pads_[1]); }
        if (pads_.size() == 4) { pb[0] = static_cast<int>(pads_[0]); pb[1] = static_cast<int>(pads_[1]); pe[0] = static_cast<int>(pads_[2]); pe[1] = static_cast<int>(pads_[3]); }
        auto out_dim = [&](int64_t in, int k, int s, int p0, int p1, bool cover_all) {
            return cover_all ? (in + p0 + p1 - k + s - 1) / s + 1 : (in + p0 + p1 - k) / s + 1;
        };
        const bool cover_all = is_max_ && flag_ != 0;
        const chainerx::Shape shape{x.shape()[0], x.shape()[1], out_dim(x.shape()[2], kh, sh, pb[0], pe[0], cover_all),
                                    out_dim(x.shape()[3], kw, sw, pb[1], pe[1], cover_all)};
        const bool channels_last = !x.IsContiguous() && x.strides()[1] == x.GetItemSize();
        chainerx::Array y = channels_last ? chainerx::EmptyChannelsLastPadded(shape, yz.dtype()) : chainerx::Empty(shape, yz.dtype());
        chx_hip_tensor xt = x.hip(), yt = y.hip();
        if (is_max_) {
            // the maximum of the codes is the quantized maximum only when both sides share the quantization
            CHECK(xs == ys && static_cast<int64_t>(xz) == static_cast<int64_t>(yz) && xz.dtype() == yz.dtype())
                    << "a quantized MaxPool needs the same scale and zero point before and after";
            // (for int8 the kernel returns max + (max < 0): the reference's QuantizeLinear truncates after adding
            // 0.5, so a negative code comes back one higher)
            CHXVM_HIP_CALL(chx_hip_max_pool_q8(&xt, kh, kw, sh, sw, pb[0], pb[1], pe[0], pe[1], cover_all ? 1 : 0, &yt, chainerx::CurrentStream()));
        } else {
            CHECK(pb[0] == pe[0] && pb[1] == pe[1]) << "AveragePool pads must be symmetric";
            CHXVM_HIP_CALL(chx_hip_average_pool_q8(&xt, xs, static_cast<int32_t>(static_cast<int64_t>(xz)), kh, kw, sh, sw, pb[0], pb[1],
                                                   flag_, ys, static_cast<int32_t>(static_cast<int64_t>(yz)), CHX_HIP_ROUND_REFERENCE,
                                                   &yt, chainerx::CurrentStream()));
        }
        st->SetArray(y_, y);
    }

private:
    bool is_max_;
    int x_, x_scale_, x_zp_, y_scale_, y_zp_, y_;
    std::vector<int64_t> kernel_, strides_, pads_;
    int flag_;
};

// MaxPoolOp / AveragePoolOp::RunImpl on a float32 array (runtime/ops/pooling.cc:47-75) that is not between a
// DequantizeLinear and a QuantizeLinear: operands as above.  The second output of the reference's ops, the opaque
// context of a backward pass, is not produced; a program that reads it is refused when it is loaded.
class FloatPoolOp : public ChxVMOp {
public:
    FloatPoolOp(const ChxVMInstructionProto& pool, bool is_max)
        : ChxVMOp(pool), is_max_(is_max), x_(pool.inputs[0].array), y_(pool.outputs[0]), kernel_(pool.inputs[1].ints),
          strides_(pool.inputs[2].ints), pads_(pool.inputs[3].ints), flag_(static_cast<int>(pool.inputs[4].i)) {
        CHECK_EQ(2u, kernel_.size()) << "only 2-D pooling on the hip backend";
        CHECK(pool.outputs.size() < 2 || pool.outputs[1] < 0) << "the backward context of a pool is not produced on the hip backend";
        if (is_max) CHECK(pool.inputs[5].s.empty() || pool.inputs[5].s == "NOTSET") << "auto_pad is not supported for MaxPool on the hip backend";
    }

    void Run(ChxVMState* st) override {
        if (st->trace_level()) std::cerr << (is_max_ ? "MaxPool" : "AveragePool") << "($" << x_ << ") -> $" << y_ << std::endl;
        const chainerx::Array x = st->GetArray(x_);
        CHECK_EQ(4, x.ndim());
        CHECK(x.dtype() == chainerx::Dtype::kFloat32) << "a pool outside a DequantizeLinear / QuantizeLinear pair takes float32, not " << x.dtype();
        const int kh = static_cast<int>(kernel_[0]), kw = static_cast<int>(kernel_[1]);
        const int sh = strides_.empty() ? 1 : static_cast<int>(strides_[0]), sw = strides_.empty() ? 1 : static_cast<int>(strides_[1]);
        int ph = 0, pw = 0;
        if (pads_.size() >= 2) { ph = static_cast<int>(pads_[0]); pw = static_cast<int>(pads_[1]); }
        if (pads_.size() == 4) CHECK(pads_[0] == pads_[2] && pads_[1] == pads_[3]) << "paddings for beginning and end must be the same";
        const bool cover_all = is_max_ && flag_ != 0;
        auto out_dim = [&](int64_t in, int k, int s, int p) { return cover_all ? (in + 2 * p - k + s - 1) / s + 1 : (in + 2 * p - k) / s + 1; };
        const chainerx::Shape shape{x.shape()[0], x.shape()[1], out_dim(x.shape()[2], kh, sh, ph), out_dim(x.shape()[3], kw, sw, pw)};
        chainerx::Array y = chainerx::Empty(shape, chainerx::Dtype::kFloat32);
        chx_hip_tensor xt = x.hip(), yt = y.hip();
        if (is_max_) {
            CHXVM_HIP_CALL(chx_hip_max_pool_f32(&xt, kh, kw, sh, sw, ph, pw, ph, pw, cover_all ? 1 : 0, &yt, chainerx::CurrentStream()));
        } else {
            CHXVM_HIP_CALL(chx_hip_average_pool_f32(&xt, kh, kw, sh, sw, ph, pw, flag_, &yt, chainerx::CurrentStream()));
        }
        st->SetArray(y_, y);
    }

private:
    bool is_max_;
    int x_, y_;
    std::vector<int64_t> kernel_, strides_, pads_;
    int flag_;
};

// A QLinearConv whose result is read only by a residual-sum FusionGroup (and that group): the
// convolution gets the chance to compute the group inside its kernel.  When it does, the group's
// result is stored in the group's output slot now and the group instruction later does nothing;
// when it does not (other quantization constants at run time, operands the kernel does not take),
// both instructions run as they are.
bool g_fuse_residual = true;
bool g_pair_convolutions = true;
bool g_store_minus_128 = true;

struct ResidualFusionState {
    bool fused = false;  // of the current run
};

class QLinearConvWithResidualOp : public ChxVMOp {
public:
    QLinearConvWithResidualOp(const ChxVMInstructionProto& conv, const ChxVMInstructionProto& group, const chx_hip_residual_group& g,
                              int conv_operand, std::shared_ptr<ResidualFusionState> state)
        : ChxVMOp(conv), conv_(MakeChxVMOp(conv)), g_(g), k_(conv_operand), conv_out_(conv.outputs[0]),
          other_(group.inputs[0].array_list[1 - conv_operand]), group_out_(group.outputs[0]), state_(std::move(state)) {
    }
    void InitImpl() override {
        conv_->InitImpl();
    }
    void Run(ChxVMState* st) override {
        QLinearConvResidualRequest req;
        ChxVMVar* other = st->GetVar(other_);
        if (!other->IsNull()) req.r = other->GetArray();
        auto dt = [](int32_t d) { return static_cast<chainerx::Dtype>(d); };
        req.y_scale = g_.in_scale[k_]; req.y_zero_point = g_.in_zero_point[k_]; req.y_dtype = dt(g_.in_dtype[k_]);
        req.r_scale = g_.in_scale[1 - k_]; req.r_zero_point = g_.in_zero_point[1 - k_];
        req.out_scale = g_.out_scale; req.out_zero_point = g_.out_zero_point; req.out_dtype = dt(g_.out_dtype);
        req.relu = g_.relu != 0;
        req.out_slot = group_out_;
        bool r_fits = !req.r.IsNullHandle() && req.r.dtype() == dt(g_.in_dtype[1 - k_]);
        // the other operand kept as code - 128: an int8 tensor with the zero point 128 lower
        const bool r_minus_128 = !req.r.IsNullHandle() && st->store_minus_128(other_) && req.r.dtype() == chainerx::Dtype::kInt8 &&
                                 dt(g_.in_dtype[1 - k_]) == chainerx::Dtype::kUInt8;
        if (r_minus_128) {
            req.r_zero_point -= 128;
            r_fits = true;
        }
        st->set_residual_request(r_fits ? &req : nullptr);
        try {
            conv_->Run(st);
        } catch (...) {
            st->set_residual_request(nullptr);
            throw;
        }
        st->set_residual_request(nullptr);
        state_->fused = req.done;
        if (req.done) {
            if (st->trace_level()) std::cerr << "  (residual sum $" << group_out_ << " computed by the convolution)" << std::endl;
            st->FreeVar(conv_out_);  // holds a null array: the convolution's own result was never written
            st->SetArray(group_out_, req.out);
        } else if (r_minus_128) {
            // the group instruction will run as the program wrote it: it reads plain codes
            const chainerx::Array plain = PlainCodes(req.r);
            st->FreeVar(other_);
            st->SetArray(other_, plain);
        }
    }

private:
    std::unique_ptr<ChxVMOp> conv_;
    chx_hip_residual_group g_;
    int k_, conv_out_, other_, group_out_;
    std::shared_ptr<ResidualFusionState> state_;
};

class ResidualGroupOp : public ChxVMOp {
public:
    ResidualGroupOp(const ChxVMInstructionProto& group, std::shared_ptr<ResidualFusionState> state)
        : ChxVMOp(group), group_(MakeChxVMOp(group)), state_(std::move(state)) {
    }
    void InitImpl() override {
        group_->InitImpl();
    }
    void Run(ChxVMState* st) override {
        if (state_->fused) return;
        group_->Run(st);
    }

private:
    std::unique_ptr<ChxVMOp> group_;
    std::shared_ptr<ResidualFusionState> state_;
};

// A fused op followed by the Free instructions of its operands that the program had placed
// between the instructions it replaces.
class SequenceOp : public ChxVMOp {
public:
    SequenceOp(const ChxVMInstructionProto& inst, std::vector<std::unique_ptr<ChxVMOp>> ops) : ChxVMOp(inst), ops_(std::move(ops)) {
    }
    void InitImpl() override {
        for (auto& op : ops_) op->InitImpl();
    }
    void Run(ChxVMState* st) override {
        for (auto& op : ops_) op->Run(st);
    }

private:
    std::vector<std::unique_ptr<ChxVMOp>> ops_;
};

class NopOp : public ChxVMOp {
public:
    explicit NopOp(const ChxVMInstructionProto& inst) : ChxVMOp(inst) {
    }
    void Run(ChxVMState*) override {
    }
};

// Number of times a variable slot is read by the program.
int CountUses(const ChxVMProgramProto& program, int slot) {
    int n = 0;
    for (const ChxVMInstructionProto& inst : program.instructions)
        for (const ChxVMValueProto& v : inst.inputs) {
            if ((v.type == ChxVMValueProto::ARRAY || v.type == ChxVMValueProto::OPTIONAL_ARRAY) && v.array == slot) ++n;
            if (v.type == ChxVMValueProto::ARRAY_LIST)
                for (int id : v.array_list) n += id == slot;
        }
    return n;
}

}  // namespace

ChxVM::ChxVM(const ChxVMProgramProto& program) : input_names_(program.input_names), input_types_(program.input_types) {
    // number of variable slots = highest id mentioned + 1 (runtime/chxvm.cc:104-140)
    int max_id = -1;
    for (const ChxVMInstructionProto& inst : program.instructions) {
        for (int o : inst.outputs) max_id = o > max_id ? o : max_id;
        for (const ChxVMValueProto& v : inst.inputs) {
            for (int id : {v.array, v.sequence, v.opaque, v.shape, v.scalar}) max_id = id > max_id ? id : max_id;
            for (int id : v.array_list) max_id = id > max_id ? id : max_id;
        }
    }
    num_variables_ = max_id + 1;
    // Find the QLinearMatMul sequences: QuantizeLinear <- MatMul <- two DequantizeLinear, every
    // intermediate read exactly once apart from its Free.
    const int n = static_cast<int>(program.instructions.size());
    const int kDequantize = OpNumber("DequantizeLinear"), kMatMul = OpNumber("MatMul"), kQuantize = OpNumber("QuantizeLinear"),
              kFree = OpNumber("Free"), kMaxPool = OpNumber("MaxPool"), kAveragePool = OpNumber("AveragePool");
    std::vector<int> producer(num_variables_ > 0 ? num_variables_ : 1, -1);
    for (int i = 0; i < n; ++i)
        for (int o : program.instructions[i].outputs)
            if (o >= 0) producer[o] = i;
    std::vector<int> role(n, 0);  // 0 plain, 1 dropped, 2 fused product, 3 fused pool (both at the QuantizeLinear)
    std::vector<std::pair<int, int>> fused_inputs(n);
    auto single_use = [&](int slot) {
        // one consumer plus at most one Free
        int frees = 0;
        for (const ChxVMInstructionProto& inst : program.instructions)
            if (inst.op == kFree && inst.inputs.size() == 1 && inst.inputs[0].array == slot) ++frees;
        return CountUses(program, slot) - frees == 1;
    };
    for (int q = 0; q < n; ++q) {
        const ChxVMInstructionProto& qi = program.instructions[q];
        if (qi.op != kQuantize || qi.inputs.size() != 3 || qi.inputs[0].array < 0) continue;
        const int m = producer[qi.inputs[0].array];
        if (m >= 0 && (program.instructions[m].op == kMaxPool || program.instructions[m].op == kAveragePool) &&
            single_use(qi.inputs[0].array)) {
            // DequantizeLinear -> pool -> QuantizeLinear; the pool's opaque context output must be unused
            const ChxVMInstructionProto& pi = program.instructions[m];
            const bool is_max = pi.op == kMaxPool;
            const bool shape_ok = pi.inputs.size() == (is_max ? 6u : 5u) && pi.inputs[0].array >= 0 &&
                                  (pi.outputs.size() < 2 || pi.outputs[1] < 0);
            const int d = shape_ok ? producer[pi.inputs[0].array] : -1;
            if (d >= 0 && program.instructions[d].op == kDequantize && program.instructions[d].inputs.size() == 3 &&
                single_use(pi.inputs[0].array)) {
                role[q] = 3;
                fused_inputs[q] = std::make_pair(d, m);
                role[m] = role[d] = 1;
            }
            continue;
        }
        if (m < 0 || program.instructions[m].op != kMatMul || !single_use(qi.inputs[0].array)) continue;
        const ChxVMInstructionProto& mi = program.instructions[m];
        const int da = producer[mi.inputs[0].array], db = producer[mi.inputs[1].array];
        if (da < 0 || db < 0 || da == db || program.instructions[da].op != kDequantize ||
            program.instructions[db].op != kDequantize)
            continue;
        if (!single_use(mi.inputs[0].array) || !single_use(mi.inputs[1].array)) continue;
        role[q] = 2;
        fused_inputs[q] = std::make_pair(da, db);
        role[m] = role[da] = role[db] = 1;
    }
    // Two QLinearConv that read the same value with the same activation quantization, strides, pads and kernel size
    // (the main-path and the shortcut convolution of a down-sampling block): the second moves up to the first and the
    // two run as one launch (role 6 = the first, now the pair; role 7 = the second, now nothing).  Every operand of the
    // second must exist where the first stands, or be a literal constant that stands between the two (the compiler
    // emits a constant in front of its first reader): those constants move up as well (role 7, run in front of the
    // pair).  The second's result then exists from the first's place on (`position` says where a value is produced
    // after this move).
    const int kQLinearConv = OpNumber("QLinearConv");
    const std::set<int> literal_ops = {OpNumber("FloatScalarConstant"), OpNumber("IntScalarConstant"), OpNumber("FloatConstant"),
                                       OpNumber("IntConstant")};
    std::vector<int> position(n);
    for (int i = 0; i < n; ++i) position[i] = i;
    std::vector<int> pair_second(n, -1);
    std::vector<std::vector<int>> pair_constants(n);
    for (int i = 0; i < n && g_pair_convolutions; ++i) {
        const ChxVMInstructionProto& ai = program.instructions[i];
        if (ai.op != kQLinearConv || role[i] != 0 || ai.inputs.size() != 13 || ai.outputs.empty()) continue;
        for (int j = i + 1; j < n; ++j) {
            const ChxVMInstructionProto& bi = program.instructions[j];
            if (bi.op == kFree && bi.inputs.size() == 1 && bi.inputs[0].array == ai.inputs[0].array) break;  // x ends here
            if (bi.op != kQLinearConv || role[j] != 0 || bi.inputs.size() != 13 || bi.outputs.empty()) continue;
            if (bi.inputs[0].array != ai.inputs[0].array) continue;
            bool same = bi.inputs[9].ints == ai.inputs[9].ints && bi.inputs[10].ints == ai.inputs[10].ints &&
                        bi.inputs[11].i == 1 && ai.inputs[11].i == 1 && bi.inputs[12].s == ai.inputs[12].s;
            // the second one's operands: produced before the first, or literal constants in between that can move up
            std::vector<int> moved;
            auto available = [&](int slot) {
                if (slot < 0 || producer[slot] < 0) return false;
                const int pr = producer[slot];
                if (pr < i) return role[pr] == 0 || position[pr] < i;
                if (pr > j || role[pr] != 0 || !literal_ops.count(program.instructions[pr].op) || program.instructions[pr].outputs.size() != 1) return false;
                moved.push_back(pr);
                return true;
            };
            for (int k : {1, 2, 6, 7}) same = same && available(bi.inputs[k].scalar);
            for (int k : {3, 4, 5}) same = same && available(bi.inputs[k].array);
            if (bi.inputs[8].array >= 0) same = same && available(bi.inputs[8].array);
            // nothing between the two may free one of them (the compiler frees a value after its last reader, which
            // the second convolution is at the latest)
            for (int f = i; f < j && same; ++f) {
                const ChxVMInstructionProto& fi = program.instructions[f];
                if (fi.op != kFree || fi.inputs.size() != 1) continue;
                for (int k : {3, 4, 5, 8}) same = same && fi.inputs[0].array != bi.inputs[k].array;
                for (int k : {1, 2, 6, 7}) same = same && fi.inputs[0].array != bi.inputs[k].scalar;
            }
            if (!same) continue;
            role[i] = 6;
            role[j] = 7;
            pair_second[i] = j;
            position[j] = i;
            std::sort(moved.begin(), moved.end());
            moved.erase(std::unique(moved.begin(), moved.end()), moved.end());
            for (int c : moved) {
                role[c] = 7;
                position[c] = i;
            }
            pair_constants[i] = moved;
            break;
        }
    }
    // Residual sums: an ElementWiseNvrtc group of the form Q(act(DQ(a) + DQ(b))) one of whose operands
    // is the result of a QLinearConv that nobody else reads, with the other operand produced
    // before that convolution.  role 4 = the convolution, role 5 = the group.
    const int kElementWise = OpNumber("ElementWiseNvrtc");
    std::vector<int> partner(n, -1), conv_operand(n, 0);
    std::vector<chx_hip_residual_group> groups(n);
    for (int e = 0; e < n && g_fuse_residual; ++e) {
        const ChxVMInstructionProto& ei = program.instructions[e];
        if (ei.op != kElementWise || role[e] != 0 || ei.inputs.size() != 4 || ei.inputs[0].array_list.size() != 2 ||
            ei.outputs.size() != 1)
            continue;
        int32_t matches = 0;
        chx_hip_residual_group g;
        if (chx_hip_elementwise_match_residual_add(ei.inputs[2].s.c_str(), &matches, &g) != 0 || !matches) continue;
        for (int k = 1; k >= 0; --k) {
            const int slot = ei.inputs[0].array_list[k], other = ei.inputs[0].array_list[1 - k];
            if (slot < 0 || other < 0 || slot == other) continue;
            const int c = producer[slot];
            if (c < 0 || program.instructions[c].op != kQLinearConv || role[c] != 0 || !single_use(slot)) continue;
            if (producer[other] < 0 || position[producer[other]] >= c) continue;  // the other operand must exist when the convolution runs
            bool other_alive = true;             // ... and still exist: no Free of it before the group
            for (int i = c; i < e; ++i)
                if (program.instructions[i].op == kFree && program.instructions[i].inputs[0].array == other) other_alive = false;
            if (!other_alive) continue;
            role[c] = 4;
            role[e] = 5;
            partner[c] = e;
            partner[e] = c;
            conv_operand[c] = k;
            groups[c] = g;
            break;
        }
    }
    // Values that may be kept as code - 128 in int8 arrays (ChxVMState::store_minus_128): every writer is a QLinearConv
    // or a residual-sum group computed inside one (the producers that know the storage; a writer that runs some other
    // way stores plain codes and the readers see that from the array's type), and every reader is a QLinearConv that
    // without groups that takes the value as its input, or a residual-sum group computed inside a convolution that takes it as the other
    // operand (QLinearConvWithResidualOp puts plain codes back when its convolution does not compute the group after
    // all).  A reading convolution with pads above 1 is left out: it pads with its input's zero point, and beyond one
    // row or column per side only a zero point stored as the byte 0 comes from the padding that costs nothing; the
    // codes of a zero point of 0, the usual one behind a Relu, are stored as 0x80.
    minus_128_slots_.assign(num_variables_ > 0 ? num_variables_ : 1, false);
    if (g_store_minus_128) {
        std::vector<int> verdict(minus_128_slots_.size(), 0);  // 0 unseen, 1 possible so far, -1 no
        auto rule_out = [&](int slot) {
            if (slot >= 0 && slot < static_cast<int>(verdict.size())) verdict[slot] = -1;
        };
        auto candidate = [&](int slot) {
            if (slot >= 0 && slot < static_cast<int>(verdict.size()) && verdict[slot] == 0) verdict[slot] = 1;
        };
        for (int i = 0; i < n; ++i) {
            const ChxVMInstructionProto& inst = program.instructions[i];
            const bool conv = inst.op == kQLinearConv && inst.inputs.size() == 13 && !inst.outputs.empty();
            // writers
            for (size_t o = 0; o < inst.outputs.size(); ++o) {
                const bool knows = (conv && o == 0 && role[i] != 1) || (role[i] == 5 && o == 0);
                if (knows) candidate(inst.outputs[o]);
                else rule_out(inst.outputs[o]);
            }
            // readers
            if (inst.op == kFree) continue;
            int conv_input = -1, residual_operand = -1;
            if (conv && role[i] != 1) {
                bool small_pads = inst.inputs[12].s.empty() || inst.inputs[12].s == "NOTSET" || inst.inputs[12].s == "VALID";
                for (int64_t pad : inst.inputs[10].ints) small_pads = small_pads && pad >= 0 && pad <= 1;
                // (a grouped convolution gains nothing from the storage)
                if (small_pads && inst.inputs[11].i == 1) conv_input = inst.inputs[0].array;
            }
            if (role[i] == 5) residual_operand = inst.inputs[0].array_list[1 - conv_operand[partner[i]]];
            for (const ChxVMValueProto& v : inst.inputs) {
                switch (v.type) {
                    case ChxVMValueProto::ARRAY:
                    case ChxVMValueProto::OPTIONAL_ARRAY:
                        if (!(v.array == conv_input && &v == &inst.inputs[0])) rule_out(v.array);
                        break;
                    case ChxVMValueProto::ARRAY_LIST:
                        for (int id : v.array_list)
                            if (!(id == residual_operand && id != inst.inputs[0].array_list[conv_operand[partner[i]]])) rule_out(id);
                        break;
                    case ChxVMValueProto::SEQUENCE: rule_out(v.sequence); break;
                    case ChxVMValueProto::OPAQUE: rule_out(v.opaque); break;
                    case ChxVMValueProto::SHAPE: rule_out(v.shape); break;
                    case ChxVMValueProto::SCALAR:
                    case ChxVMValueProto::OPTIONAL_SCALAR: rule_out(v.scalar); break;
                    default: break;
                }
            }
        }
        for (size_t v = 0; v < verdict.size(); ++v) minus_128_slots_[v] = verdict[v] == 1;
    }
    // A fused op runs where its last instruction stood but reads the operands of the earlier ones: a
    // Free of such an operand between the two (the compiler frees a value right after its last
    // reader) moves behind the fused op.
    std::vector<std::vector<int>> deferred_frees(n);
    std::vector<bool> deferred(n, false);
    for (int q = 0; q < n; ++q) {
        if (role[q] != 2 && role[q] != 3) continue;
        std::vector<int> dropped = {fused_inputs[q].first, fused_inputs[q].second};
        if (role[q] == 2) dropped.push_back(producer[program.instructions[q].inputs[0].array]);
        std::set<int> operands;
        int first = q;
        for (int d : dropped) {
            first = d < first ? d : first;
            for (const ChxVMValueProto& v : program.instructions[d].inputs) {
                if (v.type == ChxVMValueProto::ARRAY || v.type == ChxVMValueProto::OPTIONAL_ARRAY) operands.insert(v.array);
                if (v.type == ChxVMValueProto::SCALAR || v.type == ChxVMValueProto::OPTIONAL_SCALAR) operands.insert(v.scalar);
            }
        }
        for (int i = first; i < q; ++i) {
            const ChxVMInstructionProto& fi = program.instructions[i];
            if (fi.op == kFree && fi.inputs.size() == 1 && fi.inputs[0].array >= 0 && operands.count(fi.inputs[0].array)) {
                deferred[i] = true;
                deferred_frees[q].push_back(i);
            }
        }
    }
    std::vector<std::shared_ptr<ResidualFusionState>> fusion_state(n);
    std::vector<bool> dead(num_variables_ > 0 ? num_variables_ : 1, false);
    for (int i = 0; i < n; ++i)
        if (role[i] == 1)
            for (int o : program.instructions[i].outputs)
                if (o >= 0) dead[o] = true;
    for (int i = 0; i < n; ++i) {
        const ChxVMInstructionProto& inst = program.instructions[i];
        const bool frees_dead = inst.op == kFree && inst.inputs.size() == 1 && inst.inputs[0].array >= 0 && dead[inst.inputs[0].array];
        if (role[i] == 1 || role[i] == 7 || frees_dead || deferred[i]) {
            program_.emplace_back(new NopOp(inst));
        } else if (role[i] == 6) {
            std::vector<std::unique_ptr<ChxVMOp>> seq;
            for (int c : pair_constants[i]) seq.emplace_back(MakeChxVMOp(program.instructions[c]));
            seq.emplace_back(MakeQLinearConvPairOp(inst, program.instructions[pair_second[i]]));
            program_.emplace_back(new SequenceOp(inst, std::move(seq)));
        } else if (role[i] == 3) {
            const ChxVMInstructionProto& pool = program.instructions[fused_inputs[i].second];
            program_.emplace_back(new FusedQuantizedPoolOp(inst, pool, program.instructions[fused_inputs[i].first], pool.op == kMaxPool));
        } else if (role[i] == 4) {
            fusion_state[i] = std::make_shared<ResidualFusionState>();
            program_.emplace_back(new QLinearConvWithResidualOp(inst, program.instructions[partner[i]], groups[i], conv_operand[i],
                                                                fusion_state[i]));
        } else if (role[i] == 5) {
            program_.emplace_back(new ResidualGroupOp(inst, fusion_state[partner[i]]));
        } else if (role[i] == 2) {
            program_.emplace_back(new FusedQLinearMatMulOp(inst, program.instructions[fused_inputs[i].first],
                                                           program.instructions[fused_inputs[i].second]));
        } else if ((inst.op == kMaxPool || inst.op == kAveragePool) && inst.inputs.size() == (inst.op == kMaxPool ? 6u : 5u) &&
                   inst.inputs[0].array >= 0 && !inst.outputs.empty()) {
            program_.emplace_back(new FloatPoolOp(inst, inst.op == kMaxPool));
        } else {
            program_.emplace_back(MakeChxVMOp(inst));
        }
        if (!deferred_frees[i].empty()) {
            std::vector<std::unique_ptr<ChxVMOp>> seq;
            seq.push_back(std::move(program_.back()));
            for (int f : deferred_frees[i]) seq.emplace_back(MakeChxVMOp(program.instructions[f]));
            program_.back().reset(new SequenceOp(inst, std::move(seq)));
        }
        program_.back()->InitImpl();
    }
}

ChxVM::~ChxVM() = default;

void SetFuseResidual(bool on) {
    g_fuse_residual = on;
}

void SetPairConvolutions(bool on) {
    g_pair_convolutions = on;
}

void SetStoreMinus128(bool on) {
    g_store_minus_128 = on;
}

namespace {

// .npy (format 1.0) with the elements in logical (row-major) order, whatever the strides on the device
void SaveNpy(const chainerx::Array& a, const std::string& filename) {
    static const std::map<chainerx::Dtype, const char*> descr = {
            {chainerx::Dtype::kBool, "|b1"},   {chainerx::Dtype::kInt8, "|i1"},     {chainerx::Dtype::kInt16, "<i2"},
            {chainerx::Dtype::kInt32, "<i4"},  {chainerx::Dtype::kInt64, "<i8"},    {chainerx::Dtype::kUInt8, "|u1"},
            {chainerx::Dtype::kFloat16, "<f2"}, {chainerx::Dtype::kFloat32, "<f4"}, {chainerx::Dtype::kFloat64, "<f8"}};
    auto it = descr.find(a.dtype());
    CHECK(it != descr.end()) << "no .npy type for " << a.dtype();
    const int64_t item = a.GetItemSize(), total = a.GetTotalSize();
    // the bytes the array spans on the device, then a gather by strides on the host
    int64_t span = total ? item : 0;
    for (int i = 0; i < a.ndim() && total; ++i) {
        CHECK_LE(0, a.strides()[i]) << "negative strides in an output dump";
        span += (a.shape()[i] - 1) * a.strides()[i];
    }
    std::vector<char> raw(static_cast<size_t>(span)), packed(static_cast<size_t>(total * item));
    if (span) {
        const chx_hip_tensor t = a.hip();
        CHXVM_HIP_CALL(chx_hip_memcpy_d2h(raw.data(), t.data, static_cast<size_t>(span), chainerx::CurrentStream()));
    }
    std::vector<int64_t> index(static_cast<size_t>(a.ndim()), 0);
    for (int64_t flat = 0; flat < total; ++flat) {
        int64_t off = 0;
        for (int i = 0; i < a.ndim(); ++i) off += index[i] * a.strides()[i];
        std::memcpy(&packed[static_cast<size_t>(flat * item)], &raw[static_cast<size_t>(off)], static_cast<size_t>(item));
        for (int i = a.ndim() - 1; i >= 0; --i) {
            if (++index[i] < a.shape()[i]) break;
            index[i] = 0;
        }
    }
    std::ostringstream header;
    header << "{'descr': '" << it->second << "', 'fortran_order': False, 'shape': (";
    for (int i = 0; i < a.ndim(); ++i) header << a.shape()[i] << (a.ndim() == 1 || i + 1 < a.ndim() ? "," : "") << (i + 1 < a.ndim() ? " " : "");
    header << "), }";
    std::string h = header.str();
    while ((10 + h.size() + 1) % 64 != 0) h += ' ';
    h += '\n';
    std::ofstream ofs(filename, std::ios::binary);
    CHECK(ofs) << "cannot write " << filename;
    const unsigned char magic[10] = {0x93, 'N', 'U', 'M', 'P', 'Y', 1, 0, static_cast<unsigned char>(h.size() & 0xff),
                                     static_cast<unsigned char>(h.size() >> 8)};
    ofs.write(reinterpret_cast<const char*>(magic), 10);
    ofs.write(h.data(), static_cast<std::streamsize>(h.size()));
    ofs.write(packed.data(), static_cast<std::streamsize>(packed.size()));
}

// runtime/chxvm.cc:70-92
void DumpOutput(ChxVMState* st, const ChxVMOp* op, const std::string& output_dir) {
    const ChxVMInstructionProto& inst = op->instruction();
    for (size_t i = 0; i < inst.outputs.size() && i < inst.output_names.size(); ++i) {
        const int id = inst.outputs[i];
        const std::string& name = inst.output_names[i];
        if (id <= 0 || name.empty()) continue;
        // an instruction fused away when the program was loaded leaves its named outputs unset
        ChxVMVar* var = st->PeekVar(id);
        if (!var || !var->IsArray()) continue;
        std::string clean = name;
        for (char& c : clean)
            if (c == '/') c = '_';
        std::ostringstream oss;
        oss << output_dir << '/' << std::setfill('0') << std::setw(5) << inst.id << '_' << clean << ".npy";
        SaveNpy(var->GetArray(), oss.str());
    }
}

chainerx::Shape ShapeOf(const ChxVMTypeProto& type) {
    return chainerx::Shape(type.shape.begin(), type.shape.end());
}

// runtime/chxvm.cc:38-64: an instruction that names its outputs also types them; dtype 0 = untyped
void CheckType(ChxVMState* st, const ChxVMOp* op) {
    const ChxVMInstructionProto& inst = op->instruction();
    if (inst.output_names.empty()) return;
    CHECK_EQ(inst.outputs.size(), inst.output_types.size()) << op->name() << ": " << op->debug_info();
    for (size_t i = 0; i < inst.outputs.size(); ++i) {
        const ChxVMTypeProto& type = inst.output_types[i];
        if (type.dtype == 0) continue;
        const int id = inst.outputs[i];
        CHECK_LT(0, id);
        // unset: the instruction was fused into a neighbour when the program was loaded (or its result freed already)
        ChxVMVar* var = st->PeekVar(id);
        if (!var || var->IsNull() || !var->IsArray()) continue;
        const chainerx::Array& a = st->GetArray(id);
        CHECK_EQ(static_cast<chainerx::Dtype>(type.dtype), a.dtype()) << "Dtype check failed in output #" << i << ": " << op->debug_info();
        CHECK_EQ(ShapeOf(type), a.shape()) << "Shape check failed in output #" << i << ": " << op->debug_info();
    }
}

int64_t InMbs(int64_t bytes) {
    return bytes / 1000 / 1000;
}

}  // namespace

InOuts ChxVM::Run(const InOuts& program_inputs, const ChxVMOptions& options) {
    CHECK_EQ(input_names_.size(), input_types_.size());
    for (size_t i = 0; i < input_names_.size(); ++i) {
        const std::string& name = input_names_[i];
        auto found = program_inputs.find(name);
        CHECK(found != program_inputs.end()) << "Input '" << name << "' not found";  // runtime/chxvm.cc:142-143
        if (!options.check_types) continue;
        const ChxVMTypeProto& type = input_types_[i];
        const ChxVMVar& var = *found->second;
        if (var.IsArray()) {
            if (type.dtype == 0) continue;
            const chainerx::Array& a = var.GetArray();
            CHECK_EQ(static_cast<chainerx::Dtype>(type.dtype), a.dtype()) << "Input '" << name << "' has an unexpected dtype";
            CHECK_EQ(ShapeOf(type), a.shape()) << "Input '" << name << "' has an unexpected shape";
        } else {
            CHECK_EQ(0, type.dtype) << "Input '" << name << "' must be a tensor";
        }
    }
    ChxVMState state(options, num_variables_, program_inputs);
    // (a run that checks result types against the program's or writes results to files sees plain codes everywhere)
    if (!options.check_types && options.dump_outputs_dir.empty()) state.set_minus_128_slots(&minus_128_slots_);
    int64_t peak_used_mbs = 0;
    while (state.pc() < static_cast<int>(program_.size())) {
        const int pc = state.pc();
        ChxVMOp* op = program_[pc].get();
        size_t event = 0;
        if (options.chrome_tracing) event = options.chrome_tracing->Begin("ChxVM", op->name(), pc, op->instruction().flops);
        try {
            op->Run(&state);
        } catch (...) {
            std::cerr << "Exception in " << op->name() << " (pc " << pc << ") " << op->debug_info() << std::endl;
            throw;
        }
        if (options.chrome_tracing) {
            CHXVM_HIP_CALL(chx_hip_stream_synchronize(chainerx::CurrentStream()));
            options.chrome_tracing->End(event);
        }
        state.set_pc(state.pc() + 1);  // jumps set pc - 1 themselves (runtime/ops/controlflow.cc:7-21)
        if (options.check_types) CheckType(&state, op);
        if (!options.dump_outputs_dir.empty()) DumpOutput(&state, op, options.dump_outputs_dir);
        if (options.dump_memory_usage >= 1) {
            const int64_t used_mbs = InMbs(state.GetTotalVariableSize());
            peak_used_mbs = std::max(peak_used_mbs, used_mbs);
            if (options.dump_memory_usage >= 2) std::cerr << " Memory usage=" << used_mbs << "MB" << std::endl;
        }
    }
    if (options.dump_memory_usage >= 1) {
        state.ShowVariableStatus();
        std::cerr << "Peak memory usage=" << peak_used_mbs << "MB" << std::endl;
    }
    residual_fusions_ += state.residual_fusions();
    return state.GetOutputs();
}

}  // namespace runtime
}  // namespace chainer_compiler
