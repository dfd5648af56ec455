#include "chxvm_state.h"

#include <algorithm>
#include <iostream>
#include <map>
#include <sstream>

namespace chainer_compiler {
namespace runtime {

ChxVMState::ChxVMState(const ChxVMOptions& options, int num_variables, const InOuts& inputs)
    : variables_(num_variables), inputs_(inputs), options_(options) {
}

ChxVMVar* ChxVMState::GetVar(int index) {
    CHECK_LE(0, index) << "negative variable id";
    CHECK_GT(static_cast<int>(variables_.size()), index);
    CHECK(variables_[index].get()) << "variable $" << index << " is read before it is set";
    return variables_[index].get();
}

ChxVMVar* ChxVMState::PeekVar(int index) {
    if (index < 0 || index >= static_cast<int>(variables_.size())) return nullptr;
    return variables_[index].get();
}

void ChxVMState::SetVar(int index, const ChxVMVar& var) {
    CHECK_LE(0, index);
    CHECK_GT(static_cast<int>(variables_.size()), index);
    // a slot is written once between two Free's (runtime/chxvm_state.cc:171-176)
    CHECK(!variables_[index].get()) << "variable $" << index << " is set twice";
    variables_[index].reset(new ChxVMVar(var));
}

chainerx::Array ChxVMState::GetArray(int index) {
    return GetVar(index)->GetArray();
}

absl::optional<chainerx::Array> ChxVMState::GetOptionalArray(int index) {
    if (index < 0) return absl::nullopt;  // -1 marks an absent optional operand
    return GetArray(index);
}

void ChxVMState::SetArray(int index, const chainerx::Array& value) {
    SetVar(index, ChxVMVar(value));
}

void ChxVMState::FreeVar(int index) {
    CHECK_LE(0, index);
    CHECK_GT(static_cast<int>(variables_.size()), index);
    variables_[index].reset();
}

std::vector<chainerx::Array> ChxVMState::GetArrayList(const std::vector<int>& index) {
    std::vector<chainerx::Array> out;
    for (int i : index) out.push_back(GetArray(i));
    return out;
}

void ChxVMState::SetArrayList(const std::vector<int>& index, const std::vector<chainerx::Array>& vars) {
    CHECK_EQ(index.size(), vars.size());
    for (size_t i = 0; i < index.size(); ++i) SetArray(index[i], vars[i]);
}

const chainerx::Shape& ChxVMState::GetShape(int index) {
    return GetVar(index)->GetShape();
}

void ChxVMState::SetShape(int index, chainerx::Shape s) {
    SetVar(index, ChxVMVar(s));
}

const StrictScalar& ChxVMState::GetScalar(int index) {
    return GetVar(index)->GetScalar();
}

absl::optional<StrictScalar> ChxVMState::GetOptionalScalar(int index) {
    if (index < 0) return absl::nullopt;
    return GetScalar(index);
}

void ChxVMState::SetScalar(int index, StrictScalar s) {
    SetVar(index, ChxVMVar(s));
}

std::string ChxVMState::GetVarString(int index) {
    if (index < 0) return "null";
    return GetVar(index)->ToString();
}

std::string ChxVMState::GetVarListString(const std::vector<int>& indices) {
    std::ostringstream oss;  // "[a, b]" as runtime/chxvm_state.cc:147-167 prints a list
    oss << '[';
    for (size_t i = 0; i < indices.size(); ++i) oss << (i ? ", " : "") << GetVarString(indices[i]);
    oss << ']';
    return oss.str();
}

namespace {

bool HasNonFinite(const ChxVMVar& var, bool infinities) {
    if (var.kind() != ChxVMVar::Kind::kArray) return false;  // scalars live on the host and are what the program says
    const chainerx::Array& a = var.GetArray();
    if (a.dtype() != chainerx::Dtype::kFloat32 || a.GetTotalSize() == 0) return false;
    chx_hip_tensor t = a.hip();
    int64_t count = 0;
    CHXVM_HIP_CALL(chx_hip_count_nonfinite(&t, infinities ? 1 : 0, &count, chainerx::CurrentStream()));
    return count != 0;
}

}  // namespace

void ChxVMState::CheckNonFinite(const std::vector<int>& inputs, const std::vector<int>& outputs, bool infinities) {
    for (int output : outputs) {
        if (output < 0) continue;
        if (!HasNonFinite(*GetVar(output), infinities)) continue;
        std::ostringstream oss;
        oss << (infinities ? "Inf" : "NaN") << " detected!\n";
        for (size_t i = 0; i < inputs.size(); ++i) oss << "input #" << i << ": " << GetVarString(inputs[i]) << "\n";
        for (size_t i = 0; i < outputs.size(); ++i) oss << "output #" << i << ": " << GetVarString(outputs[i]) << "\n";
        std::cerr << oss.str();
        CHECK(false) << oss.str();
    }
}

void ChxVMState::CheckNans(const std::vector<int>& inputs, const std::vector<int>& outputs) {
    CheckNonFinite(inputs, outputs, false);
}

void ChxVMState::CheckInfs(const std::vector<int>& inputs, const std::vector<int>& outputs) {
    CheckNonFinite(inputs, outputs, true);
}

int64_t ChxVMState::GetTotalVariableSize() const {
    std::map<const void*, int64_t> sizes;
    for (const auto& v : variables_) {
        if (!v || !v->IsArray()) continue;
        const chainerx::Array& a = v->GetArray();
        if (a.IsNullHandle()) continue;
        int64_t& bytes = sizes[a.raw_data()];
        bytes = std::max(bytes, a.GetNBytes());
    }
    int64_t total = 0;
    for (const auto& p : sizes) total += p.second;
    return total;
}

void ChxVMState::ShowVariableStatus() const {
    for (size_t i = 0; i < variables_.size(); ++i) {
        if (!variables_[i]) continue;
        std::cerr << "$" << i << ": " << variables_[i]->GetNBytes() << std::endl;
    }
}

void ChxVMState::Input(const std::string& name, int index) {
    auto found = inputs_.find(name);
    CHECK(found != inputs_.end()) << "Input value not exist: " << name;  // runtime/chxvm_state.cc Input()
    SetVar(index, *found->second);
}

void ChxVMState::Output(const std::string& name, int index) {
    CHECK(outputs_.emplace(name, std::make_shared<ChxVMVar>(*GetVar(index))).second) << "Duplicated output name: " << name;
}

}  // namespace runtime
}  // namespace chainer_compiler
