// The quantizer pass: float Conv / MatMul nodes become their quantized forms, the rewrite of
// compiler/quantize.cc of the chainer-compiler tree (options: compiler/quantize.h).
//   IntegerOps: QuantizeLinear -> ConvInteger | MatMulInteger -> Cast(float) -> Mul(x_scale * w_scale)
//   QLinearOps: QuantizeLinear -> QLinearConv | QLinearMatMul -> DequantizeLinear
// Weights (operands with a constant behind them) are quantized here, on the host; activations get a
// QuantizeLinear whose scale and zero point are constants from the options (static) or a small
// ReduceMin / ReduceMax sub-graph (dynamic).
#pragma once

#include <map>
#include <string>

#include "graph.h"

namespace chainer_compiler {

enum class QuantizationMode { IntegerOps, QLinearOps };

struct QuantizationParams {
    float scale = 1.f;
    int64_t zero_point = 0;
    CDtype zero_point_dtype = kUInt8;
};

struct QuantizationOptions {
    int nbits = 8;
    bool per_channel = true;  // compiler/quantize.h:34; --disable_per_channel_quantize clears it (compiler/passes.cc:123)
    bool is_static = false;
    bool asymmertic_input_types = false;  // (spelled as in the reference) int8 weights instead of uint8
    QuantizationMode mode = QuantizationMode::IntegerOps;
    std::map<std::string, QuantizationParams> input_quantization_params;   // by the name of the float operand
    std::map<std::string, QuantizationParams> output_quantization_params;  // by the name of the node's output
};

// Returns whether anything was rewritten.
bool Quantize(const QuantizationOptions& opts, Graph* graph);

// Replaces every DynamicQuantizeLinear node by the body of the ONNX function of that name
// (what the FunctionExpander of compiler/simplifier.cc:825-888 does with the schema's function,
// enabled by configs/chxvm.json:55-57): ReduceMin/ReduceMax, the range widened to contain 0,
// scale = range / 255, zero point = Cast(Round(Clip(0 - min / scale, 0, 255))), QuantizeLinear.
// Returns the number of nodes replaced.
int ExpandDynamicQuantizeLinear(Graph* graph);

// One tensor quantized the way the pass quantizes weights (compiler/quantize.cc:68-89), exposed for tests.
struct QuantizedData {
    float rmin, rmax, scale;
    int64_t zero_point;
    std::vector<int32_t> data;  // the codes
};
QuantizedData QuantizeData(const std::vector<float>& data, CDtype qtype);

}  // namespace chainer_compiler
