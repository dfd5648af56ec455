/* C face of the compiler side: ONNX model in, passes (quantizer, fusion), ChxVM program out.
 * The role of the reference's `run_onnx --quantize --fuse_operations ... --out_onnx / --dump`
 * front end over compiler/passes.cc:84-170 of the chainer-compiler tree, for the hip backend.
 * All functions return 0 on success; chxvm_last_error() (chxvm_capi.h) has the message otherwise.
 *
 * options: a JSON document (// comments allowed), every member optional:
 *   {"quantize": {"mode": "IntegerOps" | "QLinearOps",      // default IntegerOps (compiler/passes.cc:121-125)
 *                 "per_channel": true, "static": false, "asymmetric_input_types": false,   // defaults of compiler/quantize.h:30-40
 *                 "inputs":  {"<value name>": {"scale": 0.02, "zero_point": 128}},
 *                 "outputs": {"<value name>": {"scale": 0.05, "zero_point": 128, "dtype": "uint8" | "int8"}}},
 *    "fuse": "hip" | "nvrtc" | "none"}                      // default "hip"; "nvrtc" = the reference's fusable set
 * The reference's own flag names (scripts/generate_flags_code.py:4-173) are accepted as members too:
 *   "quantize": true (the default mode), "disable_per_channel_quantize": bool, "backend_name": "hip", and, when
 *   "fuse" is absent, "fuse_operations" with "use_hip" / "use_nvrtc" (no groups unless fuse_operations is true).
 */
#pragma once

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Runs the passes and emits a serialized ChxVMProgramProto; release *program with chxc_free. */
int32_t chxc_compile(const void* onnx_model, size_t size, const char* options_json, void** program, size_t* program_size);

/* Runs the passes only.  *out_model: the graph as a serialized ONNX ModelProto (fusion groups
 * written as the nodes they hold); *description: one line per node in topological order,
 * "Op(in, ...) -> (out, ...)", a fusion group followed by " [type #id: Op Op ...]".  Release both
 * with chxc_free.  Either output pointer may be NULL. */
int32_t chxc_transform(const void* onnx_model, size_t size, const char* options_json, void** out_model, size_t* out_size,
                       char** description);

/* The hip program text of fusion group number `group` (1-based) of the transformed graph. */
int32_t chxc_fusion_program(const void* onnx_model, size_t size, const char* options_json, int32_t group, char** text);

/* compiler/quantize.cc:68-89 on one float tensor: qtype 6 (uint8) or 2 (int8); codes as int32. */
int32_t chxc_quantize_data(const float* data, size_t n, int32_t qtype, float* scale, int64_t* zero_point, int32_t* codes);

void chxc_free(void* p);

#ifdef __cplusplus
}
#endif
