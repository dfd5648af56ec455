/* C face of the hip ChxVM runtime (libchxvm_hip_runtime.so), for hosts that embed the VM without
 * C++ linkage -- the role of the pybind module `chainer_compiler_core` in the chainer-compiler tree
 * (tools/run_onnx_core.cc, python/chainer_compiler_core.cc).  Programs are serialized
 * ChxVMProgramProto messages (runtime/chxvm.proto.tmpl); arrays are device memory described by
 * chx_hip_tensor.  Every function returns 0 on success; after a failure chxvm_last_error() holds
 * the message of the failed CHECK (this thread's last one). */
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "chx_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct chxvm_program chxvm_program;
typedef struct chxvm_outputs chxvm_outputs;

const char* chxvm_last_error(void);

/* op enum: 1-based position in the op table; name of 0 or of an unknown number is "?" */
int32_t chxvm_num_ops(void);
const char* chxvm_op_name(int32_t op);
int32_t chxvm_op_number(const char* name);

/* Parses and re-serializes a program (wire-format round trip); *out is malloc'ed, free with chxvm_free. */
int32_t chxvm_proto_roundtrip(const void* bytes, size_t size, void** out, size_t* out_size);
void chxvm_free(void* p);

/* Builds the instruction objects (constants are uploaded, InitImpl runs). */
int32_t chxvm_program_create(const void* bytes, size_t size, chxvm_program** out);
void chxvm_program_destroy(chxvm_program* program);
int32_t chxvm_program_num_instructions(const chxvm_program* program);
int32_t chxvm_program_num_inputs(const chxvm_program* program);
const char* chxvm_program_input_name(const chxvm_program* program, int32_t i);

/* Runs the program.  inputs[i] describes device memory the caller keeps alive until the outputs
 * are destroyed.  trace_level: 0 silent, 1 one line per instruction on stderr, 2 adds values. */
int32_t chxvm_program_run(
        chxvm_program* program,
        const char* const* input_names,
        const chx_hip_tensor* inputs,
        int32_t num_inputs,
        int32_t trace_level,
        chxvm_outputs** out);
int32_t chxvm_outputs_count(const chxvm_outputs* outputs);
const char* chxvm_outputs_name(const chxvm_outputs* outputs, int32_t i);
/* Descriptor of output i (device memory owned by `outputs`). */
int32_t chxvm_outputs_get(const chxvm_outputs* outputs, int32_t i, chx_hip_tensor* out);
void chxvm_outputs_destroy(chxvm_outputs* outputs);

/* One run of the program recorded into a device graph.  A program of the quantized-inference path does the
 * same work on every run, so the run is recorded once and replayed without the host walking the
 * instructions (the reference's interpreter launches every kernel from the host, runtime/chxvm.cc:168-236).
 * capture() runs the program eagerly until its device memory comes out of a pool of the replay's own without
 * growing it (plans are built and launch configurations measured on the way), then records one more run.
 * The inputs are the device buffers of the descriptors: the caller keeps them alive and refills them before a
 * launch.  A program whose run reads results back to the host (data-dependent scalars, as in a dynamically
 * quantized graph; the debugging options) cannot be recorded: capture() fails with the reason, nothing is left
 * recording.  launch() enqueues the recorded run on `stream`, or on the replay's own stream when that is
 * null (synchronize() waits for it); the outputs (same names and shapes on every launch) are device memory of
 * the replay, valid until destroy, rewritten by every launch.  One replay must not be launched concurrently
 * with itself.
 * The recorded kernels address memory of the program's convolution plans (packed weights, transposition and
 * expansion scratch), which eager runs of the same program share.  The plans a recording has used are therefore
 * pinned until the replay is destroyed: an eager run of the program on larger inputs, which would have to move
 * that scratch memory, fails with an error instead (run the largest inputs before capture()), and a plan that
 * the program gives up (other weight operands) is released only with the replay.  Eager runs and launches of a
 * replay of one program must not overlap in time: both write that scratch memory. */
typedef struct chxvm_replay chxvm_replay;
int32_t chxvm_program_capture(
        chxvm_program* program, const char* const* input_names, const chx_hip_tensor* inputs, int32_t num_inputs, chxvm_replay** out);
int32_t chxvm_replay_launch(chxvm_replay* replay, void* stream);
int32_t chxvm_replay_synchronize(chxvm_replay* replay);
const chxvm_outputs* chxvm_replay_outputs(const chxvm_replay* replay);  /* owned by the replay: do not destroy */
/* name "pool_bytes" / "pool_blocks": device memory the replay holds; "warm_runs": eager runs before the recorded one */
int64_t chxvm_replay_info(const chxvm_replay* replay, const char* name);
void chxvm_replay_destroy(chxvm_replay* replay);

/* Options of one program, which override the process-wide ones below.  name "qlinearconv_bias": value
 * "reference", "onnx_int32", or "default" (follow chxvm_set_option again).  Programs with different
 * settings may run in one process, also concurrently. */
int32_t chxvm_program_set_option(chxvm_program* program, const char* name, const char* value);
/* Event counts of one program over all its runs; names as for chxvm_counter.  "minus_128_variables": how many
 * variables of the program the loader marked to be kept as code - 128 between convolutions (fixed at load). */
int64_t chxvm_program_counter(const chxvm_program* program, const char* name);

/* Process-wide defaults, read when a run starts.
 * name "qlinearconv_bias": value "reference" (unscaled float bias, the default) or "onnx_int32";
 * name "fuse_residual": value "on" (default) or "off": whether a QLinearConv read only by a
 * residual-sum group computes that group inside its kernel (decided when a program is loaded);
 * name "pair_convolutions": value "on" (default) or "off": whether two QLinearConv that read the same
 * value with the same strides, pads and kernel size (the main-path and the shortcut convolution of a
 * down-sampling block) run as one launch (decided when a program is loaded);
 * name "store_minus_128": value "on" (default) or "off": whether a uint8 value that only QLinearConv with pads of at most 1
 * read (as input, or as the residual operand of a sum computed inside one) is kept as code - 128 in an int8
 * array between them, which spares the reading kernel its sign flips (decided when a program is loaded; a
 * run with check_types or dump_outputs_dir stores plain codes);
 * name "chrome_tracing": value a file name; every later chxvm_program_run writes its
 * per-instruction timeline there in the Chrome tracing format (the device is synchronized after
 * each instruction while this is on), "" switches it off;
 * name "dump_outputs_dir": value a directory; every later run writes each named array output of
 * each instruction there as <5-digit instruction id>_<name>.npy, "" switches it off. */
int32_t chxvm_set_option(const char* name, const char* value);
/* Process-wide event counts.  name "qlinearconv_residual_fusions": runs of a QLinearConv that
 * computed the residual-sum group behind it inside its kernel; "qlinearconv_pair_fusions": pairs of
 * QLinearConv that ran as one launch; "minus_128_stores": results written as code - 128.  Unknown names give -1. */
int64_t chxvm_counter(const char* name);

/* BackendConfig queries.  `config` is a built-in name ("chxvm", "chxvm_test", "hip") or, with
 * is_json != 0, a JSON document.  section: "simplify_preproc", "simplify", "merge",
 * "expanding_functions" (membership) or "supported_ops" (HasOp).  *out = 0 or 1. */
int32_t chxvm_backend_config_has(const char* config, int32_t is_json, const char* section, const char* key, int32_t* out);
/* Name of the configuration ("custom" for a JSON document) into buf. */
int32_t chxvm_backend_config_name(const char* config, int32_t is_json, char* buf, size_t buf_size);

#ifdef __cplusplus
}
#endif
