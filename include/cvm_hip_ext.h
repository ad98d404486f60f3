/*
 * Additions of the gfx950 backend that have no counterpart in the reference's
 * C API.  They exist for measurement and for testing the host logic; a caller
 * that only knows include/cvm_c_api.h never needs them.
 */
#ifndef CVM_HIP_EXT_H_
#define CVM_HIP_EXT_H_

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

/* CVMAPIInference split in its three stages (src/core/model.cc:154-291):
 * stage the input on the device, run the graph, fetch and post-process the
 * outputs.  Lets a harness time the device-resident part alone. */
int CVMHIPSetInput(void* net, const char* input_data, int input_len);
int CVMHIPRun(void* net);
int CVMHIPGetOutput(void* net, char* output_data);
/* Runs the graph `iterations` times on the input already on the device and
 * returns the elapsed device time in milliseconds, measured with events
 * recorded on the runtime's own stream. */
int CVMHIPTimeRun(void* net, int iterations, float* elapsed_ms);
/* What a run of the model issues: kernel launches per run, how many of them are layer-sequence launches
 * (cvmhip_conv_seq_launch) and how many convolutions those contain.  Any pointer may be NULL. */
int CVMHIPLaunchCounts(void* net, int* launches_per_run, int* sequence_launches, int* layers_in_sequences);
/* The configuration of the tile kernel chosen for every convolution inside the model's layer-sequence launches, in
 * order: *count receives how many there are, the first min(capacity, *count) are written to configs (may be NULL). */
int CVMHIPSequenceConfigs(void* net, int* configs, int capacity, int* count);
/* Per-operator device time of one run as a JSON object {"op": ms, ...}
 * (the table the reference prints under -DPROFILE, graph_runtime.cc:62-87). */
int CVMHIPProfileOps(void* net, char* json_out, int capacity);

/* Host-side inference for ONE node, no device needed: parses `attr_json`
 * (string-valued dict) and applies the operator's shape and precision rules
 * (src/top/**).  Shapes are rows of 6 int64.  Returns SUCCEED / ERROR_LOGIC /
 * ERROR_RUNTIME with the message in err. */
int CVMHIPInferNode(const char* op, const char* attr_json, int n_in,
                    const long long* in_shapes, const int* in_ndims, const int* in_precs,
                    int* n_out, long long* out_shapes, int* out_ndims, int* out_precs,
                    char* err, int errlen);
/* ONE registered operator on host tensors: the single-operator call that the reference's own operator
 * test makes for each case directory (tests/test_op.cc:479-660: parse the attributes, FInferShape,
 * allocate, copy in, call cvm.runtime.<dev>.<op> with its extra space, copy out).  int32 tensors, shapes
 * as rows of 6 int64.  Outputs are first filled from the caller's buffers (some operators leave part of
 * an output untouched), `out_capacity[i]` is the room of `out_data[i]` in elements.  With
 * `out_data == NULL` only the attributes are parsed and the output shapes inferred (no device needed).
 * `*failed_stage` tells what a non-zero status came from: 0 = attributes / shape inference (the failure
 * a case directory announces in err.txt), 1 = execution.  Returns SUCCEED / ERROR_LOGIC / ERROR_RUNTIME
 * with the message in err. */
int CVMHIPRunOp(const char* op, const char* attr_json, int n_in,
                const long long* in_shapes, const int* in_ndims, const int* const* in_data,
                int max_out, int* n_out, long long* out_shapes, int* out_ndims,
                int* const* out_data, const long long* out_capacity,
                int* failed_stage, char* err, int errlen);
/* Newline-separated names registered for the device: cvm.runtime.hip.<op> */
int CVMHIPListOps(char* out, int capacity);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* CVM_HIP_EXT_H_ */
