/*
 * Model-level C ABI of the MI355X (gfx950) CVM backend.
 *
 * These are the twelve functions of the reference's C API
 * (include/cvm/c_api.h:29-52, identical copy kernel/c_api.h:26-49; implemented
 * in src/core/c_api.cc:22-152) with the same names, argument meaning, status
 * codes and ownership rules, so the existing bindings -- Go via dlopen/dlsym
 * (kernel/dlopen.h:48-78, kernel/libcvm.go:57-141), Python ctypes
 * (python/cvm/_ctypes/runtime.py) -- load this library unchanged.
 *
 * device_type (reference: 0 CPU, 1 GPU, 2 FORMAL, src/core/c_api.cc:15-20):
 * this library serves 1 (GPU) and 3 (HIP) with the gfx950 backend.  Types 0 and
 * 2 name backends that are not built into this library and fail with
 * ERROR_RUNTIME, as the reference does for a backend it was built without.
 *
 * Errors never cross the ABI as exceptions: every function returns SUCCEED,
 * ERROR_LOGIC (a VERIFY on the model or arguments failed) or ERROR_RUNTIME and
 * prints "ERROR: <message>" on stdout (include/cvm/errors.h:15-36).
 * One `net` must not be used from two threads at once.
 */
#ifndef CVM_C_API_H_
#define CVM_C_API_H_

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

enum { SUCCEED = 0, ERROR_LOGIC = 1, ERROR_RUNTIME = 2 };

/* c_api.cc:22-43.  *net is owned by the library until CVMAPIFreeModel. */
int CVMAPILoadModel(const char* graph_json, int graph_strlen,
                    const char* param_bytes, int param_strlen,
                    void** net, int device_type, int device_id);
/* c_api.cc:46-51 */
int CVMAPIFreeModel(void* net);
/* c_api.cc:53-77.  input_len must equal CVMAPIGetInputLength; output_data must
 * hold CVMAPIGetOutputLength bytes. */
int CVMAPIInference(void* net, char* input_data, int input_len, char* output_data);

/* c_api.cc:79-95: copy at most 32 characters plus NUL */
int CVMAPIGetVersion(void* net, char* version);
int CVMAPIGetPreprocessMethod(void* net, char* method); /* returns the *postprocess* string */

/* c_api.cc:97-127 */
int CVMAPIGetInputLength(void* net, unsigned long long* size);
int CVMAPIGetOutputLength(void* net, unsigned long long* size);
int CVMAPIGetInputTypeSize(void* net, unsigned long long* size);
int CVMAPIGetOutputTypeSize(void* net, unsigned long long* size);

/* c_api.cc:129-152 */
int CVMAPIGetStorageSize(void* net, unsigned long long* gas);
int CVMAPIGetGasFromModel(void* net, unsigned long long* gas);
int CVMAPIGetGasFromGraphFile(const char* graph_json, unsigned long long* gas);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* CVM_C_API_H_ */
