/*
 * plaidml/exec/ffi.h -- execution part of the C ABI (reference: plaidml/exec/ffi.h:11-40).
 * plaidml_jit binds a compiled program to a device ("hip.0"; an empty string means
 * the PLAIDML_DEVICE setting, reference plaidml/exec/ffi.cc:61-73) and
 * plaidml_executable_run checks arity and shapes, runs, and returns the
 * execution time in milliseconds (reference plaidml/exec/ffi.cc:83-123).
 */
#ifndef PLAIDML_EXEC_FFI_H_
#define PLAIDML_EXEC_FFI_H_

#include "plaidml/core/ffi.h"

#ifdef __cplusplus
extern "C" {
#endif

void plaidml_exec_init(plaidml_error* err);
plaidml_strings* plaidml_devices_get(plaidml_error* err);
plaidml_executable* plaidml_jit(plaidml_error* err, plaidml_program* program, const char* device);
void plaidml_executable_free(plaidml_error* err, plaidml_executable* exec);
double plaidml_executable_run(plaidml_error* err, plaidml_executable* exec, size_t ninputs, plaidml_buffer** inputs,
                              size_t noutputs, plaidml_buffer** outputs);

#ifdef __cplusplus
}
#endif
#endif /* PLAIDML_EXEC_FFI_H_ */
