/*
 * plaidml/op/ffi.h -- the operation library's single entry point
 * (reference: plaidml/op/ffi.h:11-14, dispatch table plaidml/op/lib/ops.cc:3632-3681).
 */
#ifndef PLAIDML_OP_FFI_H_
#define PLAIDML_OP_FFI_H_

#include "plaidml/core/ffi.h"

#ifdef __cplusplus
extern "C" {
#endif

plaidml_value* plaidml_op_make(plaidml_error* err, const char* op_name, plaidml_value* value);

#ifdef __cplusplus
}
#endif
#endif /* PLAIDML_OP_FFI_H_ */
