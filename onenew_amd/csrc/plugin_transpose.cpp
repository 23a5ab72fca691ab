// libTranspose_hip.so: the `eval` symbol the oneNew host resolves with dlsym (host/op.h:41-80) for the
// Transpose operator, forwarding to the shared kernel library.
#include "../../include/onenew_hip.h"

extern "C" __attribute__((visibility("default"))) int eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                           BUFFER_INFO_S *outputs) {
    return onhip_transpose_eval(params, inputs, outputs);
}
