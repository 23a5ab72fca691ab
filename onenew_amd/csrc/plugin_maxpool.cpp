// libMaxPool_hip.so: the `eval` symbol the oneNew host resolves with dlsym (host/op.h:41-80) for the
// MaxPool operator, forwarding to the shared kernel library.
#include "../../include/onenew_hip.h"

extern "C" __attribute__((visibility("default"))) int eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                           BUFFER_INFO_S *outputs) {
    return onhip_maxpool_eval(params, inputs, outputs);
}

// Not in the reference: the same operator on int8 NHWC tensors (channels padded to 16), between int8 convolutions whose
// operands travel that way.  Slots and operand descriptors (NCHW shapes) as for `eval`.
extern "C" __attribute__((visibility("default"))) int eval_s8(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                              BUFFER_INFO_S *outputs) {
    return onhip_maxpool_s8_eval(params, inputs, outputs);
}
