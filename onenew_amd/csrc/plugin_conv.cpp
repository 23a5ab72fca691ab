// libConv_hip.so: the `eval` symbol the oneNew host resolves with dlsym (host/op.h:41-80) for the
// Conv operator, forwarding to the shared kernel library.
#include "../../include/onenew_hip.h"

extern "C" __attribute__((visibility("default"))) int eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                           BUFFER_INFO_S *outputs) {
    return onhip_conv_eval(params, inputs, outputs);
}

// Not in the reference: the convolution that ends a residual block together with the Add (and the Relu) after it.
// Slots as for `eval`, plus inputs[3] = the other operand of the Add (a tensor of the output's shape); outputs[0]
// receives the block's result.  The device-resident runtime calls these when a model has that pattern.
extern "C" __attribute__((visibility("default"))) int eval_add(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                               BUFFER_INFO_S *outputs) {
    return onhip_conv_add_eval(params, inputs, outputs);
}

// Not in the reference: a whole inverted-residual block, Conv (1x1) -> Conv (depthwise 3x3) -> Conv (1x1) [-> Add], as one
// call.  Slots as for the first convolution's `eval` with the block's result operand in params[4] and outputs[0];
// inputs[3] = the addend or null; params[5], params[6], inputs[5], inputs[6] = the depthwise convolution's CONV_CONFIG_S,
// weight operand, weights and bias; params[7], params[8], inputs[7], inputs[8] = the same of the last convolution.
// eval_block_takes: same params, no tensors touched; 1 when the library recommends the call for these shapes, else 0.
extern "C" __attribute__((visibility("default"))) int eval_block(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                 BUFFER_INFO_S *outputs) {
    return onhip_conv_block_eval(params, inputs, outputs);
}
extern "C" __attribute__((visibility("default"))) int eval_block_takes(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                       BUFFER_INFO_S *outputs) {
    return onhip_conv_block_takes(params, inputs, outputs);
}

// Not in the reference: a dense convolution with at most 64 output channels and the 1x1 convolution over its result
// [-> Add [-> Relu]] as one call.  Slots as for the first convolution's `eval` with the pair's result operand in params[4]
// and outputs[0]; inputs[3] = the addend or null; params[5], params[6], inputs[5], inputs[6] = the second convolution's
// CONV_CONFIG_S, weight operand, weights and bias.  eval_pair_relu: with the Relu after the Add.  eval_pair_takes: same
// params, no tensors touched; 1 when the library recommends the call for these shapes, else 0.
extern "C" __attribute__((visibility("default"))) int eval_pair(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                BUFFER_INFO_S *outputs) {
    return onhip_conv_pair_eval(params, inputs, outputs);
}
extern "C" __attribute__((visibility("default"))) int eval_pair_relu(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                     BUFFER_INFO_S *outputs) {
    return onhip_conv_pair_relu_eval(params, inputs, outputs);
}
extern "C" __attribute__((visibility("default"))) int eval_pair_takes(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                      BUFFER_INFO_S *outputs) {
    return onhip_conv_pair_takes(params, inputs, outputs);
}

extern "C" __attribute__((visibility("default"))) int eval_add_relu(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                    BUFFER_INFO_S *outputs) {
    return onhip_conv_add_relu_eval(params, inputs, outputs);
}

// Not in the reference: a dense int8 convolution inside a chain of them, taking and/or leaving its activations as int8
// NHWC.  Slots as for `eval`; inputs[4] = {int32 in_s8, int32 out_s8, float out_scale, int32 twin} in host memory (twin:
// outputs[1] = device buffer that receives an fp32 result with a folded Add once more as int8 NHWC); inputs[5] = null or
// an int32 fold code (1 Add, 2 Add + Relu, the other operand in inputs[3]).
extern "C" __attribute__((visibility("default"))) int eval_link(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                BUFFER_INFO_S *outputs) {
    return onhip_conv_link_eval(params, inputs, outputs);
}

// eval_link_takes: params[0..2] only, no tensors touched; 1 when eval_link can run this convolution (dense int8, or a
// depthwise int8 shape the NHWC kernel takes), else 0.
extern "C" __attribute__((visibility("default"))) int eval_link_takes(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                      BUFFER_INFO_S *outputs) {
    return onhip_conv_link_takes(params, inputs, outputs);
}
