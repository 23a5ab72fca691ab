// libMatMul_hip.so: the `eval` symbol the oneNew host resolves with dlsym (host/op.h:41-80) for the
// MatMul operator, forwarding to the shared kernel library.
#include "../../include/onenew_hip.h"

extern "C" __attribute__((visibility("default"))) int eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                           BUFFER_INFO_S *outputs) {
    return onhip_matmul_eval(params, inputs, outputs);
}

// Not in the reference: MatMul(q, Transpose(k)) -> Softmax -> MatMul(., v) of an attention block as one call.  Slots:
// params[1..3] / inputs[0..2] = q, k (as it is before its Transpose), v, all [..., tokens, head_dim]; params[4] /
// outputs[0] = the result.  inputs[4]: null, or four int32 flags (q, k, v, result): non-zero = that rank-4 tensor is stored
// [batch, tokens, heads, head_dim] (the other side of a head-split / head-merge Transpose (0, 2, 1, 3), which the caller
// then leaves out) and its operand carries that shape.  The device-resident runtime calls it when a model has that pattern and the shape is one the
// fused kernel takes (head_dim 32 or 64, at most 256 tokens).
extern "C" __attribute__((visibility("default"))) int eval_attention(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                     BUFFER_INFO_S *outputs) {
    return onhip_matmul_attention_eval(params, inputs, outputs);
}

// Not in the reference: MatMul -> Add of a bias over the last axis (-> Gelu) as one call, the linear layers of a
// transformer block.  Slots as for `eval`, plus params[3] / inputs[2] = the bias (as many elements as the result has
// columns); the result's operand moves to params[4]; eval_bias_gelu reads the Gelu table from inputs[11] like the Gelu
// operator (host/ops/gelu.h:80-96).  Values equal those of the separate operators bit for bit.
extern "C" __attribute__((visibility("default"))) int eval_bias(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                BUFFER_INFO_S *outputs) {
    return onhip_matmul_bias_eval(params, inputs, outputs);
}
extern "C" __attribute__((visibility("default"))) int eval_bias_gelu(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                     BUFFER_INFO_S *outputs) {
    return onhip_matmul_bias_gelu_eval(params, inputs, outputs);
}
// eval_bias -> Add of a tensor shaped like the result (the skip connection after a projection): the addend's address in
// inputs[3], as with the Conv plugin's eval_add.
extern "C" __attribute__((visibility("default"))) int eval_bias_add(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs,
                                                                    BUFFER_INFO_S *outputs) {
    return onhip_matmul_bias_add_eval(params, inputs, outputs);
}
