/* Prints sizes and member offsets of the structs that cross the backend boundary, as JSON.
 * Compiled twice: against the reference's include tree (make_golden.py -> abi_layout.json)
 * and against this repository's include/ (tests/test_host_core.py); the two must agree. */
#include <stddef.h>
#include <stdio.h>

#include "axiom/internal/backend_ops.h"
#include "axiom/layer.h"
#include "axiom/quantize.h"
#include "axiom/tensor.h"

#define OFF(type, member) printf("  \"%s.%s\": %zu,\n", #type, #member, offsetof(type, member))
#define SIZE(type) printf("  \"sizeof(%s)\": %zu,\n", #type, sizeof(type))
#define VAL(name) printf("  \"%s\": %d,\n", #name, (int)(name))

int main(void) {
    printf("{\n");
    SIZE(ax_storage_t);
    OFF(ax_storage_t, data); OFF(ax_storage_t, size_bytes); OFF(ax_storage_t, refcount);
    OFF(ax_storage_t, device); OFF(ax_storage_t, is_arena_temp); OFF(ax_storage_t, generation);
    SIZE(ax_tensor_t);
    OFF(ax_tensor_t, storage); OFF(ax_tensor_t, shape); OFF(ax_tensor_t, strides); OFF(ax_tensor_t, ndim);
    OFF(ax_tensor_t, dtype); OFF(ax_tensor_t, offset); OFF(ax_tensor_t, requires_grad);
    OFF(ax_tensor_t, grad); OFF(ax_tensor_t, grad_fn); OFF(ax_tensor_t, layout);
    SIZE(ax_qweight_t);
    OFF(ax_qweight_t, data); OFF(ax_qweight_t, scales); OFF(ax_qweight_t, N); OFF(ax_qweight_t, K);
    SIZE(ax_layer_t); SIZE(ax_dense_t); SIZE(ax_sequential_t);
    OFF(ax_layer_t, ops); OFF(ax_layer_t, type); OFF(ax_layer_t, params); OFF(ax_layer_t, n_params);
    OFF(ax_layer_t, input_features); OFF(ax_layer_t, output_features);
    OFF(ax_dense_t, weight); OFF(ax_dense_t, bias); OFF(ax_dense_t, use_bias);
    OFF(ax_sequential_t, layers); OFF(ax_sequential_t, n_layers);
#define SLOT(m) OFF(struct ax_backend_ops, m)
    SLOT(name); SLOT(add); SLOT(sub); SLOT(mul); SLOT(div_op); SLOT(neg); SLOT(abs_op); SLOT(exp_op);
    SLOT(log_op); SLOT(sqrt_op); SLOT(square); SLOT(add_scalar); SLOT(mul_scalar); SLOT(gemm);
    SLOT(gemm_nt); SLOT(gemm_tn); SLOT(dwqkv_split_acc); SLOT(dwqkv_split_acc_hm); SLOT(qkv_head_gemm);
    SLOT(dattn_head_gemm_nt); SLOT(mha_output_proj_fused); SLOT(gemm_relu); SLOT(gemm_ex); SLOT(add_relu);
    SLOT(axpy); SLOT(softmax_rowwise); SLOT(bias_add); SLOT(conv_gemm); SLOT(conv_gemm_nt_dw); SLOT(sum);
    SLOT(mean); SLOT(max_op); SLOT(min_op); SLOT(argmax); SLOT(equal); SLOT(greater); SLOT(fill); SLOT(copy);
    SLOT(relu); SLOT(sigmoid); SLOT(tanh_op); SLOT(leaky_relu); SLOT(elu_op); SLOT(gelu_op); SLOT(swish_op);
    SLOT(adam_update); SLOT(sgd_update); SLOT(device); SLOT(init); SLOT(shutdown); SLOT(synchronize);
    SLOT(device_count); SLOT(storage_alloc); SLOT(storage_free); SLOT(memcpy_h2d); SLOT(memcpy_d2h);
    SLOT(memcpy_d2d);
    VAL(AX_OK); VAL(AX_ERR_NULL_ARG); VAL(AX_ERR_ALLOC); VAL(AX_ERR_SHAPE_MISMATCH); VAL(AX_ERR_DTYPE_MISMATCH);
    VAL(AX_ERR_INVALID_AXIS); VAL(AX_ERR_BACKEND); VAL(AX_ERR_NOT_IMPLEMENTED); VAL(AX_ERR_INTERNAL);
    VAL(AX_FLOAT32); VAL(AX_INT32); VAL(AX_UINT8); VAL(AX_DEVICE_CPU); VAL(AX_DEVICE_CUDA);
    VAL(AX_BACKEND_CPU_NAIVE); VAL(AX_BACKEND_CPU_SIMD); VAL(AX_BACKEND_CUDA);
    VAL(AX_LAYER_DENSE); VAL(AX_LAYER_RELU); VAL(AX_LAYER_GELU); VAL(AX_LAYER_SEQUENTIAL);
    VAL(AX_MAX_DIMS); VAL(AX_SEQ_MAX_LAYERS);
    printf("  \"end\": 0\n}\n");
    return 0;
}
