// Compiled (never run) by tests/test_abi_mirror.py where the reference tree is mounted: the reference's own
// headers and this repository's mirror of them must agree on every size and offset a backend relies on.
#include "ggml.h"
#include "ggml-impl.h"
#include "ggml-backend.h"
#include "ggml-backend-impl.h"
#include "ggml-common.h"

#include <cstddef>

namespace mirror {
#undef LM_GGML_MAX_DIMS
#undef LM_GGML_MAX_SRC
#undef LM_GGML_MAX_OP_PARAMS
#undef LM_GGML_MAX_NAME
#undef LM_GGML_BACKEND_API_VERSION
#define CACTUS_MIRROR_TYPES_ONLY
// the mirror spells enum values as anonymous enums: rename them out of the way of the real ones
#define LM_GGML_TYPE_F32 M_TYPE_F32
#define LM_GGML_TYPE_F16 M_TYPE_F16
#define LM_GGML_TYPE_Q4_0 M_TYPE_Q4_0
#define LM_GGML_TYPE_Q8_0 M_TYPE_Q8_0
#define LM_GGML_TYPE_Q4_K M_TYPE_Q4_K
#define LM_GGML_TYPE_Q6_K M_TYPE_Q6_K
#define LM_GGML_TYPE_Q8_K M_TYPE_Q8_K
#define LM_GGML_TYPE_Q2_K M_TYPE_Q2_K
#define LM_GGML_TYPE_Q3_K M_TYPE_Q3_K
#define LM_GGML_TYPE_IQ4_XS M_TYPE_IQ4_XS
#define LM_GGML_TYPE_I32 M_TYPE_I32
#define LM_GGML_OP_NONE M_OP_NONE
#define LM_GGML_OP_MUL_MAT M_OP_MUL_MAT
#define LM_GGML_UNARY_OP_SILU M_UNARY_OP_SILU
#define LM_GGML_UNARY_OP_GELU M_UNARY_OP_GELU
#define LM_GGML_TENSOR_FLAG_INPUT M_TENSOR_FLAG_INPUT
#define LM_GGML_TENSOR_FLAG_OUTPUT M_TENSOR_FLAG_OUTPUT
#define LM_GGML_OP_SCALE M_OP_SCALE
#define LM_GGML_OP_UNARY M_OP_UNARY
#define LM_GGML_OP_RMS_NORM M_OP_RMS_NORM
#define LM_GGML_OP_MUL M_OP_MUL
#define LM_GGML_OP_ADD M_OP_ADD
#define LM_GGML_OP_MUL_MAT_ID M_OP_MUL_MAT_ID
#define LM_GGML_OP_DUP M_OP_DUP
#define LM_GGML_OP_GET_ROWS M_OP_GET_ROWS
#define LM_GGML_OP_CPY M_OP_CPY
#define LM_GGML_OP_CONT M_OP_CONT
#define LM_GGML_OP_SOFT_MAX M_OP_SOFT_MAX
#define LM_GGML_OP_ROPE M_OP_ROPE
#define LM_GGML_OP_RESHAPE M_OP_RESHAPE
#define LM_GGML_OP_VIEW M_OP_VIEW
#define LM_GGML_OP_PERMUTE M_OP_PERMUTE
#define LM_GGML_OP_TRANSPOSE M_OP_TRANSPOSE
#define LM_GGML_OP_COUNT M_OP_COUNT
#define LM_GGML_STATUS_ALLOC_FAILED M_STATUS_ALLOC_FAILED
#define LM_GGML_STATUS_FAILED M_STATUS_FAILED
#define LM_GGML_STATUS_SUCCESS M_STATUS_SUCCESS
#define LM_GGML_STATUS_ABORTED M_STATUS_ABORTED
#define LM_GGML_BACKEND_DEVICE_TYPE_CPU M_DEV_CPU
#define LM_GGML_BACKEND_DEVICE_TYPE_GPU M_DEV_GPU
#define LM_GGML_BACKEND_DEVICE_TYPE_ACCEL M_DEV_ACCEL
#define LM_GGML_BACKEND_BUFFER_USAGE_ANY M_USAGE_ANY
#define LM_GGML_BACKEND_BUFFER_USAGE_WEIGHTS M_USAGE_WEIGHTS
#define LM_GGML_BACKEND_BUFFER_USAGE_COMPUTE M_USAGE_COMPUTE
#define LM_GGML_LOG_LEVEL_NONE M_LOG_NONE
#define LM_GGML_LOG_LEVEL_DEBUG M_LOG_DEBUG
#define LM_GGML_LOG_LEVEL_INFO M_LOG_INFO
#define LM_GGML_LOG_LEVEL_WARN M_LOG_WARN
#define LM_GGML_LOG_LEVEL_ERROR M_LOG_ERROR
#define LM_GGML_LOG_LEVEL_CONT M_LOG_CONT
#include "ggml_abi_mirror.h"
constexpr int k_max_dims = LM_GGML_MAX_DIMS, k_max_src = LM_GGML_MAX_SRC, k_max_op_params = LM_GGML_MAX_OP_PARAMS,
              k_max_name = LM_GGML_MAX_NAME, k_api = LM_GGML_BACKEND_API_VERSION;
#undef LM_GGML_TYPE_F32
#undef LM_GGML_TYPE_F16
#undef LM_GGML_TYPE_Q4_0
#undef LM_GGML_TYPE_Q8_0
#undef LM_GGML_TYPE_Q4_K
#undef LM_GGML_TYPE_Q6_K
#undef LM_GGML_TYPE_Q2_K
#undef LM_GGML_TYPE_Q3_K
#undef LM_GGML_TYPE_IQ4_XS
#undef LM_GGML_TYPE_Q8_K
#undef LM_GGML_TYPE_I32
#undef LM_GGML_OP_NONE
#undef LM_GGML_OP_MUL_MAT
#undef LM_GGML_UNARY_OP_SILU
#undef LM_GGML_UNARY_OP_GELU
#undef LM_GGML_TENSOR_FLAG_INPUT
#undef LM_GGML_TENSOR_FLAG_OUTPUT
#undef LM_GGML_OP_SCALE
#undef LM_GGML_OP_UNARY
#undef LM_GGML_OP_RMS_NORM
#undef LM_GGML_OP_MUL
#undef LM_GGML_OP_ADD
#undef LM_GGML_OP_MUL_MAT_ID
#undef LM_GGML_OP_DUP
#undef LM_GGML_OP_GET_ROWS
#undef LM_GGML_OP_CPY
#undef LM_GGML_OP_CONT
#undef LM_GGML_OP_SOFT_MAX
#undef LM_GGML_OP_ROPE
#undef LM_GGML_OP_RESHAPE
#undef LM_GGML_OP_VIEW
#undef LM_GGML_OP_PERMUTE
#undef LM_GGML_OP_TRANSPOSE
#undef LM_GGML_OP_COUNT
#undef LM_GGML_STATUS_ALLOC_FAILED
#undef LM_GGML_STATUS_FAILED
#undef LM_GGML_STATUS_SUCCESS
#undef LM_GGML_STATUS_ABORTED
#undef LM_GGML_BACKEND_DEVICE_TYPE_CPU
#undef LM_GGML_BACKEND_DEVICE_TYPE_GPU
#undef LM_GGML_BACKEND_DEVICE_TYPE_ACCEL
#undef LM_GGML_BACKEND_BUFFER_USAGE_ANY
#undef LM_GGML_BACKEND_BUFFER_USAGE_WEIGHTS
#undef LM_GGML_BACKEND_BUFFER_USAGE_COMPUTE
#undef LM_GGML_LOG_LEVEL_NONE
#undef LM_GGML_LOG_LEVEL_DEBUG
#undef LM_GGML_LOG_LEVEL_INFO
#undef LM_GGML_LOG_LEVEL_WARN
#undef LM_GGML_LOG_LEVEL_ERROR
#undef LM_GGML_LOG_LEVEL_CONT
}  // namespace mirror

#define SAME_SIZE(T) static_assert(sizeof(::T) == sizeof(mirror::T), "sizeof " #T)
#define SAME_OFF(T, F) static_assert(offsetof(::T, F) == offsetof(mirror::T, F), "offsetof " #T "." #F)

SAME_SIZE(lm_ggml_tensor);
SAME_OFF(lm_ggml_tensor, type); SAME_OFF(lm_ggml_tensor, buffer); SAME_OFF(lm_ggml_tensor, ne); SAME_OFF(lm_ggml_tensor, nb);
SAME_OFF(lm_ggml_tensor, op); SAME_OFF(lm_ggml_tensor, op_params); SAME_OFF(lm_ggml_tensor, flags); SAME_OFF(lm_ggml_tensor, src);
SAME_OFF(lm_ggml_tensor, view_src); SAME_OFF(lm_ggml_tensor, view_offs); SAME_OFF(lm_ggml_tensor, data); SAME_OFF(lm_ggml_tensor, name);
SAME_OFF(lm_ggml_tensor, extra);
SAME_SIZE(lm_ggml_cgraph);
SAME_OFF(lm_ggml_cgraph, n_nodes); SAME_OFF(lm_ggml_cgraph, nodes); SAME_OFF(lm_ggml_cgraph, leafs);
SAME_SIZE(lm_ggml_backend_buffer_type_i); SAME_SIZE(lm_ggml_backend_buffer_type);
SAME_OFF(lm_ggml_backend_buffer_type, device); SAME_OFF(lm_ggml_backend_buffer_type, context);
SAME_OFF(lm_ggml_backend_buffer_type_i, alloc_buffer); SAME_OFF(lm_ggml_backend_buffer_type_i, get_alloc_size); SAME_OFF(lm_ggml_backend_buffer_type_i, is_host);
SAME_SIZE(lm_ggml_backend_buffer_i); SAME_SIZE(lm_ggml_backend_buffer);
SAME_OFF(lm_ggml_backend_buffer_i, get_base); SAME_OFF(lm_ggml_backend_buffer_i, set_tensor); SAME_OFF(lm_ggml_backend_buffer_i, get_tensor);
SAME_OFF(lm_ggml_backend_buffer_i, cpy_tensor); SAME_OFF(lm_ggml_backend_buffer_i, clear); SAME_OFF(lm_ggml_backend_buffer_i, reset);
SAME_OFF(lm_ggml_backend_buffer, buft); SAME_OFF(lm_ggml_backend_buffer, context); SAME_OFF(lm_ggml_backend_buffer, size); SAME_OFF(lm_ggml_backend_buffer, usage);
SAME_SIZE(lm_ggml_backend_i); SAME_SIZE(lm_ggml_backend);
SAME_OFF(lm_ggml_backend_i, synchronize); SAME_OFF(lm_ggml_backend_i, graph_compute); SAME_OFF(lm_ggml_backend_i, event_wait);
SAME_OFF(lm_ggml_backend, guid); SAME_OFF(lm_ggml_backend, iface); SAME_OFF(lm_ggml_backend, device); SAME_OFF(lm_ggml_backend, context);
SAME_SIZE(lm_ggml_backend_device_i); SAME_SIZE(lm_ggml_backend_device);
SAME_OFF(lm_ggml_backend_device_i, get_props); SAME_OFF(lm_ggml_backend_device_i, init_backend); SAME_OFF(lm_ggml_backend_device_i, supports_op);
SAME_OFF(lm_ggml_backend_device_i, supports_buft); SAME_OFF(lm_ggml_backend_device_i, offload_op); SAME_OFF(lm_ggml_backend_device_i, event_synchronize);
SAME_OFF(lm_ggml_backend_device, reg); SAME_OFF(lm_ggml_backend_device, context);
SAME_SIZE(lm_ggml_backend_reg_i); SAME_SIZE(lm_ggml_backend_reg);
SAME_OFF(lm_ggml_backend_reg, api_version); SAME_OFF(lm_ggml_backend_reg, iface); SAME_OFF(lm_ggml_backend_reg, context);
SAME_SIZE(lm_ggml_backend_dev_props); SAME_SIZE(lm_ggml_backend_dev_caps);
SAME_OFF(lm_ggml_backend_dev_props, memory_free); SAME_OFF(lm_ggml_backend_dev_props, type); SAME_OFF(lm_ggml_backend_dev_props, caps);
SAME_SIZE(lm_ggml_backend_event);

static_assert(mirror::k_max_dims == LM_GGML_MAX_DIMS && mirror::k_max_src == LM_GGML_MAX_SRC, "limits");
static_assert(mirror::k_max_op_params == LM_GGML_MAX_OP_PARAMS && mirror::k_max_name == LM_GGML_MAX_NAME, "limits");
static_assert(mirror::k_api == LM_GGML_BACKEND_API_VERSION, "api version");
static_assert(mirror::M_TYPE_F32 == LM_GGML_TYPE_F32 && mirror::M_TYPE_F16 == LM_GGML_TYPE_F16 && mirror::M_TYPE_Q4_0 == LM_GGML_TYPE_Q4_0 &&
              mirror::M_TYPE_Q8_0 == LM_GGML_TYPE_Q8_0 && mirror::M_TYPE_Q4_K == LM_GGML_TYPE_Q4_K && mirror::M_TYPE_Q6_K == LM_GGML_TYPE_Q6_K &&
              mirror::M_TYPE_Q8_K == LM_GGML_TYPE_Q8_K && mirror::M_TYPE_I32 == LM_GGML_TYPE_I32 && mirror::M_TYPE_Q2_K == LM_GGML_TYPE_Q2_K &&
              mirror::M_TYPE_Q3_K == LM_GGML_TYPE_Q3_K && mirror::M_TYPE_IQ4_XS == LM_GGML_TYPE_IQ4_XS, "type ids");
static_assert(mirror::M_OP_NONE == LM_GGML_OP_NONE && mirror::M_OP_MUL_MAT == LM_GGML_OP_MUL_MAT && mirror::M_OP_RESHAPE == LM_GGML_OP_RESHAPE &&
              mirror::M_OP_VIEW == LM_GGML_OP_VIEW && mirror::M_OP_PERMUTE == LM_GGML_OP_PERMUTE && mirror::M_OP_TRANSPOSE == LM_GGML_OP_TRANSPOSE &&
              mirror::M_OP_COUNT == LM_GGML_OP_COUNT && mirror::M_OP_MUL_MAT_ID == LM_GGML_OP_MUL_MAT_ID &&
              mirror::M_OP_ADD == LM_GGML_OP_ADD && mirror::M_OP_MUL == LM_GGML_OP_MUL && mirror::M_OP_RMS_NORM == LM_GGML_OP_RMS_NORM &&
              mirror::M_OP_UNARY == LM_GGML_OP_UNARY && mirror::M_UNARY_OP_SILU == LM_GGML_UNARY_OP_SILU &&
              mirror::M_OP_DUP == LM_GGML_OP_DUP && mirror::M_OP_GET_ROWS == LM_GGML_OP_GET_ROWS && mirror::M_OP_CPY == LM_GGML_OP_CPY && mirror::M_OP_CONT == LM_GGML_OP_CONT && mirror::M_OP_SOFT_MAX == LM_GGML_OP_SOFT_MAX && mirror::M_OP_ROPE == LM_GGML_OP_ROPE &&
              mirror::M_OP_SCALE == LM_GGML_OP_SCALE && mirror::M_UNARY_OP_GELU == LM_GGML_UNARY_OP_GELU, "op ids");
static_assert(mirror::M_TENSOR_FLAG_INPUT == LM_GGML_TENSOR_FLAG_INPUT && mirror::M_TENSOR_FLAG_OUTPUT == LM_GGML_TENSOR_FLAG_OUTPUT, "tensor flags");
static_assert(mirror::M_STATUS_ALLOC_FAILED == LM_GGML_STATUS_ALLOC_FAILED && mirror::M_STATUS_FAILED == LM_GGML_STATUS_FAILED &&
              mirror::M_STATUS_SUCCESS == LM_GGML_STATUS_SUCCESS && mirror::M_STATUS_ABORTED == LM_GGML_STATUS_ABORTED, "status");
static_assert(mirror::M_DEV_CPU == LM_GGML_BACKEND_DEVICE_TYPE_CPU && mirror::M_DEV_GPU == LM_GGML_BACKEND_DEVICE_TYPE_GPU &&
              mirror::M_DEV_ACCEL == LM_GGML_BACKEND_DEVICE_TYPE_ACCEL, "device types");
static_assert(mirror::M_USAGE_ANY == LM_GGML_BACKEND_BUFFER_USAGE_ANY && mirror::M_USAGE_WEIGHTS == LM_GGML_BACKEND_BUFFER_USAGE_WEIGHTS &&
              mirror::M_USAGE_COMPUTE == LM_GGML_BACKEND_BUFFER_USAGE_COMPUTE, "buffer usage");
static_assert(mirror::M_LOG_ERROR == LM_GGML_LOG_LEVEL_ERROR && mirror::M_LOG_INFO == LM_GGML_LOG_LEVEL_INFO, "log levels");
static_assert(sizeof(block_q4_0) == 18 && sizeof(block_q8_0) == 34 && sizeof(block_q4_K) == 144 && sizeof(block_q6_K) == 210 &&
              sizeof(block_q8_K) == 292, "block sizes");
static_assert(offsetof(block_q4_K, scales) == 4 && offsetof(block_q4_K, qs) == 16 && offsetof(block_q6_K, qh) == 128 &&
              offsetof(block_q6_K, scales) == 192 && offsetof(block_q6_K, d) == 208 && offsetof(block_q8_K, qs) == 4 &&
              offsetof(block_q8_K, bsums) == 260, "block field offsets");
int main() { return 0; }
