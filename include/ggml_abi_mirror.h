/*
 * ggml_abi_mirror.h -- layout-compatible declarations of the parts of the reference's ggml ABI that a backend
 * touches, written out here so the backend builds (and is tested) without the reference's headers.
 *
 * These are interface facts of the reference at the vendored revision (paths relative to its cactus/ directory):
 *   struct lm_ggml_tensor            ggml.h:575-607         (336 bytes on x86-64)
 *   struct lm_ggml_cgraph            ggml-impl.h:293-306    (80 bytes)
 *   backend vtables and objects      ggml-backend-impl.h:17-207
 *   dev props / caps / enums         ggml-backend.h:49-53,130-159
 *   limits and enum values           ggml.h:218-225,320-325,351-391,429-521
 * tests/test_abi_mirror.py compiles a translation unit that includes both this header (inside a namespace)
 * and the reference's headers and static_asserts that every size and field offset agrees; it runs wherever the
 * reference tree is mounted.
 *
 * Define CACTUS_MIRROR_TYPES_ONLY before including to leave out the host function declarations.
 */
#ifndef CACTUS_GGML_ABI_MIRROR_H
#define CACTUS_GGML_ABI_MIRROR_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LM_GGML_MAX_DIMS       4
#define LM_GGML_MAX_SRC        10
#define LM_GGML_MAX_OP_PARAMS  64
#define LM_GGML_MAX_NAME       64
#define LM_GGML_BACKEND_API_VERSION 1

/* enum values used on this path (the enums themselves are plain ints in the ABI) */
enum {
    LM_GGML_TYPE_F32 = 0, LM_GGML_TYPE_F16 = 1, LM_GGML_TYPE_Q4_0 = 2, LM_GGML_TYPE_Q8_0 = 8,
    LM_GGML_TYPE_Q2_K = 10, LM_GGML_TYPE_Q3_K = 11, LM_GGML_TYPE_IQ4_XS = 23,
    LM_GGML_TYPE_Q4_K = 12, LM_GGML_TYPE_Q6_K = 14, LM_GGML_TYPE_Q8_K = 15, LM_GGML_TYPE_I32 = 26,
};
enum {
    LM_GGML_OP_NONE = 0, LM_GGML_OP_ADD = 2, LM_GGML_OP_MUL = 6, LM_GGML_OP_RMS_NORM = 23,
    LM_GGML_OP_MUL_MAT = 27, LM_GGML_OP_MUL_MAT_ID = 28, LM_GGML_OP_SCALE = 30, LM_GGML_OP_UNARY = 74,
    LM_GGML_OP_DUP = 1, LM_GGML_OP_GET_ROWS = 38, LM_GGML_OP_CPY = 32, LM_GGML_OP_CONT = 33, LM_GGML_OP_SOFT_MAX = 43, LM_GGML_OP_ROPE = 45,
    LM_GGML_OP_RESHAPE = 34, LM_GGML_OP_VIEW = 35, LM_GGML_OP_PERMUTE = 36, LM_GGML_OP_TRANSPOSE = 37,
    LM_GGML_OP_COUNT = 82,
};
enum { LM_GGML_UNARY_OP_GELU = 8, LM_GGML_UNARY_OP_SILU = 10 };
enum { LM_GGML_TENSOR_FLAG_INPUT = 1, LM_GGML_TENSOR_FLAG_OUTPUT = 2 };      /* enum lm_ggml_tensor_flag (ggml.h:560-563) */
enum { LM_GGML_STATUS_ALLOC_FAILED = -2, LM_GGML_STATUS_FAILED = -1, LM_GGML_STATUS_SUCCESS = 0, LM_GGML_STATUS_ABORTED = 1 };
enum { LM_GGML_BACKEND_DEVICE_TYPE_CPU = 0, LM_GGML_BACKEND_DEVICE_TYPE_GPU = 1, LM_GGML_BACKEND_DEVICE_TYPE_ACCEL = 2 };
enum { LM_GGML_BACKEND_BUFFER_USAGE_ANY = 0, LM_GGML_BACKEND_BUFFER_USAGE_WEIGHTS = 1, LM_GGML_BACKEND_BUFFER_USAGE_COMPUTE = 2 };
enum { LM_GGML_LOG_LEVEL_NONE = 0, LM_GGML_LOG_LEVEL_DEBUG = 1, LM_GGML_LOG_LEVEL_INFO = 2, LM_GGML_LOG_LEVEL_WARN = 3,
       LM_GGML_LOG_LEVEL_ERROR = 4, LM_GGML_LOG_LEVEL_CONT = 5 };

struct lm_ggml_backend_buffer;

struct lm_ggml_tensor {
    int      type;                              /* enum lm_ggml_type */
    struct lm_ggml_backend_buffer *buffer;
    int64_t  ne[LM_GGML_MAX_DIMS];
    size_t   nb[LM_GGML_MAX_DIMS];
    int      op;                                /* enum lm_ggml_op */
    int32_t  op_params[LM_GGML_MAX_OP_PARAMS / sizeof(int32_t)];
    int32_t  flags;
    struct lm_ggml_tensor *src[LM_GGML_MAX_SRC];
    struct lm_ggml_tensor *view_src;
    size_t   view_offs;
    void    *data;
    char     name[LM_GGML_MAX_NAME];
    void    *extra;
    char     padding[8];
};

struct lm_ggml_hash_set_mirror { size_t size; uint32_t *used; struct lm_ggml_tensor **keys; };

struct lm_ggml_cgraph {
    int size;
    int n_nodes;
    int n_leafs;
    struct lm_ggml_tensor **nodes;
    struct lm_ggml_tensor **grads;
    struct lm_ggml_tensor **grad_accs;
    struct lm_ggml_tensor **leafs;
    struct lm_ggml_hash_set_mirror visited_hash_set;
    int order;
};

typedef struct lm_ggml_backend_buffer_type *lm_ggml_backend_buffer_type_t;
typedef struct lm_ggml_backend_buffer      *lm_ggml_backend_buffer_t;
typedef struct lm_ggml_backend             *lm_ggml_backend_t;
typedef struct lm_ggml_backend_device      *lm_ggml_backend_dev_t;
typedef struct lm_ggml_backend_reg         *lm_ggml_backend_reg_t;
typedef struct lm_ggml_backend_event       *lm_ggml_backend_event_t;
typedef void                               *lm_ggml_backend_graph_plan_t;
typedef uint8_t lm_ggml_guid[16];
typedef lm_ggml_guid *lm_ggml_guid_t;

struct lm_ggml_backend_dev_caps { bool async; bool host_buffer; bool buffer_from_host_ptr; bool events; };
struct lm_ggml_backend_dev_props {
    const char *name;
    const char *description;
    size_t memory_free;
    size_t memory_total;
    int type;                                   /* enum lm_ggml_backend_dev_type */
    struct lm_ggml_backend_dev_caps caps;
};

struct lm_ggml_backend_buffer_type_i {
    const char *             (*get_name)      (lm_ggml_backend_buffer_type_t buft);
    lm_ggml_backend_buffer_t (*alloc_buffer)  (lm_ggml_backend_buffer_type_t buft, size_t size);
    size_t                   (*get_alignment) (lm_ggml_backend_buffer_type_t buft);
    size_t                   (*get_max_size)  (lm_ggml_backend_buffer_type_t buft);
    size_t                   (*get_alloc_size)(lm_ggml_backend_buffer_type_t buft, const struct lm_ggml_tensor *tensor);
    bool                     (*is_host)       (lm_ggml_backend_buffer_type_t buft);
};
struct lm_ggml_backend_buffer_type {
    struct lm_ggml_backend_buffer_type_i iface;
    lm_ggml_backend_dev_t device;
    void *context;
};

struct lm_ggml_backend_buffer_i {
    void   (*free_buffer)  (lm_ggml_backend_buffer_t buffer);
    void * (*get_base)     (lm_ggml_backend_buffer_t buffer);
    int    (*init_tensor)  (lm_ggml_backend_buffer_t buffer, struct lm_ggml_tensor *tensor);     /* enum lm_ggml_status */
    void   (*memset_tensor)(lm_ggml_backend_buffer_t buffer, struct lm_ggml_tensor *tensor, uint8_t value, size_t offset, size_t size);
    void   (*set_tensor)   (lm_ggml_backend_buffer_t buffer, struct lm_ggml_tensor *tensor, const void *data, size_t offset, size_t size);
    void   (*get_tensor)   (lm_ggml_backend_buffer_t buffer, const struct lm_ggml_tensor *tensor, void *data, size_t offset, size_t size);
    bool   (*cpy_tensor)   (lm_ggml_backend_buffer_t buffer, const struct lm_ggml_tensor *src, struct lm_ggml_tensor *dst);
    void   (*clear)        (lm_ggml_backend_buffer_t buffer, uint8_t value);
    void   (*reset)        (lm_ggml_backend_buffer_t buffer);
};
struct lm_ggml_backend_buffer {
    struct lm_ggml_backend_buffer_i iface;
    lm_ggml_backend_buffer_type_t buft;
    void *context;
    size_t size;
    int usage;                                  /* enum lm_ggml_backend_buffer_usage */
};

struct lm_ggml_backend_i {
    const char * (*get_name)(lm_ggml_backend_t backend);
    void (*free)(lm_ggml_backend_t backend);
    void (*set_tensor_async)(lm_ggml_backend_t backend, struct lm_ggml_tensor *tensor, const void *data, size_t offset, size_t size);
    void (*get_tensor_async)(lm_ggml_backend_t backend, const struct lm_ggml_tensor *tensor, void *data, size_t offset, size_t size);
    bool (*cpy_tensor_async)(lm_ggml_backend_t backend_src, lm_ggml_backend_t backend_dst, const struct lm_ggml_tensor *src, struct lm_ggml_tensor *dst);
    void (*synchronize)(lm_ggml_backend_t backend);
    lm_ggml_backend_graph_plan_t (*graph_plan_create) (lm_ggml_backend_t backend, const struct lm_ggml_cgraph *cgraph);
    void                         (*graph_plan_free)   (lm_ggml_backend_t backend, lm_ggml_backend_graph_plan_t plan);
    void                         (*graph_plan_update) (lm_ggml_backend_t backend, lm_ggml_backend_graph_plan_t plan, const struct lm_ggml_cgraph *cgraph);
    int                          (*graph_plan_compute)(lm_ggml_backend_t backend, lm_ggml_backend_graph_plan_t plan);
    int                          (*graph_compute)     (lm_ggml_backend_t backend, struct lm_ggml_cgraph *cgraph);
    void (*event_record)(lm_ggml_backend_t backend, lm_ggml_backend_event_t event);
    void (*event_wait)  (lm_ggml_backend_t backend, lm_ggml_backend_event_t event);
};
struct lm_ggml_backend {
    lm_ggml_guid_t guid;
    struct lm_ggml_backend_i iface;
    lm_ggml_backend_dev_t device;
    void *context;
};
struct lm_ggml_backend_event { struct lm_ggml_backend_device *device; void *context; };

struct lm_ggml_backend_device_i {
    const char * (*get_name)(lm_ggml_backend_dev_t dev);
    const char * (*get_description)(lm_ggml_backend_dev_t dev);
    void         (*get_memory)(lm_ggml_backend_dev_t dev, size_t *free, size_t *total);
    int          (*get_type)(lm_ggml_backend_dev_t dev);                                          /* enum lm_ggml_backend_dev_type */
    void         (*get_props)(lm_ggml_backend_dev_t dev, struct lm_ggml_backend_dev_props *props);
    lm_ggml_backend_t             (*init_backend)(lm_ggml_backend_dev_t dev, const char *params);
    lm_ggml_backend_buffer_type_t (*get_buffer_type)(lm_ggml_backend_dev_t dev);
    lm_ggml_backend_buffer_type_t (*get_host_buffer_type)(lm_ggml_backend_dev_t dev);
    lm_ggml_backend_buffer_t      (*buffer_from_host_ptr)(lm_ggml_backend_dev_t dev, void *ptr, size_t size, size_t max_tensor_size);
    bool (*supports_op)(lm_ggml_backend_dev_t dev, const struct lm_ggml_tensor *op);
    bool (*supports_buft)(lm_ggml_backend_dev_t dev, lm_ggml_backend_buffer_type_t buft);
    bool (*offload_op)(lm_ggml_backend_dev_t dev, const struct lm_ggml_tensor *op);
    lm_ggml_backend_event_t (*event_new)(lm_ggml_backend_dev_t dev);
    void (*event_free)(lm_ggml_backend_dev_t dev, lm_ggml_backend_event_t event);
    void (*event_synchronize)(lm_ggml_backend_dev_t dev, lm_ggml_backend_event_t event);
};
struct lm_ggml_backend_device {
    struct lm_ggml_backend_device_i iface;
    lm_ggml_backend_reg_t reg;
    void *context;
};

struct lm_ggml_backend_reg_i {
    const char *          (*get_name)(lm_ggml_backend_reg_t reg);
    size_t                (*get_device_count)(lm_ggml_backend_reg_t reg);
    lm_ggml_backend_dev_t (*get_device)(lm_ggml_backend_reg_t reg, size_t index);
    void *                (*get_proc_address)(lm_ggml_backend_reg_t reg, const char *name);
};
struct lm_ggml_backend_reg {
    int api_version;
    struct lm_ggml_backend_reg_i iface;
    void *context;
};

#ifndef CACTUS_MIRROR_TYPES_ONLY
/* Host functions the backend calls; resolved from the process that loads it (ggml-backend-impl.h:66-76,
 * ggml.h:700, ggml-impl.h:79). */
lm_ggml_backend_buffer_t lm_ggml_backend_buffer_init(lm_ggml_backend_buffer_type_t buft, struct lm_ggml_backend_buffer_i iface,
                                                     void *context, size_t size);
size_t lm_ggml_nbytes(const struct lm_ggml_tensor *tensor);
void   lm_ggml_log_internal(int level, const char *format, ...);
#endif

#ifdef __cplusplus
}
#endif
#endif
