/*
 * The reference's accelerator-backend boundary, re-declared so that libpowerinfer_hip.so can be linked in place
 * of ggml-cuda.cu: the 28 entry points of ggml-cuda.h:21-60 with the same names, argument meaning and "handled?"
 * contract, and the slice of ggml.h's ABI they read (tensor struct, enums, compute params).  Field order,
 * types and enumerator values follow ggml.h:229-235, 333-470, 513-553, 639-655 of the reference
 * (PowerInfer inserts GGML_OP_MUL_MAT_SPARSE and GGML_OP_AXPY after GGML_OP_MUL_MAT and adds is_finish/aic);
 * tests/test_abi_layout.py checks every offset and value against the reference's own header.
 *
 * A host program that already includes the reference's ggml.h must NOT include this file: it declares the same
 * names.  It exists for this library's own translation units and for hosts that have no ggml.h.
 */
#ifndef PI_GGML_BACKEND_ABI_H
#define PI_GGML_BACKEND_ABI_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GGML_API __attribute__((visibility("default")))

#define GGML_MAX_DIMS      4
#define GGML_MAX_SRC       6
#define GGML_MAX_NAME      64
#define GGML_MAX_OP_PARAMS 64
#define GGML_CUDA_MAX_DEVICES 16

enum ggml_type {
    GGML_TYPE_F32 = 0, GGML_TYPE_F16 = 1, GGML_TYPE_Q4_0 = 2, GGML_TYPE_Q4_1 = 3,
    GGML_TYPE_Q5_0 = 6, GGML_TYPE_Q5_1 = 7, GGML_TYPE_Q8_0 = 8, GGML_TYPE_Q8_1 = 9,
    GGML_TYPE_Q2_K = 10, GGML_TYPE_Q3_K = 11, GGML_TYPE_Q4_K = 12, GGML_TYPE_Q5_K = 13, GGML_TYPE_Q6_K = 14, GGML_TYPE_Q8_K = 15,
    GGML_TYPE_I8 = 16, GGML_TYPE_I16 = 17, GGML_TYPE_I32 = 18, GGML_TYPE_COUNT
};

enum ggml_backend_type { GGML_BACKEND_CPU = 0, GGML_BACKEND_GPU = 10, GGML_BACKEND_GPU_SPLIT = 20 };

/* only the operators this backend dispatches are named; the values are positions in the reference's enum */
enum ggml_op {
    GGML_OP_NONE = 0, GGML_OP_DUP = 1, GGML_OP_ADD = 2, GGML_OP_MUL = 6,
    GGML_OP_NORM = 19, GGML_OP_RMS_NORM = 20,
    GGML_OP_MUL_MAT = 23, GGML_OP_MUL_MAT_SPARSE = 24, GGML_OP_AXPY = 25,
    GGML_OP_SCALE = 27, GGML_OP_CPY = 29, GGML_OP_CONT = 30, GGML_OP_RESHAPE = 31, GGML_OP_VIEW = 32,
    GGML_OP_PERMUTE = 33, GGML_OP_TRANSPOSE = 34, GGML_OP_GET_ROWS = 35,
    GGML_OP_SOFT_MAX = 40, GGML_OP_ROPE = 42, GGML_OP_UNARY = 59,
    GGML_OP_ENUM_FORCE_INT = 0x7fffffff
};

enum ggml_unary_op { GGML_UNARY_OP_RELU = 6 };

enum ggml_task_type { GGML_TASK_INIT = 0, GGML_TASK_COMPUTE = 1, GGML_TASK_FINALIZE = 2 };

struct ggml_backend_buffer;

struct ggml_tensor {
    enum ggml_type         type;
    enum ggml_backend_type backend;
    struct ggml_backend_buffer * buffer;
    int     n_dims;
    int64_t ne[GGML_MAX_DIMS];      /* number of elements */
    size_t  nb[GGML_MAX_DIMS];      /* stride in bytes */
    enum ggml_op op;
    int32_t op_params[GGML_MAX_OP_PARAMS / sizeof(int32_t)];
    bool    is_param;
    struct ggml_tensor * grad;
    struct ggml_tensor * src[GGML_MAX_SRC];
    int     is_finish;              /* atomic_int in the reference */
    int     perf_runs;
    int64_t perf_cycles;
    int64_t perf_time_us;
    struct ggml_tensor * view_src;
    size_t  view_offs;
    void *  data;
    char    name[GGML_MAX_NAME];
    void *  extra;                  /* backend-private: this library keeps the device address here */
    char    padding[12];
};

struct ggml_compute_params {
    enum ggml_task_type type;
    int    ith, nth;                /* thread index, number of threads */
    size_t wsize;
    void * wdata;
    int *  aic;                     /* atomic_int * in the reference: shared work-stealing counter */
};

typedef struct ggml_backend * ggml_backend_t;

/* ---- ggml-cuda.h:21-60 ------------------------------------------------------------------------------ */
GGML_API void   ggml_init_cublas(void);                                   /* always succeeds (ggml-cuda.cu:6463) */
GGML_API bool   ggml_cublas_loaded(void);

GGML_API void * ggml_cuda_host_malloc(size_t size);                       /* pinned; NULL => caller falls back to malloc */
GGML_API void   ggml_cuda_host_free(void * ptr);

GGML_API bool   ggml_cuda_can_mul_mat(const struct ggml_tensor * src0, const struct ggml_tensor * src1, struct ggml_tensor * dst);
GGML_API void   ggml_cuda_set_tensor_split(const float * tensor_split);
GGML_API void   ggml_cuda_transform_tensor(void * data, struct ggml_tensor * tensor);   /* weight upload; owns tensor->extra */
GGML_API void   ggml_cuda_alloc_tensor(struct ggml_tensor * tensor);
GGML_API void   ggml_cuda_free_data(struct ggml_tensor * tensor);
GGML_API void   ggml_cuda_cpy_1d(struct ggml_tensor * dst, const struct ggml_tensor * src);
GGML_API void **ggml_cuda_get_data_pp(struct ggml_tensor * tensor);

GGML_API void   ggml_cuda_assign_buffers(struct ggml_tensor * tensor);
GGML_API void   ggml_cuda_assign_buffers_no_scratch(struct ggml_tensor * tensor);
GGML_API void   ggml_cuda_assign_buffers_force_inplace(struct ggml_tensor * tensor);
GGML_API void   ggml_cuda_assign_buffers_no_alloc(struct ggml_tensor * tensor);
GGML_API void   ggml_cuda_assign_scratch_offset(struct ggml_tensor * tensor, size_t offset);
GGML_API void   ggml_cuda_copy_to_device(struct ggml_tensor * tensor);
GGML_API void   ggml_cuda_copy_to_host(struct ggml_tensor * tensor);

GGML_API void   ggml_cuda_set_main_device(int main_device);
GGML_API void   ggml_cuda_set_mul_mat_q(bool mul_mat_q);
GGML_API void   ggml_cuda_set_scratch_size(size_t scratch_size);
GGML_API void   ggml_cuda_free_scratch(void);
/* called by every worker thread for every node and phase; false => the caller runs its CPU kernel
 * (ggml.c:14791-14798); true => handled (work happens only for ith == 0 in the COMPUTE phase) */
GGML_API bool   ggml_cuda_compute_forward(struct ggml_compute_params * params, struct ggml_tensor * tensor);

GGML_API int    ggml_cuda_get_device_count(void);
GGML_API void   ggml_cuda_get_device_description(int device, char * description, size_t description_size);
GGML_API size_t ggml_cuda_get_free_memory(int device);

GGML_API void   ggml_cuda_set_device_constants(float sparse_pred_threshold);       /* ggml-cuda.cu:9634 */

/* backend-v2 entry (ggml-backend-impl.h:46-83); llama.cpp does not use it for inference: returns NULL here */
GGML_API ggml_backend_t ggml_backend_cuda_init(void);

#ifdef __cplusplus
}
#endif
#endif
