/*
 * art.h — the C ABI of NART's `art` case runtime, as a single header.
 *
 * A case module (libart_module_<name>.so) and a runner talk to each other only through the types and
 * functions below.  They are declared here, from the layouts of the reference's public headers
 * (art/include/art/{data_type,mem,tensor,settings,op,op_tp,op_settings,workspace,module,parade,
 * serialize}.h of ModelTC/NART v1.2.14), so that
 *   - the `hip` case module built against this header loads into an unmodified NART runtime, and
 *   - the repo's own small host core (libart.so under nart_amd/lib) can host it where NART itself is
 *     not installed (the GPU test box).
 * Everything here is ABI: field order, field types, enum values, symbol names.  The reference builds
 * with ART_CONSTRAINT_WITH_NAME (top-level CMakeLists.txt:19), so setting_constraint_t carries `name`.
 * tests/test_engine_cpu.py compiles a probe against BOTH header sets and compares every size and offset.
 */
#ifndef NART_HIP_ART_H
#define NART_HIP_ART_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ART_PUBLIC __attribute__((visibility("default")))

/* ---- element types (data_type.h:24-44) ---------------------------------------------------------- */
enum {
    dtUNKNOWN = 0, dtINT8 = 1, dtINT16 = 2, dtINT32 = 3, dtINT64 = 4,
    dtUINT8 = 5, dtUINT16 = 6, dtUINT32 = 7, dtUINT64 = 8,
    dtFLOAT16 = 9, dtFLOAT32 = 10, dtFLOAT64 = 11,
    dtSTR = 12, dtPTR = 13, dtCPTR = 14, dtBOOL = 15
};
size_t datatype_sizeof(uint32_t dtype);
const char *datatype_name_from_type(uint32_t dtype);
uint32_t datatype_type_from_name(const char *name);

/* ---- errors (log.h:29-34, 82-101): a failed CHECK aborts, LOG(error) exits ------------------------ */
#define ART_CHECK(cond)                                                                 \
    do {                                                                                \
        if (!(cond)) {                                                                  \
            fprintf(stderr, "[art] CHECK failed: %s (%s:%d)\n", #cond, __FILE__, __LINE__); \
            abort();                                                                    \
        }                                                                               \
    } while (0)
#define ART_FATAL(...)                     \
    do {                                   \
        fprintf(stderr, "[art] error: ");  \
        fprintf(stderr, __VA_ARGS__);      \
        exit(-1);                          \
    } while (0)

/* ---- memory objects (mem.h:48-101) ---------------------------------------------------------------- */
struct mem_t;
typedef struct mem_tp {
    const char *name;
    struct mem_t *(*new_func)(void);
    void (*delete_func)(struct mem_t *);
    bool (*alloc_func)(struct mem_t *, size_t);          /* grow-only: a smaller request keeps the buffer */
    void (*free_func)(struct mem_t *);
    void *(*data_func)(const struct mem_t *);            /* pointer in the module's own address space */
    void *(*cpu_data_func)(const struct mem_t *);        /* host pointer; the core reads and writes through it */
    size_t (*size_func)(struct mem_t *);
    void *(*copy_from_cpu_func)(void *to, const void *from, size_t sz);
    void *(*copy_to_cpu_func)(void *to, const void *from, size_t sz);
    struct mem_t *(*share_from_func)(void *data, size_t size);
} mem_tp;

typedef struct mem_t {
    const mem_tp *tp;
    uint32_t refcount;
} mem_t;

static inline mem_t *mem_new(const mem_tp *tp)
{
    mem_t *m = tp->new_func();
    m->refcount = 1;
    m->tp = tp;
    return m;
}
static inline bool mem_alloc(mem_t *m, size_t sz) { return m->tp->alloc_func(m, sz); }
static inline void mem_delete(mem_t *m)
{
    if (m != NULL && --m->refcount == 0)
        m->tp->delete_func(m);
}
static inline void *mem_data(const mem_t *m) { return m->tp->data_func(m); }
static inline void *mem_cpu_data(mem_t *m) { return m->tp->cpu_data_func(m); }
static inline size_t mem_sizeof(mem_t *m) { return m->tp->size_func(m); }

extern const mem_tp *cpu_mem_tp;
mem_t *extern_mem_from_data(void *data, size_t sz);
mem_t *mem_dup(mem_t *m);

/* ---- tensors (tensor.h:28-111) ---------------------------------------------------------------------- */
#define MAX_DIM 8
typedef struct shape_t {
    uint32_t dim[MAX_DIM];
    int32_t dim_size;
    int32_t batch_axis;
    int32_t channel_axis;
} shape_t;

typedef struct tensor_t {
    char *name;
    mem_t *mem;
    uint32_t dtype;
    shape_t shape;
    int32_t with_transform;
} tensor_t;

tensor_t *tensor_new(const mem_tp *tp, uint32_t dtype);
void tensor_free(tensor_t *tensor);   /* releases mem and name, not the struct */
void tensor_delete(tensor_t *tensor); /* tensor_free + free(struct) */
void tensor_set_name(tensor_t *tensor, const char *name);
bool tensor_shape_eq(const shape_t *a, const shape_t *b);
bool tensor_reshape(tensor_t *tensor, const int shape_size, const int shape[]);
void tensor_share(tensor_t *share_from, tensor_t *share_to);

static inline size_t shape_count(const shape_t *s)
{
    size_t c = 1;
    if (s->dim_size == 0)
        return 0;
    for (int i = 0; i < s->dim_size; ++i)
        c *= s->dim[i];
    return c;
}
static inline size_t shape_part_count(const shape_t *s, int axis)
{
    size_t c = 1;
    if (s->dim_size == 0)
        return 0;
    for (int i = axis >= 0 ? axis : s->dim_size + axis; i < s->dim_size; ++i)
        c *= s->dim[i];
    return c;
}
static inline void tensor_alloc(tensor_t *t)
{
    if (t != NULL && t->dtype != dtUNKNOWN)
        mem_alloc(t->mem, datatype_sizeof(t->dtype) * shape_count(&t->shape));
}

/* ---- settings (settings.h:27-113) --------------------------------------------------------------------- */
typedef union {
    uint8_t u8; uint16_t u16; uint32_t u32; uint64_t u64;
    int8_t i8; int16_t i16; int32_t i32; int64_t i64;
    float f32; double f64;
    char *str; const void *cptr; void *ptr;
    int i; unsigned int u; bool b;
} uvalue_t;

typedef enum { ENUM_SETTING_VALUE_SINGLE = 1, ENUM_SETTING_VALUE_REPEATED = 2 } enum_setting_value_tp_t;
typedef enum {
    ENUM_SETTING_CONSTRAINT_REQUIRED = 1,
    ENUM_SETTING_CONSTRAINT_OPTIONAL = 2,
    ENUM_SETTING_CONSTRAINT_REPEATED = 3
} enum_setting_constraint_tp_t;

typedef struct {
    uint32_t item;
    uint32_t dtype;
    enum_setting_constraint_tp_t ctp;
    union {
        struct { int _; } required;
        struct { uvalue_t default_value; } optional;
        struct { int _; } repeated;
    } constraint;
    const char *name; /* present because NART builds with ART_CONSTRAINT_WITH_NAME */
} setting_constraint_t;

typedef struct setting_entry_t {
    uint32_t item;
    uint32_t dtype;
    enum_setting_value_tp_t tp;
    union {
        struct { uvalue_t value; } single;
        struct { void *values; size_t len; } repeated;
    } v;
} setting_entry_t;

typedef struct _setting_t {
    size_t len;
    size_t reserved;
    setting_entry_t entries[];
} *setting_t;

#define SETTING_END 0xffffffffu

setting_t setting_new(void);
setting_t setting_new_with_reserved(size_t count);
void setting_delete(setting_t setting);
void setting_shrink(setting_t *setting);
setting_entry_t *setting_search(setting_t setting, uint32_t item);
void setting_set_single(setting_t *setting, uint32_t item, uint32_t dtype, uvalue_t v);
void *setting_alloc_repeated(setting_t *setting, uint32_t item, uint32_t dtype, size_t count);

/* ---- operators (op.h:100-186) ---------------------------------------------------------------------------- */
struct op_t;
struct workspace_t;

typedef struct {
    uint64_t op_tp_code;
    const char *name;
    uint16_t min_input_size, max_input_size, min_output_size, max_output_size;
    bool (*infer_output_func)(struct op_t *);
    setting_constraint_t constraints[]; /* terminated by item == SETTING_END */
} op_tp_t;

typedef struct {
    const op_tp_t *tp;
    struct op_t *(*alloc_func)(struct workspace_t *);
    void (*config_func)(struct op_t *);
    void (*destroy_func)(struct op_t *);
    void (*dealloc_func)(struct op_t *);
    void (*prepare_func)(struct op_t *);
} op_tp_entry_t; /* a module's table ends with an entry whose tp is NULL */

typedef struct op_t {
    op_tp_entry_t *entry;
    struct workspace_t *workspace;
    size_t input_size;
    size_t output_size;
    tensor_t **input_tensors; /* borrowed */
    tensor_t *output_tensors; /* owned: array of structs, filled by tp->infer_output_func */
    void (*run_func)(struct op_t *);
    setting_t setting;
} op_t;

/* The reference wraps run_func in profiler point-cuts (op.h:145-165); the hook is a no-op here. */
static inline void op_run(op_t *op) { op->run_func(op); }
static inline bool op_infer_output(op_t *op) { return op->entry->tp->infer_output_func(op); }

void op_init_default(op_t *op, op_tp_entry_t *entry, struct workspace_t *ws, uint16_t input_size,
                     tensor_t *const *input_tensor);
void op_destroy_default(op_t *op);
void op_delete(op_t *op);
bool op_config(op_t *op);
void op_prepare(op_t *op);

bool op_setting_if_set(const op_t *op, uint32_t item);
bool op_setting_single_get(const op_t *op, uint32_t item, uint32_t dtype, void *out);
bool op_setting_single_set(op_t *op, uint32_t item, uint32_t dtype, ...);
bool op_setting_array_set(op_t *op, uint32_t item, uint32_t dtype, size_t len, const void *in);
bool op_setting_array_get(const op_t *op, uint32_t item, uint32_t dtype, size_t *len, void *out);

/* op type codes (op_tp.h:20-129): group << 32 | code; bit 31 of the code marks module-private ops */
#define OP_GROUP_CODE_DEFAULT 0x0000ull
#define OP_GROUP_CODE_QUANT   0x0006ull
#define OP_DECLARE(group, code) (((uint64_t)(group) << 32) | (uint64_t)(code))
#define OP_ADD      OP_DECLARE(OP_GROUP_CODE_DEFAULT, 0x0011)
#define OP_CONV_2D  OP_DECLARE(OP_GROUP_CODE_DEFAULT, 0x0100)
#define OP_RELU     OP_DECLARE(OP_GROUP_CODE_DEFAULT, 0x0101)
#define OP_POOL     OP_DECLARE(OP_GROUP_CODE_DEFAULT, 0x0102)
#define OP_IP       OP_DECLARE(OP_GROUP_CODE_DEFAULT, 0x0104)
#define OP_CONCAT   OP_DECLARE(OP_GROUP_CODE_DEFAULT, 0x0106)
#define OP_SOFTMAX  OP_DECLARE(OP_GROUP_CODE_DEFAULT, 0x010B)
#define OP_ELTWISE  OP_DECLARE(OP_GROUP_CODE_DEFAULT, 0x010C)
#define OP_RESHAPE  OP_DECLARE(OP_GROUP_CODE_DEFAULT, 0x010E)
#define OP_QUANT_QUANTIZE   OP_DECLARE(OP_GROUP_CODE_QUANT, 0x80000000u) /* quant_op_tp.h:23 */
#define OP_QUANT_DEQUANTIZE OP_DECLARE(OP_GROUP_CODE_QUANT, 0x80000001u) /* quant_op_tp.h:24 */

/* shared op types of the generic ops: shape inference lives in the core (art/src/op.c) */
extern const op_tp_t op_conv_2d_tp, op_ip_tp, op_pool_tp, op_relu_tp, op_add_tp, op_eltwise_tp, op_reshape_tp;
extern const op_tp_t op_concat_tp, op_softmax_tp;

/* setting ids (op_settings.h, quant_op_settings.h:24-40) */
enum {
    SETTING_CONV_2D_NUM_OUTPUT = 1, SETTING_CONV_2D_PAD_H = 2, SETTING_CONV_2D_PAD_W = 3,
    SETTING_CONV_2D_KERNEL_H = 4, SETTING_CONV_2D_KERNEL_W = 5, SETTING_CONV_2D_STRIDE_H = 6,
    SETTING_CONV_2D_STRIDE_W = 7, SETTING_CONV_2D_GROUP = 8, SETTING_CONV_2D_RELU_FLAG = 9,
    SETTING_CONV_2D_DEFORM_GROUP = 10, SETTING_CONV_2D_HOLE_H = 11, SETTING_CONV_2D_HOLE_W = 12
};
enum {
    SETTING_POOL_METHOD = 1, SETTING_POOL_PAD_H = 2, SETTING_POOL_PAD_W = 3, SETTING_POOL_KERNEL_H = 4,
    SETTING_POOL_KERNEL_W = 5, SETTING_POOL_STRIDE_H = 6, SETTING_POOL_STRIDE_W = 7, SETTING_POOL_CEIL_MODE = 8,
    SETTING_POOL_MAX = 0, SETTING_POOL_AVE = 1
};
enum { SETTING_IP_NUM_OUTPUT = 1, SETTING_IP_RELU_FLAG = 2, SETTING_IP_AXIS = 3 };
enum {
    SETTING_ELTWISE_OPERATION = 1, SETTING_ELTWISE_COEFF = 2, SETTING_ELTWISE_RELU_FLAG = 3,
    SETTING_ELTWISE_OP_PROD = 0, SETTING_ELTWISE_OP_SUM = 1, SETTING_ELTWISE_OP_MAX = 2
};
enum { SETTING_CONCAT_AXIS = 1 };  /* op_settings.h:74 */
enum { SETTING_SOFTMAX_AXIS = 1 }; /* op_settings.h:89 */
enum { SETTING_RESHAPE_DIMS = 1, SETTING_RESHAPE_DIM_SIZE = 2, SETTING_RESHAPE_AXIS = 3, SETTING_RESHAPE_NUM_AXES = 4 };
#define SETTING_QUANT(code) ((uint32_t)((OP_GROUP_CODE_QUANT << 16) | (code)))
#define SETTING_QUANT_IALPHA      SETTING_QUANT(0x0101)
#define SETTING_QUANT_IZERO_POINT SETTING_QUANT(0x0102)
#define SETTING_QUANT_IBITS       SETTING_QUANT(0x0103)
#define SETTING_QUANT_WALPHA      SETTING_QUANT(0x0104)
#define SETTING_QUANT_WZERO_POINT SETTING_QUANT(0x0105)
#define SETTING_QUANT_WBITS       SETTING_QUANT(0x0106)
#define SETTING_QUANT_OALPHA      SETTING_QUANT(0x0107)
#define SETTING_QUANT_OZERO_POINT SETTING_QUANT(0x0108)
#define SETTING_QUANT_OBITS       SETTING_QUANT(0x0109)
#define SETTING_QUANT_QTYPE       SETTING_QUANT(0x010a)

/* ---- workspaces and modules (workspace.h:27-29, module.h:45-79) ----------------------------------------- */
struct _module_t;
typedef struct workspace_t {
    const struct _module_t *module_type; /* must be the first member of every module's workspace struct */
} workspace_t;

typedef struct _module_t {
    uint32_t op_group;
    const char *(*name_func)(const workspace_t *);
    const mem_tp *(*memtype_func)(const workspace_t *);
    workspace_t *(*new_func)(const setting_entry_t *); /* runners pass NULL; else terminated by item == 0 */
    void (*delete_func)(workspace_t *);
    op_tp_entry_t *op_tp_entry;
} module_t;

static inline workspace_t *workspace_new(const module_t *m, const setting_entry_t *s) { return m->new_func(s); }
static inline void workspace_delete(workspace_t *ws) { ws->module_type->delete_func(ws); }
static inline const char *workspace_name(workspace_t *ws) { return ws->module_type->name_func(ws); }
static inline const mem_tp *workspace_memtype(workspace_t *ws) { return ws->module_type->memtype_func(ws); }

op_t *workspace_new_op(workspace_t *ws, uint64_t op_tp_code, uint8_t input_size, tensor_t *const *input_tensor);
bool workspace_support_op(workspace_t *ws, uint64_t op_tp_code, bool strict);

/* ---- parade: the flat, ordered operator list of a loaded case (parade.h:27-52) ----------------------------- */
typedef struct _parade_t parade_t;
typedef tensor_t *const *tensor_array_t;
parade_t *parade_new(void);
void parade_delete(parade_t *parade);
bool parade_get_input_tensors(parade_t *parade, size_t *count, tensor_array_t *tensors);
bool parade_get_output_tensors(parade_t *parade, size_t *count, tensor_array_t *tensors);
void parade_prepare(parade_t *parade);
void parade_run(parade_t *parade);
bool parade_apply_reshape(parade_t *parade);

/* Input pre-processing description that a version-2 engine file may attach to an input (transform.h:25-73).  The
 * runtime only carries it for the caller's image pipeline (parade.c:128-153); nothing here applies it. */
typedef struct frame_t frame_t;
typedef struct pixel_t {
    float r, g, b;
} pixel_t;
typedef struct transform_param_t {
    const char *tensor_name;
    uint32_t operators;
    size_t batch;
    frame_t **frames;
    int32_t tensor_type;
    int32_t (*rois)[4];
    int32_t (*dst_rois)[4];
    float (*mats)[3][3];
    pixel_t means, stds, paddings;
} transform_param_t;
typedef struct transform_tensor_t { /* what an input tensor with with_transform == 1 really is */
    tensor_t tensor;
    size_t capacity;
    transform_param_t param;
} transform_tensor_t;
bool parade_get_transfrom_param(parade_t *parade, size_t *count, transform_param_t *params); /* sic, parade.h:40 */
void parade_set_transfrom_param(parade_t *parade, transform_param_t *params);

/* ---- engine file reader (serialize.h:27-75; formats: serialize_v1.c:26-95, serialize_v2.c:25-98) --------------------------------- */
typedef size_t (*nart_buffer_read_func)(size_t sz, void *data, void *param);
typedef struct buffer_t buffer_t;
buffer_t *nart_buffer_new(size_t buffer_size);
void nart_buffer_delete(buffer_t *buf);
void buffer_set_buffer_read_func(buffer_t *buf, nart_buffer_read_func func, void *param);
size_t nart_buffer_read(buffer_t *buf, size_t sz, void *data);

typedef struct {
    workspace_t *const *workspaces; /* NULL-terminated */
    const mem_tp *input_mem_tp;
} deserialize_param_t;
parade_t *deserialize_parade(buffer_t *buf, const deserialize_param_t *param);

#ifdef __cplusplus
}
#endif
#endif /* NART_HIP_ART_H */
