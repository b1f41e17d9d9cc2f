/*
 * A small host core implementing the art C API (include/art/art.h): element types, host memory,
 * tensors, typed settings, operator life cycle, op lookup in a module's table, the parade (ordered op
 * list) and the engine file reader (versions 1 and 2).  It exists so that the `hip` case module can be loaded and
 * driven where a NART installation is not available; it follows the behaviour of the reference core
 * (art/src/{data_type,mem,tensor,settings,op,module,parade,serialize,serialize_v1}.c) for the parts a
 * quantized CNN case uses and makes no attempt to cover the rest of NART.
 */
#include <inttypes.h>
#include <stdarg.h>
#include <string.h>

#include "art/art.h"
#include "core_internal.h"

/* ---- element types (data_type.c:22-80) ------------------------------------------------------------ */
static const char *const k_dtype_names[] = {"UNKNOWN", "INT8", "INT16", "INT32", "INT64", "UINT8", "UINT16", "UINT32",
                                            "UINT64", "FLOAT16", "FLOAT32", "FLOAT64", "STR", "PTR", "CPTR", "BOOL"};
#define N_DTYPES (sizeof(k_dtype_names) / sizeof(k_dtype_names[0]))

ART_PUBLIC size_t datatype_sizeof(uint32_t dtype)
{
    static const uint8_t sz[N_DTYPES] = {0, 1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8, sizeof(void *), sizeof(void *), 0,
                                         sizeof(bool)};
    return dtype < N_DTYPES ? sz[dtype] : 0;
}

ART_PUBLIC const char *datatype_name_from_type(uint32_t dtype) { return dtype < N_DTYPES ? k_dtype_names[dtype] : NULL; }

ART_PUBLIC uint32_t datatype_type_from_name(const char *name)
{
    if (name == NULL)
        return 0;
    for (uint32_t i = 0; i < N_DTYPES; ++i)
        if (strncmp(name, k_dtype_names[i], strlen(k_dtype_names[i])) == 0)
            return i;
    return 0;
}

/* ---- host memory (mem.c:24-121) --------------------------------------------------------------------- */
typedef struct {
    mem_t m;
    size_t sz;
    void *data;
} host_mem_t;

static mem_t *host_mem_new(void) { return (mem_t *)calloc(1, sizeof(host_mem_t)); }

static void host_mem_free(mem_t *mm)
{
    host_mem_t *m = (host_mem_t *)mm;
    free(m->data);
    m->data = NULL;
    m->sz = 0;
}

static void host_mem_delete(mem_t *m)
{
    host_mem_free(m);
    free(m);
}

static bool host_mem_alloc(mem_t *mm, size_t sz)
{
    host_mem_t *m = (host_mem_t *)mm;
    if (m->sz >= sz)
        return true; /* grow-only */
    void *p = realloc(m->data, sz);
    if (p == NULL)
        return false;
    memset((char *)p + m->sz, 0, sz - m->sz); /* unlike the reference, fresh bytes are defined */
    m->data = p;
    m->sz = sz;
    return true;
}

static void *host_mem_data(const mem_t *m) { return ((const host_mem_t *)m)->data; }
static size_t host_mem_size(mem_t *m) { return ((host_mem_t *)m)->sz; }
static void *host_copy(void *to, const void *from, size_t sz) { return memcpy(to, from, sz); }

static const mem_tp k_cpu_mem_tp = {
    .name = "cpu_mem",
    .new_func = host_mem_new,
    .delete_func = host_mem_delete,
    .alloc_func = host_mem_alloc,
    .free_func = host_mem_free,
    .data_func = host_mem_data,
    .cpu_data_func = host_mem_data,
    .size_func = host_mem_size,
    .copy_from_cpu_func = host_copy,
    .copy_to_cpu_func = host_copy,
    .share_from_func = extern_mem_from_data,
};
ART_PUBLIC const mem_tp *cpu_mem_tp = &k_cpu_mem_tp;

static void extern_mem_delete(mem_t *m) { free(m); } /* the wrapped buffer belongs to the caller */
static const mem_tp k_extern_mem_tp = {
    .name = "cpu_mem",
    .delete_func = extern_mem_delete,
    .data_func = host_mem_data,
    .cpu_data_func = host_mem_data,
    .size_func = host_mem_size,
};

ART_PUBLIC mem_t *extern_mem_from_data(void *data, size_t sz)
{
    host_mem_t *m = (host_mem_t *)calloc(1, sizeof(host_mem_t));
    m->m.tp = &k_extern_mem_tp;
    m->m.refcount = 1;
    m->data = data;
    m->sz = sz;
    return &m->m;
}

ART_PUBLIC mem_t *mem_dup(mem_t *m)
{
    if (m != NULL)
        m->refcount++;
    return m;
}

/* ---- tensors (tensor.c:22-148) ------------------------------------------------------------------------ */
ART_PUBLIC tensor_t *tensor_new(const mem_tp *tp, uint32_t dtype)
{
    tensor_t *t = (tensor_t *)calloc(1, sizeof(tensor_t));
    t->mem = mem_new(tp);
    t->dtype = dtype;
    t->shape.dim_size = 4;
    t->shape.channel_axis = 1;
    for (int i = 0; i < MAX_DIM; ++i)
        t->shape.dim[i] = 1; /* dims beyond dim_size read as 1 (the reference leaves them undefined) */
    return t;
}

ART_PUBLIC void tensor_set_name(tensor_t *t, const char *name)
{
    free(t->name);
    t->name = name ? strdup(name) : NULL;
}

ART_PUBLIC void tensor_free(tensor_t *t)
{
    if (t->mem != NULL) {
        mem_delete(t->mem);
        t->mem = NULL;
    }
    free(t->name);
    t->name = NULL;
}

ART_PUBLIC void tensor_delete(tensor_t *t)
{
    tensor_free(t);
    free(t);
}

ART_PUBLIC bool tensor_shape_eq(const shape_t *a, const shape_t *b)
{
    if (a->dim_size != b->dim_size || a->batch_axis != b->batch_axis || a->channel_axis != b->channel_axis)
        return false;
    for (int i = 0; i < a->dim_size; ++i)
        if (a->dim[i] != b->dim[i])
            return false;
    return true;
}

/* 0 keeps a dimension, -1 (at most once) is inferred from the element count (tensor.c:78-137) */
ART_PUBLIC bool tensor_reshape(tensor_t *t, const int n, const int shape[])
{
    ART_CHECK(n >= 0 && n <= MAX_DIM);
    uint64_t old_count = shape_count(&t->shape), known = 1;
    uint32_t dims[MAX_DIM];
    int infer = -1;
    for (int i = 0; i < n; ++i) {
        if (shape[i] == -1) {
            if (infer >= 0) {
                fprintf(stderr, "[art] reshape: -1 given more than once\n");
                return false;
            }
            infer = i;
            continue;
        }
        if (shape[i] == 0)
            ART_CHECK(i < t->shape.dim_size);
        dims[i] = shape[i] == 0 ? t->shape.dim[i] : (uint32_t)shape[i];
        known *= dims[i];
    }
    if (infer >= 0) {
        ART_CHECK(known != 0 && old_count % known == 0);
        dims[infer] = (uint32_t)(old_count / known);
    }
    if (t->shape.batch_axis > n)
        t->shape.batch_axis = -1;
    if (t->shape.channel_axis > n)
        t->shape.channel_axis = -1;
    t->shape.dim_size = n;
    for (int i = 0; i < MAX_DIM; ++i)
        t->shape.dim[i] = i < n ? dims[i] : 1;
    if (old_count != 0 && shape_count(&t->shape) > old_count)
        tensor_alloc(t);
    return true;
}

ART_PUBLIC void tensor_share(tensor_t *from, tensor_t *to)
{
    if (from == NULL || to == NULL)
        return;
    mem_delete(to->mem);
    to->mem = mem_dup(from->mem);
}

/* ---- settings (settings.c:24-166) ---------------------------------------------------------------------- */
static size_t setting_bytes(size_t n) { return sizeof(struct _setting_t) + n * sizeof(setting_entry_t); }

ART_PUBLIC setting_t setting_new_with_reserved(size_t count)
{
    setting_t s = (setting_t)malloc(setting_bytes(count));
    s->len = 0;
    s->reserved = count;
    return s;
}

ART_PUBLIC setting_t setting_new(void) { return setting_new_with_reserved(4); }

static void entry_release(setting_entry_t *e)
{
    if (e->tp == ENUM_SETTING_VALUE_REPEATED) {
        if (e->dtype == dtSTR)
            for (size_t j = 0; j < e->v.repeated.len; ++j)
                free(((char **)e->v.repeated.values)[j]);
        free(e->v.repeated.values);
    } else if (e->dtype == dtSTR) {
        free(e->v.single.value.str);
    }
}

ART_PUBLIC void setting_delete(setting_t s)
{
    if (s == NULL)
        return;
    for (size_t i = 0; i < s->len; ++i)
        entry_release(&s->entries[i]);
    free(s);
}

ART_PUBLIC void setting_shrink(setting_t *s)
{
    if (s == NULL || *s == NULL || (*s)->len == (*s)->reserved)
        return;
    setting_t r = (setting_t)realloc(*s, setting_bytes((*s)->len));
    if (r != NULL) {
        r->reserved = r->len;
        *s = r;
    }
}

ART_PUBLIC setting_entry_t *setting_search(setting_t s, uint32_t item)
{
    if (s == NULL)
        return NULL;
    for (size_t i = 0; i < s->len; ++i)
        if (s->entries[i].item == item)
            return &s->entries[i];
    return NULL;
}

/* the slot for `item`: an existing one (its old value released) or a fresh one at the end */
static setting_entry_t *setting_slot(setting_t *s, uint32_t item)
{
    setting_entry_t *e = setting_search(*s, item);
    if (e != NULL) {
        entry_release(e);
        return e;
    }
    if ((*s)->len >= (*s)->reserved) {
        size_t n = (*s)->reserved ? (*s)->reserved * 2 : 1;
        setting_t r = (setting_t)realloc(*s, setting_bytes(n));
        ART_CHECK(r != NULL);
        r->reserved = n;
        *s = r;
    }
    return &(*s)->entries[(*s)->len++];
}

ART_PUBLIC void setting_set_single(setting_t *s, uint32_t item, uint32_t dtype, uvalue_t v)
{
    setting_entry_t *e = setting_slot(s, item);
    e->item = item;
    e->dtype = dtype;
    e->tp = ENUM_SETTING_VALUE_SINGLE;
    e->v.single.value = v;
    if (dtype == dtSTR && v.str != NULL)
        e->v.single.value.str = strdup(v.str);
}

ART_PUBLIC void *setting_alloc_repeated(setting_t *s, uint32_t item, uint32_t dtype, size_t count)
{
    setting_entry_t *e = setting_slot(s, item);
    e->item = item;
    e->dtype = dtype;
    e->tp = ENUM_SETTING_VALUE_REPEATED;
    e->v.repeated.values = count ? calloc(count, datatype_sizeof(dtype)) : NULL;
    e->v.repeated.len = count;
    return e->v.repeated.values;
}

/* ---- operator life cycle (op.c:27-77) -------------------------------------------------------------------- */
ART_PUBLIC void op_init_default(op_t *op, op_tp_entry_t *entry, workspace_t *ws, uint16_t n_in,
                                tensor_t *const *inputs)
{
    op->entry = entry;
    op->workspace = ws;
    op->input_size = n_in;
    op->input_tensors = (tensor_t **)malloc(sizeof(tensor_t *) * (n_in ? n_in : 1));
    memcpy(op->input_tensors, inputs, sizeof(tensor_t *) * n_in);
    op->setting = setting_new();
}

ART_PUBLIC void op_destroy_default(op_t *op)
{
    free(op->input_tensors);
    op->input_tensors = NULL;
    if (op->output_size > 0) {
        for (size_t i = 0; i < op->output_size; ++i)
            tensor_free(&op->output_tensors[i]);
        free(op->output_tensors);
        op->output_tensors = NULL;
        op->output_size = 0;
    }
    setting_delete(op->setting);
    op->setting = NULL;
}

ART_PUBLIC void op_delete(op_t *op)
{
    op->entry->destroy_func(op);
    op_destroy_default(op);
    op->entry->dealloc_func(op);
}

ART_PUBLIC bool op_config(op_t *op)
{
    if (op == NULL)
        return false;
    op->entry->config_func(op);
    return op->entry->tp->infer_output_func(op);
}

ART_PUBLIC void op_prepare(op_t *op)
{
    setting_shrink(&op->setting);
    op->entry->prepare_func(op);
}

/* ---- typed settings on an op (op.c:79-277) ----------------------------------------------------------------- */
static const setting_constraint_t *find_constraint(const op_t *op, uint32_t item)
{
    for (const setting_constraint_t *c = op->entry->tp->constraints; c->item != SETTING_END; ++c)
        if (c->item == item)
            return c;
    return NULL;
}

ART_PUBLIC bool op_setting_if_set(const op_t *op, uint32_t item)
{
    return op != NULL && setting_search(op->setting, item) != NULL;
}

static void store_by_dtype(uint32_t dtype, uvalue_t v, void *out)
{
    switch (datatype_sizeof(dtype)) {
    case 1:
        *(uint8_t *)out = v.u8;
        break;
    case 2:
        *(uint16_t *)out = v.u16;
        break;
    case 4:
        *(uint32_t *)out = v.u32;
        break;
    case 8:
        *(uint64_t *)out = v.u64;
        break;
    default:
        break;
    }
}

ART_PUBLIC bool op_setting_single_get(const op_t *op, uint32_t item, uint32_t dtype, void *out)
{
    if (op == NULL)
        return false;
    const setting_entry_t *e = setting_search(op->setting, item);
    uvalue_t v;
    if (e != NULL) {
        if (e->dtype != dtype || e->tp != ENUM_SETTING_VALUE_SINGLE)
            return false;
        v = e->v.single.value;
    } else { /* fall back to the op type's default for an optional setting */
        const setting_constraint_t *c = find_constraint(op, item);
        if (c == NULL || c->dtype != dtype || c->ctp != ENUM_SETTING_CONSTRAINT_OPTIONAL)
            return false;
        v = c->constraint.optional.default_value;
    }
    if (dtype == dtCPTR)
        *(const void **)out = v.cptr;
    else
        store_by_dtype(dtype, v, out);
    return true;
}

ART_PUBLIC bool op_setting_single_set(op_t *op, uint32_t item, uint32_t dtype, ...)
{
    if (op == NULL)
        return false;
    const setting_constraint_t *c = find_constraint(op, item);
    if (c != NULL && (c->dtype != dtype || c->ctp == ENUM_SETTING_CONSTRAINT_REPEATED))
        return false;
    uvalue_t v;
    memset(&v, 0, sizeof v);
    va_list ap;
    va_start(ap, dtype);
    switch (dtype) { /* values arrive promoted: narrow integers as 32-bit, float as double */
    case dtBOOL:
        v.b = va_arg(ap, uint32_t) != 0;
        break;
    case dtINT8:
    case dtUINT8:
        v.u8 = (uint8_t)va_arg(ap, uint32_t);
        break;
    case dtINT16:
    case dtUINT16:
    case dtFLOAT16:
        v.u16 = (uint16_t)va_arg(ap, uint32_t);
        break;
    case dtINT32:
    case dtUINT32:
        v.u32 = va_arg(ap, uint32_t);
        break;
    case dtFLOAT32:
        v.f32 = (float)va_arg(ap, double);
        break;
    case dtINT64:
    case dtUINT64:
    case dtFLOAT64:
        v.u64 = va_arg(ap, uint64_t);
        break;
    case dtSTR:
    case dtPTR:
    case dtCPTR:
        v.cptr = va_arg(ap, void *);
        break;
    default:
        break;
    }
    va_end(ap);
    setting_set_single(&op->setting, item, dtype, v);
    return true;
}

ART_PUBLIC bool op_setting_array_set(op_t *op, uint32_t item, uint32_t dtype, size_t len, const void *in)
{
    if (op == NULL)
        return false;
    const setting_constraint_t *c = find_constraint(op, item);
    if (c != NULL && (c->dtype != dtype || c->ctp != ENUM_SETTING_CONSTRAINT_REPEATED))
        return false;
    void *dst = setting_alloc_repeated(&op->setting, item, dtype, len);
    if (dst == NULL)
        return len == 0;
    if (dtype == dtSTR) {
        for (size_t i = 0; i < len; ++i)
            ((char **)dst)[i] = strdup(((const char *const *)in)[i]);
    } else {
        memcpy(dst, in, datatype_sizeof(dtype) * len);
    }
    return true;
}

ART_PUBLIC bool op_setting_array_get(const op_t *op, uint32_t item, uint32_t dtype, size_t *len, void *out)
{
    if (op == NULL)
        return false;
    size_t n = 0;
    void *values = NULL; /* handed out by reference: valid for the life of the op */
    const setting_entry_t *e = setting_search(op->setting, item);
    if (e != NULL) {
        if (e->dtype != dtype || e->tp != ENUM_SETTING_VALUE_REPEATED)
            return false;
        n = e->v.repeated.len;
        values = e->v.repeated.values;
    } else {
        const setting_constraint_t *c = find_constraint(op, item);
        if (c == NULL || c->ctp != ENUM_SETTING_CONSTRAINT_REPEATED)
            return false; /* an unset repeated setting of the op type reads as empty */
    }
    if (len != NULL)
        *len = n;
    if (out != NULL)
        *(void **)out = values;
    return true;
}

/* ---- op lookup in a module's table (module.c:23-75) -------------------------------------------------------- */
ART_PUBLIC op_t *workspace_new_op(workspace_t *ws, uint64_t code, uint8_t n_in, tensor_t *const *inputs)
{
    ART_CHECK(ws != NULL);
    const module_t *mod = ws->module_type;
    for (op_tp_entry_t *e = mod->op_tp_entry; e != NULL && e->tp != NULL; ++e) {
        if (e->tp->op_tp_code != code)
            continue;
        op_t *op = e->alloc_func(ws);
        if (op != NULL)
            op_init_default(op, e, ws, n_in, inputs);
        return op;
    }
    ART_FATAL("Op typecode: 0x%" PRIx64 " not found\n", code);
    return NULL;
}

ART_PUBLIC bool workspace_support_op(workspace_t *ws, uint64_t code, bool strict)
{
    const module_t *mod = ws->module_type;
    if (code & 0x80000000ull)
        strict = true; /* module-private ops never match across groups */
    for (op_tp_entry_t *e = mod->op_tp_entry; e != NULL && e->tp != NULL; ++e) {
        if (strict ? code == (e->tp->op_tp_code | ((uint64_t)mod->op_group << 32))
                   : (code & 0xffffffffull) == (e->tp->op_tp_code & 0xffffffffull))
            return true;
    }
    return false;
}

/* ---- parade (parade.c, parade_impl.h:23-32) ------------------------------------------------------------------ */
ART_PUBLIC parade_t *parade_new(void) { return (parade_t *)calloc(1, sizeof(parade_t)); }

ART_PUBLIC void parade_delete(parade_t *p)
{
    if (p == NULL)
        return;
    for (size_t i = 0; i < p->op_count; ++i)
        op_delete(p->ops[i]);
    for (size_t i = 0; i < p->input_tensor_count; ++i)
        tensor_delete(p->input_tensors[i]);
    for (size_t i = 0; i < p->weight_tensor_count; ++i)
        tensor_delete(p->weight_tensors[i]);
    free(p->ops);
    free(p->input_tensors);
    free(p->weight_tensors);
    free(p->output_tensors);
    free(p);
}

ART_PUBLIC bool parade_get_input_tensors(parade_t *p, size_t *count, tensor_array_t *tensors)
{
    *count = p->input_tensor_count;
    *tensors = p->input_tensors;
    return true;
}

ART_PUBLIC bool parade_get_output_tensors(parade_t *p, size_t *count, tensor_array_t *tensors)
{
    *count = p->output_tensor_count;
    *tensors = p->output_tensors;
    return true;
}

ART_PUBLIC void parade_prepare(parade_t *p)
{
    for (size_t i = 0; p != NULL && i < p->op_count; ++i)
        op_prepare(p->ops[i]);
}

ART_PUBLIC void parade_run(parade_t *p)
{
    for (size_t i = 0; p != NULL && i < p->op_count; ++i)
        op_run(p->ops[i]);
}

/* after the caller changed an input shape: re-infer and re-prepare every op in order (parade.c:199-215) */
ART_PUBLIC bool parade_apply_reshape(parade_t *p)
{
    if (p == NULL)
        return false;
    for (size_t i = 0; i < p->op_count; ++i) {
        if (!p->ops[i]->entry->tp->infer_output_func(p->ops[i]))
            return false;
        p->ops[i]->entry->prepare_func(p->ops[i]);
    }
    return true;
}

void parade_push_op(parade_t *p, op_t *op)
{
    p->ops = (op_t **)realloc(p->ops, sizeof(op_t *) * (p->op_count + 1));
    p->ops[p->op_count++] = op;
}

/* ---- streaming read buffer (serialize.c:26-90) ------------------------------------------------------------------ */
struct buffer_t {
    size_t pos, len, cap;
    nart_buffer_read_func read_func;
    void *param;
    uint8_t data[];
};

ART_PUBLIC buffer_t *nart_buffer_new(size_t cap)
{
    buffer_t *b = (buffer_t *)calloc(1, sizeof(buffer_t) + cap);
    if (b != NULL)
        b->cap = cap;
    return b;
}

ART_PUBLIC void nart_buffer_delete(buffer_t *b) { free(b); }

ART_PUBLIC void buffer_set_buffer_read_func(buffer_t *b, nart_buffer_read_func f, void *param)
{
    b->read_func = f;
    b->param = param;
}

ART_PUBLIC size_t nart_buffer_read(buffer_t *b, size_t sz, void *out)
{
    size_t done = 0;
    while (b != NULL && out != NULL && done < sz) {
        if (b->pos == b->len) { /* refill */
            if (b->read_func == NULL)
                break;
            b->len = b->read_func(b->cap, b->data, b->param);
            b->pos = 0;
            if (b->len == 0)
                break;
        }
        size_t n = sz - done < b->len - b->pos ? sz - done : b->len - b->pos;
        memcpy((uint8_t *)out + done, b->data + b->pos, n);
        b->pos += n;
        done += n;
    }
    return done;
}

/* ---- engine file, versions 1 and 2 (layouts: serialize_v1.c:26-95, serialize_v2.c:25-98; readers :203-340) ----------------------------------- */
static int32_t rd_i32(buffer_t *b)
{
    int32_t v = 0;
    ART_CHECK(nart_buffer_read(b, 4, &v) == 4);
    return v;
}

static uint64_t rd_u64(buffer_t *b)
{
    uint64_t v = 0;
    ART_CHECK(nart_buffer_read(b, 8, &v) == 8);
    return v;
}

static char *rd_string(buffer_t *b) /* int32 length, then that many bytes (no terminator in the file) */
{
    int32_t n = rd_i32(b);
    ART_CHECK(n >= 0);
    if (n == 0)
        return NULL; /* like the reference: an empty string reads as no string */
    char *s = (char *)calloc((size_t)n + 1, 1);
    ART_CHECK(nart_buffer_read(b, (size_t)n, s) == (size_t)n);
    return s;
}

static shape_t rd_shape(buffer_t *b) /* dim_size, dims, channel_axis, batch_axis — in this order (serialize.c:230-240) */
{
    shape_t s;
    for (int i = 0; i < MAX_DIM; ++i)
        s.dim[i] = 1;
    uint32_t n = (uint32_t)rd_i32(b);
    ART_CHECK(n <= MAX_DIM);
    s.dim_size = (int32_t)n;
    if (n > 0)
        ART_CHECK(nart_buffer_read(b, n * sizeof(uint32_t), s.dim) == n * sizeof(uint32_t));
    s.channel_axis = rd_i32(b);
    s.batch_axis = rd_i32(b);
    return s;
}

static tensor_t *rd_tensor_decl(buffer_t *b, const mem_tp *tp)
{
    uint32_t dtype = (uint32_t)rd_i32(b);
    char *name = rd_string(b);
    shape_t shape = rd_shape(b);
    tensor_t *t = tensor_new(tp, dtype);
    t->shape = shape;
    t->name = name;
    return t;
}

static workspace_t *pick_workspace(uint64_t code, workspace_t *const *wss)
{
    for (int strict = 1; strict >= 0 && wss != NULL; --strict) /* exact group first, then by op code alone */
        for (workspace_t *const *w = wss; *w != NULL; ++w)
            if (workspace_support_op(*w, code, strict))
                return *w;
    return NULL;
}

static void rd_setting(op_t *op, buffer_t *b)
{
    bool repeated = rd_i32(b) != 0;
    uint32_t item = (uint32_t)rd_i32(b), dtype = (uint32_t)rd_i32(b);
    if (!repeated) {
        if (dtype == dtSTR) {
            char *s = rd_string(b);
            ART_CHECK(op_setting_single_set(op, item, dtype, s));
            free(s);
            return;
        }
        uvalue_t u;
        memset(&u, 0, sizeof u);
        size_t sz = datatype_sizeof(dtype);
        ART_CHECK(sz > 0 && nart_buffer_read(b, sz, &u) == sz);
        switch (dtype) {
        case dtFLOAT32:
            ART_CHECK(op_setting_single_set(op, item, dtype, (double)u.f32));
            break;
        case dtINT64:
        case dtUINT64:
        case dtFLOAT64:
            ART_CHECK(op_setting_single_set(op, item, dtype, u.u64));
            break;
        default:
            ART_CHECK(op_setting_single_set(op, item, dtype, u.u32));
            break;
        }
        return;
    }
    int32_t count32 = rd_i32(b);
    ART_CHECK(count32 >= 0);
    size_t count = (size_t)count32;
    if (dtype == dtSTR) {
        char **strs = (char **)calloc(count ? count : 1, sizeof(char *));
        ART_CHECK(strs != NULL);
        for (size_t i = 0; i < count; ++i)
            strs[i] = rd_string(b);
        ART_CHECK(op_setting_array_set(op, item, dtype, count, strs));
        for (size_t i = 0; i < count; ++i)
            free(strs[i]);
        free(strs);
        return;
    }
    size_t bytes = count * datatype_sizeof(dtype);
    void *m = malloc(bytes ? bytes : 1);
    if (bytes)
        ART_CHECK(nart_buffer_read(b, bytes, m) == bytes);
    ART_CHECK(op_setting_array_set(op, item, dtype, count, m));
    free(m);
}

/* version 2 (serialize_v2.c:25-98, :215-249): every input declaration is followed by a flag and, if it is set, by the
 * pre-processing parameters {operators, frame type, mean, std, padding}; the tensor then is a transform_tensor_t */
static tensor_t *rd_input_transform(buffer_t *b, tensor_t *plain)
{
    if (rd_i32(b) == 0)
        return plain;
    transform_tensor_t *tt = (transform_tensor_t *)calloc(1, sizeof(transform_tensor_t));
    tt->tensor = *plain; /* takes over mem and name */
    free(plain);
    tt->tensor.with_transform = 1;
    tt->param.operators = (uint32_t)rd_i32(b);
    (void)rd_i32(b); /* frame type: read and dropped, as in the reference */
    pixel_t *px[3] = {&tt->param.means, &tt->param.stds, &tt->param.paddings};
    for (int i = 0; i < 3; ++i)
        ART_CHECK(nart_buffer_read(b, sizeof(pixel_t), px[i]) == sizeof(pixel_t));
    return &tt->tensor;
}

ART_PUBLIC bool parade_get_transfrom_param(parade_t *parade, size_t *count, transform_param_t *params)
{
    if (parade == NULL)
        return false;
    if (count != NULL)
        *count = parade->input_tensor_count;
    if (params != NULL) { /* the reference returns input 0's block unconditionally (parade.c:128-138) */
        if (parade->input_tensor_count == 0 || !parade->input_tensors[0]->with_transform)
            return false;
        *params = ((transform_tensor_t *)parade->input_tensors[0])->param;
    }
    return true;
}

ART_PUBLIC void parade_set_transfrom_param(parade_t *parade, transform_param_t *params)
{
    for (size_t i = 0; parade != NULL && params != NULL && params->tensor_name != NULL && i < parade->input_tensor_count; ++i) {
        tensor_t *t = parade->input_tensors[i];
        if (t->name != NULL && strncmp(params->tensor_name, t->name, 64) == 0) {
            if (t->with_transform) {
                ((transform_tensor_t *)t)->param = *params;
                return;
            }
            printf("tensor [%s] found, but with no transform flag\n", params->tensor_name);
        }
    }
}

static parade_t *read_parade(buffer_t *b, const deserialize_param_t *param, uint32_t version)
{
    parade_t *p = parade_new();
    int32_t n_tensors = rd_i32(b);
    ART_CHECK(n_tensors >= 0);
    tensor_t **tab = (tensor_t **)calloc((size_t)n_tensors + 1, sizeof(tensor_t *));
    size_t cur = 0;

    int32_t n_in = rd_i32(b);
    ART_CHECK(n_in >= 0 && n_in <= n_tensors); /* every count below comes from the file: none may outrun the table */
    p->input_tensors = (tensor_t **)calloc((size_t)n_in + 1, sizeof(tensor_t *));
    for (int32_t i = 0; i < n_in; ++i) {
        tensor_t *t = rd_tensor_decl(b, param->input_mem_tp);
        if (version >= 2)
            t = rd_input_transform(b, t);
        tab[cur++] = p->input_tensors[p->input_tensor_count++] = t;
    }

    int32_t n_w = rd_i32(b);
    ART_CHECK(n_w >= 0 && n_w <= n_tensors - n_in);
    p->weight_tensors = (tensor_t **)calloc((size_t)n_w + 1, sizeof(tensor_t *));
    for (int32_t i = 0; i < n_w; ++i) { /* weights carry their data inline; it is written through the host view */
        tensor_t *t = rd_tensor_decl(b, param->input_mem_tp);
        tensor_alloc(t);
        size_t bytes = shape_count(&t->shape) * datatype_sizeof(t->dtype);
        if (bytes)
            ART_CHECK(nart_buffer_read(b, bytes, mem_cpu_data(t->mem)) == bytes);
        tab[cur++] = p->weight_tensors[p->weight_tensor_count++] = t;
    }

    int32_t n_ops = rd_i32(b);
    for (int32_t i = 0; i < n_ops; ++i) {
        int32_t op_in = rd_i32(b), op_out = rd_i32(b);
        ART_CHECK(op_in >= 0 && op_in <= 255 && op_out >= 0); /* workspace_new_op takes the input count as a byte */
        uint64_t code = rd_u64(b);
        tensor_t **ins = (tensor_t **)calloc((size_t)op_in + 1, sizeof(tensor_t *));
        for (int32_t j = 0; j < op_in; ++j) {
            int32_t idx = rd_i32(b);
            ART_CHECK(idx >= 0 && (size_t)idx < cur);
            ins[j] = tab[idx];
        }
        workspace_t *ws = pick_workspace(code, param->workspaces);
        if (ws == NULL)
            ART_FATAL("no workspace supports op 0x%" PRIx64 "\n", code);
        if ((code & 0x80000000ull) == 0)
            code &= 0xffffffffull; /* generic ops are registered without their group */
        op_t *op = workspace_new_op(ws, code, (uint8_t)op_in, ins);
        for (int32_t n_set = rd_i32(b); n_set > 0; --n_set)
            rd_setting(op, b);
        ART_CHECK(op_config(op));
        ART_CHECK((size_t)op_out == op->output_size);
        for (int32_t j = 0; j < op_out; ++j) {
            ART_CHECK(cur < (size_t)n_tensors);
            tab[cur++] = &op->output_tensors[j];
        }
        free(ins);
        parade_push_op(p, op);
    }

    int32_t n_out = rd_i32(b);
    ART_CHECK(n_out >= 0 && n_out <= n_tensors);
    p->output_tensors = (tensor_t **)calloc((size_t)n_out + 1, sizeof(tensor_t *));
    for (int32_t i = 0; i < n_out; ++i) {
        int32_t idx = rd_i32(b);
        char *name = rd_string(b);
        ART_CHECK(idx >= 0 && (size_t)idx < cur);
        p->output_tensors[p->output_tensor_count++] = tab[idx];
        tensor_set_name(tab[idx], name);
        free(name);
    }

    for (int32_t n_share = rd_i32(b); n_share > 0; --n_share) {
        int32_t from = rd_i32(b), to = rd_i32(b);
        ART_CHECK(from >= 0 && to >= 0 && (size_t)from < cur && (size_t)to < cur);
        tensor_share(tab[from], tab[to]);
    }
    free(tab);
    return p;
}

ART_PUBLIC parade_t *deserialize_parade(buffer_t *b, const deserialize_param_t *param)
{
    uint32_t version = (uint32_t)rd_i32(b); /* head: version, name (serialize.c:143-160) */
    char *name = rd_string(b);
    free(name);
    if (version != 1 && version != 2)
        ART_FATAL("engine file version %u is not supported by this core (versions 1 and 2)\n", version);
    return read_parade(b, param, version);
}
