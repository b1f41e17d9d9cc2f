/*
 * Shape inference and the shared op-type objects of the generic operators a quantized CNN case uses:
 * conv_2d, ip, pool, relu, add, eltwise, reshape.  Case modules point their table entries at these
 * objects (the reference keeps them in art/src/op.c); `infer_output_func` creates the op's output
 * tensors on first use — with the memory type of input 0 — and (re)computes their shapes.
 */
#include <math.h>
#include <string.h>

#include "art/art.h"

/* first call: one output tensor whose memory comes from the same mem_tp as input 0 (op.c:557-563) */
static tensor_t *single_output(op_t *op, bool share_input_mem)
{
    if (op->output_size == 0) {
        op->output_size = 1;
        op->output_tensors = (tensor_t *)calloc(1, sizeof(tensor_t));
        tensor_t *in = op->input_tensors[0];
        op->output_tensors[0].mem = share_input_mem ? mem_dup(in->mem) : mem_new(in->mem->tp);
        op->output_tensors[0].dtype = in->dtype;
    }
    ART_CHECK(op->output_size == 1);
    return &op->output_tensors[0];
}

static uint32_t get_u32(const op_t *op, uint32_t item)
{
    uint32_t v = 0;
    ART_CHECK(op_setting_single_get(op, item, dtUINT32, &v));
    return v;
}

/* ---- conv_2d (op.c:481-566) ------------------------------------------------------------------------- */
static bool infer_conv_2d(op_t *op)
{
    ART_CHECK(op->input_size == 2 || op->input_size == 3);
    const tensor_t *x = op->input_tensors[0], *w = op->input_tensors[1];
    const uint32_t group = get_u32(op, SETTING_CONV_2D_GROUP), K = get_u32(op, SETTING_CONV_2D_NUM_OUTPUT);
    const uint32_t ph = get_u32(op, SETTING_CONV_2D_PAD_H), pw = get_u32(op, SETTING_CONV_2D_PAD_W);
    const uint32_t kh = get_u32(op, SETTING_CONV_2D_KERNEL_H), kw = get_u32(op, SETTING_CONV_2D_KERNEL_W);
    const uint32_t sh = get_u32(op, SETTING_CONV_2D_STRIDE_H), sw = get_u32(op, SETTING_CONV_2D_STRIDE_W);
    const uint32_t dh = get_u32(op, SETTING_CONV_2D_HOLE_H), dw = get_u32(op, SETTING_CONV_2D_HOLE_W);
    ART_CHECK(x->shape.dim_size == 4 && w->shape.dim_size == 4);
    ART_CHECK(x->shape.batch_axis == 0 && x->shape.channel_axis == 1); /* NCHW only in this core */
    ART_CHECK(group > 0 && sh > 0 && sw > 0);
    ART_CHECK(x->shape.dim[1] % group == 0 && K % group == 0);
    ART_CHECK(w->shape.dim[0] == K && w->shape.dim[1] == x->shape.dim[1] / group);
    if (op->input_size == 3)
        ART_CHECK(op->input_tensors[2]->shape.dim_size == 1 && op->input_tensors[2]->shape.dim[0] == K);
    const uint32_t keh = kh + (kh - 1) * (dh - 1), kew = kw + (kw - 1) * (dw - 1);
    tensor_t *y = single_output(op, false);
    y->shape = x->shape;
    y->shape.dim[1] = K;
    y->shape.dim[2] = (x->shape.dim[2] + 2 * ph - keh) / sh + 1; /* unsigned, as in the reference */
    y->shape.dim[3] = (x->shape.dim[3] + 2 * pw - kew) / sw + 1;
    return true;
}

/* ---- ip (op.c:799-870): flatten from `axis`, output [.., num_output] with dim_size = axis + 1 ------------ */
static bool infer_ip(op_t *op)
{
    ART_CHECK(op->input_size == 2 || op->input_size == 3);
    const tensor_t *x = op->input_tensors[0], *w = op->input_tensors[1];
    const uint32_t K = get_u32(op, SETTING_IP_NUM_OUTPUT);
    int32_t axis = 1;
    ART_CHECK(op_setting_single_get(op, SETTING_IP_AXIS, dtINT32, &axis));
    const int nd = x->shape.dim_size;
    if (axis < 0)
        axis += nd;
    ART_CHECK(axis >= 0 && axis < nd);
    size_t inner = 1;
    for (int i = axis; i < nd; ++i)
        inner *= x->shape.dim[i];
    ART_CHECK(w->shape.dim[w->shape.batch_axis] == K);
    ART_CHECK(shape_count(&w->shape) / K == inner);
    tensor_t *y = single_output(op, false);
    y->shape = x->shape;
    y->shape.dim_size = axis + 1;
    y->shape.channel_axis = axis;
    y->shape.dim[axis] = K;
    for (int i = axis + 1; i < MAX_DIM; ++i)
        y->shape.dim[i] = 1;
    return true;
}

/* ---- pool (op.c:903-967) --------------------------------------------------------------------------------- */
static bool infer_pool(op_t *op)
{
    ART_CHECK(op->input_size == 1);
    const tensor_t *x = op->input_tensors[0];
    ART_CHECK(x->shape.dim_size == 4 && x->shape.batch_axis == 0 && x->shape.channel_axis == 1);
    const uint32_t kh = get_u32(op, SETTING_POOL_KERNEL_H), kw = get_u32(op, SETTING_POOL_KERNEL_W);
    const uint32_t ph = get_u32(op, SETTING_POOL_PAD_H), pw = get_u32(op, SETTING_POOL_PAD_W);
    const uint32_t sh = get_u32(op, SETTING_POOL_STRIDE_H), sw = get_u32(op, SETTING_POOL_STRIDE_W);
    bool ceil_mode = true;
    ART_CHECK(op_setting_single_get(op, SETTING_POOL_CEIL_MODE, dtBOOL, &ceil_mode));
    const uint32_t H = x->shape.dim[2], W = x->shape.dim[3];
    const double vh = (H + ph * 2.0 - kh) / sh + 1, vw = (W + pw * 2.0 - kw) / sw + 1;
    uint32_t oh = (uint32_t)(ceil_mode ? ceil(vh) : floor(vh)), ow = (uint32_t)(ceil_mode ? ceil(vw) : floor(vw));
    if (ph || pw) { /* the last window must start inside the (left-)padded image */
        if ((oh - 1) * sh >= H + ph)
            --oh;
        if ((ow - 1) * sw >= W + pw)
            --ow;
    }
    tensor_t *y = single_output(op, false);
    y->shape = x->shape;
    y->shape.dim[2] = oh;
    y->shape.dim[3] = ow;
    return true;
}

/* ---- relu and other unary ops (op.c:279-294) ------------------------------------------------------------------ */
static bool infer_unary(op_t *op)
{
    ART_CHECK(op->input_size == 1 && op->input_tensors[0]->shape.dim_size >= 1);
    single_output(op, false)->shape = op->input_tensors[0]->shape;
    return true;
}

/* ---- add: numpy-style broadcast of two inputs (op.c:296-346) ------------------------------------------------- */
static bool infer_binary(op_t *op)
{
    ART_CHECK(op->input_size == 2);
    const shape_t *a = &op->input_tensors[0]->shape, *b = &op->input_tensors[1]->shape;
    ART_CHECK(op->input_tensors[0]->dtype == op->input_tensors[1]->dtype && a->dim_size >= 1);
    const int nd = a->dim_size > b->dim_size ? a->dim_size : b->dim_size;
    tensor_t *y = single_output(op, false);
    y->shape = *a;
    y->shape.dim_size = nd;
    for (int i = 0; i < nd; ++i) { /* align trailing dimensions */
        const int ia = a->dim_size - 1 - i, ib = b->dim_size - 1 - i;
        const uint32_t da = ia >= 0 ? a->dim[ia] : 1, db = ib >= 0 ? b->dim[ib] : 1;
        if (da != db && da != 1 && db != 1)
            ART_FATAL("cannot broadcast dim %d: %u vs %u\n", nd - 1 - i, da, db);
        y->shape.dim[nd - 1 - i] = da == 1 ? db : da;
    }
    return true;
}

/* ---- eltwise (op.c:1075-1088) ------------------------------------------------------------------------------------ */
static bool infer_eltwise(op_t *op)
{
    ART_CHECK(op->input_size >= 2);
    single_output(op, false)->shape = op->input_tensors[0]->shape;
    return true;
}

/* ---- reshape (op.c:1090-1160): zero-copy, the output shares the input's memory ---------------------------- */
static bool infer_reshape(op_t *op)
{
    ART_CHECK(op->input_size == 1);
    const tensor_t *x = op->input_tensors[0];
    int32_t axis = 0, *dims = NULL;
    size_t n = 0;
    ART_CHECK(op_setting_single_get(op, SETTING_RESHAPE_AXIS, dtINT32, &axis));
    ART_CHECK(op_setting_array_get(op, SETTING_RESHAPE_DIMS, dtINT32, &n, &dims));
    if (axis < 0)
        axis += x->shape.dim_size;
    ART_CHECK(axis >= 0 && axis <= x->shape.dim_size && axis + (int)n <= MAX_DIM);
    /* dimensions before `axis` are kept; `dims` replaces everything from `axis` on (0 = keep, -1 = infer) */
    int full[MAX_DIM];
    for (int i = 0; i < axis; ++i)
        full[i] = 0;
    for (size_t i = 0; i < n; ++i)
        full[axis + i] = dims[i];
    tensor_t *y = single_output(op, true);
    y->shape = x->shape;
    return tensor_reshape(y, axis + (int)n, full);
}

/* ---- concat (op.c:872-901): all dims equal except `axis`, which adds up ---------------------------------------- */
static bool infer_concat(op_t *op)
{
    const uint32_t axis = get_u32(op, SETTING_CONCAT_AXIS);
    ART_CHECK(op->input_size >= 2);
    const tensor_t *x0 = op->input_tensors[0];
    ART_CHECK((int)axis < x0->shape.dim_size);
    uint32_t total = x0->shape.dim[axis];
    for (size_t i = 1; i < op->input_size; ++i) {
        const tensor_t *xi = op->input_tensors[i];
        ART_CHECK(xi->shape.dim_size == x0->shape.dim_size && xi->dtype == x0->dtype);
        for (int j = 0; j < x0->shape.dim_size; ++j)
            ART_CHECK(j == (int)axis || xi->shape.dim[j] == x0->shape.dim[j]);
        total += xi->shape.dim[axis];
    }
    tensor_t *y = single_output(op, false);
    y->shape = x0->shape;
    y->shape.dim[axis] = total;
    return true;
}

/* ---- the op-type objects ------------------------------------------------------------------------------------------- */
#define C_REQ(i, t) {.item = i, .dtype = t, .ctp = ENUM_SETTING_CONSTRAINT_REQUIRED, .name = #i}
#define C_OPT(i, t, member, dft) \
    {.item = i, .dtype = t, .ctp = ENUM_SETTING_CONSTRAINT_OPTIONAL, .constraint.optional.default_value.member = dft, .name = #i}
#define C_REP(i, t) {.item = i, .dtype = t, .ctp = ENUM_SETTING_CONSTRAINT_REPEATED, .name = #i}
#define C_END() {.item = SETTING_END, .dtype = dtUNKNOWN, .ctp = ENUM_SETTING_CONSTRAINT_OPTIONAL, .name = NULL}

ART_PUBLIC const op_tp_t op_conv_2d_tp = { /* op.c:2328-2358 */
    .op_tp_code = OP_CONV_2D, .name = "conv_2d", .min_input_size = 2, .max_input_size = 3,
    .min_output_size = 1, .max_output_size = 1, .infer_output_func = infer_conv_2d,
    .constraints = {C_REQ(SETTING_CONV_2D_NUM_OUTPUT, dtUINT32), C_REQ(SETTING_CONV_2D_KERNEL_H, dtUINT32),
                    C_REQ(SETTING_CONV_2D_KERNEL_W, dtUINT32), C_OPT(SETTING_CONV_2D_PAD_H, dtUINT32, u32, 0),
                    C_OPT(SETTING_CONV_2D_PAD_W, dtUINT32, u32, 0), C_OPT(SETTING_CONV_2D_STRIDE_H, dtUINT32, u32, 1),
                    C_OPT(SETTING_CONV_2D_STRIDE_W, dtUINT32, u32, 1), C_OPT(SETTING_CONV_2D_HOLE_H, dtUINT32, u32, 1),
                    C_OPT(SETTING_CONV_2D_HOLE_W, dtUINT32, u32, 1), C_OPT(SETTING_CONV_2D_GROUP, dtUINT32, u32, 1),
                    C_OPT(SETTING_CONV_2D_RELU_FLAG, dtBOOL, b, false), C_END()}};

ART_PUBLIC const op_tp_t op_ip_tp = { /* op.c:2600-2612 */
    .op_tp_code = OP_IP, .name = "ip", .min_input_size = 2, .max_input_size = 3, .min_output_size = 1,
    .max_output_size = 1, .infer_output_func = infer_ip,
    .constraints = {C_REQ(SETTING_IP_NUM_OUTPUT, dtUINT32), C_OPT(SETTING_IP_RELU_FLAG, dtBOOL, b, false),
                    C_OPT(SETTING_IP_AXIS, dtINT32, i32, 1), C_END()}};

ART_PUBLIC const op_tp_t op_pool_tp = { /* op.c:2626-2645: ceil_mode defaults to true */
    .op_tp_code = OP_POOL, .name = "pool", .min_input_size = 1, .max_input_size = 1, .min_output_size = 1,
    .max_output_size = 1, .infer_output_func = infer_pool,
    .constraints = {C_REQ(SETTING_POOL_KERNEL_H, dtUINT32), C_REQ(SETTING_POOL_KERNEL_W, dtUINT32),
                    C_OPT(SETTING_POOL_METHOD, dtUINT32, u32, SETTING_POOL_MAX), C_OPT(SETTING_POOL_PAD_H, dtUINT32, u32, 0),
                    C_OPT(SETTING_POOL_PAD_W, dtUINT32, u32, 0), C_OPT(SETTING_POOL_STRIDE_H, dtUINT32, u32, 1),
                    C_OPT(SETTING_POOL_STRIDE_W, dtUINT32, u32, 1), C_OPT(SETTING_POOL_CEIL_MODE, dtBOOL, b, true), C_END()}};

ART_PUBLIC const op_tp_t op_relu_tp = { /* op.c:2479-2486 */
    .op_tp_code = OP_RELU, .name = "relu", .min_input_size = 1, .max_input_size = 1, .min_output_size = 1,
    .max_output_size = 1, .infer_output_func = infer_unary, .constraints = {C_END()}};

ART_PUBLIC const op_tp_t op_add_tp = { /* op.c:2252-2259 */
    .op_tp_code = OP_ADD, .name = "add", .min_input_size = 2, .max_input_size = 2, .min_output_size = 1,
    .max_output_size = 1, .infer_output_func = infer_binary, .constraints = {C_END()}};

ART_PUBLIC const op_tp_t op_eltwise_tp = { /* op.c:2562-2574 */
    .op_tp_code = OP_ELTWISE, .name = "eltwise", .min_input_size = 2, .max_input_size = 0xffff, .min_output_size = 1,
    .max_output_size = 1, .infer_output_func = infer_eltwise,
    .constraints = {C_OPT(SETTING_ELTWISE_OPERATION, dtUINT32, u32, SETTING_ELTWISE_OP_SUM),
                    C_REP(SETTING_ELTWISE_COEFF, dtFLOAT32), C_END()}};

ART_PUBLIC const op_tp_t op_reshape_tp = { /* op.c:2691-2703 */
    .op_tp_code = OP_RESHAPE, .name = "reshape", .min_input_size = 1, .max_input_size = 1, .min_output_size = 1,
    .max_output_size = 1, .infer_output_func = infer_reshape,
    .constraints = {C_REP(SETTING_RESHAPE_DIMS, dtINT32), C_OPT(SETTING_RESHAPE_AXIS, dtINT32, i32, 0),
                    C_OPT(SETTING_RESHAPE_NUM_AXES, dtINT32, i32, -1), C_END()}};

ART_PUBLIC const op_tp_t op_concat_tp = { /* op.c:2614-2624 */
    .op_tp_code = OP_CONCAT, .name = "concat", .min_input_size = 2, .max_input_size = 0xffff, .min_output_size = 1,
    .max_output_size = 1, .infer_output_func = infer_concat, .constraints = {C_REQ(SETTING_CONCAT_AXIS, dtUINT32), C_END()}};

ART_PUBLIC const op_tp_t op_softmax_tp = { /* op.c:2544-2560 */
    .op_tp_code = OP_SOFTMAX, .name = "softmax", .min_input_size = 1, .max_input_size = 1, .min_output_size = 1,
    .max_output_size = 1, .infer_output_func = infer_unary, .constraints = {C_OPT(SETTING_SOFTMAX_AXIS, dtUINT32, u32, 1), C_END()}};
