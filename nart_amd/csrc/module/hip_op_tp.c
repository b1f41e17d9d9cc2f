/*
 * Op-type objects of the two module-private operators, quantize (fp32 -> uint8) and dequantize
 * (uint8 -> fp32).  They carry the quant group's private codes 0x0006_8000_0000 / _0001, which is what the
 * unchanged quant converter writes into an engine file, and the same setting constraints as the reference's
 * (art/modules/quant/src/op/quantize.c:40-102, dequantize.c:30-60).  Plain C because of the designated
 * initialisers on a flexible array member.
 */
#include <string.h>

#ifdef NART_HIP_USE_NART_HEADERS
#include "art/op.h"
#include "art/op_tp.h"
#include "art/quant/quant_op_settings.h"
#include "art/quant/quant_op_tp.h"
#define ART_PUBLIC __attribute__((visibility("default")))
#define ART_CHECK(c) CHECK(c)
#else
#include "art/art.h"
#endif

static tensor_t *one_output(op_t *op, uint32_t dtype)
{
    ART_CHECK(op->input_size == 1 && op->output_size <= 1);
    ART_CHECK(op->input_tensors[0]->shape.dim_size >= 1);
    if (op->output_size == 0) {
        op->output_size = 1;
        op->output_tensors = (tensor_t *)calloc(1, sizeof(tensor_t));
        op->output_tensors[0].mem = mem_new(op->input_tensors[0]->mem->tp);
        op->output_tensors[0].dtype = dtype;
    }
    op->output_tensors[0].shape = op->input_tensors[0]->shape;
    return &op->output_tensors[0];
}

/* quantize.c:40-86 maps (qtype << 8 | bits) to an output dtype; this module implements the uint8 and int8 rows
 * (prepare rejects the others).  The qtype setting sits right after op_t in the module's quantize struct. */
static bool infer_quantize(op_t *op)
{
    int32_t qtype = 0;
    uint8_t *bits = NULL;
    size_t n = 0;
    uint32_t dt = dtUINT8;
    if (op_setting_single_get(op, SETTING_QUANT_QTYPE, dtINT32, &qtype)
        && op_setting_array_get(op, SETTING_QUANT_OBITS, dtUINT8, &n, &bits) && n >= 1) {
        const int32_t key = qtype << 8 | bits[0];
        if (key >= 0x0202 && key <= 0x0208 && key != 0x0205)
            dt = dtINT8;
    }
    if (op->output_size == 1)
        op->output_tensors[0].dtype = dt; /* settings may have changed since the first inference */
    one_output(op, dt);
    return true;
}

static bool infer_dequantize(op_t *op)
{
    one_output(op, dtFLOAT32);
    return true;
}

#define C_OPT_I32(i, dft) \
    {.item = i, .dtype = dtINT32, .ctp = ENUM_SETTING_CONSTRAINT_OPTIONAL, .constraint.optional.default_value.i32 = dft, .name = #i}
#define C_REP(i, t) {.item = i, .dtype = t, .ctp = ENUM_SETTING_CONSTRAINT_REPEATED, .name = #i}
#define C_END() {.item = SETTING_END, .dtype = dtUNKNOWN, .ctp = ENUM_SETTING_CONSTRAINT_OPTIONAL, .name = NULL}

ART_PUBLIC const op_tp_t op_hip_quantize_tp = {
    .op_tp_code = OP_QUANT_QUANTIZE, .name = "quantize", .min_input_size = 1, .max_input_size = 1,
    .min_output_size = 1, .max_output_size = 1, .infer_output_func = infer_quantize,
    .constraints = {C_REP(SETTING_QUANT_OALPHA, dtFLOAT32), C_REP(SETTING_QUANT_OZERO_POINT, dtUINT8),
                    C_REP(SETTING_QUANT_OBITS, dtUINT8), C_OPT_I32(SETTING_QUANT_QTYPE, 0), C_END()}};

ART_PUBLIC const op_tp_t op_hip_dequantize_tp = {
    .op_tp_code = OP_QUANT_DEQUANTIZE, .name = "dequantize", .min_input_size = 1, .max_input_size = 1,
    .min_output_size = 1, .max_output_size = 1, .infer_output_func = infer_dequantize,
    .constraints = {C_REP(SETTING_QUANT_IALPHA, dtFLOAT32), C_REP(SETTING_QUANT_IZERO_POINT, dtUINT8),
                    C_REP(SETTING_QUANT_IBITS, dtUINT8), C_OPT_I32(SETTING_QUANT_QTYPE, 0), C_END()}};
