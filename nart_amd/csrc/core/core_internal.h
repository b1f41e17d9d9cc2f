/* Private to the host core: the parade's own storage (the reference keeps the same in parade_impl.h:23-32). */
#ifndef NART_HIP_CORE_INTERNAL_H
#define NART_HIP_CORE_INTERNAL_H

#include "art/art.h"

struct _parade_t {
    size_t op_count;
    op_t **ops;
    size_t input_tensor_count;
    tensor_t **input_tensors;
    size_t weight_tensor_count;
    tensor_t **weight_tensors;
    size_t output_tensor_count;
    tensor_t **output_tensors;
};

void parade_push_op(parade_t *p, op_t *op);

#endif
