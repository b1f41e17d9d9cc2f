// Internal declarations of the `hip` case module (libart_module_hip.so).
//
// The module plugs into NART's art runtime exactly like art/modules/quant does: it exports one
// `module_t hip_module_tp` (op group 6, the quant group) whose table lists the quantized operators, each
// with alloc/config/destroy/dealloc/prepare entry points; `prepare` picks the run function, which launches
// hand-written HIP kernels through the hipq C ABI (include/hipq.h).
#pragma once

#ifdef NART_HIP_USE_NART_HEADERS
// built inside a NART source tree: use the runtime's own headers
extern "C" {
#include "art/module.h"
#include "art/op.h"
#include "art/op_settings.h"
#include "art/op_tp.h"
#include "art/quant/quant_op_settings.h"
#include "art/quant/quant_op_tp.h"
// the shared op types of the generic ops live in libart (art/src/op.c:2252-2703)
extern const op_tp_t op_conv_2d_tp, op_ip_tp, op_pool_tp, op_relu_tp, op_add_tp, op_eltwise_tp, op_reshape_tp;
extern const op_tp_t op_concat_tp, op_softmax_tp;
}
#define ART_PUBLIC __attribute__((visibility("default")))
#else
#include "art/art.h"
#endif

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "hipq.h"

// errors follow the runtime's convention (art/include/art/log.h:82-101): report and abort
#define HIPM_CHECK(cond)                                                                        \
    do {                                                                                        \
        if (!(cond)) {                                                                          \
            fprintf(stderr, "[hip module] check failed: %s (%s:%d)\n", #cond, __FILE__, __LINE__); \
            abort();                                                                            \
        }                                                                                       \
    } while (0)
#define HIPM_HIP(expr)                                                                                       \
    do {                                                                                                     \
        hipError_t e_ = (expr);                                                                              \
        if (e_ != hipSuccess) {                                                                              \
            fprintf(stderr, "[hip module] %s: %s (%s:%d)\n", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
            abort();                                                                                         \
        }                                                                                                    \
    } while (0)
#define HIPM_HIPQ(expr)                                                                             \
    do {                                                                                            \
        if ((expr) != 0) {                                                                          \
            fprintf(stderr, "[hip module] %s: %s (%s:%d)\n", #expr, hipq_last_error(), __FILE__, __LINE__); \
            abort();                                                                                \
        }                                                                                           \
    } while (0)

struct hip_workspace_t {
    workspace_t ws; // must be first (art/include/art/workspace.h:27-29)
    char name[32];
    int dev_id;
    hipStream_t stream; // every kernel of this workspace is launched here
    bool own_stream;
};

// ---- device memory with a host mirror -------------------------------------------------------------------
// The runtime and the runners read and write tensors only through mem_cpu_data(), always in the reference's
// dense NCHW order.  On the device, 4-D uint8 activations live channels-last with a padded channel stride
// (include/hipq.h); the conversion happens on the device at the moment a side that is out of date is asked
// for (precedent: art/modules/cuda_quant/src/cuda_quant_mem.cpp:25-92).
enum hip_layout_t { HIP_LAYOUT_RAW = 0, HIP_LAYOUT_NHWC_U8 = 1 };

struct hip_mem_t {
    mem_t m;            // must be first (art/include/art/mem.h:66-69)
    size_t size;        // logical size in bytes (dense NCHW), as requested through mem_alloc
    void *host;         // pinned host mirror, allocated on first mem_cpu_data()
    size_t host_cap;
    void *dev;          // device buffer in `layout`
    size_t dev_cap;
    void *stage;        // device scratch for the dense side of a layout conversion
    size_t stage_cap;
    hip_layout_t layout;
    int N, C, H, W, cs; // geometry for HIP_LAYOUT_NHWC_U8
    bool host_valid, dev_valid;
    // An upload reads the pinned mirror asynchronously on `up_stream`: the mirror may only be handed out for writing
    // once that copy has finished.
    bool up_pending;
    hipStream_t up_stream;
    // The stream whose work last wrote `dev` (a workspace's, or the null stream for an upload on behalf of foreign code):
    // a reader outside that stream waits for it, and for nothing else.
    hipStream_t prod_stream;
    // Deferred producer.  A convolution whose only reader is an add does not launch at its own run(): it leaves this
    // hook, and the add runs both as one fused kernel (hip_ops.cpp).  Whoever else asks for the contents first - the
    // host, another workspace, a re-run - makes the hook launch the plain convolution into `dev` (hip_mem_settle).
    void (*pending)(void *ctx);
    void *pending_ctx;
};

// make the device contents current: run the deferred producer, if any
static inline void hip_mem_settle(hip_mem_t *m)
{
    if (m->pending) {
        void (*f)(void *) = m->pending;
        m->pending = nullptr;
        f(m->pending_ctx);
    }
}

extern const mem_tp hip_mem_tp_st;

// Tag the device layout of a tensor's memory from its shape and dtype (4-D and 2-D uint8 -> NHWC).
// An existing tag with the same element count is kept: a reshape()d view shares its producer's geometry.
void hip_mem_tag(tensor_t *t);
// Device pointer for reading (uploads / converts the host mirror if that is the newer side).
// the streams hip_mem_tp may wait on by name: a workspace registers the stream it launches on, retires the one it owns
// (synchronise, then forget) before destroying it and forgets a caller's stream when it stops using it
void hip_stream_register(hipStream_t st);
void hip_stream_retire(hipStream_t st);
void hip_stream_forget(hipStream_t st);
const void *hip_mem_dev_in(mem_t *m, hipStream_t st);
// Device pointer for writing: the device side becomes the valid one.
void *hip_mem_dev_out(mem_t *m, hipStream_t st);
// Host pointer with current contents (downloads / converts if the device is the newer side); read-only use.
const void *hip_mem_host_in(mem_t *m);
static inline hip_mem_t *as_hip(mem_t *m) { return reinterpret_cast<hip_mem_t *>(m); }
static inline bool is_hip_mem(const mem_t *m) { return m->tp == &hip_mem_tp_st; }

static inline hipStream_t op_stream(const op_t *op) { return reinterpret_cast<hip_workspace_t *>(op->workspace)->stream; }

extern "C" {
extern const op_tp_t op_hip_quantize_tp, op_hip_dequantize_tp;
extern op_tp_entry_t hip_op_table[];
}
