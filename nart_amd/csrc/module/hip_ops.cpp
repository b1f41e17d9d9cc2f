// The `hip` case module: workspace, op table and the operators' alloc/config/destroy/dealloc/prepare/run.
//
// Each operator mirrors its counterpart in the reference CPU quant module (art/modules/quant/src/op/*.c):
// the same settings are read in `config` (missing required ones abort, as there), `prepare` allocates the
// tensors, derives everything that does not depend on the activations (for conv/ip: the packed weights and
// folded per-channel constants, which the reference recomputes on every run) and selects the run function;
// `run` only launches kernels on the workspace stream.
#include <cstring>
#include <map>
#include <new>
#include <set>
#include <vector>

#include "hip_module.h"

namespace {

// ---- the quantisation settings every op reads (e.g. conv_2d.c:42-69) ----------------------------------------
struct QSet {
    float *alpha = nullptr;
    uint8_t *zp = nullptr;
    uint8_t *bits = nullptr;
    size_t n = 0;
    size_t n_alpha = 0; // length of the alpha array alone (a weight scale per output channel has K entries)
};

void read_qset(op_t *op, uint32_t ia, uint32_t iz, uint32_t ib, QSet *q)
{
    size_t n1 = 0, n2 = 0, n3 = 0;
    HIPM_CHECK(op_setting_array_get(op, ia, dtFLOAT32, &n1, &q->alpha));
    HIPM_CHECK(op_setting_array_get(op, iz, dtUINT8, &n2, &q->zp));
    HIPM_CHECK(op_setting_array_get(op, ib, dtUINT8, &n3, &q->bits));
    HIPM_CHECK(q->alpha && q->zp && q->bits && n1 >= 1 && n2 >= 1 && n3 >= 1);
    q->n = n1 < n2 ? n1 : n2;
    q->n_alpha = n1;
}
#define READ_I(op, q) read_qset(op, SETTING_QUANT_IALPHA, SETTING_QUANT_IZERO_POINT, SETTING_QUANT_IBITS, q)
#define READ_W(op, q) read_qset(op, SETTING_QUANT_WALPHA, SETTING_QUANT_WZERO_POINT, SETTING_QUANT_WBITS, q)
#define READ_O(op, q) read_qset(op, SETTING_QUANT_OALPHA, SETTING_QUANT_OZERO_POINT, SETTING_QUANT_OBITS, q)

// The device geometry of a tensor's memory is its producer's (a reshape that keeps the element count does not move
// bytes, hip_mem_tag).  An operator that takes N/C/H/W from the tensor's SHAPE but strides from the memory must see
// the two agree: a reshape that regroups channels and pixels (channel shuffle, space-to-depth) in front of it would
// otherwise compute on the wrong layout; like every unsupported case, it aborts.
void same_shape_and_geometry(const op_t *op, const tensor_t *t)
{
    const hip_mem_t *m = as_hip(t->mem);
    const shape_t &s = t->shape;
    const bool ok = m->layout == HIP_LAYOUT_NHWC_U8 && s.dim_size == 4 && m->N == (int)s.dim[0] && m->C == (int)s.dim[1]
        && m->H == (int)s.dim[2] && m->W == (int)s.dim[3];
    if (!ok) {
        fprintf(stderr, "[hip module] %s: tensor %s has shape [%u, %u, %u, %u] but its memory holds [%d, %d, %d, %d]: a "
                        "reshape that regroups channels and pixels in front of this operator is not implemented\n",
                op->entry->tp->name, t->name ? t->name : "?", s.dim[0], s.dim[1], s.dim[2], s.dim[3], m->N, m->C, m->H, m->W);
        abort();
    }
}

void alloc_and_tag(op_t *op)
{
    for (size_t i = 0; i < op->input_size; ++i) {
        tensor_alloc(op->input_tensors[i]);
    }
    for (size_t i = 0; i < op->output_size; ++i) {
        tensor_alloc(&op->output_tensors[i]);
        hip_mem_tag(&op->output_tensors[i]);
    }
}

void forget_reader(op_t *op);

template <class T>
op_t *alloc_op(workspace_t *)
{
    T *p = static_cast<T *>(calloc(1, sizeof(T)));
    return reinterpret_cast<op_t *>(p);
}

void dealloc_op(op_t *op)
{
    // forget what the operator read (the registry of the convolution + add fusion, below)
    forget_reader(op);
    free(op);
}
void destroy_nothing(op_t *) {}

const void *in_ptr(op_t *op, int i) { return hip_mem_dev_in(op->input_tensors[i]->mem, op_stream(op)); }
void *out_ptr(op_t *op) { return hip_mem_dev_out(op->output_tensors[0].mem, op_stream(op)); }

// Which operators of this workspace read which memory, collected as the operators are prepared (every prepare of the
// pass has run before the first run()).  A convolution asks it whether an add is the ONLY reader of its output.
typedef std::map<const mem_t *, std::set<const op_t *>> reader_map;

// keyed by workspace (the runtime is single-threaded, art/include/art/workspace.h has no locking either)
std::map<const workspace_t *, reader_map> g_readers;
long g_fused_adds = 0, g_fused_relus = 0, g_fused_pools = 0, g_chained_convs = 0, g_fused_dequants = 0; // fused launches so far (hip_module_fused_*)
long g_fused_blocks = 0, g_fused_tails = 0; // whole bottleneck blocks / blocks from their 3x3 layer on, as one launch

reader_map &readers_of(op_t *op) { return g_readers[op->workspace]; }

void forget_reader(op_t *op)
{
    const auto it = g_readers.find(op->workspace);
    if (it != g_readers.end())
        for (auto &kv : it->second)
            kv.second.erase(op);
}

// allow_i8: conv_2d, ip and dequantize also exist for int8 symmetric tensors (conv_2d.c:120-141, ip.cpp:312-331,
// dequantize.c:156-163); every other operator of the reference module is uint8 only.
void require_hip_u8(op_t *op, size_t n_act, bool allow_i8 = false)
{
    for (size_t i = 0; i < n_act; ++i) {
        const uint32_t dt = op->input_tensors[i]->dtype;
        if (dt != dtUINT8 && !(allow_i8 && dt == dtINT8)) {
            fprintf(stderr, "[hip module] %s: input %zu has dtype %u; this operator is implemented for uint8%s activations\n",
                    op->entry->tp->name, i, dt, allow_i8 ? " and int8" : "");
            abort(); // the reference aborts on unsupported dtypes as well (conv_2d.c:143-145)
        }
        HIPM_CHECK(is_hip_mem(op->input_tensors[i]->mem));
        hip_mem_tag(op->input_tensors[i]);
        readers_of(op)[op->input_tensors[i]->mem].insert(op);
    }
}

// ---- conv_2d and ip share one structure: both run a hipq convolution plan -------------------------------------
struct conv_op_t {
    op_t o;
    uint32_t num_output, pad_h, pad_w, kernel_h, kernel_w, stride_h, stride_w, group;
    QSet qi, qw, qo;
    hipq_conv2d_plan *plan;
    hipq_conv2d_desc desc; // what the plan was built for (re-used when prepare is called again unchanged)
    const void *w_seen;    // identity of the weights the plan was packed from
    uint64_t pc_seen;      // checksum of the per-channel weight scales the plan was built with (0: per tensor)
    int defer;             // 0 undecided, 1 leave the launch to the add / relu that reads the output, -1 launch at run()
    // A convolution that heads a bottleneck block (1x1, then 3x3, then 1x1 and the add with the block's input) which
    // hipq_bottleneck_run computes in one launch: the block's 3x3 convolution and its add (else null).
    const op_t *blk_next, *blk_add;
    // this pass's output has already been written by the kernel of the pooling operator whose output this convolution
    // reads (hipq_conv2d_run_maxpool_conv): run() has nothing left to do
    bool computed_ahead;
};

void conv_config(op_t *op)
{
    conv_op_t *c = reinterpret_cast<conv_op_t *>(op);
    HIPM_CHECK(op_setting_single_get(op, SETTING_CONV_2D_NUM_OUTPUT, dtUINT32, &c->num_output));
    HIPM_CHECK(op_setting_single_get(op, SETTING_CONV_2D_KERNEL_H, dtUINT32, &c->kernel_h));
    HIPM_CHECK(op_setting_single_get(op, SETTING_CONV_2D_KERNEL_W, dtUINT32, &c->kernel_w));
    HIPM_CHECK(op_setting_single_get(op, SETTING_CONV_2D_PAD_H, dtUINT32, &c->pad_h));
    HIPM_CHECK(op_setting_single_get(op, SETTING_CONV_2D_PAD_W, dtUINT32, &c->pad_w));
    HIPM_CHECK(op_setting_single_get(op, SETTING_CONV_2D_STRIDE_H, dtUINT32, &c->stride_h));
    HIPM_CHECK(op_setting_single_get(op, SETTING_CONV_2D_STRIDE_W, dtUINT32, &c->stride_w));
    HIPM_CHECK(op_setting_single_get(op, SETTING_CONV_2D_GROUP, dtUINT32, &c->group));
    READ_I(op, &c->qi);
    READ_W(op, &c->qw);
    READ_O(op, &c->qo);
}

void ip_config(op_t *op)
{
    conv_op_t *c = reinterpret_cast<conv_op_t *>(op);
    HIPM_CHECK(op_setting_single_get(op, SETTING_IP_NUM_OUTPUT, dtUINT32, &c->num_output));
    READ_I(op, &c->qi);
    READ_W(op, &c->qw);
    READ_O(op, &c->qo);
}

void conv_destroy(op_t *op)
{
    conv_op_t *c = reinterpret_cast<conv_op_t *>(op);
    // a launch left to an add (conv_run) must not outlive the plan: the output's memory may, as a view's
    if (op->output_size > 0 && op->output_tensors != nullptr && op->output_tensors[0].mem != nullptr
        && is_hip_mem(op->output_tensors[0].mem) && as_hip(op->output_tensors[0].mem)->pending_ctx == op)
        as_hip(op->output_tensors[0].mem)->pending = nullptr;
    hipq_conv2d_plan_destroy(c->plan);
    c->plan = nullptr;
}

// ---- convolution + add / relu fusion -----------------------------------------------------------------------------
// In a residual network the expanding convolution's output is read by the add and by nothing else; where the converter
// emits ReLU as an operator of its own (the CPU module ignores the convolution's relu flag, conv_2d.c:27-70), the
// convolution's output is read by that relu and by nothing else.  Such a convolution does not launch at its own run():
// it leaves a hook on its output memory, and the reader's run() launches hipq_conv2d_run_add / hipq_conv2d_run_relu - the
// convolution with the add / the clamp in its epilogue, bit-identical to the two operators - so the convolution's
// output is never written or read.  Anything else that asks for that memory (the host through
// mem_cpu_data, a foreign workspace through mem_data) settles the hook first, which launches the plain convolution.
void conv_launch_plain(void *ctx)
{
    op_t *op = static_cast<op_t *>(ctx);
    conv_op_t *c = reinterpret_cast<conv_op_t *>(op);
    hip_mem_t *ym = as_hip(op->output_tensors[0].mem);
    HIPM_HIPQ(hipq_conv2d_run(c->plan, in_ptr(op, 0), ym->dev, nullptr, op_stream(op)));
}

bool eltwise_is_plain_sum(const op_t *op); // two inputs, SUM, unit coefficients: computes what add computes
struct QSet;
const QSet &add_inputs(const op_t *add_op);  // the input / output quantisation settings of an add or eltwise operator
const QSet &add_output(const op_t *add_op);
bool conv_heads_block(op_t *op, const op_t *r);
bool conv_continues_block(op_t *op, const op_t *r);
// a dequantize that the fully-connected layer's kernel can compute in its epilogue (hipq_conv2d_dequant_fusable)
bool dequantize_fuses_with(const op_t *deq_op, const hipq_conv2d_plan *plan);
// a max pooling that the stem convolution's kernel can compute as well (hipq_conv2d_maxpool_fusable)
bool pool_fuses_with(const op_t *pool_op, const hipq_conv2d_plan *plan);
// the convolution `op` as the tail of the kernel that computes the add it reads (hipq_conv2d_run_add_conv); y: where its
// output goes, relu: with the ReLU clamp.  false: not possible, run it plainly
bool conv_run_chained(op_t *op, void *y, int relu);

// ---- whole bottleneck blocks ---------------------------------------------------------------------------------------
// 1x1 -> 3x3 -> 1x1 -> add(., block input), every intermediate tensor read by its successor only: the 1x1 head and the
// 3x3 leave hooks like the widening convolution does, and the add's run() launches hipq_bottleneck_run (all three
// convolutions and the add) or, where only that form applies, hipq_bottleneck_tail_run (from the 3x3 on, with any
// residual; the 1x1 convolution that reads the sum may ride along, conv_run_chained).  Hooks settle in a chain: asking
// for the 3x3's output runs the head first.
const op_t *only_reader(const op_t *op)
{
    const auto wit = g_readers.find(op->workspace);
    if (wit == g_readers.end())
        return nullptr;
    const auto it = wit->second.find(op->output_tensors[0].mem);
    if (it == wit->second.end() || it->second.size() != 1 || (*it->second.begin())->workspace != op->workspace)
        return nullptr;
    return *it->second.begin();
}

// the add (or plain two-input SUM) that is the only reader of convolution r's output and reads it with the scale it is
// written with; *idx: which of its inputs that is
const op_t *add_reading(const op_t *r, int *idx)
{
    const op_t *a = only_reader(r);
    if (a == nullptr || !(a->entry->tp == &op_add_tp || eltwise_is_plain_sum(a)) || a->input_size != 2
        || a->input_tensors[0]->mem == a->input_tensors[1]->mem)
        return nullptr;
    const int i = a->input_tensors[0]->mem == r->output_tensors[0].mem ? 0 : 1;
    const conv_op_t *c = reinterpret_cast<const conv_op_t *>(r);
    const QSet &qi = add_inputs(a);
    if (qi.alpha[i] != c->desc.oalpha || qi.zp[i] != c->desc.ozp)
        return nullptr;
    *idx = i;
    return a;
}

// op: a 1x1 convolution, r (its only reader): a 3x3 convolution, then a 1x1 convolution, then the add with op's input
bool conv_heads_block(op_t *op, const op_t *r)
{
    conv_op_t *c1 = reinterpret_cast<conv_op_t *>(op);
    c1->blk_next = c1->blk_add = nullptr;
    const op_t *r2 = only_reader(r);
    if (r2 == nullptr || r2->entry->tp != &op_conv_2d_tp)
        return false;
    int i = 0;
    const op_t *a = add_reading(r2, &i);
    if (a == nullptr || a->input_tensors[1 - i]->mem != op->input_tensors[0]->mem)
        return false;
    const conv_op_t *c2 = reinterpret_cast<const conv_op_t *>(r), *c3 = reinterpret_cast<const conv_op_t *>(r2);
    const QSet &qi = add_inputs(a), &qo = add_output(a);
    if (!c1->plan || !c2->plan || !c3->plan || qi.alpha[1 - i] != c1->desc.ialpha || qi.zp[1 - i] != c1->desc.izp
        || !hipq_bottleneck_fusable(c1->plan, c2->plan, c3->plan, i == 1, qo.alpha[0], qo.zp[0], qo.bits[0]))
        return false;
    c1->blk_next = r;
    c1->blk_add = a;
    return true;
}

// op: a 3x3 convolution whose only reader r is a 1x1 convolution read by an add only - the middle of a block whose head
// has just left its launch to this chain, or of one that hipq_bottleneck_tail_run computes from here on
bool conv_continues_block(op_t *op, const op_t *r)
{
    const conv_op_t *c2 = reinterpret_cast<const conv_op_t *>(op), *c3 = reinterpret_cast<const conv_op_t *>(r);
    int i = 0;
    const op_t *a = add_reading(r, &i);
    if (a == nullptr || !c2->plan || !c3->plan)
        return false;
    const hip_mem_t *in = as_hip(op->input_tensors[0]->mem);
    if (in->pending == conv_launch_plain && reinterpret_cast<const conv_op_t *>(static_cast<op_t *>(in->pending_ctx))->blk_next == op)
        return true;
    const QSet &qi = add_inputs(a), &qo = add_output(a);
    if (hipq_bottleneck_tail_fusable(c2->plan, c3->plan, i == 1, qi.alpha[1 - i], qi.zp[1 - i], qo.alpha[0], qo.zp[0], qo.bits[0], nullptr))
        return true;
    // a form that pays only when the 1x1 convolution that reads the sum rides along (add_defers will hand the launch on to it)
    const reader_map &rm = readers_of(op);
    const auto it = rm.find(a->output_tensors[0].mem);
    if (it != rm.end())
        for (const op_t *rn : it->second) {
            if (rn->workspace != op->workspace || rn->entry->tp != &op_conv_2d_tp || rn->input_tensors[0]->mem != a->output_tensors[0].mem)
                continue;
            const conv_op_t *cn = reinterpret_cast<const conv_op_t *>(rn);
            if (cn->plan != nullptr
                && hipq_bottleneck_tail_fusable(c2->plan, c3->plan, i == 1, qi.alpha[1 - i], qi.zp[1 - i], qo.alpha[0], qo.zp[0], qo.bits[0],
                                                cn->plan))
                return true;
        }
    return false;
}

// 1: the only reader of the convolution's output is an add or a relu of this workspace that can take over the launch
bool sole_reader_fuses(op_t *op)
{
    static const bool off = getenv("NART_HIP_NO_FUSION") != nullptr;
    conv_op_t *c = reinterpret_cast<conv_op_t *>(op);
    if (off || c->desc.dtype != HIPQ_DTYPE_U8)
        return false;
    const reader_map &rm = readers_of(op);
    const auto it = rm.find(op->output_tensors[0].mem);
    if (it == rm.end() || it->second.size() != 1)
        return false;
    const op_t *r = *it->second.begin();
    if (r->workspace != op->workspace)
        return false;
    if (r->entry->tp == &op_relu_tp)
        return true; // any plan runs with the ReLU clamp (hipq_conv2d_run_relu)
    if (r->entry->tp == &op_conv_2d_tp)
        return conv_heads_block(op, r) || conv_continues_block(op, r);
    if (r->entry->tp == &op_pool_tp)
        return pool_fuses_with(r, c->plan);
    if (r->entry->tp == &op_hip_dequantize_tp)
        return dequantize_fuses_with(r, c->plan);
    // hipq_conv2d_run_add exists for the MFMA plans
    return (r->entry->tp == &op_add_tp || eltwise_is_plain_sum(r)) && r->input_size == 2
        && r->input_tensors[0]->mem != r->input_tensors[1]->mem && strncmp(hipq_conv2d_plan_kernel(c->plan), "conv_mfma", 9) == 0;
}

void conv_run(op_t *op)
{
    conv_op_t *c = reinterpret_cast<conv_op_t *>(op);
    if (c->computed_ahead) {
        c->computed_ahead = false;
        return;
    }
    if (c->defer == 0)
        c->defer = sole_reader_fuses(op) ? 1 : -1;
    if (c->defer == 1) {
        hip_mem_t *ym = as_hip(op->output_tensors[0].mem);
        (void)out_ptr(op); // the buffer exists and the device side is the current one - once the hook has run
        ym->pending = conv_launch_plain;
        ym->pending_ctx = op;
        return;
    }
    if (conv_run_chained(op, out_ptr(op), 0))
        return;
    HIPM_HIPQ(hipq_conv2d_run(c->plan, in_ptr(op, 0), out_ptr(op), nullptr, op_stream(op)));
}

// A walpha array with one entry per output channel (and more than one channel) selects per-channel requantisation, the
// convention of the reference's CUDA sibling (cuda_quant/src/op/conv_2d_quant.cu:751-764); a single entry is the
// per-tensor scale the reference CPU module reads (conv_2d_uint8_impl.c:57-66).  The reference's converter writes one
// entry per CONSTANT input (python/nart/modules/quant.py:178-208: the weights' scale, then the bias's), of which the CPU
// module reads the first (conv_2d_uint8_impl.c:61, ip.cpp:148): an array of that length is that convention and stays
// per tensor even when it happens to equal the channel count (a two-channel layer with a bias).
const float *per_channel_walpha(const conv_op_t *c)
{
    const op_t *op = reinterpret_cast<const op_t *>(c);
    const uint32_t n_const = op->input_size > 0 ? (uint32_t)op->input_size - 1 : 0;
    if (c->num_output <= 1 || (uint32_t)c->qw.n_alpha != (uint32_t)c->num_output || (uint32_t)c->qw.n_alpha == n_const)
        return nullptr;
    return c->qw.alpha;
}

void build_plan(op_t *op, const hipq_conv2d_desc &d, const uint8_t *w, const void *w_id)
{
    conv_op_t *c = reinterpret_cast<conv_op_t *>(op);
    c->defer = 0; // decided at the next run, when every operator of the pass has been prepared
    const float *wa_pc = per_channel_walpha(c);
    uint64_t pc_id = 0;
    if (wa_pc) {
        pc_id = 1469598103934665603ull;
        for (size_t i = 0; i < c->num_output * sizeof(float); ++i)
            pc_id = (pc_id ^ reinterpret_cast<const uint8_t *>(wa_pc)[i]) * 1099511628211ull;
        pc_id |= 1;
    }
    if (c->plan && memcmp(&c->desc, &d, sizeof d) == 0 && c->w_seen == w_id && c->pc_seen == pc_id)
        return; // prepare is called again after a reshape (art/src/parade.c:199-215): nothing changed
    hipq_conv2d_plan_destroy(c->plan);
    c->plan = nullptr;
    const int32_t *bias = nullptr;
    if (op->input_size == 3) {
        HIPM_CHECK(op->input_tensors[2]->dtype == dtINT32);
        bias = static_cast<const int32_t *>(is_hip_mem(op->input_tensors[2]->mem)
                                                ? hip_mem_host_in(op->input_tensors[2]->mem)
                                                : mem_cpu_data(op->input_tensors[2]->mem));
    } // without a bias the accumulator starts at zero (the reference reads an unset buffer there)
    if (wa_pc)
        HIPM_HIPQ(hipq_conv2d_plan_create_per_channel(&d, w, bias, wa_pc, &c->plan));
    else
        HIPM_HIPQ(hipq_conv2d_plan_create(&d, w, bias, &c->plan));
    c->desc = d;
    c->w_seen = w_id;
    c->pc_seen = pc_id;
    op->run_func = conv_run;
}

const uint8_t *host_weights(op_t *op)
{
    tensor_t *w = op->input_tensors[1];
    HIPM_CHECK(w->dtype == op->input_tensors[0]->dtype); // u8 x u8 or i8 x i8, as in the reference
    return static_cast<const uint8_t *>(is_hip_mem(w->mem) ? hip_mem_host_in(w->mem) : mem_cpu_data(w->mem));
}

// int8 tensors select the symmetric operators.  The reference picks special low-bit GEMMs that exist on aarch64 only
// when ibits and wbits are both below 8 (conv_2d.c:121-139, ip.cpp:313-318); their results equal the plain int8
// product for in-range values, which is what runs here.
int signed_dtype(op_t *op) { return op->input_tensors[0]->dtype == dtINT8 ? HIPQ_DTYPE_I8 : HIPQ_DTYPE_U8; }

void conv_prepare(op_t *op)
{
    conv_op_t *c = reinterpret_cast<conv_op_t *>(op);
    require_hip_u8(op, 1, true);
    alloc_and_tag(op);
    const shape_t &xs = op->input_tensors[0]->shape;
    const hip_mem_t *xm = as_hip(op->input_tensors[0]->mem), *ym = as_hip(op->output_tensors[0].mem);
    HIPM_CHECK(xs.dim_size == 4 && xm->layout == HIP_LAYOUT_NHWC_U8 && ym->layout == HIP_LAYOUT_NHWC_U8);
    same_shape_and_geometry(op, op->input_tensors[0]);
    hipq_conv2d_desc d;
    memset(&d, 0, sizeof d);
    d.N = (int)xs.dim[0], d.C = (int)xs.dim[1], d.H = (int)xs.dim[2], d.W = (int)xs.dim[3];
    d.K = (int)c->num_output, d.R = (int)c->kernel_h, d.S = (int)c->kernel_w;
    d.pad_h = (int)c->pad_h, d.pad_w = (int)c->pad_w, d.stride_h = (int)c->stride_h, d.stride_w = (int)c->stride_w;
    d.group = (int)c->group;
    d.in_cs = xm->cs, d.out_cs = ym->cs;
    // per-tensor parameters: element [0] of each array, like the reference (conv_2d_uint8_impl.c:57-66)
    d.ialpha = c->qi.alpha[0], d.walpha = c->qw.alpha[0], d.oalpha = c->qo.alpha[0];
    d.izp = c->qi.zp[0], d.wzp = c->qw.zp[0], d.ozp = c->qo.zp[0];
    d.obits = c->qo.bits[0];
    d.relu = 0; // the reference CPU module ignores SETTING_CONV_2D_RELU_FLAG (conv_2d.c:27-70); so does this one
    d.dtype = signed_dtype(op);
    build_plan(op, d, host_weights(op), op->input_tensors[1]->mem);
}

void ip_prepare(op_t *op)
{
    conv_op_t *c = reinterpret_cast<conv_op_t *>(op);
    require_hip_u8(op, 1, true);
    alloc_and_tag(op);
    const hip_mem_t *xm = as_hip(op->input_tensors[0]->mem), *ym = as_hip(op->output_tensors[0].mem);
    HIPM_CHECK(xm->layout == HIP_LAYOUT_NHWC_U8 && ym->layout == HIP_LAYOUT_NHWC_U8);
    const int dtype = signed_dtype(op);
    // the input's true geometry is the producer's (a flatten/reshape in between does not move bytes)
    const int M = xm->N, kd = xm->H * xm->W * xm->cs;
    const size_t kin = (size_t)xm->C * xm->H * xm->W;
    HIPM_CHECK(shape_count(&op->input_tensors[1]->shape) == (size_t)c->num_output * kin);
    HIPM_CHECK(ym->N == M && ym->C == (int)c->num_output && ym->H == 1 && ym->W == 1);
    const uint8_t *w = host_weights(op);
    std::vector<uint8_t> reordered;
    if (xm->H * xm->W > 1 || xm->cs != xm->C) { // (c,h,w) order of the reference -> (h,w,c) with channel stride
        reordered.resize((size_t)c->num_output * kd);
        HIPM_HIPQ(hipq_ip_reorder_weights(w, reordered.data(), (int)c->num_output, xm->C, xm->H, xm->W, xm->cs,
                                          dtype == HIPQ_DTYPE_I8 ? 0 : c->qw.zp[0])); // pad channels weigh nothing
        w = reordered.data();
    }
    hipq_conv2d_desc d;
    memset(&d, 0, sizeof d);
    d.N = M, d.C = kd, d.H = 1, d.W = 1, d.K = (int)c->num_output, d.R = 1, d.S = 1;
    d.stride_h = d.stride_w = 1, d.group = 1;
    d.in_cs = kd, d.out_cs = ym->cs;
    d.ialpha = c->qi.alpha[0], d.walpha = c->qw.alpha[0], d.oalpha = c->qo.alpha[0];
    d.izp = c->qi.zp[0], d.wzp = c->qw.zp[0], d.ozp = c->qo.zp[0];
    d.obits = c->qo.bits[0];
    d.dtype = dtype;
    build_plan(op, d, w, op->input_tensors[1]->mem);
}

// ---- element-wise ops ------------------------------------------------------------------------------------------
struct ew_op_t {
    op_t o;
    QSet qi, qo;
    uint32_t operation;
    float *coeff;
    size_t bytes; // device bytes to process (pad channels included)
    int defer;    // 0 undecided, 1 leave the (fused) launch to a reader of the output (relu: a max pooling; add: a 1x1
                  // convolution), -1 launch at run()
};

const QSet &add_inputs(const op_t *add_op) { return reinterpret_cast<const ew_op_t *>(add_op)->qi; }
const QSet &add_output(const op_t *add_op) { return reinterpret_cast<const ew_op_t *>(add_op)->qo; }

size_t device_bytes_of(const tensor_t *t)
{
    const hip_mem_t *m = as_hip(t->mem);
    return m->layout == HIP_LAYOUT_NHWC_U8 ? (size_t)m->N * m->H * m->W * m->cs : m->size;
}

void same_geometry(op_t *op)
{
    const hip_mem_t *a = as_hip(op->input_tensors[0]->mem);
    for (size_t i = 1; i < op->input_size; ++i) {
        const hip_mem_t *b = as_hip(op->input_tensors[i]->mem);
        HIPM_CHECK(shape_count(&op->input_tensors[i]->shape) == shape_count(&op->input_tensors[0]->shape));
        HIPM_CHECK(a->layout == b->layout && a->N == b->N && a->C == b->C && a->H == b->H && a->W == b->W);
    }
    const hip_mem_t *y = as_hip(op->output_tensors[0].mem);
    HIPM_CHECK(a->layout == y->layout && a->N == y->N && a->C == y->C && a->H == y->H && a->W == y->W);
}

void add_config(op_t *op)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    READ_I(op, &e->qi);
    READ_O(op, &e->qo);
    HIPM_CHECK(e->qi.n >= 2);
}

// A two-input SUM with unit coefficients gives add's bytes on the same inputs (eltwise.c:137-271 against add.c:83-148:
// the oracle's two restatements, both pinned against the reference, agree on every case tried), so it takes the same
// fused path.
bool eltwise_is_plain_sum(const op_t *op)
{
    const ew_op_t *e = reinterpret_cast<const ew_op_t *>(op);
    return op->entry->tp == &op_eltwise_tp && op->input_size == 2 && e->operation == SETTING_ELTWISE_OP_SUM && e->coeff != nullptr
        && e->coeff[0] == 1.0f && e->coeff[1] == 1.0f;
}

// which input of the add (or plain two-input SUM) `op` is a convolution that left it its launch (conv_run) and whose
// output the add reads with the scale it was written with; -1: none
int deferred_conv_input(op_t *op)
{
    const ew_op_t *e = reinterpret_cast<const ew_op_t *>(op);
    for (int i = 0; i < 2; ++i) {
        hip_mem_t *m = as_hip(op->input_tensors[i]->mem);
        if (m->pending != conv_launch_plain)
            continue;
        const conv_op_t *c = reinterpret_cast<const conv_op_t *>(static_cast<op_t *>(m->pending_ctx));
        return e->qi.alpha[i] == c->desc.oalpha && e->qi.zp[i] == c->desc.ozp ? i : -1;
    }
    return -1;
}

// the 3x3 convolution that left its launch to the widening convolution cop (which left its own to an add); null: none
op_t *deferred_mid_of(op_t *cop)
{
    hip_mem_t *m2 = as_hip(cop->input_tensors[0]->mem);
    if (m2->pending != conv_launch_plain)
        return nullptr;
    op_t *cop2 = static_cast<op_t *>(m2->pending_ctx);
    return cop2->entry->tp == &op_conv_2d_tp && only_reader(cop2) == cop ? cop2 : nullptr;
}

// The add `op`, whose input i is the widening convolution cop that left it its launch, as one launch with the block's
// earlier convolutions where those left theirs as well: the whole block (hipq_bottleneck_run) or the block from its 3x3
// layer on (hipq_bottleneck_tail_run), the sum into y; nxt: the 1x1 convolution that reads the sum and rides along
// (output into y_next, relu: with the ReLU clamp), or null.  false: nothing launched.
bool block_launch(op_t *op, op_t *cop, int i, void *y, op_t *nxt, int relu, void *y_next)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    op_t *cop2 = deferred_mid_of(cop);
    if (cop2 == nullptr)
        return false;
    conv_op_t *c3 = reinterpret_cast<conv_op_t *>(cop), *c2 = reinterpret_cast<conv_op_t *>(cop2);
    const int o = 1 - i;
    hip_mem_t *m1 = as_hip(cop2->input_tensors[0]->mem);
    const conv_op_t *cn = reinterpret_cast<const conv_op_t *>(nxt);
    if (m1->pending == conv_launch_plain) {
        op_t *cop1 = static_cast<op_t *>(m1->pending_ctx);
        conv_op_t *c1 = reinterpret_cast<conv_op_t *>(cop1);
        if (cop1->entry->tp == &op_conv_2d_tp && c1->blk_next == cop2 && c1->blk_add == op
            && op->input_tensors[o]->mem == cop1->input_tensors[0]->mem && e->qi.alpha[o] == c1->desc.ialpha && e->qi.zp[o] == c1->desc.izp
            && (nxt ? hipq_bottleneck_conv_fusable(c1->plan, c2->plan, c3->plan, o == 0, e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0], cn->plan)
                    : hipq_bottleneck_fusable(c1->plan, c2->plan, c3->plan, o == 0, e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0]))) {
            const void *x = in_ptr(cop1, 0);
            if (x != y
                && (nxt ? hipq_bottleneck_run_conv(c1->plan, c2->plan, c3->plan, x, o == 0, e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0], y,
                                                   cn->plan, relu, y_next, op_stream(op))
                        : hipq_bottleneck_run(c1->plan, c2->plan, c3->plan, x, o == 0, e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0], y,
                                              op_stream(op)))
                       == 0) {
                ++g_fused_adds;
                ++g_fused_blocks;
                if (nxt)
                    ++g_chained_convs;
                return true; // the three convolutions' outputs stay unwritten; their hooks stay for whoever asks
            }
        }
    }
    if (!hipq_bottleneck_tail_fusable(c2->plan, c3->plan, o == 0, e->qi.alpha[o], e->qi.zp[o], e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0],
                                      nxt ? cn->plan : nullptr))
        return false;
    const void *res = in_ptr(op, o);  // settles the other input if it is deferred
    const void *x = in_ptr(cop2, 0);  // and the block's head, whose output this form reads
    if (deferred_mid_of(cop) != cop2)
        return false; // settling reached the 3x3 convolution itself: it has run, the caller's path reads its output
    if (hipq_bottleneck_tail_run(c2->plan, c3->plan, x, res, o == 0, e->qi.alpha[o], e->qi.zp[o], e->qo.alpha[0], e->qo.zp[0],
                                 e->qo.bits[0], y, nxt ? cn->plan : nullptr, relu, y_next, op_stream(op)) != 0)
        return false;
    ++g_fused_adds;
    ++g_fused_tails;
    if (nxt)
        ++g_chained_convs;
    return true;
}

// the add `op` as the epilogue of the convolution that left it its launch, into y; false: run it plainly
bool run_fused_into_convolution(op_t *op, void *y)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    const int i = deferred_conv_input(op);
    if (i < 0)
        return false;
    op_t *cop = static_cast<op_t *>(as_hip(op->input_tensors[i]->mem)->pending_ctx);
    conv_op_t *c = reinterpret_cast<conv_op_t *>(cop);
    if (block_launch(op, cop, i, y, nullptr, 0, nullptr))
        return true;
    const int o = 1 - i;
    const void *res = in_ptr(op, o); // settles the other input if it is deferred as well
    const void *x = in_ptr(cop, 0);
    if (hipq_conv2d_run_add(c->plan, x, res, o == 0, e->qi.alpha[o], e->qi.zp[o], e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0], y,
                            op_stream(op)) != 0)
        return false; // parameters outside the fused kernel's range: the caller's plain path settles the hook
    ++g_fused_adds;
    return true; // the convolution's own output stays unwritten; its hook stays for whoever asks
}

void add_plain_into(op_t *op, void *y)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    if (op->entry->tp == &op_add_tp) {
        HIPM_HIPQ(hipq_add_u8(in_ptr(op, 0), in_ptr(op, 1), y, e->bytes, e->qi.alpha[0], e->qi.zp[0], e->qi.alpha[1], e->qi.zp[1],
                              e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0], op_stream(op)));
        return;
    }
    const void *ins[HIPQ_MAX_ELTWISE_INPUTS];
    for (size_t i = 0; i < op->input_size; ++i)
        ins[i] = in_ptr(op, (int)i);
    HIPM_HIPQ(hipq_eltwise_u8(ins, (int)op->input_size, e->coeff, e->qi.alpha, e->qi.zp, y, e->bytes, (int)e->operation,
                              e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0], op_stream(op)));
}

// The hook an add leaves on its output when a 1x1 convolution that reads the sum can run in the same kernel
// (add_defers): that convolution's run() launches hipq_conv2d_run_add_conv; whoever else asks for the sum first gets
// the convolution + add launch (or the plain add).
void add_launch_deferred(void *ctx)
{
    op_t *op = static_cast<op_t *>(ctx);
    void *y = as_hip(op->output_tensors[0].mem)->dev;
    if (!run_fused_into_convolution(op, y))
        add_plain_into(op, y);
}

// the add `op` closes a whole block (head -> mid -> c -> add with the head's input) that hipq_bottleneck_run_conv computes
// together with the 1x1 convolution rc that reads the sum
static bool whole_block_chains(op_t *op, op_t *mid, const conv_op_t *c, int o, const conv_op_t *rc)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    hip_mem_t *m1 = as_hip(mid->input_tensors[0]->mem);
    if (m1->pending != conv_launch_plain)
        return false;
    op_t *cop1 = static_cast<op_t *>(m1->pending_ctx);
    const conv_op_t *c1 = reinterpret_cast<const conv_op_t *>(cop1);
    return cop1->entry->tp == &op_conv_2d_tp && c1->blk_next == mid && c1->blk_add == op
        && op->input_tensors[o]->mem == cop1->input_tensors[0]->mem && e->qi.alpha[o] == c1->desc.ialpha && e->qi.zp[o] == c1->desc.izp
        && hipq_bottleneck_conv_fusable(c1->plan, reinterpret_cast<conv_op_t *>(mid)->plan, c->plan, o == 0, e->qo.alpha[0], e->qo.zp[0],
                                        e->qo.bits[0], rc->plan);
}

// Does the add leave its launch to a reader?  Decided once per prepare: a convolution was deferred into this add, and a
// 1x1 convolution of this workspace reads the sum and can run as the tail of the same kernel.
bool add_defers(op_t *op)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    const int i = deferred_conv_input(op);
    if (i < 0)
        return false;
    if (e->defer == 0) {
        static const bool off = getenv("NART_HIP_NO_FUSION") != nullptr;
        e->defer = -1;
        const conv_op_t *c = reinterpret_cast<const conv_op_t *>(static_cast<op_t *>(as_hip(op->input_tensors[i]->mem)->pending_ctx));
        const int o = 1 - i;
        const reader_map &rm = readers_of(op);
        const auto it = rm.find(op->output_tensors[0].mem);
        if (!off && it != rm.end())
            for (const op_t *r : it->second) {
                if (r->workspace != op->workspace || r->entry->tp != &op_conv_2d_tp)
                    continue;
                const conv_op_t *rc = reinterpret_cast<const conv_op_t *>(r);
                op_t *mid = deferred_mid_of(static_cast<op_t *>(as_hip(op->input_tensors[i]->mem)->pending_ctx));
                if (rc->plan != nullptr && r->input_tensors[0]->mem == op->output_tensors[0].mem
                    && (hipq_conv2d_add_conv_fusable(c->plan, o == 0, e->qi.alpha[o], e->qi.zp[o], e->qo.alpha[0], e->qo.zp[0],
                                                     e->qo.bits[0], rc->plan)
                        || (mid != nullptr
                            && (hipq_bottleneck_tail_fusable(reinterpret_cast<conv_op_t *>(mid)->plan, c->plan, o == 0, e->qi.alpha[o],
                                                             e->qi.zp[o], e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0], rc->plan)
                                || whole_block_chains(op, mid, c, o, rc))))) {
                    e->defer = 1;
                    break;
                }
            }
    }
    return e->defer == 1;
}

bool add_or_sum_run_fused(op_t *op)
{
    if (add_defers(op)) {
        hip_mem_t *ym = as_hip(op->output_tensors[0].mem);
        (void)out_ptr(op); // the buffer exists and the device side is the current one - once the hook has run
        ym->pending = add_launch_deferred;
        ym->pending_ctx = op;
        return true;
    }
    return run_fused_into_convolution(op, out_ptr(op));
}

bool conv_run_chained(op_t *op, void *y, int relu)
{
    hip_mem_t *sm = as_hip(op->input_tensors[0]->mem); // the sum
    if (sm->pending != add_launch_deferred)
        return false;
    op_t *aop = static_cast<op_t *>(sm->pending_ctx);
    ew_op_t *e = reinterpret_cast<ew_op_t *>(aop);
    const int i = deferred_conv_input(aop);
    if (i < 0)
        return false; // somebody asked for the first convolution's own output in between: it has run
    op_t *cop = static_cast<op_t *>(as_hip(aop->input_tensors[i]->mem)->pending_ctx);
    conv_op_t *c = reinterpret_cast<conv_op_t *>(cop), *c2 = reinterpret_cast<conv_op_t *>(op);
    const int o = 1 - i;
    if (deferred_mid_of(cop) != nullptr) {
        // the block from its 3x3 layer on, the add and this convolution as one launch
        sm->pending = nullptr; // the sum is written by that launch
        if (block_launch(aop, cop, i, sm->dev, op, relu, y))
            return true;
        sm->pending = add_launch_deferred;
        sm->pending_ctx = aop;
    }
    if (!hipq_conv2d_add_conv_fusable(c->plan, o == 0, e->qi.alpha[o], e->qi.zp[o], e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0],
                                      c2->plan))
        return false;
    const void *res = in_ptr(aop, o);
    const void *x = in_ptr(cop, 0);
    if (sm->pending != add_launch_deferred)
        return false; // settling the residual reached the sum (it cannot: the sum is not its own input), be safe
    sm->pending = nullptr; // the sum is written by the launch below
    if (hipq_conv2d_run_add_conv(c->plan, x, res, o == 0, e->qi.alpha[o], e->qi.zp[o], e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0],
                                 sm->dev, c2->plan, relu, y, op_stream(op)) != 0) {
        add_launch_deferred(aop); // cannot happen after the check above; keep the sum correct anyway
        return false;
    }
    ++g_fused_adds;
    ++g_chained_convs;
    return true;
}

void add_run(op_t *op)
{
    if (add_or_sum_run_fused(op))
        return;
    add_plain_into(op, out_ptr(op));
}

void add_prepare(op_t *op)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    require_hip_u8(op, 2);
    alloc_and_tag(op);
    same_geometry(op); // broadcasting adds are not implemented (the reference's loop has none either, add.c:135)
    e->bytes = device_bytes_of(&op->output_tensors[0]);
    e->defer = 0;
    op->run_func = add_run;
}

void eltwise_config(op_t *op)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    HIPM_CHECK(op_setting_single_get(op, SETTING_ELTWISE_OPERATION, dtUINT32, &e->operation));
    if (!op_setting_if_set(op, SETTING_ELTWISE_COEFF)) { // default coefficients: all ones (eltwise.c:60-68)
        std::vector<float> ones(op->input_size, 1.0f);
        HIPM_CHECK(op_setting_array_set(op, SETTING_ELTWISE_COEFF, dtFLOAT32, op->input_size, ones.data()));
    }
    size_t n = 0;
    HIPM_CHECK(op_setting_array_get(op, SETTING_ELTWISE_COEFF, dtFLOAT32, &n, &e->coeff));
    HIPM_CHECK(n == op->input_size);
    READ_I(op, &e->qi);
    READ_O(op, &e->qo);
    HIPM_CHECK(e->qi.n >= op->input_size);
}

void eltwise_run(op_t *op)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    if (eltwise_is_plain_sum(op) && add_or_sum_run_fused(op))
        return;
    const void *ins[HIPQ_MAX_ELTWISE_INPUTS];
    for (size_t i = 0; i < op->input_size; ++i)
        ins[i] = in_ptr(op, (int)i);
    HIPM_HIPQ(hipq_eltwise_u8(ins, (int)op->input_size, e->coeff, e->qi.alpha, e->qi.zp, out_ptr(op), e->bytes,
                              (int)e->operation, e->qo.alpha[0], e->qo.zp[0], e->qo.bits[0], op_stream(op)));
}

void eltwise_prepare(op_t *op)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    HIPM_CHECK(e->operation == SETTING_ELTWISE_OP_SUM || e->operation == SETTING_ELTWISE_OP_MAX); // PROD: eltwise.c:237
    HIPM_CHECK(op->input_size <= HIPQ_MAX_ELTWISE_INPUTS);
    require_hip_u8(op, op->input_size);
    alloc_and_tag(op);
    same_geometry(op);
    e->bytes = device_bytes_of(&op->output_tensors[0]);
    e->defer = 0;
    op->run_func = eltwise_run;
}

void relu_config(op_t *op)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    READ_I(op, &e->qi);
    READ_O(op, &e->qo);
}

// the relu `op` whose input is a convolution that left it its launch (conv_run): with equal scales and zero points on
// both sides the relu is max(x, zp), the convolution's lower clamp
bool relu_is_clamp_of(const ew_op_t *e, const conv_op_t *c)
{
    return e->qi.alpha[0] == c->desc.oalpha && e->qi.zp[0] == c->desc.ozp && e->qo.alpha[0] == c->desc.oalpha
        && e->qo.zp[0] == c->desc.ozp && e->qo.bits[0] == c->desc.obits;
}

// convolution + relu as one launch into the relu's output memory `y`; false: not possible, run the relu plainly
bool relu_launch_into(op_t *op, void *y)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    hip_mem_t *m = as_hip(op->input_tensors[0]->mem);
    if (m->pending != conv_launch_plain)
        return false;
    op_t *cop = static_cast<op_t *>(m->pending_ctx);
    conv_op_t *c = reinterpret_cast<conv_op_t *>(cop);
    if (!relu_is_clamp_of(e, c))
        return false;
    if (!conv_run_chained(cop, y, 1) && hipq_conv2d_run_relu(c->plan, in_ptr(cop, 0), y, op_stream(op)) != 0)
        return false;
    ++g_fused_relus;
    return true;
}

// the hook a relu leaves on its output when a max pooling will take over (relu_run): whoever else asks first gets the
// convolution and the relu as one launch, or as two
void relu_launch_deferred(void *ctx)
{
    op_t *op = static_cast<op_t *>(ctx);
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    void *y = as_hip(op->output_tensors[0].mem)->dev;
    if (!relu_launch_into(op, y))
        HIPM_HIPQ(hipq_relu_u8(in_ptr(op, 0), y, e->bytes, e->qi.alpha[0], e->qi.zp[0], e->qo.alpha[0], e->qo.zp[0],
                               e->qo.bits[0], op_stream(op)));
}

void relu_run(op_t *op)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    hip_mem_t *m = as_hip(op->input_tensors[0]->mem);
    if (m->pending == conv_launch_plain && relu_is_clamp_of(e, reinterpret_cast<conv_op_t *>(m->pending_ctx))) {
        // conv -> relu -> max pooling (the stem of a residual network): if the pooling is this relu's only reader and can
        // run inside the convolution's kernel, the relu passes the launch on to it
        if (e->defer == 0) {
            static const bool off = getenv("NART_HIP_NO_FUSION") != nullptr;
            e->defer = -1;
            const reader_map &rm = readers_of(op);
            const auto it = rm.find(op->output_tensors[0].mem);
            if (!off && it != rm.end() && it->second.size() == 1) {
                const op_t *r = *it->second.begin();
                if (r->workspace == op->workspace && r->entry->tp == &op_pool_tp
                    && pool_fuses_with(r, reinterpret_cast<conv_op_t *>(m->pending_ctx)->plan))
                    e->defer = 1;
            }
        }
        if (e->defer == 1) {
            hip_mem_t *ym = as_hip(op->output_tensors[0].mem);
            (void)out_ptr(op); // the buffer exists and the device side is the current one - once the hook has run
            ym->pending = relu_launch_deferred;
            ym->pending_ctx = op;
            return;
        }
    }
    if (relu_launch_into(op, out_ptr(op)))
        return;
    HIPM_HIPQ(hipq_relu_u8(in_ptr(op, 0), out_ptr(op), e->bytes, e->qi.alpha[0], e->qi.zp[0], e->qo.alpha[0], e->qo.zp[0],
                           e->qo.bits[0], op_stream(op)));
}

void deferred_launch_destroy(op_t *op)
{
    // a launch left to a reader (relu_run, add_or_sum_run_fused) must not outlive the operator
    if (op->output_size > 0 && op->output_tensors != nullptr && op->output_tensors[0].mem != nullptr
        && is_hip_mem(op->output_tensors[0].mem) && as_hip(op->output_tensors[0].mem)->pending_ctx == op)
        as_hip(op->output_tensors[0].mem)->pending = nullptr;
}

void relu_prepare(op_t *op)
{
    ew_op_t *e = reinterpret_cast<ew_op_t *>(op);
    require_hip_u8(op, 1);
    alloc_and_tag(op);
    same_geometry(op);
    e->bytes = device_bytes_of(&op->output_tensors[0]);
    e->defer = 0;
    op->run_func = relu_run;
}

// ---- concat / softmax (uint8 only, along the channels) --------------------------------------------------------------------
struct axis_op_t {
    op_t o;
    uint32_t axis;
    QSet qi, qo;
};

void concat_config(op_t *op)
{
    axis_op_t *a = reinterpret_cast<axis_op_t *>(op);
    HIPM_CHECK(op_setting_single_get(op, SETTING_CONCAT_AXIS, dtUINT32, &a->axis));
    READ_I(op, &a->qi);
    READ_O(op, &a->qo);
    HIPM_CHECK(a->qi.n >= op->input_size);
}

void concat_run(op_t *op)
{
    axis_op_t *a = reinterpret_cast<axis_op_t *>(op);
    const void *in[HIPQ_MAX_ELTWISE_INPUTS];
    int ch[HIPQ_MAX_ELTWISE_INPUTS];
    for (size_t i = 0; i < op->input_size; ++i) {
        in[i] = in_ptr(op, (int)i);
        ch[i] = as_hip(op->input_tensors[i]->mem)->C;
    }
    const hip_mem_t *y = as_hip(op->output_tensors[0].mem);
    HIPM_HIPQ(hipq_concat_u8(in, (int)op->input_size, ch, a->qi.alpha, a->qi.zp, out_ptr(op), (size_t)y->N * y->H * y->W,
                             a->qo.alpha[0], a->qo.zp[0], a->qo.bits[0], op_stream(op)));
}

void concat_prepare(op_t *op)
{
    axis_op_t *a = reinterpret_cast<axis_op_t *>(op);
    HIPM_CHECK(op->input_size <= HIPQ_MAX_ELTWISE_INPUTS);
    require_hip_u8(op, op->input_size);
    alloc_and_tag(op);
    // the reference's loop copies image by image, input by input (concat.c:99-121): that is a concatenation along
    // dimension 1 whatever the axis setting says, so only axis 1 has a meaning to reproduce
    if (a->axis != 1) {
        fprintf(stderr, "[hip module] concat along axis %u is not implemented (channels only)\n", a->axis);
        abort();
    }
    const hip_mem_t *y = as_hip(op->output_tensors[0].mem);
    HIPM_CHECK(y->layout == HIP_LAYOUT_NHWC_U8);
    for (size_t i = 0; i < op->input_size; ++i) {
        const hip_mem_t *x = as_hip(op->input_tensors[i]->mem);
        HIPM_CHECK(x->layout == HIP_LAYOUT_NHWC_U8 && x->N == y->N && x->H == y->H && x->W == y->W);
        if (op->input_tensors[i]->shape.dim_size == 4)
            same_shape_and_geometry(op, op->input_tensors[i]);
    }
    op->run_func = concat_run;
}

void softmax_config(op_t *op)
{
    axis_op_t *a = reinterpret_cast<axis_op_t *>(op);
    HIPM_CHECK(op_setting_single_get(op, SETTING_SOFTMAX_AXIS, dtUINT32, &a->axis));
    READ_I(op, &a->qi);
    READ_O(op, &a->qo);
}

void softmax_run(op_t *op)
{
    axis_op_t *a = reinterpret_cast<axis_op_t *>(op);
    const hip_mem_t *x = as_hip(op->input_tensors[0]->mem);
    HIPM_HIPQ(hipq_softmax_u8(in_ptr(op, 0), out_ptr(op), (size_t)x->N * x->H * x->W, x->C, x->cs, a->qi.alpha[0], a->qi.zp[0],
                              a->qo.alpha[0], a->qo.zp[0], a->qo.bits[0], op_stream(op)));
}

void softmax_prepare(op_t *op)
{
    axis_op_t *a = reinterpret_cast<axis_op_t *>(op);
    require_hip_u8(op, 1);
    alloc_and_tag(op);
    same_geometry(op);
    if (a->axis != 1) { // other axes would need a strided walk over the channels-last device layout
        fprintf(stderr, "[hip module] softmax along axis %u is not implemented (channels only)\n", a->axis);
        abort();
    }
    HIPM_CHECK(as_hip(op->input_tensors[0]->mem)->layout == HIP_LAYOUT_NHWC_U8);
    if (op->input_tensors[0]->shape.dim_size == 4)
        same_shape_and_geometry(op, op->input_tensors[0]);
    op->run_func = softmax_run;
}

// ---- pool ----------------------------------------------------------------------------------------------------------
struct pool_op_t {
    op_t o;
    uint32_t method, pad_h, pad_w, kernel_h, kernel_w, stride_h, stride_w;
    bool ceil_mode;
    QSet qi, qo;
};

void pool_config(op_t *op)
{
    pool_op_t *p = reinterpret_cast<pool_op_t *>(op);
    HIPM_CHECK(op_setting_single_get(op, SETTING_POOL_KERNEL_H, dtUINT32, &p->kernel_h));
    HIPM_CHECK(op_setting_single_get(op, SETTING_POOL_KERNEL_W, dtUINT32, &p->kernel_w));
    HIPM_CHECK(op_setting_single_get(op, SETTING_POOL_METHOD, dtUINT32, &p->method));
    HIPM_CHECK(op_setting_single_get(op, SETTING_POOL_PAD_H, dtUINT32, &p->pad_h));
    HIPM_CHECK(op_setting_single_get(op, SETTING_POOL_PAD_W, dtUINT32, &p->pad_w));
    HIPM_CHECK(op_setting_single_get(op, SETTING_POOL_STRIDE_H, dtUINT32, &p->stride_h));
    HIPM_CHECK(op_setting_single_get(op, SETTING_POOL_STRIDE_W, dtUINT32, &p->stride_w));
    HIPM_CHECK(op_setting_single_get(op, SETTING_POOL_CEIL_MODE, dtBOOL, &p->ceil_mode));
    READ_I(op, &p->qi);
    READ_O(op, &p->qo);
}

bool pool_fuses_with(const op_t *op, const hipq_conv2d_plan *plan)
{
    const pool_op_t *p = reinterpret_cast<const pool_op_t *>(op);
    if (p->method != SETTING_POOL_MAX || p->kernel_h != p->kernel_w || p->stride_h != p->stride_w || p->pad_h != p->pad_w
        || op->output_tensors[0].mem == nullptr || !is_hip_mem(op->output_tensors[0].mem))
        return false;
    const hip_mem_t *y = as_hip(op->output_tensors[0].mem);
    return hipq_conv2d_maxpool_fusable(plan, y->H, y->W, (int)p->kernel_h, (int)p->stride_h, (int)p->pad_h, p->qi.alpha[0],
                                       p->qi.zp[0], p->qo.alpha[0], p->qo.zp[0], p->qo.bits[0]) != 0;
}

// the pooling `op` inside the kernel of the convolution that left it its launch, directly (conv_run) or through a relu
// (relu_run); false: run it plainly
bool pool_run_fused(op_t *op)
{
    hip_mem_t *x = as_hip(op->input_tensors[0]->mem);
    op_t *cop = nullptr;
    int relu = 0;
    if (x->pending == conv_launch_plain) {
        cop = static_cast<op_t *>(x->pending_ctx);
    } else if (x->pending == relu_launch_deferred) {
        hip_mem_t *cm = as_hip(static_cast<op_t *>(x->pending_ctx)->input_tensors[0]->mem);
        if (cm->pending != conv_launch_plain)
            return false; // someone asked for the convolution's own output in between: it has run
        cop = static_cast<op_t *>(cm->pending_ctx);
        relu = 1;
    } else {
        return false;
    }
    conv_op_t *c = reinterpret_cast<conv_op_t *>(cop);
    if (!pool_fuses_with(op, c->plan))
        return false;
    const hip_mem_t *y = as_hip(op->output_tensors[0].mem);
    const void *xin = in_ptr(cop, 0);
    // The 1x1 convolutions that read the pooled tensor - a residual network's first layer and its projection shortcut -
    // are computed by the same kernel while a pooled row is in LDS, when they are its only readers (one or two): their
    // run() then finds its work done.
    static const bool no_chain = getenv("NART_HIP_NO_FUSION") != nullptr;
    const reader_map &rm = readers_of(op);
    const auto it = rm.find(op->output_tensors[0].mem);
    if (!no_chain && it != rm.end() && (it->second.size() == 1 || it->second.size() == 2)) {
        conv_op_t *nx[2] = {nullptr, nullptr};
        int n = 0;
        bool ok = true;
        for (const op_t *r : it->second) {
            conv_op_t *cn = reinterpret_cast<conv_op_t *>(const_cast<op_t *>(r));
            ok = ok && r->workspace == op->workspace && r->entry->tp == &op_conv_2d_tp
                && r->input_tensors[0]->mem == op->output_tensors[0].mem && cn->plan != nullptr;
            nx[n++] = cn;
        }
        if (ok && hipq_conv2d_maxpool_conv_fusable(c->plan, y->H, y->W, nx[0]->plan, nx[1] ? nx[1]->plan : nullptr)) {
            void *y0 = out_ptr(&nx[0]->o), *y1 = nx[1] ? out_ptr(&nx[1]->o) : nullptr;
            if (hipq_conv2d_run_maxpool_conv(c->plan, xin, out_ptr(op), y->H, y->W, relu, nx[0]->plan, 0, y0,
                                             nx[1] ? nx[1]->plan : nullptr, 0, y1, op_stream(op)) == 0) {
                nx[0]->computed_ahead = true;
                if (nx[1])
                    nx[1]->computed_ahead = true;
                ++g_fused_pools;
                g_chained_convs += n;
                return true;
            }
        }
    }
    if (hipq_conv2d_run_maxpool(c->plan, xin, out_ptr(op), y->H, y->W, relu, op_stream(op)) != 0)
        return false;
    ++g_fused_pools;
    return true; // the hooks stay for whoever asks for the intermediate tensors
}

void pool_run(op_t *op)
{
    pool_op_t *p = reinterpret_cast<pool_op_t *>(op);
    if (pool_run_fused(op))
        return;
    const hip_mem_t *x = as_hip(op->input_tensors[0]->mem), *y = as_hip(op->output_tensors[0].mem);
    HIPM_HIPQ(hipq_pool_u8(in_ptr(op, 0), out_ptr(op), x->N, x->C, x->H, x->W, y->H, y->W, x->cs, (int)p->kernel_h,
                           (int)p->kernel_w, (int)p->pad_h, (int)p->pad_w, (int)p->stride_h, (int)p->stride_w,
                           p->method == SETTING_POOL_MAX ? HIPQ_POOL_MAX : HIPQ_POOL_AVE, p->qi.alpha[0], p->qi.zp[0],
                           p->qo.alpha[0], p->qo.zp[0], p->qo.bits[0], op_stream(op)));
}

void pool_prepare(op_t *op)
{
    require_hip_u8(op, 1);
    alloc_and_tag(op);
    HIPM_CHECK(op->input_tensors[0]->shape.dim_size == 4);
    same_shape_and_geometry(op, op->input_tensors[0]);
    op->run_func = pool_run;
}

// ---- reshape: zero-copy view (the output shares the input's memory, art/src/op.c:1115) -----------------------
void reshape_config(op_t *) {}
void reshape_run(op_t *) {}
void reshape_prepare(op_t *op)
{
    for (size_t i = 0; i < op->input_size; ++i)
        tensor_alloc(op->input_tensors[i]);
    op->run_func = reshape_run;
}

// ---- quantize / dequantize -------------------------------------------------------------------------------------------
struct qdq_op_t {
    op_t o;
    QSet q;
    int32_t qtype;
};

void dims4(const tensor_t *t, int d[4])
{
    const int nd = t->shape.dim_size;
    d[0] = (int)t->shape.dim[0];
    d[1] = nd > 1 ? (int)t->shape.dim[1] : 1;
    d[2] = nd > 2 ? (int)t->shape.dim[2] : 1;
    d[3] = nd > 3 ? (int)t->shape.dim[3] : 1;
}

void quantize_config(op_t *op)
{
    qdq_op_t *q = reinterpret_cast<qdq_op_t *>(op);
    READ_O(op, &q->q);
    HIPM_CHECK(op_setting_single_get(op, SETTING_QUANT_QTYPE, dtINT32, &q->qtype));
}

void quantize_run(op_t *op)
{
    qdq_op_t *q = reinterpret_cast<qdq_op_t *>(op);
    int d[4];
    dims4(op->input_tensors[0], d);
    const hip_mem_t *y = as_hip(op->output_tensors[0].mem);
    if (op->output_tensors[0].dtype == dtINT8)
        HIPM_HIPQ(hipq_quantize_i8(static_cast<const float *>(in_ptr(op, 0)), out_ptr(op), d[0], d[1], d[2], d[3], y->cs,
                                   q->q.alpha[0], q->q.bits[0], op_stream(op)));
    else
        HIPM_HIPQ(hipq_quantize_u8(static_cast<const float *>(in_ptr(op, 0)), out_ptr(op), d[0], d[1], d[2], d[3], y->cs,
                                   q->q.alpha[0], q->q.zp[0], q->q.bits[0], op_stream(op)));
}

// (qtype << 8 | bits) rows of quantize.c:233-262 / dequantize.c:150-167 that exist here: 1 = uint8, 2 = int8
int qdq_row(int32_t key)
{
    if (key == 0x0008 || key == 0x0108)
        return 1;
    if (key >= 0x0202 && key <= 0x0208 && key != 0x0205)
        return 2;
    return 0;
}

void quantize_prepare(op_t *op)
{
    qdq_op_t *q = reinterpret_cast<qdq_op_t *>(op);
    HIPM_CHECK(op->input_tensors[0]->dtype == dtFLOAT32 && is_hip_mem(op->input_tensors[0]->mem));
    const int row = qdq_row(q->qtype << 8 | q->q.bits[0]);
    if (row == 0) { // the 16- and 32-bit rows of quantize.c:233-262 are not implemented
        fprintf(stderr, "[hip module] quantization for %d bits with type %d is not implemented\n", q->q.bits[0], q->qtype);
        abort();
    }
    HIPM_CHECK(op->output_tensors[0].dtype == (row == 2 ? dtINT8 : dtUINT8));
    const int nd = op->input_tensors[0]->shape.dim_size;
    HIPM_CHECK(nd == 4 || nd == 2);
    hip_mem_tag(op->input_tensors[0]);
    alloc_and_tag(op);
    op->run_func = quantize_run;
}

void dequantize_config(op_t *op)
{
    qdq_op_t *q = reinterpret_cast<qdq_op_t *>(op);
    READ_I(op, &q->q);
    HIPM_CHECK(op_setting_single_get(op, SETTING_QUANT_QTYPE, dtINT32, &q->qtype));
}

bool dequantize_fuses_with(const op_t *deq_op, const hipq_conv2d_plan *plan)
{
    const qdq_op_t *q = reinterpret_cast<const qdq_op_t *>(deq_op);
    return qdq_row(q->qtype << 8 | q->q.bits[0]) == 1 && hipq_conv2d_dequant_fusable(plan, q->q.alpha[0], q->q.zp[0]) != 0;
}

void dequantize_run(op_t *op)
{
    qdq_op_t *q = reinterpret_cast<qdq_op_t *>(op);
    hip_mem_t *xm = as_hip(op->input_tensors[0]->mem);
    if (xm->pending == conv_launch_plain) {
        // a fully-connected layer left its launch to this operator (conv_run): one kernel computes the layer and writes
        // the float values; the layer's own bytes stay unwritten, its hook stays for whoever asks for them
        op_t *cop = static_cast<op_t *>(xm->pending_ctx);
        conv_op_t *c = reinterpret_cast<conv_op_t *>(cop);
        if (dequantize_fuses_with(op, c->plan)
            && hipq_conv2d_run_dequant(c->plan, in_ptr(cop, 0), static_cast<float *>(out_ptr(op)), op_stream(op)) == 0) {
            ++g_fused_dequants;
            return;
        }
    }
    const hip_mem_t *x = xm;
    if (qdq_row(q->qtype << 8 | q->q.bits[0]) == 2) // chosen from the settings, not from the tensor's dtype (dequantize.c:141-163)
        HIPM_HIPQ(hipq_dequantize_i8(in_ptr(op, 0), static_cast<float *>(out_ptr(op)), x->N, x->C, x->H, x->W, x->cs,
                                     q->q.alpha[0], op_stream(op)));
    else
        HIPM_HIPQ(hipq_dequantize_u8(in_ptr(op, 0), static_cast<float *>(out_ptr(op)), x->N, x->C, x->H, x->W, x->cs,
                                     q->q.alpha[0], q->q.zp[0], op_stream(op)));
}

void dequantize_prepare(op_t *op)
{
    qdq_op_t *q = reinterpret_cast<qdq_op_t *>(op);
    if (qdq_row(q->qtype << 8 | q->q.bits[0]) == 0) { // dequantize.c:150-167
        fprintf(stderr, "[hip module] dequantization for %d bits with type %d is not implemented\n", q->q.bits[0], q->qtype);
        abort();
    }
    require_hip_u8(op, 1, true);
    alloc_and_tag(op);
    HIPM_CHECK(as_hip(op->input_tensors[0]->mem)->layout == HIP_LAYOUT_NHWC_U8);
    op->run_func = dequantize_run;
}

// ---- workspace ------------------------------------------------------------------------------------------------------------
int g_ws_count = 0;

const char *ws_name(const workspace_t *ws) { return reinterpret_cast<const hip_workspace_t *>(ws)->name; }
const mem_tp *ws_memtype(const workspace_t *) { return &hip_mem_tp_st; }

void ws_delete(workspace_t *w)
{
    hip_workspace_t *ws = reinterpret_cast<hip_workspace_t *>(w);
    if (ws->own_stream && ws->stream) {
        hip_stream_retire(ws->stream); // memories that outlive the workspace remember this stream
        (void)hipStreamDestroy(ws->stream);
    } else if (ws->stream) {
        hip_stream_forget(ws->stream);
    }
    g_readers.erase(w);
    free(ws);
}

} // namespace

extern "C" {

extern const module_t hip_module_tp;

#define SETTING_HIP_WORKSPACE_DEVID 1 /* same id as SETTING_CUDA_QUANT_WORKSPACE_DEVID (cuda_quant_module.c:98-114) */

static workspace_t *ws_new(const setting_entry_t *settings)
{
    hip_workspace_t *ws = static_cast<hip_workspace_t *>(calloc(1, sizeof(hip_workspace_t)));
    ws->ws.module_type = &hip_module_tp;
    snprintf(ws->name, sizeof ws->name, "hip:%d", g_ws_count++);
    for (const setting_entry_t *s = settings; s != nullptr && s->item != 0; ++s)
        if (s->item == SETTING_HIP_WORKSPACE_DEVID)
            ws->dev_id = (int)s->v.single.value.u32;
    // the device is touched here, once; without a usable GPU the workspace cannot exist
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= ws->dev_id) {
        fprintf(stderr, "[hip module] no usable GPU for device id %d (%s)\n", ws->dev_id,
                e == hipSuccess ? "device count too small" : hipGetErrorString(e));
        free(ws);
        return nullptr;
    }
    HIPM_HIP(hipSetDevice(ws->dev_id));
    HIPM_HIP(hipStreamCreateWithFlags(&ws->stream, hipStreamNonBlocking)); // default priority
    ws->own_stream = true;
    hip_stream_register(ws->stream);
    return &ws->ws;
}

// Extra entry points for runners that own a stream already (graph capture, event timing).
// How many add operators have run fused into the convolution that produces one of their inputs (diagnostics, tests).
ART_PUBLIC long hip_module_fused_adds(void) { return g_fused_adds; }
ART_PUBLIC long hip_module_fused_relus(void) { return g_fused_relus; }
ART_PUBLIC long hip_module_fused_pools(void) { return g_fused_pools; }
ART_PUBLIC long hip_module_chained_convs(void) { return g_chained_convs; }
ART_PUBLIC long hip_module_fused_dequants(void) { return g_fused_dequants; }
ART_PUBLIC long hip_module_fused_blocks(void) { return g_fused_blocks; }
ART_PUBLIC long hip_module_fused_tails(void) { return g_fused_tails; }

ART_PUBLIC void *hip_workspace_stream(workspace_t *w) { return reinterpret_cast<hip_workspace_t *>(w)->stream; }

ART_PUBLIC void hip_workspace_set_stream(workspace_t *w, void *stream)
{
    hip_workspace_t *ws = reinterpret_cast<hip_workspace_t *>(w);
    if (ws->own_stream && ws->stream) {
        hip_stream_retire(ws->stream);
        (void)hipStreamDestroy(ws->stream);
    } else if (ws->stream) {
        hip_stream_forget(ws->stream);
    }
    ws->stream = static_cast<hipStream_t>(stream);
    ws->own_stream = false;
    if (ws->stream)
        hip_stream_register(ws->stream);
}

// Blocks until everything the workspace has launched is done; runners that time a run call it (operators return
// as soon as their kernels are queued).
ART_PUBLIC void hip_workspace_synchronize(workspace_t *w)
{
    HIPM_HIP(hipStreamSynchronize(reinterpret_cast<hip_workspace_t *>(w)->stream));
}

#define HIP_ENTRY(TP, T, CONFIG, DESTROY, PREPARE) {&TP, alloc_op<T>, CONFIG, DESTROY, dealloc_op, PREPARE}

ART_PUBLIC op_tp_entry_t hip_op_table[] = {
    HIP_ENTRY(op_hip_quantize_tp, qdq_op_t, quantize_config, destroy_nothing, quantize_prepare),
    HIP_ENTRY(op_hip_dequantize_tp, qdq_op_t, dequantize_config, destroy_nothing, dequantize_prepare),
    HIP_ENTRY(op_conv_2d_tp, conv_op_t, conv_config, conv_destroy, conv_prepare),
    HIP_ENTRY(op_ip_tp, conv_op_t, ip_config, conv_destroy, ip_prepare),
    HIP_ENTRY(op_relu_tp, ew_op_t, relu_config, deferred_launch_destroy, relu_prepare),
    HIP_ENTRY(op_add_tp, ew_op_t, add_config, deferred_launch_destroy, add_prepare),
    HIP_ENTRY(op_eltwise_tp, ew_op_t, eltwise_config, deferred_launch_destroy, eltwise_prepare),
    HIP_ENTRY(op_pool_tp, pool_op_t, pool_config, destroy_nothing, pool_prepare),
    HIP_ENTRY(op_reshape_tp, ew_op_t, reshape_config, destroy_nothing, reshape_prepare),
    HIP_ENTRY(op_concat_tp, axis_op_t, concat_config, destroy_nothing, concat_prepare),
    HIP_ENTRY(op_softmax_tp, axis_op_t, softmax_config, destroy_nothing, softmax_prepare),
    {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr},
};

// op_group 6 = OP_GROUP_CODE_QUANT: an engine file written by the quant converter stamps every op with it,
// so the strict pass of the loader's workspace choice picks this module (art/src/serialize_v1.c:103-120).
ART_PUBLIC const module_t hip_module_tp = {
    6, ws_name, ws_memtype, ws_new, ws_delete, hip_op_table,
};

} // extern "C"
