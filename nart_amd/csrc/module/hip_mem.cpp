// hip_mem_tp: the memory type of the `hip` workspace — a device buffer plus a pinned host mirror, kept
// coherent on demand.  Implements the mem_tp vtable of art/include/art/mem.h:48-64.
#include <algorithm>
#include <cstring>
#include <vector>

#include "hip_module.h"

// The streams of the live `hip` workspaces.  A memory remembers the stream that last wrote its device side and the one
// that last read its host mirror, and may outlive the workspace that owned it: a stream that has been retired was
// synchronised when its workspace went away, so there is nothing left to wait for (and nothing valid to wait on).
static std::vector<hipStream_t> &live_streams()
{
    static std::vector<hipStream_t> v;
    return v;
}

void hip_stream_register(hipStream_t st) { live_streams().push_back(st); }

void hip_stream_retire(hipStream_t st)
{
    HIPM_HIP(hipStreamSynchronize(st));
    auto &v = live_streams();
    v.erase(std::remove(v.begin(), v.end(), st), v.end());
}

void hip_stream_forget(hipStream_t st)
{
    auto &v = live_streams();
    v.erase(std::remove(v.begin(), v.end(), st), v.end());
}

// wait for the work queued on st - and only on st: another workspace's kernels keep running.  A stream this module no
// longer knows (its workspace is gone, or it was a caller's stream that has been replaced) cannot be named any more:
// then the whole device is waited for, as the runtime's other GPU modules always do.
static void wait_stream(hipStream_t st)
{
    auto &v = live_streams();
    if (st == nullptr || std::find(v.begin(), v.end(), st) != v.end())
        HIPM_HIP(hipStreamSynchronize(st));
    else
        HIPM_HIP(hipDeviceSynchronize());
}

static void grow_dev(void **p, size_t *cap, size_t need)
{
    if (*cap >= need)
        return;
    if (*p)
        HIPM_HIP(hipFree(*p));
    HIPM_HIP(hipMalloc(p, need));
    *cap = need;
}

static size_t dev_bytes(const hip_mem_t *m)
{
    return m->layout == HIP_LAYOUT_NHWC_U8 ? (size_t)m->N * m->H * m->W * m->cs : m->size;
}

static mem_t *hm_new(void)
{
    auto *m = static_cast<hip_mem_t *>(calloc(1, sizeof(hip_mem_t)));
    return &m->m;
}

static void hm_free(mem_t *mm)
{
    hip_mem_t *m = as_hip(mm);
    if (m->host)
        HIPM_HIP(hipHostFree(m->host));
    if (m->dev)
        HIPM_HIP(hipFree(m->dev));
    if (m->stage)
        HIPM_HIP(hipFree(m->stage));
    m->host = m->dev = m->stage = nullptr;
    m->host_cap = m->dev_cap = m->stage_cap = m->size = 0;
    m->host_valid = m->dev_valid = false;
    m->up_pending = false;
    m->pending = nullptr;
}

static void hm_delete(mem_t *mm)
{
    hm_free(mm);
    free(mm);
}

// grow-only, like every mem_tp of the runtime (art/src/mem.c:45-55); buffers appear lazily
static bool hm_alloc(mem_t *mm, size_t sz)
{
    hip_mem_t *m = as_hip(mm);
    if (sz > m->size)
        m->size = sz;
    return true;
}

static size_t hm_size(mem_t *mm) { return as_hip(mm)->size; }

static void ensure_host(hip_mem_t *m)
{
    if (m->host_cap >= m->size && m->host)
        return;
    void *p = nullptr;
    HIPM_HIP(hipHostMalloc(&p, m->size ? m->size : 1, hipHostMallocDefault));
    memset(p, 0, m->size);
    if (m->host) {
        if (m->up_pending) { // an upload may still read the old mirror
            wait_stream(m->up_stream);
            m->up_pending = false;
        }
        memcpy(p, m->host, m->host_cap);
        HIPM_HIP(hipHostFree(m->host));
    }
    m->host = p;
    m->host_cap = m->size;
}

// device -> host (dense NCHW); synchronous
static void download(hip_mem_t *m)
{
    ensure_host(m);
    if (m->layout == HIP_LAYOUT_NHWC_U8) {
        grow_dev(&m->stage, &m->stage_cap, m->size);
        HIPM_HIPQ(hipq_nhwc_to_nchw_u8(m->dev, m->stage, m->N, m->C, m->H, m->W, m->cs, nullptr));
        HIPM_HIP(hipMemcpy(m->host, m->stage, m->size, hipMemcpyDeviceToHost));
    } else {
        HIPM_HIP(hipMemcpy(m->host, m->dev, m->size, hipMemcpyDeviceToHost));
    }
    m->host_valid = true;
}

static void upload(hip_mem_t *m, hipStream_t st)
{
    grow_dev(&m->dev, &m->dev_cap, dev_bytes(m));
    if (m->layout == HIP_LAYOUT_NHWC_U8) {
        grow_dev(&m->stage, &m->stage_cap, m->size);
        HIPM_HIP(hipMemcpyAsync(m->stage, m->host, m->size, hipMemcpyHostToDevice, st));
        HIPM_HIPQ(hipq_nchw_to_nhwc_u8(m->stage, m->dev, m->N, m->C, m->H, m->W, m->cs, st));
    } else {
        HIPM_HIP(hipMemcpyAsync(m->dev, m->host, m->size, hipMemcpyHostToDevice, st));
    }
    m->dev_valid = true;
    m->up_pending = true; // the copy still reads the mirror
    m->up_stream = st;
    m->prod_stream = st;
}

// the mirror is about to be handed out for writing: an upload that still reads it must finish first
static void finish_upload(hip_mem_t *m)
{
    if (m->up_pending) {
        wait_stream(m->up_stream);
        m->up_pending = false;
    }
}

// mem_cpu_data(): the caller may read or WRITE through the pointer (the runtime fills inputs and weights this
// way, art/src/serialize_v1.c:239-241), so afterwards the host side is the master copy.
static void *hm_cpu_data(const mem_t *mm)
{
    hip_mem_t *m = as_hip(const_cast<mem_t *>(mm));
    hip_mem_settle(m);
    if (m->dev_valid && !m->host_valid) {
        wait_stream(m->prod_stream); // the producing kernels run on that workspace's stream; other workspaces are not waited for
        download(m);
    }
    ensure_host(m);
    finish_upload(m);
    m->host_valid = true;
    m->dev_valid = false;
    return m->host;
}

const void *hip_mem_host_in(mem_t *mm)
{
    hip_mem_t *m = as_hip(mm);
    hip_mem_settle(m);
    if (m->dev_valid && !m->host_valid) {
        wait_stream(m->prod_stream);
        download(m);
    }
    ensure_host(m);
    m->host_valid = true; // read-only: the device copy stays valid
    return m->host;
}

const void *hip_mem_dev_in(mem_t *mm, hipStream_t st)
{
    hip_mem_t *m = as_hip(mm);
    hip_mem_settle(m);
    if (!m->dev_valid) {
        ensure_host(m); // never-written memory reads as zeros
        m->host_valid = true;
        upload(m, st);
    }
    return m->dev;
}

void *hip_mem_dev_out(mem_t *mm, hipStream_t st)
{
    hip_mem_t *m = as_hip(mm);
    m->pending = nullptr; // about to be overwritten: a deferred producer's result is dead
    m->prod_stream = st;  // whoever reads the contents from outside that stream waits for it first
    grow_dev(&m->dev, &m->dev_cap, dev_bytes(m));
    m->dev_valid = true;
    m->host_valid = false;
    return m->dev;
}

// mem_data(): device pointer for callers outside the module; they may read or write it
static void *hm_data(const mem_t *mm)
{
    mem_t *m = const_cast<mem_t *>(mm);
    const void *p = hip_mem_dev_in(m, nullptr);
    // the caller is foreign code with streams of its own: every producer of this memory (kernels on a workspace
    // stream, a settled convolution, the upload on the null stream) must have finished
    HIPM_HIP(hipDeviceSynchronize());
    as_hip(m)->up_pending = false;
    as_hip(m)->host_valid = false;
    return const_cast<void *>(p);
}

static void *hm_copy_from_cpu(void *to, const void *from, size_t sz)
{
    HIPM_HIP(hipMemcpy(to, from, sz, hipMemcpyHostToDevice));
    return to;
}

static void *hm_copy_to_cpu(void *to, const void *from, size_t sz)
{
    HIPM_HIP(hipMemcpy(to, from, sz, hipMemcpyDeviceToHost));
    return to;
}

const mem_tp hip_mem_tp_st = {
    "hip_mem", hm_new, hm_delete, hm_alloc, hm_free, hm_data, hm_cpu_data, hm_size, hm_copy_from_cpu, hm_copy_to_cpu,
    nullptr,
};

void hip_mem_tag(tensor_t *t)
{
    if (!is_hip_mem(t->mem))
        return;
    hip_mem_t *m = as_hip(t->mem);
    const size_t count = shape_count(&t->shape);
    if (m->layout == HIP_LAYOUT_NHWC_U8 && (size_t)m->N * m->C * m->H * m->W == count && m->size == count)
        return; // a view (reshape) of a tagged tensor keeps the producer's geometry
    const int nd = t->shape.dim_size;
    hip_layout_t layout = HIP_LAYOUT_RAW;
    int N = 0, C = 0, H = 1, W = 1;
    if ((t->dtype == dtUINT8 || t->dtype == dtINT8) && (nd == 4 || nd == 2)) { // one byte per element either way
        layout = HIP_LAYOUT_NHWC_U8;
        N = (int)t->shape.dim[0], C = (int)t->shape.dim[1];
        if (nd == 4)
            H = (int)t->shape.dim[2], W = (int)t->shape.dim[3];
    }
    if (layout != m->layout || N != m->N || C != m->C || H != m->H || W != m->W) {
        // geometry changed (first use, or a batch reshape): what the device holds is no longer addressable
        if (m->pending) { // a convolution that never launched: there is nothing to keep
            m->pending = nullptr;
            m->dev_valid = false;
        }
        if (m->dev_valid && !m->host_valid && m->dev) {
            wait_stream(m->prod_stream); // the producing kernels run on that workspace's stream
            download(m);
        }
        m->dev_valid = false;
        m->layout = layout;
        m->N = N, m->C = C, m->H = H, m->W = W;
        m->cs = layout == HIP_LAYOUT_NHWC_U8 ? hipq_channel_stride(C) : 0;
    }
}
