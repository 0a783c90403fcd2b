// Backend core: init / shutdown, buffers, flush, scratch arenas.
// Replaces the buffer and queue half of the reference's src/nn/fast_metal.m
// (:69-249): one device, one in-order stream, explicit HBM allocations.
#include "backend.h"
#include <string.h>
#include <vector>

namespace {
int         g_refcount = 0;
hipStream_t g_stream = nullptr;
int         g_num_cus = 0;
struct Arena { void *p = nullptr; size_t cap = 0; };
Arena       g_scratch[lmhip::SCR_COUNT];
}  // namespace

namespace lmhip {

hipStream_t stream() { return g_stream; }
int initialized() { return g_refcount > 0; }
int num_cus() { return g_num_cus; }

void die(const char *what, hipError_t e, const char *file, int line)
{
    fprintf(stderr, "[fast_hip] %s failed: %s (%s:%d)\n", what, hipGetErrorString(e), file, line);
    fflush(stderr);
    abort();
}

void *scratch(ScratchSlot slot, size_t bytes)
{
    Arena &a = g_scratch[slot];
    if (bytes > a.cap) {
        if (a.p) {                                   // kernels already enqueued may still read the old arena
            HIP_CHECK(hipStreamSynchronize(g_stream));
            HIP_CHECK(hipFree(a.p));
        }
        size_t cap = bytes + bytes / 4 + 4096;
        HIP_CHECK(hipMalloc(&a.p, cap));
        a.cap = cap;
    }
    return a.p;
}

}  // namespace lmhip

extern "C" {

int fast_metal_init(void)
{
    if (g_refcount > 0) { g_refcount++; return 0; }
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        fprintf(stderr, "[fast_hip] no HIP device available (%s); this library has no CPU path\n",
                e == hipSuccess ? "device count 0" : hipGetErrorString(e));
        return -1;
    }
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return -1;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return -1;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        fprintf(stderr, "[fast_hip] device %d is %s; kernels are built for gfx950 only\n", dev, prop.gcnArchName);
        return -1;
    }
    g_num_cus = prop.multiProcessorCount;
    if (hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking) != hipSuccess) {
        fprintf(stderr, "[fast_hip] stream creation failed\n");
        return -1;
    }
    g_refcount = 1;
    lmhip::noalloc_setup();                            // a failure is reported there and again by the entry point that needs it
    return 0;
}

void fast_metal_shutdown(void)
{
    if (g_refcount <= 0) return;
    if (--g_refcount > 0) return;
    hipStreamSynchronize(g_stream);
    for (auto &a : g_scratch) { if (a.p) hipFree(a.p); a.p = nullptr; a.cap = 0; }
    hipStreamDestroy(g_stream);
    g_stream = nullptr;
}

MetalBuf *metal_buf_create(size_t size)
{
    if (!lmhip::initialized()) { fprintf(stderr, "[fast_hip] metal_buf_create before fast_metal_init\n"); return nullptr; }
    MetalBuf *b = (MetalBuf *)calloc(1, sizeof(MetalBuf));
    b->size = size;
    b->owns = 1;
    HIP_CHECK(hipMalloc(&b->dev, size ? size : 4));
    return b;
}

MetalBuf *metal_buf_from_data(const void *data, size_t sz)
{
    MetalBuf *b = metal_buf_create(sz);
    if (b && sz) {
        // synchronous copy: the caller may free `data` as soon as this returns (src/nn/wmat.c:58-59)
        HIP_CHECK(hipMemcpyAsync(b->dev, data, sz, hipMemcpyHostToDevice, g_stream));
        HIP_CHECK(hipStreamSynchronize(g_stream));
    }
    return b;
}

MetalBuf *metal_buf_view(MetalBuf *parent, size_t offset, size_t size)
{
    if (!parent || offset + size > parent->size) return nullptr;
    MetalBuf *b = (MetalBuf *)calloc(1, sizeof(MetalBuf));
    b->dev = nullptr;              // resolved through the parent at every use
    while (parent->parent) { offset += parent->parent_off; parent = parent->parent; }
    b->size = size;
    b->owns = 0;
    b->parent = parent;
    b->parent_off = offset;
    return b;
}

void metal_buf_free(MetalBuf *b)
{
    if (!b) return;
    if (g_stream) hipStreamSynchronize(g_stream);
    for (auto &t : b->tiled) if (t.dev) hipFree(t.dev);
    if (b->owns) {
        if (b->host) hipHostFree(b->host);
        else if (b->dev) hipFree(b->dev);
    }
    free(b);
}

size_t metal_buf_size(MetalBuf *b) { return b ? b->size : 0; }

void *hip_buf_device_ptr(MetalBuf *b) { return b ? lmhip::dptr(b) : nullptr; }

void hip_mem_info(size_t *free_bytes, size_t *total_bytes)
{
    size_t f = 0, t = 0;
    HIP_CHECK(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
}

void *metal_buf_ptr(MetalBuf *b)
{
    if (!b) return nullptr;
    if (b->host) return b->host;
    if (!b->owns)                  // a view follows its parent into host memory (device side: lmhip::dptr)
        return (char *)metal_buf_ptr(b->parent) + b->parent_off;
    void *h = nullptr;
    HIP_CHECK(hipHostMalloc(&h, b->size ? b->size : 4, hipHostMallocMapped | hipHostMallocCoherent));
    HIP_CHECK(hipStreamSynchronize(g_stream));
    if (b->size) HIP_CHECK(hipMemcpy(h, b->dev, b->size, hipMemcpyDeviceToHost));
    HIP_CHECK(hipFree(b->dev));
    void *d = nullptr;
    HIP_CHECK(hipHostGetDevicePointer(&d, h, 0));
    b->dev = d;
    b->host = h;
    b->version++;                  // the CPU may now write it at any time: cached derivatives are void
    return h;
}

void metal_buf_read(MetalBuf *b, size_t offset, void *dst, size_t n)
{
    if (!b || offset + n > b->size) { fprintf(stderr, "[fast_hip] metal_buf_read out of range\n"); return; }
    HIP_CHECK(hipStreamSynchronize(g_stream));
    MetalBuf *root = b->parent ? b->parent : b;
    size_t off = offset + (b->parent ? b->parent_off : 0);
    if (root->host) memcpy(dst, (char *)root->host + off, n);
    else HIP_CHECK(hipMemcpy(dst, (char *)root->dev + off, n, hipMemcpyDeviceToHost));
}

void metal_buf_write(MetalBuf *b, size_t offset, const void *src, size_t n)
{
    if (!b || offset + n > b->size) { fprintf(stderr, "[fast_hip] metal_buf_write out of range\n"); return; }
    HIP_CHECK(hipStreamSynchronize(g_stream));
    MetalBuf *root = b->parent ? b->parent : b;
    size_t off = offset + (b->parent ? b->parent_off : 0);
    if (root->host) memcpy((char *)root->host + off, src, n);
    else HIP_CHECK(hipMemcpy((char *)root->dev + off, src, n, hipMemcpyHostToDevice));
    lmhip::mark_written(b);
}

void metal_flush(void)
{
    if (!g_stream) return;
    HIP_CHECK(hipStreamSynchronize(g_stream));
}

}  // extern "C"
