// The allocation-free entry point of libw4a16hip.so and the fixed device scratch behind it.
//
// w4a16_lin_forward may allocate: a decode launch that splits k across workgroups parks partial tiles in a workspace the
// context grows on demand (hipMalloc), and looks its tickets up there.  Callers that cannot allocate — code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc — get w4a16_lin_forward_noalloc, the same decode
// launch with that workspace in a file-scope device array of fixed size.  This is the one source file of the host
// library compiled by hipcc: the array lives in the library's own device image, one copy per GPU, held until the
// process ends.
#include <hip/hip_runtime.h>

#include <mutex>

#include "w4a16_internal.h"

#define W4_NOALLOC_WS_BYTES (8u << 20)       // partial tiles: workgroups x row blocks per wave x 1 KiB x k slices
#define W4_NOALLOC_TICKET_BYTES (64u << 10)  // one int per workgroup of a slice
#define W4_NOALLOC_MAX_DEVICES 64

static __device__ __align__(256) unsigned char scratch[W4_NOALLOC_WS_BYTES + W4_NOALLOC_TICKET_BYTES];

// Device address of each GPU's copy of the array.  In host code the array's name is only a handle for
// hipGetSymbolAddress; every use of the memory goes through the address obtained here.
static void* g_scratch_ptr[W4_NOALLOC_MAX_DEVICES];
// The context that uses each GPU's array.  Partial tiles and tickets of two contexts would mix (either could draw the
// last ticket early and sum the other's tiles), so the first caller on a GPU owns its array until it is destroyed.
static w4a16_ctx* g_scratch_owner[W4_NOALLOC_MAX_DEVICES];
static std::mutex g_owner_lock;

extern "C" size_t w4a16_noalloc_workspace_bytes(void) { return W4_NOALLOC_WS_BYTES; }

// Once per device, with that device current (called from w4a16_ctx_create).  The array is zero when the device image
// is loaded; the tickets are all the entry point needs at zero, and every launch leaves them at zero again.
int w4_noalloc_init(w4a16_ctx* ctx) {
    if (ctx->device < 0 || ctx->device >= W4_NOALLOC_MAX_DEVICES)
        return w4_fail(W4A16_ERR_ARG, "noalloc: device ordinal %d beyond %d", ctx->device, W4_NOALLOC_MAX_DEVICES);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    if (!g_scratch_ptr[ctx->device]) {
        void* ptr = nullptr;
        W4_TRY(w4_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)"));
        if (!ptr) return w4_fail(W4A16_ERR_ARG, "noalloc: hipGetSymbolAddress returned a null address");
        size_t bytes = 0;
        W4_TRY(w4_hip(hipGetSymbolSize(&bytes, HIP_SYMBOL(scratch)), "hipGetSymbolSize(scratch)"));
        if (bytes != W4_NOALLOC_WS_BYTES + W4_NOALLOC_TICKET_BYTES)
            return w4_fail(W4A16_ERR_ARG, "noalloc: scratch symbol is %zu bytes", bytes);
        g_scratch_ptr[ctx->device] = ptr;
    }
    ctx->fixed_scratch = (uint64_t)g_scratch_ptr[ctx->device];
    return 0;
}

// Called when a context is destroyed: its GPU's array is free for the next caller.
void w4_noalloc_release(w4a16_ctx* ctx) {
    if (ctx->device < 0 || ctx->device >= W4_NOALLOC_MAX_DEVICES) return;
    std::lock_guard<std::mutex> hold(g_owner_lock);
    if (g_scratch_owner[ctx->device] == ctx) g_scratch_owner[ctx->device] = nullptr;
}

extern "C" int w4a16_lin_forward_noalloc(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t y_dev, size_t t,
                                         int out_f16) {
    if (!ctx || !name) return w4_fail(W4A16_ERR_ARG, "lin_forward_noalloc: null argument");
    if (!ctx->fixed_scratch) return w4_fail(W4A16_ERR_ARG, "lin_forward_noalloc: the fixed scratch was not set up");
    {
        std::lock_guard<std::mutex> hold(g_owner_lock);  // no allocation: a mutex and two pointer compares
        w4a16_ctx*& owner = g_scratch_owner[ctx->device];
        if (!owner) owner = ctx;
        if (owner != ctx)
            return w4_fail(W4A16_ERR_ARG, "lin_forward_noalloc: the fixed scratch of GPU %d is in use by another context (one context per GPU may use this entry point until it is destroyed)", ctx->device);
    }
    const uint64_t ws = ctx->fixed_scratch, tickets = ctx->fixed_scratch + W4_NOALLOC_WS_BYTES;
    return w4_lin_forward_fixed_ws(ctx, name, x_dev, y_dev, t, out_f16, ws, W4_NOALLOC_WS_BYTES, tickets,
                                   W4_NOALLOC_TICKET_BYTES);
}
