// Driver layer of libw4a16hip.so: context, code-object loading, launches, memory, events.
// Stands in for CudaCtx over the dlopen'ed CUDA driver table in the reference
// (crates/backend-gpu/src/rawcuda/ffi.rs:237-459, ctx/mod.rs:62-419, ctx/mem.rs, ctx/prof.rs, assets.rs).
#include <dlfcn.h>

#include <algorithm>
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "w4a16_internal.h"

// ------------------------------------------------------------------------------------------------ errors
static thread_local char g_err[512] = "";

extern "C" const char* w4a16_last_error(void) { return g_err; }

int w4_fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    int off = snprintf(g_err, sizeof g_err, "w4a16hip: ");
    vsnprintf(g_err + off, sizeof g_err - (size_t)off, fmt, ap);
    va_end(ap);
    return code;
}

std::string w4_err_save() { return std::string(g_err); }

void w4_err_restore(const std::string& msg) {
    strncpy(g_err, msg.c_str(), sizeof g_err - 1);
    g_err[sizeof g_err - 1] = 0;
}

int w4_hip(hipError_t e, const char* api) {
    if (e == hipSuccess) return 0;
    return w4_fail((int)e, "%s: %s (%d)", api, hipGetErrorString(e), (int)e);
}

// ------------------------------------------------------------------------------------------------ manifest
// Asset registry: code object name -> kernel symbols.  Counterpart of assets.rs:276-334 / FATBINS.manifest; a test
// checks that these lists equal the extern "C" __global__ symbols of the kernel sources (assets.rs:394-443).
static const char* const kLaneSyms[] = {"w4a16_lane_g128_f16", "w4a16_lane_g128_bf16", "w4a16_lane_g32_f16",
                                        "w4a16_lane_g32_bf16", nullptr};
static const char* const kLayoutSyms[] = {"w4a16_tile_q",         "w4a16_tile_s",          "w4a16_untile_q",
                                          "w4a16_untile_s",       "w4a16_dump_tiled_f16",  "w4a16_dump_tiled_bf16",
                                          "w4a16_dump_raw_f16",   "w4a16_dump_raw_bf16",   "w4a16_row_norm_max_f16",
                                          "w4a16_row_norm_max_bf16", nullptr};
static const char* const kDecodeSyms[] = {
    "w4a16_decode_g128_f16_rb1_x1", "w4a16_decode_g128_f16_rb1_x2", "w4a16_decode_g128_f16_rb1_x4",
    "w4a16_decode_g128_f16_rb2_x1", "w4a16_decode_g128_f16_rb2_x2", "w4a16_decode_g128_f16_rb2_x4",
    "w4a16_decode_g128_f16_rb4_x1", "w4a16_decode_g128_f16_rb4_x2", "w4a16_decode_g128_f16_rb4_x4",
    "w4a16_decode_g128_bf16_rb1_x1", "w4a16_decode_g128_bf16_rb1_x2", "w4a16_decode_g128_bf16_rb1_x4",
    "w4a16_decode_g128_bf16_rb2_x1", "w4a16_decode_g128_bf16_rb2_x2", "w4a16_decode_g128_bf16_rb2_x4",
    "w4a16_decode_g128_bf16_rb4_x1", "w4a16_decode_g128_bf16_rb4_x2", "w4a16_decode_g128_bf16_rb4_x4",
    "w4a16_decode_g32_f16_rb1_x1", "w4a16_decode_g32_f16_rb1_x2", "w4a16_decode_g32_f16_rb1_x4",
    "w4a16_decode_g32_f16_rb2_x1", "w4a16_decode_g32_f16_rb2_x2", "w4a16_decode_g32_f16_rb2_x4",
    "w4a16_decode_g32_f16_rb4_x1", "w4a16_decode_g32_f16_rb4_x2", "w4a16_decode_g32_f16_rb4_x4",
    "w4a16_decode_g32_bf16_rb1_x1", "w4a16_decode_g32_bf16_rb1_x2", "w4a16_decode_g32_bf16_rb1_x4",
    "w4a16_decode_g32_bf16_rb2_x1", "w4a16_decode_g32_bf16_rb2_x2", "w4a16_decode_g32_bf16_rb2_x4",
    "w4a16_decode_g32_bf16_rb4_x1", "w4a16_decode_g32_bf16_rb4_x2", "w4a16_decode_g32_bf16_rb4_x4",
    "w4a16_decode_g128_f16_glu_x1", "w4a16_decode_g128_f16_glu_x2", "w4a16_decode_g128_f16_glu_x4",
    "w4a16_decode_g128_bf16_glu_x1", "w4a16_decode_g128_bf16_glu_x2", "w4a16_decode_g128_bf16_glu_x4",
    "w4a16_decode_g32_f16_glu_x1", "w4a16_decode_g32_f16_glu_x2", "w4a16_decode_g32_f16_glu_x4",
    "w4a16_decode_g32_bf16_glu_x1", "w4a16_decode_g32_bf16_glu_x2", "w4a16_decode_g32_bf16_glu_x4",
    "w4a16_decode_g128_f16_multi_x1", "w4a16_decode_g128_f16_multi_x2", "w4a16_decode_g128_f16_multi_x4",
    "w4a16_decode_g128_bf16_multi_x1", "w4a16_decode_g128_bf16_multi_x2", "w4a16_decode_g128_bf16_multi_x4",
    "w4a16_decode_g32_f16_multi_x1", "w4a16_decode_g32_f16_multi_x2", "w4a16_decode_g32_f16_multi_x4",
    "w4a16_decode_g32_bf16_multi_x1", "w4a16_decode_g32_bf16_multi_x2", "w4a16_decode_g32_bf16_multi_x4",
    nullptr};
static const char* const kPrefillG128Syms[] = {
    "w4a16_prefill_g128_f16", "w4a16_prefill_g128_bf16", "w4a16_prefill_g128_f16_m64", "w4a16_prefill_g128_bf16_m64",
    "w4a16_prefill_g128_f16_m96", "w4a16_prefill_g128_bf16_m96", "w4a16_prefill_g128_f16_glu", "w4a16_prefill_g128_bf16_glu",
    "w4a16_prefill_g128_f16_m64_glu", "w4a16_prefill_g128_bf16_m64_glu", "w4a16_prefill_g128_f16_m96_glu",
    "w4a16_prefill_g128_bf16_m96_glu", nullptr};
static const char* const kPrefillSyms[] = {"w4a16_prefill_g32_f16", "w4a16_prefill_g32_bf16", "w4a16_prefill_g32_f16_m64",
                                           "w4a16_prefill_g32_bf16_m64", "w4a16_prefill_splitk_sum", "w4a16_prefill_splitk_finish",
                                           "w4a16_prefill_g32_f16_glu", "w4a16_prefill_g32_bf16_glu",
                                           "w4a16_prefill_g32_f16_m64_glu", "w4a16_prefill_g32_bf16_m64_glu",
                                           "w4a16_prefill_g32_f16_m96", "w4a16_prefill_g32_bf16_m96",
                                           "w4a16_prefill_g32_f16_m96_glu", "w4a16_prefill_g32_bf16_m96_glu",
                                           "w4a16_moe_g128_f16_pf_glu", "w4a16_moe_g128_f16_pf_lin", "w4a16_moe_g128_bf16_pf_glu",
                                           "w4a16_moe_g128_bf16_pf_lin", "w4a16_moe_g32_f16_pf_glu", "w4a16_moe_g32_f16_pf_lin",
                                           "w4a16_moe_g32_bf16_pf_glu", "w4a16_moe_g32_bf16_pf_lin", nullptr};
static const char* const kUtilSyms[] = {"w4a16_fill0_u32", nullptr};
static const char* const kGlueSyms[] = {"w4a16_rms_rescale_f16", "w4a16_silu_mul_f16", "w4a16_synth_q", "w4a16_synth_s",
                                        "w4a16_norm_resid", nullptr};
#define W4_MOE_FAMILY(P)                                                                                      \
    P "_dec_glu_x1", P "_dec_glu_x4", P "_dec_lin_x1", P "_dec_lin_x4", P "_mm_glu_t1", P "_mm_glu_t2",       \
        P "_mm_glu_t3", P "_mm_glu_t4", P "_mm_lin_t1", P "_mm_lin_t2", P "_mm_lin_t3", P "_mm_lin_t4",       \
        P "_mm_lin_t1_ks", P "_mm_lin_t2_ks", P "_mm_lin_t3_ks", P "_mm_lin_t4_ks"
static const char* const kMoeSyms[] = {W4_MOE_FAMILY("w4a16_moe_g32_f16"),
                                       W4_MOE_FAMILY("w4a16_moe_g32_bf16"),
                                       W4_MOE_FAMILY("w4a16_moe_g128_f16"),
                                       W4_MOE_FAMILY("w4a16_moe_g128_bf16"),
                                       "w4a16_moe_g32_f16_down_sum",
                                       "w4a16_moe_g32_bf16_down_sum",
                                       "w4a16_moe_g128_f16_down_sum",
                                       "w4a16_moe_g128_bf16_down_sum",
                                       "w4a16_moe_g32_f16_down_sum1",
                                       "w4a16_moe_g32_bf16_down_sum1",
                                       "w4a16_moe_g128_f16_down_sum1",
                                       "w4a16_moe_g128_bf16_down_sum1",
                                       "w4a16_moe_topk_t",
                                       "w4a16_moe_align",
                                       "w4a16_moe_topk_sum_f16",
                                       nullptr};

struct W4Asset {
    const char* name;
    const char* const* syms;
};
static const W4Asset kAssets[] = {
    {"lane", kLaneSyms},
    {"layout", kLayoutSyms},
    {"decode", kDecodeSyms},
    {"prefill", kPrefillSyms},
    {"prefill_g128", kPrefillG128Syms},
    {"moe", kMoeSyms},
    {"glue", kGlueSyms},
    {"util", kUtilSyms},
};
static const size_t kAssetCount = sizeof kAssets / sizeof kAssets[0];

extern "C" size_t w4a16_manifest(size_t asset, const char** name, const char* const** symbols) {
    if (asset < kAssetCount) {
        if (name) *name = kAssets[asset].name;
        if (symbols) *symbols = kAssets[asset].syms;
    }
    return kAssetCount;
}

static std::string default_asset_dir() {
    Dl_info info;
    if (dladdr((void*)&w4a16_last_error, &info) && info.dli_fname) {
        std::string p(info.dli_fname);
        size_t slash = p.rfind('/');
        return (slash == std::string::npos ? std::string(".") : p.substr(0, slash)) + "/assets";
    }
    return "assets";
}

static int read_file(const std::string& path, std::vector<char>* out) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) return w4_fail(W4A16_ERR_ASSET, "asset: cannot open %s (build the gfx950 code objects first)", path.c_str());
    fseek(f, 0, SEEK_END);
    long sz = ftell(f);
    fseek(f, 0, SEEK_SET);
    out->resize(sz > 0 ? (size_t)sz : 0);
    size_t got = sz > 0 ? fread(out->data(), 1, (size_t)sz, f) : 0;
    fclose(f);
    if (sz <= 0 || got != (size_t)sz) return w4_fail(W4A16_ERR_ASSET, "asset: short read on %s", path.c_str());
    return 0;
}

// ------------------------------------------------------------------------------------------------ context
extern "C" int w4a16_module_load(w4a16_ctx* ctx, const char* key, const void* image, size_t len,
                                 const char* const* symbols, size_t nsym) {
    if (!ctx || !key || !image || len == 0 || (nsym && !symbols)) return w4_fail(W4A16_ERR_ARG, "module_load: null argument");
    for (size_t i = 0; i < nsym; i++)
        if (!symbols[i]) return w4_fail(W4A16_ERR_ARG, "module_load(%s): symbol %zu is null", key, i);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    hipModule_t mod = nullptr;
    hipError_t e = hipModuleLoadData(&mod, image);
    if (e != hipSuccess) {
        // the reference's hint on load failure is an architecture mismatch (ctx/mod.rs:207-210)
        return w4_fail((int)e, "hipModuleLoadData(%s): %s (%d) — the code object must be built for gfx950", key,
                       hipGetErrorString(e), (int)e);
    }
    std::vector<std::pair<std::string, hipFunction_t>> found;
    for (size_t i = 0; i < nsym; i++) {
        hipFunction_t f = nullptr;
        e = hipModuleGetFunction(&f, mod, symbols[i]);
        if (e != hipSuccess || !f) {
            hipModuleUnload(mod);
            return w4_fail(W4A16_ERR_SYMBOL, "module_load(%s): symbol %s not in the code object (%s)", key, symbols[i],
                           hipGetErrorString(e));
        }
        found.emplace_back(symbols[i], f);
    }
    ctx->modules.push_back(mod);
    for (auto& p : found) ctx->functions[p.first] = p.second;
    return 0;
}

extern "C" int w4a16_ctx_create(int device_ordinal, const char* asset_dir, w4a16_ctx** out) {
    if (!out) return w4_fail(W4A16_ERR_ARG, "ctx_create: out is null");
    *out = nullptr;
    W4_TRY(w4_hip(hipInit(0), "hipInit"));
    int count = 0;
    W4_TRY(w4_hip(hipGetDeviceCount(&count), "hipGetDeviceCount"));
    if (device_ordinal < 0 || device_ordinal >= count)
        return w4_fail(W4A16_ERR_ARG, "ctx_create: device %d of %d", device_ordinal, count);
    W4_TRY(w4_hip(hipSetDevice(device_ordinal), "hipSetDevice"));
    w4a16_ctx* ctx = new w4a16_ctx();
    ctx->device = device_ordinal;
    hipDeviceProp_t prop;
    int rc = w4_hip(hipGetDeviceProperties(&prop, device_ordinal), "hipGetDeviceProperties");
    if (!rc && strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        rc = w4_fail(W4A16_ERR_UNSUPPORTED, "ctx_create: device is %s; the kernels are built for gfx950 only",
                     prop.gcnArchName);
    if (!rc) ctx->cu_count = prop.multiProcessorCount;
    // both streams non-blocking, default priority (reference: flag 1 = CU_STREAM_NON_BLOCKING, ctx/mod.rs:366-396)
    if (!rc) rc = w4_hip(hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking), "hipStreamCreateWithFlags");
    if (!rc) rc = w4_hip(hipStreamCreateWithFlags(&ctx->stream2, hipStreamNonBlocking), "hipStreamCreateWithFlags");
    std::string dir = asset_dir ? std::string(asset_dir) : default_asset_dir();
    for (size_t a = 0; a < kAssetCount && !rc; a++) {
        std::string env = "LLM170_HIP_";
        for (const char* c = kAssets[a].name; *c; c++) env.push_back((char)toupper((unsigned char)*c));
        env += "_HSACO_PATH";
        const char* over = getenv(env.c_str());
        std::string path = over && *over ? std::string(over) : dir + "/" + kAssets[a].name + ".hsaco";
        std::vector<char> image;
        rc = read_file(path, &image);
        if (rc) break;
        size_t nsym = 0;
        while (kAssets[a].syms[nsym]) nsym++;
        rc = w4a16_module_load(ctx, kAssets[a].name, image.data(), image.size(), kAssets[a].syms, nsym);
    }
    if (!rc) rc = w4_noalloc_init(ctx);
    if (rc) {
        const std::string keep = w4_err_save();
        w4a16_ctx_destroy(ctx);
        w4_err_restore(keep);
        return rc;
    }
    *out = ctx;
    return 0;
}

extern "C" void w4a16_ctx_destroy(w4a16_ctx* ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->capturing) {  // a capture left open: end it and drop what it recorded
        hipGraph_t dangling = nullptr;
        (void)hipStreamEndCapture(ctx->stream, &dangling);
        if (dangling) (void)hipGraphDestroy(dangling);
        ctx->capturing = false;
    }
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (ctx->stream2) (void)hipStreamSynchronize(ctx->stream2);
    w4_noalloc_release(ctx);
    for (auto& a : ctx->allocs) (void)hipFree((void*)a.first);
    for (auto m : ctx->modules) (void)hipModuleUnload(m);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    if (ctx->stream2) (void)hipStreamDestroy(ctx->stream2);
    delete ctx;
}

extern "C" int w4a16_has_symbol(w4a16_ctx* ctx, const char* symbol) {
    if (!ctx || !symbol) return w4_fail(W4A16_ERR_ARG, "has_symbol: null argument");
    if (ctx->functions.find(std::string_view(symbol)) == ctx->functions.end())
        return w4_fail(W4A16_ERR_SYMBOL, "function: symbol %s is not loaded", symbol);
    return 0;
}

int w4_launch(w4a16_ctx* ctx, const char* symbol, unsigned gx, unsigned gy, unsigned block, unsigned shmem,
              void** params) {
    auto it = ctx->functions.find(std::string_view(symbol));
    if (it == ctx->functions.end()) return w4_fail(W4A16_ERR_SYMBOL, "function: symbol %s is not loaded", symbol);
    if (gx == 0 || gy == 0 || block == 0 || block > 1024)
        return w4_fail(W4A16_ERR_ARG, "launch %s: grid %ux%u block %u", symbol, gx, gy, block);
    hipError_t e = hipSuccess;
    if (shmem > 64 * 1024) {  // beyond the default limit on dynamic LDS the function has to be told (gfx950: 160 KiB)
        if (shmem > 160 * 1024) return w4_fail(W4A16_ERR_ARG, "launch %s: %u bytes of LDS", symbol, shmem);
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(it->second), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)shmem);
        if (e != hipSuccess)
            return w4_fail((int)e, "hipFuncSetAttribute(%s, dynamic LDS %u): %s (%d)", symbol, shmem, hipGetErrorString(e),
                           (int)e);
    }
    ctx->last_symbol = it->first.c_str();
    e = hipModuleLaunchKernel(it->second, gx, gy, 1, block, 1, 1, shmem, ctx->stream, params, nullptr);
    if (e != hipSuccess)
        return w4_fail((int)e, "hipModuleLaunchKernel(%s grid %ux%u block %u shmem %u): %s (%d)", symbol, gx, gy, block,
                       shmem, hipGetErrorString(e), (int)e);
    return 0;
}

extern "C" const char* w4a16_last_launch_symbol(w4a16_ctx* ctx) { return ctx ? ctx->last_symbol : ""; }

extern "C" int w4a16_launch(w4a16_ctx* ctx, const char* symbol, unsigned gx, unsigned gy, unsigned block,
                            unsigned shmem, void** params) {
    if (!ctx || !symbol || !params) return w4_fail(W4A16_ERR_ARG, "launch: null argument");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    return w4_launch(ctx, symbol, gx, gy, block, shmem, params);
}

// ------------------------------------------------------------------------------------------------ memory
extern "C" int w4a16_alloc(w4a16_ctx* ctx, size_t bytes, uint64_t* dptr) {
    if (!ctx || !dptr) return w4_fail(W4A16_ERR_ARG, "alloc: null argument");
    *dptr = 0;
    if (bytes == 0) return w4_fail(W4A16_ERR_ARG, "alloc: zero bytes");
    if (ctx->capturing)
        return w4_fail(W4A16_ERR_ARG, "alloc(%zu) while the launch stream is capturing: run the sequence once before the capture so that every scratch buffer has its size", bytes);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) return w4_fail((int)e, "hipMalloc(%zu): %s (%d)", bytes, hipGetErrorString(e), (int)e);
    ctx->allocs[(uint64_t)p] = bytes;
    ctx->allocated += bytes;
    *dptr = (uint64_t)p;
    return 0;
}

extern "C" int w4a16_free(w4a16_ctx* ctx, uint64_t dptr) {
    if (!ctx) return w4_fail(W4A16_ERR_ARG, "free: null context");
    if (dptr == 0) return 0;
    auto it = ctx->allocs.find(dptr);
    if (it == ctx->allocs.end()) return w4_fail(W4A16_ERR_ARG, "free: %#llx was not allocated by this context",
                                                (unsigned long long)dptr);
    if (ctx->capturing) return w4_fail(W4A16_ERR_ARG, "free while the launch stream is capturing");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    // work queued on the launch stream may still use the buffer
    W4_TRY(w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"));
    ctx->allocated -= it->second;
    ctx->allocs.erase(it);
    return w4_hip(hipFree((void*)dptr), "hipFree");
}

extern "C" size_t w4a16_allocated_bytes(w4a16_ctx* ctx) { return ctx ? ctx->allocated : 0; }

extern "C" int w4a16_h2d(w4a16_ctx* ctx, uint64_t dst, const void* src, size_t bytes) {
    if (!ctx || !dst || !src) return w4_fail(W4A16_ERR_ARG, "h2d: null argument");
    if (bytes == 0) return 0;
    if (ctx->capturing) return w4_fail(W4A16_ERR_ARG, "h2d while the launch stream is capturing");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    W4_TRY(w4_hip(hipMemcpyAsync((void*)dst, src, bytes, hipMemcpyHostToDevice, ctx->stream), "hipMemcpyAsync(h2d)"));
    return w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

extern "C" int w4a16_d2h(w4a16_ctx* ctx, void* dst, uint64_t src, size_t bytes) {
    if (!ctx || !dst || !src) return w4_fail(W4A16_ERR_ARG, "d2h: null argument");
    if (bytes == 0) return 0;
    if (ctx->capturing) return w4_fail(W4A16_ERR_ARG, "d2h while the launch stream is capturing");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    W4_TRY(w4_hip(hipMemcpyAsync(dst, (const void*)src, bytes, hipMemcpyDeviceToHost, ctx->stream), "hipMemcpyAsync(d2h)"));
    return w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

extern "C" int w4a16_d2d(w4a16_ctx* ctx, uint64_t dst, uint64_t src, size_t bytes) {
    if (!ctx || !dst || !src) return w4_fail(W4A16_ERR_ARG, "d2d: null argument");
    if (bytes == 0) return 0;
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    return w4_hip(hipMemcpyAsync((void*)dst, (const void*)src, bytes, hipMemcpyDeviceToDevice, ctx->stream),
                  "hipMemcpyAsync(d2d)");
}

extern "C" int w4a16_memset0(w4a16_ctx* ctx, uint64_t dst, size_t bytes) {
    if (!ctx || !dst) return w4_fail(W4A16_ERR_ARG, "memset0: null argument");
    if (bytes == 0) return 0;
    if ((dst & 3) || (bytes & 3)) return w4_fail(W4A16_ERR_ARG, "memset0: address and size must be multiples of 4");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    // a fill kernel rather than a memset node: memset nodes are not replay-safe inside captured graphs here
    size_t words = bytes / 4;
    unsigned grid = (unsigned)std::min<size_t>((words + 255) / 256, 4096);
    void* params[] = {&dst, &words};
    return w4_launch(ctx, "w4a16_fill0_u32", grid, 1, 256, 0, params);
}

extern "C" int w4a16_sync(w4a16_ctx* ctx) {
    if (!ctx) return w4_fail(W4A16_ERR_ARG, "sync: null context");
    if (ctx->capturing) return w4_fail(W4A16_ERR_ARG, "sync while the launch stream is capturing");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    return w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
}

// ------------------------------------------------------------------------------------------------ graphs
// Capture of the launch stream into a HIP graph (reference: CudaCtx::capture_begin / capture_end / graph_instantiate /
// graph_upload / graph_launch / graph_destroy, ctx/graph.rs:4-85).  Between begin and end every launch entry point of
// this library records a kernel node instead of running; nothing may allocate, free, copy to or from the host or wait
// (the entry points that would refuse).  Clearing memory inside a capture goes through the fill kernel of
// w4a16_memset0, never a memset node.
extern "C" int w4a16_capture_begin(w4a16_ctx* ctx) {
    if (!ctx) return w4_fail(W4A16_ERR_ARG, "capture_begin: null context");
    if (ctx->capturing) return w4_fail(W4A16_ERR_ARG, "capture_begin: the launch stream is capturing already");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    W4_TRY(w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"));
    W4_TRY(w4_hip(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture"));
    ctx->capturing = true;
    return 0;
}

extern "C" int w4a16_capture_end(w4a16_ctx* ctx, w4a16_graph** out) {
    if (!ctx || !out) return w4_fail(W4A16_ERR_ARG, "capture_end: null argument");
    *out = nullptr;
    if (!ctx->capturing) return w4_fail(W4A16_ERR_ARG, "capture_end: the launch stream is not capturing");
    ctx->capturing = false;
    w4a16_graph* g = new w4a16_graph();
    int rc = w4_hip(hipStreamEndCapture(ctx->stream, &g->graph), "hipStreamEndCapture");
    if (!rc && !g->graph) rc = w4_fail(W4A16_ERR_ARG, "capture_end: the capture was invalidated");
    if (!rc) rc = w4_hip(hipGraphGetNodes(g->graph, nullptr, &g->nodes), "hipGraphGetNodes");
    if (!rc && g->nodes == 0) rc = w4_fail(W4A16_ERR_ARG, "capture_end: nothing was launched between begin and end");
    if (!rc) rc = w4_hip(hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0), "hipGraphInstantiate");
    if (!rc) rc = w4_hip(hipGraphUpload(g->exec, ctx->stream), "hipGraphUpload");
    g->scratch_gen = ctx->scratch_gen;
    if (rc) {
        const std::string keep = w4_err_save();
        w4a16_graph_destroy(ctx, g);
        w4_err_restore(keep);
        return rc;
    }
    *out = g;
    return 0;
}

extern "C" int w4a16_graph_launch(w4a16_ctx* ctx, w4a16_graph* g) {
    if (!ctx || !g || !g->exec) return w4_fail(W4A16_ERR_ARG, "graph_launch: null argument");
    if (ctx->capturing) return w4_fail(W4A16_ERR_ARG, "graph_launch while the launch stream is capturing");
    if (g->scratch_gen != ctx->scratch_gen)
        return w4_fail(W4A16_ERR_STALE_GRAPH, "graph_launch: a scratch buffer of the context was replaced by a larger one after this graph was captured (generation %llu, now %llu); its nodes hold the freed address: capture again",
                       (unsigned long long)g->scratch_gen, (unsigned long long)ctx->scratch_gen);
    return w4_hip(hipGraphLaunch(g->exec, ctx->stream), "hipGraphLaunch");
}

extern "C" size_t w4a16_graph_nodes(const w4a16_graph* g) { return g ? g->nodes : 0; }

extern "C" void w4a16_graph_destroy(w4a16_ctx* ctx, w4a16_graph* g) {
    if (!g) return;
    if (ctx) {
        (void)hipSetDevice(ctx->device);
        if (ctx->stream && !ctx->capturing) (void)hipStreamSynchronize(ctx->stream);  // a replay may still be running
    }
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
}

// ------------------------------------------------------------------------------------------------ events
extern "C" int w4a16_event_create(w4a16_ctx* ctx, w4a16_event** out) {
    if (!ctx || !out) return w4_fail(W4A16_ERR_ARG, "event_create: null argument");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    w4a16_event* ev = new w4a16_event();
    int rc = w4_hip(hipEventCreate(&ev->ev), "hipEventCreate");
    if (rc) {
        delete ev;
        return rc;
    }
    *out = ev;
    return 0;
}

extern "C" int w4a16_event_record(w4a16_ctx* ctx, w4a16_event* ev) {
    if (!ctx || !ev) return w4_fail(W4A16_ERR_ARG, "event_record: null argument");
    return w4_hip(hipEventRecord(ev->ev, ctx->stream), "hipEventRecord");
}

extern "C" int w4a16_event_elapsed_ms(w4a16_ctx* ctx, w4a16_event* start, w4a16_event* stop, float* ms) {
    if (!ctx || !start || !stop || !ms) return w4_fail(W4A16_ERR_ARG, "event_elapsed_ms: null argument");
    W4_TRY(w4_hip(hipEventSynchronize(stop->ev), "hipEventSynchronize"));
    return w4_hip(hipEventElapsedTime(ms, start->ev, stop->ev), "hipEventElapsedTime");
}

extern "C" void w4a16_event_destroy(w4a16_ctx* ctx, w4a16_event* ev) {
    (void)ctx;
    if (!ev) return;
    (void)hipEventDestroy(ev->ev);
    delete ev;
}
