// Internal state of libw4a16hip.so shared by the driver layer (w4a16_ctx.cc) and the operator layer (w4a16_ops.cc).
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdint>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

#include "w4a16_hip.h"

// One registered linear: the operands as given (raw) and the tiled copy (see kernels/w4a16_common.hpp).
// Counterpart of the reference's weight maps lins / lin_grp / lins_mk / lins_msc
// (crates/backend-gpu/src/rawcuda/w4a16_dec/mod.rs:547-556).
struct W4Lin {
    uint64_t q_raw = 0, s_raw = 0;      // u32 [n][k/8], u16 [n][k/group]
    uint64_t q_tiled = 0, s_tiled = 0;  // 1 KiB tiles [row_blocks][k/128], u16 [row_blocks][k/group][16]
    size_t n = 0, k = 0, group = 0;
    int scale_bf16 = 0;
    size_t row_blocks = 0;
    bool scales_regular = true;  // every scale finite and non-zero (the MFMA prefill kernel divides by them)
};

struct w4a16_event {
    hipEvent_t ev;
};

struct w4a16_ctx {
    int device = 0;
    hipStream_t stream = nullptr;   // launch stream (reference: CudaCtx.stream)
    hipStream_t stream2 = nullptr;  // second stream (reference: CudaCtx.stream2); copies that must not serialise
    std::vector<hipModule_t> modules;
    std::unordered_map<std::string, hipFunction_t> functions;
    std::unordered_map<uint64_t, size_t> allocs;
    size_t allocated = 0;
    std::map<std::string, W4Lin> lins;
    int decode_rows_per_wave = 0, decode_waves_per_block = 0;  // 0 = automatic
    int cu_count = 0;
};

int w4_fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int w4_hip(hipError_t e, const char* api);
// Keep the message of a failing step across clean-up calls that may fail themselves.
std::string w4_err_save();
void w4_err_restore(const std::string& msg);
int w4_launch(w4a16_ctx* ctx, const char* symbol, unsigned gx, unsigned gy, unsigned block, unsigned shmem,
              void** params);

#define W4_TRY(expr)          \
    do {                      \
        int rc__ = (expr);    \
        if (rc__) return rc__; \
    } while (0)
