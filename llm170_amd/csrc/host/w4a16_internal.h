// Internal state of libw4a16hip.so shared by the driver layer (w4a16_ctx.cc) and the operator layer (w4a16_ops.cc).
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdint>
#include <array>
#include <map>
#include <string>
#include <string_view>
#include <tuple>
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
    float row_norm_max = -1.0f;  // largest row norm of the dequantised weights, computed on first request (< 0: not yet)
    std::vector<size_t> part_n;  // a fused linear: the rows of each part, in order (empty for a linear uploaded as one)
};

// The experts of one MoE layer: two arenas in the tiled layout, experts at a fixed stride
// (reference: moe_m13 / moe_s13 / moe_m2 / moe_s2, w4a16_dec/upload.rs:1116-1235).
struct W4Experts {
    uint64_t q13 = 0, s13 = 0, q2 = 0, s2 = 0;
    size_t n_exp = 0, h = 0, n_ff = 0, group = 0;
    int scale_bf16 = 0;
    size_t q13_stride = 0, s13_stride = 0, q2_stride = 0, s2_stride = 0;  // bytes per expert
    bool scales_regular = true;  // same rule as W4Lin::scales_regular, over both arenas: the MFMA-tiled grouped kernels need it
};

// Scratch of the MoE FFN, grown on demand (reference: moe_msorted / moe_mexp / moe_mnpost / moe_mact / moe_mc2,
// kernels/marlin_moe.rs:322-342).
struct W4MoeScratch {
    uint64_t sorted = 0, expert_ids = 0, num_post = 0, act = 0, c2 = 0;
    size_t sorted_cap = 0, expert_cap = 0, act_cap = 0, c2_cap = 0;       // bytes
    size_t sorted_len = 0, expert_len = 0, act_len = 0, c2_len = 0;       // bytes used by the last call
    size_t block = 0;
    uint64_t iota = 0, always = 0;  // direct mode: identity segment table and a "padded total" no slot index reaches
    size_t iota_cap = 0;            // entries
    uint64_t zeros = 0;             // all-zero expert table for a dense linear run as one expert
    size_t zeros_cap = 0;           // entries
};

// Scratch of the layer chain, grown on demand (reference: dchain / dx16 / dy buffers, w4a16_dec/buffers.rs).
struct W4ChainScratch {
    uint64_t y32 = 0, h16a = 0, h16b = 0, ping[2] = {0, 0};
    size_t y32_cap = 0, h16a_cap = 0, h16b_cap = 0, ping_cap[2] = {0, 0};
    uint64_t a16 = 0, stats[3] = {0, 0, 0};  // fused chain: f16 qkv output, partial sums of squares per stage
    size_t a16_cap = 0, stats_cap[3] = {0, 0, 0};
};

struct w4a16_event {
    hipEvent_t ev;
};

// A captured and instantiated sequence of launches (reference: GraphEntry {exec, handle}, w4a16_dec/mod.rs; the pair
// ctx/graph.rs hands to graph_destroy).
struct w4a16_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    size_t nodes = 0;
    uint64_t scratch_gen = 0;  // w4a16_ctx::scratch_gen when the capture ended: the nodes hold addresses of that generation
};

struct w4a16_ctx {
    int device = 0;
    hipStream_t stream = nullptr;   // launch stream (reference: CudaCtx.stream)
    hipStream_t stream2 = nullptr;  // second stream (reference: CudaCtx.stream2); copies that must not serialise
    std::vector<hipModule_t> modules;
    std::map<std::string, hipFunction_t, std::less<>> functions;  // looked up by string_view: a launch allocates nothing
    std::unordered_map<uint64_t, size_t> allocs;
    size_t allocated = 0;
    std::map<std::string, W4Lin, std::less<>> lins;
    std::map<std::string, W4Experts, std::less<>> experts;
    W4MoeScratch moe;
    W4ChainScratch chain;
    // prefill launch plans: (t, n, k, forced tile, forced slices) -> {tile rows, k slices, super-tile m, n, count}
    std::map<std::tuple<size_t, size_t, size_t, int, int>, std::array<size_t, 5>> prefill_plans;
    int moe_block = 0, moe_waves = 0;  // 0 = automatic
    int moe_tiled = 0;                 // MFMA-tiled grouped kernel: 0 = automatic (long runs per expert), -1 = never, 1 = always
    int moe_act_kind = 0;              // activation of the expert FFN call in progress (W4A16_ACT_*)
    int decode_rows_per_wave = 0, decode_waves_per_block = 0;  // 0 = automatic
    uint64_t norm_word = 0;  // one device word for w4a16_lin_row_norm_max
    size_t norm_word_cap = 0;
    int decode_ksplit = 0;                                      // 0 = automatic, -1 = never, n = exactly n k slices
    uint64_t decode_ws = 0, decode_tickets = 0;                 // partial tiles and per-block tickets of a split launch
    size_t decode_ws_cap = 0, decode_tickets_cap = 0;
    int prefill_ksplit = 0;                                     // 0 = automatic, -1 = never, n = exactly n slices
    int prefill_tile_m = 0;                                     // 0 = automatic, 64 or 128 rows per block tile
    uint64_t prefill_ws = 0;                                    // f32 partials of a split-K prefill launch
    size_t prefill_ws_cap = 0;
    int cu_count = 0;
    const char* last_symbol = "";  // kernel of the most recent launch (a key of `functions`: stable storage)
    uint64_t fixed_scratch = 0;  // this device's copy of the static scratch array of w4a16_noalloc.hip (device address)
    bool capturing = false;  // between w4a16_capture_begin and w4a16_capture_end: nothing may allocate, free or wait
    // Counts the replacements of context-owned scratch buffers (w4_ensure).  A captured graph holds the addresses of
    // the buffers of its time; once one of them has been replaced a replay would touch freed memory, so
    // w4a16_graph_launch refuses a graph of an older generation (reference: graph_invalidate() on every scratch
    // reallocation, w4a16_dec/buffers.rs:6-31).
    uint64_t scratch_gen = 0;
};

// Launch constants that mirror #defines of the kernel sources (a CPU test reads both texts and compares the values):
// name here = kW4 + CamelCase of the kernel-side macro.
constexpr int kW4TileK = 128;               // W4_TILE_K (w4a16_common.hpp)
constexpr int kW4TileRows = 16;             // W4_TILE_ROWS
constexpr int kW4LaneTt = 8;                // LANE_TT (lane.hip): tokens per pass of the lane-order kernel
constexpr int kW4DecodeMaxKsplit = 8;       // W4_DECODE_MAX_KSPLIT (decode.hip)
constexpr int kW4MoeMaxKsplit = 8;          // MOE_MAX_KSPLIT (moe.hip)
constexpr int kW4MoeLdx = 136;              // MOE_LDX (moe.hip): halves per staged x row
constexpr int kW4MoeAlignWaves = 16;        // MOE_ALIGN_WAVES (moe.hip)
constexpr int kW4RmsLanes = 1024;           // RMS_LANES (glue.hip)
constexpr int kW4PfBn = 256;                // PF_BN (prefill.hip): block tile columns
constexpr int kW4PfKs = 64;                 // PF_KS (prefill.hip): k per LDS stage
constexpr int kW4PfThreads = 256;           // PF_THREADS (prefill.hip)

int w4_fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int w4_hip(hipError_t e, const char* api);
// Keep the message of a failing step across clean-up calls that may fail themselves.
std::string w4_err_save();
void w4_err_restore(const std::string& msg);
int w4_launch(w4a16_ctx* ctx, const char* symbol, unsigned gx, unsigned gy, unsigned block, unsigned shmem,
              void** params);

int w4_register_lin(w4a16_ctx* ctx, const char* name, W4Lin& L);
int w4_find_lin(w4a16_ctx* ctx, const char* name, W4Lin** out);
// true when every scale of `count` u16 entries is finite, non-zero and (bf16) inside [2^-60, 2^60]: what a kernel that
// carries the running unit s_prev / s_cur can take
bool w4_scales_regular(const uint16_t* s, size_t count, int scale_bf16);
int w4_ensure(w4a16_ctx* ctx, uint64_t* buf, size_t* cap, size_t bytes);
// glu_act >= 0: L is a fused gate|up linear and y_dev receives f16 [t][n/2] = act(gate) * up on the f32 sums
int w4_dense_grouped(w4a16_ctx* ctx, const W4Lin& L, uint64_t x_dev, uint64_t y_dev, size_t t, int out_f16, int glu_act = -1);
int w4_lin_forward_fixed_ws(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t y_dev, size_t t, int out_f16,
                            uint64_t ws, size_t ws_bytes, uint64_t tickets, size_t ticket_bytes);
// per-device fixed scratch of the allocation-free entry point (w4a16_noalloc.hip)
int w4_noalloc_init(w4a16_ctx* ctx);
void w4_noalloc_release(w4a16_ctx* ctx);

#define W4_TRY(expr)          \
    do {                      \
        int rc__ = (expr);    \
        if (rc__) return rc__; \
    } while (0)
