/*
 * w4a16_hip.h — C ABI of the MI355X (gfx950) W4A16 linear-op library, libw4a16hip.so.
 *
 * The library replaces, for the W4A16 linear path only, the reference's CUDA driver layer and the operators built
 * on it.  Each entry point names the reference interface it stands in for (paths relative to the reference
 * checkout).  Plain C types only: a Rust `extern "C"` block, cgo or ctypes can bind this file 1:1.
 *
 * Conventions
 *   - Every function returning int returns 0 on success.  Non-zero is either a hipError_t value or one of the
 *     W4A16_ERR_* codes below; w4a16_last_error() then returns a NUL-terminated message (thread-local, valid until
 *     the next failing call on the same thread).  The reference returns Result<_, String> with text
 *     "rawcuda: <api>: <err>" (crates/backend-gpu/src/rawcuda/ctx/mod.rs:294-309); messages here read
 *     "w4a16hip: <api>: <err>".
 *   - Device pointers are uint64_t, as CUdeviceptr is in the reference (ffi.rs).  The context owns device memory it
 *     allocated and frees what is left at destroy (ctx/mem.rs:4-44); the caller owns host buffers.
 *   - A context is used by one thread at a time (the reference context is Send, not Sync: w4a16_dec/mod.rs:626).
 *   - Operands: x  u16 [t][k] f16;  q  u32 [n][k/8], element i of a row = nibble (q[i>>3] >> 4*(i&7)) & 0xF,
 *     weight = nibble - 8;  s  u16 [n][k/group] f16 (or bf16);  y [t][n] f32 or f16
 *     (crates/core/src/quant/lane.rs:62-63).
 */
#ifndef W4A16_HIP_H
#define W4A16_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct w4a16_ctx w4a16_ctx;
typedef struct w4a16_event w4a16_event;
typedef struct w4a16_graph w4a16_graph;

enum {
    W4A16_OK = 0,
    W4A16_ERR_SHAPE = 10001,       /* shape contract violated (gptq4.rs:31-58, upload.rs:26-32)            */
    W4A16_ERR_SYMBOL = 10002,      /* kernel symbol not loaded (ctx/mod.rs:262-267)                         */
    W4A16_ERR_UNSUPPORTED = 10003, /* group / scale dtype combination has no kernel (gptq4.rs:60-70)        */
    W4A16_ERR_NOT_FOUND = 10004,   /* linear name not registered (w4a16_dec/kernels/gemv.rs:10-13)          */
    W4A16_ERR_ARG = 10005,         /* null pointer, zero size, bad enum                                     */
    W4A16_ERR_ASSET = 10006,       /* code object file missing or unreadable (assets.rs:336-346)            */
    W4A16_ERR_STALE_GRAPH = 10007  /* a scratch buffer the graph's nodes address was replaced (buffers.rs:6-31) */
};

/* Message of the last failing call on this thread ("" if none). */
const char* w4a16_last_error(void);

/* ------------------------------------------------------------------------------------------------------------
 * Driver layer — stands in for CudaCtx over the dlopen'ed libcuda table
 * (crates/backend-gpu/src/rawcuda/ffi.rs:237-292, ctx/mod.rs:62-77, 100-419, ctx/mem.rs, ctx/prof.rs).
 * ---------------------------------------------------------------------------------------------------------- */

/* CudaCtx::new_dev (ctx/mod.rs:100-152): initialise HIP, select the device, create the launch stream and a second
 * stream (both non-blocking, default priority), and load every code object of the built-in manifest from
 * `asset_dir` (NULL = the directory "assets" beside the shared library; a single asset can be redirected with the
 * environment variable LLM170_HIP_<NAME>_HSACO_PATH, as LLM170_CUDA_<NAME>_FATBIN_PATH does in assets.rs:336-339). */
int w4a16_ctx_create(int device_ordinal, const char* asset_dir, w4a16_ctx** out);
/* Drop of CudaCtx: frees every tracked allocation (ctx/mem.rs:32-44), modules, streams. */
void w4a16_ctx_destroy(w4a16_ctx* ctx);

/* CudaCtx::load_fatbin (ctx/mod.rs:196-228): hipModuleLoadData on a gfx950 code object image, then resolve every
 * listed symbol eagerly; a missing symbol fails the load and names it. */
int w4a16_module_load(w4a16_ctx* ctx, const char* key, const void* image, size_t len, const char* const* symbols,
                      size_t nsym);
/* CudaCtx::function (ctx/mod.rs:262-267): 0 if `symbol` is resolved, W4A16_ERR_SYMBOL otherwise. */
int w4a16_has_symbol(w4a16_ctx* ctx, const char* symbol);
/* CudaCtx::launch / launch_shared (ctx/mod.rs:270-363): hipModuleLaunchKernel(f, gx,gy,1, block,1,1, shmem,
 * launch stream, params, NULL); params is an array of pointers to the argument values (args.rs:4-31). */
int w4a16_launch(w4a16_ctx* ctx, const char* symbol, unsigned gx, unsigned gy, unsigned block, unsigned shmem,
                 void** params);

/* Name of the kernel the most recent launch of this context used ("" before the first), whichever entry point made
 * it: what a profile is matched against (the reference resolves the launched function's name per launch for its
 * profile report, prof_mark, ctx/prof.rs:56-72).  Valid until the context is destroyed. */
const char* w4a16_last_launch_symbol(w4a16_ctx* ctx);

/* CudaCtx::alloc / free / h2d / d2h / d2d / memset (ctx/mem.rs:4-44, 164-336).  Copies and the fill are ordered on
 * the launch stream; h2d and d2h return after the data has moved. */
int w4a16_alloc(w4a16_ctx* ctx, size_t bytes, uint64_t* dptr);
int w4a16_free(w4a16_ctx* ctx, uint64_t dptr);
int w4a16_h2d(w4a16_ctx* ctx, uint64_t dst, const void* src, size_t bytes);
int w4a16_d2h(w4a16_ctx* ctx, void* dst, uint64_t src, size_t bytes);
int w4a16_d2d(w4a16_ctx* ctx, uint64_t dst, uint64_t src, size_t bytes);
int w4a16_memset0(w4a16_ctx* ctx, uint64_t dst, size_t bytes);
/* CudaCtx::sync (ctx/mod.rs:407-412): wait for the launch stream. */
int w4a16_sync(w4a16_ctx* ctx);
/* Bytes currently allocated through this context (CudaCtx::allocs bookkeeping, ctx/mem.rs:4-30). */
size_t w4a16_allocated_bytes(w4a16_ctx* ctx);

/* Event timing on the launch stream (ctx/prof.rs:4-54: event create / record / elapsed). */
int w4a16_event_create(w4a16_ctx* ctx, w4a16_event** out);
int w4a16_event_record(w4a16_ctx* ctx, w4a16_event* ev);
int w4a16_event_elapsed_ms(w4a16_ctx* ctx, w4a16_event* start, w4a16_event* stop, float* ms); /* waits for stop */
void w4a16_event_destroy(w4a16_ctx* ctx, w4a16_event* ev);

/* Capture of the launch stream into a graph and its replay (CudaCtx::capture_begin / capture_end / graph_instantiate /
 * graph_upload / graph_launch / graph_destroy, ctx/graph.rs:4-85).  Between w4a16_capture_begin and w4a16_capture_end every
 * launching entry point of this library (w4a16_launch, w4a16_lin_forward*, w4a16_moe_ffn*, w4a16_chain_forward*,
 * w4a16_memset0, w4a16_d2d, ...) records a node instead of running.  Nothing may allocate, free, wait or copy to or from
 * the host in between: w4a16_alloc, w4a16_free, w4a16_sync, w4a16_h2d, w4a16_d2h and any call whose scratch buffer would
 * have to grow return W4A16_ERR_ARG (and invalidate nothing) — run the sequence once before capturing it, as the
 * reference does (warm_for_capture, w4a16_dec/graphs.rs:55).  w4a16_capture_end ends the capture, instantiates and
 * uploads the graph.  A graph replays the recorded launches with the recorded arguments: same buffers, same shapes.
 * Replays are ordered on the launch stream like any other launch.  w4a16_graph_destroy waits for the launch stream.
 * The recorded arguments include addresses of scratch buffers the context owns (split-K partials and tickets, the
 * expert FFN's and the chain's intermediates).  A later eager call that needs one of them LARGER (more rows, a wider
 * linear, more experts) frees it and allocates a new one; every graph captured before that is stale from then on and
 * w4a16_graph_launch refuses it with W4A16_ERR_STALE_GRAPH instead of replaying onto freed memory — destroy it and
 * capture again (the reference invalidates its graphs on every scratch reallocation, w4a16_dec/buffers.rs:6-31).
 * Calls that fit the buffers as they are never invalidate a graph. */
int w4a16_capture_begin(w4a16_ctx* ctx);
int w4a16_capture_end(w4a16_ctx* ctx, w4a16_graph** out);
int w4a16_graph_launch(w4a16_ctx* ctx, w4a16_graph* graph);
size_t w4a16_graph_nodes(const w4a16_graph* graph); /* kernel and copy nodes recorded */
void w4a16_graph_destroy(w4a16_ctx* ctx, w4a16_graph* graph);

/* Names in the built-in asset manifest (assets.rs:276-334): returns the number of assets; when `asset` is in range
 * stores its name and NULL-terminated symbol list. */
size_t w4a16_manifest(size_t asset, const char** name, const char* const** symbols);

/* ------------------------------------------------------------------------------------------------------------
 * Operator layer
 * ---------------------------------------------------------------------------------------------------------- */

/* check_shapes (gptq4.rs:31-58): group in {128,32}, k % group == 0, t >= 1, qlen == n*(k/8) words,
 * slen == n*(k/group) halves, xlen == t*k halves.  (The reference's extra t==1 limit k <= 256*group exists only
 * for its shared-memory scale cache; the kernels here have no such limit and the rule is not carried over.) */
int w4a16_check_shapes(size_t t, size_t qlen, size_t slen, size_t xlen, size_t n, size_t k, size_t group);

/* kernel_sym (gptq4.rs:60-70): name of the bit-exact kernel serving (group, scale dtype); NULL + W4A16_ERR_UNSUPPORTED
 * for other combinations.  Served here: (128,f16) (32,bf16) as in the reference, plus (32,f16) and (128,bf16). */
const char* w4a16_kernel_sym(int group, int scale_bf16);

/* Gptq4::gemm / Gptq4::gemv (gptq4.rs:85-190): upload x, q, s; run the kernel that reproduces
 * dot_row_w4a16_lane_group bit for bit (64 strided f32 lanes, un-fused multiply and add, f64 tree;
 * crates/core/src/quant/lane.rs:2-70); download out f32 [t][n]; free.  A test operator, not the fast path. */
int w4a16_gemm_host(w4a16_ctx* ctx, const uint16_t* x_f16, size_t t, const uint32_t* q, const uint16_t* s, size_t n,
                    size_t k, size_t group, int scale_bf16, float* out_f32);

/* W4a16Dec::upload_lin_g (w4a16_dec/upload.rs:15-65): register a linear by name.  q: n*k/2 bytes, s: n*(k/group)*2
 * bytes in the operand format above; lengths are enforced.  Keeps the operands resident as given and, when
 * k % 128 == 0 (rows are padded to a multiple of 16), also in the tiled layout the streaming and MFMA kernels read (the reference likewise
 * keeps a repacked copy next to the original, upload.rs:99-179).  Re-registering a name frees the old buffers. */
int w4a16_upload_lin(w4a16_ctx* ctx, const char* name, const void* q, size_t qlen_bytes, const void* s,
                     size_t slen_bytes, size_t n, size_t k, size_t group, int scale_bf16);
/* consolidate_marlin_dense (upload.rs:67-97): free the as-given copy of one linear once the tiled one exists
 * (bit-exact path and raw dump then report W4A16_ERR_NOT_FOUND for it). */
int w4a16_lin_drop_raw(w4a16_ctx* ctx, const char* name);
/* Fuse registered linears that read the same activations (q/k/v, gate/up) into one, rows concatenated in the order
 * given, so that one launch serves them all: y[:, 0:n0] is part 0, y[:, n0:n0+n1] part 1, ...  The reference reaches the
 * same end with a table of segments for its multi-linear GEMV (build_multi_tables, w4a16_dec/buffers.rs:229-366) and with
 * fused gate|up arenas (upload.rs:1116-1235).  Parts need the same k, group and scale type and their as-given operands;
 * drop_parts != 0 unregisters them afterwards.  A fused gate|up linear is what w4a16_lin_forward_glu takes. */
int w4a16_lin_fuse(w4a16_ctx* ctx, const char* name, const char* const* parts, size_t n_parts, int drop_parts);
/* gemv_multi_dev / gemv_multi_t_dev (w4a16_dec/kernels/gemv.rs:189-332) over the segment table {weights, scales, out,
 * n, k} that build_multi_tables writes per layer (w4a16_dec/buffers.rs:229-366): ONE decode launch for the linears
 * fused under `name`, every part into its own output.  outs_dev: n_outs device addresses (a host array), n_outs = the
 * number of parts given to w4a16_lin_fuse (2..4); output i receives f16 or f32 [t][n_i], the rows of part i, with the
 * bits w4a16_lin_forward writes to y[:, first_i : first_i + n_i] of the fused linear when that launch runs two row blocks
 * per wave as this one always does (w4a16_set_decode_shape(ctx, 32, 0); another launch shape may split k differently
 * and differ in the last bits).  Parts must be multiples of 16
 * rows (W4A16_ERR_SHAPE otherwise); decode steps only: t > 16 is W4A16_ERR_UNSUPPORTED (w4a16_lin_forward then writes
 * the parts side by side in one tensor, which the consumers in this library read through a row stride). */
int w4a16_lin_forward_multi(w4a16_ctx* ctx, const char* name, uint64_t x_dev, const uint64_t* outs_dev, size_t n_outs,
                            size_t t, int out_f16);
/* lin_spec (w4a16_dec/mod.rs:1193-1206): shape of a registered linear. */
int w4a16_lin_info(w4a16_ctx* ctx, const char* name, size_t* n, size_t* k, size_t* group, int* scale_bf16,
                   int* has_tiled, int* has_raw);

/* LinPath (w4a16_dec/mod.rs:79-84) */
enum {
    W4A16_PATH_AUTO = 0,   /* t <= 16 -> DECODE, t <= 64 -> STREAM, else PREFILL; LANE without a tiled copy             */
    W4A16_PATH_LANE = 1,   /* bit-exact twin of lane.rs (reference: w4a16_gemm_g128, gptq4.cu:825-951)            */
    W4A16_PATH_DECODE = 2, /* HBM-streaming skinny GEMM, t <= 16 (reference: gemv_t_launch / sk_*_dev)            */
    W4A16_PATH_PREFILL = 3, /* LDS-staged MFMA GEMM, any t (reference: gemm_launch -> marlin_gemm_try)            */
    W4A16_PATH_STREAM = 4   /* weight-streaming kernel with x shared through LDS, segments of up to 64 rows       */
};

/* lin_forward (w4a16_dec/kernels/mod.rs:121-144): y[t][n] = x[t][k] * W^T on the launch stream, no host sync.
 * x_dev: f16 [t][k].  y_dev: f32 [t][n] if out_f16 == 0 else f16 [t][n] (f32 accumulation, one rounding). */
int w4a16_lin_forward(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t y_dev, size_t t, int out_f16,
                      int path);

/* The launch plan w4a16_lin_forward would pick on the decode path (t = 1..16) for a linear of this shape on a GPU of
 * `cu_count` compute units with every setting automatic — rows of the output per wave (16, 32 or 64), waves per
 * workgroup, k slices across workgroups, dynamic LDS bytes — without a context or a GPU (sk_ksp, w4a16_dec/kernels/
 * decode.rs:3-16, is the reference's rule of the same role).  A shape whose staged scales would pass the LDS of a CU is
 * planned with fewer rows per wave or more k slices; W4A16_ERR_SHAPE only when nothing fits.  `glu` != 0 plans the gated
 * kernel of w4a16_lin_forward_glu.  Out pointers may be NULL. */
int w4a16_plan_decode(size_t n, size_t k, size_t group, size_t t, int cu_count, int glu, int* rows_per_wave,
                      int* waves_per_block, int* k_slices, size_t* lds_bytes);
/* The launch plan of the prefill path (W4A16_PATH_PREFILL) for t rows: out = {block tile rows (64, 96 or 128), k slices,
 * super-tile rows, super-tile columns, super-tile count}; `tile_rows` and `k_slices` pin a choice as
 * w4a16_set_prefill_tile / w4a16_set_prefill_ksplit do (0 = automatic); *price_us (may be NULL) receives the model's
 * estimate for the chosen plan.  Role of the reference's per-problem choice of thread-block shape
 * (kernels/marlin.rs:94-213).  Needs neither a context nor a GPU. */
int w4a16_plan_prefill(size_t t, size_t n, size_t k, size_t group, int cu_count, int tile_rows, int k_slices,
                       size_t out[5], double* price_us);

/* w4a16_lin_forward for callers that cannot allocate.  NO COUNTERPART IN THE REFERENCE: it exists for code under HIP graph
 * capture, tight serving loops and harnesses that forbid hipMalloc.  w4a16_lin_forward's decode launch, when it splits k
 * across workgroups (the 27B down projection does), parks partial tiles and tickets in a workspace that the context
 * grows on demand; this entry point runs the same launch with that workspace in a fixed array in the library's own
 * device image (8 MiB of partial tiles + 64 KiB of tickets per GPU, held until the process ends) and calls no
 * hipMalloc, hipFree or any other allocating routine.  Decode regime only: t <= 16 (W4A16_ERR_SHAPE beyond), a linear
 * with a tiled copy.  A launch whose split needs more than the array holds — workgroups x row blocks per wave x 1 KiB x
 * k slices > w4a16_noalloc_workspace_bytes(), or more than 16384 workgroups per slice — is refused with W4A16_ERR_SHAPE
 * and a message that gives both sizes.  Same results, bit for bit, as w4a16_lin_forward(..., W4A16_PATH_DECODE) under
 * the same w4a16_set_decode_* settings.  A GPU has ONE such array.  The first context that calls this entry point on a
 * GPU owns the array until that context is destroyed; the call from any other context on that GPU is refused with
 * W4A16_ERR_ARG (two contexts sharing the tickets would sum each other's partial tiles).  Calls of the owning context
 * are ordered on its launch stream and safe; the array keeps the last call's contents between calls (the tickets are
 * left at zero by every launch). */
int w4a16_lin_forward_noalloc(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t y_dev, size_t t, int out_f16);
size_t w4a16_noalloc_workspace_bytes(void);

/* The gate|up projection of a dense FFN with the elementwise kernel that follows it folded in
 * (gemv_multi_dev of the gate/up group + ew_dev_fused, w4a16_dec/chains.rs:271-287, assets/ew.cu:9-32):
 * y[r][c] = f16(silu(g) * u), g = (W x)[r][c], u = (W x)[r][n/2 + c], f32 arithmetic, for a linear whose rows 0..n/2 are
 * the gate and n/2..n the up projection (n % 32 == 0).  y_f16_dev: f16 [t][n/2].  Any t: up to 16 rows the decode
 * kernel, up to 64 (and for a linear with a zero or non-finite scale) the weight-streaming kernel, beyond that the
 * MFMA-tiled prefill kernel, each with the activation in its epilogue — the pair lin_forward + ew of the reference's
 * prefill chain (w4a16_dec/prefill.rs:148-207) in one launch.  Same values, bit for bit, as w4a16_lin_forward on the
 * same path and launch shape followed by w4a16_silu_mul_f16 (the gated streaming kernel never splits over k; compare
 * with w4a16_set_decode_ksplit(-1)), without the [t][n] f32 round trip. */
int w4a16_lin_forward_glu(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t y_f16_dev, size_t t);
/* The same with the activation named: act = W4A16_ACT_SILU (above) or W4A16_ACT_GELU_TANH, the elementwise kernel the
 * reference launches for gelu-gated models (ew_gelu, assets/ew.cu:34-57):
 * y = f16(0.5 g (1 + tanh(0.7978846 (g + 0.044715 g^3))) * u).  Same values as w4a16_lin_forward followed by
 * w4a16_act_mul_f16 with the same act. */
int w4a16_lin_forward_glu_act(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t y_f16_dev, size_t t, int act);

/* A decode-regime linear (t <= 16) with the RMS normalisation of its input deferred across it.  The reference runs
 * norm_resid as a launch of its own ahead of each linear (assets/norm.cu:4-48, kernels/mod.rs:11-54); a per-row
 * factor commutes with the linear, so here the launch that PRODUCES the activations leaves partial sums of their
 * squares and the launch that CONSUMES them scales its output instead:
 *   y[r][c] = s[r] * (W x[r])[c],   s[r] = 1 / sqrt(sum_r / in_cols + 1e-6),
 *   sum_r = the n_stats_in partial sums stats_in_dev[i][r] (f32 [n_stats_in][16], added in a fixed order);
 *   stats_in_dev == 0: s = 1.
 * x rows are ldx halves apart (0 = k; a column slice of a wider f16 matrix is allowed, ldx % 8 == 0).
 * stats_out_dev != 0: the launch writes *n_stats_out entries [i][16] of partial sums of y[r][c]^2 (the f32 values,
 * before any rounding to f16) over columns c < stat_rows; the buffer must hold ceil(n / 16) entries of 64 bytes.
 * A chain of such launches needs no normalisation launch between its linears: the f16 activations travel
 * un-normalised (same relative precision), every consumer applies the factor.
 * The rest of norm_resid belongs to the producer and is folded into the same launch when the pointers are non-zero:
 *   resid_dev  f32 [t][n], the residual stream: v = resid + y is written back to it (norm.cu:11-13), the statistics are
 *              those of v, and v is what continues;
 *   nw_dev     f32 [n], the norm weight of the output rows (norm.cu:19-23): y_dev receives v * nw.
 * The consumer's output is then 1/rms(v) * W2 (v * nw), the reference's W2 (v * 1/rms(v) * nw) with the f16 rounding
 * of the activations taken before the 1/rms factor instead of after it.
 * RANGE PRECONDITION: the activations travel between the two launches as f16 WITHOUT their 1/rms factor, so every
 * element of v (of v * nw with a norm weight) must lie inside the f16 range: beyond 65504 it becomes Inf (and the
 * consumer's output NaN) where norm_resid, which normalises in f32 first, stays finite; rows whose elements fall below
 * 6e-5 lose relative precision to f16 subnormals.  Nothing is detected at run time.  Residual streams of trained
 * models sit well inside; the synthetic 64-layer chain of random projections does not: the _scaled forms below lift the
 * precondition. */
/* Row count: any t.  Up to 16 rows the decode kernel serves the call and a statistics array is [entries][16] floats
 * (row m of entry e at e*16 + m); beyond 16 rows the MFMA-tiled kernel does (the linear must then hold only scales that
 * kernel can divide by, W4A16_ERR_UNSUPPORTED otherwise) and a statistics array is [entries][ld] floats with ld = t
 * rounded up to a multiple of 4.  *n_stats_out entries are written (at most n/16 resp. n/64: size stats_out_dev for
 * that); producer and consumer of one array run at the same t. */
int w4a16_lin_forward_deferred_norm(w4a16_ctx* ctx, const char* name, uint64_t x_dev, size_t ldx, size_t t,
                                    uint64_t stats_in_dev, size_t n_stats_in, size_t in_cols, uint64_t y_dev,
                                    int out_f16, uint64_t stats_out_dev, size_t stat_rows, size_t* n_stats_out,
                                    uint64_t resid_dev, uint64_t nw_dev);
/* The same for the fused gate|up projection: the factor multiplies gate and up before the activation (act as in
 * w4a16_lin_forward_glu_act). */
int w4a16_lin_forward_glu_deferred_norm(w4a16_ctx* ctx, const char* name, uint64_t x_dev, size_t ldx, size_t t,
                                        uint64_t stats_in_dev, size_t n_stats_in, size_t in_cols, uint64_t y_f16_dev,
                                        int act);
/* Both with a power-of-two factor on each hand-over, which lifts the range precondition above when the exponents come
 * from a bound on the values: x_dev holds the true activations times 2^-in_exp and y_dev receives the true output
 * times 2^-out_exp (for the gated form: the true silu(g)*u times 2^-out_exp).  The statistics, the residual stream and
 * the norm weight see true values.  Both factors are exact in f32, so an element gives the same number as in the
 * un-scaled call exactly when BOTH its un-scaled value and its scaled value 2^-out_exp * v are normal f16 numbers
 * (6.1e-5 <= |.| <= 65504).  A positive exponent trades range at the top for range at the bottom: an element with
 * |v| < 2^(out_exp-14) is handed over as an f16 subnormal, with an absolute error of up to 2^(out_exp-25) instead of
 * a relative one of 2^-11, and below 2^(out_exp-25) it becomes zero.  With exponents taken from the Cauchy-Schwarz
 * bound below — orders of magnitude above the elements a trained layer produces — such elements are far below the
 * row's root mean square and carry almost none of its energy (measured on the synthetic 64-layer chain: rel-L2 2e-4
 * against the chain that normalises before rounding); parity on trained-weight activation statistics is not pinned by
 * a test.  Exponents in -120..120; 0, 0 is the un-scaled call.
 * A bound for the output of a linear fed rows of unit root mean square: w4a16_lin_row_norm_max(W) * sqrt(k)
 * (norm_resid of the reference hands over normalised values and needs none of this, assets/norm.cu:4-48). */
int w4a16_lin_forward_deferred_norm_scaled(w4a16_ctx* ctx, const char* name, uint64_t x_dev, size_t ldx, size_t t,
                                           uint64_t stats_in_dev, size_t n_stats_in, size_t in_cols, int in_exp,
                                           uint64_t y_dev, int out_f16, int out_exp, uint64_t stats_out_dev,
                                           size_t stat_rows, size_t* n_stats_out, uint64_t resid_dev, uint64_t nw_dev);
int w4a16_lin_forward_glu_deferred_norm_scaled(w4a16_ctx* ctx, const char* name, uint64_t x_dev, size_t ldx, size_t t,
                                               uint64_t stats_in_dev, size_t n_stats_in, size_t in_cols, int in_exp,
                                               uint64_t y_f16_dev, int out_exp, int act);
/* max over rows r of sqrt(sum_c ((nibble - 8) * scale)^2) of a registered linear's dequantised weights (the values of
 * dequant_row_w4a16_split, crates/core/src/matmul/cpu.rs:167-194), f32 arithmetic on the device.  By Cauchy-Schwarz no
 * element of W x exceeds it times the Euclidean norm of x.  Computed on the first request (a launch and a 4-byte
 * read-back, so not while capturing) and kept with the linear.  Needs the tiled copy (k % 128 == 0). */
int w4a16_lin_row_norm_max(w4a16_ctx* ctx, const char* name, float* out);

/* gemv_host (w4a16_dec/mod.rs, host-operand convenience used by probes): lin_forward with host x / y. */
int w4a16_lin_forward_host(w4a16_ctx* ctx, const char* name, const uint16_t* x_f16, void* y, size_t t, int out_f16,
                           int path);

/* Dequantised weights of a registered linear as f32 [n][k] = (nibble - 8) * scale
 * (dequant_row_w4a16_split, crates/core/src/matmul/cpu.rs:167-194).  from_tiled != 0 reads the tiled copy (so the
 * re-layout is covered), else the as-given copy. */
int w4a16_dequant_dump(w4a16_ctx* ctx, const char* name, int from_tiled, uint64_t out_f32_dev);
/* Inverse of the upload re-layout: writes q u32 [n][k/8] and s u16 [n][k/group] in the operand format from the
 * tiled copy (round-trip check, as repack_roundtrip / scale_perm_roundtrip in crates/core/src/marlin.rs:106-132). */
int w4a16_lin_untile(w4a16_ctx* ctx, const char* name, uint64_t q_out_dev, uint64_t s_out_dev);

/* Launch-shape override for the decode kernel (0 = choose automatically): rows_per_wave in {16,32,64},
 * waves_per_block in 1..8.  For tuning sweeps (the reference exposes its split-K factor the same way,
 * sk_ksp, w4a16_dec/kernels/decode.rs:3-16). */
int w4a16_set_decode_shape(w4a16_ctx* ctx, int rows_per_wave, int waves_per_block);
/* Split-K across workgroups for the decode kernel: 0 = automatic (outputs too narrow to give every CU several equal
 * shares of row blocks), -1 = never, 1..8 = exactly that many k slices (clamped to two k tiles per slice).  Still one
 * launch: the workgroup that finishes last adds the slices in slice order.  Counterpart of the reference's split-K
 * factor for its decode GEMV (sk_ksp, w4a16_dec/kernels/decode.rs:3-16, 59-127). */
int w4a16_set_decode_ksplit(w4a16_ctx* ctx, int ksplit);

/* Split-K override for the prefill kernel: 0 = automatic (split when the tile grid alone would leave most of the chip
 * idle — narrow outputs at moderate t; the reference's prefill path makes the same choice inside its vendored GEMM),
 * -1 = never, n >= 1 = exactly n k slices (clamped so a slice has at least 4 k tiles). */
int w4a16_set_prefill_ksplit(w4a16_ctx* ctx, int ksplit);
/* Rows of the prefill kernel's block tile: 0 = automatic (priced with the k slices, w4a16_plan_prefill), 64, 96 or 128.  The reference's
 * vendored GEMM picks its thread-block shape per problem the same way (marlin_gemm_try, kernels/marlin.rs:94-213). */
int w4a16_set_prefill_tile(w4a16_ctx* ctx, int rows);

/* run_bench_gemv / run_bench_gemm (crates/server/src/probes/w4a16/gpu/bench.rs:366-433): `warmup` untimed then
 * `reps` timed back-to-back lin_forward launches on the launch stream, one synchronisation at the end.  Launch i
 * uses linear names[i % n_names] — rotating over copies whose total size exceeds the last-level caches gives the
 * cold-HBM figure, a single name the warm one (the reference flushes with a 256 MiB copy instead, probe.rs:1198-1230).
 * All named linears must have the same shape.  ms_events = elapsed between HIP events recorded on the launch stream
 * around the timed launches; ms_wall = host wall clock around the same region including the final sync. */
int w4a16_bench_forward(w4a16_ctx* ctx, const char* const* names, size_t n_names, uint64_t x_dev, uint64_t y_dev,
                        size_t t, int out_f16, int path, size_t warmup, size_t reps, float* ms_events,
                        double* ms_wall);

/* ------------------------------------------------------------------------------------------------------------
 * MoE expert FFN (grouped / ragged W4A16 GEMM)
 * ---------------------------------------------------------------------------------------------------------- */

/* build_marlin_moe_arenas (w4a16_dec/upload.rs:1116-1235): register the experts of one MoE layer by name.
 *   q13: u32 [n_experts][2*n_ff][h/8]      fused gate|up projection, rows 0..n_ff gate, n_ff..2*n_ff up
 *   s13: u16 [n_experts][2*n_ff][h/group]
 *   q2 : u32 [n_experts][h][n_ff/8]        down projection
 *   s2 : u16 [n_experts][h][n_ff/group]
 * Byte lengths are enforced.  Needs h % 128 == 0, n_ff % 128 == 0 (whole k tiles) — true of the reference's MoE
 * shapes.  The experts are kept only in the tiled layout, one arena per projection, experts at a fixed stride. */
int w4a16_upload_experts(w4a16_ctx* ctx, const char* name, size_t n_experts, const void* q13, size_t q13_bytes,
                         const void* s13, size_t s13_bytes, const void* q2, size_t q2_bytes, const void* s2,
                         size_t s2_bytes, size_t h, size_t n_ff, size_t group, int scale_bf16);
int w4a16_experts_info(w4a16_ctx* ctx, const char* name, size_t* n_experts, size_t* h, size_t* n_ff, size_t* group,
                       int* scale_bf16);
/* Dequantised weights of one expert's projection (which: 0 = gate|up [2*n_ff][h], 1 = down [h][n_ff]) as f32,
 * read back from the arena (covers the arena re-layout bit for bit). */
int w4a16_experts_dequant_dump(w4a16_ctx* ctx, const char* name, int which, size_t expert, uint64_t out_f32_dev);

/* moe_topk (w4a16_dec/mod.rs:168-185): host routing of t tokens.  Softmax over all n_exp logits in f32, the top_k
 * largest probabilities with ties to the lower index, weights renormalised by the selected sum.
 * idx: int32 [t][top_k], w: f32 [t][top_k]. */
int w4a16_moe_topk_host(const float* logits, size_t t, size_t n_exp, size_t top_k, int32_t* idx, float* w);
/* Device kernel w4a16_moe_topk_t, assets/moe.cu:686-759: the same rule on the device, logits f32 [t][n_exp] already resident.
 * n_exp <= 1024, top_k <= 64.  The exponential and the softmax sum are evaluated in a different order than on the
 * host, so weights agree to rounding, not bit for bit. */
int w4a16_moe_route(w4a16_ctx* ctx, uint64_t logits_dev, size_t t, size_t n_exp, size_t top_k, uint64_t idx_dev,
                    uint64_t wt_dev);
/* Device kernels w4a16_moe_align2 and w4a16_moe_align_marlin, assets/moe.cu:860-908 and 1599-1633: stable counting sort of the
 * ns = t*top_k slots by expert, every expert's run padded to a multiple of `block` with the sentinel ns.
 *   sorted_dev: int32, capacity >= ns + n_exp*block; expert_ids_dev: int32 per block of `block` sorted entries,
 *   capacity >= ns/block + n_exp + 1; num_post_dev: int32 [2] = {padded total, experts hit}. */
int w4a16_moe_align(w4a16_ctx* ctx, uint64_t idx_dev, size_t ns, size_t n_exp, size_t block, uint64_t sorted_dev,
                    uint64_t expert_ids_dev, uint64_t num_post_dev);

/* marlin_moe_ffn_dev (w4a16_dec/kernels/marlin_moe.rs:290-422): the routed-expert FFN of t tokens on the launch
 * stream, no host synchronisation:
 *   align slots -> act[slot] = f16(silu(f16(gate)) * f16(up)), gate|up = W13[expert] * x[token]
 *               -> c2[slot] = f16(wt[slot] * (W2[expert] * act[slot]))
 *               -> y[token] = sum over the token's slots of c2, in slot order, f32.
 *   x_dev f16 [t][h]; idx_dev int32 [t*top_k]; wt_dev f32 [t*top_k]; y_dev f32 [t][h].
 * Scratch (sorted ids, act, c2) is owned by the context and grown on demand.
 * For t <= 15 and top_k <= 8 the call runs in direct mode: no alignment, the gate|up GEMM takes one segment per slot and
 * one more launch does the down projections of a token's experts, the weight multiply, the f16 rounding of c2 and
 * the slot-order sum (same values, c2 never reaches memory). */
int w4a16_moe_ffn(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t idx_dev, uint64_t wt_dev, size_t t,
                  size_t top_k, uint64_t y_dev);
/* The same with the activation chosen per call, the `gelu` flag of marlin_moe_ffn_dev (marlin_moe.rs:298, 372-376):
 * W4A16_ACT_SILU = act[slot] = f16(silu(g) * u) (w4a16_moe_act_silu_f16), W4A16_ACT_GELU_TANH =
 * f16(0.5 g (1 + tanh(0.7978846 (g + 0.044715 g^3))) * u) (w4a16_moe_act_gelu_f16, assets/moe.cu:1635-1647), g and u
 * the gate and up sums rounded to f16, f32 arithmetic. */
enum { W4A16_ACT_SILU = 0, W4A16_ACT_GELU_TANH = 1 };
int w4a16_moe_ffn_act(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t idx_dev, uint64_t wt_dev, size_t t,
                      size_t top_k, uint64_t y_dev, int act);
/* Scratch of the last w4a16_moe_ffn call, for stage-by-stage checks (the reference exposes the same buffers to
 * its moe_selfcheck, w4a16_dec/probe.rs:153): which = 0 sorted ids (int32), 1 expert ids (int32), 2 num_post
 * (int32 [2]), 3 act (f16 [ns][n_ff]), 4 c2 (f16 [ns][h]).  Also reports the segment size used (1 = direct mode, where only
 * act exists). */
int w4a16_moe_scratch(w4a16_ctx* ctx, int which, uint64_t* dptr, size_t* bytes, size_t* block);
/* Launch-shape override for the MoE GEMMs (0 = automatic): block = slots per segment (4, 16, 32, 48, 64; 1 = direct mode);
 * waves = waves per workgroup (k split for segments of <= 16 slots, output-row units otherwise). */
int w4a16_set_moe_shape(w4a16_ctx* ctx, int block, int waves);
/* The MFMA-tiled grouped kernels (the role of the reference's grouped Marlin GEMM at prefill sizes, assets/moe.cu:686-759
 * via kernels/marlin_moe.rs:290-422): workgroup = one 64-slot segment x 256 output columns on 32x32x16 MFMA tiles, the
 * segment's x rows gathered into LDS, expert weights as the B operand straight from the arena.  0 = automatic (mean run
 * per expert of at least 96 slots, i.e. t * top_k >= 96 * n_experts, and no segment size forced), -1 = never, 1 =
 * always (64-slot segments whatever t).  Same results as the streaming kernels up to the order of the f32 sums. */
int w4a16_set_moe_tiled(w4a16_ctx* ctx, int mode);
/* Timed back-to-back w4a16_moe_ffn calls (as w4a16_bench_forward); call i uses experts names[i % n_names]. */
int w4a16_bench_moe(w4a16_ctx* ctx, const char* const* names, size_t n_names, uint64_t x_dev, uint64_t idx_dev,
                    uint64_t wt_dev, size_t t, size_t top_k, uint64_t y_dev, size_t warmup, size_t reps,
                    float* ms_events, double* ms_wall);

/* ------------------------------------------------------------------------------------------------------------
 * Layer chain: the linears of a dense decoder layer run back to back with the elementwise glue between them
 * ---------------------------------------------------------------------------------------------------------- */

/* Register a linear whose operands are generated on the device from the SplitMix64 streams of the reference's
 * parity gate (crates/server/src/probes/w4a16/gates.rs:182-196): q word i = low 32 bits of output i of stream
 * seed_q; scale i = f16(lo + (hi - lo) * u_i), u_i = (output i of stream seed_s >> 40) / 2^24.  Same result as
 * uploading those operands from the host; exists so that tens of GB of synthetic layers need no host generation. */
int w4a16_upload_lin_synth(w4a16_ctx* ctx, const char* name, size_t n, size_t k, size_t group, uint64_t seed_q,
                           uint64_t seed_s, float lo, float hi);

/* RMS rescale of t rows to unit mean square, emitting f16 (the part of norm_resid, assets/norm.cu:4-48, that a chain
 * of linears needs: no residual, no weight): out[r][c] = f16(v[r*ld + c] * inv_r), inv_r = f32(1/sqrt(ms_r + 1e-6)),
 * c < ncols <= ld.  The sum of squares is taken in f64 in a fixed order (1024 strided partials, pairwise fold), so a
 * CPU restatement is bit-identical. */
int w4a16_rms_rescale_f16(w4a16_ctx* ctx, uint64_t v_f32_dev, size_t ld, size_t ncols, size_t t, uint64_t out_f16_dev);
/* norm_resid / norm_resid_g (assets/norm.cu:4-48, 97-148; launched by norm_resid_at, w4a16_dec/kernels/mod.rs:11-54):
 * the residual add and RMS normalisation that produces the f16 A operand of a layer's first linear.  Per token row,
 * with v = x + ab:  x <- v;  xn = v * inv * nw[w_off + c], inv = 1/sqrtf(sum(v^2)/hidden + 1e-6f);  xn32 (0 = skip) =
 * xn rounded to f16 and widened back;  xn16 (0 = skip) = the f16 bits.  x, ab, xn, xn32: f32 [t][hidden]; nw: f32, at
 * least w_off + hidden long; hidden <= 8192.  Same f32 operations in the same order as the reference kernel (one fused
 * multiply-add per square, its tree reduction, correctly rounded divide and square root): bit-identical results. */
int w4a16_norm_resid(w4a16_ctx* ctx, uint64_t x_dev, uint64_t nw_dev, uint64_t ab_dev, uint64_t xn_dev, uint64_t xn32_dev,
                     uint64_t xn16_dev, size_t t, size_t w_off, size_t hidden);
/* ew (assets/ew.cu:9-32): out[r][c] = f16(silu(gu[r][c]) * gu[r][n_ff + c]) for gu f32 [t][2*n_ff], f32 arithmetic. */
int w4a16_silu_mul_f16(w4a16_ctx* ctx, uint64_t gu_f32_dev, size_t n_ff, size_t t, uint64_t out_f16_dev);
/* ew / ew_gelu (assets/ew.cu:9-32, 34-57) chosen by act (W4A16_ACT_SILU, W4A16_ACT_GELU_TANH); the gelu is the tanh
 * form, out = f16(0.5 g (1 + tanh(0.7978846 (g + 0.044715 g^3))) * u) in f32 arithmetic. */
int w4a16_act_mul_f16(w4a16_ctx* ctx, uint64_t gu_f32_dev, size_t n_ff, size_t t, uint64_t out_f16_dev, int act);

/* chain_device_body (w4a16_dec/chains.rs:195-304) reduced to its linears: for layer l = layer0 .. layer0+n_layers-1,
 * with the linears registered as "<prefix>.<l>.attn_qkv", ".attn_output", ".ffn_gate_up", ".ffn_down":
 *     a = rms_f16(qkv(x)[:, :hidden])      (stands in for the token mixer)
 *     b = rms_f16(attn_output(a))
 *     c = silu_mul_f16(ffn_gate_up(b))     (gate = columns 0..n_ff, up = n_ff..2 n_ff)
 *     x = rms_f16(ffn_down(c))
 * x_dev / y_dev: f16 [t][hidden], hidden = k of attn_qkv.  Every linear goes through w4a16_lin_forward (f32 output).
 * No host synchronisation. */
int w4a16_chain_forward(w4a16_ctx* ctx, const char* prefix, size_t layer0, size_t n_layers, uint64_t x_dev, size_t t,
                        uint64_t y_dev);
/* The same chain with the normalisations inside it deferred across the linears (w4a16_lin_forward_deferred_norm), four
 * launches per layer instead of seven (any t; beyond 16 rows on the MFMA-tiled kernels, plus a finish launch where a
 * linear is split over k).  With r(v) = 1/sqrt(mean(v^2) + 1e-6) per row, s0 = 1 and x0 = x:
 *     v1 = s[l] * qkv(x[l])[:, :hidden]      a = f16(v1)
 *     v2 = r(v1) * attn_output(a)            b = f16(v2)
 *     gu = r(v2) * ffn_gate_up(b)            c = silu_mul_f16(gu)
 *     v4 = ffn_down(c)                       x[l+1] = f16(v4), s[l+1] = r(v4)
 * and y = rms_f16(v4) after the last layer: the function of w4a16_chain_forward with the factors applied after the
 * linears instead of before the roundings to f16 (results agree to those roundings).  a, b, c and x[l+1] cross from
 * launch to launch without their 1/rms factor; each crossing carries a power-of-two factor 2^-e
 * (w4a16_lin_forward_deferred_norm_scaled) with e the smallest exponent that brings a bound on the values under 32768:
 * row_norm_max(W) * sqrt(k) for a linear fed unit-rms rows, the square of that for the gated product, and for the down
 * projection row_norm_max * sqrt(n_ff) * the bound of c.  So nothing leaves the f16 range whatever the weights (random
 * weights of mean -0.5 with no residual stream push v4 beyond 65504 within three layers), and wherever the un-scaled
 * values stay in range the result is the same.  The first call on a set of linears computes their row norms (a small
 * launch and read-back each): call it once before capturing it in a graph. */
int w4a16_chain_forward_fused(w4a16_ctx* ctx, const char* prefix, size_t layer0, size_t n_layers, uint64_t x_dev,
                              size_t t, uint64_t y_dev);
/* ensure_graph (w4a16_dec/graphs.rs:41-134): one decode step of the chain as a replayable graph.  Runs the chain once
 * eagerly (which sizes every scratch buffer and leaves its result in y_dev), then captures the same call —
 * w4a16_chain_forward, or w4a16_chain_forward_fused when fused != 0 — and returns the instantiated graph.  Each
 * w4a16_graph_launch recomputes y_dev from whatever x_dev holds at that moment; the reference keeps one such graph
 * per slot and replays it every token. */
int w4a16_chain_graph_create(w4a16_ctx* ctx, const char* prefix, size_t layer0, size_t n_layers, uint64_t x_dev, size_t t,
                             uint64_t y_dev, int fused, w4a16_graph** out);

/* Timed chain passes (decode_bench, w4a16_dec/probe.rs:1123-1289): `warmup` untimed then `reps` timed passes over
 * layers 0..n_layers-1.  use_graph != 0 captures one pass into a HIP graph and times graph launches
 * (forward_graph, w4a16_dec/graphs.rs); fused != 0 times w4a16_chain_forward_fused. */
int w4a16_bench_chain(w4a16_ctx* ctx, const char* prefix, size_t n_layers, uint64_t x_dev, size_t t, uint64_t y_dev,
                      size_t warmup, size_t reps, int use_graph, int fused, float* ms_events, double* ms_wall);

#ifdef __cplusplus
}
#endif
#endif /* W4A16_HIP_H */
