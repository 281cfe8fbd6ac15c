/*
 * turq.h — C ABI of libturq: GGUF block-quantized linear layers on MI355X (gfx950).
 *
 * This is the boundary a host engine binds (Rust `extern "C"`, ctypes, cgo ...).  Every entry
 * point takes plain pointers and sizes, returns an integer status, and never aborts; the text of
 * the last error is kept per context (and per thread when no context exists yet).
 *
 * Each declaration cites the reference interface it stands in for (paths are relative to the
 * danylokravchenko/tur tree; "candle" means candle-core 0.10.2 as pinned by its Cargo.lock).
 *
 * Threading: a context is thread-compatible (calls on one context must be serialised by the
 * caller, as the reference does by owning the model on one thread, src/server/worker.rs:69-100);
 * different contexts may be used from different threads.  Weights are immutable after upload and
 * reference counted, so clones of a layer share one device copy (LinearX is Clone,
 * src/models/layers/linear.rs:8).
 */
#ifndef TURQ_H
#define TURQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct turq_ctx turq_ctx;       /* device + stream + scratch, one per engine thread */
typedef struct turq_weight turq_weight; /* one quantized [n, k] tensor resident in HBM */
typedef struct turq_gguf turq_gguf;     /* an opened GGUF file (header parsed, tensors lazy) */
typedef struct turq_graph turq_graph;   /* a captured sequence of forward calls (hipGraphExec) */

/* status codes */
enum {
    TURQ_OK = 0,
    TURQ_ERR_INVALID = 1,   /* null pointer, bad flag, bad argument */
    TURQ_ERR_SHAPE = 2,     /* shape mismatch, k not a multiple of the block size, ld too small */
    TURQ_ERR_DTYPE = 3,     /* ggml dtype or activation dtype not supported */
    TURQ_ERR_HIP = 4,       /* a HIP runtime call failed (message holds hipGetErrorString) */
    TURQ_ERR_OOM = 5,       /* host or device allocation failed */
    TURQ_ERR_IO = 6,        /* file open/read/parse failure */
    TURQ_ERR_NOT_FOUND = 7  /* tensor or metadata key absent */
};

/* ggml dtype ids as stored in GGUF tensor infos (candle GgmlDType) */
enum {
    TURQ_F32 = 0,
    TURQ_F16 = 1,
    TURQ_Q8_0 = 8,
    TURQ_Q4_K = 12,
    TURQ_Q5_K = 13,
    TURQ_Q6_K = 14,
    TURQ_BF16 = 30
};

/* element type of activation / output buffers */
enum { TURQ_ACT_F32 = 0, TURQ_ACT_BF16 = 1, TURQ_ACT_F16 = 2 };
/* OR-ed into the y_dtype of turq_qmatmul, turq_qmatmul_noalloc or turq_mlp: the results are ADDED to what y holds,
 * y[m, n] += x * W^T (+ bias), in f32 before the one rounding to y's type.  It is the residual connection of the reference's decoder layer,
 * `(x + h)` after o_proj and `x + h2` after the MLP (src/models/qwen3.rs:633-640), taken into the matmul kernel's store: y is the
 * residual stream, and the separate elementwise launch and its round trip of the outputs go away. */
#define TURQ_OUT_ACCUMULATE 0x100

/* weight layouts in HBM */
enum {
    TURQ_LAYOUT_NATIVE = 0, /* GGUF bytes as they are: rows of consecutive blocks */
    TURQ_LAYOUT_TILED = 1   /* 16-row x 256-column tiles, lane-linear planes (see tur_amd/csrc/layout.h) */
};

/* where the pointers of a call live */
enum { TURQ_MEM_HOST = 0, TURQ_MEM_DEVICE = 1 };

/* matmul algorithm selection (TURQ_ALGO_AUTO picks by layout and m) */
enum {
    TURQ_ALGO_AUTO = 0,
    TURQ_ALGO_SIMPLE = 1, /* one wave per output row, f32 FMA on dequantized values */
    TURQ_ALGO_GEMV = 2,   /* MFMA skinny kernel for m <= 32, tiled layout */
    TURQ_ALGO_GEMM = 3    /* LDS-tiled MFMA kernel for prefill chunks, tiled layout */
};

/* ---- library ---- */
const char *turq_version(void);
/* geometry of a ggml dtype: elements and bytes per block; 0 when the dtype is not supported */
int turq_block_elems(int ggml_dtype);
int turq_block_bytes(int ggml_dtype);
/* bytes of an [n, k] tensor in GGUF = n * k / block_elems * block_bytes; 0 on invalid input.
 * Replaces: the length computed inside candle `gguf_file::TensorInfo::read`. */
size_t turq_weight_nbytes(int ggml_dtype, int64_t n, int64_t k);

/* ---- context ---- */
/* Replaces: the `Device` handed to `VarBuilderX::new` / `QVarBuilder::from_gguf`
 * (src/weights/mod.rs:37-67, src/weights/gguf_varbuilder.rs:20-30; chosen at src/main.rs:188). */
int turq_ctx_create(int device_ordinal, turq_ctx **out);
void turq_ctx_destroy(turq_ctx *ctx);
/* message of the most recent failing call on ctx (ctx may be NULL: last failure of this thread
 * in a call that had no context).  Replaces: candle_core::Error -> TurError::CandleError
 * (src/shared/errors.rs:5-6). */
const char *turq_last_error(const turq_ctx *ctx);
/* block until all work queued on the context's stream is done */
int turq_sync(turq_ctx *ctx);
/* the context's hipStream_t, for hosts that time or order their own work on it */
void *turq_ctx_stream(turq_ctx *ctx);
/* Activation range of forward calls on device pointers.  The matrix kernels round activations to f16: magnitudes from 65504 on
 * become infinities and rows whose values all sit far below 6e-5 lose precision, where the reference takes f32 activations of
 * any magnitude (src/weights/mod.rs:84-99; candle scales every 256-element block of them on its own).  With `on` != 0 every
 * turq_qmatmul / turq_qmatmul_multi / turq_qmatmul_gate_up on device pointers with f32 or bf16 activations is bracketed by two
 * small kernels: rows multiplied by the power of two that puts their largest magnitude into [2^9, 2^10) and written as f16,
 * output rows multiplied back (both exact) - any finite f32 row then stays within the 1e-3 bar, infinities and NaNs
 * propagate.  It costs two launches per call and the grouped launches of turq_qmatmul_multi / turq_qmatmul_gate_up.  Default:
 * off, for engines whose activations are known to be bounded (after an RmsNorm, say); turq_ctx_nonfinite_count tells a host
 * that left it off whether a call overflowed.  Calls on HOST pointers always take the wide path: they are the reference's own
 * contract, and the staging copies dominate them anyway.  turq_qmatmul_noalloc cannot take it (it has no scratch for the
 * scaled rows) and refuses f32 / bf16 activations with TURQ_ERR_INVALID while the switch is on. */
int turq_ctx_set_wide_activations(turq_ctx *ctx, int on);
/* Whether a forward call left the number range of its kernels.  Every kernel that stores results (the matmuls, turq_rms_norm,
 * the fragment preparation of calls with more than 32 rows, the f16 intermediate of turq_mlp) counts the elements it stores
 * that are no finite numbers: the output of a row that held a finite value of magnitude 65520 or more while wide activations
 * were off (f16 turns it into an infinity), or of a row that held an infinity or a NaN to begin with.  The call waits for the
 * context's stream and returns the count since the last reset (it stops at about 2^20; the counters live in device memory of
 * the context's GPU and are shared by all contexts on it); reset != 0 clears it.  A host that sees a non-zero count re-runs
 * the step after turq_ctx_set_wide_activations(ctx, 1), with which finite inputs of any magnitude give finite results.  Not
 * inside a graph capture.
 * Stands in for: the reference's f32 activations of any magnitude (src/weights/mod.rs:84-99), which never overflow. */
int turq_ctx_nonfinite_count(turq_ctx *ctx, uint64_t *count, int reset);
/* name and compute-unit count of the context's device */
int turq_ctx_device_info(turq_ctx *ctx, char *name, size_t name_cap, int *compute_units);

/* ---- device memory helpers for hosts without HIP bindings of their own ---- */
int turq_dev_alloc(turq_ctx *ctx, size_t nbytes, void **out);
int turq_dev_free(turq_ctx *ctx, void *ptr);
/* synchronous copies (they wait for the context's stream first) */
int turq_memcpy_h2d(turq_ctx *ctx, void *dst_dev, const void *src_host, size_t nbytes);
int turq_memcpy_d2h(turq_ctx *ctx, void *dst_host, const void *src_dev, size_t nbytes);

/* ---- weights ---- */
/* Upload raw GGUF block bytes of a tensor of shape (n, k) (n output features, k input features,
 * each row = k/block consecutive blocks).  `layout` picks how it is kept in HBM.
 * Errors: unsupported dtype, k % block != 0, nbytes != turq_weight_nbytes(..).
 * Replaces: candle `gguf_file::Content::tensor(reader, name, device)` -> `QTensor` as called by
 * `QVarBuilder::get` (src/weights/gguf_varbuilder.rs:72-74) and `QMatMul::from_arc`
 * (src/models/layers/linear.rs:69). */
int turq_weight_upload(turq_ctx *ctx, int ggml_dtype, int64_t n, int64_t k, const void *host_bytes,
                       size_t nbytes, int layout, turq_weight **out);
/* Arc<QTensor> clone / drop.  The release that drops the last reference waits for the whole device to go idle before it frees
 * the memory (a weight may be in use by launches of any context of that device); do it at teardown, not inside a decode loop. */
int turq_weight_retain(turq_weight *w);
int turq_weight_release(turq_weight *w);
/* QTensor::shape / dtype; any out pointer may be NULL */
int turq_weight_info(const turq_weight *w, int *ggml_dtype, int64_t *n, int64_t *k, int *layout,
                     size_t *device_bytes);
/* Copy the tensor back to host in GGUF byte order whatever its HBM layout (round-trip check). */
int turq_weight_export(turq_ctx *ctx, const turq_weight *w, void *host_bytes, size_t nbytes);

/* Host-side layout transforms used by upload/export (no GPU needed): native GGUF bytes <-> tiled. */
size_t turq_tiled_nbytes(int ggml_dtype, int64_t n, int64_t k);
int turq_tile_host(int ggml_dtype, int64_t n, int64_t k, const void *native, void *tiled);
int turq_untile_host(int ggml_dtype, int64_t n, int64_t k, const void *tiled, void *native);

/* ---- dequantize ---- */
/* out = f32 [n, k] row-major, bit-exact with candle's to_float.  `out_mem` says whether `out` is
 * a host or a device pointer.
 * Replaces: `QTensor::dequantize(device)` (call sites src/weights/mod.rs:150,161;
 * src/models/layers/mod.rs:37; src/models/layers/norm.rs:84; src/models/layers/linear.rs:66). */
int turq_dequantize(turq_ctx *ctx, const turq_weight *w, float *out, int out_mem);

/* Rows of the dequantized tensor picked by index: out[i, 0..k) = dequantize(w)[ids[i], :] for i < count, the same numbers
 * as turq_dequantize bit for bit (then rounded once if out_dtype is bf16 or f16), without the f32 copy of the whole table
 * (2.5 GB for the 151936 x 4096 token_embd of Qwen3-8B against 0.5 GB quantized).  Any ggml dtype turq_dequantize takes,
 * either layout.  `out` has row stride ldo >= k elements; `mem` says where ids and out live.  An index >= n is
 * TURQ_ERR_INVALID with host pointers; with device pointers, where the call cannot look at the indices, that row of `out`
 * is filled with NaN.
 * Replaces: candle's `Embedding::forward` (index_select) on the table that `layers::embedding` dequantizes whole at load
 * (src/models/layers/mod.rs:30-37). */
int turq_embedding_lookup(turq_ctx *ctx, const turq_weight *w, const uint32_t *ids, int64_t count, void *out, int out_dtype,
                          int64_t ldo, int mem);

/* ---- RmsNorm ---- */
/* y[r][c] = x[r][c] / sqrt(mean_c(x[r][c]^2) + eps) * weight[c] for m rows of k elements, in f32 and in candle's order (sum of
 * squares, one square root, per element a division and a multiplication).  weight: f32 [k] in the same memory space as x
 * and y - the `weight` tensor of the GGUF file as turq_dequantize returns it (a Gemma model adds 1 to it at load,
 * src/models/layers/norm.rs:89).  x, y, strides and `mem` as in turq_qmatmul; y may be x.
 * Replaces: `NormX::forward` over candle_nn::RmsNorm built by `layers::norm::rms_norm` (src/models/layers/norm.rs:52-94),
 * which the decoder layers apply in front of the q / k / v and gate / up projections. */
int turq_rms_norm(turq_ctx *ctx, const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, const float *weight,
                  float eps, void *y, int y_dtype, int64_t ldy, int mem);

/* ---- forward ---- */
/* y[m, n] = x[m, k] * W^T  (+ bias[n] when bias != NULL).
 *   x: m rows of k elements of `x_dtype`, row stride ldx elements (ldx >= k);
 *   y: m rows of n elements of `y_dtype`, row stride ldy elements (ldy >= n);
 *   bias: f32 [n] (in the same memory space as x and y) or NULL (the reference adds it with a separate broadcast_add,
 *         src/models/layers/linear.rs:25-28);
 *   mem: TURQ_MEM_DEVICE (x, y are device pointers; the call is asynchronous on the context's
 *        stream) or TURQ_MEM_HOST (x, y are host pointers; staged through the context and
 *        synchronous);
 *   algo: TURQ_ALGO_*.
 * y_dtype | TURQ_OUT_ACCUMULATE adds the results to y instead of overwriting it (see there).
 * Errors instead of panics for m < 0, ld too small, unsupported dtypes.  m == 0 is a no-op.
 * Device calls of 33 - 64 rows on large weights of up to 4096 columns (gate / up of an 8B model) go through the kernels of up
 * to 32 rows in two chunks.  Device calls of more than 32 rows (prompt chunks) whose workgroup tiles would leave most compute units idle - the tall
 * down_proj of a model up to about 256 rows, every matrix of a layer up to 64 - split the columns of every tile over several
 * workgroups, which meet in a scratch buffer of the context (partial tiles, at most 256 MiB per launch and 512 MiB per call; grown like the other scratch
 * buffers: not during a graph capture).  The sums of a result are the same numbers in the same order on every call.
 * Replaces: `LinearX::forward` -> `QMatMul::forward(&Tensor)` (src/models/layers/linear.rs:19-31)
 * -> candle `CustomOp1::cpu_fwd` -> `k_quants::matmul`. */
int turq_qmatmul(turq_ctx *ctx, const turq_weight *w, const void *x, int x_dtype, int64_t m,
                 int64_t ldx, void *y, int y_dtype, int64_t ldy, const float *bias, int mem, int algo);

/* turq_qmatmul for callers that cannot allocate device memory around the call (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same product, same kernels and bit-identical results as turq_qmatmul with
 * TURQ_MEM_DEVICE and TURQ_ALGO_AUTO (one exception: where turq_qmatmul gives the columns of every workgroup tile to several
 * workgroups - see there - this call runs the same kernel unsplit, the same products added in another order: within 2e-6
 * relative L2 of each other), but the prepared activation fragments of the calls that use them
 * (more than 32 rows, and 17 - 32 rows on all but small weights) live in a static device array of TURQ_NOALLOC_SCRATCH_BYTES (one copy per GPU, held until
 * the process ends) instead of the context's growable buffer: the call runs no hipMalloc / hipFree
 * and creates no stream or event.  A call that needs more is refused with TURQ_ERR_SHAPE and a
 * message that names the bytes needed: fragments take 2.25 * mpad * k bytes for up to 32 rows (mpad
 * = m rounded up to 1, 2, 4, 8, 16 or 32) and 2.125 * 32 * ceil(m / 32) * k bytes above, so 16 MiB
 * hold e.g. m = 512 at k = 12288 or m = 1920 at k = 4096.  x, y and bias are device pointers.
 * All contexts of a GPU share that GPU's array and it keeps the last call's contents (every call
 * writes all it reads, nothing has to start at zero): calls through this entry point that overlap
 * on one GPU - two contexts, i.e. two streams - race; serialise them. */
#define TURQ_NOALLOC_SCRATCH_BYTES (16u << 20)
int turq_qmatmul_noalloc(turq_ctx *ctx, const turq_weight *w, const void *x, int x_dtype, int64_t m,
                         int64_t ldx, void *y, int y_dtype, int64_t ldy, const float *bias);

/* The same product for `count` weights that take the same activations: ys[i][m, n_i] = x[m, k] * W_i^T (+ biases[i]).
 * All weights must share k.  With device pointers, tiled weights and m <= 32, neighbouring weights of one format
 * go out as ONE kernel launch, and so do Q4_K or Q5_K weights followed by Q6_K ones (q, k and v of a Q4_K_M file); up to
 * 16 rows that launch is all there is (the kernel makes its MFMA operands from the activation rows themselves), with 17 - 32
 * rows on all but small weights, with activation rows that are not 16-byte aligned, and with k that is not a multiple of 512,
 * one preparation of the activations for all the weights comes first; with more than 32 rows the
 * activations are prepared once for all the weights and each weight runs its GEMM on them (the results of the single
 * calls, bit for bit; GEMMs that leave half of the GPU free, such as k_proj and v_proj of a prompt chunk, run next to each other,
 * up to three at a time, on further streams of the context that are joined to the first before the call returns, so the
 * caller still sees one stream; neighbouring large weights of one format and shape - gate_proj and up_proj - go out as ONE
 * GEMM launch over the rows of all of them where that fills the GPU better, with the tile chosen for all the rows: the same
 * products, in another order of the f32 sums where the tile's waves split k, within 2e-6 relative L2 of the single calls); every other case is exactly the turq_qmatmul calls one after the other (including their errors).  `biases` may be NULL, and so may its entries.
 * Replaces: the back-to-back `forward` calls on one input in the reference's decoder layer - q_proj / k_proj /
 * v_proj (src/models/qwen3.rs:272-274) and gate_proj / up_proj (src/models/qwen3.rs:161-167). */
int turq_qmatmul_multi(turq_ctx *ctx, int count, const turq_weight *const *weights, const void *x, int x_dtype, int64_t m,
                       int64_t ldx, void *const *ys, int y_dtype, const int64_t *ldys, const float *const *biases, int mem,
                       int algo);

/* Activation functions of turq_qmatmul_gate_up (candle_nn::Activation; the reference reads it from the model's config,
 * `act_fn: cfg.hidden_act`, src/models/qwen3.rs:156; Qwen3 and Granite use SiLU). */
enum { TURQ_ACTFN_SILU = 0 };

/* The first half of the reference's MLP in one call: y[m, n] = act(x * gate^T + bias_gate) * (x * up^T + bias_up), with
 * act = SiLU, v / (1 + exp(-v)), computed in f32.  gate and up are two weights of one shape [n, k]; x, y, the strides, the
 * biases (NULL: none) and `mem` as in turq_qmatmul.  With device pointers, tiled weights of one format and up to 32
 * activation rows the activation and the product are applied inside the matmul kernel, which writes one output instead of
 * two: up to 16 rows that kernel is the one launch of the call, for more rows (and for the k and alignments named at
 * turq_qmatmul_multi) it follows one preparation of the activations (scratch memory of the context, which grows on demand,
 * never inside a graph capture).  Every other case computes the two products through turq_qmatmul_multi into scratch memory of the context and
 * combines them in one elementwise pass (with TURQ_MEM_HOST that pass runs on the host CPU, in the same f32 arithmetic: the
 * host form is for tests and one-off calls).  Errors as turq_qmatmul; gate and up of different shapes: TURQ_ERR_SHAPE; an activation other
 * than TURQ_ACTFN_SILU: TURQ_ERR_INVALID.
 * Replaces: `x.apply(&self.gate_proj)?.apply(&self.act_fn)?` times `x.apply(&self.up_proj)?` in `Qwen3MLP::forward`
 * (src/models/qwen3.rs:161-167; the Granite MLP, src/models/granite_41.rs:151-155, has the same form). */
int turq_qmatmul_gate_up(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const void *x, int x_dtype, int64_t m,
                         int64_t ldx, void *y, int y_dtype, int64_t ldy, const float *bias_gate, const float *bias_up, int act,
                         int mem);

/* The reference's whole MLP in one call: y[m, n_out] = (act(x * gate^T + bias_gate) * (x * up^T + bias_up)) * down^T + bias_down.
 * gate and up are two weights of one shape [n_ff, k], down is [n_out, n_ff]; the intermediate lives in scratch memory of the
 * context (m * n_ff values, which grows on demand, never inside a graph capture).  The results are those of
 * turq_qmatmul_gate_up into an f32 buffer followed by turq_qmatmul on it, bit for bit, and so are the errors and the meaning of
 * x, y, the strides, the biases (NULL: none), `act` and `mem`.  (Where down_proj runs on the matrix cores - a tiled
 * quantized weight, wide activations off - its kernels round the activations to f16 first thing, so the intermediate is
 * stored as f16 to begin with: the same values, half the bytes that every compute unit reads for down_proj.)
 * The call is those two calls one after the other on the context's stream.  (A single launch for the whole MLP - one
 * persistent workgroup per compute unit, down_proj's first tiles requested while the last gate / up tiles are computed, a grid-wide
 * barrier on device counters before down_proj reads the intermediate - was built, gave the same bits and was slower: 26 us
 * against 20.4 us for a Qwen3-8B MLP row, the barrier alone 4.7 us; it is not in the library.)
 * Replaces: `Qwen3MLP::forward` (src/models/qwen3.rs:161-167; the Granite MLP, src/models/granite_41.rs:151-155, has the
 * same form). */
int turq_mlp(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const turq_weight *down, const void *x, int x_dtype,
             int64_t m, int64_t ldx, void *y, int y_dtype, int64_t ldy, const float *bias_gate, const float *bias_up,
             const float *bias_down, int act, int mem);

/* turq_qmatmul_multi on RmsNorm(x): ys[i][m, n_i] = (x / sqrt(mean(x^2) + eps) * norm_weight) * W_i^T (+ biases[i]), for the
 * weights that the reference applies to a normalised tensor - q / k / v behind `ln1`, the LM head behind the final norm
 * (count = 1).  norm_weight: f32 [k] in the memory space of x (the `weight` of the norm as turq_dequantize returns it); every
 * other argument as in turq_qmatmul_multi (the algorithm is chosen by the call).  With device pointers and tiled weights the norm costs no launch of its own where
 * the kernels can apply it themselves: for ONE activation row the matmul kernel multiplies its columns by norm_weight while it
 * stages them, adds up their squares, and scales the results by the row's 1 / sqrt(mean + eps) (it rounds x * norm_weight to f16
 * where the separate calls round the normalised value: within 5e-4 relative L2 of them, inside the 1e-3 bar against an f64 norm
 * followed by the f32 matmul); for MORE THAN 32 rows the norm writes the fragments of the prefill GEMM directly (the results of turq_rms_norm into f32
 * followed by turq_qmatmul_multi, bit for bit).  Every other case runs the norm into scratch memory of the context - as f16
 * where the matmul kernels would round its output to f16 anyway: the same values, half the bytes for them to read - and then
 * the plain call (also bit-equal to the separate calls).  Range: the one-row route rounds x * norm_weight, not the normalised
 * value, to f16, so a residual stream with |x * norm_weight| >= 65520 overflows there (turq_ctx_nonfinite_count sees it); with
 * wide activations on (turq_ctx_set_wide_activations) every case runs the norm into f32 scratch and takes any finite magnitude.
 * Replaces: `self.ln1.forward(x)` followed by the three projections (src/models/qwen3.rs:633-634, 272-274), `self.norm` followed
 * by `lm_head` (src/models/qwen3.rs:979-985). */
int turq_norm_qmatmul_multi(turq_ctx *ctx, int count, const turq_weight *const *weights, const void *x, int x_dtype, int64_t m,
                            int64_t ldx, const float *norm_weight, float eps, void *const *ys, int y_dtype, const int64_t *ldys,
                            const float *const *biases, int mem);

/* turq_mlp on RmsNorm(x), the second half of the reference's decoder layer: with y_dtype | TURQ_OUT_ACCUMULATE and y = the
 * residual stream it is `x + mlp(ln2(x))` in one call (src/models/qwen3.rs:637-640).  norm_weight and eps as above, everything
 * else as in turq_mlp; the norm is taken into the kernels in the same two cases (one row: into the gate / up kernel; more than
 * 32 rows: the norm writes the fragments of the gate / up GEMMs) and runs into scratch memory otherwise. */
int turq_norm_mlp(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const turq_weight *down, const void *x, int x_dtype,
                  int64_t m, int64_t ldx, const float *norm_weight, float eps, void *y, int y_dtype, int64_t ldy, const float *bias_gate,
                  const float *bias_up, const float *bias_down, int act, int mem);

/* A hint that `w` is the weight of one of the next forward calls: one read-only pass over its bytes on a stream of the
 * context's own, which starts where the context's stream stands when the call is made (so it runs next to whatever is queued
 * after it) and which nothing waits for.  A decode launch of a few tens of MB spends a third of its time before its first
 * bytes arrive and after its last request has left, and cannot start before the launch that makes its activations has ended;
 * its weights depend on nothing, so the memory system can fetch them during those gaps, and the forward call then finds
 * them in the GPU's memory-side cache (256 MB on an MI355X: hint one or two launches ahead, not a whole model).  Results
 * are unaffected.  Inside a graph capture the pass becomes a parallel branch of the graph that turq_graph_end joins.
 * Replaces nothing in the reference, whose CPU path has no launches; the order it serves is the reference's: gate / up then
 * down in `Qwen3MLP::forward` (src/models/qwen3.rs:161-167), q / k / v, o, gate / up, down per decoder layer
 * (src/models/qwen3.rs:633-640), one layer after the other. */
int turq_weight_prefetch(turq_ctx *ctx, const turq_weight *w);

/* ---- activation quantisation (candle's VecDotType::from_float, bit-exact) ---- */
/* x f32 [m, k] (row stride k) -> Q8_0 blocks (34 B per 32) / Q8_K blocks (292 B per 256).
 * The GPU forward path does not use them (it keeps activations in f16); they are the device
 * counterpart of candle `BlockQ8_0::from_float` / `BlockQ8K::from_float`, the first step of
 * `k_quants::matmul`. */
int turq_quantize_q8_0(turq_ctx *ctx, const float *x, int64_t m, int64_t k, void *out, int mem);
int turq_quantize_q8_k(turq_ctx *ctx, const float *x, int64_t m, int64_t k, void *out, int mem);

/* ---- launch-overhead control and kernel timing (no counterpart in the reference, whose CPU path
 * has no launches; a decode step here is hundreds of ~5 us kernels) ---- */
/* Capture every TURQ_MEM_DEVICE forward call made on ctx between begin and end into a graph and
 * replay it with one launch.  Run the same calls once eagerly first: scratch buffers must already
 * have their final size, allocation is not allowed while capturing.  The captured calls keep
 * referring to the same x / y / weight pointers, and to the context's scratch buffers by address.
 * Scratch lifetime: while a graph of the context is alive (between turq_graph_end and
 * turq_graph_destroy), a scratch buffer that a later, larger eager call outgrows is kept allocated
 * next to its replacement instead of being freed, so the graph stays valid to launch; outgrown
 * buffers are released once no graph of the context is alive, or with the context.  Destroy the
 * graphs of a context before the context.
 * A call that fails between begin and end (bad argument, a scratch buffer that would have to grow)
 * ends the capture and discards what was recorded: the stream and the context stay usable, and
 * turq_graph_end then returns TURQ_ERR_INVALID. */
int turq_graph_begin(turq_ctx *ctx);
int turq_graph_end(turq_ctx *ctx, turq_graph **out);
int turq_graph_launch(turq_ctx *ctx, turq_graph *g);
void turq_graph_destroy(turq_graph *g);
/* Bookkeeping behind the rule above, for hosts and tests that want to see it: graphs of the context
 * that are alive, outgrown scratch buffers kept for them, and the size of the activation-fragment
 * buffer.  Any out pointer may be NULL. */
int turq_ctx_scratch_info(const turq_ctx *ctx, int *live_graphs, int *retired_buffers, size_t *act_prep_bytes);
/* Between begin and end every MFMA matmul kernel (not the activation preparation) is launched
 * with a pair of HIP events that the runtime stamps with the dispatch's own begin and end times;
 * end waits for the stream and returns the number of timed launches and the sum of their
 * execution times (launch gaps excluded). */
int turq_profile_begin(turq_ctx *ctx);
int turq_profile_end(turq_ctx *ctx, int64_t *launches, double *total_ms);
/* A yardstick for the numbers above, not part of the path: one launch that only READS nbytes of device memory at dev_ptr
 * (16-byte aligned; rounded down to whole 4 KiB) with the launch shape of the decode kernels - one 16-wave workgroup per
 * compute unit, two 4 KiB chunks in flight per wave - on the context's stream, timed like a matmul kernel when kernel timing
 * is on.  A launch of a few tens of MB is short enough for the launch itself to weigh as much as its bytes (on an MI355X
 * 28 MB take 5.0 us and 57 MB 9.2 us, where 8 TB/s would mean 3.5 and 7.1): this is what the decode kernels are up against. */
int turq_read_yardstick(turq_ctx *ctx, const void *dev_ptr, size_t nbytes);
/* Which launch the rules for prompt chunks (more than 32 rows, K-quant or Q8_0 weights in the tiled layout) make for a weight of
 * n rows and k columns on a device with `compute_units` CUs; no GPU is needed and nothing is launched.  tile: 1 = 128 x 128,
 * 2 = 128 x 192 (Q8_0: 128 x 64), 3 = 128 x 256, 4 = 64 x 128; split: workgroups that share the columns of every tile (1: none);
 * wave_groups: 2 where the 64 x 128 tile runs eight waves as two groups on alternate super-blocks.  Not part of the path, no
 * counterpart in the reference: for tests of the rules and for tuning them on another device. */
int turq_prefill_plan(int dtype, int64_t n, int64_t k, int64_t m, int compute_units, int *tile, int *split, int *wave_groups);
/* ... and whether turq_qmatmul_multi sends `count` (1 .. 4) neighbouring weights of that format and shape - gate_proj and up_proj -
 * out as ONE launch over the rows of all of them (merged = 1) or as a launch each (0).  The rule compares how well the two
 * choices fill their rounds over the device's CUs, so the answer depends on compute_units; the kernels give the same products
 * either way (another order of the f32 sums where a tile's waves split k: within 2e-6). */
int turq_prefill_plan_multi(int dtype, int64_t n, int64_t k, int64_t m, int count, int compute_units, int *merged);
/* The environment switches that override the library's kernel-selection rules (names TURQ_*; for A/B timing and tests, none
 * is needed in production), as this process runs with them: one line per switch, "NAME=value  (default | set)  what it
 * overrides".  The environment is read once, when the first context is created; a process that has any of them set says so in
 * one line on stderr then.  buf may be null; *needed receives the bytes the whole text takes, terminator included.  (No
 * counterpart in the reference, whose CPU path has no such rules.) */
int turq_tuning_describe(char *buf, size_t cap, size_t *needed);

/* ---- GGUF files ---- */
/* Parse the header (magic, version 1..3, metadata, tensor infos, alignment).
 * Replaces: `QVarBuilder::from_gguf` -> candle `gguf_file::Content::read`
 * (src/weights/gguf_varbuilder.rs:20-30). */
int turq_gguf_open(const char *path, turq_gguf **out);
void turq_gguf_close(turq_gguf *g);
const char *turq_gguf_last_error(const turq_gguf *g);
/* `all_keys` (gguf_varbuilder.rs:110-117) */
int64_t turq_gguf_tensor_count(const turq_gguf *g);
const char *turq_gguf_tensor_name(const turq_gguf *g, int64_t index);
/* `contains_key` / `tensor_shape` (gguf_varbuilder.rs:100-108): dims come back outermost first
 * ((n, k) for a matrix, i.e. GGUF order reversed as candle does).  TURQ_ERR_NOT_FOUND if absent. */
int turq_gguf_tensor_info(const turq_gguf *g, const char *name, int *ggml_dtype, int *n_dims,
                          int64_t dims[4], uint64_t *file_offset, size_t *nbytes);
/* metadata lookups (Content::metadata): integer-like and string values */
int turq_gguf_meta_u64(const turq_gguf *g, const char *key, uint64_t *out);
int turq_gguf_meta_f64(const turq_gguf *g, const char *key, double *out);
int turq_gguf_meta_str(const turq_gguf *g, const char *key, char *out, size_t cap);
/* Read one tensor's raw bytes from the file (seek + read, nothing cached). */
int turq_gguf_read_tensor(turq_gguf *g, const char *name, void *host_bytes, size_t nbytes);
/* `QVarBuilder::get((n, k), name)` / `get_no_shape(name)` (gguf_varbuilder.rs:52-94): read the
 * tensor and upload it.  expect_n/expect_k < 0 skip the shape check; a mismatch is TURQ_ERR_SHAPE
 * ("shape mismatch for NAME, got .., expected .."). 1-D tensors load as (1, k). */
int turq_gguf_load_weight(turq_ctx *ctx, turq_gguf *g, const char *name, int64_t expect_n,
                          int64_t expect_k, int layout, turq_weight **out);

#ifdef __cplusplus
}
#endif
#endif /* TURQ_H */
