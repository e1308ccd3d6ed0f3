/* mi355q — quantized-linear engine for AMD Instinct MI355X (gfx950).
 *
 * C ABI of the drop-in replacement for the quantized linear / matmul calls of
 * the llm-in-c C runtimes.  Plain pointers and sizes only.  Every entry point
 * returns an int status and, on failure, writes a message into the caller's
 * buffer (NULL / zero capacity is tolerated) — the convention of the
 * reference's C entry points (models/qwen3.8-27b/targets/apple-m3-pro/
 * qwen38_m3.m:35-41,342-345; models/minimax-h3/targets/apple-m3-pro/
 * minimax_h3_m3_gemm.m:309-315: 0 ok, 1 device/runtime failure, 2 invalid
 * argument).  Nothing aborts.
 *
 * Weight images are consumed in the byte layouts the reference's packers
 * write; `*_weight_prepare` uploads them once into HBM (in a tiled order the
 * kernels stream) and the handle is then used for any number of calls —
 * the prepare-once / run-many shape of the reference's operators
 * (models/whisper-large-v3-turbo/targets/rk3588/native/opencl_w4a16.h:93-133;
 * minimax_h3_m3_gemm.m:338-346).
 *
 * Threading: one context owns one HIP stream and one workspace and permits
 * one call in flight (as the reference's model handle does,
 * qwen38_m3_decode.h:73-75).  Distinct contexts are independent.
 */
#ifndef MI355Q_H
#define MI355Q_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mi355q_context mi355q_context;
typedef struct mi355q_q4_weight mi355q_q4_weight;
typedef struct mi355q_graph mi355q_graph;
typedef struct mi355q_w8a8_weight mi355q_w8a8_weight;

enum {
    MI355Q_OK = 0,
    MI355Q_ERROR_RUNTIME = 1,
    MI355Q_ERROR_INVALID = 2
};

/* element types of activations, outputs and residuals */
enum {
    MI355Q_F16 = 0,
    MI355Q_F32 = 1,
    MI355Q_BF16 = 2
};

/* affine-Q4 group-64 metadata layouts */
enum {
    /* meta[N][K/64] of {uint16 fp16 scale, uint16 fp16 bias}: the Q38 image's
     * metadata plane (qwen38_m3.m:19-33; qwen38_m3_image.h:40-51) */
    MI355Q_META_F16_INTERLEAVED = 0,
    /* scales[N][K/64] and biases[N][K/64], bf16: the MLX source planes
     * (compiler/minimax-h3/apple-m3-pro/minimax_h3_q4_layer.h:14-24;
     * qwen38_m3_pack.c:618-637) */
    MI355Q_META_BF16_PLANES = 1
};

/* flags */
enum {
    MI355Q_X_DEVICE = 1u << 0,        /* x is a device pointer */
    MI355Q_Y_DEVICE = 1u << 1,        /* y is a device pointer */
    MI355Q_RESIDUAL_DEVICE = 1u << 2, /* residual is a device pointer */
    MI355Q_ASYNC = 1u << 3,           /* do not wait; all pointers must be device */
    MI355Q_SOURCE_DEVICE = 1u << 4,   /* prepare: image pointers are device pointers */
    /* the residual is one row [N] added to every activation row: the `bias` of the
     * reference's grouped linear (whisper_turbo_encoder.c:127-157) */
    MI355Q_RESIDUAL_IS_BIAS = 1u << 5,
    /* mi355q_q4_linear_multi with exactly two targets {gate, up} of equal shape and at most
     * 16 activation rows (8 when x is fp32): targets[0].y = silu(gate . x) * (up . x),
     * silu(g) = g / (1 + exp(-g)) in fp32; targets[1].y is not written and may be NULL; no
     * residuals.  The reference's fused decode kernel qwen38_q4_gate_up_silu
     * (qwen38_q4.metal:129-151; source_mlp_reference_first_8, qwen38_m3_pack.c:244-349) */
    MI355Q_FUSE_GATE_UP_SILU = 1u << 6,
    /* mi355q_w8a8_linear: the streaming convolution's epilogue and layout,
     * out[n][m] = bias[n] + (weight_scale[n] * x_scales[m]) * (float)acc
     * (stream_conv_cells, minimindo_mimi.c:869-880) */
    MI355Q_W8A8_CHANNEL_MAJOR = 1u << 7,
    /* mi355q_causal_q8_windows: the two-sample windows of a transposed convolution */
    MI355Q_WINDOWS_PAIRS = 1u << 8
};

/* record order of a symmetric group-128 Q4 tensor */
enum {
    /* record (n, g) at index n*(K/128) + g (compiler/q4_image.py:120-146) */
    MI355Q_SYM128_ROW_MAJOR = 0,
    /* four output rows interleaved: index ((n/4)*(K/128) + g)*4 + n%4
     * (compiler/q4_image.py:44-61; KIND_Q4_OUTPUT_BLOCKED, qwen35_task.c:324-345,432-435);
     * N must be a multiple of 4 */
    MI355Q_SYM128_OUTPUT_BLOCKED = 1
};

typedef struct {
    char name[128];
    char arch[32];
    int compute_units;
    int wavefront;
    size_t hbm_bytes;
    size_t lds_per_workgroup;
    int clock_mhz;
    int memory_clock_mhz;
    int memory_bus_bits;
} mi355q_device_info;

/* ---- context ---------------------------------------------------------------
 * The opaque handle that owns device state, as qwen38_m3_model / the Metal
 * device+queue do in the reference (qwen38_m3_decode.h:62-75). */
int mi355q_context_create(int device, mi355q_context **out,
                          char *error, size_t error_capacity);
void mi355q_context_destroy(mi355q_context *ctx);
int mi355q_context_info(mi355q_context *ctx, mi355q_device_info *info,
                        char *error, size_t error_capacity);
/* Experiment knobs of one context — the counterpart of the reference's QWEN38_* /
 * MINIMAX_* environment switches that its benches read (qwen38_m3_decode.m:1217-1283
 * QWEN38_PROFILE; qwen38_m3.m:342-345).  The environment variables MI355Q_Q4_STREAM,
 * MI355Q_Q4_GEMM, MI355Q_TRACE and MI355Q_NO_ARRIVALS are read once, when the context is
 * created; this call changes the same knobs afterwards.  A NULL or empty value clears one.
 *   "q4_stream" = "TILES,DEPTH,WAVES[,SLICES]"  forces the streaming kernel's launch shape
 *   "q4_gemm"   = "VARIANT,SPLITS"              forces the GEMM's kernel variant and K split
 *   "trace"     = "1"                           prints every launch's decomposition to stderr
 *   "in_kernel_slices" = "0"                    K slices are added by a second kernel
 *   "w8a8"      = "1" .. "4"                    W8A8: weight tiles per workgroup
 *   "gemm_loads" = "plain"                      GEMM variant 7 built with ordinary weight loads
 *                                               (compiler-placed waits): the cross-check of the
 *                                               hand-scheduled kernel, same bits, slower
 *   "batch_invariant" = "1"                     decode-identical verify: for up to eight activation
 *                                               rows (four of fp32) row m of y is bit for bit what the
 *                                               one-row call on x[m] gives, as the reference's exact
 *                                               batched kernels guarantee (qwen38_prefill.metal:5-9,
 *                                               142-248; tests/qwen38_m3_prefill_parity_test.c:115-199):
 *                                               the launch takes the waves and K slices of the one-row
 *                                               launch instead of the fastest ones for its row count
 *   "three_tiles" = "0"                         the streaming launch never takes three tiles per
 *                                               workgroup (unset: where two would not fit one round)
 *   "gemm_order" = "xcd" / "launch"             the pipelined GEMM numbers its blocks so that the row
 *                                               blocks of one tile block share an XCD's L2 / takes them
 *                                               in launch order; unset: by the number of tile blocks
 *   "q8_gemm"   = "doubled" / "native"          8-bit weights above 16 rows: the Q4 GEMM kernels on
 *                                               the doubled weight / the kernel on the bytes
 *                                               themselves where it applies (the default)
 *   "half_tiles" = "1" / "0"                    the streaming launch's half-tile form (a workgroup takes
 *                                               eight of a tile's rows and two 128-column steps at a
 *                                               time) wherever the kernel has it (up to four 16-bit
 *                                               rows) / never; unset: where it measured faster
 *   "chain" = "1"                               mi355q_q4_linear_sequence runs gate|up-SiLU and the
 *                                               linear that reads its output as ONE launch (see there;
 *                                               also MI355Q_CHAIN=1 in the environment).  Off by default:
 *                                               measured on the 27B MLP it is 3 us slower than the two
 *                                               launches at one row and level with them at two
 *   "chain_spin_limit" = "N"                    polls after which a waiting wave of such a one-launch
 *                                               pair gives up (the call that next waits for the
 *                                               stream then returns status 1)
 *   "chain_withhold" = "1"                      such launches wait for a count they cannot reach: the
 *                                               test of that bounded wait
 * Unknown names and malformed values: status 2. */
int mi355q_context_set_option(mi355q_context *ctx, const char *name, const char *value,
                              char *error, size_t error_capacity);
/* Counters of one context, for tests and reports (no counterpart in the reference):
 *   "chained_launches"    pairs of linears that went out as one launch (see mi355q_q4_linear_sequence)
 *   "staging_bytes"       bytes of the context's growable staging buffers
 *   "staging_generation"  how often a staging buffer has been reallocated
 * Unknown names: status 2. */
int mi355q_context_get(mi355q_context *ctx, const char *name, uint64_t *value,
                       char *error, size_t error_capacity);
/* Waits for everything queued on the context's stream
 * (the reference's waitUntilCompleted, qwen38_m3_decode.m:1701-1716). */
int mi355q_sync(mi355q_context *ctx, char *error, size_t error_capacity);

/* Device buffers for callers that keep activations resident between calls
 * (the reference's MTLBuffer allocations, qwen38_m3.m:523-552). */
int mi355q_device_alloc(mi355q_context *ctx, size_t bytes, void **out,
                        char *error, size_t error_capacity);
int mi355q_device_free(mi355q_context *ctx, void *pointer,
                       char *error, size_t error_capacity);
int mi355q_upload(mi355q_context *ctx, void *device_dst, const void *host_src,
                  size_t bytes, char *error, size_t error_capacity);
int mi355q_download(mi355q_context *ctx, void *host_dst, const void *device_src,
                    size_t bytes, char *error, size_t error_capacity);

/* GPU time of the work queued between the two calls, from HIP events on the
 * context's stream — the `double *gpu_ms` the reference's projection call
 * reports (minimax_h3_m3_gemm.h:58-66; GPUEndTime-GPUStartTime,
 * qwen38_m3_decode.m:1217-1283). */
int mi355q_timer_begin(mi355q_context *ctx, char *error, size_t error_capacity);
int mi355q_timer_end(mi355q_context *ctx, double *gpu_ms,
                     char *error, size_t error_capacity);

/* Per-kernel GPU time: between the two calls every compute kernel the context
 * launches carries its own start/stop event pair; `kernel_ms` is the sum of
 * the kernels' own durations (no gaps between launches) and `launches` their
 * number.  The reference's QWEN38_PROFILE mode sums GPUEndTime-GPUStartTime per
 * kernel class the same way (qwen38_m3_decode.m:1217-1283). */
int mi355q_profile_begin(mi355q_context *ctx, char *error, size_t error_capacity);
int mi355q_profile_end(mi355q_context *ctx, double *kernel_ms, uint64_t *launches,
                       char *error, size_t error_capacity);
/* After mi355q_profile_end: the individual durations, in launch order, of the kernels the
 * last profile covered (`count` = how many there were; at most `capacity` are written). */
int mi355q_profile_durations(mi355q_context *ctx, double *kernel_us, size_t capacity,
                             size_t *count, char *error, size_t error_capacity);

/* Measured read bandwidth of HBM: one pass of 128-bit loads over a private
 * buffer of `bytes` (use >= 1 GiB to defeat the 256 MB memory-side cache),
 * best of `repeats`.  `launch_bytes` (0 = the whole buffer) splits the pass
 * into back-to-back kernel launches of that size each, which shows what a
 * kernel as short as one weight matrix can reach.  variant 0: plain loads,
 * 1: streaming (non-temporal) loads, 2: plain loads with a larger grid.  The
 * analogue of the reference's bandwidth probes (tools/target_probe.c;
 * qwen38_jetson_memory_probe.cu:25-35). */
int mi355q_probe_read_bandwidth(mi355q_context *ctx, size_t bytes, size_t launch_bytes,
                                int repeats, int variant, double *gb_per_s,
                                char *error, size_t error_capacity);

/* Where workgroups run: *xcds = number of XCDs (accelerator dies) a small grid was spread
 * over; *columns_share_xcd = 1 if the workgroups (x, 0), (x, 1), ... of a grid whose width
 * is a multiple of eight all ran on the XCD of (x, 0).  The streaming kernel adds K slices
 * inside the kernel only then (their partial sums meet in that XCD's L2); the context
 * probes this once at creation and otherwise adds them with a second kernel.  No
 * counterpart in the reference (single-die targets). */
int mi355q_probe_xcd_columns(mi355q_context *ctx, int *columns_share_xcd, int *xcds,
                             char *error, size_t error_capacity);

/* Measured rate of the fp16 matrix instruction (v_mfma_f32_16x16x32_f16, fp32
 * accumulation) with every SIMD issuing independent ones from registers and
 * `valu_per_mfma` (0..4) packed-fp16 vector instructions between them — the mix of
 * a GEMM that dequantizes weights in registers.  The figure to read a GEMM's
 * TFLOP/s against, next to the datasheet's.  No counterpart in the reference (its
 * targets have no matrix-instruction probe); same role as its bandwidth probes. */
int mi355q_probe_mfma_rate(mi355q_context *ctx, int valu_per_mfma, int repeats,
                           double *tflops, char *error, size_t error_capacity);

/* ---- affine Q4, group 64: w[n][k] = scale[n][k/64] * q[n][k] + bias[n][k/64]
 *
 * quants: [N][K/64][32] bytes, element k of a row in byte k/2, even k in the
 *         low nibble (== little-endian uint32 [N][K/8], element k%8 at bits
 *         4*(k%8)) — qwen38_m3.m:113-116; minimax_h3_attention.metal:246-255.
 * meta_a / meta_b: per `meta_kind`; meta_b is NULL for the interleaved kind.
 * K must be a non-zero multiple of 64 (minimax_h3_m3_gemm.m:309-315 rejects
 * anything else with status 2); N is any non-zero row count.
 * Replaces: the image-to-buffer step of qwen38_m3.m:523-552 and
 * minimax_h3_m3_gemm.m:338-346. */
int mi355q_q4_weight_prepare(mi355q_context *ctx,
                             const void *quants, const void *meta_a,
                             const void *meta_b, uint32_t N, uint32_t K,
                             int meta_kind, uint32_t flags,
                             mi355q_q4_weight **out,
                             char *error, size_t error_capacity);
/* Symmetric Q4, group 128 — the tensor format of compiler/q4_image.py that the
 * portable C runtimes read: per (row, 128-column group) a 66-byte record = bf16
 * scale then 64 code bytes, element j in byte j/2, even j in the low nibble, the
 * nibble a two's complement value v in [-8, 7], w = scale * v
 * (qwen35_task.c:36-38,286-303,426-450).  The records are mapped on the GPU,
 * without loss, to the affine layout (q = v + 8, bias = -8 * scale, each group
 * as two 64-column groups), and the returned handle is an ordinary Q4 weight:
 * every mi355q_q4_linear* entry point takes it.  K must be a non-zero multiple
 * of 128.  Replaces the record walk of q4_gemv (qwen35_task.c:318-362) and of
 * linear_grouped (whisper_turbo_encoder.c:127-157). */
int mi355q_sym128_weight_prepare(mi355q_context *ctx, const void *records,
                                 uint32_t N, uint32_t K, int record_order,
                                 uint32_t flags, mi355q_q4_weight **out,
                                 char *error, size_t error_capacity);
void mi355q_q4_weight_destroy(mi355q_q4_weight *weight);
/* Bytes of the original image this weight stands for: N*K/2 + N*(K/64)*4. */
size_t mi355q_q4_weight_image_bytes(const mi355q_q4_weight *weight);
/* Rows (outputs) and columns (inputs) of a prepared weight. */
void mi355q_q4_weight_shape(const mi355q_q4_weight *weight, uint32_t *N, uint32_t *K);

/* ---- affine Q8, group 64 ---------------------------------------------------------
 * w = scale * q + bias with one 8-bit code per byte, quants[N][K] (element k of group g of
 * row n at byte (n * K/64 + g) * 64 + k), metadata as for Q4 (bf16 planes scales[N][K/64],
 * biases[N][K/64], or fp16 pairs): the projection format of minimax_h3_q8_gemm_bf16_meta
 * (minimax_h3_attention.metal:594-676).  prepare splits the codes into nibbles once:
 * scale*q + bias = (16*scale)*hi + bias + scale*lo, i.e. one ordinary Q4 weight of twice
 * the columns, [high part | low part], which mi355q_q8_linear applies to [x | x] in one Q4
 * linear: the kernels start the activation row over at the weight's second half (K a
 * multiple of 128; otherwise a small kernel first writes the rows twice into a staging
 * buffer); arguments and flags as mi355q_q4_linear.  Up to 16 rows the weight stays exact.
 * Above (the GEMM path), when K is a multiple of 128, a kernel multiplies the bytes
 * themselves, each weight rounded to fp16 as the reference rounds half(scale*q + bias); for
 * that, prepare keeps the weight a second time in GEMM tiles (device memory: about twice the
 * image).  Otherwise, and under option "q8_gemm" = "doubled", the Q4 GEMM kernels run on the
 * doubled weight and round its two parts to fp16 separately. */
typedef struct mi355q_q8_weight mi355q_q8_weight;
int mi355q_q8_weight_prepare(mi355q_context *ctx, const void *quants, const void *meta_a,
                             const void *meta_b, uint32_t N, uint32_t K, int meta_kind,
                             uint32_t flags, mi355q_q8_weight **out,
                             char *error, size_t error_capacity);
/* Q8 rows: per output row an fp32 scale followed by K signed bytes, w = scale * v — the
 * MMO_Q8_ROW tensors of minimindo_thinker.c (:84-86,112-122) and the Q8 payload of
 * minimindo_audio_encoder.c (:90,216-217), records [N][4 + K].  Prepared the same way
 * with integer metadata (v + 128 = 16*hi + lo), so mi355q_q8_linear on such a weight
 * computes the exact integer-weighted sum in fp32 and multiplies it by the row's scale at
 * the end, as q8_f32_dot's callers do (minimindo_thinker.c:124-213, q8_matvec /
 * q8_matmul_sequence: fp32 activations in, fp32 out); a residual is added after the scale.
 * K must be a non-zero multiple of 64. */
int mi355q_q8rows_weight_prepare(mi355q_context *ctx, const void *records, uint32_t N,
                                 uint32_t K, uint32_t flags, mi355q_q8_weight **out,
                                 char *error, size_t error_capacity);
void mi355q_q8_weight_destroy(mi355q_q8_weight *weight);
size_t mi355q_q8_weight_image_bytes(const mi355q_q8_weight *weight); /* N*K + N*(K/64)*4 */
int mi355q_q8_linear(mi355q_context *ctx, const mi355q_q8_weight *weight, const void *x,
                     int x_dtype, uint32_t M, void *y, int y_dtype, const void *residual,
                     int residual_dtype, uint32_t flags, char *error, size_t error_capacity);

/* ---- Qwen3.8 image files --------------------------------------------------------
 * The reference's Apple M3 target keeps the model in four kinds of image file: a
 * 4096-byte header, then per linear a code plane and a {fp16 scale, fp16 bias}
 * metadata plane at the offsets the header names:
 *   kind 0 "layer"     (.q38delta, magic "Q38M3Q4\0", versions 3 and 2 = MLP only):
 *                      gate, up, down, delta_input, delta_output   (qwen38_m3_image.h:26-87)
 *   kind 1 "attention" (.q38att, "Q38M3ATT"): gate, up, down, attention_input,
 *                      attention_output                            (qwen38_m3_attention_image.h:21-70)
 *   kind 2 "global"    (.q38global, "Q38M3GLB"): embedding, lm_head (qwen38_m3_global_image.h:15-44)
 *   kind 3 "mtp"       (.q38mtp, "Q38M3MTP"): fc                    (qwen38_m3_mtp_image.h:16-45)
 * mi355q_q38_image_open takes the bytes of one such file (read or mapped by the caller,
 * who keeps them only for the duration of the call), checks magic, version, header size,
 * group size, and that every linear's byte counts match its own row and column counts and
 * lie inside the image (anything else: status 2, as the reference's loaders refuse a bad
 * header, qwen38_m3.m:468-505, qwen38_m3_attention.m:138-160, qwen38_m3_decode.m:405-470),
 * and prepares every linear as an ordinary Q4 weight owned by the image handle.  Unlike
 * the reference it does not insist on the 27B dimensions or the source checksum.
 * Replaces the header validation and newBufferWithBytesNoCopy mapping of those files. */
typedef struct mi355q_q38_image mi355q_q38_image;
int mi355q_q38_image_open(mi355q_context *ctx, const void *bytes, size_t size,
                          mi355q_q38_image **out, char *error, size_t error_capacity);
void mi355q_q38_image_close(mi355q_q38_image *image);
int mi355q_q38_image_kind(const mi355q_q38_image *image);          /* 0..3 as above */
const char *mi355q_q38_kind_name(int kind);
uint32_t mi355q_q38_image_version(const mi355q_q38_image *image);
uint32_t mi355q_q38_image_layer_index(const mi355q_q38_image *image); /* 0 for global / mtp */
size_t mi355q_q38_image_linear_count(const mi355q_q38_image *image);
/* The index-th linear (borrowed: valid until the image is closed) and its name. */
const mi355q_q4_weight *mi355q_q38_image_linear(const mi355q_q38_image *image, size_t index,
                                                const char **name);
const mi355q_q4_weight *mi355q_q38_image_find(const mi355q_q38_image *image, const char *name);
/* The header fields the loader reads, for checking against the reference's structs:
 * field `index` of kind `kind` -> name, byte offset, size; status 2 past the end. */
int mi355q_q38_layout_field(int kind, size_t index, const char **name, uint32_t *offset,
                            uint32_t *bytes);

/* out[i][k] = scale * q + bias of row rows[i] (fp32 multiply then add, rounded once to
 * out_dtype), [count][K]: the token-embedding lookup on a Q4 table,
 * qwen38_q4_embedding_lookup (qwen38_global.metal:13-29).  MI355Q_X_DEVICE: `rows` is a
 * device pointer (ids past the table then write nothing, as in the reference; host ids
 * are checked and rejected with status 2); MI355Q_Y_DEVICE: `out` is a device pointer. */
int mi355q_q4_dequant_rows(mi355q_context *ctx, const mi355q_q4_weight *weight,
                           const uint32_t *rows, uint32_t count, void *out, int out_dtype,
                           uint32_t flags, char *error, size_t error_capacity);

/* y[m][j] = (row rows[j] of the weight) . x[m], j < count, for 1..16 activation rows (8 of
 * fp32): the linear restricted to some of its output rows.  rows == NULL takes the
 * first `count` rows (count <= N).  This is the reference's restricted-vocabulary draft head:
 * qwen38_q4_lm_head over a static low-id prefix of the vocabulary and
 * qwen38_q4_lm_head_gathered over a list of further token ids (qwen38_global.metal:39-96).
 * The weight bytes of the selected rows are read once; the arithmetic is that of
 * mi355q_q4_linear.  MI355Q_X_DEVICE / MI355Q_Y_DEVICE as there; MI355Q_SOURCE_DEVICE: `rows`
 * is a device pointer (an id past the matrix then yields 0; host ids are checked and
 * rejected with status 2).  MI355Q_ASYNC needs all three on the device. */
int mi355q_q4_linear_rows(mi355q_context *ctx, const mi355q_q4_weight *weight,
                          const uint32_t *rows, uint32_t count, const void *x, int x_dtype,
                          uint32_t M, void *y, int y_dtype, uint32_t flags,
                          char *error, size_t error_capacity);

/* y[m][n] = sum_k w[n][k] * x[m][k]  (+ residual[m][n] when residual != NULL)
 *
 * x: [M][K] of x_dtype (F16, F32 or BF16); y: [M][N] of y_dtype; residual:
 * [M][N] of residual_dtype.  The weight is evaluated as scale*q + bias without
 * rounding for M <= 16 (fp32 accumulation throughout); for larger M the weight
 * is rounded to fp16 before an fp16 matrix multiply with fp32 accumulation.
 * Activations are never rounded to fp16 as they come: at every M, rows that are
 * not fp16 are scaled by a power of two per row (undone in the epilogue), bf16
 * rows then convert exactly and fp32 rows go through the matrix units as two
 * fp16 rows, value and rounding remainder (about 22 significant bits) - the
 * reference's grouped linear and its float-activation dots keep fp32
 * activations at any row count (whisper_turbo_encoder.c:128-176;
 * qwen38_m3_layer.m:375-393).
 * Replaces: cpu_row_dot / qwen38_q4_matvec (qwen38_m3.m:102-121;
 * qwen38_q4.metal:111-127), qwen38_q4_down_residual (qwen38_q4.metal:163-191),
 * the batched qwen38_prefill_q4_gemm_f16* family (qwen38_prefill.metal:144-248,
 * 797-1502) and minimax_h3_m3_run_q4_projection_bf16 (minimax_h3_m3_gemm.h:58-66). */
int mi355q_q4_linear(mi355q_context *ctx, const mi355q_q4_weight *weight,
                     const void *x, int x_dtype, uint32_t M,
                     void *y, int y_dtype,
                     const void *residual, int residual_dtype,
                     uint32_t flags, char *error, size_t error_capacity);

/* mi355q_q4_linear for callers that cannot allocate device memory while they run: tight
 * serving loops, harnesses that forbid hipMalloc, hosts whose allocator must stay quiet
 * between two points (the call runs on the context's own stream, so it is not a node a
 * caller's graph capture could record; mi355q_q4_sequence_record is the graph path).  No
 * counterpart in the reference.  Same result as mi355q_q4_linear, bit for bit (same kernels, same launch
 * shapes), for 1..16 activation rows (8 of fp32); x, y and residual are DEVICE pointers
 * (the *_DEVICE flags are implied), x 16-byte aligned.  It calls no hipMalloc / hipFree
 * and no other allocating routine: what the ordinary call keeps in growable staging
 * buffers — activations converted to fp16 (bf16 / fp32 x), the fp32 partial sums of K
 * slices, their arrival counters — lives in one fixed array of 3 MiB + 16 KiB that the library
 * holds on every GPU it is loaded on until the process ends.  Limits (status 2 beyond
 * them): 256 + rows * K * 2 <= 1 MiB for x that is not fp16 (rows = 2 M for fp32), and
 * slices * M * N * 4 <= 2 MiB when the launch is cut in K slices (the 27B down projection
 * at M = 16: 0.94 MiB).  Refused (status 2) while mi355q_profile_begin is active.
 * Flags: MI355Q_ASYNC, MI355Q_RESIDUAL_IS_BIAS.  All calls on one GPU share the array,
 * which keeps what the last call left (the counters a launch uses are cleared by a small
 * kernel in front of it): two such calls in flight at once on one GPU — two contexts, two
 * threads — race on it; serialise them. */
int mi355q_q4_linear_noalloc(mi355q_context *ctx, const mi355q_q4_weight *weight,
                             const void *x, int x_dtype, uint32_t M,
                             void *y, int y_dtype,
                             const void *residual, int residual_dtype,
                             uint32_t flags, char *error, size_t error_capacity);

/* One activation matrix against up to four weights that share K and the
 * metadata kind, in ONE kernel launch for M <= 16: y_t = x * w_t^T (+ residual_t).
 * This is how a decoder layer uses the path — q, k and v read the same x, and
 * so do gate and up (the reference fuses them the same way: one 14336-row
 * q|k|v matrix, qwen38_m3_attention_image.h:11-14; qwen38_q4_gate_up_silu,
 * qwen38_q4.metal:129-151) — and it spares the small matrices their own launch.
 * For M > 16 the targets run one after the other. */
typedef struct {
    const mi355q_q4_weight *weight;
    void *y;              /* [M][N_t] of y_dtype */
    const void *residual; /* [M][N_t] of residual_dtype, or NULL */
} mi355q_q4_target;

int mi355q_q4_linear_multi(mi355q_context *ctx, const mi355q_q4_target *targets,
                           uint32_t count, const void *x, int x_dtype, uint32_t M,
                           int y_dtype, int residual_dtype, uint32_t flags,
                           char *error, size_t error_capacity);

/* A run of (multi-)linears queued back to back on the context's stream with one
 * host call, all pointers on the device and nothing waited for — the way the
 * reference encodes every matvec of a forward pass into one command buffer
 * before committing it (qwen38_m3_decode.m:1614-1699).  Stops at the first
 * call that fails and reports its index in the message.
 *
 * With the context option "chain" = "1", two consecutive calls of the form  {gate, up} with
 * MI355Q_FUSE_GATE_UP_SILU writing fp16, then one weight whose x is that output (fp16, same
 * M <= 16; fp16 or bf16 x for the first) - the MLP of a decoder layer as the reference encodes
 * it, mlp_gate_up then mlp_down with nothing between them (qwen38_m3_layer.m:314-336) - go
 * out as ONE kernel launch when the launch shapes of the two linears allow it: the second
 * linear's workgroups ask for their first weights at once and start multiplying when the
 * first linear's outputs for their K slice are complete.  Same bits as the two launches.
 * The wait is bounded; if a wave ever gives up, the next call that waits for the stream
 * (mi355q_sync, mi355q_download, mi355q_timer_end, mi355q_profile_end) returns status 1 and
 * the outputs are not valid.  Not used while a sequence is being recorded into a graph. */
typedef struct {
    const void *x;
    uint32_t M;
    int x_dtype, y_dtype, residual_dtype;
    uint32_t target_count; /* 1..4 */
    mi355q_q4_target targets[4];
    uint32_t flags; /* MI355Q_RESIDUAL_IS_BIAS, MI355Q_FUSE_GATE_UP_SILU or 0 */
} mi355q_q4_call;

int mi355q_q4_linear_sequence(mi355q_context *ctx, const mi355q_q4_call *calls,
                              size_t count, char *error, size_t error_capacity);

/* The same run of calls recorded once into a HIP graph and replayed with one host call
 * per run: for loops whose kernels are shorter than the host's per-launch cost (a small
 * model's decode step).  Recording executes the calls once (which also sizes the
 * library's staging buffers), then captures them; replays use the recorded pointers and
 * shapes.  A replay is asynchronous on the context's stream.  If a later call makes the
 * context grow a staging buffer, recorded graphs refuse to launch (status 2): record
 * again.  The counterpart of the reference committing one pre-encoded command buffer per
 * token (qwen38_m3_decode.m:1614-1716). */
int mi355q_q4_sequence_record(mi355q_context *ctx, const mi355q_q4_call *calls, size_t count,
                              mi355q_graph **out, char *error, size_t error_capacity);
int mi355q_graph_launch(mi355q_context *ctx, mi355q_graph *graph,
                        char *error, size_t error_capacity);
void mi355q_graph_destroy(mi355q_graph *graph);

/* ---- drop-ins with the reference's own hook signatures ----------------------
 *
 * The portable runtimes call their Q4 linear through two compile-time hooks
 * that take the raw record pointer of the mapped image on every call.  These
 * two functions have those argument lists (plus an int status where the
 * reference returns void) and can be bound by a one-line macro or wrapper in the
 * target's kernel header.  They run on a process-wide context on device 0,
 * created on first use, and prepare each distinct `weights` pointer once (the
 * image is mapped read-only for the life of the process, so the pointer
 * identifies the tensor); activations and outputs are host arrays, fp32.
 * Status and message of the last failing call: mi355q_hook_last_error.
 * mi355q_hook_release frees the cached weights and the context. */

/* whisper_turbo_q4_gemm (whisper_turbo_a113x_kernels.h:270-280), called from
 * linear_any when WHISPER_TURBO_HAVE_Q4_GEMM is defined
 * (whisper_turbo_encoder.c:160-176): output[r][n] = bias[n] + sum_k w[n][k] *
 * input[r][k], row-major records, bias may be NULL. */
int mi355q_hook_q4_gemm(const unsigned char *weights, const float *input, size_t rows,
                        size_t input_width, size_t output_width, const float *bias,
                        float *output);
/* q4_gemv (qwen35_task.c:318-362) with the descriptor's fields passed flat:
 * output[n] = sum_k w[n][k] * input[k]; record_order as above. */
int mi355q_hook_q4_gemv(const unsigned char *records, int record_order, size_t rows,
                        size_t columns, const float *input, float *output);
int mi355q_hook_last_error(char *message, size_t capacity);
void mi355q_hook_release(void);


/* ---- W8A8: per-token int8 activations x per-output-row int8 weights ---------
 *
 * rows_with_scale: [N][4 + K] bytes, each row an fp32 scale followed by K int8
 * weights — the Q8 tensor payload of the MMOSENS1 image
 * (minimindo_audio_encoder.c:90,216-217; written by
 * compiler/compile_minimindo_sensevoice_image.py:38-46).  K must be a non-zero
 * multiple of 16.  Replaces the tensor lookup `row()` for the GPU path. */
int mi355q_w8a8_weight_prepare(mi355q_context *ctx, const void *rows_with_scale,
                               uint32_t N, uint32_t K, uint32_t flags,
                               mi355q_w8a8_weight **out,
                               char *error, size_t error_capacity);
void mi355q_w8a8_weight_destroy(mi355q_w8a8_weight *weight);

/* Per-token symmetric quantization of x[M][K] (fp32): scales[m] = max|x[m]|/127,
 * q = (int8) round_half_even(x * (1/scale)); an all-zero row gives zero codes
 * and scale 0.  Bit-exact with quantize_i8 / quantize_sequence_i8
 * (minimindo_audio_encoder.c:186-215,291-297).  flags: 0 for host pointers, or
 * MI355Q_X_DEVICE|MI355Q_Y_DEVICE (x, q and scales all on the device),
 * optionally with MI355Q_ASYNC. */
int mi355q_quantize_i8(mi355q_context *ctx, const float *x, uint32_t M, uint32_t K,
                       int8_t *q, float *scales, uint32_t flags,
                       char *error, size_t error_capacity);

/* The quantized input windows of a streaming causal convolution: for every position t the
 * window [channels][kernel] of input[in][t-(kernel-1)+k] (input is channel-major
 * [channels][length]; samples before the start come from history [channels][kernel-1], or
 * are zero when history is NULL), quantized per position like mi355q_quantize_i8:
 * q [length][channels*kernel], scales [length].  Bit-exact with causal_q8_windows
 * (minimindo_mimi.c:552-598); with MI355Q_WINDOWS_PAIRS the windows are those of
 * deconv_q8_windows (:631-670): [input[in][t] for all in, then input[in][t-1] or
 * history[in]], `kernel` ignored.  Followed by mi355q_w8a8_linear with
 * MI355Q_W8A8_CHANNEL_MAJOR on the convolution's Q8 weight [out][channels*kernel] this is
 * stream_conv1d (:882-917) without the history update, which stays with the caller.
 * flags as for mi355q_quantize_i8. */
int mi355q_causal_q8_windows(mi355q_context *ctx, const float *input, const float *history,
                             uint32_t channels, uint32_t kernel, uint32_t length,
                             int8_t *q, float *scales, uint32_t flags,
                             char *error, size_t error_capacity);

/* out[m][n] = ((float)acc[m][n] * weight_scale[n]) * x_scales[m] + bias[n], with
 * acc[m][n] = sum_k w[n][k] * q[m][k] in int32; bias may be NULL; when `acc` is
 * not NULL the int32 accumulators are written there as well.  Replaces
 * matrix_sequence_i8_quantized (minimindo_audio_encoder.c:267-306): same
 * argument meaning, position-major fp32 output.  flags as for
 * mi355q_quantize_i8 (all pointers host, or all device). */
int mi355q_w8a8_linear(mi355q_context *ctx, const mi355q_w8a8_weight *weight,
                       const int8_t *q, const float *x_scales, uint32_t M,
                       const float *bias, float *out, int32_t *acc, uint32_t flags,
                       char *error, size_t error_capacity);

/* Up to four weights of the same K against one quantized activation, in one
 * launch: the reference quantizes a layer's normalised input once and multiplies
 * it with the q, k and v weights in turn (minimindo_audio_encoder.c:400-403);
 * here the three products share the launch as well.  Each target is one
 * mi355q_w8a8_linear call's (weight, bias, out, acc). */
typedef struct mi355q_w8a8_target {
    const mi355q_w8a8_weight *weight;
    const float *bias; /* [N] or NULL */
    float *out;        /* [M][N] */
    int32_t *acc;      /* [M][N] or NULL */
} mi355q_w8a8_target;
int mi355q_w8a8_linear_multi(mi355q_context *ctx, const mi355q_w8a8_target *targets,
                             uint32_t count, const int8_t *q, const float *x_scales,
                             uint32_t M, uint32_t flags, char *error, size_t error_capacity);

#ifdef __cplusplus
}
#endif

#endif
