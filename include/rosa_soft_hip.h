/*
 * C ABI of librosa_soft_hip.so: the MI355X (gfx950) device side of the
 * rosa_soft / rosa_soft_varlen training operators.
 *
 * Plain pointers and sizes only.  Every pointer is a DEVICE pointer unless the
 * comment says otherwise; `stream` is a hipStream_t passed as void*.  Nothing
 * here synchronises with the host and nothing allocates: the caller owns the
 * outputs and the workspace.  All entry points return 0 on success or a
 * non-zero code; rosa_hip_last_error() then describes the failure (thread
 * local).
 *
 * Each entry point replaces one launcher of the reference
 * (/root/reference/rosa_soft/csrc/cuda/rosa_soft_kernels.cu), cited below.
 * The dispatcher layer above it (rosa_soft_amd/csrc/rosa_dispatch.cpp) plays
 * the role of the reference's rosa_soft/csrc/rosa_soft.cpp:379-549.
 */
#ifndef ROSA_SOFT_HIP_H_
#define ROSA_SOFT_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type of query/key/value/grad_output/output */
enum { ROSA_DTYPE_F32 = 0, ROSA_DTYPE_F16 = 1, ROSA_DTYPE_BF16 = 2 };

/* gradient_mask bits, as in the reference (rosa_soft_kernels.cu:24-26) */
enum { ROSA_GRAD_QUERY = 1, ROSA_GRAD_KEY = 2, ROSA_GRAD_VALUE = 4 };

/*
 * Problem description shared by all entry points.
 *   dense  layout: query/key [B,T,H,D], value [B,T,Hv,Dv]; set S = 0,
 *                  cu_seqlens = NULL, N = B*T.
 *   packed layout: query/key [N,H,D], value [N,Hv,Dv], cu_seqlens int32 [S+1]
 *                  on the device; set B = 0, T = 0.
 * W is max_suffix_length already clamped to T (dense) or N (packed).
 */
typedef struct rosa_problem {
  int dtype;
  int B, T;      /* dense only */
  int N, S;      /* packed token count, number of packed sequences */
  int H, D;      /* query/key heads and symbol width (1..32) */
  int Hv, Dv;    /* value heads (H % Hv == 0) and value width */
  int W;
  const int32_t* cu_seqlens; /* device, packed layout only */
} rosa_problem;

/* Library version (major*10000 + minor*100 + patch) and build target string. */
int rosa_hip_version(void);
const char* rosa_hip_target(void);
const char* rosa_hip_last_error(void);

/*
 * Workspace sizes in bytes for the calls below (host-side arithmetic only).
 * `dropout` is non-zero when dropout_p > 0.
 */
size_t rosa_hip_forward_workspace_bytes(const rosa_problem* problem);
size_t rosa_hip_vjp_workspace_bytes(const rosa_problem* problem, int gradient_mask,
                                    float scale, int dropout);

/*
 * Upper bound in bytes on the chunk records (evidence checkpoints and dropout keep
 * decisions) that the backward workspace holds between its two passes; the default is
 * 4 GiB, (size_t)-1 restores it, 0 forbids the records.  A backward whose records do not
 * fit recomputes instead (forward sweeps and a second hash evaluation in the gradient
 * pass): same results, less memory, more time.  Process-wide; call it before sizing the
 * workspace, and not while another thread sizes a workspace or runs a backward: the value
 * is read atomically, but a size query and the launch it was made for must see the same
 * one.  The reference has no counterpart (its backward keeps no state between
 * kernels); the knob exists for callers that must bound the workspace.
 */
void rosa_hip_set_record_budget(size_t bytes);

/*
 * Waves per block of the backward's gradient kernel: 1, 2, or 0 for the library's choice by
 * shape (the default).  With two waves the blocks own pairs of neighbouring diagonal bands
 * and add their column sums in LDS before the global atomics.  The reference has no
 * counterpart (one block per row there); the knob exists for measurements and so that
 * tests can run both forms on small problems.  Process-wide, with the same rule as the
 * record budget: do not change it between a size query and its launch, nor while another
 * thread does either.
 */
void rosa_hip_set_gradient_block_waves(int waves);

/*
 * Rows of a piece of a diagonal band in the backward's gradient kernel: 0 for the library's
 * choice by shape (the default: bands are cut only when there are fewer than two of them per
 * resident wave, into pieces of at least four windows), -1 for never, or a number of rows
 * (rounded up to whole 32-row segments, at least 64).  Pieces of one band are walked by
 * different waves, each starting max_suffix_length - 1 rows below its last row.  No
 * counterpart in the reference; the knob exists for measurements and so that tests can
 * force cuts on small problems.  Like the other setters it must not race with size queries
 * or launches of other threads.
 */
void rosa_hip_set_gradient_piece_rows(int rows);

/*
 * How the hard forward finds its routes: 0 (the default) = through an index of the keys by
 * symbol where the shape suits it (symbols of six bits or more, sequences of 512 tokens or
 * more, in a packed batch on average; a row then visits only the routes whose key symbol equals its own, and row blocks
 * that this does not suit are handed back to the scan over all routes), 1 = always the scan
 * over all routes, 2 = the index with every row block handed back, 3 = the index at every
 * shape (2 and 3 are for tests).  The routes are the same in every mode.  The workspace
 * size does not depend on the mode.  No
 * counterpart in the reference (its forward kernel steps over every route,
 * rosa_soft_kernels.cu:367-531); the knob exists for measurements and tests, with the
 * thread rule of the other setters.
 */
void rosa_hip_set_forward_index(int mode);

/*
 * How the backward's gradient kernel will be launched for `problem` (no counterpart in the
 * reference): waves per block (1 or 2), whether row tiles are queued between the two bands
 * of a block, and the dynamic LDS of a block in bytes.  Any of the three may be NULL.
 * Benchmarks use it to count the global atomics of a launch.
 */
int rosa_hip_gradient_block_plan(const rosa_problem* problem, int* waves, int* row_queue,
                                 size_t* lds_bytes);

/*
 * Whether and how the gradient kernel will cut the diagonal bands of `problem` into pieces
 * (no counterpart in the reference; see rosa_hip_set_gradient_piece_rows): `piece_rows` is
 * the length of a piece in rows, 0 for whole bands, `pieces` the work items per band.  Host
 * arithmetic only; returns 0 or a problem-check status.
 */
int rosa_hip_gradient_piece_plan(const rosa_problem* problem, int* piece_rows, int* pieces);

/*
 * Measurement aid, no counterpart in the reference: the rate at which this GPU performs
 * global float atomic adds in the access pattern of the backward's gradient flush
 * (16 x 16 tiles at random rows of `buffer`, rows `row_floats` floats apart, `columns` <= 16
 * floats of every row touched).  The result is in row segments per second: the atomics of
 * one wave instruction that fall into one row count once, whatever their number, which is
 * how the hardware bounds them.  `buffer` is device memory of `buffer_bytes` bytes that the
 * call overwrites; the call synchronises the stream.
 */
int rosa_hip_measure_atomic_rate(void* buffer, size_t buffer_bytes, int row_floats, int columns,
                                 double* segments_per_second, void* stream);

/*
 * Exact hard forward.  Replaces hard_forward_cuda (rosa_soft_kernels.cu:1766-1834)
 * and hard_forward_varlen_cuda (:1837-1920): sign-packs query and key into
 * head-major int32 words (dense [B,H,T], packed [H,N]), finds the
 * latest-longest route of every row and gathers sign(value[route]) (exact zero
 * for the null route) into `output` (same dtype as the inputs).
 * `routes` is optional (may be NULL): int32 in the packed-symbol layout, the
 * selected route index local to its sequence, 0 for null.  The reference's
 * device API has no such output; it exists so that index parity can be
 * checked.
 */
int rosa_hip_hard_forward(const rosa_problem* problem, const void* query,
                          const void* key, const void* value, void* output,
                          int32_t* packed_query, int32_t* packed_key,
                          int32_t* routes, void* workspace,
                          size_t workspace_bytes, void* stream);

/*
 * Hard forward that also reports what it selected: `routes` as above and
 * `lengths`, the exact matched suffix length of the selected route (0 for the
 * null route), both optional int32 tensors in the packed-symbol layout.  This
 * is the selected-route part of inspect_rosa_soft (rosa_soft/testing.py:28-117:
 * selected_route_indices, and exact_suffix_lengths taken at the selected route)
 * without its O(T^2) tensors, so route statistics such as
 * examples/fit_soft_reference.py:419-459 can be computed at training shapes.
 */
int rosa_hip_hard_routes(const rosa_problem* problem, const void* query,
                         const void* key, const void* value, void* output,
                         int32_t* packed_query, int32_t* packed_key,
                         int32_t* routes, int32_t* lengths, void* workspace,
                         size_t workspace_bytes, void* stream);

/*
 * Hard forward whose result leaves as bits instead of ternary elements, for the step that
 * follows the operator in its callers (the output projection of
 * examples/fit_soft_reference.py:405-417 reads the output once and can expand it in its
 * own prologue): `sign_words` uint32 [tokens][H][ceil(Dv/32)], bit d of word w set iff
 * output[..., 32 w + d] == +1, and `routed` uint8 [tokens][H], 1 where a route was
 * selected and 0 for the null route (whose words are zero): output = routed ? (bit ? +1
 * : -1) : 0.  Invalid device cu_seqlens give routed = 0xff everywhere.  Same workspace as
 * rosa_hip_hard_forward.  The reference has no such output; it replaces the element-wise
 * tail of hard_forward_cuda (rosa_soft_kernels.cu:509-530) for such a consumer.
 */
int rosa_hip_hard_forward_bits(const rosa_problem* problem, const void* query,
                               const void* key, const void* value,
                               uint32_t* sign_words, uint8_t* routed,
                               int32_t* packed_query, int32_t* packed_key,
                               void* workspace, size_t workspace_bytes, void* stream);

/*
 * Hard forward from symbol words that a producer has already written: the projections in
 * front of the operator (self.query / self.key of examples/fit_soft_reference.py:374-392)
 * can ballot the signs of their accumulators straight into the head-major word tensors
 * that pack_sign_bits_pair_kernel writes (rosa_soft_kernels.cu:202-241), and this entry
 * skips that packing pass.  `packed_query` / `packed_key` are inputs here (int32 [B,H,T] or
 * [H,N], bit i = logit i > 0); `dtype` of the problem is that of `value` and `output`.
 * The result leaves as `output` or, when `output` is NULL, as the bit form of
 * rosa_hip_hard_forward_bits (`sign_words`, `routed`).  Same workspace as
 * rosa_hip_hard_forward.
 */
int rosa_hip_hard_forward_words(const rosa_problem* problem, const int32_t* packed_query,
                                const int32_t* packed_key, const void* value, void* output,
                                uint32_t* sign_words, uint8_t* routed, int32_t* routes,
                                void* workspace, size_t workspace_bytes, void* stream);

/*
 * The projection behind the operator, fed with the bit form of its output:
 *   out[t, n] = residual[t, n] + sum_{h, d} y[t, h, d] * weight[n, h * Dv + d],
 *   y = routed ? (sign bit ? +1 : -1) : 0,
 * i.e. `residual + self.output(routed.flatten(2))` of examples/fit_soft_reference.py:415-416
 * without the ternary tensor in between: the matrix products (bfloat16 inputs, float32
 * accumulation) expand the operand that holds y from `sign_words` / `routed` in registers.
 * `weight` is the [N][H * Dv] matrix of the linear layer, `residual` (optional) and `out`
 * are [tokens][N]; all three bfloat16.  Dv must be 8, 16 or a multiple of 32, H * Dv a
 * multiple of 32 and N a multiple of 64 (other shapes expand the bits and use a library
 * product).  `weight` and `sign_words` must be 16-byte aligned, `out` and `residual`
 * 8-byte, `routed` 4-byte (error 1 otherwise).  The reference has no such kernel.
 */
int rosa_hip_project_routed_bits(const uint32_t* sign_words, const uint8_t* routed,
                                 int64_t tokens, int H, int Dv, const void* weight, int N,
                                 const void* residual, void* out, void* stream);

/*
 * rosa_hip_hard_forward for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The workspace is a 16 MiB array that lives in the
 * library's device image (one copy per GPU, held until the process ends), so the call
 * takes no workspace argument and calls no allocator; it handles problems whose forward
 * workspace fits, i.e. about tokens * H <= 4 190 000, and returns 3 with a message
 * beyond that (up to about tokens * H <= 680 000 the array also holds the index of the
 * keys, see rosa_hip_set_forward_index; beyond that the call scans all routes).  All calls on one GPU share that GPU's array: calls that overlap in time
 * on one GPU (different streams or threads) race and must be ordered by the caller.
 * The first call on a device looks up the array's address (hipGetSymbolAddress), which is
 * not a stream operation: make that call before recording the stream into a graph; every
 * later call on the device is kernel launches only.
 * Outputs and their meaning are those of rosa_hip_hard_forward.
 */
int rosa_hip_hard_forward_static(const rosa_problem* problem, const void* query,
                                 const void* key, const void* value, void* output,
                                 int32_t* packed_query, int32_t* packed_key,
                                 int32_t* routes, void* stream);

/*
 * Sign symbols of a contiguous [rows][bits] tensor, in row order: bit i of a symbol is
 * x[row, i] > 0 (so 0, -0, NaN and -inf give 0).  `symbol_bytes` = 1 writes uint8
 * symbols (bits <= 8), the input format of rosa_hip_router_update; 4 writes uint32 words
 * (bits <= 32).  Replaces pack_sign_bits of the reference's runtime front end
 * (rosa_soft/runtime.py:130-146) and, for a caller that fuses the packing into its
 * projection epilogue, stands for pack_sign_bits_pair_kernel
 * (rosa_soft_kernels.cu:202-241) without the head-major transposition.
 */
int rosa_hip_pack_symbols(int dtype, const void* logits, int64_t rows, int bits,
                          void* symbols, int symbol_bytes, void* stream);

/*
 * Dense surrogate VJP.  Replaces surrogate_vjp_cuda (rosa_soft_kernels.cu:1923-2379)
 * and surrogate_vjp_varlen_cuda (:2382-2638).  Gradients are float32 in the
 * layout of the corresponding input and are fully overwritten; pass NULL for
 * a gradient whose mask bit is clear.  `dropout_seed` is a device int64
 * scalar, read only when dropout_p > 0.  `inverse_keep` is 1.0f/(1.0f-p)
 * computed by the caller in float32 (rosa_soft.cpp:101-128).
 */
int rosa_hip_surrogate_vjp(const rosa_problem* problem, const void* query,
                           const void* key, const void* value,
                           const void* grad_output, const int32_t* packed_query,
                           const int32_t* packed_key, const int64_t* dropout_seed,
                           float scale, float dropout_p, float inverse_keep,
                           float mismatch_scale, int gradient_mask,
                           float* grad_query, float* grad_key, float* grad_value,
                           void* workspace, size_t workspace_bytes, void* stream);

/*
 * Streaming hard router: the device-resident counterpart of RosaRuntime::update_packed
 * (rosa_soft/csrc/rosa_runtime.cpp:333-487), whose per-(slot, head) suffix automaton
 * (:34-227) answers, for every new token, "which earlier key position ends the longest
 * (at most W) match of the query suffix, latest on ties".  Here every (slot, head) keeps
 * its masked query, key and payload symbols as bytes in caller-owned device memory
 * (`capacity` bytes per run, layouts [S][H][capacity] and [S][Hp][capacity]) and an
 * update appends the chunk and routes its rows against all earlier keys with the kernel
 * of the hard forward.  Outputs follow the reference: `matched_key_end` int64 [tokens][H],
 * the global key end position in the slot's history or -1; `output` uint8 [tokens][H], the
 * payload symbol after the matched key, 0 for the null route.  `chunk_offsets` [S+1]
 * (device int32) may be NULL when every slot brings `uniform_chunk` tokens.
 * `history_lengths` [S] (device int32) is read and then advanced by the chunk lengths, so
 * consecutive updates need no host traffic; the caller keeps
 * history length + chunk length <= capacity.  `longest_chunk` is the largest number of new
 * tokens of any slot (small chunks are routed by a per-row kernel).
 * `workspace` (optional) lets an update with a long chunk route through an index of the keys
 * by symbol, rebuilt by that update over every run's whole history (see
 * rosa_hip_set_forward_index; same routes): `longest_total` is then the largest history
 * length + chunk length of any slot, and `workspace_bytes` at least
 * rosa_hip_router_workspace_bytes(update), which is 0 for updates that would not use it
 * (symbols below six bits, chunks of up to 8 tokens, histories below 512 tokens).  With
 * `workspace` NULL every route is scanned.  A run that is longer than `longest_total` says
 * finds no room in the index and is scanned as well.  The workspace carries nothing from one
 * update to the next.
 * `history_lengths_out` [S] (optional, another array than `history_lengths`): the advanced
 * lengths are written there and `history_lengths` is left as it was; the caller passes that
 * array as `history_lengths` of the next update.  A decoding step (chunks of up to 8 tokens)
 * is then a single kernel launch, because no wave has to wait for the lengths to change.
 */
typedef struct rosa_router_update {
  int32_t S, H, Hp, W;
  int32_t qk_bits, payload_bits;
  int32_t capacity;
  int32_t tokens;
  int32_t longest_chunk;
  int32_t uniform_chunk;
  const int32_t* chunk_offsets;
  int32_t* history_lengths;
  uint8_t* query_history;
  uint8_t* key_history;
  uint8_t* payload_history;
  const uint8_t* query;
  const uint8_t* key;
  const uint8_t* payload;
  uint8_t* output;
  int64_t* matched_key_end;
  int32_t longest_total;
  void* workspace;
  size_t workspace_bytes;
  int32_t* history_lengths_out;
} rosa_router_update;

size_t rosa_hip_router_workspace_bytes(const rosa_router_update* update);
int rosa_hip_router_update(const rosa_router_update* update, void* stream);

/*
 * Invalid device cu_seqlens values (not starting at 0, decreasing, or not ending
 * at N) cannot be seen by the host without a synchronisation.  The reference
 * aborts the process with a device assert (rosa_soft_kernels.cu:287-308); here no
 * kernel touches a token in that case (every sequence is treated as empty) and the
 * results carry the signal: every element of `output` and of every requested
 * gradient is NaN.  The fact is also recorded in the first int32 of the workspace;
 * this call copies that word back (it synchronises `stream`) and returns it:
 * 0 = offsets were valid.
 */
int rosa_hip_read_offset_error(const void* workspace, void* stream);

/*
 * Stage timing for measurement (no counterpart in the reference, whose
 * benchmark times whole calls with CUDA events, benchmarks/rosa_soft.py:159-173).
 * While enabled, every call above brackets its stages with HIP events recorded
 * on the caller's stream, and the host waits for nothing; rosa_hip_stage_times()
 * waits for those events and returns the elapsed milliseconds of the LAST call
 * per stage (-1 for a stage that did not run).  rosa_hip_stage_totals() is for a
 * loop of calls timed as a whole: per stage it returns the summed milliseconds of
 * the runs since timing was enabled or the totals were last read (of the last 64
 * of them, if there were more) and how many runs that sum covers (0: none), and
 * starts a new sum.  Stages: 0 hard_forward (pack + route + gather),
 * 1 vjp_prepare, 2 vjp_row_max, 3 vjp_row_stats, 4 vjp_gradients,
 * 5 vjp_finalize.  Not thread safe; meant for benchmarks.
 */
int rosa_hip_stage_timing(int enable);
int rosa_hip_stage_count(void);
const char* rosa_hip_stage_name(int stage);
int rosa_hip_stage_times(float* milliseconds, int count);
int rosa_hip_stage_totals(float* milliseconds, int* runs, int count);

#ifdef __cplusplus
}
#endif
#endif /* ROSA_SOFT_HIP_H_ */
