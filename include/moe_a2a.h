/*
 * moe_a2a.h — C ABI of the MI355X (gfx950) MoE dispatch/combine library.
 *
 * One rank's share of the single-node MoE all-to-all of the reference's
 * `all2all` task: count -> stable order -> pack -> [exchange] -> expert-major
 * placement -> [expert] -> gather -> [exchange] -> weighted combine.
 *
 * Conventions shared by every entry point
 *   - all pointers are DEVICE pointers unless a parameter says "host";
 *   - token rows are 2-byte elements (fp16 or bf16), `hidden_dim` of them,
 *     contiguous, rows back to back; meta rows are 5 x int32
 *     {global_expert, src_rank, src_token, src_k, pad}
 *     (reference: all2all/reference.py:56 `META_DIM = 5`);
 *   - nothing is allocated, freed or cleared by the library; every output
 *     buffer is owned by the caller; no entry point synchronises the host;
 *   - `stream` is a hipStream_t passed as void*; NULL is the null stream;
 *   - every `rows_hint` is a host-side guess of the number of rows the call
 *     will move. Kernels read the true row count from device memory and
 *     stride over it, so a hint that is too small or too large costs time,
 *     never correctness;
 *   - every `*capacity_rows` is the number of rows the named row buffer and
 *     its meta buffer were allocated with. No kernel reads or writes a row at
 *     or past it, whatever the device-side counts claim: counts that add up
 *     to more are cut off there (the reference would raise an index error).
 *     Rows between the true count and min(rows_hint, capacity) may be read
 *     before the count is known; they are never used. capacity * world_size
 *     must fit an int32 (MOE_A2A_EINVAL beyond);
 *   - return value: MOE_A2A_OK (0) or a negative MOE_A2A_E* code. Argument
 *     errors are detected before anything is launched.
 *
 * Ordering contract (what makes results identical to the reference): every
 * permutation below is a STABLE partition of its input stream, computed by
 * ranking (no atomics), so slots do not depend on scheduling.
 */
#ifndef MOE_A2A_H_
#define MOE_A2A_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE_A2A_META_DIM 5

/* element types of token rows (reference: MoEConfig.in_dtype / out_dtype,
 * all2all/reference.py:16-17) */
#define MOE_A2A_F16 0
#define MOE_A2A_BF16 1

#define MOE_A2A_OK 0
#define MOE_A2A_EINVAL (-1)   /* bad size / null pointer / unsupported value */
#define MOE_A2A_EALIGN (-2)   /* a row buffer is not 2-byte aligned */
#define MOE_A2A_ELAUNCH (-3)  /* hipGetLastError() != hipSuccess after launch */
#define MOE_A2A_ESCRATCH (-4) /* shape beyond the library's static buffer         */

/* Static shape of one rank's problem (reference: MoEConfig,
 * all2all/reference.py:10-17, and PyTorchAllToAll.__init__, :58-65). */
typedef struct moe_a2a_shape {
  int32_t world_size;        /* W; num_local_experts = num_experts / W     */
  int32_t rank;              /* this rank, 0 <= rank < W                    */
  int32_t num_experts;       /* E, multiple of W, <= 65536                  */
  int32_t experts_per_token; /* K                                           */
  int32_t hidden_dim;        /* H elements per token row                    */
  int32_t max_num_tokens;    /* per-rank token capacity; max_recv = this*W  */
} moe_a2a_shape;

/* Library version / build probe. Returns a static string such as
 * "moe_a2a 0.6 gfx950"; the number changes with the ABI. Never NULL. */
const char* moe_a2a_version(void);

/* Identifies the sources this library was built from: the first 16 hex digits of
 * the SHA-256 of the kernel source followed by this header, as the build step
 * computed it, or "unknown" for a build that did not pass it. Measurements kept
 * on file name the build they were taken on with it. Never NULL. */
const char* moe_a2a_build_id(void);

/* Human-readable text for a status code. Never NULL. */
const char* moe_a2a_strerror(int status);

/*
 * Dispatch, send side.
 * Replaces all2all/reference.py:74-86,93,100-102 (loop over indices building
 * send_counts / token_map / meta_map, then the per-destination row gather).
 *
 *   x           [num_tokens, H]  token rows
 *   indices     [num_tokens, K]  int32 global expert ids
 *   send_buf    [num_tokens*K, H] out: rows grouped by destination rank
 *                                (rank 0 first), inside a group in (t, k)
 *                                order — a stable sort of the t-major,
 *                                k-minor stream by indices[t,k] / nle
 *   send_meta   [num_tokens*K, 5] out: {e, rank, t, k, 0} per sent row
 *   send_counts [W] int32        out: rows per destination rank
 *   send_slot   [num_tokens*K]   out, optional (may be NULL): row of
 *                                send_buf that entry t*K+k went to
 * An entry whose expert id is outside [0, E) names no destination (the
 * reference indexes out of range there, all2all/reference.py:80-81): its row is
 * placed behind the rows of all destinations, in (t, k) order, and counted for
 * no rank, so it is never exchanged and adds nothing to the combine.
 */
int moe_a2a_dispatch_send(const moe_a2a_shape* shape, const void* x,
                          const int32_t* indices, int32_t num_tokens,
                          void* send_buf, int32_t* send_meta,
                          int32_t* send_counts, int32_t* send_slot,
                          void* stream);

/*
 * The plan of the send side without moving any row: counts, offsets and both
 * index maps of the stable sort that moe_a2a_dispatch_send applies
 * (all2all/reference.py:79-86,93: entries grouped by destination rank, inside
 * a group in (t, k) order).
 *
 *   indices       [num_tokens, K] int32
 *   rank_counts   [W]   out: entries per destination rank (= send_counts)
 *   rank_offsets  [W+1] out: exclusive prefix of rank_counts; [W] = total
 *   expert_counts [E]   out: entries per global expert id
 *   dst_slot      [num_tokens*K] out: send row of entry t*K+k
 *   src_entry     [num_tokens*K] out: entry t*K+k held by each send row
 * Entries whose expert id is outside [0, E) are left out of every output.
 * Limits: W <= 64, E <= 8192 (MOE_A2A_EINVAL beyond).
 */
int moe_a2a_plan_send(const moe_a2a_shape* shape, const int32_t* indices,
                      int32_t num_tokens, int32_t* rank_counts,
                      int32_t* rank_offsets, int32_t* expert_counts,
                      int32_t* dst_slot, int32_t* src_entry, void* stream);

/*
 * Dispatch, receive side: received stream -> expert-major buffers.
 * Replaces all2all/reference.py:123-146 (per received row:
 * le = meta[0] % nle; expert_x[le, cnt[le]++] = row).
 *
 *   recv_buf    [R, H]  rows as the exchange delivered them: source rank 0's
 *                       segment first, each in the sender's order
 *   recv_meta   [R, 5]
 *   recv_counts [W] int32, rows received from each source rank; R = their sum
 *   capacity_rows       rows recv_buf / recv_meta were allocated with
 *   expert_num_tokens [nle] int32 out (every entry written, zeros included)
 *   expert_x    [nle, max_recv, H] out; only rows < expert_num_tokens[le] are
 *                       written (the reference leaves the rest uninitialised
 *                       too: torch.empty at reference.py:127)
 *   expert_meta [nle, max_recv, 5] out, same rule
 *   send_back_plan [2 * num_experts] int32 out, optional (may be NULL):
 *                       where moe_a2a_combine_send will put every row, worked
 *                       out here because the keys are being counted anyway.
 *                       Opaque to the caller. Written only when W <= 64 and
 *                       nle <= 64 (ignored otherwise, by both entry points).
 *                       It takes the origin of a row from the segment the row
 *                       arrived in, which is what every sender writes into
 *                       meta[1] (all2all/reference.py:84).
 * A row whose position inside its expert would reach max_recv is not stored;
 * expert_num_tokens still counts it, so overflow is visible to the caller.
 */
int moe_a2a_dispatch_recv(const moe_a2a_shape* shape, const void* recv_buf,
                          const int32_t* recv_meta, const int32_t* recv_counts,
                          int32_t rows_hint, int32_t capacity_rows,
                          int32_t* expert_num_tokens, void* expert_x,
                          int32_t* expert_meta, int32_t* send_back_plan,
                          void* stream);

/*
 * moe_a2a_dispatch_recv for long streams (thousands of received rows). The
 * reference places a row with a running counter per expert
 * (all2all/reference.py:140-146); moe_a2a_dispatch_recv finds that position by
 * counting the keys ahead of the row in every workgroup, work that grows with
 * the square of the row count. Here a planning launch works the positions out
 * once (a histogram of the experts ahead of every tile of 1024 rows, ballot
 * ranks inside the tile) and the movers read them. Same arguments and the same
 * results, bit for bit, plus
 *
 *   row_position [capacity_rows] int32 workspace, overwritten: position of
 *                every received row inside its expert
 *
 * Two launches instead of one: at hidden_dim 7168 this form pays from about
 * 8192 rows (at 32768 rows: 200 us against 323 us). With more than 256 local
 * experts the call falls back to the scanning kernel.
 */
int moe_a2a_dispatch_recv_long(const moe_a2a_shape* shape, const void* recv_buf,
                               const int32_t* recv_meta, const int32_t* recv_counts,
                               int32_t rows_hint, int32_t capacity_rows,
                               int32_t* expert_num_tokens, void* expert_x,
                               int32_t* expert_meta, int32_t* send_back_plan,
                               int32_t* row_position, void* stream);

/*
 * moe_a2a_dispatch_recv with the send-back plan kept in device memory that the
 * library owns, for callers that cannot allocate: code under HIP graph
 * capture, serving loops and harnesses that must not call hipMalloc. It has no
 * counterpart in the reference. Same arguments, results and kernels as
 * moe_a2a_dispatch_recv, except that the plan is not brought by the caller:
 *
 *   send_back_plan  host pointer, out: where the call left the plan (a device
 *                   address inside the library's static buffer), to be handed
 *                   to moe_a2a_combine_send as its send_back_plan under the
 *                   same rule as a caller-owned plan. NULL on any error.
 *
 * The call allocates and frees nothing and clears nothing (every int of the
 * plan that the shape uses is written). The buffer is one static device array
 * of 2 * 4096 ints (32 KB) per GPU, held until the process ends; its address
 * is looked up once per GPU, on the first call made with that GPU current
 * (make that call outside a graph capture). Limits: world_size <= 64,
 * num_local_experts <= 64 (so num_experts <= 4096): MOE_A2A_ESCRATCH beyond,
 * before anything is launched.
 * All calls on one GPU share the buffer, which keeps what the last call wrote:
 * a second call overwrites the plan of the first, so finish (or at least
 * enqueue on the same stream) the moe_a2a_combine_send that uses a plan before
 * the next moe_a2a_dispatch_recv_static on that GPU. Calls that overlap on one
 * GPU on different streams race.
 */
int moe_a2a_dispatch_recv_static(const moe_a2a_shape* shape, const void* recv_buf,
                                 const int32_t* recv_meta, const int32_t* recv_counts,
                                 int32_t rows_hint, int32_t capacity_rows,
                                 int32_t* expert_num_tokens, void* expert_x,
                                 int32_t* expert_meta, const int32_t** send_back_plan,
                                 void* stream);

/*
 * Combine, send side: expert-major results -> rows grouped by origin rank.
 * Replaces all2all/reference.py:163-199 (loop le ascending, j < cnt[le]
 * ascending, bucket by meta[1]; concatenate buckets in rank order).
 *
 *   expert_y    [nle, max_recv, H], expert_meta [nle, max_recv, 5],
 *   expert_num_tokens [nle] (values above max_recv are clamped)
 *   send_buf    [R, H] out, send_meta [R, 5] out (meta rows copied unchanged);
 *               capacity_rows is their allocation
 *   send_counts [W] int32 out
 *               A row whose meta[1] names no rank (below 0, W or above) is
 *               counted for nobody and placed behind the rows of all origins.
 *   send_back_plan [2 * num_experts] int32, optional (may be NULL): the plan
 *               moe_a2a_dispatch_recv wrote together with this expert_meta and
 *               expert_num_tokens. With it rows are placed without reading the
 *               origin column of expert_meta, so it must be passed only while
 *               both are as that call left them (the order of the rows of an
 *               expert, the origin ranks, the counts); pass NULL after changing
 *               any of them. Results are the same with and without it.
 */
int moe_a2a_combine_send(const moe_a2a_shape* shape, const void* expert_y,
                         const int32_t* expert_meta,
                         const int32_t* expert_num_tokens, int32_t rows_hint,
                         int32_t capacity_rows, void* send_buf,
                         int32_t* send_meta, int32_t* send_counts,
                         const int32_t* send_back_plan, void* stream);

/*
 * Combine, receive side: weighted sum back into token order.
 * Replaces all2all/reference.py:227-232
 *   out_tokens[src_token] += recv_buf[i].to(float32) * weights[src_token, src_k]
 * for i in arrival order. out_tokens has the 16-bit element type, so the
 * running sum is rounded to it after EVERY addend:
 *   p = RN32(f32(v) * w);  a = RN32(f32(acc) + p);  acc = RN16(a)
 * (separate multiply and add, no fma). The kernel reproduces exactly that.
 *
 *   recv_buf    [R, H], recv_meta [R, 5], recv_counts [W] int32 (R = sum)
 *   weights     [num_tokens, K] float32
 *   out_tokens  [num_tokens, H] in/out
 *   accumulate  nonzero: start from the values already in out_tokens (the
 *               reference's in-place +=); zero: start from +0 and overwrite,
 *               which equals the reference on its zero-initialised buffer
 *               (reference.py:263-268) without reading it
 *   dtype       MOE_A2A_F16 or MOE_A2A_BF16: element type of recv_buf and
 *               out_tokens
 * Rows whose src_token or src_k is out of range are ignored.
 */
int moe_a2a_combine_recv(const moe_a2a_shape* shape, const void* recv_buf,
                         const int32_t* recv_meta, const int32_t* recv_counts,
                         int32_t rows_hint, int32_t capacity_rows,
                         const float* weights, int32_t num_tokens,
                         void* out_tokens, int32_t accumulate, int32_t dtype,
                         void* stream);

/*
 * moe_a2a_combine_recv for long streams. In moe_a2a_combine_recv every
 * workgroup of a token scans the src_token column of the whole arriving stream
 * (tokens x rows reads); here a first launch writes, for every arriving row, its
 * row number at entry_row[src_token * K + src_k], and a token's workgroups look
 * their K rows up. Same arguments, same arithmetic and order
 * (all2all/reference.py:227-232), same results bit for bit, plus
 *
 *   entry_row [num_tokens * K] int32 workspace, overwritten. It needs no
 *             clearing: an entry is used only if the meta row it names carries
 *             this token and this k in the stream of this call.
 *
 * Precondition: no (src_token, src_k) pair arrives twice, which holds for every
 * stream that came out of a dispatch (each entry of `indices` is sent once). If
 * one does, only one of the duplicates is added.
 * Two launches instead of one: it pays from about 4096 rows (at 32768 rows of
 * hidden_dim 7168: 111 us against 381 us).
 */
int moe_a2a_combine_recv_long(const moe_a2a_shape* shape, const void* recv_buf,
                              const int32_t* recv_meta, const int32_t* recv_counts,
                              int32_t rows_hint, int32_t capacity_rows,
                              const float* weights, int32_t num_tokens,
                              void* out_tokens, int32_t accumulate, int32_t dtype,
                              int32_t* entry_row, void* stream);

/*
 * Stand-in for the expert computation between dispatch and combine.
 * Replaces all2all/reference.py:262
 *   expert_y = expert_x.to(out_dtype) * (1 + rank)
 * on the valid rows only (j < expert_num_tokens[le]): per element
 *   RN_out( f32( RN_out( f32(x) ) ) * float(1 + rank) ).
 */
int moe_a2a_expert_scale(const moe_a2a_shape* shape, const void* expert_x,
                         const int32_t* expert_num_tokens, int32_t rows_hint,
                         int32_t in_dtype, int32_t out_dtype, void* expert_y,
                         void* stream);

/*
 * The expert computation between dispatch and combine as a grouped linear layer
 * over the expert-major layout: for every local expert le and every valid row
 * j < expert_num_tokens[le]
 *   expert_y[le, j, :] = expert_x[le, j, :] @ weights[le]^T (+ bias[le])
 * It fills the place of all2all/reference.py:262, where the reference has the
 * simulated expert `expert_x.to(out_dtype) * (1 + rank)` (moe_a2a_expert_scale
 * keeps that arithmetic for parity with the reference; this is what a model
 * runs there). An expert of several layers is several calls: hidden_dim ->
 * intermediate with in_dim = hidden_dim, then intermediate -> hidden_dim with
 * out_dim = hidden_dim, whose result moe_a2a_combine_send takes.
 *
 *   expert_x   [nle, max_recv, in_dim], expert_num_tokens [nle]: for the first
 *              layer what moe_a2a_dispatch_recv leaves (in_dim = hidden_dim);
 *              counts above max_recv are clamped
 *   weights    [nle, out_dim, in_dim] of the same 16-bit type: weights[le][n][k]
 *              multiplies input element k into output element n (the layout of
 *              a linear layer's weight, input index contiguous)
 *   bias       [nle, out_dim] of the same type, or NULL
 *   dtype      MOE_A2A_F16 or MOE_A2A_BF16: element type of all four
 *   expert_y   [nle, max_recv, out_dim] out; rows at or past
 *              expert_num_tokens[le] are not written
 * Arithmetic: float32 accumulation and one rounding to the 16-bit type; a bias
 * is then added to that rounded value in float32 and the sum rounded again,
 * which is what `x @ w.T + b` on 16-bit tensors does (the same as
 * moe_a2a_linear).
 * Rows are processed in blocks found from the device-side counts, so the work
 * follows the rows, not the experts. rows_hint (the rows the caller expects
 * over all experts) picks the kernel and sizes the launch, and changes no bit
 * of the result: from 56 rows per expert on average, output tiles of 128 x 128
 * (64 x 128 when those would be too few for the GPU, 256 x 256 from 768 rows
 * per expert) of the kernel behind moe_a2a_linear, numbered over the experts;
 * below, a kernel built around streaming every weight once, in blocks of 64 or
 * 128 tokens and workgroups 128 to 256 columns wide. The first call on a GPU
 * sets kernel attributes (tiles can use more LDS than a kernel gets by default):
 * make that call outside a graph capture.
 * Limits: out_dim a multiple of 32, in_dim a multiple of 8, expert_x / weights /
 * expert_y 16-byte and bias 8-byte aligned (MOE_A2A_EINVAL / EALIGN).
 * Sums are formed in float32 in the order of the matrix unit, which is not the
 * order of a CPU matmul: results lie within what float32 accumulation in any
 * order plus the roundings allow around the exact value, and are exact when
 * every order gives the same float32 sum (identity and signed permutation
 * weights, small integers).
 */
int moe_a2a_expert_gemm(const moe_a2a_shape* shape, const void* expert_x,
                        const int32_t* expert_num_tokens, int32_t rows_hint,
                        const void* weights, const void* bias, int32_t in_dim,
                        int32_t out_dim, int32_t dtype, void* expert_y,
                        void* stream);

/*
 * output[m, n] = input[m, k] @ weight[n, k]^T (+ bias[n]): the product one rank
 * computes in the reference's gemm-rs task before the reduce-scatter
 * (gemm-rs/reference.py:54-57: `torch.matmul(input, weight.T)`, then
 * `output + bias`). All tensors are of the 16-bit type `dtype` (MOE_A2A_F16 /
 * MOE_A2A_BF16), row-major, k contiguous in input and weight. Accumulation is
 * float32 with one rounding to the 16-bit type; a bias is then added to that
 * rounded value and the sum rounded again, which is what the two torch
 * statements do. bias may be NULL.
 * One of three kernels runs, picked from the shape alone (so a shape always
 * gives the same bits): for m <= 64, k >= 449 (eight steps of 64 elements) and
 * n <= 24448 (fewer than 192 tiles of 128 columns), a kernel whose
 * workgroups own 32 columns and split k over their waves (partial sums added in
 * a fixed order); else a kernel bound by the matrix cores, whose workgroups own
 * output tiles of 256 x 256, 128 x 128 or 64 x 128 (the largest that still
 * gives every compute unit work; all three add the same terms in the same
 * order); for shapes beyond their index ranges, the kernel of
 * moe_a2a_expert_gemm with one group of m rows.
 * Limits: n a multiple of 32, k a multiple of 8, input / weight / output 16-byte
 * and bias 8-byte aligned (MOE_A2A_EINVAL / EALIGN). m == 0 is a no-op.
 * The first call on a GPU sets kernel attributes (tiles can use more LDS than a
 * kernel gets by default): make that call outside a graph capture.
 * The reduce-scatter that follows in the reference (gemm-rs/reference.py:58-59)
 * is an exchange between GPUs and not part of this library.
 */
int moe_a2a_linear(const void* input, const void* weight, const void* bias, int32_t m,
                   int32_t n, int32_t k, int32_t dtype, void* output, void* stream);

/*
 * Stand-in for one (source rank -> destination rank) leg of the exchange,
 * done as a device copy on one GPU. Replaces, for that leg, the three
 * dist.all_to_all_single calls at all2all/reference.py:107-119 (dispatch)
 * and :210-222 (combine).
 *
 * Copies the segment the source holds for `dst_rank` (rows
 * [sum(send_counts[:dst_rank]), +send_counts[dst_rank])) of send_buf/send_meta
 * to rows [sum(recv_counts[:src_rank]), ...) of recv_buf/recv_meta.
 * send_counts belongs to the source rank, recv_counts to the destination;
 * the copy moves min(send_counts[dst_rank], recv_counts[src_rank]) rows.
 */
int moe_a2a_exchange_local(int32_t world_size, int32_t hidden_dim,
                           const void* send_buf, const int32_t* send_meta,
                           const int32_t* send_counts, int32_t dst_rank,
                           void* recv_buf, int32_t* recv_meta,
                           const int32_t* recv_counts, int32_t src_rank,
                           int32_t rows_hint, int32_t send_capacity_rows,
                           int32_t recv_capacity_rows, void* stream);

/*
 * The compact expert-major layout: the four entry points between the two
 * exchanges with the experts' rows back to back instead of in the reference's
 * padded buffers. all2all/reference.py:123-136 allocates
 * expert_x[nle, max_recv, H] and expert_meta[nle, max_recv, 5] with
 * max_recv = max_num_tokens * world_size rows for EVERY local expert (939 MB per
 * buffer at 32 experts, 2048 rows, hidden_dim 7168) and fills what arrives
 * (about 29 MB of it). Here row pos of local expert le lies at row
 *   expert_offsets[le] + pos
 * of buffers of compact_capacity_rows rows, with expert_offsets the exclusive
 * prefix of the rows per expert; the order of the rows (le ascending, arrival
 * order inside an expert) is the reference's. Expanding the compact buffers to
 * the padded ones reproduces what moe_a2a_dispatch_recv writes, row for row.
 *
 * compact_capacity_rows is the caller's choice: at least the rows the rank
 * receives (max_num_tokens * world_size * min(experts_per_token, nle) always
 * suffices; balanced routing delivers about max_num_tokens * experts_per_token).
 * Rows that find no room are not stored (they are the last of the (le, pos)
 * order); expert_num_tokens still reports every row that arrived, as in the
 * padded layout, and the three consumers below cut the counts they are given
 * to the rows that fit, so counts that add up to more than the buffers hold
 * never send a load or a store past their end. send_back_plan is used as in
 * the padded entry points (moe_a2a_combine_send_compact sets it aside by itself
 * when rows found no room).
 *
 * moe_a2a_dispatch_recv_compact: as moe_a2a_dispatch_recv, plus
 *   expert_offsets  int32[nle + 1] out: first row of every expert, the exclusive
 *                   prefix of expert_num_tokens; [nle] = rows that arrived
 *   expert_x        [compact_capacity_rows, H], expert_meta [compact_capacity_rows, 5]
 * Every mover workgroup counts the rows of lower experts over the whole stream
 * (one pass over all keys instead of the keys ahead of it), so this entry point
 * is meant for the streams of a few thousand rows the one-launch entry points
 * serve; there is no long-stream form of it.
 */
int moe_a2a_dispatch_recv_compact(const moe_a2a_shape* shape, const void* recv_buf,
                                  const int32_t* recv_meta, const int32_t* recv_counts,
                                  int32_t rows_hint, int32_t capacity_rows,
                                  int32_t* expert_num_tokens, int32_t* expert_offsets,
                                  void* expert_x, int32_t* expert_meta,
                                  int32_t compact_capacity_rows, int32_t* send_back_plan,
                                  void* stream);

/* moe_a2a_expert_scale on compact buffers: expert_x, expert_y [compact_capacity_rows, H]. */
int moe_a2a_expert_scale_compact(const moe_a2a_shape* shape, const void* expert_x,
                                 const int32_t* expert_num_tokens, int32_t rows_hint,
                                 int32_t compact_capacity_rows, int32_t in_dtype,
                                 int32_t out_dtype, void* expert_y, void* stream);

/*
 * moe_a2a_expert_gemm on compact buffers: expert_x [compact_capacity_rows, in_dim],
 * expert_y [compact_capacity_rows, out_dim]; row j of expert le is row
 * (rows of the experts below le) + j of both. The same kernels, limits and
 * arithmetic; which layout the rows lie in changes no bit of a result.
 */
int moe_a2a_expert_gemm_compact(const moe_a2a_shape* shape, const void* expert_x,
                                const int32_t* expert_num_tokens, int32_t rows_hint,
                                int32_t compact_capacity_rows, const void* weights,
                                const void* bias, int32_t in_dim, int32_t out_dim,
                                int32_t dtype, void* expert_y, void* stream);

/*
 * moe_a2a_combine_send on compact buffers: expert_y [compact_capacity_rows, H],
 * expert_meta [compact_capacity_rows, 5] as moe_a2a_dispatch_recv_compact left
 * them; capacity_rows is that of send_buf / send_meta as before.
 */
int moe_a2a_combine_send_compact(const moe_a2a_shape* shape, const void* expert_y,
                                 const int32_t* expert_meta, const int32_t* expert_num_tokens,
                                 int32_t rows_hint, int32_t compact_capacity_rows,
                                 int32_t capacity_rows, void* send_buf, int32_t* send_meta,
                                 int32_t* send_counts, const int32_t* send_back_plan,
                                 void* stream);

/*
 * The same stand-in for every source of one destination rank in one launch:
 * what the three dist.all_to_all_single calls at all2all/reference.py:88-91 and
 * :107-119 (dispatch), :181-185 and :210-222 (combine) deliver to ONE rank.
 *
 *   send_bufs, send_metas, send_counts   host arrays of world_size device
 *                 pointers: what each source rank's send half wrote
 *                 (send_counts[s] is int32[world_size] of source s)
 *   recv_buf, recv_meta   the destination's receive buffers; the rows of source
 *                 s land behind the rows of the sources below it
 *   recv_counts   int32[world_size] out: recv_counts[s] = send_counts[s][dst_rank]
 *                 (cut to send_capacity_rows), written by the same launch
 *   rows_hint     rows expected from one source (sizes the launch; any number
 *                 of rows is moved)
 *   send_capacity_rows   rows every send buffer was allocated with
 *   recv_capacity_rows   rows the receive buffers were allocated with
 * world_size <= 64 (MOE_A2A_EINVAL beyond: use one moe_a2a_exchange_local per
 * leg). One launch instead of world_size launches and a copy of the counts.
 */
int moe_a2a_exchange_gather_local(int32_t world_size, int32_t hidden_dim,
                                  const void* const* send_bufs,
                                  const int32_t* const* send_metas,
                                  const int32_t* const* send_counts, int32_t dst_rank,
                                  void* recv_buf, int32_t* recv_meta, int32_t* recv_counts,
                                  int32_t rows_hint, int32_t send_capacity_rows,
                                  int32_t recv_capacity_rows, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOE_A2A_H_ */
