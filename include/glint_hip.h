/*
 * glint_hip.h -- C-ABI of libglint_hip.so, the MI355X (gfx950) backend for Glinthawk's per-stage
 * Llama2 KV-cache path.
 *
 * This is the boundary a `hip` target of the reference binds to: its C++ `Operations` /
 * `LlamaOperations` / `Context` / `VirtualMemoryRegion` classes (glinthawk_amd/host/) are thin
 * wrappers over these entry points, one per method of the reference's compile-time interface
 * (models/common/ops/concept.hh:16-40, models/llama2/ops/concept.hh:15-36, models/llama2/context.hh:17-45).
 * Each declaration cites the reference method it replaces (paths relative to the reference root).
 *
 * Conventions
 *  - plain pointers and sizes only; no C++ or torch types.  Device pointers are raw HIP device
 *    addresses, `gh_stream` is a `hipStream_t` (NULL = the default stream).
 *  - every function returns GH_OK (0) or a negative gh_status; gh_last_error() gives the text for
 *    the calling thread.  The reference aborts on any device error (arch/cuda/common/ops.cu:5-19);
 *    the C++ wrappers do the same on a non-zero status.
 *  - launches are asynchronous on `stream` unless stated; gh_sync() waits.
 *  - "row" = one token's [K | V] = 2 * kv_dim elements, token-major inside a layer
 *    (models/llama2/context.hh:61-133).  A NULL row / layer pointer is the reference's *empty*
 *    context: that batch entry is skipped, exactly like the reference's ops do.
 *  - ops that take per-context tables come in two forms: `*_host` receives HOST arrays of device
 *    pointers / positions (what the reference's ops receive: models/llama2/base.hh:199-202) and
 *    stages them itself; the plain form takes tables that already live in device memory (what the
 *    stage driver and the benchmark use; one upload per step instead of one per op).
 *  - nothing here falls back to the CPU: if no gfx950 device is present every call fails.
 */
#ifndef GLINT_HIP_H
#define GLINT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* gh_stream;

/* values equal glinthawk::DataType (models/types.hh:19-24) */
typedef enum gh_dtype
{
  GH_F16 = 0,
  GH_F32 = 1,
  GH_BF16 = 2 /* declared for wire compatibility; no kernel accepts it (the reference's amd64 bf16 is an alias of fp16, arch/float.hh:13) */
} gh_dtype;

/* values equal glinthawk::CopyType (models/types.hh:127-133) */
typedef enum gh_copy_kind
{
  GH_HOST_TO_DEVICE = 0,
  GH_DEVICE_TO_HOST = 1,
  GH_DEVICE_TO_DEVICE = 2,
  GH_HOST_TO_HOST = 3
} gh_copy_kind;

typedef enum gh_status
{
  GH_OK = 0,
  GH_ERR_INVALID = -1,     /* bad argument / unsupported shape */
  GH_ERR_DEVICE = -2,      /* a HIP call failed */
  GH_ERR_NO_DEVICE = -3,   /* no gfx950 GPU visible */
  GH_ERR_OOM = -4,
  GH_ERR_WORKSPACE = -5    /* caller-provided workspace too small */
} gh_status;

/* Llama2 shape: the constants of models/llama2/variants.hh:9-32 as run-time values */
typedef struct gh_shape
{
  uint32_t dim;
  uint32_t kv_dim;
  uint32_t hidden_dim;
  uint32_t n_layers;
  uint32_t head_size;
  uint32_t n_heads;
  uint32_t n_kv_heads;
  uint32_t gqa_size;
  uint32_t vocab_size;
  uint32_t seq_len;
} gh_shape;

/* ---- runtime ------------------------------------------------------------------------------ */
int gh_init( int device );              /* selects the device, checks it is gfx950, creates staging; idempotent */
const char* gh_last_error( void );
int gh_device_name( char* out, size_t len );
int gh_sync( gh_stream stream );        /* hipStreamSynchronize (NULL: whole device) */
/* Streams and events for callers that overlap copies with compute (the reference's CUDA target keeps streams of its own,
 * arch/cuda/common/ops.cuh:78-80,100-108).  A created stream has the default priority and does not synchronise with the
 * default stream; gh_stream_wait_event makes later work on `stream` wait for what `event` recorded. */
typedef void* gh_event;
int gh_stream_create( gh_stream* out );
int gh_stream_destroy( gh_stream stream );
int gh_event_create( gh_event* out );
int gh_event_destroy( gh_event event );
int gh_event_record( gh_event event, gh_stream stream );
int gh_stream_wait_event( gh_stream stream, gh_event event );
/* Measurement support (the reference times whole calls with steady_clock, profiler.hh:153-192; on a device whose calls are
 * asynchronous the span between two points of a stream takes events): an event that keeps its time stamp, and the milliseconds
 * between two such events.  gh_event_elapsed_ms waits for `end`. */
int gh_event_create_timed( gh_event* out );
int gh_event_elapsed_ms( gh_event begin, gh_event end, float* ms );

/* Operations::device_allocate / DeviceUniquePtr deleter (arch/cuda/common/ops.cuh:27-35,748-756) */
int gh_malloc( void** out, uint64_t bytes );
int gh_free( void* ptr );
/* host-only: allocations (device memory, page-locked host memory, physical blocks of the paged arena) this library has made since the
 * process started, its own scratch buffers included; no counterpart in the reference.  Lets a caller that must not allocate check
 * that a call did not. */
uint64_t gh_allocation_count( void );
/* pinned host memory for the staging buffers of a caller (hipHostMalloc) */
int gh_host_malloc( void** out, uint64_t bytes );
int gh_host_free( void* ptr );
/* Operations::copy (arch/cuda/common/ops.cuh:758-780): byte copy; `async` != 0 returns before completion */
int gh_memcpy( void* dst, const void* src, uint64_t bytes, gh_copy_kind kind, int async, gh_stream stream );
int gh_memset_zero( void* dst, uint64_t bytes, gh_stream stream ); /* fill kernel, graph-capture safe */

/* Operations::randomize_device_buffer (arch/cuda/common/ops.cuh:782-792): uniform [lo, hi), counter-based, seeded */
int gh_fill_uniform( void* dst, uint64_t n, float lo, float hi, uint64_t seed, gh_dtype dt, gh_stream stream );
/* synthetic inputs of the benchmark configs: N(mean, std) */
int gh_fill_normal( void* dst, uint64_t n, float mean, float std, uint64_t seed, gh_dtype dt, gh_stream stream );

/* LlamaOperations::convert_and_copy (arch/cuda/llama2/ops.cuh:455-492, arch/amd64/llama2/ops.hh:354-368): n elements,
 * static_cast per element (f32 -> f16 rounds to nearest even, f16 -> f32 is exact); dst/src may each be host or device
 * as `kind` says.  Queued on `stream` and waited for before returning (the reference's is synchronous).  A converting
 * host-to-host copy is refused, as on the reference's device target. */
int gh_convert_and_copy( void* dst, gh_dtype dst_dt, const void* src, gh_dtype src_dt, uint64_t n, gh_copy_kind kind, gh_stream stream );
/* same conversion, device to device, asynchronous */
int gh_convert( void* dst, gh_dtype dst_dt, const void* src, gh_dtype src_dt, uint64_t n, gh_stream stream );

/* ---- paged KV arena: common::cuda::VirtualMemoryRegion (arch/cuda/common/vmem.cuh:22-160),
 *      amd64 semantics in arch/amd64/common/vmem.hh:43-79 ---------------------------------- */
typedef struct gh_vmm gh_vmm;
int gh_vmm_granularity( uint64_t* out );                       /* minimum commit size of the device */
int gh_vmm_reserve( gh_vmm** out, uint64_t bytes );            /* VirtualMemoryRegion(len): address range only */
void* gh_vmm_ptr( const gh_vmm* r );                           /* ptr() */
uint64_t gh_vmm_max_len( const gh_vmm* r );                    /* max_len() */
int gh_vmm_commit( gh_vmm* r, uint64_t offset, uint64_t len ); /* allocate_span(ptr()+offset, len): out of range -> GH_ERR_INVALID */
int gh_vmm_clear( gh_vmm* r );                                 /* clear(): unmap + release every committed span */
uint64_t gh_vmm_committed_bytes( const gh_vmm* r );
int gh_vmm_free( gh_vmm* r );

/* ---- common ops: models/common/ops/concept.hh:28-39 --------------------------------------- */
/* Operations::accum<size>    arch/amd64/common/ops.hh:124-137 : a = DType(float(a) + float(b)) over batch*size */
int gh_accum( void* a, const void* b, uint64_t size, uint64_t batch, gh_dtype dt, gh_stream stream );
/* Operations::rmsnorm<size>  arch/amd64/common/ops.hh:139-169 : eps 1e-5 after the mean; out may alias x */
int gh_rmsnorm( void* out, const void* x, const void* weight, uint64_t size, uint64_t batch, gh_dtype dt, gh_stream stream );
/* Operations::silu<hidden>   arch/amd64/common/ops.hh:194-210 : hb = DType(x / (1 + exp(-x)) * hb2) */
int gh_silu( void* hb, const void* hb2, uint64_t hidden_dim, uint64_t batch, gh_dtype dt, gh_stream stream );
/* Operations::argmax<n>      arch/amd64/common/ops.hh:171-192 : first index of the row maximum.
 * `out_dev` (batch uint32, device) receives the indices; if `out_host` is non-NULL they are also
 * copied there and the call synchronises (the reference writes a host array: arch/cuda/common/ops.cuh:646-650) */
int gh_argmax( uint32_t* out_host, uint32_t* out_dev, const void* v, uint64_t n, uint64_t batch, gh_dtype dt, gh_stream stream );
/* Operations::matmul<s,r> / untemplated_matmul  arch/amd64/common/ops.hh:74-93,212-271 :
 * xout(b, r) = sum_p w(r, p) * x(b, p); w row-major (r, s); fp32 accumulate */
/* tuning hook: kernel 0 auto / 1 small tiled / 2 streaming (decode) / 3 128x128 tile / 4 256-token tile (many rows); the number of compute units the
 * streaming kernel's K split is balanced for (<= 0 keeps the current value; the default is the device's own count); the 256-token tile kernel: 256 or
 * 384 weight rows per work-group of eight waves, 128 = four waves of 128 x 128 with one tile per work-group, 129 = four waves over equal shares of
 * all K steps with the fix-up kernel, 0 = the library's choice (GLINT_TILE_ROWS in the environment sets the start value) */
int gh_gemm_set_tuning( int kernel, int target_workgroups, int tile_rows );
/* measurement / test hook: waves per work-group of the decode product that computes w1 and w3 in one launch and applies the SiLU gate itself
 * (gh_matmul_silu_gate at up to 64 rows without a K split): 4, 8, or 0 = the library's choice (8 where work-groups of 4 would come two to a CU) */
int gh_gemm_set_gate_waves( int waves );
/* Opt-in: plain f16 products (gh_matmul, the two of gh_matmul_pair, the product inside gh_matmul_accum and gh_matmul_silu_gate where no
 * kernel of this library fuses it) of `rows` activation rows and more go to the vendor's GEMM library, as every product of the
 * reference's GPU target does (cublasGemmEx, arch/cuda/common/ops.cuh:666-700); from half as many rows on for weight matrices that
 * are not much wider than tall.  Default 0: never, every product runs on the kernels of this library.  A forced kernel
 * (gh_gemm_set_tuning) also keeps the vendor library out.  GLINT_LIBRARY_ROWS in the environment replaces the default. */
int gh_gemm_set_library_rows( uint64_t rows );
uint64_t gh_gemm_library_rows( void ); /* the row count in force */
/* host-only: how many products the vendor's GEMM library has run for this process so far (a declined product -- library or
 * algorithm missing -- is not counted and runs on the kernels of this library): lets a test or a benchmark say which route ran */
uint64_t gh_gemm_library_calls( void );
/* host-only query: 1 when gh_matmul_accum runs a product of this shape (16-byte aligned operands) in the large tile kernel with the residual added
 * in its epilogue, i.e. without fp32 partial sums of (b, r): the caller's test for taking the fused call on many rows */
int gh_matmul_fuses_many_rows( uint64_t s, uint64_t r, uint64_t b, gh_dtype dt );
/* host-only query: how the weight-streaming kernel would cut an (r x s) . (b x s)^T product for the initialised device (256 compute
 * units before initialisation): number of K ranges, k per range (a multiple of 256), weight rows per work-group */
int gh_gemm_stream_plan( uint64_t s, uint64_t r, uint64_t b, uint32_t* splits, uint32_t* k_per_split, uint32_t* rows_per_workgroup );
int gh_matmul( void* xout, const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, gh_stream stream );
/* Two products that share their activations, their weights one behind the other ((r_a + r_b, s) row-major, as the reference lays out
 * wq and wkv, models/llama2/base.hh:410-433): xout_a = x . w[0:r_a]^T (b, r_a), xout_b = x . w[r_a:]^T (b, r_b).  The same results as
 * two gh_matmul calls; with many rows one launch serves both, so that a narrow product does not leave the chip idle. */
int gh_matmul_pair( void* xout_a, void* xout_b, const void* x, const void* w, uint64_t s, uint64_t r_a, uint64_t r_b, uint64_t b, gh_dtype dt,
                    gh_stream stream );
/* A projection fused with the ops that follow it in the reference's layer; same arithmetic and the
 * same rounding points as the separate calls (every matmul result is rounded to DType first).
 *
 * matmul + accum [+ rmsnorm]  (post_attention_ops, models/llama2/model.hh:390-427: wo/accum/rmsnorm and w2/accum):
 *   residual(b, r) = DType(float(residual) + float(DType(x . w^T)));
 *   if norm_out: norm_out(b, r) = rmsnorm(residual) * norm_weight                                   */
int gh_matmul_accum( void* residual, const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, void* norm_out, const void* norm_weight,
                     gh_dtype dt, gh_stream stream );
/* matmul w1, matmul w3, silu  (model.hh:411-418): w13 = w1 rows followed by w3 rows, (2 * hidden, s);
 *   hb(b, hidden) = DType(silu(DType(x . w1^T)) * DType(x . w3^T))                                  */
int gh_matmul_silu_gate( void* hb, const void* x, const void* w13, uint64_t s, uint64_t hidden_dim, uint64_t b, gh_dtype dt, gh_stream stream );
/* matmul wq, matmul wkv, copy_kv_cache, apply_rope  (model.hh:326-364): wqkv = wq rows followed by wkv rows;
 *   q(b, dim) = rope(DType(x . wq^T)); cache row i = [rope(DType(x . wk^T)) | DType(x . wv^T)];
 *   kv_out (optional, (b, 2 kv_dim)) receives the unrotated [K | V] the reference keeps in its scratchpad.
 *   Rows of empty contexts (NULL) are skipped and their queries stay unrotated, as in the separate ops. */
int gh_matmul_qkv_rope_append( void* q, void* kv_out, const void* x, const void* wqkv, uint64_t s, uint64_t b, const uint32_t* pos_dev, const void* freq_real,
                               const void* freq_imag, void* const* token_rows_dev, uint32_t n_kv_heads, uint32_t gqa_size, uint32_t head_size, gh_dtype dt,
                               gh_stream stream );
/* Operations::soft_sample   arch/amd64/common/ops.hh:97-107,273-283 : rows with temperature > 0 get
 * v / T - log(-log(u)), u from a counter-based generator keyed by (seed, row, column).
 * `temperatures` is a HOST array (batch floats), as in the reference. */
int gh_soft_sample( void* v, const float* temperatures, uint64_t vocab, uint64_t batch, uint64_t seed, gh_dtype dt, gh_stream stream );

/* ---- llama2 ops: models/llama2/ops/concept.hh:29-35 ---------------------------------------- */
/* LlamaOperations::copy_kv_cache  arch/amd64/llama2/ops.hh:335-352 : row_i <- state_kv[i] (2*kv_dim elems), bit copy */
int gh_kv_append( void* const* token_rows_dev, const void* state_kv, uint64_t batch, uint32_t kv_dim, gh_dtype dt, gh_stream stream );
int gh_kv_append_host( void* const* token_rows_host, const void* state_kv, uint64_t batch, uint32_t kv_dim, gh_dtype dt, gh_stream stream );

/* LlamaOperations::apply_rope  arch/amd64/llama2/ops.hh:138-164,300-333 : rotates the K half of each
 * row in place and the query heads in `q` (batch, n_kv_heads*gqa*head_size); tables are (seq_len, head_size/2) */
int gh_rope( uint64_t batch, const uint32_t* pos_dev, const void* freq_real, const void* freq_imag, void* q,
             void* const* token_rows_dev, uint32_t n_kv_heads, uint32_t gqa_size, uint32_t head_size, gh_dtype dt, gh_stream stream );
int gh_rope_host( uint64_t batch, const uint32_t* pos_host, const void* freq_real, const void* freq_imag, void* q,
                  void* const* token_rows_host, uint32_t n_kv_heads, uint32_t gqa_size, uint32_t head_size, gh_dtype dt, gh_stream stream );

/* LlamaOperations::attention_0_gemm  arch/amd64/llama2/ops.hh:170-223 : att (batch, n_heads, seq_len),
 * entries [0, pos_i] written, the rest untouched */
int gh_attn_scores( const void* q, const void* const* layer_rows_dev, void* att, uint64_t batch, const uint32_t* pos_dev,
                    const gh_shape* shape, gh_dtype dt, gh_stream stream );
int gh_attn_scores_host( const void* q, const void* const* layer_rows_host, void* att, uint64_t batch, const uint32_t* pos_host,
                         const gh_shape* shape, gh_dtype dt, gh_stream stream );
/* LlamaOperations::attention_softmax  arch/amd64/llama2/ops.hh:110-132,283-298 : over [0, pos_i] of every head row */
int gh_attn_softmax( void* att, const uint32_t* pos_dev, uint64_t batch, const gh_shape* shape, gh_dtype dt, gh_stream stream );
int gh_attn_softmax_host( void* att, const uint32_t* pos_host, uint64_t batch, const gh_shape* shape, gh_dtype dt, gh_stream stream );
/* LlamaOperations::attention_2_gemm  arch/amd64/llama2/ops.hh:225-281 : xb (batch, dim) */
int gh_attn_pv( const void* att, const void* const* layer_rows_dev, void* xb, uint64_t batch, const uint32_t* pos_dev,
                const gh_shape* shape, gh_dtype dt, gh_stream stream );
int gh_attn_pv_host( const void* att, const void* const* layer_rows_host, void* xb, uint64_t batch, const uint32_t* pos_host,
                     const gh_shape* shape, gh_dtype dt, gh_stream stream );

/* Fused decode attention = attention_0_gemm + attention_softmax + attention_2_gemm of
 * Llama2::attention_ops (models/llama2/model.hh:354-387) without the `att` scratch: split-K over the
 * cached rows with an online softmax, partial (max, sum, out) per split merged by a second kernel.
 * q must already be rotated (gh_rope) and the current row appended (gh_kv_append).
 *   layer_rows_dev[i]  base of context i's rows for this layer (NULL: skipped, xb row untouched)
 *   pos_dev[i]         position of the current token; keys [0, pos_i] are attended
 *   max_pos            host-side upper bound of pos (sizes the grid; seq_len - 1 if unknown); a context whose position lies
 *                      beyond it is attended over the keys the grid covers only, never outside the workspace
 *   workspace          device scratch of at least gh_attn_decode_workspace() bytes
 *   variant            GH_ATTN_AUTO, or force a kernel (tests / measurements) */
typedef enum gh_attn_variant
{
  GH_ATTN_AUTO = 0,
  GH_ATTN_GENERIC = 1, /* any head_size <= 256, any gqa, f16 / f32 */
  GH_ATTN_VALU = 2,    /* f16, head_size 128, wave-per-kv-head dot2/DPP kernel */
  GH_ATTN_MFMA = 3     /* f16, head_size 128, gqa in [2, 16]: MFMA score / weighted-sum tiles */
} gh_attn_variant;

/* tokens per split of the fused kernel; 0 (default) lets the library choose from the batch shape */
int gh_attn_set_chunk( uint32_t tokens_per_split );
/* measurement / test hook.  1 (default): a plan of 2 or 4 splits on the f16 head-128 kernels whose waves are all resident at once makes the splits of a
 * (context, kv head) stream waves of one work-group, which adds them up itself: no partial sums in the workspace, no merge kernel, results within one
 * rounding of the two-kernel route.  4, 8: that route with work-groups of 4 or 8 waves for every plan of 2 or 4 splits.  0: every split plan writes
 * partial sums and runs the merge kernel. */
int gh_attn_set_split_join( int on );
/* measurement hook: which kernel GH_ATTN_AUTO picks where the shape permits it (GH_ATTN_AUTO restores the library's choice) */
int gh_attn_set_auto_variant( int variant );
/* bytes that serve every call with at most `batch` rows and positions up to `max_pos` (a smaller batch is cut into more splits per context, so the
 * largest need over all batch sizes in [1, batch] is returned) */
uint64_t gh_attn_decode_workspace( uint64_t batch, uint32_t max_pos, const gh_shape* shape );
/* host-only query: how gh_attn_decode would cut this call (tokens per split, splits of the longest context) and the workspace bytes it would use
 * (0 for a plan whose splits are added up inside the work-groups) */
int gh_attn_decode_plan( uint64_t batch, uint32_t max_pos, const gh_shape* shape, gh_dtype dt, int variant, uint32_t* tokens_per_split, uint32_t* max_splits,
                         uint64_t* partial_bytes );
/* host-only query: waves per work-group if gh_attn_decode would add the splits of this call up inside its work-groups (no partial sums, no merge
 * kernel: see gh_attn_set_split_join), 0 if it would write partial sums to the workspace and run the merge kernel, or needs no split at all */
uint32_t gh_attn_decode_join_waves( uint64_t batch, uint32_t max_pos, const gh_shape* shape, gh_dtype dt, int variant );
int gh_attn_decode( const void* q, const void* const* layer_rows_dev, const uint32_t* pos_dev, void* xb, uint64_t batch,
                    uint32_t max_pos, const gh_shape* shape, gh_dtype dt, void* workspace, uint64_t workspace_bytes,
                    int variant, gh_stream stream );
/* gh_attn_decode without a workspace argument and without any allocation.  It has no counterpart in the reference; it is
 * for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  The split partials go to a fixed array in the library's device image instead
 * (gh_attn_decode_static_limit() bytes, 16 MiB, per GPU, held until the process ends); a call whose plan needs more
 * (see gh_attn_decode_plan) fails with GH_ERR_WORKSPACE.  Same kernels, same plan, same result as gh_attn_decode.
 * gh_init() must have been called before: this entry point never initialises the library, because that allocates.
 * All calls on one GPU share the one array: calls that overlap in time on one GPU (two streams, two threads) race.
 * Nothing in the array needs clearing between calls: every partial that the merge reads was written by the same call. */
uint64_t gh_attn_decode_static_limit( void );
int gh_attn_decode_static( const void* q, const void* const* layer_rows_dev, const uint32_t* pos_dev, void* xb, uint64_t batch, uint32_t max_pos,
                           const gh_shape* shape, gh_dtype dt, int variant, gh_stream stream );
/* Decode attention for batches whose contexts differ in length (the same result as gh_attn_decode: attention_0_gemm, attention_softmax
 * and attention_2_gemm of arch/amd64/llama2/ops.hh:170-298 in one pass; the reference runs one task per (context, kv head),
 * ops.hh:192-193, whatever their lengths).  The keys of all contexts are cut into equal runs, one per resident work-group, so that
 * no CU is left with the longest contexts while others idle.  f16, head size 128, gqa in {1, 2, 4, 8, 16}.
 *   gh_attn_balanced_workspace  bytes for the cuts and the partial results of `batch` contexts (needs the device: 0 on failure)
 *   gh_attn_balance             makes the cuts from the positions (pos_dev[i] = position of the current token, keys [0, pos_i];
 *                               contexts with a NULL row in layer_rows_dev have none); once per step: the cuts do not depend on the layer
 *   gh_attn_decode_balanced     one layer, with the cuts gh_attn_balance left in `workspace`; layer_rows_dev must have its NULL
 *                               rows where that call's table had them.  Calls on one workspace must not overlap in time. */
uint64_t gh_attn_balanced_workspace( uint64_t batch, const gh_shape* shape );
int gh_attn_balance( const void* const* layer_rows_dev, const uint32_t* pos_dev, uint64_t batch, uint32_t max_pos, const gh_shape* shape, void* workspace,
                     uint64_t workspace_bytes, gh_stream stream );
int gh_attn_decode_balanced( const void* q, const void* const* layer_rows_dev, void* xb, uint64_t batch, uint32_t max_pos, const gh_shape* shape, gh_dtype dt,
                             void* workspace, uint64_t workspace_bytes, gh_stream stream );
int gh_attn_decode_host( const void* q, const void* const* layer_rows_host, const uint32_t* pos_host, void* xb, uint64_t batch,
                         const gh_shape* shape, gh_dtype dt, void* workspace, uint64_t workspace_bytes, int variant, gh_stream stream );

/* Batched prefill (no counterpart in the reference, which feeds prompts one token per forward:
 * frontend/infer.cc:124-125, models/llama2/model.hh:356-357).  `n_tokens` new tokens per context at
 * positions [start_pos_i, start_pos_i + n_tokens); activations are (batch * n_tokens, dim) with row
 * index context * n_tokens + token.  The result equals n_tokens sequential decode steps.
 *
 * gh_prefill_tables expands per-context tables to one entry per (context, token) -- the tables the
 * decode-style entry points (gh_matmul_qkv_rope_append, gh_kv_append, gh_rope, gh_attn_decode) take:
 *   layer_rows_out[i*T+t] = layer_rows[i], token_rows_out[i*T+t] = layer_rows[i] + (start_i + t) * row_bytes,
 *   pos_out[i*T+t] = start_i + t.  Any output may be NULL. */
int gh_prefill_tables( const void* const* layer_rows_dev, const uint32_t* start_pos_dev, uint64_t batch, uint32_t n_tokens, uint64_t row_bytes,
                       const void** layer_rows_out, void** token_rows_out, uint32_t* pos_out, gh_stream stream );
/* Causal attention of the new tokens over the cache (their rows already appended and rotated):
 * query token t of context i attends keys [0, start_i + t].  f16 / head size 128 runs a tiled MFMA
 * kernel; other shapes run the decode kernels on expanded tables (workspace needed, see
 * gh_attn_prefill_workspace).  max_start_pos: host-side upper bound of start_pos. */
uint64_t gh_attn_prefill_workspace( uint64_t batch, uint32_t n_tokens, const gh_shape* shape );
/* measurement hook: 32-column query tiles a wave of the tiled MFMA kernel owns (1: two waves per SIMD, the default; 2: one) */
int gh_attn_set_prefill_tiles( int column_tiles_per_wave );
int gh_attn_prefill( const void* q, const void* const* layer_rows_dev, const uint32_t* start_pos_dev, void* xb, uint64_t batch, uint32_t n_tokens,
                     uint32_t max_start_pos, const gh_shape* shape, gh_dtype dt, void* workspace, uint64_t workspace_bytes, int variant, gh_stream stream );

/* Timing hooks for the benchmark: HIP events recorded on `stream` around the two kernels of
 * gh_attn_decode.  gh_attn_timing_read() synchronises and returns, accumulated since
 * gh_attn_timing_reset(): milliseconds in the split-K attention kernel, milliseconds in the merge
 * kernel (0 when no split was needed) and the number of gh_attn_decode calls sampled.  on = 2: events only in front of and
 * behind the pair of kernels, nothing between them, as the pair runs in production (an event record holds the next kernel
 * back by a few microseconds); the whole span is then returned as kernel_ms and merge_ms is 0.  Read before changing the mode. */
int gh_attn_timing_enable( int on );
int gh_attn_timing_reset( void );
int gh_attn_timing_read( double* kernel_ms, double* merge_ms, uint64_t* launches );

#ifdef __cplusplus
}
#endif
#endif
