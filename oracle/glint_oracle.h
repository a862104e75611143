/*
 * glint_oracle.h -- CPU restatement of Glinthawk's amd64/OpenMP Llama2 KV-cache path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke check and the
 * "cpu_baseline" leg of the benchmark may load this library, and only as the checker.  The
 * shipped HIP path never calls into it and there is no CPU fallback anywhere in the product.
 *
 * Every function restates one function of the reference (cited as file:line, relative to the
 * reference's root).  Shapes are run-time values here (the reference bakes them in as template
 * parameters).  Two storage types exist, exactly as in the reference: `f32` (DType = float) and
 * `f16` (DType = _Float16: IEEE binary16 storage, every store rounds to nearest-even, all
 * arithmetic in fp32).  Suffix `_f32` / `_f16` selects the storage type.
 *
 * Parity pinning status (what independent evidence fixes each function) is listed in the header
 * of glint_oracle.c.
 */
#ifndef GLINT_ORACLE_H
#define GLINT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t go_half; /* IEEE binary16 bit pattern */

/* Llama2 shape, mirrors the constants of models/llama2/variants.hh:9-32 */
typedef struct go_config
{
  uint64_t dim;
  uint64_t kv_dim;
  uint64_t hidden_dim;
  uint64_t n_layers;
  uint64_t head_size;
  uint64_t n_heads;
  uint64_t n_kv_heads;
  uint64_t gqa_size;
  uint64_t vocab_size;
  uint64_t seq_len;
  uint64_t attention_rounds; /* only changes the OpenMP work split, never the result */
} go_config;

/* ---- scalar conversions (binary16 <-> binary32, round-to-nearest-even) ------------------- */
float go_half_to_float( go_half h );
go_half go_float_to_half( float f );
void go_convert_f16_to_f32( float* dst, const go_half* src, uint64_t n );
void go_convert_f32_to_f16( go_half* dst, const float* src, uint64_t n );

/* ---- common ops: arch/amd64/common/ops.hh ------------------------------------------------- */
#define GO_DECLARE_COMMON( SFX, T )                                                                                    \
  void go_accum_##SFX( T* a, const T* b, uint64_t size, uint64_t batch );                                              \
  void go_rmsnorm_##SFX( T* out, const T* x, const T* weight, uint64_t size, uint64_t batch );                         \
  void go_argmax_##SFX( uint32_t* out, const T* v, uint64_t n, uint64_t batch );                                       \
  void go_silu_##SFX( T* hb, const T* hb2, uint64_t hidden_dim, uint64_t batch );                                      \
  void go_matmul_##SFX( T* xout, const T* x, const T* w, uint64_t s, uint64_t r, uint64_t b );                         \
  void go_gumbel_##SFX( T* v, const float* uniforms, const float* temperatures, uint64_t vocab, uint64_t batch );

GO_DECLARE_COMMON( f32, float )
GO_DECLARE_COMMON( f16, go_half )

/* ---- llama2 ops: arch/amd64/llama2/ops.hh ------------------------------------------------
 * `layer_ctx[i]` is the base of context i's KV rows for the current layer (LayerContext::buffer_),
 * `token_ctx[i]` the row for the current position (TokenContext::buffer_); NULL == empty context
 * (the row is skipped, exactly like the reference). */
#define GO_DECLARE_LLAMA( SFX, T )                                                                                     \
  void go_copy_kv_cache_##SFX( const go_config* c, T* const* token_ctx, const T* state_kv, uint64_t batch );           \
  void go_apply_rope_##SFX( const go_config* c,                                                                        \
                            uint64_t batch,                                                                            \
                            const uint32_t* token_positions,                                                           \
                            const T* freq_cis_real,                                                                    \
                            const T* freq_cis_imag,                                                                    \
                            T* state_q,                                                                                \
                            T* const* token_ctx );                                                                     \
  void go_attention_0_gemm_##SFX( const go_config* c,                                                                  \
                                  const T* query,                                                                      \
                                  const T* const* layer_ctx,                                                           \
                                  T* att,                                                                              \
                                  uint64_t batch,                                                                      \
                                  const uint32_t* token_positions );                                                   \
  void go_attention_softmax_##SFX( const go_config* c, T* att, const uint32_t* token_positions, uint64_t batch );      \
  void go_attention_2_gemm_##SFX( const go_config* c,                                                                  \
                                  const T* att,                                                                        \
                                  const T* const* layer_ctx,                                                           \
                                  T* xb,                                                                               \
                                  uint64_t batch,                                                                      \
                                  const uint32_t* token_positions );                                                   \
  void go_softmax_row_##SFX( T* x, uint64_t size );

GO_DECLARE_LLAMA( f32, float )
GO_DECLARE_LLAMA( f16, go_half )

/* attention_ops(): rope -> scores -> softmax -> weighted sum; models/llama2/model.hh:354-387 */
#define GO_DECLARE_ATTN_OPS( SFX, T )                                                                                  \
  void go_attention_ops_##SFX( const go_config* c,                                                                     \
                               uint64_t batch,                                                                         \
                               const uint32_t* token_positions,                                                        \
                               const T* freq_cis_real,                                                                 \
                               const T* freq_cis_imag,                                                                 \
                               T* q,                                                                                   \
                               T* const* layer_ctx,                                                                    \
                               T* att,                                                                                 \
                               T* xb );
GO_DECLARE_ATTN_OPS( f32, float )
GO_DECLARE_ATTN_OPS( f16, go_half )

/* RoPE tables, tools/bin2glint.py:19-25: cos/sin( pos * theta^(-2k/head_size) ), shape (seq_len, head_size/2) */
void go_rope_tables_f32( float* real, float* imag, uint64_t seq_len, uint64_t head_size, float theta );

/* ---- one layer / one stage of the model driver: models/llama2/model.hh:326-442,534-571 ---- */
#define GO_DECLARE_LAYER( T, SFX )                                                                                     \
  typedef struct go_layer_weights_##SFX                                                                                \
  {                                                                                                                    \
    const T* rms_att_weight; /* (dim) */                                                                               \
    const T* wq;             /* (dim, dim) row-major, row = output feature */                                          \
    const T* wkv;            /* (2*kv_dim, dim): wk rows then wv rows */                                               \
    const T* wo;             /* (dim, dim) */                                                                          \
    const T* rms_ffn_weight; /* (dim) */                                                                               \
    const T* w1;             /* (hidden_dim, dim) */                                                                   \
    const T* w2;             /* (dim, hidden_dim) */                                                                   \
    const T* w3;             /* (hidden_dim, dim) */                                                                   \
  } go_layer_weights_##SFX;                                                                                            \
  typedef struct go_scratch_##SFX                                                                                      \
  {                                                                                                                    \
    T* x;   /* (B, dim) residual stream, in/out */                                                                     \
    T* xb;  /* (B, dim) */                                                                                             \
    T* xb2; /* (B, dim) */                                                                                             \
    T* q;   /* (B, dim) */                                                                                             \
    T* kv;  /* (B, 2*kv_dim) */                                                                                        \
    T* hb;  /* (B, hidden) */                                                                                          \
    T* hb2; /* (B, hidden) */                                                                                          \
    T* att; /* (B, n_heads, seq_len) */                                                                                \
  } go_scratch_##SFX;                                                                                                  \
  /* pre_attention_ops(update_kv_cache=true) + attention_ops() + post_attention_ops() for one layer.                   \
   * layer_ctx[i] = base of this layer's rows for context i (NULL = empty). */                                         \
  void go_layer_forward_##SFX( const go_config* c, const go_layer_weights_##SFX* w, const T* freq_cis_real, const T* freq_cis_imag,            \
                               go_scratch_##SFX* s, T* const* layer_ctx, const uint32_t* token_positions, uint64_t batch );                  \
  /* classify_ops(): final rmsnorm (in place on x) + logits = x . wcls^T ; model.hh:430-442 */                        \
  void go_classify_##SFX( const go_config* c, const T* rms_final_weight, const T* wcls, T* x, T* logits, uint64_t batch );

GO_DECLARE_LAYER( float, f32 )
GO_DECLARE_LAYER( go_half, f16 ) /* every intermediate rounded to binary16 where the reference's DType = _Float16 build rounds it */

/* ---- bookkeeping models (pure integer semantics) ------------------------------------------ */

/* KV addressing, models/llama2/context.hh:61-190.  Offsets are in ELEMENTS from the context base.
 * hosted[l] != 0 iff the node hosts (layer l, Attention).  Returns UINT64_MAX for a layer that is
 * not hosted (the reference yields a null LayerContext). */
uint64_t go_ctx_layer_offset( const go_config* c, const uint8_t* hosted, uint64_t layer );
uint64_t go_ctx_token_offset( const go_config* c, const uint8_t* hosted, uint64_t layer, uint64_t pos );
uint64_t go_ctx_key_head_offset( const go_config* c, const uint8_t* hosted, uint64_t layer, uint64_t pos, uint64_t h );
uint64_t go_ctx_value_head_offset( const go_config* c, const uint8_t* hosted, uint64_t layer, uint64_t pos, uint64_t h );
uint64_t go_ctx_max_size_bytes( const go_config* c, uint64_t n_hosted_layers, uint64_t elem_size );

/* DynamicContext::prepare block accounting, context.hh:221-248.  `allocated[l]` is the committed
 * length (bytes) of layer l, updated in place.  Returns the number of 2 MiB blocks committed by
 * this call (reference: 0 or 1); *cleared is set when can_release dropped all pages first.
 * If `commit_all` is non-zero every missing block is committed (superset behaviour of the HIP
 * target); with commit_all == 0 this is the reference's one-block-per-call rule. */
uint64_t go_dynctx_prepare( const go_config* c,
                            uint64_t elem_size,
                            uint64_t* allocated,
                            uint64_t layer,
                            uint64_t token_pos,
                            int can_release,
                            int commit_all,
                            int* cleared );

/* PreallocatingContextManager, compute/contextman.hh:56-196 */
typedef struct go_ctxman go_ctxman;
go_ctxman* go_ctxman_new( uint64_t max_context_count );
void go_ctxman_delete( go_ctxman* m );
uint64_t go_ctxman_free( const go_ctxman* m );
uint64_t go_ctxman_allocated( const go_ctxman* m );
/* Two-phase batched lookup.  active[i], context_id[i] describe row i of the state, rows
 * [start, end).  On success returns 1 and writes slot indices (0..max-1; -1 = the shared empty
 * context) to slots_out[0..end-start).  Returns 0 (nothing changed) when not enough free slots. */
int go_ctxman_get_contexts( go_ctxman* m,
                            const uint8_t* active,
                            const uint32_t* context_id,
                            uint64_t start,
                            uint64_t end,
                            int32_t* slots_out );
/* single lookup (deprecated path, contextman.hh:103-124): slot index or -1 when exhausted */
int32_t go_ctxman_get_context( go_ctxman* m, uint32_t context_id );
/* the reference aborts on release; this restates the dead code after the abort
 * (contextman.hh:186-195): returns 1 if released (slot appended to the free list's tail). */
int go_ctxman_release( go_ctxman* m, uint32_t context_id );

/* BatchedInferenceState::check_finished, models/common/state.hh:621-631 */
int go_check_finished( uint32_t token,
                       uint32_t token_pos,
                       uint32_t prompt_length,
                       uint32_t max_completion_length,
                       uint32_t token_eos,
                       uint32_t token_eot,
                       uint64_t seq_len );
/* temperature wire encoding, state.hh:270,612 */
uint8_t go_encode_temperature( float t );
float go_decode_temperature( uint8_t t );

int go_num_threads( void );

#ifdef __cplusplus
}
#endif
#endif
