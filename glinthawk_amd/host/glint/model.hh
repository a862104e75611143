// Llama2 stage driver for the hip target: owns the hosted weights and the scratchpad, and issues the
// ops of one stage step in the reference's order (models/llama2/model.hh:311-442, 444-808):
//
//   pre-attention   rmsnorm -> wq -> wkv -> KV append
//   attention       RoPE (q and the appended K row) -> scores -> softmax -> weighted sum
//   post-attention  wo -> residual -> rmsnorm -> w1, w3 -> SiLU gate -> w2 -> residual
//   classification  final rmsnorm -> wcls -> (Gumbel noise if temperature > 0) -> argmax
//
// Two attention paths produce the same result: the fused split-K kernel (default; per-step tables
// of row addresses are uploaded once and shared by all layers) and the three unfused ops of the
// reference's interface with the (batch, n_heads, seq_len) score buffer.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <filesystem>
#include <memory>
#include <type_traits>
#include <vector>

#include "glint/concepts.hh"
#include "glint/config.hh"
#include "glint/context.hh"
#include "glint/hip/ops.hh"
#include "glint/state.hh"

namespace glint {

constexpr size_t MAX_BATCH_SIZE = 1024; // models/llama2/base.hh:26

// element counts of the weight files, in file order (models/llama2/base.hh:357-373,477-499)
template<typename Config>
struct WeightLayout
{
  // base: token_embedding_table, rms_final_weight, freq_cis_real, freq_cis_imag, wcls
  static std::array<uint64_t, 5> base_on_disk()
  {
    return { Config::vocab_size * Config::dim, Config::dim, Config::seq_len * Config::head_size / 2, Config::seq_len * Config::head_size / 2,
             Config::wcls_present ? Config::vocab_size * Config::dim : 0 };
  }
  // layer: rms_att_weight, wq, wkv (wk rows then wv rows), wo, rms_ffn_weight, w1, w2, w3
  static std::array<uint64_t, 8> layer_on_disk()
  {
    return { Config::dim, Config::dim * Config::dim, Config::dim * Config::kv_dim * 2, Config::dim * Config::dim, Config::dim, Config::dim * Config::hidden_dim,
             Config::dim * Config::hidden_dim, Config::dim * Config::hidden_dim };
  }
  // what a node keeps in memory depends on what it hosts (models/llama2/base.hh:410-433,520-545)
  template<typename Settings>
  static std::array<uint64_t, 5> base_in_memory( const Settings& s )
  {
    const bool emb = s.hosts( 0, InferenceStage::PreAttention ) || ( s.hosts_in_any_layer( InferenceStage::Classification ) && !Config::wcls_present );
    const bool att = s.hosts_in_any_layer( InferenceStage::Attention );
    const bool cls = s.hosts_in_any_layer( InferenceStage::Classification );
    auto d = base_on_disk();
    return { emb ? d[0] : 0, cls ? d[1] : 0, att ? d[2] : 0, att ? d[3] : 0, ( Config::wcls_present && cls ) ? d[4] : 0 };
  }
  template<typename Settings>
  static std::array<uint64_t, 8> layer_in_memory( const Settings& s, size_t layer )
  {
    const bool pre = s.hosts( layer, InferenceStage::PreAttention );
    const bool post = s.hosts( layer, InferenceStage::PostAttention );
    auto d = layer_on_disk();
    return { pre ? d[0] : 0, pre ? d[1] : 0, pre ? d[2] : 0, post ? d[3] : 0, post ? d[4] : 0, post ? d[5] : 0, post ? d[6] : 0, post ? d[7] : 0 };
  }
};

// Positions arrive in a state that was parsed from the wire unvalidated.  A row of a non-empty context
// at or beyond seq_len would address cache rows and RoPE table entries past their allocations, so every
// entry point that turns positions into addresses checks this on the host before anything is launched.
template<typename State, typename ContextVector>
bool positions_fit( const State& states, const ContextVector& contexts, const uint64_t seq_len )
{
  for ( size_t i = 0; i < contexts.size() && i < states.batch_size(); i++ ) {
    if ( !contexts[i]->empty() && states.token_pos( i ) >= seq_len ) {
      return false;
    }
  }
  return true;
}

// glint/loader.hh: copies the hosted tensors out of the reference's model directory
template<typename Model>
std::string load_model_dir( Model& model, const std::filesystem::path& model_dir );

template<typename DType>
struct BaseWeights
{
  DType* token_embedding_table {};
  DType* rms_final_weight {};
  DType* freq_cis_real {};
  DType* freq_cis_imag {};
  DType* wcls {}; // aliases the embedding table when the model has no separate classifier
};

template<typename DType>
struct LayerWeights
{
  DType* rms_att_weight {};
  DType* wq {};
  DType* wkv {};
  DType* wo {};
  DType* rms_ffn_weight {};
  DType* w1 {};
  DType* w2 {};
  DType* w3 {};
  DType* tensor( size_t k ) const
  {
    DType* const t[8] = { rms_att_weight, wq, wkv, wo, rms_ffn_weight, w1, w2, w3 };
    return t[k];
  }
};

struct ModelOptions
{
  bool fused_attention { true };  // false: the reference's three unfused ops + score buffer
  bool fused_projections { true }; // with fused_attention: projections fused with the ops that follow them
  int balanced_attention { 0 };   // fused decode attention over equal runs of keys: 0 where the step's lengths call for it, 1 always (shapes that have it), -1 never
  bool allocate_logits { true };  // only needed when the classifier is hosted
  uint64_t seed { 1 };            // random initialisation of weights
  float weight_std { 0.02f };     // N(0, std) for every tensor, as the benchmark configurations say
  bool randomize { true };        // false: leave the weights for load() / set_*_tensor()
};

template<typename Config, typename DType, typename LlamaOperations = hip::LlamaOperations<Config, DType>, typename Context = hip::Context<Config, DType>>
requires ModelConfig<Config>
class Llama2
{
public:
  using ConfigType = Config;
  using DataTypeT = DType;
  using ContextType = Context;
  using SettingsType = StageSettings<Config>;
  using StateType = BatchedInferenceState<Config>;
  using ContextVector = std::vector<std::shared_ptr<Context>>;
  using DevicePtr = typename LlamaOperations::DeviceUniquePtr;

  static_assert( LlamaOperationsConcept<LlamaOperations, DType, SettingsType> );
  static_assert( ContextConcept<Context, DType> );

  // weights are drawn N(0, weight_std) from `options.seed`; RoPE tables come from the closed form
  explicit Llama2( const SettingsType& settings, const ModelOptions options = {} )
    : settings_( settings )
    , options_( options )
    , ops_( settings )
  {
    GLINT_CHECK( settings_.concurrency_limit <= MAX_BATCH_SIZE );
    allocate_weights();
    allocate_scratch();
    if ( options_.randomize ) {
      randomize_weights();
    }
    write_rope_tables();
  }

  // The reference's constructor (models/llama2/model.hh:150-270): settings + model directory.  The
  // CONFIG file must describe Config, every weight file opened must have the size the shape implies;
  // anything else aborts, as the reference's CHECKs do.  Needs glint/loader.hh at the point of use.
  Llama2( const std::filesystem::path& model_dir, const SettingsType& settings, ModelOptions options = {} )
    : Llama2( settings, without_random_weights( options, settings ) )
  {
    if ( !settings.randomize_parameters ) {
      load( model_dir );
    }
  }

  void load( const std::filesystem::path& model_dir )
  {
    const std::string err = load_model_dir( *this, model_dir );
    if ( !err.empty() ) {
      std::fprintf( stderr, "glint: %s\n", err.c_str() );
      std::abort();
    }
  }

  const SettingsType& settings() const { return settings_; }
  LlamaOperations& ops() { return ops_; }
  // device time of forward() (see SpanTimer): switch it on or off, read the accumulated milliseconds and steps, which a read resets
  void time_device_spans( const bool on )
  {
    if ( on && !span_timer_ ) {
      span_timer_ = std::make_unique<SpanTimer>();
    } else if ( !on ) {
      span_timer_.reset();
    }
  }
  std::pair<double, uint64_t> device_spans()
  {
    std::pair<double, uint64_t> out { 0.0, 0 };
    if ( span_timer_ ) {
      out = { span_timer_->total_ms, span_timer_->spans };
      span_timer_->total_ms = 0;
      span_timer_->spans = 0;
    }
    return out;
  }
  const BaseWeights<DType>& base_weights() const { return base_; }
  const LayerWeights<DType>& layer_weights( size_t l ) const { return layers_[l]; }

  // copies `n` elements from host memory into tensor `k` (file order) of a hosted layer
  void set_layer_tensor( size_t layer, size_t k, const DType* host, uint64_t n )
  {
    GLINT_CHECK( layer < Config::n_layers && k < 8 );
    GLINT_CHECK( n == WeightLayout<Config>::layer_in_memory( settings_, layer )[k] );
    ops_.copy( layers_[layer].tensor( k ), host, n * sizeof( DType ), CopyType::HostToDevice );
  }
  // k: 0 token_embedding_table, 1 rms_final_weight, 2 freq_cis_real, 3 freq_cis_imag, 4 wcls
  void set_base_tensor( size_t k, const DType* host, uint64_t n )
  {
    DType* const t[5] = { base_.token_embedding_table, base_.rms_final_weight, base_.freq_cis_real, base_.freq_cis_imag, base_.wcls };
    GLINT_CHECK( k < 5 && t[k] != nullptr && n == WeightLayout<Config>::base_in_memory( settings_ )[k] );
    ops_.copy( t[k], host, n * sizeof( DType ), CopyType::HostToDevice );
  }

  // ------------------------------------------------------------------------------------------
  // forward(): every stage of every hosted layer, starting at states.next_layer()
  // ------------------------------------------------------------------------------------------
  void forward( StateType& states, const ContextVector& contexts )
  {
    check_batch( states, contexts.size(), InferenceStage::PreAttention );
    GLINT_CHECK( positions_fit( states, contexts, Config::seq_len ) );
    batch_ = states.batch_size();
    const uint32_t first = states.next_layer();

    // contexts first: position 0 on the first served layer restarts a slot (paged contexts drop their pages)
    for ( size_t i = 0; i < contexts.size(); i++ ) {
      GLINT_CHECK( contexts[i]->prepare( first, states.token_pos( i ), states.token_pos( i ) == 0 && settings_.first_layer_served == first ) );
      token_positions_[i] = states.token_pos( i );
    }

    if ( first == 0 ) {
      load_embedding( states );
    } else {
      ops_.copy( x_, reinterpret_cast<const DType*>( states.activations().data() ), states.activations().len(), CopyType::HostToDevice, true );
    }

    size_t last = Config::n_layers;
    std::vector<size_t> run;
    for ( size_t l = first; l < Config::n_layers && settings_.hosts( l, InferenceStage::PreAttention ); l++ ) {
      run.push_back( l );
    }
    for ( size_t l : run ) {
      for ( size_t i = 0; i < contexts.size(); i++ ) {
        GLINT_CHECK( contexts[i]->prepare( l, states.token_pos( i ), false ) );
      }
    }
    if ( options_.fused_attention ) {
      upload_tables( contexts, run );
    }

    mark_device_span( 0 ); // the activations and the tables are queued: from here to the copy back it is kernels only
    const bool fused_layers = options_.fused_attention && options_.fused_projections;
    if ( fused_layers && !run.empty() ) {
      // the first attention norm stands alone; every later one rides on the epilogue of the previous w2
      ops_.template rmsnorm<Config::dim>( xb_, x_, reinterpret_cast<float32_t*>( temp_ ), layers_[run[0]].rms_att_weight, batch_ );
    }
    for ( size_t k = 0; k < run.size(); k++ ) {
      const size_t l = run[k];
      GLINT_CHECK( settings_.hosts( l, InferenceStage::Attention ) && settings_.hosts( l, InferenceStage::PostAttention ) );
      if ( fused_layers ) {
        const DType* next_norm = k + 1 < run.size() ? layers_[run[k + 1]].rms_att_weight : nullptr;
        fused_layer_ops( l, k, next_norm );
      } else {
        for ( size_t i = 0; i < contexts.size(); i++ ) {
          layer_contexts_[i] = contexts[i]->layer( l );
          token_contexts_[i] = contexts[i]->layer( l ).token( states.token_pos( i ) );
        }
        pre_attention_ops( l, true, k );
        attention_ops( k );
        post_attention_ops( l );
      }
      last = l;
    }
    GLINT_CHECK( last < Config::n_layers );

    if ( last == Config::n_layers - 1 && settings_.hosts( last, InferenceStage::Classification ) ) {
      classify_ops();
      mark_device_span( 1 );
      postlude( states, last, true );
    } else {
      mark_device_span( 1 );
      postlude( states, last, false );
    }
    close_device_span();
  }

  // ------------------------------------------------------------------------------------------
  // stage-at-a-time entry points (disaggregated execution)
  // ------------------------------------------------------------------------------------------
  void forward_pre_attention( StateType& states )
  {
    check_batch( states, 0, InferenceStage::PreAttention );
    batch_ = states.batch_size();
    if ( states.next_layer() == 0 ) {
      load_embedding( states );
    } else {
      ops_.copy( x_, reinterpret_cast<const DType*>( states.activations().data() ), states.activations().len(), CopyType::HostToDevice, true );
    }
    pre_attention_ops( states.next_layer(), false, 0 );
    export_pre_attention( states );
  }

  void forward_attention( StateType& states, const ContextVector& contexts )
  {
    check_batch( states, contexts.size(), InferenceStage::Attention );
    GLINT_CHECK( positions_fit( states, contexts, Config::seq_len ) );
    batch_ = states.batch_size();
    const uint32_t l = states.next_layer();
    for ( size_t i = 0; i < states.batch_size(); i++ ) {
      GLINT_CHECK( contexts[i]->prepare( l, states.token_pos( i ), states.token_pos( i ) == 0 && settings_.first_layer_served == l ) );
      token_positions_[i] = states.token_pos( i );
      layer_contexts_[i] = contexts[i]->layer( l );
      token_contexts_[i] = contexts[i]->layer( l ).token( states.token_pos( i ) );
    }

    // the wire dtype may differ from the attention dtype (fp16 activations, fp32 attention)
    import_converted( q_, states.queries().data(), states.queries().len(), states.dtype() );
    if ( options_.fused_attention ) {
      upload_tables( contexts, { static_cast<size_t>( l ) } );
    }
    if ( states.has_kvs() ) {
      // all rows in one transfer, then the append kernel scatters them into the slots (rows of
      // inactive prompts have no token row and are skipped, like the reference's per-row loop)
      import_converted( kv_, states.kvs().data(), states.kvs().len(), states.dtype() );
      if ( options_.fused_attention ) {
        GLINT_GH( gh_kv_append( token_rows_dev( 0 ), kv_, batch_, Config::kv_dim, hip::gh_type<DType>(), ops_.stream() ) );
      } else {
        ops_.copy_kv_cache( token_contexts_, kv_, batch_ );
      }
    }
    attention_ops( 0 );

    if ( !states.has_queries() ) {
      states.allocate_queries();
    }
    export_converted( states.queries().data(), xb_, states.queries().len(), states.dtype() ); // the output travels in the query buffer
    states.set_next_stage( InferenceStage::PostAttention );
  }

  void forward_post_attention( StateType& states, const bool fuse_to_pre = false, const bool fuse_to_cls = false )
  {
    check_batch( states, 0, InferenceStage::PostAttention );
    batch_ = states.batch_size();
    ops_.copy( x_, reinterpret_cast<const DType*>( states.activations().data() ), states.activations().len(), CopyType::HostToDevice );
    ops_.copy( xb_, reinterpret_cast<const DType*>( states.queries().data() ), states.queries().len(), CopyType::HostToDevice );
    post_attention_ops( states.next_layer() );

    const uint32_t l = states.next_layer();
    if ( fuse_to_cls && l == Config::n_layers - 1 && settings_.hosts( l, InferenceStage::Classification ) ) {
      classify_ops();
      postlude( states, l, true );
    } else if ( fuse_to_pre && l < Config::n_layers - 1 && settings_.hosts( l + 1, InferenceStage::PreAttention ) ) {
      states.set_next_layer( l + 1 );
      pre_attention_ops( l + 1, false, 0 );
      export_pre_attention( states );
    } else {
      postlude( states, l, false );
    }
  }

  void forward_classify( StateType& states )
  {
    check_batch( states, 0, InferenceStage::Classification );
    batch_ = states.batch_size();
    ops_.copy( x_, reinterpret_cast<const DType*>( states.activations().data() ), states.activations().len(), CopyType::HostToDevice );
    classify_ops();
    postlude( states, states.next_layer(), true );
  }

  // ------------------------------------------------------------------------------------------
  // Batched prefill (new functionality: the reference feeds prompts one token per forward).
  // `n_tokens` consecutive tokens per context, context i starting at position start_pos[i]; runs
  // every hosted layer from `first_layer` on all batch * n_tokens tokens at once.  The cache rows
  // and the outputs equal those of n_tokens sequential forward() calls.
  //   token_ids     (batch * n_tokens) when the embedding is hosted and first_layer == 0, else nullptr
  //   acts_in_host  (batch * n_tokens, dim) activations otherwise
  //   acts_out_host (batch * n_tokens, dim) residual stream after the last hosted layer (may be nullptr)
  //   next_tokens   (batch) greedy token after the last prompt token, when the classifier is hosted (may be nullptr)
  // ------------------------------------------------------------------------------------------
  void prefill( const ContextVector& contexts,
                const uint32_t* start_pos,
                const uint32_t n_tokens,
                const uint32_t first_layer,
                const uint32_t* token_ids,
                const DType* acts_in_host,
                DType* acts_out_host,
                uint32_t* next_tokens )
  {
    GLINT_CHECK( options_.fused_attention && options_.fused_projections );
    const size_t batch = contexts.size();
    GLINT_CHECK( batch > 0 && batch <= settings_.concurrency_limit && n_tokens > 0 );
    const uint64_t n = (uint64_t)batch * n_tokens;
    ensure_prefill_scratch( n );
    batch_ = batch;

    std::vector<size_t> run;
    for ( size_t l = first_layer; l < Config::n_layers && settings_.hosts( l, InferenceStage::PreAttention ); l++ ) {
      run.push_back( l );
    }
    GLINT_CHECK( !run.empty() );
    uint32_t max_start = 0;
    for ( size_t i = 0; i < batch; i++ ) {
      GLINT_CHECK( (uint64_t)start_pos[i] + n_tokens <= Config::seq_len );
      token_positions_[i] = start_pos[i];
      max_start = std::max( max_start, start_pos[i] );
      for ( size_t k = 0; k < run.size(); k++ ) {
        GLINT_CHECK( contexts[i]->prepare( run[k], start_pos[i] + n_tokens - 1,
                                           k == 0 && start_pos[i] == 0 && settings_.first_layer_served == first_layer ) );
      }
    }
    upload_tables( contexts, run, false ); // per-context tables: pos = start positions, layer bases per layer

    DType* px = pf_x_.get();
    DType* pxb = pf_xb_.get();
    DType* pq = pf_q_.get();
    DType* phb = pf_hb_.get();
    // Many tokens arriving from and leaving for the host: the rows are cut into four runs, and the copies of a run go over a
    // stream of their own, so that the first layer's projections of run c (row-wise work: norm, wq, wkv, append, RoPE) overlap the
    // upload of run c + 1 and the download of run c overlaps the last layer's w2 product of run c + 1.  Everything in between
    // (attention needs all rows of a context) runs on all rows at once.
    const bool pipelined = n >= 8192 && !( first_layer == 0 && token_ids != nullptr ) && ( acts_in_host != nullptr );
    std::vector<std::pair<uint64_t, uint64_t>> chunks; // (first row, rows)
    if ( pipelined ) {
      ensure_copy_stream();
      const uint64_t per = ( ( n + N_CHUNKS - 1 ) / N_CHUNKS + 255 ) / 256 * 256;
      for ( uint64_t r0 = 0; r0 < n; r0 += per ) {
        chunks.emplace_back( r0, std::min( per, n - r0 ) );
      }
    } else {
      chunks.emplace_back( 0, n );
    }
    if ( first_layer == 0 && token_ids != nullptr ) {
      for ( uint64_t r = 0; r < n; r++ ) {
        GLINT_CHECK( token_ids[r] < Config::vocab_size );
        ops_.copy( px + r * Config::dim, base_.token_embedding_table + (uint64_t)token_ids[r] * Config::dim, Config::dim * sizeof( DType ),
                   CopyType::DeviceToDevice, true );
      }
    } else {
      GLINT_CHECK( acts_in_host != nullptr );
      if ( pipelined ) {
        for ( size_t c = 0; c < chunks.size(); c++ ) {
          const uint64_t off = chunks[c].first * Config::dim;
          GLINT_GH( gh_memcpy( px + off, acts_in_host + off, chunks[c].second * Config::dim * sizeof( DType ), GH_HOST_TO_DEVICE, 1, copy_lane_->stream ) );
          GLINT_GH( gh_event_record( copy_lane_->in[c], copy_lane_->stream ) );
        }
      } else {
        ops_.copy( px, acts_in_host, n * Config::dim * sizeof( DType ), CopyType::HostToDevice, true );
      }
    }

    const gh_shape shape = LlamaOperations::shape();
    const uint64_t row_bytes = 2ull * Config::kv_dim * sizeof( DType );
    const bool fuse_wo = n <= 65535 && gh_matmul_fuses_many_rows( Config::dim, Config::dim, n, hip::gh_type<DType>() ) == 1;
    if ( !pipelined ) {
      ops_.template rmsnorm<Config::dim>( pxb, px, reinterpret_cast<float32_t*>( temp_ ), layers_[run[0]].rms_att_weight, n );
    }
    for ( size_t k = 0; k < run.size(); k++ ) {
      const auto& w = layers_[run[k]];
      // one table entry per (context, token) for this layer's rows
      GLINT_GH( gh_prefill_tables( layer_rows_dev( k ), pos_dev(), batch, n_tokens, row_bytes, nullptr, pf_token_rows(), pf_pos(), ops_.stream() ) );
      if ( n < 128 ) {
        // few tokens: the weight-streaming GEMM with fused follow-up ops, as in decode
        ops_.matmul_qkv_rope_append( pq, pxb, w.wq, n, pf_pos(), base_.freq_cis_real, base_.freq_cis_imag, pf_token_rows() );
        GLINT_GH( gh_attn_prefill( pq, layer_rows_dev( k ), pos_dev(), pxb, batch, n_tokens, max_start, &shape, hip::gh_type<DType>(), pf_attn_ws_.get(),
                                   pf_attn_ws_bytes_, GH_ATTN_AUTO, ops_.stream() ) );
        ops_.template matmul_accum<Config::dim, Config::dim>( px, pxb, w.wo, n, pxb, w.rms_ffn_weight );
        ops_.matmul_silu_gate( phb, pxb, w.w1, n );
        const DType* next_norm = k + 1 < run.size() ? layers_[run[k + 1]].rms_att_weight : nullptr;
        ops_.template matmul_accum<Config::hidden_dim, Config::dim>( px, phb, w.w2, n, next_norm ? pxb : nullptr, next_norm );
      } else {
        // many tokens: MFMA-bound tile GEMMs storing DType directly, element-wise ops as separate
        // (bandwidth-trivial) kernels -- the reference's op sequence on batch * n_tokens rows
        DType* pkv = pf_kv_.get();
        DType* pxb2 = pf_xb2_.get();
        DType* phb2 = pf_hb2_.get();
        // the row-wise work in front of the attention: run by run while the runs arrive (first layer of a pipelined call), else on all rows
        const bool by_run = pipelined && k == 0;
        for ( size_t c = 0; c < ( by_run ? chunks.size() : 1 ); c++ ) {
          const uint64_t r0 = by_run ? chunks[c].first : 0, rows = by_run ? chunks[c].second : n;
          if ( by_run ) {
            GLINT_GH( gh_stream_wait_event( ops_.stream(), copy_lane_->in[c] ) );
            ops_.template rmsnorm<Config::dim>( pxb + r0 * Config::dim, px + r0 * Config::dim, reinterpret_cast<float32_t*>( temp_ ), w.rms_att_weight, rows );
          }
          if ( w.wkv == w.wq + (uint64_t)Config::dim * Config::dim ) { // wkv lies behind wq: one launch for the two products
            ops_.template matmul_pair<Config::dim, Config::dim, Config::kv_dim * 2>( pq + r0 * Config::dim, pkv + r0 * Config::kv_dim * 2, pxb + r0 * Config::dim,
                                                                                      w.wq, rows );
          } else {
            ops_.template matmul<Config::dim, Config::dim>( pq + r0 * Config::dim, pxb + r0 * Config::dim, w.wq, rows );
            ops_.template matmul<Config::dim, Config::kv_dim * 2>( pkv + r0 * Config::kv_dim * 2, pxb + r0 * Config::dim, w.wkv, rows );
          }
          GLINT_GH( gh_kv_append( pf_token_rows() + r0, pkv + r0 * Config::kv_dim * 2, rows, Config::kv_dim, hip::gh_type<DType>(), ops_.stream() ) );
          GLINT_GH( gh_rope( rows, pf_pos() + r0, base_.freq_cis_real, base_.freq_cis_imag, pq + r0 * Config::dim, pf_token_rows() + r0, Config::n_kv_heads,
                             Config::gqa_size, Config::head_size, hip::gh_type<DType>(), ops_.stream() ) );
        }
        GLINT_GH( gh_attn_prefill( pq, layer_rows_dev( k ), pos_dev(), pxb, batch, n_tokens, max_start, &shape, hip::gh_type<DType>(), pf_attn_ws_.get(),
                                   pf_attn_ws_bytes_, GH_ATTN_AUTO, ops_.stream() ) );
        // the residual add rides in the tile kernel's epilogue where the library does that for the shape
        // (same roundings as the separate op); elsewhere the ops stay separate kernels
        if ( fuse_wo ) {
          ops_.template matmul_accum<Config::dim, Config::dim>( px, pxb, w.wo, n, pxb, w.rms_ffn_weight );
        } else {
          ops_.template matmul<Config::dim, Config::dim>( pxb2, pxb, w.wo, n );
          ops_.template accum<Config::dim>( px, pxb2, n );
          ops_.template rmsnorm<Config::dim>( pxb, px, reinterpret_cast<float32_t*>( temp_ ), w.rms_ffn_weight, n );
        }
        ops_.template matmul<Config::dim, Config::hidden_dim>( phb, pxb, w.w1, n );
        ops_.template matmul<Config::dim, Config::hidden_dim>( phb2, pxb, w.w3, n );
        ops_.template silu<Config::hidden_dim>( phb, phb2, n );
        const DType* next_norm = k + 1 < run.size() ? layers_[run[k + 1]].rms_att_weight : nullptr;
        // the last product of the call run by run when its result leaves for the host, each run's download behind it
        const bool out_by_run = pipelined && k + 1 == run.size() && acts_out_host != nullptr;
        for ( size_t c = 0; c < ( out_by_run ? chunks.size() : 1 ); c++ ) {
          const uint64_t r0 = out_by_run ? chunks[c].first : 0, rows = out_by_run ? chunks[c].second : n;
          DType* cx = px + r0 * Config::dim;
          DType* cxb = pxb + r0 * Config::dim;
          const DType* chb = phb + r0 * Config::hidden_dim;
          // whether the residual add rides in the product's epilogue is a property of the shape, so it is asked per run
          if ( rows <= 65535 && gh_matmul_fuses_many_rows( Config::hidden_dim, Config::dim, rows, hip::gh_type<DType>() ) == 1 ) {
            ops_.template matmul_accum<Config::hidden_dim, Config::dim>( cx, chb, w.w2, rows, next_norm ? cxb : nullptr, next_norm );
          } else {
            ops_.template matmul<Config::hidden_dim, Config::dim>( cxb, chb, w.w2, rows );
            ops_.template accum<Config::dim>( cx, cxb, rows );
            if ( next_norm != nullptr ) {
              ops_.template rmsnorm<Config::dim>( cxb, cx, reinterpret_cast<float32_t*>( temp_ ), next_norm, rows );
            }
          }
          if ( out_by_run ) {
            GLINT_GH( gh_event_record( copy_lane_->out[c], ops_.stream() ) );
            GLINT_GH( gh_stream_wait_event( copy_lane_->stream, copy_lane_->out[c] ) );
            GLINT_GH( gh_memcpy( acts_out_host + r0 * Config::dim, cx, rows * Config::dim * sizeof( DType ), GH_DEVICE_TO_HOST, 1, copy_lane_->stream ) );
          }
        }
      }
    }

    if ( acts_out_host != nullptr ) {
      if ( pipelined ) {
        GLINT_GH( gh_sync( copy_lane_->stream ) ); // the downloads queued behind the last layer
      } else {
        ops_.copy( acts_out_host, px, n * Config::dim * sizeof( DType ), CopyType::DeviceToHost );
      }
    }
    const size_t last = run.back();
    if ( next_tokens != nullptr && last == Config::n_layers - 1 && settings_.hosts( last, InferenceStage::Classification ) ) {
      // only the last prompt token of each context is classified
      for ( size_t i = 0; i < batch; i++ ) {
        ops_.copy( x_ + i * Config::dim, px + ( (uint64_t)i * n_tokens + n_tokens - 1 ) * Config::dim, Config::dim * sizeof( DType ), CopyType::DeviceToDevice,
                   true );
      }
      classify_ops();
      ops_.template argmax<Config::vocab_size>( argmax_pos_, logits_, temp_, batch );
      for ( size_t i = 0; i < batch; i++ ) {
        next_tokens[i] = argmax_pos_[i];
      }
    } else {
      // Also the end of the uploads of a pipelined call: the stage's stream waited for every run's upload event before that run's
      // first kernel, so once it is empty the caller's input buffer is free again, whether or not anything was downloaded.
      ops_.synchronize();
    }
  }

  // scratch views for tests (device pointers)
  DType* scratch_x() const { return x_; }
  DType* scratch_xb() const { return xb_; }
  DType* scratch_q() const { return q_; }
  DType* scratch_kv() const { return kv_; }
  DType* scratch_logits() const { return logits_; }
  const uint32_t* argmax_pos() const { return argmax_pos_; }

private:
  // ---- ops of one layer ----------------------------------------------------------------------
  void pre_attention_ops( const size_t layer, const bool update_kv_cache, const size_t table_index )
  {
    const auto& w = layers_[layer];
    ops_.template rmsnorm<Config::dim>( xb_, x_, reinterpret_cast<float32_t*>( temp_ ), w.rms_att_weight, batch_ );
    ops_.template matmul<Config::dim, Config::dim>( q_, xb_, w.wq, batch_ );
    ops_.template matmul<Config::dim, Config::kv_dim * 2>( kv_, xb_, w.wkv, batch_ );
    if ( update_kv_cache ) {
      if ( options_.fused_attention ) {
        GLINT_GH( gh_kv_append( token_rows_dev( table_index ), kv_, batch_, Config::kv_dim, hip::gh_type<DType>(), ops_.stream() ) );
      } else {
        ops_.copy_kv_cache( token_contexts_, kv_, batch_ );
      }
    }
  }

  // the fused decode attention of one layer: over equal runs of keys where upload_tables() found the lengths of this
  // step's contexts far apart (the cuts are made there, once for all layers), else one wave per (context, kv head, split)
  void fused_attention( const size_t table_index )
  {
    if ( balanced_step_ ) {
      const gh_shape s = LlamaOperations::shape();
      GLINT_GH( gh_attn_decode_balanced( q_, layer_rows_dev( table_index ), xb_, batch_, max_pos_, &s, hip::gh_type<DType>(), attn_bal_ws_.get(),
                                         attn_bal_ws_bytes_, ops_.stream() ) );
    } else {
      ops_.attention_fused( q_, layer_rows_dev( table_index ), pos_dev(), xb_, batch_, max_pos_, attn_ws_.get(), attn_ws_bytes_ );
    }
  }

  void attention_ops( const size_t table_index )
  {
    if ( options_.fused_attention ) {
      GLINT_GH( gh_rope( batch_, pos_dev(), base_.freq_cis_real, base_.freq_cis_imag, q_, token_rows_dev( table_index ), Config::n_kv_heads, Config::gqa_size,
                         Config::head_size, hip::gh_type<DType>(), ops_.stream() ) );
      fused_attention( table_index );
    } else {
      ops_.apply_rope( batch_, token_positions_, base_.freq_cis_real, base_.freq_cis_imag, q_, token_contexts_ );
      ops_.attention_0_gemm( q_, layer_contexts_, att_, batch_, token_positions_ );
      ops_.attention_softmax( att_, token_positions_, temp_, batch_ );
      ops_.attention_2_gemm( att_, layer_contexts_, xb_, batch_, token_positions_ );
    }
  }

  void post_attention_ops( const size_t layer )
  {
    const auto& w = layers_[layer];
    if ( options_.fused_attention && options_.fused_projections ) {
      // same three fused launches as in forward(): wo + residual + rmsnorm, w1|w3 + SiLU gate, w2 + residual
      ops_.template matmul_accum<Config::dim, Config::dim>( x_, xb_, w.wo, batch_, xb_, w.rms_ffn_weight );
      ops_.matmul_silu_gate( hb_, xb_, w.w1, batch_ );
      ops_.template matmul_accum<Config::hidden_dim, Config::dim>( x_, hb_, w.w2, batch_, nullptr, nullptr );
      return;
    }
    ops_.template matmul<Config::dim, Config::dim>( xb2_, xb_, w.wo, batch_ );
    ops_.template accum<Config::dim>( x_, xb2_, batch_ );
    ops_.template rmsnorm<Config::dim>( xb_, x_, reinterpret_cast<float32_t*>( temp_ ), w.rms_ffn_weight, batch_ );
    ops_.template matmul<Config::dim, Config::hidden_dim>( hb_, xb_, w.w1, batch_ );
    ops_.template matmul<Config::dim, Config::hidden_dim>( hb2_, xb_, w.w3, batch_ );
    ops_.template silu<Config::hidden_dim>( hb_, hb2_, batch_ );
    ops_.template matmul<Config::hidden_dim, Config::dim>( xb_, hb_, w.w2, batch_ );
    ops_.template accum<Config::dim>( x_, xb_, batch_ );
  }

  // One whole layer with the projections fused with their follow-up ops: 9 or 10 launches instead of 21.
  // Expects xb_ = rmsnorm(x_) * rms_att_weight on entry; leaves the same for the next layer when
  // `next_att_norm` is given.
  void fused_layer_ops( const size_t layer, const size_t table_index, const DType* next_att_norm )
  {
    const auto& w = layers_[layer];
    ops_.matmul_qkv_rope_append( q_, xb_, w.wq, batch_, pos_dev(), base_.freq_cis_real, base_.freq_cis_imag, token_rows_dev( table_index ) );
    fused_attention( table_index );
    ops_.template matmul_accum<Config::dim, Config::dim>( x_, xb_, w.wo, batch_, xb_, w.rms_ffn_weight );
    ops_.matmul_silu_gate( hb_, xb_, w.w1, batch_ );
    ops_.template matmul_accum<Config::hidden_dim, Config::dim>( x_, hb_, w.w2, batch_, next_att_norm ? xb_ : nullptr, next_att_norm );
  }

  void classify_ops()
  {
    ops_.template rmsnorm<Config::dim>( x_, x_, reinterpret_cast<float32_t*>( temp_ ), base_.rms_final_weight, batch_ );
    ops_.template matmul<Config::dim, Config::vocab_size>( logits_, x_, base_.wcls, batch_ );
  }

  // ---- staging ---------------------------------------------------------------------------------
  void check_batch( const StateType& states, const size_t n_contexts, const InferenceStage stage ) const
  {
    GLINT_CHECK( states.batch_size() > 0 && states.batch_size() <= settings_.concurrency_limit );
    GLINT_CHECK( states.next_stage() == stage );
    GLINT_CHECK( settings_.hosts( states.next_layer(), stage ) );
    if ( stage == InferenceStage::Attention || n_contexts != 0 ) {
      GLINT_CHECK( n_contexts == states.batch_size() );
    }
    if ( stage != InferenceStage::Attention ) {
      GLINT_CHECK( states.dtype() == dtype_of<DType>() );
    }
  }

  void load_embedding( const StateType& states )
  {
    for ( size_t i = 0; i < states.batch_size(); i++ ) {
      if ( states.active( i ) ) {
        GLINT_CHECK( states.token( i ) < Config::vocab_size );
        ops_.copy( x_ + i * Config::dim, base_.token_embedding_table + (uint64_t)states.token( i ) * Config::dim, Config::dim * sizeof( DType ),
                   CopyType::DeviceToDevice, true );
      }
    }
  }

  void export_pre_attention( StateType& states )
  {
    if ( !states.has_activations() ) {
      states.allocate_activations();
    }
    if ( !states.has_queries() ) {
      states.allocate_queries();
    }
    if ( !states.has_kvs() ) {
      states.allocate_kvs();
    }
    ops_.copy( reinterpret_cast<DType*>( states.activations().data() ), x_, states.activations().len(), CopyType::DeviceToHost );
    ops_.copy( reinterpret_cast<DType*>( states.queries().data() ), q_, states.queries().len(), CopyType::DeviceToHost );
    ops_.copy( reinterpret_cast<DType*>( states.kvs().data() ), kv_, states.kvs().len(), CopyType::DeviceToHost );
    states.set_next_stage( InferenceStage::Attention );
  }

  void import_converted( DType* dst_dev, const uint8_t* src_host, const uint64_t src_bytes, const DataType wire )
  {
    if ( wire == DataType::Float32 ) {
      ops_.template convert_and_copy<DType, float32_t>( dst_dev, reinterpret_cast<const float32_t*>( src_host ), src_bytes / sizeof( float32_t ), CopyType::HostToDevice );
    } else if ( wire == DataType::Float16 ) {
      ops_.template convert_and_copy<DType, float16_t>( dst_dev, reinterpret_cast<const float16_t*>( src_host ), src_bytes / sizeof( float16_t ), CopyType::HostToDevice );
    } else {
      fatal( __FILE__, __LINE__, "invalid dtype" );
    }
  }

  void export_converted( uint8_t* dst_host, const DType* src_dev, const uint64_t dst_bytes, const DataType wire )
  {
    if ( wire == DataType::Float32 ) {
      ops_.template convert_and_copy<float32_t, DType>( reinterpret_cast<float32_t*>( dst_host ), src_dev, dst_bytes / sizeof( float32_t ), CopyType::DeviceToHost );
    } else if ( wire == DataType::Float16 ) {
      ops_.template convert_and_copy<float16_t, DType>( reinterpret_cast<float16_t*>( dst_host ), src_dev, dst_bytes / sizeof( float16_t ), CopyType::DeviceToHost );
    } else {
      fatal( __FILE__, __LINE__, "invalid dtype" );
    }
  }

  void postlude( StateType& states, const size_t most_recent_layer, const bool classification_done )
  {
    if ( classification_done ) {
      std::vector<float> temps;
      for ( size_t i = 0; i < states.batch_size(); i++ ) {
        temps.push_back( states.temperature( i ) );
      }
      ops_.soft_sample( logits_, temps, Config::vocab_size );
      ops_.template argmax<Config::vocab_size>( argmax_pos_, logits_, temp_, temps.size() );

      states.deallocate_activations();
      states.deallocate_queries();
      states.deallocate_kvs();
      states.set_next_layer( 0 );
      states.set_next_stage( InferenceStage::PreAttention );
      for ( size_t i = 0; i < states.batch_size(); i++ ) {
        if ( states.active( i ) ) {
          states.set_token( i, argmax_pos_[i] );
          states.set_token_pos( i, states.token_pos( i ) + 1 );
          if ( states.check_finished( i ) ) {
            states.set_finished( i ); // discarding the row is the caller's business
          }
        }
      }
    } else {
      states.allocate_activations();
      states.deallocate_queries();
      states.deallocate_kvs();
      ops_.copy( reinterpret_cast<DType*>( states.activations().data() ), x_, states.batch_size() * Config::dim * sizeof( DType ), CopyType::DeviceToHost );
      if ( most_recent_layer == Config::n_layers - 1 ) {
        states.set_next_stage( InferenceStage::Classification );
      } else {
        states.set_next_stage( InferenceStage::PreAttention );
        states.set_next_layer( static_cast<uint32_t>( most_recent_layer + 1 ) );
      }
    }
  }

  // ---- device-side tables of the fused path --------------------------------------------------
  // layout of one upload: pos[cap] (u32) | for each layer of the run: layer_rows[cap], token_rows[cap] (pointers)
  size_t table_stride() const { return settings_.concurrency_limit; }
  const uint32_t* pos_dev() const { return reinterpret_cast<const uint32_t*>( tables_dev_.get() ); }
  uint8_t* ptr_tables( uint8_t* base ) const { return base + ( ( table_stride() * sizeof( uint32_t ) + 15 ) / 16 * 16 ); }
  const void* const* layer_rows_dev( size_t k ) const
  {
    return reinterpret_cast<const void* const*>( ptr_tables( reinterpret_cast<uint8_t*>( tables_dev_.get() ) ) ) + ( 2 * k ) * table_stride();
  }
  void* const* token_rows_dev( size_t k ) const
  {
    return reinterpret_cast<void* const*>( ptr_tables( reinterpret_cast<uint8_t*>( tables_dev_.get() ) ) ) + ( 2 * k + 1 ) * table_stride();
  }

  // `decode`: the positions are those of one new token per context (a batched prefill attends from many)
  void upload_tables( const ContextVector& contexts, const std::vector<size_t>& run, const bool decode = true )
  {
    // The previous upload reads the pinned buffer asynchronously: it has to be over before the buffer is rewritten.  A step
    // ends with a blocking copy of its results, which is such a wait already; only without one since the last upload is
    // the stream waited for here (that wait would also sit out the copy of this step's activations, queued just before).
    if ( tables_uploaded_ && ops_.drain_count() == tables_drain_count_ ) {
      ops_.synchronize();
    }
    auto* pos = reinterpret_cast<uint32_t*>( tables_host_ );
    auto** ptrs = reinterpret_cast<void**>( ptr_tables( tables_host_ ) );
    max_pos_ = 0;
    uint64_t keys = 0, live = 0;
    for ( size_t i = 0; i < batch_; i++ ) {
      pos[i] = token_positions_[i];
      if ( !contexts[i]->empty() ) {
        GLINT_CHECK( token_positions_[i] < Config::seq_len );
        max_pos_ = std::max( max_pos_, token_positions_[i] );
        keys += token_positions_[i] + 1;
        live++;
      }
    }
    balanced_step_ = decode && attn_bal_ws_bytes_ > 0 && !run.empty() && options_.balanced_attention >= 0
                     && ( options_.balanced_attention > 0 || lengths_far_apart( keys, live, max_pos_ + 1 ) );
    for ( size_t k = 0; k < run.size(); k++ ) {
      for ( size_t i = 0; i < batch_; i++ ) {
        const auto layer = contexts[i]->layer( run[k] );
        ptrs[( 2 * k ) * table_stride() + i] = layer.data();
        ptrs[( 2 * k + 1 ) * table_stride() + i] = layer.token( token_positions_[i] ).key();
      }
    }
    const size_t bytes = ( ptr_tables( tables_host_ ) - tables_host_ ) + run.size() * 2 * table_stride() * sizeof( void* );
    GLINT_GH( gh_memcpy( tables_dev_.get(), tables_host_, bytes, GH_HOST_TO_DEVICE, 1, ops_.stream() ) );
    tables_uploaded_ = true;
    tables_drain_count_ = ops_.drain_count();
    if ( balanced_step_ ) {
      const gh_shape s = LlamaOperations::shape();
      GLINT_GH( gh_attn_balance( layer_rows_dev( 0 ), pos_dev(), batch_, max_pos_, &s, attn_bal_ws_.get(), attn_bal_ws_bytes_, ops_.stream() ) );
    }
  }

  // Whether the attention over equal runs of keys pays for this step: measured on the 70B shape, it costs 2 % where the
  // contexts are equally long and start-up where there is little to even out, and gains 10-25 % for lengths spread over
  // 16..4096 (a launch of the plain kernel lasts as long as the CU that drew the longest contexts), several times for one
  // long context among many short ones (with 1024 and more (context, kv head) pairs the plain kernel does not split).
  static bool lengths_far_apart( const uint64_t keys, const uint64_t live, const uint64_t longest )
  {
    if ( live == 0 || keys * 100 >= 85 * live * longest ) {
      return false; // mean length within 15 % of the longest
    }
    const uint64_t head_groups = ( Config::n_kv_heads + 3 ) / 4;
    if ( keys * head_groups >= 131072 ) {
      return true; // enough keys for runs of 256 and more on every CU
    }
    return live * Config::n_kv_heads >= 1024 && longest >= 1024 && longest * live >= 4 * keys;
  }

  // ---- allocation ----------------------------------------------------------------------------
  static DType* carve( DType*& cursor, uint64_t n )
  {
    DType* p = n ? cursor : nullptr;
    cursor += ( n + 7 ) / 8 * 8; // keep every tensor 16-byte aligned
    return p;
  }
  static uint64_t padded( uint64_t n ) { return ( n + 7 ) / 8 * 8; }

  static ModelOptions without_random_weights( ModelOptions o, const SettingsType& s )
  {
    o.randomize = s.randomize_parameters;
    return o;
  }

  void allocate_weights()
  {
    const auto b = WeightLayout<Config>::base_in_memory( settings_ );
    uint64_t total = 0;
    for ( auto n : b ) {
      total += padded( n );
    }
    base_storage_ = ops_.device_allocate( std::max<uint64_t>( total, 8 ) * sizeof( DType ) );
    DType* cur = base_storage_.get();
    base_.token_embedding_table = carve( cur, b[0] );
    base_.rms_final_weight = carve( cur, b[1] );
    base_.freq_cis_real = carve( cur, b[2] );
    base_.freq_cis_imag = carve( cur, b[3] );
    base_.wcls = carve( cur, b[4] );
    if ( !Config::wcls_present && settings_.hosts_in_any_layer( InferenceStage::Classification ) ) {
      base_.wcls = base_.token_embedding_table; // shared classifier (models/llama2/model.hh weight tying)
    }

    total = 0;
    for ( size_t l = 0; l < Config::n_layers; l++ ) {
      for ( auto n : WeightLayout<Config>::layer_in_memory( settings_, l ) ) {
        total += padded( n );
      }
    }
    layer_storage_ = ops_.device_allocate( std::max<uint64_t>( total, 8 ) * sizeof( DType ) );
    cur = layer_storage_.get();
    layers_.resize( Config::n_layers );
    for ( size_t l = 0; l < Config::n_layers; l++ ) {
      const auto n = WeightLayout<Config>::layer_in_memory( settings_, l );
      auto& w = layers_[l];
      w.rms_att_weight = carve( cur, n[0] );
      w.wq = carve( cur, n[1] );
      w.wkv = carve( cur, n[2] );
      w.wo = carve( cur, n[3] );
      w.rms_ffn_weight = carve( cur, n[4] );
      // w3 is placed right after w1 (and wkv right after wq) so that each pair is one row-major
      // matrix for the fused projections; the file order (w1, w2, w3) only matters when loading
      w.w1 = carve( cur, n[5] );
      w.w3 = carve( cur, n[7] );
      w.w2 = carve( cur, n[6] );
      if ( n[1] && n[2] ) {
        GLINT_CHECK( w.wkv == w.wq + n[1] );
      }
      if ( n[5] && n[7] ) {
        GLINT_CHECK( w.w3 == w.w1 + n[5] );
      }
    }
  }

  void allocate_scratch()
  {
    const uint64_t cap = settings_.concurrency_limit;
    const bool cls = settings_.hosts_in_any_layer( InferenceStage::Classification ) && options_.allocate_logits;
    const uint64_t att_elems = options_.fused_attention ? 0 : cap * Config::n_heads * Config::seq_len;
    const uint64_t temp_elems = cap * std::max<uint64_t>( Config::n_heads, Config::dim ) * 4 / sizeof( DType );
    const uint64_t total = padded( cap * Config::dim ) * 4 + padded( cap * Config::kv_dim * 2 ) + padded( cap * Config::hidden_dim ) * 2 + padded( att_elems )
                           + padded( cls ? cap * Config::vocab_size : 0 ) + padded( temp_elems );
    scratch_storage_ = ops_.device_allocate( total * sizeof( DType ) );
    GLINT_GH( gh_memset_zero( scratch_storage_.get(), total * sizeof( DType ), ops_.stream() ) );
    DType* cur = scratch_storage_.get();
    x_ = carve( cur, cap * Config::dim );
    xb_ = carve( cur, cap * Config::dim );
    xb2_ = carve( cur, cap * Config::dim );
    q_ = carve( cur, cap * Config::dim );
    kv_ = carve( cur, cap * Config::kv_dim * 2 );
    hb_ = carve( cur, cap * Config::hidden_dim );
    hb2_ = carve( cur, cap * Config::hidden_dim );
    att_ = carve( cur, att_elems );
    logits_ = carve( cur, cls ? cap * Config::vocab_size : 0 );
    temp_ = carve( cur, temp_elems );

    if ( options_.fused_attention ) {
      const gh_shape s = LlamaOperations::shape();
      attn_ws_bytes_ = gh_attn_decode_workspace( cap, Config::seq_len - 1, &s );
      attn_ws_ = ops_.device_allocate( std::max<uint64_t>( attn_ws_bytes_, 16 ) );
      if ( std::is_same_v<DType, glint::float16_t> && Config::head_size == 128
           && ( Config::gqa_size == 1 || Config::gqa_size == 2 || Config::gqa_size == 4 || Config::gqa_size == 8 || Config::gqa_size == 16 ) ) {
        attn_bal_ws_bytes_ = gh_attn_balanced_workspace( cap, &s ); // the shapes gh_attn_decode_balanced takes
        attn_bal_ws_ = ops_.device_allocate( std::max<uint64_t>( attn_bal_ws_bytes_, 16 ) );
      }
      const size_t n_run = std::max<size_t>( 1, settings_.num_attention_layers_hosted() );
      const size_t bytes = ( cap * sizeof( uint32_t ) + 15 ) / 16 * 16 + n_run * 2 * cap * sizeof( void* );
      tables_dev_ = ops_.device_allocate( bytes );
      void* pinned = nullptr;
      GLINT_GH( gh_host_malloc( &pinned, bytes ) );
      tables_host_ = static_cast<uint8_t*>( pinned );
    }
  }

  void randomize_weights()
  {
    uint64_t seed = options_.seed * 1000003ull;
    auto fill = [&]( DType* p, uint64_t n ) {
      if ( p && n ) {
        GLINT_GH( gh_fill_normal( p, n, 0.0f, options_.weight_std, seed++, hip::gh_type<DType>(), ops_.stream() ) );
      } else {
        seed++;
      }
    };
    const auto b = WeightLayout<Config>::base_in_memory( settings_ );
    fill( base_.token_embedding_table, b[0] );
    fill( base_.rms_final_weight, b[1] );
    if ( Config::wcls_present ) {
      fill( base_.wcls, b[4] );
    }
    for ( size_t l = 0; l < Config::n_layers; l++ ) {
      const auto n = WeightLayout<Config>::layer_in_memory( settings_, l );
      for ( size_t k = 0; k < 8; k++ ) {
        fill( layers_[l].tensor( k ), n[k] );
      }
    }
  }

  // cos / sin( pos * theta^(-2k / head_size) ), theta 10000, computed in fp32 (tools/bin2glint.py:19-25)
  void write_rope_tables()
  {
    if ( base_.freq_cis_real == nullptr ) {
      return;
    }
    const uint64_t half = Config::head_size / 2;
    std::vector<DType> re( Config::seq_len * half ), im( Config::seq_len * half );
    for ( uint64_t k = 0; k < half; k++ ) {
      const float freq = 1.0f / std::pow( 10000.0f, static_cast<float>( 2 * k ) / static_cast<float>( Config::head_size ) );
      for ( uint64_t p = 0; p < Config::seq_len; p++ ) {
        const float angle = static_cast<float>( p ) * freq;
        re[p * half + k] = static_cast<DType>( std::cos( angle ) );
        im[p * half + k] = static_cast<DType>( std::sin( angle ) );
      }
    }
    ops_.copy( base_.freq_cis_real, re.data(), re.size() * sizeof( DType ), CopyType::HostToDevice );
    ops_.copy( base_.freq_cis_imag, im.data(), im.size() * sizeof( DType ), CopyType::HostToDevice );
  }

  SettingsType settings_;
  ModelOptions options_;
  LlamaOperations ops_;

  // prefill scratch: activations for `pf_capacity_` tokens, grown on demand
  void ensure_prefill_scratch( const uint64_t n )
  {
    if ( n <= pf_capacity_ ) {
      return;
    }
    ops_.synchronize();
    pf_x_ = ops_.device_allocate( n * Config::dim * sizeof( DType ) );
    pf_xb_ = ops_.device_allocate( n * Config::dim * sizeof( DType ) );
    pf_q_ = ops_.device_allocate( n * Config::dim * sizeof( DType ) );
    pf_hb_ = ops_.device_allocate( n * Config::hidden_dim * sizeof( DType ) );
    if ( n >= 128 ) {
      pf_hb2_ = ops_.device_allocate( n * Config::hidden_dim * sizeof( DType ) );
      pf_xb2_ = ops_.device_allocate( n * Config::dim * sizeof( DType ) );
      pf_kv_ = ops_.device_allocate( n * Config::kv_dim * 2 * sizeof( DType ) );
    }
    pf_tables_ = ops_.device_allocate( n * ( sizeof( void* ) + sizeof( uint32_t ) ) + 64 );
    const gh_shape shape = LlamaOperations::shape();
    // sized for the widest call: every context contributes all n tokens
    pf_attn_ws_bytes_ = gh_attn_prefill_workspace( 1, static_cast<uint32_t>( n ), &shape );
    pf_attn_ws_ = ops_.device_allocate( std::max<uint64_t>( pf_attn_ws_bytes_, 16 ) );
    pf_capacity_ = n;
  }
  // the stream and events of the pipelined prefill, created on first use and kept for the life of the model
  static constexpr size_t N_CHUNKS = 4;
  struct CopyLane
  {
    gh_stream stream { nullptr };
    gh_event in[N_CHUNKS] {}, out[N_CHUNKS] {};
    CopyLane()
    {
      GLINT_GH( gh_stream_create( &stream ) );
      for ( size_t c = 0; c < N_CHUNKS; c++ ) {
        GLINT_GH( gh_event_create( &in[c] ) );
        GLINT_GH( gh_event_create( &out[c] ) );
      }
    }
    ~CopyLane()
    {
      for ( size_t c = 0; c < N_CHUNKS; c++ ) {
        (void)gh_event_destroy( in[c] );
        (void)gh_event_destroy( out[c] );
      }
      (void)gh_stream_destroy( stream );
    }
    CopyLane( const CopyLane& ) = delete;
    CopyLane& operator=( const CopyLane& ) = delete;
  };
  // Device time of forward(): the span on the stream from the first kernel of a step to its last, without the copies of the
  // state over the host boundary on either side.  Off by default; two event records per step when on.
  struct SpanTimer
  {
    gh_event mark[2] {};
    double total_ms { 0 };
    uint64_t spans { 0 };
    bool open { false };
    SpanTimer()
    {
      GLINT_GH( gh_event_create_timed( &mark[0] ) );
      GLINT_GH( gh_event_create_timed( &mark[1] ) );
    }
    ~SpanTimer()
    {
      (void)gh_event_destroy( mark[0] );
      (void)gh_event_destroy( mark[1] );
    }
    SpanTimer( const SpanTimer& ) = delete;
    SpanTimer& operator=( const SpanTimer& ) = delete;
  };
  void mark_device_span( const int which )
  {
    if ( span_timer_ ) {
      GLINT_GH( gh_event_record( span_timer_->mark[which], ops_.stream() ) );
      span_timer_->open = which == 1;
    }
  }
  void close_device_span()
  {
    if ( span_timer_ && span_timer_->open ) {
      float ms = 0;
      GLINT_GH( gh_event_elapsed_ms( span_timer_->mark[0], span_timer_->mark[1], &ms ) );
      span_timer_->total_ms += ms;
      span_timer_->spans++;
      span_timer_->open = false;
    }
  }
  void ensure_copy_stream()
  {
    if ( !copy_lane_ ) {
      copy_lane_ = std::make_unique<CopyLane>();
    }
  }
  void** pf_token_rows() const { return reinterpret_cast<void**>( pf_tables_.get() ); }
  uint32_t* pf_pos() const { return reinterpret_cast<uint32_t*>( pf_token_rows() + pf_capacity_ ); }

  DevicePtr base_storage_ {}, layer_storage_ {}, scratch_storage_ {}, attn_ws_ {}, tables_dev_ {};
  DevicePtr pf_x_ {}, pf_xb_ {}, pf_q_ {}, pf_hb_ {}, pf_hb2_ {}, pf_xb2_ {}, pf_kv_ {}, pf_tables_ {}, pf_attn_ws_ {};
  uint64_t pf_capacity_ { 0 }, pf_attn_ws_bytes_ { 0 };
  std::unique_ptr<CopyLane> copy_lane_ {};
  std::unique_ptr<SpanTimer> span_timer_ {};
  uint64_t attn_ws_bytes_ { 0 };
  DevicePtr attn_bal_ws_ {};
  uint64_t attn_bal_ws_bytes_ { 0 };
  bool balanced_step_ { false };
  uint8_t* tables_host_ { nullptr };
  bool tables_uploaded_ { false };
  uint64_t tables_drain_count_ { 0 };
  BaseWeights<DType> base_ {};
  std::vector<LayerWeights<DType>> layers_ {};

  // scratchpad: device buffers ...
  DType *x_ {}, *xb_ {}, *xb2_ {}, *q_ {}, *kv_ {}, *hb_ {}, *hb2_ {}, *att_ {}, *logits_ {}, *temp_ {};
  // ... and host arrays (models/llama2/base.hh:196-202)
  uint64_t batch_ { 1 };
  uint32_t max_pos_ { 0 };
  uint32_t argmax_pos_[MAX_BATCH_SIZE] {};
  uint32_t token_positions_[MAX_BATCH_SIZE] {};
  typename Context::LayerContextType layer_contexts_[MAX_BATCH_SIZE] {};
  typename Context::TokenContextType token_contexts_[MAX_BATCH_SIZE] {};
};

} // namespace glint
