// Model shapes and per-node settings.
//
// `ModelConfig` restates the requirements of the reference's concept of the same name
// (models/llama2/variants.hh:9-32): a struct of static constexpr unsigned constants.  Any of the
// reference's own config structs satisfies it, so the classes of this layer can be instantiated with
// them directly.  The structs below are the shapes the benchmark configurations need, including two
// the reference does not define (stories15M and a 13B variant with a 4K window).
//
// `StageSettings` carries what the ops, contexts and the model driver read from the reference's
// ConfigRuntime (models/llama2/base.hh:28-70): the hosting table, concurrency_limit,
// max_context_count, num_attention_layers_hosted(), first_layer_served.  The classes only use that
// read interface (duck-typed template parameter), so a ConfigRuntime<Config> can be passed instead.
#pragma once

#include <array>
#include <concepts>
#include <cstdint>
#include <type_traits>

#include "glint/types.hh"

namespace glint {

template<class T>
concept ModelConfig = requires {
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::dim )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::kv_dim )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::hidden_dim )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::n_layers )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::head_size )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::n_heads )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::n_kv_heads )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::gqa_size )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::vocab_size )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::seq_len )>>;
  requires std::is_convertible_v<decltype( T::wcls_present ), bool>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::attention_rounds )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::token_bos )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::token_eos )>>;
  requires std::is_unsigned_v<std::remove_cv_t<decltype( T::token_eot )>>;
  requires T::gqa_size == T::n_heads / T::n_kv_heads;
  requires T::kv_dim == T::dim / T::gqa_size;
  requires T::head_size == T::dim / T::n_heads;
};

namespace configs {

struct Llama2Family
{
  constexpr static uint64_t vocab_size = 32'000;
  constexpr static uint32_t token_bos = 1;
  constexpr static uint32_t token_eos = 2;
  constexpr static uint32_t token_eot = 2;
};

template<uint64_t Dim, uint64_t Hidden, uint64_t Layers, uint64_t Heads, uint64_t KvHeads, uint64_t SeqLen, bool Wcls, uint64_t Rounds>
struct Shape : Llama2Family
{
  constexpr static uint64_t dim = Dim;
  constexpr static uint64_t hidden_dim = Hidden;
  constexpr static uint64_t n_layers = Layers;
  constexpr static uint64_t n_heads = Heads;
  constexpr static uint64_t n_kv_heads = KvHeads;
  constexpr static uint64_t gqa_size = Heads / KvHeads;
  constexpr static uint64_t kv_dim = Dim / gqa_size;
  constexpr static uint64_t head_size = Dim / Heads;
  constexpr static uint64_t seq_len = SeqLen;
  constexpr static bool wcls_present = Wcls;
  constexpr static uint64_t attention_rounds = Rounds;
};

// shapes of models/llama2/variants.hh:98-116,143-186
using Llama2_70B_Chat = Shape<8192, 28672, 80, 64, 8, 2048, true, 1>;
using Llama2_70B_Chat_4K = Shape<8192, 28672, 80, 64, 8, 4096, true, 1>;
using Llama2_70B_Chat_8K = Shape<8192, 28672, 80, 64, 8, 8192, true, 1>;
using Llama2_13B_Chat = Shape<5120, 13824, 40, 40, 40, 2048, true, 2>;
using Llama2_7B_Chat = Shape<4096, 11008, 32, 32, 32, 2048, true, 2>;
using Stories_110M = Shape<768, 2048, 12, 12, 12, 1024, false, 4>;
// shapes the benchmark configurations name that the reference does not define
using Llama2_13B_Chat_4K = Shape<5120, 13824, 40, 40, 40, 4096, true, 2>; // 2048-token prompts + 64 decode steps need > 2048 positions
using Stories_15M = Shape<288, 768, 6, 6, 6, 256, false, 2>;
// small shapes for tests: fast-kernel head size with and without query grouping, and a generic one
using Test_GQA4 = Shape<1024, 1536, 3, 8, 2, 320, true, 1>;
using Test_MHA = Shape<512, 768, 2, 4, 4, 192, false, 2>;
using Test_Tiny = Shape<32, 48, 2, 4, 2, 16, true, 1>;

static_assert( ModelConfig<Llama2_70B_Chat_4K> && ModelConfig<Llama2_13B_Chat_4K> && ModelConfig<Llama2_7B_Chat> && ModelConfig<Stories_15M> );
static_assert( ModelConfig<Test_GQA4> && ModelConfig<Test_MHA> && ModelConfig<Test_Tiny> );
static_assert( Llama2_70B_Chat_4K::kv_dim == 1024 && Llama2_70B_Chat_4K::gqa_size == 8 && Llama2_70B_Chat_4K::head_size == 128 );

} // namespace configs

template<typename Config>
requires ModelConfig<Config>
struct StageSettings
{
  using HostingTable = std::array<std::array<bool, N_STAGES>, Config::n_layers>;

  HostingTable hosting_table_ {};
  std::array<bool, N_STAGES> hosting_stage_table_ {};
  uint64_t concurrency_limit { 1 };
  uint64_t max_context_count { 1 };
  size_t num_attention_layers_hosted_ { 0 };
  bool randomize_parameters { false };
  uint32_t first_layer_served { 0 };

  StageSettings() = default;

  // same derivations as ConfigRuntime's constructor (models/llama2/base.hh:283-313)
  StageSettings( const HostingTable& table, uint64_t concurrency, uint64_t max_contexts, bool randomize = false )
    : hosting_table_( table )
    , concurrency_limit( concurrency )
    , max_context_count( max_contexts )
    , randomize_parameters( randomize )
  {
    GLINT_CHECK( concurrency_limit > 0 );
    bool any = false;
    for ( size_t st = 0; st < N_STAGES; st++ ) {
      for ( size_t l = 0; l < Config::n_layers; l++ ) {
        hosting_stage_table_[st] = hosting_stage_table_[st] || hosting_table_[l][st];
      }
      any = any || hosting_stage_table_[st];
    }
    GLINT_CHECK( any );
    for ( size_t l = 0; l < Config::n_layers; l++ ) {
      num_attention_layers_hosted_ += hosting_table_[l][static_cast<size_t>( InferenceStage::Attention )] ? 1 : 0;
    }
    bool found = false;
    for ( size_t l = 0; l < Config::n_layers && !found; l++ ) {
      for ( size_t st = 0; st < N_STAGES; st++ ) {
        if ( hosting_table_[l][st] ) {
          first_layer_served = static_cast<uint32_t>( l );
          found = true;
          break;
        }
      }
    }
  }

  // hosts layers [first, first + count) completely; the classifier too when `with_cls` and the last layer is included
  static StageSettings slice( size_t first, size_t count, uint64_t concurrency, uint64_t max_contexts, bool with_cls = false )
  {
    HostingTable t {};
    for ( size_t l = first; l < first + count && l < Config::n_layers; l++ ) {
      t[l][0] = t[l][1] = t[l][2] = true;
      t[l][3] = with_cls && l == Config::n_layers - 1;
    }
    return StageSettings( t, concurrency, max_contexts );
  }

  [[nodiscard]] bool hosts( size_t layer, InferenceStage stage ) const { return hosting_table_[layer][static_cast<size_t>( stage )]; }
  [[nodiscard]] bool hosts_in_any_layer( InferenceStage stage ) const { return hosting_stage_table_[static_cast<size_t>( stage )]; }
  [[nodiscard]] size_t num_attention_layers_hosted() const { return num_attention_layers_hosted_; }
};

} // namespace glint
