// KV-cache addressing: TokenContext / LayerContext / Context / DynamicContext, with the layout and
// the method names of the reference (models/llama2/context.hh:17-249):
//   context  = hosted layers back to back, each seq_len rows
//   row      = [K (kv_dim) | V (kv_dim)] of one token
//   K head h = row + h * head_size, V head h = row + kv_dim + h * head_size
// A null buffer is the *empty* context (make_empty = true): ops skip such rows.
#pragma once

#include <algorithm>
#include <array>
#include <concepts>
#include <cstddef>
#include <optional>
#include <vector>

#include "glint/config.hh"

namespace glint {

// the read interface every context type offers (models/llama2/context.hh:17-45)
template<typename T, typename DType>
concept TokenContextConcept = requires( T t ) {
  { T() };
  { t.key() } -> std::same_as<DType*>;
  { t.value() } -> std::same_as<DType*>;
  { t.key_head( 0ull ) } -> std::same_as<DType*>;
  { t.value_head( 0ull ) } -> std::same_as<DType*>;
  { t.empty() } -> std::same_as<bool>;
  { T::size() } -> std::same_as<size_t>;
};

template<typename T, typename DType>
concept LayerContextConcept = TokenContextConcept<typename T::TokenContextType, DType> && requires( T t ) {
  { T() };
  { t.token( 0ull ) } -> std::same_as<typename T::TokenContextType>;
  { T::max_size() } -> std::same_as<size_t>;
  { t.empty() } -> std::same_as<bool>;
  { t.is_contiguous() } -> std::same_as<bool>;
};

template<typename T, typename DType>
concept ContextConcept = LayerContextConcept<typename T::LayerContextType, DType> && TokenContextConcept<typename T::TokenContextType, DType>
                         && requires( T t ) {
                              { T() };
                              { t.prepare( 0ull, 0ull, false ) } -> std::same_as<bool>;
                              { t.layer( 0ull ) } -> std::same_as<typename T::LayerContextType>;
                              { t.empty() } -> std::same_as<bool>;
                              { T::max_size( 0ull ) } -> std::same_as<size_t>;
                            };

template<typename Config, typename DType>
requires ModelConfig<Config>
class LayerContext;

template<typename Config, typename DType>
requires ModelConfig<Config>
class Context;

template<typename Config, typename DType>
requires ModelConfig<Config>
class TokenContext
{
  friend class LayerContext<Config, DType>;
  DType* buffer_ { nullptr };
  explicit TokenContext( DType* buffer )
    : buffer_( buffer )
  {
  }

public:
  TokenContext() = default;

  DType* key() { return buffer_; }
  const DType* key() const { return buffer_; }
  DType* value() { return buffer_ + Config::kv_dim; }
  const DType* value() const { return buffer_ + Config::kv_dim; }
  DType* key_head( const size_t h ) { return key() + h * Config::head_size; }
  const DType* key_head( const size_t h ) const { return key() + h * Config::head_size; }
  DType* value_head( const size_t h ) { return value() + h * Config::head_size; }
  const DType* value_head( const size_t h ) const { return value() + h * Config::head_size; }

  constexpr static size_t size() { return Config::kv_dim * 2 * sizeof( DType ); }
  bool empty() const { return buffer_ == nullptr; }
};

template<typename Config, typename DType>
requires ModelConfig<Config>
class LayerContext
{
  friend class Context<Config, DType>;
  DType* buffer_ { nullptr };
  explicit LayerContext( DType* buffer )
    : buffer_( buffer )
  {
  }

public:
  using TokenContextType = TokenContext<Config, DType>;

  LayerContext() = default;

  TokenContextType token( const size_t token_num ) const
  {
    return buffer_ == nullptr ? TokenContextType {} : TokenContextType { buffer_ + token_num * Config::kv_dim * 2 };
  }

  DType* data() const { return buffer_; }
  bool empty() const { return buffer_ == nullptr; }
  constexpr static size_t max_size() { return Config::seq_len * TokenContextType::size(); }
  constexpr static bool is_contiguous() { return true; }
};

template<typename Config, typename DType>
requires ModelConfig<Config>
class Context
{
  DType* buffer_ { nullptr };
  std::array<DType*, Config::n_layers> layer_buffer_ {};

public:
  using LayerContextType = LayerContext<Config, DType>;
  using TokenContextType = TokenContext<Config, DType>;

  Context() = default;

  template<typename Settings>
  Context( const Settings& settings, DType* buffer )
  {
    set_buffer( settings, buffer );
  }

  // static contexts have nothing to do here; paged ones commit memory (see DynamicContext)
  bool prepare( const size_t, const size_t, const bool ) { return true; }

  LayerContextType layer( const size_t layer_num ) const { return LayerContextType { layer_buffer_[layer_num] }; }
  DType* data() const { return buffer_; }

  static size_t max_size( const size_t n_layers ) { return n_layers * LayerContextType::max_size(); }
  bool empty() const { return buffer_ == nullptr; }

protected:
  // only layers whose Attention stage is hosted get storage, packed in layer order
  template<typename Settings>
  void set_buffer( const Settings& settings, DType* buffer )
  {
    buffer_ = buffer;
    DType* next = buffer;
    for ( size_t l = 0; l < Config::n_layers; l++ ) {
      if ( buffer_ != nullptr && settings.hosts( l, InferenceStage::Attention ) ) {
        layer_buffer_[l] = next;
        next += LayerContextType::max_size() / sizeof( DType );
      } else {
        layer_buffer_[l] = nullptr;
      }
    }
  }
};

// Paged context: the whole span is reserved as address space, 2 MiB blocks are committed as the
// context grows, and everything is dropped when the slot restarts at position 0
// (models/llama2/context.hh:192-249).  One difference, a superset: the reference commits at most
// one block per call, which leaves holes if a fresh slot is asked for a far position; this version
// commits every missing block.  Under sequential growth both do exactly the same.
template<typename Config, typename DType, typename VirtualMemoryRegion>
class DynamicContext : public Context<Config, DType>
{
  std::optional<VirtualMemoryRegion> storage_ {};
  std::array<size_t, Config::n_layers> layer_allocated_offsets_ {};
  std::vector<bool> block_committed_ {};
  size_t blocks_committed_ { 0 };
  size_t clears_ { 0 };

public:
  static constexpr size_t BLOCK_SIZE = 2 * 1024 * 1024;

  DynamicContext() = default;

  template<typename Settings>
  explicit DynamicContext( const Settings& settings, const bool make_empty = false )
  {
    if ( !make_empty ) {
      storage_.emplace( Context<Config, DType>::max_size( settings.num_attention_layers_hosted() ) );
    }
    this->set_buffer( settings, storage_.has_value() ? reinterpret_cast<DType*>( storage_->ptr() ) : nullptr );
  }

  bool prepare( const size_t layer_num, const size_t token_pos, const bool can_release )
  {
    if ( this->empty() ) {
      return true;
    }
    if ( can_release ) {
      storage_->clear();
      layer_allocated_offsets_.fill( 0 );
      std::fill( block_committed_.begin(), block_committed_.end(), false );
      clears_++;
    }
    const auto layer = this->layer( layer_num );
    if ( layer.empty() ) {
      return true;
    }
    // Blocks are 2 MiB pieces of the region counted from its base.  Every real shape has layer spans
    // that are multiples of 2 MiB, so a layer's blocks start at the layer and this is the reference's
    // rule (one more block whenever the needed length exceeds what the layer has).  Shapes smaller
    // than that abort in the reference ("Out of bounds allocation"); here the last block is cut at
    // the end of the region and a block shared by two layers is committed once.
    const size_t needed = ( token_pos + 1 ) * Config::kv_dim * 2 * sizeof( DType );
    if ( needed > layer_allocated_offsets_[layer_num] ) {
      const size_t region_len = storage_->max_len();
      const size_t layer_off = static_cast<size_t>( reinterpret_cast<const uint8_t*>( layer.data() ) - static_cast<const uint8_t*>( storage_->ptr() ) );
      const size_t last_block = ( layer_off + needed - 1 ) / BLOCK_SIZE;
      if ( block_committed_.size() < ( region_len + BLOCK_SIZE - 1 ) / BLOCK_SIZE ) {
        block_committed_.resize( ( region_len + BLOCK_SIZE - 1 ) / BLOCK_SIZE, false );
      }
      for ( size_t b = layer_off / BLOCK_SIZE; b <= last_block; b++ ) {
        if ( !block_committed_[b] ) {
          const size_t begin = b * BLOCK_SIZE;
          storage_->allocate_span( static_cast<const uint8_t*>( storage_->ptr() ) + begin, std::min( BLOCK_SIZE, region_len - begin ) );
          block_committed_[b] = true;
          blocks_committed_++;
        }
      }
      layer_allocated_offsets_[layer_num] = std::min( ( last_block + 1 ) * BLOCK_SIZE, region_len ) - layer_off;
    }
    return true;
  }

  size_t allocated_bytes( const size_t layer_num ) const { return layer_allocated_offsets_[layer_num]; }
  size_t blocks_committed() const { return blocks_committed_; }
  size_t clears() const { return clears_; }
};

static_assert( ContextConcept<Context<configs::Stories_110M, float>, float> );
static_assert( LayerContextConcept<LayerContext<configs::Stories_110M, float>, float> );
static_assert( TokenContextConcept<TokenContext<configs::Stories_110M, float>, float> );

} // namespace glint
