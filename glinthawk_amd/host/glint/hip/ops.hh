// The `hip` target: Operations<DType> and LlamaOperations<Config, DType, Ctx>, the two classes a
// Glinthawk backend provides (models/common/ops/concept.hh:16-40, models/llama2/ops/concept.hh:15-42),
// with the method names, argument order and meaning of the amd64 / cuda targets
// (arch/amd64/common/ops.hh:13-63, arch/amd64/llama2/ops.hh:23-68).  Every method is one call into
// libglint_hip.so; a non-zero status aborts, as every device error does in the reference.
#pragma once

#include <memory>
#include <string>
#include <type_traits>
#include <vector>

#include "glint/config.hh"
#include "glint/context.hh"
#include "glint/state.hh"
#include "glint/types.hh"
#include "glint_hip.h"

namespace glint::hip {

#define GLINT_GH( call )                                                                                               \
  do {                                                                                                                 \
    if ( ( call ) != GH_OK ) {                                                                                         \
      ::glint::fatal( __FILE__, __LINE__, #call, gh_last_error() );                                                    \
    }                                                                                                                  \
  } while ( 0 )

template<typename DType>
constexpr gh_dtype gh_type()
{
  return sizeof( DType ) == 2 ? GH_F16 : GH_F32;
}

inline gh_copy_kind gh_kind( const CopyType t )
{
  switch ( t ) {
    case CopyType::HostToDevice: return GH_HOST_TO_DEVICE;
    case CopyType::DeviceToHost: return GH_DEVICE_TO_HOST;
    case CopyType::DeviceToDevice: return GH_DEVICE_TO_DEVICE;
    default: return GH_HOST_TO_HOST;
  }
}

template<typename PtrType>
struct DeviceDeleter
{
  void operator()( PtrType* ptr ) const
  {
    if ( ptr ) {
      GLINT_GH( gh_free( ptr ) );
    }
  }
};

// From the first Operations object on, the state's host buffers (activations, queries, kvs) are
// page-locked: their transfers need no staging copy.  Installed once per process.
inline void use_pinned_state_buffers()
{
  static const bool installed = [] {
    HostBufferPool::instance().set_source(
      []( size_t n ) -> void* {
        void* p = nullptr;
        return gh_host_malloc( &p, n ) == GH_OK ? p : nullptr;
      },
      []( void* p ) { (void)gh_host_free( p ); } );
    return true;
  }();
  (void)installed;
}

template<typename DType>
class Operations
{
public:
  using DeviceUniquePtr = std::unique_ptr<DType, DeviceDeleter<DType>>;

  Operations()
  {
    GLINT_GH( gh_init( 0 ) );
    use_pinned_state_buffers();
  }
  ~Operations() = default;
  Operations( const Operations& ) = delete;
  Operations& operator=( const Operations& ) = delete;
  Operations( Operations&& ) = default;
  Operations& operator=( Operations&& ) = default;

  // all work is queued on this stream (NULL = the default stream)
  void set_stream( gh_stream s ) { stream_ = s; }
  gh_stream stream() const { return stream_; }
  void synchronize() const
  {
    GLINT_GH( gh_sync( stream_ ) );
    drains_++;
  }
  // how often the stream has been waited for until it was empty (synchronize(), blocking copies): work queued before the last
  // of them has finished
  uint64_t drain_count() const { return drains_; }

  template<uint64_t size>
  void accum( DType* a, const DType* b, const uint64_t batch_size ) const
  {
    GLINT_GH( gh_accum( a, b, size, batch_size, gh_type<DType>(), stream_ ) );
  }

  // `temp` is unused: the kernel reduces in registers / LDS
  template<uint64_t size>
  void rmsnorm( DType* o, const DType* x, float32_t*, const DType* weight, const uint64_t batch_size ) const
  {
    GLINT_GH( gh_rmsnorm( o, x, weight, size, batch_size, gh_type<DType>(), stream_ ) );
  }

  // `output` is a HOST array (ScratchPad::argmax_pos); `temp` is device scratch with room for batch_size uint32
  template<uint64_t n>
  void argmax( uint32_t* output, const DType* v, DType* temp, const uint64_t batch_size ) const
  {
    GLINT_GH( gh_argmax( output, reinterpret_cast<uint32_t*>( temp ), v, n, batch_size, gh_type<DType>(), stream_ ) );
  }

  template<uint64_t hidden_dim>
  void silu( DType* hb, DType* hb2, const uint64_t batch_size ) const
  {
    GLINT_GH( gh_silu( hb, hb2, hidden_dim, batch_size, gh_type<DType>(), stream_ ) );
  }

  template<uint64_t s, uint64_t r>
  void matmul( DType* xo, const DType* x, const DType* w, const uint64_t b ) const
  {
    GLINT_GH( gh_matmul( xo, x, w, s, r, b, gh_type<DType>(), stream_ ) );
  }

  void untemplated_matmul( DType* xo, const DType* x, const DType* w, const uint64_t s, const uint64_t r, const uint64_t b ) const
  {
    GLINT_GH( gh_matmul( xo, x, w, s, r, b, gh_type<DType>(), stream_ ) );
  }

  void soft_sample( DType* v, const std::vector<float>& temperatures, const size_t vocab_size ) const
  {
    GLINT_GH( gh_soft_sample( v, temperatures.data(), vocab_size, temperatures.size(), sample_seed_++, gh_type<DType>(), stream_ ) );
  }

  DeviceUniquePtr device_allocate( const uint64_t size_bytes ) const
  {
    void* p = nullptr;
    GLINT_GH( gh_malloc( &p, size_bytes ) );
    return DeviceUniquePtr { static_cast<DType*>( p ) };
  }

  void randomize_device_buffer( DType* buffer, const uint64_t len, const float min, const float max ) const
  {
    GLINT_GH( gh_fill_uniform( buffer, len, min, max, fill_seed_++, gh_type<DType>(), stream_ ) );
  }

  void copy( DType* dst, const DType* src, const uint64_t len_bytes, const CopyType type, const bool async = false ) const
  {
    GLINT_GH( gh_memcpy( dst, src, len_bytes, gh_kind( type ), async ? 1 : 0, stream_ ) );
    if ( !async && len_bytes > 0 ) { // a copy of nothing returns without waiting for the stream
      drains_++;
    }
  }

  void print( const DType* x, const uint64_t b, const std::string base ) const
  {
    std::vector<DType> host( b );
    GLINT_GH( gh_memcpy( host.data(), x, b * sizeof( DType ), GH_DEVICE_TO_HOST, 0, stream_ ) );
    std::printf( "%s", base.c_str() );
    for ( uint64_t i = 0; i < b; i++ ) {
      std::printf( "\t%.10f", static_cast<float>( host[i] ) );
    }
    std::printf( "\n" );
  }

protected:
  gh_stream stream_ { nullptr };
  mutable uint64_t drains_ { 0 };
  mutable uint64_t sample_seed_ { 0x5eed };
  mutable uint64_t fill_seed_ { 0xf111 };
};

// platform-specific context: storage is one device allocation owned by the context
// (arch/cuda/llama2/ops.cuh:66-76,108-126)
template<typename Config, typename DType>
class Context : public glint::Context<Config, DType>
{
  typename Operations<DType>::DeviceUniquePtr storage_ {};

public:
  Context() = default;

  template<typename Settings>
  explicit Context( const Settings& settings, const bool make_empty = false )
  {
    DType* ptr = nullptr;
    if ( !make_empty ) {
      void* p = nullptr;
      GLINT_GH( gh_malloc( &p, glint::Context<Config, DType>::max_size( settings.num_attention_layers_hosted() ) ) );
      ptr = static_cast<DType*>( p );
    }
    storage_.reset( ptr );
    this->set_buffer( settings, ptr );
  }
};

// common::hip::VirtualMemoryRegion: address-space reservation with 2 MiB commits
// (arch/cuda/common/vmem.cuh:60-160, arch/amd64/common/vmem.hh:43-79)
class VirtualMemoryRegion
{
  gh_vmm* region_ { nullptr };

public:
  explicit VirtualMemoryRegion( const size_t len ) { GLINT_GH( gh_vmm_reserve( &region_, len ) ); }
  ~VirtualMemoryRegion()
  {
    if ( region_ ) {
      GLINT_GH( gh_vmm_free( region_ ) );
    }
  }
  VirtualMemoryRegion( const VirtualMemoryRegion& ) = delete;
  VirtualMemoryRegion& operator=( const VirtualMemoryRegion& ) = delete;
  VirtualMemoryRegion( VirtualMemoryRegion&& other ) noexcept
    : region_( other.region_ )
  {
    other.region_ = nullptr;
  }
  VirtualMemoryRegion& operator=( VirtualMemoryRegion&& other ) noexcept
  {
    std::swap( region_, other.region_ );
    return *this;
  }

  // out-of-range spans abort ("Out of bounds allocation" in the reference)
  void allocate_span( const void* ptr, const size_t len )
  {
    const auto offset = static_cast<uint64_t>( static_cast<const uint8_t*>( ptr ) - static_cast<const uint8_t*>( this->ptr() ) );
    GLINT_GH( gh_vmm_commit( region_, offset, len ) );
  }

  void* ptr() const { return gh_vmm_ptr( region_ ); }
  size_t max_len() const { return gh_vmm_max_len( region_ ); }
  size_t committed() const { return gh_vmm_committed_bytes( region_ ); }
  void clear() { GLINT_GH( gh_vmm_clear( region_ ) ); }
};

template<typename Config, typename DType>
using DynamicContext = glint::DynamicContext<Config, DType, VirtualMemoryRegion>;

template<typename Config, typename DType, typename Ctx = Context<Config, DType>>
requires ModelConfig<Config> && ContextConcept<Ctx, DType>
class LlamaOperations : public Operations<DType>
{
public:
  using typename Operations<DType>::DeviceUniquePtr;
  using ContextType = Ctx;

  template<typename Settings>
  explicit LlamaOperations( const Settings& )
  {
  }
  ~LlamaOperations() = default;

  static gh_shape shape()
  {
    return gh_shape { (uint32_t)Config::dim,     (uint32_t)Config::kv_dim,     (uint32_t)Config::hidden_dim, (uint32_t)Config::n_layers,
                      (uint32_t)Config::head_size, (uint32_t)Config::n_heads,  (uint32_t)Config::n_kv_heads, (uint32_t)Config::gqa_size,
                      (uint32_t)Config::vocab_size, (uint32_t)Config::seq_len };
  }

  // `layer_contexts` / `token_contexts` / `token_positions` are HOST arrays (ScratchPad members,
  // models/llama2/base.hh:199-202) holding device addresses; the library stages them.
  void attention_0_gemm( const DType* query,
                         const typename ContextType::LayerContextType layer_contexts[],
                         DType* att,
                         const uint64_t batch_size,
                         const uint32_t* token_positions ) const
  {
    const gh_shape s = shape();
    GLINT_GH( gh_attn_scores_host( query, layer_table( layer_contexts, batch_size ), att, batch_size, token_positions, &s, gh_type<DType>(), this->stream_ ) );
  }

  void attention_2_gemm( const DType* att,
                         const typename ContextType::LayerContextType layer_contexts[],
                         DType* xb,
                         const uint64_t batch_size,
                         const uint32_t* token_positions ) const
  {
    const gh_shape s = shape();
    GLINT_GH( gh_attn_pv_host( att, layer_table( layer_contexts, batch_size ), xb, batch_size, token_positions, &s, gh_type<DType>(), this->stream_ ) );
  }

  void attention_softmax( DType* att, const uint32_t* token_positions, DType*, const uint64_t batch_size ) const
  {
    const gh_shape s = shape();
    GLINT_GH( gh_attn_softmax_host( att, token_positions, batch_size, &s, gh_type<DType>(), this->stream_ ) );
  }

  void apply_rope( const uint64_t batch_size,
                   const uint32_t* token_positions,
                   const DType* freq_cis_real,
                   const DType* freq_cis_imag,
                   DType* state_q,
                   typename ContextType::TokenContextType token_contexts[] ) const
  {
    GLINT_GH( gh_rope_host( batch_size, token_positions, freq_cis_real, freq_cis_imag, state_q, token_table( token_contexts, batch_size ),
                            Config::n_kv_heads, Config::gqa_size, Config::head_size, gh_type<DType>(), this->stream_ ) );
  }

  void copy_kv_cache( typename ContextType::TokenContextType token_contexts[], const DType* state_kv, const uint64_t batch_size ) const
  {
    GLINT_GH( gh_kv_append_host( token_table( token_contexts, batch_size ), state_kv, batch_size, Config::kv_dim, gh_type<DType>(), this->stream_ ) );
  }

  // <void, void> is the instantiation the reference's concept names (models/llama2/ops/concept.hh:36): the element is
  // then a byte (sizeof( void ) is 1 in the reference's GNU dialect, arch/amd64/llama2/ops.hh:361-362), i.e. a plain
  // synchronous copy of `size` bytes.
  template<typename DTypeDst, typename DTypeSrc>
  void convert_and_copy( DTypeDst* dst, const DTypeSrc* src, const uint64_t size, const CopyType type ) const
  {
    if constexpr ( std::is_void_v<DTypeDst> && std::is_void_v<DTypeSrc> ) {
      GLINT_GH( gh_memcpy( dst, src, size, gh_kind( type ), 0, this->stream_ ) );
    } else {
      static_assert( !std::is_void_v<DTypeDst> && !std::is_void_v<DTypeSrc>, "convert_and_copy: void on one side only" );
      GLINT_GH( gh_convert_and_copy( dst, gh_type<DTypeDst>(), src, gh_type<DTypeSrc>(), size, gh_kind( type ), this->stream_ ) );
    }
  }

  // Extension used by the stage driver: attention_0_gemm + attention_softmax + attention_2_gemm in
  // one fused split-K kernel without the `att` buffer.  Tables live in device memory.
  void attention_fused( const DType* query,
                        const void* const* layer_rows_dev,
                        const uint32_t* token_positions_dev,
                        DType* xb,
                        const uint64_t batch_size,
                        const uint32_t max_pos,
                        void* workspace,
                        const uint64_t workspace_bytes ) const
  {
    const gh_shape s = shape();
    GLINT_GH( gh_attn_decode( query, layer_rows_dev, token_positions_dev, xb, batch_size, max_pos, &s, gh_type<DType>(), workspace, workspace_bytes,
                              GH_ATTN_AUTO, this->stream_ ) );
  }

  // Extensions used by the stage driver: a projection together with the ops that follow it in the
  // layer (same arithmetic and rounding points as the separate calls, fewer launches).
  // wo / w2 + accum (+ the rmsnorm that follows): x += xb . w^T; norm_out = rmsnorm(x) * norm_weight
  template<uint64_t s, uint64_t r>
  void matmul_accum( DType* x, const DType* xb, const DType* w, const uint64_t batch_size, DType* norm_out = nullptr, const DType* norm_weight = nullptr ) const
  {
    GLINT_GH( gh_matmul_accum( x, xb, w, s, r, batch_size, norm_out, norm_weight, gh_type<DType>(), this->stream_ ) );
  }
  // two products that share their activations, their weights one behind the other (wq then wkv): xa = xb . w[0:ra]^T, xo_b = xb . w[ra:]^T
  template<uint64_t s, uint64_t ra, uint64_t rb>
  void matmul_pair( DType* xo_a, DType* xo_b, const DType* xb, const DType* w, const uint64_t batch_size ) const
  {
    GLINT_GH( gh_matmul_pair( xo_a, xo_b, xb, w, s, ra, rb, batch_size, gh_type<DType>(), this->stream_ ) );
  }
  // w1, w3, silu: hb = silu(xb . w1^T) * (xb . w3^T); w13 holds the rows of w1 followed by those of w3
  void matmul_silu_gate( DType* hb, const DType* xb, const DType* w13, const uint64_t batch_size ) const
  {
    GLINT_GH( gh_matmul_silu_gate( hb, xb, w13, Config::dim, Config::hidden_dim, batch_size, gh_type<DType>(), this->stream_ ) );
  }
  // wq, wkv, copy_kv_cache, apply_rope: wqkv holds the rows of wq followed by those of wkv
  void matmul_qkv_rope_append( DType* q,
                               const DType* xb,
                               const DType* wqkv,
                               const uint64_t batch_size,
                               const uint32_t* token_positions_dev,
                               const DType* freq_cis_real,
                               const DType* freq_cis_imag,
                               void* const* token_rows_dev ) const
  {
    GLINT_GH( gh_matmul_qkv_rope_append( q, nullptr, xb, wqkv, Config::dim, batch_size, token_positions_dev, freq_cis_real, freq_cis_imag, token_rows_dev,
                                         Config::n_kv_heads, Config::gqa_size, Config::head_size, gh_type<DType>(), this->stream_ ) );
  }

private:
  // TokenContext / LayerContext are a single pointer each, so an array of them is a pointer table
  static_assert( sizeof( typename ContextType::TokenContextType ) == sizeof( void* ) );
  static_assert( sizeof( typename ContextType::LayerContextType ) == sizeof( void* ) );

  static void* const* token_table( typename ContextType::TokenContextType token_contexts[], uint64_t )
  {
    return reinterpret_cast<void* const*>( token_contexts );
  }
  static const void* const* layer_table( const typename ContextType::LayerContextType layer_contexts[], uint64_t )
  {
    return reinterpret_cast<const void* const*>( layer_contexts );
  }
};

} // namespace glint::hip
