// C entry points over the C++ host layer (libglint_host.so): a stage harness -- model driver +
// context manager + one batched state -- for the benchmark and the tests, and host-only hooks that
// exercise the slot bookkeeping and the paging rule without a GPU.
#include <cstring>
#include <deque>
#include <memory>
#include <chrono>
#include <string>
#include <thread>
#include <vector>

#include "glint/contextman.hh"
#include "glint/kernel.hh"
#include "glint/loader.hh"
#include "glint/model.hh"

using namespace glint;

namespace {

// ---------------------------------------------------------------------------------------------
// type-erased stage harness
// ---------------------------------------------------------------------------------------------
struct StageBase
{
  virtual ~StageBase() = default;
  virtual void set_layer_tensor( size_t layer, size_t k, const void* host, uint64_t n ) = 0;
  virtual void set_base_tensor( size_t k, const void* host, uint64_t n ) = 0;
  virtual const void* layer_tensor_ptr( size_t layer, size_t k, uint64_t* n ) = 0;
  virtual const void* base_tensor_ptr( size_t k, uint64_t* n ) = 0;
  virtual std::string load_dir( const char* model_dir ) = 0;
  virtual std::string set_state_bytes( const void* bytes, uint64_t len ) = 0;
  virtual std::string get_state_bytes() = 0;
  virtual void new_state( uint32_t batch, uint32_t next_layer, int next_stage ) = 0;
  virtual void set_prompt( size_t i, uint32_t context_id, uint32_t token, uint32_t pos, float temp, uint32_t plen, uint32_t mcl ) = 0;
  virtual void discard( size_t i ) = 0;
  virtual void set_next( uint32_t layer, int stage ) = 0;
  virtual int acquire_contexts() = 0;
  virtual int forward( int which ) = 0;
  virtual void* buffer( int which, uint64_t* bytes, bool allocate ) = 0;
  virtual void row_info( size_t i, uint32_t out[6] ) = 0;
  virtual void state_info( uint32_t out[4] ) = 0;
  virtual void* context_layer_ptr( size_t row, size_t layer ) = 0;
  virtual int32_t context_slot( size_t row ) = 0;
  virtual void slot_counts( uint64_t out[3] ) = 0;
  virtual void* scratch( int which ) = 0;
  virtual int release_context( uint32_t id ) = 0;
  virtual void paging_info( size_t row, size_t layer, uint64_t out[3] ) = 0;
  virtual void sync() = 0;
  virtual void copy_bytes( void* dst, const void* src, uint64_t bytes, int kind ) = 0;
  virtual void time_device_spans( bool on ) = 0;
  virtual void device_spans( double* ms, uint64_t* spans ) = 0;
  virtual int prefill( uint32_t batch, const uint32_t* context_ids, const uint32_t* start_pos, uint32_t n_tokens, uint32_t first_layer,
                       const uint32_t* token_ids, const void* acts_in, void* acts_out, uint32_t* next_tokens ) = 0;
};

template<typename Config, typename DType, typename Ctx>
struct StageImpl : StageBase
{
  using Model = Llama2<Config, DType, hip::LlamaOperations<Config, DType, Ctx>, Ctx>;
  using State = typename Model::StateType;

  Model model;
  PreallocatingContextManager<Model> contexts;
  State state {};
  typename Model::ContextVector held {};

  StageImpl( const StageSettings<Config>& s, const ModelOptions& o )
    : model( s, o )
    , contexts( s )
  {
  }
  std::string load_dir( const char* model_dir ) override { return load_model_dir( model, model_dir ); }
  // a state as it arrives from / leaves for the neighbouring stage (models/common/state.hh:512-594)
  std::string set_state_bytes( const void* bytes, uint64_t len ) override
  {
    std::string why;
    State parsed;
    if ( !State::parse( std::string_view( static_cast<const char*>( bytes ), len ), parsed, &why ) ) {
      return why;
    }
    if ( parsed.dtype() != dtype_of<DType>() && parsed.next_stage() != InferenceStage::Attention ) {
      return "state data type does not match the stage";
    }
    state = std::move( parsed );
    held.clear();
    return {};
  }
  std::string get_state_bytes() override { return state.serialize(); }

  void set_layer_tensor( size_t layer, size_t k, const void* host, uint64_t n ) override
  {
    model.set_layer_tensor( layer, k, static_cast<const DType*>( host ), n );
  }
  void set_base_tensor( size_t k, const void* host, uint64_t n ) override { model.set_base_tensor( k, static_cast<const DType*>( host ), n ); }
  // device address and element count of a resident tensor (file order), nullptr / 0 when the stage does not host it
  const void* layer_tensor_ptr( size_t layer, size_t k, uint64_t* n ) override
  {
    *n = 0;
    if ( layer >= Config::n_layers || k >= 8 ) {
      return nullptr;
    }
    *n = WeightLayout<Config>::layer_in_memory( model.settings(), layer )[k];
    return *n ? model.layer_weights( layer ).tensor( k ) : nullptr;
  }
  const void* base_tensor_ptr( size_t k, uint64_t* n ) override
  {
    *n = 0;
    if ( k >= 5 ) {
      return nullptr;
    }
    const auto& b = model.base_weights();
    const DType* const t[5] = { b.token_embedding_table, b.rms_final_weight, b.freq_cis_real, b.freq_cis_imag, b.wcls };
    *n = t[k] ? WeightLayout<Config>::base_in_memory( model.settings() )[k] : 0;
    return t[k];
  }

  void new_state( uint32_t batch, uint32_t next_layer, int next_stage ) override
  {
    state = State( batch, dtype_of<DType>() );
    state.set_next_layer( next_layer );
    state.set_next_stage( static_cast<InferenceStage>( next_stage ) );
    held.clear();
  }
  void set_prompt( size_t i, uint32_t context_id, uint32_t token, uint32_t pos, float temp, uint32_t plen, uint32_t mcl ) override
  {
    GLINT_CHECK( i < state.batch_size() );
    state.set_prompt( i, context_id, token, pos, temp, plen, mcl );
  }
  void discard( size_t i ) override
  {
    GLINT_CHECK( i < state.batch_size() );
    state.discard( i );
  }
  void set_next( uint32_t layer, int stage ) override
  {
    state.set_next_layer( layer );
    state.set_next_stage( static_cast<InferenceStage>( stage ) );
  }

  int acquire_contexts() override
  {
    auto got = contexts.get_contexts( state );
    if ( !got.has_value() ) {
      return -1; // not enough free slots: nothing was allocated
    }
    held = std::move( *got );
    return 0;
  }

  // which: 0 forward (all hosted stages), 1 pre-attention, 2 attention, 3 post-attention, 4 classify
  int forward( int which ) override
  {
    if ( which == 0 || which == 2 ) {
      if ( acquire_contexts() != 0 ) {
        return -1;
      }
    }
    switch ( which ) {
      case 0: model.forward( state, held ); break;
      case 1: model.forward_pre_attention( state ); break;
      case 2: model.forward_attention( state, held ); break;
      case 3: model.forward_post_attention( state ); break;
      case 4: model.forward_classify( state ); break;
      default: return -2;
    }
    return 0;
  }

  // which: 0 activations, 1 queries, 2 kvs (host buffers of the state)
  void* buffer( int which, uint64_t* bytes, bool allocate ) override
  {
    DataBuffer* b = which == 0 ? &state.activations() : which == 1 ? &state.queries() : &state.kvs();
    if ( allocate && b->len() == 0 ) {
      if ( which == 0 ) {
        state.allocate_activations();
      } else if ( which == 1 ) {
        state.allocate_queries();
      } else {
        state.allocate_kvs();
      }
    }
    *bytes = b->len();
    return b->data();
  }

  void row_info( size_t i, uint32_t out[6] ) override
  {
    out[0] = state.active( i );
    out[1] = state.context_id( i );
    out[2] = state.token( i );
    out[3] = state.token_pos( i );
    out[4] = state.finished( i );
    out[5] = static_cast<uint32_t>( state.temperature( i ) * 255.0f + 0.5f );
  }
  void state_info( uint32_t out[4] ) override
  {
    out[0] = state.batch_size();
    out[1] = state.next_layer();
    out[2] = static_cast<uint32_t>( state.next_stage() );
    out[3] = ( state.has_activations() ? 1u : 0u ) | ( state.has_queries() ? 2u : 0u ) | ( state.has_kvs() ? 4u : 0u );
  }

  void* context_layer_ptr( size_t row, size_t layer ) override { return row < held.size() ? held[row]->layer( layer ).data() : nullptr; }
  int32_t context_slot( size_t row ) override { return row < held.size() ? contexts.slot_index( held[row] ) : -2; }
  void slot_counts( uint64_t out[3] ) override
  {
    out[0] = contexts.free();
    out[1] = contexts.allocated();
    out[2] = contexts.total();
  }
  int release_context( uint32_t id ) override { return contexts.release_context( id ) ? 1 : 0; }

  void paging_info( size_t row, size_t layer, uint64_t out[3] ) override
  {
    out[0] = out[1] = out[2] = 0;
    if constexpr ( requires( Ctx c ) { c.allocated_bytes( 0 ); } ) {
      if ( row < held.size() ) {
        out[0] = held[row]->allocated_bytes( layer );
        out[1] = held[row]->blocks_committed();
        out[2] = held[row]->clears();
      }
    }
  }

  // which: 0 x, 1 xb, 2 q, 3 kv, 4 logits
  void* scratch( int which ) override
  {
    switch ( which ) {
      case 0: return model.scratch_x();
      case 1: return model.scratch_xb();
      case 2: return model.scratch_q();
      case 3: return model.scratch_kv();
      default: return model.scratch_logits();
    }
  }
  void sync() override { model.ops().synchronize(); }
  // the instantiation the reference's concept names: convert_and_copy<void, void>, a copy of `bytes` bytes
  void copy_bytes( void* dst, const void* src, uint64_t bytes, int kind ) override
  {
    model.ops().template convert_and_copy<void, void>( dst, src, bytes, static_cast<CopyType>( kind ) );
  }
  void time_device_spans( bool on ) override { model.time_device_spans( on ); }
  void device_spans( double* ms, uint64_t* spans ) override
  {
    const auto [total, n] = model.device_spans();
    *ms = total;
    *spans = n;
  }

  int prefill( uint32_t batch, const uint32_t* context_ids, const uint32_t* start_pos, uint32_t n_tokens, uint32_t first_layer, const uint32_t* token_ids,
               const void* acts_in, void* acts_out, uint32_t* next_tokens ) override
  {
    State tmp( batch, dtype_of<DType>() );
    for ( uint32_t i = 0; i < batch; i++ ) {
      tmp.set_prompt( i, context_ids[i], 0, start_pos[i], 0.0f, n_tokens, 0 );
    }
    auto got = contexts.get_contexts( tmp );
    if ( !got.has_value() ) {
      return -1;
    }
    held = std::move( *got );
    model.prefill( held, start_pos, n_tokens, first_layer, token_ids, static_cast<const DType*>( acts_in ), static_cast<DType*>( acts_out ), next_tokens );
    return 0;
  }
};

template<typename Config>
StageBase* make_for_config( int dtype, bool paged, const StageSettings<Config>& s, const ModelOptions& o )
{
  if ( dtype == 0 ) {
    if ( paged ) {
      return new StageImpl<Config, float16_t, hip::DynamicContext<Config, float16_t>>( s, o );
    }
    return new StageImpl<Config, float16_t, hip::Context<Config, float16_t>>( s, o );
  }
  if ( paged ) {
    return new StageImpl<Config, float32_t, hip::DynamicContext<Config, float32_t>>( s, o );
  }
  return new StageImpl<Config, float32_t, hip::Context<Config, float32_t>>( s, o );
}

template<typename Config>
StageBase* make_stage( int dtype, uint32_t first_layer, uint32_t n_hosted, uint32_t concurrency, uint32_t max_contexts, uint32_t flags, uint64_t seed, float std )
{
  const bool with_cls = flags & 2u;
  auto s = StageSettings<Config>::slice( first_layer, n_hosted, concurrency, max_contexts, with_cls );
  ModelOptions o;
  o.fused_attention = flags & 1u;
  o.fused_projections = !( flags & 8u );
  o.balanced_attention = ( flags & 16u ) ? 1 : ( ( flags & 32u ) ? -1 : 0 );
  o.seed = seed;
  o.weight_std = std;
  return make_for_config<Config>( dtype, flags & 4u, s, o );
}

// ---------------------------------------------------------------------------------------------
// host-only stand-ins for the bookkeeping tests (no device memory involved)
// ---------------------------------------------------------------------------------------------
struct CountingRegion // VirtualMemoryRegion surface without memory: records what would be committed
{
  size_t len_;
  std::vector<std::pair<size_t, size_t>> spans_ {};
  size_t clears_ { 0 };
  explicit CountingRegion( size_t len )
    : len_( len )
  {
  }
  void allocate_span( const void* ptr, size_t len )
  {
    const size_t off = reinterpret_cast<uintptr_t>( ptr ) - reinterpret_cast<uintptr_t>( this->ptr() );
    GLINT_CHECK( off + len <= len_ );
    spans_.emplace_back( off, len );
  }
  void* ptr() const { return reinterpret_cast<void*>( uintptr_t { 1 } << 40 ); } // fake, never dereferenced
  size_t max_len() const { return len_; }
  void clear()
  {
    spans_.clear();
    clears_++;
  }
};

using BookConfig = configs::Llama2_70B_Chat_4K;

struct HostOnlyContext : glint::Context<BookConfig, float16_t>
{
  HostOnlyContext() = default;
  template<typename Settings>
  explicit HostOnlyContext( const Settings& s, bool make_empty = false )
  {
    this->set_buffer( s, make_empty ? nullptr : reinterpret_cast<float16_t*>( uintptr_t { 1 } << 40 ) );
  }
};

struct BookModel
{
  using ConfigType = BookConfig;
  using ContextType = HostOnlyContext;
  using SettingsType = StageSettings<BookConfig>;
};

struct BookManager
{
  PreallocatingContextManager<BookModel> man;
  explicit BookManager( uint64_t n )
    : man( StageSettings<BookConfig>::slice( 0, 1, 1024, n ) )
  {
  }
};

using PagedBookContext = glint::DynamicContext<BookConfig, float16_t, CountingRegion>;

thread_local std::string g_last_error;
thread_local std::string g_bytes; // result of the last call that returns bytes

// host-only: states of one fixed shape for the tests of the wire format and of refill / split / merge
using BookState = BatchedInferenceState<configs::Test_Tiny>;
BookState* as_state( void* h ) { return static_cast<BookState*>( h ); }

// ---------------------------------------------------------------------------------------------
// compute kernel (push / pop / eventfd), type-erased; states cross as wire-format bytes
// ---------------------------------------------------------------------------------------------
struct KernelBase
{
  virtual ~KernelBase() = default;
  virtual std::string push_bytes( const void* bytes, uint64_t len ) = 0;
  virtual bool pop_bytes( std::string& out ) = 0;
  virtual EventFD& event_fd() = 0;
  virtual void slot_counts( uint64_t out[3] ) = 0;
  virtual std::string load_dir( const char* ) { return "this kernel has no weights to load"; }
};

template<typename Model>
struct KernelImpl : KernelBase
{
  BatchedComputeKernel<Model> kernel;
  template<typename... Args>
  explicit KernelImpl( Args&&... args )
    : kernel( std::forward<Args>( args )... )
  {
  }
  std::string push_bytes( const void* bytes, uint64_t len ) override
  {
    typename BatchedComputeKernel<Model>::BatchedState state;
    std::string why;
    if ( !BatchedComputeKernel<Model>::BatchedState::parse( std::string_view( static_cast<const char*>( bytes ), len ), state, &why ) ) {
      return why;
    }
    if ( state.batch_size() == 0 || state.batch_size() > kernel.model().settings().concurrency_limit ) {
      return "batch size outside the kernel's concurrency limit";
    }
    kernel.push( std::move( state ) );
    return {};
  }
  bool pop_bytes( std::string& out ) override
  {
    typename BatchedComputeKernel<Model>::BatchedState state;
    if ( !kernel.pop( state ) ) {
      return false;
    }
    out = state.serialize();
    return true;
  }
  EventFD& event_fd() override { return kernel.event_fd(); }
  void slot_counts( uint64_t out[3] ) override
  {
    out[0] = kernel.context_manager().free();
    out[1] = kernel.context_manager().allocated();
    out[2] = kernel.context_manager().total();
  }
  std::string load_dir( const char* dir ) override
  {
    if constexpr ( requires( Model& m ) { m.base_weights(); } ) {
      return load_model_dir( kernel.model(), dir );
    } else {
      return KernelBase::load_dir( dir );
    }
  }
};

// host-only model for the queue tests: no device, forward() advances every active row by one
// token and takes a data-dependent nap so that the two threads interleave differently every time
struct EchoContext : glint::Context<configs::Test_Tiny, float16_t>
{
  EchoContext() = default;
  template<typename Settings>
  explicit EchoContext( const Settings& s, bool make_empty = false )
  {
    this->set_buffer( s, make_empty ? nullptr : reinterpret_cast<float16_t*>( uintptr_t { 1 } << 40 ) );
  }
};
struct EchoModel
{
  using ConfigType = configs::Test_Tiny;
  using ContextType = EchoContext;
  using SettingsType = StageSettings<configs::Test_Tiny>;
  using StateType = BatchedInferenceState<configs::Test_Tiny>;
  SettingsType settings_;
  explicit EchoModel( const SettingsType& s )
    : settings_( s )
  {
  }
  const SettingsType& settings() const { return settings_; }
  void forward( StateType& states, const std::vector<std::shared_ptr<EchoContext>>& contexts )
  {
    GLINT_CHECK( contexts.size() == states.batch_size() );
    uint32_t nap = 0;
    for ( size_t i = 0; i < states.batch_size(); i++ ) {
      GLINT_CHECK( states.active( i ) != contexts[i]->empty() ); // active rows got a slot, the others the shared empty context
      if ( states.active( i ) ) {
        nap += states.token( i );
        states.set_token( i, states.token( i ) + 1 );
        states.set_token_pos( i, states.token_pos( i ) + 1 );
      }
    }
    std::this_thread::sleep_for( std::chrono::microseconds( ( nap % 7 ) * 30 ) );
  }
};

} // namespace

extern "C" {

// ---- stage harness --------------------------------------------------------------------------
// flags: 1 fused attention, 2 host the classifier, 4 paged (virtual-memory) contexts, 8 keep the projections unfused,
// 16 / 32 decode attention over equal runs of keys always / never (neither: where a step's lengths call for it)
void* glint_stage_create( const char* config, int dtype, uint32_t first_layer, uint32_t n_hosted, uint32_t concurrency, uint32_t max_contexts,
                          uint32_t flags, uint64_t seed, float weight_std )
{
  const std::string name( config );
#define GLINT_CASE( NAME, CFG )                                                                                        \
  if ( name == NAME ) {                                                                                                \
    return make_stage<configs::CFG>( dtype, first_layer, n_hosted, concurrency, max_contexts, flags, seed, weight_std ); \
  }
  GLINT_CASE( "llama2-70b-4k", Llama2_70B_Chat_4K )
  GLINT_CASE( "llama2-70b-8k", Llama2_70B_Chat_8K )
  GLINT_CASE( "llama2-13b-4k", Llama2_13B_Chat_4K )
  GLINT_CASE( "llama2-7b", Llama2_7B_Chat )
  GLINT_CASE( "stories15m", Stories_15M )
  GLINT_CASE( "test-gqa4", Test_GQA4 )
  GLINT_CASE( "test-mha", Test_MHA )
  GLINT_CASE( "test-tiny", Test_Tiny )
#undef GLINT_CASE
  return nullptr;
}

void glint_stage_destroy( void* h ) { delete static_cast<StageBase*>( h ); }

// the reference's model directory (CONFIG, BASEWEIGHTS_<DT>, LAYER<i>_<DT>) -> the tensors this stage hosts.
// 0 on success; otherwise nothing is guaranteed about the weights and glint_last_error() says what was wrong.
int glint_stage_load( void* h, const char* model_dir )
{
  g_last_error = static_cast<StageBase*>( h )->load_dir( model_dir );
  return g_last_error.empty() ? 0 : -1;
}
const char* glint_last_error() { return g_last_error.c_str(); }

// Host-only walk over a model directory for a stage hosting layers [first_layer, first_layer + n_hosted)
// (flags & 2: the classifier too): checks CONFIG and the size of every file the stage would open, and
// records each resident tensor as 4 numbers (is_base, layer, k in file order, byte offset in the file)
// followed by its element count, up to `max_records`.  Returns the number of tensors, or -1 (see glint_last_error()).
int64_t glint_model_dir_walk( const char* config, int dtype, uint32_t first_layer, uint32_t n_hosted, uint32_t flags, const char* model_dir, uint64_t* records,
                              uint64_t max_records )
{
  const std::string name( config );
  uint64_t count = 0;
  auto sink = [&]( bool is_base, size_t layer, size_t k, const auto*, uint64_t n, uint64_t offset ) {
    if ( count < max_records && records != nullptr ) {
      uint64_t* r = records + 5 * count;
      r[0] = is_base ? 1 : 0;
      r[1] = layer;
      r[2] = k;
      r[3] = offset;
      r[4] = n;
    }
    count++;
  };
  bool known = false;
#define GLINT_CASE( NAME, CFG )                                                                                         \
  if ( name == NAME ) {                                                                                                 \
    known = true;                                                                                                       \
    const auto s = StageSettings<configs::CFG>::slice( first_layer, n_hosted, 1, 1, flags & 2u );                        \
    g_last_error = dtype == 0 ? walk_model_dir<configs::CFG, float16_t>( s, model_dir, sink ) : walk_model_dir<configs::CFG, float32_t>( s, model_dir, sink ); \
  }
  GLINT_CASE( "llama2-7b", Llama2_7B_Chat )
  GLINT_CASE( "stories15m", Stories_15M )
  GLINT_CASE( "test-gqa4", Test_GQA4 )
  GLINT_CASE( "test-mha", Test_MHA )
  GLINT_CASE( "test-tiny", Test_Tiny )
#undef GLINT_CASE
  if ( !known ) {
    g_last_error = "unknown configuration " + name;
  }
  return g_last_error.empty() ? (int64_t)count : -1;
}
void glint_stage_set_layer_tensor( void* h, uint32_t layer, uint32_t k, const void* host, uint64_t n ) { static_cast<StageBase*>( h )->set_layer_tensor( layer, k, host, n ); }
void glint_stage_set_base_tensor( void* h, uint32_t k, const void* host, uint64_t n ) { static_cast<StageBase*>( h )->set_base_tensor( k, host, n ); }
const void* glint_stage_layer_tensor_ptr( void* h, uint32_t layer, uint32_t k, uint64_t* n ) { return static_cast<StageBase*>( h )->layer_tensor_ptr( layer, k, n ); }
const void* glint_stage_base_tensor_ptr( void* h, uint32_t k, uint64_t* n ) { return static_cast<StageBase*>( h )->base_tensor_ptr( k, n ); }
void glint_stage_new_state( void* h, uint32_t batch, uint32_t next_layer, int next_stage ) { static_cast<StageBase*>( h )->new_state( batch, next_layer, next_stage ); }
void glint_stage_set_prompt( void* h, uint32_t row, uint32_t context_id, uint32_t token, uint32_t pos, float temperature, uint32_t prompt_length,
                             uint32_t max_completion_length )
{
  static_cast<StageBase*>( h )->set_prompt( row, context_id, token, pos, temperature, prompt_length, max_completion_length );
}
// rows [0, n) at once: one call per batch instead of one per row (a serving loop fills hundreds of rows per step)
void glint_stage_set_prompts( void* h, uint32_t n, const uint32_t* context_ids, const uint32_t* tokens, const uint32_t* positions, float temperature,
                              uint32_t prompt_length, uint32_t max_completion_length )
{
  auto* stage = static_cast<StageBase*>( h );
  for ( uint32_t i = 0; i < n; i++ ) {
    stage->set_prompt( i, context_ids[i], tokens[i], positions[i], temperature, prompt_length, max_completion_length );
  }
}
void glint_stage_discard( void* h, uint32_t row ) { static_cast<StageBase*>( h )->discard( row ); }
void glint_stage_set_next( void* h, uint32_t layer, int stage ) { static_cast<StageBase*>( h )->set_next( layer, stage ); }
int glint_stage_acquire_contexts( void* h ) { return static_cast<StageBase*>( h )->acquire_contexts(); }
int glint_stage_forward( void* h, int which ) { return static_cast<StageBase*>( h )->forward( which ); }
void* glint_stage_buffer( void* h, int which, uint64_t* bytes, int allocate ) { return static_cast<StageBase*>( h )->buffer( which, bytes, allocate != 0 ); }
void glint_stage_row_info( void* h, uint32_t row, uint32_t out[6] ) { static_cast<StageBase*>( h )->row_info( row, out ); }
void glint_stage_state_info( void* h, uint32_t out[4] ) { static_cast<StageBase*>( h )->state_info( out ); }
void* glint_stage_context_layer_ptr( void* h, uint32_t row, uint32_t layer ) { return static_cast<StageBase*>( h )->context_layer_ptr( row, layer ); }
int32_t glint_stage_context_slot( void* h, uint32_t row ) { return static_cast<StageBase*>( h )->context_slot( row ); }
void glint_stage_slot_counts( void* h, uint64_t out[3] ) { static_cast<StageBase*>( h )->slot_counts( out ); }
int glint_stage_release_context( void* h, uint32_t id ) { return static_cast<StageBase*>( h )->release_context( id ); }
void glint_stage_paging_info( void* h, uint32_t row, uint32_t layer, uint64_t out[3] ) { static_cast<StageBase*>( h )->paging_info( row, layer, out ); }
void* glint_stage_scratch( void* h, int which ) { return static_cast<StageBase*>( h )->scratch( which ); }
void glint_stage_sync( void* h ) { static_cast<StageBase*>( h )->sync(); }
void glint_stage_copy_bytes( void* h, void* dst, const void* src, uint64_t bytes, int kind ) { static_cast<StageBase*>( h )->copy_bytes( dst, src, bytes, kind ); }
// device time of forward() without the copies over the host boundary: on / off, then total milliseconds and steps since the last read
void glint_stage_time_device_spans( void* h, int on ) { static_cast<StageBase*>( h )->time_device_spans( on != 0 ); }
void glint_stage_device_spans( void* h, double* ms, uint64_t* spans ) { static_cast<StageBase*>( h )->device_spans( ms, spans ); }
// batched prefill of n_tokens tokens per context; -1 when the contexts cannot be served
int glint_stage_prefill( void* h, uint32_t batch, const uint32_t* context_ids, const uint32_t* start_pos, uint32_t n_tokens, uint32_t first_layer,
                         const uint32_t* token_ids, const void* acts_in, void* acts_out, uint32_t* next_tokens )
{
  return static_cast<StageBase*>( h )->prefill( batch, context_ids, start_pos, n_tokens, first_layer, token_ids, acts_in, acts_out, next_tokens );
}

// ---- host-only bookkeeping hooks ---------------------------------------------------------------
void* glint_book_manager_new( uint64_t max_context_count ) { return new BookManager( max_context_count ); }
void glint_book_manager_delete( void* m ) { delete static_cast<BookManager*>( m ); }
uint64_t glint_book_manager_free( void* m ) { return static_cast<BookManager*>( m )->man.free(); }
uint64_t glint_book_manager_allocated( void* m ) { return static_cast<BookManager*>( m )->man.allocated(); }

// rows [start, end) of a state described by active[] / context_id[]; slots_out gets creation indices (-1 = empty context)
int glint_book_manager_get_contexts( void* m, const uint8_t* active, const uint32_t* context_id, uint64_t batch, uint64_t start, uint64_t end, int32_t* slots_out )
{
  auto& man = static_cast<BookManager*>( m )->man;
  BatchedInferenceState<BookConfig> st( static_cast<uint32_t>( batch ), DataType::Float16 );
  for ( uint64_t i = 0; i < batch; i++ ) {
    if ( active[i] ) {
      st.set_prompt( i, context_id[i], 1, 0, 0.0f, 1, 0 );
    } else {
      st.set_context_id( i, context_id[i] );
    }
  }
  auto got = man.get_contexts( st, start, end );
  if ( !got.has_value() ) {
    return 0;
  }
  for ( size_t k = 0; k < got->size(); k++ ) {
    slots_out[k] = man.slot_index( ( *got )[k] );
  }
  return 1;
}

int32_t glint_book_manager_get_context( void* m, uint32_t context_id )
{
  auto& man = static_cast<BookManager*>( m )->man;
  auto ctx = man.get_context( context_id );
  return ctx ? man.slot_index( ctx ) : -1;
}

int glint_book_manager_release( void* m, uint32_t context_id ) { return static_cast<BookManager*>( m )->man.release_context( context_id ) ? 1 : 0; }

// paged context over a counting region: hosts `n_hosted` layers of the 70B-4K shape
void* glint_book_paged_new( uint32_t n_hosted ) { return new PagedBookContext( StageSettings<BookConfig>::slice( 0, n_hosted, 1, 1 ) ); }
void glint_book_paged_delete( void* c ) { delete static_cast<PagedBookContext*>( c ); }
// returns the committed bytes of `layer` after the call; out[0] = blocks committed so far, out[1] = clears so far
uint64_t glint_book_paged_prepare( void* c, uint32_t layer, uint32_t token_pos, int can_release, uint64_t out[2] )
{
  auto* ctx = static_cast<PagedBookContext*>( c );
  GLINT_CHECK( ctx->prepare( layer, token_pos, can_release != 0 ) );
  out[0] = ctx->blocks_committed();
  out[1] = ctx->clears();
  return ctx->allocated_bytes( layer );
}

// KV addressing of the host layer, in elements from the context base (UINT64_MAX: layer not hosted)
uint64_t glint_book_key_head_offset( const uint8_t* hosted, uint32_t layer, uint32_t pos, uint32_t head, int value )
{
  StageSettings<BookConfig>::HostingTable t {};
  for ( size_t l = 0; l < BookConfig::n_layers; l++ ) {
    t[l][static_cast<size_t>( InferenceStage::Attention )] = hosted[l] != 0;
    t[l][0] = t[l][0] || hosted[l] != 0;
  }
  bool any = false;
  for ( size_t l = 0; l < BookConfig::n_layers; l++ ) {
    any = any || hosted[l];
  }
  if ( !any ) {
    return UINT64_MAX;
  }
  StageSettings<BookConfig> s( t, 1, 1 );
  auto* base = reinterpret_cast<float16_t*>( uintptr_t { 1 } << 40 );
  glint::Context<BookConfig, float16_t> ctx( s, base );
  auto lc = ctx.layer( layer );
  if ( lc.empty() ) {
    return UINT64_MAX;
  }
  auto tc = lc.token( pos );
  return static_cast<uint64_t>( ( value ? tc.value_head( head ) : tc.key_head( head ) ) - base );
}

// ---- stage state on the wire --------------------------------------------------------------------
int glint_stage_set_state_bytes( void* h, const void* bytes, uint64_t len )
{
  g_last_error = static_cast<StageBase*>( h )->set_state_bytes( bytes, len );
  return g_last_error.empty() ? 0 : -1;
}
// the serialized state stays valid until the next call on this thread
const void* glint_stage_get_state_bytes( void* h, uint64_t* len )
{
  g_bytes = static_cast<StageBase*>( h )->get_state_bytes();
  *len = g_bytes.size();
  return g_bytes.data();
}

// ---- host-only states (shape of "test-tiny": dim 32, kv_dim 16) -----------------------------------
void* glint_state_new( uint32_t batch, int dtype, uint32_t route_id, uint32_t model_id )
{
  return new BookState( batch, dtype == 0 ? DataType::Float16 : DataType::Float32, route_id, model_id );
}
void* glint_state_parse( const void* bytes, uint64_t len )
{
  auto* s = new BookState();
  if ( !BookState::parse( std::string_view( static_cast<const char*>( bytes ), len ), *s, &g_last_error ) ) {
    delete s;
    return nullptr;
  }
  return s;
}
void glint_state_delete( void* h ) { delete as_state( h ); }
const void* glint_state_serialize( void* h, uint64_t* len )
{
  g_bytes = as_state( h )->serialize();
  *len = g_bytes.size();
  return g_bytes.data();
}
void glint_state_set_meta( void* h, uint64_t id, uint32_t next_layer, int next_stage, int next_tier, uint32_t next_rank, int is_sharded )
{
  auto* s = as_state( h );
  s->set_id( id );
  s->set_next_layer( next_layer );
  s->set_next_stage( static_cast<InferenceStage>( next_stage ) );
  s->set_next_tier( (int8_t)next_tier );
  s->set_next_rank( (uint8_t)next_rank );
  s->set_is_sharded( is_sharded != 0 );
}
void glint_state_set_prompt( void* h, uint32_t i, const uint8_t prompt_id[32], uint32_t context_id, uint32_t token, uint32_t token_pos, float temperature,
                             uint32_t prompt_length, uint32_t max_completion_length, int kv_tier, uint32_t kv_rank )
{
  PromptID id;
  std::memcpy( id.hash.data(), prompt_id, 32 );
  as_state( h )->set_prompt( i, id, context_id, token, token_pos, temperature, prompt_length, max_completion_length, (int8_t)kv_tier, (uint8_t)kv_rank );
}
void glint_state_discard( void* h, uint32_t i ) { as_state( h )->discard( i ); }
void glint_state_set_finished( void* h, uint32_t i ) { as_state( h )->set_finished( i ); }
int glint_state_check_finished( void* h, uint32_t i ) { return as_state( h )->check_finished( i ) ? 1 : 0; }
// host-only: the stage driver's position check (positions_fit) on this state, with a slot for every active row and the shared empty
// context for the others, as the context manager hands them out
int glint_state_positions_fit( void* h, uint64_t seq_len )
{
  const auto settings = StageSettings<configs::Test_Tiny>::slice( 0, 1, 1024, 1024 );
  std::vector<std::shared_ptr<EchoContext>> contexts;
  for ( size_t i = 0; i < as_state( h )->batch_size(); i++ ) {
    contexts.push_back( std::make_shared<EchoContext>( settings, !as_state( h )->active( i ) ) );
  }
  return positions_fit( *as_state( h ), contexts, seq_len ) ? 1 : 0;
}
uint64_t glint_state_free_slots( void* h ) { return as_state( h )->free_slots(); }
uint32_t glint_state_batch_size( void* h ) { return as_state( h )->batch_size(); }
int glint_state_all_assigned( void* h ) { return as_state( h )->all_assigned_to_nodes() ? 1 : 0; }
// which: 0 activations, 1 queries, 2 kvs; allocates when asked to and absent; *bytes = 0 when absent
void* glint_state_buffer( void* h, int which, uint64_t* bytes, int allocate )
{
  auto* s = as_state( h );
  DataBuffer* b = which == 0 ? &s->activations() : which == 1 ? &s->queries() : &s->kvs();
  const bool present = which == 0 ? s->has_activations() : which == 1 ? s->has_queries() : s->has_kvs();
  if ( allocate && !present ) {
    if ( which == 0 ) {
      s->allocate_activations();
    } else if ( which == 1 ) {
      s->allocate_queries();
    } else {
      s->allocate_kvs();
    }
  }
  *bytes = b->len();
  return b->data();
}
int glint_state_replenish_from( void* h, void* other ) { return as_state( h )->replenish_from( *as_state( other ) ) ? 1 : 0; }
void glint_state_merge( void* h, void* other ) { as_state( h )->merge( std::move( *as_state( other ) ) ); }
// rows [0, n) and [n, batch) as two new states
void glint_state_split( void* h, uint64_t n, void** first, void** second )
{
  auto [a, b] = as_state( h )->split( n );
  *first = new BookState( std::move( a ) );
  *second = new BookState( std::move( b ) );
}
// splits `h` (left empty) by kv placement; up to `cap` new states in `out`, returns how many pieces there are
uint64_t glint_state_split_on_kv( void* h, void** out, uint64_t cap )
{
  auto pieces = BookState::split_on_kv( std::move( *as_state( h ) ) );
  const uint64_t n = pieces.size();
  for ( uint64_t i = 0; i < n && i < cap; i++ ) {
    out[i] = new BookState( std::move( pieces[i] ) );
  }
  return n;
}

// ---- compute kernel -----------------------------------------------------------------------------
// same arguments as glint_stage_create; the model sits behind push / pop / eventfd on two threads
void* glint_kernel_create( const char* config, int dtype, uint32_t first_layer, uint32_t n_hosted, uint32_t concurrency, uint32_t max_contexts, uint32_t flags,
                           uint64_t seed, float weight_std )
{
  const std::string name( config );
  ModelOptions o;
  o.fused_attention = flags & 1u;
  o.fused_projections = !( flags & 8u );
  o.balanced_attention = ( flags & 16u ) ? 1 : ( ( flags & 32u ) ? -1 : 0 );
  o.seed = seed;
  o.weight_std = weight_std;
  const bool with_cls = flags & 2u;
#define GLINT_CASE( NAME, CFG )                                                                                              \
  if ( name == NAME ) {                                                                                                      \
    const auto s = StageSettings<configs::CFG>::slice( first_layer, n_hosted, concurrency, max_contexts, with_cls );           \
    if ( dtype == 0 ) {                                                                                                      \
      using M = Llama2<configs::CFG, float16_t, hip::LlamaOperations<configs::CFG, float16_t>, hip::Context<configs::CFG, float16_t>>; \
      return static_cast<KernelBase*>( new KernelImpl<M>( s, o ) );                                                           \
    }                                                                                                                        \
    using M = Llama2<configs::CFG, float32_t, hip::LlamaOperations<configs::CFG, float32_t>, hip::Context<configs::CFG, float32_t>>; \
    return static_cast<KernelBase*>( new KernelImpl<M>( s, o ) );                                                             \
  }
  GLINT_CASE( "llama2-70b-4k", Llama2_70B_Chat_4K )
  GLINT_CASE( "llama2-7b", Llama2_7B_Chat )
  GLINT_CASE( "stories15m", Stories_15M )
  GLINT_CASE( "test-gqa4", Test_GQA4 )
  GLINT_CASE( "test-tiny", Test_Tiny )
#undef GLINT_CASE
  return nullptr;
}
// host-only kernel around a model that just advances tokens (shape of "test-tiny")
void* glint_kernel_create_echo( uint32_t concurrency, uint32_t max_contexts )
{
  return static_cast<KernelBase*>( new KernelImpl<EchoModel>( StageSettings<configs::Test_Tiny>::slice( 0, 2, concurrency, max_contexts ) ) );
}
void glint_kernel_destroy( void* h ) { delete static_cast<KernelBase*>( h ); }
int glint_kernel_load( void* h, const char* model_dir )
{
  g_last_error = static_cast<KernelBase*>( h )->load_dir( model_dir );
  return g_last_error.empty() ? 0 : -1;
}
int glint_kernel_push( void* h, const void* bytes, uint64_t len )
{
  g_last_error = static_cast<KernelBase*>( h )->push_bytes( bytes, len );
  return g_last_error.empty() ? 0 : -1;
}
// NULL when nothing has finished; otherwise the serialized state, valid until the next call on this thread
const void* glint_kernel_pop( void* h, uint64_t* len )
{
  if ( !static_cast<KernelBase*>( h )->pop_bytes( g_bytes ) ) {
    *len = 0;
    return nullptr;
  }
  *len = g_bytes.size();
  return g_bytes.data();
}
int glint_kernel_event_fd( void* h ) { return static_cast<KernelBase*>( h )->event_fd().fd_num(); }
// 1 and the number of states finished since the last read, or 0 when none
int glint_kernel_read_event( void* h, uint64_t* count ) { return static_cast<KernelBase*>( h )->event_fd().read_event( count ) ? 1 : 0; }
void glint_kernel_slot_counts( void* h, uint64_t out[3] ) { static_cast<KernelBase*>( h )->slot_counts( out ); }

} // extern "C"
