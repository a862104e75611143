// The reference's BatchedInferenceState (models/common/state.hh): the batch metadata and per-prompt
// fields the model driver reads and writes, the three host buffers (activations, queries, kvs), and
// what the stages around this one do with a state -- the wire format (state.hh:512-594), refill of
// finished slots (replenish_from, :696-752), splitting by kv placement and merging (:760-1050).
//
// Wire format, all fields packed, host byte order (the reference memcpy's its packed structs):
//
//   StateMetadata  32 bytes  id u64 | batch_size u32 | dtype u8 | route_id u32 | model_id u32 |
//                            next_layer u32 | next_stage u8 | next_tier i8 | next_rank u8 |
//                            has_activations u8 | has_queries u8 | has_kvs u8 | is_sharded u8
//   PromptData     57 bytes  active u8 | prompt_id 32 B | context_id u32 | token u32 | token_pos u32 |
//                  x batch   temperature u8 | prompt_length u32 | max_completion_length u32 |
//                            finished u8 | kv_tier i8 | kv_rank u8
//   activations    batch x dim x sizeof(dtype)        if has_activations
//   queries        batch x dim x sizeof(dtype)        if has_queries
//   kvs            batch x 2 kv_dim x sizeof(dtype)   if has_kvs
//
// The reference only DCHECKs the length of what it parses (a release build reads past a short
// buffer); parse() here refuses short, long and inconsistent input and says why.
#pragma once

#include <algorithm>
#include <array>
#include <cstdint>
#include <cstring>
#include <cstdlib>
#include <deque>
#include <map>
#include <mutex>
#include <sstream>
#include <string>
#include <string_view>
#include <utility>
#include <vector>

#include "glint/config.hh"
#include "glint/types.hh"

namespace glint {

// util/digest.hh:15-18: 32 raw bytes
struct __attribute__( ( packed ) ) PromptID
{
  std::array<uint8_t, 32> hash {};
  bool operator==( const PromptID& other ) const { return hash == other.hash; }
};

using RouteID = uint32_t; // models/types.hh:15-16
using ModelID = uint32_t;
constexpr ContextID NULL_CONTEXT {};

struct __attribute__( ( packed ) ) StateMetadata // models/common/state.hh:17-34
{
  uint64_t id {};
  uint32_t batch_size {};
  DataType dtype { DataType::Float32 };
  RouteID route_id {};
  ModelID model_id {};
  uint32_t next_layer { 0 };
  InferenceStage next_stage { InferenceStage::PreAttention };
  int8_t next_tier { 0 };
  uint8_t next_rank { 0 };
  bool has_activations { false };
  bool has_queries { false };
  bool has_kvs { false };
  bool is_sharded { false };
};

struct __attribute__( ( packed ) ) PromptData // models/common/state.hh:36-50
{
  bool active { false };
  PromptID prompt_id {};
  ContextID context_id {};
  uint32_t token {};
  uint32_t token_pos {};
  uint8_t temperature {}; // compact: value / 255.0f
  uint32_t prompt_length {};
  uint32_t max_completion_length {};
  bool finished { false };
  int8_t kv_tier { -1 }; // which tier holds this prompt's kv cache, -1 = unassigned
  uint8_t kv_rank { 0 };
};

static_assert( sizeof( StateMetadata ) == 32 );
static_assert( sizeof( PromptData ) == 57 );

// Host memory for the state buffers.  Freed buffers are kept by size and handed out again
// (models/types.hh:58-76 has the same idea): a stage allocates the same few sizes every step.  The
// memory comes from `malloc` unless a backend installs page-locked allocation with set_source()
// (the hip target does, once the device is up: the activations then reach the GPU without a
// staging copy).  Buffers are recycled only while the source that made them is still installed.
class HostBufferPool
{
public:
  using AllocFn = void* (*)( size_t );
  using FreeFn = void ( * )( void* );

  static HostBufferPool& instance()
  {
    // never destroyed: buffers may be returned during static destruction, and page-locked memory
    // must not be freed after the device runtime has shut down
    static HostBufferPool* pool = new HostBufferPool;
    return *pool;
  }

  void set_source( AllocFn alloc, FreeFn free )
  {
    std::lock_guard<std::mutex> lock( mutex_ );
    drop_unused();
    alloc_ = alloc;
    free_ = free;
    generation_++;
  }

  struct Block
  {
    uint8_t* ptr { nullptr };
    FreeFn free { nullptr };
    uint64_t generation { 0 };
  };

  Block get( const size_t n )
  {
    if ( n == 0 ) {
      return {};
    }
    std::lock_guard<std::mutex> lock( mutex_ );
    auto it = unused_.find( n );
    if ( it != unused_.end() && !it->second.empty() ) {
      Block b = it->second.back();
      it->second.pop_back();
      reused_++;
      return b;
    }
    void* p = alloc_( n );
    if ( p == nullptr ) {
      fatal( __FILE__, __LINE__, "HostBufferPool: out of host memory" );
    }
    return { static_cast<uint8_t*>( p ), free_, generation_ };
  }

  void put( const Block b, const size_t n )
  {
    if ( b.ptr == nullptr ) {
      return;
    }
    std::lock_guard<std::mutex> lock( mutex_ );
    if ( b.generation == generation_ && n >= MIN_POOLED ) {
      unused_[n].push_back( b );
    } else {
      b.free( b.ptr );
    }
  }

  uint64_t reused() const { return reused_; }

private:
  static constexpr size_t MIN_POOLED = 4096; // smaller buffers are cheap to allocate

  HostBufferPool() = default;
  void drop_unused()
  {
    for ( auto& [n, blocks] : unused_ ) {
      for ( auto& b : blocks ) {
        b.free( b.ptr );
      }
    }
    unused_.clear();
  }

  std::mutex mutex_ {};
  AllocFn alloc_ { &std::malloc };
  FreeFn free_ { &std::free };
  uint64_t generation_ { 0 };
  std::map<size_t, std::vector<Block>> unused_ {};
  uint64_t reused_ { 0 };
};

// host buffer with the DataBuffer surface the driver uses (models/types.hh:78-125); zero-filled when made
class DataBuffer
{
  HostBufferPool::Block block_ {};
  uint64_t len_ { 0 };

public:
  DataBuffer() = default;
  explicit DataBuffer( size_t n )
    : block_( HostBufferPool::instance().get( n ) )
    , len_( n )
  {
    if ( n > 0 ) {
      std::memset( block_.ptr, 0, n );
    }
  }
  DataBuffer( const DataBuffer& ) = delete;
  DataBuffer& operator=( const DataBuffer& ) = delete;
  DataBuffer( DataBuffer&& other ) noexcept
    : block_( other.block_ )
    , len_( other.len_ )
  {
    other.block_ = {};
    other.len_ = 0;
  }
  DataBuffer& operator=( DataBuffer&& other ) noexcept
  {
    if ( this != &other ) {
      HostBufferPool::instance().put( block_, len_ );
      block_ = other.block_;
      len_ = other.len_;
      other.block_ = {};
      other.len_ = 0;
    }
    return *this;
  }
  ~DataBuffer() { HostBufferPool::instance().put( block_, len_ ); }

  uint64_t len() const { return len_; }
  uint8_t* data() { return block_.ptr; }
  const uint8_t* data() const { return block_.ptr; }
};

template<typename Config>
requires ModelConfig<Config>
class BatchedInferenceState
{
  StateMetadata metadata_ {};
  std::vector<PromptData> prompts_ {};
  DataBuffer activations_ {}, queries_ {}, kvs_ {};

  size_t activation_len() const { return Config::dim * DataTypeSize( metadata_.dtype ); }
  size_t q_len() const { return Config::dim * DataTypeSize( metadata_.dtype ); }
  size_t kv_len() const { return 2 * Config::kv_dim * DataTypeSize( metadata_.dtype ); }

  // rows [first, first + n) of `from` become rows [at, at + n) of this state's buffers
  void copy_rows( size_t at, const BatchedInferenceState& from, size_t first, size_t n )
  {
    if ( n == 0 ) {
      return; // nothing to move; an empty buffer's null pointer must not reach memcpy
    }
    if ( metadata_.has_activations ) {
      std::memcpy( activations_.data() + at * activation_len(), from.activations_.data() + first * activation_len(), n * activation_len() );
    }
    if ( metadata_.has_queries ) {
      std::memcpy( queries_.data() + at * q_len(), from.queries_.data() + first * q_len(), n * q_len() );
    }
    if ( metadata_.has_kvs ) {
      std::memcpy( kvs_.data() + at * kv_len(), from.kvs_.data() + first * kv_len(), n * kv_len() );
    }
  }

  // a state of `n` rows with this state's metadata and allocated buffers, prompts default
  BatchedInferenceState like_this( size_t n ) const
  {
    BatchedInferenceState s;
    s.metadata_ = metadata_;
    s.metadata_.batch_size = static_cast<uint32_t>( n );
    s.prompts_.resize( n );
    if ( metadata_.has_activations ) {
      s.allocate_activations();
    }
    if ( metadata_.has_queries ) {
      s.allocate_queries();
    }
    if ( metadata_.has_kvs ) {
      s.allocate_kvs();
    }
    return s;
  }

public:
  using ConfigType = Config;

  BatchedInferenceState() = default;
  BatchedInferenceState( uint32_t batch_size, DataType dtype, RouteID route_id = {}, ModelID model_id = {} )
    : prompts_( batch_size )
  {
    metadata_.batch_size = batch_size;
    metadata_.dtype = dtype;
    metadata_.route_id = route_id;
    metadata_.model_id = model_id;
  }

  // movable, not copyable (the buffers are large)
  BatchedInferenceState( const BatchedInferenceState& ) = delete;
  BatchedInferenceState& operator=( const BatchedInferenceState& ) = delete;
  // a moved-from state is an empty state (batch size 0), not one whose metadata still names rows it no longer has
  BatchedInferenceState( BatchedInferenceState&& other ) noexcept { *this = std::move( other ); }
  BatchedInferenceState& operator=( BatchedInferenceState&& other ) noexcept
  {
    if ( this != &other ) {
      metadata_ = other.metadata_;
      prompts_ = std::move( other.prompts_ );
      activations_ = std::move( other.activations_ );
      queries_ = std::move( other.queries_ );
      kvs_ = std::move( other.kvs_ );
      other.metadata_ = StateMetadata {};
      other.prompts_.clear();
      other.activations_ = DataBuffer {};
      other.queries_ = DataBuffer {};
      other.kvs_ = DataBuffer {};
    }
    return *this;
  }

  // ---- wire format ---------------------------------------------------------------------------
  static size_t wire_size( const StateMetadata& m )
  {
    const size_t elem = DataTypeSize( m.dtype );
    return sizeof( StateMetadata ) + sizeof( PromptData ) * (size_t)m.batch_size + ( m.has_activations ? (size_t)m.batch_size * Config::dim * elem : 0 )
           + ( m.has_queries ? (size_t)m.batch_size * Config::dim * elem : 0 ) + ( m.has_kvs ? (size_t)m.batch_size * 2 * Config::kv_dim * elem : 0 );
  }

  // false (and the reason in *why) unless `bytes` is exactly one serialized state of this model
  static bool parse( const std::string_view bytes, BatchedInferenceState& out, std::string* why = nullptr )
  {
    auto refuse = [&]( const char* msg ) {
      if ( why != nullptr ) {
        *why = msg;
      }
      return false;
    };
    if ( bytes.size() < sizeof( StateMetadata ) ) {
      return refuse( "serialized state is too small to contain metadata" );
    }
    StateMetadata m;
    std::memcpy( &m, bytes.data(), sizeof( m ) );
    if ( static_cast<uint8_t>( m.dtype ) > static_cast<uint8_t>( DataType::BFloat16 ) ) {
      return refuse( "serialized state has an unknown data type" );
    }
    if ( static_cast<uint8_t>( m.next_stage ) >= static_cast<uint8_t>( InferenceStage::__COUNT__ ) ) {
      return refuse( "serialized state has an unknown next stage" );
    }
    const size_t need = wire_size( m );
    if ( bytes.size() < need ) {
      return refuse( "serialized state is too small for its batch size and buffers" );
    }
    if ( bytes.size() > need ) {
      return refuse( "serialized state contains more data than expected" );
    }
    BatchedInferenceState s;
    s.metadata_ = m;
    s.prompts_.resize( m.batch_size );
    const char* p = bytes.data() + sizeof( m );
    if ( m.batch_size > 0 ) { // an empty vector has no storage: a null pointer must not reach memcpy, even with a length of zero
      std::memcpy( reinterpret_cast<char*>( s.prompts_.data() ), p, sizeof( PromptData ) * (size_t)m.batch_size );
    }
    p += sizeof( PromptData ) * (size_t)m.batch_size;
    auto take = [&]( DataBuffer& buf, size_t n ) {
      buf = DataBuffer( n );
      if ( n > 0 ) {
        std::memcpy( buf.data(), p, n );
      }
      p += n;
    };
    if ( m.has_activations ) {
      take( s.activations_, m.batch_size * s.activation_len() );
    }
    if ( m.has_queries ) {
      take( s.queries_, m.batch_size * s.q_len() );
    }
    if ( m.has_kvs ) {
      take( s.kvs_, m.batch_size * s.kv_len() );
    }
    out = std::move( s );
    return true;
  }

  // the reference's deserializing constructor; malformed input aborts
  explicit BatchedInferenceState( const std::string_view serialized_state )
  {
    std::string why;
    if ( !parse( serialized_state, *this, &why ) ) {
      fatal( __FILE__, __LINE__, "BatchedInferenceState:", why.c_str() );
    }
  }

  std::string serialize() const
  {
    std::string out;
    out.reserve( wire_size( metadata_ ) );
    out.append( reinterpret_cast<const char*>( &metadata_ ), sizeof( StateMetadata ) );
    out.append( reinterpret_cast<const char*>( prompts_.data() ), sizeof( PromptData ) * (size_t)metadata_.batch_size );
    if ( metadata_.has_activations ) {
      out.append( reinterpret_cast<const char*>( activations_.data() ), metadata_.batch_size * activation_len() );
    }
    if ( metadata_.has_queries ) {
      out.append( reinterpret_cast<const char*>( queries_.data() ), metadata_.batch_size * q_len() );
    }
    if ( metadata_.has_kvs ) {
      out.append( reinterpret_cast<const char*>( kvs_.data() ), metadata_.batch_size * kv_len() );
    }
    GLINT_CHECK( out.size() == wire_size( metadata_ ) );
    return out;
  }

  // ---- metadata ------------------------------------------------------------------------------
  bool empty() const { return metadata_.batch_size == 0; }
  uint64_t id() const { return metadata_.id; }
  uint32_t batch_size() const { return metadata_.batch_size; }
  DataType dtype() const { return metadata_.dtype; }
  RouteID route_id() const { return metadata_.route_id; }
  ModelID model_id() const { return metadata_.model_id; }
  uint32_t next_layer() const { return metadata_.next_layer; }
  InferenceStage next_stage() const { return metadata_.next_stage; }
  int8_t next_tier() const { return metadata_.next_tier; }
  uint8_t next_rank() const { return metadata_.next_rank; }
  bool has_activations() const { return metadata_.has_activations; }
  bool has_queries() const { return metadata_.has_queries; }
  bool has_kvs() const { return metadata_.has_kvs; }
  bool is_sharded() const { return metadata_.is_sharded; }
  bool all_assigned_to_nodes() const
  {
    return std::all_of( prompts_.begin(), prompts_.end(), []( const PromptData& p ) { return p.kv_tier != -1; } );
  }

  void set_id( uint64_t id ) { metadata_.id = id; }
  void set_dtype( DataType dtype ) { metadata_.dtype = dtype; }
  void set_route_id( RouteID id ) { metadata_.route_id = id; }
  void set_model_id( ModelID id ) { metadata_.model_id = id; }
  void set_next_layer( uint32_t l ) { metadata_.next_layer = l; }
  void set_next_stage( InferenceStage s ) { metadata_.next_stage = s; }
  void set_next_tier( int8_t t ) { metadata_.next_tier = t; }
  void set_next_rank( uint8_t r ) { metadata_.next_rank = r; }
  void set_has_activations( bool v ) { metadata_.has_activations = v; }
  void set_has_queries( bool v ) { metadata_.has_queries = v; }
  void set_has_kvs( bool v ) { metadata_.has_kvs = v; }
  void set_is_sharded( bool v ) { metadata_.is_sharded = v; }

  // ---- prompts -------------------------------------------------------------------------------
  void set_prompt( size_t i, PromptID prompt_id, ContextID context_id, uint32_t token, uint32_t token_pos, float temperature, uint32_t prompt_length,
                   uint32_t max_completion_length, int8_t kv_tier, uint8_t kv_rank )
  {
    PromptData p;
    p.prompt_id = prompt_id;
    p.context_id = context_id;
    p.token = token;
    p.token_pos = token_pos;
    p.temperature = static_cast<uint8_t>( temperature * 255.0f );
    p.prompt_length = prompt_length;
    p.max_completion_length = max_completion_length;
    p.finished = false;
    p.active = true;
    p.kv_tier = kv_tier;
    p.kv_rank = kv_rank;
    prompts_[i] = p;
  }
  // same without a prompt id (a single stage has no use for it)
  void set_prompt( size_t i, ContextID context_id, uint32_t token, uint32_t token_pos, float temperature, uint32_t prompt_length,
                   uint32_t max_completion_length, int8_t kv_tier = 0, uint8_t kv_rank = 0 )
  {
    set_prompt( i, PromptID {}, context_id, token, token_pos, temperature, prompt_length, max_completion_length, kv_tier, kv_rank );
  }

  PromptID prompt_id( size_t i ) const { return prompts_[i].prompt_id; }
  ContextID context_id( size_t i ) const { return prompts_[i].context_id; }
  uint32_t token( size_t i ) const { return prompts_[i].token; }
  uint32_t token_pos( size_t i ) const { return prompts_[i].token_pos; }
  uint32_t prompt_length( size_t i ) const { return prompts_[i].prompt_length; }
  uint32_t max_completion_length( size_t i ) const { return prompts_[i].max_completion_length; }
  float temperature( size_t i ) const { return prompts_[i].temperature / 255.0f; }
  bool finished( size_t i ) const { return prompts_[i].finished; }
  int8_t kv_tier( size_t i ) const { return prompts_[i].kv_tier; }
  uint8_t kv_rank( size_t i ) const { return prompts_[i].kv_rank; }
  bool assigned_to_node( size_t i ) const { return prompts_[i].kv_tier != -1; }
  bool active( size_t i ) const { return prompts_[i].active; }
  const PromptData& prompt( size_t i ) const { return prompts_[i]; }

  void set_prompt_id( size_t i, PromptID id ) { prompts_[i].prompt_id = id; }
  void set_context_id( size_t i, ContextID id ) { prompts_[i].context_id = id; }
  void set_token( size_t i, uint32_t token ) { prompts_[i].token = token; }
  void set_token_pos( size_t i, uint32_t pos ) { prompts_[i].token_pos = pos; }
  void set_prompt_length( size_t i, uint32_t n ) { prompts_[i].prompt_length = n; }
  void set_max_completion_length( size_t i, uint32_t n ) { prompts_[i].max_completion_length = n; }
  void set_temperature( size_t i, float t ) { prompts_[i].temperature = static_cast<uint8_t>( t * 255.0f ); }
  void set_finished( size_t i ) { prompts_[i].finished = true; }
  void set_kv_tier( size_t i, int8_t t ) { prompts_[i].kv_tier = t; }
  void set_kv_rank( size_t i, uint8_t r ) { prompts_[i].kv_rank = r; }

  // keeps the slot's context id and placement so that a refill inherits the same context
  void discard( size_t i )
  {
    PromptData p;
    p.context_id = prompts_[i].context_id;
    p.kv_tier = prompts_[i].kv_tier;
    p.kv_rank = prompts_[i].kv_rank;
    p.active = false;
    prompts_[i] = p;
  }

  bool check_finished( size_t i ) const
  {
    const PromptData p = prompts_[i];
    const bool saw_end = p.max_completion_length == 0 && ( p.token == Config::token_eos || p.token == Config::token_eot );
    const bool out_of_seq = p.token_pos >= Config::seq_len;
    const bool end_of_gen = p.max_completion_length > 0 && p.token_pos >= p.max_completion_length + p.prompt_length;
    return saw_end || out_of_seq || end_of_gen;
  }

  size_t free_slots() const
  {
    return (size_t)std::count_if( prompts_.begin(), prompts_.end(), []( const PromptData& p ) { return !p.active; } );
  }

  // ---- buffers -------------------------------------------------------------------------------
  DataBuffer& activations() { return activations_; }
  DataBuffer& queries() { return queries_; }
  DataBuffer& kvs() { return kvs_; }
  const DataBuffer& activations() const { return activations_; }
  const DataBuffer& queries() const { return queries_; }
  const DataBuffer& kvs() const { return kvs_; }
  uint8_t* activations( size_t i ) { return activations_.data() + i * activation_len(); }
  uint8_t* q( size_t i ) { return queries_.data() + i * q_len(); }
  uint8_t* kv( size_t i ) { return kvs_.data() + i * kv_len(); }
  const uint8_t* kv( size_t i ) const { return kvs_.data() + i * kv_len(); }

  void allocate_activations()
  {
    activations_ = DataBuffer( metadata_.batch_size * activation_len() );
    metadata_.has_activations = true;
  }
  void allocate_queries()
  {
    queries_ = DataBuffer( metadata_.batch_size * q_len() );
    metadata_.has_queries = true;
  }
  void allocate_kvs()
  {
    kvs_ = DataBuffer( metadata_.batch_size * kv_len() );
    metadata_.has_kvs = true;
  }
  void deallocate_activations()
  {
    activations_ = {};
    metadata_.has_activations = false;
  }
  void deallocate_queries()
  {
    queries_ = {};
    metadata_.has_queries = false;
  }
  void deallocate_kvs()
  {
    kvs_ = {};
    metadata_.has_kvs = false;
  }

  // ---- refill, split, merge ------------------------------------------------------------------
  // Every inactive row of this state takes over, in order, the next active row of `other` (prompt
  // fields and buffer rows) but keeps its own context id; the donor row is cleared.  False when
  // `other` runs out of active rows first.  (models/common/state.hh:696-752)
  bool replenish_from( BatchedInferenceState& other )
  {
    GLINT_CHECK( metadata_.batch_size == other.metadata_.batch_size && metadata_.dtype == other.metadata_.dtype );
    GLINT_CHECK( metadata_.has_activations == other.metadata_.has_activations && metadata_.has_queries == other.metadata_.has_queries
                 && metadata_.has_kvs == other.metadata_.has_kvs );
    size_t other_idx = 0;
    for ( size_t my_idx = 0; my_idx < prompts_.size(); my_idx++ ) {
      if ( prompts_[my_idx].active ) {
        continue;
      }
      while ( other_idx < other.prompts_.size() && !other.prompts_[other_idx].active ) {
        other_idx++;
      }
      if ( other_idx >= other.prompts_.size() ) {
        return false; // no more active prompts in the other state
      }
      const ContextID mine = prompts_[my_idx].context_id;
      prompts_[my_idx] = other.prompts_[other_idx];
      prompts_[my_idx].context_id = mine;
      copy_rows( my_idx, other, other_idx, 1 );
      other.prompts_[other_idx] = PromptData {};
      other_idx++;
    }
    return true;
  }

  // consecutive pieces of the given sizes (which must add up to the batch); `state` is left empty
  static std::deque<BatchedInferenceState> split_states( BatchedInferenceState&& state, const std::vector<size_t>& sizes, bool ignore_empty )
  {
    GLINT_CHECK( !sizes.empty() );
    size_t sum = 0;
    for ( size_t n : sizes ) {
      sum += n;
    }
    GLINT_CHECK( sum == state.metadata_.batch_size );
    std::deque<BatchedInferenceState> pieces;
    if ( sizes.size() == 1 ) {
      pieces.push_back( std::move( state ) );
      return pieces;
    }
    size_t first = 0;
    for ( size_t n : sizes ) {
      if ( n == 0 && ignore_empty ) {
        continue;
      }
      BatchedInferenceState piece = state.like_this( n );
      std::copy( state.prompts_.begin() + first, state.prompts_.begin() + first + n, piece.prompts_.begin() );
      piece.copy_rows( 0, state, first, n );
      first += n;
      pieces.push_back( std::move( piece ) );
    }
    state = BatchedInferenceState {};
    return pieces;
  }

  // one piece per run of rows whose kv cache lives on the same (tier, rank)
  static std::deque<BatchedInferenceState> split_on_kv( BatchedInferenceState&& state )
  {
    std::vector<size_t> sizes;
    size_t last_cut = 0;
    for ( size_t i = 1; i < state.metadata_.batch_size; i++ ) {
      if ( state.kv_tier( i ) != state.kv_tier( i - 1 ) || state.kv_rank( i ) != state.kv_rank( i - 1 ) ) {
        sizes.push_back( i - last_cut );
        last_cut = i;
      }
    }
    sizes.push_back( state.metadata_.batch_size - last_cut );
    return split_states( std::move( state ), sizes, true );
  }

  // rows [0, n) and [n, batch); this state is left as it was
  std::pair<BatchedInferenceState, BatchedInferenceState> split( size_t n )
  {
    GLINT_CHECK( n > 0 && n < metadata_.batch_size );
    BatchedInferenceState a = like_this( n ), b = like_this( metadata_.batch_size - n );
    std::copy( prompts_.begin(), prompts_.begin() + n, a.prompts_.begin() );
    std::copy( prompts_.begin() + n, prompts_.end(), b.prompts_.begin() );
    a.copy_rows( 0, *this, 0, n );
    b.copy_rows( 0, *this, n, metadata_.batch_size - n );
    return { std::move( a ), std::move( b ) };
  }

  // appends the rows of `other`, which is left empty
  void merge( BatchedInferenceState&& other )
  {
    if ( metadata_.batch_size == 0 ) {
      *this = std::move( other );
      other = BatchedInferenceState {};
      return;
    }
    if ( other.metadata_.batch_size == 0 ) {
      return;
    }
    GLINT_CHECK( metadata_.dtype == other.metadata_.dtype && metadata_.next_layer == other.metadata_.next_layer && metadata_.next_stage == other.metadata_.next_stage );
    GLINT_CHECK( metadata_.has_activations == other.metadata_.has_activations && metadata_.has_queries == other.metadata_.has_queries
                 && metadata_.has_kvs == other.metadata_.has_kvs );
    const size_t mine = metadata_.batch_size, theirs = other.metadata_.batch_size;
    BatchedInferenceState merged = like_this( mine + theirs );
    std::copy( prompts_.begin(), prompts_.end(), merged.prompts_.begin() );
    std::copy( other.prompts_.begin(), other.prompts_.end(), merged.prompts_.begin() + mine );
    merged.copy_rows( 0, *this, 0, mine );
    merged.copy_rows( mine, other, 0, theirs );
    *this = std::move( merged );
    other = BatchedInferenceState {};
  }

  static BatchedInferenceState merge_states( std::deque<BatchedInferenceState>&& states )
  {
    GLINT_CHECK( !states.empty() );
    BatchedInferenceState out = std::move( states.front() );
    states.pop_front();
    while ( !states.empty() ) {
      out.merge( std::move( states.front() ) );
      states.pop_front();
    }
    return out;
  }

  std::string debug_string( bool prompt_details = false ) const
  {
    std::ostringstream oss;
    oss << "BatchedInferenceState(id=" << metadata_.id << ", batch_size=" << metadata_.batch_size << ", dtype=" << (int)metadata_.dtype
        << ", route_id=" << metadata_.route_id << ", model_id=" << metadata_.model_id << ", next_layer=" << metadata_.next_layer
        << ", next_stage=" << (int)metadata_.next_stage << ", next_tier=" << (int)metadata_.next_tier << ", next_rank=" << (int)metadata_.next_rank
        << ", has_activations=" << metadata_.has_activations << ", has_queries=" << metadata_.has_queries << ", has_kvs=" << metadata_.has_kvs
        << ", is_sharded=" << metadata_.is_sharded << ")";
    if ( prompt_details ) {
      for ( size_t i = 0; i < prompts_.size(); i++ ) {
        const PromptData p = prompts_[i];
        oss << "\n  [" << i << "] active=" << p.active << " context_id=" << p.context_id << " token=" << p.token << " token_pos=" << p.token_pos
            << " finished=" << p.finished << " kv=(" << (int)p.kv_tier << "," << (int)p.kv_rank << ")";
      }
    }
    return oss.str();
  }
};

} // namespace glint
