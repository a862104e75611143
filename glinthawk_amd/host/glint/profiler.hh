// Stage and GEMM profilers for the hip target: the reference's profile-stage / profile-gemm
// (profile/profiler.hh, profile/gemm_profiler.hh, frontend/profile-stage.cc, frontend/profile-gemm.cc)
// with the same command lines and the same log format
//
//   # model='<name>', stage=<Pre|Att|Post|Cls|Pre+Att+Post|Pre+Att+Post+Cls>, batch_size=B, token_pos=P, duration_s=D
//   repeat,timestamp_ms,duration_us
//   0,1732500000000,6123
//   ...
//
// which py/configuration_opt.py:22-38 reads (file name <model>_<stage>_<ctx>_<token_pos>_<duration>_<batch>.csv,
// first line skipped, mean of duration_us without the first row).  One call = one host-synchronous
// forward*() of the last layer, timed with steady_clock around the call like the reference.
//
// Differences, all on the side of defined behaviour: the hosting table is value-initialised (the
// reference leaves every row but the last uninitialised, profiler.hh:57-68); contexts are prepared
// for `token_pos` before they are filled (the reference fills a paged context's whole span before
// any page is mapped, :88-92); the states carry the buffers the profiled stage reads, filled once
// with uniform noise of the reference's ranges (the reference randomises buffers of length zero,
// :115-128); a ring of 8 states is reused instead of 1000 preallocated ones.
#pragma once

#include <chrono>
#include <cmath>
#include <filesystem>
#include <fstream>
#include <memory>
#include <random>
#include <string>
#include <vector>

#include "glint/model.hh"

namespace glint {

inline const char* stage_text( const InferenceStage s ) // models/types.cc:123-137
{
  switch ( s ) {
    case InferenceStage::PreAttention: return "Pre";
    case InferenceStage::Attention: return "Att";
    case InferenceStage::PostAttention: return "Post";
    case InferenceStage::Classification: return "Cls";
    case InferenceStage::__COUNT__: return "__COUNT__";
    case InferenceStage::__ALL_NO_CLS__: return "Pre+Att+Post";
    case InferenceStage::__ALL__: return "Pre+Att+Post+Cls";
  }
  return "Unknown";
}

// all|all_no_cls|pre|att|post|cls -> stage; false when the word is none of them (frontend/profile-stage.cc:50-66)
inline bool parse_stage_word( const std::string& word, InferenceStage& out )
{
  static const std::pair<const char*, InferenceStage> words[] = {
    { "all", InferenceStage::__ALL__ },        { "all_no_cls", InferenceStage::__ALL_NO_CLS__ }, { "pre", InferenceStage::PreAttention },
    { "att", InferenceStage::Attention },      { "post", InferenceStage::PostAttention },         { "cls", InferenceStage::Classification },
  };
  for ( const auto& [w, s] : words ) {
    if ( word == w ) {
      out = s;
      return true;
    }
  }
  return false;
}

struct ProfileRow
{
  uint64_t repeat, timestamp_ms, duration_us;
};

inline void write_profile_header( std::ostream& out, const std::string& first_line )
{
  out << "# " << first_line << '\n' << "repeat,timestamp_ms,duration_us\n";
}
inline void write_profile_row( std::ostream& out, const ProfileRow& r ) { out << r.repeat << ',' << r.timestamp_ms << ',' << r.duration_us << '\n'; }

template<typename Model>
class Profiler
{
public:
  using Config = typename Model::ConfigType;
  using DType = typename Model::DataTypeT;
  using Context = typename Model::ContextType;
  using State = typename Model::StateType;
  using Settings = typename Model::SettingsType;

  static constexpr size_t RING = 8;

  Profiler( const std::string& model_name, const InferenceStage stage, const uint32_t batch_size, const uint64_t token_pos, const size_t duration_s )
    : model_( make_settings( stage, batch_size ), make_options() )
    , stage_( stage )
    , starting_stage_( stage == InferenceStage::__ALL__ || stage == InferenceStage::__ALL_NO_CLS__ ? InferenceStage::PreAttention : stage )
    , batch_size_( batch_size )
    , token_pos_( token_pos )
    , duration_( duration_s )
  {
    GLINT_CHECK( token_pos < Config::seq_len );
    header_ = "model='" + model_name + "', stage=" + stage_text( stage ) + ", batch_size=" + std::to_string( batch_size )
              + ", token_pos=" + std::to_string( token_pos ) + ", duration_s=" + std::to_string( duration_s );
    const bool attention = model_.settings().hosts_in_any_layer( InferenceStage::Attention );
    const float a = 10.0f / std::sqrt( (float)Config::dim );
    for ( uint32_t i = 0; i < batch_size; i++ ) {
      contexts_.push_back( std::make_shared<Context>( model_.settings(), !attention ) ); // no cache without an attention stage
      if ( attention ) {
        // rows [0, token_pos] exist before anything is written into them
        GLINT_CHECK( contexts_[i]->prepare( layer_, (uint32_t)token_pos, false ) );
        auto first = contexts_[i]->layer( layer_ ).token( 0 );
        model_.ops().randomize_device_buffer( first.key(), ( token_pos + 1 ) * 2 * Config::kv_dim, -a, a );
      }
    }
    states_.resize( RING );
    std::mt19937_64 rng( 12345 );
    for ( auto& st : states_ ) {
      st = State( batch_size, dtype_of<DType>() );
      allocate_inputs( st );
      fill( st.activations(), rng, a );
      fill( st.queries(), rng, 10.0f / std::sqrt( (float)Config::kv_dim ) );
      fill( st.kvs(), rng, 10.0f / std::sqrt( (float)Config::kv_dim ) );
      rewind( st );
    }
  }

  const std::string& header() const { return header_; }

  // one timed call; the state it used is rewound outside the timed region
  ProfileRow step( const uint64_t repeat )
  {
    State& st = states_[repeat % RING];
    const auto wall = std::chrono::system_clock::now();
    const auto start = std::chrono::steady_clock::now();
    switch ( stage_ ) {
      case InferenceStage::PreAttention: model_.forward_pre_attention( st ); break;
      case InferenceStage::Attention: model_.forward_attention( st, contexts_ ); break;
      case InferenceStage::PostAttention: model_.forward_post_attention( st ); break;
      case InferenceStage::Classification: model_.forward_classify( st ); break;
      case InferenceStage::__ALL__:
      case InferenceStage::__ALL_NO_CLS__: model_.forward( st, contexts_ ); break;
      default: fatal( __FILE__, __LINE__, "unknown stage" );
    }
    const auto end = std::chrono::steady_clock::now();
    rewind( st );
    return { repeat, (uint64_t)std::chrono::duration_cast<std::chrono::milliseconds>( wall.time_since_epoch() ).count(),
             (uint64_t)std::chrono::duration_cast<std::chrono::microseconds>( end - start ).count() };
  }

  // calls until `duration_s` has passed (at least one), rows into `out`; returns the number of calls
  uint64_t run( std::ostream& out )
  {
    write_profile_header( out, header_ );
    const auto end_time = std::chrono::steady_clock::now() + duration_;
    uint64_t r = 0;
    for ( ;; r++ ) {
      write_profile_row( out, step( r ) );
      if ( std::chrono::steady_clock::now() >= end_time ) {
        break;
      }
    }
    return r + 1;
  }

private:
  static constexpr uint32_t layer_ = Config::n_layers - 1; // one layer of the model is enough (profiler.hh:30)

  static Settings make_settings( const InferenceStage stage, const uint32_t batch_size )
  {
    typename Settings::HostingTable table {};
    auto& row = table[layer_];
    if ( stage == InferenceStage::__ALL__ ) {
      row[0] = row[1] = row[2] = row[3] = true;
    } else if ( stage == InferenceStage::__ALL_NO_CLS__ ) {
      row[0] = row[1] = row[2] = true;
    } else {
      row[static_cast<size_t>( stage )] = true;
    }
    return Settings( table, batch_size, batch_size, true );
  }
  static ModelOptions make_options()
  {
    ModelOptions o;
    o.seed = 7;
    return o;
  }

  void allocate_inputs( State& st ) const
  {
    switch ( starting_stage_ ) {
      case InferenceStage::PreAttention: st.allocate_activations(); break;
      case InferenceStage::Attention:
        st.allocate_queries();
        st.allocate_kvs();
        break;
      case InferenceStage::PostAttention:
        st.allocate_activations();
        st.allocate_queries();
        break;
      default: st.allocate_activations(); break;
    }
  }

  static void fill( DataBuffer& buf, std::mt19937_64& rng, const float a )
  {
    std::uniform_real_distribution<float> dist( -a, a );
    DType* p = reinterpret_cast<DType*>( buf.data() );
    for ( uint64_t i = 0; i < buf.len() / sizeof( DType ); i++ ) {
      p[i] = static_cast<DType>( dist( rng ) );
    }
  }

  // back to "about to enter the profiled stage at token_pos" (profiler.hh:103-135)
  void rewind( State& st ) const
  {
    st.set_next_layer( layer_ );
    st.set_next_stage( starting_stage_ );
    for ( uint32_t i = 0; i < batch_size_; i++ ) {
      st.set_prompt( i, PromptID {}, ContextID { i + 1 }, 1, (uint32_t)token_pos_, 0.5f, 1, 0, 0, 0 );
    }
  }

  Model model_;
  const InferenceStage stage_, starting_stage_;
  const uint32_t batch_size_;
  const uint64_t token_pos_;
  const std::chrono::seconds duration_;
  std::string header_ {};
  typename Model::ContextVector contexts_ {};
  std::vector<State> states_ {};
};

// untemplated_matmul( out(dim1, dim3), in(dim1, dim2), w(dim3, dim2) ) over 128 rotating input/output
// buffers (profile/gemm_profiler.hh); every call is bracketed by a device synchronisation
template<typename DType>
class GEMMProfiler
{
public:
  static constexpr size_t REPEATS = 128;

  GEMMProfiler( const size_t dim1, const size_t dim2, const size_t dim3, const size_t duration_s )
    : dim1_( dim1 )
    , dim2_( dim2 )
    , dim3_( dim3 )
    , in_( ops_.device_allocate( REPEATS * dim1 * dim2 * sizeof( DType ) ) )
    , w_( ops_.device_allocate( dim3 * dim2 * sizeof( DType ) ) )
    , out_( ops_.device_allocate( REPEATS * dim1 * dim3 * sizeof( DType ) ) )
    , duration_( duration_s )
  {
    const float a = 10.0f / std::sqrt( (float)dim2 );
    ops_.randomize_device_buffer( in_.get(), REPEATS * dim1 * dim2, -a, a );
    ops_.randomize_device_buffer( w_.get(), dim3 * dim2, -a, a );
    ops_.randomize_device_buffer( out_.get(), REPEATS * dim1 * dim3, -a, a );
    header_ = "dim1='" + std::to_string( dim1 ) + "', dim2=" + std::to_string( dim2 ) + ", dim3=" + std::to_string( dim3 )
              + ", duration_s=" + std::to_string( duration_s );
    ops_.synchronize();
  }

  const std::string& header() const { return header_; }

  ProfileRow step( const uint64_t repeat )
  {
    const DType* in = in_.get() + ( repeat % REPEATS ) * dim1_ * dim2_;
    DType* out = out_.get() + ( repeat % REPEATS ) * dim1_ * dim3_;
    const auto wall = std::chrono::system_clock::now();
    const auto start = std::chrono::steady_clock::now();
    ops_.synchronize();
    ops_.untemplated_matmul( out, in, w_.get(), dim2_, dim3_, dim1_ );
    ops_.synchronize();
    const auto end = std::chrono::steady_clock::now();
    return { repeat, (uint64_t)std::chrono::duration_cast<std::chrono::milliseconds>( wall.time_since_epoch() ).count(),
             (uint64_t)std::chrono::duration_cast<std::chrono::microseconds>( end - start ).count() };
  }

  uint64_t run( std::ostream& out )
  {
    write_profile_header( out, header_ );
    const auto end_time = std::chrono::steady_clock::now() + duration_;
    uint64_t r = 0;
    for ( ;; r++ ) {
      write_profile_row( out, step( r ) );
      if ( std::chrono::steady_clock::now() >= end_time ) {
        break;
      }
    }
    return r + 1;
  }

private:
  hip::Operations<DType> ops_ {};
  const size_t dim1_, dim2_, dim3_;
  typename hip::Operations<DType>::DeviceUniquePtr in_, w_, out_;
  const std::chrono::seconds duration_;
  std::string header_ {};
};

} // namespace glint
