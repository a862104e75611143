// The reference's on-disk model directory (written by tools/bin2glint.py:45-86, read by the Llama2
// constructor, models/llama2/model.hh:180-270):
//
//   CONFIG                 7 x int32: dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len;
//                          a negative vocab_size says that a separate classifier matrix is present
//                          (models/llama2/base.hh:241-258)
//   BASEWEIGHTS_<DT>       token_embedding_table, rms_final_weight, freq_cis_real, freq_cis_imag, [wcls]
//   LAYER<i>_<DT>          rms_att_weight, wq, wk, wv, wo, rms_ffn_weight, w1, w2, w3
//
// <DT> is FP16 or FP32, tensors are raw row-major arrays without padding.  A node copies only the
// tensors of the stages it hosts (models/llama2/base.hh:410-433,520-545); every file it opens must
// have exactly the size the model shape implies (model.hh:191-192).
//
// One deliberate difference: the reference opens every LAYER<i> file as soon as the node hosts
// anything (it passes the byte size of all layers as the "anything to copy?" test,
// model.hh:254-262); here only the files of layers with resident tensors are opened, so a node can
// keep just its own slice on disk.  A directory that works for the reference works here.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <array>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <filesystem>
#include <fstream>
#include <string>

#include "glint/config.hh"
#include "glint/model.hh"
#include "glint/types.hh"

namespace glint {

struct ConfigFile
{
  int32_t dim {}, hidden_dim {}, n_layers {}, n_heads {}, n_kv_heads {}, vocab_size {}, seq_len {};
  static constexpr size_t byte_size = 7 * sizeof( int32_t );
};

// reads the 28 bytes; empty string on success, else what went wrong
inline std::string read_config_file( const std::filesystem::path& file, ConfigFile& out )
{
  std::ifstream fin { file, std::ios::binary };
  if ( !fin ) {
    return "failed to open config file: " + file.string();
  }
  char raw[ConfigFile::byte_size];
  fin.read( raw, sizeof( raw ) );
  if ( fin.gcount() != static_cast<std::streamsize>( sizeof( raw ) ) ) {
    return "failed to read config file: " + file.string();
  }
  int32_t v[7];
  std::memcpy( v, raw, sizeof( raw ) );
  out = ConfigFile { v[0], v[1], v[2], v[3], v[4], v[5], v[6] };
  return {};
}

// the checks of ConfigRuntime's constructor (models/llama2/base.hh:260-282): empty string when the file describes Config
template<typename Config>
std::string config_file_mismatch( const ConfigFile& f )
{
  if ( f.dim <= 0 || f.hidden_dim <= 0 || f.n_layers <= 0 || f.n_heads <= 0 || f.n_kv_heads <= 0 || f.vocab_size == 0 || f.seq_len <= 0
       || f.n_heads % f.n_kv_heads != 0 || f.dim % f.n_heads != 0 ) {
    return "config file holds a non-positive or inconsistent dimension";
  }
  const int64_t gqa = f.n_heads / f.n_kv_heads;
  const int64_t vocab = std::abs( (int64_t)f.vocab_size );
  const bool wcls = f.vocab_size < 0;
  const struct
  {
    const char* what;
    int64_t got, want;
  } rows[] = {
    { "dim", f.dim, (int64_t)Config::dim },
    { "kv_dim", f.dim / gqa, (int64_t)Config::kv_dim },
    { "hidden_dim", f.hidden_dim, (int64_t)Config::hidden_dim },
    { "n_layers", f.n_layers, (int64_t)Config::n_layers },
    { "head_size", f.dim / f.n_heads, (int64_t)Config::head_size },
    { "n_heads", f.n_heads, (int64_t)Config::n_heads },
    { "n_kv_heads", f.n_kv_heads, (int64_t)Config::n_kv_heads },
    { "gqa_size", gqa, (int64_t)Config::gqa_size },
    { "vocab_size", vocab, (int64_t)Config::vocab_size },
    { "seq_len", f.seq_len, (int64_t)Config::seq_len },
    { "wcls_present", wcls ? 1 : 0, Config::wcls_present ? 1 : 0 },
  };
  for ( const auto& r : rows ) {
    if ( r.got != r.want ) {
      return std::string( r.what ) + " does not match config file (" + std::to_string( r.got ) + " in the file, " + std::to_string( r.want ) + " in the model)";
    }
  }
  return {};
}

template<typename DType>
constexpr const char* dtype_suffix()
{
  return sizeof( DType ) == 2 ? "FP16" : "FP32"; // models/types.hh dtype_str
}

// read-only private mapping of a whole file (util/file_descriptor.hh + MMap_Region in the reference)
class MappedFile
{
public:
  MappedFile() = default;
  MappedFile( const MappedFile& ) = delete;
  MappedFile& operator=( const MappedFile& ) = delete;
  ~MappedFile() { close(); }

  // empty string on success
  std::string open( const std::filesystem::path& path, uint64_t expected_bytes )
  {
    close();
    std::error_code ec;
    const auto size = std::filesystem::file_size( path, ec );
    if ( ec ) {
      return "cannot stat " + path.string() + ": " + ec.message();
    }
    if ( size != expected_bytes ) {
      return "file " + path.string() + " is not the expected size (" + std::to_string( size ) + " bytes, " + std::to_string( expected_bytes ) + " expected)";
    }
    fd_ = ::open( path.c_str(), O_RDONLY );
    if ( fd_ < 0 ) {
      return "cannot open " + path.string() + ": " + std::strerror( errno );
    }
    if ( size == 0 ) {
      return {};
    }
    void* p = ::mmap( nullptr, size, PROT_READ, MAP_PRIVATE, fd_, 0 );
    if ( p == MAP_FAILED ) {
      const std::string msg = "cannot map " + path.string() + ": " + std::strerror( errno );
      close();
      return msg;
    }
    addr_ = static_cast<const uint8_t*>( p );
    len_ = size;
    return {};
  }

  void close()
  {
    if ( addr_ != nullptr ) {
      ::munmap( const_cast<uint8_t*>( addr_ ), len_ );
      addr_ = nullptr;
      len_ = 0;
    }
    if ( fd_ >= 0 ) {
      ::close( fd_ );
      fd_ = -1;
    }
  }

  [[nodiscard]] const uint8_t* addr() const { return addr_; }
  [[nodiscard]] uint64_t len() const { return len_; }

private:
  int fd_ { -1 };
  const uint8_t* addr_ { nullptr };
  uint64_t len_ { 0 };
};

// element offsets of the tensors inside their file (prefix sums of the on-disk sizes, base.hh:385-400,511-530)
template<size_t N>
std::array<uint64_t, N> prefix_offsets( const std::array<uint64_t, N>& sizes, uint64_t* total = nullptr )
{
  std::array<uint64_t, N> off {};
  uint64_t run = 0;
  for ( size_t i = 0; i < N; i++ ) {
    off[i] = run;
    run += sizes[i];
  }
  if ( total != nullptr ) {
    *total = run;
  }
  return off;
}

// Walks the files of `model_dir` that a node with `settings` needs and hands every resident tensor
// to `sink( is_base, layer, k, const DType* src, n_elements, file_offset_bytes )`, k in file order.
// Returns an empty string on success; on the first failure it stops and says which file or field
// was wrong.
template<typename Config, typename DType, typename Sink>
std::string walk_model_dir( const StageSettings<Config>& settings, const std::filesystem::path& model_dir, Sink&& sink )
{
  ConfigFile cf;
  if ( auto err = read_config_file( model_dir / "CONFIG", cf ); !err.empty() ) {
    return err;
  }
  if ( auto err = config_file_mismatch<Config>( cf ); !err.empty() ) {
    return err;
  }

  const std::string suffix = std::string( "_" ) + dtype_suffix<DType>();

  {
    const auto on_disk = WeightLayout<Config>::base_on_disk();
    const auto in_memory = WeightLayout<Config>::base_in_memory( settings );
    uint64_t total = 0, resident = 0;
    const auto off = prefix_offsets( on_disk, &total );
    for ( auto n : in_memory ) {
      resident += n;
    }
    if ( resident > 0 ) {
      MappedFile file;
      if ( auto err = file.open( model_dir / ( "BASEWEIGHTS" + suffix ), total * sizeof( DType ) ); !err.empty() ) {
        return err;
      }
      for ( size_t k = 0; k < on_disk.size(); k++ ) {
        if ( in_memory[k] > 0 ) {
          sink( true, size_t { 0 }, k, reinterpret_cast<const DType*>( file.addr() ) + off[k], in_memory[k], off[k] * sizeof( DType ) );
        }
      }
    }
  }

  const auto on_disk = WeightLayout<Config>::layer_on_disk();
  uint64_t total = 0;
  const auto off = prefix_offsets( on_disk, &total );
  for ( size_t l = 0; l < Config::n_layers; l++ ) {
    const auto in_memory = WeightLayout<Config>::layer_in_memory( settings, l );
    uint64_t resident = 0;
    for ( auto n : in_memory ) {
      resident += n;
    }
    if ( resident == 0 ) {
      continue;
    }
    MappedFile file;
    if ( auto err = file.open( model_dir / ( "LAYER" + std::to_string( l ) + suffix ), total * sizeof( DType ) ); !err.empty() ) {
      return err;
    }
    for ( size_t k = 0; k < on_disk.size(); k++ ) {
      if ( in_memory[k] > 0 ) {
        sink( false, l, k, reinterpret_cast<const DType*>( file.addr() ) + off[k], in_memory[k], off[k] * sizeof( DType ) );
      }
    }
  }
  return {};
}

// Copies what `model` hosts out of `model_dir`.  (Llama2::load() turns a failure into an abort,
// which is what the reference's CHECKs do.)
template<typename Model>
std::string load_model_dir( Model& model, const std::filesystem::path& model_dir )
{
  using Config = typename Model::ConfigType;
  using DType = typename Model::DataTypeT;
  return walk_model_dir<Config, DType>( model.settings(), model_dir, [&]( bool is_base, size_t layer, size_t k, const DType* src, uint64_t n, uint64_t ) {
    if ( is_base ) {
      model.set_base_tensor( k, src, n );
    } else {
      model.set_layer_tensor( layer, k, src, n );
    }
  } );
}

} // namespace glint
