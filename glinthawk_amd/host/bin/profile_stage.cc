// profile-stage for the hip target; command line of the reference's frontend/profile-stage.cc:
//
//   profile-stage-hip <model_root> <model_name> (paged|static) <stage=(all|all_no_cls|pre|att|post|cls)>
//                     <batch_size> <token_pos> <duration_s> <output_log>
//
// Weights are random, as in the reference's profiler (profile/profiler.hh:68); <model_root> is
// only consulted for its CONFIG file, which must describe <model_name> when it exists ("-" skips it).
#include <cstdlib>
#include <fstream>
#include <iostream>

#include "glint/loader.hh"
#include "glint/profiler.hh"

using namespace glint;

namespace {

void usage( const char* argv0 )
{
  std::cerr << "Usage: " << argv0
            << " <model_root> <model_name> (paged|static) <stage=(all|all_no_cls|pre|att|post|cls)> <batch_size> <token_pos> <duration_s> <output_log>\n";
}

template<typename Config, typename Ctx>
int run( const std::string& model_root, const std::string& model_name, InferenceStage stage, uint32_t batch, uint64_t token_pos, uint64_t duration_s,
         const std::string& log_path )
{
  using DType = float16_t;
  using Model = Llama2<Config, DType, hip::LlamaOperations<Config, DType, Ctx>, Ctx>;
  if ( token_pos >= Config::seq_len ) {
    std::cerr << "Token position out of range\n";
    return EXIT_FAILURE;
  }
  if ( batch == 0 || batch > MAX_BATCH_SIZE ) {
    std::cerr << "Batch size out of range (1.." << MAX_BATCH_SIZE << ")\n";
    return EXIT_FAILURE;
  }
  if ( model_root != "-" && std::filesystem::exists( std::filesystem::path( model_root ) / "CONFIG" ) ) {
    ConfigFile cf;
    std::string err = read_config_file( std::filesystem::path( model_root ) / "CONFIG", cf );
    if ( err.empty() ) {
      err = config_file_mismatch<Config>( cf );
    }
    if ( !err.empty() ) {
      std::cerr << "Error: " << err << '\n';
      return EXIT_FAILURE;
    }
  }
  std::ofstream out( log_path, std::ios::out | std::ios::trunc );
  if ( !out ) {
    std::cerr << "Error: cannot open " << log_path << '\n';
    return EXIT_FAILURE;
  }
  Profiler<Model> profiler( model_name, stage, batch, token_pos, duration_s );
  const uint64_t calls = profiler.run( out );
  std::cerr << "profile-stage-hip: " << profiler.header() << ": " << calls << " calls\n";
  return EXIT_SUCCESS;
}

} // namespace

int main( int argc, char* argv[] )
{
  if ( argc != 9 ) {
    usage( argc > 0 ? argv[0] : "profile-stage-hip" );
    return EXIT_FAILURE;
  }
  const std::string model_root { argv[1] }, model_name { argv[2] }, context_name { argv[3] }, stage_word { argv[4] }, log_path { argv[8] };
  const uint32_t batch = (uint32_t)std::atoi( argv[5] );
  const uint64_t token_pos = (uint64_t)std::atoll( argv[6] ), duration_s = (uint64_t)std::atoll( argv[7] );
  InferenceStage stage;
  if ( !parse_stage_word( stage_word, stage ) ) {
    std::cerr << "Unknown stage: " << stage_word << '\n';
    return EXIT_FAILURE;
  }
  if ( context_name != "paged" && context_name != "static" ) {
    std::cerr << "Unknown context name: " << context_name << '\n';
    return EXIT_FAILURE;
  }
  const bool paged = context_name == "paged";
#define GLINT_MODEL( NAME, CFG )                                                                                                      \
  if ( model_name == NAME ) {                                                                                                       \
    return paged ? run<configs::CFG, hip::DynamicContext<configs::CFG, float16_t>>( model_root, model_name, stage, batch, token_pos, duration_s, log_path ) \
                 : run<configs::CFG, hip::Context<configs::CFG, float16_t>>( model_root, model_name, stage, batch, token_pos, duration_s, log_path );      \
  }
  GLINT_MODEL( "llama2-7b-chat", Llama2_7B_Chat )
  GLINT_MODEL( "llama2-13b-chat", Llama2_13B_Chat )
  GLINT_MODEL( "llama2-70b-chat", Llama2_70B_Chat )
  GLINT_MODEL( "stories-110m", Stories_110M )
  GLINT_MODEL( "test-gqa4", Test_GQA4 )
#undef GLINT_MODEL
  std::cerr << "Unknown model name: " << model_name << ", or context name: " << context_name << '\n';
  return EXIT_FAILURE;
}
