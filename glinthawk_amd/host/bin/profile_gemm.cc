// profile-gemm for the hip target; command line of the reference's frontend/profile-gemm.cc:
//
//   profile-gemm-hip <dim1> <dim2> <dim3> <duration_s> <output_log>
//
// times out(dim1, dim3) = in(dim1, dim2) x w(dim3, dim2)^T in fp16.
#include <cstdlib>
#include <fstream>
#include <iostream>

#include "glint/profiler.hh"

int main( int argc, char* argv[] )
{
  if ( argc != 6 ) {
    std::cerr << "Usage: " << ( argc > 0 ? argv[0] : "profile-gemm-hip" ) << " <dim1> <dim2> <dim3> <duration_s> <output_log>\n";
    return EXIT_FAILURE;
  }
  const long long d1 = std::atoll( argv[1] ), d2 = std::atoll( argv[2] ), d3 = std::atoll( argv[3] ), dur = std::atoll( argv[4] );
  if ( d1 <= 0 || d2 <= 0 || d3 <= 0 || dur < 0 ) {
    std::cerr << "Error: dimensions must be positive\n";
    return EXIT_FAILURE;
  }
  std::ofstream out( argv[5], std::ios::out | std::ios::trunc );
  if ( !out ) {
    std::cerr << "Error: cannot open " << argv[5] << '\n';
    return EXIT_FAILURE;
  }
  glint::GEMMProfiler<glint::float16_t> profiler( (size_t)d1, (size_t)d2, (size_t)d3, (size_t)dur );
  const uint64_t calls = profiler.run( out );
  std::cerr << "profile-gemm-hip: " << profiler.header() << ": " << calls << " calls\n";
  return EXIT_SUCCESS;
}
