// Plain types shared by the host layer.  Enumerator values equal the reference's
// (models/types.hh:19-38,127-133) so that states and settings can cross the boundary unchanged.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>

namespace glint {

using ContextID = uint32_t; // models/types.hh:14

enum class DataType : uint8_t
{
  Float16 = 0,
  Float32 = 1,
  BFloat16 = 2,
};

inline size_t DataTypeSize( const DataType dt ) { return dt == DataType::Float32 ? 4 : 2; }

enum class InferenceStage : uint8_t
{
  PreAttention,
  Attention,
  PostAttention,
  Classification,
  __COUNT__,
  __ALL_NO_CLS__,
  __ALL__,
};

constexpr size_t N_STAGES = static_cast<size_t>( InferenceStage::__COUNT__ );

enum class CopyType
{
  HostToDevice,
  DeviceToHost,
  DeviceToDevice,
  HostToHost
};

using float16_t = _Float16;
using float32_t = float;

template<typename DType>
constexpr DataType dtype_of()
{
  static_assert( sizeof( DType ) == 2 || sizeof( DType ) == 4 );
  return sizeof( DType ) == 2 ? DataType::Float16 : DataType::Float32;
}

// The reference aborts on every failed check on the op path (glog CHECK / LOG(FATAL),
// arch/cuda/common/ops.cu:5-19); the host layer does the same.
[[noreturn]] inline void fatal( const char* file, int line, const char* what, const char* detail = "" )
{
  std::fprintf( stderr, "[glint] FATAL %s:%d: %s %s\n", file, line, what, detail );
  std::abort();
}

#define GLINT_CHECK( cond )                                                                                            \
  do {                                                                                                                 \
    if ( !( cond ) ) {                                                                                                 \
      ::glint::fatal( __FILE__, __LINE__, "check failed:", #cond );                                                    \
    }                                                                                                                  \
  } while ( 0 )

} // namespace glint
