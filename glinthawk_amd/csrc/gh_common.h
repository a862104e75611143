// Internal helpers shared by the HIP translation units of libglint_hip.so (gfx950 only).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>

#include "glint_hip.h"

namespace gh {

// ---- error plumbing ---------------------------------------------------------------------------
void set_error( const char* fmt, ... ) __attribute__( ( format( printf, 1, 2 ) ) );
int fail( int status, const char* fmt, ... ) __attribute__( ( format( printf, 2, 3 ) ) );

#define GH_HIP( expr )                                                                                                 \
  do {                                                                                                                 \
    hipError_t gh_err_ = ( expr );                                                                                     \
    if ( gh_err_ != hipSuccess ) {                                                                                     \
      return ::gh::fail( gh_err_ == hipErrorOutOfMemory ? GH_ERR_OOM : GH_ERR_DEVICE,                                  \
                         "%s failed: %s (%s:%d)",                                                                      \
                         #expr,                                                                                        \
                         hipGetErrorString( gh_err_ ),                                                                 \
                         __FILE__,                                                                                     \
                         __LINE__ );                                                                                   \
    }                                                                                                                  \
  } while ( 0 )

#define GH_REQUIRE( cond, ... )                                                                                        \
  do {                                                                                                                 \
    if ( !( cond ) ) {                                                                                                 \
      return ::gh::fail( GH_ERR_INVALID, __VA_ARGS__ );                                                                \
    }                                                                                                                  \
  } while ( 0 )

// after a kernel launch: surface launch-configuration errors
#define GH_LAUNCH_CHECK() GH_HIP( hipGetLastError() )

int ensure_init();
// device the library was initialised on, -1 before initialisation (never initialises)
int initialised_device();
// gh_attn_decode.hip: looks up the address of this device's static split-partial array; called once by the initialisation, with `device` current
int attn_static_scratch_init( int device );
// compute units of the device the library was initialised on (256 before initialisation)
int cu_count();

inline hipStream_t as_stream( gh_stream s ) { return reinterpret_cast<hipStream_t>( s ); }

inline size_t dtype_size( gh_dtype dt ) { return dt == GH_F32 ? 4 : 2; }

// ---- staging of host-side pointer / position tables ------------------------------------------
// Copies `bytes` from a host array into a slot of a device-side ring (via pinned memory) on
// `stream` and returns the device address; a table identical to one staged a moment ago on the same
// stream gets that slot again without a copy.  A slot is rewritten only after the work that was
// queued behind its last use has finished, and never between being handed out and the fence.
int stage_table( const void* host_src, size_t bytes, hipStream_t stream, void** dev_out );
// Marks the end of the work that reads the slots handed out on this stream since its last fence.
int stage_fence( hipStream_t stream );
// Fences on every way out of an entry point that staged tables, also when the op in between failed.
class StageScope
{
  hipStream_t stream_;
  bool done_ = false;

public:
  explicit StageScope( hipStream_t stream )
    : stream_( stream )
  {
  }
  StageScope( const StageScope& ) = delete;
  StageScope& operator=( const StageScope& ) = delete;
  ~StageScope()
  {
    if ( !done_ ) {
      (void)stage_fence( stream_ );
    }
  }
  int finish()
  {
    done_ = true;
    return stage_fence( stream_ );
  }
};

// ---- library-owned device scratch ---------------------------------------------------------------
// Grow-only buffer for purpose `which`, private to `stream`: work queued on different streams never
// shares one.  Growing waits for that stream only.  `min_bytes` is the size of the first allocation.
enum { SCRATCH_GEMM_PARTIALS = 0, SCRATCH_CONVERT = 1, SCRATCH_ATTN_PV = 2, SCRATCH_GATE_FACTOR = 3, SCRATCH_LIBRARY = 4, SCRATCH_PRODUCT = 5, SCRATCH_GEMM_PIECES = 6 };
int stream_scratch( hipStream_t stream, int which, uint64_t bytes, uint64_t min_bytes, void** out );
// gh_gemm_lib.hip: a plain f16 product through the vendor's GEMM library; *done = false: declined, nothing queued
int gemm_library( void* xout, const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, hipStream_t st, bool* done );
bool gemm_library_available( uint64_t s, uint64_t r, uint64_t b );
bool gemm_library_wanted( uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, const void* x, const void* w, const void* xout );
bool gemm_library_wanted_wide( uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, const void* x, const void* w, const void* xout );

// Three events per sampled attention call when the benchmark's timer is enabled (slot == -1: off):
// before the split-K kernel, between it and the merge kernel, after the merge kernel.
int timer_mark( hipStream_t stream, int* slot_inout, int which );

constexpr size_t STAGE_SLOT_BYTES = 16 * 1024; // 1024 rows x (8-byte pointer + 4-byte position) fits
constexpr uint64_t MAX_BATCH = 1024;           // models/llama2/base.hh:26

// ---- device helpers ---------------------------------------------------------------------------
constexpr int WAVE = 64;

__device__ __forceinline__ float dpp_quad_xor1( float v )
{
  return __builtin_bit_cast( float, __builtin_amdgcn_update_dpp( 0, __builtin_bit_cast( int, v ), 0xB1, 0xF, 0xF, true ) );
}
__device__ __forceinline__ float dpp_quad_xor2( float v )
{
  return __builtin_bit_cast( float, __builtin_amdgcn_update_dpp( 0, __builtin_bit_cast( int, v ), 0x4E, 0xF, 0xF, true ) );
}
__device__ __forceinline__ float dpp_half_mirror( float v )
{
  return __builtin_bit_cast( float, __builtin_amdgcn_update_dpp( 0, __builtin_bit_cast( int, v ), 0x141, 0xF, 0xF, true ) );
}
__device__ __forceinline__ float dpp_row_mirror( float v )
{
  return __builtin_bit_cast( float, __builtin_amdgcn_update_dpp( 0, __builtin_bit_cast( int, v ), 0x140, 0xF, 0xF, true ) );
}
// sum over the 16 lanes of a DPP row; every lane of the row gets the total
__device__ __forceinline__ float row16_sum( float v )
{
  v += dpp_quad_xor1( v );
  v += dpp_quad_xor2( v );
  v += dpp_half_mirror( v );
  v += dpp_row_mirror( v );
  return v;
}

__device__ __forceinline__ float row16_max( float v )
{
  v = fmaxf( v, dpp_quad_xor1( v ) );
  v = fmaxf( v, dpp_quad_xor2( v ) );
  v = fmaxf( v, dpp_half_mirror( v ) );
  v = fmaxf( v, dpp_row_mirror( v ) );
  return v;
}
__device__ __forceinline__ float lane_value( float v, int lane )
{
  return __builtin_bit_cast( float, __builtin_amdgcn_readlane( __builtin_bit_cast( int, v ), lane ) );
}

// Reductions over the wave, the result in every lane: within each row of 16 lanes by DPP, whose operand arrives with the
// instruction, then the four rows by lane reads.  A butterfly of lane exchanges goes through the LDS crossbar six times, a round
// trip each.
__device__ __forceinline__ float wave_sum( float v )
{
  v = row16_sum( v );
  return ( lane_value( v, 0 ) + lane_value( v, 16 ) ) + ( lane_value( v, 32 ) + lane_value( v, 48 ) );
}

__device__ __forceinline__ float wave_max( float v )
{
  v = row16_max( v );
  return fmaxf( fmaxf( lane_value( v, 0 ), lane_value( v, 16 ) ), fmaxf( lane_value( v, 32 ), lane_value( v, 48 ) ) );
}

template<typename T>
__device__ __forceinline__ float to_f32( T v );
template<>
__device__ __forceinline__ float to_f32<float>( float v )
{
  return v;
}
template<>
__device__ __forceinline__ float to_f32<__half>( __half v )
{
  return __half2float( v );
}

template<typename T>
__device__ __forceinline__ T from_f32( float v );
template<>
__device__ __forceinline__ float from_f32<float>( float v )
{
  return v;
}
template<>
__device__ __forceinline__ __half from_f32<__half>( float v )
{
  return __float2half_rn( v );
}

} // namespace gh
