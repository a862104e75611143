// KV append (LlamaOperations::copy_kv_cache) and RoPE (LlamaOperations::apply_rope) for a whole
// batch in one launch each.  The per-context row pointers come from a device-side table; a NULL
// entry is the reference's empty context and is skipped.
#include "gh_common.h"

namespace gh {
namespace {

// One block column per context; threads copy 16 bytes each.  Bit copy, no conversion.
__global__ __launch_bounds__( 256 ) void kv_append_kernel( void* const* __restrict__ rows,
                                                           const uint8_t* __restrict__ state_kv,
                                                           uint32_t row_bytes )
{
  uint8_t* dst = static_cast<uint8_t*>( rows[blockIdx.y] );
  if ( dst == nullptr ) {
    return;
  }
  const uint8_t* src = state_kv + (uint64_t)blockIdx.y * row_bytes;
  const bool vec_ok = ( ( reinterpret_cast<uintptr_t>( dst ) | reinterpret_cast<uintptr_t>( src ) | row_bytes ) & 15u ) == 0;
  if ( vec_ok ) {
    const uint32_t n = row_bytes / 16;
    for ( uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x ) {
      reinterpret_cast<uint4*>( dst )[i] = reinterpret_cast<const uint4*>( src )[i];
    }
  } else {
    // rows are at least element aligned (2 bytes)
    const uint32_t n = row_bytes / 2;
    for ( uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x ) {
      reinterpret_cast<uint16_t*>( dst )[i] = reinterpret_cast<const uint16_t*>( src )[i];
    }
  }
}

// thread <-> (kv head j, pair k): rotates K[j][2k, 2k+1] in the cache row and the gqa query heads
// that share kv head j.  fp32 math on DType storage (arch/amd64/llama2/ops.hh:138-164).
template<typename T>
__global__ __launch_bounds__( 256 ) void rope_kernel( const uint32_t* __restrict__ pos,
                                                      const T* __restrict__ freq_real,
                                                      const T* __restrict__ freq_imag,
                                                      T* __restrict__ q,
                                                      void* const* __restrict__ rows,
                                                      uint32_t n_kv_heads,
                                                      uint32_t gqa,
                                                      uint32_t head_size )
{
  const uint32_t ctx = blockIdx.y;
  T* krow = static_cast<T*>( rows[ctx] );
  if ( krow == nullptr ) {
    return;
  }
  const uint32_t half = head_size / 2;
  const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
  if ( idx >= n_kv_heads * half ) {
    return;
  }
  const uint32_t j = idx / half;
  const uint32_t k = idx % half;
  const uint64_t p = pos[ctx];
  const float fcr = to_f32( freq_real[p * half + k] );
  const float fci = to_f32( freq_imag[p * half + k] );

  T* kp = krow + (uint64_t)j * head_size + 2 * k;
  const float k0 = to_f32( kp[0] );
  const float k1 = to_f32( kp[1] );
  kp[0] = from_f32<T>( k0 * fcr - k1 * fci );
  kp[1] = from_f32<T>( k0 * fci + k1 * fcr );

  T* qp = q + (uint64_t)ctx * n_kv_heads * gqa * head_size + (uint64_t)j * gqa * head_size + 2 * k;
  for ( uint32_t g = 0; g < gqa; g++ ) {
    const float q0 = to_f32( qp[g * head_size] );
    const float q1 = to_f32( qp[g * head_size + 1] );
    qp[g * head_size] = from_f32<T>( q0 * fcr - q1 * fci );
    qp[g * head_size + 1] = from_f32<T>( q0 * fci + q1 * fcr );
  }
}

// The same for f16 with 16-byte accesses: thread <-> (kv head j, four pairs 4m .. 4m+3).  Used when the head
// size is a multiple of 8 and q and the tables are aligned; a cache row that is not 16-byte aligned
// makes its block take two-byte accesses (same arithmetic, same rounding).
__global__ __launch_bounds__( 256 ) void rope_f16x8_kernel( const uint32_t* __restrict__ pos,
                                                            const __half* __restrict__ freq_real,
                                                            const __half* __restrict__ freq_imag,
                                                            __half* __restrict__ q,
                                                            void* const* __restrict__ rows,
                                                            uint32_t n_kv_heads,
                                                            uint32_t gqa,
                                                            uint32_t head_size )
{
  const uint32_t ctx = blockIdx.y;
  __half* krow = static_cast<__half*>( rows[ctx] );
  if ( krow == nullptr ) {
    return;
  }
  const uint32_t half = head_size / 2;
  const uint32_t groups = head_size / 8; // groups of four pairs per head
  const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
  if ( idx >= n_kv_heads * groups ) {
    return;
  }
  const uint32_t j = idx / groups;
  const uint32_t m = idx % groups;
  const uint64_t p = pos[ctx];
  union H4
  {
    uint2 raw;
    __half h[4];
  };
  union H8
  {
    uint4 raw;
    __half h[8];
  };
  H4 fr, fi;
  fr.raw = *reinterpret_cast<const uint2*>( freq_real + p * half + 4 * m );
  fi.raw = *reinterpret_cast<const uint2*>( freq_imag + p * half + 4 * m );
  float c[4], sn[4];
#pragma unroll
  for ( int e = 0; e < 4; e++ ) {
    c[e] = __half2float( fr.h[e] );
    sn[e] = __half2float( fi.h[e] );
  }
  auto rotate = [&]( H8& v ) {
#pragma unroll
    for ( int e = 0; e < 4; e++ ) {
      const float x0 = __half2float( v.h[2 * e] );
      const float x1 = __half2float( v.h[2 * e + 1] );
      v.h[2 * e] = __float2half_rn( x0 * c[e] - x1 * sn[e] );
      v.h[2 * e + 1] = __float2half_rn( x0 * sn[e] + x1 * c[e] );
    }
  };
  __half* kp = krow + (uint64_t)j * head_size + 8 * m;
  H8 v;
  if ( ( reinterpret_cast<uintptr_t>( krow ) & 15u ) == 0 ) { // uniform across the block
    v.raw = *reinterpret_cast<const uint4*>( kp );
    rotate( v );
    *reinterpret_cast<uint4*>( kp ) = v.raw;
  } else {
#pragma unroll
    for ( int e = 0; e < 8; e++ ) {
      v.h[e] = kp[e];
    }
    rotate( v );
#pragma unroll
    for ( int e = 0; e < 8; e++ ) {
      kp[e] = v.h[e];
    }
  }
  __half* qp = q + (uint64_t)ctx * n_kv_heads * gqa * head_size + (uint64_t)j * gqa * head_size + 8 * m;
  for ( uint32_t g = 0; g < gqa; g++ ) {
    v.raw = *reinterpret_cast<const uint4*>( qp + g * head_size );
    rotate( v );
    *reinterpret_cast<uint4*>( qp + g * head_size ) = v.raw;
  }
}

} // namespace
} // namespace gh

using namespace gh;

extern "C" {

int gh_kv_append( void* const* token_rows_dev, const void* state_kv, uint64_t batch, uint32_t kv_dim, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( token_rows_dev && state_kv, "gh_kv_append: NULL pointer" );
  GH_REQUIRE( dt == GH_F16 || dt == GH_F32, "gh_kv_append: unsupported dtype %d", (int)dt );
  GH_REQUIRE( kv_dim > 0 && batch <= 65535, "gh_kv_append: bad shape" );
  const uint32_t row_bytes = 2u * kv_dim * (uint32_t)dtype_size( dt );
  const unsigned bx = ( row_bytes / 16 + 255 ) / 256;
  kv_append_kernel<<<dim3( bx ? bx : 1, (unsigned)batch ), 256, 0, as_stream( stream )>>>(
    token_rows_dev, static_cast<const uint8_t*>( state_kv ), row_bytes );
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_kv_append_host( void* const* token_rows_host, const void* state_kv, uint64_t batch, uint32_t kv_dim, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( token_rows_host, "gh_kv_append_host: NULL table" );
  GH_REQUIRE( batch <= MAX_BATCH, "gh_kv_append_host: batch %llu > %llu", (unsigned long long)batch, (unsigned long long)MAX_BATCH );
  void* d_rows = nullptr;
  StageScope scope( as_stream( stream ) );
  if ( int rc = stage_table( token_rows_host, batch * sizeof( void* ), as_stream( stream ), &d_rows ) ) {
    return rc;
  }
  if ( int rc = gh_kv_append( static_cast<void* const*>( d_rows ), state_kv, batch, kv_dim, dt, stream ) ) {
    return rc;
  }
  return scope.finish();
}

int gh_rope( uint64_t batch, const uint32_t* pos_dev, const void* freq_real, const void* freq_imag, void* q,
             void* const* token_rows_dev, uint32_t n_kv_heads, uint32_t gqa_size, uint32_t head_size, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( pos_dev && freq_real && freq_imag && q && token_rows_dev, "gh_rope: NULL pointer" );
  GH_REQUIRE( head_size % 2 == 0 && head_size > 0 && n_kv_heads > 0 && gqa_size > 0 && batch <= 65535, "gh_rope: bad shape" );
  const unsigned threads = n_kv_heads * ( head_size / 2 );
  const dim3 grid( ( threads + 255 ) / 256, (unsigned)batch );
  const bool vec_ok = dt == GH_F16 && head_size % 8 == 0 && ( reinterpret_cast<uintptr_t>( q ) & 15u ) == 0
                      && ( ( reinterpret_cast<uintptr_t>( freq_real ) | reinterpret_cast<uintptr_t>( freq_imag ) ) & 7u ) == 0;
  if ( vec_ok ) {
    const unsigned vthreads = n_kv_heads * ( head_size / 8 );
    const dim3 vgrid( ( vthreads + 255 ) / 256, (unsigned)batch );
    rope_f16x8_kernel<<<vgrid, 256, 0, as_stream( stream )>>>( pos_dev, static_cast<const __half*>( freq_real ), static_cast<const __half*>( freq_imag ),
                                                             static_cast<__half*>( q ), token_rows_dev, n_kv_heads, gqa_size, head_size );
  } else if ( dt == GH_F16 ) {
    rope_kernel<__half><<<grid, 256, 0, as_stream( stream )>>>( pos_dev, static_cast<const __half*>( freq_real ), static_cast<const __half*>( freq_imag ),
                                                              static_cast<__half*>( q ), token_rows_dev, n_kv_heads, gqa_size, head_size );
  } else if ( dt == GH_F32 ) {
    rope_kernel<float><<<grid, 256, 0, as_stream( stream )>>>( pos_dev, static_cast<const float*>( freq_real ), static_cast<const float*>( freq_imag ),
                                                             static_cast<float*>( q ), token_rows_dev, n_kv_heads, gqa_size, head_size );
  } else {
    return fail( GH_ERR_INVALID, "gh_rope: unsupported dtype %d", (int)dt );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_rope_host( uint64_t batch, const uint32_t* pos_host, const void* freq_real, const void* freq_imag, void* q,
                  void* const* token_rows_host, uint32_t n_kv_heads, uint32_t gqa_size, uint32_t head_size, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( pos_host && token_rows_host, "gh_rope_host: NULL table" );
  GH_REQUIRE( batch <= MAX_BATCH, "gh_rope_host: batch %llu > %llu", (unsigned long long)batch, (unsigned long long)MAX_BATCH );
  void* d_rows = nullptr;
  void* d_pos = nullptr;
  StageScope scope( as_stream( stream ) );
  if ( int rc = stage_table( token_rows_host, batch * sizeof( void* ), as_stream( stream ), &d_rows ) ) {
    return rc;
  }
  if ( int rc = stage_table( pos_host, batch * sizeof( uint32_t ), as_stream( stream ), &d_pos ) ) {
    return rc;
  }
  if ( int rc = gh_rope( batch, static_cast<const uint32_t*>( d_pos ), freq_real, freq_imag, q, static_cast<void* const*>( d_rows ),
                         n_kv_heads, gqa_size, head_size, dt, stream ) ) {
    return rc;
  }
  return scope.finish();
}

} // extern "C"
