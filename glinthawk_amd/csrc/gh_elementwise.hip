// Small bandwidth-bound ops of the stage: accum, rmsnorm, silu, argmax, soft_sample, dtype
// conversion and buffer fills.  All math in fp32 on fp16/fp32 storage, one rounding per store,
// following the reference's CPU path (arch/amd64/common/ops.hh).
#include "gh_common.h"

#include <vector>

namespace gh {
namespace {

constexpr int EW_THREADS = 256;

// 16-byte vector of T
template<typename T>
struct Vec16
{
  static constexpr int N = 16 / sizeof( T );
  union
  {
    uint4 raw;
    T v[N];
  };
};

inline unsigned blocks_for( uint64_t items, int per_block, unsigned cap = 65535u * 16u )
{
  uint64_t b = ( items + per_block - 1 ) / per_block;
  if ( b < 1 ) {
    b = 1;
  }
  return (unsigned)( b > cap ? cap : b );
}

// ---- accum ---------------------------------------------------------------------------------
template<typename T>
__global__ __launch_bounds__( EW_THREADS ) void accum_kernel( T* __restrict__ a, const T* __restrict__ b, uint64_t n )
{
  constexpr int N = Vec16<T>::N;
  const uint64_t n_vec = n / N;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for ( uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride ) {
    Vec16<T> va, vb;
    va.raw = reinterpret_cast<const uint4*>( a )[i];
    vb.raw = reinterpret_cast<const uint4*>( b )[i];
#pragma unroll
    for ( int k = 0; k < N; k++ ) {
      va.v[k] = from_f32<T>( to_f32( va.v[k] ) + to_f32( vb.v[k] ) );
    }
    reinterpret_cast<uint4*>( a )[i] = va.raw;
  }
  for ( uint64_t i = n_vec * N + (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride ) {
    a[i] = from_f32<T>( to_f32( a[i] ) + to_f32( b[i] ) );
  }
}

// ---- silu ----------------------------------------------------------------------------------
__device__ __forceinline__ float silu_mul( float x, float y ) { return x / ( 1.0f + __expf( -x ) ) * y; }

template<typename T>
__global__ __launch_bounds__( EW_THREADS ) void silu_kernel( T* __restrict__ hb, const T* __restrict__ hb2, uint64_t n )
{
  constexpr int N = Vec16<T>::N;
  const uint64_t n_vec = n / N;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for ( uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride ) {
    Vec16<T> va, vb;
    va.raw = reinterpret_cast<const uint4*>( hb )[i];
    vb.raw = reinterpret_cast<const uint4*>( hb2 )[i];
#pragma unroll
    for ( int k = 0; k < N; k++ ) {
      va.v[k] = from_f32<T>( silu_mul( to_f32( va.v[k] ), to_f32( vb.v[k] ) ) );
    }
    reinterpret_cast<uint4*>( hb )[i] = va.raw;
  }
  for ( uint64_t i = n_vec * N + (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride ) {
    hb[i] = from_f32<T>( silu_mul( to_f32( hb[i] ), to_f32( hb2[i] ) ) );
  }
}

// ---- block reductions -------------------------------------------------------------------------
__device__ __forceinline__ float block_sum( float v, float* smem )
{
  v = wave_sum( v );
  const int wave = threadIdx.x / WAVE;
  const int n_waves = blockDim.x / WAVE;
  if ( threadIdx.x % WAVE == 0 ) {
    smem[wave] = v;
  }
  __syncthreads();
  float total = 0.0f;
  for ( int w = 0; w < n_waves; w++ ) {
    total += smem[w];
  }
  __syncthreads();
  return total;
}

// ---- rmsnorm: one block per row ----------------------------------------------------------------
template<typename T>
__global__ __launch_bounds__( EW_THREADS ) void rmsnorm_kernel( T* __restrict__ out,
                                                               const T* __restrict__ x,
                                                               const T* __restrict__ weight,
                                                               uint32_t size )
{
  __shared__ float smem[EW_THREADS / WAVE];
  constexpr int N = Vec16<T>::N;
  const T* X = x + (uint64_t)blockIdx.x * size;
  T* O = out + (uint64_t)blockIdx.x * size;
  const uint32_t n_vec = ( size % N == 0 ) ? size / N : 0; // vector path only for aligned rows

  float ss = 0.0f;
  for ( uint32_t i = threadIdx.x; i < n_vec; i += blockDim.x ) {
    Vec16<T> v;
    v.raw = reinterpret_cast<const uint4*>( X )[i];
#pragma unroll
    for ( int k = 0; k < N; k++ ) {
      const float f = to_f32( v.v[k] );
      ss += f * f;
    }
  }
  for ( uint32_t i = n_vec * N + threadIdx.x; i < size; i += blockDim.x ) {
    const float f = to_f32( X[i] );
    ss += f * f;
  }
  ss = block_sum( ss, smem );
  ss = ss / (float)size + 1e-5f;
  const float inv = 1.0f / sqrtf( ss );

  for ( uint32_t i = threadIdx.x; i < n_vec; i += blockDim.x ) {
    Vec16<T> v, w;
    v.raw = reinterpret_cast<const uint4*>( X )[i];
    w.raw = reinterpret_cast<const uint4*>( weight )[i];
#pragma unroll
    for ( int k = 0; k < N; k++ ) {
      v.v[k] = from_f32<T>( to_f32( w.v[k] ) * ( inv * to_f32( v.v[k] ) ) );
    }
    reinterpret_cast<uint4*>( O )[i] = v.raw;
  }
  for ( uint32_t i = n_vec * N + threadIdx.x; i < size; i += blockDim.x ) {
    O[i] = from_f32<T>( to_f32( weight[i] ) * ( inv * to_f32( X[i] ) ) );
  }
}

// ---- argmax: one block per row, first index of the maximum --------------------------------------
template<typename T>
__global__ __launch_bounds__( EW_THREADS ) void argmax_kernel( uint32_t* __restrict__ out, const T* __restrict__ v, uint32_t n )
{
  __shared__ float s_val[EW_THREADS / WAVE];
  __shared__ uint32_t s_idx[EW_THREADS / WAVE];
  const T* row = v + (uint64_t)blockIdx.x * n;

  float best = -INFINITY;
  uint32_t best_i = 0xffffffffu;
  // ascending indices per thread, strict '>' keeps the lowest index of equal values
  for ( uint32_t i = threadIdx.x; i < n; i += blockDim.x ) {
    const float f = to_f32( row[i] );
    if ( f > best || best_i == 0xffffffffu ) {
      best = f;
      best_i = i;
    }
  }
#pragma unroll
  for ( int off = 32; off > 0; off >>= 1 ) {
    const float o_val = __shfl_xor( best, off, WAVE );
    const uint32_t o_idx = __shfl_xor( best_i, off, WAVE );
    if ( o_idx != 0xffffffffu && ( best_i == 0xffffffffu || o_val > best || ( o_val == best && o_idx < best_i ) ) ) {
      best = o_val;
      best_i = o_idx;
    }
  }
  const int wave = threadIdx.x / WAVE;
  if ( threadIdx.x % WAVE == 0 ) {
    s_val[wave] = best;
    s_idx[wave] = best_i;
  }
  __syncthreads();
  if ( threadIdx.x == 0 ) {
    for ( int w = 1; w < (int)( blockDim.x / WAVE ); w++ ) {
      const float o_val = s_val[w];
      const uint32_t o_idx = s_idx[w];
      if ( o_idx != 0xffffffffu && ( best_i == 0xffffffffu || o_val > best || ( o_val == best && o_idx < best_i ) ) ) {
        best = o_val;
        best_i = o_idx;
      }
    }
    out[blockIdx.x] = best_i;
  }
}

// ---- counter-based random numbers (Philox-4x32-10) ----------------------------------------------
__device__ __forceinline__ uint4 philox( uint64_t counter, uint64_t stream_id, uint64_t seed )
{
  uint32_t c0 = (uint32_t)counter, c1 = (uint32_t)( counter >> 32 ), c2 = (uint32_t)stream_id, c3 = (uint32_t)( stream_id >> 32 );
  uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)( seed >> 32 );
#pragma unroll
  for ( int r = 0; r < 10; r++ ) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)( p1 >> 32 ) ^ c1 ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)( p0 >> 32 ) ^ c3 ^ k1;
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0;
    c1 = n1;
    c2 = n2;
    c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return make_uint4( c0, c1, c2, c3 );
}

__device__ __forceinline__ float u01( uint32_t bits ) { return ( (float)( bits >> 8 ) + 0.5f ) * ( 1.0f / 16777216.0f ); } // (0,1)

template<typename T>
__global__ __launch_bounds__( EW_THREADS ) void fill_uniform_kernel( T* __restrict__ dst, uint64_t n, float lo, float hi, uint64_t seed )
{
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  const uint64_t n4 = ( n + 3 ) / 4;
  for ( uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride ) {
    const uint4 r = philox( i, 0, seed );
    const uint32_t w[4] = { r.x, r.y, r.z, r.w };
#pragma unroll
    for ( int k = 0; k < 4; k++ ) {
      const uint64_t idx = i * 4 + k;
      if ( idx < n ) {
        dst[idx] = from_f32<T>( lo + ( hi - lo ) * u01( w[k] ) );
      }
    }
  }
}

template<typename T>
__global__ __launch_bounds__( EW_THREADS ) void fill_normal_kernel( T* __restrict__ dst, uint64_t n, float mean, float stdv, uint64_t seed )
{
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  const uint64_t n4 = ( n + 3 ) / 4;
  for ( uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride ) {
    const uint4 r = philox( i, 1, seed );
    // Box-Muller, two pairs
    const float r0 = sqrtf( -2.0f * __logf( u01( r.x ) ) );
    const float r1 = sqrtf( -2.0f * __logf( u01( r.z ) ) );
    float s0, c0, s1, c1;
    __sincosf( 6.2831853071795865f * u01( r.y ), &s0, &c0 );
    __sincosf( 6.2831853071795865f * u01( r.w ), &s1, &c1 );
    const float z[4] = { r0 * c0, r0 * s0, r1 * c1, r1 * s1 };
#pragma unroll
    for ( int k = 0; k < 4; k++ ) {
      const uint64_t idx = i * 4 + k;
      if ( idx < n ) {
        dst[idx] = from_f32<T>( mean + stdv * z[k] );
      }
    }
  }
}

// ---- soft_sample: Gumbel-max noise on rows with temperature > 0 ---------------------------------
template<typename T>
__global__ __launch_bounds__( EW_THREADS ) void gumbel_kernel( T* __restrict__ v, const float* __restrict__ temps, uint32_t vocab, uint64_t seed )
{
  const float temp = temps[blockIdx.y];
  if ( !( temp > 0.0f ) ) {
    return;
  }
  T* row = v + (uint64_t)blockIdx.y * vocab;
  const uint32_t n4 = ( vocab + 3 ) / 4;
  for ( uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += gridDim.x * blockDim.x ) {
    const uint4 r = philox( i, 2 + blockIdx.y, seed );
    const uint32_t w[4] = { r.x, r.y, r.z, r.w };
#pragma unroll
    for ( int k = 0; k < 4; k++ ) {
      const uint32_t idx = i * 4 + k;
      if ( idx < vocab ) {
        const float noise = logf( -logf( u01( w[k] ) ) );
        row[idx] = from_f32<T>( to_f32( row[idx] ) / temp - noise );
      }
    }
  }
}

// ---- conversion / zero fill --------------------------------------------------------------------
template<typename D, typename S>
__global__ __launch_bounds__( EW_THREADS ) void convert_kernel( D* __restrict__ dst, const S* __restrict__ src, uint64_t n )
{
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for ( uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride ) {
    dst[i] = from_f32<D>( to_f32( src[i] ) );
  }
}

__global__ __launch_bounds__( EW_THREADS ) void zero_kernel( uint32_t* __restrict__ dst, uint64_t n_words, uint8_t* tail, uint32_t n_tail )
{
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for ( uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += stride ) {
    dst[i] = 0u;
  }
  if ( blockIdx.x == 0 && threadIdx.x < n_tail ) {
    tail[threadIdx.x] = 0;
  }
}

inline bool aligned16( const void* p ) { return ( reinterpret_cast<uintptr_t>( p ) & 15u ) == 0; }

} // namespace
} // namespace gh

using namespace gh;

#define GH_DISPATCH_DT( dt, ... )                                                                                      \
  do {                                                                                                                 \
    if ( ( dt ) == GH_F16 ) {                                                                                          \
      using T = __half;                                                                                                \
      __VA_ARGS__;                                                                                                     \
    } else if ( ( dt ) == GH_F32 ) {                                                                                   \
      using T = float;                                                                                                 \
      __VA_ARGS__;                                                                                                     \
    } else {                                                                                                           \
      return fail( GH_ERR_INVALID, "unsupported dtype %d (f16 and f32 only)", (int)( dt ) );                           \
    }                                                                                                                  \
  } while ( 0 )

extern "C" {

int gh_accum( void* a, const void* b, uint64_t size, uint64_t batch, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  const uint64_t n = size * batch;
  if ( n == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( a && b, "gh_accum: NULL pointer" );
  GH_REQUIRE( aligned16( a ) && aligned16( b ), "gh_accum: buffers must be 16-byte aligned" );
  GH_DISPATCH_DT( dt, accum_kernel<T><<<blocks_for( n / Vec16<T>::N + 1, EW_THREADS, 8192 ), EW_THREADS, 0, as_stream( stream )>>>(
                        static_cast<T*>( a ), static_cast<const T*>( b ), n ) );
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_silu( void* hb, const void* hb2, uint64_t hidden_dim, uint64_t batch, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  const uint64_t n = hidden_dim * batch;
  if ( n == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( hb && hb2, "gh_silu: NULL pointer" );
  GH_REQUIRE( aligned16( hb ) && aligned16( hb2 ), "gh_silu: buffers must be 16-byte aligned" );
  GH_DISPATCH_DT( dt, silu_kernel<T><<<blocks_for( n / Vec16<T>::N + 1, EW_THREADS, 8192 ), EW_THREADS, 0, as_stream( stream )>>>(
                        static_cast<T*>( hb ), static_cast<const T*>( hb2 ), n ) );
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_rmsnorm( void* out, const void* x, const void* weight, uint64_t size, uint64_t batch, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 || size == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( out && x && weight, "gh_rmsnorm: NULL pointer" );
  GH_REQUIRE( size <= 0xffffffffull && batch <= 0x7fffffffull, "gh_rmsnorm: shape too large" );
  GH_REQUIRE( aligned16( out ) && aligned16( x ) && aligned16( weight ), "gh_rmsnorm: buffers must be 16-byte aligned" );
  GH_DISPATCH_DT( dt, rmsnorm_kernel<T><<<(unsigned)batch, EW_THREADS, 0, as_stream( stream )>>>(
                        static_cast<T*>( out ), static_cast<const T*>( x ), static_cast<const T*>( weight ), (uint32_t)size ) );
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_argmax( uint32_t* out_host, uint32_t* out_dev, const void* v, uint64_t n, uint64_t batch, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( out_dev && v, "gh_argmax: NULL pointer" );
  GH_REQUIRE( n > 0 && n <= 0xfffffffeull && batch <= 0x7fffffffull, "gh_argmax: bad shape" );
  GH_DISPATCH_DT( dt, argmax_kernel<T><<<(unsigned)batch, EW_THREADS, 0, as_stream( stream )>>>( out_dev, static_cast<const T*>( v ), (uint32_t)n ) );
  GH_LAUNCH_CHECK();
  if ( out_host ) {
    GH_HIP( hipMemcpyAsync( out_host, out_dev, batch * sizeof( uint32_t ), hipMemcpyDeviceToHost, as_stream( stream ) ) );
    GH_HIP( hipStreamSynchronize( as_stream( stream ) ) );
  }
  return GH_OK;
}

int gh_soft_sample( void* v, const float* temperatures, uint64_t vocab, uint64_t batch, uint64_t seed, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 || vocab == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( v && temperatures, "gh_soft_sample: NULL pointer" );
  GH_REQUIRE( batch <= MAX_BATCH && vocab <= 0xffffffffull, "gh_soft_sample: batch > %llu", (unsigned long long)MAX_BATCH );
  bool any = false;
  for ( uint64_t i = 0; i < batch; i++ ) {
    any = any || temperatures[i] > 0.0f;
  }
  if ( !any ) {
    return GH_OK; // greedy rows are untouched, as in the reference
  }
  void* d_temps = nullptr;
  StageScope scope( as_stream( stream ) );
  if ( int rc = stage_table( temperatures, batch * sizeof( float ), as_stream( stream ), &d_temps ) ) {
    return rc;
  }
  const dim3 grid( blocks_for( vocab / 4 + 1, EW_THREADS, 64 ), (unsigned)batch );
  GH_DISPATCH_DT( dt, gumbel_kernel<T><<<grid, EW_THREADS, 0, as_stream( stream )>>>(
                        static_cast<T*>( v ), static_cast<const float*>( d_temps ), (uint32_t)vocab, seed ) );
  GH_LAUNCH_CHECK();
  return scope.finish();
}

int gh_fill_uniform( void* dst, uint64_t n, float lo, float hi, uint64_t seed, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( n == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( dst, "gh_fill_uniform: NULL pointer" );
  GH_DISPATCH_DT( dt, fill_uniform_kernel<T><<<blocks_for( n / 4 + 1, EW_THREADS, 16384 ), EW_THREADS, 0, as_stream( stream )>>>(
                        static_cast<T*>( dst ), n, lo, hi, seed ) );
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_fill_normal( void* dst, uint64_t n, float mean, float std, uint64_t seed, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( n == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( dst, "gh_fill_normal: NULL pointer" );
  GH_DISPATCH_DT( dt, fill_normal_kernel<T><<<blocks_for( n / 4 + 1, EW_THREADS, 16384 ), EW_THREADS, 0, as_stream( stream )>>>(
                        static_cast<T*>( dst ), n, mean, std, seed ) );
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_memset_zero( void* dst, uint64_t bytes, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( bytes == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( dst && ( reinterpret_cast<uintptr_t>( dst ) & 3u ) == 0, "gh_memset_zero: pointer must be 4-byte aligned" );
  const uint64_t words = bytes / 4;
  zero_kernel<<<blocks_for( words + 1, EW_THREADS, 8192 ), EW_THREADS, 0, as_stream( stream )>>>(
    static_cast<uint32_t*>( dst ), words, static_cast<uint8_t*>( dst ) + words * 4, (uint32_t)( bytes % 4 ) );
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_convert( void* dst, gh_dtype dst_dt, const void* src, gh_dtype src_dt, uint64_t n, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( n == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( dst && src, "gh_convert: NULL pointer" );
  const unsigned blocks = blocks_for( n, EW_THREADS, 8192 );
  hipStream_t s = as_stream( stream );
  if ( dst_dt == src_dt ) {
    GH_REQUIRE( dst_dt == GH_F16 || dst_dt == GH_F32, "gh_convert: unsupported dtype" );
    GH_HIP( hipMemcpyAsync( dst, src, n * dtype_size( dst_dt ), hipMemcpyDeviceToDevice, s ) );
    return GH_OK;
  }
  if ( dst_dt == GH_F16 && src_dt == GH_F32 ) {
    convert_kernel<__half, float><<<blocks, EW_THREADS, 0, s>>>( static_cast<__half*>( dst ), static_cast<const float*>( src ), n );
  } else if ( dst_dt == GH_F32 && src_dt == GH_F16 ) {
    convert_kernel<float, __half><<<blocks, EW_THREADS, 0, s>>>( static_cast<float*>( dst ), static_cast<const __half*>( src ), n );
  } else {
    return fail( GH_ERR_INVALID, "gh_convert: unsupported dtype pair %d <- %d", (int)dst_dt, (int)src_dt );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

// LlamaOperations::convert_and_copy: the conversion runs on the side that is the device; the host
// side only sees a byte copy of its own dtype.  Everything is queued on the caller's stream, which
// is waited for before the call returns (the reference's conversion is synchronous).
int gh_convert_and_copy( void* dst, gh_dtype dst_dt, const void* src, gh_dtype src_dt, uint64_t n, gh_copy_kind kind, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( n == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( dst && src, "gh_convert_and_copy: NULL pointer" );
  GH_REQUIRE( ( dst_dt == GH_F16 || dst_dt == GH_F32 ) && ( src_dt == GH_F16 || src_dt == GH_F32 ), "gh_convert_and_copy: unsupported dtype" );
  GH_REQUIRE( kind == GH_HOST_TO_DEVICE || kind == GH_DEVICE_TO_HOST || kind == GH_DEVICE_TO_DEVICE || kind == GH_HOST_TO_HOST,
              "gh_convert_and_copy: bad copy kind %d", (int)kind );
  if ( dst_dt == src_dt ) {
    return gh_memcpy( dst, src, n * dtype_size( dst_dt ), kind, 0, stream );
  }
  hipStream_t st = as_stream( stream );
  if ( kind == GH_DEVICE_TO_DEVICE ) {
    if ( int rc = gh_convert( dst, dst_dt, src, src_dt, n, stream ) ) {
      return rc;
    }
    GH_HIP( hipStreamSynchronize( st ) );
    return GH_OK;
  }
  // a device target never converts host memory into host memory (LOG(FATAL) "Invalid copy type" in arch/cuda/llama2/ops.cuh:490)
  GH_REQUIRE( kind != GH_HOST_TO_HOST, "gh_convert_and_copy: a converting copy needs a device side" );
  void* tmp = nullptr;
  const gh_dtype tmp_dt = kind == GH_HOST_TO_DEVICE ? src_dt : dst_dt;
  if ( int rc = stream_scratch( st, SCRATCH_CONVERT, n * dtype_size( tmp_dt ), 4ull << 20, &tmp ) ) {
    return rc;
  }
  if ( kind == GH_HOST_TO_DEVICE ) {
    GH_HIP( hipMemcpyAsync( tmp, src, n * dtype_size( src_dt ), hipMemcpyHostToDevice, st ) );
    if ( int rc = gh_convert( dst, dst_dt, tmp, src_dt, n, stream ) ) {
      (void)hipStreamSynchronize( st );
      return rc;
    }
  } else {
    if ( int rc = gh_convert( tmp, dst_dt, src, src_dt, n, stream ) ) {
      return rc;
    }
    GH_HIP( hipMemcpyAsync( dst, tmp, n * dtype_size( dst_dt ), hipMemcpyDeviceToHost, st ) );
  }
  GH_HIP( hipStreamSynchronize( st ) );
  return GH_OK;
}

} // extern "C"
