// Dense projection GEMM of the stage: xout(b, r) = sum_p w(r, p) * x(b, p), w row-major (r, s),
// fp32 accumulate (Operations::matmul / untemplated_matmul, arch/amd64/common/ops.hh:74-93,212-271).
//
// f16: MFMA kernel.  The weight matrix is the streamed operand (read exactly once), the
// activations are the small operand.  A work-group owns a 64-row slab of w and a 64-column slab of
// the batch, walks K in steps of 128, stages both tiles in LDS with 16-byte chunks XOR-swizzled so
// that the MFMA-operand reads are bank-conflict free, and keeps 4 x (16x16) fp32 accumulators per
// wave (v_mfma_f32_16x16x32_f16).  When r / 64 is too small to fill the chip K is split across
// work-groups and an fp32 partial buffer is reduced by a second kernel.
//
// f32: plain wave-per-row kernel (only the tiny fp32 configuration uses it).
#include "gh_common.h"

#include <cstdlib>
#include <mutex>

namespace gh {

// streaming decode kernel (gh_gemm_stream.hip)
bool gemm_stream_applicable( uint64_t s, uint64_t r, uint64_t b, const void* x, const void* w, const void* xout );
void gemm_stream_plan( uint64_t s, uint64_t r, uint64_t b, uint32_t* splits_out, uint32_t* k_per_split_out, uint32_t* rows_per_wg_out );
int gemm_stream_launch( __half* xout, float* partial, const __half* x, const __half* w, uint64_t s, uint64_t r, uint64_t b, uint32_t splits,
                        uint32_t k_per_split, uint32_t rows_per_wg, bool write_partials, hipStream_t st );
void gemm_stream_tuning( int target_wgs, int depth );
void gemm_stream_gate_waves( int waves );
bool gemm_stream_gate_applicable( uint64_t s, uint64_t hidden, uint64_t b, const void* x, const void* w13, const void* hb );
int gemm_stream_gate_launch( __half* hb, const __half* x, const __half* w13, uint64_t s, uint64_t hidden, uint64_t b, hipStream_t st );
// 256 x 256 tile kernel for products with enough tiles (gh_gemm_tile256.hip)
bool gemm_tile256_applicable( uint64_t s, uint64_t r, uint64_t b, const void* x, const void* w, const void* xout );
int gemm_tile256_launch( __half* xout, float* partial, const __half* x, const __half* w, uint64_t s, uint64_t r, uint64_t b, int epilogue, hipStream_t st,
                         uint32_t splits, uint32_t k_len, __half* xout2 = nullptr, uint64_t r_first = 0 );
uint64_t gemm_tile256_token_split( uint64_t s, uint64_t r, uint64_t b );
void gemm_tile256_split_plan( uint64_t s, uint64_t r, uint64_t b, const void* x, const void* w, uint32_t* splits, uint32_t* k_len );
void gemm_tile256_tuning( int rows );
// large-batch (prefill) kernel (gh_gemm_tile.hip)
bool gemm_tile_applicable( uint64_t s, uint64_t r, uint64_t b, const void* x, const void* w, const void* xout );
void gemm_tile_plan( uint64_t s, uint64_t r, uint64_t b, uint32_t* splits_out, uint32_t* k_per_split_out );
int gemm_tile_launch( __half* xout, float* partial, const __half* x, const __half* w, uint64_t s, uint64_t r, uint64_t b, uint32_t splits, uint32_t k_per_split,
                      hipStream_t st );

namespace {

int g_force_kernel = 0; // 0 auto, 1 small tiled kernel of this file, 2 streaming kernel, 3 large tile kernel
// GLINT_LIBRARY_ROWS in the environment overrides the default (for the command-line profilers, which have no other way in)
uint64_t library_rows_default()
{
  const char* env = getenv( "GLINT_LIBRARY_ROWS" );
  return env != nullptr && *env != '\0' ? strtoull( env, nullptr, 10 ) : 0;
}
uint64_t g_library_rows = library_rows_default(); // 0: never; else plain products of this many rows and more go to the vendor's GEMM library (gh_gemm_set_library_rows)

typedef _Float16 f16x8 __attribute__( ( ext_vector_type( 8 ) ) );
typedef float f32x4 __attribute__( ( ext_vector_type( 4 ) ) );

constexpr int BM = 64;  // weight rows per work-group
constexpr int BN = 64;  // batch columns per work-group
constexpr int BK = 128; // k per stage (16 chunks of 8 halves)

// split-K partials: a grow-only buffer per stream, so that products queued on different streams never share one
int ensure_workspace( uint64_t bytes, float** out, hipStream_t st )
{
  void* p = nullptr;
  if ( int rc = stream_scratch( st, SCRATCH_GEMM_PARTIALS, bytes, 64ull << 20, &p ) ) {
    return rc;
  }
  *out = static_cast<float*>( p );
  return GH_OK;
}

// Loads one (64 x 128) f16 tile, rows [row0, row0+64) x k [k0, k0+128) of a row-major matrix with
// leading dimension ld, into registers: thread t handles chunk (t % 16) of rows t/16 + 16*i.
// Rows >= n_rows and k >= k_end read as zero.
struct TileRegs
{
  uint4 v[4];
};

__device__ __forceinline__ TileRegs load_tile( const __half* __restrict__ mat, uint64_t ld, uint32_t row0, uint32_t n_rows, uint32_t k0, uint32_t k_end, bool k_vec_ok )
{
  TileRegs t;
  const uint32_t chunk = threadIdx.x & 15;
  const uint32_t k = k0 + chunk * 8;
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    const uint32_t row = row0 + ( threadIdx.x >> 4 ) + 16 * i;
    uint4 v = make_uint4( 0, 0, 0, 0 );
    if ( row < n_rows && k < k_end ) {
      const __half* p = mat + (uint64_t)row * ld + k;
      if ( k_vec_ok && k + 8 <= k_end ) {
        v = *reinterpret_cast<const uint4*>( p );
      } else {
        union
        {
          uint4 raw;
          __half h[8];
        } u;
        u.raw = make_uint4( 0, 0, 0, 0 );
        for ( int e = 0; e < 8; e++ ) {
          if ( k + e < k_end ) {
            u.h[e] = p[e];
          }
        }
        v = u.raw;
      }
    }
    t.v[i] = v;
  }
  return t;
}

__device__ __forceinline__ void store_tile( uint4* lds, const TileRegs& t )
{
  const uint32_t chunk = threadIdx.x & 15;
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    const uint32_t row = ( threadIdx.x >> 4 ) + 16 * i;
    lds[row * 16 + ( chunk ^ ( row & 15 ) )] = t.v[i];
  }
}

// grid: (ceil(r / 64), ceil(b / 64), k_splits)
template<bool SPLIT>
__global__ __launch_bounds__( 256 ) void gemm_f16_kernel( __half* __restrict__ xout,
                                                          float* __restrict__ partial,
                                                          const __half* __restrict__ x,
                                                          const __half* __restrict__ w,
                                                          uint32_t s,
                                                          uint32_t r,
                                                          uint32_t b,
                                                          uint32_t k_per_split,
                                                          bool k_vec_ok )
{
  __shared__ uint4 s_w[2][BM * 16];
  __shared__ uint4 s_x[2][BN * 16];

  const uint32_t row0 = blockIdx.x * BM;
  const uint32_t col0 = blockIdx.y * BN;
  const uint32_t k_begin = blockIdx.z * k_per_split;
  const uint32_t k_end = min( s, k_begin + k_per_split );
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t g4 = lane >> 4;

  f32x4 acc[4];
#pragma unroll
  for ( int j = 0; j < 4; j++ ) {
    acc[j] = f32x4 { 0.0f, 0.0f, 0.0f, 0.0f };
  }

  TileRegs tw = load_tile( w, s, row0, r, k_begin, k_end, k_vec_ok );
  TileRegs tx = load_tile( x, s, col0, b, k_begin, k_end, k_vec_ok );
  int buf = 0;
  for ( uint32_t k0 = k_begin; k0 < k_end; k0 += BK ) {
    store_tile( s_w[buf], tw );
    store_tile( s_x[buf], tx );
    __syncthreads();
    if ( k0 + BK < k_end ) {
      tw = load_tile( w, s, row0, r, k0 + BK, k_end, k_vec_ok );
      tx = load_tile( x, s, col0, b, k0 + BK, k_end, k_vec_ok );
    }
    const uint4* lw = s_w[buf];
    const uint4* lx = s_x[buf];
    const uint32_t arow = wave * 16 + c;
#pragma unroll
    for ( int kk = 0; kk < 4; kk++ ) {
      const uint32_t ch = 4 * kk + g4;
      const f16x8 a = __builtin_bit_cast( f16x8, lw[arow * 16 + ( ch ^ ( arow & 15 ) )] );
#pragma unroll
      for ( int j = 0; j < 4; j++ ) {
        const uint32_t brow = 16 * j + c;
        const f16x8 bb = __builtin_bit_cast( f16x8, lx[brow * 16 + ( ch ^ ( brow & 15 ) )] );
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16( a, bb, acc[j], 0, 0, 0 );
      }
    }
    buf ^= 1; // the other buffer is free: its readers passed the barrier of this iteration
  }

  // acc[j][i] = out(row0 + 16*wave + 4*g4 + i, col0 + 16*j + c)
#pragma unroll
  for ( int j = 0; j < 4; j++ ) {
    const uint32_t col = col0 + 16 * j + c;
    if ( col >= b ) {
      continue;
    }
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      const uint32_t row = row0 + 16 * wave + 4 * g4 + i;
      if ( row < r ) {
        if ( SPLIT ) {
          partial[( (uint64_t)blockIdx.z * b + col ) * r + row] = acc[j][i];
        } else {
          xout[(uint64_t)col * r + row] = __float2half_rn( acc[j][i] );
        }
      }
    }
  }
}

__global__ __launch_bounds__( 256 ) void gemm_reduce_kernel( __half* __restrict__ xout, const float* __restrict__ partial, uint64_t n, uint32_t splits )
{
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for ( uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride ) {
    // ascending order of the split, four loads in flight: a split past the last reads the last again and is not added
    float sum = 0.0f;
    for ( uint32_t k0 = 0; k0 < splits; k0 += 4 ) {
      float p[4];
#pragma unroll
      for ( uint32_t u = 0; u < 4; u++ ) {
        p[u] = partial[(uint64_t)min( k0 + u, splits - 1 ) * n + i];
      }
#pragma unroll
      for ( uint32_t u = 0; u < 4; u++ ) {
        sum += k0 + u < splits ? p[u] : 0.0f;
      }
    }
    xout[i] = __float2half_rn( sum );
  }
}

// f32: one wave per weight row, batch columns looped
__global__ __launch_bounds__( 256 ) void gemm_f32_kernel( float* __restrict__ xout, const float* __restrict__ x, const float* __restrict__ w, uint32_t s, uint32_t r, uint32_t b )
{
  const uint32_t row = blockIdx.x * 4 + ( threadIdx.x >> 6 );
  if ( row >= r ) {
    return;
  }
  const uint32_t lane = threadIdx.x & 63;
  const float* wr = w + (uint64_t)row * s;
  for ( uint32_t col = 0; col < b; col++ ) {
    const float* xc = x + (uint64_t)col * s;
    float sum = 0.0f;
    for ( uint32_t p = lane; p < s; p += 64 ) {
      sum += wr[p] * xc[p];
    }
    sum = wave_sum( sum );
    if ( lane == 0 ) {
      xout[(uint64_t)col * r + row] = sum;
    }
  }
}

} // namespace
} // namespace gh

namespace gh {

// Runs the GEMM proper.  With `want_partials` the result is always left as fp32 partial sums
// `[splits][b][r]` in the library's workspace (*partial_out, *splits_out) for a fused epilogue;
// otherwise the kernel may store DType results straight into `xout` (*splits_out == 0 then).
// w1, w3 and the SiLU gate in one launch of the streaming kernel, where gemm_partials() would pick that
// kernel without a K split.  *done = false: nothing was launched, the caller takes the two-kernel route.
int gemm_gate_one_launch( void* hb, const void* x, const void* w13, uint64_t s, uint64_t hidden, uint64_t b, gh_dtype dt, hipStream_t st, bool* done )
{
  *done = false;
  if ( dt != GH_F16 || ( g_force_kernel != 0 && g_force_kernel != 2 ) || b > 64 || !gemm_stream_gate_applicable( s, hidden, b, x, w13, hb ) ) {
    return GH_OK;
  }
  *done = true;
  return gemm_stream_gate_launch( static_cast<__half*>( hb ), static_cast<const __half*>( x ), static_cast<const __half*>( w13 ), s, hidden, b, st );
}

// Tokens of the first part when a many-row product is better run as two products along the tokens (see
// gemm_tile256_token_split), 0 otherwise.
uint64_t gemm_token_split( uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, const void* x, const void* w, const void* xout )
{
  if ( dt != GH_F16 || g_force_kernel != 0 || !gemm_tile256_applicable( s, r, b, x, w, xout ) ) {
    return 0;
  }
  const uint64_t b1 = gemm_tile256_token_split( s, r, b );
  return b1 != 0 && gemm_tile256_applicable( s, r, b1, x, w, xout ) && ( b1 * r * 2 ) % 16 == 0 && ( b1 * s * 2 ) % 16 == 0 ? b1 : 0;
}

// Many rows: the large tile kernel with the op that follows the product in its epilogue, 1 = xout += product
// (accum).  *done = false: nothing was launched (shape or alignment not for that kernel), the caller takes
// its other route.
bool gemm_tile_epilogue_applicable( uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, const void* x, const void* w, const void* xout )
{
  return dt == GH_F16 && r % 8 == 0 && ( g_force_kernel == 0 || g_force_kernel == 4 ) && gemm_tile256_applicable( s, r, b, x, w, xout );
}

int gemm_tile_epilogue_launch( void* xout, const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, int epilogue, hipStream_t st,
                               bool* done )
{
  *done = false;
  if ( !gemm_tile_epilogue_applicable( s, r, b, dt, x, w, xout ) ) {
    return GH_OK;
  }
  *done = true;
  return gemm_tile256_launch( static_cast<__half*>( xout ), nullptr, static_cast<const __half*>( x ), static_cast<const __half*>( w ), s, r, b, epilogue, st, 1, 0 );
}

int gemm_partials( void* xout, const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, hipStream_t st, bool want_partials,
                   float** partial_out, uint32_t* splits_out )
{
  *partial_out = nullptr;
  *splits_out = 0;
  if ( dt == GH_F32 ) {
    float* dst = static_cast<float*>( xout );
    if ( want_partials ) {
      if ( int rc = ensure_workspace( b * r * sizeof( float ), &dst, st ) ) {
        return rc;
      }
      *partial_out = dst;
      *splits_out = 1;
    }
    gemm_f32_kernel<<<(unsigned)( ( r + 3 ) / 4 ), 256, 0, st>>>( dst, static_cast<const float*>( x ), static_cast<const float*>( w ), (uint32_t)s, (uint32_t)r,
                                                                 (uint32_t)b );
    GH_LAUNCH_CHECK();
    return GH_OK;
  }
  GH_REQUIRE( dt == GH_F16, "gh_matmul: unsupported dtype %d", (int)dt );

  // many tokens at once (prefill): the MFMA-bound tile kernel; few (decode): the weight-streaming one
  if ( ( g_force_kernel == 0 || g_force_kernel == 4 ) && gemm_tile256_applicable( s, r, b, x, w, xout ? xout : x ) ) {
    float* ws = nullptr;
    if ( want_partials ) {
      if ( int rc = ensure_workspace( b * r * sizeof( float ), &ws, st ) ) {
        return rc;
      }
      *partial_out = ws;
      *splits_out = 1;
    }
    return gemm_tile256_launch( static_cast<__half*>( xout ), ws, static_cast<const __half*>( x ), static_cast<const __half*>( w ), s, r, b, 0, st, 1, 0 );
  }
  if ( g_force_kernel == 0 || g_force_kernel == 4 ) { // some hundred rows and few tiles: the same kernel with the K range split
    uint32_t splits = 0, k_len = 0;
    gemm_tile256_split_plan( s, r, b, x, w, &splits, &k_len );
    if ( splits > 1 ) {
      float* ws = nullptr;
      if ( int rc = ensure_workspace( (uint64_t)splits * b * r * sizeof( float ), &ws, st ) ) {
        return rc;
      }
      *partial_out = ws;
      *splits_out = splits;
      return gemm_tile256_launch( nullptr, ws, static_cast<const __half*>( x ), static_cast<const __half*>( w ), s, r, b, 0, st, splits, k_len );
    }
  }
  GH_REQUIRE( g_force_kernel != 4, "gh_matmul: the 256 x 256 tile kernel needs b >= 192, at least 192 tiles with a last round that is not mostly empty, s %% 64 == 0 and 16-byte aligned operands" );
  if ( ( g_force_kernel == 0 || g_force_kernel == 3 ) && gemm_tile_applicable( s, r, b, x, w, xout ? xout : x ) ) {
    uint32_t splits = 1, k_per_split = 0;
    gemm_tile_plan( s, r, b, &splits, &k_per_split );
    float* ws = nullptr;
    if ( want_partials || splits > 1 ) {
      if ( int rc = ensure_workspace( (uint64_t)splits * b * r * sizeof( float ), &ws, st ) ) {
        return rc;
      }
      *partial_out = ws;
      *splits_out = splits;
    }
    return gemm_tile_launch( static_cast<__half*>( xout ), ws, static_cast<const __half*>( x ), static_cast<const __half*>( w ), s, r, b, splits, k_per_split, st );
  }
  GH_REQUIRE( g_force_kernel != 3, "gh_matmul: the tile kernel needs b > 64, s %% 8 == 0 and 16-byte aligned operands" );

  if ( g_force_kernel != 1 && gemm_stream_applicable( s, r, b, x, w, xout ? xout : x ) ) {
    uint32_t splits = 1, k_per_split = 0, rows_per_wg = 0;
    gemm_stream_plan( s, r, b, &splits, &k_per_split, &rows_per_wg );
    float* ws = nullptr;
    const bool partial = want_partials || splits > 1;
    if ( partial ) {
      if ( int rc = ensure_workspace( (uint64_t)splits * b * r * sizeof( float ), &ws, st ) ) {
        return rc;
      }
      *partial_out = ws;
      *splits_out = splits;
    }
    return gemm_stream_launch( static_cast<__half*>( xout ), ws, static_cast<const __half*>( x ), static_cast<const __half*>( w ), s, r, b, splits, k_per_split,
                               rows_per_wg, partial, st );
  }
  GH_REQUIRE( g_force_kernel != 2, "gh_matmul: the streaming kernel needs s %% 256 == 0, r %% 4 == 0 and 16-byte aligned operands" );

  const bool k_vec_ok = ( s % 8 == 0 ) && ( ( reinterpret_cast<uintptr_t>( x ) | reinterpret_cast<uintptr_t>( w ) ) & 15u ) == 0;
  const uint32_t grid_m = (uint32_t)( ( r + BM - 1 ) / BM );
  const uint32_t grid_n = (uint32_t)( ( b + BN - 1 ) / BN );
  GH_REQUIRE( grid_n <= 65535, "gh_matmul: batch too large" );
  // split K until there are about 1024 work-groups (4 per CU), keeping at least 1024 k per split
  uint32_t splits = 1;
  const uint64_t tiles = (uint64_t)grid_m * grid_n;
  if ( tiles < 1024 ) {
    splits = (uint32_t)( ( 1024 + tiles - 1 ) / tiles );
    const uint32_t max_by_k = (uint32_t)std::max<uint64_t>( 1, s / 1024 );
    splits = std::min( splits, max_by_k );
    splits = std::min<uint32_t>( splits, 16 );
  }
  uint32_t k_per_split = (uint32_t)( ( s + splits - 1 ) / splits );
  k_per_split = ( k_per_split + BK - 1 ) / BK * BK;
  splits = (uint32_t)( ( s + k_per_split - 1 ) / k_per_split );

  const dim3 grid( grid_m, grid_n, splits );
  if ( splits == 1 && !want_partials ) {
    gemm_f16_kernel<false><<<grid, 256, 0, st>>>( static_cast<__half*>( xout ), nullptr, static_cast<const __half*>( x ), static_cast<const __half*>( w ),
                                                 (uint32_t)s, (uint32_t)r, (uint32_t)b, k_per_split, k_vec_ok );
    GH_LAUNCH_CHECK();
    return GH_OK;
  }
  float* ws = nullptr;
  if ( int rc = ensure_workspace( (uint64_t)splits * b * r * sizeof( float ), &ws, st ) ) {
    return rc;
  }
  gemm_f16_kernel<true><<<grid, 256, 0, st>>>( nullptr, ws, static_cast<const __half*>( x ), static_cast<const __half*>( w ), (uint32_t)s, (uint32_t)r,
                                              (uint32_t)b, k_per_split, k_vec_ok );
  GH_LAUNCH_CHECK();
  *partial_out = ws;
  *splits_out = splits;
  return GH_OK;
}

} // namespace gh

namespace gh {
// whether a plain product goes to the vendor's library (gh_gemm_lib.hip)
bool gemm_library_wanted( uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, const void* x, const void* w, const void* xout )
{
  const bool aligned = ( ( reinterpret_cast<uintptr_t>( x ) | reinterpret_cast<uintptr_t>( w ) | reinterpret_cast<uintptr_t>( xout ) ) & 15u ) == 0;
  // measured (13B and 70B shapes): from g_library_rows rows on the library's kernels win nearly everywhere; below, the split-K
  // tile kernel and the two-output launch do (w1 and w3 of the 70B shape at 256 rows as two library products: the decode step
  // of 256 slots 10.07 ms against 9.84)
  // from half that row count on as well unless the weight matrix is much wider than tall (w2): measured with the residual add and
  // the norm behind the product, 384-704 rows, 4-50 % faster for every such product of the 7B, 13B and 70B shapes; for w2 the
  // split-K tile kernel keeps up
  const bool rows_enough = b >= g_library_rows || ( 2 * b >= g_library_rows && 2 * r >= s );
  return dt == GH_F16 && g_force_kernel == 0 && g_library_rows > 0 && rows_enough && s % 8 == 0 && r % 8 == 0 && aligned;
}
// a product with many weight rows (w1 and w3 together) of some hundred activation rows, below gemm_library_wanted()'s row count:
// measured on the 13B and 70B shapes, the library wins there from 128 rows on (1.1-1.6 x), which it does not for narrower products
bool gemm_library_wanted_wide( uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, const void* x, const void* w, const void* xout )
{
  const bool aligned = ( ( reinterpret_cast<uintptr_t>( x ) | reinterpret_cast<uintptr_t>( w ) | reinterpret_cast<uintptr_t>( xout ) ) & 15u ) == 0;
  return dt == GH_F16 && g_force_kernel == 0 && g_library_rows > 0 && b >= 128 && b < g_library_rows && r >= 16384 && s % 8 == 0 && r % 8 == 0 && aligned;
}
} // namespace gh

using namespace gh;

extern "C" {

int gh_gemm_set_tuning( int kernel, int target_workgroups, int tile_rows )
{
  g_force_kernel = kernel;
  gemm_stream_tuning( target_workgroups, 0 );
  gemm_tile256_tuning( tile_rows );
  return GH_OK;
}

int gh_gemm_set_gate_waves( int waves )
{
  GH_REQUIRE( waves == 0 || waves == 4 || waves == 8, "gh_gemm_set_gate_waves: %d is not 0, 4 or 8", waves );
  gemm_stream_gate_waves( waves );
  return GH_OK;
}

int gh_gemm_set_library_rows( uint64_t rows )
{
  g_library_rows = rows;
  return GH_OK;
}

uint64_t gh_gemm_library_rows( void ) { return g_library_rows; }

int gh_matmul_fuses_many_rows( uint64_t s, uint64_t r, uint64_t b, gh_dtype dt )
{
  static const char aligned[16] __attribute__( ( aligned( 16 ) ) ) = { 0 };
  return gemm_tile_epilogue_applicable( s, r, b, dt, aligned, aligned, aligned ) ? 1 : 0;
}

int gh_gemm_stream_plan( uint64_t s, uint64_t r, uint64_t b, uint32_t* splits, uint32_t* k_per_split, uint32_t* rows_per_workgroup )
{
  GH_REQUIRE( splits && k_per_split && rows_per_workgroup, "gh_gemm_stream_plan: NULL output" );
  GH_REQUIRE( s >= 256 && s % 256 == 0 && r > 0 && b > 0, "gh_gemm_stream_plan: the streaming kernel takes s %% 256 == 0, r > 0, b > 0" );
  gemm_stream_plan( s, r, b, splits, k_per_split, rows_per_workgroup );
  return GH_OK;
}

int gh_matmul_pair( void* xout_a, void* xout_b, const void* x, const void* w, uint64_t s, uint64_t r_a, uint64_t r_b, uint64_t b, gh_dtype dt,
                    gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( b == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( xout_a && xout_b && x && w, "gh_matmul_pair: NULL pointer" );
  GH_REQUIRE( dt == GH_F16 || dt == GH_F32, "gh_matmul_pair: unsupported dtype %d", (int)dt );
  const uint64_t elem = dt == GH_F16 ? 2 : 4;
  const uint64_t r = r_a + r_b;
  GH_REQUIRE( s > 0 && s <= 0x7fffffffull && r <= 0x7fffffffull && b <= 0x7fffffffull, "gh_matmul_pair: bad shape" );
  if ( r_a > 0 && r_b > 0 && gemm_library_wanted( s, r_a, b, dt, x, w, xout_a ) && gemm_library_wanted( s, r_b, b, dt, x, w, xout_b ) ) {
    if ( int rc = gh_matmul( xout_a, x, w, s, r_a, b, dt, stream ) ) { // the library's kernels cut their work finer than whole tiles
      return rc;
    }
    return gh_matmul( xout_b, x, static_cast<const char*>( w ) + r_a * s * elem, s, r_b, b, dt, stream );
  }
  // many rows: one launch of the large tile kernel whose work-groups store to the matrix their rows belong to, so that the two
  // products fill their rounds together (a product of 2048 rows alone leaves most of the chip idle)
  if ( dt == GH_F16 && g_force_kernel == 0 && r_a > 0 && r_b > 0 && r_a % 8 == 0 && r_b % 8 == 0 && gemm_tile256_applicable( s, r, b, x, w, xout_a )
       && ( reinterpret_cast<uintptr_t>( xout_b ) & 15u ) == 0 ) {
    if ( const uint64_t b1 = gemm_token_split( s, r, b, dt, x, w, xout_a ) ) {
      if ( ( b1 * r_a * elem ) % 16 == 0 && ( b1 * r_b * elem ) % 16 == 0 ) {
        if ( int rc = gh_matmul_pair( xout_a, xout_b, x, w, s, r_a, r_b, b1, dt, stream ) ) {
          return rc;
        }
        return gh_matmul_pair( static_cast<char*>( xout_a ) + b1 * r_a * elem, static_cast<char*>( xout_b ) + b1 * r_b * elem,
                               static_cast<const char*>( x ) + b1 * s * elem, w, s, r_a, r_b, b - b1, dt, stream );
      }
    }
    return gemm_tile256_launch( static_cast<__half*>( xout_a ), nullptr, static_cast<const __half*>( x ), static_cast<const __half*>( w ), s, r, b, 0,
                                as_stream( stream ), 1, 0, static_cast<__half*>( xout_b ), r_a );
  }
  if ( int rc = gh_matmul( xout_a, x, w, s, r_a, b, dt, stream ) ) {
    return rc;
  }
  return gh_matmul( xout_b, x, static_cast<const char*>( w ) + r_a * s * elem, s, r_b, b, dt, stream );
}

int gh_matmul( void* xout, const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( b == 0 || r == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( xout && x && w, "gh_matmul: NULL pointer" );
  GH_REQUIRE( s > 0 && s <= 0x7fffffffull && r <= 0x7fffffffull && b <= 0x7fffffffull, "gh_matmul: bad shape" );
  hipStream_t st = as_stream( stream );
  if ( gemm_library_wanted( s, r, b, dt, x, w, xout ) ) { // a plain product of many rows
    bool done = false;
    if ( int rc = gemm_library( xout, x, w, s, r, b, st, &done ) ) {
      return rc;
    }
    if ( done ) {
      return GH_OK;
    }
  }
  if ( const uint64_t b1 = gemm_token_split( s, r, b, dt, x, w, xout ) ) { // two products along the tokens
    const uint64_t elem = 2;
    if ( int rc = gh_matmul( xout, x, w, s, r, b1, dt, stream ) ) {
      return rc;
    }
    return gh_matmul( static_cast<char*>( xout ) + b1 * r * elem, static_cast<const char*>( x ) + b1 * s * elem, w, s, r, b - b1, dt, stream );
  }
  float* partial = nullptr;
  uint32_t splits = 0;
  if ( int rc = gemm_partials( xout, x, w, s, r, b, dt, st, false, &partial, &splits ) ) {
    return rc;
  }
  if ( splits > 0 ) { // only the f16 kernels leave partials when not asked to
    const uint64_t n = b * r;
    const unsigned blocks = (unsigned)std::min<uint64_t>( ( n + 255 ) / 256, 4096 );
    gemm_reduce_kernel<<<blocks, 256, 0, st>>>( static_cast<__half*>( xout ), partial, n, splits );
    GH_LAUNCH_CHECK();
  }
  return GH_OK;
}

} // extern "C"
