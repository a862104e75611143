// Projection GEMMs fused with the ops that follow them in the reference's layer
// (models/llama2/model.hh:326-427).  The GEMM kernel leaves fp32 partial sums [splits][b][r]; one
// epilogue kernel per call sums the splits and applies the follow-up ops (w1, w3 and the SiLU gate
// are a single launch when no K split is needed), so a layer needs 9 launches instead of 21.
// Rounding points are those of the unfused sequence: every matmul result is rounded to DType first
// (the reference stores it), later math is fp32 with one rounding per store.
#include "gh_common.h"

namespace gh {

int gemm_partials( void* xout, const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, hipStream_t st, bool want_partials,
                   float** partial_out, uint32_t* splits_out );
int gemm_gate_one_launch( void* hb, const void* x, const void* w13, uint64_t s, uint64_t hidden, uint64_t b, gh_dtype dt, hipStream_t st, bool* done );
uint64_t gemm_token_split( uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, const void* x, const void* w, const void* xout );
bool gemm_tile_epilogue_applicable( uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, const void* x, const void* w, const void* xout );
int gemm_tile_epilogue_launch( void* xout, const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, int epilogue, hipStream_t st,
                               bool* done );

namespace {

// Sum over the splits in ascending order, four loads in flight at a time: a split past the last reads the last again and is not
// added, so no load sits under a branch (a load under a branch is waited for before the next is issued).
constexpr uint32_t SPLIT_BATCH = 4;
__device__ __forceinline__ float sum_splits( const float* __restrict__ partial, uint64_t idx, uint64_t n, uint32_t splits )
{
  float acc = 0.0f;
  for ( uint32_t k0 = 0; k0 < splits; k0 += SPLIT_BATCH ) {
    float p[SPLIT_BATCH];
#pragma unroll
    for ( uint32_t u = 0; u < SPLIT_BATCH; u++ ) {
      p[u] = partial[(uint64_t)min( k0 + u, splits - 1 ) * n + idx];
    }
#pragma unroll
    for ( uint32_t u = 0; u < SPLIT_BATCH; u++ ) {
      acc += k0 + u < splits ? p[u] : 0.0f;
    }
  }
  return acc;
}
// two neighbouring columns, idx even and the partials 8-byte aligned
__device__ __forceinline__ float2 sum_splits2( const float* __restrict__ partial, uint64_t idx, uint64_t n, uint32_t splits )
{
  float2 acc = make_float2( 0.0f, 0.0f );
  for ( uint32_t k0 = 0; k0 < splits; k0 += SPLIT_BATCH ) {
    float2 p[SPLIT_BATCH];
#pragma unroll
    for ( uint32_t u = 0; u < SPLIT_BATCH; u++ ) {
      p[u] = *reinterpret_cast<const float2*>( partial + (uint64_t)min( k0 + u, splits - 1 ) * n + idx );
    }
#pragma unroll
    for ( uint32_t u = 0; u < SPLIT_BATCH; u++ ) {
      acc.x += k0 + u < splits ? p[u].x : 0.0f;
      acc.y += k0 + u < splits ? p[u].y : 0.0f;
    }
  }
  return acc;
}

// residual(b, r) += DType(matmul); optionally norm_out = rmsnorm(residual) * norm_weight.
// block <-> batch row, 1024 threads, four columns per thread and pass so that a row's partials are
// fetched with independent 16-byte loads (the kernel is latency-bound: only `b` blocks exist)
constexpr int EPI_THREADS = 1024;

template<typename T>
__global__ __launch_bounds__( EPI_THREADS ) void epi_accum_norm_kernel( T* __restrict__ residual,
                                                                       const float* __restrict__ partial,
                                                                       uint32_t r,
                                                                       uint32_t b,
                                                                       uint32_t splits,
                                                                       T* __restrict__ norm_out,
                                                                       const T* __restrict__ norm_weight )
{
  __shared__ float smem[EPI_THREADS / WAVE];
  const uint32_t row = blockIdx.x;
  const uint64_t n = (uint64_t)b * r;
  T* res = residual + (uint64_t)row * r;
  const float* prow = partial + (uint64_t)row * r;
  const bool vec = ( r % 4 == 0 ) && ( ( reinterpret_cast<uintptr_t>( res ) & 7u ) == 0 );
  float ss = 0.0f;
  if ( vec ) {
    for ( uint32_t j = threadIdx.x * 4; j < r; j += blockDim.x * 4 ) {
      float4 acc = make_float4( 0.0f, 0.0f, 0.0f, 0.0f );
      for ( uint32_t k = 0; k < splits; k++ ) {
        const float4 p = *reinterpret_cast<const float4*>( prow + (uint64_t)k * n + j );
        acc.x += p.x;
        acc.y += p.y;
        acc.z += p.z;
        acc.w += p.w;
      }
      const float y[4] = { acc.x, acc.y, acc.z, acc.w };
#pragma unroll
      for ( int e = 0; e < 4; e++ ) {
        const T v = from_f32<T>( to_f32( res[j + e] ) + to_f32( from_f32<T>( y[e] ) ) ); // xb2 = DType(matmul), then accum
        res[j + e] = v;
        const float f = to_f32( v );
        ss += f * f;
      }
    }
  } else {
    for ( uint32_t j = threadIdx.x; j < r; j += blockDim.x ) {
      const T y = from_f32<T>( sum_splits( partial, (uint64_t)row * r + j, n, splits ) );
      const T v = from_f32<T>( to_f32( res[j] ) + to_f32( y ) );
      res[j] = v;
      const float f = to_f32( v );
      ss += f * f;
    }
  }
  if ( norm_out == nullptr ) {
    return;
  }
  ss = wave_sum( ss );
  if ( threadIdx.x % WAVE == 0 ) {
    smem[threadIdx.x / WAVE] = ss;
  }
  __syncthreads();
  ss = 0.0f;
  for ( int w = 0; w < EPI_THREADS / WAVE; w++ ) {
    ss += smem[w];
  }
  ss = ss / (float)r + 1e-5f;
  const float inv = 1.0f / sqrtf( ss );
  T* o = norm_out + (uint64_t)row * r;
  // each thread re-reads only what it wrote itself
  if ( vec ) {
    for ( uint32_t j = threadIdx.x * 4; j < r; j += blockDim.x * 4 ) {
#pragma unroll
      for ( int e = 0; e < 4; e++ ) {
        o[j + e] = from_f32<T>( to_f32( norm_weight[j + e] ) * ( inv * to_f32( res[j + e] ) ) );
      }
    }
  } else {
    for ( uint32_t j = threadIdx.x; j < r; j += blockDim.x ) {
      o[j] = from_f32<T>( to_f32( norm_weight[j] ) * ( inv * to_f32( res[j] ) ) );
    }
  }
}

// The same for rows of at most 8192 f16 elements (r % 4 == 0, 8-byte aligned rows): a thread owns
// two groups of four columns for the whole kernel.  Every load -- partials, residual, norm weight --
// is issued before the first use, and the updated residual stays in registers across the row
// reduction, so the kernel is two memory round trips deep instead of four.
__global__ __launch_bounds__( EPI_THREADS ) void epi_accum_norm_row8k_kernel( __half* __restrict__ residual,
                                                                             const float* __restrict__ partial,
                                                                             uint32_t r,
                                                                             uint32_t b,
                                                                             uint32_t splits,
                                                                             __half* __restrict__ norm_out,
                                                                             const __half* __restrict__ norm_weight )
{
  __shared__ float smem[EPI_THREADS / WAVE];
  const uint32_t row = blockIdx.x;
  const uint64_t n = (uint64_t)b * r;
  __half* res = residual + (uint64_t)row * r;
  const float* prow = partial + (uint64_t)row * r;
  union H4
  {
    uint2 raw;
    __half h[4];
  };
  float4 acc[2];
  H4 old[2], nw[2];
  bool live[2];
  uint32_t col[2];
  // A column group past the row's end reads group 0 instead and stores nothing: loads without a branch around them can all be in
  // flight together, loads under a branch are waited for one by one.
#pragma unroll
  for ( int it = 0; it < 2; it++ ) {
    const uint32_t j = ( it * EPI_THREADS + threadIdx.x ) * 4;
    live[it] = j < r;
    col[it] = live[it] ? j : 0;
    acc[it] = make_float4( 0.0f, 0.0f, 0.0f, 0.0f );
    old[it].raw = *reinterpret_cast<const uint2*>( res + col[it] );
    nw[it].raw = *reinterpret_cast<const uint2*>( ( norm_out != nullptr ? norm_weight : res ) + col[it] );
  }
  // Partial sums four splits at a time, eight loads in flight; a split past the last reads the last again and is not added.  Added in
  // ascending order of the split, as one at a time would.
  constexpr uint32_t BATCH = 4;
  for ( uint32_t k0 = 0; k0 < splits; k0 += BATCH ) {
    float4 p[BATCH][2];
#pragma unroll
    for ( uint32_t u = 0; u < BATCH; u++ ) {
      const uint32_t k = min( k0 + u, splits - 1 );
#pragma unroll
      for ( int it = 0; it < 2; it++ ) {
        p[u][it] = *reinterpret_cast<const float4*>( prow + (uint64_t)k * n + col[it] );
      }
    }
#pragma unroll
    for ( uint32_t u = 0; u < BATCH; u++ ) {
      const bool use = k0 + u < splits;
#pragma unroll
      for ( int it = 0; it < 2; it++ ) {
        acc[it].x += use ? p[u][it].x : 0.0f;
        acc[it].y += use ? p[u][it].y : 0.0f;
        acc[it].z += use ? p[u][it].z : 0.0f;
        acc[it].w += use ? p[u][it].w : 0.0f;
      }
    }
  }
  float ss = 0.0f;
  float v[2][4];
#pragma unroll
  for ( int it = 0; it < 2; it++ ) {
    const float y[4] = { acc[it].x, acc[it].y, acc[it].z, acc[it].w };
    H4 o;
#pragma unroll
    for ( int e = 0; e < 4; e++ ) {
      o.h[e] = __float2half_rn( __half2float( old[it].h[e] ) + __half2float( __float2half_rn( y[e] ) ) ); // xb2 = DType(matmul), then accum
      v[it][e] = live[it] ? __half2float( o.h[e] ) : 0.0f; // a group past the row's end holds group 0's values: not part of the norm
      ss += v[it][e] * v[it][e];
    }
    if ( live[it] ) {
      *reinterpret_cast<uint2*>( res + ( it * EPI_THREADS + threadIdx.x ) * 4 ) = o.raw;
    }
  }
  if ( norm_out == nullptr ) {
    return;
  }
  ss = wave_sum( ss );
  if ( threadIdx.x % WAVE == 0 ) {
    smem[threadIdx.x / WAVE] = ss;
  }
  __syncthreads();
  ss = 0.0f;
  for ( int w = 0; w < EPI_THREADS / WAVE; w++ ) {
    ss += smem[w];
  }
  ss = ss / (float)r + 1e-5f;
  const float inv = 1.0f / sqrtf( ss );
  __half* o = norm_out + (uint64_t)row * r;
#pragma unroll
  for ( int it = 0; it < 2; it++ ) {
    if ( live[it] ) {
      H4 out;
#pragma unroll
      for ( int e = 0; e < 4; e++ ) {
        out.h[e] = __float2half_rn( __half2float( nw[it].h[e] ) * ( inv * v[it][e] ) );
      }
      *reinterpret_cast<uint2*>( o + ( it * EPI_THREADS + threadIdx.x ) * 4 ) = out.raw;
    }
  }
}

// residual(b, r) += product(b, r), both f16 (the product already rounded, as a library GEMM leaves it), and the norm of the new
// residual in the same pass: accum and rmsnorm of the reference in one kernel, one read of each operand.  Rows of at most 8192
// elements, r % 4 == 0, 8-byte aligned rows.
__global__ __launch_bounds__( EPI_THREADS ) void accum_norm_row8k_kernel( __half* __restrict__ residual,
                                                                         const __half* __restrict__ product,
                                                                         uint32_t r,
                                                                         __half* __restrict__ norm_out,
                                                                         const __half* __restrict__ norm_weight )
{
  __shared__ float smem[EPI_THREADS / WAVE];
  const uint32_t row = blockIdx.x;
  __half* res = residual + (uint64_t)row * r;
  const __half* prod = product + (uint64_t)row * r;
  union H4
  {
    uint2 raw;
    __half h[4];
  };
  H4 old[2], add[2], nw[2];
  bool live[2];
  uint32_t col[2];
#pragma unroll
  for ( int it = 0; it < 2; it++ ) { // a column group past the row's end reads group 0 and stores nothing: no load under a branch
    const uint32_t j = ( it * EPI_THREADS + threadIdx.x ) * 4;
    live[it] = j < r;
    col[it] = live[it] ? j : 0;
    old[it].raw = *reinterpret_cast<const uint2*>( res + col[it] );
    add[it].raw = *reinterpret_cast<const uint2*>( prod + col[it] );
    nw[it].raw = *reinterpret_cast<const uint2*>( norm_weight + col[it] );
  }
  float ss = 0.0f;
  float v[2][4];
#pragma unroll
  for ( int it = 0; it < 2; it++ ) {
    H4 o;
#pragma unroll
    for ( int e = 0; e < 4; e++ ) {
      o.h[e] = __float2half_rn( __half2float( old[it].h[e] ) + __half2float( add[it].h[e] ) );
      v[it][e] = live[it] ? __half2float( o.h[e] ) : 0.0f;
      ss += v[it][e] * v[it][e];
    }
    if ( live[it] ) {
      *reinterpret_cast<uint2*>( res + col[it] ) = o.raw;
    }
  }
  ss = wave_sum( ss );
  if ( threadIdx.x % WAVE == 0 ) {
    smem[threadIdx.x / WAVE] = ss;
  }
  __syncthreads();
  ss = 0.0f;
  for ( int w = 0; w < EPI_THREADS / WAVE; w++ ) {
    ss += smem[w];
  }
  ss = ss / (float)r + 1e-5f;
  const float inv = 1.0f / sqrtf( ss );
  __half* o = norm_out + (uint64_t)row * r;
#pragma unroll
  for ( int it = 0; it < 2; it++ ) {
    if ( live[it] ) {
      H4 out;
#pragma unroll
      for ( int e = 0; e < 4; e++ ) {
        out.h[e] = __float2half_rn( __half2float( nw[it].h[e] ) * ( inv * v[it][e] ) );
      }
      *reinterpret_cast<uint2*>( o + col[it] ) = out.raw;
    }
  }
}

// hb(b, hidden) = DType( silu(y1) * y3 ) with y1 | y3 the two halves of each row of `both` (b, 2 hidden), f16 and already rounded:
// the gate behind one product of [w1; w3].  hidden % 8 == 0, 16-byte aligned.
__global__ __launch_bounds__( 256 ) void silu_gate_rows_kernel( __half* __restrict__ hb, const __half* __restrict__ both, uint32_t hidden, uint64_t b )
{
  union V8
  {
    uint4 raw;
    __half h[8];
  };
  const uint32_t per_row = hidden / 8;
  const uint64_t total = b * per_row;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for ( uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride ) {
    const uint64_t row = i / per_row, j = i % per_row;
    const uint4* src = reinterpret_cast<const uint4*>( both + row * 2 * hidden );
    V8 y1, y3, o;
    y1.raw = src[j];
    y3.raw = src[per_row + j];
#pragma unroll
    for ( int e = 0; e < 8; e++ ) {
      const float x = __half2float( y1.h[e] );
      o.h[e] = __float2half_rn( x / ( 1.0f + __expf( -x ) ) * __half2float( y3.h[e] ) );
    }
    reinterpret_cast<uint4*>( hb + row * hidden )[j] = o.raw;
  }
}

// hb(b, hidden) = DType( silu(DType(y1)) * DType(y3) ), partial rows [0, hidden) = w1, [hidden, 2 hidden) = w3
template<typename T>
__global__ __launch_bounds__( 256 ) void epi_silu_gate_kernel( T* __restrict__ hb, const float* __restrict__ partial, uint32_t hidden, uint32_t b, uint32_t splits )
{
  const uint64_t n = (uint64_t)b * 2 * hidden;
  const uint64_t total = (uint64_t)b * hidden;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for ( uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride ) {
    const uint64_t row = i / hidden, j = i % hidden;
    const float x = to_f32( from_f32<T>( sum_splits( partial, row * 2 * hidden + j, n, splits ) ) );
    const float y = to_f32( from_f32<T>( sum_splits( partial, row * 2 * hidden + hidden + j, n, splits ) ) );
    hb[i] = from_f32<T>( x / ( 1.0f + __expf( -x ) ) * y );
  }
}

// partial rows: [0, dim) q, [dim, dim + kv_dim) k, [dim + kv_dim, dim + 2 kv_dim) v.  thread <-> pair of columns.
// q(b, dim) = rope(DType(q)); cache row = [rope(DType(k)) | DType(v)]; kv_out (optional) = [DType(k) | DType(v)] unrotated
template<typename T>
__global__ __launch_bounds__( 256 ) void epi_qkv_kernel( T* __restrict__ q,
                                                        T* __restrict__ kv_out,
                                                        const float* __restrict__ partial,
                                                        uint32_t b,
                                                        uint32_t splits,
                                                        const uint32_t* __restrict__ pos,
                                                        const T* __restrict__ freq_real,
                                                        const T* __restrict__ freq_imag,
                                                        void* const* __restrict__ token_rows,
                                                        uint32_t dim,
                                                        uint32_t kv_dim,
                                                        uint32_t head_size )
{
  const uint32_t ctx = blockIdx.y;
  const uint32_t r = dim + 2 * kv_dim;
  const uint64_t n = (uint64_t)b * r;
  const uint32_t pair = blockIdx.x * blockDim.x + threadIdx.x;
  if ( pair >= r / 2 ) {
    return;
  }
  const uint32_t col = 2 * pair;
  const float2 y = sum_splits2( partial, (uint64_t)ctx * r + col, n, splits ); // r and n are even: 8-byte aligned
  const T y0 = from_f32<T>( y.x );
  const T y1 = from_f32<T>( y.y );
  T* row = static_cast<T*>( token_rows[ctx] );

  if ( kv_out != nullptr && col >= dim ) {
    kv_out[(uint64_t)ctx * 2 * kv_dim + ( col - dim )] = y0;
    kv_out[(uint64_t)ctx * 2 * kv_dim + ( col - dim ) + 1] = y1;
  }
  if ( col >= dim + kv_dim ) { // V: stored as is
    if ( row != nullptr ) {
      row[col - dim] = y0;
      row[col - dim + 1] = y1;
    }
    return;
  }
  // q and k rotate by the angle of (position, pair index inside the head); an empty context keeps its
  // query unrotated and has no row, as in the unfused ops
  T o0 = y0, o1 = y1;
  if ( row != nullptr ) {
    const uint32_t k = ( col % head_size ) / 2;
    const uint64_t p = pos[ctx];
    const float fcr = to_f32( freq_real[p * ( head_size / 2 ) + k] );
    const float fci = to_f32( freq_imag[p * ( head_size / 2 ) + k] );
    const float a = to_f32( y0 ), c = to_f32( y1 );
    o0 = from_f32<T>( a * fcr - c * fci );
    o1 = from_f32<T>( a * fci + c * fcr );
  }
  if ( col < dim ) {
    q[(uint64_t)ctx * dim + col] = o0;
    q[(uint64_t)ctx * dim + col + 1] = o1;
  } else if ( row != nullptr ) {
    row[col - dim] = o0;
    row[col - dim + 1] = o1;
  }
}

int check_common( const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, gh_dtype dt, const char* who )
{
  GH_REQUIRE( x && w, "%s: NULL pointer", who );
  GH_REQUIRE( dt == GH_F16 || dt == GH_F32, "%s: unsupported dtype %d", who, (int)dt );
  GH_REQUIRE( s > 0 && s <= 0x7fffffffull && r > 0 && r <= 0x7fffffffull && b <= 65535, "%s: bad shape", who );
  return GH_OK;
}

} // namespace
} // namespace gh

using namespace gh;

extern "C" {

int gh_matmul_accum( void* residual, const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, void* norm_out, const void* norm_weight,
                     gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( b == 0 ) {
    return GH_OK;
  }
  if ( int rc = check_common( x, w, s, r, b, dt, "gh_matmul_accum" ) ) {
    return rc;
  }
  GH_REQUIRE( residual != nullptr, "gh_matmul_accum: NULL residual" );
  GH_REQUIRE( ( norm_out == nullptr ) == ( norm_weight == nullptr ), "gh_matmul_accum: norm_out and norm_weight go together" );
  hipStream_t st = as_stream( stream );
  bool done = false;
  // many rows (prompt tokens), the product by the vendor's library where the dispatcher sends plain products there: the rounded
  // product, then the reference's own next ops on it (accum, rmsnorm) -- the same roundings as fused
  if ( gemm_library_wanted( s, r, b, dt, x, w, residual ) && gemm_library_available( s, r, b ) ) { // the product's buffer only when it will be used
    void* product = nullptr;
    if ( int rc = stream_scratch( st, SCRATCH_PRODUCT, b * r * sizeof( __half ), 64ull << 20, &product ) ) {
      return rc;
    }
    if ( int rc = gemm_library( product, x, w, s, r, b, st, &done ) ) {
      return rc;
    }
    if ( done ) {
      const bool rows_8byte
        = ( ( reinterpret_cast<uintptr_t>( residual ) | reinterpret_cast<uintptr_t>( norm_out ) | reinterpret_cast<uintptr_t>( norm_weight ) ) & 7u ) == 0;
      if ( norm_out != nullptr && r % 4 == 0 && r <= 2 * 4 * EPI_THREADS && rows_8byte && b <= 0x7fffffffull ) {
        accum_norm_row8k_kernel<<<(unsigned)b, EPI_THREADS, 0, st>>>( static_cast<__half*>( residual ), static_cast<const __half*>( product ), (uint32_t)r,
                                                                     static_cast<__half*>( norm_out ), static_cast<const __half*>( norm_weight ) );
        GH_LAUNCH_CHECK();
        return GH_OK;
      }
      if ( int rc = gh_accum( residual, product, r, b, dt, stream ) ) {
        return rc;
      }
      return norm_out != nullptr ? gh_rmsnorm( norm_out, residual, norm_weight, r, b, dt, stream ) : GH_OK;
    }
  }
  if ( const uint64_t b1 = gemm_token_split( s, r, b, dt, x, w, residual ) ) { // two products along the tokens (rows are independent)
    const uint64_t elem = 2;
    if ( int rc = gh_matmul_accum( residual, x, w, s, r, b1, norm_out, norm_weight, dt, stream ) ) {
      return rc;
    }
    return gh_matmul_accum( static_cast<char*>( residual ) + b1 * r * elem, static_cast<const char*>( x ) + b1 * s * elem, w, s, r, b - b1,
                            norm_out ? static_cast<char*>( norm_out ) + b1 * r * elem : nullptr, norm_weight, dt, stream );
  }
  // many rows: the residual is added in the tile kernel's epilogue, no fp32 partials;
  // the norm of the new residual, when asked for, is the plain row kernel
  done = false;
  if ( int rc = gemm_tile_epilogue_launch( residual, x, w, s, r, b, dt, 1, st, &done ) ) {
    return rc;
  }
  if ( done ) {
    return norm_out != nullptr ? gh_rmsnorm( norm_out, residual, norm_weight, r, b, dt, stream ) : GH_OK;
  }
  float* partial = nullptr;
  uint32_t splits = 0;
  if ( int rc = gemm_partials( nullptr, x, w, s, r, b, dt, st, true, &partial, &splits ) ) {
    return rc;
  }
  const bool rows_8byte = ( ( reinterpret_cast<uintptr_t>( residual ) | reinterpret_cast<uintptr_t>( norm_out ) | reinterpret_cast<uintptr_t>( norm_weight ) ) & 7u ) == 0;
  if ( dt == GH_F16 && r % 4 == 0 && r <= 2 * 4 * EPI_THREADS && rows_8byte ) {
    epi_accum_norm_row8k_kernel<<<(unsigned)b, EPI_THREADS, 0, st>>>( static_cast<__half*>( residual ), partial, (uint32_t)r, (uint32_t)b, splits,
                                                                     static_cast<__half*>( norm_out ), static_cast<const __half*>( norm_weight ) );
  } else if ( dt == GH_F16 ) {
    epi_accum_norm_kernel<__half><<<(unsigned)b, EPI_THREADS, 0, st>>>( static_cast<__half*>( residual ), partial, (uint32_t)r, (uint32_t)b, splits,
                                                               static_cast<__half*>( norm_out ), static_cast<const __half*>( norm_weight ) );
  } else {
    epi_accum_norm_kernel<float><<<(unsigned)b, EPI_THREADS, 0, st>>>( static_cast<float*>( residual ), partial, (uint32_t)r, (uint32_t)b, splits,
                                                              static_cast<float*>( norm_out ), static_cast<const float*>( norm_weight ) );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_matmul_silu_gate( void* hb, const void* x, const void* w13, uint64_t s, uint64_t hidden_dim, uint64_t b, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( b == 0 ) {
    return GH_OK;
  }
  if ( int rc = check_common( x, w13, s, 2 * hidden_dim, b, dt, "gh_matmul_silu_gate" ) ) {
    return rc;
  }
  GH_REQUIRE( hb != nullptr, "gh_matmul_silu_gate: NULL output" );
  hipStream_t st = as_stream( stream );
  bool done = false;
  if ( int rc = gemm_gate_one_launch( hb, x, w13, s, hidden_dim, b, dt, st, &done ) ) {
    return rc;
  }
  if ( done ) {
    return GH_OK;
  }
  // Some hundred rows, short of where every plain product goes to the vendor's library: [w1; w3] as one product of that library, whose
  // kernels cut a wide product finer than whole tiles (70B shape, 256 rows: 207 us against 262 for the route below), then the gate
  // over the two halves of each row.  The same roundings: each factor to DType, then the gate.
  if ( gemm_library_wanted_wide( s, 2 * hidden_dim, b, dt, x, w13, hb ) && hidden_dim % 8 == 0 && gemm_library_available( s, 2 * hidden_dim, b ) ) {
    void* both = nullptr;
    if ( int rc = stream_scratch( st, SCRATCH_PRODUCT, b * 2 * hidden_dim * sizeof( __half ), 64ull << 20, &both ) ) {
      return rc;
    }
    if ( int rc = gemm_library( both, x, w13, s, 2 * hidden_dim, b, st, &done ) ) {
      return rc;
    }
    if ( done ) {
      const uint64_t total = b * hidden_dim / 8;
      silu_gate_rows_kernel<<<(unsigned)std::min<uint64_t>( ( total + 255 ) / 256, 8192 ), 256, 0, st>>>( static_cast<__half*>( hb ), static_cast<const __half*>( both ),
                                                                                                          (uint32_t)hidden_dim, b );
      GH_LAUNCH_CHECK();
      return GH_OK;
    }
  }
  // Some hundred rows and more with enough tiles for the large tile kernel: both factors in one launch of it, stored as DType whole
  // row segments (the second factor into a scratch buffer), then the gate as the element-wise kernel.  The fp32 sums that the
  // route below leaves for its gate kernel are stored from the accumulator registers, 16 bytes to each of 32 lines per
  // instruction, and are twice the bytes: at 256 rows of the 70B shape 277 + 19 us against 257 + 12.  Same roundings either way
  // (each factor to DType, then the gate).
  if ( dt == GH_F16 && hidden_dim % 8 == 0
       && ( gemm_tile_epilogue_applicable( s, 2 * hidden_dim, b, dt, x, w13, hb ) || gemm_library_wanted( s, hidden_dim, b, dt, x, w13, hb ) ) ) {
    void* factor = nullptr;
    if ( int rc = stream_scratch( st, SCRATCH_GATE_FACTOR, b * hidden_dim * sizeof( __half ), 16ull << 20, &factor ) ) {
      return rc;
    }
    if ( int rc = gh_matmul_pair( hb, factor, x, w13, s, hidden_dim, hidden_dim, b, dt, stream ) ) {
      return rc;
    }
    return gh_silu( hb, factor, hidden_dim, b, dt, stream );
  }
  float* partial = nullptr;
  uint32_t splits = 0;
  if ( int rc = gemm_partials( nullptr, x, w13, s, 2 * hidden_dim, b, dt, st, true, &partial, &splits ) ) {
    return rc;
  }
  const uint64_t total = b * hidden_dim;
  const unsigned blocks = (unsigned)std::min<uint64_t>( ( total + 255 ) / 256, 8192 );
  if ( dt == GH_F16 ) {
    epi_silu_gate_kernel<__half><<<blocks, 256, 0, st>>>( static_cast<__half*>( hb ), partial, (uint32_t)hidden_dim, (uint32_t)b, splits );
  } else {
    epi_silu_gate_kernel<float><<<blocks, 256, 0, st>>>( static_cast<float*>( hb ), partial, (uint32_t)hidden_dim, (uint32_t)b, splits );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_matmul_qkv_rope_append( void* q, void* kv_out, const void* x, const void* wqkv, uint64_t s, uint64_t b, const uint32_t* pos_dev, const void* freq_real,
                               const void* freq_imag, void* const* token_rows_dev, uint32_t n_kv_heads, uint32_t gqa_size, uint32_t head_size, gh_dtype dt,
                               gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( b == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( n_kv_heads > 0 && gqa_size > 0 && head_size > 0 && head_size % 2 == 0, "gh_matmul_qkv_rope_append: bad head shape" );
  const uint64_t kv_dim = (uint64_t)n_kv_heads * head_size;
  const uint64_t dim = kv_dim * gqa_size;
  const uint64_t r = dim + 2 * kv_dim;
  if ( int rc = check_common( x, wqkv, s, r, b, dt, "gh_matmul_qkv_rope_append" ) ) {
    return rc;
  }
  GH_REQUIRE( q && pos_dev && freq_real && freq_imag && token_rows_dev, "gh_matmul_qkv_rope_append: NULL pointer" );
  hipStream_t st = as_stream( stream );
  float* partial = nullptr;
  uint32_t splits = 0;
  if ( int rc = gemm_partials( nullptr, x, wqkv, s, r, b, dt, st, true, &partial, &splits ) ) {
    return rc;
  }
  const dim3 grid( (unsigned)( ( r / 2 + 255 ) / 256 ), (unsigned)b );
  if ( dt == GH_F16 ) {
    epi_qkv_kernel<__half><<<grid, 256, 0, st>>>( static_cast<__half*>( q ), static_cast<__half*>( kv_out ), partial, (uint32_t)b, splits, pos_dev,
                                                 static_cast<const __half*>( freq_real ), static_cast<const __half*>( freq_imag ), token_rows_dev, (uint32_t)dim,
                                                 (uint32_t)kv_dim, head_size );
  } else {
    epi_qkv_kernel<float><<<grid, 256, 0, st>>>( static_cast<float*>( q ), static_cast<float*>( kv_out ), partial, (uint32_t)b, splits, pos_dev,
                                                static_cast<const float*>( freq_real ), static_cast<const float*>( freq_imag ), token_rows_dev, (uint32_t)dim,
                                                (uint32_t)kv_dim, head_size );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

} // extern "C"
