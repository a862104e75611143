// Unfused attention ops with the `att` score buffer, one kernel per method of the reference's
// interface: attention_0_gemm, attention_softmax, attention_2_gemm
// (arch/amd64/llama2/ops.hh:170-298).  They exist for op-level conformance; the stage driver uses
// the fused split-K kernel instead.
#include "gh_common.h"

namespace gh {
namespace {

constexpr int MAX_GQA = 16;

// ---- scores: thread <-> cached token, block <-> (token block, kv head, context) -------------------
template<typename T>
__global__ __launch_bounds__( 256 ) void attn_scores_kernel( const T* __restrict__ q,
                                                             const T* const* __restrict__ layer_rows,
                                                             T* __restrict__ att,
                                                             const uint32_t* __restrict__ pos,
                                                             uint32_t n_kv_heads,
                                                             uint32_t gqa,
                                                             uint32_t head_size,
                                                             uint32_t seq_len,
                                                             float scale )
{
  extern __shared__ float s_q[]; // gqa * head_size
  const uint32_t ctx = blockIdx.z;
  const uint32_t h = blockIdx.y;
  const T* base = layer_rows[ctx];
  if ( base == nullptr ) {
    return;
  }
  const uint32_t n_tok = pos[ctx] + 1;
  if ( blockIdx.x * blockDim.x >= n_tok ) {
    return;
  }
  const uint32_t n_heads = n_kv_heads * gqa;
  const T* qh = q + ( (uint64_t)ctx * n_heads + (uint64_t)h * gqa ) * head_size;
  for ( uint32_t i = threadIdx.x; i < gqa * head_size; i += blockDim.x ) {
    s_q[i] = to_f32( qh[i] );
  }
  __syncthreads();

  const uint32_t p = blockIdx.x * blockDim.x + threadIdx.x;
  if ( p >= n_tok ) {
    return;
  }
  const T* key = base + (uint64_t)p * ( 2ull * n_kv_heads * head_size ) + (uint64_t)h * head_size;
  float sums[MAX_GQA];
#pragma unroll
  for ( int g = 0; g < MAX_GQA; g++ ) {
    sums[g] = 0.0f;
  }
  for ( uint32_t d = 0; d < head_size; d++ ) {
    const float kd = to_f32( key[d] );
#pragma unroll
    for ( int g = 0; g < MAX_GQA; g++ ) {
      if ( g < (int)gqa ) {
        sums[g] += kd * s_q[g * head_size + d];
      }
    }
  }
  T* out = att + ( (uint64_t)ctx * n_heads + (uint64_t)h * gqa ) * seq_len + p;
#pragma unroll
  for ( int g = 0; g < MAX_GQA; g++ ) {
    if ( g < (int)gqa ) {
      out[(uint64_t)g * seq_len] = from_f32<T>( scale * sums[g] );
    }
  }
}

// ---- softmax over [0, pos] of one head row, block <-> (head, context) ---------------------------
// Rounding points follow the CPU path: DType max, DType difference, exp rounded to DType before the
// fp32 sum, fp32 division rounded to DType (arch/amd64/llama2/ops.hh:110-132).
template<typename T>
__global__ __launch_bounds__( 256 ) void attn_softmax_kernel( T* __restrict__ att, const uint32_t* __restrict__ pos, uint32_t n_heads, uint32_t seq_len )
{
  __shared__ float s_red[4];
  const uint32_t ctx = blockIdx.y;
  const uint32_t head = blockIdx.x;
  const uint32_t n = pos[ctx] + 1;
  T* row = att + ( (uint64_t)ctx * n_heads + head ) * seq_len;

  float mx = -INFINITY;
  for ( uint32_t i = threadIdx.x; i < n; i += blockDim.x ) {
    mx = fmaxf( mx, to_f32( row[i] ) );
  }
  mx = wave_max( mx );
  if ( threadIdx.x % WAVE == 0 ) {
    s_red[threadIdx.x / WAVE] = mx;
  }
  __syncthreads();
  mx = fmaxf( fmaxf( s_red[0], s_red[1] ), fmaxf( s_red[2], s_red[3] ) );
  __syncthreads();

  float sum = 0.0f;
  for ( uint32_t i = threadIdx.x; i < n; i += blockDim.x ) {
    const T diff = from_f32<T>( to_f32( row[i] ) - mx );
    const T e = from_f32<T>( expf( to_f32( diff ) ) );
    row[i] = e;
    sum += to_f32( e );
  }
  sum = wave_sum( sum );
  if ( threadIdx.x % WAVE == 0 ) {
    s_red[threadIdx.x / WAVE] = sum;
  }
  __syncthreads();
  sum = s_red[0] + s_red[1] + s_red[2] + s_red[3];

  // each thread re-reads only elements it wrote itself
  for ( uint32_t i = threadIdx.x; i < n; i += blockDim.x ) {
    row[i] = from_f32<T>( to_f32( row[i] ) / sum );
  }
}

// ---- weighted sum: block <-> (kv head, context); thread <-> (token slice, output dim) ------------
template<typename T>
__global__ __launch_bounds__( 256 ) void attn_pv_kernel( const T* __restrict__ att,
                                                         const T* const* __restrict__ layer_rows,
                                                         T* __restrict__ xb,
                                                         const uint32_t* __restrict__ pos,
                                                         uint32_t n_kv_heads,
                                                         uint32_t gqa,
                                                         uint32_t head_size,
                                                         uint32_t seq_len )
{
  extern __shared__ float s_acc[]; // n_slices * gqa * head_size
  const uint32_t ctx = blockIdx.y;
  const uint32_t h = blockIdx.x;
  const T* base = layer_rows[ctx];
  if ( base == nullptr ) {
    return;
  }
  const uint32_t n_tok = pos[ctx] + 1;
  const uint32_t n_heads = n_kv_heads * gqa;
  const uint32_t n_slices = blockDim.x / head_size; // host guarantees >= 1 and blockDim.x % head_size == 0
  const uint32_t d = threadIdx.x % head_size;
  const uint32_t slice = threadIdx.x / head_size;

  float acc[MAX_GQA];
#pragma unroll
  for ( int g = 0; g < MAX_GQA; g++ ) {
    acc[g] = 0.0f;
  }
  const T* a = att + ( (uint64_t)ctx * n_heads + (uint64_t)h * gqa ) * seq_len;
  const uint64_t row_elems = 2ull * n_kv_heads * head_size;
  const T* val = base + (uint64_t)n_kv_heads * head_size + (uint64_t)h * head_size + d;
  for ( uint32_t p = slice; p < n_tok; p += n_slices ) {
    const float v = to_f32( val[(uint64_t)p * row_elems] );
#pragma unroll
    for ( int g = 0; g < MAX_GQA; g++ ) {
      if ( g < (int)gqa ) {
        acc[g] += v * to_f32( a[(uint64_t)g * seq_len + p] );
      }
    }
  }
#pragma unroll
  for ( int g = 0; g < MAX_GQA; g++ ) {
    if ( g < (int)gqa ) {
      s_acc[( slice * gqa + g ) * head_size + d] = acc[g];
    }
  }
  __syncthreads();
  for ( uint32_t i = threadIdx.x; i < gqa * head_size; i += blockDim.x ) {
    float total = 0.0f;
    for ( uint32_t s = 0; s < n_slices; s++ ) {
      total += s_acc[s * gqa * head_size + i];
    }
    xb[( (uint64_t)ctx * n_heads + (uint64_t)h * gqa ) * head_size + i] = from_f32<T>( total );
  }
}

int check_shape( const gh_shape* s, uint64_t batch, const char* who )
{
  GH_REQUIRE( s != nullptr, "%s: NULL shape", who );
  GH_REQUIRE( s->n_kv_heads > 0 && s->gqa_size > 0 && s->head_size > 0 && s->seq_len > 0, "%s: zero dimension in shape", who );
  GH_REQUIRE( s->n_heads == s->n_kv_heads * s->gqa_size, "%s: n_heads != n_kv_heads * gqa_size", who );
  GH_REQUIRE( s->kv_dim == s->n_kv_heads * s->head_size, "%s: kv_dim != n_kv_heads * head_size", who );
  GH_REQUIRE( s->dim == s->n_heads * s->head_size, "%s: dim != n_heads * head_size", who );
  GH_REQUIRE( s->gqa_size <= MAX_GQA, "%s: gqa_size %u > %d", who, s->gqa_size, MAX_GQA );
  GH_REQUIRE( s->head_size <= 256, "%s: head_size %u > 256", who, s->head_size );
  GH_REQUIRE( batch <= 65535, "%s: batch too large", who );
  return GH_OK;
}

} // namespace
} // namespace gh

using namespace gh;

extern "C" {

int gh_attn_scores( const void* q, const void* const* layer_rows_dev, void* att, uint64_t batch, const uint32_t* pos_dev,
                    const gh_shape* shape, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  if ( int rc = check_shape( shape, batch, "gh_attn_scores" ) ) {
    return rc;
  }
  GH_REQUIRE( q && layer_rows_dev && att && pos_dev, "gh_attn_scores: NULL pointer" );
  const dim3 grid( ( shape->seq_len + 255 ) / 256, shape->n_kv_heads, (unsigned)batch );
  const size_t smem = (size_t)shape->gqa_size * shape->head_size * sizeof( float );
  const float scale = 1.0f / sqrtf( (float)shape->head_size );
  if ( dt == GH_F16 ) {
    attn_scores_kernel<__half><<<grid, 256, smem, as_stream( stream )>>>( static_cast<const __half*>( q ),
                                                                         reinterpret_cast<const __half* const*>( layer_rows_dev ),
                                                                         static_cast<__half*>( att ), pos_dev, shape->n_kv_heads,
                                                                         shape->gqa_size, shape->head_size, shape->seq_len, scale );
  } else if ( dt == GH_F32 ) {
    attn_scores_kernel<float><<<grid, 256, smem, as_stream( stream )>>>( static_cast<const float*>( q ),
                                                                        reinterpret_cast<const float* const*>( layer_rows_dev ),
                                                                        static_cast<float*>( att ), pos_dev, shape->n_kv_heads,
                                                                        shape->gqa_size, shape->head_size, shape->seq_len, scale );
  } else {
    return fail( GH_ERR_INVALID, "gh_attn_scores: unsupported dtype %d", (int)dt );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_attn_softmax( void* att, const uint32_t* pos_dev, uint64_t batch, const gh_shape* shape, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  if ( int rc = check_shape( shape, batch, "gh_attn_softmax" ) ) {
    return rc;
  }
  GH_REQUIRE( att && pos_dev, "gh_attn_softmax: NULL pointer" );
  const dim3 grid( shape->n_heads, (unsigned)batch );
  if ( dt == GH_F16 ) {
    attn_softmax_kernel<__half><<<grid, 256, 0, as_stream( stream )>>>( static_cast<__half*>( att ), pos_dev, shape->n_heads, shape->seq_len );
  } else if ( dt == GH_F32 ) {
    attn_softmax_kernel<float><<<grid, 256, 0, as_stream( stream )>>>( static_cast<float*>( att ), pos_dev, shape->n_heads, shape->seq_len );
  } else {
    return fail( GH_ERR_INVALID, "gh_attn_softmax: unsupported dtype %d", (int)dt );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_attn_pv( const void* att, const void* const* layer_rows_dev, void* xb, uint64_t batch, const uint32_t* pos_dev,
                const gh_shape* shape, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  if ( int rc = check_shape( shape, batch, "gh_attn_pv" ) ) {
    return rc;
  }
  GH_REQUIRE( att && layer_rows_dev && xb && pos_dev, "gh_attn_pv: NULL pointer" );
  const unsigned n_slices = 256 / shape->head_size ? 256 / shape->head_size : 1;
  const unsigned threads = n_slices * shape->head_size;
  const dim3 grid( shape->n_kv_heads, (unsigned)batch );
  const size_t smem = (size_t)n_slices * shape->gqa_size * shape->head_size * sizeof( float );
  GH_REQUIRE( smem <= 64 * 1024, "gh_attn_pv: gqa_size * head_size too large for the reduction buffer" );
  if ( dt == GH_F16 ) {
    attn_pv_kernel<__half><<<grid, threads, smem, as_stream( stream )>>>( static_cast<const __half*>( att ),
                                                                         reinterpret_cast<const __half* const*>( layer_rows_dev ),
                                                                         static_cast<__half*>( xb ), pos_dev, shape->n_kv_heads,
                                                                         shape->gqa_size, shape->head_size, shape->seq_len );
  } else if ( dt == GH_F32 ) {
    attn_pv_kernel<float><<<grid, threads, smem, as_stream( stream )>>>( static_cast<const float*>( att ),
                                                                        reinterpret_cast<const float* const*>( layer_rows_dev ),
                                                                        static_cast<float*>( xb ), pos_dev, shape->n_kv_heads,
                                                                        shape->gqa_size, shape->head_size, shape->seq_len );
  } else {
    return fail( GH_ERR_INVALID, "gh_attn_pv: unsupported dtype %d", (int)dt );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

// ---- host-table forms ---------------------------------------------------------------------------
static int stage_rows_and_pos( const void* const* rows_host, const uint32_t* pos_host, uint64_t batch, hipStream_t s,
                               const void* const** d_rows, const uint32_t** d_pos, const char* who )
{
  GH_REQUIRE( batch <= MAX_BATCH, "%s: batch %llu > %llu", who, (unsigned long long)batch, (unsigned long long)MAX_BATCH );
  void* p = nullptr;
  if ( rows_host ) {
    if ( int rc = stage_table( rows_host, batch * sizeof( void* ), s, &p ) ) {
      return rc;
    }
    *d_rows = static_cast<const void* const*>( p );
  }
  if ( pos_host ) {
    if ( int rc = stage_table( pos_host, batch * sizeof( uint32_t ), s, &p ) ) {
      return rc;
    }
    *d_pos = static_cast<const uint32_t*>( p );
  }
  return GH_OK;
}

int gh_attn_scores_host( const void* q, const void* const* layer_rows_host, void* att, uint64_t batch, const uint32_t* pos_host,
                         const gh_shape* shape, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( layer_rows_host && pos_host, "gh_attn_scores_host: NULL table" );
  const void* const* d_rows = nullptr;
  const uint32_t* d_pos = nullptr;
  StageScope scope( as_stream( stream ) );
  if ( int rc = stage_rows_and_pos( layer_rows_host, pos_host, batch, as_stream( stream ), &d_rows, &d_pos, "gh_attn_scores_host" ) ) {
    return rc;
  }
  if ( int rc = gh_attn_scores( q, d_rows, att, batch, d_pos, shape, dt, stream ) ) {
    return rc;
  }
  return scope.finish();
}

int gh_attn_softmax_host( void* att, const uint32_t* pos_host, uint64_t batch, const gh_shape* shape, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( pos_host, "gh_attn_softmax_host: NULL table" );
  const void* const* d_rows = nullptr;
  const uint32_t* d_pos = nullptr;
  StageScope scope( as_stream( stream ) );
  if ( int rc = stage_rows_and_pos( nullptr, pos_host, batch, as_stream( stream ), &d_rows, &d_pos, "gh_attn_softmax_host" ) ) {
    return rc;
  }
  if ( int rc = gh_attn_softmax( att, d_pos, batch, shape, dt, stream ) ) {
    return rc;
  }
  return scope.finish();
}

int gh_attn_pv_host( const void* att, const void* const* layer_rows_host, void* xb, uint64_t batch, const uint32_t* pos_host,
                     const gh_shape* shape, gh_dtype dt, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( layer_rows_host && pos_host, "gh_attn_pv_host: NULL table" );
  const void* const* d_rows = nullptr;
  const uint32_t* d_pos = nullptr;
  StageScope scope( as_stream( stream ) );
  if ( int rc = stage_rows_and_pos( layer_rows_host, pos_host, batch, as_stream( stream ), &d_rows, &d_pos, "gh_attn_pv_host" ) ) {
    return rc;
  }
  if ( int rc = gh_attn_pv( att, d_rows, xb, batch, d_pos, shape, dt, stream ) ) {
    return rc;
  }
  return scope.finish();
}

} // extern "C"
