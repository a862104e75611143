// Batched prefill attention: T new tokens per context at positions [start_i, start_i + T), all of
// whose [K | V] rows are already in the cache; query token t attends keys [0, start_i + t] (causal).
// The reference has no multi-token path (it feeds prompts one token per forward,
// frontend/infer.cc:124-125, models/llama2/model.hh:356-357); the result of this kernel equals T
// sequential calls of the decode path.
//
// f16, head size 128: MFMA kernel.  A wave owns 16 query columns of one (context, kv head): 16/gqa
// consecutive tokens x the gqa query heads that share the kv head.  It streams the keys in tiles of
// 16 exactly like the decode kernel (K through a wave-private swizzled LDS tile into
// v_mfma_f32_16x16x32_f16 operand order, S^T lands in the A-operand order of
// v_mfma_f32_16x16x16_f16, V transposed in registers), with a per-column causal mask.  The four
// waves of a block take neighbouring query groups and need almost the same keys: the block streams
// them once, 64 keys per step into an LDS stage (every wave fetches a quarter, the next step's rows
// are in flight in registers meanwhile), and each wave works through the four 16-key tiles of the
// stage that its queries can see.  Four blocks per CU: the per-tile chain of MFMA, softmax and
// shuffles is latency-bound, so occupancy matters more than the 4 spilled registers it costs.
//
// Any other shape: the decode kernels are run on tables expanded to one entry per (context, token).
#include "gh_common.h"

namespace gh {
namespace {

constexpr float LOG2E = 1.4426950408889634f;
constexpr int HS = 128;
#ifndef PF_WGS_PER_CU
#define PF_WGS_PER_CU 4
#endif

typedef _Float16 f16x4 __attribute__( ( ext_vector_type( 4 ) ) );
typedef _Float16 f16x8 __attribute__( ( ext_vector_type( 8 ) ) );
typedef float f32x4 __attribute__( ( ext_vector_type( 4 ) ) );

__device__ __forceinline__ float fast_exp2( float x ) { return __builtin_amdgcn_exp2f( x ); }
__device__ __forceinline__ uint4 load16( const __half* p ) { return *reinterpret_cast<const uint4*>( p ); }

// one entry per (context, token): the decode-style tables of a prefill step
__global__ __launch_bounds__( 256 ) void expand_tables_kernel( const void* const* __restrict__ layer_rows,
                                                               const uint32_t* __restrict__ start_pos,
                                                               uint32_t batch,
                                                               uint32_t n_tokens,
                                                               uint64_t row_bytes,
                                                               const void** __restrict__ layer_rows_out,
                                                               void** __restrict__ token_rows_out,
                                                               uint32_t* __restrict__ pos_out )
{
  const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
  if ( idx >= batch * n_tokens ) {
    return;
  }
  const uint32_t i = idx / n_tokens, t = idx % n_tokens;
  const uint8_t* base = static_cast<const uint8_t*>( layer_rows[i] );
  const uint32_t p = start_pos[i] + t;
  if ( layer_rows_out ) {
    layer_rows_out[idx] = base;
  }
  if ( token_rows_out ) {
    token_rows_out[idx] = base ? const_cast<uint8_t*>( base ) + (uint64_t)p * row_bytes : nullptr;
  }
  if ( pos_out ) {
    pos_out[idx] = p;
  }
}

// q, xb: (batch * n_tokens, n_kv_heads * G * 128), row index = context * n_tokens + token
template<int G>
__global__ __launch_bounds__( 256, PF_WGS_PER_CU ) void attn_prefill_mfma_kernel( const __half* __restrict__ q,
                                                                   const __half* const* __restrict__ layer_rows,
                                                                   const uint32_t* __restrict__ start_pos,
                                                                   __half* __restrict__ xb,
                                                                   uint32_t n_kv_heads,
                                                                   uint32_t n_tokens,
                                                                   uint32_t groups_per_head, // ceil(n_tokens / (16 / G))
                                                                   float scale_log2e )
{
  __shared__ uint4 s_kt[64 * 16]; // 64 keys x 256 bytes, 16-byte chunks XOR-swizzled per 16-key tile
  __shared__ uint4 s_vt[64 * 16]; // the same keys' value rows, plain
  constexpr uint32_t TPG = 16 / G; // tokens per query group

  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t g4 = lane >> 4;
  // block -> (group quad, kv head, context); wave -> group inside the quad
  const uint32_t quads = ( groups_per_head + 3 ) / 4;
  uint32_t bid = blockIdx.x;
  const uint32_t quad = bid % quads;
  bid /= quads;
  const uint32_t h = bid % n_kv_heads;
  const uint32_t ctx = bid / n_kv_heads;
  const uint32_t group = quad * 4 + wave;
  const __half* base = layer_rows[ctx];
  if ( base == nullptr ) {
    return; // the whole work-group
  }
  const bool wave_ok = group < groups_per_head; // a wave without queries still loads its share of every tile
  const uint32_t n_heads = n_kv_heads * G;
  const uint64_t row_elems = 2ull * n_kv_heads * HS;
  const uint32_t v_off = n_kv_heads * HS;
  const uint32_t start = start_pos[ctx];

  // this lane's query column: token tq, head gq; invalid beyond n_tokens
  const uint32_t tq = group * TPG + c / G;
  const uint32_t gq = c % G;
  const bool col_ok = wave_ok && tq < n_tokens;
  const int32_t qpos = col_ok ? (int32_t)( start + tq ) : -1; // last visible key of the column
  const uint32_t last_tok = min( n_tokens, ( group + 1 ) * TPG ) - 1;
  const uint32_t t_end = wave_ok ? start + last_tok + 1 : 0; // keys [0, t_end) are visible to some column of the group
  // the work-group streams the keys its last group needs; every wave loads a quarter of each 64-key tile
  const uint32_t last_group = min( groups_per_head, quad * 4 + 4 ) - 1;
  const uint32_t wg_end = start + min( n_tokens, ( last_group + 1 ) * TPG );

  f16x8 qb[4];
  {
    const __half* qp = q + ( ( (uint64_t)ctx * n_tokens + ( col_ok ? tq : 0 ) ) * n_heads + (uint64_t)h * G + gq ) * HS;
#pragma unroll
    for ( int kk = 0; kk < 4; kk++ ) {
      uint4 v = load16( qp + 8 * ( 4 * kk + g4 ) );
      if ( !col_ok ) {
        v = make_uint4( 0, 0, 0, 0 );
      }
      qb[kk] = __builtin_bit_cast( f16x8, v );
    }
  }

  f32x4 acc[8];
#pragma unroll
  for ( int nn = 0; nn < 8; nn++ ) {
    acc[nn] = f32x4 { 0.0f, 0.0f, 0.0f, 0.0f };
  }
  float m = -INFINITY;
  float l = 0.0f;

  const __half* kp = base + (uint64_t)h * HS + 8 * c;
  const uint4 zero4 = make_uint4( 0, 0, 0, 0 );
  uint4 kn[4], vn[4];
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    const uint32_t tok = 16 * wave + 4 * g4 + i;
    const bool ok = tok < wg_end;
    const __half* row = kp + (uint64_t)tok * row_elems;
    kn[i] = ok ? load16( row ) : zero4;
    vn[i] = ok ? load16( row + v_off ) : zero4;
  }

  for ( uint32_t tile0 = 0; tile0 < wg_end; tile0 += 64 ) {
    uint4* kt = s_kt;
    uint4* vt = s_vt;
    if ( tile0 != 0 ) {
      __syncthreads(); // every wave is done with the previous tile
    }
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      const uint32_t tl = 4 * g4 + i;
      kt[( 16 * wave + tl ) * 16 + ( c ^ tl )] = kn[i];
      vt[( 16 * wave + tl ) * 16 + c] = vn[i];
    }
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      const uint32_t tok = tile0 + 64 + 16 * wave + 4 * g4 + i;
      const bool ok = tok < wg_end;
      const __half* row = kp + (uint64_t)tok * row_elems;
      kn[i] = ok ? load16( row ) : zero4;
      vn[i] = ok ? load16( row + v_off ) : zero4;
    }
    __syncthreads();

    for ( uint32_t sub = 0; sub < 4; sub++ ) {
      const uint32_t t0 = tile0 + 16 * sub;
      if ( t0 >= t_end ) {
        break; // wave-uniform: nothing further is visible to this wave's queries
      }
      const uint4* tile = kt + 16 * sub * 16;
      uint4 vc[4];
#pragma unroll
      for ( int i = 0; i < 4; i++ ) {
        vc[i] = vt[( 16 * sub + 4 * g4 + i ) * 16 + c];
      }

      f32x4 st = f32x4 { 0.0f, 0.0f, 0.0f, 0.0f };
#pragma unroll
      for ( int kk = 0; kk < 4; kk++ ) {
        const uint4 kf = tile[c * 16 + ( ( 4 * kk + g4 ) ^ c )];
        st = __builtin_amdgcn_mfma_f32_16x16x32_f16( __builtin_bit_cast( f16x8, kf ), qb[kk], st, 0, 0, 0 );
      }

      // st[i] = score of key t0 + 4*g4 + i for query column c; causal mask per column
      float s[4];
      float mt = -INFINITY;
#pragma unroll
      for ( int i = 0; i < 4; i++ ) {
        const int32_t key = (int32_t)( t0 + 4 * g4 + i );
        s[i] = key <= qpos ? st[i] * scale_log2e : -INFINITY;
        mt = fmaxf( mt, s[i] );
      }
      mt = fmaxf( mt, __shfl_xor( mt, 16, WAVE ) );
      mt = fmaxf( mt, __shfl_xor( mt, 32, WAVE ) );
      const float m_new = fmaxf( m, mt );
      const float m_safe = m_new == -INFINITY ? 0.0f : m_new; // padding columns never see a key
      const float alpha = fast_exp2( m - m_safe );
      float p[4];
#pragma unroll
      for ( int i = 0; i < 4; i++ ) {
        p[i] = fast_exp2( s[i] - m_safe );
      }
      l = l * alpha + ( p[0] + p[1] ) + ( p[2] + p[3] );
      m = m_new;

      if ( __builtin_amdgcn_ballot_w64( alpha != 1.0f ) != 0 ) {
#pragma unroll
        for ( int i = 0; i < 4; i++ ) {
          const float a = __shfl( alpha, (int)( 4 * g4 + i ), WAVE );
#pragma unroll
          for ( int nn = 0; nn < 8; nn++ ) {
            acc[nn][i] *= a;
          }
        }
      }

      const f16x4 pa = f16x4 { (_Float16)p[0], (_Float16)p[1], (_Float16)p[2], (_Float16)p[3] };
      const uint32_t vw[4][4] = { { vc[0].x, vc[0].y, vc[0].z, vc[0].w },
                                  { vc[1].x, vc[1].y, vc[1].z, vc[1].w },
                                  { vc[2].x, vc[2].y, vc[2].z, vc[2].w },
                                  { vc[3].x, vc[3].y, vc[3].z, vc[3].w } };
#pragma unroll
      for ( int w = 0; w < 4; w++ ) {
        const uint2 lo = make_uint2( __builtin_amdgcn_perm( vw[1][w], vw[0][w], 0x05040100u ), __builtin_amdgcn_perm( vw[3][w], vw[2][w], 0x05040100u ) );
        const uint2 hi = make_uint2( __builtin_amdgcn_perm( vw[1][w], vw[0][w], 0x07060302u ), __builtin_amdgcn_perm( vw[3][w], vw[2][w], 0x07060302u ) );
        acc[2 * w] = __builtin_amdgcn_mfma_f32_16x16x16f16( pa, __builtin_bit_cast( f16x4, lo ), acc[2 * w], 0, 0, 0 );
        acc[2 * w + 1] = __builtin_amdgcn_mfma_f32_16x16x16f16( pa, __builtin_bit_cast( f16x4, hi ), acc[2 * w + 1], 0, 0, 0 );
      }
    }
  }

  l += __shfl_xor( l, 16, WAVE );
  l += __shfl_xor( l, 32, WAVE );

  // the accumulators of this lane belong to query columns 4*g4 + i
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    const uint32_t col = 4 * g4 + i;
    const float lc = __shfl( l, (int)col, WAVE );
    const uint32_t tok = group * TPG + col / G;
    const uint32_t hd = col % G;
    if ( tok < n_tokens ) {
      const float inv = 1.0f / lc;
      union
      {
        uint4 raw;
        __half hv[8];
      } o;
#pragma unroll
      for ( int nn = 0; nn < 8; nn++ ) {
        o.hv[nn] = __float2half_rn( acc[nn][i] * inv );
      }
      *reinterpret_cast<uint4*>( xb + ( ( (uint64_t)ctx * n_tokens + tok ) * n_heads + (uint64_t)h * G + hd ) * HS + 8 * c ) = o.raw;
    }
  }
}

template<int G>
void launch_prefill( hipStream_t st, const void* q, const void* const* rows, const uint32_t* start, void* xb, uint64_t batch, uint32_t n_tokens,
                     const gh_shape* s )
{
  const uint32_t groups = ( n_tokens + ( 16 / G ) - 1 ) / ( 16 / G );
  const uint64_t blocks = batch * s->n_kv_heads * ( ( groups + 3 ) / 4 );
  attn_prefill_mfma_kernel<G><<<(unsigned)blocks, 256, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( rows ), start,
                                                                static_cast<__half*>( xb ), s->n_kv_heads, n_tokens, groups,
                                                                LOG2E / sqrtf( (float)s->head_size ) );
}

} // namespace
} // namespace gh

using namespace gh;

extern "C" {

int gh_prefill_tables( const void* const* layer_rows_dev, const uint32_t* start_pos_dev, uint64_t batch, uint32_t n_tokens, uint64_t row_bytes,
                       const void** layer_rows_out, void** token_rows_out, uint32_t* pos_out, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 || n_tokens == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( layer_rows_dev && start_pos_dev, "gh_prefill_tables: NULL table" );
  GH_REQUIRE( batch * n_tokens <= 0x7fffffffull, "gh_prefill_tables: too many entries" );
  const uint64_t n = batch * n_tokens;
  expand_tables_kernel<<<(unsigned)( ( n + 255 ) / 256 ), 256, 0, as_stream( stream )>>>( layer_rows_dev, start_pos_dev, (uint32_t)batch, n_tokens, row_bytes,
                                                                                       layer_rows_out, token_rows_out, pos_out );
  GH_LAUNCH_CHECK();
  return GH_OK;
}

uint64_t gh_attn_prefill_workspace( uint64_t batch, uint32_t n_tokens, const gh_shape* shape )
{
  if ( shape == nullptr || batch == 0 || n_tokens == 0 ) {
    return 0;
  }
  const uint64_t n = batch * n_tokens;
  // expanded tables for the fallback path + the decode workspace for n rows
  return n * ( sizeof( void* ) + sizeof( uint32_t ) ) + 64 + gh_attn_decode_workspace( n, shape->seq_len - 1, shape );
}

int gh_attn_prefill( const void* q, const void* const* layer_rows_dev, const uint32_t* start_pos_dev, void* xb, uint64_t batch, uint32_t n_tokens,
                     uint32_t max_start_pos, const gh_shape* shape, gh_dtype dt, void* workspace, uint64_t workspace_bytes, int variant, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 || n_tokens == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( shape != nullptr && q && layer_rows_dev && start_pos_dev && xb, "gh_attn_prefill: NULL pointer" );
  GH_REQUIRE( dt == GH_F16 || dt == GH_F32, "gh_attn_prefill: unsupported dtype %d", (int)dt );
  GH_REQUIRE( shape->n_heads == shape->n_kv_heads * shape->gqa_size && shape->kv_dim == shape->n_kv_heads * shape->head_size, "gh_attn_prefill: inconsistent shape" );
  GH_REQUIRE( (uint64_t)max_start_pos + n_tokens <= shape->seq_len, "gh_attn_prefill: positions %u + %u exceed seq_len %u", max_start_pos, n_tokens, shape->seq_len );
  GH_REQUIRE( batch * n_tokens <= 65535ull * 16, "gh_attn_prefill: too many query tokens in one call" );
  hipStream_t st = as_stream( stream );
  const uint32_t g = shape->gqa_size;
  const bool mfma_ok = dt == GH_F16 && shape->head_size == HS && ( g == 1 || g == 2 || g == 4 || g == 8 || g == 16 )
                       && ( ( reinterpret_cast<uintptr_t>( q ) | reinterpret_cast<uintptr_t>( xb ) ) & 15u ) == 0;
  GH_REQUIRE( variant == GH_ATTN_AUTO || variant == GH_ATTN_GENERIC || variant == GH_ATTN_VALU || variant == GH_ATTN_MFMA, "gh_attn_prefill: unknown variant %d", variant );
  if ( variant == GH_ATTN_MFMA ) {
    GH_REQUIRE( mfma_ok, "gh_attn_prefill: the mfma kernel needs f16, head_size 128, gqa in {1,2,4,8,16}" );
  }

  if ( mfma_ok && ( variant == GH_ATTN_AUTO || variant == GH_ATTN_MFMA ) ) {
    switch ( g ) {
      case 1: launch_prefill<1>( st, q, layer_rows_dev, start_pos_dev, xb, batch, n_tokens, shape ); break;
      case 2: launch_prefill<2>( st, q, layer_rows_dev, start_pos_dev, xb, batch, n_tokens, shape ); break;
      case 4: launch_prefill<4>( st, q, layer_rows_dev, start_pos_dev, xb, batch, n_tokens, shape ); break;
      case 8: launch_prefill<8>( st, q, layer_rows_dev, start_pos_dev, xb, batch, n_tokens, shape ); break;
      default: launch_prefill<16>( st, q, layer_rows_dev, start_pos_dev, xb, batch, n_tokens, shape ); break;
    }
    GH_LAUNCH_CHECK();
    return GH_OK;
  }

  // any other shape: one decode row per (context, token)
  const uint64_t n = batch * n_tokens;
  GH_REQUIRE( n <= 65535, "gh_attn_prefill: the generic path takes at most 65535 query tokens per call" );
  const uint64_t table_bytes = ( n * ( sizeof( void* ) + sizeof( uint32_t ) ) + 63 ) / 64 * 64;
  GH_REQUIRE( workspace != nullptr && workspace_bytes >= table_bytes, "gh_attn_prefill: workspace of %llu bytes needed for the expanded tables",
              (unsigned long long)gh_attn_prefill_workspace( batch, n_tokens, shape ) );
  GH_REQUIRE( ( reinterpret_cast<uintptr_t>( workspace ) & 15u ) == 0, "gh_attn_prefill: workspace must be 16-byte aligned" );
  const void** rows_x = static_cast<const void**>( workspace );
  uint32_t* pos_x = reinterpret_cast<uint32_t*>( rows_x + n );
  const uint64_t row_bytes = 2ull * shape->kv_dim * dtype_size( dt );
  if ( int rc = gh_prefill_tables( layer_rows_dev, start_pos_dev, batch, n_tokens, row_bytes, rows_x, nullptr, pos_x, stream ) ) {
    return rc;
  }
  uint8_t* decode_ws = static_cast<uint8_t*>( workspace ) + table_bytes;
  return gh_attn_decode( q, rows_x, pos_x, xb, n, max_start_pos + n_tokens - 1, shape, dt, decode_ws, workspace_bytes - table_bytes,
                         variant == GH_ATTN_MFMA ? GH_ATTN_AUTO : variant, stream );
}

} // extern "C"
