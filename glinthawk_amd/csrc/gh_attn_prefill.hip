// Batched prefill attention: T new tokens per context at positions [start_i, start_i + T), all of
// whose [K | V] rows are already in the cache; query token t attends keys [0, start_i + t] (causal).
// The reference has no multi-token path (it feeds prompts one token per forward,
// frontend/infer.cc:124-125, models/llama2/model.hh:356-357); the result of this kernel equals T
// sequential calls of the decode path.
//
// f16, head size 128: a tiled MFMA kernel (see attn_prefill_mfma_kernel).
//
// Any other shape: the decode kernels are run on tables expanded to one entry per (context, token).
#include "gh_common.h"

namespace gh {
namespace {

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LAZY = 8.0f; // see the softmax step of the tiled prefill kernel
constexpr int HS = 128;
#ifndef PF_WGS_PER_CU
#define PF_WGS_PER_CU 1
#endif

typedef _Float16 f16x4 __attribute__( ( ext_vector_type( 4 ) ) );
typedef _Float16 f16x8 __attribute__( ( ext_vector_type( 8 ) ) );
typedef float f32x4 __attribute__( ( ext_vector_type( 4 ) ) );
typedef float f32x16 __attribute__( ( ext_vector_type( 16 ) ) );

__device__ __forceinline__ float fast_exp2( float x ) { return __builtin_amdgcn_exp2f( x ); }
// Cache rows are reached through pointers read from a table, so the compiler cannot tell that they are global memory and would
// use flat loads, which count against the LDS wait counter as well: every wait for an LDS read would then also wait for the rows
// of the next stage that are meant to stay in flight.  The cast names the address space.
typedef uint32_t u32x4_t __attribute__( ( ext_vector_type( 4 ) ) );
typedef const u32x4_t __attribute__( ( address_space( 1 ) ) ) global_u32x4_t;
__device__ __forceinline__ uint4 load16( const __half* p ) { return __builtin_bit_cast( uint4, *(global_u32x4_t*)( p ) ); }

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

// q, xb: (batch * n_tokens, n_kv_heads * G * 128), row index = context * n_tokens + token.
// Query column c of a (context, kv head): token c / G, query head c % G (the G heads that share the kv head).
//
// block = 4 waves = 256 query columns; wave = 64 columns = two 32-column MFMA tiles.  Per 64-key stage (K and V rows in LDS,
// the next stage's rows in flight in registers):
//   S^T = K Q^T   v_mfma_f32_32x32x16_f16, A = K rows out of LDS (16-byte chunks, XOR-swizzled), B = Q^T in registers; every A
//                 fragment feeds both column tiles.  A lane ends up with 16 of the 32 keys of a sub-tile for ITS query column,
//                 the lane 32 further on with the other 16: maximum and sum stay inside a lane but for one exchange per stage
//   O^T += V^T P^T  the scores of a lane are, as they lie, the B operand (keys x its column) of the same instruction; the A
//                 operand V^T (4 consecutive dims x 8 keys per lane) is put together from 8-byte LDS reads with v_perm and again
//                 feeds both column tiles.  Every accumulator of a lane belongs to its own column: rescaling needs no shuffle
// Causal mask only on stages that reach a wave's diagonal; stages beyond it are skipped.
template<int G, int NQT>
__global__ __launch_bounds__( 256, NQT == 1 ? 2 : 1 ) void attn_prefill_mfma_kernel( const __half* __restrict__ q,
                                                                   const __half* const* __restrict__ layer_rows,
                                                                   const uint32_t* __restrict__ start_pos,
                                                                   __half* __restrict__ xb,
                                                                   uint32_t n_kv_heads,
                                                                   uint32_t n_tokens,
                                                                   uint32_t col_blocks, // ceil(n_tokens * G / (128 * NQT))
                                                                   float scale_log2e )
{
  __shared__ uint4 s_kt[64 * 16]; // 64 keys x 256 bytes, 16-byte chunks XOR-swizzled by the key's low bits
  __shared__ uint4 s_vt[64 * 16]; // the same keys' value rows, plain
  static_assert( 32 * NQT >= G, "a wave holds whole tokens" );
  constexpr uint32_t TPW = 32 * NQT / G; // tokens per wave

  const uint32_t wave = __builtin_amdgcn_readfirstlane( threadIdx.x >> 6 ); // provably uniform: what derives from it stays in scalar registers
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t r = lane & 31;
  const uint32_t g2 = lane >> 5;
  // block -> (column block, kv head, context); the column blocks with the most keys are numbered first
  uint32_t bid = blockIdx.x;
  const uint32_t cb = col_blocks - 1 - bid % col_blocks;
  bid /= col_blocks;
  const uint32_t h = bid % n_kv_heads;
  const uint32_t ctx = bid / n_kv_heads;
  const __half* base = layer_rows[ctx];
  if ( base == nullptr ) {
    return; // the whole work-group
  }
  const uint32_t n_heads = n_kv_heads * G;
  const uint64_t row_elems = 2ull * n_kv_heads * HS;
  const uint32_t v_off = n_kv_heads * HS;
  const uint32_t start = start_pos[ctx];

  const uint32_t wave_tok0 = ( cb * 4 + wave ) * TPW;          // first token of the wave
  const bool wave_ok = wave_tok0 < n_tokens;                    // a wave without queries still loads its share of every stage
  const uint32_t wave_last = min( n_tokens, wave_tok0 + TPW ) - 1;
  const uint32_t t_end = wave_ok ? start + wave_last + 1 : 0;   // keys [0, t_end) are visible to some column of the wave
  const uint32_t t_all = start + wave_tok0 + 1;                 // keys [0, t_all) are visible to every column of the wave
  const uint32_t wg_end = start + min( n_tokens, ( cb + 1 ) * 4 * TPW );

  // this lane's two query columns (tile 0 and tile 1): token, head, last visible key
  uint32_t tq[NQT], gq[NQT];
  int32_t qpos[NQT];
  f16x8 qb[NQT][8];
#pragma unroll
  for ( int qt = 0; qt < NQT; qt++ ) {
    const uint32_t col = 32 * qt + r;
    tq[qt] = wave_tok0 + col / G;
    gq[qt] = col % G;
    const bool ok = wave_ok && tq[qt] < n_tokens;
    qpos[qt] = ok ? (int32_t)( start + tq[qt] ) : -1;
    const __half* qp = q + ( ( (uint64_t)ctx * n_tokens + ( ok ? tq[qt] : 0 ) ) * n_heads + (uint64_t)h * G + gq[qt] ) * HS;
#pragma unroll
    for ( int s = 0; s < 8; s++ ) {
      uint4 v = load16( qp + 8 * ( 2 * s + g2 ) );
      if ( !ok ) {
        v = make_uint4( 0, 0, 0, 0 );
      }
      qb[qt][s] = __builtin_bit_cast( f16x8, v );
    }
  }

  f32x16 acc[NQT][4]; // [column tile][dim block i]: element v <-> dim 4 * (8*(v/4) + 4*g2 + v%4) + i of this lane's column
#pragma unroll
  for ( int qt = 0; qt < NQT; qt++ ) {
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
#pragma unroll
      for ( int v = 0; v < 16; v++ ) {
        acc[qt][i][v] = 0.0f;
      }
    }
  }
  float m[NQT]; // reference point of the column's exponentials (log2 domain), identical in the two lanes that share the column;
               // within LAZY of the running maximum
  float l[NQT];                          // this lane's share of the running sum
#pragma unroll
  for ( int qt = 0; qt < NQT; qt++ ) {
    m[qt] = -INFINITY;
    l[qt] = 0.0f;
  }

  // global -> registers: thread t fetches chunk t % 16 of keys t / 16 + 16 j, K and V
  const uint32_t ld_chunk = threadIdx.x & 15;
  const uint32_t ld_key = threadIdx.x >> 4;
  const __half* kp = base + (uint64_t)h * HS + 8 * ld_chunk;
  const uint4 zero4 = make_uint4( 0, 0, 0, 0 );
  uint4 kn[4], vn[4];
  // rows of the stage after the current one: thread t fetches keys ld_key + 16 j of it; the pointer moves 64 rows per stage
  const __half* next_rows = kp + (uint64_t)ld_key * row_elems;
  const uint64_t row16 = 16 * row_elems, stage_step = 64 * row_elems;
  auto fetch_stage = [&]( uint32_t first_key ) {
    if ( __builtin_amdgcn_readfirstlane( first_key + 64 <= wg_end ) ) { // the whole stage lies inside the key range: no per-row guards
#pragma unroll
      for ( int j = 0; j < 4; j++ ) {
        kn[j] = load16( next_rows + j * row16 );
        vn[j] = load16( next_rows + j * row16 + v_off );
      }
    } else {
      // the last, partial stage: rows past the range may hold anything (a weight of zero times a NaN is a NaN), they read as zero
#pragma unroll
      for ( int j = 0; j < 4; j++ ) {
        const bool ok = first_key + ld_key + 16 * j < wg_end;
        kn[j] = ok ? load16( next_rows + j * row16 ) : zero4;
        vn[j] = ok ? load16( next_rows + j * row16 + v_off ) : zero4;
      }
    }
    next_rows += stage_step;
  };
  fetch_stage( 0 );

  for ( uint32_t t0 = 0; t0 < wg_end; t0 += 64 ) {
    if ( t0 != 0 ) {
      __syncthreads(); // every wave is done with the previous stage
    }
#pragma unroll
    for ( int j = 0; j < 4; j++ ) {
      const uint32_t key = ld_key + 16 * j;
      s_kt[key * 16 + ( ld_chunk ^ ( key & 15 ) )] = kn[j];
      s_vt[key * 16 + ld_chunk] = vn[j];
    }
    if ( __builtin_amdgcn_readfirstlane( t0 + 64 < wg_end ) ) {
      fetch_stage( t0 + 64 );
    }
    __syncthreads();
    if ( __builtin_amdgcn_readfirstlane( t0 >= t_end ) ) {
      continue; // nothing of this stage is visible to the wave's queries (it still took part in the loads and barriers)
    }
    // a stage that reaches the wave's diagonal hides keys from some columns; before it every key is visible to every column
    const bool masked = __builtin_amdgcn_readfirstlane( t0 + 64 > t_all );

    // ---- scores: st[qt][sub][v] = raw score of key t0 + 32 sub + 8*(v/4) + 4*g2 + v%4 for column tile qt.  The two sub-tiles are
    //      independent accumulation chains that alternate in the matrix pipe (keys past the diagonal are computed and masked)
    f32x16 st[NQT][2];
#pragma unroll
    for ( int qt = 0; qt < NQT; qt++ ) {
#pragma unroll
      for ( int sub = 0; sub < 2; sub++ ) {
#pragma unroll
        for ( int v = 0; v < 16; v++ ) {
          st[qt][sub][v] = 0.0f;
        }
      }
    }
#pragma unroll
    for ( int s = 0; s < 8; s++ ) {
#pragma unroll
      for ( int sub = 0; sub < 2; sub++ ) {
        const uint32_t krow = 32 * sub + r;
        const f16x8 a = __builtin_bit_cast( f16x8, s_kt[krow * 16 + ( ( 2 * s + g2 ) ^ ( krow & 15 ) )] );
#pragma unroll
        for ( int qt = 0; qt < NQT; qt++ ) {
          st[qt][sub] = __builtin_amdgcn_mfma_f32_32x32x16_f16( a, qb[qt][s], st[qt][sub], 0, 0, 0 );
        }
      }
    }
    if ( masked ) {
#pragma unroll
      for ( int qt = 0; qt < NQT; qt++ ) {
#pragma unroll
        for ( int sub = 0; sub < 2; sub++ ) {
#pragma unroll
          for ( int v = 0; v < 16; v++ ) {
            const int32_t key = (int32_t)( t0 + 32 * sub + 8 * ( v / 4 ) + 4 * g2 + ( v % 4 ) );
            st[qt][sub][v] = key <= qpos[qt] ? st[qt][sub][v] : -INFINITY;
          }
        }
      }
    }

    // ---- online softmax per column tile; p packed as B operands: pk[qt][2 sub + jj] = keys 32 sub + 16 jj + 8 (e/4) + 4 g2 + e%4, e = 0..7
    f16x8 pk[NQT][4];
#pragma unroll
    for ( int qt = 0; qt < NQT; qt++ ) {
      float mx = st[qt][0][0];
#pragma unroll
      for ( int sub = 0; sub < 2; sub++ ) {
#pragma unroll
        for ( int v = 0; v < 16; v++ ) {
          mx = fmaxf( mx, st[qt][sub][v] );
        }
      }
      mx = fmaxf( mx, __shfl_xor( mx, 32, WAVE ) ) * scale_log2e; // log2 domain from here on
      // The reference point of the exponentials only moves when the maximum has grown by more than 2^LAZY since it was set:
      // weights stay below 2^LAZY (fine for fp32 sums and fp16 operands) and the 64 accumulators are rescaled rarely.  The
      // result does not depend on the reference point.  -inf: a column that has seen no key yet (padding, or hidden so far).
      if ( __builtin_amdgcn_ballot_w64( mx > m[qt] + LAZY ) != 0 ) {
        const float m_new = fmaxf( m[qt], mx );
        const float alpha = m_new == -INFINITY ? 1.0f : fast_exp2( m[qt] - m_new );
        m[qt] = m_new;
        l[qt] *= alpha;
#pragma unroll
        for ( int i = 0; i < 4; i++ ) {
#pragma unroll
          for ( int v = 0; v < 16; v++ ) {
            acc[qt][i][v] *= alpha;
          }
        }
      }
      const float ms = m[qt] == -INFINITY ? 0.0f : m[qt];
      float sum[2] = { 0.0f, 0.0f };
#pragma unroll
      for ( int sub = 0; sub < 2; sub++ ) {
#pragma unroll
        for ( int jj = 0; jj < 2; jj++ ) {
          float p[8];
#pragma unroll
          for ( int e = 0; e < 8; e++ ) {
            p[e] = fast_exp2( st[qt][sub][8 * jj + e] * scale_log2e - ms );
            sum[e & 1] += p[e];
          }
          pk[qt][2 * sub + jj] = f16x8 { (_Float16)p[0], (_Float16)p[1], (_Float16)p[2], (_Float16)p[3],
                                         (_Float16)p[4], (_Float16)p[5], (_Float16)p[6], (_Float16)p[7] };
        }
      }
      l[qt] += sum[0] + sum[1];
    }

    // ---- O^T += V^T P^T: per 16 keys (kk) the lane reads dims 4r .. 4r+3 of its 8 key slots and transposes them into 4 A operands,
    //      one per dim block i; the four dim blocks are independent accumulation chains
#pragma unroll
    for ( int kk = 0; kk < 4; kk++ ) {
      uint2 vr[8];
#pragma unroll
      for ( int e = 0; e < 8; e++ ) {
        const uint32_t key = 16 * kk + 8 * ( e / 4 ) + 4 * g2 + ( e % 4 );
        vr[e] = *reinterpret_cast<const uint2*>( reinterpret_cast<const char*>( s_vt ) + key * 256 + 8 * r );
      }
#pragma unroll
      for ( int i = 0; i < 4; i++ ) {
        // dim 4r + i of the 8 keys: halves (i % 2) of word (i / 2) of every key's 8 bytes
        const uint32_t sel = ( i % 2 ) ? 0x07060302u : 0x05040100u;
        uint32_t w[8];
#pragma unroll
        for ( int e = 0; e < 8; e++ ) {
          w[e] = ( i / 2 ) ? vr[e].y : vr[e].x;
        }
        const uint4 a4 = make_uint4( __builtin_amdgcn_perm( w[1], w[0], sel ), __builtin_amdgcn_perm( w[3], w[2], sel ),
                                     __builtin_amdgcn_perm( w[5], w[4], sel ), __builtin_amdgcn_perm( w[7], w[6], sel ) );
        const f16x8 a = __builtin_bit_cast( f16x8, a4 );
#pragma unroll
        for ( int qt = 0; qt < NQT; qt++ ) {
          acc[qt][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16( a, pk[qt][kk], acc[qt][i], 0, 0, 0 );
        }
      }
    }
  }

  // ---- normalise and store: element v of acc[qt][i] is dim 4 * (8*(v/4) + 4*g2 + v%4) + i of the lane's column
#pragma unroll
  for ( int qt = 0; qt < NQT; qt++ ) {
    const float lsum = l[qt] + __shfl_xor( l[qt], 32, WAVE );
    if ( qpos[qt] < 0 ) {
      continue; // padding column
    }
    const float inv = 1.0f / lsum;
    __half* out = xb + ( ( (uint64_t)ctx * n_tokens + tq[qt] ) * n_heads + (uint64_t)h * G + gq[qt] ) * HS;
#pragma unroll
    for ( int v = 0; v < 16; v++ ) {
      const uint32_t d0 = 4 * ( 8 * ( v / 4 ) + 4 * g2 + ( v % 4 ) );
      union
      {
        uint2 raw;
        __half hv[4];
      } o;
#pragma unroll
      for ( int i = 0; i < 4; i++ ) {
        o.hv[i] = __float2half_rn( acc[qt][i][v] * inv );
      }
      *reinterpret_cast<uint2*>( out + d0 ) = o.raw;
    }
  }
}

template<int G, int NQT>
void launch_prefill_tiles( hipStream_t st, const void* q, const void* const* rows, const uint32_t* start, void* xb, uint64_t batch, uint32_t n_tokens,
                           const gh_shape* s )
{
  const uint32_t col_blocks = (uint32_t)( ( (uint64_t)n_tokens * G + 128 * NQT - 1 ) / ( 128 * NQT ) );
  const uint64_t blocks = batch * s->n_kv_heads * col_blocks;
  attn_prefill_mfma_kernel<G, NQT><<<(unsigned)blocks, 256, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( rows ), start,
                                                                     static_cast<__half*>( xb ), s->n_kv_heads, n_tokens, col_blocks,
                                                                     LOG2E / sqrtf( (float)s->head_size ) );
}

int g_prefill_tiles = 1; // column tiles per wave

template<int G>
void launch_prefill( hipStream_t st, const void* q, const void* const* rows, const uint32_t* start, void* xb, uint64_t batch, uint32_t n_tokens,
                     const gh_shape* s )
{
  if ( g_prefill_tiles == 2 ) {
    launch_prefill_tiles<G, 2>( st, q, rows, start, xb, batch, n_tokens, s );
  } else {
    launch_prefill_tiles<G, 1>( st, q, rows, start, xb, batch, n_tokens, s );
  }
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

int gh_attn_set_prefill_tiles( int column_tiles_per_wave )
{
  GH_REQUIRE( column_tiles_per_wave == 1 || column_tiles_per_wave == 2, "gh_attn_set_prefill_tiles: 1 or 2 column tiles per wave" );
  g_prefill_tiles = column_tiles_per_wave;
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
