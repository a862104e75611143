// Unfused attention ops with the `att` score buffer, one entry point per method of the reference's
// interface: attention_0_gemm, attention_softmax, attention_2_gemm
// (arch/amd64/llama2/ops.hh:170-298) -- what an unmodified model driver calls.
//
// f16 storage with head size 128 runs streaming kernels with the decomposition of the fused decode
// kernel: a wave owns (context, kv head, token range) and reads its K (scores) or V (weighted sum)
// head rows once with 16-byte non-temporal loads, 32 tokens per iteration.
//   scores        gqa 4/8/16: S^T = K Q^T on v_mfma_f32_16x16x32_f16, K through a wave-private swizzled LDS tile;
//                 gqa 1/2: v_dot2_f32_f16 with 16-lane DPP reductions.  A lane ends up with 8 consecutive tokens
//                 of one head row: one 16-byte store
//   softmax       a block per (head, context) keeps the whole row in registers: one read, one write
//   weighted sum  gqa 4/8/16: O += P V on v_mfma_f32_16x16x16_f16, V transposed in registers; gqa 1/2: fp32 FMAs.
//                 Token ranges give fp32 partial sums that a second kernel adds and rounds once
// Rounding points are the CPU path's: scale * fp32 sum -> DType; DType max, DType difference, exp
// rounded to DType, fp32 sum, fp32 quotient -> DType; fp32 weighted sum -> DType.
// Every other shape or type runs the generic kernels at the end of this list.
#include "gh_common.h"
#include "gh_attn_tiles.h"

#include <algorithm>

namespace gh {
namespace {

constexpr int MAX_GQA = 16;
constexpr uint32_t TOK_PER_IT = 32; // tokens a wave handles per loop iteration of the streaming kernels

// lane (g4, c) owns the 8 consecutive tokens t0 + 8*g4 .. + 7 of an iteration and chunk c (8 halves) of their head rows
__device__ __forceinline__ void load_rows8( uint4 out[8], const __half* p0, uint64_t row_elems, uint32_t tok0, uint32_t t_end, bool any )
{
  const uint4 zero4 = make_uint4( 0, 0, 0, 0 );
#pragma unroll
  for ( int i = 0; i < 8; i++ ) {
    const uint32_t tok = tok0 + i;
    out[i] = ( any && tok < t_end ) ? load16_stream( p0 + (uint64_t)tok * row_elems ) : zero4;
  }
}

__device__ __forceinline__ uint2 pack4( float a, float b, float c, float d )
{
  const f16x2 lo = f16x2 { (_Float16)a, (_Float16)b };
  const f16x2 hi = f16x2 { (_Float16)c, (_Float16)d };
  return make_uint2( __builtin_bit_cast( uint32_t, lo ), __builtin_bit_cast( uint32_t, hi ) );
}

// stores the 8 scores of a lane (tokens tok0 .. tok0 + 7 of one head row), whole where the range allows
__device__ __forceinline__ void store_scores8( __half* row, uint32_t tok0, uint32_t t_end, const float v[8] )
{
  if ( tok0 + 8 <= t_end ) {
    const uint2 a = pack4( v[0], v[1], v[2], v[3] );
    const uint2 b = pack4( v[4], v[5], v[6], v[7] );
    *reinterpret_cast<uint4*>( row + tok0 ) = make_uint4( a.x, a.y, b.x, b.y );
  } else {
#pragma unroll
    for ( int i = 0; i < 8; i++ ) {
      if ( tok0 + i < t_end ) {
        row[tok0 + i] = __float2half_rn( v[i] );
      }
    }
  }
}

// =================================================================================================
// scores, gqa 4 / 8 / 16: two 16-token MFMA tiles per iteration.  LDS row 4*g4 + i of tile A holds token
// t0 + 8*g4 + i, of tile B token t0 + 8*g4 + 4 + i, so the score rows of a lane are its own 8 tokens.
// =================================================================================================
template<int G>
__global__ __launch_bounds__( 256 ) void attn_scores_mfma_kernel( const __half* __restrict__ q,
                                                                  const __half* const* __restrict__ layer_rows,
                                                                  const uint32_t* __restrict__ pos,
                                                                  __half* __restrict__ att,
                                                                  uint32_t n_kv_heads,
                                                                  uint32_t seq_len,
                                                                  uint32_t chunk,
                                                                  uint32_t max_splits,
                                                                  float scale )
{
  __shared__ uint4 s_k[4][2][16 * 16]; // per wave: two tiles of 16 tokens x 16 chunks of 16 bytes

  const WaveJob job = wave_job( layer_rows, pos, n_kv_heads, chunk, max_splits, seq_len );
  if ( !job.valid ) {
    return; // wave-uniform; only wave-private LDS is used, no block barrier
  }
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t g4 = lane >> 4;
  const uint32_t n_heads = n_kv_heads * G;
  const uint64_t row_elems = 2ull * n_kv_heads * HS;
  uint4* tile_a = s_k[wave][0];
  uint4* tile_b = s_k[wave][1];

  // B fragments of Q^T: head c (zero for the padding heads), dims of chunk 4*kk + g4
  f16x8 qb[4];
  {
    const __half* qp = q + ( (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G + ( c < G ? c : 0 ) ) * HS;
#pragma unroll
    for ( int kk = 0; kk < 4; kk++ ) {
      uint4 v = load16( qp + 8 * ( 4 * kk + g4 ) );
      if ( c >= G ) {
        v = make_uint4( 0, 0, 0, 0 );
      }
      qb[kk] = __builtin_bit_cast( f16x8, v );
    }
  }
  __half* out_row = att + ( (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G + ( c < G ? c : 0 ) ) * seq_len;
  const __half* kp = job.base + (uint64_t)job.h * HS + 8 * c;

  // iterations in rotated order, a different start per block (blocks launched together would otherwise walk
  // power-of-two-strided ranges in lock step and share few HBM channels)
  const uint32_t n_it = ( job.t_end - job.t_begin + TOK_PER_IT - 1 ) / TOK_PER_IT;
  uint32_t it_i = ( ( job.ctx * 5u + job.split * 3u ) * 7u ) % n_it;
  uint32_t t0 = job.t_begin + TOK_PER_IT * it_i;

  uint4 kn[8];
  load_rows8( kn, kp, row_elems, t0 + 8 * g4, job.t_end, true );

  for ( uint32_t it = 0; it < n_it; it++ ) {
    it_i = it_i + 1 == n_it ? 0 : it_i + 1;
    const uint32_t t_next = job.t_begin + TOK_PER_IT * it_i;
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      const uint32_t tl = 4 * g4 + i;
      tile_a[tl * 16 + ( c ^ tl )] = kn[i];
      tile_b[tl * 16 + ( c ^ tl )] = kn[4 + i];
    }
    load_rows8( kn, kp, row_elems, t_next + 8 * g4, job.t_end, it + 1 < n_it );
    __builtin_amdgcn_fence( __ATOMIC_RELEASE, "wavefront" );
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence( __ATOMIC_ACQUIRE, "wavefront" );

    f32x4 sa = f32x4 { 0.0f, 0.0f, 0.0f, 0.0f };
    f32x4 sb = f32x4 { 0.0f, 0.0f, 0.0f, 0.0f };
#pragma unroll
    for ( int kk = 0; kk < 4; kk++ ) {
      const uint32_t at = c * 16 + ( ( 4 * kk + g4 ) ^ c );
      sa = __builtin_amdgcn_mfma_f32_16x16x32_f16( __builtin_bit_cast( f16x8, tile_a[at] ), qb[kk], sa, 0, 0, 0 );
      sb = __builtin_amdgcn_mfma_f32_16x16x32_f16( __builtin_bit_cast( f16x8, tile_b[at] ), qb[kk], sb, 0, 0, 0 );
    }
    __builtin_amdgcn_fence( __ATOMIC_RELEASE, "wavefront" );
    __builtin_amdgcn_wave_barrier(); // the tiles are rewritten at the top of the next iteration

    if ( c < G ) {
      const float v[8] = { scale * sa[0], scale * sa[1], scale * sa[2], scale * sa[3], scale * sb[0], scale * sb[1], scale * sb[2], scale * sb[3] };
      store_scores8( out_row, t0 + 8 * g4, job.t_end, v );
    }
    t0 = t_next;
  }
}

// =================================================================================================
// scores, gqa 1 / 2: lane = (r = lane / 16, c = lane % 16); the 16 lanes of a row share a token's head row
// =================================================================================================
template<int G>
__global__ __launch_bounds__( 256 ) void attn_scores_valu_kernel( const __half* __restrict__ q,
                                                                  const __half* const* __restrict__ layer_rows,
                                                                  const uint32_t* __restrict__ pos,
                                                                  __half* __restrict__ att,
                                                                  uint32_t n_kv_heads,
                                                                  uint32_t seq_len,
                                                                  uint32_t chunk,
                                                                  uint32_t max_splits,
                                                                  float scale )
{
  const WaveJob job = wave_job( layer_rows, pos, n_kv_heads, chunk, max_splits, seq_len );
  if ( !job.valid ) {
    return;
  }
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t r = lane >> 4;
  const uint32_t n_heads = n_kv_heads * G;
  const uint64_t row_elems = 2ull * n_kv_heads * HS;

  uint4 qr[G];
  {
    const __half* qp = q + ( (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G ) * HS + 8 * c;
#pragma unroll
    for ( int g = 0; g < G; g++ ) {
      qr[g] = load16( qp + g * HS );
    }
  }
  __half* out_row = att + ( (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G + ( c < G ? c : 0 ) ) * seq_len;
  const __half* kp = job.base + (uint64_t)job.h * HS + 8 * c;

  const uint32_t n_it = ( job.t_end - job.t_begin + TOK_PER_IT - 1 ) / TOK_PER_IT;
  uint32_t it_i = ( ( job.ctx * 5u + job.split * 3u ) * 7u ) % n_it;
  uint32_t t0 = job.t_begin + TOK_PER_IT * it_i;
  uint4 kn[8];
  load_rows8( kn, kp, row_elems, t0 + 8 * r, job.t_end, true );

  for ( uint32_t it = 0; it < n_it; it++ ) {
    it_i = it_i + 1 == n_it ? 0 : it_i + 1;
    const uint32_t t_next = job.t_begin + TOK_PER_IT * it_i;
    uint4 kc[8];
#pragma unroll
    for ( int i = 0; i < 8; i++ ) {
      kc[i] = kn[i];
    }
    load_rows8( kn, kp, row_elems, t_next + 8 * r, job.t_end, it + 1 < n_it );
    float mine[8];
#pragma unroll
    for ( int i = 0; i < 8; i++ ) {
      mine[i] = 0.0f;
    }
#pragma unroll
    for ( int g = 0; g < G; g++ ) {
#pragma unroll
      for ( int i = 0; i < 8; i++ ) {
        const float d = row16_sum( dot8( kc[i], qr[g], 0.0f ) );
        if ( (int)c == g ) {
          mine[i] = scale * d;
        }
      }
    }
    if ( c < G ) {
      store_scores8( out_row, t0 + 8 * r, job.t_end, mine );
    }
    t0 = t_next;
  }
}

// =================================================================================================
// softmax with the row in registers: block <-> (head, context), thread t owns the 16-byte chunks t, t + 256, ...
// =================================================================================================
template<int NCH>
__global__ __launch_bounds__( 256 ) void attn_softmax_row_kernel( __half* __restrict__ att, const uint32_t* __restrict__ pos, uint32_t n_heads, uint32_t seq_len )
{
  __shared__ float s_red[2][4];
  const uint32_t ctx = blockIdx.y;
  const uint32_t head = blockIdx.x;
  const uint32_t n = min( pos[ctx] + 1, seq_len );
  __half* row = att + ( (uint64_t)ctx * n_heads + head ) * seq_len;

  union Chunk
  {
    uint4 raw;
    __half h[8];
  };
  Chunk v[NCH];
  float mx = -INFINITY;
#pragma unroll
  for ( int k = 0; k < NCH; k++ ) {
    const uint32_t base = ( threadIdx.x + 256u * k ) * 8u;
    if ( base < n ) {
      v[k].raw = *reinterpret_cast<const uint4*>( row + base ); // a row is seq_len elements, a multiple of 8: the chunk lies inside it
#pragma unroll
      for ( int e = 0; e < 8; e++ ) {
        if ( base + e < n ) {
          mx = fmaxf( mx, __half2float( v[k].h[e] ) );
        }
      }
    }
  }
  mx = wave_max( mx );
  if ( threadIdx.x % WAVE == 0 ) {
    s_red[0][threadIdx.x / WAVE] = mx;
  }
  __syncthreads();
  mx = fmaxf( fmaxf( s_red[0][0], s_red[0][1] ), fmaxf( s_red[0][2], s_red[0][3] ) );

  float sum = 0.0f;
#pragma unroll
  for ( int k = 0; k < NCH; k++ ) {
    const uint32_t base = ( threadIdx.x + 256u * k ) * 8u;
    if ( base < n ) {
#pragma unroll
      for ( int e = 0; e < 8; e++ ) {
        if ( base + e < n ) {
          const __half diff = __float2half_rn( __half2float( v[k].h[e] ) - mx );
          const __half ex = __float2half_rn( expf( __half2float( diff ) ) );
          v[k].h[e] = ex;
          sum += __half2float( ex );
        }
      }
    }
  }
  sum = wave_sum( sum );
  if ( threadIdx.x % WAVE == 0 ) {
    s_red[1][threadIdx.x / WAVE] = sum;
  }
  __syncthreads();
  sum = s_red[1][0] + s_red[1][1] + s_red[1][2] + s_red[1][3];

#pragma unroll
  for ( int k = 0; k < NCH; k++ ) {
    const uint32_t base = ( threadIdx.x + 256u * k ) * 8u;
    if ( base < n ) {
#pragma unroll
      for ( int e = 0; e < 8; e++ ) {
        if ( base + e < n ) {
          v[k].h[e] = __float2half_rn( __half2float( v[k].h[e] ) / sum );
        }
      }
      *reinterpret_cast<uint4*>( row + base ) = v[k].raw; // elements beyond pos go back unchanged
    }
  }
}

// =================================================================================================
// weighted sum.  Partial sums per token range: part[(context * n_heads + head) * max_splits + split][head_size] fp32
// =================================================================================================
template<int G>
__global__ __launch_bounds__( 256 ) void attn_pv_mfma_kernel( const __half* __restrict__ att,
                                                              const __half* const* __restrict__ layer_rows,
                                                              const uint32_t* __restrict__ pos,
                                                              float* __restrict__ part,
                                                              __half* __restrict__ xb,
                                                              uint32_t n_kv_heads,
                                                              uint32_t seq_len,
                                                              uint32_t chunk,
                                                              uint32_t max_splits )
{
  const WaveJob job = wave_job( layer_rows, pos, n_kv_heads, chunk, max_splits, seq_len );
  if ( !job.valid ) {
    return;
  }
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t g4 = lane >> 4;
  const uint32_t n_heads = n_kv_heads * G;
  const uint64_t row_elems = 2ull * n_kv_heads * HS;
  const __half* vp = job.base + (uint64_t)n_kv_heads * HS + (uint64_t)job.h * HS + 8 * c;
  const __half* p_row = att + ( (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G + ( c < G ? c : 0 ) ) * seq_len;

  f32x4 acc[8];
#pragma unroll
  for ( int nn = 0; nn < 8; nn++ ) {
    acc[nn] = f32x4 { 0.0f, 0.0f, 0.0f, 0.0f };
  }

  const uint32_t n_it = ( job.t_end - job.t_begin + TOK_PER_IT - 1 ) / TOK_PER_IT;
  uint32_t it_i = ( ( job.ctx * 5u + job.split * 3u ) * 7u ) % n_it;
  uint32_t t0 = job.t_begin + TOK_PER_IT * it_i;
  const uint4 zero4 = make_uint4( 0, 0, 0, 0 );

  // the weights of this lane's 8 tokens for head c: one 16-byte load (zero for padding heads and tokens past the range;
  // a chunk that straddles the end of the range is cut element by element)
  auto load_p = [&]( uint32_t tok0, bool any ) -> uint4 {
    if ( !any || c >= G || tok0 >= job.t_end ) {
      return zero4;
    }
    union
    {
      uint4 raw;
      uint16_t h[8];
    } p;
    p.raw = load16( p_row + tok0 );
    if ( tok0 + 8 > job.t_end ) {
#pragma unroll
      for ( int e = 0; e < 8; e++ ) {
        if ( tok0 + e >= job.t_end ) {
          p.h[e] = 0;
        }
      }
    }
    return p.raw;
  };

  uint4 vn[8];
  load_rows8( vn, vp, row_elems, t0 + 8 * g4, job.t_end, true );
  uint4 pn = load_p( t0 + 8 * g4, true );

  for ( uint32_t it = 0; it < n_it; it++ ) {
    it_i = it_i + 1 == n_it ? 0 : it_i + 1;
    const uint32_t t_next = job.t_begin + TOK_PER_IT * it_i;
    uint4 vc[8];
#pragma unroll
    for ( int i = 0; i < 8; i++ ) {
      vc[i] = vn[i];
    }
    const uint4 pc = pn;
    load_rows8( vn, vp, row_elems, t_next + 8 * g4, job.t_end, it + 1 < n_it );
    pn = load_p( t_next + 8 * g4, it + 1 < n_it );

    // P as A fragments (head c, the lane's tokens 0..3 and 4..7); V as B fragments transposed out of the row chunks
    const f16x4 pa = __builtin_bit_cast( f16x4, make_uint2( pc.x, pc.y ) );
    const f16x4 pb = __builtin_bit_cast( f16x4, make_uint2( pc.z, pc.w ) );
    const uint32_t va[4][4] = { { vc[0].x, vc[0].y, vc[0].z, vc[0].w }, { vc[1].x, vc[1].y, vc[1].z, vc[1].w },
                                { vc[2].x, vc[2].y, vc[2].z, vc[2].w }, { vc[3].x, vc[3].y, vc[3].z, vc[3].w } };
    const uint32_t vb[4][4] = { { vc[4].x, vc[4].y, vc[4].z, vc[4].w }, { vc[5].x, vc[5].y, vc[5].z, vc[5].w },
                                { vc[6].x, vc[6].y, vc[6].z, vc[6].w }, { vc[7].x, vc[7].y, vc[7].z, vc[7].w } };
#pragma unroll
    for ( int w = 0; w < 4; w++ ) {
      const uint2 lo_a = make_uint2( __builtin_amdgcn_perm( va[1][w], va[0][w], 0x05040100u ), __builtin_amdgcn_perm( va[3][w], va[2][w], 0x05040100u ) );
      const uint2 hi_a = make_uint2( __builtin_amdgcn_perm( va[1][w], va[0][w], 0x07060302u ), __builtin_amdgcn_perm( va[3][w], va[2][w], 0x07060302u ) );
      const uint2 lo_b = make_uint2( __builtin_amdgcn_perm( vb[1][w], vb[0][w], 0x05040100u ), __builtin_amdgcn_perm( vb[3][w], vb[2][w], 0x05040100u ) );
      const uint2 hi_b = make_uint2( __builtin_amdgcn_perm( vb[1][w], vb[0][w], 0x07060302u ), __builtin_amdgcn_perm( vb[3][w], vb[2][w], 0x07060302u ) );
      acc[2 * w] = __builtin_amdgcn_mfma_f32_16x16x16f16( pa, __builtin_bit_cast( f16x4, lo_a ), acc[2 * w], 0, 0, 0 );
      acc[2 * w + 1] = __builtin_amdgcn_mfma_f32_16x16x16f16( pa, __builtin_bit_cast( f16x4, hi_a ), acc[2 * w + 1], 0, 0, 0 );
      acc[2 * w] = __builtin_amdgcn_mfma_f32_16x16x16f16( pb, __builtin_bit_cast( f16x4, lo_b ), acc[2 * w], 0, 0, 0 );
      acc[2 * w + 1] = __builtin_amdgcn_mfma_f32_16x16x16f16( pb, __builtin_bit_cast( f16x4, hi_b ), acc[2 * w + 1], 0, 0, 0 );
    }
    t0 = t_next;
  }

  // acc[nn][i] = O[head 4*g4 + i][dim 8*c + nn]
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    const uint32_t hd = 4 * g4 + i;
    if ( hd < G ) {
      const uint64_t head = (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G + hd;
      if ( max_splits == 1 ) {
        const uint2 a = pack4( acc[0][i], acc[1][i], acc[2][i], acc[3][i] );
        const uint2 b = pack4( acc[4][i], acc[5][i], acc[6][i], acc[7][i] );
        *reinterpret_cast<uint4*>( xb + head * HS + 8 * c ) = make_uint4( a.x, a.y, b.x, b.y );
      } else {
        float4* o = reinterpret_cast<float4*>( part + ( head * max_splits + job.split ) * HS + 8 * c );
        o[0] = make_float4( acc[0][i], acc[1][i], acc[2][i], acc[3][i] );
        o[1] = make_float4( acc[4][i], acc[5][i], acc[6][i], acc[7][i] );
      }
    }
  }
}

template<int G>
__global__ __launch_bounds__( 256 ) void attn_pv_valu_kernel( const __half* __restrict__ att,
                                                              const __half* const* __restrict__ layer_rows,
                                                              const uint32_t* __restrict__ pos,
                                                              float* __restrict__ part,
                                                              __half* __restrict__ xb,
                                                              uint32_t n_kv_heads,
                                                              uint32_t seq_len,
                                                              uint32_t chunk,
                                                              uint32_t max_splits )
{
  const WaveJob job = wave_job( layer_rows, pos, n_kv_heads, chunk, max_splits, seq_len );
  if ( !job.valid ) {
    return;
  }
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t r = lane >> 4;
  const uint32_t n_heads = n_kv_heads * G;
  const uint64_t row_elems = 2ull * n_kv_heads * HS;
  const __half* vp = job.base + (uint64_t)n_kv_heads * HS + (uint64_t)job.h * HS + 8 * c;
  const __half* p_rows = att + ( (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G ) * seq_len;

  float acc[G][8];
#pragma unroll
  for ( int g = 0; g < G; g++ ) {
#pragma unroll
    for ( int e = 0; e < 8; e++ ) {
      acc[g][e] = 0.0f;
    }
  }
  const uint32_t n_it = ( job.t_end - job.t_begin + TOK_PER_IT - 1 ) / TOK_PER_IT;
  uint32_t it_i = ( ( job.ctx * 5u + job.split * 3u ) * 7u ) % n_it;
  uint32_t t0 = job.t_begin + TOK_PER_IT * it_i;
  uint4 vn[8];
  load_rows8( vn, vp, row_elems, t0 + 8 * r, job.t_end, true );

  for ( uint32_t it = 0; it < n_it; it++ ) {
    it_i = it_i + 1 == n_it ? 0 : it_i + 1;
    const uint32_t t_next = job.t_begin + TOK_PER_IT * it_i;
    uint4 vc[8];
#pragma unroll
    for ( int i = 0; i < 8; i++ ) {
      vc[i] = vn[i];
    }
    load_rows8( vn, vp, row_elems, t_next + 8 * r, job.t_end, it + 1 < n_it );
    const uint32_t tok0 = t0 + 8 * r;
    if ( tok0 < job.t_end ) { // uniform within the 16 lanes of a row
      float v[8][8];
#pragma unroll
      for ( int i = 0; i < 8; i++ ) {
        unpack8( vc[i], v[i] );
      }
#pragma unroll
      for ( int g = 0; g < G; g++ ) {
        // the weights of the 8 tokens for head g: the same 16 bytes for all 16 lanes of the row
        union
        {
          uint4 raw;
          __half h[8];
        } p;
        p.raw = load16( p_rows + (uint64_t)g * seq_len + tok0 );
#pragma unroll
        for ( int i = 0; i < 8; i++ ) {
          const float w = tok0 + i < job.t_end ? __half2float( p.h[i] ) : 0.0f;
#pragma unroll
          for ( int e = 0; e < 8; e++ ) {
            acc[g][e] += w * v[i][e];
          }
        }
      }
    }
    t0 = t_next;
  }

  // add the four token groups of the wave
#pragma unroll
  for ( int g = 0; g < G; g++ ) {
#pragma unroll
    for ( int e = 0; e < 8; e++ ) {
      float a = acc[g][e];
      a += __shfl_xor( a, 16, WAVE );
      a += __shfl_xor( a, 32, WAVE );
      acc[g][e] = a;
    }
  }
  if ( r == 0 ) {
#pragma unroll
    for ( int g = 0; g < G; g++ ) {
      const uint64_t head = (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G + g;
      if ( max_splits == 1 ) {
        const uint2 a = pack4( acc[g][0], acc[g][1], acc[g][2], acc[g][3] );
        const uint2 b = pack4( acc[g][4], acc[g][5], acc[g][6], acc[g][7] );
        *reinterpret_cast<uint4*>( xb + head * HS + 8 * c ) = make_uint4( a.x, a.y, b.x, b.y );
      } else {
        float4* o = reinterpret_cast<float4*>( part + ( head * max_splits + job.split ) * HS + 8 * c );
        o[0] = make_float4( acc[g][0], acc[g][1], acc[g][2], acc[g][3] );
        o[1] = make_float4( acc[g][4], acc[g][5], acc[g][6], acc[g][7] );
      }
    }
  }
}

// sum of the token-range partials: block <-> (query head, context), thread <-> output dim
__global__ __launch_bounds__( 128 ) void attn_pv_merge_kernel( const float* __restrict__ part,
                                                               const void* const* __restrict__ layer_rows,
                                                               const uint32_t* __restrict__ pos,
                                                               __half* __restrict__ xb,
                                                               uint32_t n_heads,
                                                               uint32_t chunk,
                                                               uint32_t max_splits )
{
  const uint32_t head = blockIdx.x;
  const uint32_t ctx = blockIdx.y;
  if ( layer_rows[ctx] == nullptr ) {
    return;
  }
  const uint32_t n_splits = min( ( pos[ctx] + chunk ) / chunk, max_splits );
  const uint64_t slot0 = ( (uint64_t)ctx * n_heads + head ) * max_splits;
  const uint32_t d = threadIdx.x;
  float acc = 0.0f;
  for ( uint32_t s = 0; s < n_splits; s++ ) {
    acc += part[( slot0 + s ) * HS + d];
  }
  xb[( (uint64_t)ctx * n_heads + head ) * HS + d] = __float2half_rn( acc );
}

// token ranges of the streaming kernels: about `target_waves` waves in flight, ranges of at least 256 tokens, whole iterations
struct RangePlan
{
  uint32_t chunk;
  uint32_t max_splits;
};

RangePlan range_plan( uint64_t batch, uint32_t n_kv_heads, uint32_t max_tok, uint64_t target_waves )
{
  const uint64_t streams = std::max<uint64_t>( 1, batch * n_kv_heads );
  const uint64_t splits = streams >= target_waves ? 1 : ( target_waves + streams - 1 ) / streams;
  uint32_t chunk = (uint32_t)( ( max_tok + splits - 1 ) / splits );
  chunk = std::max<uint32_t>( chunk, 256 );
  chunk = ( chunk + TOK_PER_IT - 1 ) / TOK_PER_IT * TOK_PER_IT;
  RangePlan p;
  p.chunk = chunk;
  p.max_splits = std::max<uint32_t>( 1, ( max_tok + chunk - 1 ) / chunk );
  return p;
}

bool streaming_ok( const gh_shape* s, gh_dtype dt, const void* a, const void* b )
{
  const uint32_t g = s->gqa_size;
  return dt == GH_F16 && s->head_size == HS && s->seq_len % 8 == 0 && ( g == 1 || g == 2 || g == 4 || g == 8 || g == 16 )
         && ( ( reinterpret_cast<uintptr_t>( a ) | reinterpret_cast<uintptr_t>( b ) ) & 15u ) == 0;
}

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

// `max_tok`: host-side upper bound of pos + 1 over the batch (seq_len when the positions only live on the device); it sizes the grid
static int scores_run( const void* q, const void* const* layer_rows_dev, void* att, uint64_t batch, const uint32_t* pos_dev, const gh_shape* shape,
                       gh_dtype dt, gh_stream stream, uint32_t max_tok )
{
  if ( int rc = check_shape( shape, batch, "gh_attn_scores" ) ) {
    return rc;
  }
  GH_REQUIRE( q && layer_rows_dev && att && pos_dev, "gh_attn_scores: NULL pointer" );
  GH_REQUIRE( max_tok >= 1 && max_tok <= shape->seq_len, "gh_attn_scores: position bound %u outside seq_len %u", max_tok, shape->seq_len );
  hipStream_t st = as_stream( stream );
  const float scale = 1.0f / sqrtf( (float)shape->head_size );
  if ( streaming_ok( shape, dt, q, att ) ) {
    const RangePlan plan = range_plan( batch, shape->n_kv_heads, max_tok, 4096 );
    const uint64_t n_blocks = batch * plan.max_splits * ( ( shape->n_kv_heads + 3 ) / 4 );
    GH_REQUIRE( n_blocks <= 0x7fffffffull, "gh_attn_scores: grid too large" );
    const dim3 grid( (unsigned)n_blocks );
    const __half* qh = static_cast<const __half*>( q );
    const __half* const* rows = reinterpret_cast<const __half* const*>( layer_rows_dev );
    __half* ah = static_cast<__half*>( att );
#define GH_SCORES( KERNEL, G ) KERNEL<G><<<grid, 256, 0, st>>>( qh, rows, pos_dev, ah, shape->n_kv_heads, shape->seq_len, plan.chunk, plan.max_splits, scale )
    switch ( shape->gqa_size ) {
      case 1: GH_SCORES( attn_scores_valu_kernel, 1 ); break;
      case 2: GH_SCORES( attn_scores_valu_kernel, 2 ); break;
      case 4: GH_SCORES( attn_scores_mfma_kernel, 4 ); break;
      case 8: GH_SCORES( attn_scores_mfma_kernel, 8 ); break;
      default: GH_SCORES( attn_scores_mfma_kernel, 16 ); break;
    }
#undef GH_SCORES
    GH_LAUNCH_CHECK();
    return GH_OK;
  }
  const dim3 grid( ( max_tok + 255 ) / 256, shape->n_kv_heads, (unsigned)batch );
  const size_t smem = (size_t)shape->gqa_size * shape->head_size * sizeof( float );
  if ( dt == GH_F16 ) {
    attn_scores_kernel<__half><<<grid, 256, smem, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( layer_rows_dev ),
                                                        static_cast<__half*>( att ), pos_dev, shape->n_kv_heads, shape->gqa_size, shape->head_size,
                                                        shape->seq_len, scale );
  } else if ( dt == GH_F32 ) {
    attn_scores_kernel<float><<<grid, 256, smem, st>>>( static_cast<const float*>( q ), reinterpret_cast<const float* const*>( layer_rows_dev ),
                                                       static_cast<float*>( att ), pos_dev, shape->n_kv_heads, shape->gqa_size, shape->head_size,
                                                       shape->seq_len, scale );
  } else {
    return fail( GH_ERR_INVALID, "gh_attn_scores: unsupported dtype %d", (int)dt );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

static int pv_run( const void* att, const void* const* layer_rows_dev, void* xb, uint64_t batch, const uint32_t* pos_dev, const gh_shape* shape,
                   gh_dtype dt, gh_stream stream, uint32_t max_tok )
{
  if ( int rc = check_shape( shape, batch, "gh_attn_pv" ) ) {
    return rc;
  }
  GH_REQUIRE( att && layer_rows_dev && xb && pos_dev, "gh_attn_pv: NULL pointer" );
  GH_REQUIRE( max_tok >= 1 && max_tok <= shape->seq_len, "gh_attn_pv: position bound %u outside seq_len %u", max_tok, shape->seq_len );
  hipStream_t st = as_stream( stream );
  if ( streaming_ok( shape, dt, att, xb ) ) {
    const RangePlan plan = range_plan( batch, shape->n_kv_heads, max_tok, 2048 );
    const uint64_t n_blocks = batch * plan.max_splits * ( ( shape->n_kv_heads + 3 ) / 4 );
    GH_REQUIRE( n_blocks <= 0x7fffffffull, "gh_attn_pv: grid too large" );
    float* part = nullptr;
    if ( plan.max_splits > 1 ) {
      void* p = nullptr;
      if ( int rc = stream_scratch( st, SCRATCH_ATTN_PV, batch * shape->n_heads * (uint64_t)plan.max_splits * HS * sizeof( float ), 16ull << 20, &p ) ) {
        return rc;
      }
      part = static_cast<float*>( p );
    }
    const dim3 grid( (unsigned)n_blocks );
    const __half* ah = static_cast<const __half*>( att );
    const __half* const* rows = reinterpret_cast<const __half* const*>( layer_rows_dev );
    __half* oh = static_cast<__half*>( xb );
#define GH_PV( KERNEL, G ) KERNEL<G><<<grid, 256, 0, st>>>( ah, rows, pos_dev, part, oh, shape->n_kv_heads, shape->seq_len, plan.chunk, plan.max_splits )
    switch ( shape->gqa_size ) {
      case 1: GH_PV( attn_pv_valu_kernel, 1 ); break;
      case 2: GH_PV( attn_pv_valu_kernel, 2 ); break;
      case 4: GH_PV( attn_pv_mfma_kernel, 4 ); break;
      case 8: GH_PV( attn_pv_mfma_kernel, 8 ); break;
      default: GH_PV( attn_pv_mfma_kernel, 16 ); break;
    }
#undef GH_PV
    GH_LAUNCH_CHECK();
    if ( plan.max_splits > 1 ) {
      attn_pv_merge_kernel<<<dim3( shape->n_heads, (unsigned)batch ), HS, 0, st>>>( part, layer_rows_dev, pos_dev, oh, shape->n_heads, plan.chunk,
                                                                                  plan.max_splits );
      GH_LAUNCH_CHECK();
    }
    return GH_OK;
  }
  const unsigned n_slices = 256 / shape->head_size ? 256 / shape->head_size : 1;
  const unsigned threads = n_slices * shape->head_size;
  const dim3 grid( shape->n_kv_heads, (unsigned)batch );
  const size_t smem = (size_t)n_slices * shape->gqa_size * shape->head_size * sizeof( float );
  GH_REQUIRE( smem <= 64 * 1024, "gh_attn_pv: gqa_size * head_size too large for the reduction buffer" );
  if ( dt == GH_F16 ) {
    attn_pv_kernel<__half><<<grid, threads, smem, st>>>( static_cast<const __half*>( att ), reinterpret_cast<const __half* const*>( layer_rows_dev ),
                                                        static_cast<__half*>( xb ), pos_dev, shape->n_kv_heads, shape->gqa_size, shape->head_size,
                                                        shape->seq_len );
  } else if ( dt == GH_F32 ) {
    attn_pv_kernel<float><<<grid, threads, smem, st>>>( static_cast<const float*>( att ), reinterpret_cast<const float* const*>( layer_rows_dev ),
                                                       static_cast<float*>( xb ), pos_dev, shape->n_kv_heads, shape->gqa_size, shape->head_size,
                                                       shape->seq_len );
  } else {
    return fail( GH_ERR_INVALID, "gh_attn_pv: unsupported dtype %d", (int)dt );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

static uint32_t max_tokens_of( const void* const* rows_host, const uint32_t* pos_host, uint64_t batch, uint32_t seq_len )
{
  uint32_t m = 1;
  for ( uint64_t i = 0; i < batch; i++ ) {
    if ( rows_host == nullptr || rows_host[i] != nullptr ) {
      m = std::max( m, pos_host[i] < seq_len ? pos_host[i] + 1 : seq_len + 1 );
    }
  }
  return m;
}

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
  GH_REQUIRE( shape != nullptr, "gh_attn_scores: NULL shape" );
  return scores_run( q, layer_rows_dev, att, batch, pos_dev, shape, dt, stream, shape->seq_len );
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
  hipStream_t st = as_stream( stream );
  if ( dt == GH_F16 && shape->seq_len % 8 == 0 && shape->seq_len <= 8192 && ( reinterpret_cast<uintptr_t>( att ) & 15u ) == 0 ) {
    __half* ah = static_cast<__half*>( att );
    if ( shape->seq_len <= 2048 ) {
      attn_softmax_row_kernel<1><<<grid, 256, 0, st>>>( ah, pos_dev, shape->n_heads, shape->seq_len );
    } else if ( shape->seq_len <= 4096 ) {
      attn_softmax_row_kernel<2><<<grid, 256, 0, st>>>( ah, pos_dev, shape->n_heads, shape->seq_len );
    } else {
      attn_softmax_row_kernel<4><<<grid, 256, 0, st>>>( ah, pos_dev, shape->n_heads, shape->seq_len );
    }
  } else if ( dt == GH_F16 ) {
    attn_softmax_kernel<__half><<<grid, 256, 0, st>>>( static_cast<__half*>( att ), pos_dev, shape->n_heads, shape->seq_len );
  } else if ( dt == GH_F32 ) {
    attn_softmax_kernel<float><<<grid, 256, 0, st>>>( static_cast<float*>( att ), pos_dev, shape->n_heads, shape->seq_len );
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
  GH_REQUIRE( shape != nullptr, "gh_attn_pv: NULL shape" );
  return pv_run( att, layer_rows_dev, xb, batch, pos_dev, shape, dt, stream, shape->seq_len );
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
  GH_REQUIRE( shape != nullptr, "gh_attn_scores_host: NULL shape" );
  const uint32_t max_tok = max_tokens_of( layer_rows_host, pos_host, batch, shape->seq_len );
  if ( int rc = scores_run( q, d_rows, att, batch, d_pos, shape, dt, stream, max_tok ) ) {
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
  GH_REQUIRE( shape != nullptr, "gh_attn_pv_host: NULL shape" );
  const uint32_t max_tok = max_tokens_of( layer_rows_host, pos_host, batch, shape->seq_len );
  if ( int rc = pv_run( att, d_rows, xb, batch, d_pos, shape, dt, stream, max_tok ) ) {
    return rc;
  }
  return scope.finish();
}

} // extern "C"
