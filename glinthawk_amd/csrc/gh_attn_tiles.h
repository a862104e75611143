// Device helpers shared by the attention kernels that stream cache rows with the wave <-> (context, kv head,
// token range) decomposition (fused decode attention, unfused scores and weighted-sum kernels): operand vector
// types, the wave's job, 16-lane DPP reductions, streaming 16-byte loads.  f16 storage, head size 128.
#pragma once

#include "gh_common.h"

namespace gh {

constexpr int HS = 128; // head size of the fast kernels

typedef _Float16 f16x4 __attribute__( ( ext_vector_type( 4 ) ) );
typedef _Float16 f16x8 __attribute__( ( ext_vector_type( 8 ) ) );
typedef _Float16 f16x2 __attribute__( ( ext_vector_type( 2 ) ) );
typedef float f32x4 __attribute__( ( ext_vector_type( 4 ) ) );


__device__ __forceinline__ float fast_exp2( float x ) { return __builtin_amdgcn_exp2f( x ); }


struct WaveJob
{
  const __half* base; // layer rows of the context
  uint32_t ctx, h, split, t_begin, t_end;
  bool valid;
};

// block -> (group of 4 kv heads, split, context); wave -> kv head.  Adjacent blocks cover adjacent
// head groups of the same token range so that concurrently running blocks read whole cache rows.
__device__ __forceinline__ WaveJob wave_job( const __half* const* layer_rows,
                                             const uint32_t* pos,
                                             uint32_t n_kv_heads,
                                             uint32_t chunk,
                                             uint32_t max_splits,
                                             uint32_t seq_len )
{
  WaveJob j;
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t n_hg = ( n_kv_heads + 3 ) / 4;
  uint32_t bid = blockIdx.x;
  const uint32_t hg = bid % n_hg;
  bid /= n_hg;
  j.split = bid % max_splits;
  j.ctx = bid / max_splits;
  j.h = hg * 4 + wave;
  j.base = layer_rows[j.ctx];
  // never beyond what the host sized the grid and the partials for, nor beyond the rows a context has (chunks are rounded up, so
  // max_splits * chunk may exceed seq_len; the positions come from device memory and are not checked by the host)
  const uint32_t n_tok = min( min( pos[j.ctx] + 1, max_splits * chunk ), seq_len );
  j.t_begin = j.split * chunk;
  j.t_end = min( n_tok, j.t_begin + chunk );
  j.valid = j.h < n_kv_heads && j.base != nullptr && j.t_begin < n_tok;
  return j;
}

// Cache rows are reached through pointers that come out of a table, so the compiler cannot tell that they are global memory
// and would use flat loads.  Those count against the LDS wait counter as well: a wait for an LDS read would then also wait for
// the rows of the next tile, which are meant to stay in flight.  The casts below name the address space.
typedef uint32_t u32x4_t __attribute__( ( ext_vector_type( 4 ) ) );
typedef const u32x4_t __attribute__( ( address_space( 1 ) ) ) global_u32x4_t;
__device__ __forceinline__ uint4 load16( const __half* p ) { return __builtin_bit_cast( uint4, *(global_u32x4_t*)( p ) ); }
// cache rows are read once per launch: non-temporal, so that they do not push the queries and partials out of the L2
__device__ __forceinline__ uint4 load16_stream( const __half* p )
{
  return __builtin_bit_cast( uint4, __builtin_nontemporal_load( (global_u32x4_t*)( p ) ) );
}

__device__ __forceinline__ float dot8( const uint4& a, const uint4& b, float acc )
{
  acc = __builtin_amdgcn_fdot2( __builtin_bit_cast( f16x2, a.x ), __builtin_bit_cast( f16x2, b.x ), acc, false );
  acc = __builtin_amdgcn_fdot2( __builtin_bit_cast( f16x2, a.y ), __builtin_bit_cast( f16x2, b.y ), acc, false );
  acc = __builtin_amdgcn_fdot2( __builtin_bit_cast( f16x2, a.z ), __builtin_bit_cast( f16x2, b.z ), acc, false );
  acc = __builtin_amdgcn_fdot2( __builtin_bit_cast( f16x2, a.w ), __builtin_bit_cast( f16x2, b.w ), acc, false );
  return acc;
}

__device__ __forceinline__ void unpack8( const uint4& v, float out[8] )
{
  const uint32_t w[4] = { v.x, v.y, v.z, v.w };
#pragma unroll
  for ( int k = 0; k < 4; k++ ) {
    const f16x2 h2 = __builtin_bit_cast( f16x2, w[k] );
    out[2 * k] = (float)h2.x;
    out[2 * k + 1] = (float)h2.y;
  }
}


} // namespace gh
