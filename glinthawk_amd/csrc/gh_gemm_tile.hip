// Large-batch GEMM for prefill: xout(b, r) = sum_p w(r, p) * x(b, p) with b in the hundreds or
// thousands (all prompt tokens of a batch at once), f16 storage, fp32 accumulate.  This regime is
// MFMA-bound, not HBM-bound: both operands are re-used across a 128 x 128 output tile.
//
//   work-group = 4 waves (2 x 2), tile 128 weight rows x 128 tokens, K in steps of 64
//   wave        = 64 x 64 = 2 x 2 accumulators of v_mfma_f32_32x32x16_f16
//   operands    global -> registers (next step in flight while the current one is multiplied)
//               -> LDS, 16-byte chunks XOR-swizzled so that the MFMA-order reads are conflict free,
//               two LDS buffers, one barrier per step
//   output      through LDS, token-major, then whole row segments of 16 bytes per lane (f16 and fp32
//               partials alike): 5-7 % faster than storing from the accumulator registers where K is
//               not split, no change where it is
//   tile order  work-groups reach the 8 XCDs round robin by linear index and each XCD has its own L2.
//               An XCD owns every 8th row tile and walks its (row tile, token tile) grid in patches
//               of GM x GN tiles that are resident together (64 = 2 work-groups on each of its 32
//               CUs): a patch re-reads GM weight tiles and GN activation tiles out of L2 instead of
//               64 + 64 from memory.  Row-major order re-streamed the whole weight matrix once per
//               token tile and was bound by that (4.5 TB/s), not by MFMA.
//   split K     when the tiles are too few to fill the chip, K is split across work-groups and the
//               fp32 partials (splits, b, r) are summed by the caller's reduce / fused epilogue
#include "gh_common.h"

#include <algorithm>

namespace gh {

typedef _Float16 f16x8 __attribute__( ( ext_vector_type( 8 ) ) );
typedef float f32x16 __attribute__( ( ext_vector_type( 16 ) ) );

namespace {

constexpr int TM = 128; // weight rows per work-group
constexpr int TN = 128; // tokens per work-group
constexpr int TK = 64;  // k per step: 8 chunks of 8 halves

struct Frag
{
  uint4 v[4]; // thread t: row t/8 + 32*i, chunk t%8
};

__device__ __forceinline__ void load_frag( Frag& f, const __half* __restrict__ mat, uint64_t ld, uint32_t row0, uint32_t n_rows, uint32_t k0, uint32_t k_end )
{
  const uint32_t chunk = threadIdx.x & 7;
  const uint32_t k = k0 + 8 * chunk;
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    const uint32_t row = row0 + ( threadIdx.x >> 3 ) + 32 * i;
    f.v[i] = ( row < n_rows && k < k_end ) ? *reinterpret_cast<const uint4*>( mat + (uint64_t)row * ld + k ) : make_uint4( 0, 0, 0, 0 );
  }
}

// rows are 128 bytes (8 chunks); chunk position is XORed with bits 1..3 of the row so that 16 rows
// of one chunk column fall into 16 different 16-byte bank groups
__device__ __forceinline__ uint32_t swz( uint32_t row, uint32_t chunk ) { return row * 8 + ( chunk ^ ( ( row >> 1 ) & 7 ) ); }

__device__ __forceinline__ void store_frag( uint4* tile, const Frag& f )
{
  const uint32_t chunk = threadIdx.x & 7;
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    const uint32_t row = ( threadIdx.x >> 3 ) + 32 * i;
    tile[swz( row, chunk )] = f.v[i];
  }
}

struct TileOrder
{
  uint32_t row_tiles, token_tiles; // of the whole product
  uint32_t gm, gn;                 // patch: row tiles x token tiles
  uint32_t patches_n;              // patches along the token direction
};

// grid: (8 * padded tiles per XCD, 1, k splits).  s % 8 == 0, 16-byte aligned operands.
template<bool SPLIT>
__global__ __launch_bounds__( 256 ) void gemm_tile_kernel( __half* __restrict__ xout,
                                                           float* __restrict__ partial,
                                                           const __half* __restrict__ x,
                                                           const __half* __restrict__ w,
                                                           uint32_t s,
                                                           uint32_t r,
                                                           uint32_t b,
                                                           uint32_t k_per_split,
                                                           TileOrder ord )
{
  __shared__ uint4 s_w[2][TM * 8]; // 2 x 16 KiB
  __shared__ uint4 s_x[2][TN * 8]; // 2 x 16 KiB

  // linear index -> XCD, then patch by patch inside the XCD, token tiles fastest inside a patch
  const uint32_t xcd = blockIdx.x & 7;
  const uint32_t idx = blockIdx.x >> 3;
  const uint32_t per_patch = ord.gm * ord.gn;
  const uint32_t patch = idx / per_patch, in_patch = idx % per_patch;
  const uint32_t patch_m = patch / ord.patches_n, patch_n = patch % ord.patches_n;
  const uint32_t row_tile = ( patch_m * ord.gm + in_patch / ord.gn ) * 8 + xcd;
  const uint32_t token_tile = patch_n * ord.gn + in_patch % ord.gn;
  if ( row_tile >= ord.row_tiles || token_tile >= ord.token_tiles ) {
    return; // padding of the last patches (whole work-group)
  }

  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wm = wave & 1, wn = wave >> 1; // wave position inside the tile
  const uint32_t row0 = row_tile * TM;
  const uint32_t col0 = token_tile * TN;
  const uint32_t lr = lane & 31, g2 = lane >> 5;
  const uint32_t k_begin = blockIdx.z * k_per_split;
  const uint32_t k_end = min( s, k_begin + k_per_split );

  f32x16 acc[2][2];
#pragma unroll
  for ( int i = 0; i < 2; i++ ) {
#pragma unroll
    for ( int j = 0; j < 2; j++ ) {
#pragma unroll
      for ( int e = 0; e < 16; e++ ) {
        acc[i][j][e] = 0.0f;
      }
    }
  }

  Frag fw, fx;
  load_frag( fw, w, s, row0, r, k_begin, k_end );
  load_frag( fx, x, s, col0, b, k_begin, k_end );
  int buf = 0;
  for ( uint32_t k0 = k_begin; k0 < k_end; k0 += TK ) {
    store_frag( s_w[buf], fw );
    store_frag( s_x[buf], fx );
    __syncthreads();
    if ( k0 + TK < k_end ) {
      load_frag( fw, w, s, row0, r, k0 + TK, k_end );
      load_frag( fx, x, s, col0, b, k0 + TK, k_end );
    }
    const uint4* lw = s_w[buf];
    const uint4* lx = s_x[buf];
#pragma unroll
    for ( int st = 0; st < 4; st++ ) {
      const uint32_t ch = 2 * st + g2;
      f16x8 a[2], bb[2];
#pragma unroll
      for ( int i = 0; i < 2; i++ ) {
        a[i] = __builtin_bit_cast( f16x8, lw[swz( wm * 64 + 32 * i + lr, ch )] );
        bb[i] = __builtin_bit_cast( f16x8, lx[swz( wn * 64 + 32 * i + lr, ch )] );
      }
#pragma unroll
      for ( int i = 0; i < 2; i++ ) {
#pragma unroll
        for ( int j = 0; j < 2; j++ ) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16( a[i], bb[j], acc[i][j], 0, 0, 0 );
        }
      }
    }
    buf ^= 1;
  }

  // acc[i][j][v]: weight row = row0 + wm*64 + 32*i + 8*(v/4) + 4*g2 + v%4, token = col0 + wn*64 + 32*j + lr
  // Output through LDS (the operand stages are free now): stored from the registers, an instruction
  // would touch 32 lines (tokens) with 16 or 32 bytes each.  The tile goes to LDS token-major, 16-byte
  // chunks XOR-swizzled with the token so that neither side has bank conflicts, and from there to
  // memory as whole row segments, 16 bytes per lane.
  if ( SPLIT && ( r & 3 ) == 0 ) { // fp32: 64 tokens x 128 rows per array, the token half of the wave picks it
    __syncthreads();
    uint4* mine = wn == 0 ? &s_w[0][0] : &s_x[0][0];
#pragma unroll
    for ( int j = 0; j < 2; j++ ) {
      const uint32_t token = 32 * j + lr;
#pragma unroll
      for ( int i = 0; i < 2; i++ ) {
#pragma unroll
        for ( int q4 = 0; q4 < 4; q4++ ) {
          const uint32_t chunk = 16 * wm + 8 * i + 2 * q4 + g2; // 4 rows each
          mine[token * 32 + ( chunk ^ ( token & 31 ) )] =
            __builtin_bit_cast( uint4, make_float4( acc[i][j][4 * q4], acc[i][j][4 * q4 + 1], acc[i][j][4 * q4 + 2], acc[i][j][4 * q4 + 3] ) );
        }
      }
    }
    __syncthreads();
#pragma unroll
    for ( int it = 0; it < 16; it++ ) {
      const uint4* region = it < 8 ? &s_w[0][0] : &s_x[0][0];
      const uint32_t idx = ( it % 8 ) * 256 + threadIdx.x;
      const uint32_t token = idx / 32, slot = idx % 32;
      const uint32_t col = col0 + 64 * ( it / 8 ) + token, row = row0 + 4 * ( slot ^ ( token & 31 ) );
      if ( col < b && row < r ) {
        *reinterpret_cast<uint4*>( partial + ( (uint64_t)blockIdx.z * b + col ) * r + row ) = region[idx];
      }
    }
    return;
  }
  if ( !SPLIT && ( r & 7 ) == 0 ) { // f16: 128 tokens x 128 rows in the weight stages
    __syncthreads();
    uint2* out = reinterpret_cast<uint2*>( &s_w[0][0] );
#pragma unroll
    for ( int j = 0; j < 2; j++ ) {
      const uint32_t token = 64 * wn + 32 * j + lr;
#pragma unroll
      for ( int i = 0; i < 2; i++ ) {
#pragma unroll
        for ( int q4 = 0; q4 < 4; q4++ ) {
          union
          {
            uint2 raw;
            __half h[4];
          } o;
#pragma unroll
          for ( int e = 0; e < 4; e++ ) {
            o.h[e] = __float2half_rn( acc[i][j][4 * q4 + e] );
          }
          const uint32_t chunk = 8 * wm + 4 * i + q4; // 8 rows each; g2 picks the half of the chunk
          out[( token * 16 + ( chunk ^ ( token & 15 ) ) ) * 2 + g2] = o.raw;
        }
      }
    }
    __syncthreads();
    const uint4* region = &s_w[0][0];
#pragma unroll
    for ( int it = 0; it < 8; it++ ) {
      const uint32_t idx = it * 256 + threadIdx.x;
      const uint32_t token = idx / 16, slot = idx % 16;
      const uint32_t col = col0 + token, row = row0 + 8 * ( slot ^ ( token & 15 ) );
      if ( col < b && row < r ) {
        *reinterpret_cast<uint4*>( xout + (uint64_t)col * r + row ) = region[idx];
      }
    }
    return;
  }
#pragma unroll
  for ( int j = 0; j < 2; j++ ) {
    const uint32_t col = col0 + wn * 64 + 32 * j + lr;
    if ( col >= b ) {
      continue;
    }
#pragma unroll
    for ( int i = 0; i < 2; i++ ) {
#pragma unroll
      for ( int q4 = 0; q4 < 4; q4++ ) {
        const uint32_t row = row0 + wm * 64 + 32 * i + 8 * q4 + 4 * g2;
        if ( SPLIT ) {
          float* dst = partial + ( (uint64_t)blockIdx.z * b + col ) * r + row;
          if ( row + 3 < r && ( r & 3 ) == 0 ) {
            *reinterpret_cast<float4*>( dst ) = make_float4( acc[i][j][4 * q4], acc[i][j][4 * q4 + 1], acc[i][j][4 * q4 + 2], acc[i][j][4 * q4 + 3] );
          } else {
            for ( int e = 0; e < 4; e++ ) {
              if ( row + e < r ) {
                dst[e] = acc[i][j][4 * q4 + e];
              }
            }
          }
          continue;
        }
        __half* dst = xout + (uint64_t)col * r + row;
        if ( row + 3 < r && ( r & 3 ) == 0 ) {
          union
          {
            uint2 raw;
            __half h[4];
          } o;
#pragma unroll
          for ( int e = 0; e < 4; e++ ) {
            o.h[e] = __float2half_rn( acc[i][j][4 * q4 + e] );
          }
          *reinterpret_cast<uint2*>( dst ) = o.raw;
        } else {
          for ( int e = 0; e < 4; e++ ) {
            if ( row + e < r ) {
              dst[e] = __float2half_rn( acc[i][j][4 * q4 + e] );
            }
          }
        }
      }
    }
  }
}

} // namespace

bool gemm_tile_applicable( uint64_t s, uint64_t r, uint64_t b, const void* x, const void* w, const void* xout )
{
  (void)r;
  return b > 64 && s % 8 == 0 && ( ( reinterpret_cast<uintptr_t>( x ) | reinterpret_cast<uintptr_t>( w ) | reinterpret_cast<uintptr_t>( xout ) ) & 15u ) == 0;
}

// K split so that about two work-groups per CU exist, each with at least 8 steps of K
void gemm_tile_plan( uint64_t s, uint64_t r, uint64_t b, uint32_t* splits_out, uint32_t* k_per_split_out )
{
  const uint64_t tiles = ( ( r + TM - 1 ) / TM ) * ( ( b + TN - 1 ) / TN );
  uint32_t splits = 1;
  if ( tiles < 384 ) {
    splits = (uint32_t)( ( 512 + tiles - 1 ) / tiles );
    splits = std::min<uint32_t>( splits, (uint32_t)std::max<uint64_t>( 1, s / ( 8 * TK ) ) );
    splits = std::min<uint32_t>( splits, 16 );
  }
  uint32_t k_per_split = (uint32_t)( ( s + splits - 1 ) / splits );
  k_per_split = ( k_per_split + TK - 1 ) / TK * TK;
  *splits_out = (uint32_t)( ( s + k_per_split - 1 ) / k_per_split );
  *k_per_split_out = k_per_split;
}

// `partial` != nullptr: fp32 partial sums (splits, b, r) instead of xout
int gemm_tile_launch( __half* xout, float* partial, const __half* x, const __half* w, uint64_t s, uint64_t r, uint64_t b, uint32_t splits, uint32_t k_per_split,
                      hipStream_t st )
{
  TileOrder ord;
  ord.row_tiles = (uint32_t)( ( r + TM - 1 ) / TM );
  ord.token_tiles = (uint32_t)( ( b + TN - 1 ) / TN );
  ord.gn = std::min<uint32_t>( ord.token_tiles, 8 );
  ord.gm = std::max<uint32_t>( 1, 64 / ord.gn );
  const uint32_t rows_per_xcd = ( ord.row_tiles + 7 ) / 8;
  ord.gm = std::min( ord.gm, rows_per_xcd );
  const uint32_t patches_m = ( rows_per_xcd + ord.gm - 1 ) / ord.gm;
  ord.patches_n = ( ord.token_tiles + ord.gn - 1 ) / ord.gn;
  const uint64_t gx = 8ull * patches_m * ord.patches_n * ord.gm * ord.gn;
  GH_REQUIRE( gx < ( 1ull << 31 ) && splits <= 65535, "gh_matmul: grid too large" );
  GH_REQUIRE( partial != nullptr || splits == 1, "gh_matmul: split K needs a partials buffer" );
  const dim3 grid( (unsigned)gx, 1, splits );
  if ( partial != nullptr ) {
    gemm_tile_kernel<true><<<grid, 256, 0, st>>>( xout, partial, x, w, (uint32_t)s, (uint32_t)r, (uint32_t)b, k_per_split, ord );
  } else {
    gemm_tile_kernel<false><<<grid, 256, 0, st>>>( xout, partial, x, w, (uint32_t)s, (uint32_t)r, (uint32_t)b, k_per_split, ord );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

} // namespace gh
