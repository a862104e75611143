// Second MFMA-bound GEMM for many activation rows: a 256 x 256 output tile per work-group, i.e. per
// CU, for products with enough such tiles to fill the chip.  A 256 x 256 tile needs half the operand
// bytes per flop of a 128 x 128 one, and what limits a tile GEMM on this part is the CU's vector
// memory path, not HBM or the matrix pipes.
//
//   work-group  = 8 waves = 4 row groups x 2 token groups; a wave owns 64 weight rows x 128 tokens:
//                 2 x 4 accumulators of v_mfma_f32_32x32x16_f16 (128 registers), two waves per SIMD.
//                 With one wave per SIMD (four waves of 64 x 256, the first version of this kernel)
//                 every stall of a memory or LDS instruction also holds back that wave's MFMAs:
//                 0.82-0.97 PFLOP/s however the operands were fetched; two waves per SIMD: 0.9-1.08.
//   operands    both go global -> registers (one 64-k step ahead, coalesced 128-byte row segments,
//                 four 16-byte loads per thread and operand) -> LDS (two stages, XOR-swizzled
//                 16-byte chunks, no bank conflicts) -> MFMA operands
//   schedule    step j multiplies out of stage j % 2; in the middle of its MFMAs the registers that
//                 hold step j + 1 are written to the other stage and the loads of step j + 2 go
//                 out, so the matrix pipe works through the copy; one barrier per step; the wave's
//                 priority is raised while it issues MFMAs, so that of two waves on a SIMD the one
//                 with matrix work goes first
//   tile order  as in the 128 x 128 kernel: each XCD owns every 8th row tile and walks patches of
//                 tiles that are resident together
#include "gh_common.h"

#include <algorithm>

namespace gh {

typedef _Float16 f16x8 __attribute__( ( ext_vector_type( 8 ) ) );
typedef float f32x16 __attribute__( ( ext_vector_type( 16 ) ) );

namespace {

constexpr int TM2 = 256; // weight rows per work-group: 4 waves x 64
constexpr int TN2 = 256; // tokens per work-group
constexpr int TKS = 64;  // k per step

__device__ __forceinline__ uint4 bload( __amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff )
{
  return __builtin_bit_cast( uint4, __builtin_amdgcn_raw_buffer_load_b128( rsrc, voff, soff, 0 ) );
}
__device__ __forceinline__ uint32_t swz( uint32_t row, uint32_t chunk ) { return row * 8 + ( chunk ^ ( ( row >> 1 ) & 7 ) ); }

struct TileOrder
{
  uint32_t row_tiles, token_tiles, gm, gn, patches_n;
};

constexpr int T256_THREADS = 512;

struct Step8
{
  uint4 v[4]; // thread t: row t/8 + 64*i, chunk t%8
};

__device__ __forceinline__ void load8( Step8& d, __amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t ld_bytes, uint32_t kb )
{
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    d.v[i] = bload( rsrc, voff, 64 * i * ld_bytes + kb );
  }
}

// grid: 8 * padded tiles per XCD.  s % 64 == 0, 16-byte aligned operands.  PARTIAL: fp32 (1, b, r) instead of xout.
template<bool PARTIAL>
__global__ __launch_bounds__( T256_THREADS, 1 ) void gemm_tile256_kernel( __half* __restrict__ xout,
                                                                        float* __restrict__ partial,
                                                                        const __half* __restrict__ x,
                                                                        const __half* __restrict__ w,
                                                                        uint32_t s,
                                                                        uint32_t r,
                                                                        uint32_t b,
                                                                        TileOrder ord )
{
  __shared__ uint4 s_x[2][TN2 * 8]; // 2 x 32 KiB
  __shared__ uint4 s_w[2][TM2 * 8]; // 2 x 32 KiB
  const uint32_t xcd = blockIdx.x & 7;
  const uint32_t idx = blockIdx.x >> 3;
  const uint32_t per_patch = ord.gm * ord.gn;
  const uint32_t patch = idx / per_patch, in_patch = idx % per_patch;
  const uint32_t patch_m = patch / ord.patches_n, patch_n = patch % ord.patches_n;
  const uint32_t row_tile = ( patch_m * ord.gm + in_patch / ord.gn ) * 8 + xcd;
  const uint32_t token_tile = patch_n * ord.gn + in_patch % ord.gn;
  if ( row_tile >= ord.row_tiles || token_tile >= ord.token_tiles ) {
    return;
  }
  const uint32_t wave = __builtin_amdgcn_readfirstlane( threadIdx.x >> 6 );
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wr = wave >> 1, wc = wave & 1;
  const uint32_t tile_row0 = row_tile * TM2;
  const uint32_t tile_col0 = token_tile * TN2;
  const uint32_t ld_bytes = s * 2;
  const uint32_t w_rows = min( (uint32_t)TM2, r - tile_row0 );
  const uint32_t x_cols = min( (uint32_t)TN2, b - tile_col0 );
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( w + (uint64_t)tile_row0 * s ), 0, (int)( w_rows * ld_bytes ), 0x00020000 );
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( x + (uint64_t)tile_col0 * s ), 0, (int)( x_cols * ld_bytes ), 0x00020000 );
  const uint32_t voff = ( threadIdx.x >> 3 ) * ld_bytes + ( threadIdx.x & 7 ) * 16;

  f32x16 acc[2][4];
#pragma unroll
  for ( int rt = 0; rt < 2; rt++ ) {
#pragma unroll
    for ( int t = 0; t < 4; t++ ) {
#pragma unroll
      for ( int e = 0; e < 16; e++ ) {
        acc[rt][t][e] = 0.f;
      }
    }
  }
  const uint32_t n_steps = s / TKS;
  Step8 wreg, xreg;
  const uint32_t fr = lane & 31, g2 = lane >> 5;
  auto stage = [&]( uint32_t p ) { // registers -> LDS stage p
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      const uint32_t row = ( threadIdx.x >> 3 ) + 64 * i;
      s_w[p][swz( row, threadIdx.x & 7 )] = wreg.v[i];
      s_x[p][swz( row, threadIdx.x & 7 )] = xreg.v[i];
    }
  };
  auto mfma_k16 = [&]( const uint4* wt, const uint4* xt, int kk ) {
    const uint32_t ch = 2 * kk + g2;
    const f16x8 a0 = __builtin_bit_cast( f16x8, wt[swz( 64 * wr + fr, ch )] );
    const f16x8 a1 = __builtin_bit_cast( f16x8, wt[swz( 64 * wr + 32 + fr, ch )] );
#pragma unroll
    for ( int t = 0; t < 4; t++ ) {
      const f16x8 bb = __builtin_bit_cast( f16x8, xt[swz( 128 * wc + 32 * t + fr, ch )] );
      acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16( a0, bb, acc[0][t], 0, 0, 0 );
      acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16( a1, bb, acc[1][t], 0, 0, 0 );
    }
  };
  load8( wreg, w_rsrc, voff, ld_bytes, 0 );
  load8( xreg, x_rsrc, voff, ld_bytes, 0 );
  stage( 0 );
  load8( wreg, w_rsrc, voff, ld_bytes, TKS * 2 );
  load8( xreg, x_rsrc, voff, ld_bytes, TKS * 2 );
  __syncthreads();
  // Step j computes out of stage j % 2 while the registers that hold step j + 1 are written to the
  // other stage in the middle of its MFMAs (that stage was last read in step j - 1, behind a
  // barrier) and the loads of step j + 2 go out: the matrix pipe keeps working through the copy.
  // The loads behind the last step read the start of the next rows (bounded by the descriptors);
  // what they bring is staged but never multiplied.
  for ( uint32_t j = 0; j < n_steps; j++ ) {
    const uint4* wt = s_w[j & 1];
    const uint4* xt = s_x[j & 1];
    __builtin_amdgcn_s_setprio( 1 );
    mfma_k16( wt, xt, 0 );
    mfma_k16( wt, xt, 1 );
    __builtin_amdgcn_s_setprio( 0 );
    stage( ( j & 1 ) ^ 1 );
    load8( wreg, w_rsrc, voff, ld_bytes, ( j + 2 ) * TKS * 2 );
    load8( xreg, x_rsrc, voff, ld_bytes, ( j + 2 ) * TKS * 2 );
    __builtin_amdgcn_s_setprio( 1 );
    mfma_k16( wt, xt, 2 );
    mfma_k16( wt, xt, 3 );
    __builtin_amdgcn_s_setprio( 0 );
    __syncthreads();
  }
  // acc[rt][t][v]: row = tile_row0 + 64*wr + 32*rt + 8*(v/4) + 4*(lane/32) + v%4, token = tile_col0 + 128*wc + 32*t + lane%32
#pragma unroll
  for ( int t = 0; t < 4; t++ ) {
    const uint32_t col = tile_col0 + 128 * wc + 32 * t + fr;
    if ( col >= b ) {
      continue;
    }
#pragma unroll
    for ( int rt = 0; rt < 2; rt++ ) {
#pragma unroll
      for ( int q4 = 0; q4 < 4; q4++ ) {
        const uint32_t row = tile_row0 + 64 * wr + 32 * rt + 8 * q4 + 4 * g2;
        const bool whole = row + 3 < r && ( r & 3 ) == 0;
        if ( PARTIAL ) {
          float* dst = partial + (uint64_t)col * r + row;
          if ( whole ) {
            *reinterpret_cast<float4*>( dst ) = make_float4( acc[rt][t][4 * q4], acc[rt][t][4 * q4 + 1], acc[rt][t][4 * q4 + 2], acc[rt][t][4 * q4 + 3] );
          } else {
            for ( int e = 0; e < 4; e++ ) {
              if ( row + e < r ) {
                dst[e] = acc[rt][t][4 * q4 + e];
              }
            }
          }
        } else {
          __half* dst = xout + (uint64_t)col * r + row;
          if ( whole ) {
            union
            {
              uint2 raw;
              __half h[4];
            } o;
#pragma unroll
            for ( int e = 0; e < 4; e++ ) {
              o.h[e] = __float2half_rn( acc[rt][t][4 * q4 + e] );
            }
            *reinterpret_cast<uint2*>( dst ) = o.raw;
          } else {
            for ( int e = 0; e < 4; e++ ) {
              if ( row + e < r ) {
                dst[e] = __float2half_rn( acc[rt][t][4 * q4 + e] );
              }
            }
          }
        }
      }
    }
  }
}

} // namespace

// Worth it when the 256 x 256 tiles alone fill the chip (no K split here) and the last round of them
// is not mostly empty (measured against the 128 x 128 kernel: 15-40 % faster from 192 tiles up, except
// at 258-260 tiles, where the second round runs 4 tiles on 256 CUs).
bool gemm_tile256_applicable( uint64_t s, uint64_t r, uint64_t b, const void* x, const void* w, const void* xout )
{
  const uint64_t tiles = ( ( r + TM2 - 1 ) / TM2 ) * ( ( b + TN2 - 1 ) / TN2 );
  // one work-group per CU: a last round that leaves more than 40 % of the chip idle goes to the 128 x 128 kernel instead
  const uint64_t cus = (uint64_t)cu_count();
  const uint64_t rounds = ( tiles + cus - 1 ) / cus;
  const bool enough = 4 * tiles >= 3 * cus && 10 * tiles >= 6 * rounds * cus;
  return b >= 192 && enough && s % TKS == 0 && s >= 2 * TKS && s < ( 1u << 22 )
         && ( ( reinterpret_cast<uintptr_t>( x ) | reinterpret_cast<uintptr_t>( w ) | reinterpret_cast<uintptr_t>( xout ) ) & 15u ) == 0;
}

// `partial` != nullptr: fp32 sums (1, b, r) instead of xout
int gemm_tile256_launch( __half* xout, float* partial, const __half* x, const __half* w, uint64_t s, uint64_t r, uint64_t b, hipStream_t st )
{
  TileOrder ord;
  ord.row_tiles = (uint32_t)( ( r + TM2 - 1 ) / TM2 );
  ord.token_tiles = (uint32_t)( ( b + TN2 - 1 ) / TN2 );
  ord.gn = std::min<uint32_t>( ord.token_tiles, 8 );
  ord.gm = std::max<uint32_t>( 1, 32 / ord.gn ); // 32 CUs per XCD, one work-group each
  const uint32_t rows_per_xcd = ( ord.row_tiles + 7 ) / 8;
  ord.gm = std::min( ord.gm, rows_per_xcd );
  const uint32_t patches_m = ( rows_per_xcd + ord.gm - 1 ) / ord.gm;
  ord.patches_n = ( ord.token_tiles + ord.gn - 1 ) / ord.gn;
  const uint64_t gx = 8ull * patches_m * ord.patches_n * ord.gm * ord.gn;
  GH_REQUIRE( gx < ( 1ull << 31 ), "gh_matmul: grid too large" );
  if ( partial != nullptr ) {
    gemm_tile256_kernel<true><<<(unsigned)gx, T256_THREADS, 0, st>>>( xout, partial, x, w, (uint32_t)s, (uint32_t)r, (uint32_t)b, ord );
  } else {
    gemm_tile256_kernel<false><<<(unsigned)gx, T256_THREADS, 0, st>>>( xout, partial, x, w, (uint32_t)s, (uint32_t)r, (uint32_t)b, ord );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

} // namespace gh
