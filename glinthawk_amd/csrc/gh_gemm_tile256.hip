// Second MFMA-bound GEMM for many activation rows: a 256 x 256 output tile per work-group, i.e. per
// CU (one work-group of 4 waves is resident), for products with enough such tiles to fill the chip.
// What limits a tile GEMM on this part is the rate at which bytes enter a CU through the vector
// memory path; a 256 x 256 tile needs half the bytes per flop of a 128 x 128 one.
//
//   wave        = 64 weight rows x all 256 tokens: 2 x 8 accumulators of v_mfma_f32_32x32x16_f16
//                 (256 accumulator registers; the work-group runs at one wave per SIMD)
//   weights     never touch LDS: a buffer load puts row (lane % 32), k chunk (lane / 32) of a
//                 32 x 16 block into the lane that needs it as MFMA A operand.  Three register sets,
//                 loads two 64-k steps ahead.
//   activations global -> registers (one step ahead) -> LDS (two stages, XOR-swizzled 16-byte
//                 chunks, one barrier per step), read as B operands; every fragment feeds 2 MFMAs
//   schedule    the LDS reads are issued three fragments ahead of their use with hand-placed
//                 s_waitcnt (the compiler's scheduler otherwise sinks each read down to its MFMAs
//                 and the wave, alone on its SIMD, waits out every LDS latency).  The loop body has
//                 no joins -- loads past the end of K are issued anyway, bounded by the descriptors --
//                 so that the compiler's own vmcnt waits stay exact.
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
struct WStep { uint4 v[2][4]; }; // [row tile][k16 step]: lane l = row 32*rt + l%32, k 16*kk + 8*(l/32)
struct XStep { uint4 v[8]; };    // thread t: token t/8 + 32*i, chunk t%8

__device__ __forceinline__ void load_w( WStep& d, __amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t ld_bytes, uint32_t kb )
{
#pragma unroll
  for ( int rt = 0; rt < 2; rt++ ) {
#pragma unroll
    for ( int kk = 0; kk < 4; kk++ ) {
      d.v[rt][kk] = bload( rsrc, voff + 32 * kk, 32 * rt * ld_bytes + kb );
    }
  }
}
__device__ __forceinline__ void load_x( XStep& d, __amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t ld_bytes, uint32_t kb )
{
#pragma unroll
  for ( int i = 0; i < 8; i++ ) {
    d.v[i] = bload( rsrc, voff, 32 * i * ld_bytes + kb );
  }
}
__device__ __forceinline__ uint32_t swz( uint32_t row, uint32_t chunk ) { return row * 8 + ( chunk ^ ( ( row >> 1 ) & 7 ) ); }

struct TileOrder
{
  uint32_t row_tiles, token_tiles, gm, gn, patches_n;
};

// grid: 8 * padded tiles per XCD.  s % 64 == 0, 16-byte aligned operands.  PARTIAL: fp32 (1, b, r) instead of xout.
template<bool PARTIAL>
__global__ __launch_bounds__( 256, 1 ) void gemm_tile256_kernel( __half* __restrict__ xout,
                                                                float* __restrict__ partial,
                                                                const __half* __restrict__ x,
                                                                const __half* __restrict__ w,
                                                                uint32_t s,
                                                                uint32_t r,
                                                                uint32_t b,
                                                                TileOrder ord )
{
  __shared__ uint4 s_x[2][TN2 * 8]; // 2 x 32 KiB
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
  const uint32_t row0 = row_tile * TM2 + wave * 64;
  const uint32_t col0 = token_tile * TN2;
  const uint32_t ld_bytes = s * 2;
  const uint32_t w_rows = row0 < r ? min( 64u, r - row0 ) : 0u;
  const uint32_t x_cols = min( (uint32_t)TN2, b - col0 );
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( w + (uint64_t)row0 * s ), 0, (int)( w_rows * ld_bytes ), 0x00020000 );
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( x + (uint64_t)col0 * s ), 0, (int)( x_cols * ld_bytes ), 0x00020000 );
  const uint32_t w_voff = ( lane & 31 ) * ld_bytes + ( lane >> 5 ) * 16;
  const uint32_t x_voff = ( threadIdx.x >> 3 ) * ld_bytes + ( threadIdx.x & 7 ) * 16;

  f32x16 acc[2][8];
#pragma unroll
  for ( int rt = 0; rt < 2; rt++ ) {
#pragma unroll
    for ( int t = 0; t < 8; t++ ) {
#pragma unroll
      for ( int e = 0; e < 16; e++ ) {
        acc[rt][t][e] = 0.f;
      }
    }
  }
  const uint32_t n_steps = s / TKS;
  // LDS byte addresses of this lane's fragments of token tile 0 in stage 0, one per k16 step
  const uint32_t lds0 = (uint32_t)(uintptr_t)( __attribute__( ( address_space( 3 ) ) ) uint4* )&s_x[0][0];
  uint32_t frag_addr[4];
#pragma unroll
  for ( int kk = 0; kk < 4; kk++ ) {
    frag_addr[kk] = lds0 + swz( lane & 31, 2 * kk + ( lane >> 5 ) ) * 16;
  }
  WStep wr[3];
  XStep xr;
  // Loads past the end of K are issued unconditionally (the descriptors bound them, nothing reads the
  // result) and the prologue issues in the order of the steady state: the loop body then has no joins,
  // and the compiler's wait counts at the loop head are exact instead of a pessimistic merge.
  load_w( wr[0], w_rsrc, w_voff, ld_bytes, 0 );
  load_x( xr, x_rsrc, x_voff, ld_bytes, 0 );
  load_w( wr[1], w_rsrc, w_voff, ld_bytes, TKS * 2 );
  bool done = false;
  for ( uint32_t j0 = 0; !done; j0 += 6 ) {
#pragma unroll
    for ( int p = 0; p < 6; p++ ) {
      const uint32_t j = j0 + p;
      if ( j >= n_steps ) {
        done = true;
        break;
      }
      {
        uint4* xt = s_x[p & 1];
        // activations of this step: registers -> LDS
#pragma unroll
        for ( int i = 0; i < 8; i++ ) {
          xt[swz( ( threadIdx.x >> 3 ) + 32 * i, threadIdx.x & 7 )] = xr.v[i];
        }
        // next activations first, then the weights two steps ahead: loads retire in order
        load_x( xr, x_rsrc, x_voff, ld_bytes, ( j + 1 ) * TKS * 2 );
        load_w( wr[( p + 2 ) % 3], w_rsrc, w_voff, ld_bytes, ( j + 2 ) * TKS * 2 );
        __syncthreads();
        const WStep& ws = wr[p % 3];
        // 32 activation fragments per step (4 k16 steps x 8 token tiles), each feeding 2 MFMAs.  The LDS
        // read of fragment f+3 is in flight while the MFMAs of fragment f run: reads and waits are
        // written out by hand because the compiler's scheduler sinks every read down to its use.
        f16x8 bf[4];
        const uint32_t stage_off = ( p & 1 ) * ( TN2 * 8 * 16 );
#define GH_FRAG_READ( dst, f ) \
  asm volatile( "ds_read_b128 %0, %1" : "=v"( dst ) : "v"( frag_addr[( f ) >> 3] + stage_off + ( ( f ) & 7 ) * 4096u ) : "memory" )
        GH_FRAG_READ( bf[0], 0 );
        GH_FRAG_READ( bf[1], 1 );
        GH_FRAG_READ( bf[2], 2 );
#pragma unroll
        for ( int f = 0; f < 32; f++ ) {
          if ( f + 3 < 32 ) {
            GH_FRAG_READ( bf[( f + 3 ) % 4], f + 3 );
            asm volatile( "s_waitcnt lgkmcnt(3)" : "+v"( bf[f % 4] ) );
          } else if ( f + 2 < 32 ) {
            asm volatile( "s_waitcnt lgkmcnt(2)" : "+v"( bf[f % 4] ) );
          } else if ( f + 1 < 32 ) {
            asm volatile( "s_waitcnt lgkmcnt(1)" : "+v"( bf[f % 4] ) );
          } else {
            asm volatile( "s_waitcnt lgkmcnt(0)" : "+v"( bf[f % 4] ) );
          }
          const int kk = f >> 3, t = f & 7;
#pragma unroll
          for ( int rt = 0; rt < 2; rt++ ) {
            acc[rt][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16( __builtin_bit_cast( f16x8, ws.v[rt][kk] ), bf[f % 4], acc[rt][t], 0, 0, 0 );
          }
        }
#undef GH_FRAG_READ
      }
    }
  }
  // acc[rt][t][v]: row = row0 + 32*rt + 8*(v/4) + 4*(lane/32) + v%4, token = col0 + 32*t + lane%32
#pragma unroll
  for ( int t = 0; t < 8; t++ ) {
    const uint32_t col = col0 + 32 * t + ( lane & 31 );
    if ( col >= b ) {
      continue;
    }
#pragma unroll
    for ( int rt = 0; rt < 2; rt++ ) {
#pragma unroll
      for ( int q4 = 0; q4 < 4; q4++ ) {
        const uint32_t row = row0 + 32 * rt + 8 * q4 + 4 * ( lane >> 5 );
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

// Worth it only when the 256 x 256 tiles alone fill the chip (no K split here), and, with a short K,
// only when there are several rounds of them: the tile's prologue and its strided epilogue weigh more
// then, and a partly filled last round costs a quarter of the chip (measured: 13B w1 at 3328 rows,
// K 5120, 702 tiles: 756 us against 696 us with 128 x 128 tiles; 70B shapes, K 8192+: 10-20 % faster).
bool gemm_tile256_applicable( uint64_t s, uint64_t r, uint64_t b, const void* x, const void* w, const void* xout )
{
  const uint64_t tiles = ( ( r + TM2 - 1 ) / TM2 ) * ( ( b + TN2 - 1 ) / TN2 );
  const bool enough = tiles >= 192 && ( s >= 8192 || tiles >= 1024 );
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
    gemm_tile256_kernel<true><<<(unsigned)gx, 256, 0, st>>>( xout, partial, x, w, (uint32_t)s, (uint32_t)r, (uint32_t)b, ord );
  } else {
    gemm_tile256_kernel<false><<<(unsigned)gx, 256, 0, st>>>( xout, partial, x, w, (uint32_t)s, (uint32_t)r, (uint32_t)b, ord );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

} // namespace gh
