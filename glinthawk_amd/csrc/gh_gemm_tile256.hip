// Second MFMA-bound GEMM for many activation rows: a 256 x 256 or 384 x 256 (weight rows x tokens)
// output tile per work-group, i.e. per CU, for products with enough such tiles to fill the chip.  A
// 256 x 256 tile needs half the operand bytes per flop of a 128 x 128 one, and what limits a tile GEMM
// on this part is the path from L2 into the CU, not HBM or the matrix pipes.
//
//   work-group  = 8 waves = 4 row groups x 2 token groups; a wave owns 64 or 96 weight rows x 128
//                 tokens: 2 or 3 x 4 accumulators of v_mfma_f32_32x32x16_f16 (128 or 192 registers),
//                 two waves per SIMD.
//                 With one wave per SIMD (four waves of 64 x 256, the first version of this kernel)
//                 every stall of a memory or LDS instruction also holds back that wave's MFMAs:
//                 0.82-0.97 PFLOP/s however the operands were fetched.  Four waves of 128 x 128 (256
//                 accumulator registers, a third less LDS traffic per flop than 64 x 128, the step's
//                 barrier in front of the last 16-k group with the next stage's first fragments
//                 requested behind it): 0.68-0.79.
//   384 rows    bring 80 KiB per 64 k for 1.5 x the flops of 256 rows (64 KiB) and fill the LDS
//                 (2 x 80 KiB) and the registers (one set of MFMA operands instead of two); a round
//                 of them takes 1.24-1.44 x as long, so they win where their rounds fit the shape
//                 at least as well (tile256_rows() below)
//   output      through LDS, token-major, and from there as whole row segments (16 bytes per lane,
//                 512 or 768 contiguous bytes per token): stored from the accumulator registers, an
//                 instruction touches 32 lines with 16 bytes each, which cost 10-16 % of the kernel
//                 at K 5120-8192
//   operands    both go global -> LDS without passing through registers (`buffer_load ... lds`, 16
//                 bytes per lane: a wave's instruction writes 1 KiB of LDS, lane l at + 16 l, so the
//                 XOR swizzle that keeps the MFMA reads free of bank conflicts is applied to the
//                 global address each lane fetches) -> MFMA operands; two 64-k stages
//   schedule    step j multiplies out of stage j % 2 while the loads of step j + 1 fill the other
//                 stage; the barrier that ends the step waits for them.  The fragments of the next
//                 16 k are read from LDS before the MFMAs of the current 16 k are issued; the
//                 wave's priority is raised while it issues MFMAs, so that of two waves on a SIMD
//                 the one with matrix work goes first.  Against staging through registers (loads
//                 one step ahead, ds_write in the middle of the MFMAs): 1.02 -> 1.15 PFLOP/s at
//                 16384 x 8192 x 57344.
//   what binds  measured at 16384 tokens, 70B shapes, 256 rows (1.15-1.19 PFLOP/s as is; variants
//                 that keep every LDS read: the compiler folds reads of a stage nothing writes):
//                 loads taken out of the loop, both stages filled once, barrier kept: 1.33-1.45;
//                 loads issued into one stage pair but never waited for, reads from the other:
//                 1.16-1.22.  So waiting for the loads costs nothing to speak of, their traffic
//                 through the CU about 15 %, and the rest is the loop of LDS reads, MFMAs and one
//                 barrier per 64 k itself (MFMA pipes busy 55 %; a wave sits in s_waitcnt 15 % of
//                 its time, LDS reads take 4 cycles per instruction without conflicts).  Tried and
//                 not kept: a third stage for the activations (their loads two steps ahead, -6..+7 %),
//                 that plus the weights two steps ahead through registers (-5..+3 %), five 32-k
//                 stages as a ring (two barriers per 64 k: -5..-15 %), non-temporal loads (-10 %), the
//                 barrier in front of the last MFMA group of a step with the next stage's first
//                 fragments requested right behind it, so that the waves leave the barrier with matrix
//                 work in hand (256 rows -5..-8 %, 384 rows +-1 %).
//   clock       the graphics clock counter (GRBM_GUI_ACTIVE over the kernel's duration) reads 1.69-1.80 GHz
//                 while this kernel runs and 2.3-2.4 GHz in the bandwidth-bound decode kernels: under
//                 sustained matrix load the part lowers its clock, so at 70-78 % matrix-pipe use the
//                 kernel delivers 1.2-1.3 PFLOP/s, and 100 % at that clock would be 1.77, not 2.5.
//   tile order  as in the 128 x 128 kernel: each XCD owns every 8th row tile and walks patches of
//                 tiles that are resident together.  The row tiles beyond a multiple of 8 are cut
//                 into 8 equal runs of tiles instead, so that every XCD gets the same number of
//                 tiles whatever the row count (with whole row tiles per XCD, 5120 rows x 16384
//                 tokens took 6 rounds instead of 5: 0.99 -> 1.15 PFLOP/s).
#include "gh_common.h"

#include <algorithm>
#include <cstdlib>

namespace gh {

typedef _Float16 f16x8 __attribute__( ( ext_vector_type( 8 ) ) );
typedef float f32x16 __attribute__( ( ext_vector_type( 16 ) ) );
typedef __attribute__( ( address_space( 3 ) ) ) void* lds_ptr;

namespace {

constexpr int TM2 = 256; // weight rows per work-group: 4 waves x 64
constexpr int TN2 = 256; // tokens per work-group
constexpr int TKS = 64;  // k per step

__device__ __forceinline__ uint32_t swz( uint32_t row, uint32_t chunk ) { return row * 8 + ( chunk ^ ( ( row >> 1 ) & 7 ) ); }

// Row tiles [0, 8 * rows_per_xcd): XCD x owns row tiles x, x + 8, ... and walks (row tile, token tile)
// in patches of gm x gn, token direction fastest.  The row tiles left over (fewer than 8) are cut
// into 8 equal runs of tiles, one per XCD, in patches of (all of those rows) x 8 token tiles.
struct TileOrder
{
  uint32_t row_tiles, token_tiles, gm, gn, patches_n;
  uint32_t rows_per_xcd, main_per_xcd; // main part: row tiles and work-groups (patch padding included) of one XCD
  uint32_t rest_rows, rest_share;      // left-over row tiles; tiles of them per XCD
};

// Which tile work-group blockIdx.x takes; false: none (padding of the last patches).
__device__ __forceinline__ bool tile_of_workgroup( const TileOrder& ord, uint32_t& row_tile, uint32_t& token_tile )
{
  const uint32_t xcd = blockIdx.x & 7; // work-groups go to the XCDs in turn
  const uint32_t idx = blockIdx.x >> 3;
  if ( idx < ord.main_per_xcd ) {
    const uint32_t per_patch = ord.gm * ord.gn;
    const uint32_t patch = idx / per_patch, in_patch = idx % per_patch;
    const uint32_t patch_m = patch / ord.patches_n, patch_n = patch % ord.patches_n;
    const uint32_t own_row = patch_m * ord.gm + in_patch / ord.gn;
    row_tile = own_row * 8 + xcd;
    token_tile = patch_n * ord.gn + in_patch % ord.gn;
    return own_row < ord.rows_per_xcd && token_tile < ord.token_tiles;
  }
  const uint32_t mine = idx - ord.main_per_xcd;
  const uint32_t u = xcd * ord.rest_share + mine;
  if ( mine >= ord.rest_share || u >= ord.rest_rows * ord.token_tiles ) {
    return false;
  }
  const uint32_t per_patch_col = ord.rest_rows * 8; // the last one may be narrower
  const uint32_t patch_col = u / per_patch_col, in_col = u % per_patch_col;
  const uint32_t width = min( 8u, ord.token_tiles - patch_col * 8 );
  row_tile = ord.rows_per_xcd * 8 + in_col / width;
  token_tile = patch_col * 8 + in_col % width;
  return true;
}

constexpr int T256_THREADS = 512;

// What a work-group does with its sums: xout = DType(sum); the reference's next op on top of that,
// xout = DType(float(xout) + float(DType(sum))) (accum; only with r % 8 == 0); or the fp32 sums, (1, b, r).
// (The SiLU gate was tried here as well: with one work-group per CU nothing hides the epilogue's
// divisions and exponentials, and the separate element-wise kernel is faster.)
constexpr int EPI_STORE = 0, EPI_ACCUM = 1, EPI_PARTIAL = 3;

// grid: 8 x (padded tiles of one XCD) by K splits (more than one only with EPI_PARTIAL: split z leaves its sums in
// partial[z]).  s % 64 == 0, k_len % 64 == 0, 16-byte aligned operands.
// NA: 32-row accumulator tiles per wave, 2 (256 weight rows per work-group) or 3 (384).
template<int EPI, int NA>
__global__ __launch_bounds__( T256_THREADS, 1 ) void gemm_tile256_kernel( __half* __restrict__ xout,
                                                                        float* __restrict__ partial,
                                                                        const __half* __restrict__ x,
                                                                        const __half* __restrict__ w,
                                                                        uint32_t s,
                                                                        uint32_t r,
                                                                        uint32_t b,
                                                                        uint32_t k_len, // k per split
                                                                        __half* __restrict__ xout2, // rows from r_first on go here, as rows 0.. of a (b, r - r_first) matrix
                                                                        uint32_t r_first, // rows [0, r_first) go to xout, a (b, r_first) matrix; == r: one output
                                                                        TileOrder ord )
{
  // Four separate arrays, not [2][...]: the compiler orders an LDS read behind an outstanding
  // load-to-LDS only when it cannot tell their arrays apart.
  constexpr int TM = 128 * NA; // weight rows per work-group: 4 waves x NA x 32
  __shared__ uint4 s_x0[TN2 * 8], s_x1[TN2 * 8]; // 2 x 32 KiB
  __shared__ uint4 s_w0[TM * 8], s_w1[TM * 8];   // 2 x 32 KiB, or 2 x 48 KiB: all 160 KiB of the CU
  uint32_t row_tile, token_tile;
  if ( !tile_of_workgroup( ord, row_tile, token_tile ) ) {
    return; // padding of the last patches (whole work-group)
  }
  const uint32_t wave = __builtin_amdgcn_readfirstlane( threadIdx.x >> 6 );
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wr = wave >> 1, wc = wave & 1;
  const uint32_t tile_row0 = row_tile * TM;
  const uint32_t tile_col0 = token_tile * TN2;
  const uint32_t ld_bytes = s * 2;
  const uint32_t w_rows = min( (uint32_t)TM, r - tile_row0 );
  const uint32_t x_cols = min( (uint32_t)TN2, b - tile_col0 );
  const uint32_t k0 = blockIdx.y * k_len; // this split's k range starts here; the descriptors start there too and end with the tile's last row
  const __amdgpu_buffer_rsrc_t w_rsrc
    = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( w + (uint64_t)tile_row0 * s + k0 ), 0, (int)( w_rows * ld_bytes - k0 * 2 ), 0x00020000 );
  const __amdgpu_buffer_rsrc_t x_rsrc
    = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( x + (uint64_t)tile_col0 * s + k0 ), 0, (int)( x_cols * ld_bytes - k0 * 2 ), 0x00020000 );
  // A load-to-LDS writes lane l of a wave to (wave's base) + 16 l: thread t fills slot t % 8 of row
  // t / 8 (+ 64 i), so it fetches the chunk that the swizzle keeps in that slot.
  const uint32_t voff = ( threadIdx.x >> 3 ) * ld_bytes + ( ( threadIdx.x & 7 ) ^ ( ( threadIdx.x >> 4 ) & 7 ) ) * 16;
  const uint32_t wave_slot0 = 8 * wave * 8; // first uint4 of the wave's 8 rows

  f32x16 acc[NA][4];
#pragma unroll
  for ( int rt = 0; rt < NA; rt++ ) {
#pragma unroll
    for ( int t = 0; t < 4; t++ ) {
#pragma unroll
      for ( int e = 0; e < 16; e++ ) {
        acc[rt][t][e] = 0.f;
      }
    }
  }
  const uint32_t n_steps = min( k_len, s - k0 ) / TKS;
  const uint32_t fr = lane & 31, g2 = lane >> 5;
  // global -> LDS stage, 1 KiB per wave and instruction: loads [from, to) of the list W0 X0 W1 X1 W2 X2 W3 X3 (W4 W5)
  constexpr int N_LOADS = 2 * NA + 4;
  auto fetch = [&]( uint4* wt, uint4* xt, uint32_t kb, int from, int to ) {
#pragma unroll
    for ( int l = 0; l < N_LOADS; l++ ) {
      if ( l < from || l >= to ) {
        continue;
      }
      const bool is_w = l >= 8 || ( l & 1 ) == 0;
      const int i = l >= 8 ? l - 4 : l >> 1;
      if ( is_w ) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds( w_rsrc, (lds_ptr)( wt + wave_slot0 + 64 * i * 8 ), 16, voff, 64 * i * ld_bytes + kb, 0, 0 );
      } else {
        __builtin_amdgcn_raw_ptr_buffer_load_lds( x_rsrc, (lds_ptr)( xt + wave_slot0 + 64 * i * 8 ), 16, voff, 64 * i * ld_bytes + kb, 0, 0 );
      }
    }
  };
  // The loads of a step go out in front of the MFMAs of its first two (three, for 384 rows) groups of
  // 16 k: all of them at the head of the step measured 0-4 % slower, spread over all four groups
  // slower again for 256 rows (the last ones then have a quarter of a step to arrive).
  auto fetch_at = [&]( uint4* wn, uint4* xn, uint32_t kb, int kk ) {
    constexpr int parts = NA == 2 ? 2 : 3;
    if ( kk < parts ) {
      fetch( wn, xn, kb, ( N_LOADS * kk + parts - 1 ) / parts, ( N_LOADS * ( kk + 1 ) + parts - 1 ) / parts );
    }
  };
  struct Frags
  {
    f16x8 a[NA], bb[4];
  };
  auto read_k16 = [&]( Frags& f, const uint4* wt, const uint4* xt, int kk ) {
    const uint32_t ch = 2 * kk + g2;
#pragma unroll
    for ( int rt = 0; rt < NA; rt++ ) {
      f.a[rt] = __builtin_bit_cast( f16x8, wt[swz( 32 * NA * wr + 32 * rt + fr, ch )] );
    }
#pragma unroll
    for ( int t = 0; t < 4; t++ ) {
      f.bb[t] = __builtin_bit_cast( f16x8, xt[swz( 128 * wc + 32 * t + fr, ch )] );
    }
  };
  auto mfma_k16 = [&]( const Frags& f ) {
#pragma unroll
    for ( int t = 0; t < 4; t++ ) {
#pragma unroll
      for ( int rt = 0; rt < NA; rt++ ) {
        acc[rt][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16( f.a[rt], f.bb[t], acc[rt][t], 0, 0, 0 );
      }
    }
  };
  // Step j multiplies out of stage j % 2 while the memory unit writes step j + 1 straight into the
  // other stage (last read in step j - 1, behind a barrier); the barrier that ends the step also
  // waits for those loads.  The loads behind the last step read the start of the next rows (bounded
  // by the descriptors); what they bring is never multiplied.
  auto step = [&]( const uint4* wt, const uint4* xt, uint4* wn, uint4* xn, uint32_t j ) {
    const uint32_t kb = ( j + 1 ) * TKS * 2;
    if constexpr ( NA == 2 ) { // two fragment sets: the reads of the next 16 k go out before the MFMAs of these
      Frags f0, f1;
      read_k16( f0, wt, xt, 0 );
      fetch_at( wn, xn, kb, 0 );
      read_k16( f1, wt, xt, 1 );
      __builtin_amdgcn_s_setprio( 1 );
      mfma_k16( f0 );
      __builtin_amdgcn_s_setprio( 0 );
      fetch_at( wn, xn, kb, 1 );
      read_k16( f0, wt, xt, 2 );
      __builtin_amdgcn_s_setprio( 1 );
      mfma_k16( f1 );
      __builtin_amdgcn_s_setprio( 0 );
      fetch_at( wn, xn, kb, 2 );
      read_k16( f1, wt, xt, 3 );
      __builtin_amdgcn_s_setprio( 1 );
      mfma_k16( f0 );
      __builtin_amdgcn_s_setprio( 0 );
      fetch_at( wn, xn, kb, 3 );
      __builtin_amdgcn_s_setprio( 1 );
      mfma_k16( f1 );
      __builtin_amdgcn_s_setprio( 0 );
    } else { // 192 accumulator registers leave room for one set
      Frags f;
      read_k16( f, wt, xt, 0 );
#pragma unroll
      for ( int kk = 0; kk < 4; kk++ ) {
        fetch_at( wn, xn, kb, kk );
        __builtin_amdgcn_s_setprio( 1 );
        mfma_k16( f );
        __builtin_amdgcn_s_setprio( 0 );
        if ( kk < 3 ) {
          read_k16( f, wt, xt, kk + 1 );
        }
      }
    }
    __builtin_amdgcn_s_waitcnt( 0x0F70 ); // vmcnt(0): this wave's loads-to-LDS have landed (the barrier's own fence only orders LDS instructions)
    __syncthreads();
  };
  fetch( s_w0, s_x0, 0, 0, N_LOADS );
  __builtin_amdgcn_s_waitcnt( 0x0F70 );
  __syncthreads();
  for ( uint32_t j = 0;; ) {
    step( s_w0, s_x0, s_w1, s_x1, j );
    if ( ++j == n_steps ) {
      break;
    }
    step( s_w1, s_x1, s_w0, s_x0, j );
    if ( ++j == n_steps ) {
      break;
    }
  }
  // acc[rt][t][v]: row = tile_row0 + 32*NA*wr + 32*rt + 8*(v/4) + 4*(lane/32) + v%4, token = tile_col0 + 128*wc + 32*t + lane%32
  constexpr bool PARTIAL = EPI == EPI_PARTIAL;
  if ( !PARTIAL && ( r & 7 ) == 0 ) {
    // Output through LDS: a lane holds 4 rows (8 bytes) of 32 different tokens, and stored from the
    // registers every instruction would touch 32 lines, 16 bytes each (that epilogue cost 10-16 % of
    // the kernel at K 5120-8192).  The tile goes to LDS token-major instead, 64 tokens per stage array
    // (16-byte chunks of 8 rows, chunk index XORed with the token so that neither side has bank
    // conflicts), and from there to memory as whole row segments, 16 bytes per lane.
    constexpr uint32_t CHUNKS = TM / 8;                    // 16-byte chunks per token: 32 or 48
    constexpr uint32_t SWZ_MASK = NA == 2 ? 31 : 15;      // the XOR stays inside a power-of-two group of chunks
    auto put = [&]( uint4* region, int t ) { // this wave's 32 tokens of block t -> tokens 32 (t % 2) + fr of the region
      uint2* out = reinterpret_cast<uint2*>( region );
      const uint32_t token = 32 * ( t & 1 ) + fr;
#pragma unroll
      for ( int rt = 0; rt < NA; rt++ ) {
#pragma unroll
        for ( int q4 = 0; q4 < 4; q4++ ) {
          union
          {
            uint2 raw;
            __half h[4];
          } o;
#pragma unroll
          for ( int e = 0; e < 4; e++ ) {
            o.h[e] = __float2half_rn( acc[rt][t][4 * q4 + e] );
          }
          const uint32_t chunk = 4 * NA * wr + 4 * rt + q4;
          out[( token * CHUNKS + ( chunk ^ ( token & SWZ_MASK ) ) ) * 2 + g2] = o.raw;
        }
      }
    };
    auto copy_out = [&]( const uint4* region, uint32_t first_token, uint32_t j ) { // chunk j of a region of 64 tokens
      const uint32_t token = j / CHUNKS, slot = j % CHUNKS;
      const uint32_t chunk = slot ^ ( token & SWZ_MASK );
      const uint32_t col = tile_col0 + first_token + token, row = tile_row0 + 8 * chunk;
      if ( col < b && row < r ) {
        // two products that share their activations in one launch (r_first % 8 == 0: a 16-byte chunk never straddles the two)
        const bool second = row >= r_first;
        uint4* dst = reinterpret_cast<uint4*>( second ? xout2 + (uint64_t)col * ( r - r_first ) + ( row - r_first ) : xout + (uint64_t)col * r_first + row );
        union
        {
          uint4 raw;
          __half h[8];
        } y, old;
        y.raw = region[j];
        if ( EPI == EPI_ACCUM ) { // the op that follows the product, on the rounded product
          old.raw = *dst;
#pragma unroll
          for ( int e = 0; e < 8; e++ ) {
            y.h[e] = __float2half_rn( __half2float( old.h[e] ) + __half2float( y.h[e] ) );
          }
        }
        *dst = y.raw;
      }
    };
    if constexpr ( NA == 2 ) { // four regions of 64 tokens x 256 rows = the four stage arrays
#pragma unroll
      for ( int t = 0; t < 4; t++ ) {
        put( wc == 0 ? ( t < 2 ? s_x0 : s_x1 ) : ( t < 2 ? s_w0 : s_w1 ), t );
      }
      __syncthreads();
#pragma unroll
      for ( int it = 0; it < 16; it++ ) {
        const uint4* region = it < 4 ? s_x0 : it < 8 ? s_x1 : it < 12 ? s_w0 : s_w1;
        copy_out( region, 64 * ( it / 4 ), ( it % 4 ) * T256_THREADS + threadIdx.x );
      }
    } else { // 64 tokens x 384 rows fill a weight stage: the two token halves of the tile one after the other
#pragma unroll
      for ( int half = 0; half < 2; half++ ) {
        if ( half == 1 ) {
          __syncthreads();
        }
        if ( wc == (uint32_t)half ) {
#pragma unroll
          for ( int t = 0; t < 4; t++ ) {
            put( t < 2 ? s_w0 : s_w1, t );
          }
        }
        __syncthreads();
#pragma unroll
        for ( int it = 0; it < 12; it++ ) {
          copy_out( it < 6 ? s_w0 : s_w1, 128 * half + 64 * ( it / 6 ), ( it % 6 ) * T256_THREADS + threadIdx.x );
        }
      }
    }
    return;
  }
#pragma unroll
  for ( int t = 0; t < 4; t++ ) {
    const uint32_t col = tile_col0 + 128 * wc + 32 * t + fr;
    if ( col >= b ) {
      continue;
    }
#pragma unroll
    for ( int rt = 0; rt < NA; rt++ ) {
#pragma unroll
      for ( int q4 = 0; q4 < 4; q4++ ) {
        const uint32_t row = tile_row0 + 32 * NA * wr + 32 * rt + 8 * q4 + 4 * g2;
        const bool whole = row + 3 < r && ( r & 3 ) == 0;
        if ( PARTIAL ) {
          float* dst = partial + ( (uint64_t)blockIdx.y * b + col ) * r + row;
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
          __half* dst = xout + (uint64_t)col * r + row; // (one output only: the launch refuses two with r % 8 != 0)
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

// The same 256 x 256 tile with FOUR waves of 128 x 128 (2 x 2), one wave per SIMD: 16 accumulators of v_mfma_f32_32x32x16_f16,
// 256 registers, which the compiler keeps in the accumulation half of the register file (512 registers per lane with one wave per
// SIMD), so the 256 ordinary registers are free for operands and addresses.  Against 64 x 128 per wave a 16-k group of a wave
// needs 8 fragment reads for 16 MFMAs instead of 6 for 8: a third less LDS traffic per flop, half as many waves at the barrier.
//
//   schedule    With one wave per SIMD nothing else fills a stall, so the loop is laid out instruction by instruction
//               (sched_group_barrier).  A step is four groups of 16 MFMAs.  Beside the first 8 MFMAs of a group go the 8 fragment
//               reads of the NEXT group (two fragment sets in turn).  The barrier that ends the step stands in front of its last
//               group: behind it the wave requests the first fragments of the next stage and still has 16 MFMAs in hand while
//               they arrive.
//   operands    global -> registers -> LDS, two steps ahead: the 16 loads of step j + 2 go out four to a group all through step
//               j, and the 16 registers loaded during step j - 1 (step j + 1) are written to the other stage beside the first
//               three groups of step j.  Every memory instruction of the loop is spread evenly between the MFMAs; that is what
//               counts.  Measured at 16384 x 8192 x 8192 (matrix pipes busy of 4 per CU, clock): without any loads 3.74, 1.87 GHz,
//               1.8-1.9 PFLOP/s; 16 loads back to back at the head of a step and never waited for 2.92 (the wave cannot issue
//               MFMAs while its memory instructions queue for the address unit); loads straight to LDS one step ahead, in
//               two bursts, 2.57, 1.04-1.07 PFLOP/s; the same spread evenly 1.28-1.30; as built here 3.48 at 1.29 GHz, 1.30
//               PFLOP/s (the vendor library's kernel on the same box: 3.71 at 1.39 GHz, 1.31-1.52; the eight-wave kernel above
//               3.05 at 1.35 GHz, 1.13-1.26).  Under this load the part runs at the clock its power budget allows.
//   loop shape  one loop of two steps with a single exit: with the exit test between the steps (an odd number of steps) the
//               compiler moved accumulators between the two register halves inside the loop (hundreds of copies per
//               step and spills), so the kernel takes K ranges of an even number of 64-k steps only.
//   work        either one tile per work-group in the tile order above, or (gemm_w4_streamk_kernel) one work-group per CU that
//               walks an equal share of ALL the 64-k steps of the product, tile after tile: a product of 416 tiles on 256 CUs
//               then takes 1.6 tiles' time instead of 2.  Tiles that a share covers whole are finished on the spot; the two
//               pieces at the ends of a share leave fp32 sums in a buffer and gemm_w4_fixup_kernel adds the pieces of each
//               divided tile in ascending order of the share (a fixed order: results repeat bit for bit).
constexpr int T4_THREADS = 256;

struct W4Stages
{
  uint4 *w0, *x0, *w1, *x1; // four separate arrays: see gemm_tile256_kernel
};

// acc = w[tile rows] . x[tile tokens]^T over n_steps (even) steps of 64 k, both descriptors starting at the range's first k.
__device__ __forceinline__ void w4_multiply( f32x16 ( &acc )[4][4], const __amdgpu_buffer_rsrc_t w_rsrc, const __amdgpu_buffer_rsrc_t x_rsrc, uint32_t ld_bytes,
                                             uint32_t n_steps, const W4Stages& st )
{
  const uint32_t wave = __builtin_amdgcn_readfirstlane( threadIdx.x >> 6 );
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wr = wave >> 1, wc = wave & 1;
  const uint32_t fr = lane & 31, g2 = lane >> 5;
  // thread t holds slot t % 8 of row t / 8 (+ 32 i): it fetches the chunk that the swizzle keeps in that slot
  const uint32_t voff = ( threadIdx.x >> 3 ) * ld_bytes + ( ( threadIdx.x & 7 ) ^ ( ( threadIdx.x >> 4 ) & 7 ) ) * 16;
  const uint32_t slot0 = 8 * wave * 8 + lane; // this thread's uint4 in the wave's 8 rows
#pragma unroll
  for ( int rt = 0; rt < 4; rt++ ) {
#pragma unroll
    for ( int t = 0; t < 4; t++ ) {
#pragma unroll
      for ( int e = 0; e < 16; e++ ) {
        acc[rt][t][e] = 0.f;
      }
    }
  }
  struct Frags
  {
    f16x8 a[4], bb[4];
  };
  Frags f0, f1;
  uint4 ra[16], rq[16]; // W0 X0 W1 X1 ... W7 X7 of a step (32 rows of the tile each), two steps in turn
  auto read_k16 = [&]( Frags& f, const uint4* wt, const uint4* xt, int kk ) __attribute__( ( always_inline ) ) {
    const uint32_t ch = 2 * kk + g2;
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      f.a[i] = __builtin_bit_cast( f16x8, wt[swz( 128 * wr + 32 * i + fr, ch )] );
      f.bb[i] = __builtin_bit_cast( f16x8, xt[swz( 128 * wc + 32 * i + fr, ch )] );
    }
  };
  auto mfma_k16 = [&]( const Frags& f ) __attribute__( ( always_inline ) ) {
#pragma unroll
    for ( int t = 0; t < 4; t++ ) {
#pragma unroll
      for ( int rt = 0; rt < 4; rt++ ) {
        acc[rt][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16( f.a[rt], f.bb[t], acc[rt][t], 0, 0, 0 );
      }
    }
  };
  auto load_part = [&]( uint4* set, uint32_t kb, int from, int to ) __attribute__( ( always_inline ) ) {
#pragma unroll
    for ( int l = 0; l < 16; l++ ) {
      if ( l >= from && l < to ) {
        set[l] = __builtin_bit_cast( uint4, __builtin_amdgcn_raw_buffer_load_b128( ( l & 1 ) == 0 ? w_rsrc : x_rsrc, voff, 32 * ( l >> 1 ) * ld_bytes + kb, 0 ) );
      }
    }
  };
  auto store_part = [&]( const uint4* set, uint4* wn, uint4* xn, int from, int to ) __attribute__( ( always_inline ) ) {
#pragma unroll
    for ( int l = 0; l < 16; l++ ) {
      if ( l >= from && l < to ) {
        ( ( l & 1 ) == 0 ? wn : xn )[slot0 + 32 * ( l >> 1 ) * 8] = set[l];
      }
    }
  };
  // order of a group: MFMA i with an LDS read (i < 8), a load (i = 1, 5, 9, 13) and an LDS write (the first n_st of i = 2, 4, 7, 10, 12, 15)
  auto order = [&]( int n_st ) __attribute__( ( always_inline ) ) {
    int done = 0;
#pragma unroll
    for ( int i = 0; i < 16; i++ ) {
      __builtin_amdgcn_sched_group_barrier( 0x008, 1, 0 ); // one MFMA
      if ( i < 8 ) {
        __builtin_amdgcn_sched_group_barrier( 0x100, 1, 0 ); // one LDS read
      }
      if ( ( i & 3 ) == 1 ) {
        __builtin_amdgcn_sched_group_barrier( 0x020, 1, 0 ); // one load
      }
      if ( ( i == 2 || i == 4 || i == 7 || i == 10 || i == 12 || i == 15 ) && done < n_st ) {
        __builtin_amdgcn_sched_group_barrier( 0x200, 1, 0 ); // one LDS write
        done++;
      }
    }
  };
  // f0 holds the first group of stage (wt, xt) on entry and that of stage (wn, xn) on exit; `loaded` holds the operands of step
  // j + 1, `loading` receives those of step j + 2 (behind the last step: the start of the next rows, bounded by the descriptors,
  // never multiplied)
  auto step = [&]( const uint4* wt, const uint4* xt, uint4* wn, uint4* xn, uint4* loading, const uint4* loaded, uint32_t j ) __attribute__( ( always_inline ) ) {
    const uint32_t kb = ( j + 2 ) * TKS * 2;
    read_k16( f1, wt, xt, 1 );
    load_part( loading, kb, 0, 4 );
    store_part( loaded, wn, xn, 0, 6 );
    mfma_k16( f0 );
    order( 6 );
    __builtin_amdgcn_sched_barrier( 0 );
    read_k16( f0, wt, xt, 2 );
    load_part( loading, kb, 4, 8 );
    store_part( loaded, wn, xn, 6, 11 );
    mfma_k16( f1 );
    order( 5 );
    __builtin_amdgcn_sched_barrier( 0 );
    read_k16( f1, wt, xt, 3 );
    load_part( loading, kb, 8, 12 );
    store_part( loaded, wn, xn, 11, 16 );
    mfma_k16( f0 );
    order( 5 );
    __builtin_amdgcn_sched_barrier( 0 );
    __syncthreads(); // the next stage is written, and every wave has read the last fragments of this one
    __builtin_amdgcn_sched_barrier( 0 );
    read_k16( f0, wn, xn, 0 );
    load_part( loading, kb, 12, 16 );
    mfma_k16( f1 );
    order( 0 );
    __builtin_amdgcn_sched_barrier( 0 );
  };
  load_part( ra, 0, 0, 16 );
  load_part( rq, TKS * 2, 0, 16 );
  store_part( ra, st.w0, st.x0, 0, 16 );
  __syncthreads();
  read_k16( f0, st.w0, st.x0, 0 );
  for ( uint32_t j = 0; j < n_steps; j += 2 ) {
    step( st.w0, st.x0, st.w1, st.x1, ra, rq, j );
    step( st.w1, st.x1, st.w0, st.x0, rq, ra, j + 1 );
  }
}

// acc[rt][t][v]: row = tile_row0 + 128*wr + 32*rt + 8*(v/4) + 4*(lane/32) + v%4, token = tile_col0 + 128*wc + 32*t + lane%32.
// Output of a whole tile: through LDS (token-major, the four stage arrays as four regions of 64 tokens x 256 rows) as whole row
// segments where r % 8 == 0, else (and for the fp32 sums of a K split) from the registers.
struct W4Out
{
  __half* xout;
  __half* xout2;    // rows from r_first on go here, as rows 0.. of a (b, r - r_first) matrix
  float* partial;   // EPI_PARTIAL: (splits, b, r)
  uint32_t r, b, r_first, split;
};

template<int EPI>
__device__ __forceinline__ void w4_store_tile( f32x16 ( &acc )[4][4], const W4Out& o, uint32_t tile_row0, uint32_t tile_col0, const W4Stages& st )
{
  const uint32_t wave = __builtin_amdgcn_readfirstlane( threadIdx.x >> 6 );
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wr = wave >> 1, wc = wave & 1;
  const uint32_t fr = lane & 31, g2 = lane >> 5;
  constexpr bool PARTIAL = EPI == EPI_PARTIAL;
  if ( !PARTIAL && ( o.r & 7 ) == 0 ) {
    __syncthreads(); // (the fragments requested behind the last barrier are not used; nothing is in flight into the arrays any more)
    constexpr uint32_t CHUNKS = TM2 / 8; // 16-byte chunks per token
    constexpr uint32_t SWZ_MASK = 31;
#pragma unroll
    for ( int t = 0; t < 4; t++ ) {
      uint2* out = reinterpret_cast<uint2*>( wc == 0 ? ( t < 2 ? st.x0 : st.x1 ) : ( t < 2 ? st.w0 : st.w1 ) );
      const uint32_t token = 32 * ( t & 1 ) + fr;
#pragma unroll
      for ( int rt = 0; rt < 4; rt++ ) {
#pragma unroll
        for ( int q4 = 0; q4 < 4; q4++ ) {
          union
          {
            uint2 raw;
            __half h[4];
          } v;
#pragma unroll
          for ( int e = 0; e < 4; e++ ) {
            v.h[e] = __float2half_rn( acc[rt][t][4 * q4 + e] );
          }
          const uint32_t chunk = 16 * wr + 4 * rt + q4;
          out[( token * CHUNKS + ( chunk ^ ( token & SWZ_MASK ) ) ) * 2 + g2] = v.raw;
        }
      }
    }
    __syncthreads();
#pragma unroll 4
    for ( int it = 0; it < 32; it++ ) {
      const uint4* region = it < 8 ? st.x0 : it < 16 ? st.x1 : it < 24 ? st.w0 : st.w1;
      const uint32_t j = ( it % 8 ) * T4_THREADS + threadIdx.x;
      const uint32_t token = j / CHUNKS, slot = j % CHUNKS;
      const uint32_t chunk = slot ^ ( token & SWZ_MASK );
      const uint32_t col = tile_col0 + 64 * ( it / 8 ) + token, row = tile_row0 + 8 * chunk;
      if ( col < o.b && row < o.r ) {
        const bool second = row >= o.r_first; // two products that share their activations in one launch (r_first % 8 == 0)
        uint4* dst = reinterpret_cast<uint4*>( second ? o.xout2 + (uint64_t)col * ( o.r - o.r_first ) + ( row - o.r_first ) : o.xout + (uint64_t)col * o.r_first + row );
        union
        {
          uint4 raw;
          __half h[8];
        } y, old;
        y.raw = region[j];
        if ( EPI == EPI_ACCUM ) { // the op that follows the product, on the rounded product
          old.raw = *dst;
#pragma unroll
          for ( int e = 0; e < 8; e++ ) {
            y.h[e] = __float2half_rn( __half2float( old.h[e] ) + __half2float( y.h[e] ) );
          }
        }
        *dst = y.raw;
      }
    }
    return;
  }
#pragma unroll
  for ( int t = 0; t < 4; t++ ) {
    const uint32_t col = tile_col0 + 128 * wc + 32 * t + fr;
    if ( col >= o.b ) {
      continue;
    }
#pragma unroll
    for ( int rt = 0; rt < 4; rt++ ) {
#pragma unroll
      for ( int q4 = 0; q4 < 4; q4++ ) {
        const uint32_t row = tile_row0 + 128 * wr + 32 * rt + 8 * q4 + 4 * g2;
        const bool whole = row + 3 < o.r && ( o.r & 3 ) == 0;
        if ( PARTIAL ) {
          float* dst = o.partial + ( (uint64_t)o.split * o.b + col ) * o.r + row;
          if ( whole ) {
            *reinterpret_cast<float4*>( dst ) = make_float4( acc[rt][t][4 * q4], acc[rt][t][4 * q4 + 1], acc[rt][t][4 * q4 + 2], acc[rt][t][4 * q4 + 3] );
          } else {
            for ( int e = 0; e < 4; e++ ) {
              if ( row + e < o.r ) {
                dst[e] = acc[rt][t][4 * q4 + e];
              }
            }
          }
        } else {
          __half* dst = o.xout + (uint64_t)col * o.r + row; // (one output only: the launch refuses two with r % 8 != 0)
          if ( whole ) {
            union
            {
              uint2 raw;
              __half h[4];
            } v;
#pragma unroll
            for ( int e = 0; e < 4; e++ ) {
              v.h[e] = __float2half_rn( acc[rt][t][4 * q4 + e] );
            }
            *reinterpret_cast<uint2*>( dst ) = v.raw;
          } else {
            for ( int e = 0; e < 4; e++ ) {
              if ( row + e < o.r ) {
                dst[e] = __float2half_rn( acc[rt][t][4 * q4 + e] );
              }
            }
          }
        }
      }
    }
  }
}

// grid as gemm_tile256_kernel: 8 x (padded tiles of one XCD) by K splits; k_len % 128 == 0, s % 128 == 0
template<int EPI>
__global__ __launch_bounds__( T4_THREADS, 1 ) void gemm_tile256w4_kernel( __half* __restrict__ xout,
                                                                        float* __restrict__ partial,
                                                                        const __half* __restrict__ x,
                                                                        const __half* __restrict__ w,
                                                                        uint32_t s,
                                                                        uint32_t r,
                                                                        uint32_t b,
                                                                        uint32_t k_len,
                                                                        __half* __restrict__ xout2,
                                                                        uint32_t r_first,
                                                                        TileOrder ord )
{
  __shared__ uint4 s_x0[TN2 * 8], s_x1[TN2 * 8];
  __shared__ uint4 s_w0[TM2 * 8], s_w1[TM2 * 8];
  uint32_t row_tile, token_tile;
  if ( !tile_of_workgroup( ord, row_tile, token_tile ) ) {
    return;
  }
  const uint32_t tile_row0 = row_tile * TM2, tile_col0 = token_tile * TN2;
  const uint32_t ld_bytes = s * 2;
  const uint32_t w_rows = min( (uint32_t)TM2, r - tile_row0 ), x_cols = min( (uint32_t)TN2, b - tile_col0 );
  const uint32_t k0 = blockIdx.y * k_len; // this split's k range starts here; the descriptors start there too and end with the tile's last row
  const __amdgpu_buffer_rsrc_t w_rsrc
    = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( w + (uint64_t)tile_row0 * s + k0 ), 0, (int)( w_rows * ld_bytes - k0 * 2 ), 0x00020000 );
  const __amdgpu_buffer_rsrc_t x_rsrc
    = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( x + (uint64_t)tile_col0 * s + k0 ), 0, (int)( x_cols * ld_bytes - k0 * 2 ), 0x00020000 );
  const W4Stages st { s_w0, s_x0, s_w1, s_x1 };
  f32x16 acc[4][4];
  w4_multiply( acc, w_rsrc, x_rsrc, ld_bytes, min( k_len, s - k0 ) / TKS, st );
  const W4Out o { xout, xout2, partial, r, b, r_first, blockIdx.y };
  w4_store_tile<EPI>( acc, o, tile_row0, tile_col0, st );
}

// Equal shares of all the 64-k steps of a product.  Tile t (token fastest: t = row tile x token tiles + token tile) owns the steps
// [t * steps, (t + 1) * steps) of the product's list; share g takes [g * share, (g + 1) * share) of it, an even number of steps.
// Shares are dealt to the work-groups so that the 32 of an XCD (work-groups x, x + 8, ...) hold neighbouring shares: their tiles
// are a few neighbouring row tiles over all their token tiles and share their operands in that XCD's L2.
struct StreamK
{
  uint32_t tiles, token_tiles, steps, share, shares;
  float* pieces; // (shares, 2) pieces of 256 x 256 fp32 sums in register order: [wave][rt][t][v / 4][lane][v % 4]
};
constexpr uint64_t PIECE_FLOATS = (uint64_t)TM2 * TN2;

__device__ __forceinline__ uint32_t streamk_share_of_workgroup( const StreamK& sk )
{
  const uint32_t per_xcd = ( sk.shares + 7 ) / 8; // work-group g runs on XCD g % 8
  return ( blockIdx.x & 7 ) * per_xcd + ( blockIdx.x >> 3 );
}

// grid: 8 * ceil(shares / 8) work-groups, one per CU
template<int EPI>
__global__ __launch_bounds__( T4_THREADS, 1 ) void gemm_w4_streamk_kernel( __half* __restrict__ xout,
                                                                         const __half* __restrict__ x,
                                                                         const __half* __restrict__ w,
                                                                         uint32_t s,
                                                                         uint32_t r,
                                                                         uint32_t b,
                                                                         __half* __restrict__ xout2,
                                                                         uint32_t r_first,
                                                                         StreamK sk )
{
  __shared__ uint4 s_x0[TN2 * 8], s_x1[TN2 * 8];
  __shared__ uint4 s_w0[TM2 * 8], s_w1[TM2 * 8];
  const uint32_t g = streamk_share_of_workgroup( sk );
  const uint64_t total = (uint64_t)sk.tiles * sk.steps;
  const uint64_t begin = (uint64_t)g * sk.share;
  if ( g >= sk.shares || begin >= total ) {
    return;
  }
  const uint64_t end = min( total, begin + sk.share );
  const W4Stages st { s_w0, s_x0, s_w1, s_x1 };
  const uint32_t ld_bytes = s * 2;
  const uint32_t first_tile = (uint32_t)( begin / sk.steps );
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for ( uint64_t at = begin; at < end; ) {
    const uint32_t tile = (uint32_t)( at / sk.steps );
    const uint32_t step0 = (uint32_t)( at - (uint64_t)tile * sk.steps );
    const uint32_t n_steps = (uint32_t)min( (uint64_t)( sk.steps - step0 ), end - at );
    const uint32_t tile_row0 = ( tile / sk.token_tiles ) * TM2, tile_col0 = ( tile % sk.token_tiles ) * TN2;
    const uint32_t w_rows = min( (uint32_t)TM2, r - tile_row0 ), x_cols = min( (uint32_t)TN2, b - tile_col0 );
    const uint32_t k0 = step0 * TKS;
    const __amdgpu_buffer_rsrc_t w_rsrc
      = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( w + (uint64_t)tile_row0 * s + k0 ), 0, (int)( w_rows * ld_bytes - k0 * 2 ), 0x00020000 );
    const __amdgpu_buffer_rsrc_t x_rsrc
      = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( x + (uint64_t)tile_col0 * s + k0 ), 0, (int)( x_cols * ld_bytes - k0 * 2 ), 0x00020000 );
    f32x16 acc[4][4];
    w4_multiply( acc, w_rsrc, x_rsrc, ld_bytes, n_steps, st );
    if ( n_steps == sk.steps ) { // a whole tile: finished here
      const W4Out o { xout, xout2, nullptr, r, b, r_first, 0 };
      w4_store_tile<EPI>( acc, o, tile_row0, tile_col0, st );
    } else { // a piece: its sums as they lie in the registers, 1 KiB per wave and store
      float* piece = sk.pieces + ( (uint64_t)g * 2 + ( tile == first_tile ? 0 : 1 ) ) * PIECE_FLOATS + (uint64_t)wave * ( PIECE_FLOATS / 4 );
#pragma unroll
      for ( int rt = 0; rt < 4; rt++ ) {
#pragma unroll
        for ( int t = 0; t < 4; t++ ) {
#pragma unroll
          for ( int q4 = 0; q4 < 4; q4++ ) {
            *reinterpret_cast<float4*>( piece + ( ( ( rt * 4 + t ) * 4 + q4 ) * 64 + lane ) * 4 )
              = make_float4( acc[rt][t][4 * q4], acc[rt][t][4 * q4 + 1], acc[rt][t][4 * q4 + 2], acc[rt][t][4 * q4 + 3] );
          }
        }
      }
    }
    __syncthreads(); // the stage arrays serve the next tile
    at += n_steps;
  }
}

// One work-group per tile: nothing to do for a tile that one share covered whole; else the pieces of the tile added in ascending
// order of the share, then the same output path as a tile finished in the multiply kernel.
template<int EPI>
__global__ __launch_bounds__( T4_THREADS, 1 ) void gemm_w4_fixup_kernel( __half* __restrict__ xout, uint32_t r, uint32_t b, __half* __restrict__ xout2, uint32_t r_first,
                                                                       StreamK sk )
{
  __shared__ uint4 s_x0[TN2 * 8], s_x1[TN2 * 8];
  __shared__ uint4 s_w0[TM2 * 8], s_w1[TM2 * 8];
  const uint32_t tile = blockIdx.x;
  const uint64_t t_begin = (uint64_t)tile * sk.steps, t_end = t_begin + sk.steps;
  const uint32_t g_first = (uint32_t)( t_begin / sk.share ), g_last = (uint32_t)( ( t_end - 1 ) / sk.share );
  if ( g_first == g_last ) {
    return;
  }
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  f32x16 acc[4][4];
#pragma unroll
  for ( int rt = 0; rt < 4; rt++ ) {
#pragma unroll
    for ( int t = 0; t < 4; t++ ) {
#pragma unroll
      for ( int e = 0; e < 16; e++ ) {
        acc[rt][t][e] = 0.f;
      }
    }
  }
  for ( uint32_t g = g_first; g <= g_last; g++ ) {
    const uint32_t first_tile = (uint32_t)( (uint64_t)g * sk.share / sk.steps );
    const float* piece = sk.pieces + ( (uint64_t)g * 2 + ( tile == first_tile ? 0 : 1 ) ) * PIECE_FLOATS + (uint64_t)wave * ( PIECE_FLOATS / 4 );
#pragma unroll
    for ( int rt = 0; rt < 4; rt++ ) {
#pragma unroll
      for ( int t = 0; t < 4; t++ ) {
#pragma unroll
        for ( int q4 = 0; q4 < 4; q4++ ) {
          const float4 v = *reinterpret_cast<const float4*>( piece + ( ( ( rt * 4 + t ) * 4 + q4 ) * 64 + lane ) * 4 );
          acc[rt][t][4 * q4] += v.x;
          acc[rt][t][4 * q4 + 1] += v.y;
          acc[rt][t][4 * q4 + 2] += v.z;
          acc[rt][t][4 * q4 + 3] += v.w;
        }
      }
    }
  }
  const W4Stages st { s_w0, s_x0, s_w1, s_x1 };
  const W4Out o { xout, xout2, nullptr, r, b, r_first, 0 };
  w4_store_tile<EPI>( acc, o, ( tile / sk.token_tiles ) * TM2, ( tile % sk.token_tiles ) * TN2, st );
}

// GLINT_TILE_ROWS in the environment sets the start value (for the command-line profilers, which have no other way in)
int tile_rows_default()
{
  const char* env = getenv( "GLINT_TILE_ROWS" );
  return env != nullptr && *env != '\0' ? atoi( env ) : 0;
}
int g_tile_rows = tile_rows_default(); // 0: by the cost rules below; 256 or 384: the eight-wave kernel with that many rows; 128, 129: below
// measurement hook (tile rows): 256 or 384 force the eight-wave kernel, 128 the four-wave one with one tile per work-group, 129 the
// four-wave one over equal shares of all steps; 0: the four-wave kernel wherever it applies, equal shares where whole tiles fit badly

// Rounds of one work-group per CU that an XCD (32 CUs) runs for its share of the tiles.
uint64_t rounds_per_xcd( uint64_t r, uint64_t b, uint64_t tile_rows )
{
  const uint64_t row_tiles = ( r + tile_rows - 1 ) / tile_rows, token_tiles = ( b + TN2 - 1 ) / TN2;
  const uint64_t tiles = ( row_tiles / 8 ) * token_tiles + ( ( row_tiles % 8 ) * token_tiles + 7 ) / 8;
  return ( tiles + 31 ) / 32;
}

// 384 rows per work-group when that takes less time: rounds x the time of a round.  Measured at
// 16384 tokens x 12288 rows (12 rounds of 256-row tiles, 8 of 384-row tiles), a round of 384-row
// tiles takes 1.41-1.44 x a round of 256-row tiles for K 7168-13824 and 1.24-1.39 x for shorter K (the
// cost of starting and storing a tile is paid for 1.5 x the flops), against 1.5 x the flops.
uint32_t tile256_rows( uint64_t s, uint64_t r, uint64_t b )
{
  if ( g_tile_rows == 256 || g_tile_rows == 384 ) {
    return (uint32_t)g_tile_rows;
  }
  if ( g_tile_rows == 128 || g_tile_rows == 129 ) {
    return 256;
  }
  const uint64_t round_cost_pct = s >= 7168 ? 143 : 136;
  return round_cost_pct * rounds_per_xcd( r, b, 384 ) < 97 * rounds_per_xcd( r, b, 256 ) ? 384 : 256; // 3 % in hand for 256
}

// Whether a product runs over equal shares of all its steps, and how: worth it when whole tiles would leave the last round of
// one tile per CU partly empty.  `force`: whenever the shape allows.
bool streamk_plan( uint64_t s, uint64_t r, uint64_t b, bool force, StreamK* sk )
{
  const uint64_t cus = (uint64_t)cu_count();
  const uint64_t row_tiles = ( r + TM2 - 1 ) / TM2, token_tiles = ( b + TN2 - 1 ) / TN2;
  const uint64_t tiles = row_tiles * token_tiles, steps = s / TKS;
  if ( tiles == 0 || steps < 4 || steps % 2 != 0 || tiles > 0xffffffull ) {
    return false;
  }
  const uint64_t rounds = ( tiles + cus - 1 ) / cus;
  const uint64_t share = ( ( tiles * steps + 2 * cus - 1 ) / ( 2 * cus ) ) * 2; // even
  // in steps of one CU: whole tiles take rounds x steps; shares take `share` plus the pieces' way through memory (one step's
  // time for a piece written and one for a piece read is generous) and a second launch
  // Measured (3328 tokens, 70B shapes): shares that start in the middle of tiles walk K out of step with their neighbours, so an
  // operand strip is no longer fetched into the XCD's L2 once for all the tiles that use it at that moment, and the multiply
  // runs at about three quarters of its rate in whole tiles; the pieces cost a launch and 2 x 256 KiB of traffic each on top.
  // 520 tiles (2.03 rounds, 3 as whole tiles): 493 against 543 us; 416 tiles (1.63 rounds): 452 against 392 us.  So only where
  // whole tiles waste more than 30 % of their rounds.
  const bool pays = 100 * ( share + 6 ) < 70 * rounds * steps && share >= 8;
  if ( !force && !pays ) {
    return false;
  }
  sk->tiles = (uint32_t)tiles;
  sk->token_tiles = (uint32_t)token_tiles;
  sk->steps = (uint32_t)steps;
  sk->share = (uint32_t)std::max<uint64_t>( share, 2 );
  sk->shares = (uint32_t)( ( tiles * steps + sk->share - 1 ) / sk->share );
  sk->pieces = nullptr;
  return true;
}

} // namespace

void gemm_tile256_tuning( int rows ) { g_tile_rows = rows; }

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

// A launch is as slow as its number of rounds (one work-group per CU), so a product whose tiles leave the last round mostly
// empty pays for a whole round there: 8192 rows x 4480 tokens are 576 tiles of 256 x 256, 2.25 rounds, and take 3.  Such a product
// is cut in two along the tokens: the first part a number of tokens whose tiles fill their rounds, the rest a product of a few
// hundred tokens that goes its own way (smaller tiles, or this kernel with the K range split).  Returns the tokens of the first
// part, 0 to leave the product whole.  Costs in percent of a round of 256-row tiles; a round of 384-row tiles as in tile256_rows().
uint64_t gemm_tile256_token_split( uint64_t s, uint64_t r, uint64_t b )
{
  if ( g_tile_rows != 0 || b < 3 * TN2 ) {
    return 0;
  }
  const uint64_t cost384 = s >= 7168 ? 143 : 136;
  auto cost = [&]( uint64_t tokens ) { return std::min( 100 * rounds_per_xcd( r, tokens, 256 ), cost384 * rounds_per_xcd( r, tokens, 384 ) ); };
  const uint64_t whole = cost( b );
  uint64_t best = whole, best_b1 = 0;
  const uint64_t token_tiles = b / TN2;
  for ( uint64_t t = token_tiles; t + 8 >= token_tiles && t >= 2; t-- ) {
    const uint64_t b1 = t * TN2;
    if ( b1 >= b ) {
      continue;
    }
    // the rest: its flops in rounds of this kernel, at 60 % of this kernel's rate, plus a start-up
    const uint64_t rest = 100 * ( b - b1 ) * r / ( (uint64_t)TM2 * TN2 * (uint64_t)cu_count() ) * 10 / 6 + 15;
    const uint64_t c = cost( b1 ) + rest;
    if ( c < best ) {
      best = c;
      best_b1 = b1;
    }
  }
  return 100 * best < 92 * whole ? best_b1 : 0;
}

// Few tiles (a decode step of some hundred rows, or a narrow product): the K range is split over several work-groups per tile so
// that the chip is full in one round, and the fp32 sums of each split go to partial[split].  *splits = 0: not for this shape.
void gemm_tile256_split_plan( uint64_t s, uint64_t r, uint64_t b, const void* x, const void* w, uint32_t* splits, uint32_t* k_len )
{
  *splits = 0;
  *k_len = 0;
  const uint64_t tiles = ( ( r + TM2 - 1 ) / TM2 ) * ( ( b + TN2 - 1 ) / TN2 );
  const uint64_t cus = (uint64_t)cu_count();
  if ( b < 192 || tiles * 2 > cus || s % TKS != 0 || s >= ( 1u << 22 ) || ( ( reinterpret_cast<uintptr_t>( x ) | reinterpret_cast<uintptr_t>( w ) ) & 15u ) != 0 ) {
    return;
  }
  const uint64_t steps = s / TKS;
  // Very few tiles and a short K (70B wo at 256 rows: 32 tiles, 8 splits of 16 steps, fp32 sums half the size of the weights):
  // the 128 x 128 kernel with two work-groups per CU hides more of such a short work-group's start-up (60 against 73 us).
  if ( tiles * 8 <= cus && steps <= 128 ) {
    return;
  }
  uint64_t n = std::min<uint64_t>( cus / tiles, steps / 16 ); // at least 16 steps of 64 k per split
  if ( n < 2 ) {
    return;
  }
  const uint64_t steps_per_split = ( steps + n - 1 ) / n;
  *k_len = (uint32_t)( steps_per_split * TKS );
  *splits = (uint32_t)( ( steps + steps_per_split - 1 ) / steps_per_split );
}

// `partial` != nullptr: fp32 sums (splits, b, r) instead of xout; else `epilogue` 0 stores, 1 accumulates into xout (needs r % 8 == 0).
// splits > 1 (from gemm_tile256_split_plan, with its k_len) needs `partial`.
int gemm_tile256_launch( __half* xout, float* partial, const __half* x, const __half* w, uint64_t s, uint64_t r, uint64_t b, int epilogue, hipStream_t st,
                         uint32_t splits, uint32_t k_len, __half* xout2 = nullptr, uint64_t r_first = 0 )
{
  if ( xout2 == nullptr ) {
    r_first = r;
  }
  GH_REQUIRE( xout2 == nullptr || ( partial == nullptr && epilogue == EPI_STORE && splits == 1 && r % 8 == 0 && r_first % 8 == 0 && r_first > 0 && r_first < r ),
              "gh_matmul: two outputs need plain stores, no K split and row counts that are multiples of 8" );
  TileOrder ord;
  GH_REQUIRE( splits >= 1 && ( splits == 1 || ( partial != nullptr && k_len % TKS == 0 && (uint64_t)k_len * splits >= s && (uint64_t)k_len * ( splits - 1 ) < s ) ),
              "gh_matmul: bad K split for the 256-token tile kernel" );
  if ( splits == 1 ) {
    k_len = (uint32_t)s;
  }
  // four waves of 128 x 128 where the K range of every split is an even number of 64-k steps
  const bool even_steps = s % ( 2 * TKS ) == 0 && k_len % ( 2 * TKS ) == 0;
  // Measured against the eight-wave kernel (same box, same run): a round of four-wave tiles takes 0.92-0.97 of a round of
  // eight-wave 256-row tiles where the chip is full (16384 tokens: 70B shapes 1.29-1.32 against 1.20-1.29 PFLOP/s, 13B wq 1.22
  // against 1.16, w2 1.31 against 1.22), and more where it is not (1024 tokens x 8192 x 8192, half a round: 179 against 146 us --
  // with idle CUs the part is not held back by its power budget, and two waves per SIMD cover a tile's start and end better).
  const uint64_t cus = (uint64_t)cu_count();
  const uint64_t tiles256 = ( ( r + TM2 - 1 ) / TM2 ) * ( ( b + TN2 - 1 ) / TN2 );
  const uint64_t cost384 = s >= 7168 ? 143 : 136;
  // Most of a round is enough: 224 tiles (w1 and w3 of the 70B shape at 256 tokens) 221 against 254 us, at 512 tokens 428 against 484.
  const bool four_pays = 4 * tiles256 >= 3 * cus && 94 * rounds_per_xcd( r, b, 256 ) <= cost384 * rounds_per_xcd( r, b, 384 );
  const bool four_waves = even_steps && ( g_tile_rows == 128 || g_tile_rows == 129 || ( g_tile_rows == 0 && splits == 1 && four_pays ) );
  GH_REQUIRE( ( g_tile_rows != 128 && g_tile_rows != 129 ) || even_steps, "gh_matmul: the four-wave tile kernel needs K ranges that are multiples of 128" );
  const int epi_sk = epilogue;
  if ( four_waves && splits == 1 && partial == nullptr && ( epi_sk == EPI_STORE || epi_sk == EPI_ACCUM ) && ( epi_sk != EPI_ACCUM || r % 8 == 0 ) ) {
    StreamK sk;
    if ( streamk_plan( s, r, b, g_tile_rows == 129, &sk ) ) {
      void* pieces = nullptr;
      if ( int rc = stream_scratch( st, SCRATCH_GEMM_PIECES, (uint64_t)sk.shares * 2 * PIECE_FLOATS * sizeof( float ), 0, &pieces ) ) {
        return rc;
      }
      sk.pieces = static_cast<float*>( pieces );
      const unsigned wgs = 8 * ( ( sk.shares + 7 ) / 8 );
      if ( epi_sk == EPI_STORE ) {
        gemm_w4_streamk_kernel<EPI_STORE><<<wgs, T4_THREADS, 0, st>>>( xout, x, w, (uint32_t)s, (uint32_t)r, (uint32_t)b, xout2, (uint32_t)r_first, sk );
        gemm_w4_fixup_kernel<EPI_STORE><<<sk.tiles, T4_THREADS, 0, st>>>( xout, (uint32_t)r, (uint32_t)b, xout2, (uint32_t)r_first, sk );
      } else {
        gemm_w4_streamk_kernel<EPI_ACCUM><<<wgs, T4_THREADS, 0, st>>>( xout, x, w, (uint32_t)s, (uint32_t)r, (uint32_t)b, xout2, (uint32_t)r_first, sk );
        gemm_w4_fixup_kernel<EPI_ACCUM><<<sk.tiles, T4_THREADS, 0, st>>>( xout, (uint32_t)r, (uint32_t)b, xout2, (uint32_t)r_first, sk );
      }
      GH_LAUNCH_CHECK();
      return GH_OK;
    }
  }
  const uint32_t tile_rows = splits > 1 || four_waves ? 256 : tile256_rows( s, r, b );
  ord.row_tiles = (uint32_t)( ( r + tile_rows - 1 ) / tile_rows );
  ord.token_tiles = (uint32_t)( ( b + TN2 - 1 ) / TN2 );
  ord.gn = std::min<uint32_t>( ord.token_tiles, 8 );
  ord.rows_per_xcd = ord.row_tiles / 8;
  ord.gm = std::max<uint32_t>( 1, std::min<uint32_t>( std::max<uint32_t>( 1, 32 / ord.gn ), ord.rows_per_xcd ) ); // 32 CUs per XCD, one work-group each
  const uint32_t patches_m = ( ord.rows_per_xcd + ord.gm - 1 ) / ord.gm;
  ord.patches_n = ( ord.token_tiles + ord.gn - 1 ) / ord.gn;
  const uint64_t main_per_xcd = (uint64_t)patches_m * ord.patches_n * ord.gm * ord.gn;
  ord.rest_rows = ord.row_tiles - 8 * ord.rows_per_xcd;
  const uint64_t rest_share = ( (uint64_t)ord.rest_rows * ord.token_tiles + 7 ) / 8;
  const uint64_t gx = 8 * ( main_per_xcd + rest_share );
  GH_REQUIRE( gx < ( 1ull << 31 ), "gh_matmul: grid too large" );
  ord.main_per_xcd = (uint32_t)main_per_xcd;
  ord.rest_share = (uint32_t)rest_share;
  const dim3 grid( (unsigned)gx, splits ), block( four_waves ? T4_THREADS : T256_THREADS );
  const uint32_t s32 = (uint32_t)s, r32 = (uint32_t)r, b32 = (uint32_t)b;
  const int epi = partial != nullptr ? EPI_PARTIAL : epilogue;
  GH_REQUIRE( epi == EPI_STORE || epi == EPI_ACCUM || epi == EPI_PARTIAL, "gh_matmul: unknown tile epilogue %d", epi );
  GH_REQUIRE( epi != EPI_ACCUM || r % 8 == 0, "gh_matmul: the accumulating tile epilogue needs r %% 8 == 0" );
#define GH_TILE256_LAUNCH( E, N ) gemm_tile256_kernel<E, N><<<grid, block, 0, st>>>( xout, partial, x, w, s32, r32, b32, k_len, xout2, (uint32_t)r_first, ord )
#define GH_TILE256_W4( E ) gemm_tile256w4_kernel<E><<<grid, block, 0, st>>>( xout, partial, x, w, s32, r32, b32, k_len, xout2, (uint32_t)r_first, ord )
#define GH_TILE256_ROWS( E ) ( four_waves ? GH_TILE256_W4( E ) : tile_rows == 384 ? GH_TILE256_LAUNCH( E, 3 ) : GH_TILE256_LAUNCH( E, 2 ) )
  switch ( epi ) {
    case EPI_STORE: GH_TILE256_ROWS( EPI_STORE ); break;
    case EPI_ACCUM: GH_TILE256_ROWS( EPI_ACCUM ); break;
    default: GH_TILE256_ROWS( EPI_PARTIAL ); break;
  }
#undef GH_TILE256_ROWS
#undef GH_TILE256_W4
#undef GH_TILE256_LAUNCH
  GH_LAUNCH_CHECK();
  return GH_OK;
}

} // namespace gh
