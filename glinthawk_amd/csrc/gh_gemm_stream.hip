// Weight-streaming GEMM for decode: xout(b, r) = sum_p w(r, p) * x(b, p) with a small batch
// (64 columns per column slab), f16 storage, fp32 accumulate.  Every weight element is read from HBM
// exactly once, so the kernel is built like a streaming read:
//
//   work-group = 4 waves = up to 128 weight rows x one K range; wave = up to 32 rows x all 64 batch
//               columns (the planner may give a wave fewer rows of its 32-row MFMA tile so that the
//               number of work-groups suits the number of CUs)
//   weights     global -> registers with fully coalesced 16-byte buffer loads (scalar row/k offsets,
//               rows past the end read as zero by the descriptor's bound), non-temporal: they are
//               read once and should not displace the activations from L2.  A register slab is 32 rows
//               x 256 k, 512 contiguous bytes per row per visit.  Two register sets: slab i+1 is in
//               flight while slab i is consumed.  From registers each 128-k half goes through a
//               wave-private LDS tile (XOR-swizzled 16-byte chunks) into MFMA operand order.
//   k order     every work-group walks its K range from a different starting slab and wraps around.
//               Work-groups that start together would otherwise all read the same column range of
//               their rows, and rows are a power-of-two stride apart: those addresses fall on few
//               HBM channels (measured: 4.4 TB/s for 256-byte visits in lock step, 6.3 TB/s rotated).
//   activations one (64 x 128) tile per half shared by the work-group through LDS (two buffers); this
//               is the only block-level barrier and the weight loads stay in flight across it
//   math        v_mfma_f32_32x32x16_f16: A = 32 weight rows, B = 32 batch columns, two column tiles
//
// K is split across work-groups when there are too few row slabs to fill the chip; the fp32 partials
// are summed by gemm_reduce_kernel (gh_gemm.hip) or by the fused epilogues (gh_gemm_fused.hip).
// Without a split, w1 and w3 can share a launch that applies the SiLU gate itself (MODE_GATE).
#include "gh_common.h"

#include <cmath>
#include <type_traits>

namespace gh {

typedef _Float16 f16x8 __attribute__( ( ext_vector_type( 8 ) ) );
typedef float f32x16 __attribute__( ( ext_vector_type( 16 ) ) );

namespace {

constexpr int SLAB_K = 256;  // k per register slab: every row is read 512 contiguous bytes at a time
constexpr int HALF_K = 128;  // k per LDS tile: 16 chunks of 8 halves
constexpr int WG_ROWS = 128; // weight rows per work-group
constexpr int COLS = 64;     // batch columns per work-group

// one register slab of a wave: 32 rows x 256 k.  v[h][j], lane (g4, c): row 4*j + g4, 16-byte chunk c of half h
struct WSlab
{
  uint4 v[2][8];
};

// Weights are read once: the non-temporal hint keeps them from displacing the activations, which
// every work-group re-reads, from the L2 (measured: 7 to 10 % on the 70B projections).
__device__ __forceinline__ uint4 buffer_load16_stream( __amdgpu_buffer_rsrc_t rsrc, uint32_t lane_offset, uint32_t uniform_offset )
{
  return __builtin_bit_cast( uint4, __builtin_amdgcn_raw_buffer_load_b128( rsrc, lane_offset, uniform_offset, 2 /* nt */ ) );
}

__device__ __forceinline__ uint4 buffer_load16( __amdgpu_buffer_rsrc_t rsrc, uint32_t lane_offset, uint32_t uniform_offset )
{
  return __builtin_bit_cast( uint4, __builtin_amdgcn_raw_buffer_load_b128( rsrc, lane_offset, uniform_offset, 0 ) );
}

// `rsrc` starts at the wave's first row; lane_offset = g4 * row bytes + 16 c; kb = byte offset of the slab in the row
__device__ __forceinline__ void load_w_slab( WSlab& dst, __amdgpu_buffer_rsrc_t rsrc, uint32_t lane_offset, uint32_t ld_bytes, uint32_t kb )
{
#pragma unroll
  for ( int j = 0; j < 8; j++ ) {
    const uint32_t row_offset = 4 * j * ld_bytes + kb;
    // both halves of the row back to back: 512 contiguous bytes per row reach the memory system together
    dst.v[0][j] = buffer_load16_stream( rsrc, lane_offset, row_offset );
    dst.v[1][j] = buffer_load16_stream( rsrc, lane_offset + 2 * HALF_K, row_offset );
  }
}

__device__ __forceinline__ void stage_w_half( uint4* tile, const WSlab& s, int h )
{
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15, g4 = lane >> 4;
#pragma unroll
  for ( int j = 0; j < 8; j++ ) {
    const uint32_t row = 4 * j + g4;
    tile[row * 16 + ( c ^ ( row & 15 ) )] = s.v[h][j];
  }
}

// activations of one register slab: 64 columns x 256 k.  v[h][i], thread t: column t/16 + 16*i, chunk t%16 of half h
template<int W>
struct XSlab
{
  uint4 v[2][16 / W];
};

// `rsrc` starts at the work-group's first column; lane_offset = (t / 16) * row bytes + 16 * (t % 16)
template<int W>
__device__ __forceinline__ void load_x_half( XSlab<W>& dst, __amdgpu_buffer_rsrc_t rsrc, uint32_t lane_offset, uint32_t ld_bytes, uint32_t kb, int h )
{
#pragma unroll
  for ( int i = 0; i < 16 / W; i++ ) {
    dst.v[h][i] = buffer_load16( rsrc, lane_offset + h * 2 * HALF_K, 4 * W * i * ld_bytes + kb );
  }
}

template<int W>
__device__ __forceinline__ void stage_x_half( uint4* tile, const XSlab<W>& t, int h )
{
  const uint32_t chunk = threadIdx.x & 15;
#pragma unroll
  for ( int i = 0; i < 16 / W; i++ ) {
    const uint32_t col = ( threadIdx.x >> 4 ) + 4 * W * i;
    tile[col * 16 + ( chunk ^ ( col & 15 ) )] = t.v[h][i];
  }
}

// 128 k of math for a wave: 8 steps of k = 16
__device__ __forceinline__ void half_mfma( f32x16 acc[2], const uint4* wtile, const uint4* xtile )
{
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t r = lane & 31, g2 = lane >> 5;
#pragma unroll
  for ( int s = 0; s < 8; s++ ) {
    const uint32_t ch = 2 * s + g2;
    const f16x8 a = __builtin_bit_cast( f16x8, wtile[r * 16 + ( ch ^ ( r & 15 ) )] );
#pragma unroll
    for ( int t = 0; t < 2; t++ ) {
      const uint32_t col = 32 * t + r;
      const f16x8 b = __builtin_bit_cast( f16x8, xtile[col * 16 + ( ch ^ ( col & 15 ) )] );
      acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16( a, b, acc[t], 0, 0, 0 );
    }
  }
}

// what a work-group does with its accumulators
constexpr int MODE_PLAIN = 0; // round and store xout(b, r)
constexpr int MODE_SPLIT = 1; // fp32 partials of a K range
constexpr int MODE_GATE = 2;  // w = [w1 rows | w3 rows], r = rows of each: store DType(silu(DType(y1)) * DType(y3))

// grid: (row blocks x column slabs, 1, k splits).  s % 256 == 0, 16-byte aligned operands.
// MODE_GATE: a work-group takes 64 output rows; waves 0, 1 stream them from w1, waves 2, 3 the same
// rows from w3, so that the two factors of an output element sit in the same lane and accumulator
// register of a wave pair and meet through LDS after the K loop (no K split in this mode).
template<int MODE, int W = 4>
__global__ __launch_bounds__( 64 * W, W == 4 ? 2 : 1 ) void gemm_stream_kernel( __half* __restrict__ xout,
                                                             float* __restrict__ partial,
                                                             const __half* __restrict__ x,
                                                             const __half* __restrict__ w,
                                                             uint32_t s,
                                                             uint32_t r,
                                                             uint32_t b,
                                                             uint32_t k_per_split,
                                                             uint32_t n_col_slabs,
                                                             uint32_t rows_per_wave )
{
  __shared__ uint4 s_x[2][COLS * 16]; // 2 x 16 KiB
  __shared__ uint4 s_w[W][32 * 16];   // 8 KiB per wave

  const uint32_t wave = __builtin_amdgcn_readfirstlane( threadIdx.x >> 6 ); // provably uniform: keeps descriptors in SGPRs
  const uint32_t lane = threadIdx.x & 63;
  // Work-groups are handed to the 8 XCDs round robin by their linear index, and every XCD has its own
  // L2.  With more than one column slab, the slabs of one row block get indices 8 apart and adjacent
  // in time: they run on the same XCD together and the weights leave HBM once, not once per slab.
  uint32_t row_block = blockIdx.x, col_slab = 0;
  if ( n_col_slabs > 1 ) {
    const uint32_t idx = blockIdx.x >> 3;
    col_slab = idx % n_col_slabs;
    row_block = ( idx / n_col_slabs ) * 8 + ( blockIdx.x & 7 );
    if ( row_block * ( MODE == MODE_GATE ? W / 2 : W ) * rows_per_wave >= r ) {
      return; // padding of the grid to a multiple of 8 row blocks (whole work-group)
    }
  }
  // a wave owns rows_per_wave (<= 32, a multiple of 4) rows of its 32-row MFMA tile; the others read as zero and are not stored
  constexpr uint32_t HALF_W = W / 2;
  const uint32_t row0 = MODE == MODE_GATE ? ( row_block * HALF_W + ( wave % HALF_W ) ) * rows_per_wave : ( row_block * W + wave ) * rows_per_wave; // output row
  const uint32_t w_row0 = MODE == MODE_GATE ? ( wave / HALF_W ) * r + row0 : row0;
  const uint32_t col0 = col_slab * COLS;
  const uint32_t k_begin = blockIdx.z * k_per_split;
  const uint32_t k_end = min( s, k_begin + k_per_split );
  const uint32_t ld_bytes = s * 2;
  uint4* wtile = s_w[wave];

  // descriptors bounded to the wave's rows / the work-group's columns: anything past the matrix reads as zero
  const uint32_t w_rows = row0 < r ? min( rows_per_wave, r - row0 ) : 0u;
  const uint32_t x_cols = col0 < b ? min( (uint32_t)COLS, b - col0 ) : 0u;
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( w + (uint64_t)w_row0 * s ), 0, (int)( w_rows * ld_bytes ), 0x00020000 );
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( x + (uint64_t)col0 * s ), 0, (int)( x_cols * ld_bytes ), 0x00020000 );
  const uint32_t w_lane = ( lane >> 4 ) * ld_bytes + ( lane & 15 ) * 16;
  const uint32_t x_lane = ( threadIdx.x >> 4 ) * ld_bytes + ( threadIdx.x & 15 ) * 16;

  f32x16 acc[2];
#pragma unroll
  for ( int t = 0; t < 2; t++ ) {
#pragma unroll
    for ( int i = 0; i < 16; i++ ) {
      acc[t][i] = 0.0f;
    }
  }

  // Two weight register sets: while slab i is consumed out of one, slab i+1 is in flight into the
  // other.  Loads retire in order, so the issue order matters: the weight loads of slab i+1 go out
  // first in iteration i, the activation halves of slab i+1 follow as their registers are staged;
  // everything iteration i+1 waits for is then older than the weight loads it issues itself.
  //
  // The loop body has no conditional loads and no joins: the compiler counts outstanding loads per
  // path and, where paths with different counts meet, waits for the smaller count -- which here
  // would mean waiting for the slab that was just requested.  So the prologue issues in the same
  // order as an iteration leaves things (weights, then activations), the loads behind the last slab
  // are still issued but aimed past the descriptors' bounds (they return zero without touching
  // memory: the scalar offset is part of the range check on this hardware, which gh_init verifies),
  // and the loop is left by `break`.
  constexpr uint32_t PAST_THE_END = 0x80000000u; // + lane and row offsets (< 2^30) stays below 2^32 and above any descriptor's size
  const uint32_t n_slabs = ( k_end - k_begin ) / SLAB_K; // K ranges are multiples of SLAB_K
  uint32_t cur = ( ( row_block + blockIdx.z ) * 3u ) % n_slabs; // rotated start, see the header
  WSlab wr[2];
  XSlab<W> xr;
  {
    const uint32_t kb = ( k_begin + cur * SLAB_K ) * 2;
    load_w_slab( wr[0], w_rsrc, w_lane, ld_bytes, kb );
    load_x_half( xr, x_rsrc, x_lane, ld_bytes, kb, 0 );
    load_x_half( xr, x_rsrc, x_lane, ld_bytes, kb, 1 );
  }
  uint32_t j = 0;
  auto consume = [&]( auto set_tag ) {
    constexpr int set = decltype( set_tag )::value;
    cur = cur + 1 == n_slabs ? 0 : cur + 1;
    const uint32_t kb = j + 1 < n_slabs ? ( k_begin + cur * SLAB_K ) * 2 : PAST_THE_END;
    load_w_slab( wr[set ^ 1], w_rsrc, w_lane, ld_bytes, kb );
#pragma unroll
    for ( int h = 0; h < 2; h++ ) {
      stage_x_half( s_x[h], xr, h );
      stage_w_half( wtile, wr[set], h );
      load_x_half( xr, x_rsrc, x_lane, ld_bytes, kb, h ); // same registers, next slab
      __syncthreads();
      half_mfma( acc, wtile, s_x[h] );
    }
  };
  for ( ;; ) { // exits are uniform across the work-group
    consume( std::integral_constant<int, 0> {} );
    if ( ++j == n_slabs ) {
      break;
    }
    consume( std::integral_constant<int, 1> {} );
    if ( ++j == n_slabs ) {
      break;
    }
  }
  // acc[t][v]: row = 8*(v/4) + 4*(lane/32) + v%4 of the wave's 32, column = 32*t + lane%32
  const uint32_t g2 = lane >> 5;
  if ( MODE == MODE_GATE ) {
    // the waves on w3 hand DType(y3) to the waves on w1 through the activation tiles' LDS (W / 2 x 2 x 16 x 64 floats: 16 or 32 KiB)
    float* gate = reinterpret_cast<float*>( s_x[0] );
    __syncthreads(); // every wave is done reading the activation tiles
    if ( wave >= HALF_W ) {
#pragma unroll
      for ( int t = 0; t < 2; t++ ) {
#pragma unroll
        for ( int v = 0; v < 16; v++ ) {
          gate[( ( ( wave % HALF_W ) * 2 + t ) * 16 + v ) * 64 + lane] = __half2float( __float2half_rn( acc[t][v] ) );
        }
      }
    }
    __syncthreads();
    if ( wave >= HALF_W ) {
      return;
    }
#pragma unroll
    for ( int t = 0; t < 2; t++ ) {
      const uint32_t col = col0 + 32 * t + ( lane & 31 );
#pragma unroll
      for ( int q4 = 0; q4 < 4; q4++ ) {
        const uint32_t row = row0 + 8 * q4 + 4 * g2;
        union
        {
          uint2 raw;
          __half h[4];
        } o;
#pragma unroll
        for ( int i = 0; i < 4; i++ ) {
          const float y1 = __half2float( __float2half_rn( acc[t][4 * q4 + i] ) );
          const float y3 = gate[( ( wave * 2 + t ) * 16 + 4 * q4 + i ) * 64 + lane];
          o.h[i] = __float2half_rn( y1 / ( 1.0f + __expf( -y1 ) ) * y3 );
        }
        if ( col < b && 8 * q4 + 4 * g2 < rows_per_wave ) {
          __half* dst = xout + (uint64_t)col * r + row;
          if ( row + 3 < r ) {
            *reinterpret_cast<uint2*>( dst ) = o.raw;
          } else {
            for ( int i = 0; i < 4; i++ ) {
              if ( row + i < r ) {
                dst[i] = o.h[i];
              }
            }
          }
        }
      }
    }
    return;
  }
#pragma unroll
  for ( int t = 0; t < 2; t++ ) {
    const uint32_t col = col0 + 32 * t + ( lane & 31 );
    if ( col >= b ) {
      continue;
    }
#pragma unroll
    for ( int q4 = 0; q4 < 4; q4++ ) {
      const uint32_t row = row0 + 8 * q4 + 4 * g2;
      if ( 8 * q4 + 4 * g2 >= rows_per_wave ) {
        continue;
      }
      if ( MODE == MODE_SPLIT ) {
        float* dst = partial + ( (uint64_t)blockIdx.z * b + col ) * r + row;
        if ( row + 3 < r ) {
          *reinterpret_cast<float4*>( dst ) = make_float4( acc[t][4 * q4], acc[t][4 * q4 + 1], acc[t][4 * q4 + 2], acc[t][4 * q4 + 3] );
        } else {
          for ( int i = 0; i < 4; i++ ) {
            if ( row + i < r ) {
              dst[i] = acc[t][4 * q4 + i];
            }
          }
        }
      } else {
        __half* dst = xout + (uint64_t)col * r + row;
        if ( row + 3 < r ) {
          union
          {
            uint2 raw;
            __half h[4];
          } o;
#pragma unroll
          for ( int i = 0; i < 4; i++ ) {
            o.h[i] = __float2half_rn( acc[t][4 * q4 + i] );
          }
          *reinterpret_cast<uint2*>( dst ) = o.raw;
        } else {
          for ( int i = 0; i < 4; i++ ) {
            if ( row + i < r ) {
              dst[i] = __float2half_rn( acc[t][4 * q4 + i] );
            }
          }
        }
      }
    }
  }
}

int g_target_wgs = 0; // tuning override of the CU count the plan balances for (0: the device's)
int g_gate_waves = 0;  // tuning override of the waves per work-group of the one-launch gate product (0: by the rule in its launcher; 4, 8)

void launch( dim3 grid, hipStream_t st, bool split, __half* xout, float* partial, const __half* x, const __half* w, uint32_t s, uint32_t r, uint32_t b,
             uint32_t k_per_split, uint32_t n_col_slabs, uint32_t rows_per_wave )
{
  if ( split ) {
    gemm_stream_kernel<MODE_SPLIT><<<grid, 256, 0, st>>>( xout, partial, x, w, s, r, b, k_per_split, n_col_slabs, rows_per_wave );
  } else {
    gemm_stream_kernel<MODE_PLAIN><<<grid, 256, 0, st>>>( xout, partial, x, w, s, r, b, k_per_split, n_col_slabs, rows_per_wave );
  }
}

} // namespace

bool gemm_stream_applicable( uint64_t s, uint64_t r, uint64_t b, const void* x, const void* w, const void* xout )
{
  (void)b;
  return s % SLAB_K == 0 && s < ( 1u << 24 ) && r % 4 == 0 && ( ( reinterpret_cast<uintptr_t>( x ) | reinterpret_cast<uintptr_t>( w ) | reinterpret_cast<uintptr_t>( xout ) ) & 15u ) == 0;
}

// Picks the K split and the rows per work-group.
//
// What the choice has to get right (measured on the 70B shapes with cold weights, per-work-group
// time stamps): a CU pulls about 1/256 of the chip's bandwidth whatever runs on it, so a launch is
// as slow as its busiest CU (320 equal work-groups on 256 CUs: 48 us; the same bytes as 240: 38 us);
// a CU needs about 72 KiB of loads in flight to reach that rate, and a work-group keeps one
// register slab (rows x 512 bytes) in flight, so two small tiles or one full tile per CU;
// every split adds an fp32 partial tile per output element, written and read again; and a
// work-group's first slab arrives late.  The row tile only shrinks below 128 where there is no K
// split to balance the launch with (a wave keeps its 32-row MFMA tile and leaves rows unused).
void gemm_stream_plan( uint64_t s, uint64_t r, uint64_t b, uint32_t* splits_out, uint32_t* k_per_split_out, uint32_t* rows_per_wg_out )
{
  const uint64_t col_slabs = ( b + COLS - 1 ) / COLS;
  const double n_cu = (double)( g_target_wgs > 0 ? g_target_wgs : cu_count() );
  const uint64_t total_slabs = s / SLAB_K;
  double best_cost = 0.0;
  uint32_t best_rows = WG_ROWS, best_splits = 1, best_kps = (uint32_t)s;
  bool have = false;
  for ( uint32_t rows = WG_ROWS; rows >= 96; rows -= 16 ) {
    const uint64_t tiles = ( ( r + rows - 1 ) / rows ) * col_slabs;
    for ( uint32_t want = 1; want <= 16 && want <= total_slabs; want++ ) {
      const uint64_t kps = ( total_slabs + want - 1 ) / want * SLAB_K;
      const uint32_t splits = (uint32_t)( ( s + kps - 1 ) / kps );
      if ( splits != want || ( splits > 1 && ( kps < 2 * SLAB_K || rows != WG_ROWS ) ) ) {
        continue; // the same plan as a smaller `want`; too little K per work-group to pipeline; small tiles only without a split
      }
      const double slab_bytes = (double)rows * SLAB_K * 2.0;
      const double per_cu = std::ceil( (double)( tiles * splits ) / n_cu );
      const double busiest = per_cu * (double)rows * (double)kps * 2.0;
      const double rate = std::min( 1.0, std::min( per_cu, 2.0 ) * slab_bytes / ( 72.0 * 1024.0 ) );
      const double partials = splits > 1 ? 2.0 * splits * (double)b * (double)r * 4.0 / n_cu : 0.0;
      const double cost = busiest / rate + partials + per_cu * slab_bytes;
      if ( !have || cost < best_cost ) {
        have = true;
        best_cost = cost;
        best_rows = rows;
        best_splits = splits;
        best_kps = (uint32_t)kps;
      }
    }
  }
  *splits_out = best_splits;
  *k_per_split_out = best_kps;
  *rows_per_wg_out = best_rows;
}

int gemm_stream_launch( __half* xout, float* partial, const __half* x, const __half* w, uint64_t s, uint64_t r, uint64_t b, uint32_t splits,
                        uint32_t k_per_split, uint32_t rows_per_wg, bool write_partials, hipStream_t st )
{
  GH_REQUIRE( rows_per_wg % 16 == 0 && rows_per_wg >= 16 && rows_per_wg <= WG_ROWS, "gh_matmul: bad row tile %u", rows_per_wg );
  const uint64_t row_blocks = ( r + rows_per_wg - 1 ) / rows_per_wg;
  const uint64_t col_slabs = ( b + COLS - 1 ) / COLS;
  const uint64_t gx = col_slabs == 1 ? row_blocks : ( row_blocks + 7 ) / 8 * 8 * col_slabs;
  GH_REQUIRE( gx < ( 1ull << 31 ) && splits <= 65535, "gh_matmul: grid too large" );
  const dim3 grid( (unsigned)gx, 1, splits );
  launch( grid, st, write_partials, xout, partial, x, w, (uint32_t)s, (uint32_t)r, (uint32_t)b, k_per_split, (uint32_t)col_slabs, rows_per_wg / 4 );
  GH_LAUNCH_CHECK();
  return GH_OK;
}

// hb(b, hidden) = DType(silu(DType(x . w1^T)) * DType(x . w3^T)), w13 = w1 rows then w3 rows, in one launch.
// Only without a K split: the caller checks gemm_stream_gate_applicable first.
bool gemm_stream_gate_applicable( uint64_t s, uint64_t hidden, uint64_t b, const void* x, const void* w13, const void* hb )
{
  if ( hidden % 4 != 0 || !gemm_stream_applicable( s, 2 * hidden, b, x, w13, hb ) ) { // 8-byte output stores
    return false;
  }
  uint32_t splits = 1, k_per_split = 0, rows = 0;
  gemm_stream_plan( s, 2 * hidden, b, &splits, &k_per_split, &rows );
  return splits == 1;
}

int gemm_stream_gate_launch( __half* hb, const __half* x, const __half* w13, uint64_t s, uint64_t hidden, uint64_t b, hipStream_t st )
{
  uint32_t splits = 1, k_per_split = 0, rows = 0;
  gemm_stream_plan( s, 2 * hidden, b, &splits, &k_per_split, &rows );
  GH_REQUIRE( splits == 1, "gh_matmul_silu_gate: the one-launch form does not split K" );
  const uint32_t rows_per_wave = rows / 4; // half of the waves on w1, half on w3
  // Where work-groups of four waves come two to a CU, one of eight takes their place: the same waves on the same rows, but one
  // activation tile per slab for all eight instead of one per four.  The activations are a third of what a CU's L1 fetches with
  // four waves and a fifth with eight, and that L1 is what bounds the stream: 70B w1+w3 at 64 rows, cold weights, 162-167 -> 145-158 us.
  // (With a K split the work-groups would be too few, or the splits more: wo, wq+wkv and w2 gained nothing or lost.)
  const uint64_t blocks_of_four = ( hidden + 2 * rows_per_wave - 1 ) / ( 2 * rows_per_wave );
  const uint32_t waves = g_gate_waves != 0 ? (uint32_t)g_gate_waves : ( blocks_of_four >= 2ull * (uint64_t)cu_count() ? 8u : 4u );
  const uint64_t row_blocks = ( hidden + ( waves / 2 ) * rows_per_wave - 1 ) / ( ( waves / 2 ) * rows_per_wave );
  const uint64_t col_slabs = ( b + COLS - 1 ) / COLS;
  const uint64_t gx = col_slabs == 1 ? row_blocks : ( row_blocks + 7 ) / 8 * 8 * col_slabs;
  GH_REQUIRE( gx < ( 1ull << 31 ), "gh_matmul_silu_gate: grid too large" );
  if ( waves == 8 ) {
    gemm_stream_kernel<MODE_GATE, 8><<<dim3( (unsigned)gx, 1, 1 ), 512, 0, st>>>( hb, nullptr, x, w13, (uint32_t)s, (uint32_t)hidden, (uint32_t)b, (uint32_t)s,
                                                                              (uint32_t)col_slabs, rows_per_wave );
  } else {
    gemm_stream_kernel<MODE_GATE><<<dim3( (unsigned)gx, 1, 1 ), 256, 0, st>>>( hb, nullptr, x, w13, (uint32_t)s, (uint32_t)hidden, (uint32_t)b, (uint32_t)s,
                                                                           (uint32_t)col_slabs, rows_per_wave );
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

void gemm_stream_tuning( int target_wgs, int depth )
{
  if ( target_wgs > 0 ) {
    g_target_wgs = target_wgs;
  }
  (void)depth;
}

void gemm_stream_gate_waves( int waves ) { g_gate_waves = waves == 4 || waves == 8 ? waves : 0; }

} // namespace gh
