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

typedef _Float16 f16x2 __attribute__( ( ext_vector_type( 2 ) ) );
typedef _Float16 f16x4 __attribute__( ( ext_vector_type( 4 ) ) );
typedef _Float16 f16x8 __attribute__( ( ext_vector_type( 8 ) ) );
typedef float f32x4 __attribute__( ( ext_vector_type( 4 ) ) );
typedef float f32x16 __attribute__( ( ext_vector_type( 16 ) ) );
typedef __attribute__( ( address_space( 3 ) ) ) void* lds_ptr;
typedef __attribute__( ( address_space( 3 ) ) ) char lds_char;
typedef short v4s __attribute__( ( ext_vector_type( 4 ) ) );
typedef short v8s __attribute__( ( ext_vector_type( 8 ) ) );
typedef __attribute__( ( address_space( 3 ) ) ) v4s* lds_v4s;

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
// block = 4 waves; wave = NQT 32-column MFMA tiles (NQT = 1 by default: 128 query columns per block, two blocks per CU).  Per
// 64-key stage (K and V rows go from global memory straight into LDS, two buffers each, see the loop below):
//   S^T = K Q^T   v_mfma_f32_32x32x16_f16, A = K rows out of LDS (16-byte chunks, XOR-swizzled), B = Q^T in registers; every A
//                 fragment feeds all column tiles.  A lane ends up with 16 of the 32 keys of a sub-tile for ITS query column,
//                 the lane 32 further on with the other 16: maximum and sum stay inside a lane but for one exchange per stage
//   O^T += V^T P^T  the scores of a lane are, as they lie, the B operand (keys x its column) of the same instruction; the A
//                 operand V^T (one dim x 8 keys per lane) comes out of LDS with transposing reads (ds_read_b64_tr_b16).  Every
//                 accumulator of a lane belongs to its own column: rescaling needs no shuffle
// Causal mask only on stages that reach a wave's diagonal; stages beyond it are skipped.
// A wave's stage: softmax of the stage's scores (vector ALU), then 16 pairs of (one MFMA of O^T += V^T P^T, one MFMA of the NEXT
// stage's S^T), their LDS operands requested four pairs ahead and the second half of the exponentials computed beside the first pairs.
// (Two tiles per wave, NQT = 2, is kept for measurement: it does not fit the registers of two work-groups per CU and runs at half the rate.)
template<int G, int NQT>
__global__ __launch_bounds__( 256, NQT == 1 ? 2 : 1 ) void attn_prefill_mfma_kernel( const __half* __restrict__ q,
                                                                   const __half* const* __restrict__ layer_rows,
                                                                   const uint32_t* __restrict__ start_pos,
                                                                   __half* __restrict__ xb,
                                                                   uint32_t n_kv_heads,
                                                                   uint32_t n_tokens,
                                                                   uint32_t col_blocks, // ceil(n_tokens * G / (128 * NQT))
                                                                   uint32_t n_pairs,    // batch * n_kv_heads
                                                                   uint32_t paired,     // a work-group takes two column blocks (else one)
                                                                   float scale_log2e )
{
  // Two stages of 64 keys x 256 bytes for K (16-byte chunks XOR-swizzled by the key's low bits) and two for the same keys' value
  // rows.  Four separate arrays, and the loop below names the stage it works on at compile time: the compiler orders an LDS read
  // behind the outstanding loads-to-LDS (a wait for ALL of them, the ones just issued included) whenever it cannot tell that they
  // go to a different array.
  __shared__ uint4 s_k0[64 * 16], s_k1[64 * 16];
  __shared__ uint4 s_v0[64 * 16], s_v1[64 * 16];
  static_assert( 32 * NQT >= G, "a wave holds whole tokens" );
  constexpr uint32_t TPW = 32 * NQT / G; // tokens per wave

  const uint32_t wave = __builtin_amdgcn_readfirstlane( threadIdx.x >> 6 ); // provably uniform: what derives from it stays in scalar registers
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t r = lane & 31;
  const uint32_t g2 = lane >> 5;
  // block -> (two column blocks, kv head, context).  Work-groups go to the 8 XCDs in turn and every XCD has its own L2: all column
  // blocks of a (context, kv head) pair are given to one XCD, next to each other in time, so that the pair's K and V rows are
  // fetched into one L2 once instead of into all eight.  Column block c attends (c + 1) x 128 / G keys (plus the start position),
  // so a work-group takes column block col_blocks - 1 - j and then column block j: every work-group of a launch has the same
  // number of key stages, and no CU idles while another finishes a long column block.  (Not for small launches: `paired` = 0
  // keeps one column block per work-group, longest first, so that there are enough work-groups to go round.)
  const uint32_t xcd = blockIdx.x & 7;
  const uint32_t slot = blockIdx.x >> 3;
  const uint32_t half_blocks = paired ? ( col_blocks + 1 ) / 2 : col_blocks;
  const uint32_t cb_first = col_blocks - 1 - slot % half_blocks, cb_second = paired ? slot % half_blocks : cb_first;
  const uint32_t pair = ( slot / half_blocks ) * 8 + xcd;
  if ( pair >= n_pairs ) {
    return; // padding of the grid to a multiple of 8 pairs (whole work-group)
  }
  const uint32_t h = pair % n_kv_heads;
  const uint32_t ctx = pair / n_kv_heads;
  const __half* base = layer_rows[ctx];
  if ( base == nullptr ) {
    return; // the whole work-group
  }
  const uint32_t n_heads = n_kv_heads * G;
  const uint64_t row_elems = 2ull * n_kv_heads * HS;
  const uint32_t v_off = n_kv_heads * HS;
  const uint32_t start = start_pos[ctx];

  for ( uint32_t part = 0; part < 2; part++ ) {
  const uint32_t cb = part == 0 ? cb_first : cb_second;
  if ( part == 1 ) {
    if ( cb_second == cb_first ) {
      break; // odd number of column blocks: the middle one is alone
    }
    __syncthreads(); // every wave is done with the LDS stages of the first column block
  }
  const uint32_t wave_tok0 = ( cb * 4 + wave ) * TPW;          // first token of the wave
  const bool wave_ok = wave_tok0 < n_tokens;                    // a wave without queries still loads its share of every stage
  const uint32_t wave_last = min( n_tokens, wave_tok0 + TPW ) - 1;
  const uint32_t t_end = wave_ok ? start + wave_last + 1 : 0;   // keys [0, t_end) are visible to some column of the wave
  const uint32_t t_all = start + wave_tok0 + 1;                 // keys [0, t_all) are visible to every column of the wave
  const uint32_t wg_end = start + min( n_tokens, ( cb + 1 ) * 4 * TPW );

  // this lane's query column in each of the wave's tiles: token, head, last visible key
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

  f32x16 acc[NQT][4]; // [column tile][dim block i4]: element v <-> dim 32 i4 + 8*(v/4) + 4*g2 + v%4 of this lane's column
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

  // global -> LDS without passing through registers (`buffer_load ... lds`, 16 bytes per lane): lane l of a wave lands at the
  // wave's base + 16 l, i.e. an instruction fills 4 rows of 256 bytes; wave w fills rows 16 w + 4 j + l / 16, j = 0..3, of a stage.
  // The swizzle of the K tile is applied to the address a lane fetches: the chunk that belongs in its slot.  The descriptor
  // ends with the last key the work-group needs: rows past it read as zero whatever they hold (a weight of zero times a NaN
  // would be a NaN).
  const uint32_t row_bytes = (uint32_t)row_elems * 2;
  const __amdgpu_buffer_rsrc_t kv_rsrc = __builtin_amdgcn_make_buffer_rsrc( const_cast<__half*>( base + (uint64_t)h * HS ), 0, (int)( wg_end * row_bytes ), 0x00020000 );
  const uint32_t ld_g = lane >> 4, ld_pos = lane & 15;
  const uint32_t k_voff = ld_g * row_bytes + ( ( ld_pos ^ ld_g ) * 16 ); // row 4 j + ld_g keeps chunk (ld_pos ^ ld_g ^ 4 j) in slot ld_pos
  // V rows: the 16-byte chunks of a key's row are XORed with 4 x the key's low 2 bits, so that the transposing reads below (a
  // half-wave: 4 keys x 2 groups of 16 dims x 4 lanes x 8 bytes) touch 32 different 8-byte slots, i.e. every bank once: row
  // 4 j + ld_g keeps chunk ld_pos ^ 4 ld_g in slot ld_pos.  (With 2 x the low 3 bits instead, lanes of the two dim groups met in
  // the same banks at neighbouring keys: as many bank-conflict cycles as active LDS cycles.)
  const uint32_t v_voff = ld_g * row_bytes + ( ( ld_pos ^ ( 4 * ld_g ) ) * 16 ) + v_off * 2;
  auto fetch_k = [&]( uint4* kt, uint32_t stage ) {
#pragma unroll
    for ( int j = 0; j < 4; j++ ) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds( kv_rsrc, (lds_ptr)( kt + ( 16 * wave + 4 * j ) * 16 ), 16, k_voff ^ ( 64 * j ),
                                                ( 64 * stage + 16 * wave + 4 * j ) * row_bytes, 0, 0 );
    }
  };
  auto fetch_v = [&]( uint4* vt, uint32_t stage ) {
#pragma unroll
    for ( int j = 0; j < 4; j++ ) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds( kv_rsrc, (lds_ptr)( vt + ( 16 * wave + 4 * j ) * 16 ), 16, v_voff,
                                                ( 64 * stage + 16 * wave + 4 * j ) * row_bytes, 0, 0 );
    }
  };

  // transposing V reads: lane j = 4 e + q of a 16-lane group points at key slot e (0..3) of its half-wave, dims 16 grp + 4 q .. + 3
  // of dim block 0; the chunk index carries the V tile's swizzle (4 x the key's low 2 bits = 4 e), dim block i4 flips bits 2, 3 as well
  const uint32_t tr_e = ( lane & 15 ) >> 2, tr_q = lane & 3, tr_grp = ( lane >> 4 ) & 1;
  const uint32_t v_lane = ( 4 * g2 + tr_e ) * 256 + ( ( ( 2 * tr_grp + ( tr_q >> 1 ) ) ^ ( 4 * tr_e ) ) * 16 ) + ( tr_q & 1 ) * 8;

  // The two products of a stage run as 16 pairs of MFMA steps, pair n = (P-step n, S-step n):
  //   P-step n  O^T += V^T P^T for keys 16 kk .. 16 kk + 15 (kk = n / 4) and dims 32 i4 .. 32 i4 + 31 (i4 = n % 4).  The A operand (32 dims x
  //             16 keys; a lane: one dim, the 8 keys of its slots) comes out of LDS transposed: ds_read_b64_tr_b16 hands lane i of a
  //             16-lane group element i of each of four 32-byte rows that the group's lanes point at (lanes 4 e .. 4 e + 3 at row e),
  //             i.e. 4 keys of one dim per instruction.  The four dim blocks are independent accumulation chains.
  //   S-step n  S^T = K Q^T of the NEXT stage for keys 32 sub .. 32 sub + 31 (sub = n / 8) and dims 16 s .. 16 s + 15 (s = n % 8):
  //             st[qt][sub][v] = raw score of key 32 sub + 8*(v/4) + 4*g2 + v%4 of the stage for column tile qt.
  // Operands sit in rings of four register sets: the LDS read for step n + 4 is issued right behind step n, i.e. four pairs (some 250
  // cycles of matrix work) before its use; under this kernel's load an LDS read takes about 200 cycles to return, and with the reads one
  // step ahead both products ran at the pace of that latency.
  f16x8 ka[4];
  auto read_k = [&]( const uint4* kt, int n ) {
    const uint32_t krow = 32 * ( n >> 3 ) + r;
    ka[n & 3] = __builtin_bit_cast( f16x8, kt[krow * 16 + ( ( 2 * ( n & 7 ) + g2 ) ^ ( krow & 15 ) )] );
  };
  auto score_step = [&]( f32x16 ( &st )[NQT][2], int n ) {
#pragma unroll
    for ( int qt = 0; qt < NQT; qt++ ) {
      if ( ( n & 7 ) == 0 ) {
        const f32x16 zero = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
        st[qt][n >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16( ka[n & 3], qb[qt][n & 7], zero, 0, 0, 0 );
      } else {
        st[qt][n >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16( ka[n & 3], qb[qt][n & 7], st[qt][n >> 3], 0, 0, 0 );
      }
    }
  };
  v4s va[4][2];
  auto read_v = [&]( const uint4* vt, int n ) {
#pragma unroll
    for ( int half = 0; half < 2; half++ ) {
      va[n & 3][half]
        = __builtin_amdgcn_ds_read_tr16_b64_v4i16( (lds_v4s)( (lds_char*)vt + ( v_lane ^ ( 64 * ( n & 3 ) ) ) + ( 16 * ( n >> 2 ) + 8 * half ) * 256 ) );
    }
  };

  // Two LDS buffers each for K and V, one barrier per stage.  Behind the barrier of iteration i every wave is done with K of
  // stage i (its scores were computed in iteration i-1) and with V of stage i-1, so K of stage i+2 and V of stage i+1 are
  // requested into those buffers; the barrier of iteration i+1 waits for them.  The wave then turns the scores of stage i into
  // weights and, pair by pair, adds stage i's weighted values and computes the scores of stage i+1 (which do not depend on the
  // weights).
  const uint32_t n_stages = ( wg_end + 63 ) / 64;
  const uint32_t my_stages = ( t_end + 63 ) / 64; // stages that hold keys visible to this wave (it takes part in the loads and barriers of all)
  fetch_k( s_k0, 0 );
  fetch_k( s_k1, 1 );
  fetch_v( s_v0, 0 );
  __builtin_amdgcn_s_waitcnt( 0x0F70 ); // vmcnt(0)
  __syncthreads();
  f32x16 st_a[NQT][2], st_b[NQT][2]; // scores of even and of odd stages
  if ( my_stages > 0 ) {
#pragma unroll
    for ( int n = 0; n < 4; n++ ) {
      read_k( s_k0, n );
    }
#pragma unroll
    for ( int n = 0; n < 16; n++ ) {
      score_step( st_a, n );
      if ( n + 4 < 16 ) {
        read_k( s_k0, n + 4 );
      }
    }
  }

  // stage i with its K in k_cur and its V in v_cur, its scores in st; k_nxt, v_nxt, st_nxt: the other set
  auto stage = [&]( uint32_t i, uint4* k_cur, uint4* v_cur, uint4* k_nxt, uint4* v_nxt, f32x16 ( &st )[NQT][2], f32x16 ( &st_nxt )[NQT][2] ) {
    const uint32_t t0 = 64 * i;
    // Every load-to-LDS this wave has issued (K of stage i + 1, V of stage i) has landed before the wave enters the barrier, so
    // behind it all of them have.  Said explicitly: the barrier's own fence only orders LDS instructions, and the compiler's
    // tracking of loads-to-LDS against the reads of the distinct arrays is not relied upon.
    __builtin_amdgcn_s_waitcnt( 0x0F70 ); // vmcnt(0)
    __syncthreads();
    if ( i + 2 < n_stages ) {
      fetch_k( k_cur, i + 2 );
    }
    if ( i + 1 < n_stages ) {
      fetch_v( v_nxt, i + 1 );
    }
    if ( i >= my_stages ) {
      return; // wave-uniform
    }
    // the operands of the first four pairs are requested now: the softmax below gives them the time to arrive
#pragma unroll
    for ( int n = 0; n < 4; n++ ) {
      read_v( v_cur, n );
      read_k( k_nxt, n );
    }
    __builtin_amdgcn_sched_barrier( 0 );
    // a stage that reaches the wave's diagonal hides keys from some columns; before it every key is visible to every column
    if ( __builtin_amdgcn_readfirstlane( t0 + 64 > t_all ) ) {
      asm volatile( "" ::: "memory" ); // keeps this a branch: the selects are only paid for on the diagonal
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

    // ---- online softmax per column tile: the reference point first
    float ms[NQT];
#pragma unroll
    for ( int qt = 0; qt < NQT; qt++ ) {
      // four independent chains (one long chain of dependent maxima costs its latency sixteen times), then the other half of the
      // column's keys from the lane 32 further on: v_permlane32_swap exchanges the two half-waves in the vector ALU, without the
      // trip through LDS that a shuffle takes
      float m4[4];
#pragma unroll
      for ( int c = 0; c < 4; c++ ) {
        m4[c] = st[qt][c >> 1][8 * ( c & 1 )];
#pragma unroll
        for ( int e = 1; e < 8; e++ ) {
          m4[c] = fmaxf( m4[c], st[qt][c >> 1][8 * ( c & 1 ) + e] );
        }
      }
      float mx = fmaxf( fmaxf( m4[0], m4[1] ), fmaxf( m4[2], m4[3] ) );
      const auto halves = __builtin_amdgcn_permlane32_swap( __builtin_bit_cast( unsigned, mx ), __builtin_bit_cast( unsigned, mx ), false, false );
      mx = fmaxf( __builtin_bit_cast( float, halves[0] ), __builtin_bit_cast( float, halves[1] ) ) * scale_log2e; // log2 domain from here on
      // The reference point of the exponentials only moves when the maximum has grown by more than 2^LAZY since it was set:
      // weights stay below 2^LAZY (fine for fp32 sums and fp16 operands) and the 64 accumulators are rescaled rarely.  The
      // result does not depend on the reference point.  -inf: a column that has seen no key yet (padding, or hidden so far).
      if ( __builtin_amdgcn_ballot_w64( mx > m[qt] + LAZY ) != 0 ) {
        const float m_new = fmaxf( m[qt], mx );
        const float alpha = m_new == -INFINITY ? 1.0f : fast_exp2( m[qt] - m_new );
        m[qt] = m_new;
        l[qt] *= alpha;
#pragma unroll
        for ( int i4 = 0; i4 < 4; i4++ ) {
#pragma unroll
          for ( int v = 0; v < 16; v++ ) {
            acc[qt][i4][v] *= alpha;
          }
        }
      }
      ms[qt] = m[qt] == -INFINITY ? 0.0f : m[qt];
    }
    // weights of keys 16 kk .. 16 kk + 15 of the stage, packed as the B operand of their P-steps:
    // pk[qt][kk] = keys 32 (kk / 2) + 16 (kk % 2) + 8 (e / 4) + 4 g2 + e % 4, e = 0..7.  Elements e0, e0 + 1 at a time, so that the
    // exponentials of 16 keys can be spread over four pairs.
    f16x8 pk[NQT][4];
    float p[NQT][8];
    f16x2 pk2[NQT][4];
    float sum[NQT][2];
#pragma unroll
    for ( int qt = 0; qt < NQT; qt++ ) {
      sum[qt][0] = sum[qt][1] = 0.0f;
    }
    auto weights = [&]( int kk, int e0 ) {
#pragma unroll
      for ( int qt = 0; qt < NQT; qt++ ) {
#pragma unroll
        for ( int e = e0; e < e0 + 2; e++ ) {
          p[qt][e] = fast_exp2( st[qt][kk >> 1][8 * ( kk & 1 ) + e] * scale_log2e - ms[qt] );
        }
        // the running sum takes the weights as the product will see them (rounded to half), two per instruction
        const f16x2 p2 = { (_Float16)p[qt][e0], (_Float16)p[qt][e0 + 1] };
        sum[qt][( e0 >> 1 ) & 1] = __builtin_amdgcn_fdot2( p2, f16x2 { (_Float16)1.0f, (_Float16)1.0f }, sum[qt][( e0 >> 1 ) & 1], false );
        pk2[qt][e0 >> 1] = p2;
        if ( e0 == 6 ) {
          pk[qt][kk] = f16x8 { pk2[qt][0][0], pk2[qt][0][1], pk2[qt][1][0], pk2[qt][1][1], pk2[qt][2][0], pk2[qt][2][1], pk2[qt][3][0], pk2[qt][3][1] };
        }
      }
    };
    // The weights of the first 32 keys before the pairs (their scores' registers are then free for the next stage's), those of the
    // other 32 beside the MFMAs of pairs 0..7.
#pragma unroll
    for ( int kk = 0; kk < 2; kk++ ) {
#pragma unroll
      for ( int e0 = 0; e0 < 8; e0 += 2 ) {
        weights( kk, e0 );
      }
    }
    __builtin_amdgcn_sched_barrier( 0 );
#pragma unroll
    for ( int n = 0; n < 16; n++ ) {
      const int kk = n >> 2, i4 = n & 3;
      {
        const v4s lo = va[n & 3][0], hi = va[n & 3][1];
        const v8s a8 = v8s { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
        const f16x8 a = __builtin_bit_cast( f16x8, a8 );
#pragma unroll
        for ( int qt = 0; qt < NQT; qt++ ) {
          acc[qt][i4] = __builtin_amdgcn_mfma_f32_32x32x16_f16( a, pk[qt][kk], acc[qt][i4], 0, 0, 0 );
        }
      }
      // The next stage's scores are also computed behind the wave's last stage, where nothing uses them (one stage's worth of
      // S-steps per column block): a branch around every S-step cuts the sequence into pieces that the register allocator handles
      // badly (89 spilled registers), and so do two copies of the whole stage, with and without them (224).
      score_step( st_nxt, n );
      if ( n + 4 < 16 ) {
        read_v( v_cur, n + 4 );
        read_k( k_nxt, n + 4 );
      }
      if ( n < 8 ) {
        weights( 2 + kk, 2 * i4 ); // vector ALU work beside the MFMAs of this pair
      }
      __builtin_amdgcn_sched_barrier( 0 );
    }
#pragma unroll
    for ( int qt = 0; qt < NQT; qt++ ) {
      l[qt] += sum[qt][0] + sum[qt][1];
    }
  };
  for ( uint32_t i = 0; i < n_stages; i += 2 ) {
    stage( i, s_k0, s_v0, s_k1, s_v1, st_a, st_b );
    if ( i + 1 < n_stages ) {
      stage( i + 1, s_k1, s_v1, s_k0, s_v0, st_b, st_a );
    }
  }

  // ---- normalise and store: element v of acc[qt][i4] is dim 32 i4 + 8 (v / 4) + 4 g2 + v % 4 of the lane's column
#pragma unroll
  for ( int qt = 0; qt < NQT; qt++ ) {
    const float lsum = l[qt] + __shfl_xor( l[qt], 32, WAVE );
    if ( qpos[qt] < 0 ) {
      continue; // padding column
    }
    const float inv = 1.0f / lsum;
    __half* out = xb + ( ( (uint64_t)ctx * n_tokens + tq[qt] ) * n_heads + (uint64_t)h * G + gq[qt] ) * HS;
#pragma unroll
    for ( int i4 = 0; i4 < 4; i4++ ) {
#pragma unroll
      for ( int a = 0; a < 4; a++ ) {
        union
        {
          uint2 raw;
          __half hv[4];
        } o;
#pragma unroll
        for ( int e = 0; e < 4; e++ ) {
          o.hv[e] = __float2half_rn( acc[qt][i4][4 * a + e] * inv );
        }
        *reinterpret_cast<uint2*>( out + 32 * i4 + 8 * a + 4 * g2 ) = o.raw;
      }
    }
  }
  } // the work-group's two column blocks
}

template<int G, int NQT>
void launch_prefill_tiles( hipStream_t st, const void* q, const void* const* rows, const uint32_t* start, void* xb, uint64_t batch, uint32_t n_tokens,
                           const gh_shape* s )
{
  const uint32_t col_blocks = (uint32_t)( ( (uint64_t)n_tokens * G + 128 * NQT - 1 ) / ( 128 * NQT ) );
  const uint64_t n_pairs = batch * s->n_kv_heads;
  // two column blocks per work-group (equal work for all) when that still leaves at least four work-groups for each of the two
  // places a CU has; a small launch keeps one column block per work-group
  const uint64_t padded_pairs = ( n_pairs + 7 ) / 8 * 8;
  const uint32_t paired = padded_pairs * ( ( col_blocks + 1 ) / 2 ) >= 8ull * (uint64_t)cu_count() ? 1 : 0;
  const uint64_t blocks = padded_pairs * ( paired ? ( col_blocks + 1 ) / 2 : col_blocks );
  attn_prefill_mfma_kernel<G, NQT><<<(unsigned)blocks, 256, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( rows ), start,
                                                                     static_cast<__half*>( xb ), s->n_kv_heads, n_tokens, col_blocks, (uint32_t)n_pairs, paired,
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
