// Fused decode attention for one layer of a batch of contexts: scores, softmax and the weighted
// sum over the cached rows in one pass, split over the key range (split-K) with an online
// softmax; a second small kernel merges the per-split partials.  Replaces the reference's
// attention_0_gemm + attention_softmax + attention_2_gemm sequence (models/llama2/model.hh:354-387)
// and needs no (batch, n_heads, seq_len) score buffer.
//
// Cache layout (fixed by the reference, models/llama2/context.hh:61-133): a layer of a context is
// seq_len rows of [K(kv_dim) | V(kv_dim)], token-major.  For kv head h the K head is head_size
// contiguous elements at row + h*head_size, the V head at row + kv_dim + h*head_size.
//
// Three kernels produce the same partial format:
//   generic  any head_size <= 256, any gqa, f16/f32 storage; one wave per (context, query head, split)
//   valu     f16, head_size 128: one wave per (context, kv head, split); 16 lanes share a token's
//            256-byte head row (one 16-byte load per lane), dot products with v_dot2_f32_f16,
//            16-lane DPP reductions, four independent online-softmax streams per wave
//   mfma     f16, head_size 128, 2 <= gqa <= 16: same wave decomposition, but the gqa query heads
//            are a 16-wide MFMA tile: S^T = K Q^T with v_mfma_f32_16x16x32_f16 (K staged through LDS
//            into operand order), O += P V with v_mfma_f32_16x16x16_f16 (V transposed in registers)
//
// Scores are kept in the log2 domain: s2 = (q . k) * scale * log2(e), weights are exp2(s2 - m).
// Partial format per (context, query head, split): out[head_size] floats (un-normalised), then m and l.
#include "gh_common.h"
#include "gh_attn_tiles.h"

#include <algorithm>

namespace gh {
namespace {

constexpr float LOG2E = 1.4426950408889634f;

// Split-K partials of gh_attn_decode_static: one array per GPU the library runs on, held until the
// process ends.  Host code never uses the array's name as an address: the device address is looked
// up once per device at initialisation (attn_static_scratch_init) and kept in g_static_scratch.
constexpr uint64_t STATIC_SCRATCH_BYTES = 16ull << 20;
constexpr int MAX_DEVICES = 16;
static __device__ __align__( 256 ) float scratch[STATIC_SCRATCH_BYTES / sizeof( float )];
float* g_static_scratch[MAX_DEVICES] = {};

uint32_t g_chunk_override = 0;
int g_split_join = 1; // 1: plans of 2 or 4 splits run on the kernels that add the splits up inside the work-group; 4, 8: with that many waves; 0: never
int g_auto_variant = GH_ATTN_AUTO; // what GH_ATTN_AUTO resolves to when the shape allows it (gh_attn_set_auto_variant)

struct Partials
{
  float* out; // [batch][n_heads][max_splits][head_size]
  float* ml;  // [batch][n_heads][max_splits][2]
};

// =================================================================================================
// generic kernel
// =================================================================================================
template<typename T>
__global__ __launch_bounds__( 64 ) void attn_decode_generic_kernel( const T* __restrict__ q,
                                                                    const T* const* __restrict__ layer_rows,
                                                                    const uint32_t* __restrict__ pos,
                                                                    Partials part,
                                                                    T* __restrict__ xb,
                                                                    uint32_t n_kv_heads,
                                                                    uint32_t gqa,
                                                                    uint32_t head_size,
                                                                    uint32_t chunk,
                                                                    uint32_t max_splits,
                                                                    float scale_log2e )
{
  const uint32_t head = blockIdx.x;
  const uint32_t split = blockIdx.y;
  const uint32_t ctx = blockIdx.z;
  const T* base = layer_rows[ctx];
  if ( base == nullptr ) {
    return;
  }
  const uint32_t n_tok = min( pos[ctx] + 1, max_splits * chunk ); // never beyond what the host sized the grid and the partials for
  const uint32_t t_begin = split * chunk;
  if ( t_begin >= n_tok ) {
    return;
  }
  const uint32_t t_end = min( n_tok, t_begin + chunk );
  const uint32_t n_heads = n_kv_heads * gqa;
  const uint32_t h = head / gqa;
  const uint32_t lane = threadIdx.x;
  const uint64_t row_elems = 2ull * n_kv_heads * head_size;

  float qd[4], acc[4];
  const T* qh = q + ( (uint64_t)ctx * n_heads + head ) * head_size;
#pragma unroll
  for ( int k = 0; k < 4; k++ ) {
    const uint32_t d = lane + 64 * k;
    qd[k] = d < head_size ? to_f32( qh[d] ) : 0.0f;
    acc[k] = 0.0f;
  }
  float m = -INFINITY, l = 0.0f;
  const T* kbase = base + (uint64_t)h * head_size;
  const T* vbase = kbase + (uint64_t)n_kv_heads * head_size;

  for ( uint32_t t = t_begin; t < t_end; t++ ) {
    const T* kr = kbase + (uint64_t)t * row_elems;
    const T* vr = vbase + (uint64_t)t * row_elems;
    float partial = 0.0f;
    float vd[4];
#pragma unroll
    for ( int k = 0; k < 4; k++ ) {
      const uint32_t d = lane + 64 * k;
      if ( d < head_size ) {
        partial += to_f32( kr[d] ) * qd[k];
        vd[k] = to_f32( vr[d] );
      } else {
        vd[k] = 0.0f;
      }
    }
    const float s = wave_sum( partial ) * scale_log2e;
    const float m_new = fmaxf( m, s );
    const float alpha = fast_exp2( m - m_new );
    const float p = fast_exp2( s - m_new );
    l = l * alpha + p;
#pragma unroll
    for ( int k = 0; k < 4; k++ ) {
      acc[k] = acc[k] * alpha + p * vd[k];
    }
    m = m_new;
  }

  if ( max_splits == 1 ) {
    const float inv = 1.0f / l;
    T* o = xb + ( (uint64_t)ctx * n_heads + head ) * head_size;
#pragma unroll
    for ( int k = 0; k < 4; k++ ) {
      const uint32_t d = lane + 64 * k;
      if ( d < head_size ) {
        o[d] = from_f32<T>( acc[k] * inv );
      }
    }
  } else {
    const uint64_t slot = ( (uint64_t)ctx * n_heads + head ) * max_splits + split;
    float* o = part.out + slot * head_size;
#pragma unroll
    for ( int k = 0; k < 4; k++ ) {
      const uint32_t d = lane + 64 * k;
      if ( d < head_size ) {
        o[d] = acc[k];
      }
    }
    if ( lane == 0 ) {
      part.ml[slot * 2] = m;
      part.ml[slot * 2 + 1] = l;
    }
  }
}

// =================================================================================================
// merge of the split partials: block <-> (query head, context), thread <-> output dim
// =================================================================================================
template<typename T>
__global__ __launch_bounds__( 256 ) void attn_merge_kernel( Partials part,
                                                            const void* const* __restrict__ layer_rows,
                                                            const uint32_t* __restrict__ pos,
                                                            T* __restrict__ xb,
                                                            uint32_t n_heads,
                                                            uint32_t head_size,
                                                            uint32_t chunk,
                                                            uint32_t max_splits )
{
  const uint32_t head = blockIdx.x;
  const uint32_t ctx = blockIdx.y;
  const void* const rows = layer_rows[ctx];
  const uint32_t last = pos[ctx]; // read before the branch on `rows`: one round trip for the two
  if ( rows == nullptr ) {
    return;
  }
  // ceil((pos + 1) / chunk); a position beyond the host's bound must not walk into the partials of the next head
  const uint32_t n_splits = min( ( last + chunk ) / chunk, max_splits );
  const uint64_t slot0 = ( (uint64_t)ctx * n_heads + head ) * max_splits;
  const float2* ml = reinterpret_cast<const float2*>( part.ml ) + slot0; // (maximum, sum) of a split
  // The first MERGE_BATCH splits, nearly always all of them: every load issued before the first use (a split past the last reads
  // the last again and gets weight zero), so the kernel is one memory round trip deep.  Splits beyond that, one at a time.
  constexpr uint32_t MERGE_BATCH = 8;
  for ( uint32_t d0 = 0; d0 < head_size; d0 += blockDim.x ) {
    const uint32_t d = d0 + threadIdx.x;
    const uint32_t dl = min( d, head_size - 1 );
    float2 st[MERGE_BATCH];
    float o[MERGE_BATCH];
#pragma unroll
    for ( uint32_t u = 0; u < MERGE_BATCH; u++ ) {
      const uint32_t sp = min( u, n_splits - 1 );
      st[u] = ml[sp];
      o[u] = part.out[( slot0 + sp ) * head_size + dl];
    }
    float m = -INFINITY;
#pragma unroll
    for ( uint32_t u = 0; u < MERGE_BATCH; u++ ) {
      m = fmaxf( m, st[u].x ); // a repeated split repeats a value that is in the set already
    }
    for ( uint32_t sp = MERGE_BATCH; sp < n_splits; sp++ ) {
      m = fmaxf( m, ml[sp].x );
    }
    float l = 0.0f, acc = 0.0f;
#pragma unroll
    for ( uint32_t u = 0; u < MERGE_BATCH; u++ ) {
      const float wgt = u < n_splits ? fast_exp2( st[u].x - m ) : 0.0f;
      l += st[u].y * wgt;
      acc += o[u] * wgt;
    }
    for ( uint32_t sp = MERGE_BATCH; sp < n_splits; sp++ ) {
      const float2 e = ml[sp];
      const float wgt = fast_exp2( e.x - m );
      l += e.y * wgt;
      acc += part.out[( slot0 + sp ) * head_size + dl] * wgt;
    }
    if ( d < head_size ) {
      xb[( (uint64_t)ctx * n_heads + head ) * head_size + d] = from_f32<T>( acc * ( 1.0f / l ) );
    }
  }
}

// =================================================================================================
// joined splits: the splits of a (context, kv head) stream are the waves of ONE work-group, which adds them up itself
//
// With up to four splits per stream a work-group of four waves holds whole streams: wave = (stream of the work-group, split).
// Every wave walks its token range as in the kernels above; then the waves leave their maxima, sums and accumulators in LDS, lane
// for lane as they lie in the registers, and the wave of split 0 combines them in the order and with the arithmetic of
// attn_merge_kernel (the output differs from that route's by at most one rounding: the compiler contracts the two differently) and stores the rounded result.  No partial sums in memory, no second
// launch.
// =================================================================================================
struct JoinedJob
{
  const __half* base;
  uint32_t ctx, h, split, t_begin, t_end;
  uint32_t slot;     // which of the work-group's streams
  uint32_t n_splits; // splits of this context that hold keys (0: nothing to do for the stream)
  bool active;       // this wave has keys to walk
};

// splits = 2 or 4; a work-group is JOIN_WAVES (4 or 8) waves = (JOIN_WAVES / splits neighbouring kv heads) x splits, so that its waves
// read pieces of the same cache rows that lie next to each other (with four waves on one head's four ranges a CU fetched 256-byte
// pieces and the launch took 168-171 instead of 166 us at 64 contexts of 4096 keys).  Work-group b: head group b % n_groups,
// context b / n_groups.
template<uint32_t JOIN_WAVES>
__device__ __forceinline__ JoinedJob joined_job( const __half* const* layer_rows, const uint32_t* pos, uint32_t n_kv_heads, uint32_t batch,
                                                 uint32_t chunk, uint32_t splits, uint32_t seq_len )
{
  JoinedJob j;
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t heads_per_group = JOIN_WAVES / splits;
  const uint32_t n_groups = ( n_kv_heads + heads_per_group - 1 ) / heads_per_group;
  j.split = wave % splits;
  j.slot = wave / splits;
  const uint32_t ctx = blockIdx.x / n_groups;
  const uint32_t h = ( blockIdx.x % n_groups ) * heads_per_group + j.slot;
  const bool exists = ctx < batch && h < n_kv_heads;
  j.ctx = exists ? ctx : 0;
  j.h = exists ? h : 0;
  j.base = exists ? layer_rows[j.ctx] : nullptr;
  const uint32_t n_tok = j.base != nullptr ? min( min( pos[j.ctx] + 1, splits * chunk ), seq_len ) : 0;
  j.n_splits = ( n_tok + chunk - 1 ) / chunk;
  j.t_begin = j.split * chunk;
  j.t_end = min( n_tok, j.t_begin + chunk );
  j.active = j.t_begin < n_tok;
  return j;
}

// =================================================================================================
// valu kernel: lane = (r = lane / 16: token within a group of 4, c = lane % 16: 16-byte chunk of the head row)
// =================================================================================================
// One (context, kv head) stream over the tokens [t_begin, t_end), t_begin < t_end, for the G query heads of the kv head: running
// maxima m (log2 domain), sums l and the unnormalised output acc[g][e] = O[head g][dim 8*c + e], the same in the four lanes
// that share a chunk c.  `rot` moves the tile the walk starts at.
template<int G>
__device__ __forceinline__ void valu_stream_range( const __half* __restrict__ q,
                                                   const __half* base,
                                                   const uint32_t ctx,
                                                   const uint32_t h,
                                                   const uint32_t t_begin,
                                                   const uint32_t t_end,
                                                   const uint32_t rot,
                                                   const uint32_t n_kv_heads,
                                                   const float scale_log2e,
                                                   float ( &m )[G],
                                                   float ( &l )[G],
                                                   float ( &acc )[G][8] )
{
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t r = lane >> 4;
  const uint32_t n_heads = n_kv_heads * G;
  const uint64_t row_elems = 2ull * n_kv_heads * HS;
  const uint32_t v_off = n_kv_heads * HS;

  uint4 qr[G];
  {
    const __half* qp = q + ( (uint64_t)ctx * n_heads + (uint64_t)h * G ) * HS + 8 * c;
#pragma unroll
    for ( int g = 0; g < G; g++ ) {
      qr[g] = load16( qp + g * HS );
    }
  }

#pragma unroll
  for ( int g = 0; g < G; g++ ) {
    m[g] = -INFINITY;
    l[g] = 0.0f;
#pragma unroll
    for ( int e = 0; e < 8; e++ ) {
      acc[g][e] = 0.0f;
    }
  }

  const __half* kp = base + (uint64_t)h * HS + 8 * c;
  const uint4 zero4 = make_uint4( 0, 0, 0, 0 );

  // 16-token tiles in rotated order, a different starting tile per block (see the mfma kernel)
  const uint32_t n_tiles = ( t_end - t_begin + 15 ) / 16;
  uint32_t tile_i = ( ( ctx * 5u + rot * 3u ) * 7u ) % n_tiles;
  uint32_t t0 = t_begin + 16 * tile_i;

  uint4 kn[4], vn[4]; // prefetched block
#pragma unroll
  for ( int j = 0; j < 4; j++ ) {
    const uint32_t tok = t0 + 4 * j + r;
    const bool ok = tok < t_end;
    const __half* row = kp + (uint64_t)tok * row_elems;
    kn[j] = ok ? load16_stream( row ) : zero4;
    vn[j] = ok ? load16_stream( row + v_off ) : zero4;
  }

  for ( uint32_t it = 0; it < n_tiles; it++ ) {
    tile_i = tile_i + 1 == n_tiles ? 0 : tile_i + 1;
    const uint32_t t_next = t_begin + 16 * tile_i;
    const bool more = it + 1 < n_tiles;
    uint4 kc[4], vc[4];
#pragma unroll
    for ( int j = 0; j < 4; j++ ) {
      kc[j] = kn[j];
      vc[j] = vn[j];
    }
    // prefetch the next 16 tokens while this block is processed
#pragma unroll
    for ( int j = 0; j < 4; j++ ) {
      const uint32_t tok = t_next + 4 * j + r;
      const bool ok = more && tok < t_end;
      const __half* row = kp + (uint64_t)tok * row_elems;
      kn[j] = ok ? load16_stream( row ) : zero4;
      vn[j] = ok ? load16_stream( row + v_off ) : zero4;
    }

    float s[4][G];
#pragma unroll
    for ( int j = 0; j < 4; j++ ) {
      const bool ok = t0 + 4 * j + r < t_end;
#pragma unroll
      for ( int g = 0; g < G; g++ ) {
        const float d = row16_sum( dot8( kc[j], qr[g], 0.0f ) );
        s[j][g] = ok ? d * scale_log2e : -INFINITY;
      }
    }

#pragma unroll
    for ( int g = 0; g < G; g++ ) {
      float m_new = fmaxf( fmaxf( s[0][g], s[1][g] ), fmaxf( s[2][g], s[3][g] ) );
      m_new = fmaxf( m_new, m[g] );
      const float m_safe = m_new == -INFINITY ? 0.0f : m_new; // a row that has seen no token yet
      const float alpha = fast_exp2( m[g] - m_safe );
      float p[4];
#pragma unroll
      for ( int j = 0; j < 4; j++ ) {
        p[j] = fast_exp2( s[j][g] - m_safe );
      }
      l[g] = l[g] * alpha + ( p[0] + p[1] ) + ( p[2] + p[3] );
      m[g] = m_new;
#pragma unroll
      for ( int e = 0; e < 8; e++ ) {
        acc[g][e] *= alpha;
      }
#pragma unroll
      for ( int j = 0; j < 4; j++ ) {
        float v[8];
        unpack8( vc[j], v );
#pragma unroll
        for ( int e = 0; e < 8; e++ ) {
          acc[g][e] += p[j] * v[e];
        }
      }
    }
    t0 = t_next;
  }

  // merge the four token streams (lane rows) of the wave
#pragma unroll
  for ( int g = 0; g < G; g++ ) {
    float mm = fmaxf( m[g], __shfl_xor( m[g], 16, WAVE ) );
    mm = fmaxf( mm, __shfl_xor( mm, 32, WAVE ) );
    const float f = m[g] == -INFINITY ? 0.0f : fast_exp2( m[g] - mm );
    float ll = l[g] * f;
    ll += __shfl_xor( ll, 16, WAVE );
    ll += __shfl_xor( ll, 32, WAVE );
#pragma unroll
    for ( int e = 0; e < 8; e++ ) {
      float a = acc[g][e] * f;
      a += __shfl_xor( a, 16, WAVE );
      a += __shfl_xor( a, 32, WAVE );
      acc[g][e] = a;
    }
    m[g] = mm;
    l[g] = ll;
  }

}

template<int G>
__global__ __launch_bounds__( 256 ) void attn_decode_valu_kernel( const __half* __restrict__ q,
                                                                  const __half* const* __restrict__ layer_rows,
                                                                  const uint32_t* __restrict__ pos,
                                                                  Partials part,
                                                                  __half* __restrict__ xb,
                                                                  uint32_t n_kv_heads,
                                                                  uint32_t chunk,
                                                                  uint32_t max_splits,
                                                                  uint32_t seq_len,
                                                                  float scale_log2e )
{
  const WaveJob job = wave_job( layer_rows, pos, n_kv_heads, chunk, max_splits, seq_len );
  if ( !job.valid ) {
    return; // wave-uniform; the kernel has no block-level barrier
  }
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t r = lane >> 4;
  const uint32_t n_heads = n_kv_heads * G;

  float m[G], l[G], acc[G][8];
  valu_stream_range<G>( q, job.base, job.ctx, job.h, job.t_begin, job.t_end, job.split, n_kv_heads, scale_log2e, m, l, acc );

  if ( r == 0 ) {
#pragma unroll
    for ( int g = 0; g < G; g++ ) {
      const uint64_t head = (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G + g;
      if ( max_splits == 1 ) {
        const float inv = 1.0f / l[g];
        union
        {
          uint4 raw;
          __half h[8];
        } o;
#pragma unroll
        for ( int e = 0; e < 8; e++ ) {
          o.h[e] = __float2half_rn( acc[g][e] * inv );
        }
        *reinterpret_cast<uint4*>( xb + head * HS + 8 * c ) = o.raw;
      } else {
        const uint64_t slot = head * max_splits + job.split;
        float4* o = reinterpret_cast<float4*>( part.out + slot * HS + 8 * c );
        o[0] = make_float4( acc[g][0], acc[g][1], acc[g][2], acc[g][3] );
        o[1] = make_float4( acc[g][4], acc[g][5], acc[g][6], acc[g][7] );
        if ( c == 0 ) {
          part.ml[slot * 2] = m[g];
          part.ml[slot * 2 + 1] = l[g];
        }
      }
    }
  }
}

// the valu kernel with the splits of a stream joined inside the work-group (see joined_job)
template<int G, uint32_t JOIN_WAVES>
__global__ __launch_bounds__( 64 * JOIN_WAVES ) void attn_decode_valu_joined_kernel( const __half* __restrict__ q,
                                                                         const __half* const* __restrict__ layer_rows,
                                                                         const uint32_t* __restrict__ pos,
                                                                         __half* __restrict__ xb,
                                                                         uint32_t n_kv_heads,
                                                                         uint32_t batch,
                                                                         uint32_t chunk,
                                                                         uint32_t splits,
                                                                         uint32_t seq_len,
                                                                         float scale_log2e )
{
  // per wave: what the 16 lanes of token row 0 hold -- 8 accumulators, the maximum and the sum of each of the G heads
  __shared__ float s_join[JOIN_WAVES][10 * G][16];
  const JoinedJob job = joined_job<JOIN_WAVES>( layer_rows, pos, n_kv_heads, batch, chunk, splits, seq_len );
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t r = lane >> 4;
  const uint32_t n_heads = n_kv_heads * G;

  float m[G], l[G], acc[G][8];
  if ( job.active ) {
    valu_stream_range<G>( q, job.base, job.ctx, job.h, job.t_begin, job.t_end, job.split, n_kv_heads, scale_log2e, m, l, acc );
    if ( job.split != 0 && r == 0 ) {
#pragma unroll
      for ( int g = 0; g < G; g++ ) {
#pragma unroll
        for ( int e = 0; e < 8; e++ ) {
          s_join[wave][10 * g + e][c] = acc[g][e];
        }
        s_join[wave][10 * g + 8][c] = m[g];
        s_join[wave][10 * g + 9][c] = l[g];
      }
    }
  }
  __syncthreads(); // reached by every wave of the work-group, with or without keys
  if ( job.split != 0 || !job.active || r != 0 ) {
    return; // split 0 holds keys whenever any split of the stream does
  }
#pragma unroll
  for ( int g = 0; g < G; g++ ) {
    float mm = m[g];
    for ( uint32_t u = 1; u < job.n_splits; u++ ) {
      mm = fmaxf( mm, s_join[wave + u][10 * g + 8][c] );
    }
    const float w0 = fast_exp2( m[g] - mm );
    float lsum = l[g] * w0;
    float out[8];
#pragma unroll
    for ( int e = 0; e < 8; e++ ) {
      out[e] = acc[g][e] * w0;
    }
    for ( uint32_t u = 1; u < job.n_splits; u++ ) {
      const float wu = fast_exp2( s_join[wave + u][10 * g + 8][c] - mm );
      lsum = __builtin_fmaf( s_join[wave + u][10 * g + 9][c], wu, lsum );
#pragma unroll
      for ( int e = 0; e < 8; e++ ) {
        out[e] = __builtin_fmaf( s_join[wave + u][10 * g + e][c], wu, out[e] );
      }
    }
    const float inv = 1.0f / lsum;
    union
    {
      uint4 raw;
      __half h[8];
    } o;
#pragma unroll
    for ( int e = 0; e < 8; e++ ) {
      o.h[e] = __float2half_rn( out[e] * inv );
    }
    const uint64_t head = (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G + g;
    *reinterpret_cast<uint4*>( xb + head * HS + 8 * c ) = o.raw;
  }
}

// =================================================================================================
// mfma kernel: a tile is 16 tokens x 16 (padded) query heads.
//   lane = (g4 = lane / 16, c = lane % 16)
//   global loads: lane (g4, c) reads the 16-byte chunk c of tokens 4*g4 + i, i = 0..3, for K and V
//   K goes through a wave-private LDS tile (XOR-swizzled 16-byte chunks) and comes back as
//     A[m = token c][k-group g4] fragments of v_mfma_f32_16x16x32_f16; B = Q^T fragments in registers
//   S^T[token 4*g4+i][head c] lands in lane (g4, c) -- exactly the A-operand order of
//     v_mfma_f32_16x16x16_f16 for P (m = head c, k = 4*g4+i)
//   V fragments B[k = token 4*g4+i][n = c] for output column (dim 8*c + nn) are byte-permuted out of
//     the four 16-byte registers; acc[nn][i] = O[head 4*g4+i][dim 8*c+nn]
// =================================================================================================
// One (context, kv head) stream over the tokens [t_begin, t_end), t_begin < t_end: the running maximum `m` (log2 domain) and this
// lane's share `l` of the running sum of head c, and the unnormalised output acc[nn][i] = O[head 4*g4+i][dim 8*c+nn].
// `rot` moves the tile the walk starts at (see below).
template<int G>
__device__ __forceinline__ void mfma_stream_range( const __half* __restrict__ q,
                                                   const __half* base,
                                                   const uint32_t ctx,
                                                   const uint32_t h,
                                                   const uint32_t t_begin,
                                                   const uint32_t t_end,
                                                   const uint32_t rot,
                                                   const uint32_t n_kv_heads,
                                                   const float scale_log2e,
                                                   uint4* tile,
                                                   f32x4 ( &acc )[8],
                                                   float& m,
                                                   float& l )
{
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t g4 = lane >> 4;
  const uint32_t n_heads = n_kv_heads * G;
  const uint64_t row_elems = 2ull * n_kv_heads * HS;
  const uint32_t v_off = n_kv_heads * HS;

  // B fragments of Q^T: head c (zero for the padding heads), dims of chunk 4*kk + g4
  f16x8 qb[4];
  {
    const __half* qp = q + ( (uint64_t)ctx * n_heads + (uint64_t)h * G + ( c < G ? c : 0 ) ) * HS;
#pragma unroll
    for ( int kk = 0; kk < 4; kk++ ) {
      uint4 v = load16( qp + 8 * ( 4 * kk + g4 ) );
      if ( c >= G ) {
        v = make_uint4( 0, 0, 0, 0 );
      }
      qb[kk] = __builtin_bit_cast( f16x8, v );
    }
  }

#pragma unroll
  for ( int nn = 0; nn < 8; nn++ ) {
    acc[nn] = f32x4 { 0.0f, 0.0f, 0.0f, 0.0f };
  }
  m = -INFINITY; // running max of head c (log2 domain), identical in the 4 lanes that share c
  l = 0.0f;      // this lane's share of the running sum of head c

  const __half* kp = base + (uint64_t)h * HS + 8 * c;
  const uint4 zero4 = make_uint4( 0, 0, 0, 0 );

  // The 16-token tiles of the range are visited from a starting tile that differs between blocks,
  // wrapping around (the online softmax does not care about the order).  Blocks launched together
  // otherwise walk their ranges in lock step, and ranges of different contexts and splits lie
  // large power-of-two distances apart: such addresses share few HBM channels.
  const uint32_t n_tiles = ( t_end - t_begin + 15 ) / 16;
  uint32_t tile_i = ( ( ctx * 5u + rot * 3u ) * 7u ) % n_tiles;
  uint32_t t0 = t_begin + 16 * tile_i;

  uint4 kn[4], vn[4];
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    const uint32_t tok = t0 + 4 * g4 + i;
    const bool ok = tok < t_end;
    const __half* row = kp + (uint64_t)tok * row_elems;
    kn[i] = ok ? load16_stream( row ) : zero4;
    vn[i] = ok ? load16_stream( row + v_off ) : zero4;
  }

  for ( uint32_t it = 0; it < n_tiles; it++ ) {
    tile_i = tile_i + 1 == n_tiles ? 0 : tile_i + 1;
    const uint32_t t_next = t_begin + 16 * tile_i;
    const bool more = it + 1 < n_tiles;
    uint4 vc[4];
    // K tile into LDS: token 4*g4+i, chunk c, stored at chunk position c ^ token
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      const uint32_t tl = 4 * g4 + i;
      tile[tl * 16 + ( c ^ tl )] = kn[i];
      vc[i] = vn[i];
    }
    // prefetch the next tile
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      const uint32_t tok = t_next + 4 * g4 + i;
      const bool ok = more && tok < t_end;
      const __half* row = kp + (uint64_t)tok * row_elems;
      kn[i] = ok ? load16_stream( row ) : zero4;
      vn[i] = ok ? load16_stream( row + v_off ) : zero4;
    }
    __builtin_amdgcn_fence( __ATOMIC_RELEASE, "wavefront" );
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence( __ATOMIC_ACQUIRE, "wavefront" );

    // S^T = K Q^T : A fragment = token c, chunk 4*kk + g4
    f32x4 st = f32x4 { 0.0f, 0.0f, 0.0f, 0.0f };
#pragma unroll
    for ( int kk = 0; kk < 4; kk++ ) {
      const uint4 kf = tile[c * 16 + ( ( 4 * kk + g4 ) ^ c )];
      st = __builtin_amdgcn_mfma_f32_16x16x32_f16( __builtin_bit_cast( f16x8, kf ), qb[kk], st, 0, 0, 0 );
    }
    __builtin_amdgcn_fence( __ATOMIC_RELEASE, "wavefront" );
    __builtin_amdgcn_wave_barrier(); // the tile is rewritten at the top of the next iteration

    // st[i] = score of token t0 + 4*g4 + i for head c
    float s[4];
    float mt = -INFINITY;
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      const bool ok = t0 + 4 * g4 + i < t_end;
      s[i] = ok ? st[i] * scale_log2e : -INFINITY;
      mt = fmaxf( mt, s[i] );
    }
    mt = fmaxf( mt, __shfl_xor( mt, 16, WAVE ) );
    mt = fmaxf( mt, __shfl_xor( mt, 32, WAVE ) );
    const float m_new = fmaxf( m, mt ); // finite: the first token of every tile is inside the range
    const float alpha = fast_exp2( m - m_new );
    float p[4];
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      p[i] = fast_exp2( s[i] - m_new );
    }
    l = l * alpha + ( p[0] + p[1] ) + ( p[2] + p[3] );
    m = m_new;

    // rescale the accumulators when some head's maximum moved: acc[.][i] belongs to head 4*g4 + i
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

    // P as A fragment: head c, tokens 4*g4 .. 4*g4+3
    const f16x4 pa = f16x4 { (_Float16)p[0], (_Float16)p[1], (_Float16)p[2], (_Float16)p[3] };

    // V fragments: for output column nn = 2*w + hl take half `hl` of word w of the four token registers
    const uint32_t vw[4][4] = { { vc[0].x, vc[0].y, vc[0].z, vc[0].w },
                                { vc[1].x, vc[1].y, vc[1].z, vc[1].w },
                                { vc[2].x, vc[2].y, vc[2].z, vc[2].w },
                                { vc[3].x, vc[3].y, vc[3].z, vc[3].w } };
#pragma unroll
    for ( int w = 0; w < 4; w++ ) {
      // low halves: bytes 0,1 of the first source then bytes 0,1 of the second
      const uint2 lo = make_uint2( __builtin_amdgcn_perm( vw[1][w], vw[0][w], 0x05040100u ),
                                   __builtin_amdgcn_perm( vw[3][w], vw[2][w], 0x05040100u ) );
      const uint2 hi = make_uint2( __builtin_amdgcn_perm( vw[1][w], vw[0][w], 0x07060302u ),
                                   __builtin_amdgcn_perm( vw[3][w], vw[2][w], 0x07060302u ) );
      acc[2 * w] = __builtin_amdgcn_mfma_f32_16x16x16f16( pa, __builtin_bit_cast( f16x4, lo ), acc[2 * w], 0, 0, 0 );
      acc[2 * w + 1] = __builtin_amdgcn_mfma_f32_16x16x16f16( pa, __builtin_bit_cast( f16x4, hi ), acc[2 * w + 1], 0, 0, 0 );
    }
    t0 = t_next;
  }

}

template<int G>
__global__ __launch_bounds__( 256 ) void attn_decode_mfma_kernel( const __half* __restrict__ q,
                                                                  const __half* const* __restrict__ layer_rows,
                                                                  const uint32_t* __restrict__ pos,
                                                                  Partials part,
                                                                  __half* __restrict__ xb,
                                                                  uint32_t n_kv_heads,
                                                                  uint32_t chunk,
                                                                  uint32_t max_splits,
                                                                  uint32_t seq_len,
                                                                  float scale_log2e )
{
  __shared__ uint4 s_k[4][16 * 16]; // per wave: 16 tokens x 16 chunks of 16 bytes

  const WaveJob job = wave_job( layer_rows, pos, n_kv_heads, chunk, max_splits, seq_len );
  if ( !job.valid ) {
    return; // wave-uniform; only wave-private LDS is used, no block barrier
  }
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t g4 = lane >> 4;
  const uint32_t n_heads = n_kv_heads * G;
  uint4* tile = s_k[wave];

  f32x4 acc[8];
  float m, l;
  mfma_stream_range<G>( q, job.base, job.ctx, job.h, job.t_begin, job.t_end, job.split, n_kv_heads, scale_log2e, tile, acc, m, l );

  // total sum of head c over the four lane groups
  l += __shfl_xor( l, 16, WAVE );
  l += __shfl_xor( l, 32, WAVE );

  // the accumulators of this lane belong to heads 4*g4 + i; fetch their m and l from lanes c' = 4*g4 + i
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    const uint32_t hd = 4 * g4 + i;
    const float mh = __shfl( m, (int)hd, WAVE );
    const float lh = __shfl( l, (int)hd, WAVE );
    if ( hd < G ) {
      const uint64_t head = (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G + hd;
      if ( max_splits == 1 ) {
        const float inv = 1.0f / lh;
        union
        {
          uint4 raw;
          __half h[8];
        } o;
#pragma unroll
        for ( int nn = 0; nn < 8; nn++ ) {
          o.h[nn] = __float2half_rn( acc[nn][i] * inv );
        }
        *reinterpret_cast<uint4*>( xb + head * HS + 8 * c ) = o.raw;
      } else {
        const uint64_t slot = head * max_splits + job.split;
        float4* o = reinterpret_cast<float4*>( part.out + slot * HS + 8 * c );
        o[0] = make_float4( acc[0][i], acc[1][i], acc[2][i], acc[3][i] );
        o[1] = make_float4( acc[4][i], acc[5][i], acc[6][i], acc[7][i] );
        if ( c == 0 ) {
          part.ml[slot * 2] = mh;
          part.ml[slot * 2 + 1] = lh;
        }
      }
    }
  }
}

// the mfma kernel with the splits of a stream joined inside the work-group (see joined_job)
template<int G, uint32_t JOIN_WAVES>
__global__ __launch_bounds__( 64 * JOIN_WAVES ) void attn_decode_mfma_joined_kernel( const __half* __restrict__ q,
                                                                         const __half* const* __restrict__ layer_rows,
                                                                         const uint32_t* __restrict__ pos,
                                                                         __half* __restrict__ xb,
                                                                         uint32_t n_kv_heads,
                                                                         uint32_t batch,
                                                                         uint32_t chunk,
                                                                         uint32_t splits,
                                                                         uint32_t seq_len,
                                                                         float scale_log2e )
{
  __shared__ uint4 s_k[JOIN_WAVES][16 * 16]; // per wave: 16 tokens x 16 chunks of 16 bytes
  // per wave and lane: its 32 accumulators, then the maxima and the sums of its 4 heads; only the lanes whose heads exist (the first 4 G)
  constexpr int JOIN_LANES = 4 * G < 16 ? 16 : 4 * G;
  __shared__ float s_join[JOIN_WAVES][40][JOIN_LANES];
  const JoinedJob job = joined_job<JOIN_WAVES>( layer_rows, pos, n_kv_heads, batch, chunk, splits, seq_len );
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c = lane & 15;
  const uint32_t g4 = lane >> 4;
  const uint32_t n_heads = n_kv_heads * G;

  f32x4 acc[8];
  float mh[4], lh[4]; // of heads 4*g4 + i, to which this lane's accumulators acc[.][i] belong
  if ( job.active ) {
    float m, l;
    mfma_stream_range<G>( q, job.base, job.ctx, job.h, job.t_begin, job.t_end, job.split, n_kv_heads, scale_log2e, s_k[wave], acc, m, l );
    l += __shfl_xor( l, 16, WAVE );
    l += __shfl_xor( l, 32, WAVE );
#pragma unroll
    for ( int i = 0; i < 4; i++ ) {
      mh[i] = __shfl( m, (int)( 4 * g4 + i ), WAVE );
      lh[i] = __shfl( l, (int)( 4 * g4 + i ), WAVE );
    }
    if ( job.split != 0 && 4 * g4 < G ) {
#pragma unroll
      for ( int i = 0; i < 4; i++ ) {
#pragma unroll
        for ( int nn = 0; nn < 8; nn++ ) {
          s_join[wave][8 * i + nn][lane] = acc[nn][i];
        }
        s_join[wave][32 + i][lane] = mh[i];
        s_join[wave][36 + i][lane] = lh[i];
      }
    }
  }
  __syncthreads(); // reached by every wave of the work-group, with or without keys
  if ( job.split != 0 || !job.active ) {
    return; // split 0 holds keys whenever any split of the stream does
  }
#pragma unroll
  for ( int i = 0; i < 4; i++ ) {
    const uint32_t hd = 4 * g4 + i;
    if ( hd >= G ) {
      continue;
    }
    float mm = mh[i];
    for ( uint32_t u = 1; u < job.n_splits; u++ ) {
      mm = fmaxf( mm, s_join[wave + u][32 + i][lane] );
    }
    const float w0 = fast_exp2( mh[i] - mm );
    float lsum = lh[i] * w0;
    float out[8];
#pragma unroll
    for ( int nn = 0; nn < 8; nn++ ) {
      out[nn] = acc[nn][i] * w0;
    }
    for ( uint32_t u = 1; u < job.n_splits; u++ ) {
      const float wu = fast_exp2( s_join[wave + u][32 + i][lane] - mm );
      lsum = __builtin_fmaf( s_join[wave + u][36 + i][lane], wu, lsum );
#pragma unroll
      for ( int nn = 0; nn < 8; nn++ ) {
        out[nn] = __builtin_fmaf( s_join[wave + u][8 * i + nn][lane], wu, out[nn] );
      }
    }
    const float inv = 1.0f / lsum;
    union
    {
      uint4 raw;
      __half h[8];
    } o;
#pragma unroll
    for ( int nn = 0; nn < 8; nn++ ) {
      o.h[nn] = __float2half_rn( out[nn] * inv );
    }
    const uint64_t head = (uint64_t)job.ctx * n_heads + (uint64_t)job.h * G + hd;
    *reinterpret_cast<uint4*>( xb + head * HS + 8 * c ) = o.raw;
  }
}

// =================================================================================================
// balanced variant of the mfma kernel for batches whose contexts differ in length
//
// With one work-group per (context, group of 4 kv heads) and every work-group resident at once, a launch lasts as long as
// the CU that drew the longest contexts.  Here the keys of all contexts are laid end to end in chunks of BAL_CHUNK tokens
// and the list is cut into equal runs, one per resident work-group (two per CU): a work-group walks its run through as
// many contexts as it spans.  A piece that is a whole context is finished on the spot; the pieces of a context that a cut
// divides leave partials, at slot (context + work-group) -- along the list either of the two grows by one from piece to
// piece, so the sum numbers the pieces -- and the merge kernel combines them.  The cuts depend on the positions only, not
// on the layer: attn_balance_kernel makes them once per step.
//   plan (u32): header[8] (0: chunks per work-group, 1: chunks in all) | prefix[batch + 1] chunks before context c |
//               length[batch] keys of context c (0: none) | first[work-groups per head group] context a work-group starts in
// =================================================================================================
constexpr uint32_t BAL_CHUNK = 64;
constexpr uint32_t BAL_MIN_RUN = 4; // chunks: a shorter run costs more in start-up than it evens out (measured at 16 contexts)
constexpr uint32_t BAL_HEADER = 8;
constexpr int BAL_PLAN_THREADS = 1024;

struct BalancedPlan
{
  uint32_t* header;
  uint32_t* prefix;
  uint32_t* length;
  uint32_t* first;
};

__global__ __launch_bounds__( BAL_PLAN_THREADS ) void attn_balance_kernel( const void* const* __restrict__ layer_rows,
                                                                         const uint32_t* __restrict__ pos,
                                                                         uint32_t batch,
                                                                         uint32_t max_len,
                                                                         uint32_t wgs,
                                                                         BalancedPlan plan )
{
  __shared__ uint32_t s_scan[BAL_PLAN_THREADS];
  const uint32_t t = threadIdx.x;
  const uint32_t per = ( batch + BAL_PLAN_THREADS - 1 ) / BAL_PLAN_THREADS; // contexts per thread, consecutive
  const uint32_t c_begin = min( batch, t * per ), c_end = min( batch, c_begin + per );
  uint32_t own = 0;
  for ( uint32_t c = c_begin; c < c_end; c++ ) {
    const uint32_t len = layer_rows[c] != nullptr ? min( pos[c] + 1, max_len ) : 0u; // never beyond what the host sized the call for
    plan.length[c] = len;
    own += ( len + BAL_CHUNK - 1 ) / BAL_CHUNK;
  }
  s_scan[t] = own;
  __syncthreads();
  for ( uint32_t d = 1; d < BAL_PLAN_THREADS; d <<= 1 ) { // inclusive scan
    const uint32_t add = t >= d ? s_scan[t - d] : 0u;
    __syncthreads();
    s_scan[t] += add;
    __syncthreads();
  }
  const uint32_t total = s_scan[BAL_PLAN_THREADS - 1];
  const uint32_t run = max( BAL_MIN_RUN, ( total + wgs - 1 ) / wgs );
  if ( t == 0 ) {
    plan.header[0] = run;
    plan.header[1] = total;
    plan.prefix[batch] = total;
  }
  for ( uint32_t w = t; w < wgs; w += BAL_PLAN_THREADS ) {
    plan.first[w] = batch; // a work-group whose run starts behind the list has nothing to do
  }
  __syncthreads(); // first[] is initialised before any thread overwrites an entry (global memory, same block)
  uint32_t before = s_scan[t] - own;
  for ( uint32_t c = c_begin; c < c_end; c++ ) {
    const uint32_t n = ( plan.length[c] + BAL_CHUNK - 1 ) / BAL_CHUNK;
    plan.prefix[c] = before;
    // the work-groups whose run starts inside this context
    for ( uint32_t w = ( before + run - 1 ) / run; w < wgs && w * run < before + n; w++ ) {
      plan.first[w] = c;
    }
    before += n;
  }
}

// slot of the piece (context c, work-group w of head group g) for the query head (kv head `h_local` of the group, head `hd` of it)
__device__ __forceinline__ uint64_t balanced_slot( uint32_t g, uint32_t pieces, uint32_t c, uint32_t w, uint32_t h_local, uint32_t G, uint32_t hd )
{
  return ( ( (uint64_t)g * pieces + c + w ) * 4 + h_local ) * G + hd;
}

// grid: work-groups per head group x head groups; wave <-> kv head of the group.  MFMA: the streaming loop of the mfma kernel
// (gqa 2 and more), else that of the valu kernel (one query head per kv head).
template<int G, bool MFMA>
__global__ __launch_bounds__( 256 ) void attn_decode_balanced_kernel( const __half* __restrict__ q,
                                                                      const __half* const* __restrict__ layer_rows,
                                                                      BalancedPlan plan,
                                                                      Partials part,
                                                                      __half* __restrict__ xb,
                                                                      uint32_t n_kv_heads,
                                                                      uint32_t batch,
                                                                      uint32_t wgs,
                                                                      float scale_log2e )
{
  __shared__ uint4 s_k[4][16 * 16];
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t c16 = lane & 15;
  const uint32_t g4 = lane >> 4;
  const uint32_t head_groups = ( n_kv_heads + 3 ) / 4;
  const uint32_t w = blockIdx.x / head_groups; // the head groups of a run of keys start next to each other in time: whole cache rows are read together
  const uint32_t g = blockIdx.x % head_groups;
  const uint32_t h = g * 4 + wave;
  if ( h >= n_kv_heads ) {
    return; // wave-uniform; only wave-private LDS is used, no block barrier
  }
  const uint32_t n_heads = n_kv_heads * G;
  const uint32_t run = plan.header[0], total = plan.header[1];
  const uint32_t pieces = batch + wgs;
  uint32_t at = w * run; // position in the list of chunks
  const uint32_t end = min( total, at + run );
  uint32_t c = plan.first[w];
  // every turn either moves `at` forward or steps over a context without keys; at < end <= prefix[batch] keeps c < batch
  while ( at < end && c < batch ) {
    const uint32_t p0 = plan.prefix[c], p1 = plan.prefix[c + 1];
    if ( p1 <= at ) {
      c++;
      continue;
    }
    const uint32_t piece_end = min( p1, end );
    const __half* base = layer_rows[c];
    const uint32_t t_begin = ( at - p0 ) * BAL_CHUNK;
    const uint32_t t_end = min( plan.length[c], ( piece_end - p0 ) * BAL_CHUNK );
    const bool whole = at == p0 && piece_end == p1;
    if ( base != nullptr && t_begin < t_end ) {
      if constexpr ( MFMA ) {
        f32x4 acc[8];
        float m, l;
        mfma_stream_range<G>( q, base, c, h, t_begin, t_end, w, n_kv_heads, scale_log2e, s_k[wave], acc, m, l );
        l += __shfl_xor( l, 16, WAVE );
        l += __shfl_xor( l, 32, WAVE );
#pragma unroll
        for ( int i = 0; i < 4; i++ ) {
          const uint32_t hd = 4 * g4 + i;
          const float mh = __shfl( m, (int)hd, WAVE );
          const float lh = __shfl( l, (int)hd, WAVE );
          if ( hd < G ) {
            if ( whole ) {
              const uint64_t head = (uint64_t)c * n_heads + (uint64_t)h * G + hd;
              const float inv = 1.0f / lh;
              union
              {
                uint4 raw;
                __half h[8];
              } o;
#pragma unroll
              for ( int nn = 0; nn < 8; nn++ ) {
                o.h[nn] = __float2half_rn( acc[nn][i] * inv );
              }
              *reinterpret_cast<uint4*>( xb + head * HS + 8 * c16 ) = o.raw;
            } else {
              const uint64_t slot = balanced_slot( g, pieces, c, w, wave, G, hd );
              float4* o = reinterpret_cast<float4*>( part.out + slot * HS + 8 * c16 );
              o[0] = make_float4( acc[0][i], acc[1][i], acc[2][i], acc[3][i] );
              o[1] = make_float4( acc[4][i], acc[5][i], acc[6][i], acc[7][i] );
              if ( c16 == 0 ) {
                part.ml[slot * 2] = mh;
                part.ml[slot * 2 + 1] = lh;
              }
            }
          }
        }
      } else {
        float m[G], l[G], acc[G][8];
        valu_stream_range<G>( q, base, c, h, t_begin, t_end, w, n_kv_heads, scale_log2e, m, l, acc );
        if ( g4 == 0 ) { // the four lanes that share a chunk hold the same sums
#pragma unroll
          for ( int hd = 0; hd < G; hd++ ) {
            if ( whole ) {
              const uint64_t head = (uint64_t)c * n_heads + (uint64_t)h * G + hd;
              const float inv = 1.0f / l[hd];
              union
              {
                uint4 raw;
                __half h[8];
              } o;
#pragma unroll
              for ( int e = 0; e < 8; e++ ) {
                o.h[e] = __float2half_rn( acc[hd][e] * inv );
              }
              *reinterpret_cast<uint4*>( xb + head * HS + 8 * c16 ) = o.raw;
            } else {
              const uint64_t slot = balanced_slot( g, pieces, c, w, wave, G, hd );
              float4* o = reinterpret_cast<float4*>( part.out + slot * HS + 8 * c16 );
              o[0] = make_float4( acc[hd][0], acc[hd][1], acc[hd][2], acc[hd][3] );
              o[1] = make_float4( acc[hd][4], acc[hd][5], acc[hd][6], acc[hd][7] );
              if ( c16 == 0 ) {
                part.ml[slot * 2] = m[hd];
                part.ml[slot * 2 + 1] = l[hd];
              }
            }
          }
        }
      }
    }
    at = piece_end;
    if ( piece_end == p1 ) {
      c++;
    }
  }
}

// block <-> (kv head, context), thread <-> (query head of the kv head, output dim): combines the pieces of a context that the
// cuts divided.  Most blocks of a launch find their context in one piece and leave at once, so there are few and large ones.
template<int G>
__global__ __launch_bounds__( ( G < 8 ? G : 8 ) * 128 ) void attn_merge_balanced_kernel( BalancedPlan plan,
                                                                                       Partials part,
                                                                                       __half* __restrict__ xb,
                                                                                       uint32_t n_heads,
                                                                                       uint32_t batch,
                                                                                       uint32_t wgs )
{
  const uint32_t kv = blockIdx.x;
  const uint32_t ctx = blockIdx.y;
  const uint32_t p0 = plan.prefix[ctx], p1 = plan.prefix[ctx + 1], run = plan.header[0];
  if ( p1 == p0 ) {
    return; // no keys: the output row stays as it is, as in the other kernels
  }
  const uint32_t w0 = p0 / run, w1 = ( p1 - 1 ) / run;
  if ( w0 == w1 ) {
    return; // one piece: written by the work-group that ran it
  }
  const uint32_t n = w1 - w0 + 1;
  const uint64_t step = 4ull * G; // slots from one work-group's piece to the next one's
  const float2* ml = reinterpret_cast<const float2*>( part.ml );
  const uint32_t d = threadIdx.x % HS;
  constexpr uint32_t MERGE_BATCH = 4;
  for ( uint32_t hd = threadIdx.x / HS; hd < G; hd += blockDim.x / HS ) { // one turn except at gqa 16
    const uint64_t slot0 = balanced_slot( kv / 4, batch + wgs, ctx, w0, kv % 4, G, hd );
    float2 st[MERGE_BATCH];
    float o[MERGE_BATCH];
#pragma unroll
    for ( uint32_t u = 0; u < MERGE_BATCH; u++ ) { // a piece past the last reads the last again and gets weight zero
      const uint64_t slot = slot0 + min( u, n - 1 ) * step;
      st[u] = ml[slot];
      o[u] = part.out[slot * HS + d];
    }
    float m = -INFINITY;
#pragma unroll
    for ( uint32_t u = 0; u < MERGE_BATCH; u++ ) {
      m = fmaxf( m, st[u].x );
    }
    for ( uint32_t k = MERGE_BATCH; k < n; k++ ) {
      m = fmaxf( m, ml[slot0 + k * step].x );
    }
    float l = 0.0f, acc = 0.0f;
#pragma unroll
    for ( uint32_t u = 0; u < MERGE_BATCH; u++ ) {
      const float wgt = u < n ? fast_exp2( st[u].x - m ) : 0.0f;
      l += st[u].y * wgt;
      acc += o[u] * wgt;
    }
    for ( uint32_t k = MERGE_BATCH; k < n; k++ ) {
      const uint64_t slot = slot0 + k * step;
      const float2 e = ml[slot];
      const float wgt = fast_exp2( e.x - m );
      l += e.y * wgt;
      acc += part.out[slot * HS + d] * wgt;
    }
    xb[( (uint64_t)ctx * n_heads + (uint64_t)kv * G + hd ) * HS + d] = __float2half_rn( acc * ( 1.0f / l ) );
  }
}

// =================================================================================================
// host side
// =================================================================================================
struct Plan
{
  int variant;
  uint32_t chunk;       // tokens per split
  uint32_t max_splits;  // splits of the longest context
  uint32_t split_bound; // upper bound of max_splits for any shorter longest context (sizes the workspace)
  uint32_t join;        // > 0: the splits of a stream are waves of one work-group of this many waves, which adds them up itself
};

// The splits of a (context, kv head) stream as waves of one work-group (no partial sums in memory, no merge kernel), for the f16
// head-128 kernels: how many splits and how many waves per work-group, by the number of streams per CU.  A work-group of W waves
// holds W / splits neighbouring kv heads (its waves then read neighbouring pieces of the same cache rows: with one head per
// work-group of 8 waves the walk itself is slower than what the merge kernel costs), and what counts beside that is how evenly the
// work-groups fill the CUs: every range below ends where its work-groups would no longer fit the CUs in one go.  Measured on MI355X
// (256 CUs), fused op in us, partial sums + merge kernel / the choice below.  70B shape (8 kv heads, MFMA kernel), contexts x 4096 keys:
//   24: 81 / 74 (4 splits, 4 waves)   32: 87 / 81   40: 123 / 109 (4, 8)   48: 142 / 123   64: 164 / 155   66: 202 / 180 (2, 8)
//   80: 224 / 196   104: 282 / 250   112: 293 / 266 (2, 4)   128: 362 / 308   144: 408 / 386 (4, 8)   160: 457 / 397   250: 716 / 605
// 7B shape (32 kv heads with one query head each: the VALU kernel), contexts x 2048 keys:
//   10: 62 / 56 (4, 8)   16: 85 / 80   17: 104.5 / 94 (2, 8)   26: 144 / 130   27: 146 / 133 (2, 4)   32: 167 / 157
// and 32 x 1024 keys: 85.5 / 80.2.  13B shape (40 heads), x 2048 keys: 8: 62.4 / 60.8   12: 85 / 77   16: 108.5 / 109.6   21: 141 / 137.
// This kernel with more than four streams per CU or with at most one: no joined choice ahead of the merge route (13B, 32
// contexts: 204 / 212; 7B, 8 contexts: 44.5 / 45.8).
struct JoinChoice
{
  uint32_t splits, waves; // waves == 0: none
};
JoinChoice join_choice( uint64_t streams, int variant, uint32_t n_tok )
{
  const uint64_t cus = (uint64_t)cu_count();
  const uint64_t x8 = 8 * streams; // streams per CU in eighths
  JoinChoice c { 0, 0 };
  if ( x8 < 6 * cus ) {
    return c;
  } else if ( x8 <= 8 * cus ) {
    c = variant == GH_ATTN_MFMA ? JoinChoice { 4, 4 } : c; // one work-group of 4 waves per stream, at most one per CU
  } else if ( x8 < 10 * cus ) {
    return c; // work-groups of 8 waves would reach little more than half of the CUs (-9 ... +6 %)
  } else if ( x8 <= 16 * cus ) {
    c = JoinChoice { 4, 8 }; // one work-group of 8 waves per two streams, at most one per CU
  } else if ( x8 <= 26 * cus ) {
    c = JoinChoice { 2, 8 }; // ... per four streams
  } else if ( x8 <= 32 * cus ) {
    c = JoinChoice { 2, 4 }; // two work-groups of 4 waves per CU
  } else if ( x8 < 64 * cus ) {
    c = variant == GH_ATTN_MFMA ? JoinChoice { 4, 8 } : c; // several rounds of work-groups
  }
  // splits are never shorter than 256 tokens
  while ( c.waves != 0 && c.splits > 1 && (uint64_t)n_tok < 256ull * c.splits ) {
    c.splits /= 2;
  }
  if ( c.splits < 2 ) {
    c = JoinChoice { 0, 0 };
  }
  return c;
}

bool fast_ok( const gh_shape* s, gh_dtype dt ) { return dt == GH_F16 && s->head_size == HS; }
bool valu_gqa_ok( uint32_t g ) { return g == 1 || g == 2 || g == 4 || g == 8; }
bool mfma_gqa_ok( uint32_t g ) { return g == 2 || g == 4 || g == 8 || g == 16; }

Plan make_plan( uint64_t batch, uint32_t max_pos, const gh_shape* s, gh_dtype dt, int variant )
{
  Plan p;
  p.join = 0;
  p.variant = variant;
  if ( variant == GH_ATTN_AUTO && g_auto_variant == GH_ATTN_GENERIC ) {
    p.variant = GH_ATTN_GENERIC;
  } else if ( variant == GH_ATTN_AUTO && g_auto_variant == GH_ATTN_VALU && fast_ok( s, dt ) && valu_gqa_ok( s->gqa_size ) ) {
    p.variant = GH_ATTN_VALU;
  } else if ( variant == GH_ATTN_AUTO && g_auto_variant == GH_ATTN_MFMA && fast_ok( s, dt ) && mfma_gqa_ok( s->gqa_size ) ) {
    p.variant = GH_ATTN_MFMA;
  } else if ( variant == GH_ATTN_AUTO ) {
    if ( fast_ok( s, dt ) && mfma_gqa_ok( s->gqa_size ) && s->gqa_size >= 4 ) {
      p.variant = GH_ATTN_MFMA;
    } else if ( fast_ok( s, dt ) && valu_gqa_ok( s->gqa_size ) ) {
      p.variant = GH_ATTN_VALU;
    } else {
      p.variant = GH_ATTN_GENERIC;
    }
  }
  const uint32_t n_tok = max_pos + 1;
  uint32_t chunk;
  uint64_t split_cap = 0;
  if ( g_chunk_override ) {
    chunk = g_chunk_override;
  } else {
    // One wave per (context, kv head, split).  Measured on MI355X: 8 waves per CU (2048 in all), each
    // streaming a long range, is the sweet spot; with 2048 or more (context, head) streams no split is
    // needed at all and the merge kernel disappears.  Between 1024 and 2048 streams one wave per stream
    // leaves the CUs with 4-7 waves: ranges of 512 keys, which come in several rounds, are 3-11 % faster
    // (7B shape, 32 contexts of 1024 keys: 90 -> 87 us; 13B, 32 of 2048: 222 -> 203).  Splits are never
    // shorter than 256 tokens so that the partial traffic stays a few percent of the cache traffic.
    const uint64_t streams = batch * ( p.variant == GH_ATTN_GENERIC ? s->n_heads : s->n_kv_heads );
    uint64_t splits = streams >= 2048 ? 1 : streams >= 1024 ? std::max<uint64_t>( 2, n_tok / 512 ) : ( 2048 + streams - 1 ) / ( streams ? streams : 1 );
    chunk = (uint32_t)( ( n_tok + splits - 1 ) / splits );
    if ( chunk < 256 ) {
      chunk = 256;
    }
    split_cap = std::min<uint64_t>( splits, ( n_tok + 255 ) / 256 );
    // the joined route where it pays: never more splits than the rule above gives, so the workspace bound holds either way
    if ( g_split_join != 0 && p.variant != GH_ATTN_GENERIC ) {
      const JoinChoice c = join_choice( streams, p.variant, n_tok );
      if ( c.waves != 0 && c.splits <= splits ) {
        chunk = ( n_tok + c.splits - 1 ) / c.splits;
        p.join = g_split_join == 4 || g_split_join == 8 ? (uint32_t)g_split_join : c.waves;
      }
    }
  }
  chunk = ( chunk + 15 ) / 16 * 16;
  p.chunk = chunk;
  p.max_splits = ( n_tok + chunk - 1 ) / chunk;
  if ( p.max_splits < 1 ) {
    p.max_splits = 1;
  }
  p.split_bound = (uint32_t)std::max<uint64_t>( p.max_splits, split_cap );
  // a split length given from outside (tests, measurements), or a forced work-group size: joined whenever the plan has 2 or 4 splits
  if ( g_split_join != 0 && p.variant != GH_ATTN_GENERIC && ( g_chunk_override != 0 || g_split_join == 4 || g_split_join == 8 ) ) {
    p.join = g_split_join == 4 || g_split_join == 8 ? (uint32_t)g_split_join : 8u;
  }
  if ( !( p.max_splits == 2 || p.max_splits == 4 ) || p.max_splits > p.join ) {
    p.join = 0;
  }
  return p;
}

uint64_t partial_floats( uint64_t batch, const gh_shape* s, uint32_t max_splits )
{
  return batch * s->n_heads * (uint64_t)max_splits * ( s->head_size + 2ull );
}

template<int G>
void launch_valu( dim3 grid, hipStream_t st, const void* q, const void* const* rows, const uint32_t* pos, Partials part, void* xb,
                  const gh_shape* s, const Plan& p, float scale )
{
  attn_decode_valu_kernel<G><<<grid, 256, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( rows ), pos, part,
                                                   static_cast<__half*>( xb ), s->n_kv_heads, p.chunk, p.max_splits, s->seq_len, scale );
}

template<int G>
void launch_mfma( dim3 grid, hipStream_t st, const void* q, const void* const* rows, const uint32_t* pos, Partials part, void* xb,
                  const gh_shape* s, const Plan& p, float scale )
{
  attn_decode_mfma_kernel<G><<<grid, 256, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( rows ), pos, part,
                                                   static_cast<__half*>( xb ), s->n_kv_heads, p.chunk, p.max_splits, s->seq_len, scale );
}

template<int G>
void launch_valu_joined( uint32_t waves, dim3 grid, hipStream_t st, const void* q, const void* const* rows, const uint32_t* pos, void* xb, const gh_shape* s,
                         const Plan& p, uint32_t batch, float scale )
{
  if ( waves == 4 ) {
    attn_decode_valu_joined_kernel<G, 4><<<grid, 256, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( rows ), pos,
                                                               static_cast<__half*>( xb ), s->n_kv_heads, batch, p.chunk, p.max_splits, s->seq_len, scale );
  } else {
    attn_decode_valu_joined_kernel<G, 8><<<grid, 512, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( rows ), pos,
                                                               static_cast<__half*>( xb ), s->n_kv_heads, batch, p.chunk, p.max_splits, s->seq_len, scale );
  }
}

template<int G>
void launch_mfma_joined( uint32_t waves, dim3 grid, hipStream_t st, const void* q, const void* const* rows, const uint32_t* pos, void* xb, const gh_shape* s,
                         const Plan& p, uint32_t batch, float scale )
{
  if ( waves == 4 ) {
    attn_decode_mfma_joined_kernel<G, 4><<<grid, 256, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( rows ), pos,
                                                               static_cast<__half*>( xb ), s->n_kv_heads, batch, p.chunk, p.max_splits, s->seq_len, scale );
  } else {
    attn_decode_mfma_joined_kernel<G, 8><<<grid, 512, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( rows ), pos,
                                                               static_cast<__half*>( xb ), s->n_kv_heads, batch, p.chunk, p.max_splits, s->seq_len, scale );
  }
}

// where the plan and the partials of the balanced variant lie in its workspace
struct BalancedLayout
{
  uint32_t head_groups, wgs; // groups of 4 kv heads; work-groups per head group
  uint64_t plan_bytes, out_floats, ml_floats, total_bytes;
};

BalancedLayout balanced_layout( uint64_t batch, const gh_shape* s )
{
  BalancedLayout y;
  y.head_groups = ( s->n_kv_heads + 3 ) / 4;
  // two work-groups of four waves are resident per CU
  y.wgs = std::max<uint32_t>( 1, 2u * (uint32_t)cu_count() / y.head_groups );
  const uint64_t pieces = batch + y.wgs;
  const uint64_t heads = 4ull * s->gqa_size; // per (head group, piece)
  y.out_floats = y.head_groups * pieces * heads * HS;
  y.ml_floats = y.head_groups * pieces * heads * 2;
  y.plan_bytes = ( ( BAL_HEADER + ( batch + 1 ) + batch + y.wgs ) * sizeof( uint32_t ) + 255 ) / 256 * 256;
  y.total_bytes = y.plan_bytes + ( y.out_floats + y.ml_floats ) * sizeof( float );
  return y;
}

BalancedPlan balanced_plan( void* workspace, uint64_t batch )
{
  BalancedPlan p;
  p.header = static_cast<uint32_t*>( workspace );
  p.prefix = p.header + BAL_HEADER;
  p.length = p.prefix + batch + 1;
  p.first = p.length + batch;
  return p;
}

int balanced_check( const char* who, uint64_t batch, uint32_t max_pos, const gh_shape* shape, const void* workspace, uint64_t workspace_bytes )
{
  GH_REQUIRE( shape != nullptr, "%s: NULL shape", who );
  GH_REQUIRE( shape->n_kv_heads > 0 && shape->gqa_size > 0 && shape->seq_len > 0, "%s: zero dimension", who );
  GH_REQUIRE( shape->n_heads == shape->n_kv_heads * shape->gqa_size, "%s: n_heads != n_kv_heads * gqa_size", who );
  GH_REQUIRE( shape->kv_dim == shape->n_kv_heads * shape->head_size, "%s: kv_dim != n_kv_heads * head_size", who );
  GH_REQUIRE( shape->head_size == HS && ( shape->gqa_size == 1 || mfma_gqa_ok( shape->gqa_size ) ), "%s: needs head_size 128 and gqa in {1,2,4,8,16}", who );
  GH_REQUIRE( max_pos < shape->seq_len, "%s: max_pos %u outside seq_len %u", who, max_pos, shape->seq_len );
  GH_REQUIRE( batch > 0 && batch <= 65535, "%s: bad batch", who );
  GH_REQUIRE( workspace != nullptr && ( reinterpret_cast<uintptr_t>( workspace ) & 15u ) == 0, "%s: workspace missing or not 16-byte aligned", who );
  const uint64_t need = balanced_layout( batch, shape ).total_bytes;
  if ( workspace_bytes < need ) {
    return fail( GH_ERR_WORKSPACE, "%s: %llu bytes of workspace needed, %llu available", who, (unsigned long long)need, (unsigned long long)workspace_bytes );
  }
  return GH_OK;
}

template<int G, bool MFMA>
void launch_balanced( const BalancedLayout& y, hipStream_t st, const void* q, const void* const* rows, const BalancedPlan& plan, Partials part, void* xb,
                      const gh_shape* s, uint64_t batch, float scale )
{
  attn_decode_balanced_kernel<G, MFMA><<<y.head_groups * y.wgs, 256, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( rows ), plan,
                                                                        part, static_cast<__half*>( xb ), s->n_kv_heads, (uint32_t)batch, y.wgs, scale );
  attn_merge_balanced_kernel<G><<<dim3( s->n_kv_heads, (unsigned)batch ), ( G < 8 ? G : 8 ) * 128, 0, st>>>( plan, part, static_cast<__half*>( xb ), s->n_heads,
                                                                                                             (uint32_t)batch, y.wgs );
}

} // namespace

// Called by the library's initialisation with `device` current: the device address of this GPU's
// `scratch` array.  Every GPU holds its own copy of the array at its own address.
int attn_static_scratch_init( int device )
{
  GH_REQUIRE( device >= 0 && device < MAX_DEVICES, "device %d beyond the %d devices the static attention scratch is kept for", device, MAX_DEVICES );
  float* ptr = nullptr;
  GH_HIP( hipGetSymbolAddress( reinterpret_cast<void**>( &ptr ), HIP_SYMBOL( scratch ) ) );
  GH_REQUIRE( ptr != nullptr && ( reinterpret_cast<uintptr_t>( ptr ) & 255u ) == 0, "static attention scratch has no aligned device address" );
  g_static_scratch[device] = ptr;
  return GH_OK;
}

} // namespace gh

using namespace gh;

extern "C" {

int gh_attn_set_auto_variant( int variant )
{
  GH_REQUIRE( variant >= GH_ATTN_AUTO && variant <= GH_ATTN_MFMA, "gh_attn_set_auto_variant: unknown variant %d", variant );
  g_auto_variant = variant;
  return GH_OK;
}

int gh_attn_set_split_join( int on )
{
  GH_REQUIRE( on == 0 || on == 1 || on == 4 || on == 8, "gh_attn_set_split_join: %d is not 0, 1, 4 or 8", on );
  g_split_join = on;
  return GH_OK;
}

int gh_attn_set_chunk( uint32_t tokens_per_split )
{
  g_chunk_override = tokens_per_split;
  return GH_OK;
}

uint64_t gh_attn_decode_workspace( uint64_t batch, uint32_t max_pos, const gh_shape* shape )
{
  if ( shape == nullptr || batch == 0 ) {
    return 0;
  }
  // A smaller batch gets more splits per context, and batch * splits does not grow with the batch:
  // the buffer has to hold the largest need of any batch in [1, batch].  The generic kernel splits
  // per query head and may use more splits than the fast ones; size for the larger of the two.
  uint64_t floats = 0;
  for ( uint64_t b = 1; b <= batch; b++ ) {
    const Plan fast = make_plan( b, max_pos, shape, GH_F16, GH_ATTN_AUTO );
    const Plan generic = make_plan( b, max_pos, shape, GH_F32, GH_ATTN_GENERIC );
    floats = std::max( floats, partial_floats( b, shape, std::max( fast.split_bound, generic.split_bound ) ) );
  }
  return floats * sizeof( float ) + 256;
}

int gh_attn_decode_plan( uint64_t batch, uint32_t max_pos, const gh_shape* shape, gh_dtype dt, int variant, uint32_t* tokens_per_split, uint32_t* max_splits,
                         uint64_t* partial_bytes )
{
  GH_REQUIRE( shape != nullptr && batch > 0, "gh_attn_decode_plan: bad arguments" );
  GH_REQUIRE( variant >= GH_ATTN_AUTO && variant <= GH_ATTN_MFMA, "gh_attn_decode_plan: unknown variant %d", variant );
  const Plan plan = make_plan( batch, max_pos, shape, dt, variant );
  if ( tokens_per_split ) {
    *tokens_per_split = plan.chunk;
  }
  if ( max_splits ) {
    *max_splits = plan.max_splits;
  }
  if ( partial_bytes ) {
    *partial_bytes = plan.max_splits > 1 && plan.join == 0 ? partial_floats( batch, shape, plan.max_splits ) * sizeof( float ) : 0;
  }
  return GH_OK;
}

uint32_t gh_attn_decode_join_waves( uint64_t batch, uint32_t max_pos, const gh_shape* shape, gh_dtype dt, int variant )
{
  if ( shape == nullptr || batch == 0 || variant < GH_ATTN_AUTO || variant > GH_ATTN_MFMA ) {
    return 0;
  }
  return make_plan( batch, max_pos, shape, dt, variant ).join;
}

// Shared by gh_attn_decode (partials in the caller's workspace, kernel timer on request) and
// gh_attn_decode_static (partials in this GPU's `scratch` array; nothing here allocates when `timed` is false).
static int attn_decode_run( const char* who, const void* q, const void* const* layer_rows_dev, const uint32_t* pos_dev, void* xb, uint64_t batch,
                            uint32_t max_pos, const gh_shape* shape, gh_dtype dt, void* workspace, uint64_t workspace_bytes, int variant,
                            gh_stream stream, bool timed )
{
  GH_REQUIRE( shape != nullptr, "gh_attn_decode: NULL shape" );
  GH_REQUIRE( q && layer_rows_dev && pos_dev && xb, "gh_attn_decode: NULL pointer" );
  GH_REQUIRE( dt == GH_F16 || dt == GH_F32, "gh_attn_decode: unsupported dtype %d", (int)dt );
  GH_REQUIRE( shape->n_kv_heads > 0 && shape->gqa_size > 0 && shape->head_size > 0 && shape->seq_len > 0, "gh_attn_decode: zero dimension" );
  GH_REQUIRE( shape->n_heads == shape->n_kv_heads * shape->gqa_size, "gh_attn_decode: n_heads != n_kv_heads * gqa_size" );
  GH_REQUIRE( shape->kv_dim == shape->n_kv_heads * shape->head_size, "gh_attn_decode: kv_dim != n_kv_heads * head_size" );
  GH_REQUIRE( shape->head_size <= 256, "gh_attn_decode: head_size %u > 256", shape->head_size );
  GH_REQUIRE( max_pos < shape->seq_len, "gh_attn_decode: max_pos %u outside seq_len %u", max_pos, shape->seq_len );
  GH_REQUIRE( batch <= 65535, "gh_attn_decode: batch too large" );
  GH_REQUIRE( variant >= GH_ATTN_AUTO && variant <= GH_ATTN_MFMA, "gh_attn_decode: unknown variant %d", variant );
  if ( variant == GH_ATTN_VALU ) {
    GH_REQUIRE( fast_ok( shape, dt ) && valu_gqa_ok( shape->gqa_size ), "gh_attn_decode: the valu kernel needs f16, head_size 128, gqa in {1,2,4,8}" );
  }
  if ( variant == GH_ATTN_MFMA ) {
    GH_REQUIRE( fast_ok( shape, dt ) && mfma_gqa_ok( shape->gqa_size ), "gh_attn_decode: the mfma kernel needs f16, head_size 128, gqa in {2,4,8,16}" );
  }
  if ( dt == GH_F16 && shape->head_size == HS ) {
    GH_REQUIRE( ( reinterpret_cast<uintptr_t>( q ) & 15u ) == 0 && ( reinterpret_cast<uintptr_t>( xb ) & 15u ) == 0,
                "gh_attn_decode: q and xb must be 16-byte aligned" );
  }

  const Plan plan = make_plan( batch, max_pos, shape, dt, variant );
  const uint32_t join = plan.join; // > 0: no partial sums in memory, no merge kernel
  const bool joined = join > 0;
  Partials part { nullptr, nullptr };
  if ( plan.max_splits > 1 && !joined ) {
    const uint64_t need = partial_floats( batch, shape, plan.max_splits ) * sizeof( float );
    GH_REQUIRE( workspace != nullptr, "%s: workspace required (%llu bytes)", who, (unsigned long long)need );
    if ( workspace_bytes < need ) {
      return fail( GH_ERR_WORKSPACE, "%s: %llu bytes of split partials needed, %llu available", who, (unsigned long long)need,
                   (unsigned long long)workspace_bytes );
    }
    GH_REQUIRE( ( reinterpret_cast<uintptr_t>( workspace ) & 15u ) == 0, "gh_attn_decode: workspace must be 16-byte aligned" );
    part.out = static_cast<float*>( workspace );
    part.ml = part.out + batch * shape->n_heads * (uint64_t)plan.max_splits * shape->head_size;
  }

  hipStream_t st = as_stream( stream );
  const float scale = LOG2E / sqrtf( (float)shape->head_size );
  int timer = -1;
  if ( timed ) {
    if ( int rc = timer_mark( st, &timer, 0 ) ) {
      return rc;
    }
  }

  if ( plan.variant == GH_ATTN_GENERIC ) {
    const dim3 grid( shape->n_heads, plan.max_splits, (unsigned)batch );
    if ( dt == GH_F16 ) {
      attn_decode_generic_kernel<__half><<<grid, 64, 0, st>>>( static_cast<const __half*>( q ), reinterpret_cast<const __half* const*>( layer_rows_dev ),
                                                              pos_dev, part, static_cast<__half*>( xb ), shape->n_kv_heads, shape->gqa_size,
                                                              shape->head_size, plan.chunk, plan.max_splits, scale );
    } else {
      attn_decode_generic_kernel<float><<<grid, 64, 0, st>>>( static_cast<const float*>( q ), reinterpret_cast<const float* const*>( layer_rows_dev ),
                                                             pos_dev, part, static_cast<float*>( xb ), shape->n_kv_heads, shape->gqa_size,
                                                             shape->head_size, plan.chunk, plan.max_splits, scale );
    }
  } else if ( joined ) {
    const uint32_t heads_per_group = join / plan.max_splits;
    const uint64_t n_blocks = batch * ( ( shape->n_kv_heads + heads_per_group - 1 ) / heads_per_group );
    GH_REQUIRE( n_blocks <= 0x7fffffffull, "gh_attn_decode: grid too large" );
    const dim3 grid( (unsigned)n_blocks );
    if ( plan.variant == GH_ATTN_VALU ) {
      switch ( shape->gqa_size ) {
        case 1: launch_valu_joined<1>( join, grid, st, q, layer_rows_dev, pos_dev, xb, shape, plan, (uint32_t)batch, scale ); break;
        case 2: launch_valu_joined<2>( join, grid, st, q, layer_rows_dev, pos_dev, xb, shape, plan, (uint32_t)batch, scale ); break;
        case 4: launch_valu_joined<4>( join, grid, st, q, layer_rows_dev, pos_dev, xb, shape, plan, (uint32_t)batch, scale ); break;
        default: launch_valu_joined<8>( join, grid, st, q, layer_rows_dev, pos_dev, xb, shape, plan, (uint32_t)batch, scale ); break;
      }
    } else {
      switch ( shape->gqa_size ) {
        case 2: launch_mfma_joined<2>( join, grid, st, q, layer_rows_dev, pos_dev, xb, shape, plan, (uint32_t)batch, scale ); break;
        case 4: launch_mfma_joined<4>( join, grid, st, q, layer_rows_dev, pos_dev, xb, shape, plan, (uint32_t)batch, scale ); break;
        case 8: launch_mfma_joined<8>( join, grid, st, q, layer_rows_dev, pos_dev, xb, shape, plan, (uint32_t)batch, scale ); break;
        default: launch_mfma_joined<16>( join, grid, st, q, layer_rows_dev, pos_dev, xb, shape, plan, (uint32_t)batch, scale ); break;
      }
    }
  } else {
    const uint64_t n_blocks = batch * plan.max_splits * ( ( shape->n_kv_heads + 3 ) / 4 );
    GH_REQUIRE( n_blocks <= 0x7fffffffull, "gh_attn_decode: grid too large" );
    const dim3 grid( (unsigned)n_blocks );
    if ( plan.variant == GH_ATTN_VALU ) {
      switch ( shape->gqa_size ) {
        case 1: launch_valu<1>( grid, st, q, layer_rows_dev, pos_dev, part, xb, shape, plan, scale ); break;
        case 2: launch_valu<2>( grid, st, q, layer_rows_dev, pos_dev, part, xb, shape, plan, scale ); break;
        case 4: launch_valu<4>( grid, st, q, layer_rows_dev, pos_dev, part, xb, shape, plan, scale ); break;
        default: launch_valu<8>( grid, st, q, layer_rows_dev, pos_dev, part, xb, shape, plan, scale ); break;
      }
    } else {
      switch ( shape->gqa_size ) {
        case 2: launch_mfma<2>( grid, st, q, layer_rows_dev, pos_dev, part, xb, shape, plan, scale ); break;
        case 4: launch_mfma<4>( grid, st, q, layer_rows_dev, pos_dev, part, xb, shape, plan, scale ); break;
        case 8: launch_mfma<8>( grid, st, q, layer_rows_dev, pos_dev, part, xb, shape, plan, scale ); break;
        default: launch_mfma<16>( grid, st, q, layer_rows_dev, pos_dev, part, xb, shape, plan, scale ); break;
      }
    }
  }
  GH_LAUNCH_CHECK();
  if ( timed ) {
    if ( int rc = timer_mark( st, &timer, 1 ) ) {
      return rc;
    }
  }

  if ( plan.max_splits > 1 && !joined ) {
    const dim3 grid( shape->n_heads, (unsigned)batch );
    const unsigned threads = shape->head_size <= 64 ? 64 : ( shape->head_size <= 128 ? 128 : 256 );
    if ( dt == GH_F16 ) {
      attn_merge_kernel<__half><<<grid, threads, 0, st>>>( part, layer_rows_dev, pos_dev, static_cast<__half*>( xb ), shape->n_heads,
                                                          shape->head_size, plan.chunk, plan.max_splits );
    } else {
      attn_merge_kernel<float><<<grid, threads, 0, st>>>( part, layer_rows_dev, pos_dev, static_cast<float*>( xb ), shape->n_heads,
                                                         shape->head_size, plan.chunk, plan.max_splits );
    }
    GH_LAUNCH_CHECK();
  }
  return timed ? timer_mark( st, &timer, 2 ) : GH_OK;
}

int gh_attn_decode( const void* q, const void* const* layer_rows_dev, const uint32_t* pos_dev, void* xb, uint64_t batch,
                    uint32_t max_pos, const gh_shape* shape, gh_dtype dt, void* workspace, uint64_t workspace_bytes,
                    int variant, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  return attn_decode_run( "gh_attn_decode", q, layer_rows_dev, pos_dev, xb, batch, max_pos, shape, dt, workspace, workspace_bytes, variant, stream, true );
}

uint64_t gh_attn_decode_static_limit( void ) { return STATIC_SCRATCH_BYTES; }

int gh_attn_decode_static( const void* q, const void* const* layer_rows_dev, const uint32_t* pos_dev, void* xb, uint64_t batch, uint32_t max_pos,
                           const gh_shape* shape, gh_dtype dt, int variant, gh_stream stream )
{
  // no ensure_init() here: initialisation allocates (staging ring), so it has to have happened in gh_init()
  const int device = initialised_device();
  GH_REQUIRE( device >= 0, "gh_attn_decode_static: the library is not initialised; call gh_init() first (this entry point allocates nothing)" );
  GH_REQUIRE( device < MAX_DEVICES && g_static_scratch[device] != nullptr, "gh_attn_decode_static: no scratch array on device %d", device );
  int current = -1; // every GPU holds its own copy of the array at its own address: the kernels must run where that address is valid
  GH_REQUIRE( hipGetDevice( &current ) == hipSuccess && current == device,
              "gh_attn_decode_static: the calling thread's current device is %d, the library was initialised on device %d", current, device );
  if ( batch == 0 ) {
    return GH_OK;
  }
  // a plan that needs more partials than the array holds is refused by the size check of the shared path (GH_ERR_WORKSPACE)
  return attn_decode_run( "gh_attn_decode_static", q, layer_rows_dev, pos_dev, xb, batch, max_pos, shape, dt, g_static_scratch[device],
                          STATIC_SCRATCH_BYTES, variant, stream, false );
}

uint64_t gh_attn_balanced_workspace( uint64_t batch, const gh_shape* shape )
{
  if ( shape == nullptr || batch == 0 || shape->n_kv_heads == 0 || ensure_init() != GH_OK ) {
    return 0;
  }
  return balanced_layout( batch, shape ).total_bytes;
}

int gh_attn_balance( const void* const* layer_rows_dev, const uint32_t* pos_dev, uint64_t batch, uint32_t max_pos, const gh_shape* shape, void* workspace,
                     uint64_t workspace_bytes, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( layer_rows_dev && pos_dev, "gh_attn_balance: NULL pointer" );
  if ( int rc = balanced_check( "gh_attn_balance", batch, max_pos, shape, workspace, workspace_bytes ) ) {
    return rc;
  }
  const BalancedLayout y = balanced_layout( batch, shape );
  attn_balance_kernel<<<1, BAL_PLAN_THREADS, 0, as_stream( stream )>>>( layer_rows_dev, pos_dev, (uint32_t)batch, max_pos + 1, y.wgs,
                                                                        balanced_plan( workspace, batch ) );
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_attn_decode_balanced( const void* q, const void* const* layer_rows_dev, void* xb, uint64_t batch, uint32_t max_pos, const gh_shape* shape, gh_dtype dt,
                             void* workspace, uint64_t workspace_bytes, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( q && layer_rows_dev && xb, "gh_attn_decode_balanced: NULL pointer" );
  GH_REQUIRE( dt == GH_F16, "gh_attn_decode_balanced: f16 only" );
  GH_REQUIRE( ( reinterpret_cast<uintptr_t>( q ) & 15u ) == 0 && ( reinterpret_cast<uintptr_t>( xb ) & 15u ) == 0,
              "gh_attn_decode_balanced: q and xb must be 16-byte aligned" );
  if ( int rc = balanced_check( "gh_attn_decode_balanced", batch, max_pos, shape, workspace, workspace_bytes ) ) {
    return rc;
  }
  const BalancedLayout y = balanced_layout( batch, shape );
  const BalancedPlan plan = balanced_plan( workspace, batch );
  Partials part;
  part.out = reinterpret_cast<float*>( static_cast<char*>( workspace ) + y.plan_bytes );
  part.ml = part.out + y.out_floats;
  const float scale = LOG2E / sqrtf( (float)shape->head_size );
  hipStream_t st = as_stream( stream );
  switch ( shape->gqa_size ) {
    case 1: launch_balanced<1, false>( y, st, q, layer_rows_dev, plan, part, xb, shape, batch, scale ); break; // one query head per kv head: dot products
    case 2: launch_balanced<2, true>( y, st, q, layer_rows_dev, plan, part, xb, shape, batch, scale ); break;
    case 4: launch_balanced<4, true>( y, st, q, layer_rows_dev, plan, part, xb, shape, batch, scale ); break;
    case 8: launch_balanced<8, true>( y, st, q, layer_rows_dev, plan, part, xb, shape, batch, scale ); break;
    default: launch_balanced<16, true>( y, st, q, layer_rows_dev, plan, part, xb, shape, batch, scale ); break;
  }
  GH_LAUNCH_CHECK();
  return GH_OK;
}

int gh_attn_decode_host( const void* q, const void* const* layer_rows_host, const uint32_t* pos_host, void* xb, uint64_t batch,
                         const gh_shape* shape, gh_dtype dt, void* workspace, uint64_t workspace_bytes, int variant, gh_stream stream )
{
  if ( int rc = ensure_init() ) {
    return rc;
  }
  if ( batch == 0 ) {
    return GH_OK;
  }
  GH_REQUIRE( layer_rows_host && pos_host, "gh_attn_decode_host: NULL table" );
  GH_REQUIRE( batch <= MAX_BATCH, "gh_attn_decode_host: batch %llu > %llu", (unsigned long long)batch, (unsigned long long)MAX_BATCH );
  uint32_t max_pos = 0;
  for ( uint64_t i = 0; i < batch; i++ ) {
    if ( layer_rows_host[i] != nullptr ) {
      max_pos = std::max( max_pos, pos_host[i] );
    }
  }
  void* d_rows = nullptr;
  void* d_pos = nullptr;
  StageScope scope( as_stream( stream ) );
  if ( int rc = stage_table( layer_rows_host, batch * sizeof( void* ), as_stream( stream ), &d_rows ) ) {
    return rc;
  }
  if ( int rc = stage_table( pos_host, batch * sizeof( uint32_t ), as_stream( stream ), &d_pos ) ) {
    return rc;
  }
  if ( int rc = gh_attn_decode( q, static_cast<const void* const*>( d_rows ), static_cast<const uint32_t*>( d_pos ), xb, batch, max_pos, shape, dt,
                                workspace, workspace_bytes, variant, stream ) ) {
    return rc;
  }
  return scope.finish();
}

} // extern "C"
