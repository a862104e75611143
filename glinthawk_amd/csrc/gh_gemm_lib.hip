// Plain products of many activation rows through the vendor's GEMM library (hipBLASLt), as the reference's GPU target sends
// every product through its vendor library (cublasGemmEx, arch/cuda/common/ops.cuh:666-700: op(W) = T, op(x) = N,
// m = r, n = b, k = s, fp32 compute type).  Same operands, same layout, same call here: xout(b, r) row-major is the
// column-major C(m = r, n = b).  An opt-in route (gh_gemm_set_library_rows, off by default): on this part the library's kernels
// reach 1.22-1.50 PFLOP/s at 3328 and more rows where the tile kernels of this library reach 1.13-1.34, so a caller may hand it
// the products that are nothing but a product; what is fused with an epilogue, split along K or shaped for decode stays on the
// kernels of this library either way.
//
// The library is opened at the first such product, not linked: without it (or without an algorithm for a shape) the call is
// declined and the dispatcher goes on to its own tile kernels.
#include "gh_common.h"

#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <atomic>
#include <map>
#include <mutex>
#include <tuple>

namespace gh {

namespace {

struct Api
{
  decltype( &hipblasLtCreate ) create = nullptr;
  decltype( &hipblasLtMatmulDescCreate ) desc_create = nullptr;
  decltype( &hipblasLtMatmulDescSetAttribute ) desc_set = nullptr;
  decltype( &hipblasLtMatrixLayoutCreate ) layout_create = nullptr;
  decltype( &hipblasLtMatmulPreferenceCreate ) pref_create = nullptr;
  decltype( &hipblasLtMatmulPreferenceSetAttribute ) pref_set = nullptr;
  decltype( &hipblasLtMatmulPreferenceDestroy ) pref_destroy = nullptr;
  decltype( &hipblasLtMatmulAlgoGetHeuristic ) heuristic = nullptr;
  decltype( &hipblasLtMatmul ) matmul = nullptr;
  hipblasLtHandle_t handle = nullptr;
  bool tried = false, ok = false;
};

struct Product
{
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, out = nullptr;
  hipblasLtMatmulAlgo_t algo {};
  uint64_t workspace = 0;
  bool ok = false;
};

constexpr uint64_t LIB_WORKSPACE = 64ull << 20;
constexpr size_t MAX_PRODUCTS = 256; // shapes whose descriptors and algorithm are kept (a stage has a handful)

std::mutex g_lib_mutex;
std::atomic<uint64_t> g_library_calls { 0 }; // products the library has run
Api g_api;
std::map<std::tuple<uint64_t, uint64_t, uint64_t>, Product> g_products; // (s, r, b); kept until the process ends

template<typename F>
bool symbol( void* lib, const char* name, F& out )
{
  out = reinterpret_cast<F>( dlsym( lib, name ) );
  return out != nullptr;
}

bool open_library()
{
  if ( g_api.tried ) {
    return g_api.ok;
  }
  g_api.tried = true;
  void* lib = dlopen( "libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL );
  if ( lib == nullptr ) {
    lib = dlopen( "libhipblaslt.so", RTLD_NOW | RTLD_LOCAL );
  }
  if ( lib == nullptr ) {
    return false;
  }
  Api& a = g_api;
  if ( !( symbol( lib, "hipblasLtCreate", a.create ) && symbol( lib, "hipblasLtMatmulDescCreate", a.desc_create )
          && symbol( lib, "hipblasLtMatmulDescSetAttribute", a.desc_set ) && symbol( lib, "hipblasLtMatrixLayoutCreate", a.layout_create )
          && symbol( lib, "hipblasLtMatmulPreferenceCreate", a.pref_create ) && symbol( lib, "hipblasLtMatmulPreferenceSetAttribute", a.pref_set )
          && symbol( lib, "hipblasLtMatmulPreferenceDestroy", a.pref_destroy ) && symbol( lib, "hipblasLtMatmulAlgoGetHeuristic", a.heuristic )
          && symbol( lib, "hipblasLtMatmul", a.matmul ) ) ) {
    return false;
  }
  if ( a.create( &a.handle ) != HIPBLAS_STATUS_SUCCESS ) {
    return false;
  }
  a.ok = true;
  return true;
}

const Product& product_for( uint64_t s, uint64_t r, uint64_t b )
{
  static const Product declined {};
  if ( g_products.size() >= MAX_PRODUCTS && g_products.find( { s, r, b } ) == g_products.end() ) {
    return declined; // a caller with ever new shapes: the descriptors kept so far stay, further shapes run on the tile kernels
  }
  Product& p = g_products[{ s, r, b }];
  if ( p.desc != nullptr || !g_api.ok ) {
    return p; // made before (p.ok says how that went)
  }
  const Api& a = g_api;
  if ( a.desc_create( &p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F ) != HIPBLAS_STATUS_SUCCESS ) {
    return p;
  }
  const hipblasOperation_t t = HIPBLAS_OP_T, n = HIPBLAS_OP_N;
  bool good = a.desc_set( p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &t, sizeof( t ) ) == HIPBLAS_STATUS_SUCCESS
              && a.desc_set( p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &n, sizeof( n ) ) == HIPBLAS_STATUS_SUCCESS;
  // column-major: W as stored is (k = s) x (m = r) with leading dimension s, x is (s) x (n = b), the output (r) x (b)
  good = good && a.layout_create( &p.w, HIP_R_16F, s, r, (int64_t)s ) == HIPBLAS_STATUS_SUCCESS
         && a.layout_create( &p.x, HIP_R_16F, s, b, (int64_t)s ) == HIPBLAS_STATUS_SUCCESS
         && a.layout_create( &p.out, HIP_R_16F, r, b, (int64_t)r ) == HIPBLAS_STATUS_SUCCESS;
  hipblasLtMatmulPreference_t pref = nullptr;
  good = good && a.pref_create( &pref ) == HIPBLAS_STATUS_SUCCESS;
  if ( good ) {
    const uint64_t room = LIB_WORKSPACE;
    good = a.pref_set( pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &room, sizeof( room ) ) == HIPBLAS_STATUS_SUCCESS;
    hipblasLtMatmulHeuristicResult_t found {};
    int n_found = 0;
    good = good && a.heuristic( a.handle, p.desc, p.w, p.x, p.out, p.out, pref, 1, &found, &n_found ) == HIPBLAS_STATUS_SUCCESS && n_found > 0
           && found.state == HIPBLAS_STATUS_SUCCESS && found.workspaceSize <= LIB_WORKSPACE;
    if ( good ) {
      p.algo = found.algo;
      p.workspace = found.workspaceSize;
    }
  }
  if ( pref != nullptr ) {
    a.pref_destroy( pref );
  }
  p.ok = good;
  return p;
}

} // namespace

// Whether gemm_library() would run this product: the library opens and has an algorithm for the shape.  Lets a caller that needs a
// buffer for the product allocate it only then.
bool gemm_library_available( uint64_t s, uint64_t r, uint64_t b )
{
  std::lock_guard<std::mutex> lock( g_lib_mutex );
  return open_library() && product_for( s, r, b ).ok;
}

// xout(b, r) = x(b, s) . w(r, s)^T, f16 storage, fp32 sums rounded once.  *done = false: declined (no library, no algorithm):
// nothing was queued.
int gemm_library( void* xout, const void* x, const void* w, uint64_t s, uint64_t r, uint64_t b, hipStream_t st, bool* done )
{
  *done = false;
  Product p;
  {
    // the lock covers the table of descriptors only: a product's descriptors are never changed or dropped once made, and the
    // library's handle may be used from several threads at once, so stage threads do not queue behind each other's products
    std::lock_guard<std::mutex> lock( g_lib_mutex );
    if ( !open_library() ) {
      return GH_OK;
    }
    p = product_for( s, r, b );
  }
  if ( !p.ok ) {
    return GH_OK;
  }
  void* room = nullptr;
  if ( p.workspace > 0 ) {
    if ( int rc = stream_scratch( st, SCRATCH_LIBRARY, p.workspace, LIB_WORKSPACE, &room ) ) {
      return rc;
    }
  }
  const float one = 1.0f, zero = 0.0f;
  const hipblasStatus_t status = g_api.matmul( g_api.handle, p.desc, &one, w, p.w, x, p.x, &zero, xout, p.out, xout, p.out, &p.algo, room, p.workspace, st );
  if ( status != HIPBLAS_STATUS_SUCCESS ) {
    return fail( GH_ERR_DEVICE, "gemm_library: hipblasLtMatmul failed with status %d for %llu x %llu x %llu", (int)status, (unsigned long long)b,
                 (unsigned long long)s, (unsigned long long)r );
  }
  g_library_calls++;
  *done = true;
  return GH_OK;
}

} // namespace gh

extern "C" uint64_t gh_gemm_library_calls( void ) { return gh::g_library_calls.load(); }
