/* och_gemm entry point, argument checks, and the generic tiled kernel for bool, integers and
 * half (solid/src/core/gpu/template_blas.cu:99-160 uses one thread per element of C and a
 * square LDS tile; here each thread owns a 4 x 4 patch of a 64 x 64 tile).
 * bool: + is OR, * is AND. Integers wrap. half multiplies and accumulates in float. */
#include "och_gemm.h"
#include <atomic>
#include "../../include/ocean_hip.h"

namespace och {

template <class T> struct GemmElem;     /* W: LDS / accumulator type */
template <class T, class WT> struct GemmInt
{  typedef WT W;
   static __device__ W load(T x) { return (W)x; }
   static __device__ W fma(W s, W a, W b) { return (W)(s + a * b); }
   static __device__ T finish(W s, W alpha, W beta, T c) { return (T)(W)(alpha * s + beta * (W)c); }
};
template <> struct GemmElem<uint8_t>  : GemmInt<uint8_t, uint32_t> {};
template <> struct GemmElem<uint16_t> : GemmInt<uint16_t, uint32_t> {};
template <> struct GemmElem<uint32_t> : GemmInt<uint32_t, uint32_t> {};
template <> struct GemmElem<uint64_t> : GemmInt<uint64_t, uint64_t> {};
template <> struct GemmElem<int8_t>   : GemmInt<int8_t, uint32_t> {};
template <> struct GemmElem<int16_t>  : GemmInt<int16_t, uint32_t> {};
template <> struct GemmElem<int32_t>  : GemmInt<int32_t, uint32_t> {};
template <> struct GemmElem<int64_t>  : GemmInt<int64_t, uint64_t> {};
template <> struct GemmElem<obool>
{  typedef uint32_t W;
   static __device__ W load(obool x) { return x.v ? 1u : 0u; }
   static __device__ W fma(W s, W a, W b) { return s | (a & b); }
   static __device__ obool finish(W s, W alpha, W beta, obool c) { obool r; r.v = ((s & alpha) | (beta & (c.v ? 1u : 0u))) ? 1 : 0; return r; }
};
template <> struct GemmElem<half_t>
{  typedef float W;
   static __device__ W load(half_t x) { return half_to_float(x); }
   static __device__ W fma(W s, W a, W b) { return s + a * b; }
   static __device__ half_t finish(W s, W alpha, W beta, half_t c)
   {  float v = alpha * s;
      if (beta != 0) v += beta * half_to_float(c);
      return float_to_half(v);
   }
};

#define GT 64      /* tile edge */
#define GK 16      /* K slab */
template <class T>
__global__ __launch_bounds__(256) void gemm_generic_kernel(uint32_t M, uint32_t N, uint32_t K,
      T alpha_host, T beta_host, const T *alpha_dev, const T *beta_dev,
      const T *A, int64_t sAm, int64_t sAk, const T *B, int64_t sBk, int64_t sBn, T *C, int64_t ldC, const GemmBatch batch)
{
   typedef GemmElem<T> E; typedef typename E::W W;
   {  int64_t oA, oB, oC, oAlpha, oBeta;
      gemm_batch_offsets(batch, oA, oB, oC, oAlpha, oBeta);
      A = reinterpret_cast<const T *>(reinterpret_cast<const char *>(A) + oA);
      B = reinterpret_cast<const T *>(reinterpret_cast<const char *>(B) + oB);
      C = reinterpret_cast<T *>(reinterpret_cast<char *>(C) + oC);
      if (alpha_dev) alpha_dev = reinterpret_cast<const T *>(reinterpret_cast<const char *>(alpha_dev) + oAlpha);
      if (beta_dev)  beta_dev  = reinterpret_cast<const T *>(reinterpret_cast<const char *>(beta_dev) + oBeta);
   }
   __shared__ W As[GK][GT + 1], Bs[GK][GT + 1];
   const uint32_t tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
   const uint32_t m0 = blockIdx.x * GT, n0 = blockIdx.y * GT;
   W acc[4][4];
#pragma unroll
   for (int i = 0; i < 4; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) acc[i][j] = 0;
   for (uint32_t k0 = 0; k0 < K; k0 += GK)
   {
#pragma unroll
      for (int v = 0; v < 4; v++)
      {  const uint32_t q = threadIdx.x + 256 * v;
         const uint32_t mm = q % GT, kk = q / GT;
         const uint32_t gm = m0 + mm, gn = n0 + mm, gk = k0 + kk;
         As[kk][mm] = (gm < M && gk < K) ? E::load(A[(int64_t)gm * sAm + (int64_t)gk * sAk]) : (W)0;
         Bs[kk][mm] = (gn < N && gk < K) ? E::load(B[(int64_t)gk * sBk + (int64_t)gn * sBn]) : (W)0;
      }
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < GK; kk++)
      {  W a[4], b[4];
#pragma unroll
         for (int i = 0; i < 4; i++) { a[i] = As[kk][tx + 16 * i]; b[i] = Bs[kk][ty + 16 * i]; }
#pragma unroll
         for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = E::fma(acc[i][j], a[i], b[j]);
      }
      __syncthreads();
   }
   const W alpha = E::load(alpha_dev ? *alpha_dev : alpha_host), beta = E::load(beta_dev ? *beta_dev : beta_host);
#pragma unroll
   for (int j = 0; j < 4; j++)
#pragma unroll
      for (int i = 0; i < 4; i++)
      {  const uint32_t row = m0 + tx + 16 * i, col = n0 + ty + 16 * j;
         if (row < M && col < N)
         {  T *c = C + (int64_t)row + (int64_t)col * ldC;
            *c = E::finish(acc[i][j], alpha, beta, *c);
         }
      }
}

template <class T> static int gemm_generic(const GemmArgs &g)
{
   T alpha, beta; memset(&alpha, 0, sizeof(T)); memset(&beta, 0, sizeof(T));
   const T *adev = nullptr, *bdev = nullptr;
   if (g.scalar_mode_host) { memcpy(&alpha, g.alpha, sizeof(T)); memcpy(&beta, g.beta, sizeof(T)); }
   else { adev = (const T *)g.alpha; bdev = (const T *)g.beta; }
   const bool ta = (g.transA != 'N'), tb = (g.transB != 'N');
   const int64_t sAm = ta ? g.ldA : 1, sAk = ta ? 1 : g.ldA, sBk = tb ? g.ldB : 1, sBn = tb ? 1 : g.ldB;
   const uint64_t gx = (g.M + GT - 1) / GT, gy = (g.N + GT - 1) / GT;
   if (gy > 65535) return set_error("gemm: N = %zu is too large for this data type", g.N);
   hipLaunchKernelGGL((gemm_generic_kernel<T>), dim3((unsigned)gx, (unsigned)gy, g.nz), dim3(256), 0, g.stream,
                      (uint32_t)g.M, (uint32_t)g.N, (uint32_t)g.K, alpha, beta, adev, bdev,
                      (const T *)g.A, sAm, sAk, (const T *)g.B, sBk, sBn, (T *)g.C, (int64_t)g.ldC, g.batch);
   OCH_CHECK_LAUNCH();
   return 0;
}

/* dst (d0 x d1, dense, column-major) <- the v0 x v1 corner of src (leading dimension ld), zero elsewhere; elements of
   sizeof(E) bytes */
template <class E>
__global__ __launch_bounds__(256) void gemm_pad_kernel(E *dst, const E *src, uint32_t d0, uint64_t total, uint32_t v0, uint32_t v1, int64_t ld)
{
   const uint64_t e = (uint64_t)blockIdx.x * 256 + threadIdx.x;
   if (e >= total) return;
   const uint32_t j = (uint32_t)(e / d0), i = (uint32_t)(e - (uint64_t)j * d0);
   E v = E();
   if (i < v0 && j < v1) v = src[i + (int64_t)j * ld];
   dst[e] = v;
}

/* The last K - Kh (< slab) of the inner dimension as a product of one whole slab: both operands' tails are copied into
   the stream's workspace and filled up with zeros to `slab` k (the pipelined kernels take whole slabs only), laid out as
   the operands themselves are, so that *tail = g with A, B, their leading dimensions and K replaced multiplies them with
   the same transposition flags. es: bytes per element. 0: done; 1: the copies do not fit into the workspace. */
int gemm_pad_tail(const GemmArgs &g, size_t Kh, int slab, int es, GemmArgs *tail)
{
   const size_t kt = g.K - Kh;
   const size_t bytesA = g.M * (size_t)slab * es, bytesB = g.N * (size_t)slab * es;
   if (g.batch.nb != 0 || g.nz != 1 || bytesA + bytesB > OCH_GEMM_WORKSPACE) return 1;
   char *ws;
   if (stream_gemm_workspace(g.stream, &ws) != 0) return -1;
   *tail = g;
   tail->K = (size_t)slab;
   for (int operand = 0; operand < 2; operand++)
   {  /* rows contiguous (A not transposed, B transposed): rows x slab, the tail's columns first; k contiguous: slab x rows */
      const bool rows_contiguous = operand == 0 ? (g.transA == 'N') : (g.transB != 'N');
      const size_t rows = operand == 0 ? g.M : g.N;
      const ptrdiff_t ld = operand == 0 ? g.ldA : g.ldB;
      const char *src = (const char *)(operand == 0 ? g.A : g.B) + (int64_t)Kh * (rows_contiguous ? (int64_t)ld : 1) * es;
      char *dst = ws + (operand == 0 ? 0 : bytesA);
      const uint32_t d0 = (uint32_t)(rows_contiguous ? rows : (size_t)slab), v0 = (uint32_t)(rows_contiguous ? rows : kt), v1 = (uint32_t)(rows_contiguous ? kt : rows);
      const uint64_t total = (uint64_t)rows * slab;
      const dim3 grid((unsigned)((total + 255) / 256)), block(256);
      if (es == 4)      hipLaunchKernelGGL(gemm_pad_kernel<uint32_t>, grid, block, 0, g.stream, (uint32_t *)dst, (const uint32_t *)src, d0, total, v0, v1, (int64_t)ld);
      else if (es == 8) hipLaunchKernelGGL(gemm_pad_kernel<uint64_t>, grid, block, 0, g.stream, (uint64_t *)dst, (const uint64_t *)src, d0, total, v0, v1, (int64_t)ld);
      else              hipLaunchKernelGGL(gemm_pad_kernel<uint4>, grid, block, 0, g.stream, (uint4 *)dst, (const uint4 *)src, d0, total, v0, v1, (int64_t)ld);
      if (operand == 0) { tail->A = dst; tail->ldA = (ptrdiff_t)d0; } else { tail->B = dst; tail->ldB = (ptrdiff_t)d0; }
   }
   OCH_CHECK_LAUNCH();
   return 0;
}

/* 0: the cost model chooses; 1: the pipelined kernel on its large tile wherever it applies; 2: on its small tile (float,
   double); 3: never the pipelined kernel; 4: on its smallest tile (float; the other types: the tile the model prefers). For tests and measurements (och_gemm_set_kernel_choice). */
static std::atomic<int> g_gemm_kernel_choice{0};
int gemm_kernel_choice(void) { return g_gemm_kernel_choice.load(std::memory_order_relaxed); }

/* The last round of a pipelined product. `units` compute units work through tiles x batch block tiles in rounds, and
   a last round of `rest` tiles takes as long as a full one. When it is at most half full (and the product is a single one,
   not an entry of a batch, with at least 16 slabs of K) its tiles are cut along K into shares that fill the round: at most 8 per tile -- 64 when
   the whole product is less than one round -- each of at least 8 slabs, none empty, together within the stream's
   workspace (every share leaves tile_m x tile_n raw sums of elem_size bytes there); no cut that would still leave most
   of the units idle. Returns the shares per tile (1: no cut). *rounds: what the product costs in rounds of whole tiles,
   the cut round counted by the length of a share plus six slabs of fixed cost per block. Host arithmetic only. */
int gemm_pipe_split_plan(uint64_t M, uint64_t N, uint64_t K, uint64_t batch, bool single, uint32_t tile_m, uint32_t tile_n,
                         uint32_t slab, uint32_t elem_size, uint64_t units, double *rounds)
{
   if (tile_m == 0 || tile_n == 0 || slab == 0 || elem_size == 0 || units == 0) { if (rounds) *rounds = 0.0; return 1; }
   const uint64_t tiles = ((M + tile_m - 1) / tile_m) * ((N + tile_n - 1) / tile_n) * batch;
   const uint64_t rest = tiles % units, slabs = K / slab;
   uint64_t shares = 1;
   if (single && batch == 1 && rest > 0 && rest * 2 <= units && slabs >= 16)
   {  shares = units / rest;
      if (shares > (tiles < units ? 64 : 8)) shares = tiles < units ? 64 : 8;
      if (shares > slabs / 8) shares = slabs / 8;
      const uint64_t fit = OCH_GEMM_WORKSPACE / (rest * (uint64_t)tile_m * tile_n * elem_size);
      if (shares > fit) shares = fit;
      while (shares > 1 && ((slabs + shares - 1) / shares) * (shares - 1) >= slabs) shares--;
      if (shares < 2 || rest * shares * 2 < units) shares = 1;
   }
   if (rounds)
   {  const double whole = (double)(slabs + 6), cut = (double)((slabs + shares - 1) / shares + 6) + 0.02 * whole;
      *rounds = (double)(tiles / units) + (rest == 0 ? 0.0 : (shares > 1 ? cut / whole : 1.0));
   }
   return (int)shares;
}

int gemm_compute_units(void)
{  static std::atomic<int> cached[64];          /* zero-initialised; threads that meet an empty entry all store the same number */
   int device = 0;
   if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
   int n = cached[device].load(std::memory_order_relaxed);
   if (n == 0)
   {  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0) n = 256;
      cached[device].store(n, std::memory_order_relaxed);
   }
   return n;
}

static char norm_trans(char t)
{  if (t == 'N' || t == 'n') return 'N';
   if (t == 'T' || t == 't') return 'T';
   if (t == 'C' || t == 'c') return 'C';
   return 0;
}

} /* namespace och */

using namespace och;

extern "C" int och_gemm_supported(int dtype)
{  return (dtype >= 0 && dtype < DT_COUNT && dtype != OCH_CHALF) ? 1 : 0; }

static int gemm_dispatch(int dtype, const GemmArgs &g)
{
   switch (dtype)
   {  case OCH_BOOL:    { const int status = gemm_bool(g); return (status == 1) ? gemm_generic<obool>(g) : status; }
      case OCH_UINT8:   { const int status = gemm_int8(g); return (status == 1) ? gemm_generic<uint8_t>(g) : status; }
      case OCH_UINT16:  return gemm_generic<uint16_t>(g);
      case OCH_UINT32:  return gemm_generic<uint32_t>(g);
      case OCH_UINT64:  return gemm_generic<uint64_t>(g);
      case OCH_INT8:    { const int status = gemm_int8(g); return (status == 1) ? gemm_generic<int8_t>(g) : status; }
      case OCH_INT16:   return gemm_generic<int16_t>(g);
      case OCH_INT32:   return gemm_generic<int32_t>(g);
      case OCH_INT64:   return gemm_generic<int64_t>(g);
      case OCH_HALF:    { const int status = gemm_half(g); return (status == 1) ? gemm_generic<half_t>(g) : status; }
      case OCH_FLOAT:   return gemm_float(g);
      case OCH_DOUBLE:  return gemm_double(g);
      case OCH_CFLOAT:  return gemm_cfloat(g);
      case OCH_CDOUBLE: return gemm_cdouble(g);
   }
   return set_error("gemm is not available for data type %d", dtype);
}

/* argument checks shared by the single and the batched entry; returns 1 when there is nothing to do */
static int gemm_prepare(GemmArgs &g, int dtype, char transA, char transB, size_t M, size_t N, size_t K,
                        const void *alpha, const void *A, ptrdiff_t ldA, const void *B, ptrdiff_t ldB,
                        const void *beta, void *C, ptrdiff_t ldC, int scalar_mode_host, och_stream stream)
{
   if (!och_gemm_supported(dtype)) return set_error("gemm is not available for data type %d", dtype);
   g.transA = norm_trans(transA); g.transB = norm_trans(transB);
   if (!g.transA || !g.transB) return set_error("gemm: invalid transposition mode ('%c', '%c')", transA, transB);
   if (M == 0 || N == 0) return 1;                       /* empty result: tensor_blas_gpu.c:96 */
   if (M > 0xFFFFFF00ull || N > 0xFFFFFF00ull || K > 0xFFFFFF00ull) return set_error("gemm: dimensions beyond 2^32 are not supported");
   const size_t rowsA = (g.transA == 'N') ? M : K, rowsB = (g.transB == 'N') ? K : N;
   if (K > 0 && (ldA < (ptrdiff_t)(rowsA ? rowsA : 1) || ldB < (ptrdiff_t)(rowsB ? rowsB : 1)))
      return set_error("gemm: leading dimension smaller than the number of rows (ldA = %td, ldB = %td)", ldA, ldB);
   if (ldC < (ptrdiff_t)M) return set_error("gemm: ldC = %td is smaller than M = %zu", ldC, M);
   if (!alpha || !beta || !C || (K > 0 && (!A || !B))) return set_error("gemm: null pointer argument");
   g.M = M; g.N = N; g.K = K; g.alpha = alpha; g.beta = beta; g.A = A; g.B = B; g.C = C;
   g.ldA = ldA; g.ldB = ldB; g.ldC = ldC; g.scalar_mode_host = scalar_mode_host; g.stream = as_stream(stream);
   if (dtype < OCH_CHALF && g.transA == 'C') g.transA = 'T';   /* conjugating a real matrix is the identity */
   if (dtype < OCH_CHALF && g.transB == 'C') g.transB = 'T';
   memset(&g.batch, 0, sizeof(g.batch)); g.nz = 1;
   return 0;
}

extern "C" int och_gemm(int dtype, char transA, char transB, size_t M, size_t N, size_t K,
                        const void *alpha, const void *A, ptrdiff_t ldA, const void *B, ptrdiff_t ldB,
                        const void *beta, void *C, ptrdiff_t ldC, int scalar_mode_host, och_stream stream)
{
   GemmArgs g;
   const int status = gemm_prepare(g, dtype, transA, transB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, scalar_mode_host, stream);
   if (status != 0) return status < 0 ? -1 : 0;
   return gemm_dispatch(dtype, g);
}

extern "C" int och_gemm_batched(int dtype, char transA, char transB, size_t M, size_t N, size_t K,
                                const void *alpha, const void *A, ptrdiff_t ldA, const void *B, ptrdiff_t ldB,
                                const void *beta, void *C, ptrdiff_t ldC,
                                int nbatch, const size_t *batch_size,
                                const ptrdiff_t *stride_alpha, const ptrdiff_t *strideA, const ptrdiff_t *strideB,
                                const ptrdiff_t *stride_beta, const ptrdiff_t *strideC,
                                int scalar_mode_host, och_stream stream)
{
   GemmArgs g;
   if (nbatch < 0 || nbatch > OCH_GEMM_BATCH_DIMS) return set_error("gemm: invalid number of batch dimensions (%d)", nbatch);
   if (nbatch > 0 && (!batch_size || !strideA || !strideB || !strideC)) return set_error("gemm: null batch argument");
   const int status = gemm_prepare(g, dtype, transA, transB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, scalar_mode_host, stream);
   if (status != 0) return status < 0 ? -1 : 0;
   uint64_t total = 1; bool scalars_move = false;
   GemmBatch &b = g.batch;
   for (int d = 0; d < nbatch; d++)
   {  if (batch_size[d] == 0) return 0;
      if (batch_size[d] == 1) continue;
      if (batch_size[d] > 0xFFFFFFFFull || total * batch_size[d] > 0xFFFFFFFFull) return set_error("gemm: too many products in one batch");
      total *= batch_size[d];
      b.size[b.nb] = (uint32_t)batch_size[d];
      b.sA[b.nb] = strideA[d]; b.sB[b.nb] = strideB[d]; b.sC[b.nb] = strideC[d];
      b.sAlpha[b.nb] = stride_alpha ? stride_alpha[d] : 0; b.sBeta[b.nb] = stride_beta ? stride_beta[d] : 0;
      if (b.sAlpha[b.nb] != 0 || b.sBeta[b.nb] != 0) scalars_move = true;
      b.nb++;
   }
   if (b.nb == 0) return gemm_dispatch(dtype, g);
   if (scalar_mode_host && scalars_move)
   {  /* host scalars that differ between the products are passed by value: one launch per product */
      const GemmBatch all = b;
      memset(&b, 0, sizeof(b));
      for (uint64_t z = 0; z < total; z++)
      {  uint64_t q = z; int64_t oA = 0, oB = 0, oC = 0, oAl = 0, oBe = 0;
         for (int d = 0; d < all.nb; d++)
         {  const uint64_t i = q % all.size[d]; q /= all.size[d];
            oA += (int64_t)i * all.sA[d]; oB += (int64_t)i * all.sB[d]; oC += (int64_t)i * all.sC[d];
            oAl += (int64_t)i * all.sAlpha[d]; oBe += (int64_t)i * all.sBeta[d];
         }
         g.A = (const char *)A + oA; g.B = (const char *)B + oB; g.C = (char *)C + oC;
         g.alpha = (const char *)alpha + oAl; g.beta = (const char *)beta + oBe;
         if (gemm_dispatch(dtype, g) != 0) return -1;
      }
      return 0;
   }
   for (uint64_t z0 = 0; z0 < total; z0 += 65535)          /* grid z is limited to 65535 */
   {  b.z0 = (uint32_t)z0; g.nz = (unsigned)((total - z0 < 65535) ? total - z0 : 65535);
      if (gemm_dispatch(dtype, g) != 0) return -1;
   }
   return 0;
}

extern "C" int och_gemm_split_plan(size_t M, size_t N, size_t K, unsigned tile_m, unsigned tile_n, unsigned slab, unsigned elem_size,
                                   unsigned units, double *rounds)
{
   return och::gemm_pipe_split_plan(M, N, K, 1, true, tile_m, tile_n, slab, elem_size, units, rounds);
}

extern "C" int och_gemm_float_plan(size_t M, size_t N, size_t K, unsigned batch)
{
   return och::gemm_float_plan_query(M, N, K, batch);
}

extern "C" int och_gemm_set_kernel_choice(int choice)
{
   if (choice < 0 || choice > 4) return och::set_error("gemm: kernel choice %d (0 automatic, 1 pipelined large tile, 2 pipelined small tile, 3 tiled kernel, 4 pipelined smallest tile)", choice);
   och::g_gemm_kernel_choice.store(choice, std::memory_order_relaxed);
   return 0;
}
