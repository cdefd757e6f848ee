// GEMM on 16-bit matrices (binary16 / bfloat16): C = alpha * op(A) * op(B) + beta * C with fp32
// accumulation on v_mfma_f32_32x32x16_{f16,bf16} and one rounding at the store -- the Linear layers of
// a half model (the reference calls cublasHgemm: src/core/tensor/tensor_math_cuda.h:1163-1187).
//
// A workgroup of four wavefronts owns a 64 x 64 tile of C, a wavefront a 32 x 32 quarter.  Both matrix
// operands want, per lane, eight consecutive reduction indices of one tile row, so both LDS tiles are
// [row][k] with k contiguous (pitch 32 + 8 halves: 16-byte reads without bank conflicts).  How a tile is
// staged depends on which index is contiguous in memory: with k contiguous (A not transposed, B
// transposed) a thread copies one octet with a 16-byte load; with the row index contiguous (A transposed,
// B not transposed) it loads eight rows of one k with a 16-byte load and writes them as eight 2-byte LDS
// stores; pointers, pitches or edges that do not allow the 16-byte access fall back to single elements.
// The reduction is not split: results are run-to-run identical.
#include <hip/hip_runtime.h>

#include "common.h"
#include "storage.h"

namespace {

constexpr int GT = 256, GBM = 64, GBN = 64, GBK = 32, GPITCH = GBK + 8;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <bool BF16>
__device__ __forceinline__ f32x16 mfma16(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

struct Operand {
  const uint16_t *p;
  int ld;        // row pitch of the stored matrix, in elements
  int k_contig;  // 1: element (row, k) at p[row * ld + k]; 0: at p[k * ld + row]
  int vec_ok;    // pointer and pitch allow 16-byte accesses
  int rows;      // rows of op(matrix): M for A, N for B
};

// Stages rows [row0, row0 + 64) x reduction indices [k0, k0 + 32) of `o` into tile[row][k]; what lies
// outside the matrix is written as zero.
__device__ __forceinline__ void stage(const Operand &o, int row0, int k0, int K, uint16_t *tile) {
  const int t = threadIdx.x;
  if (o.k_contig) {
    const int r = t >> 2, kk = (t & 3) * 8;   // one octet of k per thread
    const int row = row0 + r, k = k0 + kk;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row < o.rows && k < K) {
      const uint16_t *src = o.p + size_t(row) * o.ld + k;
      if (o.vec_ok && k + 8 <= K) {
        v = *reinterpret_cast<const u32x4 *>(src);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (k + j < K) v[j >> 1] |= unsigned(src[j]) << (16 * (j & 1));
      }
    }
    *reinterpret_cast<u32x4 *>(tile + r * GPITCH + kk) = v;
  } else {
    const int kk = t >> 3, rr = (t & 7) * 8;  // eight rows of one k per thread
    const int k = k0 + kk, row = row0 + rr;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (k < K && row < o.rows) {
      const uint16_t *src = o.p + size_t(k) * o.ld + row;
      if (o.vec_ok && row + 8 <= o.rows) {
        v = *reinterpret_cast<const u32x4 *>(src);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (row + j < o.rows) v[j >> 1] |= unsigned(src[j]) << (16 * (j & 1));
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) tile[(rr + j) * GPITCH + kk] = uint16_t(v[j >> 1] >> (16 * (j & 1)));
  }
}

template <bool BF16>
__global__ __launch_bounds__(GT) void k_gemm16(Operand A, Operand B, uint16_t *__restrict__ C, int M, int N, int K,
                                              int ldc, float alpha, float beta) {
  __shared__ __align__(16) uint16_t As[2][GBM * GPITCH], Bs[2][GBN * GPITCH];
  const int m0 = blockIdx.y * GBM, n0 = blockIdx.x * GBN;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int wm = (w >> 1) * 32, wn = (w & 1) * 32;
  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  const int chunks = (K + GBK - 1) / GBK;
  stage(A, m0, 0, K, As[0]);
  stage(B, n0, 0, K, Bs[0]);
  __syncthreads();
  for (int c = 0; c < chunks; ++c) {
    const int cur = c & 1;
    if (c + 1 < chunks) {   // the next chunk goes to the other buffer while this one is multiplied
      stage(A, m0, (c + 1) * GBK, K, As[cur ^ 1]);
      stage(B, n0, (c + 1) * GBK, K, Bs[cur ^ 1]);
    }
    const uint16_t *a = As[cur] + (wm + (lane & 31)) * GPITCH + 8 * (lane >> 5);
    const uint16_t *b = Bs[cur] + (wn + (lane & 31)) * GPITCH + 8 * (lane >> 5);
#pragma unroll
    for (int ks = 0; ks < GBK / 16; ++ks)
      acc = mfma16<BF16>(*reinterpret_cast<const u32x4 *>(a + 16 * ks), *reinterpret_cast<const u32x4 *>(b + 16 * ks), acc);
    __syncthreads();
  }
  // accumulator v of lane l: row 8 * (v / 4) + 4 * (l / 32) + v % 4, column l % 32 of the wavefront's quarter
  const int col = n0 + wn + (lane & 31);
  if (col < N) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = m0 + wm + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
      if (row < M) {
        uint16_t *dst = C + size_t(row) * ldc + col;
        float r = alpha * acc[v];
        if (beta != 0.f) r += beta * (BF16 ? sgh_bf16_to_f32(*dst) : sgh_f16_to_f32(*dst));
        *dst = BF16 ? sgh_f32_to_bf16(r) : sgh_f32_to_f16(r);
      }
    }
  }
}

template <bool BF16>
int gemm16(int transA, int transB, int M, int N, int K, float alpha, const uint16_t *A, int lda, const uint16_t *B, int ldb,
           float beta, uint16_t *C, int ldc, void *stream) {
  if (M < 0 || N < 0 || K < 0) return SGH_EINVAL;
  if (M == 0 || N == 0) return SGH_OK;
  if (!C || ldc < N || (K > 0 && (!A || !B))) return SGH_EINVAL;
  // pitches of the stored matrices: A is [M][K] (transposed: [K][M]), B is [K][N] (transposed: [N][K])
  if (K > 0 && (lda < (transA ? M : K) || ldb < (transB ? K : N))) return SGH_EINVAL;
  const Operand a{A, lda, transA ? 0 : 1, sgh_aligned16(A) && lda % 8 == 0, M};
  const Operand b{B, ldb, transB ? 1 : 0, sgh_aligned16(B) && ldb % 8 == 0, N};
  const dim3 grid((N + GBN - 1) / GBN, (M + GBM - 1) / GBM);
  if (grid.y > 65535u) return SGH_EUNSUPPORTED;
  hipStream_t st = sgh_stream_of(stream);
  sgh_prof_scope prof("gemm16", 2.0 * M * N * K, st);
  hipLaunchKernelGGL(k_gemm16<BF16>, grid, dim3(GT), 0, st, a, b, C, M, N, K, ldc, alpha, beta);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

}  // namespace

extern "C" {

int sgh_gemm_f16(int transA, int transB, int M, int N, int K, float alpha, const uint16_t *A, int lda, const uint16_t *B,
                 int ldb, float beta, uint16_t *C, int ldc, void *stream) {
  return gemm16<false>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream);
}
int sgh_gemm_bf16(int transA, int transB, int M, int N, int K, float alpha, const uint16_t *A, int lda, const uint16_t *B,
                  int ldb, float beta, uint16_t *C, int ldc, void *stream) {
  return gemm16<true>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream);
}

}  // extern "C"
