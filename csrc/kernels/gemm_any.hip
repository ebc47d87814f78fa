// Shape-agnostic GEMM: C[M,N] = A[M,K] . W[N,K]^T for any M, N, K, strides and alignment, with
// an optional batch dimension (blockIdx.z: per-head projections that read a column slice of a
// wider activation). It serves what the tuned tile family (gemm.hip) refuses — K not a
// multiple of its 64-wide K-tile, unaligned leading dimensions, strided batches — and the fp32
// exact mode, which no MFMA tile of the library covers.
//
//  * bf16 operands: 64x64 block tile, 4 waves (2x2), v_mfma_f32_16x16x32_bf16 with the W
//    fragment as operand A (a lane's 4 accumulators are 4 consecutive columns of one output
//    row), K-tiles of 32 staged through LDS with zero fill past M / N / K.
//  * fp32 operands: 64x64 block tile, each thread a 4x4 register block of FMAs, true fp32.
// Grouped form (offsets != null): blockIdx.z is an expert; its rows are the permuted rows
// [offsets[e], offsets[e+1]) of C, read from A through `src` (row of A of each permuted row;
// null: A is permuted already), against W + e * sW. Row tiles past the expert's count exit.
// Output is bf16 or fp32 (c_f32). fp32 accumulation in a fixed K order per output element, so
// a row's result does not depend on which other rows are in the batch.
#include "common.h"

namespace {

constexpr int TM = 64, TN = 64;

struct AnyArgs {
  const void* A; long lda; const void* W; long ldw; void* C; long ldc;
  int M, N, K;
  long sA, sW, sC;
  int c_f32;
  const int* offsets;      // grouped form: [batch + 1] row offsets
  const int* src;          // grouped form: A row of each permuted row, or null
};

// Rows of this workgroup: a batch member's [0, M), or an expert's slice of the permuted rows.
// Returns false when the row tile holds nothing. `first` = first permuted row of the group.
__device__ __forceinline__ bool group_rows(AnyArgs& g, int m0, int& first) {
  first = 0;
  if (g.offsets != nullptr) {
    first = g.offsets[blockIdx.z];
    g.M = g.offsets[blockIdx.z + 1] - first;
    g.sA = 0;
    g.sC = 0;
  }
  return m0 < g.M;
}

// A row (element offset / lda) that local row m of the group reads
__device__ __forceinline__ long a_row(const AnyArgs& g, int first, int m) {
  if (g.offsets == nullptr) return m;
  return g.src != nullptr ? (long)g.src[first + m] : (long)(first + m);
}

__device__ __forceinline__ void store_c(const AnyArgs& g, long base, int m, int n, float v) {
  if (m < g.M && n < g.N) {
    if (g.c_f32) ((float*)g.C)[base + (long)m * g.ldc + n] = v;
    else ((u16*)g.C)[base + (long)m * g.ldc + n] = f2bf(v);
  }
}

constexpr int BKH = 32, LDH = 40;   // bf16 K-tile and padded LDS row (80 B, 16-B aligned)

__device__ __forceinline__ void stage_bf16(u16* dst, const u16* src, long ld, int row, int rows,
                                           int k, int K, bool vec) {
  uint4 v = {0u, 0u, 0u, 0u};
  if (row < rows) {
    const u16* p = src + (long)row * ld + k;
    if (vec && k + 8 <= K) {
      v = *reinterpret_cast<const uint4*>(p);
    } else {
      u16 e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = (k + i < K) ? p[i] : (u16)0;
      v.x = e[0] | ((uint32_t)e[1] << 16); v.y = e[2] | ((uint32_t)e[3] << 16);
      v.z = e[4] | ((uint32_t)e[5] << 16); v.w = e[6] | ((uint32_t)e[7] << 16);
    }
  }
  *reinterpret_cast<uint4*>(dst) = v;
}

__global__ void __launch_bounds__(256) gemm_any_bf16_kernel(AnyArgs g, int vecA, int vecW) {
  __shared__ __attribute__((aligned(16))) u16 As[TM * LDH];
  __shared__ __attribute__((aligned(16))) u16 Ws[TN * LDH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  int first;
  if (!group_rows(g, m0, first)) return;
  const u16* A = (const u16*)g.A + (long)blockIdx.z * g.sA;
  const u16* W = (const u16*)g.W + (long)blockIdx.z * g.sW;
  const int lr = tid >> 2, lk = (tid & 3) * 8;
  const long ar = m0 + lr < g.M ? a_row(g, first, m0 + lr) : 0;
  f32x4 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int fr = lane & 15, fq = lane >> 4;
  for (int k0 = 0; k0 < g.K; k0 += BKH) {
    __syncthreads();
    stage_bf16(As + lr * LDH + lk, A + ar * g.lda, 0, m0 + lr < g.M ? 0 : 1, 1, k0 + lk, g.K,
               vecA != 0);
    stage_bf16(Ws + lr * LDH + lk, W, g.ldw, n0 + lr, g.N, k0 + lk, g.K, vecW != 0);
    __syncthreads();
    bf16x8 af[2], wf[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
      af[i] = *reinterpret_cast<const bf16x8*>(As + (wm * 32 + i * 16 + fr) * LDH + fq * 8);
#pragma unroll
    for (int j = 0; j < 2; ++j)
      wf[j] = *reinterpret_cast<const bf16x8*>(Ws + (wn * 32 + j * 16 + fr) * LDH + fq * 8);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], af[i], acc[i][j], 0, 0, 0);
  }
  const long base = (long)blockIdx.z * g.sC + (long)first * g.ldc;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        store_c(g, base, m0 + wm * 32 + i * 16 + fr, n0 + wn * 32 + j * 16 + fq * 4 + r,
                acc[i][j][r]);
}

constexpr int BKF = 16, LDF = 68;

__global__ void __launch_bounds__(256) gemm_any_f32_kernel(AnyArgs g) {
  __shared__ float As[BKF * LDF];
  __shared__ float Ws[BKF * LDF];
  const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  int first;
  if (!group_rows(g, m0, first)) return;
  const float* A = (const float*)g.A + (long)blockIdx.z * g.sA;
  const float* W = (const float*)g.W + (long)blockIdx.z * g.sW;
  const int lr = tid >> 2, lk = (tid & 3) * 4;
  const long ar = m0 + lr < g.M ? a_row(g, first, m0 + lr) : 0;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < g.K; k0 += BKF) {
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + lk + u;
      As[(lk + u) * LDF + lr] = (m0 + lr < g.M && k < g.K) ? A[ar * g.lda + k] : 0.f;
      Ws[(lk + u) * LDF + lr] = (n0 + lr < g.N && k < g.K) ? W[(long)(n0 + lr) * g.ldw + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BKF; ++k) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k * LDF + ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[k * LDF + tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
  }
  const long base = (long)blockIdx.z * g.sC + (long)first * g.ldc;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) store_c(g, base, m0 + ty * 4 + i, n0 + tx * 4 + j, acc[i][j]);
}

}  // namespace

// dt: operand storage (0 bf16, 1 fp32); c_f32: fp32 output (always, when dt = 1).
// batch >= 1 with element strides sA / sW / sC between batch members.
extern "C" int dli_gemm_any(const void* A, long lda, const void* W, long ldw, void* C, long ldc,
                            int M, int N, int K, int dt, int c_f32, int batch, long sA, long sW,
                            long sC, hipStream_t st) {
  if (M <= 0 || N <= 0 || batch <= 0) return 0;
  if (K <= 0 || (dt != 0 && dt != 1) || (dt == 1 && !c_f32)) return (int)hipErrorInvalidValue;
  AnyArgs g{A, lda, W, ldw, C, ldc, M, N, K, sA, sW, sC, c_f32, nullptr, nullptr};
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM, batch);
  if (grid.y > 65535 || grid.z > 65535) return (int)hipErrorInvalidValue;
  if (dt == 0) {
    const int vecA = ((uintptr_t)A % 16 == 0 && lda % 8 == 0 && sA % 8 == 0) ? 1 : 0;
    const int vecW = ((uintptr_t)W % 16 == 0 && ldw % 8 == 0 && sW % 8 == 0) ? 1 : 0;
    gemm_any_bf16_kernel<<<grid, 256, 0, st>>>(g, vecA, vecW);
  } else {
    gemm_any_f32_kernel<<<grid, 256, 0, st>>>(g);
  }
  DLI_RETURN_LAUNCH();
}

// Grouped form: `rows` permuted rows in all (the grid's row tiles cover that many per expert;
// tiles past an expert's count exit at once), fp32 output [rows, N].
extern "C" int dli_gemm_any_grouped(const void* A, long lda, const void* W, long ldw, long sW,
                                    void* C, long ldc, int rows, int N, int K, int dt,
                                    int experts, const int* offsets, const int* src,
                                    hipStream_t st) {
  if (rows <= 0 || N <= 0 || experts <= 0) return 0;
  if (K <= 0 || (dt != 0 && dt != 1) || offsets == nullptr) return (int)hipErrorInvalidValue;
  AnyArgs g{A, lda, W, ldw, C, ldc, rows, N, K, 0, sW, 0, 1, offsets, src};
  dim3 grid((N + TN - 1) / TN, (rows + TM - 1) / TM, experts);
  if (grid.y > 65535 || grid.z > 65535) return (int)hipErrorInvalidValue;
  if (dt == 0) {
    const int vecA = ((uintptr_t)A % 16 == 0 && lda % 8 == 0) ? 1 : 0;
    const int vecW = ((uintptr_t)W % 16 == 0 && ldw % 8 == 0 && sW % 8 == 0) ? 1 : 0;
    gemm_any_bf16_kernel<<<grid, 256, 0, st>>>(g, vecA, vecW);
  } else {
    gemm_any_f32_kernel<<<grid, 256, 0, st>>>(g);
  }
  DLI_RETURN_LAUNCH();
}
