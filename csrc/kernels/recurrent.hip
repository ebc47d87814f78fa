// Gated linear recurrence (HGRN2 form) with per-sequence fp32 state slots.
//
// Per head, with state S [d, dv] (fp32, one slot per live sequence and layer run):
//     f_t = lower + (1 - lower) * sigmoid(fz_t + f_bias)          forget gate per channel, fp32
//     S_t = diag(f_t) S_{t-1} + (1 - f_t) v_t^T                    (1 - f) is what gets written
//     o_t = S_t^T silu(qz_t)
//     out_t = o_t / sqrt(mean(o_t^2) + eps) * norm_w               RMS norm over dv, per head
// The projection row of a token is [H*d qz | H*d fz | H*dv v] in fp32. A step's tokens of one
// sequence are consecutive rows [cu[s], cu[s+1]); positions[cu[s]] == 0 marks a sequence's
// first portion, which starts from a zero state whatever the slot held before (slots are
// reused without clearing). Sequences with slot < 0 (padding rows of a captured decode step)
// are skipped.
//
// This is the sequential form: one workgroup per (head, sequence), thread c owns column c of
// the state, which lives in LDS for the whole portion. It is what a decode step needs (one
// token: the state is read and written once); long portions pay one pass per token.
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

template <typename S>
__global__ void hgrn2_kernel(const float* __restrict__ proj, int ldp, const S* __restrict__ f_bias,
                             const S* __restrict__ lower, const S* __restrict__ norm_w, float eps,
                             float* __restrict__ state, const int* __restrict__ slots,
                             const int* __restrict__ cu, const int* __restrict__ positions,
                             S* __restrict__ out, int ldo, int H, int d, int dv) {
  extern __shared__ float sm[];
  float* St = sm;                 // [d][dv]
  float* qv = St + d * dv;        // [d] silu(qz)
  float* fv = qv + d;             // [d] forget gate
  float* red = fv + d;            // [16]
  const int h = blockIdx.x, s = blockIdx.y;
  const int slot = slots[s];
  const int t0 = cu[s], t1 = cu[s + 1];
  const int c = threadIdx.x;
  if (slot < 0) {                        // padding rows: defined (zero) output, no state
    for (int t = t0; t < t1; ++t)
      if (c < dv) stf(out + (long)t * ldo + h * dv + c, 0.f);
    return;
  }
  if (t1 <= t0) return;
  float* sp = state + ((long)slot * H + h) * d * dv;
  const bool fresh = positions[t0] == 0;
  for (int i = c; i < d * dv; i += blockDim.x) St[i] = fresh ? 0.f : sp[i];
  const float nw = c < dv ? ldf(norm_w + c) : 0.f;
  for (int t = t0; t < t1; ++t) {
    const float* row = proj + (long)t * ldp;
    __syncthreads();
    for (int i = c; i < d; i += blockDim.x) {
      const float qz = row[h * d + i];
      qv[i] = qz / (1.f + expf(-qz));
      const float lw = ldf(lower + h * d + i);
      const float fz = row[H * d + h * d + i] + ldf(f_bias + h * d + i);
      fv[i] = lw + (1.f - lw) / (1.f + expf(-fz));
    }
    __syncthreads();
    float o = 0.f;
    if (c < dv) {
      const float v = row[2 * H * d + h * dv + c];
      for (int i = 0; i < d; ++i) {
        const float f = fv[i];
        const float sv = f * St[i * dv + c] + (1.f - f) * v;
        St[i * dv + c] = sv;
        o += sv * qv[i];
      }
    }
    const float ss = block_sum(o * o, red);
    if (c < dv)
      stf(out + (long)t * ldo + h * dv + c, o * (1.f / sqrtf(ss / (float)dv + eps)) * nw);
  }
  __syncthreads();
  for (int i = c; i < d * dv; i += blockDim.x) sp[i] = St[i];
}

}  // namespace

extern "C" int dli_hgrn2(const float* proj, int ldp, const void* f_bias, const void* lower,
                         const void* norm_w, float eps, float* state, const int* slots,
                         const int* cu, const int* positions, void* out, int ldo, int num_seqs,
                         int H, int d, int dv, int dt, hipStream_t st) {
  if (num_seqs <= 0) return 0;
  const int threads = ((dv + 63) / 64) * 64;
  const size_t sh = ((size_t)d * dv + 2 * d + 16) * 4;
  if (H < 1 || d < 1 || dv < 1 || threads > 1024 || sh > 160 * 1024)
    return (int)hipErrorInvalidValue;
  if (sh > 48 * 1024) {
    static bool raised[2] = {false, false};
    if (dt >= 0 && dt < 2 && !raised[dt]) {
      const void* fn = dt == 0 ? (const void*)hgrn2_kernel<u16> : (const void*)hgrn2_kernel<float>;
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         160 * 1024);
      if (e != hipSuccess) return (int)e;
      raised[dt] = true;
    }
  }
  dim3 grid(H, num_seqs);
  if (dt == 0)
    hgrn2_kernel<u16><<<grid, threads, sh, st>>>(proj, ldp, (const u16*)f_bias, (const u16*)lower,
                                                 (const u16*)norm_w, eps, state, slots, cu,
                                                 positions, (u16*)out, ldo, H, d, dv);
  else if (dt == 1)
    hgrn2_kernel<float><<<grid, threads, sh, st>>>(proj, ldp, (const float*)f_bias,
                                                   (const float*)lower, (const float*)norm_w, eps,
                                                   state, slots, cu, positions, (float*)out, ldo,
                                                   H, d, dv);
  else return (int)hipErrorInvalidValue;
  DLI_RETURN_LAUNCH();
}
