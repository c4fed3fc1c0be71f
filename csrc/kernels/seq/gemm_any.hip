// C[M,N] fp32 = A[M,K] . W[N,K]^T (+ bias): the matrix product of the stateful models, for bf16 and
// for true-fp32 operands, with fp32 accumulation on the matrix cores.
//
// A 64 x 64 block tile, four wavefronts in a 2 x 2 grid, one 32 x 32 MFMA accumulator each (16
// fp32 per lane).  K advances 32 at a time through LDS: 256 threads stage 64 x 32 of A and of W
// (rounding A to the weight's type on the way in when the producer left fp32), then every wave
// issues 4 (bf16, 32x32x8) or 16 (fp32, 32x32x2) MFMAs per stage.  Rows, columns and K tails are
// zero-filled, so any shape runs.  A row's result depends only on that row of A and on W (the
// K order is fixed and no other row enters its accumulator), so it does not depend on what else is
// in the batch.
//
// Two batch forms share the kernel: a strided batch (block-diagonal gates: group g multiplies
// column block g % a_mod of A by its own square matrix into column block g of C) and row groups
// (mixture of experts: rows sorted by expert, offs[g] .. offs[g+1] use weight g).
#include "seq_common.h"
#include "fls_seq.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef short shortx4 __attribute__((ext_vector_type(4)));

#define BM 64
#define BN 64
#define BK 32

template <typename T> struct Lds;
template <> struct Lds<bf16_t> { static constexpr int LD = BK + 4; };   // 72-byte rows: 8-byte fragments, no 2-way conflicts
template <> struct Lds<float> { static constexpr int LD = BK + 1; };

__device__ __forceinline__ void cvt_store(bf16_t* d, float v) { *d = f_to_bf16(v); }
__device__ __forceinline__ void cvt_store(float* d, float v) { *d = v; }
__device__ __forceinline__ void cvt_store(bf16_t* d, bf16_t v) { *d = v; }

// stage rows [r0, r0 + 64) x columns [k0, k0 + 32) of X (row bound rmax, column bound K) into LDS
template <typename TS, typename TL>
__device__ __forceinline__ void stage(const TS* __restrict__ X, int ldx, int r0, int rmax, int k0, int K, TL* lds, int vec) {
  const int tid = threadIdx.x;
  const int r = tid >> 2, kc = (tid & 3) * 8;
  const int row = r0 + r;
  TL* dst = lds + r * Lds<TL>::LD + kc;
  if (row < rmax && vec && k0 + kc + 8 <= K) {
    const TS* src = X + (size_t)row * ldx + k0 + kc;
    if constexpr (sizeof(TS) == 2) {
      uint4 v = *reinterpret_cast<const uint4*>(src);
      const bf16_t* e = reinterpret_cast<const bf16_t*>(&v);
#pragma unroll
      for (int i = 0; i < 8; ++i) cvt_store(dst + i, e[i]);
    } else {
      float4 a = *reinterpret_cast<const float4*>(src), b = *reinterpret_cast<const float4*>(src + 4);
      cvt_store(dst + 0, a.x); cvt_store(dst + 1, a.y); cvt_store(dst + 2, a.z); cvt_store(dst + 3, a.w);
      cvt_store(dst + 4, b.x); cvt_store(dst + 5, b.y); cvt_store(dst + 6, b.z); cvt_store(dst + 7, b.w);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = k0 + kc + i;
      if (row < rmax && k < K) cvt_store(dst + i, X[(size_t)row * ldx + k]);
      else cvt_store(dst + i, 0.f);
    }
  }
}

template <typename TA, typename TW>
__global__ __launch_bounds__(256) void gemm_nt_any(const TA* __restrict__ A, const TW* __restrict__ W, float* __restrict__ C,
                                                   const float* __restrict__ bias, int M, int N, int K, int lda, int ldw,
                                                   int ldc, const int* __restrict__ offs, long long a_gs, int a_mod,
                                                   long long w_gs, long long c_gs, int vec_a, int vec_w) {
  __shared__ TW As[BM * Lds<TW>::LD];
  __shared__ TW Ws[BN * Lds<TW>::LD];
  const int g = blockIdx.z;
  int m0 = blockIdx.y * BM, mend = M;
  if (offs != nullptr) {
    m0 += offs[g];
    mend = offs[g + 1];
    if (m0 >= mend) return;
    W += (size_t)g * w_gs;
  } else if (gridDim.z > 1) {
    A += (size_t)(g % a_mod) * a_gs;
    W += (size_t)g * w_gs;
    C += (size_t)g * c_gs;
    if (bias != nullptr) bias += (size_t)g * c_gs;
  }
  const int n0 = blockIdx.x * BN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
  floatx16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();
    stage<TA, TW>(A, lda, m0, mend, k0, K, As, vec_a);
    stage<TW, TW>(W, ldw, n0, N, k0, K, Ws, vec_w);
    __syncthreads();
    const TW* ap = As + (wm + (lane & 31)) * Lds<TW>::LD;
    const TW* wp = Ws + (wn + (lane & 31)) * Lds<TW>::LD;
    if constexpr (sizeof(TW) == 2) {
#pragma unroll
      for (int kk = 0; kk < BK; kk += 8) {
        const int ko = kk + (lane >> 5) * 4;
        shortx4 a = *reinterpret_cast<const shortx4*>(ap + ko);
        shortx4 b = *reinterpret_cast<const shortx4*>(wp + ko);
        acc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a, b, acc, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < BK; kk += 2) {
        const int ko = kk + (lane >> 5);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ap[ko], wp[ko], acc, 0, 0, 0);
      }
    }
  }
  // accumulator element r of a lane: row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32
  const int col = n0 + wn + (lane & 31);
  if (col < N) {
    const float bv = bias != nullptr ? bias[col] : 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = m0 + wm + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
      if (row < mend) C[(size_t)row * ldc + col] = acc[r] + bv;
    }
  }
}

static bool aligned16(const void* p, long long ld_elems, int esize, int K) {
  return ((uintptr_t)p % 16 == 0) && ((ld_elems * esize) % 16 == 0) && (K % 8 == 0);
}

extern "C" int fls_seq_gemm(const void* A, int ta, const void* W, int tw, float* C, const float* bias, int M, int N, int K,
                            int lda, int ldw, int ldc, int groups, const int* offs, long long a_gs, int a_mod,
                            long long w_gs, long long c_gs, fls_stream_t s) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || groups < 1 || (ta == 1 && tw == 0)) return -1;
  const int ea = ta == 1 ? 2 : 4, ew = tw == 1 ? 2 : 4;
  const int vec_a = aligned16(A, lda, ea, K) && (a_gs * ea) % 16 == 0;
  const int vec_w = aligned16(W, ldw, ew, K) && (w_gs * ew) % 16 == 0;
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM, groups);
  hipStream_t st = (hipStream_t)s;
  if (a_mod < 1) a_mod = 1;
  if (tw == 1 && ta == 1)
    hipLaunchKernelGGL((gemm_nt_any<bf16_t, bf16_t>), grid, dim3(256), 0, st, (const bf16_t*)A, (const bf16_t*)W, C, bias,
                       M, N, K, lda, ldw, ldc, offs, a_gs, a_mod, w_gs, c_gs, vec_a, vec_w);
  else if (tw == 1)
    hipLaunchKernelGGL((gemm_nt_any<float, bf16_t>), grid, dim3(256), 0, st, (const float*)A, (const bf16_t*)W, C, bias,
                       M, N, K, lda, ldw, ldc, offs, a_gs, a_mod, w_gs, c_gs, vec_a, vec_w);
  else
    hipLaunchKernelGGL((gemm_nt_any<float, float>), grid, dim3(256), 0, st, (const float*)A, (const float*)W, C, bias,
                       M, N, K, lda, ldw, ldc, offs, a_gs, a_mod, w_gs, c_gs, vec_a, vec_w);
  SEQ_LAUNCH_CHECK();
  return 0;
}
