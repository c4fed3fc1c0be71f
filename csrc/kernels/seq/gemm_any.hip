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

// What a kernel does with a finished accumulator element: + bias, optionally the xIELU activation
// (act = {p, q}: z > 0: softplus(p) z^2 + z/2, else (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2), then the
// store as fp32 or bf16 -- so a projection whose consumer is the next matrix product writes that
// product's operand directly and the fp32 intermediate never reaches memory.
struct Epi {
  const float* bias;
  const float* act;      // null: no activation
  int tc;                // element type of C: 0 fp32, 1 bf16
};
struct EpiRegs { float ap, an; };
__device__ __forceinline__ EpiRegs epi_regs(const Epi& e) {
  EpiRegs r = {0.f, 0.f};
  if (e.act != nullptr) { r.ap = softplus_f(e.act[0]); r.an = 0.5f + softplus_f(e.act[1]); }
  return r;
}
__device__ __forceinline__ void emit(void* C, size_t idx, float v, const Epi& e, const EpiRegs& r) {
  if (e.act != nullptr) v = v > 0.f ? r.ap * v * v + 0.5f * v : r.an * (expm1f(v) - v) + 0.5f * v;
  if (e.tc == 1) reinterpret_cast<bf16_t*>(C)[idx] = f_to_bf16(v);
  else reinterpret_cast<float*>(C)[idx] = v;
}

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
__global__ __launch_bounds__(256) void gemm_nt_any(const TA* __restrict__ A, const TW* __restrict__ W, void* __restrict__ C,
                                                   Epi epi, int M, int N, int K, int lda, int ldw,
                                                   int ldc, const int* __restrict__ offs, long long a_gs, int a_mod,
                                                   long long w_gs, long long c_gs, int vec_a, int vec_w) {
  __shared__ TW As[BM * Lds<TW>::LD];
  __shared__ TW Ws[BN * Lds<TW>::LD];
  const int g = blockIdx.z;
  size_t cbase = 0;                      // column offset of this group in C and bias (strided batch)
  const EpiRegs er = epi_regs(epi);
  int m0 = blockIdx.y * BM, mend = M;
  if (offs != nullptr) {
    m0 += offs[g];
    mend = offs[g + 1];
    if (m0 >= mend) return;
    W += (size_t)g * w_gs;
  } else if (gridDim.z > 1) {
    A += (size_t)(g % a_mod) * a_gs;
    W += (size_t)g * w_gs;
    cbase = (size_t)g * c_gs;
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
    const float bv = epi.bias != nullptr ? epi.bias[cbase + col] : 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = m0 + wm + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
      if (row < mend) emit(C, cbase + (size_t)row * ldc + col, acc[r] + bv, epi, er);
    }
  }
}

// ----------------------------------------------------------------------------- the large tile
// Square block tiles for M > 64: 128 x 128 with four waves in a 2 x 2 grid (each 64 x 64 = 2 x 2 MFMA
// accumulators) and, for large problems, 256 x 256 with eight waves in a 2 x 4 grid (each 128 x 64 =
// 4 x 2 accumulators): a tile of side S moves 2 S K operand bytes for 2 S^2 K flops, so the 256 tile
// halves the L2 / HBM traffic per flop, and every fragment read from LDS feeds 2 to 4 MFMAs.  bf16 uses the 32x32x16 MFMA (16 bytes
// per lane and operand) and a K tile of 64; fp32 a K tile of 32.  LDS is double-buffered: the next K
// tile's global loads are issued into registers before the current tile's MFMAs and stored into the
// other buffer after them, one barrier per K tile, so HBM latency hides under the matrix work.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <typename T> struct Big;
template <> struct Big<bf16_t> { static constexpr int KT = 64, LD = 64 + 8; };   // 144-byte rows: 16-byte fragments stay aligned
template <> struct Big<float> { static constexpr int KT = 32, LD = 32 + 1; };

template <typename TL> struct __attribute__((aligned(16))) Frag { TL v[Big<TL>::KT / 2]; };

// KT / 2 consecutive k of one row per thread: row = tid / 2, k segment = (KT / 2) (tid % 2)
template <typename TS, typename TL>
__device__ __forceinline__ void load_frag(const TS* __restrict__ X, int ldx, int r0, int rmax, int k0, int K, int vec, Frag<TL>& f) {
  constexpr int NE = Big<TL>::KT / 2;
  const int row = r0 + (threadIdx.x >> 1), kc = k0 + (threadIdx.x & 1) * NE;
  if (row < rmax && vec && kc + NE <= K) {
    const TS* src = X + (size_t)row * ldx + kc;
    if constexpr (sizeof(TS) == 2) {
#pragma unroll
      for (int q = 0; q < NE / 8; ++q) {
        const uint4 a = *reinterpret_cast<const uint4*>(src + 8 * q);
        const bf16_t* ea = reinterpret_cast<const bf16_t*>(&a);
#pragma unroll
        for (int i = 0; i < 8; ++i) cvt_store(&f.v[8 * q + i], ea[i]);
      }
    } else {
#pragma unroll
      for (int q = 0; q < NE / 4; ++q) {
        const float4 a = *reinterpret_cast<const float4*>(src + 4 * q);
        cvt_store(&f.v[4 * q], a.x); cvt_store(&f.v[4 * q + 1], a.y); cvt_store(&f.v[4 * q + 2], a.z); cvt_store(&f.v[4 * q + 3], a.w);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < NE; ++i) {
      if (row < rmax && kc + i < K) cvt_store(&f.v[i], X[(size_t)row * ldx + kc + i]);
      else cvt_store(&f.v[i], 0.f);
    }
  }
}

template <typename TL>
__device__ __forceinline__ void store_frag(const Frag<TL>& f, TL* lds) {
  constexpr int NE = Big<TL>::KT / 2;
  TL* dst = lds + (threadIdx.x >> 1) * Big<TL>::LD + (threadIdx.x & 1) * NE;
  if constexpr (sizeof(TL) == 2) {
#pragma unroll
    for (int q = 0; q < NE / 8; ++q) *reinterpret_cast<uint4*>(dst + 8 * q) = *reinterpret_cast<const uint4*>(&f.v[8 * q]);
  } else {
#pragma unroll
    for (int i = 0; i < NE; ++i) dst[i] = f.v[i];
  }
}

template <typename TA, typename TW, int NWM, int NWN>
__global__ __launch_bounds__(64 * NWM * NWN) void gemm_nt_big(const TA* __restrict__ A, const TW* __restrict__ W, void* __restrict__ C,
                                                   Epi epi, int M, int N, int K, int lda, int ldw,
                                                   int ldc, const int* __restrict__ offs, long long a_gs, int a_mod,
                                                   long long w_gs, long long c_gs, int vec_a, int vec_w) {
  constexpr int KT = Big<TW>::KT, LD = Big<TW>::LD;
  constexpr int TM = 32 * NWM * NWN, TN = TM;          // one operand row per two threads
  constexpr int MI = TM / NWM / 32, NJ = TN / NWN / 32;
  __shared__ __attribute__((aligned(16))) TW As[2][TM * LD];
  __shared__ __attribute__((aligned(16))) TW Ws[2][TN * LD];
  const int g = blockIdx.z;
  size_t cbase = 0;
  const EpiRegs er = epi_regs(epi);
  int m0 = blockIdx.y * TM, mend = M;
  if (offs != nullptr) {
    m0 += offs[g];
    mend = offs[g + 1];
    if (m0 >= mend) return;
    W += (size_t)g * w_gs;
  } else if (gridDim.z > 1) {
    A += (size_t)(g % a_mod) * a_gs;
    W += (size_t)g * w_gs;
    cbase = (size_t)g * c_gs;
  }
  const int n0 = blockIdx.x * TN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave / NWN) * (32 * MI), wn = (wave % NWN) * (32 * NJ);
  floatx16 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  Frag<TW> fa, fw;
  load_frag<TA, TW>(A, lda, m0, mend, 0, K, vec_a, fa);
  load_frag<TW, TW>(W, ldw, n0, N, 0, K, vec_w, fw);
  store_frag<TW>(fa, As[0]);
  store_frag<TW>(fw, Ws[0]);
  __syncthreads();
  int cur = 0;
  for (int k0 = 0; k0 < K; k0 += KT) {
    const bool more = k0 + KT < K;
    if (more) {
      load_frag<TA, TW>(A, lda, m0, mend, k0 + KT, K, vec_a, fa);
      load_frag<TW, TW>(W, ldw, n0, N, k0 + KT, K, vec_w, fw);
    }
    const TW* ap = As[cur] + (wm + (lane & 31)) * LD;
    const TW* wp = Ws[cur] + (wn + (lane & 31)) * LD;
    if constexpr (sizeof(TW) == 2) {
#pragma unroll
      for (int kk = 0; kk < KT; kk += 16) {
        const int ko = kk + (lane >> 5) * 8;
        bf16x8 a[MI], b[NJ];
#pragma unroll
        for (int i = 0; i < MI; ++i) a[i] = *reinterpret_cast<const bf16x8*>(ap + i * 32 * LD + ko);
#pragma unroll
        for (int j = 0; j < NJ; ++j) b[j] = *reinterpret_cast<const bf16x8*>(wp + j * 32 * LD + ko);
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < KT; kk += 2) {
        const int ko = kk + (lane >> 5);
        float a[MI], b[NJ];
#pragma unroll
        for (int i = 0; i < MI; ++i) a[i] = ap[i * 32 * LD + ko];
#pragma unroll
        for (int j = 0; j < NJ; ++j) b[j] = wp[j * 32 * LD + ko];
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
      }
    }
    if (more) {
      store_frag<TW>(fa, As[cur ^ 1]);
      store_frag<TW>(fw, Ws[cur ^ 1]);
    }
    __syncthreads();
    cur ^= 1;
  }
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int col = n0 + wn + j * 32 + (lane & 31);
    if (col >= N) continue;
    const float bv = epi.bias != nullptr ? epi.bias[cbase + col] : 0.f;
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (row < mend) emit(C, cbase + (size_t)row * ldc + col, acc[i][j][r] + bv, epi, er);
      }
  }
}

// ------------------------------------------------------------------------- few rows (decoding)
// M <= 32 rows against bf16 weights: the product is a stream of W through the chip once, so the
// kernel is shaped for bandwidth.  A block owns 32 output columns; its four waves split K in chunks
// of 64 taken in turn, each lane reading its own W row (and A row) 16 bytes at a time straight from
// global memory -- a lane pair covers a whole 128-byte line of a row per chunk -- into one 32x32x16 MFMA
// accumulator (rows beyond M are zero).  The four partial accumulators meet in LDS.
template <typename TA>
__device__ __forceinline__ bf16x8 load8(const TA* p) {
  if constexpr (sizeof(TA) == 2) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    return *reinterpret_cast<const bf16x8*>(&v);
  } else {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    bf16_t e[8] = {f_to_bf16(a.x), f_to_bf16(a.y), f_to_bf16(a.z), f_to_bf16(a.w),
                   f_to_bf16(b.x), f_to_bf16(b.y), f_to_bf16(b.z), f_to_bf16(b.w)};
    return *reinterpret_cast<const bf16x8*>(e);
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void gemm_nt_skinny(const TA* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ C,
                                                      Epi epi, int M, int N, int K, int lda, int ldw, int ldc,
                                                      const int* __restrict__ offs, long long w_gs) {
  __shared__ float red[4][16][64];
  if (offs != nullptr) {                   // row groups (experts): this block's group owns rows offs[g] .. offs[g+1]
    const int g = blockIdx.y, r0 = offs[g];
    M = offs[g + 1] - r0;
    if (M <= 0) return;
    A += (size_t)r0 * lda;
    C = reinterpret_cast<char*>(C) + (size_t)r0 * ldc * (epi.tc == 1 ? 2 : 4);
    W += (size_t)g * w_gs;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ql = lane & 31, h2 = lane >> 5;
  const int col = blockIdx.x * 32 + ql;
  const bool rowok = ql < M, colok = col < N;
  const bf16_t* wp = W + (size_t)(colok ? col : 0) * ldw;
  const TA* ap = A + (size_t)(rowok ? ql : 0) * lda;
  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  const uint4 z4 = make_uint4(0, 0, 0, 0);
  for (int kc = wave * 64; kc < K; kc += 256) {
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) {
      const int k = kc + 16 * s2 + 8 * h2;
      bf16x8 a = *reinterpret_cast<const bf16x8*>(&z4), b = a;
      if (k + 8 <= K) {
        if (colok) b = load8<bf16_t>(wp + k);
        if (rowok) a = load8<TA>(ap + k);
      }
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) red[wave][r][lane] = acc[r];
  __syncthreads();
  if (colok) {
    const EpiRegs er = epi_regs(epi);
    const float bv = epi.bias != nullptr ? epi.bias[col] : 0.f;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int r = wave * 4 + x;
      const int row = (r >> 2) * 8 + h2 * 4 + (r & 3);
      if (row < M) emit(C, (size_t)row * ldc + col, red[0][r][lane] + red[1][r][lane] + red[2][r][lane] + red[3][r][lane] + bv, epi, er);
    }
  }
}

static bool aligned16(const void* p, long long ld_elems, int esize, int K) {
  return ((uintptr_t)p % 16 == 0) && ((ld_elems * esize) % 16 == 0) && (K % 8 == 0);
}

template <typename TA, typename TW>
static void launch(int big, dim3 grid, hipStream_t st, const void* A, const void* W, void* C, Epi bias, int M, int N,
                   int K, int lda, int ldw, int ldc, const int* offs, long long a_gs, int a_mod, long long w_gs,
                   long long c_gs, int vec_a, int vec_w) {
  if (big == 256)
    hipLaunchKernelGGL((gemm_nt_big<TA, TW, 2, 4>), grid, dim3(512), 0, st, (const TA*)A, (const TW*)W, C, bias, M, N, K, lda,
                       ldw, ldc, offs, a_gs, a_mod, w_gs, c_gs, vec_a, vec_w);
  else if (big == 128)
    hipLaunchKernelGGL((gemm_nt_big<TA, TW, 2, 2>), grid, dim3(256), 0, st, (const TA*)A, (const TW*)W, C, bias, M, N, K, lda,
                       ldw, ldc, offs, a_gs, a_mod, w_gs, c_gs, vec_a, vec_w);
  else
    hipLaunchKernelGGL((gemm_nt_any<TA, TW>), grid, dim3(256), 0, st, (const TA*)A, (const TW*)W, C, bias, M, N, K, lda, ldw,
                       ldc, offs, a_gs, a_mod, w_gs, c_gs, vec_a, vec_w);
}

extern "C" int fls_seq_gemm(const void* A, int ta, const void* W, int tw, void* C, int tc, const float* bias_p,
                            const float* act, int M, int N, int K, int lda, int ldw, int ldc, int groups, const int* offs,
                            long long a_gs, int a_mod, long long w_gs, long long c_gs, fls_stream_t s) {
  const Epi bias = {bias_p, act, tc};
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || groups < 1 || (ta == 1 && tw == 0)) return -1;
  const int ea = ta == 1 ? 2 : 4, ew = tw == 1 ? 2 : 4;
  const int vec_a = aligned16(A, lda, ea, K) && (a_gs * ea) % 16 == 0;
  const int vec_w = aligned16(W, ldw, ew, K) && (w_gs * ew) % 16 == 0;
  hipStream_t st0 = (hipStream_t)s;
  // (row groups: M bounds every group's rows, so M <= 32 means every group fits the kernel's 32 rows)
  if ((groups == 1 || offs != nullptr) && tw == 1 && M <= 32 && vec_a && vec_w) {
    dim3 g((N + 31) / 32, offs != nullptr ? groups : 1);
    if (ta == 1) hipLaunchKernelGGL((gemm_nt_skinny<bf16_t>), g, dim3(256), 0, st0, (const bf16_t*)A, (const bf16_t*)W, C, bias, M, N, K, lda, ldw, ldc, offs, w_gs);
    else hipLaunchKernelGGL((gemm_nt_skinny<float>), g, dim3(256), 0, st0, (const float*)A, (const bf16_t*)W, C, bias, M, N, K, lda, ldw, ldc, offs, w_gs);
    SEQ_LAUNCH_CHECK();
    return 0;
  }
  // tile side by the rows of a group (on average, for row groups): 64, 128, or 256 when the
  // problem still gives the chip a few hundred blocks
  const int gm = offs != nullptr ? M / groups : M;
  int big = 0;
  if (gm > 64 && N > 64) big = 128;
  if (gm > 192 && N > 128 && (long long)((M + 255) / 256) * ((N + 255) / 256) * groups >= 256) big = 256;
  const int ts = big ? big : BM;
  dim3 grid((N + ts - 1) / ts, (M + ts - 1) / ts, groups);
  hipStream_t st = (hipStream_t)s;
  if (a_mod < 1) a_mod = 1;
  if (tw == 1 && ta == 1) launch<bf16_t, bf16_t>(big, grid, st, A, W, C, bias, M, N, K, lda, ldw, ldc, offs, a_gs, a_mod, w_gs, c_gs, vec_a, vec_w);
  else if (tw == 1) launch<float, bf16_t>(big, grid, st, A, W, C, bias, M, N, K, lda, ldw, ldc, offs, a_gs, a_mod, w_gs, c_gs, vec_a, vec_w);
  else launch<float, float>(big, grid, st, A, W, C, bias, M, N, K, lda, ldw, ldc, offs, a_gs, a_mod, w_gs, c_gs, vec_a, vec_w);
  SEQ_LAUNCH_CHECK();
  return 0;
}
