// Generalized delta rule: per head a state S [key channel i, value channel c] in fp32,
//   S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,      o_t = S_t^T r_t,
// with the unit key u = k / sqrt(sum(k^2) + key_eps), the decay w = exp(-decay_scale sigmoid(wz + w0))
// and the removal rate a = sigmoid(az) per key channel.  The output is o divided by its root mean
// square over the head, times a weight, times sigmoid(g), times out_scale.
//
// One block per (head, request) walks the request's rows of this step in order; the state lives in
// registers: thread (rg, c) holds rows rg * RPG .. + RPG of column c.  With  inv^2 = 1 / (sum k^2 + eps):
//   kS[c]  = sum_i k_i S[i][c]        rS[c] = sum_i (r_i w_i) S[i][c]           (one pass over the old state)
//   S[i][c] <- w_i S[i][c] - (a_i k_i) (inv^2 kS[c]) + k_i v_c
//   o[c]   = rS[c] - (inv^2 kS[c]) (sum_i r_i a_i k_i) + v_c (sum_i r_i k_i)
// so both terms read the old state, and o needs no second pass over the new one.  Per row: the first d
// threads load the row's vectors, form w, a k and r w and put them into LDS (two buffers in turn);
// barrier; partial kS / rS per row group into LDS; barrier; every thread sums the partials of its
// column, updates its rows, and the first d threads form o.  The division by o's root mean square
// needs one more sum over the head: it rides on the next row's first barrier (and one closing barrier
// after the last row), so a row costs two barriers.  A request whose step starts at position 0 starts
// from zeros without reading its slot.
#include "seq_common.h"
#include "fls_seq.h"

#define DR_MAX_D 128
#define DR_MAX_RG 8

template <int RPG, typename TO>
__global__ __launch_bounds__(256) void delta_rule_kernel(const float* __restrict__ r, int ldr, const float* __restrict__ k, int ldk,
                                                         const float* __restrict__ v, int ldv, const float* __restrict__ az, int lda,
                                                         const float* __restrict__ wz, int ldw, const float* __restrict__ g, int ldg,
                                                         const float* __restrict__ w0, const float* __restrict__ norm_w,
                                                         float* __restrict__ state, TO* __restrict__ out, int ldo,
                                                         const int* __restrict__ cu, const int* __restrict__ pos0,
                                                         const int* __restrict__ slot, int H, int d, float decay_scale,
                                                         float key_eps, float norm_eps, float out_scale) {
  __shared__ float sk[2][DR_MAX_D], srw[2][DR_MAX_D], sw[2][DR_MAX_D], sak[2][DR_MAX_D], sv[2][DR_MAX_D];
  __shared__ float red[2][4][4];                     // [buffer][k^2 | r a k | r k | o^2][wave]
  __shared__ float pk[DR_MAX_RG][DR_MAX_D], pr[DR_MAX_RG][DR_MAX_D];
  const int h = blockIdx.x, s = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nrg = (d + RPG - 1) / RPG;
  const int rg = tid / d, c = tid % d;
  const bool owner = rg < nrg;                       // holds a part of the state
  const bool first = tid < d;                        // loads column tid of a row's vectors, forms o[tid]
  const int i0 = rg * RPG;
  const int a0 = cu[s], a1 = cu[s + 1];
  float* sp = state + ((size_t)slot[s] * H + h) * d * d;
  float S[RPG];
#pragma unroll
  for (int x = 0; x < RPG; ++x) S[x] = 0.f;
  if (owner && pos0[s] > 0) {
#pragma unroll
    for (int x = 0; x < RPG; ++x) if (i0 + x < d) S[x] = sp[(size_t)(i0 + x) * d + c];
  }
  const size_t hc = (size_t)h * d + tid;             // this thread's column of the [T, H d] inputs (first d threads)
  const float w0c = first ? w0[hc] : 0.f, nwc = first ? norm_w[hc] : 0.f;
  float o_prev = 0.f, g_prev = 0.f;                  // the previous row's o and gate, waiting for their norm
  for (int t = a0; t <= a1; ++t) {
    const int b = (t - a0) & 1;
    float kk = 0.f, rak = 0.f, rk = 0.f, gv = 0.f;
    if (t < a1 && first) {
      const float rv = r[(size_t)t * ldr + hc], kv = k[(size_t)t * ldk + hc];
      const float wv = expf(-decay_scale * sigmoid_f(wz[(size_t)t * ldw + hc] + w0c));
      const float ak = sigmoid_f(az[(size_t)t * lda + hc]) * kv;
      gv = g[(size_t)t * ldg + hc];
      sk[b][tid] = kv;
      srw[b][tid] = rv * wv;
      sw[b][tid] = wv;
      sak[b][tid] = ak;
      sv[b][tid] = v[(size_t)t * ldv + hc];
      kk = kv * kv;
      rak = rv * ak;
      rk = rv * kv;
    }
    kk = wave_sum(kk);
    rak = wave_sum(rak);
    rk = wave_sum(rk);
    const float oo = wave_sum(first ? o_prev * o_prev : 0.f);
    if (lane == 0) { red[b][0][wave] = kk; red[b][1][wave] = rak; red[b][2][wave] = rk; red[b][3][wave] = oo; }
    __syncthreads();
    if (t > a0 && first) {                           // the previous row's output, now that its sum of squares is known
      const float ss = red[b][3][0] + red[b][3][1] + red[b][3][2] + red[b][3][3];
      const float y = o_prev / sqrtf(ss / (float)d + norm_eps) * nwc * sigmoid_f(g_prev) * out_scale;
      stf(out + (size_t)(t - 1) * ldo, hc, y);
    }
    if (t == a1) break;
    const float inv2 = 1.f / (red[b][0][0] + red[b][0][1] + red[b][0][2] + red[b][0][3] + key_eps);
    if (owner) {
      float p1 = 0.f, p2 = 0.f;
#pragma unroll
      for (int x = 0; x < RPG; ++x) {
        if (i0 + x < d) { p1 += sk[b][i0 + x] * S[x]; p2 += srw[b][i0 + x] * S[x]; }
      }
      pk[rg][c] = p1;
      pr[rg][c] = p2;
    }
    __syncthreads();
    if (owner) {
      float kS = 0.f, rS = 0.f;
      for (int x = 0; x < nrg; ++x) { kS += pk[x][c]; rS += pr[x][c]; }
      const float uS = kS * inv2, vc = sv[b][c];
#pragma unroll
      for (int x = 0; x < RPG; ++x) {
        if (i0 + x < d) S[x] = sw[b][i0 + x] * S[x] - sak[b][i0 + x] * uS + sk[b][i0 + x] * vc;
      }
      if (first) {
        const float srak = red[b][1][0] + red[b][1][1] + red[b][1][2] + red[b][1][3];
        const float srk = red[b][2][0] + red[b][2][1] + red[b][2][2] + red[b][2][3];
        o_prev = rS - uS * srak + vc * srk;
        g_prev = gv;
      }
    }
  }
  if (owner) {
#pragma unroll
    for (int x = 0; x < RPG; ++x) if (i0 + x < d) sp[(size_t)(i0 + x) * d + c] = S[x];
  }
}

template <int RPG>
static void launch_delta(int to, dim3 grid, hipStream_t st, const float* r, int ldr, const float* k, int ldk, const float* v, int ldv,
                         const float* az, int lda, const float* wz, int ldw, const float* g, int ldg, const float* w0,
                         const float* norm_w, float* state, void* out, int ldo, const int* cu, const int* pos0, const int* slot,
                         int H, int d, float decay_scale, float key_eps, float norm_eps, float out_scale) {
  if (to == 1) hipLaunchKernelGGL((delta_rule_kernel<RPG, bf16_t>), grid, dim3(256), 0, st, r, ldr, k, ldk, v, ldv, az, lda, wz, ldw, g, ldg, w0, norm_w, state, (bf16_t*)out, ldo, cu, pos0, slot, H, d, decay_scale, key_eps, norm_eps, out_scale);
  else hipLaunchKernelGGL((delta_rule_kernel<RPG, float>), grid, dim3(256), 0, st, r, ldr, k, ldk, v, ldv, az, lda, wz, ldw, g, ldg, w0, norm_w, state, (float*)out, ldo, cu, pos0, slot, H, d, decay_scale, key_eps, norm_eps, out_scale);
}

extern "C" int fls_seq_delta_rule_scan(const float* r, int ldr, const float* k, int ldk, const float* v, int ldv, const float* az,
                                       int lda, const float* wz, int ldw, const float* g, int ldg, const float* w0,
                                       const float* norm_w, float* state, void* out, int to, int ldo, const int* cu,
                                       const int* pos0, const int* slot, int B, int H, int d, float decay_scale, float key_eps,
                                       float norm_eps, float out_scale, fls_stream_t s) {
  if (B <= 0 || H <= 0) return 0;
  if (d < 1 || d > DR_MAX_D) return -1;
  // rows of the state per thread: the fewest for which ceil(d / RPG) row groups of d threads fit the block
  int rpg = 4;
  while (((d + rpg - 1) / rpg) * d > 256) rpg *= 2;
  if ((d + rpg - 1) / rpg > DR_MAX_RG || rpg > 64) return -1;
  dim3 grid(H, B);
  hipStream_t st = (hipStream_t)s;
#define DR_ARGS to, grid, st, r, ldr, k, ldk, v, ldv, az, lda, wz, ldw, g, ldg, w0, norm_w, state, out, ldo, cu, pos0, slot, H, d, \
                decay_scale, key_eps, norm_eps, out_scale
  switch (rpg) {
    case 4: launch_delta<4>(DR_ARGS); break;
    case 8: launch_delta<8>(DR_ARGS); break;
    case 16: launch_delta<16>(DR_ARGS); break;
    case 32: launch_delta<32>(DR_ARGS); break;
    default: launch_delta<64>(DR_ARGS); break;
  }
#undef DR_ARGS
  SEQ_LAUNCH_CHECK();
  return 0;
}
