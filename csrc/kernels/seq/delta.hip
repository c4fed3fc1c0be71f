// Generalized delta rule: per head a state S [key channel i, value channel c] in fp32,
//   S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,      o_t = S_t^T r_t,
// with the unit key u = k / sqrt(sum(k^2) + key_eps), the decay w = exp(-decay_scale sigmoid(wz + w0))
// and the removal rate a = sigmoid(az) per key channel.  The output is o divided by its root mean
// square over the head, times a weight, times sigmoid(g), times out_scale.
//
// One block per (head, request) walks the request's rows of this step in order.  The columns of S
// are independent of each other, so each of the four waves owns a quarter of them and never waits for
// the others inside a row: lane = (row group, column), a lane holds RPG rows of its column in
// registers, and the sums over the key channel are finished by xor-shuffles across the row groups.
// With  inv2 = 1 / (sum k^2 + eps):
//   kS[c]  = sum_i k_i S[i][c]        rS[c] = sum_i (r_i w_i) S[i][c]           (one pass over the old state)
//   S[i][c] <- w_i S[i][c] - (a_i k_i) (inv2 kS[c]) + k_i v_c
//   o[c]   = rS[c] - (inv2 kS[c]) (sum_i r_i a_i k_i) + v_c (sum_i r_i k_i)
// so both terms read the old state, and o needs no second pass over the new one.
//
// Rows are taken TP = 256 / d at a time.  Everything that does not depend on the state is done for
// the TP rows at once by all threads (thread = (row, channel)): the loads (the next TP rows' are
// issued one round ahead, so their latency hides under this round's recurrence), the decay, a k, r w
// into LDS, and the three sums over the head (k^2, r a k, r k).  Then every wave walks the TP rows for
// its columns without a barrier and leaves o in LDS; after the round all threads work in parallel
// again on the outputs: o over its root mean square in the head, weight, gate, store.
// A request whose step starts at position 0 starts from zeros without reading its slot.
#include "seq_common.h"
#include "fls_seq.h"

#define DR_MAX_D 128
#define DR_ROWS 256          // LDS floats per staged vector: TP rows x d channels <= 256

template <int RPG, typename TO, bool VEC>
__global__ __launch_bounds__(256) void delta_rule_kernel(const float* __restrict__ r, int ldr, const float* __restrict__ k, int ldk,
                                                         const float* __restrict__ v, int ldv, const float* __restrict__ az, int lda,
                                                         const float* __restrict__ wz, int ldw, const float* __restrict__ g, int ldg,
                                                         const float* __restrict__ w0, const float* __restrict__ norm_w,
                                                         float* __restrict__ state, TO* __restrict__ out, int ldo,
                                                         const int* __restrict__ cu, const int* __restrict__ pos0,
                                                         const int* __restrict__ slot, int H, int d, int cw, int cwl,
                                                         float decay_scale, float key_eps, float norm_eps, float out_scale,
                                                         float* __restrict__ raw) {
  __shared__ __attribute__((aligned(16))) float sk[DR_ROWS], srw[DR_ROWS], sw[DR_ROWS], sak[DR_ROWS], sv[DR_ROWS], so[DR_ROWS];
  __shared__ float prod[3][DR_ROWS];                 // k^2 | r a k | r k per (row, channel)
  __shared__ float sums[3][DR_ROWS];                 // per row: 1 / (sum k^2 + eps) | sum r a k | sum r k; later sum o^2
  const int h = blockIdx.x, s = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int TP = 256 / d;                            // rows per round
  // as row worker: thread = (row of the round, channel)
  const int wrow = tid / d, ch = tid % d;
  const bool worker = wrow < TP;
  // as state owner: lane = (row group, column of this wave's cw columns); 1 << cwl lanes span the columns
  // gridDim.z > 1: the block owns d / gridDim.z of the columns and writes o as it is to `raw`; the division
  // by o's root mean square over the whole head, the weight and the gate follow in delta_out_kernel
  const int cl = lane & ((1 << cwl) - 1), rg = lane >> cwl;
  const int dc = d / gridDim.z;
  const int col = blockIdx.z * dc + wave * cw + cl;
  const bool colok = cl < cw && wave * cw + cl < dc;
  const bool split = gridDim.z > 1;
  const int i0 = rg * RPG;
  const int a0 = cu[s], a1 = cu[s + 1];
  float* sp = state + ((size_t)slot[s] * H + h) * d * d;
  float S[RPG];
#pragma unroll
  for (int x = 0; x < RPG; ++x) S[x] = 0.f;
  if (colok && pos0[s] > 0) {
#pragma unroll
    for (int x = 0; x < RPG; ++x) if (i0 + x < d) S[x] = sp[(size_t)(i0 + x) * d + col];
  }
  const size_t hc = (size_t)h * d + ch;
  const float w0c = w0[hc], nwc = norm_w[hc];
  // this thread's (row wrow of the round, channel ch) inputs, loaded one round ahead
  float nr = 0.f, nk = 0.f, nv = 0.f, na = 0.f, nz = 0.f, ng = 0.f;
  auto load = [&](int t0) {
    const int t = t0 + wrow;
    if (worker && t < a1) {
      nr = r[(size_t)t * ldr + hc]; nk = k[(size_t)t * ldk + hc]; nv = v[(size_t)t * ldv + hc];
      na = az[(size_t)t * lda + hc]; nz = wz[(size_t)t * ldw + hc]; ng = g[(size_t)t * ldg + hc];
    }
  };
  load(a0);
  for (int t0 = a0; t0 < a1; t0 += TP) {
    const int rows = min(TP, a1 - t0);
    const float gv = ng;
    if (worker && wrow < rows) {
      const float wv = expf(-decay_scale * sigmoid_f(nz + w0c));
      const float ak = sigmoid_f(na) * nk;
      sk[tid] = nk; srw[tid] = nr * wv; sw[tid] = wv; sak[tid] = ak; sv[tid] = nv;
      prod[0][tid] = nk * nk; prod[1][tid] = nr * ak; prod[2][tid] = nr * nk;
    }
    __syncthreads();
    load(t0 + TP);                                   // the next round's inputs travel while this round computes
    for (int row = wave; row < rows; row += 4) {     // the three sums of a row over the head, a wave each
      float q0 = 0.f, q1 = 0.f, q2 = 0.f;
      for (int i = lane; i < d; i += 64) { q0 += prod[0][row * d + i]; q1 += prod[1][row * d + i]; q2 += prod[2][row * d + i]; }
      for (int o = 32; o > 0; o >>= 1) {
        q0 += __shfl_xor(q0, o, 64); q1 += __shfl_xor(q1, o, 64); q2 += __shfl_xor(q2, o, 64);
      }
      if (lane == 0) { sums[0][row] = 1.f / (q0 + key_eps); sums[1][row] = q1; sums[2][row] = q2; }
    }
    __syncthreads();
    for (int j = 0; j < rows; ++j) {                 // (no barrier in here: a wave's columns are its own)
      const float* kj = sk + j * d;
      const float* rwj = srw + j * d;
      float p1 = 0.f, p2 = 0.f;
      if constexpr (VEC) {                           // (d % 4 == 0: four rows' factors per LDS read)
#pragma unroll
        for (int x = 0; x < RPG; x += 4) {
          if (i0 + x < d) {
            const float4 a = *reinterpret_cast<const float4*>(kj + i0 + x), b = *reinterpret_cast<const float4*>(rwj + i0 + x);
            p1 += a.x * S[x] + a.y * S[x + 1] + a.z * S[x + 2] + a.w * S[x + 3];
            p2 += b.x * S[x] + b.y * S[x + 1] + b.z * S[x + 2] + b.w * S[x + 3];
          }
        }
      } else {
#pragma unroll
        for (int x = 0; x < RPG; ++x) {
          if (i0 + x < d) { p1 += kj[i0 + x] * S[x]; p2 += rwj[i0 + x] * S[x]; }
        }
      }
      for (int o = 1 << cwl; o < 64; o <<= 1) { p1 += __shfl_xor(p1, o, 64); p2 += __shfl_xor(p2, o, 64); }
      const float uS = p1 * sums[0][j], vc = colok ? sv[j * d + col] : 0.f;
      const float* wj = sw + j * d;
      const float* akj = sak + j * d;
      if constexpr (VEC) {
#pragma unroll
        for (int x = 0; x < RPG; x += 4) {
          if (i0 + x < d) {
            const float4 w4 = *reinterpret_cast<const float4*>(wj + i0 + x), a4 = *reinterpret_cast<const float4*>(akj + i0 + x),
                         k4 = *reinterpret_cast<const float4*>(kj + i0 + x);
            S[x] = w4.x * S[x] - a4.x * uS + k4.x * vc;
            S[x + 1] = w4.y * S[x + 1] - a4.y * uS + k4.y * vc;
            S[x + 2] = w4.z * S[x + 2] - a4.z * uS + k4.z * vc;
            S[x + 3] = w4.w * S[x + 3] - a4.w * uS + k4.w * vc;
          }
        }
      } else {
#pragma unroll
        for (int x = 0; x < RPG; ++x) {
          if (i0 + x < d) S[x] = wj[i0 + x] * S[x] - akj[i0 + x] * uS + kj[i0 + x] * vc;
        }
      }
      if (rg == 0 && colok) {
        const float o = p2 - uS * sums[1][j] + vc * sums[2][j];
        if (split) raw[(size_t)(t0 + j) * H * d + (size_t)h * d + col] = o;
        else so[j * d + col] = o;
      }
    }
    __syncthreads();
    if (split) continue;                             // (uniform over the block)
    for (int row = wave; row < rows; row += 4) {     // sum of squares of each row's o over the head
      float acc = 0.f;
      for (int i = lane; i < d; i += 64) { const float o = so[row * d + i]; acc += o * o; }
      acc = wave_sum(acc);
      if (lane == 0) sums[0][row] = acc;
    }
    __syncthreads();
    if (worker && wrow < rows) {                     // outputs of the round: thread = (row, channel) again
      const float y = so[tid] / sqrtf(sums[0][wrow] / (float)d + norm_eps) * nwc * sigmoid_f(gv) * out_scale;
      stf(out + (size_t)(t0 + wrow) * ldo, hc, y);
    }
    __syncthreads();                                 // (before the next round overwrites the staged vectors and sums)
  }
  if (colok) {
#pragma unroll
    for (int x = 0; x < RPG; ++x) if (i0 + x < d) sp[(size_t)(i0 + x) * d + col] = S[x];
  }
}

// the outputs of a column-split run: one wave per (row, head) divides o by its root mean square over the
// head, applies the weight, the gate and the scale
template <typename TO>
__global__ __launch_bounds__(256) void delta_out_kernel(const float* __restrict__ raw, const float* __restrict__ g, int ldg,
                                                        const float* __restrict__ norm_w, TO* __restrict__ out, int ldo, int H,
                                                        int d, float norm_eps, float out_scale, int items) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= items) return;
  const int t = item / H, h = item % H;
  const float* o = raw + (size_t)t * H * d + (size_t)h * d;
  float v[2], ss = 0.f;
#pragma unroll
  for (int e = 0; e < 2; ++e) { const int c = lane + 64 * e; v[e] = c < d ? o[c] : 0.f; ss += v[e] * v[e]; }
  const float rs = 1.f / sqrtf(wave_sum(ss) / (float)d + norm_eps);
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const int c = lane + 64 * e;
    if (c < d) {
      const size_t hc = (size_t)h * d + c;
      stf(out + (size_t)t * ldo, hc, v[e] * rs * norm_w[hc] * sigmoid_f(g[(size_t)t * ldg + hc]) * out_scale);
    }
  }
}

template <int RPG>
static void launch_delta(int to, dim3 grid, hipStream_t st, const float* r, int ldr, const float* k, int ldk, const float* v, int ldv,
                         const float* az, int lda, const float* wz, int ldw, const float* g, int ldg, const float* w0,
                         const float* norm_w, float* state, void* out, int ldo, const int* cu, const int* pos0, const int* slot,
                         int H, int d, int cw, int cwl, float decay_scale, float key_eps, float norm_eps, float out_scale, float* raw) {
#define DR_LAUNCH(TO, VEC) hipLaunchKernelGGL((delta_rule_kernel<RPG, TO, VEC>), grid, dim3(256), 0, st, r, ldr, k, ldk, v, ldv, az, lda, wz, \
                                             ldw, g, ldg, w0, norm_w, state, (TO*)out, ldo, cu, pos0, slot, H, d, cw, cwl, decay_scale, \
                                             key_eps, norm_eps, out_scale, raw)
  if (d % 4 == 0) { if (to == 1) DR_LAUNCH(bf16_t, true); else DR_LAUNCH(float, true); }
  else { if (to == 1) DR_LAUNCH(bf16_t, false); else DR_LAUNCH(float, false); }
#undef DR_LAUNCH
}

extern "C" int fls_seq_delta_rule_scan(const float* r, int ldr, const float* k, int ldk, const float* v, int ldv, const float* az,
                                       int lda, const float* wz, int ldw, const float* g, int ldg, const float* w0,
                                       const float* norm_w, float* state, void* out, int to, int ldo, const int* cu,
                                       const int* pos0, const int* slot, int T, int B, int H, int d, float decay_scale,
                                       float key_eps, float norm_eps, float out_scale, int col_splits, float* raw,
                                       fls_stream_t s) {
  if (B <= 0 || H <= 0) return 0;
  if (d < 1 || d > DR_MAX_D || col_splits < 1 || d % col_splits || (col_splits > 1 && raw == nullptr)) return -1;
  // a wave owns cw = ceil(d / 4) columns, spanned by 1 << cwl lanes; the 64 >> cwl row groups of a wave hold
  // ceil(d / groups) rows each (rounded up to the next kernel instance)
  const int cw = (d / col_splits + 3) / 4;
  int cwl = 0;
  while ((1 << cwl) < cw) ++cwl;
  const int groups = 64 >> cwl;
  const int need = (d + groups - 1) / groups;
  int rpg = 4;
  while (rpg < need) rpg *= 2;
  if (rpg > 64) return -1;
  dim3 grid(H, B, col_splits);
  hipStream_t st = (hipStream_t)s;
#define DR_ARGS to, grid, st, r, ldr, k, ldk, v, ldv, az, lda, wz, ldw, g, ldg, w0, norm_w, state, out, ldo, cu, pos0, slot, H, d, \
                cw, cwl, decay_scale, key_eps, norm_eps, out_scale, raw
  switch (rpg) {
    case 4: launch_delta<4>(DR_ARGS); break;
    case 8: launch_delta<8>(DR_ARGS); break;
    case 16: launch_delta<16>(DR_ARGS); break;
    case 32: launch_delta<32>(DR_ARGS); break;
    default: launch_delta<64>(DR_ARGS); break;
  }
#undef DR_ARGS
  SEQ_LAUNCH_CHECK();
  if (col_splits > 1 && T > 0) {
    const int items = T * H;
    if (to == 1) hipLaunchKernelGGL((delta_out_kernel<bf16_t>), dim3((items + 3) / 4), dim3(256), 0, st, raw, g, ldg, norm_w, (bf16_t*)out, ldo, H, d, norm_eps, out_scale, items);
    else hipLaunchKernelGGL((delta_out_kernel<float>), dim3((items + 3) / 4), dim3(256), 0, st, raw, g, ldg, norm_w, (float*)out, ldo, H, d, norm_eps, out_scale, items);
    SEQ_LAUNCH_CHECK();
  }
  return 0;
}
