// mLSTM on the ragged engine: the scalar part of the recurrence (gates, running maximum, normaliser) and the
// per-head output norm with its gate.  The matrix memory itself is the scan of ragged_ops.hip with three gate arrays.
//
// Per head, with log gates i_t, f_t:   m_t = max(f_t + m_(t-1), i_t),
//   S_t = a_t S_(t-1) + b_t k_t v_t^T,  n_t = a_t n_(t-1) + b_t k_t,  a_t = e^(f_t + m_(t-1) - m_t),  b_t = e^(i_t - m_t),
//   o_t = S_t^T q_t / (max(|n_t . q_t|, e^(-m_t)) + floor).
// mlstm_prepare_kernel walks a sequence's rows once per head with n in registers and hands the matrix scan
//   qf = q_t / denominator_t,  ff = a_t (repeated over the rows),  gf = b_t k_t,
// so that the scan's S <- diag(ff) S + gf v^T, o = S^T qf is the recurrence above.  Everything here is float whatever the
// activation type of the projections is; exponentials, tanh and logarithms are the full-precision library functions.
#include "ragged_common.h"

using namespace ragged;

constexpr int ML_NR = 8;      // rows per lane: dim <= 512

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// One wavefront per (head, sequence); lane l holds rows l, l + 64, ...  vec: [slots, H, d + 1] = n[d], m.
// The projections of the next row are requested before the current row's arithmetic.
template <typename T>
__global__ __launch_bounds__(64) void mlstm_prepare_kernel(const T* __restrict__ P, int64_t ldp, int q0, int k0, int i0,
                                                           const float* __restrict__ gate_bias, float cap, float m_start,
                                                           float den_floor, float* __restrict__ vec, float* __restrict__ qf,
                                                           float* __restrict__ ff, float* __restrict__ gf, int H, int d, Batch bt) {
  const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  const int start = bt.seq_start[b], n = bt.seq_start[b + 1] - start, past = bt.seq_past[b], slot = bt.seq_slot[b];
  const int HD = H * d;
  const float qs = 1.0f / sqrtf((float)d);
  const float bi = gate_bias[h], bf = gate_bias[H + h];
  float* st = vec + ((int64_t)slot * H + h) * (d + 1);
  float nv[ML_NR];
#pragma unroll
  for (int r = 0; r < ML_NR; ++r) {
    const int row = lane + 64 * r;
    nv[r] = (past > 0 && row < d) ? st[row] : 0.f;
  }
  float m = past > 0 ? st[d] : m_start;
  float kq[2][ML_NR][2], gi[2], gfo[2];
  auto fetch = [&](int i, int s) {
    const T* row = P + (int64_t)(start + i) * ldp;
    gi[s] = to_f(row[i0 + h]);
    gfo[s] = to_f(row[i0 + H + h]);
#pragma unroll
    for (int r = 0; r < ML_NR; ++r) {
      const int c = lane + 64 * r;
      kq[s][r][0] = c < d ? to_f(row[k0 + h * d + c]) : 0.f;
      kq[s][r][1] = c < d ? to_f(row[q0 + h * d + c]) * qs : 0.f;
    }
  };
  if (n > 0) fetch(0, 0);
  for (int i = 0; i < n; ++i) {
    const int s = i & 1;
    if (i + 1 < n) fetch(i + 1, s ^ 1);
    const float li = cap * tanhf((gi[s] + bi) / cap);
    const float lf = log_sigmoid(cap * tanhf((gfo[s] + bf) / cap));
    const float m2 = fmaxf(lf + m, li);
    const float a = expf(lf + m - m2), bb = expf(li - m2);
    m = m2;
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < ML_NR; ++r) {
      nv[r] = a * nv[r] + bb * kq[s][r][0];
      dot += nv[r] * kq[s][r][1];
    }
    dot = wave_sum(dot);
    const float inv = 1.0f / (fmaxf(fabsf(dot), expf(-m)) + den_floor);
    const int64_t o = (int64_t)(start + i) * HD + h * d;
#pragma unroll
    for (int r = 0; r < ML_NR; ++r) {
      const int c = lane + 64 * r;
      if (c < d) {
        qf[o + c] = kq[s][r][1] * inv;
        ff[o + c] = a;
        gf[o + c] = bb * kq[s][r][0];
      }
    }
  }
#pragma unroll
  for (int r = 0; r < ML_NR; ++r) {
    const int row = lane + 64 * r;
    if (row < d) st[row] = nv[r];
  }
  if (lane == 0) st[d] = m;
}

extern "C" int ragged_mlstm_prepare(const void* P, int64_t ldp, int q0, int k0, int i0, const float* gate_bias, float cap,
                                    float m_start, float den_floor, float* vec, float* qf, float* ff, float* gf, int H, int d,
                                    Batch bt, int dtype, hipStream_t st) {
  if (bt.B <= 0 || H <= 0 || d <= 0 || d > 64 * ML_NR || !(cap > 0.f) || !vec || !gate_bias) return -1;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((mlstm_prepare_kernel<T>), dim3(H, bt.B), dim3(64), 0, st, (const T*)P, ldp, q0, k0, i0,
                                            gate_bias, cap, m_start, den_floor, vec, qf, ff, gf, H, d, bt))
  return RAGGED_LAUNCH_OK();
}

// out[t, h, :] = o[t, h, :] / rms(o[t, h, :]) * w[h, :] * sigmoid(gate logits of row t, columns g0 + h * vd ...).
// One wavefront per (row, head).
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                             const T* __restrict__ P, int64_t ldp, int g0, T* __restrict__ out,
                                                             int64_t items, int H, int vd, float eps) {
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (item >= items) return;
  const int64_t t = item / H;
  const int h = (int)(item % H);
  const float* row = o + item * vd;
  float ss = 0.f;
  for (int c = lane; c < vd; c += 64) { const float v = row[c]; ss += v * v; }
  const float r = 1.0f / sqrtf(wave_sum(ss) / (float)vd + eps);
  for (int c = lane; c < vd; c += 64) {
    float v = row[c] * r * w[h * vd + c];
    if (P) v *= 1.0f / (1.0f + expf(-to_f(P[t * ldp + g0 + h * vd + c])));
    out[item * vd + c] = from_f<T>(v);
  }
}

extern "C" int ragged_head_norm_gate(const float* o, const float* w, const void* P, int64_t ldp, int g0, void* out, int64_t rows,
                                     int H, int vd, float eps, int dtype, hipStream_t st) {
  if (rows <= 0 || H <= 0 || vd <= 0 || rows * H > 0x7fffffff) return -1;
  const int64_t items = rows * H;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((head_norm_gate_kernel<T>), dim3((unsigned)((items + 3) / 4)), dim3(256), 0, st, o, w,
                                            (const T*)P, ldp, g0, (T*)out, items, H, vd, eps))
  return RAGGED_LAUNCH_OK();
}
