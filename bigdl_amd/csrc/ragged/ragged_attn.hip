// Paged attention of the ragged engine: causal sliding window that also keeps the first tokens, one or two score maps
// per head over shared values (differential attention), per-head output norm and sigmoid gate in the epilogue.
// One wavefront serves one (token, query head): a cache page holds 64 keys, one per lane, so scores of a page are a
// register per map and the softmax statistics are wavefront reductions; values are read with lanes over channels.
// Prompt portions and single decoded tokens go through the same kernel (a token row knows its sequence and position).
#include "ragged_common.h"

using namespace ragged;

struct AttnArgs {
  const float* q;        // [T, H, MAPS, d]  normed and rotated
  const void* kpages;    // [num_pages, G, PAGE, MAPS * d]
  const void* vpages;    // [num_pages, G, PAGE, vd]
  void* out;             // [T, H * vd]
  const void* gate;      // gate logits: row t, column gate0 + h of a [T, ldg] matrix, or null
  int64_t ldg;
  int gate0;
  int H, G, d, vd;
  int window, keep_first;   // key j is visible from i if j <= i and (i - j < window or j < keep_first); window <= 0: all
  float scale;
  float lambda;          // two maps: o = a1 - lambda * a2
  float out_scale;       // applied after the output norm
  int out_norm;          // divide each head's output by its root mean square
  float eps;
};

constexpr int VR = 4;    // value channels per lane: vd <= 256

template <typename T, int MAPS>
__global__ __launch_bounds__(256) void paged_attn_kernel(AttnArgs a, Batch bt) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  const bool live = item < (int64_t)bt.T * a.H;
  const int t = live ? (int)(item / a.H) : 0, h = live ? (int)(item % a.H) : 0;
  const int b = bt.tok_seq[t], i = bt.tok_pos[t];
  const int g = h / (a.H / a.G);
  const int qd = MAPS * a.d;
  float* qs = smem + wave * qd;
  for (int c = lane; c < qd; c += 64) qs[c] = a.q[((int64_t)t * a.H + h) * qd + c];
  __syncthreads();
  if (!live) return;                                  // (no barrier below)

  const int lo = a.window > 0 ? (i - a.window + 1 > 0 ? i - a.window + 1 : 0) : 0;
  const int keep = a.window > 0 ? a.keep_first : 0;
  const T* K = (const T*)a.kpages;
  const T* V = (const T*)a.vpages;
  const int* pages = bt.pages + (int64_t)b * bt.max_pages;

  float m[MAPS], l[MAPS], acc[MAPS][VR];
#pragma unroll
  for (int mp = 0; mp < MAPS; ++mp) {
    m[mp] = -1e30f;
    l[mp] = 0.f;
#pragma unroll
    for (int r = 0; r < VR; ++r) acc[mp][r] = 0.f;
  }
  const int last = i / PAGE;
  for (int pg = 0; pg <= last; ++pg) {
    if (pg * PAGE >= keep && pg * PAGE + PAGE - 1 < lo) {      // nothing visible in this page: jump to the window
      pg = lo / PAGE - 1;
      continue;
    }
    const int page = pages[pg];
    const int kp = pg * PAGE + lane;
    const bool vis = kp <= i && (kp >= lo || kp < keep);
    const T* krow = K + (((int64_t)page * a.G + g) * PAGE + lane) * qd;
    float s[MAPS];
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) s[mp] = 0.f;
    if (vis) {
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp) {
        const T* kr = krow + mp * a.d;
        const float* qq = qs + mp * a.d;
        float sum = 0.f;
        for (int c = 0; c < a.d; ++c) sum += qq[c] * to_f(kr[c]);
        s[mp] = sum * a.scale;
      }
    }
    float p[MAPS];
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
      const float mx = fmaxf(m[mp], wave_max(vis ? s[mp] : -1e30f));
      const float corr = __expf(m[mp] - mx);
      p[mp] = vis ? __expf(s[mp] - mx) : 0.f;
      l[mp] = l[mp] * corr + wave_sum(p[mp]);
      m[mp] = mx;
#pragma unroll
      for (int r = 0; r < VR; ++r) acc[mp][r] *= corr;
    }
    const int nk = i - pg * PAGE + 1 < PAGE ? i - pg * PAGE + 1 : PAGE;
    const T* vbase = V + (((int64_t)page * a.G + g) * PAGE) * a.vd;
    for (int j = 0; j < nk; ++j) {
      float pj[MAPS];
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp) pj[mp] = __shfl(p[mp], j, 64);
#pragma unroll
      for (int r = 0; r < VR; ++r) {
        const int c = lane + 64 * r;
        if (c < a.vd) {
          const float v = to_f(vbase[(int64_t)j * a.vd + c]);
#pragma unroll
          for (int mp = 0; mp < MAPS; ++mp) acc[mp][r] += pj[mp] * v;
        }
      }
    }
  }
  float o[VR], ss = 0.f;
#pragma unroll
  for (int r = 0; r < VR; ++r) {
    o[r] = acc[0][r] / l[0];
    if (MAPS == 2) o[r] -= a.lambda * (acc[MAPS - 1][r] / l[MAPS - 1]);
    if (lane + 64 * r >= a.vd) o[r] = 0.f;
    ss += o[r] * o[r];
  }
  float f = a.out_scale;
  if (a.out_norm) f *= 1.0f / sqrtf(wave_sum(ss) / (float)a.vd + a.eps);
  if (a.gate) f *= sigmoidf_(to_f(((const T*)a.gate)[(int64_t)t * a.ldg + a.gate0 + h]));
  T* orow = (T*)a.out + (int64_t)t * a.H * a.vd + (int64_t)h * a.vd;
#pragma unroll
  for (int r = 0; r < VR; ++r)
    if (lane + 64 * r < a.vd) orow[lane + 64 * r] = from_f<T>(o[r] * f);
}

extern "C" int ragged_paged_attn(AttnArgs a, Batch bt, int maps, int dtype, hipStream_t st) {
  if (bt.T <= 0 || a.H <= 0 || a.G <= 0 || a.H % a.G || a.d <= 0 || a.vd <= 0 || a.vd > 64 * VR) return -1;
  if (maps != 1 && maps != 2) return -1;
  if (maps * a.d * 4 * sizeof(float) > 48 * 1024) return -1;
  const int64_t items = (int64_t)bt.T * a.H;
  const unsigned grid = (unsigned)((items + 3) / 4);
  const size_t sm = 4 * maps * a.d * sizeof(float);
  RAGGED_DISPATCH(dtype,
    if (maps == 2) hipLaunchKernelGGL((paged_attn_kernel<T, 2>), dim3(grid), dim3(256), sm, st, a, bt);
    else hipLaunchKernelGGL((paged_attn_kernel<T, 1>), dim3(grid), dim3(256), sm, st, a, bt))
  return RAGGED_LAUNCH_OK();
}
