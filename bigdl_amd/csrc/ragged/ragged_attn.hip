// Paged attention of the ragged engine: causal sliding window that also keeps the first tokens, one or two score maps
// per head over shared values (differential attention), per-head output norm and sigmoid gate in the epilogue.
//
// paged_attn_kernel (this file): one workgroup serves one (token row, query head).  A cache page holds 64 keys, one per
// lane, so the scores of a page are one register per map and the softmax statistics are wavefront reductions; values
// are read with lanes over channels.  The four wavefronts take every fourth visible page and merge their partial
// results through LDS.  It serves single decoded tokens and short portions in both activation types, and everything
// in float32; long bfloat16 prompt portions go to the MFMA kernel in ragged_attn_mfma.hip.
#include "ragged_attn.h"

using namespace ragged;

constexpr int VRP = 4;   // pairs of value channels per lane and 128 channels: vd <= 512

template <typename T> struct Vec;
template <> struct Vec<bf16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const bf16* p, float* o) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void load2(const bf16* p, float& a, float& b) {
    const uint32_t u = *reinterpret_cast<const uint32_t*>(p);
    a = __uint_as_float(u << 16);
    b = __uint_as_float(u & 0xffff0000u);
  }
};
template <> struct Vec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float* o) {
    const float4 u = *reinterpret_cast<const float4*>(p);
    o[0] = u.x; o[1] = u.y; o[2] = u.z; o[3] = u.w;
  }
  static __device__ __forceinline__ void load2(const float* p, float& a, float& b) {
    const float2 u = *reinterpret_cast<const float2*>(p);
    a = u.x; b = u.y;
  }
};

// VEC: keys are read 16 bytes at a time (d a multiple of 8 halves / 4 floats) and values two channels at a time (vd even)
template <typename T, int MAPS, bool VEC>
__global__ __launch_bounds__(256) void paged_attn_kernel(AttnArgs a, Batch bt) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int item = blockIdx.x;
  const int t = a.rows ? a.rows[item / a.H] : item / a.H, h = item % a.H;
  const int b = bt.tok_seq[t], i = bt.tok_pos[t];
  const int g = h / (a.H / a.G);
  const int qd = MAPS * a.d;
  const int vdp = (a.vd + 1) & ~1;
  float* qs = smem;                                   // [qd]
  float* part = smem + ((qd + 3) & ~3);               // per wavefront: m[MAPS] l[MAPS] acc[MAPS][vdp]
  const int pstride = 2 * MAPS + MAPS * vdp;
  for (int c = threadIdx.x; c < qd; c += 256) qs[c] = a.q[((int64_t)t * a.H + h) * qd + c];
  __syncthreads();

  const int lo = a.window > 0 ? (i - a.window + 1 > 0 ? i - a.window + 1 : 0) : 0;
  const int keep = a.window > 0 ? a.keep_first : 0;
  const T* K = (const T*)a.kpages;
  const T* V = (const T*)a.vpages;
  const int* pages = bt.pages + (int64_t)b * bt.max_pages;
  // visible pages: those of the kept first tokens that lie before the window's first page, then the window's
  const int pl = lo / PAGE, last = i / PAGE;
  const int kept_pages = (keep + PAGE - 1) / PAGE < pl ? (keep + PAGE - 1) / PAGE : pl;
  const int npg = kept_pages + last - pl + 1;

  float m[MAPS], l[MAPS], acc[MAPS][VRP][2];
#pragma unroll
  for (int mp = 0; mp < MAPS; ++mp) {
    m[mp] = -1e30f;
    l[mp] = 0.f;
#pragma unroll
    for (int r = 0; r < VRP; ++r) acc[mp][r][0] = acc[mp][r][1] = 0.f;
  }
  for (int o = wave; o < npg; o += 4) {
    const int pg = o < kept_pages ? o : pl + (o - kept_pages);
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
        if (VEC) {
          for (int c = 0; c < a.d; c += Vec<T>::N) {
            float kv[Vec<T>::N];
            Vec<T>::load(kr + c, kv);
#pragma unroll
            for (int e = 0; e < Vec<T>::N; ++e) sum += qq[c + e] * kv[e];
          }
        } else {
          for (int c = 0; c < a.d; ++c) sum += qq[c] * to_f(kr[c]);
        }
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
      for (int r = 0; r < VRP; ++r) { acc[mp][r][0] *= corr; acc[mp][r][1] *= corr; }
    }
    const int nk = i - pg * PAGE + 1 < PAGE ? i - pg * PAGE + 1 : PAGE;
    const T* vbase = V + (((int64_t)page * a.G + g) * PAGE) * a.vd;
    for (int j = 0; j < nk; ++j) {
      float pj[MAPS];
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp) pj[mp] = __shfl(p[mp], j, 64);
#pragma unroll
      for (int r = 0; r < VRP; ++r) {
        const int c = 2 * lane + 128 * r;
        if (c < a.vd) {
          float v0, v1 = 0.f;
          if (VEC) {
            Vec<T>::load2(vbase + (int64_t)j * a.vd + c, v0, v1);
          } else {
            v0 = to_f(vbase[(int64_t)j * a.vd + c]);
            if (c + 1 < a.vd) v1 = to_f(vbase[(int64_t)j * a.vd + c + 1]);
          }
#pragma unroll
          for (int mp = 0; mp < MAPS; ++mp) { acc[mp][r][0] += pj[mp] * v0; acc[mp][r][1] += pj[mp] * v1; }
        }
      }
    }
  }
  // merge the four partial results
  float* mine = part + wave * pstride;
  if (lane == 0) {
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) { mine[mp] = m[mp]; mine[MAPS + mp] = l[mp]; }
  }
#pragma unroll
  for (int mp = 0; mp < MAPS; ++mp)
#pragma unroll
    for (int r = 0; r < VRP; ++r) {
      const int c = 2 * lane + 128 * r;
      if (c < vdp) { mine[2 * MAPS + mp * vdp + c] = acc[mp][r][0]; mine[2 * MAPS + mp * vdp + c + 1] = acc[mp][r][1]; }
    }
  __syncthreads();
  if (wave != 0) return;
  float o[VRP][2], ss = 0.f;
#pragma unroll
  for (int r = 0; r < VRP; ++r) o[r][0] = o[r][1] = 0.f;
#pragma unroll
  for (int mp = 0; mp < MAPS; ++mp) {
    float M = -1e30f, L = 0.f, w[4];
    for (int wv = 0; wv < 4; ++wv) M = fmaxf(M, part[wv * pstride + mp]);
    for (int wv = 0; wv < 4; ++wv) { w[wv] = __expf(part[wv * pstride + mp] - M); L += w[wv] * part[wv * pstride + MAPS + mp]; }
    const float coef = (mp == 0 ? 1.0f : -a.lambda) / L;
#pragma unroll
    for (int r = 0; r < VRP; ++r) {
      const int c = 2 * lane + 128 * r;
      if (c < vdp) {
        float s0 = 0.f, s1 = 0.f;
        for (int wv = 0; wv < 4; ++wv) {
          s0 += w[wv] * part[wv * pstride + 2 * MAPS + mp * vdp + c];
          s1 += w[wv] * part[wv * pstride + 2 * MAPS + mp * vdp + c + 1];
        }
        o[r][0] += coef * s0;
        o[r][1] += coef * s1;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < VRP; ++r) {
    const int c = 2 * lane + 128 * r;
    if (c >= a.vd) o[r][0] = 0.f;
    if (c + 1 >= a.vd) o[r][1] = 0.f;
    ss += o[r][0] * o[r][0] + o[r][1] * o[r][1];
  }
  float f = a.out_scale;
  if (a.out_norm) f *= 1.0f / sqrtf(wave_sum(ss) / (float)a.vd + a.eps);
  if (a.gate) f *= sigmoidf_(to_f(((const T*)a.gate)[(int64_t)t * a.ldg + a.gate0 + h]));
  T* orow = (T*)a.out + (int64_t)t * a.H * a.vd + (int64_t)h * a.vd;
#pragma unroll
  for (int r = 0; r < VRP; ++r) {
    const int c = 2 * lane + 128 * r;
    if (c < a.vd) orow[c] = from_f<T>(o[r][0] * f);
    if (c + 1 < a.vd) orow[c + 1] = from_f<T>(o[r][1] * f);
  }
}

extern "C" int ragged_paged_attn(AttnArgs a, Batch bt, int maps, int dtype, hipStream_t st) {
  if (bt.T <= 0 || a.H <= 0 || a.G <= 0 || a.H % a.G || a.d <= 0 || a.vd <= 0 || a.vd > 128 * VRP) return -1;
  if (maps != 1 && maps != 2) return -1;
  const int nrows = a.rows ? a.n_rows : bt.T;
  if (nrows <= 0 || (int64_t)nrows * a.H > 0x7fffffff) return -1;
  const int vdp = (a.vd + 1) & ~1;
  const size_t sm = (((maps * a.d + 3) & ~3) + 4 * (2 * maps + maps * vdp)) * sizeof(float);
  if (sm > 60 * 1024) return -1;
  const unsigned grid = (unsigned)(nrows * a.H);
  const bool vec = (a.vd % 2 == 0) && (a.d % (dtype == 1 ? 8 : 4) == 0);
  RAGGED_DISPATCH(dtype,
    if (maps == 2 && vec) hipLaunchKernelGGL((paged_attn_kernel<T, 2, true>), dim3(grid), dim3(256), sm, st, a, bt);
    else if (maps == 2) hipLaunchKernelGGL((paged_attn_kernel<T, 2, false>), dim3(grid), dim3(256), sm, st, a, bt);
    else if (vec) hipLaunchKernelGGL((paged_attn_kernel<T, 1, true>), dim3(grid), dim3(256), sm, st, a, bt);
    else hipLaunchKernelGGL((paged_attn_kernel<T, 1, false>), dim3(grid), dim3(256), sm, st, a, bt))
  return RAGGED_LAUNCH_OK();
}
