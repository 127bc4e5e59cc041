// Helpers shared by the kernels of the ragged engine (bigdl_amd/models/ragged_engine.py): a batch is a flat list of
// token rows, each row knows its sequence and position, every sequence has a state slot and a row of page ids.
// Activations are bfloat16 or float (template parameter T); the residual stream, norms, scores and recurrent state are
// always float.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ragged {

constexpr int PAGE = 64;   // tokens per cache page == lanes of a wavefront: one key per lane

struct bf16 { uint16_t b; };

__device__ __forceinline__ float to_f(float v) { return v; }
__device__ __forceinline__ float to_f(bf16 v) { return __uint_as_float((uint32_t)v.b << 16); }

template <typename T> __device__ __forceinline__ T from_f(float f);
template <> __device__ __forceinline__ float from_f<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16 from_f<bf16>(float f) {
  uint32_t x = __float_as_uint(f);
  bf16 r;
  if ((x & 0x7fffffffu) > 0x7f800000u) { r.b = (uint16_t)((x >> 16) | 0x40); return r; }
  x += 0x7fffu + ((x >> 16) & 1);      // round to nearest even
  r.b = (uint16_t)(x >> 16);
  return r;
}

// Cross-lane steps inside a row of 16 lanes are DPP moves (a few cycles); only the two steps across rows go through
// the LDS crossbar.  DPP controls: 0xB1 / 0x4E swap lanes inside a quad (xor 1 / xor 2), 0x141 mirrors 8 lanes,
// 0x140 mirrors 16: for a sum or a maximum over a whole group a mirror serves as well as an xor.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// sum over groups of R neighbouring lanes (R a power of two), result in every lane of the group
__device__ __forceinline__ float group_sum(float v, int R) {
  if (R >= 2) v += dpp_move<0xB1>(v);
  if (R >= 4) v += dpp_move<0x4E>(v);
  if (R >= 8) v += dpp_move<0x141>(v);
  if (R >= 16) v += dpp_move<0x140>(v);
  if (R >= 32) v += __shfl_xor(v, 16, 64);
  if (R >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}
__device__ __forceinline__ float wave_sum(float v) { return group_sum(v, 64); }
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));
  v = fmaxf(v, dpp_move<0x4E>(v));
  v = fmaxf(v, dpp_move<0x141>(v));
  v = fmaxf(v, dpp_move<0x140>(v));
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  return fmaxf(v, __shfl_xor(v, 32, 64));
}
// the value of lane `j` (the same j in every lane) in all lanes: v_readlane, no trip through LDS
__device__ __forceinline__ float lane_value(float v, int j) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), j));
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + __expf(-x)); }

// Per-step description of the batch, all int32, one device buffer:
//   tok_seq[T] tok_pos[T] | seq_start[B + 1] seq_past[B] seq_slot[B] | pages[B][max_pages]
struct Batch {
  const int* tok_seq;
  const int* tok_pos;
  const int* seq_start;
  const int* seq_past;
  const int* seq_slot;
  const int* pages;
  int T, B, max_pages;
};

}  // namespace ragged

#define RAGGED_DISPATCH(dt, ...)                                   \
  if ((dt) == 1) { using T = ragged::bf16; __VA_ARGS__; }          \
  else if ((dt) == 2) { using T = float; __VA_ARGS__; }            \
  else return -2;

#define RAGGED_LAUNCH_OK() (hipGetLastError() == hipSuccess ? 0 : -9)
