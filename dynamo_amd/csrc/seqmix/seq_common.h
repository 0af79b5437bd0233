// Shared helpers for the sequence-mixer kernels (gfx950 / CDNA4 only).
//
// Every kernel here is templated on the activation type T (float or bf16
// stored as uint16_t): projections, caches and kernel outputs that feed a
// matrix product use T, while norms, gates, scores and recurrent state are
// always fp32.
//
// A batch is a flat run of token rows. Sequence s owns rows
// [seq_start[s], seq_start[s] + seq_len[s]), its first row is position
// seq_pos0[s], and its recurrent state lives in slot seq_slot[s]. A
// sequence whose seq_pos0 is 0 starts from zero state whatever the slot
// holds, so freed slots need no clearing. seq_len 0 marks a padding row.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#define DEVINL __device__ __forceinline__

typedef uint16_t bf16_t;

DEVINL float to_f(float x) { return x; }
DEVINL float to_f(bf16_t u) {
  union { float f; uint32_t i; } v;
  v.i = ((uint32_t)u) << 16;
  return v.f;
}
template <typename T> DEVINL T from_f(float f);
template <> DEVINL float from_f<float>(float f) { return f; }
template <> DEVINL bf16_t from_f<bf16_t>(float f) {
  union { float f; uint32_t i; } v;
  v.f = f;
  if ((v.i & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((v.i >> 16) | 0x40);
  uint32_t lsb = (v.i >> 16) & 1;
  return (bf16_t)((v.i + 0x7fffu + lsb) >> 16);
}

DEVINL float wave_sum(float x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
  return x;
}
DEVINL float wave_max(float x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x = fmaxf(x, __shfl_xor(x, off, 64));
  return x;
}

// Block sum over blockDim.x threads (multiple of 64, at most 1024);
// `scratch` holds 16 floats of LDS. Every thread gets the total.
DEVINL float block_sum(float x, float* scratch) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  x = wave_sum(x);
  __syncthreads();  // scratch may still be read from a previous call
  if (lane == 0) scratch[wid] = x;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; i++) t += scratch[i];
  return t;
}

DEVINL float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
DEVINL float silu_f(float x) { return x * sigmoid_f(x); }
DEVINL float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
DEVINL float logsigmoid_f(float x) {
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

// Rotation of one pair at angle pos * f, fp32 throughout. The frequency
// comes as a float pair f = hi + lo; the rounding error of pos * hi is
// recovered with an fma and, with pos * lo, applied as a first-order
// correction to sin and cos, so the angle is good to about 1e-7 rad also
// at positions in the tens of thousands (a plain fp32 product is off by
// up to 6e-8 of the angle itself).
DEVINL void rot_pair(float a, float b, float pos, float fhi, float flo,
                     float& ra, float& rb) {
  const float ang = pos * fhi;
  const float rest = fmaf(pos, fhi, -ang) + pos * flo;
  float sn, cs;
  sincosf(ang, &sn, &cs);
  const float s2 = fmaf(rest, cs, sn), c2 = fmaf(-rest, sn, cs);
  ra = a * c2 - b * s2;
  rb = b * c2 + a * s2;
}

#define SEQ_CHECK(cond, msg) TORCH_CHECK(cond, "seqmix: " msg)

inline bool is_act(const torch::Tensor& t) {
  return t.scalar_type() == torch::kFloat || t.scalar_type() == torch::kBFloat16;
}

// Calls `fn(T{})`-style code with T bound to the activation type of `t`.
#define DISPATCH_ACT(t, ...)                                      \
  do {                                                            \
    if ((t).scalar_type() == torch::kFloat) {                     \
      using T = float;                                            \
      __VA_ARGS__                                                 \
    } else if ((t).scalar_type() == torch::kBFloat16) {           \
      using T = bf16_t;                                           \
      __VA_ARGS__                                                 \
    } else {                                                      \
      TORCH_CHECK(false, "seqmix: activation must be f32 or bf16"); \
    }                                                             \
  } while (0)

template <typename T> inline T* ptr(torch::Tensor& t) {
  return reinterpret_cast<T*>(t.data_ptr());
}
template <typename T> inline const T* cptr(const torch::Tensor& t) {
  return reinterpret_cast<const T*>(t.data_ptr());
}
inline hipStream_t cur_stream() {
  return at::hip::getCurrentHIPStream().stream();
}
