// Shared helpers of the sequence-state kernels (gfx950): typed loads/stores
// for the two serving dtypes (bf16 carried as ushort, fp32), precise scalar
// math, wave/block reductions. All arithmetic is fp32.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#define DEV_INLINE __device__ __forceinline__
#define WAVE 64

typedef unsigned short bf16raw;

DEV_INLINE float bf16_to_f32(bf16raw u) {
  return __builtin_bit_cast(float, ((uint32_t)u) << 16);
}

DEV_INLINE bf16raw f32_to_bf16(float f) {
  // round to nearest even (matches torch); NaN stays NaN
  uint32_t x = __builtin_bit_cast(uint32_t, f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (bf16raw)((x >> 16) | 0x40u);
  x += ((x >> 16) & 1u) + 0x7fffu;
  return (bf16raw)(x >> 16);
}

DEV_INLINE float ldf(const float* p) { return *p; }
DEV_INLINE float ldf(const bf16raw* p) { return bf16_to_f32(*p); }
DEV_INLINE void stf(float* p, float v) { *p = v; }
DEV_INLINE void stf(bf16raw* p, float v) { *p = f32_to_bf16(v); }

// four consecutive activations as one vector load (pointer aligned to four
// elements), kept raw until they are needed
template <typename T> struct Raw4;
template <> struct Raw4<float> { typedef float4 type; };
template <> struct Raw4<bf16raw> { typedef ushort4 type; };
DEV_INLINE void cvt4(const float4& v, float* o) {
  o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
DEV_INLINE void cvt4(const ushort4& v, float* o) {
  o[0] = bf16_to_f32(v.x); o[1] = bf16_to_f32(v.y);
  o[2] = bf16_to_f32(v.z); o[3] = bf16_to_f32(v.w);
}

// one 16-byte load: 8 bf16 or 4 fp32 activations (pointer 16-byte aligned)
template <typename T> struct Vec16;
template <> struct Vec16<float> {
  static constexpr int N = 4;
  static DEV_INLINE void store(float* p, const float* o) {
    *(float4*)p = make_float4(o[0], o[1], o[2], o[3]);
  }
  static DEV_INLINE void load(const float* p, float* o) {
    const float4 v = *(const float4*)p;
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct Vec16<bf16raw> {
  static constexpr int N = 8;
  static DEV_INLINE void store(bf16raw* p, const float* o) {
    uint4 v;
    v.x = (uint32_t)f32_to_bf16(o[0]) | ((uint32_t)f32_to_bf16(o[1]) << 16);
    v.y = (uint32_t)f32_to_bf16(o[2]) | ((uint32_t)f32_to_bf16(o[3]) << 16);
    v.z = (uint32_t)f32_to_bf16(o[4]) | ((uint32_t)f32_to_bf16(o[5]) << 16);
    v.w = (uint32_t)f32_to_bf16(o[6]) | ((uint32_t)f32_to_bf16(o[7]) << 16);
    *(uint4*)p = v;
  }
  static DEV_INLINE void load(const bf16raw* p, float* o) {
    const uint4 v = *(const uint4*)p;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __builtin_bit_cast(float, w[i] << 16);
      o[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
    }
  }
};

DEV_INLINE float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
DEV_INLINE float silu_f(float x) { return x / (1.0f + expf(-x)); }

DEV_INLINE float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
  return v;
}

DEV_INLINE float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
  return v;
}

// Sum over the block (<= 16 waves); every thread gets the total. `smem`
// holds >= 16 floats and must not be reused before the next barrier.
DEV_INLINE float block_sum(float v, float* smem) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int n_waves = (blockDim.x + WAVE - 1) / WAVE;
  v = wave_sum(v);
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < n_waves; ++w) total += smem[w];
  return total;
}

#define SEQ_CHECK_LAUNCH()                                                   \
  do {                                                                       \
    hipError_t e_ = hipGetLastError();                                       \
    TORCH_CHECK(e_ == hipSuccess, "HIP launch failed: ", hipGetErrorString(e_)); \
  } while (0)

#define SEQ_STREAM() c10::hip::getCurrentHIPStream().stream()

// Run `...` with act_t bound to the kernel type of the serving dtype.
#define SEQ_DISPATCH_ACT(TENSOR, ...)                                        \
  do {                                                                       \
    if ((TENSOR).scalar_type() == torch::kBFloat16) {                        \
      using act_t = bf16raw;                                                 \
      __VA_ARGS__                                                            \
    } else if ((TENSOR).scalar_type() == torch::kFloat32) {                  \
      using act_t = float;                                                   \
      __VA_ARGS__                                                            \
    } else {                                                                 \
      TORCH_CHECK(false, "activations must be bfloat16 or float32");        \
    }                                                                        \
  } while (0)

inline void check_i32(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.scalar_type() == torch::kInt32 && t.is_contiguous() && t.is_cuda(),
              name, " must be a contiguous int32 GPU tensor");
}
inline void check_f32(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.scalar_type() == torch::kFloat32 && t.is_contiguous() && t.is_cuda(),
              name, " must be a contiguous float32 GPU tensor");
}
// [T, C] view whose rows may be strided but whose columns are dense
inline void check_rows(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.dim() == 2 && (t.size(1) == 1 || t.stride(1) == 1),
              name, " must be a 2-d GPU tensor with dense columns");
}
