// LayerNorm over an fp32 residual stream with the previous branch's add fused
// in, grouped RMS norm with an output gate, and squared ReLU.
#include "seq_common.h"

namespace {

constexpr int kNormBlock = 256;

// One block per row. residual (fp32) += branch; out = LN(residual) * w + b.
// The row is staged in LDS so the variance is the mean squared deviation
// from the exact mean (two passes, no E[x^2] - mean^2 cancellation).
template <typename T>
__global__ __launch_bounds__(kNormBlock) void add_layernorm_kernel(
    T* __restrict__ out, const T* __restrict__ branch,
    float* __restrict__ residual, const float* __restrict__ w,
    const float* __restrict__ b, int C, float eps) {
  extern __shared__ float row[];
  __shared__ float red0[16], red1[16];
  const size_t base = (size_t)blockIdx.x * C;
  float sum = 0.f;
  for (int c = threadIdx.x; c < C; c += kNormBlock) {
    float v = residual[base + c];
    if (branch != nullptr) {
      v += ldf(branch + base + c);
      residual[base + c] = v;
    }
    row[c] = v;
    sum += v;
  }
  const float mean = block_sum(sum, red0) / (float)C;
  float sq = 0.f;
  for (int c = threadIdx.x; c < C; c += kNormBlock) {
    const float d = row[c] - mean;
    sq += d * d;
  }
  const float var = block_sum(sq, red1) / (float)C;
  const float rstd = 1.0f / sqrtf(var + eps);
  for (int c = threadIdx.x; c < C; c += kNormBlock)
    stf(out + base + c, (row[c] - mean) * rstd * w[c] + b[c]);
}

// grid (T, groups): out = o / rms(o over the group) * w * act(gate) * scale.
template <typename T>
__global__ __launch_bounds__(128) void gated_rmsnorm_kernel(
    T* __restrict__ out, int64_t out_stride, const float* __restrict__ o,
    const float* __restrict__ w, const T* __restrict__ gate,
    int64_t gate_stride, int C, int gs, int act, float eps, float out_scale) {
  __shared__ float red[16];
  const int t = blockIdx.x, g0 = blockIdx.y * gs;
  const float* orow = o + (size_t)t * C + g0;
  float ss = 0.f;
  for (int i = threadIdx.x; i < gs; i += blockDim.x) ss += orow[i] * orow[i];
  const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)gs + eps);
  for (int i = threadIdx.x; i < gs; i += blockDim.x) {
    float g = ldf(gate + (size_t)t * gate_stride + g0 + i);
    if (act == 1) g = sigmoid_f(g);
    else if (act == 2) g = silu_f(g);
    stf(out + (size_t)t * out_stride + g0 + i,
        orow[i] * r * w[g0 + i] * g * out_scale);
  }
}

template <typename T>
__global__ void relu_squared_kernel(T* __restrict__ out,
                                    const T* __restrict__ x, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const float v = fmaxf(ldf(x + i), 0.f);
    stf(out + i, v * v);
  }
}

template <typename T>
__global__ void relu_squared_vec_kernel(T* __restrict__ out,
                                        const T* __restrict__ x, int64_t nvec) {
  constexpr int N = Vec16<T>::N;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < nvec) {
    float v[N];
    Vec16<T>::load(x + i * N, v);
#pragma unroll
    for (int e = 0; e < N; ++e) {
      const float r = fmaxf(v[e], 0.f);
      v[e] = r * r;
    }
    Vec16<T>::store(out + i * N, v);
  }
}

}  // namespace

void add_layernorm(torch::Tensor out, c10::optional<torch::Tensor> branch,
                   torch::Tensor residual, torch::Tensor weight,
                   torch::Tensor bias, double eps) {
  check_f32(residual, "residual");
  check_f32(weight, "weight");
  check_f32(bias, "bias");
  TORCH_CHECK(residual.dim() == 2 && out.is_contiguous() &&
              out.sizes() == residual.sizes());
  const int T = residual.size(0), C = residual.size(1);
  TORCH_CHECK(weight.numel() == C && bias.numel() == C);
  TORCH_CHECK((size_t)C * 4 <= 64 * 1024, "row too wide for the LDS row cache");
  if (branch.has_value()) {
    TORCH_CHECK(branch->is_contiguous() && branch->sizes() == residual.sizes() &&
                branch->scalar_type() == out.scalar_type());
  }
  if (T == 0) return;
  SEQ_DISPATCH_ACT(out, {
    hipLaunchKernelGGL((add_layernorm_kernel<act_t>), dim3(T), dim3(kNormBlock),
                       (size_t)C * 4, SEQ_STREAM(), (act_t*)out.data_ptr(),
                       branch.has_value() ? (const act_t*)branch->data_ptr() : nullptr,
                       (float*)residual.data_ptr(), (const float*)weight.data_ptr(),
                       (const float*)bias.data_ptr(), C, (float)eps);
  });
  SEQ_CHECK_LAUNCH();
}

void gated_rmsnorm(torch::Tensor out, torch::Tensor o, torch::Tensor weight,
                   torch::Tensor gate, int64_t groups, int64_t act, double eps,
                   double out_scale) {
  check_f32(o, "o");
  check_f32(weight, "weight");
  check_rows(out, "out");
  check_rows(gate, "gate");
  const int T = o.size(0), C = o.size(1);
  TORCH_CHECK(groups > 0 && C % groups == 0 && weight.numel() == C);
  TORCH_CHECK(out.size(0) == T && out.size(1) == C && gate.size(0) == T &&
              gate.size(1) == C && gate.scalar_type() == out.scalar_type());
  TORCH_CHECK(groups <= 65535);
  if (T == 0) return;
  SEQ_DISPATCH_ACT(out, {
    hipLaunchKernelGGL((gated_rmsnorm_kernel<act_t>), dim3(T, groups), dim3(128),
                       0, SEQ_STREAM(), (act_t*)out.data_ptr(), out.stride(0),
                       (const float*)o.data_ptr(), (const float*)weight.data_ptr(),
                       (const act_t*)gate.data_ptr(), gate.stride(0), C,
                       (int)(C / groups), (int)act, (float)eps, (float)out_scale);
  });
  SEQ_CHECK_LAUNCH();
}

void relu_squared(torch::Tensor out, torch::Tensor x) {
  TORCH_CHECK(x.is_contiguous() && out.is_contiguous() && x.is_cuda() &&
              out.scalar_type() == x.scalar_type() && out.numel() == x.numel());
  const int64_t n = x.numel();
  if (n == 0) return;
  const int64_t vn = 16 / x.element_size();
  if (n % vn == 0 && ((size_t)x.data_ptr()) % 16 == 0 &&
      ((size_t)out.data_ptr()) % 16 == 0) {
    const int64_t nvec = n / vn;
    SEQ_DISPATCH_ACT(x, {
      hipLaunchKernelGGL((relu_squared_vec_kernel<act_t>), dim3((nvec + 255) / 256),
                         dim3(256), 0, SEQ_STREAM(), (act_t*)out.data_ptr(),
                         (const act_t*)x.data_ptr(), nvec);
    });
    SEQ_CHECK_LAUNCH();
    return;
  }
  SEQ_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((relu_squared_kernel<act_t>), dim3((n + 255) / 256),
                       dim3(256), 0, SEQ_STREAM(), (act_t*)out.data_ptr(),
                       (const act_t*)x.data_ptr(), n);
  });
  SEQ_CHECK_LAUNCH();
}
