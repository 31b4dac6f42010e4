// Norms and gates of layers that normalise a sublayer's output as well as its
// input: the fused post-norm + residual add + next pre-norm, an RMS norm that
// writes straight into a paged cache, and a sigmoid output gate.
#include "seq_common.h"

namespace {

constexpr int kBlock = 256;

// One block per row. If a branch is given:
//   residual (fp32) += branch / rms(branch) * post_w
// then out = residual / rms(residual) * pre_w. Both rows are staged in LDS;
// sums of squares, roots and products are fp32. B is the branch's type
// (serving dtype, or fp32 for a branch accumulated in fp32).
template <typename T, typename B>
__global__ __launch_bounds__(kBlock) void sandwich_rmsnorm_kernel(
    T* __restrict__ out, const B* __restrict__ branch,
    const float* __restrict__ post_w, float* __restrict__ residual,
    const float* __restrict__ pre_w, int C, float eps) {
  extern __shared__ float row[];
  __shared__ float red0[16], red1[16];
  const size_t base = (size_t)blockIdx.x * C;
  if (branch != nullptr) {
    float sb = 0.f;
    for (int c = threadIdx.x; c < C; c += kBlock) {
      const float b = ldf(branch + base + c);
      row[c] = b;
      sb += b * b;
    }
    const float rb = 1.0f / sqrtf(block_sum(sb, red0) / (float)C + eps);
    for (int c = threadIdx.x; c < C; c += kBlock) {
      const float x = residual[base + c] + row[c] * rb * post_w[c];
      residual[base + c] = x;
      row[c] = x;
    }
  } else {
    for (int c = threadIdx.x; c < C; c += kBlock) row[c] = residual[base + c];
  }
  // every thread re-reads only the entries it wrote: no barrier needed here
  float sx = 0.f;
  for (int c = threadIdx.x; c < C; c += kBlock) sx += row[c] * row[c];
  const float rx = 1.0f / sqrtf(block_sum(sx, red1) / (float)C + eps);
  for (int c = threadIdx.x; c < C; c += kBlock)
    stf(out + base + c, row[c] * rx * pre_w[c]);
}

// grid (T): cache row at slot = x / rms(x) * w. Rows with slot < 0 are skipped.
template <typename T>
__global__ __launch_bounds__(kBlock) void rmsnorm_to_cache_kernel(
    T* __restrict__ cache, const T* __restrict__ x, int64_t x_stride,
    const float* __restrict__ w, const int64_t* __restrict__ slot_mapping, int C,
    float eps) {
  __shared__ float red[16];
  const int64_t slot = slot_mapping[blockIdx.x];
  if (slot < 0) return;  // uniform over the block
  const T* xr = x + (size_t)blockIdx.x * x_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < C; c += kBlock) {
    const float v = ldf(xr + c);
    ss += v * v;
  }
  const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)C + eps);
  for (int c = threadIdx.x; c < C; c += kBlock)
    stf(cache + (size_t)slot * C + c, ldf(xr + c) * r * w[c]);
}

// out[t, c] = x[t, c] * sigmoid(gate[t, c]) (fp32 inside)
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ out, int64_t out_stride,
                                    const T* __restrict__ x, int64_t x_stride,
                                    const T* __restrict__ gate, int64_t gate_stride,
                                    int C, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t t = i / C;
  const int c = (int)(i % C);
  stf(out + t * out_stride + c,
      ldf(x + t * x_stride + c) * sigmoid_f(ldf(gate + t * gate_stride + c)));
}

}  // namespace

void sandwich_rmsnorm(torch::Tensor out, c10::optional<torch::Tensor> branch,
                      c10::optional<torch::Tensor> post_weight,
                      torch::Tensor residual, torch::Tensor pre_weight, double eps) {
  check_f32(residual, "residual");
  check_f32(pre_weight, "pre_weight");
  TORCH_CHECK(residual.dim() == 2 && out.is_contiguous() && out.is_cuda() &&
              out.sizes() == residual.sizes());
  const int T = residual.size(0), C = residual.size(1);
  TORCH_CHECK(pre_weight.numel() == C);
  TORCH_CHECK((size_t)C * 4 <= 64 * 1024, "row too wide for the LDS row cache");
  TORCH_CHECK(branch.has_value() == post_weight.has_value());
  bool wide = false;
  if (branch.has_value()) {
    check_f32(*post_weight, "post_weight");
    TORCH_CHECK(post_weight->numel() == C);
    TORCH_CHECK(branch->is_contiguous() && branch->is_cuda() &&
                branch->sizes() == residual.sizes());
    wide = branch->scalar_type() == torch::kFloat32;
    TORCH_CHECK(wide || branch->scalar_type() == out.scalar_type(),
                "branch must be fp32 or the output's dtype");
  }
  if (T == 0) return;
  const void* bp = branch.has_value() ? branch->data_ptr() : nullptr;
  const float* pw = branch.has_value() ? (const float*)post_weight->data_ptr() : nullptr;
  SEQ_DISPATCH_ACT(out, {
    if (wide) {
      hipLaunchKernelGGL((sandwich_rmsnorm_kernel<act_t, float>), dim3(T), dim3(kBlock),
                         (size_t)C * 4, SEQ_STREAM(), (act_t*)out.data_ptr(),
                         (const float*)bp, pw, (float*)residual.data_ptr(),
                         (const float*)pre_weight.data_ptr(), C, (float)eps);
    } else {
      hipLaunchKernelGGL((sandwich_rmsnorm_kernel<act_t, act_t>), dim3(T), dim3(kBlock),
                         (size_t)C * 4, SEQ_STREAM(), (act_t*)out.data_ptr(),
                         (const act_t*)bp, pw, (float*)residual.data_ptr(),
                         (const float*)pre_weight.data_ptr(), C, (float)eps);
    }
  });
  SEQ_CHECK_LAUNCH();
}

void rmsnorm_to_cache(torch::Tensor cache, torch::Tensor x, torch::Tensor weight,
                      torch::Tensor slot_mapping, double eps) {
  check_rows(x, "x");
  check_f32(weight, "weight");
  TORCH_CHECK(slot_mapping.scalar_type() == torch::kInt64 &&
              slot_mapping.is_contiguous() && slot_mapping.is_cuda());
  const int T = x.size(0), C = x.size(1);
  TORCH_CHECK(cache.is_contiguous() && cache.is_cuda() && cache.dim() == 4 &&
              cache.size(1) == 1 && cache.size(3) == C &&
              cache.scalar_type() == x.scalar_type(),
              "cache must be [blocks, 1, block, C] of the activations' dtype");
  TORCH_CHECK(weight.numel() == C && slot_mapping.numel() == T);
  if (T == 0) return;
  SEQ_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((rmsnorm_to_cache_kernel<act_t>), dim3(T), dim3(kBlock), 0,
                       SEQ_STREAM(), (act_t*)cache.data_ptr(),
                       (const act_t*)x.data_ptr(), x.stride(0),
                       (const float*)weight.data_ptr(),
                       (const int64_t*)slot_mapping.data_ptr(), C, (float)eps);
  });
  SEQ_CHECK_LAUNCH();
}

void sigmoid_gate(torch::Tensor out, torch::Tensor x, torch::Tensor gate) {
  check_rows(out, "out");
  check_rows(x, "x");
  check_rows(gate, "gate");
  const int64_t T = x.size(0), C = x.size(1);
  TORCH_CHECK(out.size(0) == T && out.size(1) == C && gate.size(0) == T &&
              gate.size(1) == C && gate.scalar_type() == x.scalar_type() &&
              out.scalar_type() == x.scalar_type());
  const int64_t n = T * C;
  if (n == 0) return;
  SEQ_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((sigmoid_gate_kernel<act_t>), dim3((n + 255) / 256), dim3(256),
                       0, SEQ_STREAM(), (act_t*)out.data_ptr(), out.stride(0),
                       (const act_t*)x.data_ptr(), x.stride(0),
                       (const act_t*)gate.data_ptr(), gate.stride(0), (int)C, n);
  });
  SEQ_CHECK_LAUNCH();
}
