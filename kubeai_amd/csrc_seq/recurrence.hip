// Recurrences over the runs of a packed step: the elementwise gated
// recurrence (minGRU) and matrix-state linear attention (per-token channel
// decay with a current-token bonus, or a constant per-head decay). State is
// fp32, one slot per sequence; a run that starts at position 0 starts from
// zero whatever its slot holds.
#include "seq_common.h"

namespace {

// grid (n_seq, ceil(n / 256)): one thread walks one channel of one run.
template <typename T>
__global__ void mingru_scan_kernel(
    T* __restrict__ y, const T* __restrict__ zxg, const float* __restrict__ bz,
    const float* __restrict__ bx, float* __restrict__ state,
    const int* __restrict__ start_loc, const int* __restrict__ slots,
    const int* __restrict__ positions, int n) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= n) return;
  const int s0 = start_loc[s], s1 = start_loc[s + 1], slot = slots[s];
  if (s1 <= s0) return;
  float S = (slot >= 0 && positions[s0] > 0) ? state[(size_t)slot * n + c] : 0.f;
  const float bzc = bz[c], bxc = bx[c];
  for (int t = s0; t < s1; ++t) {
    const T* row = zxg + (size_t)t * 3 * n;
    const float z = sigmoid_f(ldf(row + c) + bzc);
    const float u = ldf(row + n + c) + bxc;
    const float g = ldf(row + 2 * n + c);
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
    S = (1.0f - z) * S + z * cand;
    stf(y + (size_t)t * n + c, S * silu_f(g));
  }
  if (slot >= 0) state[(size_t)slot * n + c] = S;
}

constexpr int kScanTile = 16;  // tokens staged per barrier

// grid (n_seq * H), block = Dv rounded up to a wave. The head's state
// S[D][Dv] lives in LDS; thread j owns column j (value channel j), so the
// token loop needs no barrier. q/k/decay/v of kScanTile tokens are staged
// per barrier with activations and decays applied once per element.
template <typename T, bool kPerToken>
__global__ void linear_attn_scan_kernel(
    float* __restrict__ o, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, const T* __restrict__ decay_pre, int64_t d_stride,
    const float* __restrict__ decay_const, const float* __restrict__ bonus,
    const float* __restrict__ w_bias, float* __restrict__ state,
    const int* __restrict__ start_loc, const int* __restrict__ slots,
    const int* __restrict__ positions, int H, int D, int Dv, int silu_inputs) {
  const int s = blockIdx.x / H, h = blockIdx.x % H;
  const int s0 = start_loc[s], s1 = start_loc[s + 1], slot = slots[s];
  if (s1 <= s0) return;
  extern __shared__ float sm[];
  float* S = sm;                       // [D][Dv]
  float* qs = S + (size_t)D * Dv;      // [tile][D]
  float* ks = qs + kScanTile * D;
  float* ws = ks + kScanTile * D;      // decays (per-token form)
  float* us = ws + kScanTile * D;      // bonus [D]
  float* vs = us + D;                  // [tile][Dv]
  const int tid = threadIdx.x, nthr = blockDim.x;
  const bool carry = slot >= 0 && positions[s0] > 0;
  float* sp = state + ((size_t)(slot < 0 ? 0 : slot) * H + h) * D * Dv;
  for (int i = tid; i < D * Dv; i += nthr) S[i] = carry ? sp[i] : 0.f;
  if (kPerToken)
    for (int i = tid; i < D; i += nthr) us[i] = bonus[h * D + i];
  const float dc = kPerToken ? 0.f : decay_const[h];
  for (int t0 = s0; t0 < s1; t0 += kScanTile) {
    const int nt = min(kScanTile, s1 - t0);
    __syncthreads();  // the previous tile's readers are done
    for (int i = tid; i < nt * D; i += nthr) {
      const int tt = i / D, d = i % D;
      float qv = ldf(q + (size_t)(t0 + tt) * q_stride + h * D + d);
      float kv = ldf(k + (size_t)(t0 + tt) * k_stride + h * D + d);
      if (silu_inputs) { qv = silu_f(qv); kv = silu_f(kv); }
      qs[i] = qv;
      ks[i] = kv;
      if (kPerToken)
        ws[i] = expf(-expf(ldf(decay_pre + (size_t)(t0 + tt) * d_stride + h * D + d) +
                           w_bias[h * D + d]));
    }
    for (int i = tid; i < nt * Dv; i += nthr) {
      const int tt = i / Dv, d = i % Dv;
      float vv = ldf(v + (size_t)(t0 + tt) * v_stride + h * Dv + d);
      if (silu_inputs) vv = silu_f(vv);
      vs[i] = vv;
    }
    __syncthreads();
    if (tid < Dv) {
      for (int tt = 0; tt < nt; ++tt) {
        const float vj = vs[tt * Dv + tid];
        const float* qt = qs + tt * D;
        const float* kt = ks + tt * D;
        float acc = 0.f;
        if (kPerToken) {
          const float* wt = ws + tt * D;
          for (int i = 0; i < D; ++i) {
            const float st = S[i * Dv + tid];
            const float kv = kt[i] * vj;
            acc += qt[i] * (st + us[i] * kv);
            S[i * Dv + tid] = wt[i] * st + kv;
          }
        } else {
          for (int i = 0; i < D; ++i) {
            const float st = dc * S[i * Dv + tid] + kt[i] * vj;
            S[i * Dv + tid] = st;
            acc += qt[i] * st;
          }
        }
        o[((size_t)(t0 + tt) * H + h) * Dv + tid] = acc;
      }
    }
  }
  __syncthreads();
  if (slot >= 0)
    for (int i = tid; i < D * Dv; i += nthr) sp[i] = S[i];
}

}  // namespace

void mingru_scan(torch::Tensor y, torch::Tensor zxg, torch::Tensor bz,
                 torch::Tensor bx, torch::Tensor state, torch::Tensor start_loc,
                 torch::Tensor slots, torch::Tensor positions) {
  check_f32(bz, "bz");
  check_f32(bx, "bx");
  check_f32(state, "state");
  check_i32(start_loc, "start_loc");
  check_i32(slots, "slots");
  check_i32(positions, "positions");
  const int n = bz.numel();
  TORCH_CHECK(zxg.is_contiguous() && zxg.dim() == 2 && zxg.size(1) == 3 * n);
  TORCH_CHECK(y.is_contiguous() && y.size(0) == zxg.size(0) && y.size(1) == n &&
              y.scalar_type() == zxg.scalar_type());
  TORCH_CHECK(bx.numel() == n && state.dim() == 2 && state.size(1) == n);
  TORCH_CHECK(start_loc.numel() == slots.numel() + 1 &&
              positions.numel() == zxg.size(0));
  const int n_seq = slots.numel();
  if (n_seq == 0 || zxg.size(0) == 0) return;
  SEQ_DISPATCH_ACT(zxg, {
    hipLaunchKernelGGL((mingru_scan_kernel<act_t>), dim3(n_seq, (n + 255) / 256),
                       dim3(256), 0, SEQ_STREAM(), (act_t*)y.data_ptr(),
                       (const act_t*)zxg.data_ptr(), (const float*)bz.data_ptr(),
                       (const float*)bx.data_ptr(), (float*)state.data_ptr(),
                       (const int*)start_loc.data_ptr(), (const int*)slots.data_ptr(),
                       (const int*)positions.data_ptr(), n);
  });
  SEQ_CHECK_LAUNCH();
}

void linear_attn_scan(torch::Tensor o, torch::Tensor q, torch::Tensor k,
                      torch::Tensor v, torch::Tensor decay,
                      c10::optional<torch::Tensor> bonus,
                      c10::optional<torch::Tensor> w_bias, torch::Tensor state,
                      torch::Tensor start_loc, torch::Tensor slots,
                      torch::Tensor positions, bool silu_inputs) {
  check_f32(o, "o");
  check_f32(state, "state");
  check_i32(start_loc, "start_loc");
  check_i32(slots, "slots");
  check_i32(positions, "positions");
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3);
  const int T = q.size(0), H = q.size(1), D = q.size(2), Dv = v.size(2);
  auto dense_heads = [](const torch::Tensor& t) {
    return t.stride(2) == 1 && t.stride(1) == t.size(2);
  };
  TORCH_CHECK(dense_heads(q) && dense_heads(k) && dense_heads(v),
              "q/k/v heads must be dense within a row");
  TORCH_CHECK(k.size(0) == T && k.size(1) == H && k.size(2) == D &&
              v.size(0) == T && v.size(1) == H);
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type());
  TORCH_CHECK(o.size(0) == T && o.size(1) == H && o.size(2) == Dv);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D &&
              state.size(3) == Dv);
  TORCH_CHECK(start_loc.numel() == slots.numel() + 1 && positions.numel() == T);
  const bool per_token = decay.dim() == 3;
  if (per_token) {
    TORCH_CHECK(decay.size(0) == T && decay.size(1) == H && decay.size(2) == D &&
                dense_heads(decay) && decay.scalar_type() == q.scalar_type());
    TORCH_CHECK(bonus.has_value() && w_bias.has_value());
    check_f32(*bonus, "bonus");
    check_f32(*w_bias, "w_bias");
    TORCH_CHECK(bonus->numel() == H * D && w_bias->numel() == H * D);
  } else {
    check_f32(decay, "decay");
    TORCH_CHECK(decay.numel() == H);
  }
  const int n_seq = slots.numel();
  if (n_seq == 0 || T == 0) return;
  const int threads = ((Dv + WAVE - 1) / WAVE) * WAVE;
  TORCH_CHECK(threads <= 1024, "value size too large");
  const size_t lds =
      ((size_t)D * Dv + 3 * kScanTile * D + D + kScanTile * Dv) * sizeof(float);
  TORCH_CHECK(lds <= 160 * 1024, "head state does not fit LDS");
  SEQ_DISPATCH_ACT(q, {
    auto launch = [&](auto kern) {
      if (lds > 48 * 1024)
        hipFuncSetAttribute((const void*)kern,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      hipLaunchKernelGGL(kern, dim3(n_seq * H), dim3(threads), lds, SEQ_STREAM(),
                         (float*)o.data_ptr(), (const act_t*)q.data_ptr(),
                         q.stride(0), (const act_t*)k.data_ptr(), k.stride(0),
                         (const act_t*)v.data_ptr(), v.stride(0),
                         per_token ? (const act_t*)decay.data_ptr() : nullptr,
                         per_token ? decay.stride(0) : 0,
                         per_token ? nullptr : (const float*)decay.data_ptr(),
                         per_token ? (const float*)bonus->data_ptr() : nullptr,
                         per_token ? (const float*)w_bias->data_ptr() : nullptr,
                         (float*)state.data_ptr(), (const int*)start_loc.data_ptr(),
                         (const int*)slots.data_ptr(),
                         (const int*)positions.data_ptr(), H, D, Dv,
                         silu_inputs ? 1 : 0);
    };
    if (per_token) launch(linear_attn_scan_kernel<act_t, true>);
    else launch(linear_attn_scan_kernel<act_t, false>);
  });
  SEQ_CHECK_LAUNCH();
}
