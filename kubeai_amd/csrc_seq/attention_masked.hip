// Rotary on interleaved pairs fused with the paged cache write, and softmax
// attention of every packed token over its own sequence's cached keys under
// a chunk / window mask, with separate key and value sizes.
#include "seq_common.h"

namespace {

// grid (T): q pairs rotate in place; k pairs rotate into the key cache;
// v copies into the value cache. Angles are fp32: position * inv_freq[i].
template <typename T>
__global__ void rope_pairs_cache_kernel(
    T* __restrict__ q, int64_t q_stride, const T* __restrict__ k,
    int64_t k_stride, const T* __restrict__ v, int64_t v_stride,
    const int* __restrict__ positions, const float* __restrict__ inv_freq,
    int half, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, int H, int G, int D, int Dv,
    int bs) {
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  const int64_t slot = slot_mapping[t];
  const int hp = D / 2;
  const int nqp = H * hp, nkp = G * hp, nv = G * Dv;
  const int64_t blk = slot >= 0 ? slot / bs : 0;
  const int off = slot >= 0 ? (int)(slot % bs) : 0;
  for (int u = threadIdx.x; u < nqp + nkp + nv; u += blockDim.x) {
    if (u < nqp + nkp) {
      const bool is_q = u < nqp;
      const int uu = is_q ? u : u - nqp;
      const int hd = uu / hp, i = uu % hp;
      const T* src = is_q ? q + (size_t)t * q_stride + hd * D + 2 * i
                          : k + (size_t)t * k_stride + hd * D + 2 * i;
      float a = ldf(src), b = ldf(src + 1);
      if (i < half) {
        float sn, cs;
        sincosf(pos * inv_freq[i], &sn, &cs);
        const float ra = a * cs - b * sn, rb = b * cs + a * sn;
        a = ra;
        b = rb;
      }
      if (is_q) {
        if (i < half) {
          T* dst = q + (size_t)t * q_stride + hd * D + 2 * i;
          stf(dst, a);
          stf(dst + 1, b);
        }
      } else if (slot >= 0) {
        T* dst = k_cache + (((size_t)blk * G + hd) * bs + off) * D + 2 * i;
        stf(dst, a);
        stf(dst + 1, b);
      }
    } else if (slot >= 0) {
      const int e = u - nqp - nkp;
      const int g = e / Dv, d = e % Dv;
      v_cache[(((size_t)blk * G + g) * bs + off) * Dv + d] =
          v[(size_t)t * v_stride + g * Dv + d];
    }
  }
}

constexpr int kMaxDvPerLane = 8;  // value size <= 512

// grid (T, H), one wave per (token, query head). Keys are walked in tiles
// of 64: each lane scores one key (fp32 dot, cap, mask), the wave keeps a
// running max / sum, then lanes switch to value channels and accumulate
// p . V for the tile. Serves single decode tokens and prompt portions alike
// (every token reads its keys, including this step's, from the cache).
template <typename T>
__global__ __launch_bounds__(WAVE) void masked_paged_attention_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ q,
    int64_t q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ block_tables,
    int max_blocks, const int* __restrict__ token_seq,
    const int* __restrict__ positions, float scale, float softcap, int chunk,
    int window, float out_scale, int H, int G, int D, int Dv, int bs) {
  extern __shared__ float sm[];
  int64_t* vbase = (int64_t*)sm;          // [64] value row offsets
  float* ps = sm + 2 * WAVE;              // [64] tile probabilities
  float* qs = ps + WAVE;                  // [D]
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (H / G);
  const int pos = positions[t];
  const int* bt = block_tables + (size_t)token_seq[t] * max_blocks;
  int lo = 0;
  if (chunk > 0) lo = (pos / chunk) * chunk;
  if (window > 0) lo = max(lo, pos - window + 1);
  for (int i = lane; i < D; i += WAVE)
    qs[i] = ldf(q + (size_t)t * q_stride + h * D + i);
  __syncthreads();
  float m = -INFINITY, l = 0.f;
  float acc[kMaxDvPerLane];
#pragma unroll
  for (int i = 0; i < kMaxDvPerLane; ++i) acc[i] = 0.f;
  for (int j0 = lo; j0 <= pos; j0 += WAVE) {
    const int j = j0 + lane;
    float sc = -INFINITY;
    int64_t vb = 0;
    if (j <= pos) {
      const int64_t blk = bt[j / bs];
      const int64_t rowi = (blk * G + g) * bs + (j % bs);
      const T* kp = k_cache + rowi * D;
      float dot = 0.f;
      for (int i = 0; i < D; ++i) dot += qs[i] * ldf(kp + i);
      sc = dot * scale;
      if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
      vb = rowi * Dv;
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float p = j <= pos ? expf(sc - m_new) : 0.f;
    const float corr = expf(m - m_new);  // m = -inf on the first tile -> 0
    l = l * corr + wave_sum(p);
    m = m_new;
    __syncthreads();  // previous tile's readers are done
    ps[lane] = p;
    vbase[lane] = vb;
    __syncthreads();
    const int nk = min(WAVE, pos - j0 + 1);
#pragma unroll
    for (int c = 0; c < kMaxDvPerLane; ++c) {
      const int d = c * WAVE + lane;
      if (d < Dv) {
        float a = acc[c] * corr;
        for (int jj = 0; jj < nk; ++jj) a += ps[jj] * ldf(v_cache + vbase[jj] + d);
        acc[c] = a;
      }
    }
  }
  const float inv = out_scale / l;
#pragma unroll
  for (int c = 0; c < kMaxDvPerLane; ++c) {
    const int d = c * WAVE + lane;
    if (d < Dv) stf(out + (size_t)t * out_stride + h * Dv + d, acc[c] * inv);
  }
}

}  // namespace

static bool dense_heads3(const torch::Tensor& t) {
  return t.dim() == 3 && t.stride(2) == 1 && t.stride(1) == t.size(2);
}

void rope_pairs_and_cache(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                          torch::Tensor positions, torch::Tensor inv_freq,
                          torch::Tensor k_cache, torch::Tensor v_cache,
                          torch::Tensor slot_mapping) {
  check_i32(positions, "positions");
  check_f32(inv_freq, "inv_freq");
  TORCH_CHECK(dense_heads3(q) && dense_heads3(k) && dense_heads3(v));
  TORCH_CHECK(slot_mapping.scalar_type() == torch::kInt64 &&
              slot_mapping.is_contiguous());
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k.size(1), Dv = v.size(2), half = inv_freq.numel();
  TORCH_CHECK(D % 2 == 0 && 2 * half <= D, "key size must be even and hold the rotated dims");
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && k.size(2) == D && v.size(1) == G);
  TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4);
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D && v_cache.size(1) == G &&
              v_cache.size(3) == Dv && v_cache.size(2) == k_cache.size(2) &&
              v_cache.size(0) == k_cache.size(0));
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type());
  if (T == 0) return;
  SEQ_DISPATCH_ACT(q, {
    hipLaunchKernelGGL((rope_pairs_cache_kernel<act_t>), dim3(T), dim3(256), 0,
                       SEQ_STREAM(), (act_t*)q.data_ptr(), q.stride(0),
                       (const act_t*)k.data_ptr(), k.stride(0),
                       (const act_t*)v.data_ptr(), v.stride(0),
                       (const int*)positions.data_ptr(),
                       (const float*)inv_freq.data_ptr(), half,
                       (act_t*)k_cache.data_ptr(), (act_t*)v_cache.data_ptr(),
                       (const int64_t*)slot_mapping.data_ptr(), H, G, D, Dv,
                       (int)k_cache.size(2));
  });
  SEQ_CHECK_LAUNCH();
}

void masked_paged_attention(torch::Tensor out, torch::Tensor q,
                            torch::Tensor k_cache, torch::Tensor v_cache,
                            torch::Tensor block_tables, torch::Tensor token_seq,
                            torch::Tensor positions, double scale,
                            double softcap, int64_t chunk, int64_t window,
                            double out_scale) {
  check_i32(block_tables, "block_tables");
  check_i32(token_seq, "token_seq");
  check_i32(positions, "positions");
  TORCH_CHECK(dense_heads3(q) && dense_heads3(out));
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4);
  const int G = k_cache.size(1), bs = k_cache.size(2), Dv = v_cache.size(3);
  TORCH_CHECK(k_cache.size(3) == D && v_cache.size(1) == G && v_cache.size(2) == bs);
  TORCH_CHECK(G > 0 && H % G == 0 && H <= 65535);
  TORCH_CHECK(out.size(0) == T && out.size(1) == H && out.size(2) == Dv);
  TORCH_CHECK(Dv <= kMaxDvPerLane * WAVE, "value size too large");
  TORCH_CHECK(block_tables.dim() == 2 && token_seq.numel() == T &&
              positions.numel() == T);
  TORCH_CHECK(k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type() &&
              out.scalar_type() == q.scalar_type());
  if (T == 0) return;
  const size_t lds = (size_t)(D + WAVE) * 4 + WAVE * 8;
  SEQ_DISPATCH_ACT(q, {
    hipLaunchKernelGGL((masked_paged_attention_kernel<act_t>), dim3(T, H),
                       dim3(WAVE), lds, SEQ_STREAM(), (act_t*)out.data_ptr(),
                       out.stride(0), (const act_t*)q.data_ptr(), q.stride(0),
                       (const act_t*)k_cache.data_ptr(),
                       (const act_t*)v_cache.data_ptr(),
                       (const int*)block_tables.data_ptr(),
                       (int)block_tables.size(1), (const int*)token_seq.data_ptr(),
                       (const int*)positions.data_ptr(), (float)scale,
                       (float)softcap, (int)chunk, (int)window, (float)out_scale,
                       H, G, D, Dv, bs);
  });
  SEQ_CHECK_LAUNCH();
}
