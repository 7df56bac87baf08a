// Kernels around several residual streams and differential attention:
// embedding lookup + sinusoidal position vector into every stream, the fused
// stream update / read / RMS norm between sublayers, the query temperature +
// paged cache write for caches whose value heads are fewer than their key
// heads, and the join of two attention maps (difference, per-head RMS norm).
#include "seq_common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kMaxStreams = 8;

// grid (T). out[t, s, c] = table[id, c] * scale + (c odd ? cos : sin)(pos * freqs[c / 2])
// for every stream s. The angle is formed and reduced to [0, 2 pi) in double
// (an fp32 product loses the phase at positions in the thousands); sinf /
// cosf are the precise library functions.
template <typename T>
__global__ __launch_bounds__(kBlock) void embed_sinusoid_kernel(
    float* __restrict__ out, const int* __restrict__ ids, const T* __restrict__ table,
    float scale, const int* __restrict__ positions, const double* __restrict__ freqs,
    int S, int C) {
  const int t = blockIdx.x;
  const T* row = table + (size_t)ids[t] * C;
  const double p = (double)positions[t];
  constexpr double kTwoPi = 6.283185307179586476925;
  for (int c = threadIdx.x; c < C; c += kBlock) {
    double a = p * freqs[c >> 1];
    a -= kTwoPi * floor(a / kTwoPi);
    const float ang = (float)a;
    const float x = ldf(row + c) * scale + ((c & 1) ? cosf(ang) : sinf(ang));
    for (int s = 0; s < S; ++s) out[((size_t)t * S + s) * C + c] = x;
  }
}

// One block per token; streams [T, S, C] fp32.
//   z = y * sigmoid(gate);  x_t <- sum_s mix[s, t] x_s + wr[t] * z   (y given)
//   u = sum_s rd[s] x_s;  out = u / sqrt(mean(u^2) + eps) * w
// y is of type A (the serving dtype, or fp32 for a branch accumulated in
// fp32), the gate's pre-activation of the serving dtype. u is staged in LDS.
template <typename T, typename A>
__global__ __launch_bounds__(kBlock) void hyper_mix_rmsnorm_kernel(
    T* __restrict__ out, float* __restrict__ streams, const A* __restrict__ y,
    const T* __restrict__ gate, int64_t gate_stride, const float* __restrict__ mix,
    const float* __restrict__ wr, const float* __restrict__ rd,
    const float* __restrict__ w, int S, int C, float eps) {
  extern __shared__ float row[];
  __shared__ float red[16];
  __shared__ float cm[kMaxStreams * kMaxStreams + 2 * kMaxStreams];
  float* cw = cm + kMaxStreams * kMaxStreams;
  float* cr = cw + kMaxStreams;
  const int t = blockIdx.x;
  if (threadIdx.x < S * S && y != nullptr) cm[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    cw[threadIdx.x] = y != nullptr ? wr[threadIdx.x] : 0.f;
    cr[threadIdx.x] = rd[threadIdx.x];
  }
  __syncthreads();
  float* xs = streams + (size_t)t * S * C;
  float ss = 0.f;
  for (int c = threadIdx.x; c < C; c += kBlock) {
    float x[kMaxStreams];
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s)
      if (s < S) x[s] = xs[(size_t)s * C + c];
    float u = 0.f;
    if (y != nullptr) {
      float z = ldf(y + (size_t)t * C + c);
      if (gate != nullptr) z *= sigmoid_f(ldf(gate + (size_t)t * gate_stride + c));
#pragma unroll
      for (int d = 0; d < kMaxStreams; ++d) {
        if (d < S) {
          float acc = cw[d] * z;
#pragma unroll
          for (int s = 0; s < kMaxStreams; ++s)
            if (s < S) acc += cm[s * S + d] * x[s];
          xs[(size_t)d * C + c] = acc;
          u += cr[d] * acc;
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s)
        if (s < S) u += cr[s] * x[s];
    }
    row[c] = u;
    ss += u * u;
  }
  // every thread re-reads only the entries it wrote
  const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)C + eps);
  for (int c = threadIdx.x; c < C; c += kBlock)
    stf(out + (size_t)t * C + c, row[c] * r * w[c]);
}

// grid (T). q rows are scaled in place by the temperature of their position,
// k and v rows are copied to their caches (their head counts may differ).
template <typename T>
__global__ __launch_bounds__(kBlock) void scale_q_cache_kernel(
    T* __restrict__ q, int64_t q_stride, const T* __restrict__ k, int64_t k_stride,
    const T* __restrict__ v, int64_t v_stride, const int* __restrict__ positions,
    float coef, int every, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, int nq, int G, int D, int Gv, int Dv,
    int bs) {
  const int t = blockIdx.x;
  if (coef != 0.f) {
    const float temp = 1.0f + coef * logf((float)((positions[t] + 1) / every) + 1.0f);
    T* qr = q + (size_t)t * q_stride;
    for (int i = threadIdx.x; i < nq; i += kBlock) stf(qr + i, ldf(qr + i) * temp);
  }
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;
  const int64_t blk = slot / bs, off = slot % bs;
  const T* kr = k + (size_t)t * k_stride;
  for (int i = threadIdx.x; i < G * D; i += kBlock) {
    const int g = i / D, d = i % D;
    k_cache[((blk * G + g) * bs + off) * D + d] = kr[i];
  }
  const T* vr = v + (size_t)t * v_stride;
  for (int i = threadIdx.x; i < Gv * Dv; i += kBlock) {
    const int g = i / Dv, d = i % Dv;
    v_cache[((blk * Gv + g) * bs + off) * Dv + d] = vr[i];
  }
}

// One wave per (token, head). att [T, G, 2, R, Dv]: o = map 0 - lam * map 1,
// out = o / sqrt(mean(o^2) + eps) * gain.
template <typename T>
__global__ __launch_bounds__(kBlock) void diff_combine_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ att, float lam,
    float gain, float eps, int64_t n_rows, int G, int R, int Dv) {
  const int64_t idx = (int64_t)blockIdx.x * (kBlock / WAVE) + threadIdx.x / WAVE;
  if (idx >= n_rows) return;
  const int lane = threadIdx.x % WAVE;
  const int H = G * R;
  const int64_t t = idx / H;
  const int h = (int)(idx % H), g = h / R, r = h % R;
  const T* a1 = att + (((t * G + g) * 2 + 0) * R + r) * (int64_t)Dv;
  const T* a2 = att + (((t * G + g) * 2 + 1) * R + r) * (int64_t)Dv;
  float ss = 0.f;
  for (int d = lane; d < Dv; d += WAVE) {
    const float o = ldf(a1 + d) - lam * ldf(a2 + d);
    ss += o * o;
  }
  const float rn = gain / sqrtf(wave_sum(ss) / (float)Dv + eps);
  T* op = out + t * out_stride + (int64_t)h * Dv;
  for (int d = lane; d < Dv; d += WAVE) stf(op + d, (ldf(a1 + d) - lam * ldf(a2 + d)) * rn);
}

}  // namespace

void embed_sinusoid(torch::Tensor out, torch::Tensor ids, torch::Tensor table,
                    double scale, torch::Tensor positions, torch::Tensor freqs) {
  check_f32(out, "out");
  check_i32(ids, "ids");
  check_i32(positions, "positions");
  TORCH_CHECK(freqs.scalar_type() == torch::kFloat64 && freqs.is_contiguous() &&
              freqs.is_cuda(), "freqs must be a contiguous float64 GPU tensor");
  TORCH_CHECK(table.is_cuda() && table.is_contiguous() && table.dim() == 2 &&
              out.dim() == 3);
  const int T = out.size(0), S = out.size(1), C = out.size(2);
  TORCH_CHECK(table.size(1) == C && ids.numel() == T && positions.numel() == T &&
              freqs.numel() >= (C + 1) / 2);
  if (T == 0) return;
  SEQ_DISPATCH_ACT(table, {
    hipLaunchKernelGGL((embed_sinusoid_kernel<act_t>), dim3(T), dim3(kBlock), 0,
                       SEQ_STREAM(), (float*)out.data_ptr(), (const int*)ids.data_ptr(),
                       (const act_t*)table.data_ptr(), (float)scale,
                       (const int*)positions.data_ptr(), (const double*)freqs.data_ptr(),
                       S, C);
  });
  SEQ_CHECK_LAUNCH();
}

void hyper_mix_rmsnorm(torch::Tensor out, torch::Tensor streams,
                       c10::optional<torch::Tensor> y, c10::optional<torch::Tensor> gate,
                       c10::optional<torch::Tensor> mix,
                       c10::optional<torch::Tensor> write_w, torch::Tensor read_w,
                       torch::Tensor weight, double eps) {
  check_f32(streams, "streams");
  check_f32(read_w, "read_w");
  check_f32(weight, "weight");
  TORCH_CHECK(streams.dim() == 3 && out.is_cuda() && out.is_contiguous() && out.dim() == 2);
  const int T = streams.size(0), S = streams.size(1), C = streams.size(2);
  TORCH_CHECK(S >= 1 && S <= kMaxStreams, "1 to ", kMaxStreams, " streams");
  TORCH_CHECK(out.size(0) == T && out.size(1) == C && weight.numel() == C &&
              read_w.numel() == S);
  TORCH_CHECK((size_t)C * 4 <= 60 * 1024, "row too wide for the LDS row cache");
  const void* yp = nullptr;
  bool wide = false;
  const float *mp = nullptr, *wp = nullptr;
  const void* gp = nullptr;
  int64_t gs = 0;
  if (y.has_value()) {
    TORCH_CHECK(y->is_cuda() && y->is_contiguous() && y->dim() == 2 && y->size(0) == T &&
                y->size(1) == C);
    wide = y->scalar_type() == torch::kFloat32;
    TORCH_CHECK(wide || y->scalar_type() == out.scalar_type(),
                "the branch must be fp32 or the output's dtype");
    yp = y->data_ptr();
    TORCH_CHECK(mix.has_value() && write_w.has_value(), "a branch needs mix and write weights");
    check_f32(*mix, "mix");
    check_f32(*write_w, "write_w");
    TORCH_CHECK(mix->numel() == S * S && write_w->numel() == S);
    mp = (const float*)mix->data_ptr();
    wp = (const float*)write_w->data_ptr();
    if (gate.has_value()) {
      check_rows(*gate, "gate");
      TORCH_CHECK(gate->size(0) == T && gate->size(1) == C &&
                  gate->scalar_type() == out.scalar_type());
      gp = gate->data_ptr();
      gs = gate->stride(0);
    }
  }
  if (T == 0) return;
  SEQ_DISPATCH_ACT(out, {
    auto launch = [&](auto kern, auto* yt) {
      hipLaunchKernelGGL(kern, dim3(T), dim3(kBlock), (size_t)C * 4, SEQ_STREAM(),
                         (act_t*)out.data_ptr(), (float*)streams.data_ptr(),
                         (decltype(yt))yp, (const act_t*)gp, gs, mp, wp,
                         (const float*)read_w.data_ptr(), (const float*)weight.data_ptr(),
                         S, C, (float)eps);
    };
    const float* f = nullptr;
    const act_t* n = nullptr;
    if (wide) launch(hyper_mix_rmsnorm_kernel<act_t, float>, f);
    else launch(hyper_mix_rmsnorm_kernel<act_t, act_t>, n);
  });
  SEQ_CHECK_LAUNCH();
}

static bool dense_heads(const torch::Tensor& t) {
  return t.is_cuda() && t.dim() == 3 && t.stride(2) == 1 && t.stride(1) == t.size(2);
}

void scale_q_and_cache(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                       torch::Tensor positions, double coef, int64_t every,
                       torch::Tensor k_cache, torch::Tensor v_cache,
                       torch::Tensor slot_mapping) {
  check_i32(positions, "positions");
  TORCH_CHECK(dense_heads(q) && dense_heads(k) && dense_heads(v));
  TORCH_CHECK(slot_mapping.scalar_type() == torch::kInt64 && slot_mapping.is_cuda() &&
              slot_mapping.is_contiguous());
  TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() && v_cache.is_cuda() &&
              v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4);
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k.size(1), Gv = v.size(1), Dv = v.size(2), bs = k_cache.size(2);
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && k.size(2) == D &&
              positions.numel() == T && slot_mapping.numel() == T && every >= 1);
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D && v_cache.size(1) == Gv &&
              v_cache.size(2) == bs && v_cache.size(3) == Dv &&
              v_cache.size(0) == k_cache.size(0),
              "cache shapes do not fit the projections");
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type());
  if (T == 0) return;
  SEQ_DISPATCH_ACT(q, {
    hipLaunchKernelGGL((scale_q_cache_kernel<act_t>), dim3(T), dim3(kBlock), 0,
                       SEQ_STREAM(), (act_t*)q.data_ptr(), q.stride(0),
                       (const act_t*)k.data_ptr(), k.stride(0), (const act_t*)v.data_ptr(),
                       v.stride(0), (const int*)positions.data_ptr(), (float)coef,
                       (int)every, (act_t*)k_cache.data_ptr(), (act_t*)v_cache.data_ptr(),
                       (const int64_t*)slot_mapping.data_ptr(), H * D, G, D, Gv, Dv, bs);
  });
  SEQ_CHECK_LAUNCH();
}

void diff_combine(torch::Tensor out, torch::Tensor att, double lam, double gain,
                  double eps) {
  TORCH_CHECK(att.is_cuda() && att.is_contiguous() && att.dim() == 5 && att.size(2) == 2);
  const int64_t T = att.size(0);
  const int G = att.size(1), R = att.size(3), Dv = att.size(4);
  TORCH_CHECK(dense_heads(out) && out.size(0) == T && out.size(1) == G * R &&
              out.size(2) == Dv && out.scalar_type() == att.scalar_type());
  const int64_t n_rows = T * G * R;
  if (n_rows == 0) return;
  const int per = kBlock / WAVE;
  SEQ_DISPATCH_ACT(att, {
    hipLaunchKernelGGL((diff_combine_kernel<act_t>), dim3((n_rows + per - 1) / per),
                       dim3(kBlock), 0, SEQ_STREAM(), (act_t*)out.data_ptr(),
                       out.stride(0), (const act_t*)att.data_ptr(), (float)lam,
                       (float)gain, (float)eps, n_rows, G, R, Dv);
  });
  SEQ_CHECK_LAUNCH();
}
