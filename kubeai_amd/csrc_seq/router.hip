// Token routing for mixtures of experts: top-k of fp32 router logits with a
// softmax over the chosen ones, and the experts' squared-ReLU activation
// with the routing weight folded in.
#include "seq_common.h"

namespace {

// One thread per token. The k-th choice is the largest logit that comes
// after the previous choice in the order (value descending, index ascending),
// so equal logits resolve to the lower index and no selection mask is kept.
// weights[t, :] is the softmax over the chosen logits; dense[t, e] holds the
// same weight at the expert's column and 0 elsewhere.
__global__ void router_topk_kernel(const float* __restrict__ logits,
                                   float* __restrict__ dense,
                                   float* __restrict__ weights,
                                   int* __restrict__ index, int T, int E, int top) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + (size_t)t * E;
  for (int e = 0; e < E; ++e) dense[(size_t)t * E + e] = 0.f;
  float last_v = INFINITY, zmax = 0.f, sum = 0.f;
  int last_i = -1;
  for (int k = 0; k < top; ++k) {
    float best_v = -INFINITY;
    int best_i = -1;
    for (int e = 0; e < E; ++e) {
      const float v = z[e];
      const bool after = v < last_v || (v == last_v && e > last_i);
      if (after && (best_i < 0 || v > best_v)) {
        best_v = v;
        best_i = e;
      }
    }
    if (best_i < 0) best_i = 0, best_v = z[0];  // NaN logits: stay in range
    if (k == 0) zmax = best_v;
    const float p = expf(best_v - zmax);
    sum += p;
    weights[(size_t)t * top + k] = p;
    index[(size_t)t * top + k] = best_i;
    last_v = best_v;
    last_i = best_i;
  }
  const float inv = 1.0f / sum;
  for (int k = 0; k < top; ++k) {
    const float w = weights[(size_t)t * top + k] * inv;
    weights[(size_t)t * top + k] = w;
    dense[(size_t)t * E + index[(size_t)t * top + k]] = w;
  }
}

// out[t, c] = relu(u[t, c])^2 * w[t, c / group] for c < groups * group,
// and relu(u)^2 beyond (columns of an expert that every token uses).
template <typename T>
__global__ void relu_squared_weighted_kernel(T* __restrict__ out,
                                             const T* __restrict__ u,
                                             const float* __restrict__ w,
                                             int64_t w_stride, int groups,
                                             int group, int C, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t t = i / C;
  const int c = (int)(i % C);
  const float r = fmaxf(ldf(u + i), 0.f);
  const int g = c / group;
  const float s = g < groups ? w[t * w_stride + g] : 1.f;
  stf(out + i, r * r * s);
}

// One thread per token: scores s = softmax(logits) over all experts; the
// `top` experts with the largest s + bias are chosen in the order (value
// descending, index ascending); their weights are their scores s as they
// are, times wscale. dense[t, e] holds the weight at a chosen expert's column, else 0.
// The scores live in dense's row until the choice is made.
__global__ void router_scores_topk_kernel(const float* __restrict__ logits,
                                          const float* __restrict__ bias,
                                          float* __restrict__ dense,
                                          float* __restrict__ weights,
                                          int* __restrict__ index, int T, int E,
                                          int top, float wscale) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + (size_t)t * E;
  float* s = dense + (size_t)t * E;
  float zmax = -INFINITY;
  for (int e = 0; e < E; ++e) zmax = fmaxf(zmax, z[e]);
  float sum = 0.f;
  for (int e = 0; e < E; ++e) {
    const float p = expf(z[e] - zmax);
    s[e] = p;
    sum += p;
  }
  for (int e = 0; e < E; ++e) s[e] = s[e] / sum;
  float last_v = INFINITY;
  int last_i = -1;
  for (int k = 0; k < top; ++k) {
    float best_v = -INFINITY;
    int best_i = -1;
    for (int e = 0; e < E; ++e) {
      const float v = s[e] + (bias != nullptr ? bias[e] : 0.f);
      const bool after = v < last_v || (v == last_v && e > last_i);
      if (after && (best_i < 0 || v > best_v)) {
        best_v = v;
        best_i = e;
      }
    }
    if (best_i < 0) best_i = 0, best_v = s[0];  // NaN logits: stay in range
    weights[(size_t)t * top + k] = s[best_i] * wscale;
    index[(size_t)t * top + k] = best_i;
    last_v = best_v;
    last_i = best_i;
  }
  for (int e = 0; e < E; ++e) s[e] = 0.f;
  for (int k = 0; k < top; ++k)
    s[index[(size_t)t * top + k]] = weights[(size_t)t * top + k];
}

// Gated activation over blocks of `group` gate columns followed by `group`
// up columns (gu [T, n * 2 * group], strided rows):
//   g = gate, u = up; limit > 0: g = min(g, limit), u = clamp(u, -limit, limit)
//   out[t, e * group + c] = g * sigmoid(alpha * g) * (u + shift) * weight[t, e]
// weight: absent (1), w itself, or sigmoid(w). One thread per N consecutive
// channels (N = 1, or the elements of a 16-byte access).
struct GluParams {
  float alpha, limit, shift;
  int w_sigmoid;
};

DEV_INLINE float glu_f(float g, float u, const GluParams& p) {
  if (p.limit > 0.f) {
    g = fminf(g, p.limit);
    u = fminf(fmaxf(u, -p.limit), p.limit);
  }
  return g / (1.0f + expf(-p.alpha * g)) * (u + p.shift);
}

template <typename T, bool kVec>
__global__ void glu_weighted_kernel(T* __restrict__ out, int64_t out_stride,
                                    const T* __restrict__ gu, int64_t gu_stride,
                                    const float* __restrict__ w, int64_t w_stride,
                                    int group, int C, int64_t n, GluParams p) {
  constexpr int N = kVec ? Vec16<T>::N : 1;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int cpr = C / N;  // threads per row
  const int64_t t = i / cpr;
  const int c = (int)(i % cpr) * N;
  const int e = c / group, j = c % group;
  const T* row = gu + t * gu_stride + (size_t)e * 2 * group;
  float wt = 1.f;
  if (w != nullptr) {
    wt = w[t * w_stride + e];
    if (p.w_sigmoid) wt = sigmoid_f(wt);
  }
  if constexpr (kVec) {
    float g[N], u[N];
    Vec16<T>::load(row + j, g);
    Vec16<T>::load(row + group + j, u);
#pragma unroll
    for (int x = 0; x < N; ++x) g[x] = glu_f(g[x], u[x], p) * wt;
    Vec16<T>::store(out + t * out_stride + c, g);
  } else {
    stf(out + t * out_stride + c, glu_f(ldf(row + j), ldf(row + group + j), p) * wt);
  }
}

}  // namespace

void router_scores_topk(torch::Tensor logits, c10::optional<torch::Tensor> bias,
                        torch::Tensor dense, torch::Tensor weights,
                        torch::Tensor index, double scale) {
  check_f32(logits, "logits");
  check_f32(dense, "dense");
  check_f32(weights, "weights");
  check_i32(index, "index");
  TORCH_CHECK(logits.dim() == 2 && weights.dim() == 2);
  const int T = logits.size(0), E = logits.size(1), top = weights.size(1);
  TORCH_CHECK(top >= 1 && top <= E, "top must be within the number of experts");
  TORCH_CHECK(dense.numel() == (int64_t)T * E && weights.size(0) == T &&
              index.numel() == (int64_t)T * top);
  const float* bp = nullptr;
  if (bias.has_value()) {
    check_f32(*bias, "bias");
    TORCH_CHECK(bias->numel() == E);
    bp = (const float*)bias->data_ptr();
  }
  if (T == 0) return;
  hipLaunchKernelGGL(router_scores_topk_kernel, dim3((T + 63) / 64), dim3(64), 0,
                     SEQ_STREAM(), (const float*)logits.data_ptr(), bp,
                     (float*)dense.data_ptr(), (float*)weights.data_ptr(),
                     (int*)index.data_ptr(), T, E, top, (float)scale);
  SEQ_CHECK_LAUNCH();
}

void glu_weighted(torch::Tensor out, torch::Tensor gu, c10::optional<torch::Tensor> w,
                  int64_t group, double alpha, double limit, double up_shift,
                  bool w_sigmoid) {
  check_rows(gu, "gu");
  check_rows(out, "out");
  TORCH_CHECK(out.scalar_type() == gu.scalar_type());
  TORCH_CHECK(group > 0 && gu.size(1) % (2 * group) == 0);
  const int64_t T = gu.size(0);
  const int C = gu.size(1) / 2, n_exp = C / group;
  TORCH_CHECK(out.size(0) == T && out.size(1) == C);
  const float* wp = nullptr;
  int64_t ws = 0;
  if (w.has_value()) {
    TORCH_CHECK(w->is_cuda() && w->scalar_type() == torch::kFloat32 && w->dim() == 2 &&
                w->size(0) == T && w->size(1) == n_exp &&
                (w->size(1) == 1 || w->stride(1) == 1));
    wp = (const float*)w->data_ptr();
    ws = w->stride(0);
  }
  if (T == 0 || C == 0) return;
  const GluParams p{(float)alpha, (float)limit, (float)up_shift, w_sigmoid ? 1 : 0};
  const int vn = 16 / gu.element_size();
  const bool vec = group % vn == 0 && gu.stride(0) % vn == 0 && out.stride(0) % vn == 0 &&
                   ((size_t)gu.data_ptr()) % 16 == 0 && ((size_t)out.data_ptr()) % 16 == 0;
  SEQ_DISPATCH_ACT(gu, {
    auto launch = [&](auto kern, int per) {
      const int64_t n = T * (C / per);
      hipLaunchKernelGGL(kern, dim3((n + 255) / 256), dim3(256), 0, SEQ_STREAM(),
                         (act_t*)out.data_ptr(), out.stride(0),
                         (const act_t*)gu.data_ptr(), gu.stride(0), wp, ws, (int)group, C,
                         n, p);
    };
    if (vec) launch(glu_weighted_kernel<act_t, true>, vn);
    else launch(glu_weighted_kernel<act_t, false>, 1);
  });
  SEQ_CHECK_LAUNCH();
}

void router_topk(torch::Tensor logits, torch::Tensor dense, torch::Tensor weights,
                 torch::Tensor index) {
  check_f32(logits, "logits");
  check_f32(dense, "dense");
  check_f32(weights, "weights");
  check_i32(index, "index");
  TORCH_CHECK(logits.dim() == 2 && weights.dim() == 2);
  const int T = logits.size(0), E = logits.size(1), top = weights.size(1);
  TORCH_CHECK(top >= 1 && top <= E, "top must be within the number of experts");
  TORCH_CHECK(dense.numel() == (int64_t)T * E && weights.size(0) == T &&
              index.numel() == (int64_t)T * top);
  if (T == 0) return;
  hipLaunchKernelGGL(router_topk_kernel, dim3((T + 63) / 64), dim3(64), 0,
                     SEQ_STREAM(), (const float*)logits.data_ptr(),
                     (float*)dense.data_ptr(), (float*)weights.data_ptr(),
                     (int*)index.data_ptr(), T, E, top);
  SEQ_CHECK_LAUNCH();
}

void relu_squared_weighted(torch::Tensor out, torch::Tensor u, torch::Tensor w,
                           int64_t group) {
  TORCH_CHECK(u.is_contiguous() && out.is_contiguous() && u.is_cuda() &&
              u.dim() == 2 && out.sizes() == u.sizes() &&
              out.scalar_type() == u.scalar_type());
  TORCH_CHECK(w.is_cuda() && w.scalar_type() == torch::kFloat32 && w.dim() == 2 &&
              w.size(0) == u.size(0) && (w.size(1) == 1 || w.stride(1) == 1));
  const int C = u.size(1), groups = w.size(1);
  TORCH_CHECK(group > 0 && (int64_t)groups * group <= C);
  const int64_t n = u.numel();
  if (n == 0) return;
  SEQ_DISPATCH_ACT(u, {
    hipLaunchKernelGGL((relu_squared_weighted_kernel<act_t>), dim3((n + 255) / 256),
                       dim3(256), 0, SEQ_STREAM(), (act_t*)out.data_ptr(),
                       (const act_t*)u.data_ptr(), (const float*)w.data_ptr(),
                       w.stride(0), groups, (int)group, C, n);
  });
  SEQ_CHECK_LAUNCH();
}
