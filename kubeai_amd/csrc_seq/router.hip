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
// are. dense[t, e] holds the weight at a chosen expert's column, else 0.
// The scores live in dense's row until the choice is made.
__global__ void router_scores_topk_kernel(const float* __restrict__ logits,
                                          const float* __restrict__ bias,
                                          float* __restrict__ dense,
                                          float* __restrict__ weights,
                                          int* __restrict__ index, int T, int E,
                                          int top) {
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
    weights[(size_t)t * top + k] = s[best_i];
    index[(size_t)t * top + k] = best_i;
    last_v = best_v;
    last_i = best_i;
  }
  for (int e = 0; e < E; ++e) s[e] = 0.f;
  for (int k = 0; k < top; ++k)
    s[index[(size_t)t * top + k]] = weights[(size_t)t * top + k];
}

// gu [T, n * 2 * group]: per expert `group` gate columns, then `group` up
// columns. out[t, e * group + c] = silu(gate) * up * w[t, e].
template <typename T>
__global__ void silu_mul_weighted_kernel(T* __restrict__ out, const T* __restrict__ gu,
                                         const float* __restrict__ w, int64_t w_stride,
                                         int group, int C, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t t = i / C;
  const int c = (int)(i % C);
  const int e = c / group, j = c % group;
  const T* row = gu + t * 2 * C + (size_t)e * 2 * group;
  const float g = ldf(row + j), u = ldf(row + group + j);
  stf(out + i, silu_f(g) * u * w[t * w_stride + e]);
}

}  // namespace

void router_scores_topk(torch::Tensor logits, c10::optional<torch::Tensor> bias,
                        torch::Tensor dense, torch::Tensor weights,
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
                     (int*)index.data_ptr(), T, E, top);
  SEQ_CHECK_LAUNCH();
}

void silu_mul_weighted(torch::Tensor out, torch::Tensor gu, torch::Tensor w,
                       int64_t group) {
  TORCH_CHECK(gu.is_contiguous() && out.is_contiguous() && gu.is_cuda() &&
              gu.dim() == 2 && out.dim() == 2 && out.scalar_type() == gu.scalar_type());
  TORCH_CHECK(group > 0 && gu.size(1) % (2 * group) == 0);
  const int64_t T = gu.size(0);
  const int C = gu.size(1) / 2, n_exp = C / group;
  TORCH_CHECK(out.size(0) == T && out.size(1) == C);
  TORCH_CHECK(w.is_cuda() && w.scalar_type() == torch::kFloat32 && w.dim() == 2 &&
              w.size(0) == T && w.size(1) == n_exp &&
              (w.size(1) == 1 || w.stride(1) == 1));
  const int64_t n = T * C;
  if (n == 0) return;
  SEQ_DISPATCH_ACT(gu, {
    hipLaunchKernelGGL((silu_mul_weighted_kernel<act_t>), dim3((n + 255) / 256),
                       dim3(256), 0, SEQ_STREAM(), (act_t*)out.data_ptr(),
                       (const act_t*)gu.data_ptr(), (const float*)w.data_ptr(),
                       w.stride(0), (int)group, C, n);
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
