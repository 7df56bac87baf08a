// Kernels of layers whose two sublayers read one norm and are summed: the
// fused residual update (scaled sum of both branches, additions made before a
// pass over a looped span of layers) + next RMS norm, a plain row RMS norm,
// the exact GELU, and the tanh cap of the logits.
#include "seq_common.h"

namespace {

constexpr int kBlock = 256;

// One block per row, the row staged in LDS:
//   x = residual + mult * (a * sa + b * sb) + extra + extra_row
//   residual = x;  out = x / sqrt(mean(x^2) + eps) * w
// a, b are branch outputs of types A, B (each the serving dtype, or fp32 for
// a branch accumulated in fp32); absent terms are null. All arithmetic is fp32.
template <typename T, typename A, typename B>
__global__ __launch_bounds__(kBlock) void scaled_add_rmsnorm_kernel(
    T* __restrict__ out, float* __restrict__ residual, const A* __restrict__ a,
    const float* __restrict__ sa, const B* __restrict__ b,
    const float* __restrict__ sb, float mult, const float* __restrict__ extra,
    const float* __restrict__ extra_row, const float* __restrict__ w, int C,
    float eps) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const size_t base = (size_t)blockIdx.x * C;
  const bool touch = a != nullptr || b != nullptr || extra != nullptr ||
                     extra_row != nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < C; c += kBlock) {
    float x = residual[base + c];
    float br = 0.f;
    if (a != nullptr) br += ldf(a + base + c) * (sa != nullptr ? sa[c] : 1.f);
    if (b != nullptr) br += ldf(b + base + c) * (sb != nullptr ? sb[c] : 1.f);
    x += mult * br;
    if (extra != nullptr) x += extra[base + c];
    if (extra_row != nullptr) x += extra_row[c];
    if (touch) residual[base + c] = x;
    row[c] = x;
    ss += x * x;
  }
  // every thread re-reads only the entries it wrote
  const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)C + eps);
  for (int c = threadIdx.x; c < C; c += kBlock) stf(out + base + c, row[c] * r * w[c]);
}

// grid (T): out row = x row / sqrt(mean(x^2) + eps) * w.
template <typename T>
__global__ __launch_bounds__(kBlock) void rmsnorm_rows_kernel(
    T* __restrict__ out, const T* __restrict__ x, int64_t x_stride,
    const float* __restrict__ w, int C, float eps) {
  __shared__ float red[16];
  const T* xr = x + (size_t)blockIdx.x * x_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < C; c += kBlock) {
    const float v = ldf(xr + c);
    ss += v * v;
  }
  const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)C + eps);
  for (int c = threadIdx.x; c < C; c += kBlock)
    stf(out + (size_t)blockIdx.x * C + c, ldf(xr + c) * r * w[c]);
}

DEV_INLINE float gelu_f(float x) {
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f));
}

template <typename T>
__global__ void gelu_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) stf(out + i, gelu_f(ldf(x + i)));
}

template <typename T>
__global__ void gelu_vec_kernel(T* __restrict__ out, const T* __restrict__ x,
                                int64_t nvec) {
  constexpr int N = Vec16<T>::N;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < nvec) {
    float v[N];
    Vec16<T>::load(x + i * N, v);
#pragma unroll
    for (int e = 0; e < N; ++e) v[e] = gelu_f(v[e]);
    Vec16<T>::store(out + i * N, v);
  }
}

__global__ void tanh_cap_kernel(float* __restrict__ x, float cap, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

}  // namespace

void scaled_add_rmsnorm(torch::Tensor out, torch::Tensor residual,
                        c10::optional<torch::Tensor> a,
                        c10::optional<torch::Tensor> a_scale,
                        c10::optional<torch::Tensor> b,
                        c10::optional<torch::Tensor> b_scale, double mult,
                        c10::optional<torch::Tensor> extra,
                        c10::optional<torch::Tensor> extra_row, torch::Tensor weight,
                        double eps) {
  check_f32(residual, "residual");
  check_f32(weight, "weight");
  TORCH_CHECK(residual.dim() == 2 && out.is_contiguous() && out.is_cuda() &&
              out.sizes() == residual.sizes());
  const int T = residual.size(0), C = residual.size(1);
  TORCH_CHECK(weight.numel() == C);
  TORCH_CHECK((size_t)C * 4 <= 64 * 1024, "row too wide for the LDS row cache");
  bool wide[2] = {false, false};
  int bi = 0;
  for (const auto* br : {&a, &b}) {
    const int at = bi++;
    if (!br->has_value()) continue;
    const torch::Tensor& t = **br;
    TORCH_CHECK(t.is_contiguous() && t.is_cuda() && t.sizes() == residual.sizes());
    wide[at] = t.scalar_type() == torch::kFloat32;
    TORCH_CHECK(wide[at] || t.scalar_type() == out.scalar_type(),
                "a branch must be fp32 or the output's dtype");
  }
  auto vec_c = [&](const c10::optional<torch::Tensor>& t, const char* name) -> const float* {
    if (!t.has_value()) return nullptr;
    check_f32(*t, name);
    TORCH_CHECK(t->numel() == C, name, " must have one entry per channel");
    return (const float*)t->data_ptr();
  };
  const float* sa = vec_c(a_scale, "a_scale");
  const float* sb = vec_c(b_scale, "b_scale");
  const float* er = vec_c(extra_row, "extra_row");
  const float* ex = nullptr;
  if (extra.has_value()) {
    check_f32(*extra, "extra");
    TORCH_CHECK(extra->sizes() == residual.sizes());
    ex = (const float*)extra->data_ptr();
  }
  if (T == 0) return;
  const void* ap = a.has_value() ? a->data_ptr() : nullptr;
  const void* bp = b.has_value() ? b->data_ptr() : nullptr;
  SEQ_DISPATCH_ACT(out, {
    auto launch = [&](auto kern, auto* at, auto* bt) {
      hipLaunchKernelGGL(kern, dim3(T), dim3(kBlock), (size_t)C * 4, SEQ_STREAM(),
                         (act_t*)out.data_ptr(), (float*)residual.data_ptr(),
                         (decltype(at))ap, sa, (decltype(bt))bp, sb, (float)mult, ex, er,
                         (const float*)weight.data_ptr(), C, (float)eps);
    };
    const float* f = nullptr;
    const act_t* n = nullptr;
    if (wide[0] && wide[1]) launch(scaled_add_rmsnorm_kernel<act_t, float, float>, f, f);
    else if (wide[0]) launch(scaled_add_rmsnorm_kernel<act_t, float, act_t>, f, n);
    else if (wide[1]) launch(scaled_add_rmsnorm_kernel<act_t, act_t, float>, n, f);
    else launch(scaled_add_rmsnorm_kernel<act_t, act_t, act_t>, n, n);
  });
  SEQ_CHECK_LAUNCH();
}

void rmsnorm_rows(torch::Tensor out, torch::Tensor x, torch::Tensor weight, double eps) {
  check_rows(x, "x");
  check_f32(weight, "weight");
  const int T = x.size(0), C = x.size(1);
  TORCH_CHECK(out.is_contiguous() && out.is_cuda() && out.dim() == 2 &&
              out.size(0) == T && out.size(1) == C &&
              out.scalar_type() == x.scalar_type() && weight.numel() == C);
  if (T == 0) return;
  SEQ_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((rmsnorm_rows_kernel<act_t>), dim3(T), dim3(kBlock), 0,
                       SEQ_STREAM(), (act_t*)out.data_ptr(), (const act_t*)x.data_ptr(),
                       x.stride(0), (const float*)weight.data_ptr(), C, (float)eps);
  });
  SEQ_CHECK_LAUNCH();
}

void gelu(torch::Tensor out, torch::Tensor x) {
  TORCH_CHECK(x.is_contiguous() && out.is_contiguous() && x.is_cuda() &&
              out.scalar_type() == x.scalar_type() && out.numel() == x.numel());
  const int64_t n = x.numel();
  if (n == 0) return;
  const int64_t vn = 16 / x.element_size();
  if (n % vn == 0 && ((size_t)x.data_ptr()) % 16 == 0 &&
      ((size_t)out.data_ptr()) % 16 == 0) {
    const int64_t nvec = n / vn;
    SEQ_DISPATCH_ACT(x, {
      hipLaunchKernelGGL((gelu_vec_kernel<act_t>), dim3((nvec + 255) / 256), dim3(256),
                         0, SEQ_STREAM(), (act_t*)out.data_ptr(),
                         (const act_t*)x.data_ptr(), nvec);
    });
    SEQ_CHECK_LAUNCH();
    return;
  }
  SEQ_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((gelu_kernel<act_t>), dim3((n + 255) / 256), dim3(256), 0,
                       SEQ_STREAM(), (act_t*)out.data_ptr(), (const act_t*)x.data_ptr(), n);
  });
  SEQ_CHECK_LAUNCH();
}

void tanh_cap(torch::Tensor x, double cap) {
  check_f32(x, "x");
  TORCH_CHECK(cap > 0, "cap must be positive");
  const int64_t n = x.numel();
  if (n == 0) return;
  hipLaunchKernelGGL(tanh_cap_kernel, dim3((n + 255) / 256), dim3(256), 0, SEQ_STREAM(),
                     (float*)x.data_ptr(), (float)cap, n);
  SEQ_CHECK_LAUNCH();
}
