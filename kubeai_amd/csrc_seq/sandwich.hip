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

// grid (T). Cache row of a latent with a rotated key part behind it:
// row[:R] = x[:R] / rms(x[:R]) * w, row[R + 2i], row[R + 2i + 1] = the pair
// (x[R + 2i], x[R + 2i + 1]) rotated by a = position * inv_freq[i] and scaled
// by mult. The same rotation is applied to the H query slices q_rot[t, h, :]
// (heads q_hs apart) into q_out[t, h, :] (heads o_hs apart). Angles, sin and
// cos are fp32. Rows with slot < 0 rotate their queries and write no cache.
template <typename T>
__global__ __launch_bounds__(kBlock) void latent_rope_to_cache_kernel(
    T* __restrict__ cache, const T* __restrict__ x, int64_t x_stride,
    const float* __restrict__ w, float eps, const T* __restrict__ q_rot,
    int64_t q_ts, int64_t q_hs, T* __restrict__ q_out, int64_t o_ts, int64_t o_hs,
    int H, const int* __restrict__ positions, const float* __restrict__ inv_freq,
    float mult, const int64_t* __restrict__ slot_mapping, int R, int half) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int64_t slot = slot_mapping[t];
  const float pos = (float)positions[t];
  for (int idx = threadIdx.x; idx < H * half; idx += kBlock) {
    const int h = idx / half, i = idx % half;
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    sn *= mult;
    cs *= mult;
    const T* qp = q_rot + (size_t)t * q_ts + (size_t)h * q_hs + 2 * i;
    const float u = ldf(qp), v = ldf(qp + 1);
    T* op = q_out + (size_t)t * o_ts + (size_t)h * o_hs + 2 * i;
    stf(op, u * cs - v * sn);
    stf(op + 1, v * cs + u * sn);
  }
  if (slot < 0) return;  // uniform over the block
  const T* xr = x + (size_t)t * x_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < R; c += kBlock) {
    const float v = ldf(xr + c);
    ss += v * v;
  }
  const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)R + eps);
  T* row = cache + (size_t)slot * (R + 2 * half);
  for (int c = threadIdx.x; c < R; c += kBlock) stf(row + c, ldf(xr + c) * r * w[c]);
  for (int i = threadIdx.x; i < half; i += kBlock) {
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    sn *= mult;
    cs *= mult;
    const float u = ldf(xr + R + 2 * i), v = ldf(xr + R + 2 * i + 1);
    stf(row + R + 2 * i, u * cs - v * sn);
    stf(row + R + 2 * i + 1, v * cs + u * sn);
  }
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

void latent_rope_to_cache(torch::Tensor cache, torch::Tensor x, torch::Tensor weight,
                          double eps, c10::optional<torch::Tensor> q_rot,
                          c10::optional<torch::Tensor> q_out, torch::Tensor positions,
                          torch::Tensor inv_freq, double rot_mult,
                          torch::Tensor slot_mapping) {
  check_rows(x, "x");
  check_f32(weight, "weight");
  check_f32(inv_freq, "inv_freq");
  check_i32(positions, "positions");
  TORCH_CHECK(slot_mapping.scalar_type() == torch::kInt64 &&
              slot_mapping.is_contiguous() && slot_mapping.is_cuda());
  const int T = x.size(0), R = weight.numel(), half = inv_freq.numel();
  const int C = R + 2 * half;
  TORCH_CHECK(x.size(1) == C, "x must hold the latent and the rotated key part");
  TORCH_CHECK(cache.is_contiguous() && cache.is_cuda() && cache.dim() == 4 &&
              cache.size(1) == 1 && cache.size(3) == C &&
              cache.scalar_type() == x.scalar_type(),
              "cache must be [blocks, 1, block, latent + rotated] of the activations' dtype");
  TORCH_CHECK(slot_mapping.numel() == T && positions.numel() == T);
  TORCH_CHECK(q_rot.has_value() == q_out.has_value());
  int H = 0;
  const void* qp = nullptr;
  void* op = nullptr;
  int64_t q_ts = 0, q_hs = 0, o_ts = 0, o_hs = 0;
  if (q_rot.has_value() && half > 0) {
    const torch::Tensor &q = *q_rot, &o = *q_out;
    TORCH_CHECK(q.is_cuda() && o.is_cuda() && q.dim() == 3 && o.dim() == 3 &&
                q.size(0) == T && o.size(0) == T && q.size(1) == o.size(1) &&
                q.size(2) == 2 * half && o.size(2) == 2 * half &&
                q.stride(2) == 1 && o.stride(2) == 1 &&
                q.scalar_type() == x.scalar_type() && o.scalar_type() == x.scalar_type());
    H = q.size(1);
    qp = q.data_ptr();
    op = o.data_ptr();
    q_ts = q.stride(0); q_hs = q.stride(1);
    o_ts = o.stride(0); o_hs = o.stride(1);
  }
  if (T == 0) return;
  SEQ_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((latent_rope_to_cache_kernel<act_t>), dim3(T), dim3(kBlock), 0,
                       SEQ_STREAM(), (act_t*)cache.data_ptr(),
                       (const act_t*)x.data_ptr(), x.stride(0),
                       (const float*)weight.data_ptr(), (float)eps, (const act_t*)qp,
                       q_ts, q_hs, (act_t*)op, o_ts, o_hs, H,
                       (const int*)positions.data_ptr(),
                       (const float*)inv_freq.data_ptr(), (float)rot_mult,
                       (const int64_t*)slot_mapping.data_ptr(), R, half);
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
