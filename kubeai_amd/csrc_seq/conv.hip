// Depthwise causal convolutions over the runs of a packed step, with each
// sequence's last taps-1 inputs carried in a state slot, and the token shift
// (previous token's activations) that uses the same carried tail.
#include "seq_common.h"

namespace {

constexpr int kMaxTail = 15;  // taps - 1

// grid (T, ceil(C / 256)). Input d steps back comes from this run's tokens
// when it lies inside the run, else from the carried tail; positions < 0
// contribute zero. tails row i holds the input at position p0 - K1 + i.
// act 1 applies silu to the sum.
template <typename T>
__global__ void causal_conv_kernel(
    T* __restrict__ y, const T* __restrict__ x, int64_t x_stride,
    const float* __restrict__ w, const float* __restrict__ tails,
    const int* __restrict__ start_loc, const int* __restrict__ slots,
    const int* __restrict__ token_seq, const int* __restrict__ positions,
    int C, int taps, int residual, int act) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int s = token_seq[t], s0 = start_loc[s], slot = slots[s];
  const int p = positions[t], p0 = positions[s0];
  const int K1 = taps - 1;
  float acc = residual ? ldf(x + (size_t)t * x_stride + c) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int d = K1 - j;
    const int sp = p - d;
    if (sp < 0) continue;
    float v = 0.f;
    if (t - d >= s0) {
      v = ldf(x + (size_t)(t - d) * x_stride + c);
    } else if (slot >= 0) {
      const int idx = sp - (p0 - K1);
      v = tails[((size_t)slot * K1 + idx) * C + c];
    }
    acc += w[(size_t)c * taps + j] * v;
  }
  if (act == 1) acc = silu_f(acc);
  stf(y + (size_t)t * C + c, acc);
}

// grid (n_seq, ceil(C / 256)): advance a run's tail past its tokens. One
// thread owns a channel's whole tail, so old rows are read before any write.
template <typename T>
__global__ void tail_update_kernel(
    float* __restrict__ tails, const T* __restrict__ x, int64_t x_stride,
    const int* __restrict__ start_loc, const int* __restrict__ slots,
    const int* __restrict__ positions, int C, int K1) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int slot = slots[s], s0 = start_loc[s], n = start_loc[s + 1] - s0;
  if (slot < 0 || n <= 0) return;
  const int p0 = positions[s0];
  float buf[kMaxTail];
  for (int i = 0; i < K1; ++i) {
    const int pp = p0 + n - K1 + i;
    float v = 0.f;
    if (pp >= p0) v = ldf(x + (size_t)(s0 + pp - p0) * x_stride + c);
    else if (pp >= 0) v = tails[((size_t)slot * K1 + (i + n)) * C + c];
    buf[i] = v;
  }
  for (int i = 0; i < K1; ++i) tails[((size_t)slot * K1 + i) * C + c] = buf[i];
}

// grid (T, ceil(C / 256)): out[s][t] = h + (h' - h) * mu[s].
template <typename T>
__global__ void token_shift_mix_kernel(
    T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ mu,
    const float* __restrict__ prev, const int* __restrict__ start_loc,
    const int* __restrict__ slots, const int* __restrict__ token_seq,
    const int* __restrict__ positions, int Ttot, int C, int S) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int s = token_seq[t], s0 = start_loc[s], slot = slots[s];
  const float cur = ldf(h + (size_t)t * C + c);
  float hp = 0.f;
  if (t - 1 >= s0) hp = ldf(h + (size_t)(t - 1) * C + c);
  else if (slot >= 0 && positions[t] > 0) hp = prev[(size_t)slot * C + c];
  const float d = hp - cur;
  for (int k = 0; k < S; ++k)
    stf(out + ((size_t)k * Ttot + t) * C + c, cur + d * mu[(size_t)k * C + c]);
}

}  // namespace

static void launch_tail_update(torch::Tensor tails, torch::Tensor x,
                               torch::Tensor start_loc, torch::Tensor slots,
                               torch::Tensor positions, int C, int K1) {
  const int n_seq = slots.numel();
  if (n_seq == 0 || K1 == 0) return;
  SEQ_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((tail_update_kernel<act_t>), dim3(n_seq, (C + 255) / 256),
                       dim3(256), 0, SEQ_STREAM(), (float*)tails.data_ptr(),
                       (const act_t*)x.data_ptr(), x.stride(0),
                       (const int*)start_loc.data_ptr(), (const int*)slots.data_ptr(),
                       (const int*)positions.data_ptr(), C, K1);
  });
  SEQ_CHECK_LAUNCH();
}

void causal_conv(torch::Tensor y, torch::Tensor x, torch::Tensor w,
                 torch::Tensor tails, torch::Tensor start_loc,
                 torch::Tensor slots, torch::Tensor token_seq,
                 torch::Tensor positions, bool residual, int64_t act) {
  check_rows(x, "x");
  TORCH_CHECK(act == 0 || act == 1, "act: 0 none, 1 silu");
  check_f32(w, "w");
  check_f32(tails, "tails");
  check_i32(start_loc, "start_loc");
  check_i32(slots, "slots");
  check_i32(token_seq, "token_seq");
  check_i32(positions, "positions");
  const int T = x.size(0), C = x.size(1), taps = w.size(1);
  TORCH_CHECK(y.is_contiguous() && y.size(0) == T && y.size(1) == C &&
              y.scalar_type() == x.scalar_type());
  TORCH_CHECK(w.size(0) == C && taps >= 1 && taps - 1 <= kMaxTail);
  TORCH_CHECK(tails.dim() == 3 && tails.size(1) == taps - 1 && tails.size(2) == C);
  TORCH_CHECK(token_seq.numel() == T && positions.numel() == T &&
              start_loc.numel() == slots.numel() + 1);
  TORCH_CHECK((C + 255) / 256 <= 65535);
  if (T == 0) return;
  SEQ_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((causal_conv_kernel<act_t>), dim3(T, (C + 255) / 256),
                       dim3(256), 0, SEQ_STREAM(), (act_t*)y.data_ptr(),
                       (const act_t*)x.data_ptr(), x.stride(0),
                       (const float*)w.data_ptr(), (const float*)tails.data_ptr(),
                       (const int*)start_loc.data_ptr(), (const int*)slots.data_ptr(),
                       (const int*)token_seq.data_ptr(),
                       (const int*)positions.data_ptr(), C, taps, residual ? 1 : 0,
                       (int)act);
  });
  SEQ_CHECK_LAUNCH();
  launch_tail_update(tails, x, start_loc, slots, positions, C, taps - 1);
}

void token_shift_mix(torch::Tensor out, torch::Tensor h, torch::Tensor mu,
                     torch::Tensor prev, torch::Tensor start_loc,
                     torch::Tensor slots, torch::Tensor token_seq,
                     torch::Tensor positions) {
  check_f32(mu, "mu");
  check_f32(prev, "prev");
  check_i32(start_loc, "start_loc");
  check_i32(slots, "slots");
  check_i32(token_seq, "token_seq");
  check_i32(positions, "positions");
  TORCH_CHECK(h.is_contiguous() && h.dim() == 2 && out.is_contiguous());
  const int T = h.size(0), C = h.size(1), S = mu.size(0);
  TORCH_CHECK(mu.size(1) == C && out.dim() == 3 && out.size(0) == S &&
              out.size(1) == T && out.size(2) == C &&
              out.scalar_type() == h.scalar_type());
  TORCH_CHECK(prev.dim() == 3 && prev.size(1) == 1 && prev.size(2) == C);
  TORCH_CHECK(token_seq.numel() == T && positions.numel() == T &&
              start_loc.numel() == slots.numel() + 1);
  if (T == 0) return;
  SEQ_DISPATCH_ACT(h, {
    hipLaunchKernelGGL((token_shift_mix_kernel<act_t>), dim3(T, (C + 255) / 256),
                       dim3(256), 0, SEQ_STREAM(), (act_t*)out.data_ptr(),
                       (const act_t*)h.data_ptr(), (const float*)mu.data_ptr(),
                       (const float*)prev.data_ptr(), (const int*)start_loc.data_ptr(),
                       (const int*)slots.data_ptr(), (const int*)token_seq.data_ptr(),
                       (const int*)positions.data_ptr(), T, C, S);
  });
  SEQ_CHECK_LAUNCH();
  launch_tail_update(prev, h, start_loc, slots, positions, C, 1);
}
