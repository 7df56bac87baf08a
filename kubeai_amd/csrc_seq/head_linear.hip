// Per-head linear maps y[t, h, :] = W[h] x[t, h, :] (W[h] is [B, A], applied
// like a Linear weight), with an optional sigmoid gate on the output (one per
// output channel, or one per head: gate_per_head). x and y may be slices of
// the heads of wider buffers: heads are x_hs / y_hs elements apart. The
// folded key / value up-projections of latent attention are such maps: the
// heads are independent small matrices, so one launch covers all of them
// and writes the token-major layout the attention kernels read.
#include "seq_common.h"

namespace {

typedef __attribute__((ext_vector_type(4))) short bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kHlWaves = 4;

// bf16 on the matrix cores. grid (ceil(T / 64), H), one wave per 16 tokens.
// Y^T = W X^T per 16-channel tile: the wave keeps its tokens' inputs as
// B-operand fragments in registers (kSteps * 16 >= A) and streams the rows of
// W[h] as A-operand fragments; a lane ends up with 4 consecutive output
// channels of one token.
template <int kSteps>
__global__ __launch_bounds__(kHlWaves * WAVE) void head_linear_mfma_kernel(
    bf16raw* __restrict__ y, int64_t y_stride, int64_t y_hs,
    const bf16raw* __restrict__ x, int64_t x_stride, int64_t x_hs,
    const bf16raw* __restrict__ w, const bf16raw* __restrict__ gate,
    int64_t gate_stride, int gate_per_head, int T, int H, int A, int B) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int col = lane & 15, grp = lane >> 4;
  const int t0 = (blockIdx.x * kHlWaves + wave) * 16;
  if (t0 >= T) return;
  const int h = blockIdx.y;
  const int t = min(t0 + col, T - 1);
  const bool t_ok = t0 + col < T;
  const int nks = A / 16;
  bf16x4 xf[kSteps];
  const bf16raw* xr = x + (size_t)t * x_stride + (size_t)h * x_hs + grp * 4;
  float hg = 1.f;
  if (gate != nullptr && gate_per_head)
    hg = sigmoid_f(bf16_to_f32(gate[(size_t)t * gate_stride + h]));
#pragma unroll
  for (int ks = 0; ks < kSteps; ++ks)
    if (ks < nks) xf[ks] = *(const bf16x4*)(xr + ks * 16);
  const bf16raw* wh = w + (size_t)h * B * A;
  for (int b0 = 0; b0 < B; b0 += 16) {
    const bf16raw* wr = wh + (size_t)(b0 + col) * A + grp * 4;
    f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < kSteps; ++ks)
      if (ks < nks)
        acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
            *(const bf16x4*)(wr + ks * 16), xf[ks], acc, 0, 0, 0);
    if (t_ok) {
      const int c = b0 + grp * 4;
      float o[4] = {acc[0], acc[1], acc[2], acc[3]};
      if (gate != nullptr && gate_per_head) {
        o[0] *= hg; o[1] *= hg; o[2] *= hg; o[3] *= hg;
      } else if (gate != nullptr) {
        const ushort4 g4 =
            *(const ushort4*)(gate + (size_t)t * gate_stride + (size_t)h * B + c);
        o[0] *= sigmoid_f(bf16_to_f32(g4.x));
        o[1] *= sigmoid_f(bf16_to_f32(g4.y));
        o[2] *= sigmoid_f(bf16_to_f32(g4.z));
        o[3] *= sigmoid_f(bf16_to_f32(g4.w));
      }
      ushort4 o4;
      o4.x = f32_to_bf16(o[0]);
      o4.y = f32_to_bf16(o[1]);
      o4.z = f32_to_bf16(o[2]);
      o4.w = f32_to_bf16(o[3]);
      *(ushort4*)(y + (size_t)t * y_stride + (size_t)h * y_hs + c) = o4;
    }
  }
}

// Any dtype and size: grid (T, H), the head's input row in LDS, one output
// channel per thread at a time, fp32 accumulation.
template <typename T_>
__global__ __launch_bounds__(256) void head_linear_kernel(
    T_* __restrict__ y, int64_t y_stride, int64_t y_hs, const T_* __restrict__ x,
    int64_t x_stride, int64_t x_hs, const T_* __restrict__ w,
    const T_* __restrict__ gate, int64_t gate_stride, int gate_per_head, int H,
    int A, int B) {
  extern __shared__ float xs[];
  const int t = blockIdx.x, h = blockIdx.y;
  for (int i = threadIdx.x; i < A; i += blockDim.x)
    xs[i] = ldf(x + (size_t)t * x_stride + (size_t)h * x_hs + i);
  __syncthreads();
  float hg = 1.f;
  if (gate != nullptr && gate_per_head)
    hg = sigmoid_f(ldf(gate + (size_t)t * gate_stride + h));
  for (int b = threadIdx.x; b < B; b += blockDim.x) {
    const T_* wr = w + ((size_t)h * B + b) * A;
    float acc = 0.f;
    for (int i = 0; i < A; ++i) acc += xs[i] * ldf(wr + i);
    if (gate != nullptr && gate_per_head)
      acc *= hg;
    else if (gate != nullptr)
      acc *= sigmoid_f(ldf(gate + (size_t)t * gate_stride + (size_t)h * B + b));
    stf(y + (size_t)t * y_stride + (size_t)h * y_hs + b, acc);
  }
}

}  // namespace

void head_linear(torch::Tensor y, torch::Tensor x, torch::Tensor w,
                 c10::optional<torch::Tensor> gate) {
  TORCH_CHECK(x.is_cuda() && y.is_cuda() && w.is_cuda());
  TORCH_CHECK(x.dim() == 3 && y.dim() == 3 && w.dim() == 3 && w.is_contiguous());
  const int T = x.size(0), H = x.size(1), A = x.size(2), B = w.size(1);
  TORCH_CHECK(w.size(0) == H && w.size(2) == A && y.size(0) == T && y.size(1) == H &&
              y.size(2) == B);
  auto dense = [](const torch::Tensor& t) {
    return (t.size(2) == 1 || t.stride(2) == 1) && t.stride(1) >= t.size(2) &&
           t.stride(0) >= (t.size(1) - 1) * t.stride(1) + t.size(2);
  };
  TORCH_CHECK(dense(x) && dense(y),
              "a head's channels must be dense and heads must not overlap");
  const int64_t x_hs = x.stride(1), y_hs = y.stride(1);
  TORCH_CHECK(y.scalar_type() == x.scalar_type() && w.scalar_type() == x.scalar_type());
  TORCH_CHECK(H <= 65535);
  const void* gp = nullptr;
  int64_t gs = 0;
  int gph = 0;
  if (gate.has_value()) {
    check_rows(*gate, "gate");
    TORCH_CHECK(gate->size(0) == T && gate->scalar_type() == x.scalar_type() &&
                (gate->size(1) == (int64_t)H * B || gate->size(1) == H),
                "gate must have one column per output channel or per head");
    gph = gate->size(1) == H && B != 1;
    gp = gate->data_ptr();
    gs = gate->stride(0);
  }
  if (T == 0) return;
  auto al8 = [](const void* p, int64_t stride) {
    return ((size_t)p) % 8 == 0 && stride % 4 == 0;
  };
  if (x.scalar_type() == torch::kBFloat16 && A % 16 == 0 && B % 16 == 0 && A <= 512 &&
      al8(x.data_ptr(), x.stride(0)) && al8(y.data_ptr(), y.stride(0)) &&
      x_hs % 4 == 0 && y_hs % 4 == 0 && al8(w.data_ptr(), 4) &&
      (gp == nullptr || gph || al8(gp, gs))) {
    const dim3 grid((T + 16 * kHlWaves - 1) / (16 * kHlWaves), H);
    auto launch = [&](auto kern) {
      hipLaunchKernelGGL(kern, grid, dim3(kHlWaves * WAVE), 0, SEQ_STREAM(),
                         (bf16raw*)y.data_ptr(), y.stride(0), y_hs,
                         (const bf16raw*)x.data_ptr(), x.stride(0), x_hs,
                         (const bf16raw*)w.data_ptr(), (const bf16raw*)gp, gs, gph, T,
                         H, A, B);
    };
    if (A <= 128) launch(head_linear_mfma_kernel<8>);
    else launch(head_linear_mfma_kernel<32>);
    SEQ_CHECK_LAUNCH();
    return;
  }
  TORCH_CHECK((size_t)A * 4 <= 64 * 1024, "head input too wide for LDS");
  SEQ_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((head_linear_kernel<act_t>), dim3(T, H), dim3(256),
                       (size_t)A * 4, SEQ_STREAM(), (act_t*)y.data_ptr(), y.stride(0),
                       y_hs, (const act_t*)x.data_ptr(), x.stride(0), x_hs,
                       (const act_t*)w.data_ptr(), (const act_t*)gp, gs, gph, H, A, B);
  });
  SEQ_CHECK_LAUNCH();
}
