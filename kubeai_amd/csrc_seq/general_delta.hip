// Generalized delta rule over the runs of a packed step. Per head a matrix
// state S [D, Dv] (fp32, one slot per sequence) whose transition is a
// diagonal decay plus a rank-one removal along the unit key, both reading
// the old state, followed by the write:
//
//   w = exp(-decay_scale * sigmoid(w_pre + w_bias)),  a = sigmoid(a_pre + a_bias)
//   n = k / sqrt(|k|^2 + key_eps)
//   S <- diag(w) S - (a * n) (n^T S) + k v^T;   o = S^T r
//
// Everything but the loads of r, k, v, w_pre, a_pre (serving dtype) is fp32.
// The value columns of a head are independent of each other, so a head is
// split over threads (and waves) by column: per token a column costs one dot
// product with n over the old column, then one pass that rewrites the column
// and accumulates the read-out.
#include "seq_common.h"

namespace {

constexpr int kTile = 8;  // tokens staged per barrier (LDS-state kernel)

// Any size: grid (n_seq * H, column blocks), block = the block's columns
// rounded up to a wave, that part of the head's state in LDS, thread j owns
// value column c0 + j.
template <typename T>
__global__ void diag_rank1_scan_kernel(
    float* __restrict__ o, const T* __restrict__ r, int64_t r_stride,
    const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, const T* __restrict__ w_pre, int64_t w_stride,
    const T* __restrict__ a_pre, int64_t a_stride, const float* __restrict__ w_bias,
    const float* __restrict__ a_bias, float* __restrict__ state,
    const int* __restrict__ start_loc, const int* __restrict__ slots,
    const int* __restrict__ positions, int H, int D, int Dv, int CB,
    float decay_scale, float key_eps) {
  const int s = blockIdx.x / H, h = blockIdx.x % H;
  const int s0 = start_loc[s], s1 = start_loc[s + 1], slot = slots[s];
  if (s1 <= s0) return;
  const int c0 = blockIdx.y * CB, nc = min(CB, Dv - c0);  // this block's columns
  extern __shared__ float sm[];
  float* S = sm;                      // [D][CB]
  float* rs = S + (size_t)D * CB;     // [tile][D] read-out vector
  float* ks = rs + kTile * D;         // [tile][D] key as written
  float* ws = ks + kTile * D;         // [tile][D] decay
  float* ns = ws + kTile * D;         // [tile][D] unit key
  float* bs = ns + kTile * D;         // [tile][D] removal rate * unit key
  float* vs = bs + kTile * D;         // [tile][CB]
  float* rk = vs + kTile * CB;        // [tile] 1 / |k|
  const int tid = threadIdx.x, nthr = blockDim.x;
  const bool carry = slot >= 0 && positions[s0] > 0;
  float* sp = state + ((size_t)(slot < 0 ? 0 : slot) * H + h) * D * Dv;
  for (int i = tid; i < D * CB; i += nthr) {
    const int row = i / CB, c = i % CB;
    S[i] = (carry && c < nc) ? sp[(size_t)row * Dv + c0 + c] : 0.f;
  }
  for (int t0 = s0; t0 < s1; t0 += kTile) {
    const int nt = min(kTile, s1 - t0);
    __syncthreads();  // the previous tile's readers are done
    for (int i = tid; i < nt * D; i += nthr) {
      const int tt = i / D, d = i % D;
      const size_t t = (size_t)(t0 + tt);
      rs[i] = ldf(r + t * r_stride + h * D + d);
      ks[i] = ldf(k + t * k_stride + h * D + d);
      ws[i] = expf(-decay_scale * sigmoid_f(ldf(w_pre + t * w_stride + h * D + d) +
                                            w_bias[h * D + d]));
      bs[i] = sigmoid_f(ldf(a_pre + t * a_stride + h * D + d) + a_bias[h * D + d]);
    }
    for (int i = tid; i < nt * CB; i += nthr) {
      const int tt = i / CB, d = i % CB;
      vs[i] = d < nc ? ldf(v + (size_t)(t0 + tt) * v_stride + h * Dv + c0 + d) : 0.f;
    }
    __syncthreads();
    if (tid < nt) {
      float sk = 0.f;
      for (int d = 0; d < D; ++d) sk += ks[tid * D + d] * ks[tid * D + d];
      rk[tid] = 1.0f / sqrtf(sk + key_eps);
    }
    __syncthreads();
    for (int i = tid; i < nt * D; i += nthr) {
      const float n = ks[i] * rk[i / D];
      ns[i] = n;
      bs[i] *= n;
    }
    __syncthreads();
    if (tid < nc) {
      for (int tt = 0; tt < nt; ++tt) {
        const float* rt = rs + tt * D;
        const float* kt = ks + tt * D;
        const float* wt = ws + tt * D;
        const float* nt_ = ns + tt * D;
        const float* bt = bs + tt * D;
        const float vj = vs[tt * CB + tid];
        float dot = 0.f;
        for (int i = 0; i < D; ++i) dot += S[i * CB + tid] * nt_[i];
        float acc = 0.f;
        for (int i = 0; i < D; ++i) {
          const float st = wt[i] * S[i * CB + tid] - bt[i] * dot + kt[i] * vj;
          S[i * CB + tid] = st;
          acc += rt[i] * st;
        }
        o[((size_t)(t0 + tt) * H + h) * Dv + c0 + tid] = acc;
      }
    }
  }
  __syncthreads();
  if (slot >= 0)
    for (int i = tid; i < D * CB; i += nthr) {
      const int row = i / CB, c = i % CB;
      if (c < nc) sp[(size_t)row * Dv + c0 + c] = S[i];
    }
}

}  // namespace

static bool head_cols(const torch::Tensor& t) {
  // [T, H, D] view of columns of a row-major matrix: heads dense, rows strided
  return t.is_cuda() && t.dim() == 3 && t.stride(2) == 1 && t.stride(1) == t.size(2);
}

void diag_rank1_scan(torch::Tensor o, torch::Tensor r, torch::Tensor k, torch::Tensor v,
                     torch::Tensor w_pre, torch::Tensor a_pre, torch::Tensor w_bias,
                     torch::Tensor a_bias, torch::Tensor state, torch::Tensor start_loc,
                     torch::Tensor slots, torch::Tensor positions, double decay_scale,
                     double key_eps, int64_t max_len) {
  check_f32(o, "o");
  check_f32(state, "state");
  check_f32(w_bias, "w_bias");
  check_f32(a_bias, "a_bias");
  check_i32(start_loc, "start_loc");
  check_i32(slots, "slots");
  check_i32(positions, "positions");
  TORCH_CHECK(head_cols(r) && head_cols(k) && head_cols(v) && head_cols(w_pre) &&
              head_cols(a_pre));
  const int T = k.size(0), H = k.size(1), D = k.size(2), Dv = v.size(2);
  for (const auto* t : {&r, &w_pre, &a_pre})
    TORCH_CHECK(t->size(0) == T && t->size(1) == H && t->size(2) == D &&
                t->scalar_type() == k.scalar_type());
  TORCH_CHECK(v.size(0) == T && v.size(1) == H && v.scalar_type() == k.scalar_type());
  TORCH_CHECK(o.dim() == 3 && o.size(0) == T && o.size(1) == H && o.size(2) == Dv);
  TORCH_CHECK(w_bias.numel() == H * D && a_bias.numel() == H * D);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D &&
              state.size(3) == Dv);
  const int n_seq = start_loc.numel() - 1;
  TORCH_CHECK(slots.numel() == n_seq && positions.numel() == T);
  if (T == 0 || n_seq == 0) return;
  (void)max_len;
  // columns per block: as many as fit LDS beside the staged tile
  int CB = std::min(256, (Dv + WAVE - 1) / WAVE * WAVE);
  auto lds_of = [&](int cb) {
    return (size_t)((size_t)D * cb + 5 * kTile * D + kTile * cb + kTile) * 4;
  };
  while (CB > WAVE && lds_of(CB) > 64 * 1024) CB -= WAVE;
  if (lds_of(CB) > 64 * 1024) {
    CB = 32;
    while (CB > 1 && lds_of(CB) > 64 * 1024) CB /= 2;
  }
  TORCH_CHECK(lds_of(CB) <= 64 * 1024, "key size too large for the LDS state");
  const int ncb = (Dv + CB - 1) / CB;
  const int threads = (CB + WAVE - 1) / WAVE * WAVE;
  SEQ_DISPATCH_ACT(k, {
    hipLaunchKernelGGL((diag_rank1_scan_kernel<act_t>), dim3(n_seq * H, ncb),
                       dim3(threads), lds_of(CB), SEQ_STREAM(), (float*)o.data_ptr(),
                       (const act_t*)r.data_ptr(), r.stride(0), (const act_t*)k.data_ptr(),
                       k.stride(0), (const act_t*)v.data_ptr(), v.stride(0),
                       (const act_t*)w_pre.data_ptr(), w_pre.stride(0),
                       (const act_t*)a_pre.data_ptr(), a_pre.stride(0),
                       (const float*)w_bias.data_ptr(), (const float*)a_bias.data_ptr(),
                       (float*)state.data_ptr(), (const int*)start_loc.data_ptr(),
                       (const int*)slots.data_ptr(), (const int*)positions.data_ptr(), H, D,
                       Dv, CB, (float)decay_scale, (float)key_eps);
  });
  SEQ_CHECK_LAUNCH();
}
