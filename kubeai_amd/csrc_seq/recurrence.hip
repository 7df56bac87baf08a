// Recurrences over the runs of a packed step: the elementwise gated
// recurrence (minGRU) and matrix-state linear attention (per-token channel
// decay with a current-token bonus, or a constant per-head decay). State is
// fp32, one slot per sequence; a run that starts at position 0 starts from
// zero whatever its slot holds.
#include "seq_common.h"

namespace {

constexpr int kGruSeg = 64;  // tokens per segment of a run

// The recurrence S_t = a_t S_(t-1) + b_t composes: a segment of a run maps
// its incoming state S to A S + B. Long runs are cut into segments of
// kGruSeg tokens that are walked in parallel.
//
// Pass 1, grid (n_seq, n_segments, ceil(n / 256)), only when a run spans
// more than one segment: (A, B) of every segment.
template <typename T>
__global__ void mingru_segments_kernel(
    float* __restrict__ segA, float* __restrict__ segB,
    const T* __restrict__ zxg, const float* __restrict__ bz,
    const float* __restrict__ bx, const int* __restrict__ start_loc, int n,
    int nseg) {
  const int s = blockIdx.x, g = blockIdx.y;
  const int c = blockIdx.z * blockDim.x + threadIdx.x;
  if (c >= n) return;
  const int s0 = start_loc[s], s1 = start_loc[s + 1];
  const int t0 = s0 + g * kGruSeg, t1 = min(t0 + kGruSeg, s1);
  if (t0 >= s1) return;
  const float bzc = bz[c], bxc = bx[c];
  float A = 1.f, B = 0.f;
  for (int t = t0; t < t1; ++t) {
    const T* row = zxg + (size_t)t * 3 * n;
    const float z = sigmoid_f(ldf(row + c) + bzc);
    const float u = ldf(row + n + c) + bxc;
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
    A *= 1.0f - z;
    B = (1.0f - z) * B + z * cand;
  }
  segA[((size_t)s * nseg + g) * n + c] = A;
  segB[((size_t)s * nseg + g) * n + c] = B;
}

// Pass 2, same grid: fold the earlier segments into the incoming state,
// then walk the own segment and write y; the last segment stores the state.
template <typename T>
__global__ void mingru_scan_kernel(
    T* __restrict__ y, const T* __restrict__ zxg, const float* __restrict__ bz,
    const float* __restrict__ bx, float* __restrict__ state,
    const float* __restrict__ segA, const float* __restrict__ segB,
    const int* __restrict__ start_loc, const int* __restrict__ slots,
    const int* __restrict__ positions, int n, int nseg) {
  const int s = blockIdx.x, g = blockIdx.y;
  const int c = blockIdx.z * blockDim.x + threadIdx.x;
  if (c >= n) return;
  const int s0 = start_loc[s], s1 = start_loc[s + 1], slot = slots[s];
  const int t0 = s0 + g * kGruSeg, t1 = min(t0 + kGruSeg, s1);
  if (t0 >= s1) return;
  float S = (slot >= 0 && positions[s0] > 0) ? state[(size_t)slot * n + c] : 0.f;
  for (int gg = 0; gg < g; ++gg) {
    const size_t i = ((size_t)s * nseg + gg) * n + c;
    S = segA[i] * S + segB[i];
  }
  const float bzc = bz[c], bxc = bx[c];
  for (int t = t0; t < t1; ++t) {
    const T* row = zxg + (size_t)t * 3 * n;
    const float z = sigmoid_f(ldf(row + c) + bzc);
    const float u = ldf(row + n + c) + bxc;
    const float gt = ldf(row + 2 * n + c);
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
    S = (1.0f - z) * S + z * cand;
    stf(y + (size_t)t * n + c, S * silu_f(gt));
  }
  if (slot >= 0 && t1 == s1) state[(size_t)slot * n + c] = S;
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

// Register-state form for key sizes D = 16 * kQ (<= 128). grid
// (n_seq * H * ceil(Dv / 16)), one wave per block: the wave owns 16 value
// columns of one head; lane (r, c) keeps rows [r D/4, (r+1) D/4) of column c
// in registers, so a token costs D/4 fused steps per lane and two shuffles
// to join the four partial outputs. q/k/decay of kScanTile tokens are staged
// through LDS with activations and decays applied once per element.
template <typename T, bool kPerToken, int kQ>
__global__ __launch_bounds__(WAVE) void linear_attn_scan_reg_kernel(
    float* __restrict__ o, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, const T* __restrict__ decay_pre, int64_t d_stride,
    const float* __restrict__ decay_const, const float* __restrict__ bonus,
    const float* __restrict__ w_bias, float* __restrict__ state,
    const int* __restrict__ start_loc, const int* __restrict__ slots,
    const int* __restrict__ positions, int H, int Dv, int ncb,
    int silu_inputs, int nseg, int seg_len, int compose,
    float* __restrict__ segB, float* __restrict__ segW) {
  constexpr int R = 4 * kQ, D = 4 * R;
  const int cb = blockIdx.x % ncb;
  const int h = (blockIdx.x / ncb) % H;
  const int seg = (blockIdx.x / (ncb * H)) % nseg;
  const int s = blockIdx.x / (ncb * H * nseg);
  const int r0 = start_loc[s], s1_run = start_loc[s + 1], slot = slots[s];
  // Long runs are cut into segments of seg_len tokens that run in parallel.
  // The state update is affine in the state, S -> diag(W) S + B, so pass 1
  // (compose) walks every segment but the last from zero and stores its
  // (W, B); pass 2 folds the earlier segments into the incoming state and
  // walks its own segment again, now writing the outputs.
  const int s0 = r0 + seg * seg_len;
  const int s1 = min(s0 + seg_len, s1_run);
  if (s0 >= s1_run) return;
  if (compose && s1 == s1_run) return;
  __shared__ __attribute__((aligned(16))) float qs[kScanTile * D];
  __shared__ __attribute__((aligned(16))) float ks[kScanTile * D];
  __shared__ __attribute__((aligned(16))) float ws[kPerToken ? kScanTile * D : 4];
  __shared__ float vs[kScanTile * 16];
  const int lane = threadIdx.x, r = lane >> 4, c = lane & 15;
  const int j = cb * 16 + c;
  const bool valid = j < Dv;
  const bool carry = !compose && slot >= 0 && positions[r0] > 0;
  float* sp = state + ((size_t)(slot < 0 ? 0 : slot) * H + h) * D * Dv;
  float S[R], U[R], Wp[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    S[i] = (carry && valid) ? sp[(size_t)(r * R + i) * Dv + j] : 0.f;
    U[i] = kPerToken ? bonus[h * D + r * R + i] : 0.f;
    Wp[i] = 1.f;
  }
  const float dc = kPerToken ? 0.f : decay_const[h];
  if (!compose && seg > 0) {
    float wfull = 1.f;  // constant decay over one full segment
    if (!kPerToken)
      for (int n = 0; n < seg_len; ++n) wfull *= dc;
    for (int gg = 0; gg < seg; ++gg) {
      const size_t base = ((size_t)(s * nseg + gg) * H + h) * D;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        const float w = kPerToken ? segW[base + r * R + i] : wfull;
        const float b = valid ? segB[(base + r * R + i) * Dv + j] : 0.f;
        S[i] = w * S[i] + b;
      }
    }
  }
  // staging: lane (st_tt, st_part) owns a quarter row of one token of the
  // tile; the next tile's vectors are fetched into registers while the
  // current tile is walked, so the lone wave never waits on memory
  typedef typename Raw4<T>::type raw4;
  const int st_tt = lane >> 2, st_part = lane & 3;
  raw4 pq[kQ], pk[kQ], pw[kQ];
  T pv[4];
  float wb[kPerToken ? R : 1];
  if (kPerToken) {
#pragma unroll
    for (int i = 0; i < R; ++i) wb[i] = w_bias[h * D + st_part * R + i];
  }
  auto prefetch = [&](int tile0) {
    const int t = tile0 + st_tt;
    if (t < s1) {
      const T* qp = q + (size_t)t * q_stride + h * D + st_part * R;
      const T* kp = k + (size_t)t * k_stride + h * D + st_part * R;
#pragma unroll
      for (int b = 0; b < kQ; ++b) {
        pq[b] = *(const raw4*)(qp + 4 * b);
        pk[b] = *(const raw4*)(kp + 4 * b);
      }
      if (kPerToken) {
        const T* wp = decay_pre + (size_t)t * d_stride + h * D + st_part * R;
#pragma unroll
        for (int b = 0; b < kQ; ++b) pw[b] = *(const raw4*)(wp + 4 * b);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int col = cb * 16 + st_part * 4 + e;
        pv[e] = col < Dv ? v[(size_t)t * v_stride + h * Dv + col] : (T)0;
      }
    }
  };
  prefetch(s0);
  for (int t0 = s0; t0 < s1; t0 += kScanTile) {
    const int nt = min(kScanTile, s1 - t0);
    __syncthreads();
    if (st_tt < nt) {
#pragma unroll
      for (int b = 0; b < kQ; ++b) {
        float a[4], bb[4];
        cvt4(pq[b], a);
        cvt4(pk[b], bb);
        if (silu_inputs) {
#pragma unroll
          for (int e = 0; e < 4; ++e) { a[e] = silu_f(a[e]); bb[e] = silu_f(bb[e]); }
        }
        const int at = st_tt * D + st_part * R + 4 * b;
        *(float4*)(qs + at) = make_float4(a[0], a[1], a[2], a[3]);
        *(float4*)(ks + at) = make_float4(bb[0], bb[1], bb[2], bb[3]);
        if (kPerToken) {
          float w[4];
          cvt4(pw[b], w);
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = expf(-expf(w[e] + wb[4 * b + e]));
          *(float4*)(ws + at) = make_float4(w[0], w[1], w[2], w[3]);
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float vv = ldf(&pv[e]);
        if (silu_inputs) vv = silu_f(vv);
        vs[st_tt * 16 + st_part * 4 + e] = vv;
      }
    }
    __syncthreads();
    if (t0 + kScanTile < s1) prefetch(t0 + kScanTile);
    for (int tt = 0; tt < nt; ++tt) {
      const float vj = vs[tt * 16 + c];
      const float4* q4 = (const float4*)(qs + tt * D + r * R);
      const float4* k4 = (const float4*)(ks + tt * D + r * R);
      const float4* w4 = (const float4*)(ws + (kPerToken ? tt * D + r * R : 0));
      float acc = 0.f;
#pragma unroll
      for (int b = 0; b < kQ; ++b) {
        const float4 qq = q4[b], kk = k4[b];
        const float qa[4] = {qq.x, qq.y, qq.z, qq.w};
        const float ka[4] = {kk.x, kk.y, kk.z, kk.w};
        float wa[4] = {0.f, 0.f, 0.f, 0.f};
        if (kPerToken) {
          const float4 ww = w4[b];
          wa[0] = ww.x; wa[1] = ww.y; wa[2] = ww.z; wa[3] = ww.w;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = b * 4 + e;
          const float kv = ka[e] * vj;
          if (kPerToken) {
            acc += qa[e] * (S[i] + U[i] * kv);
            S[i] = wa[e] * S[i] + kv;
            if (compose) Wp[i] *= wa[e];
          } else {
            S[i] = dc * S[i] + kv;
            acc += qa[e] * S[i];
          }
        }
      }
      acc += __shfl_xor(acc, 16, WAVE);
      acc += __shfl_xor(acc, 32, WAVE);
      if (!compose && r == 0 && valid) o[((size_t)(t0 + tt) * H + h) * Dv + j] = acc;
    }
  }
  if (compose) {
    const size_t base = ((size_t)(s * nseg + seg) * H + h) * D;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      if (valid) segB[(base + r * R + i) * Dv + j] = S[i];
      if (kPerToken && cb == 0 && c == 0) segW[base + r * R + i] = Wp[i];
    }
  } else if (slot >= 0 && valid && s1 == s1_run) {
#pragma unroll
    for (int i = 0; i < R; ++i) sp[(size_t)(r * R + i) * Dv + j] = S[i];
  }
}

}  // namespace

void mingru_scan(torch::Tensor y, torch::Tensor zxg, torch::Tensor bz,
                 torch::Tensor bx, torch::Tensor state, torch::Tensor start_loc,
                 torch::Tensor slots, torch::Tensor positions, int64_t max_len) {
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
  const int nseg = std::max<int>(1, (max_len + kGruSeg - 1) / kGruSeg);
  TORCH_CHECK(nseg <= 65535 && (n + 255) / 256 <= 65535);
  torch::Tensor seg;
  float* segA = nullptr;
  float* segB = nullptr;
  if (nseg > 1) {
    seg = torch::empty({2, n_seq, nseg, n}, state.options());
    segA = (float*)seg.data_ptr();
    segB = segA + (size_t)n_seq * nseg * n;
  }
  const dim3 grid(n_seq, nseg, (n + 255) / 256);
  SEQ_DISPATCH_ACT(zxg, {
    if (nseg > 1)
      hipLaunchKernelGGL((mingru_segments_kernel<act_t>), grid, dim3(256), 0,
                         SEQ_STREAM(), segA, segB, (const act_t*)zxg.data_ptr(),
                         (const float*)bz.data_ptr(), (const float*)bx.data_ptr(),
                         (const int*)start_loc.data_ptr(), n, nseg);
    hipLaunchKernelGGL((mingru_scan_kernel<act_t>), grid, dim3(256), 0,
                       SEQ_STREAM(), (act_t*)y.data_ptr(),
                       (const act_t*)zxg.data_ptr(), (const float*)bz.data_ptr(),
                       (const float*)bx.data_ptr(), (float*)state.data_ptr(), segA,
                       segB, (const int*)start_loc.data_ptr(),
                       (const int*)slots.data_ptr(),
                       (const int*)positions.data_ptr(), n, nseg);
  });
  SEQ_CHECK_LAUNCH();
}

#define SEQ_SCAN_CASE(KQ)                                                     \
  case KQ:                                                                    \
    if (per_token) launch(linear_attn_scan_reg_kernel<act_t, true, KQ>);      \
    else launch(linear_attn_scan_reg_kernel<act_t, false, KQ>);               \
    break;

void linear_attn_scan(torch::Tensor o, torch::Tensor q, torch::Tensor k,
                      torch::Tensor v, torch::Tensor decay,
                      c10::optional<torch::Tensor> bonus,
                      c10::optional<torch::Tensor> w_bias, torch::Tensor state,
                      torch::Tensor start_loc, torch::Tensor slots,
                      torch::Tensor positions, bool silu_inputs, int64_t max_len) {
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
  auto vec_ok = [&](const torch::Tensor& t) {
    const size_t bytes = 4 * t.element_size();
    return ((size_t)t.data_ptr()) % bytes == 0 && t.stride(0) % 4 == 0;
  };
  const bool aligned = vec_ok(q) && vec_ok(k) && (!per_token || vec_ok(decay));
  if (D % 16 == 0 && D <= 128 && aligned) {
    const int ncb = (Dv + 15) / 16;
    // segment-parallel walk of long runs (see the kernel); the workspace
    // holds every segment's composed (W, B)
    int seg_len = 128, nseg = 1;
    if (max_len > 2 * seg_len) {
      nseg = (int)((max_len + seg_len - 1) / seg_len);
      while ((size_t)n_seq * nseg * H * D * Dv * 4 > ((size_t)2 << 30)) {
        seg_len *= 2;
        nseg = (int)((max_len + seg_len - 1) / seg_len);
      }
    }
    if (nseg == 1) seg_len = (int)std::max<int64_t>(max_len, 1);  // one segment: the whole run
    torch::Tensor wsB, wsW;
    if (nseg > 1) {
      wsB = torch::empty({(int64_t)n_seq * nseg * H * D * Dv}, state.options());
      wsW = torch::empty({(int64_t)n_seq * nseg * H * D}, state.options());
    }
    SEQ_DISPATCH_ACT(q, {
      auto launch1 = [&](auto kern, int compose) {
        hipLaunchKernelGGL(kern, dim3(n_seq * nseg * H * ncb), dim3(WAVE), 0, SEQ_STREAM(),
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
                           (const int*)positions.data_ptr(), H, Dv, ncb,
                           silu_inputs ? 1 : 0, nseg, seg_len, compose,
                           nseg > 1 ? (float*)wsB.data_ptr() : nullptr,
                           nseg > 1 ? (float*)wsW.data_ptr() : nullptr);
      };
      auto launch = [&](auto kern) {
        if (nseg > 1) launch1(kern, 1);
        launch1(kern, 0);
      };
      switch (D / 16) {
        SEQ_SCAN_CASE(1) SEQ_SCAN_CASE(2) SEQ_SCAN_CASE(3) SEQ_SCAN_CASE(4)
        SEQ_SCAN_CASE(5) SEQ_SCAN_CASE(6) SEQ_SCAN_CASE(7) SEQ_SCAN_CASE(8)
      }
    });
    SEQ_CHECK_LAUNCH();
    return;
  }
  const int threads = ((Dv + WAVE - 1) / WAVE) * WAVE;
  TORCH_CHECK(threads <= 1024, "value size too large");
  const size_t lds =
      ((size_t)D * Dv + 3 * kScanTile * D + D + kScanTile * Dv) * sizeof(float);
  TORCH_CHECK(lds <= 160 * 1024, "head state does not fit LDS");
  SEQ_DISPATCH_ACT(q, {
    auto launch = [&](auto kern) {
      // raise the dynamic-LDS cap once per kernel, outside any capture
      static thread_local const void* raised[4] = {nullptr, nullptr, nullptr, nullptr};
      if (lds > 48 * 1024) {
        bool seen = false;
        for (auto p : raised) seen |= p == (const void*)kern;
        if (!seen) {
          hipFuncSetAttribute((const void*)kern,
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
          for (auto& p : raised)
            if (p == nullptr) { p = (const void*)kern; break; }
        }
      }
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
