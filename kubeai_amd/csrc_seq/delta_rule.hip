// Gated delta rule over the runs of a packed step. Per head a matrix state
// S [D, Dv] (fp32, one slot per sequence):
//
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//
// with q, k unit vectors per head (q times D^-1/2), beta = sigmoid(b),
// g = exp(-exp(a_log) softplus(a + dt_bias)). Everything but the loads of
// q, k, v, a, b (serving dtype) is fp32. The value columns of a head are
// independent of each other, so a head is split over waves by column.
//
// Long runs are cut into segments that run in parallel. Over a segment the
// state goes S -> P S + B with P [D, D] the product of the tokens'
// g (I - beta k k^T) and B [D, Dv] what the segment writes from zero. Both
// come out of the same recurrence: B by walking from zero, P by walking the
// identity with zero values. Pass 1 (compose) walks every segment but the
// last for P and B, pass 2 (fold) chains S_(i+1) = P_i S_i + B_i per column
// block with P_i staged in LDS, pass 3 walks every segment from its incoming
// state and writes o.
#include "seq_common.h"
#include "delta_fold.h"

namespace {

constexpr int kTile = 16;  // tokens staged per barrier

DEV_INLINE float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// Any size: grid (n_seq * H, column blocks), block = the block's columns
// rounded up to a wave, that part of the head's state in LDS, thread j owns
// value column c0 + j.
template <typename T>
__global__ void gated_delta_scan_kernel(
    float* __restrict__ o, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, const T* __restrict__ beta_pre, int64_t b_stride,
    const T* __restrict__ decay_pre, int64_t a_stride,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    float* __restrict__ state, const int* __restrict__ start_loc,
    const int* __restrict__ slots, const int* __restrict__ positions, int H, int G,
    int D, int Dv, int CB, float norm_eps) {
  const int s = blockIdx.x / H, h = blockIdx.x % H;
  const int hk = h / (H / G);
  const int s0 = start_loc[s], s1 = start_loc[s + 1], slot = slots[s];
  if (s1 <= s0) return;
  const int c0 = blockIdx.y * CB, nc = min(CB, Dv - c0);  // this block's columns
  extern __shared__ float sm[];
  float* S = sm;                      // [D][CB]
  float* qs = S + (size_t)D * CB;     // [tile][D]
  float* ks = qs + kTile * D;         // [tile][D]
  float* vs = ks + kTile * D;         // [tile][CB]
  float* gb = vs + kTile * CB;        // [tile][2]: decay, beta
  const int tid = threadIdx.x, nthr = blockDim.x;
  const bool carry = slot >= 0 && positions[s0] > 0;
  float* sp = state + ((size_t)(slot < 0 ? 0 : slot) * H + h) * D * Dv;
  for (int i = tid; i < D * CB; i += nthr) {
    const int r = i / CB, c = i % CB;
    S[i] = (carry && c < nc) ? sp[(size_t)r * Dv + c0 + c] : 0.f;
  }
  const float rate = -expf(a_log[h]), bias = dt_bias[h];
  const float qscale = 1.0f / sqrtf((float)D);
  for (int t0 = s0; t0 < s1; t0 += kTile) {
    const int nt = min(kTile, s1 - t0);
    __syncthreads();  // the previous tile's readers are done
    for (int i = tid; i < nt * D; i += nthr) {
      const int tt = i / D, d = i % D;
      qs[i] = ldf(q + (size_t)(t0 + tt) * q_stride + hk * D + d);
      ks[i] = ldf(k + (size_t)(t0 + tt) * k_stride + hk * D + d);
    }
    for (int i = tid; i < nt * CB; i += nthr) {
      const int tt = i / CB, d = i % CB;
      vs[i] = d < nc ? ldf(v + (size_t)(t0 + tt) * v_stride + h * Dv + c0 + d) : 0.f;
    }
    __syncthreads();
    if (tid < nt) {
      float sq = 0.f, sk = 0.f;
      for (int d = 0; d < D; ++d) {
        sq += qs[tid * D + d] * qs[tid * D + d];
        sk += ks[tid * D + d] * ks[tid * D + d];
      }
      const float rq = qscale / sqrtf(sq + norm_eps), rk = 1.0f / sqrtf(sk + norm_eps);
      for (int d = 0; d < D; ++d) {
        qs[tid * D + d] *= rq;
        ks[tid * D + d] *= rk;
      }
      const float a = ldf(decay_pre + (size_t)(t0 + tid) * a_stride + h);
      gb[2 * tid] = expf(rate * softplus_f(a + bias));
      gb[2 * tid + 1] = sigmoid_f(ldf(beta_pre + (size_t)(t0 + tid) * b_stride + h));
    }
    __syncthreads();
    if (tid < nc) {
      for (int tt = 0; tt < nt; ++tt) {
        const float* qt = qs + tt * D;
        const float* kt = ks + tt * D;
        const float g = gb[2 * tt], beta = gb[2 * tt + 1];
        float dot = 0.f;
        for (int i = 0; i < D; ++i) {
          const float st = g * S[i * CB + tid];
          S[i * CB + tid] = st;
          dot += st * kt[i];
        }
        const float u = beta * (vs[tt * CB + tid] - dot);
        float acc = 0.f;
        for (int i = 0; i < D; ++i) {
          const float st = S[i * CB + tid] + kt[i] * u;
          S[i * CB + tid] = st;
          acc += qt[i] * st;
        }
        o[((size_t)(t0 + tt) * H + h) * Dv + c0 + tid] = acc;
      }
    }
  }
  __syncthreads();
  if (slot >= 0)
    for (int i = tid; i < D * CB; i += nthr) {
      const int r = i / CB, c = i % CB;
      if (c < nc) sp[(size_t)r * Dv + c0 + c] = S[i];
    }
}

// Register-state form for key sizes D = 16 * kQ (<= 128). One wave per block
// owns 16 columns of one head's state over one segment of one run: lane
// (r, c) keeps rows [r D/4, (r+1) D/4) of column c in registers, so a token
// costs two passes over D/4 registers and two pairs of shuffles (the dot
// with k before the write, the dot with q after it). q, k of kTile tokens
// are staged through LDS, normalised once per token; the next tile is
// fetched into registers while the current one is walked.
//
// mode 0 (walk): columns are value columns; the segment starts from the
//   slot's state (first segment), or from seg_state[seg] (later ones);
//   writes o, and the slot's state after the run's last segment.
// mode 1 (compose): column blocks [0, D/16) are columns of the identity
//   walked with zero values (-> seg_p, stored transposed), the rest value
//   columns walked from zero (-> seg_b); the run's last segment is skipped.
template <typename T, int kQ>
__global__ __launch_bounds__(WAVE) void gated_delta_scan_reg_kernel(
    float* __restrict__ o, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, const T* __restrict__ beta_pre, int64_t b_stride,
    const T* __restrict__ decay_pre, int64_t a_stride,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    float* __restrict__ state, const int* __restrict__ start_loc,
    const int* __restrict__ slots, const int* __restrict__ positions, int H, int G,
    int Dv, int ncb, float norm_eps, int nseg, int seg_len, int mode,
    float* __restrict__ seg_p, float* __restrict__ seg_b,
    const float* __restrict__ seg_state) {
  constexpr int R = 4 * kQ, D = 4 * R;
  const int cb = blockIdx.x % ncb;
  const int h = (blockIdx.x / ncb) % H;
  const int seg = (blockIdx.x / (ncb * H)) % nseg;
  const int s = blockIdx.x / (ncb * H * nseg);
  const int hk = h / (H / G);
  const int r0 = start_loc[s], s1_run = start_loc[s + 1], slot = slots[s];
  const int s0 = r0 + seg * seg_len;
  const int s1 = min(s0 + seg_len, s1_run);
  if (s0 >= s1_run) return;
  const bool compose = mode == 1;
  if (compose && s1 == s1_run) return;
  __shared__ __attribute__((aligned(16))) float qs[kTile * D];
  __shared__ __attribute__((aligned(16))) float ks[kTile * D];
  __shared__ float vs[kTile * 16];
  __shared__ float gb[kTile * 2];
  const int lane = threadIdx.x, r = lane >> 4, c = lane & 15;
  // compose: the first D/16 column blocks walk the identity
  const int pcb = compose ? D / 16 : 0;
  const bool ident = cb < pcb;
  const int j = (cb - pcb) * 16 + c;  // value column (when not ident)
  const bool valid = ident || j < Dv;
  float S[R];
  if (compose) {
#pragma unroll
    for (int i = 0; i < R; ++i) S[i] = (ident && r * R + i == cb * 16 + c) ? 1.f : 0.f;
  } else if (seg > 0) {
    const float* ss = seg_state + (((size_t)s * nseg + seg) * H + h) * D * Dv;
#pragma unroll
    for (int i = 0; i < R; ++i) S[i] = valid ? ss[(size_t)(r * R + i) * Dv + j] : 0.f;
  } else {
    const bool carry = slot >= 0 && positions[r0] > 0;
    const float* sp = state + ((size_t)(slot < 0 ? 0 : slot) * H + h) * D * Dv;
#pragma unroll
    for (int i = 0; i < R; ++i)
      S[i] = (carry && valid) ? sp[(size_t)(r * R + i) * Dv + j] : 0.f;
  }
  const float rate = -expf(a_log[h]), bias = dt_bias[h];
  const float qscale = 1.0f / sqrtf((float)D);
  // staging: lane (st_tt, st_part) owns a quarter row of one token of the tile
  typedef typename Raw4<T>::type raw4;
  const int st_tt = lane >> 2, st_part = lane & 3;
  raw4 pq[kQ], pk[kQ];
  T pv[4], pa, pb;
  auto prefetch = [&](int tile0) {
    const int t = tile0 + st_tt;
    if (t < s1) {
      const T* qp = q + (size_t)t * q_stride + hk * D + st_part * R;
      const T* kp = k + (size_t)t * k_stride + hk * D + st_part * R;
#pragma unroll
      for (int b = 0; b < kQ; ++b) {
        pq[b] = *(const raw4*)(qp + 4 * b);
        pk[b] = *(const raw4*)(kp + 4 * b);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int col = (cb - pcb) * 16 + st_part * 4 + e;
        pv[e] = (!ident && col < Dv) ? v[(size_t)t * v_stride + h * Dv + col] : (T)0;
      }
      if (st_part == 0) {
        pa = decay_pre[(size_t)t * a_stride + h];
        pb = beta_pre[(size_t)t * b_stride + h];
      }
    }
  };
  prefetch(s0);
  for (int t0 = s0; t0 < s1; t0 += kTile) {
    const int nt = min(kTile, s1 - t0);
    __syncthreads();
    {
      float qa[R], ka[R];
      float sq = 0.f, sk = 0.f;
      if (st_tt < nt) {
#pragma unroll
        for (int b = 0; b < kQ; ++b) {
          cvt4(pq[b], qa + 4 * b);
          cvt4(pk[b], ka + 4 * b);
        }
#pragma unroll
        for (int i = 0; i < R; ++i) {
          sq += qa[i] * qa[i];
          sk += ka[i] * ka[i];
        }
      }
      // the four lanes of a token are neighbours
      sq += __shfl_xor(sq, 1, WAVE);
      sq += __shfl_xor(sq, 2, WAVE);
      sk += __shfl_xor(sk, 1, WAVE);
      sk += __shfl_xor(sk, 2, WAVE);
      if (st_tt < nt) {
        const float rq = qscale / sqrtf(sq + norm_eps), rk = 1.0f / sqrtf(sk + norm_eps);
        const int at = st_tt * D + st_part * R;
#pragma unroll
        for (int b = 0; b < kQ; ++b) {
          *(float4*)(qs + at + 4 * b) = make_float4(qa[4 * b] * rq, qa[4 * b + 1] * rq,
                                                    qa[4 * b + 2] * rq, qa[4 * b + 3] * rq);
          *(float4*)(ks + at + 4 * b) = make_float4(ka[4 * b] * rk, ka[4 * b + 1] * rk,
                                                    ka[4 * b + 2] * rk, ka[4 * b + 3] * rk);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) vs[st_tt * 16 + st_part * 4 + e] = ldf(&pv[e]);
        if (st_part == 0) {
          gb[2 * st_tt] = expf(rate * softplus_f(ldf(&pa) + bias));
          gb[2 * st_tt + 1] = sigmoid_f(ldf(&pb));
        }
      }
    }
    __syncthreads();
    if (t0 + kTile < s1) prefetch(t0 + kTile);
    for (int tt = 0; tt < nt; ++tt) {
      const float vj = vs[tt * 16 + c];
      const float g = gb[2 * tt], beta = gb[2 * tt + 1];
      const float4* q4 = (const float4*)(qs + tt * D + r * R);
      const float4* k4 = (const float4*)(ks + tt * D + r * R);
      float ka[R];
      float dot = 0.f;
#pragma unroll
      for (int b = 0; b < kQ; ++b) {
        const float4 kk = k4[b];
        ka[4 * b] = kk.x; ka[4 * b + 1] = kk.y; ka[4 * b + 2] = kk.z; ka[4 * b + 3] = kk.w;
      }
#pragma unroll
      for (int i = 0; i < R; ++i) {
        S[i] *= g;
        dot += S[i] * ka[i];
      }
      dot += __shfl_xor(dot, 16, WAVE);
      dot += __shfl_xor(dot, 32, WAVE);
      const float u = beta * (vj - dot);
      float acc = 0.f;
#pragma unroll
      for (int b = 0; b < kQ; ++b) {
        const float4 qq = q4[b];
        const float qa[4] = {qq.x, qq.y, qq.z, qq.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = 4 * b + e;
          S[i] += ka[i] * u;
          acc += qa[e] * S[i];
        }
      }
      if (!compose) {
        acc += __shfl_xor(acc, 16, WAVE);
        acc += __shfl_xor(acc, 32, WAVE);
        if (r == 0 && valid) o[((size_t)(t0 + tt) * H + h) * Dv + j] = acc;
      }
    }
  }
  if (compose) {
    const size_t sh = ((size_t)s * nseg + seg) * H + h;
    if (ident) {
      float* pp = seg_p + sh * D * D;
#pragma unroll
      for (int i = 0; i < R; ++i) pp[(size_t)(cb * 16 + c) * D + r * R + i] = S[i];  // P^T
    } else if (valid) {
      float* bp = seg_b + sh * D * Dv;
#pragma unroll
      for (int i = 0; i < R; ++i) bp[(size_t)(r * R + i) * Dv + j] = S[i];
    }
  } else if (slot >= 0 && valid && s1 == s1_run) {
    float* sp = state + ((size_t)slot * H + h) * D * Dv;
#pragma unroll
    for (int i = 0; i < R; ++i) sp[(size_t)(r * R + i) * Dv + j] = S[i];
  }
}

}  // namespace

#define DELTA_CASE(KQ)                                              \
  case KQ:                                                          \
    launch(gated_delta_scan_reg_kernel<act_t, KQ>);                 \
    break;

void gated_delta_scan(torch::Tensor o, torch::Tensor q, torch::Tensor k,
                      torch::Tensor v, torch::Tensor beta_pre, torch::Tensor decay_pre,
                      torch::Tensor a_log, torch::Tensor dt_bias, torch::Tensor state,
                      torch::Tensor start_loc, torch::Tensor slots,
                      torch::Tensor positions, double norm_eps, int64_t max_len) {
  check_f32(o, "o");
  check_f32(state, "state");
  check_f32(a_log, "a_log");
  check_f32(dt_bias, "dt_bias");
  check_i32(start_loc, "start_loc");
  check_i32(slots, "slots");
  check_i32(positions, "positions");
  check_rows(beta_pre, "beta_pre");
  check_rows(decay_pre, "decay_pre");
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3 && q.is_cuda());
  const int T = q.size(0), G = q.size(1), D = q.size(2), H = v.size(1), Dv = v.size(2);
  auto dense_heads = [](const torch::Tensor& t) {
    return t.stride(2) == 1 && (t.size(1) == 1 || t.stride(1) == t.size(2));
  };
  TORCH_CHECK(dense_heads(q) && dense_heads(k) && dense_heads(v),
              "q/k/v heads must be dense within a row");
  TORCH_CHECK(k.size(0) == T && k.size(1) == G && k.size(2) == D && v.size(0) == T);
  TORCH_CHECK(G > 0 && H % G == 0, "value heads must be a multiple of q/k heads");
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type() &&
              beta_pre.scalar_type() == q.scalar_type() &&
              decay_pre.scalar_type() == q.scalar_type());
  TORCH_CHECK(beta_pre.size(0) == T && beta_pre.size(1) == H && decay_pre.size(0) == T &&
              decay_pre.size(1) == H && a_log.numel() == H && dt_bias.numel() == H);
  TORCH_CHECK(o.size(0) == T && o.size(1) == H && o.size(2) == Dv);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D &&
              state.size(3) == Dv);
  TORCH_CHECK(start_loc.numel() == slots.numel() + 1 && positions.numel() == T);
  const int n_seq = slots.numel();
  if (n_seq == 0 || T == 0) return;
  auto vec_ok = [&](const torch::Tensor& t) {
    const size_t bytes = 4 * t.element_size();
    return ((size_t)t.data_ptr()) % bytes == 0 && t.stride(0) % 4 == 0;
  };
  if (D % 16 == 0 && D <= 128 && vec_ok(q) && vec_ok(k)) {
    const int ncb = (Dv + 15) / 16;
    int seg_len, nseg;
    delta_segments(max_len, n_seq, H, D, Dv, &seg_len, &nseg);
    torch::Tensor ws_p, ws_b, ws_s;
    if (nseg > 1) {
      ws_p = torch::empty({(int64_t)n_seq * nseg * H * D * D}, state.options());
      ws_b = torch::empty({(int64_t)n_seq * nseg * H * D * Dv}, state.options());
      ws_s = torch::empty({(int64_t)n_seq * nseg * H * D * Dv}, state.options());
    }
    SEQ_DISPATCH_ACT(q, {
      auto launch1 = [&](auto kern, int mode) {
        const int blocks_cb = mode == 1 ? ncb + D / 16 : ncb;
        hipLaunchKernelGGL(kern, dim3(n_seq * nseg * H * blocks_cb), dim3(WAVE), 0,
                           SEQ_STREAM(), (float*)o.data_ptr(),
                           (const act_t*)q.data_ptr(), q.stride(0),
                           (const act_t*)k.data_ptr(), k.stride(0),
                           (const act_t*)v.data_ptr(), v.stride(0),
                           (const act_t*)beta_pre.data_ptr(), beta_pre.stride(0),
                           (const act_t*)decay_pre.data_ptr(), decay_pre.stride(0),
                           (const float*)a_log.data_ptr(),
                           (const float*)dt_bias.data_ptr(), (float*)state.data_ptr(),
                           (const int*)start_loc.data_ptr(),
                           (const int*)slots.data_ptr(),
                           (const int*)positions.data_ptr(), H, G, Dv, blocks_cb,
                           (float)norm_eps, nseg, seg_len, mode,
                           nseg > 1 ? (float*)ws_p.data_ptr() : nullptr,
                           nseg > 1 ? (float*)ws_b.data_ptr() : nullptr,
                           nseg > 1 ? (const float*)ws_s.data_ptr() : nullptr);
      };
      auto launch = [&](auto kern) {
        if (nseg > 1) {
          launch1(kern, 1);
          delta_fold_launch(D, n_seq, H, Dv, nseg, seg_len, ws_s, ws_p, ws_b, state,
                            start_loc, slots, positions);
        }
        launch1(kern, 0);
      };
      switch (D / 16) {
        DELTA_CASE(1) DELTA_CASE(2) DELTA_CASE(3) DELTA_CASE(4)
        DELTA_CASE(5) DELTA_CASE(6) DELTA_CASE(7) DELTA_CASE(8)
      }
    });
    SEQ_CHECK_LAUNCH();
    return;
  }
  // value columns per block: all of them if the state fits LDS, else fewer
  // (columns are independent), in whole waves
  auto lds_for = [&](int cb) {
    return ((size_t)D * cb + 2 * kTile * D + (size_t)kTile * cb + 2 * kTile) * sizeof(float);
  };
  int CB = std::min(((Dv + WAVE - 1) / WAVE) * WAVE, 1024);
  while (CB > WAVE && lds_for(CB) > 144 * 1024) CB -= WAVE;
  const size_t lds = lds_for(CB);
  TORCH_CHECK(lds <= 160 * 1024, "key size too large for the LDS state");
  const int threads = CB, ncb_gen = (Dv + CB - 1) / CB;
  TORCH_CHECK(ncb_gen <= 65535);
  SEQ_DISPATCH_ACT(q, {
    auto kern = gated_delta_scan_kernel<act_t>;
    // raise the dynamic-LDS cap once per kernel, outside any capture
    static thread_local const void* raised[2] = {nullptr, nullptr};
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
    hipLaunchKernelGGL(kern, dim3(n_seq * H, ncb_gen), dim3(threads), lds, SEQ_STREAM(),
                       (float*)o.data_ptr(), (const act_t*)q.data_ptr(), q.stride(0),
                       (const act_t*)k.data_ptr(), k.stride(0),
                       (const act_t*)v.data_ptr(), v.stride(0),
                       (const act_t*)beta_pre.data_ptr(), beta_pre.stride(0),
                       (const act_t*)decay_pre.data_ptr(), decay_pre.stride(0),
                       (const float*)a_log.data_ptr(), (const float*)dt_bias.data_ptr(),
                       (float*)state.data_ptr(), (const int*)start_loc.data_ptr(),
                       (const int*)slots.data_ptr(), (const int*)positions.data_ptr(), H,
                       G, D, Dv, CB, (float)norm_eps);
  });
  SEQ_CHECK_LAUNCH();
}
