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
//
// Long runs are cut into segments that run in parallel: over a segment the
// state goes S -> P S + B with P [D, D] the product of the tokens'
// diag(w) - (a * n) n^T and B what the segment writes from zero. B comes from
// walking from zero, the columns of P from walking the identity with zero
// values; the fold that chains the segments is shared with the gated delta
// rule (delta_fold.h).
#include "seq_common.h"
#include "delta_fold.h"

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

constexpr int kRegTile = 16;  // tokens staged per barrier (register-state kernel)

// Register-state form for key sizes D = 16 * kQ (<= 128). One wave per block
// owns 16 columns of one head's state over one segment of one run: lane
// (r, c) keeps rows [r D/4, (r+1) D/4) of column c in registers. Per token
// the lanes of a column take the dot product of the old column with n (two
// shuffles), rewrite their rows and take the dot product with the read-out
// vector (two shuffles). Decay, unit key, removal vector and read-out vector
// of kRegTile tokens are staged through LDS, activated once per token; the
// key as written is n * |k|. The next tile is fetched into registers while
// the current one is walked.
//
// mode 0 (walk): columns are value columns; the segment starts from the
//   slot's state (first segment), or from seg_state[seg] (later ones);
//   writes o, and the slot's state after the run's last segment.
// mode 1 (compose): column blocks [0, D/16) are columns of the identity
//   walked with zero values (-> seg_p, stored transposed), the rest value
//   columns walked from zero (-> seg_b); the run's last segment is skipped.
template <typename T, int kQ>
__global__ __launch_bounds__(WAVE) void diag_rank1_scan_reg_kernel(
    float* __restrict__ o, const T* __restrict__ r_in, int64_t r_stride,
    const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, const T* __restrict__ w_pre, int64_t w_stride,
    const T* __restrict__ a_pre, int64_t a_stride, const float* __restrict__ w_bias,
    const float* __restrict__ a_bias, float* __restrict__ state,
    const int* __restrict__ start_loc, const int* __restrict__ slots,
    const int* __restrict__ positions, int H, int Dv, int ncb, float decay_scale,
    float key_eps, int nseg, int seg_len, int mode, float* __restrict__ seg_p,
    float* __restrict__ seg_b, const float* __restrict__ seg_state) {
  constexpr int R = 4 * kQ, D = 4 * R;
  const int cb = blockIdx.x % ncb;
  const int h = (blockIdx.x / ncb) % H;
  const int seg = (blockIdx.x / (ncb * H)) % nseg;
  const int s = blockIdx.x / (ncb * H * nseg);
  const int r0 = start_loc[s], s1_run = start_loc[s + 1], slot = slots[s];
  const int s0 = r0 + seg * seg_len;
  const int s1 = min(s0 + seg_len, s1_run);
  if (s0 >= s1_run) return;
  const bool compose = mode == 1;
  if (compose && s1 == s1_run) return;
  __shared__ __attribute__((aligned(16))) float rs[kRegTile * D];  // read-out vector
  __shared__ __attribute__((aligned(16))) float ws[kRegTile * D];  // decay
  __shared__ __attribute__((aligned(16))) float ns[kRegTile * D];  // unit key
  __shared__ __attribute__((aligned(16))) float bs[kRegTile * D];  // removal rate * unit key
  __shared__ float vs[kRegTile * 16];
  __shared__ float kl[kRegTile];  // |k| (with key_eps under the root)
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
  // staging: lane (st_tt, st_part) owns a quarter row of one token of the tile
  typedef typename Raw4<T>::type raw4;
  const int st_tt = lane >> 2, st_part = lane & 3;
  const float* wb = w_bias + h * D + st_part * R;  // re-read per tile: they stay in cache
  const float* ab = a_bias + h * D + st_part * R;
  raw4 pr[kQ], pk[kQ], pw[kQ], pa[kQ];
  T pv[4];
  auto prefetch = [&](int tile0) {
    const int t = tile0 + st_tt;
    if (t < s1) {
      const size_t at = (size_t)h * D + st_part * R;
      const T* rp = r_in + (size_t)t * r_stride + at;
      const T* kp = k + (size_t)t * k_stride + at;
      const T* wp = w_pre + (size_t)t * w_stride + at;
      const T* ap = a_pre + (size_t)t * a_stride + at;
#pragma unroll
      for (int b = 0; b < kQ; ++b) {
        pr[b] = *(const raw4*)(rp + 4 * b);
        pk[b] = *(const raw4*)(kp + 4 * b);
        pw[b] = *(const raw4*)(wp + 4 * b);
        pa[b] = *(const raw4*)(ap + 4 * b);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int col = (cb - pcb) * 16 + st_part * 4 + e;
        pv[e] = (!ident && col < Dv) ? v[(size_t)t * v_stride + h * Dv + col] : (T)0;
      }
    }
  };
  prefetch(s0);
  for (int t0 = s0; t0 < s1; t0 += kRegTile) {
    const int nt = min(kRegTile, s1 - t0);
    __syncthreads();
    {
      float ka[R], xa[R];
      float sk = 0.f;
      if (st_tt < nt) {
#pragma unroll
        for (int b = 0; b < kQ; ++b) cvt4(pk[b], ka + 4 * b);
#pragma unroll
        for (int i = 0; i < R; ++i) sk += ka[i] * ka[i];
      }
      // the four lanes of a token are neighbours
      sk += __shfl_xor(sk, 1, WAVE);
      sk += __shfl_xor(sk, 2, WAVE);
      if (st_tt < nt) {
        const float len = sqrtf(sk + key_eps), rk = 1.0f / len;
        const int at = st_tt * D + st_part * R;
#pragma unroll
        for (int i = 0; i < R; ++i) ka[i] *= rk;
#pragma unroll
        for (int b = 0; b < kQ; ++b)
          *(float4*)(ns + at + 4 * b) =
              make_float4(ka[4 * b], ka[4 * b + 1], ka[4 * b + 2], ka[4 * b + 3]);
#pragma unroll
        for (int b = 0; b < kQ; ++b) cvt4(pa[b], xa + 4 * b);
#pragma unroll
        for (int i = 0; i < R; ++i) xa[i] = sigmoid_f(xa[i] + ab[i]) * ka[i];
#pragma unroll
        for (int b = 0; b < kQ; ++b)
          *(float4*)(bs + at + 4 * b) =
              make_float4(xa[4 * b], xa[4 * b + 1], xa[4 * b + 2], xa[4 * b + 3]);
#pragma unroll
        for (int b = 0; b < kQ; ++b) cvt4(pw[b], xa + 4 * b);
#pragma unroll
        for (int i = 0; i < R; ++i) xa[i] = expf(-decay_scale * sigmoid_f(xa[i] + wb[i]));
#pragma unroll
        for (int b = 0; b < kQ; ++b)
          *(float4*)(ws + at + 4 * b) =
              make_float4(xa[4 * b], xa[4 * b + 1], xa[4 * b + 2], xa[4 * b + 3]);
#pragma unroll
        for (int b = 0; b < kQ; ++b) cvt4(pr[b], xa + 4 * b);
#pragma unroll
        for (int b = 0; b < kQ; ++b)
          *(float4*)(rs + at + 4 * b) =
              make_float4(xa[4 * b], xa[4 * b + 1], xa[4 * b + 2], xa[4 * b + 3]);
#pragma unroll
        for (int e = 0; e < 4; ++e) vs[st_tt * 16 + st_part * 4 + e] = ldf(&pv[e]);
        if (st_part == 0) kl[st_tt] = len;
      }
    }
    __syncthreads();
    if (t0 + kRegTile < s1) prefetch(t0 + kRegTile);
    for (int tt = 0; tt < nt; ++tt) {
      const float kv = kl[tt] * vs[tt * 16 + c];  // n * (|k| v) = k v
      const float4* n4 = (const float4*)(ns + tt * D + r * R);
      const float4* w4 = (const float4*)(ws + tt * D + r * R);
      const float4* b4 = (const float4*)(bs + tt * D + r * R);
      const float4* r4 = (const float4*)(rs + tt * D + r * R);
      float na[R];
      float dot = 0.f;
#pragma unroll
      for (int b = 0; b < kQ; ++b) {
        const float4 nn = n4[b];
        na[4 * b] = nn.x; na[4 * b + 1] = nn.y; na[4 * b + 2] = nn.z; na[4 * b + 3] = nn.w;
      }
#pragma unroll
      for (int i = 0; i < R; ++i) dot += S[i] * na[i];
      dot += __shfl_xor(dot, 16, WAVE);
      dot += __shfl_xor(dot, 32, WAVE);
      float acc = 0.f;
#pragma unroll
      for (int b = 0; b < kQ; ++b) {
        const float4 ww = w4[b], bb = b4[b], rr = r4[b];
        const float wa[4] = {ww.x, ww.y, ww.z, ww.w};
        const float ba[4] = {bb.x, bb.y, bb.z, bb.w};
        const float ra[4] = {rr.x, rr.y, rr.z, rr.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = 4 * b + e;
          S[i] = wa[e] * S[i] - ba[e] * dot + na[i] * kv;
          acc += ra[e] * S[i];
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
  auto vec_ok = [&](const torch::Tensor& t) {
    const size_t bytes = 4 * t.element_size();
    return ((size_t)t.data_ptr()) % bytes == 0 && t.stride(0) % 4 == 0;
  };
  if (D % 16 == 0 && D <= 128 && vec_ok(r) && vec_ok(k) && vec_ok(w_pre) && vec_ok(a_pre)) {
    const int ncb = (Dv + 15) / 16;
    int seg_len, nseg;
    delta_segments(max_len, n_seq, H, D, Dv, &seg_len, &nseg);
    torch::Tensor ws_p, ws_b, ws_s;
    if (nseg > 1) {
      ws_p = torch::empty({(int64_t)n_seq * nseg * H * D * D}, state.options());
      ws_b = torch::empty({(int64_t)n_seq * nseg * H * D * Dv}, state.options());
      ws_s = torch::empty({(int64_t)n_seq * nseg * H * D * Dv}, state.options());
    }
    SEQ_DISPATCH_ACT(k, {
      auto launch1 = [&](auto kern, int mode) {
        const int blocks_cb = mode == 1 ? ncb + D / 16 : ncb;
        hipLaunchKernelGGL(kern, dim3(n_seq * nseg * H * blocks_cb), dim3(WAVE), 0,
                           SEQ_STREAM(), (float*)o.data_ptr(),
                           (const act_t*)r.data_ptr(), r.stride(0),
                           (const act_t*)k.data_ptr(), k.stride(0),
                           (const act_t*)v.data_ptr(), v.stride(0),
                           (const act_t*)w_pre.data_ptr(), w_pre.stride(0),
                           (const act_t*)a_pre.data_ptr(), a_pre.stride(0),
                           (const float*)w_bias.data_ptr(), (const float*)a_bias.data_ptr(),
                           (float*)state.data_ptr(), (const int*)start_loc.data_ptr(),
                           (const int*)slots.data_ptr(), (const int*)positions.data_ptr(),
                           H, Dv, blocks_cb, (float)decay_scale, (float)key_eps, nseg,
                           seg_len, mode, nseg > 1 ? (float*)ws_p.data_ptr() : nullptr,
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
        case 1: launch(diag_rank1_scan_reg_kernel<act_t, 1>); break;
        case 2: launch(diag_rank1_scan_reg_kernel<act_t, 2>); break;
        case 3: launch(diag_rank1_scan_reg_kernel<act_t, 3>); break;
        case 4: launch(diag_rank1_scan_reg_kernel<act_t, 4>); break;
        case 5: launch(diag_rank1_scan_reg_kernel<act_t, 5>); break;
        case 6: launch(diag_rank1_scan_reg_kernel<act_t, 6>); break;
        case 7: launch(diag_rank1_scan_reg_kernel<act_t, 7>); break;
        case 8: launch(diag_rank1_scan_reg_kernel<act_t, 8>); break;
      }
    });
    SEQ_CHECK_LAUNCH();
    return;
  }
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
