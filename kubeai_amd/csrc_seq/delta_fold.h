// Segment-parallel walks of matrix-state recurrences whose transition is a
// full matrix per token (delta rules): over a segment of a run the state goes
// S -> P S + B with P [D, D] the product of the tokens' transition matrices
// and B [D, Dv] what the segment writes from zero. The scan kernels produce
// P (stored transposed) and B per segment; the fold kernel here chains
// S_(i+1) = P_i S_i + B_i, and the scan kernels then walk every segment from
// its incoming state. Shared by the delta-rule scans.
#pragma once

#include "seq_common.h"

namespace {

// Fold: grid (n_seq * H * column blocks), 256 threads. A block chains
// seg_state[i + 1] = P_i seg_state[i] + B_i for CB = 4 * (256 / (D / 4))
// value columns of one head (seg_state[0] is not written: the first segment
// starts from the slot). Every thread owns a 4 x 4 tile of the column block.
// P_i arrives transposed (seg_pt[k][i] = P_i[i][k]) and is staged in LDS as a
// whole, fetched into registers while the previous step is computed; the
// column block passes through LDS between the steps. Per contraction index a
// thread reads one float4 of P^T and one of S for 16 products.
template <int kD>
__global__ __launch_bounds__(256) void gated_delta_fold_kernel(
    float* __restrict__ seg_state, const float* __restrict__ seg_pt,
    const float* __restrict__ seg_b, const float* __restrict__ state,
    const int* __restrict__ start_loc, const int* __restrict__ slots,
    const int* __restrict__ positions, int H, int Dv, int ncbk, int nseg,
    int seg_len) {
  constexpr int RT = kD / 4;                       // row tiles
  constexpr int CT = 256 / RT;                     // column tiles of a block
  constexpr int CB = 4 * CT;                       // columns of a block
  constexpr int PV = (kD * kD / 4 + 255) / 256;    // float4 of P per thread
  extern __shared__ __attribute__((aligned(16))) float fold_sm[];
  float* pt = fold_sm;            // [kD][kD]
  float* sc = fold_sm + kD * kD;  // [kD][CB]
  const int cb = blockIdx.x % ncbk;
  const int h = (blockIdx.x / ncbk) % H;
  const int s = blockIdx.x / (ncbk * H);
  const int r0 = start_loc[s], n = start_loc[s + 1] - r0, slot = slots[s];
  const int used = (n + seg_len - 1) / seg_len;  // segments this run has
  if (used <= 1) return;                         // the whole block
  const int tid = threadIdx.x;
  const int rt = tid % RT, ct = tid / RT;
  const bool active = ct < CT;
  const int i0 = rt * 4, c0 = ct * 4, j0 = cb * CB + c0;
  const bool carry = slot >= 0 && positions[r0] > 0;
  const float* sp = state + ((size_t)(slot < 0 ? 0 : slot) * H + h) * kD * Dv;
  float S[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
      S[a][b] = (carry && active && j0 + b < Dv) ? sp[(size_t)(i0 + a) * Dv + j0 + b] : 0.f;
  float4 pre[PV];
  auto fetch = [&](int seg) {
    const float4* src =
        (const float4*)(seg_pt + (((size_t)s * nseg + seg) * H + h) * kD * kD);
#pragma unroll
    for (int v = 0; v < PV; ++v) {
      const int idx = v * 256 + tid;
      if (idx < kD * kD / 4) pre[v] = src[idx];
    }
  };
  fetch(0);
  for (int seg = 0; seg + 1 < used; ++seg) {
    const size_t sh = ((size_t)s * nseg + seg) * H + h;
    __syncthreads();  // the previous step's readers are done
#pragma unroll
    for (int v = 0; v < PV; ++v) {
      const int idx = v * 256 + tid;
      if (idx < kD * kD / 4) ((float4*)pt)[idx] = pre[v];
    }
    if (active) {
#pragma unroll
      for (int a = 0; a < 4; ++a)
        *(float4*)(sc + (i0 + a) * CB + c0) = make_float4(S[a][0], S[a][1], S[a][2], S[a][3]);
    }
    __syncthreads();
    if (seg + 2 < used) fetch(seg + 1);
    if (active) {
      const float* bp = seg_b + sh * kD * Dv;
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          S[a][b] = j0 + b < Dv ? bp[(size_t)(i0 + a) * Dv + j0 + b] : 0.f;
#pragma unroll 4
      for (int k = 0; k < kD; ++k) {
        const float4 p = *(const float4*)(pt + k * kD + i0);
        const float4 x = *(const float4*)(sc + k * CB + c0);
        const float pa[4] = {p.x, p.y, p.z, p.w};
        const float xa[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int b = 0; b < 4; ++b) S[a][b] += pa[a] * xa[b];
      }
      float* out = seg_state + (sh + H) * kD * Dv;  // segment seg + 1
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          if (j0 + b < Dv) out[(size_t)(i0 + a) * Dv + j0 + b] = S[a][b];
    }
  }
}


}  // namespace

// Segment length and count for runs of up to max_len tokens: the length
// balances the walk (proportional to it) against the fold (proportional to
// the number of segments); one segment means the run is walked as a whole.
static inline void delta_segments(int64_t max_len, int n_seq, int H, int D, int Dv,
                                  int* seg_len_out, int* nseg_out) {
  int seg_len = 128, nseg = 1;
  if (max_len > 2 * seg_len) {
    while ((int64_t)seg_len * seg_len < 8 * max_len) seg_len *= 2;
    nseg = (int)((max_len + seg_len - 1) / seg_len);
    while ((size_t)n_seq * nseg * H * D * (2 * Dv + D) * 4 > ((size_t)3 << 30)) {
      seg_len *= 2;
      nseg = (int)((max_len + seg_len - 1) / seg_len);
    }
  }
  if (nseg == 1) seg_len = (int)std::max<int64_t>(max_len, 1);  // one segment: the whole run
  *seg_len_out = seg_len;
  *nseg_out = nseg;
}

template <typename K>
static inline void delta_fold_launch_one(K kern, int D, int n_seq, int H, int Dv, int nseg,
                                         int seg_len, torch::Tensor& ws_s,
                                         torch::Tensor& ws_p, torch::Tensor& ws_b,
                                         torch::Tensor& state, torch::Tensor& start_loc,
                                         torch::Tensor& slots, torch::Tensor& positions) {
  const int cbk = 4 * (256 / (D / 4));  // value columns of a fold block
  const int ncbk = (Dv + cbk - 1) / cbk;
  const size_t fold_lds = ((size_t)D * D + (size_t)D * cbk) * sizeof(float);
  // raise the dynamic-LDS cap once per kernel, outside any capture
  static thread_local const void* raised[8] = {};
  if (fold_lds > 48 * 1024) {
    bool seen = false;
    for (auto p : raised) seen |= p == (const void*)kern;
    if (!seen) {
      hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                          160 * 1024);
      for (auto& p : raised)
        if (p == nullptr) { p = (const void*)kern; break; }
    }
  }
  hipLaunchKernelGGL(kern, dim3(n_seq * H * ncbk), dim3(256), fold_lds, SEQ_STREAM(),
                     (float*)ws_s.data_ptr(), (const float*)ws_p.data_ptr(),
                     (const float*)ws_b.data_ptr(), (const float*)state.data_ptr(),
                     (const int*)start_loc.data_ptr(), (const int*)slots.data_ptr(),
                     (const int*)positions.data_ptr(), H, Dv, ncbk, nseg, seg_len);
}

// D a multiple of 16, at most 128.
static inline void delta_fold_launch(int D, int n_seq, int H, int Dv, int nseg, int seg_len,
                                     torch::Tensor& ws_s, torch::Tensor& ws_p,
                                     torch::Tensor& ws_b, torch::Tensor& state,
                                     torch::Tensor& start_loc, torch::Tensor& slots,
                                     torch::Tensor& positions) {
#define DELTA_FOLD_CASE(KQ)                                                              \
  case KQ:                                                                               \
    delta_fold_launch_one(gated_delta_fold_kernel<16 * KQ>, D, n_seq, H, Dv, nseg,       \
                          seg_len, ws_s, ws_p, ws_b, state, start_loc, slots, positions); \
    break;
  switch (D / 16) {
    DELTA_FOLD_CASE(1) DELTA_FOLD_CASE(2) DELTA_FOLD_CASE(3) DELTA_FOLD_CASE(4)
    DELTA_FOLD_CASE(5) DELTA_FOLD_CASE(6) DELTA_FOLD_CASE(7) DELTA_FOLD_CASE(8)
    default: TORCH_CHECK(false, "fold: key size must be a multiple of 16 up to 128");
  }
#undef DELTA_FOLD_CASE
}
