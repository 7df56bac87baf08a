// Rotary (interleaved pairs, or split halves after a whole-row RMS norm of q
// and k) fused with the paged cache write, and softmax attention of every
// packed token over its own sequence's cached keys under a chunk / window
// mask, with separate key and value sizes and an optional sink (a key of
// score 0 without a value: one more term in the denominator).
#include "seq_common.h"

namespace {

// grid (T): q pairs rotate in place; k pairs rotate into the key cache;
// v copies into the value cache. Angles are fp32: position * inv_freq[i].
template <typename T>
__global__ void rope_pairs_cache_kernel(
    T* __restrict__ q, int64_t q_stride, const T* __restrict__ k,
    int64_t k_stride, const T* __restrict__ v, int64_t v_stride,
    const int* __restrict__ positions, const float* __restrict__ inv_freq,
    int half, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, int H, int G, int D, int Dv,
    int bs) {
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  const int64_t slot = slot_mapping[t];
  const int hp = D / 2;
  const int nqp = H * hp, nkp = G * hp, nv = G * Dv;
  const int64_t blk = slot >= 0 ? slot / bs : 0;
  const int off = slot >= 0 ? (int)(slot % bs) : 0;
  for (int u = threadIdx.x; u < nqp + nkp + nv; u += blockDim.x) {
    if (u < nqp + nkp) {
      const bool is_q = u < nqp;
      const int uu = is_q ? u : u - nqp;
      const int hd = uu / hp, i = uu % hp;
      const T* src = is_q ? q + (size_t)t * q_stride + hd * D + 2 * i
                          : k + (size_t)t * k_stride + hd * D + 2 * i;
      float a = ldf(src), b = ldf(src + 1);
      if (i < half) {
        float sn, cs;
        sincosf(pos * inv_freq[i], &sn, &cs);
        const float ra = a * cs - b * sn, rb = b * cs + a * sn;
        a = ra;
        b = rb;
      }
      if (is_q) {
        if (i < half) {
          T* dst = q + (size_t)t * q_stride + hd * D + 2 * i;
          stf(dst, a);
          stf(dst + 1, b);
        }
      } else if (slot >= 0) {
        T* dst = k_cache + (((size_t)blk * G + hd) * bs + off) * D + 2 * i;
        stf(dst, a);
        stf(dst + 1, b);
      }
    } else if (slot >= 0) {
      const int e = u - nqp - nkp;
      const int g = e / Dv, d = e % Dv;
      v_cache[(((size_t)blk * G + g) * bs + off) * Dv + d] =
          v[(size_t)t * v_stride + g * Dv + d];
    }
  }
}

// grid (T). q and k rows are RMS-normed as a whole (all heads at once, plain
// weights), then the first 2 * half dims of every head rotate with dimension
// i paired with i + half; the rest pass. q is rewritten in place, k goes to
// the key cache, v is copied to the value cache. fp32 throughout.
template <typename T>
__global__ __launch_bounds__(256) void qknorm_rope_half_cache_kernel(
    T* __restrict__ q, int64_t q_stride, const T* __restrict__ k,
    int64_t k_stride, const T* __restrict__ v, int64_t v_stride,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    const int* __restrict__ positions, const float* __restrict__ inv_freq,
    int half, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, int H, int G, int D, int Dv,
    int bs) {
  __shared__ float red0[16], red1[16];
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  const int64_t slot = slot_mapping[t];
  T* qr = q + (size_t)t * q_stride;
  const T* kr = k + (size_t)t * k_stride;
  float rq = 1.f, rk = 1.f;
  if (qw != nullptr) {
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < H * D; i += blockDim.x) {
      const float x = ldf(qr + i);
      sq += x * x;
    }
    for (int i = threadIdx.x; i < G * D; i += blockDim.x) {
      const float x = ldf(kr + i);
      sk += x * x;
    }
    rq = 1.0f / sqrtf(block_sum(sq, red0) / (float)(H * D) + eps);
    rk = 1.0f / sqrtf(block_sum(sk, red1) / (float)(G * D) + eps);
  }
  const int upr = D - half;  // units per head: `half` pairs, then single dims
  const int nq = H * upr, nk = G * upr, nv = G * Dv;
  const int64_t blk = slot >= 0 ? slot / bs : 0;
  const int off = slot >= 0 ? (int)(slot % bs) : 0;
  for (int u = threadIdx.x; u < nq + nk + nv; u += blockDim.x) {
    if (u < nq + nk) {
      const bool is_q = u < nq;
      const int uu = is_q ? u : u - nq;
      const int hd = uu / upr, i = uu % upr;
      if (!is_q && slot < 0) continue;
      const T* src = is_q ? qr + hd * D : kr + hd * D;
      const float* w = is_q ? qw : kw;
      const float r = is_q ? rq : rk;
      T* dst = is_q ? qr + hd * D
                    : k_cache + (((size_t)blk * G + hd) * bs + off) * D;
      if (i < half) {
        float a = ldf(src + i) * r, b = ldf(src + i + half) * r;
        if (w != nullptr) {
          a *= w[hd * D + i];
          b *= w[hd * D + i + half];
        }
        float sn, cs;
        sincosf(pos * inv_freq[i], &sn, &cs);
        stf(dst + i, a * cs - b * sn);
        stf(dst + i + half, b * cs + a * sn);
      } else {
        const int d = i + half;
        float a = ldf(src + d) * r;
        if (w != nullptr) a *= w[hd * D + d];
        stf(dst + d, a);
      }
    } else if (slot >= 0) {
      const int e = u - nq - nk;
      const int g = e / Dv, d = e % Dv;
      v_cache[(((size_t)blk * G + g) * bs + off) * Dv + d] =
          v[(size_t)t * v_stride + g * Dv + d];
    }
  }
}

constexpr int kMaxDvPerLane = 16;  // value size <= 1024

constexpr int kDecWaves = 4;

// grid (T, H), kDecWaves waves per (token, query head). Keys are walked in
// tiles of 64, dealt round-robin to the waves (a decode token alone cannot
// hide memory latency, so its keys are split): each lane scores one key
// (fp32 dot, cap, mask), the wave keeps a running max / sum, then its lanes
// turn to the values and accumulate p . V for the tile. The waves' partial
// results are joined through LDS at the end. Serves single decode tokens
// (and, in fp32 or at odd sizes, prompt portions): every token reads its
// keys, this step's included, from the cache.
//
// kVec: key and value rows are read with 16-byte loads. For the values a
// wave splits into 64 / (Dv / N) key groups, each lane owning N value
// channels of its group's keys.
template <typename T, bool kVec>
__global__ __launch_bounds__(kDecWaves * WAVE) void masked_paged_attention_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ q,
    int64_t q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ block_tables,
    int max_blocks, const int* __restrict__ token_seq,
    const int* __restrict__ positions, float scale, float softcap, int chunk,
    int window, float out_scale, const float* __restrict__ sink, int64_t v_rs, int H, int G, int D, int Dv, int bs,
    int kvs) {
  constexpr int N = Vec16<T>::N;
  const int lpr = kVec ? Dv / N : 1;          // lanes per value row
  const int ngrp = kVec ? WAVE / lpr : 1;     // key groups of a wave
  extern __shared__ float sm[];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  int64_t* vbase = (int64_t*)sm + wave * WAVE;       // [waves][64] value row offsets
  float* ps = sm + 2 * WAVE * kDecWaves + wave * WAVE;  // [waves][64] probabilities
  float* stat = sm + 3 * WAVE * kDecWaves;           // [waves][2] max, sum
  float* qs = stat + 2 * kDecWaves;                  // [D]
  float* red_all = qs + ((D + 3) & ~3);              // [waves][groups][Dv]
  float* red = red_all + (size_t)wave * ngrp * Dv;
  const int t = blockIdx.x, h = blockIdx.y;
  const int g = h / (H / G);
  const int pos = positions[t];
  const int* bt = block_tables + (size_t)token_seq[t] * max_blocks;
  int lo = 0;
  if (chunk > 0) lo = (pos / chunk) * chunk;
  if (window > 0) lo = max(lo, pos - window + 1);
  for (int i = threadIdx.x; i < D; i += blockDim.x)
    qs[i] = ldf(q + (size_t)t * q_stride + h * D + i);
  __syncthreads();
  const int kg = lane / lpr, lv = lane % lpr;
  const bool v_on = kVec && kg < ngrp;
  float m = -INFINITY, l = 0.f;
  float acc[kMaxDvPerLane];
#pragma unroll
  for (int i = 0; i < kMaxDvPerLane; ++i) acc[i] = 0.f;
  // the wave's own LDS rows are touched by this wave only, so the tile loop
  // needs no block barrier (a wave's LDS accesses complete in order)
  for (int j0 = lo + wave * WAVE; j0 <= pos; j0 += kDecWaves * WAVE) {
    const int j = j0 + lane;
    float sc = -INFINITY;
    int64_t vb = 0;
    if (j <= pos) {
      const int64_t blk = bt[j / bs];
      const int64_t rowi = (blk * G + g) * bs + (j % bs);
      const T* kp = k_cache + rowi * D;
      float dot = 0.f;
      if (kVec) {
        for (int i = 0; i < D; i += N) {
          float x[N];
          Vec16<T>::load(kp + i, x);
#pragma unroll
          for (int e = 0; e < N; ++e) dot += qs[i + e] * x[e];
        }
      } else {
        for (int i = 0; i < D; ++i) dot += qs[i] * ldf(kp + i);
      }
      sc = dot * scale;
      if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
      vb = ((blk * (G / kvs) + g / kvs) * bs + (j % bs)) * v_rs;
    }
    const float m_new = fmaxf(m, wave_max(sc));  // finite: lane 0's key is visible
    const float p = j <= pos ? expf(sc - m_new) : 0.f;
    const float corr = expf(m - m_new);  // m = -inf on the wave's first tile -> 0
    l = l * corr + wave_sum(p);
    m = m_new;
    ps[lane] = p;
    vbase[lane] = vb;
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's LDS writes landed
    __builtin_amdgcn_wave_barrier();
    const int nk = min(WAVE, pos - j0 + 1);
    if (kVec) {
#pragma unroll
      for (int e = 0; e < N; ++e) acc[e] *= corr;
      if (v_on) {
        for (int jj = kg; jj < nk; jj += ngrp) {
          float x[N];
          Vec16<T>::load(v_cache + vbase[jj] + lv * N, x);
          const float pj = ps[jj];
#pragma unroll
          for (int e = 0; e < N; ++e) acc[e] += pj * x[e];
        }
      }
    } else {
#pragma unroll
      for (int c = 0; c < kMaxDvPerLane; ++c) {
        const int d = c * WAVE + lane;
        if (d < Dv) {
          float a = acc[c] * corr;
          for (int jj = 0; jj < nk; ++jj) a += ps[jj] * ldf(v_cache + vbase[jj] + d);
          acc[c] = a;
        }
      }
    }
    __builtin_amdgcn_wave_barrier();  // all lanes read ps/vbase before the next tile
  }
  // join: every wave publishes (max, sum) and its unnormalised partial output
  if (lane == 0) {
    stat[2 * wave] = m;
    stat[2 * wave + 1] = l;
  }
  if (kVec) {
    if (v_on) {
#pragma unroll
      for (int e = 0; e < N; ++e) red[kg * Dv + lv * N + e] = acc[e];
    }
  } else {
#pragma unroll
    for (int c = 0; c < kMaxDvPerLane; ++c) {
      const int d = c * WAVE + lane;
      if (d < Dv) red[d] = acc[c];
    }
  }
  __syncthreads();
  float mx = -INFINITY;
  for (int w = 0; w < kDecWaves; ++w) mx = fmaxf(mx, stat[2 * w]);
  float wsc[kDecWaves], lsum = 0.f;
  for (int w = 0; w < kDecWaves; ++w) {
    const float mw = stat[2 * w];
    wsc[w] = mw == -INFINITY ? 0.f : expf(mw - mx);  // a wave may have had no tile
    lsum += stat[2 * w + 1] * wsc[w];
  }
  if (sink != nullptr) lsum += expf(sink[h] - mx);
  const float inv = out_scale / lsum;
  for (int d = threadIdx.x; d < Dv; d += blockDim.x) {
    float a = 0.f;
    for (int w = 0; w < kDecWaves; ++w) {
      const float* rw = red_all + (size_t)w * ngrp * Dv;
      float part = 0.f;
      for (int gi = 0; gi < ngrp; ++gi) part += rw[gi * Dv + d];
      a += part * wsc[w];
    }
    stf(out + (size_t)t * out_stride + h * Dv + d, a * inv);
  }
}

typedef __attribute__((ext_vector_type(4))) short bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;


// Prompt portions on the matrix cores (bf16, key and value sizes multiples
// of 16). grid (n_seq * tiles_per_run, H), one wave per 16 consecutive
// queries of a run and one query head. Per 16-key tile:
//   S^T = K Q^T   (v_mfma_f32_16x16x16_bf16, K rows straight from the cache)
//   fp32 scale, cap, mask, running max / sum per query (a query is a lane
//   column, so its statistics never leave the lane quad 16 apart)
//   O^T += V^T P^T with P^T taken from S^T's accumulator layout as is.
// kMaxDSteps * 16 bounds the key size and kMaxDvTiles * 16 the value size
// (the query fragments and the output accumulators live in registers).
template <int kMaxDSteps, int kMaxDvTiles>
__global__ __launch_bounds__(WAVE) void masked_prefill_mfma_kernel(
    bf16raw* __restrict__ out, int64_t out_stride, const bf16raw* __restrict__ q,
    int64_t q_stride, const bf16raw* __restrict__ k_cache,
    const bf16raw* __restrict__ v_cache, const int* __restrict__ block_tables,
    int max_blocks, const int* __restrict__ start_loc,
    const int* __restrict__ positions, int tiles_per_run, float scale,
    float softcap, int chunk, int window, float out_scale, const float* __restrict__ sink, int64_t v_rs, int H, int G,
    int D, int Dv, int bs, int kvs) {
  const int s = blockIdx.x / tiles_per_run, tile = blockIdx.x % tiles_per_run;
  const int h = blockIdx.y, g = h / (H / G);
  const int s0 = start_loc[s], s1 = start_loc[s + 1];
  const int q0 = s0 + tile * 16;
  if (q0 >= s1) return;
  const int nq = min(16, s1 - q0);
  const int lane = threadIdx.x, col = lane & 15, grp = lane >> 4;
  const bool q_ok = col < nq;
  const int tq = q0 + min(col, nq - 1);
  const int pos_q = q_ok ? positions[tq] : -1;
  const int pos_min = positions[q0], pos_max = pos_min + nq - 1;
  auto lower = [&](int p) {
    int lo = 0;
    if (chunk > 0) lo = (p / chunk) * chunk;
    if (window > 0) lo = max(lo, p - window + 1);
    return lo;
  };
  const int lo_q = q_ok ? lower(pos_q) : 0;
  const int lo_tile = lower(pos_min);
  const int* bt = block_tables + (size_t)s * max_blocks;
  const int nks = D / 16, ndt = Dv / 16;
  bf16x4 qf[kMaxDSteps];
#pragma unroll
  for (int ks = 0; ks < kMaxDSteps; ++ks)
    if (ks < nks)
      qf[ks] = *(const bf16x4*)(q + (size_t)tq * q_stride + h * D + ks * 16 + grp * 4);
  f32x4 oacc[kMaxDvTiles];
#pragma unroll
  for (int dt = 0; dt < kMaxDvTiles; ++dt) oacc[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  for (int j0 = lo_tile; j0 <= pos_max; j0 += 16) {
    // K operand: row = key j0 + col, 4 consecutive dims per step
    const int jk = min(j0 + col, pos_max);
    const bf16raw* kp = k_cache + (((int64_t)bt[jk / bs] * G + g) * bs + jk % bs) * D + grp * 4;
    f32x4 sacc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < kMaxDSteps; ++ks)
      if (ks < nks)
        sacc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
            *(const bf16x4*)(kp + ks * 16), qf[ks], sacc, 0, 0, 0);
    // this lane: query `col`, keys j0 + grp * 4 + i
    float sc[4];
    bool vis[4];
    int64_t vrow[4];
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = j0 + grp * 4 + i;
      float x = sacc[i] * scale;
      if (softcap > 0.f) x = softcap * tanhf(x / softcap);
      vis[i] = j <= pos_q && j >= lo_q;
      sc[i] = vis[i] ? x : -INFINITY;
      mt = fmaxf(mt, sc[i]);
      const int jv = min(j, pos_max);
      vrow[i] = (((int64_t)bt[jv / bs] * (G / kvs) + g / kvs) * bs + jv % bs) * v_rs;
    }
    mt = fmaxf(mt, __shfl_xor(mt, 16, WAVE));
    mt = fmaxf(mt, __shfl_xor(mt, 32, WAVE));
    const float m_new = fmaxf(m, mt);
    const float corr = m_new == -INFINITY ? 1.f : expf(m - m_new);
    bf16x4 pb;
    float ps = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float p = vis[i] ? expf(sc[i] - m_new) : 0.f;
      ps += p;
      pb[i] = (short)f32_to_bf16(p);
    }
    l = l * corr + ps;
    m = m_new;
#pragma unroll
    for (int dt = 0; dt < kMaxDvTiles; ++dt) {
      if (dt < ndt) {
        bf16x4 vf;  // V^T operand: row = value dim dt*16 + col, keys grp*4 + i
#pragma unroll
        for (int i = 0; i < 4; ++i) vf[i] = (short)v_cache[vrow[i] + dt * 16 + col];
        f32x4 a = oacc[dt];
        a[0] *= corr; a[1] *= corr; a[2] *= corr; a[3] *= corr;
        oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pb, a, 0, 0, 0);
      }
    }
  }
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
  if (sink != nullptr) l += expf(sink[h] - m);
  if (q_ok) {
    const float inv = out_scale / l;
    bf16raw* op = out + (size_t)tq * out_stride + h * Dv + grp * 4;
#pragma unroll
    for (int dt = 0; dt < kMaxDvTiles; ++dt) {
      if (dt < ndt) {
        ushort4 o4;
        o4.x = f32_to_bf16(oacc[dt][0] * inv);
        o4.y = f32_to_bf16(oacc[dt][1] * inv);
        o4.z = f32_to_bf16(oacc[dt][2] * inv);
        o4.w = f32_to_bf16(oacc[dt][3] * inv);
        *(ushort4*)(op + dt * 16) = o4;
      }
    }
  }
}

constexpr float kLog2e = 1.4426950408889634f;

// two fp32 -> packed bf16 pair (round to nearest even), low half first
DEV_INLINE uint32_t cvt_pk_bf16(float a, float b) {
  uint32_t r;
  asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

constexpr int kKT = 32;      // keys staged per iteration
constexpr int kKPad = 8;     // padding of a staged key row (elements)
constexpr int kVPad = 4;     // padding of a staged transposed value row

// Prompt portions on the matrix cores with the key / value tiles shared
// through LDS. A block of HW * QW waves covers QW * 16 consecutive queries of
// a run for HW query heads of one key/value head (for latent attention all
// heads share the one cached row, for grouped heads the group does). Per
// iteration the block stages 32 keys: K rows as they lie in the cache
// (16-byte loads, padded rows) and V transposed ([value dim][key]), so both
// MFMA operands are 8-byte LDS reads. Two LDS buffers: the next tile is loaded
// into registers before the products of the current one and written to the
// other buffer after them, one barrier per iteration. Masking and the fp32
// softmax statistics are those of masked_prefill_mfma_kernel; P V contracts
// all 32 keys of a tile in one v_mfma_f32_16x16x32_bf16 per 16 value dims (a
// lane's eight contraction slots are keys grp*4 + 0..3 and 16 + grp*4 + 0..3,
// for P and V alike), and so does K Q^T over 32 key dims when the key size
// allows (kWideQK).
typedef __attribute__((ext_vector_type(8))) short bf16x8;

template <int kMaxDSteps, int kMaxDvTiles, bool kWideQK>
__global__ __launch_bounds__(512) void masked_prefill_mfma_shared_kernel(
    bf16raw* __restrict__ out, int64_t out_stride, const bf16raw* __restrict__ q,
    int64_t q_stride, const bf16raw* __restrict__ k_cache,
    const bf16raw* __restrict__ v_cache, const int* __restrict__ block_tables,
    int max_blocks, const int* __restrict__ start_loc,
    const int* __restrict__ positions, int tiles_per_run, float scale,
    float softcap, int chunk, int window, float out_scale, const float* __restrict__ sink, int64_t v_rs, int H, int G,
    int D, int Dv, int bs, int HW, int QW, int kvs) {
  extern __shared__ __attribute__((aligned(16))) bf16raw lds[];
  constexpr int kKVec = kKT * kMaxDSteps * 16 / 8 / 256;   // per thread, 256 threads
  constexpr int kVVec = kKT * kMaxDvTiles * 16 / 8 / 256;
  const int nthr = blockDim.x;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int col = lane & 15, grp = lane >> 4;
  const int hw = wave % HW, qw = wave / HW;
  const int s = blockIdx.x / tiles_per_run, tile = blockIdx.x % tiles_per_run;
  const int g = blockIdx.y, rep = H / G;
  const int hz = blockIdx.z * HW + hw;
  const int s0 = start_loc[s], s1 = start_loc[s + 1];
  const int bq0 = s0 + tile * QW * 16;
  if (bq0 >= s1) return;  // the whole block: no barrier is skipped
  const int bnq = min(QW * 16, s1 - bq0);
  const int bpos_min = positions[bq0], bpos_max = bpos_min + bnq - 1;
  auto lower = [&](int p) {
    int lo = 0;
    if (chunk > 0) lo = (p / chunk) * chunk;
    if (window > 0) lo = max(lo, p - window + 1);
    return lo;
  };
  const int q0 = bq0 + qw * 16;
  const bool wave_on = q0 < s1 && hz < rep;
  const int nq = wave_on ? min(16, s1 - q0) : 0;
  const int h = g * rep + min(hz, rep - 1);
  const bool q_ok = wave_on && col < nq;
  const int tq = wave_on ? q0 + min(col, nq - 1) : bq0;
  const int pos_q = q_ok ? positions[tq] : -1;
  const int wpos_min = wave_on ? positions[q0] : 0, wpos_max = wpos_min + nq - 1;
  const int lo_q = q_ok ? lower(pos_q) : 0;
  const int wlo = lower(wpos_min);
  const int blo = lower(bpos_min);
  const int* bt = block_tables + (size_t)s * max_blocks;
  const int nks = D / 16, ndt = Dv / 16;
  const int krow = D + kKPad, vrow = kKT + kVPad;  // LDS row lengths (elements)
  const int buf_elems = kKT * krow + Dv * vrow;
  const int kcpr = D / 8, vcpr = Dv / 8;  // 16-byte chunks per cached row

  // query fragments: [ks] 4 dims at ks*16 + grp*4, or (wide) [kc] 8 dims at
  // kc*32 + grp*8
  bf16x4 qf[kWideQK ? 1 : kMaxDSteps];
  bf16x8 qf8[kWideQK ? kMaxDSteps / 2 : 1];
  const bf16raw* qrow = q + (size_t)tq * q_stride + h * D;
  if (kWideQK) {
#pragma unroll
    for (int kc = 0; kc < kMaxDSteps / 2; ++kc)
      if (kc < D / 32) {
        const bf16x4 a = *(const bf16x4*)(qrow + kc * 32 + grp * 8);
        const bf16x4 b = *(const bf16x4*)(qrow + kc * 32 + grp * 8 + 4);
        qf8[kc] = (bf16x8){a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
      }
  } else {
#pragma unroll
    for (int ks = 0; ks < kMaxDSteps; ++ks)
      if (ks < nks) qf[ks] = *(const bf16x4*)(qrow + ks * 16 + grp * 4);
  }
  f32x4 oacc[kMaxDvTiles];
#pragma unroll
  for (int dt = 0; dt < kMaxDvTiles; ++dt) oacc[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  uint4 kreg[kKVec], vreg[kVVec];
  // K: consecutive threads take consecutive chunks of a row (coalesced);
  // V: consecutive threads take consecutive keys at one chunk, so that the
  // transposed 2-byte LDS writes of a wave fall into consecutive addresses
  auto load_tile = [&](int j0) {
#pragma unroll
    for (int i = 0; i < kKVec; ++i) {
      const int v = i * nthr + threadIdx.x;
      const int row = v / kcpr, c = v % kcpr;
      if (row < kKT) {
        const int j = min(j0 + row, bpos_max);
        kreg[i] = *(const uint4*)(k_cache +
            (((int64_t)bt[j / bs] * G + g) * bs + j % bs) * D + c * 8);
      }
    }
#pragma unroll
    for (int i = 0; i < kVVec; ++i) {
      const int v = i * nthr + threadIdx.x;
      const int row = v % kKT, c = v / kKT;
      if (c < vcpr) {
        const int j = min(j0 + row, bpos_max);
        vreg[i] = *(const uint4*)(v_cache +
            (((int64_t)bt[j / bs] * (G / kvs) + g / kvs) * bs + j % bs) * v_rs + c * 8);
      }
    }
  };
  auto store_tile = [&](int buf) {
    bf16raw* ks_ = lds + buf * buf_elems;
    bf16raw* vs_ = ks_ + kKT * krow;
#pragma unroll
    for (int i = 0; i < kKVec; ++i) {
      const int v = i * nthr + threadIdx.x;
      const int row = v / kcpr, c = v % kcpr;
      if (row < kKT) *(uint4*)(ks_ + row * krow + c * 8) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < kVVec; ++i) {
      const int v = i * nthr + threadIdx.x;
      const int row = v % kKT, c = v / kKT;
      if (c < vcpr) {
        const uint32_t wv[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          vs_[(c * 8 + 2 * e) * vrow + row] = (bf16raw)(wv[e] & 0xffffu);
          vs_[(c * 8 + 2 * e + 1) * vrow + row] = (bf16raw)(wv[e] >> 16);
        }
      }
    }
  };

  load_tile(blo);
  store_tile(0);
  __syncthreads();
  int buf = 0;
  for (int j0 = blo; j0 <= bpos_max; j0 += kKT, buf ^= 1) {
    const bool more = j0 + kKT <= bpos_max;
    if (more) load_tile(j0 + kKT);
    const bf16raw* ks_ = lds + buf * buf_elems;
    const bf16raw* vs_ = ks_ + kKT * krow;
    // wave-uniform: something of this tile is visible to the wave's queries
    if (wave_on && j0 <= wpos_max && j0 + kKT - 1 >= wlo) {
      f32x4 sacc[2];
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        sacc[sub] = (f32x4){0.f, 0.f, 0.f, 0.f};
        const bf16raw* kp = ks_ + (sub * 16 + col) * krow;
        if (kWideQK) {
#pragma unroll
          for (int kc = 0; kc < kMaxDSteps / 2; ++kc)
            if (kc < D / 32)
              sacc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  *(const bf16x8*)(kp + kc * 32 + grp * 8), qf8[kc], sacc[sub], 0, 0, 0);
        } else {
#pragma unroll
          for (int ks = 0; ks < kMaxDSteps; ++ks)
            if (ks < nks)
              sacc[sub] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
                  *(const bf16x4*)(kp + ks * 16 + grp * 4), qf[ks], sacc[sub], 0, 0, 0);
        }
      }
      // this lane: query `col`, keys j0 + sub * 16 + grp * 4 + i. Scores and
      // the running max are kept in the base-2 domain (score * log2 e), so
      // every exponential is one v_exp_f32.
      float sc[8];
      float mt = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = j0 + (e >> 2) * 16 + grp * 4 + (e & 3);
        float x = sacc[e >> 2][e & 3] * scale;
        if (softcap > 0.f) x = softcap * tanhf(x / softcap);
        const bool vis = j <= pos_q && j >= lo_q;
        sc[e] = vis ? x * kLog2e : -INFINITY;
        mt = fmaxf(mt, sc[e]);
      }
      mt = fmaxf(mt, __shfl_xor(mt, 16, WAVE));
      mt = fmaxf(mt, __shfl_xor(mt, 32, WAVE));
      const float m_new = fmaxf(m, mt);
      // no visible key so far: keep everything at zero without forming inf - inf
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float corr = __builtin_amdgcn_exp2f(m - m_use);
      float pv[8];
      float ps = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        pv[e] = __builtin_amdgcn_exp2f(sc[e] - m_use);
        ps += pv[e];
      }
      union { bf16x8 v; uint32_t u[4]; } pk;
#pragma unroll
      for (int e = 0; e < 4; ++e) pk.u[e] = cvt_pk_bf16(pv[2 * e], pv[2 * e + 1]);
      const bf16x8 pb = pk.v;
      l = l * corr + ps;
      m = m_new;
      const bf16raw* vp = vs_ + col * vrow + grp * 4;
#pragma unroll
      for (int dt = 0; dt < kMaxDvTiles; ++dt) {
        if (dt < ndt) {
          const bf16x4 v0 = *(const bf16x4*)(vp + dt * 16 * vrow);
          const bf16x4 v1 = *(const bf16x4*)(vp + dt * 16 * vrow + 16);
          const bf16x8 vf = (bf16x8){v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
          f32x4 a = oacc[dt];
          a[0] *= corr; a[1] *= corr; a[2] *= corr; a[3] *= corr;
          oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb, a, 0, 0, 0);
        }
      }
    }
    if (more) store_tile(buf ^ 1);
    __syncthreads();
  }
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
  if (sink != nullptr) l += __builtin_amdgcn_exp2f(sink[h] * kLog2e - m);
  if (q_ok) {
    const float inv = out_scale / l;
    bf16raw* op = out + (size_t)tq * out_stride + h * Dv + grp * 4;
#pragma unroll
    for (int dt = 0; dt < kMaxDvTiles; ++dt) {
      if (dt < ndt) {
        ushort4 o4;
        o4.x = f32_to_bf16(oacc[dt][0] * inv);
        o4.y = f32_to_bf16(oacc[dt][1] * inv);
        o4.z = f32_to_bf16(oacc[dt][2] * inv);
        o4.w = f32_to_bf16(oacc[dt][3] * inv);
        *(ushort4*)(op + dt * 16) = o4;
      }
    }
  }
}

constexpr int kDW = 4;  // waves of a decode block; each takes every fourth key tile

// Single decode tokens on the matrix cores, bf16. grid (T, G, ceil(rep / 16)):
// the 16 rows of an MFMA tile are the query heads that share one key/value
// head (all heads of a latent layer, the group of a grouped layer), so a key
// or value row is loaded once for all of them. The four waves walk disjoint
// 32-key tiles: K rows come straight from the cache as A operands, the V tile
// is transposed through a wave-private LDS region, statistics are fp32 in the
// base-2 domain, and the waves' partial results are joined through LDS.
template <int kMaxDSteps, int kMaxDvTiles>
__global__ __launch_bounds__(kDW * WAVE) void masked_decode_mfma_kernel(
    bf16raw* __restrict__ out, int64_t out_stride, const bf16raw* __restrict__ q,
    int64_t q_stride, const bf16raw* __restrict__ k_cache,
    const bf16raw* __restrict__ v_cache, const int* __restrict__ block_tables,
    int max_blocks, const int* __restrict__ token_seq,
    const int* __restrict__ positions, float scale, float softcap, int chunk,
    int window, float out_scale, const float* __restrict__ sink, int64_t v_rs, int H, int G, int D, int Dv, int bs,
    int n_split, float* __restrict__ part_o, float* __restrict__ part_ml, int kvs) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int col = lane & 15, grp = lane >> 4;
  const int t = blockIdx.x, g = blockIdx.y, rep = H / G;
  const int zt = blockIdx.z / n_split, sp = blockIdx.z % n_split;
  const int h0 = g * rep + zt * 16;
  const int nh = min(16, (g + 1) * rep - h0);
  const int pos = positions[t];
  const int* bt = block_tables + (size_t)token_seq[t] * max_blocks;
  int lo = 0;
  if (chunk > 0) lo = (pos / chunk) * chunk;
  if (window > 0) lo = max(lo, pos - window + 1);
  const int nks = D / 16, ndt = Dv / 16;
  constexpr int vrow = kKT + kVPad;
  bf16raw* vt = (bf16raw*)smem + (size_t)wave * Dv * vrow;
  bf16x4 qf[kMaxDSteps];
#pragma unroll
  for (int ks = 0; ks < kMaxDSteps; ++ks)
    if (ks < nks)
      qf[ks] = col < nh ? *(const bf16x4*)(q + (size_t)t * q_stride + (h0 + col) * D +
                                           ks * 16 + grp * 4)
                        : (bf16x4){0, 0, 0, 0};
  f32x4 oacc[kMaxDvTiles];
#pragma unroll
  for (int dt = 0; dt < kMaxDvTiles; ++dt) oacc[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  // the visible keys in 32-key tiles, dealt to the splits in contiguous shares
  const int n_tiles = (pos - lo) / kKT + 1;
  const int per_split = (n_tiles + n_split - 1) / n_split;
  const int tile_end = min(n_tiles, (sp + 1) * per_split);
  for (int tile = sp * per_split + wave; tile < tile_end; tile += kDW) {
    const int j0 = lo + tile * kKT;
    // V tile, transposed: lane takes key (v % 32), 16-byte chunk (v / 32)
    for (int v = lane; v < kKT * (Dv / 8); v += WAVE) {
      const int row = v % kKT, c = v / kKT;
      const int j = min(j0 + row, pos);
      const uint4 x = *(const uint4*)(v_cache +
          (((int64_t)bt[j / bs] * (G / kvs) + g / kvs) * bs + j % bs) * v_rs + c * 8);
      const uint32_t wv[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        vt[(c * 8 + 2 * e) * vrow + row] = (bf16raw)(wv[e] & 0xffffu);
        vt[(c * 8 + 2 * e + 1) * vrow + row] = (bf16raw)(wv[e] >> 16);
      }
    }
    f32x4 sacc[2];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      sacc[sub] = (f32x4){0.f, 0.f, 0.f, 0.f};
      const int jk = min(j0 + sub * 16 + col, pos);
      const bf16raw* kp =
          k_cache + (((int64_t)bt[jk / bs] * G + g) * bs + jk % bs) * D + grp * 4;
#pragma unroll
      for (int ks = 0; ks < kMaxDSteps; ++ks)
        if (ks < nks)
          sacc[sub] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
              *(const bf16x4*)(kp + ks * 16), qf[ks], sacc[sub], 0, 0, 0);
    }
    // this lane: head `col`, keys j0 + sub * 16 + grp * 4 + i
    float sc[8];
    float mt = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = j0 + (e >> 2) * 16 + grp * 4 + (e & 3);
      float x = sacc[e >> 2][e & 3] * scale;
      if (softcap > 0.f) x = softcap * tanhf(x / softcap);
      sc[e] = j <= pos ? x * kLog2e : -INFINITY;  // j >= lo holds for every tile
      mt = fmaxf(mt, sc[e]);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 16, WAVE));
    mt = fmaxf(mt, __shfl_xor(mt, 32, WAVE));
    const float m_new = fmaxf(m, mt);  // finite: the tile's first key is visible
    const float corr = __builtin_amdgcn_exp2f(m - m_new);
    float pv[8];
    float ps = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      pv[e] = __builtin_amdgcn_exp2f(sc[e] - m_new);
      ps += pv[e];
    }
    union { bf16x8 v; uint32_t u[4]; } pk;
#pragma unroll
    for (int e = 0; e < 4; ++e) pk.u[e] = cvt_pk_bf16(pv[2 * e], pv[2 * e + 1]);
    l = l * corr + ps;
    m = m_new;
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's LDS writes landed
    __builtin_amdgcn_wave_barrier();
    const bf16raw* vp = vt + col * vrow + grp * 4;
#pragma unroll
    for (int dt = 0; dt < kMaxDvTiles; ++dt) {
      if (dt < ndt) {
        const bf16x4 v0 = *(const bf16x4*)(vp + dt * 16 * vrow);
        const bf16x4 v1 = *(const bf16x4*)(vp + dt * 16 * vrow + 16);
        const bf16x8 vf = (bf16x8){v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
        f32x4 a = oacc[dt];
        a[0] *= corr; a[1] *= corr; a[2] *= corr; a[3] *= corr;
        oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pk.v, a, 0, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();  // all lanes read the tile before it is rewritten
  }
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
  __syncthreads();  // the staging regions are reused for the join
  float* cm = (float*)smem;            // [waves][16] running max (base 2)
  float* cl = cm + kDW * 16;           // [waves][16] sums
  float* co = cl + kDW * 16;           // [waves][16][Dv] unnormalised outputs
  if (grp == 0) {
    cm[wave * 16 + col] = m;
    cl[wave * 16 + col] = l;
  }
#pragma unroll
  for (int dt = 0; dt < kMaxDvTiles; ++dt)
    if (dt < ndt) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        co[((size_t)wave * 16 + col) * Dv + dt * 16 + grp * 4 + i] = oacc[dt][i];
    }
  __syncthreads();
  for (int idx = threadIdx.x; idx < nh * Dv; idx += blockDim.x) {
    const int hh = idx / Dv, d = idx % Dv;
    float mx = -INFINITY;
    for (int w = 0; w < kDW; ++w) mx = fmaxf(mx, cm[w * 16 + hh]);
    float lsum = 0.f, a = 0.f;
    for (int w = 0; w < kDW; ++w) {
      const float mw = cm[w * 16 + hh];
      const float wsc = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - mx);
      lsum += cl[w * 16 + hh] * wsc;
      a += co[((size_t)w * 16 + hh) * Dv + d] * wsc;
    }
    if (n_split == 1) {
      if (sink != nullptr) lsum += __builtin_amdgcn_exp2f(sink[h0 + hh] * kLog2e - mx);
      stf(out + (size_t)t * out_stride + (h0 + hh) * Dv + d, a * out_scale / lsum);
    } else {
      // partial result of this split: [t][head][split] -> (max, sum), values
      const size_t row = ((size_t)t * H + h0 + hh) * n_split + sp;
      part_o[row * Dv + d] = a;
      if (d == 0) {
        part_ml[row * 2] = mx;
        part_ml[row * 2 + 1] = lsum;
      }
    }
  }
}

// Join of the key splits of masked_decode_mfma_kernel: grid (T, H).
__global__ void decode_split_join_kernel(bf16raw* __restrict__ out, int64_t out_stride,
                                         const float* __restrict__ part_o,
                                         const float* __restrict__ part_ml, int H,
                                         int Dv, int n_split, float out_scale,
                                         const float* __restrict__ sink) {
  const int t = blockIdx.x, h = blockIdx.y;
  const size_t row0 = ((size_t)t * H + h) * n_split;
  float mx = -INFINITY;
  for (int s = 0; s < n_split; ++s) mx = fmaxf(mx, part_ml[(row0 + s) * 2]);
  for (int d = threadIdx.x; d < Dv; d += blockDim.x) {
    float lsum = 0.f, a = 0.f;
    for (int s = 0; s < n_split; ++s) {
      const float ms = part_ml[(row0 + s) * 2];
      if (ms == -INFINITY) continue;  // a split without keys wrote nothing usable
      const float w = __builtin_amdgcn_exp2f(ms - mx);
      lsum += part_ml[(row0 + s) * 2 + 1] * w;
      a += part_o[(row0 + s) * Dv + d] * w;
    }
    if (sink != nullptr) lsum += __builtin_amdgcn_exp2f(sink[h] * kLog2e - mx);
    stf(out + (size_t)t * out_stride + h * Dv + d, a * out_scale / lsum);
  }
}

}  // namespace

static bool dense_heads3(const torch::Tensor& t) {
  // heads are addressed as row + h * size(2): a single head's stride is free
  return t.dim() == 3 && (t.size(2) == 1 || t.stride(2) == 1) &&
         (t.size(1) == 1 || t.stride(1) == t.size(2));
}

void rope_pairs_and_cache(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                          torch::Tensor positions, torch::Tensor inv_freq,
                          torch::Tensor k_cache, torch::Tensor v_cache,
                          torch::Tensor slot_mapping) {
  check_i32(positions, "positions");
  check_f32(inv_freq, "inv_freq");
  TORCH_CHECK(dense_heads3(q) && dense_heads3(k) && dense_heads3(v));
  TORCH_CHECK(slot_mapping.scalar_type() == torch::kInt64 &&
              slot_mapping.is_contiguous());
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k.size(1), Dv = v.size(2), half = inv_freq.numel();
  TORCH_CHECK(D % 2 == 0 && 2 * half <= D, "key size must be even and hold the rotated dims");
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && k.size(2) == D && v.size(1) == G);
  TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4);
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D && v_cache.size(1) == G &&
              v_cache.size(3) == Dv && v_cache.size(2) == k_cache.size(2) &&
              v_cache.size(0) == k_cache.size(0));
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type());
  if (T == 0) return;
  SEQ_DISPATCH_ACT(q, {
    hipLaunchKernelGGL((rope_pairs_cache_kernel<act_t>), dim3(T), dim3(256), 0,
                       SEQ_STREAM(), (act_t*)q.data_ptr(), q.stride(0),
                       (const act_t*)k.data_ptr(), k.stride(0),
                       (const act_t*)v.data_ptr(), v.stride(0),
                       (const int*)positions.data_ptr(),
                       (const float*)inv_freq.data_ptr(), half,
                       (act_t*)k_cache.data_ptr(), (act_t*)v_cache.data_ptr(),
                       (const int64_t*)slot_mapping.data_ptr(), H, G, D, Dv,
                       (int)k_cache.size(2));
  });
  SEQ_CHECK_LAUNCH();
}

void qknorm_rope_half_and_cache(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                                c10::optional<torch::Tensor> q_weight,
                                c10::optional<torch::Tensor> k_weight, double eps,
                                torch::Tensor positions, torch::Tensor inv_freq,
                                torch::Tensor k_cache, torch::Tensor v_cache,
                                torch::Tensor slot_mapping) {
  check_i32(positions, "positions");
  check_f32(inv_freq, "inv_freq");
  TORCH_CHECK(dense_heads3(q) && dense_heads3(k) && dense_heads3(v));
  TORCH_CHECK(slot_mapping.scalar_type() == torch::kInt64 &&
              slot_mapping.is_contiguous());
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k.size(1), Dv = v.size(2), half = inv_freq.numel();
  TORCH_CHECK(2 * half <= D, "rotated dims exceed the key size");
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && k.size(2) == D && v.size(1) == G);
  TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
  TORCH_CHECK(q_weight.has_value() == k_weight.has_value());
  if (q_weight.has_value()) {
    check_f32(*q_weight, "q_weight");
    check_f32(*k_weight, "k_weight");
    TORCH_CHECK(q_weight->numel() == (int64_t)H * D && k_weight->numel() == (int64_t)G * D);
  }
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4);
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D && v_cache.size(1) == G &&
              v_cache.size(3) == Dv && v_cache.size(2) == k_cache.size(2) &&
              v_cache.size(0) == k_cache.size(0));
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type());
  if (T == 0) return;
  SEQ_DISPATCH_ACT(q, {
    hipLaunchKernelGGL((qknorm_rope_half_cache_kernel<act_t>), dim3(T), dim3(256), 0,
                       SEQ_STREAM(), (act_t*)q.data_ptr(), q.stride(0),
                       (const act_t*)k.data_ptr(), k.stride(0),
                       (const act_t*)v.data_ptr(), v.stride(0),
                       q_weight.has_value() ? (const float*)q_weight->data_ptr() : nullptr,
                       k_weight.has_value() ? (const float*)k_weight->data_ptr() : nullptr,
                       (float)eps, (const int*)positions.data_ptr(),
                       (const float*)inv_freq.data_ptr(), half,
                       (act_t*)k_cache.data_ptr(), (act_t*)v_cache.data_ptr(),
                       (const int64_t*)slot_mapping.data_ptr(), H, G, D, Dv,
                       (int)k_cache.size(2));
  });
  SEQ_CHECK_LAUNCH();
}

void masked_paged_attention(torch::Tensor out, torch::Tensor q,
                            torch::Tensor k_cache, torch::Tensor v_cache,
                            torch::Tensor block_tables, torch::Tensor start_loc,
                            torch::Tensor token_seq, torch::Tensor positions,
                            int64_t max_len, double scale, double softcap,
                            int64_t chunk, int64_t window, double out_scale,
                            c10::optional<torch::Tensor> sink_scores) {
  check_i32(start_loc, "start_loc");
  check_i32(block_tables, "block_tables");
  check_i32(token_seq, "token_seq");
  check_i32(positions, "positions");
  TORCH_CHECK(dense_heads3(q) && dense_heads3(out));
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  TORCH_CHECK(k_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4);
  const int G = k_cache.size(1), bs = k_cache.size(2), Dv = v_cache.size(3);
  // the value cache may have fewer heads than the key cache: kvs key heads
  // (score maps over the same values) share one value head
  const int Gv = v_cache.size(1);
  TORCH_CHECK(k_cache.size(3) == D && Gv > 0 && G % Gv == 0 && v_cache.size(2) == bs);
  const int kvs = G / Gv;
  // value rows may be the leading columns of wider rows (of the key rows,
  // when a layer caches one row per token that serves as both)
  const int64_t v_rs = v_cache.stride(2);
  TORCH_CHECK(v_cache.is_cuda() && (Dv == 1 || v_cache.stride(3) == 1) && v_rs >= Dv &&
              v_cache.stride(1) == (int64_t)bs * v_rs &&
              v_cache.stride(0) == (int64_t)Gv * bs * v_rs,
              "value cache rows must be evenly spaced");
  const float* sink = nullptr;
  if (sink_scores.has_value()) {
    check_f32(*sink_scores, "sink_scores");
    TORCH_CHECK(sink_scores->numel() == H, "one sink score per head");
    sink = (const float*)sink_scores->data_ptr();
  }
  TORCH_CHECK(G > 0 && H % G == 0 && H <= 65535);
  TORCH_CHECK(out.size(0) == T && out.size(1) == H && out.size(2) == Dv);
  TORCH_CHECK(Dv <= kMaxDvPerLane * WAVE, "value size too large");
  TORCH_CHECK(block_tables.dim() == 2 && token_seq.numel() == T &&
              positions.numel() == T);
  TORCH_CHECK(k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type() &&
              out.scalar_type() == q.scalar_type());
  if (T == 0) return;
  const int n_seq = start_loc.numel() - 1;
  TORCH_CHECK(block_tables.size(0) >= n_seq);
  auto al8 = [](const torch::Tensor& t) {
    return ((size_t)t.data_ptr()) % 8 == 0 && t.stride(0) % 4 == 0;
  };
  if (q.scalar_type() == torch::kBFloat16 && max_len > 1 && D % 16 == 0 &&
      Dv % 16 == 0 && D <= 512 && Dv <= 512 && al8(q) && al8(out) && v_rs % 8 == 0) {
    // prompt portions: matrix-core kernel over 16-query tiles of every run
    const int tiles = (int)((max_len + 15) / 16);
    auto launch = [&](auto kern) {
      hipLaunchKernelGGL(kern, dim3(n_seq * tiles, H), dim3(WAVE), 0, SEQ_STREAM(),
                         (bf16raw*)out.data_ptr(), out.stride(0),
                         (const bf16raw*)q.data_ptr(), q.stride(0),
                         (const bf16raw*)k_cache.data_ptr(),
                         (const bf16raw*)v_cache.data_ptr(),
                         (const int*)block_tables.data_ptr(),
                         (int)block_tables.size(1), (const int*)start_loc.data_ptr(),
                         (const int*)positions.data_ptr(), tiles, (float)scale,
                         (float)softcap, (int)chunk, (int)window, (float)out_scale,
                         sink, v_rs, H, G, D, Dv, bs, kvs);
    };
    const size_t lds_shared =
        (size_t)2 * (kKT * (D + kKPad) + Dv * (kKT + kVPad)) * sizeof(bf16raw);
    const bool cache_al16 = ((size_t)k_cache.data_ptr()) % 16 == 0 &&
                            ((size_t)v_cache.data_ptr()) % 16 == 0;
    if (D <= 256 && Dv <= 256 && lds_shared <= 64 * 1024 && cache_al16) {
      // tiles shared through LDS by up to 8 waves: heads of a group first,
      // then neighbouring query tiles
      const int rep = H / G;
      int HW = 1;
      while (HW * 2 <= rep && HW < 8) HW *= 2;
      const int WPB = HW < 4 ? 4 : HW;
      const int QW = WPB / HW;
      const int btiles = (int)((max_len + QW * 16 - 1) / (QW * 16));
      const int zb = (rep + HW - 1) / HW;
      TORCH_CHECK(G <= 65535 && zb <= 65535);
      auto launch_shared = [&](auto kern) {
      hipLaunchKernelGGL(kern,
                         dim3(n_seq * btiles, G, zb), dim3(WPB * WAVE), lds_shared,
                         SEQ_STREAM(), (bf16raw*)out.data_ptr(), out.stride(0),
                         (const bf16raw*)q.data_ptr(), q.stride(0),
                         (const bf16raw*)k_cache.data_ptr(),
                         (const bf16raw*)v_cache.data_ptr(),
                         (const int*)block_tables.data_ptr(),
                         (int)block_tables.size(1), (const int*)start_loc.data_ptr(),
                         (const int*)positions.data_ptr(), btiles, (float)scale,
                         (float)softcap, (int)chunk, (int)window, (float)out_scale,
                         sink, v_rs, H, G, D, Dv, bs, HW, QW, kvs);
      };
      // key sizes above 128 (a latent with a rotated part behind it) keep
      // twice as many query fragments in registers
      if (D <= 128) {
        if (D % 32 == 0) launch_shared(masked_prefill_mfma_shared_kernel<8, 16, true>);
        else launch_shared(masked_prefill_mfma_shared_kernel<8, 16, false>);
      } else {
        if (D % 32 == 0) launch_shared(masked_prefill_mfma_shared_kernel<16, 16, true>);
        else launch_shared(masked_prefill_mfma_shared_kernel<16, 16, false>);
      }
    } else if (D <= 128 && Dv <= 256) {
      launch(masked_prefill_mfma_kernel<8, 16>);
    } else {
      launch(masked_prefill_mfma_kernel<32, 32>);
    }
    SEQ_CHECK_LAUNCH();
    return;
  }
  // worth it when several heads share a key row (measured at 64 sequences of
  // 1536 tokens: 16 heads on one latent 60 -> 28 us per call; groups of 4 with
  // 128-wide keys 89 -> 65 us, with two 64-wide score maps per value head
  // 132 -> 93 us)
  if (q.scalar_type() == torch::kBFloat16 && max_len == 1 && H / G >= 4 && D % 16 == 0 &&
      Dv % 16 == 0 && D <= 256 && Dv <= 128 && al8(q) && v_rs % 8 == 0 &&
      ((size_t)k_cache.data_ptr()) % 16 == 0 && ((size_t)v_cache.data_ptr()) % 16 == 0) {
    // decode tokens: the heads of a key/value group are the rows of a tile
    const int rep = H / G, zb = (rep + 15) / 16;
    const size_t stage = (size_t)kDW * Dv * (kKT + kVPad) * sizeof(bf16raw);
    const size_t join = (size_t)kDW * (32 + 16 * Dv) * sizeof(float);
    // split the keys over blocks so that a wave walks about two tiles at the
    // longest context the block tables can describe; splits beyond a
    // sequence's keys exit at once
    const int64_t cap = (int64_t)block_tables.size(1) * bs;
    int n_split = (int)std::min<int64_t>(16, std::max<int64_t>(1, (cap + 255) / 256));
    // past about eight blocks a CU more splits only add joins (64 sequences of
    // 1536 tokens on 8 key heads: 144 us with 16 splits, 91 us with 4)
    while (n_split > 1 && (int64_t)T * G * zb * n_split > 2048) n_split /= 2;
    TORCH_CHECK(G <= 65535 && (int64_t)zb * n_split <= 65535);
    torch::Tensor part_o, part_ml;
    if (n_split > 1) {
      auto f32 = torch::TensorOptions().dtype(torch::kFloat32).device(q.device());
      part_o = torch::empty({(int64_t)T * H * n_split, Dv}, f32);
      part_ml = torch::empty({(int64_t)T * H * n_split, 2}, f32);
    }
    auto decode_kern = D <= 128 ? masked_decode_mfma_kernel<8, 8>
                                : masked_decode_mfma_kernel<16, 8>;
    hipLaunchKernelGGL(decode_kern, dim3(T, G, zb * n_split),
                       dim3(kDW * WAVE), stage > join ? stage : join, SEQ_STREAM(),
                       (bf16raw*)out.data_ptr(), out.stride(0),
                       (const bf16raw*)q.data_ptr(), q.stride(0),
                       (const bf16raw*)k_cache.data_ptr(),
                       (const bf16raw*)v_cache.data_ptr(),
                       (const int*)block_tables.data_ptr(), (int)block_tables.size(1),
                       (const int*)token_seq.data_ptr(), (const int*)positions.data_ptr(),
                       (float)scale, (float)softcap, (int)chunk, (int)window,
                       (float)out_scale, sink, v_rs, H, G, D, Dv, bs, n_split,
                       n_split > 1 ? (float*)part_o.data_ptr() : nullptr,
                       n_split > 1 ? (float*)part_ml.data_ptr() : nullptr, kvs);
    if (n_split > 1) {
      SEQ_CHECK_LAUNCH();
      hipLaunchKernelGGL(decode_split_join_kernel, dim3(T, H), dim3(64), 0, SEQ_STREAM(),
                         (bf16raw*)out.data_ptr(), out.stride(0),
                         (const float*)part_o.data_ptr(),
                         (const float*)part_ml.data_ptr(), H, (int)Dv, n_split,
                         (float)out_scale, sink);
    }
    SEQ_CHECK_LAUNCH();
    return;
  }
  SEQ_DISPATCH_ACT(q, {
    constexpr int N = Vec16<act_t>::N;
    // 16-byte row loads need whole vectors per key / value row and at most
    // one wave of lanes per value row
    const bool vec = D % N == 0 && Dv % N == 0 && Dv / N <= WAVE && Dv >= N &&
                     N <= kMaxDvPerLane && v_rs % N == 0 &&
                     ((size_t)v_cache.data_ptr()) % 16 == 0;
    const int ngrp = vec ? WAVE / (Dv / N) : 1;
    const size_t lds = (size_t)(3 * WAVE * kDecWaves + 2 * kDecWaves +
                                ((D + 3) & ~3) + kDecWaves * ngrp * Dv) * 4;
    TORCH_CHECK(lds <= 64 * 1024, "attention scratch exceeds LDS");
    auto launch = [&](auto kern) {
      hipLaunchKernelGGL(kern, dim3(T, H), dim3(kDecWaves * WAVE), lds, SEQ_STREAM(),
                         (act_t*)out.data_ptr(), out.stride(0),
                         (const act_t*)q.data_ptr(), q.stride(0),
                         (const act_t*)k_cache.data_ptr(),
                         (const act_t*)v_cache.data_ptr(),
                         (const int*)block_tables.data_ptr(),
                         (int)block_tables.size(1), (const int*)token_seq.data_ptr(),
                         (const int*)positions.data_ptr(), (float)scale,
                         (float)softcap, (int)chunk, (int)window, (float)out_scale,
                         sink, v_rs, H, G, D, Dv, bs, kvs);
    };
    if (vec) launch(masked_paged_attention_kernel<act_t, true>);
    else launch(masked_paged_attention_kernel<act_t, false>);
  });
  SEQ_CHECK_LAUNCH();
}
