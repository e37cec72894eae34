// Kernels of the heterogeneous decoder stacks (models/mixers.py, ops/seqmix.py): layer norm with token shift,
// post-norm residual update, unit-RMS q/k + cache write, latent-attention cache write with pair rotation,
// attention over token-major pages (sliding window, distance penalty, two-part scores), the decayed
// linear-attention scan over per-sequence state, and the element-wise pieces around them.
//
// Arithmetic: the residual stream, norm statistics, scores, softmax weights, rotation angles and the recurrent
// state are fp32 (angles: double until reduced); activations are the template type A = float or bf16 (uint16_t
// bit pattern).  Small parameters (norm weights / biases, per-head constants) are fp32 tensors.
//
// Step metadata (all int32, static device buffers → capturable): positions[T], slot_mapping[T] (cache row, < 0:
// padding), token_seq[T] (batch row of a token, < 0: padding), query_start_loc[B+1], state_slots[B] (< 0: none),
// counts[3] = number of valid batch rows (grids over batch rows are launched at an upper bound).
#include <algorithm>

#include "common.h"
#include "kernels.h"

namespace dli {

namespace {

constexpr int NT = 256;

template <typename A> __device__ __forceinline__ float ldf(const A* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <typename A> __device__ __forceinline__ void stf(A* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }

__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }

// mean and 1/sqrt(var + eps) of a row held in LDS (two passes: the variance is the mean squared deviation)
__device__ __forceinline__ void row_stats(const float* row, int W, float eps, float* red, float& mean, float& inv) {
  float s = 0.f;
  for (int i = threadIdx.x; i < W; i += NT) s += row[i];
  mean = block_sum<NT>(s, red) / (float)W;
  float v = 0.f;
  for (int i = threadIdx.x; i < W; i += NT) {
    const float d = row[i] - mean;
    v += d * d;
  }
  inv = 1.f / sqrtf(block_sum<NT>(v, red) / (float)W + eps);
}

// ------------------------------------------------------------------------------------------------ norms
template <typename O>
__global__ __launch_bounds__(NT) void layer_norm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                        const float* __restrict__ b, float eps, int W, O* __restrict__ out) {
  extern __shared__ float sh[];
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < W; i += NT) sh[i] = x[t * W + i];
  __syncthreads();
  float mean, inv;
  row_stats(sh, W, eps, red, mean, inv);
  for (int i = threadIdx.x; i < W; i += NT) stf<O>(out + t * W + i, (sh[i] - mean) * inv * w[i] + b[i]);
}

// h[t] = g[t] + (g[t-1] - g[t]) * mix with g = layer_norm(x (+ add)); g[t-1] is recomputed from the row above inside a
// chunk, read from the sequence's state row at a chunk start, zero at position 0.  xout (with add): the new stream.
template <typename O>
__global__ __launch_bounds__(NT) void ln_shift_kernel(const float* __restrict__ x, const float* __restrict__ add,
                                                      float* __restrict__ xout, const float* __restrict__ w,
                                                      const float* __restrict__ b, const float* __restrict__ mix,
                                                      const float* __restrict__ state, const int* __restrict__ positions,
                                                      const int* __restrict__ token_seq, const int* __restrict__ qsl,
                                                      const int* __restrict__ state_slots, float eps, int W,
                                                      O* __restrict__ out) {
  extern __shared__ float sh[];
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int seq = token_seq[t];
  if (seq < 0) return;
  const int slot = state_slots[seq];
  const int pos = positions[t];
  const bool first = (int)t == qsl[seq];
  const int mode = pos == 0 ? 0 : (first ? (slot >= 0 ? 1 : 0) : 2);
  float* cur = sh;
  float* prv = sh + W;
  for (int i = threadIdx.x; i < W; i += NT) {
    float v = x[t * W + i];
    if (add != nullptr) {
      v += add[t * W + i];
      xout[t * W + i] = v;
    }
    cur[i] = v;
    if (mode == 2) prv[i] = x[(t - 1) * W + i] + (add != nullptr ? add[(t - 1) * W + i] : 0.f);
  }
  __syncthreads();
  float mean, inv, pmean = 0.f, pinv = 0.f;
  row_stats(cur, W, eps, red, mean, inv);
  if (mode == 2) row_stats(prv, W, eps, red, pmean, pinv);
  for (int i = threadIdx.x; i < W; i += NT) {
    const float g = (cur[i] - mean) * inv * w[i] + b[i];
    float p = 0.f;
    if (mode == 1) p = state[(int64_t)slot * W + i];
    else if (mode == 2) p = (prv[i] - pmean) * pinv * w[i] + b[i];
    stf<O>(out + t * W + i, g + (p - g) * mix[i]);
  }
}

// state[slot] = layer_norm(x (+ add)) of every sequence's last token of the step (runs behind ln_shift_kernel)
__global__ __launch_bounds__(NT) void ln_state_kernel(const float* __restrict__ x, const float* __restrict__ add,
                                                      const float* __restrict__ w, const float* __restrict__ b,
                                                      float* __restrict__ state, const int* __restrict__ qsl,
                                                      const int* __restrict__ state_slots, const int* __restrict__ counts,
                                                      float eps, int W) {
  extern __shared__ float sh[];
  __shared__ float red[NT / 64];
  const int seq = blockIdx.x;
  if (seq >= counts[3]) return;
  const int slot = state_slots[seq];
  const int t0 = qsl[seq], t1 = qsl[seq + 1];
  if (slot < 0 || t1 <= t0) return;
  const int64_t t = t1 - 1;
  for (int i = threadIdx.x; i < W; i += NT) sh[i] = x[t * W + i] + (add != nullptr ? add[t * W + i] : 0.f);
  __syncthreads();
  float mean, inv;
  row_stats(sh, W, eps, red, mean, inv);
  for (int i = threadIdx.x; i < W; i += NT) state[(int64_t)slot * W + i] = (sh[i] - mean) * inv * w[i] + b[i];
}

// x += mult * layer_norm(y; w1, b1); optionally out = layer_norm(x; w2, b2)
template <typename Y, typename O>
__global__ __launch_bounds__(NT) void add_ln_kernel(float* __restrict__ x, const Y* __restrict__ y, int64_t y_stride,
                                                    const float* __restrict__ w1, const float* __restrict__ b1, float mult,
                                                    const float* __restrict__ w2, const float* __restrict__ b2, float eps,
                                                    int W, O* __restrict__ out) {
  extern __shared__ float sh[];
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < W; i += NT) sh[i] = ldf<Y>(y + t * y_stride + i);
  __syncthreads();
  float mean, inv;
  row_stats(sh, W, eps, red, mean, inv);
  for (int i = threadIdx.x; i < W; i += NT) {
    const float v = x[t * W + i] + mult * ((sh[i] - mean) * inv * w1[i] + b1[i]);
    x[t * W + i] = v;
    sh[i] = v;
  }
  if (w2 == nullptr) return;
  __syncthreads();
  row_stats(sh, W, eps, red, mean, inv);
  for (int i = threadIdx.x; i < W; i += NT) stf<O>(out + t * W + i, (sh[i] - mean) * inv * w2[i] + b2[i]);
}

template <typename G, typename O>
__global__ __launch_bounds__(NT) void rms_gate_kernel(const float* __restrict__ o, const float* __restrict__ w, float eps,
                                                      const G* __restrict__ gate, int64_t gate_stride, int N,
                                                      O* __restrict__ out) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  float s = 0.f;
  for (int i = threadIdx.x; i < N; i += NT) {
    const float v = o[t * N + i];
    s += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum<NT>(s, red) / (float)N + eps);
  for (int i = threadIdx.x; i < N; i += NT) {
    const float g = ldf<G>(gate + t * gate_stride + i);
    stf<O>(out + t * N + i, o[t * N + i] * inv * w[i] / (1.f + expf(-g)));
  }
}

template <typename A>
__global__ __launch_bounds__(NT) void relu2_kernel(const A* __restrict__ x, A* __restrict__ out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x; i < n; i += (int64_t)gridDim.x * NT) {
    const float v = fmaxf(ldf<A>(x + i), 0.f);
    stf<A>(out + i, v * v);
  }
}

template <typename A>
__global__ __launch_bounds__(NT) void softcap_kernel(const A* __restrict__ x, float* __restrict__ out, float cap, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x; i < n; i += (int64_t)gridDim.x * NT)
    out[i] = cap * tanhf(ldf<A>(x + i) / cap);
}

// ------------------------------------------------------------------------------------------------ cache writers
// one workgroup per token; a wave per head vector: unit RMS times weight; q in place, k and v to the token's cache rows
template <typename A>
__global__ __launch_bounds__(NT) void qk_norm_cache_kernel(A* __restrict__ qkv, int64_t row_stride,
                                                           const float* __restrict__ qw, const float* __restrict__ kw,
                                                           float eps, const int* __restrict__ slot_mapping,
                                                           A* __restrict__ k_cache, A* __restrict__ v_cache, int H, int G,
                                                           int D, int Dv) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slot = slot_mapping[t];
  A* row = qkv + t * row_stride;
  for (int u = wave; u < H + G; u += NT / 64) {
    A* p = row + (int64_t)u * D;
    float ss = 0.f;
    for (int i = lane; i < D; i += 64) {
      const float v = ldf<A>(p + i);
      ss += v * v;
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
    if (u < H) {
      for (int i = lane; i < D; i += 64) stf<A>(p + i, ldf<A>(p + i) * inv * qw[i]);
    } else if (slot >= 0) {
      A* dst = k_cache + ((int64_t)slot * G + (u - H)) * D;
      for (int i = lane; i < D; i += 64) stf<A>(dst + i, ldf<A>(p + i) * inv * kw[i]);
    }
  }
  if (slot >= 0) {
    const A* v = row + (int64_t)(H + G) * D;
    A* dst = v_cache + (int64_t)slot * G * Dv;
    for (int i = threadIdx.x; i < G * Dv; i += NT) dst[i] = v[i];
  }
}

// latent attention: cache row = [unit-RMS latent * cw | rotated shared key]; the rotated part of every q head in place
template <typename A>
__global__ __launch_bounds__(NT) void latent_prep_kernel(A* __restrict__ q, int64_t q_stride, const A* __restrict__ dkv,
                                                         int64_t dkv_stride, const float* __restrict__ cw, float eps,
                                                         const int* __restrict__ positions, const double* __restrict__ inv_freq,
                                                         int rot_dims, const int* __restrict__ slot_mapping,
                                                         A* __restrict__ cache, int H, int D, int R, int C) {
  extern __shared__ float sh[];          // cos[rot_dims/2], sin[rot_dims/2]
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int slot = slot_mapping[t];
  const int half = rot_dims >> 1;
  const double pos = (double)positions[t];
  for (int i = threadIdx.x; i < half; i += NT) {
    double a = pos * inv_freq[i];
    a -= 6.283185307179586476925 * floor(a * 0.15915494309189533577);    // reduced in double, then exact enough in fp32
    double sn, cs;
    sincos(a, &sn, &cs);
    sh[i] = (float)cs;
    sh[half + i] = (float)sn;
  }
  const A* crow = dkv + t * dkv_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < C; i += NT) {
    const float v = ldf<A>(crow + i);
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)C + eps);      // (block_sum's barriers also publish sh)
  A* dst = cache + (int64_t)slot * (C + R);
  if (slot >= 0) {
    for (int i = threadIdx.x; i < C; i += NT) stf<A>(dst + i, ldf<A>(crow + i) * inv * cw[i]);
    for (int i = threadIdx.x; i < R; i += NT) {
      float v = ldf<A>(crow + C + i);
      if (i < rot_dims) {
        const int pr = i >> 1;
        const float o = ldf<A>(crow + C + (i ^ 1));
        v = (i & 1) ? v * sh[pr] + o * sh[half + pr] : v * sh[pr] - o * sh[half + pr];
      }
      stf<A>(dst + C + i, v);
    }
  }
  // q heads: one pair per thread and trip (both entries read before either is written)
  A* qrow = q + t * q_stride;
  for (int idx = threadIdx.x; idx < H * half; idx += NT) {
    const int h = idx / half, pr = idx - h * half;
    A* p = qrow + (int64_t)h * (D + R) + D + 2 * pr;
    const float u = ldf<A>(p), v = ldf<A>(p + 1);
    stf<A>(p, u * sh[pr] - v * sh[half + pr]);
    stf<A>(p + 1, v * sh[pr] + u * sh[half + pr]);
  }
}

// ------------------------------------------------------------------------------------------------ attention
// One workgroup per (token, query head); every wave takes chunks of 64 consecutive keys, a lane per key for the scores
// (q broadcast from LDS), then lanes over the value columns for P·V (weights and cache rows broadcast by shuffles).
// Online softmax per wave, the four waves merged through LDS.  Serves decode rows and prefill-chunk tokens alike: a
// token's position and batch row come from the step metadata, keys from the sequence's block-table row.
template <typename A, int NV>
__global__ __launch_bounds__(NT) void token_attention_kernel(
    A* __restrict__ out, int64_t o_ts, int64_t o_hs, const A* __restrict__ q1, int64_t q1_ts, int64_t q1_hs, int D1,
    const A* __restrict__ q2, int64_t q2_ts, int64_t q2_hs, int D2, const A* __restrict__ kc, int rowk,
    const A* __restrict__ vc, int rowv, int vhead, int Dv, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ positions, const int* __restrict__ token_seq, int H, int G, float scale, int window,
    const float* __restrict__ temp, const float* __restrict__ r1, const float* __restrict__ r2) {
  extern __shared__ float sh[];          // q [Dk] | per wave: acc [Dv] | m[4] | l[4]
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int seq = token_seq[t];
  if (seq < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int Dk = D1 + D2;
  const int p = positions[t];
  const int lo = window > 0 ? max(p - window + 1, 0) : 0;
  const int g = h / (H / G);
  float* qs = sh;
  float* accs = sh + Dk;
  float* ms = accs + (NT / 64) * Dv;
  float* ls = ms + NT / 64;
  const float qmul = scale * (temp != nullptr ? temp[h] : 1.f);
  for (int i = threadIdx.x; i < Dk; i += NT)
    qs[i] = qmul * (i < D1 ? ldf<A>(q1 + t * q1_ts + h * q1_hs + i) : ldf<A>(q2 + t * q2_ts + h * q2_hs + (i - D1)));
  __syncthreads();
  const bool pen = r1 != nullptr;
  const float r1h = pen ? r1[h] : 0.f, r2h = pen ? r2[h] : 0.f;
  const int* bt = block_tables + (int64_t)seq * max_blocks;

  float m = -INFINITY, l = 0.f;
  float acc[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) acc[v] = 0.f;

  for (int base = lo + wave * 64; base <= p; base += (NT / 64) * 64) {
    const int j = base + lane;
    const bool valid = j <= p;
    int slot = 0;
    float s = -INFINITY;
    if (valid) {
      slot = bt[j / kBlockTokens] * kBlockTokens + (j % kBlockTokens);
      const A* kr = kc + (int64_t)slot * rowk + g * Dk;
      float d = 0.f;
      for (int i = 0; i < Dk; ++i) d += qs[i] * ldf<A>(kr + i);
      s = pen ? d - r1h * log1pf(r2h * (float)(p - j)) : d;
    }
    const float mn = fmaxf(m, wave_max(s));
    const float corr = expf(m - mn);               // first chunk: exp(-inf) = 0
    const float pl = valid ? expf(s - mn) : 0.f;
    l = l * corr + wave_sum(pl);
    m = mn;
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] *= corr;
    const int nvalid = min(p - base + 1, 64);
    for (int jj = 0; jj < nvalid; ++jj) {
      const float pj = __shfl(pl, jj, 64);
      const int sj = __shfl(slot, jj, 64);
      const A* vr = vc + (int64_t)sj * rowv + g * vhead;
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const int e = lane + 64 * v;
        if (e < Dv) acc[v] += pj * ldf<A>(vr + e);
      }
    }
  }
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int e = lane + 64 * v;
    if (e < Dv) accs[wave * Dv + e] = acc[v];
  }
  if (lane == 0) {
    ms[wave] = m;
    ls[wave] = l;
  }
  __syncthreads();
  float M = ms[0];
#pragma unroll
  for (int w = 1; w < NT / 64; ++w) M = fmaxf(M, ms[w]);
  float L = 0.f;
  float f[NT / 64];
#pragma unroll
  for (int w = 0; w < NT / 64; ++w) {
    f[w] = expf(ms[w] - M);
    L += f[w] * ls[w];
  }
  for (int e = threadIdx.x; e < Dv; e += NT) {
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < NT / 64; ++w) o += f[w] * accs[w * Dv + e];
    stf<A>(out + t * o_ts + h * o_hs + e, o / L);
  }
}

// ------------------------------------------------------------------------------------------------ linear attention
// One wave per (sequence, head, 64 value columns): lane e keeps column e of the [D, Dv] state in registers and walks the
// step's tokens in order: S ← decay·S + silu(k)·silu(v)ᵀ, o = Sᵀ silu(q).  The next token's q / k / v are fetched while
// the current one is applied.  DMAX: compile-time bound of D (registers per lane).
template <typename A, int DMAX>
__global__ __launch_bounds__(64) void lightning_scan_kernel(const A* __restrict__ qkvg, int64_t row_stride,
                                                            float* __restrict__ state, const int* __restrict__ positions,
                                                            const int* __restrict__ qsl, const int* __restrict__ state_slots,
                                                            const int* __restrict__ counts, int H, int D, int Dv,
                                                            const float* __restrict__ decay, float* __restrict__ out) {
  __shared__ float qs[2][DMAX], ks[2][DMAX];
  const int seq = blockIdx.x;
  if (seq >= counts[3]) return;
  const int slot = state_slots[seq];
  const int t0 = qsl[seq], t1 = qsl[seq + 1];
  if (slot < 0 || t1 <= t0) return;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int e = blockIdx.z * 64 + lane;
  const bool active = e < Dv;
  const float lam = decay[h];
  float S[DMAX];
  float* srow = state + ((int64_t)slot * H + h) * D * Dv;
  const bool carry = positions[t0] > 0;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) S[d] = (carry && active && d < D) ? srow[(int64_t)d * Dv + e] : 0.f;

  const int64_t qoff = (int64_t)h * D, koff = (int64_t)H * D + (int64_t)h * D, voff = 2 * (int64_t)H * D + (int64_t)h * Dv;
  constexpr int PER = (DMAX + 63) / 64;
  float nq[PER], nk[PER], nv = 0.f;
  auto fetch = [&](int t) {
    const A* row = qkvg + (int64_t)t * row_stride;
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = lane + 64 * r;
      nq[r] = i < D ? ldf<A>(row + qoff + i) : 0.f;
      nk[r] = i < D ? ldf<A>(row + koff + i) : 0.f;
    }
    nv = active ? ldf<A>(row + voff + e) : 0.f;
  };
  fetch(t0);
  for (int t = t0; t < t1; ++t) {
    const int buf = (t - t0) & 1;
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = lane + 64 * r;
      if (i < DMAX) {
        qs[buf][i] = silu_f(nq[r]);
        ks[buf][i] = silu_f(nk[r]);
      }
    }
    const float ve = silu_f(nv);
    if (t + 1 < t1) fetch(t + 1);
    __syncthreads();                       // one wave: publishes qs / ks of this token (the other buffer is being refilled next trip)
    float o = 0.f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < D) {
        S[d] = lam * S[d] + ks[buf][d] * ve;
        o += S[d] * qs[buf][d];
      }
    }
    if (active) out[(int64_t)t * H * Dv + (int64_t)h * Dv + e] = o;
  }
  if (active) {
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
      if (d < D) srow[(int64_t)d * Dv + e] = S[d];
  }
}

}  // namespace

// ================================================================================================ launchers
#define SM_DISPATCH_BF16(flag, T, ...) \
  do {                                 \
    if (flag) {                        \
      using T = uint16_t;              \
      __VA_ARGS__;                     \
    } else {                           \
      using T = float;                 \
      __VA_ARGS__;                     \
    }                                  \
  } while (0)

void launch_sm_layer_norm(const float* x, const float* w, const float* b, float eps, int rows, int W, void* out, bool out_bf16,
                          hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(out_bf16, O, hipLaunchKernelGGL(layer_norm_kernel<O>, dim3(rows), dim3(NT), W * sizeof(float), stream, x, w, b,
                                                   eps, W, (O*)out));
}

void launch_sm_ln_shift(const float* x, const float* add, float* xout, const float* w, const float* b, const float* mix,
                        float* state, const int* positions, const int* token_seq, const int* qsl, const int* state_slots,
                        const int* counts, int rows, int seqs, float eps, int W, void* out, bool out_bf16, hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(out_bf16, O, hipLaunchKernelGGL(ln_shift_kernel<O>, dim3(rows), dim3(NT), 2 * W * sizeof(float), stream, x, add,
                                                   xout, w, b, mix, (const float*)state, positions, token_seq, qsl, state_slots,
                                                   eps, W, (O*)out));
  if (seqs > 0)
    hipLaunchKernelGGL(ln_state_kernel, dim3(seqs), dim3(NT), W * sizeof(float), stream, x, add, w, b, state, qsl, state_slots,
                       counts, eps, W);
}

void launch_sm_add_ln(float* x, const void* y, bool y_bf16, int64_t y_stride, const float* w1, const float* b1, float mult,
                      const float* w2, const float* b2, float eps, int rows, int W, void* out, bool out_bf16,
                      hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(y_bf16, Y, SM_DISPATCH_BF16(out_bf16, O, hipLaunchKernelGGL((add_ln_kernel<Y, O>), dim3(rows), dim3(NT),
                                                                                W * sizeof(float), stream, x, (const Y*)y,
                                                                                y_stride, w1, b1, mult, w2, b2, eps, W, (O*)out)));
}

void launch_sm_rms_gate(const float* o, const float* w, float eps, const void* gate, bool gate_bf16, int64_t gate_stride, int rows,
                        int N, void* out, bool out_bf16, hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(gate_bf16, G, SM_DISPATCH_BF16(out_bf16, O, hipLaunchKernelGGL((rms_gate_kernel<G, O>), dim3(rows), dim3(NT), 0,
                                                                                   stream, o, w, eps, (const G*)gate, gate_stride,
                                                                                   N, (O*)out)));
}

void launch_sm_relu2(const void* x, void* out, int64_t n, bool bf16, hipStream_t stream) {
  if (n == 0) return;
  const int blocks = (int)std::min<int64_t>((n + NT - 1) / NT, 4096);
  SM_DISPATCH_BF16(bf16, A, hipLaunchKernelGGL(relu2_kernel<A>, dim3(blocks), dim3(NT), 0, stream, (const A*)x, (A*)out, n));
}

void launch_sm_softcap(const void* x, bool bf16, float* out, float cap, int64_t n, hipStream_t stream) {
  if (n == 0) return;
  const int blocks = (int)std::min<int64_t>((n + NT - 1) / NT, 4096);
  SM_DISPATCH_BF16(bf16, A, hipLaunchKernelGGL(softcap_kernel<A>, dim3(blocks), dim3(NT), 0, stream, (const A*)x, out, cap, n));
}

void launch_sm_qk_norm_cache(void* qkv, bool bf16, int64_t row_stride, const float* qw, const float* kw, float eps,
                             const int* slot_mapping, void* k_cache, void* v_cache, int rows, int H, int G, int D, int Dv,
                             hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(bf16, A, hipLaunchKernelGGL(qk_norm_cache_kernel<A>, dim3(rows), dim3(NT), 0, stream, (A*)qkv, row_stride, qw, kw,
                                               eps, slot_mapping, (A*)k_cache, (A*)v_cache, H, G, D, Dv));
}

void launch_sm_latent_prep(void* q, bool bf16, int64_t q_stride, const void* dkv, int64_t dkv_stride, const float* cw, float eps,
                           const int* positions, const double* inv_freq, int rot_dims, const int* slot_mapping, void* cache,
                           int rows, int H, int D, int R, int C, hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(bf16, A, hipLaunchKernelGGL(latent_prep_kernel<A>, dim3(rows), dim3(NT), std::max(rot_dims, 2) * sizeof(float),
                                               stream, (A*)q, q_stride, (const A*)dkv, dkv_stride, cw, eps, positions, inv_freq,
                                               rot_dims, slot_mapping, (A*)cache, H, D, R, C));
}

template <typename A>
static void token_attention_nv(int nv, dim3 grid, size_t lds, hipStream_t stream, A* out, int64_t o_ts, int64_t o_hs, const A* q1,
                               int64_t q1_ts, int64_t q1_hs, int D1, const A* q2, int64_t q2_ts, int64_t q2_hs, int D2, const A* kc,
                               int rowk, const A* vc, int rowv, int vhead, int Dv, const int* bt, int max_blocks, const int* pos,
                               const int* tseq, int H, int G, float scale, int window, const float* temp, const float* r1,
                               const float* r2) {
#define SM_ATT(NVV)                                                                                                              \
  hipLaunchKernelGGL((token_attention_kernel<A, NVV>), grid, dim3(NT), lds, stream, out, o_ts, o_hs, q1, q1_ts, q1_hs, D1, q2,   \
                     q2_ts, q2_hs, D2, kc, rowk, vc, rowv, vhead, Dv, bt, max_blocks, pos, tseq, H, G, scale, window, temp, r1, r2)
  if (nv <= 1) SM_ATT(1);
  else if (nv <= 2) SM_ATT(2);
  else if (nv <= 4) SM_ATT(4);
  else SM_ATT(8);
#undef SM_ATT
}

void launch_sm_token_attention(void* out, int64_t o_ts, int64_t o_hs, const void* q1, int64_t q1_ts, int64_t q1_hs, int D1,
                               const void* q2, int64_t q2_ts, int64_t q2_hs, int D2, const void* kc, int rowk, const void* vc,
                               int rowv, int vhead, int Dv, const int* block_tables, int max_blocks, const int* positions,
                               const int* token_seq, int rows, int H, int G, float scale, int window, const float* temp,
                               const float* r1, const float* r2, bool bf16, hipStream_t stream) {
  if (rows == 0) return;
  const size_t lds = (size_t)(D1 + D2 + (NT / 64) * Dv + 2 * (NT / 64)) * sizeof(float);
  const dim3 grid(rows, H);
  const int nv = (Dv + 63) / 64;
  SM_DISPATCH_BF16(bf16, A, token_attention_nv<A>(nv, grid, lds, stream, (A*)out, o_ts, o_hs, (const A*)q1, q1_ts, q1_hs, D1,
                                                  (const A*)q2, q2_ts, q2_hs, D2, (const A*)kc, rowk, (const A*)vc, rowv, vhead, Dv,
                                                  block_tables, max_blocks, positions, token_seq, H, G, scale, window, temp, r1, r2));
}

void launch_sm_lightning_scan(const void* qkvg, bool bf16, int64_t row_stride, float* state, const int* positions, const int* qsl,
                              const int* state_slots, const int* counts, int seqs, int H, int D, int Dv, const float* decay,
                              float* out, hipStream_t stream) {
  if (seqs == 0) return;
  const dim3 grid(seqs, H, (Dv + 63) / 64);
#define SM_SCAN(DM)                                                                                                                \
  SM_DISPATCH_BF16(bf16, A, hipLaunchKernelGGL((lightning_scan_kernel<A, DM>), grid, dim3(64), 0, stream, (const A*)qkvg, row_stride, \
                                               state, positions, qsl, state_slots, counts, H, D, Dv, decay, out))
  if (D <= 32) SM_SCAN(32);
  else if (D <= 64) SM_SCAN(64);
  else if (D <= 128) SM_SCAN(128);
  else SM_SCAN(256);
#undef SM_SCAN
}

}  // namespace dli
