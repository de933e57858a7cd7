// Mixers that carry a fixed-size state per sequence instead of a cache of keys.
//
// Gated diagonal recurrence ("rglru"): per channel c
//     u_t = conv_b + sum_j taps[c][j] * xin_{t-(K-1-j)}          (short causal convolution)
//     r_t, i_t = sigmoid(block-diagonal products of u_t + bias)
//     a_t = exp(-c0 * r_t * softplus(lam)),  S_t = a_t S_{t-1} + sqrt(1 - a_t^2) * i_t * u_t
//     out_t = S_t * gelu_tanh(y_t)
//   in two kernels: `rglru_gates` forms a_t and the input term for all tokens at once (they do
//   not depend on S), `rglru_scan` walks each sequence's tokens in order, one thread a channel.
//
// Gated linear attention ("gla"): per head a matrix state S [dk][dv]
//     alpha_t = sigmoid(z_t)^(1/tau) per key channel, z_t = A2 (a1h_t) + bias
//     S_t = diag(alpha_t) S_{t-1} + k_t v_t^T,  o_t = S_t^T q_t
//   `gla_recurrent` walks a sequence's tokens in order with S in registers; `gla_out` applies the
//   per-head RMS norm and the output gate.
//
// All state, decays, gates and sums are float32; tokens are walked in the same order however a
// sequence was cut into steps, so the cut does not change a bit of the result.
#include "common.h"

__device__ __forceinline__ int seq_of_token_r(const int* __restrict__ cu_q, int batch, int t) {
  int lo = 0, hi = batch - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float gelu_tanhf_(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ------------------------------------------------------------------ rglru: gates
#define RG_TT 8     // tokens per workgroup

template <typename T, typename TW>
__global__ __launch_bounds__(256) void rglru_gates_kernel(
    const T* __restrict__ yx, int stride, int xoff, const float* __restrict__ xbias,
    const float* __restrict__ taps, const float* __restrict__ conv_bias, int K,
    const float* __restrict__ conv_state, const TW* __restrict__ gates_w,
    const float* __restrict__ gates_b, const float* __restrict__ lam, float c0,
    const int* __restrict__ cu_q, const int* __restrict__ slots, int batch, int nt, int C, int nb,
    float* __restrict__ a_out, float* __restrict__ b_out) {
  extern __shared__ float u[];            // [RG_TT][bs]
  __shared__ int s_start[RG_TT], s_slot[RG_TT];
  const int bs = C / nb;
  const int t0 = blockIdx.x * RG_TT, blk = blockIdx.y;
  if (threadIdx.x < RG_TT) {
    const int t = t0 + threadIdx.x;
    int st = 0, sl = 0;
    if (t < nt) {
      const int b = seq_of_token_r(cu_q, batch, t);
      st = cu_q[b];
      sl = slots[b];
    }
    s_start[threadIdx.x] = st;
    s_slot[threadIdx.x] = sl;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < RG_TT * bs; idx += 256) {
    const int tt = idx / bs, cc = idx - tt * bs;
    const int t = t0 + tt, c = blk * bs + cc;
    float acc = 0.f;
    if (t < nt) {
      acc = conv_bias[c];
      const int start = s_start[tt];
      const float* cs = conv_state + ((size_t)s_slot[tt] * (K - 1)) * C;
      for (int j = 0; j < K; ++j) {
        const int tp = t - (K - 1 - j);
        float xin;
        if (tp >= start) xin = to_f32(yx[(size_t)tp * stride + xoff + c]) + xbias[c];
        else xin = cs[(size_t)(K - 1 + (tp - start)) * C + c];
        acc = fmaf(taps[(size_t)c * K + j], xin, acc);
      }
    }
    u[idx] = acc;
  }
  __syncthreads();
  for (int o = threadIdx.x; o < bs; o += 256) {
    const int c = blk * bs + o;
    float ar[RG_TT], ai[RG_TT];
#pragma unroll
    for (int tt = 0; tt < RG_TT; ++tt) ar[tt] = ai[tt] = 0.f;
    const TW* wr = gates_w + ((size_t)blk * bs + o) * bs;                 // recurrence gate, block blk
    const TW* wi = gates_w + ((size_t)(nb + blk) * bs + o) * bs;          // input gate
    for (int in = 0; in < bs; ++in) {
      const float a = to_f32(wr[in]), b = to_f32(wi[in]);
#pragma unroll
      for (int tt = 0; tt < RG_TT; ++tt) {
        const float uu = u[tt * bs + in];
        ar[tt] = fmaf(a, uu, ar[tt]);
        ai[tt] = fmaf(b, uu, ai[tt]);
      }
    }
    const float br = gates_b[(size_t)blk * bs + o], bi = gates_b[(size_t)(nb + blk) * bs + o];
    const float sp = softplusf_(lam[c]);
#pragma unroll
    for (int tt = 0; tt < RG_TT; ++tt) {
      const int t = t0 + tt;
      if (t < nt) {
        const float r = sigmoidf_(ar[tt] + br), g = sigmoidf_(ai[tt] + bi);
        const float loga = -c0 * r * sp;
        a_out[(size_t)t * C + c] = expf(loga);
        b_out[(size_t)t * C + c] = sqrtf(-expm1f(2.0f * loga)) * g * u[tt * bs + o];
      }
    }
  }
}

// yx: [nt, stride] rows holding the y branch at column 0 and the x branch at column xoff (C each);
// xbias [C]; taps [C, K]; conv_state [slots, K-1, C] float32 (inputs of the last K-1 tokens);
// gates_w [2*nb, bs, bs] (recurrence gate blocks, then input gate blocks), gates_b [2*nb, bs];
// a_out, b_out: [nt, C] float32.
extern "C" int ta_rglru_gates(hipStream_t stream, int dtype, int wdtype, const void* yx, int stride, int xoff,
                              const float* xbias, const float* taps, const float* conv_bias, int K,
                              const float* conv_state, const void* gates_w, const float* gates_b,
                              const float* lam, float c0, const int* cu_q, const int* slots, int batch,
                              int nt, int C, int nb, float* a_out, float* b_out) {
  TA_REQUIRE(batch > 0 && nt >= batch && C > 0 && nb > 0 && C % nb == 0 && K >= 1,
             "ta_rglru_gates: bad sizes nt=%d C=%d blocks=%d taps=%d", nt, C, nb, K);
  TA_REQUIRE(nb <= 65535, "ta_rglru_gates: too many blocks");
  const int bs = C / nb;
  const size_t lds = (size_t)RG_TT * bs * sizeof(float);
  TA_REQUIRE(lds <= 60000, "ta_rglru_gates: blocks of %d channels do not fit", bs);
  dim3 g((nt + RG_TT - 1) / RG_TT, nb);
#define RG_LAUNCH(T, TW)                                                                          \
  rglru_gates_kernel<T, TW><<<g, 256, lds, stream>>>((const T*)yx, stride, xoff, xbias, taps, conv_bias, K, \
      conv_state, (const TW*)gates_w, gates_b, lam, c0, cu_q, slots, batch, nt, C, nb, a_out, b_out)
  if (dtype == TA_F32 && wdtype == TA_F32) RG_LAUNCH(float, float);
  else if (dtype == TA_BF16 && wdtype == TA_BF16) RG_LAUNCH(bf16_t, bf16_t);
  else if (dtype == TA_BF16 && wdtype == TA_F32) RG_LAUNCH(bf16_t, float);
  else return ta_fail("ta_rglru_gates: unsupported dtypes %d / %d", dtype, wdtype);
#undef RG_LAUNCH
  return ta_check_launch("ta_rglru_gates");
}

// ------------------------------------------------------------------ rglru: scan
template <typename T>
__global__ __launch_bounds__(256) void rglru_scan_kernel(
    const T* __restrict__ yx, int stride, int xoff, const float* __restrict__ ybias,
    const float* __restrict__ xbias, const float* __restrict__ a_in, const float* __restrict__ b_in,
    float* __restrict__ state, float* __restrict__ conv_state, int K, const int* __restrict__ cu_q,
    const int* __restrict__ slots, int C, T* __restrict__ out) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int start = cu_q[b], end = cu_q[b + 1];
  const size_t slot = (size_t)slots[b];
  float S = state[slot * C + c];
  const float yb = ybias[c];
  int t = start;
  for (; t + 4 <= end; t += 4) {
    float a[4], bb[4], y[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[i] = a_in[(size_t)(t + i) * C + c];
      bb[i] = b_in[(size_t)(t + i) * C + c];
      y[i] = to_f32(yx[(size_t)(t + i) * stride + c]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      S = fmaf(a[i], S, bb[i]);
      out[(size_t)(t + i) * C + c] = from_f32<T>(S * gelu_tanhf_(y[i] + yb));
    }
  }
  for (; t < end; ++t) {
    S = fmaf(a_in[(size_t)t * C + c], S, b_in[(size_t)t * C + c]);
    out[(size_t)t * C + c] = from_f32<T>(S * gelu_tanhf_(to_f32(yx[(size_t)t * stride + c]) + yb));
  }
  state[slot * C + c] = S;
  // the convolution's memory: inputs of the sequence's last K-1 tokens, oldest first
  const int n = end - start;
  float* cs = conv_state + slot * (size_t)(K - 1) * C;
  const float xb = xbias[c];
  for (int j = 0; j < K - 1; ++j) {
    const int src = j + n;            // index into (old memory, then this step's tokens)
    float v;
    if (src < K - 1) v = cs[(size_t)src * C + c];
    else v = to_f32(yx[(size_t)(start + src - (K - 1)) * stride + xoff + c]) + xb;
    cs[(size_t)j * C + c] = v;
  }
}

// state [slots, C] float32; out [nt, C]. Runs after ta_rglru_gates of the same step.
extern "C" int ta_rglru_scan(hipStream_t stream, int dtype, const void* yx, int stride, int xoff,
                             const float* ybias, const float* xbias, const float* a_in, const float* b_in,
                             float* state, float* conv_state, int K, const int* cu_q, const int* slots,
                             int batch, int C, void* out) {
  TA_REQUIRE(batch > 0 && batch <= 65535 && C > 0 && K >= 1, "ta_rglru_scan: bad sizes");
  dim3 g((C + 255) / 256, batch);
  if (dtype == TA_F32)
    rglru_scan_kernel<float><<<g, 256, 0, stream>>>((const float*)yx, stride, xoff, ybias, xbias, a_in, b_in, state,
                                                   conv_state, K, cu_q, slots, C, (float*)out);
  else if (dtype == TA_BF16)
    rglru_scan_kernel<bf16_t><<<g, 256, 0, stream>>>((const bf16_t*)yx, stride, xoff, ybias, xbias, a_in, b_in, state,
                                                    conv_state, K, cu_q, slots, C, (bf16_t*)out);
  else
    return ta_fail("ta_rglru_scan: unknown dtype %d", dtype);
  return ta_check_launch("ta_rglru_scan");
}

// ------------------------------------------------------------------ gla: recurrence
#define GLA_TC 8      // tokens whose operands are staged together

template <typename T, typename TW, int R>
__global__ __launch_bounds__(256) void gla_recurrent_kernel(
    const T* __restrict__ proj, int stride, int qoff, int koff, int voff, int aoff, int rank,
    const TW* __restrict__ a2, const float* __restrict__ a2b, float inv_tau, float qscale,
    float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ slots,
    int H, int dk, int dv, int CT, int P, float* __restrict__ o_out) {
  extern __shared__ float sm[];
  const int PR = P * R;                    // padded key width
  float* sq = sm;                          // [TC][PR]
  float* sk = sq + GLA_TC * PR;            // [TC][PR]
  float* sa = sk + GLA_TC * PR;            // [TC][PR]
  float* sv = sa + GLA_TC * PR;            // [TC][CT]
  float* s1 = sv + GLA_TC * CT;            // [TC][rank]
  float* part = s1 + GLA_TC * rank;        // [TC][P][CT]
  const int b = blockIdx.x, h = blockIdx.y, col0 = blockIdx.z * CT;
  const int start = cu_q[b], end = cu_q[b + 1];
  const size_t slot = (size_t)slots[b];
  const int j = threadIdx.x % CT, p = threadIdx.x / CT;
  const bool active = p < P && col0 + j < dv;
  float* st = state + ((slot * H + h) * dk) * (size_t)dv;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = p * R + r;
    S[r] = (active && i < dk) ? st[(size_t)i * dv + col0 + j] : 0.f;
  }
  for (int t0 = start; t0 < end; t0 += GLA_TC) {
    const int n = end - t0 < GLA_TC ? end - t0 : GLA_TC;
    for (int idx = threadIdx.x; idx < GLA_TC * PR; idx += 256) {
      const int tt = idx / PR, i = idx - tt * PR;
      float qv = 0.f, kv = 0.f;
      if (tt < n && i < dk) {
        const T* row = proj + (size_t)(t0 + tt) * stride;
        qv = to_f32(row[qoff + h * dk + i]) * qscale;
        kv = to_f32(row[koff + h * dk + i]);
      }
      sq[idx] = qv;
      sk[idx] = kv;
    }
    for (int idx = threadIdx.x; idx < GLA_TC * CT; idx += 256) {
      const int tt = idx / CT, c = idx - tt * CT;
      sv[idx] = (tt < n && col0 + c < dv) ? to_f32(proj[(size_t)(t0 + tt) * stride + voff + h * dv + col0 + c]) : 0.f;
    }
    for (int idx = threadIdx.x; idx < GLA_TC * rank; idx += 256) {
      const int tt = idx / rank, r = idx - tt * rank;
      s1[idx] = tt < n ? to_f32(proj[(size_t)(t0 + tt) * stride + aoff + r]) : 0.f;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < GLA_TC * PR; idx += 256) {
      const int tt = idx / PR, i = idx - tt * PR;
      float al = 0.f;
      if (tt < n && i < dk) {
        const TW* w = a2 + (size_t)(h * dk + i) * rank;
        float z = a2b[h * dk + i];
        for (int r = 0; r < rank; ++r) z = fmaf(to_f32(w[r]), s1[tt * rank + r], z);
        // log sigmoid(z) = min(z, 0) - log1p(exp(-|z|))
        al = expf((fminf(z, 0.f) - log1pf(expf(-fabsf(z)))) * inv_tau);
      }
      sa[idx] = al;
    }
    __syncthreads();
    if (active) {
      for (int tt = 0; tt < n; ++tt) {
        const float vj = sv[tt * CT + j];
        const float* qa = sq + tt * PR + p * R;
        const float* ka = sk + tt * PR + p * R;
        const float* aa = sa + tt * PR + p * R;
        float po = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          S[r] = fmaf(aa[r], S[r], ka[r] * vj);
          po = fmaf(S[r], qa[r], po);
        }
        part[(tt * P + p) * CT + j] = po;
      }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < n * CT; idx += 256) {
      const int tt = idx / CT, c = idx - tt * CT;
      if (col0 + c < dv) {
        float o = 0.f;
        for (int pp = 0; pp < P; ++pp) o += part[(tt * P + pp) * CT + c];
        o_out[((size_t)(t0 + tt) * H + h) * dv + col0 + c] = o;
      }
    }
    // the next turn's loads touch sq/sk/sv/s1 only; `part` is rewritten after two barriers
  }
  if (active) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = p * R + r;
      if (i < dk) st[(size_t)i * dv + col0 + j] = S[r];
    }
  }
}

// proj: [nt, stride] rows holding q (H*dk) at qoff, k (H*dk) at koff, v (H*dv) at voff and the
// low-rank decay input (rank) at aoff. a2: [H*dk, rank], a2b [H*dk]. state: [slots, H, dk, dv]
// float32. o_out: [nt, H, dv] float32 (not yet normalised).
extern "C" int ta_gla_recurrent(hipStream_t stream, int dtype, int wdtype, const void* proj, int stride,
                                int qoff, int koff, int voff, int aoff, int rank, const void* a2,
                                const float* a2b, float inv_tau, float qscale, float* state,
                                const int* cu_q, const int* slots, int batch, int H, int dk, int dv,
                                float* o_out) {
  TA_REQUIRE(batch > 0 && batch <= 65535 && H > 0 && H <= 65535, "ta_gla_recurrent: bad batch %d / heads %d", batch, H);
  TA_REQUIRE(dk >= 1 && dk <= 256 && dv >= 1 && rank >= 1, "ta_gla_recurrent: key width %d outside [1, 256]", dk);
  const int CT = dv < 64 ? dv : 64;
  const int Pmax = 256 / CT;
  int need = (dk + Pmax - 1) / Pmax;
  const int R = need <= 4 ? 4 : need <= 8 ? 8 : need <= 16 ? 16 : need <= 32 ? 32 : 64;
  const int P = (dk + R - 1) / R;
  const size_t lds = (size_t)GLA_TC * (3 * P * R + CT + rank + P * CT) * sizeof(float);
  TA_REQUIRE(lds <= 64000, "ta_gla_recurrent: rank %d does not fit", rank);
  dim3 g(batch, H, (dv + CT - 1) / CT);
#define GLA_LAUNCH(T, TW, RR)                                                                          \
  gla_recurrent_kernel<T, TW, RR><<<g, 256, lds, stream>>>((const T*)proj, stride, qoff, koff, voff, aoff, rank, \
      (const TW*)a2, a2b, inv_tau, qscale, state, cu_q, slots, H, dk, dv, CT, P, o_out)
#define GLA_BY_R(T, TW)                                     \
  do {                                                      \
    if (R == 4) GLA_LAUNCH(T, TW, 4);                       \
    else if (R == 8) GLA_LAUNCH(T, TW, 8);                  \
    else if (R == 16) GLA_LAUNCH(T, TW, 16);                \
    else if (R == 32) GLA_LAUNCH(T, TW, 32);                \
    else GLA_LAUNCH(T, TW, 64);                             \
  } while (0)
  if (dtype == TA_F32 && wdtype == TA_F32) GLA_BY_R(float, float);
  else if (dtype == TA_BF16 && wdtype == TA_BF16) GLA_BY_R(bf16_t, bf16_t);
  else if (dtype == TA_BF16 && wdtype == TA_F32) GLA_BY_R(bf16_t, float);
  else return ta_fail("ta_gla_recurrent: unsupported dtypes %d / %d", dtype, wdtype);
#undef GLA_BY_R
#undef GLA_LAUNCH
  return ta_check_launch("ta_gla_recurrent");
}

// ------------------------------------------------------------------ gla: head norm and output gate
template <typename T>
__global__ __launch_bounds__(64) void gla_out_kernel(const float* __restrict__ o, const T* __restrict__ proj,
                                                     int stride, int goff, const float* __restrict__ w,
                                                     float eps, int H, int dv, T* __restrict__ out) {
  const size_t t = blockIdx.x;
  const int h = blockIdx.y;
  const float* src = o + (t * H + h) * dv;
  float ss = 0.f;
  for (int c = threadIdx.x; c < dv; c += 64) ss += src[c] * src[c];
  const float f = rsqrtf(wave_sum(ss) / (float)dv + eps);
  for (int c = threadIdx.x; c < dv; c += 64) {
    const float g = to_f32(proj[t * stride + goff + h * dv + c]);
    out[t * (size_t)(H * dv) + h * dv + c] = from_f32<T>(src[c] * f * w[c] * (g / (1.0f + expf(-g))));
  }
}

// o: [nt, H, dv] float32; the gate's pre-activation sits at column goff of proj; w [dv];
// out [nt, H*dv] = rms_norm(o per head) * w * silu(gate).
extern "C" int ta_gla_out(hipStream_t stream, int dtype, const float* o, const void* proj, int stride,
                          int goff, const float* w, float eps, int nt, int H, int dv, void* out) {
  TA_REQUIRE(nt >= 0 && H > 0 && H <= 65535 && dv > 0, "ta_gla_out: bad sizes");
  if (nt == 0) return 0;
  dim3 g(nt, H);
  if (dtype == TA_F32)
    gla_out_kernel<float><<<g, 64, 0, stream>>>(o, (const float*)proj, stride, goff, w, eps, H, dv, (float*)out);
  else if (dtype == TA_BF16)
    gla_out_kernel<bf16_t><<<g, 64, 0, stream>>>(o, (const bf16_t*)proj, stride, goff, w, eps, H, dv, (bf16_t*)out);
  else
    return ta_fail("ta_gla_out: unknown dtype %d", dtype);
  return ta_check_launch("ta_gla_out");
}
