// Pieces of a block whose sublayers are gated and whose mixer reads a token-shifted input,
// and of an embedding that adds a hashed row for the pair (previous token, token).
//
//   gated_add_rmsnorm : v = x + mult * sigmoid(gate + gate_bias) * (sum of delta planes + delta_bias),
//                       x = v, out = v / sqrt(mean(v^2) + eps) * weight      (all float32, one rounding)
//   token_shift       : hs_t = h_t + (h_{t-1} - h_t) * mu, h_{-1} from the sequence's state
//   pair_embed_add    : x_t += table[hash(previous token, token)]
//   scale             : t *= s
//
// Per-sequence state (the last row of h, the last token) is read and then written by the
// workgroup of the sequence's FIRST token of the step only, so no other workgroup races it.
#include "common.h"

// sequence that owns token t: the last b with cu_q[b] <= t
__device__ __forceinline__ int seq_of_token(const int* __restrict__ cu_q, int batch, int t) {
  int lo = 0, hi = batch - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x / TA_WAVE;
  __syncthreads();
  if (threadIdx.x % TA_WAVE == 0) red[w] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < (int)(blockDim.x / TA_WAVE); ++i) s += red[i];
  return s;
}

template <typename TO>
__global__ __launch_bounds__(256) void gated_add_rmsnorm_kernel(
    float* __restrict__ x, const float* __restrict__ delta, int planes, size_t plane,
    const float* __restrict__ delta_bias, const float* __restrict__ gate,
    const float* __restrict__ gate_bias, float mult, const float* __restrict__ weight,
    const int* __restrict__ rows, TO* __restrict__ out, int d, float eps, int store) {
  extern __shared__ float row[];          // [d]
  __shared__ float red[4];
  const int i = blockIdx.x;
  const size_t r = rows ? (size_t)rows[i] : (size_t)i;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += 256) {
    const size_t at = r * d + c;
    float v = x[at];
    if (delta) {
      float s = delta[at];
      for (int p = 1; p < planes; ++p) s += delta[at + p * plane];
      if (delta_bias) s += delta_bias[c];
      if (gate) {
        float g = gate[at];
        if (gate_bias) g += gate_bias[c];
        s *= 1.0f / (1.0f + expf(-g));
      }
      v += mult * s;
      if (store) x[at] = v;
    }
    row[c] = v;
    ss += v * v;
  }
  const float f = rsqrtf(block_sum_256(ss, red) / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += 256)
    out[(size_t)i * d + c] = from_f32<TO>(row[c] * f * weight[c]);
}

// The same for rows whose length is a multiple of four and at most 4,096: 1,024 threads, four
// columns each, everything a thread needs asked for at once (a row of a single-token step is
// otherwise sixteen trips to memory, one after the other).
template <typename TO>
__global__ __launch_bounds__(1024) void gated_add_rmsnorm_wide_kernel(
    float* __restrict__ x, const float* __restrict__ delta, int planes, size_t plane,
    const float* __restrict__ delta_bias, const float* __restrict__ gate,
    const float* __restrict__ gate_bias, float mult, const float* __restrict__ weight,
    const int* __restrict__ rows, TO* __restrict__ out, int d, float eps, int store,
    const float* __restrict__ mu, float* __restrict__ state, const int* __restrict__ slots,
    TO* __restrict__ shifted) {
  __shared__ float red[16];
  const int i = blockIdx.x;
  const size_t r = rows ? (size_t)rows[i] : (size_t)i;
  const int c = threadIdx.x * 4;
  const bool on = c < d;
  const size_t at = r * d + (on ? c : 0);
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 v = *reinterpret_cast<const float4*>(x + at);
  float4 w = *reinterpret_cast<const float4*>(weight + (on ? c : 0));
  if (delta) {
    float4 s = *reinterpret_cast<const float4*>(delta + at);
    float4 g = gate ? *reinterpret_cast<const float4*>(gate + at) : zero;
    const float4 gb = gate_bias ? *reinterpret_cast<const float4*>(gate_bias + (on ? c : 0)) : zero;
    const float4 db = delta_bias ? *reinterpret_cast<const float4*>(delta_bias + (on ? c : 0)) : zero;
    for (int p = 1; p < planes; ++p) {
      const float4 e = *reinterpret_cast<const float4*>(delta + at + p * plane);
      s.x += e.x; s.y += e.y; s.z += e.z; s.w += e.w;
    }
    s.x += db.x; s.y += db.y; s.z += db.z; s.w += db.w;
    if (gate) {
      s.x *= 1.0f / (1.0f + expf(-(g.x + gb.x)));
      s.y *= 1.0f / (1.0f + expf(-(g.y + gb.y)));
      s.z *= 1.0f / (1.0f + expf(-(g.z + gb.z)));
      s.w *= 1.0f / (1.0f + expf(-(g.w + gb.w)));
    }
    v.x += mult * s.x; v.y += mult * s.y; v.z += mult * s.z; v.w += mult * s.w;
    if (store && on) *reinterpret_cast<float4*>(x + at) = v;
  }
  float ss = on ? v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w : 0.f;
  ss = wave_sum(ss);
  if (threadIdx.x % TA_WAVE == 0) red[threadIdx.x / TA_WAVE] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int k = 0; k < 16; ++k) tot += red[k];
  const float f = rsqrtf(tot / (float)d + eps);
  if (on) {
    TO* o = out + (size_t)i * d + c;
    const TO h[4] = {from_f32<TO>(v.x * f * w.x), from_f32<TO>(v.y * f * w.y), from_f32<TO>(v.z * f * w.z),
                     from_f32<TO>(v.w * f * w.w)};
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = h[e];
    if (shifted) {
      // steps of single tokens: row i is sequence i's only token, so the row before it is the
      // sequence's state row, which then takes this row (the token shift, without a kernel of
      // its own)
      float* st = state + (size_t)slots[i] * d + c;
      const float4 prev = *reinterpret_cast<const float4*>(st);
      const float4 m = *reinterpret_cast<const float4*>(mu + c);
      const float cur[4] = {to_f32(h[0]), to_f32(h[1]), to_f32(h[2]), to_f32(h[3])};
      const float pv[4] = {prev.x, prev.y, prev.z, prev.w}, mv[4] = {m.x, m.y, m.z, m.w};
      TO* hs = shifted + (size_t)i * d + c;
#pragma unroll
      for (int e = 0; e < 4; ++e) hs[e] = from_f32<TO>(cur[e] + (pv[e] - cur[e]) * mv[e]);
      *reinterpret_cast<float4*>(st) = make_float4(cur[0], cur[1], cur[2], cur[3]);
    }
  }
}

static int gated_add_rmsnorm_launch(hipStream_t stream, int out_dtype, float* x, const float* delta,
                                    int planes, long long plane, const float* delta_bias,
                                    const float* gate, const float* gate_bias, float mult,
                                    const float* weight, const int* rows, void* out, int n_out, int d,
                                    float eps, int store, const float* mu, float* state, const int* slots,
                                    void* shifted) {
  TA_REQUIRE(n_out >= 0 && d > 0 && d <= 16000, "ta_gated_add_rmsnorm: bad sizes n=%d d=%d", n_out, d);
  TA_REQUIRE(planes >= 1 && planes <= TA_MAX_PLANES, "ta_gated_add_rmsnorm: %d planes", planes);
  if (n_out == 0) return 0;
  const bool aligned = (((uintptr_t)x | (uintptr_t)delta | (uintptr_t)gate | (uintptr_t)gate_bias |
                         (uintptr_t)delta_bias | (uintptr_t)weight | (uintptr_t)((size_t)plane * 4) |
                         (uintptr_t)mu | (uintptr_t)state) & 15) == 0;
  if (d % 4 == 0 && d <= 4096 && aligned && (out_dtype == TA_F32 || out_dtype == TA_BF16)) {
    if (out_dtype == TA_F32)
      gated_add_rmsnorm_wide_kernel<float><<<n_out, 1024, 0, stream>>>(
          x, delta, planes, (size_t)plane, delta_bias, gate, gate_bias, mult, weight, rows, (float*)out, d, eps, store,
          mu, state, slots, (float*)shifted);
    else
      gated_add_rmsnorm_wide_kernel<bf16_t><<<n_out, 1024, 0, stream>>>(
          x, delta, planes, (size_t)plane, delta_bias, gate, gate_bias, mult, weight, rows, (bf16_t*)out, d, eps, store,
          mu, state, slots, (bf16_t*)shifted);
    return ta_check_launch("ta_gated_add_rmsnorm");
  }
  TA_REQUIRE(shifted == nullptr, "ta_gated_add_rmsnorm_shift: rows of %d coordinates are not taken (a multiple "
             "of 4 up to 4096, on 16-byte boundaries)", d);
  const size_t lds = (size_t)d * sizeof(float);
  if (out_dtype == TA_F32)
    gated_add_rmsnorm_kernel<float><<<n_out, 256, lds, stream>>>(
        x, delta, planes, (size_t)plane, delta_bias, gate, gate_bias, mult, weight, rows, (float*)out, d, eps, store);
  else if (out_dtype == TA_BF16)
    gated_add_rmsnorm_kernel<bf16_t><<<n_out, 256, lds, stream>>>(
        x, delta, planes, (size_t)plane, delta_bias, gate, gate_bias, mult, weight, rows, (bf16_t*)out, d, eps, store);
  else
    return ta_fail("ta_gated_add_rmsnorm: unknown dtype %d", out_dtype);
  return ta_check_launch("ta_gated_add_rmsnorm");
}

extern "C" int ta_gated_add_rmsnorm(hipStream_t stream, int out_dtype, float* x, const float* delta,
                                    int planes, long long plane, const float* delta_bias,
                                    const float* gate, const float* gate_bias, float mult,
                                    const float* weight, const int* rows, void* out, int n_out, int d,
                                    float eps, int store) {
  return gated_add_rmsnorm_launch(stream, out_dtype, x, delta, planes, plane, delta_bias, gate, gate_bias, mult,
                                  weight, rows, out, n_out, d, eps, store, nullptr, nullptr, nullptr, nullptr);
}

// The same for a step in which every sequence brings ONE token (row i belongs to slots[i]),
// with the token shift behind the norm: shifted[i] = out[i] + (state[slots[i]] - out[i]) * mu,
// then state[slots[i]] = out[i]. Rows of a multiple of 4 up to 4,096 coordinates only.
extern "C" int ta_gated_add_rmsnorm_shift(hipStream_t stream, int out_dtype, float* x, const float* delta,
                                          int planes, long long plane, const float* delta_bias,
                                          const float* gate, const float* gate_bias, float mult,
                                          const float* weight, void* out, int n_out, int d, float eps,
                                          const float* mu, float* state, const int* slots, void* shifted) {
  TA_REQUIRE(mu && state && slots && shifted, "ta_gated_add_rmsnorm_shift: shift operands missing");
  return gated_add_rmsnorm_launch(stream, out_dtype, x, delta, planes, plane, delta_bias, gate, gate_bias, mult,
                                  weight, nullptr, out, n_out, d, eps, 1, mu, state, slots, shifted);
}

// ------------------------------------------------------------------ token shift
template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(
    const T* __restrict__ h, T* __restrict__ hs, const float* __restrict__ mu, int n_mu,
    float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ slots,
    int batch, int nt, int d) {
  const int t = blockIdx.x;
  const int b = seq_of_token(cu_q, batch, t);
  const int first = cu_q[b], last = cu_q[b + 1] - 1;
  float* st = state + (size_t)slots[b] * d;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < d; c += gridDim.y * 256) {
    const float cur = to_f32(h[(size_t)t * d + c]);
    float prev;
    if (t == first) {
      prev = st[c];
      st[c] = to_f32(h[(size_t)last * d + c]);
    } else {
      prev = to_f32(h[(size_t)(t - 1) * d + c]);
    }
    for (int s = 0; s < n_mu; ++s)
      hs[((size_t)s * nt + t) * d + c] = from_f32<T>(cur + (prev - cur) * mu[(size_t)s * d + c]);
  }
}

// h: [nt, d]; mu: [n_mu, d]; hs: [n_mu, nt, d], one shifted copy of the rows per mu; state:
// [slots, d] float32, the sequence's last unshifted row.
extern "C" int ta_token_shift_multi(hipStream_t stream, int dtype, const void* h, void* hs, const float* mu,
                                    int n_mu, float* state, const int* cu_q, const int* slots, int batch,
                                    int nt, int d) {
  TA_REQUIRE(batch > 0 && nt >= batch && d > 0 && n_mu >= 1 && n_mu <= 64,
             "ta_token_shift: bad sizes batch=%d nt=%d d=%d mus=%d", batch, nt, d, n_mu);
  // few rows: a column tile per workgroup, so that a thread makes one trip to memory
  dim3 g(nt, nt <= 256 ? (d + 255) / 256 : 1);
  if (dtype == TA_F32)
    token_shift_kernel<float><<<g, 256, 0, stream>>>((const float*)h, (float*)hs, mu, n_mu, state, cu_q, slots, batch, nt, d);
  else if (dtype == TA_BF16)
    token_shift_kernel<bf16_t><<<g, 256, 0, stream>>>((const bf16_t*)h, (bf16_t*)hs, mu, n_mu, state, cu_q, slots, batch, nt, d);
  else
    return ta_fail("ta_token_shift: unknown dtype %d", dtype);
  return ta_check_launch("ta_token_shift");
}

// The same with one mu: hs [nt, d].
extern "C" int ta_token_shift(hipStream_t stream, int dtype, const void* h, void* hs, const float* mu,
                              float* state, const int* cu_q, const int* slots, int batch, int nt, int d) {
  return ta_token_shift_multi(stream, dtype, h, hs, mu, 1, state, cu_q, slots, batch, nt, d);
}

// ------------------------------------------------------------------ hashed pair embedding
template <typename T>
__global__ __launch_bounds__(256) void pair_embed_add_kernel(
    float* __restrict__ x, const T* __restrict__ table, const int* __restrict__ tokens,
    int* __restrict__ last_token, const int* __restrict__ cu_q, const int* __restrict__ pos0,
    const int* __restrict__ slots, int batch, int d, int buckets, long long mul_prev, long long mul_cur) {
  const int t = blockIdx.x;
  const int b = seq_of_token(cu_q, batch, t);
  const int first = cu_q[b];
  long long prev;
  if (t == first) {
    prev = pos0[b] == 0 ? -1 : (long long)last_token[slots[b]];
  } else {
    prev = tokens[t - 1];
  }
  const long long rowi = prev < 0 ? (long long)buckets : (prev * mul_prev + (long long)tokens[t] * mul_cur) % buckets;
  const T* src = table + (size_t)rowi * d;
  for (int c = threadIdx.x; c < d; c += 256) x[(size_t)t * d + c] += to_f32(src[c]);
  if (t == first && threadIdx.x == 0) last_token[slots[b]] = tokens[cu_q[b + 1] - 1];
}

// x: [nt, d] float32; table: [buckets + 1, d]; last_token: [slots] int32 state.
extern "C" int ta_pair_embed_add(hipStream_t stream, int dtype, float* x, const void* table,
                                 const int* tokens, int* last_token, const int* cu_q, const int* pos0,
                                 const int* slots, int batch, int nt, int d, int buckets,
                                 long long mul_prev, long long mul_cur) {
  TA_REQUIRE(batch > 0 && nt >= batch && d > 0 && buckets > 0, "ta_pair_embed_add: bad sizes");
  TA_REQUIRE(mul_prev >= 0 && mul_cur >= 0 && mul_prev < (1ll << 31) && mul_cur < (1ll << 31),
             "ta_pair_embed_add: multipliers out of range");
  if (dtype == TA_F32)
    pair_embed_add_kernel<float><<<nt, 256, 0, stream>>>(x, (const float*)table, tokens, last_token, cu_q,
                                                        pos0, slots, batch, d, buckets, mul_prev, mul_cur);
  else if (dtype == TA_BF16)
    pair_embed_add_kernel<bf16_t><<<nt, 256, 0, stream>>>(x, (const bf16_t*)table, tokens, last_token, cu_q,
                                                         pos0, slots, batch, d, buckets, mul_prev, mul_cur);
  else
    return ta_fail("ta_pair_embed_add: unknown dtype %d", dtype);
  return ta_check_launch("ta_pair_embed_add");
}

// ------------------------------------------------------------------ scaling in place
__global__ void scale_kernel(float* __restrict__ t, size_t n, float s) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) t[i] *= s;
}

extern "C" int ta_scale_f32(hipStream_t stream, float* t, long long n, float s) {
  TA_REQUIRE(n >= 0, "ta_scale_f32: negative size");
  if (n == 0) return 0;
  size_t blocks = ((size_t)n + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  scale_kernel<<<(unsigned)blocks, 256, 0, stream>>>(t, (size_t)n, s);
  return ta_check_launch("ta_scale_f32");
}
